#pragma once
// BinaryGradientTester<Logic, Input1Dim, Input2Dim, OutputDim>: analytic
// backward of a two-operand logic against its own central-difference backward,
// in double, on random inputs and random upstream gradients; the gradients of
// both operands are compared.
//
// Same class name, entry points and arguments as the tester of xyz-autodiff-cuda
// (include/xyz_autodiff/testing/binary_gradient_tester.cuh: kernel :31-106, test()
// :124-187, test_custom() :190-306, kernel taking a logic instance :310-384), so
// a call written for it compiles as is:
//     using Logic = op::MulLogic<VariableRef<3, double>, VariableRef<3, double>>;
//     BinaryGradientTester<Logic, 3, 3, 3>::test_custom("MulLogic", 50, 1e-5, 1e-7, -3.0, 3.0);
// Leaves are VariableRef<InputNDim, double> on buffers, as the logic's template
// arguments in such a call expect.  The error of an element is
// min(|a - n|, |a - n| / (|a| + 1e-15)).  What differs (one launch for all cases,
// reproducible inputs, a report instead of gtest) is described in gradient_report.cuh.

#include <cstddef>
#include <string>
#include <vector>

#include <xyz_autodiff/operations/operation.cuh>
#include <xyz_autodiff/testing/gradient_report.cuh>
#include <xyz_autodiff/variable.cuh>

namespace xyz_autodiff {
namespace testing {
namespace detail {

// One case: both gradients of the Input1Dim + Input2Dim inputs (first operand first).
template <typename Logic, std::size_t Input1Dim, std::size_t Input2Dim, std::size_t OutputDim>
XAD_INLINE void binary_case(const Logic& logic, const double* input, const double* upstream, double delta, double* analytic,
                            double* numeric) {
    double value1[Input1Dim], grad1[Input1Dim], value2[Input2Dim], grad2[Input2Dim];
    for (std::size_t i = 0; i < Input1Dim; ++i) value1[i] = input[i];
    for (std::size_t i = 0; i < Input2Dim; ++i) value2[i] = input[Input1Dim + i];
    for (int numerical = 0; numerical < 2; ++numerical) {
        for (std::size_t i = 0; i < Input1Dim; ++i) grad1[i] = 0.0;
        for (std::size_t i = 0; i < Input2Dim; ++i) grad2[i] = 0.0;
        VariableRef<Input1Dim, double> first(value1, grad1);
        VariableRef<Input2Dim, double> second(value2, grad2);
        BinaryOperation<OutputDim, Logic, VariableRef<Input1Dim, double>, VariableRef<Input2Dim, double>> node(logic, first, second);
        node.forward();
        node.zero_grad();
        for (std::size_t j = 0; j < OutputDim; ++j) node.add_grad(j, upstream[j]);
        if (numerical)
            node.backward_numerical(delta);
        else
            node.backward();
        double* out = numerical ? numeric : analytic;
        for (std::size_t i = 0; i < Input1Dim; ++i) out[i] = grad1[i];
        for (std::size_t i = 0; i < Input2Dim; ++i) out[Input1Dim + i] = grad2[i];
    }
}

#if defined(__HIPCC__)
template <typename Logic, std::size_t Input1Dim, std::size_t Input2Dim, std::size_t OutputDim>
__global__ void binary_cases_kernel(Logic logic, std::size_t cases, const double* inputs, const double* upstream, double delta,
                                    double* analytic, double* numeric) {
    constexpr std::size_t kIn = Input1Dim + Input2Dim;
    const std::size_t c = static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (c >= cases) return;
    binary_case<Logic, Input1Dim, Input2Dim, OutputDim>(logic, inputs + c * kIn, upstream + c * OutputDim, delta, analytic + c * kIn,
                                                        numeric + c * kIn);
}
#endif

template <typename Logic, std::size_t Input1Dim, std::size_t Input2Dim, std::size_t OutputDim>
bool evaluate_binary_cases(const Logic& logic, std::size_t cases, const std::vector<double>& inputs,
                           const std::vector<double>& upstream, double delta, std::vector<double>& analytic,
                           std::vector<double>& numeric) {
    constexpr std::size_t kIn = Input1Dim + Input2Dim;
    analytic.assign(cases * kIn, 0.0);
    numeric.assign(cases * kIn, 0.0);
    if (cases == 0) return false;
#if defined(__HIPCC__)
    DeviceDoubles d_in(inputs), d_up(upstream), d_an(cases * kIn), d_nu(cases * kIn);
    const unsigned blocks = static_cast<unsigned>((cases + kCaseLanes - 1) / kCaseLanes);
    hipLaunchKernelGGL((binary_cases_kernel<Logic, Input1Dim, Input2Dim, OutputDim>), dim3(blocks), dim3(kCaseLanes), 0, 0, logic,
                       cases, d_in.get(), d_up.get(), delta, d_an.get(), d_nu.get());
    finish_launch();
    d_an.download(analytic);
    d_nu.download(numeric);
    return true;
#else
    for (std::size_t c = 0; c < cases; ++c)
        binary_case<Logic, Input1Dim, Input2Dim, OutputDim>(logic, inputs.data() + c * kIn, upstream.data() + c * OutputDim, delta,
                                                            analytic.data() + c * kIn, numeric.data() + c * kIn);
    return false;
#endif
}

}  // namespace detail

template <typename Logic, std::size_t Input1Dim, std::size_t Input2Dim, std::size_t OutputDim>
class BinaryGradientTester {
    static constexpr std::size_t NUM_TESTS = 100;
    static constexpr double TOLERANCE = 1e-5;
    static constexpr double DELTA = 1e-5;
    static constexpr std::size_t kIn = Input1Dim + Input2Dim;

public:
    // 100 cases, inputs and upstream gradients uniform in [-2, 2], delta 1e-5, tolerance 1e-5.
    static GradientReport test(const std::string& operation_name) {
        return run(Logic{}, operation_name, NUM_TESTS, TOLERANCE, DELTA, -2.0, 2.0);
    }

    // A tolerance outside [0, 1e-5] is refused, as there.
    static GradientReport test_custom(const std::string& operation_name, std::size_t num_tests, double tolerance, double delta,
                                      double input_min = -2.0, double input_max = 2.0) {
        if (!(tolerance >= 0.0 && tolerance <= 1e-5)) {
            GradientReport refused;
            refused.name = operation_name;
            refused.rejected = true;
            report_failure(operation_name + ": tolerance " + std::to_string(tolerance) +
                           " is not allowed; double-precision gradient tests take a tolerance in [0, 1e-5]");
            return refused;
        }
        return run(Logic{}, operation_name, num_tests, tolerance, delta, input_min, input_max);
    }

    // The same for a logic that carries state: the instance is given.
    static GradientReport test_logic(const Logic& logic, const std::string& operation_name, std::size_t num_tests = NUM_TESTS,
                                     double tolerance = TOLERANCE, double delta = DELTA, double input_min = -2.0,
                                     double input_max = 2.0) {
        return run(logic, operation_name, num_tests, tolerance, delta, input_min, input_max);
    }

private:
    static GradientReport run(const Logic& logic, const std::string& name, std::size_t cases, double tolerance, double delta,
                              double lo, double hi) {
        GradientReport report;
        report.name = name;
        report.cases = cases;
        CaseNumbers numbers(name);
        std::vector<double> inputs(cases * kIn), upstream(cases * OutputDim), analytic, numeric;
        for (std::size_t c = 0; c < cases; ++c) {
            for (std::size_t i = 0; i < kIn; ++i) inputs[c * kIn + i] = numbers.uniform(lo, hi);
            for (std::size_t j = 0; j < OutputDim; ++j) upstream[c * OutputDim + j] = numbers.uniform(lo, hi);
        }
        report.on_device =
            detail::evaluate_binary_cases<Logic, Input1Dim, Input2Dim, OutputDim>(logic, cases, inputs, upstream, delta, analytic, numeric);
        for (std::size_t c = 0; c < cases; ++c)
            for (std::size_t i = 0; i < kIn; ++i) {
                const double a = analytic[c * kIn + i], n = numeric[c * kIn + i];
                const std::string element = i < Input1Dim ? "input1[" + std::to_string(i) + "]" : "input2[" + std::to_string(i - Input1Dim) + "]";
                detail::record(report, tolerance, c, element, a, n, detail::min_abs_rel(a, n, a, 1e-15));
            }
        detail::conclude(report, tolerance);
        return report;
    }
};

}  // namespace testing
}  // namespace xyz_autodiff

// With gtest in scope, the one-line test definitions of the reference's header.
#if defined(TEST)
#define TEST_BINARY_GRADIENT(LogicType, Input1Dim, Input2Dim, OutputDim, TestName)                                        \
    TEST(GradientTest, TestName) {                                                                                        \
        xyz_autodiff::testing::BinaryGradientTester<LogicType, Input1Dim, Input2Dim, OutputDim>::test(#TestName);         \
    }
#define TEST_BINARY_GRADIENT_CUSTOM(LogicType, Input1Dim, Input2Dim, OutputDim, TestName, NumTests, Tolerance, Delta)     \
    TEST(GradientTest, TestName) {                                                                                        \
        xyz_autodiff::testing::BinaryGradientTester<LogicType, Input1Dim, Input2Dim, OutputDim>::test_custom(             \
            #TestName, NumTests, Tolerance, Delta);                                                                       \
    }
#endif
