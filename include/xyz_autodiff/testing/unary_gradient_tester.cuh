#pragma once
// UnaryGradientTester<Logic, InputDim, OutputDim>: analytic backward of a
// one-operand logic against its own central-difference backward, in double, on
// random inputs and random upstream gradients.
//
// Same class name, entry points and arguments as the tester of xyz-autodiff-cuda
// (include/xyz_autodiff/testing/unary_gradient_tester.cuh: kernel :35-93, test()
// :104-154, test_custom() :157-247), so a call written for it compiles as is:
//     UnaryGradientTester<op::L2NormLogic<3>, 3, 1>::test_custom("L2Norm", 50, 1e-5, 1e-7, -2.0, 2.0);
// The node is built the same way: leaves are VariableRef<InputDim, double> on
// buffers, the logic is default-constructed, and a user logic may therefore
// spell its operand type as VariableRef<InputDim, double>.  The error of an
// element is min(|a - n|, |a - n| / (|a| + 1e-15)).  What differs (one launch
// for all cases, reproducible inputs, a report instead of gtest) is described in
// gradient_report.cuh.

#include <cstddef>
#include <string>
#include <vector>

#include <xyz_autodiff/operations/operation.cuh>
#include <xyz_autodiff/testing/gradient_report.cuh>
#include <xyz_autodiff/variable.cuh>

namespace xyz_autodiff {
namespace testing {
namespace detail {

// One case: both gradients of the InputDim inputs for one upstream gradient.
template <typename Logic, std::size_t InputDim, std::size_t OutputDim>
XAD_INLINE void unary_case(const Logic& logic, const double* input, const double* upstream, double delta, double* analytic,
                           double* numeric) {
    double value[InputDim], grad[InputDim];
    for (std::size_t i = 0; i < InputDim; ++i) value[i] = input[i];
    for (int numerical = 0; numerical < 2; ++numerical) {
        for (std::size_t i = 0; i < InputDim; ++i) grad[i] = 0.0;
        VariableRef<InputDim, double> leaf(value, grad);
        UnaryOperation<OutputDim, Logic, VariableRef<InputDim, double>> node(logic, leaf);
        node.forward();
        node.zero_grad();
        for (std::size_t j = 0; j < OutputDim; ++j) node.add_grad(j, upstream[j]);
        if (numerical)
            node.backward_numerical(delta);
        else
            node.backward();
        double* out = numerical ? numeric : analytic;
        for (std::size_t i = 0; i < InputDim; ++i) out[i] = grad[i];
    }
}

#if defined(__HIPCC__)
template <typename Logic, std::size_t InputDim, std::size_t OutputDim>
__global__ void unary_cases_kernel(Logic logic, std::size_t cases, const double* inputs, const double* upstream, double delta,
                                   double* analytic, double* numeric) {
    const std::size_t c = static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (c >= cases) return;
    unary_case<Logic, InputDim, OutputDim>(logic, inputs + c * InputDim, upstream + c * OutputDim, delta, analytic + c * InputDim,
                                           numeric + c * InputDim);
}
#endif

// All cases: in a kernel when this is a HIP translation unit, else on the calling thread.
template <typename Logic, std::size_t InputDim, std::size_t OutputDim>
bool evaluate_unary_cases(const Logic& logic, std::size_t cases, const std::vector<double>& inputs,
                          const std::vector<double>& upstream, double delta, std::vector<double>& analytic,
                          std::vector<double>& numeric) {
    analytic.assign(cases * InputDim, 0.0);
    numeric.assign(cases * InputDim, 0.0);
    if (cases == 0) return false;
#if defined(__HIPCC__)
    DeviceDoubles d_in(inputs), d_up(upstream), d_an(cases * InputDim), d_nu(cases * InputDim);
    const unsigned blocks = static_cast<unsigned>((cases + kCaseLanes - 1) / kCaseLanes);
    hipLaunchKernelGGL((unary_cases_kernel<Logic, InputDim, OutputDim>), dim3(blocks), dim3(kCaseLanes), 0, 0, logic, cases,
                       d_in.get(), d_up.get(), delta, d_an.get(), d_nu.get());
    finish_launch();
    d_an.download(analytic);
    d_nu.download(numeric);
    return true;
#else
    for (std::size_t c = 0; c < cases; ++c)
        unary_case<Logic, InputDim, OutputDim>(logic, inputs.data() + c * InputDim, upstream.data() + c * OutputDim, delta,
                                               analytic.data() + c * InputDim, numeric.data() + c * InputDim);
    return false;
#endif
}

}  // namespace detail

template <typename Logic, std::size_t InputDim, std::size_t OutputDim>
class UnaryGradientTester {
    static constexpr std::size_t NUM_TESTS = 100;
    static constexpr double TOLERANCE = 1e-5;
    static constexpr double DELTA = 1e-5;

public:
    // 100 cases, inputs and upstream gradients uniform in [-2, 2], delta 1e-5, tolerance 1e-5.
    static GradientReport test(const std::string& operation_name) {
        return run(Logic{}, operation_name, NUM_TESTS, TOLERANCE, DELTA, -2.0, 2.0);
    }

    // A tolerance outside [0, 1e-5] is refused, as there: double-precision gradient tests are not to be loosened.
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

    // The same for a logic that carries state (a constant, a reference to an array): the instance is given.
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
        std::vector<double> inputs(cases * InputDim), upstream(cases * OutputDim), analytic, numeric;
        for (std::size_t c = 0; c < cases; ++c) {
            for (std::size_t i = 0; i < InputDim; ++i) inputs[c * InputDim + i] = numbers.uniform(lo, hi);
            for (std::size_t j = 0; j < OutputDim; ++j) upstream[c * OutputDim + j] = numbers.uniform(lo, hi);
        }
        report.on_device = detail::evaluate_unary_cases<Logic, InputDim, OutputDim>(logic, cases, inputs, upstream, delta, analytic, numeric);
        for (std::size_t c = 0; c < cases; ++c)
            for (std::size_t i = 0; i < InputDim; ++i) {
                const double a = analytic[c * InputDim + i], n = numeric[c * InputDim + i];
                detail::record(report, tolerance, c, "input[" + std::to_string(i) + "]", a, n, detail::min_abs_rel(a, n, a, 1e-15));
            }
        detail::conclude(report, tolerance);
        return report;
    }
};

}  // namespace testing
}  // namespace xyz_autodiff

// With gtest in scope, the one-line test definitions of the reference's header.
#if defined(TEST)
#define TEST_UNARY_GRADIENT(LogicType, InputDim, OutputDim, TestName) \
    TEST(GradientTest, TestName) { xyz_autodiff::testing::UnaryGradientTester<LogicType, InputDim, OutputDim>::test(#TestName); }
#define TEST_UNARY_GRADIENT_CUSTOM(LogicType, InputDim, OutputDim, TestName, NumTests, Tolerance, Delta)                       \
    TEST(GradientTest, TestName) {                                                                                             \
        xyz_autodiff::testing::UnaryGradientTester<LogicType, InputDim, OutputDim>::test_custom(#TestName, NumTests, Tolerance, \
                                                                                                 Delta);                        \
    }
#endif
