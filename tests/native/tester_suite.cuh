#pragma once
// The gradient testers of the library (xyz_autodiff/testing/*.cuh) run the way
// the tests of xyz-autodiff-cuda run theirs: every tester call of those tests, with
// its logic type, dimensions and numbers (tester_suite_entries.inc), the user
// logics and networks those tests define, and checks that a tester does report
// a wrong backward and refuses a loosened tolerance.  Compiled by hipcc the
// cases run in kernels, compiled by g++ on the calling thread.
#include <cstdio>
#include <exception>
#include <string>
#include <vector>

#include <xyz_autodiff/xyz_autodiff.cuh>
#include <operations/covariance_generation.cuh>
#include <operations/mahalanobis_distance.cuh>

namespace xad_suite {

using namespace xyz_autodiff;

// User logics in the shape of tests/operation/unary/test_add_constant_operations_gradient.cu:98-118, :131-151 and
// test_sub_constant_operations_gradient.cu:98-118, :131-151: operand types spelled out, device-only methods,
// a default-constructible logic carrying its constant (2.5, 1.7, 1.8, 0.42).
template <typename T>
struct AddConstantTestLogic {
    using value_type = T;
    static constexpr std::size_t outputDim = 3;
    T constant_c;
    __host__ __device__ explicit AddConstantTestLogic(T c = static_cast<T>(2.5)) : constant_c(c) {}
    __device__ void forward(Variable<3, T>& output, const VariableRef<3, T>& input) const {
        for (std::size_t i = 0; i < 3; ++i) output[i] = input[i] + constant_c;
    }
    __device__ void backward(const Variable<3, T>& output, VariableRef<3, T>& input) const {
        for (std::size_t i = 0; i < 3; ++i) input.add_grad(i, output.grad(i));
    }
};

struct AddConstant5DLogic {
    using value_type = double;
    static constexpr std::size_t outputDim = 5;
    double constant_c;
    __host__ __device__ explicit AddConstant5DLogic(double c = 1.7) : constant_c(c) {}
    __device__ void forward(Variable<5, double>& output, const VariableRef<5, double>& input) const {
        for (std::size_t i = 0; i < 5; ++i) output[i] = input[i] + constant_c;
    }
    __device__ void backward(const Variable<5, double>& output, VariableRef<5, double>& input) const {
        for (std::size_t i = 0; i < 5; ++i) input.add_grad(i, output.grad(i));
    }
};

template <typename T>
struct SubConstantTestLogic {
    using value_type = T;
    static constexpr std::size_t outputDim = 3;
    T constant_c;
    __host__ __device__ explicit SubConstantTestLogic(T c = static_cast<T>(1.8)) : constant_c(c) {}
    __device__ void forward(Variable<3, T>& output, const VariableRef<3, T>& input) const {
        for (std::size_t i = 0; i < 3; ++i) output[i] = input[i] - constant_c;
    }
    __device__ void backward(const Variable<3, T>& output, VariableRef<3, T>& input) const {
        for (std::size_t i = 0; i < 3; ++i) input.add_grad(i, output.grad(i));
    }
};

struct SubConstant5DLogic {
    using value_type = double;
    static constexpr std::size_t outputDim = 5;
    double constant_c;
    __host__ __device__ explicit SubConstant5DLogic(double c = 0.42) : constant_c(c) {}
    __device__ void forward(Variable<5, double>& output, const VariableRef<5, double>& input) const {
        for (std::size_t i = 0; i < 5; ++i) output[i] = input[i] - constant_c;
    }
    __device__ void backward(const Variable<5, double>& output, VariableRef<5, double>& input) const {
        for (std::size_t i = 0; i < 5; ++i) input.add_grad(i, output.grad(i));
    }
};

// y = x^2 with the sign of the derivative wrong: a tester has to notice.
struct WrongSignLogic {
    static constexpr std::size_t outputDim = 2;
    __device__ void forward(Variable<2, double>& output, const VariableRef<2, double>& input) const {
        for (std::size_t i = 0; i < 2; ++i) output[i] = input[i] * input[i];
    }
    __device__ void backward(const Variable<2, double>& output, VariableRef<2, double>& input) const {
        for (std::size_t i = 0; i < 2; ++i) input.add_grad(i, -2.0 * input[i] * output.grad(i));
    }
};

// a * b with the second operand's gradient forgotten.
struct ForgetfulMulLogic {
    static constexpr std::size_t outputDim = 1;
    __device__ void forward(Variable<1, double>& output, const VariableRef<1, double>& a, const VariableRef<1, double>& b) const {
        output[0] = a[0] * b[0];
    }
    __device__ void backward(const Variable<1, double>& output, VariableRef<1, double>& a, VariableRef<1, double>& b) const {
        a.add_grad(0, output.grad(0) * b[0]);
    }
};

// The parameter struct and the networks of tests/operation/base/test_linear_regression_network.cu:25-165:
// y = (x1 - a)^2 + b (x2 - c)^2 + d, loss = (y - y_target)^2, written with the operator overloads.
struct OptimizationParameters {
    double a, b, c, d, x1, x2, y_target;
};

struct SimpleLinearRegressionNetwork {
    template <testing::GradientTag tag>
    __device__ void operator()(OptimizationParameters* value, OptimizationParameters* diff, double delta = 1e-7) const {
        VariableRef<1, double> a_var(&value->a, &diff->a), b_var(&value->b, &diff->b), c_var(&value->c, &diff->c),
            d_var(&value->d, &diff->d);
        auto x1_minus_a = a_var - value->x1;
        auto x1_term = op::squared(x1_minus_a);
        auto x2_minus_c = c_var - value->x2;
        auto x2_squared = op::squared(x2_minus_c);
        auto x2_term = b_var * x2_squared;
        auto combined_terms = x1_term + x2_term;
        auto y_pred = combined_terms + d_var;
        auto y_diff = y_pred - value->y_target;
        auto loss = op::squared(y_diff);
        if constexpr (tag == testing::GradientTag::Analytical)
            loss.run();
        else
            loss.run_numerical(delta);
    }
};

// :84-120 there: the same graph reached through a reference to its root.
struct RegularizedLinearRegressionNetwork {
    template <testing::GradientTag tag>
    __device__ void operator()(OptimizationParameters* value, OptimizationParameters* diff, double delta = 1e-7) const {
        VariableRef<1, double> a_var(&value->a, &diff->a), b_var(&value->b, &diff->b), c_var(&value->c, &diff->c),
            d_var(&value->d, &diff->d);
        auto x1_minus_a = a_var - value->x1;
        auto x1_term = op::squared(x1_minus_a);
        auto x2_minus_c = c_var - value->x2;
        auto x2_squared = op::squared(x2_minus_c);
        auto x2_term = b_var * x2_squared;
        auto combined_terms = x1_term + x2_term;
        auto y_pred = combined_terms + d_var;
        auto y_diff = y_pred - value->y_target;
        auto main_loss = op::squared(y_diff);
        auto& total_loss = main_loss;
        if constexpr (tag == testing::GradientTag::Analytical)
            total_loss.run();
        else
            total_loss.run_numerical(delta);
    }
};

struct SubtractSquareOnlyNetwork {
    template <testing::GradientTag tag>
    __device__ void operator()(OptimizationParameters* value, OptimizationParameters* diff, double delta = 1e-7) const {
        VariableRef<1, double> a_var(&value->a, &diff->a);
        auto a_minus_x1 = op::sub_constant(a_var, value->x1);
        auto result = op::squared(a_minus_x1);
        if constexpr (tag == testing::GradientTag::Analytical)
            result.run();
        else
            result.run_numerical(delta);
    }
};

struct DuplicateAddNetwork {
    template <testing::GradientTag tag>
    __device__ void operator()(OptimizationParameters* value, OptimizationParameters* diff, double delta = 1e-7) const {
        VariableRef<1, double> a_var(&value->a, &diff->a), b_var(&value->b, &diff->b);
        auto ab = a_var + b_var;
        auto ab2 = a_var + b_var;
        auto ab_sum = ab + ab2;
        if constexpr (tag == testing::GradientTag::Analytical)
            ab_sum.run();
        else
            ab_sum.run_numerical(delta);
    }
};

// A network whose analytic gradient is wrong by construction: the numerical pass differentiates a^2, the analytic one a^3.
struct InconsistentNetwork {
    template <testing::GradientTag tag>
    __device__ void operator()(OptimizationParameters* value, OptimizationParameters* diff, double delta = 1e-7) const {
        VariableRef<1, double> a_var(&value->a, &diff->a);
        auto square = op::squared(a_var);
        if constexpr (tag == testing::GradientTag::Analytical) {
            auto cube = square * a_var;
            cube.run();
        } else {
            square.run_numerical(delta);
        }
    }
};

struct Entry {
    std::string citation;
    testing::GradientReport report;
};

// Every tester call of the reference's tests.  Returns the entries in file order.
inline std::vector<Entry> run_reference_calls() {
    std::vector<Entry> entries;
    auto add = [&](const char* citation, testing::GradientReport report) { entries.push_back({citation, std::move(report)}); };
#include "tester_suite_entries.inc"
    // tests/operation/base/test_linear_regression_network.cu: (a, b, c, d, x1, x2, y_target) and the arguments of test_network
    using Params = OptimizationParameters;
    add("tests/operation/base/test_linear_regression_network.cu:199",
        testing::NetworkGradientTester<Params, SimpleLinearRegressionNetwork>::test_network(
            "SimpleLinearRegressionNetwork", {}, Params{1.0, 1.5, 0.5, 0.2, 2.0, 1.5, 3.0}, 100, 1e-5, 1e-6, 0.3));
    add("tests/operation/base/test_linear_regression_network.cu:222",
        testing::NetworkGradientTester<Params, RegularizedLinearRegressionNetwork>::test_network(
            "RegularizedLinearRegressionNetwork", {}, Params{0.8, 1.2, -0.3, 0.5, 1.0, 0.8, 2.5}, 50, 1e-5, 1e-6, 0.2));
    add("tests/operation/base/test_linear_regression_network.cu:246",
        testing::NetworkGradientTester<Params, SubtractSquareOnlyNetwork>::test_network(
            "SubtractSquareOnlyNetwork", {}, Params{1.0, 0.0, 0.0, 0.0, 2.0, 0.0, 0.0}, 50, 1e-5, 1e-7, 0.5));
    add("tests/operation/base/test_linear_regression_network.cu:269",
        testing::NetworkGradientTester<Params, DuplicateAddNetwork>::test_network(
            "DuplicateAddNetwork", {}, Params{0.5, 0.8, 0.3, 0.2, 1.0, 0.5, 1.5}, 50, 1e-5, 1e-6, 0.2));
    add("tests/operation/base/test_linear_regression_network.cu:293",
        testing::NetworkGradientTester<Params, SimpleLinearRegressionNetwork>::test_network(
            "SimpleLinearRegressionNetwork_LargeValues", {}, Params{10.0, 15.0, -8.0, 5.0, 20.0, -10.0, 100.0}, 20, 1e-3, 1e-5, 1.0));
    add("tests/operation/base/test_linear_regression_network.cu:317",
        testing::NetworkGradientTester<Params, SimpleLinearRegressionNetwork>::test_network(
            "SimpleLinearRegressionNetwork_NearZero", {}, Params{0.001, 0.002, -0.001, 0.0001, 0.01, -0.01, 0.001}, 30, 1e-5, 1e-8,
            0.001));
    return entries;
}

// "citation|name|cases|failures|worst error|device(1)/host(0)" per line.
inline std::string describe(const std::vector<Entry>& entries) {
    std::string text;
    for (const Entry& e : entries) {
        char line[512];
        std::snprintf(line, sizeof line, "%s|%s|%zu|%zu|%.3e|%d\n", e.citation.c_str(), e.report.name.c_str(), e.report.cases,
                      e.report.failures, e.report.worst_error, e.report.on_device ? 1 : 0);
        text += line;
    }
    return text;
}

// Bit k set = check k behaved as it must:
//   0  a wrong backward sign is reported for (nearly) every element   1  and counted in failure_count()
//   2  a missing operand gradient is reported, on that operand only   3  a tolerance above 1e-5 is refused, nothing runs
//   4  a negative tolerance is refused                                5  an inconsistent network fails test_single_case
//   6  ... and test_network                                           7  a correct network passes test_single_case
//   8  a logic instance with another constant is used by test_logic   9  zero cases is an empty, passing report;
//                                                                      compute_error_min is min(absolute, relative)
inline unsigned run_self_checks() {
    unsigned ok = 0;
    const std::size_t before = testing::failure_count();
    const auto wrong = testing::UnaryGradientTester<WrongSignLogic, 2, 2>::test("WrongSignLogic (must be reported)");
    if (!wrong && wrong.failures >= 190 && wrong.failures <= 200 && wrong.cases == 100) ok |= 1u << 0;
    if (testing::failure_count() == before + 1) ok |= 1u << 1;
    const auto forgetful = testing::BinaryGradientTester<ForgetfulMulLogic, 1, 1, 1>::test_custom(
        "ForgetfulMulLogic (must be reported)", 40, 1e-5, 1e-6, 0.5, 2.0);
    if (!forgetful && forgetful.failures == 40 && forgetful.worst.find("input2[0]") != std::string::npos) ok |= 1u << 2;
    const auto loose = testing::UnaryGradientTester<op::ExpLogic<2>, 2, 2>::test_custom("loosened tolerance (must be refused)", 10, 1e-4, 1e-6);
    if (!loose && loose.rejected && loose.cases == 0) ok |= 1u << 3;
    using Mul = op::MulLogic<VariableRef<1, double>, VariableRef<1, double>>;
    const auto negative = testing::BinaryGradientTester<Mul, 1, 1, 1>::test_custom("negative tolerance (must be refused)", 10, -1.0, 1e-6);
    if (!negative && negative.rejected) ok |= 1u << 4;
    const OptimizationParameters params{1.0, 1.5, 0.5, 0.2, 2.0, 1.5, 3.0};
    {
        auto [passed, error, details] = testing::NetworkGradientTester<OptimizationParameters, InconsistentNetwork>::test_single_case({}, params);
        if (!passed && error > 0.9 && error < 1.1 && details.find("Parameter 0") == 0) ok |= 1u << 5;  // 3 a^2 - 2 a = 1 at a = 1
    }
    const auto bad_network = testing::NetworkGradientTester<OptimizationParameters, InconsistentNetwork>::test_network(
        "InconsistentNetwork (must be reported)", {}, params, 25, 1e-5, 1e-7, 0.1);
    if (!bad_network && bad_network.failures == 25) ok |= 1u << 6;
    {
        auto [passed, error, details] =
            testing::NetworkGradientTester<OptimizationParameters, SimpleLinearRegressionNetwork>::test_single_case({}, params, 1e-5, 1e-6);
        if (passed && error == 0.0 && details.empty()) ok |= 1u << 7;
    }
    const auto shifted = testing::UnaryGradientTester<AddConstantTestLogic<double>, 3, 3>::test_logic(
        AddConstantTestLogic<double>(-40.0), "AddConstantTestLogic(-40)", 20, 1e-5, 1e-6, -1.0, 1.0);
    if (shifted && shifted.cases == 20) ok |= 1u << 8;
    const auto none = testing::UnaryGradientTester<op::ExpLogic<2>, 2, 2>::test_custom("no cases", 0, 1e-5, 1e-6);
    if (none && none.cases == 0 && none.failures == 0 && testing::compute_error_min(0.5, 0.75) == 0.25 &&  // absolute
        testing::detail::absolute(testing::compute_error_min(8.0, 10.0) - 0.25) < 1e-12 &&  // relative
        testing::compute_error_min(4.0f, 4.0f) == 0.0f)
        ok |= 1u << 9;
    return ok;
}

// C-side glue shared by the two builds: writes describe(run_reference_calls()) into text (NUL-terminated,
// truncated to capacity) and the self-check bits; returns the number of entries, or -1 with the error text.
inline int export_suite(char* text, std::size_t capacity, unsigned* self_checks) {
    auto put = [&](const std::string& s) {
        if (!text || capacity == 0) return;
        const std::size_t n = s.size() < capacity - 1 ? s.size() : capacity - 1;
        s.copy(text, n);
        text[n] = '\0';
    };
    try {
        const std::vector<Entry> entries = run_reference_calls();
        if (self_checks) *self_checks = run_self_checks();
        put(describe(entries));
        return static_cast<int>(entries.size());
    } catch (const std::exception& e) {
        put(e.what());
        return -1;
    }
}

}  // namespace xad_suite
