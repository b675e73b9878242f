#pragma once
// NetworkGradientTester<ParameterStruct, NetworkFunction>: analytic against
// central-difference gradients of a whole graph, for every member of a
// parameter struct.
//
// Same class name, entry points and arguments as the tester of xyz-autodiff-cuda
// (include/xyz_autodiff/testing/network_gradient_tester.cuh: calling convention of
// the network :21-38, test_single_case() :45-118, test_network() :121-189):
//   * ParameterStruct is a struct of doubles and nothing else;
//   * NetworkFunction is a callable with
//         template <GradientTag tag> void operator()(ParameterStruct* value, ParameterStruct* diff, double delta) const
//     that builds its graph on VariableRefs into *value and *diff and calls
//     run() for GradientTag::Analytical or run_numerical(delta) for
//     GradientTag::Numerical (in a HIP translation unit it must be callable on
//     the device);
//   * the error of a parameter is min(|a - n|, |a - n| / (|n| + 1e-10)); every
//     member is compared, also those the network treats as constants (both
//     gradients are then zero).
// test_network() perturbs every member of initial_params by a uniform number in
// [-parameter_range, parameter_range] per case.  What differs (one launch for
// all cases, reproducible perturbations, a report instead of gtest) is described
// in gradient_report.cuh.

#include <cstddef>
#include <cstring>
#include <string>
#include <tuple>
#include <type_traits>
#include <vector>

#include <xyz_autodiff/testing/gradient_check.cuh>  // GradientTag
#include <xyz_autodiff/testing/gradient_report.cuh>

namespace xyz_autodiff {
namespace testing {
namespace detail {

template <typename ParameterStruct, typename NetworkFunction>
XAD_INLINE void network_case(const NetworkFunction& network, const ParameterStruct& start, double delta, ParameterStruct& analytic,
                             ParameterStruct& numeric) {
    ParameterStruct value = start;
    analytic = ParameterStruct{};
    network.template operator()<GradientTag::Analytical>(&value, &analytic, delta);
    value = start;
    numeric = ParameterStruct{};
    network.template operator()<GradientTag::Numerical>(&value, &numeric, delta);
}

#if defined(__HIPCC__)
template <typename ParameterStruct, typename NetworkFunction>
__global__ void network_cases_kernel(NetworkFunction network, std::size_t cases, const ParameterStruct* start, double delta,
                                     ParameterStruct* analytic, ParameterStruct* numeric) {
    const std::size_t c = static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (c >= cases) return;
    ParameterStruct a, n;
    network_case(network, start[c], delta, a, n);
    analytic[c] = a;
    numeric[c] = n;
}
#endif

}  // namespace detail

template <typename ParameterStruct, typename NetworkFunction>
class NetworkGradientTester {
    static_assert(std::is_trivially_copyable_v<ParameterStruct> && sizeof(ParameterStruct) % sizeof(double) == 0,
                  "ParameterStruct must be a plain struct of doubles");
    static constexpr std::size_t kParams = sizeof(ParameterStruct) / sizeof(double);

public:
    // One parameter set.  Returns (passed, largest absolute error among the failing parameters, which one).
    static std::tuple<bool, double, std::string> test_single_case(NetworkFunction network, const ParameterStruct& initial_params,
                                                                   double tolerance = 1e-5, double delta = 1e-7, int seed = 42) {
        (void)seed;  // the reference takes it and does not use it either
        std::vector<ParameterStruct> start(1, initial_params), analytic, numeric;
        evaluate(network, start, delta, analytic, numeric);
        return compare(analytic[0], numeric[0], tolerance);
    }

    // num_tests perturbed parameter sets; every one must pass.
    static GradientReport test_network(const std::string& network_name, NetworkFunction network, const ParameterStruct& initial_params,
                                       int num_tests = 100, double tolerance = 1e-5, double delta = 1e-7,
                                       double parameter_range = 0.5) {
        GradientReport report;
        report.name = network_name;
        report.cases = num_tests > 0 ? static_cast<std::size_t>(num_tests) : 0;
        CaseNumbers numbers(network_name);
        std::vector<ParameterStruct> start(report.cases, initial_params), analytic, numeric;
        for (ParameterStruct& params : start) {
            double member[kParams];
            std::memcpy(member, &params, sizeof params);
            for (std::size_t i = 0; i < kParams; ++i) member[i] += numbers.uniform(-parameter_range, parameter_range);
            std::memcpy(&params, member, sizeof params);
        }
        report.on_device = evaluate(network, start, delta, analytic, numeric);
        for (std::size_t c = 0; c < report.cases; ++c) {
            double a[kParams], n[kParams];
            std::memcpy(a, &analytic[c], sizeof a);
            std::memcpy(n, &numeric[c], sizeof n);
            for (std::size_t i = 0; i < kParams; ++i)
                detail::record(report, tolerance, c, "parameter " + std::to_string(i), a[i], n[i],
                               detail::min_abs_rel(a[i], n[i], n[i], 1e-10));
        }
        detail::conclude(report, tolerance);
        return report;
    }

private:
    static bool evaluate(const NetworkFunction& network, const std::vector<ParameterStruct>& start, double delta,
                         std::vector<ParameterStruct>& analytic, std::vector<ParameterStruct>& numeric) {
        const std::size_t cases = start.size();
        analytic.assign(cases, ParameterStruct{});
        numeric.assign(cases, ParameterStruct{});
        if (cases == 0) return false;
#if defined(__HIPCC__)
        auto d_start = makeHipUniqueArray<ParameterStruct>(cases);
        auto d_analytic = makeHipUniqueArray<ParameterStruct>(cases);
        auto d_numeric = makeHipUniqueArray<ParameterStruct>(cases);
        const std::size_t bytes = cases * sizeof(ParameterStruct);
        CHECK_HIP_ERROR(hipMemcpy(d_start.get(), start.data(), bytes, hipMemcpyHostToDevice));
        const unsigned blocks = static_cast<unsigned>((cases + detail::kCaseLanes - 1) / detail::kCaseLanes);
        hipLaunchKernelGGL((detail::network_cases_kernel<ParameterStruct, NetworkFunction>), dim3(blocks), dim3(detail::kCaseLanes), 0,
                           0, network, cases, d_start.get(), delta, d_analytic.get(), d_numeric.get());
        detail::finish_launch();
        CHECK_HIP_ERROR(hipMemcpy(analytic.data(), d_analytic.get(), bytes, hipMemcpyDeviceToHost));
        CHECK_HIP_ERROR(hipMemcpy(numeric.data(), d_numeric.get(), bytes, hipMemcpyDeviceToHost));
        return true;
#else
        for (std::size_t c = 0; c < cases; ++c) detail::network_case(network, start[c], delta, analytic[c], numeric[c]);
        return false;
#endif
    }

    static std::tuple<bool, double, std::string> compare(const ParameterStruct& analytic, const ParameterStruct& numeric,
                                                         double tolerance) {
        double a[kParams], n[kParams];
        std::memcpy(a, &analytic, sizeof a);
        std::memcpy(n, &numeric, sizeof n);
        bool passed = true;
        double max_error = 0.0;
        std::string details;
        for (std::size_t i = 0; i < kParams; ++i) {
            const double error = detail::absolute(a[i] - n[i]);
            if (!(detail::min_abs_rel(a[i], n[i], n[i], 1e-10) <= tolerance)) {
                passed = false;
                if (details.empty() || !(error <= max_error)) {
                    max_error = error;
                    details = "Parameter " + std::to_string(i) + ": analytical=" + std::to_string(a[i]) +
                              ", numerical=" + std::to_string(n[i]) + ", error=" + std::to_string(error);
                }
            }
        }
        return {passed, max_error, details};
    }
};

}  // namespace testing
}  // namespace xyz_autodiff
