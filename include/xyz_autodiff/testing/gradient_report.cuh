#pragma once
// Shared parts of the gradient testers (unary_gradient_tester.cuh,
// binary_gradient_tester.cuh, network_gradient_tester.cuh): what a tester hands
// back, where a failed check is reported, the reproducible numbers the cases are
// drawn from, and device buffers for the batched kernels.
//
// The testers of xyz-autodiff-cuda (include/xyz_autodiff/testing/*.cuh) are gtest
// helpers: they report through EXPECT_*/FAIL, draw their cases from
// std::random_device and launch one <<<1,1>>> kernel per case with a copy in
// and a copy out around each.  These keep the class names, the static entry
// points and their arguments, and differ in three ways:
//   * no test framework is needed: a tester returns a GradientReport, prints a
//     failure to stderr and counts it in failure_count().  If the including file
//     has gtest's ADD_FAILURE macro in scope, failures go there as well, so a
//     TEST_F body written for the reference behaves as before;
//   * cases are reproducible: they come from a counter-based generator keyed by
//     the test's name (and case_seed()), not from the machine's entropy source;
//   * all cases of a call run in ONE kernel launch, one lane per case, with one
//     upload and one download; compiled by a plain host compiler they run on the
//     calling thread instead.

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include <xyz_autodiff/detail/config.cuh>

#if defined(__HIPCC__)
#include <xyz_autodiff/util/error_checker.cuh>
#include <xyz_autodiff/util/hip_unique_ptr.cuh>
#endif

namespace xyz_autodiff {
namespace testing {

struct GradientReport {
    std::string name;
    std::size_t cases = 0;     // cases evaluated
    std::size_t failures = 0;  // gradient elements whose error exceeds the tolerance (a NaN counts)
    double worst_error = 0.0;  // largest error seen, failing or not
    std::string worst;         // case, element and both gradients of worst_error
    bool on_device = false;    // evaluated in a kernel; false: on the calling thread
    bool rejected = false;     // the request itself was refused and nothing ran
    explicit operator bool() const { return !rejected && failures == 0; }
};

// Failed checks since the program started (all testers).
inline std::size_t& failure_count() {
    static std::size_t count = 0;
    return count;
}

// Mixed into every generator, so a whole run can be repeated with other numbers.
inline std::uint64_t& case_seed() {
    static std::uint64_t seed = 0;
    return seed;
}

inline void report_failure(const std::string& message) {
    ++failure_count();
    std::fprintf(stderr, "[xyz_autodiff::testing] %s\n", message.c_str());
#if defined(ADD_FAILURE)
    ADD_FAILURE() << message;
#endif
}

// Uniform doubles from a splitmix64 stream keyed by a name.
class CaseNumbers {
public:
    explicit CaseNumbers(const std::string& key) : state_(0xcbf29ce484222325ull ^ case_seed()) {
        for (unsigned char ch : key) state_ = (state_ ^ ch) * 0x100000001b3ull;  // FNV-1a
    }
    double uniform(double lo, double hi) {
        const double unit = static_cast<double>(next() >> 11) * 0x1.0p-53;  // [0, 1)
        return lo + (hi - lo) * unit;
    }

private:
    std::uint64_t next() {
        std::uint64_t z = (state_ += 0x9e3779b97f4a7c15ull);
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        return z ^ (z >> 31);
    }
    std::uint64_t state_;
};

namespace detail {

inline double absolute(double v) { return v < 0.0 ? -v : v; }

// min(|a - n|, |a - n| / (|reference| + floor)); NaN if either gradient is.
inline double min_abs_rel(double analytic, double numeric, double reference, double floor) {
    const double diff = absolute(analytic - numeric);
    const double rel = diff / (absolute(reference) + floor);
    return diff < rel ? diff : rel;  // a NaN diff makes the comparison false and returns the NaN rel
}

}  // namespace detail

// The testers' error measure for one gradient element: min(|a - n|, |a - n| / (|a| + 1e-15))
// (unary_gradient_tester.cuh:27-32 of the reference, same name).
template <typename T>
inline T compute_error_min(T analytical, T numerical) {
    return static_cast<T>(detail::min_abs_rel(static_cast<double>(analytical), static_cast<double>(numerical),
                                              static_cast<double>(analytical), 1e-15));
}

namespace detail {

inline std::string describe(std::size_t test_case, const std::string& element, double analytic, double numeric, double error) {
    char text[256];
    std::snprintf(text, sizeof text, "test case %zu, %s: analytical=%.12g, numerical=%.12g, error_min=%.3g", test_case,
                  element.c_str(), analytic, numeric, error);
    return text;
}

// Folds one compared element into the report.
inline void record(GradientReport& report, double tolerance, std::size_t test_case, const std::string& element,
                   double analytic, double numeric, double error) {
    const bool failed = !(error <= tolerance);
    if (failed) ++report.failures;
    if (report.worst.empty() || !(error <= report.worst_error)) {
        report.worst_error = error;
        report.worst = describe(test_case, element, analytic, numeric, error);
    }
}

inline void conclude(const GradientReport& report, double tolerance) {
    if (report.failures == 0) return;
    char head[160];
    std::snprintf(head, sizeof head, ": %zu gradient element(s) of %zu case(s) above tolerance %.3g; worst: ", report.failures,
                  report.cases, tolerance);
    report_failure(report.name + head + report.worst);
}

#if defined(__HIPCC__)
// A device array of doubles with the two copies the batched kernels need.
class DeviceDoubles {
public:
    explicit DeviceDoubles(std::size_t count) : count_(count), memory_(makeHipUniqueArray<double>(count ? count : 1)) {}
    DeviceDoubles(const std::vector<double>& host) : DeviceDoubles(host.size()) {
        if (count_) CHECK_HIP_ERROR(hipMemcpy(memory_.get(), host.data(), count_ * sizeof(double), hipMemcpyHostToDevice));
    }
    double* get() const { return memory_.get(); }
    void download(std::vector<double>& host) const {
        host.resize(count_);
        if (count_) CHECK_HIP_ERROR(hipMemcpy(host.data(), memory_.get(), count_ * sizeof(double), hipMemcpyDeviceToHost));
    }

private:
    std::size_t count_;
    hip_unique_ptr<double[]> memory_;
};

constexpr unsigned kCaseLanes = 64;  // one wavefront per block; a case per lane

inline void finish_launch() {
    CHECK_HIP_ERROR(hipGetLastError());
    CHECK_HIP_ERROR(hipDeviceSynchronize());
}
#endif

}  // namespace detail
}  // namespace testing
}  // namespace xyz_autodiff
