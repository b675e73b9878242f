#pragma once
// Counter-based random numbers for the synthetic workloads.
//
// Every draw is a pure function of (seed, stream, index): no state, so any
// lane can produce element i of any array, host and device produce the same
// 64 random bits for it, and a workload is reproducible from three integers.
//
//   bits(seed, stream, i) = mix(mix(seed + G*(stream+1)) + G*(i+1))
//
// with G the 64-bit golden-ratio constant and mix the splitmix64 finaliser.
// The transformations to float use only operations that round identically on
// host and device (integer to float conversion, one explicit fused
// multiply-add), except normal(), whose log/cos differ in the last ulp between
// the device library and libm.

#include <cmath>
#include <cstdint>

#include <xyz_autodiff/detail/config.cuh>

namespace xad_rng {

XAD_INLINE std::uint64_t mix64(std::uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

constexpr std::uint64_t kGolden = 0x9E3779B97F4A7C15ull;

XAD_INLINE std::uint64_t stream_key(std::uint64_t seed, std::uint64_t stream) {
    return mix64(seed + kGolden * (stream + 1));
}

XAD_INLINE std::uint64_t bits(std::uint64_t key, std::uint64_t index) {
    return mix64(key + kGolden * (index + 1));
}

// Uniform in [0, 1): the top 24 bits, exactly representable in fp32.
XAD_INLINE float unit_float(std::uint64_t b) {
    return static_cast<float>(b >> 40) * 0x1.0p-24f;
}

// Uniform in [lo, hi).
XAD_INLINE float uniform(std::uint64_t b, float lo, float hi) {
    return ::fmaf(unit_float(b), hi - lo, lo);
}

// Normal(mean, stddev) by Box-Muller from the two 24-bit halves of one draw;
// the radius uses (k+1)/2^24 in (0, 1] so the logarithm is finite.
XAD_INLINE float normal(std::uint64_t b, float mean, float stddev) {
    const float u1 = static_cast<float>((b >> 40) + 1) * 0x1.0p-24f;
    const float u2 = static_cast<float>((b >> 16) & 0xFFFFFFu) * 0x1.0p-24f;
    const float radius = ::sqrtf(-2.0f * ::logf(u1));
    return ::fmaf(radius * ::cosf(6.283185307179586f * u2), stddev, mean);
}

}  // namespace xad_rng
