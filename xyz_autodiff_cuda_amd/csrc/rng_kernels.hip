// Device and host fills from the counter-based generator.
#include <algorithm>

#include "common.cuh"
#include "rng.cuh"

namespace {

constexpr unsigned kBlock = 256;

enum class Law { Uniform, Normal };

template <Law law>
__global__ void __launch_bounds__(kBlock) fill_kernel(float* dst, std::size_t n, std::uint64_t key, float a, float b) {
    const std::size_t stride = static_cast<std::size_t>(gridDim.x) * kBlock;
    for (std::size_t i = static_cast<std::size_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) {
        const std::uint64_t r = xad_rng::bits(key, i);
        dst[i] = law == Law::Uniform ? xad_rng::uniform(r, a, b) : xad_rng::normal(r, a, b);
    }
}

template <Law law>
int fill(float* dst, std::size_t n, std::uint64_t seed, std::uint64_t stream_id, float a, float b, void* stream) {
    if (n == 0) return XAD_OK;
    XAD_REQUIRE(dst, "rng fill: destination is null");
    const unsigned grid = static_cast<unsigned>(std::min<std::size_t>(xad::blocks_for(n, kBlock), 256u * 32u));
    hipLaunchKernelGGL(fill_kernel<law>, dim3(grid), dim3(kBlock), 0, xad::as_stream(stream), dst, n,
                       xad_rng::stream_key(seed, stream_id), a, b);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

}  // namespace

extern "C" int xad_rng_uniform_f32(float* dst, std::size_t n, std::uint64_t seed, std::uint64_t stream_id, float lo,
                                   float hi, void* stream) {
    return fill<Law::Uniform>(dst, n, seed, stream_id, lo, hi, stream);
}

extern "C" int xad_rng_normal_f32(float* dst, std::size_t n, std::uint64_t seed, std::uint64_t stream_id, float mean,
                                  float stddev, void* stream) {
    return fill<Law::Normal>(dst, n, seed, stream_id, mean, stddev, stream);
}

extern "C" int xad_host_rng_bits(std::uint64_t* dst, std::size_t n, std::uint64_t seed, std::uint64_t stream_id,
                                 std::uint64_t first) {
    XAD_REQUIRE(n == 0 || dst, "xad_host_rng_bits: destination is null");
    const std::uint64_t key = xad_rng::stream_key(seed, stream_id);
    for (std::size_t i = 0; i < n; ++i) dst[i] = xad_rng::bits(key, first + i);
    return XAD_OK;
}

extern "C" int xad_host_rng_uniform_f32(float* dst, std::size_t n, std::uint64_t seed, std::uint64_t stream_id,
                                        float lo, float hi) {
    XAD_REQUIRE(n == 0 || dst, "xad_host_rng_uniform_f32: destination is null");
    const std::uint64_t key = xad_rng::stream_key(seed, stream_id);
    for (std::size_t i = 0; i < n; ++i) dst[i] = xad_rng::uniform(xad_rng::bits(key, i), lo, hi);
    return XAD_OK;
}
