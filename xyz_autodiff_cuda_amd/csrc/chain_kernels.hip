// Per-thread forward+backward of the benchmark graph over structure-of-arrays
// buffers: the launcher of the GPU kernel (chain_device.cuh), the host-core
// build of the same body, and their C-ABI entry points.
#include <algorithm>
#include <thread>
#include <vector>

#include "chain_device.cuh"
#include "common.cuh"

namespace {

using xad_chain::ChainBuffers;
using xad_chain::kSingleBlock;
using xad_chain::StorePolicy;

template <typename T>
void host_chain_range(std::size_t begin, std::size_t end, const T* const* in, T* const* out) {
    for (std::size_t i = begin; i < end; ++i) {
        const auto r = xad_chain::forward_backward<T>(in[0][i], in[1][i], in[2][i], in[3][i], in[4][i], in[5][i]);
        out[0][i] = r.w;
        out[1][i] = r.d_sx;
        out[2][i] = r.d_sy;
        out[3][i] = r.d_theta;
        out[4][i] = r.d_o;
        out[5][i] = r.d_px;
        out[6][i] = r.d_py;
    }
}

template <typename T>
int host_chain(std::size_t n, const T* const* in, T* const* out, int num_threads) {
    for (int a = 0; a < 6; ++a) XAD_REQUIRE(n == 0 || in[a], "host chain: input array %d is null", a);
    for (int a = 0; a < 7; ++a) XAD_REQUIRE(n == 0 || out[a], "host chain: output array %d is null", a);
    unsigned threads = num_threads > 0 ? static_cast<unsigned>(num_threads) : std::thread::hardware_concurrency();
    if (threads == 0) threads = 1;
    threads = static_cast<unsigned>(std::min<std::size_t>(threads, std::max<std::size_t>(n / 1024, 1)));
    if (threads == 1) {
        host_chain_range<T>(0, n, in, out);
        return XAD_OK;
    }
    std::vector<std::thread> pool;
    pool.reserve(threads);
    const std::size_t chunk = (n + threads - 1) / threads;
    for (unsigned t = 0; t < threads; ++t) {
        const std::size_t b = std::min(n, t * chunk), e = std::min(n, b + chunk);
        pool.emplace_back(host_chain_range<T>, b, e, in, out);
    }
    for (auto& th : pool) th.join();
    return XAD_OK;
}

}  // namespace

extern "C" int xad_chain_forward_backward_f32(std::size_t n, const float* sx, const float* sy, const float* theta,
                                              const float* o, const float* px, const float* py, float* w,
                                              float* d_sx, float* d_sy, float* d_theta, float* d_o, float* d_px,
                                              float* d_py, void* stream) {
    const char* who = "xad_chain_forward_backward_f32";
    const ChainBuffers buf{{sx, sy, theta, o, px, py}, {w, d_sx, d_sy, d_theta, d_o, d_px, d_py}};
    if (n == 0) return XAD_OK;
    for (int a = 0; a < 6; ++a) XAD_REQUIRE(buf.in[a], "%s: input array %d is null", who, a);
    for (int a = 0; a < 7; ++a) XAD_REQUIRE(buf.out[a], "%s: output array %d is null", who, a);
    // a launch holds fewer than 2^32 lanes; larger arrays (they fit: 13 arrays of 2^32 floats are 223 GB) take several
    constexpr std::size_t kLaunchLanes = (std::size_t(1) << 32) - (std::size_t(1) << 20);
    hipStream_t s = xad::as_stream(stream);
    for (std::size_t done = 0; done < n;) {
        const std::size_t part = std::min(n - done, kLaunchLanes);
        hipLaunchKernelGGL(xad_chain::chain_single_kernel<StorePolicy::WriteThrough>, dim3(xad::blocks_for(part, kSingleBlock)),
                           dim3(kSingleBlock), 0, s, buf, done, done + part);
        XAD_HIP_TRY(hipGetLastError());
        done += part;
    }
    return XAD_OK;
}

extern "C" int xad_host_chain_forward_backward_f32(std::size_t n, const float* sx, const float* sy,
                                                   const float* theta, const float* o, const float* px,
                                                   const float* py, float* w, float* d_sx, float* d_sy,
                                                   float* d_theta, float* d_o, float* d_px, float* d_py,
                                                   int num_threads) {
    const float* in[6] = {sx, sy, theta, o, px, py};
    float* out[7] = {w, d_sx, d_sy, d_theta, d_o, d_px, d_py};
    return host_chain<float>(n, in, out, num_threads);
}

extern "C" int xad_host_chain_forward_backward_f64(std::size_t n, const double* sx, const double* sy,
                                                   const double* theta, const double* o, const double* px,
                                                   const double* py, double* w, double* d_sx, double* d_sy,
                                                   double* d_theta, double* d_o, double* d_px, double* d_py,
                                                   int num_threads) {
    const double* in[6] = {sx, sy, theta, o, px, py};
    double* out[7] = {w, d_sx, d_sy, d_theta, d_o, d_px, d_py};
    return host_chain<double>(n, in, out, num_threads);
}
