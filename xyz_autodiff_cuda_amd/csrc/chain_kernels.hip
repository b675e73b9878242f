// Per-thread forward+backward of the benchmark graph over structure-of-arrays
// buffers: the GPU kernels, the host-core build of the same body, and their
// C-ABI entry points.
//
// Memory traffic per problem is fixed by the interface: 6 floats in, 7 floats
// out, 52 bytes, each touched once; the whole graph lives in VGPRs (no LDS, no
// scratch, no atomics), so the kernels are a 13-stream copy with arithmetic in
// the middle and the only design freedom is how lanes map to addresses.  Two
// mappings are built:
//   - one problem per lane, 4-byte accesses, 512-lane blocks: each wavefront
//     instruction covers 256 contiguous bytes of one array and a block covers
//     2 KiB of each.  This is the faster one on MI355X for 13 concurrent streams
//     (measured ~5.9 TB/s against ~5.0 TB/s) and the default;
//   - four consecutive problems per lane, 16-byte accesses (1 KiB per wavefront
//     instruction), selectable for comparison.
// Loads are marked non-temporal (nothing is reused).  Stores of the default
// kernel are relaxed atomic stores at agent scope, which on gfx950 are ordinary
// 4-byte stores with the sc1 cache-policy bit (written through the L2 instead of
// being held there).  Measured in alternating trials of the same kernel body:
// 6.18-6.20 TB/s, against 5.91-5.92 with plain stores, 5.80-5.81 with
// non-temporal stores, 5.99-6.04 with sc1 and nt together, and 5.67 with plain
// loads and stores; the stream-copy yardstick and the 16-byte kernel keep
// non-temporal stores.
#include <algorithm>
#include <thread>
#include <vector>

#include <xyz_autodiff/soa.cuh>

#include "chain.cuh"
#include "common.cuh"

namespace {

using xyz_autodiff::soa::Quad;

struct ChainBuffers {
    const float* in[6];  // sx, sy, theta, o, px, py
    float* out[7];       // w, d_sx, d_sy, d_theta, d_o, d_px, d_py
};

constexpr unsigned kQuadBlock = 256;
constexpr unsigned kSingleBlock = 512;

// One lane, four consecutive problems, 16-byte accesses.  `groups` = n / 4.
__global__ void __launch_bounds__(kQuadBlock) chain_quad_kernel(ChainBuffers buf, std::size_t groups) {
    using namespace xyz_autodiff::soa;
    const std::size_t g = static_cast<std::size_t>(blockIdx.x) * kQuadBlock + threadIdx.x;
    if (g >= groups) return;

    Quad<float> in[6];
#pragma unroll
    for (int a = 0; a < 6; ++a) in[a] = load4_stream(buf.in[a], g);

    Quad<float> out[7];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const auto r = xad_chain::forward_backward<float>(in[0][k], in[1][k], in[2][k], in[3][k], in[4][k], in[5][k]);
        out[0][k] = r.w;
        out[1][k] = r.d_sx;
        out[2][k] = r.d_sy;
        out[3][k] = r.d_theta;
        out[4][k] = r.d_o;
        out[5][k] = r.d_px;
        out[6][k] = r.d_py;
    }
#pragma unroll
    for (int a = 0; a < 7; ++a) store4_stream(buf.out[a], g, out[a]);
}

// How the seven results are stored.  WriteThrough is what the library uses; the other two exist
// so that the choice can be measured again (xad_probe_chain_store_policy).
enum class StorePolicy { WriteThrough = 0, Plain = 1, NonTemporal = 2 };

template <StorePolicy P>
__device__ __forceinline__ void store_result(float* address, float value) {
    if constexpr (P == StorePolicy::WriteThrough)
        __hip_atomic_store(address, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // global_store_dword ... sc1
    else if constexpr (P == StorePolicy::Plain)
        *address = value;
    else
        __builtin_nontemporal_store(value, address);
}

// One lane, one problem, 4-byte accesses; problems first .. n-1.  Non-temporal loads.
template <StorePolicy P>
__global__ void __launch_bounds__(kSingleBlock) chain_single_kernel(ChainBuffers buf, std::size_t first, std::size_t n) {
    const std::size_t i = first + static_cast<std::size_t>(blockIdx.x) * kSingleBlock + threadIdx.x;
    if (i >= n) return;
    float x[6];
#pragma unroll
    for (int a = 0; a < 6; ++a) x[a] = __builtin_nontemporal_load(buf.in[a] + i);
    const auto r = xad_chain::forward_backward<float>(x[0], x[1], x[2], x[3], x[4], x[5]);
    const float y[7] = {r.w, r.d_sx, r.d_sy, r.d_theta, r.d_o, r.d_px, r.d_py};
#pragma unroll
    for (int a = 0; a < 7; ++a) store_result<P>(buf.out[a] + i, y[a]);
}

// Plain copy with the chain kernel's access pattern (4 bytes per lane, non-temporal):
// the yardstick that hardware counters and achievable bandwidth are scaled by.
__global__ void __launch_bounds__(kSingleBlock) stream_copy_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                                   std::size_t n) {
    const std::size_t i = static_cast<std::size_t>(blockIdx.x) * kSingleBlock + threadIdx.x;
    if (i < n) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

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

namespace {

int launch_chain(std::size_t n, const ChainBuffers& buf, int problems_per_lane, void* stream, const char* who) {
    if (n == 0) return XAD_OK;
    XAD_REQUIRE(problems_per_lane == 1 || problems_per_lane == 4, "%s: problems_per_lane must be 1 or 4, got %d", who,
                problems_per_lane);
    bool vector_ok = problems_per_lane == 4;
    for (int a = 0; a < 6; ++a) {
        XAD_REQUIRE(buf.in[a], "%s: input array %d is null", who, a);
        vector_ok = vector_ok && xad::aligned16(buf.in[a]);
    }
    for (int a = 0; a < 7; ++a) {
        XAD_REQUIRE(buf.out[a], "%s: output array %d is null", who, a);
        vector_ok = vector_ok && xad::aligned16(buf.out[a]);
    }
    // a launch holds fewer than 2^32 lanes; larger arrays (they fit: 13 arrays of 2^32 floats are 223 GB) take several
    constexpr std::size_t kLaunchLanes = (std::size_t(1) << 32) - (std::size_t(1) << 20);
    hipStream_t s = xad::as_stream(stream);
    const std::size_t groups = vector_ok ? n / 4 : 0;
    XAD_REQUIRE(groups <= kLaunchLanes, "%s: n = %zu exceeds one launch of the four-problems-per-lane mapping", who, n);
    if (groups) {
        hipLaunchKernelGGL(chain_quad_kernel, dim3(xad::blocks_for(groups, kQuadBlock)), dim3(kQuadBlock), 0, s, buf,
                           groups);
        XAD_HIP_TRY(hipGetLastError());
    }
    for (std::size_t done = groups * 4; done < n;) {
        const std::size_t part = std::min(n - done, kLaunchLanes);
        hipLaunchKernelGGL(chain_single_kernel<StorePolicy::WriteThrough>, dim3(xad::blocks_for(part, kSingleBlock)),
                           dim3(kSingleBlock), 0, s, buf, done, done + part);
        XAD_HIP_TRY(hipGetLastError());
        done += part;
    }
    return XAD_OK;
}

}  // namespace

extern "C" int xad_chain_kernel_resources(int* out) {
    XAD_REQUIRE(out, "xad_chain_kernel_resources: out is null");
    const void* kernel = reinterpret_cast<const void*>(chain_single_kernel<StorePolicy::WriteThrough>);
    hipFuncAttributes attr;
    XAD_HIP_TRY(hipFuncGetAttributes(&attr, kernel));
    int blocks_per_cu = 0;
    XAD_HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks_per_cu, kernel, static_cast<int>(kSingleBlock), 0));
    out[0] = attr.numRegs;
    out[1] = static_cast<int>(attr.localSizeBytes);
    out[2] = static_cast<int>(attr.sharedSizeBytes);
    out[3] = static_cast<int>(kSingleBlock);
    out[4] = blocks_per_cu;
    return XAD_OK;
}

extern "C" int xad_probe_chain_store_policy(int policy, std::size_t n, const float* sx, const float* sy,
                                            const float* theta, const float* o, const float* px, const float* py,
                                            float* w, float* d_sx, float* d_sy, float* d_theta, float* d_o,
                                            float* d_px, float* d_py, void* stream) {
    const char* who = "xad_probe_chain_store_policy";
    const ChainBuffers buf{{sx, sy, theta, o, px, py}, {w, d_sx, d_sy, d_theta, d_o, d_px, d_py}};
    if (n == 0) return XAD_OK;
    for (int a = 0; a < 6; ++a) XAD_REQUIRE(buf.in[a], "%s: input array %d is null", who, a);
    for (int a = 0; a < 7; ++a) XAD_REQUIRE(buf.out[a], "%s: output array %d is null", who, a);
    XAD_REQUIRE(n <= 0x7fffffffull * 64, "%s: n = %zu exceeds the grid limit", who, n);
    const dim3 grid(xad::blocks_for(n, kSingleBlock)), block(kSingleBlock);
    hipStream_t s = xad::as_stream(stream);
    switch (policy) {
        case 0: hipLaunchKernelGGL(chain_single_kernel<StorePolicy::WriteThrough>, grid, block, 0, s, buf, 0, n); break;
        case 1: hipLaunchKernelGGL(chain_single_kernel<StorePolicy::Plain>, grid, block, 0, s, buf, 0, n); break;
        case 2: hipLaunchKernelGGL(chain_single_kernel<StorePolicy::NonTemporal>, grid, block, 0, s, buf, 0, n); break;
        default: return xad::fail(XAD_ERR_INVALID_ARGUMENT, "%s: policy must be 0, 1 or 2, got %d", who, policy);
    }
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

extern "C" int xad_chain_forward_backward_f32(std::size_t n, const float* sx, const float* sy, const float* theta,
                                              const float* o, const float* px, const float* py, float* w,
                                              float* d_sx, float* d_sy, float* d_theta, float* d_o, float* d_px,
                                              float* d_py, void* stream) {
    const ChainBuffers buf{{sx, sy, theta, o, px, py}, {w, d_sx, d_sy, d_theta, d_o, d_px, d_py}};
    return launch_chain(n, buf, 1, stream, "xad_chain_forward_backward_f32");
}

extern "C" int xad_chain_forward_backward_f32_layout(std::size_t n, const float* sx, const float* sy,
                                                     const float* theta, const float* o, const float* px,
                                                     const float* py, float* w, float* d_sx, float* d_sy,
                                                     float* d_theta, float* d_o, float* d_px, float* d_py,
                                                     int problems_per_lane, void* stream) {
    const ChainBuffers buf{{sx, sy, theta, o, px, py}, {w, d_sx, d_sy, d_theta, d_o, d_px, d_py}};
    return launch_chain(n, buf, problems_per_lane, stream, "xad_chain_forward_backward_f32_layout");
}

extern "C" int xad_stream_copy_f32(std::size_t n, const float* src, float* dst, void* stream) {
    if (n == 0) return XAD_OK;
    XAD_REQUIRE(src && dst, "xad_stream_copy_f32: null array");
    XAD_REQUIRE(n <= 0x7fffffffull * 64, "xad_stream_copy_f32: n = %zu exceeds the grid limit", n);
    hipLaunchKernelGGL(stream_copy_kernel, dim3(xad::blocks_for(n, kSingleBlock)), dim3(kSingleBlock), 0,
                       xad::as_stream(stream), src, dst, n);
    XAD_HIP_TRY(hipGetLastError());
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
