// Measurement instruments (see xad_instruments.h): the alternative forms of the chain kernel, a
// plain copy, the chain kernel's resources, and the LDS atomic probe.  Not part of the product.
#include <algorithm>
#include <vector>

#include "../xyz_autodiff_cuda_amd/csrc/chain_device.cuh"
#include "../xyz_autodiff_cuda_amd/csrc/common.cuh"
#include "xad_instruments.h"

#define XADI_EXPORT extern "C" __attribute__((visibility("default")))

namespace xad {
// this library's own error text (the build hides every symbol but the xadi_ entry points)
char* last_error_buffer() {
    static thread_local char buffer[kLastErrorCapacity] = {0};
    return buffer;
}
}  // namespace xad

#ifndef XADI_SOURCE_DIGEST
#define XADI_SOURCE_DIGEST ""
#endif
XADI_EXPORT const char* xadi_last_error(void) { return xad::last_error_buffer(); }
XADI_EXPORT const char* xadi_source_digest(void) { return XADI_SOURCE_DIGEST; }

namespace {

using xad_chain::ChainBuffers;
using xad_chain::kQuadBlock;
using xad_chain::kSingleBlock;
using xad_chain::StorePolicy;

int check_buffers(const ChainBuffers& buf, const char* who) {
    for (int a = 0; a < 6; ++a) XAD_REQUIRE(buf.in[a], "%s: input array %d is null", who, a);
    for (int a = 0; a < 7; ++a) XAD_REQUIRE(buf.out[a], "%s: output array %d is null", who, a);
    return 0;
}

}  // namespace

XADI_EXPORT int xadi_chain_forward_backward_f32_layout(std::size_t n, const float* sx, const float* sy,
                                                       const float* theta, const float* o, const float* px,
                                                       const float* py, float* w, float* d_sx, float* d_sy,
                                                       float* d_theta, float* d_o, float* d_px, float* d_py,
                                                       int problems_per_lane, void* stream) {
    const char* who = "xadi_chain_forward_backward_f32_layout";
    const ChainBuffers buf{{sx, sy, theta, o, px, py}, {w, d_sx, d_sy, d_theta, d_o, d_px, d_py}};
    if (n == 0) return 0;
    XAD_REQUIRE(problems_per_lane == 1 || problems_per_lane == 4, "%s: problems_per_lane must be 1 or 4, got %d", who,
                problems_per_lane);
    if (int st = check_buffers(buf, who)) return st;
    bool vector_ok = problems_per_lane == 4;
    for (int a = 0; a < 6; ++a) vector_ok = vector_ok && xad::aligned16(buf.in[a]);
    for (int a = 0; a < 7; ++a) vector_ok = vector_ok && xad::aligned16(buf.out[a]);
    XAD_REQUIRE(n <= 0x7fffffffull * 64, "%s: n = %zu exceeds one launch", who, n);
    hipStream_t s = xad::as_stream(stream);
    const std::size_t groups = vector_ok ? n / 4 : 0;
    if (groups) {
        hipLaunchKernelGGL(xad_chain::chain_quad_kernel<>, dim3(xad::blocks_for(groups, kQuadBlock)), dim3(kQuadBlock), 0, s,
                           buf, groups);
        XAD_HIP_TRY(hipGetLastError());
    }
    if (groups * 4 < n) {
        hipLaunchKernelGGL(xad_chain::chain_single_kernel<StorePolicy::WriteThrough>,
                           dim3(xad::blocks_for(n - groups * 4, kSingleBlock)), dim3(kSingleBlock), 0, s, buf, groups * 4, n);
        XAD_HIP_TRY(hipGetLastError());
    }
    return 0;
}

XADI_EXPORT int xadi_chain_store_policy(int policy, std::size_t n, const float* sx, const float* sy, const float* theta,
                                        const float* o, const float* px, const float* py, float* w, float* d_sx,
                                        float* d_sy, float* d_theta, float* d_o, float* d_px, float* d_py,
                                        void* stream) {
    const char* who = "xadi_chain_store_policy";
    const ChainBuffers buf{{sx, sy, theta, o, px, py}, {w, d_sx, d_sy, d_theta, d_o, d_px, d_py}};
    if (n == 0) return 0;
    if (int st = check_buffers(buf, who)) return st;
    XAD_REQUIRE(n <= 0x7fffffffull * 64, "%s: n = %zu exceeds the grid limit", who, n);
    const dim3 grid(xad::blocks_for(n, kSingleBlock)), block(kSingleBlock);
    hipStream_t s = xad::as_stream(stream);
    switch (policy) {
        case 0: hipLaunchKernelGGL(xad_chain::chain_single_kernel<StorePolicy::WriteThrough>, grid, block, 0, s, buf, 0, n); break;
        case 1: hipLaunchKernelGGL(xad_chain::chain_single_kernel<StorePolicy::Plain>, grid, block, 0, s, buf, 0, n); break;
        case 2: hipLaunchKernelGGL(xad_chain::chain_single_kernel<StorePolicy::NonTemporal>, grid, block, 0, s, buf, 0, n); break;
        default: return xad::fail(XAD_ERR_INVALID_ARGUMENT, "%s: policy must be 0, 1 or 2, got %d", who, policy);
    }
    XAD_HIP_TRY(hipGetLastError());
    return 0;
}

XADI_EXPORT int xadi_stream_copy_f32(std::size_t n, const float* src, float* dst, void* stream) {
    if (n == 0) return 0;
    XAD_REQUIRE(src && dst, "xadi_stream_copy_f32: null array");
    XAD_REQUIRE(n <= 0x7fffffffull * 64, "xadi_stream_copy_f32: n = %zu exceeds the grid limit", n);
    hipLaunchKernelGGL(xad_chain::stream_copy_kernel<>, dim3(xad::blocks_for(n, kSingleBlock)), dim3(kSingleBlock), 0,
                       xad::as_stream(stream), src, dst, n);
    XAD_HIP_TRY(hipGetLastError());
    return 0;
}

XADI_EXPORT int xadi_copy_variant_f32(int variant, std::size_t n, const float* src, float* dst, void* stream) {
    const char* who = "xadi_copy_variant_f32";
    if (n == 0) return 0;
    XAD_REQUIRE(src && dst, "%s: null array", who);
    XAD_REQUIRE(n % 4 == 0 && xad::aligned16(src) && xad::aligned16(dst), "%s: n must be a multiple of 4 and the arrays 16-byte aligned", who);
    XAD_REQUIRE(n <= 0x7fffffffull * 64, "%s: n = %zu exceeds the grid limit", who, n);
    hipStream_t s = xad::as_stream(stream);
    auto launch = [&](auto kernel, int floats, int in_flight) {
        const std::size_t per_block = static_cast<std::size_t>(kSingleBlock) * floats * in_flight;
        hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>((n + per_block - 1) / per_block)), dim3(kSingleBlock), 0, s, src, dst, n);
    };
    using xad_chain::copy_variant_kernel;
    switch (variant) {
        case 0: launch(copy_variant_kernel<1, 1, StorePolicy::WriteThrough>, 1, 1); break;
        case 1: launch(copy_variant_kernel<1, 8, StorePolicy::WriteThrough>, 1, 8); break;
        case 2: launch(copy_variant_kernel<4, 1, StorePolicy::Plain>, 4, 1); break;
        case 3: launch(copy_variant_kernel<4, 4, StorePolicy::Plain>, 4, 4); break;
        case 4: launch(copy_variant_kernel<4, 4, StorePolicy::NonTemporal>, 4, 4); break;
        case 5: launch(copy_variant_kernel<4, 2, StorePolicy::WriteThrough>, 4, 2); break;
        case 6: launch(copy_variant_kernel<1, 8, StorePolicy::Plain>, 1, 8); break;
        default: return xad::fail(XAD_ERR_INVALID_ARGUMENT, "%s: variant must be 0..6, got %d", who, variant);
    }
    XAD_HIP_TRY(hipGetLastError());
    return 0;
}

XADI_EXPORT int xadi_chain_kernel_resources(int* out) {
    XAD_REQUIRE(out, "xadi_chain_kernel_resources: out is null");
    const void* kernel = reinterpret_cast<const void*>(xad_chain::chain_single_kernel<StorePolicy::WriteThrough>);
    hipFuncAttributes attr;
    XAD_HIP_TRY(hipFuncGetAttributes(&attr, kernel));
    int blocks_per_cu = 0;
    XAD_HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks_per_cu, kernel, static_cast<int>(kSingleBlock), 0));
    out[0] = attr.numRegs;
    out[1] = static_cast<int>(attr.localSizeBytes);
    out[2] = static_cast<int>(attr.sharedSizeBytes);
    out[3] = static_cast<int>(kSingleBlock);
    out[4] = blocks_per_cu;
    return 0;
}

// ---- cost of LDS atomic adds by element type and address pattern ----------------------------------
namespace {

constexpr int kWaves = 16;
constexpr int kBlocks = 256;

template <typename T>
__global__ void __launch_bounds__(kWaves * 64) lds_atomic_probe_kernel(int pattern, int iterations, T* sink,
                                                                       long long* cycles) {
    __shared__ T table[4096];
    for (int i = threadIdx.x; i < 4096; i += blockDim.x) table[i] = T(0);
    __syncthreads();
    const int lane = threadIdx.x & 63;
    int at;
    switch (pattern) {
        case 0: at = lane; break;                   // 64 distinct consecutive addresses
        case 1: at = 0; break;                      // all lanes one address
        case 2: at = lane < 16 ? 0 : lane; break;   // 16 lanes share an address
        case 3: at = lane & 7; break;               // eight lanes per address
        default: at = lane * 6; break;              // stride of six elements
    }
    T v = T(1) + T(lane);
    const long long t0 = clock64();
    for (int i = 0; i < iterations; ++i) {
        atomicAdd(&table[at], v);
        v += T(1);
    }
    __syncthreads();
    const long long t1 = clock64();
    if (threadIdx.x == 0) cycles[blockIdx.x] = t1 - t0;
    if (threadIdx.x < 64) sink[blockIdx.x * 64 + threadIdx.x] = table[threadIdx.x];
}

template <typename T>
int run_probe(int pattern, double* cycles_per_instruction) {
    const int iterations = 1000;
    T* sink = nullptr;
    long long* cycles = nullptr;
    XAD_HIP_TRY(hipMalloc(&sink, sizeof(T) * kBlocks * 64));
    hipError_t st = hipMalloc(&cycles, sizeof(long long) * kBlocks);
    std::vector<long long> host(kBlocks);
    if (st == hipSuccess) {
        for (int rep = 0; rep < 2; ++rep)  // the second launch is the measurement
            hipLaunchKernelGGL(lds_atomic_probe_kernel<T>, dim3(kBlocks), dim3(kWaves * 64), 0, nullptr, pattern, iterations, sink,
                               cycles);
        st = hipDeviceSynchronize();
    }
    if (st == hipSuccess) st = hipMemcpy(host.data(), cycles, sizeof(long long) * kBlocks, hipMemcpyDeviceToHost);
    (void)hipFree(sink);
    (void)hipFree(cycles);
    if (st != hipSuccess) return xad::fail(XAD_ERR_HIP, "xadi_lds_atomic_cycles: %s", hipGetErrorString(st));
    double total = 0.0;
    for (long long c : host) total += static_cast<double>(c);
    // 16 wavefronts share one LDS pipeline: cycles the pipeline spends per wavefront instruction
    *cycles_per_instruction = total / kBlocks / iterations / kWaves;
    return XAD_OK;
}

}  // namespace

XADI_EXPORT int xadi_lds_atomic_cycles(int element, int pattern, double* cycles_per_instruction) {
    XAD_REQUIRE(cycles_per_instruction, "xadi_lds_atomic_cycles: output is null");
    XAD_REQUIRE(pattern >= 0 && pattern <= 4, "xadi_lds_atomic_cycles: pattern must be 0..4, got %d", pattern);
    switch (element) {
        case 0: return run_probe<float>(pattern, cycles_per_instruction);
        case 1: return run_probe<double>(pattern, cycles_per_instruction);
        case 2: return run_probe<unsigned int>(pattern, cycles_per_instruction);
        case 3: return run_probe<unsigned long long>(pattern, cycles_per_instruction);
        default: return xad::fail(XAD_ERR_INVALID_ARGUMENT, "xadi_lds_atomic_cycles: element must be 0..3, got %d", element);
    }
}
