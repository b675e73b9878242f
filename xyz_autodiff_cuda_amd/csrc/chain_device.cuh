#pragma once
// Device kernels of the per-thread forward+backward over structure-of-arrays buffers.
//
// Memory traffic per problem is fixed by the interface: 6 floats in, 7 floats
// out, 52 bytes, each touched once; the whole graph lives in VGPRs (no LDS, no
// scratch, no atomics), so the kernels are a 13-stream copy with arithmetic in
// the middle and the only design freedom is how lanes map to addresses and how
// the stores are issued.  The library launches chain_single_kernel with
// write-through stores; the other store policies, the four-problems-per-lane
// mapping and the plain copy exist so that those choices can be measured again
// (they are instantiated by the measurement library, not by the product).
#include <cstddef>
#include <type_traits>

#include <hip/hip_runtime.h>

#include <xyz_autodiff/soa.cuh>

#include "chain.cuh"

namespace xad_chain {

struct ChainBuffers {
    const float* in[6];  // sx, sy, theta, o, px, py
    float* out[7];       // w, d_sx, d_sy, d_theta, d_o, d_px, d_py
};

constexpr unsigned kQuadBlock = 256;
constexpr unsigned kSingleBlock = 512;

// How the seven results are stored.  Measured on MI355X in alternating trials of the same kernel
// body: relaxed atomic stores at agent scope (on gfx950 ordinary 4-byte stores with the sc1
// cache-policy bit: written through the L2 instead of being held there) 6.18-6.20 TB/s, plain stores
// 5.91-5.92, non-temporal stores 5.80-5.81.
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

// One lane, one problem, 4-byte accesses; problems first .. n-1.  Non-temporal loads (nothing is reused).
// Each wavefront instruction covers 256 contiguous bytes of one array and a 512-lane block 2 KiB of
// each: the faster mapping on MI355X for 13 concurrent streams.
template <StorePolicy P>
__global__ void __launch_bounds__(kSingleBlock) chain_single_kernel(ChainBuffers buf, std::size_t first, std::size_t n) {
    const std::size_t i = first + static_cast<std::size_t>(blockIdx.x) * kSingleBlock + threadIdx.x;
    if (i >= n) return;
    float x[6];
#pragma unroll
    for (int a = 0; a < 6; ++a) x[a] = __builtin_nontemporal_load(buf.in[a] + i);
    const auto r = forward_backward<float>(x[0], x[1], x[2], x[3], x[4], x[5]);
    const float y[7] = {r.w, r.d_sx, r.d_sy, r.d_theta, r.d_o, r.d_px, r.d_py};
#pragma unroll
    for (int a = 0; a < 7; ++a) store_result<P>(buf.out[a] + i, y[a]);
}

// One lane, four consecutive problems, 16-byte accesses (1 KiB per wavefront instruction).  `groups` = n / 4.
// (A template, like the copy below, so that only a translation unit that launches it carries its code.)
template <int kUnused = 0>
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
        const auto r = forward_backward<float>(in[0][k], in[1][k], in[2][k], in[3][k], in[4][k], in[5][k]);
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

// Plain copy with the chain kernel's access pattern (4 bytes per lane, non-temporal):
// the yardstick that hardware counters and achievable bandwidth are scaled by.
template <int kUnused = 0>
__global__ void __launch_bounds__(kSingleBlock) stream_copy_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                                   std::size_t n) {
    const std::size_t i = static_cast<std::size_t>(blockIdx.x) * kSingleBlock + threadIdx.x;
    if (i < n) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// Plain copies in other shapes, to find what this memory system gives a copy at best: kFloats floats per
// access (1 or 4: 4 or 16 bytes), kInFlight accesses of a lane issued before the first store (each a block's
// width apart, so every wavefront instruction stays contiguous), stores by policy P.
template <int kFloats, int kInFlight, StorePolicy P>
__global__ void __launch_bounds__(kSingleBlock) copy_variant_kernel(const float* __restrict__ src, float* __restrict__ dst,
                                                                    std::size_t n) {
    typedef float NativeFloat4 __attribute__((ext_vector_type(4)));
    using Word = std::conditional_t<kFloats == 4, NativeFloat4, float>;
    const std::size_t words = n / kFloats;
    const std::size_t base = static_cast<std::size_t>(blockIdx.x) * kSingleBlock * kInFlight + threadIdx.x;
    const Word* in = reinterpret_cast<const Word*>(src);
    Word* out = reinterpret_cast<Word*>(dst);
    Word v[kInFlight];
#pragma unroll
    for (int k = 0; k < kInFlight; ++k) {
        const std::size_t i = base + static_cast<std::size_t>(k) * kSingleBlock;
        if (i < words) v[k] = __builtin_nontemporal_load(in + i);
    }
#pragma unroll
    for (int k = 0; k < kInFlight; ++k) {
        const std::size_t i = base + static_cast<std::size_t>(k) * kSingleBlock;
        if (i < words) {
            if constexpr (kFloats == 1) {
                store_result<P>(out + i, v[k]);
            } else if constexpr (P == StorePolicy::NonTemporal) {
                __builtin_nontemporal_store(v[k], out + i);
            } else if constexpr (P == StorePolicy::WriteThrough) {
                float* o = reinterpret_cast<float*>(out + i);
                store_result<P>(o, v[k].x);
                store_result<P>(o + 1, v[k].y);
                store_result<P>(o + 2, v[k].z);
                store_result<P>(o + 3, v[k].w);
            } else {
                out[i] = v[k];
            }
        }
    }
}

}  // namespace xad_chain
