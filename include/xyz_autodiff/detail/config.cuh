#pragma once
// Compilation modes of the library.
//
//  * hipcc (HIP language): the HIP runtime header supplies __host__/__device__
//    and every accessor is usable from gfx950 kernels and from the host pass.
//  * a plain C++20 host compiler (g++, clang++): the attribute macros expand to
//    nothing, so the very same templates build for the host cores.  That build
//    is what the host-core throughput run and the CPU test tier use.
//
// XAD_HD marks a function callable from both sides, XAD_INLINE additionally
// forces inlining: a graph of nodes only stays in VGPRs when every accessor of
// it disappears into the calling kernel.

#include <cstddef>
#include <cstdint>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define XAD_HD __host__ __device__
#define XAD_INLINE __host__ __device__ __forceinline__
#else
#ifndef __host__
#define __host__
#endif
#ifndef __device__
#define __device__
#endif
#ifndef __forceinline__
#define __forceinline__ inline __attribute__((always_inline))
#endif
#define XAD_HD
#define XAD_INLINE inline __attribute__((always_inline))
#endif

// Full unrolling of the fixed trip-count loops (1..16 iterations) is what lets
// scalar replacement turn data_[N]/grad_[N] into individual registers.
#if defined(__clang__)
#define XAD_UNROLL _Pragma("unroll")
#elif defined(__GNUC__)
#define XAD_UNROLL _Pragma("GCC unroll 16")
#else
#define XAD_UNROLL
#endif

// True while compiling the gfx950 pass of a HIP translation unit.
#if defined(__HIP_DEVICE_COMPILE__) && __HIP_DEVICE_COMPILE__
#define XAD_DEVICE_PASS 1
#else
#define XAD_DEVICE_PASS 0
#endif
