/* Measurement instruments of this build: kernels and probes that bench.py and
 * the profiling runs use to justify design choices of libxad_hip.so.  They are
 * NOT part of the library's boundary (include/xad_capi.h): nothing here has a
 * counterpart in xyz-autodiff-cuda, and no product code loads this library.
 *
 * Built as instruments/libxad_instruments.so from instruments/instruments.hip
 * and the same device headers the product kernels come from
 * (xyz_autodiff_cuda_amd/csrc/chain_device.cuh), with the same compiler flags,
 * so a kernel measured here is the code the product launches.
 *
 * Every function returns 0 on success; xadi_last_error() gives the text of the
 * last failure on the calling thread.  Pointers are device memory of the
 * current HIP device unless stated; `stream` is a hipStream_t as void*.
 */
#ifndef XAD_INSTRUMENTS_H
#define XAD_INSTRUMENTS_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* xadi_last_error(void);
/* SHA-256 (hex) of the sources this library was built from (its build script records it). */
const char* xadi_source_digest(void);

/* The chain kernel of xad_chain_forward_backward_f32 with the lane-to-address mapping chosen by the
 * caller: problems_per_lane = 1 (4-byte accesses, what the product launches) or 4 (16-byte accesses;
 * needs all arrays 16-byte aligned, otherwise, and for the last n % 4 problems, the 4-byte kernel is
 * used).  Results are identical; only the time differs. */
int xadi_chain_forward_backward_f32_layout(size_t n,
                                           const float* sx, const float* sy, const float* theta,
                                           const float* o, const float* px, const float* py,
                                           float* w, float* d_sx, float* d_sy, float* d_theta,
                                           float* d_o, float* d_px, float* d_py,
                                           int problems_per_lane, void* stream);

/* The same kernel (one problem per lane, non-temporal loads) with its seven results stored as
 * 0 write-through stores (relaxed atomic stores at agent scope: the product's choice), 1 plain stores,
 * 2 non-temporal stores.  Same results; only the time differs. */
int xadi_chain_store_policy(int policy, size_t n,
                            const float* sx, const float* sy, const float* theta,
                            const float* o, const float* px, const float* py,
                            float* w, float* d_sx, float* d_sy, float* d_theta,
                            float* d_o, float* d_px, float* d_py, void* stream);

/* dst[i] = src[i] for n floats with the access pattern of the chain kernel: a copy of known size
 * to calibrate counters and bandwidth against. */
int xadi_stream_copy_f32(size_t n, const float* src, float* dst, void* stream);

/* The same copy in other shapes, to find the best this memory system gives one stream in and one out:
 * variant 0: 4 bytes per access, one access per lane, write-through stores; 1: 4 bytes, eight accesses of a
 * lane in flight, write-through; 2: 16 bytes, one, plain stores; 3: 16 bytes, four in flight, plain;
 * 4: 16 bytes, four, non-temporal stores; 5: 16 bytes read, written through as four 4-byte stores, two in
 * flight; 6: 4 bytes, eight in flight, plain.  All loads non-temporal.  n a multiple of 4, arrays 16-byte
 * aligned. */
int xadi_copy_variant_f32(int variant, size_t n, const float* src, float* dst, void* stream);

/* Resources of the chain kernel (write-through stores) as the loaded code object and the current
 * device report them: vector registers per lane, scratch (spill) bytes per lane, static LDS bytes per
 * block, lanes per block, and how many such blocks one compute unit holds at once.  out[5], host. */
int xadi_chain_kernel_resources(int* out);

/* Shader cycles the LDS pipeline of a CU spends on one wavefront-wide atomic add (16 wavefronts of
 * one block issuing back to back), by element type (0 float, 1 double, 2 uint32, 3 uint64) and
 * address pattern (0 sixty-four distinct addresses, 1 one address, 2 sixteen lanes on one address,
 * 3 eight lanes per address, 4 stride of six elements).  Synchronous; allocates and frees small
 * device buffers.  The accumulator's fp64 table rests on these numbers. */
int xadi_lds_atomic_cycles(int element, int pattern, double* cycles_per_instruction);

#ifdef __cplusplus
}
#endif
#endif /* XAD_INSTRUMENTS_H */
