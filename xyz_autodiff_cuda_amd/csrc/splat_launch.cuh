#pragma once
// Host-callable launchers of the splatting kernels and of the scan/sort stage,
// so that the translation unit that instantiates the device-wide primitives is
// compiled separately from the hand-written kernels.
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "splat.cuh"

namespace xad_splat {

// Also sets *depth_changed to 1 if any depth differs (bitwise) from ordered_depth, and zeroes
// record_grads (G rows of kRecordGradStride floats) and *loss for the compositing backward.
int launch_project(hipStream_t s, int G, const float* params, const float* depth, const float* ordered_depth,
                   std::uint32_t* depth_changed, int width, int height, Record* records, TileRect* rects,
                   std::uint32_t* counts, float* record_grads, double* loss);
// Depth order: keys[g] = order-preserving bits of depth[g], identity[g] = g; the stable sort of
// those pairs gives by_depth.  counts_by_depth[i] = counts[by_depth[i]].
int launch_depth_keys(hipStream_t s, int G, const float* depth, std::uint32_t* keys, std::uint32_t* identity);
int launch_permute_counts(hipStream_t s, int G, const std::uint32_t* by_depth, const std::uint32_t* counts,
                          std::uint32_t* counts_by_depth);
// Pairs are emitted in depth order with the tile index as key: 16 bits wide, or 32 (wide_keys)
// when there are more than 65 536 tiles.
// Also zeroes the range_words words of tile_ranges and resets *depth_changed.
int launch_emit(hipStream_t s, int G, const std::uint32_t* by_depth, const TileRect* rects, const std::uint32_t* offsets,
                int tiles_x, bool wide_keys, void* keys, std::uint32_t* values, std::uint32_t capacity,
                std::uint32_t* tile_ranges, int range_words, std::uint32_t* depth_changed);
int launch_ranges(hipStream_t s, std::uint32_t K, bool wide_keys, const void* keys, std::uint32_t* range_begin,
                  std::uint32_t* range_end);
int launch_render_forward(hipStream_t s, int width, int height, const std::uint32_t* range_begin,
                          const std::uint32_t* range_end, const std::uint32_t* sorted_ids, const Record* records,
                          float* image, float* final_T, std::uint32_t* n_contrib);
int launch_render_backward(hipStream_t s, int width, int height, const std::uint32_t* range_begin,
                           const std::uint32_t* range_end, const std::uint32_t* sorted_ids, const Record* records,
                           const float* image, const float* target, const float* final_T,
                           const std::uint32_t* n_contrib, float* record_grads, double* loss);
int launch_gaussian_backward(hipStream_t s, int G, const float* params, const float* record_grads, float* grads);

// Device-wide primitives (rocPRIM): exclusive scan of the per-Gaussian tile
// counts (offsets has G + 1 entries, the last is the number of pairs), the
// stable radix sort of (depth bits, index) that yields the depth order, and the
// stable radix sort of the (tile, index) pairs over the `key_bits` bits of a tile index.
std::size_t scan_temp_bytes(int G);
int exclusive_scan_counts(hipStream_t s, void* temp, std::size_t temp_bytes, const std::uint32_t* counts,
                          std::uint32_t* offsets, int G);
std::size_t depth_sort_temp_bytes(int G);
int sort_by_depth(hipStream_t s, void* temp, std::size_t temp_bytes, const std::uint32_t* keys_in,
                  std::uint32_t* keys_out, const std::uint32_t* values_in, std::uint32_t* values_out, int G);
std::size_t sort_temp_bytes(std::uint32_t capacity, bool wide_keys);
int sort_pairs(hipStream_t s, void* temp, std::size_t temp_bytes, bool wide_keys, const void* keys_in, void* keys_out,
               const std::uint32_t* values_in, std::uint32_t* values_out, std::uint32_t K, int key_bits);

}  // namespace xad_splat
