#pragma once
// Host-callable launchers of the splatting kernels and of the scan/sort stage,
// so that the translation unit that instantiates the device-wide primitives is
// compiled separately from the hand-written kernels.
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "splat.cuh"

namespace xad_splat {

int launch_project(hipStream_t s, int G, const float* params, int width, int height, Record* records, TileRect* rects,
                   std::uint32_t* counts);
int launch_emit(hipStream_t s, int G, const TileRect* rects, const std::uint32_t* offsets, const float* depth,
                int tiles_x, std::uint64_t* keys, std::uint32_t* values, std::uint32_t capacity);
int launch_ranges(hipStream_t s, std::uint32_t K, const std::uint64_t* keys, std::uint32_t* range_begin,
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
// counts (offsets has G + 1 entries, the last is the number of pairs) and the
// stable radix sort of the (tile | depth, index) pairs.
std::size_t scan_temp_bytes(int G);
int exclusive_scan_counts(hipStream_t s, void* temp, std::size_t temp_bytes, const std::uint32_t* counts,
                          std::uint32_t* offsets, int G);
std::size_t sort_temp_bytes(std::uint32_t capacity);
int sort_pairs(hipStream_t s, void* temp, std::size_t temp_bytes, const std::uint64_t* keys_in, std::uint64_t* keys_out,
               const std::uint32_t* values_in, std::uint32_t* values_out, std::uint32_t K, int key_bits);

}  // namespace xad_splat
