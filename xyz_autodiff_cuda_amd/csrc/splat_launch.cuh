#pragma once
// Host-callable launchers of the splatting kernels, of the binning stage and of the depth sort, each
// in a translation unit of its own.
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "splat.cuh"

namespace xad_splat {

// Words of the step's status block on the device (read by the host whenever it next waits for the stream).
enum : int {
    kStatusPairs = 0,         // (tile, Gaussian) pairs of the last binning
    kStatusOverflow = 1,      // 1 if the pairs did not fit the lists: the lists of that step are incomplete
    kStatusSuperPairs = 2,    // (supertile, Gaussian) pairs
    kStatusDepthChanged = 3,  // 1 if a depth differed from the depths the kept order was computed from
    kStatusOverflowSticky = 4,  // largest pair count of any step that overflowed since the host last cleared this word
    kStatusStickyBefore = 5,    // that word as it stood when the last step began: what steps before it left there
    kStatusWords = 6,
};

// Also sets status[kStatusDepthChanged] if any depth differs (bitwise) from ordered_depth, and zeroes
// record_grads (G rows of kRecordGradStride floats) and *loss for the compositing backward.
// rank[g] = position of Gaussian g in the depth order: the rectangle is also written to rects_by_depth[rank[g]].
int launch_project(hipStream_t s, int G, const float* params, const float* depth, const float* ordered_depth,
                   const std::uint32_t* rank, std::uint32_t* status, int width, int height, Record* records, TileRect* rects,
                   TileRect* rects_by_depth, float* record_grads, double* loss, bool first_of_step);

// Binning (splat_binning.hip): tile lists from tile rectangles, Gaussians taken in the order by_depth.
constexpr std::uint32_t kBinRangeB = 64;  // list entries a wavefront handles at level B: one per lane
struct BinPlan {
    int G, tiles_x, tiles_y;
    int super_x, super_y;          // supertiles of 8 x 8 tiles across and down the image
    int group_x, groups;           // groups of 8 x 8 supertiles: across the image, and in all
    int supers;                    // supertile numbers: 64 per group, whether inside the image or not
    int range_a, ranges_a;         // Gaussians per wavefront at level A, and how many such ranges
    std::uint32_t capacity;        // (tile, Gaussian) pairs the lists can hold
    std::uint32_t capacity_a;      // (supertile, Gaussian) pairs level A may produce: at most capacity (the buffer's size)
    std::uint32_t waves_b;         // wavefronts launched at level B: capacity_a / kBinRangeB + supers
};
constexpr int kScanControlWords = 3;
struct BinScratch {
    std::uint32_t* matrix_a = nullptr;    // bin_matrix_a_words: counts, then offsets, per (supertile, range)
    std::uint32_t* matrix_b = nullptr;    // bin_matrix_b_words: the same per (tile, range of its supertile's list)
    std::uint32_t* list_a = nullptr;      // capacity: the supertiles' lists
    std::uint32_t* first_wave = nullptr;  // supers + 1
    std::uint64_t* scan_state = nullptr;  // bin_scan_state_words, zero before the first launch
    std::uint32_t* scan_control = nullptr;  // kScanControlWords: tickets given out, blocks finished (both zero between launches), epoch (never zero)
};
// The buffers are sized by a plan with capacity_a = capacity; a plan with a smaller capacity_a (once the host
// has seen how many supertile pairs a scene produces) uses less of them and launches fewer wavefronts.
BinPlan make_bin_plan(int G, int tiles_x, int tiles_y, std::uint32_t capacity, std::uint32_t capacity_a);
std::size_t bin_matrix_a_words(const BinPlan& p);
std::size_t bin_matrix_b_words(const BinPlan& p);
std::size_t bin_scan_state_words(const BinPlan& p);
// Fills list (capacity entries), range_begin / range_end (one entry per tile, adjacent arrays) and
// status[kStatusPairs, kStatusOverflow, kStatusSuperPairs]; clears status[kStatusDepthChanged] when asked to.
// rects_by_depth[i] = rects[by_depth[i]].
int launch_binning(hipStream_t s, const BinPlan& p, const std::uint32_t* by_depth, const TileRect* rects_by_depth,
                   const TileRect* rects, BinScratch& scratch,
                   std::uint32_t* list, std::uint32_t* range_begin, std::uint32_t* range_end, std::uint32_t* status,
                   bool clear_depth_flag);
int launch_render_forward(hipStream_t s, int width, int height, const std::uint32_t* range_begin,
                          const std::uint32_t* range_end, const std::uint32_t* sorted_ids, const Record* records,
                          float* image, float* final_T, std::uint32_t* n_contrib, int segments, float4* segment_state,
                          std::uint32_t* tile_order);
int launch_render_backward(hipStream_t s, int width, int height, const std::uint32_t* range_begin,
                           const std::uint32_t* range_end, const std::uint32_t* sorted_ids, const Record* records,
                           const float* image, const float* target, const float* final_T,
                           const std::uint32_t* n_contrib, float* record_grads, double* loss, int segments,
                           const float4* segment_state, const std::uint32_t* tile_order);
// tile_order: 8 * ceil(tiles / 8) words, written by launch_render_forward (the order, longest list first within
// each XCD's band of tiles, in which the blocks of both kernels take the tiles) and read by launch_render_backward.
// Pieces a tile's list is cut into for the backward walk (1, 2, 4 or 8: more for images with few tiles);
// segment_state holds that many float4 per pixel when it is more than one.
int render_segments(int width, int height);
// Also adds the parts of the loss up into loss[0].
int launch_gaussian_backward(hipStream_t s, int G, const float* params, const float* record_grads, float* grads, double* loss);

// The depth order (splat_sort.hip): by_depth = the Gaussians in (depth, index) order, rank its inverse
// (rank[by_depth[i]] = i), ordered_depth = a copy of depth.  keys_a, keys_b, values_a: G words each of scratch;
// temp: depth_sort_temp_bytes(G) bytes that are zero before the first sort and are left ready by every sort.
std::size_t depth_sort_temp_bytes(int G);
std::size_t depth_sort_gave_up_offset();  // byte offset in temp of a word that counts blocks whose bounded wait ran out
int sort_by_depth(hipStream_t s, void* temp, std::size_t temp_bytes, const float* depth, std::uint32_t* keys_a,
                  std::uint32_t* keys_b, std::uint32_t* values_a, std::uint32_t* by_depth, std::uint32_t* rank,
                  float* ordered_depth, int G);

}  // namespace xad_splat
