// Kernels of the tile-binned splatting step: per-Gaussian projection, per-tile
// compositing forward and reverse-order backward, per-Gaussian parameter
// backward.  (The tile lists come from splat_binning.hip.)
//
// Every kernel is HBM-, LDS- or VALU-bound streaming work on small records;
// nothing here is a dense contraction.
#include <xyz_autodiff/accumulate.cuh>
#include <xyz_autodiff/variable.cuh>
#include <xyz_autodiff/operations/unary/exp_logic.cuh>
#include <xyz_autodiff/operations/unary/sigmoid_logic.cuh>
#include <xyz_autodiff/operations/unary/sym_matrix2_inv_logic.cuh>
#include <operations/covariance_generation.cuh>
#include <operations/mahalanobis_distance.cuh>

#include <type_traits>

#include "common.cuh"
#include "splat.cuh"
#include "splat_launch.cuh"
#include "splat_staged.cuh"

namespace xad_splat {

using namespace xyz_autodiff;

// ---------------------------------------------------------------------------
// Projection: one lane per Gaussian.  Builds the graph
//   es = exp(log-scale); cov = scale_rotation_to_covariance_3param(es, theta);
//   inv = sym_matrix2_inv(cov); alpha0 = sigmoid(opacity)
// from the library's nodes, runs it forward, and derives the 3-sigma tile
// rectangle.
__global__ void __launch_bounds__(256) project_kernel(int G, const float* __restrict__ params,
                                                      const float* __restrict__ depth,
                                                      const float* __restrict__ ordered_depth,
                                                      const std::uint32_t* __restrict__ rank,
                                                      std::uint32_t* __restrict__ status, int width, int height,
                                                      Record* __restrict__ records, TileRect* __restrict__ rects,
                                                      TileRect* __restrict__ rects_by_depth,
                                                      float* __restrict__ record_grads, double* __restrict__ loss,
                                                      bool first_of_step) {
    const int g = blockIdx.x * 256 + threadIdx.x;
    // what the steps before this one left in the sticky overflow word (this step's own binning may add to it)
    if (first_of_step && g == 0) status[kStatusStickyBefore] = status[kStatusOverflowSticky];
    // what the compositing backward adds into starts from zero: the parts of the loss, this Gaussian's accumulator row
    if (blockIdx.x == 0 && threadIdx.x < kLossParts) loss[kLossStride * (1 + threadIdx.x)] = 0.0;
    if (g >= G) return;
    {
        float4* row = reinterpret_cast<float4*>(record_grads + static_cast<std::size_t>(g) * kRecordGradStride);
#pragma unroll
        for (int k = 0; k < kRecordGradStride / 4; ++k) row[k] = float4{0.f, 0.f, 0.f, 0.f};
    }
    // the depth order of the previous call stays valid while every depth keeps its bits
    if (__builtin_bit_cast(std::uint32_t, depth[g]) != __builtin_bit_cast(std::uint32_t, ordered_depth[g]))
        atomicOr(status + kStatusDepthChanged, 1u);
    const std::size_t n = static_cast<std::size_t>(G);
    const float cx = params[0 * n + g], cy = params[1 * n + g];
    Variable<2, float> log_scale;
    log_scale[0] = params[2 * n + g];
    log_scale[1] = params[3 * n + g];
    Variable<1, float> theta(params[4 * n + g]);
    Variable<1, float> opacity(params[8 * n + g]);

    auto es = op::exp(log_scale);
    auto cov = op::scale_rotation_to_covariance_3param(es, theta);
    auto inv = op::sym_matrix2_inv(cov);
    auto alpha0 = op::sigmoid(opacity);
    inv.forward();
    alpha0.forward();

    Record rec;
    rec.cx = cx;
    rec.cy = cy;
    rec.a = inv[0];
    rec.b = inv[1];
    rec.c = inv[2];
    rec.red = params[5 * n + g];
    rec.green = params[6 * n + g];
    rec.blue = params[7 * n + g];
    rec.alpha0 = alpha0[0];
    rec.pad0 = rec.pad1 = rec.pad2 = 0.f;
    records[g] = rec;

    const int tiles_x = (width + kTile - 1) / kTile, tiles_y = (height + kTile - 1) / kTile;
    const float rx = 3.f * ::sqrtf(cov[0]), ry = 3.f * ::sqrtf(cov[2]);
    TileRect rc{1, 1, 0, 0};
    const bool finite = ::isfinite(cx) && ::isfinite(cy) && ::isfinite(rx) && ::isfinite(ry) && ::isfinite(rec.a) &&
                        ::isfinite(rec.b) && ::isfinite(rec.c) && ::isfinite(rec.alpha0);
    if (finite) {
        const float lo_x = ::floorf((cx - rx) / kTile), hi_x = ::floorf((cx + rx) / kTile);
        const float lo_y = ::floorf((cy - ry) / kTile), hi_y = ::floorf((cy + ry) / kTile);
        if (!(hi_x < 0.f || hi_y < 0.f || lo_x > static_cast<float>(tiles_x - 1) || lo_y > static_cast<float>(tiles_y - 1))) {
            rc.x0 = static_cast<std::int16_t>(lo_x < 0.f ? 0 : static_cast<int>(lo_x));
            rc.y0 = static_cast<std::int16_t>(lo_y < 0.f ? 0 : static_cast<int>(lo_y));
            rc.x1 = static_cast<std::int16_t>(hi_x > static_cast<float>(tiles_x - 1) ? tiles_x - 1 : static_cast<int>(hi_x));
            rc.y1 = static_cast<std::int16_t>(hi_y > static_cast<float>(tiles_y - 1) ? tiles_y - 1 : static_cast<int>(hi_y));
        }
    }
    rects[g] = rc;
    rects_by_depth[rank[g]] = rc;  // the binning walks the Gaussians in depth order
}


// Blocks are handed to the eight XCDs round-robin; giving each XCD a contiguous band of tiles keeps the
// records of a Gaussian that spans neighbouring tiles in one L2.
// Within its band every XCD takes its tiles longest list first: blocks are started in order of their
// index, and a tile with a long list that starts late leaves the SIMDs around it idle at the end of the
// launch.  One block per band: a histogram of the list lengths (in units of eight entries) in LDS, a
// descending prefix, and a scatter; the order within a bucket is whatever the atomics make it.
// order[band * per_band + i] = the tile that the band's i-th block takes, or ~0 for none.
constexpr int kOrderBuckets = 512;
__global__ void __launch_bounds__(1024) tile_order_kernel(int tiles, const std::uint32_t* __restrict__ range_begin,
                                                          const std::uint32_t* __restrict__ range_end,
                                                          std::uint32_t* __restrict__ order) {
    __shared__ std::uint32_t bucket[kOrderBuckets];
    const int per = (tiles + 7) / 8;
    const int band_first = static_cast<int>(blockIdx.x) * per;
    const int band_last = band_first + per < tiles ? band_first + per : (band_first < tiles ? tiles : band_first);  // an empty band for few tiles
    const int t = static_cast<int>(threadIdx.x);
    for (int k = t; k < kOrderBuckets; k += 1024) bucket[k] = 0;
    __syncthreads();
    auto bucket_of = [&](int tile) {
        const std::uint32_t length = range_end[tile] - range_begin[tile];
        const std::uint32_t b = length >> 3;
        return kOrderBuckets - 1 - static_cast<int>(b < kOrderBuckets - 1 ? b : kOrderBuckets - 1);  // longest first
    };
    for (int tile = band_first + t; tile < band_last; tile += 1024) atomicAdd(&bucket[bucket_of(tile)], 1u);
    __syncthreads();
    // exclusive prefix over the buckets, by the first wavefront: eight buckets per lane
    if (t < 64) {
        std::uint32_t mine[kOrderBuckets / 64], sum = 0;
#pragma unroll
        for (int k = 0; k < kOrderBuckets / 64; ++k) {
            mine[k] = bucket[t * (kOrderBuckets / 64) + k];
            sum += mine[k];
        }
        std::uint32_t inclusive = sum;
#pragma unroll
        for (int step = 1; step < 64; step *= 2) {
            const std::uint32_t other = __shfl_up(inclusive, step, 64);
            if (t >= step) inclusive += other;
        }
        std::uint32_t running = inclusive - sum;
#pragma unroll
        for (int k = 0; k < kOrderBuckets / 64; ++k) {
            bucket[t * (kOrderBuckets / 64) + k] = running;
            running += mine[k];
        }
    }
    __syncthreads();
    for (int tile = band_first + t; tile < band_last; tile += 1024)
        order[band_first + atomicAdd(&bucket[bucket_of(tile)], 1u)] = static_cast<std::uint32_t>(tile);
    for (int k = band_last - band_first + t; k < per; k += 1024) order[band_first + k] = ~0u;  // the last band may be short
}

// Tile of a block: block b belongs to XCD b % 8 and is that XCD's (b / 8)-th block.
__device__ __forceinline__ int ordered_tile_of_block(int block, int tiles, const std::uint32_t* __restrict__ order) {
    const int per = (tiles + 7) / 8;
    const std::uint32_t tile = order[(block % 8) * per + block / 8];
    return tile == ~0u ? tiles : static_cast<int>(tile);
}

// ---------------------------------------------------------------------------
// Compositing kernels.  One wavefront per tile; lane l owns the four
// horizontally adjacent pixels x = 4 (l % 4) .. +3 of row y = l / 4.  Four
// pixels per lane amortise everything that is per Gaussian (the LDS reads of
// its record, and in the backward pass the wavefront reduction of its
// gradient) over four times the arithmetic, and a one-wavefront block needs no
// block barrier.
//
// The tile's list is staged through LDS 64 records at a time, in a form made
// for the inner loop: the inverse covariance is pre-multiplied by
// -log2(e)/2 so that the falloff exp(-q/2) is a single v_exp_f32 of
//     q' = a' dx^2 + b2' dx dy + c' dy^2,
// the graph  q = mahalanobis(pixel - centre; inv), falloff = exp(-(q * 0.5)),
// a = falloff * alpha0  of the reference kernel
// (examples/mini-gaussian-splatting/gaussian_splatting_kernel.cu:45-55) in fused form.
constexpr int kLanePixels = 4;
constexpr int kChunk = 64;
constexpr int kPark = 16;  // list entries whose gradient sums are finished and written out together
__device__ __forceinline__ std::uint32_t wave_max(std::uint32_t v) {
    // 64-lane maximum through the LDS crossbar-free DPP path: rows, then row heads
    auto step = [](std::uint32_t x, auto ctrl) {
        const std::uint32_t other = static_cast<std::uint32_t>(
            __builtin_amdgcn_update_dpp(0, static_cast<int>(x), decltype(ctrl)::value, 0xF, 0xF, true));
        return x > other ? x : other;
    };
    v = step(v, std::integral_constant<int, 0xB1>{});
    v = step(v, std::integral_constant<int, 0x4E>{});
    v = step(v, std::integral_constant<int, 0x141>{});
    v = step(v, std::integral_constant<int, 0x140>{});
    const std::uint32_t r0 = __builtin_amdgcn_readlane(static_cast<int>(v), 0);
    const std::uint32_t r1 = __builtin_amdgcn_readlane(static_cast<int>(v), 16);
    const std::uint32_t r2 = __builtin_amdgcn_readlane(static_cast<int>(v), 32);
    const std::uint32_t r3 = __builtin_amdgcn_readlane(static_cast<int>(v), 48);
    const std::uint32_t m01 = r0 > r1 ? r0 : r1, m23 = r2 > r3 ? r2 : r3;
    return m01 > m23 ? m01 : m23;
}

// Small images have fewer tiles than the GPU has SIMDs, and a tile's backward walk is one long chain
// of dependent instructions: a wavefront alone on its SIMD spends most of its time waiting for its own
// results.  With kSplit the list of every tile is cut into `segments` pieces (whole groups of kPark
// entries), each walked by a wavefront of its own in the backward pass.  For that the forward pass
// leaves, per pixel and segment, the transmittance after the segment's last entry and the colour
// composited behind it.  That colour is formed from the later segments' own sums (the colour sum is
// restarted at every boundary), not as a difference of running totals, which would cancel.
constexpr int kMaxSegments = 8;

__device__ __forceinline__ std::uint32_t segment_length(std::uint32_t entries, int segments) {
    const std::uint32_t groups = (entries + kPark - 1) / kPark;
    return kPark * ((groups + static_cast<std::uint32_t>(segments) - 1) / static_cast<std::uint32_t>(segments));
}

template <bool kSplit>
__global__ void __launch_bounds__(kChunk) render_forward_kernel(
    int width, int height, int tiles_x, int tiles, const std::uint32_t* __restrict__ range_begin,
    const std::uint32_t* __restrict__ range_end, const std::uint32_t* __restrict__ sorted_ids,
    const Record* __restrict__ records, float* __restrict__ image, float* __restrict__ final_T,
    std::uint32_t* __restrict__ n_contrib, int segments, float4* __restrict__ segment_state,
    const std::uint32_t* __restrict__ tile_order) {
    __shared__ Staged staged[kChunk];
    const int tile = ordered_tile_of_block(blockIdx.x, tiles, tile_order);
    if (tile >= tiles) return;
    const int lane = threadIdx.x;
    const int x0 = (tile % tiles_x) * kTile + (lane & 3) * kLanePixels;
    const int y = (tile / tiles_x) * kTile + (lane >> 2);
    const float py = static_cast<float>(y);
    const float px0 = static_cast<float>(x0);

    // the same for every lane: said so, which keeps the loop counters in scalar registers
    const std::uint32_t first = __builtin_amdgcn_readfirstlane(range_begin[tile]);
    const std::uint32_t last = __builtin_amdgcn_readfirstlane(range_end[tile]);
    float T[kLanePixels], red[kLanePixels], green[kLanePixels], blue[kLanePixels];
    std::uint32_t used[kLanePixels];
#pragma unroll
    for (int p = 0; p < kLanePixels; ++p) {
        // pixels outside the image start out finished (see below) and are never stored
        T[p] = (x0 + p < width && y < height) ? 1.f : 0.f;
        red[p] = green[p] = blue[p] = 0.f;
        used[p] = 0;
    }

    // kSplit: colour of the finished segments; red, green and blue hold the current segment's own
    float done_red[kLanePixels], done_green[kLanePixels], done_blue[kLanePixels];
#pragma unroll
    for (int p = 0; p < kLanePixels; ++p) done_red[p] = done_green[p] = done_blue[p] = 0.f;
    const std::uint32_t seg_len = kSplit ? segment_length(last - first, segments) : 0u;
    std::uint32_t boundary = seg_len;
    int segment = 0;
    auto leave_segment_state = [&]() {
#pragma unroll
        for (int p = 0; p < kLanePixels; ++p)
            if (x0 + p < width && y < height)
                segment_state[(static_cast<std::size_t>(y) * width + x0 + p) * static_cast<std::size_t>(segments) + segment] =
                    float4{T[p], red[p], green[p], blue[p]};  // the states of a pixel lie next to each other
    };

    const float tile_x = static_cast<float>((tile % tiles_x) * kTile), tile_y = static_cast<float>((tile / tiles_x) * kTile);
    for (std::uint32_t base = first; base < last; base += kChunk) {
        __syncthreads();
        bool visible = false;
        if (base + lane < last) {
            const Staged mine = stage_record(records, sorted_ids[base + lane]);
            staged[lane] = mine;
            visible = !negligible_in_tile(mine, tile_x, tile_y);
        }
        __syncthreads();
        // the staged entries that can be seen from this tile, front to back
        for (std::uint64_t todo = accumulate::wave::ballot(visible); todo != 0; todo &= todo - 1) {
            const int j = __builtin_ctzll(todo);
            if constexpr (kSplit) {
                // the first entry at or beyond a boundary closes the segments before it (the same for every lane)
                while (base - first + j >= boundary) {
                    leave_segment_state();
#pragma unroll
                    for (int p = 0; p < kLanePixels; ++p) {
                        done_red[p] += red[p];
                        done_green[p] += green[p];
                        done_blue[p] += blue[p];
                        red[p] = green[p] = blue[p] = 0.f;
                    }
                    ++segment;
                    boundary += seg_len;
                }
            }
            const Staged r = staged[j];
            // exponent of the falloff as a polynomial in dx: (a_s dx + e) dx + f
            const float dy = py - r.cy;
            const float e = r.b2_s * dy;
            const float f = r.c_s * dy * dy;
            const float dx0 = px0 - r.cx;
#pragma unroll
            for (int p = 0; p < kLanePixels; ++p) {
                // A pixel stops, for good, before the first Gaussian it meets with T below the
                // threshold: from then on alpha = 0 leaves T where it is, so the test stays true.
                const bool done = T[p] < kMinTransmittance;
                const float dx = dx0 + static_cast<float>(p);
                const float a = math::fp32::exp2_raw(::fmaf(::fmaf(r.a_s, dx, e), dx, f)) * r.alpha0;
                const float alpha = done ? 0.f : __builtin_fminf(a, kAlphaMax);  // a is finite: non-finite Gaussians are not binned
                const float weight = T[p] * alpha;
                red[p] = ::fmaf(weight, r.red, red[p]);
                green[p] = ::fmaf(weight, r.green, green[p]);
                blue[p] = ::fmaf(weight, r.blue, blue[p]);
                T[p] *= 1.f - alpha;
                used[p] = done ? used[p] : base - first + j + 1;
            }
        }
        const bool all_done = T[0] < kMinTransmittance && T[1] < kMinTransmittance && T[2] < kMinTransmittance &&
                              T[3] < kMinTransmittance;
        if (accumulate::wave::ballot(!all_done) == 0) break;
    }
    if constexpr (kSplit) {
        leave_segment_state();  // of the segment the walk ended in
#pragma unroll
        for (int p = 0; p < kLanePixels; ++p) {
            red[p] += done_red[p];
            green[p] += done_green[p];
            blue[p] += done_blue[p];
        }
        // What the backward walk of a segment needs is the colour behind it: the sum of the later segments'
        // own colours.  Each state's colour is replaced by that sum (all loads first, then one pass).
#pragma unroll
        for (int p = 0; p < kLanePixels; ++p) {
            if (x0 + p < width && y < height) {
                float4* mine = segment_state + (static_cast<std::size_t>(y) * width + x0 + p) * static_cast<std::size_t>(segments);
                float4 state[kMaxSegments];
#pragma unroll
                for (int k = 0; k < kMaxSegments; ++k) state[k] = mine[k < segment ? k : segment];
                float behind[3] = {0.f, 0.f, 0.f};
#pragma unroll
                for (int k = kMaxSegments - 1; k >= 0; --k) {
                    if (k <= segment) {  // the same for every lane
                        mine[k] = float4{state[k].x, behind[0], behind[1], behind[2]};
                        behind[0] += state[k].y;
                        behind[1] += state[k].z;
                        behind[2] += state[k].w;
                    }
                }
            }
        }
    }
#pragma unroll
    for (int p = 0; p < kLanePixels; ++p) {
        if (x0 + p < width && y < height) {
            const std::size_t at = static_cast<std::size_t>(y) * width + x0 + p;
            image[at * 3 + 0] = red[p];
            image[at * 3 + 1] = green[p];
            image[at * 3 + 2] = blue[p];
            final_T[at] = T[p];
            n_contrib[at] = used[p];
        }
    }
}

// Sum of nine per-lane values over each row of 16 lanes, cheaper than nine separate
// reductions.  v[0..7] go through a reduce-scatter: at each of three steps a lane
// keeps half of its values, the half chosen by one bit of its lane number, and
// adds the copies held by the partner lane that differs in that bit.  For bits 2
// and 3 (partners 4 and 8 lanes away) the choice is made by the bank mask of the
// DPP add itself: one instruction serves the lanes whose bit is clear, a second
// one the others, and no select is needed.  Bit 0 takes the ordinary select and
// quad swap; a last quad swap over bit 1 completes the row.  v[8] takes the
// ordinary four row steps.
// Result: lane l of a row holds the row's sum of v[reduced_index(l)].
__device__ __forceinline__ int reduced_index(int lane) {
    const int r = lane & 15;
    return (r & 2) ? 8 : ((r & 1) << 2) | ((r >> 3) << 1) | ((r >> 2) & 1);
}

__device__ __forceinline__ float reduce_scatter9(const float (&v)[9], int lane) {
    // bit 2: banks 0 and 2 (lanes 0-3, 8-11 of a row) keep the even value and read lane + 4,
    // banks 1 and 3 keep the odd one and read lane - 4.  The leading wait covers the two idle
    // cycles a DPP read needs after a vector write of the same register.
    float w0, w1, w2, w3;
    asm volatile(
        "s_nop 1\n\t"
        "v_add_f32_dpp %0, %4, %4 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %0, %5, %5 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
        "v_add_f32_dpp %1, %6, %6 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %1, %7, %7 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
        "v_add_f32_dpp %2, %8, %8 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %2, %9, %9 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
        "v_add_f32_dpp %3, %10, %10 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %3, %11, %11 row_shr:4 row_mask:0xf bank_mask:0xa"
        : "=&v"(w0), "=&v"(w1), "=&v"(w2), "=&v"(w3)
        : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]));
    // bit 3: banks 0 and 1 (lanes 0-7) keep the even value, banks 2 and 3 the odd one; the partner is 8 lanes round the row
    float u0, u1;
    asm volatile(
        "s_nop 1\n\t"
        "v_add_f32_dpp %0, %2, %2 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %0, %3, %3 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %1, %4, %4 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %1, %5, %5 row_ror:8 row_mask:0xf bank_mask:0xc"
        : "=&v"(u0), "=&v"(u1)
        : "v"(w0), "v"(w1), "v"(w2), "v"(w3));
    const bool b0 = lane & 1;
    const float keep = b0 ? u1 : u0;
    const float send = b0 ? u0 : u1;
    float t = keep + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, send), 0xB1, 0xF, 0xF, true));
    t = accumulate::wave::dpp_add<0x4E>(t);  // bit 1

    float x = v[8];
    x = accumulate::wave::dpp_add<0xB1>(x);
    x = accumulate::wave::dpp_add<0x4E>(x);
    x = accumulate::wave::dpp_add<0x141>(x);
    x = accumulate::wave::dpp_add<0x140>(x);
    return (lane & 2) ? x : t;
}

// Compositing backward.  Lists are walked back to front.  For every Gaussian
// each lane adds up, over its four pixels, the nine sums that determine
// d loss / d record:
//   S_x, S_y, S_xx, S_xy, S_yy = sum of g_q {dx, dy, dx^2, dx dy, dy^2},  g_q = d loss / d q
//   the three colour gradients, and d loss / d alpha0
// (the Mahalanobis backward rule, d centre = -g_q (2a dx + 2b dy, 2b dx + 2c dy),
// d inv = g_q (dx^2, 2 dx dy, dy^2), is linear in those sums, so it is applied
// once per Gaussian instead of once per pixel).  The nine values are reduced
// over each row of 16 lanes by reduce_scatter9 and parked in LDS; after every kPark
// list entries lane j finishes entry j of the group, and the group's record
// gradients are added to the global accumulator with consecutive lanes on
// consecutive fields of consecutive entries: one atomic per (tile, Gaussian,
// field), about seven accumulator rows (cache lines) per instruction.
template <bool kSplit>
__global__ void __launch_bounds__(kChunk) render_backward_kernel(
    int width, int height, int tiles_x, int tiles, const std::uint32_t* __restrict__ range_begin,
    const std::uint32_t* __restrict__ range_end, const std::uint32_t* __restrict__ sorted_ids,
    const Record* __restrict__ records, const float* __restrict__ image, const float* __restrict__ target,
    const float* __restrict__ final_T, const std::uint32_t* __restrict__ n_contrib, float* __restrict__ record_grads,
    double* __restrict__ loss, int segments, const float4* __restrict__ segment_state,
    const std::uint32_t* __restrict__ tile_order) {
    __shared__ Staged staged[kChunk];
    __shared__ std::uint32_t staged_id[kChunk];
    // Row sums wait here until a group of kPark list entries is complete.  Small on purpose: LDS per
    // block, not registers, is what limits the number of resident wavefronts.
    __shared__ float parked[kPark][4][9];  // [list entry within its group][row of 16 lanes][value]
    __shared__ int parked_entry[kPark];    // which staged entry that is

    // kSplit: all tiles' first segments, then all second ones, ...: every XCD gets its band of tiles of every
    // segment (the late segments are the ones that often have nothing to walk)
    const unsigned blocks_per_segment = kSplit ? gridDim.x / static_cast<unsigned>(segments) : gridDim.x;
    const int segment = kSplit ? static_cast<int>(blockIdx.x / blocks_per_segment) : 0;
    const int tile = ordered_tile_of_block(static_cast<int>(blockIdx.x % blocks_per_segment), tiles, tile_order);
    if (tile >= tiles) return;
    const int lane = threadIdx.x;
    const int x0 = (tile % tiles_x) * kTile + (lane & 3) * kLanePixels;
    const int y = (tile / tiles_x) * kTile + (lane >> 2);
    const float py = static_cast<float>(y);

    // Per pixel: dC = d loss / d colour, T = transmittance behind the Gaussian the walk is at,
    // D = -dC . (colour composited behind that Gaussian), in absolute (not normalised) terms.  (Kept
    // negated so that no negated reciprocal is needed: the compiler would compute one separately.)
    float dC[kLanePixels][3], T[kLanePixels], D[kLanePixels];
    std::uint32_t used[kLanePixels];
    float my_loss = 0.f;
    std::uint32_t my_max = 0;
#pragma unroll
    for (int p = 0; p < kLanePixels; ++p) {
        T[p] = 1.f;
        D[p] = 0.f;
        used[p] = 0;
#pragma unroll
        for (int c = 0; c < 3; ++c) dC[p][c] = 0.f;
        if (x0 + p < width && y < height) {
            const std::size_t at = static_cast<std::size_t>(y) * width + x0 + p;
#pragma unroll
            for (int c = 0; c < 3; ++c) {
                const float d = image[at * 3 + c] - target[at * 3 + c];
                my_loss = ::fmaf(d, d, my_loss);
                dC[p][c] = 2.f * d;
            }
            T[p] = final_T[at];
            used[p] = n_contrib[at];
            my_max = used[p] > my_max ? used[p] : my_max;
        }
    }
    if (segment == 0) {
        const float tile_loss = accumulate::wave::sum(my_loss);
        if (lane == 0 && tile_loss != 0.f)
            detail::atomic_add(loss + kLossStride * (1 + tile % kLossParts), static_cast<double>(tile_loss));
    }
    const std::uint32_t deepest = wave_max(my_max);  // entries [0, deepest) were composited by some pixel
    if (deepest == 0) return;
    const std::uint32_t first = range_begin[tile];
    const float px0 = static_cast<float>(x0);
    // this block walks entries [walk_first, walk_last) of the list, back to front
    std::uint32_t walk_first = 0, walk_last = deepest;
    if constexpr (kSplit) {
        const std::uint32_t seg_len = segment_length(range_end[tile] - first, segments);
        walk_first = static_cast<std::uint32_t>(segment) * seg_len;
        if (walk_first >= deepest) return;
        walk_last = walk_first + seg_len < deepest ? walk_first + seg_len : deepest;
        // A pixel that went on beyond this segment starts from what the forward pass left for the
        // segment's end: the transmittance there, and the colour composited behind it.
#pragma unroll
        for (int p = 0; p < kLanePixels; ++p) {
            if (used[p] > walk_last) {
                // the states of a pixel lie next to each other
                const float4* mine = segment_state + (static_cast<std::size_t>(y) * width + x0 + p) * static_cast<std::size_t>(segments);
                const float4 state = mine[segment];
                T[p] = state.x;
                const float behind[3] = {state.y, state.z, state.w};
                D[p] = -::fmaf(dC[p][2], behind[2], ::fmaf(dC[p][1], behind[1], dC[p][0] * behind[0]));
            }
        }
    }
    // What has been loaded so far is first needed inside the loop over the entries.  Left to itself the
    // wait for those loads ends up there, where it also waits, at every entry, for the atomics issued
    // since; a use of the values here settles them before the loop.
#pragma unroll
    for (int p = 0; p < kLanePixels; ++p) asm volatile("" : "+v"(T[p]), "+v"(D[p]));
    // which of the nine row sums this lane ends up with; eight lanes and one more per row park theirs
    const int park_index = reduced_index(lane);
    const bool parks = !(lane & 2) || (lane & 15) == 2;

    const float tile_x = static_cast<float>((tile % tiles_x) * kTile), tile_y = static_cast<float>((tile / tiles_x) * kTile);
    for (std::uint32_t chunk = (walk_last - walk_first + kChunk - 1) / kChunk; chunk-- > 0;) {
        const std::uint32_t chunk_first = walk_first + chunk * kChunk;
        const int count = static_cast<int>(walk_last - chunk_first < kChunk ? walk_last - chunk_first : kChunk);
        __syncthreads();
        bool visible = false;
        if (lane < count) {
            const std::uint32_t id = sorted_ids[first + chunk_first + lane];
            staged_id[lane] = id;
            const Staged mine = stage_record(records, id);
            staged[lane] = mine;
            visible = !negligible_in_tile(mine, tile_x, tile_y);  // the forward pass left the same entries out
        }
        __syncthreads();

        // the staged entries that can be seen from this tile, back to front, in groups of up to kPark
        std::uint64_t todo = accumulate::wave::ballot(visible);
        while (todo != 0) {
            int members = 0;
            for (; todo != 0 && members < kPark; ++members) {
                const int j = 63 - __builtin_clzll(todo);
                todo &= ~(std::uint64_t(1) << j);
                const std::uint32_t position = chunk_first + j;
                const Staged r = staged[j];
                // exponent of the falloff as a polynomial in dx: (a_s dx + e) dx + f
                const float dy = py - r.cy;
                const float e = r.b2_s * dy;
                const float f = r.c_s * dy * dy;
                const float dx0 = px0 - r.cx;
                float through[kLanePixels];  // d loss / d alpha0 of this Gaussian, per pixel
                float colour[3] = {0.f, 0.f, 0.f};
#pragma unroll
                for (int p = 0; p < kLanePixels; ++p) {
                    // A pixel is idle until the walk reaches the last Gaussian it composited, and
                    // active from there on.  While idle, alpha = 0 leaves T and D at their initial
                    // values, so no branch is needed.
                    const bool active = position < used[p];
                    const float dx = dx0 + static_cast<float>(p);
                    const float falloff = math::fp32::exp2_raw(::fmaf(::fmaf(r.a_s, dx, e), dx, f));
                    const float a = falloff * r.alpha0;
                    const bool clamped = a > kAlphaMax;
                    const float alpha = active ? __builtin_fminf(a, kAlphaMax) : 0.f;
                    // 1 / (1 - alpha): v_rcp_f32 and one Newton step.  The hardware reciprocal alone leans one way,
                    // and T is rebuilt from the back by one such factor per entry, so over lists of hundreds of
                    // entries every gradient leaned with it (measured at 200 000 Gaussians: the sum of
                    // sign(g) (gpu - exact) over the sum of the terms' magnitudes 6.1e-7, with the step 3.5e-7,
                    // the median error of the colour gradients 7.0e-7 -> 4.8e-7 of that mass; +2 % on the kernel).
                    const float keep = 1.f - alpha;
                    float inv = __builtin_amdgcn_rcpf(keep);
                    inv = ::fmaf(::fmaf(-keep, inv, 1.f), inv, inv);
                    const float T_front = T[p] * inv;  // transmittance in front of this Gaussian
                    const float dot = ::fmaf(dC[p][2], r.blue, ::fmaf(dC[p][1], r.green, dC[p][0] * r.red));
                    // d loss / d alpha = T_front (dC . colour) - (dC . colour behind) / (1 - alpha)
                    //                  = T_front dot + D inv
                    const float d_alpha = ::fmaf(D[p], inv, T_front * dot);
                    const float weight = alpha * T_front;
                    D[p] = ::fmaf(-weight, dot, D[p]);
                    T[p] = T_front;
#pragma unroll
                    for (int c = 0; c < 3; ++c) colour[c] = ::fmaf(weight, dC[p][c], colour[c]);
                    through[p] = (active && !clamped) ? d_alpha * falloff : 0.f;
                }
                // Moments of `through` over the lane's four pixels (offsets 0..3 from dx0) give the five
                // sums  sum t dx^i dy^j  the Mahalanobis backward rule needs; their common factor
                // d alpha / d q / falloff = -alpha0 / 2 is applied once per Gaussian below.
                const float m0 = (through[0] + through[1]) + (through[2] + through[3]);
                const float m1 = ::fmaf(3.f, through[3], ::fmaf(2.f, through[2], through[1]));
                const float m2 = ::fmaf(9.f, through[3], ::fmaf(4.f, through[2], through[1]));
                const float sx = ::fmaf(dx0, m0, m1);
                const float sy = dy * m0;
                const float v[9] = {sx, sy, ::fmaf(dx0, sx + m1, m2), dy * sx, dy * sy, colour[0], colour[1], colour[2], m0};
                const float mine = reduce_scatter9(v, lane);
                if (parks) parked[members][lane >> 4][park_index] = mine;
                if (lane == 0) parked_entry[members] = j;
            }
            __syncthreads();
            if (lane < members) {
                float s[9];
#pragma unroll
                for (int k = 0; k < 9; ++k) s[k] = (parked[lane][0][k] + parked[lane][1][k]) + (parked[lane][2][k] + parked[lane][3][k]);
                const Staged r = staged[parked_entry[lane]];
                const float g_q_scale = -0.5f * r.alpha0;
#pragma unroll
                for (int k = 0; k < 5; ++k) s[k] *= g_q_scale;
                const float out[kRecordGrads] = {
                    -(2.f * r.a * s[0] + 2.f * r.b * s[1]),  // d centre x
                    -(2.f * r.b * s[0] + 2.f * r.c * s[1]),  // d centre y
                    s[2], 2.f * s[3], s[4],                  // d inverse covariance
                    s[5], s[6], s[7],                        // d colour
                    s[8],                                    // d alpha0
                };
#pragma unroll
                for (int k = 0; k < kRecordGrads; ++k) parked[lane][0][k] = out[k];
            }
            __syncthreads();
            // The lanes of one atomic instruction take consecutive fields of consecutive list entries, so
            // an instruction touches about seven accumulator rows (cache lines) instead of 64.
            for (int item = lane; item < members * kRecordGrads; item += kChunk) {
                const int entry = item / kRecordGrads, field = item - entry * kRecordGrads;
                const float value = parked[entry][0][field];
                if (value != 0.f)
                    detail::atomic_add(
                        record_grads + static_cast<std::size_t>(staged_id[parked_entry[entry]]) * kRecordGradStride + field, value);
            }
            __syncthreads();  // the next group parks into the same rows
        }
    }
}

// ---------------------------------------------------------------------------
// Parameter backward: one lane per Gaussian.  Rebuilds the projection graph,
// seeds the gradients of its two roots (inverse covariance and alpha0) with the
// accumulated record gradients, and lets the nodes' backward rules carry them
// to log-scale, theta and the opacity logit.  Centre and colour gradients pass
// straight through.
__global__ void __launch_bounds__(256) gaussian_backward_kernel(int G, const float* __restrict__ params,
                                                                const float* __restrict__ record_grads,
                                                                float* __restrict__ grads, double* __restrict__ loss) {
    const int g = blockIdx.x * 256 + threadIdx.x;
    if (g >= G) return;
    if (g == 0) {
        double total = 0.0;
#pragma unroll 8
        for (int k = 0; k < kLossParts; ++k) total += loss[kLossStride * (1 + k)];
        loss[0] = total;
    }
    const std::size_t n = static_cast<std::size_t>(G);
    const float* acc = record_grads + static_cast<std::size_t>(g) * kRecordGradStride;

    Variable<2, float> log_scale;
    log_scale[0] = params[2 * n + g];
    log_scale[1] = params[3 * n + g];
    Variable<1, float> theta(params[4 * n + g]);
    Variable<1, float> opacity(params[8 * n + g]);
    auto es = op::exp(log_scale);
    auto cov = op::scale_rotation_to_covariance_3param(es, theta);
    auto inv = op::sym_matrix2_inv(cov);
    auto alpha0 = op::sigmoid(opacity);

    inv.forward();
    inv.add_grad(0, acc[2]);
    inv.add_grad(1, acc[3]);
    inv.add_grad(2, acc[4]);
    inv.backward();
    alpha0.forward();
    alpha0.add_grad(0, acc[8]);
    alpha0.backward();

    grads[0 * n + g] = acc[0];
    grads[1 * n + g] = acc[1];
    grads[2 * n + g] = log_scale.grad(0);
    grads[3 * n + g] = log_scale.grad(1);
    grads[4 * n + g] = theta.grad(0);
    grads[5 * n + g] = acc[5];
    grads[6 * n + g] = acc[6];
    grads[7 * n + g] = acc[7];
    grads[8 * n + g] = opacity.grad(0);
}

// ---------------------------------------------------------------------------
// launchers (declared in splat_launch.cuh)

int launch_project(hipStream_t s, int G, const float* params, const float* depth, const float* ordered_depth,
                   const std::uint32_t* rank, std::uint32_t* status, int width, int height, Record* records, TileRect* rects,
                   TileRect* rects_by_depth, float* record_grads, double* loss, bool first_of_step) {
    hipLaunchKernelGGL(project_kernel, dim3(xad::blocks_for(G, 256)), dim3(256), 0, s, G, params, depth, ordered_depth, rank,
                       status, width, height, records, rects, rects_by_depth, record_grads, loss, first_of_step);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

static unsigned padded_tile_blocks(int tiles) { return static_cast<unsigned>(((tiles + 7) / 8) * 8); }

int render_segments(int width, int height) {
    const int tiles = ((width + kTile - 1) / kTile) * ((height + kTile - 1) / kTile);
    return tiles <= 1024 ? 8 : (tiles <= 2048 ? 4 : (tiles <= 4096 ? 2 : 1));
}

int launch_render_forward(hipStream_t s, int width, int height, const std::uint32_t* range_begin,
                          const std::uint32_t* range_end, const std::uint32_t* sorted_ids, const Record* records,
                          float* image, float* final_T, std::uint32_t* n_contrib, int segments, float4* segment_state,
                          std::uint32_t* tile_order) {
    const int tiles_x = (width + kTile - 1) / kTile, tiles = tiles_x * ((height + kTile - 1) / kTile);
    // the order both compositing kernels of this step take the tiles in
    hipLaunchKernelGGL(tile_order_kernel, dim3(8), dim3(1024), 0, s, tiles, range_begin, range_end, tile_order);
    XAD_HIP_TRY(hipGetLastError());
    XAD_REQUIRE(segments >= 1 && (segments == 1 || segment_state), "splat: a split walk needs its per-segment state");
    if (segments > 1)
        hipLaunchKernelGGL(render_forward_kernel<true>, dim3(padded_tile_blocks(tiles)), dim3(kChunk), 0, s, width, height,
                           tiles_x, tiles, range_begin, range_end, sorted_ids, records, image, final_T, n_contrib, segments,
                           segment_state, tile_order);
    else
        hipLaunchKernelGGL(render_forward_kernel<false>, dim3(padded_tile_blocks(tiles)), dim3(kChunk), 0, s, width, height,
                           tiles_x, tiles, range_begin, range_end, sorted_ids, records, image, final_T, n_contrib, 1, nullptr, tile_order);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

int launch_render_backward(hipStream_t s, int width, int height, const std::uint32_t* range_begin,
                           const std::uint32_t* range_end, const std::uint32_t* sorted_ids, const Record* records,
                           const float* image, const float* target, const float* final_T,
                           const std::uint32_t* n_contrib, float* record_grads, double* loss, int segments,
                           const float4* segment_state, const std::uint32_t* tile_order) {
    const int tiles_x = (width + kTile - 1) / kTile, tiles = tiles_x * ((height + kTile - 1) / kTile);
    XAD_REQUIRE(segments >= 1 && segments <= kMaxSegments && (segments == 1 || segment_state),
                "splat: a split walk takes up to %d segments and needs its per-segment state", kMaxSegments);
    if (segments > 1)
        hipLaunchKernelGGL(render_backward_kernel<true>, dim3(padded_tile_blocks(tiles) * static_cast<unsigned>(segments)),
                           dim3(kChunk), 0, s, width, height, tiles_x, tiles, range_begin, range_end, sorted_ids, records, image,
                           target, final_T, n_contrib, record_grads, loss, segments, segment_state, tile_order);
    else
        hipLaunchKernelGGL(render_backward_kernel<false>, dim3(padded_tile_blocks(tiles)), dim3(kChunk), 0, s, width, height,
                           tiles_x, tiles, range_begin, range_end, sorted_ids, records, image, target, final_T, n_contrib,
                           record_grads, loss, 1, nullptr, tile_order);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

int launch_gaussian_backward(hipStream_t s, int G, const float* params, const float* record_grads, float* grads, double* loss) {
    hipLaunchKernelGGL(gaussian_backward_kernel, dim3(xad::blocks_for(G, 256)), dim3(256), 0, s, G, params, record_grads,
                       grads, loss);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

}  // namespace xad_splat
