// Kernels of the tile-binned splatting step: per-Gaussian projection, pair
// emission, tile ranges, per-tile compositing forward and reverse-order
// backward, per-Gaussian parameter backward.
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

#include "common.cuh"
#include "splat.cuh"
#include "splat_launch.cuh"

namespace xad_splat {

using namespace xyz_autodiff;

// ---------------------------------------------------------------------------
// Projection: one lane per Gaussian.  Builds the graph
//   es = exp(log-scale); cov = scale_rotation_to_covariance_3param(es, theta);
//   inv = sym_matrix2_inv(cov); alpha0 = sigmoid(opacity)
// from the library's nodes, runs it forward, and derives the 3-sigma tile
// rectangle and the number of tiles.
__global__ void __launch_bounds__(256) project_kernel(int G, const float* __restrict__ params, int width, int height,
                                                      Record* __restrict__ records, TileRect* __restrict__ rects,
                                                      std::uint32_t* __restrict__ counts) {
    const int g = blockIdx.x * 256 + threadIdx.x;
    if (g >= G) return;
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
    std::uint32_t count = 0;
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
            count = static_cast<std::uint32_t>(rc.x1 - rc.x0 + 1) * static_cast<std::uint32_t>(rc.y1 - rc.y0 + 1);
        }
    }
    rects[g] = rc;
    counts[g] = count;
}

// Order-preserving map from float to unsigned (any sign).
__device__ __forceinline__ std::uint32_t ordered_bits(float f) {
    const std::uint32_t u = __builtin_bit_cast(std::uint32_t, f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Pair emission: Gaussian g writes one (tile | depth, g) pair per tile of its
// rectangle into the segment [offsets[g], offsets[g+1]).  A wavefront takes 64
// consecutive Gaussians; within it lanes walk their own rectangles.
__global__ void __launch_bounds__(256) emit_kernel(int G, const TileRect* __restrict__ rects,
                                                   const std::uint32_t* __restrict__ offsets,
                                                   const float* __restrict__ depth, int tiles_x,
                                                   std::uint64_t* __restrict__ keys, std::uint32_t* __restrict__ values,
                                                   std::uint32_t capacity) {
    const int g = blockIdx.x * 256 + threadIdx.x;
    if (g >= G) return;
    const TileRect rc = rects[g];
    if (rc.x0 > rc.x1) return;
    std::uint32_t at = offsets[g];
    const std::uint64_t low = ordered_bits(depth[g]);
    for (int ty = rc.y0; ty <= rc.y1; ++ty)
        for (int tx = rc.x0; tx <= rc.x1; ++tx) {
            if (at < capacity) {
                keys[at] = (static_cast<std::uint64_t>(ty * tiles_x + tx) << 32) | low;
                values[at] = static_cast<std::uint32_t>(g);
            }
            ++at;
        }
}

// Tile ranges from the sorted keys: ranges[t] = [first, last) positions of tile t.
__global__ void __launch_bounds__(256) ranges_kernel(std::uint32_t K, const std::uint64_t* __restrict__ keys,
                                                     std::uint32_t* __restrict__ range_begin,
                                                     std::uint32_t* __restrict__ range_end) {
    const std::uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= K) return;
    const std::uint32_t t = static_cast<std::uint32_t>(keys[i] >> 32);
    if (i == 0 || static_cast<std::uint32_t>(keys[i - 1] >> 32) != t) range_begin[t] = i;
    if (i + 1 == K || static_cast<std::uint32_t>(keys[i + 1] >> 32) != t) range_end[t] = i + 1;
}

// Blocks are handed to the eight XCDs round-robin; giving each XCD a contiguous
// band of tiles keeps the records of a Gaussian that spans neighbouring tiles
// in one L2.
__device__ __forceinline__ int tile_of_block(int block, int tiles) {
    constexpr int kXcds = 8;
    const int per = (tiles + kXcds - 1) / kXcds;
    const int t = (block % kXcds) * per + block / kXcds;
    return t;  // may be >= tiles for the padding blocks of the last band
}

// alpha of one Gaussian at one pixel, before the clamp, through the library's
// op logic (forward rules only): q = mahalanobis(pixel - centre; inv),
// falloff = exp(-(q/2)), a = falloff * alpha0.
struct PixelAlpha {
    float q, falloff, a;
};
__device__ __forceinline__ PixelAlpha pixel_alpha(const Record& r, float px, float py) {
    const float dx = px - r.cx, dy = py - r.cy;
    PixelAlpha out;
    out.q = op::detail_maha::quadratic_form<float>(dx, dy, r.a, r.b, r.c);
    out.falloff = math::exp(-(out.q * 0.5f));
    out.a = out.falloff * r.alpha0;
    return out;
}

__device__ __forceinline__ Record load_record(const Record* __restrict__ records, std::uint32_t g) {
    const float4* src = reinterpret_cast<const float4*>(records + g);
    const float4 v0 = src[0], v1 = src[1], v2 = src[2];
    Record r;
    r.cx = v0.x; r.cy = v0.y; r.a = v0.z; r.b = v0.w;
    r.c = v1.x; r.red = v1.y; r.green = v1.z; r.blue = v1.w;
    r.alpha0 = v2.x; r.pad0 = r.pad1 = r.pad2 = 0.f;
    return r;
}

// ---------------------------------------------------------------------------
// Compositing forward: one 256-lane block per tile, one lane per pixel.  The
// tile's list is staged through LDS 256 records at a time; every lane then
// reads the same record at the same time (an LDS broadcast).
__global__ void __launch_bounds__(kTilePixels) render_forward_kernel(
    int width, int height, int tiles_x, int tiles, const std::uint32_t* __restrict__ range_begin,
    const std::uint32_t* __restrict__ range_end, const std::uint32_t* __restrict__ sorted_ids,
    const Record* __restrict__ records, float* __restrict__ image, float* __restrict__ final_T,
    std::uint32_t* __restrict__ n_contrib) {
    __shared__ Record staged[kTilePixels];
    const int tile = tile_of_block(blockIdx.x, tiles);
    if (tile >= tiles) return;
    const int tx = tile % tiles_x, ty = tile / tiles_x;
    const int lx = threadIdx.x % kTile, ly = threadIdx.x / kTile;
    const int x = tx * kTile + lx, y = ty * kTile + ly;
    const bool inside = x < width && y < height;
    const float px = static_cast<float>(x), py = static_cast<float>(y);

    const std::uint32_t first = range_begin[tile], last = range_end[tile];
    float T = 1.f, red = 0.f, green = 0.f, blue = 0.f;
    std::uint32_t used = 0;
    bool done = !inside;

    for (std::uint32_t base = first; base < last; base += kTilePixels) {
        __syncthreads();
        const std::uint32_t mine = base + threadIdx.x;
        if (mine < last) staged[threadIdx.x] = load_record(records, sorted_ids[mine]);
        __syncthreads();
        const int count = static_cast<int>(last - base < kTilePixels ? last - base : kTilePixels);
        if (!done) {
            for (int j = 0; j < count; ++j) {
                if (T < kMinTransmittance) {
                    done = true;
                    break;
                }
                const Record& r = staged[j];
                const PixelAlpha pa = pixel_alpha(r, px, py);
                const float alpha = pa.a > kAlphaMax ? kAlphaMax : pa.a;
                const float weight = T * alpha;
                red += weight * r.red;
                green += weight * r.green;
                blue += weight * r.blue;
                T *= 1.f - alpha;
                used = base - first + j + 1;
            }
        }
        if (__syncthreads_and(done)) break;
    }
    if (inside) {
        const std::size_t p = static_cast<std::size_t>(y) * width + x;
        image[p * 3 + 0] = red;
        image[p * 3 + 1] = green;
        image[p * 3 + 2] = blue;
        final_T[p] = T;
        n_contrib[p] = used;
    }
}

// ---------------------------------------------------------------------------
// Compositing backward: same tiling, lists walked back to front.  For every
// (pixel, Gaussian) the lane computes d loss / d (centre, inverse covariance,
// colour, alpha0); the nine values are summed over the 64 lanes of each
// wavefront with DPP, the four wavefront sums are combined through LDS, and one
// lane per Gaussian adds the block's totals to the global accumulator: one
// global atomic per (tile, Gaussian, field).
__global__ void __launch_bounds__(kTilePixels) render_backward_kernel(
    int width, int height, int tiles_x, int tiles, const std::uint32_t* __restrict__ range_begin,
    const std::uint32_t* __restrict__ range_end, const std::uint32_t* __restrict__ sorted_ids,
    const Record* __restrict__ records, const float* __restrict__ image, const float* __restrict__ target,
    const float* __restrict__ final_T, const std::uint32_t* __restrict__ n_contrib, float* __restrict__ record_grads,
    double* __restrict__ loss) {
    constexpr int kWaves = kTilePixels / 64;
    __shared__ Record staged[kTilePixels];
    __shared__ std::uint32_t staged_id[kTilePixels];
    __shared__ float partial[kWaves][kTilePixels][kRecordGrads];  // [wave][list entry][field]
    __shared__ std::uint32_t block_max_used;
    __shared__ double wave_loss[kWaves];

    const int tile = tile_of_block(blockIdx.x, tiles);
    if (tile >= tiles) return;
    const int tx = tile % tiles_x, ty = tile / tiles_x;
    const int lx = threadIdx.x % kTile, ly = threadIdx.x / kTile;
    const int x = tx * kTile + lx, y = ty * kTile + ly;
    const bool inside = x < width && y < height;
    const float px = static_cast<float>(x), py = static_cast<float>(y);
    const int wave = threadIdx.x / 64;
    const std::size_t p = static_cast<std::size_t>(y) * width + x;

    float dC[3] = {0.f, 0.f, 0.f};
    float T = 1.f;
    std::uint32_t used = 0;
    float my_loss = 0.f;
    if (inside) {
#pragma unroll
        for (int c = 0; c < 3; ++c) {
            const float d = image[p * 3 + c] - target[p * 3 + c];
            my_loss += d * d;
            dC[c] = 2.f * d;
        }
        T = final_T[p];
        used = n_contrib[p];
    }
    // loss: per-wavefront DPP sum, then one fp64 atomic per block
    {
        const float s = accumulate::wave::sum(my_loss);
        if (threadIdx.x % 64 == 0) wave_loss[wave] = static_cast<double>(s);
        if (threadIdx.x == 0) block_max_used = 0;
        __syncthreads();
        atomicMax(&block_max_used, used);
        if (threadIdx.x == 0) {
            double total = 0.0;
            for (int w = 0; w < kWaves; ++w) total += wave_loss[w];
            if (total != 0.0) detail::atomic_add(loss, total);
        }
        __syncthreads();
    }
    const std::uint32_t first = range_begin[tile];
    const std::uint32_t deepest = block_max_used;  // entries [0, deepest) of the list were used by some pixel
    if (deepest == 0) return;

    float behind[3] = {0.f, 0.f, 0.f}, last_col[3] = {0.f, 0.f, 0.f};
    float last_alpha = 0.f;

    const std::uint32_t chunks = (deepest + kTilePixels - 1) / kTilePixels;
    for (std::uint32_t chunk = chunks; chunk-- > 0;) {
        const std::uint32_t chunk_first = chunk * kTilePixels;  // list position of staged[0]
        const int count = static_cast<int>(deepest - chunk_first < kTilePixels ? deepest - chunk_first : kTilePixels);
        __syncthreads();
        if (static_cast<int>(threadIdx.x) < count) {
            const std::uint32_t id = sorted_ids[first + chunk_first + threadIdx.x];
            staged_id[threadIdx.x] = id;
            staged[threadIdx.x] = load_record(records, id);
        }
        __syncthreads();

        for (int j = count - 1; j >= 0; --j) {
            const std::uint32_t position = chunk_first + j;
            const bool active = position < used;  // `used` is 0 for lanes outside the image
            if (accumulate::wave::ballot(active) == 0) {
                // no pixel of this wavefront composited this Gaussian
                if (threadIdx.x % 64 < kRecordGrads) partial[wave][j][threadIdx.x % 64] = 0.f;
                continue;
            }
            float g[kRecordGrads] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            if (active) {
                const Record& r = staged[j];
                const PixelAlpha pa = pixel_alpha(r, px, py);
                const float alpha = pa.a > kAlphaMax ? kAlphaMax : pa.a;
                T = T / (1.f - alpha);
                const float col[3] = {r.red, r.green, r.blue};
                float d_alpha = 0.f;
#pragma unroll
                for (int c = 0; c < 3; ++c) {
                    behind[c] = last_alpha * last_col[c] + (1.f - last_alpha) * behind[c];
                    d_alpha += (col[c] - behind[c]) * dC[c];
                    g[5 + c] = alpha * T * dC[c];
                    last_col[c] = col[c];
                }
                d_alpha *= T;
                last_alpha = alpha;
                if (!(pa.a > kAlphaMax)) {
                    // a = falloff * alpha0; falloff = exp(-(q/2)); q = mahalanobis(pixel, centre, inv):
                    // the library's backward rules, applied to thread-local operands
                    g[8] = d_alpha * pa.falloff;
                    const float g_q = -0.5f * (d_alpha * r.alpha0 * pa.falloff);
                    Variable<2, float> centre;
                    centre[0] = r.cx;
                    centre[1] = r.cy;
                    Variable<3, float> inv;
                    inv[0] = r.a;
                    inv[1] = r.b;
                    inv[2] = r.c;
                    Variable<1, float> q_out;
                    q_out.add_grad(0, g_q);
                    const op::MahalanobisDistanceWithCenterLogic<Variable<2, float>, Variable<3, float>> rule(px, py);
                    rule.backward(q_out, centre, inv);
                    g[0] = centre.grad(0);
                    g[1] = centre.grad(1);
                    g[2] = inv.grad(0);
                    g[3] = inv.grad(1);
                    g[4] = inv.grad(2);
                }
            }
            // level 1: wavefront sums
#pragma unroll
            for (int k = 0; k < kRecordGrads; ++k) {
                const float s = accumulate::wave::sum(g[k]);
                if (threadIdx.x % 64 == 0) partial[wave][j][k] = s;
            }
        }
        __syncthreads();
        // level 2 + 3: lane j combines the four wavefront sums of list entry j and
        // adds them to the Gaussian's accumulator row
        if (static_cast<int>(threadIdx.x) < count) {
            float* row = record_grads + static_cast<std::size_t>(staged_id[threadIdx.x]) * kRecordGrads;
#pragma unroll
            for (int k = 0; k < kRecordGrads; ++k) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < kWaves; ++w) s += partial[w][threadIdx.x][k];
                if (s != 0.f) detail::atomic_add(row + k, s);
            }
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
                                                                float* __restrict__ grads) {
    const int g = blockIdx.x * 256 + threadIdx.x;
    if (g >= G) return;
    const std::size_t n = static_cast<std::size_t>(G);
    const float* acc = record_grads + static_cast<std::size_t>(g) * kRecordGrads;

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

int launch_project(hipStream_t s, int G, const float* params, int width, int height, Record* records, TileRect* rects,
                   std::uint32_t* counts) {
    hipLaunchKernelGGL(project_kernel, dim3(xad::blocks_for(G, 256)), dim3(256), 0, s, G, params, width, height, records,
                       rects, counts);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

int launch_emit(hipStream_t s, int G, const TileRect* rects, const std::uint32_t* offsets, const float* depth,
                int tiles_x, std::uint64_t* keys, std::uint32_t* values, std::uint32_t capacity) {
    hipLaunchKernelGGL(emit_kernel, dim3(xad::blocks_for(G, 256)), dim3(256), 0, s, G, rects, offsets, depth, tiles_x, keys,
                       values, capacity);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

int launch_ranges(hipStream_t s, std::uint32_t K, const std::uint64_t* keys, std::uint32_t* range_begin,
                  std::uint32_t* range_end) {
    if (K == 0) return XAD_OK;
    hipLaunchKernelGGL(ranges_kernel, dim3(xad::blocks_for(K, 256)), dim3(256), 0, s, K, keys, range_begin, range_end);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

static unsigned padded_tile_blocks(int tiles) { return static_cast<unsigned>(((tiles + 7) / 8) * 8); }

int launch_render_forward(hipStream_t s, int width, int height, const std::uint32_t* range_begin,
                          const std::uint32_t* range_end, const std::uint32_t* sorted_ids, const Record* records,
                          float* image, float* final_T, std::uint32_t* n_contrib) {
    const int tiles_x = (width + kTile - 1) / kTile, tiles = tiles_x * ((height + kTile - 1) / kTile);
    hipLaunchKernelGGL(render_forward_kernel, dim3(padded_tile_blocks(tiles)), dim3(kTilePixels), 0, s, width, height,
                       tiles_x, tiles, range_begin, range_end, sorted_ids, records, image, final_T, n_contrib);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

int launch_render_backward(hipStream_t s, int width, int height, const std::uint32_t* range_begin,
                           const std::uint32_t* range_end, const std::uint32_t* sorted_ids, const Record* records,
                           const float* image, const float* target, const float* final_T,
                           const std::uint32_t* n_contrib, float* record_grads, double* loss) {
    const int tiles_x = (width + kTile - 1) / kTile, tiles = tiles_x * ((height + kTile - 1) / kTile);
    hipLaunchKernelGGL(render_backward_kernel, dim3(padded_tile_blocks(tiles)), dim3(kTilePixels), 0, s, width, height,
                       tiles_x, tiles, range_begin, range_end, sorted_ids, records, image, target, final_T, n_contrib,
                       record_grads, loss);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

int launch_gaussian_backward(hipStream_t s, int G, const float* params, const float* record_grads, float* grads) {
    hipLaunchKernelGGL(gaussian_backward_kernel, dim3(xad::blocks_for(G, 256)), dim3(256), 0, s, G, params, record_grads,
                       grads);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

}  // namespace xad_splat
