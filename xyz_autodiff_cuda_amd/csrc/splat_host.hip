// The tile-binned splatting step on the host cores, built from the library's own templates: the CPU
// figure the GPU step is reported beside (xad_host_splat_step_f32).  Host code only; the GPU entry points
// never route through it.
//
// Same model as the GPU step (splat.cuh): 16 x 16 tiles, 3-sigma box binning, lists in (depth, index)
// order, alpha = min(0.99, sigmoid(o) exp(-q / 2)), a pixel stops before a Gaussian once its
// transmittance is below 1e-4, sum of squared errors.  What differs is how the work is laid out: tiles
// are dealt to threads, a pixel walks its list alone, and every (pixel, Gaussian) pair builds the
// reference's per-pair graph
//     q = mahalanobis_distance_with_center(pixel, centre, inv);  w = exp(-(q * 0.5))
// (examples/mini-gaussian-splatting/gaussian_splatting_kernel.cu:45-55 forward, :86-97 backward) from the
// library's nodes and runs its forward() and backward(), as the reference's kernel does per pair.  Every
// thread adds into its own copy of the record gradients; the copies are summed at the end.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <numeric>
#include <thread>
#include <vector>

#include <xyz_autodiff/variable.cuh>
#include <xyz_autodiff/variable_operators.cuh>
#include <xyz_autodiff/operations/unary/exp_logic.cuh>
#include <xyz_autodiff/operations/unary/neg_logic.cuh>
#include <xyz_autodiff/operations/unary/sigmoid_logic.cuh>
#include <xyz_autodiff/operations/unary/sym_matrix2_inv_logic.cuh>
#include <operations/covariance_generation.cuh>
#include <operations/mahalanobis_distance.cuh>

#include "common.cuh"
#include "splat.cuh"

namespace {

using namespace xyz_autodiff;
using xad_splat::kAlphaMax;
using xad_splat::kMinTransmittance;
using xad_splat::kTile;

struct HostRecord {
    float cx, cy, inv[3], colour[3], alpha0;
};
struct HostRect {
    int x0, y0, x1, y1;  // tiles, inclusive; empty when x0 > x1
};

// alpha before clamping, through the per-pair graph; also leaves q's falloff for the backward pass
struct PairGraph {
    Variable<2, float> centre;
    Variable<3, float> inv;
    explicit PairGraph(const HostRecord& r) {
        centre[0] = r.cx;
        centre[1] = r.cy;
        inv[0] = r.inv[0];
        inv[1] = r.inv[1];
        inv[2] = r.inv[2];
    }
};

template <typename F>
void run_threads(int threads, F&& body) {
    if (threads <= 1) {
        body(0);
        return;
    }
    std::vector<std::thread> pool;
    pool.reserve(static_cast<std::size_t>(threads));
    for (int t = 0; t < threads; ++t) pool.emplace_back([&body, t] { body(t); });
    for (auto& th : pool) th.join();
}

}  // namespace

extern "C" int xad_host_splat_step_f32(int width, int height, int num_gaussians, const float* params, const float* depth,
                                       const float* target, float* image, float* grads, double* loss_out,
                                       uint64_t* pairs_out, int num_threads) {
    const char* who = "xad_host_splat_step_f32";
    XAD_REQUIRE(width > 0 && height > 0 && num_gaussians > 0, "%s: width, height and num_gaussians must be positive", who);
    XAD_REQUIRE(params && depth && target && image, "%s: null argument", who);
    const int G = num_gaussians;
    const std::size_t n = static_cast<std::size_t>(G);
    const int tiles_x = (width + kTile - 1) / kTile, tiles_y = (height + kTile - 1) / kTile, tiles = tiles_x * tiles_y;
    int threads = num_threads > 0 ? num_threads : static_cast<int>(std::thread::hardware_concurrency());
    if (threads < 1) threads = 1;

    // ---- per Gaussian: record and tile rectangle, through the projection graph
    std::vector<HostRecord> records(n);
    std::vector<HostRect> rects(n);
    run_threads(threads, [&](int t) {
        for (std::size_t g = static_cast<std::size_t>(t); g < n; g += static_cast<std::size_t>(threads)) {
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
            HostRecord& r = records[g];
            r.cx = params[0 * n + g];
            r.cy = params[1 * n + g];
            r.inv[0] = inv[0];
            r.inv[1] = inv[1];
            r.inv[2] = inv[2];
            r.colour[0] = params[5 * n + g];
            r.colour[1] = params[6 * n + g];
            r.colour[2] = params[7 * n + g];
            r.alpha0 = alpha0[0];
            const float rx = 3.f * std::sqrt(cov[0]), ry = 3.f * std::sqrt(cov[2]);
            HostRect rc{1, 1, 0, 0};
            const bool finite = std::isfinite(r.cx) && std::isfinite(r.cy) && std::isfinite(rx) && std::isfinite(ry) &&
                                std::isfinite(r.inv[0]) && std::isfinite(r.inv[1]) && std::isfinite(r.inv[2]) &&
                                std::isfinite(r.alpha0);
            if (finite) {
                const float lo_x = std::floor((r.cx - rx) / kTile), hi_x = std::floor((r.cx + rx) / kTile);
                const float lo_y = std::floor((r.cy - ry) / kTile), hi_y = std::floor((r.cy + ry) / kTile);
                if (!(hi_x < 0.f || hi_y < 0.f || lo_x > static_cast<float>(tiles_x - 1) || lo_y > static_cast<float>(tiles_y - 1))) {
                    rc.x0 = lo_x < 0.f ? 0 : static_cast<int>(lo_x);
                    rc.y0 = lo_y < 0.f ? 0 : static_cast<int>(lo_y);
                    rc.x1 = hi_x > static_cast<float>(tiles_x - 1) ? tiles_x - 1 : static_cast<int>(hi_x);
                    rc.y1 = hi_y > static_cast<float>(tiles_y - 1) ? tiles_y - 1 : static_cast<int>(hi_y);
                }
            }
            rects[g] = rc;
        }
    });

    // ---- tile lists in (depth, index) order: stable sort of the Gaussians, then a counting pass
    std::vector<int> order(n);
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return depth[a] < depth[b]; });
    std::vector<std::size_t> first(static_cast<std::size_t>(tiles) + 1, 0);
    for (std::size_t g = 0; g < n; ++g)
        for (int ty = rects[g].y0; ty <= rects[g].y1; ++ty)
            for (int tx = rects[g].x0; tx <= rects[g].x1; ++tx) ++first[static_cast<std::size_t>(ty) * tiles_x + tx + 1];
    for (int t = 0; t < tiles; ++t) first[t + 1] += first[t];
    std::vector<int> list(first[tiles]);
    {
        std::vector<std::size_t> cursor(first.begin(), first.end() - 1);
        for (int g : order)
            for (int ty = rects[g].y0; ty <= rects[g].y1; ++ty)
                for (int tx = rects[g].x0; tx <= rects[g].x1; ++tx) list[cursor[static_cast<std::size_t>(ty) * tiles_x + tx]++] = g;
    }
    if (pairs_out) *pairs_out = first[tiles];

    // ---- per tile: compositing forward, and backward into the thread's own record gradients
    std::vector<float> acc(grads ? static_cast<std::size_t>(threads) * n * 9 : 0, 0.f);
    std::vector<double> loss_parts(static_cast<std::size_t>(threads), 0.0);
    std::atomic<int> next_tile{0};
    run_threads(threads, [&](int t) {
        float* mine = grads ? acc.data() + static_cast<std::size_t>(t) * n * 9 : nullptr;
        double loss = 0.0;
        std::vector<float> alphas;
        for (int tile = next_tile.fetch_add(1); tile < tiles; tile = next_tile.fetch_add(1)) {
            const int* entries = list.data() + first[tile];
            const int count = static_cast<int>(first[tile + 1] - first[tile]);
            alphas.resize(static_cast<std::size_t>(count));
            for (int ly = 0; ly < kTile; ++ly)
                for (int lx = 0; lx < kTile; ++lx) {
                    const int x = (tile % tiles_x) * kTile + lx, y = (tile / tiles_x) * kTile + ly;
                    if (x >= width || y >= height) continue;
                    const std::size_t at = static_cast<std::size_t>(y) * width + x;
                    float T = 1.f, C[3] = {0.f, 0.f, 0.f};
                    int used = 0;
                    for (int k = 0; k < count; ++k) {
                        if (T < kMinTransmittance) break;
                        const HostRecord& r = records[entries[k]];
                        PairGraph leaves(r);
                        auto q = op::mahalanobis_distance_with_center(static_cast<float>(x), static_cast<float>(y), leaves.centre, leaves.inv);
                        auto half = q * 0.5f;
                        auto minus = op::neg(half);
                        auto w = op::exp(minus);
                        w.forward();
                        const float a = w[0] * r.alpha0;
                        const float alpha = a > kAlphaMax ? kAlphaMax : a;
                        alphas[k] = a;
                        const float weight = T * alpha;
                        C[0] += weight * r.colour[0];
                        C[1] += weight * r.colour[1];
                        C[2] += weight * r.colour[2];
                        T *= 1.f - alpha;
                        used = k + 1;
                    }
                    float dC[3];
                    for (int c = 0; c < 3; ++c) {
                        image[at * 3 + c] = C[c];
                        const float d = C[c] - target[at * 3 + c];
                        loss += static_cast<double>(d) * d;
                        dC[c] = 2.f * d;
                    }
                    if (!mine) continue;
                    // back to front: transmittance in front of each Gaussian, colour composited behind it
                    float behind[3] = {0.f, 0.f, 0.f};
                    for (int k = used - 1; k >= 0; --k) {
                        const int g = entries[k];
                        const HostRecord& r = records[g];
                        const float a = alphas[k];
                        const float alpha = a > kAlphaMax ? kAlphaMax : a;
                        T = T / (1.f - alpha);
                        float* out = mine + static_cast<std::size_t>(g) * 9;
                        float d_alpha = 0.f;
                        for (int c = 0; c < 3; ++c) {
                            d_alpha += (r.colour[c] - behind[c]) * dC[c];
                            out[5 + c] += alpha * T * dC[c];
                            behind[c] = alpha * r.colour[c] + (1.f - alpha) * behind[c];
                        }
                        d_alpha *= T;
                        if (a > kAlphaMax) continue;  // clamped: no gradient through alpha
                        PairGraph leaves(r);
                        auto q = op::mahalanobis_distance_with_center(static_cast<float>(x), static_cast<float>(y), leaves.centre, leaves.inv);
                        auto half = q * 0.5f;
                        auto minus = op::neg(half);
                        auto w = op::exp(minus);
                        w.forward();
                        out[8] += d_alpha * w[0];           // d loss / d alpha0
                        w.add_grad(0, d_alpha * r.alpha0);  // d loss / d falloff
                        w.backward();
                        out[0] += leaves.centre.grad(0);
                        out[1] += leaves.centre.grad(1);
                        out[2] += leaves.inv.grad(0);
                        out[3] += leaves.inv.grad(1);
                        out[4] += leaves.inv.grad(2);
                    }
                }
        }
        loss_parts[static_cast<std::size_t>(t)] = loss;
    });
    double loss = 0.0;
    for (double part : loss_parts) loss += part;
    if (loss_out) *loss_out = loss;
    if (!grads) return XAD_OK;

    // ---- sum the threads' copies; per Gaussian, back through the projection graph
    run_threads(threads, [&](int t) {
        for (std::size_t g = static_cast<std::size_t>(t); g < n; g += static_cast<std::size_t>(threads)) {
            float a[9] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            for (int copy = 0; copy < threads; ++copy)
                for (int k = 0; k < 9; ++k) a[k] += acc[(static_cast<std::size_t>(copy) * n + g) * 9 + k];
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
            inv.add_grad(0, a[2]);
            inv.add_grad(1, a[3]);
            inv.add_grad(2, a[4]);
            inv.backward();
            alpha0.forward();
            alpha0.add_grad(0, a[8]);
            alpha0.backward();
            grads[0 * n + g] = a[0];
            grads[1 * n + g] = a[1];
            grads[2 * n + g] = log_scale.grad(0);
            grads[3 * n + g] = log_scale.grad(1);
            grads[4 * n + g] = theta.grad(0);
            grads[5 * n + g] = a[5];
            grads[6 * n + g] = a[6];
            grads[7 * n + g] = a[7];
            grads[8 * n + g] = opacity.grad(0);
        }
    });
    return XAD_OK;
}
