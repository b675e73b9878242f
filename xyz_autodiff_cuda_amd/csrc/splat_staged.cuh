#pragma once
// A Gaussian's record as the compositing kernels stage it in LDS, and the test that leaves an entry
// of a tile's list out of both compositing passes.  In a header of its own, and callable on the host
// as well, so that the test can be checked against brute force over a tile's pixels without a GPU.
#include <cstdint>

#include <xyz_autodiff/detail/config.cuh>
#include <xyz_autodiff/operations/math.cuh>

#include "splat.cuh"

namespace xad_splat {

using namespace xyz_autodiff;

constexpr float kHalfLog2e = 0.72134752044448170368f;  // log2(e) / 2

struct alignas(16) Staged {
    float cx, cy, a_s, b2_s;          // centre; a' and 2b'
    float c_s, alpha0, red, green;    // c'; sigmoid(opacity); colour
    float blue, a, b, c;              // colour; inverse covariance as stored
};
static_assert(sizeof(Staged) == 48, "Staged must be three float4");

XAD_INLINE Staged stage_record(const Record* __restrict__ records, std::uint32_t g) {
    const float4* src = reinterpret_cast<const float4*>(records + g);
    const float4 v0 = src[0], v1 = src[1], v2 = src[2];
    Staged s;
    s.cx = v0.x;
    s.cy = v0.y;
    s.a = v0.z;
    s.b = v0.w;
    s.c = v1.x;
    s.red = v1.y;
    s.green = v1.z;
    s.blue = v1.w;
    s.alpha0 = v2.x;
    s.a_s = -kHalfLog2e * s.a;
    s.b2_s = -2.f * kHalfLog2e * s.b;
    s.c_s = -kHalfLog2e * s.c;
    return s;
}

// List entries that cannot be seen from a tile.  The binning rectangle is the 3-sigma box of the
// Gaussian's own axes-aligned extent, so a rotated, elongated Gaussian is listed in corner tiles that
// its ellipse never comes near (about a fifth of all pairs when scales span 0.5 to 40 pixels).  Such
// an entry is recognised when its record is staged: the minimum of q over the tile's pixel centres
// is bounded from below by the minimum over their bounding box, which for a convex quadratic whose
// centre lies outside the box is attained on one of the four edges.  If even there alpha stays below
// kNegligibleAlpha, the entry is left out of the compositing loops of this tile, forward and backward
// alike: it would change a pixel by less than 1e-8 (an fp32 ulp of 0.5 is 6e-8).  Lists and pair
// counts are not affected.  Comparisons with NaN are false, so an odd record is kept.
constexpr float kNegligibleAlpha = 1e-8f;

XAD_INLINE bool negligible_in_tile(const Staged& s, float tile_x, float tile_y) {
    const float x0 = tile_x - s.cx, x1 = x0 + static_cast<float>(kTile - 1);
    const float y0 = tile_y - s.cy, y1 = y0 + static_cast<float>(kTile - 1);
    float q_min = 0.f;
    if (!(x0 <= 0.f && x1 >= 0.f && y0 <= 0.f && y1 >= 0.f)) {
        auto along_x = [&](float y) {  // min over x in [x0, x1] of a x^2 + 2 b x y + c y^2
            const float x = __builtin_fminf(__builtin_fmaxf(-s.b * y / s.a, x0), x1);
            return ::fmaf(::fmaf(s.a, x, 2.f * s.b * y), x, s.c * y * y);
        };
        auto along_y = [&](float x) {
            const float y = __builtin_fminf(__builtin_fmaxf(-s.b * x / s.c, y0), y1);
            return ::fmaf(::fmaf(s.c, y, 2.f * s.b * x), y, s.a * x * x);
        };
        q_min = __builtin_fminf(__builtin_fminf(along_x(y0), along_x(y1)), __builtin_fminf(along_y(x0), along_y(x1)));
    }
    return s.alpha0 * math::fp32::exp2_raw(-kHalfLog2e * q_min) < kNegligibleAlpha;
}

}  // namespace xad_splat
