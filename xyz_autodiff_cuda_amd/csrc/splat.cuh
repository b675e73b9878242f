#pragma once
// Shared definitions of the tile-binned 2D Gaussian-splatting step.
//
// Model (the one the benchmark configuration specifies; the renderer of
// xyz-autodiff-cuda, examples/mini-gaussian-splatting/gaussian_splatting_kernel.cu:8-112,
// adds every Gaussian at every pixel instead):
//   - parameters: nine rows of G floats (cx, cy, log-scale x, log-scale y, theta,
//     r, g, b, opacity logit), the fields of the reference's GaussianParams
//     (examples/mini-gaussian-splatting/gaussian_parameters.h:12-18) as a structure
//     of arrays, plus one row of depths that is not trained;
//   - 16x16-pixel tiles; a Gaussian belongs to every tile its 3-sigma
//     axis-aligned box touches and contributes to exactly those tiles' pixels;
//   - per tile, Gaussians ordered by (depth, index); front-to-back compositing
//     with alpha = min(0.99, sigmoid(o) exp(-q/2)); a pixel stops before a
//     Gaussian once its transmittance is below 1e-4; black background;
//   - loss = sum over pixels and channels of (C - target)^2.
// The per-Gaussian falloff is the reference's graph (gaussian_splatting_kernel.cu:42-55)
// built from the library's op logic.

#include <cstdint>

namespace xad_splat {

constexpr int kTile = 16;
constexpr int kTilePixels = kTile * kTile;
constexpr float kAlphaMax = 0.99f;
constexpr float kMinTransmittance = 1e-4f;
constexpr int kParamRows = 9;

// What the render kernels read per Gaussian: 48 bytes, three 16-byte loads.
struct alignas(16) Record {
    float cx, cy, a, b;      // centre; inverse covariance [a b; b c]
    float c, red, green, blue;
    float alpha0;            // sigmoid(opacity logit)
    float pad0, pad1, pad2;
};
static_assert(sizeof(Record) == 48, "Record must be three float4");

// Tile rectangle of a Gaussian, inclusive; empty when x0 > x1.
struct TileRect {
    std::int16_t x0, y0, x1, y1;
};

// Gradient of the loss with respect to the fields of a Record the parameters
// reach: centre (2), inverse covariance (3), colour (3), alpha0 (1).
constexpr int kRecordGrads = 9;
// Rows of the accumulator are 64 bytes apart, so the atomics on one Gaussian stay in one cache line.
constexpr int kRecordGradStride = 16;

// The loss is summed in kLossParts places, one cache line each (atomics on one address are taken one
// after the other: a single sum would make every tile wait for all the others); the parameter
// backward adds them up into element 0.  Part k is element kLossStride (1 + k).
constexpr int kLossParts = 64;
constexpr int kLossStride = 16;
constexpr int kLossWords = kLossStride * (1 + kLossParts);

}  // namespace xad_splat
