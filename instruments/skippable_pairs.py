"""How many (tile, Gaussian) pairs of a scene a tile's pixels cannot see.

    python3 -m instruments.skippable_pairs [--gaussians 200000 --width 2048 --height 2048 --scale 0.5 40]

The binning rectangle of a Gaussian is the 3-sigma box of its axis-aligned extent, so a rotated, elongated
Gaussian is listed in corner tiles its ellipse never comes near.  For every pair of a random scene with the
benchmark's distributions (numpy, on the CPU) this computes the largest alpha the Gaussian reaches at any
pixel centre of the tile's bounding box, the quantity the compositing kernels test when they stage a record
(negligible_in_tile in csrc/splat_kernels.hip), and prints the fraction of pairs below a few thresholds.
"""
import argparse

import numpy as np


def skippable_fractions(num_gaussians, width, height, scale_px, seed=1234, thresholds=(1e-8, 1e-6, 1e-4, 1 / 255)):
    rng = np.random.default_rng(seed)
    G = num_gaussians
    cx, cy = rng.uniform(0, width, G), rng.uniform(0, height, G)
    sx, sy = (np.exp(rng.uniform(np.log(scale_px[0]), np.log(scale_px[1]), G)) for _ in range(2))
    theta = rng.uniform(-np.pi, np.pi, G)
    alpha0 = 1 / (1 + np.exp(-rng.standard_normal(G)))
    c, s = np.cos(theta), np.sin(theta)
    cov_xx, cov_yy = c * c * sx**2 + s * s * sy**2, s * s * sx**2 + c * c * sy**2
    A, B, C = c * c / sx**2 + s * s / sy**2, c * s * (1 / sx**2 - 1 / sy**2), s * s / sx**2 + c * c / sy**2
    tiles_x, tiles_y = (width + 15) // 16, (height + 15) // 16
    rx, ry = 3 * np.sqrt(cov_xx), 3 * np.sqrt(cov_yy)
    x_lo, x_hi = np.floor((cx - rx) / 16), np.floor((cx + rx) / 16)
    y_lo, y_hi = np.floor((cy - ry) / 16), np.floor((cy + ry) / 16)
    on = ~((x_hi < 0) | (y_hi < 0) | (x_lo > tiles_x - 1) | (y_lo > tiles_y - 1))
    x_lo, x_hi = np.clip(x_lo, 0, tiles_x - 1).astype(np.int64), np.clip(x_hi, 0, tiles_x - 1).astype(np.int64)
    y_lo, y_hi = np.clip(y_lo, 0, tiles_y - 1).astype(np.int64), np.clip(y_hi, 0, tiles_y - 1).astype(np.int64)
    nx, ny = np.where(on, x_hi - x_lo + 1, 0), np.where(on, y_hi - y_lo + 1, 0)
    count = nx * ny
    g = np.repeat(np.arange(G), count)
    k = np.arange(count.sum()) - np.repeat(np.cumsum(count) - count, count)
    tx, ty = x_lo[g] + k % nx[g], y_lo[g] + k // nx[g]
    # the tile's pixel centres, relative to the Gaussian's centre
    x0, y0 = tx * 16 - cx[g], ty * 16 - cy[g]
    x1, y1 = x0 + 15, y0 + 15
    a, b, cc = A[g], B[g], C[g]

    def along_x(y):  # min over x in [x0, x1] of a x^2 + 2 b x y + c y^2
        x = np.clip(-b * y / a, x0, x1)
        return a * x * x + 2 * b * x * y + cc * y * y

    def along_y(x):
        y = np.clip(-b * x / cc, y0, y1)
        return a * x * x + 2 * b * x * y + cc * y * y

    inside = (x0 <= 0) & (x1 >= 0) & (y0 <= 0) & (y1 >= 0)
    q_min = np.where(inside, 0.0, np.minimum(np.minimum(along_x(y0), along_x(y1)), np.minimum(along_y(x0), along_y(x1))))
    largest_alpha = alpha0[g] * np.exp(-0.5 * q_min)
    return int(count.sum()), {t: float((largest_alpha < t).mean()) for t in thresholds}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gaussians", type=int, default=200_000)
    ap.add_argument("--width", type=int, default=2048)
    ap.add_argument("--height", type=int, default=2048)
    ap.add_argument("--scale", type=float, nargs=2, default=(0.5, 40.0))
    args = ap.parse_args()
    pairs, fractions = skippable_fractions(args.gaussians, args.width, args.height, tuple(args.scale))
    print("%d Gaussians, %d x %d, scales %g..%g px: %d pairs" % (args.gaussians, args.width, args.height, *args.scale, pairs))
    for threshold, fraction in fractions.items():
        print("  largest alpha over the tile < %-8.3g : %.3f of the pairs" % (threshold, fraction))


if __name__ == "__main__":
    main()
