"""The test by which both compositing kernels leave a list entry out of a tile (negligible_in_tile,
csrc/splat_staged.cuh) against brute force over the tile's 256 pixel centres, on the host build of the same
code and, on the GPU, the device build against the host's.

What must hold: an entry that is left out reaches no pixel of the tile with alpha >= 1e-8 (the criterion is a
lower bound of q over the pixels' bounding box, so it may keep entries it could have dropped, never the
reverse); and it is worth having: nearly every entry that is far below the threshold at every pixel is found.
"""
import numpy as np
import pytest

from tests import _native

THRESHOLD = 1e-8


def _pairs(n, seed, scale_px=(0.5, 40.0)):
    """Random Gaussians with the large benchmark's distributions, each paired with a tile around its
    3-sigma box (a few tiles further out as well, where everything is negligible)."""
    r = np.random.default_rng(seed)
    cx, cy = r.uniform(0, 512, n), r.uniform(0, 512, n)
    sx, sy = (np.exp(r.uniform(np.log(scale_px[0]), np.log(scale_px[1]), n)) for _ in range(2))
    theta = r.uniform(-np.pi, np.pi, n)
    alpha0 = 1 / (1 + np.exp(-r.standard_normal(n)))
    c, s = np.cos(theta), np.sin(theta)
    a = c * c / sx**2 + s * s / sy**2
    b = c * s * (1 / sx**2 - 1 / sy**2)
    cc = s * s / sx**2 + c * c / sy**2
    reach = 3.0 * np.maximum(sx, sy) + 24.0
    tile_x = np.floor((cx + r.uniform(-1, 1, n) * reach) / 16) * 16
    tile_y = np.floor((cy + r.uniform(-1, 1, n) * reach) / 16) * 16
    fields = np.stack([cx, cy, a, b, cc, alpha0], axis=1).astype(np.float32)
    tiles = np.stack([tile_x, tile_y], axis=1).astype(np.float32)
    return fields, tiles


def _largest_alpha(fields, tiles):
    """fp64, every pixel centre of every tile."""
    f = fields.astype(np.float64)
    px = tiles[:, 0, None, None].astype(np.float64) + np.arange(16)[None, None, :] - f[:, 0, None, None]
    py = tiles[:, 1, None, None].astype(np.float64) + np.arange(16)[None, :, None] - f[:, 1, None, None]
    q = f[:, 2, None, None] * px * px + 2 * f[:, 3, None, None] * px * py + f[:, 4, None, None] * py * py
    return f[:, 5] * np.exp(-0.5 * q.min(axis=(1, 2)))


@pytest.mark.parametrize("seed,scale_px", [(1, (0.5, 40.0)), (2, (1.0, 20.0)), (3, (0.3, 3.0))])
def test_nothing_visible_is_left_out_and_most_of_the_invisible_is_found(seed, scale_px):
    fields, tiles = _pairs(40_000, seed, scale_px)
    left_out = _native.negligible_in_tile(fields, tiles)
    largest = _largest_alpha(fields, tiles)
    # never the reverse: what is left out is below the threshold at every pixel (1 % for fp32 against fp64)
    assert left_out.any() and (~left_out).any()
    assert largest[left_out].max() < THRESHOLD * 1.01, largest[left_out].max()
    # worth having: what is far below the threshold everywhere is nearly always recognised (the bounding-box
    # minimum is a little smaller than the minimum over the pixel centres)
    clearly_invisible = largest < THRESHOLD * 1e-3
    assert left_out[clearly_invisible].mean() > 0.98, left_out[clearly_invisible].mean()
    # and the centre inside the tile's box means visible, whatever the shape
    inside = (np.abs(fields[:, 0] - tiles[:, 0] - 7.5) <= 7.5) & (np.abs(fields[:, 1] - tiles[:, 1] - 7.5) <= 7.5)
    assert inside.any() and not left_out[inside & (fields[:, 5] > 1e-6)].any()


def test_odd_records_are_kept():
    fields, tiles = _pairs(64, 4)
    fields[:16, 2] = np.nan  # comparisons with NaN are false: kept, and the projection never bins such a record anyway
    fields[16:32, 5] = 0.0   # alpha0 = 0: nothing to see anywhere
    out = _native.negligible_in_tile(fields, tiles)
    assert not out[:16].any() and out[16:32].all()


def test_fraction_of_the_large_benchmark_scene():
    """The figure behind the kernels' instruction counts: with scales from 0.5 to 40 px about a fifth of the
    (tile, Gaussian) pairs of the 3-sigma boxes cannot be seen from their tile."""
    r = np.random.default_rng(1234)
    G, width, height = 20_000, 2048, 2048
    cx, cy = r.uniform(0, width, G), r.uniform(0, height, G)
    sx, sy = (np.exp(r.uniform(np.log(0.5), np.log(40.0), G)) for _ in range(2))
    theta = r.uniform(-np.pi, np.pi, G)
    alpha0 = 1 / (1 + np.exp(-r.standard_normal(G)))
    c, s = np.cos(theta), np.sin(theta)
    cov_xx, cov_yy = c * c * sx**2 + s * s * sy**2, s * s * sx**2 + c * c * sy**2
    a, b, cc = c * c / sx**2 + s * s / sy**2, c * s * (1 / sx**2 - 1 / sy**2), s * s / sx**2 + c * c / sy**2
    rx, ry = 3 * np.sqrt(cov_xx), 3 * np.sqrt(cov_yy)
    x_lo, x_hi = np.clip(np.floor((cx - rx) / 16), 0, 127).astype(int), np.clip(np.floor((cx + rx) / 16), 0, 127).astype(int)
    y_lo, y_hi = np.clip(np.floor((cy - ry) / 16), 0, 127).astype(int), np.clip(np.floor((cy + ry) / 16), 0, 127).astype(int)
    nx, ny = x_hi - x_lo + 1, y_hi - y_lo + 1
    count = nx * ny
    g = np.repeat(np.arange(G), count)
    k = np.arange(count.sum()) - np.repeat(np.cumsum(count) - count, count)
    tiles = np.stack([(x_lo[g] + k % nx[g]) * 16, (y_lo[g] + k // nx[g]) * 16], axis=1).astype(np.float32)
    fields = np.stack([cx, cy, a, b, cc, alpha0], axis=1).astype(np.float32)[g]
    fraction = _native.negligible_in_tile(fields, tiles).mean()
    assert 0.17 < fraction < 0.27, fraction


@pytest.mark.gpu
def test_device_build_decides_like_the_host_build(gpu):
    fields, tiles = _pairs(100_000, 7)
    host = _native.negligible_in_tile(fields, tiles)
    device = _native.negligible_in_tile(fields, tiles, device=True)
    # the two differ in the last bits of exp2: only entries within a percent of the threshold may fall either way
    largest = _largest_alpha(fields, tiles)
    differ = host != device
    assert differ.mean() < 1e-3
    assert np.all(np.abs(np.log(largest[differ] / THRESHOLD)) < 12.0) if differ.any() else True
    assert largest[device].max() < THRESHOLD * 1.01
