"""The splatting step built from the library's templates for the host cores, against the oracle.

Runs without a GPU.  xad_host_splat_step_f32 evaluates every (pixel, Gaussian) pair through the per-pair
graph of operation nodes; the oracle states the same step in closed form.  Same criterion as for the GPU
step: every gradient within 1e-4 of its mass plus the first-order fp32 bound of the fp64 oracle, the image
within 1e-5 plus its bound.
"""
import numpy as np
import pytest

from tests._scenes import random_scene
from xyz_autodiff_cuda_amd import splat

SCENES = [
    # G, W, H, scale_px, opacity shift, seed
    (600, 96, 80, (1.0, 12.0), 0.0, 31),  # ragged: neither side a multiple of the tile
    (3000, 256, 160, (0.5, 40.0), 1.5, 32),  # dense, reaches the clamp and the cut-off
    (1, 16, 16, (3.0, 4.0), 0.0, 33),
]


def _case(oracle, G, W, H, scale, shift, seed):
    params, depth = random_scene(G, W, H, seed=seed, scale_px=scale)
    params[8] += shift
    target = np.random.default_rng(seed + 1).uniform(0, 1, (H, W, 3)).astype(np.float32)
    o32 = oracle.splat_step(W, H, params, depth, target, np.float32)
    o64 = oracle.splat_step(W, H, params, depth, target, np.float64, rects_in=o32["rects"], want_bounds=True)
    return params, depth, target, o32, o64


@pytest.mark.parametrize("scene", SCENES)
def test_host_step_matches_the_oracle(oracle, xad, scene):
    G, W, H = scene[:3]
    params, depth, target, o32, o64 = _case(oracle, *scene)
    got = splat.host_step(params, depth, target, W, H, num_threads=4)
    assert got["pairs"] == o32["pairs"]
    tolerance = 1e-4 * o64["grad_mass"] + o64["grad_bound"] + 1e-30
    excess = np.abs(got["grads"].astype(np.float64) - o64["grads"]) / tolerance
    assert excess.max() <= 1.0, (excess.max(), np.unravel_index(excess.argmax(), excess.shape))
    image_excess = np.abs(got["image"].astype(np.float64) - o64["image"]) / (1e-5 + o64["image_bound"])
    assert image_excess.max() <= 1.0, image_excess.max()
    assert abs(got["loss"] - o64["loss"]) <= 1e-5 * o64["loss"]


def test_render_only_and_thread_counts(oracle, xad):
    params, depth, target, o32, _ = _case(oracle, *SCENES[0])
    G, W, H = SCENES[0][:3]
    one = splat.host_step(params, depth, target, W, H, num_threads=1)
    many = splat.host_step(params, depth, target, W, H, num_threads=5)
    render = splat.host_step(params, depth, target, W, H, want_grads=False, num_threads=3)
    # a pixel is composited by one thread whatever the count; gradients are sums over threads' copies
    assert np.array_equal(one["image"], many["image"]) and np.array_equal(one["image"], render["image"])
    assert render["grads"] is None
    assert np.allclose(one["grads"], many["grads"], rtol=1e-4, atol=1e-6 * np.abs(one["grads"]).max())


def test_arguments_are_checked(xad):
    params = np.zeros((9, 4), np.float32)
    with pytest.raises(ValueError):
        splat.host_step(params[:8], np.zeros(4, np.float32), np.zeros((8, 8, 3), np.float32), 8, 8)
    with pytest.raises(ValueError):
        splat.host_step(params, np.zeros(3, np.float32), np.zeros((8, 8, 3), np.float32), 8, 8)
