"""GPU parity of the tile-binned splatting step and Adam, through the C ABI.

Checker: the CPU oracle (tests/test_oracle_splat.py pins it), run on the same
parameters in fp32 and fp64.  Tolerances:
  - binning is integer work: pair count and longest list must be equal;
  - image: 1e-5 absolute (values are in [0, 1]);
  - loss: 1e-6 relative;
  - gradients (summed over pixels with atomics, then pushed through the
    per-Gaussian graph): |error| <= (1e-4 + 2e-5 cond_g) S_g, S_g the largest
    gradient magnitude of that Gaussian and cond_g = e^(2 |log sx - log sy|) the
    condition number of its covariance, whose inverse both implementations form
    in fp32; and never more than twice the fp32 oracle's own distance from fp64.
"""
import numpy as np
import pytest

from tests._scenes import one_gaussian, random_scene

pytestmark = pytest.mark.gpu


def _gpu_step(gpu, W, H, params, depth, target, forward_only=False):
    import torch

    from xyz_autodiff_cuda_amd import splat

    ctx = splat.SplatContext(W, H, params.shape[1])
    p, d, t = (torch.from_numpy(np.ascontiguousarray(a)).to(gpu) for a in (params, depth, target))
    if forward_only:
        image = ctx.forward(p, d)
        torch.cuda.synchronize()
        out = {"image": image.cpu().numpy()}
    else:
        image, grads, loss = ctx.step(p, d, t)
        torch.cuda.synchronize()
        out = {"image": image.cpu().numpy(), "grads": grads.cpu().numpy(), "loss": loss}
    out.update(ctx.stats(longest_list=True))
    ctx.close()
    return out


def _check_against_oracle(oracle, got, W, H, params, depth, target):
    o32 = oracle.splat_step(W, H, params, depth, target, np.float32)
    o64 = oracle.splat_step(W, H, params, depth, target, np.float64)
    assert got["pairs"] == o32["pairs"] and got["longest_list"] == o32["longest_list"]
    assert np.isfinite(got["image"]).all() and np.isfinite(got["grads"]).all()
    if o64["pairs"] != o32["pairs"]:
        # a 3-sigma box that ends within rounding of a tile edge is binned differently in fp64: the
        # scenes then differ by whole (tile, Gaussian) pairs and only the fp32 oracle is comparable
        o64 = o32
    for ref in (o32, o64):
        assert np.abs(got["image"].astype(np.float64) - ref["image"]).max() < 1e-5
        assert abs(got["loss"] - ref["loss"]) <= 1e-6 * ref["loss"] + 1e-9
    cond = np.exp(2.0 * np.abs(params[2].astype(np.float64) - params[3]))
    scale = np.abs(o64["grads"]).max(axis=0) + 1e-20
    bound = (1e-4 + 2e-5 * cond) * scale
    g = got["grads"].astype(np.float64)
    for ref in (o32, o64):
        assert (np.abs(g - ref["grads"]) <= bound).all(), (np.abs(g - ref["grads"]) / bound).max()
    dev_err = (np.abs(g - o64["grads"]) / scale).max()
    ref_err = (np.abs(o32["grads"].astype(np.float64) - o64["grads"]) / scale).max()
    assert dev_err <= 2.0 * ref_err + 1e-5


@pytest.mark.parametrize("G,W,H,scale", [
    (1, 16, 16, (2.0, 4.0)),
    (7, 33, 17, (1.0, 6.0)),        # ragged image: partial tiles on both edges
    (300, 100, 60, (1.0, 12.0)),
    (3000, 256, 192, (1.0, 20.0)),  # lists longer than one 256-entry chunk in dense tiles
])
def test_step_matches_oracle(gpu, oracle, G, W, H, scale):
    params, depth = random_scene(G, W, H, seed=G, scale_px=scale)
    target = np.random.default_rng(G + 1).uniform(0, 1, (H, W, 3)).astype(np.float32)
    _check_against_oracle(oracle, _gpu_step(gpu, W, H, params, depth, target), W, H, params, depth, target)


def test_depth_ranks_follow_the_depths_of_each_call(gpu, oracle):
    """The context keeps the depth ranks of the previous call while the depths stay the same;
    a call with other depths (even one changed value) must be ordered by them."""
    import torch

    from xyz_autodiff_cuda_amd import splat

    W, H, G = 96, 80, 400
    params, depth = random_scene(G, W, H, seed=8, scale_px=(3.0, 15.0))
    params[8] += 2.0  # opaque enough for the order to matter
    reversed_depth = (1.0 - depth).astype(np.float32)
    one_changed = depth.copy()
    one_changed[np.argmax(depth)] = -1.0  # the farthest Gaussian comes to the front
    ctx = splat.SplatContext(W, H, G)
    p = torch.from_numpy(params).to(gpu)
    for d in (depth, depth, reversed_depth, one_changed, depth):
        image = ctx.forward(p, torch.from_numpy(d).to(gpu)).cpu().numpy()
        want = oracle.splat_step(W, H, params, d, np.zeros((H, W, 3), np.float32), np.float32, want_grads=False)["image"]
        assert np.abs(image - want).max() < 1e-5
    assert np.abs(oracle.splat_step(W, H, params, one_changed, np.zeros((H, W, 3), np.float32), np.float32, want_grads=False)["image"] - want).max() > 1e-3
    ctx.close()


def test_more_than_65536_tiles(gpu, oracle):
    """256 x 257 tiles: the pair keys (tile indices) take the 32-bit path.  Small Gaussians keep
    the oracle fast."""
    W, H, G = 4096, 4112, 60_000
    params, depth = random_scene(G, W, H, seed=21, scale_px=(0.5, 1.5))
    params[1, :2000] = np.random.default_rng(5).uniform(H - 40, H, 2000)  # populate the last tile rows
    depth[::7] = depth[3]  # many depth ties: order falls back to the index
    target = np.zeros((H, W, 3), np.float32)
    _check_against_oracle(oracle, _gpu_step(gpu, W, H, params, depth, target), W, H, params, depth, target)


def test_long_lists_and_early_termination(gpu, oracle):
    """Many opaque Gaussians stacked on a few tiles: lists span several LDS
    chunks and most pixels stop long before the end of their list."""
    G, W, H = 1500, 48, 48
    params, depth = random_scene(G, W, H, seed=21, scale_px=(4.0, 16.0))
    params[8] += 3.0  # opacity logits around 3: alpha near 0.95
    target = np.random.default_rng(2).uniform(0, 1, (H, W, 3)).astype(np.float32)
    got = _gpu_step(gpu, W, H, params, depth, target)
    assert got["longest_list"] > 512
    _check_against_oracle(oracle, got, W, H, params, depth, target)


def test_forward_only_equals_step_image(gpu, oracle):
    G, W, H = 200, 64, 64
    params, depth = random_scene(G, W, H, seed=4, scale_px=(1.0, 10.0))
    target = np.zeros((H, W, 3), np.float32)
    a = _gpu_step(gpu, W, H, params, depth, target, forward_only=True)["image"]
    b = _gpu_step(gpu, W, H, params, depth, target)["image"]
    assert np.array_equal(a, b)


def test_clamp_cutoff_and_depth_ties(gpu, oracle):
    W = H = 16
    layers = [one_gaussian(8, 8, np.log(1000.0), np.log(1000.0), 0.0, (1.0, 0.0, 0.0), 12.0) for _ in range(5)]
    layers[3][5:8, 0] = (0.0, 1.0, 0.0)
    params = np.concatenate(layers, axis=1)
    depth = np.full(5, 0.5, np.float32)  # all equal: index order decides
    target = np.zeros((H, W, 3), np.float32)
    got = _gpu_step(gpu, W, H, params, depth, target)
    # in fp32, (1 - 0.99)^2 falls just below the 1e-4 threshold, so two layers are drawn
    # (three in fp64, tests/test_oracle_splat.py); the fp32 oracle is the judge here
    ref = oracle.splat_step(W, H, params, depth, target, np.float32)
    assert np.allclose(got["image"], ref["image"], rtol=1e-6, atol=0)
    assert np.allclose(got["image"][..., 0], 0.99 * 1.01, rtol=1e-6)
    assert np.all(got["image"][..., 1:] == 0.0)
    assert np.all(got["grads"][:, 2:] == 0.0)               # never composited
    assert np.all(got["grads"][[0, 1, 2, 3, 4, 8]] == 0.0)  # clamped alpha passes nothing
    assert np.allclose(got["grads"], ref["grads"], rtol=1e-5, atol=1e-6)


def test_offscreen_and_nonfinite_gaussians(gpu, oracle):
    W = H = 32
    params, depth = random_scene(6, W, H, 5, scale_px=(1.0, 4.0))
    params[0, 0] = -500.0
    params[1, 1] = 1e6
    params[2, 2] = np.nan
    target = np.zeros((H, W, 3), np.float32)
    got = _gpu_step(gpu, W, H, params, depth, target)
    ref = oracle.splat_step(W, H, params, depth, target, np.float32)
    assert got["pairs"] == ref["pairs"]
    assert np.isfinite(got["image"]).all()
    assert np.abs(got["image"] - ref["image"]).max() < 1e-5
    assert np.all(got["grads"][:, :2] == 0.0)


@pytest.mark.parametrize("W,H", [(8, 8), (40, 24), (1100, 1100)])
def test_a_scene_with_nothing_on_screen(gpu, W, H):
    """No pair at all: every tile's list is empty, the image is the background, the loss is the target's
    energy and no gradient is touched (images smaller than a tile, a few tiles, and many tiles)."""
    G = 50
    params, depth = random_scene(G, W, H, 3, scale_px=(1.0, 3.0))
    params[0] = -1000.0 - np.arange(G)  # far off to the left
    target = np.random.default_rng(2).uniform(0, 1, (H, W, 3)).astype(np.float32)
    got = _gpu_step(gpu, W, H, params, depth, target)
    assert got["pairs"] == 0 and got["longest_list"] == 0
    assert np.all(got["image"] == 0.0) and np.all(got["grads"] == 0.0)
    assert got["loss"] == pytest.approx(float((target.astype(np.float64) ** 2).sum()), rel=1e-6)


def test_host_core_step_and_gpu_step_agree(gpu, oracle):
    """The step from the library's templates on the host cores and the GPU step, on one scene: the same pairs, the
    same image to 1e-5, gradients within the tolerance either is held to against the oracle."""
    from xyz_autodiff_cuda_amd import splat

    G, W, H = 1500, 200, 136
    params, depth = random_scene(G, W, H, seed=41, scale_px=(1.0, 16.0))
    target = np.random.default_rng(8).uniform(0, 1, (H, W, 3)).astype(np.float32)
    got = _gpu_step(gpu, W, H, params, depth, target)
    host = splat.host_step(params, depth, target, W, H, num_threads=4)
    assert host["pairs"] == got["pairs"]
    assert np.abs(host["image"] - got["image"]).max() < 1e-5
    assert abs(host["loss"] - got["loss"]) <= 1e-6 * got["loss"]
    o64 = oracle.splat_step(W, H, params, depth, target, np.float64,
                            rects_in=oracle.splat_step(W, H, params, depth, target, np.float32)["rects"], want_bounds=True)
    tolerance = 1e-4 * o64["grad_mass"] + o64["grad_bound"] + 1e-30
    assert (np.abs(host["grads"].astype(np.float64) - got["grads"]) <= 2.0 * tolerance).all()


def test_pair_buffers_grow_on_demand(gpu, oracle):
    import torch

    from xyz_autodiff_cuda_amd import splat

    G, W, H = 400, 128, 128
    params, depth = random_scene(G, W, H, seed=8, scale_px=(8.0, 20.0))
    target = np.zeros((H, W, 3), np.float32)
    ctx = splat.SplatContext(W, H, G, pair_capacity_hint=16)  # far too small on purpose
    p, d, t = (torch.from_numpy(a).to(gpu) for a in (params, depth, target))
    image, grads, loss = ctx.step(p, d, t)
    torch.cuda.synchronize()
    ref = oracle.splat_step(W, H, params, depth, target, np.float32)
    assert ctx.stats()["pairs"] == ref["pairs"] > 16
    assert np.abs(image.cpu().numpy() - ref["image"]).max() < 1e-5
    ctx.close()


def test_repeated_steps_are_independent(gpu):
    import torch

    from xyz_autodiff_cuda_amd import splat

    G, W, H = 500, 96, 96
    params, depth = random_scene(G, W, H, seed=9, scale_px=(1.0, 12.0))
    target = np.random.default_rng(1).uniform(0, 1, (H, W, 3)).astype(np.float32)
    ctx = splat.SplatContext(W, H, G)
    p, d, t = (torch.from_numpy(a).to(gpu) for a in (params, depth, target))
    first = [x.clone() if hasattr(x, "clone") else x for x in ctx.step(p, d, t)]
    for _ in range(3):
        again = ctx.step(p, d, t)
    torch.cuda.synchronize()
    assert torch.equal(first[0], again[0])
    scale = first[1].abs().amax(dim=0) + 1e-20
    # atomics: the order of the per-tile sums varies from run to run (1e-4 relative is the figure allowed for
    # that); the values do not pile up from call to call
    assert float(((first[1] - again[1]).abs() / scale).max()) < 1e-4
    assert abs(first[2] - again[2]) <= 1e-9 * first[2]
    ctx.close()


def test_adam_matches_oracle_over_steps(gpu, oracle):
    import torch

    from xyz_autodiff_cuda_amd import splat

    rows, n = 9, 1237
    r = np.random.default_rng(3)
    p0 = r.normal(0, 1, (rows, n)).astype(np.float32)
    lrs = [1e-2, 1e-2, 5e-3, 5e-3, 1e-3, 2e-2, 2e-2, 2e-2, 1e-2]
    p = torch.from_numpy(p0.copy()).to(gpu)
    m = torch.zeros_like(p)
    v = torch.zeros_like(p)
    hp, hm, hv = p0.copy(), np.zeros_like(p0), np.zeros_like(p0)
    for t in range(1, 21):
        g = r.normal(0, 2, (rows, n)).astype(np.float32)
        g[:, ::97] = 0.0
        splat.adam_step(p, torch.from_numpy(g).to(gpu), m, v, lrs, t)
        for row in range(rows):
            oracle.adam_step(hp[row], np.ascontiguousarray(g[row]), hm[row], hv[row], lrs[row], 0.9, 0.999, 1e-8, t)
    torch.cuda.synchronize()
    assert np.allclose(p.cpu().numpy(), hp, rtol=1e-5, atol=1e-6)
    assert np.allclose(m.cpu().numpy(), hm, rtol=1e-5, atol=1e-7)
    assert np.allclose(v.cpu().numpy(), hv, rtol=1e-5, atol=1e-9)


def test_training_reduces_the_loss(gpu):
    """Forward + backward + Adam (lr 1e-2) for a few iterations on a small
    instance of the benchmark recipe: the loss must go down."""
    import torch

    from xyz_autodiff_cuda_amd import splat

    G, W, H = 2000, 128, 128
    target = splat.synthetic_target(G, W, H, seed=77, noise=0.02)
    params, depth = splat.synthetic_scene(G, W, H, seed=1234)
    ctx = splat.SplatContext(W, H, G)
    m, v = torch.zeros_like(params), torch.zeros_like(params)
    losses = []
    for it in range(1, 31):
        _, grads, loss = ctx.step(params, depth, target)
        splat.adam_step(params, grads, m, v, 1e-2, it)
        losses.append(loss)
    ctx.close()
    assert np.isfinite(losses).all()
    assert losses[-1] < 0.9 * losses[0]


def test_full_size_config5_properties(gpu):
    """200k Gaussians at 2048 x 2048: too large for the oracle in a test, so
    check what does not depend on it: the image is finite and within [0, 1],
    transmittance bookkeeping is consistent, gradients are finite, and a second
    context reproduces the pair count and the image bit for bit."""
    import torch

    from xyz_autodiff_cuda_amd import splat

    G, W, H = 200_000, 2048, 2048
    params, depth = splat.synthetic_scene(G, W, H, seed=1234, scale_px=(0.5, 40.0))
    target = torch.zeros(H, W, 3, device=gpu)
    ctx = splat.SplatContext(W, H, G, pair_capacity_hint=9_000_000)
    image, grads, loss = ctx.step(params, depth, target)
    torch.cuda.synchronize()
    stats = ctx.stats(longest_list=True)
    assert 4_000_000 < stats["pairs"] < 12_000_000 and stats["longest_list"] < 5000
    assert bool(torch.isfinite(image).all()) and bool(torch.isfinite(grads).all())
    assert float(image.min()) >= 0.0 and float(image.max()) <= 1.0 + 1e-5
    assert abs(loss - float((image.double() ** 2).sum())) <= 1e-6 * loss
    ctx2 = splat.SplatContext(W, H, G)
    image2 = ctx2.forward(params, depth)
    torch.cuda.synchronize()
    assert ctx2.stats()["pairs"] == stats["pairs"]
    assert torch.equal(image, image2)
    ctx.close()
    ctx2.close()


def test_the_getters_report_and_settle_an_overflow_too(gpu, oracle, xad):
    """xad_splat_get_stats and xad_splat_get_lists wait for the device, so they are calls that report what a
    step that did not wait has left behind, and enlarge the lists."""
    import torch

    from xyz_autodiff_cuda_amd import splat

    G, W, H = 600, 256, 256
    small, depth = random_scene(G, W, H, seed=5, scale_px=(0.5, 1.0))
    large = small.copy()
    large[2:4] += np.log(30.0)
    target = np.zeros((H, W, 3), np.float32)
    d, t = torch.from_numpy(depth).to(gpu), torch.from_numpy(target).to(gpu)
    ref = oracle.splat_step(W, H, large, depth, target, np.float32)
    for getter in ("stats", "lists"):
        ctx = splat.SplatContext(W, H, G, pair_capacity_hint=4000, depth_mode="static")
        ctx.step(torch.from_numpy(small).to(gpu), d, t)
        ctx.step(torch.from_numpy(large).to(gpu), d, t, want_loss=False)
        with pytest.raises(xad.XadError, match="incomplete"):
            getattr(ctx, getter)()
        # settled: the same step fits now without anybody waiting for it, and the getters answer
        image, _, _ = ctx.step(torch.from_numpy(large).to(gpu), d, t, want_loss=False)
        assert ctx.stats()["pairs"] == ref["pairs"]
        begin, end, ids = ctx.lists()
        assert int((end - begin).sum()) == ref["pairs"] == ids.size
        assert np.abs(image.cpu().numpy() - ref["image"]).max() < 5e-5
        ctx.close()


def test_forward_only_calls_enlarge_the_lists_themselves(gpu, oracle):
    """In the default depth mode a forward call waits for the binning anyway: a scene that has outgrown the lists
    is binned again into larger ones before anything is composited, also when no call ever asks for a loss."""
    import torch

    from xyz_autodiff_cuda_amd import splat

    G, W, H = 600, 256, 256
    small, depth = random_scene(G, W, H, seed=5, scale_px=(0.5, 1.0))
    target = np.zeros((H, W, 3), np.float32)
    d = torch.from_numpy(depth).to(gpu)
    ctx = splat.SplatContext(W, H, G, pair_capacity_hint=4000)
    ctx.forward(torch.from_numpy(small).to(gpu), d)
    for widen in (6.0, 30.0, 90.0):  # each many times the pairs of the one before
        scene = small.copy()
        scene[2:4] += np.log(widen)
        image = ctx.forward(torch.from_numpy(scene).to(gpu), d)
        torch.cuda.synchronize()
        ref = oracle.splat_step(W, H, scene, depth, target, np.float32)
        assert np.abs(image.cpu().numpy() - ref["image"]).max() < 5e-5, widen
        assert ctx.stats()["pairs"] == ref["pairs"], widen
    ctx.close()


def test_gated_adam_holds_the_update_when_told_to(gpu, oracle):
    import torch

    from xyz_autodiff_cuda_amd import splat

    rows, n = 9, 1000
    r = np.random.default_rng(5)
    p0 = r.normal(0, 1, (rows, n)).astype(np.float32)
    g = torch.from_numpy(r.normal(0, 2, (rows, n)).astype(np.float32)).to(gpu)
    gate = torch.zeros(1, dtype=torch.int32, device=gpu)
    held = torch.zeros(1, dtype=torch.int32, device=gpu)
    plain = [torch.from_numpy(p0.copy()).to(gpu), torch.zeros(rows, n, device=gpu), torch.zeros(rows, n, device=gpu)]
    gated = [x.clone() for x in plain]
    splat.adam_step(plain[0], g, plain[1], plain[2], 1e-2, 1)
    splat.adam_step(gated[0], g, gated[1], gated[2], 1e-2, 1, hold_if_nonzero=gate, held_count=held)
    assert all(torch.equal(a, b) for a, b in zip(plain, gated)) and int(held) == 0
    gate.fill_(7)
    before = [x.clone() for x in gated]
    for _ in range(3):
        splat.adam_step(gated[0], g, gated[1], gated[2], 1e-2, 2, hold_if_nonzero=gate, held_count=held)
    assert all(torch.equal(a, b) for a, b in zip(before, gated)) and int(held) == 3
    gate.zero_()
    splat.adam_step(plain[0], g, plain[1], plain[2], 1e-2, 2)
    splat.adam_step(gated[0], g, gated[1], gated[2], 1e-2, 2, hold_if_nonzero=gate, held_count=held)
    assert all(torch.equal(a, b) for a, b in zip(plain, gated)) and int(held) == 3


# ---- the tile lists themselves (integer work: must equal what the oracle's rectangles and the depths imply) ----

def _expected_lists(rects, depth, tiles_x, tiles_y):
    """Per tile (row-major), the Gaussians whose rectangle covers it, by (depth, index)."""
    rc = rects.astype(np.int64)
    nx = np.maximum(0, rc[:, 2] - rc[:, 0] + 1)
    ny = np.maximum(0, rc[:, 3] - rc[:, 1] + 1)
    count = nx * ny
    g = np.repeat(np.arange(rc.shape[0]), count)
    local = np.arange(count.sum()) - np.repeat(np.cumsum(count) - count, count)
    tile = (rc[g, 1] + local // np.maximum(nx[g], 1)) * tiles_x + rc[g, 0] + local % np.maximum(nx[g], 1)
    order = np.lexsort((g, depth[g], tile))
    tile, g = tile[order], g[order]
    begin = np.searchsorted(tile, np.arange(tiles_x * tiles_y), side="left")
    end = np.searchsorted(tile, np.arange(tiles_x * tiles_y), side="right")
    return begin, end, g


def _assert_lists(ctx, oracle, W, H, params, depth):
    ref = oracle.splat_step(W, H, params, depth, np.zeros((H, W, 3), np.float32), np.float32, want_grads=False)
    tiles_x, tiles_y = (W + 15) // 16, (H + 15) // 16
    want_begin, want_end, want_ids = _expected_lists(ref["rects"], depth, tiles_x, tiles_y)
    begin, end, ids = ctx.lists()
    assert ids.size == want_ids.size == ref["pairs"]
    assert np.array_equal(end - begin, want_end - want_begin)  # every tile's length
    # the lists may sit anywhere in the array; tile by tile their contents must be equal, in order
    got = np.concatenate([ids[b:e] for b, e in zip(begin, end)]) if ids.size else ids
    assert np.array_equal(got, want_ids.astype(np.uint32))
    # and they tile the array exactly once
    covered = np.zeros(ids.size + 1, np.int64)
    np.add.at(covered, begin, 1)
    np.add.at(covered, end, -1)
    assert np.all(np.cumsum(covered)[:-1] == 1)


@pytest.mark.parametrize("G,W,H,scale", [
    (1, 16, 16, (2.0, 4.0)),
    (50, 33, 17, (1.0, 6.0)),        # one supertile, ragged image
    (700, 130, 260, (1.0, 30.0)),    # several supertiles, the last ones partly outside the image
    (5000, 640, 400, (0.5, 40.0)),   # rectangles that span many supertiles
    (20000, 2100, 1100, (1.0, 8.0)), # more than one group of 64 supertiles
])
def test_tile_lists_equal_what_rectangles_and_depths_imply(gpu, oracle, G, W, H, scale):
    import torch

    from xyz_autodiff_cuda_amd import splat

    params, depth = random_scene(G, W, H, seed=G + 3, scale_px=scale)
    depth[::5] = depth[min(2, G - 1)]  # ties: the index decides
    if G > 100:
        params[0, :3] = -1e4   # off screen: no pairs
        params[2:4, 3] = np.log(5000.0)  # one Gaussian over the whole image
    ctx = splat.SplatContext(W, H, G)
    ctx.forward(torch.from_numpy(params).to(gpu), torch.from_numpy(depth).to(gpu))
    _assert_lists(ctx, oracle, W, H, params, depth)
    ctx.close()


@pytest.mark.parametrize("mode", ["static", "every_step"])
def test_steps_that_do_not_wait(gpu, oracle, mode):
    """Without a loss read-back a step only queues work; results equal those of the default mode."""
    import torch

    from xyz_autodiff_cuda_amd import splat

    G, W, H = 900, 160, 112
    params, depth = random_scene(G, W, H, seed=31, scale_px=(1.0, 14.0))
    target = np.random.default_rng(4).uniform(0, 1, (H, W, 3)).astype(np.float32)
    p, t = torch.from_numpy(params).to(gpu), torch.from_numpy(target).to(gpu)
    ctx = splat.SplatContext(W, H, G, depth_mode=mode)
    depths = [depth, depth, (1.0 - depth).astype(np.float32)] if mode == "every_step" else [depth, depth, depth]
    for d in depths:
        image, grads, loss = ctx.step(p, torch.from_numpy(d).to(gpu), t, want_loss=False)
        assert loss is None
        torch.cuda.synchronize()
        ref = oracle.splat_step(W, H, params, d, target, np.float32)
        assert np.abs(image.cpu().numpy() - ref["image"]).max() < 1e-5
        scale = np.abs(ref["grads"]).max(axis=0) + 1e-20
        assert (np.abs(grads.cpu().numpy() - ref["grads"]) / scale).max() < 5e-3
        assert ctx.stats()["pairs"] == ref["pairs"]
    ctx.close()


@pytest.mark.parametrize("G,W,H,scale", [
    (3000, 256, 192, (1.0, 20.0)),    # few tiles: the backward walk in pieces
    (20000, 1100, 1100, (1.0, 24.0)),  # many tiles: one wavefront per tile
])
def test_a_recorded_step_can_be_replayed(gpu, oracle, G, W, H, scale):
    """A step that asks for no loss, in a context whose buffers are sized and whose depths are promised constant, is
    kernel launches only and keeps no host-side state that a launch depends on: recorded into a HIP graph, it can be
    replayed.  Every replay, with the parameters changed in between by ordinary launches, against the same step
    launched the ordinary way."""
    import torch

    from xyz_autodiff_cuda_amd import splat

    params, depth = random_scene(G, W, H, seed=17, scale_px=scale)
    target = np.random.default_rng(6).uniform(0, 1, (H, W, 3)).astype(np.float32)
    p, d, t = (torch.from_numpy(a).to(gpu) for a in (params, depth, target))
    image, grads = torch.empty(H, W, 3, device=gpu), torch.empty(9, G, device=gpu)
    m, v = torch.zeros_like(p), torch.zeros_like(p)
    ctx = splat.SplatContext(W, H, G, depth_mode="static")
    eager = splat.SplatContext(W, H, G)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        ctx.step(p, d, t, image, grads)  # sizes the buffers
        ctx.step(p, d, t, image, grads, want_loss=False)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        ctx.step(p, d, t, image, grads, want_loss=False)
    torch.cuda.synchronize()
    for replay in range(4):
        if replay:
            splat.adam_step(p, grads, m, v, 2e-2, replay)  # other parameters for the next replay
            torch.cuda.synchronize()
        image.fill_(-1.0)
        grads.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        # the same step launched the ordinary way, in a context of its own: the same image bit for bit, the same
        # gradients up to the order of the atomic sums
        want_image, want_grads, want_loss = eager.step(p, d, t)
        torch.cuda.synchronize()
        assert torch.equal(image, want_image), replay
        scale_g = want_grads.abs().amax(dim=0) + 1e-20
        # (sums of terms of either sign, added in another order: 1e-4 of their mass, which in a dense scene
        # is several times the sum itself)
        off = (grads - want_grads).abs() / scale_g
        assert float(off.max()) < 1e-2 and float((off < 1e-4).float().mean()) > 0.999, (replay, float(off.max()))
        assert ctx.stats()["pairs"] == eager.stats()["pairs"], replay
    # the last replay against the oracle, and the context outside the graph
    ref = oracle.splat_step(W, H, p.cpu().numpy(), depth, target, np.float32)
    assert np.abs(image.cpu().numpy() - ref["image"]).max() < 2e-5 and ctx.stats()["pairs"] == ref["pairs"]
    _, _, loss = ctx.step(p, d, t, image, grads)
    assert abs(loss - ref["loss"]) <= 1e-5 * ref["loss"] and abs(loss - want_loss) <= 1e-6 * want_loss
    ctx.close()
    eager.close()


def test_static_mode_reports_a_changed_depth(gpu, xad):
    import torch

    from xyz_autodiff_cuda_amd import splat

    G, W, H = 300, 96, 96
    params, depth = random_scene(G, W, H, seed=12, scale_px=(2.0, 10.0))
    p, t = torch.from_numpy(params).to(gpu), torch.zeros(H, W, 3, device=gpu)
    ctx = splat.SplatContext(W, H, G, depth_mode="static")
    ctx.step(p, torch.from_numpy(depth).to(gpu), t)
    changed = depth.copy()
    changed[7] += 0.25
    ctx.step(p, torch.from_numpy(changed).to(gpu), t, want_loss=False)  # queued; cannot report anything
    with pytest.raises(xad.XadError, match="XAD_SPLAT_DEPTH_STATIC"):
        ctx.step(p, torch.from_numpy(changed).to(gpu), t)
    ctx.step(p, torch.from_numpy(changed).to(gpu), t)  # reordered by the call after the report: fine again
    ctx.close()


def test_overflow_in_a_step_that_does_not_wait_is_reported_later(gpu, oracle, xad):
    import torch

    from xyz_autodiff_cuda_amd import splat

    G, W, H = 600, 256, 256
    small, depth = random_scene(G, W, H, seed=5, scale_px=(0.5, 1.0))
    large = small.copy()
    large[2:4] += np.log(30.0)  # the same Gaussians, thirty times wider: many times the pairs
    target = np.zeros((H, W, 3), np.float32)
    d, t = torch.from_numpy(depth).to(gpu), torch.from_numpy(target).to(gpu)
    ctx = splat.SplatContext(W, H, G, pair_capacity_hint=4000, depth_mode="static")
    ctx.step(torch.from_numpy(small).to(gpu), d, t)  # sized for the small scene
    few = ctx.stats()["pairs"]
    ctx.step(torch.from_numpy(large).to(gpu), d, t, want_loss=False)  # does not fit, and nobody is told yet
    # the next step that waits says so; its own outputs are complete and are handed out
    with pytest.warns(RuntimeWarning, match="incomplete"):
        image, _, loss = ctx.step(torch.from_numpy(small).to(gpu), d, t)
    ref_small = oracle.splat_step(W, H, small, depth, target, np.float32)
    assert np.abs(image.cpu().numpy() - ref_small["image"]).max() < 1e-5 and abs(loss - ref_small["loss"]) <= 1e-6 * ref_small["loss"]
    image, grads, loss = ctx.step(torch.from_numpy(large).to(gpu), d, t)  # the lists were enlarged: complete now
    ref = oracle.splat_step(W, H, large, depth, target, np.float32)
    assert ctx.stats()["pairs"] == ref["pairs"] > 4 * few
    # (every pixel composites hundreds of these wide Gaussians: a few 1e-5 of fp32 rounding; what is being
    # checked is that no pair is missing, which would show as an error of the size of an alpha)
    assert np.abs(image.cpu().numpy() - ref["image"]).max() < 5e-5
    # a step that reads the loss and does not fit is simply run again with larger lists
    ctx2 = splat.SplatContext(W, H, G, pair_capacity_hint=4000, depth_mode="static")
    ctx2.step(torch.from_numpy(small).to(gpu), d, t)
    image2, _, loss2 = ctx2.step(torch.from_numpy(large).to(gpu), d, t)
    assert np.abs(image2.cpu().numpy() - ref["image"]).max() < 5e-5 and abs(loss2 - ref["loss"]) <= 1e-5 * ref["loss"] + 1e-9
    ctx.close()
    ctx2.close()


def test_the_getters_report_and_settle_an_overflow_too(gpu, oracle, xad):
    """xad_splat_get_stats and xad_splat_get_lists wait for the device, so they are calls that report what a
    step that did not wait has left behind, and enlarge the lists."""
    import torch

    from xyz_autodiff_cuda_amd import splat

    G, W, H = 600, 256, 256
    small, depth = random_scene(G, W, H, seed=5, scale_px=(0.5, 1.0))
    large = small.copy()
    large[2:4] += np.log(30.0)
    target = np.zeros((H, W, 3), np.float32)
    d, t = torch.from_numpy(depth).to(gpu), torch.from_numpy(target).to(gpu)
    ref = oracle.splat_step(W, H, large, depth, target, np.float32)
    for getter in ("stats", "lists"):
        ctx = splat.SplatContext(W, H, G, pair_capacity_hint=4000, depth_mode="static")
        ctx.step(torch.from_numpy(small).to(gpu), d, t)
        ctx.step(torch.from_numpy(large).to(gpu), d, t, want_loss=False)
        with pytest.raises(xad.XadError, match="incomplete"):
            getattr(ctx, getter)()
        # settled: the same step fits now without anybody waiting for it, and the getters answer
        image, _, _ = ctx.step(torch.from_numpy(large).to(gpu), d, t, want_loss=False)
        assert ctx.stats()["pairs"] == ref["pairs"]
        begin, end, ids = ctx.lists()
        assert int((end - begin).sum()) == ref["pairs"] == ids.size
        assert np.abs(image.cpu().numpy() - ref["image"]).max() < 5e-5
        ctx.close()


def test_forward_only_calls_enlarge_the_lists_themselves(gpu, oracle):
    """In the default depth mode a forward call waits for the binning anyway: a scene that has outgrown the lists
    is binned again into larger ones before anything is composited, also when no call ever asks for a loss."""
    import torch

    from xyz_autodiff_cuda_amd import splat

    G, W, H = 600, 256, 256
    small, depth = random_scene(G, W, H, seed=5, scale_px=(0.5, 1.0))
    target = np.zeros((H, W, 3), np.float32)
    d = torch.from_numpy(depth).to(gpu)
    ctx = splat.SplatContext(W, H, G, pair_capacity_hint=4000)
    ctx.forward(torch.from_numpy(small).to(gpu), d)
    for widen in (6.0, 30.0, 90.0):  # each many times the pairs of the one before
        scene = small.copy()
        scene[2:4] += np.log(widen)
        image = ctx.forward(torch.from_numpy(scene).to(gpu), d)
        torch.cuda.synchronize()
        ref = oracle.splat_step(W, H, scene, depth, target, np.float32)
        assert np.abs(image.cpu().numpy() - ref["image"]).max() < 5e-5, widen
        assert ctx.stats()["pairs"] == ref["pairs"], widen
    ctx.close()


def test_gated_adam_holds_the_update_when_told_to(gpu, oracle):
    import torch

    from xyz_autodiff_cuda_amd import splat

    rows, n = 9, 1000
    r = np.random.default_rng(5)
    p0 = r.normal(0, 1, (rows, n)).astype(np.float32)
    g = torch.from_numpy(r.normal(0, 2, (rows, n)).astype(np.float32)).to(gpu)
    gate = torch.zeros(1, dtype=torch.int32, device=gpu)
    held = torch.zeros(1, dtype=torch.int32, device=gpu)
    plain = [torch.from_numpy(p0.copy()).to(gpu), torch.zeros(rows, n, device=gpu), torch.zeros(rows, n, device=gpu)]
    gated = [x.clone() for x in plain]
    splat.adam_step(plain[0], g, plain[1], plain[2], 1e-2, 1)
    splat.adam_step(gated[0], g, gated[1], gated[2], 1e-2, 1, hold_if_nonzero=gate, held_count=held)
    assert all(torch.equal(a, b) for a, b in zip(plain, gated)) and int(held) == 0
    gate.fill_(7)
    before = [x.clone() for x in gated]
    for _ in range(3):
        splat.adam_step(gated[0], g, gated[1], gated[2], 1e-2, 2, hold_if_nonzero=gate, held_count=held)
    assert all(torch.equal(a, b) for a, b in zip(before, gated)) and int(held) == 3
    gate.zero_()
    splat.adam_step(plain[0], g, plain[1], plain[2], 1e-2, 2)
    splat.adam_step(gated[0], g, gated[1], gated[2], 1e-2, 2, hold_if_nonzero=gate, held_count=held)
    assert all(torch.equal(a, b) for a, b in zip(plain, gated)) and int(held) == 3
