"""The depth order computed on the GPU (csrc/splat_sort.hip, through xad_depth_order_f32) against a stable
host sort: integer work, so bit for bit.

Policy under test: ascending depth, equal depths in index order, -0.0 and +0.0 one depth; NaNs by bit
pattern (sign bit set: before everything; clear: after everything).  For data without NaNs that is exactly
numpy's stable argsort of the floats, which is what the expectations use (nothing of the kernel's key
mapping is repeated here); for NaNs the expectation sorts the three groups separately.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _expected_order(depth):
    nan = np.isnan(depth)
    if not nan.any():
        return np.argsort(depth, kind="stable")
    bits = depth.view(np.uint32)
    negative_nan = np.flatnonzero(nan & ((bits >> 31) == 1))
    positive_nan = np.flatnonzero(nan & ((bits >> 31) == 0))
    rest = np.flatnonzero(~nan)
    # a NaN with the sign bit set is "more negative" the larger its payload; one without, larger the larger
    first = negative_nan[np.argsort(-(bits[negative_nan] & 0x7FFFFFFF).astype(np.int64), kind="stable")]
    last = positive_nan[np.argsort(bits[positive_nan], kind="stable")]
    return np.concatenate([first, rest[np.argsort(depth[rest], kind="stable")], last])


def _check(gpu, depth):
    import torch

    from xyz_autodiff_cuda_amd import splat

    depth = np.ascontiguousarray(depth, dtype=np.float32)
    order, rank = splat.depth_order(torch.from_numpy(depth).to(gpu))
    order = order.cpu().numpy().view(np.uint32).astype(np.int64)
    rank = rank.cpu().numpy().view(np.uint32).astype(np.int64)
    want = _expected_order(depth)
    np.testing.assert_array_equal(order, want)
    inverse = np.empty_like(want)
    inverse[want] = np.arange(want.size)
    np.testing.assert_array_equal(rank, inverse)


# (up to 4096 keys one block sorts alone, with 2 or 4 keys per lane; above, tiles of 4096 keys)
@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 511, 512, 513, 1024, 1025, 2047, 2048, 2049, 4096, 4097, 8192, 8193, 10_000, 12_287,
                               12_288, 12_289, 16_384, 200_000, 1_000_003])
def test_uniform_depths(gpu, n):
    _check(gpu, np.random.default_rng(n).uniform(0.0, 1.0, n))


@pytest.mark.parametrize("n", [5, 2048, 9000, 50_000, 300_001])
def test_ties_keep_index_order(gpu, n):
    r = np.random.default_rng(n)
    _check(gpu, r.integers(0, 4, n).astype(np.float32) * 0.25)  # four distinct depths
    _check(gpu, np.full(n, 0.5, np.float32))                    # one
    _check(gpu, np.round(r.uniform(0, 1, n), 2))                # a hundred


@pytest.mark.parametrize("n", [9, 3000, 70_000])
def test_signs_zeros_infinities_and_denormals(gpu, n):
    r = np.random.default_rng(n)
    d = r.normal(0.0, 1e3, n).astype(np.float32)
    d[r.integers(0, n, n // 7 + 1)] = 0.0
    d[r.integers(0, n, n // 7 + 1)] = -0.0
    d[r.integers(0, n, n // 9 + 1)] = np.inf
    d[r.integers(0, n, n // 9 + 1)] = -np.inf
    d[r.integers(0, n, n // 9 + 1)] = 1e-42   # denormal
    d[r.integers(0, n, n // 9 + 1)] = -1e-42
    d[r.integers(0, n, n // 9 + 1)] = np.float32(3.4e38)
    _check(gpu, d)
    # the two zeros alternate: one depth, so the indices come out in order
    z = np.zeros(n, np.float32)
    z[::2] = -0.0
    _check(gpu, z)


def test_nans_sort_by_their_bits(gpu):
    r = np.random.default_rng(1)
    n = 5000
    d = r.normal(0.0, 1.0, n).astype(np.float32)
    bits = d.view(np.uint32)
    where = r.permutation(n)[:400]
    bits[where[:100]] = 0x7FC00000                                                # the usual quiet NaN
    bits[where[100:200]] = 0xFFC00000                                             # with the sign bit
    bits[where[200:300]] = 0x7F800001 + r.integers(0, 1 << 22, 100).astype(np.uint32)  # other payloads
    bits[where[300:400]] = 0xFF800001 + r.integers(0, 1 << 22, 100).astype(np.uint32)
    _check(gpu, d)


@pytest.mark.parametrize("n", [700, 4097, 11_111, 123_457])
def test_sorted_and_reversed_inputs(gpu, n):
    d = np.linspace(-1.0, 1.0, n).astype(np.float32)
    _check(gpu, d)
    _check(gpu, d[::-1])


def test_every_byte_position_decides_somewhere(gpu):
    """Keys that differ in one byte only, for each of the four bytes a pass looks at."""
    base = np.uint32(0x3F000000)
    for n in (20_000, 6_000):
        for byte in range(4):
            r = np.random.default_rng(byte)
            bits = (base + (r.integers(0, 256 if byte < 3 else 64, n).astype(np.uint32) << np.uint32(8 * byte))).astype(np.uint32)
            _check(gpu, bits.view(np.float32))


def test_calls_in_a_row_share_nothing(gpu):
    """The workspace of a context is left clean by every sort: a large sort, a small one, a large one."""
    import torch

    from tests._scenes import random_scene
    from xyz_autodiff_cuda_amd import splat

    G, W, H = 30_000, 256, 256
    params, depth = random_scene(G, W, H, seed=3, scale_px=(1.0, 3.0))
    p = torch.from_numpy(params).to(gpu)
    ctx = splat.SplatContext(W, H, G, depth_mode="every_step")
    images = []
    for k in range(4):
        d = np.roll(depth, 977 * k).astype(np.float32)
        images.append((d, ctx.forward(p, torch.from_numpy(d).to(gpu)).clone()))
    torch.cuda.synchronize()
    fresh = splat.SplatContext(W, H, G)
    for d, image in images:
        want = fresh.forward(p, torch.from_numpy(d).to(gpu))
        torch.cuda.synchronize()
        assert torch.equal(image, want)
    ctx.close()
    fresh.close()
