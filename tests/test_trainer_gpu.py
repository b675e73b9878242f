"""Trainer front-end on the GPU: initial state, iterations against the oracle,
checkpoints, and the command-line program end to end."""
import os
import re
import subprocess

import numpy as np
import pytest

from xyz_autodiff_cuda_amd import rng, trainer

pytestmark = pytest.mark.gpu

LRS = dict(lr_center=0.05, lr_scale=0.01, lr_rotation=0.02, lr_color=0.03, lr_opacity=0.04)
ROW_LRS = [0.05, 0.05, 0.01, 0.01, 0.02, 0.03, 0.03, 0.03, 0.04]


def _config(**kw):
    base = dict(num_gaussians=300, seed=5, target_image_path="unused", **LRS)
    base.update(kw)
    return trainer.TrainingConfig.defaults(**base)


def test_initial_gaussians_follow_the_reference_distributions(gpu):
    # GaussianCollection::initialize_random (gaussian_parameters.cu:27-66)
    W, H, G = 96, 64, 5000
    t = trainer.Trainer(_config(num_gaussians=G, seed=11), trainer.test_pattern(W, H))
    s = t.state()
    p = s["params"]
    assert t.iteration == 0 and not s["m"].any() and not s["v"].any() and not t.image().any()
    assert 0 <= p[0].min() and p[0].max() < W and abs(p[0].mean() - W / 2) < 2
    assert 0 <= p[1].min() and p[1].max() < H and abs(p[1].mean() - H / 2) < 2
    for row in (2, 3):  # max(1, U(0, 2)): half the mass sits at exactly 1
        assert p[row].min() == 1.0 and p[row].max() < 2.0 and 0.45 < np.mean(p[row] == 1.0) < 0.55
    assert not p[4].any()
    for row in (5, 6, 7):
        assert 0.1 <= p[row].min() and p[row].max() <= 0.2
    assert 0.05 <= p[8].min() and p[8].max() <= 0.1
    assert 0 <= s["depth"].min() and s["depth"].max() < 1
    # a pure function of the seed, and of the documented random streams
    np.testing.assert_array_equal(p[0], rng.host_uniform(G, 11, 0, 0.0, float(W)))
    np.testing.assert_array_equal(p[5], rng.host_uniform(G, 11, 5, 0.1, 0.2))
    other = trainer.Trainer(_config(num_gaussians=G, seed=12), trainer.test_pattern(W, H)).state()["params"]
    assert not np.array_equal(other[0], p[0])
    t.close()


def test_iterations_match_oracle_step_plus_oracle_adam(gpu, oracle):
    """Every iteration is checked on its own: the oracle's step and Adam are applied to the state the
    trainer had before the iteration and compared with the state it has after, so differences do not
    compound."""
    W, H, G = 64, 48, 300
    target = trainer.test_pattern(W, H)
    t = trainer.Trainer(_config(num_gaussians=G), target)
    for it in range(1, 6):
        before = t.state()
        ref = oracle.splat_step(W, H, before["params"], before["depth"], target, np.float32)
        loss = t.run(1)
        assert t.iteration == it
        assert abs(loss - ref["loss"]) <= 1e-5 * ref["loss"]
        np.testing.assert_allclose(t.image(), ref["image"], atol=1e-5)
        p, m, v = before["params"].copy(), before["m"].copy(), before["v"].copy()
        for row in range(9):
            oracle.adam_step(p[row], np.ascontiguousarray(ref["grads"][row]), m[row], v[row], ROW_LRS[row], 0.9, 0.999, 1e-8, it)
        after = t.state()
        np.testing.assert_array_equal(after["depth"], before["depth"])
        for row in range(9):
            # m = beta1 m + (1 - beta1) g: the gradient's tolerance (1e-3 of the row's largest), times 0.1
            g_scale = np.abs(ref["grads"][row]).max()
            assert np.abs(after["m"][row] - m[row]).max() <= 1e-4 * g_scale + 1e-12, (it, row)
            assert np.abs(after["v"][row] - v[row]).max() <= 2e-6 * g_scale ** 2 + 1e-20, (it, row)
            # Adam moves a parameter by about lr whatever the gradient's size, so compare in units of lr.
            # Nearly all elements agree closely; one whose gradient is rounding noise around zero (the
            # rotation of the exactly round Gaussians, a quarter of the initial ones) may step differently.
            err = np.abs(after["params"][row] - p[row]) / ROW_LRS[row]
            typical = np.quantile(err, 0.5 if row == 4 else 0.95)
            assert typical <= 2e-3 and err.max() <= 1.0, (it, row, typical, err.max())
    t.close()


def test_training_fits_the_test_pattern(gpu):
    W = H = 128
    target = trainer.test_pattern(W, H)
    t = trainer.Trainer(_config(num_gaussians=2000, lr_center=0.2, lr_scale=0.02, lr_color=0.02, lr_opacity=0.02), target)
    first = t.run(1)
    last = t.run(299)
    assert t.iteration == 300 and np.isfinite(last) and last < 0.25 * first
    assert np.mean((t.image() - target) ** 2) * 3 * W * H == pytest.approx(last, rel=1e-3)
    t.close()


def _grown_state(W, H, G, target):
    """State of a short run whose Gaussians were then made seven times as wide (about twenty times the pairs)."""
    t = trainer.Trainer(_config(num_gaussians=G), target)
    t.run(2)
    state = t.state()
    t.close()
    state["params"][2:4] += 2.0
    return state


@pytest.mark.parametrize("iterations,loss_every", [(40, 0), (24, 6), (7, 1)])
def test_a_run_whose_lists_outgrow_their_buffers_equals_a_run_with_ample_buffers(gpu, iterations, loss_every):
    """Iterations that do not report a loss never wait for the device, so nobody sees that the tile lists of a
    scene that has grown no longer fit.  No update may use such gradients (the loop of the reference computes all
    gradients, then steps: gaussian_splatting_training.cu:127-160): the updates are withheld on the device, and the
    iterations are run again once the host has looked.  The result must be that of a run whose buffers were ample
    from the start, step numbers included."""
    W = H = 256
    G = 4000
    target = trainer.test_pattern(W, H)
    state = _grown_state(W, H, G, target)

    def run(t):
        losses = []
        if loss_every:
            for _ in range(iterations // loss_every):
                losses.append(t.run(loss_every))
            if iterations % loss_every:
                losses.append(t.run(iterations % loss_every))
        else:
            t.run(iterations, want_loss=False)
            losses.append(t.run(1))
        return losses

    tight = trainer.Trainer(_config(num_gaussians=G), target)
    tight.run(2)  # its buffers are sized for the initial Gaussians, a few pixels across
    tight.set_params(state["params"])
    ample = trainer.Trainer(_config(num_gaussians=G), target)
    ample.set_params(state["params"])
    ample.run(2)  # its buffers are sized for the wide ones
    # the same starting point for both: the wide scene, iteration 2, the moments of `tight`
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "start.ckpt")
        tight.save_checkpoint(path)
        ample.load_checkpoint(path)
    start = tight.iteration
    import warnings

    with warnings.catch_warnings():
        warnings.simplefilter("error")
        loss_tight = run(tight)
        loss_ample = run(ample)
    # (a run that reports every iteration's loss waits every time: the step itself is run again, no iteration is)
    assert (tight.repeated_iterations > 0) == (loss_every != 1) and ample.repeated_iterations == 0
    assert tight.iteration == ample.iteration == start + iterations + (0 if loss_every else 1)
    a, b = tight.state(), ample.state()
    for x, y in zip(loss_tight, loss_ample):
        assert abs(x - y) <= 1e-3 * abs(y), (loss_tight, loss_ample)
    for row in range(9):
        # the two runs differ by the order of the atomic sums only: nearly every element agrees to a small part
        # of a step; an element whose gradient is rounding noise around zero may move the other way in some
        # iteration (Adam moves by about lr whatever the gradient's size)
        off = np.abs(a["params"][row] - b["params"][row]) / ROW_LRS[row]
        assert np.quantile(off, 0.99) <= 0.02 * iterations and off.max() <= 2.0 * iterations, (row, np.quantile(off, 0.99), off.max())
        scale_m = np.abs(b["m"][row]).max() + 1e-20
        assert np.quantile(np.abs(a["m"][row] - b["m"][row]), 0.99) <= 1e-2 * scale_m, row
    np.testing.assert_array_equal(a["depth"], b["depth"])
    # and the tight trainer works normally afterwards, its buffers enlarged
    before = tight.repeated_iterations
    again = tight.run(3)
    assert tight.repeated_iterations == before and np.isfinite(again)
    assert np.mean((tight.image() - target) ** 2) * 3 * W * H == pytest.approx(again, rel=1e-3)
    tight.close()
    ample.close()


def test_a_withheld_update_changes_nothing(gpu, tmp_path):
    """One iteration from a known state with buffers that are too small, nobody asking for the loss: afterwards the
    state is that of one complete iteration with step number 3 (not of a step on truncated lists, not of two
    updates), and the trainer says that it ran one iteration twice."""
    W = H = 256
    G = 4000
    target = trainer.test_pattern(W, H)
    state = _grown_state(W, H, G, target)
    path = str(tmp_path / "start.ckpt")
    t = trainer.Trainer(_config(num_gaussians=G), target)
    t.run(2)
    t.set_params(state["params"])
    t.save_checkpoint(path)
    t.run(1, want_loss=False)
    assert t.iteration == 3 and t.repeated_iterations == 1
    after = t.state()
    fresh = trainer.Trainer(_config(num_gaussians=G), target)
    fresh.set_params(state["params"])
    fresh.run(1)  # waits: sizes its lists for the wide scene
    fresh.load_checkpoint(path)
    fresh.run(1)
    assert fresh.iteration == 3 and fresh.repeated_iterations == 0
    want = fresh.state()
    for row in range(9):
        off = np.abs(after["params"][row] - want["params"][row]) / ROW_LRS[row]
        assert np.quantile(off, 0.99) <= 0.02 and off.max() <= 2.0, (row, np.quantile(off, 0.99), off.max())
        g_scale = np.abs(want["m"][row]).max() + 1e-20
        assert np.abs(after["m"][row] - want["m"][row]).max() <= 1e-3 * g_scale, row
        v_scale = np.abs(want["v"][row]).max() + 1e-30
        assert np.abs(after["v"][row] - want["v"][row]).max() <= 1e-3 * v_scale, row
    t.close()
    fresh.close()


def test_a_checkpoint_with_other_depths_loaded_into_a_trainer_that_has_run(gpu, tmp_path):
    """The renderer keeps the depth order of the depths it saw first (the trainer promises constant depths).  A
    checkpoint or set_params that brings other depths must make it order again: the continuation equals that of
    a fresh trainer that loaded the same file."""
    W, H, G = 96, 64, 500
    target = trainer.test_pattern(W, H)
    path = str(tmp_path / "other.ckpt")
    other = trainer.Trainer(_config(num_gaussians=G, seed=77), target)  # other Gaussians, other depths
    other.run(5, want_loss=False)
    other.save_checkpoint(path)
    used = trainer.Trainer(_config(num_gaussians=G, seed=5), target)
    used.run(5)  # has ordered by its own depths
    used.load_checkpoint(path)
    fresh = trainer.Trainer(_config(num_gaussians=G, seed=5), target)
    fresh.load_checkpoint(path)
    la = used.run(1)
    lb = fresh.run(1)
    assert abs(la - lb) <= 1e-6 * lb
    np.testing.assert_array_equal(used.image(), fresh.image())  # same lists, same order: the same image bit for bit
    used.run(6, want_loss=False)  # iterations that do not report a loss: nothing may have been composited in a stale order
    fresh.run(6, want_loss=False)
    la, lb = used.run(1), fresh.run(1)
    assert abs(la - lb) <= 1e-3 * lb and used.iteration == fresh.iteration == 13
    # and through set_params
    s = other.state()
    used.set_params(depth=s["depth"][::-1].copy())
    fresh2 = trainer.Trainer(_config(num_gaussians=G, seed=5), target)
    fresh2.set_params(params=used.state()["params"], depth=s["depth"][::-1].copy())
    used.run(1)
    fresh2.run(1)
    np.testing.assert_array_equal(used.image(), fresh2.image())
    for t in (other, used, fresh, fresh2):
        t.close()


def test_checkpoint_round_trip_and_resume(gpu, tmp_path, xad):
    W, H, G = 80, 56, 400
    target = trainer.test_pattern(W, H)
    path = str(tmp_path / "state.ckpt")
    a = trainer.Trainer(_config(num_gaussians=G), target)
    a.run(20, want_loss=False)
    a.save_checkpoint(path)
    saved = a.state()
    assert not os.path.exists(path + ".tmp")
    assert os.path.getsize(path) == 72 + 4 * (28 * G) + 4

    b = trainer.Trainer(_config(num_gaussians=G, seed=999), target)  # other initial Gaussians
    b.load_checkpoint(path)
    assert b.iteration == 20
    loaded = b.state()
    for key in ("params", "m", "v", "depth"):
        np.testing.assert_array_equal(loaded[key], saved[key])

    # continuing from the file follows the uninterrupted run (gradient sums are order-dependent in
    # the last bits, so not bit for bit)
    a.run(10, want_loss=False)
    loss_b = b.run(10)
    assert a.iteration == b.iteration == 30
    pa, pb = a.state()["params"], b.state()["params"]
    for row in range(9):
        assert np.abs(pa[row] - pb[row]).max() <= 0.05 * ROW_LRS[row] * 10, row
    assert np.isfinite(loss_b)

    # damaged or mismatching files are refused and leave the trainer as it was
    raw = open(path, "rb").read()
    before = b.state()
    cases = {"flip": raw[:1000] + bytes([raw[1000] ^ 4]) + raw[1001:], "short": raw[:-9], "long": raw + b"\0",
             "magic": b"NOTSPLAT" + raw[8:], "empty": b""}
    for name, data in cases.items():
        bad = str(tmp_path / name)
        open(bad, "wb").write(data)
        with pytest.raises(xad.XadError, match="checkpoint"):
            b.load_checkpoint(bad)
    c = trainer.Trainer(_config(num_gaussians=G + 1), target)
    with pytest.raises(xad.XadError, match="Gaussians"):
        c.load_checkpoint(path)
    d = trainer.Trainer(_config(num_gaussians=G), trainer.test_pattern(W + 16, H))
    with pytest.raises(xad.XadError, match="image"):
        d.load_checkpoint(path)
    with pytest.raises(xad.XadError, match="cannot open"):
        b.load_checkpoint(str(tmp_path / "missing"))
    with pytest.raises(xad.XadError, match="cannot create"):
        b.save_checkpoint(str(tmp_path / "no_dir" / "x"))
    after = b.state()
    assert b.iteration == 30 and all(np.array_equal(before[k], after[k]) for k in before)
    for t in (a, b, c, d):
        t.close()


def test_bad_arguments(gpu, xad):
    target = trainer.test_pattern(32, 32)
    with pytest.raises(xad.XadError, match="Number of Gaussians"):
        trainer.Trainer(_config(num_gaussians=0), target)
    with pytest.raises(xad.XadError, match="learning rates"):
        trainer.Trainer(_config(lr_color=0.0), target)
    t = trainer.Trainer(_config(), target)
    with pytest.raises(xad.XadError, match="negative"):
        t.run(-1)
    assert t.run(0) == 0.0 and t.iteration == 0
    t.close()


def _run_program(args, cwd):
    proc = subprocess.run([trainer.PROGRAM_PATH] + args, cwd=cwd, capture_output=True, text=True, timeout=100)
    return proc.returncode, proc.stdout, proc.stderr


def test_command_line_program(gpu, tmp_path):
    assert os.path.exists(trainer.PROGRAM_PATH), "xad_splat_train is not built"
    target = trainer.test_pattern(96, 64)
    trainer.save_image(tmp_path / "target.png", target)
    args = ["0.2", "0.02", "0.02", "0.02", "0.02", "--target", "target.png", "--num-gaussians", "800", "--max-iterations", "60",
            "--save-interval", "25", "--output-dir", "out", "--checkpoint", "run.ckpt", "--seed", "3", "--image-format", "png"]
    code, out, err = _run_program(args, tmp_path)
    assert code == 0, err
    losses = [float(x) for x in re.findall(r"average Loss: ([0-9.e+-]+)", out)]
    assert len(losses) == 6 and losses[-1] < 0.5 * losses[0]  # iterations 0, 10, .., 50
    names = sorted(os.listdir(tmp_path / "out"))
    assert names == ["iteration_000000.png", "iteration_000025.png", "iteration_000050.png", "iteration_000060.png", "target.png"]
    quantised = np.floor(np.clip(target, 0, 1) * np.float32(255) + np.float32(0.5)) / np.float32(255)
    np.testing.assert_array_equal(trainer.load_image(tmp_path / "out" / "target.png"), quantised.astype(np.float32))
    final = trainer.load_image(tmp_path / "out" / "iteration_000060.png")
    first = trainer.load_image(tmp_path / "out" / "iteration_000000.png")
    assert np.mean((final - target) ** 2) < 0.5 * np.mean((first - target) ** 2)
    assert "Program completed successfully!" in out and "Checkpoint: run.ckpt (iteration 60)" in out

    # without --image-format: the names and the format of the reference (gaussian_splatting_training.cu:106, :124),
    # from a JPEG target; another JPEG decoder reads the snapshots and agrees with the trainer's reader
    from PIL import Image

    trainer.save_image(tmp_path / "target.jpg", target)
    code, out, err = _run_program(args[:5] + ["--target", "target.jpg", "--num-gaussians", "300", "--max-iterations", "10",
                                              "--save-interval", "5", "--output-dir", "jpg_out"], tmp_path)
    assert code == 0, err
    assert "Target image: 96x64" in out
    assert sorted(os.listdir(tmp_path / "jpg_out")) == ["iteration_000000.jpg", "iteration_000005.jpg", "iteration_000010.jpg", "target.jpg"]
    for name in ("iteration_000010.jpg", "target.jpg"):
        theirs = np.asarray(Image.open(tmp_path / "jpg_out" / name).convert("RGB")).astype(np.int32)
        ours = np.rint(trainer.load_image(tmp_path / "jpg_out" / name) * 255).astype(np.int32)
        assert theirs.shape == (64, 96, 3) and np.abs(theirs - ours).max() <= 4
    assert np.abs(np.asarray(Image.open(tmp_path / "jpg_out" / "target.jpg").convert("RGB")) / 255.0 - target).mean() < 0.02

    # resume: continues at iteration 60 and stops at 80
    code, out, err = _run_program(args[:5] + ["--target", "target.png", "--num-gaussians", "800", "--max-iterations", "80", "--no-save-images",
                                              "--resume", "run.ckpt", "--checkpoint", "run2.ckpt"], tmp_path)
    assert code == 0, err
    assert "Resumed from run.ckpt at iteration 60" in out and "Checkpoint: run2.ckpt (iteration 80)" in out
    resumed = [float(x) for x in re.findall(r"average Loss: ([0-9.e+-]+)", out)]
    assert len(resumed) == 2 and resumed[0] < losses[-1] * 1.2

    # a missing image falls back to the 256 x 256 test pattern (gaussian_splatting_training.cu:47-50)
    code, out, err = _run_program(["0.01"] * 5 + ["--target", "nope.png", "--max-iterations", "2", "--no-save-images", "--num-gaussians", "100"], tmp_path)
    assert code == 0 and "creating test image instead" in out and "Target image: 256x256" in out

    # failures: usage and the reference's message, non-zero exit
    code, out, err = _run_program(["0.01", "0.01"], tmp_path)
    assert code != 0 and "Insufficient arguments" in err and "Usage:" in err
    code, out, err = _run_program(["--help"], tmp_path)
    assert code == 0 and "Usage:" in out
