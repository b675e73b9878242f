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


def test_lists_that_outgrow_their_buffers_during_a_run_are_reported_and_the_run_goes_on(gpu):
    """Iterations that do not report a loss never wait for the device, so a run whose Gaussians have grown
    outgrows the tile lists' buffers unnoticed.  The run must finish, say so once its last iteration reads the
    device's report, and work normally afterwards with the enlarged buffers."""
    W = H = 256
    target = trainer.test_pattern(W, H)
    t = trainer.Trainer(_config(num_gaussians=4000), target)
    t.run(2)  # sizes the buffers for the initial Gaussians (a few pixels across)
    params = t.state()["params"]
    params[2:4] += 2.0  # seven times as wide: about twenty times the pairs
    t.set_params(params)
    with pytest.warns(RuntimeWarning, match="outgrown their buffers"):
        loss = t.run(8)
    assert t.iteration == 10 and np.isfinite(loss)
    state = t.state()
    assert all(np.isfinite(v).all() for v in state.values() if isinstance(v, np.ndarray))
    # the report has been taken and the buffers fit again: a rendering with every contribution
    import warnings

    with warnings.catch_warnings():
        warnings.simplefilter("error")
        again = t.run(1)
    assert np.isfinite(again) and np.mean((t.image() - target) ** 2) * 3 * W * H == pytest.approx(again, rel=1e-3)
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
            "--save-interval", "25", "--output-dir", "out", "--checkpoint", "run.ckpt", "--seed", "3"]
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
