#!/usr/bin/env python3
"""Benchmark of the per-thread forward+backward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the forward+backward kernels over the whole batch of
synthetic problems (N = 64 Mi, inputs already resident in HBM).  Prints one JSON
line: throughput in evaluations per second, the HBM roofline of the kernel
(algorithmic bytes = 52 B per evaluation) and a CPU baseline measured in the
same run on the host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
# HBM bytes per evaluation of the chain kernel, from FETCH_SIZE / WRITE_SIZE counter
# passes scaled by a copy of known size (profiles/chain_single_kernel_hbm_traffic.md)
MEASURED_TRAFFIC_BYTES_PER_EVAL = 52.000
TRAFFIC_SOURCE = {"profile": "profiles/chain_single_kernel_hbm_traffic.md", "bytes_per_eval": MEASURED_TRAFFIC_BYTES_PER_EVAL,
                  "note": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of `bench.py --counter-probe chain`, each scaled by a copy of "
                          "known size; a constant from that profile, not a reading of this run"}
N_FULL = 64 * 1024 * 1024
# Atomic requests that reach L2 in one iteration of the splatting step, from counter passes over
# `bench.py --counter-probe splat` / `--counter-probe splat4` (TCC_ATOMIC_sum per kernel, summed over the
# iteration's kernels); constants from those profiles, not readings of this run.
ATOMIC_TRAFFIC = {
    "config4_10k_512": {"l2_atomic_requests_measured": 132_498, "pairs_in_that_run": 129_843,
                        "source": "profiles/splat_10k_512_kernel_counters.md (TCC_ATOMIC_sum: render_backward_kernel 132 490, scans 8)"},
    "config5_200k_2048": {"l2_atomic_requests_measured": 3_666_035, "pairs_in_that_run": 5_500_959,
                          "source": "profiles/splat_200k_2048_kernel_counters.md (TCC_ATOMIC_sum: render_backward_kernel 3 665 877, scans 158)"},
}


def cpu_baseline(host_inputs, budget_s=12.0):
    """Times the CPU oracle (the reference's formulas restated in C, OpenMP over
    all host cores the box gives us) on a bounded sample of the same workload."""
    import numpy as np

    from tests import _oracle

    oracle = _oracle.load()
    cores = min(oracle.max_threads(), int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or oracle.max_threads())
    oracle.set_threads(cores)
    n = host_inputs[0].size
    oracle.chain_soa(host_inputs, np.float32)  # warm-up
    reps, t0 = 0, time.perf_counter()
    while True:
        oracle.chain_soa(host_inputs, np.float32)
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s:
            break
    return {
        "value": n * reps / dt,
        "unit": "evals/s",
        "cores": cores,
        "kind": "port",
        "sample": "first %d problems of the workload, %d passes, %.1f s" % (n, reps, dt),
    }


def chain_parity(host_inputs, got):
    """The first problems of the workload against the fp64 oracle: the fraction meeting the flat figures
    (value within 1e-5, all six gradients within 1e-4; the testers' min(abs, rel)) and the largest error
    in units of the parity tests' tolerance, 1e-5 x max(1, cond(Sigma))."""
    import numpy as np

    from tests import _oracle
    from tests._metrics import abs_or_rel, covariance_condition

    ref = _oracle.load().chain_soa(host_inputs, np.float64)
    e = abs_or_rel(got, ref)
    kappa = np.maximum(1.0, covariance_condition(host_inputs[0], host_inputs[1]))
    return {"problems": int(host_inputs[0].size), "value_within_1e-5": float((e[0] <= 1e-5).mean()),
            "all_gradients_within_1e-4": float((e[1:] <= 1e-4).all(axis=0).mean()),
            "worst_error_over_1e-5_cond": float((e / kappa).max() / 1e-5)}


def host_templates(host_inputs):
    """The library's own templates compiled for the host cores (N = 1e6)."""
    import numpy as np

    from xyz_autodiff_cuda_amd import chain

    threads = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1)
    sample = [a[:1_000_000] for a in host_inputs]
    chain.host_forward_backward(sample, np.float32, threads)
    best = float("inf")
    for _ in range(10):
        t0 = time.perf_counter()
        chain.host_forward_backward(sample, np.float32, threads)
        best = min(best, time.perf_counter() - t0)
    n = sample[0].size
    return {"value": n / best, "unit": "evals/s", "threads": threads, "n": n, "GBps": 52.0 * n / best / 1e9}


def accumulate_report(ins, seed, with_oracle):
    """Config 3: 16 Mi threads add their six gradients into P Zipf(1.1)-distributed
    slots.  Times the naive per-thread global atomics against the staged path and
    checks both against the oracle's fp64 sums."""
    import numpy as np
    import torch

    import instruments
    from xyz_autodiff_cuda_amd import accumulate

    dev = ins[0].device
    n = min(ins[0].numel(), 16 * 1024 * 1024)
    sub = [t[:n] for t in ins]
    host = [t.cpu().numpy() for t in sub] if with_oracle else None
    out = {"n": n, "bytes_per_thread": accumulate.BYTES_PER_THREAD, "slots": {},
           "lds_atomic_cycles_per_wavefront_instruction": instruments.lds_atomic_cycles()}
    for num_slots in (64, 4096, 262144):
        slot = torch.empty(n, dtype=torch.int32, device=dev)
        accumulate.zipf_(slot, seed, 10, num_slots, 1.1)
        grads = torch.zeros(num_slots, 6, dtype=torch.float32, device=dev)
        entry = {}
        ref = None
        if with_oracle:
            from tests import _oracle

            ref = _oracle.load().accumulate_chain(host, slot.cpu().numpy(), num_slots, chain_in_double=True)
        for name, reps in (("auto", 10), ("wave_lds", 5), ("lds_f32", 5), ("global_atomics", 1)):
            # `reps` launches back to back between one pair of events (the sums simply keep growing), after a
            # warm-up launch; then one launch from zero, which is the one checked below
            grads.zero_()
            if reps > 1:
                accumulate.accumulate_chain_gradients(sub, slot, grads, name)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(reps):
                accumulate.accumulate_chain_gradients(sub, slot, grads, name)
            b.record()
            torch.cuda.synchronize()
            ms = a.elapsed_time(b) / reps
            if reps > 1:
                grads.zero_()
                accumulate.accumulate_chain_gradients(sub, slot, grads, name)
                torch.cuda.synchronize()
            item = {"ms": ms, "GBps": (accumulate.BYTES_PER_THREAD * n + 24.0 * num_slots) / ms / 1e6}
            if ref is not None:
                got = grads.cpu().numpy().astype(np.float64)
                item["max_err_over_mass"] = float((np.abs(got - ref[0]) / (ref[1] + 1e-30))[ref[1] > 1e-3].max())
                item["sums_within_1e-4_of_their_mass"] = float((np.abs(got - ref[0]) <= 1e-4 * ref[1])[ref[1] > 0].mean())
            entry[name] = item
        entry["speedup_vs_global_atomics"] = entry["global_atomics"]["ms"] / entry["auto"]["ms"]
        out["slots"][str(num_slots)] = entry
    return out


def trainer_report():
    """The trainer front-end at the size of config 5: iterations/s of xad_trainer_run (splatting
    step + Adam per iteration, state resident on the device) on a synthetic target."""
    import time

    from xyz_autodiff_cuda_amd import splat, trainer

    G, W, H = 200_000, 2048, 2048
    target = splat.synthetic_target(G, W, H, seed=77, scale_px=(0.5, 40.0), noise=0.02).cpu().numpy()
    config = trainer.TrainingConfig.defaults(num_gaussians=G, seed=1, target_image_path="synthetic")
    t = trainer.Trainer(config, target)
    first = t.run(5)
    repeated_before = t.repeated_iterations
    t0 = time.perf_counter()
    last = t.run(50)
    dt = time.perf_counter() - t0
    repeated = t.repeated_iterations - repeated_before
    # a second stretch, for a figure without the repeats of the first (the lists have been enlarged by then)
    t0 = time.perf_counter()
    t.run(50, want_loss=False)
    dt2 = time.perf_counter() - t0
    repeated2 = t.repeated_iterations - repeated_before - repeated
    t.close()
    # ms_per_iter divides by the 50 iterations that count; the timed region also ran `repeated_iterations` of them twice
    # (their first run found the tile lists too small and changed nothing: the update is withheld on the device)
    return {"gaussians": G, "image": [W, H], "iterations": 50, "iters_per_s": 50 / dt, "ms_per_iter": dt / 50 * 1e3,
            "repeated_iterations": int(repeated), "ms_per_iteration_run": dt / (50 + repeated) * 1e3,
            "next_50": {"ms_per_iter": dt2 / 50 * 1e3, "repeated_iterations": int(repeated2)},
            "loss_after_5": first, "loss_after_55": last}


def linreg_report(with_oracle):
    """Least-squares example (fp64, four parameters shared by all samples): gradient
    sums over 16 Mi samples per strategy, and the reference's training run (100 000
    samples, batch 8192, 10 000 steps) entirely on the device."""
    import time

    import numpy as np
    import torch

    from xyz_autodiff_cuda_amd import linreg

    dev = torch.device("cuda:0")
    n = 16 * 1024 * 1024
    x1, x2, y = (torch.from_numpy(a).to(dev) for a in linreg.synthetic_data(n, seed=1))
    params = torch.tensor([0.4, 1.3, -0.2, 0.1], dtype=torch.float64, device=dev)
    out = {"n": n, "bytes_per_sample": linreg.BYTES_PER_SAMPLE, "gradient": {}}
    want = None
    if with_oracle:
        from tests import _oracle

        t0 = time.perf_counter()
        want = _oracle.load().linreg_gradient(x1.cpu().numpy(), x2.cpu().numpy(), y.cpu().numpy(), params.cpu().numpy())
        out["cpu_oracle_ms"] = (time.perf_counter() - t0) * 1e3
    for name, reps in (("wave_lds", 10), ("lds_leaves", 3), ("global_atomics", 1)):
        times = []
        for _ in range(reps + 1):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            got = linreg.batch_gradient(x1, x2, y, params, strategy=name)
            b.record()
            torch.cuda.synchronize()
            times.append(a.elapsed_time(b))
        ms = sorted(times[1:])[len(times[1:]) // 2]
        item = {"ms": ms, "GBps": linreg.BYTES_PER_SAMPLE * n / ms / 1e6}
        if want is not None:
            item["max_rel_err"] = float(np.max(np.abs(got.cpu().numpy() - want) / np.abs(want)))
        out["gradient"][name] = item
    out["gradient"]["speedup_vs_global_atomics"] = out["gradient"]["global_atomics"]["ms"] / out["gradient"]["wave_lds"]["ms"]

    total, batch, epochs = 100_000, 8192, 10_000
    sx1, sx2, sy = (torch.from_numpy(a).to(dev) for a in linreg.synthetic_data(total, seed=0))
    p = torch.tensor(linreg.INITIAL_PARAMS, dtype=torch.float64, device=dev)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    linreg.sgd(sx1, sx2, sy, p, batch, epochs, seed=1)
    dt = time.perf_counter() - t0
    out["sgd"] = {"samples": total, "batch": batch, "steps": epochs, "seconds": dt, "steps_per_s": epochs / dt,
                  "final_params": p.cpu().tolist(), "true_params": list(linreg.TRUE_PARAMS)}
    return out


def splat_report(with_oracle, iters=30):
    """Configs 4 and 5: one training iteration = forward + backward + Adam (lr 1e-2).
    Reports iterations/s, the per-kernel time split, pair statistics, and the CPU
    oracle's time for the same iteration on the host cores."""
    import numpy as np
    import torch

    from xyz_autodiff_cuda_amd import splat

    dev = torch.device("cuda:0")
    out = {}
    for name, G, W, H, scale in (("config4_10k_512", 10_000, 512, 512, (1.0, 20.0)),
                                 ("config5_200k_2048", 200_000, 2048, 2048, (0.5, 40.0))):
        target = splat.synthetic_target(G, W, H, seed=77, scale_px=scale, noise=0.02)
        params, depth = splat.synthetic_scene(G, W, H, seed=1234, scale_px=scale)
        start_params = params.clone()
        # depths never change in this loop: say so, and an iteration never waits for the device
        ctx = splat.SplatContext(W, H, G, pair_capacity_hint=9_000_000 if G > 50_000 else 0, depth_mode="static")
        m, v = torch.zeros_like(params), torch.zeros_like(params)
        image = torch.empty(H, W, 3, device=dev)
        grads = torch.empty(9, G, device=dev)
        # no update on gradients from lists that have outgrown their buffers: decided on the device, counted here
        gate, held = ctx.overflow_word(), torch.zeros(1, dtype=torch.int32, device=dev)
        _, _, first_loss = ctx.step(params, depth, target, image, grads)
        first_grads = grads.cpu().numpy().astype(np.float64) if with_oracle else None
        first_image = image.cpu().numpy() if with_oracle else None
        first_pairs = ctx.stats()["pairs"]
        for it in range(1, 4):
            ctx.step(params, depth, target, image, grads, want_loss=False)
            splat.adam_step(params, grads, m, v, 1e-2, it, hold_if_nonzero=gate, held_count=held)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for it in range(4, 4 + iters):
            ctx.step(params, depth, target, image, grads, want_loss=False)
            splat.adam_step(params, grads, m, v, 1e-2, it, hold_if_nonzero=gate, held_count=held)
        torch.cuda.synchronize()
        per_iter = (time.perf_counter() - t0) / iters
        # the same iterations with the depth order recomputed by every step (what a caller whose depths change pays)
        ctx.set_depth_mode("every_step")
        ctx.step(params, depth, target, image, grads, want_loss=False)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for it in range(4 + iters, 4 + 2 * iters):
            ctx.step(params, depth, target, image, grads, want_loss=False)
            splat.adam_step(params, grads, m, v, 1e-2, it, hold_if_nonzero=gate, held_count=held)
        torch.cuda.synchronize()
        per_iter_every_step = (time.perf_counter() - t0) / iters
        withheld_updates = int(held)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for it in range(10):
            splat.adam_step(params, grads, m, v, 1e-2, 100 + it)
        b.record()
        torch.cuda.synchronize()
        adam_ms = a.elapsed_time(b) / 10
        ctx.set_profiling(True)  # (still in the every_step mode: the split has its sort stage)
        acc = None
        for _ in range(5):
            ctx.step(params, depth, target, image, grads, want_loss=False)
            ms = ctx.stats()["stage_ms"]
            acc = ms if acc is None else {k: acc[k] + ms[k] for k in ms}
        ctx.set_profiling(False)
        ctx.set_depth_mode("static")
        _, _, last_loss = ctx.step(params, depth, target, image, grads)
        stats = ctx.stats(longest_list=True)
        tiles = ((W + 15) // 16) * ((H + 15) // 16)
        entry = {
            "gaussians": G, "image": [W, H], "iters_per_s": 1.0 / per_iter, "ms_per_iter": per_iter * 1e3,
            "iters_per_s_every_step": 1.0 / per_iter_every_step, "ms_per_iter_every_step": per_iter_every_step * 1e3,
            "every_step_over_static": per_iter_every_step / per_iter,
            "updates_withheld_in_timed_loops": withheld_updates,
            "stage_ms": {**{k: v / 5 for k, v in acc.items()}, "adam": adam_ms},
            "pairs": stats["pairs"], "mean_list": stats["pairs"] / tiles, "longest_list": stats["longest_list"],
            "global_atomics_per_iter": {**ATOMIC_TRAFFIC.get(name, {}),
                                        "values_added_if_one_atomic_per_pair_and_field": stats["pairs"] * 9 + tiles,
                                        "values_added_if_one_atomic_per_pixel_pair_and_field": int(stats["pairs"]) * 256 * 9},
            "loss_first": first_loss, "loss_after_%d_iters" % (2 * iters + 10): last_loss,
        }
        if with_oracle:
            from tests import _oracle

            oracle = _oracle.load()
            hp, hd, ht = start_params.cpu().numpy(), depth.cpu().numpy(), target.cpu().numpy()
            hp0 = hp.copy()
            t0 = time.perf_counter()
            ref = oracle.splat_step(W, H, hp, hd, ht, np.float32)
            cpu_s = time.perf_counter() - t0
            hm, hv = np.zeros_like(hp), np.zeros_like(hp)
            t0 = time.perf_counter()
            oracle.adam_step(hp, ref["grads"], hm, hv, 1e-2, 0.9, 0.999, 1e-8, 1)
            cpu_s += time.perf_counter() - t0
            entry["cpu_oracle"] = {"s_per_iter": cpu_s, "iters_per_s": 1.0 / cpu_s, "cores": oracle.max_threads(),
                                   "stage_s": ref["seconds"], "sample": "one full iteration"}
            entry["speedup_vs_cpu"] = cpu_s / per_iter
            # The library's own templates on the host cores (xad_host_splat_step_f32: the per-pair graph of
            # operation nodes, tiles dealt to threads), one full iteration with Adam in numpy.
            cores = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or os.cpu_count()
            splat.host_step(hp0[:, :64], hd[:64], ht[:16, :16], 16, 16, num_threads=cores)  # loads and warms the library
            t0 = time.perf_counter()
            host = splat.host_step(hp0, hd, ht, W, H, num_threads=cores)
            hm2 = 0.1 * host["grads"]
            hv2 = 0.001 * host["grads"] ** 2
            stepped = hp0 - 1e-2 * (hm2 / 0.1) / (np.sqrt(hv2 / 0.001) + 1e-8)
            host_s = time.perf_counter() - t0
            entry["host_templates"] = {"s_per_iter": host_s, "iters_per_s": 1.0 / host_s, "cores": cores, "sample": "one full iteration",
                                       "loss_matches_gpu": bool(abs(host["loss"] - first_loss) <= 1e-5 * first_loss),
                                       "pairs": int(host["pairs"]),
                                       "largest_parameter_change": float(np.abs(stepped - hp0).max())}
            entry["speedup_vs_host_templates"] = host_s / per_iter
            entry["first_loss_matches_cpu"] = abs(first_loss - ref["loss"]) <= 1e-5 * ref["loss"]
            # Gradients of the first step against the fp64 oracle (binned with the fp32 projection's tile
            # rectangles), every one of the 9 x G against  1e-4 x mass + bound:  mass = the sum of the
            # magnitudes of the per-pixel terms behind it, bound = the oracle's first-order bound on the
            # distance of an fp32 evaluation of the step from the fp64 one (oracle/oracle_splat.inc).  The
            # same criterion as tests/test_full_size_gpu.py, on the merits of every Gaussian.
            ref64 = oracle.splat_step(W, H, hp0, hd, ht, np.float64, rects_in=ref["rects"], want_bounds=True)
            err = np.abs(first_grads - ref64["grads"])
            excess = err / (1e-4 * ref64["grad_mass"] + ref64["grad_bound"] + 1e-30)
            live = np.abs(ref64["grads"]).max(axis=0) > 0
            image_excess = np.abs(first_image.astype(np.float64) - ref64["image"]) / (1e-5 + ref64["image_bound"])
            entry["first_step_vs_fp64_oracle"] = {
                "pairs": {"gpu": int(first_pairs), "fp32_oracle": int(ref["pairs"]), "fp64_oracle_on_fp32_rectangles": int(ref64["pairs"])},
                "gaussians_within_1e-4_mass_plus_bound": float((excess <= 1.0).all(axis=0).mean()),
                "worst_error_over_that_tolerance": float(excess.max()),
                "median_tolerance_over_gradient": float(np.median(((1e-4 * ref64["grad_mass"] + ref64["grad_bound"]) / (np.abs(ref64["grads"]) + 1e-300))[:, live])),
                # the flat figures: all nine gradients of a Gaussian within 1e-4 relative; pixels within 1e-5
                "gaussians_with_all_gradients_within_1e-4_relative": float((err <= 1e-4 * np.abs(ref64["grads"])).all(axis=0)[live].mean()),
                "fp32_oracle_same_figure": float((np.abs(ref["grads"].astype(np.float64) - ref64["grads"]) <= 1e-4 * np.abs(ref64["grads"])).all(axis=0)[live].mean()),
                "pixels_within_1e-5": float((np.abs(first_image - ref64["image"]) <= 1e-5).mean()),
                "worst_pixel_error_over_1e-5_plus_bound": float(image_excess.max()),
                "match": bool(first_pairs == ref["pairs"] and (excess <= 1.0).all() and image_excess.max() <= 1.0),
            }
        ctx.close()
        out[name] = entry
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--n", type=int, default=N_FULL, help="problems per step (default: the full 64 Mi)")
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs (profiling runs)")
    ap.add_argument("--counter-probe", choices=("chain", "accumulate", "splat", "splat4"), default=None,
                    help="launch a few kernels of one leg and exit, for rocprofv3 --pmc runs: chain = a 256 Mi-float "
                         "copy then three chain passes; accumulate = naive and staged accumulation at 64, 4096 and 262144 slots; "
                         "splat = two iterations of the 200k-Gaussian step; splat4 = two of the 10k-Gaussian step")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (got --gpus %d)" % args.gpus)

    import numpy as np
    import torch

    import instruments
    from xyz_autodiff_cuda_amd import chain, rng

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    dev = torch.device("cuda:0")
    n = args.n
    ins = [torch.empty(n, dtype=torch.float32, device=dev) for _ in range(6)]
    outs = [torch.empty(n, dtype=torch.float32, device=dev) for _ in range(7)]
    rng.chain_inputs_(ins, args.seed)
    torch.cuda.synchronize()

    if args.counter_probe == "chain":
        # known traffic first (1 GiB read + 1 GiB written), then the kernel under study
        instruments.stream_copy(torch.cat(ins[:4]), torch.cat(outs[:4]))
        for _ in range(3):
            chain.forward_backward(ins, outs)
        torch.cuda.synchronize()
        print(json.dumps({"counter_probe": "chain", "n": n, "copy_floats": 4 * n}))
        return
    if args.counter_probe == "accumulate":
        from xyz_autodiff_cuda_amd import accumulate

        m = 16 * 1024 * 1024
        sub = [t[:m] for t in ins]
        for num_slots in (64, 4096, 262144):
            slot = torch.empty(m, dtype=torch.int32, device=dev)
            accumulate.zipf_(slot, args.seed, 10, num_slots, 1.1)
            grads = torch.zeros(num_slots, 6, dtype=torch.float32, device=dev)
            for name in ("global_atomics", "auto", "wave_lds"):
                accumulate.accumulate_chain_gradients(sub, slot, grads, name)
        torch.cuda.synchronize()
        print(json.dumps({"counter_probe": "accumulate", "n": m, "order": "per slots in (64, 4096, 262144): global_atomics, auto, wave_lds"}))
        return
    if args.counter_probe in ("splat", "splat4"):
        from xyz_autodiff_cuda_amd import splat

        del ins, outs
        G, W, H, scale = (200_000, 2048, 2048, (0.5, 40.0)) if args.counter_probe == "splat" else (10_000, 512, 512, (1.0, 20.0))
        target = splat.synthetic_target(G, W, H, seed=77, scale_px=scale, noise=0.02)
        params, depth = splat.synthetic_scene(G, W, H, seed=args.seed, scale_px=scale)
        ctx = splat.SplatContext(W, H, G, pair_capacity_hint=9_000_000 if G > 50_000 else 0)
        for _ in range(2):
            ctx.step(params, depth, target, want_loss=False)
        torch.cuda.synchronize()
        print(json.dumps({"counter_probe": args.counter_probe, "pairs": ctx.stats()["pairs"]}))
        return

    for _ in range(args.warmup):
        chain.forward_backward(ins, outs)
    torch.cuda.synchronize()

    starts = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        starts[k].record()
        chain.forward_backward(ins, outs)
        stops[k].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    kernel_ms = [a.elapsed_time(b) for a, b in zip(starts, stops)]
    avg_kernel_s = sum(kernel_ms) / len(kernel_ms) / 1e3
    algorithmic_bytes = float(chain.BYTES_PER_EVAL) * n
    achieved = algorithmic_bytes / avg_kernel_s / 1e9

    finite = all(bool(torch.isfinite(o).all()) for o in outs)

    # the alternative lane-to-address mapping, for the record (not part of `value`)
    alt = {}
    for lanes in (1, 4):
        instruments.chain_with_layout(ins, outs, lanes)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(10):
            instruments.chain_with_layout(ins, outs, lanes)
        b.record()
        torch.cuda.synchronize()
        alt["problems_per_lane=%d" % lanes] = algorithmic_bytes / (a.elapsed_time(b) / 10 / 1e3) / 1e9

    # the store policy of the default kernel, measured again: alternating rounds of ten launches each
    policy_ms = {name: [] for name in instruments.STORE_POLICIES}
    for _ in range(3):
        for name in instruments.STORE_POLICIES:
            instruments.chain_with_store_policy(ins, outs, name)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(10):
                instruments.chain_with_store_policy(ins, outs, name)
            b.record()
            torch.cuda.synchronize()
            policy_ms[name].append(a.elapsed_time(b) / 10)
    store_policy = {name: algorithmic_bytes / (sorted(v)[1] / 1e3) / 1e9 for name, v in policy_ms.items()}

    # what this memory system gives a plain copy in the same process on the same day: one stream in, one out,
    # 1 GiB each way (far beyond the caches), the median of three rounds of ten launches
    copy_src = torch.cat(ins[:4]) if n * 4 <= (1 << 28) else torch.cat([t[: (1 << 26)] for t in ins[:4]])
    copy_dst = torch.empty_like(copy_src)
    copy_rates = {}
    for variant in ("chain_pattern_4B_x1_non_temporal",) + instruments.COPY_VARIANTS:
        def launch():
            if variant.startswith("chain_pattern"):
                instruments.stream_copy(copy_src, copy_dst)
            else:
                instruments.copy_variant(copy_src, copy_dst, variant)
        ms = []
        for _ in range(3):
            launch()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(10):
                launch()
            b.record()
            torch.cuda.synchronize()
            ms.append(a.elapsed_time(b) / 10)
        copy_rates[variant] = 2.0 * copy_src.numel() * 4 / (sorted(ms)[1] / 1e3) / 1e9
    copy_ceiling = max(copy_rates.values())
    del copy_src, copy_dst

    record = {
        "metric": "per-thread fwd+bwd evals/sec",
        "value": n * args.steps / wall,
        "unit": "evals/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "config 2: per-thread forward+backward chain, N=%d, fp32, SoA (6 in, 7 out), seed %d" % (n, args.seed),
            "n": n,
            "bytes_per_eval": chain.BYTES_PER_EVAL,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "copy_ceiling_GBps": copy_ceiling,
            "copy_GBps_by_shape": copy_rates,
            "frac_of_copy_ceiling": achieved / copy_ceiling,
            "traffic": MEASURED_TRAFFIC_BYTES_PER_EVAL * n,
            "traffic_source": TRAFFIC_SOURCE,
            "kernel": "chain_single_kernel",
            "kernel_ms_avg": avg_kernel_s * 1e3,
            "kernel_ms_min": min(kernel_ms),
        },
        "outputs_finite": finite,
        "mapping_GBps": alt,
        "store_policy_GBps": store_policy,
        "kernel_resources": instruments.chain_kernel_resources(),
    }
    record["accumulate"] = accumulate_report(ins, args.seed, with_oracle=not args.no_cpu)
    if not args.no_cpu:
        sample_n = min(n, 8 * 1024 * 1024)
        host_inputs = [t[:sample_n].cpu().numpy() for t in ins]
        record["parity_vs_fp64_oracle"] = chain_parity(host_inputs, np.stack([o[:sample_n].cpu().numpy() for o in outs]))
        record["cpu_baseline"] = cpu_baseline(host_inputs)
        record["host_templates"] = host_templates(host_inputs)
    del ins, outs
    torch.cuda.empty_cache()
    record["splat"] = splat_report(with_oracle=not args.no_cpu)
    record["linreg"] = linreg_report(with_oracle=not args.no_cpu)
    record["trainer"] = trainer_report()
    print(json.dumps(record))


if __name__ == "__main__":
    main()
