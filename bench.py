#!/usr/bin/env python3
"""Benchmark of the 2-D Gaussian-splatting hot path on one MI355X.

A "step" is one forward + one backward of `gaussian_splatting_2d` over one batch of
synthetic inputs (already resident in HBM) at the headline configuration
B=16, N=8192, 256x256, C=3, fp32.  Prints ONE JSON line:

  metric/value : Gaussian-pixel evaluations per second, forward+backward = B*N*H*W / t_step
  roofline     : the dominant kernel (backward per-Gaussian reduction), algorithmic FLOPs per
                 launch / its HIP-event-timed launch duration, against the fp32 vector peak
  cpu_baseline : the chunked torch autograd path of the reference restated on the CPU
                 (oracle/chunked_cpu.py), timed on this box's host cores on a bounded sample.

usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1] [--no-cpu] | --all | --sweep
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_VECTOR_PEAK_TFLOPS = 157.3  # MI355X published fp32 vector (packed-FMA) peak


# Per-launch counter readings of the two hot kernels at c1, taken from the committed rocprofv3 summary
# (profiles/k_fwd_sep_k_bwd_sep_c1_B16_N8192_256x256_C3.md): wave-level instruction counts and HBM KiB.
# executed FLOPs = (2 FMA + MUL + ADD + TRANS) x 64 lanes; HBM bytes = FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0
# (factors from the plain-copy calibration of the same profile run).
C1_PROFILE = {
    "source": "profiles/k_fwd_sep_k_bwd_sep_c1_B16_N8192_256x256_C3.md",
    "bwd": {"fma": 7.643e8, "mul": 1.465e8, "add": 8.396e7, "trans": 6.902e7, "fetch_kib": 54010, "write_kib": 201500},
    "fwd": {"fma": 4.182e8, "mul": 1.316e7, "add": 7.403e7, "trans": 6.971e7, "fetch_kib": 11920, "write_kib": 131100},
}


def executed_flops(k):
    return (2 * k["fma"] + k["mul"] + k["add"] + k["trans"]) * 64


def hbm_bytes(k):
    return (k["fetch_kib"] * 2.0 + k["write_kib"] * 1.0) * 1024


def flops_per_pair(C: int):
    """Algorithmic FLOPs per Gaussian-pixel pair (FMA = 2, exp = 1)."""
    return 12 + 2 * C, 30 + 4 * C


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="c1", choices=["c0", "c1", "c2", "c4"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--cpu-full", action="store_true",
                    help="time the CPU baseline on the whole batch of the configuration (c1: about two minutes on 16 "
                         "threads) instead of the bounded sample")
    ap.add_argument("--sweep", action="store_true",
                    help="instead of the JSON line, print the operator-level table of the reference's "
                         "scripts/profiling.py (B x N x H sweep, median of 32 timed calls after 4 warm-ups)")
    ap.add_argument("--sweep-shape", default=None, metavar="BxNxH",
                    help="with --sweep: this one shape only, forward+backward with all eight gradients (for profiling "
                         "the general-grid kernels)")
    ap.add_argument("--sweep-no-grid-grads", action="store_true",
                    help="with --sweep: the two coordinate grids do not require gradients (six gradients instead of "
                         "the eight of the reference's protocol)")
    ap.add_argument("--all", action="store_true",
                    help="instead of the JSON line, print forward and forward+backward times of all five "
                         "configurations (c0-c4; c3 is the module, c2 also as the fused fit step)")
    ap.add_argument("--koleo", action="store_true",
                    help="instead of the JSON line, print forward and forward+backward times of the KoLeo "
                         "diversity loss (src/igs/reg.py of the reference) beside the plain torch expression")
    ap.add_argument("--koleo-shape", default=None, metavar="BxNxD",
                    help="with --koleo: time this one shape only, without the torch and CPU columns (for profiling)")
    ap.add_argument("--skip-tolerance", type=float, default=None, metavar="T",
                    help="bound on what skipped pairs may change in an output element, as a fraction of the largest "
                         "colour (default: the library's 1e-7; 0 = skip exact zeros only)")
    ap.add_argument("--no-cull", action="store_true", help="evaluate every pair (IGS_OPT_NO_CULL)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 256 MiB device copies (known traffic) so that a rocprofv3 "
                         "--pmc FETCH_SIZE / WRITE_SIZE run of this command carries its own scale")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path shards over the batch with no "
              "exchange; no multi-GPU run is part of it). Use --gpus 1.", file=sys.stderr)
        return 2

    # what the separable kernels may skip, for every mode below (explicit arguments of each library call)
    from igs_amd._splat import library_options
    with library_options(no_cull=args.no_cull, skip_tolerance=args.skip_tolerance):
        return run(args)


def run(args) -> int:
    if args.sweep:
        return sweep(args.sweep_shape, not args.sweep_no_grid_grads)
    if args.all:
        return all_configs(args.steps, args.warmup)
    if args.koleo:
        return koleo_table(args.no_cpu, args.koleo_shape)

    import torch

    import igs_amd
    from igs_amd import _lib
    from igs_amd._splat import Grid as _Grid, Splat as _Splat, _ptr, _stream
    from oracle import gs2d_oracle as O

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    d = {k: v.to(dev) for k, v in O.make_config_inputs(args.config).items()}
    B, N, C = d["colors"].shape
    H, W = d["x_grid"].shape[-2:]
    # the configuration's grids are linspaces *expanded* to [B,1,H,W]; .to(device) materialises
    # them, so restore the stride-0 form on the device
    d["x_grid"] = d["x_grid"][:1, :, :1, :].expand(B, 1, H, W)
    d["y_grid"] = d["y_grid"][:1, :, :, :1].expand(B, 1, H, W)
    pairs = B * N * H * W
    names = ("positions", "colors", "scales", "rotations", "alphas")
    leaves = {k: d[k].clone().requires_grad_(True) for k in names}

    def forward():
        return igs_amd.gaussian_splatting_2d(leaves["positions"], leaves["colors"], leaves["scales"],
                                             leaves["rotations"], leaves["alphas"], d["x_grid"], d["y_grid"])

    def step():
        out = forward()
        out.backward(d["grad_out"])
        for v in leaves.values():
            v.grad = None

    # ---- the timed path must be the correct one: image 0 of its output against the fp64 oracle
    with torch.no_grad():
        chk = forward()[:1].double()
    g64 = {k: d[k][:1].double() for k in names + ("x_grid", "y_grid")}
    ca, cb, cd = O.cov_inverse_closed(g64["scales"], g64["rotations"])
    ref, _ = O.forward_strips(g64["x_grid"], g64["y_grid"], g64["positions"], ca, cb, cd, g64["alphas"], g64["colors"],
                              rows=8)
    err = (chk - ref).abs()
    if not bool((err <= 1e-6 + 1e-5 * ref.abs()).all()):
        print(f"bench.py: output differs from the oracle (max err {float(err.max()):.3e}); not timing a wrong result",
              file=sys.stderr)
        return 1
    del chk, ref, err, g64

    if args.copy_calibration:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- whole step: W warm-ups, then exactly K steps between two synchronisations
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t_step = (time.perf_counter() - t0) / args.steps

    # ---- forward only (reported next to it)
    with torch.no_grad():
        for _ in range(3):
            forward()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            forward()
        torch.cuda.synchronize()
        t_fwd = (time.perf_counter() - t0) / args.steps

    # ---- dominant kernel alone, HIP events on the stream it is launched on
    grid = _Grid(d["x_grid"], d["y_grid"], B)
    op = _Splat(B, N, C, grid, 1e-6, dev)
    f32 = lambda t: t.detach().float().contiguous()
    col = f32(d["colors"])
    packed = op.pack_scale_rot(f32(d["positions"]), f32(d["scales"]), f32(d["rotations"]), f32(d["alphas"]), col)
    out, den = op.forward(packed)
    pix = op._empty(op.plan.pix_bytes)
    partial = op._empty(op.plan.partial_bytes)
    lib = _lib.load()
    st = _stream(dev)
    _lib.check(lib.igs_gs2d_backward_prologue(_ptr(grid.x), _ptr(grid.y), grid.strides, grid.mode, _ptr(grid.flag),
                                              _ptr(out),
                                              _ptr(den), _ptr(f32(d["grad_out"])), B, N, H, W, C, 1e-6, _ptr(pix),
                                              int(op.plan.pix_bytes), st), "prologue")

    built = [False]   # the first call builds the tile lists; the timed ones find them in place: k_bwd_sep alone

    def reduce_kernel():
        mode = grid.mode | (_lib.IGS_OPT_LISTS_BUILT if built[0] else 0)
        built[0] = True
        _lib.check(lib.igs_gs2d_backward_reduce(_ptr(packed), _ptr(col), _ptr(grid.y), grid.strides, mode,
                                                _ptr(grid.flag), B, N,
                                                H, W, C, _ptr(pix), int(op.plan.pix_bytes), _ptr(partial),
                                                int(op.plan.partial_bytes), st), "reduce")

    fwd_ws = op._empty(op.plan.fwd_ws_bytes)
    fwd_out, fwd_den = op._new(B, C, H, W), op._new(B, H, W)

    def fwd_kernel():
        _lib.check(lib.igs_gs2d_forward(_ptr(packed), _ptr(grid.x), _ptr(grid.y), grid.strides, grid.mode,
                                        _ptr(grid.flag), B, N, H, W, C, 1e-6, _ptr(fwd_out), _ptr(fwd_den), _ptr(fwd_ws),
                                        int(op.plan.fwd_ws_bytes), st), "forward")

    def event_time(fn, reps):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(torch.cuda.current_stream(dev))
        for _ in range(reps):
            fn()
        e1.record(torch.cuda.current_stream(dev))
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / reps

    t_bwd_kernel = event_time(reduce_kernel, args.steps)
    t_fwd_kernel = event_time(fwd_kernel, args.steps)
    f_fwd, f_bwd = flops_per_pair(C)

    # Pairs the backward kernel evaluated: its per-tile Gaussian lists (behind the pixel records in the
    # workspace; written by the k_bin launch inside the bracket) times the pixels of each tile.  Pairs
    # that are not listed are exact zeros and are skipped.
    plan = op.plan
    scratch = (B * H * plan.w_padded * plan.pix_stride + B * plan.w_padded) * 4
    counts = pix.view(torch.int32)[(scratch + 15) // 16 * 4:][: B * plan.bwd_tiles].view(B, -1, plan.bwd_tiles_x).cpu()
    rows = torch.tensor([min(H, (i + 1) * plan.bwd_per_tile) - i * plan.bwd_per_tile for i in range(counts.shape[1])])
    tw = plan.bwd_tile_w
    cols = torch.tensor([min(W, (i + 1) * tw) - i * tw for i in range(plan.bwd_tiles_x)])
    evaluated = int((counts.long() * (rows[:, None] * cols[None, :])[None]).sum())
    achieved = evaluated * f_bwd / t_bwd_kernel / 1e12
    prof = C1_PROFILE if (args.config == "c1" and C == 3) else None
    # The same for the forward (C <= 8: one list per wave rectangle of 32 columns x 2P rows, P = 16 for
    # C <= 3 and 8 above, numbered row after row of rectangles over the 64 x 4P tiles' extent; behind the
    # split partials in the forward's workspace).
    fwd_evaluated = None
    if C <= 8:
        P = 16 if C <= 3 else 8
        split = plan.fwd_split * B * (C + 1) * H * W * 4 if plan.fwd_split > 1 else 0
        tx_n, ty_n = -(-W // 64), -(-H // (4 * P))
        cols_n, rows_n = -(-W // 32), -(-H // (2 * P))
        fc = fwd_ws.view(torch.int32)[(split + 15) // 16 * 4:][: B * plan.fwd_tiles].view(B, 2 * ty_n, 2 * tx_n)
        fc = fc[:, :rows_n, :cols_n].cpu()
        frows = torch.tensor([min(H, (i + 1) * 2 * P) - i * 2 * P for i in range(rows_n)])
        fcols = torch.tensor([min(W, (i + 1) * 32) - i * 32 for i in range(cols_n)])
        fwd_evaluated = int((fc.long() * (frows[None, :, None] * fcols[None, None, :])).sum())

    result = {
        "metric": "gaussian_pixel_evals_per_sec_fwd_bwd",
        "value": pairs / t_step,
        "unit": "pairs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": t_step * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{args.config}: gaussian_splatting_2d fwd+bwd, B={B} N={N} {H}x{W} C={C} fp32, "
                               "linspace grids, seeded U/N inputs", "B": B, "N": N, "H": H, "W": W, "C": C},
        "fwd_pairs_per_s": pairs / t_fwd,
        "fwd_ms": t_fwd * 1e3,
        "step_tflops": pairs * (f_fwd + f_bwd) / t_step / 1e12,
        "step_frac_of_fp32_vector_peak": pairs * (f_fwd + f_bwd) / t_step / 1e12 / FP32_VECTOR_PEAK_TFLOPS,
        "step_frac_counting_evaluated_pairs": ((fwd_evaluated or pairs) * f_fwd + evaluated * f_bwd) / t_step / 1e12
                                              / FP32_VECTOR_PEAK_TFLOPS,
        "roofline": {
            "bound": "valu",
            "kernel": f"k_bwd_sep<{C},1> (backward per-Gaussian reduction)",
            "achieved": achieved,
            "peak": FP32_VECTOR_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / FP32_VECTOR_PEAK_TFLOPS,
            "flops_per_pair": f_bwd,
            "pairs_per_launch": pairs,
            "pairs_evaluated_per_launch": evaluated,
            "frac_counting_all_pairs": pairs * f_bwd / t_bwd_kernel / 1e12 / FP32_VECTOR_PEAK_TFLOPS,
            "launch_ms": t_bwd_kernel * 1e3,
            "executed_frac": executed_flops(prof["bwd"]) / t_bwd_kernel / 1e12 / FP32_VECTOR_PEAK_TFLOPS if prof else None,
            "traffic": hbm_bytes(prof["bwd"]) if prof else None,
            "forward_kernel": {"launch_ms": t_fwd_kernel * 1e3, "flops_per_pair": f_fwd,
                               "pairs_evaluated_per_launch": fwd_evaluated,
                               "achieved": (fwd_evaluated or pairs) * f_fwd / t_fwd_kernel / 1e12,
                               "frac": (fwd_evaluated or pairs) * f_fwd / t_fwd_kernel / 1e12 / FP32_VECTOR_PEAK_TFLOPS,
                               "frac_counting_all_pairs": pairs * f_fwd / t_fwd_kernel / 1e12 / FP32_VECTOR_PEAK_TFLOPS,
                               "executed_frac": executed_flops(prof["fwd"]) / t_fwd_kernel / 1e12 / FP32_VECTOR_PEAK_TFLOPS
                               if prof else None,
                               "traffic": hbm_bytes(prof["fwd"]) if prof else None},
            "counter_source": prof["source"] if prof else None,
            "note": "achieved / frac: the 30+4C FLOP model of one backward pair x the pairs the kernel evaluated (a tile's "
                    "list leaves out the Gaussians with the smallest weights there as long as their sum stays within the "
                    "call's allowance, which bounds the change of every output element by 1e-7 max|colour|; frac_counting_all_pairs uses all B N H W as the metric does and can "
                    "exceed 1) / launch_ms, measured live with HIP events around igs_gs2d_backward_reduce with the tile lists "
                    "in place (IGS_OPT_LISTS_BUILT: k_bwd_sep alone; a training step builds the lists once, in its "
                    "forward); the forward's launch_ms holds k_bin + k_fwd_sep + combine.  executed_frac: the arithmetic the hardware ran, (2 FMA + MUL + ADD + TRANS) x 64 per "
                    "launch from the rocprofv3 counters of counter_source (separable grids hoist the row/column part of "
                    "the model's operations, so it is below frac) / the live launch_ms.  traffic: HBM bytes per launch "
                    "from FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 of the same summary (copy-calibrated); c1 only.  peak: "
                    "published fp32 vector peak at 2.4 GHz; the kernels use plain fp32 VALU ops with VGPR-only operands, "
                    "v_exp_f32 counted as 1 FLOP.",
        },
    }

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(args.config, O, full=args.cpu_full)
    print(json.dumps(result), flush=True)
    return 0


def all_configs(steps: int, warmup: int) -> int:
    """Forward and forward+backward wall time of the five configurations through the public API
    (allocation included), pairs/s counting all B N H W pairs as scripts/profiling.py:199-211 does,
    and the fraction of the fp32 vector peak by the 42 + 6 C FLOP/pair model (above 1 is possible
    where culling skips pairs).  "c0 1 thread" is the c0 step under
    torch.autograd.set_multithreading_enabled(False).  The "fit step" rows are the graph-replayed fused iteration of
    igs_amd.fit on the same problem: at c0 the public call is bound by the host's per-call cost
    (Python, torch allocation, autograd: 0.13-0.25 ms depending on the box), the replay is not."""
    import torch

    import igs_amd
    from igs_amd.fit import GaussianImageFit
    from oracle import gs2d_oracle as O

    dev = torch.device("cuda:0")
    names = ("positions", "colors", "scales", "rotations", "alphas")

    def timeit(fn, n):
        # Small configurations finish a step in a fraction of a millisecond: warm up and time for a
        # minimum duration as well as a minimum count, or the numbers show the GPU's clock ramp
        # (c0 reads 0.23 ms over 30 steps after 10 warm-ups and 0.145 ms once the clocks are up).
        t0 = time.perf_counter()
        k = 0
        while k < warmup or time.perf_counter() - t0 < 0.25:
            fn()
            k += 1
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        n = max(n, min(2000, int(0.25 / max(time.perf_counter() - t0, 1e-6))))
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n

    rows = []
    for cfg in ("c0", "c1", "c2", "c3", "c4"):
        if cfg == "c3":
            torch.manual_seed(1003)
            m = igs_amd.GaussianSplatting2D(32, 1024).to(dev)
            x = torch.randn(8, 128, 1024, device=dev, requires_grad=True)
            go = torch.randn(8, 3, 256, 256, device=dev)
            B, N, H, W, C = 8, 4096, 256, 256, 3

            def fwd():
                with torch.no_grad():
                    m(x, size=(256, 256))

            def step():
                m(x, size=(256, 256))[0].backward(go)
                x.grad = None
                m.zero_grad(set_to_none=True)
        else:
            d = {k: v.to(dev) for k, v in O.make_config_inputs(cfg).items()}
            B, N, C = d["colors"].shape
            H, W = d["x_grid"].shape[-2:]
            d["x_grid"] = d["x_grid"][:1, :, :1, :].expand(B, 1, H, W)
            d["y_grid"] = d["y_grid"][:1, :, :, :1].expand(B, 1, H, W)
            lv = {k: d[k].clone().requires_grad_(True) for k in names}

            def fwd(d=d, lv=lv):
                with torch.no_grad():
                    igs_amd.gaussian_splatting_2d(*(lv[k] for k in names), d["x_grid"], d["y_grid"])

            def step(d=d, lv=lv):
                igs_amd.gaussian_splatting_2d(*(lv[k] for k in names), d["x_grid"], d["y_grid"]).backward(d["grad_out"])
                for v in lv.values():
                    v.grad = None
        n = max(3, steps // 3) if cfg == "c4" else steps
        rows.append((cfg, B, N, H, W, C, timeit(fwd, n), timeit(step, n)))
        if cfg == "c0":   # the same public call with autograd's backward run on the calling thread: the hand-over to
            # the engine's device thread and back is 60-130 us of the host's time per step on the boxes seen
            with torch.autograd.set_multithreading_enabled(False):
                rows.append((cfg + " 1 thread", B, N, H, W, C, float("nan"), timeit(step, n)))
        if cfg in ("c0", "c2"):   # the fused fit iteration (render, MSE, backward, AdamW) on the same problem,
            # replayed from a HIP graph: the step without the host's per-call cost
            block = torch.cat([d["positions"], d["scales"].log(), d["rotations"][..., None],
                               torch.zeros_like(d["rotations"])[..., None], d["colors"]], -1)
            fit = GaussianImageFit(block, O.smooth_noise_target(H, W, seed=1002).to(dev), d["x_grid"], d["y_grid"],
                                   lr=min(0.05 * 4096 / N, 0.03))
            fit.capture()
            rows.append((cfg + " fit step", B, N, H, W, C, float("nan"), timeit(fit.step, n)))
    print("%-12s %3s %6s %4s %4s %3s %10s %12s %14s %10s" % ("config", "B", "N", "H", "W", "C", "fwd ms", "fwd+bwd ms",
                                                           "pairs/s", "of peak"))
    for cfg, B, N, H, W, C, tf, t in rows:
        pairs = B * N * H * W
        print("%-12s %3d %6d %4d %4d %3d %10.3f %12.3f %14.3e %10.2f" % (cfg, B, N, H, W, C, tf * 1e3, t * 1e3, pairs / t,
                                                                       pairs * (42 + 6 * C) / t / 1e12 / FP32_VECTOR_PEAK_TFLOPS))
    return 0


def koleo_table(no_cpu: bool, only: str = None) -> int:
    """KoLeo diversity loss: events around `koleo_diversity_loss(x)` and around loss + backward (4 warm-ups,
    median of 32), for the two shapes scripts/gs2d_test.py:146,172 of the reference passes ([1, N, 9] Gaussian
    features, [1, k <= 128, 512] latent features) and larger ones; beside it the same expression in eager fp32
    torch on the GPU (the oracle's restatement of src/igs/reg.py:22-37, which holds the [B,N,N] matrix; skipped
    above 4 GiB) and on the host cores.  FLOP model: 2 B N^2 D for the similarities (forward)."""
    import torch

    import igs_amd
    from oracle import koleo_oracle as K

    dev = torch.device("cuda:0")

    def median_ms(fn):
        for _ in range(4):
            fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(32):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1))
        return sorted(ts)[len(ts) // 2]

    def both(loss_fn, x):
        xg = x.clone().requires_grad_(True)

        def step():
            xg.grad = None
            loss_fn(xg).backward()

        with torch.no_grad():
            f = median_ms(lambda: loss_fn(x))
        return f, median_ms(step)

    print("%-16s %10s %10s %12s %12s %12s %10s" % ("B x N x D", "fwd ms", "f+b ms", "torch fwd", "torch f+b",
                                                   "TFLOP/s fwd", "cpu f+b ms"))
    shapes = [(1, 128, 512), (1, 4096, 9), (8, 4096, 9), (1, 16384, 9), (4, 16384, 32), (1, 65536, 9)]
    if only:
        shapes, no_cpu = [tuple(int(v) for v in only.split("x"))], True
    for shape in shapes:
        B, N, D = shape
        x = torch.randn(*shape, device=dev, generator=torch.Generator(dev).manual_seed(0))
        f, fb = both(igs_amd.koleo_diversity_loss, x)
        tf = tfb = float("nan")
        if not only and B * N * N * 4 <= 4 << 30:
            tf, tfb = both(K.koleo_diversity_loss, x)
        cpu = float("nan")
        if not no_cpu and B * N * N <= 1 << 28:
            xc = x.cpu()
            t0 = time.perf_counter()
            K.autograd_gradient(xc)
            cpu = (time.perf_counter() - t0) * 1e3
        print("%-16s %10.4f %10.4f %12.4f %12.4f %12.2f %10.1f" % ("%dx%dx%d" % shape, f, fb, tf, tfb,
                                                                  2.0 * B * N * N * D / (f * 1e-3) / 1e12, cpu))
    return 0


def sweep(only: str = None, grid_grads: bool = True) -> int:
    """Operator-level sweep in the protocol of the reference's scripts/profiling.py:30-49, :69-151, :199-211:
    `.apply(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors)` on randn/rand inputs (per-pixel
    random coordinates, so the general-grid kernels run), 4 warm-ups, 32 timed calls with events, median;
    forward+backward uses `output.mean().backward()`.  Columns as in the reference's table."""
    import itertools

    import torch

    from igs_amd import GaussianSplatting2DKernel

    dev = torch.device("cuda:0")
    rows = []
    shapes = list(itertools.product([4, 8], [4096, 8192, 16384], [128, 256]))
    if only:
        shapes = [tuple(int(v) for v in only.split("x"))]
    for B, N, H in shapes:
        W = H
        for mode in ("fwd", "fwd_bwd"):
            rg = mode == "fwd_bwd"
            mk = lambda *sh, fn=torch.randn: fn(*sh, device=dev).requires_grad_(rg)
            mkg = (lambda *sh: mk(*sh)) if grid_grads else (lambda *sh: torch.randn(*sh, device=dev))
            inputs = (mkg(B, 1, H, W), mkg(B, 1, H, W), mk(B, N, 2), mk(B, N, 1, 1), mk(B, N, 1, 1), mk(B, N, 1, 1),
                      mk(B, N, fn=torch.rand), mk(B, N, 3, fn=torch.rand))

            def call():
                out = GaussianSplatting2DKernel.apply(*inputs)
                if rg:
                    out.mean().backward()
                    for t in inputs:
                        t.grad = None

            for _ in range(4):
                call()
            torch.cuda.synchronize()
            ts = []
            for _ in range(32):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                call()
                e1.record()
                torch.cuda.synchronize()
                ts.append(e0.elapsed_time(e1))
            ms = sorted(ts)[len(ts) // 2]
            rows.append(("HipGaussianSplatting2D", B, N, H, "Forward" if mode == "fwd" else "Fwd+Bwd", ms,
                         B * N * H * W / (ms * 1e-3) / 1e9, B * N / (ms * 1e-3) / 1e6))
    print("%-24s %3s %6s %4s %-8s %10s %12s %14s" % ("Kernel", "B", "N", "H", "Pass", "ms", "G-pixels/s", "M-Gaussians/s"))
    for r in rows:
        print("%-24s %3d %6d %4d %-8s %10.4f %12.2f %14.2f" % r)
    return 0


def host_cpu():
    """(model name, physical cores) of the host, from /proc/cpuinfo."""
    model, cores = "unknown", set()
    try:
        phys = core = None
        for line in open("/proc/cpuinfo"):
            k, _, v = line.partition(":")
            k, v = k.strip(), v.strip()
            if k == "model name":
                model = v
            elif k == "physical id":
                phys = v
            elif k == "core id":
                core = v
            elif not k and phys is not None:
                cores.add((phys, core))
                phys = core = None
    except OSError:
        pass
    return model, len(cores) or (os.cpu_count() or 0)


def cpu_baseline(config: str, O, full: bool = False):
    """Chunked torch autograd path on the host cores, on a bounded sample of the same workload
    (a few images of it; cost is linear in the number of images) or, with `full`, on all of it."""
    import torch

    from oracle.chunked_cpu import render_chunked_cpu

    threads = torch.get_num_threads()
    cfg = O.CONFIGS[config]
    nb = cfg["B"] if full else {"c0": 1, "c1": 4, "c2": 1, "c4": 1}[config]
    N = cfg["N"] // 8 if (config == "c4" and not full) else cfg["N"]
    d = O.make_config_inputs(config, B=nb, N=N)
    B, N, C = d["colors"].shape
    H, W = d["x_grid"].shape[-2:]
    names = ("positions", "colors", "scales", "rotations", "alphas")
    leaves = {k: d[k].clone().requires_grad_(True) for k in names}
    xg, yg = d["x_grid"].contiguous(), d["y_grid"].contiguous()

    def run():
        out = render_chunked_cpu(leaves["positions"], leaves["colors"], leaves["scales"], leaves["rotations"],
                                 leaves["alphas"], xg, yg)
        out.backward(d["grad_out"])
        for v in leaves.values():
            v.grad = None

    # warm-up on a 1/16 slice of the Gaussians, then one timed pass
    small = {k: v[:, : max(N // 16, 32)].detach().clone().requires_grad_(True) for k, v in leaves.items()}
    o = render_chunked_cpu(small["positions"], small["colors"], small["scales"], small["rotations"], small["alphas"], xg, yg)
    o.backward(d["grad_out"])
    t0 = time.perf_counter()
    run()
    t = time.perf_counter() - t0
    pairs = B * N * H * W
    model, physical = host_cpu()
    what = "the whole batch" if (B == cfg["B"] and N == cfg["N"]) else "a bounded sample"
    return {"value": pairs / t, "unit": "pairs/s", "cores": threads, "kind": "port",
            "cpu_model": model, "physical_cores": physical,
            "sample": f"{what}: {B} image(s) of {config} (B={B}, N={N}, {H}x{W}, C={C}), fwd+bwd once, {t:.1f} s, "
                      f"eager torch fp32 with {threads} threads on {model} ({physical} physical cores visible)"}


if __name__ == "__main__":
    sys.exit(main())
