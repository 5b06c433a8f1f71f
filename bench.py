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

usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1] [--no-cpu] [--default-only] | --fit | --all | --sweep | --koleo
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
# executed FLOPs = (2 FMA + MUL + ADD + TRANS) x 64 lanes + 512 per 4x4x1 matrix instruction (16 blocks x 4 x 4 FMA);
# HBM bytes = FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0
# (factors from the plain-copy calibration of the same profile run).  `csrc_sha16` names the kernel sources
# the counters were read from (csrc_sha16() below): with other sources the instruction counts no longer
# belong to the kernels being timed, and the fields derived from them are reported as null.
C1_PROFILE = {
    "source": "profiles/k_fwd_sep_k_bwd_sep_c1_B16_N8192_256x256_C3.md",
    "csrc_sha16": "a244c3e3a6718d95",
    "bwd": {"fma": 6.862e8, "mul": 7.632e7, "add": 7.615e7, "trans": 6.770e7, "fetch_kib": 55720, "write_kib": 147400},
    "fwd": {"fma": 1.386e8, "mul": 1.269e7, "add": 8.919e6, "trans": 6.714e7, "mfma": 6.707e7, "fetch_kib": 12700, "write_kib": 131100},
}


def csrc_sha16():
    """First 16 hex digits of the SHA-256 over the kernel sources (igs_amd/csrc/*, include/igs_hip.h), in name order."""
    import hashlib

    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "igs_amd", "csrc")
    for path in sorted(os.path.join(csrc, f) for f in os.listdir(csrc)) + [os.path.join(ROOT, "include", "igs_hip.h")]:
        if os.path.isfile(path):
            h.update(os.path.basename(path).encode())
            h.update(open(path, "rb").read())
    return h.hexdigest()[:16]


def executed_flops(k):
    return (2 * k["fma"] + k["mul"] + k["add"] + k["trans"]) * 64 + 512 * k.get("mfma", 0.0)


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
    ap.add_argument("--config", default="c1", choices=["c0", "c1", "c2", "c3", "c4"],
                    help="c3 (the module) prints the step figures only: its kernels are the same as c1's")
    ap.add_argument("--csrc-sha", action="store_true", help="print csrc_sha16() of this tree and exit")
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
    ap.add_argument("--fit", action="store_true",
                    help="instead of the JSON line of the operator, time the fused fit iteration (render, MSE, backward, "
                         "AdamW; igs_amd.fit) of --config c0 or c2, replayed from a HIP graph, and print its own line")
    ap.add_argument("--default-only", action="store_true",
                    help="leave out the `exact` and `no_cull` legs (for profiling: every launch of the run then belongs "
                         "to the default path)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 256 MiB device copies (known traffic) so that a rocprofv3 "
                         "--pmc FETCH_SIZE / WRITE_SIZE run of this command carries its own scale")
    args = ap.parse_args()
    if args.csrc_sha:
        print(csrc_sha16())
        return 0
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
        return all_configs(args.steps, args.warmup, args.no_cpu)
    if args.koleo:
        return koleo_table(args.no_cpu, args.koleo_shape)
    if args.fit:
        return fit_step(args.config, args.steps, args.warmup)

    import torch

    import igs_amd
    from igs_amd._splat import library_options
    from oracle import gs2d_oracle as O

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    names = ("positions", "colors", "scales", "rotations", "alphas")
    module_path = args.config == "c3"
    if module_path:   # the module: 32 Gaussians per feature, feature_dim 1024, x [8,128,1024] -> [8,3,256,256]
        torch.manual_seed(1003)
        model = igs_amd.GaussianSplatting2D(32, 1024).to(dev)
        feat = torch.randn(8, 128, 1024, device=dev, requires_grad=True)
        grad_out = torch.randn(8, 3, 256, 256, device=dev)
        B, N, H, W, C = 8, 4096, 256, 256, 3

        def forward():
            return model(feat, size=(H, W))[0]

        def step():
            forward().backward(grad_out)
            feat.grad = None
            model.zero_grad(set_to_none=True)
    else:
        d = {k: v.to(dev) for k, v in O.make_config_inputs(args.config).items()}
        B, N, C = d["colors"].shape
        H, W = d["x_grid"].shape[-2:]
        # the configuration's grids are linspaces *expanded* to [B,1,H,W]; .to(device) materialises
        # them, so restore the stride-0 form on the device
        d["x_grid"] = d["x_grid"][:1, :, :1, :].expand(B, 1, H, W)
        d["y_grid"] = d["y_grid"][:1, :, :, :1].expand(B, 1, H, W)
        leaves = {k: d[k].clone().requires_grad_(True) for k in names}

        def forward():
            return igs_amd.gaussian_splatting_2d(leaves["positions"], leaves["colors"], leaves["scales"],
                                                 leaves["rotations"], leaves["alphas"], d["x_grid"], d["y_grid"])

        def step():
            out = forward()
            out.backward(d["grad_out"])
            for v in leaves.values():
                v.grad = None
    pairs = B * N * H * W

    # ---- the timed path must be the correct one: image 0 of its output against the fp64 oracle
    if not module_path:
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

    # ---- whole step: W warm-up steps (and as many more as it takes to keep the GPU busy for 0.3 s: a
    # step of a few milliseconds otherwise lands on the clock ramp), then exactly K steps between two
    # synchronisations; then the same K steps timed one by one with events on the launch stream, whose
    # median is the protocol of the reference's benchmark (scripts/profiling.py:103-151)
    def timed(fn, steps, warmup, min_warm_s=0.3):
        t0 = time.perf_counter()
        k = 0
        while k < warmup or time.perf_counter() - t0 < min_warm_s:
            fn()
            k += 1
            if k % 8 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        mean = (time.perf_counter() - t0) / steps
        ts = []
        stream = torch.cuda.current_stream(dev)
        for _ in range(steps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            fn()
            e1.record(stream)
            torch.cuda.synchronize()
            ts.append(e0.elapsed_time(e1) * 1e-3)
        return mean, sorted(ts)[len(ts) // 2]

    t_step, t_step_median = timed(step, args.steps, args.warmup)

    # ---- forward only (reported next to it)
    with torch.no_grad():
        t_fwd, t_fwd_median = timed(forward, args.steps, 3, 0.1)

    # ---- the same step with nothing but exact zeros skipped, and with every pair evaluated (what the
    # reference does): the default leaves out pairs within the call's allowance, so `value` counts pairs
    # that were never evaluated; these two are the figures without that
    f_fwd, f_bwd = flops_per_pair(C)
    side = {}
    for key, opts in (("exact", dict(skip_tolerance=0.0)), ("no_cull", dict(no_cull=True))):
        if args.default_only:
            side[key] = None
            continue
        with library_options(**opts):
            t_mean, t_med = timed(step, min(args.steps, 10), 3, 0.1)
        side[key] = {"ms_per_step": t_mean * 1e3, "median_ms_per_step": t_med * 1e3, "value": pairs / t_mean,
                     "what": {"exact": "skip_tolerance = 0: only pairs whose fp32 weight is exactly zero are left out",
                              "no_cull": "IGS_OPT_NO_CULL: every Gaussian listed for every tile, all B N H W pairs evaluated"}[key]}
    if side["no_cull"]:
        side["no_cull"]["frac"] = pairs * (f_fwd + f_bwd) / (side["no_cull"]["ms_per_step"] * 1e-3) / 1e12 / FP32_VECTOR_PEAK_TFLOPS

    result = {
        "metric": "gaussian_pixel_evals_per_sec_fwd_bwd",
        "value": pairs / t_step,
        "unit": "pairs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": t_step * 1e3,
        "median_ms_per_step": t_step_median * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": (f"{args.config}: GaussianSplatting2D(32, 1024) module fwd+bwd, x [8,128,1024] -> "
                                if module_path else f"{args.config}: gaussian_splatting_2d fwd+bwd, ") +
                               f"B={B} N={N} {H}x{W} C={C} fp32, linspace grids, seeded U/N inputs",
                   "B": B, "N": N, "H": H, "W": W, "C": C},
        "fwd_pairs_per_s": pairs / t_fwd,
        "fwd_ms": t_fwd * 1e3,
        "fwd_median_ms": t_fwd_median * 1e3,
        "step_tflops": pairs * (f_fwd + f_bwd) / t_step / 1e12,
        "step_frac_counting_all_pairs": pairs * (f_fwd + f_bwd) / t_step / 1e12 / FP32_VECTOR_PEAK_TFLOPS,
        "exact": side["exact"],
        "no_cull": side["no_cull"],
        "timing": "value / ms_per_step: `steps` steps between two synchronisations after `warmup` steps and at least 0.3 s "
                  "of steps; median_*: the same number of steps timed one by one with events on the launch stream",
    }
    if module_path:
        result["roofline"] = None
        print(json.dumps(result), flush=True)
        return 0

    # ---- dominant kernel alone, HIP events on the stream it is launched on
    probe = KernelProbe(d, B, N, H, W, C, dev)

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

    t_bwd_kernel = event_time(probe.reduce_kernel, args.steps)
    t_fwd_kernel = event_time(probe.fwd_kernel, args.steps)
    fwd_evaluated, evaluated = probe.evaluated()
    achieved = evaluated * f_bwd / t_bwd_kernel / 1e12
    prof = C1_PROFILE if (args.config == "c1" and C == 3 and C1_PROFILE["csrc_sha16"] == csrc_sha16()) else None

    result["step_frac_counting_evaluated_pairs"] = (((fwd_evaluated or pairs) * f_fwd + evaluated * f_bwd) / t_step / 1e12
                                                    / FP32_VECTOR_PEAK_TFLOPS)
    result.update({
        "roofline": {
            "bound": "valu",
            "kernel": f"k_bwd_sep<{C}> (backward per-Gaussian reduction)",
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
                    "forward); the forward's launch_ms holds k_bin + k_fwd_sep + combine.  executed_frac: the arithmetic the hardware ran, (2 FMA + MUL + ADD + TRANS) x 64 + 512 per 4x4x1 matrix instruction (the forward's sums) per "
                    "launch from the rocprofv3 counters of counter_source (separable grids hoist the row/column part of "
                    "the model's operations, so it is below frac) / the live launch_ms.  traffic: HBM bytes per launch "
                    "from FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 of the same summary (copy-calibrated); c1 only.  peak: "
                    "published fp32 vector peak at 2.4 GHz; the kernels use plain fp32 VALU ops with VGPR-only operands and, for the forward's "
                    "channel sums, fp32 v_mfma_f32_4x4x1 (same published peak); v_exp_f32 counted as 1 FLOP.",
        },
    })

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(args.config, O, full=args.cpu_full)
    print(json.dumps(result), flush=True)
    return 0


class KernelProbe:
    """The two hot launches of one function-path problem on their own, through the C ABI with buffers kept
    here: `reduce_kernel` = igs_gs2d_backward_reduce (the first call builds the tile lists, later ones
    find them in place: the per-Gaussian reduction kernel alone), `fwd_kernel` = igs_gs2d_forward (tile
    lists + kernel + combine), and the pairs both evaluated, read back from their tile lists."""

    def __init__(self, d, B, N, H, W, C, dev):
        import torch

        from igs_amd import _lib
        from igs_amd._splat import Grid, Splat, _ptr, _stream

        self.torch, self._lib, self._ptr = torch, _lib, _ptr
        self.dims = (B, N, H, W, C)
        self.grid = grid = Grid(d["x_grid"], d["y_grid"], B)
        self.op = op = Splat(B, N, C, grid, 1e-6, dev)
        f32 = lambda t: t.detach().float().contiguous()
        self.col = f32(d["colors"])
        self.packed = op.pack_scale_rot(f32(d["positions"]), f32(d["scales"]), f32(d["rotations"]), f32(d["alphas"]),
                                        self.col)
        self.out, self.den = op.forward(self.packed)
        self.pix = op._empty(op.plan.pix_bytes)
        self.partial = op._empty(op.plan.partial_bytes)
        self.lib = _lib.load()
        self.st = _stream(dev)
        _lib.check(self.lib.igs_gs2d_backward_prologue(_ptr(grid.x), _ptr(grid.y), grid.strides, grid.mode,
                                                       _ptr(grid.flag), _ptr(self.out), _ptr(self.den),
                                                       _ptr(f32(d["grad_out"])), B, N, H, W, C, 1e-6, _ptr(self.pix),
                                                       int(op.plan.pix_bytes), self.st), "prologue")
        self.built = False
        self.fwd_ws = op._empty(op.plan.fwd_ws_bytes)
        self.fwd_out, self.fwd_den = op._new(B, C, H, W), op._new(B, H, W)

    def reduce_kernel(self):
        B, N, H, W, C = self.dims
        g, op, _ptr = self.grid, self.op, self._ptr
        mode = g.mode | (self._lib.IGS_OPT_LISTS_BUILT if self.built else 0)
        self.built = True
        self._lib.check(self.lib.igs_gs2d_backward_reduce(_ptr(self.packed), _ptr(self.col), _ptr(g.y), g.strides, mode,
                                                          _ptr(g.flag), B, N, H, W, C, _ptr(self.pix),
                                                          int(op.plan.pix_bytes), _ptr(self.partial),
                                                          int(op.plan.partial_bytes), self.st), "reduce")

    def fwd_kernel(self):
        B, N, H, W, C = self.dims
        g, op, _ptr = self.grid, self.op, self._ptr
        self._lib.check(self.lib.igs_gs2d_forward(_ptr(self.packed), _ptr(g.x), _ptr(g.y), g.strides, g.mode,
                                                  _ptr(g.flag), B, N, H, W, C, 1e-6, _ptr(self.fwd_out),
                                                  _ptr(self.fwd_den), _ptr(self.fwd_ws), int(op.plan.fwd_ws_bytes),
                                                  self.st), "forward")

    def evaluated(self):
        """(forward, backward) pairs evaluated, after both launches ran: a launch's per-tile Gaussian lists
        (counts behind the pixel records / the split partials in its workspace) times the pixels of each
        tile; pairs that are not listed are skipped.  Forward: None for C > 8 where its workgroup tiles are
        not the backward's 32 x 32."""
        torch = self.torch
        B, N, H, W, C = self.dims
        plan = self.op.plan
        if not self.built:
            self.reduce_kernel()
        self.fwd_kernel()
        torch.cuda.synchronize()
        scratch = (B * H * plan.w_padded * plan.pix_stride + B * plan.w_padded) * 4
        counts = self.pix.view(torch.int32)[(scratch + 15) // 16 * 4:][: B * plan.bwd_tiles]
        counts = counts.view(B, -1, plan.bwd_tiles_x).cpu()
        rows = torch.tensor([min(H, (i + 1) * plan.bwd_per_tile) - i * plan.bwd_per_tile for i in range(counts.shape[1])])
        tw = plan.bwd_tile_w
        cols = torch.tensor([min(W, (i + 1) * tw) - i * tw for i in range(plan.bwd_tiles_x)])
        bwd = int((counts.long() * (rows[:, None] * cols[None, :])[None]).sum())
        fwd = None
        if C <= 8:   # one list per wave rectangle of 32 columns x 2P rows, numbered row after row of rectangles
            P = 16 if C <= 3 else 8
            split = plan.fwd_split * B * (C + 1) * H * W * 4 if plan.fwd_split > 1 else 0
            tx_n, ty_n = -(-W // 64), -(-H // (4 * P))
            cols_n, rows_n = -(-W // 32), -(-H // (2 * P))
            fc = self.fwd_ws.view(torch.int32)[(split + 15) // 16 * 4:][: B * plan.fwd_tiles].view(B, 2 * ty_n, 2 * tx_n)
            fc = fc[:, :rows_n, :cols_n].cpu()
            frows = torch.tensor([min(H, (i + 1) * 2 * P) - i * 2 * P for i in range(rows_n)])
            fcols = torch.tensor([min(W, (i + 1) * 32) - i * 32 for i in range(cols_n)])
            fwd = int((fc.long() * (frows[None, :, None] * fcols[None, None, :])).sum())
        elif plan.fwd_tiles == plan.bwd_tiles and plan.bwd_per_tile == 32:
            # one list per workgroup tile of 32 x 32 pixels, the backward's tiling
            split = plan.fwd_split * B * (C + 1) * H * W * 4 if plan.fwd_split > 1 else 0
            fc = self.fwd_ws.view(torch.int32)[(split + 15) // 16 * 4:][: B * plan.fwd_tiles]
            fc = fc.view(B, -1, plan.bwd_tiles_x).cpu()
            fwd = int((fc.long() * (rows[:, None] * cols[None, :])[None]).sum())
        return fwd, bwd


def all_configs(steps: int, warmup: int, no_cpu: bool = False) -> int:
    """Forward and forward+backward wall time of the five configurations through the public API
    (allocation included), pairs/s counting all B N H W pairs as scripts/profiling.py:199-211 does, the
    pairs the two hot kernels evaluated (read back from their tile lists) and the fraction of the fp32
    vector peak that the 12 + 2 C / 30 + 4 C FLOP-per-pair model gives on those (counting all pairs it
    exceeds 1 where culling skips most of them).  "c0 1 thread" is the c0 step under
    torch.autograd.set_multithreading_enabled(False).  The "fit step" rows are the graph-replayed fused iteration of
    igs_amd.fit on the same problem: at c0 the public call is bound by the host's per-call cost
    (Python, torch allocation, autograd: 0.13-0.25 ms depending on the box), the replay is not.
    CPU column: the reference's chunked torch autograd path restated (oracle/chunked_cpu.py) on the host
    cores for the configurations that name it, c0 and c3 (through the module's linear head): 1 warm-up,
    then the median of 3 runs of forward + backward."""
    import torch

    import igs_amd
    from igs_amd.fit import GaussianImageFit
    from oracle import gs2d_oracle as O
    from oracle.chunked_cpu import render_chunked_cpu

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

    def cpu_median(fn):
        fn()
        ts = []
        for _ in range(3):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[1]

    nan = float("nan")
    rows = []
    for cfg in ("c0", "c1", "c2", "c3", "c4"):
        cpu_s = nan
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

            # the same Gaussians as function-path inputs, for the tile lists (and for the CPU path)
            with torch.no_grad():
                f = m.proj(x).view(B, N, 6 + C)
                xs, ys = m.xy_grid((H, W), device=dev)
                d = {"positions": f[..., :2].contiguous(), "scales": (f[..., 2:4].exp() + 1e-6).contiguous(),
                     "rotations": f[..., 4].contiguous(), "alphas": torch.ones(B, N, device=dev),
                     "colors": f[..., 6:].contiguous(), "grad_out": go,
                     "x_grid": xs[None].expand(B, 1, H, W), "y_grid": ys[None].expand(B, 1, H, W)}
            if not no_cpu:
                wc, bc, xc, goc = m.proj.weight.detach().cpu(), m.proj.bias.detach().cpu(), x.detach().cpu(), go.cpu()
                xg, yg = d["x_grid"].cpu().contiguous(), d["y_grid"].cpu().contiguous()

                def cpu_step():
                    w, bb, xi = (t.clone().requires_grad_(True) for t in (wc, bc, xc))
                    fc = torch.nn.functional.linear(xi, w, bb).view(B, N, 6 + C)
                    out = render_chunked_cpu(fc[..., :2], fc[..., 6:], fc[..., 2:4].exp() + 1e-6, fc[..., 4],
                                             torch.ones(B, N), xg, yg)
                    out.backward(goc)

                cpu_s = cpu_median(cpu_step)
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
            if cfg == "c0" and not no_cpu:
                dc = {k: v.cpu() for k, v in d.items()}
                xg, yg = dc["x_grid"].contiguous(), dc["y_grid"].contiguous()

                def cpu_step():
                    l = {k: dc[k].clone().requires_grad_(True) for k in names}
                    render_chunked_cpu(*(l[k] for k in names), xg, yg).backward(dc["grad_out"])

                cpu_s = cpu_median(cpu_step)
        n = max(3, steps // 3) if cfg == "c4" else steps
        ev_f, ev_b = KernelProbe(d, B, N, H, W, C, dev).evaluated()
        rows.append((cfg, B, N, H, W, C, timeit(fwd, n), timeit(step, n), ev_f, ev_b, cpu_s))
        if cfg == "c0":   # the same public call with autograd's backward run on the calling thread: the hand-over to
            # the engine's device thread and back is 60-130 us of the host's time per step on the boxes seen
            with torch.autograd.set_multithreading_enabled(False):
                rows.append((cfg + " 1 thread", B, N, H, W, C, nan, timeit(step, n), ev_f, ev_b, nan))
        if cfg in ("c0", "c2"):   # the fused fit iteration (render, MSE, backward, AdamW) on the same problem,
            # replayed from a HIP graph: the step without the host's per-call cost
            block = torch.cat([d["positions"], d["scales"].log(), d["rotations"][..., None],
                               torch.zeros_like(d["rotations"])[..., None], d["colors"]], -1)
            fit = GaussianImageFit(block, O.smooth_noise_target(H, W, seed=1002).to(dev), d["x_grid"], d["y_grid"],
                                   lr=min(0.05 * 4096 / N, 0.03))
            fit.capture()
            fit.set_lr(0.0)   # every kernel of the iteration runs, the Gaussians stay those the pair columns count
            rows.append((cfg + " fit step", B, N, H, W, C, nan, timeit(fit.step, n), ev_f, ev_b, nan))
    print("%-12s %3s %6s %4s %4s %3s %9s %11s %11s %10s %10s %9s %9s %10s" % (
        "config", "B", "N", "H", "W", "C", "fwd ms", "fwd+bwd ms", "pairs/s", "fwd pairs", "bwd pairs", "evaluated",
        "of peak", "CPU f+b s"))
    for cfg, B, N, H, W, C, tf, t, ev_f, ev_b, cpu_s in rows:
        pairs = B * N * H * W
        ev_f = pairs if ev_f is None else ev_f   # (forward lists not read back: counted in full)
        flop = ev_f * (12 + 2 * C) + ev_b * (30 + 4 * C)
        print("%-12s %3d %6d %4d %4d %3d %9.3f %11.3f %11.3e %10.3e %10.3e %8.1f%% %9.2f %10.2f" % (
            cfg, B, N, H, W, C, tf * 1e3, t * 1e3, pairs / t, ev_f, ev_b, 100.0 * (ev_f + ev_b) / (2 * pairs),
            flop / t / 1e12 / FP32_VECTOR_PEAK_TFLOPS, cpu_s))
    model, physical = host_cpu()
    print("pairs/s counts all B N H W pairs; of peak = (12 + 2 C) x forward pairs + (30 + 4 C) x backward pairs evaluated "
          "/ fwd+bwd time / %.1f TFLOP/s; CPU: %d torch threads on %s (%d "
          "physical cores visible)" % (FP32_VECTOR_PEAK_TFLOPS, torch.get_num_threads(), model, physical))
    return 0


def fit_step(cfg: str, steps: int, warmup: int) -> int:
    """The fused fit iteration of the reference's image-fitting script (scripts/2dgs_img_comp.py:186-240: render, MSE
    against the target, backward, AdamW on one parameter block) on the Gaussians of `cfg`, captured once and replayed
    from a HIP graph: `warmup` replays and at least 0.3 s of them, then `steps` replays between two synchronisations,
    at learning rate 0 so that every replay sees the same Gaussians."""
    import torch

    from igs_amd.fit import GaussianImageFit
    from oracle import gs2d_oracle as O

    if cfg not in ("c0", "c2"):
        print("bench.py --fit: one image per fit (c0 or c2)", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    d = {k: v.to(dev) for k, v in O.make_config_inputs(cfg).items()}
    B, N, C = d["colors"].shape
    H, W = d["x_grid"].shape[-2:]
    xg = d["x_grid"][:1, :, :1, :].expand(B, 1, H, W)
    yg = d["y_grid"][:1, :, :, :1].expand(B, 1, H, W)
    block = torch.cat([d["positions"], d["scales"].log(), d["rotations"][..., None],
                       torch.zeros_like(d["rotations"])[..., None], d["colors"]], -1)
    fit = GaussianImageFit(block, O.smooth_noise_target(H, W, seed=1002).to(dev), xg, yg, lr=min(0.05 * 4096 / N, 0.03))
    fit.capture()
    # learning rate 0 (read from device memory by the captured AdamW kernel): all kernels of the iteration run, but
    # the Gaussians stay the configuration's.  With the script's rate they shrink towards the smooth target within a
    # few hundred iterations, the lists get three times shorter, and the timed step is no longer this workload.
    fit.set_lr(0.0)
    t0 = time.perf_counter()
    k = 0
    while k < warmup or time.perf_counter() - t0 < 0.3:
        fit.step()
        k += 1
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fit.step()
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / steps
    pairs = B * N * H * W
    # The configuration's own protocol for a fit (c2): 100 iterations from the initial Gaussians at the script's
    # learning rate, losses at iterations 0 / 10 / 100.  The scene changes while it runs (the lists get shorter), so
    # this is the time of that loop, not of the step above.
    fit = GaussianImageFit(block, O.smooth_noise_target(H, W, seed=1002).to(dev), xg, yg, lr=min(0.05 * 4096 / N, 0.03))
    fit.capture()
    losses = {}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(101):
        loss = fit.step()
        if i in (0, 10, 100):
            losses[str(i)] = float(loss)     # (synchronises: three times in the loop)
    torch.cuda.synchronize()
    t_loop = time.perf_counter() - t0
    print(json.dumps({"metric": "fit_step_ms", "value": t * 1e3, "unit": "ms", "higher_is_better": False, "n_gpus": 1,
                      "loop": {"iterations": 101, "ms_total": t_loop * 1e3, "ms_per_iteration": t_loop * 1e3 / 101,
                               "pairs_per_s": pairs * 101 / t_loop, "loss": losses,
                               "what": "101 iterations from the initial Gaussians at the script's learning rate (the loss "
                                       "returned by iteration i is that of the image before its update)"},
                      "steps": steps, "warmup": warmup, "pairs_per_s": pairs / t, "dtype": "f32", "data": "synthetic",
                      "config": {"workload": f"{cfg}: fit iteration (render + MSE + backward + AdamW), HIP graph replay, "
                                             f"B={B} N={N} {H}x{W} C={C}", "B": B, "N": N, "H": H, "W": W, "C": C}}),
          flush=True)
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
