"""Seeded random problem shapes through the public API: what the tile lists leave out.

Each case runs `gaussian_splatting_2d` forward + backward with the default skip tolerance, with
skip tolerance 0 (exact zeros only) and with every Gaussian listed for every tile (IGS_OPT_NO_CULL),
and a forward without gradients (which bins for itself where the step with gradients shares one set
of tile lists between both passes).  Shapes are drawn so that odd image sizes, one or several
forward splits, one list or four per tile, shared and separate lists and both binning depths occur.
The fp64 oracle covers the same API at fixed shapes in test_gpu_parity.py / test_gpu_bench_plans.py;
here the reference point is the run that skips nothing, which a shape of any size can afford.
"""
import random

import pytest
import torch

from oracle import gs2d_oracle as O

pytestmark = pytest.mark.gpu
NAMES = ("positions", "colors", "scales", "rotations", "alphas")


def _cases():
    rng = random.Random(20)
    out = []
    while len(out) < 14:
        B = rng.choice([1, 2, 4, 8, 16, 33])
        N = rng.choice([300, 2000, 5000, 9000, 20000, 50000])
        H = rng.choice([33, 64, 96, 100, 128, 200, 256])
        W = rng.choice([31, 64, 96, 130, 160, 256])
        C = rng.choice([1, 3, 3, 5, 8, 16])
        scales = rng.choice([(0.004, 0.04), (0.02, 0.3), (0.002, 0.02), (0.01, 0.1)])
        if B * N * H * W > 1.5e10 or B * N * (H // 32 + 1) * (W // 32 + 1) * (6 + C) * 4 > 4e9:
            continue
        out.append((B, N, H, W, C, scales))
    # large enough for the backward's tiles to be the forward's wave rectangles (one set of lists for
    # both passes), with a last band of fewer rows / a last column of fewer pixels
    out += [(16, 5000, 200, 130, 3, (0.01, 0.1)), (4, 20000, 100, 260, 1, (0.004, 0.04)),
            (3, 30000, 200, 96, 16, (0.002, 0.02)), (1, 140000, 130, 100, 3, (0.002, 0.02))]
    return out


@pytest.mark.parametrize("case", _cases(), ids=lambda c: "B%d-N%d-%dx%d-C%d-s%g" % (*c[:5], c[5][1]))
def test_default_and_exact_lists_against_listing_everything(case):
    import igs_amd
    from igs_amd import _lib
    from igs_amd._splat import SKIP_TOLERANCE, library_options, padded_channels

    if not torch.cuda.is_available():
        pytest.skip("needs the GPU")
    dev = torch.device("cuda:0")
    B, N, H, W, C, (smin, smax) = case
    d = O.make_inputs(B, N, H, W, C, smin, smax, seed=N + H + W, dtype=torch.float32)
    g = {k: v.to(dev) for k, v in d.items()}
    plan = _lib.plan(B, N, H, W, padded_channels(C), 1)
    print(f"lists_shared={plan.lists_shared} fwd_split={plan.fwd_split} bwd_tiles={plan.bwd_tiles}", flush=True)
    if (B, N, H, W) in ((16, 5000, 200, 130), (4, 20000, 100, 260), (3, 30000, 200, 96), (1, 140000, 130, 100)):
        assert plan.lists_shared == 1

    def run(grad=True):
        lv = {k: g[k].clone().requires_grad_(grad) for k in NAMES}
        out = igs_amd.gaussian_splatting_2d(*(lv[k] for k in NAMES), g["x_grid"], g["y_grid"])
        if grad:
            out.backward(g["grad_out"])
        return out.detach(), {k: lv[k].grad for k in NAMES}

    out, grads = run()
    out_nograd, _ = run(grad=False)
    with library_options(no_cull=True):
        out0, grads0 = run()
    with library_options(skip_tolerance=0.0):
        oute, gradse = run()
    cmax = float(g["colors"].abs().max())
    assert float(out0.abs().max()) > 0 and bool(torch.isfinite(out0).all())
    # the bound of the default tolerance, plus the fp32 rounding of sums that are grouped differently
    for o in (out, out_nograd):
        assert float((o - out0).abs().max()) <= SKIP_TOLERANCE * cmax + 1e-6
    assert float((oute - out0).abs().max()) <= 2e-6
    for k in NAMES:
        n0 = float(grads0[k].double().norm())
        assert float((grads[k] - grads0[k]).double().norm()) <= 1e-5 * n0, k
        assert float((gradse[k] - grads0[k]).double().norm()) <= 1e-5 * n0, k
