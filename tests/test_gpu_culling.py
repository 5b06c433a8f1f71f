"""Culling on separable grids: a Gaussian is skipped for a pixel tile when its reach box misses the
tile or its ellipse does not reach the tile's rectangle.  Two claims are under test.  With a skip
weight of 0 (`library_options(skip_tolerance=0)`; the box bounds q <= 221.8, beyond which exp2 of
the kernels' exponent is exactly 0) only exact zeros are dropped: with IGS_OPT_NO_CULL the library
lists everything, and both runs must agree exactly (one forward split) or to fp32 rounding (several,
where the grouping of the terms changes).  With the default skip tolerance only pairs below the
skip weight are dropped: the run stays within the stated bound of the run that lists everything.
Beside that: sparse scenes against the fp64 oracle, non-finite parameters, grids whose coordinates
are not monotone, and the boxes and tile lists themselves against the oracle's restatement."""
import os

import pytest
import torch

from oracle import gs2d_oracle as O

pytestmark = pytest.mark.gpu
NAMES = ("positions", "colors", "scales", "rotations", "alphas")


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def igs():
    import igs_amd

    return igs_amd


def sparse_case(dev, B, N, H, W, C, seed, smin=0.004, smax=0.04, dtype=torch.float32):
    d = O.make_inputs(B, N, H, W, C, smin, smax, seed=seed, dtype=torch.float64, expand_grids=True)
    g = {k: v.to(dev, dtype) for k, v in d.items()}
    g["x_grid"] = g["x_grid"][:1, :, :1, :].expand(B, 1, H, W)
    g["y_grid"] = g["y_grid"][:1, :, :, :1].expand(B, 1, H, W)
    return d, g


def run(igs, g, x=None, y=None):
    leaves = {k: g[k].clone().requires_grad_(True) for k in NAMES}
    out = igs.gaussian_splatting_2d(*(leaves[k] for k in NAMES), g["x_grid"] if x is None else x,
                                    g["y_grid"] if y is None else y)
    out.backward(g["grad_out"])
    return out.detach(), {k: v.grad for k, v in leaves.items()}


@pytest.fixture
def no_cull():
    """Context in which the library lists every Gaussian for every tile (IGS_OPT_NO_CULL)."""
    from igs_amd._splat import library_options

    class Ctx:  # re-enterable: a fresh context per `with`
        def __enter__(self):
            self.ctx = library_options(no_cull=True)
            return self.ctx.__enter__()

        def __exit__(self, *a):
            return self.ctx.__exit__(*a)

    return Ctx()


def exact():
    """Context in which only pairs whose weight is exactly zero are skipped (skip weight 0)."""
    from igs_amd._splat import library_options

    return library_options(skip_tolerance=0.0)


@pytest.mark.parametrize("shape", [(2, 120, 70, 150, 3), (1, 100, 200, 64, 16), (3, 64, 33, 257, 1)],
                         ids=lambda s: "x".join(map(str, s)))
def test_culled_equals_unculled_bit_for_bit(igs, dev, no_cull, shape):
    """N < 128 keeps the forward in one Gaussian split, so that both runs add the same terms in
    the same order and the skipped ones are exact zeros."""
    B, N, H, W, C = shape
    _, g = sparse_case(dev, B, N, H, W, C, seed=sum(shape))
    with exact():
        out, grads = run(igs, g)
    with no_cull:
        out0, grads0 = run(igs, g)
    assert float(out.abs().max()) > 0
    assert torch.equal(out, out0)
    for k in NAMES:
        assert torch.equal(grads[k], grads0[k]), k


def test_long_rotated_gaussians_bit_for_bit(igs, dev, no_cull):
    """Aspect ratios up to 100 at random angles: the reach boxes are mostly empty and the second,
    ellipse-against-tile test of the binning decides; it must drop exact zeros only."""
    B, N, H, W, C = 2, 120, 192, 320, 3
    _, g = sparse_case(dev, B, N, H, W, C, seed=77, smin=0.002, smax=0.2)
    with exact():
        out, grads = run(igs, g)
    with no_cull:
        out0, grads0 = run(igs, g)
    assert float(out.abs().max()) > 0
    assert torch.equal(out, out0)
    for k in NAMES:
        assert torch.equal(grads[k], grads0[k]), k


def _Env(name, value):
    """The one- or two-level construction of the tile lists, forced (IGS_OPT_BIN_LEVELS_1 | _2)."""
    from igs_amd._splat import library_options

    assert name == "IGS_BIN_LEVELS"
    return library_options(bin_levels=int(value))


def _kernel_channels(C):
    from igs_amd import _lib

    return next(c for c in _lib.COMPILED_CHANNELS if c >= C)


@pytest.mark.parametrize("shape,scales", [((2, 700, 256, 512, 3), (0.004, 0.04)), ((1, 1500, 384, 640, 16), (0.005, 0.05)),
                                          ((3, 333, 200, 530, 1), (0.004, 0.1)), ((1, 70000, 256, 512, 3), (0.002, 0.01)),
                                          ((1, 9000, 520, 1000, 3), (0.002, 0.02)), ((2, 20000, 256, 512, 3), (0.002, 0.01))],
                         ids=lambda v: "x".join(map(str, v)))
def test_two_level_binning(igs, dev, shape, scales):
    """IGS_OPT_BIN_LEVELS_2 lists the Gaussians per super-tile (4 x 4 tiles, several workgroups per
    super-tile, each filling its own segment) first and lets every tile scan those segments only.
    With only exact zeros skipped the tile lists are the same as with one level, hence the forward bit
    for bit; the finalize kernel then adds the tiles super-tile by super-tile, so the gradients agree
    to rounding.  With the default tolerance a tile settles what it skips from the candidates it sees
    (and a small forward bins per wave rectangle with one level, per tile with two), so the lists may
    differ and the images agree within the tolerance's bound."""
    from igs_amd import _lib

    B, N, H, W, C = shape
    plan = _lib.plan(B, N, H, W, _kernel_channels(C), 1)
    assert plan.fwd_tiles >= 32 and plan.bwd_tiles >= 32          # both launches have super-tiles
    _, g = sparse_case(dev, B, N, H, W, C, seed=sum(shape), smin=scales[0], smax=scales[1])
    with _Env("IGS_BIN_LEVELS", "1"):
        out1d, _ = run(igs, g)
    with _Env("IGS_BIN_LEVELS", "2"):
        out2d, _ = run(igs, g)
    cmax = float(g["colors"].abs().max())
    assert float((out1d - out2d).abs().max()) <= 2e-7 * cmax + 1e-6
    with exact():
        with _Env("IGS_BIN_LEVELS", "1"):
            out1, grads1 = run(igs, g)
        with _Env("IGS_BIN_LEVELS", "2"):
            out2, grads2 = run(igs, g)
            out3, grads3 = run(igs, g)
    assert float(out1.abs().max()) > 0
    assert torch.equal(out1, out2)
    for k in NAMES:
        assert float(grads1[k].abs().max()) > 0
        d = (grads1[k] - grads2[k]).double()
        assert float(d.norm()) <= 1e-5 * float(grads1[k].double().norm()), k   # another order of the tile sums
        assert torch.equal(grads2[k], grads3[k]), k                # reproducible run to run


def test_two_level_binning_on_materialised_grids(igs, dev):
    """Grids stored in full are classified on the device and both kernel variants are enqueued
    behind the flag; the two binning passes are gated like the kernels they serve."""
    B, N, H, W, C = 2, 9000, 256, 512, 3
    _, g = sparse_case(dev, B, N, H, W, C, seed=12, smin=0.003, smax=0.03)
    xg, yg = g["x_grid"].contiguous(), g["y_grid"].contiguous()
    with _Env("IGS_BIN_LEVELS", "2"):
        out_e, grads_e = run(igs, g)
        out_m, grads_m = run(igs, g, xg, yg)
    assert torch.equal(out_e, out_m)
    for k in NAMES:
        assert torch.equal(grads_e[k], grads_m[k]), k


def test_two_level_setting_on_a_general_grid(igs, dev):
    """A stored grid that is not separable runs the general backward (dense partials, no slot
    tables) whatever the binning setting; the finalize kernel of the two-level setting must then
    read them as such.  Function level, operator level and the module head."""
    B, N, H, W, C = 2, 900, 128, 256, 3
    _, g = sparse_case(dev, B, N, H, W, C, seed=19, smin=0.01, smax=0.1)
    xg = (g["x_grid"] + 0.01 * torch.sin(7 * g["y_grid"])).contiguous()
    yg = g["y_grid"].contiguous()
    res = []
    for lv in ("1", "2"):
        with _Env("IGS_BIN_LEVELS", lv):
            out, grads = run(igs, g, xg, yg)
            pos = g["positions"].clone().requires_grad_(True)
            torch.manual_seed(3)
            cov = [torch.rand(B, N, 1, 1, device=dev).mul_(m).add_(a).requires_grad_(True)
                   for m, a in ((300, 100), (40, -20), (300, 100))]   # positive definite forms
            al, col = g["alphas"].clone().requires_grad_(True), g["colors"].clone().requires_grad_(True)
            igs.GaussianSplatting2DKernel.apply(xg, yg, pos, *cov, al, col).backward(g["grad_out"])
            torch.manual_seed(5)
            m = igs.GaussianSplatting2D(8, 64).to(dev)
            x = torch.randn(B, 100, 64, device=dev, requires_grad=True)
            grid = torch.cat([yg, xg], dim=1)
            m(x, grid=grid)[0].backward(g["grad_out"])
            res.append((out, *grads.values(), pos.grad, *(c.grad for c in cov), al.grad, col.grad, x.grad))
    for a, b in zip(*res):
        assert float(a.abs().max()) > 0
        assert float((a - b).double().norm()) <= 1e-5 * float(a.double().norm())


def test_two_level_binning_against_oracle(igs, dev):
    """Long thin Gaussians (aspect ratios up to 40) under two levels against the fp64 oracle."""
    B, N, H, W, C = 1, 300, 256, 512, 3
    d, g = sparse_case(dev, B, N, H, W, C, seed=41, smin=0.005, smax=0.2)
    ref_out, ref_g = O.render_autograd(d["positions"], d["colors"], d["scales"], d["rotations"], d["alphas"],
                                       d["x_grid"], d["y_grid"], d["grad_out"])
    with _Env("IGS_BIN_LEVELS", "2"):
        out, grads = run(igs, g)
    err = (out.double() - ref_out.to(dev)).abs()
    assert bool((err <= 1e-6 + 1e-5 * ref_out.to(dev).abs()).all()), float(err.max())
    for k in NAMES:
        r = ref_g[k].to(dev)
        dlt = grads[k].double() - r
        assert float(dlt.abs().max()) <= 1e-4 * float(r.abs().max()), k
        assert float(dlt.norm()) <= 1e-4 * float(r.norm()), k


def test_two_level_binning_culled_equals_unculled(igs, dev, no_cull):
    """Under two levels, too, culling drops exact zeros only (one forward split: N < 128)."""
    B, N, H, W, C = 2, 120, 256, 512, 3
    _, g = sparse_case(dev, B, N, H, W, C, seed=21, smin=0.002, smax=0.2)
    with _Env("IGS_BIN_LEVELS", "2"):
        with exact():
            out, grads = run(igs, g)
        with no_cull:
            out0, grads0 = run(igs, g)
    assert torch.equal(out, out0)
    for k in NAMES:
        assert torch.equal(grads[k], grads0[k]), k


def test_two_level_binning_module_and_nan_tiles(igs, dev):
    """The module path (feature parameterisation) and a grid with a NaN coordinate (its tiles list
    everything at both levels) under both settings."""
    torch.manual_seed(5)
    m = igs.GaussianSplatting2D(8, 64).to(dev)
    x = torch.randn(2, 100, 64, device=dev)
    go = torch.randn(2, 3, 256, 512, device=dev)
    res = []
    for lv in ("1", "2"):
        with _Env("IGS_BIN_LEVELS", lv), exact():
            xx = x.clone().requires_grad_(True)
            img, _ = m(xx, size=(256, 512))
            img.backward(go)
            res.append((img.detach(), xx.grad.clone(), m.proj.weight.grad.clone()))
            m.zero_grad()
    assert torch.equal(res[0][0], res[1][0])
    for a, b in zip(res[0][1:], res[1][1:]):
        assert float((a - b).norm()) <= 1e-5 * float(a.norm())
    _, g = sparse_case(dev, 1, 300, 256, 512, 3, seed=3)
    xs = g["x_grid"][0, 0, 0, :].clone()
    xs[100] = float("nan")
    xg = xs.view(1, 1, 1, -1).expand(1, 1, 256, 512)
    outs = []
    for lv in ("1", "2"):
        with _Env("IGS_BIN_LEVELS", lv), exact():
            outs.append(run(igs, g, xg, None))
    assert torch.equal(torch.nan_to_num(outs[0][0], nan=7.0), torch.nan_to_num(outs[1][0], nan=7.0))
    for k in NAMES:   # NaN in the same places, the rest to rounding
        a, b = outs[0][1][k], outs[1][1][k]
        assert torch.equal(torch.isnan(a), torch.isnan(b)), k
        a, b = torch.nan_to_num(a, nan=0.0), torch.nan_to_num(b, nan=0.0)
        assert float((a - b).norm()) <= 1e-5 * float(a.norm()) + 1e-30, k


def test_culled_equals_unculled_with_several_forward_splits(igs, dev, no_cull):
    """With S > 1 forward splits a tile's list (not the index range) is cut into S parts, so the
    same terms are grouped into other partial sums: equal to fp32 rounding, not bit for bit."""
    from igs_amd import _lib

    B, N, H, W, C = 1, 3000, 96, 160, 3
    assert _lib.plan(B, N, H, W, C, 1).fwd_split > 1
    _, g = sparse_case(dev, B, N, H, W, C, seed=5)
    with exact():
        out, grads = run(igs, g)
    with no_cull:
        out0, grads0 = run(igs, g)
    torch.testing.assert_close(out, out0, rtol=0, atol=1e-6)
    for k in NAMES:
        d = (grads[k] - grads0[k]).double()
        assert float(d.norm()) <= 1e-6 * float(grads0[k].double().norm()), k


def test_sparse_scene_against_oracle(igs, dev):
    """Small Gaussians (sigma of 1-10 pixels) on a 96x160 image, several tiles in both directions,
    more than one forward split: forward and every gradient against the fp64 oracle."""
    B, N, H, W, C = 2, 700, 96, 160, 3
    d, g = sparse_case(dev, B, N, H, W, C, seed=31, smin=0.01, smax=0.1)
    ref_out, ref_g = O.render_autograd(d["positions"], d["colors"], d["scales"], d["rotations"], d["alphas"],
                                       d["x_grid"], d["y_grid"], d["grad_out"])
    out, grads = run(igs, g)
    err = (out.double() - ref_out.to(dev)).abs()
    assert bool((err <= 1e-6 + 1e-5 * ref_out.to(dev).abs()).all()), float(err.max())
    for k in NAMES:
        r = ref_g[k].to(dev)
        dlt = grads[k].double() - r
        assert float(dlt.abs().max()) <= 1e-4 * float(r.abs().max()), k
        assert float(dlt.norm()) <= 1e-4 * float(r.norm()), k


def test_non_monotone_separable_grid(igs, dev, no_cull):
    """A separable grid need not be sorted: tiles take [min, max] of their coordinates.  Permuting
    the columns and rows of the grid permutes the image, and culling still changes no bit."""
    B, N, H, W, C = 1, 90, 80, 140, 3
    _, g = sparse_case(dev, B, N, H, W, C, seed=8)
    gen = torch.Generator().manual_seed(3)
    pc, pr = torch.randperm(W, generator=gen).to(dev), torch.randperm(H, generator=gen).to(dev)
    xs = g["x_grid"][0, 0, 0, :][pc].contiguous()
    ys = g["y_grid"][0, 0, :, 0][pr].contiguous()
    xg = xs.view(1, 1, 1, W).expand(B, 1, H, W)
    yg = ys.view(1, 1, H, 1).expand(B, 1, H, W)
    g2 = dict(g)
    g2["grad_out"] = g["grad_out"][:, :, pr][:, :, :, pc].contiguous()
    with exact():
        out, grads = run(igs, g2, xg, yg)
    with no_cull:
        out0, grads0 = run(igs, g2, xg, yg)
    assert torch.equal(out, out0)
    for k in NAMES:
        assert torch.equal(grads[k], grads0[k]), k
    base, base_g = run(igs, g)
    # Both against the fp64 oracle on the same fp32 inputs, at the forward's bound.  (Between themselves
    # the two images agree less closely than each does with the oracle's on a regular grid: where a
    # tile's coordinates jump, the kernels evaluate the exponent term by term instead of through the
    # completed square, and the two forms round the coefficients of these thin ellipses, aspect ratios
    # up to 10, differently: up to 6e-8 x the largest term, which is 100 x the exponent here.)
    g64 = {k: g[k].double().cpu() for k in NAMES}
    for image, xs64, ys64 in ((base, g["x_grid"], g["y_grid"]), (out, xg, yg)):
        ref, _ = O.render_autograd(g64["positions"], g64["colors"], g64["scales"], g64["rotations"], g64["alphas"],
                                   xs64.double().cpu().contiguous(), ys64.double().cpu().contiguous(),
                                   torch.zeros(B, C, H, W, dtype=torch.float64))
        err = (image.double().cpu() - ref).abs()
        assert bool((err <= 1e-6 + 1e-5 * ref.abs()).all()), float((err - 1e-5 * ref.abs()).max())
    torch.testing.assert_close(out, base[:, :, pr][:, :, :, pc], rtol=1e-4, atol=1e-5)
    for k in NAMES:   # the same sums in another pixel order (and, where coordinates jump, with more rounding in the completed square)
        torch.testing.assert_close(grads[k], base_g[k], rtol=2e-4, atol=1e-5 * float(base_g[k].abs().max()))


def test_non_finite_parameters_propagate_as_without_culling(igs, dev, no_cull):
    """A Gaussian with a NaN position or rotation or an infinite alpha poisons every pixel in the
    plain torch expression (NaN - x, 0 * inf), an infinite colour every pixel of its channel that
    the Gaussian's weight reaches or underflows at; the reach box of such a record is unbounded,
    so the fused result has its NaN/inf exactly where the run without culling has them."""
    B, N, H, W, C = 1, 40, 70, 130, 3
    _, g = sparse_case(dev, B, N, H, W, C, seed=12)
    for field, index, value, all_nan in (("positions", (0, 3, 0), float("nan"), True),
                                         ("alphas", (0, 5), float("inf"), True),
                                         ("colors", (0, 7, 1), float("inf"), False),
                                         ("rotations", (0, 9), float("nan"), True)):
        h = {k: v.clone() for k, v in g.items()}
        h[field][index] = value
        with torch.no_grad():
            with exact():
                got = igs.gaussian_splatting_2d(*(h[k] for k in NAMES), g["x_grid"], g["y_grid"])
            dflt = igs.gaussian_splatting_2d(*(h[k] for k in NAMES), g["x_grid"], g["y_grid"])
            with no_cull:
                ref = igs.gaussian_splatting_2d(*(h[k] for k in NAMES), g["x_grid"], g["y_grid"])
            want = igs.gaussian_splatting_2d(*(h[k] for k in NAMES), g["x_grid"], g["y_grid"], fused=False)
        assert torch.equal(torch.isnan(got), torch.isnan(ref)), field
        assert torch.equal(torch.nan_to_num(got, nan=7.0), torch.nan_to_num(ref, nan=7.0)), field
        # under the default skip weight such a record is never skipped either
        assert torch.equal(torch.isfinite(dflt), torch.isfinite(ref)), field
        fin = torch.isfinite(ref)
        torch.testing.assert_close(dflt[fin], ref[fin], rtol=1e-6, atol=2e-7)
        if all_nan:
            assert bool(torch.isnan(want).all()) and bool(torch.isnan(got).all()), field
        else:   # the other channels are untouched
            torch.testing.assert_close(got[:, [0, 2]], want[:, [0, 2]], rtol=1e-4, atol=1e-5)
            assert not bool(torch.isfinite(got[:, 1]).any())


def test_operator_level_with_indefinite_cov_inverse(igs, dev, no_cull):
    """cov_inv entries that are not positive definite (the operator accepts anything) grow instead
    of decaying: such a Gaussian is never culled."""
    B, N, H, W = 1, 30, 66, 130
    _, g = sparse_case(dev, B, N, H, W, 3, seed=4)
    with torch.no_grad():
        a, b, d = O.cov_inverse_closed(g["scales"].double(), g["rotations"].double())
    a, b, d = (t.float().reshape(B, N, 1, 1).contiguous() for t in (a, b, d))
    a[0, 2] = -1e-3          # saddle: exp(+...) along x
    d[0, 4] = 0.0            # degenerate: constant along y
    K = igs.GaussianSplatting2DKernel
    args = (g["x_grid"], g["y_grid"], g["positions"], a, b, d, g["alphas"], g["colors"])
    with torch.no_grad():
        with exact():
            out = K.apply(*args)
        dflt = K.apply(*args)
        with no_cull:
            out0 = K.apply(*args)
        want = igs.naive_gaussian_2d(g["x_grid"], g["y_grid"], g["positions"], a, b, d, g["alphas"], g["colors"])
    assert torch.equal(torch.isnan(dflt), torch.isnan(out0))
    fin = torch.isfinite(out0)
    torch.testing.assert_close(dflt[fin], out0[fin], rtol=1e-6, atol=2e-7)
    # the saddle overflows where it grows (inf / inf): same places, same values elsewhere
    assert torch.equal(torch.isnan(out), torch.isnan(out0))
    assert torch.equal(torch.nan_to_num(out, nan=7.0), torch.nan_to_num(out0, nan=7.0))
    ok = torch.isfinite(want) & torch.isfinite(out)
    assert float(ok.float().mean()) > 0.3
    torch.testing.assert_close(out[ok], want[ok], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("tolerance", [0.0, 1e-7, 1e-3], ids=lambda t: f"tol{t:g}")
def test_reach_boxes_of_the_pack_kernels_match_the_oracle(igs, dev, tolerance):
    """The boxes behind the packed records (scale/rotation, cov-inverse and module-feature
    packing) against the oracle's restatement, for the exact-zero limit and for two skip weights,
    with alphas on both sides of 1: never inside it, and no more than the stated outward rounding
    (1e-5 relative on the half extent) beyond it.  The skip limit itself sits behind the boxes."""
    import math

    from igs_amd._splat import Grid, Splat, _f32c, library_options

    B, N, C = 2, 257, 3
    d64, g = sparse_case(dev, B, N, 40, 72, C, seed=2, smin=0.003, smax=0.4)
    g["alphas"] = (g["alphas"] * 6).contiguous()                       # a third of them above 1
    grid = Grid(g["x_grid"], g["y_grid"], B)
    with library_options(skip_tolerance=tolerance):
        op = Splat(B, N, C, grid, 1e-6, dev)
    w = O.skip_weight(N, 1e-6, tolerance)
    assert op.skip_weight == pytest.approx((w, O.skip_weight(N, 1.0, tolerance)), rel=1e-6)
    a, b, dd = O.cov_inverse_closed(d64["scales"].float().double(), d64["rotations"].float().double())
    pos = d64["positions"].float().double()

    def boxes(packed):
        p = op.plan   # bin records (px, py, hx, hy | a, b2, d, alpha): the box is px -+ hx, py -+ hy
        q = packed[B * p.n_padded * p.rec_stride:][:B * p.n_padded * 8].view(B, p.n_padded, 8)
        return torch.stack([q[..., 0] - q[..., 2], q[..., 0] + q[..., 2], q[..., 1] - q[..., 3], q[..., 1] + q[..., 3]], -1)

    col = _f32c(g["colors"])
    cases = {"scale_rot": (op.pack_scale_rot(_f32c(g["positions"]), _f32c(g["scales"]), _f32c(g["rotations"]),
                                             _f32c(g["alphas"]), col), g["alphas"].cpu().double())}
    f = lambda t: t.to(dev, torch.float32).reshape(B, N).contiguous()
    cases["covinv"] = (op.pack_covinv(_f32c(g["positions"]), f(a), f(b), f(dd), _f32c(g["alphas"]), col),
                       g["alphas"].cpu().double())
    feat = torch.cat([g["positions"], (g["scales"] - 1e-6).log(), g["rotations"][..., None],
                      torch.zeros_like(g["rotations"])[..., None], g["colors"]], dim=-1).contiguous()
    cases["feature"] = (op.pack_feature(feat, None)[0], torch.ones(B, N, dtype=torch.float64))   # the module's alpha
    sign = torch.tensor([-1.0, 1.0, -1.0, 1.0], device=dev, dtype=torch.float64)
    for name, (packed, alphas) in cases.items():
        want = O.reach_box(pos, a, b, dd, O.reach_q(alphas, w)).to(dev)
        half = torch.stack([want[..., 1] - want[..., 0], want[..., 3] - want[..., 2]], -1).repeat_interleave(2, -1) / 2
        got = boxes(packed)[:, :N].double()
        out = (got - want) * sign                      # how far outside the exact box each edge lies
        # cov-inverse / feature inputs are fp32 roundings of the fp64 route: allow their error too
        slack = 1e-4 if name != "scale_rot" else 3e-5
        assert bool((out >= -slack * half).all()), (name, float((out / half).min()))
        assert bool((out <= slack * half + 1e-6).all()), (name, float((out / half).max()))
        pad = boxes(packed)[:, N:]
        assert bool((pad[..., 0] > pad[..., 1]).all())  # padding records: empty boxes
        limit, fraction = packed[B * op.plan.n_padded * (op.plan.rec_stride + 8):][:2].tolist()
        assert limit == pytest.approx(O.EXACT_LIMIT if w == 0 else min(O.EXACT_LIMIT, -math.log2(w)), rel=1e-6)
        assert fraction == pytest.approx(O.skip_weight(N, 1.0, tolerance), rel=1e-6)
    if tolerance > 0:    # smaller boxes than the exact-zero ones, by sqrt of the limits' ratio
        ratio = math.sqrt((-math.log2(w) + 5) / (O.EXACT_LIMIT + 5))
        exact_box = O.reach_box(pos, a, b, dd)
        got = boxes(cases["feature"][0])[:, :N].double().cpu()
        r = (got[..., 1] - got[..., 0]) / (exact_box[..., 1] - exact_box[..., 0])
        assert float((r - ratio).abs().max()) < 1e-4


def _tile_counts(op, packed, dev, with_lists=False):
    """Per-tile list lengths [B, tiles_y, tiles_x] of the separable backward for `packed` (read back
    from the workspace behind the pixel records, where the binning of the reduce call writes them),
    and on request the lists themselves [B, tiles_y, tiles_x, Np]."""
    from igs_amd import _lib
    from igs_amd._splat import _ptr

    g, p = op.grid, op.plan
    B, H, W = op.B, g.H, g.W
    pix = op._empty(p.pix_bytes)
    partial = op._empty(p.partial_bytes)
    out, den = op.forward(packed)
    go = torch.ones(B, op.Cp, H, W, device=dev)
    col = torch.zeros(B, op.N, op.Cp, device=dev)
    _lib.check(op.lib.igs_gs2d_backward(_ptr(packed), _ptr(col), _ptr(g.x), _ptr(g.y), g.strides, g.mode, _ptr(g.flag),
                                        _ptr(out), _ptr(den), _ptr(go), B, op.N, H, W, op.Cp, op.eps, _ptr(pix),
                                        int(p.pix_bytes), _ptr(partial), int(p.partial_bytes), op.stream), "backward")
    scratch = (B * H * p.w_padded * p.pix_stride + B * p.w_padded) * 4
    ints = pix.view(torch.int32)[(scratch + 15) // 16 * 4:]
    counts = ints[: B * p.bwd_tiles].view(B, -1, p.bwd_tiles_x).cpu()
    if not with_lists:
        return counts
    lists = ints[(B * p.bwd_tiles + 3) // 4 * 4:][: B * p.bwd_tiles * p.n_padded]
    return counts, lists.view(B, counts.shape[1], p.bwd_tiles_x, p.n_padded).cpu()


@pytest.mark.parametrize("tolerance,scales,alpha_scale", [(1e-7, (0.004, 0.15), 3.0), (1e-7, (0.03, 0.3), 3.0),
                                                          (1e-3, (0.03, 0.3), 0.5)],
                         ids=["default-sparse", "default-dense", "loose-dense"])
def test_tile_lists_against_the_oracle_s_allowance(igs, dev, tolerance, scales, alpha_scale):
    """What the binning leaves out of each backward tile's list against the oracle's statement of the
    rule (`tile_first_skipped_class`), from both sides.  Safety: the largest terms (fp64 maxima over
    the tile's rectangle, `min_q_over_rect`) of the Gaussians that are not listed sum to at most
    N (w + f S), S the tile's denominator floor -- the premise of the error bound.  Effect: the list
    is at most one weight class longer than the oracle's own for an allowance cut by 5 % and with
    every Gaussian moved towards the heavy side by the kernel's rounding margin (4e-6 of the largest
    term of the form over the rectangle), so a rule that skips too little fails as well."""
    from igs_amd._splat import Grid, Splat, _f32c, library_options

    B, N, H, W, C = 2, 900, 96, 200, 3
    d64, g = sparse_case(dev, B, N, H, W, C, seed=19, smin=scales[0], smax=scales[1])
    g["alphas"] = (g["alphas"] * alpha_scale).contiguous()
    with library_options(skip_tolerance=tolerance):
        op = Splat(B, N, C, Grid(g["x_grid"], g["y_grid"], B), 1e-6, dev)
    packed = op.pack_scale_rot(_f32c(g["positions"]), _f32c(g["scales"]), _f32c(g["rotations"]), _f32c(g["alphas"]),
                               _f32c(g["colors"]))
    counts, lists = _tile_counts(op, packed, dev, with_lists=True)
    p = op.plan
    a, b, dd = (t.reshape(B, N) for t in O.cov_inverse_closed(d64["scales"].float().double(),
                                                               d64["rotations"].float().double()))
    pos = d64["positions"].float().double()
    al = g["alphas"].cpu().double()
    w, f = O.skip_weight(N, 1e-6, tolerance), O.skip_weight(N, 1.0, tolerance)
    xs, ys = g["x_grid"][0, 0, 0, :].cpu().double(), g["y_grid"][0, 0, :, 0].cpu().double()
    k = 0.5 * 1.4426950408889634
    beyond_w = 0      # Gaussians left out although their largest term on the tile exceeds the call's skip weight
    used = []
    for ty in range(counts.shape[1]):
        for tx in range(counts.shape[2]):
            r0, r1 = ty * p.bwd_per_tile, min(H, (ty + 1) * p.bwd_per_tile)
            c0, c1 = tx * p.bwd_tile_w, min(W, (tx + 1) * p.bwd_tile_w)
            rect = (xs[c0], xs[c1 - 1], ys[r0], ys[r1 - 1])
            mq = O.min_q_over_rect(pos[..., 0], pos[..., 1], a, b, dd, *rect)
            S = O.tile_weight_floor(pos[..., 0], pos[..., 1], a, b, dd, al, *rect)
            mx = torch.maximum((rect[0] - pos[..., 0]).abs(), (rect[1] - pos[..., 0]).abs())
            my = torch.maximum((rect[2] - pos[..., 1]).abs(), (rect[3] - pos[..., 1]).abs())
            T = a * mx * mx + 2 * b.abs() * mx * my + dd * my * my                # in units of q
            for i in range(B):
                n = int(counts[i, ty, tx])
                listed = torch.zeros(N, dtype=torch.bool)
                listed[lists[i, ty, tx, :n].long()] = True
                assert int(listed.sum()) == n
                term = torch.clamp(al[i].abs(), min=1.0) * torch.exp(-0.5 * mq[i])
                allowance = N * float(O.tile_skip_weight(w, f, S[i]))
                assert float(term[~listed].sum()) <= allowance, (ty, tx, i)
                used.append(float(term[~listed].sum()) / allowance)
                beyond_w += int((term[~listed] > w).sum())
                heavy = O.weight_class(torch.clamp(mq[i] - 5e-6 * T[i] - 2e-3, min=1e-30), al[i])
                first = O.tile_first_skipped_class(heavy, N, w, f, 0.95 * float(S[i]))
                may = int(((heavy < first + 1) | (mq[i] - 5e-6 * T[i] - 2e-3 <= 0)).sum())
                assert n <= may, (ty, tx, i, n, may)
    assert beyond_w > 0 and max(used) > 0.3


@pytest.mark.parametrize("tolerance,scales", [(0.0, (0.004, 0.15))], ids=["exact-sparse"])
def test_tile_lists_against_the_oracle_s_rectangle_minimum(igs, dev, tolerance, scales):
    """What the binning lists for each backward tile against the oracle: a Gaussian whose minimum
    of -q' over the tile's coordinate rectangle (`min_q_over_rect`) is below its skip limit must be
    listed; one whose minimum is beyond the limit by more than the kernel's rounding allowance must
    not (aspect ratios stay far below the 1:600 beyond which the kernel lists an ellipse anyway).
    The limit of a tile comes from the call's skip weight plus the skip fraction of the tile's
    denominator floor (`tile_weight_floor`; the kernel rounds its floor down by 1e-3 and sums only
    the Gaussians whose box meets the tile, which differ by less than that).
    Counted per tile: must <= listed <= may."""
    from igs_amd._splat import Grid, Splat, _f32c, library_options

    B, N, H, W, C = 2, 900, 96, 200, 3
    d64, g = sparse_case(dev, B, N, H, W, C, seed=19, smin=scales[0], smax=scales[1])
    g["alphas"] = (g["alphas"] * 3).contiguous()
    with library_options(skip_tolerance=tolerance):
        op = Splat(B, N, C, Grid(g["x_grid"], g["y_grid"], B), 1e-6, dev)
    packed = op.pack_scale_rot(_f32c(g["positions"]), _f32c(g["scales"]), _f32c(g["rotations"]), _f32c(g["alphas"]),
                               _f32c(g["colors"]))
    counts = _tile_counts(op, packed, dev)
    p = op.plan
    a, b, dd = (t.reshape(B, N) for t in O.cov_inverse_closed(d64["scales"].float().double(),
                                                               d64["rotations"].float().double()))
    pos = d64["positions"].float().double()
    al = g["alphas"].cpu().double()
    w, f = O.skip_weight(N, 1e-6, tolerance), O.skip_weight(N, 1.0, tolerance)
    xs, ys = g["x_grid"][0, 0, 0, :].cpu().double(), g["y_grid"][0, 0, :, 0].cpu().double()
    k = 0.5 * 1.4426950408889634
    saw_less = False
    floors = []
    for ty in range(counts.shape[1]):
        for tx in range(counts.shape[2]):
            r0, r1 = ty * p.bwd_per_tile, min(H, (ty + 1) * p.bwd_per_tile)
            c0, c1 = tx * p.bwd_tile_w, min(W, (tx + 1) * p.bwd_tile_w)
            m = k * O.min_q_over_rect(pos[..., 0], pos[..., 1], a, b, dd, xs[c0], xs[c1 - 1], ys[r0], ys[r1 - 1])
            S = O.tile_weight_floor(pos[..., 0], pos[..., 1], a, b, dd, al, xs[c0], xs[c1 - 1], ys[r0], ys[r1 - 1])
            floors.append(S)
            lim_lo = torch.stack([O.skip_limit(al[i], float(O.tile_skip_weight(w, f, S[i]))) for i in range(B)])
            lim_hi = torch.stack([O.skip_limit(al[i], float(O.tile_skip_weight(w, f, 0.997 * S[i]))) for i in range(B)])
            # the kernel's allowance for the fp32 rounding of its own evaluation: 4e-6 of the largest
            # term of the form over the rectangle (here with a little room for its rounding)
            mx = torch.maximum((xs[c0] - pos[..., 0]).abs(), (xs[c1 - 1] - pos[..., 0]).abs())
            my = torch.maximum((ys[r0] - pos[..., 1]).abs(), (ys[r1 - 1] - pos[..., 1]).abs())
            T = k * (a * mx * mx + 2 * b.abs() * mx * my + dd * my * my)
            must = (m <= lim_lo * (1 - 1e-4)).sum(1)
            may = (m - 5e-6 * T <= lim_hi * (1 + 1e-4) + 1e-3).sum(1)
            got = counts[:, ty, tx]
            assert bool((must <= got).all()) and bool((got <= may).all()), (ty, tx, must, got, may)
            saw_less = saw_less or bool((got < N).any())
    assert saw_less
    if scales[0] > 0.01:    # the scene is dense enough for the floors to matter: they beat the call's weight
        assert float(torch.stack(floors).median()) * f > 10 * w


@pytest.mark.parametrize("alpha_scale", [1.0, 25.0, 1e30])
def test_default_skip_tolerance_stays_within_its_bound(igs, dev, alpha_scale):
    """The default skip weight against the run that lists every Gaussian for every tile, on sparse
    scenes where most pixels have a denominator far below eps (the worst case of the bound): every
    output element within 1e-7 max|colors| (plus the rounding of sums that now miss their smallest
    terms), every gradient within 1e-5 of the unculled one in norm."""
    from igs_amd._splat import SKIP_TOLERANCE

    B, N, H, W, C = 2, 120, 160, 192, 3
    _, g = sparse_case(dev, B, N, H, W, C, seed=23, smin=0.003, smax=0.03)
    if alpha_scale > 1e20:   # one enormous alpha: its tiles' denominator floors are enormous too
        g["alphas"] = g["alphas"].clone()
        g["alphas"][:, 7] = alpha_scale
    else:
        g["alphas"] = (g["alphas"] * alpha_scale).contiguous()
    out, grads = run(igs, g)
    with no_cull_ctx():
        out0, grads0 = run(igs, g)
    assert bool(torch.isfinite(out0).all())
    cmax = float(g["colors"].abs().max())
    assert SKIP_TOLERANCE == 1e-7
    err = (out - out0).abs()
    assert bool((err <= SKIP_TOLERANCE * cmax + 3e-7 * out0.abs()).all()), float(err.max())
    for k in NAMES:
        d = (grads[k] - grads0[k]).double()
        assert float(d.norm()) <= 1e-5 * float(grads0[k].double().norm()), k


@pytest.mark.parametrize("tolerance,alpha_scale,smax", [(1e-7, 1.0, 0.03), (1e-3, 1.0, 0.03), (1e-3, 25.0, 0.03),
                                                        (1e-2, 0.05, 0.3)])
def test_gradients_under_culling_stay_within_their_bound(igs, dev, tolerance, alpha_scale, smax):
    """The gradients of the default lists (and of far coarser ones) against the run that lists every
    Gaussian for every tile: every element within the oracle's bound T Lam^k P + tau Gam
    (`culling_gradient_bound`, chained to scales and rotations with absolute coefficients), plus the
    rounding of two fp32 evaluations whose sums are grouped differently, priced at 2e-6 Gam (Gam is
    the gradient's own sum with every term taken by its bound); and over each tensor the summed form."""
    from igs_amd._splat import library_options

    B, N, H, W, C = 2, 120, 96, 128, 3
    d64, g = sparse_case(dev, B, N, H, W, C, seed=29, smin=0.003, smax=smax)
    g["alphas"] = (g["alphas"] * alpha_scale).contiguous()
    assert bool((g["alphas"] >= 0).all())
    with library_options(skip_tolerance=tolerance):
        out, grads = run(igs, g)
    with library_options(no_cull=True):
        out0, grads0 = run(igs, g)
    assert bool((out - out0).abs().max() <= tolerance * g["colors"].abs().max() + 3e-7 * out0.abs().max())
    c = {k: v.double().cpu() for k, v in g.items()}
    a, b, dd = (t.reshape(B, N) for t in O.cov_inverse_closed(c["scales"], c["rotations"], 1e-6))
    first, gamma, tau = O.culling_gradient_bound(c["x_grid"], c["y_grid"], c["positions"], a, b, dd, c["alphas"],
                                                 c["colors"], c["grad_out"], 1e-6, tolerance)

    def chained(t):
        bs, bth = O.chain_bound_to_scale_rotation(c["scales"], c["rotations"], t["cov_inv_00"], t["cov_inv_01"],
                                                  t["cov_inv_11"], 1e-6)
        return dict(positions=t["position"], colors=t["colors"], alphas=t["alphas"], scales=bs, rotations=bth)

    first, gamma = chained(first), chained(gamma)
    used = {}
    for k in NAMES:
        delta = (grads[k] - grads0[k]).double().cpu().abs()
        bound = first[k] + (tau + 2e-6) * gamma[k]
        assert bool((delta <= bound).all()), (k, float((delta / bound).max()))
        assert bool((gamma[k] * (1 + 1e-5) >= grads0[k].double().cpu().abs()).all()), k
        if k != "colors":
            lhs = float((delta / first[k]).sum())
            rhs = 1.0 + (tau + 2e-6) * float((gamma[k] / first[k]).sum())
            assert lhs <= rhs, (k, lhs, rhs)
        used[k] = float(delta.max())
    if tolerance >= 1e-3:     # coarse lists do leave pairs out that count
        assert max(used.values()) > 0, used


@pytest.mark.parametrize("shape", [(1, 140000, 48, 48, 1), (33, 33000, 64, 256, 3)], ids=lambda v: "x".join(map(str, v)))
def test_more_candidates_than_the_class_store_holds(igs, dev, no_cull, shape):
    """The binning keeps each candidate's weight class in LDS between the scan that settles what a
    tile skips and the scan that lists (one byte per candidate, four with the forward's four lists
    per tile; 128 KB at most).  Beyond that -- N > 131072, or N > 32768 where the forward bins per
    tile, i.e. with more than 512 wave rectangles in the batch -- the second scan evaluates the
    rectangle test again, with the same arithmetic.  Both shapes: the default tolerance against the
    run that lists everything (within its bound), and the exact mode against it (to rounding: the
    forward cuts lists, not index ranges, into its splits)."""
    from igs_amd._splat import SKIP_TOLERANCE

    B, N, H, W, C = shape
    _, g = sparse_case(dev, B, N, H, W, C, seed=sum(shape), smin=0.02, smax=0.3)
    out, grads = run(igs, g)
    with exact():
        oute, gradse = run(igs, g)
    with no_cull:
        out0, grads0 = run(igs, g)
    cmax = float(g["colors"].abs().max())
    err = (out - out0).abs()
    assert bool((err <= SKIP_TOLERANCE * cmax + 1e-6 * out0.abs().clamp(min=1.0)).all()), float(err.max())
    torch.testing.assert_close(oute, out0, rtol=0, atol=2e-6)
    assert not torch.equal(out, oute)          # the default did leave something out
    for k in NAMES:
        n0 = float(grads0[k].double().norm())
        assert float((grads[k] - grads0[k]).double().norm()) <= 1e-5 * n0, k
        assert float((gradse[k] - grads0[k]).double().norm()) <= 1e-5 * n0, k


@pytest.mark.parametrize("shape,scales", [((8, 4096, 256, 256, 3), (0.01, 0.2)), ((8, 16384, 128, 160, 3), (0.005, 0.1)),
                                          ((4, 32768, 96, 128, 16), (0.005, 0.08)), ((2, 200000, 192, 256, 3), (0.002, 0.02))],
                         ids=lambda v: "x".join(map(str, v)))
def test_one_set_of_tile_lists_for_both_passes(igs, dev, shape, scales):
    """Where the backward's tiles are the forward's wave rectangles (`plan.lists_shared`) a step that
    needs gradients builds the tile lists once, in the backward's workspaces
    (`igs_gs2d_forward_train`, then IGS_OPT_LISTS_BUILT), instead of once per pass.  Against
    the path that bins twice: every gradient bit for bit (the backward's lists are the same lists);
    the image within what the tolerance allows (the forward's own binning settles a 64 x 64 tile's
    allowance with one floor for its four rectangles), and bit for bit when only exact zeros are
    skipped.  The last shape bins in two levels."""
    from igs_amd import _lib, _splat

    B, N, H, W, C = shape
    plan = _lib.plan(B, N, H, W, _kernel_channels(C), 1)
    assert plan.lists_shared == 1
    _, g = sparse_case(dev, B, N, H, W, C, seed=sum(shape), smin=scales[0], smax=scales[1])
    params = [g[k] for k in NAMES]
    need = [True] * 5

    def both(train):
        op, keep, packed, col, out, den = _splat.run_forward(_splat.KIND_SCALE_ROT, params, g["x_grid"], g["y_grid"],
                                                             1e-6, train=train)
        assert (op.shared is not None) == train
        grads, _, _ = _splat.run_backward(_splat.KIND_SCALE_ROT, op, keep, packed, col, out, den, g["grad_out"], need,
                                          False, False, None)
        return out[:, :C], grads

    out_a, grads_a = both(False)
    out_b, grads_b = both(True)
    cmax = float(g["colors"].abs().max())
    assert float((out_a - out_b).abs().max()) <= 2e-7 * cmax + 1e-6
    for k, ga, gb in zip(NAMES, grads_a, grads_b):
        assert float(ga.abs().max()) > 0 and torch.equal(ga, gb), k
    with exact():
        out_a, grads_a = both(False)
        out_b, grads_b = both(True)
    assert torch.equal(out_a, out_b)
    for k, ga, gb in zip(NAMES, grads_a, grads_b):
        assert torch.equal(ga, gb), k


def test_training_forward_where_the_tilings_differ(igs, dev, monkeypatch):
    """A small problem's backward tiles have fewer rows than the forward's wave rectangles (the plan
    says so): the training forward then builds the backward's lists beside its own, in one launch,
    and image and gradients are those of a forward and a backward that each bin for themselves, bit
    for bit."""
    from igs_amd._splat import Grid, Splat

    B, N, H, W, C = 1, 300, 96, 160, 3
    _, g = sparse_case(dev, B, N, H, W, C, seed=2)
    assert Splat(B, N, C, Grid(g["x_grid"], g["y_grid"], B), 1e-6, dev).plan.lists_shared == 0
    used = []
    real = Splat.forward_train
    monkeypatch.setattr(Splat, "forward_train", lambda self, packed: (used.append(1), real(self, packed))[1])
    out, grads = run(igs, g)
    assert used, "the training forward was not taken"
    monkeypatch.setattr(Splat, "forward_train", lambda self, packed: self.forward(packed))   # (leaves `shared` unset)
    out0, grads0 = run(igs, g)
    assert float(out.abs().max()) > 0 and torch.equal(out, out0)
    for k in NAMES:
        assert torch.equal(grads[k], grads0[k]), k


def test_partial_sums_sized_by_the_lists_and_too_small(igs, dev):
    """The separable backward stores one record per listed (Gaussian, tile) pair, tile after tile: an
    array of `listed_total` records (the count the training forward leaves) gives the gradients of the
    full-size array bit for bit, and one that is too small is not overrun: the finalize call then
    returns NaN everywhere."""
    from igs_amd import _lib
    from igs_amd._splat import Grid, Splat, _f32c, _ptr

    B, N, H, W, C = 2, 500, 96, 160, 3
    _, g = sparse_case(dev, B, N, H, W, C, seed=21)
    op = Splat(B, N, C, Grid(g["x_grid"], g["y_grid"], B), 1e-6, dev)
    p, grid, lib = op.plan, op.grid, op.lib
    col = _f32c(g["colors"])
    sc, rot, al = _f32c(g["scales"]), _f32c(g["rotations"]), _f32c(g["alphas"])
    packed = op.pack_scale_rot(_f32c(g["positions"]), sc, rot, al, col)
    out, den = op._new(B, C, H, W), op._new(B, H, W)
    ws, pix = op._empty(p.fwd_ws_bytes), op._empty(p.pix_bytes)
    total = torch.zeros(1, dtype=torch.int64, device=dev)
    _lib.check(lib.igs_gs2d_forward_train(_ptr(packed), _ptr(grid.x), _ptr(grid.y), grid.strides, grid.mode, _ptr(grid.flag),
                                          B, N, H, W, C, 1e-6, _ptr(out), _ptr(den), _ptr(ws), int(p.fwd_ws_bytes),
                                          _ptr(pix), int(p.pix_bytes), _ptr(total), op.stream), "forward_train")
    listed = int(total.item())
    assert 0 < listed < B * p.bwd_tiles * N                 # a sparse scene: far fewer pairs than all
    go = _f32c(g["grad_out"])

    def gradients(records):
        nonlocal pix
        partial = torch.full((max(records, 1) * (6 + C),), float("nan"), device=dev)
        _lib.check(lib.igs_gs2d_backward(_ptr(packed), _ptr(col), _ptr(grid.x), _ptr(grid.y), grid.strides,
                                         grid.mode | _lib.IGS_OPT_LISTS_BUILT, _ptr(grid.flag), _ptr(out), _ptr(den),
                                         _ptr(go), B, N, H, W, C, 1e-6, _ptr(pix), int(p.pix_bytes), _ptr(partial),
                                         partial.numel() * 4, op.stream), "backward")
        gp, gs, gr, ga, gc = op._new(B, N, 2), op._new(B, N, 2), op._new(B, N), op._new(B, N), op._new(B, N, C)
        _lib.check(lib.igs_gs2d_finalize_scale_rot(_ptr(partial), _ptr(pix), grid.mode, _ptr(grid.flag), _ptr(sc), _ptr(rot),
                                                   _ptr(al), B, N, H, W, C, 1e-6, _ptr(gp), _ptr(gs), _ptr(gr), _ptr(ga),
                                                   _ptr(gc), op.stream), "finalize")
        torch.cuda.synchronize()
        return gp, gs, gr, ga, gc

    full = gradients(B * p.bwd_tiles * N)
    assert all(bool(torch.isfinite(t).all()) for t in full) and float(full[0].abs().max()) > 0
    exact_fit = gradients(listed)
    assert all(torch.equal(a, b) for a, b in zip(full, exact_fit))
    for records in (listed - 1, listed // 2, 1):
        assert all(bool(torch.isnan(t).all()) for t in gradients(records)), records
    again = gradients(listed)                               # the flag follows the array of each call
    assert all(torch.equal(a, b) for a, b in zip(full, again))
    # IGS_OPT_LISTS_BUILT on a workspace whose tables were never built (here: bytes of another problem's
    # run) is not trusted: the tables carry a stamp of their problem, nothing is read through them and
    # the gradients come back NaN
    good = pix
    for fill in (0.0, 1.0e9, -3.0):
        pix = torch.full_like(good, fill)
        assert all(bool(torch.isnan(t).all()) for t in gradients(B * p.bwd_tiles * N)), fill
    pix = good


def no_cull_ctx():
    from igs_amd._splat import library_options

    return library_options(no_cull=True)


@pytest.mark.parametrize("dtype", [torch.float64, torch.bfloat16, torch.float16])
def test_other_input_dtypes_round_trip(igs, dev, dtype):
    """The kernels compute in fp32; other floating dtypes are converted on the way in and the
    image and the gradients come back in the caller's dtype (the reference allocates its output
    with the inputs' dtype, src/igs/gs_triton_chunked.py:606)."""
    B, N, H, W, C = 1, 50, 20, 36, 3
    _, g32 = sparse_case(dev, B, N, H, W, C, seed=9, smin=0.05, smax=0.3)
    g = {k: v.to(dtype) for k, v in g32.items()}
    g["x_grid"] = g["x_grid"][:1, :, :1, :].expand(B, 1, H, W)
    g["y_grid"] = g["y_grid"][:1, :, :, :1].expand(B, 1, H, W)
    out, grads = run(igs, g)
    assert out.dtype == dtype and all(v.dtype == dtype for v in grads.values())
    ref = {k: v.to(torch.float32) for k, v in g.items()}      # the same rounded values in fp32
    ref["x_grid"] = ref["x_grid"][:1, :, :1, :].expand(B, 1, H, W)
    ref["y_grid"] = ref["y_grid"][:1, :, :, :1].expand(B, 1, H, W)
    out32, grads32 = run(igs, ref)
    assert torch.equal(out, out32.to(dtype))
    for k in NAMES:
        assert torch.equal(grads[k], grads32[k].to(dtype)), k
