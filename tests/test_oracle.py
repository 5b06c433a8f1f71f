"""Pins for the CPU oracle (no GPU).  The reference ships no golden vectors for this
path, so the oracle is pinned by independent restatements and by what the mathematics
fixes; each test is chosen so that a plausible slip (dropped term, wrong sign/index,
transposed operand) fails it."""
import ctypes
import math

import numpy as np
import pytest
import torch

from oracle import gs2d_oracle as O
from oracle.chunked_cpu import ChunkedCPUSplat

torch.manual_seed(0)
F64 = torch.float64


def tiny(B=2, N=5, H=3, W=4, C=3, seed=0, dtype=F64):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.rand(*s, generator=g, dtype=dtype)
    x = r(B, 1, H, W) * 2 - 1
    y = r(B, 1, H, W) * 2 - 1
    pos = r(B, N, 2) * 2 - 1
    sc = r(B, N, 2) * 0.5 + 0.2
    rot = r(B, N) * 2 * math.pi
    al = r(B, N)
    col = torch.randn(B, N, C, generator=g, dtype=dtype)
    go = torch.randn(B, C, H, W, generator=g, dtype=dtype)
    return x, y, pos, sc, rot, al, col, go


def _p(t):
    return np.ascontiguousarray(t.detach().numpy(), dtype=np.float64)


def c_forward(lib, x, y, pos, a, b, d, al, col, eps):
    B, N, C = col.shape
    H, W = x.shape[-2:]
    arrs = [_p(x.reshape(B, H, W)), _p(y.reshape(B, H, W)), _p(pos), _p(a.reshape(B, N)),
            _p(b.reshape(B, N)), _p(d.reshape(B, N)), _p(al), _p(col)]
    out = np.zeros((B, C, H, W))
    den = np.zeros((B, H, W))
    dp = ctypes.POINTER(ctypes.c_double)
    lib.gs2d_bf_forward.restype = None
    lib.gs2d_bf_forward(*[v.ctypes.data_as(dp) for v in arrs], B, N, H, W, C,
                        ctypes.c_double(eps), out.ctypes.data_as(dp), den.ctypes.data_as(dp))
    return arrs, out, den


def c_backward(lib, arrs, out, den, go, B, N, H, W, C, eps):
    dp = ctypes.POINTER(ctypes.c_double)
    g = dict(position=np.zeros((B, N, 2)), cov_inv_00=np.zeros((B, N)), cov_inv_01=np.zeros((B, N)),
             cov_inv_11=np.zeros((B, N)), alphas=np.zeros((B, N)), colors=np.zeros((B, N, C)),
             x=np.zeros((B, 1, H, W)), y=np.zeros((B, 1, H, W)))
    gon = _p(go)
    lib.gs2d_bf_backward.restype = None
    lib.gs2d_bf_backward(*[v.ctypes.data_as(dp) for v in arrs], out.ctypes.data_as(dp),
                         den.ctypes.data_as(dp), gon.ctypes.data_as(dp), B, N, H, W, C,
                         ctypes.c_double(eps),
                         *[g[k].ctypes.data_as(dp) for k in
                           ("position", "cov_inv_00", "cov_inv_01", "cov_inv_11", "alphas", "colors", "x", "y")])
    return g


# ---------------------------------------------------------------- covariance inverse
def test_cov_inverse_closed_equals_matrix_route():
    _, _, _, sc, rot, *_ = tiny(N=64)
    for eps in (1e-6, 1e-2):
        m = O.cov_inverse_matrix(sc, rot, eps)
        c = O.cov_inverse_closed(sc, rot, eps)
        for u, v in zip(m, c):
            assert torch.allclose(u, v, rtol=1e-12, atol=1e-12)


def test_cov_inverse_is_inverse_of_sigma():
    # (A,B;B,D) times R diag(s^2+eps) R^T must be the identity (catches a transposed R).
    _, _, _, sc, rot, *_ = tiny(N=16)
    eps = 1e-3
    a, b, d = [t.reshape(-1) for t in O.cov_inverse_closed(sc, rot, eps)]
    c, s = torch.cos(rot).reshape(-1), torch.sin(rot).reshape(-1)
    l0, l1 = (sc[..., 0] ** 2 + eps).reshape(-1), (sc[..., 1] ** 2 + eps).reshape(-1)
    s00 = c * c * l0 + s * s * l1
    s01 = c * s * (l0 - l1)
    s11 = s * s * l0 + c * c * l1
    assert torch.allclose(a * s00 + b * s01, torch.ones_like(a), atol=1e-10)
    assert torch.allclose(a * s01 + b * s11, torch.zeros_like(a), atol=1e-10)
    assert torch.allclose(b * s01 + d * s11, torch.ones_like(a), atol=1e-10)
    # axis-aligned special case: theta = 0 -> A = 1/(s0^2+eps), B = 0, D = 1/(s1^2+eps)
    a0, b0, d0 = O.cov_inverse_closed(sc, torch.zeros_like(rot), eps)
    assert torch.allclose(a0.reshape(-1), 1 / l0) and torch.all(b0 == 0)
    assert torch.allclose(d0.reshape(-1), 1 / l1)


# ---------------------------------------------------------------- forward
@pytest.mark.parametrize("C", [1, 3, 4])
def test_forward_vs_bruteforce_python_and_c(bruteforce_lib, C):
    x, y, pos, sc, rot, al, col, go = tiny(C=C, seed=C)
    a, b, d = O.cov_inverse_closed(sc, rot)
    ref = O.naive_gaussian_2d(x, y, pos, a, b, d, al, col)
    bf = O.brute_force_forward(x, y, pos, a, b, d, al, col)
    assert torch.allclose(ref, bf, rtol=1e-12, atol=1e-14)
    _, cout, cden = c_forward(bruteforce_lib, x, y, pos, a, b, d, al, col, 1e-6)
    assert np.allclose(ref.numpy(), cout, rtol=1e-12, atol=1e-14)
    out_s, den_s = O.forward_strips(x, y, pos, a, b, d, al, col, rows=2)
    assert torch.allclose(out_s, ref, rtol=1e-12, atol=1e-14)
    assert np.allclose(den_s.numpy(), cden, rtol=1e-12)


def test_forward_single_gaussian_closed_form():
    x, y, pos, sc, rot, al, col, _ = tiny(B=1, N=1, C=3)
    eps = 1e-6
    out = O.render_naive(pos, col, sc, rot, al, x, y, eps)
    # isotropic-free closed form: rotate the offset into the Gaussian's frame.
    c, s = math.cos(float(rot[0, 0])), math.sin(float(rot[0, 0]))
    dx, dy = x[0, 0] - pos[0, 0, 0], y[0, 0] - pos[0, 0, 1]
    u, v = c * dx + s * dy, -s * dx + c * dy
    q = u * u / (sc[0, 0, 0] ** 2 + eps) + v * v / (sc[0, 0, 1] ** 2 + eps)
    w = al[0, 0] * torch.exp(-0.5 * q)
    expect = col[0, 0, :, None, None] * (w / (w + eps))
    assert torch.allclose(out[0], expect, rtol=1e-10, atol=1e-14)


def test_forward_invariants():
    x, y, pos, sc, rot, al, col, _ = tiny(N=7)
    base = O.render_naive(pos, col, sc, rot, al, x, y)
    # constant colour k -> k * den/(den+eps)
    a, b, d = O.cov_inverse_closed(sc, rot)
    _, den = O.forward_strips(x, y, pos, a, b, d, al, col)
    k = 0.37
    outk = O.render_naive(pos, torch.full_like(col, k), sc, rot, al, x, y)
    assert torch.allclose(outk, (k * den / (den + 1e-6))[:, None].expand_as(outk), rtol=1e-12)
    # permutation of the Gaussians
    perm = torch.randperm(7)
    outp = O.render_naive(pos[:, perm], col[:, perm], sc[:, perm], rot[:, perm], al[:, perm], x, y)
    assert torch.allclose(outp, base, rtol=1e-12, atol=1e-15)
    # appending alpha = 0 Gaussians
    z = lambda t: torch.cat([t, t[:, :2]], 1)
    al0 = torch.cat([al, torch.zeros_like(al[:, :2])], 1)
    out0 = O.render_naive(z(pos), z(col), z(sc), z(rot), al0, x, y)
    assert torch.allclose(out0, base, rtol=1e-13, atol=1e-15)
    # joint translation of grid and positions
    t = torch.tensor([0.3, -0.2], dtype=F64)
    outt = O.render_naive(pos + t, col, sc, rot, al, x + t[0], y + t[1])
    assert torch.allclose(outt, base, rtol=1e-10, atol=1e-13)
    # theta -> theta + pi; (s0, s1, theta) -> (s1, s0, theta + pi/2)
    assert torch.allclose(O.render_naive(pos, col, sc, rot + math.pi, al, x, y), base, rtol=1e-10)
    assert torch.allclose(O.render_naive(pos, col, sc.flip(-1), rot + math.pi / 2, al, x, y), base, rtol=1e-10)
    # convexity: alphas >= 0 -> min_c <= out <= max_c per channel
    assert (base <= col.amax(1)[:, :, None, None] + 1e-12).all()
    assert (base >= torch.minimum(col.amin(1), torch.zeros(1, dtype=F64))[:, :, None, None] - 1e-12).all()


# ---------------------------------------------------------------- backward
def test_backward_analytic_vs_autograd_and_c(bruteforce_lib):
    x, y, pos, sc, rot, al, col, go = tiny(N=6, H=4, W=5)
    a, b, d = O.cov_inverse_closed(sc, rot)
    out, ga = O.operator_autograd(x, y, pos, a, b, d, al, col, go)
    gs = O.backward_strips(x, y, pos, a, b, d, al, col, go, rows=3, grid_grads=True)
    B, N, C = col.shape
    H, W = x.shape[-2:]
    arrs, cout, cden = c_forward(bruteforce_lib, x, y, pos, a, b, d, al, col, 1e-6)
    gc = c_backward(bruteforce_lib, arrs, cout, cden, go, B, N, H, W, C, 1e-6)
    for k in ("x", "y", "position", "cov_inv_00", "cov_inv_01", "cov_inv_11", "alphas", "colors"):
        ref = ga[k].reshape(gs[k].shape)
        assert torch.allclose(gs[k], ref, rtol=1e-9, atol=1e-12), k
        assert np.allclose(gc[k], ref.numpy().reshape(gc[k].shape), rtol=1e-9, atol=1e-12), k


def test_backward_function_level_vs_autograd_both_cov_routes():
    x, y, pos, sc, rot, al, col, go = tiny(N=6, H=4, W=5, seed=3)
    g = O.render_backward_strips(pos, col, sc, rot, al, x, y, go)
    for closed in (False, True):
        _, ga = O.render_autograd(pos, col, sc, rot, al, x, y, go, closed_form=closed)
        for k in g:
            assert torch.allclose(g[k], ga[k], rtol=1e-8, atol=1e-11), (k, closed)


def test_backward_finite_differences():
    # central differences on the scalar L = sum(out * go), independent of autograd.
    x, y, pos, sc, rot, al, col, go = tiny(B=1, N=3, H=3, W=3, seed=5)
    g = O.render_backward_strips(pos, col, sc, rot, al, x, y, go)
    L = lambda **kw: float((O.render_naive(kw.get("pos", pos), kw.get("col", col), kw.get("sc", sc),
                                          kw.get("rot", rot), kw.get("al", al), x, y) * go).sum())
    h = 1e-6
    for name, key, t in (("pos", "positions", pos), ("col", "colors", col), ("sc", "scales", sc),
                         ("rot", "rotations", rot), ("al", "alphas", al)):
        flat = t.reshape(-1)
        for i in range(flat.numel()):
            tp, tm = flat.clone(), flat.clone()
            tp[i] += h
            tm[i] -= h
            fd = (L(**{name: tp.view_as(t)}) - L(**{name: tm.view_as(t)})) / (2 * h)
            an = float(g[key].reshape(-1)[i])
            assert abs(fd - an) <= 1e-6 * max(1.0, abs(an)), (name, i, fd, an)


def test_backward_identities():
    x, y, pos, sc, rot, al, col, go = tiny(N=9, H=5, W=4, seed=7)
    eps = 1e-6
    a, b, d = O.cov_inverse_closed(sc, rot, eps)
    g = O.backward_strips(x, y, pos, a, b, d, al, col, go, eps, grid_grads=True)
    # translation: sum_n dL/dpos_n = - sum_px (dL/dx, dL/dy)
    assert torch.allclose(g["position"][..., 0].sum(1), -g["x"].sum((1, 2, 3)), rtol=1e-9, atol=1e-12)
    assert torch.allclose(g["position"][..., 1].sum(1), -g["y"].sum((1, 2, 3)), rtol=1e-9, atol=1e-12)
    # Euler (degree-0 homogeneity in alphas up to eps): sum alpha dL/dalpha = eps sum <g,out>/(den+eps)
    out, den = O.forward_strips(x, y, pos, a, b, d, al, col, eps)
    rhs = eps * ((go * out).sum(1) / (den + eps)).sum((1, 2))
    assert torch.allclose((al * g["alphas"]).sum(1), rhs, rtol=1e-6, atol=1e-13)
    # isotropic Gaussians: dL/dtheta = 0
    iso = sc[..., :1].expand(-1, -1, 2)
    gi = O.render_backward_strips(pos, col, iso, rot, al, x, y, go)
    assert gi["rotations"].abs().max() < 1e-9 * max(1.0, float(gi["positions"].abs().max()))
    # linearity in grad_out
    g2 = O.backward_strips(x, y, pos, a, b, d, al, col, 2.5 * go, eps)
    assert torch.allclose(g2["alphas"], 2.5 * g["alphas"], rtol=1e-12)


# ---------------------------------------------------------------- CPU baseline + helpers
def test_chunked_cpu_baseline_matches_oracle():
    x, y, pos, sc, rot, al, col, go = tiny(B=2, N=70, H=6, W=7, seed=11)  # N not a multiple of 32
    a, b, d = O.cov_inverse_closed(sc, rot)
    out, ga = O.operator_autograd(x, y, pos, a, b, d, al, col, go)
    leaves = [t.clone().requires_grad_(True) for t in (x, y, pos, a, b, d, al, col)]
    o2 = ChunkedCPUSplat.apply(*leaves, 1e-6)
    o2.backward(go)
    assert torch.allclose(o2, out, rtol=1e-11, atol=1e-14)
    for t, k in zip(leaves, ("x", "y", "position", "cov_inv_00", "cov_inv_01", "cov_inv_11", "alphas", "colors")):
        assert torch.allclose(t.grad, ga[k], rtol=1e-9, atol=1e-12), k


def test_xy_grid_ranges():
    xg, yg = O.xy_grid((384, 640))
    assert xg.shape == (1, 384, 640) and yg.shape == (1, 384, 640)
    assert xg.stride(1) == 0 and yg.stride(2) == 0
    assert math.isclose(float(xg[0, 0, -1]), math.sqrt(640 / 384), rel_tol=1e-6)
    assert math.isclose(float(yg[0, -1, 0]), math.sqrt(384 / 640), rel_tol=1e-6)
    assert math.isclose(float(xg[0, 0, -1]) * float(yg[0, -1, 0]), 1.0, rel_tol=1e-6)


def test_make_inputs_is_seeded_and_shaped():
    a = O.make_config_inputs("c0", N=16, H=8, W=8)
    b = O.make_config_inputs("c0", N=16, H=8, W=8)
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert a["x_grid"].shape == (1, 1, 8, 8) and a["x_grid"].stride(2) == 0
    assert a["scales"].min() >= 0.25 and a["scales"].max() <= 0.75
    c4 = O.make_config_inputs("c4", B=1, N=8, H=12, W=20)
    assert math.isclose(float(c4["x_grid"].max()), 20 / 12, rel_tol=1e-6)


# ---------------------------------------------------------------- committed fixtures
def test_oracle_reproduces_golden_fixture():
    import importlib.util
    import os

    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(here, "make_golden.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    blob = np.load(os.path.join(here, "gs2d_golden.npz"))
    for case in mg.CASES:
        _, res = mg.compute(case)
        for k, v in res.items():
            assert np.allclose(v.numpy(), blob[f"{case}/{k}"], rtol=1e-11, atol=1e-14), (case, k)


# ---------------------------------------------------------------- culling bound
def test_reach_box_bounds_the_ellipse_tightly():
    """Pins the bounding-box formula of the culling pass by brute force, not by retyping it:
    the box must contain every point of the ellipse q <= Q (no point with q <= Q lies outside)
    and touch it (the boundary point with the largest x sits on the box's right edge, same for
    y), for rotated anisotropic Gaussians.  A swapped Sigma_xx/Sigma_yy, a wrong sign of the
    rotation or a missing eps fails this."""
    g = torch.Generator().manual_seed(7)
    n = 64
    sc = torch.rand(1, n, 2, generator=g, dtype=F64) * 0.3 + 0.005
    rot = torch.rand(1, n, generator=g, dtype=F64) * 2 * math.pi
    pos = torch.rand(1, n, 2, generator=g, dtype=F64) * 2 - 1
    a, b, d = O.cov_inverse_closed(sc, rot)
    a, b, d = (t.reshape(1, n) for t in (a, b, d))
    Q = O.REACH_Q
    assert math.isclose(-0.5 * math.log2(math.e) * Q, -160.0, rel_tol=1e-12)
    box = O.reach_box(pos, a, b, d)
    # points on the ellipse q = Q: p = pos + sqrt(Q) L^-T u(theta) with [[a,b],[b,d]] = L L^T
    th = torch.linspace(0, 2 * math.pi, 20001, dtype=F64)
    l11 = torch.sqrt(a)
    l21 = b / l11
    l22 = torch.sqrt(d - l21 * l21)
    u, v = torch.cos(th), torch.sin(th)
    dy = math.sqrt(Q) * v[None, None, :] / l22[..., None]
    dx = (math.sqrt(Q) * u[None, None, :] - l21[..., None] * dy) / l11[..., None]
    q = a[..., None] * dx * dx + 2 * b[..., None] * dx * dy + d[..., None] * dy * dy
    assert torch.allclose(q, torch.full_like(q, Q), rtol=1e-9)
    x, y = pos[..., 0, None] + dx, pos[..., 1, None] + dy
    xlo, xhi, ylo, yhi = (box[..., k, None] for k in range(4))
    tol = 1e-9
    assert bool(((x >= xlo - tol) & (x <= xhi + tol) & (y >= ylo - tol) & (y <= yhi + tol)).all())   # contains
    for ext, edge in ((x.max(-1).values, box[..., 1]), (x.min(-1).values, box[..., 0]),
                      (y.max(-1).values, box[..., 3]), (y.min(-1).values, box[..., 2])):
        assert torch.allclose(ext, edge, rtol=0, atol=1e-6 * float(edge.abs().max() + 1))           # tight
    # and therefore: a point outside the box has q > Q
    gx = torch.rand(1, n, 4000, generator=g, dtype=F64) * 8 - 4
    gy = torch.rand(1, n, 4000, generator=g, dtype=F64) * 8 - 4
    outside = (gx < xlo) | (gx > xhi) | (gy < ylo) | (gy > yhi)
    ddx, ddy = gx - pos[..., 0, None], gy - pos[..., 1, None]
    qq = a[..., None] * ddx * ddx + 2 * b[..., None] * ddx * ddy + d[..., None] * ddy * ddy
    assert bool(outside.any()) and bool((qq[outside] > Q).all())


def test_min_q_over_rect_against_dense_sampling():
    """Pins the rectangle minimum used by the second culling test: never above the minimum over a
    dense sample of the rectangle (it is a lower bound of every pixel's q), equal to it up to the
    sampling step, 0 when the centre is inside, and the closed form a dist_x^2 + d dist_y^2 for
    axis-aligned Gaussians.  A wrong vertex (sign, a/d swapped, factor 2) fails the first two."""
    g = torch.Generator().manual_seed(11)
    n = 300
    sc = torch.rand(1, n, 2, generator=g, dtype=F64) * 0.3 + 0.01
    rot = torch.rand(1, n, generator=g, dtype=F64) * 2 * math.pi
    a, b, d = (t.reshape(n) for t in O.cov_inverse_closed(sc, rot))
    px, py = (torch.rand(n, generator=g, dtype=F64) * 2 - 1 for _ in range(2))
    cx, cy = (torch.rand(n, generator=g, dtype=F64) * 2 - 1 for _ in range(2))
    hw, hh = (torch.rand(n, generator=g, dtype=F64) * 0.3 + 0.01 for _ in range(2))
    xlo, xhi, ylo, yhi = cx - hw, cx + hw, cy - hh, cy + hh
    m = O.min_q_over_rect(px, py, a, b, d, xlo, xhi, ylo, yhi)
    k = 401
    t = torch.linspace(0, 1, k, dtype=F64)
    xs = xlo[:, None] + (xhi - xlo)[:, None] * t            # [n,k]
    ys = ylo[:, None] + (yhi - ylo)[:, None] * t
    dx = xs[:, :, None] - px[:, None, None]
    dy = ys[:, None, :] - py[:, None, None]
    q = a[:, None, None] * dx * dx + 2 * b[:, None, None] * dx * dy + d[:, None, None] * dy * dy
    sampled = q.flatten(1).min(dim=1).values
    assert bool((m <= sampled * (1 + 1e-12) + 1e-12).all())                       # a lower bound
    # the sampled minimum is within one grid step of the true one: |grad q| * step
    gmax = 2 * (a + b.abs() + d) * (hw + hh + (cx - px).abs() + (cy - py).abs())
    assert bool((sampled - m <= gmax * (hw + hh) * 2 / (k - 1) + 1e-9).all())      # and attained
    inside = (xlo <= px) & (px <= xhi) & (ylo <= py) & (py <= yhi)
    assert bool(inside.any()) and bool((m[inside] == 0).all()) and bool((m[~inside] > 0).all())
    # axis-aligned: distance to the rectangle per axis
    z = torch.zeros(n, dtype=F64)
    m0 = O.min_q_over_rect(px, py, a, z, d, xlo, xhi, ylo, yhi)
    ddx = torch.clamp(torch.maximum(xlo - px, px - xhi), min=0)
    ddy = torch.clamp(torch.maximum(ylo - py, py - yhi), min=0)
    torch.testing.assert_close(m0, a * ddx * ddx + d * ddy * ddy, rtol=1e-12, atol=1e-15)


def test_skip_weight_bound_by_brute_force():
    """Pins the claim behind the skip weight, not its formula: evaluate the plain expression in
    fp64 with and without the pairs that `skip_limit` allows to drop (e < w / max(1, |alpha|)) on
    scenes built to be the worst case -- sparse small Gaussians, so that many pixels have a
    denominator far below eps and nearly everything they see is below the weight, alphas of either
    magnitude -- and check |d out| <= tolerance max|c| with w = skip_weight(N, eps, tolerance) (then
    also on a dense scene with the per-tile weight w + f S, S the tile's denominator floor), that
    the bound is not vacuous (a constructed pixel comes within a factor 2.1 of it) and that each per-Gaussian sum of exponentials, which is what the gradient of
    alpha adds up, loses less than w per pixel.  A missing factor N, eps or 2, or a limit that
    ignores |alpha| > 1, fails the first check."""
    g = torch.Generator().manual_seed(3)
    N, H, W, C, eps = 60, 48, 64, 3, 1e-6
    for tol, amax in ((1e-7, 1.0), (1e-3, 1.0), (1e-3, 30.0), (0.3, 5.0)):
        pos = torch.rand(1, N, 2, generator=g, dtype=F64) * 2 - 1
        sc = torch.rand(1, N, 2, generator=g, dtype=F64) * 0.03 + 0.004
        rot = torch.rand(1, N, generator=g, dtype=F64) * 2 * math.pi
        al = torch.rand(1, N, generator=g, dtype=F64) * amax
        col = torch.rand(1, N, C, generator=g, dtype=F64) * 2 - 1
        a, b, d = (t.reshape(1, N, 1, 1) for t in O.cov_inverse_closed(sc, rot, eps))
        x = torch.linspace(-1, 1, W, dtype=F64).view(1, 1, 1, W)
        y = torch.linspace(-1, 1, H, dtype=F64).view(1, 1, H, 1)
        dx, dy = x - pos[..., 0, None, None], y - pos[..., 1, None, None]
        q = a * dx * dx + 2 * b * dx * dy + d * dy * dy
        e = torch.exp(-0.5 * q)                                                  # [1,N,H,W]
        w = O.skip_weight(N, eps, tol)
        assert w == tol * eps / (2 * N)
        lim = O.skip_limit(al, w).view(1, N, 1, 1)
        drop = 0.5 * math.log2(math.e) * q > lim
        assert bool(drop.any()) and bool((e[drop] * torch.clamp(al.abs(), min=1).view(1, N, 1, 1).expand_as(e)[drop]
                                          <= w * (1 + 1e-12)).all())

        def image(ee):
            wgt = ee * al.view(1, N, 1, 1)
            return torch.einsum("bnhw,bnc->bchw", wgt, col) / (wgt.sum(1, keepdim=True) + eps)

        full, kept = image(e), image(torch.where(drop, torch.zeros_like(e), e))
        err = float((full - kept).abs().max())
        assert err <= tol * float(col.abs().max()), (tol, amax, err)
        assert float((e * drop).max()) <= w
    # the bound is attained to within a factor of 2.1 when all N Gaussians coincide, carry the same
    # colour and a pixel sees each of them just below the weight: out = N e / (N e + eps) ~ tol / 2
    tol = 1e-3
    w = O.skip_weight(N, eps, tol)
    r = math.sqrt(-2 * math.log(w * 0.999))                       # distance in sigma at which e = 0.999 w
    sig = 0.05
    xs = torch.tensor([0.0, r * sig], dtype=F64)
    e = torch.exp(-0.5 * (xs / sig) ** 2)
    assert float(e[1]) < w and bool(0.5 * math.log2(math.e) * (xs[1] / sig) ** 2 > O.skip_limit(torch.ones(1, dtype=F64), w))
    full = N * e[1] / (N * e[1] + eps)
    assert tol / 2.1 <= float(full) <= tol                         # kept: 0
    # With the skip fraction: a dense scene cut into tiles, each tile skipping up to
    # w + f S (S = tile_weight_floor, which must bound the tile's denominators from below).
    N, H, W = 300, 48, 64
    tol = 1e-3
    pos = torch.rand(1, N, 2, generator=g, dtype=F64) * 2 - 1
    sc = torch.rand(1, N, 2, generator=g, dtype=F64) * 0.25 + 0.02
    rot = torch.rand(1, N, generator=g, dtype=F64) * 2 * math.pi
    al = torch.rand(1, N, generator=g, dtype=F64)
    col = torch.rand(1, N, C, generator=g, dtype=F64) * 2 - 1
    a, b, d = (t.reshape(1, N) for t in O.cov_inverse_closed(sc, rot, eps))
    xs, ys = torch.linspace(-1, 1, W, dtype=F64), torch.linspace(-1, 1, H, dtype=F64)
    dx, dy = xs.view(1, 1, 1, W) - pos[..., 0, None, None], ys.view(1, 1, H, 1) - pos[..., 1, None, None]
    q = a[..., None, None] * dx * dx + 2 * b[..., None, None] * dx * dy + d[..., None, None] * dy * dy
    e = torch.exp(-0.5 * q)
    den = (e * al[..., None, None]).sum(1)
    w, f = O.skip_weight(N, eps, tol), O.skip_weight(N, 1.0, tol)
    assert f == tol / (2 * N)
    drop = torch.zeros_like(e, dtype=torch.bool)
    gained = 0
    for r0 in range(0, H, 16):
        for c0 in range(0, W, 16):
            S = O.tile_weight_floor(pos[..., 0], pos[..., 1], a, b, d, al, xs[c0], xs[c0 + 15], ys[r0], ys[r0 + 15])
            assert bool((den[:, r0:r0 + 16, c0:c0 + 16] >= S[:, None, None] * (1 - 1e-12)).all())     # a floor indeed
            assert float(S) > 100 * eps                                                              # and not a vacuous one
            wt = O.tile_skip_weight(w, f, S)
            et = e[:, :, r0:r0 + 16, c0:c0 + 16]
            drop[:, :, r0:r0 + 16, c0:c0 + 16] = et < wt
            gained += int((et < wt).sum()) - int((et < w).sum())
    assert gained > 0.05 * e.numel()                                 # the fraction is what skips most here
    full = torch.einsum("bnhw,bnc->bchw", e * al[..., None, None], col) / (den[:, None] + eps)
    ek = torch.where(drop, torch.zeros_like(e), e) * al[..., None, None]
    kept = torch.einsum("bnhw,bnc->bchw", ek, col) / (ek.sum(1)[:, None] + eps)
    assert float((full - kept).abs().max()) <= tol * float(col.abs().max())
    assert float(O.tile_weight_floor(pos[..., 0], pos[..., 1], a, b, d, -al, xs[0], xs[5], ys[0], ys[5])) == 0.0
    # The rule the binning kernel applies per tile (`tile_first_skipped_class`): whole weight classes
    # are left out of a tile's list while the sum of their members' largest terms stays within
    # N (w + f S).  Checked by brute force: the sum of the true maxima of the left-out Gaussians over
    # the tile's pixels is within the allowance (and uses a good part of it), more is left out than
    # by the per-pair weight w + f S, and the image stays within the tolerance.
    drop2 = torch.zeros_like(e, dtype=torch.bool)
    used, by_weight = [], 0
    amax1 = torch.clamp(al.abs(), min=1.0)
    for r0 in range(0, H, 16):
        for c0 in range(0, W, 16):
            S = float(O.tile_weight_floor(pos[..., 0], pos[..., 1], a, b, d, al, xs[c0], xs[c0 + 15], ys[r0], ys[r0 + 15]))
            mq = O.min_q_over_rect(pos[..., 0], pos[..., 1], a, b, d, xs[c0], xs[c0 + 15], ys[r0], ys[r0 + 15])
            cls = O.weight_class(mq, al)[0]
            first = O.tile_first_skipped_class(cls, N, w, f, S)
            out_n = cls >= first
            et = e[0, :, r0:r0 + 16, c0:c0 + 16] * amax1[0, :, None, None]
            true_max = et.amax((1, 2))
            # the class bounds the Gaussian's terms on the tile from above
            assert bool((true_max[cls >= 0] <= 2.0 ** (-cls[cls >= 0].double() / O.WEIGHT_CLASSES_PER_BINADE) * (1 + 1e-12)).all())
            allowance = N * O.tile_skip_weight(w, f, S)
            assert float(true_max[out_n].sum()) <= allowance
            used.append(float(true_max[out_n].sum()) / allowance)
            by_weight += 256 * int((amax1[0] * torch.exp(-0.5 * mq[0]) < O.tile_skip_weight(w, f, S)).sum())
            drop2[0, :, r0:r0 + 16, c0:c0 + 16] = out_n[:, None, None]
    assert int(drop2.sum()) > 1.05 * by_weight and sorted(used)[len(used) // 2] > 0.1, (int(drop2.sum()), by_weight, used)
    ek = torch.where(drop2, torch.zeros_like(e), e) * al[..., None, None]
    kept = torch.einsum("bnhw,bnc->bchw", ek, col) / (ek.sum(1)[:, None] + eps)
    assert float((full - kept).abs().max()) <= tol * float(col.abs().max())
    # N coincident Gaussians seen just beyond the class edge at w from the nearest pixel of a tile
    # whose floor is ~0: all are left out and the pixel, out = N e / (N e + eps) ~ tolerance / 2,
    # comes within a factor 2.1 sqrt(2) of the bound; one class nearer, none is left out.
    kb = math.ceil(-math.log2(w) * O.WEIGHT_CLASSES_PER_BINADE)

    def left_out(classes, floor):
        first = O.tile_first_skipped_class(classes, N, w, f, floor)
        return sorted(classes[(classes >= 0) & (classes >= first)].tolist())

    assert left_out(torch.full((N,), kb), 0.0) == [kb] * N and left_out(torch.full((N,), kb - 1), 0.0) == []
    e_edge = 2.0 ** (-kb / O.WEIGHT_CLASSES_PER_BINADE)
    assert tol / (2.1 * math.sqrt(2)) <= N * e_edge / (N * e_edge + eps) <= tol
    # with a floor, N (w + f S) is spent on the lightest classes first: ten classed members allow
    # 10 w, which the three of class kb - 1 (at most sqrt(2) w each) fit into and the five of class
    # kb - 9 (16 w each) do not; a floor of 1000 eps adds N f S = 1000 N w
    few = torch.tensor([kb - 1] * 3 + [kb - 9] * 5 + [-1, 0, 1])
    assert left_out(few, 0.0) == [kb - 1] * 3
    assert left_out(few, 1e3 * eps) == [kb - 9] * 5 + [kb - 1] * 3
    assert O.tile_first_skipped_class(few, N, 0.0, f, 1.0) is None
    assert O.weight_class(torch.tensor([0.0, 4.0, 4.0]), torch.tensor([1.0, 1.0, 1e3])).tolist()[::2] == [-1, -1]
    assert O.skip_weight(100, 0.0, 1e-7) == 0.0 and O.skip_weight(100, 1e-6, 0.0) == 0.0
    assert bool((O.skip_limit(torch.tensor([0.5, 4.0]), 0.0) == O.EXACT_LIMIT).all())
    assert math.isclose(float(O.reach_q(torch.tensor([1.0], dtype=F64), 0.0)[0]), O.REACH_Q, rel_tol=1e-12)
    # |alpha| = 4 moves the limit by two binades, |alpha| < 1 by nothing
    l = O.skip_limit(torch.tensor([0.25, 1.0, 4.0], dtype=F64), 2.0 ** -50)
    assert l.tolist() == [50.0, 50.0, 52.0]


def _tile_keep_mask(pos, a, b, d, al, xs, ys, th, tw, w, f):
    """[1,N,H,W] mask of the pairs that tiles of th x tw pixels keep under `tile_first_skipped_class`."""
    N, H, W = al.shape[1], ys.numel(), xs.numel()
    keep = torch.ones(1, N, H, W, dtype=torch.bool)
    for r0 in range(0, H, th):
        for c0 in range(0, W, tw):
            r1, c1 = min(r0 + th, H) - 1, min(c0 + tw, W) - 1
            rect = (xs[c0], xs[c1], ys[r0], ys[r1])
            S = float(O.tile_weight_floor(pos[..., 0], pos[..., 1], a, b, d, al, *rect))
            cls = O.weight_class(O.min_q_over_rect(pos[..., 0], pos[..., 1], a, b, d, *rect), al)[0]
            first = O.tile_first_skipped_class(cls, N, w, f, S)
            keep[0, :, r0:r1 + 1, c0:c1 + 1] = ~(cls >= first)[:, None, None]
    return keep


def test_gradient_bound_under_culling_by_brute_force():
    """Pins `culling_gradient_bound`, not its formula: fp64 gradients with and without the pairs the
    per-tile rule leaves out -- the forward's tiling and the backward's differ, as in the kernels, and
    the backward uses the culled image -- on the worst-case scenes of the forward's bound (sparse,
    most denominators far below eps, alphas beyond 1) and on a dense one where the floors carry the
    allowance; every element within its bound, every tensor within the summed bound.  Two constructed
    pixels come close to the two terms, so neither is slack by more than a small factor; dropping the
    1/(den+eps), the factor K, or the second term fails them."""
    g = torch.Generator().manual_seed(11)
    C, eps = 3, 1e-6
    names = ("position", "cov_inv_00", "cov_inv_01", "cov_inv_11", "alphas", "colors")
    worst = {k: 0.0 for k in names}
    scenes = [(60, 0.004, 0.034, 1e-7, 1.0), (60, 0.004, 0.034, 1e-3, 1.0), (60, 0.004, 0.034, 1e-3, 30.0),
              (300, 0.02, 0.27, 1e-3, 1.0), (300, 0.02, 0.27, 0.05, 0.02), (120, 0.01, 0.1, 0.2, 5.0)]
    for N, smin, smax, tol, amax in scenes:
        H, W = 48, 64
        pos = torch.rand(1, N, 2, generator=g, dtype=F64) * 2 - 1
        sc = torch.rand(1, N, 2, generator=g, dtype=F64) * (smax - smin) + smin
        rot = torch.rand(1, N, generator=g, dtype=F64) * 2 * math.pi
        al = torch.rand(1, N, generator=g, dtype=F64) * amax
        col = torch.rand(1, N, C, generator=g, dtype=F64) * 2 - 1
        go = torch.randn(1, C, H, W, generator=g, dtype=F64)
        a, b, d = (t.reshape(1, N) for t in O.cov_inverse_closed(sc, rot, eps))
        xs, ys = torch.linspace(-1, 1, W, dtype=F64), torch.linspace(-1, 1, H, dtype=F64)
        x, y = xs.view(1, 1, 1, W).expand(1, 1, H, W), ys.view(1, 1, H, 1).expand(1, 1, H, W)
        w, f = O.skip_weight(N, eps, tol), O.skip_weight(N, 1.0, tol)
        keep_f = _tile_keep_mask(pos, a, b, d, al, xs, ys, 16, 32, w, f)
        keep_b = _tile_keep_mask(pos, a, b, d, al, xs, ys, 32, 8, w, f)
        assert not bool(keep_f.all()) and not bool(keep_b.all()) and not bool((keep_f == keep_b).all())
        every = torch.ones_like(keep_f)
        out0, g0 = O.backward_with_lists(x, y, pos, a, b, d, al, col, go, eps, every, every)
        ref = O.backward_strips(x, y, pos, a, b, d, al, col, go, eps)
        for k in names:
            torch.testing.assert_close(g0[k], ref[k], rtol=1e-11, atol=1e-13)
        out1, g1 = O.backward_with_lists(x, y, pos, a, b, d, al, col, go, eps, keep_f, keep_b)
        assert float((out1 - out0).abs().max()) <= tol * float(col.abs().max())
        first, gamma, tau = O.culling_gradient_bound(x, y, pos, a, b, d, al, col, go, eps, tol)
        assert tau >= 2 * tol
        for k in names:
            delta = (g1[k] - g0[k]).abs()
            bound = first[k] + tau * gamma[k]
            assert bool((delta <= bound).all()), (k, N, tol, float((delta / bound).max()))
            if k != "colors":        # the summed form: all Gaussians share one allowance per pixel
                lhs = float((delta / first[k]).sum())
                rhs = 1.0 + tau * float((gamma[k] / first[k]).sum())
                assert lhs <= rhs, (k, N, tol, lhs, rhs)
                worst[k] = max(worst[k], lhs / rhs)
            else:
                worst[k] = max(worst[k], float((delta / bound).max()))
            assert bool((gamma[k] >= g0[k].abs() * (1 - 1e-12)).all())    # Gam bounds the gradient itself
    # (random scenes use little of it, as they use little of the forward's tolerance: few of a tile's
    # Gaussians sit just under the threshold; the constructed pixels below are what comes close)
    assert max(worst.values()) < 1e-2, worst

    # One pixel that sees a heavy Gaussian of colour -1, a light one of colour +1 (k) and Nd faint
    # ones of colour +1 whose weights add up to the whole allowance tolerance (den + eps).
    Nd, tol = 20, 1e-3
    N = Nd + 2
    x = y = torch.zeros(1, 1, 1, 1, dtype=F64)
    pos = torch.zeros(1, N, 2, dtype=F64)
    a = d = torch.full((1, N), 100.0, dtype=F64)
    b = torch.zeros(1, N, dtype=F64)
    col = torch.ones(1, N, 1, dtype=F64)
    col[0, 0, 0] = -1.0
    al = torch.ones(1, N, dtype=F64)
    al[0, 1] = 1e-3
    Dfull = (1.0 + 1e-3 + eps) / (1 - tol)
    u = tol * Dfull / Nd
    r = math.sqrt(-2 * math.log(u) / 100.0)                      # e = u at distance r
    pos[0, 2:, 0] = r
    go = torch.ones(1, 1, 1, 1, dtype=F64)
    every = torch.ones(1, N, 1, 1, dtype=torch.bool)
    faint = every.clone()
    faint[0, 2:] = False
    _, g0 = O.backward_with_lists(x, y, pos, a, b, d, al, col, go, eps, every, every)
    first, gamma, tau = O.culling_gradient_bound(x, y, pos, a, b, d, al, col, go, eps, tol)
    # (2): the forward leaves the faint ones out, the backward nothing: d alpha_k moves by nearly tau Gam
    _, g2 = O.backward_with_lists(x, y, pos, a, b, d, al, col, go, eps, faint, every)
    moved = float((g2["alphas"] - g0["alphas"]).abs()[0, 1])
    assert 0.9 * tau * float(gamma["alphas"][0, 1]) <= moved <= tau * float(gamma["alphas"][0, 1])
    # (1): the backward leaves them out, the forward nothing: their d alpha, summed, lose nearly T
    _, g3 = O.backward_with_lists(x, y, pos, a, b, d, al, col, go, eps, every, faint)
    lost = float((g3["alphas"] - g0["alphas"]).abs().sum())
    T = float(first["alphas"][0, 0])                              # m = 1: T itself
    assert 0.9 * T <= lost <= T
    assert bool((g3["alphas"][0, 2:] == 0).all()) and float(g3["alphas"][0, 1]) == float(g0["alphas"][0, 1])
    # and their moments stay within the log factor's bound while using more than the bare allowance
    lost_a = float((g3["cov_inv_00"] - g0["cov_inv_00"]).abs().sum())
    sxx = 1.0 / 100.0
    assert T * 0.5 * sxx < lost_a <= float(first["cov_inv_00"][0, 2]) 

    # scale / rotation: the chain with absolute coefficients bounds the chained difference
    sc = torch.rand(1, 7, 2, generator=g, dtype=F64) * 0.2 + 0.01
    rot = torch.rand(1, 7, generator=g, dtype=F64) * 6
    dA, dB, dD = (torch.randn(1, 7, generator=g, dtype=F64) for _ in range(3))
    gs, gth = O.chain_to_scale_rotation(sc, rot, dA, dB, dD, eps)
    bs, bth = O.chain_bound_to_scale_rotation(sc, rot, dA.abs(), dB.abs(), dD.abs(), eps)
    assert bool((gs.abs() <= bs * (1 + 1e-12)).all()) and bool((gth.abs() <= bth * (1 + 1e-12)).all())
    same = O.chain_bound_to_scale_rotation(sc, torch.zeros_like(rot), dA.abs(), dB.abs() * 0, dD.abs(), eps)
    exact = O.chain_to_scale_rotation(sc, torch.zeros_like(rot), dA.abs(), dB * 0, dD.abs(), eps)
    torch.testing.assert_close(same[0], exact[0].abs(), rtol=1e-12, atol=0)   # attained where nothing cancels
