"""Configuration-shaped end-to-end checks on the GPU: the module at the config-3 shape against
the fp64 oracle, and the single-image fit loop (config 2) in the reference's call convention
(`xy_grid -> [None] -> render`, AdamW as in scripts/2dgs_img_comp.py:186-193)."""
import math

import pytest
import torch

from oracle import gs2d_oracle as O

pytestmark = pytest.mark.gpu
F64 = torch.float64


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def igs():
    import igs_amd

    return igs_amd


def rel(a, b):
    return float((a.double() - b.double()).norm() / b.double().norm())


def test_config3_module_forward_backward_vs_oracle(igs, dev):
    """GaussianSplatting2D(32, 1024), x [8,128,1024] -> 4096 Gaussians per image, 256x256.
    The oracle runs in fp64 on the device in strips; its gradients w.r.t. the Gaussian
    parameters are pushed through the (fp64) linear head with torch autograd."""
    torch.manual_seed(1003)
    m = igs.GaussianSplatting2D(32, 1024).to(dev)
    x = torch.randn(8, 128, 1024, device=dev, requires_grad=True)
    g = torch.Generator().manual_seed(2003)
    go = torch.randn(8, 3, 256, 256, generator=g).to(dev)
    img, feat = m(x, size=(256, 256))
    assert img.shape == (8, 3, 256, 256) and feat.shape == (8, 4096, 9)
    feat.retain_grad()
    img.backward(go)

    # The oracle starts from the module's own fp32 gs_feature (the head is a torch GEMM whose
    # fp32 rounding of positions/log-scales would otherwise dominate: dq = 2 A dx dp with
    # A ~ 3000 here), in fp64 from there on.
    f64 = feat.detach().double().requires_grad_(True)
    pos, ls, rot, _, col = f64.split([2, 2, 1, 1, 3], dim=-1)
    sc = torch.exp(ls) + 1e-6
    al = torch.ones_like(rot[..., 0])
    xg, yg = O.xy_grid((256, 256))                    # the same fp32 coordinates the module uses
    xg = xg.to(dev, F64)[None].expand(8, 1, -1, -1)
    yg = yg.to(dev, F64)[None].expand(8, 1, -1, -1)
    with torch.no_grad():
        a, b_, d = O.cov_inverse_closed(sc, rot[..., 0])
        ref, _ = O.forward_strips(xg, yg, pos, a, b_, d, al, col, rows=8)
        rg = O.render_backward_strips(pos, col, sc, rot[..., 0], al, xg, yg, go.double(), rows=8)
    err = (img.detach().double() - ref).abs()
    tol = 1e-6 + 1e-5 * ref.abs()
    assert float((err > tol).double().mean()) == 0.0, f"forward: max err {float(err.max()):.3e}"
    (gfeat,) = torch.autograd.grad([pos, col, sc, rot], [f64],
                                   [rg["positions"], rg["colors"], rg["scales"], rg["rotations"][..., None]])
    # per field of gs_feature (position, log-scale, rotation, colour); the opacity logit gets 0
    for name, sl in (("positions", slice(0, 2)), ("log_scales", slice(2, 4)), ("rotations", slice(4, 5)),
                     ("colors", slice(6, 9))):
        g_hip, g_ref = feat.grad[..., sl].double(), gfeat[..., sl]
        assert float((g_hip - g_ref).abs().max()) <= 1e-4 * float(g_ref.abs().max()), name
        assert rel(g_hip, g_ref) <= 1e-4, name
    assert float(feat.grad[..., 5].abs().max()) == 0.0
    # the head's own backward (torch GEMMs) from the oracle's d gs_feature, in fp64
    w64 = m.proj.weight.detach().double()
    x64 = x.detach().double()
    g2 = gfeat.unflatten(1, (128, 32)).flatten(2, 3)            # [8,128,288]
    gw = torch.einsum("bfo,bfi->oi", g2, x64)
    gx = g2 @ w64
    assert rel(m.proj.weight.grad, gw) < 2e-4
    assert rel(m.proj.bias.grad, g2.sum((0, 1))) < 2e-4
    assert rel(x.grad, gx) < 2e-4


def _fit(render, N, size, steps, dev, seed=1002):
    H, W = size
    d = O.make_inputs(1, N, H, W, 3, 0.01, 0.1, seed=seed)
    target = O.smooth_noise_target(H, W, seed + 1).to(dev)
    pos = d["positions"].to(dev).requires_grad_(True)
    col = d["colors"].to(dev).requires_grad_(True)
    log_scale = d["scales"].log().to(dev).requires_grad_(True)
    rot = d["rotations"].to(dev).requires_grad_(True)
    alphas = torch.ones(1, N, device=dev)
    lr = min(0.05 * 4096 / N, 0.03)
    opt = torch.optim.AdamW([pos, col, log_scale, rot], lr=lr, eps=1e-6, betas=(0.9, 0.995), weight_decay=1e-4)
    import igs_amd

    xg, yg = igs_amd.GaussianSplatting2D.xy_grid((H, W), dev)
    xg, yg = xg[None], yg[None]
    losses = []
    for _ in range(steps):
        out = render(pos, col, torch.exp(log_scale) + 1e-6, rot, alphas, xg, yg)
        loss = torch.nn.functional.mse_loss(out, target)
        loss.backward()
        opt.step()
        opt.zero_grad()
        losses.append(float(loss.detach()))
    return losses


def test_config2_fit_loop_reduced_matches_naive_torch(igs, dev):
    """Same loop driven by the HIP path and by the plain-torch naive expression (fused=False):
    the loss curves must agree (reduced size so that the naive [N,H,W] intermediate fits)."""
    hip = _fit(lambda *a: igs.gaussian_splatting_2d(*a), 2048, (96, 96), 25, dev)
    ref = _fit(lambda *a: igs.gaussian_splatting_2d(*a, fused=False), 2048, (96, 96), 25, dev)
    assert hip[-1] < 0.6 * hip[0]
    for s in (0, 5, 10, 24):
        assert math.isclose(hip[s], ref[s], rel_tol=2e-3), (s, hip[s], ref[s])


def test_config2_fit_loop_full_size(igs, dev):
    """N = 16384, 512x512, 100 AdamW steps: the loss must fall steadily."""
    losses = _fit(lambda *a: igs.gaussian_splatting_2d(*a), 16384, (512, 512), 100, dev)
    print("c2 loss at steps 0/10/100: %.5f %.5f %.5f" % (losses[0], losses[10], losses[-1]))
    assert all(math.isfinite(v) for v in losses)
    assert losses[10] < losses[0] and losses[-1] < 0.5 * losses[0]


def test_config4_full_size_properties(igs, dev):
    """B4 N32768 384x640 C16 at full size, through size-independent properties: convexity of
    the output, linearity of the backward in grad_out, bit-identical rerun, and the Euler
    identity sum_n alpha_n dL/dalpha_n = eps sum_px <g,out>/(den+eps)."""
    d = {k: v.to(dev) for k, v in O.make_config_inputs("c4").items()}
    B, N, C = d["colors"].shape
    H, W = d["x_grid"].shape[-2:]
    xg = d["x_grid"][:1, :, :1, :].expand(B, 1, H, W)
    yg = d["y_grid"][:1, :, :, :1].expand(B, 1, H, W)
    names = ("positions", "colors", "scales", "rotations", "alphas")

    def run(go):
        lv = {k: d[k].clone().requires_grad_(True) for k in names}
        out = igs.gaussian_splatting_2d(*[lv[k] for k in names], xg, yg)
        out.backward(go)
        return out.detach(), {k: lv[k].grad for k in names}

    out, g1 = run(d["grad_out"])
    out2, g1b = run(d["grad_out"])
    assert torch.equal(out, out2) and all(torch.equal(g1[k], g1b[k]) for k in names)
    lo = d["colors"].amin(1)[:, :, None, None].clamp(max=0)
    hi = d["colors"].amax(1)[:, :, None, None].clamp(min=0)
    assert bool((out >= lo - 1e-5).all()) and bool((out <= hi + 1e-5).all())
    _, g2 = run(-2.0 * d["grad_out"])
    for k in names:
        assert torch.allclose(g2[k], -2.0 * g1[k], rtol=1e-5, atol=1e-6 * float(g1[k].abs().max()))
    # Euler identity needs den: take it from a forward through the operator-level pieces
    a, b_, dd = O.cov_inverse_closed(d["scales"], d["rotations"])
    from igs_amd._splat import Grid as _Grid, Splat as _Splat

    grid = _Grid(xg, yg, B)
    op = _Splat(B, N, C, grid, 1e-6, dev)
    packed = op.pack_scale_rot(d["positions"].contiguous(), d["scales"].contiguous(), d["rotations"].contiguous(),
                               d["alphas"].contiguous(), d["colors"].contiguous())
    o3, den = op.forward(packed)
    assert torch.equal(o3, out)
    lhs = (d["alphas"].double() * g1["alphas"].double()).sum(1)
    rhs = 1e-6 * ((d["grad_out"].double() * out.double()).sum(1) / (den.double() + 1e-6)).sum((1, 2))
    scale = float((d["alphas"].double() * g1["alphas"].double()).abs().sum(1).max())
    assert float((lhs - rhs).abs().max()) < 2e-5 * scale


def test_module_fused_head_equals_unfused_render(igs, dev):
    """The module's fused head (pack/finalize from gs_feature) against the same module driving
    `render` through torch ops, incl. pos_map_offset and a user grid."""
    for pos_off in (False, True):
        torch.manual_seed(5)
        m = igs.GaussianSplatting2D(4, 48, output_dim=3, pos_map_offset=pos_off).to(dev)
        h, w = (8, 12)
        x = torch.randn(2, h * w, 48, device=dev)
        ys, xs = torch.meshgrid(torch.linspace(-1, 1, h, device=dev), torch.linspace(-1.5, 1.5, w, device=dev),
                                indexing="ij")
        grid = torch.stack([ys, xs])[None].repeat(2, 1, 1, 1)          # [B,2,H,W], (y, x) order
        go = torch.randn(2, 3, h, w, device=dev)
        res = []
        for fused_head in (True, False):
            xi = x.clone().requires_grad_(True)
            m.zero_grad()
            if fused_head:
                img, feat = m(xi, grid=grid)
            else:
                feat = m.proj(xi).unflatten(-1, (-1, 9)).flatten(1, 2)
                pos, ls, rot, op_, col = feat.split([2, 2, 1, 1, 3], dim=-1)
                gx, gy = grid.flip(1).split([1, 1], dim=1)
                if pos_off:
                    pm = torch.concat([gx, gy], 1).flatten(2, 3).transpose(1, 2)
                    pos = pos + pm[..., None, :].repeat(1, 1, 4, 1).flatten(1, 2)
                img = igs.gaussian_splatting_2d(pos, col, torch.exp(ls) + 1e-6, rot[..., 0],
                                                torch.ones_like(op_[..., 0]), gx, gy)
            img.backward(go)
            res.append((img.detach(), xi.grad.clone(), m.proj.weight.grad.clone(), m.proj.bias.grad.clone()))
        (i1, x1, w1, b1), (i2, x2, w2, b2) = res
        assert torch.allclose(i1, i2, rtol=1e-5, atol=1e-6)
        for u, v in ((x1, x2), (w1, w2), (b1, b2)):
            assert rel(u, v) < 1e-4


@pytest.mark.parametrize("sized_by_lists", [False, True], ids=["dense", "compact"])
def test_step_is_hip_graph_capturable(igs, dev, monkeypatch, sized_by_lists):
    """A forward+backward step recorded into a HIP graph (the library only launches kernels on the
    stream it is given: no allocation, no synchronisation, no memset).  The graph is replayed
    several times with new inputs, with eager work and synchronisations in between, and every
    replay is checked against the eager result.  `compact`: the problem counts as one whose partial
    sums are sized by the lists (a host read of the forward's count before the backward); under
    capture that read is left out and the eager steps in between still take it."""
    if sized_by_lists:
        monkeypatch.setattr("igs_amd._splat.COMPACT_PARTIALS_FROM", 0)
    B, N, H, W = 2, 300, 40, 56
    names = ("positions", "colors", "scales", "rotations", "alphas")
    cases = [O.make_inputs(B, N, H, W, 3, 0.05, 0.4, seed=600 + i) for i in range(4)]
    static = {k: cases[0][k].to(dev).clone() for k in names}
    for k in names:
        static[k].requires_grad_(True)
    go = cases[0]["grad_out"].to(dev).clone()
    xg, yg = igs.GaussianSplatting2D.xy_grid((H, W), dev)
    xg, yg = xg[None].expand(B, 1, H, W), yg[None].expand(B, 1, H, W)

    def step():
        out = igs.gaussian_splatting_2d(*[static[k] for k in names], xg, yg)
        grads = torch.autograd.grad(out, [static[k] for k in names], go)
        return out, grads

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out, g_grads = step()
    for i, c in enumerate(cases):
        with torch.no_grad():
            for k in names:
                static[k].copy_(c[k].to(dev))
            go.copy_(c["grad_out"].to(dev))
        graph.replay()
        torch.cuda.synchronize()
        r_out, r_grads = g_out.clone(), [g.clone() for g in g_grads]
        e_out, e_grads = step()                       # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(r_out, e_out), f"replay {i}: forward differs"
        for k, a, b in zip(names, r_grads, e_grads):
            assert torch.equal(a, b), f"replay {i}: grad {k} differs"
