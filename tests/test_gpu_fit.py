"""The fused fit step (render -> MSE -> backward -> AdamW, scripts/2dgs_img_comp.py:107-126,
:186-193, :219-232) against the same iteration written with torch: this build's differentiable
`gaussian_splatting_2d` (itself checked against the fp64 oracle elsewhere), `F.mse_loss` and
`torch.optim.AdamW` with the fit script's hyper-parameters."""
import pytest
import torch
import torch.nn.functional as F

from oracle import gs2d_oracle as O

pytestmark = pytest.mark.gpu

HYPER = dict(eps=1e-6, betas=(0.9, 0.995), weight_decay=1e-4)


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def igs():
    import igs_amd

    return igs_amd


def make_block(B, N, C, seed, dev):
    g = torch.Generator().manual_seed(seed)
    pos = torch.rand(B, N, 2, generator=g) * 2 - 1
    ls = torch.log(torch.rand(B, N, 2, generator=g) * 0.15 + 0.05)
    rot = torch.rand(B, N, 1, generator=g) * 6.283
    col = torch.rand(B, N, C, generator=g)
    return torch.cat([pos, ls, rot, torch.zeros(B, N, 1), col], dim=-1).to(dev)


def grids(igs, B, H, W, dev, general=False, seed=0):
    if general:
        g = torch.Generator().manual_seed(seed)
        return ((torch.rand(B, 1, H, W, generator=g) * 2 - 1).to(dev), (torch.rand(B, 1, H, W, generator=g) * 2 - 1).to(dev))
    x, y = igs.GaussianSplatting2D.xy_grid((H, W), dev)
    return x[None].expand(B, 1, H, W), y[None].expand(B, 1, H, W)


def torch_steps(igs, block0, target, xg, yg, steps, lr, n=None):
    C = block0.shape[-1] - 6
    p = block0.clone().requires_grad_(True)
    opt = torch.optim.AdamW([p], lr=lr, **HYPER)
    losses = []
    for _ in range(steps):
        q = p if n is None else p[:, :n]
        pos, ls, rot, _, col = q.split([2, 2, 1, 1, C], dim=-1)
        img = igs.gaussian_splatting_2d(pos, col, torch.exp(ls) + 1e-6, rot[..., 0], torch.ones_like(rot[..., 0]),
                                        xg, yg)
        loss = F.mse_loss(img, target)
        loss.backward()
        opt.step()
        opt.zero_grad()
        losses.append(loss.detach().clone())
    return p.detach(), torch.stack(losses)


def close(a, b, what, rtol=2e-5, atol=2e-6):
    err = (a - b).abs()
    ok = err <= atol + rtol * b.abs()
    assert bool(ok.all()), f"{what}: max err {float(err.max()):.3e}, {int((~ok).sum())} of {ok.numel()} outside"


@pytest.mark.parametrize("B,N,H,W,C,general", [(1, 200, 32, 48, 3, False), (2, 67, 17, 70, 3, True), (1, 96, 24, 40, 5, False)],
                         ids=["B1-C3-linspace", "B2-C3-general", "B1-C5-padded-channels"])
def test_fused_step_matches_torch_iteration(igs, dev, B, N, H, W, C, general):
    from igs_amd.fit import GaussianImageFit

    block = make_block(B, N, C, 1, dev)
    xg, yg = grids(igs, B, H, W, dev, general, seed=3)
    target = O.smooth_noise_target(H, W, seed=7, C=C).to(dev).expand(B, C, H, W).contiguous()
    lr, steps = 0.02, 6
    ref, ref_losses = torch_steps(igs, block, target, xg, yg, steps, lr)
    fit = GaussianImageFit(block.clone(), target, xg, yg, lr=lr, adam_eps=HYPER["eps"], betas=HYPER["betas"],
                           weight_decay=HYPER["weight_decay"])
    losses = torch.stack([fit.step().clone() for _ in range(steps)])
    assert fit.step_count == steps
    close(losses, ref_losses, "loss", rtol=1e-5, atol=1e-9)
    # the unused column has no gradient; torch leaves it at 0 * (1 - lr wd)^k = 0 as well
    close(fit.params, ref, "parameters after 6 steps")
    assert float((fit.params - block).abs().max()) > 1e-3          # it did move
    named = fit.named_parameters()
    assert named["position"].shape == (B, N, 2) and named["color"].shape == (B, N, C)


def test_adamw_kernel_against_torch_optimizer(igs, dev):
    """igs_adamw_step alone on random gradients of widely varying magnitude, 20 steps."""
    from igs_amd import _lib
    from igs_amd._splat import _ptr, _stream

    lib = _lib.load()
    g = torch.Generator().manual_seed(5)
    n = 10007
    p0 = torch.randn(n, generator=g).to(dev)
    p = p0.clone()
    m, v = torch.zeros_like(p), torch.zeros_like(p)
    state = torch.tensor([0.01, 0, 0, 0, 0, 0, 0, 0], dtype=torch.float32, device=dev)   # lr, t, corrections, ticket
    q = p0.clone().requires_grad_(True)
    opt = torch.optim.AdamW([q], lr=0.01, **HYPER)
    for k in range(20):
        grad = (torch.randn(n, generator=g) * 10.0 ** torch.randint(-9, 1, (n,), generator=g).float()).to(dev)
        if k == 10:                                     # learning-rate change mid-run
            state[0] = 0.003
            opt.param_groups[0]["lr"] = 0.003
        _lib.check(lib.igs_adamw_step(_ptr(p), _ptr(grad), _ptr(m), _ptr(v), n, _ptr(state), 0.9, 0.995, 1e-6, 1e-4,
                                      _stream(dev)), "igs_adamw_step")
        q.grad = grad.clone()
        opt.step()
    close(p, q.detach(), "AdamW parameters", rtol=1e-5, atol=1e-6)
    st = opt.state[q]
    # moments: sums of terms of either sign up to |g| ~ 30, so a few ulp of the largest term
    close(m, st["exp_avg"], "exp_avg", rtol=1e-5, atol=1e-6)
    close(v, st["exp_avg_sq"], "exp_avg_sq", rtol=1e-5, atol=1e-6)
    assert float(state[1]) == 20.0


def test_graph_replay_equals_eager_fused_steps(igs, dev):
    from igs_amd.fit import GaussianImageFit

    B, N, H, W, C = 1, 300, 40, 64, 3
    block = make_block(B, N, C, 2, dev)
    xg, yg = grids(igs, B, H, W, dev)
    target = O.smooth_noise_target(H, W, seed=9, C=C).to(dev)
    eager = GaussianImageFit(block.clone(), target, xg, yg, lr=0.02)
    graphed = GaussianImageFit(block.clone(), target, xg, yg, lr=0.02)
    graphed.capture()
    assert torch.equal(graphed.params, block) and graphed.step_count == 0   # capture executes nothing
    for k in range(8):
        if k == 4:
            eager.set_lr(0.005)
            graphed.set_lr(0.005)
        le = eager.step().clone()
        lg = graphed.step().clone()
        torch.cuda.synchronize()                       # the program's own work between replays
        assert torch.equal(le, lg), k
        assert torch.equal(eager.params, graphed.params), k
    assert graphed.step_count == 8


def test_graph_capture_with_many_gaussians(igs, dev):
    """With more than 49152 Gaussians the binning kernel asks for more dynamic LDS than a launch gets
    by default and raises its limit at the first such launch on the device; here that launch is the
    one being captured.  The replayed steps equal eager ones bit for bit."""
    from igs_amd.fit import GaussianImageFit

    B, N, H, W, C = 1, 60000, 64, 64, 3
    g = torch.Generator().manual_seed(4)
    block = torch.cat([torch.rand(B, N, 2, generator=g) * 2 - 1, torch.log(torch.rand(B, N, 2, generator=g) * 0.05 + 0.01),
                       torch.rand(B, N, 1, generator=g), torch.zeros(B, N, 1), torch.rand(B, N, C, generator=g)], -1).to(dev)
    xg, yg = grids(igs, B, H, W, dev)
    target = O.smooth_noise_target(H, W, seed=3, C=C).to(dev)
    eager = GaussianImageFit(block.clone(), target, xg, yg, lr=1e-3)
    graphed = GaussianImageFit(block.clone(), target, xg, yg, lr=1e-3)
    graphed.capture()
    for k in range(3):
        le = eager.step().clone()
        lg = graphed.step().clone()
        torch.cuda.synchronize()
        assert torch.equal(le, lg), k
        assert torch.equal(eager.params, graphed.params), k
    assert float(le) > 0


def test_prefix_of_gaussians_and_new_resolution(igs, dev):
    """num_active (scripts/2dgs_img_comp.py:107-111) and a change of target size (:208-217)."""
    from igs_amd.fit import GaussianImageFit

    B, N, C = 1, 128, 3
    block = make_block(B, N, C, 4, dev)
    xg, yg = grids(igs, B, 24, 40, dev)
    target = O.smooth_noise_target(24, 40, seed=11, C=C).to(dev)
    fit = GaussianImageFit(block.clone(), target, xg, yg, lr=0.02)
    ref, _ = torch_steps(igs, block, target, xg, yg, 3, 0.02, n=50)
    for _ in range(3):
        fit.step(num_active=50)
    close(fit.params[:, :50], ref[:, :50], "active prefix")
    assert torch.equal(fit.params[:, 50:], block[:, 50:])          # inactive Gaussians untouched
    img = fit.render()
    assert img.shape == (1, 3, 24, 40)
    xg2, yg2 = grids(igs, B, 48, 80, dev)
    fit.set_target(O.smooth_noise_target(48, 80, seed=11, C=C).to(dev), xg2, yg2)
    l0 = float(fit.step())
    for _ in range(30):
        l = float(fit.step())
    assert l < l0
    with pytest.raises(ValueError):
        GaussianImageFit(make_block(2, 16, 3, 0, dev), target.expand(2, -1, -1, -1), xg, yg).step(num_active=4)


def test_fit_converges_config2_reduced(igs, dev):
    """c2-shaped (one image, sigma 0.01-0.1) at reduced size: 100 fused steps lower the loss
    steadily, as the same loop through torch does."""
    from igs_amd.fit import GaussianImageFit

    N, H, W = 2048, 128, 128
    g = torch.Generator().manual_seed(1002)
    pos = torch.rand(1, N, 2, generator=g) * 2 - 1
    col = torch.rand(1, N, 3, generator=g)
    sc = torch.rand(1, N, 2, generator=g) * 0.09 + 0.01
    rot = torch.rand(1, N, generator=g) * 6.283
    xg, yg = grids(igs, 1, H, W, dev)
    target = O.smooth_noise_target(H, W, seed=1002).to(dev)
    fit = GaussianImageFit.from_parameters(pos.to(dev), sc.log().to(dev), rot.to(dev), col.to(dev), target, xg, yg,
                                           lr=min(0.05 * 4096 / N, 0.03))
    fit.capture()
    losses = [float(fit.step()) for _ in range(100)]
    assert losses[10] < losses[0] and losses[99] < 0.5 * losses[10]
    assert bool(torch.isfinite(fit.params).all())


def test_fused_step_under_two_level_binning(igs, dev):
    """IGS_OPT_BIN_LEVELS_2 (the tile lists built through super-tiles) changes the order in which the
    finalize kernel adds the tiles and nothing else: the first loss is bit-identical, the
    parameters after a few steps agree to rounding."""
    from igs_amd._splat import library_options

    B, N, H, W, C = 1, 3000, 256, 512, 3
    block0 = make_block(B, N, C, 5, dev)
    block0[..., 2:4] -= 2.0                                   # small Gaussians: sigma of 1-4 pixels
    xg, yg = grids(igs, B, H, W, dev)
    target = torch.rand(B, C, H, W, generator=torch.Generator().manual_seed(6)).to(dev)
    res = {}
    for levels in ("1", "2"):
        with library_options(bin_levels=int(levels)):
            fit = igs.GaussianImageFit(block0.clone(), target, xg, yg, lr=0.01)
            losses = [float(fit.step()) for _ in range(4)]
            res[levels] = (losses, fit.params.clone())
    assert res["1"][0][0] == res["2"][0][0]
    assert res["1"][0][-1] < res["1"][0][0]
    torch.testing.assert_close(res["1"][1], res["2"][1], rtol=1e-4, atol=1e-5)
    for a, b in zip(res["1"][0], res["2"][0]):
        assert a == pytest.approx(b, rel=1e-5)


def _oracle_loss_and_grad(block, target, xg, yg, penalty=0.0, loss_fn=None):
    """fp64 truth of one iteration's loss and d loss / d block: the naive expression of the oracle
    under autograd (no HIP code on this side), the script's activations exp(log_scale) + eps and
    alpha = 1 (src/igs/gs2d.py:673-675), F.mse_loss (or `loss_fn`) and the position regulariser of
    scripts/2dgs_img_comp.py:224-228."""
    C = block.shape[-1] - 6
    p = block.detach().double().cpu().requires_grad_(True)
    pos, ls, rot, _, col = p.split([2, 2, 1, 1, C], dim=-1)
    img = O.render_naive(pos, col, torch.exp(ls) + 1e-6, rot[..., 0], torch.ones_like(rot[..., 0]),
                         xg.double().cpu(), yg.double().cpu(), 1e-6)
    t = target.double().cpu()
    loss = F.mse_loss(img, t) if loss_fn is None else loss_fn(img, t)
    if penalty:
        loss = loss + penalty * torch.mean(F.relu(pos.abs() - 1.0))
    (g,) = torch.autograd.grad(loss, p)
    return float(loss.detach()), g


@pytest.mark.parametrize("penalty", [0.0, 0.01], ids=["mse", "mse+position-penalty"])
def test_first_fused_step_against_the_fp64_oracle(igs, dev, penalty):
    """Step-0 loss, d block and the updated parameters against the fp64 oracle and AdamW's closed
    form for the first step, p1 = p0 (1 - lr wd) - lr g / (|g| + eps): no HIP render on the
    reference side."""
    from igs_amd.fit import GaussianImageFit

    B, N, H, W, C = 2, 300, 40, 56, 3
    block = make_block(B, N, C, 11, dev)
    block[..., 0:2] *= 1.3                                  # some positions beyond +-1: the penalty is active
    xg, yg = grids(igs, B, H, W, dev)
    target = torch.rand(B, C, H, W, generator=torch.Generator().manual_seed(12)).to(dev)
    lr, wd, aeps = 0.02, HYPER["weight_decay"], HYPER["eps"]
    ref_loss, g64 = _oracle_loss_and_grad(block, target, xg, yg, penalty)
    fit = GaussianImageFit(block.clone(), target, xg, yg, lr=lr, adam_eps=aeps, betas=HYPER["betas"], weight_decay=wd,
                           position_penalty=penalty)
    loss0 = float(fit.step())
    assert loss0 == pytest.approx(ref_loss, rel=1e-5)
    g = fit._ws[N]["g_feat"].double().cpu()
    for name, sl in (("position", slice(0, 2)), ("log_scale", slice(2, 4)), ("rotation", slice(4, 5)),
                     ("color", slice(6, 6 + C))):
        d, r = g[..., sl] - g64[..., sl], g64[..., sl]
        assert float(d.abs().max()) <= 1e-4 * float(r.abs().max()), name
        assert float(d.norm()) <= 1e-4 * float(r.norm()), name
    assert float(g[..., 5].abs().max()) == 0.0 and float(g64[..., 5].abs().max()) == 0.0    # the unused column
    if penalty:   # the regulariser's own part: weight * sign(p) / (2 B N) where |p| > 1
        outside = block[..., 0:2].abs().cpu() > 1.0
        assert int(outside.sum()) > 20
    p0 = block.double().cpu()
    p1 = p0 * (1 - lr * wd) - lr * g64 / (g64.abs() + aeps)
    # where |g| is not far above AdamW's eps the update depends on g to first order: compare there
    # only up to the gradient's own tolerance
    big = g64.abs() > 1e-3 * g64.abs().max()
    err = (fit.params.double().cpu() - p1).abs()
    assert float(err[big].max()) <= 2e-6 + 1e-6 * float(p1.abs().max())
    assert float(err.max()) <= lr * 1.01                     # every update is bounded by lr


def test_step_with_an_external_image_loss(igs, dev):
    """`step(loss_fn=...)`: torch differentiates the caller's loss down to the image, the fused
    backward takes that gradient.  Checked against the fp64 oracle for the first step and against
    the torch iteration over four steps; with F.mse_loss as `loss_fn` it equals the built-in
    mean-squared-error step to rounding."""
    from igs_amd.fit import GaussianImageFit

    B, N, H, W, C = 1, 260, 36, 52, 3
    block = make_block(B, N, C, 21, dev)
    xg, yg = grids(igs, B, H, W, dev)
    target = O.smooth_noise_target(H, W, seed=22, C=C).to(dev)
    mixed = lambda img, t: F.l1_loss(img, t) + 0.25 * F.mse_loss(img, t) + 0.1 * (img[..., 1:] - img[..., :-1]).abs().mean()
    lr = 0.02
    ref_loss, g64 = _oracle_loss_and_grad(block, target, xg, yg, loss_fn=mixed)
    fit = GaussianImageFit(block.clone(), target, xg, yg, lr=lr, adam_eps=HYPER["eps"], betas=HYPER["betas"],
                           weight_decay=HYPER["weight_decay"])
    loss0 = float(fit.step(loss_fn=lambda img: mixed(img, target)))
    assert loss0 == pytest.approx(ref_loss, rel=1e-5)
    g = fit._ws[N]["g_feat"].double().cpu()
    assert float((g - g64).abs().max()) <= 1e-4 * float(g64.abs().max())
    assert float((g - g64).norm()) <= 1e-4 * float(g64.norm())
    # four steps against the torch iteration with the same loss
    p = block.clone().requires_grad_(True)
    opt = torch.optim.AdamW([p], lr=lr, **HYPER)
    fit2 = GaussianImageFit(block.clone(), target, xg, yg, lr=lr, adam_eps=HYPER["eps"], betas=HYPER["betas"],
                            weight_decay=HYPER["weight_decay"])
    for _ in range(4):
        pos, ls, rot, _, col = p.split([2, 2, 1, 1, C], dim=-1)
        img = igs.gaussian_splatting_2d(pos, col, torch.exp(ls) + 1e-6, rot[..., 0], torch.ones_like(rot[..., 0]), xg, yg)
        loss = mixed(img, target)
        loss.backward()
        opt.step()
        opt.zero_grad()
        l2 = fit2.step(loss_fn=lambda im: mixed(im, target))
        assert float(l2) == pytest.approx(float(loss), rel=1e-5)
    # |d l1 / d image| is a constant 1/n: gradients of many parameters sit near AdamW's eps, where the
    # update amplifies rounding; bound by a small multiple of lr there
    close(fit2.params, p.detach(), "parameters after 4 steps with an external loss", rtol=1e-4, atol=2e-4)
    # F.mse_loss as the external loss == the built-in step
    fa = GaussianImageFit(block.clone(), target, xg, yg, lr=lr)
    fb = GaussianImageFit(block.clone(), target, xg, yg, lr=lr)
    for _ in range(3):
        la, lb = fa.step(), fb.step(loss_fn=lambda im: F.mse_loss(im, target))
        assert float(la) == pytest.approx(float(lb), rel=1e-6)
    close(fa.params, fb.params, "mse as external loss", rtol=1e-5, atol=1e-6)
