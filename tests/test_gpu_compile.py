"""The splat under `torch.compile` (the reference compiles `render`, src/igs/gs2d.py:525, and its
users compile models around it): the registered `igs_amd::splat_fwd` / `splat_bwd` operators must
give bit-identical results to the eager autograd.Function path (same kernels, same order), trace
as single graph nodes (fullgraph, dynamic shapes), and pass torch's own operator checks."""
import pytest
import torch

from oracle import gs2d_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def igs():
    import igs_amd

    return igs_amd


NAMES = ("positions", "colors", "scales", "rotations", "alphas")


def case(dev, B, N, H, W, C, seed, general=False, grid_grad=False):
    d = O.make_inputs(B, N, H, W, C, 0.05, 0.5, seed=seed, dtype=torch.float32, expand_grids=True)
    d = {k: v.to(dev) for k, v in d.items()}
    if general:
        g = torch.Generator().manual_seed(seed + 5)
        d["x_grid"] = (torch.rand(B, 1, H, W, generator=g) * 2 - 1).to(dev)
        d["y_grid"] = (torch.rand(B, 1, H, W, generator=g) * 2 - 1).to(dev)
    else:  # expanded again: .to(dev) materialises
        d["x_grid"] = d["x_grid"][:, :, :1, :].expand(B, 1, H, W)
        d["y_grid"] = d["y_grid"][:, :, :, :1].expand(B, 1, H, W)
    for k in NAMES:
        d[k].requires_grad_(True)
    if grid_grad:
        d["x_grid"] = d["x_grid"].contiguous().requires_grad_(True)
        d["y_grid"] = d["y_grid"].contiguous().requires_grad_(True)
    return d


def run(fn, d, names):
    for k in names:
        d[k].grad = None
    out = fn(d["positions"], d["colors"], d["scales"], d["rotations"], d["alphas"], d["x_grid"], d["y_grid"])
    out.backward(d["grad_out"])
    return out.detach(), [d[k].grad.clone() for k in names]


@pytest.mark.parametrize("general,grid_grad", [(False, False), (True, False), (True, True)],
                         ids=["separable", "general", "general+gridgrad"])
@pytest.mark.parametrize("C", [3, 5])
def test_operator_path_equals_eager_function_path(igs, dev, C, general, grid_grad):
    """`_ops.splat` (what compiled callers reach) against `_RenderFused.apply`, both eager."""
    from igs_amd import _ops

    d = case(dev, 2, 67, 17, 70, C, seed=11, general=general, grid_grad=grid_grad)
    names = NAMES + (("x_grid", "y_grid") if grid_grad else ())
    o1, g1 = run(igs.gaussian_splatting_2d, d, names)
    via_ops = lambda p, c, s, r, a, x, y: _ops.splat(_ops.KIND_SCALE_ROT, [p, c, s, r, a], x, y, 1e-6, C, p.dtype)
    o2, g2 = run(via_ops, d, names)
    assert torch.equal(o1, o2)
    for n, a, b in zip(names, g1, g2):
        assert torch.equal(a, b), n


def test_opcheck(igs, dev):
    """torch's checks of schema, shape function, autograd registration and AOT dispatch."""
    d = case(dev, 2, 37, 9, 20, 3, seed=3)
    params = [d[k] for k in NAMES]
    torch.library.opcheck(torch.ops.igs_amd.splat_fwd.default, (1, params, d["x_grid"], d["y_grid"], 1e-6))
    with torch.no_grad():
        out, den, packed, col = torch.ops.igs_amd.splat_fwd(1, params, d["x_grid"], d["y_grid"], 1e-6)
    torch.library.opcheck(torch.ops.igs_amd.splat_bwd.default,
                          (1, [p.detach() for p in params], d["x_grid"], d["y_grid"], packed, col, out, den,
                           d["grad_out"], 1e-6, False))


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_compiled_render_fullgraph_dynamic(igs, dev, backend):
    """torch.compile(gaussian_splatting_2d, dynamic=True, fullgraph=True): one graph, no break,
    results identical to eager, also after a shape change."""
    f = torch.compile(igs.gaussian_splatting_2d, dynamic=True, fullgraph=True, backend=backend)
    for (B, N, H, W) in [(2, 67, 17, 70), (1, 130, 33, 65)]:
        d = case(dev, B, N, H, W, 3, seed=N)
        o1, g1 = run(igs.gaussian_splatting_2d, d, NAMES)
        o2, g2 = run(f, d, NAMES)
        assert torch.equal(o1, o2)
        for n, a, b in zip(NAMES, g1, g2):
            assert torch.equal(a, b), n


def test_compiled_operator_apply(igs, dev):
    d = case(dev, 2, 40, 12, 33, 4, seed=21, general=True)
    with torch.no_grad():
        a, b_, c_ = O.cov_inverse_closed(d["scales"].double(), d["rotations"].double())
    cov = [t.float()[..., None, None].contiguous().requires_grad_(True) for t in (a, b_, c_)]
    K = igs.GaussianSplatting2DKernel

    def fn(x, y, p, a, b, c, al, col):
        return K.apply(x, y, p, a, b, c, al, col, 1e-6)

    args = (d["x_grid"], d["y_grid"], d["positions"], *cov, d["alphas"], d["colors"])
    leaves = [d["positions"], *cov, d["alphas"], d["colors"]]

    def go(f):
        for t in leaves:
            t.grad = None
        out = f(*args)
        out.backward(d["grad_out"])
        return out.detach(), [t.grad.clone() for t in leaves]

    o1, g1 = go(fn)
    o2, g2 = go(torch.compile(fn, fullgraph=True, backend="aot_eager"))
    assert torch.equal(o1, o2)
    for a, b in zip(g1, g2):
        assert a.shape == b.shape and torch.equal(a, b)


def test_compiled_module(igs, dev):
    """A compiled model around the module: the head's GEMMs may be scheduled differently by the
    compiler, so the comparison is to tolerance."""
    torch.manual_seed(5)
    m = igs.GaussianSplatting2D(4, 64).to(dev)
    x = torch.randn(2, 16, 64, device=dev)
    go = torch.randn(2, 3, 32, 48, device=dev)

    def step(mod):
        mod.zero_grad()
        xi = x.clone().requires_grad_(True)
        out, feat = mod(xi, size=(32, 48))
        out.backward(go)
        return out.detach(), xi.grad, m.proj.weight.grad.clone(), m.proj.bias.grad.clone()

    ref = step(m)
    got = step(torch.compile(m, dynamic=True, fullgraph=True, backend="aot_eager"))
    for a, b in zip(ref, got):
        torch.testing.assert_close(b, a, rtol=1e-4, atol=1e-6)
