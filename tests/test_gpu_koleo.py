"""KoLeo diversity loss on the GPU (through the C ABI) against the fp64 oracle.

Tolerances: loss |d| <= 1e-6 + 1e-5 |ref|; gradient per tensor max|d| <= 1e-4 max|ref| and
||d|| <= 1e-4 ||ref||.  The gradient of a row maximum is discontinuous where two similarities
are equal, so the neighbour the fp32 kernels chose is first checked to be a maximum to fp32
rounding (2e-6, times D/1024 for longer dot products) and the oracle's chain rule is then
evaluated with that choice."""
import math

import pytest
import torch

from oracle import koleo_oracle as K

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


def features(shape, seed, kind="normal"):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=g, dtype=F64)
    if kind == "offset":       # all rows in one orthant, similarities near 1
        x = x * 0.2 + 1.0
    elif kind == "scaled":     # row norms over six decades
        x = x * torch.logspace(-3, 3, shape[1], dtype=F64)[None, :, None]
    return x


def gpu_loss_and_grad(igs, x64, dev, scale=1.0):
    x = x64.to(dev, torch.float32).requires_grad_(True)
    loss = igs.koleo_diversity_loss(x)
    (loss * scale).backward()
    return loss.detach(), x.grad


SHAPES = [(1, 2, 3), (2, 7, 4), (1, 65, 17), (3, 130, 9), (1, 128, 512), (2, 1000, 9), (1, 4096, 9),
          (4, 300, 33), (5, 64, 16), (1, 257, 1), (2, 70, 300), (1, 40, 2500), (2, 33, 4100), (3, 2100, 16),
          (1, 3000, 20)]


@pytest.mark.parametrize("kind", ["normal", "offset", "scaled"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_loss_and_gradient_against_oracle(igs, dev, shape, kind):
    from igs_amd.reg import koleo_nearest_neighbours

    x64 = features(shape, seed=sum(shape), kind=kind)
    x32 = x64.to(torch.float32).to(F64)      # the oracle sees the fp32 inputs exactly
    ref = K.koleo_diversity_loss(x32)
    loss, grad = gpu_loss_and_grad(igs, x32, dev, scale=1.3)
    assert abs(float(loss) - float(ref)) <= 1e-6 + 1e-5 * abs(float(ref))
    # the neighbour the kernels chose is a maximum of the row to fp32 rounding
    val, idx = koleo_nearest_neighbours(x32.to(dev, torch.float32))
    rval, ridx, gap = K.nearest_neighbours(x32)
    tol = 2e-6 * max(1.0, shape[2] / 1024)
    assert float((val.cpu().double() - rval).abs().max()) <= tol
    idx = idx.cpu().long()
    open_gate = idx >= 0
    assert bool((open_gate | (rval + 1 <= tol)).all())
    fn, _ = K.normalize_rows(x32)
    chosen = torch.where(open_gate, idx, ridx)
    sim_chosen = (fn * torch.gather(fn, 1, chosen[..., None].expand_as(fn))).sum(-1)
    assert float((rval - sim_chosen).max()) <= tol
    assert bool((chosen != torch.arange(shape[1])[None]).all())
    differs = (chosen != ridx)
    assert bool((gap[differs] <= tol).all())            # only genuine near-ties may differ
    if kind == "normal" and shape[2] > 1:
        assert int(differs.sum()) <= max(1, shape[0] * shape[1] // 500)
    rgrad = K.koleo_backward(x32, grad_loss=1.3, neighbours=chosen)
    d = grad.cpu().double() - rgrad
    assert float(d.abs().max()) <= 1e-4 * float(rgrad.abs().max()) + 1e-30
    assert float(d.norm()) <= 1e-4 * float(rgrad.norm()) + 1e-30


def test_against_plain_torch_fp32_expression(igs, dev):
    """The reference's expression (src/igs/reg.py:22-37) in eager fp32 torch on the GPU."""
    x = features((2, 777, 9), 5).to(dev, torch.float32)
    xr = x.clone().requires_grad_(True)
    ref = K.koleo_diversity_loss(xr)
    ref.backward()
    xg = x.clone().requires_grad_(True)
    loss = igs.koleo_diversity_loss(xg)
    loss.backward()
    torch.testing.assert_close(loss, ref, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(xg.grad, xr.grad, rtol=1e-4, atol=1e-4 * float(xr.grad.abs().max()))


def test_closed_forms_and_edge_cases(igs, dev):
    f = lambda rows: torch.tensor(rows, dtype=torch.float32, device=dev)[None]
    loss = igs.koleo_diversity_loss
    assert float(loss(f([[3.0, 0.0], [1.0, 1.0]]))) == pytest.approx(1 + math.cos(math.pi / 4), rel=1e-6)
    eye = torch.eye(70, device=dev) * torch.arange(1, 71, device=dev)[:, None]
    assert float(loss(eye[None])) == 1.0
    r = features((1, 40, 6), 2).to(dev, torch.float32)
    assert float(loss(torch.cat([r, 2.5 * r], dim=1))) == pytest.approx(2.0, rel=1e-6)
    assert float(loss(f([[1.0, 0, 0], [-1.0, 0, 0], [0, 1.0, 0], [0, 0, 1.0]]))) == 1.0
    assert float(loss(f([[1.0, 0.0], [-2.0, 0.0]]))) == 0.0
    assert float(loss(f([[0.0, 0.0], [1.0, 0.0], [-1.0, 0.0]]))) == 1.0
    # N <= 1: constant 0 without gradient, like the reference
    one = loss(torch.randn(4, 1, 3, device=dev, requires_grad=True))
    assert float(one) == 0.0 and not one.requires_grad
    # NaN and inf propagate as in the plain expression
    x = features((1, 50, 4), 3).to(dev, torch.float32)
    x[0, 7, 2] = float("nan")
    assert math.isnan(float(loss(x)))
    x[0, 7, 2] = float("inf")
    assert math.isnan(float(loss(x))) and math.isnan(float(K.koleo_diversity_loss(x)))


def test_equal_similarities_go_to_the_lowest_index(igs, dev):
    from igs_amd.reg import koleo_nearest_neighbours

    # rows 1, 3 and 200 are the same direction: each one's nearest neighbour is the lowest other
    x = features((1, 300, 5), 4).to(dev, torch.float32)
    x[0, 3] = x[0, 1] * 2
    x[0, 200] = x[0, 1] * 4      # exact scalings by powers of two normalise to the same bits
    val, idx = koleo_nearest_neighbours(x)
    assert [int(idx[0, i]) for i in (1, 3, 200)] == [3, 1, 1]
    # antipodal pair: relu(0) passes no gradient
    y = torch.tensor([[[1.0, 0.0], [-2.0, 0.0]]], device=dev, requires_grad=True)
    igs.koleo_diversity_loss(y).backward()
    assert float(y.grad.abs().max()) == 0.0
    _, idx = koleo_nearest_neighbours(y.detach())
    assert idx.tolist() == [[-1, -1]]
    # a row below the normalisation clamp (x / 1e-12 there)
    z = features((1, 6, 3), 9).to(torch.float32)
    z[0, 2] = torch.tensor([3e-13, 0.0, -1e-13])
    zg = z.to(dev).requires_grad_(True)
    igs.koleo_diversity_loss(zg).backward()
    ref = K.koleo_backward(z.double())
    torch.testing.assert_close(zg.grad.cpu().double(), ref, rtol=1e-4, atol=1e-4 * float(ref.abs().max()) * 1e-3)


def test_properties_at_a_large_size(igs, dev):
    """B=2, N=20000, D=9 (a 3.2 GB similarity matrix in the reference): invariances, the Euler
    identity of the gradient, bit-identical reruns."""
    x = features((2, 20000, 9), 6).to(dev, torch.float32)
    xg = x.clone().requires_grad_(True)
    loss = igs.koleo_diversity_loss(xg)
    loss.backward()
    g = xg.grad
    assert 1.0 < float(loss) < 2.0 and bool(torch.isfinite(g).all())
    # degree-0 homogeneity per row: <x_i, dL/dx_i> = 0
    rel = (x * g).sum(-1).abs() / (x.norm(dim=-1) * g.norm(dim=-1) + 1e-30)
    assert float(rel.max()) < 1e-5
    # positive row scaling (powers of two: exact) leaves every bit of the loss
    s = torch.pow(2.0, torch.randint(-6, 7, (2, 20000, 1), device=dev).float())
    assert float(igs.koleo_diversity_loss(x * s)) == float(loss)
    # a row permutation only reorders the mean
    perm = torch.randperm(20000, device=dev)
    assert float(igs.koleo_diversity_loss(x[:, perm])) == pytest.approx(float(loss), rel=1e-6)
    # the mean over B*N rows is the mean of the per-image losses
    parts = [float(igs.koleo_diversity_loss(x[i:i + 1])) for i in range(2)]
    assert float(loss) == pytest.approx(sum(parts) / 2, rel=1e-6)
    # rerun: bit-identical loss and gradient
    xg2 = x.clone().requires_grad_(True)
    loss2 = igs.koleo_diversity_loss(xg2)
    loss2.backward()
    assert torch.equal(loss, loss2) and torch.equal(g, xg2.grad)
    # nearest neighbours are mutual at least once: the closest pair of an image points at each other
    from igs_amd.reg import koleo_nearest_neighbours
    val, idx = koleo_nearest_neighbours(x)
    top = val.argmax(dim=1)
    for b in range(2):
        j = int(idx[b, top[b]])
        assert float(val[b, j]) == float(val[b, top[b]])


def test_dtypes_layouts_and_upstream_gradient(igs, dev):
    x = features((2, 90, 9), 7).to(dev, torch.float32)
    base = igs.koleo_diversity_loss(x)
    for dt in (torch.float64, torch.bfloat16, torch.float16):
        xd = x.to(dt).requires_grad_(True)
        out = igs.koleo_diversity_loss(xd)
        assert out.dtype == dt
        out.backward()
        assert xd.grad.dtype == dt and xd.grad.shape == x.shape
        ref = igs.koleo_diversity_loss(xd.detach().float())
        assert float(out) == pytest.approx(float(ref), rel=1e-2 if dt != torch.float64 else 1e-7)
    # non-contiguous input (a slice of a wider feature block, as in scripts/gs2d_test.py:172)
    wide = torch.randn(2, 120, 9, device=dev)
    wide[:, :90] = x
    view = wide[:, :90].requires_grad_(True)
    out = igs.koleo_diversity_loss(view)
    assert torch.equal(out, base)
    xg = x.clone().requires_grad_(True)
    (igs.koleo_diversity_loss(xg) * -0.25 + 3).backward()
    (out * -0.25).backward()
    assert torch.equal(view.grad, xg.grad)
    with pytest.raises(RuntimeError):
        igs.koleo_diversity_loss(torch.randn(2, 5, 3))    # CPU tensors have no path
    with pytest.raises(ValueError):
        igs.koleo_diversity_loss(torch.randn(5, 3, device=dev))


def test_under_torch_compile_and_opcheck(igs, dev):
    x = features((2, 150, 9), 8).to(dev, torch.float32)
    torch.library.opcheck(torch.ops.igs_amd.koleo_fwd.default, (x.clone().requires_grad_(True),))

    def f(t):
        return igs.koleo_diversity_loss(t * 1.5) * 2.0

    xe = x.clone().requires_grad_(True)
    f(xe).backward()
    xc = x.clone().requires_grad_(True)
    out = torch.compile(f, fullgraph=True, dynamic=True)(xc)
    out.backward()
    assert torch.equal(out, f(x)) and torch.equal(xc.grad, xe.grad)


def test_against_committed_golden_fixture(igs, dev):
    """tests/golden/koleo_golden.npz (fp64 oracle results of seeded cases, made by
    tests/golden/make_golden_koleo.py); every case has gaps between the two nearest similarities
    far above fp32 rounding, so indices and gradients compare directly."""
    import importlib.util
    import os

    import numpy as np
    from igs_amd.reg import koleo_nearest_neighbours

    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_golden_koleo", os.path.join(here, "make_golden_koleo.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    blob = np.load(os.path.join(here, "koleo_golden.npz"))
    for case in mg.CASES:
        x = mg.inputs(case).to(dev, torch.float32)
        ref = {k: torch.from_numpy(blob[f"{case}/{k}"]) for k in ("loss", "nearest", "index", "gap", "grad")}
        assert float(ref["gap"].min()) > 1e-5, case
        xg = x.clone().requires_grad_(True)
        loss = igs.koleo_diversity_loss(xg)
        loss.backward()
        assert abs(float(loss) - float(ref["loss"])) <= 1e-6 + 1e-5 * abs(float(ref["loss"])), case
        val, idx = koleo_nearest_neighbours(x)
        assert torch.equal(idx.cpu().long(), ref["index"]), case
        assert float((val.cpu().double() - ref["nearest"]).abs().max()) <= 2e-6, case
        d = xg.grad.cpu().double() - ref["grad"]
        assert float(d.abs().max()) <= 1e-4 * float(ref["grad"].abs().max()), case
        assert float(d.norm()) <= 1e-4 * float(ref["grad"].norm()), case
