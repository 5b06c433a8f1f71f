"""Pins for the CPU oracle of the KoLeo diversity loss (no GPU).  The reference holds no test or
golden vector for it, so the restatement is pinned by an independent brute force and by what the
mathematics fixes."""
import math

import pytest
import torch

from oracle import koleo_oracle as K

F64 = torch.float64


def rand(B, N, D, seed=0):
    return torch.randn(B, N, D, generator=torch.Generator().manual_seed(seed), dtype=F64)


@pytest.mark.parametrize("shape", [(1, 2, 3), (2, 7, 4), (3, 5, 9), (1, 9, 1)], ids=str)
def test_loss_against_plain_loops(shape):
    x = rand(*shape, seed=sum(shape))
    assert float(K.koleo_diversity_loss(x)) == pytest.approx(K.koleo_loops(x.tolist()), rel=1e-13, abs=1e-15)


def test_closed_forms():
    # two rows: both see each other, loss = relu(cos + 1)
    a, b = torch.tensor([3.0, 0.0], dtype=F64), torch.tensor([1.0, 1.0], dtype=F64)
    x = torch.stack([a, b])[None]
    assert float(K.koleo_diversity_loss(x)) == pytest.approx(1 + math.cos(math.pi / 4), rel=1e-14)
    # an orthonormal set (scaled rows): every similarity 0 -> 1
    x = (torch.eye(5, dtype=F64) * torch.arange(1, 6, dtype=F64)[:, None])[None]
    assert float(K.koleo_diversity_loss(x)) == pytest.approx(1.0, abs=1e-15)
    # duplicated rows: nearest similarity 1 -> 2
    r = rand(1, 3, 4, seed=2)
    x = torch.cat([r, 2.5 * r], dim=1)
    assert float(K.koleo_diversity_loss(x)) == pytest.approx(2.0, rel=1e-14)
    # e0 and -e0 among e1, e2: the antipodal pair's nearest neighbours are the orthogonal rows
    x = torch.tensor([[1.0, 0, 0], [-1.0, 0, 0], [0, 1.0, 0], [0, 0, 1.0]], dtype=F64)[None]
    assert float(K.koleo_diversity_loss(x)) == pytest.approx(1.0, abs=1e-15)
    # exactly antipodal pair alone: relu(-1 + 1) = 0
    assert float(K.koleo_diversity_loss(x[:, :2])) == 0.0
    # N <= 1 (src/igs/reg.py:19-20)
    assert float(K.koleo_diversity_loss(rand(4, 1, 3))) == 0.0
    # a zero row is left at zero by the normalisation: its similarities are 0
    x = torch.tensor([[0.0, 0.0], [1.0, 0.0], [-1.0, 0.0]], dtype=F64)[None]
    assert float(K.koleo_diversity_loss(x)) == pytest.approx(1.0, abs=1e-15)   # rows see the zero row (sim 0)


def test_invariants():
    x = rand(2, 11, 5, seed=3)
    base = float(K.koleo_diversity_loss(x))
    g = torch.Generator().manual_seed(4)
    scale = torch.rand(2, 11, 1, generator=g, dtype=F64) * 5 + 0.1
    assert float(K.koleo_diversity_loss(x * scale)) == pytest.approx(base, rel=1e-13)
    q, _ = torch.linalg.qr(torch.randn(5, 5, generator=g, dtype=F64))
    assert float(K.koleo_diversity_loss(x @ q)) == pytest.approx(base, rel=1e-13)
    perm = torch.randperm(11, generator=g)
    assert float(K.koleo_diversity_loss(x[:, perm])) == pytest.approx(base, rel=1e-13)
    # the mean runs over B*N rows: stacking images averages their losses
    l0 = float(K.koleo_diversity_loss(x[:1])), float(K.koleo_diversity_loss(x[1:]))
    assert base == pytest.approx(0.5 * (l0[0] + l0[1]), rel=1e-13)


def test_nearest_neighbours_indices_and_gap():
    x = rand(2, 9, 3, seed=6)
    val, idx, gap = K.nearest_neighbours(x)
    fn, _ = K.normalize_rows(x)
    for b in range(2):
        for i in range(9):
            sims = sorted((float(fn[b, i] @ fn[b, j]), -j) for j in range(9) if j != i)
            assert float(val[b, i]) == pytest.approx(sims[-1][0], abs=1e-15)
            assert int(idx[b, i]) == -sims[-1][1]
            assert float(gap[b, i]) == pytest.approx(sims[-1][0] - sims[-2][0], abs=1e-14)


def test_backward_restated_against_autograd_and_finite_differences():
    x = rand(2, 8, 4, seed=7)
    loss, g_auto = K.autograd_gradient(x, grad_loss=1.7)
    g = K.koleo_backward(x, grad_loss=1.7)
    torch.testing.assert_close(g, g_auto, rtol=1e-12, atol=1e-14)
    assert float(g.abs().max()) > 0
    # central differences on a few coordinates (the loss is piecewise smooth; the step stays far
    # below the smallest gap between a row's two nearest similarities)
    assert float(K.nearest_neighbours(x)[2].min()) > 1e-3
    h = 1e-6
    for (b, i, d) in [(0, 0, 0), (1, 3, 2), (0, 7, 3), (1, 5, 1)]:
        xp, xm = x.clone(), x.clone()
        xp[b, i, d] += h
        xm[b, i, d] -= h
        fd = 1.7 * float(K.koleo_diversity_loss(xp) - K.koleo_diversity_loss(xm)) / (2 * h)
        assert float(g[b, i, d]) == pytest.approx(fd, rel=1e-6, abs=1e-9)
    # degree-0 homogeneity per row: <x_i, dL/dx_i> = 0
    assert float((x * g).sum(-1).abs().max()) < 1e-15


def test_backward_gate_and_tiny_rows():
    # an exactly antipodal pair has sim + 1 = 0: relu passes no gradient
    x = torch.tensor([[[1.0, 0.0], [-2.0, 0.0]]], dtype=F64)
    assert float(K.koleo_backward(x).abs().max()) == 0.0
    _, g_auto = K.autograd_gradient(x)
    assert float(g_auto.abs().max()) == 0.0
    # a row shorter than the clamp: the normalisation is x / 1e-12 there
    x = rand(1, 4, 3, seed=9)
    x[0, 2] = torch.tensor([3e-13, 0.0, -1e-13], dtype=F64)
    _, g_auto = K.autograd_gradient(x)
    torch.testing.assert_close(K.koleo_backward(x), g_auto, rtol=1e-12, atol=0)


def test_backward_with_given_neighbours():
    """Passing the oracle's own neighbours changes nothing; passing another neighbour gives the
    autograd gradient of the loss with that column chosen."""
    x = rand(2, 6, 3, seed=11)
    _, idx, _ = K.nearest_neighbours(x)
    torch.testing.assert_close(K.koleo_backward(x, 0.7, neighbours=idx), K.koleo_backward(x, 0.7), rtol=0, atol=0)
    other = (idx + 1) % 6
    other = torch.where(other == torch.arange(6)[None], (other + 1) % 6, other)
    xr = x.clone().requires_grad_(True)
    fn, _ = K.normalize_rows(xr)
    sim = (fn * torch.gather(fn, 1, other[..., None].expand(2, 6, 3))).sum(-1)
    (g,) = torch.autograd.grad(torch.relu(sim + 1).mean() * 0.7, xr)
    torch.testing.assert_close(K.koleo_backward(x, 0.7, neighbours=other), g, rtol=1e-12, atol=1e-15)


def _golden():
    import importlib.util
    import os

    import numpy as np

    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_golden_koleo", os.path.join(here, "make_golden_koleo.py"))
    mg = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mg)
    return mg, np.load(os.path.join(here, "koleo_golden.npz"))


def test_oracle_reproduces_golden_fixture():
    import numpy as np

    mg, blob = _golden()
    for case in mg.CASES:
        x, res = mg.compute(case)
        assert float(K.koleo_diversity_loss(x)) == pytest.approx(K.koleo_loops(x.tolist()), rel=1e-12)
        for k, v in res.items():
            assert np.allclose(v.numpy(), blob[f"{case}/{k}"], rtol=1e-11, atol=1e-14), (case, k)
