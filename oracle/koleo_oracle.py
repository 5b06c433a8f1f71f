"""CPU restatement of the reference's KoLeo diversity loss (TEST INFRASTRUCTURE ONLY).

The checker that the HIP path of ``igs_amd.reg.koleo_diversity_loss`` is compared with.  It is
never imported by the product package.  Functions are dtype-generic torch code (fp64 for the
truth, fp32 for the "plain PyTorch fp32" comparison) and cite the reference lines they restate
(paths relative to the reference checkout).

Pins (tests/test_oracle_koleo.py): a plain-Python double loop over the rows, closed forms (two rows:
relu(cos + 1); an orthonormal set: 1; duplicated rows: 2; antipodal pair among orthogonal rows),
invariance under positive row scaling, orthogonal maps and row permutations, finite-difference
gradcheck of the restated analytic backward, and x . dL/dx = 0 per row (degree-0 homogeneity).
The reference holds no test or golden vector for this function, so parity with its runtime
output is unpinned by the reference itself; these pins replace it.
"""
from __future__ import annotations

import math
from typing import Tuple

import torch

Tensor = torch.Tensor
NORM_EPS = 1e-12  # torch.nn.functional.normalize's default, which src/igs/reg.py:22 relies on


def normalize_rows(features: Tensor) -> Tuple[Tensor, Tensor]:
    """x / max(||x||_2, 1e-12) along the last axis (src/igs/reg.py:22); also returns the
    clamped norms [B, N, 1]."""
    norm = features.pow(2).sum(-1, keepdim=True).sqrt().clamp_min(NORM_EPS)
    return features / norm, norm


def koleo_diversity_loss(features: Tensor) -> Tensor:
    """mean_i relu(max_{j != i} cos(x_i, x_j) + 1) over all B*N rows; src/igs/reg.py:18-40.
    N <= 1 gives 0 (:19-20)."""
    n = features.shape[1]
    if n <= 1:
        return torch.zeros((), dtype=features.dtype, device=features.device)
    fn, _ = normalize_rows(features)
    sim = fn @ fn.transpose(1, 2)                                    # :25
    eye = torch.eye(n, dtype=torch.bool, device=features.device)
    sim = sim.masked_fill(eye, -math.inf)                            # :28
    nearest = sim.max(dim=-1).values                                 # :31
    return torch.relu(nearest + 1.0).mean()                          # :35-37


def nearest_neighbours(features: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """(nearest similarity [B,N], index of that neighbour [B,N] (lowest index among equals), gap
    to the second-nearest similarity [B,N]).  The gap tells a test which rows an fp32 evaluation
    may legitimately assign to another neighbour."""
    n = features.shape[1]
    fn, _ = normalize_rows(features)
    sim = fn @ fn.transpose(1, 2)
    eye = torch.eye(n, dtype=torch.bool, device=features.device)
    sim = sim.masked_fill(eye, -math.inf)
    top = sim.topk(min(2, n - 1), dim=-1)
    val = top.values[..., 0]
    # lowest index among equal maxima
    idx = (sim == val[..., None]).to(torch.int64).argmax(dim=-1)
    gap = val - top.values[..., 1] if n > 2 else torch.full_like(val, math.inf)
    return val, idx, gap


def koleo_backward(features: Tensor, grad_loss: float = 1.0, neighbours: Tensor = None) -> Tensor:
    """Analytic gradient of koleo_diversity_loss, restated from the chain of src/igs/reg.py:22-37:
    with j(i) the nearest neighbour of row i, gate_i = [sim_i + 1 > 0] and c = grad / (B N),
      d fn_i = c gate_i fn_j(i) + c sum_{k: j(k) = i} gate_k fn_k      (max, bmm)
      d x_i  = (d fn_i - fn_i <fn_i, d fn_i>) / ||x_i||               (normalize; ||x|| > 1e-12)
      d x_i  = d fn_i / 1e-12                                          (otherwise: the clamp is constant).
    `neighbours` [B,N] overrides j(i): a test passes the choice an fp32 evaluation made among
    similarities that are equal to rounding, so that the rest of the chain is compared exactly."""
    b, n, d = features.shape
    if n <= 1:
        return torch.zeros_like(features)
    fn, norm = normalize_rows(features)
    val, idx, _ = nearest_neighbours(features)
    if neighbours is not None:
        idx = neighbours.to(torch.int64)
        val = (fn * torch.gather(fn, 1, idx[..., None].expand(b, n, d))).sum(-1)
    gate = (val + 1.0 > 0).to(features.dtype)
    c = grad_loss / (b * n)
    pulled = torch.gather(fn, 1, idx[..., None].expand(b, n, d)) * gate[..., None]
    dfn = pulled.clone()
    dfn.scatter_add_(1, idx[..., None].expand(b, n, d), fn * gate[..., None])
    dfn = dfn * c
    raw = features.pow(2).sum(-1, keepdim=True).sqrt()
    proj = (dfn - fn * (fn * dfn).sum(-1, keepdim=True)) / norm
    return torch.where(raw > NORM_EPS, proj, dfn / NORM_EPS)


def koleo_loops(features) -> float:
    """The same loss by plain Python loops over nested lists [B][N][D] (brute force for tiny
    inputs; shares no code with the tensor version)."""
    total, rows = 0.0, 0
    for img in features:
        unit = []
        for row in img:
            nrm = max(math.sqrt(sum(v * v for v in row)), NORM_EPS)
            unit.append([v / nrm for v in row])
        for i, u in enumerate(unit):
            best = -math.inf
            for j, w in enumerate(unit):
                if j != i:
                    best = max(best, sum(p * q for p, q in zip(u, w)))
            total += max(best + 1.0, 0.0)
            rows += 1
    return total / rows


def autograd_gradient(features: Tensor, grad_loss: float = 1.0) -> Tuple[Tensor, Tensor]:
    """(loss, d loss / d features) by torch autograd of koleo_diversity_loss."""
    x = features.detach().clone().requires_grad_(True)
    loss = koleo_diversity_loss(x)
    (g,) = torch.autograd.grad(loss * grad_loss, x)
    return loss.detach(), g
