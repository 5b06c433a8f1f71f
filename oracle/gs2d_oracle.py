"""CPU restatement of the reference's 2-D Gaussian splatting (TEST INFRASTRUCTURE ONLY).

This file is the checker that the HIP path is compared with.  It is never imported by the
product package; the product fails loudly when its HIP library is missing instead of
falling back to anything in here.

Every function cites the reference lines it restates (paths relative to the reference
checkout).  All functions are dtype-generic torch code: call them with float64 tensors to
obtain the fp64 truth and with float32 tensors for the "naive PyTorch fp32" comparison.

Pins (see tests/test_oracle.py): a scalar brute-force triple loop in plain C
(oracle/gs2d_bruteforce.c) and in Python, the N=1 closed form, colour-constancy,
permutation/zero-alpha/translation/rotation invariants, matrix-route vs closed-form
covariance inverse, finite-difference gradcheck of the analytic backward, Euler and
translation identities of the gradients.  The reference ships no golden vectors or tests
for this path, so parity with the reference's *runtime* output is unpinned by the
reference itself; these mathematical pins replace it.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Tuple

import torch

Tensor = torch.Tensor


# --------------------------------------------------------------------------------------
# covariance inverse
# --------------------------------------------------------------------------------------
def cov_inverse_matrix(scales: Tensor, rotations: Tensor, eps: float = 1e-6):
    """(R S S^T R^T + eps I)^-1 by the matrix route; follows src/igs/gs2d.py:548-580.

    The reference builds ``scale_matrices`` and ``eye`` without a dtype (:561, :572), so
    it cannot run in fp64; this restatement creates them in the input dtype.
    Returns (cov_inv_00, cov_inv_01, cov_inv_11), each [B, N, 1, 1].
    """
    b, ng, _ = scales.shape
    c, s = torch.cos(rotations), torch.sin(rotations)
    rot = torch.stack([torch.stack([c, -s], dim=2), torch.stack([s, c], dim=2)], dim=2)
    sm = torch.zeros(b, ng, 2, 2, dtype=scales.dtype, device=scales.device)
    sm = sm + torch.diag_embed(scales)
    rs = torch.bmm(rot.flatten(0, 1), sm.flatten(0, 1))
    cov = torch.bmm(rs, rs.transpose(-2, -1)).unflatten(0, (b, ng))
    eye = torch.eye(2, dtype=cov.dtype, device=cov.device).expand(b, ng, -1, -1)
    inv = torch.inverse(cov + eps * eye)
    return (
        inv[..., 0, 0, None, None],
        inv[..., 0, 1, None, None],
        inv[..., 1, 1, None, None],
    )


def cov_inverse_closed(scales: Tensor, rotations: Tensor, eps: float = 1e-6):
    """Closed form of the same inverse: Sigma + eps I = R diag(s0^2+eps, s1^2+eps) R^T.

    A = c^2 i0 + s^2 i1, B = c s (i0 - i1), D = s^2 i0 + c^2 i1, i_k = 1/(s_k^2 + eps).
    Equivalent to src/igs/gs2d.py:548-580.  Returns three [B, N, 1, 1] tensors.
    """
    c, s = torch.cos(rotations), torch.sin(rotations)
    i0 = 1.0 / (scales[..., 0] ** 2 + eps)
    i1 = 1.0 / (scales[..., 1] ** 2 + eps)
    a = c * c * i0 + s * s * i1
    b = c * s * (i0 - i1)
    d = s * s * i0 + c * c * i1
    return a[..., None, None], b[..., None, None], d[..., None, None]


# --------------------------------------------------------------------------------------
# forward
# --------------------------------------------------------------------------------------
def naive_gaussian_2d(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors,
                      eps: float = 1e-6) -> Tensor:
    """Normative expression; follows src/igs/gs2d.py:24-44 (README.md:66-103).

    x, y [B,1,H,W]; position [B,N,2]; cov_inv_* [B,N,1,1]; alphas [B,N]; colors [B,N,C].
    Materialises the [B,N,H,W] weight, so only for sizes where that fits.
    """
    dx = x - position[..., 0, None, None]
    dy = y - position[..., 1, None, None]
    q = dx * dx * cov_inv_00 + 2 * dx * dy * cov_inv_01 + dy * dy * cov_inv_11
    weight = torch.exp(-0.5 * q) * alphas[..., None, None]
    weight_sum = weight.sum(dim=1, keepdim=True)
    b, ng, h, w = weight.shape
    nw = (weight / (weight_sum + eps)).permute(0, 2, 3, 1).flatten(1, 2)
    result = torch.bmm(nw, colors)
    return result.unflatten(1, (h, w)).permute(0, 3, 1, 2)


def render_naive(positions, colors, scales, rotations, alphas, x_grid, y_grid,
                 eps: float = 1e-6, closed_form: bool = False) -> Tensor:
    """`render(..., fused=False)`; follows src/igs/gs2d.py:524-609."""
    f = cov_inverse_closed if closed_form else cov_inverse_matrix
    a, b, d = f(scales, rotations, eps)
    return naive_gaussian_2d(x_grid, y_grid, positions, a, b, d, alphas, colors, eps)


def _as4(g: Tensor, b: int) -> Tensor:
    if g.dim() == 3:
        g = g[:, None]
    if g.shape[0] == 1 and b > 1:
        g = g.expand(b, -1, -1, -1)
    return g


def forward_strips(x, y, position, a, b_, d, alphas, colors, eps=1e-6, rows=8):
    """Same expression evaluated per image and per strip of rows (pixels are independent),
    so that large shapes fit.  Returns (out [B,C,H,W], den [B,H,W])."""
    B, N, C = colors.shape
    x, y = _as4(x, B), _as4(y, B)
    H, W = x.shape[-2:]
    out = torch.empty(B, C, H, W, dtype=x.dtype, device=x.device)
    den = torch.empty(B, H, W, dtype=x.dtype, device=x.device)
    for ib in range(B):
        for r0 in range(0, H, rows):
            xs, ys = x[ib, :, r0:r0 + rows], y[ib, :, r0:r0 + rows]   # [1,r,W]
            dx = xs - position[ib, :, 0, None, None]
            dy = ys - position[ib, :, 1, None, None]
            q = dx * dx * a[ib] + 2 * dx * dy * b_[ib] + dy * dy * d[ib]
            wgt = torch.exp(-0.5 * q) * alphas[ib, :, None, None]        # [N,r,W]
            s = wgt.sum(0)
            num = torch.einsum("nhw,nc->chw", wgt, colors[ib])
            den[ib, r0:r0 + rows] = s
            out[ib, :, r0:r0 + rows] = num / (s + eps)
    return out, den


# --------------------------------------------------------------------------------------
# backward, analytic (closed form); pinned by autograd of the naive expression and by
# finite differences in tests/test_oracle.py
# --------------------------------------------------------------------------------------
def backward_strips(x, y, position, a, b_, d, alphas, colors, grad_out, eps=1e-6, rows=8,
                    grid_grads: bool = False) -> Dict[str, Tensor]:
    """Gradients of sum(out * grad_out) w.r.t. the operator inputs.

    With g^ = g/(den+eps), s = <g^, out>, G_n = <g^, c_n> - s, w_n = alpha_n e_n:
      d alpha_n = sum_px G e        d color_nc = sum_px g^_c w
      d px = sum G w (A dx + B dy)  d py = sum G w (B dx + D dy)
      d A = sum -1/2 G w dx^2       d B = sum -G w dx dy      d D = sum -1/2 G w dy^2
      d x_px = -sum_n G w (A dx + B dy), d y_px likewise.
    (The hand-written backward in src/igs/gs2d.py:176,370 uses grad*grad for the d/d den
    term and is not followed; the naive expression under autograd is the reference.)
    """
    B, N, C = colors.shape
    x, y = _as4(x, B), _as4(y, B)
    H, W = x.shape[-2:]
    dt, dev = x.dtype, x.device
    g = dict(
        position=torch.zeros(B, N, 2, dtype=dt, device=dev),
        cov_inv_00=torch.zeros(B, N, dtype=dt, device=dev),
        cov_inv_01=torch.zeros(B, N, dtype=dt, device=dev),
        cov_inv_11=torch.zeros(B, N, dtype=dt, device=dev),
        alphas=torch.zeros(B, N, dtype=dt, device=dev),
        colors=torch.zeros(B, N, C, dtype=dt, device=dev),
    )
    if grid_grads:
        g["x"] = torch.zeros(B, 1, H, W, dtype=dt, device=dev)
        g["y"] = torch.zeros(B, 1, H, W, dtype=dt, device=dev)
    for ib in range(B):
        A, Bc, D = a[ib].reshape(N, 1, 1), b_[ib].reshape(N, 1, 1), d[ib].reshape(N, 1, 1)
        for r0 in range(0, H, rows):
            xs, ys = x[ib, :, r0:r0 + rows], y[ib, :, r0:r0 + rows]
            dx = xs - position[ib, :, 0, None, None]
            dy = ys - position[ib, :, 1, None, None]
            e = torch.exp(-0.5 * (dx * dx * A + 2 * dx * dy * Bc + dy * dy * D))
            wgt = e * alphas[ib, :, None, None]
            den = wgt.sum(0) + eps
            out = torch.einsum("nhw,nc->chw", wgt, colors[ib]) / den
            gh = grad_out[ib, :, r0:r0 + rows] / den                      # [C,r,W]
            s = (gh * out).sum(0)
            G = torch.einsum("chw,nc->nhw", gh, colors[ib]) - s
            Gw = G * wgt
            lx = A * dx + Bc * dy
            ly = Bc * dx + D * dy
            g["alphas"][ib] += (G * e).sum((1, 2))
            g["colors"][ib] += torch.einsum("chw,nhw->nc", gh, wgt)
            g["position"][ib, :, 0] += (Gw * lx).sum((1, 2))
            g["position"][ib, :, 1] += (Gw * ly).sum((1, 2))
            g["cov_inv_00"][ib] += (-0.5 * Gw * dx * dx).sum((1, 2))
            g["cov_inv_01"][ib] += (-Gw * dx * dy).sum((1, 2))
            g["cov_inv_11"][ib] += (-0.5 * Gw * dy * dy).sum((1, 2))
            if grid_grads:
                g["x"][ib, 0, r0:r0 + rows] = -(Gw * lx).sum(0)
                g["y"][ib, 0, r0:r0 + rows] = -(Gw * ly).sum(0)
    return g


def chain_to_scale_rotation(scales, rotations, gA, gB, gD, eps=1e-6):
    """Chain rule from (dA, dB, dD) to (d scales [B,N,2], d rotations [B,N]) through the
    closed form of cov_inverse_closed."""
    c, s = torch.cos(rotations), torch.sin(rotations)
    i0 = 1.0 / (scales[..., 0] ** 2 + eps)
    i1 = 1.0 / (scales[..., 1] ** 2 + eps)
    gi0 = gA * c * c + gB * c * s + gD * s * s
    gi1 = gA * s * s - gB * c * s + gD * c * c
    gs = torch.stack([gi0 * (-2 * scales[..., 0] * i0 * i0),
                      gi1 * (-2 * scales[..., 1] * i1 * i1)], dim=-1)
    Bv = c * s * (i0 - i1)
    gth = (gD - gA) * 2 * Bv + gB * (c * c - s * s) * (i0 - i1)
    return gs, gth


def render_backward_strips(positions, colors, scales, rotations, alphas, x_grid, y_grid,
                           grad_out, eps=1e-6, rows=8) -> Dict[str, Tensor]:
    """Gradients w.r.t. the function-level inputs (positions, colors, scales, rotations,
    alphas), evaluated in strips."""
    a, b_, d = cov_inverse_closed(scales, rotations, eps)
    g = backward_strips(x_grid, y_grid, positions, a, b_, d, alphas, colors, grad_out, eps, rows)
    gs, gth = chain_to_scale_rotation(scales, rotations, g["cov_inv_00"], g["cov_inv_01"],
                                      g["cov_inv_11"], eps)
    return dict(positions=g["position"], colors=g["colors"], scales=gs, rotations=gth,
                alphas=g["alphas"])


def render_autograd(positions, colors, scales, rotations, alphas, x_grid, y_grid, grad_out,
                    eps=1e-6, closed_form=False) -> Tuple[Tensor, Dict[str, Tensor]]:
    """Naive expression under torch autograd (the stated gradient oracle when run in
    fp64).  Returns (out, grads)."""
    leaves = dict(positions=positions, colors=colors, scales=scales, rotations=rotations,
                  alphas=alphas)
    leaves = {k: v.detach().clone().requires_grad_(True) for k, v in leaves.items()}
    out = render_naive(leaves["positions"], leaves["colors"], leaves["scales"],
                       leaves["rotations"], leaves["alphas"], x_grid, y_grid, eps, closed_form)
    gr = torch.autograd.grad(out, list(leaves.values()), grad_out)
    return out.detach(), dict(zip(leaves.keys(), gr))


def operator_autograd(x, y, position, a, b_, d, alphas, colors, grad_out, eps=1e-6):
    """Naive operator-level expression under autograd, all 8 tensor inputs as leaves."""
    names = ["x", "y", "position", "cov_inv_00", "cov_inv_01", "cov_inv_11", "alphas", "colors"]
    leaves = [t.detach().clone().requires_grad_(True) for t in (x, y, position, a, b_, d, alphas, colors)]
    out = naive_gaussian_2d(*leaves, eps)
    gr = torch.autograd.grad(out, leaves, grad_out)
    return out.detach(), dict(zip(names, gr))


# --------------------------------------------------------------------------------------
# scalar brute force (tiny inputs only) -- an independent pin for the vectorised code
# --------------------------------------------------------------------------------------
REACH_Q = 160.0 / (0.5 * math.log2(math.e))   # q beyond which the fp32 kernels' exp2 argument is < -160


EXACT_LIMIT = 155.0                           # tile-test limit (in units of -q') when only exact zeros are skipped


def skip_weight(N: int, eps: float, tolerance: float) -> float:
    """Weight below which a (Gaussian, pixel) pair may be skipped so that no output element moves by
    more than tolerance * max|colors|: with every skipped |alpha e| <= w, a pixel's numerator loses
    at most N w max|c| and its denominator at most N w, hence
    |d out| <= N w (max|c| + |out|) / (den + eps) <= 2 N w max|c| / eps  (den >= 0, |out| <= max|c|),
    which is the tolerance for w = tolerance eps / (2 N).  Test infrastructure's restatement of
    igs_gs2d_skip_weight (no counterpart in the reference, which evaluates every pair:
    src/igs/gs_triton_chunked.py:100-200)."""
    if not (tolerance > 0 and eps > 0 and N > 0):
        return 0.0
    return min(tolerance * eps / (2.0 * N), 0.5)


def skip_limit(alphas, w: float):
    """Per-Gaussian limit L_n on -q' = 0.5 log2(e) q beyond which the kernels may skip a pair:
    e = 2^q' < w / max(1, |alpha_n|)  <=>  -q' > -log2 w + log2 max(1, |alpha_n|), capped at the
    exact-zero limit; w = 0 is that cap."""
    if w <= 0:
        return torch.full_like(alphas, EXACT_LIMIT)
    return torch.clamp(-math.log2(w) + torch.log2(torch.clamp(alphas.abs(), min=1.0)), max=EXACT_LIMIT)


def tile_weight_floor(px, py, a, b_, d, alphas, xlo, xhi, ylo, yhi):
    """Lower bound of the denominator sum_n alpha_n exp(-q_n / 2) at every point of the rectangle
    [xlo, xhi] x [ylo, yhi], for alphas >= 0 (else 0): q_n is convex, so its maximum over the
    rectangle is at a corner and exp(-max q_n / 2) is the least weight Gaussian n has on it.
    Sums over the last dimension of the Gaussian tensors.  Test infrastructure's restatement of the
    per-tile bound of the HIP binning kernel (no counterpart in the reference)."""
    if bool((alphas < 0).any()) or not bool(torch.isfinite(alphas).all()):
        return torch.zeros(alphas.shape[:-1], dtype=alphas.dtype)
    qmax = None
    for xe in (xlo, xhi):
        for ye in (ylo, yhi):
            dx, dy = xe - px, ye - py
            q = a * dx * dx + 2 * b_ * dx * dy + d * dy * dy
            qmax = q if qmax is None else torch.maximum(qmax, q)
    return (alphas * torch.exp(-0.5 * qmax)).sum(-1)


def tile_skip_weight(w: float, f: float, floor):
    """Weight below which pairs of a tile may be skipped: the call's skip weight plus the skip
    fraction of the tile's denominator floor.  With w = tolerance eps / (2 N), f = tolerance / (2 N):
    N (w + f S) (max|c| + |out|) / (den + eps) <= tolerance max|c| wherever den >= S."""
    return w + f * floor


WEIGHT_CLASSES_PER_BINADE = 2


def weight_class(min_q, alphas):
    """Weight class of each (Gaussian, tile) pair from the minimum of q over the tile's rectangle
    (`min_q_over_rect`): the Gaussian's largest term of a denominator there is
    max(1, |alpha|) exp(-min_q / 2) = 2^-p, p = 0.5 log2(e) min_q - log2 max(1, |alpha|), and the
    class is floor(p R) with R classes per binade, i.e. the term lies in (2^-((k+1)/R), 2^-(k/R)].
    -1 (never skipped) where the rectangle holds the centre (min_q = 0) or the bound exceeds 1."""
    p = 0.5 * math.log2(math.e) * min_q - torch.log2(torch.clamp(alphas.abs(), min=1.0))
    k = torch.floor(p * WEIGHT_CLASSES_PER_BINADE)
    return torch.where((min_q > 0) & (p >= 0), k, torch.full_like(k, -1.0)).long()


def tile_first_skipped_class(classes, N: int, w: float, f: float, floor: float):
    """The per-tile rule of the HIP binning kernel, restated: which weight classes a tile leaves out
    of its list.  Leaving out a set of Gaussians changes a denominator of the tile by at most the sum
    of their largest terms there, and that sum may reach N (w + f S) (`tile_skip_weight` times N; S =
    `floor` bounds the tile's denominators from below): then
    |d out| <= N (w + f S) (max|c| + |out|) / (den + eps) <= tolerance max|c|.
    Classes from kbase = ceil(-log2(w) R) on hold terms of at most w and are always left out; so are
    the Gaussians that the kernel never examines for the tile (terms below w as well).  With n the
    number of classed pairs below kbase these take at most (N - n) w of the allowance, which leaves
    n w + N f S: the lightest classes below kbase are left out as long as the sum of (members x upper
    end of the class) stays within that.  Returns the first class left out (kbase if none is);
    `classes` is a 1-D integer tensor (-1 = never skipped).  w = 0: nothing but exact zeros is
    skipped, returns None.  No counterpart in the reference, which evaluates every pair
    (src/igs/gs_triton_chunked.py:100-200)."""
    R = WEIGHT_CLASSES_PER_BINADE
    if not w > 0 or -math.log2(w) >= EXACT_LIMIT:
        return None
    kbase = math.ceil(-math.log2(w) * R)
    hi = classes[(classes >= 0) & (classes < kbase)]
    budget = hi.numel() * w + N * f * floor
    hist = torch.bincount(hi, minlength=kbase).tolist()
    first, run = kbase, 0.0
    for k in range(kbase - 1, -1, -1):
        run += hist[k] * 2.0 ** (-k / R)
        if run > budget:
            break
        first = k
    return first


def backward_with_lists(x, y, position, a, b_, d, alphas, colors, grad_out, eps, keep_fwd, keep_bwd):
    """What the kernels compute when lists leave pairs out, restated densely (small inputs only):
    the forward sums the pairs of `keep_fwd` [B,N,H,W] (bool), the backward takes that forward's
    image and denominator and sums, for every Gaussian, the pairs of `keep_bwd`; the formulas are
    those of `backward_strips`.  With both masks all true this is `backward_strips` itself.
    Returns (out, grads).  No counterpart in the reference, which evaluates every pair
    (src/igs/gs_triton_chunked.py:100-200)."""
    B, N, C = colors.shape
    x, y = _as4(x, B), _as4(y, B)
    A, Bc, D = (t.reshape(B, N, 1, 1) for t in (a, b_, d))
    dx = x - position[..., 0, None, None]
    dy = y - position[..., 1, None, None]
    e = torch.exp(-0.5 * (dx * dx * A + 2 * dx * dy * Bc + dy * dy * D))
    wgt = e * alphas[..., None, None]
    wf = wgt * keep_fwd
    den = wf.sum(1, keepdim=True) + eps                                   # [B,1,H,W]
    out = torch.einsum("bnhw,bnc->bchw", wf, colors) / den
    gh = grad_out / den
    G = torch.einsum("bchw,bnc->bnhw", gh, colors) - (gh * out).sum(1, keepdim=True)
    G = G * keep_bwd
    Gw = G * wgt
    lx, ly = A * dx + Bc * dy, Bc * dx + D * dy
    grads = dict(
        position=torch.stack([(Gw * lx).sum((2, 3)), (Gw * ly).sum((2, 3))], dim=-1),
        cov_inv_00=(-0.5 * Gw * dx * dx).sum((2, 3)),
        cov_inv_01=(-Gw * dx * dy).sum((2, 3)),
        cov_inv_11=(-0.5 * Gw * dy * dy).sum((2, 3)),
        alphas=(G * e).sum((2, 3)),
        colors=torch.einsum("bchw,bnhw->bnc", gh, wgt * keep_bwd),
    )
    return out, grads


def culling_gradient_bound(x, y, position, a, b_, d, alphas, colors, grad_out, eps, tolerance):
    """How far the lists can move a gradient, for alphas >= 0 (so every denominator is >= 0 and
    |out| <= max|c|).  Write D = den + eps, g1 = sum_c |g_c| of a pixel, K = max|c| + max|out|,
    m_n = max(1, alpha_n).  Per pixel the largest terms u_n of the Gaussians a tile leaves out add up
    to at most the allowance A = N (w + f S) <= tolerance D (`tile_first_skipped_class`; both the
    forward's and the backward's tiling keep to it, each with its own floor S).

    The kernels' gradient of a parameter th of Gaussian n is sum over the backward's kept pixels of
    G' dw/dth with G' = <g, c_n - out'> / D' taken from the forward's own (culled) image.  Against
    the sum over all pixels of G dw/dth it differs by
      (1) the pairs the backward leaves out.  |G| <= g1 K / D and, with e <= u / m, q >= 2 ln(m / u):
          e q^k <= (u / m) (2 ln(m / u) + 2 k)^k  (e q^k falls beyond q = 2 k, where it is (2 k / e)^k),
          |dw/dth| <= |w| P_th q^k  with  (P, k) = (1 / m, 0) for alpha (dw/dalpha = e),
          (sqrt(A), 1/2), (sqrt(D), 1/2) for the position (Cauchy-Schwarz in the metric of q),
          (Sxx / 2, 1), (sqrt(Sxx Syy), 1), (Syy / 2, 1) for cov_inv_00 / 01 / 11 (S the covariance:
          dx^2 <= q Sxx, dy^2 <= q Syy), and for a colour |g_c| |w| / D.
          u (2 ln(m / u) + 2 k)^k grows with u and is concave on u <= m (k <= 1), the u_n of a pixel
          add up to at most tolerance D and D >= eps, so (Jensen) over ALL Gaussians
              sum_n |(1)| / P_th,n  <=  tolerance Lam^k sum_px g1 K  =: T Lam^k,
          Lam = max(2, 2 + 2 ln(N max m / (tolerance eps)));  for the colours sum_n |(1)| <= tolerance sum |g_c|.
      (2) G' - G on the kept pairs.  With a = A / D <= tolerance: D' >= (1 - a) D,
          |1/D' - 1/D| <= a / ((1 - a) D), |out' - out| <= a K / (1 - a), hence
          |G' - G| <= tau g1 K / D with tau = tolerance (2 - tolerance) / (1 - tolerance)^2, and
              |(2)| <= tau Gam_th,n,   Gam_th,n = sum_px g1 K / D |dw_n/dth|
          -- the gradient's own sum with every term replaced by the bound of its absolute value; for
          a colour |(2)| <= tolerance / (1 - tolerance) sum_px |g_c| |w| / D  (<= tau Gam).
    So  |d th_n| <= T Lam^k P_th,n + tau Gam_th,n  for every element, and over a whole tensor
    sum_n |d th_n| / P_th,n <= T Lam^k + tau sum_n Gam_th,n / P_th,n.

    Returns (first, gamma, tau): dicts of per-element tensors first = T Lam^k P (the colours:
    tolerance sum_px |g_c|, the same for every Gaussian) and gamma = Gam, named like the gradients of
    `backward_strips`; dense evaluation, small inputs only.  No counterpart in the reference, which
    evaluates every pair (src/igs/gs_triton_chunked.py:100-200)."""
    B, N, C = colors.shape
    x, y = _as4(x, B), _as4(y, B)
    A, Bc, D = (t.reshape(B, N, 1, 1) for t in (a, b_, d))
    dx = x - position[..., 0, None, None]
    dy = y - position[..., 1, None, None]
    q = dx * dx * A + 2 * dx * dy * Bc + dy * dy * D
    e = torch.exp(-0.5 * q)
    wgt = (e * alphas[..., None, None]).abs()
    den = (e * alphas[..., None, None]).sum(1, keepdim=True) + eps
    out = torch.einsum("bnhw,bnc->bchw", e * alphas[..., None, None], colors) / den
    K = colors.abs().max() + out.abs().amax(1, keepdim=True)                # [B,1,H,W]
    g1 = grad_out.abs().sum(1, keepdim=True)
    s = g1 * K / den.abs()
    m = torch.clamp(alphas.abs(), min=1.0)
    lam = max(2.0, 2.0 + 2.0 * math.log(N * float(m.max()) / (tolerance * eps)))
    T = tolerance * (g1 * K).sum((1, 2, 3))[:, None]                        # [B,1]
    tau = tolerance * (2 - tolerance) / (1 - tolerance) ** 2
    An, Bn, Dn = (t.reshape(B, N) for t in (a, b_, d))
    det = An * Dn - Bn * Bn
    sxx, syy = Dn / det, An / det
    first = dict(
        alphas=T / m,
        position=T[..., None] * math.sqrt(lam) * torch.stack([An.sqrt(), Dn.sqrt()], dim=-1),
        cov_inv_00=T * lam * 0.5 * sxx,
        cov_inv_01=T * lam * (sxx * syy).sqrt(),
        cov_inv_11=T * lam * 0.5 * syy,
        colors=(tolerance * grad_out.abs().sum((2, 3)))[:, None, :].expand(B, N, C),
    )
    sw = s * wgt
    gamma = dict(
        alphas=(s * e).sum((2, 3)),
        position=torch.stack([(sw * (A * dx + Bc * dy).abs()).sum((2, 3)),
                              (sw * (Bc * dx + D * dy).abs()).sum((2, 3))], dim=-1),
        cov_inv_00=(0.5 * sw * dx * dx).sum((2, 3)),
        cov_inv_01=(sw * (dx * dy).abs()).sum((2, 3)),
        cov_inv_11=(0.5 * sw * dy * dy).sum((2, 3)),
        colors=torch.einsum("bchw,bnhw->bnc", grad_out.abs() / den.abs(), wgt),
    )
    return first, gamma, tau


def chain_bound_to_scale_rotation(scales, rotations, bA, bB, bD, eps=1e-6):
    """Carries element-wise bounds on the gradients of (cov_inv_00, 01, 11) to bounds on those of
    (scales [B,N,2], rotations [B,N]): `chain_to_scale_rotation` with every coefficient replaced by
    its absolute value (the chain is linear per Gaussian)."""
    c, s = torch.cos(rotations), torch.sin(rotations)
    i0 = 1.0 / (scales[..., 0] ** 2 + eps)
    i1 = 1.0 / (scales[..., 1] ** 2 + eps)
    bi0 = bA * c * c + bB * (c * s).abs() + bD * s * s
    bi1 = bA * s * s + bB * (c * s).abs() + bD * c * c
    bs = torch.stack([bi0 * (2 * scales[..., 0].abs() * i0 * i0),
                      bi1 * (2 * scales[..., 1].abs() * i1 * i1)], dim=-1)
    bth = (bD + bA) * 2 * (c * s * (i0 - i1)).abs() + bB * ((c * c - s * s) * (i0 - i1)).abs()
    return bs, bth


def reach_q(alphas, w: float):
    """q_max of each Gaussian's reach box under skip weight w: five binades beyond its skip limit
    (the exact-zero case gives REACH_Q)."""
    return (skip_limit(alphas, w) + 5.0) / (0.5 * math.log2(math.e))


def reach_box(position, a, b_, d, q_max=REACH_Q):
    """Axis-aligned bounding box of the ellipse q(dx, dy) = a dx^2 + 2 b dx dy + d dy^2 <= q_max
    around each Gaussian, as (xlo, xhi, ylo, yhi) [...,4].  Textbook result: the extreme of dx on
    the ellipse is sqrt(q_max * Sigma_xx) with Sigma = [[a, b], [b, d]]^-1, i.e.
    Sigma_xx = d / (a d - b^2), Sigma_yy = a / (a d - b^2).  This is the test infrastructure's
    restatement of the culling bound of the HIP pack kernels (no counterpart in the reference,
    which evaluates every pair: src/igs/gs_triton_chunked.py:100-200); pixels outside the box
    have q > q_max and therefore a weight of exactly zero in the fp32 kernels (q_max = REACH_Q) or
    one below the call's skip weight (q_max = reach_q(alphas, w), a tensor per Gaussian)."""
    a, b_, d = (t.reshape(position.shape[:-1]) for t in (a, b_, d))
    det = a * d - b_ * b_
    hx = torch.sqrt(q_max * d / det)
    hy = torch.sqrt(q_max * a / det)
    px, py = position[..., 0], position[..., 1]
    return torch.stack([px - hx, px + hx, py - hy, py + hy], dim=-1)


def min_q_over_rect(px, py, a, b_, d, xlo, xhi, ylo, yhi):
    """Minimum of q(dx, dy) = a dx^2 + 2 b dx dy + d dy^2 (positive definite) over the rectangle
    [xlo, xhi] x [ylo, yhi], dx = x - px, dy = y - py; tensors broadcast.  0 if the rectangle holds
    the centre; else the minimum of a convex function lies on the boundary, and on an edge q is a
    parabola in one variable whose vertex is clamped to the edge.  Restates the second culling test
    of the HIP binning kernel (a tile is dropped for a Gaussian when this minimum is beyond the
    zero-weight threshold); no counterpart in the reference."""
    x0, x1, y0, y1 = xlo - px, xhi - px, ylo - py, yhi - py

    def q(dx, dy):
        return a * dx * dx + 2 * b_ * dx * dy + d * dy * dy

    def clamp(v, lo, hi):
        return torch.minimum(torch.maximum(v, lo), hi)

    edges = torch.stack(torch.broadcast_tensors(
        q(x0, clamp(-b_ * x0 / d, y0, y1)), q(x1, clamp(-b_ * x1 / d, y0, y1)),
        q(clamp(-b_ * y0 / a, x0, x1), y0), q(clamp(-b_ * y1 / a, x0, x1), y1)))
    inside = (x0 <= 0) & (x1 >= 0) & (y0 <= 0) & (y1 >= 0)
    m = edges.min(dim=0).values
    return torch.where(inside, torch.zeros_like(m), m)


def brute_force_forward(x, y, position, a, b_, d, alphas, colors, eps=1e-6):
    """Plain Python triple loop over (image, pixel, gaussian) in Python floats (fp64)."""
    B, N, C = colors.shape
    x, y = _as4(x, B), _as4(y, B)
    H, W = x.shape[-2:]
    out = torch.zeros(B, C, H, W, dtype=torch.float64)
    for ib in range(B):
        for i in range(H):
            for j in range(W):
                xv, yv = float(x[ib, 0, i, j]), float(y[ib, 0, i, j])
                den, num = 0.0, [0.0] * C
                for n in range(N):
                    dx = xv - float(position[ib, n, 0])
                    dy = yv - float(position[ib, n, 1])
                    q = (float(a.reshape(B, N)[ib, n]) * dx * dx
                         + 2.0 * float(b_.reshape(B, N)[ib, n]) * dx * dy
                         + float(d.reshape(B, N)[ib, n]) * dy * dy)
                    wv = math.exp(-0.5 * q) * float(alphas[ib, n])
                    den += wv
                    for c in range(C):
                        num[c] += wv * float(colors[ib, n, c])
                for c in range(C):
                    out[ib, c, i, j] = num[c] / (den + eps)
    return out


# --------------------------------------------------------------------------------------
# grids, module head
# --------------------------------------------------------------------------------------
def xy_grid(size, dtype=torch.float32):
    """Follows src/igs/gs2d.py:503-522: x in +-sqrt(w/h), y in +-sqrt(h/w), each [1,h,w]."""
    h, w = size
    ar = h / w
    hr, wr = ar ** 0.5, 1 / ar ** 0.5
    xg = torch.linspace(-wr, wr, w, dtype=dtype).view(1, 1, w).expand(1, h, w)
    yg = torch.linspace(-hr, hr, h, dtype=dtype).view(1, h, 1).expand(1, h, w)
    return xg, yg


def module_forward(weight, bias, feature, size, num_gaussians_per_emb, output_dim=3,
                   eps=1e-6):
    """Module head + render; follows src/igs/gs2d.py:611-689 for grid=None,
    pos_map_offset=False.  Returns (image, gs_feature)."""
    gs_feature = torch.nn.functional.linear(feature, weight, bias)
    gs_feature = gs_feature.unflatten(-1, (-1, 6 + output_dim)).flatten(1, 2)
    b = gs_feature.shape[0]
    positions, log_scales, rotations, logit_opacity, colors = gs_feature.split(
        [2, 2, 1, 1, output_dim], dim=-1)
    xg, yg = xy_grid(size, dtype=feature.dtype)
    xg = xg[None].repeat(b, 1, 1, 1)
    yg = yg[None].repeat(b, 1, 1, 1)
    alphas = torch.ones_like(logit_opacity[..., 0])
    scales = torch.exp(log_scales) + eps
    img = render_naive(positions, colors, scales, rotations[..., 0], alphas, xg, yg, eps)
    return img, gs_feature


# --------------------------------------------------------------------------------------
# seeded synthetic inputs for the benchmark configurations
# --------------------------------------------------------------------------------------
CONFIGS = {
    # name: B, N, H, W, C, scale range, colour law
    "c0": dict(B=1, N=2048, H=256, W=256, C=3, smin=0.25, smax=0.75, colors="uniform"),
    "c1": dict(B=16, N=8192, H=256, W=256, C=3, smin=0.02, smax=0.3, colors="uniform"),
    "c2": dict(B=1, N=16384, H=512, W=512, C=3, smin=0.01, smax=0.1, colors="uniform"),
    "c4": dict(B=4, N=32768, H=384, W=640, C=16, smin=0.005, smax=0.05, colors="normal"),
}


def make_inputs(B, N, H, W, C, smin, smax, colors="uniform", seed=0, dtype=torch.float32,
                x_extent: Optional[float] = None, expand_grids=True):
    """Seeded inputs in the draw order positions, colors, scales, rotations, alphas,
    grad_out (CPU generator).  Grids: x = linspace(-xe, xe, W), y = linspace(-1, 1, H)
    with xe = W/H unless given (1 for square images)."""
    g = torch.Generator().manual_seed(seed)
    xe = (W / H) if x_extent is None else x_extent
    pos = torch.rand(B, N, 2, generator=g, dtype=torch.float64) * 2 - 1
    pos[..., 0] *= xe
    if colors == "uniform":
        col = torch.rand(B, N, C, generator=g, dtype=torch.float64)
    else:
        col = torch.randn(B, N, C, generator=g, dtype=torch.float64)
    sc = torch.rand(B, N, 2, generator=g, dtype=torch.float64) * (smax - smin) + smin
    rot = torch.rand(B, N, generator=g, dtype=torch.float64) * (2 * math.pi)
    al = torch.rand(B, N, generator=g, dtype=torch.float64)
    go = torch.randn(B, C, H, W, generator=g, dtype=torch.float64)
    # everything is rounded to fp32 first so that the fp64 truth and the fp32 kernels see
    # the same numbers
    t = lambda v: v.to(torch.float32).to(dtype)
    xg = torch.linspace(-xe, xe, W, dtype=torch.float32).to(dtype)
    yg = torch.linspace(-1, 1, H, dtype=torch.float32).to(dtype)
    xg = xg.view(1, 1, 1, W).expand(B, 1, H, W)     # stride 0 over B and H
    yg = yg.view(1, 1, H, 1).expand(B, 1, H, W)     # stride 0 over B and W
    if not expand_grids:
        xg, yg = xg.contiguous(), yg.contiguous()
    return dict(positions=t(pos), colors=t(col), scales=t(sc), rotations=t(rot), alphas=t(al),
                x_grid=xg, y_grid=yg, grad_out=t(go))


def make_config_inputs(name: str, dtype=torch.float32, **override):
    cfg = dict(CONFIGS[name])
    cfg.update(override)
    seed = 1000 + int(name[1:])
    return make_inputs(seed=seed, dtype=dtype, **cfg)


def smooth_noise_target(H, W, seed, C=3, dtype=torch.float32):
    """Seeded smooth target image for the single-image fit configuration: 64 random
    sinusoids, `clip(0.5 + 1/8 sum_k a_kc sin(pi (fx_k x + fy_k y) + phi_k), 0, 1)` on the
    x = linspace(-W/H, W/H, W), y = linspace(-1, 1, H) grid.  Returns [1, C, H, W]."""
    g = torch.Generator().manual_seed(seed)
    fx = torch.rand(64, generator=g, dtype=torch.float64) * 8 - 4
    fy = torch.rand(64, generator=g, dtype=torch.float64) * 8 - 4
    ph = torch.rand(64, generator=g, dtype=torch.float64) * (2 * math.pi)
    amp = torch.rand(64, C, generator=g, dtype=torch.float64)
    x = torch.linspace(-W / H, W / H, W, dtype=torch.float64).view(1, 1, W)
    y = torch.linspace(-1, 1, H, dtype=torch.float64).view(1, H, 1)
    s = torch.sin(math.pi * (fx.view(-1, 1, 1) * x + fy.view(-1, 1, 1) * y) + ph.view(-1, 1, 1))   # [64,H,W]
    img = 0.5 + 0.125 * torch.einsum("khw,kc->chw", s, amp)
    return img.clamp(0, 1)[None].to(dtype)
