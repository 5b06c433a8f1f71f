"""CPU baseline: the reference's chunked torch autograd path, restated (TEST/BENCH
INFRASTRUCTURE ONLY -- never on the product path).

Follows the structure of `GaussianSplatting2DChunkedKernel` (src/igs/gs2d.py:265-465,
N_CHUNK_SIZE = 32 at :273): per chunk of 32 Gaussians a [B,32,H,W] weight block, an
einsum into the [B,C,H,W] accumulator in the forward (:296-323), and a recomputing
hand-written backward (:374-453).  One deliberate difference: the d/d(den) term is
-<g^, out> (the reference uses grad*grad at :370, which is not the derivative of the
forward expression; the naive expression under autograd is the oracle).  `out` is therefore
saved next to `weight_sum`.  Eager torch ops, so it uses however many host threads torch
has been given.
"""
from __future__ import annotations

import torch

N_CHUNK_SIZE = 32


def _block(x, y, position, a, b_, d, alphas, lo, hi):
    dx = x - position[:, lo:hi, 0, None, None]
    dy = y - position[:, lo:hi, 1, None, None]
    q = a[:, lo:hi] * dx.square() + d[:, lo:hi] * dy.square() + b_[:, lo:hi] * (2 * dx * dy)
    e = torch.exp(-0.5 * q)
    return dx, dy, e, e * alphas[:, lo:hi, None, None]


class ChunkedCPUSplat(torch.autograd.Function):
    """`.apply(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors, eps)`
    with x, y [B,1,H,W]; cov_inv_* [B,N,1,1]; same 9-tuple backward as the reference."""

    @staticmethod
    def forward(ctx, x, y, position, a, b_, d, alphas, colors, eps=1e-6):
        B, _, H, W = x.shape
        N, C = colors.shape[1:]
        num = x.new_zeros(B, C, H, W)
        den = x.new_zeros(B, H, W)
        for lo in range(0, N, N_CHUNK_SIZE):
            hi = min(lo + N_CHUNK_SIZE, N)
            _, _, _, w = _block(x, y, position, a, b_, d, alphas, lo, hi)
            num += torch.einsum("bnhw,bnc->bchw", w, colors[:, lo:hi])
            den += w.sum(dim=1)
        out = num / (den + eps)[:, None]
        ctx.save_for_backward(x, y, position, a, b_, d, alphas, colors, den, out)
        ctx.eps = eps
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, y, position, a, b_, d, alphas, colors, den, out = ctx.saved_tensors
        N = position.shape[1]
        gx, gy = torch.zeros_like(x), torch.zeros_like(y)
        gpos = torch.zeros_like(position)
        gA, gB, gD = torch.zeros_like(a), torch.zeros_like(b_), torch.zeros_like(d)
        galpha, gcol = torch.zeros_like(alphas), torch.zeros_like(colors)
        gh = grad_out / (den + ctx.eps)[:, None]             # [B,C,H,W]
        gden = -(gh * out).sum(dim=1)                        # [B,H,W]
        for lo in range(0, N, N_CHUNK_SIZE):
            hi = min(lo + N_CHUNK_SIZE, N)
            dx, dy, e, w = _block(x, y, position, a, b_, d, alphas, lo, hi)
            G = torch.einsum("bchw,bnc->bnhw", gh, colors[:, lo:hi]) + gden[:, None]
            gcol[:, lo:hi] = (gh[:, None] * w[:, :, None]).sum(dim=(3, 4))
            galpha[:, lo:hi] = (G * e).sum(dim=(2, 3))
            cf = G * w * (-0.5)
            ddx = cf * (2 * a[:, lo:hi] * dx + 2 * b_[:, lo:hi] * dy)
            ddy = cf * (2 * d[:, lo:hi] * dy + 2 * b_[:, lo:hi] * dx)
            gx += ddx.sum(dim=1, keepdim=True)
            gy += ddy.sum(dim=1, keepdim=True)
            gpos[:, lo:hi, 0] = -ddx.sum(dim=(2, 3))
            gpos[:, lo:hi, 1] = -ddy.sum(dim=(2, 3))
            gA[:, lo:hi] = (cf * dx.square()).sum(dim=(2, 3), keepdim=True)
            gD[:, lo:hi] = (cf * dy.square()).sum(dim=(2, 3), keepdim=True)
            gB[:, lo:hi] = (cf * (2 * dx * dy)).sum(dim=(2, 3), keepdim=True)
        return gx, gy, gpos, gA, gB, gD, galpha, gcol, None


def render_chunked_cpu(positions, colors, scales, rotations, alphas, x_grid, y_grid, eps=1e-6):
    """Function-level CPU path: covariance preamble by the matrix route
    (src/igs/gs2d.py:548-580) followed by the chunked operator."""
    from .gs2d_oracle import cov_inverse_matrix

    a, b_, d = cov_inverse_matrix(scales, rotations, eps)
    return ChunkedCPUSplat.apply(x_grid, y_grid, positions, a, b_, d, alphas, colors, eps)
