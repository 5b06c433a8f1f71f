"""`koleo_diversity_loss` of the reference (src/igs/reg.py:5-40) on the HIP library.

loss = mean over the B*N rows of relu(max_{j != i} cos(x_i, x_j) + 1).  The reference forms the
whole [B, N, N] similarity matrix (bmm, diagonal fill, row max) under `torch.compile`; here the
row maxima come out of a tiled kernel that never stores the matrix, and the backward sends the
gradient through each row's nearest neighbour only, as autograd does for `max`.  Eager callers go
through a `torch.autograd.Function`; under `torch.compile` the same two library calls are the
registered operators `igs_amd::koleo_fwd` / `igs_amd::koleo_bwd`.  There is no CPU path: tensors
must live on the GPU.
"""
from __future__ import annotations

from typing import List

import torch

from . import _lib
from ._splat import _ptr, _stream, require_gpu

Tensor = torch.Tensor


def saved_numel(B: int, N: int, D: int) -> int:
    """float32 elements of the buffer kept for the backward (`saved_bytes` of igs_koleo_plan,
    restated so that shape inference needs no library call): the normalised rows padded to a
    multiple of 4 floats, then norm, nearest similarity and neighbour index per row."""
    rows = B * N
    return rows * ((D + 3) // 4 * 4) + 3 * ((rows + 3) // 4 * 4)


def _forward(features: Tensor) -> List[Tensor]:
    require_gpu(features)
    B, N, D = features.shape
    p = _lib.koleo_plan(B, N, D)
    dev = features.device
    with torch.cuda.device(dev):
        x = features.detach()
        if x.dtype != torch.float32 or not x.is_contiguous():
            x = x.to(torch.float32).contiguous()
        loss = torch.empty((), device=dev, dtype=torch.float32)
        saved = torch.empty(p.saved_bytes // 4, device=dev, dtype=torch.float32)
        scratch = torch.empty((p.scratch_bytes + 7) // 8, device=dev, dtype=torch.float64)
        _lib.check(_lib.load().igs_koleo_forward(_ptr(x), B, N, D, _ptr(loss), _ptr(saved), p.saved_bytes,
                                                  _ptr(scratch), p.scratch_bytes, _stream(dev)),
                   "igs_koleo_forward")
    return [loss, saved]


def _backward_call(saved: Tensor, grad_loss: Tensor, B: int, N: int, D: int) -> Tensor:
    require_gpu(saved)
    dev = saved.device
    with torch.cuda.device(dev):
        g = grad_loss.detach().to(torch.float32).reshape(1).contiguous()
        out = torch.empty(B, N, D, device=dev, dtype=torch.float32)
        _lib.check(_lib.load().igs_koleo_backward(_ptr(saved), saved.numel() * 4, _ptr(g), B, N, D, _ptr(out),
                                                   _stream(dev)), "igs_koleo_backward")
    return out


class _Koleo(torch.autograd.Function):
    """Eager path: the same two library calls without the operator dispatch (tens of microseconds
    per call, which is most of the cost at the sizes the loss is used at)."""

    @staticmethod
    def forward(ctx, features):
        loss, saved = _forward(features)
        ctx.dims = tuple(features.shape)
        ctx.save_for_backward(saved)
        return loss

    @staticmethod
    def backward(ctx, g_loss):
        (saved,) = ctx.saved_tensors
        return _backward_call(saved, g_loss, *ctx.dims)


@torch.library.custom_op("igs_amd::koleo_fwd", mutates_args=(), device_types="cuda")
def koleo_fwd(features: Tensor) -> List[Tensor]:
    """[loss (0-dim fp32), saved] for fp32 contiguous features [B, N >= 2, D]."""
    return _forward(features)


@koleo_fwd.register_fake
def _(features):
    B, N, D = features.shape
    return [features.new_empty((), dtype=torch.float32),
            features.new_empty((saved_numel(B, N, D),), dtype=torch.float32)]


@torch.library.custom_op("igs_amd::koleo_bwd", mutates_args=(), device_types="cuda")
def koleo_bwd(saved: Tensor, grad_loss: Tensor, B: int, N: int, D: int) -> Tensor:
    return _backward_call(saved, grad_loss, B, N, D)


@koleo_bwd.register_fake
def _(saved, grad_loss, B, N, D):
    return saved.new_empty((B, N, D), dtype=torch.float32)


def _setup_context(ctx, inputs, output):
    (features,) = inputs
    ctx.dims = tuple(features.shape)
    ctx.save_for_backward(output[1])


def _backward(ctx, grads):
    g_loss = grads[0]
    if g_loss is None:
        return None
    (saved,) = ctx.saved_tensors
    return torch.ops.igs_amd.koleo_bwd(saved, g_loss, *ctx.dims)


koleo_fwd.register_autograd(_backward, setup_context=_setup_context)


def koleo_nearest_neighbours(features: Tensor):
    """(similarity [B,N] fp32, index [B,N] int32) of each row's nearest neighbour by cosine
    similarity, as the loss kernels found them; the index is -1 where similarity + 1 <= 0 (relu
    passes no gradient there).  No gradient flows through this call."""
    B, N, D = features.shape
    if N < 2:
        raise ValueError("nearest neighbours need N >= 2")
    saved = torch.ops.igs_amd.koleo_fwd(features.detach().to(torch.float32).contiguous())[1]
    rows = B * N
    rp = (rows + 3) // 4 * 4
    off = rows * ((D + 3) // 4 * 4) + rp
    val = saved[off:off + rows].view(B, N)
    idx = saved[off + rp:off + rp + rows].view(torch.int32).view(B, N)
    return val, idx


def koleo_diversity_loss(features: Tensor) -> Tensor:
    """Drop-in for src/igs/reg.py:6: features [B, N, D] -> scalar loss in features.dtype.

    N <= 1 returns a constant 0 like the reference (:19-20).  Among equal similarities the
    gradient goes to the neighbour with the lowest index."""
    if features.dim() != 3:
        raise ValueError(f"features must be [B, N, D], got {tuple(features.shape)}")
    B, N, D = features.shape
    if N <= 1 or B == 0 or D == 0:
        if N <= 1:
            return torch.tensor(0.0, device=features.device)
        # no rows / no dimensions: what the plain expression gives (mean of nothing is NaN; zero
        # vectors normalise to zero, every similarity is 0, loss 1)
        return (features.sum() * 0 + (float("nan") if B == 0 else 1.0)).to(features.dtype)
    x = features.to(torch.float32).contiguous()
    if torch.compiler.is_compiling():
        loss = torch.ops.igs_amd.koleo_fwd(x)[0]
    else:
        loss = _Koleo.apply(x)
    return loss if features.dtype == torch.float32 else loss.to(features.dtype)
