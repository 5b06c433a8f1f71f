"""`torch.library` registration of the HIP splat, for callers under `torch.compile`.

The reference wraps `render` in `torch.compile(dynamic=True)` (src/igs/gs2d.py:525) and its users
compile whole models around it.  ctypes calls are opaque to Dynamo, so the splat is registered as
two operators with shape functions; Dynamo then records them as single graph nodes and AOT
autograd differentiates through `igs_amd::splat_fwd` by calling `igs_amd::splat_bwd`:

  igs_amd::splat_fwd(kind, params, x, y, eps) -> [out[B,Cp,H,W], den[B,H,W], packed, col[B,N,Cp]]
  igs_amd::splat_bwd(kind, params, x, y, packed, col, out, den, grad_out, eps, grid_grads)
        -> gradients in the order of `params` (+ d/dx, d/dy when grid_grads)

`kind` and `params` are those of `_splat.py`.  Eager callers do not come through here: the
`torch.autograd.Function`s of gs2d.py drive the same `run_forward` / `run_backward` directly,
without the operator dispatch cost.
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from . import _splat
from ._splat import KIND_COVINV, KIND_FEATURE, KIND_SCALE_ROT  # noqa: F401

Tensor = torch.Tensor


def _grid_hw(x: Tensor):
    return x.shape[-2], x.shape[-1]


def _fresh(t: Tensor, *inputs: Tensor) -> Tensor:
    """Operator outputs may not alias inputs: copy when a conversion was a no-op."""
    p = t.data_ptr()
    return t.clone() if any(p == i.data_ptr() for i in inputs) else t


@torch.library.custom_op("igs_amd::splat_fwd", mutates_args=(), device_types="cuda")
def splat_fwd(kind: int, params: Sequence[Tensor], x: Tensor, y: Tensor, eps: float) -> List[Tensor]:
    op, keep, packed, col, out, den = _splat.run_forward(kind, list(params), x, y, eps)
    return [out, den, packed, _fresh(col, *params)]


@splat_fwd.register_fake
def _(kind, params, x, y, eps):
    B, N, C = _splat.problem_dims(kind, params)
    Cp = _splat.padded_channels(C)
    H, W = _grid_hw(x)
    new = lambda *s: params[0].new_empty(s, dtype=torch.float32)
    return [new(B, Cp, H, W), new(B, H, W), new(_splat.packed_numel(B, N, Cp)), new(B, N, Cp)]


@torch.library.custom_op("igs_amd::splat_bwd", mutates_args=(), device_types="cuda")
def splat_bwd(kind: int, params: Sequence[Tensor], x: Tensor, y: Tensor, packed: Tensor, col: Tensor, out: Tensor,
              den: Tensor, grad_out: Tensor, eps: float, grid_grads: bool) -> List[Tensor]:
    params = list(params)
    _splat.require_gpu(params[0])
    B, N, C = _splat.problem_dims(kind, params)
    dev = params[0].device
    with torch.cuda.device(dev):
        # rebuilt from the same tensors as in the forward; a non-expanded grid is classified again
        # (one O(BHW) kernel) instead of carrying the flag between the two operators
        op = _splat.Splat(B, N, C, _splat.Grid(x, y, B), eps, dev)
        f = _splat._f32c
        if kind == KIND_COVINV:
            keep = tuple(f(params[i]) for i in (1, 2, 3, 4))
        elif kind == KIND_SCALE_ROT:
            keep = tuple(f(params[i]) for i in (2, 3, 4))
        else:
            keep = (f(params[0]),)
    like = ((x.shape, x.dtype), (y.shape, y.dtype))
    grads, g_x, g_y = _splat.run_backward(kind, op, keep, packed, col, out, den, grad_out,
                                          [True] * len(params), grid_grads, grid_grads, like)
    res = [g.reshape(p.shape).contiguous() for g, p in zip(grads, params)]
    if grid_grads:
        res += [g_x, g_y]
    return res


@splat_bwd.register_fake
def _(kind, params, x, y, packed, col, out, den, grad_out, eps, grid_grads):
    res = [p.new_empty(p.shape, dtype=torch.float32) for p in params]
    if grid_grads:
        res += [torch.empty_like(x), torch.empty_like(y)]
    return res


def _setup_context(ctx, inputs, output):
    kind, params, x, y, eps = inputs
    out, den, packed, col = output
    ctx.kind, ctx.eps, ctx.n_params = kind, eps, len(params)
    ctx.save_for_backward(*params, x, y, out, den, packed, col)


def _backward(ctx, grads):
    g_out = grads[0]
    saved = ctx.saved_tensors
    n = ctx.n_params
    params = list(saved[:n])
    x, y, out, den, packed, col = saved[n:]
    if g_out is None:
        return None, [None] * n, None, None, None
    need_grid = bool(ctx.needs_input_grad[2] or ctx.needs_input_grad[3])
    res = torch.ops.igs_amd.splat_bwd(ctx.kind, params, x, y, packed, col, out, den, g_out.contiguous(), ctx.eps,
                                      need_grid)
    g_x = res[n] if need_grid and ctx.needs_input_grad[2] else None
    g_y = res[n + 1] if need_grid and ctx.needs_input_grad[3] else None
    return None, list(res[:n]), g_x, g_y, None


splat_fwd.register_autograd(_backward, setup_context=_setup_context)


def splat(kind: int, params: Sequence[Tensor], x: Tensor, y: Tensor, eps: float, C: int, dtype) -> Tensor:
    """Differentiable [B,C,H,W] image through the registered operators.  The conversions to the
    operators' canonical form (fp32, contiguous, [B,1,H,W] grids) are ordinary torch ops, so
    autograd (and Inductor) handle them and their gradients."""
    params = [p.to(torch.float32).contiguous() for p in params]
    if x.dim() == 3:
        x = x[:, None]
    if y.dim() == 3:
        y = y[:, None]
    x, y = x.to(torch.float32), y.to(torch.float32)
    out = torch.ops.igs_amd.splat_fwd(kind, params, x, y, float(eps))[0]
    if out.shape[1] != C:
        out = out[:, :C]
    return out if dtype == torch.float32 else out.to(dtype)
