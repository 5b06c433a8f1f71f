"""Host-side mirror of the reference's `igs.gs2d` interface on top of the HIP library.

Public names follow the reference (src/igs/gs2d.py): `naive_gaussian_2d` (:24-44),
`GaussianSplatting2DKernel` (the `.apply(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11,
alphas, colors, eps)` operator, :47-262 / :468-476), `GaussianSplatting2D` (module, :479-689)
with `xy_grid` (:503-522) and `render` (:524-609), and `gaussian_splatting_2d` (:692).

PyTorch is used for device memory, streams and autograd plumbing only; all arithmetic of the
fused path runs in the hand-written HIP kernels of libigs_hip.so, reached through its C ABI.
There is no CPU or eager fallback for the fused path: without the library (or on a CPU tensor)
it raises.
"""
from __future__ import annotations

import functools

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.autograd.function import once_differentiable

from . import _lib, _ops
from ._splat import KIND_COVINV, KIND_FEATURE, KIND_SCALE_ROT, channel_groups, run_backward, run_forward

Tensor = torch.Tensor


# --------------------------------------------------------------------------------------
# debug path (fused=False), as in the reference: plain torch, materialises [B,N,H,W]
# --------------------------------------------------------------------------------------
def naive_gaussian_2d(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors, eps=1e-6):
    """Unfused expression of the splat (reference src/igs/gs2d.py:24-44); "heavy, just for
    debugging" there and here.  Differentiable through torch autograd."""
    dx = x - position[..., 0, None, None]
    dy = y - position[..., 1, None, None]
    q = dx * dx * cov_inv_00 + 2 * dx * dy * cov_inv_01 + dy * dy * cov_inv_11
    weight = torch.exp(-0.5 * q) * alphas[..., None, None]
    weight_sum = weight.sum(dim=1, keepdim=True)
    b, ng, h, w = weight.shape
    nw = (weight / (weight_sum + eps)).permute(0, 2, 3, 1).flatten(1, 2)
    return torch.bmm(nw, colors).unflatten(1, (h, w)).permute(0, 3, 1, 2)


# --------------------------------------------------------------------------------------
# operator level: the `.apply` plugin boundary of the reference
# --------------------------------------------------------------------------------------
def _degenerate(params, x_grid, B, N, C, dtype):
    """No Gaussian, no image or no pixel: the plain expression (src/igs/gs2d.py:24-44) gives an
    all-zero [B,C,H,W] image (den = 0, 0 / (0 + eps) = 0) and zero gradients; there is nothing
    to launch.  Returns None for a real problem."""
    H, W = x_grid.shape[-2:]
    if B and N and H and W:
        return None
    out = torch.zeros(B, C, H, W, dtype=dtype, device=params[0].device)
    for p in params:   # keeps the result attached to its inputs (their gradients are zeros)
        if p.requires_grad:
            out = out + p.sum() * 0
    return out


def _as(t: Tensor, dtype) -> Tensor:
    return t if t.dtype == dtype else t.to(dtype)


def _visible(op, out: Tensor, dtype) -> Tensor:
    """The caller's view of the kernel's [B,Cp,H,W] fp32 output."""
    return _as(out if op.Cp == op.C else out[:, :op.C], dtype)


class _Operator(torch.autograd.Function):
    """(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors, eps) -> [B,C,H,W]
    for C <= IGS_MAX_CHANNELS; backward returns the reference's 9-tuple (src/igs/gs2d.py:252-262)."""

    @staticmethod
    def forward(ctx, x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors, eps=1e-6):
        params = (position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors)
        op, keep, packed, col, out, den = run_forward(KIND_COVINV, params, x, y, eps, train=any(ctx.needs_input_grad))
        ctx.op = op
        ctx.grid_like = ((x.shape, x.dtype), (y.shape, y.dtype))
        ctx.n_keep = len(keep)
        ctx.save_for_backward(*keep, packed, col, out, den)
        ctx.like = tuple((t.shape, t.dtype) for t in params)
        return _visible(op, out, x.dtype)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_result):
        saved = ctx.saved_tensors
        keep, (packed, col, out, den) = saved[:ctx.n_keep], saved[ctx.n_keep:]
        need = ctx.needs_input_grad
        grads, g_x, g_y = run_backward(KIND_COVINV, ctx.op, keep, packed, col, out, den, grad_result, need[2:8],
                                       need[0], need[1], ctx.grid_like)
        grads = [None if g is None else _as(g, dt).reshape(sh) for g, (sh, dt) in zip(grads, ctx.like)]
        return (g_x, g_y, *grads, None)


class GaussianSplatting2DKernel:
    """HIP-backed drop-in for the reference operator (src/igs/gs2d.py:47-262 and its Triton
    variants): `.apply(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors,
    eps=1e-6) -> [B,C,H,W]`, differentiable w.r.t. all eight tensors.

    x, y: [B,1,H,W] (batch-1 and stride-0/expanded grids are taken as they are);
    position [B,N,2]; cov_inv_* [B,N,1,1] (any shape with B*N elements); alphas [B,N];
    colors [B,N,C].  The backward computes the exact derivative of the forward expression
    (the d/d(den) term is -<g^, out>).

    A plain class with the `torch.autograd.Function` calling convention rather than a Function
    itself: `.apply` routes eager callers to the autograd.Function above and callers under
    `torch.compile` to the registered operators (Dynamo would otherwise trace into the ctypes
    calls of a Function's forward).
    """

    # advisory tunables kept for callers that set them (scripts/profiling.py:89-95); the
    # compiled tile shapes are chosen by the library's launch plan.
    BLOCK_SIZE_H = BLOCK_SIZE_W = BWD_BLOCK_SIZE_H = BWD_BLOCK_SIZE_W = -1
    N_CHUNK_SIZE = 32

    @staticmethod
    def apply(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors, eps=1e-6):
        C = colors.shape[-1]
        empty = _degenerate((position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors), x, position.shape[0],
                            position.shape[1], C, x.dtype)
        if empty is not None:
            return empty
        if C > _lib.IGS_MAX_CHANNELS:
            return torch.cat([GaussianSplatting2DKernel.apply(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11,
                                                              alphas, colors[..., lo:hi], eps)
                              for lo, hi in channel_groups(C)], dim=1)
        if torch.compiler.is_compiling():
            B, N = position.shape[:2]
            params = [position, cov_inv_00.reshape(B, N), cov_inv_01.reshape(B, N), cov_inv_11.reshape(B, N),
                      alphas, colors]
            return _ops.splat(KIND_COVINV, params, x, y, eps, C, x.dtype)
        return _Operator.apply(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors, eps)


# The reference exposes its torch variants under these names (src/igs/gs2d.py:468-469) and
# picks one implementation at import (:471-476).  Here there is a single implementation.
TorchGaussianSplatting2DKernel = GaussianSplatting2DKernel
TorchGaussianSplatting2DChunked = GaussianSplatting2DKernel
GaussianSplatting2DChunkedKernel = GaussianSplatting2DKernel


# --------------------------------------------------------------------------------------
# function level: render(fused=True) with the covariance preamble folded into the kernels
# --------------------------------------------------------------------------------------
class _RenderFused(torch.autograd.Function):
    """(positions, colors, scales, rotations, alphas, x_grid, y_grid, eps) -> [B,C,H,W].

    Forward = closed-form (R S S^T R^T + eps I)^-1 (replacing src/igs/gs2d.py:548-580) inside
    the pack kernel + the splat; backward = splat backward + chain rule to scales/rotations
    inside the finalize kernel."""

    @staticmethod
    def forward(ctx, positions, colors, scales, rotations, alphas, x_grid, y_grid, eps):
        params = (positions, colors, scales, rotations, alphas)
        op, keep, packed, col, out, den = run_forward(KIND_SCALE_ROT, params, x_grid, y_grid, eps, train=any(ctx.needs_input_grad))
        ctx.op = op
        ctx.grid_like = ((x_grid.shape, x_grid.dtype), (y_grid.shape, y_grid.dtype))
        ctx.n_keep = len(keep)
        ctx.save_for_backward(*keep, packed, col, out, den)
        ctx.in_dtypes = tuple(t.dtype for t in params)
        return _visible(op, out, positions.dtype)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_result):
        saved = ctx.saved_tensors
        keep, (packed, col, out, den) = saved[:ctx.n_keep], saved[ctx.n_keep:]
        need = ctx.needs_input_grad
        grads, g_x, g_y = run_backward(KIND_SCALE_ROT, ctx.op, keep, packed, col, out, den, grad_result, need[0:5],
                                       need[5], need[6], ctx.grid_like)
        grads = [None if g is None else _as(g, dt) for g, dt in zip(grads, ctx.in_dtypes)]
        return (*grads, g_x, g_y, None)


class _RenderFromFeature(torch.autograd.Function):
    """(gs_feature [B,N,6+C], pos_offset or None, x_grid, y_grid, eps) -> [B,C,H,W].

    The module's split / exp(log_scale)+eps / alpha = 1 (src/igs/gs2d.py:638-675) run inside the
    pack kernel and their autograd inside the finalize kernel, so the only torch ops left around
    the splat are the two GEMMs of `proj`."""

    @staticmethod
    def forward(ctx, gs_feature, pos_offset, x_grid, y_grid, eps):
        params = (gs_feature,) if pos_offset is None else (gs_feature, pos_offset)
        op, keep, packed, col, out, den = run_forward(KIND_FEATURE, params, x_grid, y_grid, eps, train=any(ctx.needs_input_grad))
        ctx.op = op
        ctx.grid_like = ((x_grid.shape, x_grid.dtype), (y_grid.shape, y_grid.dtype))
        ctx.n_keep = len(keep)
        ctx.save_for_backward(*keep, packed, col, out, den)
        ctx.in_dtypes = tuple(t.dtype for t in params)
        return _visible(op, out, gs_feature.dtype)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_result):
        saved = ctx.saved_tensors
        keep, (packed, col, out, den) = saved[:ctx.n_keep], saved[ctx.n_keep:]
        need = ctx.needs_input_grad
        n = len(ctx.in_dtypes)
        grads, g_x, g_y = run_backward(KIND_FEATURE, ctx.op, keep, packed, col, out, den, grad_result, need[0:n],
                                       need[2], need[3], ctx.grid_like)
        grads = [None if g is None else _as(g, dt) for g, dt in zip(grads, ctx.in_dtypes)]
        if n == 1:
            grads.append(None)
        return (*grads, g_x, g_y, None)


def _render_fused(positions, colors, scales, rotations, alphas, x_grid, y_grid, eps):
    empty = _degenerate((positions, colors, scales, rotations, alphas), x_grid, positions.shape[0],
                        positions.shape[1], colors.shape[-1], positions.dtype)
    if empty is not None:
        return empty
    if torch.compiler.is_compiling():
        return _ops.splat(KIND_SCALE_ROT, [positions, colors, scales, rotations, alphas], x_grid, y_grid, eps,
                          colors.shape[-1], positions.dtype)
    return _RenderFused.apply(positions, colors, scales, rotations, alphas, x_grid, y_grid, eps)


def _render_from_feature(gs_feature, pos_offset, x_grid, y_grid, eps):
    empty = _degenerate((gs_feature,) if pos_offset is None else (gs_feature, pos_offset), x_grid,
                        gs_feature.shape[0], gs_feature.shape[1], gs_feature.shape[-1] - 6, gs_feature.dtype)
    if empty is not None:
        return empty
    if torch.compiler.is_compiling():
        params = [gs_feature] if pos_offset is None else [gs_feature, pos_offset]
        return _ops.splat(KIND_FEATURE, params, x_grid, y_grid, eps, gs_feature.shape[-1] - 6, gs_feature.dtype)
    return _RenderFromFeature.apply(gs_feature, pos_offset, x_grid, y_grid, eps)


def _cov_inverse_torch(scales, rotations, eps):
    """Matrix route of the reference preamble (src/igs/gs2d.py:548-580) for the debug path,
    in the dtype of its inputs."""
    b, ng, _ = scales.shape
    c, s = torch.cos(rotations), torch.sin(rotations)
    rot = torch.stack([torch.stack([c, -s], dim=2), torch.stack([s, c], dim=2)], dim=2)
    sm = torch.diag_embed(scales)
    rs = torch.bmm(rot.flatten(0, 1), sm.flatten(0, 1))
    cov = torch.bmm(rs, rs.transpose(-2, -1)).unflatten(0, (b, ng))
    eye = torch.eye(2, device=cov.device, dtype=cov.dtype).expand(b, ng, -1, -1)
    inv = torch.inverse(cov + eps * eye)
    return inv[..., 0, 0, None, None], inv[..., 0, 1, None, None], inv[..., 1, 1, None, None]


@functools.lru_cache(maxsize=32)
def _grid_vectors(h: int, w: int, device):
    """The two coordinate vectors of xy_grid, kept per (size, device) for the module's forward.
    Built outside inference mode so that a first call under torch.inference_mode() does not leave
    inference tensors behind for later training calls."""
    aspect_ratio = h / w
    h_range = aspect_ratio ** 0.5
    w_range = 1 / aspect_ratio ** 0.5
    with torch.inference_mode(False):
        return torch.linspace(-w_range, w_range, w).to(device), torch.linspace(-h_range, h_range, h).to(device)


class GaussianSplatting2D(nn.Module):
    """Drop-in for the reference module (src/igs/gs2d.py:479-689): a linear head producing
    `num_gaussians_per_emb` Gaussians (2 position, 2 log-scale, 1 rotation, 1 unused opacity
    logit, `output_dim` colours) per input feature, rendered by the fused HIP splat.
    Parameter names and init follow the reference (`proj.weight`, `proj.bias`), so its
    checkpoints load."""

    def __init__(self, num_gaussians_per_emb, emb_dim, output_dim=3, pos_map_offset=False):
        super().__init__()
        self.num_gaussians_per_emb = num_gaussians_per_emb
        self.emb_dim = emb_dim
        self.chunk_size = 0
        self.output_dim = output_dim
        self.pos_map_offset = pos_map_offset

        self.proj = nn.Linear(emb_dim, num_gaussians_per_emb * (6 + output_dim))
        nn.init.normal_(self.proj.weight, mean=0.0, std=0.01)
        # same RNG draw order as the reference (:498-501): positions bias 0, log-scale bias -4
        gaussian_bias = torch.randn(num_gaussians_per_emb, 6 + output_dim) * 0.01
        gaussian_bias[:, :2] = 0
        gaussian_bias[:, 2:4] = -4
        self.proj.bias.data.copy_(gaussian_bias.view_as(self.proj.bias))

    @staticmethod
    def xy_grid(size=None, device=None):
        """x in +-sqrt(w/h), y in +-sqrt(h/w) as stride-0 expanded [1,h,w] tensors
        (src/igs/gs2d.py:503-522).  Like the reference, every call returns tensors of its own (the
        caller may write into what they view); the module's forward uses vectors kept per
        (size, device) instead, see `_shared_xy_grid`."""
        h, w = size
        xs, ys = _grid_vectors(int(h), int(w), None if device is None else torch.device(device))
        return xs.clone().view(1, 1, w).expand(1, h, w), ys.clone().view(1, h, 1).expand(1, h, w)

    @staticmethod
    def _shared_xy_grid(size, device):
        """xy_grid without the copy: read-only views of the kept coordinate vectors (the reference
        rebuilds them on the host and copies them over in every forward)."""
        h, w = size
        xs, ys = _grid_vectors(int(h), int(w), None if device is None else torch.device(device))
        return xs.view(1, 1, w).expand(1, h, w), ys.view(1, h, 1).expand(1, h, w)

    @staticmethod
    def render(positions, colors, scales, rotations, alphas, x_grid, y_grid, eps=1e-6, fused=True):
        """scales [B,N,2]; alphas [B,N]; positions [B,N,2]; rotations [B,N]; colors [B,N,C];
        x_grid, y_grid [B,1,H,W] (also accepted: [B,H,W], batch 1, expanded/stride-0).
        Returns [B,C,H,W] (src/igs/gs2d.py:524-609)."""
        if fused:
            C = colors.shape[-1]
            if C <= _lib.IGS_MAX_CHANNELS:
                return _render_fused(positions, colors, scales, rotations, alphas, x_grid, y_grid, eps)
            return torch.cat([_render_fused(positions, colors[..., lo:hi], scales, rotations, alphas, x_grid,
                                            y_grid, eps) for lo, hi in channel_groups(C)], dim=1)
        # heavy debug path, plain torch (src/igs/gs2d.py:598-609)
        if x_grid.dim() == 3:
            x_grid, y_grid = x_grid[:, None], y_grid[:, None]
        a, b, d = _cov_inverse_torch(scales, rotations, eps)
        return naive_gaussian_2d(x_grid, y_grid, positions, a, b, d, alphas, colors, eps)

    def forward(self, feature, size=None, grid=None, pos_map=None, eps=1e-6, fused=True, scale=None):
        """feature [B,F,D] -> (image [B,C,H,W], gs_feature [B,F*n,6+C]) (src/igs/gs2d.py:611-689)."""
        gs_feature = self.proj(feature).unflatten(-1, (-1, 6 + self.output_dim)).flatten(1, 2)
        b = gs_feature.shape[0]

        if grid is None:
            x_grid, y_grid = self._shared_xy_grid(size, feature.device)
            # kept expanded (stride 0) instead of the reference's .repeat: same values, and
            # the kernels then take the separable-grid path
            x_grid = x_grid[None].expand(b, 1, -1, -1)
            y_grid = y_grid[None].expand(b, 1, -1, -1)
        else:
            grid = grid.flip(1)  # pos_map order is (h, w): y first
            x_grid, y_grid = grid.split([1, 1], dim=1)
        pos_map = None  # the argument is not read by the reference either (:654-655 overwrites it)
        if self.pos_map_offset:
            pos_map = torch.concat([x_grid, y_grid], dim=1)
            if scale is not None:
                pos_map = F.interpolate(pos_map, scale_factor=1 / scale, mode="bilinear", align_corners=True)
            pos_map = pos_map.flatten(2, 3).transpose(1, 2)
            assert pos_map.size(1) == feature.size(1)
            pos_map = pos_map[..., None, :].repeat(1, 1, self.num_gaussians_per_emb, 1).flatten(1, 2)

        if fused and self.output_dim <= _lib.IGS_MAX_CHANNELS:
            # split, exp(log_scale) + eps, alpha = 1 and their autograd run inside the HIP pack /
            # finalize kernels
            output = _render_from_feature(gs_feature, pos_map, x_grid, y_grid, eps)
            return output, gs_feature

        positions, log_scales, rotations, logit_opacity, colors = gs_feature.split(
            [2, 2, 1, 1, self.output_dim], dim=-1)
        if pos_map is not None:
            positions = positions + pos_map
        alphas = torch.ones_like(logit_opacity[..., 0])  # opacity logit is unused, as in the reference
        scales = torch.exp(log_scales) + eps
        rotations = rotations[..., 0]
        output = self.render(positions, colors, scales, rotations, alphas, x_grid, y_grid, eps, fused)
        return output, gs_feature


gaussian_splatting_2d = GaussianSplatting2D.render
