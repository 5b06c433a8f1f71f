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

import ctypes
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.autograd.function import once_differentiable

from . import _lib

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
# helpers around the C ABI
# --------------------------------------------------------------------------------------
def _ptr(t: Optional[Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(dev) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _f32c(t: Tensor) -> Tensor:
    return t.detach().to(torch.float32).contiguous()


def _padded_channels(C: int) -> int:
    for c in _lib.COMPILED_CHANNELS:
        if c >= C:
            return c
    raise ValueError(f"C={C} exceeds the {_lib.IGS_MAX_CHANNELS} channels of one kernel pass")


def _channel_groups(C: int):
    """More than IGS_MAX_CHANNELS channels are rendered in groups of that many: each group's output
    depends on its own colours only, and autograd adds the groups' gradients w.r.t. the shared
    geometry (the backward moments are additive over channel groups: s = sum_groups <g^, out>_group)."""
    m = _lib.IGS_MAX_CHANNELS
    return [(i, min(i + m, C)) for i in range(0, C, m)]


def _pad_last(t: Tensor, Cp: int) -> Tensor:
    C = t.shape[-1]
    return t if C == Cp else F.pad(t, (0, Cp - C))


class _Grid:
    """x/y coordinate tensors described by element strides (no copy for expanded grids)."""

    def __init__(self, x: Tensor, y: Tensor, B: int):
        if x.dim() == 3:
            x = x[:, None]
        if y.dim() == 3:
            y = y[:, None]
        if x.dim() != 4 or y.dim() != 4 or x.shape[1] != 1 or y.shape[1] != 1:
            raise ValueError(f"x_grid/y_grid must be [B,1,H,W] (or [B,H,W]); got {tuple(x.shape)}, {tuple(y.shape)}")
        if x.shape[-2:] != y.shape[-2:]:
            raise ValueError("x_grid and y_grid must have the same H, W")
        for g in (x, y):
            if g.shape[0] not in (1, B):
                raise ValueError(f"grid batch {g.shape[0]} does not match B={B}")
        x = x.detach()
        y = y.detach()
        if x.dtype != torch.float32:
            x = x.to(torch.float32)
        if y.dtype != torch.float32:
            y = y.to(torch.float32)
        self.x, self.y = x, y
        self.H, self.W = x.shape[-2:]

        def st(g):
            sb = 0 if (g.shape[0] == 1) else g.stride(0)
            sh = 0 if self.H == 1 else g.stride(2)
            sw = 0 if self.W == 1 else g.stride(3)
            return (sb, sh, sw)

        self.sx, self.sy = st(x), st(y)
        if min(self.sx + self.sy) < 0:
            self.x, self.y = x.contiguous(), y.contiguous()
            self.sx, self.sy = st(self.x), st(self.y)
        self.strides = _lib.strides6(self.sx, self.sy)
        # x independent of the row and y independent of the column -> factored kernels.  Expanded
        # (stride-0) grids prove it on the host; anything else is classified on the device into a
        # flag that the kernels read, so there is no host synchronisation either way.
        self.flag = None
        if self.sx[1] == 0 and self.sy[2] == 0:
            self.mode = _lib.IGS_GRID_SEPARABLE
        else:
            self.mode = _lib.IGS_GRID_AUTO
            self.flag = torch.empty(1, dtype=torch.int32, device=x.device)
            _lib.check(_lib.load().igs_gs2d_grid_classify(_ptr(self.x), _ptr(self.y), self.strides, B, self.H,
                                                          self.W, _ptr(self.flag), _stream(x.device)),
                       "igs_gs2d_grid_classify")


class _Splat:
    """One fused forward (+ backward) through the C ABI for a fixed problem."""

    def __init__(self, B, N, C, grid: _Grid, eps: float, device):
        self.lib = _lib.load()
        self.B, self.N, self.C = B, N, C
        self.Cp = _padded_channels(C)
        self.grid, self.eps, self.device = grid, float(eps), device
        self.plan = _lib.plan(B, N, grid.H, grid.W, self.Cp, grid.mode)

    def _empty(self, nbytes: int) -> Tensor:
        return torch.empty(max(int(nbytes) // 4, 1), dtype=torch.float32, device=self.device)

    def pack_covinv(self, position, a, b, d, alphas, colors_p) -> Tensor:
        packed = self._empty(self.plan.packed_bytes)
        _lib.check(self.lib.igs_gs2d_pack_covinv(_ptr(position), _ptr(a), _ptr(b), _ptr(d), _ptr(alphas),
                                                 _ptr(colors_p), self.B, self.N, self.Cp, _ptr(packed),
                                                 _stream(self.device)), "igs_gs2d_pack_covinv")
        return packed

    def pack_scale_rot(self, positions, scales, rotations, alphas, colors_p) -> Tensor:
        packed = self._empty(self.plan.packed_bytes)
        _lib.check(self.lib.igs_gs2d_pack_scale_rot(_ptr(positions), _ptr(scales), _ptr(rotations), _ptr(alphas),
                                                    _ptr(colors_p), self.B, self.N, self.Cp, self.eps,
                                                    _ptr(packed), _stream(self.device)), "igs_gs2d_pack_scale_rot")
        return packed

    def forward(self, packed: Tensor) -> Tuple[Tensor, Tensor]:
        g, p = self.grid, self.plan
        out = torch.empty(self.B, self.Cp, g.H, g.W, dtype=torch.float32, device=self.device)
        den = torch.empty(self.B, g.H, g.W, dtype=torch.float32, device=self.device)
        ws = self._empty(p.fwd_ws_bytes) if p.fwd_ws_bytes else None
        _lib.check(self.lib.igs_gs2d_forward(_ptr(packed), _ptr(g.x), _ptr(g.y), g.strides, g.mode, _ptr(g.flag),
                                             self.B, self.N,
                                             g.H, g.W, self.Cp, self.eps, _ptr(out), _ptr(den), _ptr(ws),
                                             int(p.fwd_ws_bytes), _stream(self.device)), "igs_gs2d_forward")
        return out, den

    def backward_partials(self, packed, colors_p, out, den, grad_out_p) -> Tensor:
        g, p = self.grid, self.plan
        pix = self._empty(p.pix_bytes)
        partial = self._empty(p.partial_bytes)
        _lib.check(self.lib.igs_gs2d_backward(_ptr(packed), _ptr(colors_p), _ptr(g.x), _ptr(g.y), g.strides, g.mode,
                                              _ptr(g.flag), _ptr(out), _ptr(den), _ptr(grad_out_p), self.B, self.N, g.H, g.W,
                                              self.Cp, self.eps, _ptr(pix), int(p.pix_bytes), _ptr(partial),
                                              int(p.partial_bytes), _stream(self.device)), "igs_gs2d_backward")
        return partial

    def grid_grads(self, packed, out, den, grad_out_p, x_like, y_like):
        """d L / d x_grid, d L / d y_grid in the (shape, dtype) of the tensors the caller passed."""
        g = self.grid
        gx = torch.empty(self.B, g.H, g.W, dtype=torch.float32, device=self.device)
        gy = torch.empty_like(gx)
        _lib.check(self.lib.igs_gs2d_backward_grid(_ptr(packed), _ptr(g.x), _ptr(g.y), g.strides, _ptr(out),
                                                   _ptr(den), _ptr(grad_out_p), self.B, self.N, g.H, g.W, self.Cp,
                                                   self.eps, _ptr(gx), _ptr(gy), _stream(self.device)),
                   "igs_gs2d_backward_grid")

        def fit(gr, like):
            shape, dtype = like
            if shape[0] == 1 and self.B > 1:      # batch-1 grid shared by all images
                gr = gr.sum(0, keepdim=True)
            return gr.reshape(shape).to(dtype)

        return fit(gx, x_like), fit(gy, y_like)

    def pad_grad_out(self, grad_out: Tensor) -> Tensor:
        go = _f32c(grad_out)
        if self.Cp != self.C:
            go = F.pad(go, (0, 0, 0, 0, 0, self.Cp - self.C)).contiguous()
        return go


def _check_gaussian_shapes(position, alphas, colors):
    if position.dim() != 3 or position.shape[-1] != 2:
        raise ValueError(f"positions must be [B,N,2]; got {tuple(position.shape)}")
    B, N, _ = position.shape
    if alphas.shape != (B, N):
        raise ValueError(f"alphas must be [B,N]={B, N}; got {tuple(alphas.shape)}")
    if colors.dim() != 3 or colors.shape[:2] != (B, N):
        raise ValueError(f"colors must be [B,N,C]; got {tuple(colors.shape)}")
    if N == 0:
        raise ValueError("need at least one Gaussian")
    return B, N, colors.shape[-1]


def _require_gpu(t: Tensor):
    if t.device.type != "cuda":
        raise RuntimeError("the fused Gaussian-splatting path runs on the GPU only (HIP kernels); got a tensor on "
                           f"{t.device}. Use fused=False for the plain-torch debug path.")
    _lib.load()


# --------------------------------------------------------------------------------------
# operator level: the `.apply` plugin boundary of the reference
# --------------------------------------------------------------------------------------
class GaussianSplatting2DKernel(torch.autograd.Function):
    """HIP-backed drop-in for the reference operator (src/igs/gs2d.py:47-262 and its Triton
    variants): `.apply(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors,
    eps=1e-6) -> [B,C,H,W]`; backward returns the same 9-tuple (last entry None).

    x, y: [B,1,H,W] (batch-1 and stride-0/expanded grids are taken as they are);
    position [B,N,2]; cov_inv_* [B,N,1,1] (any shape with B*N elements); alphas [B,N];
    colors [B,N,C].  The backward computes the exact derivative of the forward expression
    (the d/d(den) term is -<g^, out>).
    """

    # advisory tunables kept for callers that set them (scripts/profiling.py:89-95); the
    # compiled tile shapes are chosen by the library's launch plan.
    BLOCK_SIZE_H = BLOCK_SIZE_W = BWD_BLOCK_SIZE_H = BWD_BLOCK_SIZE_W = -1
    N_CHUNK_SIZE = 32

    @classmethod
    def apply(cls, x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors, eps=1e-6):
        C = colors.shape[-1]
        if C <= _lib.IGS_MAX_CHANNELS:
            return super().apply(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors, eps)
        return torch.cat([super(GaussianSplatting2DKernel, cls).apply(
            x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors[..., lo:hi], eps)
            for lo, hi in _channel_groups(C)], dim=1)

    @staticmethod
    def forward(ctx, x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors, eps=1e-6):
        _require_gpu(position)
        B, N, C = _check_gaussian_shapes(position, alphas, colors)
        for t in (cov_inv_00, cov_inv_01, cov_inv_11):
            if t.numel() != B * N:
                raise ValueError(f"cov_inv_* must hold B*N={B * N} elements; got {tuple(t.shape)}")
        dev = position.device
        with torch.cuda.device(dev):
            grid = _Grid(x, y, B)
            op = _Splat(B, N, C, grid, eps, dev)
            pos, a, b, d, al = (_f32c(t) for t in (position, cov_inv_00, cov_inv_01, cov_inv_11, alphas))
            col = _pad_last(_f32c(colors), op.Cp).contiguous()
            packed = op.pack_covinv(pos, a, b, d, al, col)
            out, den = op.forward(packed)
        ctx.op = op
        ctx.grid_like = ((x.shape, x.dtype), (y.shape, y.dtype))
        ctx.save_for_backward(packed, col, a, b, d, al, out, den)
        ctx.in_dtypes = tuple(t.dtype for t in (position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors))
        ctx.cov_shapes = (cov_inv_00.shape, cov_inv_01.shape, cov_inv_11.shape)
        res = out if op.Cp == C else out[:, :C]
        return res.to(x.dtype) if x.dtype != torch.float32 else res

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_result):
        op: _Splat = ctx.op
        packed, col, a, b, d, al, out, den = ctx.saved_tensors
        B, N, C, Cp, dev = op.B, op.N, op.C, op.Cp, op.device
        need = ctx.needs_input_grad
        g_x = g_y = None
        with torch.cuda.device(dev):
            go = op.pad_grad_out(grad_result)
            if need[0] or need[1]:
                g_x, g_y = op.grid_grads(packed, out, den, go, *ctx.grid_like)
                g_x, g_y = (g_x if need[0] else None), (g_y if need[1] else None)
            partial = op.backward_partials(packed, col, out, den, go)
            new = lambda *s: torch.empty(*s, dtype=torch.float32, device=dev)
            g_pos = new(B, N, 2) if need[2] else None
            g_a = new(B, N) if need[3] else None
            g_b = new(B, N) if need[4] else None
            g_d = new(B, N) if need[5] else None
            g_al = new(B, N) if need[6] else None
            g_col = new(B, N, Cp) if need[7] else None
            _lib.check(op.lib.igs_gs2d_finalize_covinv(_ptr(partial), op.grid.mode, _ptr(op.grid.flag), _ptr(a),
                                                       _ptr(b), _ptr(d), _ptr(al), B, N, op.grid.H, op.grid.W,
                                                       Cp, _ptr(g_pos), _ptr(g_a), _ptr(g_b),
                                                       _ptr(g_d), _ptr(g_al), _ptr(g_col), _stream(dev)),
                       "igs_gs2d_finalize_covinv")
        if g_col is not None and Cp != C:
            g_col = g_col[..., :C]
        dt = ctx.in_dtypes
        cast = lambda g, k: None if g is None else g.to(dt[k])
        sh = ctx.cov_shapes
        return (g_x, g_y, cast(g_pos, 0),
                None if g_a is None else cast(g_a, 1).reshape(sh[0]),
                None if g_b is None else cast(g_b, 2).reshape(sh[1]),
                None if g_d is None else cast(g_d, 3).reshape(sh[2]),
                cast(g_al, 4), cast(g_col, 5), None)


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
        _require_gpu(positions)
        B, N, C = _check_gaussian_shapes(positions, alphas, colors)
        if scales.shape != (B, N, 2) or rotations.shape != (B, N):
            raise ValueError(f"scales must be [B,N,2] and rotations [B,N]; got {tuple(scales.shape)}, {tuple(rotations.shape)}")
        dev = positions.device
        with torch.cuda.device(dev):
            grid = _Grid(x_grid, y_grid, B)
            op = _Splat(B, N, C, grid, eps, dev)
            pos, sc, rot, al = (_f32c(t) for t in (positions, scales, rotations, alphas))
            col = _pad_last(_f32c(colors), op.Cp).contiguous()
            packed = op.pack_scale_rot(pos, sc, rot, al, col)
            out, den = op.forward(packed)
        ctx.op = op
        ctx.grid_like = ((x_grid.shape, x_grid.dtype), (y_grid.shape, y_grid.dtype))
        ctx.save_for_backward(packed, col, sc, rot, al, out, den)
        ctx.in_dtypes = tuple(t.dtype for t in (positions, colors, scales, rotations, alphas))
        res = out if op.Cp == C else out[:, :C]
        return res.to(positions.dtype) if positions.dtype != torch.float32 else res

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_result):
        op: _Splat = ctx.op
        packed, col, sc, rot, al, out, den = ctx.saved_tensors
        B, N, C, Cp, dev = op.B, op.N, op.C, op.Cp, op.device
        need = ctx.needs_input_grad
        g_x = g_y = None
        with torch.cuda.device(dev):
            go = op.pad_grad_out(grad_result)
            if need[5] or need[6]:
                g_x, g_y = op.grid_grads(packed, out, den, go, *ctx.grid_like)
                g_x, g_y = (g_x if need[5] else None), (g_y if need[6] else None)
            partial = op.backward_partials(packed, col, out, den, go)
            new = lambda *s: torch.empty(*s, dtype=torch.float32, device=dev)
            g_pos = new(B, N, 2) if need[0] else None
            g_col = new(B, N, Cp) if need[1] else None
            g_sc = new(B, N, 2) if need[2] else None
            g_rot = new(B, N) if need[3] else None
            g_al = new(B, N) if need[4] else None
            _lib.check(op.lib.igs_gs2d_finalize_scale_rot(_ptr(partial), op.grid.mode, _ptr(op.grid.flag), _ptr(sc),
                                                          _ptr(rot), _ptr(al), B, N, op.grid.H, op.grid.W, Cp,
                                                          op.eps, _ptr(g_pos), _ptr(g_sc),
                                                          _ptr(g_rot), _ptr(g_al), _ptr(g_col), _stream(dev)),
                       "igs_gs2d_finalize_scale_rot")
        if g_col is not None and Cp != C:
            g_col = g_col[..., :C]
        dt = ctx.in_dtypes
        cast = lambda g, k: None if g is None else g.to(dt[k])
        return cast(g_pos, 0), cast(g_col, 1), cast(g_sc, 2), cast(g_rot, 3), cast(g_al, 4), g_x, g_y, None


class _RenderFromFeature(torch.autograd.Function):
    """(gs_feature [B,N,6+C], pos_offset or None, x_grid, y_grid, eps) -> [B,C,H,W].

    The module's split / exp(log_scale)+eps / alpha = 1 (src/igs/gs2d.py:638-675) run inside the
    pack kernel and their autograd inside the finalize kernel, so the only torch ops left around
    the splat are the two GEMMs of `proj`."""

    @staticmethod
    def forward(ctx, gs_feature, pos_offset, x_grid, y_grid, eps):
        _require_gpu(gs_feature)
        if gs_feature.dim() != 3 or gs_feature.shape[-1] < 7:
            raise ValueError(f"gs_feature must be [B,N,6+C]; got {tuple(gs_feature.shape)}")
        B, N, F6 = gs_feature.shape
        C = F6 - 6
        dev = gs_feature.device
        with torch.cuda.device(dev):
            grid = _Grid(x_grid, y_grid, B)
            op = _Splat(B, N, C, grid, eps, dev)
            feat = _f32c(gs_feature)
            off = None if pos_offset is None else _f32c(pos_offset)
            if off is not None and off.shape != (B, N, 2):
                raise ValueError(f"pos_offset must be [B,N,2]; got {tuple(off.shape)}")
            packed = op._empty(op.plan.packed_bytes)
            col = torch.empty(B, N, op.Cp, dtype=torch.float32, device=dev)
            _lib.check(op.lib.igs_gs2d_pack_feature(_ptr(feat), _ptr(off), B, N, C, op.Cp, op.eps, _ptr(packed),
                                                    _ptr(col), _stream(dev)), "igs_gs2d_pack_feature")
            out, den = op.forward(packed)
        ctx.op = op
        ctx.save_for_backward(packed, col, feat, out, den)
        ctx.in_dtype = gs_feature.dtype
        ctx.grid_like = ((x_grid.shape, x_grid.dtype), (y_grid.shape, y_grid.dtype))
        res = out if op.Cp == C else out[:, :C]
        return res.to(gs_feature.dtype) if gs_feature.dtype != torch.float32 else res

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_result):
        op: _Splat = ctx.op
        packed, col, feat, out, den = ctx.saved_tensors
        B, N, C, Cp, dev = op.B, op.N, op.C, op.Cp, op.device
        need = ctx.needs_input_grad
        g_x = g_y = g_feat = g_off = None
        with torch.cuda.device(dev):
            go = op.pad_grad_out(grad_result)
            if need[2] or need[3]:
                g_x, g_y = op.grid_grads(packed, out, den, go, *ctx.grid_like)
                g_x, g_y = (g_x if need[2] else None), (g_y if need[3] else None)
            if need[0] or need[1]:
                partial = op.backward_partials(packed, col, out, den, go)
                g_feat = torch.empty(B, N, 6 + C, dtype=torch.float32, device=dev)
                _lib.check(op.lib.igs_gs2d_finalize_feature(_ptr(partial), op.grid.mode, _ptr(op.grid.flag), _ptr(feat),
                                                            B, N, op.grid.H, op.grid.W, C, Cp, op.eps, _ptr(g_feat),
                                                            _stream(dev)), "igs_gs2d_finalize_feature")
                if need[1]:
                    g_off = g_feat[..., :2].contiguous()
                g_feat = g_feat.to(ctx.in_dtype) if need[0] else None
        return g_feat, g_off, g_x, g_y, None


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
        (src/igs/gs2d.py:503-522)."""
        h, w = size
        aspect_ratio = h / w
        h_range = aspect_ratio ** 0.5
        w_range = 1 / aspect_ratio ** 0.5
        x_grid = torch.linspace(-w_range, w_range, w).to(device).view(1, 1, w).expand(1, h, w)
        y_grid = torch.linspace(-h_range, h_range, h).to(device).view(1, h, 1).expand(1, h, w)
        return x_grid, y_grid

    @staticmethod
    def render(positions, colors, scales, rotations, alphas, x_grid, y_grid, eps=1e-6, fused=True):
        """scales [B,N,2]; alphas [B,N]; positions [B,N,2]; rotations [B,N]; colors [B,N,C];
        x_grid, y_grid [B,1,H,W] (also accepted: [B,H,W], batch 1, expanded/stride-0).
        Returns [B,C,H,W] (src/igs/gs2d.py:524-609)."""
        if fused:
            C = colors.shape[-1]
            if C <= _lib.IGS_MAX_CHANNELS:
                return _RenderFused.apply(positions, colors, scales, rotations, alphas, x_grid, y_grid, eps)
            return torch.cat([_RenderFused.apply(positions, colors[..., lo:hi], scales, rotations, alphas, x_grid,
                                                 y_grid, eps) for lo, hi in _channel_groups(C)], dim=1)
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
            x_grid, y_grid = self.xy_grid(size, feature.device)
            # kept expanded (stride 0) instead of the reference's .repeat: same values, and
            # the kernels then take the separable-grid path
            x_grid = x_grid[None].expand(b, 1, -1, -1)
            y_grid = y_grid[None].expand(b, 1, -1, -1)
        else:
            grid = grid.flip(1)  # pos_map order is (h, w): y first
            x_grid, y_grid = grid.split([1, 1], dim=1)
        pos_map = None
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
            output = _RenderFromFeature.apply(gs_feature, pos_map, x_grid, y_grid, eps)
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
