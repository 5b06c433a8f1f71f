"""Host-side driver of the HIP splat: allocation, grid description and the call sequence through
the C ABI for the three parameterisations that reach the same kernels.

  KIND_COVINV     (position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors)
                  -- the reference operator's arguments (src/igs/gs2d.py:50-62)
  KIND_SCALE_ROT  (positions, colors, scales, rotations, alphas)
                  -- `render`'s arguments (src/igs/gs2d.py:526-536); the covariance preamble
                     (:548-580) is evaluated in closed form inside the pack / finalize kernels
  KIND_FEATURE    (gs_feature [, pos_offset])
                  -- the module head's output (src/igs/gs2d.py:635-675); split, exp(log_scale)+eps
                     and alpha = 1 run inside the pack / finalize kernels

`run_forward` / `run_backward` are shared by the eager `torch.autograd.Function`s and by the
`torch.library` operators that `torch.compile` callers reach.  torch allocates and provides the
stream; every FLOP happens in libigs_hip.so.
"""
from __future__ import annotations

import contextlib
import contextvars
import functools
from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

from . import _lib

Tensor = torch.Tensor

KIND_COVINV = 0
KIND_SCALE_ROT = 1
KIND_FEATURE = 2


# Bound on what skipping far-away (Gaussian, pixel) pairs may change in an output element, as a
# fraction of the largest colour magnitude: the pack calls get the skip weight w =
# igs_gs2d_skip_weight(N, eps, SKIP_TOLERANCE) = SKIP_TOLERANCE * eps / (2 N) and the skip fraction
# f = SKIP_TOLERANCE / (2 N), and a pixel tile leaves out Gaussians whose largest weights on it add
# up to at most N (w + f S), S bounding its denominators from below.  The forward is held to
# 1e-6 + 1e-5 |ref| against the plain expression; 1e-7 leaves that budget to the fp32 rounding.
# 0 skips exact zeros only (bit-identical to evaluating every pair).
SKIP_TOLERANCE = 1e-7

# Partial sums of the separable backward: one record per listed (Gaussian, tile) pair.  Above this many
# bytes for *every* pair (plan.partial_bytes: B=4, N=32768, 384x640, C=16 is 2.8 GB, of which 4 % are
# listed), a training forward leaves the number of listed pairs in pinned host memory and the backward
# allocates by it, which makes the host wait until the device has passed the forward's binning (2 % of
# that step; a step of a fraction of a millisecond would lose a third, its host no longer running ahead);
# below, the array is allocated in full (B=16, N=8192, 256x256: 0.3 GB for the duration of the backward)
# and nothing waits for the device.
COMPACT_PARTIALS_FROM = 512 << 20

# (igs_option bits OR-ed into the grid_mode word of every Grid built, skip tolerance) in effect for the
# calling thread (and asyncio task): a context variable, so that two threads, or a `with` block and
# another thread's calls, do not see each other's settings.  Both are read when a call's forward
# is set up, on the caller's thread; the backward, whichever thread autograd runs it on, uses what
# its forward recorded (the grid's mode word, the packed buffer's skip settings).
_options = contextvars.ContextVar("igs_amd_library_options", default=(0, SKIP_TOLERANCE))


@contextlib.contextmanager
def library_options(no_cull: bool = False, bin_levels: Optional[int] = None,
                    skip_tolerance: Optional[float] = None):
    """Problems set up inside this context, by this thread, run with the given igs_option bits of
    include/igs_hip.h -- `no_cull` lists every Gaussian for every pixel tile (the reference point
    for what culling changes), `bin_levels` = 1 | 2 forces the one- or two-level construction
    of the tile lists -- and with the given `skip_tolerance` (see SKIP_TOLERANCE; 0 = only pairs
    whose weight is exactly zero are skipped).  The bits and the skip weight travel as explicit
    arguments of each library call; the library itself holds no such state."""
    bits = _lib.IGS_OPT_NO_CULL if no_cull else 0
    if bin_levels is not None:
        bits |= {1: _lib.IGS_OPT_BIN_LEVELS_1, 2: _lib.IGS_OPT_BIN_LEVELS_2}[int(bin_levels)]
    old_bits, tolerance = _options.get()
    if skip_tolerance is not None:
        if not 0.0 <= float(skip_tolerance) < 1.0:
            raise ValueError("skip_tolerance must be in [0, 1)")
        tolerance = float(skip_tolerance)
    token = _options.set((old_bits | bits, tolerance))   # nested contexts add up
    try:
        yield
    finally:
        _options.reset(token)


def exact():
    """Context in which the calling thread's renders skip exact zeros only: every (Gaussian, pixel)
    pair whose fp32 weight is not exactly zero is evaluated, as the reference does
    (`library_options(skip_tolerance=0)`)."""
    return library_options(skip_tolerance=0.0)


@functools.lru_cache(maxsize=256)
def _skip_weight(N: int, eps: float, tolerance: float) -> Tuple[float, float]:
    f = _lib.load().igs_gs2d_skip_weight
    return float(f(N, eps, tolerance)), float(f(N, 1.0, tolerance))


def skip_weight(N: int, eps: float) -> Tuple[float, float]:
    """(skip_weight, skip_fraction) the pack calls of a problem get under the current skip tolerance."""
    return _skip_weight(int(N), float(eps), float(_options.get()[1]))


# The host side of a call is what bounds small problems (a 512-Gaussian 256x256 forward+backward
# is ~0.1 ms of kernels), so the per-call helpers below take the short routes: addresses and
# streams travel as plain integers (the signatures convert them), the current stream comes from
# torch's raw accessor, and the device is switched only when it is not the current one already.
def _ptr(t: Optional[Tensor]):
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)
_no_guard = contextlib.nullcontext()


def _stream(dev) -> int:
    if _raw_stream is not None and dev.index is not None:
        return _raw_stream(dev.index)
    return torch.cuda.current_stream(dev).cuda_stream


def _on(dev):
    """Context in which `dev` is the current device."""
    if _current_device is not None and dev.index is not None and _current_device() == dev.index:
        return _no_guard
    return torch.cuda.device(dev)


def _f32c(t: Tensor) -> Tensor:
    t = t.detach()
    if t.dtype != torch.float32:
        t = t.to(torch.float32)
    return t if t.is_contiguous() else t.contiguous()


def padded_channels(C: int) -> int:
    for c in _lib.COMPILED_CHANNELS:
        if c >= C:
            return c
    raise ValueError(f"C={C} exceeds the {_lib.IGS_MAX_CHANNELS} channels of one kernel pass")


def channel_groups(C: int):
    """More than IGS_MAX_CHANNELS channels are rendered in groups of that many: each group's output
    depends on its own colours only, and autograd adds the groups' gradients w.r.t. the shared
    geometry (the backward moments are additive over channel groups: s = sum_groups <g^, out>_group)."""
    m = _lib.IGS_MAX_CHANNELS
    return [(i, min(i + m, C)) for i in range(0, C, m)]


def _pad_last(t: Tensor, Cp: int) -> Tensor:
    C = t.shape[-1]
    return t if C == Cp else F.pad(t, (0, Cp - C))


def round_up(v, m):
    return (v + m - 1) // m * m


def packed_numel(B, N, Cp):
    """float32 elements of the packed buffer: per image roundup4(N) records of roundup4(6+Cp)
    floats plus an 8-float bin record each, the separable kernels' forward records (roundup4(10+Cp); none for
    more than 8 channels) and backward records (4), then 4 floats for the skip settings and a zero record of
    28 (the `packed_bytes` of igs_gs2d_plan, restated so that shape inference under torch.compile needs no
    library call)."""
    sep = (round_up(10 + Cp, 4) if Cp <= 8 else 0) + 4
    return B * round_up(N, 4) * (round_up(6 + Cp, 4) + 8 + sep) + 32


class Grid:
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
            self.mode = _lib.IGS_GRID_SEPARABLE | _options.get()[0]
        else:
            self.mode = _lib.IGS_GRID_AUTO | _options.get()[0]
            self.flag = torch.empty(1, dtype=torch.int32, device=x.device)
            _lib.check(_lib.load().igs_gs2d_grid_classify(_ptr(self.x), _ptr(self.y), self.strides, B, self.H,
                                                          self.W, _ptr(self.flag), _stream(x.device)),
                       "igs_gs2d_grid_classify")


class Splat:
    """One fused forward (+ backward) through the C ABI for a fixed problem."""

    def __init__(self, B, N, C, grid: Grid, eps: float, device):
        self.lib = _lib.load()
        self.B, self.N, self.C = B, N, C
        self.Cp = padded_channels(C)
        self.grid, self.eps, self.device = grid, float(eps), device
        self.plan = _lib.plan(B, N, grid.H, grid.W, self.Cp, grid.mode)
        self.skip_weight = skip_weight(N, self.eps)
        self.shared = None   # (pix, partial) with the tile lists in place, after forward_train
        self.stream = None
        self.use_current_stream()

    def use_current_stream(self):
        """Launch on the calling thread's current stream from here on (autograd runs the backward
        on its own thread, with the forward's stream made current there)."""
        self.stream = _stream(self.device)

    def _empty(self, nbytes: int) -> Tensor:
        return torch.empty(max(int(nbytes) // 4, 1), dtype=torch.float32, device=self.device)

    def _new(self, *shape) -> Tensor:
        return torch.empty(*shape, dtype=torch.float32, device=self.device)

    def pack_covinv(self, position, a, b, d, alphas, colors_p) -> Tensor:
        packed = self._empty(self.plan.packed_bytes)
        _lib.check(self.lib.igs_gs2d_pack_covinv(_ptr(position), _ptr(a), _ptr(b), _ptr(d), _ptr(alphas),
                                                 _ptr(colors_p), self.B, self.N, self.Cp, *self.skip_weight,
                                                 _ptr(packed), self.stream), "igs_gs2d_pack_covinv")
        return packed

    def pack_scale_rot(self, positions, scales, rotations, alphas, colors_p) -> Tensor:
        packed = self._empty(self.plan.packed_bytes)
        _lib.check(self.lib.igs_gs2d_pack_scale_rot(_ptr(positions), _ptr(scales), _ptr(rotations), _ptr(alphas),
                                                    _ptr(colors_p), self.B, self.N, self.Cp, self.eps,
                                                    *self.skip_weight, _ptr(packed), self.stream),
                   "igs_gs2d_pack_scale_rot")
        return packed

    def pack_feature(self, feat, off) -> Tuple[Tensor, Tensor]:
        packed = self._empty(self.plan.packed_bytes)
        col = self._new(self.B, self.N, self.Cp)
        _lib.check(self.lib.igs_gs2d_pack_feature(_ptr(feat), _ptr(off), self.B, self.N, self.C, self.Cp, self.eps,
                                                  *self.skip_weight, _ptr(packed), _ptr(col), self.stream),
                   "igs_gs2d_pack_feature")
        return packed, col

    def forward(self, packed: Tensor) -> Tuple[Tensor, Tensor]:
        g, p = self.grid, self.plan
        out = self._new(self.B, self.Cp, g.H, g.W)
        den = self._new(self.B, g.H, g.W)
        ws = self._empty(p.fwd_ws_bytes) if p.fwd_ws_bytes else None
        _lib.check(self.lib.igs_gs2d_forward(_ptr(packed), _ptr(g.x), _ptr(g.y), g.strides, g.mode, _ptr(g.flag),
                                             self.B, self.N,
                                             g.H, g.W, self.Cp, self.eps, _ptr(out), _ptr(den), _ptr(ws),
                                             int(p.fwd_ws_bytes), self.stream), "igs_gs2d_forward")
        return out, den

    def forward_train(self, packed: Tensor) -> Tuple[Tensor, Tensor]:
        """The forward of a step whose backward will follow: the backward's tile lists and tables are
        built now, in the backward's pixel workspace, which this object keeps for `backward_partials*`
        -- one set of lists for both passes where the plan says their tilings coincide
        (`plan.lists_shared`), else beside the forward's own, in the same launch.  Where the partial
        sums of every (Gaussian, tile) pair would be large, the number of listed pairs is written to
        pinned host memory, and the backward sizes its partial-sum array by it."""
        g, p = self.grid, self.plan
        out = self._new(self.B, self.Cp, g.H, g.W)
        den = self._new(self.B, g.H, g.W)
        ws = self._empty(p.fwd_ws_bytes) if p.fwd_ws_bytes else None
        pix = self._empty(p.pix_bytes)
        total = done = None
        # (not while the stream is being captured into a graph: a replay cannot wait for a host read;
        # the backward then takes the array for every pair)
        if p.partial_bytes > COMPACT_PARTIALS_FROM and not torch.cuda.is_current_stream_capturing():
            total = torch.empty(1, dtype=torch.int64, pin_memory=True)
        _lib.check(self.lib.igs_gs2d_forward_train(
            _ptr(packed), _ptr(g.x), _ptr(g.y), g.strides, g.mode, _ptr(g.flag), self.B, self.N, g.H, g.W, self.Cp,
            self.eps, _ptr(out), _ptr(den), _ptr(ws), int(p.fwd_ws_bytes), _ptr(pix), int(p.pix_bytes), _ptr(total),
            self.stream), "igs_gs2d_forward_train")
        if total is not None:
            done = torch.cuda.Event()
            done.record(torch.cuda.current_stream(self.device))
        self.shared = (pix, total, done)
        return out, den

    def _backward_workspaces(self):
        """(pix, partial, grid_mode): the pixel workspace that holds the tile lists already, if the
        forward built them, else a fresh one; the partial-sum array, sized by the number of listed
        (Gaussian, tile) pairs where the forward left it (the wait is for a point of the stream that
        lies before the forward's own kernels), else for every pair."""
        nbytes = int(self.plan.partial_bytes)
        if self.shared is not None:
            pix, total, done = self.shared
            if total is not None and (self.grid.mode & 0xff) == _lib.IGS_GRID_SEPARABLE:
                done.synchronize()
                nbytes = max(int(total.item()), 1) * (6 + self.Cp) * 4
            return pix, self._empty(nbytes), self.grid.mode | _lib.IGS_OPT_LISTS_BUILT
        return self._empty(self.plan.pix_bytes), self._empty(nbytes), self.grid.mode

    def backward_partials(self, packed, colors_p, out, den, grad_out_p) -> Tuple[Tensor, Tensor]:
        """(partial, pix): the partial sums and the pixel workspace whose tables the finalize call reads."""
        g, p = self.grid, self.plan
        pix, partial, mode = self._backward_workspaces()
        _lib.check(self.lib.igs_gs2d_backward(_ptr(packed), _ptr(colors_p), _ptr(g.x), _ptr(g.y), g.strides, mode,
                                              _ptr(g.flag), _ptr(out), _ptr(den), _ptr(grad_out_p), self.B, self.N, g.H, g.W,
                                              self.Cp, self.eps, _ptr(pix), int(p.pix_bytes), _ptr(partial),
                                              partial.numel() * 4, self.stream), "igs_gs2d_backward")
        return partial, pix

    def backward_partials_with_grid(self, packed, colors_p, out, den, grad_out_p, x_like, y_like):
        """The per-Gaussian partial sums and d L / d x_grid, d L / d y_grid from one call (on general
        grids the grid sums are formed inside the per-Gaussian reduction)."""
        g, p = self.grid, self.plan
        pix, partial, mode = self._backward_workspaces()
        # host-proven separable grids run the pixel-major grid kernel, which needs no workspace
        separable = (g.mode & 0xff) == _lib.IGS_GRID_SEPARABLE
        gws_bytes = 0 if separable else int(self.lib.igs_gs2d_grid_workspace_bytes(self.B, self.N, g.H, g.W, self.Cp))
        gws = None if separable else self._empty(gws_bytes)
        gx = self._new(self.B, g.H, g.W)
        gy = torch.empty_like(gx)
        _lib.check(self.lib.igs_gs2d_backward_with_grid(
            _ptr(packed), _ptr(colors_p), _ptr(g.x), _ptr(g.y), g.strides, mode, _ptr(g.flag), _ptr(out), _ptr(den),
            _ptr(grad_out_p), self.B, self.N, g.H, g.W, self.Cp, self.eps, _ptr(pix), int(p.pix_bytes), _ptr(partial),
            partial.numel() * 4, _ptr(gws), gws_bytes, _ptr(gx), _ptr(gy), self.stream), "igs_gs2d_backward_with_grid")
        return partial, pix, self._fit_grid(gx, x_like), self._fit_grid(gy, y_like)

    def _fit_grid(self, gr, like):
        shape, dtype = like
        if shape[0] == 1 and self.B > 1:      # batch-1 grid shared by all images
            gr = gr.sum(0, keepdim=True)
        return gr.reshape(shape).to(dtype)

    def grid_grads(self, packed, out, den, grad_out_p, x_like, y_like):
        """d L / d x_grid, d L / d y_grid in the (shape, dtype) of the tensors the caller passed."""
        g = self.grid
        gx = self._new(self.B, g.H, g.W)
        gy = torch.empty_like(gx)
        _lib.check(self.lib.igs_gs2d_backward_grid(_ptr(packed), _ptr(g.x), _ptr(g.y), g.strides, _ptr(out),
                                                   _ptr(den), _ptr(grad_out_p), self.B, self.N, g.H, g.W, self.Cp,
                                                   self.eps, _ptr(gx), _ptr(gy), self.stream),
                   "igs_gs2d_backward_grid")

        return self._fit_grid(gx, x_like), self._fit_grid(gy, y_like)

    def pad_grad_out(self, grad_out: Tensor) -> Tensor:
        """fp32 contiguous [B,Cp,H,W] upstream gradient (zero in the padding channels)."""
        go = _f32c(grad_out)
        if go.shape[1] != self.Cp:
            go = F.pad(go, (0, 0, 0, 0, 0, self.Cp - go.shape[1])).contiguous()
        return go


def check_gaussian_shapes(position, alphas, colors):
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


def problem_dims(kind: int, params: Sequence[Tensor]):
    """(B, N, C) of a parameter list, with the shape checks of its kind."""
    if kind == KIND_COVINV:
        if len(params) != 6:
            raise ValueError("expected (position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors)")
        position, a, b, d, alphas, colors = params
        B, N, C = check_gaussian_shapes(position, alphas, colors)
        for t in (a, b, d):
            if t.numel() != B * N:
                raise ValueError(f"cov_inv_* must hold B*N={B * N} elements; got {tuple(t.shape)}")
        return B, N, C
    if kind == KIND_SCALE_ROT:
        if len(params) != 5:
            raise ValueError("expected (positions, colors, scales, rotations, alphas)")
        positions, colors, scales, rotations, alphas = params
        B, N, C = check_gaussian_shapes(positions, alphas, colors)
        if scales.shape != (B, N, 2) or rotations.shape != (B, N):
            raise ValueError(f"scales must be [B,N,2] and rotations [B,N]; got {tuple(scales.shape)}, "
                             f"{tuple(rotations.shape)}")
        return B, N, C
    if kind == KIND_FEATURE:
        if len(params) not in (1, 2):
            raise ValueError("expected (gs_feature [, pos_offset])")
        feat = params[0]
        if feat.dim() != 3 or feat.shape[-1] < 7:
            raise ValueError(f"gs_feature must be [B,N,6+C]; got {tuple(feat.shape)}")
        B, N, F6 = feat.shape
        if N == 0:
            raise ValueError("need at least one Gaussian")
        if len(params) == 2 and params[1].shape != (B, N, 2):
            raise ValueError(f"pos_offset must be [B,N,2]; got {tuple(params[1].shape)}")
        return B, N, F6 - 6
    raise ValueError(f"unknown parameterisation {kind}")


def require_gpu(t: Tensor):
    if t.device.type != "cuda":
        raise RuntimeError("the fused Gaussian-splatting path runs on the GPU only (HIP kernels); got a tensor on "
                           f"{t.device}. Use fused=False for the plain-torch debug path.")
    _lib.load()


def require_same_device(dev, tensors: Sequence[Optional[Tensor]], what: str):
    """Every tensor whose address goes to the kernels must live on `dev`: a host pointer (or one of
    another GPU) handed to a launch is a memory fault, not an exception.  The reference raises
    torch's device-mismatch RuntimeError for mixed arguments; so does this, before any launch."""
    for t in tensors:
        if t is not None and t.device != dev:
            raise RuntimeError(f"Expected all tensors to be on the same device, but {what} has a tensor on "
                               f"{t.device} while the Gaussian parameters are on {dev}")


def run_forward(kind: int, params: Sequence[Tensor], x: Tensor, y: Tensor, eps: float, train: bool = False):
    """pack + splat.  Returns (op, keep, packed, col, out, den): `keep` are the fp32 contiguous
    copies of the parameters that the finalize kernel of this kind reads again, `col` the colours
    padded to the compiled channel count Cp, `out` [B,Cp,H,W] and `den` [B,H,W] in fp32.
    `train`: a backward through `op` will follow; where the plan allows, the tile lists are then
    built once for both passes (and `op` holds the backward's workspaces until it is released)."""
    require_gpu(params[0])
    B, N, C = problem_dims(kind, params)
    dev = params[0].device
    require_same_device(dev, list(params) + [x, y], "the forward")
    with _on(dev):
        grid = Grid(x, y, B)
        op = Splat(B, N, C, grid, eps, dev)
        if kind == KIND_COVINV:
            pos, a, b, d, al = (_f32c(t) for t in params[:5])
            col = _pad_last(_f32c(params[5]), op.Cp).contiguous()
            packed = op.pack_covinv(pos, a, b, d, al, col)
            keep = (a, b, d, al)
        elif kind == KIND_SCALE_ROT:
            pos, sc, rot, al = (_f32c(params[i]) for i in (0, 2, 3, 4))
            col = _pad_last(_f32c(params[1]), op.Cp).contiguous()
            packed = op.pack_scale_rot(pos, sc, rot, al, col)
            keep = (sc, rot, al)
        else:
            feat = _f32c(params[0])
            off = _f32c(params[1]) if len(params) == 2 else None
            packed, col = op.pack_feature(feat, off)
            keep = (feat,)
        general = (grid.mode & 0xff) == _lib.IGS_GRID_GENERAL   # (no tile lists on general grids)
        out, den = op.forward_train(packed) if (train and not general) else op.forward(packed)
    return op, keep, packed, col, out, den


def run_backward(kind: int, op: Splat, keep, packed, col, out, den, grad_result: Tensor, need: Sequence[bool],
                 need_x: bool, need_y: bool, grid_like) -> Tuple[List[Optional[Tensor]], Optional[Tensor],
                                                                   Optional[Tensor]]:
    """Splat backward + the chain rule of `kind`.  Returns (grads, g_x, g_y): `grads` in the order
    of the kind's parameter list, fp32, None where `need` is False; colour gradients cut back to
    C channels; cov_inv gradients as [B,N]."""
    B, N, C, Cp, dev = op.B, op.N, op.C, op.Cp, op.device
    require_same_device(dev, [grad_result, packed, col, out, den, *keep], "the backward")
    g_x = g_y = None
    grads: List[Optional[Tensor]] = [None] * len(need)
    with _on(dev):
        op.use_current_stream()
        go = op.pad_grad_out(grad_result)
        if (need_x or need_y) and any(need):
            partial, pix, g_x, g_y = op.backward_partials_with_grid(packed, col, out, den, go, *grid_like)
            g_x, g_y = (g_x if need_x else None), (g_y if need_y else None)
        else:
            if need_x or need_y:
                g_x, g_y = op.grid_grads(packed, out, den, go, *grid_like)
                g_x, g_y = (g_x if need_x else None), (g_y if need_y else None)
            if not any(need):
                return grads, g_x, g_y
            partial, pix = op.backward_partials(packed, col, out, den, go)
        mode, flag, H, W = op.grid.mode, _ptr(op.grid.flag), op.grid.H, op.grid.W
        if kind == KIND_COVINV:
            a, b, d, al = keep
            g_pos = op._new(B, N, 2) if need[0] else None
            g_a, g_b, g_d, g_al = (op._new(B, N) if need[k] else None for k in (1, 2, 3, 4))
            g_col = op._new(B, N, Cp) if need[5] else None
            _lib.check(op.lib.igs_gs2d_finalize_covinv(_ptr(partial), _ptr(pix), mode, flag, _ptr(a), _ptr(b), _ptr(d), _ptr(al),
                                                       B, N, H, W, Cp, _ptr(g_pos), _ptr(g_a), _ptr(g_b), _ptr(g_d),
                                                       _ptr(g_al), _ptr(g_col), op.stream),
                       "igs_gs2d_finalize_covinv")
            if g_col is not None and Cp != C:
                g_col = g_col[..., :C]
            grads = [g_pos, g_a, g_b, g_d, g_al, g_col]
        elif kind == KIND_SCALE_ROT:
            sc, rot, al = keep
            g_pos = op._new(B, N, 2) if need[0] else None
            g_col = op._new(B, N, Cp) if need[1] else None
            g_sc = op._new(B, N, 2) if need[2] else None
            g_rot = op._new(B, N) if need[3] else None
            g_al = op._new(B, N) if need[4] else None
            _lib.check(op.lib.igs_gs2d_finalize_scale_rot(_ptr(partial), _ptr(pix), mode, flag, _ptr(sc), _ptr(rot), _ptr(al),
                                                          B, N, H, W, Cp, op.eps, _ptr(g_pos), _ptr(g_sc), _ptr(g_rot),
                                                          _ptr(g_al), _ptr(g_col), op.stream),
                       "igs_gs2d_finalize_scale_rot")
            if g_col is not None and Cp != C:
                g_col = g_col[..., :C]
            grads = [g_pos, g_col, g_sc, g_rot, g_al]
        else:
            (feat,) = keep
            g_feat = op._new(B, N, 6 + C)
            _lib.check(op.lib.igs_gs2d_finalize_feature(_ptr(partial), _ptr(pix), mode, flag, _ptr(feat), B, N, H, W, C, Cp,
                                                        op.eps, _ptr(g_feat), op.stream),
                       "igs_gs2d_finalize_feature")
            grads = [g_feat if need[0] else None]
            if len(need) == 2:
                # the offset is added to the position: same gradient
                grads.append(g_feat[..., :2].contiguous() if need[1] else None)
    return grads, g_x, g_y
