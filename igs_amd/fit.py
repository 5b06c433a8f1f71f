"""Fused optimisation step of the reference's image-fitting loop.

The reference fits one set of Gaussians to an image with
`render -> loss -> loss.backward() -> AdamW.step()` per iteration
(scripts/2dgs_img_comp.py:107-126 for the render call, :186-193 for the optimiser, :219-232 for
the loop).  `GaussianImageFit.step()` runs that iteration for a mean-squared-error loss as one
sequence of HIP kernels on buffers allocated once:

    pack (split, exp(log_scale)+eps, alpha = 1, closed-form covariance inverse)
    -> splat forward -> per-pixel prologue with the MSE gradient formed in place (+ loss value)
    -> per-Gaussian backward reduction -> finalize (chain rule to the parameter block)
    -> AdamW on the block

No torch op and no allocation happens inside a step, so it can be captured in a HIP graph
(`capture()`), which removes the host launch cost from small problems; the step counter and the
learning rate live in device memory so that replays advance.

Two things of the script's loop beyond the mean-squared error are covered as well: its position
regulariser `0.01 * mean(relu(|position| - 1))` (scripts/2dgs_img_comp.py:224-228;
`position_penalty=`) is added to the gradient and the loss inside the step, and any other image
loss -- the script mixes SSIM-type terms, :133-142 -- can be supplied as `step(loss_fn=...)`: the
image goes to `loss_fn` as a torch leaf, torch differentiates the loss down to the image, and the
splat backward, the chain rule and AdamW run fused from that upstream gradient.

The parameters are one block `[B, N, 6+C]` in the layout of the module's `gs_feature`
(src/igs/gs2d.py:638-644): position (2), log-scale (2), rotation (1), an unused column,
colours (C) -- the same parameterisation as the fit script's `ProgressiveGaussianSplatter`
(position, log_scale, rotation, color with alphas = 1, scripts/2dgs_img_comp.py:95-126).  AdamW
is element-wise, so one step on the block equals one step on the four tensors.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch
import torch.nn.functional as F

from . import _lib
from ._splat import Grid, _ptr, _stream, padded_channels, skip_weight

Tensor = torch.Tensor


class GaussianImageFit:
    """State and fused step of an image fit.

    params   [B,N,6+C] float32 CUDA tensor; taken over (contiguous copy if needed) and updated
             in place by `step()`; read it through `.params` or `.named_parameters()`.
    target   [B,C,H,W] image(s) to fit.
    x_grid, y_grid  as for `gaussian_splatting_2d` ([B,1,H,W], [1,1,H,W], [B,H,W]; expanded
             linspace grids take the factored kernels).
    lr, betas, adam_eps, weight_decay  AdamW hyper-parameters (defaults: those of
             scripts/2dgs_img_comp.py:186-193 with lr for 4096 Gaussians).
    eps      the splat's eps (covariance regulariser and denominator guard).
    position_penalty  weight of `mean(relu(|position| - 1))` in the loss (the script uses 0.01; the
             mean runs over the positions of all B*N Gaussians, also in a prefix step, which moves
             only the active ones).
    """

    def __init__(self, params: Tensor, target: Tensor, x_grid: Tensor, y_grid: Tensor, lr: float = 0.03,
                 betas: Tuple[float, float] = (0.9, 0.995), adam_eps: float = 1e-6, weight_decay: float = 1e-4,
                 eps: float = 1e-6, position_penalty: float = 0.0):
        if params.device.type != "cuda":
            raise RuntimeError("GaussianImageFit runs on the GPU only (HIP kernels)")
        if params.dim() != 3 or params.shape[-1] < 7:
            raise ValueError(f"params must be [B,N,6+C]; got {tuple(params.shape)}")
        self.lib = _lib.load()
        self.device = params.device
        self.params = params.detach().to(torch.float32).contiguous()
        self.B, self.N, F6 = self.params.shape
        self.C = F6 - 6
        self.Cp = padded_channels(self.C)
        self.eps = float(eps)
        self.betas = (float(betas[0]), float(betas[1]))
        self.adam_eps, self.weight_decay = float(adam_eps), float(weight_decay)
        self.position_penalty = float(position_penalty)
        with torch.cuda.device(self.device):
            self.exp_avg = torch.zeros_like(self.params)
            self.exp_avg_sq = torch.zeros_like(self.params)
            # {lr, t, 1 - beta1^t, sqrt(1 - beta2^t)}
            self.state = torch.zeros(8, dtype=torch.float32, device=self.device)   # lr, t, bias corrections, ticket
            self.loss = torch.zeros((), dtype=torch.float32, device=self.device)
        self._ws: Dict[int, dict] = {}
        self._graphs: Dict[int, torch.cuda.CUDAGraph] = {}
        self.set_lr(lr)
        self.set_target(target, x_grid, y_grid)

    # ------------------------------------------------------------------ construction helpers
    @classmethod
    def from_parameters(cls, position: Tensor, log_scale: Tensor, rotation: Tensor, color: Tensor, *args, **kwargs):
        """Build the block from the fit script's four tensors: position [B,N,2], log_scale [B,N,2],
        rotation [B,N], color [B,N,C]."""
        B, N, _ = position.shape
        block = torch.cat([position, log_scale, rotation[..., None], torch.zeros_like(rotation)[..., None], color],
                          dim=-1)
        return cls(block, *args, **kwargs)

    def named_parameters(self) -> Dict[str, Tensor]:
        """Views of the block under the fit script's parameter names."""
        p = self.params
        return {"position": p[..., 0:2], "log_scale": p[..., 2:4], "rotation": p[..., 4], "color": p[..., 6:]}

    # ------------------------------------------------------------------ configuration
    def set_lr(self, lr: float):
        """Learning rate of the following steps (a stream-ordered device write: also valid between
        graph replays)."""
        self.lr = float(lr)
        self.state[0:1].fill_(self.lr)

    def set_target(self, target: Tensor, x_grid: Tensor, y_grid: Tensor):
        """(New) target image and grids, e.g. the next level of a progressive-resolution schedule
        (scripts/2dgs_img_comp.py:208-217).  Workspaces and captured graphs are rebuilt."""
        if target.dim() != 4 or target.shape[0] != self.B or target.shape[1] != self.C:
            raise ValueError(f"target must be [B,C,H,W] = [{self.B},{self.C},H,W]; got {tuple(target.shape)}")
        with torch.cuda.device(self.device):
            self.grid = Grid(x_grid.to(self.device), y_grid.to(self.device), self.B)
            if (self.grid.H, self.grid.W) != tuple(target.shape[-2:]):
                raise ValueError("target and grids differ in H, W")
            t = target.detach().to(device=self.device, dtype=torch.float32)
            if self.Cp != self.C:
                t = F.pad(t, (0, 0, 0, 0, 0, self.Cp - self.C))
            self.target = t.contiguous()
        self._ws.clear()
        self._graphs.clear()

    def _active(self, num_active: Optional[int]) -> int:
        n = self.N if num_active is None else max(1, min(int(num_active), self.N))
        if n != self.N and self.B != 1:
            raise ValueError("a prefix of the Gaussians (num_active) needs B == 1, as in the reference's fit script")
        return n

    def _workspace(self, n: int) -> dict:
        ws = self._ws.get(n)
        if ws is None:
            g = self.grid
            plan = _lib.plan(self.B, n, g.H, g.W, self.Cp, g.mode)
            loss_bytes = int(self.lib.igs_gs2d_mse_workspace_bytes(self.B, g.H, g.W))
            with torch.cuda.device(self.device):
                buf = lambda nbytes: torch.empty(max(int(nbytes) // 4, 1), dtype=torch.float32, device=self.device)
                new = lambda *s: torch.empty(*s, dtype=torch.float32, device=self.device)
                ws = dict(plan=plan, skip_weight=skip_weight(n, self.eps), packed=buf(plan.packed_bytes),
                          col=new(self.B, n, self.Cp),
                          out=new(self.B, self.Cp, g.H, g.W), den=new(self.B, g.H, g.W),
                          fwd_ws=buf(plan.fwd_ws_bytes) if plan.fwd_ws_bytes else None, pix=buf(plan.pix_bytes),
                          partial=buf(plan.partial_bytes), loss_ws=buf(loss_bytes), loss_bytes=loss_bytes,
                          g_feat=new(self.B, n, 6 + self.C))
            self._ws[n] = ws
        return ws

    # ------------------------------------------------------------------ the step
    def _enqueue_render(self, n: int, ws: dict, st, train: bool = False):
        """pack + forward.  `train`: the backward follows; its tile lists are then built by the forward's
        binning launch, in the backward's workspaces (one set for both passes where the plan's tilings
        coincide, `lists_shared`)."""
        lib, g, p = self.lib, self.grid, ws["plan"]
        B, C, Cp, H, W = self.B, self.C, self.Cp, g.H, g.W
        _lib.check(lib.igs_gs2d_pack_feature(_ptr(self.params), None, B, n, C, Cp, self.eps, *ws["skip_weight"],
                                             _ptr(ws["packed"]), _ptr(ws["col"]), st), "igs_gs2d_pack_feature")
        if train:
            _lib.check(lib.igs_gs2d_forward_train(
                _ptr(ws["packed"]), _ptr(g.x), _ptr(g.y), g.strides, g.mode, _ptr(g.flag), B, n, H, W, Cp, self.eps,
                _ptr(ws["out"]), _ptr(ws["den"]), _ptr(ws["fwd_ws"]), int(p.fwd_ws_bytes), _ptr(ws["pix"]),
                int(p.pix_bytes), None, st), "igs_gs2d_forward_train")
            return
        _lib.check(lib.igs_gs2d_forward(_ptr(ws["packed"]), _ptr(g.x), _ptr(g.y), g.strides, g.mode, _ptr(g.flag), B, n,
                                        H, W, Cp, self.eps, _ptr(ws["out"]), _ptr(ws["den"]), _ptr(ws["fwd_ws"]),
                                        int(p.fwd_ws_bytes), st), "igs_gs2d_forward")

    def _enqueue_backward(self, n: int, ws: dict, st, grad_out: Optional[Tensor]):
        """Everything after the render: per-pixel prologue (from `grad_out` [B,Cp,H,W], or with the
        mean-squared-error gradient and loss formed in place when it is None), per-Gaussian
        reduction, chain rule, position penalty, AdamW."""
        lib, g, p = self.lib, self.grid, ws["plan"]
        B, C, Cp, H, W = self.B, self.C, self.Cp, g.H, g.W
        if grad_out is None:
            _lib.check(lib.igs_gs2d_backward_prologue_mse(_ptr(g.x), _ptr(g.y), g.strides, g.mode, _ptr(g.flag),
                                                          _ptr(ws["out"]), _ptr(ws["den"]), _ptr(self.target), C, B, n,
                                                          H, W, Cp, self.eps, _ptr(ws["pix"]), int(p.pix_bytes),
                                                          _ptr(ws["loss_ws"]), ws["loss_bytes"], _ptr(self.loss), st),
                       "igs_gs2d_backward_prologue_mse")
        else:
            _lib.check(lib.igs_gs2d_backward_prologue(_ptr(g.x), _ptr(g.y), g.strides, g.mode, _ptr(g.flag),
                                                      _ptr(ws["out"]), _ptr(ws["den"]), _ptr(grad_out), B, n, H, W, Cp,
                                                      self.eps, _ptr(ws["pix"]), int(p.pix_bytes), st),
                       "igs_gs2d_backward_prologue")
        mode = g.mode | _lib.IGS_OPT_LISTS_BUILT  # (the render of a step built them)
        _lib.check(lib.igs_gs2d_backward_reduce(_ptr(ws["packed"]), _ptr(ws["col"]), _ptr(g.y), g.strides, mode,
                                                _ptr(g.flag), B, n, H, W, Cp, _ptr(ws["pix"]), int(p.pix_bytes),
                                                _ptr(ws["partial"]), int(p.partial_bytes), st),
                   "igs_gs2d_backward_reduce")
        _lib.check(lib.igs_gs2d_finalize_feature(_ptr(ws["partial"]), _ptr(ws["pix"]), g.mode, _ptr(g.flag), _ptr(self.params), B, n, H,
                                                 W, C, Cp, self.eps, _ptr(ws["g_feat"]), st),
                   "igs_gs2d_finalize_feature")
        if self.position_penalty != 0.0:
            _lib.check(lib.igs_gs2d_position_penalty(_ptr(self.params), B * n, 6 + C, self.position_penalty,
                                                     2 * B * self.N, _ptr(ws["g_feat"]), _ptr(self.loss), st),
                       "igs_gs2d_position_penalty")
        # B == 1 or n == N: the active prefix is the first B*n*(6+C) floats of every block
        _lib.check(lib.igs_adamw_step(_ptr(self.params), _ptr(ws["g_feat"]), _ptr(self.exp_avg), _ptr(self.exp_avg_sq),
                                      B * n * (6 + C), _ptr(self.state), self.betas[0], self.betas[1], self.adam_eps,
                                      self.weight_decay, st), "igs_adamw_step")

    def _enqueue_step(self, n: int):
        ws = self._workspace(n)
        st = _stream(self.device)
        self._enqueue_render(n, ws, st, train=True)
        self._enqueue_backward(n, ws, st, None)

    def _step_with_loss_fn(self, n: int, loss_fn):
        ws = self._workspace(n)
        st = _stream(self.device)
        self._enqueue_render(n, ws, st, train=True)
        image = ws["out"][:, :self.C].detach().requires_grad_(True)       # a view: no copy
        with torch.enable_grad():
            loss = loss_fn(image)
            if loss.dim() != 0:
                raise ValueError("loss_fn must return a scalar tensor")
            (g,) = torch.autograd.grad(loss, image)
        g = g.to(torch.float32)
        if self.Cp != self.C:
            g = F.pad(g, (0, 0, 0, 0, 0, self.Cp - self.C))
        self.loss.copy_(loss.detach())
        self._enqueue_backward(n, ws, st, g.contiguous())

    def step(self, num_active: Optional[int] = None, loss_fn=None) -> Tensor:
        """One iteration on the first `num_active` Gaussians (default all; the progressive
        schedule of scripts/2dgs_img_comp.py:107-111).  Returns the loss of the image rendered
        *before* the update as a 0-dim device tensor that the next step overwrites; nothing
        synchronises.  Replays the captured graph when `capture()` was called for this count.

        With `loss_fn` (image [B,C,H,W] -> scalar tensor, differentiable torch code; the target is
        the caller's business) that loss replaces the mean-squared error: torch differentiates it
        down to the image and the fused backward starts from that gradient.  Such a step is not
        replayed from a graph (the loss runs in torch)."""
        n = self._active(num_active)
        if loss_fn is not None:
            with torch.cuda.device(self.device):
                self._step_with_loss_fn(n, loss_fn)
            return self.loss
        graph = self._graphs.get(n)
        if graph is not None:
            graph.replay()
        else:
            with torch.cuda.device(self.device):
                self._enqueue_step(n)
        return self.loss

    def capture(self, num_active: Optional[int] = None):
        """Record the step for `num_active` Gaussians into a HIP graph; later `step()` calls with
        the same count replay it.  Recording executes nothing: parameters and optimiser state
        are unchanged by this call."""
        n = self._active(num_active)
        with torch.cuda.device(self.device):
            self._workspace(n)             # allocate outside the capture
            torch.cuda.synchronize(self.device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                self._enqueue_step(n)
        self._graphs[n] = graph

    @torch.no_grad()
    def render(self, num_active: Optional[int] = None) -> Tensor:
        """The current image [B,C,H,W] (a copy)."""
        n = self._active(num_active)
        with torch.cuda.device(self.device):
            ws = self._workspace(n)
            self._enqueue_render(n, ws, _stream(self.device))
            return ws["out"][:, :self.C].clone()

    @property
    def step_count(self) -> int:
        """Steps taken so far (reads the device counter: synchronises)."""
        return int(self.state[1].item())
