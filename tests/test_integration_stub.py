"""Executes the binding stub that the integration guide publishes for maintainers of the reference
(the `HipGaussianSplatting2D` autograd Function a maintainer would add as src/igs/gs_hip.py and
select at src/igs/gs2d.py:471): the code block is taken from the guide as written, pointed at the
in-tree library, and its `.apply` is checked against the fp64 oracle, so the published text cannot
drift from the ABI.
"""
import os
import re

import pytest
import torch

from oracle import gs2d_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GUIDE = os.path.join(ROOT, "INTEGRATION.md")


def _stub_namespace():
    text = open(GUIDE).read()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    src = [b for b in blocks if "class HipGaussianSplatting2D" in b]
    assert len(src) == 1, "the guide must hold exactly one stub block"
    code = src[0]
    assert 'ctypes.CDLL("libigs_hip.so")' in code
    code = code.replace('ctypes.CDLL("libigs_hip.so")',
                        "ctypes.CDLL(%r)" % os.path.join(ROOT, "igs_amd", "libigs_hip.so"))
    ns = {}
    exec(compile(code, "integration_stub", "exec"), ns)
    return ns


def test_stub_block_compiles_and_binds_the_in_tree_library():
    ns = _stub_namespace()
    assert issubclass(ns["HipGaussianSplatting2D"], torch.autograd.Function)
    from igs_amd import _lib

    # the plan mirror in the stub has the layout of the header's struct
    import ctypes

    assert ctypes.sizeof(ns["_Plan"]) == ctypes.sizeof(_lib.Plan)
    assert [f[0] for f in ns["_Plan"]._fields_] == [f[0] for f in _lib.Plan._fields_]
    p = ns["_Plan"]()
    assert ns["_lib"].igs_gs2d_plan(2, 100, 8, 8, 3, 2, ctypes.byref(p)) == 0 and p.n_padded == 100


@pytest.mark.gpu
@pytest.mark.parametrize("general", [False, True])
def test_stub_apply_matches_the_oracle(general):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    dev = torch.device("cuda:0")
    Fn = _stub_namespace()["HipGaussianSplatting2D"]
    B, N, H, W, C = 2, 700, 37, 45, 3
    d = O.make_inputs(B, N, H, W, C, 0.05, 0.4, seed=31, dtype=torch.float64, expand_grids=False)
    if general:
        g = torch.Generator().manual_seed(5)
        d["x_grid"] = (torch.rand(B, 1, H, W, generator=g, dtype=torch.float64) * 2 - 1).float().double() * (W / H)
        d["y_grid"] = (torch.rand(B, 1, H, W, generator=g, dtype=torch.float64) * 2 - 1).float().double()
    a, b, c_ = (t.float().double() for t in O.cov_inverse_closed(d["scales"], d["rotations"]))
    ref_out, ref_g = O.operator_autograd(d["x_grid"], d["y_grid"], d["positions"], a, b, c_, d["alphas"], d["colors"],
                                         d["grad_out"])
    f = lambda t: t.to(dev, torch.float32)
    assert a.shape == (B, N, 1, 1)                       # the reference passes cov_inv_* as [B,N,1,1]
    leaves = [f(t).requires_grad_(True) for t in (d["positions"], a, b, c_, d["alphas"], d["colors"])]
    out = Fn.apply(f(d["x_grid"]), f(d["y_grid"]), *leaves)
    err = (out.detach().double().cpu() - ref_out).abs()
    assert bool((err <= 1e-6 + 1e-5 * ref_out.abs()).all()), float(err.max())
    out.backward(f(d["grad_out"]))
    for t, name in zip(leaves, ("position", "cov_inv_00", "cov_inv_01", "cov_inv_11", "alphas", "colors")):
        r = ref_g[name].reshape(t.grad.shape)
        diff = t.grad.double().cpu() - r
        assert float(diff.abs().max()) <= 1e-4 * float(r.abs().max()), name
        assert float(diff.norm()) <= 1e-4 * float(r.norm()), name
