"""The drop-in conventions against vectors written by the reference's own Python
(tests/golden/reference_conventions.npz, made by tests/golden/make_reference_golden.py from
src/igs/gs2d.py run on the CPU, plain-torch path): module initialisation (RNG order), the
gs_feature split order and activations, xy_grid, pos_map_offset, naive_gaussian_2d and the
covariance preamble.  Checked here: the oracle, this package's plain-torch path (CPU) and, on a
GPU, the fused HIP path.
"""
import os

import numpy as np
import pytest
import torch

from oracle import gs2d_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def ref():
    z = np.load(os.path.join(HERE, "golden", "reference_conventions.npz"), allow_pickle=False)
    return {k: torch.from_numpy(z[k]) if z[k].shape else z[k] for k in z.files}


def _close(a, b, rtol=1e-5, atol=1e-6):
    a, b = a.detach().cpu().double(), b.double()
    assert a.shape == b.shape, (a.shape, b.shape)
    err = (a - b).abs()
    assert bool((err <= atol + rtol * b.abs()).all()), f"max err {float(err.max()):.3e}"


def _modules(ref):
    import igs_amd

    m = igs_amd.GaussianSplatting2D(4, 32)
    m.load_state_dict({"proj.weight": ref["fwd_weight"], "proj.bias": ref["fwd_bias"]})
    mo = igs_amd.GaussianSplatting2D(3, 16, output_dim=2, pos_map_offset=True)
    mo.load_state_dict({"proj.weight": ref["off_weight"], "proj.bias": ref["off_bias"]})
    return m, mo


# ------------------------------------------------------------------ CPU: host logic + oracle
def test_seeded_module_init_equals_the_reference_bit_for_bit(ref):
    import igs_amd

    torch.manual_seed(int(ref["init_seed"]))
    m = igs_amd.GaussianSplatting2D(4, 32)
    sd = m.state_dict()
    assert sorted(sd) == ["proj.bias", "proj.weight"]
    assert torch.equal(sd["proj.weight"], ref["init_weight"])
    assert torch.equal(sd["proj.bias"], ref["init_bias"])


def test_xy_grid_equals_the_reference(ref):
    import igs_amd

    size = tuple(int(v) for v in ref["xy_size"])
    for fn in (igs_amd.GaussianSplatting2D.xy_grid, O.xy_grid):
        xg, yg = fn(size)
        assert xg.shape == ref["xy_x"].shape
        assert torch.equal(xg.contiguous(), ref["xy_x"]) and torch.equal(yg.contiguous(), ref["xy_y"])


def test_oracle_naive_expression_equals_the_reference(ref):
    for tag in ("naive_a", "naive_b"):
        a = {k[len(tag) + 1:]: v for k, v in ref.items() if k.startswith(tag + "_")}
        out = O.naive_gaussian_2d(*(a[k].double() for k in ("x", "y", "position", "a", "b", "d", "alphas", "colors")))
        _close(out, a["out"], rtol=2e-5, atol=2e-6)          # fp64 oracle vs the reference in fp32
        out32 = O.naive_gaussian_2d(*(a[k] for k in ("x", "y", "position", "a", "b", "d", "alphas", "colors")))
        _close(out32, a["out"], rtol=2e-6, atol=2e-7)        # same expression in fp32


def test_oracle_render_and_closed_form_preamble_equal_the_reference(ref):
    r = {k[7:]: v for k, v in ref.items() if k.startswith("render_")}
    for closed in (False, True):
        out = O.render_naive(*(r[k].double() for k in ("positions", "colors", "scales", "rotations", "alphas")),
                             r["x"].double(), r["y"].double(), 1e-6, closed)
        _close(out, r["out"], rtol=3e-5, atol=3e-6)


def test_oracle_module_forward_equals_the_reference(ref):
    img, feat = O.module_forward(ref["fwd_weight"].double(), ref["fwd_bias"].double(), ref["fwd_x"].double(), (6, 10), 4)
    _close(feat, ref["fwd_gs_feature"], rtol=1e-5, atol=1e-5)
    _close(img, ref["fwd_image"], rtol=1e-4, atol=1e-5)


def test_plain_torch_path_of_the_package_equals_the_reference(ref):
    import igs_amd

    m, mo = _modules(ref)
    with torch.no_grad():
        img, feat = m(ref["fwd_x"], size=(6, 10), fused=False)
        img_o, feat_o = mo(ref["off_x"], grid=ref["off_grid"], fused=False)
    _close(feat, ref["fwd_gs_feature"], rtol=1e-6, atol=1e-6)
    _close(img, ref["fwd_image"], rtol=1e-5, atol=1e-6)
    _close(feat_o, ref["off_gs_feature"], rtol=1e-6, atol=1e-6)
    _close(img_o, ref["off_image"], rtol=1e-5, atol=1e-6)
    r = {k[7:]: v for k, v in ref.items() if k.startswith("render_")}
    out = igs_amd.gaussian_splatting_2d(r["positions"], r["colors"], r["scales"], r["rotations"], r["alphas"],
                                        r["x"], r["y"], 1e-6, False)
    _close(out, r["out"], rtol=1e-5, atol=1e-6)
    a = {k[8:]: v for k, v in ref.items() if k.startswith("naive_a_")}
    out = igs_amd.naive_gaussian_2d(*(a[k] for k in ("x", "y", "position", "a", "b", "d", "alphas", "colors")))
    _close(out, a["out"], rtol=2e-6, atol=2e-7)


# ------------------------------------------------------------------ GPU: the fused HIP path
@pytest.mark.gpu
def test_fused_hip_path_equals_the_reference(ref):
    import igs_amd

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    dev = torch.device("cuda:0")
    m, mo = _modules(ref)
    m, mo = m.to(dev), mo.to(dev)
    with torch.no_grad():
        img, feat = m(ref["fwd_x"].to(dev), size=(6, 10))
        img_o, feat_o = mo(ref["off_x"].to(dev), grid=ref["off_grid"].to(dev))
    # both sides are fp32 evaluations with different roundings (the reference inverts the covariance
    # matrix in fp32, src/igs/gs2d.py:567-573, and its linear head runs on the CPU): a few 1e-5; a
    # wrong split order, activation or grid convention would show at order 1
    _close(feat, ref["fwd_gs_feature"], rtol=1e-5, atol=5e-6)
    _close(img, ref["fwd_image"], rtol=5e-5, atol=5e-6)
    _close(feat_o, ref["off_gs_feature"], rtol=1e-5, atol=5e-6)
    _close(img_o, ref["off_image"], rtol=5e-5, atol=5e-6)
    r = {k[7:]: v.to(dev) for k, v in ref.items() if k.startswith("render_")}
    out = igs_amd.gaussian_splatting_2d(r["positions"], r["colors"], r["scales"], r["rotations"], r["alphas"],
                                        r["x"], r["y"])
    _close(out, r["out"].cpu(), rtol=5e-5, atol=5e-6)
    for tag in ("naive_a", "naive_b"):
        a = {k[len(tag) + 1:]: v.to(dev) for k, v in ref.items() if k.startswith(tag + "_")}
        out = igs_amd.GaussianSplatting2DKernel.apply(a["x"], a["y"], a["position"], a["a"], a["b"], a["d"],
                                                      a["alphas"], a["colors"])
        _close(out, a["out"].cpu(), rtol=1e-5, atol=2e-6)
