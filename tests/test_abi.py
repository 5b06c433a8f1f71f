"""The C-ABI library loads and exports every symbol include/igs_hip.h declares; host-side
plan arithmetic and argument checks (no kernel is launched, no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "igs_hip.h")


@pytest.fixture(scope="module")
def lib():
    from igs_amd import _lib, build

    if build.is_stale():
        build.build(verbose=False)
    return _lib.load()


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(igs_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(lib):
    from igs_amd import _lib

    names = declared_symbols()
    assert "igs_gs2d_forward" in names and "igs_gs2d_backward_reduce" in names and len(names) >= 12
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in igs_hip.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names


def test_header_cites_reference_for_each_entry_point():
    text = open(HEADER).read()
    assert text.count("src/igs/") >= 8


def test_plan_struct_matches_header_layout(lib):
    from igs_amd import _lib

    text = open(HEADER).read()
    body = text[text.index("typedef struct igs_gs2d_plan_t {"):text.index("} igs_gs2d_plan_t;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = []
    for decl in body.split("{", 1)[1].split(";"):
        decl = decl.strip()
        if not decl:
            continue
        typ, rest = decl.split(None, 1)
        fields += [(f.strip(), typ) for f in rest.split(",")]
    assert [f for f, _ in fields] == [f for f, _ in _lib.Plan._fields_]
    for (name, typ), (_, ct) in zip(fields, _lib.Plan._fields_):
        assert ct is {"int32_t": ctypes.c_int32, "uint64_t": ctypes.c_uint64}[typ], name


def _sep_record_floats(C):
    """Floats per Gaussian of the separable kernels' own records: the forward's (px, py, three terms, alpha,
    C colours, a tag, the three plain terms; rounded up to 4; none for more than 8 channels) and the backward's 4."""
    return ((10 + C + 3) // 4 * 4 if C <= 8 else 0) + 4


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_plan_arithmetic(lib, mode):
    from igs_amd import _lib

    for (B, N, H, W, C) in [(1, 2048, 256, 256, 3), (16, 8192, 256, 256, 3), (4, 32768, 384, 640, 16), (2, 5, 3, 4, 1)]:
        p = _lib.plan(B, N, H, W, C, mode)
        assert p.n_padded % 4 == 0 and p.n_padded >= N
        assert p.fwd_n_per_split % 4 == 0 and p.fwd_split * p.fwd_n_per_split >= p.n_padded
        assert (p.fwd_split - 1) * p.fwd_n_per_split < p.n_padded          # no empty split
        # records + bin records + the separable kernels' forward and backward records, skip settings + zero record
        assert p.packed_bytes == (B * p.n_padded * (p.rec_stride + 8 + _sep_record_floats(C)) + 32) * 4
        assert p.rec_stride % 4 == 0 and p.rec_stride >= 6 + C
        assert p.bwd_tiles >= 1 and p.partial_bytes >= B * p.bwd_tiles * (6 + C) * N * 4
        if mode != 0:
            assert p.w_padded % 8 == 0 and p.bwd_tiles % p.bwd_tiles_x == 0
            assert (p.bwd_tiles // p.bwd_tiles_x) * p.bwd_per_tile >= H and p.bwd_tiles_x * p.bwd_tile_w >= W
            # room for the per-tile Gaussian lists behind the other scratch
            assert p.fwd_tiles >= 1 and p.fwd_ws_bytes >= B * p.fwd_tiles * (p.n_padded + 1) * 4
            assert p.pix_bytes >= B * H * W * (C + 1) * 4 + B * p.bwd_tiles * (p.n_padded + 1) * 4
        assert p.pix_bytes >= B * H * W * (C + 1) * 4
    a, s_, g = (_lib.plan(8, 4096, 256, 256, 3, m) for m in (2, 1, 0))
    assert a.pix_bytes == max(s_.pix_bytes, g.pix_bytes) and a.fwd_ws_bytes == max(s_.fwd_ws_bytes, g.fwd_ws_bytes)


def test_argument_errors_are_status_codes_not_crashes(lib):
    from igs_amd import _lib

    p = _lib.Plan()
    assert lib.igs_gs2d_plan(0, 8, 4, 4, 3, 1, ctypes.byref(p)) == -2
    assert lib.igs_gs2d_plan(1, 8, 4, 4, 0, 1, ctypes.byref(p)) == -3
    assert lib.igs_gs2d_plan(1, 8, 4, 4, 17, 1, ctypes.byref(p)) == -3
    assert lib.igs_gs2d_plan(1, 8, 4, 4, 5, 1, ctypes.byref(p)) == -3     # not a compiled channel count
    assert lib.igs_gs2d_plan(1, 8, 4, 4, 3, 7, ctypes.byref(p)) == -5
    assert lib.igs_gs2d_plan(1, 8, 4, 4, 3, 1, None) == -1
    # size limits: B <= 65535, N <= 2^24, B N <= 2^28, H W <= 2^28
    assert lib.igs_gs2d_plan(65536, 8, 4, 4, 3, 1, ctypes.byref(p)) == -2
    assert lib.igs_gs2d_plan(1, (1 << 24) + 1, 4, 4, 3, 1, ctypes.byref(p)) == -2
    assert lib.igs_gs2d_plan(32, 1 << 24, 4, 4, 3, 1, ctypes.byref(p)) == -2
    assert lib.igs_gs2d_plan(1, 8, 1 << 14, (1 << 14) + 1, 3, 1, ctypes.byref(p)) == -2
    assert lib.igs_gs2d_plan(1, 1 << 24, 64, 64, 3, 1, ctypes.byref(p)) == 0
    assert lib.igs_gs2d_plan(1, 8, 1 << 14, 1 << 14, 3, 1, ctypes.byref(p)) == 0
    # null pointers are rejected before anything is launched
    fake = ctypes.c_void_p(4096)
    st = _lib.strides6((0, 0, 1), (0, 4, 0))
    assert lib.igs_gs2d_forward(None, None, None, st, 1, None, 1, 8, 4, 4, 3, 1e-6, None, None, None, 0, None) == -1
    assert lib.igs_gs2d_pack_covinv(None, None, None, None, None, None, 1, 8, 3, 0.0, 0.0, None, None) == -1
    # the skip weight of a pack call: 0 <= w < 1
    for bad in (-1e-9, 1.0, float("nan")):
        assert lib.igs_gs2d_pack_covinv(fake, fake, fake, fake, fake, fake, 1, 8, 3, bad, 0.0, fake, None) == -9
        assert lib.igs_gs2d_pack_covinv(fake, fake, fake, fake, fake, fake, 1, 8, 3, 0.0, bad, fake, None) == -9
        assert lib.igs_gs2d_pack_scale_rot(fake, fake, fake, fake, fake, 1, 8, 3, 1e-6, bad, 0.0, fake, None) == -9
        assert lib.igs_gs2d_pack_feature(fake, None, 1, 8, 3, 3, 1e-6, 0.0, bad, fake, fake, None) == -9
    assert b"skip weight" in lib.igs_status_string(-9)
    # tolerance * eps / (2 N); nothing may be skipped without an eps to measure against
    assert lib.igs_gs2d_skip_weight(8192, 1e-6, 1e-7) == pytest.approx(1e-13 / 16384, rel=1e-6)
    assert lib.igs_gs2d_skip_weight(8192, 0.0, 1e-7) == 0.0 and lib.igs_gs2d_skip_weight(8192, 1e-6, 0.0) == 0.0
    assert lib.igs_gs2d_skip_weight(1, 1.0, 0.9) < 1.0
    assert lib.igs_gs2d_finalize_covinv(None, None, 1, None, None, None, None, None, 1, 8, 4, 4, 3,
                                        None, None, None, None, None, None, None) == -1
    assert lib.igs_gs2d_backward_with_grid(None, None, None, None, st, 1, None, None, None, None, 1, 8, 4, 4, 3, 1e-6,
                                           None, 0, None, 0, None, 0, None, None, None) == -1
    assert lib.igs_gs2d_grid_workspace_bytes(2, 3000, 10, 13, 3) == 2 * 3 * 132 * 8     # B x groups x roundup4(HW) x float2
    assert lib.igs_gs2d_grid_workspace_bytes(2, 3000, 10, 13, 5) == 0                   # not a compiled channel count
    assert lib.igs_gs2d_backward_with_grid(fake, fake, fake, fake, st, 0, None, fake, fake, fake, 2, 3000, 10, 13, 3,
                                           1e-6, fake, 1 << 30, fake, 1 << 30, fake, 8, fake, fake, None) == -4
    assert b"workspace" in lib.igs_status_string(-4)
    # host-proven separable grids need no grid workspace: the call gets past that check (and stops
    # at the next one, the pixel workspace, here 0 bytes) ...
    assert lib.igs_gs2d_backward_with_grid(fake, fake, fake, fake, st, 1, None, fake, fake, fake, 2, 3000, 10, 13, 3,
                                           1e-6, fake, 0, fake, 1 << 30, None, 0, fake, fake, None) == -4
    # ... while general grids insist on it
    assert lib.igs_gs2d_backward_with_grid(fake, fake, fake, fake, st, 0, None, fake, fake, fake, 2, 3000, 10, 13, 3,
                                           1e-6, fake, 1 << 30, fake, 1 << 30, None, 0, fake, fake, None) == -1
    # option bits ride in the grid_mode word; unknown or contradictory ones are rejected
    assert lib.igs_gs2d_forward(fake, fake, fake, st, 1 | 0x1000, None, 1, 8, 4, 4, 3, 1e-6, fake, fake, fake, 1 << 30,
                                None) == -5
    assert lib.igs_gs2d_forward(fake, fake, fake, st, 1 | 0x200 | 0x400, None, 1, 8, 4, 4, 3, 1e-6, fake, fake, fake,
                                1 << 30, None) == -5
    assert lib.igs_gs2d_plan(1, 8, 4, 4, 3, 1 | 0x100 | 0x400, ctypes.byref(p)) == 0      # sizes ignore them
    with pytest.raises(RuntimeError):
        _lib.check(-2, "x")


def test_missing_library_fails_loudly(monkeypatch):
    from igs_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libigs_hip.so")
    with pytest.raises(_lib.IGSLibraryError):
        _lib.load()


def test_fused_path_refuses_cpu_tensors():
    import torch

    import igs_amd
    from oracle import gs2d_oracle as O

    d = O.make_config_inputs("c0", N=16, H=8, W=8)
    with pytest.raises(RuntimeError, match="GPU only"):
        igs_amd.gaussian_splatting_2d(d["positions"], d["colors"], d["scales"], d["rotations"], d["alphas"],
                                      d["x_grid"], d["y_grid"])
    with pytest.raises(RuntimeError, match="GPU only"):
        a = torch.ones(1, 16, 1, 1)
        igs_amd.GaussianSplatting2DKernel.apply(d["x_grid"], d["y_grid"], d["positions"], a, a * 0, a, d["alphas"], d["colors"])


def test_mixed_device_arguments_are_refused_before_any_launch():
    """A host tensor among device tensors must raise, never reach a kernel as a host pointer (the
    check itself needs no GPU: a torch.device is only a name)."""
    import torch

    from igs_amd import _splat

    gpu = torch.device("cuda", 0)
    host = torch.zeros(2)
    with pytest.raises(RuntimeError, match="same device"):
        _splat.require_same_device(gpu, [None, host], "the forward")
    _splat.require_same_device(host.device, [host, None, host], "the forward")


def test_host_api_surface_and_module_init():
    import torch

    import igs_amd
    from oracle import gs2d_oracle as O

    for n in ("GaussianSplatting2D", "gaussian_splatting_2d", "naive_gaussian_2d", "GaussianSplatting2DKernel",
              "TorchGaussianSplatting2DKernel", "TorchGaussianSplatting2DChunked", "GaussianSplatting2DChunkedKernel"):
        assert hasattr(igs_amd, n)
    torch.manual_seed(0)
    m = igs_amd.GaussianSplatting2D(4, 32, output_dim=3)
    assert sorted(m.state_dict()) == ["proj.bias", "proj.weight"]
    assert m.proj.weight.shape == (4 * 9, 32)
    b = m.proj.bias.view(4, 9)
    assert torch.all(b[:, :2] == 0) and torch.all(b[:, 2:4] == -4)
    xg, yg = igs_amd.GaussianSplatting2D.xy_grid((6, 10))
    ox, oy = O.xy_grid((6, 10))
    assert torch.equal(xg, ox) and torch.equal(yg, oy) and xg.stride(1) == 0 and yg.stride(2) == 0
    # fused=False debug path on the CPU equals the oracle's naive expression
    x = torch.randn(2, 3, 32)
    img, feat = m(x, size=(6, 10), fused=False)
    rimg, rfeat = O.module_forward(m.proj.weight.detach(), m.proj.bias.detach(), x, (6, 10), 4)
    assert torch.allclose(img, rimg, rtol=1e-5, atol=1e-6) and torch.equal(feat, rfeat)


@pytest.mark.parametrize("B,N,H,W,C", [(2, 37, 8, 12, 3), (1, 1, 1, 1, 1), (3, 130, 5, 70, 5), (1, 64, 9, 9, 16)])
def test_registered_operator_shape_functions(B, N, H, W, C):
    """The shape functions that torch.compile uses for igs_amd::splat_fwd / splat_bwd agree with
    the library's own plan (evaluated on meta tensors: no GPU, no kernel)."""
    import torch

    import igs_amd  # noqa: F401  (registers the operators)
    from igs_amd import _lib, _splat

    m = lambda *s: torch.empty(*s, device="meta")
    Cp = _splat.padded_channels(C)
    grids = (m(B, 1, H, W), m(1, 1, H, W))
    for kind, params in ((_splat.KIND_SCALE_ROT, [m(B, N, 2), m(B, N, C), m(B, N, 2), m(B, N), m(B, N)]),
                         (_splat.KIND_COVINV, [m(B, N, 2), m(B, N, 1, 1), m(B, N), m(B, N, 1), m(B, N), m(B, N, C)]),
                         (_splat.KIND_FEATURE, [m(B, N, 6 + C), m(B, N, 2)])):
        out, den, packed, col = torch.ops.igs_amd.splat_fwd(kind, params, *grids, 1e-6)
        assert out.shape == (B, Cp, H, W) and den.shape == (B, H, W) and col.shape == (B, N, Cp)
        assert packed.numel() * 4 == _lib.plan(B, N, H, W, Cp, _lib.IGS_GRID_AUTO).packed_bytes
        assert out.dtype == torch.float32
        g = torch.ops.igs_amd.splat_bwd(kind, params, *grids, packed, col, out, den, out, 1e-6, True)
        assert [t.shape for t in g] == [p.shape for p in params] + [grids[0].shape, grids[1].shape]
        assert len(torch.ops.igs_amd.splat_bwd(kind, params, *grids, packed, col, out, den, out, 1e-6, False)) == len(params)
    with pytest.raises(ValueError):
        torch.ops.igs_amd.splat_fwd(_splat.KIND_SCALE_ROT, [m(B, N, 2), m(B, N, C), m(B, N, 3), m(B, N), m(B, N)],
                                    *grids, 1e-6)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; with --gpus above 1 it exits with a message instead of running."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_bench_counter_constants_belong_to_the_current_kernel_sources():
    """bench.py derives `executed_frac` and `traffic` from per-launch counter readings stored in the file, and only
    while the kernel sources are the ones those readings were taken from: the stored hash is the current one (a
    kernel change that leaves it behind would make the bench line report null for those fields)."""
    import importlib.util
    import os

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("igs_bench_module", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    assert bench.C1_PROFILE["csrc_sha16"] == bench.csrc_sha16()
    assert os.path.exists(os.path.join(root, bench.C1_PROFILE["source"]))
    for leg in ("fwd", "bwd"):
        assert bench.executed_flops(bench.C1_PROFILE[leg]) > 0 and bench.hbm_bytes(bench.C1_PROFILE[leg]) > 0


def test_plan_invariants_over_random_shapes(lib):
    """igs_gs2d_plan over a few hundred seeded random shapes (tiny to large, square to extreme
    aspect ratios): every size positive and consistent, tiles cover the image, splits cover N."""
    import random

    from igs_amd import _lib

    rng = random.Random(1234)
    dims = [1, 2, 3, 7, 8, 9, 15, 16, 17, 31, 33, 63, 64, 65, 100, 127, 128, 129, 255, 256, 257, 384, 511, 640, 1000,
            2048, 4099]
    for _ in range(400):
        B = rng.choice([1, 2, 3, 8, 16, 33])
        N = rng.choice([1, 2, 3, 4, 5, 63, 64, 65, 100, 511, 512, 513, 2048, 8192, 32768, 100003])
        H, W = rng.choice(dims), rng.choice(dims)
        C = rng.choice(_lib.COMPILED_CHANNELS)
        if B * N > 1 << 24:
            continue
        for mode in (0, 1, 2):
            p = _lib.plan(B, N, H, W, C, mode)
            Np = p.n_padded
            assert Np % 4 == 0 and N <= Np < N + 4
            assert p.rec_stride % 4 == 0 and p.rec_stride >= 6 + C
            assert p.packed_bytes == (B * Np * (p.rec_stride + 8 + _sep_record_floats(C)) + 32) * 4
            assert 1 <= p.fwd_split <= 64 and p.fwd_n_per_split % 4 == 0
            assert p.fwd_split * p.fwd_n_per_split >= Np > (p.fwd_split - 1) * p.fwd_n_per_split
            assert p.bwd_tiles >= 1 and p.bwd_per_tile >= 1
            assert p.partial_bytes >= B * p.bwd_tiles * (6 + C) * N * 4
            if mode != 0:
                rows = p.bwd_tiles // p.bwd_tiles_x
                assert p.bwd_tiles == rows * p.bwd_tiles_x and rows * p.bwd_per_tile >= H > (rows - 1) * p.bwd_per_tile
                assert p.bwd_tiles_x * p.bwd_tile_w >= p.w_padded >= W and p.w_padded % 8 == 0
                assert p.fwd_tiles >= 1
                assert p.fwd_ws_bytes >= B * p.fwd_tiles * (Np + 1) * 4
                # pixel records and column coordinates, tile lists, slot tables, the tiles' record offsets
                assert p.pix_bytes >= ((B * H * p.w_padded * p.pix_stride + B * p.w_padded) * 4
                                       + B * p.bwd_tiles * (2 * Np + 1) * 4 + (B * p.bwd_tiles + 1) * 8)
                if mode == 1:    # a record for every (Gaussian, tile) pair (AUTO: the larger of the two variants')
                    assert p.partial_bytes == B * p.bwd_tiles * (6 + C) * N * 4
            else:
                assert p.hw_padded % 4 == 0 and p.bwd_tiles * p.bwd_per_tile >= p.hw_padded >= H * W


def test_header_is_valid_c_and_links_from_a_c_program(lib, tmp_path):
    """include/igs_hip.h compiled as C (gcc -std=c99 -pedantic -Wall -Werror) by a program that
    links the shared library and calls the plan entry point: the boundary is a C ABI, usable
    without C++ or Python."""
    import os
    import subprocess

    from igs_amd import _lib

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = str(tmp_path / "plan_from_c")
    libdir = os.path.dirname(_lib.LIB_PATH)
    subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-I", os.path.join(root, "include"),
                    os.path.join(root, "tests", "c_abi", "plan_from_c.c"), "-o", exe, "-L", libdir, "-ligs_hip",
                    "-Wl,-rpath," + libdir], check=True, capture_output=True, text=True, timeout=120)
    r = subprocess.run([exe], check=True, capture_output=True, text=True, timeout=60)
    first, second = r.stdout.strip().splitlines()
    p = _lib.plan(16, 8192, 256, 256, 3, _lib.IGS_GRID_SEPARABLE)
    assert [int(v) for v in first.split()] == [_lib.ABI_VERSION, p.n_padded, p.rec_stride, p.bwd_tiles, p.packed_bytes,
                                               p.fwd_ws_bytes, p.pix_bytes, p.partial_bytes]
    assert second.startswith("-2 ")


def test_empty_inputs_give_the_plain_expression_s_result():
    """No Gaussians, no images or no pixels: zeros / empty of the right shape, zero gradients --
    what the plain expression (fused=False) gives; nothing is launched, so this runs anywhere."""
    import torch

    import igs_amd

    z = lambda *s: torch.zeros(*s, requires_grad=True)
    for (B, N, H, W, C) in [(2, 0, 4, 5, 3), (0, 7, 4, 5, 3), (1, 7, 0, 5, 2), (1, 7, 4, 0, 1)]:
        p, c, s, r, a = z(B, N, 2), z(B, N, C), torch.ones(B, N, 2), torch.zeros(B, N), torch.ones(B, N)
        x, y = torch.zeros(B, 1, H, W), torch.zeros(B, 1, H, W)
        out = igs_amd.gaussian_splatting_2d(p, c, s, r, a, x, y)
        assert out.shape == (B, C, H, W) and float(out.detach().abs().sum()) == 0.0
        if B and H and W:
            want = igs_amd.gaussian_splatting_2d(p, c, s, r, a, x, y, fused=False)
            assert torch.equal(out, want)
        out.sum().backward()
        assert p.grad.shape == p.shape and c.grad.shape == c.shape and float(c.grad.abs().sum()) == 0.0
        cov = torch.ones(B, N, 1, 1)
        assert igs_amd.GaussianSplatting2DKernel.apply(x, y, p, cov, cov * 0, cov, a, c).shape == (B, C, H, W)
    m = igs_amd.GaussianSplatting2D(4, 8)
    img, feat = m(torch.zeros(2, 0, 8), size=(4, 6))       # no features -> no Gaussians
    assert img.shape == (2, 3, 4, 6) and feat.shape == (2, 0, 9) and float(img.detach().abs().sum()) == 0.0


def test_koleo_plan_and_argument_errors(lib):
    """Plan arithmetic of the diversity loss and its status codes (no GPU call is made)."""
    from igs_amd import _lib
    from igs_amd.reg import saved_numel

    import random
    rnd = random.Random(3)
    for _ in range(200):
        B, N, D = rnd.randint(1, 9), rnd.randint(2, 70000), rnd.randint(1, 600)
        if B * N * ((D + 3) // 4 * 4) > 1 << 31:
            continue
        p = _lib.KoleoPlan()
        assert lib.igs_koleo_plan(B, N, D, ctypes.byref(p)) == 0
        assert (p.B, p.N, p.D) == (B, N, D) and p.d_padded == (D + 3) // 4 * 4
        if p.d_padded <= 64:      # matrix-core kernel: 128 queries per workgroup, candidate tiles of 32
            assert (p.tile_rows, p.tile) == (128, 32)
        else:
            assert (p.tile_rows, p.tile) in ((128, 64), (64, 64), (32, 32))
        tiles = -(-N // p.tile)
        assert 1 <= p.splits <= tiles and p.splits * p.tiles_per_split >= tiles
        assert (p.splits - 1) * p.tiles_per_split < tiles            # no empty split
        assert p.saved_bytes == 4 * saved_numel(B, N, D)
        assert p.scratch_bytes >= 8 * -(-B * N // 256) + 8 * B * p.splits * N
        assert 1 <= p.bwd_rows <= 64 and p.bwd_chunk % 4 == 0 and p.bwd_chunk <= 2048
        assert p.bwd_rows * p.bwd_chunk <= 8192
    p = _lib.KoleoPlan()
    assert lib.igs_koleo_plan(1, 1, 3, ctypes.byref(p)) == -2          # N >= 2
    assert lib.igs_koleo_plan(0, 5, 3, ctypes.byref(p)) == -2
    assert lib.igs_koleo_plan(1, 5, 0, ctypes.byref(p)) == -2
    assert lib.igs_koleo_plan(70000, 5, 3, ctypes.byref(p)) == -2
    assert lib.igs_koleo_plan(1, 5, 3, None) == -1
    assert lib.igs_koleo_forward(None, 1, 5, 3, None, None, 0, None, 0, None) == -1
    assert lib.igs_koleo_backward(None, 0, None, 1, 5, 3, None, None) == -1
    # workspace too small / misaligned are reported before anything is launched
    fake = ctypes.c_void_p(4096)
    assert lib.igs_koleo_forward(fake, 1, 5, 3, fake, fake, 8, fake, 8, None) == -4
    assert lib.igs_koleo_forward(fake, 1, 5, 3, fake, ctypes.c_void_p(4100), 1 << 20, fake, 1 << 20, None) == -7
    assert lib.igs_koleo_backward(fake, 8, fake, 1, 5, 3, fake, None) == -4


def test_koleo_host_surface():
    import torch

    import igs_amd

    assert float(igs_amd.koleo_diversity_loss(torch.randn(3, 1, 4))) == 0.0     # N <= 1: constant 0
    assert float(igs_amd.koleo_diversity_loss(torch.randn(3, 0, 4))) == 0.0
    with pytest.raises(RuntimeError):
        igs_amd.koleo_diversity_loss(torch.randn(2, 5, 3))                      # no CPU path
    with pytest.raises(ValueError):
        igs_amd.koleo_diversity_loss(torch.randn(5, 3))
    out = torch.ops.igs_amd.koleo_fwd(torch.empty(2, 50, 9, device="meta"))
    assert out[0].shape == () and out[1].shape == (igs_amd.reg.saved_numel(2, 50, 9),)
    assert torch.ops.igs_amd.koleo_bwd(out[1], out[0], 2, 50, 9).shape == (2, 50, 9)


def test_library_options_are_per_thread():
    """`library_options` / `exact` change what the calling thread's renders may skip, not another thread's
    (nor what the same thread does after the block)."""
    import threading

    import igs_amd
    from igs_amd import _lib, _splat

    default = (0, _splat.SKIP_TOLERANCE)
    assert _splat._options.get() == default
    seen = []
    with igs_amd.exact():
        assert _splat._options.get() == (0, 0.0)
        with igs_amd.library_options(no_cull=True):   # nested contexts add up
            assert _splat._options.get() == (_lib.IGS_OPT_NO_CULL, 0.0)
            t = threading.Thread(target=lambda: seen.append(_splat._options.get()))
            t.start()
            t.join()
        assert _splat._options.get() == (0, 0.0)
    assert seen == [default] and _splat._options.get() == default
    with pytest.raises(ValueError):
        with igs_amd.library_options(skip_tolerance=1.5):
            pass
