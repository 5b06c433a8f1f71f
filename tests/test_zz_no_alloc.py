"""igs_gs2d_forward_static_ws (forward with its scratch in a static device array, no allocation)
against igs_gs2d_forward (caller-allocated workspace), through the C ABI: same kernels and plan, so
`out` and `den` must be bit-identical.  Two calls in a row, the second on a smaller problem (the
array keeps the first call's contents), then a problem that exceeds the array.  Needs an MI355X.
"""
import ctypes

import pytest
import torch

from oracle import gs2d_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


_set_up = False


def _both_forwards(dev, B, N, H, W, C, seed, general=False):
    from igs_amd import _lib
    from igs_amd._splat import Grid, Splat, _ptr, _stream

    lib = _lib.load()
    d = {k: v.to(dev) for k, v in O.make_inputs(B, N, H, W, C, 0.02, 0.3, seed=seed).items()}
    if general:
        g = torch.Generator().manual_seed(seed)
        xg = (torch.rand(B, 1, H, W, generator=g) * 2 - 1).to(dev)
        yg = (torch.rand(B, 1, H, W, generator=g) * 2 - 1).to(dev)
    else:
        xg = d["x_grid"][:1, :, :1, :].expand(B, 1, H, W)
        yg = d["y_grid"][:1, :, :, :1].expand(B, 1, H, W)
    with torch.cuda.device(dev):
        grid = Grid(xg, yg, B)
        op = Splat(B, N, C, grid, 1e-6, dev)
        packed = op.pack_scale_rot(d["positions"].contiguous(), d["scales"].contiguous(), d["rotations"].contiguous(),
                                   d["alphas"].contiguous(), d["colors"].contiguous())
        ref_out, ref_den = op.forward(packed)
        # outputs are allocated before the call; the call itself allocates nothing
        out = torch.full_like(ref_out, float("nan"))
        den = torch.full_like(ref_den, float("nan"))
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info(dev)[0]     # the device's own count: sees allocations made past torch
        rc = lib.igs_gs2d_forward_static_ws(_ptr(packed), _ptr(grid.x), _ptr(grid.y), grid.strides, grid.mode,
                                            _ptr(grid.flag), B, N, H, W, op.Cp, 1e-6, _ptr(out), _ptr(den),
                                            _stream(dev))
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before
        # (the first call on a device resolves the array's address and creates the guard's event: set-up, not
        # checked; every later call must leave the device's free memory where it was)
        global _set_up
        if _set_up:
            assert torch.cuda.mem_get_info(dev)[0] >= free_before
        _set_up = True
    return rc, op.plan, (out, den), (ref_out, ref_den)


def test_static_scratch_forward_equals_workspace_forward_twice_then_smaller(dev):
    from igs_amd import _lib

    # first call: several Gaussian splits (split partials + tile lists in the scratch), 32 MiB of it
    rc, plan, got, ref = _both_forwards(dev, 1, 2048, 256, 256, 3, seed=5)
    assert rc == 0 and plan.fwd_split > 1
    assert 16 << 20 < plan.fwd_ws_bytes <= _lib.IGS_STATIC_SCRATCH_BYTES
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    assert bool(torch.isfinite(got[0]).all())
    # second call, smaller problem with other tile counts: stale lists / partials of the first call
    # lie behind and between the regions this one uses
    rc, plan, got, ref = _both_forwards(dev, 2, 300, 40, 72, 3, seed=6)
    assert rc == 0
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    # third: general (per-pixel) grids through the same entry point
    rc, plan, got, ref = _both_forwards(dev, 1, 500, 33, 47, 4, seed=7, general=True)
    assert rc == 0
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])


def test_static_scratch_forward_rejects_what_does_not_fit(dev):
    from igs_amd import _lib

    lib = _lib.load()
    p = _lib.plan(16, 8192, 256, 256, 3, _lib.IGS_GRID_SEPARABLE)
    assert p.fwd_ws_bytes > _lib.IGS_STATIC_SCRATCH_BYTES
    one = torch.zeros(64, device=dev)
    strides = (ctypes.c_int64 * 6)(0, 0, 1, 0, 1, 0)
    ptr = ctypes.c_void_p(one.data_ptr())
    rc = lib.igs_gs2d_forward_static_ws(ptr, ptr, ptr, strides, _lib.IGS_GRID_SEPARABLE, None, 16, 8192, 256, 256, 3,
                                        1e-6, ptr, ptr, None)
    assert rc == -8
    assert b"static" in lib.igs_status_string(rc)


def test_static_scratch_forward_refuses_an_overlapping_call_on_another_stream(dev):
    """One array per GPU: a call on another stream than the previous one, while that one's work is
    still running, gets a status instead of the array; on the same stream, or once the work is done,
    calls go through."""
    from igs_amd import _lib
    from igs_amd._splat import Grid, Splat, _ptr

    lib = _lib.load()
    B, N, H, W, C = 1, 512, 64, 64, 3
    d = {k: v.to(dev, torch.float32) for k, v in O.make_config_inputs("c1", B=B, N=N, H=H, W=W).items()}
    xg = d["x_grid"][:1, :, :1, :].expand(B, 1, H, W)
    yg = d["y_grid"][:1, :, :, :1].expand(B, 1, H, W)
    with torch.cuda.device(dev):
        grid = Grid(xg, yg, B)
        op = Splat(B, N, C, grid, 1e-6, dev)
        packed = op.pack_scale_rot(d["positions"].contiguous(), d["scales"].contiguous(), d["rotations"].contiguous(),
                                   d["alphas"].contiguous(), d["colors"].contiguous())
        ref_out, _ = op.forward(packed)
        out, den = torch.empty_like(ref_out), op._new(B, H, W)
        s1, s2 = torch.cuda.Stream(dev), torch.cuda.Stream(dev)
        torch.cuda.synchronize()

        def call(stream):
            return lib.igs_gs2d_forward_static_ws(_ptr(packed), _ptr(grid.x), _ptr(grid.y), grid.strides, grid.mode,
                                                  _ptr(grid.flag), B, N, H, W, op.Cp, 1e-6, _ptr(out), _ptr(den),
                                                  stream.cuda_stream)

        with torch.cuda.stream(s1):
            torch.cuda._sleep(200_000_000)      # keeps s1 busy for a fraction of a second: the call behind it cannot have finished
        assert call(s1) == 0
        assert call(s1) == 0                    # the same stream: ordered, never refused
        rc = call(s2)
        assert rc == -10 and b"still in use" in lib.igs_status_string(rc)
        torch.cuda.synchronize()
        assert call(s2) == 0                    # the earlier work is done
        torch.cuda.synchronize()
        assert torch.equal(out, ref_out)
