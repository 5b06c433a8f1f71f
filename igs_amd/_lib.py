"""ctypes binding of libigs_hip.so (the C ABI declared in include/igs_hip.h).

There is no fallback: if the shared library is missing or an entry point is absent the
import of the product path raises.  Build it with ``python -m igs_amd.build``.
"""
from __future__ import annotations

import ctypes
import functools
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_uint64, c_void_p

# IGS_HIP_LIBRARY overrides the in-tree location (e.g. to try a differently tuned build)
LIB_PATH = os.environ.get("IGS_HIP_LIBRARY") or os.path.join(os.path.dirname(os.path.abspath(__file__)),
                                                               "libigs_hip.so")

ABI_VERSION = 8  # IGS_ABI_VERSION of include/igs_hip.h this binding was written against
IGS_GRID_GENERAL = 0
IGS_GRID_SEPARABLE = 1
IGS_GRID_AUTO = 2
IGS_OPT_NO_CULL = 0x100
IGS_OPT_BIN_LEVELS_1 = 0x200
IGS_OPT_BIN_LEVELS_2 = 0x400
IGS_OPT_LISTS_BUILT = 0x800
IGS_MAX_CHANNELS = 16
IGS_STATIC_SCRATCH_BYTES = 64 << 20
COMPILED_CHANNELS = (1, 2, 3, 4, 8, 16)


class Plan(ctypes.Structure):
    """Mirror of igs_gs2d_plan_t."""

    _fields_ = [
        ("B", c_int32), ("N", c_int32), ("H", c_int32), ("W", c_int32), ("C", c_int32),
        ("rec_stride", c_int32),
        ("n_padded", c_int32),
        ("w_padded", c_int32),
        ("hw_padded", c_int32),
        ("fwd_split", c_int32),
        ("fwd_n_per_split", c_int32),
        ("bwd_tiles", c_int32),
        ("bwd_per_tile", c_int32),
        ("pix_stride", c_int32),
        ("packed_bytes", c_uint64),
        ("fwd_ws_bytes", c_uint64),
        ("pix_bytes", c_uint64),
        ("partial_bytes", c_uint64),
        ("fwd_tiles", c_int32),
        ("bwd_tiles_x", c_int32),
        ("bwd_tile_w", c_int32),
        ("lists_shared", c_int32),
    ]


class KoleoPlan(ctypes.Structure):
    """Mirror of igs_koleo_plan_t."""

    _fields_ = [
        ("B", c_int32), ("N", c_int32), ("D", c_int32),
        ("d_padded", c_int32),
        ("tile_rows", c_int32),
        ("tile", c_int32),
        ("splits", c_int32),
        ("tiles_per_split", c_int32),
        ("bwd_rows", c_int32),
        ("bwd_chunk", c_int32),
        ("saved_bytes", c_uint64),
        ("scratch_bytes", c_uint64),
    ]


_FP = c_void_p  # device pointers travel as plain addresses
_STRIDES = POINTER(c_int64)

# name -> (restype, argtypes); must list every symbol include/igs_hip.h declares
SIGNATURES = {
    "igs_abi_version": (c_int, []),
    "igs_status_string": (c_char_p, [c_int]),
    "igs_gs2d_plan": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int, POINTER(Plan)]),
    "igs_gs2d_skip_weight": (c_float, [c_int, c_float, c_float]),
    "igs_gs2d_pack_covinv": (c_int, [_FP, _FP, _FP, _FP, _FP, _FP, c_int, c_int, c_int, c_float, c_float, _FP,
                                     c_void_p]),
    "igs_gs2d_pack_scale_rot": (c_int, [_FP, _FP, _FP, _FP, _FP, c_int, c_int, c_int, c_float, c_float, c_float,
                                        _FP, c_void_p]),
    "igs_gs2d_grid_classify": (c_int, [_FP, _FP, _STRIDES, c_int, c_int, c_int, _FP, c_void_p]),
    "igs_gs2d_forward": (c_int, [_FP, _FP, _FP, _STRIDES, c_int, _FP, c_int, c_int, c_int, c_int, c_int,
                                 c_float, _FP, _FP, c_void_p, c_size_t, c_void_p]),
    "igs_gs2d_forward_train": (c_int, [_FP, _FP, _FP, _STRIDES, c_int, _FP, c_int, c_int, c_int, c_int, c_int,
                                       c_float, _FP, _FP, c_void_p, c_size_t, _FP, c_size_t, _FP, c_void_p]),
    "igs_gs2d_forward_static_ws": (c_int, [_FP, _FP, _FP, _STRIDES, c_int, _FP, c_int, c_int, c_int, c_int, c_int,
                                           c_float, _FP, _FP, c_void_p]),
    "igs_gs2d_backward_prologue": (c_int, [_FP, _FP, _STRIDES, c_int, _FP, _FP, _FP, _FP, c_int, c_int, c_int,
                                           c_int, c_int, c_float, _FP, c_size_t, c_void_p]),
    "igs_gs2d_backward_reduce": (c_int, [_FP, _FP, _FP, _STRIDES, c_int, _FP, c_int, c_int, c_int, c_int, c_int,
                                         _FP, c_size_t, _FP, c_size_t, c_void_p]),
    "igs_gs2d_backward": (c_int, [_FP, _FP, _FP, _FP, _STRIDES, c_int, _FP, _FP, _FP, _FP, c_int, c_int,
                                  c_int, c_int, c_int, c_float, _FP, c_size_t, _FP, c_size_t, c_void_p]),
    "igs_gs2d_grid_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "igs_gs2d_backward_with_grid": (c_int, [_FP, _FP, _FP, _FP, _STRIDES, c_int, _FP, _FP, _FP, _FP, c_int, c_int,
                                            c_int, c_int, c_int, c_float, _FP, c_size_t, _FP, c_size_t, _FP,
                                            c_size_t, _FP, _FP, c_void_p]),
    "igs_gs2d_backward_grid": (c_int, [_FP, _FP, _FP, _STRIDES, _FP, _FP, _FP, c_int, c_int, c_int, c_int, c_int,
                                       c_float, _FP, _FP, c_void_p]),
    "igs_gs2d_finalize_covinv": (c_int, [_FP, _FP, c_int, _FP, _FP, _FP, _FP, _FP, c_int, c_int, c_int, c_int, c_int,
                                         _FP, _FP, _FP, _FP, _FP, _FP, c_void_p]),
    "igs_gs2d_finalize_scale_rot": (c_int, [_FP, _FP, c_int, _FP, _FP, _FP, _FP, c_int, c_int, c_int, c_int, c_int,
                                            c_float, _FP, _FP, _FP, _FP, _FP, c_void_p]),
    "igs_gs2d_pack_feature": (c_int, [_FP, _FP, c_int, c_int, c_int, c_int, c_float, c_float, c_float, _FP, _FP,
                                      c_void_p]),
    "igs_gs2d_finalize_feature": (c_int, [_FP, _FP, c_int, _FP, _FP, c_int, c_int, c_int, c_int, c_int, c_int, c_float,
                                          _FP, c_void_p]),
    "igs_gs2d_mse_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "igs_gs2d_backward_prologue_mse": (c_int, [_FP, _FP, _STRIDES, c_int, _FP, _FP, _FP, _FP, c_int, c_int, c_int,
                                               c_int, c_int, c_int, c_float, _FP, c_size_t, _FP, c_size_t, _FP,
                                               c_void_p]),
    "igs_gs2d_position_penalty": (c_int, [_FP, c_int64, c_int, c_float, c_int64, _FP, _FP, c_void_p]),
    "igs_adamw_step": (c_int, [_FP, _FP, _FP, _FP, c_int64, _FP, c_float, c_float, c_float, c_float, c_void_p]),
    "igs_koleo_plan": (c_int, [c_int, c_int, c_int, POINTER(KoleoPlan)]),
    "igs_koleo_forward": (c_int, [_FP, c_int, c_int, c_int, _FP, _FP, c_size_t, _FP, c_size_t, c_void_p]),
    "igs_koleo_backward": (c_int, [_FP, c_size_t, _FP, c_int, c_int, c_int, _FP, c_void_p]),
}

_lib = None


class IGSLibraryError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the shared library once and attach the signatures.  Raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise IGSLibraryError(
            f"{LIB_PATH} not found: build the HIP library first (python -m igs_amd.build). "
            "There is no CPU or PyTorch fallback for the fused path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise IGSLibraryError(f"{LIB_PATH} does not export {name}") from e
        fn.restype = res
        fn.argtypes = args
    if lib.igs_abi_version() != ABI_VERSION:
        raise IGSLibraryError(f"ABI version mismatch: library reports {lib.igs_abi_version()}, binding expects "
                              f"{ABI_VERSION}")
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().igs_status_string(status).decode()
        raise RuntimeError(f"{what} failed: {msg} (status {status})")


@functools.lru_cache(maxsize=256)
def plan(B: int, N: int, H: int, W: int, C: int, grid_mode: int) -> Plan:
    """Launch plan / buffer sizes of a problem (pure host arithmetic in the library; cached, since
    training loops ask for the same shape every step).  Treat the result as read-only."""
    p = Plan()
    check(load().igs_gs2d_plan(B, N, H, W, C, grid_mode, ctypes.byref(p)), "igs_gs2d_plan")
    return p


@functools.lru_cache(maxsize=64)
def koleo_plan(B: int, N: int, D: int) -> KoleoPlan:
    """Buffer sizes of the diversity loss for a [B, N, D] feature block (cached; read-only)."""
    p = KoleoPlan()
    check(load().igs_koleo_plan(B, N, D, ctypes.byref(p)), "igs_koleo_plan")
    return p


def strides6(sx, sy):
    return (c_int64 * 6)(*sx, *sy)
