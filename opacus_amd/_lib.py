"""ctypes binding of ``libdpsgd_hip.so`` (the C ABI declared in ``include/dpk.h``).

The library is loaded from ``opacus_amd/lib`` where ``python -m opacus_amd.build``
put it. There is no fallback: if it is missing, :func:`lib` raises, and so does
every kernel wrapper built on it.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_uint64, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libdpsgd_hip.so"

ABI_VERSION = 3

DPK_OK = 0
DPK_F32 = 0
DPK_BF16 = 1
DPK_MULTI_MAX = 48
DPK_TILE_AUTO, DPK_TILE_128, DPK_TILE_256 = 0, 128, 256
DPK_ROUTE_AUTO, DPK_ROUTE_GRAM, DPK_ROUTE_DIRECT = 0, 1, 2
DPK_STATIC_SCRATCH_BYTES = 8 << 20
DPK_GHOST_MULTI_MAX = 256


class GhostLayer(ctypes.Structure):
    """``dpk_ghost_layer`` of include/dpk.h."""

    _fields_ = [
        ("b", c_void_p), ("a", c_void_p), ("norm_w", c_void_p), ("norm_b", c_void_p),
        ("T", c_int64), ("out", c_int64), ("inp", c_int64), ("scale", c_float),
    ]

class WsumLayer(ctypes.Structure):
    """``dpk_wsum_layer`` of include/dpk.h."""

    _fields_ = [
        ("b", c_void_p), ("a", c_void_p), ("coef", c_void_p), ("out_sum", c_void_p),
        ("n", c_int64), ("T", c_int64), ("out", c_int64), ("inp", c_int64), ("scale", c_float),
    ]


STATUS_NAMES = {
    0: "DPK_OK",
    -1: "DPK_E_SHAPE",
    -2: "DPK_E_DTYPE",
    -3: "DPK_E_ALIGN",
    -4: "DPK_E_LAUNCH",
    -5: "DPK_E_WORKSPACE",
    -6: "DPK_E_ARG",
}

_P = c_void_p
_I = c_int64

# name -> (restype, argtypes); one row per declaration in include/dpk.h
SIGNATURES = {
    "dpk_abi_version": (c_int, []),
    "dpk_last_error": (c_char_p, []),
    "dpk_device_cus": (c_int, []),
    "dpk_linear_gs_workspace_bytes": (c_size_t, [_I, _I, _I, _I]),
    "dpk_linear_gs": (c_int, [_P, _P, c_int, _P, c_int, _P, _I, _I, _I, _I, c_float, c_int, _P, c_size_t, _P]),
    "dpk_linear_weighted_sum_workspace_bytes": (c_size_t, [_I, _I, _I, _I, c_int, c_int]),
    "dpk_linear_bias_weighted_sum_workspace_bytes": (c_size_t, [_I, _I, _I]),
    "dpk_linear_bias_weighted_sum": (c_int, [_P, c_int, _P, _P, c_int, _I, _I, _I, c_float, _P, c_size_t, _P]),
    "dpk_embedding_weighted_sum_workspace_bytes": (c_size_t, [_I, _I, _I]),
    "dpk_embedding_weighted_sum": (
        c_int, [_P, _P, c_int, _P, _P, c_int, _I, _I, _I, _I, c_float, _P, _P, c_size_t, _P]
    ),
    "dpk_linear_weighted_sum": (
        c_int, [_P, _P, c_int, _P, _P, c_int, _I, _I, _I, _I, c_float, c_int, _P, c_size_t, _P]
    ),
    "dpk_linear_weighted_sum_multi_workspace_bytes": (c_size_t, [_P, c_int]),
    "dpk_linear_weighted_sum_multi": (c_int, [_P, c_int, c_int, c_int, _P, c_size_t, _P]),
    "dpk_linear_bias_gs": (c_int, [_P, c_int, _P, c_int, _P, _I, _I, _I, c_float, _P]),
    "dpk_linear_ghost_norm_workspace_bytes": (c_size_t, [_I, _I, _I, _I]),
    "dpk_linear_ghost_norm": (c_int, [_P, _P, c_int, _P, _P, _I, _I, _I, _I, c_float, c_int, _P, c_size_t, _P]),
    "dpk_linear_ghost_norm_multi_workspace_bytes": (c_size_t, [_P, c_int, _I]),
    "dpk_linear_ghost_norm_multi": (c_int, [_P, c_int, c_int, _I, _P, c_size_t, _P]),
    "dpk_linear_ghost_norm_static": (c_int, [_P, _P, c_int, _P, _P, _I, _I, _I, _I, c_float, c_int, _P]),
    "dpk_conv2d_gs_workspace_bytes": (c_size_t, [_I, _I, _I, _I, _I, _I, _I]),
    "dpk_conv2d_gs": (
        c_int,
        [_P, _P, c_int, _P, c_int, _P] + [_I] * 16 + [c_float, _P, c_size_t, _P],
    ),
    "dpk_conv3d_gs_workspace_bytes": (c_size_t, [_I, _I, _I, _I, _I, _I, _I, _I]),
    "dpk_conv3d_gs": (
        c_int,
        [_P, _P, c_int, _P, c_int, _P, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _I, c_float, _P, c_size_t, _P],
    ),
    "dpk_conv_bias_gs": (c_int, [_P, c_int, _P, c_int, _P, _I, _I, _I, c_float, _P]),
    "dpk_embedding_workspace_bytes": (c_size_t, [_I, _I, _I]),
    "dpk_embedding_unique_pairs": (c_int, [_P, _I, _I, _P, _P, _P, _P, c_size_t, _P]),
    "dpk_embedding_gs": (c_int, [_P, _P, c_int, _P, c_int, _I, _I, _I, _I, c_float, _P, _P, c_size_t, _P]),
    "dpk_embedding_bag_gs": (
        c_int,
        [_P, _P, _P, c_int, _P, c_int, _I, _I, _I, _I, c_int, c_float, _P, _P],
    ),
    "dpk_embedding_ghost_norm": (c_int, [_P, _P, c_int, _P, _I, _I, _I, c_float, _P, c_size_t, _P]),
    "dpk_tied_embedding_cross_workspace_bytes": (c_size_t, [_I, _I, _I, _I, c_int]),
    "dpk_tied_embedding_cross": (
        c_int,
        [_P, _P, c_int, _P, _P, c_int, _P, _I, _I, _I, _I, _I, c_float, _P, c_size_t, _P],
    ),
    "dpk_group_norm_gs": (c_int, [_P, _P, c_int, _P, _P, c_int, _P, _P, _I, _I, _I, _I, c_float, c_float, _P]),
    "dpk_rms_norm_gs_workspace_bytes": (c_size_t, [_I, _I, _I]),
    "dpk_rms_norm_gs": (c_int, [_P, _P, c_int, _P, c_int, _P, _I, _I, _I, c_float, c_float, _P, c_size_t, _P]),
    "dpk_layer_norm_gs_workspace_bytes": (c_size_t, [_I, _I, _I]),
    "dpk_layer_norm_gs": (
        c_int,
        [_P, _P, c_int, _P, _P, c_int, _P, _P, _I, _I, _I, c_float, c_float, _P, c_size_t, _P],
    ),
    "dpk_sumsq_rows_workspace_bytes": (c_size_t, [_I, _I]),
    "dpk_sumsq_rows": (c_int, [_P, c_int, _I, _I, _P, _P, c_size_t, _P]),
    "dpk_clip_factor": (c_int, [_P, _I, _I, c_int, c_float, _P, _P, _P]),
    "dpk_clip_accumulate": (c_int, [_P, c_int, _P, _P, c_int, _I, _I, c_int, _P]),
    "dpk_sumsq_rows_multi_workspace_bytes": (c_size_t, [_I, _P, _I]),
    "dpk_sumsq_rows_multi": (c_int, [_P, _P, _I, c_int, _I, _P, _P, c_size_t, _P]),
    "dpk_clip_accumulate_multi": (c_int, [_P, _P, _P, _I, c_int, c_int, _P, _I, c_int, _P]),
    "dpk_add_noise": (c_int, [_P, c_int, _P, c_int, _I, c_float, c_float, c_uint64, c_uint64, c_int, _P]),
    "dpk_clip_factor_per_layer": (c_int, [_P, _I, _I, c_int, _P, _P, _P]),
    "dpk_clip_accumulate_per_layer": (c_int, [_P, _P, _P, _I, c_int, c_int, _P, _I, c_int, _P]),
    "dpk_clip_noise_step": (
        c_int, [_P, _P, _P, _P, _P, _I, c_int, c_int, _I, c_float, c_float, c_float, c_uint64, c_uint64, c_int, _P]
    ),
    "dpk_add_noise_multi": (
        c_int,
        [_P, _P, _P, _I, c_int, c_int, c_float, c_float, c_uint64, c_uint64, c_int, _P],
    ),
    "dpk_fill_normal": (c_int, [_P, _I, c_float, c_uint64, c_uint64, _P]),
}


class DpkError(RuntimeError):
    """A dpk_* entry point returned a negative status."""

    def __init__(self, fn: str, status: int, message: str):
        self.fn = fn
        self.status = status
        super().__init__(f"{fn} failed with {STATUS_NAMES.get(status, status)}: {message}")


_LIB = None


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built or does not match this binding."""
    global _LIB
    if _LIB is not None:
        return _LIB
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP kernels are not built. Run `python -m opacus_amd.build` "
            "(needs hipcc, no GPU). There is no CPU fallback."
        )
    handle = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(handle, name)  # AttributeError names the missing symbol
        fn.restype = restype
        fn.argtypes = argtypes
    if handle.dpk_abi_version() != ABI_VERSION:
        raise RuntimeError(
            f"{LIB_PATH} has ABI {handle.dpk_abi_version()}, this package expects {ABI_VERSION}: rebuild it"
        )
    _LIB = handle
    return _LIB


def check(fn: str, status: int) -> None:
    if status != DPK_OK:
        raise DpkError(fn, status, lib().dpk_last_error().decode("utf-8", "replace"))
