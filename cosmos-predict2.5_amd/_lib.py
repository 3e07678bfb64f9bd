"""ctypes binding of ``libcosmos_attn_hip.so`` (declarations: ``include/cosmos_attn_hip.h``).

There is no fallback: if the library is missing or its ABI version differs, importing the
operators raises.  ``import torch`` must happen before the library is loaded so that both use the
one HIP runtime already in the process (this module imports torch first for that reason).
"""
from __future__ import annotations

import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime the library binds to)

from .build import LIB_PATH as _BUILT_LIB_PATH

# COSMOS_ATTN_LIB: load another build of the same ABI instead of the in-tree one (deployments, A/B timing)
LIB_PATH = os.environ.get("COSMOS_ATTN_LIB") or _BUILT_LIB_PATH

ABI_VERSION = 2
DTYPE_BF16, DTYPE_FP16 = 0, 1

ST_OK, ST_BAD_ARG, ST_BAD_SHAPE, ST_BAD_STRIDE, ST_UNSUPPORTED, ST_WORKSPACE, ST_LAUNCH, ST_STATIC_SCRATCH, ST_WRONG_DEVICE = range(9)


class AttnDesc(ctypes.Structure):
    """Mirror of ``struct cosmos_attn_desc``."""

    _fields_ = [
        ("abi_version", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("B", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("Lq", ctypes.c_int32),
        ("Lkv", ctypes.c_int32),
        ("d_qk", ctypes.c_int32),
        ("d_v", ctypes.c_int32),
        ("causal", ctypes.c_int32),
        ("sm_scale", ctypes.c_float),
        ("q", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("tq", ctypes.c_void_p),
        ("tk", ctypes.c_void_p),
        ("tv", ctypes.c_void_p),
        ("q_stride", ctypes.c_int64 * 3),
        ("k_stride", ctypes.c_int64 * 3),
        ("v_stride", ctypes.c_int64 * 3),
        ("o", ctypes.c_void_p),
        ("to", ctypes.c_void_p),
        ("o_stride", ctypes.c_int64 * 3),
        ("lse", ctypes.c_void_p),
        ("key_lens", ctypes.c_void_p),
    ]


class AttnBwdDesc(ctypes.Structure):
    """Mirror of ``struct cosmos_attn_bwd_desc``."""

    _fields_ = [
        ("abi_version", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("B", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("Lq", ctypes.c_int32),
        ("Lkv", ctypes.c_int32),
        ("d", ctypes.c_int32),
        ("causal", ctypes.c_int32),
        ("sm_scale", ctypes.c_float),
        ("max_ds_mib", ctypes.c_int32),
        ("q", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("o", ctypes.c_void_p),
        ("dout", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("dq", ctypes.c_void_p),
        ("dk", ctypes.c_void_p),
        ("dv", ctypes.c_void_p),
        ("q_stride", ctypes.c_int64 * 3),
        ("k_stride", ctypes.c_int64 * 3),
        ("v_stride", ctypes.c_int64 * 3),
        ("o_stride", ctypes.c_int64 * 3),
        ("dout_stride", ctypes.c_int64 * 3),
        ("dq_stride", ctypes.c_int64 * 3),
        ("dk_stride", ctypes.c_int64 * 3),
        ("dv_stride", ctypes.c_int64 * 3),
    ]


class NormRopeDesc(ctypes.Structure):
    """Mirror of ``struct cosmos_norm_rope_desc``."""

    _fields_ = [
        ("abi_version", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("B", ctypes.c_int32),
        ("S", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("eps", ctypes.c_float),
        ("reserved", ctypes.c_int32),
        ("x", ctypes.c_void_p),
        ("tx", ctypes.c_void_p),
        ("weight", ctypes.c_void_p),
        ("angles", ctypes.c_void_p),
        ("y", ctypes.c_void_p),
        ("ty", ctypes.c_void_p),
        ("x_stride", ctypes.c_int64 * 3),
        ("y_stride", ctypes.c_int64 * 3),
    ]


class NormRopeBwdDesc(ctypes.Structure):
    """Mirror of ``struct cosmos_norm_rope_bwd_desc``."""

    _fields_ = [
        ("abi_version", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("B", ctypes.c_int32),
        ("S", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("eps", ctypes.c_float),
        ("reserved", ctypes.c_int32),
        ("x", ctypes.c_void_p),
        ("dy", ctypes.c_void_p),
        ("weight", ctypes.c_void_p),
        ("angles", ctypes.c_void_p),
        ("dx", ctypes.c_void_p),
        ("dweight", ctypes.c_void_p),
        ("x_stride", ctypes.c_int64 * 3),
        ("dy_stride", ctypes.c_int64 * 3),
        ("dx_stride", ctypes.c_int64 * 3),
    ]


class LnModulateDesc(ctypes.Structure):
    """Mirror of ``struct cosmos_ln_modulate_desc``."""

    _fields_ = [
        ("abi_version", ctypes.c_int32), ("dtype", ctypes.c_int32),
        ("D", ctypes.c_int32), ("rows_per_group", ctypes.c_int32),
        ("eps", ctypes.c_float), ("reserved", ctypes.c_int32),
        ("rows", ctypes.c_int64),
        ("x", ctypes.c_void_p), ("tx", ctypes.c_void_p),
        ("shift", ctypes.c_void_p), ("scale", ctypes.c_void_p),
        ("tshift", ctypes.c_void_p), ("tscale", ctypes.c_void_p),
        ("y", ctypes.c_void_p), ("ty", ctypes.c_void_p),
    ]


class GatedResidualDesc(ctypes.Structure):
    """Mirror of ``struct cosmos_gated_residual_desc``."""

    _fields_ = [
        ("abi_version", ctypes.c_int32), ("dtype", ctypes.c_int32),
        ("D", ctypes.c_int32), ("rows_per_group", ctypes.c_int32),
        ("rows", ctypes.c_int64),
        ("x", ctypes.c_void_p), ("tx", ctypes.c_void_p), ("res", ctypes.c_void_p), ("tres", ctypes.c_void_p),
        ("gate", ctypes.c_void_p), ("tgate", ctypes.c_void_p),
        ("out", ctypes.c_void_p), ("tout", ctypes.c_void_p),
    ]


class GeluDesc(ctypes.Structure):
    """Mirror of ``struct cosmos_gelu_desc``."""

    _fields_ = [
        ("abi_version", ctypes.c_int32), ("dtype", ctypes.c_int32),
        ("n", ctypes.c_int64),
        ("h", ctypes.c_void_p), ("th", ctypes.c_void_p), ("a", ctypes.c_void_p), ("ta", ctypes.c_void_p),
    ]


EXPORTS = {
    "cosmos_attn_abi_version": (ctypes.c_int, []),
    "cosmos_attn_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "cosmos_attn_set_stream_override": (None, [ctypes.c_int, ctypes.c_int]),
    "cosmos_attn_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(AttnDesc)]),
    "cosmos_attn_fwd_jvp": (ctypes.c_int, [ctypes.POINTER(AttnDesc), ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "cosmos_attn_static_scratch_bytes": (ctypes.c_size_t, []),
    "cosmos_attn_fwd_jvp_static": (ctypes.c_int, [ctypes.POINTER(AttnDesc), ctypes.c_void_p]),
    "cosmos_attn_packed_bytes": (ctypes.c_size_t, [ctypes.POINTER(AttnDesc)]),
    "cosmos_attn_pack_kv": (ctypes.c_int, [ctypes.POINTER(AttnDesc), ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "cosmos_attn_run": (ctypes.c_int, [ctypes.POINTER(AttnDesc), ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "cosmos_attn_bwd_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(AttnBwdDesc)]),
    "cosmos_attn_bwd": (ctypes.c_int, [ctypes.POINTER(AttnBwdDesc), ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "cosmos_norm_rope": (ctypes.c_int, [ctypes.POINTER(NormRopeDesc), ctypes.c_void_p]),
    "cosmos_norm_rope_bwd_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(NormRopeBwdDesc)]),
    "cosmos_norm_rope_bwd": (ctypes.c_int, [ctypes.POINTER(NormRopeBwdDesc), ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "cosmos_ln_modulate": (ctypes.c_int, [ctypes.POINTER(LnModulateDesc), ctypes.c_void_p]),
    "cosmos_gated_residual": (ctypes.c_int, [ctypes.POINTER(GatedResidualDesc), ctypes.c_void_p]),
    "cosmos_gelu": (ctypes.c_int, [ctypes.POINTER(GeluDesc), ctypes.c_void_p]),
}

_lib = None


def load_library() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP attention library has not been built "
            f"(run `python __graft_entry__.py build`). There is no fallback path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in EXPORTS.items():
        fn = getattr(lib, name)  # AttributeError if a declared symbol is not exported
        fn.restype, fn.argtypes = restype, argtypes
    got = lib.cosmos_attn_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH}: ABI version {got}, expected {ABI_VERSION}; rebuild the library")
    _lib = lib
    return lib


def status_string(status: int) -> str:
    return load_library().cosmos_attn_status_string(status).decode()


def raise_for_status(status: int) -> None:
    """Status code -> the exception type the reference raises for the same condition."""
    if status == ST_OK:
        return
    msg = f"cosmos_attn: {status_string(status)} (status {status})"
    if status in (ST_BAD_SHAPE, ST_BAD_STRIDE):
        raise AssertionError(msg)
    if status == ST_UNSUPPORTED:
        raise NotImplementedError(msg)
    if status == ST_BAD_ARG:
        raise ValueError(msg)
    raise RuntimeError(msg)
