"""ctypes binding of libcosmos_dm_hip.so (the C ABI declared in include/cosmos_dm.h).

The product path has no CPU fallback: if the library is missing it is built once with hipcc, and if
that fails, or a call returns a non-zero status, a RuntimeError is raised.

The product library has no process-wide state.  The cross-check build of the same sources
(libcosmos_dm_hip_crosscheck.so, -DCDM_CROSSCHECK) additionally carries the superseded kernels and
``cdm_set_variant``; ``set_variant`` loads it and, while some variant is selected, ``load()`` hands out that
library instead (tests and measurement aids only).
"""
from __future__ import annotations

import ctypes as C
import os
import threading

from . import build as _build

_LOCK = threading.Lock()
_LIB = None
_XLIB = None                               # the cross-check build, loaded on the first set_variant
_VARIANTS = {"attn": 0, "gemm": 0}         # what set_variant last selected

OK = 0
ERR_BAD_ARG, ERR_BAD_SHAPE, ERR_BAD_ALIGN, ERR_NO_DEVICE, ERR_LAUNCH, ERR_UNSUPPORTED = -1, -2, -3, -4, -5, -6
EPI_NONE, EPI_SWIGLU, EPI_GATE_RESIDUAL, EPI_ROPE_QK, EPI_GATE_RESIDUAL_F32 = 0, 1, 2, 3, 4

_P, _I64, _I32, _F32 = C.c_void_p, C.c_int64, C.c_int32, C.c_float

# name -> (restype, argtypes); mirrors include/cosmos_dm.h one to one
class QkNorm(C.Structure):
    """Mirror of ``cdm_qk_norm``: device weight tables [n_seg, head_dim] fp32, host segment ends, eps."""
    _fields_ = [("q_weight", C.c_void_p), ("k_weight", C.c_void_p), ("seg_end", C.POINTER(C.c_int64)),
                ("n_seg", C.c_int32), ("eps", C.c_float)]


SIGNATURES = {
    "cdm_version": (_I32, []),
    "cdm_last_error": (C.c_char_p, []),
    "cdm_source_hash": (C.c_char_p, []),
    "cdm_device_count": (_I32, []),
    "cdm_adaln_rmsnorm_bf16": (_I32, [_P, _P, _P, _P, _P, _I64, _I64, _F32, _P]),
    "cdm_adaln_rmsnorm_quant_e4m3": (_I32, [_P, _P, _P, _P, _P, _P, _I64, _I64, _F32, _P]),
    "cdm_adaln_rmsnorm_f32": (_I32, [_P, _P, _P, _P, _P, _I64, _I64, _F32, _P]),
    "cdm_adaln_rmsnorm_f32_quant_e4m3": (_I32, [_P, _P, _P, _P, _P, _P, _I64, _I64, _F32, _P]),
    "cdm_quant_rows_e4m3": (_I32, [_P, _I64, _P, _P, _I64, _I64, _P]),
    "cdm_quant_rows_from_parts_e4m3": (_I32, [_P, _I64, _P, _I64, _I64, _P, _P, _I64, _I64, _P]),
    "cdm_gemm_bf16": (_I32, [_P, _I64, _P, _I64, _P, _P, _I64, _I64, _I64, _I64, _I32, _P, _I64, _P, _P, _P, _I64,
                             _I32, _P]),
    "cdm_gemm_fp8": (_I32, [_P, _I64, _P, _P, _I64, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I32, _P, _I64, _P, _P,
                            _P, _I64, _I32, _P, _I64, _P]),
    "cdm_mrope_qk_bf16": (_I32, [_P, _I64, _P, _I64, _P, _P, _I64, _I32, _I32, _P]),
    "cdm_attn_workspace_bytes": (_I64, [_I64, _I32, _I32]),
    "cdm_attn_fwd_bf16": (_I32, [_P, _I64, _P, _I64, _P, _I64, _P, _P, _P, _I64, _I64, _I32, _I32, _I32, _P, _I64, _P, _I64,
                                 _P]),
    "cdm_attn_static_scratch_bytes": (_I64, []),
    "cdm_attn_fwd_static_bf16": (_I32, [_P, _I64, _P, _I64, _P, _I64, _P, _P, _P, _I64, _I64, _I32, _I32, _I32, _P, _I64, _P]),
    "cdm_attn_pack_kv_bf16": (_I32, [_P, _I64, _P, _I64, _P, _P, _P, _I64, _I64, _I32, _I32, _P, _P]),
    "cdm_attn_fwd_packed_bf16": (_I32, [_P, _I64, _P, _P, _P, _P, _I64, _I64, _I32, _I32, _I32, _P, _P, _I64, _I64, _P, _P,
                                        _I64, _P]),
    "cdm_attn_split_scratch_bytes": (_I64, [_I64, _I32, _I32]),
    "cdm_linear_bias_bf16": (_I32, [_P, _I64, _P, _I64, _P, _P, _I64, _I64, _I64, _I64, _P]),
    "cdm_grouped_gemm_fp8": (_I32, [_P, _I64, _P, C.POINTER(_P), C.POINTER(_P), _I64, C.POINTER(_P), C.POINTER(_P), _P, _I64,
                                    C.POINTER(_I64), C.POINTER(_I64), _I32, _I64, _I64, _I32, _P, _I64, C.POINTER(_P), _P,
                                    _P, _I64, _I32, _P, _I64, _P]),
    "cdm_cfg_step_f32": (_I32, [_P, _P, _P, _F32, C.POINTER(_P), _I32, C.POINTER(_F32), C.POINTER(_P), _I32, _I64, _P]),
    "cdm_grouped_gemm_qkv_pack_bf16": (_I32, [_P, _I64, C.POINTER(_P), _I64, _P, _I64, C.POINTER(_I64), C.POINTER(_I64), _I32,
                                              _I64, _I32, _I32, _I32, _P, _P, _P, _P, _I64, _P]),
    "cdm_grouped_gemm_qkv_pack_fp8": (_I32, [_P, _I64, _P, C.POINTER(_P), C.POINTER(_P), _I64, _P, _I64, C.POINTER(_I64),
                                             C.POINTER(_I64), _I32, _I64, _I32, _I32, _I32, _P, _P, _P, _P, _I64, _P]),
    "cdm_grouped_gemm_bf16": (_I32, [_P, _I64, C.POINTER(_P), _I64, C.POINTER(_P), _P, _I64, C.POINTER(_I64),
                                     C.POINTER(_I64), _I32, _I64, _I64, _I32, _P, _I64, C.POINTER(_P), _P, _P, _I64,
                                     _I32, _P]),
}


CROSSCHECK_SIGNATURES = {"cdm_set_variant": (_I32, [C.c_char_p, _I32])}      # exported by the cross-check build only


def lib_path() -> str:
    """Path of the shared library; COSMOS_DM_LIB overrides the in-tree build (e.g. an experimental build)."""
    return os.environ.get("COSMOS_DM_LIB") or _build.LIB_PATH


def _bind(path: str, signatures: dict):
    lib = C.CDLL(path)
    for name, (res, args) in signatures.items():
        fn = getattr(lib, name)     # AttributeError here = the library does not export the ABI
        fn.restype, fn.argtypes = res, args
    return lib


def _fresh(path: str) -> None:
    """Rebuild the in-tree libraries if `path` is missing or was built from other sources than the ones present."""
    want = _build.source_hash()
    if _build.built_hash(path) != want:
        _build.build(verbose=False, only_if_stale=True)
        if _build.built_hash(path) != want:
            raise RuntimeError(f"{path} does not carry the hash of the present sources after a rebuild")


def load():
    """Return the loaded library.  The in-tree build is (re)built first if it is missing or was built from other
    sources than the ones present (a stale build is never run); a library named by COSMOS_DM_LIB is taken as is.
    While ``set_variant`` has a non-default kernel selected this is the cross-check build."""
    global _LIB
    if _XLIB is not None and any(_VARIANTS.values()):
        return _XLIB
    with _LOCK:
        if _LIB is not None:
            return _LIB
        path = lib_path()
        if path == _build.LIB_PATH:
            _fresh(path)
        elif not os.path.exists(path):
            raise RuntimeError(f"COSMOS_DM_LIB={path} does not exist")
        _LIB = _bind(path, SIGNATURES)
        return _LIB


def load_crosscheck():
    """The cross-check build (default kernels + their predecessors + ``cdm_set_variant``)."""
    global _XLIB
    with _LOCK:
        if _XLIB is None:
            _fresh(_build.CROSSCHECK_PATH)
            _XLIB = _bind(_build.CROSSCHECK_PATH, {**SIGNATURES, **CROSSCHECK_SIGNATURES})
        return _XLIB


def set_variant(op: str, variant: int) -> int:
    """Select a kernel variant of the cross-check build (0 = the product's kernel); returns the previous selection.
    Variant 0 everywhere hands ``load()`` back to the product library."""
    if op not in _VARIANTS:
        raise ValueError(f"unknown op {op!r}")
    variant = int(variant)
    prev = _VARIANTS[op]
    if variant == prev == 0 and _XLIB is None:
        return 0                            # nothing selected, nothing to load
    rc = load_crosscheck().cdm_set_variant(op.encode(), variant)
    if rc < 0:
        raise RuntimeError(f"set_variant failed: {_XLIB.cdm_last_error().decode('utf-8', 'replace')}")
    _VARIANTS[op] = variant
    return prev


def last_error() -> str:
    return load().cdm_last_error().decode("utf-8", "replace")


def check(status: int, what: str) -> None:
    if status != OK:
        raise RuntimeError(f"{what} failed with status {status}: {last_error()}")
