"""ctypes binding of libcosmos_dm_hip.so (the C ABI declared in include/cosmos_dm.h).

The product path has no CPU fallback: if the library is missing it is built once with hipcc, and if
that fails, or a call returns a non-zero status, a RuntimeError is raised.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

from . import build as _build

_LOCK = threading.Lock()
_LIB = None

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
    "cdm_set_variant": (_I32, [C.c_char_p, _I32]),
    "cdm_adaln_rmsnorm_bf16": (_I32, [_P, _P, _P, _P, _P, _I64, _I64, _F32, _P]),
    "cdm_adaln_rmsnorm_quant_e4m3": (_I32, [_P, _P, _P, _P, _P, _P, _I64, _I64, _F32, _P]),
    "cdm_adaln_rmsnorm_f32": (_I32, [_P, _P, _P, _P, _P, _I64, _I64, _F32, _P]),
    "cdm_adaln_rmsnorm_f32_quant_e4m3": (_I32, [_P, _P, _P, _P, _P, _P, _I64, _I64, _F32, _P]),
    "cdm_quant_rows_e4m3": (_I32, [_P, _I64, _P, _P, _I64, _I64, _P]),
    "cdm_gemm_bf16": (_I32, [_P, _I64, _P, _I64, _P, _P, _I64, _I64, _I64, _I64, _I32, _P, _I64, _P, _P, _P, _I64,
                             _I32, _P]),
    "cdm_gemm_fp8": (_I32, [_P, _I64, _P, _P, _I64, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I32, _P, _I64, _P, _P,
                            _P, _I64, _I32, _P]),
    "cdm_mrope_qk_bf16": (_I32, [_P, _I64, _P, _I64, _P, _P, _I64, _I32, _I32, _P]),
    "cdm_attn_workspace_bytes": (_I64, [_I64, _I32, _I32]),
    "cdm_attn_fwd_bf16": (_I32, [_P, _I64, _P, _I64, _P, _I64, _P, _P, _P, _I64, _I64, _I32, _I32, _I32, _P, _I64, _P, _I64,
                                 _P]),
    "cdm_attn_static_scratch_bytes": (_I64, []),
    "cdm_attn_fwd_static_bf16": (_I32, [_P, _I64, _P, _I64, _P, _I64, _P, _P, _P, _I64, _I64, _I32, _I32, _I32, _P, _I64, _P]),
    "cdm_attn_pack_kv_bf16": (_I32, [_P, _I64, _P, _I64, _P, _P, _P, _I64, _I64, _I32, _I32, _P, _P]),
    "cdm_attn_fwd_packed_bf16": (_I32, [_P, _I64, _P, _P, _P, _P, _I64, _I64, _I32, _I32, _I32, _P, _P, _I64, _I64, _P]),
    "cdm_grouped_gemm_fp8": (_I32, [_P, _I64, _P, C.POINTER(_P), C.POINTER(_P), _I64, C.POINTER(_P), C.POINTER(_P), _P, _I64,
                                    C.POINTER(_I64), C.POINTER(_I64), _I32, _I64, _I64, _I32, _P, _I64, C.POINTER(_P), _P,
                                    _P, _I64, _I32, _P]),
    "cdm_cfg_step_f32": (_I32, [_P, _P, _P, _F32, C.POINTER(_P), _I32, C.POINTER(_F32), C.POINTER(_P), _I32, _I64, _P]),
    "cdm_grouped_gemm_qkv_pack_bf16": (_I32, [_P, _I64, C.POINTER(_P), _I64, _P, _I64, C.POINTER(_I64), C.POINTER(_I64), _I32,
                                              _I64, _I32, _I32, _I32, _P, _P, _P, _P, _I64, _P]),
    "cdm_grouped_gemm_qkv_pack_fp8": (_I32, [_P, _I64, _P, C.POINTER(_P), C.POINTER(_P), _I64, _P, _I64, C.POINTER(_I64),
                                             C.POINTER(_I64), _I32, _I64, _I32, _I32, _I32, _P, _P, _P, _P, _I64, _P]),
    "cdm_grouped_gemm_bf16": (_I32, [_P, _I64, C.POINTER(_P), _I64, C.POINTER(_P), _P, _I64, C.POINTER(_I64),
                                     C.POINTER(_I64), _I32, _I64, _I64, _I32, _P, _I64, C.POINTER(_P), _P, _P, _I64,
                                     _I32, _P]),
}


def lib_path() -> str:
    """Path of the shared library; COSMOS_DM_LIB overrides the in-tree build (e.g. an experimental build)."""
    return os.environ.get("COSMOS_DM_LIB") or _build.LIB_PATH


def load():
    """Return the loaded library.  The in-tree build is (re)built first if it is missing or was built from other
    sources than the ones present (a stale build is never run); a library named by COSMOS_DM_LIB is taken as is."""
    global _LIB
    with _LOCK:
        if _LIB is not None:
            return _LIB
        path = lib_path()
        if path == _build.LIB_PATH:
            want = _build.source_hash()
            if _build.built_hash(path) != want:
                _build.build(verbose=False)
                if _build.built_hash(path) != want:
                    raise RuntimeError(f"{path} does not carry the hash of the present sources after a rebuild")
        elif not os.path.exists(path):
            raise RuntimeError(f"COSMOS_DM_LIB={path} does not exist")
        lib = C.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)     # AttributeError here = the library does not export the ABI
            fn.restype, fn.argtypes = res, args
        _LIB = lib
        return lib


def last_error() -> str:
    return load().cdm_last_error().decode("utf-8", "replace")


def check(status: int, what: str) -> None:
    if status != OK:
        raise RuntimeError(f"{what} failed with status {status}: {last_error()}")
