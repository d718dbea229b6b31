"""Thin torch-tensor wrappers over the C ABI (include/cosmos_dm.h).

Each function validates what the C side cannot see (dtype, device, innermost stride), then passes raw
device pointers, sizes, row strides and the current HIP stream.  There is no fallback path.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import EPI_GATE_RESIDUAL, EPI_GATE_RESIDUAL_F32, EPI_NONE, EPI_ROPE_QK, EPI_SWIGLU

_EPI = {"none": EPI_NONE, "swiglu": EPI_SWIGLU, "gate_residual": EPI_GATE_RESIDUAL, "rope_qk": EPI_ROPE_QK}
FP8_DTYPE = torch.float8_e4m3fn


def _epilogue(name: str, out: torch.Tensor, residual: Optional[torch.Tensor]):
    """(epilogue code, dtype of out / residual): "gate_residual" takes its fp32 form when ``out`` is fp32 (the
    residual stream kept in fp32); every other epilogue writes bf16."""
    if name == "gate_residual" and out.dtype == torch.float32:
        if residual is None or residual.dtype != torch.float32:
            raise TypeError("an fp32 output of the gated residual needs an fp32 residual")
        return EPI_GATE_RESIDUAL_F32, torch.float32
    return _EPI[name], torch.bfloat16


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _chk(t: Optional[torch.Tensor], name: str, dtype=None, ndim: Optional[int] = None) -> int:
    if t is None:
        return 0
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (the HIP path has no CPU fallback)")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if ndim is not None and t.dim() != ndim:
        raise ValueError(f"{name} must be {ndim}-D, got shape {tuple(t.shape)}")
    if t.dim() and t.stride(-1) != 1:
        raise ValueError(f"{name} must be contiguous along its last dimension")
    return t.data_ptr()


def _f32vec(t: Optional[torch.Tensor], name: str, n: int) -> int:
    if t is None:
        return 0
    if t.numel() != n:
        raise ValueError(f"{name} must have {n} elements, got {t.numel()}")
    if t.dtype != torch.float32 or not t.is_contiguous():
        raise TypeError(f"{name} must be a contiguous fp32 tensor")
    return _chk(t.reshape(-1), name)


_OP_TIMER = None     # None, or the list that collects (category, start event, end event) while timing is on


def _timed(category: str):
    """While ``time_ops(True)`` is in force, bracket every call of the wrapped launcher with a pair of HIP events on
    the current stream (the stream the kernels are launched on)."""
    def deco(fn):
        def wrapper(*args, **kw):
            rec = _OP_TIMER
            if rec is None:
                return fn(*args, **kw)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            out = fn(*args, **kw)
            e1.record()
            rec.append((category, e0, e1))
            return out
        wrapper.__name__, wrapper.__doc__ = fn.__name__, fn.__doc__
        return wrapper
    return deco


def time_ops(enable: bool):
    """Start (True) or stop (False) collecting (category, start, end) HIP event triples around every kernel launcher
    of this module ("norm", "gemm", "rope", "pack_kv", "quant", "step"; the attention kernel itself is covered by
    ``time_attention``); stopping returns the list."""
    global _OP_TIMER
    prev, _OP_TIMER = _OP_TIMER, ([] if enable else None)
    return prev


def set_variant(op: str, variant: int) -> int:
    """Cross-check aid (tests, measurements): run ``op`` ("attn" / "gemm") on a superseded kernel of the cross-check
    build; 0 = back to the product library's kernel.  Returns the previous selection."""
    return _lib.set_variant(op, variant)


# ----------------------------------------------------------------------------- norm / quant
@_timed("norm")
def adaln_rmsnorm(x: torch.Tensor, w: torch.Tensor, shift: Optional[torch.Tensor] = None,
                  scale: Optional[torch.Tensor] = None, eps: float = 1e-6,
                  out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = rmsnorm(x) * w * (1 + scale) + shift; x [n, d] contiguous, bf16 or fp32 (residual stream kept in fp32);
    y is bf16."""
    lib = _lib.load()
    n, d = x.shape
    if not x.is_contiguous():
        raise ValueError("x must be contiguous")
    out = torch.empty((n, d), dtype=torch.bfloat16, device=x.device) if out is None else out
    if not out.is_contiguous() or out.shape != x.shape:
        raise ValueError("out must be a contiguous tensor of x's shape")
    fn = lib.cdm_adaln_rmsnorm_f32 if x.dtype == torch.float32 else lib.cdm_adaln_rmsnorm_bf16
    rc = fn(_chk(x, "x", x.dtype if x.dtype == torch.float32 else torch.bfloat16, 2), _chk(w, "w", torch.bfloat16, 1),
            _f32vec(shift, "shift", d), _f32vec(scale, "scale", d), _chk(out, "out", torch.bfloat16, 2), n, d, float(eps),
            _stream())
    _lib.check(rc, "cdm_adaln_rmsnorm")
    return out


@_timed("norm")
def adaln_rmsnorm_quant(x, w, shift=None, scale=None, eps: float = 1e-6, out_q: Optional[torch.Tensor] = None,
                        out_s: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Same norm, output quantised per token to e4m3: returns (yq [n, d] float8_e4m3fn, s_tok [n] fp32)."""
    lib = _lib.load()
    n, d = x.shape
    if not x.is_contiguous():
        raise ValueError("x must be contiguous")
    yq = torch.empty((n, d), dtype=FP8_DTYPE, device=x.device) if out_q is None else out_q
    s = torch.empty((n,), dtype=torch.float32, device=x.device) if out_s is None else out_s
    if yq.shape != (n, d) or not yq.is_contiguous() or s.shape != (n,) or not s.is_contiguous():
        raise ValueError("out_q / out_s must be contiguous [n, d] e4m3 and [n] fp32")
    fn = lib.cdm_adaln_rmsnorm_f32_quant_e4m3 if x.dtype == torch.float32 else lib.cdm_adaln_rmsnorm_quant_e4m3
    rc = fn(_chk(x, "x", x.dtype if x.dtype == torch.float32 else torch.bfloat16, 2), _chk(w, "w", torch.bfloat16, 1),
            _f32vec(shift, "shift", d), _f32vec(scale, "scale", d), _chk(yq, "out_q", FP8_DTYPE, 2),
            _chk(s, "out_s", torch.float32, 1), n, d, float(eps), _stream())
    _lib.check(rc, "cdm_adaln_rmsnorm_quant_e4m3")
    return yq, s


@_timed("quant")
def quant_rows(a: torch.Tensor, out_q: Optional[torch.Tensor] = None,
               out_s: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row e4m3 quantisation of a bf16 matrix [rows, cols] (row stride may exceed cols); ``out_q`` / ``out_s``:
    caller-owned [rows, cols] e4m3 and [rows] fp32 outputs."""
    lib = _lib.load()
    rows, cols = a.shape
    q = torch.empty((rows, cols), dtype=FP8_DTYPE, device=a.device) if out_q is None else out_q
    s = torch.empty((rows,), dtype=torch.float32, device=a.device) if out_s is None else out_s
    if q.shape != (rows, cols) or not q.is_contiguous() or s.shape != (rows,) or not s.is_contiguous():
        raise ValueError("out_q / out_s must be contiguous [rows, cols] e4m3 and [rows] fp32")
    rc = lib.cdm_quant_rows_e4m3(_chk(a, "a", torch.bfloat16, 2), a.stride(0), _chk(q, "out_q", FP8_DTYPE, 2),
                                 _chk(s, "out_s", torch.float32, 1), rows, cols, _stream())
    _lib.check(rc, "cdm_quant_rows_e4m3")
    return q, s


@_timed("quant")
def quant_rows_from_parts(a: torch.Tensor, parts: torch.Tensor, out_q: Optional[torch.Tensor] = None,
                          out_s: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """``quant_rows`` (same result, bit for bit) from partial row maxima the producer of ``a`` left behind: ``parts``
    [rows, n_parts] fp32, entry (i, c) = max |a[i, j]| over one column range, the ranges covering the row
    (``attention_packed(row_amax=...)``: one per head; ``gemm_fp8(epilogue="swiglu", row_amax=...)``: one per 64
    columns).  The row is read once."""
    lib = _lib.load()
    rows, cols = a.shape
    q = torch.empty((rows, cols), dtype=FP8_DTYPE, device=a.device) if out_q is None else out_q
    s = torch.empty((rows,), dtype=torch.float32, device=a.device) if out_s is None else out_s
    if q.shape != (rows, cols) or not q.is_contiguous() or s.shape != (rows,) or not s.is_contiguous():
        raise ValueError("out_q / out_s must be contiguous [rows, cols] e4m3 and [rows] fp32")
    if parts.dim() != 2 or parts.shape[0] != rows:
        raise ValueError("parts must be [rows, n_parts]")
    rc = lib.cdm_quant_rows_from_parts_e4m3(_chk(a, "a", torch.bfloat16, 2), a.stride(0), _chk(parts, "parts", torch.float32, 2),
                                            parts.stride(0), parts.shape[1], _chk(q, "out_q", FP8_DTYPE, 2),
                                            _chk(s, "out_s", torch.float32, 1), rows, cols, _stream())
    _lib.check(rc, "cdm_quant_rows_from_parts_e4m3")
    return q, s


def _amax_arg(row_amax: Optional[torch.Tensor], rows: int, min_cols: int):
    """(pointer, row stride) of an optional [rows, >= min_cols] fp32 output of partial row maxima."""
    if row_amax is None:
        return None, 0
    if row_amax.dim() != 2 or row_amax.shape[0] != rows or row_amax.shape[1] < min_cols:
        raise ValueError(f"row_amax must be [{rows}, >= {min_cols}] fp32")
    return _chk(row_amax, "row_amax", torch.float32, 2), row_amax.stride(0)


# ----------------------------------------------------------------------------- GEMM
@_timed("gemm")
def gemm(a: torch.Tensor, w: torch.Tensor, *, w2: Optional[torch.Tensor] = None, epilogue: str = "none",
         residual: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
         cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None, rope_cols: int = 0,
         head_dim: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[M, N] = epilogue(a[M, K] @ w[N, K]^T); bf16 in / fp32 accumulate / bf16 out."""
    lib = _lib.load()
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or (w2 is not None and w2.shape != w.shape):
        raise ValueError("weight shape mismatch")
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
    if out.shape != (M, N):
        raise ValueError("out shape mismatch")
    if w2 is not None and w2.stride(0) != w.stride(0):
        raise ValueError("w and w2 must share a row stride")
    half = head_dim // 2 if head_dim else 0
    epi, odt = _epilogue(epilogue, out, residual)
    rc = lib.cdm_gemm_bf16(_chk(a, "a", torch.bfloat16, 2), a.stride(0), _chk(w, "w", torch.bfloat16, 2), w.stride(0),
                           _chk(w2, "w2", torch.bfloat16, 2), _chk(out, "out", odt, 2), out.stride(0),
                           M, N, K, epi, _chk(residual, "residual", odt, 2),
                           residual.stride(0) if residual is not None else 0, _f32vec(gate, "gate", N),
                           _f32vec(cos, "cos", M * half), _f32vec(sin, "sin", M * half), int(rope_cols), int(head_dim),
                           _stream())
    _lib.check(rc, "cdm_gemm_bf16")
    return out


@_timed("edge")
def linear_bias(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T + bias[N] for the narrow linear layers at the edges of the stack (patchify /
    un-patchify, action and audio projections); bf16 in / fp32 accumulate / bf16 out; any widths (16-byte accesses where
    rows are 16-byte aligned and N, K are multiples of 8)."""
    lib = _lib.load()
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or (bias is not None and bias.shape != (N,)):
        raise ValueError("weight / bias shape mismatch")
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
    if out.shape != (M, N):
        raise ValueError("out shape mismatch")
    rc = lib.cdm_linear_bias_bf16(_chk(a, "a", torch.bfloat16, 2), a.stride(0), _chk(w, "w", torch.bfloat16, 2), w.stride(0),
                                  _chk(bias, "bias", torch.bfloat16, 1), _chk(out, "out", torch.bfloat16, 2), out.stride(0),
                                  M, N, K, _stream())
    _lib.check(rc, "cdm_linear_bias_bf16")
    return out


@_timed("gemm")
def gemm_fp8(aq: torch.Tensor, sa: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor, *,
             w2q: Optional[torch.Tensor] = None, sw2: Optional[torch.Tensor] = None, epilogue: str = "none",
             residual=None, gate=None, cos=None, sin=None, rope_cols: int = 0, head_dim: int = 0,
             out: Optional[torch.Tensor] = None, row_amax: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[M, N] = epilogue((aq @ wq^T) * sa[:, None] * sw[None, :]); e4m3 operands, bf16 out.  ``row_amax`` (SwiGLU
    epilogue only): [M, >= ceil(N / 64)] fp32 that receives the largest |out| of each row within every 64 columns."""
    lib = _lib.load()
    M, K = aq.shape
    N = wq.shape[0]
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=aq.device)
    half = head_dim // 2 if head_dim else 0
    epi, odt = _epilogue(epilogue, out, residual)
    rc = lib.cdm_gemm_fp8(_chk(aq, "aq", FP8_DTYPE, 2), aq.stride(0), _f32vec(sa, "sa", M),
                          _chk(wq, "wq", FP8_DTYPE, 2), wq.stride(0), _f32vec(sw, "sw", N),
                          _chk(w2q, "w2q", FP8_DTYPE, 2), _f32vec(sw2, "sw2", N),
                          _chk(out, "out", odt, 2), out.stride(0), M, N, K, epi,
                          _chk(residual, "residual", odt, 2),
                          residual.stride(0) if residual is not None else 0, _f32vec(gate, "gate", N),
                          _f32vec(cos, "cos", M * half), _f32vec(sin, "sin", M * half), int(rope_cols), int(head_dim),
                          *_amax_arg(row_amax, M, (N + 63) // 64), _stream())
    _lib.check(rc, "cdm_gemm_fp8")
    return out


@_timed("gemm")
def grouped_gemm(a: torch.Tensor, ws: Sequence[torch.Tensor], segments: Sequence[Tuple[int, int]], *,
                 w2s: Optional[Sequence[torch.Tensor]] = None, epilogue: str = "none", residual=None,
                 gates: Optional[Sequence[Optional[torch.Tensor]]] = None, cos=None, sin=None, rope_cols: int = 0,
                 head_dim: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """MoT routed linear: rows [start, start+len) of ``a`` use ws[g] (w2s[g], gates[g])."""
    lib = _lib.load()
    M, K = a.shape
    N = ws[0].shape[0]
    n_seg = len(segments)
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
    ldw = ws[0].stride(0)
    for w in list(ws) + list(w2s or []):
        if w.shape != ws[0].shape or w.stride(0) != ldw:
            raise ValueError("all segment weights must share shape and row stride")
    PP = C.c_void_p * n_seg
    wp = PP(*[_chk(w, "w", torch.bfloat16, 2) for w in ws])
    w2p = PP(*[_chk(w, "w2", torch.bfloat16, 2) for w in w2s]) if w2s is not None else None
    gp = PP(*[(_f32vec(g, "gate", N) or None) for g in gates]) if gates is not None else None
    I64 = C.c_int64 * n_seg
    st, ln = I64(*[int(s) for s, _ in segments]), I64(*[int(l) for _, l in segments])
    half = head_dim // 2 if head_dim else 0
    epi, odt = _epilogue(epilogue, out, residual)
    rc = lib.cdm_grouped_gemm_bf16(_chk(a, "a", torch.bfloat16, 2), a.stride(0), wp, ldw, w2p,
                                   _chk(out, "out", odt, 2), out.stride(0), st, ln, n_seg, N, K,
                                   epi, _chk(residual, "residual", odt, 2),
                                   residual.stride(0) if residual is not None else 0, gp,
                                   _f32vec(cos, "cos", M * half), _f32vec(sin, "sin", M * half), int(rope_cols),
                                   int(head_dim), _stream())
    _lib.check(rc, "cdm_grouped_gemm_bf16")
    return out


@_timed("gemm")
def grouped_gemm_fp8(aq: torch.Tensor, sa: torch.Tensor, wqs: Sequence[torch.Tensor], sws: Sequence[torch.Tensor],
                     segments: Sequence[Tuple[int, int]], *, w2qs: Optional[Sequence[torch.Tensor]] = None,
                     sw2s: Optional[Sequence[torch.Tensor]] = None, epilogue: str = "none", residual=None,
                     gates: Optional[Sequence[Optional[torch.Tensor]]] = None, cos=None, sin=None, rope_cols: int = 0,
                     head_dim: int = 0, out: Optional[torch.Tensor] = None,
                     row_amax: Optional[torch.Tensor] = None) -> torch.Tensor:
    """e4m3 form of ``grouped_gemm``: ``sa`` [M] per-token scales, ``sws[g]`` / ``sw2s[g]`` per-channel weight scales;
    ``row_amax`` as in ``gemm_fp8``."""
    lib = _lib.load()
    M, K = aq.shape
    N = wqs[0].shape[0]
    n_seg = len(segments)
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=aq.device)
    ldw = wqs[0].stride(0)
    for w in list(wqs) + list(w2qs or []):
        if w.shape != wqs[0].shape or w.stride(0) != ldw:
            raise ValueError("all segment weights must share shape and row stride")
    PP = C.c_void_p * n_seg
    wp = PP(*[_chk(w, "wq", FP8_DTYPE, 2) for w in wqs])
    swp = PP(*[_f32vec(s, "sw", N) for s in sws])
    w2p = PP(*[_chk(w, "w2q", FP8_DTYPE, 2) for w in w2qs]) if w2qs is not None else None
    sw2p = PP(*[_f32vec(s, "sw2", N) for s in sw2s]) if sw2s is not None else None
    gp = PP(*[(_f32vec(g, "gate", N) or None) for g in gates]) if gates is not None else None
    I64 = C.c_int64 * n_seg
    st, ln = I64(*[int(s) for s, _ in segments]), I64(*[int(l) for _, l in segments])
    half = head_dim // 2 if head_dim else 0
    epi, odt = _epilogue(epilogue, out, residual)
    rc = lib.cdm_grouped_gemm_fp8(_chk(aq, "aq", FP8_DTYPE, 2), aq.stride(0), _f32vec(sa, "sa", M), wp, swp, ldw, w2p, sw2p,
                                  _chk(out, "out", odt, 2), out.stride(0), st, ln, n_seg, N, K,
                                  epi, _chk(residual, "residual", odt, 2),
                                  residual.stride(0) if residual is not None else 0, gp,
                                  _f32vec(cos, "cos", M * half), _f32vec(sin, "sin", M * half), int(rope_cols),
                                  int(head_dim), *_amax_arg(row_amax, M, (N + 63) // 64), _stream())
    _lib.check(rc, "cdm_grouped_gemm_fp8")
    return out


@_timed("gemm")
def gemm_qkv_pack(a: torch.Tensor, sa: Optional[torch.Tensor], ws: Sequence[torch.Tensor],
                  sws: Optional[Sequence[torch.Tensor]], segments: Sequence[Tuple[int, int]], n_heads: int,
                  n_kv_heads: int, head_dim: int, q_out: torch.Tensor, workspace: torch.Tensor,
                  cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None, qk_norm=None) -> None:
    """Fused QKV projection: rows [start, start+len) of ``a`` use ws[g] = [d_q + 2 d_kv, K]; Q goes to ``q_out``
    ([n, >= d_q] bf16 rows, neither normalised nor rotated), K (normalised per head with row g of ``qk_norm``'s K
    weights when given, then rotated with cos/sin when given) and V go straight into the attention kernel's tile
    images in ``workspace`` (for ``attention_packed``, which takes the same ``qk_norm`` for Q).  ``qk_norm`` =
    (q_weight, k_weight, seg_ends, eps) with one segment per GEMM segment.  e4m3 operands when ``sa`` / ``sws`` are
    given.  Raises where the fused form does not apply (``qkv_pack_applies`` tells beforehand)."""
    lib = _lib.load()
    M, K = a.shape
    n_seg = len(segments)
    ldw = ws[0].stride(0)
    for w in ws:
        if w.shape != ws[0].shape or w.stride(0) != ldw:
            raise ValueError("all segment weights must share shape and row stride")
    if ws[0].shape[0] != (n_heads + 2 * n_kv_heads) * head_dim:
        raise ValueError("fused QKV weights must have (n_heads + 2 n_kv_heads) * head_dim rows")
    PP = C.c_void_p * n_seg
    I64 = C.c_int64 * n_seg
    st, ln = I64(*[int(s) for s, _ in segments]), I64(*[int(l) for _, l in segments])
    half = head_dim // 2
    n = sum(int(l) for _, l in segments)
    qn, _keep = _qk_norm_arg(qk_norm, head_dim)
    tail = (_f32vec(cos, "cos", n * half), _f32vec(sin, "sin", n * half), qn, _chk(workspace, "workspace", torch.uint8, 1),
            workspace.numel(), _stream())
    if sa is None:
        wp = PP(*[_chk(w, "w", torch.bfloat16, 2) for w in ws])
        rc = lib.cdm_grouped_gemm_qkv_pack_bf16(_chk(a, "a", torch.bfloat16, 2), a.stride(0), wp, ldw,
                                                _chk(q_out, "q_out", torch.bfloat16, 2), q_out.stride(0), st, ln, n_seg, K,
                                                n_heads, n_kv_heads, head_dim, *tail)
        _lib.check(rc, "cdm_grouped_gemm_qkv_pack_bf16")
    else:
        N = ws[0].shape[0]
        wp = PP(*[_chk(w, "wq", FP8_DTYPE, 2) for w in ws])
        swp = PP(*[_f32vec(s, "sw", N) for s in sws])
        rc = lib.cdm_grouped_gemm_qkv_pack_fp8(_chk(a, "aq", FP8_DTYPE, 2), a.stride(0), _f32vec(sa, "sa", M), wp, swp, ldw,
                                               _chk(q_out, "q_out", torch.bfloat16, 2), q_out.stride(0), st, ln, n_seg, K,
                                               n_heads, n_kv_heads, head_dim, *tail)
        _lib.check(rc, "cdm_grouped_gemm_qkv_pack_fp8")


def qkv_pack_applies(segments: Sequence[Tuple[int, int]], head_dim: int, n_heads: int = 2, n_kv_heads: int = 2) -> bool:
    """Whether ``gemm_qkv_pack`` accepts this layout: head_dim 128, or 64 with even head counts (a wave writes the
    images of 128 consecutive columns), segments tiling [0, n) in order, each starting on a multiple of 64 tokens (a
    64-key tile image is written by one wave from one weight set)."""
    pos = 0
    for s, l in segments:
        if int(s) != pos or pos % 64:
            return False
        pos += int(l)
    return pos > 0 and (head_dim == 128 or (head_dim == 64 and n_heads % 2 == 0 and n_kv_heads % 2 == 0))


# ----------------------------------------------------------------------------- RoPE / attention
@_timed("rope")
def mrope_qk_(q: torch.Tensor, k: Optional[torch.Tensor], cos: torch.Tensor, sin: torch.Tensor, n_heads: int,
              head_dim: int) -> None:
    """In-place rotate-half mRoPE on q and k ([n, n_heads*head_dim] views, any row stride)."""
    lib = _lib.load()
    n = q.shape[0]
    half = head_dim // 2
    rc = lib.cdm_mrope_qk_bf16(_chk(q, "q", torch.bfloat16, 2), q.stride(0), _chk(k, "k", torch.bfloat16, 2),
                               k.stride(0) if k is not None else 0, _f32vec(cos, "cos", n * half),
                               _f32vec(sin, "sin", n * half), n, n_heads, head_dim, _stream())
    _lib.check(rc, "cdm_mrope_qk_bf16")


def attn_workspace_bytes(n_tokens: int, n_kv_heads: int, head_dim: int) -> int:
    """Bytes of the K / V tile images of ``n_tokens`` tokens (``n_kv_heads`` = K / V heads)."""
    return int(_lib.load().cdm_attn_workspace_bytes(n_tokens, n_kv_heads, head_dim))


def attn_workspace_total_bytes(n_tokens: int, n_heads: int, n_kv_heads: int, head_dim: int) -> int:
    """Tile images (rounded up to 256 bytes) plus the scratch of the split: the workspace ``attention`` allocates."""
    need = attn_workspace_bytes(n_tokens, n_kv_heads, head_dim)
    return max((need + 255) // 256 * 256 + attn_split_scratch_bytes(n_tokens, n_heads, head_dim), 16)


def attn_split_scratch_bytes(n_tokens: int, n_heads: int, head_dim: int) -> int:
    """Bytes of scratch with which ``attention_packed`` splits the last, partial round of its workgroups by key range
    (0: nothing to split for this shape).  ``n_heads`` counts query heads."""
    return int(_lib.load().cdm_attn_split_scratch_bytes(n_tokens, n_heads, head_dim))


def _extra_of(workspace: torch.Tensor, need: int) -> Optional[torch.Tensor]:
    """What a workspace holds beyond the tile images (rounded up to 256 bytes), or None."""
    used = (need + 255) // 256 * 256
    return workspace[used:] if workspace.numel() > used else None


def _qk_norm_arg(qk_norm, head_dim: int):
    """-> (pointer or None, keep-alive objects) for the optional ``cdm_qk_norm`` argument."""
    if qk_norm is None:
        return None, None
    qw, kw, seg_ends, eps = qk_norm
    seg_ends = [int(e) for e in seg_ends]
    ends = (C.c_int64 * len(seg_ends))(*seg_ends)
    st = _lib.QkNorm(_f32vec(qw, "qk_norm q_weight", len(seg_ends) * head_dim),
                     _f32vec(kw, "qk_norm k_weight", len(seg_ends) * head_dim), ends, len(seg_ends), float(eps))
    return C.addressof(st), (st, ends)


@_timed("pack_kv")
def attention_pack_kv(k: torch.Tensor, v: torch.Tensor, n_heads: int, head_dim: int,
                      workspace: Optional[torch.Tensor] = None, cos: Optional[torch.Tensor] = None,
                      sin: Optional[torch.Tensor] = None, qk_norm=None) -> torch.Tensor:
    """First stage of ``attention``: K (normalised / rotated if asked) and V of ``n`` tokens -> tile images in
    ``workspace`` (returned).  The images can be kept and passed to ``attention_packed`` as its ``prefix``.
    ``n_heads`` counts K / V heads here (fewer than query heads under grouped-query attention)."""
    lib = _lib.load()
    n, d = k.shape[0], n_heads * head_dim
    if k.shape != (n, d) or v.shape != (n, d):
        raise ValueError("k, v must be [n_tokens, n_heads*head_dim]")
    if workspace is None:
        workspace = torch.empty((max(attn_workspace_bytes(n, n_heads, head_dim), 16),), dtype=torch.uint8, device=k.device)
    half = head_dim // 2
    qn, _keep = _qk_norm_arg(qk_norm, head_dim)
    rc = lib.cdm_attn_pack_kv_bf16(_chk(k, "k", torch.bfloat16, 2), k.stride(0), _chk(v, "v", torch.bfloat16, 2),
                                   v.stride(0), _f32vec(cos, "cos", n * half), _f32vec(sin, "sin", n * half),
                                   _chk(workspace, "workspace", torch.uint8, 1), workspace.numel(), n, n_heads, head_dim,
                                   qn, _stream())
    _lib.check(rc, "cdm_attn_pack_kv_bf16")
    return workspace


def attention_packed(q: torch.Tensor, workspace: torch.Tensor, n_heads: int, head_dim: int,
                     out: Optional[torch.Tensor] = None, cos: Optional[torch.Tensor] = None,
                     sin: Optional[torch.Tensor] = None, qk_norm=None, prefix=None,
                     causal_prefix: int = 0, n_kv_heads: Optional[int] = None,
                     row_amax: Optional[torch.Tensor] = None,
                     split_scratch: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Second stage of ``attention``: the ``n`` query rows against the keys packed in ``workspace`` (``n`` tokens),
    preceded by the keys of ``prefix`` = (images, n_prefix_tokens) if given.  ``row_amax``: optional contiguous
    [n, n_heads] fp32 that receives the largest |out| of each row within each head (for ``quant_rows_from_parts``).
    ``split_scratch``: optional uint8 buffer of ``attn_split_scratch_bytes`` bytes; default: what ``workspace`` holds
    beyond the images."""
    lib = _lib.load()
    n, d = q.shape[0], n_heads * head_dim
    n_kv_heads = n_heads if n_kv_heads is None else int(n_kv_heads)
    if out is None:
        out = torch.empty((n, d), dtype=torch.bfloat16, device=q.device)
    half = head_dim // 2
    qn, _keep = _qk_norm_arg(qk_norm, head_dim)
    pws, npre = (None, 0) if prefix is None else (_chk(prefix[0], "prefix images", torch.uint8, 1), int(prefix[1]))
    if prefix is not None and prefix[0].numel() < attn_workspace_bytes(npre, n_kv_heads, head_dim):
        raise ValueError("prefix images are smaller than the workspace of n_prefix tokens")
    if workspace.numel() < attn_workspace_bytes(n, n_kv_heads, head_dim):
        raise ValueError("workspace is smaller than the images of n tokens")
    amax_ptr = None
    if row_amax is not None:
        if row_amax.shape != (n, n_heads) or not row_amax.is_contiguous():
            raise ValueError("row_amax must be a contiguous [n_tokens, n_heads] fp32 tensor")
        amax_ptr = _chk(row_amax, "row_amax", torch.float32, 2)
    if split_scratch is None:
        split_scratch = _extra_of(workspace, attn_workspace_bytes(n, n_kv_heads, head_dim))
    ss_ptr = None if split_scratch is None else _chk(split_scratch, "split_scratch", torch.uint8, 1)
    ss_bytes = 0 if split_scratch is None else split_scratch.numel()
    timer = _ATTN_TIMER
    if timer is not None:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
    rc = lib.cdm_attn_fwd_packed_bf16(_chk(q, "q", torch.bfloat16, 2), q.stride(0), _f32vec(cos, "cos", n * half),
                                      _f32vec(sin, "sin", n * half), _chk(workspace, "workspace", torch.uint8, 1),
                                      _chk(out, "out", torch.bfloat16, 2), out.stride(0), n, n_heads, n_kv_heads, head_dim,
                                      qn, pws, npre, int(causal_prefix), amax_ptr, ss_ptr, ss_bytes, _stream())
    if timer is not None:
        e1.record()
        timer.append((e0, e1))
    _lib.check(rc, "cdm_attn_fwd_packed_bf16")
    return out


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, n_heads: int, head_dim: int,
              out: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None,
              cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None,
              qk_norm=None, causal_prefix: int = 0, prefix=None, n_kv_heads: Optional[int] = None) -> torch.Tensor:
    """Attention over the joint sequence; q: [n, n_heads*head_dim], k, v: [n, n_kv_heads*head_dim] bf16 views (row
    stride free; ``n_kv_heads`` defaults to ``n_heads``, fewer = grouped-query attention).
    With cos/sin ([n, head_dim/2] fp32) rotate-half mRoPE is applied to Q and K inside the kernels.
    ``qk_norm`` = (q_weight, k_weight, seg_ends, eps) switches on the per-head RMSNorm of Q and K ahead of the
    rotation: weights [n_seg, head_dim] fp32 on the device, ``seg_ends`` the exclusive end token of each segment.
    ``causal_prefix`` = P > 0 selects the hybrid mask (the first P tokens causal among themselves, blind to the
    rest; all others see everything); ``prefix`` = (images, n_prefix_tokens) prepends already packed keys."""
    lib = _lib.load()
    n = q.shape[0]
    d = n_heads * head_dim
    n_kv_heads = n_heads if n_kv_heads is None else int(n_kv_heads)
    dkv = n_kv_heads * head_dim
    if q.shape != (n, d) or k.shape != (n, dkv) or v.shape != (n, dkv):
        raise ValueError("q must be [n_tokens, n_heads*head_dim] and k, v [n_tokens, n_kv_heads*head_dim]")
    if out is None:
        out = torch.empty((n, d), dtype=torch.bfloat16, device=q.device)
    need = attn_workspace_bytes(n, n_kv_heads, head_dim)
    if workspace is None:
        workspace = torch.empty((attn_workspace_total_bytes(n, n_heads, n_kv_heads, head_dim),), dtype=torch.uint8,
                                device=q.device)
    if _ATTN_TIMER is None and _OP_TIMER is None and prefix is None:
        half = head_dim // 2
        qn, _keep = _qk_norm_arg(qk_norm, head_dim)
        rc = lib.cdm_attn_fwd_bf16(_chk(q, "q", torch.bfloat16, 2), q.stride(0), _chk(k, "k", torch.bfloat16, 2),
                                   k.stride(0), _chk(v, "v", torch.bfloat16, 2), v.stride(0),
                                   _f32vec(cos, "cos", n * half), _f32vec(sin, "sin", n * half),
                                   _chk(out, "out", torch.bfloat16, 2), out.stride(0), n, n_heads, n_kv_heads, head_dim,
                                   _chk(workspace, "workspace", torch.uint8, 1), workspace.numel(), qn,
                                   int(causal_prefix), _stream())
        _lib.check(rc, "cdm_attn_fwd_bf16")
        return out
    # two-stage form: prefix images, or HIP events around the attention kernel alone while timing is on
    attention_pack_kv(k, v, n_kv_heads, head_dim, workspace, cos, sin, qk_norm)
    return attention_packed(q, workspace, n_heads, head_dim, out, cos, sin, qk_norm, prefix, causal_prefix, n_kv_heads)


@_timed("step")
def cfg_multistep(x: torch.Tensor, v_cond: torch.Tensor, v_uncond: Optional[torch.Tensor], guidance: float,
                  coef: Sequence[Sequence[float]], hist: Sequence[torch.Tensor], outs: Sequence[torch.Tensor]) -> None:
    """outs[j] = coef[j][0] x + coef[j][1] v + sum_k coef[j][2+k] hist[k] with v = v_uncond + guidance (v_cond -
    v_uncond) (v = v_cond without v_uncond), all outputs in ONE pass.  x, hist, outs: fp32; v_cond, v_uncond: bf16; all
    of one shape, contiguous.  An output may be ``x`` or one of ``hist`` (in place)."""
    lib = _lib.load()
    n = x.numel()
    if not 1 <= len(outs) <= 3 or len(coef) != len(outs) or any(len(r) != 2 + len(hist) for r in coef):
        raise ValueError("coef must have one row of 2 + len(hist) values per output (1..3 outputs)")
    for t, name, dt in [(x, "x", torch.float32), (v_cond, "v_cond", torch.bfloat16)] + \
                       ([(v_uncond, "v_uncond", torch.bfloat16)] if v_uncond is not None else []) + \
                       [(h, "hist", torch.float32) for h in hist] + [(o, "out", torch.float32) for o in outs]:
        if t.numel() != n or not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous with {n} elements")
        _chk(t.reshape(-1), name, dt)
    hp = (C.c_void_p * max(len(hist), 1))(*[h.data_ptr() for h in hist])
    op = (C.c_void_p * len(outs))(*[o.data_ptr() for o in outs])
    flat = [float(c) for row in coef for c in row]
    cf = (C.c_float * len(flat))(*flat)
    rc = lib.cdm_cfg_step_f32(x.data_ptr(), v_cond.data_ptr(), v_uncond.data_ptr() if v_uncond is not None else None,
                              float(guidance), hp, len(hist), cf, op, len(outs), n, _stream())
    _lib.check(rc, "cdm_cfg_step_f32")


def cfg_step(x: torch.Tensor, v_cond: torch.Tensor, v_uncond: Optional[torch.Tensor], guidance: float,
             coef: Sequence[float], hist: Sequence[torch.Tensor] = (), v_out: Optional[torch.Tensor] = None,
             out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = coef[0] x + coef[1] v + sum_i coef[2+i] hist[i]; ``v_out`` (optional) receives the guided prediction v.
    ``out`` may be ``x`` itself.  The single-update form of ``cfg_multistep``."""
    if len(coef) != 2 + len(hist):
        raise ValueError("coef must hold 2 + len(hist) values")
    if out is None:
        out = torch.empty_like(x)
    rows, outs = [list(coef)], [out]
    if v_out is not None:
        rows.append([0.0, 1.0] + [0.0] * len(hist))
        outs.append(v_out)
    cfg_multistep(x, v_cond, v_uncond, guidance, rows, hist, outs)
    return out


_ATTN_TIMER = None


def time_attention(enable: bool):
    """Start (True) or stop (False) collecting HIP event pairs around every attention kernel launch on the
    current stream; stopping returns the list of (start, end) events."""
    global _ATTN_TIMER
    prev, _ATTN_TIMER = _ATTN_TIMER, ([] if enable else None)
    return prev
