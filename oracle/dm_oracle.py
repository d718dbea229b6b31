"""fp32 PyTorch restatement of the Cosmos 3 generator (DM) block forward.

Test infrastructure: see the package docstring for who may import this and
for the pinning status of every function.  Everything is fp32 (statistics,
softmax and accumulation included) and never rounds to bf16.  The functions
allocate on the device of their inputs: the pinning tests and the parity tests
run them on the CPU; for free-running checks of a whole stack at full size (hours
on host cores) a GPU test may also hand them device tensors, which runs the very
same statements through stock PyTorch fp32 operators (and checks that run
against the CPU run on sampled rows first).

Citations use ``REF/`` for the reference repository and ``TF/`` for the
installed third-party ``transformers 5.15.0`` package, whose Cosmos 3 AR tower
("identical to Qwen3-VL", TF/models/cosmos3_omni/modular_cosmos3_omni.py:25-26)
supplies the operator conventions the generator branch shares.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import torch

__all__ = [
    "timestep_embedding", "time_mlp", "adaln_modulation", "rms_norm", "adaln_rms_norm",
    "mrope_axis_map", "text_positions", "vision_positions", "joint_positions",
    "mrope_cos_sin", "apply_mrope", "attention", "attention_rows", "swiglu",
    "dm_block", "dm_stack", "quant_e4m3_rows", "quant_e4m3_weight", "fp8_linear",
    "max_rel_err", "cos_sim", "E4M3_MAX", "cfg_step", "flow_sigmas", "hybrid_kv_end",
]

E4M3_MAX = 448.0


# --------------------------------------------------------------------------
# conditioning (stays in PyTorch in the product too; conventions unpinned)
# --------------------------------------------------------------------------
def timestep_embedding(t: torch.Tensor, dim: int = 256, max_period: float = 10000.0) -> torch.Tensor:
    """256-d sinusoidal embedding [cos(t f), sin(t f)], f_k = max_period^(-k/half).

    The benchmark configuration asks for "a 256-d sinusoidal embedding of
    t ~ U[0,1000)"; the ``time_embedder`` module is attested by
    TF/models/cosmos3_omni/modeling_cosmos3_omni.py:50.  sin/cos order is a
    choice (parity unpinned).
    """
    half = dim // 2
    k = torch.arange(half, dtype=torch.float32)
    f = torch.exp(-math.log(max_period) * k / half)
    a = t.to(torch.float32).reshape(-1, 1) * f.reshape(1, -1)
    return torch.cat([a.cos(), a.sin()], dim=-1)


def time_mlp(e: torch.Tensor, w1, b1, w2, b2) -> torch.Tensor:
    """c = W2 silu(W1 e + b1) + b2 (parity unpinned: activation choice)."""
    h = torch.nn.functional.silu(e @ w1.t() + b1)
    return h @ w2.t() + b2


def adaln_modulation(c: torch.Tensor, w_ada, b_ada) -> Tuple[torch.Tensor, ...]:
    """m = W_ada silu(c) + b_ada, split (shift1, scale1, gate1, shift2, scale2, gate2)."""
    m = torch.nn.functional.silu(c) @ w_ada.t() + b_ada
    return tuple(m.reshape(-1).chunk(6))


# --------------------------------------------------------------------------
# norms
# --------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """RMSNorm: x * rsqrt(mean(x^2) + eps) * w, all fp32.

    Follows TF/models/qwen3_vl/modeling_qwen3_vl.py:400-405.
    """
    x = x.to(torch.float32)
    var = x.pow(2).mean(-1, keepdim=True)
    return w.to(torch.float32) * (x * torch.rsqrt(var + eps))


def adaln_rms_norm(x, w, shift: Optional[torch.Tensor], scale: Optional[torch.Tensor], eps: float = 1e-6):
    """y = rms_norm(x; w) * (1 + scale) + shift  (shift/scale per channel, shared by all tokens).

    The per-branch norm is REF/README.md:74 ("per-branch norm"); the
    shift/scale/gate modulation is the benchmark configuration's adaLN.
    ``None`` modulation is the AR-branch plain RMSNorm.
    """
    y = rms_norm(x, w, eps)
    if scale is not None:
        y = y * (1.0 + scale.to(torch.float32))
    if shift is not None:
        y = y + shift.to(torch.float32)
    return y


# --------------------------------------------------------------------------
# 3-D mRoPE
# --------------------------------------------------------------------------
def mrope_axis_map(head_dim: int, sections: Sequence[int], layout: str = "chunked") -> torch.Tensor:
    """Axis (0=t, 1=h, 2=w) that rotary pair i = (i, i + head_dim/2) follows.

    ``sections`` counts channels (sum == head_dim), i.e. section/2 pairs each.
    chunked:     [t]*s_t/2 + [h]*s_h/2 + [w]*s_w/2
                 (TF/models/qwen2_vl/modeling_qwen2_vl.py:212-217 with
                 mrope_section = pairs per axis)
    interleaved: t h w t h w ... with the tail given to t
                 (TF/models/qwen3_vl/modeling_qwen3_vl.py:372-388)
    """
    assert sum(sections) == head_dim and all(s % 2 == 0 for s in sections)
    half = head_dim // 2
    pairs = [s // 2 for s in sections]
    amap = torch.zeros(half, dtype=torch.long)
    if layout == "chunked":
        amap[pairs[0]:pairs[0] + pairs[1]] = 1
        amap[pairs[0] + pairs[1]:] = 2
    elif layout == "interleaved":
        for axis, offset in ((1, 1), (2, 2)):
            amap[offset:pairs[axis] * 3:3] = axis
    else:
        raise ValueError(layout)
    return amap


def text_positions(start: int, n: int) -> torch.Tensor:
    """1-D run: p = (s+j, s+j, s+j). TF/models/cosmos3_omni/modeling_cosmos3_omni.py:247-252."""
    return (torch.arange(n, dtype=torch.long) + start).view(1, -1).expand(3, -1).clone()


def vision_positions(start: int, grid: Sequence[int]) -> torch.Tensor:
    """T x H x W grid in row-major (t, h, w) order, each axis offset by ``start``.

    TF/models/cosmos3_omni/modeling_cosmos3_omni.py:124-174 (merge sizes 1,
    time_interval 1).
    """
    T, H, W = grid
    t = torch.arange(T, dtype=torch.long) + start
    h = torch.arange(H, dtype=torch.long) + start
    w = torch.arange(W, dtype=torch.long) + start
    tg, hg, wg = torch.meshgrid(t, h, w, indexing="ij")
    return torch.stack([tg, hg, wg], 0).reshape(3, -1)


def joint_positions(segments: Sequence[Tuple[str, object]]) -> torch.Tensor:
    """Positions of a joint sequence of ("text", n) / ("video", (T,H,W)) / ("audio", n) / ("action", n) runs.

    Offsets advance by the run length after a 1-D run and by max(H, W) after a
    grid (TF/models/cosmos3_omni/modeling_cosmos3_omni.py:241-259).  Audio and
    action tokens are 1-D runs like text (a choice; parity unpinned).
    """
    pos, cur = [], 0
    for kind, spec in segments:
        if kind in ("text", "audio", "action"):
            pos.append(text_positions(cur, int(spec)))
            cur += int(spec)
        elif kind == "video":
            pos.append(vision_positions(cur, spec))
            cur += max(spec[1], spec[2])
        else:
            raise ValueError(kind)
    return torch.cat(pos, dim=1)


def mrope_cos_sin(pos: torch.Tensor, head_dim: int, sections: Sequence[int], base: float = 10000.0,
                  layout: str = "chunked") -> Tuple[torch.Tensor, torch.Tensor]:
    """cos/sin tables [N, head_dim/2]: angle_i = pos[axis(i)] * base^(-2i/head_dim).

    inv_freq in fp32 as TF/models/qwen3_vl/modeling_qwen3_vl.py:337-338; the
    product position*inv_freq in fp32 as :362-364.
    """
    half = head_dim // 2
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    amap = mrope_axis_map(head_dim, sections, layout)
    p = pos.to(torch.float32)[amap, :].t()          # [N, half]
    ang = p * inv_freq.view(1, half)
    return ang.cos(), ang.sin()


def apply_mrope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate-half RoPE on x[N, H, dh] with tables [N, dh/2].

    x'_i = x_i cos_i - x_{i+h} sin_i ; x'_{i+h} = x_{i+h} cos_i + x_i sin_i
    (TF/models/qwen3_vl/modeling_qwen3_vl.py:138-142 and :430-434 with
    cos = cat(c, c), sin = cat(s, s)).
    """
    x = x.to(torch.float32)
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    c, s = cos.unsqueeze(1), sin.unsqueeze(1)
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)


# --------------------------------------------------------------------------
# attention
# --------------------------------------------------------------------------
def hybrid_kv_end(n_tokens: int, causal_prefix: int, device=None) -> torch.Tensor:
    """Per-query key limit of the hybrid mask (architecture figure, right panel; REF/README.md:74): the first
    ``causal_prefix`` tokens (the AR / text run) see keys 0..i (causal, and no generator keys), all later tokens
    (DM, full attention) see every key.  Query i sees key j iff j < kv_end[i]."""
    i = torch.arange(n_tokens, device=device)
    return torch.where(i < causal_prefix, i + 1, torch.full_like(i, n_tokens))


def attention_rows(q_rows: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                   kv_end: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Exact attention for a subset of query rows: q_rows[R,H,dh], k,v[N,Hkv,dh] -> [R,H,dh].
    Hkv divides H: query head h uses K/V head h // (H/Hkv) (grouped-query attention, repeat_kv:
    TF/models/qwen3_vl/modeling_qwen3_vl.py:159-168,181-182).

    softmax(q k^T / sqrt(dh)) v, fp32 softmax
    (TF/models/qwen3_vl/modeling_qwen3_vl.py:171-193; non-causal full
    attention for DM tokens per REF/README.md:74).  ``kv_end[R]``: row r sees
    keys j < kv_end[r] only (additive -inf mask ahead of the softmax, as the
    eager form does with its attention_mask, TF/...modeling_qwen3_vl.py:185-186).
    """
    q = q_rows.to(torch.float32).transpose(0, 1).contiguous()   # [H,R,dh]
    kk, vv = _kv_heads(k, q.shape[0]), _kv_heads(v, q.shape[0])   # [H,N,dh]
    s = torch.matmul(q, kk.transpose(1, 2)) * (1.0 / math.sqrt(q.shape[-1]))
    if kv_end is not None:
        hidden = torch.arange(k.shape[0], device=k.device).view(1, 1, -1) >= kv_end.view(1, -1, 1)
        s = s.masked_fill(hidden, float("-inf"))
    p = torch.softmax(s, dim=-1, dtype=torch.float32)
    return torch.matmul(p, vv).transpose(0, 1).contiguous()


def _kv_heads(t: torch.Tensor, n_heads: int) -> torch.Tensor:
    """k or v [N,Hkv,dh] -> [H,N,dh] fp32 with every K/V head repeated H/Hkv times in place (repeat_kv)."""
    t = t.to(torch.float32).transpose(0, 1).contiguous()
    if t.shape[0] == n_heads:
        return t
    if n_heads % t.shape[0]:
        raise ValueError("number of K/V heads must divide the number of query heads")
    return t.repeat_interleave(n_heads // t.shape[0], dim=0)


def attention(q, k, v, chunk: int = 1024, kv_end: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention, chunked over query rows so scores are never all resident; ``kv_end`` and grouped K/V heads as
    in attention_rows."""
    kk, vv = _kv_heads(k, q.shape[1]), _kv_heads(v, q.shape[1])
    scale = 1.0 / math.sqrt(q.shape[-1])
    out = []
    for i in range(0, q.shape[0], chunk):
        qq = q[i:i + chunk].to(torch.float32).transpose(0, 1).contiguous()
        s = torch.matmul(qq, kk.transpose(1, 2)) * scale
        if kv_end is not None:
            hidden = torch.arange(k.shape[0], device=k.device).view(1, 1, -1) >= kv_end[i:i + chunk].view(1, -1, 1)
            s = s.masked_fill(hidden, float("-inf"))
        p = torch.softmax(s, dim=-1, dtype=torch.float32)
        out.append(torch.matmul(p, vv).transpose(0, 1))
    return torch.cat(out, 0).contiguous()


# --------------------------------------------------------------------------
# MLP
# --------------------------------------------------------------------------
def swiglu(y, wg, wu, wd) -> torch.Tensor:
    """down(silu(gate(y)) * up(y)), no bias. TF/models/qwen3_vl/modeling_qwen3_vl.py:510-523."""
    y = y.to(torch.float32)
    return (torch.nn.functional.silu(y @ wg.t()) * (y @ wu.t())) @ wd.t()


# --------------------------------------------------------------------------
# fp8 e4m3 (OCP "fn", max 448) emulation
# --------------------------------------------------------------------------
def _e4m3_round(x: torch.Tensor) -> torch.Tensor:
    return x.clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn).to(torch.float32)


def quant_e4m3_rows(a: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row dynamic quantisation: s = absmax/448 (0 -> 1), q = e4m3(a / s). Returns (q as fp32, s)."""
    a = a.to(torch.float32)
    s = a.abs().amax(dim=-1, keepdim=True) / E4M3_MAX
    s = torch.where(s == 0, torch.ones_like(s), s)
    return _e4m3_round(a / s), s


def quant_e4m3_weight(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-output-channel weight quantisation for W[out, in]."""
    return quant_e4m3_rows(w)


def fp8_linear(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """C_ij = s_a[i] s_w[j] sum_k A_q[i,k] W_q[j,k] with fp32 accumulation."""
    aq, sa = quant_e4m3_rows(a)
    wq, sw = quant_e4m3_weight(w)
    return (aq @ wq.t()) * sa * sw.t()


# --------------------------------------------------------------------------
# block / stack
# --------------------------------------------------------------------------
Segment = Tuple[int, int, int, bool]   # (start, length, weight_set, modulated)


def _linear(a, w, fp8):
    return fp8_linear(a, w) if fp8 else a.to(torch.float32) @ w.to(torch.float32).t()


def dm_block(x: torch.Tensor, weight_sets: Sequence[Dict[str, torch.Tensor]],
             mod: Optional[Sequence[torch.Tensor]], cos: torch.Tensor, sin: torch.Tensor,
             n_heads: int, segments: Optional[Sequence[Segment]] = None, eps: float = 1e-6,
             fp8: bool = False, attn_rows: Optional[torch.Tensor] = None, causal_prefix: int = 0) -> torch.Tensor:
    """One Mixture-of-Transformers layer over x[N, d].  ``causal_prefix`` > 0 selects the hybrid mask
    (hybrid_kv_end) for the shared attention.

    per-branch norm -> per-branch QKV -> mRoPE -> ONE shared full attention
    over all N tokens -> per-branch out-proj, gated residual -> per-branch norm
    -> per-branch SwiGLU, gated residual (REF/README.md:74; pre-norm residual
    order as TF/models/qwen3_vl/modeling_qwen3_vl.py:548-567).
    ``segments`` lists contiguous (start, len, weight_set, modulated) runs; a
    non-modulated run uses plain RMSNorm and gate 1 (the AR/text branch).
    ``mod`` = (shift1, scale1, gate1, shift2, scale2, gate2), each [d].
    Each weight set: norm1_w, wq, wk, wv, wo, norm2_w, wg, wu, wd ([out, in]);
    optional norm_q_w / norm_k_w [dh] switch on the per-head QK-RMSNorm.  wk / wv
    may have fewer rows than wq (n_kv_heads * dh: grouped-query attention).
    ``attn_rows``: optional index tensor; if given only those token rows are
    carried past attention (exact for those rows) and [R, d] is returned.
    """
    x = x.to(torch.float32)
    N, d = x.shape
    dh = d // n_heads
    if segments is None:
        segments = [(0, N, 0, mod is not None)]
    dkv = weight_sets[segments[0][2]]["wk"].shape[0]
    n_kv = dkv // dh
    dev = x.device
    q = torch.empty(N, d, device=dev); k = torch.empty(N, dkv, device=dev); v = torch.empty(N, dkv, device=dev)
    for (s0, ln, ws, modulated) in segments:
        p = weight_sets[ws]
        sl = slice(s0, s0 + ln)
        sh, sc = (mod[0], mod[1]) if modulated else (None, None)
        y = adaln_rms_norm(x[sl], p["norm1_w"], sh, sc, eps)
        q[sl] = _linear(y, p["wq"], fp8); k[sl] = _linear(y, p["wk"], fp8); v[sl] = _linear(y, p["wv"], fp8)
        if "norm_q_w" in p:   # per-head QK-RMSNorm (TF/models/qwen3_vl/modeling_qwen3_vl.py:463-466,479-480)
            q[sl] = rms_norm(q[sl].view(ln, n_heads, dh), p["norm_q_w"], eps).reshape(ln, d)
            k[sl] = rms_norm(k[sl].view(ln, n_kv, dh), p["norm_k_w"], eps).reshape(ln, dkv)
    q = apply_mrope(q.view(N, n_heads, dh), cos, sin)
    k = apply_mrope(k.view(N, n_kv, dh), cos, sin)
    v = v.view(N, n_kv, dh)
    kv_end = hybrid_kv_end(N, causal_prefix, dev) if causal_prefix else None
    if attn_rows is None:
        o = attention(q, k, v, kv_end=kv_end).reshape(N, d)
        rows = torch.arange(N, device=dev)
    else:
        rows = attn_rows.to(dev)
        o = attention_rows(q[rows], k, v, kv_end[rows] if kv_end is not None else None).reshape(-1, d)
    xr = x[rows]
    out = torch.empty_like(xr)
    for (s0, ln, ws, modulated) in segments:
        p = weight_sets[ws]
        m = (rows >= s0) & (rows < s0 + ln)
        if not bool(m.any()):
            continue
        xs = xr[m]
        a = _linear(o[m], p["wo"], fp8)
        xs = xs + (mod[2].to(torch.float32) * a if modulated else a)
        sh, sc = (mod[3], mod[4]) if modulated else (None, None)
        y2 = adaln_rms_norm(xs, p["norm2_w"], sh, sc, eps)
        if fp8:
            u = torch.nn.functional.silu(fp8_linear(y2, p["wg"])) * fp8_linear(y2, p["wu"])
            f = fp8_linear(u, p["wd"])
        else:
            f = swiglu(y2, p["wg"].float(), p["wu"].float(), p["wd"].float())
        out[m] = xs + (mod[5].to(torch.float32) * f if modulated else f)
    return out


def dm_stack(x, blocks: Sequence[Sequence[Dict[str, torch.Tensor]]], mods: Sequence[Optional[Sequence[torch.Tensor]]],
             cos, sin, n_heads: int, segments: Optional[Sequence[Segment]] = None, eps: float = 1e-6,
             fp8: bool = False, causal_prefix: int = 0) -> torch.Tensor:
    """L blocks in sequence; ``blocks[l]`` is the list of weight sets of layer l, ``mods[l]`` its modulation."""
    for ws, m in zip(blocks, mods):
        x = dm_block(x, ws, m, cos, sin, n_heads, segments, eps, fp8, causal_prefix=causal_prefix)
    return x


# --------------------------------------------------------------------------
# error measures used by every parity test
# --------------------------------------------------------------------------
def cfg_step(x, v_cond, v_uncond, guidance: float, coef: Sequence[float], hist: Sequence[torch.Tensor] = ()):
    """Guidance combine + linear scheduler update, fp32:
        v = v_uncond + guidance (v_cond - v_uncond)        (v = v_cond without v_uncond)
        out = coef[0] x + coef[1] v + sum_i coef[2+i] hist[i]
    Returns (out, v).  The reference sets guidance_scale and a flow-shifted multistep scheduler at its call site
    (README.md:247,258); the combine is the standard classifier-free-guidance formula, and every linear multistep
    scheduler update has this form once its scalar coefficients are known.  Pinned by closed forms only
    (guidance 1 -> v_cond, guidance 0 -> v_uncond, linearity)."""
    vc = v_cond.to(torch.float32)
    v = vc if v_uncond is None else v_uncond.to(torch.float32) + guidance * (vc - v_uncond.to(torch.float32))
    out = coef[0] * x.to(torch.float32) + coef[1] * v
    for c, h in zip(coef[2:], hist):
        out = out + c * h.to(torch.float32)
    return out, v


def flow_sigmas(num_steps: int, flow_shift: float = 1.0) -> torch.Tensor:
    """Flow-matching noise levels 1 -> 0 in ``num_steps`` steps with the time shift
    sigma' = shift sigma / (1 + (shift - 1) sigma)  (the ``flow_shift`` of README.md:247); float64."""
    s = torch.linspace(1.0, 0.0, num_steps + 1, dtype=torch.float64)
    return flow_shift * s / (1.0 + (flow_shift - 1.0) * s)


def max_rel_err(a: torch.Tensor, b: torch.Tensor) -> float:
    """max|a-b| / max|b| over the whole tensor (b = oracle)."""
    a = a.detach().to(torch.float64).cpu(); b = b.detach().to(torch.float64).cpu()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


def cos_sim(a: torch.Tensor, b: torch.Tensor) -> float:
    a = a.detach().to(torch.float64).cpu().reshape(-1); b = b.detach().to(torch.float64).cpu().reshape(-1)
    return float((a @ b) / (a.norm() * b.norm()).clamp_min(1e-30))
