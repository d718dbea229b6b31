"""Diffusers-style host side of the Cosmos 3 generator (DM) block: transformer stack -> block ->
attention module -> pluggable attention processor, all of whose tensor work runs in the HIP library.

Calling idiom mirrored (NVIDIA/cosmos README.md:238-263 drives it through the diffusers pipeline):
    stack(hidden_states, timestep, encoder_hidden_states) -> for block in blocks: block(...)
    block: per-branch adaLN-RMSNorm -> attn.processor(attn, ...) -> gated residual ->
           per-branch adaLN-RMSNorm -> per-branch SwiGLU -> gated residual          (README.md:74)
Per-branch ("Mixture-of-Transformers") weights: branch b of a layer owns
    attn.qkv_weight[b]  rows [0,d) | [d,2d) | [2d,3d) = add_q_proj | add_k_proj | add_v_proj (DM) or to_q | to_k | to_v (AR)
    attn.out_weight[b]  = to_add_out (DM) / to_out (AR)
    norm1_weight[b], norm2_weight[b], gate_weight[b], up_weight[b], down_weight[b] = the branch's norms and MLP
(parameter names as in transformers models/cosmos3_omni/modeling_cosmos3_omni.py:39-60).
Only timestep conditioning (a one-row MLP) is left to torch ops.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch
from torch import nn

from . import ops, rotary
from .config import DMConfig

Segment = rotary.Segment


def _as2d(t: torch.Tensor) -> torch.Tensor:
    if t.dim() == 3:
        if t.shape[0] != 1:
            raise NotImplementedError("batch size must be 1 (one joint sequence per forward)")
        return t[0]
    return t


def _batch_size(t: Optional[torch.Tensor], batched_dim: int) -> int:
    return t.shape[0] if t is not None and t.dim() == batched_dim else 1


def _sample(t: Optional[torch.Tensor], b: int, batched_dim: int, batch: int) -> Optional[torch.Tensor]:
    """Entry b of a batched argument (kept batched, size 1); an argument of batch size 1 is shared by all samples."""
    if t is None or t.dim() != batched_dim or t.shape[0] == 1:
        return t
    if t.shape[0] != batch:
        raise ValueError(f"batch size mismatch: {t.shape[0]} vs {batch}")
    return t[b:b + 1]


def _over_batch(fn, batch: int, return_dict: bool):
    """Run fn(b) for every sample and join the results (tuples or dicts of tensors / None) along the batch axis.  The
    joint sequence of a forward is ONE sample (attention spans it), so a batch is a loop, e.g. the conditional and the
    unconditional pass of classifier-free guidance given as a batch of two."""
    outs = [fn(b) for b in range(batch)]
    # per-sample results carry a leading batch axis of size 1, except the 2-D joint sequence of the stack's dict form
    cat = lambda xs: None if xs[0] is None else (torch.cat(xs, 0) if xs[0].dim() >= 3 else torch.stack(xs, 0))
    if isinstance(outs[0], dict):
        return {k: cat([o[k] for o in outs]) for k in outs[0]}
    return tuple(cat([o[i] for o in outs]) for i in range(len(outs[0])))


class Workspace:
    """Caller-owned scratch tensors of one (n_tokens, d, hidden) shape, reused by every block."""

    def __init__(self, n: int, d: int, hidden: int, n_heads: int, head_dim: int, device,
                 n_kv_heads: Optional[int] = None, fp8: bool = False):
        bf = dict(dtype=torch.bfloat16, device=device)
        n_kv_heads = n_heads if n_kv_heads is None else n_kv_heads
        self.n, self.d, self.hidden, self.fp8 = n, d, hidden, fp8
        if fp8:     # e4m3 operands of the four linears and their per-token scales
            q8, f32 = dict(dtype=ops.FP8_DTYPE, device=device), dict(dtype=torch.float32, device=device)
            self.yq, self.ys = torch.empty((n, d), **q8), torch.empty((n,), **f32)
            self.oq, self.os = torch.empty((n, d), **q8), torch.empty((n,), **f32)
            self.hq, self.hs = torch.empty((n, hidden), **q8), torch.empty((n,), **f32)
            # partial row maxima the producing kernels leave for the quantisers: per head (attention output) and per 64
            # columns (SwiGLU hidden)
            self.o_amax = torch.empty((n, n_heads), **f32)
            self.h_amax = torch.empty((n, (hidden + 63) // 64), **f32)
        self.y = torch.empty((n, d), **bf)
        self.qkv = torch.empty((n, d + 2 * n_kv_heads * head_dim), **bf)       # [Q | K | V] columns
        self.attn_out = torch.empty((n, d), **bf)
        self.h = torch.empty((n, hidden), **bf)
        # K / V tile images, then the scratch with which the attention kernel splits its last round of workgroups
        self.attn_ws = torch.empty((ops.attn_workspace_total_bytes(n, n_heads, n_kv_heads, head_dim),), dtype=torch.uint8,
                                   device=device)

    def fits(self, n: int, d: int, hidden: int, fp8: bool = False) -> bool:
        return (self.n, self.d, self.hidden) == (n, d, hidden) and (self.fp8 or not fp8)


class DMAttnProcessor:
    """Attention processor: per-branch QKV projection, rotate-half mRoPE, ONE shared full attention over the joint
    sequence, per-branch output projection (optionally fused with the gated residual).

    ``rope`` selects where mRoPE is applied: "in_attention" (default: in registers, to K while it is re-tiled for
    the attention kernel and to Q when that kernel loads it - no extra pass over memory), "gemm_epilogue" (on the
    fp32 accumulators of the QKV GEMM) or "streaming" (the in-place kernel after a plain QKV GEMM).
    ``fuse_kv_pack`` (with "in_attention"): the QKV GEMM writes K and V straight into the attention kernel's tile
    images instead of rows that a second kernel re-tiles; taken where the layout allows it (head_dim 128, or 64 with
    even head counts; every token segment starting on a multiple of 64), the two-kernel form otherwise.
    """

    def __init__(self, rope: str = "in_attention", fuse_kv_pack: bool = True):
        if rope not in ("in_attention", "gemm_epilogue", "streaming"):
            raise ValueError(f"unknown rope placement {rope!r}")
        self.rope = rope
        self.fuse_kv_pack = bool(fuse_kv_pack)

    def __call__(self, attn: "DMAttention", hidden_states: torch.Tensor,
                 encoder_hidden_states: Optional[torch.Tensor] = None, attention_mask: Optional[torch.Tensor] = None,
                 image_rotary_emb: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, *,
                 modality_segments: Optional[Sequence[Segment]] = None, residual: Optional[torch.Tensor] = None,
                 gate: Optional[torch.Tensor] = None, quant_scale: Optional[torch.Tensor] = None,
                 workspace: Optional[Workspace] = None, causal_prefix: int = 0, prefix=None,
                 kv_images: Optional[torch.Tensor] = None):
        """``causal_prefix`` = P selects the hybrid mask (the first P tokens, the AR run, causal among themselves and
        blind to the rest); ``prefix`` = (images, n_tokens) prepends keys packed by an earlier call; ``kv_images``
        is the buffer this call packs its own K/V into (kept by the caller when it wants to reuse them)."""
        if attention_mask is not None:
            raise NotImplementedError("masks are selected with causal_prefix; attention_mask must be None")
        if not isinstance(attn, _AttentionCore):
            attn = adopt_attention(attn)      # a diffusers-style attention module: fused views, built once
        if image_rotary_emb is None:
            raise ValueError("image_rotary_emb=(cos, sin) is required")
        batched = hidden_states.dim() == 3
        x = _as2d(hidden_states)
        n_enc = 0
        if encoder_hidden_states is not None:
            # diffusers joint-attention convention: context tokens first, then the latent tokens
            if quant_scale is not None or residual is not None:
                raise NotImplementedError("encoder_hidden_states cannot be combined with fused residual / fp8 input")
            enc = _as2d(encoder_hidden_states)
            n_enc = enc.shape[0]
            x = torch.cat([enc, x], dim=0)
            if modality_segments is None:
                dm = min(1, attn.n_branches - 1)      # branch 0 serves the context tokens
                modality_segments = [(0, n_enc, 0, False), (n_enc, x.shape[0] - n_enc, dm, True)]
        n, d = x.shape[0], attn.d_model
        if modality_segments is None:
            modality_segments = [(0, n, 0, True)]
        cos, sin = image_rotary_emb
        ws = workspace
        dkv = attn.n_kv_heads * attn.head_dim
        qkv = ws.qkv if ws is not None else torch.empty((n, d + 2 * dkv), dtype=torch.bfloat16, device=x.device)
        if qkv.shape[1] != d + 2 * dkv:
            raise ValueError("workspace was made for another number of K/V heads")
        o = ws.attn_out if ws is not None else torch.empty((n, d), dtype=torch.bfloat16, device=x.device)

        wsb = kv_images if kv_images is not None else (ws.attn_ws if ws is not None else None)
        mask_kw = dict(causal_prefix=causal_prefix, prefix=prefix, n_kv_heads=attn.n_kv_heads)
        q, k, v = qkv[:, :d], qkv[:, d:d + dkv], qkv[:, d + dkv:]
        qkn = attn.qk_norm_args(modality_segments)
        o_amax = None      # per-head maxima of the attention output rows, where the attention kernel leaves them
        if qkn is not None and self.rope != "in_attention":
            raise NotImplementedError("QK-RMSNorm precedes the rotation: it needs rope='in_attention'")
        if self.rope == "gemm_epilogue":
            attn._linear(x, quant_scale, "qkv", modality_segments, out=qkv, epilogue="rope_qk", cos=cos, sin=sin,
                         rope_cols=d + dkv, head_dim=attn.head_dim)
            ops.attention(q, k, v, attn.n_heads, attn.head_dim, out=o, workspace=wsb, **mask_kw)
        elif (self.rope == "in_attention" and self.fuse_kv_pack
              and ops.qkv_pack_applies([(s0, ln) for (s0, ln, _, _) in modality_segments], attn.head_dim, attn.n_heads,
                                       attn.n_kv_heads)):
            if wsb is None:
                wsb = torch.empty((ops.attn_workspace_total_bytes(n, attn.n_heads, attn.n_kv_heads, attn.head_dim),),
                                  dtype=torch.uint8, device=x.device)
            attn._qkv_pack(x, quant_scale, modality_segments, qkv, wsb, cos, sin, qkn)
            o_amax = ws.o_amax if (attn.fp8 and ws is not None and ws.fp8) else None
            ops.attention_packed(q, wsb, attn.n_heads, attn.head_dim, o, cos, sin, qkn, prefix, causal_prefix,
                                 attn.n_kv_heads, row_amax=o_amax)
        else:
            attn._linear(x, quant_scale, "qkv", modality_segments, out=qkv, epilogue="none")
            if self.rope == "streaming":
                if attn.n_kv_heads == attn.n_heads:
                    ops.mrope_qk_(q, k, cos, sin, attn.n_heads, attn.head_dim)
                else:
                    ops.mrope_qk_(q, None, cos, sin, attn.n_heads, attn.head_dim)
                    ops.mrope_qk_(k, None, cos, sin, attn.n_kv_heads, attn.head_dim)
                ops.attention(q, k, v, attn.n_heads, attn.head_dim, out=o, workspace=wsb, **mask_kw)
            else:     # in registers, inside the attention kernels
                ops.attention(q, k, v, attn.n_heads, attn.head_dim, out=o, workspace=wsb, cos=cos, sin=sin,
                              qk_norm=qkn, **mask_kw)
        if attn.fp8 and o_amax is not None:
            oq, so = ops.quant_rows_from_parts(o, o_amax, ws.oq, ws.os)
        elif attn.fp8:
            oq, so = ops.quant_rows(o, ws.oq, ws.os) if ws is not None and ws.fp8 else ops.quant_rows(o)
        else:
            oq, so = o, None
        if residual is not None:
            res = _as2d(residual)
            gates = [gate if modulated else None for (_, _, _, modulated) in modality_segments]
            attn._linear(oq, so, "out", modality_segments, out=res, epilogue="gate_residual", residual=res,
                         gates=gates)
            return residual
        out = torch.empty((n, d), dtype=torch.bfloat16, device=x.device)
        attn._linear(oq, so, "out", modality_segments, out=out, epilogue="none")
        if encoder_hidden_states is not None:
            h, e = out[n_enc:], out[:n_enc]
            return (h.unsqueeze(0), e.unsqueeze(0)) if batched else (h, e)
        return out.unsqueeze(0) if batched else out


class _AttentionCore:
    """What the processor needs of an attention module: geometry (d_model, n_heads, n_kv_heads, head_dim, n_branches),
    per-branch fused QKV / output weights (``qkv_weight[b]``, ``out_weight[b]``), optional per-branch QK-RMSNorm rows
    (``norm_q_weight`` / ``norm_k_weight`` [n_branches, head_dim] fp32) and optional e4m3 copies (``_q``)."""

    def _weights(self, which: str):
        return self.qkv_weight if which == "qkv" else self.out_weight

    def quantize_(self) -> None:
        """Offline per-output-channel e4m3 quantisation of this module's weights (fp8 variant)."""
        self._q["qkv"] = [ops.quant_rows(_data(w)) for w in self.qkv_weight]
        self._q["out"] = [ops.quant_rows(_data(w)) for w in self.out_weight]

    def qk_norm_args(self, segments: Sequence[Segment]):
        """(q_weight, k_weight, seg_ends, eps) for ``ops.attention``: one weight row per token segment."""
        if not self.qk_norm:
            return None
        branches = [b for (_, _, b, _) in segments]
        ends = [s0 + ln for (s0, ln, _, _) in segments]
        qw, kw = _data(self.norm_q_weight), _data(self.norm_k_weight)
        if branches != list(range(self.n_branches)):
            # the index tensor is made once per segment layout: a later call may run under graph capture, where a
            # host-to-device copy is not allowed
            cache = self.__dict__.setdefault("_branch_idx", {})
            key = (tuple(branches), str(qw.device))
            if key not in cache:
                cache[key] = torch.tensor(branches, device=qw.device)
            qw, kw = qw.index_select(0, cache[key]).contiguous(), kw.index_select(0, cache[key]).contiguous()
        return qw, kw, ends, self.qk_eps

    def _linear(self, a: torch.Tensor, sa: Optional[torch.Tensor], which: str, segments: Sequence[Segment], *,
                out: torch.Tensor, epilogue: str, residual=None, gates=None, cos=None, sin=None, rope_cols=0,
                head_dim=0) -> None:
        _routed_linear(a, sa, self._weights(which), self._q.get(which) if self.fp8 else None, None, segments, out=out,
                       epilogue=epilogue, residual=residual, gates=gates, cos=cos, sin=sin, rope_cols=rope_cols,
                       head_dim=head_dim)

    def _qkv_pack(self, a: torch.Tensor, sa: Optional[torch.Tensor], segments: Sequence[Segment], qkv: torch.Tensor,
                  images: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, qk_norm=None) -> None:
        """QKV projection with K (normalised, rotated) and V written as the attention kernel's tile images; Q into
        qkv[:, :d]."""
        segl = [(s0, ln) for (s0, ln, _, _) in segments]
        if self.fp8:
            qw = self._q["qkv"]
            ws, sws = [qw[b][0] for (_, _, b, _) in segments], [qw[b][1] for (_, _, b, _) in segments]
        else:
            ws, sws = [_data(self.qkv_weight[b]) for (_, _, b, _) in segments], None
        ops.gemm_qkv_pack(a, sa if self.fp8 else None, ws, sws, segl, self.n_heads, self.n_kv_heads, self.head_dim,
                          qkv[:, :self.d_model], images, cos, sin, qk_norm)


def _data(t):
    return t.data if isinstance(t, nn.Parameter) else t


class AdoptedAttention(_AttentionCore):
    """The HIP path's view of a diffusers-style joint-attention module that carries the sub-module names of the
    reference's attention layers (transformers models/cosmos3_omni/modeling_cosmos3_omni.py:41-46): ``to_q / to_k /
    to_v / to_out[0]`` (AR branch: the context tokens, branch 0), ``add_q_proj / add_k_proj / add_v_proj /
    to_add_out`` (DM branch: the generator tokens, branch 1), optional ``norm_q / norm_k / norm_added_q /
    norm_added_k``.

    The three projections of a branch are concatenated ONCE into the fused ``[d + 2 d_kv, d]`` weight the QKV GEMM
    reads, and the module's own ``weight`` tensors are re-pointed at row ranges of that fused tensor: one copy of the
    weights stays alive, ``state_dict`` / ``load_state_dict`` / ``.to()`` of the module keep working on it (a
    ``load_state_dict`` writes through the views), and the separate originals are released."""

    def __init__(self, mod: nn.Module):
        lin = lambda m: m[0] if isinstance(m, (nn.ModuleList, nn.Sequential)) else m
        branches = [(mod.to_q, mod.to_k, mod.to_v, lin(mod.to_out))]
        if getattr(mod, "add_q_proj", None) is not None:
            branches.append((mod.add_q_proj, mod.add_k_proj, mod.add_v_proj, lin(mod.to_add_out)))
        wq = mod.to_q.weight
        if not wq.is_cuda or wq.dtype != torch.bfloat16:
            raise RuntimeError("the HIP path needs the attention module on the GPU in bfloat16 (pipe.to('cuda'), bf16)")
        self.d_model = wq.shape[1]
        heads = getattr(mod, "heads", None) or getattr(mod, "num_heads", None) or getattr(mod, "n_heads", None)
        if not heads:
            raise ValueError("cannot tell the number of heads of this attention module (no .heads attribute)")
        self.n_heads = int(heads)
        if wq.shape[0] != self.d_model or self.d_model % self.n_heads:
            raise ValueError("query projection must be square with a width divisible by the number of heads")
        self.head_dim = self.d_model // self.n_heads
        dkv = mod.to_k.weight.shape[0]
        if dkv % self.head_dim or self.n_heads % (dkv // self.head_dim):
            raise ValueError("K/V projection width does not give a whole number of heads that divides the query heads")
        self.n_kv_heads = dkv // self.head_dim
        self.n_branches, self.fp8, self._q = len(branches), False, {}
        self.qkv_weight, self.out_weight, self._views = [], [], []
        d = self.d_model
        for (q, k, v, o) in branches:
            for m in (q, k, v, o):
                if getattr(m, "bias", None) is not None:
                    raise NotImplementedError("projections with a bias are not supported by the fused kernels")
            if q.weight.shape != (d, d) or k.weight.shape != (dkv, d) or v.weight.shape != (dkv, d) or o.weight.shape != (d, d):
                raise ValueError("projection shapes do not match [d, d] / [d_kv, d] / [d_kv, d] / [d, d]")
            fused = torch.cat([q.weight.data, k.weight.data, v.weight.data], dim=0).contiguous()
            q.weight.data, k.weight.data, v.weight.data = fused[:d], fused[d:d + dkv], fused[d + dkv:]
            self.qkv_weight.append(fused)
            self.out_weight.append(o.weight.data if o.weight.data.is_contiguous() else o.weight.data.contiguous())
            self._views.append((q.weight, k.weight, v.weight, o.weight))
        nq = [getattr(mod, n, None) for n in ("norm_q", "norm_added_q")][:self.n_branches]
        nk = [getattr(mod, n, None) for n in ("norm_k", "norm_added_k")][:self.n_branches]
        self.qk_norm = all(m is not None and getattr(m, "weight", None) is not None for m in nq + nk)
        self.qk_eps = 1e-6
        if self.qk_norm:
            self._norm_mods = (nq, nk)
            self.qk_eps = float(getattr(nq[0], "eps", getattr(nq[0], "variance_epsilon", 1e-6)))
            self.norm_q_weight = torch.stack([m.weight.data.float() for m in nq]).contiguous()
            self.norm_k_weight = torch.stack([m.weight.data.float() for m in nk]).contiguous()
            self._norm_seen = [(m.weight.data_ptr(), m.weight._version) for m in nq + nk]

    def still_valid(self) -> bool:
        """False once some weight of the module has been replaced (a new tensor assigned, moved to another device)."""
        d, dkv = self.d_model, self.n_kv_heads * self.head_dim
        for fused, o, (q, k, v, ow) in zip(self.qkv_weight, self.out_weight, self._views):
            es = fused.element_size()
            if (q.data_ptr(), k.data_ptr(), v.data_ptr()) != (fused.data_ptr(), fused.data_ptr() + d * d * es,
                                                              fused.data_ptr() + (d + dkv) * d * es):
                return False
            if ow.data_ptr() != o.data_ptr() and ow.data.is_contiguous():
                return False
        if self.qk_norm:      # the fp32 norm rows are copies: rebuilt when a norm weight was replaced or written to
            nq, nk = self._norm_mods
            if [(m.weight.data_ptr(), m.weight._version) for m in nq + nk] != self._norm_seen:
                return False
        return True


def adopt_attention(mod: nn.Module) -> AdoptedAttention:
    """The cached ``AdoptedAttention`` of a diffusers-style attention module (built at the first call)."""
    ad = mod.__dict__.get("_cdm_adopted")
    if ad is None or not ad.still_valid():
        ad = AdoptedAttention(mod)
        mod.__dict__["_cdm_adopted"] = ad       # not a sub-module: the module's state_dict is unchanged
    return ad


class DMAttention(nn.Module, _AttentionCore):
    """Attention module of one MoT layer: per-branch projections around one shared attention."""

    def __init__(self, d_model: int, n_heads: int, head_dim: int, n_branches: int = 1, fp8: bool = False,
                 processor: Optional[DMAttnProcessor] = None, device=None, dtype=torch.bfloat16,
                 qk_norm: bool = False, eps: float = 1e-6, n_kv_heads: Optional[int] = None):
        super().__init__()
        if n_heads * head_dim != d_model:
            raise ValueError("n_heads * head_dim must equal d_model")
        n_kv_heads = n_heads if n_kv_heads is None else n_kv_heads
        if n_kv_heads < 1 or n_heads % n_kv_heads:
            raise ValueError("n_kv_heads must divide n_heads")
        self.d_model, self.n_heads, self.head_dim, self.n_branches, self.fp8 = d_model, n_heads, head_dim, n_branches, fp8
        self.n_kv_heads = n_kv_heads      # K / V heads (num_key_value_heads); fewer than n_heads = grouped-query attention
        kw = dict(device=device, dtype=dtype)
        # per-head QK-RMSNorm weights, one row per branch (norm_q / norm_added_q and norm_k / norm_added_k of the
        # reference's attention layer); fp32 because the kernels normalise in fp32
        self.qk_norm, self.qk_eps = qk_norm, eps
        if qk_norm:
            self.norm_q_weight = nn.Parameter(torch.ones(n_branches, head_dim, device=device, dtype=torch.float32),
                                              requires_grad=False)
            self.norm_k_weight = nn.Parameter(torch.ones(n_branches, head_dim, device=device, dtype=torch.float32),
                                              requires_grad=False)
        qkv_rows = d_model + 2 * n_kv_heads * head_dim            # rows [Wq | Wk | Wv]
        self.qkv_weight = nn.ParameterList([nn.Parameter(torch.empty(qkv_rows, d_model, **kw), requires_grad=False)
                                            for _ in range(n_branches)])
        self.out_weight = nn.ParameterList([nn.Parameter(torch.empty(d_model, d_model, **kw), requires_grad=False)
                                            for _ in range(n_branches)])
        self.processor = processor or DMAttnProcessor()
        self._q = {}     # fp8 copies: name -> list of (wq, sw)

    def set_processor(self, processor) -> None:
        self.processor = processor

    def forward(self, hidden_states, encoder_hidden_states=None, attention_mask=None, image_rotary_emb=None, **kw):
        return self.processor(self, hidden_states, encoder_hidden_states=encoder_hidden_states,
                              attention_mask=attention_mask, image_rotary_emb=image_rotary_emb, **kw)


def _routed_linear(a, sa, weights, qweights, weights2, segments, *, out, epilogue, residual=None, gates=None, cos=None,
                   sin=None, rope_cols=0, head_dim=0, qweights2=None, row_amax=None) -> None:
    """Per-modality linear over contiguous token segments: one grouped launch over all segments."""
    segl = [(s, l) for (s, l, _, _) in segments]
    if qweights is None:
        if len(segments) == 1:
            (s0, ln, b, _), = segments
            sl = slice(s0, s0 + ln)
            ops.gemm(a[sl], weights[b], w2=weights2[b] if weights2 is not None else None, epilogue=epilogue,
                     residual=residual[sl] if residual is not None else None, gate=gates[0] if gates is not None else None,
                     cos=cos[sl] if cos is not None else None, sin=sin[sl] if sin is not None else None,
                     rope_cols=rope_cols, head_dim=head_dim, out=out[sl])
            return
        ops.grouped_gemm(a, [weights[b] for (_, _, b, _) in segments], segl,
                         w2s=[weights2[b] for (_, _, b, _) in segments] if weights2 is not None else None,
                         epilogue=epilogue, residual=residual, gates=gates, cos=cos, sin=sin, rope_cols=rope_cols,
                         head_dim=head_dim, out=out)
        return
    ops.grouped_gemm_fp8(a, sa, [qweights[b][0] for (_, _, b, _) in segments], [qweights[b][1] for (_, _, b, _) in segments],
                         segl, w2qs=[qweights2[b][0] for (_, _, b, _) in segments] if qweights2 is not None else None,
                         sw2s=[qweights2[b][1] for (_, _, b, _) in segments] if qweights2 is not None else None,
                         epilogue=epilogue, residual=residual, gates=gates, cos=cos, sin=sin, rope_cols=rope_cols,
                         head_dim=head_dim, out=out, row_amax=row_amax)


class DMBlock(nn.Module):
    """One Mixture-of-Transformers layer (generator side)."""

    def __init__(self, d_model: int, n_heads: int, head_dim: int, hidden: int, n_branches: int = 1,
                 eps: float = 1e-6, fp8: bool = False, device=None, dtype=torch.bfloat16, qk_norm: bool = False,
                 n_kv_heads: Optional[int] = None):
        super().__init__()
        kw = dict(device=device, dtype=dtype)
        self.d_model, self.hidden, self.eps, self.fp8, self.n_branches = d_model, hidden, eps, fp8, n_branches
        self.attn = DMAttention(d_model, n_heads, head_dim, n_branches, fp8, device=device, dtype=dtype,
                                qk_norm=qk_norm, eps=eps, n_kv_heads=n_kv_heads)
        P = lambda *shape: nn.Parameter(torch.empty(*shape, **kw), requires_grad=False)
        self.norm1_weight = nn.ParameterList([P(d_model) for _ in range(n_branches)])
        self.norm2_weight = nn.ParameterList([P(d_model) for _ in range(n_branches)])
        self.gate_weight = nn.ParameterList([P(hidden, d_model) for _ in range(n_branches)])
        self.up_weight = nn.ParameterList([P(hidden, d_model) for _ in range(n_branches)])
        self.down_weight = nn.ParameterList([P(d_model, hidden) for _ in range(n_branches)])
        self.adaLN_modulation = nn.Linear(d_model, 6 * d_model, bias=True, **kw)
        self._q = {}
        self._ws: Optional[Workspace] = None

    @torch.no_grad()
    def reset_parameters(self, generator: Optional[torch.Generator] = None, std: float = 0.02) -> None:
        for name, p in self.named_parameters():
            if "norm" in name:
                p.fill_(1.0)
            elif name.endswith("bias"):
                p.zero_()
            else:
                p.copy_((torch.randn(p.shape, generator=generator, device=p.device, dtype=torch.float32) * std).to(p.dtype))
        if self.fp8:
            self.quantize_()

    def quantize_(self) -> None:
        self.attn.quantize_()
        for name, plist in (("gate", self.gate_weight), ("up", self.up_weight), ("down", self.down_weight)):
            self._q[name] = [ops.quant_rows(w.data) for w in plist]

    def modulation(self, temb: torch.Tensor) -> Tuple[torch.Tensor, ...]:
        """(shift1, scale1, gate1, shift2, scale2, gate2), each [d] fp32, from the conditioning vector."""
        c = temb.reshape(1, -1).to(self.adaLN_modulation.weight.dtype)
        m = self.adaLN_modulation(torch.nn.functional.silu(c)).float().reshape(-1)
        return tuple(t.contiguous() for t in m.chunk(6))

    def _norm(self, x, weights, shift, scale, segments, ws):
        """Per-branch adaLN-RMSNorm of x (bf16 or fp32) into the workspace: y (bf16), or (e4m3, per-token scale) for
        the fp8 variant."""
        if not self.fp8:
            y = ws.y
            for (s0, ln, b, modulated) in segments:
                ops.adaln_rmsnorm(x[s0:s0 + ln], weights[b], shift if modulated else None, scale if modulated else None,
                                  self.eps, out=y[s0:s0 + ln])
            return y, None
        yq, st = ws.yq, ws.ys
        for (s0, ln, b, modulated) in segments:
            ops.adaln_rmsnorm_quant(x[s0:s0 + ln], weights[b], shift if modulated else None,
                                    scale if modulated else None, self.eps, out_q=yq[s0:s0 + ln], out_s=st[s0:s0 + ln])
        return yq, st

    def forward(self, hidden_states: torch.Tensor, temb: torch.Tensor,
                image_rotary_emb: Tuple[torch.Tensor, torch.Tensor],
                modality_segments: Optional[Sequence[Segment]] = None, *, inplace: bool = False,
                modulation: Optional[Sequence[torch.Tensor]] = None, workspace: Optional[Workspace] = None,
                causal_prefix: int = 0, prefix=None, kv_images: Optional[torch.Tensor] = None):
        """``hidden_states`` [N, d] (or [1, N, d]) is the residual stream, bf16 or fp32; the result has its dtype (a
        stack keeps the stream in fp32 between blocks: only the operands of the matrix products are bf16)."""
        batched = hidden_states.dim() == 3
        x = _as2d(hidden_states)
        if not inplace:
            x = x.clone()
        n, d = x.shape
        segs = list(modality_segments) if modality_segments is not None else [(0, n, 0, True)]
        ws = workspace or self._ws
        if ws is None or not ws.fits(n, d, self.hidden, self.fp8) or ws.y.device != x.device:
            ws = Workspace(n, d, self.hidden, self.attn.n_heads, self.attn.head_dim, x.device, self.attn.n_kv_heads,
                           self.fp8)
            if workspace is None:
                self._ws = ws
        sh1, sc1, g1, sh2, sc2, g2 = modulation if modulation is not None else self.modulation(temb)

        y, sy = self._norm(x, self.norm1_weight, sh1, sc1, segs, ws)
        self.attn(y, image_rotary_emb=image_rotary_emb, modality_segments=segs, residual=x, gate=g1, quant_scale=sy,
                  workspace=ws, causal_prefix=causal_prefix, prefix=prefix, kv_images=kv_images)
        y, sy = self._norm(x, self.norm2_weight, sh2, sc2, segs, ws)
        q = self._q if self.fp8 else {}
        _routed_linear(y, sy, self.gate_weight, q.get("gate"), self.up_weight, segs, out=ws.h, epilogue="swiglu",
                       qweights2=q.get("up"), row_amax=ws.h_amax if self.fp8 else None)
        if self.fp8:      # the SwiGLU epilogue left the maxima of every 64 columns: the quantiser reads each row once
            hq, sh = ops.quant_rows_from_parts(ws.h, ws.h_amax, ws.hq, ws.hs)
        else:
            hq, sh = ws.h, None
        gates = [g2 if modulated else None for (_, _, _, modulated) in segs]
        _routed_linear(hq, sh, self.down_weight, q.get("down"), None, segs, out=x, epilogue="gate_residual",
                       residual=x, gates=gates)
        return x.unsqueeze(0) if batched else x


class TimestepEmbedder(nn.Module):
    """256-d sinusoidal embedding of t -> Linear -> SiLU -> Linear (stays in torch: a one-row MLP)."""

    def __init__(self, d_model: int, freq_dim: int = 256, device=None, dtype=torch.float32):
        super().__init__()
        self.freq_dim = freq_dim
        self.linear_1 = nn.Linear(freq_dim, d_model, device=device, dtype=dtype)
        self.linear_2 = nn.Linear(d_model, d_model, device=device, dtype=dtype)

    def sinusoid(self, t: torch.Tensor) -> torch.Tensor:
        half = self.freq_dim // 2
        k = torch.arange(half, dtype=torch.float32, device=t.device)
        f = torch.exp(-math.log(10000.0) * k / half)
        a = t.to(torch.float32).reshape(-1, 1) * f.reshape(1, -1)
        return torch.cat([a.cos(), a.sin()], dim=-1)

    def forward(self, t: torch.Tensor) -> torch.Tensor:
        e = self.sinusoid(t).to(self.linear_1.weight.dtype)
        return self.linear_2(torch.nn.functional.silu(self.linear_1(e)))


class ContextCache:
    """Per-layer K/V tile images of the text run (see ``DMStack.precompute_context``)."""

    def __init__(self, images: List[torch.Tensor], n_tokens: int):
        self.images, self.n_tokens = images, n_tokens


class DMStack(nn.Module):
    """L blocks over the joint sequence text | video | audio | action (diffusers transformer forward shape)."""

    def __init__(self, cfg: DMConfig, device=None, dtype=torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        self.time_embedder = TimestepEmbedder(cfg.d_model, device=device)
        self.blocks = nn.ModuleList([DMBlock(cfg.d_model, cfg.n_heads, cfg.head_dim, cfg.hidden, cfg.n_branches,
                                             cfg.eps, cfg.fp8, device=device, dtype=dtype, qk_norm=cfg.qk_norm,
                                             n_kv_heads=cfg.kv_heads)
                                     for _ in range(cfg.n_blocks)])
        self._rot = None
        self._ws: Optional[Workspace] = None
        self._rot_gen = None
        self._ws_gen: Optional[Workspace] = None

    @torch.no_grad()
    def reset_parameters(self, seed: Optional[int] = None) -> None:
        dev = next(self.parameters()).device
        g = torch.Generator(device=dev).manual_seed(self.cfg.seed if seed is None else seed)
        for p in self.time_embedder.parameters():
            if p.dim() == 2:
                p.copy_(torch.randn(p.shape, generator=g, device=dev) * 0.02)
            else:
                p.zero_()
        for b in self.blocks:
            b.reset_parameters(g)

    def segments(self) -> List[Segment]:
        """(start, len, branch, modulated): text uses branch 0 un-modulated; the generator's modalities - video, audio,
        action - are modulated.  Video uses the generator (DM) weight set, branch 1 of a multi-branch stack; action its
        own third set when there is one; audio its own fourth set when there is one, else the generator's."""
        c = self.cfg
        gen = 1 if c.n_branches > 1 else 0
        segs, s = [], 0
        if c.n_text:
            segs.append((s, c.n_text, 0, False)); s += c.n_text
        segs.append((s, c.n_video, gen, True)); s += c.n_video
        if c.n_audio:
            segs.append((s, c.n_audio, 3 if c.n_branches > 3 else gen, True)); s += c.n_audio
        if c.n_action:
            segs.append((s, c.n_action, min(2, c.n_branches - 1), True))
        return segs

    def rotary(self, device) -> Tuple[torch.Tensor, torch.Tensor]:
        if self._rot is None or self._rot[0].device != torch.device(device):
            c = self.cfg
            pos, _ = rotary.build_positions(c.n_text, c.grid, c.n_action, c.n_audio)
            self._rot = rotary.rotary_tables(pos, c.head_dim, c.mrope_sections, c.rope_base, c.rope_layout, device)
        return self._rot

    @torch.no_grad()
    def precompute_context(self, encoder_hidden_states: torch.Tensor) -> "ContextCache":
        """Under the hybrid mask the text run never sees a generator token and its branch is not modulated, so its
        keys and values in every layer depend on the prompt only.  Runs the text run alone (causal) through the stack
        once and keeps the per-layer K/V tile images; ``forward(..., context_cache=...)`` then carries only the
        generator tokens at every denoising step."""
        c = self.cfg
        if not c.hybrid_mask:
            raise RuntimeError("context reuse needs the hybrid mask (DMConfig.hybrid_mask)")
        if c.n_text == 0:
            raise ValueError("context reuse needs a text run")
        x = self._stream(_as2d(encoder_hidden_states))
        if x.shape != (c.n_text, c.d_model):
            raise ValueError(f"context has shape {tuple(x.shape)}, expected {(c.n_text, c.d_model)}")
        cos, sin = self.rotary(x.device)
        rot = (cos[:c.n_text].contiguous(), sin[:c.n_text].contiguous())
        segs = [(0, c.n_text, 0, False)]
        ws = Workspace(c.n_text, c.d_model, c.hidden, c.n_heads, c.head_dim, x.device, c.kv_heads, c.fp8)
        nbytes = ops.attn_workspace_bytes(c.n_text, c.kv_heads, c.head_dim)
        images = []
        for blk in self.blocks:
            img = torch.empty((nbytes,), dtype=torch.uint8, device=x.device)
            blk(x, None, rot, segs, inplace=True, workspace=ws, modulation=(None,) * 6, causal_prefix=c.n_text,
                kv_images=img)
            images.append(img)
        return ContextCache(images, c.n_text)

    @torch.no_grad()
    def forward(self, hidden_states: torch.Tensor, timestep: torch.Tensor,
                encoder_hidden_states: Optional[torch.Tensor] = None, action_states: Optional[torch.Tensor] = None,
                return_dict: bool = False, context_cache: Optional["ContextCache"] = None,
                audio_states: Optional[torch.Tensor] = None):
        c = self.cfg
        batch = _batch_size(hidden_states, 3)
        if batch > 1:
            ts = timestep.reshape(-1)
            return _over_batch(lambda b: self.forward(hidden_states[b:b + 1], ts[b:b + 1] if ts.numel() == batch else ts,
                                                      _sample(encoder_hidden_states, b, 3, batch),
                                                      _sample(action_states, b, 3, batch), return_dict, context_cache,
                                                      _sample(audio_states, b, 3, batch)),
                               batch, return_dict)
        if context_cache is not None:
            return self._forward_cached(hidden_states, timestep, action_states, return_dict, context_cache, audio_states)
        parts = []
        if c.n_text:
            if encoder_hidden_states is None:
                raise ValueError("this configuration expects encoder_hidden_states (text context)")
            parts.append(_as2d(encoder_hidden_states))
        parts.append(_as2d(hidden_states))
        parts += self._generator_extras(audio_states, action_states)
        x = self._stream(torch.cat(parts, dim=0) if len(parts) > 1 else parts[0])
        if x.shape != (c.n_tokens, c.d_model):
            raise ValueError(f"joint sequence has shape {tuple(x.shape)}, expected {(c.n_tokens, c.d_model)}")
        rot = self.rotary(x.device)
        segs = self.segments()
        temb = self.time_embedder(timestep.reshape(-1)[:1])
        if self._ws is None or not self._ws.fits(c.n_tokens, c.d_model, c.hidden, c.fp8) or self._ws.y.device != x.device:
            self._ws = Workspace(c.n_tokens, c.d_model, c.hidden, c.n_heads, c.head_dim, x.device, c.kv_heads, c.fp8)
        for blk in self.blocks:
            blk(x, temb, rot, segs, inplace=True, workspace=self._ws, causal_prefix=c.n_text if c.hybrid_mask else 0)
        return self._result(x, c.n_text, hidden_states.dim() == 3, return_dict)

    def capture(self, hidden_states: torch.Tensor, timestep: torch.Tensor,
                encoder_hidden_states: Optional[torch.Tensor] = None, action_states: Optional[torch.Tensor] = None,
                audio_states: Optional[torch.Tensor] = None, context_cache: Optional["ContextCache"] = None) -> "GraphedStack":
        """Record one forward (batch 1) on inputs of these shapes into a HIP graph and return the replayer: for
        launch-bound shapes (a few thousand tokens at small width: a dozen launches per block of microseconds each) a
        replay costs one launch instead of a dozen per block.  The kernels take every size from host arguments at
        capture time, so a graph serves exactly the shapes it was recorded with."""
        return GraphedStack(self, dict(hidden_states=hidden_states, timestep=timestep,
                                       encoder_hidden_states=encoder_hidden_states, action_states=action_states,
                                       audio_states=audio_states), context_cache)

    def _stream(self, x: torch.Tensor) -> torch.Tensor:
        """A private, contiguous copy of the joint sequence in the dtype the residual stream is kept in."""
        dt = torch.float32 if self.cfg.residual_fp32 else torch.bfloat16
        return x.to(dt).contiguous() if x.dtype != dt else x.contiguous().clone()

    def _result(self, x: torch.Tensor, first_video: int, batched: bool, return_dict: bool):
        """The video rows of the final stream as bf16 (the transformer's output dtype); "joint" is the stream itself."""
        video = x[first_video:first_video + self.cfg.n_video].to(torch.bfloat16)
        out = video.unsqueeze(0) if batched else video
        if return_dict:
            return {"sample": out, "joint": x}
        return (out,)


    def _generator_extras(self, audio_states, action_states) -> List[torch.Tensor]:
        """The audio and action runs that follow the video tokens in the joint sequence."""
        c, parts = self.cfg, []
        for n, t, name in ((c.n_audio, audio_states, "audio_states"), (c.n_action, action_states, "action_states")):
            if n:
                if t is None:
                    raise ValueError(f"this configuration expects {name}")
                parts.append(_as2d(t))
        return parts

    def _forward_cached(self, hidden_states, timestep, action_states, return_dict, cache: "ContextCache",
                        audio_states=None):
        c = self.cfg
        P = c.n_text
        if cache.n_tokens != P or len(cache.images) != len(self.blocks):
            raise ValueError("context cache does not belong to this stack")
        parts = [_as2d(hidden_states)] + self._generator_extras(audio_states, action_states)
        x = self._stream(torch.cat(parts, dim=0) if len(parts) > 1 else parts[0])
        n = c.n_tokens - P
        if x.shape != (n, c.d_model):
            raise ValueError(f"generator sequence has shape {tuple(x.shape)}, expected {(n, c.d_model)}")
        if self._rot_gen is None or self._rot_gen[0].device != x.device:
            cos, sin = self.rotary(x.device)
            self._rot_gen = (cos[P:].contiguous(), sin[P:].contiguous())
        segs = [(s0 - P, ln, b, m) for (s0, ln, b, m) in self.segments() if s0 >= P]
        temb = self.time_embedder(timestep.reshape(-1)[:1])
        if self._ws_gen is None or not self._ws_gen.fits(n, c.d_model, c.hidden, c.fp8) or self._ws_gen.y.device != x.device:
            self._ws_gen = Workspace(n, c.d_model, c.hidden, c.n_heads, c.head_dim, x.device, c.kv_heads, c.fp8)
        for blk, img in zip(self.blocks, cache.images):
            blk(x, temb, self._rot_gen, segs, inplace=True, workspace=self._ws_gen, prefix=(img, P))
        return self._result(x, 0, hidden_states.dim() == 3, return_dict)


class GraphedStack:
    """A recorded ``DMStack.forward``: ``__call__`` copies the inputs into the recorded buffers, replays the graph and
    returns the recorded outputs ({"sample", "joint"}; overwritten by the next call).  Nothing inside the recording
    clears memory with a memset node or copies from pageable host memory; the stack's workspaces are the ones the
    eager path uses, so eager and recorded forwards of one stack must not overlap in time."""

    def __init__(self, stack: "DMStack", inputs: dict, context_cache: Optional["ContextCache"]):
        if _batch_size(inputs["hidden_states"], 3) != 1:
            raise NotImplementedError("a graph records one sample; run a batch as a loop over replays")
        dev = inputs["hidden_states"].device
        self.stack, self.cache = stack, context_cache
        self.static = {k: (v.to(dev).clone() if v is not None else None) for k, v in inputs.items()}
        side = torch.cuda.Stream(device=dev)            # default priority
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            for _ in range(2):                          # allocate workspaces, tables and library handles outside the graph
                self._run()
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.out = self._run()

    def _run(self):
        return self.stack(return_dict=True, context_cache=self.cache, **self.static)

    def __call__(self, hidden_states: torch.Tensor, timestep: torch.Tensor,
                 encoder_hidden_states: Optional[torch.Tensor] = None, action_states: Optional[torch.Tensor] = None,
                 audio_states: Optional[torch.Tensor] = None) -> dict:
        given = dict(hidden_states=hidden_states, timestep=timestep, encoder_hidden_states=encoder_hidden_states,
                     action_states=action_states, audio_states=audio_states)
        for k, v in given.items():
            dst = self.static[k]
            if (v is None) != (dst is None):
                raise ValueError(f"{k}: the graph was recorded {'with' if dst is not None else 'without'} it")
            if v is not None:
                if tuple(v.shape) != tuple(dst.shape):
                    raise ValueError(f"{k}: shape {tuple(v.shape)} differs from the recorded {tuple(dst.shape)}")
                dst.copy_(v)
        self.graph.replay()
        return self.out


def _edge_linear(lin: nn.Linear, x: torch.Tensor) -> torch.Tensor:
    """A narrow linear layer with bias at the edge of the stack (patchify / un-patchify, action and audio
    projections) through the HIP kernel made for it; ``lin`` only holds the parameters under their checkpoint names."""
    return ops.linear_bias(x if x.stride(-1) == 1 else x.contiguous(), lin.weight, lin.bias)


class DMTransformer(nn.Module):
    """The transformer-shaped object a diffusers pipeline drives (``pipe.transformer``): latents in, velocity out.

    Stack edges around ``DMStack``: patchify + ``proj_in``, the block stack, a final RMSNorm, ``proj_out`` +
    unpatchify; an optional action stream (``action_proj_in`` + ``action_modality_embed`` in, ``action_proj_out``
    out) and an optional audio stream (``audio_proj_in`` + ``audio_modality_embed`` in, ``audio_proj_out`` out: the
    sound the reference generates with ``enable_sound``, README.md:259).  The edge linears are one-off projections with
    K or N = patch width (64 for 16 latent channels and 1x2x2 patches), bound by moving the token rows once: they run
    through ``ops.linear_bias``; the ``nn.Linear`` modules only hold the parameters.  Parameter
    names follow the checkpoint keys the reference's model files attest (``proj_in``, ``proj_out``,
    ``time_embedder``, ``action_proj_in``, ``action_proj_out``, ``action_modality_embed``, ``audio_proj_in``,
    ``audio_proj_out``, ``audio_modality_embed``); the patch order
    (channel-major inside a patch) and the un-modulated final norm are this build's choices.
    """

    def __init__(self, cfg: DMConfig, latent_channels: int = 16, patch: Tuple[int, int, int] = (1, 2, 2),
                 action_dim: int = 0, audio_dim: int = 0, device=None, dtype=torch.bfloat16):
        super().__init__()
        self.cfg, self.latent_channels, self.patch, self.action_dim = cfg, latent_channels, tuple(patch), action_dim
        self.audio_dim = audio_dim
        pd = latent_channels * patch[0] * patch[1] * patch[2]
        self.stack = DMStack(cfg, device=device, dtype=dtype)
        self.proj_in = nn.Linear(pd, cfg.d_model, device=device, dtype=dtype)
        self.proj_out = nn.Linear(cfg.d_model, pd, device=device, dtype=dtype)
        self.norm_out = nn.Parameter(torch.ones(cfg.d_model, device=device, dtype=dtype), requires_grad=False)
        if cfg.n_action:
            if action_dim <= 0:
                raise ValueError("a configuration with action tokens needs action_dim")
            self.action_proj_in = nn.Linear(action_dim, cfg.d_model, device=device, dtype=dtype)
            self.action_proj_out = nn.Linear(cfg.d_model, action_dim, device=device, dtype=dtype)
            self.action_modality_embed = nn.Parameter(torch.zeros(cfg.d_model, device=device, dtype=dtype),
                                                      requires_grad=False)
        if cfg.n_audio:
            if audio_dim <= 0:
                raise ValueError("a configuration with audio tokens needs audio_dim")
            self.audio_proj_in = nn.Linear(audio_dim, cfg.d_model, device=device, dtype=dtype)
            self.audio_proj_out = nn.Linear(cfg.d_model, audio_dim, device=device, dtype=dtype)
            self.audio_modality_embed = nn.Parameter(torch.zeros(cfg.d_model, device=device, dtype=dtype),
                                                     requires_grad=False)
        for p in self.parameters():
            p.requires_grad_(False)

    def _streams(self):
        """(name, token count, in projection, out projection, embed) of the generator's 1-D side streams, in
        sequence order."""
        c, out = self.cfg, []
        if c.n_audio:
            out.append(("audio", c.n_audio, self.audio_proj_in, self.audio_proj_out, self.audio_modality_embed))
        if c.n_action:
            out.append(("action", c.n_action, self.action_proj_in, self.action_proj_out, self.action_modality_embed))
        return out

    @property
    def time_embedder(self):
        return self.stack.time_embedder

    @torch.no_grad()
    def reset_parameters(self, seed: Optional[int] = None) -> None:
        self.stack.reset_parameters(seed)
        dev = self.proj_in.weight.device
        g = torch.Generator(device=dev).manual_seed((self.cfg.seed if seed is None else seed) + 7919)
        mods = [self.proj_in, self.proj_out] + [m for st in self._streams() for m in st[2:4]]
        for m in mods:
            m.weight.copy_((torch.randn(m.weight.shape, generator=g, device=dev) * 0.02).to(m.weight.dtype))
            m.bias.zero_()

    # ---- patch layout: token (t, h, w) of the grid holds the latent patch [C, pt, ph, pw] flattened channel-major
    def patchify(self, latents: torch.Tensor) -> torch.Tensor:
        C, (pt, ph, pw) = self.latent_channels, self.patch
        T, H, W = self.cfg.grid
        x = latents.reshape(C, T, pt, H, ph, W, pw).permute(1, 3, 5, 0, 2, 4, 6)
        return x.reshape(T * H * W, C * pt * ph * pw)

    def unpatchify(self, tokens: torch.Tensor) -> torch.Tensor:
        C, (pt, ph, pw) = self.latent_channels, self.patch
        T, H, W = self.cfg.grid
        x = tokens.reshape(T, H, W, C, pt, ph, pw).permute(3, 0, 4, 1, 5, 2, 6)
        return x.reshape(1, C, T * pt, H * ph, W * pw)

    @torch.no_grad()
    def forward(self, hidden_states: torch.Tensor, timestep: torch.Tensor,
                encoder_hidden_states: Optional[torch.Tensor] = None, action_states: Optional[torch.Tensor] = None,
                return_dict: bool = False, context_cache: Optional["ContextCache"] = None,
                audio_states: Optional[torch.Tensor] = None):
        """hidden_states: latents [1, C, T*pt, H*ph, W*pw]; encoder_hidden_states: [1, n_text, d] context already in
        model width; action_states: [1, n_action, action_dim]; audio_states: [1, n_audio, audio_dim].  Returns the
        velocity prediction, latents-shaped and bf16, followed by the audio and the action prediction when those
        streams exist (keys "sample", "audio", "action" with ``return_dict``).  ``context_cache`` (from
        ``stack.precompute_context``, hybrid mask only) replaces ``encoder_hidden_states``: the text run's K/V are
        reused and the forward carries only the generator tokens."""
        c = self.cfg
        batch = _batch_size(hidden_states, 5)
        if batch > 1:
            ts = timestep.reshape(-1)
            return _over_batch(lambda b: self.forward(hidden_states[b:b + 1], ts[b:b + 1] if ts.numel() == batch else ts,
                                                      _sample(encoder_hidden_states, b, 3, batch),
                                                      _sample(action_states, b, 3, batch), return_dict, context_cache,
                                                      _sample(audio_states, b, 3, batch)),
                               batch, return_dict)
        dt = self.proj_in.weight.dtype
        tok = _edge_linear(self.proj_in, self.patchify(hidden_states[0].to(dt)))
        given = {"audio": audio_states, "action": action_states}
        emb = {}
        for name, _, p_in, _, embed in self._streams():
            if given[name] is None:
                raise ValueError(f"this configuration expects {name}_states")
            emb[name] = _edge_linear(p_in, _as2d(given[name]).to(dt)) + embed
        res = self.stack(tok, timestep, encoder_hidden_states=None if context_cache is not None else encoder_hidden_states,
                         action_states=emb.get("action"), return_dict=True, context_cache=context_cache,
                         audio_states=emb.get("audio"))
        joint = res["joint"]            # with a context cache: the generator tokens only
        first = 0 if context_cache is not None else c.n_text
        y = ops.adaln_rmsnorm(joint, self.norm_out.data, None, None, c.eps)
        video = y[first:first + c.n_video]
        sample = self.unpatchify(_edge_linear(self.proj_out, video))
        outs, at = {"audio": None, "action": None}, first + c.n_video
        for name, n, _, p_out, _ in self._streams():
            outs[name] = _edge_linear(p_out, y[at:at + n]).unsqueeze(0)
            at += n
        if return_dict:
            return {"sample": sample, **outs}
        return (sample,) + tuple(o for o in (outs["audio"], outs["action"]) if o is not None)

    # ---- checkpoint plumbing (see cosmos_amd.checkpoint)
    def _top(self):
        mods = {"proj_in": self.proj_in, "proj_out": self.proj_out, "time_embedder.linear_1": self.stack.time_embedder.linear_1,
                "time_embedder.linear_2": self.stack.time_embedder.linear_2}
        for name, _, p_in, p_out, _ in self._streams():
            mods.update({f"{name}_proj_in": p_in, f"{name}_proj_out": p_out})
        t = {f"{k}.{p}": getattr(m, p) for k, m in mods.items() for p in ("weight", "bias")}
        t["norm_out.weight"] = self.norm_out
        for name, _, _, _, embed in self._streams():
            t[f"{name}_modality_embed"] = embed
        return t

    def top_level_keys(self) -> List[str]:
        return list(self._top())

    def assign_top_level(self, key: str, t: torch.Tensor) -> None:
        dst = self._top()[key].data
        if tuple(dst.shape) != tuple(t.shape):
            raise RuntimeError(f"shape {tuple(t.shape)} does not match the model's {tuple(dst.shape)}")
        dst.copy_(t)

    def export_top_level(self):
        return {k: p.data.clone() for k, p in self._top().items()}
