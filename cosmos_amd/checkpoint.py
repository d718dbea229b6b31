"""Checkpoint key mapping and a safetensors loader for the generator (DM) side of a Cosmos 3 unified checkpoint.

What is attested about the key names (transformers models/cosmos3_omni/modeling_cosmos3_omni.py:39-60, the list of
keys the Reasoner-only model drops, and conversion_mapping.py:920-941, the renames of the AR twin):
  * per layer ``layers.<i>.self_attn.``: AR branch ``to_q, to_k, to_v, to_out, norm_q, norm_k``; DM branch
    ``add_q_proj, add_k_proj, add_v_proj, to_add_out, norm_added_q, norm_added_k``;
  * the DM branch's norms and MLP carry ``moe_gen`` in their names;
  * top level: ``proj_in., proj_out., time_embedder.``, ``action_proj_in., action_proj_out., action_modality_embed``,
    ``audio_proj_in., audio_proj_out., audio_modality_embed`` (the sound stream).
Only the substring ``moe_gen`` is attested for the DM norms / MLP; the patterns below accept it anywhere in the
module name together with the usual ``gate_proj / up_proj / down_proj / input_layernorm / post_attention_layernorm``
words.  The AR twin's norms and MLP use the plain Qwen3-VL names (``input_layernorm``, ``post_attention_layernorm``,
``mlp.gate_proj`` ...).  Where the per-block adaLN projection lives in a real checkpoint is not attested: keys that
match ``adaLN_modulation`` / ``adaln`` inside a layer are accepted, everything else is reported as unexpected.
"""
from __future__ import annotations

import re
from typing import Dict, Iterable, List, Mapping, Optional, Tuple, Union

import torch

AR, DM = 0, 1       # branch indices of a two-branch (text | video) stack

# (regex on the key, target, branch).  Targets: ("qkv", part) part 0/1/2 = q/k/v rows of the fused weight;
# ("attr", name) a per-branch parameter list of the block / its attention module; ("top", name) a stack-level tensor.
_LAYER = r"^(?:model\.language_model\.)?layers\.(\d+)\."
_RULES: List[Tuple[str, Tuple, Optional[int]]] = [
    (_LAYER + r"self_attn\.(?:to_q|q_proj)\.weight$", ("qkv", 0), AR),
    (_LAYER + r"self_attn\.(?:to_k|k_proj)\.weight$", ("qkv", 1), AR),
    (_LAYER + r"self_attn\.(?:to_v|v_proj)\.weight$", ("qkv", 2), AR),
    (_LAYER + r"self_attn\.(?:to_out|o_proj)(?:\.0)?\.weight$", ("attn", "out_weight"), AR),
    (_LAYER + r"self_attn\.(?:norm_q|q_norm)\.weight$", ("qknorm", "norm_q_weight"), AR),
    (_LAYER + r"self_attn\.(?:norm_k|k_norm)\.weight$", ("qknorm", "norm_k_weight"), AR),
    (_LAYER + r"self_attn\.add_q_proj\.weight$", ("qkv", 0), DM),
    (_LAYER + r"self_attn\.add_k_proj\.weight$", ("qkv", 1), DM),
    (_LAYER + r"self_attn\.add_v_proj\.weight$", ("qkv", 2), DM),
    (_LAYER + r"self_attn\.to_add_out(?:\.0)?\.weight$", ("attn", "out_weight"), DM),
    (_LAYER + r"self_attn\.norm_added_q\.weight$", ("qknorm", "norm_q_weight"), DM),
    (_LAYER + r"self_attn\.norm_added_k\.weight$", ("qknorm", "norm_k_weight"), DM),
    (_LAYER + r"(?=[^ ]*moe_gen)[\w.]*input_layernorm[\w.]*\.weight$", ("block", "norm1_weight"), DM),
    (_LAYER + r"(?=[^ ]*moe_gen)[\w.]*post_attention_layernorm[\w.]*\.weight$", ("block", "norm2_weight"), DM),
    (_LAYER + r"(?=[^ ]*moe_gen)[\w.]*gate_proj\.weight$", ("block", "gate_weight"), DM),
    (_LAYER + r"(?=[^ ]*moe_gen)[\w.]*up_proj\.weight$", ("block", "up_weight"), DM),
    (_LAYER + r"(?=[^ ]*moe_gen)[\w.]*down_proj\.weight$", ("block", "down_weight"), DM),
    (_LAYER + r"input_layernorm\.weight$", ("block", "norm1_weight"), AR),
    (_LAYER + r"post_attention_layernorm\.weight$", ("block", "norm2_weight"), AR),
    (_LAYER + r"mlp\.gate_proj\.weight$", ("block", "gate_weight"), AR),
    (_LAYER + r"mlp\.up_proj\.weight$", ("block", "up_weight"), AR),
    (_LAYER + r"mlp\.down_proj\.weight$", ("block", "down_weight"), AR),
    (_LAYER + r"[\w.]*ada(?:LN|ln)[\w.]*\.(weight|bias)$", ("adaln", None), None),
]
_TOP = [r"^proj_in\.", r"^proj_out\.", r"^time_embedder\.", r"^action_proj_in\.", r"^action_proj_out\.",
        r"^action_modality_embed$", r"^audio_proj_in\.", r"^audio_proj_out\.", r"^audio_modality_embed$", r"^norm_out\."]
_COMPILED = [(re.compile(rx), tgt, br) for rx, tgt, br in _RULES]


def _copy_exact(dst: torch.Tensor, t: torch.Tensor) -> None:
    """copy_ broadcasts silently; a checkpoint tensor must have exactly the shape of its destination."""
    if tuple(dst.shape) != tuple(t.shape):
        raise RuntimeError(f"shape {tuple(t.shape)} does not match the model's {tuple(dst.shape)}")
    dst.copy_(t)


def classify(key: str):
    """-> (layer index or None, target tuple, branch) or None when the key is not part of the generator path."""
    for rx, tgt, br in _COMPILED:
        m = rx.match(key)
        if m:
            return int(m.group(1)), tgt + ((m.group(2),) if tgt[0] == "adaln" else ()), br
    for rx in _TOP:
        if re.match(rx, key):
            return None, ("top", key), None
    return None


def _iter_tensors(source) -> Iterable[Tuple[str, torch.Tensor]]:
    if isinstance(source, Mapping):
        yield from source.items()
        return
    from safetensors import safe_open      # streams one tensor at a time: a 15 GB stack never sits in host RAM twice
    paths = [source] if isinstance(source, str) else list(source)
    for path in paths:
        with safe_open(path, framework="pt", device="cpu") as f:
            for key in f.keys():
                yield key, f.get_tensor(key)


@torch.no_grad()
def load_generator_weights(model, source: Union[str, Iterable[str], Mapping[str, torch.Tensor]],
                           strict: bool = False) -> Dict[str, List[str]]:
    """Copy the tensors of ``source`` (a safetensors path, several shards, or a name -> tensor mapping) into a
    ``DMTransformer`` / ``DMStack``.  Returns {"loaded", "unexpected", "missing"} key lists; ``strict`` raises when
    either of the last two is non-empty.  The fused QKV weight is filled row-block by row-block, so the three
    projections never exist concatenated on the host."""
    stack = getattr(model, "stack", model)
    d = stack.cfg.d_model
    loaded, unexpected = [], []
    want = set(_expected_keys(model))
    seen = set()
    for key, t in _iter_tensors(source):
        c = classify(key)
        if c is None:
            unexpected.append(key)
            continue
        layer, tgt, br = c
        try:
            if tgt[0] == "top":
                if hasattr(model, "top_level_keys") and key not in model.top_level_keys():
                    unexpected.append(key)          # an edge this model was built without (e.g. no audio stream)
                    continue
                _assign_top(model, key, t)
                seen.add(key)
            else:
                if layer >= len(stack.blocks) or (br is not None and br >= stack.cfg.n_branches):
                    unexpected.append(key)
                    continue
                blk = stack.blocks[layer]
                if tgt[0] == "qkv":
                    # rows of the fused weight: [q: d | k: d_kv | v: d_kv] (d_kv < d under grouped-query attention)
                    dkv = blk.attn.n_kv_heads * blk.attn.head_dim
                    r0 = (0, d, d + dkv)[tgt[1]]
                    _copy_exact(blk.attn.qkv_weight[br].data[r0:r0 + (d if tgt[1] == 0 else dkv)], t)
                    seen.add(f"layers.{layer}.qkv.{br}.{tgt[1]}")
                elif tgt[0] == "attn":
                    _copy_exact(getattr(blk.attn, tgt[1])[br].data, t)
                    seen.add(f"layers.{layer}.{tgt[1]}.{br}")
                elif tgt[0] == "qknorm":
                    if not blk.attn.qk_norm:
                        unexpected.append(key)
                        continue
                    _copy_exact(getattr(blk.attn, tgt[1]).data[br], t)
                    seen.add(f"layers.{layer}.{tgt[1]}.{br}")
                elif tgt[0] == "block":
                    _copy_exact(getattr(blk, tgt[1])[br].data, t)
                    seen.add(f"layers.{layer}.{tgt[1]}.{br}")
                else:   # adaLN projection of the block
                    _copy_exact(getattr(blk.adaLN_modulation, tgt[-1]).data, t)
                    seen.add(f"layers.{layer}.adaLN.{tgt[-1]}")
            loaded.append(key)
        except (RuntimeError, AttributeError) as e:      # shape mismatch or a part this model does not have
            raise ValueError(f"cannot load {key} {tuple(t.shape)}: {e}") from None
    missing = sorted(want - seen)
    if stack.cfg.fp8:
        for blk in stack.blocks:
            blk.quantize_()
    if strict and (missing or unexpected):
        raise KeyError(f"missing: {missing[:8]}{'...' if len(missing) > 8 else ''}; "
                       f"unexpected: {unexpected[:8]}{'...' if len(unexpected) > 8 else ''}")
    return {"loaded": loaded, "unexpected": unexpected, "missing": missing}


def _expected_keys(model) -> List[str]:
    stack = getattr(model, "stack", model)
    out = []
    for i, blk in enumerate(stack.blocks):
        for b in range(stack.cfg.n_branches):
            out += [f"layers.{i}.qkv.{b}.{p}" for p in range(3)]
            out += [f"layers.{i}.{n}.{b}" for n in ("out_weight", "norm1_weight", "norm2_weight", "gate_weight", "up_weight",
                                                     "down_weight")]
            if blk.attn.qk_norm:
                out += [f"layers.{i}.{n}.{b}" for n in ("norm_q_weight", "norm_k_weight")]
        out += [f"layers.{i}.adaLN.weight", f"layers.{i}.adaLN.bias"]
    if hasattr(model, "top_level_keys"):
        out += model.top_level_keys()
    return out


def _assign_top(model, key: str, t: torch.Tensor) -> None:
    if not hasattr(model, "assign_top_level"):
        raise AttributeError("this model has no stack-edge modules")
    model.assign_top_level(key, t)


def export_generator_weights(model) -> Dict[str, torch.Tensor]:
    """Inverse of ``load_generator_weights`` with the attested key names (DM norms / MLP written as
    ``*_moe_gen``); used to round-trip a model through a safetensors file."""
    stack = getattr(model, "stack", model)
    d = stack.cfg.d_model
    out: Dict[str, torch.Tensor] = {}
    names = {AR: ("to_q", "to_k", "to_v", "to_out", "norm_q", "norm_k"),
             DM: ("add_q_proj", "add_k_proj", "add_v_proj", "to_add_out", "norm_added_q", "norm_added_k")}
    for i, blk in enumerate(stack.blocks):
        pre = f"layers.{i}."
        for b in range(min(stack.cfg.n_branches, 2)):
            q, k, v, o, nq, nk = names[b]
            w = blk.attn.qkv_weight[b].data
            dkv = blk.attn.n_kv_heads * blk.attn.head_dim
            out[pre + f"self_attn.{q}.weight"], out[pre + f"self_attn.{k}.weight"] = w[:d].clone(), w[d:d + dkv].clone()
            out[pre + f"self_attn.{v}.weight"] = w[d + dkv:].clone()
            out[pre + f"self_attn.{o}.weight"] = blk.attn.out_weight[b].data.clone()
            if blk.attn.qk_norm:
                out[pre + f"self_attn.{nq}.weight"] = blk.attn.norm_q_weight.data[b].clone()
                out[pre + f"self_attn.{nk}.weight"] = blk.attn.norm_k_weight.data[b].clone()
            sfx = "_moe_gen" if b == DM else ""
            out[pre + f"input_layernorm{sfx}.weight"] = blk.norm1_weight[b].data.clone()
            out[pre + f"post_attention_layernorm{sfx}.weight"] = blk.norm2_weight[b].data.clone()
            for n, plist in (("gate_proj", blk.gate_weight), ("up_proj", blk.up_weight), ("down_proj", blk.down_weight)):
                out[pre + f"mlp{sfx}.{n}.weight"] = plist[b].data.clone()
        out[pre + "adaLN_modulation.weight"] = blk.adaLN_modulation.weight.data.clone()
        out[pre + "adaLN_modulation.bias"] = blk.adaLN_modulation.bias.data.clone()
    if hasattr(model, "export_top_level"):
        out.update(model.export_top_level())
    return out
