"""Helpers shared by the GPU parity tests."""
import json
import os

import torch

import oracle as O

BF16_COS, BF16_REL = 0.999, 2e-2       # bf16 path vs fp32 oracle (benchmark tolerance)
FP8_COS, FP8_REL = 0.999, 5e-2         # fp8 path vs fp32 unquantised oracle


def dev():
    return torch.device("cuda:0")


def rand_bf16(shape, gen, scale=1.0):
    """fp32 draw on the CPU generator, rounded to bf16; returns (gpu bf16 tensor, cpu fp32 copy of the same values)."""
    t = (torch.randn(shape, generator=gen) * scale).to(torch.bfloat16)
    return t.to(dev()), t.float()


MARGINS = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gpurun_out", "parity_margins.jsonl")


def record(what, c, r, cos, rel):
    """Keep the measured margins (one JSON line per check) next to the other run artefacts; best effort."""
    try:
        os.makedirs(os.path.dirname(MARGINS), exist_ok=True)
        with open(MARGINS, "a") as fh:
            fh.write(json.dumps({"check": what, "cos": round(c, 7), "max_rel": float(f"{r:.3e}"), "cos_min": cos, "max_rel_max": rel}) + "\n")
    except OSError:
        pass


def assert_close(got, want, cos=BF16_COS, rel=BF16_REL, what=""):
    got = got.detach().float().cpu()
    want = want.detach().float().cpu()
    c, r = O.cos_sim(got, want), O.max_rel_err(got, want)
    record(what, c, r, cos, rel)
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    assert c >= cos and r <= rel, f"{what}: cos={c:.6f} (>= {cos}) max_rel={r:.3e} (<= {rel})"
    return c, r


def oracle_weights(block, branch_count, device="cpu"):
    """fp32 copies of a DMBlock's weights in the oracle's dictionary layout (on the CPU unless asked otherwise)."""
    d = block.d_model
    f = lambda p: p.detach().float().to(device)
    out = []
    for b in range(branch_count):
        qkv = f(block.attn.qkv_weight[b])
        dkv = getattr(block.attn, "n_kv_heads", block.attn.n_heads) * block.attn.head_dim
        out.append(dict(norm1_w=f(block.norm1_weight[b]), wq=qkv[:d], wk=qkv[d:d + dkv], wv=qkv[d + dkv:],
                        wo=f(block.attn.out_weight[b]), norm2_w=f(block.norm2_weight[b]),
                        wg=f(block.gate_weight[b]), wu=f(block.up_weight[b]), wd=f(block.down_weight[b])))
        if getattr(block.attn, "qk_norm", False):
            out[-1]["norm_q_w"] = f(block.attn.norm_q_weight[b])
            out[-1]["norm_k_w"] = f(block.attn.norm_k_weight[b])
    return out
