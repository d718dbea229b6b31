"""Helpers shared by the GPU parity tests."""
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


def assert_close(got, want, cos=BF16_COS, rel=BF16_REL, what=""):
    got = got.detach().float().cpu()
    c, r = O.cos_sim(got, want), O.max_rel_err(got, want)
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    assert c >= cos and r <= rel, f"{what}: cos={c:.6f} (>= {cos}) max_rel={r:.3e} (<= {rel})"
    return c, r


def oracle_weights(block, branch_count):
    """fp32 CPU copies of a DMBlock's weights in the oracle's dictionary layout."""
    d = block.d_model
    out = []
    for b in range(branch_count):
        qkv = block.attn.qkv_weight[b].detach().float().cpu()
        dkv = getattr(block.attn, "n_kv_heads", block.attn.n_heads) * block.attn.head_dim
        out.append(dict(norm1_w=block.norm1_weight[b].detach().float().cpu(), wq=qkv[:d], wk=qkv[d:d + dkv], wv=qkv[d + dkv:],
                        wo=block.attn.out_weight[b].detach().float().cpu(),
                        norm2_w=block.norm2_weight[b].detach().float().cpu(),
                        wg=block.gate_weight[b].detach().float().cpu(), wu=block.up_weight[b].detach().float().cpu(),
                        wd=block.down_weight[b].detach().float().cpu()))
        if getattr(block.attn, "qk_norm", False):
            out[-1]["norm_q_w"] = block.attn.norm_q_weight[b].detach().float().cpu()
            out[-1]["norm_k_w"] = block.attn.norm_k_weight[b].detach().float().cpu()
    return out
