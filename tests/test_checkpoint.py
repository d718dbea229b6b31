"""Checkpoint key mapping and the safetensors round trip (host logic; no GPU needed)."""
import os

import pytest
import torch

from cosmos_amd import DMTransformer, export_generator_weights, load_generator_weights
from cosmos_amd.checkpoint import AR, DM, classify
from cosmos_amd.config import DMConfig


def test_attested_key_names_are_classified():
    # names the reference's model files attest for the generator side, plus the renamed AR twin
    assert classify("layers.3.self_attn.add_q_proj.weight") == (3, ("qkv", 0), DM)
    assert classify("layers.3.self_attn.add_k_proj.weight") == (3, ("qkv", 1), DM)
    assert classify("layers.3.self_attn.add_v_proj.weight") == (3, ("qkv", 2), DM)
    assert classify("layers.0.self_attn.to_add_out.weight") == (0, ("attn", "out_weight"), DM)
    assert classify("layers.7.self_attn.norm_added_q.weight") == (7, ("qknorm", "norm_q_weight"), DM)
    assert classify("layers.7.self_attn.to_q.weight") == (7, ("qkv", 0), AR)
    assert classify("model.language_model.layers.7.self_attn.q_proj.weight") == (7, ("qkv", 0), AR)
    assert classify("layers.7.self_attn.norm_k.weight") == (7, ("qknorm", "norm_k_weight"), AR)
    assert classify("layers.1.mlp_moe_gen.down_proj.weight") == (1, ("block", "down_weight"), DM)
    assert classify("layers.1.mlp.down_proj.weight") == (1, ("block", "down_weight"), AR)
    assert classify("layers.1.post_attention_layernorm_moe_gen.weight") == (1, ("block", "norm2_weight"), DM)
    assert classify("layers.1.post_attention_layernorm.weight") == (1, ("block", "norm2_weight"), AR)
    assert classify("proj_in.bias")[1] == ("top", "proj_in.bias")
    assert classify("time_embedder.linear_1.weight")[1][0] == "top"
    # the sound stream's edges are stack-level tensors like the action stream's
    assert classify("audio_proj_in.weight")[1] == ("top", "audio_proj_in.weight")
    assert classify("audio_modality_embed")[1] == ("top", "audio_modality_embed")
    # not part of the generator path: embeddings, the vision encoder
    for k in ("embed_tokens.weight", "blocks.0.attn.qkv.weight", "lm_head.weight", "audio_encoder.conv.weight"):
        assert classify(k) is None


def small_model(seed, n_kv_heads=None):
    cfg = DMConfig("ck", 128, 2, 64, 256, 2, (1, 2, 4), n_text=4, n_action=2, n_branches=2, qk_norm=True,
                   mrope_sections=(16, 24, 24), n_kv_heads=n_kv_heads)
    m = DMTransformer(cfg, latent_channels=4, patch=(1, 2, 2), action_dim=6, device="cpu")
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for p in m.parameters():
            p.copy_(torch.randn(p.shape, generator=g).to(p.dtype))
    return m


def test_safetensors_round_trip(tmp_path):
    from safetensors.torch import save_file
    a, b = small_model(1), small_model(2)
    sd = export_generator_weights(a)
    assert "layers.1.self_attn.add_q_proj.weight" in sd and "layers.0.mlp_moe_gen.gate_proj.weight" in sd
    # split over two shards, plus a tensor that does not belong to the generator path
    keys = sorted(sd)
    p1, p2 = str(tmp_path / "a.safetensors"), str(tmp_path / "b.safetensors")
    save_file({k: sd[k].contiguous() for k in keys[::2]}, p1)
    extra = {k: sd[k].contiguous() for k in keys[1::2]}
    extra["embed_tokens.weight"] = torch.zeros(3, 3)
    save_file(extra, p2)
    rep = load_generator_weights(b, [p1, p2])
    assert rep["missing"] == [] and rep["unexpected"] == ["embed_tokens.weight"] and len(rep["loaded"]) == len(sd)
    for (na, pa), (nb, pb) in zip(a.named_parameters(), b.named_parameters()):
        assert na == nb and torch.equal(pa, pb), na
    with pytest.raises(KeyError):
        load_generator_weights(b, [p1, p2], strict=True)          # the stray tensor
    c = small_model(3)
    rep = load_generator_weights(c, p1)
    assert rep["missing"] and set(rep["loaded"]) == set(keys[::2])  # half a checkpoint is reported, not hidden
    bad = dict(sd)
    bad["layers.0.self_attn.add_q_proj.weight"] = torch.zeros(5, 5)
    with pytest.raises(ValueError):
        load_generator_weights(small_model(4), bad)


def test_round_trip_with_grouped_kv_heads():
    """One K/V head for two query heads: k_proj / v_proj have d_kv = 64 rows and land behind the 128 q rows."""
    a, b = small_model(6, n_kv_heads=1), small_model(7, n_kv_heads=1)
    sd = export_generator_weights(a)
    assert sd["layers.0.self_attn.add_q_proj.weight"].shape == (128, 128)
    assert sd["layers.0.self_attn.add_k_proj.weight"].shape == (64, 128)
    assert sd["layers.0.self_attn.to_v.weight"].shape == (64, 128)
    w = a.stack.blocks[0].attn.qkv_weight[1]
    assert w.shape == (256, 128) and torch.equal(sd["layers.0.self_attn.add_v_proj.weight"], w[192:])
    rep = load_generator_weights(b, sd)
    assert rep["missing"] == [] and rep["unexpected"] == []
    for (na, pa), (nb, pb) in zip(a.named_parameters(), b.named_parameters()):
        assert na == nb and torch.equal(pa, pb), na
    with pytest.raises(ValueError):      # a multi-head checkpoint does not fit a grouped-query model
        load_generator_weights(small_model(8, n_kv_heads=1), export_generator_weights(small_model(9)))


def test_patchify_round_trip_and_order():
    m = small_model(5)
    lat = torch.arange(4 * 1 * 4 * 8, dtype=torch.float32).reshape(1, 4, 1, 4, 8)
    tok = m.patchify(lat[0])
    assert tok.shape == (8, 16)
    assert torch.equal(m.unpatchify(tok), lat)
    # token (t=0, h=1, w=2) holds the 2x2 patch at rows 2..3, columns 4..5, channel-major
    want = lat[0, :, 0, 2:4, 4:6].reshape(-1)
    assert torch.equal(tok[1 * 4 + 2], want)
