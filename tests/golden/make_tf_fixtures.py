"""Writes tests/golden/tf_fixtures.npz: input/output vectors of the operator
routines that the installed third-party ``transformers`` package (5.15.0)
carries for the Cosmos 3 AR tower (= Qwen3-VL) and for Qwen2-VL's chunked
mRoPE.  The generator branch shares these operator conventions, so the vectors
pin the oracle's rms_norm, rotate-half RoPE, both mRoPE table layouts,
position ids, attention, SwiGLU and the un-modulated pre-norm block wiring.

Run once in the build container (``python tests/golden/make_tf_fixtures.py``);
the .npz is committed and nothing else imports transformers.  Only inputs and
outputs are stored - no source text.
"""
import os
import types

import numpy as np
import torch

from transformers.models.cosmos3_omni import modeling_cosmos3_omni as c3
from transformers.models.qwen2_vl import modeling_qwen2_vl as q2
from transformers.models.qwen3_vl import modeling_qwen3_vl as q3
from transformers.models.qwen3_vl.configuration_qwen3_vl import Qwen3VLTextConfig

torch.manual_seed(20260101)
out = {}


def put(name, t):
    out[name] = t.detach().cpu().numpy() if torch.is_tensor(t) else np.asarray(t)


# 1. RMSNorm ---------------------------------------------------------------
norm = q3.Qwen3VLTextRMSNorm(48, eps=1e-6)
with torch.no_grad():
    norm.weight.copy_(torch.randn(48))
x = torch.randn(7, 48) * 3.0
put("rms_x", x); put("rms_w", norm.weight); put("rms_y", norm(x))

# 2. rotate_half -------------------------------------------------------------
x = torch.randn(3, 16)
put("rh_x", x); put("rh_y", q3.rotate_half(x))

# 3. interleaved mRoPE tables + apply (Qwen3-VL) ----------------------------------
dh, H, N = 128, 2, 24
cfg = Qwen3VLTextConfig(hidden_size=H * dh, num_attention_heads=H, num_key_value_heads=H, head_dim=dh,
                        intermediate_size=64, num_hidden_layers=1, vocab_size=32,
                        rope_parameters={"rope_type": "default", "rope_theta": 10000.0,
                                         "mrope_section": [16, 24, 24], "mrope_interleaved": True})
rot = q3.Qwen3VLTextRotaryEmbedding(cfg)
pos = torch.stack([torch.randint(0, 700, (N,)), torch.randint(0, 90, (N,)), torch.randint(0, 130, (N,))], 0)
cos, sin = rot(torch.zeros(1, dtype=torch.float32), pos[:, None, :])     # [1, N, dh]
q = torch.randn(1, H, N, dh); k = torch.randn(1, H, N, dh)
qe, ke = q3.apply_rotary_pos_emb(q, k, cos, sin)
put("il_pos", pos); put("il_cos", cos[0]); put("il_sin", sin[0])
put("il_q", q[0]); put("il_k", k[0]); put("il_qe", qe[0]); put("il_ke", ke[0])
put("il_pairs", [16, 24, 24])

# 4. chunked mRoPE (Qwen2-VL) ---------------------------------------------------
for tag, dh_c, pairs in (("ch128", 128, [16, 24, 24]), ("ch64", 64, [8, 12, 12])):
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, dh_c, 2, dtype=torch.float) / dh_c))
    rot2 = types.SimpleNamespace(inv_freq=inv_freq, attention_scaling=1.0)
    cos3, sin3 = q2.Qwen2VLRotaryEmbedding.forward(rot2, torch.zeros(1), pos[:, None, :])   # [3,1,N,dh]
    q = torch.randn(1, H, N, dh_c); k = torch.randn(1, H, N, dh_c)
    qe, ke = q2.apply_multimodal_rotary_pos_emb(q, k, cos3, sin3, list(pairs))
    put(f"{tag}_pos", pos); put(f"{tag}_q", q[0]); put(f"{tag}_k", k[0])
    put(f"{tag}_qe", qe[0]); put(f"{tag}_ke", ke[0]); put(f"{tag}_pairs", pairs)

# 5. eager attention -----------------------------------------------------------
Hh, Nq, dh_a = 3, 17, 32
q = torch.randn(1, Hh, Nq, dh_a); k = torch.randn(1, Hh, Nq, dh_a); v = torch.randn(1, Hh, Nq, dh_a)
mod = types.SimpleNamespace(num_key_value_groups=1, training=False)
o, _ = q3.eager_attention_forward(mod, q, k, v, None, scaling=dh_a ** -0.5)   # [1, N, H, dh]
put("at_q", q[0]); put("at_k", k[0]); put("at_v", v[0]); put("at_o", o[0])

# 6. SwiGLU --------------------------------------------------------------------
cfg_m = Qwen3VLTextConfig(hidden_size=24, intermediate_size=40, hidden_act="silu", num_hidden_layers=1,
                          num_attention_heads=2, num_key_value_heads=2, vocab_size=32)
mlp = q3.Qwen3VLTextMLP(cfg_m)
x = torch.randn(5, 24)
put("mlp_x", x); put("mlp_wg", mlp.gate_proj.weight); put("mlp_wu", mlp.up_proj.weight)
put("mlp_wd", mlp.down_proj.weight); put("mlp_y", mlp(x))

# 7. position ids ----------------------------------------------------------------
vp = c3.Cosmos3OmniModel.get_vision_position_ids(None, 7, torch.tensor([3, 4, 5]))
put("vis_start", 7); put("vis_grid", [3, 4, 5]); put("vis_pos", vp)
# joint text(6) + image grid (1,4,6) + text(3) through get_rope_index
fake = types.SimpleNamespace(config=types.SimpleNamespace(vision_config=types.SimpleNamespace(spatial_merge_size=1)))
fake.get_vision_position_ids = lambda *a, **kw: c3.Cosmos3OmniModel.get_vision_position_ids(None, *a, **kw)
types_ids = torch.tensor([[0] * 6 + [1] * 24 + [0] * 3], dtype=torch.int32)
ids = torch.zeros_like(types_ids, dtype=torch.long)
jp, _ = c3.Cosmos3OmniModel.get_rope_index(fake, ids, types_ids, image_grid_thw=torch.tensor([[1, 4, 6]]))
put("joint_pos", jp[:, 0]); put("joint_spec_text0", 6); put("joint_spec_grid", [1, 4, 6]); put("joint_spec_text1", 3)

# 8. un-modulated decoder layer (norm -> attn(+QK-norm, interleaved mRoPE) -> residual -> norm -> MLP -> residual)
dh_l, H_l, N_l = 16, 2, 12
cfg_l = Qwen3VLTextConfig(hidden_size=H_l * dh_l, num_attention_heads=H_l, num_key_value_heads=H_l, head_dim=dh_l,
                          intermediate_size=48, num_hidden_layers=1, vocab_size=32, hidden_act="silu",
                          attention_bias=False, rms_norm_eps=1e-6,
                          rope_parameters={"rope_type": "default", "rope_theta": 10000.0,
                                           "mrope_section": [2, 3, 3], "mrope_interleaved": True})
cfg_l._attn_implementation = "eager"
layer = q3.Qwen3VLTextDecoderLayer(cfg_l, 0).eval()
with torch.no_grad():
    for p_ in layer.parameters():
        p_.copy_(torch.randn_like(p_) * (0.2 if p_.ndim == 2 else 1.0))
rot_l = q3.Qwen3VLTextRotaryEmbedding(cfg_l)
pos_l = torch.stack([torch.randint(0, 30, (N_l,)), torch.randint(0, 9, (N_l,)), torch.randint(0, 9, (N_l,))], 0)
x = torch.randn(1, N_l, H_l * dh_l)
pe = rot_l(x, pos_l[:, None, :])
with torch.no_grad():
    y = layer(x, position_embeddings=pe, attention_mask=None)
a = layer.self_attn
put("ly_x", x[0]); put("ly_y", y[0]); put("ly_pos", pos_l); put("ly_sections", [4, 6, 6]); put("ly_heads", H_l)
put("ly_norm1_w", layer.input_layernorm.weight); put("ly_norm2_w", layer.post_attention_layernorm.weight)
put("ly_wq", a.q_proj.weight); put("ly_wk", a.k_proj.weight); put("ly_wv", a.v_proj.weight); put("ly_wo", a.o_proj.weight)
put("ly_norm_q_w", a.q_norm.weight); put("ly_norm_k_w", a.k_norm.weight)
put("ly_wg", layer.mlp.gate_proj.weight); put("ly_wu", layer.mlp.up_proj.weight); put("ly_wd", layer.mlp.down_proj.weight)

# 8. grouped-query attention (appended last so that the random stream of the sections above is unchanged) -----
# eager attention with 4 query heads on 2 K/V heads (repeat_kv), and a whole decoder layer with the same grouping
Hq, Hkv, Ng, dh_g = 4, 2, 19, 32
q = torch.randn(1, Hq, Ng, dh_g); k = torch.randn(1, Hkv, Ng, dh_g); v = torch.randn(1, Hkv, Ng, dh_g)
mod = types.SimpleNamespace(num_key_value_groups=Hq // Hkv, training=False)
o, _ = q3.eager_attention_forward(mod, q, k, v, None, scaling=dh_g ** -0.5)   # [1, N, Hq, dh]
put("gq_q", q[0]); put("gq_k", k[0]); put("gq_v", v[0]); put("gq_o", o[0])

cfg_g = Qwen3VLTextConfig(hidden_size=Hq * 16, num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=16,
                          intermediate_size=96, hidden_act="silu", num_hidden_layers=1, vocab_size=32, rms_norm_eps=1e-6,
                          rope_parameters={"rope_type": "default", "rope_theta": 10000.0, "mrope_section": [2, 3, 3],
                                           "mrope_interleaved": True})
cfg_g._attn_implementation = "eager"
layer_g = q3.Qwen3VLTextDecoderLayer(cfg_g, 0).eval()
with torch.no_grad():
    for p_ in layer_g.parameters():
        p_.copy_(torch.randn_like(p_) * (0.2 if p_.ndim == 2 else 1.0))
rot_g = q3.Qwen3VLTextRotaryEmbedding(cfg_g)
N_g = 13
pos_g = torch.stack([torch.randint(0, 30, (N_g,)), torch.randint(0, 9, (N_g,)), torch.randint(0, 9, (N_g,))], 0)
x = torch.randn(1, N_g, Hq * 16)
pe = rot_g(x, pos_g[:, None, :])
with torch.no_grad():
    y = layer_g(x, position_embeddings=pe, attention_mask=None)
a = layer_g.self_attn
put("lg_x", x[0]); put("lg_y", y[0]); put("lg_pos", pos_g); put("lg_sections", [4, 6, 6]); put("lg_heads", Hq)
put("lg_norm1_w", layer_g.input_layernorm.weight); put("lg_norm2_w", layer_g.post_attention_layernorm.weight)
put("lg_wq", a.q_proj.weight); put("lg_wk", a.k_proj.weight); put("lg_wv", a.v_proj.weight); put("lg_wo", a.o_proj.weight)
put("lg_norm_q_w", a.q_norm.weight); put("lg_norm_k_w", a.k_norm.weight)
put("lg_wg", layer_g.mlp.gate_proj.weight); put("lg_wu", layer_g.mlp.up_proj.weight); put("lg_wd", layer_g.mlp.down_proj.weight)

path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tf_fixtures.npz")
np.savez_compressed(path, **out)
print("wrote", path, {k: v.shape for k, v in out.items()})
