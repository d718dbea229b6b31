"""The oracle against library golden vectors (tests/golden/tf_fixtures.npz, written by
tests/golden/make_tf_fixtures.py from the installed transformers' Qwen3-VL / Qwen2-VL /
Cosmos3-Omni operator routines)."""
import numpy as np
import torch

import oracle as O

T = lambda a: torch.from_numpy(np.asarray(a))


def close(a, b, tol=2e-6):
    a = torch.as_tensor(a, dtype=torch.float64); b = torch.as_tensor(b, dtype=torch.float64)
    assert a.shape == b.shape
    assert float((a - b).abs().max()) <= tol * max(1.0, float(b.abs().max())), float((a - b).abs().max())


def test_rms_norm(golden):
    close(O.rms_norm(T(golden["rms_x"]), T(golden["rms_w"])), golden["rms_y"])


def test_rotate_half_convention(golden):
    # rotate_half(x) = cat(-x2, x1): apply_mrope with cos=0, sin=1 must reproduce it.
    x = T(golden["rh_x"]).unsqueeze(1)                 # [N,1,dh]
    z = torch.zeros(x.shape[0], x.shape[-1] // 2)
    close(O.apply_mrope(x, z, z + 1.0)[:, 0], golden["rh_y"])


def test_mrope_interleaved_tables_and_apply(golden):
    pos = T(golden["il_pos"]); sections = [2 * int(p) for p in golden["il_pairs"]]
    cos, sin = O.mrope_cos_sin(pos, 128, sections, 10000.0, "interleaved")
    close(torch.cat([cos, cos], -1), golden["il_cos"], 1e-5)
    close(torch.cat([sin, sin], -1), golden["il_sin"], 1e-5)
    for a, b in (("il_q", "il_qe"), ("il_k", "il_ke")):
        x = T(golden[a]).transpose(0, 1)               # [N,H,dh]
        close(O.apply_mrope(x, cos, sin).transpose(0, 1), golden[b], 1e-5)


def test_mrope_chunked(golden):
    for tag, dh in (("ch128", 128), ("ch64", 64)):
        pos = T(golden[f"{tag}_pos"]); sections = [2 * int(p) for p in golden[f"{tag}_pairs"]]
        cos, sin = O.mrope_cos_sin(pos, dh, sections, 10000.0, "chunked")
        for a, b in ((f"{tag}_q", f"{tag}_qe"), (f"{tag}_k", f"{tag}_ke")):
            x = T(golden[a]).transpose(0, 1)
            close(O.apply_mrope(x, cos, sin).transpose(0, 1), golden[b], 1e-5)


def test_attention(golden):
    q, k, v = (T(golden[n]).transpose(0, 1) for n in ("at_q", "at_k", "at_v"))   # [N,H,dh]
    close(O.attention(q, k, v, chunk=5), golden["at_o"], 1e-5)
    close(O.attention_rows(q[[3, 11]], k, v), golden["at_o"][[3, 11]], 1e-5)


def test_swiglu(golden):
    close(O.swiglu(T(golden["mlp_x"]), T(golden["mlp_wg"]), T(golden["mlp_wu"]), T(golden["mlp_wd"])),
          golden["mlp_y"], 1e-5)


def test_vision_and_joint_positions(golden):
    vp = O.vision_positions(int(golden["vis_start"]), [int(g) for g in golden["vis_grid"]])
    assert torch.equal(vp, T(golden["vis_pos"]))
    jp = O.joint_positions([("text", int(golden["joint_spec_text0"])),
                            ("video", [int(g) for g in golden["joint_spec_grid"]]),
                            ("text", int(golden["joint_spec_text1"]))])
    assert torch.equal(jp, T(golden["joint_pos"]))


def test_unmodulated_block_wiring_against_decoder_layer(golden):
    g = golden
    w = {k: T(g["ly_" + k]) for k in ("norm1_w", "norm2_w", "wq", "wk", "wv", "wo", "wg", "wu", "wd",
                                       "norm_q_w", "norm_k_w")}
    H = int(g["ly_heads"]); d = g["ly_x"].shape[1]
    cos, sin = O.mrope_cos_sin(T(g["ly_pos"]), d // H, [int(s) for s in g["ly_sections"]], 10000.0, "interleaved")
    y = O.dm_block(T(g["ly_x"]), [w], None, cos, sin, H)
    close(y, g["ly_y"], 2e-5)
    # row-sampled form is exact for the sampled rows
    rows = torch.tensor([0, 5, 11])
    close(O.dm_block(T(g["ly_x"]), [w], None, cos, sin, H, attn_rows=rows), g["ly_y"][[0, 5, 11]], 2e-5)


def test_grouped_query_attention(golden):
    """4 query heads on 2 K/V heads against the library's eager attention (repeat_kv)."""
    q, k, v = (T(golden[n]).transpose(0, 1) for n in ("gq_q", "gq_k", "gq_v"))   # [N,Hq,dh], [N,Hkv,dh]
    assert q.shape[1] == 4 and k.shape[1] == 2
    close(O.attention(q, k, v, chunk=7), golden["gq_o"], 1e-5)
    close(O.attention_rows(q[[0, 9, 18]], k, v), golden["gq_o"][[0, 9, 18]], 1e-5)
    # a wrong head pairing (interleaved instead of blocked repetition) is a different function
    wrong = O.attention(q, k.flip(1), v.flip(1))
    assert float((wrong - T(golden["gq_o"])).abs().max()) > 1e-2


def test_grouped_query_block_wiring_against_decoder_layer(golden):
    g = golden
    w = {k: T(g["lg_" + k]) for k in ("norm1_w", "norm2_w", "wq", "wk", "wv", "wo", "wg", "wu", "wd",
                                       "norm_q_w", "norm_k_w")}
    H = int(g["lg_heads"]); d = g["lg_x"].shape[1]
    assert w["wk"].shape[0] * 2 == w["wq"].shape[0]
    cos, sin = O.mrope_cos_sin(T(g["lg_pos"]), d // H, [int(s) for s in g["lg_sections"]], 10000.0, "interleaved")
    close(O.dm_block(T(g["lg_x"]), [w], None, cos, sin, H), g["lg_y"], 2e-5)
