"""Block / stack parity with the fp32 CPU oracle: the single-block benchmark configuration (C0), a
three-branch Mixture-of-Transformers block, a small stack, the fp8 variant, and the full-size
attention (C1 shape) on sampled query rows."""
import pytest
import torch

import oracle as O
from cosmos_amd import CONFIGS, DMBlock, DMStack, ops, rotary
from cosmos_amd.config import DMConfig
from gpu_util import BF16_COS, BF16_REL, FP8_COS, FP8_REL, assert_close, dev, oracle_weights, rand_bf16, record

pytestmark = pytest.mark.gpu


def make_block(cfg, seed, randomize_norms=True):
    blk = DMBlock(cfg.d_model, cfg.n_heads, cfg.head_dim, cfg.hidden, cfg.n_branches, cfg.eps, cfg.fp8, device=dev())
    g = torch.Generator(device=dev()).manual_seed(seed)
    blk.reset_parameters(g)
    if randomize_norms:
        with torch.no_grad():
            for p in list(blk.norm1_weight) + list(blk.norm2_weight):
                p.copy_(1 + 0.2 * torch.randn(p.shape, generator=g, device=dev()))
            blk.adaLN_modulation.bias.copy_(0.3 * torch.randn(blk.adaLN_modulation.bias.shape, generator=g, device=dev()))
    return blk


def test_c0_single_block_parity():
    """Benchmark configuration 0: d=1024, 16x64 heads, hidden 4096, grid 4x16x16, sections 16/24/24."""
    cfg = CONFIGS["C0"]
    st = DMStack(cfg, device=dev())
    st.reset_parameters()
    g = torch.Generator().manual_seed(cfg.seed)
    x, xr = rand_bf16((cfg.n_tokens, cfg.d_model), g)
    t = torch.rand(1, generator=g) * 1000.0
    (y,) = st(x.unsqueeze(0), t.to(dev()))
    # oracle: same weights in fp32, conditioning through the oracle's own embedding / MLP
    te = st.time_embedder
    c = O.time_mlp(O.timestep_embedding(t), te.linear_1.weight.float().cpu(), te.linear_1.bias.float().cpu(),
                   te.linear_2.weight.float().cpu(), te.linear_2.bias.float().cpu())
    blk = st.blocks[0]
    mod = O.adaln_modulation(c, blk.adaLN_modulation.weight.float().cpu(), blk.adaLN_modulation.bias.float().cpu())
    pos = O.vision_positions(0, cfg.grid)
    cos, sin = O.mrope_cos_sin(pos, cfg.head_dim, cfg.mrope_sections, cfg.rope_base, cfg.rope_layout)
    want = O.dm_block(xr, oracle_weights(blk, 1), mod, cos, sin, cfg.n_heads)
    assert_close(y[0], want, BF16_COS, BF16_REL, "C0 block")
    # With N(0, 0.02) weights and zero biases the adaLN gates are nearly zero and the block is close to the
    # identity, so repeat with order-one modulation (gates included) and check the UPDATE y - x as well.
    gm = torch.Generator().manual_seed(99)
    strong = [torch.randn(cfg.d_model, generator=gm) * s for s in (0.5, 0.5, 8.0, 0.5, 0.5, 8.0)]
    y2 = blk(x, None, st.rotary(dev()), modulation=[m.to(dev()) for m in strong])
    want2 = O.dm_block(xr, oracle_weights(blk, 1), strong, cos, sin, cfg.n_heads)
    assert float((want2 - xr).abs().max()) > 1.0
    assert_close(y2, want2, BF16_COS, BF16_REL, "C0 block, strong modulation")
    assert_close(y2.float().cpu() - xr, want2 - xr, 0.999, BF16_REL, "C0 block update")


def test_rope_placements_agree():
    from cosmos_amd import DMAttnProcessor
    cfg = DMConfig("t", 256, 2, 128, 512, 1, (2, 4, 8), n_text=8)
    blk = make_block(cfg, 5)
    g = torch.Generator().manual_seed(5)
    x, _ = rand_bf16((cfg.n_tokens, 256), g)
    temb, _ = rand_bf16((256,), g)
    st = DMStack(cfg, device=dev())
    ys = []
    for mode in ("in_attention", "gemm_epilogue", "streaming"):
        blk.attn.set_processor(DMAttnProcessor(rope=mode))
        ys.append(blk(x, temb, st.rotary(dev()), st.segments()))
    assert_close(ys[1], ys[0].float().cpu(), 0.99999, 4e-3, "rope in GEMM epilogue vs in attention")
    assert_close(ys[2], ys[0].float().cpu(), 0.99999, 4e-3, "streaming rope vs in attention")


def test_block_gate_zero_is_identity():
    cfg = DMConfig("t", 256, 2, 128, 512, 1, (2, 4, 8))
    blk = make_block(cfg, 3)
    g = torch.Generator().manual_seed(3)
    x, _ = rand_bf16((cfg.n_tokens, 256), g)
    pos, _ = rotary.build_positions(0, cfg.grid)
    rot = rotary.rotary_tables(pos, 128, cfg.mrope_sections, device=dev())
    z, o = torch.zeros(256, device=dev()), torch.ones(256, device=dev())
    y = blk(x, None, rot, modulation=(o, o, z, o, o, z))
    assert torch.equal(y, x)


def test_mot_three_branch_block():
    cfg = DMConfig("mot", 256, 2, 128, 512, 1, (2, 4, 8), n_text=40, n_action=24, n_branches=3)
    st = DMStack(cfg, device=dev())
    blk = make_block(cfg, 11)
    g = torch.Generator().manual_seed(11)
    x, xr = rand_bf16((cfg.n_tokens, 256), g)
    temb, tembr = rand_bf16((256,), g)
    rot = st.rotary(dev())
    segs = st.segments()
    assert segs == [(0, 40, 0, False), (40, 64, 1, True), (104, 24, 2, True)]
    y = blk(x, temb, rot, segs)
    mod = O.adaln_modulation(tembr.view(1, -1), blk.adaLN_modulation.weight.float().cpu(),
                             blk.adaLN_modulation.bias.float().cpu())
    pos = O.joint_positions([("text", 40), ("video", cfg.grid), ("action", 24)])
    cos, sin = O.mrope_cos_sin(pos, 128, cfg.mrope_sections)
    ws = oracle_weights(blk, 3)
    want = O.dm_block(xr, ws, mod, cos, sin, 2, segs)
    assert_close(y, want, BF16_COS, BF16_REL, "MoT block")
    # equal weight sets, everything modulated == single-branch block on the same kernels
    with torch.no_grad():
        for plist in (blk.attn.qkv_weight, blk.attn.out_weight, blk.norm1_weight, blk.norm2_weight, blk.gate_weight,
                      blk.up_weight, blk.down_weight):
            for b in (0, 2):
                plist[b].copy_(plist[1])
    y3 = blk(x, temb, rot, [(0, 40, 0, True), (40, 64, 1, True), (104, 24, 2, True)])
    y1 = blk(x, temb, rot, [(0, cfg.n_tokens, 1, True)])
    # (the single segment takes the QKV GEMM that writes the K / V tile images itself and rotates K ahead of its one
    # rounding; segments starting at 40 and 104 are not tile boundaries and take the GEMM + re-tiling pair)
    assert_close(y3, y1.float().cpu(), 0.99999, 6e-3, "equal weights == single branch")


@pytest.mark.parametrize("n_kv_heads", [None, 1])
def test_mot_block_with_qk_norm(n_kv_heads):
    """Three-branch block with the per-head QK-RMSNorm switched on (own weight row per branch); with one K/V head
    for the two query heads as well (grouped-query attention: the fused QKV weight then has d + 2 d_kv rows)."""
    cfg = DMConfig("motn", 256, 2, 128, 512, 1, (2, 4, 8), n_text=40, n_action=24, n_branches=3, qk_norm=True,
                   n_kv_heads=n_kv_heads)
    st = DMStack(cfg, device=dev())
    blk = st.blocks[0]
    g = torch.Generator(device=dev()).manual_seed(21)
    blk.reset_parameters(g)
    with torch.no_grad():
        blk.attn.norm_q_weight.copy_(1 + 0.3 * torch.randn(3, 128, generator=g, device=dev()))
        blk.attn.norm_k_weight.copy_(1 + 0.3 * torch.randn(3, 128, generator=g, device=dev()))
        blk.adaLN_modulation.bias.copy_(0.3 * torch.randn(blk.adaLN_modulation.bias.shape, generator=g, device=dev()))
    gc = torch.Generator().manual_seed(21)
    x, xr = rand_bf16((cfg.n_tokens, 256), gc)
    temb, tembr = rand_bf16((256,), gc)
    segs = st.segments()
    y = blk(x, temb, st.rotary(dev()), segs)
    mod = O.adaln_modulation(tembr.view(1, -1), blk.adaLN_modulation.weight.float().cpu(),
                             blk.adaLN_modulation.bias.float().cpu())
    pos = O.joint_positions([("text", 40), ("video", cfg.grid), ("action", 24)])
    cos, sin = O.mrope_cos_sin(pos, 128, cfg.mrope_sections)
    ws = oracle_weights(blk, 3)
    assert "norm_q_w" in ws[0]
    want = O.dm_block(xr, ws, mod, cos, sin, 2, segs)
    assert_close(y, want, BF16_COS, BF16_REL, "MoT block with QK-norm")
    # a permuted segment order (video branch first in the table) must pick the same weight rows
    y2 = blk(x, temb, st.rotary(dev()), [(0, 40, 0, False), (40, 64, 1, True), (104, 24, 2, True)])
    assert torch.equal(y, y2)
    # without the norm the result differs (the switch is live)
    want_plain = O.dm_block(xr, [{k: v for k, v in w.items() if k not in ("norm_q_w", "norm_k_w")} for w in ws], mod, cos,
                            sin, 2, segs)
    assert O.max_rel_err(want, want_plain) > 1e-2


def test_small_stack_and_encoder_path():
    cfg = DMConfig("s", 256, 4, 64, 640, 3, (2, 3, 10), n_text=20, mrope_sections=(16, 24, 24))
    st = DMStack(cfg, device=dev())
    st.reset_parameters(5)
    g = torch.Generator().manual_seed(5)
    xv, xvr = rand_bf16((1, cfg.n_video, 256), g)
    xt, xtr = rand_bf16((1, cfg.n_text, 256), g)
    t = torch.tensor([417.0])
    out = st(xv, t.to(dev()), encoder_hidden_states=xt, return_dict=True)
    te = st.time_embedder
    c = O.time_mlp(O.timestep_embedding(t), te.linear_1.weight.float().cpu(), te.linear_1.bias.float().cpu(),
                   te.linear_2.weight.float().cpu(), te.linear_2.bias.float().cpu())
    mods = [O.adaln_modulation(c, b.adaLN_modulation.weight.float().cpu(), b.adaLN_modulation.bias.float().cpu())
            for b in st.blocks]
    pos = O.joint_positions([("text", cfg.n_text), ("video", cfg.grid)])
    cos, sin = O.mrope_cos_sin(pos, 64, cfg.mrope_sections)
    want = O.dm_stack(torch.cat([xtr[0], xvr[0]]), [oracle_weights(b, 1) for b in st.blocks], mods, cos, sin, 4,
                      st.segments())
    assert_close(out["joint"], want, BF16_COS, BF16_REL, "3-block stack (joint)")
    assert_close(out["sample"][0], want[cfg.n_text:], BF16_COS, BF16_REL, "3-block stack (video part)")


def test_attention_processor_diffusers_call_shape():
    """processor(attn, hidden_states, encoder_hidden_states=..., image_rotary_emb=...) -> (hidden, encoder)."""
    cfg = DMConfig("p", 256, 2, 128, 512, 1, (1, 4, 8), n_text=16, n_branches=2)
    blk = make_block(cfg, 21, randomize_norms=False)
    g = torch.Generator().manual_seed(21)
    h, hr = rand_bf16((1, 32, 256), g)
    e, er = rand_bf16((1, 16, 256), g)
    pos, _ = rotary.build_positions(16, cfg.grid)
    cos, sin = rotary.rotary_tables(pos, 128, cfg.mrope_sections)
    ho, eo = blk.attn(h, encoder_hidden_states=e, image_rotary_emb=(cos.to(dev()), sin.to(dev())))
    assert ho.shape == (1, 32, 256) and eo.shape == (1, 16, 256)
    ws = oracle_weights(blk, 2)
    xr = torch.cat([er[0], hr[0]])
    q = torch.cat([xr[:16] @ ws[0]["wq"].t(), xr[16:] @ ws[1]["wq"].t()]); k = torch.cat([xr[:16] @ ws[0]["wk"].t(), xr[16:] @ ws[1]["wk"].t()])
    v = torch.cat([xr[:16] @ ws[0]["wv"].t(), xr[16:] @ ws[1]["wv"].t()])
    o = O.attention(O.apply_mrope(q.view(48, 2, 128), cos, sin), O.apply_mrope(k.view(48, 2, 128), cos, sin), v.view(48, 2, 128)).reshape(48, 256)
    assert_close(eo[0], o[:16] @ ws[0]["wo"].t(), BF16_COS, BF16_REL, "processor encoder stream")
    assert_close(ho[0], o[16:] @ ws[1]["wo"].t(), BF16_COS, BF16_REL, "processor hidden stream")
    with pytest.raises(NotImplementedError):
        blk.attn(h, attention_mask=torch.ones(1, 32, device=dev()), image_rotary_emb=(cos.to(dev()), sin.to(dev())))


def test_fp8_block_vs_fp32_oracle():
    cfg = DMConfig("f8", 512, 4, 128, 1024, 1, (2, 8, 16), n_text=32, fp8=True)
    st = DMStack(cfg, device=dev())
    blk = make_block(cfg, 17)
    g = torch.Generator().manual_seed(17)
    x, xr = rand_bf16((cfg.n_tokens, 512), g)
    temb, tembr = rand_bf16((512,), g)
    y = blk(x, temb, st.rotary(dev()), st.segments())
    mod = O.adaln_modulation(tembr.view(1, -1), blk.adaLN_modulation.weight.float().cpu(),
                             blk.adaLN_modulation.bias.float().cpu())
    pos = O.joint_positions([("text", 32), ("video", cfg.grid)])
    cos, sin = O.mrope_cos_sin(pos, 128, cfg.mrope_sections)
    ws = oracle_weights(blk, 1)
    want32 = O.dm_block(xr, ws, mod, cos, sin, 4, st.segments())
    assert_close(y, want32, FP8_COS, FP8_REL, "fp8 block vs fp32 unquantised oracle")
    want8 = O.dm_block(xr, ws, mod, cos, sin, 4, st.segments(), fp8=True)
    assert_close(y, want8, 0.9995, 3e-2, "fp8 block vs quantised oracle")


def test_c1_full_size_attention_sampled_rows():
    """Benchmark configuration 1: 32 heads x 128, grid 16x44x80 = 56,320 tokens, mRoPE 32/48/48, bf16.
    Attention rows are independent given K and V, so exact fp32 attention on sampled query rows is an exact
    check of those rows."""
    cfg = CONFIGS["C1"]
    n, H, hd, d = cfg.n_tokens, cfg.n_heads, cfg.head_dim, cfg.d_model
    g = torch.Generator(device=dev()).manual_seed(cfg.seed)
    qkv = (torch.randn((n, 3 * d), generator=g, device=dev()) / (hd ** 0.5)).to(torch.bfloat16)
    pos, _ = rotary.build_positions(0, cfg.grid)
    cos, sin = rotary.rotary_tables(pos, hd, cfg.mrope_sections)
    pre = qkv
    q, k, v = qkv[:, :d], qkv[:, d:2 * d], qkv[:, 2 * d:]
    o = ops.attention(q, k, v, H, hd, cos=cos.to(dev()), sin=sin.to(dev()))      # mRoPE in registers
    torch.cuda.synchronize()
    rows = torch.cat([torch.tensor([0, 1, 31, 32, 255, 256, n - 1, n - 64]),
                      torch.randint(0, n, (56,), generator=torch.Generator().manual_seed(1))])
    heads = [0, 13, 31]                                       # three heads keep the CPU side to a few seconds
    for h in heads:
        sl = slice(h * hd, (h + 1) * hd)
        kr = O.apply_mrope(pre[:, d + h * hd:d + (h + 1) * hd].float().cpu().view(n, 1, hd), cos, sin)
        qr = O.apply_mrope(pre[rows.to(dev()), sl].float().cpu().view(-1, 1, hd), cos[rows], sin[rows])
        vr = pre[:, 2 * d + h * hd:2 * d + (h + 1) * hd].float().cpu().view(n, 1, hd)
        want = O.attention_rows(qr, kr, vr).reshape(-1, hd)
        assert_close(o[rows.to(dev()), sl], want, BF16_COS, BF16_REL, f"C1 attention head {h}")
    # size-independent property on the whole output: every output row is a convex combination of V rows
    vmin, vmax = v.float().amin(0), v.float().amax(0)
    of = o.float()
    assert bool((of >= vmin - 1e-2).all()) and bool((of <= vmax + 1e-2).all())
    # the kernel has no atomics and a fixed summation order: repeated launches agree bit for bit.  A tile read
    # before it has landed in LDS shows up here as a last-bit difference in a few rows (one tile of 880 is
    # below the bf16 resolution of the output, so the comparison with the oracle above cannot see it).
    for _ in range(4):
        again = ops.attention(q, k, v, H, hd, cos=cos.to(dev()), sin=sin.to(dev()))
        assert torch.equal(o, again), "attention output differs between identical launches"


def test_full_size_attention_with_outlier_keys():
    """56,832 tokens (the joint length of benchmark configuration 2), 32 heads x 128, mRoPE in registers, with one
    outlier key in each of two heads.  The kernel decides per key tile and per wave whether the tile's key-norm bound
    allows it to skip the row maxima: head 0 gets an outlier whose norm is the MEDIAN of the waves' thresholds, so in
    that one tile about half of the waves of every workgroup take the maxima and the others do not (mixed waves in
    one workgroup, at full size); head 13 gets a key of norm 4000 that beats everything else by far more than 2^60
    for many rows (the reference moves by a hundred and more).  All other tiles of both heads, and every tile of the other
    heads, run without maxima.  Sampled rows against the fp32 oracle, and bit-reproducibility."""
    cfg = CONFIGS["C2"]
    n, H, hd, d = cfg.n_tokens, cfg.n_heads, cfg.head_dim, cfg.d_model
    g = torch.Generator(device=dev()).manual_seed(77)
    qkv = (torch.randn((n, 3 * d), generator=g, device=dev()) / (hd ** 0.5)).to(torch.bfloat16)
    pos, _ = rotary.build_positions(cfg.n_text, cfg.grid)
    cos, sin = rotary.rotary_tables(pos, hd, cfg.mrope_sections)
    cg, sg = cos.to(dev()), sin.to(dev())
    # the waves' thresholds in head 0, restated on the host: a wave owns 32 consecutive query rows; a row tolerates a
    # tile whose largest key norm is at most (60 + m0) / (1.01 |q'|), q' = rotated Q times log2(e)/sqrt(hd), m0 = its
    # largest score against the first 64 keys
    c = 1.4426950408889634 / hd ** 0.5
    q0 = O.apply_mrope(qkv[:, :hd].float().view(n, 1, hd), cg, sg).view(n, hd) * c
    k0 = O.apply_mrope(qkv[:64, d:d + hd].float().view(64, 1, hd), cg[:64], sg[:64]).view(64, hd)
    thr = (60.0 + (q0 @ k0.t()).amax(1)) / (1.01 * q0.norm(dim=1))
    t_wave = thr.view(-1, 32).amin(1)
    spike0 = float(t_wave.median())
    assert 100.0 < spike0 < 2000.0
    per_wg = (t_wave.view(-1, 8) >= spike0).float().mean(1)
    assert float(((per_wg > 0) & (per_wg < 1)).float().mean()) > 0.9      # both kinds of waves in most workgroups
    at0, at13 = 40000, 100
    u = torch.randn(2, hd, generator=g, device=dev())
    u = u / u.norm(dim=1, keepdim=True)
    qkv[at0, d:d + hd] = (u[0] * spike0).to(torch.bfloat16)
    qkv[at13, d + 13 * hd:d + 14 * hd] = (u[1] * 4000.0).to(torch.bfloat16)
    q, k, v = qkv[:, :d], qkv[:, d:2 * d], qkv[:, 2 * d:]
    o = ops.attention(q, k, v, H, hd, cos=cg, sin=sg)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(o.float()).all())
    rows = torch.cat([torch.tensor([0, 1, 31, 32, 255, 256, n - 1, n - 64, at0, at13]),
                      torch.randint(0, n, (54,), generator=torch.Generator().manual_seed(2))])
    for h in (0, 13, 5):
        sl = slice(h * hd, (h + 1) * hd)
        kr = O.apply_mrope(qkv[:, d + h * hd:d + (h + 1) * hd].float().cpu().view(n, 1, hd), cos, sin)
        qr = O.apply_mrope(qkv[rows.to(dev()), sl].float().cpu().view(-1, 1, hd), cos[rows], sin[rows])
        vr = qkv[:, 2 * d + h * hd:2 * d + (h + 1) * hd].float().cpu().view(n, 1, hd)
        want = O.attention_rows(qr, kr, vr).reshape(-1, hd)
        if h == 13:      # the spike decides many rows: they return (nearly) V of the outlier key
            sc = (qr.view(-1, hd) @ kr.view(n, hd).t()) * c
            assert int(((sc[:, at13] - sc.amax(1)) == 0).sum()) >= 10 and float(sc[:, at13].amax()) > 80.0
        assert_close(o[rows.to(dev()), sl], want, BF16_COS, BF16_REL, f"full-size attention with outlier keys, head {h}")
    for _ in range(3):
        again = ops.attention(q, k, v, H, hd, cos=cg, sin=sg)
        assert torch.equal(o, again), "attention output differs between identical launches"


def test_transformer_with_stack_edges_and_loaded_checkpoint(tmp_path):
    """latents -> patchify/proj_in -> 2 MoT blocks (QK-norm) -> final norm -> proj_out/unpatchify, with the weights
    taken through a safetensors file; checked against the fp32 oracle composed from the same tensors."""
    from safetensors.torch import save_file
    from cosmos_amd import DMTransformer, export_generator_weights, load_generator_weights
    cfg = DMConfig("edge", 256, 2, 128, 512, 2, (2, 3, 4), n_text=12, n_action=5, n_branches=3, qk_norm=True)
    src = DMTransformer(cfg, latent_channels=4, action_dim=6, device=dev())
    src.reset_parameters(31)
    g = torch.Generator(device=dev()).manual_seed(31)
    with torch.no_grad():
        for blk in src.stack.blocks:
            blk.attn.norm_q_weight.copy_(1 + 0.2 * torch.randn(3, 128, generator=g, device=dev()))
            blk.attn.norm_k_weight.copy_(1 + 0.2 * torch.randn(3, 128, generator=g, device=dev()))
            blk.adaLN_modulation.bias.copy_(0.2 * torch.randn(blk.adaLN_modulation.bias.shape, generator=g, device=dev()))
        src.norm_out.copy_(1 + 0.2 * torch.randn(256, generator=g, device=dev()))
        src.action_modality_embed.copy_(0.5 * torch.randn(256, generator=g, device=dev()))
    # the third (action) branch has no attested key names: it travels as the DM names of an extra mapping
    path = str(tmp_path / "gen.safetensors")
    save_file({k: v.contiguous().cpu() for k, v in export_generator_weights(src).items()}, path)
    m = DMTransformer(cfg, latent_channels=4, action_dim=6, device=dev())
    m.reset_parameters(99)
    rep = load_generator_weights(m, path)
    assert not rep["unexpected"] and all(".2" in k for k in rep["missing"])     # only branch 2 is absent from the file
    with torch.no_grad():
        for bs, bm in zip(src.stack.blocks, m.stack.blocks):
            for name in ("norm1_weight", "norm2_weight", "gate_weight", "up_weight", "down_weight"):
                getattr(bm, name)[2].copy_(getattr(bs, name)[2])
            bm.attn.qkv_weight[2].copy_(bs.attn.qkv_weight[2]); bm.attn.out_weight[2].copy_(bs.attn.out_weight[2])
            bm.attn.norm_q_weight[2].copy_(bs.attn.norm_q_weight[2]); bm.attn.norm_k_weight[2].copy_(bs.attn.norm_k_weight[2])
    gc = torch.Generator().manual_seed(32)
    lat = torch.randn(1, 4, 2, 6, 8, generator=gc)
    ctx, ctxr = rand_bf16((1, 12, 256), gc)
    act, actr = rand_bf16((1, 5, 6), gc)
    t = torch.tensor([640.0])
    out = m(lat.to(dev()), t.to(dev()), encoder_hidden_states=ctx, action_states=act, return_dict=True)
    out_src = src(lat.to(dev()), t.to(dev()), encoder_hidden_states=ctx, action_states=act, return_dict=True)
    assert torch.equal(out["sample"], out_src["sample"])            # the file carried every tensor exactly
    # oracle composition (fp32)
    f = lambda p: p.detach().float().cpu()
    latb = lat.to(torch.bfloat16).float()
    tok = m.patchify(latb[0]) @ f(m.proj_in.weight).t() + f(m.proj_in.bias)
    a_in = actr[0] @ f(m.action_proj_in.weight).t() + f(m.action_proj_in.bias) + f(m.action_modality_embed)
    x = torch.cat([ctxr[0], tok, a_in])
    te = m.time_embedder
    c = O.time_mlp(O.timestep_embedding(t), f(te.linear_1.weight), f(te.linear_1.bias), f(te.linear_2.weight), f(te.linear_2.bias))
    mods = [O.adaln_modulation(c, f(b.adaLN_modulation.weight), f(b.adaLN_modulation.bias)) for b in m.stack.blocks]
    pos = O.joint_positions([("text", 12), ("video", cfg.grid), ("action", 5)])
    cos, sin = O.mrope_cos_sin(pos, 128, cfg.mrope_sections)
    y = O.dm_stack(x, [oracle_weights(b, 3) for b in m.stack.blocks], mods, cos, sin, 2, m.stack.segments())
    y = O.rms_norm(y, f(m.norm_out), cfg.eps)
    want = m.unpatchify(y[12:12 + cfg.n_video] @ f(m.proj_out.weight).t() + f(m.proj_out.bias))
    assert out["sample"].shape == lat.shape
    assert_close(out["sample"], want, BF16_COS, BF16_REL, "transformer with stack edges")
    want_act = y[12 + cfg.n_video:] @ f(m.action_proj_out.weight).t() + f(m.action_proj_out.bias)
    assert_close(out["action"][0], want_act, BF16_COS, BF16_REL, "action head")


@pytest.mark.parametrize("n_kv_heads,P", [(None, 64), (1, 64), (None, 70), (1, 37)])
def test_hybrid_mask_stack_and_context_reuse(n_kv_heads, P):
    """Two-branch stack under the hybrid mask: (1) joint forward vs the masked fp32 oracle; (2) the text run's K/V
    packed once per prompt and reused: same video output from a forward that carries only the generator tokens;
    (3) the reused cache stays valid for another timestep.  Also with one K/V head for the two query heads (the kept
    images then hold K/V heads only), and with text runs that do not fill their last 64-key tile (70, 37 tokens: the joint
    forward then takes the GEMM + re-tiling pair for the segments off a tile boundary, the cached forward masks the padding
    of the prefix images)."""
    cfg = DMConfig("hyb", 256, 2, 128, 512, 2, (2, 5, 8), n_text=P, n_action=7, n_branches=3, qk_norm=True,
                   hybrid_mask=True, n_kv_heads=n_kv_heads)
    st = DMStack(cfg, device=dev())
    st.reset_parameters(41)
    g = torch.Generator(device=dev()).manual_seed(41)
    with torch.no_grad():
        for blk in st.blocks:
            blk.attn.norm_q_weight.copy_(1 + 0.2 * torch.randn(3, 128, generator=g, device=dev()))
            blk.attn.norm_k_weight.copy_(1 + 0.2 * torch.randn(3, 128, generator=g, device=dev()))
            blk.adaLN_modulation.bias.copy_(0.2 * torch.randn(blk.adaLN_modulation.bias.shape, generator=g, device=dev()))
    gc = torch.Generator().manual_seed(42)
    xv, xvr = rand_bf16((1, cfg.n_video, 256), gc)
    xt, xtr = rand_bf16((1, P, 256), gc)
    xa, xar = rand_bf16((1, 7, 256), gc)
    t = torch.tensor([333.0])
    out = st(xv, t.to(dev()), encoder_hidden_states=xt, action_states=xa, return_dict=True)
    te = st.time_embedder
    f = lambda p: p.detach().float().cpu()
    c = O.time_mlp(O.timestep_embedding(t), f(te.linear_1.weight), f(te.linear_1.bias), f(te.linear_2.weight), f(te.linear_2.bias))
    mods = [O.adaln_modulation(c, f(b.adaLN_modulation.weight), f(b.adaLN_modulation.bias)) for b in st.blocks]
    pos = O.joint_positions([("text", P), ("video", cfg.grid), ("action", 7)])
    cos, sin = O.mrope_cos_sin(pos, 128, cfg.mrope_sections)
    x0 = torch.cat([xtr[0], xvr[0], xar[0]])
    want = O.dm_stack(x0, [oracle_weights(b, 3) for b in st.blocks], mods, cos, sin, 2, st.segments(), causal_prefix=P)
    assert_close(out["joint"], want, BF16_COS, BF16_REL, "hybrid-mask stack (joint)")
    want_full = O.dm_stack(x0, [oracle_weights(b, 3) for b in st.blocks], mods, cos, sin, 2, st.segments())
    assert O.max_rel_err(want[:P], want_full[:P]) > 1e-2           # the mask is live
    # (2) context reuse
    cache = st.precompute_context(xt)
    out2 = st(xv, t.to(dev()), action_states=xa, return_dict=True, context_cache=cache)
    assert_close(out2["sample"][0], out["sample"][0].float().cpu(), 0.99999, 4e-3, "cached context == joint forward")
    assert_close(out2["sample"][0], want[P:P + cfg.n_video], BF16_COS, BF16_REL, "cached context vs oracle")
    # (3) another timestep with the same cache
    t2 = torch.tensor([871.0])
    out3 = st(xv, t2.to(dev()), action_states=xa, return_dict=True, context_cache=cache)
    ref3 = st(xv, t2.to(dev()), encoder_hidden_states=xt, action_states=xa, return_dict=True)
    assert_close(out3["sample"][0], ref3["sample"][0].float().cpu(), 0.99999, 4e-3, "cache reused at another timestep")
    # without the hybrid mask the reuse is refused
    cfg_full = DMConfig("full", 256, 2, 128, 512, 1, (2, 5, 8), n_text=64)
    with pytest.raises(RuntimeError):
        DMStack(cfg_full, device=dev()).precompute_context(xt)


@pytest.mark.parametrize("fp8", [False, True])
def test_c2_full_size_gemms_sampled_rows(fp8):
    """The four linear layers of a block at the full C2 / C4 shape (56,832 tokens, d 4096, hidden 16384) on the GPU;
    512 sampled token rows are recomputed in fp32 on the host (rows of a linear layer are independent, so a row
    sample is an exact check of those rows), plus linearity in the activation at full size."""
    N, d, h = 56832, 4096, 16384
    g = torch.Generator(device=dev()).manual_seed(1236)
    rnd = lambda *s, sd=1.0: (torch.randn(s, generator=g, device=dev()) * sd).to(torch.bfloat16)
    x, hid = rnd(N, d), rnd(N, h)
    wqkv, wo, wg, wu, wd = rnd(3 * d, d, sd=0.02), rnd(d, d, sd=0.02), rnd(h, d, sd=0.02), rnd(h, d, sd=0.02), rnd(d, h, sd=0.02)
    res = rnd(N, d)
    gate = torch.randn(d, generator=g, device=dev())
    rows = torch.randperm(N, generator=torch.Generator().manual_seed(3))[:512].sort().values
    rd = rows.to(dev())
    f = lambda t: t.float().cpu()
    xs, hs, rs = f(x[rd]), f(hid[rd]), f(res[rd])
    tol = (FP8_COS, FP8_REL) if fp8 else (BF16_COS, 1e-2)
    if fp8:
        xq, sx = ops.quant_rows(x); hq, sh = ops.quant_rows(hid)
        q = {n: ops.quant_rows(w) for n, w in dict(qkv=wqkv, o=wo, g=wg, u=wu, d=wd).items()}
        qkv = ops.gemm_fp8(xq, sx, *q["qkv"])
        o = ops.gemm_fp8(xq, sx, *q["o"], epilogue="gate_residual", residual=res, gate=gate)
        hh = ops.gemm_fp8(xq, sx, *q["g"], w2q=q["u"][0], sw2=q["u"][1], epilogue="swiglu")
        dn = ops.gemm_fp8(hq, sh, *q["d"], epilogue="gate_residual", residual=res, gate=gate)
    else:
        qkv = ops.gemm(x, wqkv)
        o = ops.gemm(x, wo, epilogue="gate_residual", residual=res, gate=gate)
        hh = ops.gemm(x, wg, w2=wu, epilogue="swiglu")
        dn = ops.gemm(hid, wd, epilogue="gate_residual", residual=res, gate=gate)
    assert_close(qkv[rd], xs @ f(wqkv).t(), *tol, "QKV rows")
    assert_close(o[rd], rs + f(gate) * (xs @ f(wo).t()), *tol, "out-proj + gated residual rows")
    assert_close(hh[rd], torch.nn.functional.silu(xs @ f(wg).t()) * (xs @ f(wu).t()), tol[0] - (0.002 if fp8 else 0), tol[1] * (1.6 if fp8 else 1), "SwiGLU rows")
    assert_close(dn[rd], rs + f(gate) * (hs @ f(wd).t()), *tol, "down-proj + gated residual rows")
    assert bool(torch.isfinite(qkv.float()).all()) and bool(torch.isfinite(dn.float()).all())
    if not fp8:
        # linearity at full size: gemm(2x) == 2 gemm(x) exactly (a power of two commutes with every rounding)
        assert torch.equal(ops.gemm(x * 2, wo), qkv.new_tensor(2.0) * ops.gemm(x, wo))


@pytest.mark.parametrize("name", ["C2", "C3", "C4"])
def test_full_size_block_is_bit_reproducible(name):
    """One block of each full-size benchmark configuration, run four times on the same input.  No kernel on the path
    uses atomics or an order that depends on timing, so the outputs must agree bit for bit; a difference means
    that some wave read a tile (LDS ring slot, staged row) before it was complete."""
    import dataclasses
    cfg = dataclasses.replace(CONFIGS[name], n_blocks=1)
    st = DMStack(cfg, device=dev())
    st.reset_parameters()
    g = torch.Generator(device=dev()).manual_seed(7)
    with torch.no_grad():
        for b in st.blocks:
            b.adaLN_modulation.bias.copy_(0.5 * torch.randn(b.adaLN_modulation.bias.shape, generator=g, device=dev()))
    mk = lambda n: torch.randn((1, n, cfg.d_model), generator=g, device=dev()).to(torch.bfloat16)
    x, kw = mk(cfg.n_video), {}
    if cfg.n_text:
        kw["encoder_hidden_states"] = mk(cfg.n_text)
    if cfg.n_action:
        kw["action_states"] = mk(cfg.n_action)
    t = torch.tensor([500.0], device=dev())
    (first,) = st(x, t, **kw)
    first = first.clone()
    assert bool(torch.isfinite(first.float()).all())
    assert float((first.float() - x.float()).abs().max()) > 0.1          # the block does something
    for _ in range(3):
        (again,) = st(x, t, **kw)
        assert torch.equal(first, again), f"{name}: block output differs between identical launches"


def test_c2_full_size_cached_context_forward():
    """One production forward at the size of benchmark configuration 2 under the hybrid mask: the 512-token text run is
    packed once (``precompute_context``: its K / V tile images per layer), then the 56,320 generator tokens run alone
    against those prefix images.  Sampled generator rows against the masked fp32 oracle of the joint sequence; the
    joint forward (text and video together) must give the same video rows; two cached forwards agree bit for bit."""
    import dataclasses
    cfg = dataclasses.replace(CONFIGS["C2"], n_blocks=1, hybrid_mask=True)
    st = DMStack(cfg, device=dev())
    st.reset_parameters()
    blk = st.blocks[0]
    g = torch.Generator(device=dev()).manual_seed(23)
    with torch.no_grad():      # order-one modulation, so that both residual updates are visible in the output
        blk.adaLN_modulation.bias.copy_(torch.randn(blk.adaLN_modulation.bias.shape, generator=g, device=dev()))
    P, n, d = cfg.n_text, cfg.n_tokens, cfg.d_model
    xt = torch.randn((1, P, d), generator=g, device=dev()).to(torch.bfloat16)
    xv = torch.randn((1, cfg.n_video, d), generator=g, device=dev()).to(torch.bfloat16)
    t = torch.tensor([640.0], device=dev())
    cache = st.precompute_context(xt)
    out = st(xv, t, return_dict=True, context_cache=cache)
    first = out["joint"].clone()
    torch.cuda.synchronize()
    assert first.shape == (cfg.n_video, d) and bool(torch.isfinite(first).all())
    # oracle on sampled generator rows (first / last rows, rows next to tile and query-block boundaries, random ones)
    te = st.time_embedder
    f = lambda p: p.detach().float().cpu()
    c = O.time_mlp(O.timestep_embedding(t.cpu()), f(te.linear_1.weight), f(te.linear_1.bias), f(te.linear_2.weight), f(te.linear_2.bias))
    mod = O.adaln_modulation(c, f(blk.adaLN_modulation.weight), f(blk.adaLN_modulation.bias))
    pos = O.joint_positions([("text", P), ("video", cfg.grid)])
    cos, sin = O.mrope_cos_sin(pos, cfg.head_dim, cfg.mrope_sections, cfg.rope_base, cfg.rope_layout)
    rows = torch.tensor(sorted({P, P + 1, P + 63, P + 64, P + 255, P + 256, n - 1, n - 64, n - 257})
                        + (P + torch.randint(0, cfg.n_video, (20,), generator=torch.Generator().manual_seed(5))).tolist())
    xj = torch.cat([xt[0], xv[0]]).float().cpu()
    want = O.dm_block(xj, oracle_weights(blk, 1), mod, cos, sin, cfg.n_heads, st.segments(), attn_rows=rows, causal_prefix=P)
    got = first[(rows - P).to(dev())]
    assert_close(got, want, BF16_COS, BF16_REL, "C2 cached-context forward at full size, sampled generator rows")
    upd = xj[rows]
    assert float((want - upd).abs().max()) > 0.5
    assert_close(got.float().cpu() - upd, want - upd, 0.999, BF16_REL, "C2 cached-context forward: the update alone")
    # the joint forward under the same mask gives the same video rows; a tolerance instead of equality: 220 query blocks
    # per head end in half a round of workgroups, which the cached forward splits by key range (its partial results are
    # rounded to bf16 once more), while the joint forward's 222 are left alone
    joint = st(xv, t, encoder_hidden_states=xt, return_dict=True)["joint"]
    assert_close(first, joint[P:].float().cpu(), 0.99999, 8e-3, "cached context == joint forward at full size")
    again = st(xv, t, return_dict=True, context_cache=cache)["joint"]
    assert torch.equal(first, again), "cached-context forward differs between identical launches"


@pytest.mark.parametrize("name", ["C2", "C3", "C4"])
def test_full_size_block_sampled_rows(name):
    """One whole block at the full size of benchmark configurations 2 (56,832 tokens, text + video, one weight set),
    3 (29,440 tokens, three MoT weight sets, hybrid mask) and 4 (configuration 2 with e4m3 GEMMs, held to the fp8
    tolerance against the UNQUANTISED oracle) against the fp32 oracle.  The oracle computes Q, K, V
    of every token and carries a sample of token rows through attention, out-projection and MLP: attention rows
    are independent given K and V and everything after attention is row-wise, so those rows are checked exactly."""
    import dataclasses
    cfg = dataclasses.replace(CONFIGS[name], n_blocks=1, hybrid_mask=(name == "C3"))
    st = DMStack(cfg, device=dev())
    st.reset_parameters()
    blk = st.blocks[0]
    g = torch.Generator(device=dev()).manual_seed(17)
    n, d = cfg.n_tokens, cfg.d_model
    x = torch.randn((n, d), generator=g, device=dev()).to(torch.bfloat16)
    # order-one modulation, gates included, so that both residual updates are visible in the output
    gs = 1.0 if cfg.fp8 else 4.0
    mod = [torch.randn(d, generator=g, device=dev()) * s for s in (0.5, 0.5, gs, 0.5, 0.5, gs)]
    segs = st.segments()
    P = cfg.n_text if cfg.hybrid_mask else 0
    y = blk(x, None, st.rotary(dev()), segs, modulation=mod, causal_prefix=P)
    torch.cuda.synchronize()
    bounds = sorted({0, 1, n - 1, n - 64} | {s0 for (s0, _, _, _) in segs} | {s0 + ln - 1 for (s0, ln, _, _) in segs}
                    | ({P - 1, P, 255, 256} if P else set()))
    rows = torch.tensor(bounds + torch.randint(0, n, (24,), generator=torch.Generator().manual_seed(3)).tolist())
    pos = O.joint_positions(([("text", cfg.n_text)] if cfg.n_text else []) + [("video", cfg.grid)] +
                            ([("action", cfg.n_action)] if cfg.n_action else []))
    cos, sin = O.mrope_cos_sin(pos, cfg.head_dim, cfg.mrope_sections, cfg.rope_base, cfg.rope_layout)
    want = O.dm_block(x.float().cpu(), oracle_weights(blk, cfg.n_branches), [m.float().cpu() for m in mod], cos, sin,
                      cfg.n_heads, segs, attn_rows=rows, causal_prefix=P)
    got = y[rows.to(dev())]
    upd = x[rows.to(dev())].float().cpu()
    if cfg.fp8:
        want8 = O.dm_block(x.float().cpu(), oracle_weights(blk, cfg.n_branches), [m.float().cpu() for m in mod], cos, sin,
                           cfg.n_heads, segs, attn_rows=rows, causal_prefix=P, fp8=True)
        # e4m3 operands carry about 5 % noise per product on random data whatever K is, so with order-one gates not
        # even the oracle that quantises at the same places stays within 5e-2 of the fp32 one.  What the kernels owe
        # is the recipe: they must be much closer to the quantising oracle than that oracle is to fp32 ...
        noise_cos, noise_rel = 1.0 - O.cos_sim(want8, want), O.max_rel_err(want8, want)
        record(f"{name} full-size block vs the quantising oracle (limits: 0.6 x and 1.5 x that oracle's distance to fp32)",
               O.cos_sim(got, want8), O.max_rel_err(got, want8), 1.0 - 0.6 * noise_cos, 1.5 * noise_rel)
        assert 1.0 - O.cos_sim(got, want8) < 0.6 * noise_cos, (O.cos_sim(got, want8), noise_cos)
        # (the maximum is one element out of 200,000: a per-token scale that differs in its last bit moves the whole
        # row's e4m3 grid, so the largest single deviation from the quantising oracle is of the size of the recipe's own
        # largest deviation - measured 1.07 x - while the energy of the difference, the cosine above, is half of it)
        assert O.max_rel_err(got, want8) < 1.5 * noise_rel, (O.max_rel_err(got, want8), noise_rel)
        assert O.max_rel_err(got, want) < 1.25 * noise_rel and 1.0 - O.cos_sim(got, want) < 1.25 * noise_cos
        # ... and with the benchmark's own modulation (time embedding through N(0, 0.02) weights: small gates) the
        # block is within the fp8 tolerance of the UNQUANTISED oracle
        t = torch.tensor([500.0], device=dev())
        temb = st.time_embedder(t)
        y_nat = blk(x, temb, st.rotary(dev()), segs, causal_prefix=P)
        te = st.time_embedder
        c = O.time_mlp(O.timestep_embedding(t.cpu()), te.linear_1.weight.float().cpu(), te.linear_1.bias.float().cpu(),
                       te.linear_2.weight.float().cpu(), te.linear_2.bias.float().cpu())
        mod_nat = O.adaln_modulation(c, blk.adaLN_modulation.weight.float().cpu(), blk.adaLN_modulation.bias.float().cpu())
        ow = oracle_weights(blk, cfg.n_branches)
        want_nat = O.dm_block(x.float().cpu(), ow, mod_nat, cos, sin, cfg.n_heads, segs, attn_rows=rows, causal_prefix=P)
        got_nat = y_nat[rows.to(dev())]
        gated = torch.zeros(len(rows), dtype=torch.bool)
        for (s0, ln, _, modulated) in segs:
            if modulated:
                gated |= (rows >= s0) & (rows < s0 + ln)
        # generator rows (adaLN-gated): inside the fp8 tolerance of the unquantised oracle
        assert_close(got_nat[gated.to(dev())], want_nat[gated], FP8_COS, FP8_REL, f"{name} full-size block, gated rows vs fp32 oracle")
        # text rows have no gate (their updates enter at full size), so there the recipe's own noise exceeds 5e-2 of
        # the output range: hold the kernels to the noise of the quantising oracle on the same rows instead
        want8_nat = O.dm_block(x.float().cpu(), ow, mod_nat, cos, sin, cfg.n_heads, segs, attn_rows=rows, causal_prefix=P,
                               fp8=True)
        ung = ~gated
        assert int(ung.sum()) >= 2
        noise = O.max_rel_err(want8_nat[ung], want_nat[ung])
        assert O.max_rel_err(got_nat[ung.to(dev())], want_nat[ung]) < 1.25 * noise
        assert O.max_rel_err(got_nat[ung.to(dev())], want8_nat[ung]) < noise
    else:
        assert_close(got, want, BF16_COS, BF16_REL, f"{name} full-size block, sampled rows")
        assert float((want - upd).abs().max()) > 0.5
        assert_close(got.float().cpu() - upd, want - upd, 0.999, BF16_REL, f"{name} full-size block update")


def test_batched_forward_is_a_loop_over_samples():
    """A batch (e.g. the conditional and unconditional pass of classifier-free guidance as a batch of two) gives the
    per-sample results, sample by sample: per-sample timesteps and contexts, a shared context when its batch is 1."""
    from cosmos_amd import DMTransformer
    cfg = DMConfig("bt", 256, 2, 128, 512, 2, (2, 3, 4), n_text=12, n_action=5, n_branches=3, qk_norm=True)
    m = DMTransformer(cfg, latent_channels=4, action_dim=6, device=dev())
    m.reset_parameters(5)
    g = torch.Generator(device=dev()).manual_seed(5)
    lat = torch.randn((2, 4, 2, 6, 8), generator=g, device=dev())
    ctx = torch.randn((2, 12, 256), generator=g, device=dev()).to(torch.bfloat16)
    act = torch.randn((2, 5, 6), generator=g, device=dev())
    t = torch.tensor([100.0, 900.0], device=dev())
    both = m(lat, t, encoder_hidden_states=ctx, action_states=act)
    assert both[0].shape == (2, 4, 2, 6, 8) and both[1].shape[0] == 2
    for b in range(2):
        one = m(lat[b:b + 1], t[b:b + 1], encoder_hidden_states=ctx[b:b + 1], action_states=act[b:b + 1])
        assert torch.equal(both[0][b:b + 1], one[0]) and torch.equal(both[1][b:b + 1], one[1])
    assert not torch.equal(both[0][0], both[0][1])
    shared = m(lat, t, encoder_hidden_states=ctx[:1], action_states=act)          # one context for both samples
    assert torch.equal(shared[0][0], both[0][0]) and not torch.equal(shared[0][1], both[0][1])
    d = m.stack(torch.randn((2, cfg.n_video, 256), generator=g, device=dev()).to(torch.bfloat16), t, encoder_hidden_states=ctx,
                action_states=torch.randn((2, 5, 256), generator=g, device=dev()).to(torch.bfloat16), return_dict=True)
    assert d["sample"].shape == (2, cfg.n_video, 256) and d["joint"].shape == (2, cfg.n_tokens, 256)


class _RMSNorm(torch.nn.Module):
    def __init__(self, dim, eps=1e-6):
        super().__init__()
        self.weight, self.eps = torch.nn.Parameter(torch.ones(dim)), eps


class _JointAttention(torch.nn.Module):
    """Stand-in for the attention module of the reference's transformer: nothing but the attested sub-module names
    (to_q / to_k / to_v / to_out[0], add_q_proj / add_k_proj / add_v_proj / to_add_out, norm_q / norm_k /
    norm_added_q / norm_added_k), a head count and the diffusers processor plumbing."""

    def __init__(self, d, heads, kv_heads, qk_norm=True):
        super().__init__()
        L = lambda i, o: torch.nn.Linear(i, o, bias=False)
        hd = d // heads
        self.heads = heads
        self.to_q, self.to_k, self.to_v = L(d, d), L(d, kv_heads * hd), L(d, kv_heads * hd)
        self.to_out = torch.nn.ModuleList([L(d, d), torch.nn.Dropout(0.0)])
        self.add_q_proj, self.add_k_proj, self.add_v_proj, self.to_add_out = L(d, d), L(d, kv_heads * hd), L(d, kv_heads * hd), L(d, d)
        if qk_norm:
            self.norm_q, self.norm_k, self.norm_added_q, self.norm_added_k = (_RMSNorm(hd) for _ in range(4))
        self.processor = None

    def set_processor(self, processor):
        self.processor = processor

    def forward(self, hidden_states, encoder_hidden_states=None, attention_mask=None, image_rotary_emb=None, **kw):
        return self.processor(self, hidden_states, encoder_hidden_states=encoder_hidden_states,
                              attention_mask=attention_mask, image_rotary_emb=image_rotary_emb, **kw)


@pytest.mark.parametrize("kv_heads", [2, 1])
def test_processor_drops_onto_a_diffusers_style_attention_module(kv_heads):
    """attn.set_processor(DMAttnProcessor()) on a module that only carries the reference's sub-module names: the fused
    QKV views are built once, the module's own weights become views of them (one copy of the weights), and the result
    matches the oracle; a later change of the weights is picked up."""
    from cosmos_amd import DMAttnProcessor
    d, heads, hd, n_ctx, n_lat = 256, 2, 128, 16, 32
    torch.manual_seed(3)
    attn = _JointAttention(d, heads, kv_heads).to(dev()).to(torch.bfloat16)
    with torch.no_grad():
        for p in attn.parameters():
            p.copy_(torch.randn_like(p.float()) * (0.06 if p.dim() == 2 else 0.3) + (0.0 if p.dim() == 2 else 1.0))
    attn.set_processor(DMAttnProcessor())
    n_bytes_before = sum(p.numel() * p.element_size() for p in attn.parameters())
    g = torch.Generator().manual_seed(21)
    h, hr = rand_bf16((1, n_lat, d), g)
    e, er = rand_bf16((1, n_ctx, d), g)
    pos, _ = rotary.build_positions(n_ctx, (1, 4, 8))
    cos, sin = rotary.rotary_tables(pos, hd, (32, 48, 48))
    rot = (cos.to(dev()), sin.to(dev()))

    def oracle():
        f = lambda m: m.weight.detach().float().cpu()
        x = torch.cat([er[0], hr[0]])
        br = [(attn.to_q, attn.to_k, attn.to_v, attn.to_out[0], attn.norm_q, attn.norm_k),
              (attn.add_q_proj, attn.add_k_proj, attn.add_v_proj, attn.to_add_out, attn.norm_added_q, attn.norm_added_k)]
        sl = [slice(0, n_ctx), slice(n_ctx, n_ctx + n_lat)]
        q = torch.cat([O.rms_norm((x[s] @ f(b[0]).t()).view(-1, heads, hd), f(b[4])).reshape(-1, d) for b, s in zip(br, sl)])
        k = torch.cat([O.rms_norm((x[s] @ f(b[1]).t()).view(-1, kv_heads, hd), f(b[5])).reshape(-1, kv_heads * hd) for b, s in zip(br, sl)])
        v = torch.cat([x[s] @ f(b[2]).t() for b, s in zip(br, sl)])
        n = n_ctx + n_lat
        o = O.attention(O.apply_mrope(q.view(n, heads, hd), cos, sin), O.apply_mrope(k.view(n, kv_heads, hd), cos, sin),
                        v.view(n, kv_heads, hd)).reshape(n, d)
        return o[n_ctx:] @ f(attn.to_add_out).t(), o[:n_ctx] @ f(attn.to_out[0]).t()

    ho, eo = attn(h, encoder_hidden_states=e, image_rotary_emb=rot)
    assert ho.shape == (1, n_lat, d) and eo.shape == (1, n_ctx, d)
    want_h, want_e = oracle()
    assert_close(ho[0], want_h, BF16_COS, BF16_REL, "adopted module: latent stream")
    assert_close(eo[0], want_e, BF16_COS, BF16_REL, "adopted module: context stream")
    # one copy of the weights: q / k / v of a branch are consecutive row ranges of one fused tensor
    dkv = kv_heads * hd
    assert attn.to_k.weight.data_ptr() == attn.to_q.weight.data_ptr() + d * d * 2
    assert attn.add_v_proj.weight.data_ptr() == attn.add_q_proj.weight.data_ptr() + (d + dkv) * d * 2
    assert sum(p.numel() * p.element_size() for p in attn.parameters()) == n_bytes_before
    assert "_cdm_adopted" not in dict(attn.named_modules()) and all("cdm" not in k for k in attn.state_dict())
    adopted = attn.__dict__["_cdm_adopted"]
    ho2, _ = attn(h, encoder_hidden_states=e, image_rotary_emb=rot)
    assert attn.__dict__["_cdm_adopted"] is adopted and torch.equal(ho, ho2)          # built once
    # load_state_dict writes through the views; a replaced norm weight is noticed
    sd = {k: (v.float() * 1.5).to(v.dtype) if k.startswith("add_v_proj") else v.clone() for k, v in attn.state_dict().items()}
    attn.load_state_dict(sd)
    with torch.no_grad():
        attn.norm_added_q.weight.mul_(0.5)
    ho3, eo3 = attn(h, encoder_hidden_states=e, image_rotary_emb=rot)
    want_h3, want_e3 = oracle()
    assert O.max_rel_err(want_h3, want_h) > 5e-2
    assert_close(ho3[0], want_h3, BF16_COS, BF16_REL, "adopted module after a weight update: latent stream")
    assert_close(eo3[0], want_e3, BF16_COS, BF16_REL, "adopted module after a weight update: context stream")
    with pytest.raises(NotImplementedError):
        attn(h, attention_mask=torch.ones(1, n_lat, device=dev()), image_rotary_emb=rot)


def test_four_modality_block_with_audio():
    """text | video | audio | action with four weight sets (and with audio on the generator's set when there are only
    three): the block against the fp32 oracle (which the CPU suite pins to the float64 brute force on this layout)."""
    for nb in (4, 3):
        cfg = DMConfig("av", 256, 2, 128, 512, 1, (2, 4, 8), n_text=40, n_action=24, n_audio=19, n_branches=nb)
        st = DMStack(cfg, device=dev())
        blk = make_block(cfg, 61 + nb)
        g = torch.Generator().manual_seed(61)
        x, xr = rand_bf16((cfg.n_tokens, 256), g)
        temb, tembr = rand_bf16((256,), g)
        segs = st.segments()
        audio_branch = 3 if nb == 4 else 1
        assert segs == [(0, 40, 0, False), (40, 64, 1, True), (104, 19, audio_branch, True), (123, 24, 2, True)]
        y = blk(x, temb, st.rotary(dev()), segs)
        mod = O.adaln_modulation(tembr.view(1, -1), blk.adaLN_modulation.weight.float().cpu(),
                                 blk.adaLN_modulation.bias.float().cpu())
        pos = O.joint_positions([("text", 40), ("video", cfg.grid), ("audio", 19), ("action", 24)])
        assert torch.equal(pos, rotary.build_positions(40, cfg.grid, 24, 19)[0])
        # audio positions continue after the grid's offset max(H, W) and action positions after the audio run
        assert int(pos[0, 104]) == 40 + 8 and int(pos[0, 123]) == 40 + 8 + 19
        cos, sin = O.mrope_cos_sin(pos, 128, cfg.mrope_sections)
        want = O.dm_block(xr, oracle_weights(blk, nb), mod, cos, sin, 2, segs)
        assert_close(y, want, BF16_COS, BF16_REL, f"four-modality block, {nb} weight sets")


def test_transformer_with_audio_stream_and_context_cache():
    """DMTransformer with sound and action streams: outputs per stream; under the hybrid mask the cached text K/V
    (context_cache) give the same prediction as the joint forward."""
    from cosmos_amd import DMTransformer
    cfg = DMConfig("snd", 256, 2, 128, 512, 2, (2, 3, 4), n_text=64, n_action=5, n_audio=9, n_branches=4, qk_norm=True,
                   hybrid_mask=True)
    m = DMTransformer(cfg, latent_channels=4, action_dim=6, audio_dim=10, device=dev())
    m.reset_parameters(5)
    g = torch.Generator(device=dev()).manual_seed(5)
    with torch.no_grad():
        m.audio_modality_embed.copy_(0.5 * torch.randn(256, generator=g, device=dev()))
        for blk in m.stack.blocks:
            blk.adaLN_modulation.bias.copy_(0.3 * torch.randn(blk.adaLN_modulation.bias.shape, generator=g, device=dev()))
    assert {"audio_proj_in.weight", "audio_proj_out.bias", "audio_modality_embed"} <= set(m.top_level_keys())
    lat = torch.randn((1, 4, 2, 6, 8), generator=g, device=dev())
    ctx = torch.randn((1, 64, 256), generator=g, device=dev()).to(torch.bfloat16)
    act = torch.randn((1, 5, 6), generator=g, device=dev())
    snd = torch.randn((1, 9, 10), generator=g, device=dev())
    t = torch.tensor([450.0], device=dev())
    out = m(lat, t, encoder_hidden_states=ctx, action_states=act, audio_states=snd, return_dict=True)
    assert out["sample"].shape == lat.shape and out["audio"].shape == (1, 9, 10) and out["action"].shape == (1, 5, 6)
    tup = m(lat, t, encoder_hidden_states=ctx, action_states=act, audio_states=snd)
    assert len(tup) == 3 and torch.equal(tup[1], out["audio"]) and torch.equal(tup[2], out["action"])
    with pytest.raises(ValueError):
        m(lat, t, encoder_hidden_states=ctx, action_states=act)
    cache = m.stack.precompute_context(ctx)
    out2 = m(lat, t, action_states=act, audio_states=snd, return_dict=True, context_cache=cache)
    for k in ("sample", "audio", "action"):
        assert_close(out2[k], out[k].float().cpu(), 0.9999, 1e-2, f"transformer with context cache: {k}")
    # oracle: audio rows of the stack
    f = lambda p: p.detach().float().cpu()
    tok = m.patchify(lat[0].to(torch.bfloat16)).float().cpu() @ f(m.proj_in.weight).t() + f(m.proj_in.bias)
    a_in = f(act[0].to(torch.bfloat16)) @ f(m.action_proj_in.weight).t() + f(m.action_proj_in.bias) + f(m.action_modality_embed)
    s_in = f(snd[0].to(torch.bfloat16)) @ f(m.audio_proj_in.weight).t() + f(m.audio_proj_in.bias) + f(m.audio_modality_embed)
    x = torch.cat([f(ctx[0]), tok, s_in, a_in])
    te = m.time_embedder
    c = O.time_mlp(O.timestep_embedding(t.cpu()), f(te.linear_1.weight), f(te.linear_1.bias), f(te.linear_2.weight), f(te.linear_2.bias))
    mods = [O.adaln_modulation(c, f(b.adaLN_modulation.weight), f(b.adaLN_modulation.bias)) for b in m.stack.blocks]
    pos = O.joint_positions([("text", 64), ("video", cfg.grid), ("audio", 9), ("action", 5)])
    cos, sin = O.mrope_cos_sin(pos, 128, cfg.mrope_sections)
    y = O.dm_stack(x, [oracle_weights(b, 4) for b in m.stack.blocks], mods, cos, sin, 2, m.stack.segments(), causal_prefix=64)
    y = O.rms_norm(y, f(m.norm_out), cfg.eps)
    n0 = 64 + cfg.n_video
    assert_close(out["audio"][0], y[n0:n0 + 9] @ f(m.audio_proj_out.weight).t() + f(m.audio_proj_out.bias), BF16_COS, BF16_REL, "audio head")
    assert_close(out["action"][0], y[n0 + 9:] @ f(m.action_proj_out.weight).t() + f(m.action_proj_out.bias), BF16_COS, BF16_REL, "action head (after audio)")


def test_stack_forward_recorded_as_a_graph():
    """A forward recorded into a HIP graph (launch-bound shapes): every replay - with the program's own eager work and
    synchronisations between them, on new inputs - gives the bits of the eager forward; a wrong shape is refused."""
    cfg = DMConfig("g", 256, 2, 128, 512, 3, (2, 4, 8), n_text=24, n_action=6, n_audio=5, n_branches=4, qk_norm=True)
    st = DMStack(cfg, device=dev())
    st.reset_parameters(9)
    g = torch.Generator(device=dev()).manual_seed(9)
    with torch.no_grad():
        for blk in st.blocks:
            blk.adaLN_modulation.bias.copy_(0.3 * torch.randn(blk.adaLN_modulation.bias.shape, generator=g, device=dev()))
    mk = lambda n: torch.randn((1, n, 256), generator=g, device=dev()).to(torch.bfloat16)
    def inputs():
        return dict(hidden_states=mk(cfg.n_video), timestep=torch.rand(1, generator=g, device=dev()) * 1000,
                    encoder_hidden_states=mk(24), action_states=mk(6), audio_states=mk(5))
    first = inputs()
    graphed = st.capture(**first)
    for i in range(4):
        inp = first if i == 0 else inputs()
        want = st(return_dict=True, **inp)
        want = {k: v.clone() for k, v in want.items()}
        torch.cuda.synchronize()
        # eager work of other shapes between the replays (its launches must not disturb the recording's buffers)
        other = DMConfig("o", 256, 2, 128, 512, 1, (1, 4, 8))
        ops.adaln_rmsnorm(mk(40)[0], torch.ones(256, dtype=torch.bfloat16, device=dev()))
        got = graphed(**inp)
        torch.cuda.synchronize()
        assert torch.equal(got["sample"], want["sample"]) and torch.equal(got["joint"], want["joint"]), f"replay {i}"
    with pytest.raises(ValueError):
        graphed(**{**first, "hidden_states": mk(cfg.n_video - 1)})
    with pytest.raises(ValueError):
        graphed(**{**first, "audio_states": None})
