"""Parity at DEPTH: whole stacks against the fp32 oracle, free-running (errors of earlier blocks feed later ones)
and teacher-forced (each checked block starts from the GPU stack's own input to it).

 * reduced width (d = 512, 1,024 - 1,064 tokens), full depth: 28 bf16 blocks, 28 e4m3 blocks, 8 three-branch MoT
   blocks, with order-one modulation (the blocks are far from the identity), against the CPU oracle;
 * full size (benchmark configurations 2, 3, 4): teacher-forced sampled token rows of layers 1, 14 and 28 (1, 4, 8
   for the 8-block MoT stack) against the CPU oracle, and the free-running output of the whole stack against the same
   oracle statements executed in fp32 by stock PyTorch on the GPU (the CPU would need hours), after that execution has
   been checked against the CPU one on sampled rows.
Tolerances are the benchmark's: cos >= 0.999, max|a-b|/max|b| <= 2e-2 (bf16) / 5e-2 (e4m3 GEMMs)."""
import dataclasses

import pytest
import torch

import oracle as O
from cosmos_amd import CONFIGS, DMStack, Workspace
from cosmos_amd.config import DMConfig
from gpu_util import BF16_COS, BF16_REL, FP8_COS, FP8_REL, assert_close, dev, oracle_weights, rand_bf16

pytestmark = pytest.mark.gpu


def f32(p, device="cpu"):
    return p.detach().float().to(device)


def oracle_inputs(st, t, device="cpu"):
    """Per-layer modulation (through the oracle's own embedding / MLP) and rotary tables of a stack."""
    cfg, te = st.cfg, st.time_embedder
    c = O.time_mlp(O.timestep_embedding(t.cpu()), f32(te.linear_1.weight), f32(te.linear_1.bias), f32(te.linear_2.weight),
                   f32(te.linear_2.bias))
    mods = [tuple(m.to(device) for m in O.adaln_modulation(c, f32(b.adaLN_modulation.weight), f32(b.adaLN_modulation.bias)))
            for b in st.blocks]
    pos = O.joint_positions(([("text", cfg.n_text)] if cfg.n_text else []) + [("video", cfg.grid)] +
                            ([("action", cfg.n_action)] if cfg.n_action else []))
    cos, sin = O.mrope_cos_sin(pos, cfg.head_dim, cfg.mrope_sections, cfg.rope_base, cfg.rope_layout)
    return mods, cos.to(device), sin.to(device)


def strong_modulation_(st, seed, std, gate_bias=0.3, mod_bias=0.3):
    """Weights of order 1/sqrt(d) and order-one adaLN biases: every block moves the residual stream visibly."""
    g = torch.Generator(device=dev()).manual_seed(seed)
    with torch.no_grad():
        for b in st.blocks:
            b.reset_parameters(g, std=std)
            for p in list(b.norm1_weight) + list(b.norm2_weight):
                p.copy_(1 + 0.1 * torch.randn(p.shape, generator=g, device=dev()))
            bias = mod_bias * torch.randn(6, st.cfg.d_model, generator=g, device=dev())
            bias[2] *= gate_bias / mod_bias
            bias[5] *= gate_bias / mod_bias
            b.adaLN_modulation.bias.copy_(bias.reshape(-1))


@pytest.mark.parametrize("kind", ["bf16", "bf16-stream", "fp8", "mot"])
def test_full_depth_stack_at_reduced_width(kind):
    """"bf16-stream" keeps the residual stream in bf16 between blocks instead of fp32: 56 roundings of the stream
    alone cost percent-level accuracy at this depth, which is why a stack keeps it in fp32 (measured here against a
    looser bound, for the record)."""
    if kind == "mot":
        cfg = DMConfig("mot8", 512, 4, 128, 2048, 8, (4, 12, 20), n_text=64, n_action=40, n_branches=3)
    else:
        cfg = DMConfig("d28", 512, 4, 128, 2048, 28, (4, 12, 20), n_text=64, fp8=(kind == "fp8"),
                       residual_fp32=(kind != "bf16-stream"))
    st = DMStack(cfg, device=dev())
    st.reset_parameters(77)
    strong_modulation_(st, 78, std=0.05, gate_bias=0.3)
    gc = torch.Generator().manual_seed(79)
    xv, xvr = rand_bf16((1, cfg.n_video, cfg.d_model), gc)
    xt, xtr = rand_bf16((1, cfg.n_text, cfg.d_model), gc)
    kw, parts = dict(encoder_hidden_states=xt), [xtr[0], xvr[0]]
    if cfg.n_action:
        xa, xar = rand_bf16((1, cfg.n_action, cfg.d_model), gc)
        kw["action_states"] = xa
        parts.append(xar[0])
    t = torch.tensor([612.0])
    out = st(xv, t.to(dev()), return_dict=True, **kw)
    mods, cos, sin = oracle_inputs(st, t)
    x0 = torch.cat(parts)
    want = O.dm_stack(x0, [oracle_weights(b, cfg.n_branches) for b in st.blocks], mods, cos, sin, cfg.n_heads, st.segments())
    assert float((want - x0).abs().max()) > 2.0 and O.cos_sim(want, x0) < 0.9      # far from the identity
    assert out["joint"].dtype == (torch.float32 if cfg.residual_fp32 else torch.bfloat16) and out["sample"].dtype == torch.bfloat16
    v0, v1 = cfg.n_text, cfg.n_text + cfg.n_video
    if cfg.fp8:
        # e4m3 operands carry percent-level noise per product and the un-gated text rows take every block's update at
        # full size: over 28 blocks the recipe itself is far outside 5e-2 of the unquantised oracle, whatever the
        # implementation.  The yardstick is the oracle that quantises at the same places: the kernels must be about as
        # close to the unquantised oracle as it is, and closer to it than it is to the unquantised one.
        want8 = O.dm_stack(x0, [oracle_weights(b, cfg.n_branches) for b in st.blocks], mods, cos, sin, cfg.n_heads,
                           st.segments(), fp8=True)
        got = out["joint"].float().cpu()
        noise_c, noise_r = 1.0 - O.cos_sim(want8, want), O.max_rel_err(want8, want)
        assert_close(want8, want, 0.0, 10.0, "28-block e4m3 recipe at d=512: QUANTISING ORACLE vs fp32 oracle (joint)")
        assert_close(got, want8, 0.0, 10.0, "28-block fp8 stack at d=512 vs quantising oracle (joint)")
        assert_close(got, want, 0.0, 10.0, "28-block fp8 stack at d=512, free-running (joint)")
        assert 1.0 - O.cos_sim(got, want) < 1.5 * noise_c and O.max_rel_err(got, want) < 1.5 * noise_r
        assert 1.0 - O.cos_sim(got, want8) < 1.5 * noise_c and O.max_rel_err(got, want8) < 1.5 * noise_r
        return
    tol = (BF16_COS, BF16_REL if cfg.residual_fp32 else 5e-2)
    assert_close(out["joint"], want, *tol, f"{cfg.n_blocks}-block {kind} stack at d=512, free-running (joint)")
    assert_close(out["sample"][0], want[v0:v1], *tol, f"{cfg.n_blocks}-block {kind} stack at d=512, free-running (video rows)")


def _full_size_stack(name):
    cfg = CONFIGS[name]
    st = DMStack(cfg, device=dev())
    st.reset_parameters()
    g = torch.Generator(device=dev()).manual_seed(cfg.seed + 100)
    mk = lambda n: torch.randn((n, cfg.d_model), generator=g, device=dev()).to(torch.bfloat16)
    parts = ([mk(cfg.n_text)] if cfg.n_text else []) + [mk(cfg.n_video)] + ([mk(cfg.n_action)] if cfg.n_action else [])
    x0 = torch.cat(parts).contiguous()
    t = torch.tensor([(torch.rand(1, generator=torch.Generator().manual_seed(cfg.seed)) * 1000.0).item()])
    return cfg, st, x0, t


@pytest.mark.timeout(900)
@pytest.mark.parametrize("name", ["C2", "C3", "C4"])
def test_full_size_stack_at_depth(name):
    """The benchmark's own inputs (weights N(0, 0.02), modulation from a random timestep through the embedder) at full
    size and full depth."""
    cfg, st, x0, t = _full_size_stack(name)
    L = cfg.n_blocks
    layers = sorted({0, L // 2 - 1, L - 1})
    segs, rot = st.segments(), st.rotary(dev())
    temb = st.time_embedder(t.to(dev()))
    ws = Workspace(cfg.n_tokens, cfg.d_model, cfg.hidden, cfg.n_heads, cfg.head_dim, dev(), cfg.kv_heads)
    x, taken = st._stream(x0), {}
    for l, blk in enumerate(st.blocks):
        if l in layers:
            taken[l] = x.clone()
        blk(x, temb, rot, segs, inplace=True, workspace=ws)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(x.float()).all())
    tol = (FP8_COS, FP8_REL) if cfg.fp8 else (BF16_COS, BF16_REL)

    # ---- free-running: the oracle's statements in fp32 on the GPU, block by block (one layer's fp32 weights at a time)
    mods_g, cos_g, sin_g = oracle_inputs(st, t, dev())
    n = cfg.n_tokens
    bounds = sorted({0, 1, n - 1} | {s0 for (s0, _, _, _) in segs} | {s0 + ln - 1 for (s0, ln, _, _) in segs})
    rows = torch.tensor(bounds + torch.randint(0, n, (16,), generator=torch.Generator().manual_seed(5)).tolist())
    xo = x0.float()
    for l, blk in enumerate(st.blocks):
        wg = oracle_weights(blk, cfg.n_branches, dev())
        if l == 0:
            # the GPU execution of the oracle against its CPU execution, same input, sampled rows
            on_gpu = O.dm_block(xo, wg, mods_g[0], cos_g, sin_g, cfg.n_heads, segs, attn_rows=rows)
            mods_c, cos_c, sin_c = oracle_inputs(st, t)
            on_cpu = O.dm_block(xo.cpu(), oracle_weights(blk, cfg.n_branches), mods_c[0], cos_c, sin_c, cfg.n_heads, segs,
                                attn_rows=rows)
            assert_close(on_gpu, on_cpu, 0.999999, 2e-4, f"{name}: oracle on the GPU vs oracle on the CPU (layer 1 rows)")
        xo = O.dm_block(xo, wg, mods_g[l], cos_g, sin_g, cfg.n_heads, segs)
        del wg
    moved = float((xo - x0.float()).abs().max())
    assert moved > 1.0, moved
    v0, v1 = cfg.n_text, cfg.n_text + cfg.n_video
    if cfg.fp8:
        # e4m3 operands carry percent-level noise per product.  The un-gated text rows take every block's update at
        # full size, so over 28 blocks that noise is no longer small there, whatever the implementation: the oracle
        # that quantises at the same places (same statements, fp8=True) is the yardstick for the joint sequence, and
        # the kernels must be closer to it than it is to the unquantised one
        xq = x0.float()
        for l, blk in enumerate(st.blocks):
            xq = O.dm_block(xq, oracle_weights(blk, cfg.n_branches, dev()), mods_g[l], cos_g, sin_g, cfg.n_heads, segs, fp8=True)
        noise_c, noise_r = 1.0 - O.cos_sim(xq, xo), O.max_rel_err(xq, xo)
        assert_close(xq, xo, 0.0, 10.0, f"{name}: QUANTISING ORACLE vs fp32 oracle, {L} blocks (joint) - the recipe's own noise")
        assert_close(xq[v0:v1], xo[v0:v1], 0.0, 10.0, f"{name}: QUANTISING ORACLE vs fp32 oracle, {L} blocks (video rows)")
        assert_close(x, xq, 0.0, 10.0, f"{name}: {L}-block stack at full size vs quantising oracle (joint)")
        assert 1.0 - O.cos_sim(x, xq) < noise_c and O.max_rel_err(x, xq) < 1.25 * noise_r
        assert_close(x, xo, 0.0, 10.0, f"{name}: {L}-block stack at full size, free-running (joint)")
        assert 1.0 - O.cos_sim(x, xo) < 1.5 * noise_c and O.max_rel_err(x, xo) < 1.5 * noise_r
        # the video rows (the transformer's output): the recipe's own noise there is about 1e-1 at this depth, so the
        # 5e-2 of a single block is out of reach for ANY implementation of the recipe; held to the recipe's noise
        noise_vc, noise_vr = 1.0 - O.cos_sim(xq[v0:v1], xo[v0:v1]), O.max_rel_err(xq[v0:v1], xo[v0:v1])
        assert_close(x[v0:v1], xo[v0:v1], 0.0, 10.0, f"{name}: {L}-block stack at full size, free-running (video rows)")
        assert 1.0 - O.cos_sim(x[v0:v1], xo[v0:v1]) < 1.25 * noise_vc and O.max_rel_err(x[v0:v1], xo[v0:v1]) < 1.25 * noise_vr
        del xq
    else:
        assert_close(x, xo, *tol, f"{name}: {L}-block stack at full size, free-running (joint)")
        assert_close(x[v0:v1], xo[v0:v1], *tol, f"{name}: {L}-block stack at full size, free-running (video rows)")
    del xo

    # ---- teacher-forced: layer l alone from the GPU stack's own input to it, sampled rows, CPU oracle
    mods_c, cos_c, sin_c = oracle_inputs(st, t)
    for l in layers:
        blk = st.blocks[l]
        y = blk(taken[l], temb, rot, segs, workspace=ws)
        want = O.dm_block(taken[l].float().cpu(), oracle_weights(blk, cfg.n_branches), mods_c[l], cos_c, sin_c, cfg.n_heads, segs,
                          attn_rows=rows)
        got = y[rows.to(dev())]
        if not cfg.fp8:
            assert_close(got, want, *tol, f"{name}: layer {l + 1} of {L} at full size, teacher-forced rows")
            continue
        # e4m3: the adaLN-gated generator rows meet 5e-2 against the UNQUANTISED oracle; the un-gated text rows take the
        # block's update at full size and are held to the noise of the oracle that quantises at the same places
        gated = torch.zeros(len(rows), dtype=torch.bool)
        for (s0, ln, _, modulated) in segs:
            if modulated:
                gated |= (rows >= s0) & (rows < s0 + ln)
        assert_close(got[gated.to(dev())], want[gated], *tol, f"{name}: layer {l + 1} of {L} at full size, teacher-forced gated rows")
        want8 = O.dm_block(taken[l].float().cpu(), oracle_weights(blk, cfg.n_branches), mods_c[l], cos_c, sin_c, cfg.n_heads, segs,
                           attn_rows=rows, fp8=True)
        ung = ~gated
        noise = O.max_rel_err(want8[ung], want[ung])
        assert_close(got[ung.to(dev())], want[ung], 0.0, 10.0, f"{name}: layer {l + 1} of {L} at full size, teacher-forced un-gated rows")
        assert O.max_rel_err(got[ung.to(dev())], want[ung]) < 1.25 * noise and O.max_rel_err(got[ung.to(dev())], want8[ung]) < noise
