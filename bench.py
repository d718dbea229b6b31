#!/usr/bin/env python3
"""Benchmark of the DM-block hot path on one MI355X.

A "step" is one denoising step = one forward of the whole DiT stack over one synthetic joint sequence.
Default workload: the full video DiT stack (28 blocks, d=4096, 32x128 heads, SwiGLU 16384, 512 text +
16x44x80 video tokens = 56,832 tokens, bf16, random-init weights N(0, 0.02)).
Prints ONE JSON line: ms per denoising step, the MFMA roofline of the dominant kernel (attention; duration
from HIP events around every attention launch inside the timed region), a CPU baseline (the fp32 oracle on
this host's cores, bounded sample, extrapolated) with the parity of the HIP block against that very oracle run,
and - for the default workload - short legs of the other workloads under ``extra.workloads``: C1 (mRoPE +
attention alone), C3 (Mixture-of-Transformers stack), C4 (e4m3 GEMMs), the C2 shapes with QK-RMSNorm and grouped
K / V heads, and one production step (conditional + unconditional forward on a cached text context + the fused
UniPC update).
"""
import argparse
import dataclasses
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
PEAK_FP8_TFLOPS = 5000.0
PEAK_HBM_GBS = 8000.0
# HBM-side bytes per attention launch (L2 fetches + writes) for the 56,832-token, 32x128-head shape, from two
# rocprofv3 --pmc passes (FETCH_SIZE, WRITE_SIZE), each scaled by the same counter's reading for a plain streaming
# kernel of known size (FETCH_SIZE unit = 2 KiB, WRITE_SIZE unit = 1 KiB on this chip).  Counters cannot be read
# from inside this process; the figure is only reported while the kernel's source is the one it was measured on.
ATTN_TRAFFIC = {"shape": (56832, 32, 128), "bytes": 8.616e9 + 0.466e9, "attn_source_sha256_16": "e241ef1061e23461"}

T_START = time.perf_counter()


def attn_source_hash() -> str:
    with open(os.path.join(ROOT, "cosmos_amd", "csrc", "attn.hip"), "rb") as fh:
        return hashlib.sha256(fh.read()).hexdigest()[:16]


def attention_traffic(cfg, attn_variant: int):
    """(bytes or None, note): the stored counter figure, only for the shape and the kernel source it was taken with."""
    if (attn_variant != 0 or (cfg.n_tokens, cfg.n_heads, cfg.head_dim) != ATTN_TRAFFIC["shape"] or cfg.kv_heads != cfg.n_heads
            or cfg.qk_norm or cfg.hybrid_mask):
        return None, "no stored counter pass for this shape / variant"
    if attn_source_hash() != ATTN_TRAFFIC["attn_source_sha256_16"]:
        return None, "attn.hip changed since the stored rocprofv3 --pmc passes: re-measure (profiles/c2_one_block_pmc_counters.txt)"
    return ATTN_TRAFFIC["bytes"], ("stored figure of two rocprofv3 --pmc passes (FETCH_SIZE, WRITE_SIZE) over this kernel at this "
                                   "shape, profiles/c2_one_block_pmc_counters.txt; counters cannot be read in-process")


def cpu_baseline(cfg, sample_tokens: int, dev):
    """fp32 oracle of ONE block on `sample_tokens` tokens of the same width (0 = all tokens: minutes of CPU time at the
    benchmark sizes), timed on the host cores; the GEMM part scales linearly and the attention part quadratically with
    the token count.  The HIP block then runs on the same inputs and weights (all bf16-representable), and its output
    is compared with the oracle's: the parity figures of the line."""
    import torch
    import oracle as O
    from cosmos_amd import DMBlock
    d, h, H = cfg.d_model, cfg.hidden, cfg.n_heads
    g = torch.Generator().manual_seed(0)
    n = min(sample_tokens, cfg.n_tokens) if sample_tokens > 0 else cfg.n_tokens
    rb = lambda t: t.to(torch.bfloat16).float()
    x = rb(torch.randn(n, d, generator=g))
    w = dict(norm1_w=torch.ones(d), norm2_w=torch.ones(d))
    for name, shape in (("wq", (d, d)), ("wk", (d, d)), ("wv", (d, d)), ("wo", (d, d)), ("wg", (h, d)), ("wu", (h, d)),
                        ("wd", (d, h))):
        w[name] = rb(torch.randn(shape, generator=g) * 0.02)
    mod = [torch.randn(d, generator=g) * 0.1 for _ in range(6)]
    pos = O.text_positions(0, n)
    cos, sin = O.mrope_cos_sin(pos, cfg.head_dim, cfg.mrope_sections)
    q = torch.randn(n, H, cfg.head_dim, generator=g)
    out = {}

    def best_of_two(fn, key=None):
        best = float("inf")
        for _ in range(2):          # the first call of a size pays allocator growth / page faults
            t0 = time.perf_counter()
            r = fn()
            best = min(best, time.perf_counter() - t0)
        if key:
            out[key] = r
        return best
    t_attn = best_of_two(lambda: O.attention(q, q, q))
    t_block = best_of_two(lambda: O.dm_block(x, [w], mod, cos, sin, H), "y")
    t_lin = max(t_block - t_attn, 0.0)
    ratio = cfg.n_tokens / n
    per_block = t_lin * ratio + t_attn * ratio * ratio
    base = {"value": round(per_block * max(cfg.n_blocks, 1) * 1e3, 1),
            "unit": "ms per denoising step (extrapolated)" if (ratio > 1 or cfg.n_blocks > 1) else "ms per denoising step",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"fp32 oracle, one block on {n} of {cfg.n_tokens} tokens at full width: {t_block:.2f} s "
                      f"(attention {t_attn:.2f} s); linear part x{ratio:.2f}, attention x{ratio * ratio:.1f}, "
                      f"x{max(cfg.n_blocks, 1)} blocks",
            "ms_per_block": round(per_block * 1e3, 1), "extrapolated": bool(ratio > 1 or cfg.n_blocks > 1)}
    # the HIP block on the same sample
    blk = DMBlock(d, H, cfg.head_dim, h, 1, cfg.eps, cfg.fp8, device=dev)
    with torch.no_grad():
        blk.attn.qkv_weight[0].copy_(torch.cat([w["wq"], w["wk"], w["wv"]]).to(torch.bfloat16))
        blk.attn.out_weight[0].copy_(w["wo"].to(torch.bfloat16))
        blk.norm1_weight[0].fill_(1.0); blk.norm2_weight[0].fill_(1.0)
        blk.gate_weight[0].copy_(w["wg"].to(torch.bfloat16)); blk.up_weight[0].copy_(w["wu"].to(torch.bfloat16))
        blk.down_weight[0].copy_(w["wd"].to(torch.bfloat16))
        if cfg.fp8:
            blk.quantize_()
        y = blk(x.to(dev), None, (cos.to(dev).contiguous(), sin.to(dev).contiguous()), modulation=[m.to(dev) for m in mod])
    torch.cuda.synchronize()
    got = y.float().cpu()
    tol = 5e-2 if cfg.fp8 else 2e-2
    parity = {"cos_sim": round(O.cos_sim(got, out["y"]), 6), "max_rel_err": float(f"{O.max_rel_err(got, out['y']):.3e}"),
              "tolerance": {"cos_sim_min": 0.999, "max_rel_err_max": tol},
              "what": f"HIP block vs the fp32 oracle run timed above: one block, {n} tokens at full width, same inputs and weights"}
    del blk, y
    return base, parity


def make_inputs(cfg, dev):
    import torch
    # the weights were drawn from a generator seeded with cfg.seed: the inputs take another stream (the same seed would
    # reproduce the weights' random numbers, i.e. token rows parallel to weight rows)
    g = torch.Generator(device=dev).manual_seed(cfg.seed + 1000)
    xv = torch.randn((1, cfg.n_video, cfg.d_model), generator=g, device=dev).to(torch.bfloat16)
    xt = torch.randn((1, cfg.n_text, cfg.d_model), generator=g, device=dev).to(torch.bfloat16) if cfg.n_text else None
    xa = torch.randn((1, cfg.n_action, cfg.d_model), generator=g, device=dev).to(torch.bfloat16) if cfg.n_action else None
    t = torch.rand(1, generator=g, device=dev) * 1000.0
    return xv, xt, xa, t


def time_steps(step, steps: int, warmup: int):
    """Time `steps` calls of `step` after `warmup`: wall clock bracketed by device synchronisation, HIP events around
    every kernel launcher.  -> (ms per step, attention events, per-category events, last output)"""
    import torch
    from cosmos_amd import ops
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    ops.time_attention(True)
    ops.time_ops(True)
    t0 = time.perf_counter()
    for _ in range(steps):
        out = step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall * 1e3 / steps, ops.time_attention(False), ops.time_ops(False), out


def stack_metrics(cfg, ms_per_step, attn_events, op_events, steps, attn_variant=0, forwards_per_step=1, n_tokens=None):
    """roofline / kernels / extra objects of a stack run from its events."""
    n_tok = cfg.n_tokens if n_tokens is None else n_tokens
    attn_ms = [a.elapsed_time(b) for a, b in attn_events]
    launches = len(attn_ms)
    attn_avg = sum(attn_ms) / len(attn_ms) if attn_ms else float("nan")
    attn_flops = cfg.attn_flops_per_block()
    attn_tf = attn_flops / (attn_avg * 1e-3) / 1e12
    cat_ms = {}
    for cat, a, b in op_events:
        cat_ms[cat] = cat_ms.get(cat, 0.0) + a.elapsed_time(b)
    nb = max(cfg.n_blocks, 1) * forwards_per_step
    per_block = {k: v / (steps * nb) for k, v in cat_ms.items()}
    gemm_peak = PEAK_FP8_TFLOPS if cfg.fp8 else PEAK_BF16_TFLOPS
    kernels = {}
    if per_block.get("gemm"):
        tf = cfg.gemm_flops_per_block() / (per_block["gemm"] * 1e-3) / 1e12
        kernels["gemm"] = {"ms_per_block": round(per_block["gemm"], 3), "tflops": round(tf, 1), "frac_of_mfma_peak": round(tf / gemm_peak, 4)}
    nd = n_tok * cfg.d_model
    xb = 4 if cfg.residual_fp32 else 2                         # bytes per element of the residual stream
    hbm_bytes = {"norm": 2 * (xb + (1 if cfg.fp8 else 2)) * nd,  # two norms per block: read the stream, write bf16 (or e4m3)
                 "pack_kv": 8 * nd + 8 * n_tok * (cfg.head_dim // 2),   # K, V in; two tile images out; cos/sin
                 "quant": 2 * 3 * nd + 3 * n_tok * cfg.hidden,           # attention output and SwiGLU hidden -> e4m3
                 "rope": 8 * nd}
    for cat, nbytes in hbm_bytes.items():
        if per_block.get(cat):
            gbs = nbytes / (per_block[cat] * 1e-3) / 1e9
            kernels[cat] = {"ms_per_block": round(per_block[cat], 3), "GBps": round(gbs, 0), "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 3)}
    if per_block.get("step"):
        kernels["step"] = {"ms_per_launch": round(cat_ms["step"] / steps, 4)}
    traffic, note = attention_traffic(cfg, attn_variant)
    roofline = {"bound": "mfma", "kernel": "attn_fwd_pipe_kernel", "achieved": round(attn_tf, 1), "peak": PEAK_BF16_TFLOPS,
                "unit": "TFLOP/s", "frac": round(attn_tf / PEAK_BF16_TFLOPS, 4), "traffic": traffic, "traffic_source": note,
                "flops_per_launch": attn_flops, "avg_launch_ms": round(attn_avg, 3), "launches": launches}
    ms_block = ms_per_step / nb
    non_attn = ms_block - attn_avg
    gemm_lb = cfg.gemm_flops_per_block() / (non_attn * 1e-3) / 1e12
    extra = {"ms_per_block": round(ms_block, 3), "non_attention_ms_per_block": round(non_attn, 3),
             "gemm_tflops_lower_bound": round(gemm_lb, 1), "gemm_frac_of_peak_lower_bound": round(gemm_lb / gemm_peak, 4),
             "total_tflops": round((attn_flops + cfg.gemm_flops_per_block()) * nb / (ms_per_step * 1e-3) / 1e12, 1)}
    return roofline, kernels, extra


def workload_name(cfg):
    kv = f", {cfg.kv_heads} K/V heads" if cfg.kv_heads != cfg.n_heads else ""
    qn = ", QK-RMSNorm" if cfg.qk_norm else ""
    return (f"{cfg.name}: {cfg.n_blocks} DM blocks, d={cfg.d_model}, {cfg.n_heads}x{cfg.head_dim} heads{kv}{qn}, SwiGLU {cfg.hidden}, "
            f"{cfg.n_text} text + {cfg.grid[0]}x{cfg.grid[1]}x{cfg.grid[2]} video + {cfg.n_action} action = {cfg.n_tokens} tokens, batch 1")


def report_line(cfg, ms_per_step, roofline, kernels, cpu=None, parity=None, rope_gbps=None):
    """The per-configuration reporting object (field names of the baseline plan)."""
    nb = max(cfg.n_blocks, 1)
    g = kernels.get("gemm", {})
    return {"config": cfg.name, "n_tokens": cfg.n_tokens, "ms_per_block_gpu": round(ms_per_step / nb, 3),
            "ms_per_step_gpu": round(ms_per_step, 2), "gemm_tflops": g.get("tflops"),
            "gemm_pct_peak": round(100 * g["frac_of_mfma_peak"], 2) if g else None,
            "attn_tflops": roofline["achieved"], "attn_pct_peak": round(100 * roofline["frac"], 2),
            "norm_gbps": kernels.get("norm", {}).get("GBps"), "rope_gbps": rope_gbps,
            "cos_sim": parity["cos_sim"] if parity else None, "max_rel_err": parity["max_rel_err"] if parity else None,
            "cpu_ms_per_block": cpu["ms_per_block"] if cpu else None, "cpu_ms_per_step": cpu["value"] if cpu else None,
            "cpu_extrapolated": cpu["extrapolated"] if cpu else None, "cpu_cores": cpu["cores"] if cpu else None,
            "peak_bf16": PEAK_BF16_TFLOPS, "peak_fp8": PEAK_FP8_TFLOPS, "peak_hbm": PEAK_HBM_GBS}


def bench_attention_only(cfg, steps, warmup, dev, attn_variant=0):
    """Workload C1: 3-D mRoPE + full attention alone on the 16x44x80 grid (56,320 tokens, 32 x 128 heads)."""
    import torch
    from cosmos_amd import ops, rotary
    n, H, hd = cfg.n_tokens, cfg.n_heads, cfg.head_dim
    d = H * hd
    g = torch.Generator(device=dev).manual_seed(cfg.seed)
    qkv = (torch.randn((n, 3 * d), generator=g, device=dev) / hd ** 0.5).to(torch.bfloat16)
    pos, _ = rotary.build_positions(0, cfg.grid, 0)
    cos, sin = rotary.rotary_tables(pos, hd, cfg.mrope_sections, cfg.rope_base, cfg.rope_layout, dev)
    out = torch.empty((n, d), dtype=torch.bfloat16, device=dev)
    # K / V tile images plus the scratch of the split of the last round of workgroups (220 query blocks x 4 heads per XCD
    # = 27.5 rounds of 32: the last 16 blocks of every XCD run as two key ranges each)
    ws = torch.empty(ops.attn_workspace_total_bytes(n, H, H, hd), dtype=torch.uint8, device=dev)
    step = lambda: ops.attention(qkv[:, :d], qkv[:, d:2 * d], qkv[:, 2 * d:], H, hd, out=out, workspace=ws, cos=cos, sin=sin)
    ms, ev, _, _ = time_steps(step, steps, warmup)
    assert bool(torch.isfinite(out.float()).all()), "non-finite output"
    k_ms = sum(a.elapsed_time(b) for a, b in ev) / len(ev)
    flops = 4.0 * float(n) ** 2 * d
    tf = flops / (k_ms * 1e-3) / 1e12
    # the streaming rotation kernel on the same Q / K (the stand-alone form of what the attention kernels do in registers)
    q2, k2 = qkv[:, :d].clone(), qkv[:, d:2 * d].clone()
    ops.mrope_qk_(q2, k2, cos, sin, H, hd)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        ops.mrope_qk_(q2, k2, cos, sin, H, hd)
    e1.record()
    torch.cuda.synchronize()
    rope_gbps = 8.0 * n * d / (e0.elapsed_time(e1) / 5 * 1e-3) / 1e9
    return {
        "metric": "ms per mRoPE + attention pass on 1 GPU", "value": round(ms, 3), "unit": "ms", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 3), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"C1: mRoPE + full attention, {H}x{hd} heads, grid {cfg.grid[0]}x{cfg.grid[1]}x{cfg.grid[2]} = {n} tokens",
                   "n_tokens": n, "attn_variant": attn_variant},
        "roofline": {"bound": "mfma", "kernel": "attn_fwd_pipe_kernel", "achieved": round(tf, 1), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tf / PEAK_BF16_TFLOPS, 4), "traffic": None,
                     "flops_per_launch": flops, "avg_launch_ms": round(k_ms, 3), "launches": len(ev)},
        "kernels": {"rope_streaming": {"GBps": round(rope_gbps, 0), "frac_of_hbm_peak": round(rope_gbps / PEAK_HBM_GBS, 3)}},
        "extra": {"pack_kv_and_launch_overhead_ms": round(ms - k_ms, 3), "device": torch.cuda.get_device_name(0)}}


def run_stack_workload(cfg, args, dev, steps, warmup, keep=False):
    """Build the stack of `cfg`, time `steps` forwards -> (result dict, transformer or None)."""
    import torch
    from cosmos_amd import DMAttnProcessor, DMTransformer
    tr = DMTransformer(cfg, action_dim=16 if cfg.n_action else 0, device=dev)
    tr.reset_parameters()
    stack = tr.stack
    if args.rope != "in_attention" or args.no_fused_pack:
        for blk in stack.blocks:
            blk.attn.set_processor(DMAttnProcessor(rope=args.rope, fuse_kv_pack=not args.no_fused_pack))
    xv, xt, xa, t = make_inputs(cfg, dev)
    if args.graph:
        graphed = stack.capture(xv, t, encoder_hidden_states=xt, action_states=xa)
        step = lambda: graphed(xv, t, encoder_hidden_states=xt, action_states=xa)["sample"]
    else:
        step = lambda: stack(xv, t, encoder_hidden_states=xt, action_states=xa)[0]
    ms, ev, opev, out = time_steps(step, steps, warmup)
    assert bool(torch.isfinite(out.float()).all()), "non-finite output"
    if args.pmc_copy_mib:
        src = torch.zeros(args.pmc_copy_mib << 18, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        torch.bitwise_not(src, out=dst)
        torch.cuda.synchronize()
        del src, dst
    roofline, kernels, extra = stack_metrics(cfg, ms, ev, opev, steps, args.attn_variant)
    extra["device"] = torch.cuda.get_device_name(0)
    res = {
        "metric": "ms per denoising step (DiT stack) on 1 GPU",
        "value": round(ms, 2), "unit": "ms", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms, 2), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8-e4m3 GEMMs, bf16 attention" if cfg.fp8 else "bf16", "data": "synthetic",
        "config": {"workload": workload_name(cfg), "n_tokens": cfg.n_tokens, "n_blocks": cfg.n_blocks,
                   "attn_variant": args.attn_variant, "gemm_variant": args.gemm_variant, "rope": args.rope,
                   "kv_pack": "separate kernel" if args.no_fused_pack or args.rope != "in_attention" else "qkv gemm epilogue",
                   "qk_norm": cfg.qk_norm, "kv_heads": cfg.kv_heads, "residual_stream": args.residual, "hip_graph": bool(args.graph)},
        "roofline": roofline, "kernels": kernels, "extra": extra}
    if not keep:
        del tr, stack
        tr = None
    return res, tr


def production_leg(tr, cfg, dev, steps=2, warmup=1):
    """One production denoising step on the C2 stack (hybrid mask): the text context's K / V are packed once per prompt,
    a step = conditional + unconditional forward of the generator tokens against the cached context (latents in,
    velocity out, through the patch projections) + ONE launch of the fused guidance-combine + UniPC update."""
    import torch
    from cosmos_amd import UniPCStepper
    hcfg = dataclasses.replace(cfg, hybrid_mask=True)
    tr.cfg = hcfg
    tr.stack.cfg = hcfg
    g = torch.Generator(device=dev).manual_seed(cfg.seed + 2000)
    ctx_c = torch.randn((1, cfg.n_text, cfg.d_model), generator=g, device=dev).to(torch.bfloat16)
    ctx_u = torch.randn((1, cfg.n_text, cfg.d_model), generator=g, device=dev).to(torch.bfloat16)
    T, H, W = cfg.grid
    lat = torch.randn((1, tr.latent_channels, T * tr.patch[0], H * tr.patch[1], W * tr.patch[2]), generator=g, device=dev)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    cache_c = tr.stack.precompute_context(ctx_c)
    cache_u = tr.stack.precompute_context(ctx_u)
    torch.cuda.synchronize()
    ctx_ms = (time.perf_counter() - t0) * 1e3 / 2
    num_steps = 35
    stepper = UniPCStepper.from_flow_shift(num_steps, 10.0, guidance_scale=6.0)

    def step():
        ts = torch.full((1,), stepper.timesteps[stepper.index], device=dev)
        v_c = tr(lat, ts, context_cache=cache_c)[0]
        v_u = tr(lat, ts, context_cache=cache_u)[0]
        stepper.step(v_c, v_u, lat)
        return lat
    n_gen = cfg.n_tokens - cfg.n_text
    ms, ev, opev, out = time_steps(step, steps, warmup)
    assert bool(torch.isfinite(out).all()), "non-finite latents"
    gcfg = dataclasses.replace(cfg, n_text=0)
    roofline, kernels, extra = stack_metrics(gcfg, ms, ev, opev, steps, forwards_per_step=2, n_tokens=n_gen)
    # attention flops of a generator-only forward against n_text + n_gen keys
    flops = 4.0 * n_gen * cfg.n_tokens * cfg.d_model
    roofline["flops_per_launch"] = flops
    roofline["achieved"] = round(flops / (roofline["avg_launch_ms"] * 1e-3) / 1e12, 1)
    roofline["frac"] = round(roofline["achieved"] / PEAK_BF16_TFLOPS, 4)
    roofline["traffic"], roofline["traffic_source"] = None, "no counter pass for this shape"
    n_lat = lat.numel()
    step_ms = kernels.get("step", {}).get("ms_per_launch")
    if step_ms:
        kernels["step"]["note"] = f"fused guidance combine + UniPC update over {n_lat} latent values, one launch"
        # the same kernel on tensors large enough to show its rate: a full UniPC step reads the latents, two predictions
        # and three kept tensors (4 + 2 + 2 + 12 bytes per value) and writes three (12 bytes)
        from cosmos_amd import ops
        m = 1 << 26
        xs = torch.randn(m, device=dev)
        vc, vu = xs.to(torch.bfloat16), (0.5 * xs).to(torch.bfloat16)
        hist = [torch.randn(m, device=dev) for _ in range(3)]
        outs = [xs, torch.empty_like(xs), torch.empty_like(xs)]
        rows = [[1.0, -0.1, 0.2, 0.1, -0.05], [1.0, -0.5, 0.0, 0.0, 0.0], [0.9, 0.05, 0.1, 0.0, 0.0]]
        ops.cfg_multistep(xs, vc, vu, 6.0, rows, hist, outs)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            ops.cfg_multistep(xs, vc, vu, 6.0, rows, hist, outs)
        e1.record()
        torch.cuda.synchronize()
        gbs = 32.0 * m / (e0.elapsed_time(e1) / 5 * 1e-3) / 1e9
        kernels["step"].update({"GBps_on_64Mi_values": round(gbs, 0), "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 3)})
        del xs, vc, vu, hist, outs
    tr.cfg = cfg
    tr.stack.cfg = cfg
    return {"metric": "ms per production denoising step (cond + uncond forward on a cached text context + fused UniPC update)",
            "value": round(ms, 2), "unit": "ms", "steps": steps, "warmup": warmup,
            "config": {"workload": f"C2 stack under the hybrid mask: {cfg.n_blocks} blocks, {n_gen} generator tokens against "
                                   f"{cfg.n_text} cached text keys + their own, guidance 6.0, UniPC flow_shift 10 ({num_steps}-step grid)",
                       "latents": list(lat.shape)},
            "ms_per_forward": round((ms - (step_ms or 0.0)) / 2, 2), "context_precompute_ms_per_prompt": round(ctx_ms, 2),
            "roofline": roofline, "kernels": kernels}


def compact(res):
    """What an extra leg contributes to the headline line."""
    keep = ("metric", "value", "unit", "steps", "warmup", "dtype", "config", "roofline", "kernels", "ms_per_forward",
            "context_precompute_ms_per_prompt", "report")
    out = {k: res[k] for k in keep if k in res}
    if "extra" in res:
        out["ms_per_block"] = res["extra"].get("ms_per_block")
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", default="C2", choices=["C0", "C1", "C2", "C3", "C4"])
    ap.add_argument("--blocks", type=int, default=0, help="override the number of blocks (measurement aid; 0 = config)")
    ap.add_argument("--attn-variant", type=int, default=0)
    ap.add_argument("--gemm-variant", type=int, default=0)
    ap.add_argument("--rope", default="in_attention", choices=["in_attention", "gemm_epilogue", "streaming"])
    ap.add_argument("--no-fused-pack", action="store_true",
                    help="K / V rows from the QKV GEMM and a re-tiling kernel instead of tile images from its epilogue")
    ap.add_argument("--graph", action="store_true",
                    help="record the forward into a HIP graph once and time replays (launch-bound shapes such as C0)")
    ap.add_argument("--residual", default="fp32", choices=["fp32", "bf16"],
                    help="dtype the residual stream is kept in between blocks (fp32 = the default of a stack)")
    ap.add_argument("--qk-norm", action="store_true", help="per-head RMSNorm of Q and K ahead of the rotation (real-checkpoint layout)")
    ap.add_argument("--kv-heads", type=int, default=0, help="K / V heads (grouped-query attention; 0 = as many as query heads)")
    ap.add_argument("--production", action="store_true",
                    help="time production steps instead (C2 only): cond + uncond forward on a cached context + fused UniPC update")
    ap.add_argument("--extras", default="auto", choices=["auto", "all", "none"],
                    help="short legs of the other workloads under extra.workloads (auto = with the plain default workload)")
    ap.add_argument("--extras-budget-s", type=float, default=240.0,
                    help="no further extra leg is started once the run is this many seconds old")
    ap.add_argument("--cpu-sample-tokens", type=int, default=8192)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-copy-mib", type=int, default=0,
                    help="counter calibration aid: after the timed region run ONE plain streaming kernel that reads and "
                         "writes this many MiB (torch.bitwise_not on int32), so that a rocprofv3 --pmc pass of this "
                         "command also holds FETCH_SIZE / WRITE_SIZE for a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        sys.exit(2)

    import torch
    from cosmos_amd import CONFIGS, _lib, ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    cfg = CONFIGS[args.workload]
    plain = not (args.blocks or args.qk_norm or args.kv_heads or args.production or args.graph or args.no_fused_pack
                 or args.attn_variant or args.gemm_variant or args.rope != "in_attention" or args.residual != "fp32"
                 or args.pmc_copy_mib)
    if args.blocks:
        cfg = dataclasses.replace(cfg, n_blocks=args.blocks)
    cfg = dataclasses.replace(cfg, residual_fp32=(args.residual == "fp32"), qk_norm=cfg.qk_norm or args.qk_norm,
                              n_kv_heads=args.kv_heads or cfg.n_kv_heads)
    _lib.load()
    ops.set_variant("attn", args.attn_variant)
    ops.set_variant("gemm", args.gemm_variant)

    def no_nan(o):
        if isinstance(o, dict):
            return {k: no_nan(v) for k, v in o.items()}
        if isinstance(o, (list, tuple)):
            return [no_nan(v) for v in o]
        return None if isinstance(o, float) and o != o else o

    if args.workload == "C1":
        res = bench_attention_only(cfg, 10 if args.steps == 3 else args.steps, args.warmup, dev, args.attn_variant)
        print(json.dumps(no_nan(res)))
        return
    extras = args.extras == "all" or (args.extras == "auto" and plain and args.workload == "C2")
    if args.production:
        if args.workload != "C2":
            print("bench.py: --production runs on the C2 stack", file=sys.stderr)
            sys.exit(2)
        _, tr = run_stack_workload(cfg, args, dev, 1, 0, keep=True)
        res = production_leg(tr, cfg, dev, args.steps, args.warmup)
        res.update({"n_gpus": 1, "ms_per_step": res["value"], "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
                    "dtype": "bf16", "data": "synthetic"})
        print(json.dumps(no_nan(res)))
        return

    res, tr = run_stack_workload(cfg, args, dev, args.steps, args.warmup, keep=extras and args.workload == "C2")
    workloads = {}
    budget_left = lambda: args.extras_budget_s - (time.perf_counter() - T_START)
    if extras:
        def leg(name, fn):
            if budget_left() <= 0:
                workloads[name] = {"skipped": f"run older than --extras-budget-s {args.extras_budget_s:.0f} s"}
                return
            try:
                workloads[name] = compact(fn())
            except Exception as e:      # an extra leg never costs the headline line
                workloads[name] = {"failed": repr(e)[:300]}
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
        if tr is not None:
            leg("C2-production-step", lambda: production_leg(tr, cfg, dev))
            tr = None
            import gc
            gc.collect()
            torch.cuda.empty_cache()
        leg("C1", lambda: bench_attention_only(CONFIGS["C1"], 10, 1, dev))
        for name, steps_, over in (("C3", 3, {}), ("C4", 2, {}),
                                   ("C2-qknorm-gqa8", 2, dict(n_blocks=4, qk_norm=True, n_kv_heads=8))):
            base = CONFIGS["C2" if name.startswith("C2") else name]
            c = dataclasses.replace(base, residual_fp32=True, **over)

            def run(c=c, steps_=steps_):
                r, _ = run_stack_workload(c, args, dev, steps_, 1)
                r["report"] = report_line(c, r["value"], r["roofline"], r["kernels"])
                return r
            leg(name, run)
        res["extra"]["workloads"] = workloads
    cpu = parity = None
    if not args.no_cpu_baseline:
        cpu, parity = cpu_baseline(cfg, args.cpu_sample_tokens, dev)
        res["cpu_baseline"] = {k: v for k, v in cpu.items() if k not in ("ms_per_block", "extrapolated")}
        res["parity"] = parity
    rope_gbps = workloads.get("C1", {}).get("kernels", {}).get("rope_streaming", {}).get("GBps")
    res["report"] = report_line(cfg, res["value"], res["roofline"], res["kernels"], cpu, parity, rope_gbps)
    res["extra"]["bench_wall_s"] = round(time.perf_counter() - T_START, 1)
    print(json.dumps(no_nan(res)))


if __name__ == "__main__":
    main()
