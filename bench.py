#!/usr/bin/env python3
"""Benchmark of the DM-block hot path on one MI355X.

A "step" is one denoising step = one forward of the whole DiT stack over one synthetic joint sequence.
Default workload: the full video DiT stack (28 blocks, d=4096, 32x128 heads, SwiGLU 16384, 512 text +
16x44x80 video tokens = 56,832 tokens, bf16, random-init weights N(0, 0.02)).
Prints ONE JSON line: ms per denoising step, the MFMA roofline of the dominant kernel (attention; duration
from HIP events around every attention launch inside the timed region) and a CPU baseline (the fp32 oracle on
this host's cores, bounded sample, extrapolated).
"""
import argparse
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
# from inside this process, so other shapes report null.
ATTN_TRAFFIC_BYTES = {(56832, 32, 128): 8.61e9 + 0.466e9}


def cpu_baseline(cfg, sample_tokens: int):
    """fp32 oracle of ONE block on `sample_tokens` tokens of the same width (0 = all tokens: minutes of CPU time at the
    benchmark sizes), timed on the host cores; the GEMM part scales linearly and the attention part quadratically with
    the token count."""
    import torch
    import oracle as O
    d, h, H = cfg.d_model, cfg.hidden, cfg.n_heads
    g = torch.Generator().manual_seed(0)
    n = min(sample_tokens, cfg.n_tokens) if sample_tokens > 0 else cfg.n_tokens
    x = torch.randn(n, d, generator=g)
    w = dict(norm1_w=torch.ones(d), norm2_w=torch.ones(d))
    for name, shape in (("wq", (d, d)), ("wk", (d, d)), ("wv", (d, d)), ("wo", (d, d)), ("wg", (h, d)), ("wu", (h, d)),
                        ("wd", (d, h))):
        w[name] = torch.randn(shape, generator=g) * 0.02
    mod = [torch.randn(d, generator=g) * 0.1 for _ in range(6)]
    pos = O.text_positions(0, n)
    cos, sin = O.mrope_cos_sin(pos, cfg.head_dim, cfg.mrope_sections)
    q = torch.randn(n, H, cfg.head_dim, generator=g)
    def best_of_two(fn):
        best = float("inf")
        for _ in range(2):          # the first call of a size pays allocator growth / page faults
            t0 = time.perf_counter()
            fn()
            best = min(best, time.perf_counter() - t0)
        return best
    t_attn = best_of_two(lambda: O.attention(q, q, q))
    t_block = best_of_two(lambda: O.dm_block(x, [w], mod, cos, sin, H))
    t_lin = max(t_block - t_attn, 0.0)
    ratio = cfg.n_tokens / n
    per_block = t_lin * ratio + t_attn * ratio * ratio
    return {"value": round(per_block * max(cfg.n_blocks, 1) * 1e3, 1),
            "unit": "ms per denoising step (extrapolated)" if (ratio > 1 or cfg.n_blocks > 1) else "ms per denoising step",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"fp32 oracle, one block on {n} of {cfg.n_tokens} tokens at full width: {t_block:.2f} s "
                      f"(attention {t_attn:.2f} s); linear part x{ratio:.2f}, attention x{ratio * ratio:.1f}, "
                      f"x{max(cfg.n_blocks, 1)} blocks"}


def bench_attention_only(cfg, args, dev):
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
    ws = torch.empty(ops.attn_workspace_bytes(n, H, hd), dtype=torch.uint8, device=dev)
    step = lambda: ops.attention(qkv[:, :d], qkv[:, d:2 * d], qkv[:, 2 * d:], H, hd, out=out, workspace=ws, cos=cos, sin=sin)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ops.time_attention(True)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ev = ops.time_attention(False)
    assert bool(torch.isfinite(out.float()).all()), "non-finite output"
    ms = wall * 1e3 / args.steps
    k_ms = sum(a.elapsed_time(b) for a, b in ev) / len(ev)
    flops = 4.0 * float(n) ** 2 * d
    tf = flops / (k_ms * 1e-3) / 1e12
    print(json.dumps({
        "metric": "ms per mRoPE + attention pass on 1 GPU", "value": round(ms, 3), "unit": "ms", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 3), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"C1: mRoPE + full attention, {H}x{hd} heads, grid {cfg.grid[0]}x{cfg.grid[1]}x{cfg.grid[2]} = {n} tokens",
                   "n_tokens": n, "attn_variant": args.attn_variant},
        "roofline": {"bound": "mfma", "kernel": "attn_fwd_pipe_kernel", "achieved": round(tf, 1), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tf / PEAK_BF16_TFLOPS, 4), "traffic": None,
                     "flops_per_launch": flops, "avg_launch_ms": round(k_ms, 3), "launches": len(ev)},
        "extra": {"pack_kv_and_launch_overhead_ms": round(ms - k_ms, 3), "device": torch.cuda.get_device_name(0)}}))


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

    import dataclasses
    import torch
    from cosmos_amd import CONFIGS, DMStack, _lib, ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    cfg = CONFIGS[args.workload]
    if args.blocks:
        cfg = dataclasses.replace(cfg, n_blocks=args.blocks)
    cfg = dataclasses.replace(cfg, residual_fp32=(args.residual == "fp32"))
    _lib.load()
    if args.workload == "C1" and args.steps == 3:
        args.steps = 10
    ops.set_variant("attn", args.attn_variant)
    ops.set_variant("gemm", args.gemm_variant)

    if args.workload == "C1":
        return bench_attention_only(cfg, args, dev)
    stack = DMStack(cfg, device=dev)
    stack.reset_parameters()
    if args.rope != "in_attention" or args.no_fused_pack:
        from cosmos_amd import DMAttnProcessor
        for blk in stack.blocks:
            blk.attn.set_processor(DMAttnProcessor(rope=args.rope, fuse_kv_pack=not args.no_fused_pack))
    # the weights were drawn from a generator seeded with cfg.seed: the inputs take another stream (the same seed would
    # reproduce the weights' random numbers, i.e. token rows parallel to weight rows)
    g = torch.Generator(device=dev).manual_seed(cfg.seed + 1000)
    xv = torch.randn((1, cfg.n_video, cfg.d_model), generator=g, device=dev).to(torch.bfloat16)
    xt = torch.randn((1, cfg.n_text, cfg.d_model), generator=g, device=dev).to(torch.bfloat16) if cfg.n_text else None
    xa = torch.randn((1, cfg.n_action, cfg.d_model), generator=g, device=dev).to(torch.bfloat16) if cfg.n_action else None
    t = torch.rand(1, generator=g, device=dev) * 1000.0

    if args.graph:
        graphed = stack.capture(xv, t, encoder_hidden_states=xt, action_states=xa)

        def step():
            return graphed(xv, t, encoder_hidden_states=xt, action_states=xa)["sample"]
    else:
        def step():
            return stack(xv, t, encoder_hidden_states=xt, action_states=xa)[0]

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ops.time_attention(True)
    ops.time_ops(True)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    events = ops.time_attention(False)
    op_events = ops.time_ops(False)
    assert bool(torch.isfinite(out.float()).all()), "non-finite output"
    if args.pmc_copy_mib:
        src = torch.zeros(args.pmc_copy_mib << 18, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        torch.bitwise_not(src, out=dst)
        torch.cuda.synchronize()
        del src, dst

    ms_per_step = wall * 1e3 / args.steps
    attn_ms = [a.elapsed_time(b) for a, b in events]
    timed_launches = len(attn_ms)
    if not attn_ms:      # graph replays launch nothing from Python: no per-launch events; figures below are then null
        attn_ms = [float("nan")]
    attn_avg_ms = sum(attn_ms) / len(attn_ms)
    attn_flops = cfg.attn_flops_per_block()
    attn_tflops = attn_flops / (attn_avg_ms * 1e-3) / 1e12
    gemm_ms_per_block = ms_per_step / cfg.n_blocks - attn_avg_ms     # everything that is not attention
    gemm_tflops = cfg.gemm_flops_per_block() / (gemm_ms_per_block * 1e-3) / 1e12
    peak = PEAK_BF16_TFLOPS
    # per-category kernel time from HIP events around every launcher (ms per block)
    cat_ms = {}
    for cat, a, b in op_events:
        cat_ms[cat] = cat_ms.get(cat, 0.0) + a.elapsed_time(b)
    per_block = {k: v / (args.steps * cfg.n_blocks) for k, v in cat_ms.items()}
    gemm_peak = PEAK_FP8_TFLOPS if cfg.fp8 else peak
    kernels = {}
    if per_block.get("gemm"):
        tf = cfg.gemm_flops_per_block() / (per_block["gemm"] * 1e-3) / 1e12
        kernels["gemm"] = {"ms_per_block": round(per_block["gemm"], 3), "tflops": round(tf, 1), "frac_of_mfma_peak": round(tf / gemm_peak, 4)}
    nd = cfg.n_tokens * cfg.d_model
    xb = 4 if cfg.residual_fp32 else 2                         # bytes per element of the residual stream
    hbm_bytes = {"norm": 2 * (xb + (1 if cfg.fp8 else 2)) * nd,  # two norms per block: read the stream, write bf16 (or e4m3)
                 "pack_kv": 8 * nd + 8 * cfg.n_tokens * (cfg.head_dim // 2),   # K, V in; two tile images out; cos/sin
                 "quant": 2 * 3 * nd + 3 * cfg.n_tokens * cfg.hidden,           # attention output and SwiGLU hidden -> e4m3
                 "rope": 8 * nd}
    for cat, nbytes in hbm_bytes.items():
        if per_block.get(cat):
            gbs = nbytes / (per_block[cat] * 1e-3) / 1e9
            kernels[cat] = {"ms_per_block": round(per_block[cat], 3), "GBps": round(gbs, 0), "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 3)}
    res = {
        "metric": "ms per denoising step (DiT stack) on 1 GPU",
        "value": round(ms_per_step, 2), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 2), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8-e4m3 GEMMs, bf16 attention" if cfg.fp8 else "bf16", "data": "synthetic",
        "config": {"workload": f"{cfg.name}: {cfg.n_blocks} DM blocks, d={cfg.d_model}, {cfg.n_heads}x{cfg.head_dim} heads, "
                               f"SwiGLU {cfg.hidden}, {cfg.n_text} text + {cfg.grid[0]}x{cfg.grid[1]}x{cfg.grid[2]} video"
                               f" + {cfg.n_action} action = {cfg.n_tokens} tokens, batch 1",
                   "n_tokens": cfg.n_tokens, "n_blocks": cfg.n_blocks, "attn_variant": args.attn_variant, "gemm_variant": args.gemm_variant, "rope": args.rope, "kv_pack": "separate kernel" if args.no_fused_pack or args.rope != "in_attention" else "qkv gemm epilogue",
                   "residual_stream": args.residual, "hip_graph": bool(args.graph)},
        "roofline": {"bound": "mfma", "kernel": "attn_fwd_pipe_kernel", "achieved": round(attn_tflops, 1), "peak": peak,
                     "unit": "TFLOP/s", "frac": round(attn_tflops / peak, 4),
                     "traffic": ATTN_TRAFFIC_BYTES.get((cfg.n_tokens, cfg.n_heads, cfg.head_dim))
                     if args.attn_variant == 0 else None,
                     "traffic_source": "stored figure of two rocprofv3 --pmc passes (FETCH_SIZE, WRITE_SIZE) over this kernel at "
                                       "this shape, profiles/c2_one_block_pmc_counters.txt; counters cannot be read in-process",
                     "flops_per_launch": attn_flops, "avg_launch_ms": round(attn_avg_ms, 3), "launches": len(attn_ms)},
        "kernels": kernels,
        "extra": {"ms_per_block": round(ms_per_step / cfg.n_blocks, 3),
                  "non_attention_ms_per_block": round(gemm_ms_per_block, 3),
                  "gemm_tflops_lower_bound": round(gemm_tflops, 1),
                  "gemm_frac_of_peak_lower_bound": round(gemm_tflops / (PEAK_FP8_TFLOPS if cfg.fp8 else peak), 4),
                  "total_tflops": round((attn_flops + cfg.gemm_flops_per_block()) * cfg.n_blocks / (ms_per_step * 1e-3) / 1e12, 1),
                  "device": torch.cuda.get_device_name(0)},
    }
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(cfg, args.cpu_sample_tokens)
    def no_nan(o):
        if isinstance(o, dict):
            return {k: no_nan(v) for k, v in o.items()}
        return None if isinstance(o, float) and o != o else o
    res["roofline"]["launches"] = timed_launches
    print(json.dumps(no_nan(res)))


if __name__ == "__main__":
    main()
