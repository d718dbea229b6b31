"""Host-side logic of the product (positions, rotary tables, segments, configs) against the oracle."""
import pytest
import torch

import oracle as O
from cosmos_amd import CONFIGS, rotary
from cosmos_amd.config import DMConfig


@pytest.mark.parametrize("n_text,grid,n_action", [(0, (4, 16, 16), 0), (5, (2, 3, 4), 0), (7, (2, 4, 3), 6)])
def test_positions_match_oracle(n_text, grid, n_action):
    pos, runs = rotary.build_positions(n_text, grid, n_action)
    spec = ([("text", n_text)] if n_text else []) + [("video", grid)] + ([("action", n_action)] if n_action else [])
    assert torch.equal(pos, O.joint_positions(spec))
    assert sum(r[2] for r in runs) == pos.shape[1]


@pytest.mark.parametrize("layout", ["chunked", "interleaved"])
@pytest.mark.parametrize("hd,sections", [(64, (16, 24, 24)), (128, (32, 48, 48))])
def test_tables_match_oracle(layout, hd, sections):
    pos, _ = rotary.build_positions(9, (3, 5, 4), 2)
    c1, s1 = rotary.rotary_tables(pos, hd, sections, 10000.0, layout)
    c2, s2 = O.mrope_cos_sin(pos, hd, sections, 10000.0, layout)
    assert torch.equal(c1, c2) and torch.equal(s1, s2)
    assert torch.equal(rotary.axis_map(hd, sections, layout), O.mrope_axis_map(hd, sections, layout))


def test_bad_sections_raise():
    with pytest.raises(ValueError):
        rotary.axis_map(64, (16, 24, 20))
    with pytest.raises(ValueError):
        rotary.axis_map(64, (16, 24, 24), "spiral")


def test_configs_match_the_benchmark_text():
    c0, c1, c2, c3, c4 = (CONFIGS[k] for k in ("C0", "C1", "C2", "C3", "C4"))
    assert (c0.n_tokens, c0.d_model, c0.n_heads * c0.head_dim, c0.hidden) == (1024, 1024, 1024, 4096)
    assert c1.n_tokens == 56320 and c2.n_tokens == 56832 and c3.n_tokens == 29440 and c4.fp8
    assert abs(c2.gemm_flops_per_block() / 1e12 - 30.51) < 0.01 and abs(c2.attn_flops_per_block() / 1e12 - 52.92) < 0.01
    assert abs(c0.gemm_flops_per_block() / 1e9 - 34.4) < 0.1
    for c in (c0, c1, c2, c3, c4):
        assert sum(c.mrope_sections) == c.head_dim


def test_stack_segments_meta():
    from cosmos_amd.modules import DMStack
    cfg = DMConfig("t", 128, 2, 64, 256, 0, (2, 2, 2), n_text=3, n_action=2, n_branches=3, mrope_sections=(16, 24, 24))
    st = DMStack(cfg, device="meta")
    assert st.segments() == [(0, 3, 0, False), (3, 8, 1, True), (11, 2, 2, True)]
    cfg1 = DMConfig("t", 128, 2, 64, 256, 0, (2, 2, 2), n_text=3, mrope_sections=(16, 24, 24))
    assert DMStack(cfg1, device="meta").segments() == [(0, 3, 0, False), (3, 8, 0, True)]


@pytest.mark.parametrize("order,corrector,solver_type,grid", [(1, True, "bh2", "plain"), (2, True, "bh2", "plain"), (3, True, "bh1", "library"),
                                                              (2, False, "bh2", "library"), (3, True, "bh2", "plain"),
                                                              (1, True, "bh1", "plain"), (2, True, "bh1", "plain"), (3, True, "bh1", "plain")])
def test_unipc_coefficient_rows_on_the_host(monkeypatch, order, corrector, solver_type, grid):
    """The stepper's host side (folding corrector + predictor + data prediction into three coefficient rows, history
    and buffer rotation) with the fused launch replaced by the same linear combinations in float64 on the CPU:
    must reproduce the tensor-level oracle sampler step by step."""
    import numpy as np
    from cosmos_amd import ops, sampler
    from oracle import unipc as U

    def fake_multistep(x, v_cond, v_uncond, guidance, coef, hist, outs):
        v = v_cond.double() if v_uncond is None else v_uncond.double() + guidance * (v_cond.double() - v_uncond.double())
        ins = [x.double().clone(), v] + [h.double().clone() for h in hist]       # read everything before any write
        for row, out in zip(coef, outs):
            out.copy_(sum(c * t for c, t in zip(row, ins)))

    monkeypatch.setattr(ops, "cfg_multistep", fake_multistep)
    steps, n, guidance = 7, 64, 2.5
    sig = U.flow_sigmas(steps, 3.0) if grid == "plain" else U.diffusers_flow_sigmas(steps, 3.0)
    st = sampler.UniPCStepper(sig, guidance_scale=guidance, solver_order=order, solver_type=solver_type,
                              use_corrector=corrector)
    ref = U.UniPCSampler(sig, solver_order=order, solver_type=solver_type, use_corrector=corrector)
    g = torch.Generator().manual_seed(order)
    x = torch.randn(n, generator=g, dtype=torch.float64)
    xr = x.numpy().copy()
    for i in range(steps):
        vc = torch.randn(n, generator=g, dtype=torch.float64)
        vu = torch.randn(n, generator=g, dtype=torch.float64)
        x = st.step(vc, vu, x)
        xr = ref.step((vu + guidance * (vc - vu)).numpy(), xr)
        assert st.this_order == ref.this_order
        assert np.isfinite(xr).all() and bool(torch.isfinite(x).all()), f"step {i}: non-finite latents"
        assert np.allclose(x.numpy(), xr, rtol=1e-9, atol=1e-9), f"step {i}"
    assert len(st.m_hist) <= order and len(st._spare) <= 1
    with pytest.raises(RuntimeError):
        st.step(vc, vu, x)
    with pytest.raises(ValueError):
        sampler.UniPCStepper([0.5, 0.7, 0.0])
    with pytest.raises(ValueError):
        sampler.UniPCStepper(sig, solver_order=4)
