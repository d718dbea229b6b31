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
