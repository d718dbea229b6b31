"""The fp32 torch oracle against the independent float64 NumPy brute force (oracle/brute.py)
and against closed forms the mathematics fixes."""
import math

import numpy as np
import pytest
import torch

import oracle as O
from oracle import brute as B


def _weights(g, d, h, dh=None, qk=False):
    r = lambda *s: torch.randn(*s, generator=g) * 0.3
    w = dict(norm1_w=1 + r(d), wq=r(d, d), wk=r(d, d), wv=r(d, d), wo=r(d, d), norm2_w=1 + r(d),
             wg=r(h, d), wu=r(h, d), wd=r(d, h))
    return w


def _np(w):
    return {k: v.double().numpy() for k, v in w.items()}


@pytest.mark.parametrize("layout", ["chunked", "interleaved"])
def test_block_vs_brute_single_segment(layout):
    g = torch.Generator().manual_seed(1)
    N, d, H, h = 12, 16, 2, 24
    x = torch.randn(N, d, generator=g)
    w = _weights(g, d, h)
    mod = [torch.randn(d, generator=g) * 0.5 for _ in range(6)]
    pos = O.vision_positions(3, (2, 2, 3))
    sections = (2, 2, 4)
    cos, sin = O.mrope_cos_sin(pos, d // H, sections, 10000.0, layout)
    y = O.dm_block(x, [w], mod, cos, sin, H)
    amap = O.mrope_axis_map(d // H, sections, layout).numpy()
    yb = B.dm_block(x.numpy(), [_np(w)], [m.double().numpy() for m in mod], pos.numpy(), amap, H)
    assert np.abs(y.numpy() - yb).max() < 2e-4 * np.abs(yb).max()


def test_block_vs_brute_mot_three_segments():
    g = torch.Generator().manual_seed(2)
    d, H, h = 16, 2, 24
    segs_spec = [("text", 5), ("video", (2, 2, 2)), ("action", 3)]
    pos = O.joint_positions(segs_spec)
    N = pos.shape[1]
    segments = [(0, 5, 0, False), (5, 8, 1, True), (13, 3, 2, True)]
    ws = [_weights(g, d, h) for _ in range(3)]
    x = torch.randn(N, d, generator=g)
    mod = [torch.randn(d, generator=g) * 0.5 for _ in range(6)]
    cos, sin = O.mrope_cos_sin(pos, d // H, (4, 2, 2), 10000.0, "chunked")
    y = O.dm_block(x, ws, mod, cos, sin, H, segments)
    amap = O.mrope_axis_map(d // H, (4, 2, 2)).numpy()
    yb = B.dm_block(x.numpy(), [_np(w) for w in ws], [m.double().numpy() for m in mod], pos.numpy(), amap, H, segments)
    assert np.abs(y.numpy() - yb).max() < 2e-4 * np.abs(yb).max()
    # equal weight sets + all modulated == single-segment block
    same = [ws[1]] * 3
    y1 = O.dm_block(x, same, mod, cos, sin, H, [(0, 5, 0, True), (5, 8, 1, True), (13, 3, 2, True)])
    y2 = O.dm_block(x, [ws[1]], mod, cos, sin, H)
    assert torch.allclose(y1, y2, atol=1e-5)
    # row-sampled form
    rows = torch.tensor([1, 6, 14])
    yr = O.dm_block(x, ws, mod, cos, sin, H, segments, attn_rows=rows)
    assert torch.allclose(yr, y[rows], atol=1e-5)


def test_block_vs_brute_four_modalities_with_audio():
    """text | video | audio | action, four weight sets: audio is a 1-D run after the video grid (offset max(H, W)),
    action follows it."""
    g = torch.Generator().manual_seed(4)
    d, H, h = 16, 2, 24
    pos = O.joint_positions([("text", 4), ("video", (1, 2, 3)), ("audio", 3), ("action", 2)])
    assert pos[:, 10:13].tolist() == [[7, 8, 9]] * 3 and pos[:, 13:].tolist() == [[10, 11]] * 3      # 4 + max(2, 3) = 7
    N = pos.shape[1]
    segments = [(0, 4, 0, False), (4, 6, 1, True), (10, 3, 3, True), (13, 2, 2, True)]
    ws = [_weights(g, d, h) for _ in range(4)]
    x = torch.randn(N, d, generator=g)
    mod = [torch.randn(d, generator=g) * 0.5 for _ in range(6)]
    cos, sin = O.mrope_cos_sin(pos, d // H, (4, 2, 2), 10000.0, "chunked")
    y = O.dm_block(x, ws, mod, cos, sin, H, segments)
    amap = O.mrope_axis_map(d // H, (4, 2, 2)).numpy()
    yb = B.dm_block(x.numpy(), [_np(w) for w in ws], [m.double().numpy() for m in mod], pos.numpy(), amap, H, segments)
    assert np.abs(y.numpy() - yb).max() < 2e-4 * np.abs(yb).max()
    # the audio run really uses its own weights
    ws2 = ws[:3] + [ws[1]]
    assert float((O.dm_block(x, ws2, mod, cos, sin, H, segments) - y)[10:13].abs().max()) > 1e-3


def test_rms_norm_closed_forms():
    d = 32
    w = torch.linspace(0.5, 1.5, d); sc = torch.linspace(-0.2, 0.3, d); sh = torch.linspace(-1, 1, d)
    x = torch.full((3, d), 2.5)
    y = O.adaln_rms_norm(x, w, sh, sc, eps=0.0)      # constant row -> x/rms = 1
    assert torch.allclose(y, (w * (1 + sc) + sh).expand(3, d), atol=1e-6)
    x = torch.randn(4, d)
    assert torch.allclose(O.rms_norm(7.0 * x, w, 0.0), O.rms_norm(x, w, 0.0), atol=1e-5)
    # eps term: x = 0 -> 0 ; mean-square definition (not sum, not variance-about-mean)
    assert torch.equal(O.rms_norm(torch.zeros(1, d), w), torch.zeros(1, d))
    e = torch.zeros(1, d); e[0, 3] = 4.0
    assert math.isclose(float(O.rms_norm(e, torch.ones(d), 0.0)[0, 3]), math.sqrt(d), rel_tol=1e-6)


def test_rope_properties():
    g = torch.Generator().manual_seed(3)
    dh, H = 32, 2
    sections = (8, 12, 12)
    q = torch.randn(1, H, dh, generator=g); k = torch.randn(1, H, dh, generator=g)

    def rot(x, p):
        cos, sin = O.mrope_cos_sin(torch.tensor(p).view(3, 1), dh, sections)
        return O.apply_mrope(x, cos, sin)
    # identity at position 0, isometry, relative-position property per axis
    assert torch.allclose(rot(q, (0, 0, 0)), q, atol=1e-6)
    assert torch.allclose(rot(q, (5, 9, 2)).norm(), q.norm(), rtol=1e-5)
    a = (rot(q, (5, 9, 2)) * rot(k, (3, 4, 7))).sum()
    b = (rot(q, (12, 15, 1)) * rot(k, (10, 10, 6))).sum()       # same differences (2, 5, -5)
    assert torch.allclose(a, b, rtol=1e-4, atol=1e-4)
    c = (rot(q, (5, 9, 2)) * rot(k, (3, 4, 6))).sum()           # different w difference
    assert not torch.allclose(a, c, rtol=1e-3, atol=1e-3)
    # pair 0 has frequency 1: position pi on its axis negates channels 0 and dh/2 only
    x = torch.zeros(1, 1, dh); x[0, 0, 0] = 1.0
    cos, sin = O.mrope_cos_sin(torch.tensor([[1], [0], [0]]), dh, sections)
    y = O.apply_mrope(x, cos, sin)[0, 0]
    assert math.isclose(float(y[0]), math.cos(1.0), rel_tol=1e-6) and math.isclose(float(y[dh // 2]), math.sin(1.0), rel_tol=1e-6)
    # axis map: chunked pair counts
    assert O.mrope_axis_map(64, (16, 24, 24)).tolist() == [0] * 8 + [1] * 12 + [2] * 12
    assert O.mrope_axis_map(128, (32, 48, 48)).tolist() == [0] * 16 + [1] * 24 + [2] * 24


def test_attention_closed_forms():
    g = torch.Generator().manual_seed(4)
    N, H, dh = 9, 2, 8
    q = torch.randn(N, H, dh, generator=g); k = torch.randn(N, H, dh, generator=g); v = torch.randn(N, H, dh, generator=g)
    # V constant along keys -> output equals it; one key -> output is its V
    vc = v[:1].expand(N, H, dh)
    assert torch.allclose(O.attention(q, k, vc), vc, atol=1e-6)
    assert torch.allclose(O.attention(q, k[:1], v[:1]), v[:1].expand(N, H, dh), atol=1e-6)
    # key permutation invariance; zero queries -> mean of V
    perm = torch.randperm(N, generator=g)
    assert torch.allclose(O.attention(q, k, v), O.attention(q, k[perm], v[perm]), atol=1e-5)
    assert torch.allclose(O.attention(torch.zeros_like(q), k, v), v.mean(0, keepdim=True).expand(N, H, dh), atol=1e-6)
    # scaling is 1/sqrt(dh): two keys, explicit softmax
    q1 = torch.ones(1, 1, 4); k2 = torch.tensor([[[1.0, 0, 0, 0]], [[0, 0, 0, 0.0]]]); v2 = torch.tensor([[[1.0, 0, 0, 0]], [[0, 1.0, 0, 0]]])
    p = math.exp(0.5) / (math.exp(0.5) + 1.0)
    assert torch.allclose(O.attention(q1, k2, v2)[0, 0, :2], torch.tensor([p, 1 - p]), atol=1e-6)


def test_gate_zero_is_identity_and_swiglu_zero():
    g = torch.Generator().manual_seed(5)
    N, d, H, h = 6, 16, 2, 24
    x = torch.randn(N, d, generator=g); w = _weights(g, d, h)
    mod = [torch.randn(d, generator=g) for _ in range(6)]; mod[2] = torch.zeros(d); mod[5] = torch.zeros(d)
    cos, sin = O.mrope_cos_sin(O.text_positions(0, N), d // H, (4, 2, 2))
    assert torch.allclose(O.dm_block(x, [w], mod, cos, sin, H), x, atol=1e-6)
    assert torch.equal(O.swiglu(torch.zeros(2, d), w["wg"], w["wu"], w["wd"]), torch.zeros(2, d))


def test_timestep_embedding_and_modulation_split():
    e = O.timestep_embedding(torch.tensor([0.0]), 256)
    assert e.shape == (1, 256) and torch.equal(e[0, :128], torch.ones(128)) and torch.equal(e[0, 128:], torch.zeros(128))
    e = O.timestep_embedding(torch.tensor([3.0]), 256)
    assert math.isclose(float(e[0, 0]), math.cos(3.0), rel_tol=1e-6) and math.isclose(float(e[0, 128]), math.sin(3.0), rel_tol=1e-6)
    assert math.isclose(float(e[0, 127 + 128]), math.sin(3.0 * 10000 ** (-127 / 128)), rel_tol=1e-5)
    d = 4
    c = torch.zeros(1, d)                  # silu(0)=0 -> m = bias
    b = torch.arange(6 * d, dtype=torch.float32)
    m = O.adaln_modulation(c, torch.randn(6 * d, d), b)
    assert len(m) == 6 and torch.equal(m[1], b[d:2 * d]) and torch.equal(m[5], b[5 * d:])


def test_e4m3_quant():
    g = torch.Generator().manual_seed(6)
    a = torch.randn(5, 64, generator=g) * torch.tensor([1e-3, 1.0, 30.0, 1e4, 0.0]).view(5, 1)
    q, s = O.quant_e4m3_rows(a)
    assert float(s[4]) == 1.0 and torch.equal(q[4], torch.zeros(64))
    assert torch.all(q.abs().amax(-1)[:4] == 448.0)                     # absmax maps to exactly 448
    rel = ((q * s - a).abs() / a.abs().amax(-1, keepdim=True).clamp_min(1e-30))[:4]
    assert float(rel.max()) <= 2 ** -4
    # values are exactly representable e4m3 numbers
    assert torch.equal(q, q.to(torch.float8_e4m3fn).to(torch.float32))
    # scale outer-product identity
    w = torch.randn(7, 64, generator=g)
    wq, sw = O.quant_e4m3_weight(w)
    c1 = O.fp8_linear(a, w)
    c2 = (q * s) @ (wq * sw).t()
    assert torch.allclose(c1, c2, rtol=1e-4, atol=1e-3)
    assert O.max_rel_err(c1[:4], a[:4] @ w.t()) < 5e-2


def test_cfg_step_closed_forms():
    g = torch.Generator().manual_seed(1)
    x, vc, vu, h = (torch.randn(64, generator=g) for _ in range(4))
    out, v = O.cfg_step(x, vc, vu, 1.0, [0.0, 1.0])
    assert torch.allclose(out, vc, atol=1e-6) and torch.allclose(v, vc, atol=1e-6)           # guidance 1 -> cond
    assert torch.equal(O.cfg_step(x, vc, vu, 0.0, [0.0, 1.0])[0], vu)                        # guidance 0 -> uncond
    assert torch.equal(O.cfg_step(x, vc, None, 9.0, [1.0, 0.0])[0], x)                       # no update
    # the guided prediction extrapolates: v - vu = g (vc - vu)
    _, v6 = O.cfg_step(x, vc, vu, 6.0, [1.0, 0.0])
    assert torch.allclose(v6 - vu, 6.0 * (vc - vu), atol=1e-5)
    # linear in every tensor and coefficient (float64 brute force)
    want = (0.5 * x.double() - 0.25 * (vu.double() + 2.0 * (vc.double() - vu.double())) + 0.125 * h.double())
    got, _ = O.cfg_step(x, vc, vu, 2.0, [0.5, -0.25, 0.125], [h])
    assert torch.allclose(got.double(), want, atol=1e-6)
    # noise levels: endpoints, monotone, shift 1 = uniform grid, shift identity sigma' (1 + (s-1) sigma) = s sigma
    s1, s3 = O.flow_sigmas(10, 1.0), O.flow_sigmas(10, 3.0)
    assert s1[0] == 1.0 and s1[-1] == 0.0 and torch.allclose(s1, torch.linspace(1, 0, 11, dtype=torch.float64))
    assert s3[0] == 1.0 and s3[-1] == 0.0 and bool((s3[1:] < s3[:-1]).all()) and bool((s3[1:-1] > s1[1:-1]).all())
    assert torch.allclose(s3 * (1 + 2.0 * s1), 3.0 * s1)


def test_hybrid_mask_attention():
    """Masked oracle attention against the float64 brute force (which simply drops the hidden keys) and against
    the decomposition the mask implies: a prefix row is plain attention over the keys up to itself, a later row is
    plain attention over everything."""
    g = torch.Generator().manual_seed(12)
    N, H, dh, P = 11, 2, 8, 4
    q, k, v = (torch.randn(N, H, dh, generator=g) for _ in range(3))
    kv_end = O.hybrid_kv_end(N, P)
    assert kv_end.tolist() == [1, 2, 3, 4] + [N] * (N - P)
    got = O.attention(q, k, v, chunk=3, kv_end=kv_end)
    want = B.attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), kv_end.numpy())
    assert np.abs(got.double().numpy() - want).max() < 1e-5
    for i in range(N):
        e = int(kv_end[i])
        row = O.attention(q[i:i + 1], k[:e], v[:e])
        assert torch.allclose(got[i:i + 1], row, atol=1e-6)
    rows = torch.tensor([0, 3, 4, 10])
    assert torch.allclose(O.attention_rows(q[rows], k, v, kv_end[rows]), got[rows], atol=1e-6)
    assert torch.allclose(got[0], v[0], atol=1e-6)            # the first token sees only itself
    # inside a block: the prefix rows do not depend on anything after the prefix
    d = H * dh
    x = torch.randn(N, d, generator=g)
    w = {n: torch.randn(s, generator=g) * 0.3 for n, s in dict(wq=(d, d), wk=(d, d), wv=(d, d), wo=(d, d), wg=(2 * d, d),
                                                              wu=(2 * d, d), wd=(d, 2 * d)).items()}
    w.update(norm1_w=torch.ones(d), norm2_w=torch.ones(d))
    mod = [torch.randn(d, generator=g) * 0.1 for _ in range(6)]
    pos = O.text_positions(0, N)
    cos, sin = O.mrope_cos_sin(pos, dh, (2, 2, 4))
    segs = [(0, P, 0, False), (P, N - P, 0, True)]
    y = O.dm_block(x, [w], mod, cos, sin, H, segs, causal_prefix=P)
    x2 = x.clone(); x2[P:] = torch.randn(N - P, d, generator=g)
    y2 = O.dm_block(x2, [w], mod, cos, sin, H, segs, causal_prefix=P)
    assert torch.allclose(y[:P], y2[:P], atol=1e-6) and not torch.allclose(y[P:], y2[P:], atol=1e-3)
    # ... and equal the block run on the prefix alone with a causal mask
    y3 = O.dm_block(x[:P], [w], mod, cos[:P], sin[:P], H, [(0, P, 0, False)], causal_prefix=P)
    assert torch.allclose(y[:P], y3, atol=1e-5)


def test_grouped_query_attention_brute_and_equivalence():
    """Grouped K/V heads: against the float64 brute force (with the hybrid mask on top), and against plain
    multi-head attention on K/V whose heads were repeated by hand."""
    g = torch.Generator().manual_seed(13)
    N, H, Hkv, dh = 9, 6, 2, 8
    q = torch.randn(N, H, dh, generator=g)
    k, v = (torch.randn(N, Hkv, dh, generator=g) for _ in range(2))
    kv_end = O.hybrid_kv_end(N, 3)
    got = O.attention(q, k, v, chunk=4, kv_end=kv_end)
    want = B.attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), kv_end.numpy())
    assert np.abs(got.double().numpy() - want).max() < 1e-5
    rep = lambda t: torch.stack([t[:, h // (H // Hkv)] for h in range(H)], dim=1)
    assert torch.allclose(O.attention(q, k, v), O.attention(q, rep(k), rep(v)), atol=1e-6)
