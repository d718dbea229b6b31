"""float64 NumPy brute force of the DM block for tiny shapes (N <= 64, d <= 64).

Test infrastructure.  Written with explicit loops and scalar formulas so that
it shares no vectorised code path (and no torch call) with ``dm_oracle``; a
dropped term, wrong sign, wrong pair index or transposed operand in either
shows up as a disagreement in tests/test_oracle_brute.py.
Formulas: REF/README.md:74 (block structure) and the operator definitions
cited function by function in ``dm_oracle``.
"""
from __future__ import annotations

import math

import numpy as np


def silu(z):
    return z / (1.0 + np.exp(-z))


def rms_norm(x, w, eps=1e-6):
    out = np.zeros_like(x, dtype=np.float64)
    for i in range(x.shape[0]):
        ms = sum(float(x[i, j]) ** 2 for j in range(x.shape[1])) / x.shape[1]
        r = 1.0 / math.sqrt(ms + eps)
        for j in range(x.shape[1]):
            out[i, j] = x[i, j] * r * w[j]
    return out


def adaln_rms_norm(x, w, shift, scale, eps=1e-6):
    y = rms_norm(x, w, eps)
    for i in range(y.shape[0]):
        for j in range(y.shape[1]):
            y[i, j] = y[i, j] * (1.0 + scale[j]) + shift[j]
    return y


def rope_angles(pos, head_dim, axis_map, base=10000.0):
    """pos[3, N] ints; axis_map[head_dim/2] in {0,1,2}. Returns angle[N, head_dim/2]."""
    half = head_dim // 2
    ang = np.zeros((pos.shape[1], half))
    for n in range(pos.shape[1]):
        for i in range(half):
            ang[n, i] = pos[axis_map[i], n] * base ** (-2.0 * i / head_dim)
    return ang


def apply_rope(x, ang):
    """x[N, H, dh]; each pair (i, i+dh/2) is rotated counter-clockwise by ang[n, i]."""
    N, H, dh = x.shape
    half = dh // 2
    y = np.zeros_like(x, dtype=np.float64)
    for n in range(N):
        for h in range(H):
            for i in range(half):
                c, s = math.cos(ang[n, i]), math.sin(ang[n, i])
                a, b = x[n, h, i], x[n, h, i + half]
                y[n, h, i] = a * c - b * s
                y[n, h, i + half] = a * s + b * c
    return y


def attention(q, k, v, kv_end=None):
    """kv_end[n] (optional): query n sees keys 0 .. kv_end[n]-1 only.  k, v may have fewer heads than q
    (grouped-query attention): query head h then reads K/V head h // (H // Hkv)."""
    N, H, dh = q.shape
    group = H // k.shape[1]
    o = np.zeros((N, H, dh))
    for h in range(H):
        g = h // group
        for n in range(N):
            M = k.shape[0] if kv_end is None else int(kv_end[n])
            sc = np.array([sum(q[n, h, c] * k[m, g, c] for c in range(dh)) for m in range(M)]) / math.sqrt(dh)
            e = np.exp(sc - sc.max())
            p = e / e.sum()
            for c in range(dh):
                o[n, h, c] = sum(p[m] * v[m, g, c] for m in range(M))
    return o


def linear(a, w):
    """a[N, K] . w[O, K]^T"""
    out = np.zeros((a.shape[0], w.shape[0]))
    for i in range(a.shape[0]):
        for j in range(w.shape[0]):
            out[i, j] = float(np.dot(a[i].astype(np.float64), w[j].astype(np.float64)))
    return out


def dm_block(x, weight_sets, mod, pos, axis_map, n_heads, segments=None, eps=1e-6, base=10000.0):
    """Same contract as dm_oracle.dm_block but takes positions + axis map instead of tables."""
    x = x.astype(np.float64)
    N, d = x.shape
    dh = d // n_heads
    if segments is None:
        segments = [(0, N, 0, mod is not None)]
    zeros, ones = np.zeros(d), np.ones(d)
    q = np.zeros((N, d)); k = np.zeros((N, d)); v = np.zeros((N, d))
    for (s0, ln, ws, modulated) in segments:
        p = weight_sets[ws]
        sh, sc = (mod[0], mod[1]) if modulated else (zeros, zeros)
        y = adaln_rms_norm(x[s0:s0 + ln], p["norm1_w"], sh, sc, eps)
        q[s0:s0 + ln] = linear(y, p["wq"]); k[s0:s0 + ln] = linear(y, p["wk"]); v[s0:s0 + ln] = linear(y, p["wv"])
    ang = rope_angles(pos, dh, axis_map, base)
    qh = apply_rope(q.reshape(N, n_heads, dh), ang)
    kh = apply_rope(k.reshape(N, n_heads, dh), ang)
    o = attention(qh, kh, v.reshape(N, n_heads, dh)).reshape(N, d)
    out = np.zeros((N, d))
    for (s0, ln, ws, modulated) in segments:
        p = weight_sets[ws]
        g1, sh2, sc2, g2 = (mod[2], mod[3], mod[4], mod[5]) if modulated else (ones, zeros, zeros, ones)
        xs = x[s0:s0 + ln] + g1 * linear(o[s0:s0 + ln], p["wo"])
        y2 = adaln_rms_norm(xs, p["norm2_w"], sh2, sc2, eps)
        u = silu(linear(y2, p["wg"])) * linear(y2, p["wu"])
        out[s0:s0 + ln] = xs + g2 * linear(u, p["wd"])
    return out
