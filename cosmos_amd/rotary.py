"""Host-side 3-D mRoPE bookkeeping: position ids of a joint text / video / action sequence and the
cos/sin tables the kernels consume (``image_rotary_emb`` in the diffusers calling idiom).

Everything that distinguishes mRoPE layouts lives here, in the tables; the kernels only see
cos/sin[N, head_dim/2] for rotate-half pairs (i, i + head_dim/2).
Position rules follow transformers models/cosmos3_omni/modeling_cosmos3_omni.py:124-174,241-259;
table layouts follow models/qwen2_vl/modeling_qwen2_vl.py:212-217 (chunked) and
models/qwen3_vl/modeling_qwen3_vl.py:372-388 (interleaved).
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import torch

Segment = Tuple[int, int, int, bool]      # (start, length, branch index, modulated)


def axis_map(head_dim: int, sections: Sequence[int], layout: str = "chunked") -> torch.Tensor:
    """Axis (0 = t, 1 = h, 2 = w) followed by each of the head_dim/2 rotary pairs."""
    if sum(sections) != head_dim or any(s % 2 for s in sections):
        raise ValueError(f"mrope sections {tuple(sections)} must be even and sum to head_dim={head_dim}")
    n_t, n_h, n_w = (s // 2 for s in sections)
    half = head_dim // 2
    out = torch.zeros(half, dtype=torch.long)
    if layout == "chunked":
        out[n_t:n_t + n_h] = 1
        out[n_t + n_h:] = 2
    elif layout == "interleaved":
        out[1:n_h * 3:3] = 1
        out[2:n_w * 3:3] = 2
    else:
        raise ValueError(f"unknown mrope layout {layout!r}")
    return out


def build_positions(n_text: int, grid: Sequence[int], n_action: int = 0,
                    n_audio: int = 0) -> Tuple[torch.Tensor, List[Tuple[str, int, int]]]:
    """Positions [3, N] of the joint sequence text | video | audio | action, plus the (kind, start, length) runs.

    A 1-D run at offset s gets (s+j, s+j, s+j) and advances s by its length; a T x H x W grid gets
    (s+t, s+h, s+w) in row-major order and advances s by max(H, W).
    """
    runs, pos, cur, tok = [], [], 0, 0
    if n_text:
        p = torch.arange(n_text, dtype=torch.long) + cur
        pos.append(torch.stack([p, p, p]))
        runs.append(("text", tok, n_text)); tok += n_text; cur += n_text
    T, H, W = (int(g) for g in grid)
    if T * H * W:
        t = (torch.arange(T) + cur).view(T, 1, 1).expand(T, H, W)
        h = (torch.arange(H) + cur).view(1, H, 1).expand(T, H, W)
        w = (torch.arange(W) + cur).view(1, 1, W).expand(T, H, W)
        pos.append(torch.stack([t.reshape(-1), h.reshape(-1), w.reshape(-1)]))
        runs.append(("video", tok, T * H * W)); tok += T * H * W; cur += max(H, W)
    for kind, n in (("audio", n_audio), ("action", n_action)):      # 1-D runs like text
        if n:
            p = torch.arange(n, dtype=torch.long) + cur
            pos.append(torch.stack([p, p, p]))
            runs.append((kind, tok, n)); tok += n; cur += n
    return torch.cat(pos, dim=1), runs


def rotary_tables(positions: torch.Tensor, head_dim: int, sections: Sequence[int], base: float = 10000.0,
                  layout: str = "chunked", device=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos, sin [N, head_dim/2] in fp32: angle[n, i] = positions[axis(i), n] * base^(-2i/head_dim)."""
    half = head_dim // 2
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    amap = axis_map(head_dim, sections, layout)
    ang = positions.to(torch.float32)[amap, :].t().contiguous() * inv_freq.view(1, half)
    cos, sin = ang.cos().contiguous(), ang.sin().contiguous()
    if device is not None:
        cos, sin = cos.to(device), sin.to(device)
    return cos, sin
