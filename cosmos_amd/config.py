"""Frozen configurations of the benchmark workloads (C0..C4)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class DMConfig:
    name: str
    d_model: int
    n_heads: int
    head_dim: int
    hidden: int
    n_blocks: int
    grid: Tuple[int, int, int]               # video latent grid T x H x W
    n_text: int = 0                          # text tokens placed before the video tokens
    n_action: int = 0                        # action tokens placed at the end of the joint sequence
    n_audio: int = 0                         # audio (sound) tokens placed after the video tokens, before the action tokens
    n_branches: int = 1                      # weight sets (1 = shared, 2 = text / generator, 3 = + action, 4 = + audio)
    mrope_sections: Tuple[int, int, int] = (32, 48, 48)   # channels per axis (t, h, w), sum = head_dim
    rope_base: float = 10000.0
    rope_layout: str = "chunked"
    eps: float = 1e-6
    fp8: bool = False
    qk_norm: bool = False                    # per-head RMSNorm of Q and K ahead of the rotation
    hybrid_mask: bool = False                # text run causal and blind to the generator tokens (else full attention)
    n_kv_heads: Optional[int] = None         # K / V heads (None = n_heads; fewer = grouped-query attention)
    residual_fp32: bool = True               # residual stream of a stack kept in fp32 between blocks (else bf16)
    seed: int = 1234

    @property
    def kv_heads(self) -> int:
        return self.n_heads if self.n_kv_heads is None else self.n_kv_heads

    @property
    def n_video(self) -> int:
        return self.grid[0] * self.grid[1] * self.grid[2]

    @property
    def n_tokens(self) -> int:
        return self.n_text + self.n_video + self.n_audio + self.n_action

    def gemm_flops_per_block(self) -> float:
        n, d, h = self.n_tokens, self.d_model, self.hidden
        d_kv = self.kv_heads * self.head_dim          # = d unless K / V heads are grouped
        return 2.0 * n * d * (2 * d + 2 * d_kv) + 6.0 * n * d * h

    def attn_flops_per_block(self) -> float:
        return 4.0 * float(self.n_tokens) ** 2 * self.d_model


CONFIGS = {
    "C0": DMConfig("C0", 1024, 16, 64, 4096, 1, (4, 16, 16), mrope_sections=(16, 24, 24), seed=1234),
    "C1": DMConfig("C1", 4096, 32, 128, 16384, 0, (16, 44, 80), seed=1235),
    "C2": DMConfig("C2", 4096, 32, 128, 16384, 28, (16, 44, 80), n_text=512, seed=1236),
    "C3": DMConfig("C3", 4096, 32, 128, 16384, 8, (8, 44, 80), n_text=1024, n_action=256, n_branches=3, seed=1237),
    "C4": DMConfig("C4", 4096, 32, 128, 16384, 28, (16, 44, 80), n_text=512, fp8=True, seed=1238),
}
