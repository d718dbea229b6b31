"""Host side of the elementwise step around the transformer forward: noise levels and the fused
guidance-combine + latent update (``ops.cfg_step``).

The reference configures a flow-shifted multistep scheduler and a guidance scale at its call site
(``UniPCMultistepScheduler.from_config(..., flow_shift=...)``, ``guidance_scale=...``; README.md:247,258).  Any such
scheduler reduces, per step, to scalar coefficients of a linear combination of the latents, the current guided
prediction and earlier predictions; this module supplies the first-order (Euler) coefficients and the plumbing for
higher orders.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from . import ops


def flow_sigmas(num_steps: int, flow_shift: float = 1.0) -> List[float]:
    """Noise levels from 1 to 0 with the time shift sigma' = shift sigma / (1 + (shift - 1) sigma)."""
    out = []
    for i in range(num_steps + 1):
        s = 1.0 - i / num_steps
        out.append(flow_shift * s / (1.0 + (flow_shift - 1.0) * s))
    return out


class FlowEulerStepper:
    """``scheduler.step``-shaped helper: x <- x + (sigma_next - sigma) v with v the guided velocity prediction.

    ``step`` makes ONE pass over the tensors on the GPU; ``history`` keeps the last guided predictions (fp32) for
    callers that add their own multistep coefficients through ``extra_coef``."""

    def __init__(self, num_steps: int, flow_shift: float = 1.0, guidance_scale: float = 1.0, keep_history: int = 0):
        self.sigmas = flow_sigmas(num_steps, flow_shift)
        self.timesteps = [1000.0 * s for s in self.sigmas[:-1]]
        self.guidance_scale = guidance_scale
        self.keep_history = keep_history
        self.history: List[torch.Tensor] = []
        self.index = 0

    def step(self, v_cond: torch.Tensor, v_uncond: Optional[torch.Tensor], sample: torch.Tensor,
             extra_coef: Sequence[float] = ()) -> torch.Tensor:
        if self.index >= len(self.sigmas) - 1:
            raise RuntimeError("all steps have been taken")
        dt = self.sigmas[self.index + 1] - self.sigmas[self.index]
        hist = self.history[:len(extra_coef)]
        v_out = torch.empty_like(sample) if self.keep_history else None
        ops.cfg_step(sample, v_cond, v_uncond, self.guidance_scale, [1.0, dt, *extra_coef[:len(hist)]], hist,
                     v_out=v_out, out=sample)
        if v_out is not None:
            self.history = [v_out] + self.history[:self.keep_history - 1]
        self.index += 1
        return sample
