"""Host side of the elementwise step around the transformer forward: noise levels and the fused
guidance-combine + latent update (``ops.cfg_step``).

The reference configures a flow-shifted multistep scheduler and a guidance scale at its call site
(``UniPCMultistepScheduler.from_config(..., flow_shift=...)``, ``guidance_scale=...``; README.md:247,258).  Any such
scheduler reduces, per step, to scalar coefficients of a linear combination of the latents, the current guided
prediction and earlier predictions.  ``FlowEulerStepper`` supplies the first-order (Euler) coefficients;
``UniPCStepper`` the coefficients of the UniPC predictor-corrector (Zhao et al. 2023, data-prediction form) of order
1..3.  In both, all tensor work of a step is ONE launch of the fused kernel.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence

import numpy as np
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


def _lam(sigma: float) -> float:
    """Half log-SNR of a flow-matching noise level: log((1 - sigma) / sigma); +-inf at the ends."""
    if sigma <= 0.0:
        return math.inf
    if sigma >= 1.0:
        return -math.inf
    return math.log(1.0 - sigma) - math.log(sigma)


class _Update:
    """Scalar coefficients of one UniPC update from noise level ``s0`` to ``st``:
        x_t = c_x * x_s0 + c_m0 * m0 + sum_k c_old[k] * m_{-1-k} (+ c_new * m_t for the corrector)
    with m0 the data prediction at s0, m_{-1-k} the one k+1 steps before it and m_t the one at st."""

    def __init__(self, st: float, s0: float, older: Sequence[float], corrector: bool, solver_type: str):
        order = len(older) + 1
        alpha_t = 1.0 - st
        lam_s0 = _lam(s0)
        h = _lam(st) - lam_s0
        hh = -h
        h_phi_1 = math.expm1(hh)
        finite = math.isfinite(hh)
        # B(h) = h ("bh1") has no limit when the step starts at sigma = 1 (lambda = -inf, h infinite), while
        # e^h - 1 ("bh2") tends to -1; both variants agree to first order in h, so that step takes the bh2 form
        B_h = h_phi_1 if (solver_type == "bh2" or not finite) else hh
        # divided-difference abscissae of the older predictions (an abscissa at -inf switches its term off)
        rks = [(_lam(sg) - lam_s0) / h if finite else 0.0 for sg in older] + [1.0]
        inv_rk = [0.0 if (rk == 0.0 or math.isinf(rk)) else 1.0 / rk for rk in rks[:-1]]
        # right-hand sides b_i = hh phi_{i+1}(hh) i! / B(h)
        b, fact = [], 1.0
        h_phi_k = h_phi_1 / hh - 1.0 if finite else -1.0
        for i in range(1, order + 1):
            b.append(h_phi_k * fact / B_h)
            fact *= i + 1
            h_phi_k = h_phi_k / hh - 1.0 / fact if finite else -1.0 / fact
        if corrector:
            if order == 1:
                rhos = [0.5]
            else:
                R = np.array([[rk ** (i - 1) for rk in rks] for i in range(1, order + 1)], dtype=np.float64)
                rhos = list(np.linalg.solve(R, np.array(b, dtype=np.float64)))
        else:
            if order == 1:
                rhos = []
            elif order == 2:
                rhos = [0.5]
            else:
                R = np.array([[rk ** (i - 1) for rk in rks[:-1]] for i in range(1, order)], dtype=np.float64)
                rhos = list(np.linalg.solve(R, np.array(b[:-1], dtype=np.float64)))
            rhos = rhos + [0.0]            # no term for a prediction at st
        self.c_x = st / s0
        self.c_old = [-alpha_t * B_h * r * ir for r, ir in zip(rhos[:-1], inv_rk)]
        self.c_new = -alpha_t * B_h * rhos[-1] if corrector else 0.0
        self.c_m0 = -alpha_t * h_phi_1 - sum(self.c_old) - self.c_new


class UniPCStepper:
    """``scheduler.step``-shaped UniPC sampler for flow-matching noise levels (alpha = 1 - sigma; the data
    prediction of a velocity output v at latents x is x - sigma v).  Per step: the corrector refines the current
    latents with the new evaluation (from the second step on; it needs no extra model call), then the predictor of
    order ``this_order`` (warm-up from 1, lowered at the final steps) moves them to the next noise level.

    Both updates are linear in the tensors at hand - current latents, guided prediction, previous corrected latents
    and the kept data predictions - so ``step`` folds them into three coefficient rows and makes ONE pass on the GPU
    (``ops.cfg_multistep``): next latents (in place), corrected latents, data prediction.  Keeps
    ``solver_order`` + 1 fp32 tensors of the latents' size."""

    def __init__(self, sigmas: Sequence[float], guidance_scale: float = 1.0, solver_order: int = 2,
                 solver_type: str = "bh2", lower_order_final: bool = True, use_corrector: bool = True):
        if not 1 <= solver_order <= 3:
            raise ValueError("solver_order must be 1, 2 or 3")
        if solver_type not in ("bh1", "bh2"):
            raise ValueError("solver_type must be 'bh1' or 'bh2'")
        self.sigmas = [float(s) for s in sigmas]
        if len(self.sigmas) < 2 or any(a <= b for a, b in zip(self.sigmas, self.sigmas[1:])) or self.sigmas[-1] < 0 \
                or self.sigmas[0] > 1:
            raise ValueError("sigmas must decrease strictly within [1, 0]")
        self.timesteps = [1000.0 * s for s in self.sigmas[:-1]]
        self.guidance_scale, self.solver_order, self.solver_type = guidance_scale, solver_order, solver_type
        self.lower_order_final, self.use_corrector = lower_order_final, use_corrector
        self.m_hist: List[torch.Tensor] = []        # data predictions, newest last
        self.sig_hist: List[float] = []
        self.last_sample: Optional[torch.Tensor] = None
        self._spare: List[torch.Tensor] = []
        self.lower_order_nums, self.this_order, self.index = 0, 1, 0

    @classmethod
    def from_flow_shift(cls, num_steps: int, flow_shift: float = 1.0, **kw) -> "UniPCStepper":
        return cls(flow_sigmas(num_steps, flow_shift), **kw)

    def step(self, v_cond: torch.Tensor, v_uncond: Optional[torch.Tensor], sample: torch.Tensor) -> torch.Tensor:
        """``sample`` (fp32, updated in place and returned): latents at ``sigmas[index]``; ``v_cond`` / ``v_uncond``
        (bf16): the transformer's velocity predictions there."""
        i = self.index
        n_steps = len(self.sigmas) - 1
        if i >= n_steps:
            raise RuntimeError("all steps have been taken")
        sigma, sigma_next = self.sigmas[i], self.sigmas[i + 1]
        olds = list(reversed(self.m_hist))                     # m_{i-1}, m_{i-2}, ...
        old_sig = list(reversed(self.sig_hist))
        n_old = len(olds)
        width = 3 + n_old                                       # basis: x, v, last_sample, m_{i-1}, m_{i-2}, ...
        e = lambda k, c=1.0: [c if j == k else 0.0 for j in range(width)]
        add = lambda a, b, cb=1.0: [p + cb * q for p, q in zip(a, b)]
        m_row = add(e(0), e(1), -sigma)                         # m_i = x - sigma v
        corrected = self.use_corrector and i > 0 and self.last_sample is not None
        if corrected:
            u = _Update(sigma, old_sig[0], old_sig[1:self.this_order], True, self.solver_type)
            xc_row = add(e(2, u.c_x), e(3, u.c_m0))
            for k, c in enumerate(u.c_old):
                xc_row = add(xc_row, e(4 + k, c))
            xc_row = add(xc_row, m_row, u.c_new)
        else:
            xc_row = e(0)
        order = min(self.solver_order, n_steps - i) if self.lower_order_final else self.solver_order
        order = min(order, self.lower_order_nums + 1)
        # a kept level at sigma = 1 (lambda = -inf) cannot enter the solved coefficients of order 3
        while order > 2 and any(sg >= 1.0 for sg in old_sig[:order - 1]):
            order -= 1
        if sigma_next <= 0.0:
            order = 1                                           # the step to sigma = 0 returns the data prediction
        self.this_order = order
        u = _Update(sigma_next, sigma, old_sig[:order - 1], False, self.solver_type)
        nx_row = add([u.c_x * c for c in xc_row], m_row, u.c_m0)
        for k, c in enumerate(u.c_old):
            nx_row = add(nx_row, e(3 + k, c))
        # tensors: inputs (a dummy for the slots that do not exist yet - their coefficients are zero)
        fill = sample
        hist = [self.last_sample if self.last_sample is not None else fill] + olds
        m_new = self._spare.pop() if self._spare else torch.empty_like(sample)
        if self.last_sample is None:
            self.last_sample = torch.empty_like(sample)
        rows = [[r[0], r[1]] + r[2:] for r in (nx_row, m_row, xc_row)]
        ops.cfg_multistep(sample, v_cond, v_uncond, self.guidance_scale, rows, hist, [sample, m_new, self.last_sample])
        self.m_hist.append(m_new)
        self.sig_hist.append(sigma)
        if len(self.m_hist) > self.solver_order:
            self._spare.append(self.m_hist.pop(0))
            self.sig_hist.pop(0)
        if self.lower_order_nums < self.solver_order:
            self.lower_order_nums += 1
        self.index += 1
        return sample
