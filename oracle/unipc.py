"""CPU restatement of the UniPC multistep sampler for flow-matching noise levels (TEST INFRASTRUCTURE ONLY).

The reference selects this sampler at its call site, ``UniPCMultistepScheduler.from_config(..., flow_shift=...)``
(README.md:247) and drives it through the diffusers pipeline (README.md:249-263).  The scheduler's code lives in
``diffusers`` (git main, unpinned; not installed here and absent from the reference), so this file restates the
PUBLISHED algorithm: Zhao et al., "UniPC: A Unified Predictor-Corrector Framework for Fast Sampling of Diffusion
Models" (2023), data-prediction form, B(h) = e^h - 1 ("bh2") or h ("bh1"), with the usual multistep conventions of
its public implementations: order warm-up from 1, lower order at the final steps, corrector from the second step on
(it re-uses the model evaluation of the step, so it costs nothing extra), and the order-1 / order-2 shortcuts
rho = 1/2.  For flow matching alpha = 1 - sigma, lambda = log(alpha / sigma), and the data prediction of a velocity
output v at latents x is x - sigma v.

Pinning (tests/test_oracle_unipc.py): order 1 without corrector is the Euler flow step in closed form; the
solved-coefficient updates (corrector of order 2 and 3, predictor of order 3) are EXACT when the data prediction is a
polynomial in lambda of matching degree, which is checked against numerical quadrature of the exact solution
x_t = (sigma_t / sigma_s) x_s + sigma_t * int e^lambda x0(lambda) dlambda; the shortcut updates are checked for their
error order; the whole sampler for its convergence order on a linear ODE with known solution.
PARITY UNPINNED against diffusers' UniPCMultistepScheduler itself: its defaults (solver_order, the noise-level
grid of ``diffusers_flow_sigmas``, final-step handling) are restated from its public documentation, not executed.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence

import numpy as np


def flow_sigmas(num_steps: int, flow_shift: float = 1.0) -> List[float]:
    """Noise levels 1 -> 0 with the time shift sigma' = shift sigma / (1 + (shift - 1) sigma)."""
    out = []
    for i in range(num_steps + 1):
        s = 1.0 - i / num_steps
        out.append(flow_shift * s / (1.0 + (flow_shift - 1.0) * s))
    return out


def diffusers_flow_sigmas(num_steps: int, flow_shift: float = 1.0, num_train_timesteps: int = 1000) -> List[float]:
    """The grid the public UniPC implementation documents for ``use_flow_sigmas``: 1 - linspace(1, 1/T, n+1), shifted,
    reversed, without its zero, and a final 0 appended (starts at shift(1 - 1/T), not at 1).  Unpinned."""
    al = np.linspace(1.0, 1.0 / num_train_timesteps, num_steps + 1)
    s = 1.0 - al
    s = flow_shift * s / (1.0 + (flow_shift - 1.0) * s)
    return list(s[::-1][:-1]) + [0.0]


def _lam(sigma: float) -> float:
    a = 1.0 - sigma
    if sigma <= 0.0:
        return math.inf
    if a <= 0.0:
        return -math.inf
    return math.log(a) - math.log(sigma)


def _rhos(rks: Sequence[float], hh: float, B_h: float):
    """Right-hand sides b_i = hh phi_{i+1}(hh) i! / B(h) and the Vandermonde matrix R_ij = rk_j^(i-1)."""
    h_phi_1 = math.expm1(hh)
    h_phi_k = h_phi_1 / hh - 1.0 if math.isfinite(hh) else -1.0
    fact = 1.0
    R, b = [], []
    for i in range(1, len(rks) + 1):
        R.append([rk ** (i - 1) for rk in rks])
        b.append(h_phi_k * fact / B_h)
        fact *= i + 1
        h_phi_k = h_phi_k / hh - 1.0 / fact if math.isfinite(hh) else -1.0 / fact
    return np.array(R, dtype=np.float64), np.array(b, dtype=np.float64)


def unip_update(x, m_hist: Sequence, sig_hist: Sequence[float], sigma_t: float, order: int, solver_type: str = "bh2"):
    """Predictor.  x: latents at sig_hist[-1]; m_hist[-1-i] / sig_hist[-1-i]: data prediction and noise level i steps
    back (i = 0 .. order-1).  Returns the latents at sigma_t."""
    s0 = sig_hist[-1]
    m0 = m_hist[-1]
    alpha_t = 1.0 - sigma_t
    lam_t, lam_s0 = _lam(sigma_t), _lam(s0)
    h = lam_t - lam_s0
    hh = -h
    h_phi_1 = math.expm1(hh)
    # a step that starts at sigma = 1 has infinite h: B(h) = h ("bh1") has no limit there, e^h - 1 ("bh2") tends to -1
    B_h = math.expm1(hh) if (solver_type == "bh2" or not math.isfinite(hh)) else hh
    rks, D1s = [], []
    for i in range(1, order):
        rk = (_lam(sig_hist[-1 - i]) - lam_s0) / h
        rks.append(rk)
        D1s.append((m_hist[-1 - i] - m0) / rk)
    rks.append(1.0)
    R, b = _rhos(rks, hh, B_h)
    x_t = (sigma_t / s0) * x - alpha_t * h_phi_1 * m0
    if D1s:
        rhos = np.array([0.5]) if order == 2 else np.linalg.solve(R[:-1, :-1], b[:-1])
        res = sum(r * d for r, d in zip(rhos, D1s))
        x_t = x_t - alpha_t * B_h * res
    return x_t


def unic_update(x_last, m_hist: Sequence, sig_hist: Sequence[float], m_t, sigma_t: float, order: int,
                solver_type: str = "bh2"):
    """Corrector.  x_last: the latents the previous predictor started from (noise level sig_hist[-1]); m_hist /
    sig_hist as in unip_update (history up to that step); m_t: data prediction at sigma_t, taken at the PREDICTED
    latents.  Returns the corrected latents at sigma_t."""
    s0 = sig_hist[-1]
    m0 = m_hist[-1]
    alpha_t = 1.0 - sigma_t
    lam_t, lam_s0 = _lam(sigma_t), _lam(s0)
    h = lam_t - lam_s0
    hh = -h
    h_phi_1 = math.expm1(hh)
    # a step that starts at sigma = 1 has infinite h: B(h) = h ("bh1") has no limit there, e^h - 1 ("bh2") tends to -1
    B_h = math.expm1(hh) if (solver_type == "bh2" or not math.isfinite(hh)) else hh
    rks, D1s = [], []
    for i in range(1, order):
        rk = (_lam(sig_hist[-1 - i]) - lam_s0) / h
        rks.append(rk)
        D1s.append((m_hist[-1 - i] - m0) / rk)
    rks.append(1.0)
    R, b = _rhos(rks, hh, B_h)
    rhos = np.array([0.5]) if order == 1 else np.linalg.solve(R, b)
    x_t = (sigma_t / s0) * x_last - alpha_t * h_phi_1 * m0
    res = sum(r * d for r, d in zip(rhos[:-1], D1s)) if D1s else 0.0
    return x_t - alpha_t * B_h * (res + rhos[-1] * (m_t - m0))


class UniPCSampler:
    """``scheduler.step``-shaped driver of the two updates above (float64 arrays)."""

    def __init__(self, sigmas: Sequence[float], solver_order: int = 2, solver_type: str = "bh2",
                 lower_order_final: bool = True, use_corrector: bool = True):
        self.sigmas = [float(s) for s in sigmas]
        self.n_steps = len(self.sigmas) - 1
        self.solver_order, self.solver_type = solver_order, solver_type
        self.lower_order_final, self.use_corrector = lower_order_final, use_corrector
        self.m_hist: List[np.ndarray] = []
        self.sig_hist: List[float] = []
        self.last_sample: Optional[np.ndarray] = None
        self.lower_order_nums = 0
        self.this_order = 1
        self.index = 0

    def step(self, v, sample):
        """v: the model's (guided) velocity at (sample, sigmas[index]).  Returns the latents at sigmas[index + 1]."""
        i = self.index
        sigma = self.sigmas[i]
        sample = np.asarray(sample, dtype=np.float64)
        m = sample - sigma * np.asarray(v, dtype=np.float64)            # data prediction at the uncorrected latents
        if self.use_corrector and i > 0 and self.last_sample is not None:
            sample = unic_update(self.last_sample, self.m_hist, self.sig_hist, m, sigma, self.this_order, self.solver_type)
        self.m_hist = (self.m_hist + [m])[-self.solver_order:]
        self.sig_hist = (self.sig_hist + [sigma])[-self.solver_order:]
        order = min(self.solver_order, self.n_steps - i) if self.lower_order_final else self.solver_order
        order = min(order, self.lower_order_nums + 1)
        # a history level at sigma = 1 has lambda = -inf: its divided difference vanishes (harmless with the order-2
        # shortcut) but the solved coefficients of higher orders are undefined, so such a level caps the order at 2
        while order > 2 and any(sg >= 1.0 for sg in self.sig_hist[-order:-1]):
            order -= 1
        self.this_order = order
        self.last_sample = sample
        nxt = unip_update(sample, self.m_hist, self.sig_hist, self.sigmas[i + 1], self.this_order, self.solver_type)
        if self.lower_order_nums < self.solver_order:
            self.lower_order_nums += 1
        self.index += 1
        return nxt
