"""Pins oracle/unipc.py by what the mathematics fixes: closed form of the first-order step, exactness of the
solved-coefficient updates on polynomial data predictions (against quadrature of the exact solution), error order of
the shortcut updates, and convergence order of the whole sampler on a linear ODE with known solution."""
import math

import numpy as np
import pytest

from oracle import unipc as U


def lam(s):
    return math.log((1.0 - s) / s)


def exact_step(x_s, sig_s, sig_t, m_of_lam):
    """x_t = (sigma_t / sigma_s) x_s + sigma_t * int_{lam_s}^{lam_t} e^lam m(lam) dlam  (data-prediction ODE),
    by 60-point Gauss-Legendre quadrature (the integrand is entire: exact to rounding)."""
    a, b = lam(sig_s), lam(sig_t)
    t, w = np.polynomial.legendre.leggauss(60)
    ls = 0.5 * (b - a) * t + 0.5 * (b + a)
    integ = sum(wi * math.exp(li) * m_of_lam(li) for wi, li in zip(w, ls)) * 0.5 * (b - a)
    return (sig_t / sig_s) * x_s + sig_t * integ


def poly(coefs, l0):
    coefs = [np.asarray(c, dtype=np.float64) for c in coefs]
    return lambda l: sum(c * (l - l0) ** k for k, c in enumerate(coefs))


def test_first_order_step_is_the_euler_flow_step():
    rng = np.random.default_rng(0)
    x, v = rng.standard_normal(7), rng.standard_normal(7)
    for s0, s1 in [(0.9, 0.7), (0.5, 0.49), (0.3, 0.0), (1.0, 0.8)]:
        m = x - s0 * v
        got = U.unip_update(x, [m], [s0], s1, 1)
        assert np.allclose(got, x + (s1 - s0) * v, atol=1e-12), (s0, s1)
    smp = U.UniPCSampler(U.flow_sigmas(5, 3.0), solver_order=1, use_corrector=False)
    y = x.copy()
    for i in range(5):
        vi = rng.standard_normal(7)
        want = y + (smp.sigmas[i + 1] - smp.sigmas[i]) * vi
        y = smp.step(vi, y)
        assert np.allclose(y, want, atol=1e-12)


def test_step_that_starts_at_sigma_one_is_the_limit_of_steps_that_start_just_below():
    """A step from sigma = 1 has lambda = -inf and an infinite h; there both the oracle and the product's scheduler
    take B(h) = e^h - 1 -> -1 whatever the solver type (B(h) = h, "bh1", has no limit).  Pinned from the other side:
    the generic finite-h "bh2" code path at sigma_0 = 1 - eps must converge to the special case as eps -> 0, for
    the predictor and the corrector; the corrector of order 1 must equal its closed form
    sigma_t x + (1 - sigma_t) (m_0 + m_t) / 2; and a constant data prediction must be integrated exactly,
    x_t = sigma_t x + (1 - sigma_t) c.  "bh1" on that one step is therefore "bh2": a recorded deviation."""
    from cosmos_amd.sampler import _Update
    rng = np.random.default_rng(5)
    x, m0, mt = rng.standard_normal(6), rng.standard_normal(6), rng.standard_normal(6)
    st = 0.83
    at_one_p = U.unip_update(x, [m0], [1.0], st, 1)
    at_one_c = U.unic_update(x, [m0], [1.0], mt, st, 1)
    assert np.allclose(at_one_c, st * x + (1 - st) * 0.5 * (m0 + mt), atol=1e-13)
    assert np.allclose(U.unic_update(x, [m0], [1.0], m0, st, 1), st * x + (1 - st) * m0, atol=1e-13)
    for solver_type in ("bh1", "bh2"):
        assert np.allclose(U.unic_update(x, [m0], [1.0], mt, st, 1, solver_type), at_one_c, atol=1e-13)
    prev_p = prev_c = None
    for eps in (1e-3, 1e-5, 1e-7, 1e-9):
        s0 = 1.0 - eps
        dp = np.abs(U.unip_update(x, [m0], [s0], st, 1, "bh2") - at_one_p).max()
        dc = np.abs(U.unic_update(x, [m0], [s0], mt, st, 1, "bh2") - at_one_c).max()
        assert dp <= 20 * eps and dc <= 20 * eps, (eps, dp, dc)
        assert prev_p is None or (dp <= prev_p and dc <= prev_c)
        prev_p, prev_c = dp, dc
    # the product's scalar coefficients: same limit, predictor and corrector
    for corrector in (False, True):
        one = _Update(st, 1.0, [], corrector, "bh1")
        near = _Update(st, 1.0 - 1e-9, [], corrector, "bh2")
        for a, b in ((one.c_x, near.c_x), (one.c_m0, near.c_m0), (one.c_new, near.c_new)):
            assert abs(a - b) <= 1e-7, (corrector, a, b)
    u = _Update(st, 1.0, [], True, "bh1")
    assert abs(u.c_x - st) < 1e-15 and abs(u.c_m0 - 0.5 * (1 - st)) < 1e-15 and abs(u.c_new - 0.5 * (1 - st)) < 1e-15


@pytest.mark.parametrize("solver_type", ["bh1", "bh2"])
def test_solved_updates_are_exact_on_polynomial_data_predictions(solver_type):
    rng = np.random.default_rng(1)
    sig = [0.82, 0.71, 0.55, 0.43]            # three history levels and the target
    l0 = lam(sig[2])
    x_s = rng.standard_normal(5)
    # corrector of order 3: history at sig[0..2] and the new evaluation at sig[3]; exact up to degree 3
    m3 = poly([rng.standard_normal(5) for _ in range(4)], l0)
    got = U.unic_update(x_s, [m3(lam(s)) for s in sig[:3]], sig[:3], m3(lam(sig[3])), sig[3], 3, solver_type)
    assert np.allclose(got, exact_step(x_s, sig[2], sig[3], m3), atol=1e-11)
    # corrector of order 2: exact up to degree 2, and NOT for degree 3
    m2 = poly([rng.standard_normal(5) for _ in range(3)], l0)
    got = U.unic_update(x_s, [m2(lam(s)) for s in sig[1:3]], sig[1:3], m2(lam(sig[3])), sig[3], 2, solver_type)
    assert np.allclose(got, exact_step(x_s, sig[2], sig[3], m2), atol=1e-11)
    got = U.unic_update(x_s, [m3(lam(s)) for s in sig[1:3]], sig[1:3], m3(lam(sig[3])), sig[3], 2, solver_type)
    assert np.abs(got - exact_step(x_s, sig[2], sig[3], m3)).max() > 1e-6
    # predictor of order 3 (two solved coefficients): exact up to degree 2
    got = U.unip_update(x_s, [m2(lam(s)) for s in sig[:3]], sig[:3], sig[3], 3, solver_type)
    assert np.allclose(got, exact_step(x_s, sig[2], sig[3], m2), atol=1e-11)
    # every order is exact for a constant data prediction
    m0 = poly([rng.standard_normal(5)], l0)
    for order in (1, 2, 3):
        hist = [m0(0.0)] * order
        assert np.allclose(U.unip_update(x_s, hist, sig[3 - order:3], sig[3], order, solver_type),
                           exact_step(x_s, sig[2], sig[3], m0), atol=1e-12)
        assert np.allclose(U.unic_update(x_s, hist, sig[3 - order:3], m0(0.0), sig[3], order, solver_type),
                           exact_step(x_s, sig[2], sig[3], m0), atol=1e-12)


def test_shortcut_updates_have_third_order_local_error():
    """Predictor of order 2 and corrector of order 1 use rho = 1/2 instead of the solved value: exact only in the
    limit, with a local error that falls eightfold when the step in lambda halves."""
    rng = np.random.default_rng(2)
    c = [rng.standard_normal(3) for _ in range(2)]
    x_s = rng.standard_normal(3)

    def errs(h):
        l1 = 0.3
        ls = [l1 - h, l1, l1 + h]
        sg = [1.0 / (1.0 + math.exp(l)) for l in ls]          # sigma of lambda
        m = poly(c, l1)
        ex = exact_step(x_s, sg[1], sg[2], m)
        p2 = U.unip_update(x_s, [m(ls[0]), m(ls[1])], sg[:2], sg[2], 2)
        c1 = U.unic_update(x_s, [m(ls[1])], sg[1:2], m(ls[2]), sg[2], 1)
        return np.abs(p2 - ex).max(), np.abs(c1 - ex).max()

    (p_a, c_a), (p_b, c_b) = errs(0.2), errs(0.1)
    assert 6.0 < p_a / p_b < 10.5 and 6.0 < c_a / c_b < 10.5


def gaussian_flow(mu, s):
    """Velocity field and exact probability-flow solution for data ~ N(mu, s^2) under x_sigma = (1 - sigma) x0 +
    sigma eps:  x(sigma) = (1 - sigma) mu + sqrt((1 - sigma)^2 s^2 + sigma^2) z."""
    def v(x, sg):
        var = (1 - sg) ** 2 * s * s + sg * sg
        d = x - (1 - sg) * mu
        return sg / var * d - (mu + (1 - sg) * s * s / var * d)
    sol = lambda z, sg: (1 - sg) * mu + math.sqrt((1 - sg) ** 2 * s * s + sg * sg) * z
    return v, sol


def run(sigmas, v, sol, z, **kw):
    smp = U.UniPCSampler(sigmas, **kw)
    x = sol(z, smp.sigmas[0])
    for i in range(smp.n_steps):
        x = smp.step(v(x, smp.sigmas[i]), x)
    return np.abs(x - sol(z, smp.sigmas[-1])).max()


def test_sampler_convergence_orders():
    """On a grid uniform in lambda between two interior noise levels the global error falls as N^-p for the
    predictor of order p alone and as N^-(p+1) with the corrector - the defining property of the method."""
    v, sol = gaussian_flow(mu=1.5, s=0.4)
    z = np.array([-1.3, -0.2, 0.7, 2.1])

    def grid(n, s_a=0.9, s_b=0.2):
        la, lb = lam(s_a), lam(s_b)
        return [1.0 / (1.0 + math.exp(la + (lb - la) * i / n)) for i in range(n + 1)]

    def ratio(**kw):
        e = [run(grid(n), v, sol, z, lower_order_final=False, **kw) for n in (32, 64, 128)]
        return e[1] / e[2]

    assert 1.8 < ratio(solver_order=1, use_corrector=False) < 2.2          # order 1
    assert 3.5 < ratio(solver_order=1) < 4.5                               # order 2
    assert 3.7 < ratio(solver_order=2, use_corrector=False) < 5.2          # order 2
    assert 6.5 < ratio(solver_order=2) < 9.5                               # order 3
    assert 6.5 < ratio(solver_order=2, solver_type="bh1") < 9.5
    assert 13.0 < ratio(solver_order=3) < 28.0                             # order 4


@pytest.mark.parametrize("shift", [1.0, 3.0])
@pytest.mark.parametrize("grid", [U.flow_sigmas, U.diffusers_flow_sigmas])
def test_full_schedule_is_finite_and_beats_euler(shift, grid):
    """From pure noise to sigma = 0 (first level at lambda = -inf for the plain grid, last step with infinite h): every
    order stays finite, and the second- and third-order samplers are far more accurate than Euler at 80 steps."""
    v, sol = gaussian_flow(mu=1.5, s=0.4)
    z = np.array([-1.3, -0.2, 0.7, 2.1])
    e1 = run(grid(80, shift), v, sol, z, solver_order=1, use_corrector=False)
    e2 = run(grid(80, shift), v, sol, z, solver_order=2)
    e3 = run(grid(80, shift), v, sol, z, solver_order=3)
    assert all(np.isfinite(e) for e in (e1, e2, e3))
    assert e2 < e1 / 8 and e3 < e1 / 8
    # B(h) = h: a grid that starts at sigma = 1 has an infinite first step, which takes the e^h - 1 form
    for order in (1, 2, 3):
        eb = run(grid(80, shift), v, sol, z, solver_order=order, solver_type="bh1")
        assert np.isfinite(eb) and eb < e1 / 2, (order, eb, e1)


def test_diffusers_style_grid_shape():
    s = U.diffusers_flow_sigmas(10, 3.0)
    assert len(s) == 11 and s[-1] == 0.0 and all(a > b for a, b in zip(s, s[1:]))
    assert abs(s[0] - 3.0 * 0.999 / (1 + 2.0 * 0.999)) < 1e-12
