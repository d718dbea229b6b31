"""GPU parity of the fused guidance-combine + scheduler update against the oracle."""
import pytest
import torch

import oracle as O
from cosmos_amd import ops
from cosmos_amd.sampler import FlowEulerStepper, flow_sigmas
from gpu_util import dev, rand_bf16

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,n_hist,guided", [(4096, 0, True), (1003, 2, True), (3604480, 4, True), (517, 1, False), (3, 0, True)])
def test_cfg_step_vs_oracle(n, n_hist, guided):
    g = torch.Generator().manual_seed(n + n_hist)
    x = torch.randn(n, generator=g)
    vc, vcr = rand_bf16((n,), g)
    vu, vur = rand_bf16((n,), g)
    hist = [torch.randn(n, generator=g) for _ in range(n_hist)]
    coef = [0.9, -0.37] + [0.1 * (i + 1) for i in range(n_hist)]
    v_out = torch.empty(n, device=dev())
    out = ops.cfg_step(x.to(dev()), vc, vu if guided else None, 6.0, coef, [h.to(dev()) for h in hist], v_out=v_out)
    want, v = O.cfg_step(x, vcr, vur if guided else None, 6.0, coef, hist)
    # fp32 arithmetic on both sides; only the order of the additions may differ
    assert torch.allclose(out.cpu(), want, rtol=1e-5, atol=1e-5)
    assert torch.allclose(v_out.cpu(), v, rtol=1e-6, atol=1e-6)


def test_cfg_step_closed_forms_and_in_place():
    g = torch.Generator().manual_seed(3)
    n = 2048
    x = torch.randn(n, generator=g).to(dev())
    vc, vcr = rand_bf16((n,), g)
    vu, vur = rand_bf16((n,), g)
    assert torch.equal(ops.cfg_step(x, vc, vu, 1.0, [0.0, 1.0]).cpu(), vur + 1.0 * (vcr - vur))   # guidance 1 -> cond (same fp32 ops)
    assert torch.equal(ops.cfg_step(x, vc, vu, 0.0, [0.0, 1.0]).cpu(), vur)                        # guidance 0 -> uncond
    assert torch.equal(ops.cfg_step(x, vc, None, 7.0, [1.0, 0.0]).cpu(), x.cpu())                  # identity
    a, b = ops.cfg_step(x, vc, vu, 3.0, [1.0, 0.5]), ops.cfg_step(x, vc, vu, 3.0, [2.0, 1.0])
    assert torch.allclose(2 * a, b, rtol=1e-6, atol=1e-6)                                          # linear in coef
    y = x.clone()
    ops.cfg_step(y, vc, vu, 3.0, [1.0, 0.5], out=y)
    assert torch.equal(y, a)


def test_flow_euler_stepper_matches_oracle_schedule():
    steps, shift = 8, 3.0
    assert torch.allclose(torch.tensor(flow_sigmas(steps, shift), dtype=torch.float64), O.flow_sigmas(steps, shift))
    g = torch.Generator().manual_seed(8)
    n = 4096
    x0 = torch.randn(n, generator=g)
    st = FlowEulerStepper(steps, flow_shift=shift, guidance_scale=4.0, keep_history=1)
    x = x0.clone().to(dev())
    xr = x0.clone()
    sig = O.flow_sigmas(steps, shift)
    for i in range(steps):
        vc, vcr = rand_bf16((n,), g)
        vu, vur = rand_bf16((n,), g)
        x = st.step(vc, vu, x)
        xr, v = O.cfg_step(xr, vcr, vur, 4.0, [1.0, float(sig[i + 1] - sig[i])])
        assert torch.allclose(st.history[0].cpu(), v, rtol=1e-6, atol=1e-6)
    assert torch.allclose(x.cpu(), xr, rtol=1e-4, atol=1e-4)
    with pytest.raises(RuntimeError):
        st.step(vc, vu, x)
