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


@pytest.mark.parametrize("n_out,n_hist", [(1, 0), (2, 1), (3, 4), (3, 0)])
def test_cfg_multistep_rows_and_aliasing(n_out, n_hist):
    """Several linear combinations in one pass; outputs written over the latents and over a history tensor."""
    g = torch.Generator().manual_seed(10 * n_out + n_hist)
    n = 70001
    x = torch.randn(n, generator=g)
    vc, vcr = rand_bf16((n,), g)
    vu, vur = rand_bf16((n,), g)
    hist = [torch.randn(n, generator=g) for _ in range(n_hist)]
    rows = [[float(c) for c in torch.randn(2 + n_hist, generator=g)] for _ in range(n_out)]
    xd, hd = x.to(dev()), [h.to(dev()) for h in hist]
    outs = [xd] + ([hd[-1]] if n_hist and n_out > 1 else [torch.empty(n, device=dev())] if n_out > 1 else []) + \
           ([torch.empty(n, device=dev())] if n_out > 2 else [])
    ops.cfg_multistep(xd, vc, vu, 2.5, rows, hd, outs)
    for r, o in zip(rows, outs):
        want, _ = O.cfg_step(x, vcr, vur, 2.5, r, hist)
        assert torch.allclose(o.cpu(), want, rtol=1e-5, atol=2e-5)
    with pytest.raises(RuntimeError, match="coincide"):
        ops.cfg_multistep(xd, vc, vu, 2.5, [rows[0], rows[0]], hd, [xd, xd])


@pytest.mark.parametrize("order,corrector,solver_type,shift,grid", [
    (1, False, "bh2", 1.0, "plain"), (2, True, "bh2", 3.0, "plain"), (3, True, "bh2", 3.0, "plain"),
    (2, True, "bh1", 5.0, "library"), (3, True, "bh2", 1.0, "library"), (2, False, "bh2", 3.0, "library"),
    (2, True, "bh1", 3.0, "plain"), (3, True, "bh1", 10.0, "plain")])
def test_unipc_stepper_matches_oracle(order, corrector, solver_type, shift, grid):
    """The stepper's folded coefficient rows + one fused launch per step against the tensor-level float64 sampler,
    fed with the same random 'model outputs' (so any slip in the algebra shows at once)."""
    from cosmos_amd import UniPCStepper
    from oracle import unipc as U
    steps, n, guidance = 9, 5000, 4.0
    sig = U.flow_sigmas(steps, shift) if grid == "plain" else U.diffusers_flow_sigmas(steps, shift)
    st = UniPCStepper(sig, guidance_scale=guidance, solver_order=order, solver_type=solver_type, use_corrector=corrector)
    ref = U.UniPCSampler(sig, solver_order=order, solver_type=solver_type, use_corrector=corrector)
    g = torch.Generator().manual_seed(order * 7 + int(shift))
    x0 = torch.randn(n, generator=g)
    x, xr = x0.clone().to(dev()), x0.double().numpy()
    for i in range(steps):
        vc, vcr = rand_bf16((n,), g)
        vu, vur = rand_bf16((n,), g)
        x = st.step(vc, vu, x)
        v = (vur + guidance * (vcr - vur)).double().numpy()
        xr = ref.step(v, xr)
        assert st.this_order == ref.this_order
        assert bool(torch.isfinite(x).all()), f"step {i}: non-finite latents"
        err = float((x.double().cpu() - torch.from_numpy(xr)).abs().max())
        assert err < 2e-4 * max(1.0, float(abs(xr).max())), f"step {i}: {err}"
    with pytest.raises(RuntimeError):
        st.step(vc, vu, x)


def test_unipc_stepper_on_a_known_flow():
    """Whole sampling loop on the linear flow of a Gaussian (exact solution known): 20 steps of order 2 land within
    1e-2 of the exact sample, where Euler is off by more than 5e-2."""
    import math
    from cosmos_amd import UniPCStepper
    mu, s = 1.5, 0.4
    n = 4096
    z = torch.randn(n, generator=torch.Generator().manual_seed(2))

    def velocity(x, sg):
        var = (1 - sg) ** 2 * s * s + sg * sg
        d = x - (1 - sg) * mu
        return sg / var * d - (mu + (1 - sg) * s * s / var * d)

    def sample(stepper):
        x = z.clone().to(dev())
        for i in range(len(stepper.sigmas) - 1):
            v = velocity(x, stepper.sigmas[i]).to(torch.bfloat16)
            x = stepper.step(v, None, x)
        return float((x.cpu() - (mu + s * z)).abs().max())

    e2 = sample(UniPCStepper.from_flow_shift(20, 1.0, solver_order=2))
    e1 = sample(FlowEulerStepper(20, 1.0))
    assert e2 < 2e-2 and e1 > 5e-2


def test_denoising_loop_with_transformer_and_stepper():
    """The pieces either side of the block forward in one loop: DMTransformer forward (cond / uncond) -> UniPCStepper.
    Checked: the loop is finite and repeatable bit for bit, the batched form (cond and uncond as a batch of two) gives
    the same latents, and one Euler step equals x + (sigma' - sigma)(v_u + g (v_c - v_u)) on the model's own outputs."""
    from cosmos_amd import DMTransformer, UniPCStepper
    from cosmos_amd.config import DMConfig
    cfg = DMConfig("loop", 256, 2, 128, 512, 2, (2, 3, 4), n_text=12, n_branches=2, qk_norm=True)
    m = DMTransformer(cfg, latent_channels=4, device=dev())
    m.reset_parameters(9)
    g = torch.Generator(device=dev()).manual_seed(9)
    ctx = torch.randn((1, 12, 256), generator=g, device=dev()).to(torch.bfloat16)
    null = torch.zeros_like(ctx)
    lat0 = torch.randn((1, 4, 2, 6, 8), generator=g, device=dev())

    def run(batched):
        st = UniPCStepper(flow_sigmas(4, 10.0), guidance_scale=3.0, solver_order=2)     # flow_shift of the reference's call site
        lat = lat0.clone()
        for t in st.timesteps:
            ts = torch.tensor([t], device=dev())
            if batched:
                v, = m(torch.cat([lat, lat]), ts, encoder_hidden_states=torch.cat([ctx, null]))
                vc, vu = v[:1], v[1:]
            else:
                vc, = m(lat, ts, encoder_hidden_states=ctx)
                vu, = m(lat, ts, encoder_hidden_states=null)
            st.step(vc.contiguous(), vu.contiguous(), lat)
        return lat

    a, b, c = run(False), run(False), run(True)
    assert bool(torch.isfinite(a).all()) and torch.equal(a, b) and torch.equal(a, c)
    assert float((a - lat0).abs().max()) > 1e-3
    # one Euler step against the formula
    eu = FlowEulerStepper(4, 3.0, guidance_scale=3.0)
    ts = torch.tensor([eu.timesteps[0]], device=dev())
    vc, = m(lat0, ts, encoder_hidden_states=ctx)
    vu, = m(lat0, ts, encoder_hidden_states=null)
    x1 = eu.step(vc.contiguous(), vu.contiguous(), lat0.clone())
    want = lat0 + (eu.sigmas[1] - eu.sigmas[0]) * (vu.float() + 3.0 * (vc.float() - vu.float()))
    assert torch.allclose(x1, want, rtol=1e-5, atol=1e-5)


def test_denoising_loop_with_cached_text_context():
    """The loop of the integration notes under the hybrid mask: the text run's K/V (conditional and null prompt) are
    packed once and every step carries only the generator tokens; same latents as the loop that re-runs the text."""
    from cosmos_amd import DMTransformer, UniPCStepper
    from cosmos_amd.config import DMConfig
    cfg = DMConfig("loopc", 256, 2, 128, 512, 2, (2, 3, 4), n_text=64, n_branches=2, qk_norm=True, hybrid_mask=True)
    m = DMTransformer(cfg, latent_channels=4, device=dev())
    m.reset_parameters(11)
    g = torch.Generator(device=dev()).manual_seed(11)
    ctx = torch.randn((1, 64, 256), generator=g, device=dev()).to(torch.bfloat16)
    null = torch.zeros_like(ctx)
    lat0 = torch.randn((1, 4, 2, 6, 8), generator=g, device=dev())
    cache, null_cache = m.stack.precompute_context(ctx), m.stack.precompute_context(null)

    def run(cached):
        st = UniPCStepper(flow_sigmas(4, 10.0), guidance_scale=3.0, solver_order=2)
        lat = lat0.clone()
        for t in st.timesteps:
            ts = torch.tensor([t], device=dev())
            vc, = m(lat, ts, encoder_hidden_states=ctx, context_cache=cache if cached else None)
            vu, = m(lat, ts, encoder_hidden_states=null, context_cache=null_cache if cached else None)
            st.step(vc.contiguous(), vu.contiguous(), lat)
        return lat

    a, b = run(True), run(False)
    assert bool(torch.isfinite(a).all()) and float((a - lat0).abs().max()) > 1e-3
    assert float((a - b).abs().max()) <= 1e-2 * float(b.abs().max())
