"""UniPC flow-matching sampler: the oracle (oracle/unipc_oracle.py) against what the mathematics fixes, and
the torch scheduler (longlive_amd/utils/unipc.py) against the oracle.  CPU only."""
import math

import numpy as np
import pytest
import torch
from scipy.integrate import quad

import unipc_oracle as uo
from longlive_amd.utils.unipc import FlowUniPCMultistepScheduler, convert_flow_pred_to_x0


def test_schedule_closed_form():
    sig, ts = uo.schedule(4, 1.0)
    assert np.allclose(sig, [0.999, 0.74925, 0.4995, 0.24975, 0.0], atol=1e-7) and list(ts) == [999, 749, 499, 249]
    assert list(uo.schedule(6, 1.0)[1]) == [999, 832, 666, 499, 333, 166]  # 666: sigma_max is float32(0.999) > 0.999
    sig5, ts5 = uo.schedule(4, 5.0)
    assert np.allclose(sig5[:-1], [5 * s / (1 + 4 * s) for s in sig[:-1]]) and sig5[-1] == 0.0
    sch = FlowUniPCMultistepScheduler(num_train_timesteps=1000, shift=1)
    sch.set_timesteps(4, shift=5.0)
    assert np.allclose(sch.sigmas.numpy(), sig5, atol=1e-7) and sch.timesteps.tolist() == list(ts5)


def test_phi_functions_and_weights():
    for z in (-3.0, -0.7, -1e-3, 0.4, 2.0):
        assert math.isclose(uo.phi(1, z), math.expm1(z) / z, rel_tol=1e-12)
        # phi_(k+1)(z) = integral_0^1 e^{(1 - t) z} t^k / k! dt
        for k in (1, 2, 3):
            ref = quad(lambda t: math.exp((1 - t) * z) * t ** k / math.factorial(k), 0, 1)[0]
            assert math.isclose(uo.phi(k + 1, z), ref, rel_tol=1e-9)


def _exact_solution(x_s, sigma_s, sigma_t, m_of_lambda):
    """x_t = (sigma_t / sigma_s) x_s + sigma_t * integral exp(lambda) m(lambda) d lambda (data prediction)."""
    ls, lt = uo.lam(sigma_s), uo.lam(sigma_t)
    integral = quad(lambda l: math.exp(l) * m_of_lambda(l), ls, lt, epsabs=1e-13, epsrel=1e-13)[0]
    return sigma_t / sigma_s * x_s + sigma_t * integral


def test_first_order_is_the_exponential_integrator():
    x_s, m = 0.37, -1.2
    for sigma_s, sigma_t in ((0.999, 0.75), (0.5, 0.25), (0.9, 0.1)):
        got = uo.uni_p(x_s, [m], [sigma_s], sigma_t, 1)
        h = uo.lam(sigma_t) - uo.lam(sigma_s)
        assert math.isclose(got, sigma_t / sigma_s * x_s - (1 - sigma_t) * math.expm1(-h) * m, rel_tol=1e-13)
        assert math.isclose(got, _exact_solution(x_s, sigma_s, sigma_t, lambda l: m), rel_tol=1e-10)
    assert uo.uni_p(x_s, [m], [0.25], 0.0, 1) == m  # the last step returns the x0 prediction


@pytest.mark.parametrize("coeffs", [(0.8, -0.5, 0.0), (0.3, 1.1, -0.7)])
def test_second_order_corrector_is_exact_for_quadratics_in_lambda(coeffs):
    """UniC-2 uses the previous node, the step's start and the predicted point: three nodes, exact up to
    degree 2.  A wrong R, b, phi recurrence or node position breaks this."""
    c0, c1, c2 = coeffs
    sigma_prev, sigma_s, sigma_t = 0.8, 0.6, 0.35
    ls = uo.lam(sigma_s)
    m = lambda l: c0 + c1 * (l - ls) + c2 * (l - ls) ** 2
    x_s = 0.21
    got = uo.uni_c(x_s, [m(uo.lam(sigma_prev)), m(ls)], [sigma_prev, sigma_s], sigma_t, m(uo.lam(sigma_t)), 2)
    assert math.isclose(got, _exact_solution(x_s, sigma_s, sigma_t, m), rel_tol=1e-9)
    # the order-1 corrector (fixed weight 1/2) is exact for constants only
    got1 = uo.uni_c(x_s, [m(ls)], [sigma_s], sigma_t, m(uo.lam(sigma_t)), 1)
    assert (abs(got1 - _exact_solution(x_s, sigma_s, sigma_t, m)) < 1e-9) == (c1 == 0 and c2 == 0)


def test_constant_x0_prediction_is_reproduced_by_every_step():
    rng = np.random.default_rng(0)
    x0, noise = rng.standard_normal(8), rng.standard_normal(8)
    sig, _ = uo.schedule(4, 5.0)
    x = (1 - sig[0]) * x0 + sig[0] * noise
    traj = uo.sample(lambda x, s, t: (x - x0) / s, x, 4, 5.0)  # flow = noise - x0 along the straight line
    for i, xi in enumerate(traj):
        assert np.allclose(xi, (1 - sig[i + 1]) * x0 + sig[i + 1] * noise, atol=1e-12)
    assert np.allclose(traj[-1], x0, atol=1e-12)


@pytest.mark.parametrize("steps,shift", [(4, 5.0), (6, 1.0), (3, 3.0), (1, 5.0)])
def test_torch_scheduler_follows_the_oracle(steps, shift):
    rng = np.random.default_rng(steps)
    A = rng.standard_normal((12, 12)) * 0.3
    flow_np = lambda x, s, t: np.tanh(x @ A) + 0.1 * s - 0.001 * (t % 7)
    x0 = rng.standard_normal((2, 12))
    want = uo.sample(flow_np, x0.copy(), steps, shift)
    sch = FlowUniPCMultistepScheduler(num_train_timesteps=1000, shift=1)
    sch.set_timesteps(steps, shift=shift)
    x = torch.from_numpy(x0).float()
    for i, t in enumerate(sch.timesteps):
        flow = torch.from_numpy(flow_np(x.double().numpy(), float(sch.sigmas[i]), int(t))).float()
        x = sch.step(flow, t, x, return_dict=False)[0]
        assert np.allclose(x.numpy(), want[i], atol=2e-5, rtol=2e-5), i
    assert sch.step_index == steps
    with pytest.raises(IndexError):
        fresh = FlowUniPCMultistepScheduler()
        fresh.set_timesteps(4)
        fresh.step(x, torch.tensor(123), x)


def test_scheduler_keeps_the_sample_dtype_and_rejects_unbuilt_modes():
    sch = FlowUniPCMultistepScheduler()
    sch.set_timesteps(4, shift=5.0)
    x = torch.randn(1, 3, 4, 4, generator=torch.Generator().manual_seed(0)).bfloat16()
    for t in sch.timesteps:
        x = sch.step(torch.randn_like(x), t, x).prev_sample
        assert x.dtype == torch.bfloat16 and torch.isfinite(x).all()
    with pytest.raises(NotImplementedError):
        FlowUniPCMultistepScheduler(solver_type="rk4")
    with pytest.raises(NotImplementedError):
        FlowUniPCMultistepScheduler(predict_x0=False)
    with pytest.raises(ValueError):
        FlowUniPCMultistepScheduler().step(x, 0, x)


def test_flow_to_x0_conversion():
    xt = torch.tensor([[1.0, -2.0]], dtype=torch.bfloat16)
    flow = torch.tensor([[0.5, 0.25]], dtype=torch.bfloat16)
    out = convert_flow_pred_to_x0(flow, xt, 0.75)
    assert out.dtype == torch.bfloat16 and torch.equal(out, torch.tensor([[0.625, -2.1875]]).bfloat16())


def _sigma_of(lmbda):
    return 1.0 / (1.0 + math.exp(lmbda))


@pytest.mark.parametrize("which", ["predictor_order_2", "corrector_order_1"])
def test_the_fixed_weight_one_half_is_what_makes_the_step_second_order(which):
    """The order-2 predictor and the order-1 corrector do not solve for their single weight; the reference
    writes 1/2 (wan_5b/utils/fm_solvers_unipc.py:461-463, 603-604).  What determines that number: with a
    difference of two x0 predictions as the only correction term, the local error of a step of size h in lambda
    falls like h^3 for the weight 1/2 and only like h^2 for any other.  Measured on an x0 prediction that is
    linear in lambda: halving h divides the error by ~8 for the oracle's step, and by ~4 when the correction
    term is rescaled to a weight of 0.45 or 0.55."""
    c0, c1, x_s, lam_s = 0.3, 0.9, 0.21, 0.4
    m = lambda l: c0 + c1 * (l - lam_s)

    def errors(h):
        s_prev, s_s, s_t = _sigma_of(lam_s - h), _sigma_of(lam_s), _sigma_of(lam_s + h)
        exact = _exact_solution(x_s, s_s, s_t, m)
        first_order = uo.uni_p(x_s, [m(lam_s)], [s_s], s_t, 1)
        if which == "predictor_order_2":
            step = uo.uni_p(x_s, [m(lam_s - h), m(lam_s)], [s_prev, s_s], s_t, 2)
        else:
            step = uo.uni_c(x_s, [m(lam_s)], [s_s], s_t, m(lam_s + h), 1)
        correction = step - first_order  # the term that carries the weight 1/2
        return {w: first_order + correction * (w / 0.5) - exact for w in (0.5, 0.45, 0.55)}

    coarse, fine = errors(0.2), errors(0.1)
    assert 6.5 < coarse[0.5] / fine[0.5] < 9.5, coarse[0.5] / fine[0.5]
    for w in (0.45, 0.55):
        assert 2.8 < coarse[w] / fine[w] < 5.5, (w, coarse[w] / fine[w])
        assert abs(fine[w]) > 5 * abs(fine[0.5])
