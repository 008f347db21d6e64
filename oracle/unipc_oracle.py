"""CPU restatement (numpy float64) of the flow-matching UniPC sampler the reference pipeline steps with
(wan_5b/utils/fm_solvers_unipc.py:162-229 schedule, :281-350 x0 conversion, :352-486 UniP, :488-628 UniC,
:657-741 step; configuration of pipeline/causal_diffusion_inference.py:892-900: order 2, "bh2",
lower_order_final, flow prediction in data-prediction form).

TEST INFRASTRUCTURE ONLY: used by tests/ as the checker of longlive_amd/utils/unipc.py, never by the product.

The reference module needs `diffusers`, which is not installed here, so it was read, not run.  What pins this
restatement (tests/test_unipc.py): the closed-form schedule for given (steps, shift); a constant x0 prediction
is reproduced exactly by every step; order 1 equals the exponential-integrator (DDIM) formula; the order-2
corrector is exact for x0 predictions that are polynomials of degree <= 2 in lambda (checked against numerical
quadrature of the exact solution), which fixes R, b and the phi recurrence; the last step returns the x0
prediction; the fixed weight 1/2 of the order-2 predictor and of the order-1 corrector (:461-463, :603-604)
is the only weight for which the local error of those steps falls like h^3 instead of h^2 (measured by halving h).

The weights are built from closed-form phi functions here, not from the reference's recurrence, so that the
two formulations check each other.
"""
import math

import numpy as np


def schedule(num_steps: int, shift: float = 1.0, num_train_timesteps: int = 1000):
    """(sigmas [n+1] with a final 0, integer timesteps [n]) of set_timesteps (:162-229)."""
    # The ends come from the constructor's training schedule, which is held in float32 (:108-133; its own
    # shift is 1 in the pipeline): sigma_max is the float32 neighbour of 0.999, and that decides which way
    # some integer timesteps truncate.
    alphas = np.linspace(1, 1 / num_train_timesteps, num_train_timesteps)[::-1]
    train = (1.0 - alphas).astype(np.float32)
    sigma_max, sigma_min = float(train[0]), float(train[-1])
    s = np.linspace(sigma_max, sigma_min, num_steps + 1)[:-1]
    s = shift * s / (1 + (shift - 1) * s)
    return np.concatenate([s, [0.0]]), (s * num_train_timesteps).astype(np.int64)


def lam(sigma):
    return math.log(1 - sigma) - math.log(sigma) if sigma > 0 else math.inf


def phi(k: int, z: float) -> float:
    """phi_k(z) = (e^z - sum_{j<k} z^j / j!) / z^k; a series for small |z| (the closed form cancels)."""
    if abs(z) < 0.5:
        return sum(z ** j / math.factorial(j + k) for j in range(30))
    if z == -math.inf:
        return 0.0
    return (math.exp(z) - sum(z ** j / math.factorial(j) for j in range(k))) / z ** k


def weights(order: int, rks, hh: float):
    """R [order, order] and b [order]: sum_i rho_i rks_i^(k-1) = k! hh phi_(k+1)(hh) / B(hh), B = expm1."""
    rks = np.asarray(rks, dtype=np.float64)
    B = math.expm1(hh)
    R = np.stack([rks ** (k - 1) for k in range(1, order + 1)])
    if hh == -math.inf:  # final step to sigma 0: hh phi_(k+1)(hh) -> -1/k! ... only order 1 reaches here
        b = np.array([(-1.0 / math.factorial(k)) * math.factorial(k) / B for k in range(1, order + 1)])
    else:
        b = np.array([math.factorial(k) * hh * phi(k + 1, hh) / B for k in range(1, order + 1)])
    return R, b, B


def _differences(ms, lambdas, lambda_s0, h, order):
    """ms / lambdas: newest last; divided differences against the newest (:416-426)."""
    rks = [(lambdas[-(i + 1)] - lambda_s0) / h for i in range(1, order)]
    d1s = [(ms[-(i + 1)] - ms[-1]) / rk for i, rk in zip(range(1, order), rks)]
    return rks + [1.0], d1s


def uni_p(x, ms, sig_hist, sigma_t, order):
    """Predictor from sig_hist[-1] to sigma_t; ms / sig_hist hold the last `order` x0 predictions and their
    sigmas, newest last (:352-486)."""
    sigma_s0 = sig_hist[-1]
    alpha_t = 1 - sigma_t
    lambda_s0 = lam(sigma_s0)
    h = lam(sigma_t) - lambda_s0
    rks, d1s = _differences(ms, [lam(s) for s in sig_hist], lambda_s0, h, order)
    R, b, B = weights(order, rks, -h)
    x_t = sigma_t / sigma_s0 * x - alpha_t * math.expm1(-h) * ms[-1]
    if d1s:
        rhos = np.array([0.5]) if order == 2 else np.linalg.solve(R[:-1, :-1], b[:-1])
        x_t = x_t - alpha_t * B * sum(r * d for r, d in zip(rhos, d1s))
    return x_t


def uni_c(x_last, ms, sig_hist, sigma_t, m_t, order):
    """Corrector: the step from sig_hist[-1] to sigma_t redone with m_t, the x0 prediction at the predicted
    point, as an extra node (:488-628)."""
    sigma_s0 = sig_hist[-1]
    alpha_t = 1 - sigma_t
    lambda_s0 = lam(sigma_s0)
    h = lam(sigma_t) - lambda_s0
    rks, d1s = _differences(ms, [lam(s) for s in sig_hist], lambda_s0, h, order)
    R, b, B = weights(order, rks, -h)
    rhos = np.array([0.5]) if order == 1 else np.linalg.solve(R, b)
    x_t = sigma_t / sigma_s0 * x_last - alpha_t * math.expm1(-h) * ms[-1]
    res = sum(r * d for r, d in zip(rhos[:-1], d1s)) if d1s else 0.0
    return x_t - alpha_t * B * (res + rhos[-1] * (m_t - ms[-1]))


def sample(flow_fn, x, num_steps: int, shift: float = 1.0, solver_order: int = 2):
    """The loop of pipeline/causal_diffusion_inference.py:566-612 around step (:657-741).
    flow_fn(x, sigma, timestep) -> flow prediction.  Returns the list of samples after each step."""
    sigmas, timesteps = schedule(num_steps, shift)
    ms, sig_hist, last_sample, this_order, lower = [], [], None, 1, 0
    out = []
    for i in range(num_steps):
        m = x - sigmas[i] * flow_fn(x, sigmas[i], int(timesteps[i]))
        if i > 0 and last_sample is not None:
            x = uni_c(last_sample, ms, sig_hist, sigmas[i], m, this_order)
        ms = (ms + [m])[-solver_order:]
        sig_hist = (sig_hist + [sigmas[i]])[-solver_order:]
        this_order = min(min(solver_order, num_steps - i), lower + 1)
        last_sample = x
        x = uni_p(x, ms, sig_hist, sigmas[i + 1], this_order)
        lower = min(lower + 1, solver_order)
        out.append(x)
    return out
