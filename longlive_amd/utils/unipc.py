"""Flow-matching UniPC multistep scheduler (mirror of wan_5b/utils/fm_solvers_unipc.py:22-802 for the
configuration LongLive uses: flow prediction, data-prediction form, B(h) = expm1(h) ("bh2"), order 2 with
lower-order final steps; pipeline/causal_diffusion_inference.py:566-612, 892-900 drives it through
``set_timesteps`` / ``timesteps`` / ``step``).

Everything here is host-side scalar work plus a handful of element-wise tensor expressions per step; the
scalars are float32 CPU tensors and the tensor expressions are written in the reference's association order,
so the same inputs give the same roundings.

The schedule is sigma in (0, 1), alpha = 1 - sigma, lambda = log(alpha / sigma).  With m the model's x0
prediction (x0 = x - sigma * flow) and h = lambda_t - lambda_s, the exact solution of the sampling ODE is

    x_t = (sigma_t / sigma_s) x_s + sigma_t * integral_{lambda_s}^{lambda_t} exp(lambda) m(lambda) d lambda.

UniP / UniC replace m(lambda) by m_s plus a combination of divided differences D_i = (m_i - m_s) / r_i taken at
r_i = (lambda_i - lambda_s) / h, with weights rho that solve sum_i rho_i r_i^(k-1) = k! z phi_(k+1)(z) / B(z),
z = -h, k = 1..p (the conditions that make the update exact for m polynomial in lambda up to degree p).
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np
import torch


@dataclass
class SchedulerOutput:
    prev_sample: torch.Tensor


def unipc_weights(order: int, rks: torch.Tensor, hh: torch.Tensor, solver_type: str = "bh2"):
    """(R, b, h_phi_1, B_h) of fm_solvers_unipc.py:428-456 / 571-599: row k (k = 1..order) of R holds
    rks**(k-1) and b_k = k! hh phi_(k+1)(hh) / B(hh), with phi_1 = expm1(hh) / hh and
    phi_(j+1) = (phi_j - 1/j!) / hh built by the reference's recurrence in the reference's order.
    ``rks`` ends with the 1.0 of the newest point."""
    h_phi_1 = torch.expm1(hh)
    if solver_type == "bh1":
        B_h = hh
    elif solver_type == "bh2":
        B_h = torch.expm1(hh)
    else:
        raise NotImplementedError(f"solver_type {solver_type!r}")
    h_phi_k = h_phi_1 / hh - 1
    factorial = 1
    rows, rhs = [], []
    for k in range(1, order + 1):
        rows.append(torch.pow(rks, k - 1))
        rhs.append(h_phi_k * factorial / B_h)
        factorial *= k + 1
        h_phi_k = h_phi_k / hh - 1 / factorial
    return torch.stack(rows), torch.tensor(rhs), h_phi_1, B_h


class FlowUniPCMultistepScheduler:
    """``set_timesteps(n, device=, shift=)`` then ``step(flow_pred, t, sample)`` once per entry of
    ``timesteps``; the last step returns the model's x0 prediction (final sigma 0)."""

    order = 1

    def __init__(self, num_train_timesteps: int = 1000, solver_order: int = 2, shift: float = 1.0,
                 use_dynamic_shifting: bool = False, solver_type: str = "bh2", lower_order_final: bool = True,
                 disable_corrector=(), prediction_type: str = "flow_prediction", predict_x0: bool = True) -> None:
        if solver_type in ("midpoint", "heun", "logrho"):
            solver_type = "bh2"  # the reference maps these names to bh2 (:99-104)
        if solver_type not in ("bh1", "bh2"):
            raise NotImplementedError(f"{solver_type} is not implemented for {type(self).__name__}")
        if prediction_type != "flow_prediction" or not predict_x0 or use_dynamic_shifting:
            raise NotImplementedError("only flow prediction in data-prediction form with a static shift is built")
        self.num_train_timesteps, self.solver_order, self.shift = num_train_timesteps, solver_order, shift
        self.solver_type, self.lower_order_final = solver_type, lower_order_final
        self.disable_corrector = list(disable_corrector)
        # training schedule (:108-117): sigma_i = 1 - alpha_i over num_train_timesteps levels, shifted
        alphas = np.linspace(1, 1 / num_train_timesteps, num_train_timesteps)[::-1].copy()
        sigmas = torch.from_numpy(1.0 - alphas).to(torch.float32)
        sigmas = shift * sigmas / (1 + (shift - 1) * sigmas)
        self.sigmas = sigmas
        self.timesteps = sigmas * num_train_timesteps
        self.sigma_min, self.sigma_max = sigmas[-1].item(), sigmas[0].item()
        self.num_inference_steps = None
        self._reset()

    def _reset(self) -> None:
        self.model_outputs = [None] * self.solver_order
        self.timestep_list = [None] * self.solver_order
        self.lower_order_nums = 0
        self.last_sample = None
        self.this_order = 1
        self.step_index = None

    def set_timesteps(self, num_inference_steps: int | None = None, device=None, sigmas=None, mu=None,
                      shift: float | None = None) -> None:
        """:162-229.  n sigmas equally spaced from sigma_max down to (not including) sigma_min, shifted by
        ``shift * s / (1 + (shift - 1) s)``, plus a final 0; timesteps = sigma * num_train_timesteps as int64."""
        if sigmas is None:
            sigmas = np.linspace(self.sigma_max, self.sigma_min, num_inference_steps + 1).copy()[:-1]
        sigmas = np.asarray(sigmas)
        shift = self.shift if shift is None else shift
        sigmas = shift * sigmas / (1 + (shift - 1) * sigmas)
        timesteps = sigmas * self.num_train_timesteps
        self.sigmas = torch.from_numpy(np.concatenate([sigmas, [0.0]]).astype(np.float32))
        self.timesteps = torch.from_numpy(timesteps).to(device=device, dtype=torch.int64)
        self.num_inference_steps = len(timesteps)
        self._reset()

    # ------------------------------------------------------------------ pieces of one step
    @staticmethod
    def _lambda(sigma: torch.Tensor) -> torch.Tensor:
        return torch.log(1 - sigma) - torch.log(sigma)

    def convert_model_output(self, model_output: torch.Tensor, sample: torch.Tensor) -> torch.Tensor:
        """flow prediction -> x0 prediction at the current sigma (:281-350)."""
        return sample - self.sigmas[self.step_index] * model_output

    def _differences(self, order: int, newest_index: int, lambda_s0, h):
        """Divided differences of the stored x0 predictions against the newest one (:416-426 / :560-570):
        point i steps back sits at sigma index ``newest_index - i``."""
        m0 = self.model_outputs[-1]
        rks, d1s = [], []
        for i in range(1, order):
            rk = (self._lambda(self.sigmas[newest_index - i]) - lambda_s0) / h
            rks.append(rk)
            d1s.append((self.model_outputs[-(i + 1)] - m0) / rk)
        rks.append(1.0)
        return torch.tensor(rks), d1s

    def _predict(self, sample: torch.Tensor, order: int) -> torch.Tensor:
        """UniP (:352-486): from sigma[step_index] to sigma[step_index + 1]."""
        m0, x = self.model_outputs[-1], sample
        sigma_t, sigma_s0 = self.sigmas[self.step_index + 1], self.sigmas[self.step_index]
        alpha_t = 1 - sigma_t
        lambda_s0 = self._lambda(sigma_s0)
        h = self._lambda(sigma_t) - lambda_s0
        rks, d1s = self._differences(order, self.step_index, lambda_s0, h)
        R, b, h_phi_1, B_h = unipc_weights(order, rks, -h, self.solver_type)
        x_t = sigma_t / sigma_s0 * x - alpha_t * h_phi_1 * m0
        if d1s:
            # order 2 uses the fixed weight 1/2 (:461-463); higher orders solve the leading block
            rhos = torch.tensor([0.5]) if order == 2 else torch.linalg.solve(R[:-1, :-1], b[:-1])
            res = sum(rho.to(x.dtype) * d for rho, d in zip(rhos, d1s))
            x_t = x_t - alpha_t * B_h * res
        return x_t.to(x.dtype)

    def _correct(self, this_model_output: torch.Tensor, last_sample: torch.Tensor, order: int) -> torch.Tensor:
        """UniC (:488-628): redo the step from sigma[step_index - 1] to sigma[step_index] with the x0
        prediction at the predicted point as an extra node."""
        m0, x = self.model_outputs[-1], last_sample
        sigma_t, sigma_s0 = self.sigmas[self.step_index], self.sigmas[self.step_index - 1]
        alpha_t = 1 - sigma_t
        lambda_s0 = self._lambda(sigma_s0)
        h = self._lambda(sigma_t) - lambda_s0
        rks, d1s = self._differences(order, self.step_index - 1, lambda_s0, h)
        R, b, h_phi_1, B_h = unipc_weights(order, rks, -h, self.solver_type)
        rhos = torch.tensor([0.5]) if order == 1 else torch.linalg.solve(R, b)  # order 1: fixed weight (:603-604)
        rhos = rhos.to(x.dtype)
        x_t = sigma_t / sigma_s0 * x - alpha_t * h_phi_1 * m0
        res = sum(rho * d for rho, d in zip(rhos[:-1], d1s)) if d1s else 0
        x_t = x_t - alpha_t * B_h * (res + rhos[-1] * (this_model_output - m0))
        return x_t.to(x.dtype)

    # ------------------------------------------------------------------ the step
    def step(self, model_output: torch.Tensor, timestep, sample: torch.Tensor, return_dict: bool = True,
             generator=None):
        """:657-741.  Corrector for the step just taken (when there is one), shift the history, predictor for
        the next step; the order ramps 1, 2, ... and drops again at the end (``lower_order_final``)."""
        if self.num_inference_steps is None:
            raise ValueError("Number of inference steps is 'None', you need to run 'set_timesteps' after creating "
                             "the scheduler")
        if self.step_index is None:
            self.step_index = self._index_for_timestep(timestep)
        converted = self.convert_model_output(model_output, sample)
        if self.step_index > 0 and self.step_index - 1 not in self.disable_corrector and self.last_sample is not None:
            sample = self._correct(converted, self.last_sample, self.this_order)
        self.model_outputs = self.model_outputs[1:] + [converted]
        self.timestep_list = self.timestep_list[1:] + [timestep]
        order = self.solver_order
        if self.lower_order_final:
            order = min(order, len(self.timesteps) - self.step_index)
        self.this_order = min(order, self.lower_order_nums + 1)
        self.last_sample = sample
        prev_sample = self._predict(sample, self.this_order)
        if self.lower_order_nums < self.solver_order:
            self.lower_order_nums += 1
        self.step_index += 1
        return SchedulerOutput(prev_sample) if return_dict else (prev_sample,)

    def _index_for_timestep(self, timestep) -> int:
        """:630-655: the position of ``timestep`` in ``timesteps`` (the second match if it occurs twice; an
        ``IndexError`` if it does not occur, as in the reference)."""
        t = torch.as_tensor(timestep).to(self.timesteps.device)
        hits = (self.timesteps == t).nonzero()
        return hits[1 if len(hits) > 1 else 0].item()

    def scale_model_input(self, sample: torch.Tensor, *args, **kwargs) -> torch.Tensor:
        return sample

    def __len__(self) -> int:
        return self.num_train_timesteps


def convert_flow_pred_to_x0(flow_pred: torch.Tensor, xt: torch.Tensor, sigma_t) -> torch.Tensor:
    """x0 = x_t - sigma_t * flow in float64, cast back (utils/wan_5b_wrapper.py:404-428; ``sigma_t`` is the
    schedule's sigma at the sample's timestep, a float or a tensor broadcastable to ``xt``)."""
    sigma_t = torch.as_tensor(sigma_t, dtype=torch.float64, device=flow_pred.device)
    return (xt.double() - sigma_t * flow_pred.double()).to(flow_pred.dtype)
