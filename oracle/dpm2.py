"""DPM-Solver-2 deterministic sampler (oracle; test infrastructure only).

Eager-torch CPU restatement of the stateful ODE strategy of unirl/sde/kernels.py:
  solver state (two most recent x0 predictions, warm-up counter)   :342-358
  x0 prediction  sample - sigma * model_output                     :360-368
  first-order update                                               :377-391
  multistep second-order update                                    :394-425
  branch selection, DDIM update of the first and last step         :428-471
  DPM2Strategy.step / StepStrategy.denoise: fp32 upcast, no log-prob   :43-99, :492-516
The scalar coefficients are 0-dim tensors exactly as there: in the dtype of the schedule for the
DDIM update, in float64 for the two DPM updates; torch multiplies an fp32 tensor by such a scalar
after rounding the scalar to fp32.
"""

from __future__ import annotations

from typing import List, Optional

import numpy as np
import torch


def _half_log_snr(sigma: torch.Tensor) -> torch.Tensor:
    """lambda = log(alpha) - log(sigma) with alpha = 1 - sigma (flow-matching schedule)."""
    return torch.log(1 - sigma) - torch.log(sigma)


class Dpm2Solver:
    """One sampling trajectory; ``step`` must be called with consecutive ``step_index`` values."""

    def __init__(self, sigmas: torch.Tensor) -> None:
        self.sigmas = sigmas
        self.history: List[Optional[torch.Tensor]] = [None, None]  # x0 predictions, oldest first
        self.warm = 0  # completed steps, saturating at 2

    def step(self, model_output: torch.Tensor, sample: torch.Tensor, step_index: int) -> torch.Tensor:
        sig = self.sigmas
        n_steps = int(sig.shape[0]) - 1
        v, x = model_output.float(), sample.float()
        x0 = x - sig[step_index].to(dtype=v.dtype) * v
        self.history = [self.history[1], x0]
        last = step_index == n_steps - 1
        if self.warm < 1 or last:
            if step_index == 0 or last:
                t, s = sig[step_index + 1], sig[step_index]
                eps = (x - (1 - s) * x0) / s
                # sqrt with numpy: correctly rounded on every host, which torch's CPU sqrt is not
                root = torch.tensor(np.sqrt((t**2).numpy()), dtype=t.dtype)
                out = (1 - t) * x0 + root * eps
            else:
                out = self._first_order(x0, x, step_index)
        else:
            out = self._second_order(x, step_index)
        if self.warm < 2:
            self.warm += 1
        return out.to(v.dtype)

    def _first_order(self, x0: torch.Tensor, x: torch.Tensor, i: int) -> torch.Tensor:
        sig = self.sigmas.to(torch.float64)
        s_t, s_s = sig[i + 1], sig[i]
        h = _half_log_snr(s_t) - _half_log_snr(s_s)
        return (s_t / s_s) * x - ((1 - s_t) * (torch.exp(-h) - 1.0)) * x0

    def _second_order(self, x: torch.Tensor, i: int) -> torch.Tensor:
        sig = self.sigmas.to(torch.float64)
        s_t, s_0, s_1 = sig[i + 1], sig[i], sig[i - 1]
        lam_t, lam_0, lam_1 = _half_log_snr(s_t), _half_log_snr(s_0), _half_log_snr(s_1)
        m_old, m_new = self.history
        h, h_prev = lam_t - lam_0, lam_0 - lam_1
        r0 = h_prev / h
        d0, d1 = m_new, (1.0 / r0) * (m_new - m_old)
        growth = (1 - s_t) * (torch.exp(-h) - 1.0)
        return (s_t / s_0) * x - growth * d0 - 0.5 * growth * d1


def sample_trajectory(velocity_fn, x_init: torch.Tensor, sigmas: torch.Tensor) -> torch.Tensor:
    """Run the solver over the whole schedule with ``velocity_fn(x, sigma) -> model output``."""
    solver = Dpm2Solver(sigmas)
    x = x_init
    for i in range(int(sigmas.shape[0]) - 1):
        x = solver.step(velocity_fn(x, sigmas[i]), x, i)
    return x
