"""SDE transition + per-sample Gaussian log-prob (oracle; test infrastructure only).

Eager-torch CPU restatement of unirl/sde/kernels.py:
  denoise prologue / epilogue   :60-99   (fp32 upcast, sigma broadcast)
  _finalize_logp                :168-177 (dtype round trip, mean over dims >= 1)
  flow   step / log-prob        :222-236 / :200-204
  dance  step / log-prob        :319-333 / :297-301
  cps    step / log-prob        :270-279 / :253
The only deviation: sampling noise is an argument instead of being drawn inside.

``ieee_sqrt=True`` evaluates the square roots of the scalar coefficients with
numpy (hardware sqrt, correctly rounded on every CPU) instead of ``torch.sqrt``,
whose CPU path goes through a vendor math library that returns a 1-ulp-different
fp32 root on some hosts (seen: sqrt(0x3c47ce40) = 0x3de22a0a, the correctly
rounded value, on one CPU and 0x3de22a09 on another).  Every other operation in
the chain is an IEEE add / sub / mul / div, so with this switch the element-wise
outputs are reproducible bit for bit across machines.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch

KINDS = ("flow", "dance", "cps")


def _sqrt(t: torch.Tensor, ieee: bool) -> torch.Tensor:
    if ieee and t.dtype == torch.float32 and not t.requires_grad:
        return torch.from_numpy(np.sqrt(t.detach().contiguous().numpy()))
    return torch.sqrt(t)


def _broadcast_sigma(s: torch.Tensor, ndim: int) -> torch.Tensor:
    s = s.float()
    if s.dim() == 0:
        s = s.unsqueeze(0)
    while s.dim() < ndim:
        s = s.unsqueeze(-1)
    return s


def sde_step(
    kind: str,
    noise_pred: torch.Tensor,
    sample: torch.Tensor,
    sigma: torch.Tensor,
    sigma_next: torch.Tensor,
    eta: float,
    prev_sample: Optional[torch.Tensor],
    noise: Optional[torch.Tensor],
    sigma_max,
    ieee_sqrt: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(prev_sample, prev_sample_mean, std_var) on fp32 inputs with broadcast sigmas."""
    if kind == "cps":
        std_dev_t = sigma_next * math.sin(eta * math.pi / 2)
        pred_original = sample - sigma * noise_pred
        noise_estimate = sample + noise_pred * (1 - sigma)
        mean = pred_original * (1 - sigma_next) + noise_estimate * _sqrt(sigma_next**2 - std_dev_t**2, ieee_sqrt)
        if prev_sample is None:
            prev_sample = mean + std_dev_t * noise
        return prev_sample, mean, std_dev_t
    dt = sigma_next - sigma
    if kind == "flow":
        std_dev_t = _sqrt(sigma / (1 - torch.where(sigma == 1, sigma_max, sigma)), ieee_sqrt) * eta
    elif kind == "dance":
        std_dev_t = eta
    else:
        raise ValueError(kind)
    mean = sample * (1 + std_dev_t**2 / (2 * sigma) * dt) + noise_pred * (
        1 + std_dev_t**2 * (1 - sigma) / (2 * sigma)
    ) * dt
    if prev_sample is None:
        prev_sample = mean + std_dev_t * _sqrt(-dt, ieee_sqrt) * noise
    std_var = std_dev_t * _sqrt(-dt, ieee_sqrt)
    return prev_sample, mean, std_var


def elem_log_prob(kind: str, prev_sample: torch.Tensor, mean: torch.Tensor, std_var) -> torch.Tensor:
    # the sample is detached: gradients reach the log-prob through the mean only
    if kind == "cps":
        return -((prev_sample.detach() - mean) ** 2)
    return (
        -((prev_sample.detach() - mean) ** 2) / (2 * std_var**2) - torch.log(std_var) - 0.5 * math.log(2 * math.pi)
    )


def sde_denoise(
    kind: str,
    noise_pred: torch.Tensor,
    sample: torch.Tensor,
    sigma: torch.Tensor,
    sigma_next: torch.Tensor,
    *,
    eta: float = 1.0,
    prev_sample: Optional[torch.Tensor] = None,
    noise: Optional[torch.Tensor] = None,
    sigma_max=0.99,
    ieee_sqrt: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor], torch.Tensor]:
    """Full denoise: returns (prev_sample fp32, log_prob [B] or None, prev_sample_mean fp32)."""
    input_dtype = sample.dtype
    noise_pred = noise_pred.float()
    sample = sample.float()
    if prev_sample is not None:
        prev_sample = prev_sample.float()
    elif noise is None:
        noise = torch.zeros_like(sample)
    sigma = _broadcast_sigma(sigma, sample.dim())
    sigma_next = _broadcast_sigma(sigma_next, sample.dim())
    prev, mean, std_var = sde_step(
        kind, noise_pred, sample, sigma, sigma_next, eta, prev_sample, noise, sigma_max, ieee_sqrt
    )
    if eta < 1e-7:
        return prev, None, mean
    prev = prev.to(dtype=input_dtype).float()
    lp = elem_log_prob(kind, prev, mean, std_var)
    lp = lp.mean(dim=tuple(range(1, lp.ndim)))
    return prev, lp, mean


def sde_rollout(
    kind: str,
    x0: torch.Tensor,
    velocities,
    noises,
    sigmas: torch.Tensor,
    etas,
    sigma_max=None,
    ieee_sqrt: bool = False,
):
    """Chain of denoise calls as in the stage loop (unirl/models/sd3/diffusion.py:364-390):
    sigma_max = sigmas[1]; the latent is cast back to the trajectory dtype (= x0.dtype)
    between steps.  Returns (x_final fp32, logp [B,S] with NaN where eta<1e-7, trajectory)."""
    S = len(velocities)
    if isinstance(etas, (int, float)):
        etas = [float(etas)] * S
    if sigma_max is None:
        sigma_max = sigmas[1].float()
    x = x0
    cols, traj = [], []
    for k in range(S):
        prev, lp, _ = sde_denoise(
            kind, velocities[k], x, sigmas[k], sigmas[k + 1], eta=etas[k], noise=noises[k], sigma_max=sigma_max,
            ieee_sqrt=ieee_sqrt,
        )
        if lp is None:
            lp = torch.full((x0.shape[0],), float("nan"))
        cols.append(lp)
        x = prev.to(x0.dtype)
        traj.append(x.float())
    return x.float(), torch.stack(cols, dim=1), torch.stack(traj, dim=0)


# ---------------------------------------------------------------------------
# float64 brute force (tiny inputs): independent of torch broadcasting rules
# ---------------------------------------------------------------------------
def sde_denoise_f64(kind, v, x, sigma, sigma_next, eta, prev=None, noise=None, sigma_max=0.99):
    """Nested python lists / floats in, python floats out. v, x, prev, noise are
    [B][D] lists; sigma, sigma_next floats.  Returns (prev[B][D], logp[B], mean[B][D])."""
    B, D = len(x), len(x[0])
    s, sn = float(sigma), float(sigma_next)
    dt = sn - s
    out_prev, out_mean, out_lp = [], [], []
    for b in range(B):
        pm, pp, acc = [], [], 0.0
        for j in range(D):
            if kind == "cps":
                std = sn * math.sin(eta * math.pi / 2)
                po = x[b][j] - s * v[b][j]
                ne = x[b][j] + v[b][j] * (1 - s)
                m = po * (1 - sn) + ne * math.sqrt(sn * sn - std * std)
                sv = std
            else:
                if kind == "flow":
                    den = 1 - (float(sigma_max) if s == 1 else s)
                    std = math.sqrt(s / den) * eta
                else:
                    std = eta
                m = x[b][j] * (1 + std * std / (2 * s) * dt) + v[b][j] * (1 + std * std * (1 - s) / (2 * s)) * dt
                sv = std * math.sqrt(-dt)
            p = prev[b][j] if prev is not None else m + sv * (noise[b][j] if noise is not None else 0.0)
            if kind == "cps":
                lp = -((p - m) ** 2)
            else:
                lp = -((p - m) ** 2) / (2 * sv * sv) - math.log(sv) - 0.5 * math.log(2 * math.pi)
            acc += lp
            pm.append(m)
            pp.append(p)
        out_prev.append(pp)
        out_mean.append(pm)
        out_lp.append(acc / D)
    return out_prev, out_lp, out_mean
