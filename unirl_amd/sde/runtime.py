"""Sigma schedule for flow-matching samplers (host-side, a few dozen floats).

``get_sigma_schedule`` keeps the signature of ``unirl/sde/runtime.py:71-110``.
Only the static branch (``mu is None``) is evaluated here; the dynamic-shift
branch of the reference delegates to ``diffusers``' scheduler and needs that
package at call time.
"""

from __future__ import annotations

from typing import Optional

import torch


def get_sigma_schedule(
    num_steps: int,
    shift: float = 3.0,
    device: Optional[torch.device] = None,
    *,
    mu: Optional[float] = None,
    time_shift_type: str = "exponential",
) -> torch.Tensor:
    """``[num_steps + 1]`` fp32 sigmas from 1 down to 0.

    Static mode (``mu is None``): ``t = linspace(1, 0, T+1)``, ``sigma = shift*t / (1 + (shift-1)*t)``.
    """
    if mu is not None:
        try:
            from diffusers.schedulers import FlowMatchEulerDiscreteScheduler
        except ImportError as exc:  # pragma: no cover - depends on the environment
            raise RuntimeError(
                "get_sigma_schedule(mu=...) uses diffusers' FlowMatchEulerDiscreteScheduler, "
                "which is not installed; only the static schedule (mu=None) is built in"
            ) from exc
        import numpy as np

        scheduler = FlowMatchEulerDiscreteScheduler(
            num_train_timesteps=1000, use_dynamic_shifting=True, time_shift_type=time_shift_type
        )
        scheduler.set_timesteps(
            num_inference_steps=num_steps, sigmas=np.linspace(1.0, 1.0 / num_steps, num_steps), mu=mu
        )
        sigmas = scheduler.sigmas
    else:
        t = torch.linspace(1.0, 0.0, num_steps + 1)
        sigmas = (shift * t) / (1 + (shift - 1) * t)
    return sigmas if device is None else sigmas.to(device)


def calculate_dynamic_mu(
    image_seq_len: int,
    base_seq_len: int = 256,
    max_seq_len: int = 4096,
    base_shift: float = 0.5,
    max_shift: float = 1.15,
) -> float:
    """Linear map from image sequence length to the dynamic-shift mu (unirl/sde/runtime.py:113-130)."""
    slope = (max_shift - base_shift) / (max_seq_len - base_seq_len)
    return image_seq_len * slope + (base_shift - slope * base_seq_len)


__all__ = ["calculate_dynamic_mu", "get_sigma_schedule"]
