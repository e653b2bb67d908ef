"""Static flow-matching sigma schedule (oracle; test infrastructure only).

Follows unirl/sde/runtime.py:92-96: ``t = linspace(1, 0, T+1)`` in fp32 and
``sigma = shift*t / (1 + (shift-1)*t)``.
"""

from __future__ import annotations

import torch


def sigma_schedule(num_steps: int, shift: float = 3.0) -> torch.Tensor:
    t = torch.linspace(1.0, 0.0, num_steps + 1)
    return (shift * t) / (1 + (shift - 1) * t)


def sigma_schedule_f64(num_steps: int, shift: float = 3.0) -> list:
    """Exact-arithmetic statement in python floats (float64)."""
    out = []
    for i in range(num_steps + 1):
        t = 1.0 - i / num_steps
        out.append(shift * t / (1.0 + (shift - 1.0) * t))
    return out
