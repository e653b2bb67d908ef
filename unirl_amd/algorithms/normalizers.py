"""Reward normalisers with the signatures of ``unirl/algorithms/normalizers.py:8-84``.

``normalize_grouped`` takes arbitrary index lists, optional trimmed statistics and a
final clip; it runs as one kernel (``unirl_normalize_grouped``, one lane per group).
``normalize_global`` is the batch-wide z-score on the group-advantage kernel.
Both use the unbiased std with epsilon added outside the square root, unlike the
live ``compute_advantages`` path.
"""

from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops


def _on_device(rewards: torch.Tensor) -> torch.Tensor:
    if rewards.is_cuda:
        return rewards
    if not torch.cuda.is_available():
        raise RuntimeError("reward normalisation kernels need a HIP device; there is no CPU fallback")
    return rewards.to(torch.device("cuda", torch.cuda.current_device()))


def normalize_grouped(
    rewards: torch.Tensor,
    group_indices: List[List[int]],
    epsilon: float = 1e-8,
    clip_max: Optional[float] = None,
    trim_outliers_ratio: float = 0.0,
    use_global_std: bool = False,
) -> torch.Tensor:
    """Advantages ``[N]``: per group ``(r - mean_g) / (std_g + eps)``; samples in no group stay 0."""
    out = ops.normalize_grouped(
        _on_device(rewards), group_indices, eps=epsilon, clip_max=clip_max,
        trim_outliers_ratio=trim_outliers_ratio, use_global_std=use_global_std,
    )
    return out.to(device=rewards.device, dtype=rewards.dtype)


def normalize_global(rewards: torch.Tensor, epsilon: float = 1e-8, clip_max: Optional[float] = None) -> torch.Tensor:
    """``(r - mean) / (std_unbiased + eps)`` over the whole batch, optionally clipped."""
    n = int(rewards.numel())
    out = ops.normalize_grouped(
        _on_device(rewards), [list(range(n))], eps=epsilon, clip_max=clip_max, trim_outliers_ratio=0.0,
        use_global_std=False,
    )
    return out.to(device=rewards.device, dtype=rewards.dtype)


__all__ = ["normalize_global", "normalize_grouped"]
