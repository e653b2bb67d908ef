"""Group-normalised advantages (oracle; test infrastructure only).

Eager-torch restatement of
  RolloutTrack.compute_advantages   unirl/types/rollout_resp.py:277-333
    (rewards tensor + parent ids in, advantages out; the track container itself
     is not restated)
  normalize_grouped / normalize_global   unirl/algorithms/normalizers.py:32-84
"""

from __future__ import annotations

from typing import List, Optional, Sequence

import torch


def compute_advantages(
    rewards: torch.Tensor,
    parent_ids: Optional[Sequence],
    normalize: bool = True,
    eps: float = 1e-8,
    scope: str = "group",
    use_global_std: bool = False,
) -> torch.Tensor:
    n = int(rewards.shape[0])
    if n == 0:
        return rewards.to(torch.float32)
    if scope == "global":
        r = rewards.to(torch.float32)
        return (r - r.mean()) / (r.std() + eps) if normalize else r - r.mean()
    if parent_ids is None:
        return torch.zeros_like(rewards, dtype=torch.float32)
    unique = list(dict.fromkeys(parent_ids))
    n_groups = len(unique)
    if n_groups == 0 or n % n_groups != 0:
        raise ValueError(f"compute_advantages: non-uniform group sizes (n={n}, n_groups={n_groups})")
    branch = n // n_groups
    if list(parent_ids) != [p for p in unique for _ in range(branch)]:
        raise ValueError("compute_advantages: parent_ids not in group-by-parent contiguous order")
    r = rewards.to(torch.float32)
    g = r.view(n_groups, branch)
    mean = g.mean(dim=1, keepdim=True)
    if not normalize:
        return (g - mean).flatten()
    if use_global_std:
        std = r.std() + eps
    else:
        std = (g.var(dim=1, unbiased=False, keepdim=True) + eps).sqrt()
    return ((g - mean) / std).flatten()


def normalize_grouped(
    rewards: torch.Tensor,
    group_indices: List[List[int]],
    epsilon: float = 1e-8,
    clip_max: Optional[float] = None,
    trim_outliers_ratio: float = 0.0,
    use_global_std: bool = False,
) -> torch.Tensor:
    out = torch.zeros_like(rewards)
    batch_std = rewards.std() + epsilon if use_global_std else None
    for idx in group_indices:
        if not idx:
            continue
        g = rewards[idx]
        stats = g
        if trim_outliers_ratio > 0 and len(idx) > 2:
            srt, _ = torch.sort(g)
            k = int(len(srt) * trim_outliers_ratio)
            stats = srt[k:-k] if (k > 0 and 2 * k < len(srt)) else srt
        mean = stats.mean()
        std = batch_std if use_global_std else (stats.std() + epsilon)
        out[idx] = (g - mean) / std
    if clip_max is not None:
        out = torch.clamp(out, -clip_max, clip_max)
    return out


def normalize_global(rewards: torch.Tensor, epsilon: float = 1e-8, clip_max: Optional[float] = None) -> torch.Tensor:
    out = (rewards - rewards.mean()) / (rewards.std() + epsilon)
    if clip_max is not None:
        out = torch.clamp(out, -clip_max, clip_max)
    return out
