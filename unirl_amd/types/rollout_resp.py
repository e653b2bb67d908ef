"""Group advantages with the contract of ``RolloutTrack.compute_advantages``
(``unirl/types/rollout_resp.py:220-333``).

The reference method lives on its rollout-track container; the track machinery
(tensor handles, fork / split) is not part of this package, so the arithmetic is
exposed as :func:`compute_advantages` over ``(rewards, parent_ids)`` and on a minimal
:class:`RolloutTrack` that carries just the fields the method reads and writes.
Validation, error types and messages follow the reference; the statistics run in
one kernel (``unirl_group_advantages``).
"""

from __future__ import annotations

import dataclasses
from typing import Any, Dict, List, Optional, Sequence

import torch

from .. import ops


def _compute_device(rewards: torch.Tensor, device: Optional[torch.device]) -> torch.device:
    if device is not None:
        return torch.device(device)
    if rewards.is_cuda:
        return rewards.device
    if not torch.cuda.is_available():
        raise RuntimeError(
            "compute_advantages: no HIP device is visible; the group-advantage kernel has no CPU fallback"
        )
    return torch.device("cuda", torch.cuda.current_device())


def compute_advantages(
    rewards: torch.Tensor,
    parent_ids: Optional[Sequence[Any]],
    normalize: bool = True,
    eps: float = 1e-8,
    scope: str = "group",
    use_global_std: bool = False,
    *,
    device: Optional[torch.device] = None,
) -> torch.Tensor:
    """fp32 advantages ``[n]`` on the device of ``rewards`` (host rewards, as the driver of the
    reference holds them, are uploaded, reduced on the GPU and copied back).

    ``scope="group"``: ``(r - mean_g) / sqrt(var_pop_g + eps)``; ``use_global_std`` divides by one
    batch-wide unbiased ``std + eps`` instead; ``normalize=False`` only centres.
    ``scope="global"``: ``(r - mean) / (std_unbiased + eps)``.  ``parent_ids=None`` (a root track,
    every sample its own group) gives zeros.
    """
    if rewards is None:
        raise ValueError("RolloutTrack.compute_advantages: track has no rewards")
    n = int(rewards.shape[0])
    if n == 0:
        return rewards.to(torch.float32)
    home = rewards.device
    if scope != "global" and parent_ids is None:
        return torch.zeros_like(rewards, dtype=torch.float32)
    if scope == "global":
        n_groups = 1
    else:
        unique_pids = list(dict.fromkeys(parent_ids))
        n_groups = len(unique_pids)
        if n_groups == 0 or n % n_groups != 0:
            raise ValueError(
                f"compute_advantages: non-uniform group sizes (n={n}, n_groups={n_groups}). Expected uniform "
                f"branching factor with group-by-parent ordering — use fork_track / make_root_track to build "
                f"the track."
            )
        branch = n // n_groups
        if list(parent_ids) != [pid for pid in unique_pids for _ in range(branch)]:
            raise ValueError(
                "compute_advantages: parent_ids not in group-by-parent contiguous order. Siblings must be "
                "consecutive (use fork_track / make_root_track), got interleaved ordering."
            )
    dev = _compute_device(rewards, device)
    adv = ops.group_advantages(
        rewards.detach().to(device=dev, dtype=torch.float32), n_groups, normalize=normalize, eps=eps,
        scope="global" if scope == "global" else "group", use_global_std=use_global_std,
    )
    return adv if adv.device == home else adv.to(home)


@dataclasses.dataclass
class RolloutTrack:
    """The slice of the reference's rollout track that advantage computation touches."""

    sample_ids: List[str]
    parent_ids: Optional[List[str]] = None
    rewards: Optional[torch.Tensor] = None
    advantages: Optional[torch.Tensor] = None
    extras: Dict[str, Any] = dataclasses.field(default_factory=dict)

    def compute_advantages(
        self, normalize: bool = True, eps: float = 1e-8, scope: str = "group", use_global_std: bool = False
    ) -> "RolloutTrack":
        """A new track with ``advantages`` set (the input track is left untouched)."""
        if self.rewards is None:
            raise ValueError("RolloutTrack.compute_advantages: track has no rewards")
        if len(self.sample_ids) == 0:
            return self
        adv = compute_advantages(
            self.rewards, self.parent_ids, normalize=normalize, eps=eps, scope=scope, use_global_std=use_global_std
        )
        return dataclasses.replace(self, advantages=adv)


__all__ = ["RolloutTrack", "compute_advantages"]
