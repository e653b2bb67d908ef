"""Flow-DPPO Gaussian-KL trust-region mask and masked loss (oracle; test infrastructure only).

Eager-torch restatement of unirl/algorithms/flowdppo.py:
  gaussian KL per element      :51
  KL-ADV masked loss + metrics :86-138
  sigma_t                      :353-368
and of the step gather, unirl/algorithms/base.py:61-80.
"""

from __future__ import annotations

from typing import List

import torch


def gaussian_kl(p: torch.Tensor, q: torch.Tensor, sigma: torch.Tensor) -> torch.Tensor:
    return (p - q) ** 2 / (2 * sigma**2)


def kl_per_sample(new_means, old_means, sigma_t) -> torch.Tensor:
    kl = gaussian_kl(new_means, old_means, sigma_t)
    return kl.mean(dim=tuple(range(2, kl.ndim)))


def flowdppo_loss(new_logp, old_logp, new_means, old_means, advantages, sigma_t, kl_mask_threshold):
    log_diff = new_logp - old_logp
    ratio = torch.exp(log_diff)
    adv = advantages.detach()
    unclipped = -adv * ratio
    kl = kl_per_sample(new_means, old_means, sigma_t)
    kl_mask = kl < kl_mask_threshold
    pos_rm = (~kl_mask) & (ratio > 1.0) & (adv > 0)
    neg_rm = (~kl_mask) & (ratio < 1.0) & (adv < 0)
    rm = pos_rm | neg_rm
    keep = (~rm).detach()
    loss = torch.where(keep, unclipped, torch.zeros((), dtype=unclipped.dtype))
    ratio_std = ratio.std() if ratio.numel() > 1 else torch.zeros((), dtype=ratio.dtype)
    metrics = {
        "ratio_mean": ratio.mean().detach(),
        "ratio_std": ratio_std.detach(),
        "ratio_min": ratio.min().detach(),
        "ratio_max": ratio.max().detach(),
        "approx_kl": (0.5 * log_diff.pow(2)).mean().detach(),
        "kl_new_old_mean": kl.mean().detach(),
        "kl_new_old_max": kl.max().detach(),
        "kl_mask_fraction": (~kl_mask).float().mean().detach(),
        "pos_rm_fraction": pos_rm.float().mean().detach(),
        "neg_rm_fraction": neg_rm.float().mean().detach(),
        "masked_fraction": rm.float().mean().detach(),
        "unmasked_fraction": keep.float().mean().detach(),
    }
    return loss, metrics


def sigma_t(sigmas: torch.Tensor, target_steps: List[int], eta: float, add_kl_coefficient: bool = True):
    if not add_kl_coefficient:
        return torch.ones(1, len(target_steps), 1, 1, 1)
    sigmas = sigmas.to(dtype=torch.float32)
    idx = torch.tensor(target_steps, dtype=torch.long)
    s = sigmas[idx]
    s_next = sigmas[idx + 1]
    dt = s_next - s
    std_dev_t = torch.sqrt(s / (1.0 - torch.clamp(s, max=0.99))) * eta
    return (std_dev_t * torch.sqrt(-dt)).reshape(1, -1, 1, 1, 1)


def gather_sde_field(tensor, sde_indices, target_steps, field_name="field"):
    if tensor is None or sde_indices is None:
        raise ValueError(
            f"gather_sde_field: {field_name} or sde_indices is None "
            "(ensure prepare_segment ran before compute_loss_and_backward)."
        )
    target_t = torch.tensor(target_steps, dtype=sde_indices.dtype)
    order = sde_indices.argsort()
    sorted_idx = sde_indices[order]
    tensor = tensor[:, order.tolist()]
    pos = torch.searchsorted(sorted_idx, target_t).clamp(max=sorted_idx.shape[0] - 1)
    if (sorted_idx[pos] != target_t).any():
        bad = [int(t) for t, p in zip(target_steps, pos) if sorted_idx[p] != t]
        raise ValueError(
            f"gather_sde_field({field_name}): target steps {bad} not in sde_indices={sorted_idx.tolist()}"
        )
    return tensor[:, pos.tolist()]


def gather_by_lookup(tensor, sde_indices, target_steps):
    """Brute-force statement of the same gather: a python dict from step to slot."""
    slot = {int(s): i for i, s in enumerate(sde_indices.tolist())}
    missing = [t for t in target_steps if t not in slot]
    if missing:
        raise ValueError(f"target steps {missing} not recorded")
    return torch.stack([tensor[:, slot[int(t)]] for t in target_steps], dim=1)
