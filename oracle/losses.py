"""Token-level ratio losses (oracle; test infrastructure only).

Eager-torch restatement of
  PPO-clip loss + metrics      unirl/algorithms/base.py:133-157
  DRPO loss + metrics          unirl/algorithms/drpo.py:131-159
  |dlogp| drift gauge          unirl/algorithms/base.py:98-103
  advantage expansion          unirl/algorithms/grpo.py:187-198
  aggregation modes            unirl/algorithms/grpo.py:148-155, drpo.py:318-330
Both loss functions keep ``new_logp`` differentiable, so autograd through them
is the reference's backward.
"""

from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch


def grpo_clip_loss(new_logp, old_logp, advantages, clip_range, clip_range_high=None):
    high = clip_range if clip_range_high is None else clip_range_high
    log_diff = new_logp - old_logp
    ratio = torch.exp(log_diff)
    adv = advantages.detach()
    unclipped = -adv * ratio
    clipped = -adv * torch.clamp(ratio, 1.0 - clip_range, 1.0 + high)
    loss = torch.maximum(unclipped, clipped)
    ratio_std = ratio.std() if ratio.numel() > 1 else torch.zeros((), dtype=ratio.dtype)
    gt = (ratio - 1.0 > high).float()
    lt = (1.0 - ratio > clip_range).float()
    metrics = {
        "ratio_mean": ratio.mean().detach(),
        "ratio_std": ratio_std.detach(),
        "ratio_min": ratio.min().detach(),
        "ratio_max": ratio.max().detach(),
        "clip_fraction": torch.maximum(gt, lt).mean().detach(),
        "clipfrac_gt_one": gt.mean().detach(),
        "clipfrac_lt_one": lt.mean().detach(),
        "approx_kl": (0.5 * log_diff.pow(2)).mean().detach(),
    }
    return loss, metrics


def drpo_loss(new_logp, old_logp, advantages, epsilon, mu_weighted=True):
    log_diff = torch.clamp(new_logp - old_logp, min=-20.0, max=20.0)
    ratio = torch.exp(log_diff)
    adv = advantages.detach()
    old_prob = torch.exp(old_logp).detach()
    ratio_delta = ratio - 1.0
    if mu_weighted:
        weight = old_prob
        adaptive_eps = torch.where(old_prob > 0.0, epsilon / old_prob, torch.full_like(old_prob, float("inf")))
    else:
        weight = torch.ones_like(old_prob)
        adaptive_eps = torch.full_like(old_prob, epsilon)
    penalty = adv.abs() * weight * ratio_delta.square() / (2.0 * epsilon)
    loss = -adv * ratio + penalty
    metrics = {
        "ratio_mean": ratio.mean().detach(),
        "ratio_max": ratio.max().detach(),
        "approx_kl": ((ratio - 1.0) - log_diff).mean().detach(),
        "drpo_penalty_mean": penalty.mean().detach(),
        "clipfrac_upper": (ratio > (1.0 + adaptive_eps)).float().mean().detach(),
        "clipfrac_lower": (ratio < (1.0 - adaptive_eps)).float().mean().detach(),
    }
    return loss, metrics


def logp_absdiff(new_logp, old_logp) -> Dict[str, float]:
    with torch.no_grad():
        d = (new_logp - old_logp).abs()
    return {"rollout_replay_logp_absdiff_mean": float(d.mean()), "rollout_replay_logp_absdiff_max": float(d.max())}


def expand_advantages(advantages: torch.Tensor, lengths: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    bs = int(advantages.shape[0])
    if int(lengths.shape[0]) != bs:
        raise ValueError(f"advantages batch={bs} != lengths={int(lengths.shape[0])}")
    adv = advantages.detach().to(dtype)
    parts = [adv[k].expand(int(lengths[k])) for k in range(bs) if int(lengths[k]) > 0]
    if not parts:
        return torch.zeros(0, dtype=dtype)
    return torch.cat(parts, dim=0)


def aggregate(loss_per_elem: torch.Tensor, lengths: Optional[torch.Tensor], mode: str, horizon: int = 8192):
    """Packed [total_tokens] loss -> scalar."""
    if mode in ("seq-mean-token-sum-norm", "seq-mean-token-mean") and lengths is not None:
        parts = torch.split(loss_per_elem, [int(n) for n in lengths.tolist()])
        if mode == "seq-mean-token-sum-norm":
            return torch.stack([p.sum() for p in parts]).mean() / float(horizon)
        return torch.stack([p.mean() if p.numel() else p.new_zeros(()) for p in parts]).mean()
    return loss_per_elem.mean()


def pack_padded(x: torch.Tensor, lengths: torch.Tensor) -> torch.Tensor:
    """[n_seq, max_len] padded -> packed [sum(lengths)] (row r contributes its first lengths[r] slots)."""
    return torch.cat([x[r, : int(lengths[r])] for r in range(x.shape[0])], dim=0)


def token_loss(
    kind: str,
    new_logp: torch.Tensor,
    old_logp: torch.Tensor,
    seq_advantages: torch.Tensor,
    lengths: torch.Tensor,
    *,
    mode: str = "token-mean",
    horizon: int = 8192,
    clip_range: float = 0.2,
    clip_range_high: Optional[float] = None,
    epsilon: float = 12.5,
    mu_weighted: bool = True,
    loss_mask: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, Dict[str, torch.Tensor]]:
    """The per-micro-batch loss of GRPO / DRPO on PACKED tokens: expand advantages,
    element loss, optional mask (DRPO), aggregation.  Returns (scalar loss, metrics)."""
    adv_tok = expand_advantages(seq_advantages, lengths, dtype=new_logp.dtype)
    if kind == "grpo":
        elem, metrics = grpo_clip_loss(new_logp, old_logp, adv_tok, clip_range, clip_range_high)
    elif kind == "drpo":
        elem, metrics = drpo_loss(new_logp, old_logp, adv_tok, epsilon, mu_weighted)
    else:
        raise ValueError(kind)
    if loss_mask is not None:
        elem = elem * loss_mask.to(elem.dtype)
    loss = aggregate(elem, lengths, mode, horizon)
    metrics = dict(metrics)
    metrics.update({k: torch.tensor(v) for k, v in logp_absdiff(new_logp, old_logp).items()})
    return loss, metrics
