"""Autograd bindings of the fused ratio-loss kernels."""

from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from .. import _native as N
from ..ops import RatioLossPlan


class _ElemLossFn(torch.autograd.Function):
    """``loss_per_elem`` (caller reduces) + metrics vector; backward is one kernel."""

    @staticmethod
    def forward(ctx, new_logp: torch.Tensor, plan: RatioLossPlan):
        elem, metrics = plan.forward(want_elem=True)
        ctx.plan = plan
        ctx.mark_non_differentiable(metrics)
        return elem, metrics

    @staticmethod
    def backward(ctx, g_elem, _g_metrics):
        grad = ctx.plan.backward(g_scale=None, g_elem=g_elem, aggregate=False, n_valid=None)
        return grad, None


class _ScalarLossFn(torch.autograd.Function):
    """Aggregated scalar loss + metrics vector in one launch; backward is one kernel."""

    @staticmethod
    def forward(ctx, new_logp: torch.Tensor, plan: RatioLossPlan):
        _, metrics = plan.forward(want_elem=False)
        ctx.plan = plan
        ctx.metrics = metrics  # slot M_NUM_TOKENS is the token-mean denominator of the backward
        # a view, not a copy: a clone would be one more launch on a path of two
        loss = metrics[N.M_LOSS]
        ctx.mark_non_differentiable(metrics)
        return loss, metrics

    @staticmethod
    def backward(ctx, g_loss, _g_metrics):
        n_valid = ctx.metrics[N.M_NUM_TOKENS : N.M_NUM_TOKENS + 1]
        grad = ctx.plan.backward(g_scale=g_loss, g_elem=None, aggregate=True, n_valid=n_valid)
        return grad, None


def elem_loss(new_logp: torch.Tensor, plan: RatioLossPlan) -> Tuple[torch.Tensor, torch.Tensor]:
    if torch.is_grad_enabled() and new_logp.requires_grad:
        elem, metrics = _ElemLossFn.apply(new_logp, plan)
    else:
        elem, metrics = plan.forward(want_elem=True)
    if elem.dtype != new_logp.dtype:
        elem = elem.to(new_logp.dtype)
    return elem, metrics


def scalar_loss(new_logp: torch.Tensor, plan: RatioLossPlan) -> Tuple[torch.Tensor, torch.Tensor]:
    if torch.is_grad_enabled() and new_logp.requires_grad:
        return _ScalarLossFn.apply(new_logp, plan)
    _, metrics = plan.forward(want_elem=False)
    return metrics[N.M_LOSS], metrics


def fused_token_loss_backward(
    kind: str,
    new_logp: torch.Tensor,
    old_logp: torch.Tensor,
    advantages: torch.Tensor,
    *,
    loss_scale: float,
    lengths: Optional[torch.Tensor] = None,
    cu_seqlens: Optional[torch.Tensor] = None,
    loss_mask: Optional[torch.Tensor] = None,
    loss_agg_mode: str = "token-mean",
    horizon: int = 8192,
    clip_range: float = 0.2,
    clip_range_high: Optional[float] = None,
    drpo_epsilon: float = 12.5,
    mu_weighted: bool = True,
    adv_per_token: Optional[bool] = None,
) -> torch.Tensor:
    """``(loss * loss_scale).backward()`` of :func:`fused_token_loss` without building the loss
    in autograd: one kernel reads ``new_logp`` / ``old_logp`` once, reduces the loss and every
    metric and writes the gradient, which is then pushed into ``new_logp``'s graph.  Returns the
    ``[16]`` metrics vector (``M_LOSS`` holds the unscaled loss).  Without a graph behind
    ``new_logp`` only the forward runs."""
    code = {"grpo": N.LOSS_GRPO, "drpo": N.LOSS_DRPO}[kind]
    plan = RatioLossPlan(
        new_logp, old_logp, advantages, kind=code, lengths=lengths, cu_seqlens=cu_seqlens, loss_mask=loss_mask,
        agg_mode=loss_agg_mode, clip_low=clip_range, clip_high=clip_range_high, drpo_epsilon=drpo_epsilon,
        mu_weighted=mu_weighted, horizon=horizon, adv_per_token=adv_per_token,
    )
    if not (torch.is_grad_enabled() and new_logp.requires_grad):
        return plan.forward(want_elem=False)[1]
    grad, metrics = plan.forward_backward(float(loss_scale))
    if grad.dtype != new_logp.dtype:
        grad = grad.to(new_logp.dtype)
    new_logp.backward(grad)
    return metrics


GRPO_METRICS: Dict[str, int] = {
    "ratio_mean": N.M_RATIO_MEAN,
    "ratio_std": N.M_RATIO_STD,
    "ratio_min": N.M_RATIO_MIN,
    "ratio_max": N.M_RATIO_MAX,
    "clip_fraction": N.M_CLIP_FRACTION,
    "clipfrac_gt_one": N.M_CLIPFRAC_HI,
    "clipfrac_lt_one": N.M_CLIPFRAC_LO,
    "approx_kl": N.M_APPROX_KL,
}

DRPO_METRICS: Dict[str, int] = {
    "ratio_mean": N.M_RATIO_MEAN,
    "ratio_max": N.M_RATIO_MAX,
    "approx_kl": N.M_APPROX_KL,
    "drpo_penalty_mean": N.M_PENALTY_MEAN,
    "clipfrac_upper": N.M_CLIPFRAC_HI,
    "clipfrac_lower": N.M_CLIPFRAC_LO,
}

ABSDIFF_METRICS: Dict[str, int] = {
    "rollout_replay_logp_absdiff_mean": N.M_ABSDIFF_MEAN,
    "rollout_replay_logp_absdiff_max": N.M_ABSDIFF_MAX,
}


def metric_tensors(metrics: torch.Tensor, slots: Dict[str, int]) -> Dict[str, torch.Tensor]:
    """0-dim detached views into the metrics vector, keyed by the reference's metric names."""
    m = metrics.detach().unbind(0)  # one call for the sixteen 0-dim views
    return {name: m[slot] for name, slot in slots.items()}


def fused_token_loss(
    kind: str,
    new_logp: torch.Tensor,
    old_logp: torch.Tensor,
    advantages: torch.Tensor,
    *,
    lengths: Optional[torch.Tensor] = None,
    cu_seqlens: Optional[torch.Tensor] = None,
    loss_mask: Optional[torch.Tensor] = None,
    loss_agg_mode: str = "token-mean",
    horizon: int = 8192,
    clip_range: float = 0.2,
    clip_range_high: Optional[float] = None,
    drpo_epsilon: float = 12.5,
    mu_weighted: bool = True,
    adv_per_token: Optional[bool] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Whole micro-batch loss of GRPO / DRPO in one launch.

    ``new_logp`` / ``old_logp`` are padded ``[n_seq, max_len]`` with ``lengths``, packed
    ``[total_tokens]`` with ``cu_seqlens``, or flat with per-token ``advantages``.
    ``advantages`` is per sequence ``[n_seq]`` or per token; a packed batch with as many tokens
    as sequences fits both, and is read per sequence unless ``adv_per_token`` is given.  Returns the differentiable
    scalar loss and the ``[16]`` metrics vector (slots: ``unirl_amd._native.M_*``).
    """
    code = {"grpo": N.LOSS_GRPO, "drpo": N.LOSS_DRPO}[kind]
    plan = RatioLossPlan(
        new_logp, old_logp, advantages, kind=code, lengths=lengths, cu_seqlens=cu_seqlens, loss_mask=loss_mask,
        agg_mode=loss_agg_mode, clip_low=clip_range, clip_high=clip_range_high, drpo_epsilon=drpo_epsilon,
        mu_weighted=mu_weighted, horizon=horizon, adv_per_token=adv_per_token,
    )
    return scalar_loss(new_logp, plan)
