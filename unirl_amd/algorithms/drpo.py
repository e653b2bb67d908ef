"""DRPO token loss (contract of ``unirl/algorithms/drpo.py:97-345``).

Per token: ``L = -A*r + |A| * mu * (r-1)^2 / (2*eps)`` with ``r = exp(clamp(new-old, +-20))``
and ``mu = exp(old)`` (``mu_weighted``) or 1.  ``_drpo_loss`` returns the per-element
loss and the six metrics from one kernel; ``DRPO.compute_loss_and_backward`` fuses
expansion, mask, aggregation and metrics into one forward and one backward launch.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple, Type

import torch

from .. import _native as N
from .. import ops
from ._fused import ABSDIFF_METRICS, DRPO_METRICS, elem_loss, fused_token_loss_backward, metric_tensors
from .base import (
    NO_STEP,
    AlgorithmStepResult,
    BaseAlgorithmConfig,
    StageAlgorithm,
    parse_old_logp_source,
    typed_conditions,
)
from .grpo import _DEFAULT_AR_TEMPERATURE, cu_seqlens_from_lengths


@dataclass
class DRPOConfig(BaseAlgorithmConfig):
    stage_attr: str = "ar"
    conditions_cls: str = ""
    drpo_epsilon: float = 12.5
    penalty_mu_weighted: bool = True
    loss_agg_mode: str = "token-mean"
    horizon: int = 8192
    sampling_temperature: Optional[float] = None
    old_logp_source: str = "rollout"


def _drpo_loss(
    *,
    new_logp: torch.Tensor,
    old_logp: torch.Tensor,
    advantages: torch.Tensor,
    epsilon: float,
    mu_weighted: bool = True,
) -> Tuple[torch.Tensor, Dict[str, torch.Tensor]]:
    """``(loss_per_elem, metrics)``; reduction is the caller's job."""
    adv = advantages.detach()
    if adv.shape != new_logp.shape:
        adv = adv.expand(new_logp.shape)
    plan = ops.RatioLossPlan(
        new_logp, old_logp, adv, kind=N.LOSS_DRPO, drpo_epsilon=epsilon, mu_weighted=mu_weighted
    )
    elem, metrics = elem_loss(new_logp, plan)
    return elem, metric_tensors(metrics, DRPO_METRICS)


class DRPO(StageAlgorithm):
    """Divergence-regularised policy optimisation for token-level policies."""

    def __init__(
        self,
        *,
        pipeline: Any = None,
        stage_attr: str = "ar",
        drpo_epsilon: float = 12.5,
        penalty_mu_weighted: bool = True,
        loss_agg_mode: str = "token-mean",
        horizon: int = 8192,
        sampling_temperature: Optional[float] = None,
        old_logp_source: str = "rollout",
        conditions_cls: Optional[Type[Any]] = None,
    ) -> None:
        if pipeline is None:
            raise ValueError("DRPO: `pipeline` must be provided (the v2 trainer injects it)")
        self.stage = getattr(pipeline, stage_attr)
        self.drpo_epsilon = float(drpo_epsilon)
        self.penalty_mu_weighted = bool(penalty_mu_weighted)
        self.loss_agg_mode = str(loss_agg_mode)
        self.horizon = int(horizon)
        self.sampling_temperature = float(
            _DEFAULT_AR_TEMPERATURE if sampling_temperature is None else sampling_temperature
        )
        self.conditions_cls = conditions_cls
        self.old_logp_source = parse_old_logp_source("DRPO", old_logp_source)
        self.supports_multi_update = True

    def prepare_segment(self, *, conditions: Mapping[str, Any], segment: Any) -> None:
        """``old_logp_source='replay'``: freeze a train-side anchor in ``segment.log_probs``."""
        if self.old_logp_source != "replay":
            return
        if segment.tokens is None or segment.log_probs is None or int(segment.tokens.shape[0]) == 0:
            return
        with torch.no_grad():
            frozen = self.stage.replay(
                typed_conditions(conditions, self.conditions_cls), segment=segment,
                temperature=self.sampling_temperature,
            )
        segment.log_probs = frozen.detach()

    def compute_loss_and_backward(
        self,
        *,
        conditions: Mapping[str, Any],
        segment: Any,
        advantages: torch.Tensor,
        training_progress: float,
        loss_scale: float,
    ) -> AlgorithmStepResult:
        if segment.tokens is None or segment.lengths is None or segment.log_probs is None:
            return NO_STEP
        if int(segment.tokens.shape[0]) == 0:
            return NO_STEP

        new_logp = self.stage.replay(
            typed_conditions(conditions, self.conditions_cls), segment=segment, temperature=self.sampling_temperature
        )
        bs = int(advantages.shape[0])
        if int(segment.lengths.shape[0]) != bs:
            raise ValueError(
                f"GRPO advantage expansion: advantages batch={bs} != lengths={int(segment.lengths.shape[0])}"
            )
        mode = "seq-mean-token-sum-norm" if self.loss_agg_mode == "seq-mean-token-sum-norm" else "token-mean"
        # loss, metrics and `(loss * loss_scale).backward()` in one pass over the tokens
        mvec = fused_token_loss_backward(
            "drpo", new_logp, segment.log_probs, advantages, loss_scale=loss_scale,
            cu_seqlens=cu_seqlens_from_lengths(segment.lengths, new_logp.device),
            loss_mask=getattr(segment, "loss_mask", None), loss_agg_mode=mode, horizon=self.horizon,
            drpo_epsilon=self.drpo_epsilon, mu_weighted=self.penalty_mu_weighted, adv_per_token=False,
        )

        vals = mvec.tolist()
        metrics: Dict[str, Any] = {"policy_loss": vals[N.M_LOSS], "drpo_epsilon": self.drpo_epsilon}
        metrics.update({k: vals[s] for k, s in ABSDIFF_METRICS.items()})
        metrics.update({k: vals[s] for k, s in DRPO_METRICS.items()})
        return AlgorithmStepResult(
            loss=vals[N.M_LOSS], metrics=metrics, num_steps_or_tokens=int(new_logp.shape[0]), has_backward=True
        )


__all__ = ["DRPO", "DRPOConfig"]
