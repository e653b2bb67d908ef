"""FlowGRPO: the clipped ratio on per-step diffusion log-probs ``[B, S']``
(contract of ``unirl/algorithms/flowgrpo.py:67-206``)."""

from __future__ import annotations

from dataclasses import dataclass
from dataclasses import field as dc_field
from typing import Any, Dict, Mapping, Optional, Type

import torch

from .. import _native as N
from ._fused import GRPO_METRICS, fused_token_loss_backward
from .base import (
    NO_STEP,
    AlgorithmStepResult,
    BaseAlgorithmConfig,
    SdeStepAlgorithm,
    _resolve_clip_range_from_schedule,
    gather_sde_field,
)


@dataclass
class FlowGRPOConfig(BaseAlgorithmConfig):
    stage_attr: str = "diffusion"
    conditions_cls: str = ""
    clip_range: float = 1e-4
    clip_schedule: str = "constant"
    old_logp_source: str = "rollout"
    params: Any = dc_field(default=None)


class FlowGRPO(SdeStepAlgorithm):
    """PPO-clip over the SDE steps a diffusion rollout recorded."""

    anchor_fields = ("sde_logp",)

    def __init__(
        self,
        *,
        params: Any,
        stage: Any = None,
        pipeline: Any = None,
        stage_attr: str = "diffusion",
        clip_range: float = 1e-4,
        clip_schedule: str = "constant",
        old_logp_source: str = "rollout",
        conditions_cls: Optional[Type[Any]] = None,
    ) -> None:
        self._setup(params=params, stage=stage, pipeline=pipeline, stage_attr=stage_attr,
                    old_logp_source=old_logp_source, conditions_cls=conditions_cls)
        self.clip_range, self.clip_schedule = float(clip_range), str(clip_schedule)

    def _freeze(self, segment: Any, result: Any) -> None:
        segment.sde_logp = result.log_probs.detach()  # stays on the device; no host bounce

    def compute_loss_and_backward(
        self,
        *,
        conditions: Mapping[str, Any],
        segment: Any,
        advantages: torch.Tensor,
        training_progress: float,
        loss_scale: float,
    ) -> AlgorithmStepResult:
        steps = self._resolve_target_steps(segment)
        if not steps:
            return NO_STEP
        new_logp = self._replay(conditions, segment, steps).log_probs  # [B, S']
        old_logp = gather_sde_field(segment.sde_logp, segment.sde_indices, steps, field_name="sde_logp")
        eps = _resolve_clip_range_from_schedule(self.clip_range, self.clip_schedule, training_progress)
        # every step of sample b shares advantages[b]: the padded layout with S' tokens per row
        rows, n_steps = new_logp.shape
        full = torch.full((rows,), n_steps, dtype=torch.int64)  # host lengths: the token count is known
        mvec = fused_token_loss_backward("grpo", new_logp, old_logp, advantages.detach().reshape(-1),
                                         loss_scale=loss_scale, lengths=full, clip_range=eps, adv_per_token=False)
        vals = mvec.tolist()  # the step's only device-to-host copy
        metrics: Dict[str, Any] = {k: vals[slot] for k, slot in GRPO_METRICS.items()}
        metrics.update(policy_loss=vals[N.M_LOSS], clip_range=float(eps))
        return AlgorithmStepResult(loss=vals[N.M_LOSS], metrics=metrics, num_steps_or_tokens=len(steps),
                                   has_backward=True)


__all__ = ["FlowGRPO", "FlowGRPOConfig"]
