"""FlowGRPO: the clipped ratio on per-step diffusion log-probs ``[B, S']``
(contract of ``unirl/algorithms/flowgrpo.py:67-206``)."""

from __future__ import annotations

from dataclasses import dataclass
from dataclasses import field as dc_field
from typing import Any, Dict, List, Mapping, Optional, Type

import torch

from .. import _native as N
from ._fused import GRPO_METRICS, fused_token_loss
from .base import (
    AlgorithmStepResult,
    BaseAlgorithmConfig,
    StageAlgorithm,
    _resolve_clip_range_from_schedule,
    gather_sde_field,
    typed_conditions,
)


@dataclass
class FlowGRPOConfig(BaseAlgorithmConfig):
    stage_attr: str = "diffusion"
    conditions_cls: str = ""
    clip_range: float = 1e-4
    clip_schedule: str = "constant"
    old_logp_source: str = "rollout"
    params: Any = dc_field(default=None)


class FlowGRPO(StageAlgorithm):
    """PPO-clip over the SDE steps a diffusion rollout recorded."""

    supports_multi_update = True
    anchor_fields = ("sde_logp",)

    def recomputes_anchor(self) -> bool:
        return self.old_logp_source == "replay"

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
        if stage is None and pipeline is None:
            raise ValueError("FlowGRPO: either `stage` or `pipeline` must be provided")
        self.stage = stage if stage is not None else getattr(pipeline, stage_attr)
        self.params = params
        self.clip_range = float(clip_range)
        self.clip_schedule = str(clip_schedule)
        self.old_logp_source = str(old_logp_source).strip().lower()
        if self.old_logp_source not in ("rollout", "replay"):
            raise ValueError(f"FlowGRPO: old_logp_source must be 'rollout' or 'replay'; got {old_logp_source!r}")
        self.conditions_cls = conditions_cls

    def prepare_segment(self, *, conditions: Mapping[str, Any], segment: Any) -> None:
        if segment.sde_indices is None:
            return
        target_steps = self._resolve_target_steps(segment)
        if not target_steps:
            return
        if self.old_logp_source == "rollout":
            if segment.sde_logp is None:
                raise RuntimeError(
                    "FlowGRPO.prepare_segment: old_logp_source='rollout' but the rollout engine emitted no "
                    "per-step log-probs (segment.sde_logp is None). Pin a rollout build that emits trajectory "
                    "log-probs, or set old_logp_source='replay'."
                )
            return
        with torch.no_grad():
            result = self.stage.replay(
                typed_conditions(conditions, self.conditions_cls), segment=segment, params=self.params,
                step_indices=target_steps,
            )
        segment.sde_logp = result.log_probs.detach()

    def compute_loss_and_backward(
        self,
        *,
        conditions: Mapping[str, Any],
        segment: Any,
        advantages: torch.Tensor,
        training_progress: float,
        loss_scale: float,
    ) -> AlgorithmStepResult:
        target_steps = self._resolve_target_steps(segment)
        if not target_steps:
            return AlgorithmStepResult(loss=0.0, metrics={}, num_steps_or_tokens=0, has_backward=False)
        replay = self.stage.replay(
            typed_conditions(conditions, self.conditions_cls), segment=segment, params=self.params,
            step_indices=target_steps,
        )
        new_logp = replay.log_probs  # [B, S']
        old_logp = gather_sde_field(segment.sde_logp, segment.sde_indices, target_steps, field_name="sde_logp")
        clip_range = _resolve_clip_range_from_schedule(self.clip_range, self.clip_schedule, training_progress)
        # every step of sample b shares advantages[b]: the padded layout with full-length rows
        n_steps = new_logp.shape[1]
        lengths = torch.full((new_logp.shape[0],), n_steps, dtype=torch.int64, device=new_logp.device)
        loss, mvec = fused_token_loss(
            "grpo", new_logp, old_logp, advantages.detach().reshape(-1), lengths=lengths, clip_range=clip_range
        )
        (loss * loss_scale).backward()
        vals = mvec.tolist()
        metrics: Dict[str, Any] = {"policy_loss": vals[N.M_LOSS], "clip_range": float(clip_range)}
        metrics.update({k: vals[s] for k, s in GRPO_METRICS.items()})
        return AlgorithmStepResult(
            loss=vals[N.M_LOSS], metrics=metrics, num_steps_or_tokens=len(target_steps), has_backward=True
        )

    def _resolve_target_steps(self, segment: Any) -> List[int]:
        if segment.sde_indices is None:
            return []
        return [int(i) for i in segment.sde_indices.tolist()]


__all__ = ["FlowGRPO", "FlowGRPOConfig"]
