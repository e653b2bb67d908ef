"""GRPO over a packed ``TextSegment`` (contract of ``unirl/algorithms/grpo.py:40-198``).

``stage.replay`` still owns the teacher-forced forward; everything after it --
advantage expansion (:172-198), the clipped ratio (base.py:115-157), the
aggregation mode (:148-155), the drift gauge, all metric reductions and the
gradient that ``(loss * loss_scale).backward()`` sends into ``new_logp`` -- is one
kernel that reads the tokens once.  The metrics reach the host with a single
device-to-host copy instead of one ``.item()`` each.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Type

import torch

from .. import _native as N
from .. import ops
from ._fused import ABSDIFF_METRICS, GRPO_METRICS, fused_token_loss_backward
from .base import (
    NO_STEP,
    AlgorithmStepResult,
    BaseAlgorithmConfig,
    StageAlgorithm,
    _resolve_clip_range_from_schedule,
    bind_stage,
    typed_conditions,
)

# ARSamplingParams.temperature default of the reference (unirl/types/sampling.py:136)
_DEFAULT_AR_TEMPERATURE = 0.7


@dataclass
class GRPOConfig(BaseAlgorithmConfig):
    stage_attr: str = "ar"
    conditions_cls: str = ""
    clip_range: float = 1e-4
    clip_schedule: str = "constant"


def cu_seqlens_from_lengths(lengths: torch.Tensor, device: torch.device) -> torch.Tensor:
    """``[n_seq + 1]`` int64 prefix sum of ``lengths`` on ``device``."""
    lens = lengths.detach().to(device=device, dtype=torch.int64).reshape(-1)
    cu = torch.zeros(lens.numel() + 1, dtype=torch.int64, device=device)
    torch.cumsum(lens, dim=0, out=cu[1:])
    return cu


class GRPO(StageAlgorithm):
    """Token-level clipped-ratio policy loss via ``ARStage.replay``."""

    supports_multi_update = True

    def __init__(
        self,
        *,
        stage: Any = None,
        pipeline: Any = None,
        stage_attr: str = "ar",
        clip_range: float = 1e-4,
        clip_schedule: str = "constant",
        clip_range_high: Optional[float] = None,
        loss_agg_mode: str = "token-mean",
        horizon: int = 8192,
        conditions_cls: Optional[Type[Any]] = None,
        sampling_temperature: Optional[float] = None,
    ) -> None:
        self.stage = bind_stage("GRPO", stage, pipeline, stage_attr)
        self.clip_range = float(clip_range)
        self.clip_range_high = None if clip_range_high is None else float(clip_range_high)
        self.clip_schedule = str(clip_schedule)
        self.loss_agg_mode = str(loss_agg_mode)
        self.horizon = int(horizon)
        self.conditions_cls = conditions_cls
        self.sampling_temperature = float(
            _DEFAULT_AR_TEMPERATURE if sampling_temperature is None else sampling_temperature
        )

    def compute_loss_and_backward(
        self,
        *,
        conditions: Mapping[str, Any],
        segment: Any,
        advantages: torch.Tensor,
        training_progress: float,
        loss_scale: float,
    ) -> AlgorithmStepResult:
        stored = (segment.tokens, segment.lengths, segment.log_probs)
        if any(t is None for t in stored) or int(segment.tokens.shape[0]) == 0:
            return NO_STEP  # nothing recorded for this stage, or an empty micro-batch

        new_logp = self.stage.replay(
            typed_conditions(conditions, self.conditions_cls), segment=segment, temperature=self.sampling_temperature
        )  # [total_tokens]
        bs = int(advantages.shape[0])
        if int(segment.lengths.shape[0]) != bs:
            raise ValueError(
                f"GRPO advantage expansion: advantages batch={bs} != lengths={int(segment.lengths.shape[0])}"
            )
        # both epsilons follow the schedule; no upper epsilon means a symmetric clip
        clip_range, clip_high = (
            None if eps is None else _resolve_clip_range_from_schedule(eps, self.clip_schedule, training_progress)
            for eps in (self.clip_range, self.clip_range_high)
        )
        mode = self.loss_agg_mode
        if mode not in ("seq-mean-token-sum-norm", "seq-mean-token-mean"):
            mode = "token-mean"
        # loss, metrics and `(loss * loss_scale).backward()` in one pass over the tokens
        mvec = fused_token_loss_backward(
            "grpo", new_logp, segment.log_probs, advantages, loss_scale=loss_scale,
            cu_seqlens=cu_seqlens_from_lengths(segment.lengths, new_logp.device), loss_agg_mode=mode,
            horizon=self.horizon, clip_range=clip_range, clip_range_high=clip_high, adv_per_token=False,
        )

        vals = mvec.tolist()  # the step's only device-to-host copy
        metrics: Dict[str, Any] = {"policy_loss": vals[N.M_LOSS], "clip_range": float(clip_range)}
        metrics.update({k: vals[s] for k, s in ABSDIFF_METRICS.items()})
        metrics.update({k: vals[s] for k, s in GRPO_METRICS.items()})
        return AlgorithmStepResult(
            loss=vals[N.M_LOSS], metrics=metrics, num_steps_or_tokens=int(new_logp.shape[0]), has_backward=True
        )

    @staticmethod
    def _expand_advantages_to_tokens(
        advantages: torch.Tensor, lengths: torch.Tensor, *, dtype: torch.dtype, device: torch.device
    ) -> torch.Tensor:
        """Per-sample ``advantages [B]`` repeated over each sample's ``lengths[k]`` tokens."""
        bs = int(advantages.shape[0])
        if int(lengths.shape[0]) != bs:
            raise ValueError(f"GRPO advantage expansion: advantages batch={bs} != lengths={int(lengths.shape[0])}")
        device = torch.device(device)
        if device.type != "cuda":
            raise RuntimeError("GRPO._expand_advantages_to_tokens: the expansion kernel needs a HIP device")
        cu = cu_seqlens_from_lengths(lengths, device)
        n_tok = int(cu[-1].item()) if bs else 0
        if n_tok == 0:
            return torch.zeros(0, dtype=dtype, device=device)
        out = ops.expand_per_seq(advantages.detach().to(device=device, dtype=torch.float32), cu, n_tok)
        return out if dtype == torch.float32 else out.to(dtype)


__all__ = ["GRPO", "GRPOConfig", "cu_seqlens_from_lengths"]
