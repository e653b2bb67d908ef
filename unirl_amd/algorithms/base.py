"""Shared loss helpers and the stage-algorithm contract.

Keeps the call signatures of ``unirl/algorithms/base.py``:
``gather_sde_field`` (:46-80), ``rollout_replay_logp_absdiff`` (:83-103),
``_resolve_clip_range_from_schedule`` (:106-112), ``_grpo_clip_loss`` (:115-157),
``AlgorithmStepResult`` (:160-171) and the ``StageAlgorithm`` hooks (:182-298).
The element-wise chain and its eight metric reductions are one kernel launch
(``unirl_ratio_loss_fwd``); autograd gets a one-kernel backward.
"""

from __future__ import annotations

import math
from abc import ABC, abstractmethod
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple, Type

import torch

from .. import _native as N
from .. import ops
from ._fused import ABSDIFF_METRICS, GRPO_METRICS, elem_loss, metric_tensors


def typed_conditions(conditions: Mapping[str, Any], conditions_cls: Optional[Type[Any]]) -> Any:
    """The stage's typed conditions container, or the mapping itself when no class is given."""
    return conditions if conditions_cls is None else conditions_cls.from_dict(dict(conditions))


def gather_sde_field(
    tensor: Optional[torch.Tensor],
    sde_indices: Optional[torch.Tensor],
    target_steps: List[int],
    *,
    field_name: str = "field",
) -> torch.Tensor:
    """``tensor[:, slots]`` where ``slots`` are the positions of ``target_steps`` in ``sde_indices``.

    ``sde_indices`` need not be sorted.  A device tensor is gathered by one copy kernel;
    a host tensor is indexed where its bytes are (the caller uploads only the gathered
    slices, as the reference does).  When the targets are all recorded steps in recorded order
    the tensor itself is returned (callers only read the result).
    """
    if tensor is None or sde_indices is None:
        raise ValueError(
            f"gather_sde_field: {field_name} or sde_indices is None "
            f"(ensure prepare_segment ran before compute_loss_and_backward)."
        )
    recorded = [int(i) for i in sde_indices.tolist()]
    slot_of: Dict[int, int] = {}
    for slot, step in enumerate(recorded):
        slot_of.setdefault(step, slot)
    missing = [int(t) for t in target_steps if int(t) not in slot_of]
    if missing:
        raise ValueError(
            f"gather_sde_field({field_name}): target steps {missing} not in sde_indices={sorted(recorded)}"
        )
    positions = [slot_of[int(t)] for t in target_steps]
    if positions == list(range(int(tensor.shape[1]))):
        return tensor  # every recorded step, in recorded order: nothing to move
    if tensor.is_cuda:
        return ops.gather_steps(tensor, positions)
    return tensor[:, positions]


def rollout_replay_logp_absdiff(new_logp: torch.Tensor, old_logp: torch.Tensor) -> Dict[str, float]:
    """``mean|new-old|`` and ``max|new-old|`` over all tokens, as python floats (one sync)."""
    with torch.no_grad():
        flat_new = new_logp.detach().reshape(-1)
        # advantages only feed the loss; reuse new_logp as a same-shape stand-in
        plan = ops.RatioLossPlan(flat_new, old_logp.detach().reshape(-1), flat_new, kind=N.LOSS_GRPO)
        _, metrics = plan.forward(want_elem=False)
        mean_v, max_v = metrics[N.M_ABSDIFF_MEAN : N.M_ABSDIFF_MAX + 1].tolist()
    return {"rollout_replay_logp_absdiff_mean": float(mean_v), "rollout_replay_logp_absdiff_max": float(max_v)}


def _resolve_clip_range_from_schedule(clip_range: float, schedule: str, progress: float) -> float:
    if schedule == "linear_decay":
        return clip_range * (1.0 - 0.5 * float(progress))
    if schedule == "cosine_decay":
        return clip_range * (0.5 * (1.0 + math.cos(math.pi * float(progress))))
    return clip_range


def _grpo_clip_loss(
    *,
    new_logp: torch.Tensor,
    old_logp: torch.Tensor,
    advantages: torch.Tensor,
    clip_range: float,
    clip_range_high: Optional[float] = None,
) -> Tuple[torch.Tensor, Dict[str, torch.Tensor]]:
    """PPO clipped objective per element plus the ratio metrics.

    ``clip_range`` is the lower epsilon, ``clip_range_high`` the upper one (``None`` =
    symmetric).  Returns ``(loss_per_elem, metrics)``; ``loss_per_elem`` is differentiable
    w.r.t. ``new_logp`` and the metrics are detached 0-dim tensors.
    """
    adv = advantages.detach()
    if adv.shape != new_logp.shape:
        adv = adv.expand(new_logp.shape)
    plan = ops.RatioLossPlan(
        new_logp, old_logp, adv, kind=N.LOSS_GRPO, clip_low=clip_range, clip_high=clip_range_high
    )
    elem, metrics = elem_loss(new_logp, plan)
    return elem, metric_tensors(metrics, GRPO_METRICS)


@dataclass(frozen=True)
class AlgorithmStepResult:
    """One micro-step: scalar loss, logged metrics, step / token count, whether backward ran."""

    loss: float
    metrics: Mapping[str, Any]
    num_steps_or_tokens: int
    has_backward: bool


class BaseAlgorithmConfig(ABC):
    """Marker base of the per-stage algorithm config dataclasses."""


class StageAlgorithm(ABC):
    """``(conditions, segment, advantages) -> loss``; holds the stage whose ``replay`` it calls."""

    requires_ema_rollout: bool = False
    supports_multi_update: bool = False
    anchor_fields: Tuple[str, ...] = ()

    def recomputes_anchor(self) -> bool:
        return False

    def prepare_segment(self, *, conditions: Mapping[str, Any], segment: Any) -> None:
        return None

    @abstractmethod
    def compute_loss_and_backward(
        self,
        *,
        conditions: Mapping[str, Any],
        segment: Any,
        advantages: torch.Tensor,
        training_progress: float,
        loss_scale: float,
    ) -> AlgorithmStepResult:
        ...


NO_STEP = AlgorithmStepResult(loss=0.0, metrics={}, num_steps_or_tokens=0, has_backward=False)


def bind_stage(owner: str, stage: Any, pipeline: Any, stage_attr: str) -> Any:
    """The stage an algorithm drives: given directly, or looked up on a pipeline."""
    if stage is not None:
        return stage
    if pipeline is None:
        raise ValueError(f"{owner}: either `stage` or `pipeline` must be provided")
    return getattr(pipeline, stage_attr)


def parse_old_logp_source(owner: str, value: Any) -> str:
    source = str(value).strip().lower()
    if source not in ("rollout", "replay"):
        raise ValueError(f"{owner}: old_logp_source must be 'rollout' or 'replay'; got {value!r}")
    return source


class SdeStepAlgorithm(StageAlgorithm):
    """Shared plumbing of the diffusion algorithms that train on the SDE steps a rollout recorded
    (FlowGRPO, FlowDPPO): which steps, how the stage is replayed on them, and how the old
    policy's per-step quantities are frozen on the segment before the update loop.

    Subclasses set ``anchor_fields``, implement ``_freeze(segment, replay_result)`` and the loss.
    ``_needs_replay_for_anchor`` says whether ``prepare_segment`` must replay even when the
    rollout's own log-probs are trusted (FlowDPPO: always, for the means).
    """

    supports_multi_update = True
    _needs_replay_for_anchor = False
    stage: Any
    params: Any
    conditions_cls: Optional[Type[Any]]
    old_logp_source: str

    def _setup(self, *, params, stage, pipeline, stage_attr, old_logp_source, conditions_cls) -> None:
        owner = type(self).__name__
        self.stage = bind_stage(owner, stage, pipeline, stage_attr)
        self.params = params
        self.old_logp_source = parse_old_logp_source(owner, old_logp_source)
        self.conditions_cls = conditions_cls

    def recomputes_anchor(self) -> bool:
        return self._needs_replay_for_anchor or self.old_logp_source == "replay"

    def _resolve_target_steps(self, segment: Any) -> List[int]:
        """Every SDE step the rollout recorded; subclasses may filter."""
        indices = segment.sde_indices
        return [] if indices is None else [int(i) for i in indices.tolist()]

    def _velocity_replay(self, conditions: Mapping[str, Any], segment: Any, steps: List[int]) -> Optional[Dict[str, Any]]:
        """The operands of a batched replay, when the stage can hand over the model's velocities of
        all target steps at once instead of looping ``denoise`` itself.

        Opt-in protocol (no counterpart in the reference, whose stages loop step by step,
        ``unirl/models/sd3/diffusion.py:467-497``): a stage with a ``replay_velocities(conditions, *,
        segment, params, step_indices)`` method returns an object whose ``noise_pred`` holds the
        velocities as ``[B, S', ...]`` (or ``[S', B, ...]`` with ``step_major=True``: a model pass
        over the steps stacked into the batch); its SDE strategy is ``stage.strategy`` (or the
        result's ``strategy``).  Everything else is read from the segment as the reference's loop
        reads it: ``latents_at(step)`` / ``latents_at(step + 1)`` become slot tables into
        ``segment.latents``, sigma pairs come from ``segment.sigmas``, ``sigma_max = sigmas[1]``.
        Returns ``None`` for a stage without the method."""
        hook = getattr(self.stage, "replay_velocities", None)
        if hook is None:
            return None
        from ..sde.kernels import replay_slots

        out = hook(typed_conditions(conditions, self.conditions_cls), segment=segment, params=self.params,
                   step_indices=steps)
        v = out.noise_pred
        strategy = getattr(out, "strategy", None) or getattr(self.stage, "strategy", None)
        if strategy is None or getattr(strategy, "_kind", None) is None:
            raise RuntimeError(f"{type(self).__name__}: replay_velocities needs a stage.strategy with a fused SDE kernel")
        device = v.device
        latents = segment.latents if segment.latents.device == device else segment.latents.to(device)
        sigmas = segment.sigmas.detach().to(device=device, dtype=torch.float32)
        idx = torch.tensor(steps, dtype=torch.long, device=device)
        slot_x, slot_p = replay_slots(segment.indices, steps)
        return dict(
            noise_pred=v, latents=latents, slot_sample=slot_x, slot_prev=slot_p, sigma=sigmas[idx], sigma_next=sigmas[idx + 1],
            sigma_max=sigmas[1] if int(sigmas.shape[0]) > 1 else 0.99, eta=float(self.params.eta), strategy=strategy,
            step_major=bool(getattr(out, "step_major", False)),
        )

    def _replay(self, conditions: Mapping[str, Any], segment: Any, steps: List[int]) -> Any:
        vr = self._velocity_replay(conditions, segment, steps)
        if vr is not None:
            # every (sample, step) transition in one launch pair, differentiable w.r.t. the velocities
            import types

            lp, means = vr["strategy"].replay_steps(
                vr["noise_pred"], vr["latents"], vr["slot_sample"], vr["slot_prev"], vr["sigma"], vr["sigma_next"],
                eta=vr["eta"], sigma_max=vr["sigma_max"], step_major=vr["step_major"])
            return types.SimpleNamespace(log_probs=lp, prev_sample_means=means)
        return self.stage.replay(
            typed_conditions(conditions, self.conditions_cls), segment=segment, params=self.params, step_indices=steps
        )

    def _freeze(self, segment: Any, result: Any) -> None:
        raise NotImplementedError

    def prepare_segment(self, *, conditions: Mapping[str, Any], segment: Any) -> None:
        steps = self._resolve_target_steps(segment)
        if not steps:
            return
        if self.old_logp_source == "rollout" and segment.sde_logp is None:
            raise RuntimeError(
                f"{type(self).__name__}.prepare_segment: old_logp_source='rollout' but the rollout engine emitted no "
                "per-step log-probs (segment.sde_logp is None). Pin a rollout build that emits trajectory "
                "log-probs, or set old_logp_source='replay'."
            )
        if not self.recomputes_anchor():
            return
        with torch.no_grad():
            self._freeze(segment, self._replay(conditions, segment, steps))


__all__ = [
    "ABSDIFF_METRICS",
    "AlgorithmStepResult",
    "BaseAlgorithmConfig",
    "NO_STEP",
    "SdeStepAlgorithm",
    "StageAlgorithm",
    "bind_stage",
    "parse_old_logp_source",
    "gather_sde_field",
    "rollout_replay_logp_absdiff",
    "typed_conditions",
]
