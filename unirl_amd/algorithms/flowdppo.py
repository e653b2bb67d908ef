"""Flow-DPPO: Gaussian-KL trust-region mask on the ratio loss
(contract of ``unirl/algorithms/flowdppo.py:43-368``).

``_flowdppo_kl_adv_loss`` is two launches: the KL of the transition means reduced
per ``(sample, step)`` and thresholded (``unirl_gaussian_kl_mask``, one pass over the
``[B, S', *latent]`` means), then the ``[B, S']`` ratio / mask / metric arithmetic
(``unirl_flowdppo_loss``).  No gradient flows through the KL (the reference detaches
the mask), and ``d loss_elem / d new_logp == loss_elem``.
"""

from __future__ import annotations

from dataclasses import dataclass
from dataclasses import field as dc_field
from typing import Any, Dict, List, Mapping, Optional, Tuple, Type

import torch

from .. import ops
from .base import AlgorithmStepResult, BaseAlgorithmConfig, StageAlgorithm, gather_sde_field, typed_conditions


@dataclass
class FlowDPPOConfig(BaseAlgorithmConfig):
    stage_attr: str = "diffusion"
    conditions_cls: str = ""
    kl_mask_threshold: float = 1e-5
    add_kl_coefficient: bool = True
    old_logp_source: str = "rollout"
    params: Any = dc_field(default=None)


def _sigma_axis(p: torch.Tensor, sigma: torch.Tensor) -> Optional[int]:
    """The single axis along which ``sigma`` varies when broadcast against ``p`` (None = scalar)."""
    if sigma.numel() == 1:
        return None
    if sigma.dim() > p.dim():
        raise ValueError(f"sigma {tuple(sigma.shape)} has more dims than the means {tuple(p.shape)}")
    shape = (1,) * (p.dim() - sigma.dim()) + tuple(sigma.shape)
    axes = [i for i, n in enumerate(shape) if n != 1]
    if len(axes) != 1 or shape[axes[0]] != p.shape[axes[0]]:
        raise ValueError(
            f"sigma {tuple(sigma.shape)} must vary along exactly one axis of the means {tuple(p.shape)}"
        )
    return axes[0]


def _gaussian_kl_div(p: torch.Tensor, q: torch.Tensor, sigma: torch.Tensor) -> torch.Tensor:
    """Per-element ``(p - q)^2 / (2 sigma^2)`` (fp32; 16-bit inputs subtract and square in
    their own dtype first, as torch's type promotion does)."""
    axis = _sigma_axis(p, sigma)
    return ops.gaussian_kl_elem(p, q, sigma, sigma_dim=1 if axis is None else axis)


class _MaskedRatioLossFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, new_logp, old_logp, advantages, kl, threshold):
        elem, metrics = ops.flowdppo_loss(new_logp, old_logp, advantages, kl, threshold)
        ctx.save_for_backward(elem)
        ctx.mark_non_differentiable(metrics)
        return elem, metrics

    @staticmethod
    def backward(ctx, g_elem, _g_metrics):
        (elem,) = ctx.saved_tensors
        return g_elem * elem, None, None, None, None


def _flowdppo_kl_adv_loss(
    *,
    new_logp: torch.Tensor,
    old_logp: torch.Tensor,
    new_means: torch.Tensor,
    old_means: torch.Tensor,
    advantages: torch.Tensor,
    sigma_t: torch.Tensor,
    kl_mask_threshold: float,
) -> Tuple[torch.Tensor, Dict[str, torch.Tensor]]:
    """KL-ADV masked loss per element ``[B, S']`` and the twelve logged metrics."""
    if new_means.dim() < 3:
        raise ValueError(f"means need [B, S', ...latent]; got {tuple(new_means.shape)}")
    axis = _sigma_axis(new_means, sigma_t)
    if axis not in (None, 1):
        raise ValueError(f"sigma_t {tuple(sigma_t.shape)} must be a scalar or vary along the step axis (dim 1)")
    kl, _ = ops.gaussian_kl_mask(new_means, old_means, sigma_t, kl_mask_threshold, reduce_from_dim=2, want_mask=False)
    if torch.is_grad_enabled() and new_logp.requires_grad:
        elem, mvec = _MaskedRatioLossFn.apply(new_logp, old_logp, advantages, kl, float(kl_mask_threshold))
    else:
        elem, mvec = ops.flowdppo_loss(new_logp, old_logp, advantages, kl, float(kl_mask_threshold))
    if elem.dtype != new_logp.dtype:
        elem = elem.to(new_logp.dtype)
    m = mvec.detach()
    metrics = {name: m[slot] for name, slot in ops.FLOWDPPO_METRIC_SLOTS.items() if name != "loss_mean"}
    return elem, metrics


class FlowDPPO(StageAlgorithm):
    """KL-divergence masking in place of ratio clipping for diffusion RL."""

    supports_multi_update = True
    anchor_fields = ("sde_logp", "sde_means")

    def recomputes_anchor(self) -> bool:
        return True

    def __init__(
        self,
        *,
        params: Any,
        stage: Any = None,
        pipeline: Any = None,
        stage_attr: str = "diffusion",
        kl_mask_threshold: float = 1e-5,
        add_kl_coefficient: bool = True,
        old_logp_source: str = "rollout",
        conditions_cls: Optional[Type[Any]] = None,
    ) -> None:
        if stage is None and pipeline is not None:
            stage = getattr(pipeline, stage_attr)
        if stage is None:
            raise ValueError("FlowDPPO: either `stage` or `pipeline` must be provided")
        self.stage = stage
        self.params = params
        self.kl_mask_threshold = float(kl_mask_threshold)
        self.add_kl_coefficient = bool(add_kl_coefficient)
        self.old_logp_source = str(old_logp_source).strip().lower()
        if self.old_logp_source not in ("rollout", "replay"):
            raise ValueError(f"FlowDPPO: old_logp_source must be 'rollout' or 'replay'; got {old_logp_source!r}")
        self.conditions_cls = conditions_cls

    def prepare_segment(self, *, conditions: Mapping[str, Any], segment: Any) -> None:
        """Freeze the old policy's means (always) and log-probs (``'replay'``) on the segment.
        They stay on the device they were computed on."""
        if segment.sde_indices is None:
            return
        target_steps = self._resolve_target_steps(segment)
        if not target_steps:
            return
        if self.old_logp_source == "rollout" and segment.sde_logp is None:
            raise RuntimeError(
                "FlowDPPO.prepare_segment: old_logp_source='rollout' but the rollout engine emitted no "
                "per-step log-probs (segment.sde_logp is None). Pin a rollout build that emits trajectory "
                "log-probs, or set old_logp_source='replay'."
            )
        with torch.no_grad():
            result = self.stage.replay(
                typed_conditions(conditions, self.conditions_cls), segment=segment, params=self.params,
                step_indices=target_steps,
            )
        if self.old_logp_source == "replay":
            segment.sde_logp = result.log_probs.detach()
        if result.prev_sample_means is None:
            raise RuntimeError(
                "FlowDPPO.prepare_segment: stage.replay() returned prev_sample_means=None. Ensure the "
                "stage's replay method produces means (required for KL-ADV masking)."
            )
        segment.sde_means = result.prev_sample_means.detach()

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
        new_logp, new_means = replay.log_probs, replay.prev_sample_means
        if new_means is None:
            raise RuntimeError(
                "FlowDPPO requires stage.replay() to return prev_sample_means, but got None. "
                "Ensure the stage's replay method produces means."
            )
        device = new_logp.device
        old_logp = gather_sde_field(segment.sde_logp, segment.sde_indices, target_steps, field_name="sde_logp").to(
            dtype=new_logp.dtype, device=device
        )
        old_means = gather_sde_field(segment.sde_means, segment.sde_indices, target_steps, field_name="sde_means").to(
            dtype=new_means.dtype, device=new_means.device
        )
        sigma_t = self._compute_sigma_t(segment, target_steps, device=device)
        adv_b = advantages.detach().to(dtype=new_logp.dtype, device=device).reshape(-1, 1).expand_as(new_logp)

        elem, mvec = self._loss_with_metrics(new_logp, old_logp, new_means, old_means, adv_b, sigma_t)
        loss = elem.mean()
        (loss * loss_scale).backward()

        vals = mvec.tolist()
        slots = ops.FLOWDPPO_METRIC_SLOTS
        metrics: Dict[str, Any] = {
            "policy_loss": vals[slots["loss_mean"]],
            "kl_mask_threshold": float(self.kl_mask_threshold),
        }
        metrics.update({k: vals[s] for k, s in slots.items() if k != "loss_mean"})
        return AlgorithmStepResult(
            loss=vals[slots["loss_mean"]], metrics=metrics, num_steps_or_tokens=len(target_steps), has_backward=True
        )

    def _loss_with_metrics(self, new_logp, old_logp, new_means, old_means, adv_b, sigma_t):
        kl, _ = ops.gaussian_kl_mask(
            new_means, old_means, sigma_t, self.kl_mask_threshold, reduce_from_dim=2, want_mask=False
        )
        return _MaskedRatioLossFn.apply(new_logp, old_logp, adv_b, kl, self.kl_mask_threshold)

    def _resolve_target_steps(self, segment: Any) -> List[int]:
        if segment.sde_indices is None:
            return []
        return [int(i) for i in segment.sde_indices.tolist()]

    def _compute_sigma_t(self, segment: Any, target_steps: List[int], device: torch.device) -> torch.Tensor:
        """``std_dev_t * sqrt(-dt)`` per target step, ``[1, S', 1, 1, 1]`` (ones when
        ``add_kl_coefficient`` is off).  ``S'`` scalars, evaluated with the reference's fp32
        operation order on the device the schedule lives on."""
        if not self.add_kl_coefficient:
            return torch.ones(1, len(target_steps), 1, 1, 1, device=device)
        if segment.sigmas is None:
            raise ValueError("FlowDPPO with add_kl_coefficient=True requires segment.sigmas.")
        sigmas = segment.sigmas.detach().to(dtype=torch.float32)  # stays where the schedule lives
        eta = float(self.params.eta)
        idx = torch.tensor(target_steps, dtype=torch.long, device=sigmas.device)
        s, s_next = sigmas[idx], sigmas[idx + 1]
        std_dev_t = torch.sqrt(s / (1.0 - torch.clamp(s, max=0.99))) * eta
        return (std_dev_t * torch.sqrt(-(s_next - s))).reshape(1, -1, 1, 1, 1).to(device)


__all__ = ["FlowDPPO", "FlowDPPOConfig"]
