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
from .base import NO_STEP, AlgorithmStepResult, BaseAlgorithmConfig, SdeStepAlgorithm, gather_sde_field


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


class _KlElemFn(torch.autograd.Function):
    """Element-wise KL with gradients to both means (sigma is treated as a constant)."""

    @staticmethod
    def forward(ctx, p, q, sigma, sigma_dim):
        ctx.save_for_backward(p.detach(), q.detach(), sigma.detach())
        ctx.sigma_dim = sigma_dim
        ctx.dtypes = (p.dtype, q.dtype)
        return ops.gaussian_kl_elem(p, q, sigma, sigma_dim=sigma_dim)

    @staticmethod
    def backward(ctx, g_out):
        p, q, sigma = ctx.saved_tensors
        gp, gq = ops.gaussian_kl_elem_bwd(
            p, q, sigma, g_out, sigma_dim=ctx.sigma_dim, need_p=ctx.needs_input_grad[0],
            need_q=ctx.needs_input_grad[1],
        )
        if gp is not None:
            gp = gp.reshape(p.shape).to(ctx.dtypes[0])
        if gq is not None:
            gq = gq.reshape(q.shape).to(ctx.dtypes[1])
        return gp, gq, None, None


def _gaussian_kl_div(p: torch.Tensor, q: torch.Tensor, sigma: torch.Tensor) -> torch.Tensor:
    """Per-element ``(p - q)^2 / (2 sigma^2)`` (fp32; 16-bit inputs subtract and square in
    their own dtype first, as torch's type promotion does).  Differentiable w.r.t. ``p`` and ``q``.
    The result is always fp32: with a 0-dim ``sigma`` eager torch would keep a 16-bit result
    (0-dim tensors do not promote); the reference always passes ``[1, S', 1, 1, 1]``."""
    axis = _sigma_axis(p, sigma)
    sigma_dim = 1 if axis is None else axis
    if torch.is_grad_enabled() and (p.requires_grad or q.requires_grad):
        return _KlElemFn.apply(p, q, sigma, sigma_dim)
    return ops.gaussian_kl_elem(p, q, sigma, sigma_dim=sigma_dim)


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


class _MaskedRatioStepFn(torch.autograd.Function):
    """The same loss with the KL over the means in the same call (``unirl_flowdppo_step``: the
    streaming KL kernel plus one finishing workgroup -- two launches instead of three)."""

    @staticmethod
    def forward(ctx, new_logp, old_logp, new_means, old_means, advantages, sigma_t, threshold):
        _, elem, metrics, _ = ops.flowdppo_step(new_logp, old_logp, new_means, old_means, advantages, sigma_t, threshold)
        ctx.save_for_backward(elem)
        ctx.mark_non_differentiable(metrics)
        return elem, metrics

    @staticmethod
    def backward(ctx, g_elem, _g_metrics):
        (elem,) = ctx.saved_tensors  # d(-A r)/d new_logp = -A r where kept, 0 where masked: the loss itself
        return g_elem * elem, None, None, None, None, None, None


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
    threshold = float(kl_mask_threshold)
    needs_grad = torch.is_grad_enabled() and new_logp.requires_grad
    rows = new_logp.numel()
    if new_logp.dim() == 2 and tuple(new_means.shape[:2]) == tuple(new_logp.shape) and 0 < rows <= ops.FLOWDPPO_STEP_MAX_ROWS:
        # the usual [B, S'] problem: KL, masks, loss and metrics as one call of two launches
        if needs_grad:
            elem, mvec = _MaskedRatioStepFn.apply(new_logp, old_logp, new_means, old_means, advantages, sigma_t, threshold)
        else:
            _, elem, mvec, _ = ops.flowdppo_step(new_logp, old_logp, new_means, old_means, advantages, sigma_t, threshold)
    else:
        kl, _ = ops.gaussian_kl_mask(new_means, old_means, sigma_t, threshold, reduce_from_dim=2, want_mask=False)
        if needs_grad:
            elem, mvec = _MaskedRatioLossFn.apply(new_logp, old_logp, advantages, kl, threshold)
        else:
            elem, mvec = ops.flowdppo_loss(new_logp, old_logp, advantages, kl, threshold)
    if elem.dtype != new_logp.dtype:
        elem = elem.to(new_logp.dtype)
    m = mvec.detach().unbind(0)  # one call for the sixteen 0-dim views
    metrics = {name: m[slot] for name, slot in ops.FLOWDPPO_METRIC_SLOTS.items() if name != "loss_mean"}
    return elem, metrics


class FlowDPPO(SdeStepAlgorithm):
    """KL-divergence masking in place of ratio clipping for diffusion RL."""

    anchor_fields = ("sde_logp", "sde_means")
    _needs_replay_for_anchor = True  # the old policy's means exist only after a replay

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
        self._setup(params=params, stage=stage, pipeline=pipeline, stage_attr=stage_attr,
                    old_logp_source=old_logp_source, conditions_cls=conditions_cls)
        self.kl_mask_threshold = float(kl_mask_threshold)
        self.add_kl_coefficient = bool(add_kl_coefficient)

    def _freeze(self, segment: Any, result: Any) -> None:
        """Old means always, old log-probs only under ``'replay'``; both stay on the device."""
        if result.prev_sample_means is None:
            raise RuntimeError(
                "FlowDPPO.prepare_segment: stage.replay() returned prev_sample_means=None. Ensure the "
                "stage's replay method produces means (required for KL-ADV masking)."
            )
        if self.old_logp_source == "replay":
            segment.sde_logp = result.log_probs.detach()
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
        del training_progress
        steps = self._resolve_target_steps(segment)
        if not steps:
            return NO_STEP
        fused = self._step_from_velocities(conditions, segment, steps, advantages, loss_scale)
        if fused is not None:
            return fused
        replay = self._replay(conditions, segment, steps)
        new_logp, new_means = replay.log_probs, replay.prev_sample_means
        if new_means is None:
            raise RuntimeError(
                "FlowDPPO requires stage.replay() to return prev_sample_means, but got None. "
                "Ensure the stage's replay method produces means."
            )
        device = new_logp.device

        def frozen(name, like):
            t = gather_sde_field(getattr(segment, name), segment.sde_indices, steps, field_name=name)
            return t.to(dtype=like.dtype, device=like.device)

        old_logp, old_means = frozen("sde_logp", new_logp), frozen("sde_means", new_means)
        sigma_t = self._compute_sigma_t(segment, steps, device=device)
        adv_b = advantages.detach().to(dtype=new_logp.dtype, device=device).reshape(-1, 1).expand_as(new_logp)

        if new_logp.dim() == 2 and 0 < new_logp.numel() <= ops.FLOWDPPO_STEP_MAX_ROWS:
            # KL, masks, loss, metrics and `(elem.mean() * loss_scale).backward()` in two launches
            need_grad = torch.is_grad_enabled() and new_logp.requires_grad
            _, _, mvec, grad = ops.flowdppo_step(
                new_logp, old_logp, new_means, old_means, adv_b, sigma_t, self.kl_mask_threshold,
                loss_scale=loss_scale if need_grad else None,
            )
            if need_grad:
                new_logp.backward(grad if grad.dtype == new_logp.dtype else grad.to(new_logp.dtype))
        else:
            elem, mvec = self._loss_with_metrics(new_logp, old_logp, new_means, old_means, adv_b, sigma_t)
            (elem.mean() * loss_scale).backward()

        vals = mvec.tolist()  # the step's only device-to-host copy
        slots = dict(ops.FLOWDPPO_METRIC_SLOTS)
        loss_value = vals[slots.pop("loss_mean")]
        metrics: Dict[str, Any] = {k: vals[slot] for k, slot in slots.items()}
        metrics.update(policy_loss=loss_value, kl_mask_threshold=float(self.kl_mask_threshold))
        return AlgorithmStepResult(loss=loss_value, metrics=metrics, num_steps_or_tokens=len(steps),
                                   has_backward=True)

    def _step_from_velocities(self, conditions, segment, steps, advantages, loss_scale) -> Optional[AlgorithmStepResult]:
        """The whole micro-step from the model's stacked velocities (a stage with ``replay_velocities``):
        replay log-probs, the KL against the frozen means, masks, loss, metrics and the gradient with
        respect to the new log-probs in one streaming pass plus one finishing workgroup
        (``unirl_flowdppo_replay_step`` -- the new means are never written), then the replay's
        backward kernel hands the velocities their gradient.  Three launches for what the reference
        does in ``S'`` ``denoise`` chains, a stack, a KL pass and autograd (``unirl/models/sd3/
        diffusion.py:467-497``, ``unirl/algorithms/flowdppo.py:286-320``).  ``None`` when the stage
        has no such method or the problem is beyond the fused kernel's row limit."""
        if len(steps) == 0 or getattr(self.stage, "replay_velocities", None) is None:
            return None
        B = int(segment.latents.shape[0])
        if not 0 < B * len(steps) <= ops.FLOWDPPO_REPLAY_MAX_ROWS:
            return None
        vr = self._velocity_replay(conditions, segment, steps)
        v = vr["noise_pred"]
        device = v.device

        def frozen(name):
            return gather_sde_field(getattr(segment, name), segment.sde_indices, steps, field_name=name).to(device)

        old_logp, old_means = frozen("sde_logp"), frozen("sde_means")
        sigma_t = self._compute_sigma_t(segment, steps, device=device).reshape(-1)
        adv_b = advantages.detach().to(dtype=torch.float32, device=device).reshape(-1, 1).expand(B, len(steps))
        need_grad = torch.is_grad_enabled() and v.requires_grad
        kw = dict(kind=vr["strategy"]._kind, eta=vr["eta"], sigma_max=vr["sigma_max"], step_major=vr["step_major"])
        out = ops.flowdppo_replay_step(
            v, vr["latents"], vr["slot_sample"], vr["slot_prev"], vr["sigma"], vr["sigma_next"], old_logp, old_means,
            adv_b, sigma_t, self.kl_mask_threshold, loss_scale=loss_scale if need_grad else None, **kw)
        if need_grad:
            grad_v = ops.sde_replay_logp_bwd(
                v, vr["latents"], vr["slot_sample"], vr["slot_prev"], vr["sigma"], vr["sigma_next"],
                g_logp=out["grad_logp"], g_mean=None, **kw)
            v.backward(grad_v)
        vals = out["metrics"].tolist()  # the step's only device-to-host copy
        slots = dict(ops.FLOWDPPO_METRIC_SLOTS)
        loss_value = vals[slots.pop("loss_mean")]
        metrics: Dict[str, Any] = {k: vals[slot] for k, slot in slots.items()}
        metrics.update(policy_loss=loss_value, kl_mask_threshold=float(self.kl_mask_threshold))
        return AlgorithmStepResult(loss=loss_value, metrics=metrics, num_steps_or_tokens=len(steps), has_backward=True)

    def _loss_with_metrics(self, new_logp, old_logp, new_means, old_means, adv_b, sigma_t):
        kl, _ = ops.gaussian_kl_mask(
            new_means, old_means, sigma_t, self.kl_mask_threshold, reduce_from_dim=2, want_mask=False
        )
        return _MaskedRatioLossFn.apply(new_logp, old_logp, adv_b, kl, self.kl_mask_threshold)

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
