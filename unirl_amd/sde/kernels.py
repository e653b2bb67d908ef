"""SDE step strategies with the reference's call contract, on fused HIP kernels.

Mirrors the public surface of ``unirl/sde/kernels.py`` (``StepStrategy.denoise``
:43-99, ``SDEStrategy`` :115-177, ``FlowSDEStrategy`` :185, ``CPSSDEStrategy``
:239, ``DanceSDEStrategy`` :282): same class names, ``canonical_name`` values,
constructor and method signatures, return tuples and ``None`` rules, so a recipe
``_target_`` can point here.  Where the reference runs ~15 eager element-wise
ops and a reduction per call, ``denoise`` here is one kernel launch
(``unirl_sde_step_logp``) that reads each operand once and writes ``prev_sample``,
``prev_sample_mean`` and the per-sample log-prob; under autograd a second kernel
(``unirl_sde_step_logp_bwd``) produces the gradients w.r.t. ``noise_pred`` and
``sample``.

Additions over the reference signature (keyword-only, optional): ``noise`` lets
the caller supply the sampling noise instead of drawing it inside the step.

``DPM2Strategy`` (:474-516, the deterministic second-order sampler: no log-prob,
``prev_sample_mean`` and ``std_var`` are ``None``) runs its element-wise update as
one kernel per step (``unirl_dpm2_step``) with the scalar coefficients derived on
the host from the schedule.
"""

from __future__ import annotations

import math
from abc import ABC, abstractmethod
from typing import Any, ClassVar, Optional, Tuple, Union

import numpy as np
import torch

from .. import _native as N
from .. import ops

SigmaMax = Union[float, torch.Tensor]


class _SdeStepFn(torch.autograd.Function):
    """Differentiable fused step: gradients flow to ``noise_pred`` and ``sample`` through
    ``prev_sample_mean``, the log-prob and (when sampling) ``prev_sample``."""

    @staticmethod
    def forward(ctx, noise_pred, sample, prev_sample, noise, sigma, sigma_next, sigma_max, eta, kind):
        prev, logp, mean = ops.sde_step_logp(
            noise_pred, sample, sigma, sigma_next, kind=kind, eta=eta, prev_sample=prev_sample, noise=noise,
            sigma_max=sigma_max,
        )
        ctx.set_materialize_grads(False)  # an unused output hands back None, not a zero tensor to read
        ctx.kind, ctx.eta = kind, eta
        ctx.sampling = prev_sample is None
        ctx.has_logp = logp is not None
        ctx.sigma_max = sigma_max
        ctx.saved = (noise_pred.detach(), sample.detach(), None if prev_sample is None else prev_sample.detach(),
                     None if noise is None else noise.detach(), sigma.detach(), sigma_next.detach())
        if not ctx.sampling:
            ctx.mark_non_differentiable(prev)
        if logp is None:
            logp = torch.empty(0, device=sample.device)
            ctx.mark_non_differentiable(logp)
        return prev, logp, mean

    @staticmethod
    def backward(ctx, g_prev, g_logp, g_mean):
        v, x, prev_sample, noise, sigma, sigma_next = ctx.saved
        if g_prev is None and g_logp is None and g_mean is None:
            return (None,) * 9
        grad_v, grad_x = ops.sde_step_logp_bwd(
            v, x, sigma, sigma_next, kind=ctx.kind, eta=ctx.eta, prev_sample=prev_sample, noise=noise,
            sigma_max=ctx.sigma_max, g_logp=g_logp if ctx.has_logp else None, g_mean=g_mean,
            g_prev=g_prev if ctx.sampling else None, need_grad_v=ctx.needs_input_grad[0],
            need_grad_x=ctx.needs_input_grad[1],
        )
        if grad_v is not None and grad_v.dtype != v.dtype:
            grad_v = grad_v.to(v.dtype)
        if grad_x is not None and grad_x.dtype != x.dtype:
            grad_x = grad_x.to(x.dtype)
        return grad_v, grad_x, None, None, None, None, None, None, None


class _SdeReplayFn(torch.autograd.Function):
    """Differentiable batched replay: gradients flow to ``noise_pred`` through the log-probs and the
    means; the stored latents take none."""

    @staticmethod
    def forward(ctx, noise_pred, latents, sigma, sigma_next, sigma_max, eta, kind, slots, step_major, means_dtype):
        logp, means = ops.sde_replay_logp(
            noise_pred, latents, slots[0], slots[1], sigma, sigma_next, kind=kind, eta=eta, sigma_max=sigma_max,
            step_major=step_major, means_dtype=means_dtype,
        )
        ctx.set_materialize_grads(False)
        ctx.cfg = (kind, eta, sigma_max, slots, step_major)
        ctx.has_logp = logp is not None
        ctx.saved = (noise_pred.detach(), latents.detach(), sigma, sigma_next)
        if logp is None:
            logp = torch.empty(0, device=latents.device)
            ctx.mark_non_differentiable(logp)
        return logp, means

    @staticmethod
    def backward(ctx, g_logp, g_means):
        if (g_logp is None or not ctx.has_logp) and g_means is None:
            return (None,) * 10
        v, latents, sigma, sigma_next = ctx.saved
        kind, eta, sigma_max, slots, step_major = ctx.cfg
        grad_v = ops.sde_replay_logp_bwd(
            v, latents, slots[0], slots[1], sigma, sigma_next, kind=kind, eta=eta, sigma_max=sigma_max,
            step_major=step_major, g_logp=g_logp if ctx.has_logp else None, g_mean=g_means,
        )
        return (grad_v,) + (None,) * 9


def next_rng(device: torch.device) -> Optional[Tuple[int, int]]:
    """``(seed, offset)`` for one in-kernel noise draw, taken from -- and advancing -- the device's
    default torch generator, so that ``torch.manual_seed`` governs the sampling noise as it governs
    ``torch.randn``: same seed, same sequence of calls, same noise.  (The kernel keys its own
    Philox stream with the seed; torch's offset is only the counter that tells calls apart.)
    ``None`` while a HIP graph is being captured: the generator's state then belongs to the graph."""
    if torch.cuda.is_current_stream_capturing():
        return None
    index = device.index if device.index is not None else torch.cuda.current_device()
    gen = torch.cuda.default_generators[index]
    offset = gen.get_offset()
    gen.set_offset(offset + 4)  # torch keeps its offsets multiples of four
    # another key than torch's own kernels use with this seed: the two streams never meet
    return (gen.initial_seed() ^ 0x9E3779B97F4A7C15) & 0xFFFFFFFFFFFFFFFF, offset


class StepStrategy(ABC):
    """Base class of all sampling step strategies."""

    #: kernel family; ``None`` for strategies without a fused kernel
    _kind: ClassVar[Optional[str]] = None

    @abstractmethod
    def step(
        self,
        noise_pred: torch.Tensor,
        sample: torch.Tensor,
        sigma: torch.Tensor,
        sigma_next: torch.Tensor,
        eta: float = 1.0,
        prev_sample: Optional[torch.Tensor] = None,
        generator: Optional[torch.Generator] = None,
        sigma_max: SigmaMax = 0.99,
        step_index: int = 0,
    ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """One sampling step: ``(prev_sample, prev_sample_mean, std_var)``."""

    def reset(self) -> None:
        """Stateless strategies have nothing to reset."""

    def init_schedule(self, sigmas: torch.Tensor) -> None:
        """Stateless strategies ignore the full schedule."""

    def denoise(
        self,
        noise_pred: torch.Tensor,
        sample: torch.Tensor,
        sigma: torch.Tensor,
        sigma_next: torch.Tensor,
        *,
        eta: float = 1.0,
        prev_sample: Optional[torch.Tensor] = None,
        sigma_max: SigmaMax = 0.99,
        step_index: int = 0,
        noise: Optional[torch.Tensor] = None,
    ) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
        """One denoising transition: ``(prev_sample, log_prob, prev_sample_mean)``, all fp32.

        ``prev_sample=None`` samples (noise is drawn on the device unless given);
        otherwise the log-prob of the stored transition is replayed.  ``log_prob``
        is ``None`` when ``eta < 1e-7``.
        """
        del step_index
        kind = self._kind
        if kind is None:
            raise NotImplementedError(f"{type(self).__name__} has no fused kernel")
        if not sample.is_cuda:
            raise RuntimeError(
                f"{type(self).__name__}.denoise: sample lives on {sample.device}; the fused SDE kernel "
                "runs on a HIP device only and there is no CPU fallback"
            )
        needs_grad = torch.is_grad_enabled() and (noise_pred.requires_grad or sample.requires_grad)
        rng = None
        if prev_sample is None and noise is None and float(eta) != 0.0:
            # The reference draws with generator=None on noise_pred's device, in fp32
            # (unirl/sde/kernels.py:230-232).  Here the kernel draws the noise itself from the device's
            # default generator state (seed, offset) -- no noise tensor is written and read back --
            # except under autograd, whose backward wants the noise tensor, and under graph capture,
            # where the generator's state is the graph's business.
            rng = None if needs_grad else next_rng(sample.device)
            if rng is None:
                noise = torch.randn(sample.shape, device=sample.device, dtype=torch.float32)
        # fp32 replay: the reference's .float() / .to(float32) round trip is the identity, so the
        # caller's own tensor is handed back and the kernel need not write a copy of it
        reuse_prev = (
            prev_sample is not None and prev_sample.dtype == torch.float32 and sample.dtype == torch.float32
        )
        if needs_grad:
            prev, logp, mean = _SdeStepFn.apply(
                noise_pred, sample, prev_sample, noise, sigma, sigma_next, sigma_max, float(eta), kind
            )
            if eta < 1e-7:
                logp = None
        else:
            prev, logp, mean = ops.sde_step_logp(
                noise_pred, sample, sigma, sigma_next, kind=kind, eta=float(eta), prev_sample=prev_sample,
                noise=noise, sigma_max=sigma_max, want_prev=not reuse_prev, rng=rng,
            )
        if reuse_prev:
            prev = prev_sample
        return prev, logp, mean


    def denoise_into(
        self,
        noise_pred: torch.Tensor,
        sample: torch.Tensor,
        sigma: torch.Tensor,
        sigma_next: torch.Tensor,
        *,
        eta: float = 1.0,
        prev_sample: Optional[torch.Tensor] = None,
        sigma_max: SigmaMax = 0.99,
        noise: Optional[torch.Tensor] = None,
        prev_out: Optional[torch.Tensor] = None,
        mean_out: Optional[torch.Tensor] = None,
        logp_out: Optional[torch.Tensor] = None,
    ) -> bool:
        """``denoise`` for the stage loops that keep trajectories as ``[B, K, ...]`` stacks
        (``unirl/models/sd3/diffusion.py:366-406`` and ``:467-497``), without autograd.

        ``sample`` / ``prev_sample`` may be ``latents[:, k]`` views (read in place);
        ``prev_out`` / ``mean_out`` may be views into fp32 / bf16 / fp16 stacks and
        ``logp_out`` a column ``log_probs[:, j]`` -- the kernel writes them directly, so the
        loop needs no ``.to(trajectory_dtype)``, ``clone`` or ``torch.stack`` copies.  Storing
        ``prev`` in ``sample.dtype`` is exact (it has been rounded to that dtype already);
        storing the mean in a 16-bit dtype rounds once, like ``stack(...).to(dtype)``.
        Returns ``False`` when ``eta < 1e-7`` (no log-prob; ``logp_out`` untouched).
        """
        if self._kind is None:
            raise NotImplementedError(f"{type(self).__name__} has no fused kernel")
        if not sample.is_cuda:
            raise RuntimeError(
                f"{type(self).__name__}.denoise_into: sample lives on {sample.device}; the fused SDE kernel "
                "runs on a HIP device only and there is no CPU fallback"
            )
        rng = None
        if prev_sample is None and noise is None and float(eta) != 0.0:
            rng = next_rng(sample.device)  # the kernel draws the noise itself (see denoise)
            if rng is None:
                noise = torch.randn(sample.shape, device=sample.device, dtype=torch.float32)
        ops.sde_step_logp_into(
            noise_pred, sample, sigma, sigma_next, kind=self._kind, eta=float(eta), prev_sample=prev_sample,
            noise=noise, sigma_max=sigma_max, prev_out=prev_out, mean_out=mean_out, logp_out=logp_out, rng=rng,
        )
        return not (eta < 1e-7)

    def replay_steps(self, noise_pred, latents, slot_sample, slot_prev, sigma, sigma_next, *, eta=1.0, sigma_max=0.99,
                     step_major=False, means_dtype=None):
        """The replay loop of a diffusion stage (``unirl/models/sd3/diffusion.py:467-497``) for velocities
        that are all known, as ONE fused launch over the ``B * S`` (sample, step) transitions:
        ``(log_probs [B, S] fp32, prev_sample_means [B, S, ...])``.

        ``noise_pred``: ``[B, S, ...]`` (``[S, B, ...]`` with ``step_major``, the layout of a model pass
        over the steps stacked into the batch); ``latents``: the segment's ``[B, K, ...]`` trajectory
        stack, read in place -- step ``j`` starts from slot ``slot_sample[j]`` and is scored against
        the stored latent in slot ``slot_prev[j]`` (see :func:`replay_slots`); ``sigma`` /
        ``sigma_next``: one value per step.  The means come back in ``means_dtype`` (default: the
        stack's dtype, i.e. ``stack(means, dim=1).to(trajectory_dtype)``).  Per row the arithmetic is
        ``denoise(..., prev_sample=...)``'s.  Differentiable with respect to ``noise_pred``.
        Raises ``RuntimeError`` when ``eta < 1e-7``: a replay needs a stochastic step, as in the
        reference's loop."""
        kind = self._kind
        if kind is None:
            raise NotImplementedError(f"{type(self).__name__} has no fused kernel")
        if eta < 1e-7:
            raise RuntimeError(
                f"{type(self).__name__}.replay_steps: eta={eta} is a deterministic step (no log-prob); "
                "replay requires a stochastic SDE strategy"
            )
        if not latents.is_cuda:
            raise RuntimeError(
                f"{type(self).__name__}.replay_steps: latents live on {latents.device}; the fused SDE kernel "
                "runs on a HIP device only and there is no CPU fallback"
            )
        slots = ([int(k) for k in slot_sample], [int(k) for k in slot_prev])
        if torch.is_grad_enabled() and noise_pred.requires_grad:
            return _SdeReplayFn.apply(noise_pred, latents, sigma, sigma_next, sigma_max, float(eta), kind, slots,
                                      bool(step_major), means_dtype)
        return ops.sde_replay_logp(noise_pred, latents, slots[0], slots[1], sigma, sigma_next, kind=kind, eta=float(eta),
                                   sigma_max=sigma_max, step_major=step_major, means_dtype=means_dtype)


def replay_slots(indices, step_indices) -> Tuple[list, list]:
    """Storage slots ``(of each step's latent, of its stored next latent)`` inside a trajectory stack
    whose slot ``k`` holds the latent of step ``indices[k]`` (``LatentSegment.latents_at``,
    ``unirl/types/segments/latent.py:82-97``, for ``step`` and ``step + 1``)."""
    if indices is None:
        raise RuntimeError("replay_slots: missing indices")
    stored = [int(i) for i in (indices.tolist() if isinstance(indices, torch.Tensor) else indices)]
    where = {}
    for k, i in enumerate(stored):
        where.setdefault(i, k)  # the first slot holding a step, as list.index finds it
    out = ([], [])
    for step in step_indices:
        for offset, slots in zip((0, 1), out):
            if int(step) + offset not in where:
                raise KeyError(f"latents_at: step_idx={int(step) + offset} not in stored indices={stored}")
            slots.append(where[int(step) + offset])
    return out


def latents_at(latents: Optional[torch.Tensor], indices: Optional[torch.Tensor], step_idx: int) -> torch.Tensor:
    """``latents[:, k]`` (a view) for the storage slot ``k`` with ``indices[k] == step_idx`` --
    ``LatentSegment.latents_at`` (``unirl/types/segments/latent.py:82-97``) as a free function."""
    if indices is None or latents is None:
        raise RuntimeError("latents_at: missing indices or latents")
    stored = [int(i) for i in indices.tolist()]
    try:
        k = stored.index(int(step_idx))
    except ValueError:
        raise KeyError(f"latents_at: step_idx={step_idx} not in stored indices={stored}") from None
    return latents[:, k]


class SDEStrategy(StepStrategy, ABC):
    """Stochastic strategies: a transition mean, a noise scale and a Gaussian log-prob."""

    @abstractmethod
    def compute_log_prob(self, prev_sample: torch.Tensor, prev_sample_mean: torch.Tensor, **kwargs) -> torch.Tensor:
        """Element-wise log-prob of ``prev_sample`` under the transition."""

    def _coefficients(self, sigma, sigma_next, eta, sigma_max, ndim, device):
        """std_var with the reference's fp32 operation order, broadcast to ``ndim`` dims."""
        raise NotImplementedError

    def step(
        self,
        noise_pred: torch.Tensor,
        sample: torch.Tensor,
        sigma: torch.Tensor,
        sigma_next: torch.Tensor,
        eta: float = 1.0,
        prev_sample: Optional[torch.Tensor] = None,
        generator: Optional[torch.Generator] = None,
        sigma_max: SigmaMax = 0.99,
        step_index: int = 0,
    ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """``(prev_sample, prev_sample_mean, std_var)`` without the log-prob or the dtype
        round trip; the same fused kernel with the reduction switched off."""
        del step_index
        noise = None
        if prev_sample is None:
            noise = torch.randn(sample.shape, generator=generator, device=sample.device, dtype=torch.float32)
        prev, _, mean = ops.sde_step_logp(
            noise_pred.float(), sample.float(), sigma, sigma_next, kind=self._kind, eta=float(eta),
            prev_sample=None if prev_sample is None else prev_sample.float(), noise=noise, sigma_max=sigma_max,
            want_logp=False,
        )
        if prev_sample is not None:
            prev = prev_sample
        std_var = self._coefficients(sigma, sigma_next, float(eta), sigma_max, sample.dim(), sample.device)
        return prev, mean, std_var


def _as_broadcast(s: torch.Tensor, ndim: int, device) -> torch.Tensor:
    s = s.detach().to(device=device, dtype=torch.float32)
    if s.dim() == 0:
        s = s.unsqueeze(0)
    while s.dim() < ndim:
        s = s.unsqueeze(-1)
    return s


def _gaussian_elem_log_prob(prev_sample, prev_sample_mean, std_var):
    return (
        -((prev_sample.detach() - prev_sample_mean) ** 2) / (2 * std_var**2)
        - torch.log(std_var)
        - 0.5 * math.log(2 * math.pi)
    )


class FlowSDEStrategy(SDEStrategy):
    """FlowGRPO's SDE: ``std = sqrt(sigma / (1 - sigma)) * eta`` (``sigma_max`` where sigma is 1)."""

    canonical_name: ClassVar[str] = "flow"
    _kind: ClassVar[str] = "flow"

    def __init__(self, *, config: Optional[Any] = None) -> None:
        del config

    def compute_log_prob(self, prev_sample, prev_sample_mean, std_var, **kwargs) -> torch.Tensor:
        return _gaussian_elem_log_prob(prev_sample, prev_sample_mean, std_var)

    def _coefficients(self, sigma, sigma_next, eta, sigma_max, ndim, device):
        s = _as_broadcast(sigma, ndim, device)
        sn = _as_broadcast(sigma_next, ndim, device)
        if isinstance(sigma_max, torch.Tensor):
            sigma_max = sigma_max.to(device)
        std_dev_t = torch.sqrt(s / (1 - torch.where(s == 1, sigma_max, s))) * eta
        return std_dev_t * torch.sqrt(-(sn - s))


class DanceSDEStrategy(SDEStrategy):
    """DanceGRPO's SDE: constant ``std = eta``."""

    canonical_name: ClassVar[str] = "dance"
    _kind: ClassVar[str] = "dance"

    def __init__(self, *, config: Optional[Any] = None) -> None:
        del config

    def compute_log_prob(self, prev_sample, prev_sample_mean, std_var, **kwargs) -> torch.Tensor:
        return _gaussian_elem_log_prob(prev_sample, prev_sample_mean, std_var)

    def _coefficients(self, sigma, sigma_next, eta, sigma_max, ndim, device):
        s = _as_broadcast(sigma, ndim, device)
        sn = _as_broadcast(sigma_next, ndim, device)
        return eta * torch.sqrt(-(sn - s))


class CPSSDEStrategy(SDEStrategy):
    """Coefficient-preserving sampling: ``std = sigma_next * sin(eta*pi/2)``, un-normalised log-prob."""

    canonical_name: ClassVar[str] = "cps"
    _kind: ClassVar[str] = "cps"

    def __init__(self, *, config: Optional[Any] = None) -> None:
        del config

    def compute_log_prob(self, prev_sample, prev_sample_mean, **kwargs) -> torch.Tensor:
        return -((prev_sample.detach() - prev_sample_mean) ** 2)

    def _coefficients(self, sigma, sigma_next, eta, sigma_max, ndim, device):
        sn = _as_broadcast(sigma_next, ndim, device)
        return sn * math.sin(eta * math.pi / 2)


STRATEGIES = {cls.canonical_name: cls for cls in (FlowSDEStrategy, DanceSDEStrategy, CPSSDEStrategy)}


def _half_log_snr(sigma: torch.Tensor) -> torch.Tensor:
    return torch.log(1 - sigma) - torch.log(sigma)


def _f32(t: torch.Tensor) -> float:
    """A 0-dim tensor rounded to fp32: the value torch multiplies an fp32 tensor by."""
    return float(t.to(torch.float32))


def dpm2_coefficients(sigmas: torch.Tensor, step_index: int, warm: int) -> Tuple[int, "N.Dpm2Coeffs"]:
    """Branch and scalar coefficients of one DPM-Solver-2 step (``_dpm_step``,
    ``unirl/sde/kernels.py:428-471``) from a host copy of the schedule: the DDIM update on the
    first and the last step (scalars in the schedule's dtype), else the first-order update until
    one step has been taken and the multistep second-order update afterwards (scalars in
    float64, :377-425).  ``warm`` counts the steps taken since the last reset."""
    n_steps = int(sigmas.shape[0]) - 1
    i = int(step_index)
    if not 0 <= i < n_steps:
        raise IndexError(f"step_index {i} outside the schedule's {n_steps} steps")
    c = N.Dpm2Coeffs()
    c.sigma = _f32(sigmas[i])
    last = i == n_steps - 1
    if (warm < 1 or last) and (i == 0 or last):
        t, s = sigmas[i + 1], sigmas[i]
        c.one_minus_s, c.s, c.one_minus_t = _f32(1 - s), _f32(s), _f32(1 - t)
        # sqrt(t**2) in the schedule's dtype; numpy's root is correctly rounded on every host
        c.sqrt_t2 = float(np.float32(np.sqrt((t**2).numpy())))
        return N.DPM2_DDIM, c
    sig = sigmas.to(torch.float64)
    s_t, s_0 = sig[i + 1], sig[i]
    lam_t, lam_0 = _half_log_snr(s_t), _half_log_snr(s_0)
    h = lam_t - lam_0
    growth = (1 - s_t) * (torch.exp(-h) - 1.0)
    c.c1, c.c2 = _f32(s_t / s_0), _f32(growth)
    if warm < 1 or last:
        return N.DPM2_FIRST, c
    r0 = (lam_0 - _half_log_snr(sig[i - 1])) / h
    c.inv_r0, c.half_c2 = _f32(1.0 / r0), _f32(0.5 * growth)
    return N.DPM2_SECOND, c


class DPM2Strategy(StepStrategy):
    """DPM-Solver-2 multistep ODE sampler (deterministic, stateful): ``init_schedule`` before the
    first step, consecutive ``step_index`` values afterwards.  No log-prob, so it cannot train."""

    canonical_name: ClassVar[str] = "dpm2"

    def __init__(self, *, config: Optional[Any] = None) -> None:
        del config
        self.reset()

    def reset(self) -> None:
        self._sigmas: Optional[torch.Tensor] = None  # host copy of the schedule
        self._x0: list = [None, None]  # x0 predictions, oldest first; the buffers alternate
        self._warm = 0

    def init_schedule(self, sigmas: torch.Tensor) -> None:
        self.reset()
        self._sigmas = sigmas.detach().cpu()

    def _advance(self, noise_pred: torch.Tensor, sample: torch.Tensor, step_index: int) -> torch.Tensor:
        if self._sigmas is None:
            raise RuntimeError("DPM2Strategy requires init_schedule() before stepping.")
        if not sample.is_cuda:
            raise RuntimeError(
                f"DPM2Strategy: sample lives on {sample.device}; the fused kernel runs on a HIP device only "
                "and there is no CPU fallback"
            )
        branch, coeffs = dpm2_coefficients(self._sigmas, step_index, self._warm)
        older, newer = self._x0
        x0, prev = ops.dpm2_step(noise_pred, sample, newer, branch, coeffs, x0_out=older)
        self._x0 = [newer, x0]
        self._warm = min(2, self._warm + 1)
        return prev

    def step(
        self,
        noise_pred: torch.Tensor,
        sample: torch.Tensor,
        sigma: torch.Tensor,
        sigma_next: torch.Tensor,
        eta: float = 1.0,
        prev_sample: Optional[torch.Tensor] = None,
        generator: Optional[torch.Generator] = None,
        sigma_max: SigmaMax = 0.99,
        step_index: int = 0,
    ) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
        del sigma, sigma_next, eta, prev_sample, generator, sigma_max  # the schedule and the index say it all
        return self._advance(noise_pred, sample, step_index), None, None

    def denoise(
        self,
        noise_pred: torch.Tensor,
        sample: torch.Tensor,
        sigma: torch.Tensor,
        sigma_next: torch.Tensor,
        *,
        eta: float = 1.0,
        prev_sample: Optional[torch.Tensor] = None,
        sigma_max: SigmaMax = 0.99,
        step_index: int = 0,
        noise: Optional[torch.Tensor] = None,
    ) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
        """``(prev_sample fp32, None, None)``: an ODE step has no log-prob and no transition mean."""
        del sigma, sigma_next, eta, prev_sample, sigma_max, noise
        return self._advance(noise_pred, sample, step_index), None, None


def sde_rollout(
    strategy: SDEStrategy,
    latents: torch.Tensor,
    velocities,
    sigmas: torch.Tensor,
    etas,
    *,
    noises=None,
    sigma_max: Optional[SigmaMax] = None,
    return_trajectory: bool = False,
):
    """``S`` chained ``denoise`` calls for known velocities in ONE launch, the latent
    held in registers between steps (the loop at ``unirl/models/sd3/diffusion.py:366-390``
    with ``predict_noise`` factored out).  ``etas`` is one float or one per step; steps
    with ``eta < 1e-7`` are Euler steps and report NaN in their log-prob column.
    Returns ``(final latent fp32, log_probs [B,S] fp32, trajectory [S,B,...] or None)``.
    """
    S = len(velocities)
    if noises is None:
        noises = [torch.randn(latents.shape, device=latents.device, dtype=torch.float32) for _ in range(S)]
    x, logp, traj = ops.sde_rollout_logp(
        latents, velocities, noises, sigmas, etas, kind=strategy._kind, sigma_max=sigma_max,
        want_trajectory=return_trajectory,
    )
    return x, logp, traj


__all__ = [
    "CPSSDEStrategy",
    "DPM2Strategy",
    "DanceSDEStrategy",
    "FlowSDEStrategy",
    "SDEStrategy",
    "STRATEGIES",
    "StepStrategy",
    "latents_at",
    "replay_slots",
    "sde_rollout",
]
