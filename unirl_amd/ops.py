"""Tensor-level wrappers over the C ABI: validate, allocate outputs, launch.

Every function takes HIP tensors, enqueues one fused kernel on the current
torch stream and returns without synchronising.  The reference-shaped Python
API (``unirl_amd.sde``, ``unirl_amd.algorithms``, ...) is built on these.
"""

from __future__ import annotations

import ctypes
import functools
import math
from typing import Dict, List, Optional, Sequence, Tuple, Union

import torch

from . import _native as N

SDE_KINDS = {"flow": N.SDE_FLOW, "dance": N.SDE_DANCE, "cps": N.SDE_CPS}


def _flat2(t: torch.Tensor, name: str) -> torch.Tensor:
    """``t`` itself when it is a contiguous device tensor (only its address is used, so a tensor
    that requires grad needs no detach), else a contiguous copy."""
    N.require_device(t, name)
    return t if t.is_contiguous() else t.detach().contiguous()


def _kernel_dtype(t: torch.Tensor) -> torch.Tensor:
    """fp32 / bf16 / fp16 tensors pass; anything else (float64, ...) is cast to fp32."""
    return t if t.dtype in N._DTYPE_CODE else t.detach().float()


def _sigma_arg(sigma: torch.Tensor, B: int, device: torch.device, name: str) -> Tuple[torch.Tensor, int]:
    """f32 device tensor with 1 or B values, and the per-sample stride (0 or 1)."""
    s = sigma
    if s.dtype is torch.float32 and s.dim() == 1 and s.device == device and s.stride(0) == 1 and not s.requires_grad:
        n = s.shape[0]  # already what the kernel reads: no view is made
        if n == 1 or n == B:
            return s, (0 if n == 1 else 1)
    if s.dtype != torch.float32 or s.device != device or s.requires_grad:
        s = s.detach().to(device=device, dtype=torch.float32)
    n = s.numel()
    if n == 1:
        return (s if s.dim() <= 1 else s.reshape(-1)), 0
    s = s.reshape(-1).contiguous()
    if s.numel() == 1:
        return s, 0
    if s.numel() == B:
        return s, 1
    raise ValueError(f"{name} must hold one value or one per sample ({B}); got {tuple(sigma.shape)}")


def _sigma_max_arg(sigma_max, device: torch.device):
    """(device tensor or None, float value)."""
    if isinstance(sigma_max, torch.Tensor):
        if sigma_max.is_cuda:
            if sigma_max.numel() == 1 and sigma_max.dtype is torch.float32 and sigma_max.device == device:
                return sigma_max, 0.0  # one fp32 value on the device: its address is all that is needed
            t = sigma_max.detach().to(device=device, dtype=torch.float32).reshape(-1)[:1].contiguous()
            return t, 0.0
        return None, float(sigma_max)
    return None, float(sigma_max)


def sde_step_logp(
    noise_pred: torch.Tensor,
    sample: torch.Tensor,
    sigma: torch.Tensor,
    sigma_next: torch.Tensor,
    *,
    kind: str = "flow",
    eta: float = 1.0,
    prev_sample: Optional[torch.Tensor] = None,
    noise: Optional[torch.Tensor] = None,
    sigma_max: Union[float, torch.Tensor] = 0.99,
    want_prev: bool = True,
    want_mean: bool = True,
    want_logp: bool = True,
    logp_sum: bool = False,
    rng: Optional[Tuple[int, int]] = None,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor]]:
    """One fused SDE transition. Returns ``(prev f32, logp [B] f32 or None, mean f32)``.

    ``prev_sample`` given = replay, else sampling with ``noise`` (f32, same shape;
    ``None`` adds no noise, or -- with ``rng = (seed, offset)`` -- standard normal noise drawn
    inside the kernel: no noise tensor is written or read).  ``sample.dtype`` is the dtype of the
    round trip applied to ``prev`` before the log-prob.
    """
    if sample.dim() < 2:
        raise ValueError(f"sample needs a batch dimension and at least one more; got {tuple(sample.shape)}")
    if noise_pred.shape != sample.shape:
        raise ValueError(f"noise_pred {tuple(noise_pred.shape)} != sample {tuple(sample.shape)}")
    device = sample.device
    if rng is not None and prev_sample is None and noise is None:
        # the generator rides in the descriptor of the strided entry point; the outputs are fresh fp32 tensors
        B = sample.shape[0]
        logp_wanted = want_logp and not (eta < 1e-7)
        prev_out = torch.empty(sample.shape, dtype=torch.float32, device=device) if want_prev else None
        mean_out = torch.empty(sample.shape, dtype=torch.float32, device=device) if want_mean else None
        logp_out = torch.empty(B, dtype=torch.float32, device=device) if logp_wanted else None
        if B == 0 or sample.numel() == 0:
            if logp_out is not None:
                logp_out.fill_(float("nan"))
            return prev_out, logp_out, mean_out
        sde_step_logp_into(noise_pred, sample, sigma, sigma_next, kind=kind, eta=eta, sigma_max=sigma_max,
                           prev_out=prev_out, mean_out=mean_out, logp_out=logp_out, logp_sum=logp_sum, rng=rng)
        return prev_out, logp_out, mean_out
    v = _kernel_dtype(_flat2(noise_pred, "noise_pred"))
    x = _kernel_dtype(_flat2(sample, "sample"))
    B = x.shape[0]
    D = x.numel() // B if B else 0
    prev_in = None
    if prev_sample is not None:
        if prev_sample.shape != sample.shape:
            raise ValueError(f"prev_sample {tuple(prev_sample.shape)} != sample {tuple(sample.shape)}")
        # prev.float().to(x.dtype) == prev.to(x.dtype): casting here is the reference's round trip
        prev_in = _flat2(prev_sample, "prev_sample")
        if prev_in.dtype is not x.dtype:
            prev_in = prev_in.detach().to(x.dtype)
    nz = None
    if noise is not None and prev_sample is None:
        if noise.shape != sample.shape:
            raise ValueError(f"noise {tuple(noise.shape)} != sample {tuple(sample.shape)}")
        nz = _flat2(noise, "noise")
        if nz.dtype is not torch.float32:
            nz = nz.detach().float()
    sig, stride = _sigma_arg(sigma, B, device, "sigma")
    sig_n, stride_n = _sigma_arg(sigma_next, B, device, "sigma_next")
    if stride != stride_n:
        if stride == 0:
            sig, stride = sig.expand(B).contiguous(), 1
        else:
            sig_n = sig_n.expand(B).contiguous()
    smax_t, smax_v = _sigma_max_arg(sigma_max, device)

    logp_wanted = want_logp and not (eta < 1e-7)
    prev_out = torch.empty(x.shape, dtype=torch.float32, device=device) if want_prev else None
    mean_out = torch.empty(x.shape, dtype=torch.float32, device=device) if want_mean else None
    logp_out = torch.empty(B, dtype=torch.float32, device=device) if logp_wanted else None
    if B == 0 or D == 0:
        if logp_out is not None:
            logp_out.fill_(float("nan"))
        return prev_out, logp_out, mean_out
    stream = N.current_stream(device)
    ws, ws_bytes = N.workspace(device, stream)
    with N.on_device(device):
        rc = N.F.unirl_sde_step_logp(
            N.ptr(v), N.dtype_code(v.dtype), N.ptr(x), N.dtype_code(x.dtype), N.ptr(prev_in), N.ptr(nz),
            N.ptr(sig), N.ptr(sig_n), stride, N.ptr(smax_t), smax_v, float(eta), SDE_KINDS[kind], B, D,
            N.ptr(prev_out), N.ptr(mean_out), N.ptr(logp_out), int(bool(logp_sum)), N.ptr(ws), ws_bytes,
            stream,
        )
    N.check(rc, "unirl_sde_step_logp")
    return prev_out, logp_out, mean_out


def _per_sample_view(t: torch.Tensor, name: str, *, writable: bool = False) -> Tuple[torch.Tensor, int]:
    """``(tensor, elements between consecutive samples)`` for a ``[B, ...]`` tensor whose samples
    are each one contiguous block, e.g. ``stack[:, k]`` of a ``[B, K, ...]`` stack.  Inputs of any
    other layout are copied; outputs must already have it."""
    N.require_device(t, name)
    B = t.shape[0]
    D = t.numel() // B if B else 0
    if t.is_contiguous():
        return t, D
    inner_ok = B == 0 or _dense_from(t, 1)
    # A sample stride of 0 means "densely packed" in the C ABI, so a tensor broadcast over the
    # samples (expand(B, ...), stride 0) cannot be handed over as it is: it is copied.
    if inner_ok and (B <= 1 or t.stride(0) >= (D if writable else 1)):
        return t, (t.stride(0) if B > 1 else D)
    if writable:
        raise ValueError(f"{name}: each sample must be one contiguous, non-overlapping block; got strides {t.stride()}")
    t = t.contiguous()
    return t, D


def sde_step_logp_into(
    noise_pred: torch.Tensor,
    sample: torch.Tensor,
    sigma: torch.Tensor,
    sigma_next: torch.Tensor,
    *,
    kind: str = "flow",
    eta: float = 1.0,
    prev_sample: Optional[torch.Tensor] = None,
    noise: Optional[torch.Tensor] = None,
    sigma_max: Union[float, torch.Tensor] = 0.99,
    prev_out: Optional[torch.Tensor] = None,
    mean_out: Optional[torch.Tensor] = None,
    logp_out: Optional[torch.Tensor] = None,
    logp_sum: bool = False,
    rng: Optional[Tuple[int, int]] = None,
    noise_out: Optional[torch.Tensor] = None,
) -> None:
    """One fused SDE transition that reads strided ``[B, ...]`` views in place and writes into
    caller-owned views (``unirl_sde_step_logp_ex``), no gradient.

    Sampling without a ``noise`` tensor and with ``rng = (seed, offset)`` draws the noise inside the
    kernel (Philox-4x32-10 keyed by ``seed``, counter ``(element index / 4, offset)``, Box-Muller):
    the draw of an element depends on nothing but ``(seed, offset, element index)``.  ``noise_out``
    (fp32, ``sample``'s shape) receives it when given.

    ``sample`` / ``prev_sample`` may be ``stack[:, k]`` slices of a ``[B, K, ...]`` trajectory in
    fp32, bf16 or fp16; ``prev_out`` / ``mean_out`` may be slices of such stacks in any of the
    three dtypes (values are rounded to nearest-even on store); ``logp_out`` is a fp32 ``[B]``
    view, e.g. ``log_probs[:, j]``.  ``logp_out`` is left untouched when ``eta < 1e-7``.
    """
    if sample.dim() < 2:
        raise ValueError(f"sample needs a batch dimension and at least one more; got {tuple(sample.shape)}")
    if noise_pred.shape != sample.shape:
        raise ValueError(f"noise_pred {tuple(noise_pred.shape)} != sample {tuple(sample.shape)}")
    device = sample.device
    B = sample.shape[0]
    D = sample.numel() // B if B else 0

    def as_input(t, name):  # only the address is used: a tensor that requires grad needs no detach
        if t.dtype not in N._DTYPE_CODE:
            t = t.detach().float()
        elif t.requires_grad and not t.is_contiguous():
            t = t.detach()  # a copy may follow; keep it out of the autograd graph
        return _per_sample_view(t, name)

    v, sv = as_input(noise_pred, "noise_pred")
    x, sx = as_input(sample, "sample")
    pin, sp = None, 0
    if prev_sample is not None:
        if prev_sample.shape != sample.shape:
            raise ValueError(f"prev_sample {tuple(prev_sample.shape)} != sample {tuple(sample.shape)}")
        pin = prev_sample
        if pin.dtype != x.dtype:
            pin = pin.detach().to(x.dtype)  # the reference's round trip through the input dtype
        elif pin.requires_grad and not pin.is_contiguous():
            pin = pin.detach()
        pin, sp = _per_sample_view(pin, "prev_sample")
    nz, sn = None, 0
    if noise is not None and prev_sample is None:
        if noise.shape != sample.shape:
            raise ValueError(f"noise {tuple(noise.shape)} != sample {tuple(sample.shape)}")
        nz, sn = _per_sample_view(noise if noise.dtype is torch.float32 and not noise.requires_grad
                                  else noise.detach().float(), "noise")

    def as_output(t, name, shape):
        if t is None:
            return None, 0
        if tuple(t.shape) != tuple(shape):
            raise ValueError(f"{name} {tuple(t.shape)} != {tuple(shape)}")
        if t.dtype not in N._DTYPE_CODE:
            raise TypeError(f"{name}: unsupported dtype {t.dtype}")
        if t.device != device:
            raise ValueError(f"{name} lives on {t.device}, the inputs on {device}")
        return _per_sample_view(t, name, writable=True)

    po, spo = as_output(prev_out, "prev_out", sample.shape)
    mo, smo = as_output(mean_out, "mean_out", sample.shape)
    lp, slp = None, 0
    if logp_out is not None:
        N.require_device(logp_out, "logp_out")
        if tuple(logp_out.shape) != (B,) or logp_out.dtype != torch.float32:
            raise ValueError(f"logp_out must be float32 [{B}]; got {logp_out.dtype} {tuple(logp_out.shape)}")
        lp, slp = logp_out, (logp_out.stride(0) if B > 1 else 1)
        if B > 1 and slp < 1:
            raise ValueError("logp_out must not alias across samples")
    sig, stride = _sigma_arg(sigma, B, device, "sigma")
    sig_n, stride_n = _sigma_arg(sigma_next, B, device, "sigma_next")
    if stride != stride_n:
        if stride == 0:
            sig, stride = sig.expand(B).contiguous(), 1
        else:
            sig_n = sig_n.expand(B).contiguous()
    smax_t, smax_v = _sigma_max_arg(sigma_max, device)
    if B == 0 or D == 0:
        return

    d = N.SdeStepDesc()
    d.noise_pred = N.SdeTensor(N.ptr(v), N.dtype_code(v.dtype), sv)
    d.sample = N.SdeTensor(N.ptr(x), N.dtype_code(x.dtype), sx)
    d.prev_sample = N.SdeTensor(N.ptr(pin), N.dtype_code(x.dtype), sp)
    d.noise, d.noise_stride = N.ptr(nz), sn
    d.sigma, d.sigma_next, d.sigma_stride = N.ptr(sig), N.ptr(sig_n), stride
    d.sigma_max_ptr, d.sigma_max_val = N.ptr(smax_t), smax_v
    d.eta, d.kind, d.B, d.D = float(eta), SDE_KINDS[kind], B, D
    d.prev_out, d.prev_dtype, d.prev_stride = N.ptr(po), (N.dtype_code(po.dtype) if po is not None else 0), spo
    d.mean_out, d.mean_dtype, d.mean_stride = N.ptr(mo), (N.dtype_code(mo.dtype) if mo is not None else 0), smo
    d.logp_out, d.logp_stride, d.logp_sum = N.ptr(lp), slp, int(bool(logp_sum))
    if rng is not None and prev_sample is None and noise is None:
        d.rng = N.Rng(1, int(rng[0]) & 0xFFFFFFFFFFFFFFFF, int(rng[1]) & 0xFFFFFFFFFFFFFFFF)
        if noise_out is not None:
            if noise_out.dtype != torch.float32 or tuple(noise_out.shape) != tuple(sample.shape) or noise_out.device != device:
                raise ValueError(f"noise_out must be float32 {tuple(sample.shape)} on {device}")
            no, sno = _per_sample_view(noise_out, "noise_out", writable=True)
            d.noise_out, d.noise_out_stride = N.ptr(no), sno
    ws, ws_bytes = N.workspace(device)
    with N.on_device(device):
        rc = N.F.unirl_sde_step_logp_ex(ctypes.byref(d), N.ptr(ws), ws_bytes, N.current_stream(device))
    N.check(rc, "unirl_sde_step_logp_ex")


def _dense_from(t: torch.Tensor, first_dim: int) -> bool:
    """Whether dimensions ``first_dim ..`` of ``t`` form one contiguous run (``t[0, .., 0].is_contiguous()``
    without making the view)."""
    shape, strides, expect = t.shape, t.stride(), 1
    for k in range(t.dim() - 1, first_dim - 1, -1):
        if shape[k] != 1 and strides[k] != expect:
            return False
        expect *= shape[k]
    return True


@functools.lru_cache(maxsize=256)
def _replay_slot_arrays(slots_x: tuple, slots_p: tuple, K: int):
    """The two checked slot tables of a replay as C arrays (the same few tuples come back call after call)."""
    slots_x, slots_p = [int(k) for k in slots_x], [int(k) for k in slots_p]
    S = len(slots_x)
    if S < 1 or len(slots_p) != S:
        raise ValueError(f"slot_sample and slot_prev must name the same, non-zero number of steps; got {S} and {len(slots_p)}")
    if S > N.MAX_ROLLOUT_STEPS:
        raise ValueError(f"at most {N.MAX_ROLLOUT_STEPS} steps per replay call; got {S}")
    for k in slots_x + slots_p:
        if not 0 <= k < K:
            raise ValueError(f"slot {k} is outside the stack's {K} slots")
    return (ctypes.c_int64 * S)(*slots_x), (ctypes.c_int64 * S)(*slots_p), S


def _blocks_disjoint(stride_a: int, n_a: int, stride_b: int, n_b: int, block: int) -> bool:
    """Whether the ``n_a x n_b`` blocks of ``block`` contiguous elements at offsets
    ``i * stride_a + j * stride_b`` are pairwise disjoint (positive strides; an extent of 1 leaves
    its stride free)."""
    dims = sorted((s, n) for s, n in ((stride_a, n_a), (stride_b, n_b)) if n > 1)
    span = block
    for stride, n in dims:  # inner dimension first: each must step past everything nested inside it
        if stride < span:
            return False
        span = (n - 1) * stride + span
    return True


def _replay_desc(noise_pred, latents, slot_sample, slot_prev, sigma, sigma_next, kind, eta, sigma_max, step_major):
    """Checked operands and the filled ``unirl_sde_replay_desc`` of a batched replay; returns
    ``(desc, keepalive, B, S, D, shape_tail)``."""
    N.require_device(latents, "latents")
    N.require_device(noise_pred, "noise_pred")
    if latents.dim() < 3:
        raise ValueError(f"latents must be a [B, K, ...] trajectory stack; got {tuple(latents.shape)}")
    device = latents.device
    B, K = int(latents.shape[0]), int(latents.shape[1])
    tail = tuple(latents.shape[2:])
    D = int(math.prod(tail))
    arr_x, arr_p, S = _replay_slot_arrays(tuple(slot_sample), tuple(slot_prev), K)
    want = ((S, B) if step_major else (B, S)) + tail
    if tuple(noise_pred.shape) != want:
        raise ValueError(f"noise_pred {tuple(noise_pred.shape)} != {want}")
    # only addresses are used: a detached alias is made only where a cast or a copy may follow
    v = noise_pred.detach() if noise_pred.requires_grad else noise_pred
    if v.dtype not in N._DTYPE_CODE:
        v = v.float()
    x = latents.detach() if latents.requires_grad else latents
    if x.dtype not in N._DTYPE_CODE:
        x = x.float()
    # every (sample, step) block must be one contiguous run of D elements.  The two leading strides
    # are free, except that 0 means "dense" in the C ABI: a tensor broadcast over the samples or the
    # steps is copied, as is a stack whose slots overlap
    b_dim, s_dim = (1, 0) if step_major else (0, 1)
    # The velocities' gradient is written in the velocities' own layout, so their (sample, step)
    # blocks must also be pairwise disjoint: a view whose samples (or steps) overlap would have its
    # overlapping gradient rows written concurrently, where autograd expects their sum.
    if B and not (_dense_from(v, 2) and _blocks_disjoint(v.stride(b_dim), B, v.stride(s_dim), S, D)):
        v = v.contiguous()
    if B and not (_dense_from(x, 2) and (B == 1 or x.stride(0) >= 1) and (K == 1 or x.stride(1) >= D)):
        x = x.contiguous()

    def steps_f32(t, name):
        if (isinstance(t, torch.Tensor) and t.dtype is torch.float32 and t.device == device and t.dim() == 1
                and t.shape[0] == S and t.stride(0) == 1 and not t.requires_grad):
            return t  # already what the kernel reads
        if not isinstance(t, torch.Tensor):
            t = torch.tensor([float(a) for a in t], dtype=torch.float32)
        t = t.detach().to(device=device, dtype=torch.float32).reshape(-1).contiguous()
        if t.numel() != S:
            raise ValueError(f"{name} must hold one value per step ({S}); got {t.numel()}")
        return t

    sig, sig_n = steps_f32(sigma, "sigma"), steps_f32(sigma_next, "sigma_next")
    smax_t, smax_v = _sigma_max_arg(sigma_max, device)
    d = N.SdeReplayDesc()
    vs, xs = v.stride(), x.stride()
    t = d.noise_pred
    t.ptr, t.dtype, t.sample_stride = v.data_ptr(), N.dtype_code(v.dtype), (vs[b_dim] if B > 1 else S * D)
    d.noise_pred_step_stride = vs[s_dim] if S > 1 else D
    t = d.latents
    t.ptr, t.dtype, t.sample_stride = x.data_ptr(), N.dtype_code(x.dtype), (xs[0] if B > 1 else 0)
    d.latents_slot_stride = xs[1] if K > 1 else 0
    d.K = K
    d.slot_sample, d.slot_prev = arr_x, arr_p
    d.sigma, d.sigma_next = N.ptr(sig), N.ptr(sig_n)
    d.sigma_max_ptr, d.sigma_max_val = N.ptr(smax_t), smax_v
    d.eta, d.kind = float(eta), SDE_KINDS[kind]
    d.B, d.S, d.D = B, S, D
    return d, (v, x, sig, sig_n, smax_t, arr_x, arr_p), B, S, D, tail


def sde_replay_logp(
    noise_pred: torch.Tensor,
    latents: torch.Tensor,
    slot_sample: Sequence[int],
    slot_prev: Sequence[int],
    sigma,
    sigma_next,
    *,
    kind: str = "flow",
    eta: float = 1.0,
    sigma_max: Union[float, torch.Tensor] = 0.99,
    step_major: bool = False,
    want_means: bool = True,
    means_dtype: Optional[torch.dtype] = None,
    logp_sum: bool = False,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """The replay of ``S`` recorded steps of every sample in one launch: ``(log_probs [B, S] fp32 or
    None when eta < 1e-7, means [B, S, ...] in means_dtype or None)``.

    ``noise_pred`` is ``[B, S, ...]`` (``[S, B, ...]`` with ``step_major``); ``latents`` the
    ``[B, K, ...]`` trajectory stack, read in place: step ``j`` starts from slot ``slot_sample[j]``
    and its stored next latent is slot ``slot_prev[j]``; ``sigma`` / ``sigma_next`` hold one value
    per step.  ``means_dtype`` defaults to the stack's dtype (the reference stores
    ``stack(means).to(trajectory_dtype)``)."""
    d, keep, B, S, D, tail = _replay_desc(noise_pred, latents, slot_sample, slot_prev, sigma, sigma_next, kind, eta,
                                          sigma_max, step_major)
    device = latents.device
    x = keep[1]
    mdt = means_dtype if means_dtype is not None else x.dtype
    if want_means and mdt not in N._DTYPE_CODE:
        raise TypeError(f"means_dtype {mdt} is not float32, bfloat16 or float16")
    means = torch.empty((B, S) + tail, dtype=mdt, device=device) if want_means else None
    logp = None if eta < 1e-7 else torch.empty((B, S), dtype=torch.float32, device=device)
    if B == 0 or D == 0:
        return logp, means
    d.mean_out, d.mean_dtype = N.ptr(means), (N.dtype_code(mdt) if want_means else 0)
    d.logp_out, d.logp_sum = N.ptr(logp), int(bool(logp_sum))
    stream = N.current_stream(device)
    ws, ws_bytes = N.workspace(device, stream)
    with N.on_device(device):
        rc = N.F.unirl_sde_replay_logp(ctypes.byref(d), N.ptr(ws), ws_bytes, stream)
    N.check(rc, "unirl_sde_replay_logp")
    return logp, means


def sde_replay_logp_bwd(
    noise_pred: torch.Tensor,
    latents: torch.Tensor,
    slot_sample: Sequence[int],
    slot_prev: Sequence[int],
    sigma,
    sigma_next,
    *,
    kind: str,
    eta: float,
    sigma_max,
    step_major: bool,
    g_logp: Optional[torch.Tensor],
    g_mean: Optional[torch.Tensor],
    logp_sum: bool = False,
) -> torch.Tensor:
    """Gradient of :func:`sde_replay_logp` with respect to ``noise_pred`` (same shape and dtype; the
    latents are stored data and take no gradient)."""
    d, keep, B, S, D, tail = _replay_desc(noise_pred, latents, slot_sample, slot_prev, sigma, sigma_next, kind, eta,
                                          sigma_max, step_major)
    device = latents.device
    v = keep[0]
    out_dtype = noise_pred.dtype if noise_pred.dtype in N._DTYPE_CODE else torch.float32
    # the gradient takes the velocity's layout: same strides as the tensor the kernel reads
    grad = torch.empty_strided(v.shape, v.stride(), dtype=out_dtype, device=device)
    if B == 0 or D == 0:
        return grad

    def f32c(t, shape):  # the upstream gradients come in the outputs' [B, S, ...] layout
        return None if t is None else t.detach().to(device=device, dtype=torch.float32).reshape(shape).contiguous()

    gl = f32c(g_logp, (B, S))
    gm = f32c(g_mean, (B, S, D))
    d.logp_sum = int(bool(logp_sum))
    with N.on_device(device):
        rc = N.F.unirl_sde_replay_logp_bwd(ctypes.byref(d), N.ptr(gl), N.ptr(gm), N.ptr(grad),
                                               N.dtype_code(out_dtype), N.current_stream(device))
    N.check(rc, "unirl_sde_replay_logp_bwd")
    return grad if grad.dtype == noise_pred.dtype else grad.to(noise_pred.dtype)


def sde_step_logp_bwd(
    noise_pred: torch.Tensor,
    sample: torch.Tensor,
    sigma: torch.Tensor,
    sigma_next: torch.Tensor,
    *,
    kind: str,
    eta: float,
    prev_sample: Optional[torch.Tensor],
    noise: Optional[torch.Tensor],
    sigma_max,
    g_logp: Optional[torch.Tensor],
    g_mean: Optional[torch.Tensor],
    g_prev: Optional[torch.Tensor],
    need_grad_v: bool,
    need_grad_x: bool,
    logp_sum: bool = False,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Gradients of :func:`sde_step_logp` w.r.t. ``noise_pred`` and ``sample``, each written by the
    kernel in its tensor's own dtype (fp32 for dtypes the kernel does not read directly)."""
    device = sample.device
    v = _flat2(noise_pred.detach(), "noise_pred")
    x = _flat2(sample.detach(), "sample")
    if v.dtype not in N._DTYPE_CODE:
        v = v.float()
    if x.dtype not in N._DTYPE_CODE:
        x = x.float()
    B = x.shape[0]
    D = x.numel() // B if B else 0
    prev_in = None if prev_sample is None else _flat2(prev_sample.detach(), "prev_sample").to(x.dtype)
    nz = None if (noise is None or prev_sample is not None) else _flat2(noise.detach(), "noise").float()
    sig, stride = _sigma_arg(sigma, B, device, "sigma")
    sig_n, stride_n = _sigma_arg(sigma_next, B, device, "sigma_next")
    if stride != stride_n:
        if stride == 0:
            sig, stride = sig.expand(B).contiguous(), 1
        else:
            sig_n = sig_n.expand(B).contiguous()
    smax_t, smax_v = _sigma_max_arg(sigma_max, device)

    def f32c(t):
        return None if t is None else t.detach().to(device=device, dtype=torch.float32).contiguous()

    gl, gm, gp = f32c(g_logp), f32c(g_mean), f32c(g_prev)
    grad_v = torch.empty(x.shape, dtype=v.dtype, device=device) if need_grad_v else None
    grad_x = torch.empty(x.shape, dtype=x.dtype, device=device) if need_grad_x else None
    if B == 0 or D == 0 or (grad_v is None and grad_x is None):
        return grad_v, grad_x
    if gl is None and gm is None and gp is None:  # nothing flows back
        return (None if grad_v is None else grad_v.zero_()), (None if grad_x is None else grad_x.zero_())
    with N.on_device(device):
        rc = N.F.unirl_sde_step_logp_bwd(
            N.ptr(v), N.dtype_code(v.dtype), N.ptr(x), N.dtype_code(x.dtype), N.ptr(prev_in), N.ptr(nz),
            N.ptr(sig), N.ptr(sig_n), stride, N.ptr(smax_t), smax_v, float(eta), SDE_KINDS[kind], B, D,
            N.ptr(gl), N.ptr(gm), N.ptr(gp), int(bool(logp_sum)), N.ptr(grad_v), N.dtype_code(v.dtype),
            N.ptr(grad_x), N.dtype_code(x.dtype), N.current_stream(device),
        )
    N.check(rc, "unirl_sde_step_logp_bwd")
    return grad_v, grad_x


def sde_rollout_logp(
    x0: torch.Tensor,
    velocities: Sequence[torch.Tensor],
    noises: Sequence[Optional[torch.Tensor]],
    sigmas: torch.Tensor,
    etas: Union[float, Sequence[float]],
    *,
    kind: str = "flow",
    sigma_max: Union[float, torch.Tensor, None] = None,
    want_trajectory: bool = False,
    logp_sum: bool = False,
    rng: Optional[Tuple[int, int]] = None,
    noise_out: Optional[Sequence[Optional[torch.Tensor]]] = None,
) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """``S = len(velocities)`` chained transitions in one launch.

    Step ``k`` moves ``sigmas[k] -> sigmas[k+1]`` with ``velocities[k]``, ``noises[k]``
    and ``etas[k]``.  ``sigma_max=None`` takes ``sigmas[1]`` like the reference's stage
    loop.  With ``rng = (seed, offset)`` a stochastic step whose ``noises[k]`` is ``None`` (or all
    of them: ``noises=None``) draws its noise inside the kernel, step ``k`` with ``offset + k`` --
    the draws of ``k`` single steps called with those offsets; ``noise_out[k]`` (fp32, ``x0``'s
    shape) receives a step's drawn noise when given.  Returns ``(x_final f32, logp [B,S] f32 (NaN
    where eta<1e-7), trajectory [S,B,...] f32 or None)``.
    """
    S = len(velocities)
    if S < 1 or S > N.MAX_ROLLOUT_STEPS:
        raise ValueError(f"number of steps must be in [1, {N.MAX_ROLLOUT_STEPS}]; got {S}")
    if noises is None:
        if rng is None:
            raise ValueError("noises=None needs rng=(seed, offset)")
        noises = [None] * S
    if len(noises) != S:
        raise ValueError(f"{S} velocities but {len(noises)} noises")
    if isinstance(etas, (int, float)):
        etas = [float(etas)] * S
    if len(etas) != S:
        raise ValueError(f"{S} velocities but {len(etas)} etas")
    device = x0.device
    x = _flat2(x0.detach(), "x0")
    if x.dtype not in N._DTYPE_CODE:
        x = x.float()
    B = x.shape[0]
    D = x.numel() // B if B else 0
    sig = sigmas.detach().to(device=device, dtype=torch.float32).reshape(-1).contiguous()
    if sig.numel() < S + 1:
        raise ValueError(f"sigmas needs {S + 1} values for {S} steps; got {sig.numel()}")
    if sigma_max is None:
        smax_t, smax_v = sig[1:2], 0.0
    else:
        smax_t, smax_v = _sigma_max_arg(sigma_max, device)
    vs: List[torch.Tensor] = []
    ns: List[Optional[torch.Tensor]] = []
    vdtype = None
    for k in range(S):
        vk = _flat2(velocities[k].detach(), f"velocities[{k}]")
        if vk.shape != x.shape:
            raise ValueError(f"velocities[{k}] {tuple(vk.shape)} != x0 {tuple(x.shape)}")
        if vk.dtype not in N._DTYPE_CODE:
            vk = vk.float()
        if vdtype is None:
            vdtype = vk.dtype
        elif vk.dtype != vdtype:
            vk = vk.to(vdtype)
        vs.append(vk)
        nk = noises[k]
        if nk is not None:
            if nk.shape != x.shape:
                raise ValueError(f"noises[{k}] {tuple(nk.shape)} != x0 {tuple(x.shape)}")
            nk = _flat2(nk.detach(), f"noises[{k}]").float()
        ns.append(nk)
    x_out = torch.empty(x.shape, dtype=torch.float32, device=device)
    logp = torch.empty((B, S), dtype=torch.float32, device=device)
    traj = torch.empty((S,) + tuple(x.shape), dtype=torch.float32, device=device) if want_trajectory else None
    if B == 0 or D == 0:
        return x_out, logp, traj
    v_arr = (ctypes.c_void_p * S)(*[t.data_ptr() for t in vs])
    n_arr = (ctypes.c_void_p * S)(*[(t.data_ptr() if t is not None else None) for t in ns])
    e_arr = (ctypes.c_double * S)(*[float(e) for e in etas])
    rng_s, no_arr = None, None
    if rng is not None:
        rng_s = ctypes.byref(N.Rng(1, int(rng[0]) & 0xFFFFFFFFFFFFFFFF, int(rng[1]) & 0xFFFFFFFFFFFFFFFF))
        if noise_out is not None:
            if len(noise_out) != S:
                raise ValueError(f"{S} steps but {len(noise_out)} noise_out entries")
            for k, t in enumerate(noise_out):
                if t is not None and (t.dtype != torch.float32 or tuple(t.shape) != tuple(x0.shape) or not t.is_contiguous()
                                      or t.device != device):
                    raise ValueError(f"noise_out[{k}] must be a contiguous float32 tensor of x0's shape on {device}")
            no_arr = (ctypes.c_void_p * S)(*[(t.data_ptr() if t is not None else None) for t in noise_out])
    ws, ws_bytes = N.workspace(device)
    with N.on_device(device):
        rc = N.F.unirl_sde_rollout_logp(
            N.ptr(x), N.dtype_code(x.dtype), v_arr, N.dtype_code(vdtype), n_arr, rng_s, no_arr, N.ptr(sig), e_arr, S,
            N.ptr(smax_t), smax_v, SDE_KINDS[kind], B, D, N.ptr(x_out), N.ptr(traj), N.ptr(logp),
            int(bool(logp_sum)), N.ptr(ws), ws_bytes, N.current_stream(device),
        )
    N.check(rc, "unirl_sde_rollout_logp")
    return x_out, logp, traj


def dpm2_step(
    model_output: torch.Tensor,
    sample: torch.Tensor,
    x0_prev: Optional[torch.Tensor],
    branch: int,
    coeffs: "N.Dpm2Coeffs",
    x0_out: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """One DPM-Solver-2 update: ``(x0 prediction, prev_sample)``, both fp32 in ``sample``'s shape.

    ``x0_prev`` is the previous step's prediction (second-order branch only); ``x0_out`` may name
    a reusable fp32 buffer for the new one (not ``x0_prev``)."""
    N.require_device(sample, "sample")
    if model_output.shape != sample.shape:
        raise ValueError(f"model_output {tuple(model_output.shape)} != sample {tuple(sample.shape)}")
    device = sample.device
    v = model_output.detach().to(device).contiguous()
    x = sample.detach().contiguous()
    if v.dtype not in N._DTYPE_CODE:
        v = v.float()
    if x.dtype not in N._DTYPE_CODE:
        x = x.float()
    m1 = None
    if branch == N.DPM2_SECOND:
        if x0_prev is None or x0_prev.shape != sample.shape:
            raise ValueError("the second-order update needs the previous x0 prediction in the sample's shape")
        m1 = x0_prev.detach().to(device=device, dtype=torch.float32).contiguous()
    if x0_out is None or x0_out.shape != sample.shape or x0_out.dtype != torch.float32 or not x0_out.is_contiguous():
        x0_out = torch.empty(sample.shape, dtype=torch.float32, device=device)
    if m1 is not None and x0_out.data_ptr() == m1.data_ptr():
        raise ValueError("x0_out must not alias x0_prev")
    prev = torch.empty(sample.shape, dtype=torch.float32, device=device)
    with N.on_device(device):
        rc = N.F.unirl_dpm2_step(
            N.ptr(v), N.dtype_code(v.dtype), N.ptr(x), N.dtype_code(x.dtype), N.ptr(m1), int(branch),
            ctypes.byref(coeffs), x.numel(), N.ptr(x0_out), N.ptr(prev), N.current_stream(device),
        )
    N.check(rc, "unirl_dpm2_step")
    return x0_out, prev


def gaussian_kl_mask(
    p: torch.Tensor,
    q: torch.Tensor,
    sigma: torch.Tensor,
    threshold: float,
    *,
    reduce_from_dim: int = 2,
    want_mask: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Per-row mean of ``(p-q)^2 / (2 sigma^2)`` and ``kl < threshold``.

    Rows are the leading ``reduce_from_dim`` dimensions of ``p``; ``sigma`` holds one
    value, or one per index of the LAST leading dimension (``[1,S',1,...]``).
    """
    if p.shape != q.shape:
        raise ValueError(f"p {tuple(p.shape)} != q {tuple(q.shape)}")
    if p.dim() <= reduce_from_dim:
        raise ValueError(f"need more than {reduce_from_dim} dims to reduce over; got {tuple(p.shape)}")
    device = p.device
    pc = _kernel_dtype(_flat2(p, "p"))
    qc = _flat2(q, "q")
    if qc.dtype is not pc.dtype:
        qc = qc.detach().to(pc.dtype)
    lead = tuple(pc.shape[:reduce_from_dim])
    R = int(math.prod(lead))
    D = pc.numel() // R if R else 0
    sig = N.as_operand(sigma, torch.float32, device)  # the kernel reads it flat, whatever its shape
    if sig.numel() not in (1, lead[-1]):
        raise ValueError(f"sigma must hold 1 or {lead[-1]} values; got {tuple(sigma.shape)}")
    kl = torch.empty(lead, dtype=torch.float32, device=device)
    mask = torch.empty(lead, dtype=torch.bool, device=device) if want_mask else None
    if R == 0 or D == 0:
        return kl, mask
    stream = N.current_stream(device)
    ws, ws_bytes = N.workspace(device, stream)
    with N.on_device(device):
        rc = N.F.unirl_gaussian_kl_mask(
            N.ptr(pc), N.ptr(qc), N.dtype_code(pc.dtype), N.ptr(sig), sig.numel(), R, D, float(threshold),
            N.ptr(kl), N.ptr(mask), N.ptr(ws), ws_bytes, stream,
        )
    N.check(rc, "unirl_gaussian_kl_mask")
    return kl, mask


FLOWDPPO_METRIC_SLOTS = {
    "ratio_mean": 0,
    "ratio_std": 1,
    "ratio_min": 2,
    "ratio_max": 3,
    "approx_kl": 4,
    "kl_new_old_mean": 5,
    "kl_new_old_max": 6,
    "kl_mask_fraction": 7,
    "pos_rm_fraction": 8,
    "neg_rm_fraction": 9,
    "masked_fraction": 10,
    "unmasked_fraction": 11,
    "loss_mean": 12,
}


def flowdppo_loss(
    new_logp: torch.Tensor, old_logp: torch.Tensor, advantages: torch.Tensor, kl: torch.Tensor, threshold: float
) -> Tuple[torch.Tensor, torch.Tensor]:
    """KL-ADV masked loss per element (same shape as ``new_logp``) and the metrics vector [16]."""
    N.require_device(new_logp, "new_logp")
    device = new_logp.device
    shape = tuple(new_logp.shape)

    def f32c(t, name):
        t = t.detach().to(device=device, dtype=torch.float32)
        if tuple(t.shape) != shape:
            t = t.expand(shape)
        return t.contiguous()

    nw, od = f32c(new_logp, "new_logp"), f32c(old_logp, "old_logp")
    ad, klc = f32c(advantages, "advantages"), f32c(kl, "kl")
    elem = torch.empty(shape, dtype=torch.float32, device=device)
    metrics = torch.empty(N.M_COUNT, dtype=torch.float32, device=device)
    with N.on_device(device):
        rc = N.F.unirl_flowdppo_loss(
            N.ptr(nw), N.ptr(od), N.ptr(ad), N.ptr(klc), nw.numel(), float(threshold), N.ptr(elem),
            N.ptr(metrics), N.current_stream(device),
        )
    N.check(rc, "unirl_flowdppo_loss")
    return elem, metrics


FLOWDPPO_STEP_MAX_ROWS = 4096
FLOWDPPO_REPLAY_MAX_ROWS = 2048  # unirl_flowdppo_replay_step: (sample, step) rows per call


def flowdppo_step(
    new_logp: torch.Tensor,
    old_logp: torch.Tensor,
    new_means: torch.Tensor,
    old_means: torch.Tensor,
    advantages: torch.Tensor,
    sigma_t: torch.Tensor,
    threshold: float,
    *,
    loss_scale: Optional[float] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """KL over the means, KL-ADV masked loss and metrics in two launches.

    ``new_logp`` / ``old_logp`` / ``advantages`` are ``[B, S']`` (advantages may broadcast), the
    means ``[B, S', ...]``, ``sigma_t`` one value or one per step.  Returns ``(kl [B,S'],
    loss_elem [B,S'], metrics [16], grad_new [B,S'] or None)`` in fp32; with ``loss_scale``
    given, ``grad_new`` is what ``(loss_elem.mean() * loss_scale).backward()`` leaves in
    ``new_logp``.  At most ``FLOWDPPO_STEP_MAX_ROWS`` rows.
    """
    N.require_device(new_logp, "new_logp")
    if new_means.shape != old_means.shape:
        raise ValueError(f"new_means {tuple(new_means.shape)} != old_means {tuple(old_means.shape)}")
    if new_logp.dim() != 2 or tuple(new_means.shape[:2]) != tuple(new_logp.shape) or new_means.dim() < 3:
        raise ValueError(
            f"need log-probs [B, S'] and means [B, S', ...]; got {tuple(new_logp.shape)} and {tuple(new_means.shape)}"
        )
    device = new_logp.device
    shape = tuple(new_logp.shape)
    R = shape[0] * shape[1]
    if R == 0 or R > FLOWDPPO_STEP_MAX_ROWS:
        raise ValueError(f"flowdppo_step handles 1..{FLOWDPPO_STEP_MAX_ROWS} rows; got {R}")
    pc = _kernel_dtype(_flat2(new_means, "new_means"))
    qc = _flat2(old_means, "old_means")
    if qc.dtype is not pc.dtype:
        qc = qc.detach().to(pc.dtype)
    D = pc.numel() // R
    sig = N.as_operand(sigma_t, torch.float32, device)  # read flat by the kernel
    if sig.numel() not in (1, shape[1]):
        raise ValueError(f"sigma_t must hold 1 or {shape[1]} values; got {tuple(sigma_t.shape)}")

    def f32c(t):
        if tuple(t.shape) != shape:
            t = t.detach().expand(shape)
        return N.as_operand(t, torch.float32, device)

    nw, od, ad = f32c(new_logp), f32c(old_logp), f32c(advantages)
    # the three [B, S'] outputs are a few dozen floats that live and die together: one allocation
    kl, elem, grad = torch.empty((3,) + shape, dtype=torch.float32, device=device).unbind(0)
    if loss_scale is None:
        grad = None
    metrics = torch.empty(N.M_COUNT, dtype=torch.float32, device=device)
    stream = N.current_stream(device)
    ws, ws_bytes = N.workspace(device, stream)
    with N.on_device(device):
        rc = N.F.unirl_flowdppo_step(
            N.ptr(pc), N.ptr(qc), N.dtype_code(pc.dtype), N.ptr(sig), sig.numel(), R, D, N.ptr(nw), N.ptr(od),
            N.ptr(ad), float(threshold), float(loss_scale or 0.0), N.ptr(kl), N.ptr(elem), N.ptr(grad),
            N.ptr(metrics), N.ptr(ws), ws_bytes, stream,
        )
    N.check(rc, "unirl_flowdppo_step")
    return kl, elem, metrics, grad


def flowdppo_replay_step(
    noise_pred: torch.Tensor,
    latents: torch.Tensor,
    slot_sample: Sequence[int],
    slot_prev: Sequence[int],
    sigma,
    sigma_next,
    old_logp: torch.Tensor,
    old_means: torch.Tensor,
    advantages: torch.Tensor,
    sigma_t: torch.Tensor,
    threshold: float,
    *,
    kind: str = "flow",
    eta: float = 1.0,
    sigma_max: Union[float, torch.Tensor] = 0.99,
    step_major: bool = False,
    loss_scale: Optional[float] = None,
    want_means: bool = False,
    want_mask: bool = False,
):
    """The forward of a Flow-DPPO micro-step from the model's velocities, as one streaming pass and
    one finishing workgroup: :func:`sde_replay_logp` and :func:`flowdppo_step` without the new means
    ever being written or re-read.

    Arguments as :func:`sde_replay_logp` (velocities ``[B, S, ...]``, the ``[B, K, ...]`` stack and
    its slot tables, one sigma pair per step) plus the frozen ``old_logp`` ``[B, S]`` and
    ``old_means`` ``[B, S, ...]``, the advantages (``[B, S]`` or broadcastable), the KL's
    ``sigma_t`` (one value or one per step) and the KL threshold.  Returns a dict with ``logp``
    ``[B, S]``, ``kl`` ``[B, S]``, ``loss_elem`` ``[B, S]``, ``metrics`` ``[16]`` (all fp32), ``grad_logp``
    ``[B, S]`` (``loss_scale`` given: what ``(loss_elem.mean() * loss_scale).backward()`` leaves in the
    new log-probs; hand it to :func:`sde_replay_logp_bwd`), and on request ``means`` (the stack's
    dtype) and ``mask`` (bool, ``kl < threshold``).  At most ``FLOWDPPO_REPLAY_MAX_ROWS`` rows."""
    d, keep, B, S, D, tail = _replay_desc(noise_pred, latents, slot_sample, slot_prev, sigma, sigma_next, kind, eta,
                                          sigma_max, step_major)
    device = latents.device
    x = keep[1]
    R = B * S
    if R == 0 or D == 0 or R > FLOWDPPO_REPLAY_MAX_ROWS:
        raise ValueError(f"flowdppo_replay_step handles 1..{FLOWDPPO_REPLAY_MAX_ROWS} (sample, step) rows; got {R}")
    if eta < 1e-7:
        raise RuntimeError(f"flowdppo_replay_step: eta={eta} is a deterministic step (no log-prob)")
    if tuple(old_means.shape) != (B, S) + tail:
        raise ValueError(f"old_means {tuple(old_means.shape)} != {(B, S) + tail}")
    qm = old_means.detach()
    if qm.dtype is not x.dtype or qm.device != device or not qm.is_contiguous():
        qm = qm.to(device=device, dtype=x.dtype).contiguous()  # the KL is taken in the trajectory dtype
    sig_t = N.as_operand(sigma_t, torch.float32, device)
    if sig_t.numel() not in (1, S):
        raise ValueError(f"sigma_t must hold 1 or {S} values; got {tuple(sigma_t.shape)}")

    def f32c(t):
        if tuple(t.shape) != (B, S):
            t = t.detach().expand((B, S))
        return N.as_operand(t, torch.float32, device)

    od, ad = f32c(old_logp), f32c(advantages)
    logp, kl, elem, grad = torch.empty((4, B, S), dtype=torch.float32, device=device).unbind(0)
    if loss_scale is None:
        grad = None
    metrics = torch.empty(N.M_COUNT, dtype=torch.float32, device=device)
    means = torch.empty((B, S) + tail, dtype=x.dtype, device=device) if want_means else None
    mask = torch.empty((B, S), dtype=torch.bool, device=device) if want_mask else None
    d.mean_out, d.mean_dtype = N.ptr(means), (N.dtype_code(x.dtype) if want_means else 0)
    d.logp_out, d.logp_sum = N.ptr(logp), 0
    stream = N.current_stream(device)
    ws, ws_bytes = N.workspace(device, stream)
    with N.on_device(device):
        rc = N.F.unirl_flowdppo_replay_step(
            ctypes.byref(d), N.ptr(qm), N.ptr(sig_t), sig_t.numel(), N.ptr(od), N.ptr(ad), float(threshold),
            float(loss_scale or 0.0), N.ptr(kl), N.ptr(mask), N.ptr(elem), N.ptr(grad), N.ptr(metrics), N.ptr(ws),
            ws_bytes, stream,
        )
    N.check(rc, "unirl_flowdppo_replay_step")
    return dict(logp=logp, kl=kl, loss_elem=elem, metrics=metrics, grad_logp=grad, means=means, mask=mask)


def expand_per_seq(values: torch.Tensor, cu_seqlens: torch.Tensor, n_tok: int) -> torch.Tensor:
    """``out[t] = values[r]`` for the tokens of packed sequence ``r`` (f32 ``[n_tok]``)."""
    N.require_device(values, "values")
    device = values.device
    v = values.detach().to(torch.float32).reshape(-1).contiguous()
    cu = cu_seqlens.detach().to(device=device, dtype=torch.int64).reshape(-1).contiguous()
    if cu.numel() != v.numel() + 1:
        raise ValueError(f"cu_seqlens needs {v.numel() + 1} entries; got {cu.numel()}")
    out = torch.empty(int(n_tok), dtype=torch.float32, device=device)
    if n_tok:
        with N.on_device(device):
            rc = N.F.unirl_expand_per_seq(
                N.ptr(v), N.ptr(cu), v.numel(), int(n_tok), N.ptr(out), N.current_stream(device)
            )
        N.check(rc, "unirl_expand_per_seq")
    return out


def gaussian_kl_elem(p: torch.Tensor, q: torch.Tensor, sigma: torch.Tensor, *, sigma_dim: int = 1) -> torch.Tensor:
    """Element-wise ``(p-q)^2 / (2 sigma^2)`` as f32; sigma broadcast along ``sigma_dim``."""
    if p.shape != q.shape:
        raise ValueError(f"p {tuple(p.shape)} != q {tuple(q.shape)}")
    device = p.device
    pc = _flat2(p.detach(), "p")
    qc = _flat2(q.detach(), "q").to(pc.dtype)
    if pc.dtype not in N._DTYPE_CODE:
        pc, qc = pc.float(), qc.float()
    sig = sigma.detach().to(device=device, dtype=torch.float32).reshape(-1).contiguous()
    if sig.numel() == 1:
        R, D = 1, pc.numel()
    else:
        if pc.dim() <= sigma_dim or sig.numel() != pc.shape[sigma_dim]:
            raise ValueError(f"sigma {tuple(sigma.shape)} does not match dim {sigma_dim} of {tuple(p.shape)}")
        R = int(math.prod(pc.shape[: sigma_dim + 1]))
        D = pc.numel() // R if R else 0
    out = torch.empty(pc.shape, dtype=torch.float32, device=device)
    if pc.numel() == 0:
        return out
    with N.on_device(device):
        rc = N.F.unirl_gaussian_kl_elem(
            N.ptr(pc), N.ptr(qc), N.dtype_code(pc.dtype), N.ptr(sig), sig.numel(), R, D, N.ptr(out),
            N.current_stream(device),
        )
    N.check(rc, "unirl_gaussian_kl_elem")
    return out


def gaussian_kl_elem_bwd(
    p: torch.Tensor, q: torch.Tensor, sigma: torch.Tensor, g_out: torch.Tensor, *, sigma_dim: int = 1,
    need_p: bool = True, need_q: bool = True,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Gradients of :func:`gaussian_kl_elem` w.r.t. ``p`` and ``q`` (in their dtype)."""
    device = p.device
    pc = _flat2(p.detach(), "p")
    qc = _flat2(q.detach(), "q").to(pc.dtype)
    if pc.dtype not in N._DTYPE_CODE:
        pc, qc = pc.float(), qc.float()
    sig = sigma.detach().to(device=device, dtype=torch.float32).reshape(-1).contiguous()
    if sig.numel() == 1:
        R, D = 1, pc.numel()
    else:
        R = int(math.prod(pc.shape[: sigma_dim + 1]))
        D = pc.numel() // R if R else 0
    g = g_out.detach().to(device=device, dtype=torch.float32).contiguous()
    gp = torch.empty_like(pc) if need_p else None
    gq = torch.empty_like(pc) if need_q else None
    if pc.numel() and (need_p or need_q):
        with N.on_device(device):
            rc = N.F.unirl_gaussian_kl_elem_bwd(
                N.ptr(pc), N.ptr(qc), N.dtype_code(pc.dtype), N.ptr(sig), sig.numel(), R, D, N.ptr(g), N.ptr(gp),
                N.ptr(gq), N.current_stream(device),
            )
        N.check(rc, "unirl_gaussian_kl_elem_bwd")
    return gp, gq


def token_logp_entropy(
    logits: torch.Tensor,
    ids: Optional[torch.Tensor],
    temperature: float = 1.0,
    *,
    want_logp: bool = True,
    want_entropy: bool = True,
    want_lse: bool = False,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor]]:
    """``(logp, entropy, logsumexp)`` per row of ``logits [..., V]``, each f32 ``[...]``."""
    N.require_device(logits, "logits")
    if logits.dim() < 1:
        raise ValueError("logits needs a vocabulary dimension")
    device = logits.device
    V = logits.shape[-1]
    lead = tuple(logits.shape[:-1])
    x = _kernel_dtype(logits)
    idc = None
    if want_logp:
        if ids is None:
            raise ValueError("ids is required for the log-prob")
        if tuple(ids.shape) != lead:
            raise ValueError(f"ids {tuple(ids.shape)} does not match logits rows {lead}")
        idc = N.as_operand(ids, torch.int64, device).reshape(-1)
    logp = torch.empty(lead, dtype=torch.float32, device=device) if want_logp else None
    ent = torch.empty(lead, dtype=torch.float32, device=device) if want_entropy else None
    lse = torch.empty(lead, dtype=torch.float32, device=device) if want_lse else None
    n_rows = math.prod(lead)
    if n_rows == 0:
        return logp, ent, lse
    if V == 0:
        raise ValueError("empty vocabulary")

    def flat(t):
        return None if t is None else t.reshape(-1)

    stream = N.current_stream(device)
    if x.is_contiguous():  # the usual case: one block, every tensor handed over whole
        with N.on_device(device):
            rc = N.F.unirl_token_logp_entropy(
                x.data_ptr(), N.dtype_code(x.dtype), n_rows, V, V, N.ptr(idc), float(temperature), N.ptr(logp),
                N.ptr(ent), N.ptr(lse), stream,
            )
        N.check(rc, "unirl_token_logp_entropy")
        return logp, ent, lse
    # One launch per block of rows that share a row stride.  `[B, S, V][:, :-1]` (the shifted
    # logits of a training step) is B such blocks: reading it in place costs B launches, flattening
    # it would cost a copy of the logits.
    off = 0
    with N.on_device(device):
        for x2 in _row_blocks(x, V):
            rows = x2.shape[0]
            row_stride = x2.stride(0) if rows > 1 else V

            def part(t):
                return None if t is None else t[off : off + rows]

            rc = N.F.unirl_token_logp_entropy(
                N.ptr(x2), N.dtype_code(x2.dtype), rows, V, row_stride, N.ptr(part(idc)), float(temperature),
                N.ptr(part(flat(logp))), N.ptr(part(flat(ent))), N.ptr(part(flat(lse))), stream,
            )
            N.check(rc, "unirl_token_logp_entropy")
            off += rows
    return logp, ent, lse


def transpose_2d(src: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """A contiguous ``[cols, rows]`` transposed copy of a 2-D tensor of 2- or 4-byte elements whose
    rows are dense (``src.stride(1) == 1``; the row stride is free)."""
    if src.dim() != 2 or not src.is_cuda or src.element_size() not in (2, 4):
        raise ValueError(f"transpose_2d needs a 2-D HIP tensor of 2- or 4-byte elements, got {src.dtype} {tuple(src.shape)}")
    rows, cols = int(src.shape[0]), int(src.shape[1])
    s = src.detach()
    if rows > 1 and cols > 0 and (s.stride(1) != 1 or s.stride(0) < cols):
        s = s.contiguous()
    if out is None:
        out = torch.empty((cols, rows), dtype=src.dtype, device=src.device)
    elif tuple(out.shape) != (cols, rows) or out.dtype != src.dtype or out.device != src.device or not out.is_contiguous():
        raise ValueError("transpose_2d: out must be a contiguous [cols, rows] tensor of the source's dtype and device")
    if rows == 0 or cols == 0:
        return out
    with N.on_device(src.device):
        N.check(
            N.F.unirl_transpose_2d(s.data_ptr(), int(s.stride(0)) if rows > 1 else cols, out.data_ptr(), rows, rows, cols,
                                   src.element_size(), N.current_stream(src.device)),
            "unirl_transpose_2d",
        )
    return out


def lmhead_logp_supported(hidden: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> bool:
    """Whether :func:`lmhead_logp` takes these operands as they are: bf16 on one HIP device, the
    hidden size a multiple of 64, rows contiguous and 16-byte aligned."""
    if not (hidden.is_cuda and weight.is_cuda and hidden.device == weight.device):
        return False
    if hidden.dtype is not torch.bfloat16 or weight.dtype is not torch.bfloat16 or weight.dim() != 2:
        return False
    K = weight.shape[1]
    if hidden.dim() < 1 or hidden.shape[-1] != K or K % 64 != 0 or weight.stride(1) != 1 or weight.stride(0) % 8 != 0:
        return False
    if bias is not None and (bias.dtype is not torch.bfloat16 or bias.numel() != weight.shape[0] or not bias.is_cuda):
        return False
    return weight.data_ptr() % 16 == 0


def lmhead_logp(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    ids: Optional[torch.Tensor],
    temperature: float = 1.0,
    *,
    want_logp: bool = True,
    want_entropy: bool = False,
    want_lse: bool = False,
    want_logits: bool = False,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor]]:
    """``(logp, entropy, logsumexp, logits)`` of ``F.linear(hidden, weight, bias)`` per row, without
    writing the logits (``want_logits`` writes them as well, for validation).  bf16 ``hidden [..., K]``
    and ``weight [V, K]``; the statistics are fp32 ``[...]``."""
    if not lmhead_logp_supported(hidden, weight, bias):
        raise ValueError(
            "lmhead_logp needs bf16 hidden states [..., K] and a bf16 weight [V, K] on one HIP device, K a multiple "
            f"of 64, 16-byte aligned rows; got {hidden.dtype} {tuple(hidden.shape)} and {weight.dtype} {tuple(weight.shape)}"
        )
    device = hidden.device
    V, K = int(weight.shape[0]), int(weight.shape[1])
    lead = tuple(hidden.shape[:-1])
    h2 = hidden.detach().reshape(-1, K)
    if h2.shape[0] and (h2.stride(1) != 1 or h2.stride(0) % 8 != 0 or h2.data_ptr() % 16 != 0):
        h2 = h2.contiguous()
    rows = int(h2.shape[0])
    idc = None
    if want_logp:
        if ids is None:
            raise ValueError("ids is required for the log-prob")
        if tuple(ids.shape) != lead:
            raise ValueError(f"ids {tuple(ids.shape)} does not match the hidden-state rows {lead}")
        idc = N.as_operand(ids, torch.int64, device).reshape(-1)
    logp = torch.empty(lead, dtype=torch.float32, device=device) if want_logp else None
    ent = torch.empty(lead, dtype=torch.float32, device=device) if want_entropy else None
    lse = torch.empty(lead, dtype=torch.float32, device=device) if want_lse else None
    logits = torch.empty(lead + (V,), dtype=torch.bfloat16, device=device) if want_logits else None
    if rows == 0:
        return logp, ent, lse, logits
    nbytes = int(N.F.unirl_lmhead_logp_scratch_bytes(rows, V))
    scratch = torch.empty(nbytes, dtype=torch.uint8, device=device)
    b = None if bias is None else bias.detach().contiguous()
    with N.on_device(device):
        rc = N.F.unirl_lmhead_logp(
            h2.data_ptr(), h2.stride(0) if rows > 1 else K, weight.data_ptr(), weight.stride(0), N.ptr(b), rows, V, K,
            N.ptr(idc), float(temperature), N.ptr(logp), N.ptr(ent), N.ptr(lse), N.ptr(logits), V, scratch.data_ptr(),
            nbytes, N.current_stream(device),
        )
    N.check(rc, "unirl_lmhead_logp")
    return logp, ent, lse, logits


def _row_blocks(x: torch.Tensor, V: int):
    """``x [..., V]`` as a sequence of 2-D ``[rows, V]`` views, in row-major order of the leading
    dimensions, each with unit element stride and one row stride >= V.  A tensor that is one such
    block yields itself; a batch of them (a slice along an inner dimension) yields one per batch
    entry; anything else is copied once."""
    if x.stride(-1) == 1 or x.shape[-1] == 1:
        try:
            x2 = x.view(-1, V)
            if x2.shape[0] <= 1 or x2.stride(0) >= V:
                yield x2
                return
        except RuntimeError:
            pass
        if x.dim() >= 3 and x.shape[0] <= 64:
            for b in range(x.shape[0]):
                yield from _row_blocks(x[b], V)
            return
    yield x.reshape(-1, V).contiguous()


def token_logp_bwd(
    logits: torch.Tensor, ids: torch.Tensor, temperature: float, lse: torch.Tensor, g_logp: torch.Tensor,
    *, in_place: bool = False,
) -> torch.Tensor:
    """``d logp / d logits`` contracted with ``g_logp``, in the dtype of ``logits``.

    ``in_place`` overwrites ``logits`` with its gradient (every element is read and written by
    the same lane, so no second ``[rows, V]`` buffer is needed); it needs contiguous logits in a
    dtype the kernel reads directly."""
    N.require_device(logits, "logits")
    device = logits.device
    V = logits.shape[-1]
    x = logits.detach()
    orig_dtype = x.dtype
    if x.dtype not in N._DTYPE_CODE:
        x = x.float()
    n_rows = math.prod(logits.shape[:-1])
    idc = ids.detach().to(device=device, dtype=torch.int64).reshape(-1).contiguous()
    lsec = lse.detach().to(device=device, dtype=torch.float32).reshape(-1).contiguous()
    gc = g_logp.detach().to(device=device, dtype=torch.float32).reshape(-1).contiguous()
    if in_place:
        if not x.is_contiguous() or x.dtype != orig_dtype:
            raise ValueError("token_logp_bwd(in_place=True) needs contiguous bf16 / fp16 / fp32 logits")
        grad = x.view(-1, V)
    else:
        grad = torch.empty((n_rows, V), dtype=x.dtype, device=device)
    if n_rows and V:
        stream = N.current_stream(device)
        off = 0
        with N.on_device(device):
            for x2 in _row_blocks(x, V):  # sliced logits are read in place, block by block
                rows = x2.shape[0]
                rc = N.F.unirl_token_logp_bwd(
                    N.ptr(x2), N.dtype_code(x2.dtype), rows, V, x2.stride(0) if rows > 1 else V,
                    N.ptr(idc[off : off + rows]), float(temperature), N.ptr(lsec[off : off + rows]),
                    N.ptr(gc[off : off + rows]), N.ptr(grad[off : off + rows]), V, stream,
                )
                N.check(rc, "unirl_token_logp_bwd")
                off += rows
    grad = grad.reshape(logits.shape)
    return grad if grad.dtype == orig_dtype else grad.to(orig_dtype)


def _ratio_params(
    kind: int,
    agg_mode: str,
    clip_low: float,
    clip_high: float,
    drpo_epsilon: float,
    mu_weighted: bool,
    horizon: float,
    adv_per_token: bool,
) -> N.RatioLossParams:
    if agg_mode not in N.AGG_MODES:
        raise ValueError(f"loss_agg_mode must be one of {sorted(N.AGG_MODES)}; got {agg_mode!r}")
    return N.RatioLossParams(
        kind=kind,
        agg_mode=N.AGG_MODES[agg_mode],
        clip_low=float(clip_low),
        clip_high=float(clip_high),
        drpo_epsilon=float(drpo_epsilon),
        mu_weighted=int(bool(mu_weighted)),
        horizon=float(horizon),
        adv_per_token=int(bool(adv_per_token)),
    )


class RatioLossPlan:
    """Validated, device-ready arguments of one ratio-loss call (forward and backward share them)."""

    def __init__(
        self,
        new_logp: torch.Tensor,
        old_logp: torch.Tensor,
        advantages: torch.Tensor,
        *,
        kind: int,
        lengths: Optional[torch.Tensor] = None,
        cu_seqlens: Optional[torch.Tensor] = None,
        loss_mask: Optional[torch.Tensor] = None,
        agg_mode: str = "token-mean",
        clip_low: float = 0.2,
        clip_high: Optional[float] = None,
        drpo_epsilon: float = 12.5,
        mu_weighted: bool = True,
        horizon: float = 8192,
        adv_per_token: Optional[bool] = None,
    ) -> None:
        N.require_device(new_logp, "new_logp")
        if new_logp.shape != old_logp.shape:
            raise ValueError(f"new_logp {tuple(new_logp.shape)} != old_logp {tuple(old_logp.shape)}")
        device = new_logp.device
        self.device = device
        self.shape = tuple(new_logp.shape)
        self.nw = N.as_operand(new_logp, torch.float32, device)
        self.od = N.as_operand(old_logp, torch.float32, device)
        self.n_tok = self.nw.numel()
        adv = N.as_operand(advantages, torch.float32, device)
        self.seq = None
        self.n_seq = 0
        self.seq_stride = 0
        self.n_valid_host = -1  # padded layout: valid-token count when known without a device sync
        if lengths is not None and cu_seqlens is not None:
            raise ValueError("pass lengths (padded layout) or cu_seqlens (packed layout), not both")
        if lengths is not None:
            if new_logp.dim() != 2:
                raise ValueError("the padded layout needs [n_seq, max_len] log-probs")
            self.n_seq, self.seq_stride = self.shape
            if lengths.device.type == "cpu":  # the token count is free on the host
                self.n_valid_host = int(lengths.detach().reshape(-1).clamp(0, self.seq_stride).sum())
            self.seq = N.as_operand(lengths, torch.int64, device)  # read flat by the kernel
            if self.seq.numel() != self.n_seq:
                raise ValueError(f"lengths has {self.seq.numel()} entries for {self.n_seq} sequences")
        elif cu_seqlens is not None:
            self.seq = N.as_operand(cu_seqlens, torch.int64, device)
            self.n_seq = self.seq.numel() - 1
            if self.n_seq < 0:
                raise ValueError("cu_seqlens needs n_seq + 1 entries")
        # One advantage per sequence, as the reference's algorithms pass them, or one per token.
        # A packed batch with as many tokens as sequences fits both readings: per sequence wins
        # unless `adv_per_token` says otherwise.
        fits_seq = self.seq is not None and adv.numel() == self.n_seq
        fits_tok = adv.shape == self.nw.shape or (adv.numel() == self.n_tok and self.seq is None)
        if adv_per_token is None:
            adv_per_token = fits_tok and not fits_seq
        if not (fits_tok if adv_per_token else fits_seq):
            raise ValueError(
                f"advantages {tuple(advantages.shape)} match neither the tokens {self.shape} "
                f"nor the {self.n_seq} sequences"
            )
        self.adv = adv
        self.mask = None
        if loss_mask is not None:
            if loss_mask.numel() != self.n_tok:
                raise ValueError(f"loss_mask {tuple(loss_mask.shape)} does not match tokens {self.shape}")
            self.mask = N.as_operand(loss_mask, torch.float32, device)
        self.params = _ratio_params(
            kind, agg_mode, clip_low, clip_low if clip_high is None else clip_high, drpo_epsilon, mu_weighted,
            horizon, adv_per_token,
        )

    def forward(self, want_elem: bool) -> Tuple[Optional[torch.Tensor], torch.Tensor]:
        """Launch the forward kernel: ``(loss_per_elem or None, metrics [16] f32)``."""
        device = self.device
        metrics = torch.empty(N.M_COUNT, dtype=torch.float32, device=device)
        elem = torch.empty(self.shape, dtype=torch.float32, device=device) if want_elem else None
        if self.n_tok == 0:
            metrics.fill_(float("nan"))
            metrics[N.M_NUM_TOKENS] = 0.0
            return elem, metrics
        stream = N.current_stream(device)
        ws, ws_bytes = N.workspace(device, stream)
        with N.on_device(device):
            rc = N.F.unirl_ratio_loss_fwd(
                N.ptr(self.nw), N.ptr(self.od), N.ptr(self.adv), N.ptr(self.seq), N.ptr(self.mask), self.n_seq,
                self.seq_stride, self.n_tok, ctypes.byref(self.params), N.ptr(elem), N.ptr(metrics), N.ptr(ws),
                ws_bytes, stream,
            )
        N.check(rc, "unirl_ratio_loss_fwd")
        return elem, metrics

    def forward_backward(self, loss_scale: float) -> Tuple[torch.Tensor, torch.Tensor]:
        """One pass for a whole training micro-step: ``(grad_new f32, metrics [16] f32)`` with
        ``grad_new`` = what ``(loss * loss_scale).backward()`` leaves in ``new_logp.grad``."""
        device = self.device
        metrics = torch.empty(N.M_COUNT, dtype=torch.float32, device=device)
        grad = torch.empty(self.shape, dtype=torch.float32, device=device)
        if self.n_tok == 0:
            metrics.fill_(float("nan"))
            metrics[N.M_NUM_TOKENS] = 0.0
            return grad, metrics
        stream = N.current_stream(device)
        ws, ws_bytes = N.workspace(device, stream)
        with N.on_device(device):
            rc = N.F.unirl_ratio_loss_fwd_bwd(
                N.ptr(self.nw), N.ptr(self.od), N.ptr(self.adv), N.ptr(self.seq), N.ptr(self.mask), self.n_seq,
                self.seq_stride, self.n_tok, ctypes.byref(self.params), float(loss_scale), int(self.n_valid_host),
                N.ptr(grad), N.ptr(metrics), N.ptr(ws), ws_bytes, stream,
            )
        N.check(rc, "unirl_ratio_loss_fwd_bwd")
        return grad, metrics

    def backward(
        self,
        *,
        g_scale: Optional[torch.Tensor],
        g_elem: Optional[torch.Tensor],
        aggregate: bool,
        n_valid: Optional[torch.Tensor],
    ) -> torch.Tensor:
        """Launch the backward kernel: gradient w.r.t. ``new_logp`` (f32, same shape)."""
        device = self.device
        grad = torch.empty(self.shape, dtype=torch.float32, device=device)
        if self.n_tok == 0:
            return grad
        gs = None if g_scale is None else g_scale.detach().to(device=device, dtype=torch.float32).reshape(-1)[:1].contiguous()
        ge = None if g_elem is None else g_elem.detach().to(device=device, dtype=torch.float32).contiguous()
        nv = None if n_valid is None else n_valid.detach().reshape(-1)[:1].contiguous()
        with N.on_device(device):
            rc = N.F.unirl_ratio_loss_bwd(
                N.ptr(self.nw), N.ptr(self.od), N.ptr(self.adv), N.ptr(self.seq), N.ptr(self.mask), self.n_seq,
                self.seq_stride, self.n_tok, ctypes.byref(self.params), N.ptr(gs), N.ptr(ge),
                int(bool(aggregate)), N.ptr(nv), N.ptr(grad), N.current_stream(device),
            )
        N.check(rc, "unirl_ratio_loss_bwd")
        return grad


def group_advantages(
    rewards: torch.Tensor,
    n_groups: int,
    *,
    normalize: bool = True,
    eps: float = 1e-8,
    scope: str = "group",
    use_global_std: bool = False,
) -> torch.Tensor:
    """Advantages of ``n_groups`` contiguous equal-size groups of ``rewards [n]`` (f32 ``[n]``)."""
    N.require_device(rewards, "rewards")
    if scope not in ("group", "global"):
        raise ValueError(f"scope must be 'group' or 'global'; got {scope!r}")
    r = rewards.detach().to(torch.float32).reshape(-1).contiguous()
    n = r.numel()
    out = torch.empty(n, dtype=torch.float32, device=r.device)
    if n == 0:
        return out
    if n_groups <= 0 or n % n_groups != 0:
        raise ValueError(f"non-uniform group sizes (n={n}, n_groups={n_groups})")
    with N.on_device(r.device):
        rc = N.F.unirl_group_advantages(
            N.ptr(r), n_groups, n // n_groups, int(bool(normalize)), float(eps), int(scope == "global"),
            int(bool(use_global_std)), N.ptr(out), N.current_stream(r.device),
        )
    N.check(rc, "unirl_group_advantages")
    return out


def normalize_grouped(
    rewards: torch.Tensor,
    group_indices: Sequence[Sequence[int]],
    *,
    eps: float = 1e-8,
    clip_max: Optional[float] = None,
    trim_outliers_ratio: float = 0.0,
    use_global_std: bool = False,
) -> torch.Tensor:
    """Grouped normalisation of ``rewards [n]`` over arbitrary index lists (f32 ``[n]``)."""
    N.require_device(rewards, "rewards")
    device = rewards.device
    r = rewards.detach().to(torch.float32).reshape(-1).contiguous()
    n = r.numel()
    out = torch.zeros(n, dtype=torch.float32, device=device)
    members: List[int] = []
    offsets: List[int] = [0]
    for g in group_indices:
        for i in g:
            i = int(i)
            if i < -n or i >= n:
                raise IndexError(f"index {i} is out of bounds for dimension 0 with size {n}")
            members.append(i % n)
        offsets.append(len(members))
    n_groups = len(offsets) - 1
    if n == 0 or n_groups == 0 or not members:
        return out
    mem_t = torch.tensor(members, dtype=torch.int64, device=device)
    off_t = torch.tensor(offsets, dtype=torch.int64, device=device)
    with N.on_device(device):
        rc = N.F.unirl_normalize_grouped(
            N.ptr(r), n, N.ptr(mem_t), N.ptr(off_t), n_groups, float(eps), float(trim_outliers_ratio),
            int(bool(use_global_std)), int(clip_max is not None), float(clip_max or 0.0), N.ptr(out),
            N.current_stream(device),
        )
    N.check(rc, "unirl_normalize_grouped")
    return out


def gather_steps(tensor: torch.Tensor, positions: Sequence[int]) -> torch.Tensor:
    """``tensor[:, positions]`` for a ``[B, S, ...]`` tensor, as one gather kernel."""
    N.require_device(tensor, "tensor")
    if tensor.dim() < 2:
        raise ValueError(f"need a [B, S, ...] tensor; got {tuple(tensor.shape)}")
    t = tensor if tensor.is_contiguous() else tensor.contiguous()
    B, S = t.shape[0], t.shape[1]
    pos = [int(p) for p in positions]
    for p in pos:
        if p < -S or p >= S:
            raise IndexError(f"index {p} is out of bounds for dimension 1 with size {S}")
    pos = [p % S for p in pos] if S else pos
    out = torch.empty((B, len(pos)) + tuple(t.shape[2:]), dtype=t.dtype, device=t.device)
    inner_bytes = (t.numel() // (B * S)) * t.element_size() if B * S else 0
    if out.numel() == 0:
        return out
    pos_t = torch.tensor(pos, dtype=torch.int64, device=t.device)
    with N.on_device(t.device):
        rc = N.F.unirl_gather_steps(
            N.ptr(t), B, S, inner_bytes, N.ptr(pos_t), len(pos), N.ptr(out), N.current_stream(t.device)
        )
    N.check(rc, "unirl_gather_steps")
    return out


def expand_groups(unique: torch.Tensor, group_of: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """``out[b] = unique[group_of[b]].to(dtype)`` for fp32 ``unique [U, ...]`` and int64 ``group_of [B]``
    (values in ``[0, U)``, checked by the caller), as one kernel."""
    N.require_device(unique, "unique")
    if unique.dtype != torch.float32:
        raise TypeError(f"unique must be float32; got {unique.dtype}")
    src = unique if unique.is_contiguous() else unique.contiguous()
    idx = group_of.detach().to(device=src.device, dtype=torch.int64).reshape(-1).contiguous()
    U, B = src.shape[0], idx.numel()
    D = src.numel() // U if U else 0
    out = torch.empty((B,) + tuple(src.shape[1:]), dtype=dtype, device=src.device)
    if B == 0 or D == 0:
        return out
    if U == 0:
        raise ValueError("no noise groups to expand")
    with N.on_device(src.device):
        rc = N.F.unirl_expand_groups(
            N.ptr(src), U, D, N.ptr(idx), B, N.ptr(out), N.dtype_code(dtype), N.current_stream(src.device)
        )
    N.check(rc, "unirl_expand_groups")
    return out


METRIC_SLOTS: Dict[str, int] = {
    "loss": N.M_LOSS,
    "ratio_mean": N.M_RATIO_MEAN,
    "ratio_std": N.M_RATIO_STD,
    "ratio_min": N.M_RATIO_MIN,
    "ratio_max": N.M_RATIO_MAX,
    "clip_fraction": N.M_CLIP_FRACTION,
    "clipfrac_hi": N.M_CLIPFRAC_HI,
    "clipfrac_lo": N.M_CLIPFRAC_LO,
    "approx_kl": N.M_APPROX_KL,
    "penalty_mean": N.M_PENALTY_MEAN,
    "absdiff_mean": N.M_ABSDIFF_MEAN,
    "absdiff_max": N.M_ABSDIFF_MAX,
    "num_tokens": N.M_NUM_TOKENS,
}
