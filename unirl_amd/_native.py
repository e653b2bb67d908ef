"""ctypes binding of libunirl_hip.so (the C ABI declared in include/unirl_hip.h).

There is no CPU implementation behind this module: if the shared library has
not been built, or a tensor does not live on a HIP device, the call raises.
"""

from __future__ import annotations

import ctypes
import threading
from ctypes import POINTER, Structure, c_char_p, c_double, c_float, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path
from typing import Dict, Optional, Tuple

import torch

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libunirl_hip.so"

# enum unirl_dtype
F32, BF16, F16 = 0, 1, 2
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}

# enum unirl_sde_kind
SDE_FLOW, SDE_DANCE, SDE_CPS = 0, 1, 2

# enum unirl_loss_kind / unirl_agg_mode
LOSS_GRPO, LOSS_DRPO = 0, 1
AGG_TOKEN_MEAN, AGG_SEQ_MEAN_TOKEN_SUM, AGG_SEQ_MEAN_TOKEN_MEAN = 0, 1, 2
AGG_MODES = {
    "token-mean": AGG_TOKEN_MEAN,
    "seq-mean-token-sum-norm": AGG_SEQ_MEAN_TOKEN_SUM,
    "seq-mean-token-mean": AGG_SEQ_MEAN_TOKEN_MEAN,
}

# enum unirl_metric_slot
M_LOSS, M_RATIO_MEAN, M_RATIO_STD, M_RATIO_MIN, M_RATIO_MAX = 0, 1, 2, 3, 4
M_CLIP_FRACTION, M_CLIPFRAC_HI, M_CLIPFRAC_LO, M_APPROX_KL, M_PENALTY_MEAN = 5, 6, 7, 8, 9
M_ABSDIFF_MEAN, M_ABSDIFF_MAX, M_NUM_TOKENS, M_COUNT = 10, 11, 12, 16

MAX_ROLLOUT_STEPS = 64


class RatioLossParams(Structure):
    """struct unirl_ratio_loss_params."""

    _fields_ = [
        ("kind", c_int),
        ("agg_mode", c_int),
        ("clip_low", c_float),
        ("clip_high", c_float),
        ("drpo_epsilon", c_float),
        ("mu_weighted", c_int),
        ("horizon", c_float),
        ("adv_per_token", c_int),
    ]


class SdeTensor(Structure):
    """struct unirl_sde_tensor."""

    _fields_ = [("ptr", c_void_p), ("dtype", c_int), ("sample_stride", c_int64)]


class Rng(Structure):
    """struct unirl_rng."""

    _fields_ = [("enabled", c_int), ("seed", ctypes.c_uint64), ("offset", ctypes.c_uint64)]


class SdeStepDesc(Structure):
    """struct unirl_sde_step_desc."""

    _fields_ = [
        ("noise_pred", SdeTensor),
        ("sample", SdeTensor),
        ("prev_sample", SdeTensor),
        ("noise", c_void_p),
        ("noise_stride", c_int64),
        ("sigma", c_void_p),
        ("sigma_next", c_void_p),
        ("sigma_stride", c_int),
        ("sigma_max_ptr", c_void_p),
        ("sigma_max_val", c_float),
        ("eta", c_double),
        ("kind", c_int),
        ("B", c_int64),
        ("D", c_int64),
        ("prev_out", c_void_p),
        ("prev_dtype", c_int),
        ("prev_stride", c_int64),
        ("mean_out", c_void_p),
        ("mean_dtype", c_int),
        ("mean_stride", c_int64),
        ("logp_out", c_void_p),
        ("logp_stride", c_int64),
        ("logp_sum", c_int),
        ("rng", Rng),
        ("noise_out", c_void_p),
        ("noise_out_stride", c_int64),
    ]


class SdeReplayDesc(Structure):
    """struct unirl_sde_replay_desc."""

    _fields_ = [
        ("noise_pred", SdeTensor),
        ("noise_pred_step_stride", c_int64),
        ("latents", SdeTensor),
        ("latents_slot_stride", c_int64),
        ("K", c_int64),
        ("slot_sample", POINTER(c_int64)),
        ("slot_prev", POINTER(c_int64)),
        ("sigma", c_void_p),
        ("sigma_next", c_void_p),
        ("sigma_max_ptr", c_void_p),
        ("sigma_max_val", c_float),
        ("eta", c_double),
        ("kind", c_int),
        ("B", c_int64),
        ("S", c_int64),
        ("D", c_int64),
        ("mean_out", c_void_p),
        ("mean_dtype", c_int),
        ("logp_out", c_void_p),
        ("logp_sum", c_int),
    ]


# enum unirl_dpm2_branch
DPM2_DDIM, DPM2_FIRST, DPM2_SECOND = 0, 1, 2


class Dpm2Coeffs(Structure):
    """struct unirl_dpm2_coeffs."""

    _fields_ = [(name, c_float) for name in
                ("sigma", "one_minus_s", "s", "one_minus_t", "sqrt_t2", "c1", "c2", "half_c2", "inv_r0")]


# UNIRL_ABI_VERSION of include/unirl_hip.h that the signatures below describe
ABI_VERSION = 6

_SIGNATURES = {
    "unirl_abi_version": (c_int, []),
    "unirl_status_string": (c_char_p, [c_int]),
    "unirl_workspace_bytes": (c_size_t, []),
    "unirl_workspace_init": (c_int, [c_void_p, c_size_t, c_void_p]),
    "unirl_sde_step_logp": (
        c_int,
        [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_float,
         c_double, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_size_t, c_void_p],
    ),
    "unirl_sde_step_logp_ex": (c_int, [POINTER(SdeStepDesc), c_void_p, c_size_t, c_void_p]),
    "unirl_sde_replay_logp": (c_int, [POINTER(SdeReplayDesc), c_void_p, c_size_t, c_void_p]),
    "unirl_sde_replay_logp_bwd": (c_int, [POINTER(SdeReplayDesc), c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "unirl_sde_step_logp_bwd": (
        c_int,
        [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_float,
         c_double, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
         c_void_p],
    ),
    "unirl_sde_rollout_logp": (
        c_int,
        [c_void_p, c_int, POINTER(c_void_p), c_int, POINTER(c_void_p), POINTER(Rng), POINTER(c_void_p), c_void_p,
         POINTER(c_double), c_int, c_void_p, c_float, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int,
         c_void_p, c_size_t, c_void_p],
    ),
    "unirl_dpm2_step": (
        c_int,
        [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, POINTER(Dpm2Coeffs), c_int64, c_void_p, c_void_p, c_void_p],
    ),
    "unirl_gaussian_kl_mask": (
        c_int,
        [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64, c_float, c_void_p, c_void_p, c_void_p,
         c_size_t, c_void_p],
    ),
    "unirl_gaussian_kl_mask_static": (
        c_int,
        [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64, c_float, c_void_p, c_void_p, c_void_p],
    ),
    "unirl_flowdppo_loss": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_float, c_void_p, c_void_p, c_void_p],
    ),
    "unirl_flowdppo_step": (
        c_int,
        [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_float,
         c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    ),
    "unirl_flowdppo_replay_step": (
        c_int,
        [POINTER(SdeReplayDesc), c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p,
         c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    ),
    "unirl_expand_per_seq": (
        c_int,
        [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p],
    ),
    "unirl_gaussian_kl_elem": (
        c_int,
        [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p],
    ),
    "unirl_gaussian_kl_elem_bwd": (
        c_int,
        [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "unirl_token_logp_entropy": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "unirl_lmhead_logp_scratch_bytes": (c_size_t, [c_int64, c_int64]),
    "unirl_lmhead_logp": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_float, c_void_p,
         c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_size_t, c_void_p],
    ),
    "unirl_transpose_2d": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p]),
    "unirl_token_logp_bwd": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_int64,
         c_void_p],
    ),
    "unirl_ratio_loss_fwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, POINTER(RatioLossParams),
         c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    ),
    "unirl_ratio_loss_bwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, POINTER(RatioLossParams),
         c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p],
    ),
    "unirl_ratio_loss_fwd_bwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, POINTER(RatioLossParams),
         c_float, c_int64, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    ),
    "unirl_group_advantages": (
        c_int,
        [c_void_p, c_int64, c_int64, c_int, c_float, c_int, c_int, c_void_p, c_void_p],
    ),
    "unirl_normalize_grouped": (
        c_int,
        [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_float, c_float, c_int, c_int, c_float, c_void_p,
         c_void_p],
    ),
    "unirl_expand_groups": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int, c_void_p]),
    "unirl_gather_steps": (
        c_int,
        [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_void_p],
    ),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib: Optional[ctypes.CDLL] = None
_lib_lock = threading.Lock()


class UnirlHipError(RuntimeError):
    """A C-ABI call returned a non-zero status."""


def lib() -> ctypes.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lib_lock:
        if _lib is None:
            if not LIB_PATH.exists():
                raise RuntimeError(
                    f"{LIB_PATH} is missing: build it with `python -m unirl_amd.build` "
                    "(hipcc, gfx950). unirl_amd has no CPU or eager-torch path behind its kernels."
                )
            handle = ctypes.CDLL(str(LIB_PATH))
            handle.unirl_abi_version.restype = c_int
            built = handle.unirl_abi_version()
            if built != ABI_VERSION:
                raise RuntimeError(
                    f"{LIB_PATH} was built for ABI version {built}, this package binds version {ABI_VERSION}: "
                    "rebuild it with `python -m unirl_amd.build`"
                )
            for name, (restype, argtypes) in _SIGNATURES.items():
                fn = getattr(handle, name)
                fn.restype = restype
                fn.argtypes = argtypes
            _lib = handle
    return _lib


class _Functions:
    """The library's entry points as plain attributes: the first use of a name loads the library
    and binds the function; later uses are one attribute read (``lib().name`` costs a call and a
    ctypes lookup every time, which shows on a path whose kernels run for ten microseconds)."""

    def __getattr__(self, name: str):
        fn = getattr(lib(), name)
        setattr(self, name, fn)
        return fn


F = _Functions()


def check(status: int, what: str) -> None:
    """Turn a C-ABI status into an exception: ValueError for argument errors,
    UnirlHipError for a failed launch."""
    if status == 0:
        return
    msg = lib().unirl_status_string(int(status)).decode()
    if status < 0:
        raise ValueError(f"{what}: {msg} (status {status})")
    raise UnirlHipError(f"{what}: HIP error {status}: {msg}")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype}; expected float32, bfloat16 or float16") from None


def require_device(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} lives on {t.device}: unirl_amd kernels run on a HIP device only "
            "(there is no CPU fallback; use the torch reference for CPU tensors)"
        )


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


# torch's raw accessors (no Stream / device objects built per call); the public API as a fallback
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def current_device_index() -> int:
    return _raw_device() if _raw_device is not None else torch.cuda.current_device()


def current_stream(device: torch.device) -> int:
    """Raw handle of torch's current stream on ``device``."""
    if _raw_stream is None:
        return torch.cuda.current_stream(device).cuda_stream
    index = device.index
    return _raw_stream(current_device_index() if index is None else index)


def as_operand(t: torch.Tensor, dtype: torch.dtype, device: torch.device) -> torch.Tensor:
    """``t`` as a contiguous ``dtype`` tensor on ``device`` -- ``t`` itself (no detach, cast or copy:
    only its address is taken) when it already is one."""
    if t.dtype is dtype and t.device == device and t.is_contiguous():
        return t
    return t.detach().to(device=device, dtype=dtype).contiguous()


class on_device:
    """``with on_device(dev):`` makes ``dev`` the current HIP device for a launch.  When it already
    is (the usual case) nothing is switched, which saves the several microseconds a
    ``torch.cuda.device`` context costs on a path whose kernels run for about ten."""

    __slots__ = ("_ctx",)

    def __init__(self, device: torch.device) -> None:
        index = device.index
        self._ctx = None if (index is None or index == current_device_index()) else torch.cuda.device(index)

    def __enter__(self):
        if self._ctx is not None:
            self._ctx.__enter__()
        return self

    def __exit__(self, *exc):
        if self._ctx is not None:
            return self._ctx.__exit__(*exc)
        return False


_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}


def workspace(device: torch.device, stream: Optional[int] = None) -> Tuple[torch.Tensor, int]:
    """Scratch for the reducing kernels (per-workgroup partial sums), one per (device, stream):
    calls on different streams may overlap and must not share it.  ``stream`` is the raw handle
    when the caller has already looked it up."""
    index = device.index if device.index is not None else current_device_index()
    key = (index, current_stream(device) if stream is None else stream)
    ws = _workspaces.get(key)
    if ws is None:
        nbytes = int(lib().unirl_workspace_bytes())
        if torch.cuda.is_current_stream_capturing():
            # First use of this stream happens inside a graph capture: the allocation belongs to
            # the graph's private pool and dies with the graph, so it must not be cached.  (The
            # workspace needs no initialisation, and the pool keeps it valid for every replay.)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=torch.device("cuda", index))
            return ws, nbytes
        ws = torch.zeros(nbytes, dtype=torch.uint8, device=torch.device("cuda", index))
        _workspaces[key] = ws
    return ws, ws.numel()
