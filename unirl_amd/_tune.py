"""ctypes binding of the MEASUREMENT build, libunirl_hip_tune.so (``python -m unirl_amd.build --tune``).

The benchmark's yardsticks live here, not in the product: a plain copy that calibrates hardware
byte counters, the launch floor of a streaming shape, a bare grid-wide reduction, and the device
timeline.  The shipped library exports none of them; nothing under ``unirl_amd`` imports this
module, and it raises when the measurement build is absent.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_double, c_int, c_size_t, c_uint, c_void_p
from typing import Optional

import torch

from . import _native as N
from .build import TUNE_LIB_PATH

_SIGNATURES = {
    "unirl_calib_copy": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "unirl_calib_stream": (c_int, [c_void_p, c_size_t, c_void_p, c_size_t, c_int, c_void_p, c_void_p]),
    "unirl_calib_reduce": (c_int, [c_void_p, c_size_t, c_int, c_uint, c_void_p, c_size_t, c_void_p, c_void_p]),
    "unirl_trace_begin": (c_int, [c_void_p, c_size_t]),
    "unirl_trace_count": (c_int, []),
    "unirl_trace_entry": (c_char_p, [c_int, ctypes.POINTER(c_uint), ctypes.POINTER(c_size_t)]),
}

_lib: Optional[ctypes.CDLL] = None


def available() -> bool:
    return TUNE_LIB_PATH.exists()


def lib() -> ctypes.CDLL:
    """The measurement build, loaded once (beside the product library, never instead of it --
    unless the caller pointed ``_native.LIB_PATH`` at it before the first product call, as the
    timeline probe does: then both names resolve to the same handle)."""
    global _lib
    if _lib is None:
        if not available():
            raise RuntimeError(f"{TUNE_LIB_PATH} is missing: build it with `python -m unirl_amd.build --tune`")
        handle = N.lib() if N.LIB_PATH == TUNE_LIB_PATH else ctypes.CDLL(str(TUNE_LIB_PATH))
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def calib_copy(src: torch.Tensor, dst: torch.Tensor) -> None:
    """Plain streaming copy of ``src`` into ``dst`` (same byte size, a multiple of 16): the
    reference kernel for calibrating hardware byte counters."""
    N.require_device(src, "src")
    N.require_device(dst, "dst")
    nbytes = src.numel() * src.element_size()
    if nbytes != dst.numel() * dst.element_size() or not (src.is_contiguous() and dst.is_contiguous()):
        raise ValueError("calib_copy needs two contiguous tensors of the same byte size")
    with N.on_device(src.device):
        rc = lib().unirl_calib_copy(N.ptr(src), N.ptr(dst), nbytes, N.current_stream(src.device))
    N.check(rc, "unirl_calib_copy")


def calib_stream(src: Optional[torch.Tensor], read_bytes: int, dst: Optional[torch.Tensor], write_bytes: int,
                 sink: torch.Tensor, *, tail_launch: bool = False) -> None:
    """Launch-floor yardstick: one kernel that reads ``read_bytes`` of ``src`` and writes
    ``write_bytes`` of ``dst`` with no arithmetic, then (``tail_launch``) a one-wavefront kernel."""
    N.require_device(sink, "sink")
    for t, nbytes, name in ((src, read_bytes, "src"), (dst, write_bytes, "dst")):
        if nbytes:
            N.require_device(t, name)
            if not t.is_contiguous() or t.numel() * t.element_size() < nbytes:
                raise ValueError(f"{name} must be contiguous and hold at least {nbytes} bytes")
    with N.on_device(sink.device):
        rc = lib().unirl_calib_stream(
            N.ptr(src) if read_bytes else None, int(read_bytes), N.ptr(dst) if write_bytes else None,
            int(write_bytes), int(bool(tail_launch)), N.ptr(sink), N.current_stream(sink.device),
        )
    N.check(rc, "unirl_calib_stream")


def calib_reduce(src: torch.Tensor, read_bytes: int, mode: int, n_workgroups: int, scratch: torch.Tensor,
                 out: torch.Tensor) -> None:
    """Measurement aid: the sum of ``read_bytes // 4`` floats of ``src``, finished by nothing (mode 0),
    a second launch (mode 1) or inside the one kernel by polling tagged partials (mode 2).
    ``scratch``: zero-filled once, at least ``16 + 16 * n_workgroups`` bytes; ``out``: float64 [1]."""
    for t, name in ((src, "src"), (scratch, "scratch"), (out, "out")):
        N.require_device(t, name)
    if not src.is_contiguous() or src.numel() * src.element_size() < read_bytes:
        raise ValueError(f"src must be contiguous and hold at least {read_bytes} bytes")
    if out.dtype != torch.float64 or out.numel() < 1:
        raise ValueError("out must be a float64 tensor")
    with N.on_device(src.device):
        rc = lib().unirl_calib_reduce(N.ptr(src), int(read_bytes), int(mode), int(n_workgroups), N.ptr(scratch),
                                        scratch.numel() * scratch.element_size(), N.ptr(out),
                                        N.current_stream(src.device))
    N.check(rc, "unirl_calib_reduce")
