"""Shared helpers of the parity tests."""

import torch

FP32_RTOL = 1e-5   # fp32 log-probs, losses, advantages (relative)
BF16_RTOL = 2e-3   # paths whose inputs are bf16 / fp16


def assert_close(got, ref, rtol, atol=0.0, what=""):
    g = torch.as_tensor(got).detach().double().cpu()
    r = torch.as_tensor(ref).detach().double().cpu()
    assert g.shape == r.shape, f"{what}: shape {tuple(g.shape)} vs {tuple(r.shape)}"
    both_nan = torch.isnan(g) & torch.isnan(r)
    err = (g - r).abs()
    bound = rtol * r.abs() + atol
    bad = (err > bound) & ~both_nan
    assert not bool(bad.any()), (
        f"{what}: max err {float(err[~both_nan].max()) if (~both_nan).any() else 0:.3e}, "
        f"worst got {g[bad].flatten()[:3].tolist()} ref {r[bad].flatten()[:3].tolist()}"
    )


def ulp_distance_f32(a, b):
    """Distance in fp32 units-in-the-last-place between two fp32 tensors (same sign assumed)."""
    ai = a.detach().cpu().contiguous().view(torch.int32).to(torch.int64)
    bi = b.detach().cpu().contiguous().view(torch.int32).to(torch.int64)
    return (ai - bi).abs()
