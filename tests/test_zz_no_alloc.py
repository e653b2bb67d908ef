"""The allocation-free row-KL entry point against the workspace one, through the C ABI.

`unirl_gaussian_kl_mask_static` keeps its per-workgroup partials in a static device array of the
library instead of a caller-owned workspace.  It runs the same kernels with the same launch
shape, so its outputs must equal `unirl_gaussian_kl_mask`'s bit for bit -- on a first call, and
on a second, smaller one that finds the first call's partials still in the array.
"""

import pytest
import torch

from unirl_amd import _native as N

pytestmark = pytest.mark.gpu


def _inputs(R, D, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    base = torch.randn(R, D, generator=g)
    p = (base + 0.05 * torch.randn(R, D, generator=g)).to(dtype).cuda()
    q = (base + 0.05 * torch.randn(R, D, generator=g)).to(dtype).cuda()
    sigma = (0.2 + torch.rand(R, generator=g)).cuda()
    return p, q, sigma


def _run_both(p, q, sigma, threshold):
    R, D = p.shape
    dev = p.device
    stream = N.current_stream(dev)
    ws, ws_bytes = N.workspace(dev, stream)
    out = {}
    for name in ("workspace", "static"):
        kl = torch.full((R,), float("nan"), dtype=torch.float32, device=dev)
        mask = torch.full((R,), 7, dtype=torch.uint8, device=dev)
        common = (N.ptr(p), N.ptr(q), N.dtype_code(p.dtype), N.ptr(sigma), sigma.numel(), R, D, float(threshold),
                  N.ptr(kl), N.ptr(mask))
        if name == "workspace":
            rc = N.lib().unirl_gaussian_kl_mask(*common, N.ptr(ws), ws_bytes, stream)
        else:
            rc = N.lib().unirl_gaussian_kl_mask_static(*common, stream)
        assert rc == 0, (name, rc)
        torch.cuda.synchronize()
        out[name] = (kl.cpu(), mask.cpu())
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_static_scratch_matches_workspace_entry_on_two_calls(dtype):
    # first call: many workgroups per row (partials are used); second call: fewer, shorter rows
    for R, D, seed in ((6, 262144, 11), (3, 40960, 12)):
        p, q, sigma = _inputs(R, D, dtype, seed)
        # threshold at the median KL so that both mask values occur
        kl_probe = _run_both(p, q, sigma, 0.0)["workspace"][0]
        thr = float(kl_probe.median())
        got = _run_both(p, q, sigma, thr)
        kl_w, mask_w = got["workspace"]
        kl_s, mask_s = got["static"]
        assert torch.isfinite(kl_w).all() and 0 < int(mask_w.sum()) < R
        assert torch.equal(kl_s, kl_w), (R, D, dtype)
        assert torch.equal(mask_s, mask_w), (R, D, dtype)
        # and both agree with a float64 evaluation of the formula (torch's promotion: 16-bit
        # subtract and square, f32 divide)
        d = (p - q)
        sq = (d * d).float().double().cpu()
        ref = (sq / (2.0 * (sigma.double().cpu() ** 2))[:, None]).mean(dim=1)
        assert torch.allclose(kl_s.double(), ref, rtol=1e-5, atol=0.0)


def test_static_scratch_single_workgroup_rows_and_unaligned():
    # rows short enough for one workgroup each (no partials at all), odd D (scalar path)
    p, q, sigma = _inputs(700, 1001, torch.float32, 13)
    got = _run_both(p, q, sigma, 0.01)
    assert torch.equal(got["static"][0], got["workspace"][0])
    assert torch.equal(got["static"][1], got["workspace"][1])


def test_static_scratch_rejects_rows_beyond_its_limit():
    p, q, sigma = _inputs(4, 64, torch.float32, 14)
    kl = torch.empty(4, dtype=torch.float32, device="cuda")
    too_many = 32768 + 1
    rc = N.lib().unirl_gaussian_kl_mask_static(N.ptr(p), N.ptr(q), N.F32, N.ptr(sigma), 1, too_many, 64, 0.01,
                                               N.ptr(kl), None, N.current_stream(p.device))
    assert rc == -6  # UNIRL_E_LIMIT
    assert b"limit" in N.lib().unirl_status_string(rc)
    torch.cuda.synchronize()
