"""The binding stub that the integration notes show to UniRL maintainers is executed as written
(only the library path is filled in) and its three wrappers are held to the oracle."""

import re
from pathlib import Path

import pytest
import torch

from oracle import flowdppo as ofd
from oracle import schedule as osch
from oracle import sde as osde
from oracle import token_logp as otok
from tests._util import BF16_RTOL, FP32_RTOL, assert_close

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parent.parent


def stub_namespace():
    from unirl_amd import _native as N

    text = (ROOT / "INTEGRATION.md").read_text()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    code = [b for b in blocks if "self.strategy." not in b]  # the two loop sketches are not runnable on their own
    assert len(code) == 4, "stub, denoise_hip, logp_chunk_hip, kl_mask_hip"
    source = "\n".join(code).replace('ctypes.CDLL("libunirl_hip.so")', f'ctypes.CDLL("{N.LIB_PATH}")')
    ns = {}
    exec(compile(source, "INTEGRATION.md", "exec"), ns)
    return ns


def test_documented_stub_runs_and_matches_the_oracle(dev):
    ns = stub_namespace()
    sig = osch.sigma_schedule(28, 3.0)
    g = torch.Generator().manual_seed(21)

    x, v, n = (torch.randn(3, 4, 16, 16, generator=g) for _ in range(3))
    ref_prev, ref_lp, ref_mean = osde.sde_denoise("flow", v, x, sig[10], sig[11], eta=0.7, noise=n, sigma_max=float(sig[1]),
                                                  ieee_sqrt=True)
    prev, lp, mean = ns["denoise_hip"](v.to(dev), x.to(dev), float(sig[10]), float(sig[11]), eta=0.7,
                                       sigma_max=float(sig[1]), noise=n.to(dev))
    assert torch.equal(prev.cpu(), ref_prev) and torch.equal(mean.cpu(), ref_mean)
    assert_close(lp, ref_lp, FP32_RTOL, 2e-6, "denoise_hip log-prob")
    _, ref_lp2, _ = osde.sde_denoise("flow", v, x, sig[10], sig[11], eta=0.7, prev_sample=ref_prev,
                                     sigma_max=float(sig[1]), ieee_sqrt=True)
    _, lp2, _ = ns["denoise_hip"](v.to(dev), x.to(dev), float(sig[10]), float(sig[11]), eta=0.7,
                                  sigma_max=float(sig[1]), prev_sample=ref_prev.to(dev))
    assert_close(lp2, ref_lp2, FP32_RTOL, 2e-6, "denoise_hip replay log-prob")
    assert ns["denoise_hip"](v.to(dev), x.to(dev), float(sig[10]), float(sig[11]), eta=0.0, noise=n.to(dev))[1] is None

    logits = (2 * torch.randn(2, 5, 4099, generator=g)).bfloat16()
    ids = torch.randint(0, 4099, (2, 5), generator=g)
    got = ns["logp_chunk_hip"](logits.to(dev), ids.to(dev), 0.7)
    assert got.shape == ids.shape
    assert_close(got, otok.token_logp(logits, ids, 0.7), 2e-5, 2e-6, "logp_chunk_hip")

    base = torch.randn(2, 3, 4, 8, 8, generator=g)
    new_m = (base + 0.02 * torch.randn(base.shape, generator=g)).bfloat16()
    old_m = (base + 0.02 * torch.randn(base.shape, generator=g)).bfloat16()
    sigma_t = torch.tensor([0.3, 0.2, 0.1]).view(1, 3, 1, 1, 1)
    ref = ofd.kl_per_sample(new_m, old_m, sigma_t)
    thr = float(ref.median())
    kl, mask = ns["kl_mask_hip"](new_m.to(dev), old_m.to(dev), sigma_t, thr)
    assert_close(kl, ref, BF16_RTOL, 1e-9, "kl_mask_hip")
    clear = (ref - thr).abs() > 1e-6 * thr
    assert torch.equal(mask.cpu()[clear], (ref < thr)[clear])

    with pytest.raises(ValueError):
        ns["_check"](-2, "x")
