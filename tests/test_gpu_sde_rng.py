"""Sampling noise drawn inside the SDE kernels (Philox-4x32-10 + Box-Muller in registers) instead of a
noise tensor written by `torch.randn` and read back -- the reference draws inside the step as well,
with `randn_tensor(generator=None)` (unirl/sde/kernels.py:230-232), so no bit pattern has to be
matched; what has to hold is that (i) the transition computed from the drawn noise is the oracle's
transition for that noise, bit for bit, (ii) the draws are standard normal and uncorrelated,
(iii) a draw depends on (seed, offset, element) only."""

import math

import numpy as np
import pytest
import torch

from oracle import schedule as osch
from oracle import sde as osde
from tests._util import FP32_RTOL, assert_close

pytestmark = pytest.mark.gpu

SIG = osch.sigma_schedule(28, 3.0)
M32 = 0xFFFFFFFF


def philox4x32_10(counter, key):
    """Reference Philox-4x32-10 on Python integers (Salmon et al. 2011)."""
    c, k = list(counter), list(key)
    for _ in range(10):
        p0, p1 = 0xD2511F53 * c[0], 0xCD9E8D57 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & M32, (p0 >> 32) ^ c[3] ^ k[1], p0 & M32]
        k = [(k[0] + 0x9E3779B9) & M32, (k[1] + 0xBB67AE85) & M32]
    return c


def test_philox_known_answers():
    """The published known-answer vectors of Philox-4x32-10 (Random123's kat_vectors) pin the reference
    implementation this file checks the kernel against."""
    assert philox4x32_10([0, 0, 0, 0], [0, 0]) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert philox4x32_10([M32] * 4, [M32] * 2) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert philox4x32_10([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0]) == \
        [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]


def expected_normals(seed, offset, step, first, count):
    """float64 Box-Muller of the reference Philox stream for elements [first, first + count)."""
    out = np.empty(count, dtype=np.float64)
    key = [seed & M32, (seed >> 32) & M32]
    for e in range(first, first + count):
        block, w = e >> 2, e & 3
        c = philox4x32_10([block & M32, (block >> 32) & M32, ((offset & M32) + step) & M32, (offset >> 32) & M32], key)
        a, b = (c[0], c[1]) if w < 2 else (c[2], c[3])
        u1 = (a + 0.5) / 2.0 ** 32
        r = math.sqrt(-2.0 * math.log(u1))
        th = 2.0 * math.pi * (b / 2.0 ** 32)
        out[e - first] = r * (math.cos(th) if w % 2 == 0 else math.sin(th))
    return out


@pytest.mark.parametrize("kind", ["flow", "dance", "cps"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_step_from_drawn_noise_is_the_oracles_step(dev, kind, dtype):
    from unirl_amd import ops

    g = torch.Generator().manual_seed(5)
    shape = (3, 4, 10, 12)
    x = torch.randn(shape, generator=g).to(dtype)
    v = torch.randn(shape, generator=g).to(dtype)
    noise = torch.full(shape, float("nan"), device=dev)
    prev, mean = torch.empty(shape, device=dev), torch.empty(shape, device=dev)
    lp = torch.empty(3, device=dev)
    ops.sde_step_logp_into(v.to(dev), x.to(dev), SIG[10].to(dev), SIG[11].to(dev), kind=kind, eta=0.7, sigma_max=SIG[1].to(dev),
                           prev_out=prev, mean_out=mean, logp_out=lp, rng=(1234567, 8), noise_out=noise)
    nz = noise.cpu()
    assert bool(torch.isfinite(nz).all())
    ref_prev, ref_lp, ref_mean = osde.sde_denoise(kind, v, x, SIG[10], SIG[11], eta=0.7, noise=nz, sigma_max=SIG[1],
                                                  ieee_sqrt=True)
    assert torch.equal(prev.cpu(), ref_prev) and torch.equal(mean.cpu(), ref_mean), "transition from the drawn noise"
    assert_close(lp, ref_lp, FP32_RTOL, 2e-6, "log-prob from the drawn noise")
    # the stream is the documented one: Philox keyed by the seed, counter (element / 4, offset), Box-Muller
    want = expected_normals(1234567, 8, 0, 0, 64)
    np.testing.assert_allclose(nz.reshape(-1)[:64].double().numpy(), want, rtol=0, atol=4e-6)
    tail = nz.numel() - 32
    np.testing.assert_allclose(nz.reshape(-1)[tail:].double().numpy(), expected_normals(1234567, 8, 0, tail, 32), rtol=0, atol=4e-6)
    # the same call without noise_out gives the same transition, and so does ops.sde_step_logp(rng=...)
    prev2, lp2, mean2 = ops.sde_step_logp(v.to(dev), x.to(dev), SIG[10].to(dev), SIG[11].to(dev), kind=kind, eta=0.7,
                                          sigma_max=SIG[1].to(dev), rng=(1234567, 8))
    assert torch.equal(prev2, prev) and torch.equal(mean2, mean) and torch.equal(lp2, lp)


def test_draws_depend_on_seed_offset_and_element_only(dev):
    """Same (seed, offset): same bits, whatever the vector width, the batch split or the output dtype;
    another seed or offset: other noise."""
    from unirl_amd import ops

    def draw(shape, rng, dtype=torch.float32, odd_base=False):
        x = torch.zeros(shape, device=dev, dtype=dtype)
        if odd_base:  # a sample base that is not 16-byte aligned: the scalar path
            buf = torch.zeros(x.numel() + 1, device=dev, dtype=dtype)
            x = buf[1:].view(shape)
        noise = torch.empty(shape, device=dev)
        ops.sde_step_logp_into(x, x, SIG[10].to(dev), SIG[11].to(dev), kind="flow", eta=0.7, sigma_max=SIG[1].to(dev),
                               prev_out=torch.empty(shape, device=dev), rng=rng, noise_out=noise)
        return noise.reshape(-1)

    a = draw((4, 1024), (99, 16))
    assert torch.equal(a, draw((4, 1024), (99, 16)))                      # repeatable
    assert torch.equal(a, draw((2, 2048), (99, 16)))                      # element index = b * D + i
    assert torch.equal(a, draw((4, 1024), (99, 16), torch.bfloat16))      # eight elements per lane
    assert torch.equal(a, draw((4, 1024), (99, 16), odd_base=True))       # one element per lane
    assert torch.equal(a[: 3 * 1021], draw((3, 1021), (99, 16)))          # D not a multiple of 4
    assert not torch.equal(a, draw((4, 1024), (100, 16)))
    assert not torch.equal(a, draw((4, 1024), (99, 20)))
    # offsets that differ by one are different streams too (the rollout steps use offset + k)
    b = draw((4, 1024), (99, 17))
    assert abs(float((a * b).mean())) < 5.0 / math.sqrt(a.numel())


def test_draws_are_standard_normal_and_uncorrelated(dev):
    """2^24 draws: mean, variance, skewness, excess kurtosis, lag-1 / lag-4 correlation and the
    correlation between the two outputs of a Box-Muller pair, each within five standard errors."""
    from unirl_amd import ops

    n = 1 << 24
    x = torch.zeros((16, n // 16), device=dev)
    noise = torch.empty_like(x)
    ops.sde_step_logp_into(x, x, SIG[10].to(dev), SIG[11].to(dev), kind="flow", eta=0.7, sigma_max=SIG[1].to(dev),
                           prev_out=torch.empty_like(x), rng=(20241125, 0), noise_out=noise)
    z = noise.reshape(-1).double()
    se = 1.0 / math.sqrt(n)
    assert abs(float(z.mean())) < 5 * se
    assert abs(float(z.var()) - 1.0) < 5 * math.sqrt(2.0) * se
    assert abs(float((z ** 3).mean())) < 5 * math.sqrt(15.0) * se          # Var(z^3) = 15
    assert abs(float((z ** 4).mean()) - 3.0) < 5 * math.sqrt(96.0) * se    # Var(z^4) = 96
    for lag in (1, 2, 4, 64):
        assert abs(float((z[:-lag] * z[lag:]).mean())) < 5 * se, f"lag {lag}"
    pair = z.view(-1, 2)
    assert abs(float((pair[:, 0] * pair[:, 1]).mean())) < 5 * math.sqrt(2.0) * se
    assert abs(float((pair[:, 0] ** 2 * pair[:, 1] ** 2).mean()) - 1.0) < 5 * math.sqrt(8.0 * 2.0) * se
    # tails: P(|z| > 3) = 2.6998e-3
    p3 = float((z.abs() > 3).double().mean())
    assert abs(p3 - 2.6998e-3) < 5 * math.sqrt(2.6998e-3 / n)
    assert float(z.abs().max()) < 6.8


def test_rollout_draws_match_single_steps(dev):
    """A rollout with a generator is the chain of single steps called with offset + k: same noise, same
    latents bit for bit; noise tensors that are given still take precedence."""
    from unirl_amd import ops

    g = torch.Generator().manual_seed(6)
    shape, S = (4, 16, 24), 5
    x0 = torch.randn(shape, generator=g).to(dev)
    vs = [torch.randn(shape, generator=g).to(dev) for _ in range(S)]
    sig = SIG.to(dev)
    given = torch.randn(shape, generator=g).to(dev)
    noises = [None, None, given, None, None]
    etas = [0.7, 0.7, 0.7, 0.0, 0.7]
    outs = [torch.full(shape, float("nan"), device=dev) for _ in range(S)]
    x_f, lp, traj = ops.sde_rollout_logp(x0, vs, noises, sig, etas, kind="flow", want_trajectory=True, rng=(77, 40),
                                         noise_out=outs)
    x = x0
    for k in range(S):
        prev = torch.empty(shape, device=dev)
        lpk = torch.empty(4, device=dev)
        no = torch.full(shape, float("nan"), device=dev)
        ops.sde_step_logp_into(vs[k], x, sig[k], sig[k + 1], kind="flow", eta=etas[k], sigma_max=sig[1], noise=noises[k],
                               prev_out=prev, logp_out=lpk, rng=(77, 40 + k), noise_out=no)
        assert torch.equal(traj[k], prev), f"latent after step {k}"
        if etas[k] >= 1e-7:
            assert_close(lp[:, k], lpk, 1e-6, 1e-7, f"log-prob of step {k}")
        else:
            assert bool(torch.isnan(lp[:, k]).all())
        if noises[k] is None and etas[k] >= 1e-7:
            assert torch.equal(outs[k], no), f"noise of step {k}"
        else:
            assert bool(torch.isnan(outs[k]).all()), "no draw where noise was given or the step is deterministic"
        x = prev
    assert torch.equal(x_f, x)
    # noises=None altogether
    x_f2, lp2, _ = ops.sde_rollout_logp(x0, vs, None, sig, 0.7, kind="flow", rng=(77, 40))
    assert bool(torch.isfinite(lp2).all())
    with pytest.raises(ValueError, match="rng"):
        ops.sde_rollout_logp(x0, vs, None, sig, 0.7, kind="flow")


def test_denoise_follows_torch_manual_seed(dev):
    """`denoise` without a noise tensor draws inside the kernel from the device generator's (seed, offset):
    the same seed gives the same samples, consecutive calls differ, and no noise tensor is made."""
    from unirl_amd import sde

    st = sde.FlowSDEStrategy()
    g = torch.Generator().manual_seed(7)
    x = torch.randn(2, 4, 16, 16, generator=g).to(dev)
    v = torch.randn(2, 4, 16, 16, generator=g).to(dev)
    args = (v, x, SIG[10].to(dev), SIG[11].to(dev))
    torch.manual_seed(31)
    a1 = st.denoise(*args, eta=0.7, sigma_max=SIG[1].to(dev))
    a2 = st.denoise(*args, eta=0.7, sigma_max=SIG[1].to(dev))
    torch.manual_seed(31)
    b1 = st.denoise(*args, eta=0.7, sigma_max=SIG[1].to(dev))
    assert torch.equal(a1[0], b1[0]) and torch.equal(a1[1], b1[1])
    assert not torch.equal(a1[0], a2[0])
    assert torch.equal(a1[2], a2[2]), "the mean does not depend on the noise"
    # the implied noise is standard normal: (prev - mean) / std_var
    c = osde.sde_denoise("flow", v.cpu(), x.cpu(), SIG[10], SIG[11], eta=0.7, noise=torch.zeros(x.shape), sigma_max=SIG[1])
    std_var = float(torch.sqrt(SIG[10] / (1 - SIG[10])) * 0.7 * torch.sqrt(SIG[10] - SIG[11]))
    z = ((a1[0] - a1[2]) / std_var).cpu()
    assert abs(float(z.mean())) < 5 / math.sqrt(z.numel()) and abs(float(z.var()) - 1) < 5 * math.sqrt(2 / z.numel())
    assert torch.equal(a1[2].cpu(), c[2])
    # eta = 0: deterministic, nothing drawn, the generator is left alone
    off = torch.cuda.default_generators[0].get_offset()
    p0 = st.denoise(*args, eta=0.0, sigma_max=SIG[1].to(dev))
    assert torch.cuda.default_generators[0].get_offset() == off and p0[1] is None
    assert torch.equal(p0[0], p0[2])
