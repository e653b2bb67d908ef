"""Pins the CPU oracle of the sigma schedule and the SDE step against what the
mathematics fixes (the reference ships no vectors for them)."""

import math

import numpy as np
import pytest
import scipy.stats
import torch

from oracle import schedule as osch
from oracle import sde as osde


# ---------------------------------------------------------------- schedule
def test_schedule_known_answers():
    s = osch.sigma_schedule(28, 3.0)
    assert s.dtype == torch.float32 and s.shape == (29,)
    # values of shift*t/(1+(shift-1)*t) at t = 1 - i/28, rounded to fp32
    known = {0: 1.0, 1: 0.98780483, 10: 0.84375006, 11: 0.82258058, 27: 0.10000001, 28: 0.0}
    for i, v in known.items():
        assert abs(float(s[i]) - v) <= 1e-7, (i, float(s[i]), v)


def test_schedule_closed_form_and_shape():
    for T, shift in ((28, 3.0), (10, 3.0), (14, 5.0), (12, 1.0)):
        s = osch.sigma_schedule(T, shift)
        ref = osch.sigma_schedule_f64(T, shift)
        assert np.allclose(s.double().numpy(), ref, rtol=0, atol=2e-7)
        assert float(s[0]) == 1.0 and float(s[-1]) == 0.0
        assert bool((s[1:] < s[:-1]).all())
    assert torch.equal(osch.sigma_schedule(12, 1.0), torch.linspace(1.0, 0.0, 13))


# ---------------------------------------------------------------- sde step
def _inputs(shape, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g).to(dtype)
    v = torch.randn(shape, generator=g).to(dtype)
    n = torch.randn(shape, generator=g)
    return x, v, n


SIG = osch.sigma_schedule(28, 3.0)


def test_flow_scalar_known_answers():
    # step 10 of 28, shift 3, eta 0.7: closed forms evaluated in float64
    s, sn, eta = float(SIG[10]), float(SIG[11]), 0.7
    dt = sn - s
    std = math.sqrt(s / (1 - s)) * eta
    assert abs(dt - (-0.02116948)) < 1e-7
    assert abs(std - 1.6266533) < 1e-6
    assert abs(std * math.sqrt(-dt) - 0.23667377) < 1e-6
    assert abs(1 + std**2 / (2 * s) * dt - 0.96680623) < 1e-6
    assert abs(1 + std**2 * (1 - s) / (2 * s) - 1.2450000) < 1e-6
    x, v, n = _inputs((1, 4), 1)
    prev, lp, mean = osde.sde_denoise("flow", v, x, SIG[10], SIG[11], eta=eta, noise=n, sigma_max=SIG[1])
    a, b = 1 + std**2 / (2 * s) * dt, 1 + std**2 * (1 - s) / (2 * s)
    assert torch.allclose(mean.double(), x.double() * a + v.double() * b * dt, rtol=0, atol=1e-6)
    assert torch.allclose(prev.double(), mean.double() + std * math.sqrt(-dt) * n.double(), rtol=0, atol=1e-6)


def test_flow_sigma_one_branch_uses_sigma_max():
    # at sigma == 1 the denominator is 1 - sigma_max, not 1 - sigma
    s, sn, eta, smax = 1.0, float(SIG[1]), 0.7, float(SIG[1])
    std = math.sqrt(1.0 / (1 - smax)) * eta
    assert abs(std - 6.3387570) < 2e-5
    assert abs(std * math.sqrt(-(sn - s)) - 0.7) < 1e-6
    x, v, n = _inputs((2, 8), 2)
    _, lp, mean = osde.sde_denoise("flow", v, x, SIG[0], SIG[1], eta=eta, noise=n, sigma_max=SIG[1])
    assert torch.isfinite(lp).all() and torch.isfinite(mean).all()
    # a different sigma_max changes the result only through this branch
    _, lp2, _ = osde.sde_denoise("flow", v, x, SIG[0], SIG[1], eta=eta, noise=n, sigma_max=0.5)
    assert not torch.allclose(lp, lp2)
    _, lp3, _ = osde.sde_denoise("flow", v, x, SIG[5], SIG[6], eta=eta, noise=n, sigma_max=0.5)
    _, lp4, _ = osde.sde_denoise("flow", v, x, SIG[5], SIG[6], eta=eta, noise=n, sigma_max=SIG[1])
    assert torch.equal(lp3, lp4)


@pytest.mark.parametrize("kind", ["flow", "dance"])
def test_eta_zero_is_euler(kind):
    x, v, n = _inputs((3, 4, 5), 3)
    prev, lp, mean = osde.sde_denoise(kind, v, x, SIG[7], SIG[8], eta=0.0, noise=n)
    assert lp is None
    euler = x + v * (SIG[8] - SIG[7])
    assert torch.allclose(mean, euler, rtol=0, atol=1e-6)
    assert torch.allclose(prev, euler, rtol=0, atol=1e-6)


def test_cps_closed_form():
    x, v, n = _inputs((2, 6), 4)
    s, sn = SIG[9], SIG[10]
    prev, lp, mean = osde.sde_denoise("cps", v, x, s, sn, eta=0.0, noise=n)
    assert lp is None
    x0 = x - s * v
    eps_hat = x + v * (1 - s)
    assert torch.allclose(mean, x0 * (1 - sn) + eps_hat * sn, rtol=0, atol=1e-6)
    # eta = 1: std = sigma_next, the noise-estimate coefficient vanishes
    prev, lp, mean = osde.sde_denoise("cps", v, x, s, sn, eta=1.0, noise=n)
    assert torch.allclose(mean, x0 * (1 - sn), rtol=0, atol=1e-6)
    assert torch.allclose(prev, mean + sn * n, rtol=0, atol=1e-6)
    assert torch.allclose(lp, -((sn * n) ** 2).mean(dim=1), rtol=1e-5, atol=1e-7)


def test_dance_is_flow_with_constant_std():
    # dance differs from flow only in std_dev_t == eta: compare with the flow formula evaluated by hand
    x, v, n = _inputs((2, 5), 5)
    s, sn, eta = float(SIG[12]), float(SIG[13]), 0.7
    dt = sn - s
    _, lp, mean = osde.sde_denoise("dance", v, x, SIG[12], SIG[13], eta=eta, noise=n)
    ref_mean = x.double() * (1 + eta**2 / (2 * s) * dt) + v.double() * (1 + eta**2 * (1 - s) / (2 * s)) * dt
    assert torch.allclose(mean.double(), ref_mean, rtol=0, atol=1e-6)
    sv = eta * math.sqrt(-dt)
    ref_lp = scipy.stats.norm.logpdf((ref_mean + sv * n.double()).numpy(), ref_mean.numpy(), sv).mean(axis=1)
    assert np.allclose(lp.double().numpy(), ref_lp, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("kind", ["flow", "dance"])
def test_logprob_is_gaussian_logpdf(kind):
    x, v, n = _inputs((4, 3, 8, 8), 6)
    i = 10
    prev, lp, mean = osde.sde_denoise(kind, v, x, SIG[i], SIG[i + 1], eta=0.7, noise=n, sigma_max=SIG[1])
    s, sn = float(SIG[i]), float(SIG[i + 1])
    std = math.sqrt(s / (1 - s)) * 0.7 if kind == "flow" else 0.7
    sv = std * math.sqrt(-(sn - s))
    ref = scipy.stats.norm.logpdf(prev.double().numpy(), mean.double().numpy(), sv).reshape(4, -1).mean(axis=1)
    assert np.allclose(lp.double().numpy(), ref, rtol=1e-5, atol=1e-6)
    ref_t = torch.distributions.Normal(mean.double(), sv).log_prob(prev.double()).reshape(4, -1).mean(dim=1)
    assert torch.allclose(lp.double(), ref_t, rtol=1e-5, atol=1e-6)
    # replaying the stored transition gives the sampling-time log-prob back
    _, lp_replay, mean_replay = osde.sde_denoise(kind, v, x, SIG[i], SIG[i + 1], eta=0.7, prev_sample=prev,
                                                 sigma_max=SIG[1])
    assert torch.equal(mean_replay, mean) and torch.equal(lp_replay, lp)


def test_sampling_identity_and_expectation():
    # prev - mean = s*n up to rounding, so lp_elem = -n^2/2 - log s - 0.5 log 2pi; E = -0.5 - log s - 0.5 log 2pi
    x, v, n = _inputs((8, 16, 64, 64), 7)
    i = 10
    _, lp, _ = osde.sde_denoise("flow", v, x, SIG[i], SIG[i + 1], eta=0.7, noise=n, sigma_max=SIG[1])
    s, sn = float(SIG[i]), float(SIG[i + 1])
    sv = math.sqrt(s / (1 - s)) * 0.7 * math.sqrt(-(sn - s))
    ident = (-(n.double() ** 2) / 2).reshape(8, -1).mean(dim=1) - math.log(sv) - 0.5 * math.log(2 * math.pi)
    assert torch.allclose(lp.double(), ident, rtol=0, atol=5e-6)
    expect = -0.5 - math.log(sv) - 0.5 * math.log(2 * math.pi)
    D = 16 * 64 * 64
    assert abs(float(lp.mean()) - expect) < 5 * math.sqrt(0.5 / (8 * D))


@pytest.mark.parametrize("kind", osde.KINDS)
def test_against_float64_brute_force(kind):
    x, v, n = _inputs((2, 3, 4, 4), 8)
    for i in (0, 10, 27):
        prev, lp, mean = osde.sde_denoise(kind, v, x, SIG[i], SIG[i + 1], eta=0.7, noise=n, sigma_max=SIG[1])
        bp, blp, bm = osde.sde_denoise_f64(
            kind, v.reshape(2, -1).tolist(), x.reshape(2, -1).tolist(), float(SIG[i]), float(SIG[i + 1]), 0.7,
            noise=n.reshape(2, -1).tolist(), sigma_max=float(SIG[1]),
        )
        assert np.allclose(mean.reshape(2, -1).double().numpy(), bm, rtol=1e-5, atol=1e-5)
        assert np.allclose(prev.reshape(2, -1).double().numpy(), bp, rtol=1e-5, atol=1e-5)
        assert np.allclose(lp.double().numpy(), blp, rtol=2e-4, atol=2e-4)  # fp32 (prev-mean)^2/(2 s^2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_dtype_round_trip(dtype):
    x, v, n = _inputs((2, 4, 8, 8), 9, dtype)
    prev, lp, mean = osde.sde_denoise("flow", v, x, SIG[10], SIG[11], eta=0.7, noise=n, sigma_max=SIG[1])
    assert prev.dtype == torch.float32 and mean.dtype == torch.float32
    assert torch.equal(prev.to(dtype).float(), prev)  # exactly representable in the input dtype
    # the log-prob is evaluated on the rounded sample
    sv = float(SIG[10])
    sv = math.sqrt(sv / (1 - sv)) * 0.7 * math.sqrt(-(float(SIG[11]) - float(SIG[10])))
    ref = torch.distributions.Normal(mean.double(), sv).log_prob(prev.double()).reshape(2, -1).mean(dim=1)
    assert torch.allclose(lp.double(), ref, rtol=1e-5, atol=1e-6)


def test_per_sample_sigma_matches_per_call():
    x, v, n = _inputs((3, 2, 4, 4), 10)
    idx = [3, 10, 20]
    s = SIG[idx]
    sn = SIG[[i + 1 for i in idx]]
    prev, lp, mean = osde.sde_denoise("flow", v, x, s, sn, eta=0.7, noise=n, sigma_max=SIG[1])
    for b, i in enumerate(idx):
        p1, l1, m1 = osde.sde_denoise("flow", v[b : b + 1], x[b : b + 1], SIG[i], SIG[i + 1], eta=0.7,
                                      noise=n[b : b + 1], sigma_max=SIG[1])
        assert torch.equal(p1[0], prev[b]) and torch.equal(m1[0], mean[b]) and torch.equal(l1[0], lp[b])


def test_rollout_is_chained_single_steps():
    g = torch.Generator().manual_seed(11)
    x0 = torch.randn(2, 16, 8, generator=g)
    vs = [torch.randn(x0.shape, generator=g) for _ in range(4)]
    ns = [torch.randn(x0.shape, generator=g) for _ in range(4)]
    etas = [0.7, 0.0, 0.7, 0.7]
    xf, lps, traj = osde.sde_rollout("flow", x0, vs, ns, SIG, etas)
    x = x0
    for k in range(4):
        prev, lp, _ = osde.sde_denoise("flow", vs[k], x, SIG[k], SIG[k + 1], eta=etas[k], noise=ns[k],
                                       sigma_max=SIG[1])
        if lp is None:
            assert torch.isnan(lps[:, k]).all()
        else:
            assert torch.equal(lps[:, k], lp)
        x = prev
        assert torch.equal(traj[k], x)
    assert torch.equal(xf, x)
