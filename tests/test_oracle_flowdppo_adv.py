"""Pins the CPU oracle of the Flow-DPPO KL mask, sigma_t, the step gather and the advantages."""

import math

import numpy as np
import pytest
import torch

from oracle import advantages as oadv
from oracle import flowdppo as ofd
from oracle import schedule as osch


def test_kl_closed_forms():
    g = torch.Generator().manual_seed(0)
    p = torch.randn(2, 3, 4, 5, 6, generator=g)
    sig = torch.tensor([0.25, 0.5, 2.0]).reshape(1, 3, 1, 1, 1)
    assert float(ofd.kl_per_sample(p, p.clone(), sig).abs().max()) == 0.0
    # constant shift delta (power of two): kl = delta^2 / (2 sigma^2) exactly, in every dtype
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        base = torch.randint(-8, 8, p.shape, generator=g).to(dtype)  # small integers: exact in bf16
        kl = ofd.kl_per_sample(base + 0.5, base, sig)
        assert kl.dtype == torch.float32
        expect = 0.25 / (2 * sig.reshape(1, 3) ** 2)
        assert torch.equal(kl, expect.expand(2, 3))
    q = p + 0.1 * torch.randn(p.shape, generator=g)
    ref = torch.distributions.kl_divergence(
        torch.distributions.Normal(p.double(), sig.double().expand_as(p)),
        torch.distributions.Normal(q.double(), sig.double().expand_as(p)),
    ).mean(dim=(2, 3, 4))
    assert torch.allclose(ofd.kl_per_sample(p, q, sig).double(), ref, rtol=1e-5, atol=1e-9)


def test_kl_16bit_promotion_rounds_difference_and_square():
    # bf16 - bf16 and **2 round to bf16 before the fp32 division
    p = torch.tensor([[[1.0078125, 3.0]]], dtype=torch.bfloat16)   # 1 + 2^-7
    q = torch.tensor([[[0.33203125, 1.0]]], dtype=torch.bfloat16)
    sig = torch.ones(1, 1, 1)
    d = (p.float() - q.float()).to(torch.bfloat16)
    sq = (d.float() * d.float()).to(torch.bfloat16).float()
    assert torch.equal(ofd.gaussian_kl(p, q, sig), sq / 2)
    assert ofd.gaussian_kl(p, q, sig).dtype == torch.float32


def test_flowdppo_truth_table_and_metrics():
    # rows: (kl high?, ratio vs 1, advantage sign) -> removed?
    cases = []
    for kl_high in (False, True):
        for ld in (-0.1, 0.0, 0.1):
            for a in (-1.0, 0.0, 1.0):
                cases.append((kl_high, ld, a))
    n = len(cases)
    new_logp = torch.tensor([c[1] for c in cases]).reshape(n, 1)
    old_logp = torch.zeros(n, 1)
    adv = torch.tensor([c[2] for c in cases]).reshape(n, 1)
    delta = torch.tensor([1.0 if c[0] else 0.0 for c in cases]).reshape(n, 1, 1, 1, 1)
    old_means = torch.zeros(n, 1, 2, 2, 2)
    new_means = old_means + delta  # kl = 1/2 (high) or 0 (low) with sigma 1
    loss, m = ofd.flowdppo_loss(new_logp, old_logp, new_means, old_means, adv, torch.ones(1, 1, 1, 1, 1), 0.01)
    for i, (kl_high, ld, a) in enumerate(cases):
        removed = kl_high and ((ld > 0 and a > 0) or (ld < 0 and a < 0))
        expect = 0.0 if removed else -a * math.exp(ld)
        assert abs(float(loss[i, 0]) - expect) < 1e-6, (i, cases[i])
    n_rm = sum(1 for (k, ld, a) in cases if k and ((ld > 0 and a > 0) or (ld < 0 and a < 0)))
    assert abs(float(m["masked_fraction"]) - n_rm / n) < 1e-7
    assert abs(float(m["unmasked_fraction"]) - (1 - n_rm / n)) < 1e-7
    assert abs(float(m["kl_mask_fraction"]) - 0.5) < 1e-7
    assert abs(float(m["kl_new_old_max"]) - 0.5) < 1e-7 and abs(float(m["kl_new_old_mean"]) - 0.25) < 1e-7


def test_sigma_t_closed_form_and_clamp_edge():
    sig = osch.sigma_schedule(28, 3.0)
    st = ofd.sigma_t(sig, [0, 10, 27], 0.7)
    assert st.shape == (1, 3, 1, 1, 1)
    for j, i in enumerate([0, 10, 27]):
        s, sn = float(sig[i]), float(sig[i + 1])
        ref = math.sqrt(s / (1 - min(s, 0.99))) * 0.7 * math.sqrt(-(sn - s))
        assert abs(float(st[0, j, 0, 0, 0]) - ref) <= 2e-6 * ref
    assert torch.equal(ofd.sigma_t(sig, [1, 2], 0.7, add_kl_coefficient=False), torch.ones(1, 2, 1, 1, 1))


def test_gather_matches_lookup_and_raises():
    g = torch.Generator().manual_seed(1)
    t = torch.randn(3, 5, 2, 4, generator=g)
    idx = torch.tensor([7, 2, 9, 0, 4])  # unsorted
    for target in ([2, 9], [0, 4, 7], [9], [4, 4]):
        assert torch.equal(ofd.gather_sde_field(t, idx, target), ofd.gather_by_lookup(t, idx, target))
    with pytest.raises(ValueError):
        ofd.gather_sde_field(t, idx, [3])
    with pytest.raises(ValueError):
        ofd.gather_sde_field(t, idx, [11])
    with pytest.raises(ValueError):
        ofd.gather_sde_field(None, idx, [2])


# ---------------------------------------------------------------- advantages
def test_group_advantages_numpy_forms():
    g = torch.Generator().manual_seed(2)
    r = torch.rand(24, generator=g)
    pids = [f"p{i // 6}" for i in range(24)]
    rn = r.double().numpy().reshape(4, 6)
    adv = oadv.compute_advantages(r, pids)
    ref = (rn - rn.mean(1, keepdims=True)) / np.sqrt(rn.var(1, ddof=0, keepdims=True) + 1e-8)
    assert np.allclose(adv.numpy().reshape(4, 6), ref, rtol=1e-5, atol=1e-6)
    adv = oadv.compute_advantages(r, pids, normalize=False)
    assert np.allclose(adv.numpy().reshape(4, 6), rn - rn.mean(1, keepdims=True), rtol=0, atol=1e-6)
    adv = oadv.compute_advantages(r, pids, use_global_std=True)
    ref = (rn - rn.mean(1, keepdims=True)) / (rn.reshape(-1).std(ddof=1) + 1e-8)
    assert np.allclose(adv.numpy().reshape(4, 6), ref, rtol=1e-5, atol=1e-6)
    adv = oadv.compute_advantages(r, pids, scope="global")
    ref = (rn.reshape(-1) - rn.mean()) / (rn.reshape(-1).std(ddof=1) + 1e-8)
    assert np.allclose(adv.numpy(), ref, rtol=1e-5, atol=1e-6)


def test_group_advantages_degenerate_and_errors():
    r = torch.tensor([1.0, 1.0, 1.0, 0.0, 1.0, 0.0])
    adv = oadv.compute_advantages(r, ["a", "a", "a", "b", "b", "b"])
    assert adv[:3].tolist() == [0.0, 0.0, 0.0]  # all-equal group -> exactly 0
    assert float(oadv.compute_advantages(torch.tensor([3.0]), ["x"])[0]) == 0.0  # single-sample group
    assert oadv.compute_advantages(r, None).tolist() == [0.0] * 6  # root track
    with pytest.raises(ValueError):
        oadv.compute_advantages(r, ["a", "b", "a", "b", "a", "b"])  # interleaved
    with pytest.raises(ValueError):
        oadv.compute_advantages(r[:5], ["a", "a", "a", "b", "b"])  # non-uniform


def test_normalize_grouped_forms():
    g = torch.Generator().manual_seed(3)
    r = torch.rand(12, generator=g)
    groups = [[0, 5, 7, 2], [1, 3, 4, 6, 8, 9, 10, 11]]
    out = oadv.normalize_grouped(r, groups)
    for idx in groups:
        v = r[idx].double().numpy()
        assert np.allclose(out[idx].numpy(), (v - v.mean()) / (v.std(ddof=1) + 1e-8), rtol=1e-5, atol=1e-6)
    out = oadv.normalize_grouped(r, groups, trim_outliers_ratio=0.25, clip_max=1.0)
    v = np.sort(r[groups[1]].double().numpy())[2:-2]
    full = r[groups[1]].double().numpy()
    ref = np.clip((full - v.mean()) / (v.std(ddof=1) + 1e-8), -1, 1)
    assert np.allclose(out[groups[1]].numpy(), ref, rtol=1e-5, atol=1e-6)
    rn = r.double().numpy()
    assert np.allclose(oadv.normalize_global(r).numpy(), (rn - rn.mean()) / (rn.std(ddof=1) + 1e-8), rtol=1e-5,
                       atol=1e-6)
