"""Pins the CPU oracle of the token log-prob / entropy and of the GRPO / DRPO losses."""

import math

import numpy as np
import pytest
import torch

from oracle import losses as olos
from oracle import token_logp as otok


# ---------------------------------------------------------------- token log-prob / entropy
def _logits(rows, V, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    x = (2 * torch.randn(rows, V, generator=g)).to(dtype)
    ids = torch.randint(0, V, (rows,), generator=g)
    return x, ids


@pytest.mark.parametrize("T", [1.0, 0.7, 2.0])
def test_logp_is_log_softmax_gather(T):
    x, ids = _logits(6, 1000, 1, torch.bfloat16)
    ref = torch.log_softmax(x.float() / T, dim=-1).gather(-1, ids[:, None])[:, 0]
    assert torch.allclose(otok.token_logp(x, ids, T), ref, rtol=1e-6, atol=1e-6)
    ref_ent = torch.distributions.Categorical(logits=x.float() / T).entropy()
    assert torch.allclose(otok.token_entropy(x, T), ref_ent, rtol=1e-5, atol=1e-6)


def test_temperature_nonpositive_means_one():
    x, ids = _logits(3, 50, 2)
    assert torch.equal(otok.token_logp(x, ids, 0.0), otok.token_logp(x, ids, 1.0))
    assert torch.equal(otok.token_logp(x, ids, -3.0), otok.token_logp(x, ids, 1.0))


def test_uniform_and_peaked_rows():
    V = 151936
    x = torch.zeros(2, V)
    ids = torch.tensor([5, V - 1])
    assert torch.allclose(otok.token_logp(x, ids), torch.full((2,), -math.log(V)), rtol=1e-6, atol=0)
    assert torch.allclose(otok.token_entropy(x), torch.full((2,), math.log(V)), rtol=1e-6, atol=0)
    assert abs(math.log(V) - 11.9312) < 1e-4
    x[0, 7] = 60.0  # one overwhelming logit: p -> 1, logp -> 0, entropy -> 0
    lp = otok.token_logp(x, torch.tensor([7, 0]))
    assert abs(float(lp[0])) < 1e-6
    assert 0.0 <= float(otok.token_entropy(x)[0]) < 1e-6


def test_shift_invariance_and_bounds():
    x, ids = _logits(5, 777, 3)
    lp, ent = otok.token_logp(x, ids), otok.token_entropy(x)
    lp2, ent2 = otok.token_logp(x + 3.25, ids), otok.token_entropy(x + 3.25)
    assert torch.allclose(lp, lp2, rtol=1e-5, atol=1e-5) and torch.allclose(ent, ent2, rtol=1e-5, atol=1e-5)
    assert bool((lp <= 0).all()) and bool((ent >= 0).all()) and bool((ent <= math.log(777) + 1e-6).all())


def test_against_float64_brute_force():
    x, ids = _logits(4, 300, 4, torch.bfloat16)
    x[1, 11] = 15.0
    for T in (1.0, 0.7):
        lp, ent = otok.token_logp(x, ids, T), otok.token_entropy(x, T)
        for r in range(4):
            blp, bent = otok.token_logp_entropy_f64(x[r].float().tolist(), int(ids[r]), T)
            assert abs(float(lp[r]) - blp) <= 1e-5 * abs(blp) + 2e-6
            assert abs(float(ent[r]) - bent) <= 1e-5 * abs(bent) + 1e-6
    a, b = otok.token_logp_entropy_chunked(x, ids, 0.7, chunk=3)
    assert torch.equal(a, otok.token_logp(x, ids, 0.7)) and torch.equal(b, otok.token_entropy(x, 0.7))


def test_entropy_of_masked_logits_follows_categorical():
    """A -inf logit (a masked token) has probability 0 and adds nothing to the entropy: the value is
    that of the remaining tokens, as ``torch.distributions.Categorical`` computes it; a row with
    one finite logit has entropy 0; NaN and +inf logits give NaN."""
    x, _ = _logits(6, 40, 9)
    x[0, 3] = x[0, 17] = -math.inf
    x[1, :] = -math.inf
    x[1, 2] = 1.5
    x[2, ::2] = -math.inf
    ent = otok.token_entropy(x[:3], 0.7)
    ref = torch.distributions.Categorical(logits=(x[:3] / 0.7).double()).entropy()
    assert torch.allclose(ent.double(), ref, rtol=1e-6, atol=1e-9)
    kept = x[0][torch.isfinite(x[0])]
    assert abs(float(ent[0]) - float(otok.token_entropy(kept[None], 0.7))) < 1e-6  # the masked entries drop out
    assert float(ent[1]) == 0.0
    x[4, 5] = math.nan
    x[5, 1] = math.inf
    assert bool(torch.isnan(otok.token_entropy(x[4:])).all())


# ---------------------------------------------------------------- GRPO clip loss
def _logps(n, seed=0, scale=0.05, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    old = (-8 * torch.rand(n, generator=g)).to(dtype)
    new = old + (scale * torch.randn(n, generator=g)).to(dtype)
    adv = torch.randn(n, generator=g).to(dtype)
    return new, old, adv


def test_grpo_on_policy_invariants():
    new, old, adv = _logps(64, 1)
    loss, m = olos.grpo_clip_loss(old.clone(), old, adv, 0.2, 0.28)
    assert torch.equal(loss, -adv)
    for k in ("clip_fraction", "clipfrac_gt_one", "clipfrac_lt_one", "approx_kl", "ratio_std"):
        assert float(m[k]) == 0.0
    assert float(m["ratio_mean"]) == 1.0 and float(m["ratio_min"]) == 1.0 and float(m["ratio_max"]) == 1.0
    loss0, _ = olos.grpo_clip_loss(new, old, torch.zeros_like(adv), 0.2)
    assert float(loss0.abs().max()) == 0.0


def test_grpo_brute_force_grid_and_symmetric_default():
    # scan the ratio across both clip edges for both advantage signs, against a scalar python formula
    lo, hi = 0.2, 0.28
    r = torch.linspace(0.6, 1.5, 181, dtype=torch.float64)
    for a in (1.0, -1.0, 0.5, -2.0):
        new = torch.log(r)
        old = torch.zeros_like(new)
        loss, m = olos.grpo_clip_loss(new, old, torch.full_like(new, a), lo, hi)
        ref = [max(-a * float(x), -a * min(max(float(x), 1 - lo), 1 + hi)) for x in r]
        assert np.allclose(loss.numpy(), ref, rtol=1e-12, atol=1e-12)
        gt = sum(float(x) - 1 > hi for x in r) / len(r)
        lt = sum(1 - float(x) > lo for x in r) / len(r)
        assert abs(float(m["clipfrac_gt_one"]) - gt) < 1e-6 and abs(float(m["clipfrac_lt_one"]) - lt) < 1e-6
        assert abs(float(m["clip_fraction"]) - (gt + lt)) < 1e-6
    new, old, adv = _logps(50, 2, scale=0.3)
    a, _ = olos.grpo_clip_loss(new, old, adv, 0.2, None)
    b, _ = olos.grpo_clip_loss(new, old, adv, 0.2, 0.2)
    assert torch.equal(a, b)


def test_grpo_backward_closed_form_and_gradcheck():
    new, old, adv = _logps(200, 3, scale=0.3, dtype=torch.float64)
    new = new.clone().requires_grad_(True)
    loss, _ = olos.grpo_clip_loss(new, old, adv, 0.2, 0.28)
    loss.sum().backward()
    r = torch.exp(new.detach() - old)
    u = -adv * r
    c = -adv * r.clamp(0.8, 1.28)
    inside = (r >= 0.8) & (r <= 1.28)
    expect = torch.where(inside, u, torch.where(u > c, u, torch.zeros_like(u)))
    assert torch.allclose(new.grad, expect, rtol=1e-12, atol=1e-12)
    n2, o2, a2 = _logps(6, 4, scale=0.3, dtype=torch.float64)
    assert torch.autograd.gradcheck(
        lambda z: olos.grpo_clip_loss(z, o2, a2, 0.2, 0.28)[0], (n2.clone().requires_grad_(True),), atol=1e-6
    )


# ---------------------------------------------------------------- DRPO loss
def test_drpo_on_policy_invariants_and_formula():
    new, old, adv = _logps(64, 5)
    loss, m = olos.drpo_loss(old.clone(), old, adv, 12.5)
    assert torch.equal(loss, -adv)
    assert float(m["drpo_penalty_mean"]) == 0.0 and float(m["approx_kl"]) == 0.0
    assert float(m["clipfrac_upper"]) == 0.0 and float(m["clipfrac_lower"]) == 0.0
    new, old, adv = _logps(40, 6, scale=0.5, dtype=torch.float64)
    for mu_w in (True, False):
        loss, m = olos.drpo_loss(new, old, adv, 5.0, mu_w)
        r = torch.exp((new - old).clamp(-20, 20))
        w = torch.exp(old) if mu_w else torch.ones_like(old)
        ref = -adv * r + adv.abs() * w * (r - 1) ** 2 / (2 * 5.0)
        assert torch.allclose(loss, ref, rtol=1e-12, atol=1e-12)
        k3 = ((r - 1) - (new - old).clamp(-20, 20)).mean()
        assert abs(float(m["approx_kl"]) - float(k3)) < 1e-12
        eps_t = 5.0 / torch.exp(old) if mu_w else torch.full_like(old, 5.0)
        assert abs(float(m["clipfrac_upper"]) - float((r > 1 + eps_t).double().mean())) < 1e-12


def test_drpo_backward_closed_form_clamp_and_gradcheck():
    new, old, adv = _logps(100, 7, scale=0.5, dtype=torch.float64)
    new = new.clone()
    new[0] = old[0] + 25.0  # clamp active: zero gradient
    new[1] = old[1] - 30.0
    new.requires_grad_(True)
    loss, _ = olos.drpo_loss(new, old, adv, 5.0, True)
    loss.sum().backward()
    d = new.detach() - old
    r = torch.exp(d.clamp(-20, 20))
    expect = (-adv + adv.abs() * torch.exp(old) * (r - 1) / 5.0) * r
    expect = torch.where(d.abs() > 20, torch.zeros_like(expect), expect)
    assert torch.allclose(new.grad, expect, rtol=1e-10, atol=1e-12)
    assert float(new.grad[0]) == 0.0 and float(new.grad[1]) == 0.0
    n2, o2, a2 = _logps(6, 8, scale=0.3, dtype=torch.float64)
    assert torch.autograd.gradcheck(
        lambda z: olos.drpo_loss(z, o2, a2, 5.0, True)[0], (n2.clone().requires_grad_(True),), atol=1e-6
    )


def test_drpo_stationary_point_is_the_trust_region_boundary():
    """What the mathematics fixes about the penalty's scale, with no formula retyped: for A > 0 the
    per-token loss -A r + |A| mu (r-1)^2 / (2 eps) is stationary in r exactly at r* = 1 + eps/mu, the
    boundary `clipfrac_upper` counts against (for A < 0 at 1 - eps/mu, the one `clipfrac_lower`
    uses).  A penalty of |A| mu (r-1)^2 / eps -- the 2 dropped -- would be stationary at
    1 + eps/(2 mu) and fail here; so would a penalty without mu, or with the wrong sign."""
    for eps, mu, sign in ((0.4, 0.5, 1.0), (12.5, 0.9, 1.0), (5.0, 0.75, 1.0), (0.3, 0.6, -1.0), (0.05, 0.25, -1.0)):
        r_star = 1.0 + sign * eps / mu
        assert r_star > 0.0
        old = torch.tensor([mu], dtype=torch.float64).log()
        adv = torch.tensor([sign * 1.7], dtype=torch.float64)

        def grad_at(r):
            new = (old + torch.tensor([r], dtype=torch.float64).log()).requires_grad_(True)
            loss, m = olos.drpo_loss(new, old, adv, eps, True)
            loss.sum().backward()
            return float(new.grad), m

        g0, _ = grad_at(r_star)
        assert abs(g0) < 1e-12 * abs(float(adv)) * r_star, (eps, mu, sign, g0)
        g_in, m_in = grad_at(1.0 + sign * (eps / mu) * (1 - 1e-3))    # inside the trust region: still descending
        g_out, m_out = grad_at(1.0 + sign * (eps / mu) * (1 + 1e-3))  # outside: the penalty has taken over
        # d loss / d new_logp = r * d loss / d r; moving r away from 1 lowers the loss inside, raises it outside
        assert sign * g_in < 0.0 < sign * g_out
        key = "clipfrac_upper" if sign > 0 else "clipfrac_lower"
        assert float(m_in[key]) == 0.0 and float(m_out[key]) == 1.0
        # the wrong scale's stationary point is not one
        g_half, _ = grad_at(1.0 + sign * eps / (2 * mu))
        assert abs(g_half) > 0.1 * abs(float(adv))


# ---------------------------------------------------------------- expansion / aggregation
def test_expand_and_aggregate():
    adv = torch.tensor([1.0, -2.0, 3.0, 0.5])
    lengths = torch.tensor([3, 0, 2, 1])
    out = olos.expand_advantages(adv, lengths)
    assert out.tolist() == [1.0, 1.0, 1.0, 3.0, 3.0, 0.5]
    with pytest.raises(ValueError):
        olos.expand_advantages(adv, lengths[:3])
    assert olos.expand_advantages(adv, torch.zeros(4, dtype=torch.int64)).shape == (0,)
    elem = torch.arange(6, dtype=torch.float32)
    assert float(olos.aggregate(elem, lengths, "token-mean")) == 2.5
    # seq sums 3, 0, 7, 5 -> mean 3.75 / horizon
    assert abs(float(olos.aggregate(elem, lengths, "seq-mean-token-sum-norm", horizon=10)) - 0.375) < 1e-7
    # seq means 1, 0 (empty), 3.5, 5 -> 2.375
    assert abs(float(olos.aggregate(elem, lengths, "seq-mean-token-mean")) - 2.375) < 1e-7


def test_masked_mean_on_padded_equals_packed_mean():
    g = torch.Generator().manual_seed(9)
    x = torch.randn(5, 12, generator=g)
    lengths = torch.tensor([12, 1, 7, 0, 5])
    mask = (torch.arange(12)[None, :] < lengths[:, None]).float()
    packed = olos.pack_padded(x, lengths)
    assert packed.numel() == int(lengths.sum())
    assert abs(float((x * mask).sum() / mask.sum()) - float(packed.mean())) < 1e-6


def test_absdiff_gauge():
    new, old, _ = _logps(33, 10, scale=0.2)
    d = olos.logp_absdiff(new, old)
    assert abs(d["rollout_replay_logp_absdiff_mean"] - float((new - old).abs().mean())) < 1e-7
    assert d["rollout_replay_logp_absdiff_max"] == float((new - old).abs().max())
