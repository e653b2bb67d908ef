"""Non-finite inputs: the kernels must treat NaN and infinities the way the reference's eager torch
chain does (torch.clamp and torch.maximum propagate NaN; min()/max()/mean() propagate NaN; the
comparisons behind clip fractions and masks are False on NaN; the FlowDPPO where() keeps inf*0 out;
DRPO clamps the log-ratio to +-20 before exp).  Checked against the CPU oracle, which runs those
torch ops themselves."""

import math

import pytest
import torch

from oracle import advantages as oadv
from oracle import flowdppo as ofd
from oracle import losses as olos
from oracle import schedule as osch
from oracle import sde as osde
from oracle import token_logp as otok
from tests._util import FP32_RTOL, assert_close

pytestmark = pytest.mark.gpu

NAN, INF = float("nan"), float("inf")


def same(got, ref, what, rtol=FP32_RTOL, atol=1e-7):
    """NaN positions and infinities coincide; finite values within tolerance."""
    g = torch.as_tensor(got).detach().double().cpu()
    r = torch.as_tensor(ref).detach().double().cpu()
    assert g.shape == r.shape, what
    assert torch.equal(torch.isnan(g), torch.isnan(r)), f"{what}: NaN positions differ: {g.flatten()[:12]} vs {r.flatten()[:12]}"
    inf_g, inf_r = torch.isinf(g), torch.isinf(r)
    assert torch.equal(inf_g, inf_r) and torch.equal(g[inf_g], r[inf_r]), f"{what}: infinities differ"
    fin = torch.isfinite(r)
    assert_close(g[fin], r[fin], rtol, atol, what)


def poisoned(n, seed):
    g = torch.Generator().manual_seed(seed)
    old = -8 * torch.rand(n, generator=g)
    new = old + 0.3 * torch.randn(n, generator=g)
    adv = torch.randn(n, generator=g)
    return new, old, adv


CASES = {
    "nan_new": lambda new, old, adv: (new.index_fill(0, torch.tensor([3]), NAN), old, adv),
    "nan_old": lambda new, old, adv: (new, old.index_fill(0, torch.tensor([5]), NAN), adv),
    "nan_adv": lambda new, old, adv: (new, old, adv.index_fill(0, torch.tensor([7]), NAN)),
    "ratio_overflow": lambda new, old, adv: (new.index_fill(0, torch.tensor([2, 9]), 100.0), old, adv),
    "ratio_overflow_zero_adv": lambda new, old, adv: (new.index_fill(0, torch.tensor([2]), 100.0), old,
                                                      adv.index_fill(0, torch.tensor([2]), 0.0)),
    "ratio_underflow": lambda new, old, adv: (new.index_fill(0, torch.tensor([4]), -200.0), old, adv),
    "old_minus_inf": lambda new, old, adv: (new, old.index_fill(0, torch.tensor([6]), -INF), adv),
    "both_minus_inf": lambda new, old, adv: (new.index_fill(0, torch.tensor([6]), -INF),
                                             old.index_fill(0, torch.tensor([6]), -INF), adv),
    "inf_adv": lambda new, old, adv: (new, old, adv.index_fill(0, torch.tensor([1]), INF)),
}


@pytest.mark.parametrize("case", sorted(CASES))
def test_grpo_clip_loss_nonfinite(dev, case):
    from unirl_amd.algorithms import _grpo_clip_loss

    new, old, adv = CASES[case](*poisoned(257, 11))
    ref_elem, ref_m = olos.grpo_clip_loss(new, old, adv, 0.2, 0.28)
    elem, m = _grpo_clip_loss(new_logp=new.to(dev), old_logp=old.to(dev), advantages=adv.to(dev), clip_range=0.2,
                              clip_range_high=0.28)
    same(elem, ref_elem, f"grpo elem [{case}]")
    for k, r in ref_m.items():
        same(m[k], r, f"grpo {k} [{case}]", rtol=2e-5, atol=1e-6)


@pytest.mark.parametrize("case", sorted(CASES))
@pytest.mark.parametrize("mu_weighted", [True, False])
def test_drpo_loss_nonfinite(dev, case, mu_weighted):
    from unirl_amd.algorithms import _drpo_loss

    new, old, adv = CASES[case](*poisoned(257, 12))
    ref_elem, ref_m = olos.drpo_loss(new, old, adv, 5.0, mu_weighted)
    elem, m = _drpo_loss(new_logp=new.to(dev), old_logp=old.to(dev), advantages=adv.to(dev), epsilon=5.0,
                         mu_weighted=mu_weighted)
    same(elem, ref_elem, f"drpo elem [{case}]", rtol=2e-5)
    for k, r in ref_m.items():
        same(m[k], r, f"drpo {k} [{case}]", rtol=2e-5, atol=1e-6)


@pytest.mark.parametrize("case", sorted(CASES))
def test_logp_absdiff_nonfinite(dev, case):
    from unirl_amd.algorithms import rollout_replay_logp_absdiff

    new, old, _ = CASES[case](*poisoned(300, 13))
    ref = olos.logp_absdiff(new, old)
    got = rollout_replay_logp_absdiff(new.to(dev), old.to(dev))
    for k in ref:
        same(torch.tensor(got[k]), torch.tensor(ref[k]), f"{k} [{case}]")


@pytest.mark.parametrize("case", sorted(CASES))
def test_flowdppo_loss_nonfinite(dev, case):
    from unirl_amd.algorithms import _flowdppo_kl_adv_loss

    B, S = 6, 4
    g = torch.Generator().manual_seed(14)
    new, old, adv = CASES[case](*poisoned(B * S, 14))
    new, old, adv = new.view(B, S), old.view(B, S), adv.view(B, S)
    base = torch.randn(B, S, 4, 8, 8, generator=g)
    om = (base + 0.05 * torch.randn(base.shape, generator=g)).bfloat16()
    nm = (base + 0.05 * torch.randn(base.shape, generator=g)).bfloat16()
    nm[1, 2, 0, 0, 0] = NAN      # one sample's KL is NaN: never "low KL"
    nm[4, 1, 1, 2, 3] = INF      # one is +inf
    sig = torch.tensor([0.3, 0.25, 0.2, 0.15]).view(1, S, 1, 1, 1)
    ref_elem, ref_m = ofd.flowdppo_loss(new, old, nm, om, adv, sig, 0.01)
    elem, m = _flowdppo_kl_adv_loss(new_logp=new.to(dev), old_logp=old.to(dev), new_means=nm.to(dev),
                                    old_means=om.to(dev), advantages=adv.to(dev), sigma_t=sig.to(dev),
                                    kl_mask_threshold=0.01)
    same(elem, ref_elem, f"flowdppo elem [{case}]")
    for k, r in ref_m.items():
        same(m[k], r, f"flowdppo {k} [{case}]", rtol=2e-3 if "kl_new_old" in k else 2e-5, atol=1e-6)


def test_token_rows_where_a_nan_precedes_every_finite_logit(dev):
    """A wavefront that has met nothing but -inf and NaN sums nothing yet; the NaN must survive
    until the row's result (three-element rows put each element into a scan step of its own)."""
    from unirl_amd import models

    x = torch.tensor([[0.5, 1.0, -1.0], [NAN, 3.0, 1.25], [-INF, NAN, 2.0], [NAN, -INF, -INF], [-INF, 0.25, NAN]])
    ids = torch.tensor([0, 1, 2, 0, 1])
    for dtype in (torch.float32, torch.bfloat16):
        xd = x.to(dtype)
        lp, ent = models.token_logp_entropy(xd.to(dev), ids.to(dev), 0.7)
        same(lp, otok.token_logp(xd, ids, 0.7), f"log-prob {dtype}", 2e-5, 2e-6)
        same(ent, otok.token_entropy(xd, 0.7), f"entropy {dtype}", 2e-5, 2e-6)
    # several +inf logits in one row: the log-sum-exp is +inf, so a finite or masked target has
    # log-prob -inf (not NaN), the +inf tokens themselves inf - inf = NaN
    many = torch.randn(4, 6000)
    many[0, [5, 4000]] = INF
    many[1, [7, 2500, 5999]] = INF
    many[1, 9] = -INF
    many[2, [1, 3000]] = INF
    many[3, [10, 5000]] = INF
    many[3, 77] = NAN
    ids = torch.tensor([100, 9, 3000, 100])
    lp, ent = models.token_logp_entropy(many.to(dev), ids.to(dev), 1.0)
    same(lp, otok.token_logp(many, ids), "log-prob, several +inf", 2e-5, 2e-6)
    assert lp.cpu().tolist()[:2] == [-INF, -INF] and math.isnan(float(lp[2])) and math.isnan(float(lp[3]))
    same(ent, otok.token_entropy(many), "entropy, several +inf", 2e-5, 2e-6)
    big = torch.randn(3, 5000)
    big[1, :700] = NAN          # the first chunks of several wavefronts hold nothing but NaN
    big[2, :300] = -INF
    big[2, 17] = NAN
    ids = torch.tensor([5, 4000, 4000])
    lp, ent = models.token_logp_entropy(big.to(dev), ids.to(dev), 1.0)
    same(lp, otok.token_logp(big, ids), "log-prob, long rows", 2e-5, 2e-6)
    same(ent, otok.token_entropy(big), "entropy, long rows", 2e-5, 2e-6)


def _poison(rng, t, values):
    t = t.clone()
    flat = t.view(-1)
    for _ in range(rng.randint(1, 3)):
        flat[rng.randrange(flat.numel())] = rng.choice(values)
    return t


@pytest.mark.parametrize("seed", range(8))
def test_random_nonfinite_injection(dev, seed):
    """One to three NaN / +-inf / overflowing values dropped at random into otherwise ordinary
    inputs of every kernel: NaN positions, infinities and the finite rest follow the oracle."""
    import random
    import warnings

    from unirl_amd import models, ops, sde
    from unirl_amd.algorithms import fused_token_loss
    from unirl_amd.algorithms._fused import ABSDIFF_METRICS, DRPO_METRICS, GRPO_METRICS

    rng = random.Random(7000 + seed)
    sig = osch.sigma_schedule(28, 3.0)
    for _ in range(6):
        g = torch.Generator().manual_seed(rng.randint(0, 10**6))
        # token log-prob and entropy (|logits| stay small: the reference's `chosen - logsumexp`
        # itself loses digits to cancellation at logits of 1e4)
        rows, V = rng.randint(1, 5), rng.choice((3, 8, 65, 300, 2049))
        dtype, T = rng.choice((torch.float32, torch.bfloat16, torch.float16)), rng.choice((1.0, 0.7))
        x = _poison(rng, 3 * torch.randn(rows, V, generator=g), (NAN, INF, -INF, 100.0, -200.0)).to(dtype)
        ids = torch.randint(0, V, (rows,), generator=g)
        bad = (~torch.isfinite(x.float())).nonzero()
        if len(bad) and rng.random() < 0.5:
            ids[bad[0, 0]] = bad[0, 1]  # the target is the poisoned token
        lp, ent = models.token_logp_entropy(x.to(dev), ids.to(dev), T)
        what = f"token [{rows},{V}] {dtype} T={T}"
        same(lp, otok.token_logp(x, ids, T), what + " log-prob", 2e-5, 2e-5)
        same(ent, otok.token_entropy(x, T), what + " entropy", 2e-5, 2e-6)

        # ratio losses, padded and packed
        n_seq, max_len = rng.randint(1, 6), rng.choice((3, 4, 8, 31, 64, 257))
        kind, mode = rng.choice(("grpo", "drpo")), rng.choice(("token-mean", "seq-mean-token-sum-norm"))
        old = -8 * torch.rand(n_seq, max_len, generator=g)
        new = old + 0.3 * torch.randn(n_seq, max_len, generator=g)
        lengths = torch.randint(1, max_len + 1, (n_seq,), generator=g)
        adv = torch.randn(n_seq, generator=g)
        which = rng.choice(("new", "old", "adv"))
        if which == "new":
            new = _poison(rng, new, (NAN, INF, -INF, 100.0, -200.0, 0.0))
        elif which == "old":
            old = _poison(rng, old, (NAN, INF, -INF, 100.0, -200.0, 0.0))
        else:
            adv = _poison(rng, adv, (NAN, INF, -INF, 0.0))
        newp, oldp = olos.pack_padded(new, lengths), olos.pack_padded(old, lengths)
        ref_loss, ref_m = olos.token_loss(kind, newp, oldp, adv, lengths, mode=mode, horizon=max_len, clip_range=0.2,
                                          clip_range_high=0.28, epsilon=5.0)
        cu = torch.cat([torch.zeros(1, dtype=torch.int64), lengths.cumsum(0)])
        kw = dict(loss_agg_mode=mode, horizon=max_len, clip_range=0.2, clip_range_high=0.28, drpo_epsilon=5.0,
                  adv_per_token=False)
        slots = dict(GRPO_METRICS if kind == "grpo" else DRPO_METRICS)
        slots.update(ABSDIFF_METRICS)
        for layout in ("padded", "packed"):
            if layout == "padded":
                loss, mvec = fused_token_loss(kind, new.to(dev), old.to(dev), adv.to(dev), lengths=lengths.to(dev), **kw)
            else:
                loss, mvec = fused_token_loss(kind, newp.to(dev), oldp.to(dev), adv.to(dev), cu_seqlens=cu.to(dev), **kw)
            what = f"{kind} {mode} [{n_seq},{max_len}] {layout}, poisoned {which}"
            same(loss, ref_loss, what + " loss", 3e-5, 1e-5)
            got = mvec.cpu()
            for name, slot in slots.items():
                if name in ref_m:
                    atol = 2.0 / newp.numel() + 1e-6 if "clip" in name else 1e-5
                    same(got[slot], ref_m[name], f"{what} {name}", 3e-5, atol)

        # Gaussian KL and mask
        B, S, inner = rng.randint(1, 3), rng.randint(1, 3), (rng.randint(1, 9), rng.randint(1, 40))
        dtype = rng.choice((torch.float32, torch.bfloat16, torch.float16))
        base = torch.randn((B, S) + inner, generator=g)
        p = base + 0.02 * torch.randn(base.shape, generator=g)
        q = base + 0.02 * torch.randn(base.shape, generator=g)
        if rng.random() < 0.5:
            p = _poison(rng, p, (NAN, INF, -INF, 1e30, 60000.0))
        else:
            q = _poison(rng, q, (NAN, INF, -INF, 1e30, 60000.0))
        p, q = p.to(dtype), q.to(dtype)
        sg = (0.1 + torch.rand(S, generator=g)).view(1, S, 1, 1)
        ref = ofd.kl_per_sample(p, q, sg)
        kl, mask = ops.gaussian_kl_mask(p.to(dev), q.to(dev), sg.to(dev), 0.01)
        same(kl, ref, f"kl {tuple(base.shape)} {dtype}", 2e-5 if dtype == torch.float32 else 2e-3, 1e-9)
        sure = ~torch.isfinite(ref) | ((ref - 0.01).abs() > 1e-5)
        assert torch.equal(mask.cpu().bool()[sure], (ref < 0.01)[sure])

        # SDE transition and log-prob
        shape, kind = (rng.randint(1, 3), rng.randint(1, 9), rng.randint(1, 40)), rng.choice(("flow", "dance", "cps"))
        i, eta = rng.randint(0, 27), rng.choice((0.3, 0.7, 1.0))
        xs, v, n = (torch.randn(shape, generator=g) for _ in range(3))
        which = rng.choice("xvn")
        vals = (NAN, INF, -INF, 100.0, 3.0e38, 0.0)
        xs, v, n = (_poison(rng, t, vals) if name == which else t for name, t in zip("xvn", (xs, v, n)))
        r_prev, r_lp, r_mean = osde.sde_denoise(kind, v, xs, sig[i], sig[i + 1], eta=eta, noise=n, sigma_max=sig[1],
                                                ieee_sqrt=True)
        prev, lp, mean = sde.STRATEGIES[kind]().denoise(v.to(dev), xs.to(dev), sig[i].to(dev), sig[i + 1].to(dev), eta=eta,
                                                        sigma_max=sig[1].to(dev), noise=n.to(dev))
        what = f"sde {kind} {shape} step {i} eta {eta}, poisoned {which}"
        same(mean, r_mean, what + " mean", 1e-6, 0)
        same(prev, r_prev, what + " prev", 1e-6, 0)
        same(lp, r_lp, what + " log-prob", 3e-5, 2e-6)

        # group-normalised advantages
        G, b = rng.randint(1, 8), rng.randint(1, 6)
        r = _poison(rng, torch.randn(G * b, generator=g), (NAN, INF, -INF, 1e-45))
        akw = dict(normalize=rng.random() < 0.7, scope=rng.choice(("group", "global")), use_global_std=rng.random() < 0.3)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # torch warns about std() of a single element
            ref = oadv.compute_advantages(r, [j // b for j in range(G * b)], **akw)
        same(ops.group_advantages(r.to(dev), G, **akw), ref, f"advantages G={G} b={b} {akw}", 3e-5, 2e-6)


def test_token_logp_nonfinite_rows(dev):
    from unirl_amd import models

    g = torch.Generator().manual_seed(15)
    V = 3001
    x = (2 * torch.randn(8, V, generator=g))
    ids = torch.randint(0, V, (8,), generator=g)
    x[1, 17] = NAN                        # NaN anywhere in the row: lse, log-prob and entropy are NaN
    x[2, 40] = INF
    ids[2] = 41                           # +inf elsewhere: log-prob of a finite token is -inf
    x[3, 50] = INF
    ids[3] = 50                           # the +inf token itself: inf - inf = NaN
    x[4, :] = -INF                        # nothing has mass: NaN
    x[5, 100:] = -INF                     # masked tail is fine
    ids[5] = 7
    x[6, 100:] = -INF
    ids[6] = 200                          # a masked token: -inf
    for dtype in (torch.float32, torch.bfloat16):
        xd = x.to(dtype)
        ref_lp = otok.token_logp(xd, ids, 1.0)
        lp, ent = models.token_logp_entropy(xd.to(dev), ids.to(dev), 1.0)
        same(lp, ref_lp, f"token logp {dtype}", rtol=2e-5, atol=1e-5)
        # entropy (not in the reference): 0 * log 0 = 0 for masked (-inf) entries, as
        # torch.distributions.Categorical has it; NaN where the log-sum-exp is not finite
        fin = torch.isfinite(torch.logsumexp(xd.float(), dim=-1))
        ref_ent = torch.distributions.Categorical(logits=xd.double()[fin]).entropy()
        assert_close(ent.cpu()[fin], ref_ent, 2e-5, 1e-5, "entropy of rows with a finite log-sum-exp")
        assert bool(torch.isnan(ent.cpu()[~fin]).all()), "rows without a finite log-sum-exp must report NaN"


def test_sde_and_kl_propagate_nan(dev):
    from unirl_amd import ops, sde

    sig = osch.sigma_schedule(28, 3.0)
    g = torch.Generator().manual_seed(16)
    x, v, n = (torch.randn(3, 4, 8, 8, generator=g) for _ in range(3))
    v[1, 0, 0, 0] = NAN
    x[2, 1, 2, 3] = INF
    ref_prev, ref_lp, ref_mean = osde.sde_denoise("flow", v, x, sig[10], sig[11], eta=0.7, noise=n, sigma_max=sig[1],
                                                  ieee_sqrt=True)
    prev, lp, mean = sde.FlowSDEStrategy().denoise(v.to(dev), x.to(dev), sig[10].to(dev), sig[11].to(dev), eta=0.7,
                                                   sigma_max=sig[1].to(dev), noise=n.to(dev))
    same(prev, ref_prev, "sde prev", rtol=0.0, atol=0.0)
    same(mean, ref_mean, "sde mean", rtol=0.0, atol=0.0)
    same(lp, ref_lp, "sde logp", atol=2e-6)
    p = torch.randn(3, 2, 4, 8, 8, generator=g).bfloat16()
    q = (p.float() + 0.01 * torch.randn(p.shape, generator=g)).bfloat16()
    q[0, 1, 0, 0, 0] = NAN
    s = torch.tensor([0.2, 0.1]).view(1, 2, 1, 1, 1)
    ref_kl = ofd.kl_per_sample(q, p, s)
    kl, mask = ops.gaussian_kl_mask(q.to(dev), p.to(dev), s.to(dev), 0.01)
    same(kl, ref_kl, "kl", rtol=2e-3)
    assert torch.equal(mask.cpu(), ref_kl < 0.01)


def test_advantages_propagate_nan(dev):
    from unirl_amd.types import compute_advantages

    r = torch.tensor([1.0, 0.0, NAN, 1.0, 0.0, 1.0, 1.0, 0.0])
    pids = [0, 0, 0, 0, 1, 1, 1, 1]
    for kw in ({}, {"use_global_std": True}, {"scope": "global"}, {"normalize": False}):
        same(compute_advantages(r.to(dev), pids, **kw), oadv.compute_advantages(r, pids, **kw), f"advantages {kw}")
