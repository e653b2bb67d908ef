"""GPU parity of the fused GRPO / DRPO token-loss kernels against the CPU oracle."""

import math

import pytest
import torch

from oracle import advantages as oadv
from oracle import losses as olos
from tests._util import FP32_RTOL, assert_close

pytestmark = pytest.mark.gpu

MODES = ("token-mean", "seq-mean-token-sum-norm", "seq-mean-token-mean")


def batch(n_seq, max_len, seed, min_len=0, scale=0.05):
    g = torch.Generator().manual_seed(seed)
    old = -8 * torch.rand(n_seq, max_len, generator=g)
    new = old + scale * torch.randn(n_seq, max_len, generator=g)
    lengths = torch.randint(min_len, max_len + 1, (n_seq,), generator=g)
    rewards = (torch.rand(n_seq, generator=g) < 0.5).float()
    group = max(1, n_seq // 4)
    adv = oadv.compute_advantages(rewards, [i // group for i in range(n_seq)])
    return new, old, lengths, adv


def loss_atol(ref_elem_abs_mean):
    """The aggregated loss is a signed sum that largely cancels; fp32 accumulation (ours per lane,
    the reference's everywhere) limits absolute accuracy to ~1e-6 of the mean magnitude."""
    return 2e-6 * ref_elem_abs_mean


def check_metrics(kind, got, ref, n_tok):
    """Counter-based fractions are exact unless a token sits within 1 ulp of its threshold."""
    for name, r in ref.items():
        g = float(got[name])
        r = float(r)
        if "clip" in name:
            assert abs(g - r) <= 2.0 / n_tok + 1e-7, (name, g, r)
        elif name in ("ratio_min", "ratio_max", "rollout_replay_logp_absdiff_max"):
            assert abs(g - r) <= 2e-6 * abs(r), (name, g, r)
        elif name == "ratio_std":
            # the spread of ratios near 1 cannot be known better than one ulp of the ratios (1.2e-7):
            # device expf and host exp may differ by that much per element
            assert abs(g - r) <= FP32_RTOL * abs(r) + 2e-7, (name, g, r)
        else:
            assert abs(g - r) <= FP32_RTOL * abs(r) + 1e-9, (name, g, r)


@pytest.mark.parametrize("kind", ["grpo", "drpo"])
@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("shape", [(16, 512), (7, 37), (3, 1000)])
def test_fused_loss_padded_and_packed(dev, kind, mode, shape):
    from unirl_amd import _native as N
    from unirl_amd.algorithms import fused_token_loss
    from unirl_amd.algorithms._fused import ABSDIFF_METRICS, DRPO_METRICS, GRPO_METRICS

    if kind == "drpo" and mode == "seq-mean-token-mean":
        pytest.skip("the reference's DRPO has no seq-mean-token-mean mode")
    new, old, lengths, adv = batch(*shape, seed=sum(shape))
    newp, oldp = olos.pack_padded(new, lengths), olos.pack_padded(old, lengths)
    kw = dict(clip_range=0.2, clip_range_high=0.28, epsilon=5.0)
    npk = newp.clone().requires_grad_(True)
    ref_loss, ref_m = olos.token_loss(kind, npk, oldp, adv, lengths, mode=mode, horizon=shape[1], **kw)
    ref_loss.backward()
    elem_abs = float(olos.token_loss(kind, newp, oldp, adv, lengths, mode="token-mean", **kw)[0].abs()) + float(adv.abs().mean())
    slots = dict(GRPO_METRICS if kind == "grpo" else DRPO_METRICS, **ABSDIFF_METRICS)

    # padded layout: [n_seq, max_len] + lengths
    nd = new.to(dev).requires_grad_(True)
    loss, mvec = fused_token_loss(kind, nd, old.to(dev), adv.to(dev), lengths=lengths.to(dev), loss_agg_mode=mode,
                                  horizon=shape[1], clip_range=0.2, clip_range_high=0.28, drpo_epsilon=5.0)
    loss.backward()
    assert_close(loss, ref_loss, FP32_RTOL, loss_atol(elem_abs), f"{kind} {mode} padded loss")
    vals = mvec.tolist()
    assert vals[N.M_NUM_TOKENS] == float(lengths.sum())
    check_metrics(kind, {k: vals[s] for k, s in slots.items()}, ref_m, int(lengths.sum()))
    gp = olos.pack_padded(nd.grad.cpu(), lengths)
    assert_close(gp, npk.grad, 1e-5, 1e-6 * float(npk.grad.abs().max()), "padded grad")
    pad_mask = torch.arange(shape[1])[None, :] >= lengths[:, None]
    assert float(nd.grad.cpu()[pad_mask].abs().sum()) == 0.0

    # packed layout: [total_tokens] + cu_seqlens
    cu = torch.cat([torch.zeros(1, dtype=torch.int64), lengths.cumsum(0)])
    nd2 = newp.to(dev).requires_grad_(True)
    loss2, mvec2 = fused_token_loss(kind, nd2, oldp.to(dev), adv.to(dev), cu_seqlens=cu.to(dev), loss_agg_mode=mode,
                                    horizon=shape[1], clip_range=0.2, clip_range_high=0.28, drpo_epsilon=5.0)
    loss2.backward()
    assert_close(loss2, ref_loss, FP32_RTOL, loss_atol(elem_abs), f"{kind} {mode} packed loss")
    assert_close(nd2.grad, npk.grad, 1e-5, 1e-6 * float(npk.grad.abs().max()), "packed grad")
    check_metrics(kind, {k: mvec2.tolist()[s] for k, s in slots.items()}, ref_m, int(lengths.sum()))


@pytest.mark.parametrize("shape", [(1000,), (4, 3), (257, 31)])
def test_grpo_clip_loss_signature(dev, shape):
    from unirl_amd.algorithms import _grpo_clip_loss

    g = torch.Generator().manual_seed(1)
    old = -8 * torch.rand(shape, generator=g)
    new = old + 0.3 * torch.randn(shape, generator=g)
    adv = torch.randn(shape, generator=g)
    for hi in (None, 0.28):
        nr = new.clone().requires_grad_(True)
        ref_elem, ref_m = olos.grpo_clip_loss(nr, old, adv, 0.2, hi)
        ref_elem.mean().backward()
        nd = new.to(dev).requires_grad_(True)
        elem, m = _grpo_clip_loss(new_logp=nd, old_logp=old.to(dev), advantages=adv.to(dev), clip_range=0.2,
                                  clip_range_high=hi)
        elem.mean().backward()
        assert elem.shape == new.shape and set(m) == set(ref_m)
        assert all(v.dim() == 0 and not v.requires_grad for v in m.values())
        assert_close(elem, ref_elem, FP32_RTOL, 1e-7, "loss_per_elem")
        assert_close(nd.grad, nr.grad, 1e-5, 1e-6 * float(nr.grad.abs().max()), "grad")
        check_metrics("grpo", m, ref_m, new.numel())


def test_grpo_clip_loss_single_element_and_broadcast_adv(dev):
    from unirl_amd.algorithms import _grpo_clip_loss

    one = torch.tensor([-1.0])
    elem, m = _grpo_clip_loss(new_logp=(one + 0.1).to(dev), old_logp=one.to(dev), advantages=torch.tensor([2.0]).to(dev),
                              clip_range=0.2)
    ref_elem, ref_m = olos.grpo_clip_loss(one + 0.1, one, torch.tensor([2.0]), 0.2)
    assert float(m["ratio_std"]) == 0.0 == float(ref_m["ratio_std"])
    assert_close(elem, ref_elem, FP32_RTOL, 0, "single element")
    # [B,1] advantages expanded over S' steps (the FlowGRPO call shape)
    g = torch.Generator().manual_seed(2)
    old = torch.randn(6, 3, generator=g) * 1e-3
    new = old + 1e-4 * torch.randn(6, 3, generator=g)
    adv = torch.randn(6, 1, generator=g)
    elem, m = _grpo_clip_loss(new_logp=new.to(dev), old_logp=old.to(dev), advantages=adv.to(dev).expand(6, 3),
                              clip_range=1e-4)
    ref_elem, ref_m = olos.grpo_clip_loss(new, old, adv.expand(6, 3), 1e-4)
    assert_close(elem, ref_elem, FP32_RTOL, 1e-9, "flowgrpo-shaped")
    check_metrics("grpo", m, ref_m, 18)


@pytest.mark.parametrize("mu_weighted", [True, False])
def test_drpo_loss_signature_and_clamp(dev, mu_weighted):
    from unirl_amd.algorithms import _drpo_loss

    g = torch.Generator().manual_seed(3)
    old = -8 * torch.rand(777, generator=g)
    new = old + 0.5 * torch.randn(777, generator=g)
    new[0], new[1], new[2] = old[0] + 25.0, old[1] - 30.0, old[2] + 20.0
    adv = torch.randn(777, generator=g)
    for eps in (5.0, 12.5):
        nr = new.clone().requires_grad_(True)
        ref_elem, ref_m = olos.drpo_loss(nr, old, adv, eps, mu_weighted)
        ref_elem.sum().backward()
        nd = new.to(dev).requires_grad_(True)
        elem, m = _drpo_loss(new_logp=nd, old_logp=old.to(dev), advantages=adv.to(dev), epsilon=eps,
                             mu_weighted=mu_weighted)
        elem.sum().backward()
        assert set(m) == set(ref_m)
        assert_close(elem, ref_elem, FP32_RTOL, 1e-7, "drpo loss_per_elem")
        assert_close(nd.grad, nr.grad, 1e-5, 1e-6 * float(nr.grad.abs().max()), "drpo grad")
        assert float(nd.grad[0]) == 0.0 and float(nd.grad[1]) == 0.0
        check_metrics("drpo", m, ref_m, 777)


def test_drpo_loss_mask_divides_by_all_tokens(dev):
    from unirl_amd.algorithms import fused_token_loss

    new, old, lengths, adv = batch(6, 40, seed=4, min_len=5)
    newp, oldp = olos.pack_padded(new, lengths), olos.pack_padded(old, lengths)
    mask = (torch.rand(newp.shape, generator=torch.Generator().manual_seed(5)) < 0.7).float()
    npk = newp.clone().requires_grad_(True)
    ref_loss, _ = olos.token_loss("drpo", npk, oldp, adv, lengths, epsilon=12.5, loss_mask=mask)
    ref_loss.backward()
    cu = torch.cat([torch.zeros(1, dtype=torch.int64), lengths.cumsum(0)])
    nd = newp.to(dev).requires_grad_(True)
    loss, _ = fused_token_loss("drpo", nd, oldp.to(dev), adv.to(dev), cu_seqlens=cu.to(dev), loss_mask=mask.to(dev),
                               drpo_epsilon=12.5)
    loss.backward()
    assert_close(loss, ref_loss, FP32_RTOL, 1e-7, "masked loss")
    assert_close(nd.grad, npk.grad, 1e-5, 1e-6 * float(npk.grad.abs().max()), "masked grad")
    assert float(nd.grad.cpu()[mask == 0].abs().sum()) == 0.0


def test_invariants_on_device(dev):
    from unirl_amd.algorithms import _drpo_loss, _grpo_clip_loss

    g = torch.Generator().manual_seed(6)
    old = (-8 * torch.rand(500, generator=g)).to(dev)
    adv = torch.randn(500, generator=g).to(dev)
    elem, m = _grpo_clip_loss(new_logp=old.clone(), old_logp=old, advantages=adv, clip_range=0.2, clip_range_high=0.28)
    assert torch.equal(elem, -adv)
    assert float(m["ratio_mean"]) == 1.0 and float(m["ratio_std"]) == 0.0 and float(m["clip_fraction"]) == 0.0
    assert float(m["approx_kl"]) == 0.0
    elem, m = _drpo_loss(new_logp=old.clone(), old_logp=old, advantages=adv, epsilon=12.5)
    assert torch.equal(elem, -adv) and float(m["drpo_penalty_mean"]) == 0.0
    elem, _ = _grpo_clip_loss(new_logp=old + 0.1, old_logp=old, advantages=torch.zeros_like(adv), clip_range=0.2)
    assert float(elem.abs().max()) == 0.0


def test_clip_counters_near_threshold_are_counted(dev):
    """Ratios placed on a fine grid across both clip edges: the device counters may differ from the
    CPU's only for tokens whose ratio lies within 1 ulp of an edge; those are counted and reported."""
    from unirl_amd.algorithms import _grpo_clip_loss

    lo, hi = 0.2, 0.28
    r = torch.cat([torch.linspace(0.79999, 0.80001, 4001), torch.linspace(1.27999, 1.28001, 4001)])
    new, old = torch.log(r), torch.zeros_like(r)
    adv = torch.ones_like(r)
    _, ref_m = olos.grpo_clip_loss(new, old, adv, lo, hi)
    _, m = _grpo_clip_loss(new_logp=new.to(dev), old_logp=old.to(dev), advantages=adv.to(dev), clip_range=lo,
                           clip_range_high=hi)
    ratio_cpu = torch.exp(new - old)
    eps32 = torch.finfo(torch.float32).eps
    near = ((ratio_cpu - 1.0 - hi).abs() <= 2 * eps32) | ((1.0 - ratio_cpu - lo).abs() <= 2 * eps32)
    n_near = int(near.sum())
    n = r.numel()
    for key in ("clipfrac_gt_one", "clipfrac_lt_one", "clip_fraction"):
        mismatched = abs(float(m[key]) - float(ref_m[key])) * n
        print(f"{key}: device {float(m[key]):.6f} cpu {float(ref_m[key]):.6f} "
              f"mismatching tokens {mismatched:.1f}, tokens within 1 ulp of an edge {n_near}")
        assert mismatched <= n_near + 0.5


def test_expand_advantages_kernel(dev):
    from unirl_amd.algorithms import GRPO

    adv = torch.tensor([1.0, -2.0, 3.0, 0.5, 7.0])
    lengths = torch.tensor([3, 0, 2, 1, 1000])
    out = GRPO._expand_advantages_to_tokens(adv.to(dev), lengths.to(dev), dtype=torch.float32, device=dev)
    assert torch.equal(out.cpu(), olos.expand_advantages(adv, lengths))
    out = GRPO._expand_advantages_to_tokens(adv, lengths, dtype=torch.bfloat16, device=dev)
    assert out.dtype == torch.bfloat16 and out.shape == (1006,)
    empty = GRPO._expand_advantages_to_tokens(adv.to(dev), torch.zeros(5, dtype=torch.int64), dtype=torch.float32,
                                              device=dev)
    assert empty.shape == (0,)


def test_absdiff_gauge(dev):
    from unirl_amd.algorithms import rollout_replay_logp_absdiff

    g = torch.Generator().manual_seed(7)
    old = -8 * torch.rand(4099, generator=g)
    new = old + 0.2 * torch.randn(4099, generator=g)
    got = rollout_replay_logp_absdiff(new.to(dev), old.to(dev))
    ref = olos.logp_absdiff(new, old)
    assert set(got) == set(ref) and all(isinstance(v, float) for v in got.values())
    assert abs(got["rollout_replay_logp_absdiff_mean"] - ref["rollout_replay_logp_absdiff_mean"]) < 1e-6
    assert got["rollout_replay_logp_absdiff_max"] == ref["rollout_replay_logp_absdiff_max"]


def test_layout_errors(dev):
    from unirl_amd.algorithms import fused_token_loss

    x = torch.zeros(4, 8, device=dev)
    with pytest.raises(ValueError):
        fused_token_loss("grpo", x, x, torch.zeros(3, device=dev), lengths=torch.ones(4, dtype=torch.int64))
    with pytest.raises(ValueError):
        fused_token_loss("grpo", x, x, torch.zeros(4, device=dev), lengths=torch.ones(3, dtype=torch.int64))
    with pytest.raises(ValueError):
        fused_token_loss("grpo", x, x[:, :4], torch.zeros(4, device=dev), lengths=torch.ones(4, dtype=torch.int64))
    with pytest.raises(ValueError):
        fused_token_loss("grpo", x, x, torch.zeros(4, device=dev), lengths=torch.ones(4, dtype=torch.int64),
                         loss_agg_mode="nope")


def test_many_sequences_and_empty_rows(dev):
    from unirl_amd.algorithms import fused_token_loss

    new, old, lengths, adv = batch(3000, 24, seed=8, min_len=0)
    lengths[::7] = 0
    newp, oldp = olos.pack_padded(new, lengths), olos.pack_padded(old, lengths)
    for mode in MODES:
        ref_loss, _ = olos.token_loss("grpo", newp, oldp, adv, lengths, mode=mode, horizon=24, clip_range=0.2)
        loss, _ = fused_token_loss("grpo", new.to(dev), old.to(dev), adv.to(dev), lengths=lengths.to(dev),
                                   loss_agg_mode=mode, horizon=24, clip_range=0.2)
        assert_close(loss, ref_loss, FP32_RTOL, 2e-6, f"3000 rows {mode}")


def test_config3_shape(dev):
    """fp32 [256, 8192], lengths U[512, 8192], 16 groups of 16 Bernoulli rewards (seed 1003);
    GRPO 0.2/0.28 and DRPO with 1/(2 eps) = 0.1 (eps 5) and eps 12.5, token-mean."""
    from unirl_amd import _native as N
    from unirl_amd.algorithms import fused_token_loss
    from unirl_amd.algorithms._fused import ABSDIFF_METRICS, DRPO_METRICS, GRPO_METRICS
    from unirl_amd.types import compute_advantages

    g = torch.Generator().manual_seed(1003)
    old = -8 * torch.rand(256, 8192, generator=g)
    new = old + 0.05 * torch.randn(256, 8192, generator=g)
    lengths = torch.randint(512, 8193, (256,), generator=g)
    rewards = (torch.rand(256, generator=g) < 0.5).float()
    pids = [i // 16 for i in range(256)]
    adv_ref = oadv.compute_advantages(rewards, pids)
    adv = compute_advantages(rewards.to(dev), pids)
    assert_close(adv, adv_ref, FP32_RTOL, 1e-7, "advantages")
    newp, oldp = olos.pack_padded(new, lengths), olos.pack_padded(old, lengths)
    n_tok = int(lengths.sum())
    for kind, kw, okw in (("grpo", dict(clip_range=0.2, clip_range_high=0.28), dict(clip_range=0.2, clip_range_high=0.28)),
                          ("drpo", dict(drpo_epsilon=5.0), dict(epsilon=5.0)),
                          ("drpo", dict(drpo_epsilon=12.5), dict(epsilon=12.5))):
        npk = newp.clone().requires_grad_(True)
        ref_loss, ref_m = olos.token_loss(kind, npk, oldp, adv_ref, lengths, **okw)
        ref_loss.backward()
        nd = new.to(dev).requires_grad_(True)
        loss, mvec = fused_token_loss(kind, nd, old.to(dev), adv, lengths=lengths.to(dev), **kw)
        loss.backward()
        # loss = mean of -A*r over ~1.1M tokens with sum(A) ~ 0: the terms cancel to ~1e-3 of their size
        assert_close(loss, ref_loss, FP32_RTOL, 2e-6 * float(adv_ref.abs().mean()), f"config-3 {kind} loss")
        vals = mvec.tolist()
        assert vals[N.M_NUM_TOKENS] == float(n_tok)
        slots = dict(GRPO_METRICS if kind == "grpo" else DRPO_METRICS, **ABSDIFF_METRICS)
        check_metrics(kind, {k: vals[s] for k, s in slots.items()}, ref_m, n_tok)
        assert_close(olos.pack_padded(nd.grad.cpu(), lengths), npk.grad, 1e-5, 1e-6 * float(npk.grad.abs().max()),
                     "config-3 grad")


@pytest.mark.parametrize("kind", ["grpo", "drpo"])
@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("shape", [(16, 512), (7, 37), (3, 1000), (40, 2048)])
@pytest.mark.parametrize("with_mask", [False, True])
def test_one_pass_loss_and_gradient(dev, kind, mode, shape, with_mask):
    """The one-pass training step: metrics of the forward, and in new_logp.grad what
    (loss * loss_scale).backward() of the oracle leaves there -- padded layout with device and host
    lengths, packed layout, with and without a loss mask."""
    from unirl_amd import _native as N
    from unirl_amd.algorithms._fused import ABSDIFF_METRICS, DRPO_METRICS, GRPO_METRICS, fused_token_loss_backward

    if kind == "drpo" and mode == "seq-mean-token-mean":
        pytest.skip("the reference's DRPO has no seq-mean-token-mean mode")
    if kind == "grpo" and with_mask:
        pytest.skip("the reference's GRPO takes no loss mask")
    loss_scale = 0.37
    new, old, lengths, adv = batch(*shape, seed=11 + sum(shape))
    newp, oldp = olos.pack_padded(new, lengths), olos.pack_padded(old, lengths)
    g = torch.Generator().manual_seed(5)
    maskp = (torch.rand(newp.shape, generator=g) < 0.7).float() if with_mask else None
    kw = dict(clip_range=0.2, clip_range_high=0.28, epsilon=5.0)
    npk = newp.clone().requires_grad_(True)
    ref_loss, ref_m = olos.token_loss(kind, npk, oldp, adv, lengths, mode=mode, horizon=shape[1], loss_mask=maskp, **kw)
    (ref_loss * loss_scale).backward()
    elem_abs = float(olos.token_loss(kind, newp, oldp, adv, lengths, mode="token-mean", **kw)[0].abs()) + float(adv.abs().mean())
    slots = dict(GRPO_METRICS if kind == "grpo" else DRPO_METRICS, **ABSDIFF_METRICS)
    gtol = 1e-6 * float(npk.grad.abs().max())
    common = dict(loss_scale=loss_scale, loss_agg_mode=mode, horizon=shape[1], clip_range=0.2, clip_range_high=0.28,
                  drpo_epsilon=5.0)
    mask2d = None
    if with_mask:
        mask2d = torch.zeros(shape)
        col = torch.arange(shape[1])[None, :] < lengths[:, None]
        mask2d[col] = maskp

    for where in ("device", "host"):  # lengths on the host let the wrapper pass the token count
        nd = new.to(dev).requires_grad_(True)
        twice = nd * 1.0  # a non-leaf: the gradient must flow on through the graph
        mvec = fused_token_loss_backward(
            kind, twice, old.to(dev), adv.to(dev), lengths=lengths.to(dev) if where == "device" else lengths,
            loss_mask=None if mask2d is None else mask2d.to(dev), **common)
        vals = mvec.tolist()
        assert_close(torch.tensor(vals[N.M_LOSS]), ref_loss, FP32_RTOL, loss_atol(elem_abs), f"{kind} {mode} loss")
        assert vals[N.M_NUM_TOKENS] == float(lengths.sum())
        check_metrics(kind, {k: vals[s] for k, s in slots.items()}, ref_m, int(lengths.sum()))
        assert_close(olos.pack_padded(nd.grad.cpu(), lengths), npk.grad, 1e-5, gtol, f"padded grad ({where} lengths)")
        pad = torch.arange(shape[1])[None, :] >= lengths[:, None]
        assert float(nd.grad.cpu()[pad].abs().sum()) == 0.0

    cu = torch.cat([torch.zeros(1, dtype=torch.int64), lengths.cumsum(0)])
    nd2 = newp.to(dev).requires_grad_(True)
    mvec2 = fused_token_loss_backward(kind, nd2, oldp.to(dev), adv.to(dev), cu_seqlens=cu.to(dev),
                                      loss_mask=None if maskp is None else maskp.to(dev), **common)
    assert_close(torch.tensor(mvec2.tolist()[N.M_LOSS]), ref_loss, FP32_RTOL, loss_atol(elem_abs), "packed loss")
    assert_close(nd2.grad, npk.grad, 1e-5, gtol, "packed grad")


def test_one_pass_matches_two_launch_backward_bitwise(dev):
    """Same expressions as the stand-alone backward kernel: identical bits, ties and clamps included."""
    from unirl_amd import _native as N
    from unirl_amd.ops import RatioLossPlan

    new, old, lengths, adv = batch(32, 777, seed=3, scale=0.3)
    new[0, :5] = old[0, :5] + math.log(1.28)  # on / next to the clip edge
    new[1, :5] = old[1, :5] + 25.0            # past DRPO's clamp
    for code, kw in ((N.LOSS_GRPO, dict(clip_low=0.2, clip_high=0.28)), (N.LOSS_DRPO, dict(drpo_epsilon=5.0))):
        plan = RatioLossPlan(new.to(dev), old.to(dev), adv.to(dev), kind=code, lengths=lengths.to(dev), **kw)
        _, m = plan.forward(False)
        scale = torch.tensor([0.37], device=dev)
        g2 = plan.backward(g_scale=scale, g_elem=None, aggregate=True, n_valid=m[N.M_NUM_TOKENS : N.M_NUM_TOKENS + 1])
        g1, m1 = plan.forward_backward(0.37)
        assert torch.equal(g1, g2)
        assert torch.equal(m1[:13], m[:13])


def test_one_pass_without_graph_runs_forward_only(dev):
    from unirl_amd.algorithms._fused import fused_token_loss_backward

    new, old, lengths, adv = batch(4, 64, seed=9)
    m = fused_token_loss_backward("grpo", new.to(dev), old.to(dev), adv.to(dev), lengths=lengths.to(dev), loss_scale=1.0)
    assert m.shape == (16,) and bool(torch.isfinite(m[:13]).all())


@pytest.mark.parametrize("kind", ["grpo", "drpo"])
@pytest.mark.parametrize("case", ["many_short", "mixed", "one", "edges"])
def test_packed_layout_sequence_tracking(dev, kind, case):
    """The packed kernel follows the sequences span by span: thousands of sequences shorter than a
    span (several boundaries per span, more than 4096 sequences: a three-round search), long and
    short ones mixed, a single sequence, boundaries exactly on span and vector edges, empty
    sequences, a token count that is no multiple of four -- loss, metrics and the one-pass
    gradient against the oracle in every aggregation mode."""
    from unirl_amd import _native as N
    from unirl_amd.algorithms._fused import fused_token_loss_backward

    g = torch.Generator().manual_seed({"many_short": 1, "mixed": 2, "one": 3, "edges": 4}[case])
    if case == "many_short":
        lengths = torch.randint(0, 41, (5000,), generator=g)
    elif case == "mixed":
        lengths = torch.cat([torch.randint(1000, 5000, (6,), generator=g), torch.randint(0, 300, (60,), generator=g)])
        lengths = lengths[torch.randperm(lengths.numel(), generator=g)]
    elif case == "one":
        lengths = torch.tensor([70001])
    else:
        lengths = torch.tensor([256, 256, 512, 0, 0, 252, 4, 1, 3, 1024, 255, 257, 768, 2])
    n_seq, T = lengths.numel(), int(lengths.sum())
    old = -8 * torch.rand(T, generator=g)
    new = old + 0.05 * torch.randn(T, generator=g)
    adv = torch.randn(n_seq, generator=g)
    cu = torch.cat([torch.zeros(1, dtype=torch.int64), lengths.cumsum(0)])
    kw = dict(clip_range=0.2, clip_range_high=0.28, epsilon=5.0)
    for mode in MODES:
        if kind == "drpo" and mode == "seq-mean-token-mean":
            continue
        leaf = new.clone().requires_grad_(True)
        ref_loss, ref_m = olos.token_loss(kind, leaf, old, adv, lengths, mode=mode, horizon=4096, **kw)
        (ref_loss * 0.5).backward()
        nd = new.to(dev).requires_grad_(True)
        mvec = fused_token_loss_backward(kind, nd, old.to(dev), adv.to(dev), cu_seqlens=cu.to(dev), loss_scale=0.5,
                                         loss_agg_mode=mode, horizon=4096, clip_range=0.2, clip_range_high=0.28,
                                         drpo_epsilon=5.0)
        vals = mvec.tolist()
        scale = float(olos.token_loss(kind, new, old, adv, lengths, mode="token-mean", **kw)[0].abs()) + float(adv.abs().mean())
        assert_close(torch.tensor(vals[N.M_LOSS]), ref_loss, FP32_RTOL, loss_atol(scale), f"{case} {mode} loss")
        assert vals[N.M_NUM_TOKENS] == float(T)
        assert_close(nd.grad.cpu(), leaf.grad, 1e-5, 1e-6 * float(leaf.grad.abs().max()), f"{case} {mode} grad")
        assert abs(vals[N.M_RATIO_MAX] - float(ref_m["ratio_max"])) <= 2e-6 * float(ref_m["ratio_max"])


@pytest.mark.parametrize("with_grad", [False, True])
def test_c_abi_empty_input_writes_the_metrics(dev, with_grad):
    """n_tok == 0 through the C ABI itself (the tensor wrapper answers empty inputs on the host):
    nothing is read, the count is 0 and the means are NaN, like ``torch.mean`` of nothing."""
    import ctypes

    from unirl_amd import _native as N
    from unirl_amd import ops

    params = ops._ratio_params(N.LOSS_GRPO, "token-mean", 0.2, 0.28, 12.5, True, 8192, True)
    dummy = torch.zeros(4, device=dev)
    metrics = torch.full((N.M_COUNT,), 7.0, device=dev)
    stream = N.current_stream(dev)
    ws, ws_bytes = N.workspace(dev, stream)
    head = (N.ptr(dummy), N.ptr(dummy), N.ptr(dummy), None, None, 0, 0, 0, ctypes.byref(params))
    tail = (N.ptr(metrics), N.ptr(ws), ws_bytes, stream)
    if with_grad:
        rc = N.lib().unirl_ratio_loss_fwd_bwd(*head, 1.0, -1, N.ptr(dummy), *tail)
    else:
        rc = N.lib().unirl_ratio_loss_fwd(*head, None, *tail)
    assert rc == 0
    torch.cuda.synchronize()
    got = metrics.cpu()
    assert float(got[N.M_NUM_TOKENS]) == 0.0
    for slot in (N.M_LOSS, N.M_RATIO_MEAN, N.M_APPROX_KL, N.M_CLIP_FRACTION, N.M_ABSDIFF_MEAN):
        assert math.isnan(float(got[slot])), slot
    assert torch.equal(dummy.cpu(), torch.zeros(4))


@pytest.mark.parametrize("lengths", [[2, 1, 0], [0, 1, 2], [1, 0, 0, 3, 1, 0, 0, 2, 1, 2, 0, 2]])
def test_packed_batch_with_as_many_tokens_as_sequences(dev, lengths):
    """``advantages [n]`` fits both readings when a packed batch holds n tokens in n sequences:
    it is read per sequence (what the reference's algorithms pass) unless the caller says per token."""
    from unirl_amd.algorithms import fused_token_loss

    lengths = torch.tensor(lengths)
    n = int(lengths.numel())
    assert int(lengths.sum()) == n
    g = torch.Generator().manual_seed(11 + n)
    old = -8 * torch.rand(n, generator=g)
    new = old + 0.3 * torch.randn(n, generator=g)
    adv = torch.randn(n, generator=g)
    cu = torch.cat([torch.zeros(1, dtype=torch.int64), lengths.cumsum(0)])
    kw = dict(clip_range=0.2, clip_range_high=0.28)
    ref_seq, _ = olos.token_loss("grpo", new, old, adv, lengths, mode="token-mean", epsilon=5.0, **kw)
    ref_tok = olos.grpo_clip_loss(new, old, adv, 0.2, 0.28)[0].mean()
    assert abs(float(ref_seq) - float(ref_tok)) > 1e-3  # the two readings differ on these inputs
    args = ("grpo", new.to(dev), old.to(dev), adv.to(dev))
    got_seq, _ = fused_token_loss(*args, cu_seqlens=cu.to(dev), **kw)
    got_seq2, _ = fused_token_loss(*args, cu_seqlens=cu.to(dev), adv_per_token=False, **kw)
    got_tok, _ = fused_token_loss(*args, cu_seqlens=cu.to(dev), adv_per_token=True, **kw)
    assert_close(got_seq, ref_seq, FP32_RTOL, 1e-6, "per sequence (default)")
    assert_close(got_seq2, ref_seq, FP32_RTOL, 1e-6, "per sequence (explicit)")
    assert_close(got_tok, ref_tok, FP32_RTOL, 1e-6, "per token (explicit)")
    with pytest.raises(ValueError):
        fused_token_loss(*args[:3], adv.to(dev)[:-1], cu_seqlens=cu.to(dev), adv_per_token=True, **kw)
