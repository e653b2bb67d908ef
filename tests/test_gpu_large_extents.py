"""Extents past 2^31 elements: every kernel indexes in 64 bits.  Checked on the device through
properties that do not depend on size (a call on the whole tensor against calls on its halves,
and exact counts), since the CPU oracle cannot visit this many elements in test time."""

import pytest
import torch

pytestmark = pytest.mark.gpu

BIG = (1 << 31) + (1 << 22)  # elements


def test_token_logp_rows_past_2g_elements(dev):
    from unirl_amd import ops

    V = 151936
    rows = BIG // V + 2
    assert rows * V > (1 << 31)
    g = torch.Generator(device=dev).manual_seed(3)
    x = torch.empty(rows, V, dtype=torch.bfloat16, device=dev)
    for s in range(0, rows, 2048):
        n = min(2048, rows - s)
        x[s : s + n] = (2 * torch.randn(n, V, generator=g, device=dev)).bfloat16()
    ids = torch.randint(0, V, (rows,), generator=g, device=dev)
    lp, ent, lse = ops.token_logp_entropy(x, ids, 1.0, want_logp=True, want_entropy=True, want_lse=True)
    half = rows // 2
    lp_a, ent_a, _ = ops.token_logp_entropy(x[:half], ids[:half], 1.0, want_logp=True, want_entropy=True)
    lp_b, ent_b, _ = ops.token_logp_entropy(x[half:], ids[half:], 1.0, want_logp=True, want_entropy=True)
    assert torch.equal(lp, torch.cat([lp_a, lp_b])) and torch.equal(ent, torch.cat([ent_a, ent_b]))
    # the last row, beyond the 2^31-th element, against torch on that row alone
    ref = torch.log_softmax(x[-1].float(), -1)[ids[-1]]
    assert abs(float(lp[-1]) - float(ref)) <= 1e-5 * abs(float(ref))
    # backward over the same extent, in place
    g_lp = torch.randn(rows, generator=g, device=dev)
    tail = x[-4:].clone()
    grad = ops.token_logp_bwd(x, ids, 1.0, lse, g_lp, in_place=True)
    ref_tail = ops.token_logp_bwd(tail, ids[-4:], 1.0, lse[-4:], g_lp[-4:])
    assert torch.equal(grad[-4:], ref_tail)


def test_ratio_loss_tokens_past_2g(dev):
    from unirl_amd import _native as N
    from unirl_amd.ops import RatioLossPlan

    n_seq, stride = 1100, 1 << 21  # 2.3e9 slots
    assert n_seq * stride > (1 << 31)
    g = torch.Generator(device=dev).manual_seed(5)
    old = torch.empty(n_seq, stride, device=dev)
    new = torch.empty(n_seq, stride, device=dev)
    for s in range(0, n_seq, 100):
        n = min(100, n_seq - s)
        old[s : s + n] = -8 * torch.rand(n, stride, generator=g, device=dev)
        new[s : s + n] = old[s : s + n] + 0.05 * torch.randn(n, stride, generator=g, device=dev)
    lengths = torch.randint(stride // 2, stride + 1, (n_seq,), generator=g, device=dev)
    adv = torch.randn(n_seq, generator=g, device=dev)
    kw = dict(kind=N.LOSS_GRPO, clip_low=0.2, clip_high=0.28)
    grad, m = RatioLossPlan(new, old, adv, lengths=lengths, **kw).forward_backward(1.0)
    vals = m.tolist()
    n_tok = int(lengths.sum())
    assert vals[N.M_NUM_TOKENS] == float(torch.tensor(float(n_tok), dtype=torch.float32))
    # halves: token counts add up, the token-mean loss is the count-weighted mean of the halves
    h = n_seq // 2
    parts = []
    for sl in (slice(0, h), slice(h, n_seq)):
        _, mp = RatioLossPlan(new[sl], old[sl], adv[sl], lengths=lengths[sl], **kw).forward(False)
        parts.append(mp.tolist())
    na, nb = parts[0][N.M_NUM_TOKENS], parts[1][N.M_NUM_TOKENS]
    mix = (parts[0][N.M_LOSS] * na + parts[1][N.M_LOSS] * nb) / (na + nb)
    assert abs(vals[N.M_LOSS] - mix) <= 1e-5 * abs(mix) + 1e-7
    assert vals[N.M_RATIO_MAX] == max(parts[0][N.M_RATIO_MAX], parts[1][N.M_RATIO_MAX])
    assert vals[N.M_RATIO_MIN] == min(parts[0][N.M_RATIO_MIN], parts[1][N.M_RATIO_MIN])
    # the gradient of the last row (past the 2^31-th slot) against a call on that row alone,
    # rescaled from its own token count to the whole batch's
    last = int(lengths[-1])
    g_row, _ = RatioLossPlan(new[-1:], old[-1:], adv[-1:], lengths=lengths[-1:], **kw).forward_backward(1.0)
    want = g_row[0, :last] * (float(last) / float(n_tok))
    got = grad[-1, :last]
    assert float((got - want).abs().max()) <= 1e-5 * float(want.abs().max())
    assert float(grad[-1, last:].abs().sum()) == 0.0


def test_sde_step_and_kl_rows_past_2g(dev):
    from unirl_amd import ops
    from unirl_amd.sde import get_sigma_schedule

    D = BIG
    g = torch.Generator(device=dev).manual_seed(7)
    sig = get_sigma_schedule(28, 3.0)
    x = torch.randn(1, D, generator=g, device=dev)
    v = torch.randn(1, D, generator=g, device=dev)
    n = torch.randn(1, D, generator=g, device=dev)
    s10, s11 = sig[10:11].to(dev), sig[11:12].to(dev)
    prev, logp, mean = ops.sde_step_logp(v, x, s10, s11, kind="flow", eta=0.7, noise=n, sigma_max=float(sig[1]))
    # the same elements as two samples of half the size: identical prev / mean; the log-prob is a mean
    h = D // 2
    prev2, logp2, mean2 = ops.sde_step_logp(v.view(2, h), x.view(2, h), s10, s11, kind="flow", eta=0.7,
                                            noise=n.view(2, h), sigma_max=float(sig[1]))
    assert torch.equal(prev.view(2, h), prev2) and torch.equal(mean.view(2, h), mean2)
    assert abs(float(logp[0]) - float(logp2.double().mean())) <= 1e-5 * abs(float(logp[0]))
    del prev2, mean2, n
    kl, mask = ops.gaussian_kl_mask(mean, prev, torch.tensor([0.5], device=dev), 0.01, reduce_from_dim=1)
    kl2, _ = ops.gaussian_kl_mask(mean.view(2, h), prev.view(2, h), torch.tensor([0.5], device=dev), 0.01,
                                  reduce_from_dim=1)
    assert abs(float(kl[0]) - float(kl2.double().mean())) <= 1e-5 * abs(float(kl[0]))
