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


def test_more_rows_than_one_launch_can_index(dev):
    """70 001 samples / rows of a few elements each: the second grid dimension holds at most 65 535
    workgroups, so every per-row entry point walks the rows in several launches.  Against the oracle."""
    from oracle import flowdppo as ofd
    from oracle import schedule as osch
    from oracle import sde as osde
    from oracle import token_logp as otok
    from tests._util import assert_close
    from unirl_amd import ops, sde

    R = 70001
    g = torch.Generator().manual_seed(12)
    sig = osch.sigma_schedule(28, 3.0)
    # SDE step, sampling and replay, and its backward
    x, v, n = (torch.randn(R, 8, generator=g) for _ in range(3))
    ref_prev, ref_lp, ref_mean = osde.sde_denoise("flow", v, x, sig[10], sig[11], eta=0.7, noise=n, sigma_max=sig[1],
                                                  ieee_sqrt=True)
    st = sde.FlowSDEStrategy()
    vd = v.to(dev).requires_grad_(True)
    prev, lp, mean = st.denoise(vd, x.to(dev), sig[10].to(dev), sig[11].to(dev), eta=0.7, sigma_max=sig[1].to(dev),
                                noise=n.to(dev))
    assert torch.equal(prev.cpu(), ref_prev) and torch.equal(mean.cpu(), ref_mean)
    assert_close(lp, ref_lp, 1e-5, 2e-6, "log-prob of 70 001 samples")
    gl = torch.randn(R, generator=g)
    vr = v.clone().requires_grad_(True)
    _, rl, _ = osde.sde_denoise("flow", vr, x, sig[10], sig[11], eta=0.7, prev_sample=ref_prev, sigma_max=sig[1])
    (rl * gl).sum().backward()
    _, lp2, _ = st.denoise(vd, x.to(dev), sig[10].to(dev), sig[11].to(dev), eta=0.7, sigma_max=sig[1].to(dev),
                           prev_sample=ref_prev.to(dev))
    (lp2 * gl.to(dev)).sum().backward()
    assert_close(vd.grad, vr.grad, 5e-5, 1e-7, "gradient over 70 001 samples")
    # Gaussian KL and mask, one sigma per row modulo 3
    base = torch.randn(23334, 3, 8, generator=g)  # 70 002 rows
    p = (base + 0.02 * torch.randn(base.shape, generator=g)).bfloat16()
    q = (base + 0.02 * torch.randn(base.shape, generator=g)).bfloat16()
    sg = torch.tensor([0.3, 0.2, 0.1]).view(1, 3, 1)
    ref = ofd.kl_per_sample(p, q, sg)
    kl, _ = ops.gaussian_kl_mask(p.to(dev), q.to(dev), sg.to(dev), 0.01)
    assert kl.shape == ref.shape and kl.numel() > 65535
    assert_close(kl, ref, 2e-3, 1e-9, "kl of 70 002 rows")
    # token log-prob, entropy and backward on 70 001 short rows
    logits = (2 * torch.randn(R, 24, generator=g)).bfloat16()
    ids = torch.randint(0, 24, (R,), generator=g)
    tlp, ent, lse = ops.token_logp_entropy(logits.to(dev), ids.to(dev), 0.7, want_lse=True)
    assert_close(tlp, otok.token_logp(logits, ids, 0.7), 2e-5, 2e-6, "token log-prob of 70 001 rows")
    assert_close(ent, otok.token_entropy(logits, 0.7), 2e-5, 2e-6, "entropy of 70 001 rows")
    lf = logits.float().requires_grad_(True)
    torch.log_softmax(lf / 0.7, -1).gather(-1, ids[:, None])[:, 0].backward(gl)
    grad = ops.token_logp_bwd(logits.to(dev), ids.to(dev), 0.7, lse, gl.to(dev))
    assert_close(grad.float(), lf.grad, 1e-2, 1e-3, "token gradient of 70 001 rows")
    # gather of 70 001 samples
    t = torch.randn(R, 3, 4, generator=g)
    assert torch.equal(ops.gather_steps(t.to(dev), [2, 0]).cpu(), t[:, [2, 0]])
