"""Seeded random shapes, dtypes, strides and lengths against the oracle: the tails, alignments and
layout switches that hand-picked shapes may miss.  Every case is small; each test draws a few dozen."""

import random

import pytest
import torch

from oracle import flowdppo as ofd
from oracle import losses as olos
from oracle import schedule as osch
from oracle import sde as osde
from oracle import token_logp as otok
from tests._util import BF16_RTOL, FP32_RTOL, assert_close

pytestmark = pytest.mark.gpu

SIG = osch.sigma_schedule(28, 3.0)
DTYPES = (torch.float32, torch.bfloat16, torch.float16)


def rand_shape(rng, max_elems=6000):
    nd = rng.choice((2, 3, 4, 5))
    while True:
        shape = tuple(rng.randint(1, 9) if i else rng.randint(1, 5) for i in range(nd - 1)) + (rng.randint(1, 67),)
        n = 1
        for s in shape[1:]:
            n *= s
        if n <= max_elems:
            return shape


@pytest.mark.parametrize("seed", range(10))
def test_sde_step_random(dev, seed):
    from unirl_amd import sde

    rng = random.Random(1000 + seed)
    for _ in range(6):
        shape, kind = rand_shape(rng), rng.choice(("flow", "dance", "cps"))
        dtype, vdtype = rng.choice(DTYPES), rng.choice(DTYPES)
        i, eta = rng.randint(0, 27), rng.choice((0.3, 0.7, 1.0))
        g = torch.Generator().manual_seed(rng.randint(0, 10**6))
        x = torch.randn(shape, generator=g).to(dtype)
        v = torch.randn(shape, generator=g).to(vdtype)
        n = torch.randn(shape, generator=g)
        what = f"{kind} {shape} {dtype}/{vdtype} step {i} eta {eta}"
        ref_prev, ref_lp, ref_mean = osde.sde_denoise(kind, v, x, SIG[i], SIG[i + 1], eta=eta, noise=n,
                                                      sigma_max=SIG[1], ieee_sqrt=True)
        st = sde.STRATEGIES[kind]()
        prev, lp, mean = st.denoise(v.to(dev), x.to(dev), SIG[i].to(dev), SIG[i + 1].to(dev), eta=eta,
                                    sigma_max=SIG[1].to(dev), noise=n.to(dev))
        assert torch.equal(mean.cpu(), ref_mean) and torch.equal(prev.cpu(), ref_prev), what
        rtol = FP32_RTOL if dtype == torch.float32 and vdtype == torch.float32 else BF16_RTOL
        assert_close(lp, ref_lp, rtol, 2e-6, what)
        # replay from a stack slice with an odd sample stride
        K = rng.randint(2, 4)
        stack = torch.zeros((shape[0], K) + shape[1:], dtype=dtype, device=dev)
        stack[:, 0], stack[:, K - 1] = x.to(dev), ref_prev.to(dtype).to(dev)
        _, r_lp, r_mean = osde.sde_denoise(kind, v, x, SIG[i], SIG[i + 1], eta=eta, prev_sample=ref_prev.to(dtype),
                                           sigma_max=SIG[1], ieee_sqrt=True)
        means = torch.zeros((shape[0], 3) + shape[1:], dtype=dtype, device=dev)
        lps = torch.zeros(shape[0], 3, device=dev)
        st.denoise_into(v.to(dev), stack[:, 0], SIG[i].to(dev), SIG[i + 1].to(dev), eta=eta,
                        prev_sample=stack[:, K - 1], sigma_max=float(SIG[1]), mean_out=means[:, 1], logp_out=lps[:, 2])
        assert torch.equal(means[:, 1].cpu(), r_mean.to(dtype)), what + " (stack replay)"
        assert_close(lps[:, 2], r_lp, rtol, 2e-6, what + " (stack replay)")


@pytest.mark.parametrize("seed", range(8))
def test_token_logp_random(dev, seed):
    from unirl_amd import models

    rng = random.Random(2000 + seed)
    for _ in range(8):
        rows, V = rng.randint(1, 9), rng.choice((1, 2, 7, 8, 9, 63, 64, 65, 255, 1023, 2049, 4100, 33001))
        dtype, T = rng.choice(DTYPES), rng.choice((1.0, 0.7, 1.3, 0.0))
        g = torch.Generator().manual_seed(rng.randint(0, 10**6))
        pad = rng.randint(0, 9)
        big = (3 * torch.randn(rows, V + pad, generator=g)).to(dtype)
        x = big[:, pad:] if rng.random() < 0.5 else big[:, :V]  # row views: odd strides, odd base alignment
        ids = torch.randint(0, V, (rows,), generator=g)
        what = f"[{rows},{V}] {dtype} T={T} pad={pad}"
        ref_lp = otok.token_logp(x, ids, T)
        ref_ent = otok.token_entropy(x, T)
        xd = big.to(dev)[:, pad:] if x.data_ptr() != big.data_ptr() else big.to(dev)[:, :V]
        lp, ent = models.token_logp_entropy(xd, ids.to(dev), T)
        assert_close(lp, ref_lp, 2e-5, 2e-6, what + " logp")
        assert_close(ent, ref_ent, 2e-5, 2e-6, what + " entropy")


@pytest.mark.parametrize("seed", range(12))
def test_ratio_loss_random(dev, seed):
    from unirl_amd.algorithms import fused_token_loss

    rng = random.Random(3000 + seed)
    for _ in range(6):
        n_seq, max_len = rng.randint(1, 40), rng.choice((1, 3, 4, 8, 31, 64, 100, 257, 1024))
        kind = rng.choice(("grpo", "drpo"))
        mode = rng.choice(("token-mean", "seq-mean-token-sum-norm") + (("seq-mean-token-mean",) if kind == "grpo" else ()))
        g = torch.Generator().manual_seed(rng.randint(0, 10**6))
        old = -8 * torch.rand(n_seq, max_len, generator=g)
        new = old + rng.choice((0.01, 0.05, 0.5)) * torch.randn(n_seq, max_len, generator=g)
        lengths = torch.randint(0 if mode != "seq-mean-token-mean" else 1, max_len + 1, (n_seq,), generator=g)
        if int(lengths.sum()) == 0:
            lengths[0] = max_len
        adv = torch.randn(n_seq, generator=g)
        what = f"{kind} {mode} [{n_seq},{max_len}]"
        newp, oldp = olos.pack_padded(new, lengths), olos.pack_padded(old, lengths)
        kw = dict(clip_range=0.2, clip_range_high=0.28, epsilon=5.0)
        npk = newp.clone().requires_grad_(True)
        ref_loss, _ = olos.token_loss(kind, npk, oldp, adv, lengths, mode=mode, horizon=max_len, **kw)
        ref_loss.backward()
        scale = float(olos.token_loss(kind, newp, oldp, adv, lengths, mode="token-mean", **kw)[0].abs()) + float(adv.abs().mean())
        nd = new.to(dev).requires_grad_(True)
        loss, _ = fused_token_loss(kind, nd, old.to(dev), adv.to(dev), lengths=lengths.to(dev), loss_agg_mode=mode,
                                   horizon=max_len, clip_range=0.2, clip_range_high=0.28, drpo_epsilon=5.0)
        loss.backward()
        assert_close(loss, ref_loss, 2e-5, 4e-6 * scale, what + " padded")
        gmax = float(npk.grad.abs().max())
        assert_close(olos.pack_padded(nd.grad.cpu(), lengths), npk.grad, 2e-5, 2e-6 * gmax, what + " padded grad")
        cu = torch.cat([torch.zeros(1, dtype=torch.int64), lengths.cumsum(0)])
        nd2 = newp.to(dev).requires_grad_(True)
        loss2, _ = fused_token_loss(kind, nd2, oldp.to(dev), adv.to(dev), cu_seqlens=cu.to(dev), loss_agg_mode=mode,
                                    horizon=max_len, clip_range=0.2, clip_range_high=0.28, drpo_epsilon=5.0)
        loss2.backward()
        assert_close(loss2, ref_loss, 2e-5, 4e-6 * scale, what + " packed")
        assert_close(nd2.grad, npk.grad, 2e-5, 2e-6 * gmax, what + " packed grad")


@pytest.mark.parametrize("seed", range(6))
def test_kl_mask_random(dev, seed):
    from unirl_amd import ops

    rng = random.Random(4000 + seed)
    for _ in range(8):
        B, S = rng.randint(1, 4), rng.randint(1, 5)
        inner = rand_shape(rng, 3000)[1:]
        dtype = rng.choice(DTYPES)
        g = torch.Generator().manual_seed(rng.randint(0, 10**6))
        base = torch.randn((B, S) + inner, generator=g)
        p = (base + 0.02 * torch.randn(base.shape, generator=g)).to(dtype)
        q = (base + 0.02 * torch.randn(base.shape, generator=g)).to(dtype)
        sig = (0.1 + torch.rand(S, generator=g)).view((1, S) + (1,) * len(inner)) if rng.random() < 0.7 else torch.tensor([0.4])  # 1-dim: a 0-dim sigma would keep torch's result in 16 bits
        ref = ofd.kl_per_sample(p, q, sig)
        thr = float(ref.median()) if ref.numel() > 1 else 0.01
        kl, mask = ops.gaussian_kl_mask(p.to(dev), q.to(dev), sig.to(dev), thr)
        rtol = FP32_RTOL if dtype == torch.float32 else BF16_RTOL
        assert_close(kl, ref, rtol, 1e-9, f"kl {tuple(base.shape)} {dtype}")
        near = (ref - thr).abs() <= 4 * torch.finfo(torch.float32).eps * abs(thr) + rtol * abs(thr) * (dtype != torch.float32)
        assert torch.equal(mask.cpu()[~near], (ref < thr)[~near])


def _offset(t, k, dev):
    """The same values in a device tensor whose storage starts ``k`` elements into a buffer."""
    buf = torch.empty(t.numel() + k, dtype=t.dtype, device=dev)
    view = buf[k:].view(t.shape)
    view.copy_(t)
    return view


@pytest.mark.parametrize("seed", range(6))
def test_misaligned_base_pointers(dev, seed):
    """Every operand starts a few elements into its buffer (4- or 2-byte aligned only), each by its
    own amount, so the kernels cannot take their 16-byte paths on all of them."""
    from oracle import dpm2 as odpm
    from unirl_amd import ops, sde
    from unirl_amd.algorithms import fused_token_loss_backward

    rng = random.Random(9000 + seed)
    for _ in range(4):
        g = torch.Generator().manual_seed(rng.randint(0, 10**6))
        k = [rng.randint(0, 7) for _ in range(4)]
        # SDE step, sampling and replay
        B, D, kind = rng.randint(1, 4), rng.choice((5, 64, 1000, 4099)), rng.choice(("flow", "dance", "cps"))
        dtype, vdtype, i = rng.choice(DTYPES), rng.choice(DTYPES), rng.randint(0, 27)
        x, v, n = torch.randn(B, D, generator=g).to(dtype), torch.randn(B, D, generator=g).to(vdtype), torch.randn(B, D, generator=g)
        ref_prev, ref_lp, ref_mean = osde.sde_denoise(kind, v, x, SIG[i], SIG[i + 1], eta=0.7, noise=n, sigma_max=SIG[1],
                                                      ieee_sqrt=True)
        st = sde.STRATEGIES[kind]()
        prev, lp, mean = st.denoise(_offset(v, k[0], dev), _offset(x, k[1], dev), SIG[i].to(dev), SIG[i + 1].to(dev),
                                    eta=0.7, sigma_max=SIG[1].to(dev), noise=_offset(n, k[2], dev))
        what = f"{kind} [{B},{D}] {dtype}/{vdtype} offsets {k}"
        rtol = FP32_RTOL if dtype == vdtype == torch.float32 else BF16_RTOL
        assert torch.equal(mean.cpu(), ref_mean) and torch.equal(prev.cpu(), ref_prev), what
        assert_close(lp, ref_lp, rtol, 2e-6, what)
        _, r_lp, r_mean = osde.sde_denoise(kind, v, x, SIG[i], SIG[i + 1], eta=0.7, prev_sample=ref_prev.to(dtype),
                                           sigma_max=SIG[1], ieee_sqrt=True)
        _, lp2, mean2 = st.denoise(_offset(v, k[0], dev), _offset(x, k[1], dev), SIG[i].to(dev), SIG[i + 1].to(dev), eta=0.7,
                                   sigma_max=SIG[1].to(dev), prev_sample=_offset(ref_prev.to(dtype), k[3], dev))
        assert torch.equal(mean2.cpu(), r_mean), what + " replay"
        assert_close(lp2, r_lp, rtol, 2e-6, what + " replay")
        # Gaussian KL
        p = (x.float() + 0.02 * torch.randn(B, D, generator=g)).to(dtype)
        ref = ofd.kl_per_sample(p.view(B, 1, D), x.view(B, 1, D), torch.tensor([0.3]).view(1, 1, 1))
        kl, _ = ops.gaussian_kl_mask(_offset(p.view(B, 1, D), k[0], dev), _offset(x.view(B, 1, D), k[3], dev),
                                     torch.tensor([0.3], device=dev), 0.01)
        assert_close(kl, ref, FP32_RTOL if dtype == torch.float32 else BF16_RTOL, 1e-9, what + " kl")
        # one-pass ratio loss, packed
        n_seq, max_len, lk = rng.randint(1, 20), rng.choice((3, 4, 31, 257, 1024)), rng.choice(("grpo", "drpo"))
        old = -8 * torch.rand(n_seq, max_len, generator=g)
        new = old + 0.05 * torch.randn(n_seq, max_len, generator=g)
        lengths = torch.randint(1, max_len + 1, (n_seq,), generator=g)
        adv = torch.randn(n_seq, generator=g)
        newp, oldp = olos.pack_padded(new, lengths), olos.pack_padded(old, lengths)
        npk = newp.clone().requires_grad_(True)
        ref_loss, _ = olos.token_loss(lk, npk, oldp, adv, lengths, mode="token-mean", clip_range=0.2, clip_range_high=0.28,
                                      epsilon=5.0)
        ref_loss.backward()
        cu = torch.cat([torch.zeros(1, dtype=torch.int64), lengths.cumsum(0)])
        nd = _offset(newp, k[0], dev).requires_grad_(True)
        mvec = fused_token_loss_backward(lk, nd * 1.0, _offset(oldp, k[1], dev), _offset(adv, k[2], dev), cu_seqlens=cu.to(dev),
                                         loss_scale=1.0, clip_range=0.2, clip_range_high=0.28, drpo_epsilon=5.0,
                                         adv_per_token=False)
        scale = float(ref_loss.detach().abs()) + float(adv.abs().mean())
        assert_close(mvec[0], ref_loss.detach(), 2e-5, 4e-6 * scale, f"{lk} [{n_seq},{max_len}] offsets {k}")
        assert_close(nd.grad, npk.grad, 2e-5, 2e-6 * float(npk.grad.abs().max()), f"{lk} gradient, offsets {k}")
        # token log-prob and backward
        rows, V, T = rng.randint(1, 6), rng.choice((7, 64, 1000, 4099)), rng.choice((1.0, 0.7))
        logits = (2 * torch.randn(rows, V, generator=g)).to(dtype)
        ids = torch.randint(0, V, (rows,), generator=g)
        ld = _offset(logits, k[3], dev)
        tlp, ent, lse = ops.token_logp_entropy(ld, ids.to(dev), T, want_lse=True)
        assert_close(tlp, otok.token_logp(logits, ids, T), 2e-5, 2e-6, f"token [{rows},{V}] {dtype} offset {k[3]}")
        assert_close(ent, otok.token_entropy(logits, T), 2e-5, 2e-6, f"entropy [{rows},{V}] {dtype} offset {k[3]}")
        gl = torch.randn(rows, generator=g)
        lf = logits.float().requires_grad_(True)
        torch.log_softmax(lf / T, -1).gather(-1, ids[:, None])[:, 0].backward(gl)
        tol = 2e-5 if dtype == torch.float32 else (1e-2 if dtype == torch.bfloat16 else 2e-3)
        grad = ops.token_logp_bwd(ld, ids.to(dev), T, lse, gl.to(dev))
        assert_close(grad.float(), lf.grad, tol, tol * float(gl.abs().max()) * 0.1 + 1e-7, f"token gradient offset {k[3]}")
        # DPM-Solver-2 step (second order needs two steps of history)
        sig = osch.sigma_schedule(6, 3.0)
        strategy, solver = sde.DPM2Strategy(), odpm.Dpm2Solver(sig)
        strategy.init_schedule(sig)
        xs = x
        for step in range(3):
            vs = torch.randn(B, D, generator=g).to(vdtype)
            want = solver.step(vs, xs, step)
            got, _, _ = strategy.denoise(_offset(vs, k[step], dev), _offset(xs, k[3 - step], dev), sig[step], sig[step + 1],
                                         step_index=step)
            assert torch.equal(got.cpu(), want), f"dpm2 step {step}, offsets {k}"
            xs = want.to(dtype)


@pytest.mark.parametrize("seed", range(8))
def test_sde_replay_random(dev, seed):
    """The batched replay on random stacks, step lists, dtypes and velocity layouts against the
    oracle's single steps: means bit-exact, log-probs to the dtype's tolerance."""
    from unirl_amd import sde

    rng = random.Random(5000 + seed)
    for _ in range(5):
        shape = rand_shape(rng, max_elems=3000)
        B, tail = shape[0], shape[1:]
        kind = rng.choice(("flow", "dance", "cps"))
        dtype, vdtype = rng.choice(DTYPES), rng.choice(DTYPES)
        n_stored = rng.randint(2, 7)
        stored = sorted(rng.sample(range(0, 12), n_stored))
        # trained steps: those whose successor is stored as well; make sure there is at least one
        if not any(s + 1 in stored for s in stored):
            stored = sorted(set(stored) | {stored[0] + 1})
        can = [s for s in stored if s + 1 in stored]
        steps = [rng.choice(can) for _ in range(rng.randint(1, 4))]
        eta = rng.choice((0.3, 0.7, 1.0))
        g = torch.Generator().manual_seed(rng.randint(0, 10**6))
        stack = torch.randn((B, len(stored)) + tail, generator=g).to(dtype)
        step_major = rng.random() < 0.4
        v = torch.randn((B, len(steps)) + tail, generator=g).to(vdtype)
        what = f"{kind} B={B} tail={tail} {dtype}/{vdtype} stored={stored} steps={steps} eta={eta} step_major={step_major}"
        refs = [osde.sde_denoise(kind, v[:, j], stack[:, stored.index(s)], SIG[s], SIG[s + 1], eta=eta,
                                 prev_sample=stack[:, stored.index(s + 1)], sigma_max=SIG[1], ieee_sqrt=True)
                for j, s in enumerate(steps)]
        slot_x, slot_p = sde.replay_slots(stored, steps)
        v_dev = v.transpose(0, 1).contiguous().to(dev) if step_major else v.to(dev)
        lp, means = sde.STRATEGIES[kind]().replay_steps(
            v_dev, stack.to(dev), slot_x, slot_p, [float(SIG[s]) for s in steps], [float(SIG[s + 1]) for s in steps],
            eta=eta, sigma_max=float(SIG[1]), step_major=step_major)
        assert torch.equal(means.cpu(), torch.stack([r[2] for r in refs], 1).to(dtype)), what
        rtol = FP32_RTOL if dtype == torch.float32 and vdtype == torch.float32 else BF16_RTOL
        assert_close(lp, torch.stack([r[1] for r in refs], 1), rtol, 2e-6, what)


@pytest.mark.parametrize("seed", range(8))
def test_lmhead_logp_random(dev, seed):
    """The fused lm_head kernel on random (rows, K, V), with and without bias, at the row counts that
    select each of its three code paths: logits within one bf16 ulp of the float64 product, statistics
    against the oracle on the kernel's own logits."""
    from unirl_amd import ops

    rng = random.Random(6000 + seed)
    for _ in range(3):
        rows = rng.choice((rng.randint(1, 255), rng.randint(256, 511), rng.randint(512, 1100)))
        K = 64 * rng.randint(1, 6)
        V = rng.choice((rng.randint(1, 300), rng.randint(300, 1500)))
        bias, T = rng.random() < 0.5, rng.choice((1.0, 0.7, 1.3))
        g = torch.Generator().manual_seed(rng.randint(0, 10**6))
        h = torch.randn(rows, K, generator=g).bfloat16()
        w = (torch.randn(V, K, generator=g) * (3.0 / K ** 0.5)).bfloat16()
        b = torch.randn(V, generator=g).bfloat16() if bias else None
        ids = torch.randint(0, V, (rows,), generator=g)
        what = f"rows={rows} K={K} V={V} bias={bias} T={T}"
        lp, ent, lse, logits = ops.lmhead_logp(h.to(dev), w.to(dev), None if b is None else b.to(dev), ids.to(dev), T,
                                               want_entropy=True, want_lse=True, want_logits=True)
        exact = h.double() @ w.double().T + (0 if b is None else b.double())
        mag = h.double().abs() @ w.double().abs().T + (0 if b is None else b.double().abs())
        ulp = torch.maximum(exact.abs(), torch.tensor(2.0 ** -126, dtype=torch.float64)).log2().floor().exp2() * 2.0 ** -7
        assert bool(((logits.cpu().double() - exact).abs() <= ulp + mag * 2.0 ** -20).all()), what
        own = logits.cpu()
        assert_close(lp, otok.token_logp(own, ids, T), 1e-5, 2e-6, what + " log-prob")
        assert_close(lse, torch.logsumexp(own.double() / T, dim=-1).float(), 1e-5, 2e-6, what + " lse")
        assert_close(ent, otok.token_entropy(own, T), 1e-5, 2e-6, what + " entropy")


@pytest.mark.parametrize("seed", range(4))
def test_transpose_random(dev, seed):
    from unirl_amd import ops

    rng = random.Random(7000 + seed)
    for _ in range(8):
        rows, cols = rng.randint(1, 400), rng.randint(1, 400)
        dtype = rng.choice((torch.bfloat16, torch.float16, torch.float32))
        pad, off = rng.randint(0, 9), rng.randint(0, 3)
        g = torch.Generator().manual_seed(rng.randint(0, 10**6))
        wide = torch.randn(rows, cols + pad + off, generator=g).to(dtype).to(dev)
        src = wide[:, off : off + cols]
        assert torch.equal(ops.transpose_2d(src), src.t().contiguous()), (rows, cols, dtype, pad, off)
