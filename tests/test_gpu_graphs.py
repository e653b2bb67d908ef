"""HIP graph capture of the fused ops: captured with no warm-up on the capture stream (so the
workspace is first requested inside the capture), replayed several times with fresh inputs and
eager work in between, every replay checked against the eager result of the same inputs."""

import pytest
import torch

from oracle import schedule as osch

pytestmark = pytest.mark.gpu

SIG = osch.sigma_schedule(28, 3.0)


def test_graph_replays_match_eager(dev):
    from unirl_amd import _native as N
    from unirl_amd import ops

    g = torch.Generator(device=dev).manual_seed(5)
    shape = (4, 16, 32, 32)
    x, v, n = (torch.randn(shape, device=dev, generator=g) for _ in range(3))
    logits = torch.randn(64, 4099, device=dev, generator=g).bfloat16()
    ids = torch.randint(0, 4099, (64,), device=dev, generator=g)
    new = -torch.rand(12, 256, device=dev, generator=g)
    old = new + 0.05 * torch.randn(12, 256, device=dev, generator=g)
    lengths = torch.randint(1, 257, (12,), device=dev, generator=g)
    adv = torch.randn(12, device=dev, generator=g)
    p = torch.randn(2, 3, 4, 16, 16, device=dev, generator=g).bfloat16()
    q = (p.float() + 0.02 * torch.randn(p.shape, device=dev, generator=g)).bfloat16()
    st = torch.tensor([0.3, 0.2, 0.1], device=dev)
    s10, s11, smax = SIG[10].to(dev), SIG[11].to(dev), SIG[1].to(dev)

    def run_all():
        prev, lp, mean = ops.sde_step_logp(v, x, s10, s11, kind="flow", eta=0.7, noise=n, sigma_max=smax)
        tlp, ent, _ = ops.token_logp_entropy(logits, ids, 1.0)
        plan = ops.RatioLossPlan(new, old, adv, kind=N.LOSS_GRPO, lengths=lengths, clip_low=0.2, clip_high=0.28)
        _, metrics = plan.forward(False)
        kl, mask = ops.gaussian_kl_mask(p, q, st, 0.01)
        return prev, lp, mean, tlp, ent, metrics, kl, mask

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):  # no warm-up on `side`
        outs = run_all()
    torch.cuda.synchronize()
    for rep in range(4):
        # fresh inputs written in place, with eager work of the library itself between replays
        for t in (x, v, n, new):
            t.copy_(torch.randn(t.shape, device=dev, generator=g) * (0.5 if t is new else 1.0) - (1.0 if t is new else 0.0))
        old.copy_(new + 0.05 * torch.randn(new.shape, device=dev, generator=g))
        logits.copy_(torch.randn(logits.shape, device=dev, generator=g).bfloat16())
        q.copy_((p.float() + 0.02 * (rep + 1) * torch.randn(p.shape, device=dev, generator=g)).bfloat16())
        ops.token_logp_entropy(logits[:8], ids[:8], 0.7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = run_all()
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"replay {rep} differs from eager"
    del graph
    # the stream's workspace was not cached from inside the capture: eager use afterwards is safe
    with torch.cuda.stream(side):
        lp_after = ops.sde_step_logp(v, x, s10, s11, kind="flow", eta=0.7, noise=n, sigma_max=smax)[1]
    torch.cuda.synchronize()
    assert torch.equal(lp_after, ops.sde_step_logp(v, x, s10, s11, kind="flow", eta=0.7, noise=n, sigma_max=smax)[1])


def test_two_streams_keep_their_own_scratch(dev):
    """The reducing kernels park workgroup partials in a workspace between their two launches; calls
    that overlap on different streams must not share it.  Two streams run different inputs at the
    same time, repeatedly; every result equals the one computed alone."""
    from unirl_amd import _native as N
    from unirl_amd import ops

    g = torch.Generator(device=dev).manual_seed(9)

    def make(scale):
        new = -torch.rand(192, 4096, device=dev, generator=g)
        old = new + scale * torch.randn(new.shape, device=dev, generator=g)
        lengths = torch.randint(1, 4097, (192,), device=dev, generator=g)
        adv = torch.randn(192, device=dev, generator=g)
        p = torch.randn(4, 1, 1 << 19, device=dev, generator=g).bfloat16()
        q = (p.float() + scale * torch.randn(p.shape, device=dev, generator=g)).bfloat16()
        x, v, n = (torch.randn(4, 1 << 19, device=dev, generator=g) for _ in range(3))
        return new, old, lengths, adv, p, q, x, v, n

    sig = torch.tensor([0.3], device=dev)
    s10, s11, smax = SIG[10].to(dev), SIG[11].to(dev), SIG[1].to(dev)

    def run(args):
        new, old, lengths, adv, p, q, x, v, n = args
        plan = ops.RatioLossPlan(new, old, adv, kind=N.LOSS_DRPO, lengths=lengths, drpo_epsilon=5.0)
        _, metrics = plan.forward(False)
        kl, _ = ops.gaussian_kl_mask(p, q, sig, 0.01)
        _, lp, _ = ops.sde_step_logp(v, x, s10, s11, kind="flow", eta=0.7, noise=n, sigma_max=smax)
        return metrics, kl, lp

    a, b = make(0.05), make(0.2)
    alone_a, alone_b = run(a), run(b)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for rep in range(10):
        with torch.cuda.stream(s1):
            got_a = run(a)
        with torch.cuda.stream(s2):
            got_b = run(b)
        torch.cuda.synchronize()
        for got, want in ((got_a, alone_a), (got_b, alone_b)):
            for u, w in zip(got, want):
                assert torch.equal(u.view(torch.uint8), w.view(torch.uint8)), f"overlapping call {rep} differs"


def test_graph_replays_of_the_batched_replay_and_the_fused_head(dev):
    """The batched SDE replay, the fused lm_head kernel (register-staged below 512 rows, loads straight
    into LDS from 512) and the transposition under capture: several replays with fresh inputs and
    eager calls in between, each bit-identical to the eager result."""
    from unirl_amd import ops, sde

    g = torch.Generator(device=dev).manual_seed(6)
    stack = torch.randn(3, 5, 4, 24, 24, device=dev, generator=g).bfloat16()
    vel = torch.randn(3, 2, 4, 24, 24, device=dev, generator=g).bfloat16()
    slot_x, slot_p = sde.replay_slots([0, 1, 2, 3, 4], [1, 3])
    sg = torch.stack([SIG[1], SIG[3]]).to(dev)
    sn = torch.stack([SIG[2], SIG[4]]).to(dev)
    smax = SIG[1].to(dev)
    w = (0.1 * torch.randn(700, 192, device=dev, generator=g)).bfloat16()
    h_small = torch.randn(300, 192, device=dev, generator=g).bfloat16()
    h_big = torch.randn(600, 192, device=dev, generator=g).bfloat16()
    ids_small = torch.randint(0, 700, (300,), device=dev, generator=g)
    ids_big = torch.randint(0, 700, (600,), device=dev, generator=g)

    def run_all():
        lp, means = ops.sde_replay_logp(vel, stack, slot_x, slot_p, sg, sn, kind="flow", eta=0.7, sigma_max=smax)
        a = ops.lmhead_logp(h_small, w, None, ids_small, 0.9, want_entropy=True, want_lse=True)[:3]
        b = ops.lmhead_logp(h_big, w, None, ids_big, 0.9, want_entropy=True, want_lse=True)[:3]
        wt = ops.transpose_2d(w)
        return (lp, means) + tuple(a) + tuple(b) + (wt,)

    run_all()  # scratch buffers of the head are torch allocations: let the caching allocator have them
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        outs = run_all()
    torch.cuda.synchronize()
    for rep in range(4):
        for t in (stack, vel, w, h_small, h_big):
            t.copy_((torch.randn(t.shape, device=dev, generator=g) * (0.1 if t is w else 1.0)).bfloat16())
        ops.lmhead_logp(h_small[:64], w, None, ids_small[:64], 1.0)  # eager work of the library between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = run_all()
        torch.cuda.synchronize()
        for k, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"replay {rep}, output {k} differs from eager"
