#!/usr/bin/env python3
"""Benchmark of the fused RL-math kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  The headline (`value`) is the fused token log-prob + entropy
kernel on bf16 logits [8192, 151936] -- the second configuration of BASELINE.json, the
one large enough to be cleanly HBM-bound -- as algorithmic GB/s over exactly K timed
steps with the inputs resident in HBM.  `roofline` prices that kernel against the
8 TB/s HBM peak from HIP-event timing of the same launches; `shapes` carries the same
figures for all five synthetic shapes (small ones timed as back-to-back launches inside
a HIP graph over rotating buffer sets, so neither the launch path nor the 256 MB
last-level cache hides the kernel time); `cpu_baseline` is the eager-torch CPU oracle of
the headline path on a bounded row sample, timed on this host's cores.

Three probe modes print their own JSON line and exit: `--traffic-probe` (three launches of every
kernel after three calibration copies, the command the hardware byte counters are collected on),
`--replay-probe` (the kernel's caller in training, the chunked lm_head + log-prob replay,
forward + backward, against the reference's torch ops under checkpoint) and `--timeline` (where
the time of a small shape goes inside the 64-launch graph: launch gaps and kernel bodies from
clock readings the kernels of the measurement build take themselves; needs
`python -m unirl_amd.build --tune`).
"""

from __future__ import annotations

import argparse
import json
import math
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak
L2_PLUS_MALL_BYTES = 256 * 2**20 + 32 * 2**20


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


# ----------------------------------------------------------------------------------------------
# timing helpers
# ----------------------------------------------------------------------------------------------
def time_steps(torch, fn, steps: int, warmup: int):
    """(wall ms per step, HIP-event ms per step) over exactly `steps` calls of fn(i)."""
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, start.elapsed_time(stop) / steps


def time_in_graph(torch, fn, n_sets: int, launches: int = 64, replays: int = 7):
    """Median per-launch microseconds of `launches` back-to-back calls captured in a HIP graph."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(n_sets):  # warm up on the capture stream (workspace, code objects)
            fn(i)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for i in range(launches):
            fn(i % n_sets)
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    times = []
    for _ in range(replays):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        graph.replay()
        stop.record()
        torch.cuda.synchronize()
        times.append(start.elapsed_time(stop) * 1e3 / launches)
    del graph
    return statistics.median(times)


def time_cpu(fn, reps: int = 5, warmup: int = 2):
    for _ in range(warmup):
        fn()
    out = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        out.append(time.perf_counter() - t0)
    return statistics.median(out) * 1e3


def wrapper_latency_us(torch, fn, reps: int = 20):
    """End-to-end call + synchronise, microseconds (median)."""
    out = []
    for i in range(reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn(i)
        torch.cuda.synchronize()
        out.append((time.perf_counter() - t0) * 1e6)
    return statistics.median(out)


def host_issue_us(torch, fn, reps: int = 300):
    """Python time per call when nothing waits for the device: `reps` calls issued back to back (the
    device queue is far deeper), microseconds per call.  This is what the wrapper itself costs."""
    best = float("inf")
    for _ in range(3):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(reps):
            fn(i)
        t1 = time.perf_counter()
        torch.cuda.synchronize()
        best = min(best, (t1 - t0) * 1e6 / reps)
    return best


# ----------------------------------------------------------------------------------------------
# the five synthetic shapes of BASELINE.json
# ----------------------------------------------------------------------------------------------
def n_sets_for(bytes_per_set: int) -> int:
    """Enough rotating input sets that consecutive launches cannot be served from cache."""
    return max(2, min(16, math.ceil(1.5 * L2_PLUS_MALL_BYTES / max(1, bytes_per_set))))


def make_shapes(torch, dev):
    """The synthetic shapes.  Every input the GPU sees comes from the package's own functions; the
    oracle is imported only inside the `cpu` callables (the CPU baseline of each shape)."""
    from unirl_amd import _native as N
    from unirl_amd import ops
    from unirl_amd.sde.runtime import get_sigma_schedule
    from unirl_amd.types import compute_advantages

    def oracle(name):
        import importlib

        return importlib.import_module(f"oracle.{name}")

    def pack_padded(x, lengths):
        return torch.cat([x[r, : int(lengths[r])] for r in range(x.shape[0])], dim=0)

    sig = get_sigma_schedule(28, 3.0)
    sig_d = sig.to(dev)
    shapes = []

    # -- config 1: SDE step + log-prob, SD3 latents fp32 [8,16,128,128], step 10 of 28 ------------
    g = torch.Generator().manual_seed(1001)
    shp = (8, 16, 128, 128)
    host1 = [torch.randn(shp, generator=g) for _ in range(3)]  # x, v, noise
    numel = host1[0].numel()
    bytes1 = 5 * numel * 4
    ns = n_sets_for(bytes1)
    sets1 = [[t.to(dev) + 0.0 * k for t in host1] for k in range(ns)]
    s10, s11, smax = sig_d[10], sig_d[11], sig_d[1]

    def run1(i):
        x, v, n = sets1[i % ns]
        return ops.sde_step_logp(v, x, s10, s11, kind="flow", eta=0.7, noise=n, sigma_max=smax)

    shapes.append(dict(
        name="sde_step_logp", config=1, shape="fp32 [8,16,128,128], step 10/28, shift 3, eta 0.7, sampling",
        bytes=bytes1, read_bytes=3 * numel * 4, write_bytes=2 * numel * 4, elements=numel, run=run1, sets=ns,
        cpu=lambda: oracle("sde").sde_denoise("flow", host1[1], host1[0], sig[10], sig[11], eta=0.7, noise=host1[2],
                                              sigma_max=sig[1]),
        cpu_bytes=bytes1,
    ))

    # the same sampling step with the noise drawn inside the kernel (Philox + Box-Muller in registers):
    # 2 reads + 2 writes, no noise tensor written by torch.randn and read back
    bytes1g = 4 * numel * 4

    def run1g(i):
        x, v, _ = sets1[i % ns]
        return ops.sde_step_logp(v, x, s10, s11, kind="flow", eta=0.7, sigma_max=smax, rng=(1001, 4 * i))

    shapes.append(dict(
        name="sde_step_logp_sample_rng", config=1,
        shape="fp32 [8,16,128,128], step 10/28, sampling, noise drawn in the kernel (2 reads, 2 writes)",
        bytes=bytes1g, read_bytes=2 * numel * 4, write_bytes=2 * numel * 4, elements=numel, run=run1g, sets=ns,
    ))

    # what that replaces: the noise drawn by torch.randn into a tensor (one more launch, one more write),
    # then the 3-read step -- the sampling step of a rollout as denoise() ran it before
    noise_buf = [torch.empty(shp, device=dev) for _ in range(ns)]

    def run1n(i):
        x, v, _ = sets1[i % ns]
        n = noise_buf[i % ns].normal_()
        return ops.sde_step_logp(v, x, s10, s11, kind="flow", eta=0.7, noise=n, sigma_max=smax)

    shapes.append(dict(
        name="sde_step_logp_sample_randn", config=1,
        shape="fp32 [8,16,128,128], step 10/28, sampling: torch's normal_() into a noise tensor, then the step "
              "(GB/s on the drawing kernel's 2 reads + 2 writes)",
        bytes=bytes1g, read_bytes=3 * numel * 4, write_bytes=3 * numel * 4, elements=numel, run=run1n, sets=ns,
    ))

    # the same step in replay mode: the stored next latent is given, mean and log-prob come back
    prev_dev = run1(0)[0]
    prev_host = prev_dev.cpu()
    prev1 = [prev_dev + 0.0 * k for k in range(ns)]
    bytes1r = 4 * numel * 4  # reads noise_pred, sample, prev_sample; writes the mean

    def run1r(i):
        x, v, _ = sets1[i % ns]
        return ops.sde_step_logp(v, x, s10, s11, kind="flow", eta=0.7, prev_sample=prev1[i % ns], sigma_max=smax,
                                 want_prev=False)

    shapes.append(dict(
        name="sde_step_logp_replay", config=1,
        shape="fp32 [8,16,128,128], step 10/28, replay of a stored transition (3 reads, 1 write)",
        bytes=bytes1r, read_bytes=3 * numel * 4, write_bytes=numel * 4, elements=numel, run=run1r, sets=ns,
        cpu=lambda: oracle("sde").sde_denoise("flow", host1[1], host1[0], sig[10], sig[11], eta=0.7,
                                              prev_sample=prev_host, sigma_max=sig[1]),
        cpu_bytes=bytes1r,
    ))

    # the replay of S' recorded steps of a whole micro-batch as one launch (what the [B,S'] losses
    # consume), against the same work as one call per step: SD3 recipe (bf16 trajectory of 10 steps,
    # 3 trained steps, micro-batch 8) and WAN recipe (fp16 trajectory of 14 steps, 7 trained, batch 2)
    from unirl_amd import sde as psde

    strat = psde.FlowSDEStrategy()
    for tag, B, tail, n_steps, shift, steps, tdt in (
            ("sd3", 8, (16, 128, 128), 10, 3.0, [0, 2, 4], torch.bfloat16),
            ("wan", 2, (16, 21, 60, 104), 14, 5.0, list(range(7)), torch.float16)):
        g = torch.Generator().manual_seed(1011)
        sg = get_sigma_schedule(n_steps, shift)
        K, S = n_steps + 1, len(steps)
        D = math.prod(tail)
        bytes_r = B * S * D * 2 * 4  # velocity, start latent, stored next latent read; mean written (16-bit each)
        nsr = n_sets_for(bytes_r)
        stacks = [torch.randn((B, K) + tail, generator=g).to(tdt).to(dev) for _ in range(min(nsr, 4))]
        vels = [torch.randn((B, S) + tail, generator=g).bfloat16().to(dev) for _ in range(min(nsr, 4))]
        nsr = len(stacks)
        slot_x, slot_p = psde.replay_slots(list(range(K)), steps)
        sg_a = torch.stack([sg[i] for i in steps]).to(dev)
        sg_b = torch.stack([sg[i + 1] for i in steps]).to(dev)
        smax_r = sg[1].to(dev)
        sg_d = sg.to(dev)

        def run_replay(i, stacks=stacks, vels=vels, nsr=nsr, slot_x=slot_x, slot_p=slot_p, sg_a=sg_a, sg_b=sg_b,
                       smax_r=smax_r):
            return strat.replay_steps(vels[i % nsr], stacks[i % nsr], slot_x, slot_p, sg_a, sg_b, eta=0.7,
                                      sigma_max=smax_r)

        out_lp = torch.empty(B, S, device=dev)
        out_mean = torch.empty((B, S) + tail, dtype=tdt, device=dev)

        def run_loop(i, stacks=stacks, vels=vels, nsr=nsr, steps=steps, slot_x=slot_x, slot_p=slot_p, sg_d=sg_d,
                     smax_r=smax_r, out_lp=out_lp, out_mean=out_mean):
            st_, v_ = stacks[i % nsr], vels[i % nsr]
            for j, k in enumerate(steps):
                strat.denoise_into(v_[:, j], st_[:, slot_x[j]], sg_d[k], sg_d[k + 1], eta=0.7, prev_sample=st_[:, slot_p[j]],
                                   sigma_max=smax_r, mean_out=out_mean[:, j], logp_out=out_lp[:, j])

        # the Flow-DPPO micro-step's forward on the same transitions: replay log-probs + KL against the frozen
        # means + masks, loss, metrics, gradient -- fused (one streaming pass over 4 reads + one finishing
        # workgroup) against the pair it replaces (batched replay writing the means, then the KL / loss step)
        old_means = [torch.randn((B, S) + tail, generator=g).to(tdt).to(dev) for _ in range(nsr)]
        old_lp = torch.randn(B, S, generator=g).to(dev)
        adv_bs = torch.randn(B, 1, generator=g).expand(B, S).contiguous().to(dev)
        sig_t = torch.full((S,), 0.1, device=dev)

        def run_dppo_fused(i, stacks=stacks, vels=vels, nsr=nsr, slot_x=slot_x, slot_p=slot_p, sg_a=sg_a, sg_b=sg_b,
                           smax_r=smax_r, old_means=old_means, old_lp=old_lp, adv_bs=adv_bs, sig_t=sig_t):
            return ops.flowdppo_replay_step(vels[i % nsr], stacks[i % nsr], slot_x, slot_p, sg_a, sg_b, old_lp,
                                            old_means[i % nsr], adv_bs, sig_t, 1.0, kind="flow", eta=0.7,
                                            sigma_max=smax_r, loss_scale=1.0)

        def run_dppo_pair(i, stacks=stacks, vels=vels, nsr=nsr, slot_x=slot_x, slot_p=slot_p, sg_a=sg_a, sg_b=sg_b,
                          smax_r=smax_r, old_means=old_means, old_lp=old_lp, adv_bs=adv_bs, sig_t=sig_t):
            lp, means = ops.sde_replay_logp(vels[i % nsr], stacks[i % nsr], slot_x, slot_p, sg_a, sg_b, kind="flow",
                                            eta=0.7, sigma_max=smax_r)
            return ops.flowdppo_step(lp, old_lp, means, old_means[i % nsr], adv_bs, sig_t, 1.0, loss_scale=1.0)

        shape_txt = f"{str(tdt).split('.')[-1]} stack [{B},{K},{','.join(map(str, tail))}], bf16 velocities, S'={S} steps"
        shapes.append(dict(
            name=f"sde_replay_BxS_{tag}", config=1, shape=shape_txt + ": one launch over the B*S' transitions",
            bytes=bytes_r, read_bytes=bytes_r * 3 // 4, write_bytes=bytes_r // 4, elements=B * S * D, run=run_replay,
            sets=nsr,
        ))
        shapes.append(dict(
            name=f"sde_replay_per_step_{tag}", config=1, shape=shape_txt + ": one call per step (S' launch pairs)",
            bytes=bytes_r, read_bytes=bytes_r * 3 // 4, write_bytes=bytes_r // 4, elements=B * S * D, run=run_loop,
            sets=nsr,
        ))
        shapes.append(dict(
            name=f"flowdppo_replay_step_{tag}", config=4,
            shape=shape_txt + " + frozen means [B,S',...]: replay log-prob + KL + loss + metrics + grad, 4 reads, 2 launches",
            bytes=bytes_r, read_bytes=bytes_r, write_bytes=0, elements=B * S * D, run=run_dppo_fused, sets=nsr,
        ))
        shapes.append(dict(
            name=f"flowdppo_replay_pair_{tag}", config=4,
            shape=shape_txt + " + frozen means: the same job as sde_replay_logp (means written) then flowdppo_step "
                              "(means re-read): 5 reads + 1 write, 4 launches; GB/s on the fused job's 4 reads",
            bytes=bytes_r, read_bytes=bytes_r * 5 // 4, write_bytes=bytes_r // 4, elements=B * S * D, run=run_dppo_pair,
            sets=nsr,
        ))

    # -- config 3: GRPO / DRPO token loss, fp32 [256, 8192], lengths U[512, 8192] -----------------
    g = torch.Generator().manual_seed(1003)
    old = -8 * torch.rand(256, 8192, generator=g)
    new = old + 0.05 * torch.randn(256, 8192, generator=g)
    lengths = torch.randint(512, 8193, (256,), generator=g)
    rewards = (torch.rand(256, generator=g) < 0.5).float()
    adv = compute_advantages(rewards.to(dev), [i // 16 for i in range(256)]).cpu()
    n_valid = int(lengths.sum())
    bytes3_padded = 2 * new.numel() * 4
    bytes3_valid = 2 * n_valid * 4
    ns3 = n_sets_for(bytes3_padded)
    sets3 = [(new.to(dev) + 0.0 * k, old.to(dev) + 0.0 * k) for k in range(ns3)]
    len_d, adv_d = lengths.to(dev), adv.to(dev)
    plans = {}
    for kind, code, kw in (("grpo", N.LOSS_GRPO, dict(clip_low=0.2, clip_high=0.28)),
                           ("drpo", N.LOSS_DRPO, dict(drpo_epsilon=5.0))):
        plans[kind] = [ops.RatioLossPlan(a, b, adv_d, kind=code, lengths=len_d, **kw) for a, b in sets3]
    newp, oldp = pack_padded(new, lengths), pack_padded(old, lengths)
    for kind, okw in (("grpo", dict(clip_range=0.2, clip_range_high=0.28)), ("drpo", dict(epsilon=5.0))):
        shapes.append(dict(
            name=f"ratio_loss_{kind}", config=3,
            shape=f"fp32 [256,8192] padded, {n_valid} valid tokens, 16x16 groups, token-mean",
            bytes=bytes3_valid, bytes_padded=bytes3_padded, read_bytes=bytes3_valid, write_bytes=0,
            elements=n_valid,
            run=(lambda i, k=kind: plans[k][i % ns3].forward(False)), sets=ns3,
            cpu=(lambda k=kind, o=okw: oracle("losses").token_loss(k, newp, oldp, adv, lengths, **o)),
            cpu_bytes=bytes3_valid,
        ))
    # the whole training micro-step: loss, metrics and the gradient w.r.t. new_logp in one pass
    # (the gradient tensor has the padded shape; the padding is written as zeros)
    bytes3_step = bytes3_valid + new.numel() * 4

    def cpu_step(k, o):
        leaf = newp.clone().requires_grad_(True)
        oracle("losses").token_loss(k, leaf, oldp, adv, lengths, **o)[0].backward()

    for kind, okw in (("grpo", dict(clip_range=0.2, clip_range_high=0.28)), ("drpo", dict(epsilon=5.0))):
        shapes.append(dict(
            name=f"ratio_step_{kind}", config=3,
            shape=f"fp32 [256,8192] padded, {n_valid} valid tokens: loss + metrics + grad_new in one pass",
            bytes=bytes3_step, read_bytes=bytes3_valid, write_bytes=new.numel() * 4, elements=n_valid,
            run=(lambda i, k=kind: plans[k][i % ns3].forward_backward(1.0)), sets=ns3,
            cpu=(lambda k=kind, o=okw: cpu_step(k, o)), cpu_bytes=bytes3_step, plain_reduction=True,
        ))

    # the same tokens in the packed layout the AR algorithms use ([total_tokens] + cu_seqlens)
    cu3 = torch.cat([torch.zeros(1, dtype=torch.int64), lengths.cumsum(0)]).to(dev)
    ns3p = n_sets_for(3 * n_valid * 4)
    sets3p = [(newp.to(dev) + 0.0 * k, oldp.to(dev) + 0.0 * k) for k in range(ns3p)]
    pplans = {}
    for kind, code, kw in (("grpo", N.LOSS_GRPO, dict(clip_low=0.2, clip_high=0.28)),
                           ("drpo", N.LOSS_DRPO, dict(drpo_epsilon=5.0))):
        pplans[kind] = [ops.RatioLossPlan(a, b, adv_d, kind=code, cu_seqlens=cu3, **kw) for a, b in sets3p]
    for kind in ("grpo", "drpo"):
        shapes.append(dict(
            name=f"ratio_step_{kind}_packed", config=3,
            shape=f"fp32 packed [{n_valid}] + cu_seqlens[257]: loss + metrics + grad_new in one pass",
            bytes=3 * n_valid * 4, read_bytes=bytes3_valid, write_bytes=n_valid * 4, elements=n_valid,
            run=(lambda i, k=kind: pplans[k][i % ns3p].forward_backward(1.0)), sets=ns3p, plain_reduction=True,
        ))

    # -- config 4: Flow-DPPO KL mask, WAN bf16 [2,16,21,60,104] -----------------------------------
    g = torch.Generator().manual_seed(1004)
    shp4 = (2, 1, 16, 21, 60, 104)
    base = torch.randn(shp4, generator=g)
    old_m = (base + 0.01 * torch.randn(shp4, generator=g)).bfloat16()
    new_m = (base + 0.01 * torch.randn(shp4, generator=g)).bfloat16()
    step = int((sig - 0.5).abs().argmin())
    sig_t = torch.tensor(0.7 * math.sqrt(float(sig[step] - sig[step + 1])))
    bytes4 = 2 * old_m.numel() * 2
    ns4 = n_sets_for(bytes4)
    sets4 = [(new_m.to(dev).clone(), old_m.to(dev).clone()) for _ in range(ns4)]
    sig_t_d = sig_t.to(dev)

    def run4(i):
        p, q = sets4[i % ns4]
        return ops.gaussian_kl_mask(p, q, sig_t_d, 0.01)

    shapes.append(dict(
        name="gaussian_kl_mask", config=4, shape="bf16 [2,16,21,60,104] old/new means, threshold 0.01",
        bytes=bytes4, read_bytes=bytes4, write_bytes=0, elements=old_m.numel(), run=run4, sets=ns4,
        cpu=lambda: oracle("flowdppo").kl_per_sample(new_m, old_m, sig_t.reshape(1, 1, 1, 1, 1, 1)) < 0.01,
        cpu_bytes=bytes4,
    ))

    # the loss step of Flow-DPPO around that kernel: KL, masks, loss, metrics and the gradient
    new_lp = 1e-3 * torch.randn(2, 1, generator=g)
    old_lp = new_lp + 2e-4 * torch.randn(2, 1, generator=g)
    adv4 = torch.tensor([[1.0], [-1.0]])
    lp_d = (new_lp.to(dev), old_lp.to(dev), adv4.to(dev))

    def run4s(i):
        p, q = sets4[i % ns4]
        return ops.flowdppo_step(lp_d[0], lp_d[1], p, q, lp_d[2], sig_t_d, 0.01, loss_scale=1.0)

    def cpu4s():
        leaf = new_lp.clone().requires_grad_(True)
        oracle("flowdppo").flowdppo_loss(leaf, old_lp, new_m, old_m, adv4, sig_t.reshape(1, 1, 1, 1, 1, 1),
                                         0.01)[0].mean().backward()

    shapes.append(dict(
        name="flowdppo_step", config=4,
        shape="bf16 [2,1,16,21,60,104] means + [2,1] log-probs: KL, masks, loss, 12 metrics, grad_new",
        bytes=bytes4, read_bytes=bytes4, write_bytes=0, elements=old_m.numel(), run=run4s, sets=ns4,
        cpu=cpu4s, cpu_bytes=bytes4,
    ))

    # -- config 5: 10-step rollout, Qwen-Image packed latents fp32 [16,4096,64] -------------------
    g = torch.Generator().manual_seed(1005)
    shp5 = (16, 4096, 64)
    x0 = torch.randn(shp5, generator=g)
    vs = [torch.randn(shp5, generator=g) for _ in range(10)]
    nz = [torch.randn(shp5, generator=g) for _ in range(10)]
    bytes5 = 22 * x0.numel() * 4
    x0_d, vs_d, nz_d = x0.to(dev), [t.to(dev) for t in vs], [t.to(dev) for t in nz]

    def run5(i):
        return ops.sde_rollout_logp(x0_d, vs_d, nz_d, sig_d, 0.7, kind="flow")

    shapes.append(dict(
        name="sde_rollout_logp", config=5, shape="fp32 [16,4096,64], 10 steps from step 0, eta 0.7",
        bytes=bytes5, read_bytes=21 * x0.numel() * 4, write_bytes=x0.numel() * 4, elements=10 * x0.numel(),
        run=run5, sets=1,
        cpu=lambda: oracle("sde").sde_rollout("flow", x0, vs, nz, sig, 0.7), cpu_bytes=bytes5, cpu_reps=3,
    ))
    return shapes


def make_floor(torch, dev, read_bytes: int, write_bytes: int, n_sets: int, tail_launch: bool):
    """The launch floor of a shape: a kernel that only moves the shape's bytes (same read / write
    split, rotating buffers), plus the minimal dependent second launch of a two-launch reduction."""
    from unirl_amd import _tune

    rb, wb = (read_bytes + 15) // 16 * 16, (write_bytes + 15) // 16 * 16
    srcs = [torch.ones(max(rb, 16), dtype=torch.uint8, device=dev) for _ in range(n_sets)]
    dsts = [torch.empty(max(wb, 16), dtype=torch.uint8, device=dev) for _ in range(n_sets)]
    sink = torch.zeros(4, dtype=torch.int32, device=dev)

    def run(i):
        _tune.calib_stream(srcs[i % n_sets], rb, dsts[i % n_sets], wb, sink, tail_launch=tail_launch)

    return run


def kernel_source_sha256() -> str:
    """Hash of the token kernel's source text (the kernel file and the helpers it includes)."""
    import hashlib

    h = hashlib.sha256()
    for name in ("token_logp.hip", "common_hip.h"):
        h.update((ROOT / "unirl_amd" / "csrc" / name).read_bytes())
    return h.hexdigest()


def make_headline(torch, dev, rows: int, vocab: int):
    """Config 2: logits bf16 [rows, vocab] ~ N(0, 2) with 1% of the rows holding one +15 spike."""
    g = torch.Generator(device=dev).manual_seed(1002)
    x = torch.empty(rows, vocab, dtype=torch.bfloat16, device=dev)
    for s in range(0, rows, 512):
        n = min(512, rows - s)
        x[s : s + n] = (2 * torch.randn(n, vocab, generator=g, device=dev)).bfloat16()
    n_spike = max(1, rows // 100)
    spiked = torch.randperm(rows, generator=g, device=dev)[:n_spike]
    x[spiked, torch.randint(0, vocab, (n_spike,), generator=g, device=dev)] = 15.0
    ids = torch.randint(0, vocab, (rows,), generator=g, device=dev)
    return x, ids, spiked


def replay_probe(torch, dev, rows: int, vocab: int, hidden: int = 2560):
    """The caller of the headline kernel in training: `lm_head` on a chunk of response tokens, their
    log-probs, and the backward with the chunk's logits rebuilt (unirl/models/qwen3/ar.py:82-99).
    One sequence of `rows` tokens, a bf16 head of Qwen3-4B's size; the fused path against the
    reference's own ops (`.float() / T`, gather, logsumexp under torch's checkpoint)."""
    from torch.utils.checkpoint import checkpoint

    from unirl_amd import models

    torch.manual_seed(0)
    head = torch.nn.Linear(hidden, vocab, bias=False).to(dev).to(torch.bfloat16)
    hidden_states = torch.randn(1, rows, hidden, device=dev, dtype=torch.bfloat16)
    tokens = torch.randint(0, vocab, (1, rows), device=dev)
    upstream = torch.randn(1, rows, device=dev)

    def reference(h_all):
        def logp_chunk(h, tok):
            lf = head(h).float() / 1.0
            return lf.gather(-1, tok.unsqueeze(-1)).squeeze(-1) - torch.logsumexp(lf, dim=-1)

        chunk = max(64, 2048 // int(h_all.shape[0]))
        parts = [checkpoint(logp_chunk, h_all[:, s : s + chunk], tokens[:, s : s + chunk], use_reentrant=False)
                 for s in range(0, rows, chunk)]
        return torch.cat(parts, dim=1)

    def timed(fn):
        for _ in range(3):  # the last of three passes is reported
            head.zero_grad(set_to_none=True)
            h = hidden_states.clone().requires_grad_(True)
            torch.cuda.synchronize()
            torch.cuda.reset_peak_memory_stats()
            base = torch.cuda.memory_allocated()
            a, b, c = (torch.cuda.Event(enable_timing=True) for _ in range(3))
            a.record()
            out = fn(h)
            b.record()
            (out * upstream).sum().backward()
            c.record()
            torch.cuda.synchronize()
        stats = {"forward_ms": round(a.elapsed_time(b), 2), "backward_ms": round(b.elapsed_time(c), 2),
                 "total_ms": round(a.elapsed_time(c), 2),
                 "peak_transient_gib": round((torch.cuda.max_memory_allocated() - base) / 2**30, 3)}
        return stats, out.detach(), h.grad.detach().float(), head.weight.grad.detach().float()

    out = {"rows": rows, "vocab": vocab, "hidden": hidden}
    ref = timed(reference)
    out["reference_torch_checkpoint_chunk2048"] = ref[0]
    for name, kw in (("fused_recompute_chunk2048", dict(chunk=2048, keep_logits=False, transposed_head=False, fused_head=False)),
                     ("fused_recompute_chunk4096", dict(keep_logits=False, transposed_head=False, fused_head=False)),
                     ("fused_keep_logits", dict(transposed_head=False)), ("fused_default", dict()),
                     ("fused_head_chunk4096", dict(keep_logits=False, transposed_head=False)),
                     ("fused_head_chunk2048_transposed", dict(keep_logits=False, chunk=2048)),
                     ("fused_head_chunk1024_transposed", dict(keep_logits=False, chunk=1024)),
                     ("fused_head_chunk512_transposed", dict(keep_logits=False, chunk=512)),
                     ("fused_recompute_chunk2048_transposed", dict(chunk=2048, keep_logits=False, fused_head=False))):
        got = timed(lambda h: models.chunked_replay_logp(head, h, tokens, 1.0, **kw))
        got[0]["max_abs_logp_diff"] = float((got[1] - ref[1]).abs().max())
        got[0]["grad_hidden_rel"] = float((got[2] - ref[2]).norm() / ref[2].norm())
        got[0]["grad_weight_rel"] = float((got[3] - ref[3]).norm() / ref[3].norm())
        out[name] = got[0]
        log(f"replay {name}: {got[0]}")
    log(f"replay reference: {ref[0]}")
    # what the default's transposed copy of the weight costs, once per replay (inside the times above)
    from unirl_amd.models import ar_logp

    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    ar_logp.transpose_weight(head.weight)
    b.record()
    torch.cuda.synchronize()
    out["weight_transposition_ms"] = round(a.elapsed_time(b), 2)
    log(f"replay: transposing the weight once takes {out['weight_transposition_ms']} ms")
    return out


MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published peak


def head_probe(torch, dev, vocab: int, hidden: int = 2560, row_counts=(64, 256, 1024, 2048, 8192)):
    """The fused lm_head + log-softmax kernel (`unirl_lmhead_logp`: the [rows, V] logits are never
    written) against the library GEMM followed by the token kernel, forward only, for a bf16 head of
    Qwen3-4B's size.  TFLOP/s count the GEMM's 2*rows*K*V flops over the whole call."""
    from unirl_amd import ops

    g = torch.Generator(device=dev).manual_seed(0)
    w = (torch.randn(vocab, hidden, generator=g, device=dev) * (3.0 / math.sqrt(hidden))).bfloat16()

    def timed(fn, n=10):
        # a quarter of a second of the same calls first: the clocks of an idle device ramp over the
        # first few hundred milliseconds of work (a 1.5 ms call measured cold reads 20 % slow)
        t_end = time.perf_counter() + 0.25
        while time.perf_counter() < t_end:
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n

    out = []
    for rows in row_counts:
        h = torch.randn(rows, hidden, generator=g, device=dev).bfloat16()
        ids = torch.randint(0, vocab, (rows,), generator=g, device=dev)
        flop = 2.0 * rows * hidden * vocab

        def unfused():
            logits = torch.nn.functional.linear(h, w)
            return ops.token_logp_entropy(logits, ids, 1.0, want_lse=True)

        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        t_f = timed(lambda: ops.lmhead_logp(h, w, None, ids, 1.0, want_entropy=True, want_lse=True))
        mem_f = torch.cuda.max_memory_allocated() - base
        torch.cuda.reset_peak_memory_stats()
        t_u = timed(unfused)
        mem_u = torch.cuda.max_memory_allocated() - base
        t_g = timed(lambda: torch.nn.functional.linear(h, w))
        lp_f = ops.lmhead_logp(h, w, None, ids, 1.0)[0]
        lp_u = unfused()[0]
        row = {
            "rows": rows, "vocab": vocab, "hidden": hidden,
            "fused_ms": round(t_f, 3), "fused_tflops": round(flop / t_f / 1e9, 0),
            "fused_frac_of_mfma_peak": round(flop / t_f / 1e9 / MFMA_BF16_PEAK_TFLOPS, 3),
            "library_gemm_plus_token_kernel_ms": round(t_u, 3), "library_gemm_alone_ms": round(t_g, 3),
            "library_gemm_tflops": round(flop / t_g / 1e9, 0),
            "fused_transient_mib": round(mem_f / 2**20, 1), "unfused_transient_mib": round(mem_u / 2**20, 1),
            "logp_rows_differing_beyond_2e-3": int(((lp_f - lp_u).abs() > 2e-3 * lp_u.abs() + 2e-3).sum()),
        }
        log(f"head probe: {row}")
        out.append(row)
    return out


def head_counters_probe(torch, dev, vocab: int, rows: int = 8192, hidden: int = 2560, calls: int = 6):
    """The command the matrix-core counters are collected on (`rocprofv3 --pmc ... -- python3 bench.py
    --head-counters-probe`): after a spin-up that brings the device to its sustained clocks, `calls`
    back-to-back calls of the fused lm_head kernel, then `calls` of the library GEMM on the same
    operands (`linear(h, w)`: the kernel the fused one is measured against).  Cycle counters of the two
    kernels divided by their durations give the shader clock each one ran at."""
    from unirl_amd import ops

    g = torch.Generator(device=dev).manual_seed(0)
    w = (torch.randn(vocab, hidden, generator=g, device=dev) * (3.0 / math.sqrt(hidden))).bfloat16()
    h = torch.randn(rows, hidden, generator=g, device=dev).bfloat16()
    ids = torch.randint(0, vocab, (rows,), generator=g, device=dev)
    t_end = time.perf_counter() + 0.5
    while time.perf_counter() < t_end:
        ops.lmhead_logp(h, w, None, ids, 1.0, want_entropy=True, want_lse=True)
        torch.nn.functional.linear(h, w)
        torch.cuda.synchronize()
    for _ in range(calls):
        ops.lmhead_logp(h, w, None, ids, 1.0, want_entropy=True, want_lse=True)
    torch.cuda.synchronize()
    for _ in range(calls):
        torch.nn.functional.linear(h, w)
    torch.cuda.synchronize()
    return {"rows": rows, "vocab": vocab, "hidden": hidden, "calls_each": calls,
            "flop_per_call": 2.0 * rows * hidden * vocab}


def tail_probe(torch, dev):
    """What finishing a grid-wide reduction costs after its streaming part, at the byte counts of the
    three small reducing shapes: the streaming kernel alone, plus a dependent second launch (the
    library's scheme), and finished inside the one launch by a polling workgroup
    (`unirl_calib_reduce` modes 0 / 1 / 2), each as 64 back-to-back calls in a HIP graph over
    rotating inputs."""
    from unirl_amd import _tune

    pool = torch.ones(160 * 2**20, dtype=torch.float32, device=dev)  # 640 MiB: beyond L2 + last-level cache
    out = torch.zeros(1, dtype=torch.float64, device=dev)
    rows = []
    for label, nbytes in (("ratio loss, config 3 (valid tokens)", 8915200), ("gaussian KL, config 4", 16773120),
                          ("SDE step replay reads, config 1", 25165824)):
        n_sets = pool.numel() * 4 // nbytes
        views = [pool.view(torch.uint8)[k * nbytes : (k + 1) * nbytes] for k in range(n_sets)]
        for nwg in (256, 512):
            scratch = torch.zeros(16 + 16 * nwg, dtype=torch.uint8, device=dev)
            got = {}
            for mode in (1, 2):  # same sum both ways, also on a second call that meets the first one's tags
                for _ in range(2):
                    _tune.calib_reduce(views[0], nbytes, mode, nwg, scratch, out)
                torch.cuda.synchronize()
                got[mode] = float(out.item())
            row = {"shape": label, "bytes": nbytes, "workgroups": nwg, "results_agree": got[1] == got[2]}
            for mode, key in ((0, "stream_only_us"), (1, "two_launches_us"), (2, "one_launch_polled_us")):
                row[key] = round(time_in_graph(torch, lambda i, m=mode: _tune.calib_reduce(views[i % n_sets], nbytes, m, nwg,
                                                                                         scratch, out), n_sets), 2)
            log(f"tail probe: {row}")
            rows.append(row)
    empty = torch.zeros(4, dtype=torch.int32, device=dev)
    rows.append({"shape": "one-wavefront kernel with one store, alone",
                 "us": round(time_in_graph(torch, lambda i: _tune.calib_stream(None, 0, None, 0, empty, tail_launch=True), 2), 2)})
    return rows


def timeline_probe(torch, dev, names):
    """Device-side timeline of the small shapes inside the 64-launch graph the bench times them in.

    A kernel-trace profiler serialises the dispatches of a graph and so cannot show the gaps
    between them; here the kernels of the measurement build (`python -m unirl_amd.build --tune`)
    read the 100 MHz device clock at entry, after their streaming loop and at exit, every
    workgroup for itself, into a buffer.  Per launch: gap = first workgroup's start minus the
    previous launch's last end; body = last end minus first start.  The marks cost about 0.5 us
    per call, so the sum sits that much above the release library's time."""
    import ctypes

    from unirl_amd import _native as N
    from unirl_amd.build import TUNE_LIB_PATH

    if not TUNE_LIB_PATH.exists():
        raise SystemExit(f"bench.py --timeline needs {TUNE_LIB_PATH}: build it with `python -m unirl_amd.build --tune`")
    N.LIB_PATH = TUNE_LIB_PATH  # before the first call binds the library: every product call runs the traced kernels
    from unirl_amd import _tune

    lib = _tune.lib()
    tick_ns = 10.0
    buf = torch.zeros(8 * 2**20, dtype=torch.int64, device=dev)
    spin = torch.randn(64 * 2**20, device=dev)
    for _ in range(300):  # bring the clocks up
        spin.mul_(1.0001)
    torch.cuda.synchronize()
    out = {}
    med = lambda v: round(statistics.median(v) / 1e3, 2) if v else None
    for sh in make_shapes(torch, dev):
        if names and sh["name"] not in names:
            continue
        fn, n_sets = sh["run"], sh["sets"]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(n_sets):
                fn(i)
        torch.cuda.synchronize()
        lib.unirl_trace_begin(buf.data_ptr(), buf.numel() * 8)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for i in range(64):
                fn(i % n_sets)
        torch.cuda.synchronize()
        entries = []
        for i in range(lib.unirl_trace_count()):
            nb, off = ctypes.c_uint(), ctypes.c_size_t()
            name = lib.unirl_trace_entry(i, ctypes.byref(nb), ctypes.byref(off)).decode()
            entries.append((name, nb.value, off.value))
        lib.unirl_trace_begin(None, 0)
        per, events = {}, []
        for rep in range(6):
            buf.zero_()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            if rep == 0:
                continue
            events.append(e0.elapsed_time(e1) * 1e3 / 64)
            host = buf.cpu()
            prev_end = None
            for name, nb, off in entries:
                t = host[off : off + nb * 4].view(nb, 4)
                t = t[t[:, 3] > 0]
                if t.numel() == 0:
                    continue
                start, end = int(t[:, 0].min()), int(t[:, 3].max())
                d = per.setdefault(name, dict(gap=[], body=[], first_wg_done=[], stream_done=[], second_mark=[]))
                d["body"].append((end - start) * tick_ns)
                d["first_wg_done"].append((int(t[:, 3].min()) - start) * tick_ns)
                marks = t[:, 1][t[:, 1] > 0]
                if marks.numel():
                    d["stream_done"].append((int(marks.max()) - start) * tick_ns)
                marks2 = t[:, 2][t[:, 2] > 0]
                if marks2.numel():
                    d["second_mark"].append((int(marks2.max()) - start) * tick_ns)
                if prev_end is not None:
                    d["gap"].append((start - prev_end) * tick_ns)
                prev_end = end
        del graph
        row = {"us_per_call_hip_events": round(statistics.median(events), 2), "launches": {}}
        total = 0.0
        for name, d in per.items():
            row["launches"][name] = {
                "gap_before_us": med(d["gap"]), "body_us": med(d["body"]),
                "first_workgroup_done_at_us": med(d["first_wg_done"]),
                "last_workgroup_past_its_loop_at_us": med(d["stream_done"]),
                "second_mark_at_us": med(d["second_mark"]),
            }
            total += (med(d["gap"]) or 0.0) + (med(d["body"]) or 0.0)
        row["sum_of_gaps_and_bodies_us"] = round(total, 2)
        log(f"timeline {sh['name']}: {row}")
        out[sh["name"]] = row
    return out


# ----------------------------------------------------------------------------------------------
def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--rows", type=int, default=8192, help="token rows of the headline workload")
    ap.add_argument("--vocab", type=int, default=151936)
    ap.add_argument("--cpu-rows", type=int, default=2048, help="rows of the bounded CPU-baseline sample")
    ap.add_argument("--spinup", type=float, default=1.0, help="seconds of untimed launches before the warm-up")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="run 3 calibration copies of 1 GiB, 3 headline launches and 3 launches of every "
                         "other shape, then exit "
                         "(the command `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE` is pointed at)")
    ap.add_argument("--replay-probe", action="store_true",
                    help="forward + backward of the chunked lm_head + log-prob replay (bf16 Linear(2560, vocab), "
                         "--rows response tokens) through the fused kernels and through the reference's torch ops "
                         "under checkpoint, then exit (time, peak transient memory; a kernel trace of this command "
                         "shows the split between the head's GEMMs and the log-prob kernels)")
    ap.add_argument("--timeline", nargs="?", const="", default=None, metavar="SHAPES",
                    help="device-side timeline (launch gaps, kernel bodies) of the small shapes inside the 64-launch "
                         "graph, from the measurement build's own clock readings; optional comma-separated shape "
                         "names; needs `python -m unirl_amd.build --tune`")
    ap.add_argument("--head-counters-probe", action="store_true",
                    help="spin up, then 6 calls of the fused lm_head kernel and 6 of the library GEMM at 8192 rows: "
                         "the command the matrix-core cycle counters are collected on")
    ap.add_argument("--head-probe", action="store_true",
                    help="the fused lm_head + log-softmax kernel (logits never written) against the library GEMM + "
                         "token kernel for a bf16 Linear(2560, --vocab) head at 64 / 2048 / 8192 rows, then exit")
    ap.add_argument("--tail-probe", action="store_true",
                    help="cost of finishing a grid-wide reduction after its streaming part: nothing, a second "
                         "launch, or polled inside the one launch (unirl_calib_reduce), then exit")
    ap.add_argument("--skip-shapes", action="store_true", help="headline only")
    ap.add_argument("--skip-cpu", action="store_true", help="no CPU baselines")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path runs on ONE GPU (independent per-sample work, no cross-GPU exchange); "
              "run it with --gpus 1", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no HIP device visible", file=sys.stderr)
        return 1
    from unirl_amd import _native as N

    if not N.LIB_PATH.exists():
        from unirl_amd.build import build

        build(verbose=False)
    from oracle import token_logp as otok
    from unirl_amd import ops

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    log(f"device {torch.cuda.get_device_name(0)}, torch {torch.__version__}, host threads {torch.get_num_threads()}")

    if args.timeline is not None:
        names = [n for n in args.timeline.split(",") if n]
        print(json.dumps({"timeline": timeline_probe(torch, dev, names)}), flush=True)
        return 0

    if args.head_counters_probe:
        print(json.dumps({"head_counters_probe": head_counters_probe(torch, dev, args.vocab)}), flush=True)
        return 0

    if args.head_probe:
        print(json.dumps({"head_probe": head_probe(torch, dev, args.vocab)}), flush=True)
        return 0

    if args.tail_probe:
        print(json.dumps({"tail_probe": tail_probe(torch, dev)}), flush=True)
        return 0

    if args.replay_probe:
        print(json.dumps({"replay_probe": replay_probe(torch, dev, args.rows, args.vocab)}), flush=True)
        return 0

    # ---------------- headline: token log-prob + entropy ----------------
    x, ids, spiked = make_headline(torch, dev, args.rows, args.vocab)
    alg_bytes = x.numel() * 2 + ids.numel() * 8 + 2 * args.rows * 4

    def step(i):
        return ops.token_logp_entropy(x, ids, 1.0, want_logp=True, want_entropy=True)

    if args.traffic_probe:
        from unirl_amd import _tune  # the calibration copy is a kernel of the measurement build

        src = torch.empty(2**30, dtype=torch.uint8, device=dev).fill_(7)
        dst = torch.empty_like(src)
        for _ in range(3):
            _tune.calib_copy(src, dst)
        for i in range(3):
            step(i)
        torch.cuda.synchronize()
        probe = {"calib_copy_bytes_each_way": 2**30, "token_kernel_algorithmic_bytes": alg_bytes}
        if not args.skip_shapes:
            del src, dst
            for sh in make_shapes(torch, dev):  # three launches of every other kernel, on distinct input sets
                for i in range(3):
                    sh["run"](i)
                torch.cuda.synchronize()
                probe[sh["name"] + "_algorithmic_bytes"] = sh.get("bytes_padded", sh["bytes"])
            # the fused lm_head kernel at 8192 rows: operands once, the tile states written and read once
            hd_rows, hd_k = 8192, 2560
            hw = torch.randn(args.vocab, hd_k, device=dev).bfloat16()
            hh = torch.randn(hd_rows, hd_k, device=dev).bfloat16()
            hid = torch.randint(0, args.vocab, (hd_rows,), device=dev)
            for _ in range(3):
                ops.lmhead_logp(hh, hw, None, hid, 1.0, want_lse=True)
            torch.cuda.synchronize()
            n_tiles = (args.vocab + 255) // 256
            probe["lmhead_logp_8192_algorithmic_bytes"] = (hw.numel() + hh.numel()) * 2 + 2 * hd_rows * n_tiles * 16
        print(json.dumps({"traffic_probe": probe}), flush=True)
        return 0

    # Untimed spin-up: the device needs a few hundred milliseconds of work to reach its sustained
    # clocks (measured: 6.2 TB/s after 5 launches, 6.8 TB/s after 200).  Then W warm-up steps,
    # then exactly K timed steps.
    t_end = time.perf_counter() + args.spinup
    while time.perf_counter() < t_end:
        for i in range(20):
            step(i)
        torch.cuda.synchronize()
    wall_ms, event_ms = time_steps(torch, step, args.steps, args.warmup)
    value = alg_bytes / (wall_ms * 1e-3) / 1e9
    achieved = alg_bytes / (event_ms * 1e-3) / 1e9
    log(f"token_logp_entropy: {wall_ms:.4f} ms/step wall, {event_ms:.4f} ms/launch (events), "
        f"{achieved:.1f} GB/s = {achieved / HBM_PEAK_GBPS:.1%} of peak")

    # parity + CPU baseline on a bounded, spike-including row sample
    lp, ent, _ = step(0)
    sample = torch.cat([spiked[: min(8, spiked.numel())],
                        torch.arange(0, args.rows, max(1, args.rows // args.cpu_rows), device=dev)])[: args.cpu_rows]
    xs, ids_s = x[sample].cpu(), ids[sample].cpu()
    ref_lp, ref_ent = otok.token_logp_entropy_chunked(xs, ids_s, 1.0, chunk=512)
    parity = {
        "rows_checked": int(sample.numel()),
        "logp_max_rel": float(((lp[sample].cpu() - ref_lp).abs() / ref_lp.abs().clamp_min(1e-6)).max()),
        "entropy_max_rel": float(((ent[sample].cpu() - ref_ent).abs() / ref_ent.abs().clamp_min(1e-6)).max()),
    }
    cpu_baseline = None
    if not args.skip_cpu:
        def cpu_fn():
            for s in range(0, xs.shape[0], 512):
                blk, idb = xs[s : s + 512], ids_s[s : s + 512]
                otok.token_logp(blk, idb, 1.0)
                otok.token_entropy_fp32(blk, 1.0)

        cpu_ms = time_cpu(cpu_fn)
        cpu_bytes = xs.numel() * 2 + ids_s.numel() * 8 + 2 * xs.shape[0] * 4
        cpu_baseline = {
            "value": round(cpu_bytes / (cpu_ms * 1e-3) / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"{xs.shape[0]} of {args.rows} rows x {args.vocab} bf16 logits, eager-torch fp32 log-prob + "
                      f"entropy in 512-row chunks, median of 5 runs ({cpu_ms:.0f} ms each)",
        }
        log(f"cpu baseline: {cpu_baseline['value']} GB/s on {cpu_baseline['cores']} threads")

    # ---------------- the other four shapes ----------------
    shapes_out = [{
        "name": "token_logp_entropy", "config": 2, "shape": f"bf16 [{args.rows},{args.vocab}] + int64 ids",
        "algorithmic_bytes": alg_bytes, "elements": x.numel(), "kernel_us": round(event_ms * 1e3, 2),
        "gbps": round(achieved, 1), "frac_of_peak": round(achieved / HBM_PEAK_GBPS, 4),
        "elements_per_s": round(x.numel() / (event_ms * 1e-3), 0), "timing": "hip events over the timed steps",
        "cpu_gbps": None if cpu_baseline is None else cpu_baseline["value"],
    }]
    if not args.skip_shapes:
        del lp, ent
        # backward of the token log-prob at the same shape: reads the logits, writes their gradient
        lse = ops.token_logp_entropy(x, ids, 1.0, want_logp=False, want_entropy=False, want_lse=True)[2]
        g_lp = torch.randn(args.rows, device=dev)
        _, bwd_ms = time_steps(torch, lambda i: ops.token_logp_bwd(x, ids, 1.0, lse, g_lp), args.steps, args.warmup)
        bwd_bytes = 2 * x.numel() * 2 + args.rows * (8 + 4 + 4)
        bwd_gbps = bwd_bytes / (bwd_ms * 1e-3) / 1e9
        log(f"token_logp_bwd: {bwd_ms:.4f} ms/launch, {bwd_gbps:.0f} GB/s = {bwd_gbps / HBM_PEAK_GBPS:.1%} of peak")
        shapes_out.append({
            "name": "token_logp_bwd", "config": 2, "shape": f"bf16 [{args.rows},{args.vocab}] logits -> bf16 gradient",
            "algorithmic_bytes": bwd_bytes, "elements": x.numel(), "kernel_us": round(bwd_ms * 1e3, 2),
            "gbps": round(bwd_gbps, 1), "frac_of_peak": round(bwd_gbps / HBM_PEAK_GBPS, 4),
            "elements_per_s": round(x.numel() / (bwd_ms * 1e-3), 0), "timing": "hip events over the timed steps",
        })
        del lse, g_lp
        from unirl_amd import _tune

        have_tune = _tune.available()
        if not have_tune:
            log("measurement build absent (python -m unirl_amd.build --tune): floors and plain reductions are null")
        for sh in make_shapes(torch, dev):
            try:
                us = time_in_graph(torch, sh["run"], sh["sets"])
                method = f"hip graph, 64 back-to-back launches over {sh['sets']} input sets"
            except Exception as exc:  # graph capture unavailable: fall back to stream-ordered events
                log(f"{sh['name']}: graph timing failed ({type(exc).__name__}: {exc}); using event loop")
                _, ms = time_steps(torch, sh["run"], 200, 20)
                us, method = ms * 1e3, "hip events over 200 stream-ordered launches (launch-bound)"
            lat = wrapper_latency_us(torch, sh["run"])
            host = host_issue_us(torch, sh["run"])
            gbps = sh["bytes"] / (us * 1e-6) / 1e9
            row = {
                "name": sh["name"], "config": sh["config"], "shape": sh["shape"], "algorithmic_bytes": sh["bytes"],
                "elements": sh["elements"], "kernel_us": round(us, 2), "gbps": round(gbps, 1),
                "frac_of_peak": round(gbps / HBM_PEAK_GBPS, 4),
                "elements_per_s": round(sh["elements"] / (us * 1e-6), 0), "wrapper_latency_us": round(lat, 1),
                "host_issue_us": round(host, 1), "timing": method,
            }
            if "bytes_padded" in sh:
                row["gbps_padded_bytes"] = round(sh["bytes_padded"] / (us * 1e-6) / 1e9, 1)
            # Yardsticks, timed in the same harness (kernels of the measurement build; null without it).
            # floor: a kernel that only moves the shape's bytes, plus a one-wavefront dependent launch.
            # plain reduction: the plainest two-launch reduction of the shape's READ bytes (one fp64
            # partial per workgroup, a dependent launch that adds them) -- what the scheme costs before
            # any of the shape's arithmetic; for a shape that also writes (the one-pass training steps)
            # it prices the reads only.
            row["floor_us"] = row["frac_of_floor"] = None
            if sh["write_bytes"] == 0 or sh.get("plain_reduction"):
                row["plain_reduction_us"] = row["frac_of_plain_reduction"] = None
            if have_tune:
                try:
                    floor_run = make_floor(torch, dev, sh["read_bytes"], sh["write_bytes"], sh["sets"], True)
                    floor_us = time_in_graph(torch, floor_run, sh["sets"])
                    row["floor_us"] = round(floor_us, 2)
                    row["frac_of_floor"] = round(floor_us / us, 4)
                    del floor_run
                except Exception as exc:
                    log(f"{sh['name']}: floor measurement failed ({type(exc).__name__}: {exc})")
                if "plain_reduction_us" in row:
                    try:
                        rb = (sh["read_bytes"] + 15) // 16 * 16
                        srcs = [torch.ones(rb, dtype=torch.uint8, device=dev) for _ in range(sh["sets"])]
                        scratch = torch.zeros(16 + 16 * 512, dtype=torch.uint8, device=dev)
                        sink = torch.zeros(1, dtype=torch.float64, device=dev)
                        red_us = time_in_graph(
                            torch, lambda i: _tune.calib_reduce(srcs[i % len(srcs)], rb, 1, 512, scratch, sink),
                            sh["sets"])
                        row["plain_reduction_us"] = round(red_us, 2)
                        row["frac_of_plain_reduction"] = round(red_us / us, 4)
                        del srcs
                    except Exception as exc:
                        log(f"{sh['name']}: plain-reduction measurement failed ({type(exc).__name__}: {exc})")
            if not args.skip_cpu and "cpu" in sh:
                cms = time_cpu(sh["cpu"], reps=sh.get("cpu_reps", 5), warmup=1)
                row["cpu_ms"] = round(cms, 2)
                row["cpu_gbps"] = round(sh["cpu_bytes"] / (cms * 1e-3) / 1e9, 3)
                row["cpu_cores"] = torch.get_num_threads()
            log(f"{sh['name']}: {us:.2f} us/launch, {gbps:.0f} GB/s = {gbps / HBM_PEAK_GBPS:.1%} of peak, "
                f"floor {row['floor_us']} us, plain reduction {row.get('plain_reduction_us')} us, "
                f"call + sync {lat:.0f} us, host {host:.0f} us")
            shapes_out.append(row)

    # HBM bytes per launch from hardware counters.  Counter runs cannot be made from inside the bench,
    # so the figure comes from the committed counter summary -- and only while that summary still
    # describes this kernel: same workload, and the same text of the kernel's two source files.
    traffic, traffic_source = None, None
    traffic_file = ROOT / "profiles" / "token_logp_entropy_traffic.json"
    if traffic_file.exists():
        try:
            rec = json.loads(traffic_file.read_text())
            same_kernel = rec.get("kernel_source_sha256") == kernel_source_sha256()
            if rec.get("rows") == args.rows and rec.get("vocab") == args.vocab and same_kernel:
                traffic = rec.get("hbm_bytes_per_launch")
                traffic_source = (f"committed counter summary profiles/{traffic_file.name} "
                                  f"(kernel sources sha256 {rec['kernel_source_sha256'][:12]}), not measured in this run")
            elif not same_kernel:
                traffic_source = "none: the kernel's sources changed since the committed counter summary was taken"
        except (ValueError, OSError, KeyError):
            traffic = None

    # the one matrix-core kernel of the path: lm_head with the log-softmax statistics in its epilogue
    # (logits never written), Qwen3-4B's head, against the library GEMM followed by the token kernel
    lmhead_out = []
    if not args.skip_shapes:
        try:
            for r in head_probe(torch, dev, args.vocab, row_counts=(2048, 8192)):
                r["roofline"] = {"bound": "mfma", "achieved": r["fused_tflops"], "peak": MFMA_BF16_PEAK_TFLOPS,
                                 "unit": "TFLOP/s", "frac": r["fused_frac_of_mfma_peak"]}
                lmhead_out.append(r)
        except Exception as exc:
            log(f"lmhead probe failed ({type(exc).__name__}: {exc})")
    result = {
        "metric": "fused-kernel HBM GB/s (token log-prob + entropy)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": None,  # one GPU: there is no scaling regime to name
        "vs_baseline": None,
        "dtype": "f32",
        "storage_dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"token log-prob + entropy, logits bf16 [{args.rows},{args.vocab}] ~N(0,2) with 1% spiked "
                        f"rows, int64 target ids, T=1 (BASELINE.json configs[1])",
            "rows": args.rows, "vocab": args.vocab,
        },
        "roofline": {
            "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic, "traffic_source": traffic_source,
            "kernel": "token_logp_entropy_kernel<bf16>", "algorithmic_bytes_per_launch": alg_bytes,
            "launch_ms": round(event_ms, 4),
        },
        "cpu_baseline": cpu_baseline,
        "parity": parity,
        "shapes": shapes_out,
        "lmhead": lmhead_out,
        "device": torch.cuda.get_device_name(0),
    }
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
