"""GPU parity of the Gaussian-KL mask, the Flow-DPPO loss, the gather and the advantage kernels."""

import math

import pytest
import torch

from oracle import advantages as oadv
from oracle import flowdppo as ofd
from oracle import schedule as osch
from tests._util import BF16_RTOL, FP32_RTOL, assert_close

pytestmark = pytest.mark.gpu

SIG = osch.sigma_schedule(28, 3.0)


def means(shape, seed, dtype, pert=0.01):
    g = torch.Generator().manual_seed(seed)
    base = torch.randn(shape, generator=g)
    old = (base + pert * torch.randn(shape, generator=g)).to(dtype)
    new = (base + pert * torch.randn(shape, generator=g)).to(dtype)
    return new, old


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(2, 3, 16, 5, 12), (4, 1, 1037), (3, 2, 4, 33, 31), (1, 5, 16, 8, 8)])
def test_kl_mask_matches_oracle(dev, dtype, shape):
    from unirl_amd import ops
    from unirl_amd.algorithms import _gaussian_kl_div

    new, old = means(shape, sum(shape), dtype)
    sig = (0.05 + 0.1 * torch.arange(shape[1], dtype=torch.float32)).reshape((1, shape[1]) + (1,) * (len(shape) - 2))
    ref = ofd.kl_per_sample(new, old, sig)
    kl, mask = ops.gaussian_kl_mask(new.to(dev), old.to(dev), sig.to(dev), 0.01)
    assert kl.shape == ref.shape and mask.dtype == torch.bool
    assert_close(kl, ref, FP32_RTOL, 0, "kl")  # the rounding emulation makes even 16-bit inputs agree to fp32 accuracy
    near = (ref - 0.01).abs() <= 4 * torch.finfo(torch.float32).eps * 0.01
    assert torch.equal(mask.cpu()[~near], (ref < 0.01)[~near])
    elem = _gaussian_kl_div(new.to(dev), old.to(dev), sig.to(dev))
    assert torch.equal(elem.cpu(), ofd.gaussian_kl(new, old, sig))


def test_kl_exact_cases(dev):
    from unirl_amd import ops

    g = torch.Generator().manual_seed(1)
    sig = torch.tensor([0.25, 0.5, 2.0]).reshape(1, 3, 1, 1, 1)
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        base = torch.randint(-8, 8, (2, 3, 4, 8, 8), generator=g).to(dtype)
        kl, mask = ops.gaussian_kl_mask((base + 0.5).to(dev), base.to(dev), sig.to(dev), 0.1)
        expect = (0.25 / (2 * sig.reshape(1, 3) ** 2)).expand(2, 3)
        assert torch.equal(kl.cpu(), expect) and torch.equal(mask.cpu(), expect < 0.1)
        kl, mask = ops.gaussian_kl_mask(base.to(dev), base.to(dev), sig.to(dev), 1e-5)
        assert float(kl.abs().max()) == 0.0 and bool(mask.all())
    # scalar sigma, and a threshold exactly at the value: `<` is strict
    base = torch.zeros(2, 1, 64)
    kl, mask = ops.gaussian_kl_mask((base + 1.0).to(dev), base.to(dev), torch.tensor(1.0), 0.5)
    assert kl.cpu().tolist() == [[0.5], [0.5]] and not bool(mask.any())


def test_mask_threshold_sweep_reports_near_threshold(dev):
    """Perturbation sweep so both mask values occur; rows whose KL lies within 1 ulp of the threshold
    are counted and excluded from the bit-exact comparison."""
    from unirl_amd import ops

    shape = (2, 1, 16, 21, 30, 52)
    total, near_total, mism = 0, 0, 0
    seen = set()
    for pert in (0.003, 0.01, 0.02, 0.03, 0.1):
        new, old = means(shape, int(pert * 1e4), torch.bfloat16, pert)
        sig = torch.tensor(0.1648)
        ref = ofd.kl_per_sample(new, old, sig.reshape(1, 1, 1, 1, 1, 1))
        kl, mask = ops.gaussian_kl_mask(new.to(dev), old.to(dev), sig.to(dev), 0.01)
        ref_mask = ref < 0.01
        near = (ref - 0.01).abs() <= 2 * torch.finfo(torch.float32).eps * 0.01
        total += ref.numel()
        near_total += int(near.sum())
        mism += int((mask.cpu() != ref_mask)[~near].sum())
        seen.update(ref_mask.flatten().tolist())
        assert_close(kl, ref, FP32_RTOL, 0, f"kl pert {pert}")
    print(f"mask rows {total}, within 1 ulp of threshold {near_total}, mismatches elsewhere {mism}")
    assert mism == 0 and seen == {True, False}


def test_flowdppo_loss_matches_oracle(dev):
    from unirl_amd.algorithms import _flowdppo_kl_adv_loss

    g = torch.Generator().manual_seed(2)
    B, S = 8, 3
    for dtype in (torch.bfloat16, torch.float32):
        new_means, old_means = means((B, S, 4, 16, 16), 3, dtype, pert=0.02)
        old_means[::2] = new_means[::2]  # half of the samples are on-policy: kl = 0
        new_logp = 1e-3 * torch.randn(B, S, generator=g)
        old_logp = new_logp + 2e-4 * torch.randn(B, S, generator=g)
        old_logp[1] = new_logp[1]  # ratio exactly 1
        adv = torch.randn(B, 1, generator=g).expand(B, S).clone()
        adv[2] = 0.0
        sig_t = ofd.sigma_t(SIG, [2, 5, 9], 0.7)
        nr = new_logp.clone().requires_grad_(True)
        ref_elem, ref_m = ofd.flowdppo_loss(nr, old_logp, new_means, old_means, adv, sig_t, 1e-3)
        ref_elem.mean().backward()
        nd = new_logp.to(dev).requires_grad_(True)
        elem, m = _flowdppo_kl_adv_loss(new_logp=nd, old_logp=old_logp.to(dev), new_means=new_means.to(dev),
                                        old_means=old_means.to(dev), advantages=adv.to(dev), sigma_t=sig_t.to(dev),
                                        kl_mask_threshold=1e-3)
        elem.mean().backward()
        assert set(m) == set(ref_m) and elem.shape == (B, S)
        assert_close(elem, ref_elem, FP32_RTOL, 1e-8, "flowdppo loss")
        assert_close(nd.grad, nr.grad, FP32_RTOL, 1e-8, "flowdppo grad")
        for k in ref_m:
            assert abs(float(m[k]) - float(ref_m[k])) <= 1e-5 * abs(float(ref_m[k])) + 1e-7, (k, float(m[k]), float(ref_m[k]))
        assert 0.0 < float(m["masked_fraction"]) < 1.0


@pytest.mark.parametrize("shape", [(8, 3, 4, 16, 16), (2, 1, 16, 21, 60, 104), (5, 7, 37), (64, 12, 8, 8)])
def test_flowdppo_step_two_launches(dev, shape):
    """The fused loss step (KL kernel + one finishing workgroup) against the oracle: KL, loss,
    metrics, and the gradient of (loss.mean() * loss_scale); and bit for bit against the
    separate entry points."""
    from unirl_amd import ops

    g = torch.Generator().manual_seed(sum(shape))
    B, S = shape[:2]
    loss_scale = 0.37
    for dtype in (torch.bfloat16, torch.float32):
        new_means, old_means = means(shape, 3, dtype, pert=0.02)
        old_means[::2] = new_means[::2]
        new_logp = 1e-3 * torch.randn(B, S, generator=g)
        old_logp = new_logp + 2e-4 * torch.randn(B, S, generator=g)
        adv = torch.randn(B, 1, generator=g).expand(B, S).clone()
        steps = sorted(torch.randperm(14, generator=g)[:S].tolist())
        sig_t = ofd.sigma_t(SIG, steps, 0.7).reshape(1, S, *([1] * (len(shape) - 2)))  # one per step
        nr = new_logp.clone().requires_grad_(True)
        ref_elem, ref_m = ofd.flowdppo_loss(nr, old_logp, new_means, old_means, adv, sig_t, 1e-3)
        (ref_elem.mean() * loss_scale).backward()
        dv = [t.to(dev) for t in (new_logp, old_logp, new_means, old_means, adv, sig_t)]
        kl, elem, mvec, grad = ops.flowdppo_step(*dv, 1e-3, loss_scale=loss_scale)
        assert_close(elem, ref_elem, FP32_RTOL, 1e-8, "loss")
        assert_close(grad, nr.grad, FP32_RTOL, 1e-9, "grad")
        vals = mvec.tolist()
        for k, slot in ops.FLOWDPPO_METRIC_SLOTS.items():
            if k != "loss_mean":
                assert abs(vals[slot] - float(ref_m[k])) <= 1e-5 * abs(float(ref_m[k])) + 1e-7, (k, vals[slot], float(ref_m[k]))
        # the separate entry points give the same bits
        kl2, _ = ops.gaussian_kl_mask(dv[2], dv[3], dv[5], 1e-3, reduce_from_dim=2, want_mask=False)
        elem2, mvec2 = ops.flowdppo_loss(dv[0], dv[1], dv[4], kl2, 1e-3)
        assert torch.equal(kl, kl2) and torch.equal(elem, elem2) and torch.equal(mvec[:13], mvec2[:13])
        _, _, _, none = ops.flowdppo_step(*dv, 1e-3)
        assert none is None


def test_flowdppo_truth_table(dev):
    from unirl_amd.algorithms import _flowdppo_kl_adv_loss

    cases = [(k, ld, a) for k in (False, True) for ld in (-0.1, 0.0, 0.1) for a in (-1.0, 0.0, 1.0)]
    n = len(cases)
    new_logp = torch.tensor([c[1] for c in cases]).reshape(n, 1)
    adv = torch.tensor([c[2] for c in cases]).reshape(n, 1)
    old_means = torch.zeros(n, 1, 2, 4, 4)
    new_means = old_means + torch.tensor([1.0 if c[0] else 0.0 for c in cases]).reshape(n, 1, 1, 1, 1)
    elem, m = _flowdppo_kl_adv_loss(new_logp=new_logp.to(dev), old_logp=torch.zeros(n, 1).to(dev),
                                    new_means=new_means.to(dev), old_means=old_means.to(dev), advantages=adv.to(dev),
                                    sigma_t=torch.ones(1, 1, 1, 1, 1).to(dev), kl_mask_threshold=0.01)
    for i, (kl_high, ld, a) in enumerate(cases):
        removed = kl_high and ((ld > 0 and a > 0) or (ld < 0 and a < 0))
        assert abs(float(elem[i, 0]) - (0.0 if removed else -a * math.exp(ld))) < 1e-6, cases[i]
    assert abs(float(m["kl_mask_fraction"]) - 0.5) < 1e-7 and abs(float(m["masked_fraction"]) - 2 / 18) < 1e-7


def test_config4_wan_shape(dev):
    """bf16 [2,16,21,60,104] means, base + N(0, 0.01) (seed 1004); sigma 0.5, eta 0.7; threshold 0.01."""
    from unirl_amd import ops

    g = torch.Generator().manual_seed(1004)
    shape = (2, 1, 16, 21, 60, 104)
    base = torch.randn(shape, generator=g)
    old = (base + 0.01 * torch.randn(shape, generator=g)).bfloat16()
    new = (base + 0.01 * torch.randn(shape, generator=g)).bfloat16()
    # per-step std: sigma = 0.5 -> std_dev_t = sqrt(0.5/0.5)*0.7 = 0.7; dt of the schedule step nearest 0.5
    i = int((SIG - 0.5).abs().argmin())
    sig_t = torch.tensor(0.7 * math.sqrt(float(SIG[i] - SIG[i + 1]))).reshape(1, 1, 1, 1, 1, 1)
    ref = ofd.kl_per_sample(new, old, sig_t)
    kl, mask = ops.gaussian_kl_mask(new.to(dev), old.to(dev), sig_t.to(dev), 0.01)
    assert_close(kl, ref, FP32_RTOL, 0, "config-4 kl")
    near = (ref - 0.01).abs() <= 2 * torch.finfo(torch.float32).eps * 0.01
    print(f"config-4 kl {kl.flatten().tolist()} mask {mask.flatten().tolist()} near-threshold rows {int(near.sum())}")
    assert torch.equal(mask.cpu()[~near], (ref < 0.01)[~near])


# ---------------------------------------------------------------- gather
def test_gather_sde_field_device(dev):
    from unirl_amd.algorithms import gather_sde_field

    g = torch.Generator().manual_seed(3)
    idx = torch.tensor([7, 2, 9, 0, 4])
    for shape, dtype in (((3, 5, 2, 4), torch.float32), ((2, 5), torch.float32), ((4, 5, 3, 5, 7), torch.bfloat16),
                         ((2, 5, 1), torch.int64), ((3, 5, 16, 21, 8), torch.bfloat16)):
        t = (torch.randn(shape, generator=g) * 100).to(dtype)
        for target in ([2, 9], [0, 4, 7], [9], [4, 4], [7, 2, 9, 0, 4]):
            got = gather_sde_field(t.to(dev), idx.to(dev), target)
            assert got.is_cuda and torch.equal(got.cpu(), ofd.gather_by_lookup(t, idx, target))
    with pytest.raises(ValueError, match="not in sde_indices"):
        gather_sde_field(t.to(dev), idx.to(dev), [3])


# ---------------------------------------------------------------- advantages
@pytest.mark.parametrize("n_groups,branch", [(16, 16), (1, 7), (40, 1), (300, 4), (3, 1000)])
def test_group_advantages_match_oracle(dev, n_groups, branch):
    from unirl_amd.types import RolloutTrack, compute_advantages

    g = torch.Generator().manual_seed(n_groups * 31 + branch)
    n = n_groups * branch
    pids = [f"p{i // branch}" for i in range(n)]
    for rewards in ((torch.rand(n, generator=g) < 0.5).float(), 10 * torch.randn(n, generator=g) + 3):
        for kw in (dict(), dict(normalize=False), dict(use_global_std=True), dict(scope="global"),
                   dict(scope="global", normalize=False), dict(eps=1e-4)):
            if n == 1 and (kw.get("use_global_std") or kw.get("scope") == "global"):
                continue
            ref = oadv.compute_advantages(rewards, pids, **kw)
            got = compute_advantages(rewards.to(dev), pids, **kw)
            assert got.is_cuda and got.dtype == torch.float32
            assert_close(got, ref, FP32_RTOL, 1e-6, f"{kw}")
            got_cpu = compute_advantages(rewards, pids, **kw)  # host rewards come back on the host
            assert not got_cpu.is_cuda and torch.equal(got_cpu, got.cpu())
    track = RolloutTrack(sample_ids=[str(i) for i in range(n)], parent_ids=pids, rewards=rewards)
    out = track.compute_advantages()
    assert out is not track and track.advantages is None
    assert_close(out.advantages, oadv.compute_advantages(rewards, pids), FP32_RTOL, 1e-6, "track")


def test_group_advantages_degenerate(dev):
    from unirl_amd.types import compute_advantages

    r = torch.tensor([1.0, 1.0, 1.0, 0.0, 1.0, 0.0], device=dev)
    adv = compute_advantages(r, ["a", "a", "a", "b", "b", "b"])
    assert adv[:3].tolist() == [0.0, 0.0, 0.0]
    assert float(compute_advantages(torch.tensor([3.0], device=dev), ["x"])[0]) == 0.0
    assert torch.isnan(compute_advantages(torch.tensor([3.0], device=dev), ["x"], scope="global")).all()
    assert torch.isnan(oadv.compute_advantages(torch.tensor([3.0]), ["x"], scope="global")).all()


def test_normalize_grouped_matches_oracle(dev):
    from unirl_amd.algorithms import normalize_global, normalize_grouped

    g = torch.Generator().manual_seed(5)
    r = torch.rand(40, generator=g)
    r[7] = r[3]  # a tie inside a trimmed group
    groups = [[0, 5, 7, 2, 3], list(range(10, 30)), [], [33, 31], [39]]
    for kw in (dict(), dict(trim_outliers_ratio=0.2), dict(clip_max=0.8), dict(use_global_std=True),
               dict(trim_outliers_ratio=0.1, use_global_std=True, clip_max=1.5), dict(epsilon=1e-3)):
        # fp32 torch loses digits in the std of a few close values; the float64 evaluation of the
        # same formulas is the yardstick, the fp32 one a looser cross-check
        truth = oadv.normalize_grouped(r.double(), groups, **kw)
        ref = oadv.normalize_grouped(r, groups, **kw)
        got = normalize_grouped(r.to(dev), groups, **kw)
        assert_close(got, truth, FP32_RTOL, 1e-6, f"{kw} vs float64")
        assert_close(got, ref, 1e-4, 1e-6, f"{kw} vs fp32")
        assert float(got[8]) == 0.0  # in no group
    assert_close(normalize_global(r.to(dev)), oadv.normalize_global(r), FP32_RTOL, 1e-6, "global")
    assert_close(normalize_global(r.to(dev), clip_max=0.5), oadv.normalize_global(r, clip_max=0.5), FP32_RTOL, 1e-6,
                 "global clipped")
    with pytest.raises(IndexError):
        normalize_grouped(r.to(dev), [[0, 40]])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_gaussian_kl_div_is_differentiable(dev, dtype):
    """The reference's _gaussian_kl_div is plain torch; a caller may differentiate it."""
    from unirl_amd.algorithms import _gaussian_kl_div

    g = torch.Generator().manual_seed(21)
    p = torch.randn(3, 4, 4, 8, 8, generator=g).to(dtype)
    q = (p.float() + 0.1 * torch.randn(p.shape, generator=g)).to(dtype)
    s = torch.tensor([0.3, 0.25, 0.2, 0.15]).view(1, 4, 1, 1, 1)
    w = torch.randn(p.shape, generator=g)
    pr, qr = p.clone().requires_grad_(True), q.clone().requires_grad_(True)
    (ofd.gaussian_kl(pr, qr, s) * w).sum().backward()
    pd, qd = p.to(dev).requires_grad_(True), q.to(dev).requires_grad_(True)
    out = _gaussian_kl_div(pd, qd, s.to(dev))
    assert out.dtype == torch.float32 and out.requires_grad
    (out * w.to(dev)).sum().backward()
    rtol = FP32_RTOL if dtype == torch.float32 else 8e-3  # two 16-bit roundings in the chain
    scale = float(pr.grad.float().abs().max())
    assert pd.grad.dtype == dtype and qd.grad.dtype == dtype
    assert_close(pd.grad, pr.grad, rtol, rtol * scale * 1e-2, "grad p")
    assert_close(qd.grad, qr.grad, rtol, rtol * scale * 1e-2, "grad q")
    # only one side needs a gradient
    pd2 = p.to(dev).requires_grad_(True)
    _gaussian_kl_div(pd2, q.to(dev), s.to(dev)).sum().backward()
    pr2 = p.clone().requires_grad_(True)
    ofd.gaussian_kl(pr2, q, s).sum().backward()
    assert_close(pd2.grad, pr2.grad, rtol, rtol * float(pr2.grad.float().abs().max()) * 1e-2, "grad p only")
