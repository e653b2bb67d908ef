"""End-to-end micro-steps of the algorithm classes on fake stages: the same fake model is run
through the GPU package and through the CPU oracle, and loss, metrics and parameter gradients
are compared."""

import math
import types

import pytest
import torch

from oracle import advantages as oadv
from oracle import flowdppo as ofd
from oracle import losses as olos
from oracle import schedule as osch
from oracle import sde as osde
from tests._util import FP32_RTOL, assert_close

pytestmark = pytest.mark.gpu

SIG = osch.sigma_schedule(10, 3.0)


# ---------------------------------------------------------------- AR: GRPO / DRPO
class FakeARStage:
    """replay() = a differentiable function of one parameter vector and the stored tokens."""

    def __init__(self, base, direction, device):
        self.base = base.to(device)
        self.direction = direction.to(device)
        self.theta = torch.tensor(0.3, device=device, requires_grad=True)
        self.seen_temperature = None

    def replay(self, conditions, *, segment, temperature):
        self.seen_temperature = temperature
        return self.base + self.theta * self.direction


def text_segment(tokens, lengths, log_probs, loss_mask=None):
    return types.SimpleNamespace(tokens=tokens, lengths=lengths, log_probs=log_probs, loss_mask=loss_mask)


def ar_case(seed=0, n_seq=12, max_len=60):
    g = torch.Generator().manual_seed(seed)
    lengths = torch.randint(0, max_len + 1, (n_seq,), generator=g)
    lengths[3] = 0
    n_tok = int(lengths.sum())
    old = -6 * torch.rand(n_tok, generator=g)
    base = old + 0.02 * torch.randn(n_tok, generator=g)
    direction = 0.3 * torch.randn(n_tok, generator=g)
    tokens = torch.randint(0, 1000, (n_tok,), generator=g)
    rewards = torch.rand(n_seq, generator=g)
    adv = oadv.compute_advantages(rewards, [i // 4 for i in range(n_seq)])
    return lengths, old, base, direction, tokens, adv


@pytest.mark.parametrize("mode", ["token-mean", "seq-mean-token-sum-norm", "seq-mean-token-mean"])
def test_grpo_micro_step(dev, mode):
    from unirl_amd.algorithms import GRPO

    lengths, old, base, direction, tokens, adv = ar_case(1)
    # oracle on the CPU
    cpu = FakeARStage(base, direction, torch.device("cpu"))
    new = cpu.replay(None, segment=None, temperature=1.0)
    ref_loss, ref_m = olos.token_loss("grpo", new, old, adv, lengths, mode=mode, horizon=64, clip_range=0.15,
                                      clip_range_high=0.25)
    (ref_loss * 0.5).backward()
    # package on the GPU
    stage = FakeARStage(base, direction, dev)
    algo = GRPO(stage=stage, clip_range=0.2, clip_range_high=0.25 / 0.75, clip_schedule="linear_decay",
                loss_agg_mode=mode, horizon=64, sampling_temperature=1.0)
    seg = text_segment(tokens.to(dev), lengths, old)  # lengths / rollout log-probs arrive on the host
    res = algo.compute_loss_and_backward(conditions={}, segment=seg, advantages=adv.to(dev), training_progress=0.5,
                                         loss_scale=0.5)
    assert res.has_backward and res.num_steps_or_tokens == int(lengths.sum()) and stage.seen_temperature == 1.0
    assert abs(res.metrics["clip_range"] - 0.15) < 1e-12
    assert abs(res.loss - float(ref_loss)) <= FP32_RTOL * abs(float(ref_loss)) + 1e-7
    assert res.metrics["policy_loss"] == res.loss
    for k, v in ref_m.items():
        assert abs(res.metrics[k] - float(v)) <= 1e-5 * abs(float(v)) + 2.0 / int(lengths.sum()) * ("clip" in k) + 1e-8, k
    assert_close(stage.theta.grad, cpu.theta.grad, 1e-5, 1e-8, "d loss / d theta")


@pytest.mark.parametrize("seed", range(6))
def test_ar_micro_steps_on_random_segments(dev, seed):
    """GRPO and DRPO micro-steps on segments of random size, among them segments with as many
    tokens as sequences (the per-sample advantages must not be mistaken for per-token ones)."""
    import random

    from unirl_amd.algorithms import DRPO, GRPO

    rng = random.Random(500 + seed)
    for case in range(6):
        n_seq, max_len = rng.randint(1, 14), rng.choice((1, 2, 3, 8, 60, 300))
        g = torch.Generator().manual_seed(rng.randint(0, 10**6))
        lengths = torch.randint(0, max_len + 1, (n_seq,), generator=g)
        if case == 0:  # n_tok == n_seq with unequal lengths
            lengths = torch.zeros(n_seq, dtype=torch.int64)
            lengths[0] = n_seq
        if int(lengths.sum()) == 0:
            lengths[-1] = max_len
        n_tok = int(lengths.sum())
        old = -6 * torch.rand(n_tok, generator=g)
        base = old + 0.05 * torch.randn(n_tok, generator=g)
        direction = 0.3 * torch.randn(n_tok, generator=g)
        adv = torch.randn(n_seq, generator=g)
        kind = rng.choice(("grpo", "drpo"))
        mode = rng.choice(("token-mean", "seq-mean-token-sum-norm"))
        scale = rng.choice((1.0, 0.25))
        cpu = FakeARStage(base, direction, torch.device("cpu"))
        new = cpu.replay(None, segment=None, temperature=1.0)
        ref_loss, ref_m = olos.token_loss(kind, new, old, adv, lengths, mode=mode, horizon=64, clip_range=0.2,
                                          clip_range_high=0.28, epsilon=12.5)
        (ref_loss * scale).backward()
        stage = FakeARStage(base, direction, dev)
        if kind == "grpo":
            algo = GRPO(stage=stage, clip_range=0.2, clip_range_high=0.28, loss_agg_mode=mode, horizon=64)
        else:
            algo = DRPO(pipeline=types.SimpleNamespace(ar=stage), loss_agg_mode=mode, horizon=64)
        seg = text_segment(torch.zeros(n_tok, dtype=torch.int64, device=dev), lengths, old.to(dev))
        res = algo.compute_loss_and_backward(conditions={}, segment=seg, advantages=adv.to(dev), training_progress=0.0,
                                             loss_scale=scale)
        what = f"{kind} {mode} lengths {lengths.tolist()}"
        assert abs(res.loss - float(ref_loss)) <= 2e-5 * abs(float(ref_loss)) + 2e-6 * float(adv.abs().max()), what
        for k, v in ref_m.items():
            if k in res.metrics:
                assert abs(res.metrics[k] - float(v)) <= 2e-5 * abs(float(v)) + 2.0 / n_tok * ("clip" in k) + 1e-6, (what, k)
        assert_close(stage.theta.grad, cpu.theta.grad, 2e-5, 1e-7, what + ": d loss / d theta")


def test_drpo_micro_step_with_mask_and_replay_anchor(dev):
    from unirl_amd.algorithms import DRPO

    lengths, old, base, direction, tokens, adv = ar_case(2)
    mask = (torch.rand(old.shape, generator=torch.Generator().manual_seed(3)) < 0.8).float()
    cpu = FakeARStage(base, direction, torch.device("cpu"))
    new = cpu.replay(None, segment=None, temperature=0.7)
    ref_loss, ref_m = olos.token_loss("drpo", new, old, adv, lengths, mode="seq-mean-token-sum-norm", horizon=64,
                                      epsilon=12.5, loss_mask=mask)
    ref_loss.backward()
    stage = FakeARStage(base, direction, dev)
    algo = DRPO(pipeline=types.SimpleNamespace(ar=stage), loss_agg_mode="seq-mean-token-sum-norm", horizon=64)
    assert algo.sampling_temperature == 0.7 and algo.drpo_epsilon == 12.5
    seg = text_segment(tokens.to(dev), lengths.to(dev), old.to(dev), mask.to(dev))
    res = algo.compute_loss_and_backward(conditions={}, segment=seg, advantages=adv.to(dev), training_progress=0.0,
                                         loss_scale=1.0)
    assert abs(res.loss - float(ref_loss)) <= FP32_RTOL * abs(float(ref_loss)) + 1e-7
    for k, v in ref_m.items():
        assert abs(res.metrics[k] - float(v)) <= 1e-5 * abs(float(v)) + 1e-7, k
    assert res.metrics["drpo_epsilon"] == 12.5
    assert_close(stage.theta.grad, cpu.theta.grad, 1e-5, 1e-8, "d loss / d theta")
    # 'replay' anchor: prepare_segment overwrites log_probs with a no-grad replay -> ratio is exactly 1
    algo2 = DRPO(pipeline=types.SimpleNamespace(ar=stage), old_logp_source="replay")
    algo2.prepare_segment(conditions={}, segment=seg)
    assert not seg.log_probs.requires_grad
    res2 = algo2.compute_loss_and_backward(conditions={}, segment=seg, advantages=adv.to(dev), training_progress=0.0,
                                           loss_scale=1.0)
    assert res2.metrics["ratio_mean"] == 1.0 and res2.metrics["approx_kl"] == 0.0


def test_empty_segments_short_circuit(dev):
    from unirl_amd.algorithms import DRPO, GRPO

    stage = FakeARStage(torch.zeros(0), torch.zeros(0), dev)
    for algo in (GRPO(stage=stage), DRPO(pipeline=types.SimpleNamespace(ar=stage))):
        for seg in (text_segment(None, None, None),
                    text_segment(torch.zeros(0, dtype=torch.int64), torch.zeros(2, dtype=torch.int64), torch.zeros(0))):
            res = algo.compute_loss_and_backward(conditions={}, segment=seg, advantages=torch.zeros(2),
                                                 training_progress=0.0, loss_scale=1.0)
            assert res.loss == 0.0 and not res.has_backward and res.metrics == {}
    with pytest.raises(ValueError, match="advantages batch=3 != lengths=2"):
        GRPO(stage=FakeARStage(torch.zeros(4), torch.zeros(4), dev)).compute_loss_and_backward(
            conditions={}, segment=text_segment(torch.zeros(4), torch.tensor([2, 2]), torch.zeros(4)),
            advantages=torch.zeros(3, device=dev), training_progress=0.0, loss_scale=1.0)


# ---------------------------------------------------------------- diffusion: FlowGRPO / FlowDPPO
class FakeDiffusionStage:
    """replay() runs the SDE log-prob replay on stored latents with velocity = w * field[step]."""

    def __init__(self, fields, device, denoise):
        self.fields = [f.to(device) for f in fields]
        self.w = torch.tensor(1.0, device=device, requires_grad=True)
        self.device = device
        self.denoise = denoise

    def replay(self, conditions, *, segment, params, step_indices):
        lps, means = [], []
        sig = segment.sigmas
        for j, step in enumerate(step_indices):
            x = segment.latents[:, step].to(self.device)
            x_next = segment.latents[:, step + 1].to(self.device)
            _, lp, mean = self.denoise(self.w * self.fields[step], x, sig[step], sig[step + 1], eta=params.eta,
                                       prev_sample=x_next, sigma_max=sig[1])
            lps.append(lp)
            means.append(mean)
        return types.SimpleNamespace(log_probs=torch.stack(lps, 1), prev_sample_means=torch.stack(means, 1))


def diffusion_case(seed=0, B=6, T=10, shape=(4, 8, 8)):
    g = torch.Generator().manual_seed(seed)
    fields = [torch.randn((B,) + shape, generator=g) for _ in range(T)]
    x = torch.randn((B,) + shape, generator=g)
    lat = [x]
    for k in range(T):  # a trajectory sampled at w = 1
        x, _, _ = osde.sde_denoise("flow", fields[k], x, SIG[k], SIG[k + 1], eta=0.7,
                                   noise=torch.randn(x.shape, generator=g), sigma_max=SIG[1])
        lat.append(x)
    latents = torch.stack(lat, 1)  # [B, T+1, ...]
    rewards = torch.rand(B, generator=g)
    adv = oadv.compute_advantages(rewards, [i // 3 for i in range(B)], use_global_std=True)
    return fields, latents, adv


def cpu_denoise(v, x, s, sn, *, eta, prev_sample, sigma_max):
    return osde.sde_denoise("flow", v, x, s, sn, eta=eta, prev_sample=prev_sample, sigma_max=sigma_max,
                            ieee_sqrt=True)


def f64_denoise(v, x, s, sn, *, eta, prev_sample, sigma_max):
    """The flow SDE replay in float64 (closed form of unirl/sde/kernels.py:207-236 and :154-177): the
    yardstick that says which of two fp32 evaluations of the same pipeline is closer to the truth."""
    v, x, prev = v.double(), x.double(), prev_sample.double()
    s, sn, smax = float(s), float(sn), float(sigma_max)
    dt = sn - s
    std = math.sqrt(s / (1.0 - (smax if s == 1.0 else s))) * eta
    mean = x * (1.0 + std * std / (2.0 * s) * dt) + v * (1.0 + std * std * (1.0 - s) / (2.0 * s)) * dt
    sv = std * math.sqrt(-dt)
    lp = -((prev - mean) ** 2) / (2.0 * sv * sv) - math.log(sv) - 0.5 * math.log(2.0 * math.pi)
    return prev, lp.mean(dim=tuple(range(1, lp.ndim))), mean


# every comparison of a micro-step test with the fp32 oracle: (what, relative to the value, relative to
# the magnitude of the summed terms).  The second is bounded by TERMS_RTOL: a mean of n terms of
# magnitude s, each carrying fp32 rounding, moves by a few ulps of s between two correct evaluations.
REL_TO_FP32_ORACLE = []
TERMS_RTOL = 1e-5


def no_worse_than_fp32(got, fp32_ref, f64_ref, what, scale=None, slack=2.0, terms_scale=None):
    """`got` (the kernels) must be as close to the float64 value as the reference's own fp32
    evaluation is (within `slack`), or within one fp32 ulp (2^-23) of `scale`, the typical magnitude
    of the terms the value is a mean of (default: the value itself) -- a mean of cancelling terms
    cannot be held to an ulp of its own small size, and the fp32 reference sometimes lands on the
    exact value by luck.  The bound is the reference's own rounding error, not a loosened constant."""
    got, fp32_ref, f64_ref = float(got), float(fp32_ref), float(f64_ref)
    scale = abs(f64_ref) if scale is None else float(scale)
    err, ref_err = abs(got - f64_ref), abs(fp32_ref - f64_ref)
    # the plain difference to the fp32 oracle, printed (pytest -s / -rP) and bounded: relative to the
    # value, and relative to the magnitude of the terms the value is a mean of
    rel_value = abs(got - fp32_ref) / max(abs(fp32_ref), 1e-30)
    rel_terms = abs(got - fp32_ref) / max(scale if terms_scale is None else float(terms_scale), 1e-30)
    print(f"[vs fp32 oracle] {what}: kernel {got:.9g}, oracle {fp32_ref:.9g}, float64 {f64_ref:.9g}; "
          f"|kernel - oracle| = {rel_value:.2e} of the value, {rel_terms:.2e} of the terms' magnitude")
    REL_TO_FP32_ORACLE.append((what, rel_value, rel_terms))
    assert rel_terms <= TERMS_RTOL, f"{what}: {rel_terms:.3e} of the terms' magnitude from the fp32 oracle"
    assert err <= slack * ref_err + 2.0 ** -23 * scale + 1e-12, (
        f"{what}: kernel {got!r} is {err:.3e} from the float64 value {f64_ref!r}, "
        f"the fp32 reference {fp32_ref!r} only {ref_err:.3e} (scale {scale:.3e})")


def mean_abs_term_gradient(elem, w):
    """Mean magnitude of d elem[i] / d w over the elements: the scale of the terms d mean(elem) / d w sums."""
    grads = [torch.autograd.grad(e, w, retain_graph=True)[0] for e in elem.reshape(-1)]
    return float(torch.stack(grads).abs().mean())


def test_flowdppo_micro_step(dev):
    from unirl_amd.algorithms import FlowDPPO
    from unirl_amd.sde import FlowSDEStrategy

    fields, latents, adv = diffusion_case(4)
    sde_idx = torch.tensor([4, 1, 2])  # unsorted on purpose
    params = types.SimpleNamespace(eta=0.7)
    steps = [4, 1, 2]
    # ---- oracle pipeline on the CPU: anchor at w = 1, then the policy moves to w = 1.05
    cpu = FakeDiffusionStage(fields, torch.device("cpu"), cpu_denoise)
    seg_cpu = types.SimpleNamespace(latents=latents, sigmas=SIG, sde_indices=sde_idx, sde_logp=None, sde_means=None)
    with torch.no_grad():
        anchor = cpu.replay(None, segment=seg_cpu, params=params, step_indices=steps)
    with torch.no_grad():
        cpu.w.fill_(1.05)
    new = cpu.replay(None, segment=seg_cpu, params=params, step_indices=steps)
    sig_t = ofd.sigma_t(SIG, steps, 0.7)
    adv_b = adv.reshape(-1, 1).expand_as(new.log_probs)
    thr = float(ofd.kl_per_sample(new.prev_sample_means, anchor.prev_sample_means, sig_t).median())
    ref_elem, ref_m = ofd.flowdppo_loss(new.log_probs, anchor.log_probs, new.prev_sample_means,
                                        anchor.prev_sample_means, adv_b, sig_t, thr)
    ref_loss = ref_elem.mean()
    (ref_loss * 0.25).backward()
    # ---- the same pipeline in float64
    f64 = FakeDiffusionStage([f.double() for f in fields], torch.device("cpu"), f64_denoise)
    seg64 = types.SimpleNamespace(latents=latents, sigmas=SIG, sde_indices=sde_idx)
    with torch.no_grad():
        anchor64 = f64.replay(None, segment=seg64, params=params, step_indices=steps)
        f64.w.fill_(1.05)
    new64 = f64.replay(None, segment=seg64, params=params, step_indices=steps)
    elem64, m64 = ofd.flowdppo_loss(new64.log_probs, anchor64.log_probs, new64.prev_sample_means,
                                    anchor64.prev_sample_means, adv_b.double(), sig_t.double(), thr)
    loss64 = elem64.mean()
    grad_scale64 = 0.25 * mean_abs_term_gradient(elem64, f64.w)
    (loss64 * 0.25).backward()
    # ---- package on the GPU
    strat = FlowSDEStrategy()
    stage = FakeDiffusionStage(fields, dev, strat.denoise)
    seg = types.SimpleNamespace(latents=latents.to(dev), sigmas=SIG.to(dev), sde_indices=sde_idx.to(dev),
                                sde_logp=None, sde_means=None)
    algo = FlowDPPO(params=params, stage=stage, kl_mask_threshold=thr, old_logp_source="replay")
    algo.prepare_segment(conditions={}, segment=seg)
    assert seg.sde_logp.shape == (6, 3) and seg.sde_means.is_cuda and not seg.sde_means.requires_grad
    assert_close(seg.sde_logp, anchor.log_probs, FP32_RTOL, 2e-6, "anchor logp")
    assert torch.equal(seg.sde_means.cpu(), anchor.prev_sample_means)
    with torch.no_grad():
        stage.w.fill_(1.05)
    res = algo.compute_loss_and_backward(conditions={}, segment=seg, advantages=adv.to(dev), training_progress=0.0,
                                         loss_scale=0.25)
    assert res.has_backward and res.num_steps_or_tokens == 3
    # The loss is a product of advantages and exp(new - old) of log-probs that each carry ~1e-7 of
    # fp32 rounding, so two correct fp32 evaluations differ by more than 1e-5 of it.  The bound is
    # therefore the reference's own distance from the float64 value.
    no_worse_than_fp32(res.loss, ref_loss, loss64, "loss", scale=elem64.abs().mean())
    # magnitude of the terms behind each metric, for the plain bound against the fp32 oracle: the ratio
    # statistics are built from ratios of magnitude 1 (their std is a small difference of those), and
    # approx_kl = mean(ld^2 / 2) moves by ld * ulp(log-prob) when a log-prob moves by an ulp
    terms = {k: 1.0 for k in ("ratio_mean", "ratio_std", "ratio_min", "ratio_max")}
    terms["approx_kl"] = float((new.log_probs - anchor.log_probs).abs().mean() * new.log_probs.abs().mean())
    for k, v in ref_m.items():
        no_worse_than_fp32(res.metrics[k], v, m64[k], k, terms_scale=terms.get(k))
    assert 0.0 < res.metrics["kl_mask_fraction"] < 1.0
    no_worse_than_fp32(stage.w.grad, cpu.w.grad, f64.w.grad, "d loss / d w through the SDE backward kernel",
                       scale=grad_scale64)
    # sigma_t helper
    assert_close(algo._compute_sigma_t(seg, steps, dev), sig_t, 1e-6, 0, "sigma_t")
    algo.add_kl_coefficient = False
    assert torch.equal(algo._compute_sigma_t(seg, steps, dev).cpu(), torch.ones(1, 3, 1, 1, 1))


def test_flowgrpo_micro_step(dev):
    from unirl_amd.algorithms import FlowGRPO
    from unirl_amd.sde import FlowSDEStrategy

    fields, latents, adv = diffusion_case(5)
    sde_idx = torch.tensor([0, 3, 7])
    params = types.SimpleNamespace(eta=0.7)
    steps = [0, 3, 7]
    cpu = FakeDiffusionStage(fields, torch.device("cpu"), cpu_denoise)
    seg_cpu = types.SimpleNamespace(latents=latents, sigmas=SIG, sde_indices=sde_idx)
    with torch.no_grad():
        anchor = cpu.replay(None, segment=seg_cpu, params=params, step_indices=steps).log_probs
        cpu.w.fill_(1.0002)
    new = cpu.replay(None, segment=seg_cpu, params=params, step_indices=steps).log_probs
    ref_elem, ref_m = olos.grpo_clip_loss(new, anchor, adv.reshape(-1, 1).expand_as(new), 1e-4)
    ref_loss = ref_elem.mean()
    ref_loss.backward()
    # the same pipeline in float64
    f64 = FakeDiffusionStage([f.double() for f in fields], torch.device("cpu"), f64_denoise)
    with torch.no_grad():
        anchor64 = f64.replay(None, segment=seg_cpu, params=params, step_indices=steps).log_probs
        f64.w.fill_(1.0002)
    new64 = f64.replay(None, segment=seg_cpu, params=params, step_indices=steps).log_probs
    elem64, m64 = olos.grpo_clip_loss(new64, anchor64, adv.double().reshape(-1, 1).expand_as(new64), 1e-4)
    loss64 = elem64.mean()
    grad_scale64 = mean_abs_term_gradient(elem64, f64.w)
    loss64.backward()

    stage = FakeDiffusionStage(fields, dev, FlowSDEStrategy().denoise)
    seg = types.SimpleNamespace(latents=latents.to(dev), sigmas=SIG.to(dev), sde_indices=sde_idx, sde_logp=None)
    algo = FlowGRPO(params=params, stage=stage, clip_range=1e-4, old_logp_source="replay")
    algo.prepare_segment(conditions={}, segment=seg)
    with torch.no_grad():
        stage.w.fill_(1.0002)
    res = algo.compute_loss_and_backward(conditions={}, segment=seg, advantages=adv.to(dev), training_progress=0.3,
                                         loss_scale=1.0)
    # the ratio is exp of a difference of two ~1 log-probs: 1e-7 of rounding in each is 1e-3 of a 1e-4
    # clip range, so no fp32 evaluation holds 1e-5 here; the bound is the fp32 reference's own distance
    # from the float64 value
    no_worse_than_fp32(res.loss, ref_loss, loss64, "loss", scale=elem64.abs().mean())
    no_worse_than_fp32(res.metrics["ratio_mean"], ref_m["ratio_mean"], m64["ratio_mean"], "ratio_mean")
    assert res.metrics["clip_range"] == 1e-4 and res.num_steps_or_tokens == 3
    no_worse_than_fp32(stage.w.grad, cpu.w.grad, f64.w.grad, "d loss / d w", scale=grad_scale64)
    rollout = FlowGRPO(params=params, stage=stage)
    with pytest.raises(RuntimeError, match="emitted no per-step log-probs"):
        rollout.prepare_segment(conditions={}, segment=types.SimpleNamespace(sde_indices=sde_idx, sde_logp=None))
    assert rollout.compute_loss_and_backward(
        conditions={}, segment=types.SimpleNamespace(sde_indices=None), advantages=adv, training_progress=0.0,
        loss_scale=1.0).has_backward is False
