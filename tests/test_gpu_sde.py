"""GPU parity of the fused SDE kernels (through the C ABI) against the CPU oracle."""

import math

import pytest
import torch

from oracle import schedule as osch
from oracle import sde as osde
from tests._util import BF16_RTOL, FP32_RTOL, assert_close

pytestmark = pytest.mark.gpu

# Oracle calls below pass ieee_sqrt=True: the scalar square roots are then correctly rounded on
# every host CPU, which is what the kernel computes, so element-wise outputs can be compared bit
# for bit.  test_plain_torch_oracle_within_tolerance compares with the unmodified torch chain.

SIG = osch.sigma_schedule(28, 3.0)
KINDS = ("flow", "dance", "cps")
DTYPES = (torch.float32, torch.bfloat16, torch.float16)


def strategy(kind):
    from unirl_amd import sde

    return sde.STRATEGIES[kind]()


def inputs(shape, seed, dtype=torch.float32, vdtype=None):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g).to(dtype)
    v = torch.randn(shape, generator=g).to(vdtype or dtype)
    n = torch.randn(shape, generator=g)
    return x, v, n


def logp_atol(kind, i, eta=0.7):
    """Each log-prob is a mean of O(1) terms that cancel to a small number; fp32 rounding of the
    terms bounds the attainable absolute accuracy (the reference's own sum carries the same)."""
    return 2e-6


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(2, 3, 4, 4), (3, 5, 7), (1, 1037), (8, 16, 32, 32), (5, 4, 33, 31)])
def test_sample_and_replay_match_oracle(dev, kind, dtype, shape):
    st = strategy(kind)
    x, v, n = inputs(shape, hash((kind, str(dtype), shape)) % 1000, dtype)
    rtol = FP32_RTOL if dtype == torch.float32 else BF16_RTOL
    for i in (0, 10, 27):
        ref_prev, ref_lp, ref_mean = osde.sde_denoise(kind, v, x, SIG[i], SIG[i + 1], eta=0.7, noise=n,
                                                      sigma_max=SIG[1], ieee_sqrt=True)
        prev, lp, mean = st.denoise(v.to(dev), x.to(dev), SIG[i].to(dev), SIG[i + 1].to(dev), eta=0.7,
                                    sigma_max=SIG[1].to(dev), noise=n.to(dev))
        assert prev.dtype == mean.dtype == lp.dtype == torch.float32 and lp.shape == (shape[0],)
        # element-wise outputs reproduce eager fp32 torch bit for bit
        assert torch.equal(mean.cpu(), ref_mean), f"mean differs at step {i}"
        assert torch.equal(prev.cpu(), ref_prev), f"prev differs at step {i}"
        assert_close(lp, ref_lp, rtol, logp_atol(kind, i), f"logp step {i}")
        # replay of the stored sample (stored in the trajectory dtype)
        stored = ref_prev.to(dtype)
        r_prev, r_lp, r_mean = osde.sde_denoise(kind, v, x, SIG[i], SIG[i + 1], eta=0.7, prev_sample=stored,
                                                sigma_max=SIG[1], ieee_sqrt=True)
        prev2, lp2, mean2 = st.denoise(v.to(dev), x.to(dev), SIG[i].to(dev), SIG[i + 1].to(dev), eta=0.7,
                                       prev_sample=stored.to(dev), sigma_max=float(SIG[1]))
        assert torch.equal(mean2.cpu(), r_mean) and torch.equal(prev2.cpu(), r_prev)
        assert_close(lp2, r_lp, rtol, logp_atol(kind, i), f"replay logp step {i}")


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_plain_torch_oracle_within_tolerance(dev, kind, dtype):
    """Against eager torch exactly as the reference runs it (torch.sqrt included): element-wise
    outputs within a few ulp, log-probs within the stated tolerance."""
    st = strategy(kind)
    x, v, n = inputs((4, 16, 32, 32), 77, dtype)
    rtol = FP32_RTOL if dtype == torch.float32 else BF16_RTOL
    exact = 0
    for i in range(0, 28, 3):
        ref_prev, ref_lp, ref_mean = osde.sde_denoise(kind, v, x, SIG[i], SIG[i + 1], eta=0.7, noise=n,
                                                      sigma_max=SIG[1])
        prev, lp, mean = st.denoise(v.to(dev), x.to(dev), SIG[i].to(dev), SIG[i + 1].to(dev), eta=0.7,
                                    sigma_max=SIG[1].to(dev), noise=n.to(dev))
        assert_close(mean, ref_mean, 1e-6, 1e-6, f"mean step {i}")
        if dtype == torch.float32:
            assert_close(prev, ref_prev, 1e-6, 1e-6, f"prev step {i}")
        else:  # a 1-ulp coefficient difference can flip the 16-bit rounding of single elements
            flips = (prev.cpu() != ref_prev).float().mean().item()
            assert flips < 1e-2, f"step {i}: {flips:.2%} of the rounded samples differ"
        assert_close(lp, ref_lp, rtol, 2e-6, f"logp step {i}")
        exact += int(torch.equal(prev.cpu(), ref_prev) and torch.equal(mean.cpu(), ref_mean))
    print(f"{kind} {dtype}: {exact}/10 steps bit-identical to this host's eager torch")


@pytest.mark.parametrize("kind", KINDS)
def test_eta_zero_returns_no_logprob(dev, kind):
    st = strategy(kind)
    x, v, n = inputs((2, 4, 8, 8), 3)
    ref_prev, ref_lp, ref_mean = osde.sde_denoise(kind, v, x, SIG[5], SIG[6], eta=0.0, noise=n, ieee_sqrt=True)
    prev, lp, mean = st.denoise(v.to(dev), x.to(dev), SIG[5].to(dev), SIG[6].to(dev), eta=0.0)
    assert lp is None and ref_lp is None
    assert torch.equal(mean.cpu(), ref_mean) and torch.equal(prev.cpu(), ref_prev)
    prev, lp, _ = st.denoise(v.to(dev), x.to(dev), SIG[5].to(dev), SIG[6].to(dev), eta=5e-8, noise=n.to(dev))
    assert lp is None


def test_mixed_dtypes_and_float64_inputs(dev):
    st = strategy("flow")
    # bf16 velocity (autocast model output) on an fp32 latent, and the reverse
    for xd, vd in ((torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32), (torch.float16, torch.bfloat16),
                   (torch.float64, torch.float64)):
        x, v, n = inputs((3, 4, 16, 16), 4, xd, vd)
        ref = osde.sde_denoise("flow", v, x, SIG[10], SIG[11], eta=0.7, noise=n, sigma_max=SIG[1], ieee_sqrt=True)
        got = st.denoise(v.to(dev), x.to(dev), SIG[10].to(dev), SIG[11].to(dev), eta=0.7, sigma_max=SIG[1],
                         noise=n.to(dev))
        assert torch.equal(got[0].cpu(), ref[0]) and torch.equal(got[2].cpu(), ref[2])
        assert_close(got[1], ref[1], BF16_RTOL, 2e-6, f"logp {xd} {vd}")


def test_per_sample_sigma(dev):
    st = strategy("flow")
    x, v, n = inputs((4, 2, 8, 8), 5)
    idx = [0, 3, 10, 27]
    s, sn = SIG[idx], SIG[[i + 1 for i in idx]]
    ref = osde.sde_denoise("flow", v, x, s, sn, eta=0.7, noise=n, sigma_max=SIG[1], ieee_sqrt=True)
    got = st.denoise(v.to(dev), x.to(dev), s.to(dev), sn.to(dev), eta=0.7, sigma_max=SIG[1].to(dev), noise=n.to(dev))
    assert torch.equal(got[0].cpu(), ref[0]) and torch.equal(got[2].cpu(), ref[2])
    assert_close(got[1], ref[1], FP32_RTOL, 2e-6, "logp")
    # [B,1,1,1] sigmas are the same thing; a mismatched count is an error
    got2 = st.denoise(v.to(dev), x.to(dev), s.reshape(4, 1, 1, 1).to(dev), sn.reshape(4, 1, 1, 1).to(dev), eta=0.7,
                      sigma_max=SIG[1].to(dev), noise=n.to(dev))
    assert torch.equal(got2[1], got[1])
    with pytest.raises(ValueError):
        st.denoise(v.to(dev), x.to(dev), s[:3].to(dev), sn[:3].to(dev), eta=0.7, noise=n.to(dev))


def test_noncontiguous_and_misaligned_views(dev):
    st = strategy("flow")
    x, v, n = inputs((2, 6, 10, 12), 6)
    xd, vd, nd = x.to(dev), v.to(dev), n.to(dev)
    ref = osde.sde_denoise("flow", v.transpose(2, 3), x.transpose(2, 3), SIG[8], SIG[9], eta=0.7,
                           noise=n.transpose(2, 3), sigma_max=SIG[1], ieee_sqrt=True)
    got = st.denoise(vd.transpose(2, 3), xd.transpose(2, 3), SIG[8].to(dev), SIG[9].to(dev), eta=0.7,
                     sigma_max=SIG[1], noise=nd.transpose(2, 3))
    assert torch.equal(got[0].cpu(), ref[0]) and torch.equal(got[2].cpu(), ref[2])
    # storage offset of one element: 4-byte aligned only -> scalar path
    big = torch.randn(2 * 720 + 1, generator=torch.Generator().manual_seed(7))
    xo = big[1:].reshape(2, 720)
    ref = osde.sde_denoise("flow", xo * 0.5, xo, SIG[8], SIG[9], eta=0.7, noise=None, sigma_max=SIG[1], ieee_sqrt=True)
    bigd = big.to(dev)
    xod = bigd[1:].reshape(2, 720)
    assert xod.data_ptr() % 16 != 0
    from unirl_amd import ops

    got = ops.sde_step_logp(xod * 0.5, xod, SIG[8], SIG[9], kind="flow", eta=0.7, noise=None, sigma_max=SIG[1])
    assert torch.equal(got[0].cpu(), ref[0]) and torch.equal(got[2].cpu(), ref[2])
    assert_close(got[1], ref[1], FP32_RTOL, 2e-6, "logp")


def test_many_samples_span_several_launches(dev):
    # more samples than ticket counters: the entry point splits the batch
    from unirl_amd import ops

    B, D = 20000, 24
    x, v, n = inputs((B, D), 8)
    ref = osde.sde_denoise("flow", v, x, SIG[10], SIG[11], eta=0.7, noise=n, sigma_max=SIG[1], ieee_sqrt=True)
    got = ops.sde_step_logp(v.to(dev), x.to(dev), SIG[10], SIG[11], kind="flow", eta=0.7, noise=n.to(dev),
                            sigma_max=SIG[1])
    assert torch.equal(got[0].cpu(), ref[0]) and torch.equal(got[2].cpu(), ref[2])
    assert_close(got[1], ref[1], FP32_RTOL, 2e-6, "logp")


def test_sum_reduction_option(dev):
    from unirl_amd import ops

    x, v, n = inputs((3, 4, 8, 8), 9)
    _, lp_mean, _ = ops.sde_step_logp(v.to(dev), x.to(dev), SIG[10], SIG[11], eta=0.7, noise=n.to(dev),
                                      sigma_max=SIG[1])
    _, lp_sum, _ = ops.sde_step_logp(v.to(dev), x.to(dev), SIG[10], SIG[11], eta=0.7, noise=n.to(dev),
                                     sigma_max=SIG[1], logp_sum=True)
    assert_close(lp_sum, lp_mean.double() * 256, 1e-6, 0, "sum = mean * D")


def test_repeated_calls_are_deterministic(dev):
    st = strategy("flow")
    x, v, n = inputs((8, 16, 64, 64), 10)
    xd, vd, nd = x.to(dev), v.to(dev), n.to(dev)
    first = st.denoise(vd, xd, SIG[10].to(dev), SIG[11].to(dev), eta=0.7, sigma_max=SIG[1].to(dev), noise=nd)
    for _ in range(5):
        again = st.denoise(vd, xd, SIG[10].to(dev), SIG[11].to(dev), eta=0.7, sigma_max=SIG[1].to(dev), noise=nd)
        assert torch.equal(again[1], first[1]) and torch.equal(again[0], first[0])


def test_sampling_draws_noise_on_device(dev):
    st = strategy("flow")
    x, v, _ = inputs((4, 16, 32, 32), 11)
    torch.manual_seed(123)
    prev, lp, mean = st.denoise(v.to(dev), x.to(dev), SIG[10].to(dev), SIG[11].to(dev), eta=0.7, sigma_max=SIG[1])
    s, sn = float(SIG[10]), float(SIG[11])
    sv = math.sqrt(s / (1 - s)) * 0.7 * math.sqrt(-(sn - s))
    z = ((prev - mean) / sv).cpu()
    assert abs(float(z.mean())) < 0.02 and abs(float(z.std()) - 1.0) < 0.02
    expect = -0.5 - math.log(sv) - 0.5 * math.log(2 * math.pi)
    assert abs(float(lp.mean()) - expect) < 0.02


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("mode", ["replay", "sample"])
def test_backward_matches_autograd_of_oracle(dev, kind, mode):
    st = strategy(kind)
    x, v, n = inputs((3, 4, 8, 8), 12)
    prev_store = osde.sde_denoise(kind, v, x, SIG[10], SIG[11], eta=0.7, noise=n, sigma_max=SIG[1], ieee_sqrt=True)[0]
    g = torch.Generator().manual_seed(13)
    w_lp, w_mean, w_prev = torch.randn(3, generator=g), torch.randn(x.shape, generator=g), torch.randn(x.shape, generator=g)

    def objective(outs, wl, wm, wp):
        prev, lp, mean = outs
        val = (lp * wl).sum() + (mean * wm).sum() * 1e-3
        if mode == "sample":
            val = val + (prev * wp).sum() * 1e-3
        return val

    vr, xr = v.clone().requires_grad_(True), x.clone().requires_grad_(True)
    kw = dict(eta=0.7, sigma_max=SIG[1])
    kw.update(dict(prev_sample=prev_store) if mode == "replay" else dict(noise=n))
    objective(osde.sde_denoise(kind, vr, xr, SIG[10], SIG[11], **kw, ieee_sqrt=True), w_lp, w_mean, w_prev).backward()

    vg, xg = v.to(dev).requires_grad_(True), x.to(dev).requires_grad_(True)
    kwd = dict(eta=0.7, sigma_max=SIG[1].to(dev))
    kwd.update(dict(prev_sample=prev_store.to(dev)) if mode == "replay" else dict(noise=n.to(dev)))
    outs = st.denoise(vg, xg, SIG[10].to(dev), SIG[11].to(dev), **kwd)
    objective(outs, w_lp.to(dev), w_mean.to(dev), w_prev.to(dev)).backward()
    scale_v, scale_x = float(vr.grad.abs().max()), float(xr.grad.abs().max())
    assert_close(vg.grad, vr.grad, 1e-4, 1e-5 * scale_v, "grad noise_pred")
    assert_close(xg.grad, xr.grad, 1e-4, 1e-5 * scale_x, "grad sample")


def test_backward_bf16_inputs_return_bf16_grads(dev):
    st = strategy("flow")
    x, v, n = inputs((2, 4, 8, 8), 14, torch.bfloat16)
    prev_store = osde.sde_denoise("flow", v, x, SIG[10], SIG[11], eta=0.7, noise=n, sigma_max=SIG[1], ieee_sqrt=True)[0].bfloat16()
    vr = v.clone().requires_grad_(True)
    osde.sde_denoise("flow", vr, x, SIG[10], SIG[11], eta=0.7, prev_sample=prev_store, sigma_max=SIG[1], ieee_sqrt=True)[1].sum().backward()
    vg = v.to(dev).requires_grad_(True)
    st.denoise(vg, x.to(dev), SIG[10].to(dev), SIG[11].to(dev), eta=0.7, prev_sample=prev_store.to(dev),
               sigma_max=SIG[1])[1].sum().backward()
    assert vg.grad.dtype == torch.bfloat16
    assert_close(vg.grad.float(), vr.grad.float(), 1e-2, 1e-2 * float(vr.grad.float().abs().max()), "bf16 grad")


def test_step_method_contract(dev):
    st = strategy("flow")
    x, v, n = inputs((2, 4, 8, 8), 15)
    s, sn = SIG[10].reshape(1, 1, 1, 1), SIG[11].reshape(1, 1, 1, 1)
    ref_prev, ref_mean, ref_sv = osde.sde_step("flow", v, x, s, sn, 0.7, x * 0.9, None, SIG[1], True)
    prev, mean, sv = st.step(v.to(dev), x.to(dev), s.to(dev), sn.to(dev), eta=0.7, prev_sample=(x * 0.9).to(dev),
                             sigma_max=SIG[1].to(dev))
    assert torch.equal(mean.cpu(), ref_mean) and torch.equal(prev.cpu(), ref_prev)
    assert_close(sv, ref_sv, 1e-6, 0, "std_var")
    lp = st.compute_log_prob(prev, mean, sv)
    assert_close(lp, osde.elem_log_prob("flow", ref_prev, ref_mean, ref_sv), 1e-5, 1e-5, "elem log-prob")


# ---------------------------------------------------------------- multi-step rollout
@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rollout_equals_chained_oracle(dev, kind, dtype):
    from unirl_amd import sde

    g = torch.Generator().manual_seed(16)
    x0 = torch.randn(3, 40, 64, generator=g).to(dtype)
    S = 6
    vs = [torch.randn(x0.shape, generator=g).to(dtype) for _ in range(S)]
    ns = [torch.randn(x0.shape, generator=g) for _ in range(S)]
    etas = [0.7, 0.7, 0.0, 0.7, 0.7, 0.7]
    rx, rlp, rtraj = osde.sde_rollout(kind, x0, vs, ns, SIG, etas, ieee_sqrt=True)
    x, lp, traj = sde.sde_rollout(sde.STRATEGIES[kind](), x0.to(dev), [t.to(dev) for t in vs], SIG.to(dev), etas,
                                  noises=[t.to(dev) for t in ns], return_trajectory=True)
    assert torch.equal(x.cpu(), rx) and torch.equal(traj.cpu(), rtraj)
    assert bool(torch.isnan(lp[:, 2]).all())
    assert_close(lp, rlp, FP32_RTOL if dtype == torch.float32 else BF16_RTOL, 2e-6, "rollout logp")


def test_rollout_equals_single_step_kernel_calls(dev):
    from unirl_amd import sde

    st = sde.FlowSDEStrategy()
    g = torch.Generator().manual_seed(17)
    x0 = torch.randn(4, 1037, generator=g).to(dev)  # odd length: scalar path
    S = 5
    vs = [torch.randn(x0.shape, generator=g).to(dev) for _ in range(S)]
    ns = [torch.randn(x0.shape, generator=g).to(dev) for _ in range(S)]
    xf, lp, _ = sde.sde_rollout(st, x0, vs, SIG.to(dev), 0.7, noises=ns)
    x = x0
    for k in range(S):
        x, l1, _ = st.denoise(vs[k], x, SIG[k].to(dev), SIG[k + 1].to(dev), eta=0.7, sigma_max=SIG[1].to(dev),
                              noise=ns[k])
        assert_close(lp[:, k], l1, 1e-6, 1e-7, f"step {k}")
    assert torch.equal(xf, x)


def test_rollout_argument_errors(dev):
    from unirl_amd import ops

    x0 = torch.randn(2, 64, device=dev)
    v = [torch.randn(2, 64, device=dev)]
    with pytest.raises(ValueError):
        ops.sde_rollout_logp(x0, v * 65, [None] * 65, torch.linspace(1, 0, 66), 0.7)
    with pytest.raises(ValueError):
        ops.sde_rollout_logp(x0, v, [None], SIG[:1], 0.7)
    with pytest.raises(ValueError):
        ops.sde_rollout_logp(x0, v, [None, None], SIG, 0.7)


# ---------------------------------------------------------------- benchmark shapes
def test_config1_sd3_shape(dev):
    """fp32 [8,16,128,128], step 10 of 28, shift 3, eta 0.7 (seed 1001)."""
    st = strategy("flow")
    g = torch.Generator().manual_seed(1001)
    x, v, n = (torch.randn(8, 16, 128, 128, generator=g) for _ in range(3))
    ref = osde.sde_denoise("flow", v, x, SIG[10], SIG[11], eta=0.7, noise=n, sigma_max=SIG[1], ieee_sqrt=True)
    got = st.denoise(v.to(dev), x.to(dev), SIG[10].to(dev), SIG[11].to(dev), eta=0.7, sigma_max=SIG[1].to(dev),
                     noise=n.to(dev))
    assert torch.equal(got[0].cpu(), ref[0]) and torch.equal(got[2].cpu(), ref[2])
    assert_close(got[1], ref[1], FP32_RTOL, 0.0, "config-1 logp (pure relative)")
    # size-independent property: the mean log-prob of N(0,1) noise
    sv = math.sqrt(float(SIG[10]) / (1 - float(SIG[10]))) * 0.7 * math.sqrt(float(SIG[10]) - float(SIG[11]))
    expect = -0.5 - math.log(sv) - 0.5 * math.log(2 * math.pi)
    assert abs(float(got[1].mean()) - expect) < 5 * math.sqrt(0.5 / (8 * 262144))


def test_config5_rollout_shape(dev):
    """fp32 [16,4096,64], 10 steps from step 0 (sigma == 1 branch), eta 0.7 (seed 1005)."""
    from unirl_amd import sde

    g = torch.Generator().manual_seed(1005)
    x0 = torch.randn(16, 4096, 64, generator=g)
    vs = [torch.randn(x0.shape, generator=g) for _ in range(10)]
    ns = [torch.randn(x0.shape, generator=g) for _ in range(10)]
    rx, rlp, _ = osde.sde_rollout("flow", x0, vs, ns, SIG, 0.7, ieee_sqrt=True)
    x, lp, _ = sde.sde_rollout(sde.FlowSDEStrategy(), x0.to(dev), [t.to(dev) for t in vs], SIG.to(dev), 0.7,
                               noises=[t.to(dev) for t in ns])
    assert lp.shape == (16, 10)
    assert torch.equal(x.cpu(), rx)
    assert_close(lp, rlp, FP32_RTOL, 1e-7, "config-5 logp")


def test_wan_video_shape_bf16_replay(dev):
    """WAN2.1-shaped bf16 latents [2,16,21,60,104]: replay of a stored bf16 trajectory."""
    st = strategy("flow")
    g = torch.Generator().manual_seed(1004)
    shape = (2, 16, 21, 60, 104)
    x = torch.randn(shape, generator=g).bfloat16()
    v = torch.randn(shape, generator=g).bfloat16()
    n = torch.randn(shape, generator=g)
    ref_s = osde.sde_denoise("flow", v, x, SIG[4], SIG[5], eta=0.7, noise=n, sigma_max=SIG[1], ieee_sqrt=True)
    stored = ref_s[0].bfloat16()
    ref = osde.sde_denoise("flow", v, x, SIG[4], SIG[5], eta=0.7, prev_sample=stored, sigma_max=SIG[1], ieee_sqrt=True)
    got = st.denoise(v.to(dev), x.to(dev), SIG[4].to(dev), SIG[5].to(dev), eta=0.7, prev_sample=stored.to(dev),
                     sigma_max=SIG[1].to(dev))
    assert torch.equal(got[2].cpu(), ref[2]) and torch.equal(got[0].cpu(), ref[0])
    assert_close(got[1], ref[1], BF16_RTOL, 0.0, "wan logp")


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("traj_dtype", DTYPES)
@pytest.mark.parametrize("shape", [(3, 4, 8, 8), (2, 5, 7), (4, 16, 16, 16)])
def test_stage_loops_on_stacks_match_oracle(dev, kind, traj_dtype, shape):
    """The reference's diffuse loop (latents.to(trajectory_dtype) stacked as [B,K,...],
    unirl/models/sd3/diffusion.py:366-406) and its replay loop (latents_at views in,
    stack(log_probs), stack(means).to(trajectory_dtype) out, :467-497), run with denoise_into on
    views of the stacks and compared with the oracle's step-by-step eager chain."""
    from unirl_amd import sde

    st = strategy(kind)
    B = shape[0]
    steps = [0, 1, 2, 5]
    g = torch.Generator().manual_seed(hash((kind, str(traj_dtype), shape)) % 997)
    x0 = torch.randn(shape, generator=g).to(traj_dtype)
    vs = [torch.randn(shape, generator=g).to(traj_dtype) for _ in steps]
    ns = [torch.randn(shape, generator=g) for _ in steps]
    rtol = FP32_RTOL if traj_dtype == torch.float32 else BF16_RTOL

    # oracle: rollout, keeping every latent in the trajectory dtype
    ref_lat, ref_lp = [x0], []
    for j, i in enumerate(steps):
        prev, lp, _ = osde.sde_denoise(kind, vs[j], ref_lat[-1], SIG[i], SIG[i + 1], eta=0.7, noise=ns[j],
                                       sigma_max=SIG[1], ieee_sqrt=True)
        ref_lat.append(prev.to(traj_dtype))
        ref_lp.append(lp)
    ref_stack = torch.stack(ref_lat, dim=1)
    ref_lp = torch.stack(ref_lp, dim=1)

    # device: one stack [B, K, ...] in the trajectory dtype, written slot by slot
    K = len(steps) + 1
    stack = torch.zeros((B, K) + tuple(shape[1:]), dtype=traj_dtype, device=dev)
    stack[:, 0] = x0.to(dev)
    logp = torch.full((B, len(steps)), float("nan"), device=dev)
    for j, i in enumerate(steps):
        ok = st.denoise_into(vs[j].to(dev), stack[:, j], SIG[i].to(dev), SIG[i + 1].to(dev), eta=0.7,
                             sigma_max=SIG[1].to(dev), noise=ns[j].to(dev), prev_out=stack[:, j + 1],
                             logp_out=logp[:, j])
        assert ok
    assert torch.equal(stack.cpu(), ref_stack), "trajectory stack differs"
    assert_close(logp, ref_lp, rtol, 2e-6, "rollout log-probs")

    # replay: fresh velocities, stored latents read in place, means and log-probs written in place
    v2 = [torch.randn(shape, generator=g).to(traj_dtype) for _ in steps]
    indices = torch.arange(K)
    ref_means, ref_rlp = [], []
    for j, i in enumerate(steps):
        _, lp, mean = osde.sde_denoise(kind, v2[j], ref_stack[:, j], SIG[i], SIG[i + 1], eta=0.7,
                                       prev_sample=ref_stack[:, j + 1], sigma_max=SIG[1], ieee_sqrt=True)
        ref_means.append(mean)
        ref_rlp.append(lp)
    ref_means = torch.stack(ref_means, dim=1).to(traj_dtype)
    ref_rlp = torch.stack(ref_rlp, dim=1)
    means = torch.zeros((B, len(steps)) + tuple(shape[1:]), dtype=traj_dtype, device=dev)
    rlp = torch.zeros((B, len(steps)), device=dev)
    for j, i in enumerate(steps):
        st.denoise_into(v2[j].to(dev), sde.latents_at(stack, indices, j), SIG[i].to(dev), SIG[i + 1].to(dev),
                        eta=0.7, prev_sample=sde.latents_at(stack, indices, j + 1), sigma_max=float(SIG[1]),
                        mean_out=means[:, j], logp_out=rlp[:, j])
    assert torch.equal(means.cpu(), ref_means), "replayed means differ"
    assert_close(rlp, ref_rlp, rtol, 2e-6, "replay log-probs")
    # eta = 0: Euler step, log-prob column untouched
    before = rlp.clone()
    assert not st.denoise_into(v2[0].to(dev), stack[:, 0], SIG[0].to(dev), SIG[1].to(dev), eta=0.0,
                               sigma_max=float(SIG[1]), mean_out=means[:, 0], logp_out=rlp[:, 0])
    assert torch.equal(rlp, before)
    with pytest.raises(KeyError):
        sde.latents_at(stack, indices, K + 3)
    with pytest.raises(ValueError):
        st.denoise_into(v2[0].to(dev), stack[:, 0], SIG[0].to(dev), SIG[1].to(dev), eta=0.7,
                        mean_out=means[:, 0].transpose(-1, -2), logp_out=rlp[:, 0])


@pytest.mark.parametrize("kind", KINDS)
def test_inputs_broadcast_over_the_samples(dev, kind):
    """noise / noise_pred / sample given as expand(B, ...) views (sample stride 0): every sample
    must see the one block, and nothing past it is read."""
    st = strategy(kind)
    B, shape = 5, (1, 4, 24, 24)
    g = torch.Generator().manual_seed(77)
    x1, v, n1 = (torch.randn(shape, generator=g) for _ in range(3))
    v = torch.randn((B,) + shape[1:], generator=g)
    xe, ne = x1.expand(B, *shape[1:]), n1.expand(B, *shape[1:])
    ref_prev, ref_lp, ref_mean = osde.sde_denoise(kind, v, xe, SIG[3], SIG[4], eta=0.7, noise=ne, sigma_max=SIG[1],
                                                  ieee_sqrt=True)
    prev = torch.empty((B,) + shape[1:], device=dev)
    mean = torch.empty_like(prev)
    lp = torch.empty(B, device=dev)
    # the expanded operands sit at the very end of their allocations
    xd, nd = x1.to(dev).expand(B, *shape[1:]), n1.to(dev).expand(B, *shape[1:])
    assert xd.stride(0) == 0 and nd.stride(0) == 0
    assert st.denoise_into(v.to(dev), xd, SIG[3].to(dev), SIG[4].to(dev), eta=0.7, sigma_max=SIG[1].to(dev),
                           noise=nd, prev_out=prev, mean_out=mean, logp_out=lp)
    assert torch.equal(prev.cpu(), ref_prev) and torch.equal(mean.cpu(), ref_mean)
    assert_close(lp, ref_lp, FP32_RTOL, 2e-6, "log-prob with broadcast inputs")
    # replay with a broadcast velocity
    ve = v[:1].expand(B, *shape[1:])
    _, ref_lp2, ref_mean2 = osde.sde_denoise(kind, ve, xe, SIG[3], SIG[4], eta=0.7, prev_sample=ref_prev,
                                             sigma_max=SIG[1], ieee_sqrt=True)
    st.denoise_into(v[:1].to(dev).expand(B, *shape[1:]), xd, SIG[3].to(dev), SIG[4].to(dev), eta=0.7,
                    sigma_max=SIG[1].to(dev), prev_sample=ref_prev.to(dev), mean_out=mean, logp_out=lp)
    assert torch.equal(mean.cpu(), ref_mean2)
    assert_close(lp, ref_lp2, FP32_RTOL, 2e-6, "replay log-prob with broadcast inputs")
