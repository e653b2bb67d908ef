"""The batched [B, S'] replay (one launch over all (sample, step) transitions) against S' calls of
the oracle's single-step replay -- the loop of unirl/models/sd3/diffusion.py:467-497 and what
unirl/algorithms/flowdppo.py:286-302 consumes."""

import pytest
import torch

from oracle import schedule as osch
from oracle import sde as osde
from tests._util import BF16_RTOL, FP32_RTOL, assert_close

pytestmark = pytest.mark.gpu

SIG = osch.sigma_schedule(28, 3.0)
KINDS = ("flow", "dance", "cps")


def strategy(kind):
    from unirl_amd import sde

    return sde.STRATEGIES[kind]()


def make_case(B, K, tail, steps, stored, traj_dtype, v_dtype, seed):
    """A trajectory stack whose slot k holds the latent of step stored[k], fresh velocities for
    `steps`, and the oracle's per-step replay (log-probs [B,S'], means [B,S',...] in traj dtype)."""
    g = torch.Generator().manual_seed(seed)
    stack = torch.randn((B, K) + tail, generator=g).to(traj_dtype)
    v = torch.randn((B, len(steps)) + tail, generator=g).to(v_dtype)
    return stack, v


def oracle_replay(kind, stack, v, steps, stored, sigmas, traj_dtype, eta=0.7):
    lps, means = [], []
    for j, i in enumerate(steps):
        x = stack[:, stored.index(i)]
        prev = stack[:, stored.index(i + 1)]
        _, lp, mean = osde.sde_denoise(kind, v[:, j], x, sigmas[i], sigmas[i + 1], eta=eta, prev_sample=prev,
                                       sigma_max=sigmas[1], ieee_sqrt=True)
        lps.append(lp)
        means.append(mean)
    return torch.stack(lps, dim=1), torch.stack(means, dim=1).to(traj_dtype)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("traj_dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_replay_steps_matches_per_step_oracle(dev, kind, traj_dtype):
    from unirl_amd import sde

    st = strategy(kind)
    B, tail = 3, (4, 12, 10)
    stored = [0, 1, 2, 3, 5, 6, 9, 10]      # slots hold these steps (not all consecutive)
    steps = [2, 0, 5, 9]                     # trained steps, in no particular order
    stack, v = make_case(B, len(stored), tail, steps, stored, traj_dtype, traj_dtype, 31)
    ref_lp, ref_means = oracle_replay(kind, stack, v, steps, stored, SIG, traj_dtype)
    slot_x, slot_p = sde.replay_slots(stored, steps)
    sig = torch.stack([SIG[i] for i in steps]).to(dev)
    sig_n = torch.stack([SIG[i + 1] for i in steps]).to(dev)
    lp, means = st.replay_steps(v.to(dev), stack.to(dev), slot_x, slot_p, sig, sig_n, eta=0.7,
                                sigma_max=SIG[1].to(dev))
    assert means.dtype == traj_dtype and tuple(means.shape) == (B, len(steps)) + tail
    assert torch.equal(means.cpu(), ref_means), "replayed means differ"
    rtol = FP32_RTOL if traj_dtype == torch.float32 else BF16_RTOL
    assert_close(lp, ref_lp, rtol, 2e-6, "replayed log-probs")
    # the same through one denoise_into call per step: bit-identical, it is the same arithmetic
    lp2 = torch.zeros_like(lp)
    means2 = torch.zeros_like(means)
    sd = stack.to(dev)
    for j, i in enumerate(steps):
        st.denoise_into(v[:, j].to(dev), sd[:, slot_x[j]], SIG[i].to(dev), SIG[i + 1].to(dev), eta=0.7,
                        prev_sample=sd[:, slot_p[j]], sigma_max=SIG[1].to(dev), mean_out=means2[:, j],
                        logp_out=lp2[:, j])
    assert torch.equal(means2, means)
    assert_close(lp2, lp, 1e-6, 1e-7, "one launch vs a launch per step")


def test_replay_steps_step_major_velocities_and_fp32_means(dev):
    """Velocities from a model pass over the steps stacked into the batch come as [S', B, ...];
    means may be asked for in fp32 from a 16-bit stack."""
    from unirl_amd import sde

    st = strategy("flow")
    B, tail = 4, (16, 8, 8)
    stored = list(range(8))
    steps = [1, 3, 4]
    stack, v = make_case(B, len(stored), tail, steps, stored, torch.bfloat16, torch.bfloat16, 32)
    ref_lp, _ = oracle_replay("flow", stack, v, steps, stored, SIG, torch.bfloat16)
    ref_means32 = torch.stack(
        [osde.sde_denoise("flow", v[:, j], stack[:, i], SIG[i], SIG[i + 1], eta=0.7, prev_sample=stack[:, i + 1],
                          sigma_max=SIG[1], ieee_sqrt=True)[2] for j, i in enumerate(steps)], dim=1)
    slot_x, slot_p = sde.replay_slots(stored, steps)
    v_sm = v.transpose(0, 1).contiguous().to(dev)  # [S', B, ...]
    lp, means = st.replay_steps(v_sm, stack.to(dev), slot_x, slot_p, [float(SIG[i]) for i in steps],
                                [float(SIG[i + 1]) for i in steps], eta=0.7, sigma_max=float(SIG[1]),
                                step_major=True, means_dtype=torch.float32)
    assert means.dtype == torch.float32
    assert torch.equal(means.cpu(), ref_means32)
    assert_close(lp, ref_lp, BF16_RTOL, 2e-6, "log-probs, step-major velocities")
    # a permuted view of a [S', B, ...] tensor used as [B, S', ...]: read in place through its strides
    lp_v, means_v = st.replay_steps(v_sm.transpose(0, 1), stack.to(dev), slot_x, slot_p, [float(SIG[i]) for i in steps],
                                    [float(SIG[i + 1]) for i in steps], eta=0.7, sigma_max=float(SIG[1]),
                                    means_dtype=torch.float32)
    assert torch.equal(lp_v, lp) and torch.equal(means_v, means)


@pytest.mark.parametrize("kind", KINDS)
def test_replay_steps_backward_matches_autograd_of_oracle(dev, kind):
    from unirl_amd import sde

    st = strategy(kind)
    B, tail = 2, (3, 6, 8)
    stored = [0, 1, 2, 3, 4]
    steps = [0, 2, 3]
    g = torch.Generator().manual_seed(33)
    stack = torch.randn((B, len(stored)) + tail, generator=g)
    v = torch.randn((B, len(steps)) + tail, generator=g)
    w_lp = torch.randn(B, len(steps), generator=g)
    w_mean = torch.randn((B, len(steps)) + tail, generator=g)
    # oracle: autograd through the eager chain, step by step
    v_ref = v.clone().requires_grad_(True)
    total = 0.0
    for j, i in enumerate(steps):
        _, lp, mean = osde.sde_denoise(kind, v_ref[:, j], stack[:, i], SIG[i], SIG[i + 1], eta=0.7,
                                       prev_sample=stack[:, i + 1], sigma_max=SIG[1])
        total = total + (lp * w_lp[:, j]).sum() + (mean * w_mean[:, j]).sum()
    total.backward()
    slot_x, slot_p = sde.replay_slots(stored, steps)
    v_dev = v.to(dev).requires_grad_(True)
    sig = torch.stack([SIG[i] for i in steps]).to(dev)
    sig_n = torch.stack([SIG[i + 1] for i in steps]).to(dev)
    lp, means = st.replay_steps(v_dev, stack.to(dev), slot_x, slot_p, sig, sig_n, eta=0.7, sigma_max=SIG[1].to(dev))
    ((lp * w_lp.to(dev)).sum() + (means * w_mean.to(dev)).sum()).backward()
    assert_close(v_dev.grad, v_ref.grad, 1e-4, 1e-6 * float(v_ref.grad.abs().max()), "grad wrt noise_pred")
    # log-prob gradient alone (what the Flow-DPPO / FlowGRPO losses send), bf16 velocities: bf16 gradient
    v16 = v.bfloat16().to(dev).requires_grad_(True)
    lp16, _ = st.replay_steps(v16, stack.bfloat16().to(dev), slot_x, slot_p, sig, sig_n, eta=0.7,
                              sigma_max=SIG[1].to(dev))
    (lp16 * w_lp.to(dev)).sum().backward()
    assert v16.grad.dtype == torch.bfloat16 and v16.grad.shape == v16.shape
    v_ref2 = v.bfloat16().float().requires_grad_(True)
    total = 0.0
    for j, i in enumerate(steps):
        _, lp, _ = osde.sde_denoise(kind, v_ref2[:, j], stack.bfloat16()[:, i], SIG[i], SIG[i + 1], eta=0.7,
                                    prev_sample=stack.bfloat16()[:, i + 1], sigma_max=SIG[1])
        total = total + (lp * w_lp[:, j]).sum()
    total.backward()
    assert_close(v16.grad.float(), v_ref2.grad, 1e-2, 1e-2 * float(v_ref2.grad.abs().max()), "bf16 grad wrt noise_pred")


def test_replay_steps_sd3_shape_three_steps(dev):
    """SD3 recipe shape: B = 8, [16,128,128] latents in a bf16 trajectory of 10 steps, S' = 3."""
    from unirl_amd import sde

    st = strategy("flow")
    sig = osch.sigma_schedule(10, 3.0)
    B, tail = 8, (16, 128, 128)
    stored = list(range(11))
    steps = [0, 2, 4]
    stack, v = make_case(B, len(stored), tail, steps, stored, torch.bfloat16, torch.bfloat16, 34)
    ref_lp, ref_means = oracle_replay("flow", stack, v, steps, stored, sig, torch.bfloat16)
    slot_x, slot_p = sde.replay_slots(stored, steps)
    lp, means = st.replay_steps(v.to(dev), stack.to(dev), slot_x, slot_p, [float(sig[i]) for i in steps],
                                [float(sig[i + 1]) for i in steps], eta=0.7, sigma_max=float(sig[1]))
    assert torch.equal(means.cpu(), ref_means)
    assert_close(lp, ref_lp, BF16_RTOL, 2e-6, "SD3-shape log-probs")


def test_replay_steps_wan_shape_seven_steps(dev):
    """WAN recipe shape: B = 2, [16,21,60,104] video latents in an fp16 trajectory, all 7 first-half
    steps of a 14-step shift-5 schedule trained."""
    from unirl_amd import sde

    st = strategy("flow")
    sig = osch.sigma_schedule(14, 5.0)
    B, tail = 2, (16, 21, 60, 104)
    stored = list(range(15))
    steps = list(range(7))
    stack, v = make_case(B, len(stored), tail, steps, stored, torch.float16, torch.bfloat16, 35)
    ref_lp, ref_means = oracle_replay("flow", stack, v, steps, stored, sig, torch.float16)
    slot_x, slot_p = sde.replay_slots(stored, steps)
    lp, means = st.replay_steps(v.to(dev), stack.to(dev), slot_x, slot_p, [float(sig[i]) for i in steps],
                                [float(sig[i + 1]) for i in steps], eta=0.7, sigma_max=float(sig[1]))
    assert means.dtype == torch.float16
    assert torch.equal(means.cpu(), ref_means)
    assert_close(lp, ref_lp, BF16_RTOL, 2e-6, "WAN-shape log-probs")


def test_replay_steps_argument_errors(dev):
    from unirl_amd import sde

    st = strategy("flow")
    stack = torch.zeros(2, 4, 8, 8, device=dev)
    v = torch.zeros(2, 2, 8, 8, device=dev)
    s2 = [0.9, 0.8]
    with pytest.raises(RuntimeError, match="stochastic"):
        st.replay_steps(v, stack, [0, 1], [1, 2], s2, s2, eta=0.0)
    with pytest.raises(ValueError, match="outside the stack"):
        st.replay_steps(v, stack, [0, 4], [1, 2], s2, s2, eta=0.7)
    with pytest.raises(ValueError, match="noise_pred"):
        st.replay_steps(v[:, :1], stack, [0, 1], [1, 2], s2, s2, eta=0.7)
    with pytest.raises(ValueError, match="one value per step"):
        st.replay_steps(v, stack, [0, 1], [1, 2], [0.9], s2, eta=0.7)
    with pytest.raises(KeyError):
        sde.replay_slots([0, 1, 2], [2])  # step 3 is not stored
    with pytest.raises(RuntimeError, match="HIP device"):
        st.replay_steps(v.cpu(), stack.cpu(), [0, 1], [1, 2], s2, s2, eta=0.7)
    # zero samples: empty outputs, no launch
    lp, means = st.replay_steps(v[:0], stack[:0], [0, 1], [1, 2], s2, s2, eta=0.7)
    assert tuple(lp.shape) == (0, 2) and tuple(means.shape) == (0, 2, 8, 8)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("traj_dtype", [torch.float32, torch.bfloat16])
def test_replay_steps_odd_extents_and_offset_views(dev, kind, traj_dtype):
    """D not a multiple of 4 (element-wise path), a stack and velocities that are offset slices of larger
    buffers (bases off the 16-byte grid, sample strides larger than the data), one sample, one step."""
    from unirl_amd import sde

    st = strategy(kind)
    stored = [0, 1, 2, 3]
    for B, tail, steps in ((3, (3, 5, 7), [1, 0]), (1, (2, 9), [2]), (2, (8, 8), [0, 1, 2])):
        stack, v = make_case(B, len(stored), tail, steps, stored, traj_dtype, traj_dtype, 40 + B)
        ref_lp, ref_means = oracle_replay(kind, stack, v, steps, stored, SIG, traj_dtype)
        slot_x, slot_p = sde.replay_slots(stored, steps)
        # device copies inside larger buffers: one leading element of padding, one extra slot / step
        big_stack = torch.zeros((B, len(stored) + 1) + tail, dtype=traj_dtype, device=dev)
        flat = torch.zeros(big_stack.numel() + 1, dtype=traj_dtype, device=dev)
        stack_view = flat[1:].view(big_stack.shape)[:, : len(stored)]
        stack_view.copy_(stack.to(dev))
        big_v = torch.zeros((B, len(steps) + 2) + tail, dtype=traj_dtype, device=dev)
        v_view = big_v[:, 1 : 1 + len(steps)]
        v_view.copy_(v.to(dev))
        assert B == 1 or not (stack_view.is_contiguous() or v_view.is_contiguous())
        sig = [float(SIG[i]) for i in steps]
        sig_n = [float(SIG[i + 1]) for i in steps]
        lp, means = st.replay_steps(v_view, stack_view, slot_x, slot_p, sig, sig_n, eta=0.7, sigma_max=float(SIG[1]))
        assert torch.equal(means.cpu(), ref_means), (B, tail)
        rtol = FP32_RTOL if traj_dtype == torch.float32 else BF16_RTOL
        assert_close(lp, ref_lp, rtol, 2e-6, f"log-probs B={B} tail={tail}")
        # the gradient takes the velocities' (strided) layout
        vg = v_view.detach().clone().requires_grad_(True)
        lp_g, _ = st.replay_steps(vg, stack_view, slot_x, slot_p, sig, sig_n, eta=0.7, sigma_max=float(SIG[1]))
        lp_g.sum().backward()
        v_ref = v.float().clone().requires_grad_(True)
        tot = 0.0
        for j, i in enumerate(steps):
            tot = tot + osde.sde_denoise(kind, v_ref[:, j], stack[:, i], SIG[i], SIG[i + 1], eta=0.7,
                                         prev_sample=stack[:, i + 1], sigma_max=SIG[1])[1].sum()
        tot.backward()
        gtol = 1e-4 if traj_dtype == torch.float32 else 1e-2
        assert_close(vg.grad.float(), v_ref.grad, gtol, gtol * float(v_ref.grad.abs().max()), "grad, strided velocities")
