"""GPU parity of the DPM-Solver-2 strategy (one kernel per step) against the CPU oracle."""

import pytest
import torch

from oracle import dpm2 as odpm
from oracle import schedule as osch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(2, 3, 37), (1, 4097), (3, 16, 8, 8)])
def test_dpm2_trajectory_matches_oracle_bitwise(dev, dtype, shape):
    from unirl_amd import sde

    T = 9
    sig = osch.sigma_schedule(T, 3.0)
    g = torch.Generator().manual_seed(31)
    strategy = sde.DPM2Strategy(config=None)
    assert strategy.canonical_name == "dpm2" and isinstance(strategy, sde.StepStrategy)
    with pytest.raises(RuntimeError, match="init_schedule"):
        strategy.denoise(torch.zeros(2, device=dev), torch.zeros(2, device=dev), sig[0], sig[1], step_index=0)
    strategy.init_schedule(sig.to(dev))
    solver = odpm.Dpm2Solver(sig)
    x = torch.randn(shape, generator=g).to(dtype)
    buffers = set()
    for i in range(T):
        v = torch.randn(shape, generator=g).to(dtype)
        want = solver.step(v, x, i)
        prev, logp, mean = strategy.denoise(v.to(dev), x.to(dev), sig[i].to(dev), sig[i + 1].to(dev), eta=0.0, step_index=i)
        assert logp is None and mean is None and prev.dtype == torch.float32 and prev.shape == x.shape
        assert torch.equal(prev.cpu(), want), f"step {i}"
        buffers.add(strategy._x0[1].data_ptr())
        x = want.to(dtype)  # the stage casts the latent back to the trajectory dtype between steps
    assert len(buffers) == 2  # the two x0 predictions alternate between two buffers
    # reset + restart in the middle of the schedule: a first-order step, then second order
    strategy.init_schedule(sig)
    solver = odpm.Dpm2Solver(sig)
    for i in (4, 5, 6):
        v = torch.randn(shape, generator=g).to(dtype)
        want = solver.step(v, x, i)
        got, _, _ = strategy.step(v.to(dev), x.to(dev), sig[i], sig[i + 1], step_index=i)
        assert torch.equal(got.cpu(), want), f"restarted, step {i}"
        x = want.to(dtype)


def test_dpm2_c_abi_argument_checks(dev):
    import ctypes

    from unirl_amd import _native as N

    c = N.Dpm2Coeffs()
    buf = torch.zeros(16, device=dev)
    L, st = N.lib(), N.current_stream(dev)
    args = (N.ptr(buf), N.F32, N.ptr(buf), N.F32)
    assert L.unirl_dpm2_step(*args, None, N.DPM2_SECOND, ctypes.byref(c), 16, N.ptr(buf), N.ptr(buf), st) == -1
    assert L.unirl_dpm2_step(*args, None, 7, ctypes.byref(c), 16, N.ptr(buf), N.ptr(buf), st) == -3
    assert L.unirl_dpm2_step(*args, None, N.DPM2_DDIM, None, 16, N.ptr(buf), N.ptr(buf), st) == -1
    assert L.unirl_dpm2_step(*args, None, N.DPM2_DDIM, ctypes.byref(c), 0, None, None, st) == 0
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        from unirl_amd import sde

        s = sde.DPM2Strategy()
        s.init_schedule(osch.sigma_schedule(4, 3.0))
        s.denoise(torch.zeros(4), torch.zeros(4), torch.tensor(1.0), torch.tensor(0.9), step_index=0)
