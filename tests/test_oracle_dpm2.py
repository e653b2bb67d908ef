"""Pins of the DPM-Solver-2 oracle (oracle/dpm2.py) by what the mathematics fixes: the DDIM and
the first-order update are Euler steps of the flow-matching ODE in exact arithmetic; the
second-order update equals the first-order one when the x0 prediction does not move; on a
Gaussian data distribution, whose probability-flow ODE has a closed-form solution, the sampler
converges faster than Euler and at the rate of a second-order multistep method."""

import torch

from oracle import dpm2
from oracle import schedule as osch


def _gaussian_velocity(c):
    """Optimal velocity for data N(0, c^2) and noise N(0, 1) under x_s = (1-s) x0 + s eps:
    v(x, s) = x (s - (1-s) c^2) / ((1-s)^2 c^2 + s^2); along the ODE x scales with the marginal
    standard deviation, so x(0) = c x(1)."""

    def velocity(x, s):
        s = s.double()
        return (x.double() * (s - (1 - s) * c * c) / ((1 - s) ** 2 * c * c + s * s)).float()

    return velocity


def _euler(velocity, x, sig):
    for i in range(sig.numel() - 1):
        x = x + velocity(x, sig[i]) * (sig[i + 1] - sig[i])
    return x


def test_ddim_and_first_order_updates_are_euler_steps():
    sig = osch.sigma_schedule(12, 3.0)
    g = torch.Generator().manual_seed(3)
    x, v = torch.randn(64, generator=g), torch.randn(64, generator=g)
    # first step (sigma == 1) and last step (sigma_next == 0): the DDIM branch
    for i in (0, 11):
        solver = dpm2.Dpm2Solver(sig)
        solver.warm = 0 if i == 0 else 2
        got = solver.step(v, x, i)
        assert torch.allclose(got, x + v * (sig[i + 1] - sig[i]), rtol=1e-5, atol=1e-6)
    # the last step lands exactly on the x0 prediction
    solver = dpm2.Dpm2Solver(sig)
    solver.warm = 2
    assert torch.equal(solver.step(v, x, 11), x - sig[11] * v)
    # a solver restarted in the middle of the schedule takes a first-order step
    solver = dpm2.Dpm2Solver(sig)
    got = solver.step(v, x, 5)
    assert torch.allclose(got, x + v * (sig[6] - sig[5]), rtol=1e-5, atol=1e-6)


def test_second_order_equals_first_order_for_a_constant_prediction():
    sig = osch.sigma_schedule(12, 3.0)
    g = torch.Generator().manual_seed(4)
    x0 = torch.randn(32, generator=g)
    eps = torch.randn(32, generator=g)
    multistep, restarted = dpm2.Dpm2Solver(sig), None
    x = eps.clone()
    for i in range(6):
        v = (x - x0) / sig[i]  # the model that always predicts x0
        if i == 5:
            restarted = dpm2.Dpm2Solver(sig).step(v, x, i)  # first order
        x_next = multistep.step(v, x, i)
        if i == 5:
            assert torch.allclose(x_next, restarted, rtol=1e-5, atol=1e-6)
        x = x_next
    # and the trajectory stays on the line between eps and x0
    assert torch.allclose(x, (1 - sig[6]) * x0 + sig[6] * eps, rtol=1e-4, atol=1e-5)


def test_convergence_order_on_a_gaussian():
    c = 0.5
    velocity = _gaussian_velocity(c)
    x_init = torch.randn(1000, generator=torch.Generator().manual_seed(0))

    def scale_error(sample_fn, T):
        out = sample_fn(velocity, x_init, osch.sigma_schedule(T, 3.0))
        return abs(float((out / x_init).mean()) - c)

    d160, d320 = (scale_error(dpm2.sample_trajectory, T) for T in (160, 320))
    e160, e320 = (scale_error(_euler, T) for T in (160, 320))
    assert 1.8 < e160 / e320 < 2.2              # Euler: first order
    assert d160 / d320 > 2.7                    # the multistep solver: close to second order
    assert d160 < 2e-3 and d160 < e160 / 5      # (a flipped sign or a dropped 1/2 in the D1 term gives 1.4e-2)
