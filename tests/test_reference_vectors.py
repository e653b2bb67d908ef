"""Vectors the UniRL reference itself produced (tests/golden/reference_vectors.npz, written by
tests/golden/make_reference_vectors.py where the reference tree is mounted) for the two functions
on the path that are control flow rather than a formula: normalize_grouped / normalize_global
(trimmed statistics, empty and singleton groups, clip, global std) and gather_sde_field (unsorted
indices, repeated targets, the error text).  The CPU oracle, the host path and the HIP kernels are
all held to them; NaN positions (singleton groups: unbiased std of one value) must coincide."""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import advantages as oadv
from oracle import flowdppo as ofd

R = np.load(Path(__file__).parent / "golden" / "reference_vectors.npz")


def meta(name):
    return json.loads(bytes(R[name]).decode())


GROUPS = meta("ng_groups")
NG_CASES = meta("ng_cases")
GS_CASES = meta("gs_cases")


def check(got, name, rtol=1e-5, atol=1e-6):
    want = np.asarray(R[name], dtype=np.float64)
    got = np.asarray(got.detach().cpu().double().numpy(), dtype=np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(want)), f"{name}: NaN positions differ"
    np.testing.assert_allclose(got, want, rtol=rtol, atol=atol, err_msg=name)


@pytest.mark.parametrize("ci", range(len(NG_CASES)))
def test_oracle_normalize_grouped(ci):
    c = NG_CASES[ci]
    got = oadv.normalize_grouped(torch.from_numpy(R["ng_rewards"]), GROUPS, epsilon=1e-8, clip_max=c["clip_max"],
                                 trim_outliers_ratio=c["trim"], use_global_std=c["use_global_std"])
    check(got, f"ng_case{ci}_out", rtol=1e-6, atol=1e-7)


def test_oracle_normalize_global():
    r = torch.from_numpy(R["ng_rewards"])
    check(oadv.normalize_global(r, epsilon=1e-8), "nglobal_out", rtol=1e-6, atol=1e-7)
    check(oadv.normalize_global(r, epsilon=1e-6, clip_max=0.75), "nglobal_clip_out", rtol=1e-6, atol=1e-7)


def run_gather_cases(gather, t, idx, what):
    n_ok = 0
    for gi, c in enumerate(GS_CASES):
        if c.get("error") is None and c["target"] is not None:
            got = gather(t, idx, c["target"], field_name="sde_means")
            assert torch.equal(got.cpu(), torch.from_numpy(R[f"gs_case{gi}_out"])), f"{what}: case {c}"
            n_ok += 1
        elif c["target"] is not None:
            with pytest.raises(ValueError) as e:
                gather(t, idx, c["target"], field_name="sde_logp")
            assert str(e.value) == c["error"], f"{what}: error text for {c['target']}"
        else:
            args = (None, idx) if c["none_arg"] == 0 else (t, None)
            with pytest.raises(ValueError) as e:
                gather(*args, [2], field_name="sde_logp")
            assert str(e.value) == c["error"]
    assert n_ok >= 6


def test_oracle_and_host_gather_sde_field():
    from unirl_amd.algorithms import gather_sde_field

    t, idx = torch.from_numpy(R["gs_tensor"]), torch.from_numpy(R["gs_indices"])
    run_gather_cases(ofd.gather_sde_field, t, idx, "oracle")
    run_gather_cases(gather_sde_field, t, idx, "host path")


@pytest.mark.gpu
@pytest.mark.parametrize("ci", range(len(NG_CASES)))
def test_kernel_normalize_grouped(dev, ci):
    from unirl_amd.algorithms import normalize_grouped

    c = NG_CASES[ci]
    got = normalize_grouped(torch.from_numpy(R["ng_rewards"]).to(dev), GROUPS, epsilon=1e-8, clip_max=c["clip_max"],
                            trim_outliers_ratio=c["trim"], use_global_std=c["use_global_std"])
    check(got, f"ng_case{ci}_out")


@pytest.mark.gpu
def test_kernel_normalize_global_and_gather(dev):
    from unirl_amd.algorithms import gather_sde_field, normalize_global

    r = torch.from_numpy(R["ng_rewards"]).to(dev)
    check(normalize_global(r, epsilon=1e-8), "nglobal_out")
    check(normalize_global(r, epsilon=1e-6, clip_max=0.75), "nglobal_clip_out")
    t, idx = torch.from_numpy(R["gs_tensor"]).to(dev), torch.from_numpy(R["gs_indices"]).to(dev)
    run_gather_cases(gather_sde_field, t, idx, "device path")
    tb = t.to(torch.bfloat16)
    got = gather_sde_field(tb, idx, [9, 0], field_name="sde_means")
    assert torch.equal(got.cpu(), tb.cpu()[:, [2, 3]])


# ---------------------------------------------------------------- x_T noise recipe (unirl/sde/noise.py)
NZ_GIDS = meta("nz_gids")
NZ_SHAPES = {"a": (4, 8, 8), "b": (3,), "c": (2, 3, 5, 7)}


def test_noise_seed_derivation_and_host_recipe():
    from unirl_amd.sde import noise

    assert [noise._derive_group_seed(1234, g) for g in NZ_GIDS] == R["nz_seeds"].tolist()
    assert noise._derive_group_seed((1 << 62) + 5, "prompt-000017") == int(R["nz_seed_big"][0])
    cpu = torch.device("cpu")
    for tag, shape in NZ_SHAPES.items():
        x = noise.regen_initial_noise(NZ_GIDS, 1234, shape, cpu, torch.float32)
        assert torch.equal(x, torch.from_numpy(R[f"nz_{tag}_f32"]))
        xb = noise.regen_initial_noise(NZ_GIDS, 1234, shape, cpu, torch.bfloat16)
        assert torch.equal(xb.view(torch.int16), torch.from_numpy(R[f"nz_{tag}_bf16_bits"]))
    same = noise.generate_latents(4, (2, 9), cpu, torch.float32, init_same_noise=True, samples_per_prompt=2,
                                  noise_group_ids=["g0", "g0", "g1", "g1"], base_seed=99)
    assert torch.equal(same, torch.from_numpy(R["nz_latents_same"]))
    assert noise.generate_latents(3, (2, 2), cpu).shape == (3, 2, 2)
    with pytest.raises(ValueError, match="requires explicit noise_group_ids aligned to batch_size"):
        noise.generate_shared_noise(3, (2,), cpu, noise_group_ids=["a", "b"])
    with pytest.raises(ValueError, match="noise_group_ids_len=None"):
        noise.generate_shared_noise(3, (2,), cpu, noise_group_ids=None)
    with pytest.raises(AssertionError):
        noise.generate_latents(2, (2,), cpu, init_same_noise=True)


@pytest.mark.gpu
def test_noise_recipe_on_device_is_byte_identical(dev):
    from unirl_amd.sde import noise

    for _ in range(2):  # the second pass reuses the pinned staging buffer
        for tag, shape in NZ_SHAPES.items():
            ref = torch.from_numpy(R[f"nz_{tag}_f32"])
            x = noise.regen_initial_noise(NZ_GIDS, 1234, shape, dev, torch.float32)
            assert x.is_cuda and x.dtype == torch.float32 and torch.equal(x.cpu(), ref)
            xb = noise.regen_initial_noise(NZ_GIDS, 1234, shape, dev, torch.bfloat16)
            assert torch.equal(xb.cpu().view(torch.int16), torch.from_numpy(R[f"nz_{tag}_bf16_bits"]))
            xh = noise.regen_initial_noise(NZ_GIDS, 1234, shape, dev, torch.float16)
            assert torch.equal(xh.cpu(), ref.to(torch.float16))
    # a realistic batch: 64 samples in 4 groups of SD3-sized latents; samples of a group are equal
    gids = [f"prompt-{i // 16}" for i in range(64)]
    x = noise.regen_initial_noise(gids, 7, (16, 64, 64), dev, torch.bfloat16)
    assert x.shape == (64, 16, 64, 64)
    assert torch.equal(x[0], x[15]) and torch.equal(x[16], x[31]) and not torch.equal(x[0], x[16])
    g = torch.Generator().manual_seed(noise._derive_group_seed(7, "prompt-2"))
    assert torch.equal(x[40].cpu(), torch.randn(16, 64, 64, generator=g).to(torch.bfloat16))
    # device-side draws (no recipe): groups still share, shapes and dtypes as asked
    y = noise.generate_shared_noise(4, (8, 8), dev, torch.float32, ["a", "b", "a", "c"], base_seed=3)
    assert y.is_cuda and torch.equal(y[0], y[2]) and not torch.equal(y[0], y[1])
    y2 = noise.generate_shared_noise(4, (8, 8), dev, torch.float32, ["a", "b", "a", "c"], base_seed=3)
    assert torch.equal(y, y2)
    assert noise.generate_shared_noise(2, (4,), dev, torch.bfloat16, ["a", "a"]).dtype == torch.bfloat16
    assert noise.regen_initial_noise([], 1, (4, 4), dev).shape == (0, 4, 4)


# ---------------------------------------------------------------- RolloutTrack.compute_advantages
CA_CASES = meta("ca_cases")
CA_PIDS = meta("ca_parent_ids")
CA_ERRORS = meta("ca_errors")


@pytest.mark.parametrize("ci", range(len(CA_CASES)))
def test_oracle_compute_advantages(ci):
    got = oadv.compute_advantages(torch.from_numpy(R["ca_rewards"]), CA_PIDS, **CA_CASES[ci])
    check(got, f"ca_case{ci}_out", rtol=1e-6, atol=1e-7)


def test_compute_advantages_host_rules_and_error_text():
    from unirl_amd.types import RolloutTrack, compute_advantages

    r = torch.from_numpy(R["ca_rewards"])
    check(compute_advantages(r, None), "ca_root_out", rtol=0, atol=0)  # root track: zeros, no kernel
    check(oadv.compute_advantages(r, None), "ca_root_out", rtol=0, atol=0)
    cases = {"interleaved": (["a", "b", "a", "b", "a", "b"], torch.arange(6.0)),
             "nonuniform": (["a", "a", "a", "b", "b"], torch.arange(5.0))}
    for name, (ids, rew) in cases.items():
        with pytest.raises(ValueError) as e:
            compute_advantages(rew, ids)
        assert str(e.value) == CA_ERRORS[name]
    with pytest.raises(ValueError) as e:
        RolloutTrack(sample_ids=["a"], parent_ids=["a"]).compute_advantages()
    assert str(e.value) == CA_ERRORS["no_rewards"]


@pytest.mark.gpu
@pytest.mark.parametrize("ci", range(len(CA_CASES)))
def test_kernel_compute_advantages(dev, ci):
    from unirl_amd.types import RolloutTrack, compute_advantages

    r = torch.from_numpy(R["ca_rewards"]).to(dev)
    check(compute_advantages(r, CA_PIDS, **CA_CASES[ci]), f"ca_case{ci}_out")
    track = RolloutTrack(sample_ids=[str(i) for i in range(24)], parent_ids=CA_PIDS, rewards=r)
    check(track.compute_advantages(**CA_CASES[ci]).advantages, f"ca_case{ci}_out")
    if ci == 0:
        one = compute_advantages(torch.tensor([1.0, 2.0, 3.0], device=dev), ["x", "y", "z"])
        check(one, "ca_singletons_out", rtol=0, atol=0)
