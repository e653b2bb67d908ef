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
