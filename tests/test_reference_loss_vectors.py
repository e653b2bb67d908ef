"""Vectors the UniRL reference's own loss functions produced (tests/golden/reference_loss_vectors.npz,
written by tests/golden/make_reference_loss_vectors.py where the reference tree is mounted):
_grpo_clip_loss, _drpo_loss, _gaussian_kl_div, _flowdppo_kl_adv_loss (loss elements, every metric
key, autograd's gradient) and get_sigma_schedule's static branch.  The CPU oracle (not gpu) and the
HIP kernels behind the same signatures (gpu) are both held to them.

Tolerances: fp32 1e-5 relative for the kernels (their `exp` is within 1.5 ulp, torch's within 1);
the oracle runs torch's own ops in the reference's order and is held to 2e-6 (the vectors were
written on another host; torch's vectorised exp may differ by an ulp between CPUs).  Flag fractions
(clip fractions, masks) are exact except for tokens whose ratio, or rows whose KL, lies within
2e-6 relative of the boundary: those are counted, and the fraction may differ by at most that
count."""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import flowdppo as ofd
from oracle import losses as olos
from oracle import schedule as osch

L = np.load(Path(__file__).parent / "golden" / "reference_loss_vectors.npz")


def meta(name):
    return json.loads(bytes(L[name]).decode())


GRPO_CASES, DRPO_CASES, KLADV_CASES, SIGMA_CASES = (meta(k) for k in ("grpo_cases", "drpo_cases", "kladv_cases", "sigma_cases"))
NEW, OLD, ADV = (torch.from_numpy(L[k]) for k in ("tok_new", "tok_old", "tok_adv"))
N_TOK = NEW.numel()
FRACTION_KEYS = {"clip_fraction", "clipfrac_gt_one", "clipfrac_lt_one", "clipfrac_upper", "clipfrac_lower",
                 "kl_mask_fraction", "pos_rm_fraction", "neg_rm_fraction", "masked_fraction", "unmasked_fraction"}


def near_boundary_tokens(edges) -> int:
    """Tokens whose exact ratio lies within 2e-6 relative of one of `edges` (per-token arrays or scalars)."""
    ratio = np.exp(np.clip(NEW.double().numpy() - OLD.double().numpy(), -700, 700))
    near = np.zeros(N_TOK, dtype=bool)
    for e in edges:
        e = np.broadcast_to(np.asarray(e, dtype=np.float64), ratio.shape)
        ok = np.isfinite(e) & (e != 0)
        near |= ok & (np.abs(ratio - e) <= 2e-6 * np.abs(e))
    return int(near.sum())


def close(got, want, rtol, atol, what):
    got = np.asarray(got.detach().cpu().double().numpy() if isinstance(got, torch.Tensor) else got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(want)), f"{what}: NaN positions differ"
    np.testing.assert_allclose(got, want, rtol=rtol, atol=atol, err_msg=what)


def check_metrics(got: dict, keys, want, rtol, slack, n, what):
    assert sorted(got) == list(keys), f"{what}: metric keys {sorted(got)} != the reference's {keys}"
    for k, w in zip(keys, want):
        g = float(got[k])
        if k in FRACTION_KEYS:
            assert abs(g - w) <= slack / n + 1e-7, f"{what}: {k} = {g}, reference {w}, {slack} boundary cases of {n}"
        else:
            assert abs(g - w) <= rtol * abs(w) + 1e-7, f"{what}: {k} = {g}, reference {w}"


def run_loss(fn, device, **kw):
    leaf = NEW.clone().to(device).requires_grad_(True)
    loss, metrics = fn(new_logp=leaf, old_logp=OLD.to(device), advantages=ADV.to(device), **kw)
    loss.sum().backward()
    return loss.detach(), leaf.grad, metrics


def grpo_edges(c):
    hi = c["clip_range"] if c["clip_range_high"] is None else c["clip_range_high"]
    return (1.0 - c["clip_range"], 1.0 + hi)


def drpo_edges(c):
    if not c["mu_weighted"]:
        return (1.0 + c["epsilon"], 1.0 - c["epsilon"])
    with np.errstate(over="ignore", divide="ignore"):
        aeps = c["epsilon"] / np.exp(OLD.double().numpy())
    return (1.0 + aeps, 1.0 - aeps)


def check_token_case(fn, device, c, tag, edges, rtol, kw):
    loss, grad, metrics = run_loss(fn, device, **kw)
    slack = near_boundary_tokens(edges)
    # an element on a clip edge takes either branch of the maximum / the clamp's gradient: leave those to the count
    ratio = np.exp(np.clip(NEW.double().numpy() - OLD.double().numpy(), -700, 700))
    edge = np.zeros(N_TOK, dtype=bool)
    for e in edges:
        e = np.broadcast_to(np.asarray(e, dtype=np.float64), ratio.shape)
        edge |= np.isfinite(e) & (np.abs(ratio - e) <= 2e-6 * np.abs(e))
    # DRPO's clamp at |log-ratio| = 20 switches the gradient off exactly there
    edge |= np.abs(np.abs(NEW.double().numpy() - OLD.double().numpy()) - 20.0) <= 1e-5
    keep = ~edge
    close(loss.cpu().numpy()[keep], L[f"{tag}_loss"][keep], rtol, 1e-7, f"{tag} loss elements")
    close(grad.cpu().numpy()[keep], L[f"{tag}_grad"][keep], rtol, 1e-7, f"{tag} gradient")
    assert int(edge.sum()) < 40
    check_metrics(metrics, c["metric_keys"], L[f"{tag}_metrics"], rtol, slack, N_TOK, tag)


# ------------------------------------------------------------------------------------------------
# the oracle (CPU)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("ci", range(len(GRPO_CASES)))
def test_oracle_grpo_clip_loss_matches_the_reference(ci):
    c = GRPO_CASES[ci]
    fn = lambda **kw: olos.grpo_clip_loss(kw["new_logp"], kw["old_logp"], kw["advantages"], kw["clip_range"],
                                          kw["clip_range_high"])
    check_token_case(fn, "cpu", c, f"grpo{ci}", grpo_edges(c), 2e-6,
                     dict(clip_range=c["clip_range"], clip_range_high=c["clip_range_high"]))


def test_oracle_grpo_single_element_std_is_zero():
    _, m = olos.grpo_clip_loss(NEW[:1], OLD[:1], ADV[:1], 0.2)
    close(np.array([float(m[k]) for k in sorted(m)]), L["grpo_single_metrics"], 2e-6, 1e-7, "single-element metrics")


@pytest.mark.parametrize("ci", range(len(DRPO_CASES)))
def test_oracle_drpo_loss_matches_the_reference(ci):
    c = DRPO_CASES[ci]
    fn = lambda **kw: olos.drpo_loss(kw["new_logp"], kw["old_logp"], kw["advantages"], kw["epsilon"], kw["mu_weighted"])
    check_token_case(fn, "cpu", c, f"drpo{ci}", drpo_edges(c), 2e-6, dict(epsilon=c["epsilon"], mu_weighted=c["mu_weighted"]))


def kl_inputs(tag, device="cpu"):
    if tag == "f32":
        p, q = torch.from_numpy(L["kl_new_f32"]), torch.from_numpy(L["kl_old_f32"])
    else:
        dt = torch.bfloat16 if tag == "bf16" else torch.float16
        p = torch.from_numpy(L[f"kl_new_{tag}_bits"]).view(dt)
        q = torch.from_numpy(L[f"kl_old_{tag}_bits"]).view(dt)
    return p.to(device), q.to(device), torch.from_numpy(L["kl_sigma"]).to(device)


@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
def test_oracle_gaussian_kl_matches_the_reference(tag):
    p, q, s = kl_inputs(tag)
    elem = ofd.gaussian_kl(p, q, s)
    assert elem.dtype is torch.float32
    assert np.array_equal(elem.numpy(), L[f"kl_{tag}_elem"]), "sub, square and divide are correctly rounded everywhere"
    close(ofd.kl_per_sample(p, q, s), L[f"kl_{tag}_rows"], 1e-6, 0.0, "row KL")


def near_threshold_rows(tag, threshold) -> int:
    rows = np.asarray(L[f"kl_{tag}_rows"], dtype=np.float64)
    return int((np.abs(rows - threshold) <= 2e-6 * abs(threshold)).sum())


def check_kladv(fn, device, c, rtol):
    tag, ti, thr = c["dtype"], c["case"], c["threshold"]
    p, q, s = kl_inputs(tag, device)
    leaf = torch.from_numpy(L["kl_new_lp"]).to(device).requires_grad_(True)
    loss, metrics = fn(new_logp=leaf, old_logp=torch.from_numpy(L["kl_old_lp"]).to(device), new_means=p, old_means=q,
                       advantages=torch.from_numpy(L["kl_adv"]).to(device), sigma_t=s, kl_mask_threshold=thr)
    loss.sum().backward()
    slack = near_threshold_rows(tag, thr)
    name = f"kladv_{tag}_{ti}"
    n = leaf.numel()
    if slack == 0:
        close(loss, L[f"{name}_loss"], rtol, 1e-9, f"{name} loss elements")
        close(leaf.grad, L[f"{name}_grad"], rtol, 1e-9, f"{name} gradient")
    else:  # the row on the threshold may fall on either side: all other elements must agree
        rows = np.asarray(L[f"kl_{tag}_rows"], dtype=np.float64)
        keep = np.abs(rows - thr) > 2e-6 * abs(thr)
        close(loss.detach().cpu().numpy()[keep], L[f"{name}_loss"][keep], rtol, 1e-9, f"{name} loss elements")
        close(leaf.grad.cpu().numpy()[keep], L[f"{name}_grad"][keep], rtol, 1e-9, f"{name} gradient")
    check_metrics(metrics, c["metric_keys"], L[f"{name}_metrics"], rtol, slack, n, name)
    return slack


@pytest.mark.parametrize("ci", range(len(KLADV_CASES)))
def test_oracle_flowdppo_kl_adv_loss_matches_the_reference(ci):
    fn = lambda **kw: ofd.flowdppo_loss(kw["new_logp"], kw["old_logp"], kw["new_means"], kw["old_means"],
                                        kw["advantages"], kw["sigma_t"], kw["kl_mask_threshold"])
    check_kladv(fn, "cpu", KLADV_CASES[ci], 2e-6)


@pytest.mark.parametrize("ci", range(len(SIGMA_CASES)))
def test_sigma_schedule_matches_the_reference(ci):
    from unirl_amd.sde.runtime import get_sigma_schedule

    c = SIGMA_CASES[ci]
    want = L[f"sigma{ci}"]
    for what, got in (("oracle", osch.sigma_schedule(c["num_steps"], c["shift"])),
                      ("host path", get_sigma_schedule(c["num_steps"], c["shift"]))):
        assert got.dtype is torch.float32 and tuple(got.shape) == want.shape
        # elementwise fp32 mul / add / div of a linspace: identical bits on the host the vectors were
        # written on; another CPU's vectorised linspace may differ in the last place
        close(got, want, 2.5e-7, 0.0, f"{what} {c}")
        assert float(got[0]) == 1.0 and float(got[-1]) == 0.0


# ------------------------------------------------------------------------------------------------
# the kernels behind the reference's signatures (GPU)
# ------------------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("ci", range(len(GRPO_CASES)))
def test_kernel_grpo_clip_loss_matches_the_reference(ci):
    from unirl_amd.algorithms import _grpo_clip_loss

    c = GRPO_CASES[ci]
    check_token_case(_grpo_clip_loss, "cuda", c, f"grpo{ci}", grpo_edges(c), 1e-5,
                     dict(clip_range=c["clip_range"], clip_range_high=c["clip_range_high"]))


@pytest.mark.gpu
def test_kernel_grpo_single_element_std_is_zero():
    from unirl_amd.algorithms import _grpo_clip_loss

    _, m = _grpo_clip_loss(new_logp=NEW[:1].cuda(), old_logp=OLD[:1].cuda(), advantages=ADV[:1].cuda(), clip_range=0.2)
    close(np.array([float(m[k]) for k in sorted(m)]), L["grpo_single_metrics"], 1e-5, 1e-7, "single-element metrics")


@pytest.mark.gpu
@pytest.mark.parametrize("ci", range(len(DRPO_CASES)))
def test_kernel_drpo_loss_matches_the_reference(ci):
    from unirl_amd.algorithms import _drpo_loss

    c = DRPO_CASES[ci]
    check_token_case(_drpo_loss, "cuda", c, f"drpo{ci}", drpo_edges(c), 1e-5,
                     dict(epsilon=c["epsilon"], mu_weighted=c["mu_weighted"]))


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["f32", "bf16", "f16"])
def test_kernel_gaussian_kl_matches_the_reference(tag):
    from unirl_amd.algorithms import _gaussian_kl_div

    p, q, s = kl_inputs(tag, "cuda")
    elem = _gaussian_kl_div(p, q, s)
    assert elem.dtype is torch.float32
    assert np.array_equal(elem.cpu().numpy(), L[f"kl_{tag}_elem"]), "element KL is bit-identical to the reference's"


@pytest.mark.gpu
@pytest.mark.parametrize("ci", range(len(KLADV_CASES)))
def test_kernel_flowdppo_kl_adv_loss_matches_the_reference(ci):
    from unirl_amd.algorithms import _flowdppo_kl_adv_loss

    slack = check_kladv(_flowdppo_kl_adv_loss, "cuda", KLADV_CASES[ci], 1e-5)
    print(f"rows within 2e-6 of the threshold (either side allowed): {slack}")
