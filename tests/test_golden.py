"""The committed float64 vectors (tests/golden/vectors.npz, written by tests/golden/make_vectors.py
from the published formulas with numpy only) against the CPU oracle and against the HIP kernels.

fp32 results are held to 1e-5 relative (plus an absolute floor where a value passes through zero);
masks are exact (the vectors sit clear of the threshold)."""
from __future__ import annotations

from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import advantages as oadv
from oracle import flowdppo as ofd
from oracle import losses as olos
from oracle import schedule as osch
from oracle import sde as osde
from oracle import token_logp as otok

G = np.load(Path(__file__).parent / "golden" / "vectors.npz")
KINDS = ("flow", "dance", "cps")
STEPS = (0, 10, 26)


def t(name, dtype=torch.float32):
    return torch.from_numpy(np.asarray(G[name])).to(dtype)


def close(got, name, rtol=1e-5, atol=1e-6):
    want = np.asarray(G[name], dtype=np.float64)
    got = np.asarray(got.detach().cpu().double().numpy() if isinstance(got, torch.Tensor) else got, dtype=np.float64)
    np.testing.assert_allclose(got.reshape(want.shape), want, rtol=rtol, atol=atol, err_msg=name)


# ------------------------------------------------------------------ oracle vs vectors (CPU)
def test_oracle_sigma_schedule():
    close(osch.sigma_schedule(28, 3.0), "sigma_T28_shift3", rtol=2e-7, atol=1e-7)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("step", STEPS)
def test_oracle_sde_step(kind, step):
    sig = osch.sigma_schedule(28, 3.0)
    prev, logp, mean = osde.sde_denoise(kind, t("sde_v"), t("sde_x"), sig[step], sig[step + 1], eta=0.7,
                                        noise=t("sde_noise"), sigma_max=sig[1])
    key = f"sde_{kind}_step{step}"
    close(prev, key + "_prev", atol=2e-6)
    close(mean, key + "_mean", atol=2e-6)
    close(logp, key + "_logp", atol=1e-5)
    # replay of the float64 answer's own prev (rounded to fp32) reproduces the log-prob
    _, logp_r, _ = osde.sde_denoise(kind, t("sde_v"), t("sde_x"), sig[step], sig[step + 1], eta=0.7,
                                    prev_sample=t(key + "_prev"), sigma_max=sig[1])
    close(logp_r, key + "_logp", atol=1e-5)


@pytest.mark.parametrize("tag", ("f32", "bf16"))
@pytest.mark.parametrize("T", (1.0, 0.7))
def test_oracle_token_logp_entropy(tag, T):
    x = t("tok_logits_f32") if tag == "f32" else t("tok_logits_bf16_as_f32").bfloat16()
    ids = t("tok_ids", torch.int64)
    close(otok.token_logp(x, ids, T), f"tok_{tag}_T{T}_logp", atol=2e-6)
    close(otok.token_entropy(x, T), f"tok_{tag}_T{T}_ent", atol=2e-6)


def _loss_inputs():
    return t("loss_new"), t("loss_old"), t("loss_adv"), t("loss_lengths", torch.int64)


def test_oracle_grpo_loss():
    new, old, adv, lengths = _loss_inputs()
    adv_tok = adv[:, None].expand_as(new)
    elem, _ = olos.grpo_clip_loss(new, old, adv_tok, 0.2, 0.28)
    mask = torch.arange(new.shape[1])[None, :] < lengths[:, None]
    close(torch.where(mask, elem, torch.zeros(())), "grpo_loss_elem")
    pn, po = olos.pack_padded(new, lengths), olos.pack_padded(old, lengths)
    for mode in ("token-mean", "seq-mean-token-sum-norm", "seq-mean-token-mean"):
        loss, m = olos.token_loss("grpo", pn, po, adv, lengths, mode=mode, horizon=64, clip_range=0.2, clip_range_high=0.28)
        close(loss, "grpo_" + mode.replace("-", "_"))
    got = [m[k] for k in ("ratio_mean", "ratio_std", "ratio_min", "ratio_max", "clip_fraction", "clipfrac_gt_one",
                          "clipfrac_lt_one", "approx_kl")]
    ad = olos.logp_absdiff(pn, po)
    got += [torch.tensor(v) for v in ad.values()]
    close(torch.stack([g.float() for g in got]), "grpo_metrics")


@pytest.mark.parametrize("mu", (True, False))
def test_oracle_drpo_loss(mu):
    new, old, adv, lengths = _loss_inputs()
    tag = "mu" if mu else "nomu"
    elem, _ = olos.drpo_loss(new, old, adv[:, None].expand_as(new), 5.0, mu)
    mask = torch.arange(new.shape[1])[None, :] < lengths[:, None]
    close(torch.where(mask, elem, torch.zeros(())), f"drpo_{tag}_loss_elem")
    pn, po = olos.pack_padded(new, lengths), olos.pack_padded(old, lengths)
    loss, m = olos.token_loss("drpo", pn, po, adv, lengths, epsilon=5.0, mu_weighted=mu)
    close(loss, f"drpo_{tag}_token_mean")
    got = torch.stack([m[k].float() for k in ("ratio_mean", "ratio_max", "approx_kl", "drpo_penalty_mean",
                                              "clipfrac_upper", "clipfrac_lower")])
    close(got, f"drpo_{tag}_metrics", atol=1e-7)


def test_oracle_gaussian_kl_mask():
    kl = ofd.kl_per_sample(t("kl_p"), t("kl_q"), t("kl_sigma_t").view(1, -1, 1))
    close(kl, "kl_value")
    assert np.array_equal((kl < float(G["kl_threshold"])).numpy(), G["kl_mask"])


def test_oracle_advantages():
    r = t("adv_rewards")
    parents = [i // 4 for i in range(16)]
    close(oadv.compute_advantages(r, parents), "adv_group_norm", atol=1e-5)
    close(oadv.compute_advantages(r, parents, normalize=False), "adv_group_center")
    close(oadv.compute_advantages(r, parents, use_global_std=True), "adv_group_global_std")
    close(oadv.compute_advantages(r, parents, scope="global"), "adv_global")


# ------------------------------------------------------------------ kernels vs vectors (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("step", STEPS)
def test_kernel_sde_step(dev, kind, step):
    from unirl_amd import ops

    sig = osch.sigma_schedule(28, 3.0).to(dev)
    v, x, n = t("sde_v").to(dev), t("sde_x").to(dev), t("sde_noise").to(dev)
    key = f"sde_{kind}_step{step}"
    prev, logp, mean = ops.sde_step_logp(v, x, sig[step], sig[step + 1], kind=kind, eta=0.7, noise=n, sigma_max=sig[1])
    close(prev.view(x.shape), key + "_prev", atol=2e-6)
    close(mean.view(x.shape), key + "_mean", atol=2e-6)
    close(logp, key + "_logp", atol=1e-5)
    _, logp_r, _ = ops.sde_step_logp(v, x, sig[step], sig[step + 1], kind=kind, eta=0.7,
                                     prev_sample=t(key + "_prev").to(dev), sigma_max=sig[1])
    close(logp_r, key + "_logp", atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ("f32", "bf16"))
@pytest.mark.parametrize("T", (1.0, 0.7))
def test_kernel_token_logp_entropy(dev, tag, T):
    from unirl_amd import ops

    x = (t("tok_logits_f32") if tag == "f32" else t("tok_logits_bf16_as_f32").bfloat16()).to(dev)
    ids = t("tok_ids", torch.int64).to(dev)
    logp, ent, lse = ops.token_logp_entropy(x, ids, T, want_lse=True)
    close(logp, f"tok_{tag}_T{T}_logp", atol=2e-6)
    close(ent, f"tok_{tag}_T{T}_ent", atol=2e-6)
    close(lse, f"tok_{tag}_T{T}_lse", atol=2e-6)


@pytest.mark.gpu
def test_kernel_grpo_loss(dev):
    from unirl_amd import _native as N
    from unirl_amd import ops

    new, old, adv, lengths = (a.to(dev) for a in _loss_inputs())
    for mode in ("token-mean", "seq-mean-token-sum-norm", "seq-mean-token-mean"):
        plan = ops.RatioLossPlan(new, old, adv, kind=N.LOSS_GRPO, lengths=lengths, agg_mode=mode, clip_low=0.2,
                                 clip_high=0.28, horizon=64)
        elem, m = plan.forward(True)
        close(m[N.M_LOSS], "grpo_" + mode.replace("-", "_"))
        close(elem, "grpo_loss_elem")
    slots = (N.M_RATIO_MEAN, N.M_RATIO_STD, N.M_RATIO_MIN, N.M_RATIO_MAX, N.M_CLIP_FRACTION, N.M_CLIPFRAC_HI,
             N.M_CLIPFRAC_LO, N.M_APPROX_KL, N.M_ABSDIFF_MEAN, N.M_ABSDIFF_MAX)
    close(m[list(slots)], "grpo_metrics")
    assert int(m[N.M_NUM_TOKENS].item()) == int(lengths.sum().item())


@pytest.mark.gpu
@pytest.mark.parametrize("mu", (True, False))
def test_kernel_drpo_loss(dev, mu):
    from unirl_amd import _native as N
    from unirl_amd import ops

    new, old, adv, lengths = (a.to(dev) for a in _loss_inputs())
    tag = "mu" if mu else "nomu"
    plan = ops.RatioLossPlan(new, old, adv, kind=N.LOSS_DRPO, lengths=lengths, drpo_epsilon=5.0, mu_weighted=mu)
    elem, m = plan.forward(True)
    close(elem, f"drpo_{tag}_loss_elem")
    close(m[N.M_LOSS], f"drpo_{tag}_token_mean")
    slots = (N.M_RATIO_MEAN, N.M_RATIO_MAX, N.M_APPROX_KL, N.M_PENALTY_MEAN, N.M_CLIPFRAC_HI, N.M_CLIPFRAC_LO)
    close(m[list(slots)], f"drpo_{tag}_metrics", atol=1e-7)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", (torch.float32,))
def test_kernel_gaussian_kl_mask(dev, dtype):
    from unirl_amd import ops

    kl, mask = ops.gaussian_kl_mask(t("kl_p").to(dev), t("kl_q").to(dev), t("kl_sigma_t").to(dev),
                                    float(G["kl_threshold"]))
    close(kl, "kl_value")
    assert np.array_equal(mask.cpu().numpy().astype(bool).reshape(G["kl_mask"].shape), G["kl_mask"])


@pytest.mark.gpu
def test_kernel_advantages(dev):
    from unirl_amd import ops

    r = t("adv_rewards").to(dev)
    close(ops.group_advantages(r, 4), "adv_group_norm", atol=1e-5)
    close(ops.group_advantages(r, 4, normalize=False), "adv_group_center")
    close(ops.group_advantages(r, 4, use_global_std=True), "adv_group_global_std")
    close(ops.group_advantages(r, 4, scope="global"), "adv_global")
