"""Writes tests/golden/vectors.npz: small input/output vectors for every function on the path.

The expected outputs are computed here in numpy float64 straight from the published formulas
(flow-matching SDE transition and Gaussian log-density, log-softmax, entropy, PPO-style clipped
ratio, DRPO quadratic penalty, Gaussian KL with shared variance, group z-scores).  Nothing from
``oracle/`` or ``unirl_amd/`` is imported, so the file is an independent third statement of the
arithmetic: the CPU oracle and the HIP kernels are both checked against it.  The UniRL sources
hold no vectors of their own for these functions; formulas follow unirl/sde/kernels.py:193-333,
unirl/algorithms/base.py:115-157, unirl/algorithms/drpo.py:97-159,
unirl/algorithms/flowdppo.py:43-138, unirl/types/rollout_resp.py:314-333 and
unirl/models/qwen3/ar.py:82-85.

Run:  python tests/golden/make_vectors.py
"""
from __future__ import annotations

import math
from pathlib import Path

import numpy as np

OUT = Path(__file__).with_name("vectors.npz")


def f32(a):
    return np.asarray(a, dtype=np.float32)


def to_bf16(a):
    """Round fp32 to the nearest bf16 (ties to even); returned as fp32."""
    u = f32(a).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def sigma_schedule(T, shift):
    t = np.linspace(1.0, 0.0, T + 1)
    return shift * t / (1.0 + (shift - 1.0) * t)


def sde_step64(kind, v, x, s, s_next, eta, noise, s_max):
    """float64 transition; returns prev, mean, std_var, per-sample mean log-prob."""
    v, x, noise = (np.asarray(a, dtype=np.float64) for a in (v, x, noise))
    dt = s_next - s
    if kind == "cps":
        std = s_next * math.sin(eta * math.pi / 2.0)
        x0 = x - s * v
        eps = x + v * (1.0 - s)
        mean = x0 * (1.0 - s_next) + eps * math.sqrt(s_next * s_next - std * std)
        prev = mean + std * noise
        lp = -((prev - mean) ** 2)
        return prev, mean, std, lp.reshape(lp.shape[0], -1).mean(axis=1)
    if kind == "flow":
        s_safe = s_max if s == 1.0 else s
        std = math.sqrt(s / (1.0 - s_safe)) * eta
    else:  # dance
        std = eta
    mean = x * (1.0 + std * std / (2.0 * s) * dt) + v * (1.0 + std * std * (1.0 - s) / (2.0 * s)) * dt
    std_var = std * math.sqrt(-dt)
    prev = mean + std_var * noise
    lp = -((prev - mean) ** 2) / (2.0 * std_var**2) - math.log(std_var) - 0.5 * math.log(2.0 * math.pi)
    return prev, mean, std_var, lp.reshape(lp.shape[0], -1).mean(axis=1)


def token64(logits, ids, T):
    lf = np.asarray(logits, dtype=np.float64) / T
    m = lf.max(axis=-1, keepdims=True)
    lse = m[..., 0] + np.log(np.exp(lf - m).sum(axis=-1))
    logp = np.take_along_axis(lf, ids[:, None], axis=-1)[:, 0] - lse
    p = np.exp(lf - lse[:, None])
    ent = lse - (p * lf).sum(axis=-1)
    return logp, ent, lse


def grpo64(new, old, adv, lo, hi):
    new, old, adv = (np.asarray(a, dtype=np.float64) for a in (new, old, adv))
    r = np.exp(new - old)
    return np.maximum(-adv * r, -adv * np.clip(r, 1.0 - lo, 1.0 + hi)), r


def drpo64(new, old, adv, eps, mu_weighted):
    new, old, adv = (np.asarray(a, dtype=np.float64) for a in (new, old, adv))
    ld = np.clip(new - old, -20.0, 20.0)
    r = np.exp(ld)
    w = np.exp(old) if mu_weighted else 1.0
    pen = np.abs(adv) * w * (r - 1.0) ** 2 / (2.0 * eps)
    return -adv * r + pen, r, pen, ld


def main() -> None:
    rng = np.random.default_rng(20240611)
    out: dict[str, np.ndarray] = {}

    # ---- sigma schedule --------------------------------------------------------------------
    sig = sigma_schedule(28, 3.0)
    out["sigma_T28_shift3"] = sig

    # ---- SDE transitions: fp32 inputs, float64 answers ----------------------------------------
    shape = (3, 4, 8, 8)
    x = f32(rng.standard_normal(shape))
    v = f32(rng.standard_normal(shape))
    n = f32(rng.standard_normal(shape))
    out["sde_x"], out["sde_v"], out["sde_noise"] = x, v, n
    sig32 = f32(sig)
    for kind in ("flow", "dance", "cps"):
        for step in (0, 10, 26):
            s, s_next, s_max = float(sig32[step]), float(sig32[step + 1]), float(sig32[1])
            prev, mean, std_var, lp = sde_step64(kind, v, x, s, s_next, 0.7, n, s_max)
            key = f"sde_{kind}_step{step}"
            out[key + "_prev"], out[key + "_mean"] = prev, mean
            out[key + "_stdvar"], out[key + "_logp"] = np.float64(std_var), lp

    # ---- token log-prob and entropy --------------------------------------------------------------
    rows, V = 12, 1537
    lg = f32(2.0 * rng.standard_normal((rows, V)))
    lg[3, 77] = 15.0       # a spiked row
    lg[5, :] = 0.25        # a uniform row
    ids = rng.integers(0, V, size=rows).astype(np.int64)
    ids[3] = 77
    out["tok_logits_f32"], out["tok_ids"] = lg, ids
    out["tok_logits_bf16_as_f32"] = to_bf16(lg)
    for tag, arr in (("f32", lg), ("bf16", out["tok_logits_bf16_as_f32"])):
        for T in (1.0, 0.7):
            logp, ent, lse = token64(arr, ids, T)
            k = f"tok_{tag}_T{T}"
            out[k + "_logp"], out[k + "_ent"], out[k + "_lse"] = logp, ent, lse

    # ---- ratio losses on a ragged padded batch -----------------------------------------------------
    n_seq, width = 5, 41
    lengths = np.array([41, 17, 0, 33, 1], dtype=np.int64)
    old = f32(-8.0 * rng.random((n_seq, width)))
    new = f32(old + 0.3 * rng.standard_normal((n_seq, width)))
    adv = f32([1.5, -0.75, 0.3, -2.0, 0.5])
    mask = np.arange(width)[None, :] < lengths[:, None]
    out["loss_new"], out["loss_old"], out["loss_adv"], out["loss_lengths"] = new, old, adv, lengths
    a_tok = np.broadcast_to(adv[:, None], new.shape)
    le, r = grpo64(new, old, a_tok, 0.2, 0.28)
    out["grpo_loss_elem"] = np.where(mask, le, 0.0)
    rv, lv = r[mask], le[mask]
    ld = (new.astype(np.float64) - old.astype(np.float64))[mask]
    out["grpo_token_mean"] = np.float64(lv.mean())
    out["grpo_seq_mean_token_sum_norm"] = np.float64(np.mean([le[i, : lengths[i]].sum() for i in range(n_seq)]) / 64.0)
    out["grpo_seq_mean_token_mean"] = np.float64(
        np.mean([le[i, : lengths[i]].mean() if lengths[i] else 0.0 for i in range(n_seq)]))
    out["grpo_metrics"] = np.array([
        rv.mean(), rv.std(ddof=1), rv.min(), rv.max(),
        np.mean(np.maximum(rv - 1.0 > 0.28, 1.0 - rv > 0.2)), np.mean(rv - 1.0 > 0.28), np.mean(1.0 - rv > 0.2),
        np.mean(0.5 * ld * ld), np.abs(ld).mean(), np.abs(ld).max(),
    ])
    for mu_w in (True, False):
        le, r, pen, ldc = drpo64(new, old, a_tok, 5.0, mu_w)
        tag = "mu" if mu_w else "nomu"
        out[f"drpo_{tag}_loss_elem"] = np.where(mask, le, 0.0)
        out[f"drpo_{tag}_token_mean"] = np.float64(le[mask].mean())
        rv, pv, lc = r[mask], pen[mask], ldc[mask]
        eps_t = 5.0 / np.exp(old.astype(np.float64))[mask] if mu_w else np.full(rv.shape, 5.0)
        out[f"drpo_{tag}_metrics"] = np.array([
            rv.mean(), rv.max(), np.mean((rv - 1.0) - lc), pv.mean(), np.mean(rv > 1.0 + eps_t), np.mean(rv < 1.0 - eps_t),
        ])

    # ---- Gaussian KL with a shared sigma and the trust-region mask -------------------------------------
    B, S, D = 3, 2, 96
    base = rng.standard_normal((B, S, D))
    scale = np.array([0.002, 0.3, 0.05])[:, None, None]        # sample 0 far inside, sample 1 far outside
    p = f32(base + scale * rng.standard_normal((B, S, D)))
    q = f32(base + scale * rng.standard_normal((B, S, D)))
    sig_t = f32([0.25, 0.125])
    kl = (((p.astype(np.float64) - q.astype(np.float64)) ** 2) / (2.0 * sig_t.astype(np.float64)[None, :, None] ** 2)).mean(axis=2)
    out["kl_p"], out["kl_q"], out["kl_sigma_t"], out["kl_value"] = p, q, sig_t, kl
    out["kl_threshold"] = np.float64(0.01)
    out["kl_mask"] = kl < 0.01
    assert np.all(np.abs(kl - 0.01) > 1e-3), "vectors must sit clear of the threshold"

    # ---- group advantages -------------------------------------------------------------------------------
    rew = f32(rng.random(16))
    rew[4:8] = 0.5                                            # an all-equal group
    g = rew.astype(np.float64).reshape(4, 4)
    out["adv_rewards"] = rew
    out["adv_group_norm"] = ((g - g.mean(1, keepdims=True)) / np.sqrt(g.var(1, keepdims=True) + 1e-8)).reshape(-1)
    out["adv_group_center"] = (g - g.mean(1, keepdims=True)).reshape(-1)
    out["adv_group_global_std"] = ((g - g.mean(1, keepdims=True)) / (g.std(ddof=1) + 1e-8)).reshape(-1)
    out["adv_global"] = ((g - g.mean()) / (g.std(ddof=1) + 1e-8)).reshape(-1)

    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(out)} arrays)")


if __name__ == "__main__":
    main()
