"""Writes tests/golden/reference_loss_vectors.npz: outputs of the UniRL reference's own pure loss
functions, so that the oracle's restatement of their formulas is held to the reference itself and
not only to mathematics and an independent numpy evaluation:

  * _grpo_clip_loss          (unirl/algorithms/base.py:115-157)   loss elements, the 8 metrics,
                                                                  autograd's gradient
  * _drpo_loss               (unirl/algorithms/drpo.py:97-159)    loss elements, the 6 metrics,
                                                                  autograd's gradient
  * _gaussian_kl_div         (unirl/algorithms/flowdppo.py:43-51) element values for fp32 / bf16 /
                                                                  fp16 means (torch's type promotion)
  * _flowdppo_kl_adv_loss    (unirl/algorithms/flowdppo.py:54-138) loss elements, the 12 metrics,
                                                                  autograd's gradient
  * get_sigma_schedule       (unirl/sde/runtime.py:92-96)         the static branch

Only runs where the reference tree is mounted (/root/reference).  The modules that hold these
functions cannot be imported (their packages pull in ray / omegaconf, which are not installed);
each function is a pure function of torch tensors, so its definition alone is compiled out of
its file's syntax tree and executed with torch in scope -- the mechanism
make_reference_vectors.py uses for gather_sde_field.  Nothing of the reference is written to the
output: the file holds the inputs drawn here and the arrays the reference returned.

Run:  python tests/golden/make_reference_loss_vectors.py
"""
from __future__ import annotations

import ast
import json
import math
from pathlib import Path
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

REF = Path("/root/reference/unirl")
OUT = Path(__file__).with_name("reference_loss_vectors.npz")


def load_functions(path: Path, *names: str):
    tree = ast.parse(path.read_text())
    nodes = [next(n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name == name) for name in names]
    scope = {"torch": torch, "math": math, "np": np, "Optional": Optional, "List": List, "Dict": Dict, "Tuple": Tuple}
    exec(compile(ast.Module(body=nodes, type_ignores=[]), str(path), "exec"), scope)
    return [scope[name] for name in names]


def meta(obj) -> np.ndarray:
    return np.frombuffer(json.dumps(obj).encode(), dtype=np.uint8)


def bits16(t: torch.Tensor) -> np.ndarray:
    return t.view(torch.int16).numpy()


def main() -> None:
    out: Dict[str, np.ndarray] = {}
    g = torch.Generator().manual_seed(20241125)

    # ---- token inputs shared by GRPO and DRPO ---------------------------------------------------
    n = 4096
    old = -8.0 * torch.rand(n, generator=g)
    new = old + 0.15 * torch.randn(n, generator=g)           # ratios from 0.6 to 1.7: both clip edges
    adv = torch.randn(n, generator=g)
    adv[::17] = 0.0                                          # zero advantages
    # hand-placed tokens: on-policy, the two GRPO clip edges to the ulp, DRPO's +-20 clamp, mu -> 0
    new[0], old[0] = -1.25, -1.25
    for k, r in enumerate((0.8, 1.28, 1.2)):                  # 1 - 0.2, 1 + 0.28, 1 + 0.2
        ld = math.log(r)
        for j, m in enumerate((-3, -1, 0, 1, 3)):             # a few fp32 ulps either side of the edge
            idx = 1 + 5 * k + j
            old[idx] = -2.0
            new[idx] = float(old[idx]) + ld * (1.0 + m * 1.2e-7)
            adv[idx] = 1.0 if j % 2 == 0 else -1.0
    new[20], old[20] = 1.5, -25.0      # log-ratio 26.5  (> 20)
    new[21], old[21] = -40.0, -3.0     # log-ratio -37   (< -20)
    new[22], old[22] = -19.0, -39.0    # log-ratio exactly 20
    new[23], old[23] = -120.0, -120.5  # mu = exp(-120.5) = 0 in fp32: adaptive eps is inf
    new[24], old[24] = -90.0, -89.5    # mu denormal
    new[25], old[25] = -0.0, 0.0       # mu = 1 exactly
    new[26], old[26] = 2.9, 0.0        # ratio 18.2 > 1 + 12.5/mu with mu = 1: DRPO's upper boundary flag set
    new[27], old[27] = 1.9, 0.0        # ratio 6.7 > 1 + 5.0: set for eps 5.0, clear for 12.5
    new[28], old[28] = -15.0, 0.5      # mu > 1 (a log-prob above 0 is not valid, but the function takes it): lower flag
    adv[20:29] = torch.tensor([1.0, -1.0, 0.5, 2.0, -2.0, 1.0, 1.0, -1.5, 1.0])
    out["tok_new"], out["tok_old"], out["tok_adv"] = new.numpy(), old.numpy(), adv.numpy()

    grpo, = load_functions(REF / "algorithms" / "base.py", "_grpo_clip_loss")
    cases = []
    for ci, (lo, hi) in enumerate(((0.2, 0.28), (0.2, None), (0.1, 0.5), (1e-4, None))):
        leaf = new.clone().requires_grad_(True)
        loss, m = grpo(new_logp=leaf, old_logp=old, advantages=adv, clip_range=lo, clip_range_high=hi)
        loss.sum().backward()
        out[f"grpo{ci}_loss"] = loss.detach().numpy()
        out[f"grpo{ci}_grad"] = leaf.grad.numpy()
        out[f"grpo{ci}_metrics"] = np.array([float(m[k]) for k in sorted(m)], dtype=np.float64)
        cases.append({"clip_range": lo, "clip_range_high": hi, "metric_keys": sorted(m)})
    # one element: the reference takes ratio_std = 0 there
    loss1, m1 = grpo(new_logp=new[:1], old_logp=old[:1], advantages=adv[:1], clip_range=0.2)
    out["grpo_single_metrics"] = np.array([float(m1[k]) for k in sorted(m1)], dtype=np.float64)
    out["grpo_cases"] = meta(cases)

    drpo, = load_functions(REF / "algorithms" / "drpo.py", "_drpo_loss")
    cases = []
    for ci, (eps, muw) in enumerate(((5.0, True), (12.5, True), (12.5, False), (0.5, True))):
        leaf = new.clone().requires_grad_(True)
        loss, m = drpo(new_logp=leaf, old_logp=old, advantages=adv, epsilon=eps, mu_weighted=muw)
        loss.sum().backward()
        out[f"drpo{ci}_loss"] = loss.detach().numpy()
        out[f"drpo{ci}_grad"] = leaf.grad.numpy()
        out[f"drpo{ci}_metrics"] = np.array([float(m[k]) for k in sorted(m)], dtype=np.float64)
        cases.append({"epsilon": eps, "mu_weighted": muw, "metric_keys": sorted(m)})
    out["drpo_cases"] = meta(cases)

    # ---- Gaussian KL and the KL-ADV loss ----------------------------------------------------------
    kl_div, kl_adv = load_functions(REF / "algorithms" / "flowdppo.py", "_gaussian_kl_div", "_flowdppo_kl_adv_loss")
    B, S, tail = 4, 3, (4, 8, 8)
    base = torch.randn((B, S) + tail, generator=g)
    # per-(sample, step) perturbation sizes so that the row KLs spread over two decades around the threshold
    scale = torch.tensor([[0.003, 0.01, 0.03], [0.1, 0.02, 0.005], [0.05, 0.05, 0.001], [0.2, 0.008, 0.012]])
    scale = scale.reshape(B, S, 1, 1, 1)
    old_m = base + scale * torch.randn(base.shape, generator=g)
    new_m = base + scale * torch.randn(base.shape, generator=g)
    sigma_t = torch.tensor([0.9, 0.35, 0.12]).reshape(1, S, 1, 1, 1)
    new_lp = 1e-3 * torch.randn(B, S, generator=g)
    old_lp = new_lp + 3e-4 * torch.randn(B, S, generator=g)
    old_lp[0, 0] = new_lp[0, 0]  # ratio exactly 1: neither removal mask can fire
    adv2 = torch.tensor([[1.0, -1.0, 0.5], [-0.5, 2.0, 0.0], [1.5, -2.0, -1.0], [-1.0, 1.0, 1.0]])
    out["kl_sigma"], out["kl_new_lp"], out["kl_old_lp"], out["kl_adv"] = (
        sigma_t.numpy(), new_lp.numpy(), old_lp.numpy(), adv2.numpy())
    cases = []
    for tag, dt in (("f32", torch.float32), ("bf16", torch.bfloat16), ("f16", torch.float16)):
        p, q = new_m.to(dt), old_m.to(dt)
        if dt is torch.float32:
            out["kl_new_f32"], out["kl_old_f32"] = p.numpy(), q.numpy()
        else:
            out[f"kl_new_{tag}_bits"], out[f"kl_old_{tag}_bits"] = bits16(p), bits16(q)
        elem = kl_div(p, q, sigma_t)
        assert elem.dtype is torch.float32
        out[f"kl_{tag}_elem"] = elem.numpy()
        rows = elem.mean(dim=(2, 3, 4))
        out[f"kl_{tag}_rows"] = rows.numpy()
        thr = float(rows.flatten().sort().values[B * S // 2])  # the median row: half the rows on each side...
        for ti, threshold in enumerate((thr * 1.0000001, 1e-5, 1e9)):  # ...then all masked, then none
            leaf = new_lp.clone().requires_grad_(True)
            loss, m = kl_adv(new_logp=leaf, old_logp=old_lp, new_means=p, old_means=q, advantages=adv2,
                             sigma_t=sigma_t, kl_mask_threshold=threshold)
            loss.sum().backward()
            out[f"kladv_{tag}_{ti}_loss"] = loss.detach().numpy()
            out[f"kladv_{tag}_{ti}_grad"] = leaf.grad.numpy()
            out[f"kladv_{tag}_{ti}_metrics"] = np.array([float(m[k]) for k in sorted(m)], dtype=np.float64)
            cases.append({"dtype": tag, "case": ti, "threshold": threshold, "metric_keys": sorted(m)})
    out["kladv_cases"] = meta(cases)

    # ---- sigma schedule, static branch --------------------------------------------------------------
    sched, = load_functions(REF / "sde" / "runtime.py", "get_sigma_schedule")
    sc = []
    for ci, (steps, shift) in enumerate(((28, 3.0), (10, 3.0), (14, 5.0), (12, 1.0), (1, 3.0), (50, 0.5))):
        out[f"sigma{ci}"] = sched(steps, shift).numpy()
        sc.append({"num_steps": steps, "shift": shift})
    out["sigma_cases"] = meta(sc)

    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(out)} arrays)")


if __name__ == "__main__":
    main()
