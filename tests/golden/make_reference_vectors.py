"""Writes tests/golden/reference_vectors.npz: outputs of the UniRL reference itself for the four
pieces of the path whose behaviour is control flow or a library recipe rather than a formula, so that closed
forms and brute force do not pin them:

  * normalize_grouped / normalize_global   (unirl/algorithms/normalizers.py:8-84) -- the
    trim-outliers branch, empty groups, the clip, the global-std switch;
  * gather_sde_field                        (unirl/algorithms/base.py:46-80) -- argsort +
    searchsorted + clamp + validation message;
  * the x_T noise recipe                    (unirl/sde/noise.py:26-187) -- blake2b seed derivation,
    one seeded CPU generator per noise group, sharing inside a group, cast as the last step;
  * RolloutTrack.compute_advantages         (unirl/types/rollout_resp.py:220-333) -- the scope /
    normalize / use_global_std switches, root tracks, and the text of the validation errors.

Only runs where the reference tree is mounted (/root/reference).  normalizers.py and noise.py
import nothing but torch and the standard library at module level, so they are loaded from their
files.  base.py cannot be imported (its
package pulls in ray, which is not installed); gather_sde_field is a pure function of torch
tensors, so its definition alone is compiled out of the file's syntax tree and executed with
torch in scope.  Nothing of the reference is written to the output: the file holds the inputs
drawn here and the arrays (or the error text) the reference returned.

Run:  python tests/golden/make_reference_vectors.py
"""
from __future__ import annotations

import ast
import importlib.util
import json
from pathlib import Path
from typing import Dict, List, Optional

import numpy as np
import torch

REF = Path("/root/reference/unirl")
OUT = Path(__file__).with_name("reference_vectors.npz")


def load_file_module(path: Path, name: str):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def load_function(path: Path, func: str):
    tree = ast.parse(path.read_text())
    node = next(n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name == func)
    scope = {"torch": torch, "Optional": Optional, "List": List, "Dict": Dict}
    exec(compile(ast.Module(body=[node], type_ignores=[]), str(path), "exec"), scope)
    return scope[func]


def load_compute_advantages():
    """RolloutTrack.compute_advantages (unirl/types/rollout_resp.py:220-333) as a function of
    (track, ...): the method's definition and the module helper _track_with_field are compiled
    out of the syntax tree.  The module's other helper, _hydrate_tensor_meta, fetches tensors
    from Ray workers; for a plain torch.Tensor it returns its argument unchanged, which is the
    only behaviour this script needs, so an identity takes its place."""
    import dataclasses
    from typing import Any

    path = REF / "types" / "rollout_resp.py"
    tree = ast.parse(path.read_text())
    cls = next(n for n in tree.body if isinstance(n, ast.ClassDef) and n.name == "RolloutTrack")
    method = next(n for n in cls.body if isinstance(n, ast.FunctionDef) and n.name == "compute_advantages")
    helper = next(n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name == "_track_with_field")
    scope = {"torch": torch, "Any": Any, "Dict": Dict, "List": List, "Optional": Optional, "TR": Any,
             "dc_fields": dataclasses.fields, "_hydrate_tensor_meta": lambda value: value}
    exec(compile(ast.Module(body=[helper, method], type_ignores=[]), str(path), "exec"), scope)

    @dataclasses.dataclass
    class Track:  # the four fields the method touches
        sample_ids: list
        parent_ids: Optional[list]
        rewards: Optional[torch.Tensor] = None
        advantages: Optional[torch.Tensor] = None

    return scope["compute_advantages"], Track


def main() -> None:
    out: Dict[str, np.ndarray] = {}
    g = torch.Generator().manual_seed(20240611)

    # ---- normalizers -------------------------------------------------------
    norm = load_file_module(REF / "algorithms" / "normalizers.py", "_ref_normalizers")
    rewards = torch.randn(24, generator=g) * 2.0 + 0.5
    rewards[5] = 9.0   # outliers for the trimmed statistics
    rewards[17] = -7.0
    groups = [
        [0, 1, 2, 3, 4, 5, 6, 7],          # 8 members
        [8, 9, 10],                         # 3 members (trim_size rounds to 0 at ratio 0.25)
        [],                                 # empty: skipped
        [11, 12],                           # 2 members: never trimmed
        [13],                               # singleton: std() is NaN
        [23, 14, 22, 15, 21, 16, 20, 17, 19, 18],  # 10 members, unordered
    ]
    out["ng_rewards"] = rewards.numpy()
    out["ng_groups"] = np.frombuffer(json.dumps(groups).encode(), dtype=np.uint8)
    cases = []
    for ci, (trim, glob, clip) in enumerate(
        [(0.0, False, None), (0.0, True, None), (0.0, False, 1.0), (0.125, False, None), (0.25, False, None),
         (0.25, True, 1.5), (0.4, False, None), (0.5, False, None), (0.1, False, 0.5)]
    ):
        res = norm.normalize_grouped(rewards.clone(), groups, epsilon=1e-8, clip_max=clip,
                                     trim_outliers_ratio=trim, use_global_std=glob)
        out[f"ng_case{ci}_out"] = res.numpy()
        cases.append({"trim": trim, "use_global_std": glob, "clip_max": clip})
    out["ng_cases"] = np.frombuffer(json.dumps(cases).encode(), dtype=np.uint8)
    out["nglobal_out"] = norm.normalize_global(rewards.clone(), epsilon=1e-8).numpy()
    out["nglobal_clip_out"] = norm.normalize_global(rewards.clone(), epsilon=1e-6, clip_max=0.75).numpy()

    # ---- gather_sde_field --------------------------------------------------
    gather = load_function(REF / "algorithms" / "base.py", "gather_sde_field")
    t = torch.randn(3, 6, 2, 5, generator=g)
    sde_indices = torch.tensor([7, 2, 9, 0, 4, 13])
    out["gs_tensor"] = t.numpy()
    out["gs_indices"] = sde_indices.numpy()
    gcases = []
    for gi, target in enumerate([[2, 9], [0, 4, 7, 13], [9], [4, 4, 0], [13, 0], [7, 2, 9, 0, 4, 13]]):
        out[f"gs_case{gi}_out"] = gather(t, sde_indices, target, field_name="sde_means").numpy()
        gcases.append({"target": target})
    for target in ([2, 3], [14], [-1, 0], [5, 6, 7]):
        try:
            gather(t, sde_indices, target, field_name="sde_logp")
            gcases.append({"target": target, "error": None})
        except ValueError as e:
            gcases.append({"target": target, "error": str(e)})
    for a, b in ((None, sde_indices), (t, None)):
        try:
            gather(a, b, [2], field_name="sde_logp")
        except ValueError as e:
            gcases.append({"target": None, "none_arg": 0 if a is None else 1, "error": str(e)})
    out["gs_cases"] = np.frombuffer(json.dumps(gcases).encode(), dtype=np.uint8)

    # ---- x_T noise recipe ----------------------------------------------------
    noise = load_file_module(REF / "sde" / "noise.py", "_ref_noise")
    gids = ["p0", "p0", "p1", "p0", "p2", "7", "p1"]
    out["nz_gids"] = np.frombuffer(json.dumps(gids).encode(), dtype=np.uint8)
    out["nz_seeds"] = np.array([noise._derive_group_seed(1234, g) for g in gids], dtype=np.int64)
    out["nz_seed_big"] = np.array([noise._derive_group_seed((1 << 62) + 5, "prompt-000017")], dtype=np.int64)
    for tag, shape in (("a", (4, 8, 8)), ("b", (3,)), ("c", (2, 3, 5, 7))):
        x = noise.regen_initial_noise(gids, 1234, shape, torch.device("cpu"), torch.float32)
        out[f"nz_{tag}_f32"] = x.numpy()
        xb = noise.regen_initial_noise(gids, 1234, shape, torch.device("cpu"), torch.bfloat16)
        out[f"nz_{tag}_bf16_bits"] = xb.view(torch.int16).numpy()
    out["nz_latents_same"] = noise.generate_latents(
        4, (2, 9), torch.device("cpu"), torch.float32, init_same_noise=True, samples_per_prompt=2,
        noise_group_ids=["g0", "g0", "g1", "g1"], base_seed=99).numpy()

    # ---- RolloutTrack.compute_advantages ------------------------------------
    compute_advantages, Track = load_compute_advantages()
    rew = (torch.rand(24, generator=g) < 0.5).float() + 0.25 * torch.randn(24, generator=g)
    rew[8:12] = 1.0  # an all-equal group
    pids = [f"p{i // 4}" for i in range(24)]
    out["ca_rewards"] = rew.numpy()
    out["ca_parent_ids"] = np.frombuffer(json.dumps(pids).encode(), dtype=np.uint8)
    ca_cases = []
    for ci, kw in enumerate([{}, {"normalize": False}, {"use_global_std": True}, {"scope": "global"},
                             {"scope": "global", "normalize": False}, {"eps": 1e-4}]):
        t = compute_advantages(Track([str(i) for i in range(24)], pids, rew.clone()), **kw)
        out[f"ca_case{ci}_out"] = t.advantages.numpy()
        ca_cases.append(kw)
    out["ca_cases"] = np.frombuffer(json.dumps(ca_cases).encode(), dtype=np.uint8)
    out["ca_root_out"] = compute_advantages(Track([str(i) for i in range(24)], None, rew.clone())).advantages.numpy()
    one = compute_advantages(Track(["a", "b", "c"], ["x", "y", "z"], torch.tensor([1.0, 2.0, 3.0])))
    out["ca_singletons_out"] = one.advantages.numpy()
    ca_errors = {}
    for name, ids, r in (("interleaved", ["a", "b", "a", "b", "a", "b"], torch.arange(6.0)),
                         ("nonuniform", ["a", "a", "a", "b", "b"], torch.arange(5.0)),
                         ("no_rewards", ["a"], None)):
        try:
            compute_advantages(Track([str(i) for i in range(len(ids))], ids, r))
            ca_errors[name] = None
        except ValueError as e:
            ca_errors[name] = str(e)
    out["ca_errors"] = np.frombuffer(json.dumps(ca_errors).encode(), dtype=np.uint8)

    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(out)} arrays)")


if __name__ == "__main__":
    main()
