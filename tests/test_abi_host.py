"""CPU-only checks: the C-ABI library loads and exports what include/unirl_hip.h declares,
argument errors come back as statuses (no kernel is launched), and the host-side logic of the
Python layer (validation, index math, error types, loud failure without a device)."""

import ctypes
import math
import re
from pathlib import Path

import pytest
import torch

from oracle import flowdppo as ofd
from oracle import schedule as osch

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "unirl_hip.h"


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(unirl_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(built_lib):
    from unirl_amd import _native

    names = declared_symbols()
    assert len(names) >= 18
    handle = ctypes.CDLL(str(built_lib))
    for name in names:
        assert hasattr(handle, name), f"{name} declared in the header but not exported"
    assert sorted(_native.EXPORTED_SYMBOLS) == names, "ctypes signature table and header disagree"


def test_shipped_library_exports_exactly_the_declared_entry_points(built_lib):
    """The dynamic symbol table of the shipped library holds the header's entry points and no other
    `unirl_*` name: no yardstick kernel, timeline hook or other measurement aid is exported.  Every
    declaration in the header cites the reference lines it replaces, except the one allocation-free
    entry point, whose comment says that it has no counterpart there."""
    import shutil
    import subprocess

    nm = shutil.which("nm") or shutil.which("llvm-nm", path="/opt/rocm/llvm/bin")
    if nm is None:
        pytest.skip("no nm on this host")
    out = subprocess.run([nm, "-D", "--defined-only", str(built_lib)], check=True, capture_output=True, text=True).stdout
    exported = sorted({line.split()[-1] for line in out.splitlines() if re.search(r"\bunirl_[a-z0-9_]+$", line)})
    assert exported == declared_symbols()
    assert not [n for n in exported if "calib" in n or "trace" in n]
    # each entry point's comment names the reference (a path under unirl/ with a line), the library-level
    # calls (version, status text, workspace size and fill, scratch size) aside
    text = HEADER.read_text()
    library_level = {"unirl_abi_version", "unirl_status_string", "unirl_workspace_bytes", "unirl_workspace_init",
                     "unirl_lmhead_logp_scratch_bytes"}
    missing = []
    starts = sorted((re.search(r"^(?:int|size_t|const char\*) " + n + r"\(", text, flags=re.M).start(), n) for n in exported)
    for k, (decl, name) in enumerate(starts):
        if name in library_level:
            continue
        comment = text[(starts[k - 1][0] if k else 0):decl]  # everything since the previous declaration
        comment = re.sub(r"\s*\n\s*\*?\s*", " ", comment)  # undo the comment's line breaks
        if name == "unirl_gaussian_kl_mask_static" or name.endswith("_noalloc"):
            assert "no counterpart in the reference" in comment, name
        elif not re.search(r"unirl/[a-z0-9_/]+\.py:\d+", comment):
            missing.append(name)
    assert not missing, f"declarations whose comment cites no reference line: {missing}"


def test_version_status_strings_and_workspace(built_lib):
    from unirl_amd import _native as N

    L = N.lib()
    assert L.unirl_abi_version() == N.ABI_VERSION == 6
    assert f"#define UNIRL_ABI_VERSION {N.ABI_VERSION}" in (ROOT / "include" / "unirl_hip.h").read_text()
    assert L.unirl_workspace_bytes() >= 64 * 1024
    assert L.unirl_status_string(0) == b"ok"
    for code in range(-6, 0):
        assert L.unirl_status_string(code) not in (b"ok", b"unknown status")
    assert L.unirl_status_string(-99) == b"unknown status"


def test_argument_errors_return_statuses_without_launching(built_lib):
    from unirl_amd import _native as N

    L = N.lib()
    # bad dtype / kind / shape / null pointers: rejected before any HIP call
    assert L.unirl_token_logp_entropy(None, 7, 1, 10, 10, None, 1.0, None, None, None, None) == -3
    assert L.unirl_token_logp_entropy(None, N.BF16, 1, 0, 0, None, 1.0, None, None, None, None) == -2
    assert L.unirl_token_logp_entropy(None, N.BF16, 1, 10, 10, None, 1.0, None, None, None, None) == -1
    assert L.unirl_token_logp_entropy(None, N.BF16, 0, 10, 10, None, 1.0, None, None, None, None) == 0
    args = [None, N.F32, None, N.F32, None, None, None, None, 0, None, 0.99, 0.7, N.SDE_FLOW, 2, 16, None, None,
            None, 0, None, 0, None]
    assert L.unirl_sde_step_logp(*args) == -1
    args[12] = 9
    assert L.unirl_sde_step_logp(*args) == -3
    args[12] = N.SDE_FLOW
    args[14] = 0
    assert L.unirl_sde_step_logp(*args) == -2
    assert L.unirl_gaussian_kl_mask(None, None, N.BF16, None, 1, 2, 8, 0.01, None, None, None, 0, None) == -1
    assert L.unirl_gaussian_kl_mask(None, None, N.BF16, None, 0, 2, 8, 0.01, None, None, None, 0, None) == -2
    assert L.unirl_workspace_init(None, 0, None) == -1
    p = N.RatioLossParams(kind=5)
    assert L.unirl_ratio_loss_fwd(None, None, None, None, None, 1, 0, 4, ctypes.byref(p), None, None, None, 0,
                                  None) == -3
    assert L.unirl_group_advantages(None, 2, 2, 1, 1e-8, 0, 0, None, None) == -1
    assert L.unirl_group_advantages(None, 0, 2, 1, 1e-8, 0, 0, None, None) == 0
    good = N.RatioLossParams(kind=N.LOSS_GRPO, agg_mode=N.AGG_TOKEN_MEAN, clip_low=0.2, clip_high=0.2, adv_per_token=1)
    fake = ctypes.c_void_p(0x10000)
    # the one-pass step: no gradient buffer, no workspace, a flat layout with per-sequence advantages
    assert L.unirl_ratio_loss_fwd_bwd(fake, fake, fake, None, None, 0, 0, 8, ctypes.byref(good), 1.0, -1, None, fake,
                                      fake, 1 << 30, None) == -1
    assert L.unirl_ratio_loss_fwd_bwd(fake, fake, fake, None, None, 0, 0, 8, ctypes.byref(good), 1.0, -1, fake, fake,
                                      None, 0, None) == -4
    good.adv_per_token = 0
    assert L.unirl_ratio_loss_fwd_bwd(fake, fake, fake, None, None, 0, 0, 8, ctypes.byref(good), 1.0, -1, fake, fake,
                                      fake, 1 << 30, None) == -1
    # the Flow-DPPO loss step: row limit, NULL outputs
    assert L.unirl_flowdppo_step(fake, fake, N.BF16, fake, 1, 1 << 20, 64, fake, fake, fake, 0.01, 1.0, fake, fake,
                                 None, fake, fake, 1 << 30, None) == -6
    assert L.unirl_flowdppo_step(fake, fake, N.BF16, fake, 1, 4, 64, fake, fake, fake, 0.01, 1.0, fake, None, None,
                                 fake, fake, 1 << 30, None) == -1
    # misaligned pointer
    assert L.unirl_token_logp_entropy(ctypes.c_void_p(0x1001), N.BF16, 1, 10, 10, ctypes.c_void_p(0x1000), 1.0,
                                      ctypes.c_void_p(0x2000), None, None, None) == -5


def test_status_to_exception_mapping(built_lib):
    from unirl_amd import _native as N

    N.check(0, "x")
    with pytest.raises(ValueError):
        N.check(-2, "x")
    with pytest.raises(N.UnirlHipError):
        N.check(1, "x")
    with pytest.raises(TypeError):
        N.dtype_code(torch.float64)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from unirl_amd import _native as N

    monkeypatch.setattr(N, "_lib", None)
    monkeypatch.setattr(N, "LIB_PATH", tmp_path / "libunirl_hip.so")
    with pytest.raises(RuntimeError, match="no CPU or eager-torch path"):
        N.lib()


def test_cpu_tensors_are_refused_not_emulated(built_lib):
    from unirl_amd import models, ops, sde
    from unirl_amd.algorithms import _drpo_loss, _grpo_clip_loss

    x = torch.randn(2, 4, 4)
    s = torch.tensor(0.5)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        sde.FlowSDEStrategy().denoise(x, x, s, s * 0.9, eta=0.7)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        models.token_logp(torch.randn(3, 10), torch.zeros(3, dtype=torch.int64))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _grpo_clip_loss(new_logp=x, old_logp=x, advantages=x, clip_range=0.2)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _drpo_loss(new_logp=x, old_logp=x, advantages=x, epsilon=5.0)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.gaussian_kl_mask(x, x, s, 0.01, reduce_from_dim=1)


def test_sigma_schedule_matches_oracle():
    from unirl_amd.sde import calculate_dynamic_mu, get_sigma_schedule

    for T, shift in ((28, 3.0), (10, 3.0), (14, 5.0), (12, 1.0)):
        assert torch.equal(get_sigma_schedule(T, shift), osch.sigma_schedule(T, shift))
    assert get_sigma_schedule(4).shape == (5,)
    # linear in the sequence length between (256, 0.5) and (4096, 1.15)
    assert abs(calculate_dynamic_mu(256) - 0.5) < 1e-12 and abs(calculate_dynamic_mu(4096) - 1.15) < 1e-12
    assert abs(calculate_dynamic_mu(2176) - 0.825) < 1e-12


def test_strategy_surface():
    from unirl_amd import sde

    assert sde.FlowSDEStrategy.canonical_name == "flow"
    assert sde.DanceSDEStrategy.canonical_name == "dance"
    assert sde.CPSSDEStrategy.canonical_name == "cps"
    for cls in sde.STRATEGIES.values():
        obj = cls(config=None)
        assert isinstance(obj, sde.SDEStrategy) and isinstance(obj, sde.StepStrategy)
        obj.reset()
        obj.init_schedule(torch.ones(3))
    with pytest.raises(TypeError):
        sde.FlowSDEStrategy(None)  # config is keyword-only
    ode = sde.DPM2Strategy(config=None)
    assert ode.canonical_name == "dpm2" and isinstance(ode, sde.StepStrategy) and not isinstance(ode, sde.SDEStrategy)
    ode.init_schedule(torch.linspace(1, 0, 5))
    ode.reset()


def test_clip_schedule():
    from unirl_amd.algorithms import _resolve_clip_range_from_schedule as f

    assert f(0.2, "constant", 0.7) == 0.2
    assert abs(f(0.2, "linear_decay", 0.5) - 0.15) < 1e-12
    assert abs(f(0.2, "cosine_decay", 0.5) - 0.1) < 1e-12
    assert abs(f(0.2, "cosine_decay", 1.0)) < 1e-12 and f(0.2, "anything-else", 1.0) == 0.2


def test_gather_sde_field_host_path_and_errors():
    from unirl_amd.algorithms import gather_sde_field

    g = torch.Generator().manual_seed(0)
    t = torch.randn(3, 5, 2, 4, generator=g)
    idx = torch.tensor([7, 2, 9, 0, 4])
    for target in ([2, 9], [0, 4, 7], [9], [4, 4], []):
        got = gather_sde_field(t, idx, target, field_name="sde_means")
        if target:
            assert torch.equal(got, ofd.gather_by_lookup(t, idx, target))
            assert torch.equal(got, ofd.gather_sde_field(t, idx, target))
        else:
            assert got.shape == (3, 0, 2, 4)
    with pytest.raises(ValueError, match=r"target steps \[3\] not in sde_indices"):
        gather_sde_field(t, idx, [2, 3], field_name="sde_logp")
    with pytest.raises(ValueError, match="is None"):
        gather_sde_field(None, idx, [2])
    with pytest.raises(ValueError, match="is None"):
        gather_sde_field(t, None, [2])


def test_compute_advantages_validation_needs_no_device():
    from unirl_amd.types import RolloutTrack, compute_advantages

    r = torch.tensor([1.0, 0.0, 1.0, 0.0, 1.0, 0.0])
    with pytest.raises(ValueError, match="not in group-by-parent contiguous order"):
        compute_advantages(r, ["a", "b", "a", "b", "a", "b"])
    with pytest.raises(ValueError, match="non-uniform group sizes"):
        compute_advantages(r[:5], ["a", "a", "a", "b", "b"])
    assert compute_advantages(r, None).tolist() == [0.0] * 6  # root track: zeros, no kernel
    assert compute_advantages(r[:0], []).shape == (0,)
    with pytest.raises(ValueError, match="no rewards"):
        RolloutTrack(sample_ids=["a"], parent_ids=["p"]).compute_advantages()
    empty = RolloutTrack(sample_ids=[], parent_ids=[], rewards=torch.zeros(0))
    assert empty.compute_advantages() is empty


def test_expand_advantages_validation():
    from unirl_amd.algorithms import GRPO

    with pytest.raises(ValueError, match="advantages batch=3 != lengths=2"):
        GRPO._expand_advantages_to_tokens(torch.zeros(3), torch.ones(2, dtype=torch.int64), dtype=torch.float32,
                                          device=torch.device("cpu"))


def test_algorithm_constructors_validate():
    from unirl_amd.algorithms import DRPO, GRPO, FlowDPPO, FlowGRPO

    with pytest.raises(ValueError):
        GRPO()
    with pytest.raises(ValueError):
        DRPO()
    with pytest.raises(ValueError):
        FlowGRPO(params=None)
    with pytest.raises(ValueError):
        FlowDPPO(params=None)

    class P:
        ar = object()
        diffusion = object()

    with pytest.raises(ValueError):
        DRPO(pipeline=P(), old_logp_source="nope")
    with pytest.raises(ValueError):
        FlowDPPO(params=None, pipeline=P(), old_logp_source="nope")
    g = GRPO(pipeline=P(), clip_range=0.2, clip_range_high=0.28)
    assert g.stage is P.ar and g.sampling_temperature == 0.7 and g.supports_multi_update
    assert FlowDPPO(params=None, pipeline=P()).recomputes_anchor()
    assert not FlowGRPO(params=None, pipeline=P()).recomputes_anchor()
    assert FlowGRPO(params=None, pipeline=P(), old_logp_source="replay").recomputes_anchor()


def test_bench_refuses_more_than_one_gpu():
    """The bench measures one GPU's share of the path; asking for more exits with a message."""
    import subprocess
    import sys

    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in (r.stderr + r.stdout)
    assert not r.stdout.strip().startswith("{")  # no result line


def test_header_is_plain_c_and_a_c_program_links(built_lib, tmp_path):
    """The boundary is a C ABI: the header compiles as C99 (no C++ in it), and a C program linked
    against the library alone (no torch, no Python) reads its version and a status string."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler on this host")
    src = tmp_path / "abi.c"
    src.write_text(
        '#include <string.h>\n#include "unirl_hip.h"\n'
        "int main(void) {\n"
        "  if (unirl_abi_version() != UNIRL_ABI_VERSION) return 1;\n"
        '  if (strcmp(unirl_status_string(UNIRL_OK), "ok") != 0) return 2;\n'
        "  if (unirl_workspace_bytes() < 65536) return 3;\n"
        "  /* argument errors come back as statuses before anything touches a device */\n"
        "  if (unirl_token_logp_entropy(0, UNIRL_BF16, 1, 10, 10, 0, 1.0f, 0, 0, 0, 0) != UNIRL_E_NULL) return 4;\n"
        "  return 0;\n}\n"
    )
    exe = tmp_path / "abi"
    lib_dir = str(Path(built_lib).parent)
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", f"-I{HEADER.parent}", str(src),
                    f"-L{lib_dir}", "-lunirl_hip", f"-Wl,-rpath,{lib_dir}", "-o", str(exe)], check=True)
    assert subprocess.run([str(exe)]).returncode == 0


def test_dpm2_coefficients_reproduce_the_oracle_on_the_host():
    """Branch selection and scalar coefficients of the DPM-Solver-2 step are host logic: evaluated
    with the kernel's fp32 operation order in torch on the CPU, they reproduce the oracle's
    trajectory bit for bit, for an fp32 and a float64 schedule and for a solver restarted mid-way."""
    from oracle import dpm2 as odpm
    from unirl_amd import _native as N
    from unirl_amd.sde.kernels import dpm2_coefficients

    def emulate(branch, c, v, x, m1):
        x0 = x - c.sigma * v
        if branch == N.DPM2_DDIM:
            eps = (x - c.one_minus_s * x0) / c.s
            return x0, c.one_minus_t * x0 + c.sqrt_t2 * eps
        if branch == N.DPM2_FIRST:
            return x0, c.c1 * x - c.c2 * x0
        d1 = c.inv_r0 * (x0 - m1)
        return x0, (c.c1 * x - c.c2 * x0) - c.half_c2 * d1

    g = torch.Generator().manual_seed(8)
    for sig, start in ((osch.sigma_schedule(12, 3.0), 0), (osch.sigma_schedule(9, 1.0).double(), 0),
                       (osch.sigma_schedule(12, 3.0), 4)):
        solver = odpm.Dpm2Solver(sig)
        x = torch.randn(3, 50, generator=g)
        warm, m1, seen = 0, None, []
        for i in range(start, sig.numel() - 1):
            v = torch.randn(3, 50, generator=g)
            want = solver.step(v, x, i)
            branch, c = dpm2_coefficients(sig, i, warm)
            seen.append(branch)
            m1, got = emulate(branch, c, v, x, m1)
            assert torch.equal(got, want), (i, branch)
            warm = min(2, warm + 1)
            x = want
        n = sig.numel() - 1 - start
        first = N.DPM2_DDIM if start == 0 else N.DPM2_FIRST
        assert seen == [first] + [N.DPM2_SECOND] * (n - 2) + [N.DPM2_DDIM]
    with pytest.raises(IndexError):
        dpm2_coefficients(osch.sigma_schedule(4, 3.0), 4, 0)


def test_metric_names_are_the_references():
    """Metric keys become W&B series, so they are part of the contract: the names below are the
    reference's (unirl/algorithms/base.py:98-103, :147-156; drpo.py:151-158; flowdppo.py:124-137)."""
    from unirl_amd import ops
    from unirl_amd.algorithms._fused import ABSDIFF_METRICS, DRPO_METRICS, GRPO_METRICS

    assert set(GRPO_METRICS) == {"ratio_mean", "ratio_std", "ratio_min", "ratio_max", "clip_fraction",
                                 "clipfrac_gt_one", "clipfrac_lt_one", "approx_kl"}
    assert set(DRPO_METRICS) == {"ratio_mean", "ratio_max", "approx_kl", "drpo_penalty_mean", "clipfrac_upper",
                                 "clipfrac_lower"}
    assert set(ABSDIFF_METRICS) == {"rollout_replay_logp_absdiff_mean", "rollout_replay_logp_absdiff_max"}
    assert set(ops.FLOWDPPO_METRIC_SLOTS) - {"loss_mean"} == {
        "ratio_mean", "ratio_std", "ratio_min", "ratio_max", "approx_kl", "kl_new_old_mean", "kl_new_old_max",
        "kl_mask_fraction", "pos_rm_fraction", "neg_rm_fraction", "masked_fraction", "unmasked_fraction"}
    for table in (GRPO_METRICS, DRPO_METRICS, ABSDIFF_METRICS, ops.FLOWDPPO_METRIC_SLOTS):
        assert len(set(table.values())) == len(table)  # one slot of the metrics vector each


def test_per_sample_view_never_hands_stride_zero_for_several_samples(monkeypatch):
    """A sample stride of 0 means "densely packed" in the C ABI: a tensor broadcast over the
    samples must be copied, not passed with its stride of 0 (the kernel would then read B blocks
    from a buffer that holds one)."""
    from unirl_amd import _native as N
    from unirl_amd import ops

    monkeypatch.setattr(N, "require_device", lambda t, name: None)
    one = torch.arange(12.0).reshape(1, 3, 4)
    for B in (2, 7):
        t, stride = ops._per_sample_view(one.expand(B, 3, 4), "noise")
        assert stride == 12 and t.is_contiguous() and t.shape == (B, 3, 4)
        assert torch.equal(t[B - 1], one[0])
    # one sample: any stride is harmless and reported as D
    t, stride = ops._per_sample_view(one.expand(1, 3, 4), "noise")
    assert stride == 12
    # slices of a stack keep their stride and are not copied
    stack = torch.zeros(4, 5, 3, 4)
    t, stride = ops._per_sample_view(stack[:, 2], "sample")
    assert stride == 60 and t.data_ptr() == stack[:, 2].data_ptr()
    # outputs may not overlap across samples
    with pytest.raises(ValueError):
        ops._per_sample_view(one.expand(3, 3, 4), "prev_out", writable=True)


def test_replay_velocity_blocks_must_be_disjoint():
    """The batched replay writes the velocities' gradient in the velocities' own layout: a view whose
    (sample, step) blocks overlap is copied first (overlapping rows would be written concurrently
    where autograd expects their sum)."""
    from unirl_amd.ops import _blocks_disjoint as disjoint

    assert disjoint(12 * 5, 4, 5, 12, 5)        # dense [B=4, S=12, D=5]
    assert disjoint(5, 4, 20, 12, 5)            # step-major dense [S=12, B=4, D=5]
    assert disjoint(70, 4, 5, 12, 5)            # padded samples
    assert not disjoint(1, 4, 5, 12, 5)         # samples one element apart
    assert not disjoint(60, 4, 4, 12, 5)        # steps closer than a block
    assert not disjoint(30, 4, 5, 12, 5)        # a sample starts inside the previous sample's steps
    assert disjoint(1, 1, 5, 12, 5) and disjoint(100, 4, 3, 1, 5)  # an extent of 1 leaves its stride free


def test_release_library_reads_no_environment_knobs(built_lib):
    """The launch-shape knobs of the measurement build (UNIRL_* environment variables) must not
    exist in the shipped library: an exported variable must never change a production launch."""
    blob = built_lib.read_bytes()
    names = set(re.findall(rb"UNIRL_[A-Z0-9_]{3,}", blob))
    assert not names, f"environment knob names in the release library: {sorted(names)}"
    assert b"getenv" not in blob or b"UNIRL_" not in blob


def test_conforming_operands_are_handed_over_without_a_copy(monkeypatch):
    """Tensors that already have the dtype, device and layout a kernel reads are passed as they
    are -- no detach, cast or contiguous() hop, each of which costs more host time than the
    whole argument check; anything else is converted once."""
    from unirl_amd import _native as N
    from unirl_amd import ops

    monkeypatch.setattr(N, "require_device", lambda t, name: None)
    cpu = torch.device("cpu")
    new = torch.randn(4, 8, requires_grad=True)
    old = torch.randn(4, 8)
    adv = torch.randn(4)
    lengths = torch.tensor([8, 4, 2, 1])
    assert N.as_operand(new, torch.float32, cpu) is new          # requires grad: still no detach
    assert N.as_operand(lengths, torch.int64, cpu) is lengths
    half = N.as_operand(old.half(), torch.float32, cpu)
    assert half.dtype == torch.float32 and half.is_contiguous()
    strided = N.as_operand(old.t(), torch.float32, cpu)
    assert strided.is_contiguous() and torch.equal(strided, old.t())
    assert ops._flat2(new, "new") is new and ops._kernel_dtype(old) is old
    assert ops._kernel_dtype(old.double()).dtype == torch.float32
    plan = ops.RatioLossPlan(new, old, adv, kind=N.LOSS_GRPO, lengths=lengths)
    assert plan.nw is new and plan.od is old and plan.adv is adv and plan.seq is lengths
    # the sigma arguments of the SDE step: an fp32 scalar passes untouched
    s = torch.tensor(0.5)
    assert ops._sigma_arg(s, 4, cpu, "sigma")[0] is s


def test_dense_from_agrees_with_torch_on_strided_views():
    """`_dense_from(t, k)` is `t[0, .., 0].is_contiguous()` (k leading indices) without making the view."""
    from unirl_amd import ops

    g = torch.Generator().manual_seed(3)
    base = torch.zeros(6, 5, 4, 3, 2)
    views = [base, base[:, 1], base[:, :, ::2], base.transpose(1, 2), base.transpose(3, 4), base[..., 0],
             base[:, :, :, :, :1], base.permute(1, 0, 2, 3, 4), base[:, :, 1:3], base.expand(6, 5, 4, 3, 2),
             torch.zeros(3, 1, 4).expand(3, 7, 4), torch.zeros(4, 4)[:, :1], torch.zeros(2, 3, 1, 5).transpose(1, 2)]
    for t in views:
        for k in range(0, t.dim()):
            idx = (0,) * k
            assert ops._dense_from(t, k) == t[idx].is_contiguous(), (tuple(t.shape), t.stride(), k)


def test_replay_slot_tables_are_checked_and_cached():
    from unirl_amd import ops

    a = ops._replay_slot_arrays((0, 2, 3), (1, 3, 4), 5)
    assert list(a[0]) == [0, 2, 3] and list(a[1]) == [1, 3, 4] and a[2] == 3
    assert ops._replay_slot_arrays((0, 2, 3), (1, 3, 4), 5) is a
    for bad in (((0, 5), (1, 2)), ((0,), (1, 2)), ((), ()), ((-1,), (0,))):
        with pytest.raises(ValueError):
            ops._replay_slot_arrays(bad[0], bad[1], 5)
    with pytest.raises(ValueError):
        ops._replay_slot_arrays(tuple(range(65)), tuple(range(65)), 100)


def test_replay_slots_follow_latents_at_on_the_host():
    """`replay_slots` is `LatentSegment.latents_at` (unirl/types/segments/latent.py:82-97) for a step and
    its successor: the first slot that holds the step, KeyError with the stored indices when it is not
    stored, RuntimeError without indices."""
    from unirl_amd import sde

    stored = torch.tensor([0, 3, 4, 4, 7, 8])
    assert sde.replay_slots(stored, [3, 7]) == ([1, 4], [2, 5])
    assert sde.replay_slots([5, 1, 2], [1]) == ([1], [2])          # unsorted storage
    assert sde.replay_slots(stored, []) == ([], [])
    with pytest.raises(KeyError, match=r"step_idx=5 not in stored indices=\[0, 3, 4, 4, 7, 8\]"):
        sde.replay_slots(stored, [4])                              # step 4 is stored, its successor is not
    with pytest.raises(KeyError, match="step_idx=1 "):
        sde.replay_slots(stored, [1])
    with pytest.raises(RuntimeError, match="missing indices"):
        sde.replay_slots(None, [0])
