"""Build libunirl_hip.so for gfx950 with hipcc, in-tree.

    python -m unirl_amd.build            # compile every csrc/*.hip and link
    python -m unirl_amd.build --tune     # measurement build beside it (libunirl_hip_tune.so)

hipcc cross-compiles without a GPU.  Objects go to ``unirl_amd/lib/obj`` and the
shared library to ``unirl_amd/lib/libunirl_hip.so``; both are git-ignored build
products.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path
from typing import List

PKG_DIR = Path(__file__).resolve().parent
CSRC_DIR = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
OBJ_DIR = LIB_DIR / "obj"
LIB_PATH = LIB_DIR / "libunirl_hip.so"

ARCH = "gfx950"

# -ffp-contract=off: a*b+c stays two roundings like eager torch; the kernels
#   spell out fmaf() where a fused multiply-add is wanted.
# -packed-fp32-ops off: keep the compiler from forming v_pk_{add,mul,fma}_f32.
HIPCC_FLAGS: List[str] = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")
    return exe


def _run(cmd: List[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # The host pass of hipcc does not know the packed-fp32 target feature and says so.
    noise = "is not a recognized feature for this target"
    out = "\n".join(line for line in proc.stdout.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if out.strip():
        print(out, file=sys.stderr)


# sources of the measurement build only (yardstick kernels, the timeline's host side)
TUNE_ONLY = ("calib_tune.hip",)


def sources(tune: bool = False) -> List[Path]:
    return sorted(p for p in CSRC_DIR.glob("*.hip") if tune or p.name not in TUNE_ONLY)


def build(verbose: bool = True, jobs: int | None = None, *, tune: bool = False, out: Path | None = None,
          extra_flags: List[str] | None = None) -> Path:
    """Compile every kernel source and link the shared library. Always recompiles.

    ``tune=True`` makes a measurement build (``-DUNIRL_TUNE -DUNIRL_TRACE``: launch-shape knobs read
    from the environment, device-side timeline marks, plus the yardstick kernels of
    ``calib_tune.hip``); it must be given its own ``out`` path and is never the library the
    package loads.
    """
    hipcc = _hipcc()
    if tune and out is None:
        raise ValueError("a tune build needs its own output path (out=...)")
    lib_path = Path(out) if out is not None else LIB_PATH
    obj_dir = OBJ_DIR if out is None else lib_path.parent / (lib_path.stem + "_obj")
    obj_dir.mkdir(parents=True, exist_ok=True)
    srcs = sources(tune)
    if not srcs:
        raise RuntimeError(f"no .hip sources under {CSRC_DIR}")
    objs = [obj_dir / (s.stem + ".o") for s in srcs]
    jobs = jobs or min(len(srcs), max(1, (os.cpu_count() or 2) // 2))
    flags = list(HIPCC_FLAGS) + (["-DUNIRL_TUNE", "-DUNIRL_TRACE"] if tune else []) + list(extra_flags or [])

    def compile_one(pair):
        src, obj = pair
        if verbose:
            print(f"[unirl_amd.build] hipcc {src.name}", flush=True)
        _run([hipcc, *flags, "-c", str(src), "-o", str(obj)])

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(srcs, objs)))

    tmp = lib_path.with_suffix(".so.tmp")
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)])
    os.replace(tmp, lib_path)
    if verbose:
        print(f"[unirl_amd.build] linked {lib_path}", flush=True)
    return lib_path


TUNE_LIB_PATH = LIB_DIR / "libunirl_hip_tune.so"


if __name__ == "__main__":
    if "--tune" in sys.argv[1:]:
        # the measurement build `bench.py --timeline` and the launch-shape sweeps load
        build(tune=True, out=TUNE_LIB_PATH)
    else:
        build()
