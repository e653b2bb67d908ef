"""Builds tests/native/abi_driver: a C++ host program linked against libunirl_hip.so alone."""

from __future__ import annotations

import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
DRIVER = HERE / "abi_driver"


def build_driver(verbose: bool = True) -> Path:
    sys.path.insert(0, str(ROOT))
    from unirl_amd import build as B

    if not B.LIB_PATH.exists():
        B.build(verbose=verbose)
    tmp = DRIVER.with_suffix(".tmp")
    # the run-time search path is relative to the binary, so the tree can be moved as a whole
    B._run([
        B._hipcc(), *[f for f in B.HIPCC_FLAGS if f != "-fPIC"], f"-I{ROOT / 'include'}", str(HERE / "abi_driver.cpp"),
        f"-L{B.LIB_DIR}", "-lunirl_hip", "-Wl,-rpath,$ORIGIN/../../unirl_amd/lib", "-o", str(tmp),
    ])
    tmp.replace(DRIVER)
    if verbose:
        print(f"[tests.native] built {DRIVER}", flush=True)
    return DRIVER


if __name__ == "__main__":
    build_driver()
