"""Build libkiln_marlin_gemm.so (hipcc, gfx950) in-tree under kiln_amd/lib/.

Mirrors the role of the reference crate's build script
(crates/kiln-marlin-gemm/build.rs:1-108): find the toolkit, compile the kernel
sources for the target architecture, link the runtime.  Unlike the reference
it does not skip silently when the toolkit is missing.
"""
from __future__ import annotations

import os
import subprocess
import sys
from pathlib import Path

CSRC = Path(__file__).resolve().parent / "csrc"
LIB = Path(__file__).resolve().parent / "lib" / "libkiln_marlin_gemm.so"
# the same sources with the plan overrides of the test suite compiled in
TUNING_LIB = LIB.with_name("libkiln_marlin_gemm_tuning.so")


def build(force: bool = True, jobs: int = 8, verbose: bool = False) -> Path:
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    hipcc = Path(rocm) / "bin" / "hipcc"
    if not hipcc.exists():
        raise RuntimeError(f"kiln-marlin-gemm: hipcc not found at {hipcc}; set ROCM_PATH")
    cmd = ["make", "-C", str(CSRC), f"-j{jobs}", f"ROCM_PATH={rocm}"]
    if force:
        cmd.append("-B")
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        sys.stderr.write(res.stdout)
    if res.returncode != 0 or not LIB.exists() or not TUNING_LIB.exists():
        raise RuntimeError("kiln-marlin-gemm: hipcc build failed")
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
