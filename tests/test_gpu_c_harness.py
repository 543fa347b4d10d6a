"""The C++ harness (tests/harness/c_abi_harness.cpp, built by kiln_amd/csrc/Makefile): the shared
library used from a plain host program through include/kiln_w4a16.h and the HIP runtime, the way
the reference's own harness links its static library (crates/kiln-marlin-gemm/tests/parity.rs).
The wrapper writes a problem's operands and the oracle's result as raw files; the program allocates
with hipMalloc, calls kiln_marlin_w4a16_gemm and applies the row bound itself."""
import subprocess
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
HARNESS = ROOT / "kiln_amd" / "lib" / "c_abi_harness"
G = np.load(Path(__file__).parent / "golden" / "w4a16_small.npz")


def _write_case(tmp_path, x_bits, b, s, y_f32):
    np.ascontiguousarray(x_bits).view(np.uint16).tofile(tmp_path / "a_bf16.bin")
    np.ascontiguousarray(b).view(np.int32).tofile(tmp_path / "b_packed.bin")
    np.ascontiguousarray(s).view(np.uint16).tofile(tmp_path / "s_tiled.bin")
    np.ascontiguousarray(y_f32, dtype=np.float32).tofile(tmp_path / "y_f32.bin")


def _run(mode, tmp_path, m, k, n, g, *extra):
    cmd = [str(HARNESS), mode, str(tmp_path), str(m), str(k), str(n), str(g), *map(str, extra)]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=110)
    assert res.returncode == 0 and res.stdout.rstrip().endswith("OK"), (res.returncode, res.stdout, res.stderr)


def test_harness_needs_nothing_but_the_public_header():
    """Built on the CPU with the library; every kiln symbol it imports is declared in kiln_w4a16.h."""
    assert HARNESS.is_file(), "run kiln_amd.build (make -C kiln_amd/csrc)"
    undefined = subprocess.run(["nm", "-D", "--undefined-only", str(HARNESS)], check=True, capture_output=True,
                               text=True).stdout.split()
    used = {u for u in undefined if u.startswith("kiln_")}
    header = (ROOT / "include" / "kiln_w4a16.h").read_text()
    assert "kiln_marlin_w4a16_gemm" in used and "kiln_w4a16_workspace_bytes" in used
    assert all(u in header for u in used), used


@pytest.mark.gpu
@pytest.mark.parametrize("tag,m,k,n,g", [("g128", 4, 256, 256, 128), ("col", 3, 256, 256, -1)])
def test_golden_vectors_through_the_cpp_harness(tmp_path, tag, m, k, n, g):
    from kiln_amd.marlin_gemm import pack
    b, s = pack.repack_gptq(G[f"{tag}_qweight"], G[f"{tag}_scales_f16"], None, g)
    _write_case(tmp_path, G[f"{tag}_x_bf16"], b, s, G[f"{tag}_y_f32"])
    _run("gemm", tmp_path, m, k, n, g)


@pytest.mark.gpu
@pytest.mark.parametrize("m,k,n,g", [
    (16, 9216, 2560, 128),    # three K slices meeting in the zero-kept region
    (16, 2560, 18432, 128),   # the headline launch
    (64, 4096, 2560, 128),    # mid-M kernel, K sliced
    (600, 2560, 2560, -1),    # matrix-core kernel, K sliced, one scale per column
])
def test_four_host_threads_enter_the_library_at_once(oracle, tmp_path, m, k, n, g):
    """Own stream, workspace and output per thread, first calls racing on a plan cache that has never
    seen the shape (a fresh process per case); every thread's 64th result must equal a serial call
    bit for bit, and that one meets the oracle bound (crates: ARCHITECTURE.md:398-401, several
    inference threads under the GPU read lock)."""
    from kiln_amd.marlin_gemm import pack
    x, q, s_bits = oracle.gen_problem(m, k, n, g, seed=m + k, sigma=0.5 if m > 64 else 1.0)
    b, s = pack.repack_gptq(q, s_bits, None, g)
    _write_case(tmp_path, x, b, s, oracle.c_w4a16_cpu_path(x, q, s_bits, g))
    _run("threads", tmp_path, m, k, n, g, 4)
