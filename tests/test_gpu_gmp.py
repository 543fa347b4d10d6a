"""GPU parity of the small-M kernel with wavefront-private staging of the activations, every
instance, through the C ABI against the CPU oracle."""
import ctypes

import numpy as np
import pytest
import torch

from kiln_amd import _lib, marlin_gemm
from kiln_amd.marlin_gemm import pack
from tests.gpu_util import bf16_bits, bf16_tensor, row_errors, upload_packed
from tests.test_gpu_parity import ROW_TOL, _run_case

pytestmark = pytest.mark.gpu


def _plan(L, m, n, k):
    out = (ctypes.c_int * 8)()
    assert L.kiln_w4a16_debug_decode_plan(m, n, k, 256, out) == 0
    return list(out)


def _instances():
    cases = []
    for tiles in (1, 2, 3, 4, 5, 6):
        for waves, gs in ((12, 12), (12, 24), (12, 36), (12, 48), (12, 60), (12, 72), (8, 20), (16, 20), (3, 3), (1, 1),
                          (12, 20), (12, 31)):
            gpw = -(-gs // waves)
            if gpw > (6 if tiles <= 2 else 3) or tiles * gpw > 16:
                continue
            cases.append((tiles, waves, gs, 1))
        cases.append((tiles, 12, 24, 3))
        cases.append((tiles, 8, 8, 2))
    return cases


@pytest.mark.parametrize("tiles,waves,gs,ks", _instances())
def test_every_private_staging_instance(oracle, tiles, waves, gs, ks):
    """Every (tiles per block, groups per wavefront) instance with 16 rows and with up to 4 (one
    load per group of A), groups dealt evenly and unevenly, one slice and several, a column count
    the tiles per block do not divide: each is straight-line code with its own wait schedule."""
    L = _lib.load_tuning()
    k, n = 128 * gs * ks, 256
    x, q, s_bits = oracle.gen_problem(16, k, n, 128, seed=tiles * 1000 + waves * 10 + gs + ks)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    L.kiln_w4a16_debug_gmp(tiles, waves, ks)
    for m in (16, 9, 3, 1):
        p = _plan(L, m, n, k)
        assert p[7] == -tiles and p[0] == ks, (m, p)
        _run_case(oracle, m, k, n, 128, x[:m], b, s, q, s_bits)


@pytest.mark.parametrize("m,k,n,tiles,waves,ks", [
    (16, 9216, 2560, 1, 12, 1), (16, 9216, 2560, 2, 12, 1), (1, 9216, 2560, 1, 12, 1), (4, 9216, 2560, 2, 12, 3),
    (16, 2560, 18432, 5, 12, 1), (1, 2560, 18432, 5, 12, 1), (16, 2560, 8192, 2, 12, 1), (16, 4096, 2560, 1, 16, 1),
])
def test_private_staging_on_the_model_shapes(oracle, m, k, n, tiles, waves, ks):
    L = _lib.load_tuning()
    L.kiln_w4a16_debug_gmp(tiles, waves, ks)
    assert _plan(L, m, n, k)[7] == -tiles
    x, q, s_bits = oracle.gen_problem(m, k, n, 128, seed=m + tiles)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    _run_case(oracle, m, k, n, 128, x, b, s, q, s_bits)


def test_private_staging_k_slices_are_deterministic_and_one_hot_exact(oracle):
    """K slices meet tile by tile (the wavefront that summed a tile stores, counts and, if last,
    adds in slice order): 1000 launches identical; and x = e_r gives bf16(dequant[r, :]) exactly."""
    L = _lib.load_tuning()
    m, k, n = 16, 9216, 2560
    L.kiln_w4a16_debug_gmp(2, 12, 3)
    x, q, s_bits = oracle.gen_problem(m, k, n, 128, seed=2)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    bt, st = upload_packed(b, s)
    xt = bf16_tensor(x)
    first = marlin_gemm.marlin_w4a16_gemm(xt, bt, st, 128).clone()
    out = torch.empty_like(first)
    same = torch.ones((), dtype=torch.bool, device=first.device)
    for i in range(1000):
        marlin_gemm.marlin_w4a16_gemm(xt, bt, st, 128, out=out)
        same &= (out == first).all()
        if i % 50 == 49:
            assert bool(same), f"launch {i - 49}...{i} differed from the first"
    rows = [0, 1, 127, 128, 4000, 9215, 77, 5000, 8191, 8192, 3071, 3072, 6143, 6144, 255, 256]
    xh = np.zeros((len(rows), k), np.float32)
    for i, r in enumerate(rows):
        xh[i, r] = 1.0
    for plan in ((2, 12, 3), (1, 12, 1)):
        L.kiln_w4a16_debug_gmp(*plan)
        y = marlin_gemm.marlin_w4a16_gemm(bf16_tensor(oracle.np_f32_to_bf16(xh)), bt, st, 128)
        want = oracle.np_f32_to_bf16(oracle.c_dequant_f32(q, s_bits, 128)[rows])
        assert np.array_equal(bf16_bits(y), want)


@pytest.mark.parametrize("tiles,waves,gs,n", [(1, 12, 48, 2560), (1, 12, 72, 2560), (2, 12, 48, 1024), (1, 12, 36, 512)])
def test_private_staging_slot_reuse_is_ordered(oracle, tiles, waves, gs, n):
    """Three and more groups per wavefront reuse the two staging slots: the request that refills a
    slot must come after the reads of its previous occupant have completed, not merely been
    issued.  Checked where a violation showed (first rows of a group overwritten early): on the
    first launch after fresh uploads against the oracle, then over 2000 launches bit for bit."""
    L = _lib.load_tuning()
    k, m = 128 * gs, 16
    x, q, s_bits = oracle.gen_problem(m, k, n, 128, seed=gs + n)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    L.kiln_w4a16_debug_gmp(tiles, waves, 1)
    assert _plan(L, m, n, k)[7] == -tiles
    _run_case(oracle, m, k, n, 128, x, b, s, q, s_bits)
    bt, st = upload_packed(b, s)
    xt = bf16_tensor(x)
    first = marlin_gemm.marlin_w4a16_gemm(xt, bt, st, 128).clone()
    out = torch.empty_like(first)
    same = torch.ones((), dtype=torch.bool, device=first.device)
    for i in range(2000):
        if i % 100 == 0:
            bt, st = upload_packed(b, s)                     # fresh copies: cold lines, as on a first call
            xt = bf16_tensor(x)
        marlin_gemm.marlin_w4a16_gemm(xt, bt, st, 128, out=out)
        same &= (out == first).all()
    assert bool(same)
