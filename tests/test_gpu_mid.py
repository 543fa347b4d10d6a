"""GPU parity of the mid-M kernel (runs of up to 64 rows per pass over the weights), through the
C ABI, against the CPU oracle.  Bound as everywhere: per row max |y - y_ref| <= 1e-2 * max |y_ref|."""
import numpy as np
import pytest
import torch

from kiln_amd import _lib, marlin_gemm
from kiln_amd.marlin_gemm import pack
from tests.gpu_util import bf16_bits, bf16_tensor, row_errors, upload_packed
from tests.test_gpu_parity import ROW_TOL, _run_case

pytestmark = pytest.mark.gpu

MODEL_SHAPES = [(2560, 8192), (4096, 2560), (2560, 18432), (9216, 2560)]


def _takes_mid(L, m, n, k):
    import ctypes
    out = (ctypes.c_int * 8)()
    assert L.kiln_w4a16_debug_gemm_plan(m, n, k, 256, out) == 0
    return bool(out[6])


@pytest.mark.parametrize("m", [33, 48, 64, 65, 96, 128])
@pytest.mark.parametrize("k,n", MODEL_SHAPES)
def test_mid_rows_on_the_model_shapes(oracle, m, k, n):
    """The automatic dispatch of the shipped library at 33...128 rows."""
    assert _takes_mid(_lib.load(), m, n, k)
    x, q, s_bits = oracle.gen_problem(m, k, n, 128, seed=m + n)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    _run_case(oracle, m, k, n, 128, x, b, s, q, s_bits)


@pytest.mark.parametrize("m", [17, 25, 32])
@pytest.mark.parametrize("k,n", MODEL_SHAPES)
def test_one_row_block_per_pass_on_the_model_shapes(oracle, m, k, n):
    """17...32 rows: the kernel computes one row block of 32 per pass (half the loads of A and half the
    products).  The automatic dispatch sends every shape there, the widest output of the shortest K from
    21 rows on; forced through the tuning build all four run it at every row count."""
    L = _lib.load_tuning()
    assert _takes_mid(_lib.load(), m, n, k) == ((k, n) != (2560, 18432) or m >= 21)
    L.kiln_w4a16_debug_mid(1, 0, 0)
    assert _takes_mid(L, m, n, k)
    x, q, s_bits = oracle.gen_problem(m, k, n, 128, seed=3 * m + n)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    _run_case(oracle, m, k, n, 128, x, b, s, q, s_bits)


def _mid_instances():
    cases = []
    for pairs in (1, 2, 3):
        # groups per slice -> (wavefronts, groups per wavefront): 1 -> (1, 1), 3 -> (3, 1), 8 -> (8, 1),
        # 9 -> (8, 2 / 1), 16 -> (8, 2), 20 -> (8, 3 / 2), 24 -> (8, 3), 27 -> (8, 4 / 3), 32 -> (8, 4)
        for gs in (1, 3, 8, 9, 16, 20, 24, 27, 32):
            if not (pairs == 3 and gs > 24):          # three pairs x four groups per wavefront is not built
                cases.append((pairs, gs, 1))
        for gs, ks in ((8, 2), (9, 3), (20, 2), (32, 2), (4, 8)):
            if not (pairs == 3 and gs > 24):
                cases.append((pairs, gs, ks))
    return cases


@pytest.mark.parametrize("m,k,n,forced", [
    (32, 5120, 1024, 0), (17, 4096, 1280, 0), (24, 3584, 2560, 0),   # 40 / 32 / 28 groups: ten wavefronts by plan
    (32, 2560, 2560, 10), (20, 2560, 8192, 10), (32, 1536, 768, 10),  # 20 and 12 groups: ten by override
    (32, 5120, 1024, 8),                                              # and the same weights through eight (two K slices)
    (32, 9216, 512, 0), (17, 18944, 256, 0),                          # K slices of 36 / 37 groups: ten, counter-free exchange
    (64, 18944, 512, 0), (48, 4736, 512, 0), (40, 4736, 512, 10),     # 37 groups a slice beyond 32 rows: no plan of eight
])
def test_ten_wavefronts_up_to_32_rows(oracle, m, k, n, forced):
    """A launch of up to 32 rows may have ten wavefronts per block (ten slots of 16 KiB are all the LDS a
    compute unit has); the planner takes them where eight would hold four groups of a slice each or more.
    Beyond 32 rows blocks of one pair may, where no plan of eight exists (37 groups a slice)."""
    L = _lib.load_tuning()
    x, q, s_bits = oracle.gen_problem(m, k, n, 128, seed=k + n + forced)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    try:
        L.kiln_w4a16_debug_mid(1, 1, {5120: 1 if forced != 8 else 0, 9216: 2, 18944: 4}.get(k, 1))
        L.kiln_w4a16_debug_mid_waves(forced)
        assert _takes_mid(L, m, n, k), (m, k, n)
        _run_case(oracle, m, k, n, 128, x, b, s, q, s_bits)
    finally:
        L.kiln_w4a16_debug_mid(-1, 0, 0)
        L.kiln_w4a16_debug_mid_waves(0)


def test_new_plans_with_one_scale_per_column(oracle):
    """groupsize = -1 through ten wavefronts, a shorter last slice, and 1000 rows on a small weight."""
    for m, k, n in ((32, 5120, 512), (64, 11008, 512), (1000, 1024, 1024)):
        assert _takes_mid(_lib.load(), m, n, k), (m, k, n)
        x, q, s_bits = oracle.gen_problem(m, k, n, -1, seed=m + k)
        b, s = pack.repack_gptq(q, s_bits, None, -1)
        _run_case(oracle, m, k, n, -1, x, b, s, q, s_bits)


@pytest.mark.parametrize("m,k,n,pairs,ks", [
    (64, 11008, 512, 2, 4), (24, 11008, 512, 1, 3), (100, 11008, 768, 2, 3),   # 86 groups: 22 + 22 + 22 + 20, 29 + 29 + 28
    (64, 18944, 256, 1, 7), (17, 8960, 512, 1, 3), (128, 2560, 512, 1, 3),      # 148 = 6 x 22 + 16; 70 = 24 + 24 + 22; 20 = 7 + 7 + 6
    (40, 1408, 256, 1, 2), (32, 3200, 256, 1, 4),                               # 11 = 6 + 5 (a wavefront fewer); 25 = 7 + 7 + 7 + 4
])
def test_a_shorter_last_k_slice(oracle, m, k, n, pairs, ks):
    """K in groups need not be a multiple of the slices: the last slice may have fewer groups (every wavefront
    of it as many as in the other slices or one fewer).  Forced here; the planner takes such a plan where no
    even slicing fits (11008 = 86 groups) or is clearly worse."""
    L = _lib.load_tuning()
    x, q, s_bits = oracle.gen_problem(m, k, n, 128, seed=k + n + ks)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    try:
        L.kiln_w4a16_debug_mid(1, pairs, ks)
        import ctypes
        out = (ctypes.c_int * 8)()
        assert L.kiln_w4a16_debug_gemm_plan(m, n, k, 256, out) == 0 and out[6] == 1 and out[7] == pairs * 16 + ks, list(out)
        _run_case(oracle, m, k, n, 128, x, b, s, q, s_bits)
    finally:
        L.kiln_w4a16_debug_mid(-1, 0, 0)


@pytest.mark.parametrize("pairs,gs,ks", _mid_instances())
def test_every_mid_instance(oracle, pairs, gs, ks):
    """Every (pairs of tiles per block, groups per wavefront) instance, with the groups dealt evenly
    and unevenly, one K slice and several, few rows, a full run, a ragged second run (and, with
    three pairs per block, a last block that holds fewer): each instance is separate straight-line
    code with its own compile-time wait schedule."""
    L = _lib.load_tuning()
    k, n = 128 * gs * ks, 512
    x, q, s_bits = oracle.gen_problem(100, k, n, 128, seed=pairs * 1000 + gs * 10 + ks)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    L.kiln_w4a16_debug_mid(1, pairs, ks)
    # three kernels per instance: one row block per pass (up to 32 rows), two (every run of 64 has more
    # than 32), and the choice by run (80 rows: a run of 64 and one of 16)
    for m in (5, 32, 64, 80, 100):
        assert _takes_mid(L, m, n, k), (m, k, n)
        _run_case(oracle, m, k, n, 128, x[:m], b, s, q, s_bits)


@pytest.mark.parametrize("m,k,n", [(64, 9216, 2560), (128, 4096, 2560), (40, 9216, 2560)])
def test_mid_k_slices_are_deterministic(oracle, m, k, n):
    """K slices of a block's tiles meet in the workspace and are added in slice order by the last
    block to arrive: 1000 launches, identical bits, stopping at the first difference."""
    L = _lib.load_tuning()
    L.kiln_w4a16_debug_mid(1, 0, 0 if k == 9216 else 2)
    x, q, s_bits = oracle.gen_problem(m, k, n, 128, seed=m)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    bt, st = upload_packed(b, s)
    xt = bf16_tensor(x)
    first = marlin_gemm.marlin_w4a16_gemm(xt, bt, st, 128).clone()
    y_ref = oracle.c_w4a16_cpu_path(x, q, s_bits, 128)
    err, _, _ = row_errors(bf16_bits(first), y_ref, oracle)
    assert err.max() <= ROW_TOL
    out = torch.empty_like(first)
    same = torch.ones((), dtype=torch.bool, device=first.device)
    for i in range(1000):
        marlin_gemm.marlin_w4a16_gemm(xt, bt, st, 128, out=out)
        same &= (out == first).all()
        if i % 50 == 49:
            assert bool(same), f"launch {i - 49}...{i} differed from the first"


def test_mid_one_hot_rows(oracle):
    """x = e_r through the mid-M kernel: every output is the dequantised weight itself, which pins
    layout, operand order and scale indexing.  The running rescale multiplies by rounded scale
    ratios, so the bound is one bf16 rounding of the exact value plus 5e-4 of the row's largest."""
    k, n, g, m = 2560, 2560, 128, 64
    codes = oracle.gen_codes(k, n, seed=3)
    s_bits = oracle.gen_scales_f16(k, n, g, seed=3)
    q = oracle.np_pack_gptq(codes)
    b, s = pack.repack_gptq(q, s_bits, None, g)
    rows = [(i * 53 + 7) % k for i in range(m)]
    x = np.zeros((m, k), np.float32)
    for i, r in enumerate(rows):
        x[i, r] = 1.0
    bt, st = upload_packed(b, s)
    assert _takes_mid(_lib.load(), m, n, k)
    y = marlin_gemm.marlin_w4a16_gemm(bf16_tensor(oracle.np_f32_to_bf16(x)), bt, st, g)
    deq = oracle.c_dequant_f32(q, s_bits, g)[rows].astype(np.float64)
    got = oracle.np_bf16_to_f32(bf16_bits(y)).astype(np.float64)
    bound = 2.0 ** -8 * np.abs(deq) + 5e-4 * np.abs(deq).max(axis=1, keepdims=True)
    assert np.all(np.abs(got - deq) <= bound)
    assert (bf16_bits(y) == oracle.np_f32_to_bf16(deq.astype(np.float32))).mean() >= 0.9


@pytest.mark.parametrize("edits", [
    [(3, 0.0)], [(0, 0.0), (19, 0.0)], [(4, 6e-8), (5, 0.02), (6, 6e-8)], [(7, 60000.0), (8, 0.002), (9, 6.1e-5)],
], ids=["zero-group", "zero-first-last", "subnormal", "near-max"])
def test_mid_scale_edge_cases(oracle, edits):
    m, k, n = 64, 2560, 2560
    x, q, _ = oracle.gen_problem(m, k, n, 128, seed=m, sigma=0.5)
    s_bits = oracle.gen_scales_f16(k, n, 128, seed=m).copy()
    for group, value in edits:
        s_bits[group, :] = np.float16(value).view(np.uint16)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    bt, st = upload_packed(b, s)
    y = marlin_gemm.marlin_w4a16_gemm(bf16_tensor(x), bt, st, 128)
    err, yv, _ = row_errors(bf16_bits(y), oracle.c_w4a16_cpu_path(x, q, s_bits, 128), oracle)
    assert np.all(np.isfinite(yv)) and err.max() <= ROW_TOL


def test_mid_closed_forms_and_positive_activations(oracle):
    m, k, n, g = 64, 9216, 2560, 128
    s7 = np.full((k // g, n), np.float16(2.0 ** -7).view(np.uint16), np.uint16)
    x1 = oracle.np_f32_to_bf16(np.ones((m, k), np.float32))
    for code, want in [(8, 0.0), (9, k * 2.0 ** -7), (0, -8 * k * 2.0 ** -7)]:
        b, s = pack.repack_gptq(oracle.np_pack_gptq(np.full((k, n), code, np.int32)), s7, None, g)
        bt, st = upload_packed(b, s)
        y = marlin_gemm.marlin_w4a16_gemm(bf16_tensor(x1), bt, st, g).float()
        assert torch.all((y - want).abs() <= abs(want) * 2.0 ** -8 + 1e-3), (code, want, y.unique()[:8])
    x, q, s_bits = oracle.gen_problem(m, k, n, g, seed=17)
    x = oracle.np_f32_to_bf16(np.abs(oracle.np_bf16_to_f32(x)))      # |N(0,1)|: what down_proj sees
    b, s = pack.repack_gptq(q, s_bits, None, g)
    _run_case(oracle, m, k, n, g, x, b, s, q, s_bits)
