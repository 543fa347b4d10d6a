"""Pins for the CPU oracle.

Each test checks the oracle against something other than its own formula: the
reference's own known answers (cited), numpy / torch library routines, an
independent big-integer or float64 computation, or a closed-form invariant.
"""
import numpy as np
import pytest
import torch


# ---------------------------------------------------------------- conversions

def test_f16_to_f32_all_patterns(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib().ko_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    # reference's own checks, quantized.rs:271-280
    assert oracle.lib().ko_f16_to_f32(0x3C00) == 1.0
    assert np.float32(oracle.lib().ko_f16_to_f32(0x8000)).view(np.uint32) == 0x80000000


def test_f32_to_f16_matches_ieee_rne(oracle):
    rng = np.random.default_rng(1)
    pats = rng.integers(0, 2**32, size=300000, dtype=np.uint64).astype(np.uint32)
    # dense coverage of the f16 range incl. subnormal / overflow boundaries and exact ties
    halfs = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    halfs = halfs[np.isfinite(halfs)]
    ties = ((halfs[:-1].astype(np.float64) + halfs[1:].astype(np.float64)) / 2).astype(np.float32)
    near = np.concatenate([np.nextafter(ties, np.float32(np.inf)),
                           np.nextafter(ties, np.float32(-np.inf))])
    edge = np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e-8, 2.98e-8, 2.9802322e-8,
                     5.96e-8, 6.1e-5, np.inf, -np.inf, 0.13333334, 2.0 / 15.0], dtype=np.float32)
    vals = np.concatenate([pats.view(np.float32), halfs, ties, near, edge])
    vals = vals[~np.isnan(vals)]
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    f = oracle.lib().ko_f32_to_f16
    got = np.array([f(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_bf16_rne_matches_torch(oracle):
    rng = np.random.default_rng(2)
    vals = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    vals = np.concatenate([vals[np.isfinite(vals)],
                           np.array([1.0, 1.00390625, 1.01171875, -0.001, 100.0], np.float32)])
    want = torch.from_numpy(vals.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got_np = oracle.np_f32_to_bf16(vals)
    # f32 values that round up to inf aside, the integer-add trick is torch's RNE
    assert np.array_equal(got_np, want)
    f = oracle.lib().ko_f32_to_bf16
    got_c = np.array([f(float(v)) for v in vals[:20000]], dtype=np.uint16)
    assert np.array_equal(got_c, want[:20000])
    back = oracle.np_bf16_to_f32(want)
    assert np.array_equal(back.view(np.uint32), want.astype(np.uint32) << 16)


# ------------------------------------------------------------------------ LCG

def _lcg_python(count, seed, mul):
    """Independent big-integer restatement of parity.rs:22-31."""
    out, state = [], seed & (2**64 - 1)
    for _ in range(count):
        state = (state * 6364136223846793005 + 1442695040888963407) % 2**64
        bits = (state >> 33) & 0x7FFFFFFF
        v = np.float32(np.float32(bits) / np.float32(2147483647)) - np.float32(0.5)
        out.append(np.float32(v * np.float32(mul)))
    return np.array(out, dtype=np.float32)


@pytest.mark.parametrize("seed,mul", [(0xC0FFEE5EED ^ 128 ^ (256 << 16), 0.5),
                                      (0xDEADBEEF ^ 16 ^ (2560 << 24), 0.25)])
def test_lcg_three_ways(oracle, seed, mul):
    want = _lcg_python(4096, seed, mul)
    assert np.array_equal(oracle.c_lcg_fill(4096, seed, mul), want)
    assert np.array_equal(oracle.np_lcg_fill(4096, seed, mul), want)
    assert want.min() >= -0.5 * mul and want.max() <= 0.5 * mul
    assert abs(float(want.mean())) < 0.02 * mul


# ------------------------------------------------------- GPTQ unpack / dequant

def test_gptq_known_answer_all_fives(oracle):
    """quantized.rs:308-372: codes 5, zero 8, scale 0.5 -> -1.5 everywhere, [out, in]."""
    k, n, g = 16, 8, 8
    qweight = np.full((k // 8, n), sum(5 << (4 * i) for i in range(8)), dtype=np.uint32)
    qzeros = np.full((k // g, n // 8), sum(8 << (4 * i) for i in range(8)), dtype=np.uint32)
    scales = np.full((k // g, n), np.float16(0.5).view(np.uint16), dtype=np.uint16)
    for fn in (oracle.c_gptq_dequant_bf16, oracle.np_gptq_dequant_bf16):
        out = fn(qweight, scales, qzeros, g)
        assert out.shape == (n, k)
        assert np.all(oracle.np_bf16_to_f32(out) == -1.5)
    # the zero-point-8 shortcut (no qzeros tensor) is the same thing
    assert np.all(oracle.np_bf16_to_f32(oracle.c_gptq_dequant_bf16(qweight, scales, None, g)) == -1.5)


def test_gptq_known_answer_nibble_order(oracle):
    """quantized.rs:375-419: codes 0..7 in one word, zero 0, scale 1 -> 0..7 along K."""
    k, n, g = 8, 8, 8
    word = sum(i << (4 * i) for i in range(8))
    qweight = np.full((1, n), word, dtype=np.uint32)
    qzeros = np.zeros((1, 1), dtype=np.uint32)
    scales = np.full((1, n), np.float16(1.0).view(np.uint16), dtype=np.uint16)
    for fn in (oracle.c_gptq_dequant_bf16, oracle.np_gptq_dequant_bf16):
        out = oracle.np_bf16_to_f32(fn(qweight, scales, qzeros, g))
        assert out.shape == (n, k)
        assert np.array_equal(out, np.tile(np.arange(8, dtype=np.float32), (n, 1)))
    assert np.array_equal(oracle.np_unpack_gptq(qweight)[:, 0], np.arange(8))


def test_gptq_known_answer_loader(oracle):
    """loader.rs:2244-2252: code 5, zero 8, f16 scale 1.0 -> -3.0, output [out, in] bf16."""
    k, n, g = 64, 128, 8
    qweight = np.full((k // 8, n), sum(5 << (4 * i) for i in range(8)), dtype=np.uint32)
    qzeros = np.full((k // g, n // 8), sum(8 << (4 * i) for i in range(8)), dtype=np.uint32)
    scales = np.full((k // g, n), 0x3C00, dtype=np.uint16)
    out = oracle.c_gptq_dequant_bf16(qweight, scales, qzeros, g)
    assert out.shape == (128, 64)
    assert np.all(oracle.np_bf16_to_f32(out) == -3.0)


def test_gptq_pack_unpack_roundtrip_and_c_vs_numpy(oracle):
    rng = np.random.default_rng(3)
    k, n, g = 256, 64, 128
    codes = rng.integers(0, 16, size=(k, n)).astype(np.int32)
    zeros = rng.integers(0, 16, size=(k // g, n)).astype(np.int32)
    scales = rng.uniform(0.002, 0.02, size=(k // g, n)).astype(np.float16).view(np.uint16)
    q_c, q_np = oracle.c_pack_gptq(codes), oracle.np_pack_gptq(codes)
    assert np.array_equal(q_c, q_np)
    assert np.array_equal(oracle.np_unpack_gptq(q_c), codes)
    # brute force with python ints for a few entries
    for (r, c) in [(0, 0), (7, 3), (8, 3), (129, 63), (255, 17)]:
        assert (int(q_c[r // 8, c]) >> (4 * (r % 8))) & 0xF == codes[r, c]
    qz = oracle.np_pack_qzeros(zeros)
    a = oracle.c_gptq_dequant_bf16(q_c, scales, qz, g)
    b = oracle.np_gptq_dequant_bf16(q_c, scales, qz, g)
    assert np.array_equal(a, b)
    # f32 dequant with zero-point 8: exact, so C, numpy and float64 agree bit for bit
    d_c, d_np = oracle.c_dequant_f32(q_c, scales, g), oracle.np_dequant_f32(q_c, scales, g)
    d64 = (codes.astype(np.float64) - 8) * np.repeat(scales.view(np.float16).astype(np.float64), g, 0)
    assert np.array_equal(d_c, d_np)
    assert np.array_equal(d_c.astype(np.float64), d64)


# ------------------------------------------------------------------ quantiser

def test_quantizer_ties_clamp_and_zero_group(oracle):
    """lib.rs:393-427: hand-computed column. max|w| = 7.5 -> s = f16(1.0) = 1."""
    k, n = 128, 256
    w = np.zeros((k, n), dtype=np.float32)
    col = np.array([7.5, -7.5, 0.5, -0.5, 1.5, 2.5, -2.5, 0.49999997, 3.4, -3.6, 6.5, -6.5],
                   dtype=np.float32)
    w[:len(col), 0] = col
    want_codes = np.array([15, 0, 9, 7, 10, 11, 5, 8, 11, 4, 15, 1])  # half AWAY from zero
    want_deq = np.array([7, -8, 1, -1, 2, 3, -3, 0, 3, -4, 7, -7], dtype=np.float32)
    for fn in (oracle.c_quantize, oracle.np_quantize):
        codes, scales, deq = fn(w, 128)
        assert scales.shape == (1, n) and codes.shape == (k, n)
        assert scales[0, 0] == 0x3C00
        assert np.array_equal(codes[:len(col), 0], want_codes)
        assert np.array_equal(deq[:len(col), 0], want_deq)
        # lib.rs:405-407: an all-zero group takes max=1.0 -> s = f16(2/15); codes 8; deq 0
        assert scales[0, 1] == np.float16(np.float32(2.0) / np.float32(15.0)).view(np.uint16)
        assert np.all(codes[:, 1] == 8) and np.all(deq[:, 1] == 0.0)


def test_quantizer_where_the_scale_rounds_to_zero_or_infinity(oracle):
    """Worked by hand from lib.rs:405-427.  A group of magnitude 1e-30: s = f16(1.3e-31) = 0, so w / s is
    +inf, -inf or (0 / 0) NaN; `as i32` gives i32::MAX, i32::MIN, 0; `raw + 8` is an i32 sum -- i32::MAX + 8
    wraps to a negative value in a release build (a debug build panics), the clamp makes it code 0; MIN + 8
    clamps to 0; NaN gives 8.  Dequantised values are (code - 8) * 0.  A group of magnitude 3e38: s = f16
    infinity, w / inf = 0, code 8, dequant 0 * inf = NaN."""
    k, n = 128, 256
    w = np.zeros((k, n), dtype=np.float32)
    w[:4, 0] = [1e-30, -1e-30, 0.0, 5e-31]
    w[:3, 1] = [3e38, -3e38, 1.0]
    for fn in (oracle.c_quantize, oracle.np_quantize):
        with np.errstate(all="ignore"):
            codes, scales, deq = fn(w, 128)
        assert scales[0, 0] == 0x0000 and scales[0, 1] == 0x7C00
        assert list(codes[:4, 0]) == [0, 0, 8, 0]
        assert np.all(deq[:4, 0] == 0.0)
        assert list(codes[:3, 1]) == [8, 8, 8] and np.all(np.isnan(deq[:3, 1]))
    from kiln_amd.marlin_gemm import pack
    with np.errstate(all="ignore"):
        b, s, deq = pack.quantize_and_pack(w, k, n, 128)          # the product's host quantiser: the same codes
    q, _ = pack.unpack_to_gptq(b, s, 128)
    got = oracle.np_unpack_gptq(q.view(np.uint32))
    assert list(got[:4, 0]) == [0, 0, 8, 0] and list(got[:3, 1]) == [8, 8, 8]


@pytest.mark.parametrize("groupsize", [128, -1])
def test_quantizer_invariants_and_c_vs_numpy(oracle, groupsize):
    k, n = 256, 256
    w = oracle.c_lcg_fill(k * n, 0xC0FFEE5EED ^ k ^ (n << 16), 0.5).reshape(k, n)
    c1, s1, d1 = oracle.c_quantize(w, groupsize)
    c2, s2, d2 = oracle.np_quantize(w, groupsize)
    assert np.array_equal(c1, c2) and np.array_equal(s1, s2) and np.array_equal(d1, d2)
    g = k if groupsize == -1 else groupsize
    assert c1.min() >= 0 and c1.max() <= 15
    s = np.repeat(s1.view(np.float16).astype(np.float64), g, axis=0)
    # scale definition against float64 arithmetic (f16 rounding allowed: rel 2^-11)
    max_abs = np.abs(w.astype(np.float64)).reshape(k // g, g, n).max(axis=1)
    assert np.allclose(s1.view(np.float16).astype(np.float64), 2 * max_abs / 15, rtol=2.0**-11)
    # nearest-grid-point property away from the +8 clamp
    err = np.abs(w.astype(np.float64) - d1.astype(np.float64))
    unclamped = (w.astype(np.float64) / s) < 7.5
    assert np.all(err[unclamped] <= s[unclamped] * (0.5 + 1e-6))
    assert np.array_equal(d1.astype(np.float64), (c1.astype(np.float64) - 8) * s)


# ------------------------------------------------------- Marlin layout (legacy)

def test_marlin_perm_values_from_reference_text(oracle):
    """Values derived by hand from lib.rs:296-357."""
    perm = oracle.marlin_weight_perm()
    assert perm.shape == (1024,)
    assert sorted(perm.tolist()) == list(range(1024))
    assert perm[0:8].tolist() == [0, 128, 8, 136, 16, 144, 24, 152]
    assert perm[32:40].tolist() == [32, 160, 40, 168, 48, 176, 56, 184]
    assert perm[1016:1024].tolist() == [871, 999, 879, 1007, 887, 1015, 895, 1023]
    assert oracle.marlin_scale_perm()[:10].tolist() == [0, 8, 16, 24, 32, 40, 48, 56, 1, 9]
    assert oracle.marlin_scale_perm_single()[:10].tolist() == [0, 1, 8, 9, 16, 17, 24, 25, 2, 3]


def test_marlin_pack_shapes_and_bijection(oracle):
    rng = np.random.default_rng(5)
    k, n = 128, 256
    codes = rng.integers(0, 16, size=(k, n)).astype(np.int32)
    scales = rng.integers(0, 65536, size=(1, n)).astype(np.uint16)
    packed, s_perm = oracle.marlin_pack(codes, scales, 128)
    assert packed.shape == (k // 16, n * 16 // 8) and packed.dtype == np.int32   # lib.rs:119
    assert s_perm.shape == (1, n)
    assert sorted(s_perm.ravel().tolist()) == sorted(scales.ravel().tolist())
    hist = np.bincount(np.concatenate([(packed.view(np.uint32) >> (4 * i)) & 0xF
                                       for i in range(8)], axis=None), minlength=16)
    assert np.array_equal(hist, np.bincount(codes.ravel(), minlength=16))
    # first word: perm[0..8] of the first 16x16 tile, tile element p = (row p/16, col p%16)
    first = [int(codes[p // 16, p % 16]) for p in [0, 128, 8, 136, 16, 144, 24, 152]]
    assert [(int(packed.view(np.uint32)[0, 0]) >> (4 * i)) & 0xF for i in range(8)] == first


# --------------------------------------------------------------------- matmul

def test_gemm_exact_special_cases(oracle):
    k, n, g = 256, 256, 128
    rng = np.random.default_rng(7)
    codes = rng.integers(0, 16, size=(k, n)).astype(np.int32)
    scales = rng.uniform(0.002, 0.02, size=(k // g, n)).astype(np.float16).view(np.uint16)
    q = oracle.np_pack_gptq(codes)
    deq = oracle.c_dequant_f32(q, scales, g)
    # one-hot activations pick out a weight row exactly
    x = np.zeros((4, k), dtype=np.float32)
    rows = [0, 127, 128, 255]
    for i, r in enumerate(rows):
        x[i, r] = 1.0
    y = oracle.c_w4a16_cpu_path(oracle.np_f32_to_bf16(x), q, scales, g)
    assert np.array_equal(y, deq[rows])
    # all codes 8 -> exactly zero whatever x is
    q8 = oracle.np_pack_gptq(np.full((k, n), 8, np.int32))
    xr = oracle.gen_normal_bf16(3, k, 1.0, seed=11)
    assert np.all(oracle.c_w4a16_cpu_path(xr, q8, scales, g) == 0.0)
    # codes 9, scale 2^-7, x = 1 -> K * 2^-7 exactly
    q9 = oracle.np_pack_gptq(np.full((k, n), 9, np.int32))
    s7 = np.full((k // g, n), np.float16(2.0**-7).view(np.uint16), np.uint16)
    ones = oracle.np_f32_to_bf16(np.ones((2, k), np.float32))
    assert np.all(oracle.c_w4a16_cpu_path(ones, q9, s7, g) == k * 2.0**-7)


def test_gemm_f32_against_float64_and_numpy(oracle):
    m, k, n, g = 5, 512, 256, 128
    x, q, s = oracle.gen_problem(m, k, n, g, seed=4)
    w = oracle.c_dequant_f32(q, s, g)
    y32 = oracle.c_gemm_f32(x, w)
    y64 = oracle.c_gemm_f64(x, w)
    ynp = oracle.np_bf16_to_f32(x).astype(np.float64) @ w.astype(np.float64)
    assert np.allclose(y64, ynp, rtol=1e-12, atol=1e-12)
    scale = np.abs(y64).max(axis=1, keepdims=True)
    assert np.all(np.abs(y32 - y64) <= 2e-5 * scale)   # f32 accumulation noise only
    assert np.array_equal(oracle.c_w4a16_cpu_path(x, q, s, g), y32)


# ----------------------------------------------------------------------- LoRA

def _bf(a):
    from oracle import ref
    return ref.np_f32_to_bf16(np.asarray(a, dtype=np.float32))


def test_lora_known_values(oracle):
    """lora_loader.rs:342-367: delta = x A^T B^T * 2 for the identity-like A."""
    x = _bf([[1, 0, 0, 0], [0, 1, 0, 0]])
    a = _bf([[1, 0, 0, 0], [0, 1, 0, 0]])          # [r=2, in=4]
    b = _bf([[1, 0], [0, 1], [1, 1]])               # [out=3, r=2]
    y = np.zeros((2, 3), dtype=np.float32)
    oracle.c_lora_delta_add(y, x, a, b, 2.0)
    assert np.array_equal(y, np.array([[2, 0, 2], [0, 2, 2]], dtype=np.float32))


def test_lora_adds_to_base(oracle):
    """lora_loader.rs:369-401: zero base weight, x=[1,2,3,4] -> [1, 2, 1.5]."""
    x = _bf([[1, 2, 3, 4]])
    a = _bf([[1, 0, 0, 0], [0, 1, 0, 0]])
    b = _bf([[1, 0], [0, 1], [0.5, 0.5]])
    y = np.zeros((1, 3), dtype=np.float32)
    oracle.c_lora_delta_add(y, x, a, b, 1.0)
    assert np.array_equal(y, np.array([[1.0, 2.0, 1.5]], dtype=np.float32))


def test_merge_concat_identity(oracle):
    """adapter_merge.rs:1444-1483: B_cat A_cat == sum_i w_i B_i A_i (ranks may differ)."""
    import ctypes
    rng = np.random.default_rng(9)
    k, n, ranks, weights = 12, 10, [2, 3], [0.7, 0.3]
    a_list = [rng.standard_normal((r, k)).astype(np.float32) for r in ranks]
    b_list = [rng.standard_normal((n, r)).astype(np.float32) for r in ranks]
    a_cat = np.empty((sum(ranks), k), np.float32)
    b_cat = np.empty((n, sum(ranks)), np.float32)
    PP = ctypes.c_void_p * len(ranks)
    L = oracle.lib()
    L.ko_merge_concat.restype = None
    L.ko_merge_concat(PP(*[a.ctypes.data for a in a_list]), PP(*[b.ctypes.data for b in b_list]),
                      (ctypes.c_int * 2)(*ranks), (ctypes.c_float * 2)(*weights), 2,
                      ctypes.c_int(k), ctypes.c_int(n), ctypes.c_void_p(a_cat.ctypes.data),
                      ctypes.c_void_p(b_cat.ctypes.data))
    assert a_cat.shape == (5, k) and np.array_equal(a_cat[:2], a_list[0])
    want = sum(w * (b.astype(np.float64) @ a.astype(np.float64))
               for w, a, b in zip(weights, a_list, b_list))
    assert np.allclose(b_cat.astype(np.float64) @ a_cat.astype(np.float64), want, atol=1e-5)


# ----------------------------------------------------------------- generators

def test_generators_are_deterministic_and_in_range(oracle):
    c1, c2 = oracle.gen_codes(256, 512, 0), oracle.gen_codes(256, 512, 0)
    assert np.array_equal(c1, c2) and c1.min() == 0 and c1.max() == 15
    assert not np.array_equal(c1, oracle.gen_codes(256, 512, 1))
    hist = np.bincount(c1.ravel(), minlength=16) / c1.size
    assert np.all(np.abs(hist - 1 / 16) < 0.005)
    s = oracle.gen_scales_f16(256, 512, 128, 0).view(np.float16).astype(np.float32)
    assert s.shape == (2, 512) and s.min() >= 0.002 - 1e-5 and s.max() <= 0.02 + 1e-5
    x = oracle.np_bf16_to_f32(oracle.gen_normal_bf16(64, 2560, 1.0, 0))
    assert abs(float(x.mean())) < 0.02 and abs(float(x.std()) - 1.0) < 0.02
    x5 = oracle.np_bf16_to_f32(oracle.gen_normal_bf16(64, 2560, 0.5, 0))
    assert abs(float(x5.std()) - 0.5) < 0.01


def test_swiglu_closed_forms_and_library(oracle):
    """silu(x) = x * sigmoid(x): silu(0) = 0, silu(x) - silu(-x) = x, silu(x) -> x for large x,
    silu(-large) -> -0, and the values of a library silu (torch, f64)."""
    import torch
    x = np.concatenate([np.array([0.0, 1.0, -1.0, 20.0, -20.0, 88.0, -88.0, 1e-8], np.float32),
                        np.linspace(-12, 12, 4001, dtype=np.float32)])
    ones = np.ones_like(x)
    s = oracle.c_swiglu_f32(x, ones)
    assert s[0] == 0.0
    assert abs(s[1] - 0.7310585786300049) < 1e-7 and abs(s[2] + 0.2689414213699951) < 1e-7
    assert s[3] == np.float32(20.0 / (1 + np.exp(-20.0))) and abs(s[4]) < 1e-7
    assert s[5] == 88.0 and -1e-35 < s[6] <= 0.0
    sm = oracle.c_swiglu_f32(-x, ones)
    assert np.allclose(s.astype(np.float64) - sm.astype(np.float64), x.astype(np.float64), rtol=0, atol=2e-6)
    lib = torch.nn.functional.silu(torch.from_numpy(x).double()).numpy()
    assert np.array_equal(s, lib.astype(np.float32))
    up = np.linspace(-3, 3, x.size, dtype=np.float32)
    h = oracle.c_swiglu_f32(x, up)
    assert np.array_equal(h, (lib * up.astype(np.float64)).astype(np.float32))
