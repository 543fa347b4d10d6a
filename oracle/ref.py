"""Python face of the CPU oracle -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Two things live here:

* a ctypes binding to ``oracle/_build/libw4a16_oracle.so`` (the C restatement
  in ``w4a16_oracle.c``), and
* an independent numpy twin of the integer / bit-level pieces (conversions,
  quantiser, GPTQ pack/unpack, dequantisation, the Marlin permutation), used
  to cross-check the C code, plus the seeded synthetic-input generators every
  test and the benchmark share.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` import this module, and only as the checker.

Reference citations are relative to the reference checkout.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "_build" / "libw4a16_oracle.so"
_lib = None


def build(force: bool = False) -> Path:
    """Compile the C oracle with gcc (oracle/Makefile)."""
    if force or not _LIB_PATH.exists():
        subprocess.run(["make", "-C", str(_HERE)] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        L = ctypes.CDLL(str(_LIB_PATH))
        c = ctypes
        vp = c.c_void_p
        L.ko_f16_to_f32.restype = c.c_float
        L.ko_f16_to_f32.argtypes = [c.c_uint16]
        L.ko_f32_to_f16.restype = c.c_uint16
        L.ko_f32_to_f16.argtypes = [c.c_float]
        L.ko_bf16_to_f32.restype = c.c_float
        L.ko_bf16_to_f32.argtypes = [c.c_uint16]
        L.ko_f32_to_bf16.restype = c.c_uint16
        L.ko_f32_to_bf16.argtypes = [c.c_float]
        L.ko_lcg_fill.restype = c.c_uint64
        L.ko_lcg_fill.argtypes = [vp, c.c_size_t, c.c_uint64, c.c_float]
        L.ko_quantize.restype = None
        L.ko_quantize.argtypes = [vp, c.c_int, c.c_int, c.c_int, vp, vp, vp]
        L.ko_pack_gptq.restype = None
        L.ko_pack_gptq.argtypes = [vp, c.c_int, c.c_int, vp]
        L.ko_gptq_dequant_bf16.restype = None
        L.ko_gptq_dequant_bf16.argtypes = [vp, vp, vp, c.c_int, c.c_int, c.c_int, vp]
        L.ko_dequant_f32.restype = None
        L.ko_dequant_f32.argtypes = [vp, vp, c.c_int, c.c_int, c.c_int, vp]
        L.ko_gemm_f32.restype = None
        L.ko_gemm_f32.argtypes = [vp, vp, c.c_int, c.c_int, c.c_int, vp]
        L.ko_swiglu_f32.restype = None
        L.ko_swiglu_f32.argtypes = [vp, vp, c.c_size_t, vp]
        L.ko_gemm_f64.restype = None
        L.ko_gemm_f64.argtypes = [vp, vp, c.c_int, c.c_int, c.c_int, vp]
        L.ko_w4a16_cpu_path.restype = None
        L.ko_w4a16_cpu_path.argtypes = [vp, vp, vp, c.c_int, c.c_int, c.c_int, c.c_int, vp, vp]
        L.ko_lora_delta_add_f32.restype = None
        L.ko_lora_delta_add_f32.argtypes = [vp, vp, vp, c.c_float, c.c_int, c.c_int, c.c_int,
                                            c.c_int, vp]
        L.ko_num_threads.restype = c.c_int
        L.ko_num_threads.argtypes = []
        _lib = L
    return _lib


def _p(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


# --------------------------------------------------------------------------
# C oracle wrappers
# --------------------------------------------------------------------------

def c_lcg_fill(count: int, seed: int, mul: float) -> np.ndarray:
    out = np.empty(count, dtype=np.float32)
    lib().ko_lcg_fill(_p(out), count, ctypes.c_uint64(seed & 0xFFFFFFFFFFFFFFFF), mul)
    return out


def c_quantize(w: np.ndarray, groupsize: int):
    """-> (codes int32 [k,n], scales f16-bits uint16 [k/g,n], dequant f32 [k,n])"""
    w = _c(w, np.float32)
    k, n = w.shape
    g = k if groupsize == -1 else groupsize
    codes = np.empty((k, n), dtype=np.int32)
    scales = np.empty((k // g, n), dtype=np.uint16)
    deq = np.empty((k, n), dtype=np.float32)
    lib().ko_quantize(_p(w), k, n, groupsize, _p(codes), _p(scales), _p(deq))
    return codes, scales, deq


def c_pack_gptq(codes: np.ndarray) -> np.ndarray:
    codes = _c(codes, np.int32)
    k, n = codes.shape
    q = np.empty((k // 8, n), dtype=np.uint32)
    lib().ko_pack_gptq(_p(codes), k, n, _p(q))
    return q


def c_gptq_dequant_bf16(qweight, scales_f16, qzeros, groupsize) -> np.ndarray:
    qweight = _c(qweight, np.uint32)
    k8, n = qweight.shape
    k = k8 * 8
    scales_f16 = _c(scales_f16, np.uint16)
    qz = None if qzeros is None else _c(qzeros, np.uint32)
    out = np.empty((n, k), dtype=np.uint16)
    lib().ko_gptq_dequant_bf16(_p(qweight), _p(scales_f16), _p(qz), k, n, groupsize, _p(out))
    return out


def c_dequant_f32(qweight, scales_f16, groupsize) -> np.ndarray:
    qweight = _c(qweight, np.uint32)
    k8, n = qweight.shape
    k = k8 * 8
    scales_f16 = _c(scales_f16, np.uint16)
    out = np.empty((k, n), dtype=np.float32)
    lib().ko_dequant_f32(_p(qweight), _p(scales_f16), k, n, groupsize, _p(out))
    return out


def c_gemm_f32(x_bf16: np.ndarray, w: np.ndarray) -> np.ndarray:
    x_bf16 = _c(x_bf16, np.uint16)
    w = _c(w, np.float32)
    m, k = x_bf16.shape
    n = w.shape[1]
    y = np.empty((m, n), dtype=np.float32)
    lib().ko_gemm_f32(_p(x_bf16), _p(w), m, k, n, _p(y))
    return y


def c_gemm_f64(x_bf16: np.ndarray, w: np.ndarray) -> np.ndarray:
    x_bf16 = _c(x_bf16, np.uint16)
    w = _c(w, np.float32)
    m, k = x_bf16.shape
    n = w.shape[1]
    y = np.empty((m, n), dtype=np.float64)
    lib().ko_gemm_f64(_p(x_bf16), _p(w), m, k, n, _p(y))
    return y


def c_swiglu_f32(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """hidden = silu(gate) * up (forward.rs:110-114, :2789-2819), f64 inside, f32 out."""
    gate = _c(gate, np.float32)
    up = _c(up, np.float32)
    assert gate.shape == up.shape
    out = np.empty_like(gate)
    lib().ko_swiglu_f32(_p(gate), _p(up), gate.size, _p(out))
    return out


def c_w4a16_cpu_path(x_bf16, qweight, scales_f16, groupsize, scratch=None) -> np.ndarray:
    """The reference CPU path: unpack + dequantise to f32, then f32 matmul."""
    x_bf16 = _c(x_bf16, np.uint16)
    qweight = _c(qweight, np.uint32)
    scales_f16 = _c(scales_f16, np.uint16)
    m, k = x_bf16.shape
    n = qweight.shape[1]
    if scratch is None:
        scratch = np.empty((k, n), dtype=np.float32)
    y = np.empty((m, n), dtype=np.float32)
    lib().ko_w4a16_cpu_path(_p(x_bf16), _p(qweight), _p(scales_f16), m, k, n, groupsize,
                            _p(scratch), _p(y))
    return y


def c_lora_delta_add(y: np.ndarray, x_bf16, a_bf16, b_bf16, scale: float) -> np.ndarray:
    """y += ((x A^T) B^T) * scale, in place on a float32 [m, n] array."""
    assert y.dtype == np.float32 and y.flags.c_contiguous
    x_bf16 = _c(x_bf16, np.uint16)
    a_bf16 = _c(a_bf16, np.uint16)
    b_bf16 = _c(b_bf16, np.uint16)
    m, k = x_bf16.shape
    r = a_bf16.shape[0]
    n = b_bf16.shape[0]
    lib().ko_lora_delta_add_f32(_p(x_bf16), _p(a_bf16), _p(b_bf16), scale, m, k, n, r, _p(y))
    return y


def num_threads() -> int:
    return int(lib().ko_num_threads())


# --------------------------------------------------------------------------
# numpy twin: conversions
# --------------------------------------------------------------------------

def np_f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """quantized.rs:260-265 -- round to nearest even by integer add."""
    bits = _c(x, np.float32).view(np.uint32)
    rnd = bits + (np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1)))
    return (rnd >> np.uint32(16)).astype(np.uint16)


def np_bf16_to_f32(b: np.ndarray) -> np.ndarray:
    """quantized.rs:254-257"""
    return (_c(b, np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def np_f16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return _c(b, np.uint16).view(np.float16).astype(np.float32)


def np_f32_to_f16_bits(x: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        return _c(x, np.float32).astype(np.float16).view(np.uint16)


# --------------------------------------------------------------------------
# numpy twin: LCG (parity.rs:22-31), vectorised by jump-ahead
# --------------------------------------------------------------------------

_LCG_A = np.uint64(6364136223846793005)
_LCG_C = np.uint64(1442695040888963407)


def np_lcg_fill(count: int, seed: int, mul: float) -> np.ndarray:
    """state_i = A^i * seed + C * (A^(i-1) + ... + 1) mod 2^64, i = 1..count."""
    with np.errstate(over="ignore"):
        a_pow = np.empty(count + 1, dtype=np.uint64)
        a_pow[0] = 1
        a_pow[1:] = _LCG_A
        a_pow = np.multiply.accumulate(a_pow)            # A^0 .. A^count, wraps mod 2^64
        geo = np.add.accumulate(a_pow[:-1])              # sum_{j<i} A^j for i = 1..count
        state = a_pow[1:] * np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + _LCG_C * geo
    bits = ((state >> np.uint64(33)) & np.uint64(0x7FFFFFFF)).astype(np.uint32)
    v = bits.astype(np.float32) / np.float32(2147483647) - np.float32(0.5)
    return (v * np.float32(mul)).astype(np.float32)


# --------------------------------------------------------------------------
# numpy twin: quantiser (lib.rs:393-427)
# --------------------------------------------------------------------------

def np_round_half_away(x: np.ndarray) -> np.ndarray:
    """Rust ``f32::round``: ties go away from zero (numpy's rint is half-even)."""
    t = np.trunc(x)
    frac = x - t                                       # exact
    return np.where(np.abs(frac) >= 0.5, t + np.sign(x), t).astype(x.dtype)


def np_quantize(w: np.ndarray, groupsize: int):
    w = _c(w, np.float32)
    k, n = w.shape
    g = k if groupsize == -1 else groupsize
    ng = k // g
    max_abs = np.abs(w.reshape(ng, g, n)).max(axis=1)
    max_abs = np.where(max_abs == 0.0, np.float32(1.0), max_abs).astype(np.float32)
    s_f32 = (np.float32(2.0) * max_abs) / np.float32(15.0)
    s_bits = np_f32_to_f16_bits(s_f32)
    s = np_f16_bits_to_f32(s_bits)
    s_full = np.repeat(s, g, axis=0)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np_round_half_away((w / s_full).astype(np.float32))
    # `as i32` saturates, NaN -> 0; the i32 sum `raw + Q_OFFSET` (lib.rs:423) wraps in a release build
    # where raw saturated at i32::MAX (w / s = +inf), and the clamp then gives code 0
    raw = np.clip(np.nan_to_num(q.astype(np.float64), nan=0.0, posinf=2147483647.0, neginf=-2147483648.0),
                  -2147483648.0, 2147483647.0).astype(np.int64)
    shifted = raw + 8
    shifted = np.where(shifted > 2147483647, shifted - 4294967296, shifted)
    codes = np.clip(shifted, 0, 15).astype(np.int32)
    deq = ((codes - 8).astype(np.float32) * s_full).astype(np.float32)
    return codes, s_bits, deq


# --------------------------------------------------------------------------
# numpy twin: GPTQ-canonical layout (quantized.rs:127-152)
# --------------------------------------------------------------------------

def np_pack_gptq(codes: np.ndarray) -> np.ndarray:
    """codes [k, n] in 0..15 -> qweight [k/8, n] uint32; row 8i+j sits in bits 4j.."""
    codes = _c(codes, np.int64)
    k, n = codes.shape
    c = codes.reshape(k // 8, 8, n).astype(np.uint32)
    out = np.zeros((k // 8, n), dtype=np.uint32)
    for j in range(8):
        out |= (c[:, j, :] & np.uint32(0xF)) << np.uint32(4 * j)
    return out


def np_unpack_gptq(qweight: np.ndarray) -> np.ndarray:
    qweight = _c(qweight, np.uint32)
    k8, n = qweight.shape
    out = np.empty((k8, 8, n), dtype=np.int32)
    for j in range(8):
        out[:, j, :] = ((qweight >> np.uint32(4 * j)) & np.uint32(0xF)).astype(np.int32)
    return out.reshape(k8 * 8, n)


def np_pack_qzeros(zeros: np.ndarray) -> np.ndarray:
    """zeros [groups, n] in 0..15 -> qzeros [groups, n/8]; column 8i+j in bits 4j.."""
    zeros = _c(zeros, np.int64)
    gr, n = zeros.shape
    z = zeros.reshape(gr, n // 8, 8).astype(np.uint32)
    out = np.zeros((gr, n // 8), dtype=np.uint32)
    for j in range(8):
        out |= (z[:, :, j] & np.uint32(0xF)) << np.uint32(4 * j)
    return out


def np_dequant_f32(qweight, scales_f16, groupsize) -> np.ndarray:
    """(code - 8) * f32(scale), [k, n] f32 (lib.rs:425)."""
    codes = np_unpack_gptq(qweight)
    k, n = codes.shape
    g = k if groupsize == -1 else groupsize
    s = np.repeat(np_f16_bits_to_f32(scales_f16), g, axis=0)
    return ((codes - 8).astype(np.float32) * s).astype(np.float32)


def np_gptq_dequant_bf16(qweight, scales_f16, qzeros, groupsize) -> np.ndarray:
    """(code - zero) * scale -> bf16 bits, [n, k] (quantized.rs:127-152)."""
    codes = np_unpack_gptq(qweight)
    k, n = codes.shape
    g = k if groupsize == -1 else groupsize
    if qzeros is None:
        zeros = np.full((k // g, n), 8, dtype=np.int32)
    else:
        qz = _c(qzeros, np.uint32)
        zeros = np.empty((k // g, n // 8, 8), dtype=np.int32)
        for j in range(8):
            zeros[:, :, j] = ((qz >> np.uint32(4 * j)) & np.uint32(0xF)).astype(np.int32)
        zeros = zeros.reshape(k // g, n)
    s = np.repeat(np_f16_bits_to_f32(scales_f16), g, axis=0)
    z = np.repeat(zeros, g, axis=0)
    deq = ((codes - z).astype(np.float32) * s).astype(np.float32)
    return np_f32_to_bf16(deq).reshape(k, n).T.copy()


# --------------------------------------------------------------------------
# numpy twin: the reference's Marlin (NVIDIA fragment) layout, lib.rs:296-357
# and :429-528.  Kept only so old Marlin-format blobs can be cross-checked;
# the MI355X kernels use their own layout.
# --------------------------------------------------------------------------

def marlin_weight_perm() -> np.ndarray:
    perm = []
    for i in range(32):
        perm1 = []
        col = i // 4
        for block in (0, 1):
            for row in (2 * (i % 4), 2 * (i % 4) + 1, 2 * (i % 4 + 4), 2 * (i % 4 + 4) + 1):
                perm1.append(16 * row + col + 8 * block)
        for j in range(4):
            perm.extend(p + 256 * j for p in perm1)
    perm = np.array(perm, dtype=np.int64).reshape(-1, 8)[:, [0, 2, 4, 6, 1, 3, 5, 7]]
    return perm.reshape(-1)


def marlin_scale_perm() -> np.ndarray:
    return np.array([i + 8 * j for i in range(8) for j in range(8)], dtype=np.int64)


def marlin_scale_perm_single() -> np.ndarray:
    return np.array([2 * i + j for i in range(4) for j in (0, 1, 8, 9, 16, 17, 24, 25)],
                    dtype=np.int64)


def marlin_pack(codes: np.ndarray, scales_f16: np.ndarray, groupsize: int):
    """codes [k,n], scales [k/g,n] -> (packed int32 [k/16, 2n], permuted scales)."""
    codes = _c(codes, np.int64)
    k, n = codes.shape
    tiled = codes.reshape(k // 16, 16, n // 16, 16).transpose(0, 2, 1, 3).reshape(k // 16, n * 16)
    perm = marlin_weight_perm()
    res = tiled.reshape(-1, perm.size)[:, perm].reshape(k // 16, n * 16)
    r = res.reshape(k // 16, n * 2, 8).astype(np.uint32)
    packed = np.zeros((k // 16, n * 2), dtype=np.uint32)
    for i in range(8):
        packed |= (r[:, :, i] & np.uint32(0xF)) << np.uint32(4 * i)
    s = _c(scales_f16, np.uint16)
    sp = marlin_scale_perm_single() if groupsize == -1 else marlin_scale_perm()
    s_perm = s.reshape(-1, sp.size)[:, sp].reshape(s.shape)
    return packed.view(np.int32), s_perm


# --------------------------------------------------------------------------
# seeded synthetic inputs for the benchmark configurations
# --------------------------------------------------------------------------

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def _splitmix64(idx: np.ndarray, stream: int) -> np.ndarray:
    """Counter-based splitmix64: element i of stream s is mix(s*2^40 + i)."""
    with np.errstate(over="ignore"):
        z = (idx.astype(np.uint64) + np.uint64((stream & 0xFFFFFF) << 40) + np.uint64(1)) * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def _uniform01(count: int, stream: int) -> np.ndarray:
    u = _splitmix64(np.arange(count, dtype=np.uint64), stream)
    return ((u >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)


def gen_codes(k: int, n: int, seed: int) -> np.ndarray:
    """int4 codes uniform in [0, 15], [k, n] int32."""
    u = _splitmix64(np.arange(k * n, dtype=np.uint64), 3 * seed + 0)
    return (u >> np.uint64(60)).astype(np.int32).reshape(k, n)


def gen_scales_f16(k: int, n: int, groupsize: int, seed: int, lo=0.002, hi=0.02) -> np.ndarray:
    """fp16 scales uniform in [lo, hi], [k/g, n] raw bits."""
    g = k if groupsize == -1 else groupsize
    u = _uniform01((k // g) * n, 3 * seed + 1)
    return np_f32_to_f16_bits((lo + (hi - lo) * u).astype(np.float32)).reshape(k // g, n)


def gen_normal_bf16(rows: int, cols: int, sigma: float, seed: int, stream: int = 2) -> np.ndarray:
    """bf16 bits of N(0, sigma^2) by Box-Muller, [rows, cols]."""
    count = rows * cols
    half = (count + 1) // 2
    u1 = _uniform01(half, 3 * seed + stream)
    u2 = _uniform01(half, 3 * seed + stream + 1000003)
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.concatenate([r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)])[:count]
    return np_f32_to_bf16((sigma * z).astype(np.float32)).reshape(rows, cols)


def gen_problem(m: int, k: int, n: int, groupsize: int = 128, seed: int = 0, sigma: float = 1.0):
    """One benchmark-style problem: (x bf16 bits [m,k], qweight u32 [k/8,n], scales f16 bits)."""
    codes = gen_codes(k, n, seed)
    return (gen_normal_bf16(m, k, sigma, seed), np_pack_gptq(codes),
            gen_scales_f16(k, n, groupsize, seed))
