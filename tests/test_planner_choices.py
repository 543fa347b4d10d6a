"""What the planners pick, pinned on the CPU (the plan queries are pure host functions): the model's
shapes and shapes of other models on which every forced plan was timed on an MI355X.  The pins are
the picks those timings justify -- a change of a cost model that moves one of them should come with
a new sweep."""
import ctypes

import pytest

from kiln_amd import _lib

CUS = 256


def _decode_plan(m, k, n):
    out = (ctypes.c_int * 8)()
    assert _lib.load().kiln_w4a16_debug_decode_plan(m, n, k, CUS, out) == 0
    ks, gs, u, bps, waves, direct, regs, gm = list(out)
    assert gm < 0, "up to 16 rows take the private-staging kernel"
    return -gm, waves, ks, bps * ks                       # tiles per block, wavefronts, K slices, blocks


def _route(m, k, n):
    out = (ctypes.c_int * 8)()
    assert _lib.load().kiln_w4a16_debug_gemm_plan(m, n, k, CUS, out) == 0
    if out[6]:
        return ("mid", out[7] // 16, out[7] % 16)          # tile pairs per block, K slices
    if out[0]:
        return ("matrix-core", out[2], out[3])             # block rows, block columns
    return ("small", out[1])                               # launches


@pytest.mark.parametrize("m,k,n,want", [
    # the model's shapes
    (16, 2560, 18432, (5, 8, 1)), (8, 2560, 18432, (5, 8, 1)), (1, 2560, 18432, (5, 12, 1)),
    (16, 9216, 2560, (2, 12, 3)), (1, 9216, 2560, (1, 12, 1)),
    (16, 2560, 8192, (2, 12, 1)), (16, 4096, 2560, (1, 16, 1)),
    # projections of one input side by side
    (16, 2560, 10240, (3, 8, 1)), (1, 2560, 12288, (3, 8, 1)),
    # other models' shapes: one round of blocks where one can be formed
    (16, 5120, 13824, (4, 16, 1)), (1, 5120, 13824, (4, 16, 1)), (1, 4096, 14336, (4, 12, 1)),
    (16, 18944, 3584, (4, 16, 4)), (1, 18944, 3584, (2, 16, 2)),
])
def test_small_m_plans(m, k, n, want):
    tiles, waves, ks, blocks = _decode_plan(m, k, n)
    assert (tiles, waves, ks) == want
    assert blocks <= CUS, "a plan of one round exists for every shape listed here"


def test_sixteen_wavefronts_only_where_twelve_cannot_form_the_plan():
    for m in (1, 4, 8, 16):
        for k, n in ((4096, 11008), (4096, 14336), (8192, 8192), (14336, 4096), (2560, 8192), (2560, 18432)):
            tiles, waves, ks, _ = _decode_plan(m, k, n)
            gs = k // 128 // ks
            if waves == 16:
                assert (tiles == 1 and gs % 16 == 0) or tiles * -(-gs // 12) > 16, (m, k, n, tiles, ks)


@pytest.mark.parametrize("m,k,n,want", [
    # from: 17 rows; wide outputs of a short K stay with the two-slab small-M instance up to 20 rows
    (16, 9216, 2560, "small"), (17, 9216, 2560, "mid"), (17, 4096, 2560, "mid"), (17, 2560, 8192, "mid"),
    (17, 2560, 1024, "mid"), (24, 4096, 4096, "mid"), (32, 8192, 8192, "mid"), (32, 5120, 13824, "mid"),
    (17, 2560, 18432, "small"), (20, 2560, 18432, "small"), (21, 2560, 18432, "mid"), (17, 3584, 18944, "mid"),
    (20, 2560, 10240, "small"), (21, 2560, 10240, "mid"), (32, 2560, 12288, "mid"), (24, 2048, 11008, "mid"),
    # to: 128 rows; 192 / 256 / 320 on small weights
    (128, 2560, 18432, "mid"), (129, 2560, 18432, "matrix-core"), (160, 14336, 4096, "matrix-core"),
    (64, 18944, 3584, "mid"), (65, 18944, 3584, "matrix-core"), (128, 18944, 3584, "matrix-core"),
    # the largest weights with a long K: one run of rows; as large but of a short K: two
    (64, 8192, 8192, "mid"), (65, 8192, 8192, "matrix-core"), (128, 5120, 13824, "matrix-core"), (128, 3584, 18944, "mid"),
    (128, 14336, 4096, "mid"), (128, 11008, 4096, "mid"),
    (160, 8192, 8192, "matrix-core"),
    (192, 9216, 2560, "mid"), (193, 9216, 2560, "matrix-core"),
    (256, 2560, 8192, "mid"), (257, 2560, 8192, "matrix-core"), (256, 2560, 12288, "mid"),
    (320, 4096, 2560, "mid"), (321, 4096, 2560, "matrix-core"), (320, 2560, 1024, "mid"),
    (1024, 2560, 1024, "mid"), (1025, 2560, 1024, "matrix-core"), (512, 3072, 3072, "mid"), (448, 2048, 2048, "mid"),
    (513, 2048, 2048, "matrix-core"), (1024, 1536, 1536, "mid"),
    # wide outputs of a short K: by output size
    (192, 896, 9728, "mid"), (193, 896, 9728, "matrix-core"), (384, 896, 4864, "mid"), (448, 896, 4864, "matrix-core"),
    (128, 1536, 17920, "mid"), (129, 1536, 17920, "matrix-core"), (64, 3584, 37888, "mid"), (65, 3584, 37888, "matrix-core"),
    (256, 2048, 11264, "mid"), (256, 1024, 8192, "mid"), (257, 1024, 8192, "matrix-core"),
    (64, 4096, 28672, "mid"), (65, 4096, 28672, "matrix-core"), (128, 4096, 22016, "mid"),
])
def test_which_kernel_takes_a_row_count(m, k, n, want):
    assert _route(m, k, n)[0] == want


@pytest.mark.parametrize("m,k,n,want", [
    (64, 2560, 8192, (1, 1)), (64, 4096, 2560, (1, 2)), (64, 2560, 18432, (3, 1)), (64, 9216, 2560, (1, 3)),
    # rounds after the first cost their start: no pile of short slices
    (64, 5120, 13824, (2, 2)), (96, 3584, 18944, (2, 1)), (128, 3584, 18944, (2, 1)),
    # ten wavefronts beyond 32 rows only where eight cannot form a plan (148 groups = 4 x 37), and in one run of rows
    (64, 13824, 5120, (2, 6)), (64, 5120, 5120, (2, 2)),
    # a shorter last slice where K in groups has no even slicing that fits: 86 = 29 + 29 + 28, 148 = 6 x 22 + 16
    (64, 11008, 4096, (2, 4)), (32, 11008, 4096, (2, 3)), (64, 18944, 3584, (2, 7)), (64, 8960, 1536, (1, 3)),
    # one round either way: four short slices through the counter-free exchange lead two long ones
    (64, 4096, 1024, (1, 4)), (17, 4096, 1024, (1, 4)), (128, 4096, 1024, (1, 4)),
])
def test_mid_m_plans(m, k, n, want):
    assert _route(m, k, n) == ("mid",) + want


@pytest.mark.parametrize("m,k,n,rows", [
    (2048, 2560, 18432, 128), (2048, 9216, 2560, 128), (4096, 2560, 18432, 128), (1024, 2560, 18432, 128),
    (384, 9216, 2560, 64), (192, 2560, 18432, 64),
    (321, 18944, 3584, 128), (256, 28672, 8192, 128), (321, 6144, 6144, 128),  # 128 x 256 in K slices from 129 rows where they lead
    (192, 4096, 12288, 64), (192, 11008, 4096, 64),
    (448, 3584, 4608, 128),                                                # (was 64 x 128, one block of two wavefronts a unit: 65 us)
    (1025, 2560, 1024, 64), (2048, 2560, 1024, 64), (4096, 2560, 1024, 64),  # narrow outputs at any row count
    (1024, 2560, 2048, 64),
    (512, 13824, 5120, 128), (512, 8192, 8192, 128), (768, 2560, 18432, 128),  # large products from 385 rows on
    (512, 9216, 2560, 64), (512, 2560, 8192, 64),
])
def test_matrix_core_block_rows(m, k, n, rows):
    kind, bm, bn = _route(m, k, n)
    assert kind == "matrix-core" and bm == rows and bn in (128, 256)
