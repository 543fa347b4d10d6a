"""The matrix-core kernel's row sums (the operand of its offset removal) formed by a few blocks of the
product's own launch instead of by a launch in front: taken where the launch is one round of blocks
with block slots to spare.  The sums are added in the same order on both routes, so the results must
agree in every bit; parity with the oracle is checked on top."""
import ctypes

import numpy as np
import pytest
import torch

from kiln_amd import _lib
from kiln_amd.marlin_gemm import pack
from tests.gpu_util import bf16_bits, bf16_tensor, row_errors, upload_packed

pytestmark = pytest.mark.gpu

# (rows, k, n, expected: producers inside the launch)
CASES = [
    (2048, 9216, 2560, True),    # cfg 2's down projection: 480 blocks of 128 rows on 512 slots
    (777, 2560, 8192, True),     # ragged rows
    (1536, 9216, 2560, True),
    (600, 2560, 12288, True),    # 128-row blocks below 768 rows
    (2500, 4096, 2560, True),    # the most producers a launch takes
    (2048, 2560, 18432, False),  # several rounds of blocks: the launch in front stays
    (400, 4096, 2560, False),    # the blocks sum their rows themselves
]
IN_FRONT, OWN_ROWS, OTHER_KERNEL = 0, -2, -3


def _cus():
    return torch.cuda.get_device_properties(0).multi_processor_count


def test_the_plan_query_says_where_the_row_sums_come_from():
    L = _lib.load_tuning()
    for m, k, n, inside in CASES:
        p = L.kiln_w4a16_debug_prefill_rowsum_producers(m, n, k, _cus())
        assert (p > 0) == inside, (m, k, n, p)
        if inside:
            assert p % 8 == 0 and 8 <= p <= 128 and p >= (m + 63) // 64
    assert L.kiln_w4a16_debug_prefill_rowsum_producers(2048, 18432, 2560, _cus()) == IN_FRONT
    assert L.kiln_w4a16_debug_prefill_rowsum_producers(400, 2560, 4096, _cus()) == OWN_ROWS
    assert L.kiln_w4a16_debug_prefill_rowsum_producers(16, 2560, 2560, _cus()) == OTHER_KERNEL
    try:
        L.kiln_w4a16_debug_rowsum_fold(0)
        assert L.kiln_w4a16_debug_prefill_rowsum_producers(2048, 2560, 9216, _cus()) == IN_FRONT
    finally:
        L.kiln_w4a16_debug_rowsum_fold(-1)
    assert L.kiln_w4a16_debug_prefill_rowsum_producers(0, 2560, 9216, _cus()) == -1


@pytest.mark.parametrize("m,k,n,inside", CASES)
def test_row_sums_inside_the_launch_equal_the_launch_in_front(oracle, m, k, n, inside):
    L = _lib.load_tuning()
    g = 128
    x, q, s_bits = oracle.gen_problem(m, k, n, g, seed=m + n)
    # activations with a mean: the offset term 136 * sum(a) is then far larger than the result
    xs = [bf16_tensor(x), bf16_tensor(oracle.np_f32_to_bf16(np.abs(oracle.np_bf16_to_f32(x))))]
    b, s = pack.repack_gptq(q, s_bits, None, g)
    bt, st = upload_packed(b, s)
    z = L.kiln_w4a16_workspace_zeroed_bytes()
    ws = torch.empty(L.kiln_w4a16_workspace_bytes(m, n, k), dtype=torch.uint8, device="cuda")
    ws[z:].fill_(0xA5)
    ws[:z].zero_()
    stream = torch.cuda.current_stream().cuda_stream

    def call(xt):
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = L.kiln_marlin_w4a16_gemm(xt.data_ptr(), bt.data_ptr(), out.data_ptr(), st.data_ptr(), m, n, k, ws.data_ptr(), g,
                                      torch.cuda.current_device(), stream, -1, -1, -1, 16)
        assert rc == _lib.OK, _lib.status_string(rc)
        torch.cuda.synchronize()
        assert int(ws[:z].count_nonzero()) == 0, "the call left words in the zeroed prefix"
        return out

    try:
        L.kiln_w4a16_debug_rowsum_fold(0)
        in_front = [call(xt) for xt in xs]
        L.kiln_w4a16_debug_rowsum_fold(-1)
        # alternating activations: every launch must see its own sums, not the previous launch's
        for i in range(12):
            assert torch.equal(call(xs[i % 2]).view(torch.int16), in_front[i % 2].view(torch.int16)), i
    finally:
        L.kiln_w4a16_debug_rowsum_fold(-1)
    word = ctypes.c_uint32(0xFFFFFFFF)
    assert L.kiln_w4a16_workspace_check(ws.data_ptr(), ctypes.byref(word), stream) == _lib.OK
    torch.cuda.synchronize()
    assert word.value == 0
    want = oracle.c_w4a16_cpu_path(x, q, s_bits, g)
    err, _, _ = row_errors(bf16_bits(in_front[0]), want, oracle)
    assert err.max() <= 1e-2, err.max()


def test_replays_of_a_captured_launch_with_the_row_sums_inside(oracle):
    """The words are raised and zeroed again inside every launch: replays of one captured launch, with
    new activations in the same buffer between them, each equal the eager result."""
    L = _lib.load()
    m, k, n, g = 2048, 9216, 2560, 128
    assert _lib.load_tuning().kiln_w4a16_debug_prefill_rowsum_producers(m, n, k, _cus()) > 0
    x, q, s_bits = oracle.gen_problem(m, k, n, g, seed=5)
    b, s = pack.repack_gptq(q, s_bits, None, g)
    bt, st = upload_packed(b, s)
    gen = torch.Generator(device="cuda").manual_seed(11)
    xs = [bf16_tensor(x)] + [(torch.randn(m, k, device="cuda", generator=gen) + 0.25 * i).to(torch.bfloat16) for i in range(1, 4)]
    ws = torch.zeros(L.kiln_w4a16_workspace_bytes(m, n, k), dtype=torch.uint8, device="cuda")
    xin = torch.empty(m, k, dtype=torch.bfloat16, device="cuda")
    out = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")

    def launch():
        rc = L.kiln_marlin_w4a16_gemm(xin.data_ptr(), bt.data_ptr(), out.data_ptr(), st.data_ptr(), m, n, k, ws.data_ptr(), g,
                                      torch.cuda.current_device(), torch.cuda.current_stream().cuda_stream, -1, -1, -1, 16)
        assert rc == _lib.OK, _lib.status_string(rc)

    eager = []
    for xt in xs:
        xin.copy_(xt)
        launch()
        torch.cuda.synchronize()
        eager.append(out.clone())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch()
    for rep in range(3):
        for xt, want in zip(xs, eager):
            xin.copy_(xt)
            out.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.int16), want.view(torch.int16)), rep


def test_fused_swiglu_launch_with_the_row_sums_inside(oracle):
    """The fused gate+up SwiGLU instance of the kernel takes the same route on a launch of one round
    (2048 rows, 9216 -> 2 x 1280): equal to the launch in front in every bit, and within the bound of
    silu(gate) * up formed from the oracle's two f32 GEMMs."""
    from kiln_amd import marlin_gemm
    L = _lib.load_tuning()
    m, k, n_out, g = 2048, 9216, 1280, 128
    assert L.kiln_w4a16_debug_prefill_rowsum_producers(m, 2 * n_out, k, _cus()) > 0
    x = oracle.gen_normal_bf16(m, k, 0.5, 77)
    sides = []
    for seed in (78, 79):
        q, s_bits = oracle.np_pack_gptq(oracle.gen_codes(k, n_out, seed)), oracle.gen_scales_f16(k, n_out, g, seed)
        sides.append((q, s_bits) + tuple(pack.repack_gptq(q, s_bits, None, g)))
    b_gu, s_gu = pack.interleave_gate_up(sides[0][2], sides[0][3], sides[1][2], sides[1][3], g)
    bt, st = upload_packed(b_gu, np.asarray(s_gu).view(np.uint16))
    xt = bf16_tensor(x)
    try:
        L.kiln_w4a16_debug_rowsum_fold(0)
        in_front = marlin_gemm.marlin_w4a16_gemm_swiglu(xt, bt, st, g).clone()
        L.kiln_w4a16_debug_rowsum_fold(-1)
        for _ in range(4):
            assert torch.equal(marlin_gemm.marlin_w4a16_gemm_swiglu(xt, bt, st, g).view(torch.int16), in_front.view(torch.int16))
    finally:
        L.kiln_w4a16_debug_rowsum_fold(-1)
    assert marlin_gemm.workspace_wait_status() == 0
    gate = oracle.c_w4a16_cpu_path(x, sides[0][0], sides[0][1], g)
    up = oracle.c_w4a16_cpu_path(x, sides[1][0], sides[1][1], g)
    err, hv, _ = row_errors(bf16_bits(in_front), oracle.c_swiglu_f32(gate, up), oracle)
    assert np.all(np.isfinite(hv)) and err.max() <= 1e-2, err.max()
