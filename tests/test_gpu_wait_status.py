"""The workspace's sticky word: a wavefront whose bounded wait runs out ORs a bit into it, the host
reads it with kiln_w4a16_workspace_check and clears the whole prefix with kiln_w4a16_workspace_reset.
No test here makes a wait run out on the GPU: the word is written from the host side, as a kernel
would have left it, and every launch of the suite is expected to leave it zero."""
import ctypes

import numpy as np
import pytest
import torch

from kiln_amd import _lib, marlin_gemm


def test_error_word_sits_inside_the_zeroed_prefix_and_outside_every_counter():
    """CPU: where the word is, against what the plans of the model's shapes use of the counter region."""
    L = _lib.load()
    off, zeroed = L.kiln_w4a16_workspace_error_offset(), L.kiln_w4a16_workspace_zeroed_bytes()
    assert off % 4 == 0 and off + 4 <= 64 * 1024 <= zeroed
    # the small-M kernels keep one arrival counter per column tile and run: the widest projection at four
    # runs per launch uses 4 * 18432 / 16 counters, far below the word
    assert 4 * (18432 // 16) * 4 <= off
    word = ctypes.c_uint32(0)
    assert L.kiln_w4a16_workspace_check(ctypes.c_void_p(4096), None, None) == _lib.ERR_ARGUMENT


@pytest.mark.gpu
def test_check_reads_the_word_and_reset_clears_the_prefix(oracle):
    L = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    zeroed, off = L.kiln_w4a16_workspace_zeroed_bytes(), L.kiln_w4a16_workspace_error_offset()
    ws = torch.zeros(zeroed + 1024, dtype=torch.uint8, device="cuda")
    word = ctypes.c_uint32(0xFFFFFFFF)
    assert L.kiln_w4a16_workspace_check(ws.data_ptr(), ctypes.byref(word), stream) == _lib.OK
    torch.cuda.synchronize()
    assert word.value == 0
    # as a launch that gave up would leave it: the bit set, and a late part somewhere in the exchange region
    ws[off:off + 4] = torch.tensor([_lib.WAIT_DECODE_EXCHANGE | _lib.WAIT_MID_FOLD, 0, 0, 0], dtype=torch.uint8, device="cuda")
    ws[64 * 1024 + 4096] = 7
    ws[zeroed:] = 0x5A
    assert L.kiln_w4a16_workspace_check(ws.data_ptr(), ctypes.byref(word), stream) == _lib.OK
    torch.cuda.synchronize()
    assert word.value == (_lib.WAIT_DECODE_EXCHANGE | _lib.WAIT_MID_FOLD)
    assert L.kiln_w4a16_workspace_reset(ws.data_ptr(), stream) == _lib.OK
    torch.cuda.synchronize()
    assert int(ws[:zeroed].max()) == 0 and int(ws[zeroed:].min()) == 0x5A     # the prefix, and nothing behind it
    assert L.kiln_w4a16_workspace_check(ws.data_ptr(), ctypes.byref(word), stream) == _lib.OK
    torch.cuda.synchronize()
    assert word.value == 0
    # a GEMM on the reset workspace works (K-sliced exchange through the zeroed region)
    from kiln_amd.marlin_gemm import pack
    from tests.gpu_util import bf16_bits, bf16_tensor, row_errors, upload_packed
    m, k, n, g = 16, 9216, 2560, 128
    x, q, s_bits = oracle.gen_problem(m, k, n, g, seed=3)
    b, s = pack.repack_gptq(q, s_bits, None, g)
    bt, st = upload_packed(b, s)
    big = torch.empty(L.kiln_w4a16_workspace_bytes(m, n, k), dtype=torch.uint8, device="cuda")
    big[:zeroed].fill_(0xFF)                                                 # a prefix somebody scribbled on
    assert L.kiln_w4a16_workspace_reset(big.data_ptr(), stream) == _lib.OK
    y = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    xt = bf16_tensor(x)
    assert L.kiln_marlin_w4a16_gemm(xt.data_ptr(), bt.data_ptr(), y.data_ptr(), st.data_ptr(), m, n, k, big.data_ptr(),
                                    g, 0, stream, -1, -1, -1, 16) == _lib.OK
    torch.cuda.synchronize()
    err, _, _ = row_errors(bf16_bits(y), oracle.c_w4a16_cpu_path(x, q, s_bits, g), oracle)
    assert err.max() <= 1e-2
    assert L.kiln_w4a16_workspace_check(big.data_ptr(), ctypes.byref(word), stream) == _lib.OK
    torch.cuda.synchronize()
    assert word.value == 0


@pytest.mark.gpu
def test_module_level_health_check_reads_zero_after_ordinary_calls():
    k, n, g = 4096, 2560, 128
    gen = torch.Generator(device="cuda").manual_seed(5)
    b = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 16, 2 * n), dtype=torch.int32, device="cuda", generator=gen)
    s = (torch.rand(k // g, n, device="cuda", generator=gen) * 0.018 + 0.002).to(torch.float16)
    for m in (1, 16, 64, 300):
        marlin_gemm.marlin_w4a16_gemm((torch.randn(m, k, device="cuda") * 0.5).to(torch.bfloat16), b, s, g)
    assert marlin_gemm.workspace_wait_status() == 0
    marlin_gemm.workspace_reset()
    y = marlin_gemm.marlin_w4a16_gemm((torch.randn(16, k, device="cuda") * 0.5).to(torch.bfloat16), b, s, g)
    assert torch.isfinite(y.float()).all() and marlin_gemm.workspace_wait_status() == 0
