"""The entry point that allocates nothing (`kiln_marlin_w4a16_gemm_static_scratch`), called through
the C ABI: its output must equal, bit for bit, that of `kiln_marlin_w4a16_gemm` with a caller
workspace (same plan, same kernels; the workspace is a device array of the library instead), on
calls in a row that share the array -- the later ones with smaller inputs -- and a shape whose plan
needs more than the array holds must be refused before anything is launched."""
import ctypes

import numpy as np
import pytest
import torch

from kiln_amd import _lib
from kiln_amd.marlin_gemm import pack
from tests.gpu_util import bf16_bits, bf16_tensor, row_errors, upload_packed

pytestmark = pytest.mark.gpu


def _both_entry_points(L, xt, bt, st, m, k, n, g=128):
    dev = torch.cuda.current_device()
    stream = torch.cuda.current_stream().cuda_stream
    ws = torch.empty(L.kiln_w4a16_workspace_bytes(m, n, k), dtype=torch.uint8, device="cuda")
    ws[:L.kiln_w4a16_workspace_zeroed_bytes()].zero_()
    want = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    rc = L.kiln_marlin_w4a16_gemm(xt.data_ptr(), bt.data_ptr(), want.data_ptr(), st.data_ptr(), m, n, k,
                                  ws.data_ptr(), g, dev, stream, -1, -1, -1, 16)
    assert rc == _lib.OK
    rc = L.kiln_marlin_w4a16_gemm_static_scratch(xt.data_ptr(), bt.data_ptr(), got.data_ptr(), st.data_ptr(),
                                                 m, n, k, g, dev, stream)
    assert rc == _lib.OK, _lib.status_string(rc)
    torch.cuda.synchronize()
    return got, want


def test_static_scratch_entry_point_matches_the_workspace_one(oracle):
    L = _lib.load()
    k, n, g = 9216, 2560, 128                      # three K slices at m <= 16: partial tiles and counters in use
    x, q, s_bits = oracle.gen_problem(32, k, n, g, seed=11)
    b, s = pack.repack_gptq(q, s_bits, None, g)
    bt, st = upload_packed(b, s)
    y_ref = oracle.c_w4a16_cpu_path(x, q, s_bits, g)
    # calls in a row on one GPU share the array: 16 rows, then fewer, then more (two slabs), then one
    for m in (16, 5, 32, 1):
        xt = bf16_tensor(x[:m])
        got, want = _both_entry_points(L, xt, bt, st, m, k, n)
        assert torch.equal(got, want), f"m={m}"
        err, _, _ = row_errors(bf16_bits(got), y_ref[:m], oracle)
        assert err.max() <= 1e-2
    # a second, smaller projection right after (its counters sit in the same prefix)
    k2, n2 = 4096, 2560
    x2, q2, s2_bits = oracle.gen_problem(8, k2, n2, g, seed=12)
    b2, s2 = pack.repack_gptq(q2, s2_bits, None, g)
    bt2, st2 = upload_packed(b2, s2)
    got, want = _both_entry_points(L, bf16_tensor(x2), bt2, st2, 8, k2, n2)
    assert torch.equal(got, want)


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    L = _lib.load()
    p = ctypes.c_void_p(1 << 20)                   # never dereferenced: the call is refused before any launch
    stream = torch.cuda.current_stream().cuda_stream
    dev = torch.cuda.current_device()
    m, n, k = 2048, 2560, 9216                     # K-sliced prefill: tens of MB of partial tiles
    assert L.kiln_w4a16_workspace_bytes(m, n, k) > _lib.STATIC_SCRATCH_BYTES
    rc = L.kiln_marlin_w4a16_gemm_static_scratch(p, p, p, p, m, n, k, 128, dev, stream)
    assert rc == _lib.ERR_SCRATCH and "scratch" in _lib.status_string(rc)
    assert L.kiln_marlin_w4a16_gemm_static_scratch(p, p, p, p, 16, 2560, 9216, 128, dev + 1, stream) == _lib.ERR_ARGUMENT
    assert L.kiln_marlin_w4a16_gemm_static_scratch(p, p, p, p, 16, 200, 9216, 128, dev, stream) == _lib.ERR_PROB_SHAPE
    assert L.kiln_marlin_w4a16_gemm_static_scratch(p, p, p, p, 0, 2560, 9216, 128, dev, stream) == _lib.OK
    torch.cuda.synchronize()


def test_static_scratch_calls_allocate_nothing_and_replay_from_a_graph(oracle):
    """What the entry point is for: device memory in use is the same before and after a run of calls, and
    after one eager call per shape on the device (the library's one-time queries: the array's address,
    the kernels' LDS limits) the calls can be captured into a graph and replayed."""
    L = _lib.load()
    g = 128
    shapes = [(16, 9216, 2560), (4, 2560, 8192)]
    problems = []
    for m, k, n in shapes:
        x, q, s_bits = oracle.gen_problem(m, k, n, g, seed=m + n)
        b, s = pack.repack_gptq(q, s_bits, None, g)
        bt, st = upload_packed(b, s)
        problems.append((m, k, n, bf16_tensor(x), bt, st, torch.empty((m, n), dtype=torch.bfloat16, device="cuda")))
    stream = torch.cuda.Stream()
    dev = torch.cuda.current_device()

    def calls():
        for m, k, n, xt, bt, st, out in problems:
            rc = L.kiln_marlin_w4a16_gemm_static_scratch(xt.data_ptr(), bt.data_ptr(), out.data_ptr(), st.data_ptr(),
                                                         m, n, k, g, dev, stream.cuda_stream)
            assert rc == _lib.OK

    with torch.cuda.stream(stream):
        for _ in range(60):                         # eager warm-up (also of the runtime's own launch pools)
            calls()
        stream.synchronize()
        eager = [p[6].clone() for p in problems]
        free_before = torch.cuda.mem_get_info()[0]
        for _ in range(50):
            calls()
        stream.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            calls()
        for replay in range(4):
            for p in problems:
                p[6].fill_(float("nan"))
            graph.replay()
            stream.synchronize()
            for p, e in zip(problems, eager):
                assert torch.equal(p[6].view(torch.int16), e.view(torch.int16)), f"replay {replay}"
            calls()                                 # eager work between replays
            stream.synchronize()
    # nothing gave up on the way: the array's sticky word reads zero
    word = ctypes.c_uint32(0xFFFFFFFF)
    assert L.kiln_w4a16_workspace_check(None, ctypes.byref(word), None) == _lib.OK
    torch.cuda.synchronize()
    assert word.value == 0
