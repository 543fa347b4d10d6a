"""kiln_w4a16_mlp: y = down(silu(gate(x)) * up(x)) as one call (crates/kiln-model/src/forward.rs:2723-2848):
the fused gate+up SwiGLU GEMM, then the down GEMM, with H = silu(gate) * up kept in the workspace.  Checked
against the oracle (gate, up and down through the CPU path, H rounded to bf16 between them as the call
rounds it) and, bit for bit, against the two entry points called one after the other."""
import ctypes

import numpy as np
import pytest
import torch

from kiln_amd import _lib, marlin_gemm
from kiln_amd.marlin_gemm import pack
from tests.gpu_util import bf16_bits, bf16_tensor, row_errors, upload_packed

pytestmark = pytest.mark.gpu
HIDDEN, INTER = 2560, 9216


def _mlp_weights(oracle, hidden, inter, n_down, g, seed):
    _, q_gate, s_gate = oracle.gen_problem(1, hidden, inter, g, seed=seed)
    _, q_up, s_up = oracle.gen_problem(1, hidden, inter, g, seed=seed + 1)
    _, q_down, s_down = oracle.gen_problem(1, inter, n_down, g, seed=seed + 2)
    bg, sg = pack.repack_gptq(q_gate, s_gate, None, g)
    bu, su = pack.repack_gptq(q_up, s_up, None, g)
    b_gu, s_gu = pack.interleave_gate_up(bg, sg, bu, su, g)
    bd, sd = pack.repack_gptq(q_down, s_down, None, g)
    dev = (*upload_packed(b_gu, np.asarray(s_gu).view(np.uint16)), *upload_packed(bd, sd))
    return (q_gate, s_gate, q_up, s_up, q_down, s_down), dev


def _oracle_mlp(oracle, x, host, g):
    q_gate, s_gate, q_up, s_up, q_down, s_down = host
    h = oracle.c_swiglu_f32(oracle.c_w4a16_cpu_path(x, q_gate, s_gate, g), oracle.c_w4a16_cpu_path(x, q_up, s_up, g))
    return oracle.c_w4a16_cpu_path(oracle.np_f32_to_bf16(h), q_down, s_down, g)


@pytest.fixture(scope="module")
def model_mlp(oracle):
    return _mlp_weights(oracle, HIDDEN, INTER, HIDDEN, 128, seed=50)


@pytest.mark.parametrize("m", [1, 4, 9, 16, 40, 130])
def test_mlp_on_the_model_shape(oracle, model_mlp, m):
    host, (b_gu, s_gu, bd, sd) = model_mlp
    x = oracle.gen_normal_bf16(m, HIDDEN, 0.5 if m > 64 else 1.0, seed=60 + m)
    xt = bf16_tensor(x)
    y = marlin_gemm.marlin_w4a16_mlp(xt, b_gu, s_gu, bd, sd, 128)
    torch.cuda.synchronize()
    err, yv, _ = row_errors(bf16_bits(y), _oracle_mlp(oracle, x, host, 128), oracle)
    assert np.all(np.isfinite(yv)) and err.max() <= 1e-2, err.max()
    h = marlin_gemm.marlin_w4a16_gemm_swiglu(xt, b_gu, s_gu, 128)
    y2 = marlin_gemm.marlin_w4a16_gemm(h, bd, sd, 128)
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))


@pytest.mark.parametrize("m,hidden,inter,n_down,g", [
    (16, 256, 512, 256, 128),
    (300, 256, 1024, 512, -1),
    (7, HIDDEN, INTER, HIDDEN, -1),
])
def test_mlp_at_other_shapes_and_per_column_scales(oracle, m, hidden, inter, n_down, g):
    host, (b_gu, s_gu, bd, sd) = _mlp_weights(oracle, hidden, inter, n_down, g, seed=m + inter)
    x = oracle.gen_normal_bf16(m, hidden, 0.5 if m > 64 else 1.0, seed=90 + m)
    y = marlin_gemm.marlin_w4a16_mlp(bf16_tensor(x), b_gu, s_gu, bd, sd, g)
    torch.cuda.synchronize()
    err, yv, _ = row_errors(bf16_bits(y), _oracle_mlp(oracle, x, host, g), oracle)
    assert np.all(np.isfinite(yv)) and err.max() <= 1e-2, err.max()


def test_mlp_replays_from_a_graph_with_a_workspace_sized_for_more_rows(oracle, model_mlp):
    """H sits behind what the two GEMMs need for the call's row count: a workspace sized once for the most
    rows serves every smaller call, also from a graph."""
    host, (b_gu, s_gu, bd, sd) = model_mlp
    L = _lib.load()
    ws = torch.empty(L.kiln_w4a16_mlp_workspace_bytes(64, HIDDEN, INTER, HIDDEN), dtype=torch.uint8, device="cuda")
    ws[:L.kiln_w4a16_workspace_zeroed_bytes()].zero_()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for m in (64, 16, 3):
            x = bf16_tensor(oracle.gen_normal_bf16(m, HIDDEN, 1.0, seed=80 + m))
            out = torch.empty(m, HIDDEN, dtype=torch.bfloat16, device="cuda")

            def call():
                assert L.kiln_w4a16_mlp(x.data_ptr(), b_gu.data_ptr(), s_gu.data_ptr(), bd.data_ptr(), sd.data_ptr(),
                                        out.data_ptr(), m, HIDDEN, INTER, HIDDEN, ws.data_ptr(), 128, 0,
                                        stream.cuda_stream) == _lib.OK
            call()
            stream.synchronize()
            eager = out.clone()
            assert torch.equal(eager, marlin_gemm.marlin_w4a16_mlp(x, b_gu, s_gu, bd, sd, 128))
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                call()
            for replay in range(3):
                out.fill_(float("nan"))
                graph.replay()
                stream.synchronize()
                assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), (m, replay)


def test_mlp_workspace_bytes_and_argument_checks():
    L = _lib.load()
    sizes = [L.kiln_w4a16_mlp_workspace_bytes(m, HIDDEN, INTER, HIDDEN) for m in (1, 4, 16, 17, 64, 512)]
    assert sizes == sorted(sizes) and sizes[0] >= L.kiln_w4a16_workspace_zeroed_bytes() + 1 * INTER * 2
    p = ctypes.c_void_p(1 << 20)
    stream = torch.cuda.current_stream().cuda_stream
    assert L.kiln_w4a16_mlp(p, p, p, p, p, p, 4, HIDDEN, INTER + 64, HIDDEN, p, 128, 0, stream) == _lib.ERR_PROB_SHAPE
    assert L.kiln_w4a16_mlp(p, p, p, p, p, p, 4, HIDDEN, INTER, HIDDEN, p, 64, 0, stream) == _lib.ERR_PROB_SHAPE
    assert L.kiln_w4a16_mlp(p, p, p, p, p, None, 4, HIDDEN, INTER, HIDDEN, p, 128, 0, stream) == _lib.ERR_ARGUMENT
    assert L.kiln_w4a16_mlp(p, p, p, p, p, p, 0, HIDDEN, INTER, HIDDEN, p, 128, 0, stream) == _lib.OK
