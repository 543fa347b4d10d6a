"""The entry points only enqueue kernels (no allocation, no synchronisation, no memset), so a caller may
capture them into a HIP graph.  Each test captures a short sequence of calls, replays the graph several times
with eager launches and synchronisations in between, and compares every replay with the eager result bit for
bit: the K-sliced exchanges and the LoRA projection inside a launch depend on flags and counters that every
launch must leave as it found them."""
import numpy as np
import pytest
import torch

from kiln_amd import marlin_gemm

pytestmark = pytest.mark.gpu
GROUP = 128


def _weights(k, n, seed):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    b = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 16, 2 * n), dtype=torch.int32, device="cuda", generator=gen)
    s = (torch.rand(k // GROUP, n, device="cuda", generator=gen) * 0.018 + 0.002).to(torch.float16)
    return b, s


def _replay_and_compare(calls, outs, inputs):
    """calls(): enqueues the sequence on the current stream, writing `outs` from `inputs` in place."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        calls()                                    # workspaces are allocated outside the capture
        stream.synchronize()
        eager = [o.clone() for o in outs]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            calls()
        for replay in range(6):
            for o in outs:
                o.fill_(float("nan"))
            graph.replay()
            stream.synchronize()
            for i, (o, e) in enumerate(zip(outs, eager)):
                assert torch.equal(o.view(torch.int16), e.view(torch.int16)), f"replay {replay}, output {i}"
            # eager work of the same kind between replays, on other activations
            saved = [x.clone() for x in inputs]
            for x in inputs:
                x.copy_((torch.randn_like(x, dtype=torch.float32) * 0.5).to(torch.bfloat16))
            calls()
            stream.synchronize()
            for x, keep in zip(inputs, saved):
                x.copy_(keep)
            stream.synchronize()


@pytest.mark.parametrize("m", [1, 16, 64, 300])
def test_graph_of_plain_gemms_incl_k_sliced_ones(m):
    """gate+up (unsliced at few rows) then down (K slices meeting in the workspace) as a decode step issues them."""
    k1, n1, k2, n2 = 2560, 18432, 9216, 2560
    w1, w2 = _weights(k1, n1, 1), _weights(k2, n2, 2)
    x1 = (torch.randn(m, k1, device="cuda") * 0.5).to(torch.bfloat16)
    x2 = (torch.randn(m, k2, device="cuda") * 0.5).to(torch.bfloat16)
    o1 = torch.empty(m, n1, dtype=torch.bfloat16, device="cuda")
    o2 = torch.empty(m, n2, dtype=torch.bfloat16, device="cuda")

    def calls():
        for _ in range(2):
            marlin_gemm.marlin_w4a16_gemm(x1, w1[0], w1[1], GROUP, out=o1)
            marlin_gemm.marlin_w4a16_gemm(x2, w2[0], w2[1], GROUP, out=o2)

    _replay_and_compare(calls, [o1, o2], [x1, x2])


@pytest.mark.parametrize("m", [4, 16, 24, 64, 512])
def test_graph_of_gemms_with_adapters(m):
    """The LoRA entry points with the projection inside the launch (flags and counts in the zeroed prefix), plain
    and with the fused SwiGLU store, on the four projection shapes of a layer."""
    shapes = [(2560, 8192), (4096, 2560), (9216, 2560)]
    ranks, scales = (16, 32), (0.5, 1.0)
    ws = [_weights(k, n, 3 + i) for i, (k, n) in enumerate(shapes)]
    gen = torch.Generator(device="cuda").manual_seed(11)
    ad = [((torch.randn(sum(ranks), k, device="cuda", generator=gen) * 0.05).to(torch.bfloat16),
           (torch.randn(n, sum(ranks), device="cuda", generator=gen) * 0.05).to(torch.bfloat16)) for k, n in shapes]
    xs = [(torch.randn(m, k, device="cuda", generator=gen) * 0.5).to(torch.bfloat16) for k, _ in shapes]
    os_ = [torch.empty(m, n, dtype=torch.bfloat16, device="cuda") for _, n in shapes]
    n_out = 9216
    w_gu = _weights(2560, 2 * n_out, 9)
    a_gu = (torch.randn(64, 2560, device="cuda", generator=gen) * 0.05).to(torch.bfloat16)
    b_gu = (torch.randn(2 * n_out, 64, device="cuda", generator=gen) * 0.05).to(torch.bfloat16)
    x_gu = (torch.randn(m, 2560, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
    o_gu = torch.empty(m, n_out, dtype=torch.bfloat16, device="cuda")

    def calls():
        for (b, s), (la, lb), x, o in zip(ws, ad, xs, os_):
            marlin_gemm.marlin_w4a16_gemm_lora(x, b, s, GROUP, la, lb, ranks, scales, out=o)
        marlin_gemm.marlin_w4a16_gemm_swiglu_lora(x_gu, w_gu[0], w_gu[1], GROUP, a_gu, b_gu, (16, 16, 16, 16),
                                                  (1.0, 0.5, 1.0, 2.0), out=o_gu)
        marlin_gemm.marlin_w4a16_gemm_lora(xs[0], ws[0][0], ws[0][1], GROUP, ad[0][0], ad[0][1], ranks, scales, out=os_[0])

    _replay_and_compare(calls, os_ + [o_gu], xs + [x_gu])


def test_graph_of_device_pack_and_gemm():
    """Quantise-and-pack on the device followed by a GEMM on the fresh pack, captured together."""
    k, n, m = 2560, 2560, 8
    w = (torch.randn(k, n, device="cuda") * 0.02).to(torch.bfloat16)
    x = (torch.randn(m, k, device="cuda") * 0.5).to(torch.bfloat16)
    o = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    b = torch.empty((k // 16, 2 * n), dtype=torch.int32, device="cuda")
    s = torch.empty((k // GROUP, n), dtype=torch.float16, device="cuda")
    from kiln_amd import _lib
    lib = _lib.load()

    def calls():
        stream = torch.cuda.current_stream().cuda_stream
        st = lib.kiln_w4a16_quantize_and_pack_device(w.data_ptr(), k, n, GROUP, b.data_ptr(), s.data_ptr(), 0, stream)
        assert st == 0
        marlin_gemm.marlin_w4a16_gemm(x, b, s, GROUP, out=o)

    _replay_and_compare(calls, [o], [x])
    b_ref, s_ref = marlin_gemm.pack.quantize_and_pack_device(w, GROUP)
    assert torch.equal(b, b_ref) and torch.equal(s, s_ref)


def test_two_streams_with_their_own_workspaces_do_not_disturb_each_other():
    """The library has no state besides the caller's workspace: calls on two streams, each with the workspace the
    wrapper keeps for that stream, may overlap in time -- K-sliced GEMMs and GEMMs with adapters (whose flags and
    counters live in the workspace prefix) give the bits of the serial run."""
    m, ranks, scales = 16, (16, 32), (0.5, 1.0)
    shapes = [(9216, 2560), (2560, 8192)]
    ws = [_weights(k, n, 20 + i) for i, (k, n) in enumerate(shapes)]
    gen = torch.Generator(device="cuda").manual_seed(5)
    ad = [((torch.randn(sum(ranks), k, device="cuda", generator=gen) * 0.05).to(torch.bfloat16),
           (torch.randn(n, sum(ranks), device="cuda", generator=gen) * 0.05).to(torch.bfloat16)) for k, n in shapes]
    xs = [[(torch.randn(m, k, device="cuda", generator=gen) * 0.5).to(torch.bfloat16) for k, _ in shapes] for _ in range(2)]

    def run(side, outs):
        for j, ((b, s), (la, lb)) in enumerate(zip(ws, ad)):
            marlin_gemm.marlin_w4a16_gemm(xs[side][j], b, s, GROUP, out=outs[2 * j])
            marlin_gemm.marlin_w4a16_gemm_lora(xs[side][j], b, s, GROUP, la, lb, ranks, scales, out=outs[2 * j + 1])

    def fresh():
        return [torch.empty(m, n, dtype=torch.bfloat16, device="cuda") for _, n in shapes for _ in range(2)]

    serial = [fresh(), fresh()]
    for side in range(2):
        run(side, serial[side])
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for _ in range(20):
        both = [fresh(), fresh()]
        for rep in range(4):
            for side in range(2):
                with torch.cuda.stream(streams[side]):
                    run(side, both[side])
        torch.cuda.synchronize()
        for side in range(2):
            for o, e in zip(both[side], serial[side]):
                assert torch.equal(o.view(torch.int16), e.view(torch.int16))
