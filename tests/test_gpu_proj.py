"""The C++ projection layer (include/kiln_marlin_proj.h) on the GPU: packing at load, the
rank-2 / rank-3 activation path, the persisted artefact.  Mirrors what the reference exercises
through crates/kiln-model/src/marlin_proj.rs and crates/kiln-model/tests/marlin_qproj_parity.rs."""
import numpy as np
import pytest
import torch

from kiln_amd import marlin_gemm, marlin_proj
from kiln_amd.marlin_gemm import pack
from tests.gpu_util import bf16_bits, bf16_tensor, row_errors

pytestmark = pytest.mark.gpu
ROW_TOL = 1e-2


def _weight(oracle, k, n, seed):
    w = oracle.c_lcg_fill(k * n, seed, 0.05).reshape(k, n)
    return w, bf16_tensor(oracle.np_f32_to_bf16(w))


def test_native_pack_matches_the_three_phases(oracle):
    k, n = 512, 768
    _, w_bf = _weight(oracle, k, n, 3)
    for g in (128, -1):
        native = marlin_proj.pack_from_bf16(w_bf, g)
        phases = marlin_proj.upload_packed(marlin_proj.pack_host(marlin_proj.prepare_pack_job(w_bf, g)), w_bf.device)
        assert native.native is not None and (native.k, native.n, native.groupsize) == (k, n, g)
        assert tuple(native.b_packed.shape) == (k // 16, n * 16 // 8) and native.b_packed.dtype == torch.int32
        assert tuple(native.scales.shape) == (1 if g == -1 else k // g, n) and native.scales.dtype == torch.float16
        assert torch.equal(native.b_packed, phases.b_packed) and torch.equal(native.scales, phases.scales)


def test_native_batch_pack_keeps_order_and_skips(monkeypatch, oracle):
    ws = [_weight(oracle, 256, 512, 1)[1], _weight(oracle, 256, 100, 2)[1], _weight(oracle, 384, 256, 3)[1]]
    singles = [marlin_proj.pack_from_bf16(w, 128) for w in ws]
    for disable in ("0", "1"):
        monkeypatch.setenv("KILN_DISABLE_PARALLEL_PACK", disable)
        out = marlin_proj.pack_from_bf16_batch([(w, 128) for w in ws])
        assert out[1] is None and singles[1] is None
        for a, b in ((out[0], singles[0]), (out[2], singles[2])):
            assert torch.equal(a.b_packed, b.b_packed) and torch.equal(a.scales, b.scales)


def test_native_gptq_repack_and_matmul_ranks(oracle, monkeypatch):
    m, k, n, g = 24, 2560, 1024, 128
    x, q, s_bits = oracle.gen_problem(m, k, n, g, seed=5)
    b, s = pack.repack_gptq(q, s_bits, None, g)
    good_zeros = torch.full((k // g, n // 8), -0x77777778, dtype=torch.int32)     # 0x88888888
    monkeypatch.setenv("KILN_W4A16_HOST_PACK", "1")                                  # the host route of the repack
    on_host = marlin_proj.pack_from_gptq(torch.from_numpy(q.view(np.int32)), torch.from_numpy(s_bits.view(np.float16)),
                                         good_zeros, g, "cuda")
    monkeypatch.delenv("KILN_W4A16_HOST_PACK")
    proj = marlin_proj.pack_from_gptq(torch.from_numpy(q.view(np.int32)), torch.from_numpy(s_bits.view(np.float16)),
                                      good_zeros, g, "cuda")
    assert torch.equal(proj.b_packed, on_host.b_packed) and torch.equal(proj.scales, on_host.scales)
    proj = marlin_proj.pack_from_gptq(torch.from_numpy(q.view(np.int32)), torch.from_numpy(s_bits.view(np.float16)),
                                      None, g, "cuda")
    assert np.array_equal(proj.b_packed.cpu().numpy(), b)
    assert np.array_equal(proj.scales.cpu().numpy().view(np.uint16), np.asarray(s).view(np.uint16))
    y_ref = oracle.c_w4a16_cpu_path(x, q, s_bits, g)
    xt = bf16_tensor(x)
    y2 = marlin_proj.matmul_bf16(xt, proj)
    y3 = marlin_proj.matmul_bf16(xt.reshape(4, 6, k), proj)
    assert tuple(y2.shape) == (m, n) and tuple(y3.shape) == (4, 6, n)
    assert torch.equal(y2, y3.reshape(m, n))
    assert torch.equal(y2, marlin_gemm.marlin_w4a16_gemm(xt, proj.b_packed, proj.scales, g))
    err, _, _ = row_errors(bf16_bits(y2), y_ref, oracle)
    assert err.max() <= ROW_TOL
    with pytest.raises(marlin_proj.MarlinProjError, match=r"x last-dim 128 != packed weight k 2560"):
        marlin_proj.matmul_bf16(torch.zeros(4, 128, dtype=torch.bfloat16, device="cuda"), proj)
    with pytest.raises(marlin_proj.MarlinProjError, match="unsupported activation rank 4"):
        marlin_proj.matmul_bf16(torch.zeros(1, 2, 2, k, dtype=torch.bfloat16, device="cuda"), proj)
    bad_zeros = torch.full((k // g, n // 8), 0x77777777, dtype=torch.int32)
    with pytest.raises(marlin_proj.MarlinProjError, match="zero-point"):
        marlin_proj.pack_from_gptq(torch.from_numpy(q.view(np.int32)), torch.from_numpy(s_bits.view(np.float16)),
                                   bad_zeros, g, "cuda")


def test_saved_projection_loads_bit_identical(tmp_path, oracle):
    m, k, n = 40, 1024, 512
    _, w_bf = _weight(oracle, k, n, 9)
    proj = marlin_proj.pack_from_bf16(w_bf, 128)
    path = tmp_path / "q_proj.kw4a16"
    marlin_proj.save(proj, path)
    again = marlin_proj.load(path, "cuda")
    assert (again.k, again.n, again.groupsize) == (k, n, 128)
    assert torch.equal(again.b_packed, proj.b_packed) and torch.equal(again.scales, proj.scales)
    x = bf16_tensor(oracle.gen_normal_bf16(m, k, 1.0, seed=2))
    assert torch.equal(marlin_proj.matmul_bf16(x, proj), marlin_proj.matmul_bf16(x, again))
    raw = bytearray(path.read_bytes()); raw[-1] ^= 1
    path.write_bytes(bytes(raw))
    with pytest.raises(marlin_proj.MarlinProjError, match="checksum mismatch"):
        marlin_proj.load(path, "cuda")
