"""Committed golden vectors: the oracle must reproduce them (CPU), the HIP path must match them (GPU)."""
from pathlib import Path

import numpy as np
import pytest

G = np.load(Path(__file__).parent / "golden" / "w4a16_small.npz")
CASES = {"g128": (4, 256, 256, 128), "col": (3, 256, 256, -1)}


@pytest.mark.parametrize("tag", CASES)
def test_oracle_reproduces_golden(oracle, tag):
    m, k, n, g = CASES[tag]
    q, s, x = G[f"{tag}_qweight"], G[f"{tag}_scales_f16"], G[f"{tag}_x_bf16"]
    y = oracle.c_w4a16_cpu_path(x, q, s, g)
    assert np.array_equal(y.view(np.uint32), G[f"{tag}_y_f32"].view(np.uint32))
    deq = oracle.c_dequant_f32(q, s, g)
    assert np.array_equal(deq[[0, 1, 127, 128, 255]], G[f"{tag}_dequant_rows"])
    # the stored weights come from the reference test's LCG + quantiser
    w = oracle.c_lcg_fill(k * n, 0xC0FFEE5EED ^ k ^ (n << 16), 0.5).reshape(k, n)
    assert np.array_equal(w[:2, :8], G[f"{tag}_w_head"])
    codes, s_bits, _ = oracle.np_quantize(w, g)
    assert np.array_equal(oracle.np_pack_gptq(codes), q) and np.array_equal(s_bits, s)


@pytest.mark.parametrize("tag", CASES)
def test_host_repack_roundtrips_golden(tag):
    from kiln_amd.marlin_gemm import pack
    m, k, n, g = CASES[tag]
    b, s = pack.repack_gptq(G[f"{tag}_qweight"], G[f"{tag}_scales_f16"], None, g)
    q2, s2 = pack.unpack_to_gptq(b, s, g)
    assert np.array_equal(q2.view(np.uint32), G[f"{tag}_qweight"])
    assert np.array_equal(s2.view(np.uint16), G[f"{tag}_scales_f16"])


@pytest.mark.gpu
@pytest.mark.parametrize("tag", CASES)
def test_gpu_matches_golden(oracle, tag):
    import torch
    from kiln_amd import marlin_gemm
    from kiln_amd.marlin_gemm import pack
    from tests.gpu_util import bf16_bits, bf16_tensor, row_errors, upload_packed
    m, k, n, g = CASES[tag]
    b, s = pack.repack_gptq(G[f"{tag}_qweight"], G[f"{tag}_scales_f16"], None, g)
    bt, st = upload_packed(b, s)
    y = marlin_gemm.marlin_w4a16_gemm(bf16_tensor(G[f"{tag}_x_bf16"]), bt, st, g)
    torch.cuda.synchronize()
    err, _, _ = row_errors(bf16_bits(y), G[f"{tag}_y_f32"], oracle)
    assert err.max() <= 1e-2
    deq = marlin_gemm.dequant_f32(bt, st, g).cpu().numpy()
    assert np.array_equal(deq[[0, 1, 127, 128, 255]], G[f"{tag}_dequant_rows"])


def test_oracle_reproduces_golden_fused_paths(oracle):
    x = G["pf_x_bf16"]
    gate = oracle.c_w4a16_cpu_path(x, G["pf_gate_qweight"], G["pf_gate_scales_f16"], 128)
    up = oracle.c_w4a16_cpu_path(x, G["pf_up_qweight"], G["pf_up_scales_f16"], 128)
    assert np.array_equal(gate.view(np.uint32), G["pf_gate_y_f32"].view(np.uint32))
    assert np.array_equal(up.view(np.uint32), G["pf_up_y_f32"].view(np.uint32))
    assert np.array_equal(oracle.c_swiglu_f32(gate, up).view(np.uint32), G["pf_swiglu_h_f32"].view(np.uint32))
    y = gate.copy()
    for a_i, b_i, sc in ((G["pf_lora_a4"], G["pf_lora_b4"], 0.5), (G["pf_lora_a8"], G["pf_lora_b8"], 2.0)):
        oracle.c_lora_delta_add(y, x, a_i, b_i, sc)
    assert np.array_equal(y.view(np.uint32), G["pf_lora_y_f32"].view(np.uint32))
    assert np.array_equal(oracle.c_swiglu_f32(y, up).view(np.uint32), G["pf_swiglu_lora_h_f32"].view(np.uint32))


@pytest.mark.gpu
def test_gpu_matches_golden_fused_paths(oracle, matrix_core_kernel_from_33_rows):
    """M = 40 through the matrix-core kernel: plain, with two stacked LoRA adapters, and the
    fused gate+up SwiGLU, each against the committed expected values."""
    import torch
    from kiln_amd import marlin_gemm
    from kiln_amd.marlin_gemm import pack
    from tests.gpu_util import bf16_bits, bf16_tensor, row_errors, upload_packed
    g = 128
    xt = bf16_tensor(G["pf_x_bf16"])
    bg, sg = pack.repack_gptq(G["pf_gate_qweight"], G["pf_gate_scales_f16"], None, g)
    bu, su = pack.repack_gptq(G["pf_up_qweight"], G["pf_up_scales_f16"], None, g)
    bt, st = upload_packed(bg, sg)
    y = marlin_gemm.marlin_w4a16_gemm(xt, bt, st, g)
    err, _, _ = row_errors(bf16_bits(y), G["pf_gate_y_f32"], oracle)
    assert err.max() <= 1e-2
    a_cat = bf16_tensor(np.concatenate([G["pf_lora_a4"], G["pf_lora_a8"]], axis=0))
    b_cat = bf16_tensor(np.concatenate([G["pf_lora_b4"], G["pf_lora_b8"]], axis=1))
    yl = marlin_gemm.marlin_w4a16_gemm_lora(xt, bt, st, g, a_cat, b_cat, [4, 8], [0.5, 2.0])
    err, _, _ = row_errors(bf16_bits(yl), G["pf_lora_y_f32"], oracle)
    assert err.max() <= 1e-2
    b_gu, s_gu = pack.interleave_gate_up(bg, sg, bu, su, g)
    bgt, sgt = upload_packed(b_gu, np.asarray(s_gu).view(np.uint16))
    h = marlin_gemm.marlin_w4a16_gemm_swiglu(xt, bgt, sgt, g)
    torch.cuda.synchronize()
    err, _, _ = row_errors(bf16_bits(h), G["pf_swiglu_h_f32"], oracle)
    assert err.max() <= 1e-2
    # the same fused call with the two adapters on gate_proj (none on up_proj)
    b_il = marlin_gemm.interleave_gate_up_lora_b(b_cat, None, 256)
    hl = marlin_gemm.marlin_w4a16_gemm_swiglu_lora(xt, bgt, sgt, g, a_cat, b_il, [4, 8], [0.5, 2.0])
    torch.cuda.synchronize()
    err, _, _ = row_errors(bf16_bits(hl), G["pf_swiglu_lora_h_f32"], oracle)
    assert err.max() <= 1e-2
