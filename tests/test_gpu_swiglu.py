"""Fused gate+up projection with the SwiGLU epilogue (`kiln_w4a16_gemm_swiglu`) against the
oracle: f32 GEMMs of the two projections (the reference CPU path), then silu(gate) * up
(crates/kiln-model/src/forward.rs:2771-2819), compared after one bf16 rounding."""
import numpy as np
import pytest
import torch

from kiln_amd import marlin_gemm
from kiln_amd.marlin_gemm import pack
from tests.gpu_util import bf16_bits, bf16_tensor, row_errors, upload_packed

pytestmark = pytest.mark.gpu
ROW_TOL = 1e-2   # max |y - y_ref| <= 1e-2 * max |y_ref| per row, y_ref = bf16(f32 oracle)


def _problem(oracle, m, k, n_out, g, seed, sigma=1.0):
    x = oracle.gen_normal_bf16(m, k, sigma, seed)
    sides = []
    for s2 in (seed * 2 + 1, seed * 2 + 2):
        codes = oracle.gen_codes(k, n_out, s2)
        s_bits = oracle.gen_scales_f16(k, n_out, g, s2)
        q = oracle.np_pack_gptq(codes)
        b, s = pack.repack_gptq(q, s_bits, None, g)
        sides.append((q, s_bits, b, s))
    b_gu, s_gu = pack.interleave_gate_up(sides[0][2], sides[0][3], sides[1][2], sides[1][3], g)
    gate = oracle.c_w4a16_cpu_path(x, sides[0][0], sides[0][1], g)
    up = oracle.c_w4a16_cpu_path(x, sides[1][0], sides[1][1], g)
    return x, b_gu, s_gu, oracle.c_swiglu_f32(gate, up)


@pytest.mark.parametrize("m,k,n_out,g,sigma", [
    (1, 2560, 1024, 128, 1.0), (16, 2560, 1024, 128, 1.0), (32, 256, 256, -1, 1.0),
    (4, 9216, 1280, 128, 1.0),      # K slices: the product is formed by the block that sums them
    (16, 2560, 9216, 128, 1.0), (24, 2560, 9216, 128, 1.0), (40, 9216, 1280, 128, 1.0),
    (33, 2560, 1024, 128, 1.0), (64, 2560, 9216, 128, 1.0), (100, 512, 256, 128, 1.0), (128, 2560, 9216, 128, 1.0),
    (300, 2560, 2560, 128, 0.5), (1000, 1024, 4096, 128, 0.5), (2048, 2560, 9216, 128, 0.5),
    # plans of the mid-M kernel that other models' shapes take: ten wavefronts (40 groups unsliced, up to 32 rows), a
    # shorter last K slice (86 groups), both with the fused store; and its longer row range on small weights
    (32, 5120, 512, 128, 1.0), (48, 11008, 512, 128, 1.0), (24, 11008, 256, 128, 1.0), (700, 1024, 512, 128, 0.5),
])
def test_swiglu_cases(oracle, m, k, n_out, g, sigma):
    x, b_gu, s_gu, h_ref = _problem(oracle, m, k, n_out, g, seed=m + k + n_out, sigma=sigma)
    bt, st = upload_packed(b_gu, np.asarray(s_gu).view(np.uint16))
    h = marlin_gemm.marlin_w4a16_gemm_swiglu(bf16_tensor(x), bt, st, g)
    torch.cuda.synchronize()
    assert tuple(h.shape) == (m, n_out) and h.dtype == torch.bfloat16
    err, hv, _ = row_errors(bf16_bits(h), h_ref, oracle)
    assert np.all(np.isfinite(hv))
    assert err.max() <= ROW_TOL, f"m={m} k={k} n_out={n_out}: worst row error {err.max():.3e}"


def test_swiglu_matches_unfused_calls_and_repeats(oracle):
    """Against the unfused route through the same library (GEMM on the interleaved pack, then
    silu * up in torch f32), and run-to-run identical in both regimes."""
    k, n_out, g = 2560, 2560, 128
    for m in (8, 200):
        x, b_gu, s_gu, _ = _problem(oracle, m, k, n_out, g, seed=m)
        bt, st = upload_packed(b_gu, np.asarray(s_gu).view(np.uint16))
        xt = bf16_tensor(x)
        h = marlin_gemm.marlin_w4a16_gemm_swiglu(xt, bt, st, g)
        for _ in range(3):
            assert torch.equal(marlin_gemm.marlin_w4a16_gemm_swiglu(xt, bt, st, g), h)
        y = marlin_gemm.marlin_w4a16_gemm(xt, bt, st, g).float().reshape(m, n_out // 8, 2, 8)
        unfused = (torch.nn.functional.silu(y[:, :, 0]) * y[:, :, 1]).reshape(m, n_out)
        scale = unfused.abs().amax(dim=1, keepdim=True)
        assert torch.all((h.float() - unfused).abs() <= 1e-2 * scale)


def test_swiglu_argument_checks():
    E = marlin_gemm.MarlinGemmError
    a = torch.zeros(4, 128, dtype=torch.bfloat16, device="cuda")
    b = torch.zeros(8, 2 * 384, dtype=torch.int32, device="cuda")     # 384 packed columns: not a multiple of 256
    s = torch.zeros(1, 384, dtype=torch.float16, device="cuda")
    with pytest.raises(E):
        marlin_gemm.marlin_w4a16_gemm_swiglu(a, b, s, 128)
