"""Fused gate+up projection with LoRA adapters on both sides and the SwiGLU epilogue
(`kiln_w4a16_gemm_swiglu_lora`) against the oracle: f32 GEMMs of the two projections (the reference
CPU path), each side's LoRA deltas added in f32 (lora_loader.rs:213-232), then silu(gate) * up
(crates/kiln-model/src/forward.rs:2771-2819), compared after one bf16 rounding."""
import numpy as np
import pytest
import torch

from kiln_amd import marlin_gemm
from kiln_amd.marlin_gemm import pack
from tests.gpu_util import bf16_bits, bf16_tensor, row_errors, upload_packed

pytestmark = pytest.mark.gpu
ROW_TOL = 1e-2   # max |h - h_ref| <= 1e-2 * max |h_ref| per row, h_ref = bf16(f32 oracle)


def _problem(oracle, m, k, n_out, gate_ranks, up_ranks, seed, sigma=1.0, sigma_ab=0.05):
    """Returns x, the interleaved pack, the stacked adapters and the oracle's result with and without them."""
    g = 128
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
    h_plain = oracle.c_swiglu_f32(gate, up)
    a_all, ranks, scales, b_side = [], [], [], []
    for side, (y, side_ranks) in enumerate(((gate, gate_ranks), (up, up_ranks))):
        bs = []
        for i, r in enumerate(side_ranks):
            a_i = oracle.gen_normal_bf16(r, k, sigma_ab, seed=seed + 100 * side + 10 + i)
            b_i = oracle.gen_normal_bf16(n_out, r, sigma_ab, seed=seed + 100 * side + 20 + i)
            sc = (0.5, 1.0, 2.0, 0.25)[(i + 2 * side) % 4]
            oracle.c_lora_delta_add(y, x, a_i, b_i, sc)
            a_all.append(a_i)
            bs.append(b_i)
            ranks.append(r)
            scales.append(sc)
        b_side.append(bf16_tensor(np.concatenate(bs, axis=1)) if bs else None)
    h_ref = oracle.c_swiglu_f32(gate, up)
    a_cat = bf16_tensor(np.concatenate(a_all, axis=0))
    b_cat = marlin_gemm.interleave_gate_up_lora_b(b_side[0], b_side[1], n_out)
    return x, b_gu, s_gu, a_cat, b_cat, ranks, scales, h_ref, h_plain


@pytest.mark.parametrize("m,k,n_out,gate_ranks,up_ranks", [
    (1, 2560, 1024, (16,), (16,)),
    (16, 2560, 9216, (16, 16), (16, 16)),   # the model's MLP at 16 rows, two adapters a side: rank 64 in all
    (4, 9216, 1280, (8,), (24,)),           # K slices of the product
    (5, 1024, 256, (4,), (5,)),             # ranks that are not multiples of 8: the kernels that read B element-wise
    (16, 2560, 1024, (16,), ()),            # an adapter on gate only
    (8, 2560, 1024, (), (32,)),             # ... on up only
    (24, 2560, 9216, (16,), (32,)),         # 17...128 rows: the mid-M kernel
    (64, 2560, 9216, (16, 16), (16, 16)),
    (100, 512, 256, (8,), (8,)),
    (40, 2560, 1024, (3,), (8,)),           # an odd stacked rank beyond 32 rows
    (200, 2560, 2560, (16,), (32,)),        # the matrix-core kernel, 64-row blocks
    (512, 2560, 9216, (16, 32), (16,)),     # ... on the model's MLP
    (1100, 1024, 4096, (16,), (16,)),       # 128-row blocks
    (2048, 2560, 9216, (16, 16), (16, 16)), # the chunked-prefill configuration's rows on the model's MLP
])
def test_swiglu_lora_cases(oracle, m, k, n_out, gate_ranks, up_ranks):
    sigma = 1.0 if m <= 128 else 0.5
    x, b_gu, s_gu, a_cat, b_cat, ranks, scales, h_ref, h_plain = _problem(
        oracle, m, k, n_out, gate_ranks, up_ranks, seed=m + k + n_out, sigma=sigma)
    bt, st = upload_packed(b_gu, np.asarray(s_gu).view(np.uint16))
    h = marlin_gemm.marlin_w4a16_gemm_swiglu_lora(bf16_tensor(x), bt, st, 128, a_cat, b_cat, ranks, scales)
    torch.cuda.synchronize()
    assert tuple(h.shape) == (m, n_out) and h.dtype == torch.bfloat16
    err, hv, _ = row_errors(bf16_bits(h), h_ref, oracle)
    assert np.all(np.isfinite(hv))
    assert err.max() <= ROW_TOL, f"m={m} k={k} n_out={n_out}: worst row error {err.max():.3e}"
    # the adapters matter at this size: the result without them is far outside the bound
    miss, _, _ = row_errors(bf16_bits(h), h_plain, oracle)
    assert miss.max() > 5 * ROW_TOL


@pytest.mark.parametrize("m", [16, 64, 300])
def test_swiglu_lora_with_zero_b_equals_the_plain_fused_call(oracle, m):
    """Adapters whose B is zero add nothing: every bit equals `marlin_w4a16_gemm_swiglu`."""
    k, n_out = 2560, 2560
    x, b_gu, s_gu, a_cat, b_cat, ranks, scales, _, _ = _problem(oracle, m, k, n_out, (16,), (16,), seed=m)
    bt, st = upload_packed(b_gu, np.asarray(s_gu).view(np.uint16))
    xt = bf16_tensor(x)
    plain = marlin_gemm.marlin_w4a16_gemm_swiglu(xt, bt, st, 128)
    h = marlin_gemm.marlin_w4a16_gemm_swiglu_lora(xt, bt, st, 128, a_cat, torch.zeros_like(b_cat), ranks, scales)
    assert torch.equal(plain.view(torch.int16), h.view(torch.int16))


def test_swiglu_lora_matches_the_unfused_library_route(oracle):
    """Against `marlin_w4a16_gemm_lora` on each side's own pack followed by silu * up in torch f32
    on the bf16 results (what the reference's call sites do): within two bf16 roundings."""
    m, k, n_out = 48, 2560, 1024
    g = 128
    x = oracle.gen_normal_bf16(m, k, 1.0, 7)
    packs, adapters = [], []
    for side in range(2):
        codes = oracle.gen_codes(k, n_out, 11 + side)
        s_bits = oracle.gen_scales_f16(k, n_out, g, 11 + side)
        b, s = pack.repack_gptq(oracle.np_pack_gptq(codes), s_bits, None, g)
        packs.append((b, s))
        adapters.append((bf16_tensor(oracle.gen_normal_bf16(16, k, 0.05, 21 + side)),
                         bf16_tensor(oracle.gen_normal_bf16(n_out, 16, 0.05, 31 + side))))
    xt = bf16_tensor(x)
    sides = []
    for (b, s), (la, lb) in zip(packs, adapters):
        bt, st = upload_packed(b, s)
        sides.append(marlin_gemm.marlin_w4a16_gemm_lora(xt, bt, st, g, la, lb, [16], [1.0]).float())
    unfused = torch.nn.functional.silu(sides[0]) * sides[1]
    b_gu, s_gu = pack.interleave_gate_up(packs[0][0], packs[0][1], packs[1][0], packs[1][1], g)
    bt, st = upload_packed(b_gu, np.asarray(s_gu).view(np.uint16))
    a_cat = torch.cat([adapters[0][0], adapters[1][0]], dim=0)
    b_cat = marlin_gemm.interleave_gate_up_lora_b(adapters[0][1], adapters[1][1], n_out)
    h = marlin_gemm.marlin_w4a16_gemm_swiglu_lora(xt, bt, st, g, a_cat, b_cat, [16, 16], [1.0, 1.0]).float()
    bound = 2.0 ** -6 * unfused.abs().amax(dim=1, keepdim=True)
    assert bool(((h - unfused).abs() <= bound).all())


def test_swiglu_lora_argument_checks():
    a = torch.zeros((4, 256), dtype=torch.bfloat16, device="cuda")
    b = torch.zeros((16, 1024), dtype=torch.int32, device="cuda")
    s = torch.zeros((2, 512), dtype=torch.float16, device="cuda")
    la = torch.zeros((8, 256), dtype=torch.bfloat16, device="cuda")
    lb = torch.zeros((512, 8), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(marlin_gemm.MarlinGemmError):
        marlin_gemm.marlin_w4a16_gemm_swiglu_lora(a, b, s, 128, la, lb[:256], [8], [1.0])   # B of one side only
    with pytest.raises(marlin_gemm.MarlinGemmError):
        marlin_gemm.marlin_w4a16_gemm_swiglu_lora(a, b, s, 128, la, lb, [4], [1.0])         # ranks do not add up
    h = marlin_gemm.marlin_w4a16_gemm_swiglu_lora(a, b, s, 128, la, lb, [8], [1.0])
    assert tuple(h.shape) == (4, 256)
