"""Fused LoRA epilogue against the f32 oracle (lora_loader.rs:213-232 semantics in f32)."""
import numpy as np
import pytest
import torch

from kiln_amd import lora as klora
from kiln_amd import marlin_gemm, marlin_proj
from kiln_amd.marlin_gemm import pack
from tests.gpu_util import bf16_bits, bf16_tensor, row_errors, upload_packed

pytestmark = pytest.mark.gpu


def _lora_case(oracle, m, k, n, ranks, scales, seed, sigma_x=1.0, sigma_ab=0.02):
    g = 128
    x, q, s_bits = oracle.gen_problem(m, k, n, g, seed=seed, sigma=sigma_x)
    b, s = pack.repack_gptq(q, s_bits, None, g)
    a_list = [oracle.gen_normal_bf16(r, k, sigma_ab, seed=seed + 10 + i) for i, r in enumerate(ranks)]
    b_list = [oracle.gen_normal_bf16(n, r, sigma_ab, seed=seed + 20 + i) for i, r in enumerate(ranks)]
    y_ref = oracle.c_w4a16_cpu_path(x, q, s_bits, g)
    for a_i, b_i, sc in zip(a_list, b_list, scales):
        oracle.c_lora_delta_add(y_ref, x, a_i, b_i, sc)
    bt, st = upload_packed(b, s)
    a_cat = bf16_tensor(np.concatenate(a_list, axis=0))
    b_cat = bf16_tensor(np.concatenate(b_list, axis=1))
    y = marlin_gemm.marlin_w4a16_gemm_lora(bf16_tensor(x), bt, st, g, a_cat, b_cat, ranks, scales)
    torch.cuda.synchronize()
    err, _, _ = row_errors(bf16_bits(y), y_ref, oracle)
    assert err.max() <= 1e-2, f"worst row error {err.max():.3e}"
    return y, y_ref


@pytest.mark.parametrize("m,k,n,ranks,scales", [
    (512, 2560, 18432, (16, 32), (0.5, 1.0)),      # the benchmark's LoRA configuration
    (1, 2560, 2560, (16,), (2.0,)),
    (16, 2560, 8192, (8, 8, 16), (1.0, 0.25, 0.5)),
    (77, 9216, 2560, (64,), (1.0,)),
    (300, 256, 256, (4, 5), (1.0, 3.0)),            # ranks that are not multiples of 8
    (1100, 4224, 256, (16, 32), (0.5, 1.0)),        # long K and many rows: the projection's 64-row blocks
    (200, 9216, 256, (7,), (1.5,)),                 # long K, few row tiles: 16 K slices meet per tile
    # the product's blocks fit the chip's block slots, but not together with all K slices of the projection in
    # front of them: the projection is cut into fewer slices
    (900, 2560, 8192, (16, 32), (0.5, 1.0)), (576, 4096, 4096, (16, 32), (0.5, 1.0)),
])
def test_fused_lora_matches_oracle(oracle, m, k, n, ranks, scales):
    _lora_case(oracle, m, k, n, ranks, scales, seed=m + n)


@pytest.mark.parametrize("k,n", [(2560, 18432), (9216, 2560), (2560, 8192)])
@pytest.mark.parametrize("m", [1, 3, 16, 17, 32, 33, 48, 64, 80, 128, 160])
def test_lora_on_few_rows(oracle, m, k, n):
    """Few rows take the small-M kernels, which add the low-rank term where they store a tile (the
    decode kernel up to 16 rows, the mid-M kernel beyond); adapters large enough that a missing term fails."""
    _lora_case(oracle, m, k, n, (16, 32), (0.5, 1.0), seed=3 * m + n, sigma_ab=0.05)


@pytest.mark.parametrize("m,k,n", [
    (1, 18944, 3584), (16, 18944, 3584),   # the projection's wavefronts take ten steps of K each
    (5, 5120, 13824), (16, 5120, 13824),   # 40 groups unsliced: 14 main wavefronts of three groups beside the adapter's
    (3, 5120, 27648),                      # ... and a launch of more blocks than compute units, the projection in its first ones
    (16, 11008, 4096), (3, 11008, 4096),   # as many small-M blocks as compute units: the mid-M kernel takes the call, from one row
])
def test_lora_on_few_rows_of_other_models_weights(oracle, m, k, n):
    _lora_case(oracle, m, k, n, (16, 32), (0.5, 1.0), seed=5 * m + n, sigma_ab=0.05)


@pytest.mark.parametrize("m,k,n", [(17, 5120, 512), (32, 5120, 768), (24, 9216, 512), (32, 8192, 1024), (20, 4096, 512),
                                   (24, 3584, 18944), (32, 2560, 18432)])   # wide outputs: blocks of three pairs
def test_lora_on_ten_wavefronts(oracle, m, k, n):
    """Up to 32 rows the blocks of a call with adapters may have ten wavefronts, in plans of one or two K slices:
    40 and 32 groups unsliced, 72 and 64 in two slices."""
    _lora_case(oracle, m, k, n, (16, 32), (0.5, 1.0), seed=13 * m + n, sigma_ab=0.05)


@pytest.mark.parametrize("m,k,n", [(128, 2560, 12288), (100, 2048, 11264), (64, 2560, 12288)])
def test_lora_where_the_mid_m_blocks_just_fill_the_chip(oracle, m, k, n):
    """Two runs of 128 three-pair blocks are one round of the chip: the projection's blocks would push the plan
    into a second round, so it runs in front there (and inside the launch at 64 rows, where there is room)."""
    _lora_case(oracle, m, k, n, (16, 32), (0.5, 1.0), seed=11 * m + n, sigma_ab=0.05)


@pytest.mark.parametrize("m", [17, 32, 48, 64, 100, 128])
@pytest.mark.parametrize("k,n", [(11008, 512), (8960, 256)])
def test_lora_with_a_shorter_last_k_slice(oracle, m, k, n):
    """86 and 70 groups of K have no even slicing that fits the mid-M kernel's wavefronts: its last slice is
    shorter, with adapters as without."""
    import ctypes
    from kiln_amd import _lib
    out = (ctypes.c_int * 8)()
    assert _lib.load().kiln_w4a16_debug_gemm_plan(m, n, k, 256, out) == 0 and out[6] == 1, list(out)
    _lora_case(oracle, m, k, n, (16, 32), (0.5, 1.0), seed=7 * m + n, sigma_ab=0.05)


@pytest.mark.parametrize("m,k,n", [
    (192, 2560, 8192), (256, 4096, 2560), (257, 4096, 2560), (300, 2560, 2560), (320, 4096, 2560), (320, 2560, 1024),
    (321, 2560, 1024),
])
def test_lora_where_small_weights_keep_the_mid_m_kernel(oracle, m, k, n):
    """Small weights keep the mid-M kernel up to 192 ... 320 rows with adapters.  Up to four runs of rows
    (256) the projection runs in the launch's first blocks, beyond that in a launch in front (a call of 320
    rows was once refused: the dispatcher asked for the former where the launch only takes the latter)."""
    _lora_case(oracle, m, k, n, (16, 32), (0.5, 1.0), seed=5 * m + n, sigma_ab=0.05)


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("m,k,n,ranks", [
    (16, 2560, 4096, (16, 32)),
    (5, 1024, 2560, (4, 5)),        # ranks that are not multiples of 8: element-wise reads of B
    (29, 2560, 2048, (64,)),
    (16, 9216, 512, (3,)),          # K slices: the term is added once, by the block that sums the slices
])
def test_lora_through_every_small_m_kernel(oracle, mode, m, k, n, ranks):
    """The three small-M kernels (tile-major runs, group-major staged, group-major in registers),
    chosen through the tuning hook."""
    from kiln_amd import _lib
    lib = _lib.load_tuning()
    lib.kiln_w4a16_debug_decode_group_major(mode)
    try:
        _lora_case(oracle, m, k, n, ranks, tuple(0.5 + i for i in range(len(ranks))), seed=m + k, sigma_ab=0.05)
    finally:
        lib.kiln_w4a16_debug_decode_group_major(-1)


@pytest.mark.parametrize("m,k,n,ranks", [
    (1, 128, 256, (1,)),             # one group of K, rank 1
    (7, 128, 256, (64,)),            # the largest rank on a single group of K
    (33, 384, 512, (9, 23)),         # a slab of 32 rows and one of 1; K not a multiple of the 256-value piece
    (64, 640, 768, (32, 32)),        # two full slabs, four row tiles of the projection
    (16, 4224, 256, (8,)),           # 33 groups: slices of unequal length
])
def test_lora_edge_shapes_on_few_rows(oracle, m, k, n, ranks):
    _lora_case(oracle, m, k, n, ranks, tuple(1.0 - 0.25 * i for i in range(len(ranks))), seed=k + n + m,
               sigma_ab=0.05)


@pytest.mark.parametrize("m,k,n,ranks", [
    (65, 128, 256, (64,)),           # one group of K: a single slice, nothing meets
    (129, 384, 256, (5,)),           # odd rank, K not a multiple of the piece
    (1030, 4352, 256, (16, 16)),     # 64-row blocks with a ragged last row tile
])
def test_lora_edge_shapes_on_many_rows(oracle, m, k, n, ranks):
    _lora_case(oracle, m, k, n, ranks, tuple(1.0 - 0.25 * i for i in range(len(ranks))), seed=k + n + m,
               sigma_ab=0.05)


def test_lora_on_few_rows_through_the_matrix_core_kernel(oracle, matrix_core_kernel_from_33_rows):
    _lora_case(oracle, 40, 2560, 2560, (16, 32), (0.5, 1.0), seed=77, sigma_ab=0.05)


def test_lora_leaves_the_workspace_clean(oracle):
    """The projection's K slices meet through the workspace counters; a plain GEMM on the same
    workspace afterwards (K split, so it counts arrivals too) and a repeat of the LoRA call must
    both be right."""
    m, k, n, g = 96, 9216, 512, 128
    x, q, s_bits = oracle.gen_problem(m, k, n, g, seed=41)
    b, s = pack.repack_gptq(q, s_bits, None, g)
    bt, st = upload_packed(b, s)
    a = bf16_tensor(oracle.gen_normal_bf16(16, k, 0.05, seed=42))
    bb = bf16_tensor(oracle.gen_normal_bf16(n, 16, 0.05, seed=43))
    xt = bf16_tensor(x)
    base_ref = oracle.c_w4a16_cpu_path(x, q, s_bits, g)
    y1 = marlin_gemm.marlin_w4a16_gemm_lora(xt, bt, st, g, a, bb, [16], [1.0])
    base = marlin_gemm.marlin_w4a16_gemm(xt, bt, st, g)
    y2 = marlin_gemm.marlin_w4a16_gemm_lora(xt, bt, st, g, a, bb, [16], [1.0])
    torch.cuda.synchronize()
    err, _, _ = row_errors(bf16_bits(base), base_ref, oracle)
    assert err.max() <= 1e-2
    assert torch.equal(y1, y2)


def test_lora_delta_is_visible_and_linear(oracle):
    """With large adapters the delta dominates: checks that it is really applied, per adapter scale."""
    m, k, n, g = 40, 256, 512, 128
    x, q, s_bits = oracle.gen_problem(m, k, n, g, seed=5)
    b, s = pack.repack_gptq(q, s_bits, None, g)
    bt, st = upload_packed(b, s)
    a = oracle.gen_normal_bf16(16, k, 0.5, seed=6)
    bb = oracle.gen_normal_bf16(n, 16, 0.5, seed=7)
    xt, at, bbt = bf16_tensor(x), bf16_tensor(a), bf16_tensor(bb)
    base = marlin_gemm.marlin_w4a16_gemm(xt, bt, st, g).float()
    y1 = marlin_gemm.marlin_w4a16_gemm_lora(xt, bt, st, g, at, bbt, [16], [1.0]).float()
    y2 = marlin_gemm.marlin_w4a16_gemm_lora(xt, bt, st, g, at, bbt, [16], [2.0]).float()
    d1, d2 = y1 - base, y2 - base
    assert d1.abs().max() > 10 * base.abs().max()
    assert torch.allclose(d2, 2 * d1, rtol=2e-2, atol=2e-2 * d1.abs().max().item())


def test_known_values_through_the_kernel(oracle):
    """lora_loader.rs:369-401 scaled up to kernel-legal shapes: zero base weight (all codes 8),
    A picks x[0], x[1]; B rows (1,0), (0,1), (.5,.5) -> y = x0, x1, (x0+x1)/2."""
    k, n, g = 128, 256, 128
    q = oracle.np_pack_gptq(np.full((k, n), 8, np.int32))
    s_bits = np.full((1, n), 0x3C00, np.uint16)
    b, s = pack.repack_gptq(q, s_bits, None, g)
    bt, st = upload_packed(b, s)
    x = np.zeros((2, k), np.float32); x[0, :4] = [1, 2, 3, 4]; x[1, :4] = [-2, 6, 0, 1]
    a = np.zeros((2, k), np.float32); a[0, 0] = 1; a[1, 1] = 1
    bm = np.zeros((n, 2), np.float32); bm[0] = [1, 0]; bm[1] = [0, 1]; bm[2] = [.5, .5]
    y = marlin_gemm.marlin_w4a16_gemm_lora(bf16_tensor(oracle.np_f32_to_bf16(x)), bt, st, g,
                                           bf16_tensor(oracle.np_f32_to_bf16(a)),
                                           bf16_tensor(oracle.np_f32_to_bf16(bm)), [2], [1.0]).float().cpu()
    assert torch.equal(y[:, :3], torch.tensor([[1.0, 2.0, 1.5], [-2.0, 6.0, 2.0]]))
    assert torch.all(y[:, 3:] == 0)


def test_proj_forward_and_merge_concat(oracle):
    """forward.rs:2923-2946 through the host mirror; merge_concat identity adapter_merge.rs:1444."""
    k, n = 256, 512
    w = oracle.c_lcg_fill(k * n, 11, 0.5).reshape(k, n)
    proj = marlin_proj.pack_from_bf16(bf16_tensor(oracle.np_f32_to_bf16(w)), 128)
    x = bf16_tensor(oracle.gen_normal_bf16(6, k, 1.0, seed=1)).reshape(2, 3, k)
    p1 = klora.LoraProjectionWeights(torch.randn(8, k, device="cuda") * 0.1, torch.randn(n, 8, device="cuda") * 0.1)
    p2 = klora.LoraProjectionWeights(torch.randn(16, k, device="cuda") * 0.1, torch.randn(n, 16, device="cuda") * 0.1)
    base = klora.proj_forward(x, proj, None)
    assert tuple(base.shape) == (2, 3, n)
    # two adapters with scales == one merged adapter (weights folded into B) with scale 1
    stacked = klora.stack_adapters([p1, p2], [0.7, 0.3])
    merged = klora.merge_concat([p1, p2], [0.7, 0.3])
    y_stacked = klora.proj_forward(x, proj, stacked).float()
    y_merged = klora.proj_forward(x, proj, merged, 1.0).float()
    ref = base.float() + 0.7 * (x.float() @ p1.a.bfloat16().float().T) @ p1.b.bfloat16().float().T \
        + 0.3 * (x.float() @ p2.a.bfloat16().float().T) @ p2.b.bfloat16().float().T
    tol = 2e-2 * ref.abs().amax(dim=-1, keepdim=True)
    assert torch.all((y_stacked - ref).abs() <= tol)
    assert torch.all((y_merged - ref).abs() <= tol)
    ba = merged.b.double() @ merged.a.double()
    want = 0.7 * p1.b.double() @ p1.a.double() + 0.3 * p2.b.double() @ p2.a.double()
    assert torch.allclose(ba, want, atol=1e-5)


@pytest.mark.parametrize("tiles,waves,ks", [(2, 12, 3), (1, 12, 6), (1, 12, 2), (3, 12, 4)])
@pytest.mark.parametrize("m", [16, 5])
def test_lora_with_the_k_slices_meeting_through_counters(oracle, tiles, waves, ks, m):
    """Forced plans of the small-M kernel on the down projection with the counter-free exchange switched off (and six
    slices, which are beyond it anyway): whichever slice arrives last finishes a tile, so the low-rank term travels in
    the last slice's part.  20 calls each: the slices of a tile run side by side and arrive in any order."""
    from kiln_amd import _lib
    L = _lib.load_tuning()
    L.kiln_w4a16_debug_gmp(tiles, waves, ks)
    L.kiln_w4a16_debug_flagged(0)
    k, n, g = 9216, 2560, 128
    x, q, s_bits = oracle.gen_problem(m, k, n, g, seed=31 * m + ks)
    b, s = pack.repack_gptq(q, s_bits, None, g)
    ranks, scales = (16, 32), (0.5, 1.0)
    a_list = [oracle.gen_normal_bf16(r, k, 0.05, seed=40 + i) for i, r in enumerate(ranks)]
    b_list = [oracle.gen_normal_bf16(n, r, 0.05, seed=50 + i) for i, r in enumerate(ranks)]
    y_ref = oracle.c_w4a16_cpu_path(x, q, s_bits, g)
    for a_i, b_i, sc in zip(a_list, b_list, scales):
        oracle.c_lora_delta_add(y_ref, x, a_i, b_i, sc)
    bt, st = upload_packed(b, s)
    a_cat, b_cat = bf16_tensor(np.concatenate(a_list, axis=0)), bf16_tensor(np.concatenate(b_list, axis=1))
    first = None
    for _ in range(20):
        y = marlin_gemm.marlin_w4a16_gemm_lora(bf16_tensor(x), bt, st, g, a_cat, b_cat, ranks, scales)
        torch.cuda.synchronize()
        first = y if first is None else first
        assert torch.equal(y, first), "the result depends on the order in which the slices arrive"
    err, _, _ = row_errors(bf16_bits(first), y_ref, oracle)
    assert err.max() <= 1e-2, f"worst row error {err.max():.3e}"


def test_lora_on_an_output_too_wide_for_the_counter_free_exchange(oracle):
    """21760 columns in three K slices are more partial tiles than the zeroed region holds: the automatic plan meets
    through counters, in a launch of several rounds of blocks (a random sweep found NaNs here)."""
    for _ in range(3):
        _lora_case(oracle, 14, 9216, 21760, (32, 32), (1.0, 1.0), seed=63, sigma_ab=0.03)


def test_host_mirror_pads_odd_stacked_ranks():
    """Ranks 4 and 5 through `proj_forward` and `swiglu_forward`: the mirror pads the stacked rank to a multiple of 8
    (zero rows of A, zero columns of B), and the result equals the unpadded call through the library's general route."""
    k, n = 2560, 512
    b = torch.randint(-2**31, 2**31 - 1, (k // 16, 2 * n), dtype=torch.int32, device="cuda")
    s = (torch.rand(k // 128, n, device="cuda") * 0.018 + 0.002).half()
    proj = marlin_proj.MarlinPackedProj(b, s, 128, k, n)
    p1 = klora.LoraProjectionWeights((torch.randn(4, k, device="cuda") * 0.05).bfloat16(), (torch.randn(n, 4, device="cuda") * 0.05).bfloat16())
    p2 = klora.LoraProjectionWeights((torch.randn(5, k, device="cuda") * 0.05).bfloat16(), (torch.randn(n, 5, device="cuda") * 0.05).bfloat16())
    stacked = klora.stack_adapters([p1, p2], [0.5, 2.0])
    assert klora.pad_rank(stacked).ranks == (4, 12)
    for m in (3, 16, 40, 200):
        x = torch.randn(m, k, device="cuda").bfloat16()
        unpadded = marlin_gemm.marlin_w4a16_gemm_lora(x, b, s, 128, stacked.a_cat, stacked.b_cat, stacked.ranks, stacked.scales)
        y = klora.proj_forward(x, proj, stacked)
        ref = x.float() @ marlin_gemm.dequant_f32(b, s, 128)
        for p, sc in ((p1, 0.5), (p2, 2.0)):
            ref = ref + (sc * (x.float() @ p.a.float().T)).bfloat16().float() @ p.b.float().T
        tol = 2e-2 * ref.abs().max()
        assert (y.float() - ref).abs().max() <= tol and (unpadded.float() - ref).abs().max() <= tol
    # the fused gate/up call: 256 gate + 256 up columns, rank 4 on the gate side and 5 on the up side
    half = n // 2
    g = klora.LoraProjectionWeights(p1.a, p1.b[:half].contiguous())
    u = klora.LoraProjectionWeights(p2.a, p2.b[:half].contiguous())
    x = torch.randn(16, k, device="cuda").bfloat16()
    h = klora.swiglu_forward(x, proj, g, u, 1.0)
    z = x.float() @ marlin_gemm.dequant_f32(b, s, 128)
    v = z.view(16, n // 16, 2, 8)
    gate = v[:, :, 0].reshape(16, half) + (x.float() @ g.a.float().T).bfloat16().float() @ g.b.float().T
    up = v[:, :, 1].reshape(16, half) + (x.float() @ u.a.float().T).bfloat16().float() @ u.b.float().T
    want = torch.nn.functional.silu(gate) * up
    assert (h.float() - want).abs().max() <= 2e-2 * want.abs().max()


def test_lora_argument_errors():
    dev = "cuda"
    a = torch.zeros(2, 128, dtype=torch.bfloat16, device=dev)
    b = torch.zeros(8, 512, dtype=torch.int32, device=dev)
    s = torch.ones(1, 256, dtype=torch.float16, device=dev)
    la = torch.zeros(8, 128, dtype=torch.bfloat16, device=dev)
    lb = torch.zeros(256, 8, dtype=torch.bfloat16, device=dev)
    E = marlin_gemm.MarlinGemmError
    with pytest.raises(E, match="LoRA shapes"):
        marlin_gemm.marlin_w4a16_gemm_lora(a, b, s, 128, la, lb, [4], [1.0])
    with pytest.raises(E, match="bf16"):
        marlin_gemm.marlin_w4a16_gemm_lora(a, b, s, 128, la.float(), lb, [8], [1.0])
    big_a = torch.zeros(72, 128, dtype=torch.bfloat16, device=dev)
    big_b = torch.zeros(256, 72, dtype=torch.bfloat16, device=dev)
    with pytest.raises(E, match="status 2"):
        marlin_gemm.marlin_w4a16_gemm_lora(a, b, s, 128, big_a, big_b, [72], [1.0])   # rank > 64
    y = marlin_gemm.marlin_w4a16_gemm_lora(a, b, s, 128, la, lb, [8], [1.0])
    assert tuple(y.shape) == (2, 256)


@pytest.mark.parametrize("m,k,n", [
    (512, 2560, 18432),    # 64-row blocks on a work-bound launch: the row sums come from a pre-pass
    (333, 2560, 18432),    # ... with a ragged last row tile
    (1100, 9216, 8192),    # 128-row blocks; the projection takes 64 rows per block
    (1030, 2560, 8192),    # 128-row blocks, 16 rows per projection block
])
def test_adapters_with_zero_b_equal_the_plain_call_bit_for_bit(m, k, n):
    """With adapters the projection's launch also writes the matrix-core kernel's row-sum operand (a
    launch of its own without them).  B = 0 makes the low-rank term vanish, so the two calls must
    agree in every bit: same operand, same order of additions."""
    gen = torch.Generator(device="cuda").manual_seed(m + k + n)
    bt = torch.randint(-2**31, 2**31 - 1, (k // 16, 2 * n), dtype=torch.int32, device="cuda", generator=gen)
    st = (torch.rand(k // 128, n, device="cuda", generator=gen) * 0.018 + 0.002).to(torch.float16)
    x = (torch.randn(m, k, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
    ranks, scales = (16, 32), (0.5, 1.0)
    a_cat = (torch.randn(sum(ranks), k, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
    b_cat = torch.zeros(n, sum(ranks), dtype=torch.bfloat16, device="cuda")
    plain = marlin_gemm.marlin_w4a16_gemm(x, bt, st, 128)
    with_adapters = marlin_gemm.marlin_w4a16_gemm_lora(x, bt, st, 128, a_cat, b_cat, ranks, scales)
    torch.cuda.synchronize()
    assert torch.equal(plain.view(torch.int16), with_adapters.view(torch.int16))


@pytest.mark.parametrize("m,k,n", [
    (512, 2560, 18432),    # the benchmark's LoRA configuration: 64-row blocks, 32 row tiles x 7 K slices of the projection
    (333, 2560, 18432),    # ragged last row tile
    (1030, 2560, 8192),    # 128-row blocks
    (512, 9216, 2560),     # blocks that sum their rows themselves: the producers write T only
    (300, 2560, 8192),     # likewise, ragged
    (64, 4096, 2560),      # the mid-M kernel: producers of 256 working threads in blocks of 512, T in K slices
    (33, 2560, 18432),     # ... three tile pairs per block, a ragged run
    (100, 2560, 8192),     # ... two runs of 64 rows
    (48, 9216, 2560),      # ... K slices of the product and of the projection
    (17, 4096, 2560),      # ... which calls with adapters take from 17 rows on
    (24, 2560, 18432),
    (128, 2560, 18432),    # ... a launch of more blocks than the chip holds at once: the producers still come first
    (192, 2560, 8192),     # ... three runs of 64 rows
    (96, 9216, 2560),
])
def test_projection_inside_the_matrix_core_launch(m, k, n):
    """Beyond 16 rows the projection (on the matrix-core path also the row sums, where they come from a
    pre-pass) is computed by extra blocks of the product's own launch where the block shape allows it; they
    raise a word per row tile in the zeroed workspace prefix.  Folded and in front must agree in every
    bit; the prefix must be clean after every call; launches with alternating activations in a row
    must each see their own T."""
    from kiln_amd import _lib
    L = _lib.load_tuning()
    gen = torch.Generator(device="cuda").manual_seed(7 * m + k + n)
    bt = torch.randint(-2**31, 2**31 - 1, (k // 16, 2 * n), dtype=torch.int32, device="cuda", generator=gen)
    st = (torch.rand(k // 128, n, device="cuda", generator=gen) * 0.018 + 0.002).to(torch.float16)
    xs = [(torch.randn(m, k, device="cuda", generator=gen) * 0.5).to(torch.bfloat16) for _ in range(2)]
    ranks, scales = (16, 32), (0.5, 1.0)
    a_cat = (torch.randn(sum(ranks), k, device="cuda", generator=gen) * 0.05).to(torch.bfloat16)
    b_cat = (torch.randn(n, sum(ranks), device="cuda", generator=gen) * 0.05).to(torch.bfloat16)
    z = L.kiln_w4a16_workspace_zeroed_bytes()
    ws = torch.empty(L.kiln_w4a16_workspace_bytes(m, n, k), dtype=torch.uint8, device="cuda")
    ws[z:].fill_(0xA5)
    ws[:z].zero_()
    import ctypes
    ranks_c = (ctypes.c_int * 2)(*ranks)
    scales_c = (ctypes.c_float * 2)(*scales)

    def call(x):
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = L.kiln_w4a16_gemm_lora(x.data_ptr(), bt.data_ptr(), out.data_ptr(), st.data_ptr(), m, n, k, ws.data_ptr(), 128,
                                    torch.cuda.current_device(), torch.cuda.current_stream().cuda_stream,
                                    a_cat.data_ptr(), b_cat.data_ptr(), sum(ranks), len(ranks), ranks_c, scales_c)
        assert rc == _lib.OK, _lib.status_string(rc)
        torch.cuda.synchronize()
        assert int(ws[:z].count_nonzero()) == 0, "the call left words in the zeroed prefix"
        return out

    try:
        L.kiln_w4a16_debug_lora_fold(0)
        in_front = [call(x) for x in xs]
        L.kiln_w4a16_debug_lora_fold(-1)
        for i in range(40):
            assert torch.equal(call(xs[i % 2]).view(torch.int16), in_front[i % 2].view(torch.int16)), i
    finally:
        L.kiln_w4a16_debug_lora_fold(-1)


@pytest.mark.parametrize("m,k,n,ranks", [(200, 9216, 256, (7,)), (16, 9216, 2560, (16, 32))])
def test_lora_run_to_run_determinism(oracle, m, k, n, ranks):
    """The projection's K slices meet as f32 tiles in the workspace (many rows) and the GEMM's own
    K slices exchange partial tiles (few rows): 1000 launches, identical bits, stopping at the
    first difference."""
    g = 128
    x, q, s_bits = oracle.gen_problem(m, k, n, g, seed=m)
    b, s = pack.repack_gptq(q, s_bits, None, g)
    bt, st = upload_packed(b, s)
    a_cat = bf16_tensor(np.concatenate([oracle.gen_normal_bf16(r, k, 0.05, seed=40 + i) for i, r in enumerate(ranks)], axis=0))
    b_cat = bf16_tensor(np.concatenate([oracle.gen_normal_bf16(n, r, 0.05, seed=50 + i) for i, r in enumerate(ranks)], axis=1))
    scales = tuple(1.0 for _ in ranks)
    xt = bf16_tensor(x)
    first = marlin_gemm.marlin_w4a16_gemm_lora(xt, bt, st, g, a_cat, b_cat, ranks, scales).clone()
    out = torch.empty_like(first)
    same = torch.ones((), dtype=torch.bool, device=first.device)
    for i in range(1000):
        marlin_gemm.marlin_w4a16_gemm_lora(xt, bt, st, g, a_cat, b_cat, ranks, scales, out=out)
        same &= (out == first).all()
        if i % 50 == 49:
            assert bool(same), f"launch {i - 49}...{i} differed from the first"
