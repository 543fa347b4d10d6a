"""GPU tests of the exchange between K slices, through the C ABI: the counter-free exchange (parts
stored as the complement of their bits into a workspace region that is all zero between launches,
the last slice polling them) against the exchange through arrival counters -- same sums in the
same order, so bit-equal outputs -- and the state both leave behind: the zeroed prefix of the
workspace must be all zero again after every call, whatever the inputs."""
import numpy as np
import pytest
import torch

from kiln_amd import _lib
from kiln_amd.marlin_gemm import pack
from tests.gpu_util import bf16_bits, bf16_tensor, row_errors, upload_packed

pytestmark = pytest.mark.gpu


def _call(L, xt, bt, st, m, k, n, ws=None):
    dev = torch.cuda.current_device()
    stream = torch.cuda.current_stream().cuda_stream
    z = L.kiln_w4a16_workspace_zeroed_bytes()
    if ws is None:
        ws = torch.empty(L.kiln_w4a16_workspace_bytes(m, n, k), dtype=torch.uint8, device="cuda")
        ws[z:].fill_(0xA5)                                   # nothing behind the prefix needs to be zero
        ws[:z].zero_()
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    rc = L.kiln_marlin_w4a16_gemm(xt.data_ptr(), bt.data_ptr(), out.data_ptr(), st.data_ptr(), m, n, k,
                                  ws.data_ptr(), 128, dev, stream, -1, -1, -1, 16)
    assert rc == _lib.OK, _lib.status_string(rc)
    torch.cuda.synchronize()
    assert int(ws[:z].count_nonzero()) == 0, "the call left words in the zeroed prefix"
    return out, ws


SMALL = [(2, 12, 3), (3, 12, 4), (2, 12, 2), (1, 12, 3), (4, 12, 4), (1, 12, 6)]   # (tiles, wavefronts, K slices)


@pytest.mark.parametrize("tiles,waves,ks", SMALL)
@pytest.mark.parametrize("m", [16, 7, 1])
def test_small_m_counter_free_exchange_equals_the_counted_one(oracle, tiles, waves, ks, m):
    """Forced plans of the private-staging kernel on the down projection; six slices are beyond the
    counter-free exchange and run through counters either way."""
    L = _lib.load_tuning()
    k, n = 9216, 2560
    x, q, s_bits = oracle.gen_problem(m, k, n, 128, seed=100 + tiles + ks)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    bt, st = upload_packed(b, s)
    xt = bf16_tensor(x)
    L.kiln_w4a16_debug_gmp(tiles, waves, ks)
    L.kiln_w4a16_debug_flagged(0)
    counted, _ = _call(L, xt, bt, st, m, k, n)
    L.kiln_w4a16_debug_flagged(-1)
    free, ws = _call(L, xt, bt, st, m, k, n)
    again, _ = _call(L, xt, bt, st, m, k, n, ws)             # the same workspace, not zeroed in between
    assert torch.equal(counted, free) and torch.equal(free, again)
    err, _, _ = row_errors(bf16_bits(free), oracle.c_w4a16_cpu_path(x, q, s_bits, 128), oracle)
    assert err.max() <= 1e-2


@pytest.mark.parametrize("m,k,n,pairs,ks", [
    (64, 4096, 2560, 1, 2), (64, 9216, 2560, 1, 3), (128, 4096, 2560, 2, 2), (40, 9216, 2560, 2, 3),
    (64, 2560, 8192, 2, 2), (96, 2560, 8192, 3, 2), (64, 4096, 2560, 1, 4), (192, 9216, 2560, 1, 3),
])
def test_mid_m_counter_free_exchange_equals_the_counted_one(oracle, m, k, n, pairs, ks):
    """Forced plans of the mid-M kernel, one to three tile pairs per block, one to three runs of 64
    rows (the last case needs more than the zeroed region holds and runs through counters)."""
    L = _lib.load_tuning()
    x, q, s_bits = oracle.gen_problem(m, k, n, 128, seed=200 + pairs + ks)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    bt, st = upload_packed(b, s)
    xt = bf16_tensor(x)
    L.kiln_w4a16_debug_mid(1, pairs, ks)
    L.kiln_w4a16_debug_flagged(0)
    counted, _ = _call(L, xt, bt, st, m, k, n)
    L.kiln_w4a16_debug_flagged(-1)
    free, ws = _call(L, xt, bt, st, m, k, n)
    again, _ = _call(L, xt, bt, st, m, k, n, ws)
    assert torch.equal(counted, free) and torch.equal(free, again)
    err, _, _ = row_errors(bf16_bits(free), oracle.c_w4a16_cpu_path(x, q, s_bits, 128), oracle)
    assert err.max() <= 1e-2


def test_counter_free_exchange_with_nan_inf_and_zero_rows(oracle):
    """The parts are their own arrival flags, so every bit pattern a sum can take must read as
    'arrived': zeros (+0 and -0), infinities and the NaNs that arithmetic produces.  Rows of such
    inputs come out non-finite where the oracle's are, the other rows are untouched by them,
    the launch ends, and the zeroed prefix is zero again."""
    L = _lib.load()                                          # the shipped library's automatic plan
    m, k, n = 16, 9216, 2560
    x, q, s_bits = oracle.gen_problem(m, k, n, 128, seed=7)
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    bt, st = upload_packed(b, s)
    x = x.copy()
    x[1, :] = 0x0000                                         # +0 row
    x[2, :] = 0x8000                                         # -0 row
    x[3, 5] = 0x7F80                                         # +inf
    x[4, 9000] = 0xFF80                                      # -inf (last slice)
    x[5, 4000] = 0x7FC0                                      # quiet NaN (middle slice)
    x[6, 10] = 0xFFFF                                        # NaN with every payload bit a bf16 can carry
    x[7, 3] = 0x7F80
    x[7, 9100] = 0xFF80                                      # inf - inf across slices: NaN formed by the adding wavefront
    xt = bf16_tensor(x)
    out, ws = _call(L, xt, bt, st, m, k, n)
    y = oracle.np_bf16_to_f32(bf16_bits(out))
    y_ref = oracle.c_w4a16_cpu_path(x, q, s_bits, 128)
    assert np.all(y[1] == 0) and np.all(y[2] == 0)
    for r in (5, 6):                                         # a NaN activation: the whole row is NaN, as the oracle's
        assert np.all(np.isnan(y[r])) and np.all(np.isnan(y_ref[r])), r
    for r in (3, 4, 7):
        # an infinite activation: no finite value in the row on either side (the oracle has +-inf where the
        # weight is not zero; here the offset removal turns the row into inf - inf = NaN)
        assert not np.any(np.isfinite(y[r])) and not np.any(np.isfinite(y_ref[r])), r
    rest = [0] + list(range(8, 16))
    err, _, _ = row_errors(bf16_bits(out)[rest], y_ref[rest], oracle)
    assert err.max() <= 1e-2
    # the next call on the same workspace is unaffected
    x2, _, _ = oracle.gen_problem(m, k, n, 128, seed=8)
    out2, _ = _call(L, bf16_tensor(x2), bt, st, m, k, n, ws)
    err, _, _ = row_errors(bf16_bits(out2), oracle.c_w4a16_cpu_path(x2, q, s_bits, 128), oracle)
    assert err.max() <= 1e-2


def _lora_call(L, xt, bt, st, la, lb, ranks, scales, m, k, n, ws=None):
    import ctypes
    dev = torch.cuda.current_device()
    stream = torch.cuda.current_stream().cuda_stream
    z = L.kiln_w4a16_workspace_zeroed_bytes()
    if ws is None:
        ws = torch.empty(L.kiln_w4a16_workspace_bytes(m, n, k), dtype=torch.uint8, device="cuda")
        ws[z:].fill_(0xA5)
        ws[:z].zero_()
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    c_ranks = (ctypes.c_int * len(ranks))(*ranks)
    c_scales = (ctypes.c_float * len(ranks))(*scales)
    rc = L.kiln_w4a16_gemm_lora(xt.data_ptr(), bt.data_ptr(), out.data_ptr(), st.data_ptr(), m, n, k, ws.data_ptr(),
                                128, dev, stream, la.data_ptr(), lb.data_ptr(), sum(ranks), len(ranks), c_ranks, c_scales)
    assert rc == _lib.OK, _lib.status_string(rc)
    torch.cuda.synchronize()
    assert int(ws[:z].count_nonzero()) == 0, "the call left words in the zeroed prefix"
    return out, ws


@pytest.mark.parametrize("m,k,n,ranks", [
    (16, 2560, 18432, (16, 32)),        # the benchmark's adapters on gate+up
    (4, 9216, 2560, (16, 32)),          # unsliced down projection, 15 producers
    (16, 9216, 2560, (8,)),             # three K slices: the last one adds the term
    (9, 4096, 2560, (64,)),             # the largest rank
    (16, 2560, 2560, (8, 8, 8, 8)),     # four adapters
    (16, 2560, 2560, (8, 8, 8, 8, 8)),  # five: the projection runs as a launch of its own
    (16, 2560, 8192, (16, 32)),         # planned with wider blocks than the plain call's 256, which leave no unit for producers
    (16, 2560, 8192, (8, 8, 8, 8, 8)),  # five adapters on that shape: planned for a fold that then cannot happen
    (1, 256, 256, (8,)),                # two groups of K, one producer
])
def test_lora_projection_inside_the_gemm_launch(oracle, m, k, n, ranks):
    """Up to 16 rows: the projection onto the adapters is computed by extra blocks of the GEMM launch,
    which raise flags in the zeroed workspace prefix; the adding blocks' extra wavefront waits for
    them, fetches T and the rows of B into LDS, and the last block zeroes the flags.  Against the
    oracle with the projection folded and as a launch of its own, the prefix clean after every call,
    a repeat on the same workspace bit-identical, and 300 launches in a row identical."""
    L = _lib.load_tuning()
    scales = tuple(0.5 + 0.25 * i for i in range(len(ranks)))
    x, q, s_bits = oracle.gen_problem(m, k, n, 128, seed=300 + m + len(ranks))
    b, s = pack.repack_gptq(q, s_bits, None, 128)
    bt, st = upload_packed(b, s)
    a_list = [oracle.gen_normal_bf16(r, k, 0.05, seed=60 + i) for i, r in enumerate(ranks)]
    b_list = [oracle.gen_normal_bf16(n, r, 0.05, seed=70 + i) for i, r in enumerate(ranks)]
    y_ref = oracle.c_w4a16_cpu_path(x, q, s_bits, 128)
    for a_i, b_i, sc in zip(a_list, b_list, scales):
        oracle.c_lora_delta_add(y_ref, x, a_i, b_i, sc)
    la, lb = bf16_tensor(np.concatenate(a_list, axis=0)), bf16_tensor(np.concatenate(b_list, axis=1))
    xt = bf16_tensor(x)
    outs = {}
    for fold in (-1, 0):
        L.kiln_w4a16_debug_lora_fold(fold)
        out, ws = _lora_call(L, xt, bt, st, la, lb, ranks, scales, m, k, n)
        again, _ = _lora_call(L, xt, bt, st, la, lb, ranks, scales, m, k, n, ws)
        assert torch.equal(out, again)
        err, _, _ = row_errors(bf16_bits(out), y_ref, oracle)
        assert err.max() <= 1e-2, (fold, err.max())
        outs[fold] = out
    L.kiln_w4a16_debug_lora_fold(-1)
    same = torch.ones((), dtype=torch.bool, device="cuda")
    out = torch.empty_like(outs[-1])
    from kiln_amd import marlin_gemm
    first = marlin_gemm.marlin_w4a16_gemm_lora(xt, bt, st, 128, la, lb, ranks, scales).clone()
    for _ in range(300):
        marlin_gemm.marlin_w4a16_gemm_lora(xt, bt, st, 128, la, lb, ranks, scales, out=out)
        same &= (out == first).all()
    assert bool(same) and torch.equal(first, outs[-1])
    # launches with changing activations in a row: every T must be this launch's, never an earlier one's
    # left in some cache (two inputs alternate, each result against the oracle's for its own input)
    x2, _, _ = oracle.gen_problem(m, k, n, 128, seed=900 + m)
    y2_ref = oracle.c_w4a16_cpu_path(x2, q, s_bits, 128)
    for a_i, b_i, sc in zip(a_list, b_list, scales):
        oracle.c_lora_delta_add(y2_ref, x2, a_i, b_i, sc)
    xt2 = bf16_tensor(x2)
    results = []
    for i in range(40):
        results.append(marlin_gemm.marlin_w4a16_gemm_lora(xt2 if i % 2 else xt, bt, st, 128, la, lb, ranks, scales))
    torch.cuda.synchronize()
    for i, y in enumerate(results):
        assert torch.equal(y, results[i % 2]), i
    err, _, _ = row_errors(bf16_bits(results[1]), y2_ref, oracle)
    assert err.max() <= 1e-2 and torch.equal(results[0], first)
