"""Quantise-and-pack on the device (`kiln_w4a16_quantize_and_pack_device`) against the host quantiser
(`kiln_w4a16_quantize_and_pack`, the restatement of crates/kiln-marlin-gemm/src/lib.rs:393-427 that
tests/test_host_pack.py pins to the oracle): packed words and scales must be the same bits."""
import numpy as np
import pytest
import torch

from kiln_amd import marlin_gemm, marlin_proj
from kiln_amd.marlin_gemm import pack
from tests.gpu_util import bf16_tensor

pytestmark = pytest.mark.gpu


def _bf16_as_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def _check(bits: np.ndarray, groupsize: int):
    k, n = bits.shape
    b_dev, s_dev = pack.quantize_and_pack_device(bf16_tensor(bits), groupsize)
    torch.cuda.synchronize()
    b_host, s_host, _ = pack.quantize_and_pack(_bf16_as_f32(bits), k, n, groupsize, want_dequant=False)
    assert np.array_equal(s_dev.cpu().numpy().view(np.uint16), np.asarray(s_host).view(np.uint16)), "scales differ"
    assert np.array_equal(b_dev.cpu().numpy(), b_host), "packed words differ"


@pytest.mark.parametrize("k,n,groupsize", [(128, 256, 128), (256, 256, -1), (2560, 2560, 128), (2560, 1024, -1),
                                           (9216, 2560, 128), (2560, 9216, 128)])
def test_device_pack_equals_host_pack(oracle, k, n, groupsize):
    _check(oracle.gen_normal_bf16(k, n, 0.02, seed=k + n), groupsize)


def test_device_pack_edge_values(oracle):
    """Rounding ties, the +8 clamp, all-zero groups, subnormal and huge magnitudes, infinities and NaN."""
    k, n = 256, 256
    bits = oracle.gen_normal_bf16(k, n, 1.0, seed=5).copy()
    f32 = lambda v: np.asarray(oracle.np_f32_to_bf16(np.asarray(v, np.float32)))   # noqa: E731
    bits[:128, 0] = 0                                     # an all-zero group: scale 1.0, code 8
    bits[:128, 1] = f32(np.where(np.arange(128) % 2, 7.5, -7.5))      # w / s = +-7.5 * 15 / 15: ties at the ends
    bits[:128, 2] = f32(np.linspace(-15.0, 15.0, 128))               # multiples of the step and halves between
    bits[:128, 3] = f32(np.full(128, 1e-30))                          # scale underflows to an f16 subnormal or zero
    bits[:128, 4] = f32(np.full(128, 3e38))                           # scale overflows to f16 infinity
    bits[:128, 5] = f32(np.where(np.arange(128) == 7, np.inf, 1.0))   # an infinity among ordinary values
    bits[:128, 6] = f32(np.where(np.arange(128) == 9, np.nan, 1.0))   # a NaN: never the maximum, code 8
    bits[:128, 7] = f32(np.where(np.arange(128) % 3 == 0, -0.0, 6e-5))   # negative zeros, values near f16's smallest normal
    bits[128:, 8] = f32(np.arange(128) * 0.5 - 32.0)                  # exact halves of the step
    for groupsize in (128, -1):
        _check(bits, groupsize)


def test_projection_layer_packs_on_the_device_with_the_host_routes_bits(oracle, monkeypatch):
    """`pack_from_bf16` of the projection layer: the default (device) route and the host route of
    marlin_proj.rs:86-181 (KILN_W4A16_HOST_PACK=1) give the same packed projection."""
    k, n = 2560, 1024
    w = bf16_tensor(oracle.gen_normal_bf16(k, n, 0.02, seed=3))
    monkeypatch.delenv("KILN_W4A16_HOST_PACK", raising=False)
    on_device = marlin_proj.pack_from_bf16(w, 128)
    monkeypatch.setenv("KILN_W4A16_HOST_PACK", "1")
    on_host = marlin_proj.pack_from_bf16(w, 128)
    assert torch.equal(on_device.b_packed, on_host.b_packed) and torch.equal(on_device.scales, on_host.scales)
    x = bf16_tensor(oracle.gen_normal_bf16(4, k, 1.0, seed=4))
    assert torch.equal(marlin_proj.matmul_bf16(x, on_device), marlin_proj.matmul_bf16(x, on_host))


@pytest.mark.parametrize("k,n_each,groupsize", [(256, 256, 128), (2560, 9216, 128), (512, 1280, -1)])
def test_device_interleave_equals_host_interleave(oracle, k, n_each, groupsize):
    """`kiln_w4a16_interleave_gate_up_device` against the host routine (which tests/test_host_pack.py
    checks column by column): same words, same scales."""
    sides = []
    for seed in (1, 2):
        codes = oracle.gen_codes(k, n_each, seed)
        s_bits = oracle.gen_scales_f16(k, n_each, groupsize, seed)
        sides.append(pack.repack_gptq(oracle.np_pack_gptq(codes), s_bits, None, groupsize))
    b_host, s_host = pack.interleave_gate_up(sides[0][0], sides[0][1], sides[1][0], sides[1][1], groupsize)
    dev = [(torch.from_numpy(np.asarray(b)).cuda(), torch.from_numpy(np.asarray(s).view(np.float16)).cuda()) for b, s in sides]
    b_dev, s_dev = pack.interleave_gate_up_device(dev[0][0], dev[0][1], dev[1][0], dev[1][1], groupsize)
    torch.cuda.synchronize()
    assert np.array_equal(b_dev.cpu().numpy(), b_host)
    assert np.array_equal(s_dev.cpu().numpy().view(np.uint16), np.asarray(s_host).view(np.uint16))


@pytest.mark.parametrize("k,n,groupsize", [(256, 256, 128), (2560, 9216, 128), (9216, 2560, 128), (512, 1280, -1)])
def test_device_gptq_repack_equals_host_repack(oracle, k, n, groupsize):
    """`kiln_w4a16_repack_gptq_device` against the host repack (pinned on the CPU by the written-layout and
    round-trip tests): same words, same scales; zero-points other than 8 are refused before anything is written."""
    q = oracle.np_pack_gptq(oracle.gen_codes(k, n, seed=k + n))
    s_bits = oracle.gen_scales_f16(k, n, groupsize, seed=k)
    b_host, s_host = pack.repack_gptq(q, s_bits, None, groupsize)
    qt = torch.from_numpy(np.asarray(q).view(np.int32)).cuda()
    st = torch.from_numpy(np.asarray(s_bits).view(np.float16)).cuda()
    g = k if groupsize == -1 else groupsize
    zeros = torch.full((k // g, n // 8), -0x77777778, dtype=torch.int32, device="cuda")     # 0x88888888
    for qz in (None, zeros):
        b_dev, s_dev = pack.repack_gptq_device(qt, st, qz, groupsize)
        torch.cuda.synchronize()
        assert np.array_equal(b_dev.cpu().numpy(), np.asarray(b_host).view(np.int32))
        assert np.array_equal(s_dev.cpu().numpy().view(np.uint16), np.asarray(s_host).view(np.uint16))
    bad = zeros.clone()
    bad[-1, -1] = 0x77777777
    with pytest.raises(marlin_gemm.MarlinGemmError, match="zero-point"):
        pack.repack_gptq_device(qt, st, bad, groupsize)
