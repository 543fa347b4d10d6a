"""Host logic and the C-ABI surface, no GPU needed: the packer against the
oracle, the tile layout against its written definition, argument checks."""
import ctypes
import re
from pathlib import Path

import numpy as np
import pytest

from kiln_amd import _lib, marlin_gemm, marlin_proj
from kiln_amd.marlin_gemm import pack

ROOT = Path(__file__).resolve().parent.parent


def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "kiln_w4a16.h").read_text()
    declared = set(re.findall(r"\b(kiln_(?:marlin_)?w4a16_\w+)\s*\(", header))
    assert declared == set(_lib.EXPORTS)
    raw = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared:
        assert hasattr(raw, name), name
    assert _lib.load().kiln_w4a16_layout_version() == 2
    assert _lib.status_string(0) == "ok" and "zero-point" in _lib.status_string(5)


def _tile_layout_reference(codes, k, n):
    """The layout as written in kiln_amd/csrc/layout.h, restated with python ints."""
    G = k // 128
    words = np.zeros(k * n // 8, dtype=np.uint32)
    for kk in range(k):
        g, kr = divmod(kk, 128)
        t, r32 = divmod(kr, 32)
        kq, j = divmod(r32, 8)
        p = j // 2 + 4 * (j & 1)
        for nn in range(n):
            nt, c = divmod(nn, 16)
            idx = (nt * G + g) * 256 + (c + 16 * kq) * 4 + t
            words[idx] |= np.uint32(int(codes[kk, nn]) << (4 * p))
    return words


def test_repack_matches_written_layout(oracle):
    k, n = 256, 256
    codes = oracle.gen_codes(k, n, seed=21)
    scales = oracle.gen_scales_f16(k, n, 128, seed=21)
    b, s = pack.repack_gptq(oracle.np_pack_gptq(codes), scales, None, 128)
    assert b.shape == (k // 16, 2 * n) and b.dtype == np.int32        # lib.rs:119
    assert s.shape == (k // 128, n) and s.dtype == np.float16         # lib.rs:144-150
    assert np.array_equal(b.view(np.uint32).ravel(), _tile_layout_reference(codes, k, n))
    # scales: [column tile][group][16]
    st = s.view(np.uint16).ravel()
    for (g, nn) in [(0, 0), (1, 17), (0, 255), (1, 128)]:
        assert st[((nn // 16) * 2 + g) * 16 + nn % 16] == scales[g, nn]


@pytest.mark.parametrize("k,n,g", [(128, 256, 128), (256, 512, -1), (2560, 256, 128)])
def test_repack_unpack_roundtrip(oracle, k, n, g):
    codes = oracle.gen_codes(k, n, seed=k + n)
    scales = oracle.gen_scales_f16(k, n, g, seed=k + n)
    q = oracle.np_pack_gptq(codes)
    b, s = pack.repack_gptq(q, scales, None, g)
    q2, s2 = pack.unpack_to_gptq(b, s, g)
    assert np.array_equal(q2.view(np.uint32), q) and np.array_equal(s2.view(np.uint16), scales)
    # words are a permutation with nibbles shuffled: code histogram is preserved
    hist = lambda w: np.bincount(np.concatenate([(w.view(np.uint32).ravel() >> (4 * i)) & 0xF
                                                 for i in range(8)]), minlength=16)
    assert np.array_equal(hist(b), hist(q))


def test_repack_zero_points(oracle):
    k, n = 128, 256
    q = oracle.np_pack_gptq(oracle.gen_codes(k, n, 1))
    sc = oracle.gen_scales_f16(k, n, 128, 1)
    z8 = oracle.np_pack_qzeros(np.full((1, n), 8))
    pack.repack_gptq(q, sc, z8, 128)                      # zero-point 8 is the supported case
    z7 = oracle.np_pack_qzeros(np.full((1, n), 7))
    with pytest.raises(marlin_gemm.MarlinGemmError, match="zero-point"):
        pack.repack_gptq(q, sc, z7, 128)


@pytest.mark.parametrize("k,n,g", [(128, 256, 128), (256, 256, -1), (512, 768, 128)])
def test_quantize_and_pack_matches_oracle(oracle, k, n, g):
    """Same LCG weights as the reference test (parity.rs:33-43,55)."""
    w = oracle.c_lcg_fill(k * n, 0xC0FFEE5EED ^ k ^ (n << 16), 0.5)
    b, s, deq = pack.quantize_and_pack(w, k, n, g)
    codes, s_bits, deq_ref = oracle.c_quantize(w.reshape(k, n), g)
    assert b.shape == (k // 16, n * 16 // 8) and deq.shape == (k, n)
    assert s.shape == ((1 if g == -1 else k // g), n)
    assert np.array_equal(deq.view(np.uint32), deq_ref.view(np.uint32))   # bit-exact
    q, s_nat = pack.unpack_to_gptq(b, s, g)
    assert np.array_equal(oracle.np_unpack_gptq(q.view(np.uint32)), codes)
    assert np.array_equal(s_nat.view(np.uint16), s_bits)
    # quantise->pack == quantise->GPTQ words->repack
    b2, s2 = pack.repack_gptq(oracle.np_pack_gptq(codes), s_bits, None, g)
    assert np.array_equal(b, b2) and np.array_equal(s.view(np.uint16), s2.view(np.uint16))


def test_quantize_and_pack_edge_rows(oracle):
    """Ties away from zero, clamp at +8 -> 15, all-zero group (lib.rs:405-407,422-423)."""
    k, n = 128, 256
    w = np.zeros((k, n), dtype=np.float32)
    w[:8, 0] = [7.5, -7.5, 0.5, -0.5, 2.5, -2.5, 0.49999997, 6.5]
    b, s, deq = pack.quantize_and_pack(w, k, n, 128)
    assert np.array_equal(deq[:8, 0], np.array([7, -8, 1, -1, 3, -3, 0, 7], np.float32))
    assert np.all(deq[:, 1:] == 0.0)
    q, s_nat = pack.unpack_to_gptq(b, s, 128)
    assert s_nat.view(np.uint16)[0, 0] == 0x3C00
    assert s_nat[0, 1] == np.float16(np.float32(2.0) / np.float32(15.0))
    assert np.all(oracle.np_unpack_gptq(q.view(np.uint32))[:, 1:] == 8)


def test_pack_argument_errors(oracle):
    w = np.zeros(128 * 256, np.float32)
    with pytest.raises(AssertionError):
        pack.quantize_and_pack(w, 100, 256, 128)          # k % 128
    with pytest.raises(AssertionError):
        pack.quantize_and_pack(w, 128, 200, 128)          # n % 256
    with pytest.raises(AssertionError):
        pack.quantize_and_pack(w[:-1], 128, 256, 128)     # length
    L = _lib.load()
    assert L.kiln_w4a16_quantize_and_pack(None, 128, 256, 128, None, None, None) == _lib.ERR_ARGUMENT
    buf = np.zeros(16, np.int32).ctypes.data
    assert L.kiln_w4a16_quantize_and_pack(buf, 128, 256, 64, buf, buf, None) == _lib.ERR_PROB_SHAPE
    assert L.kiln_w4a16_repack_gptq(buf, buf, None, 130, 256, 128, buf, buf) == _lib.ERR_PROB_SHAPE


def test_gemm_entry_status_codes_without_launch():
    """Shape checks and the m*n*k == 0 early return happen before any GPU call
    (marlin_kernel.cu:770-773)."""
    L = _lib.load()
    p = ctypes.c_void_p(0)
    call = lambda m, n, k, g=128: L.kiln_marlin_w4a16_gemm(p, p, p, p, m, n, k, p, g, 0, p, -1, -1, -1, 16)
    assert call(1, 200, 128) == _lib.ERR_PROB_SHAPE
    assert call(1, 256, 100) == _lib.ERR_PROB_SHAPE
    assert call(1, 256, 128, 64) == _lib.ERR_PROB_SHAPE
    assert call(-1, 256, 128) == _lib.ERR_PROB_SHAPE
    assert call(0, 256, 128) == _lib.OK
    assert call(4, 0, 128) == _lib.OK
    assert call(4, 256, 0) == _lib.OK
    assert call(4, 256, 128) == _lib.ERR_ARGUMENT          # null pointers
    assert L.kiln_w4a16_workspace_bytes(16, 2560, 9216) >= 64 * 1024
    assert L.kiln_w4a16_workspace_bytes(1, 18432, 2560) <= L.kiln_w4a16_workspace_bytes(2048, 18432, 2560)


def test_wrapper_validation_messages():
    """lib.rs:103-166 -- same checks, same texts (CPU tensors trip the device check first)."""
    import torch
    a = torch.zeros(1, 128, dtype=torch.bfloat16)
    b = torch.zeros(8, 512, dtype=torch.int32)
    s = torch.zeros(1, 256, dtype=torch.float16)
    with pytest.raises(marlin_gemm.MarlinGemmError, match="a must be on CUDA"):
        marlin_gemm.marlin_w4a16_gemm(a, b, s, 128)


def test_marlin_proj_host_side(monkeypatch, oracle):
    assert marlin_proj.shape_is_supported(2560, 9216) and marlin_proj.shape_is_supported(9216, 2560)
    assert not marlin_proj.shape_is_supported(2560, 32) and not marlin_proj.shape_is_supported(100, 256)
    for v, want in [("1", True), ("true", True), ("YES", True), (" 1 ", True), ("0", False), ("on", False)]:
        monkeypatch.setenv("KILN_W4A16", v)
        assert marlin_proj.env_enabled() is want
    monkeypatch.delenv("KILN_W4A16")
    assert marlin_proj.env_enabled() is False
    monkeypatch.setenv("KILN_DISABLE_PARALLEL_PACK", "True")
    assert marlin_proj.parallel_pack_disabled()
    import torch
    cpu_w = torch.zeros(128, 256, dtype=torch.bfloat16)
    assert marlin_proj.pack_from_bf16(cpu_w, 128) is None       # not on the GPU -> caller stays bf16
    assert marlin_proj.pack_from_bf16_batch([]) == []
    assert marlin_proj.pack_from_bf16_batch([(cpu_w, 128)]) == [None]
    w = oracle.c_lcg_fill(128 * 256, 5, 0.5).reshape(128, 256)
    ph = marlin_proj.pack_host(marlin_proj.PackJobHost(w, 128, 256, 128))
    b, s, _ = pack.quantize_and_pack(w, 128, 256, 128)
    assert np.array_equal(ph.b_packed_vec, b) and np.array_equal(ph.scales_vec, s)


def test_library_exports_every_projection_symbol():
    header = (ROOT / "include" / "kiln_marlin_proj.h").read_text()
    declared = set(re.findall(r"\b(kiln_(?:marlin_proj|w4a16_artifact)_\w+)\s*\(", header))
    assert declared == set(_lib.PROJ_EXPORTS)
    raw = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared:
        assert hasattr(raw, name), name


def test_projection_layer_argument_errors_without_gpu():
    """Checks that run before any GPU call, with the reference's error texts (marlin_proj.rs:96-101)."""
    L = _lib.load()
    out = ctypes.c_void_p()
    dummy = ctypes.c_void_p(16)
    assert L.kiln_marlin_proj_pack_from_bf16(dummy, 128, 256, 128, -1, ctypes.byref(out)) == _lib.PROJ_SKIPPED
    assert L.kiln_marlin_proj_pack_from_bf16(dummy, 100, 256, 128, 0, ctypes.byref(out)) == _lib.PROJ_SKIPPED
    assert L.kiln_marlin_proj_pack_from_bf16(dummy, 128, 32, 128, 0, ctypes.byref(out)) == _lib.PROJ_SKIPPED
    assert out.value is None
    assert L.kiln_marlin_proj_pack_from_bf16(dummy, 128, 256, 64, 0, ctypes.byref(out)) == _lib.PROJ_ERR
    assert L.kiln_marlin_proj_last_error().decode() == "marlin_proj: groupsize must be -1 or 128 (got 64)"
    assert L.kiln_marlin_proj_pack_from_bf16(None, 128, 256, 128, 0, ctypes.byref(out)) == _lib.PROJ_ERR
    assert "2D [k, n]" in L.kiln_marlin_proj_last_error().decode()


def test_artifact_round_trip_and_rejections(tmp_path, oracle):
    """The persisted form of a packed projection: header fields, body, checksum."""
    L = _lib.load()
    k, n, g = 256, 512, 128
    w = oracle.c_lcg_fill(k * n, 11, 0.5).reshape(k, n)
    b, s, _ = pack.quantize_and_pack(w, k, n, g)
    path = tmp_path / "proj.kw4a16"
    assert L.kiln_w4a16_artifact_write(str(path).encode(), b.ctypes.data, s.ctypes.data, k, n, g) == 0
    assert path.stat().st_size == 64 + k * n // 2 + (k // g) * n * 2
    kk, nn = ctypes.c_int64(), ctypes.c_int64()
    gg, ver = ctypes.c_int(), ctypes.c_int()
    assert L.kiln_w4a16_artifact_info(str(path).encode(), ctypes.byref(kk), ctypes.byref(nn), ctypes.byref(gg),
                                      ctypes.byref(ver)) == 0
    assert (kk.value, nn.value, gg.value, ver.value) == (k, n, g, L.kiln_w4a16_layout_version())
    b2, s2 = np.empty_like(b), np.empty_like(s)
    assert L.kiln_w4a16_artifact_read(str(path).encode(), b2.ctypes.data, s2.ctypes.data) == 0
    assert np.array_equal(b, b2) and np.array_equal(s, s2)
    raw = bytearray(path.read_bytes())
    assert bytes(raw[:8]) == b"KW4A16\0\0"

    def expect_error(data, text):
        bad = tmp_path / "bad.kw4a16"
        bad.write_bytes(bytes(data))
        assert L.kiln_w4a16_artifact_read(str(bad).encode(), b2.ctypes.data, s2.ctypes.data) == _lib.PROJ_ERR
        assert text in L.kiln_marlin_proj_last_error().decode()

    flipped = bytearray(raw); flipped[64 + 1000] ^= 0x10
    expect_error(flipped, "checksum mismatch")
    expect_error(raw[:-7], "truncated")
    expect_error(raw[:40], "too short")
    magic = bytearray(raw); magic[0] = ord("X")
    expect_error(magic, "not a packed-weight artefact")
    version = bytearray(raw); version[8] = 99
    expect_error(version, "layout version 99")
    # revision 1 interleaved gate and up by 32 columns; a fused pack of that age would be paired wrongly
    older = bytearray(raw); older[8] = 1
    expect_error(older, "layout version 1 != library's 2")
    shape = bytearray(raw); shape[16] = 1          # k = 257
    expect_error(shape, "inconsistent artefact header")
    assert L.kiln_w4a16_artifact_read(str(tmp_path / "missing").encode(), b2.ctypes.data, s2.ctypes.data) == _lib.PROJ_ERR
    assert L.kiln_w4a16_artifact_write(str(path).encode(), b.ctypes.data, s.ctypes.data, 100, n, g) == _lib.PROJ_ERR


def test_repack_cli_converts_a_safetensors_shard(tmp_path, oracle):
    """`python -m kiln_amd.repack`: GPTQ triples are repacked without touching the codes, float
    weights are quantised from their [out, in] orientation, odd shapes are skipped."""
    import torch
    from safetensors.torch import save_file
    from kiln_amd import repack

    k, n, g = 256, 512, 128
    codes = oracle.gen_codes(k, n, seed=4)
    q = oracle.np_pack_gptq(codes)
    s_bits = oracle.gen_scales_f16(k, n, g, seed=4)
    w = oracle.c_lcg_fill(k * n, 8, 0.5).reshape(k, n)
    shard = tmp_path / "model-00001.safetensors"
    save_file({
        "layers.0.mlp.down_proj.qweight": torch.from_numpy(q.view(np.int32).copy()),
        "layers.0.mlp.down_proj.scales": torch.from_numpy(s_bits.view(np.float16).copy()),
        "layers.0.mlp.down_proj.qzeros": torch.full((k // g, n // 8), 0x88888888 - (1 << 32), dtype=torch.int32),
        "layers.0.attn.q_proj.weight": torch.from_numpy(np.ascontiguousarray(w.T)).to(torch.bfloat16),
        "layers.0.attn.in_proj_a.weight": torch.zeros(32, 256, dtype=torch.bfloat16),
        "layers.0.norm.weight": torch.ones(256),
    }, str(shard))
    out = tmp_path / "packed"
    assert repack.main(["--out", str(out), "--quantize-float", str(shard)]) == 0
    L = _lib.load()

    def read(name):
        kk, nn, gg, ver = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int(), ctypes.c_int()
        path = str(out / name).encode()
        assert L.kiln_w4a16_artifact_info(path, ctypes.byref(kk), ctypes.byref(nn), ctypes.byref(gg),
                                          ctypes.byref(ver)) == 0
        b = np.empty(kk.value * nn.value // 8, dtype=np.int32)
        s = np.empty((1 if gg.value == -1 else kk.value // gg.value) * nn.value, dtype=np.uint16)
        assert L.kiln_w4a16_artifact_read(path, b.ctypes.data, s.ctypes.data) == 0
        return b, s, kk.value, nn.value, gg.value

    b, s, kk, nn, gg = read("layers.0.mlp.down_proj.kw4a16")
    b_ref, s_ref = pack.repack_gptq(q, s_bits, None, g)
    assert (kk, nn, gg) == (k, n, g)
    assert np.array_equal(b, b_ref.ravel()) and np.array_equal(s, np.asarray(s_ref).view(np.uint16).ravel())
    b, s, kk, nn, gg = read("layers.0.attn.q_proj.kw4a16")
    w_bf = oracle.np_bf16_to_f32(oracle.np_f32_to_bf16(w))          # the shard holds bf16
    b_ref, s_ref, _ = pack.quantize_and_pack(w_bf, k, n, g)
    assert np.array_equal(b, b_ref.ravel()) and np.array_equal(s, np.asarray(s_ref).view(np.uint16).ravel())
    assert not (out / "layers.0.attn.in_proj_a.kw4a16").exists() and not (out / "layers.0.norm.kw4a16").exists()


def test_interleave_gate_up_is_a_column_permutation(oracle):
    """Dequantising the interleaved pack gives, per 16 columns, 8 gate columns then the 8
    matching up columns; shapes outside n_each % 128 == 0 are rejected."""
    k, n_each, g = 256, 256, 128
    packs = []
    for seed in (1, 2):
        codes = oracle.gen_codes(k, n_each, seed)
        s_bits = oracle.gen_scales_f16(k, n_each, g, seed)
        b, s = pack.repack_gptq(oracle.np_pack_gptq(codes), s_bits, None, g)
        packs.append((b, s, oracle.np_dequant_f32(oracle.np_pack_gptq(codes), s_bits, g)))
    b_gu, s_gu = pack.interleave_gate_up(packs[0][0], packs[0][1], packs[1][0], packs[1][1], g)
    assert b_gu.shape == (k // 16, 4 * n_each) and s_gu.shape == (k // g, 2 * n_each)
    q_gu, s_plain = pack.unpack_to_gptq(b_gu, s_gu, g)
    deq = oracle.c_dequant_f32(q_gu.view(np.uint32), np.asarray(s_plain).view(np.uint16), g)
    want = np.empty((k, 2 * n_each), np.float32)
    for j in range(n_each // 8):
        want[:, 16 * j:16 * j + 8] = packs[0][2][:, 8 * j:8 * j + 8]
        want[:, 16 * j + 8:16 * j + 16] = packs[1][2][:, 8 * j:8 * j + 8]
    assert np.array_equal(deq, want)
    with pytest.raises(marlin_gemm.MarlinGemmError, match="shape"):
        pack.interleave_gate_up(packs[0][0][:, :2 * 192].copy(), packs[0][1][:, :192].copy(),
                                packs[1][0][:, :2 * 192].copy(), packs[1][1][:, :192].copy(), g)


def test_interleave_gate_up_lora_b_follows_the_packed_columns():
    """Rows of the stacked LoRA B in the column order of the interleaved pack (per 16 rows 8 gate
    columns, then the 8 matching up columns), gate's entries in gate's rank columns, up's in up's."""
    import torch
    n_out, rg, ru = 32, 3, 5
    gate = (torch.arange(n_out * rg, dtype=torch.float32).reshape(n_out, rg) + 1).to(torch.bfloat16)
    up = -(torch.arange(n_out * ru, dtype=torch.float32).reshape(n_out, ru) + 1).to(torch.bfloat16)
    out = marlin_gemm.interleave_gate_up_lora_b(gate, up, n_out)
    assert tuple(out.shape) == (2 * n_out, rg + ru) and out.dtype == torch.bfloat16
    for j in range(n_out // 8):
        assert torch.equal(out[16 * j:16 * j + 8, :rg], gate[8 * j:8 * j + 8])
        assert torch.equal(out[16 * j + 8:16 * j + 16, rg:], up[8 * j:8 * j + 8])
        assert not out[16 * j:16 * j + 8, rg:].any() and not out[16 * j + 8:16 * j + 16, :rg].any()
    only_up = marlin_gemm.interleave_gate_up_lora_b(None, up, n_out)
    assert tuple(only_up.shape) == (2 * n_out, ru) and not only_up[0:8].any() and torch.equal(only_up[8:16], up[0:8])
    with pytest.raises(marlin_gemm.MarlinGemmError):
        marlin_gemm.interleave_gate_up_lora_b(None, None, n_out)
    with pytest.raises(marlin_gemm.MarlinGemmError):
        marlin_gemm.interleave_gate_up_lora_b(gate[:16], up, n_out)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU only: --gpus 2 (or a multi-rank environment) exits with a message."""
    import os
    import subprocess
    import sys
    env = dict(os.environ)
    res = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, env=env)
    assert res.returncode != 0 and "one GPU" in res.stderr and res.stdout.strip() == ""
    env["WORLD_SIZE"] = "4"
    res = subprocess.run([sys.executable, str(ROOT / "bench.py")], capture_output=True, text=True, env=env)
    assert res.returncode != 0 and "one GPU" in res.stderr


def test_decode_plans_are_launchable_and_keep_model_shapes_exchange_free():
    """The small-M planner runs on the host.  Every plan must satisfy what the kernel that runs
    it assumes (runs no longer than a slice, a tile cut by at most one block boundary, the
    block's tiles within its flag array, the slice within LDS -- or, for the register-fragment
    instance, whole tiles, equal slices, groups dividing evenly among at most 12 wavefronts);
    for the model's projection shapes with K <= 4096 the blocks must hold whole tiles of a
    single K slice, so that nothing is exchanged through the workspace, and the down projection
    must keep its slices tile-aligned.  Slabs of 17...32 rows exist only as register plans."""
    import ctypes
    from kiln_amd import _lib
    lib = _lib.load()
    plan = lib.kiln_w4a16_debug_decode_plan
    plan.argtypes = [ctypes.c_int] * 4 + [ctypes.POINTER(ctypes.c_int)]
    out = (ctypes.c_int * 8)()
    shapes = [(k, n) for k in (128, 256, 2560, 4096, 9216, 16384) for n in (256, 1024, 2560, 8192, 9216, 18432)]
    for cus in (256, 64, 304):
        for m in (1, 4, 16, 17, 32):
            for k, n in shapes:
                rc = plan(m, n, k, cus, out)
                if m > 16 and rc == 1:
                    continue                      # no register plan: the dispatcher takes 16-row slabs
                assert rc == 0, (m, k, n, cus)
                ks, gs, u, bps, waves, direct, regs, gm_tiles = list(out)
                g, nt = k // 128, n // 16
                if gm_tiles < 0:
                    # the private-staging instance (m <= 16): whole tiles, equal slices of any length,
                    # every wavefront one to six groups (three from three tiles on), at most 16 chunks
                    tiles, gpw = -gm_tiles, -(-gs // waves)
                    assert m <= 16 and not direct and not regs and ks * gs == g and 1 <= tiles <= 6
                    assert 1 <= waves <= 16 and waves <= gs and gpw <= (6 if tiles <= 2 else 3) and tiles * gpw <= 16
                    assert u == tiles * gpw and bps == -(-nt // tiles)
                    assert waves * max(min(gpw, 3) * 4096, tiles * 1024) <= 159 * 1024
                    continue
                gs_last = g - (ks - 1) * gs
                assert 1 <= ks <= 8 and 1 <= gs_last <= gs and (ks - 1) * gs < g
                assert 1 <= u <= min(12, gs_last) and 1 <= waves <= 16
                assert waves * u >= gs and bps * waves * u >= nt * gs
                assert (waves * u) // gs_last + 2 <= 40
                assert not (direct and regs) and (regs or m <= 16) and not (gm_tiles and (regs or direct))
                if gm_tiles:
                    gpw = -(-gs // waves)
                    assert ks * gs == g and 2 <= gm_tiles <= 6 and u == gm_tiles * gpw and gpw <= 4 and gs >= waves
                    assert bps == -(-nt // gm_tiles)
                    assert 16 * (gs * 256 + 16) + waves * gm_tiles * 1024 <= 159 * 1024
                if regs:
                    tiles, gpw = waves * u // gs, gs // waves
                    assert ks * gs == g and (waves * u) % gs == 0 and gs % waves == 0 and waves <= 12
                    assert 1 <= tiles <= 6 and gpw in (1, 2, 3, 4, 5, 6, 8)
                    assert gs <= 32 and (tiles >= 2 or (m <= 4 and u <= 2))
                elif not direct:
                    assert gs <= 32 and 16 * (gs * 256 + 16) + waves * 2048 <= 159 * 1024
                if direct:
                    assert m <= 4 and u <= 3
    for k, n in [(2560, 18432), (2560, 8192), (2560, 9216), (4096, 2560), (2560, 2560)]:
        assert plan(16, n, k, 256, out) == 0
        ks, gs, u, bps, waves, _, _, gm_tiles = list(out)
        assert ks == 1 and (gm_tiles or (waves * u) % gs == 0) and bps <= 256, (k, n, list(out))
    for m in (16, 32):
        assert plan(m, 2560, 9216, 256, out) == 0
        ks, gs, u, bps, waves, _, regs, gm_tiles = list(out)
        assert ks * gs == 72 and (gm_tiles or (waves * u) % gs == 0) and ks * bps <= 256 and regs == (m > 16), list(out)
    # few rows of the down projection run unsliced (nothing through the workspace); 16 rows are sliced
    for m, want_ks in ((1, 1), (4, 1), (16, 3)):
        assert plan(m, 2560, 9216, 256, out) == 0 and out[0] == want_ks and out[7] < 0, (m, list(out))
    assert plan(33, 2560, 2560, 256, out) == 1 and plan(16, 2560, 100, 256, out) == 1


MODEL_SHAPES = [(2560, 8192), (4096, 2560), (2560, 18432), (9216, 2560)]      # (k, n)


@pytest.mark.parametrize("k,n", MODEL_SHAPES)
def test_workspace_bytes_is_monotone_in_m(k, n):
    """A workspace sized for the largest m must serve every smaller call: the size function is
    the running maximum of the per-call need, so it never decreases with m (m = 1...8192 on the
    model's four projection shapes), and it starts at no less than the zeroed counter prefix."""
    L = _lib.load()
    sizes = [L.kiln_w4a16_workspace_bytes(m, n, k) for m in range(1, 8193)]
    assert sizes[0] >= L.kiln_w4a16_workspace_zeroed_bytes()
    drops = [(m + 1, sizes[m - 1], sizes[m]) for m in range(1, len(sizes)) if sizes[m] < sizes[m - 1]]
    assert not drops, drops[:5]
    # with overrides the sizing takes them into account and is monotone as well
    tuned = [L.kiln_w4a16_workspace_bytes_tuned(m, n, k, 128, 16, -1) for m in range(1, 200)]
    assert all(b >= a for a, b in zip(tuned, tuned[1:]))
    assert tuned[15] >= sizes[15] or tuned[15] >= L.kiln_w4a16_workspace_zeroed_bytes()


def test_memoised_workspace_sizes_equal_the_computed_ones():
    """The shipped library remembers the size it computed for (m, n, k, overrides); the tuning build computes it
    every time.  Both must agree, on first and on repeated queries, also where the mid-M kernel's row range ends."""
    shipped, tuning = _lib.load(), ctypes.CDLL(str(_lib.TUNING_LIB_PATH))
    for f in (tuning.kiln_w4a16_workspace_bytes, tuning.kiln_w4a16_workspace_bytes_tuned):
        f.restype = ctypes.c_size_t
    for k, n in MODEL_SHAPES + [(11008, 4096), (1024, 1024), (2560, 1024), (18944, 3584)]:
        for m in (1, 16, 17, 64, 65, 128, 320, 512, 1024, 1025, 4096):
            want = tuning.kiln_w4a16_workspace_bytes(m, n, k)
            assert shipped.kiln_w4a16_workspace_bytes(m, n, k) == want, (m, k, n)
            assert shipped.kiln_w4a16_workspace_bytes(m, n, k) == want, (m, k, n)
            assert shipped.kiln_w4a16_workspace_bytes_tuned(m, n, k, 128, 16, -1) == tuning.kiln_w4a16_workspace_bytes_tuned(m, n, k, 128, 16, -1)


def test_workspace_is_small_where_nothing_is_exchanged():
    """Decode calls need little more than the zeroed prefix -- the counters and the region in which
    K slices exchange their parts without counters, which is where the down projection's three
    slices meet -- and the LoRA projection scratch."""
    L = _lib.load()
    z = L.kiln_w4a16_workspace_zeroed_bytes()
    assert z == 64 * 1024 + 4 * 1024 * 1024
    for k, n in [(2560, 8192), (4096, 2560), (2560, 18432)]:
        assert z <= L.kiln_w4a16_workspace_bytes(16, n, k) <= z + 64 * 1024, (k, n)
    # adapters whose stacked rank is not a multiple of 8 take the kernels whose three slices meet through
    # counters: their partial tiles
    down = L.kiln_w4a16_workspace_bytes(16, 2560, 9216)
    assert z + 3 * 2 * 2560 * 64 <= down <= z + 3 * 2 * 2560 * 64 + 64 * 1024
    # no shape, however small or unsupported, is sized below the prefix a caller zero-fills
    for m, n, k in [(1, 256, 128), (0, 256, 128), (16, 100, 128), (16, 256, 100)]:
        assert L.kiln_w4a16_workspace_bytes(m, n, k) >= z


def test_shipped_library_has_no_tuning_setters():
    """The plan overrides exist only in the tuning build; the shipped library exports none."""
    shipped, tuning = _lib.load(), _lib.load_tuning()
    for name in _lib.TUNING_EXPORTS:
        assert not hasattr(shipped, name), name
        assert hasattr(tuning, name), name
    for name in _lib.EXPORTS + _lib.PROJ_EXPORTS:
        assert hasattr(shipped, name) and hasattr(tuning, name), name


def test_long_k_falls_back_to_the_matrix_core_path():
    """A K that no small-M instance can slice has no small-M plan; such a GEMM takes the
    matrix-core kernel at any row count instead of failing (the reference accepts any k % 128 == 0)."""
    L = _lib.load()
    out = (ctypes.c_int * 8)()
    for m in (1, 16, 48):               # 257 groups: no equal slicing fits any small-M instance
        assert L.kiln_w4a16_debug_gemm_plan(m, 2560, 32896, 256, out) == 0
        assert out[0] == 1, (m, list(out))
    for m in (1, 16):                   # 320 groups = 8 slices of 40: the private-staging instance takes them
        assert L.kiln_w4a16_debug_gemm_plan(m, 2560, 40960, 256, out) == 0
        assert out[0] == 0 and out[1] == 1, (m, list(out))
    assert L.kiln_w4a16_debug_gemm_plan(16, 2560, 9216, 256, out) == 0 and out[0] == 0 and out[1] == 1


def test_layer_wiring_keeps_bf16_without_a_gpu_and_reproduces_the_reference_selection():
    """Host logic of the layer-level wiring (no GPU): weights that are not on the GPU come back
    unpacked (marlin_proj.rs:91-93) and every projection stays on its bf16 matmul; the reference's
    own selection queues q_proj and the three MLP projections only (forward.rs:1884-1890, 2002-2018)."""
    import torch
    from kiln_amd import layer_pack
    from kiln_amd.layer_pack import LayerProjections, PackKind
    torch.manual_seed(0)
    shapes = {PackKind.QProj: (256, 512), PackKind.KProj: (256, 256), PackKind.InProjA: (256, 32),
              PackKind.GateProj: (256, 512), PackKind.UpProj: (256, 512), PackKind.DownProj: (512, 256)}
    layer = LayerProjections({kind: torch.randn(k, n).to(torch.bfloat16) for kind, (k, n) in shapes.items()})
    inputs, meta = layer_pack.queue_layer(3, layer, layer_pack.REFERENCE_KINDS)
    assert [e.kind for e in meta] == [PackKind.QProj, PackKind.GateProj, PackKind.UpProj, PackKind.DownProj]
    assert all(e.layer_idx == 3 for e in meta) and all(g == 128 for _, g in inputs)
    stats = layer_pack.pack_layers([layer])
    assert stats == {"inputs": 6, "packed": 0, "kept_bf16": 6, "gate_up_fused": 0}
    x = torch.randn(2, 3, 256).to(torch.bfloat16)
    y = layer.forward(PackKind.KProj, x)
    assert tuple(y.shape) == (2, 3, 256) and torch.equal(y, x @ layer.weights_t[PackKind.KProj])
    assert marlin_proj.shape_is_supported(2560, 1024) and not marlin_proj.shape_is_supported(2560, 32)


def test_bf16_drop_switch_follows_the_environment(monkeypatch):
    """`KILN_DISABLE_MARLIN_BF16_DROP` (forward.rs:1565-1580): install drops the bf16 copy unless the
    variable says 1 / true / yes; an explicit argument wins over the environment."""
    import torch
    from kiln_amd import layer_pack
    from kiln_amd.layer_pack import LayerProjections, PackKind
    from kiln_amd.marlin_proj import MarlinPackedProj
    stand_in = MarlinPackedProj(torch.zeros(8, 512, dtype=torch.int32), torch.zeros(1, 256, dtype=torch.float16), 128, 128, 256)

    def install(**kw):
        layer = LayerProjections({PackKind.QProj: torch.zeros(128, 256, dtype=torch.bfloat16)})
        layer_pack.install_packed(layer, PackKind.QProj, stand_in, **kw)
        assert layer.is_packed(PackKind.QProj)
        return layer.weights_t[PackKind.QProj] is None

    monkeypatch.delenv("KILN_DISABLE_MARLIN_BF16_DROP", raising=False)
    assert not marlin_proj.bf16_drop_disabled() and install() is True
    for v, disabled in [("1", True), ("TRUE", True), (" yes ", True), ("0", False), ("on", False), ("", False)]:
        monkeypatch.setenv("KILN_DISABLE_MARLIN_BF16_DROP", v)
        assert marlin_proj.bf16_drop_disabled() is disabled
        assert install() is (not disabled)
    monkeypatch.setenv("KILN_DISABLE_MARLIN_BF16_DROP", "1")
    assert install(drop_bf16=True) is True


def test_adapters_of_side_by_side_projections_become_one_block_structured_set():
    """`fuse_column_blocks` (no GPU): projections packed side by side share x, so their adapters' A matrices
    stack along the rank axis and B becomes block-structured; B_fused @ A_fused restricted to a member's rows
    equals that member's own sum of scaled B_i @ A_i."""
    import torch
    from kiln_amd.lora import LoraProjectionWeights, fuse_column_blocks, stack_adapters
    torch.manual_seed(1)
    k, widths = 64, (48, 16, 32)
    mk = lambda n, r: LoraProjectionWeights(torch.randn(r, k).to(torch.bfloat16), torch.randn(n, r).to(torch.bfloat16))
    q = stack_adapters([mk(48, 4), mk(48, 8)], [0.5, 2.0])
    v = mk(32, 4)
    fused = fuse_column_blocks([q, None, v], widths, lora_scale=3.0)
    assert fused.ranks == (4, 8, 4) and fused.scales == (0.5, 2.0, 3.0)
    assert tuple(fused.a_cat.shape) == (16, k) and tuple(fused.b_cat.shape) == (96, 16)
    scale_cols = torch.tensor([0.5] * 4 + [2.0] * 8 + [3.0] * 4)
    delta = (fused.b_cat.float() * scale_cols) @ fused.a_cat.float()
    want_q = (q.b_cat.float() * torch.tensor([0.5] * 4 + [2.0] * 8)) @ q.a_cat.float()
    assert torch.allclose(delta[:48], want_q, rtol=1e-5, atol=1e-5) and torch.count_nonzero(delta[48:64]) == 0
    assert torch.allclose(delta[64:], 3.0 * (v.b.float() @ v.a.float()), rtol=1e-5, atol=1e-5)
    assert fuse_column_blocks([None, None], (8, 8)) is None
    # pad_rank: zero rows of A and zero columns of B up to a multiple of 8, the delta unchanged
    from kiln_amd.lora import pad_rank
    odd = stack_adapters([mk(48, 4), mk(48, 5)], [0.5, 2.0])
    padded = pad_rank(odd)
    assert padded.ranks == (4, 12) and tuple(padded.a_cat.shape) == (16, k) and tuple(padded.b_cat.shape) == (48, 16)
    assert torch.equal(padded.a_cat[:9], odd.a_cat) and torch.count_nonzero(padded.a_cat[9:]) == 0
    assert torch.equal(padded.b_cat[:, :9], odd.b_cat) and torch.count_nonzero(padded.b_cat[:, 9:]) == 0
    assert pad_rank(padded) is padded and pad_rank(q) is not q and pad_rank(fused) is fused
    big = stack_adapters([mk(48, 61)], [1.0])
    assert pad_rank(big).ranks == (64,) and pad_rank(stack_adapters([mk(48, 30), mk(48, 35)], [1.0, 1.0])).ranks == (30, 35)
    with pytest.raises(marlin_proj.MarlinProjError):
        fuse_column_blocks([v, None], (48, 16))


def test_workspace_sizing_for_a_part_of_the_chip():
    """`sms` may name fewer compute units than the projection of a call with adapters would take for itself (eight
    at K = 4096): the planners never plan for less than one unit.  In a child process: the failure was a division
    by zero on the host, which ends the process."""
    import os, subprocess, sys
    code = ("from kiln_amd import _lib\n"
            "L = _lib.load()\n"
            "for m, n, k, sms in [(129, 9216, 4096, 8), (24, 18432, 384, 1), (16, 2560, 9216, 3), (2048, 18432, 2560, 2), (64, 2560, 4096, 5)]:\n"
            "    v = L.kiln_w4a16_workspace_bytes_tuned(m, n, k, -1, -1, sms)\n"
            "    assert 0 < v < 1 << 31, (m, n, k, sms, v)\n"
            "print('sized')\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "sized" in r.stdout, (r.returncode, r.stderr[-500:])
