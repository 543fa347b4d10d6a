"""The load-time wiring of packed projections for both layer kinds (host mirror of
crates/kiln-model/src/forward.rs:1884-2085 widened to k/v/o_proj and the GDN projections), on
the model's real projection shapes, against the CPU oracle."""
import numpy as np
import pytest
import torch

from kiln_amd import layer_pack
from kiln_amd.layer_pack import LayerProjections, PackKind
from tests.gpu_util import bf16_bits, bf16_tensor, row_errors

pytestmark = pytest.mark.gpu

HIDDEN = 2560
# (k, n) of every projection: crates/kiln-core/src/config.rs:80-97 (16 heads x 256 gated -> 8192,
# 4 kv heads x 256 = 1024, 32 value heads x 128 = 4096, 16 + 16 + 32 heads x 128 = 8192 for qkv)
FULL = {PackKind.QProj: (HIDDEN, 8192), PackKind.KProj: (HIDDEN, 1024), PackKind.VProj: (HIDDEN, 1024),
        PackKind.OProj: (4096, HIDDEN)}
LINEAR = {PackKind.InProjQkv: (HIDDEN, 8192), PackKind.InProjZ: (HIDDEN, 4096), PackKind.OutProj: (4096, HIDDEN),
          PackKind.InProjA: (HIDDEN, 32), PackKind.InProjB: (HIDDEN, 32)}
MLP = {PackKind.GateProj: (HIDDEN, 9216), PackKind.UpProj: (HIDDEN, 9216), PackKind.DownProj: (9216, HIDDEN)}


def _weights(oracle, shapes, seed):
    host, dev = {}, {}
    for i, (kind, (k, n)) in enumerate(shapes.items()):
        w = oracle.c_lcg_fill(k * n, 0xC0FFEE5EED ^ (seed * 131 + i), 0.5).reshape(k, n)
        bits = oracle.np_f32_to_bf16(w)
        host[kind] = oracle.np_bf16_to_f32(bits)          # what the packer quantises: the bf16 weight
        dev[kind] = bf16_tensor(bits)
    return host, dev


@pytest.fixture(scope="module")
def packed_layers(oracle):
    h0, d0 = _weights(oracle, {**FULL, **MLP}, 1)
    h1, d1 = _weights(oracle, {**LINEAR, **MLP}, 2)
    layers = [LayerProjections(d0), LayerProjections(d1)]
    stats = layer_pack.pack_layers(layers, fuse_gate_up=True)
    return layers, [h0, h1], stats


def test_every_supported_projection_is_packed_and_the_rest_stay_bf16(packed_layers):
    layers, _, stats = packed_layers
    assert stats == {"inputs": 15, "packed": 13, "kept_bf16": 2, "gate_up_fused": 2}
    full, linear = layers
    for kind in (*FULL, *MLP):
        assert full.is_packed(kind) and full.weights_t[kind] is None, kind        # bf16 copy dropped
    for kind in (PackKind.InProjQkv, PackKind.InProjZ, PackKind.OutProj, *MLP):
        assert linear.is_packed(kind), kind
    for kind in (PackKind.InProjA, PackKind.InProjB):                             # n = 32: marlin_proj.rs:53-55
        assert not linear.is_packed(kind) and linear.weights_t[kind] is not None
    assert tuple(full.packed[PackKind.KProj].b_packed.shape) == (HIDDEN // 16, 2 * 1024)
    assert tuple(full.packed[PackKind.KProj].scales.shape) == (HIDDEN // 128, 1024)


def _check(oracle, layer, host_w, kind, m, seed):
    k, n = host_w[kind].shape
    x = oracle.gen_normal_bf16(m, k, 1.0, seed)
    y = layer.forward(kind, bf16_tensor(x))
    torch.cuda.synchronize()
    assert tuple(y.shape) == (m, n)
    if layer.is_packed(kind):
        codes, s_bits, _ = oracle.c_quantize(host_w[kind], 128)
        y_ref = oracle.c_w4a16_cpu_path(x, oracle.np_pack_gptq(codes), s_bits, 128)
    else:
        y_ref = oracle.c_gemm_f32(x, host_w[kind])
    err, yv, _ = row_errors(bf16_bits(y), y_ref, oracle)
    assert np.all(np.isfinite(yv)) and err.max() <= 1e-2, (kind, m, err.max())


@pytest.mark.parametrize("m", [1, 16, 512])
@pytest.mark.parametrize("kind", [PackKind.KProj, PackKind.VProj])
def test_kv_projections_n1024(oracle, packed_layers, kind, m):
    layers, host, _ = packed_layers
    _check(oracle, layers[0], host[0], kind, m, seed=m + 7)


@pytest.mark.parametrize("layer_idx,kind", [(0, PackKind.QProj), (0, PackKind.OProj), (1, PackKind.InProjQkv),
                                            (1, PackKind.InProjZ), (1, PackKind.OutProj), (1, PackKind.InProjA),
                                            (1, PackKind.InProjB), (0, PackKind.DownProj)])
def test_remaining_projections(oracle, packed_layers, layer_idx, kind):
    layers, host, _ = packed_layers
    for m in (1, 16):
        _check(oracle, layers[layer_idx], host[layer_idx], kind, m, seed=m + layer_idx)
    x3 = bf16_tensor(oracle.gen_normal_bf16(6, host[layer_idx][kind].shape[0], 1.0, 3)).reshape(2, 3, -1)
    assert tuple(layers[layer_idx].forward(kind, x3).shape) == (2, 3, host[layer_idx][kind].shape[1])   # rank 3


def test_fused_gate_up_swiglu_of_a_layer(oracle, packed_layers):
    layers, host, _ = packed_layers
    m = 16
    x = oracle.gen_normal_bf16(m, HIDDEN, 1.0, 11)
    h = layers[1].swiglu(bf16_tensor(x))
    sides = []
    for kind in (PackKind.GateProj, PackKind.UpProj):
        codes, s_bits, _ = oracle.c_quantize(host[1][kind], 128)
        sides.append(oracle.c_w4a16_cpu_path(x, oracle.np_pack_gptq(codes), s_bits, 128))
    err, _, _ = row_errors(bf16_bits(h), oracle.c_swiglu_f32(sides[0], sides[1]), oracle)
    assert tuple(h.shape) == (m, 9216) and err.max() <= 1e-2


def test_fused_gate_up_swiglu_of_a_layer_with_adapters(oracle, packed_layers):
    """`LayerProjections.swiglu` with a LoRA adapter on gate_proj and two stacked ones on up_proj: the
    fused launch against the oracle's two projections + deltas + silu * up, and against the layer's
    own unfused route (adapters too large for the fused entry point fall back to it)."""
    from kiln_amd.lora import LoraProjectionWeights, stack_adapters
    layers, host, _ = packed_layers
    m = 24
    x = oracle.gen_normal_bf16(m, HIDDEN, 1.0, 13)
    adapters = {}
    for name, ranks in (("gate", (16,)), ("up", (8, 16))):
        adapters[name] = [(oracle.gen_normal_bf16(r, HIDDEN, 0.05, 40 + 7 * i + len(name)),
                           oracle.gen_normal_bf16(9216, r, 0.05, 50 + 7 * i + len(name))) for i, r in enumerate(ranks)]
    scales = {"gate": (0.5,), "up": (1.0, 2.0)}
    sides = []
    for kind, name in ((PackKind.GateProj, "gate"), (PackKind.UpProj, "up")):
        codes, s_bits, _ = oracle.c_quantize(host[1][kind], 128)
        y = oracle.c_w4a16_cpu_path(x, oracle.np_pack_gptq(codes), s_bits, 128)
        for (a_i, b_i), sc in zip(adapters[name], scales[name]):
            oracle.c_lora_delta_add(y, x, a_i, b_i, sc)
        sides.append(y)
    h_ref = oracle.c_swiglu_f32(sides[0], sides[1])
    stacked = {name: stack_adapters([LoraProjectionWeights(bf16_tensor(a_i), bf16_tensor(b_i)) for a_i, b_i in adapters[name]],
                                    scales[name]) for name in adapters}
    h = layers[1].swiglu(bf16_tensor(x), stacked["gate"], stacked["up"])
    err, _, _ = row_errors(bf16_bits(h), h_ref, oracle)
    assert tuple(h.shape) == (m, 9216) and err.max() <= 1e-2
    # a single adapter given as LoraProjectionWeights with the call's scale, on gate only
    a0, b0 = adapters["gate"][0]
    h1 = layers[1].swiglu(bf16_tensor(x), LoraProjectionWeights(bf16_tensor(a0), bf16_tensor(b0)), None, 0.5)
    codes, s_bits, _ = oracle.c_quantize(host[1][PackKind.UpProj], 128)
    up_plain = oracle.c_w4a16_cpu_path(x, oracle.np_pack_gptq(codes), s_bits, 128)
    codes, s_bits, _ = oracle.c_quantize(host[1][PackKind.GateProj], 128)
    gate1 = oracle.c_w4a16_cpu_path(x, oracle.np_pack_gptq(codes), s_bits, 128)
    oracle.c_lora_delta_add(gate1, x, a0, b0, 0.5)
    err1, _, _ = row_errors(bf16_bits(h1), oracle.c_swiglu_f32(gate1, up_plain), oracle)
    assert err1.max() <= 1e-2


@pytest.fixture(scope="module")
def fused_layers(oracle):
    h0, d0 = _weights(oracle, FULL, 1)
    h1, d1 = _weights(oracle, LINEAR, 2)
    layers = [LayerProjections(d0), LayerProjections(d1)]
    stats = layer_pack.pack_layers(layers, fuse_same_input_groups=True)
    return layers, [h0, h1], stats


@pytest.mark.parametrize("m", [1, 16, 40, 300])
@pytest.mark.parametrize("layer_idx,kinds", [(0, (PackKind.QProj, PackKind.KProj, PackKind.VProj)),
                                             (1, (PackKind.InProjQkv, PackKind.InProjZ))])
def test_projections_of_one_input_as_one_gemm(oracle, fused_layers, layer_idx, kinds, m):
    """q | k | v (2560 -> 8192 + 1024 + 1024) and in_proj_qkv | in_proj_z (2560 -> 8192 + 4096) packed side by
    side: one launch, the members' results are column ranges of its output; each against the oracle and
    against the member's own launch."""
    layers, host, stats = fused_layers
    assert stats["same_input_fused"] == 2 and tuple(kinds) in layers[layer_idx].same_input_fused
    layer = layers[layer_idx]
    fused = layer.same_input_fused[tuple(kinds)]
    assert fused.n == sum(host[layer_idx][k].shape[1] for k in kinds) and tuple(fused.b_packed.shape) == (HIDDEN // 16, 2 * fused.n)
    x = oracle.gen_normal_bf16(m, HIDDEN, 0.5 if m > 64 else 1.0, seed=m + layer_idx)
    xt = bf16_tensor(x)
    outs = layer.forward_same_input(kinds, xt)
    torch.cuda.synchronize()
    for kind, y in zip(kinds, outs):
        codes, s_bits, _ = oracle.c_quantize(host[layer_idx][kind], 128)
        y_ref = oracle.c_w4a16_cpu_path(x, oracle.np_pack_gptq(codes), s_bits, 128)
        assert tuple(y.shape) == y_ref.shape
        err, yv, _ = row_errors(bf16_bits(y), y_ref, oracle)
        assert np.all(np.isfinite(yv)) and err.max() <= 1e-2, (kind, m, err.max())
        alone = layer.forward(kind, xt).float()
        assert torch.all((y.float() - alone).abs() <= 1e-2 * alone.abs().amax(dim=1, keepdim=True))
    # rank-3 input, as the callers pass it (marlin_proj.rs:285-319)
    outs3 = layer.forward_same_input(kinds, xt.reshape(1, m, HIDDEN))
    assert all(tuple(o.shape) == (1, m, host[layer_idx][k].shape[1]) for o, k in zip(outs3, kinds))


@pytest.mark.parametrize("m", [4, 16, 48])
def test_projections_of_one_input_with_adapters(oracle, fused_layers, m):
    """Adapters on q_proj (two, stacked) and v_proj (one), none on k_proj: on the side-by-side pack they are
    one stacked set -- A matrices row-concatenated, B block-structured -- and x is projected once."""
    from kiln_amd.lora import LoraProjectionWeights, stack_adapters
    layers, host, _ = fused_layers
    kinds = (PackKind.QProj, PackKind.KProj, PackKind.VProj)
    x = oracle.gen_normal_bf16(m, HIDDEN, 1.0, seed=70 + m)
    spec = {PackKind.QProj: ((16, 8), (0.5, 2.0)), PackKind.VProj: ((16,), (1.0,))}
    raw, loras = {}, {}
    for j, (kind, (ranks, scales)) in enumerate(spec.items()):
        n = host[0][kind].shape[1]
        raw[kind] = [(oracle.gen_normal_bf16(r, HIDDEN, 0.05, 100 + 10 * j + i), oracle.gen_normal_bf16(n, r, 0.05, 200 + 10 * j + i))
                     for i, r in enumerate(ranks)]
        loras[kind] = stack_adapters([LoraProjectionWeights(bf16_tensor(a), bf16_tensor(b)) for a, b in raw[kind]], scales)
    outs = layers[0].forward_same_input(kinds, bf16_tensor(x), loras)
    torch.cuda.synchronize()
    for kind, y in zip(kinds, outs):
        codes, s_bits, _ = oracle.c_quantize(host[0][kind], 128)
        y_ref = oracle.c_w4a16_cpu_path(x, oracle.np_pack_gptq(codes), s_bits, 128)
        for (a_i, b_i), sc in zip(raw.get(kind, []), spec.get(kind, ((), ()))[1]):
            oracle.c_lora_delta_add(y_ref, x, a_i, b_i, sc)
        err, _, _ = row_errors(bf16_bits(y), y_ref, oracle)
        assert err.max() <= 1e-2, (kind, m, err.max())
