"""Every GEMM entry point on seeded random shapes and row counts -- sizes no other test names, drawn from
multiples of 128 (K) and 256 (N) between the smallest the library takes and those of 13-B models, and
row counts on both sides of every routing boundary -- against an f32 torch product of the dequantised
weights (`kiln_w4a16_dequant_f32`, itself checked against the oracle in test_gpu_parity.py).  The oracle
covers the named shapes bit for bit elsewhere; this file is about shapes nobody thought of: a refused
launch, a plan that does not fit its kernel, a tile left unwritten.

Tolerance: max |y - y_ref| <= 2e-2 * max |y_ref| over the whole result (bf16 output, T of the low-rank
term rounded to bf16 per K slice as the reference rounds it once: lora_loader.rs:213-232)."""
import random

import pytest
import torch

from kiln_amd import marlin_gemm as mg

pytestmark = pytest.mark.gpu
TOL = 2e-2

ANY_K = [128, 256, 384, 640, 896, 1152, 1408, 2176, 2560, 3200, 4224, 5248, 6784, 9216, 11008, 13696]
ANY_N = [256, 512, 768, 1280, 2304, 2560, 3328, 4352, 6400, 9984, 13056, 18432, 21760, 32000]
MODEL_K = [896, 1024, 1536, 2048, 2560, 3072, 3584, 4096, 5120, 8192, 8960, 9216, 11008, 13824, 14336, 18944]
MODEL_N = [256, 512, 1024, 1536, 2048, 2560, 3584, 4096, 5120, 8192, 9216, 10240, 11264, 12288, 17920, 18432, 22016, 28672]
BOUNDARY_M = [16, 17, 20, 21, 32, 33, 48, 49, 64, 65, 80, 81, 128, 129, 192, 193, 256, 257, 320, 321, 384, 385,
              448, 512, 513, 576, 1024, 1025]
RANKS = [(16,), (16, 32), (8, 8, 16), (64,), (4, 5), (7,), (32, 32)]
KINDS = ["plain", "lora", "swiglu", "swiglu_lora", "mlp"]


def _any_m(rnd):
    r = rnd.random()
    if r < 0.3:
        return rnd.randint(1, 16)
    if r < 0.6:
        return rnd.randint(17, 128)
    if r < 0.9:
        return rnd.randint(129, 1100)
    return rnd.choice([2049, 3000, 4100])


def _weights(k, n, g):
    # any bit pattern is a valid packed weight
    return (torch.randint(-2**31, 2**31 - 1, (k // 16, 2 * n), dtype=torch.int32, device="cuda"),
            (torch.rand(k // 128 if g > 0 else 1, n, device="cuda") * 0.018 + 0.002).half())


def _rel(y, ref):
    return ((y.float() - ref).abs().max() / ref.abs().max().clamp_min(1e-6)).item()


def _swiglu_of(z):
    """silu(gate) * up of a stacked result: per 16 columns, 8 gate columns and then the 8 matching up columns."""
    m, n = z.shape
    v = z.view(m, n // 16, 2, 8)
    return (torch.nn.functional.silu(v[:, :, 0]) * v[:, :, 1]).reshape(m, n // 2)


def _one_case(rnd, boundary):
    k = rnd.choice(MODEL_K if boundary else ANY_K)
    n = rnd.choice(MODEL_N if boundary else ANY_N)
    m = rnd.choice(BOUNDARY_M) if boundary else _any_m(rnd)
    while m * n * k > 1.5e11:
        m = max(1, m // 2)
    g = rnd.choice([128, 128, -1])
    kind = rnd.choice(KINDS)
    if kind in ("swiglu", "swiglu_lora", "mlp") and n % 512 != 0:
        n += 256
    ranks = rnd.choice(RANKS)
    scales = tuple(rnd.choice([0.5, 1.0, 2.0]) for _ in ranks)
    n_down = rnd.choice([256, 1280, 2560, 4352])
    return kind, m, k, n, g, ranks, scales, n_down


def _run_case(kind, m, k, n, g, ranks, scales, n_down):
    b, s = _weights(k, n, g)
    x = torch.randn(m, k, device="cuda").bfloat16()
    ref = x.float() @ mg.dequant_f32(b, s, g)
    rt = sum(ranks)
    la = (torch.randn(rt, k, device="cuda") * 0.03).bfloat16()
    lb = (torch.randn(n, rt, device="cuda") * 0.03).bfloat16()
    if kind in ("lora", "swiglu_lora"):
        o = 0
        for r, sc in zip(ranks, scales):
            t = (sc * (x.float() @ la[o:o + r].float().T)).bfloat16().float()
            ref = ref + t @ lb[:, o:o + r].float().T
            o += r
    if kind == "plain":
        return _rel(mg.marlin_w4a16_gemm(x, b, s, g), ref)
    if kind == "lora":
        return _rel(mg.marlin_w4a16_gemm_lora(x, b, s, g, la, lb, ranks, scales), ref)
    if kind == "swiglu":
        return _rel(mg.marlin_w4a16_gemm_swiglu(x, b, s, g), _swiglu_of(ref))
    if kind == "swiglu_lora":
        return _rel(mg.marlin_w4a16_gemm_swiglu_lora(x, b, s, g, la, lb, ranks, scales), _swiglu_of(ref))
    bd, sd = _weights(n // 2, n_down, g)
    h = _swiglu_of(ref).bfloat16().float()   # the reference keeps silu(gate) * up in bf16 between the GEMMs
    return _rel(mg.marlin_w4a16_mlp(x, b, s, bd, sd, g), h @ mg.dequant_f32(bd, sd, g))


@pytest.mark.parametrize("seed,boundary", [(1, False), (2, False), (3, True), (4, True)])
def test_random_shapes_through_every_entry(seed, boundary):
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    worst = []
    for c in range(40):
        case = _one_case(rnd, boundary)
        print(f"case {c}: {case}", flush=True)   # names the case should the run end here
        err = _run_case(*case)
        torch.cuda.synchronize()
        if not err <= TOL:
            worst.append((err, case))
        torch.cuda.empty_cache()
    assert not worst, worst


OVERRIDE_K = [128, 256, 512, 1024, 4096]
OVERRIDE_N = [16, 32, 64, 128, 256]
UNITS = [1, 8, 40, 64, 104, 128, 200, 256, 304, 512]


@pytest.mark.parametrize("seed", [5, 6, 7])
def test_random_shapes_on_a_workspace_of_exactly_the_size_asked_for(seed):
    """The same through the C ABI itself, with what the wrappers never pass -- tile overrides and a count of
    compute units on the plain entry, eight adapters -- on a workspace of exactly `kiln_w4a16_*workspace_bytes`
    with a canary behind it, called twice without zeroing in between: the result, the canary, and the zeroed prefix
    that every call must leave as it found it."""
    import ctypes
    from kiln_amd import _lib
    L = _lib.load()
    rnd = random.Random(seed)
    torch.manual_seed(seed)
    stream = torch.cuda.current_stream().cuda_stream
    zeroed = L.kiln_w4a16_workspace_zeroed_bytes()
    worst = []
    for c in range(40):
        k, n = rnd.choice(MODEL_K + ANY_K), rnd.choice(MODEL_N + ANY_N)
        m = rnd.choice(BOUNDARY_M + [1, 3, 8, 14, 100, 300, 577, 900, 1100, 1700, 2048])
        while m * n * k > 1e11:
            m = max(1, m // 2)
        g = rnd.choice([128, 128, -1])
        kind = rnd.choice(["plain", "lora", "swiglu", "swiglu_lora"])
        if kind.startswith("swiglu") and n % 512 != 0:
            n += 256
        ranks = rnd.choice(RANKS + [(8,) * 8])
        scales = tuple(rnd.choice([0.5, 1.0, 2.0]) for _ in ranks)
        tk, tn, sms = rnd.choice([-1, -1] + OVERRIDE_K), rnd.choice([-1, -1] + OVERRIDE_N), rnd.choice([-1, -1] + UNITS)
        case = (kind, m, k, n, g, ranks, scales, tk, tn, sms)
        print(f"case {c}: {case}", flush=True)
        b, s = _weights(k, n, g)
        x = torch.randn(m, k, device="cuda").bfloat16()
        rt = sum(ranks)
        la = (torch.randn(rt, k, device="cuda") * 0.03).bfloat16()
        lb = (torch.randn(n, rt, device="cuda") * 0.03).bfloat16()
        ref = x.float() @ mg.dequant_f32(b, s, g)
        if kind in ("lora", "swiglu_lora"):
            o = 0
            for r, sc in zip(ranks, scales):
                ref = ref + (sc * (x.float() @ la[o:o + r].float().T)).bfloat16().float() @ lb[:, o:o + r].float().T
                o += r
        n_out = n // 2 if kind.startswith("swiglu") else n
        if kind.startswith("swiglu"):
            ref = _swiglu_of(ref)
        nbytes = (L.kiln_w4a16_workspace_bytes_tuned(m, n, k, tk, tn, sms) if kind == "plain" else
                  L.kiln_w4a16_workspace_bytes(m, n, k) if kind == "lora" else L.kiln_w4a16_swiglu_workspace_bytes(m, n_out, k))
        ws = torch.zeros(nbytes + 256, dtype=torch.uint8, device="cuda")
        ws[nbytes:] = 0x5A
        y = torch.empty(m, n_out, dtype=torch.bfloat16, device="cuda")
        cr, cs = (ctypes.c_int * len(ranks))(*ranks), (ctypes.c_float * len(ranks))(*scales)
        for _ in range(2):
            ptrs = (x.data_ptr(), b.data_ptr(), y.data_ptr(), s.data_ptr())
            lora = (la.data_ptr(), lb.data_ptr(), rt, len(ranks), cr, cs)
            if kind == "plain":
                st = L.kiln_marlin_w4a16_gemm(*ptrs, m, n, k, ws.data_ptr(), g, 0, stream, tk, tn, sms, 16)
            elif kind == "lora":
                st = L.kiln_w4a16_gemm_lora(*ptrs, m, n, k, ws.data_ptr(), g, 0, stream, *lora)
            elif kind == "swiglu":
                st = L.kiln_w4a16_gemm_swiglu(*ptrs, m, n_out, k, ws.data_ptr(), g, 0, stream)
            else:
                st = L.kiln_w4a16_gemm_swiglu_lora(*ptrs, m, n_out, k, ws.data_ptr(), g, 0, stream, *lora)
            torch.cuda.synchronize()
            if st == 2 and kind == "plain" and (tk > 0 or tn > 0):
                break   # a tile override the shape does not take (ERR_KERN_SHAPE), refused before anything ran
            err = float("nan") if st else _rel(y, ref)
            intact = bool((ws[nbytes:] == 0x5A).all()) and int(ws[:zeroed].count_nonzero()) == 0
            if not (err <= TOL and intact):
                worst.append((st, err, intact, case))
        torch.cuda.empty_cache()
    assert not worst, worst
