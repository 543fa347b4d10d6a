#!/usr/bin/env python3
"""Benchmark of the W4A16 GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the decode configuration the headline metric is quoted on): the two
MLP projections of a Qwen3.5-4B-class layer at M = 16 -- fused gate+up
K=2560 -> N=18432, then down K=9216 -> N=2560 -- int4 group-128 weights, fp16
scales, bf16 activations ~N(0,1).  One step = those two GEMMs for one layer.
Steps rotate over 16 layers of distinct weights (586 MB) so that the 256 MB
last-level cache cannot serve the weight stream.

The timed region replays one HIP graph holding exactly K steps, bracketed by
device synchronisation; inputs are resident in HBM.  `value` is algorithmic
bytes per step / time per step.  The roofline entry times the dominant kernel
(the gate+up GEMM) alone, the same way, with events on the launch stream.
The CPU baseline is the oracle's restatement of the reference CPU path
(dequantise, then f32 matmul), timed on the host cores on a few steps.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
GROUP = 128
LAYERS = 16
TIMED_REPLAYS = 5      # of the graph that holds the timed steps; the median replay is reported
# HBM bytes per launch of the gate+up decode kernel at M=16, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (KiB per dispatch), each scaled by what the same counter reads for a 64 MiB device
# copy (x1.9989 and x1.0): 12307.1 KiB * 1.9989 + 576.0 KiB.  Source: profiles/decode_gmp_kernel_m16_hbm_traffic.txt
# The counters cannot be read inside an untraced run, so the figure is carried as a constant -- of one
# kernel instance on one plan: where the planner picks another for the headline shape the line reports no
# traffic instead of this one.
GATE_UP_M16_TRAFFIC = {"bytes": 25780980, "kernel": "w4a16_decode_gmp_kernel<5, 3, 4, false>", "blocks": 231}
MIN_TIMED_REGION_S = 0.02   # a timed region shorter than this replays its graph several times between the events


def decode_kernel_of_plan(lib, m: int, k: int, n: int, cus: int):
    """Name and grid of the small-M kernel instance the dispatcher runs for (m, k, n), from the library's
    own plan query -- (kernel name, blocks)."""
    import ctypes
    out = (ctypes.c_int * 8)()
    if lib.kiln_w4a16_debug_decode_plan(m, n, k, cus, out) != 0:
        return "unknown", 0
    ks, gs, u, bps, waves, direct, regs, gm_tiles = list(out)
    if gm_tiles < 0:        # the private-staging instance: <tiles, groups per wavefront, LDS-direct loads per group, adapters>
        aq = 1 if m <= 4 else (2 if m <= 8 else 4)
        return f"w4a16_decode_gmp_kernel<{-gm_tiles}, {-(-gs // waves)}, {aq}, false>", bps * ks
    if gm_tiles > 0:
        return f"w4a16_decode_gm_kernel<{gm_tiles}, {-(-gs // waves)}, false>", bps * ks
    return (f"w4a16_decode_gmr_kernel (run {u})" if regs else f"w4a16_decode_kernel<{u}, {bool(direct)}>"), bps * ks


def algorithmic_bytes(m: int, k: int, n: int) -> int:
    """K*N/2 (int4) + (K/128)*N*2 (scales) + M*K*2 (A) + M*N*2 (C)."""
    return k * n // 2 + (k // GROUP) * n * 2 + m * k * 2 + m * n * 2


def other_configurations(torch, marlin_gemm, dev, make_layer, timed_graph, shapes):
    """The other benchmark configurations, reported under `extra` (not part of `value`)."""
    extra = {}
    def time_shape(m_, k_, n_, count, lora=None, n_layers=12):
        """Average time of one GEMM call over `count` graph-replayed calls rotating n_layers weights."""
        ws_ = [make_layer(k_, n_) for _ in range(n_layers)]
        x_ = torch.randn(m_, k_, device=dev).to(torch.bfloat16)
        o_ = torch.empty(m_, n_, dtype=torch.bfloat16, device=dev)
        def fn(i):
            b_, s_ = ws_[i % n_layers]
            if lora is None:
                marlin_gemm.marlin_w4a16_gemm(x_, b_, s_, GROUP, out=o_)
            else:
                marlin_gemm.marlin_w4a16_gemm_lora(x_, b_, s_, GROUP, lora[0], lora[1], lora[2], lora[3], out=o_)
        t, _ = timed_graph(fn, count)
        return t / count * 1e6

    # cfg 0: the single GEMV the reference CPU path is quoted on
    us = time_shape(1, 2560, 2560, 200, n_layers=96)
    extra["cfg0_m1_2560x2560"] = {"us": round(us, 3), "GBps": round(algorithmic_bytes(1, 2560, 2560) / us / 1e3, 1)}
    # cfg 2: chunked prefill, M = 2048 (matrix-core bound).  72 calls per replay: with 24 (5 ms) the
    # part is still settling from the light decode launches before it and reads 10 % slower
    for name, (k, n) in shapes.items():
        us = time_shape(2048, k, n, 72)
        tf = 2 * 2048 * k * n / us / 1e6
        # what a call launches: the product, and where its row sums (operand of the offset removal) come from
        from kiln_amd import _lib
        cus_ = torch.cuda.get_device_properties(dev).multi_processor_count
        src_ = _lib.load().kiln_w4a16_debug_prefill_rowsum_producers(2048, n, k, cus_)
        extra[f"cfg2_m2048_{name}"] = {"us": round(us, 2), "TFLOPs": round(tf, 1),
                                       "mfma_frac": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                                       "launches_per_call": 2 if src_ == 0 else 1,
                                       "row_sums": ("a launch in front (its time is included)" if src_ == 0 else
                                                    f"{src_} blocks of the product's own launch" if src_ > 0 else
                                                    "inside the product's blocks")}
    # cfg 4: prefill with two stacked LoRA adapters fused into the epilogue
    ranks, lscales = (16, 32), (0.5, 1.0)
    la = (torch.randn(sum(ranks), 2560, device=dev) * 0.02).to(torch.bfloat16)
    lb = (torch.randn(18432, sum(ranks), device=dev) * 0.02).to(torch.bfloat16)
    us = time_shape(512, 2560, 18432, 160, lora=(la, lb, ranks, lscales))
    fl = 2 * 512 * 2560 * 18432 + 2 * 512 * sum(ranks) * (2560 + 18432)
    extra["cfg4_m512_gate_up_lora_r16_r32"] = {"us": round(us, 2), "TFLOPs": round(fl / us / 1e6, 1),
                                               "mfma_frac": round(fl / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
    # the same adapters on a decode step's 16 rows (small-M kernels with the low-rank term)
    us = time_shape(16, 2560, 18432, 200, lora=(la, lb, ranks, lscales))
    extra["m16_gate_up_lora_r16_r32"] = {"us": round(us, 2)}
    # cfg 3: every quantised linear of a 32-layer model, one decode step, M in {1, 4, 16, 64} (and 32, which the
    # configuration does not name: the row count at which the mid-M kernel's one-row-block pass runs)
    sweep_shapes = [(2560, 8192), (4096, 2560), (2560, 18432), (9216, 2560)]
    sweep_w = [[make_layer(k, n) for (k, n) in sweep_shapes] for _ in range(32)]
    w_bytes = 32 * sum(k * n // 2 + (k // GROUP) * n * 2 for (k, n) in sweep_shapes)
    for m_sw in (1, 4, 16, 32, 64):
        xs = [torch.randn(m_sw, k, device=dev).to(torch.bfloat16) for (k, n) in sweep_shapes]
        os_ = [torch.empty(m_sw, n, dtype=torch.bfloat16, device=dev) for (k, n) in sweep_shapes]
        def sweep(_i):
            for layer in sweep_w:
                for j, (b_, s_) in enumerate(layer):
                    marlin_gemm.marlin_w4a16_gemm(xs[j], b_, s_, GROUP, out=os_[j])
        t, _ = timed_graph(sweep, 3)
        us = t / 3 * 1e6
        by = w_bytes + 32 * sum(m_sw * (k + n) * 2 for (k, n) in sweep_shapes)
        extra[f"cfg3_sweep_m{m_sw}"] = {"us_per_sweep": round(us, 1), "GBps": round(by / us / 1e3, 1),
                                        "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4), "launches": 128}
    del sweep_w

    # fused gate+up + SwiGLU epilogue against the plain GEMM of the same packed width
    from kiln_amd.marlin_gemm import marlin_w4a16_gemm_swiglu, marlin_w4a16_gemm_swiglu_lora
    sl_ranks, sl_scales = (16, 16, 16, 16), (1.0, 1.0, 1.0, 1.0)   # two adapters on gate_proj, two on up_proj
    sl_a = (torch.randn(sum(sl_ranks), 2560, device=dev) * 0.02).to(torch.bfloat16)
    sl_b = (torch.randn(18432, sum(sl_ranks), device=dev) * 0.02).to(torch.bfloat16)
    for m_sg, count in ((16, 200), (2048, 72)):
        ws_ = [make_layer(2560, 18432) for _ in range(12)]
        x_ = torch.randn(m_sg, 2560, device=dev).to(torch.bfloat16)
        o_ = torch.empty(m_sg, 9216, dtype=torch.bfloat16, device=dev)
        p_ = torch.empty(m_sg, 18432, dtype=torch.bfloat16, device=dev)
        def fn(i):
            b_, s_ = ws_[i % 12]
            marlin_w4a16_gemm_swiglu(x_, b_, s_, GROUP, out=o_)
        def fn_plain(i):
            b_, s_ = ws_[i % 12]
            marlin_gemm.marlin_w4a16_gemm(x_, b_, s_, GROUP, out=p_)
        # the plain GEMM on the same weights right next to it: at this point of the run (after the heavy
        # configurations) both read slower than the headline figure taken at the start
        def fn_lora(i):
            b_, s_ = ws_[i % 12]
            marlin_w4a16_gemm_swiglu_lora(x_, b_, s_, GROUP, sl_a, sl_b, sl_ranks, sl_scales, out=o_)
        t_plain, _ = timed_graph(fn_plain, count)
        t, _ = timed_graph(fn, count)
        t_lora, _ = timed_graph(fn_lora, count)
        extra[f"swiglu_m{m_sg}_gate_up"] = {"us": round(t / count * 1e6, 2),
                                            "plain_gemm_same_weights_us": round(t_plain / count * 1e6, 2),
                                            "with_two_lora_adapters_a_side_us": round(t_lora / count * 1e6, 2)}

    # one layer's quantised linears of a decode step at 16 rows -- in-projection, out-projection, fused gate+up
    # SwiGLU, down -- without adapters and with two stacked adapters on every projection (ranks 16 + 32; 16 + 16 on gate and on up)
    from kiln_amd.marlin_gemm import interleave_gate_up_lora_b
    lay = {"in": (2560, 8192), "out": (4096, 2560), "gate_up": (2560, 18432), "down": (9216, 2560)}
    lw = {name: [make_layer(*kn) for _ in range(8)] for name, kn in lay.items()}
    lx = {name: torch.randn(16, kn[0], device=dev).to(torch.bfloat16) for name, kn in lay.items()}
    lo_ = {name: torch.empty(16, kn[1] // (2 if name == "gate_up" else 1), dtype=torch.bfloat16, device=dev)
           for name, kn in lay.items()}
    lr, ls = (16, 32), (0.5, 1.0)
    la_ = {name: (torch.randn(sum(lr), kn[0], device=dev) * 0.02).to(torch.bfloat16) for name, kn in lay.items()}
    lb_ = {name: (torch.randn(kn[1], sum(lr), device=dev) * 0.02).to(torch.bfloat16) for name, kn in lay.items() if name != "gate_up"}
    gr, gsc = (16, 16, 16, 16), (0.5, 1.0, 0.5, 1.0)   # gate's two adapters, then up's: 64 rank columns, the fused call's limit
    gu_a = (torch.randn(sum(gr), 2560, device=dev) * 0.02).to(torch.bfloat16)
    gu_b = interleave_gate_up_lora_b((torch.randn(9216, 32, device=dev) * 0.02).to(torch.bfloat16),
                                     (torch.randn(9216, 32, device=dev) * 0.02).to(torch.bfloat16), 9216)
    def layer_plain(i):
        for name in ("in", "out"):
            marlin_gemm.marlin_w4a16_gemm(lx[name], *lw[name][i % 8], GROUP, out=lo_[name])
        marlin_w4a16_gemm_swiglu(lx["gate_up"], *lw["gate_up"][i % 8], GROUP, out=lo_["gate_up"])
        marlin_gemm.marlin_w4a16_gemm(lx["down"], *lw["down"][i % 8], GROUP, out=lo_["down"])
    def layer_lora(i):
        for name in ("in", "out"):
            marlin_gemm.marlin_w4a16_gemm_lora(lx[name], *lw[name][i % 8], GROUP, la_[name], lb_[name], lr, ls, out=lo_[name])
        marlin_w4a16_gemm_swiglu_lora(lx["gate_up"], *lw["gate_up"][i % 8], GROUP, gu_a, gu_b, gr, gsc,
                                      out=lo_["gate_up"])
        marlin_gemm.marlin_w4a16_gemm_lora(lx["down"], *lw["down"][i % 8], GROUP, la_["down"], lb_["down"], lr, ls,
                                           out=lo_["down"])
    t_p, _ = timed_graph(layer_plain, 64)
    t_l, _ = timed_graph(layer_lora, 64)
    extra["decode_layer_m16_four_linears"] = {"us": round(t_p / 64 * 1e6, 2),
                                              "with_two_lora_adapters_per_projection_us": round(t_l / 64 * 1e6, 2)}
    del lw

    # projections that read the same input, as separate launches and packed side by side as one GEMM (the columns
    # of a GEMM are independent): q | k | v of a full-attention layer, in_proj_qkv | in_proj_z of a GDN layer
    for name, widths in (("attention_qkv", (8192, 1024, 1024)), ("gdn_in_proj_qkv_z", (8192, 4096))):
        for m_f in (1, 16):
            parts = [[make_layer(2560, n_) for _ in range(8)] for n_ in widths]
            whole = [make_layer(2560, sum(widths)) for _ in range(8)]
            x_ = torch.randn(m_f, 2560, device=dev).to(torch.bfloat16)
            po = [torch.empty(m_f, n_, dtype=torch.bfloat16, device=dev) for n_ in widths]
            wo = torch.empty(m_f, sum(widths), dtype=torch.bfloat16, device=dev)
            def fn_parts(i):
                for j in range(len(widths)):
                    marlin_gemm.marlin_w4a16_gemm(x_, *parts[j][i % 8], GROUP, out=po[j])
            def fn_whole(i):
                marlin_gemm.marlin_w4a16_gemm(x_, *whole[i % 8], GROUP, out=wo)
            t_parts, _ = timed_graph(fn_parts, 64)
            t_whole, _ = timed_graph(fn_whole, 64)
            extra[f"{name}_m{m_f}"] = {"separate_launches_us": round(t_parts / 64 * 1e6, 2),
                                       "one_launch_side_by_side_us": round(t_whole / 64 * 1e6, 2)}
    # the MLP as one call (fused gate+up SwiGLU, then down: two launches)
    from kiln_amd.marlin_gemm import marlin_w4a16_mlp
    mw = [(make_layer(2560, 18432), make_layer(9216, 2560)) for _ in range(8)]
    for m_f in (1, 16):
        x_ = torch.randn(m_f, 2560, device=dev).to(torch.bfloat16)
        o_ = torch.empty(m_f, 2560, dtype=torch.bfloat16, device=dev)
        def fn_mlp(i):
            (b1, s1), (b2, s2) = mw[i % 8]
            marlin_w4a16_mlp(x_, b1, s1, b2, s2, GROUP, out=o_)
        t_mlp, _ = timed_graph(fn_mlp, 64)
        extra[f"mlp_m{m_f}_one_call_two_launches"] = {"us": round(t_mlp / 64 * 1e6, 2)}
    del mw

    # per-launch distribution and wrapper-inclusive cost of the headline GEMM (eager launches)
    ws_ = [make_layer(2560, 18432) for _ in range(16)]
    x_ = torch.randn(16, 2560, device=dev).to(torch.bfloat16)
    o_ = torch.empty(16, 18432, dtype=torch.bfloat16, device=dev)
    for i in range(50):
        marlin_gemm.marlin_w4a16_gemm(x_, ws_[i % 16][0], ws_[i % 16][1], GROUP, out=o_)
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(200)]
    t0 = time.perf_counter()
    for i, (e0, e1) in enumerate(evs):
        e0.record()
        marlin_gemm.marlin_w4a16_gemm(x_, ws_[i % 16][0], ws_[i % 16][1], GROUP, out=o_)
        e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / len(evs) * 1e6
    us = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in evs)
    extra["m16_gate_up_eager_200_launches"] = {
        "event_us_p10": round(us[20], 2), "event_us_median": round(us[100], 2), "event_us_p90": round(us[180], 2),
        "wrapper_inclusive_wall_us": round(wall, 2)}
    # host time of the C entry point alone (plan lookup + launch, no wrapper, no synchronisation):
    # 2000 back-to-back calls on one stream, wall time per call
    from kiln_amd import _lib
    L = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    wsz = L.kiln_w4a16_workspace_bytes(16, 18432, 2560)
    wbuf = torch.zeros(wsz, dtype=torch.uint8, device=dev)
    b0, s0 = ws_[0]
    for n_calls in (50, 2000):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n_calls):
            L.kiln_marlin_w4a16_gemm(x_.data_ptr(), b0.data_ptr(), o_.data_ptr(), s0.data_ptr(), 16, 18432, 2560,
                                     wbuf.data_ptr(), GROUP, 0, st, -1, -1, -1, 16)
        host = (time.perf_counter() - t0) / n_calls * 1e6
        torch.cuda.synchronize()
    extra["m16_gate_up_c_entry_host_us_per_call"] = round(host, 2)

    # quantise-and-pack of one layer's seven projections from bf16 weights in device memory (what a model load
    # does 32 times): the device route, and the reference's download / host pack / upload route on 7 of them once
    import os
    from kiln_amd import marlin_proj
    layer_shapes = [(2560, 8192), (2560, 1024), (2560, 1024), (4096, 2560), (2560, 9216), (2560, 9216), (9216, 2560)]
    layer_w = [((torch.randn(k_, n_, device=dev) * 0.02).to(torch.bfloat16), GROUP) for k_, n_ in layer_shapes]
    pack_ms = {}
    for route in ("device", "device", "host"):
        if route == "host":
            os.environ["KILN_W4A16_HOST_PACK"] = "1"
        try:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            packed = marlin_proj.pack_from_bf16_batch(layer_w)
            torch.cuda.synchronize()
            pack_ms[route] = round((time.perf_counter() - t0) * 1e3, 2)
            del packed
        finally:
            os.environ.pop("KILN_W4A16_HOST_PACK", None)
    extra["pack_one_layer_7_projections_ms"] = {"on_device": pack_ms["device"], "host_route": pack_ms["host"],
                                                 "weights_millions": round(sum(k_ * n_ for k_, n_ in layer_shapes) / 1e6, 1)}
    return extra



def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=320)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the legs reported under `extra` (every launch is then an M=16 launch of the workload)")
    ap.add_argument("--profile", choices=["decode", "decode_m1", "mid", "mid_m32", "prefill", "lora", "pack"], default=None,
                    help="for rocprofv3: launch K eager steps of the chosen regime (no graph, no CPU "
                         "baseline, no extra legs) plus one 64 MiB device copy that calibrates the "
                         "memory-traffic counters, print no JSON; prefill: the two cfg 2 GEMMs at M=2048, "
                         "K calls each in a captured graph replayed six times, as the legs under `extra` run "
                         "them; decode_m1: gate+up, down and the "
                         "2560x2560 GEMV at M=1; mid: the four projection shapes of the sweep at M=64; "
                         "lora: the decode step and the M=512 gate+up GEMM, each with two stacked "
                         "adapters (ranks 16 and 32)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the path has no multi-GPU code); "
              "run with --gpus 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch
    from kiln_amd import marlin_gemm

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    torch.manual_seed(0)

    M = 16
    shapes = {"gate_up": (2560, 18432), "down": (9216, 2560)}

    def make_layer(k, n):
        # the packed layout is opaque: uniformly random words are uniformly random codes
        b = torch.randint(-2 ** 31, 2 ** 31 - 1, (k // 16, 2 * n), dtype=torch.int32, device=dev)
        s = (torch.rand(k // GROUP, n, device=dev) * 0.018 + 0.002).to(torch.float16)
        return b, s

    layers = [{name: make_layer(*kn) for name, kn in shapes.items()} for _ in range(LAYERS)]
    x = {name: torch.randn(M, kn[0], device=dev).to(torch.bfloat16) for name, kn in shapes.items()}
    out = {name: torch.empty(M, kn[1], dtype=torch.bfloat16, device=dev) for name, kn in shapes.items()}

    def run(name, layer):
        b, s = layers[layer % LAYERS][name]
        marlin_gemm.marlin_w4a16_gemm(x[name], b, s, GROUP, out=out[name])

    def step(i):
        run("gate_up", i)
        run("down", i)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()

    if args.profile:
        src = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)                                  # reads 64 MiB, writes 64 MiB
        if args.profile == "decode":
            from kiln_amd import _lib
            cus = torch.cuda.get_device_properties(dev).multi_processor_count
            for name, kn in shapes.items():     # which instances the counters of this run belong to
                print(f"bench.py --profile decode: {name} M={M} runs %s x %d blocks" % decode_kernel_of_plan(_lib.load(), M, *kn, cus),
                      file=sys.stderr)
            for i in range(args.steps):
                step(i)
        elif args.profile == "decode_m1":
            x1 = {name: torch.randn(1, kn[0], device=dev).to(torch.bfloat16) for name, kn in shapes.items()}
            o1 = {name: torch.empty(1, kn[1], dtype=torch.bfloat16, device=dev) for name, kn in shapes.items()}
            sq = [make_layer(2560, 2560) for _ in range(LAYERS)]
            xs, os_ = torch.randn(1, 2560, device=dev).to(torch.bfloat16), torch.empty(1, 2560, dtype=torch.bfloat16, device=dev)
            for i in range(args.steps):
                for name in shapes:
                    b, s = layers[i % LAYERS][name]
                    marlin_gemm.marlin_w4a16_gemm(x1[name], b, s, GROUP, out=o1[name])
                marlin_gemm.marlin_w4a16_gemm(xs, sq[i % LAYERS][0], sq[i % LAYERS][1], GROUP, out=os_)
        elif args.profile in ("mid", "mid_m32"):
            rows = 64 if args.profile == "mid" else 32   # 32: the mid-M kernel's one-row-block pass
            sweep = {"in_proj": (2560, 8192), "out_proj": (4096, 2560), **shapes}
            sw = {name: [make_layer(*kn) for _ in range(8)] for name, kn in sweep.items() if name not in shapes}
            x64 = {name: torch.randn(rows, kn[0], device=dev).to(torch.bfloat16) for name, kn in sweep.items()}
            o64 = {name: torch.empty(rows, kn[1], dtype=torch.bfloat16, device=dev) for name, kn in sweep.items()}
            for i in range(args.steps):
                for name in sweep:
                    b, s = layers[i % LAYERS][name] if name in shapes else sw[name][i % 8]
                    marlin_gemm.marlin_w4a16_gemm(x64[name], b, s, GROUP, out=o64[name])
        elif args.profile == "pack":
            from kiln_amd.marlin_gemm import pack as kpack
            for name, kn in {"in_proj": (2560, 8192), "out_proj": (4096, 2560), **shapes}.items():
                w_ = (torch.randn(*kn, device=dev) * 0.02).to(torch.bfloat16)
                for i in range(args.steps):
                    kpack.quantize_and_pack_device(w_, GROUP)
        elif args.profile == "lora":
            ranks, lscales = (16, 32), (0.5, 1.0)
            ad = {name: ((torch.randn(sum(ranks), kn[0], device=dev) * 0.02).to(torch.bfloat16),
                         (torch.randn(kn[1], sum(ranks), device=dev) * 0.02).to(torch.bfloat16))
                  for name, kn in shapes.items()}
            x512 = torch.randn(512, 2560, device=dev).to(torch.bfloat16)
            o512 = torch.empty(512, 18432, dtype=torch.bfloat16, device=dev)
            x64 = {name: torch.randn(64, kn[0], device=dev).to(torch.bfloat16) for name, kn in shapes.items()}
            o64 = {name: torch.empty(64, kn[1], dtype=torch.bfloat16, device=dev) for name, kn in shapes.items()}
            for i in range(args.steps):
                for name in shapes:
                    b, s = layers[i % LAYERS][name]
                    marlin_gemm.marlin_w4a16_gemm_lora(x[name], b, s, GROUP, ad[name][0], ad[name][1], ranks,
                                                       lscales, out=out[name])
                for name in shapes:
                    b, s = layers[i % LAYERS][name]
                    marlin_gemm.marlin_w4a16_gemm_lora(x64[name], b, s, GROUP, ad[name][0], ad[name][1], ranks,
                                                       lscales, out=o64[name])
                b, s = layers[i % LAYERS]["gate_up"]
                marlin_gemm.marlin_w4a16_gemm_lora(x512, b, s, GROUP, ad["gate_up"][0], ad["gate_up"][1], ranks,
                                                   lscales, out=o512)
        else:
            # as the cfg 2 legs under `extra` run them: one captured graph per shape, the calls back to back,
            # replayed five times untimed (the part needs tens of milliseconds of this load to settle: the
            # first replays read up to 10 % slower) and once between events (the tracer spaces the nodes out,
            # so the figure printed here is an upper bound; the trace's durations are the kernels' own)
            xp = {name: torch.randn(2048, kn[0], device=dev).to(torch.bfloat16) for name, kn in shapes.items()}
            op = {name: torch.empty(2048, kn[1], dtype=torch.bfloat16, device=dev) for name, kn in shapes.items()}
            side = torch.cuda.Stream()
            for name in shapes:
                def call(i, name=name):
                    b, s = layers[i % LAYERS][name]
                    marlin_gemm.marlin_w4a16_gemm(xp[name], b, s, GROUP, out=op[name])
                g = torch.cuda.CUDAGraph()
                with torch.cuda.stream(side):
                    for i in range(LAYERS):
                        call(i)
                    side.synchronize()
                    with torch.cuda.graph(g, stream=side):
                        for i in range(args.steps):
                            call(i)
                    for _ in range(5):
                        g.replay()
                    side.synchronize()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(side)
                    g.replay()
                    e1.record(side)
                    side.synchronize()
                print(f"bench.py --profile prefill: {name} M=2048, {args.steps} calls per replay, sixth replay "
                      f"{e0.elapsed_time(e1) * 1e3 / args.steps:.2f} us per call between events", file=sys.stderr)
        torch.cuda.synchronize()
        return 0

    stream = torch.cuda.Stream()

    replay_log = {}

    def timed_graph(fn, count, tag=None):
        """Capture `count` calls of fn(i) into one graph; replay it untimed, then take TIMED_REPLAYS timed
        regions, each one replay between two synchronisations with HIP events on the launch stream.  Where
        `count` calls are shorter than MIN_TIMED_REGION_S the timed graph holds them several times over
        (whole passes of exactly `count` calls, back to back); returns the median region's time per pass
        (region to region the same graph reads +-3 %, the first ones after a change of workload high)."""
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            for i in range(min(count, LAYERS)):
                fn(i)                                   # allocate workspaces outside capture
            stream.synchronize()
            with torch.cuda.graph(g, stream=stream):
                for i in range(count):
                    fn(i)
            g.replay()
            stream.synchronize()

            def one_region(graph):
                e0 = torch.cuda.Event(enable_timing=True)
                e1 = torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                e0.record(stream)
                graph.replay()
                e1.record(stream)
                torch.cuda.synchronize()
                return e0.elapsed_time(e1) * 1e-3, time.perf_counter() - t0

            # sizing pass, not reported: a region shorter than MIN_TIMED_REGION_S (K = 20 steps of 15 us are
            # 0.3 ms: the clocks have not settled and the events' own cost shows) is stretched to it by a graph
            # that holds the same K calls `reps` times over, back to back, with nothing between them
            t_ev, _ = one_region(g)
            reps = max(1, min(4000 // max(count, 1), int(MIN_TIMED_REGION_S / max(t_ev, 1e-6)) + 1))
            if reps > 1:
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=stream):
                    for i in range(reps * count):
                        fn(i)
                g.replay()
                stream.synchronize()
            runs = []
            for _ in range(TIMED_REPLAYS):
                t_ev, t_wall = one_region(g)
                runs.append((t_ev / reps, t_wall / reps))
        runs.sort()
        if tag:
            replay_log[tag] = [round(t / count * 1e6, 3) for t, _ in runs]
            replay_log[tag.replace("_us_per_replay_sorted", "") + "_passes_of_k_calls_per_timed_region"] = reps
        return runs[len(runs) // 2]

    t_step, wall_step = timed_graph(step, args.steps, tag="step_us_per_replay_sorted")
    t_gu, _ = timed_graph(lambda i: run("gate_up", i), args.steps, tag="m16_gate_up_us_per_replay_sorted")
    t_dn, _ = timed_graph(lambda i: run("down", i), args.steps)

    bytes_gu = algorithmic_bytes(M, *shapes["gate_up"])
    bytes_dn = algorithmic_bytes(M, *shapes["down"])
    bytes_step = bytes_gu + bytes_dn
    sec_per_step = t_step / args.steps
    value = bytes_step / sec_per_step / 1e9
    us_gu = t_gu / args.steps * 1e6
    us_dn = t_dn / args.steps * 1e6
    achieved = bytes_gu / (us_gu * 1e-6) / 1e9

    # M = 1 on the same shapes (pure decode), reported alongside
    extra = {}
    for m_extra in (() if args.no_extra else (1,)):
        xe = {name: torch.randn(m_extra, kn[0], device=dev).to(torch.bfloat16) for name, kn in shapes.items()}
        oe = {name: torch.empty(m_extra, kn[1], dtype=torch.bfloat16, device=dev) for name, kn in shapes.items()}
        for name, kn in shapes.items():
            def fn(i, name=name):
                b, s = layers[i % LAYERS][name]
                marlin_gemm.marlin_w4a16_gemm(xe[name], b, s, GROUP, out=oe[name])
            t, _ = timed_graph(fn, args.steps)
            us = t / args.steps * 1e6
            by = algorithmic_bytes(m_extra, *kn)
            extra[f"m{m_extra}_{name}"] = {"us": round(us, 3), "GBps": round(by / us / 1e3, 1),
                                           "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4)}
    for name, us, by in (("gate_up", us_gu, bytes_gu), ("down", us_dn, bytes_dn)):
        k, n = shapes[name]
        extra[f"m{M}_{name}"] = {"us": round(us, 3), "GBps": round(by / us / 1e3, 1),
                                 "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBPS, 4),
                                 "weight_GBps": round(k * n / 2 / us / 1e3, 1),
                                 "TFLOPs": round(2 * M * k * n / us / 1e6, 2)}

    if not args.no_extra:
        extra.update(other_configurations(torch, marlin_gemm, dev, make_layer, timed_graph, shapes))
    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import ref
        rng = np.random.default_rng(0)
        host = {}
        for name, (k, n) in shapes.items():
            q = rng.integers(0, 2 ** 32, size=(k // 8, n), dtype=np.uint64).astype(np.uint32)
            sc = (rng.random((k // GROUP, n)) * 0.018 + 0.002).astype(np.float16).view(np.uint16)
            xa = ref.np_f32_to_bf16(rng.standard_normal((M, k)).astype(np.float32))
            host[name] = (xa, q, sc, np.empty((k, n), dtype=np.float32))
        def cpu_step():
            for name in shapes:
                xa, q, sc, scratch = host[name]
                ref.c_w4a16_cpu_path(xa, q, sc, GROUP, scratch=scratch)
        cpu_step()
        n_cpu, t0 = 0, time.perf_counter()
        while n_cpu < 3 or (time.perf_counter() - t0 < 10.0 and n_cpu < 200):
            cpu_step()
            n_cpu += 1
        cpu_sec = (time.perf_counter() - t0) / n_cpu
        # dequantise alone and matmul alone, gate+up, one pass each
        xa, q, sc, scratch = host["gate_up"]
        t0 = time.perf_counter()
        wf = ref.c_dequant_f32(q, sc, GROUP)
        t_deq = time.perf_counter() - t0
        t0 = time.perf_counter()
        ref.c_gemm_f32(xa, wf)
        t_mm = time.perf_counter() - t0
        del wf
        # cfg 0 (M=1, K=N=2560), the case the reference's CPU path is quoted on: median of 20 passes
        q0 = rng.integers(0, 2 ** 32, size=(2560 // 8, 2560), dtype=np.uint64).astype(np.uint32)
        s0 = (rng.random((2560 // GROUP, 2560)) * 0.018 + 0.002).astype(np.float16).view(np.uint16)
        x0 = ref.np_f32_to_bf16(rng.standard_normal((1, 2560)).astype(np.float32))
        scratch0 = np.empty((2560, 2560), dtype=np.float32)
        t_cfg0 = []
        for _ in range(21):
            t0 = time.perf_counter()
            ref.c_w4a16_cpu_path(x0, q0, s0, GROUP, scratch=scratch0)
            t_cfg0.append(time.perf_counter() - t0)
        t_cfg0 = sorted(t_cfg0[1:])[10]
        cpu_baseline = {"value": round(bytes_step / cpu_sec / 1e9, 4), "unit": "GB/s",
                        "cores": ref.num_threads(), "kind": "port",
                        "sample": f"{n_cpu} full steps (gate+up and down at M=16) of the C restatement of the "
                                  f"reference CPU path, dequantise to f32 then f32 matmul, "
                                  f"{cpu_sec * 1e3:.1f} ms per step; gate+up alone: dequantise "
                                  f"{t_deq * 1e3:.1f} ms, matmul {t_mm * 1e3:.1f} ms; "
                                  f"cfg 0 (M=1, 2560x2560) {t_cfg0 * 1e6:.0f} us per pass"}

    from kiln_amd import _lib
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    gu_kernel, gu_blocks = decode_kernel_of_plan(_lib.load(), M, *shapes["gate_up"], cus)
    traffic_known = (gu_kernel, gu_blocks) == (GATE_UP_M16_TRAFFIC["kernel"], GATE_UP_M16_TRAFFIC["blocks"])
    result = {
        "metric": "w4a16_gemm_decode_effective_bandwidth_m16",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(sec_per_step * 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "decode MLP projections, M=16: gate+up K=2560->N=18432 then down K=9216->N=2560, "
                               "int4 group-128 weights, fp16 scales, bf16 activations",
                   "m": M, "groupsize": GROUP, "layers_rotated": LAYERS,
                   "algorithmic_bytes_per_step": bytes_step,
                   "launch": "one HIP graph of whole passes of the K timed steps, back to back, replayed per timed region",
                   "passes_of_k_steps_per_timed_region": replay_log.get("step_passes_of_k_calls_per_timed_region", 1),
                   "timed_replays": TIMED_REPLAYS, "statistic": "median replay, time per pass of K steps",
                   "wall_ms_per_step": round(wall_step / args.steps * 1e3, 6)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": GATE_UP_M16_TRAFFIC["bytes"] if traffic_known else None,
                     "kernel": f"{gu_kernel} x {gu_blocks} blocks (gate+up, M=16, K=2560, N=18432)",
                     "us_per_launch": round(us_gu, 3), "algorithmic_bytes_per_launch": bytes_gu},
        "cpu_baseline": cpu_baseline,
        "extra": {**extra, **replay_log},
    }
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
