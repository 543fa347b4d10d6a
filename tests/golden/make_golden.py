"""Writes tests/golden/w4a16_small.npz: inputs and expected outputs of the CPU oracle
for a few small problems (the reference stores no vectors for this path, so these are
regression vectors of the oracle; the first two use the reference test's LCG seeds,
parity.rs:55-56; the third covers M >= 33, stacked LoRA adapters and silu(gate) * up).  Run from the repo root:  python tests/golden/make_golden.py
"""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
from oracle import ref  # noqa: E402

out = {}
for tag, (m, k, n, g) in {"g128": (4, 256, 256, 128), "col": (3, 256, 256, -1)}.items():
    w = ref.c_lcg_fill(k * n, 0xC0FFEE5EED ^ k ^ (n << 16), 0.5).reshape(k, n)
    acts = ref.c_lcg_fill(m * k, 0xDEADBEEF ^ m ^ (k << 24), 0.25).reshape(m, k)
    codes, s_bits, deq = ref.c_quantize(w, g)
    q = ref.c_pack_gptq(codes)
    x = ref.np_f32_to_bf16(acts)
    y = ref.c_w4a16_cpu_path(x, q, s_bits, g)
    out.update({f"{tag}_qweight": q, f"{tag}_scales_f16": s_bits, f"{tag}_x_bf16": x,
                f"{tag}_y_f32": y, f"{tag}_y_bf16": ref.np_f32_to_bf16(y),
                f"{tag}_dequant_rows": deq[[0, 1, 127, 128, 255]],
                f"{tag}_w_head": w[:2, :8].copy()})

# the matrix-core kernel (M >= 33), the fused LoRA epilogue and the fused SwiGLU epilogue
m, k, n, g = 40, 256, 256, 128
codes_gate, codes_up = ref.gen_codes(k, n, seed=11), ref.gen_codes(k, n, seed=12)
s_gate, s_up = ref.gen_scales_f16(k, n, g, seed=11), ref.gen_scales_f16(k, n, g, seed=12)
q_gate, q_up = ref.np_pack_gptq(codes_gate), ref.np_pack_gptq(codes_up)
x = ref.gen_normal_bf16(m, k, 1.0, seed=13)
y_gate = ref.c_w4a16_cpu_path(x, q_gate, s_gate, g)
y_up = ref.c_w4a16_cpu_path(x, q_up, s_up, g)
lora_a = [ref.gen_normal_bf16(r, k, 0.05, seed=20 + i) for i, r in enumerate((4, 8))]
lora_b = [ref.gen_normal_bf16(n, r, 0.05, seed=30 + i) for i, r in enumerate((4, 8))]
y_lora = y_gate.copy()
for a_i, b_i, sc in zip(lora_a, lora_b, (0.5, 2.0)):
    ref.c_lora_delta_add(y_lora, x, a_i, b_i, sc)
out.update({"pf_x_bf16": x, "pf_gate_qweight": q_gate, "pf_gate_scales_f16": s_gate,
            "pf_up_qweight": q_up, "pf_up_scales_f16": s_up,
            "pf_gate_y_f32": y_gate, "pf_up_y_f32": y_up,
            "pf_lora_a4": lora_a[0], "pf_lora_a8": lora_a[1], "pf_lora_b4": lora_b[0], "pf_lora_b8": lora_b[1],
            "pf_lora_y_f32": y_lora, "pf_swiglu_h_f32": ref.c_swiglu_f32(y_gate, y_up),
            # silu(gate + its two adapters' deltas) * up: the fused gate+up call with adapters on gate_proj
            "pf_swiglu_lora_h_f32": ref.c_swiglu_f32(y_lora, y_up)})
np.savez_compressed(Path(__file__).with_name("w4a16_small.npz"), **out)
print({k_: v.shape for k_, v in out.items()})
