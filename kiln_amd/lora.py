"""LoRA on top of a packed projection: host mirror of the reference call sites.

`LoraProjectionWeights` and the `A [r, in]` / `B [out, r]` convention follow
crates/kiln-model/src/lora_loader.rs:204-232; `merge_concat` follows the stacking of
crates/kiln-model/src/adapter_merge.rs:639-712 (A row-concatenated, B column-concatenated
with each block scaled by its adapter weight); `mlp_proj_forward` / `q_proj_forward` take the
place of `mlp_proj_forward_decode_if` / `q_proj_forward_decode_if`
(crates/kiln-model/src/forward.rs:2923-2946, :4776-4801) with the delta fused into the GEMM.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from . import marlin_gemm
from .marlin_proj import MarlinPackedProj, MarlinProjError, matmul_bf16


@dataclass
class LoraProjectionWeights:
    a: torch.Tensor   # [rank, in_features]
    b: torch.Tensor   # [out_features, rank]


@dataclass
class StackedLora:
    """Several adapters for one projection, stacked along the rank axis."""
    a_cat: torch.Tensor        # [r_total, in_features] bf16
    b_cat: torch.Tensor        # [out_features, r_total] bf16
    ranks: tuple
    scales: tuple              # per-adapter scale (alpha / rank times the adapter weight)


def stack_adapters(adapters: Sequence[LoraProjectionWeights], scales: Sequence[float]) -> StackedLora:
    """Row-concatenate A and column-concatenate B; the per-adapter scale stays a number and is
    applied in f32 inside the kernel."""
    if not adapters or len(adapters) != len(scales):
        raise MarlinProjError("stack_adapters: need one scale per adapter")
    a_cat = torch.cat([p.a.to(torch.bfloat16) for p in adapters], dim=0).contiguous()
    b_cat = torch.cat([p.b.to(torch.bfloat16) for p in adapters], dim=1).contiguous()
    return StackedLora(a_cat, b_cat, tuple(int(p.a.shape[0]) for p in adapters),
                       tuple(float(s) for s in scales))


def pad_rank(stacked: StackedLora) -> StackedLora:
    """The same adapters with the stacked rank rounded up to a multiple of 8 (the last adapter gets zero rows of A
    and zero columns of B, which add exact zeros): the library's kernels with the low-rank term built in take
    stacked ranks that are multiples of 8, any other goes the general route (a call of 16 rows on the widest
    projection: 14 us against 9).  Worth doing once where adapters are loaded; the calls below do it where they
    stack per call.  Unchanged if the rank is a multiple of 8 already or would pass 64."""
    r_total = sum(stacked.ranks)
    pad = -r_total % 8
    return stacked if pad == 0 or r_total + pad > 64 else _pad_by(stacked, pad)


def _pad_by(stacked: StackedLora, pad: int) -> StackedLora:
    a_cat = torch.cat([stacked.a_cat, stacked.a_cat.new_zeros(pad, stacked.a_cat.shape[1])], dim=0).contiguous()
    b_cat = torch.cat([stacked.b_cat, stacked.b_cat.new_zeros(stacked.b_cat.shape[0], pad)], dim=1).contiguous()
    return StackedLora(a_cat, b_cat, stacked.ranks[:-1] + (stacked.ranks[-1] + pad,), stacked.scales)


def merge_concat(adapters: Sequence[LoraProjectionWeights], weights: Sequence[float]) -> LoraProjectionWeights:
    """adapter_merge.rs:639-712: one adapter of rank sum(r_i) with B_i pre-multiplied by w_i, so
    that B_cat @ A_cat == sum_i w_i * B_i @ A_i."""
    a_cat = torch.cat([p.a for p in adapters], dim=0)
    b_cat = torch.cat([p.b * w for p, w in zip(adapters, weights)], dim=1)
    return LoraProjectionWeights(a_cat, b_cat)


def proj_forward(x: torch.Tensor, packed: MarlinPackedProj, lora, lora_scale: float = 1.0) -> torch.Tensor:
    """`base = matmul_bf16(x, packed)`; with LoRA, `base + delta` in one kernel
    (forward.rs:2932-2939).  `lora` is None, a LoraProjectionWeights (scaled by `lora_scale`)
    or a StackedLora."""
    if lora is None:
        return matmul_bf16(x, packed)
    if isinstance(lora, LoraProjectionWeights):
        lora = stack_adapters([lora], [lora_scale])
    if x.dim() not in (2, 3) or x.shape[-1] != packed.k:
        raise MarlinProjError(f"marlin_proj: x last-dim {x.shape[-1]} != packed weight k {packed.k}")
    x2 = x.reshape(-1, packed.k).contiguous()
    lora = pad_rank(lora)
    y2 = marlin_gemm.marlin_w4a16_gemm_lora(x2, packed.b_packed, packed.scales, packed.groupsize,
                                            lora.a_cat, lora.b_cat, lora.ranks, lora.scales)
    return y2.reshape(*x.shape[:-1], packed.n)


def _as_stacked(lora, lora_scale: float) -> Optional[StackedLora]:
    if lora is None or isinstance(lora, StackedLora):
        return lora
    return stack_adapters([lora], [lora_scale])


def swiglu_forward(x: torch.Tensor, gate_up: MarlinPackedProj, gate_lora=None, up_lora=None,
                   lora_scale: float = 1.0) -> torch.Tensor:
    """`silu(gate_proj(x) + d_gate) * (up_proj(x) + d_up)` on the interleaved gate/up pack in one launch:
    the two `mlp_proj_forward` calls with `lora_layer.gate_proj` / `up_proj`, `silu` and the multiply of
    forward.rs:2771-2819.  `gate_lora` / `up_lora` are None, a LoraProjectionWeights (scaled by
    `lora_scale`) or a StackedLora; together at most 64 rank columns and 8 adapters."""
    if x.dim() not in (2, 3) or x.shape[-1] != gate_up.k:
        raise MarlinProjError(f"marlin_proj: x last-dim {x.shape[-1]} != packed weight k {gate_up.k}")
    n_out = gate_up.n // 2
    x2 = x.reshape(-1, gate_up.k).contiguous()
    g, u = _as_stacked(gate_lora, lora_scale), _as_stacked(up_lora, lora_scale)
    if g is None and u is None:
        h = marlin_gemm.marlin_w4a16_gemm_swiglu(x2, gate_up.b_packed, gate_up.scales, gate_up.groupsize)
        return h.reshape(*x.shape[:-1], n_out)
    # the stacked rank of both sides together a multiple of 8 (pad_rank): zero columns on the last side
    r_total = sum(sum(s.ranks) for s in (g, u) if s is not None)
    pad = -r_total % 8
    if pad and r_total + pad <= 64:
        g, u = (g, _pad_by(u, pad)) if u is not None else (_pad_by(g, pad), u)
    sides = [s for s in (g, u) if s is not None]
    a_cat = torch.cat([s.a_cat for s in sides], dim=0).contiguous()
    b_cat = marlin_gemm.interleave_gate_up_lora_b(g.b_cat if g is not None else None,
                                                  u.b_cat if u is not None else None, n_out)
    ranks = tuple(r for s in sides for r in s.ranks)
    scales = tuple(v for s in sides for v in s.scales)
    h = marlin_gemm.marlin_w4a16_gemm_swiglu_lora(x2, gate_up.b_packed, gate_up.scales, gate_up.groupsize,
                                                  a_cat, b_cat, ranks, scales)
    return h.reshape(*x.shape[:-1], n_out)


def fuse_column_blocks(loras: Sequence, widths: Sequence[int], lora_scale: float = 1.0) -> Optional[StackedLora]:
    """The adapters of projections that share their input and were packed side by side as one GEMM of
    `sum(widths)` columns (projection i owns the next `widths[i]` columns): one stacked set for that GEMM.
    The A matrices are row-concatenated as they are -- they all read the same x, so one projection of x
    onto the stacked rank axis serves every member -- and B becomes block-structured: projection i's B
    entries sit in its own rows and its own adapters' rank columns, zeros elsewhere.  `loras[i]` is None,
    a LoraProjectionWeights (scaled by `lora_scale`) or a StackedLora.  None if no member has an adapter."""
    sides = [_as_stacked(l, lora_scale) for l in loras]
    if all(s is None for s in sides):
        return None
    r_total = sum(sum(s.ranks) for s in sides if s is not None)
    ref = next(s for s in sides if s is not None)
    b_cat = torch.zeros((sum(widths), r_total), dtype=torch.bfloat16, device=ref.b_cat.device)
    row = col = 0
    for s, width in zip(sides, widths):
        if s is not None:
            if s.b_cat.shape[0] != width:
                raise MarlinProjError(f"fuse_column_blocks: adapter B has {s.b_cat.shape[0]} rows, its projection {width} columns")
            r = sum(s.ranks)
            b_cat[row:row + width, col:col + r] = s.b_cat
            col += r
        row += width
    present = [s for s in sides if s is not None]
    return StackedLora(torch.cat([s.a_cat for s in present], dim=0).contiguous(), b_cat,
                       tuple(r for s in present for r in s.ranks), tuple(v for s in present for v in s.scales))


def swiglu_lora_fits(gate_lora, up_lora) -> bool:
    """Can `swiglu_forward` take these adapters (stacked rank <= 64, <= 8 adapters)?"""
    ranks = []
    for side in (gate_lora, up_lora):
        if isinstance(side, StackedLora):
            ranks += list(side.ranks)
        elif side is not None:
            ranks.append(int(side.a.shape[0]))
    return sum(ranks) <= 64 and len(ranks) <= 8


mlp_proj_forward = proj_forward
q_proj_forward = proj_forward
