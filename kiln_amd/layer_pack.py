"""Host mirror of the reference's load-time wiring of packed projections, widened to every
quantisable linear of a layer.

The reference queues only `q_proj` and the three MLP projections for the post-loop batch pack
(crates/kiln-model/src/forward.rs:1884-1890, :2002-2018: `MarlinPackKind`, `MarlinPackEntry`),
installs each packed weight into its `*_marlin` slot and drops the bf16 copy
(`install_marlin_packed`, forward.rs:1736-1771), and leaves `k/v/o_proj` and the GDN
projections on bf16 (forward.rs:1909-1980 builds them without a packed slot).  Here the same
queue / batch pack / install sequence takes every projection of both layer kinds:

    full attention   q_proj, k_proj, v_proj, o_proj
    linear attention in_proj_qkv, in_proj_z, out_proj, in_proj_a, in_proj_b
    MLP              gate_proj, up_proj, down_proj  (optionally gate and up as one fused,
                     interleaved pack for the SwiGLU entry point)

`shape_is_supported` (marlin_proj.rs:53-55) decides per projection: the 32-column
`in_proj_a` / `in_proj_b` come back unpacked and stay on bf16, exactly the `None` the reference's
`pack_from_bf16_batch` returns for an unsupported shape (marlin_proj.rs:229-262).  At run time
`LayerProjections.forward` is what `mlp_proj_forward_decode_if` / `q_proj_forward_decode_if`
(forward.rs:2923-2946, :4776-4801) are to the reference: packed GEMM where a packed weight is
installed (with the LoRA delta fused when an adapter is attached), bf16 matmul otherwise.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import marlin_gemm, marlin_proj
from .lora import fuse_column_blocks, proj_forward, swiglu_forward, swiglu_lora_fits
from .marlin_proj import MarlinPackedProj, MarlinProjError


class PackKind(Enum):
    """`MarlinPackKind` (forward.rs:1720-1725) plus the projections the reference leaves on bf16."""
    QProj = "q_proj"
    KProj = "k_proj"
    VProj = "v_proj"
    OProj = "o_proj"
    InProjQkv = "in_proj_qkv"
    InProjZ = "in_proj_z"
    OutProj = "out_proj"
    InProjA = "in_proj_a"
    InProjB = "in_proj_b"
    GateProj = "gate_proj"
    UpProj = "up_proj"
    DownProj = "down_proj"


FULL_ATTENTION_KINDS = (PackKind.QProj, PackKind.KProj, PackKind.VProj, PackKind.OProj)
LINEAR_ATTENTION_KINDS = (PackKind.InProjQkv, PackKind.InProjZ, PackKind.OutProj, PackKind.InProjA, PackKind.InProjB)
MLP_KINDS = (PackKind.GateProj, PackKind.UpProj, PackKind.DownProj)
# Projections of a layer that read the same input: packed side by side they are one GEMM -- the columns of a
# GEMM are independent of each other -- and one launch instead of three or two per decode step
# (the reference calls them one after the other: forward.rs:372 `full_attn_qkv_proj_decode_if`, and the GDN
# block's in-projections).  A launch of this size costs 3...5 us whatever its width.
SAME_INPUT_GROUPS = ((PackKind.QProj, PackKind.KProj, PackKind.VProj), (PackKind.InProjQkv, PackKind.InProjZ))
# what the reference itself queues (forward.rs:1884-1890, 2002-2018)
REFERENCE_KINDS = (PackKind.QProj, PackKind.GateProj, PackKind.UpProj, PackKind.DownProj)


@dataclass
class PackEntry:
    """`MarlinPackEntry` (forward.rs:1727-1731)."""
    layer_idx: int
    kind: PackKind


@dataclass
class LayerProjections:
    """One layer's projections: `weights_t[kind]` is the pre-transposed `[k, n]` bf16 weight (the
    reference's `*_proj_t`), `packed[kind]` the installed packed weight (its `*_proj_marlin`)."""
    weights_t: Dict[PackKind, Optional[torch.Tensor]]
    packed: Dict[PackKind, MarlinPackedProj] = field(default_factory=dict)
    gate_up_fused: Optional[MarlinPackedProj] = None   # gate and up interleaved for the SwiGLU entry point
    same_input_fused: Dict[Tuple[PackKind, ...], MarlinPackedProj] = field(default_factory=dict)   # see SAME_INPUT_GROUPS

    def is_packed(self, kind: PackKind) -> bool:
        return kind in self.packed

    def forward(self, kind: PackKind, x: torch.Tensor, lora=None, lora_scale: float = 1.0) -> torch.Tensor:
        """Packed GEMM (LoRA delta fused) where a packed weight is installed, bf16 matmul otherwise
        (forward.rs:2923-2946, :4776-4801)."""
        w = self.packed.get(kind)
        if w is not None:
            return proj_forward(x, w, lora, lora_scale)
        w_t = self.weights_t.get(kind)
        if w_t is None:
            raise MarlinProjError(f"layer_pack: {kind.value} has neither a packed nor a bf16 weight")
        y = x @ w_t
        if lora is not None:                                  # unfused, as the reference's bf16 branch
            y = y + ((x @ lora.a.t().to(x.dtype)) @ lora.b.t().to(x.dtype)) * lora_scale
        return y

    def forward_same_input(self, kinds: Sequence[PackKind], x: torch.Tensor, loras: Optional[Dict[PackKind, object]] = None,
                           lora_scale: float = 1.0) -> Tuple[torch.Tensor, ...]:
        """The projections `kinds` of one input: one launch on their side-by-side pack where `pack_layers`
        built it (the results are column ranges of one output tensor), else one `forward` each.  `loras`
        maps a kind to its adapter(s); on the fused pack they become one stacked set whose projection of x
        is computed once for all members (stacked rank <= 64 and <= 8 adapters, else the members run
        one by one)."""
        kinds = tuple(kinds)
        loras = loras or {}
        fused = self.same_input_fused.get(kinds)
        stacked = None
        if fused is not None and any(loras.get(k) is not None for k in kinds):
            widths = [self.packed[k].n for k in kinds]
            stacked = fuse_column_blocks([loras.get(k) for k in kinds], widths, lora_scale)
            if sum(stacked.ranks) > 64 or len(stacked.ranks) > 8:
                fused = None
        if fused is None:
            return tuple(self.forward(k, x, loras.get(k), lora_scale) for k in kinds)
        y = proj_forward(x, fused, stacked)
        outs, col = [], 0
        for k in kinds:
            n = self.packed[k].n
            outs.append(y[..., col:col + n])
            col += n
        return tuple(outs)

    def swiglu(self, x: torch.Tensor, gate_lora=None, up_lora=None, lora_scale: float = 1.0) -> torch.Tensor:
        """`silu(gate_proj(x)) * up_proj(x)`, each projection with its LoRA delta (forward.rs:2771-2819):
        one fused launch on the interleaved pack when it is installed and the adapters fit it (stacked
        rank <= 64), otherwise two projections and the elementwise ops."""
        if self.gate_up_fused is not None and swiglu_lora_fits(gate_lora, up_lora):
            return swiglu_forward(x, self.gate_up_fused, gate_lora, up_lora, lora_scale)
        gate = self.forward(PackKind.GateProj, x, gate_lora, lora_scale)
        up = self.forward(PackKind.UpProj, x, up_lora, lora_scale)
        return torch.nn.functional.silu(gate) * up


def queue_layer(layer_idx: int, layer: LayerProjections, kinds: Optional[Sequence[PackKind]] = None,
                groupsize: int = 128) -> Tuple[List[Tuple[torch.Tensor, int]], List[PackEntry]]:
    """The per-layer part of the reference's build loop (forward.rs:1884-1890, 2002-2018): one pack
    input and one sidecar entry per projection the layer has.  `kinds` = None queues every
    projection; `REFERENCE_KINDS` reproduces the reference's own selection."""
    inputs, meta = [], []
    for kind, w_t in layer.weights_t.items():
        if w_t is None or (kinds is not None and kind not in kinds):
            continue
        inputs.append((w_t, groupsize))
        meta.append(PackEntry(layer_idx, kind))
    return inputs, meta


def install_packed(layer: LayerProjections, kind: PackKind, packed: MarlinPackedProj,
                   drop_bf16: Optional[bool] = None) -> None:
    """`install_marlin_packed` (forward.rs:1736-1771): the packed weight goes into its slot and the
    bf16 copy is dropped -- unless the caller says otherwise or, with `drop_bf16` left at None, the
    environment does (`KILN_DISABLE_MARLIN_BF16_DROP`, forward.rs:1565-1580)."""
    if drop_bf16 is None:
        drop_bf16 = not marlin_proj.bf16_drop_disabled()
    layer.packed[kind] = packed
    if drop_bf16:
        layer.weights_t[kind] = None


def fuse_same_input(layer: LayerProjections) -> int:
    """Pack the members of every group of SAME_INPUT_GROUPS that the layer has packed (same k, same
    groupsize) side by side as one projection.  In the tile layout a packed weight is a sequence of column
    tiles, each with all of its K, and so are its scales: side by side is one after the other."""
    built = 0
    for kinds in SAME_INPUT_GROUPS:
        members = [layer.packed.get(k) for k in kinds]
        if any(p is None for p in members):
            continue
        k, g = members[0].k, members[0].groupsize
        if any(p.k != k or p.groupsize != g for p in members):
            continue
        n = sum(p.n for p in members)
        b = torch.cat([p.b_packed.reshape(-1) for p in members]).reshape(k // 16, 2 * n)
        s = torch.cat([p.scales.reshape(-1) for p in members]).reshape(-1, n)
        layer.same_input_fused[tuple(kinds)] = MarlinPackedProj(b, s, g, k, n)
        built += 1
    return built


def pack_layers(layers: Sequence[LayerProjections], kinds: Optional[Sequence[PackKind]] = None,
                groupsize: int = 128, drop_bf16: Optional[bool] = None, fuse_gate_up: bool = False,
                fuse_same_input_groups: bool = False) -> Dict[str, int]:
    """The post-loop batch pack and install (forward.rs:2040-2085): every queued projection goes
    through `pack_from_bf16_batch` (serial copies, threaded host pack); a projection whose shape the
    kernels do not take (`shape_is_supported`, e.g. the 32-column `in_proj_a` / `in_proj_b`) comes
    back as None and keeps its bf16 weight.  With `fuse_gate_up`, gate and up of a layer are also
    interleaved into one pack for the SwiGLU entry point; with `fuse_same_input_groups`, q/k/v and the GDN
    block's two wide in-projections are also packed side by side as one projection each
    (`forward_same_input`).  Returns counts for the caller's log line."""
    inputs: List[Tuple[torch.Tensor, int]] = []
    meta: List[PackEntry] = []
    for i, layer in enumerate(layers):
        li, lm = queue_layer(i, layer, kinds, groupsize)
        inputs += li
        meta += lm
    packed = marlin_proj.pack_from_bf16_batch(inputs)
    n_packed = 0
    for entry, p in zip(meta, packed):
        if p is not None:
            install_packed(layers[entry.layer_idx], entry.kind, p, drop_bf16)
            n_packed += 1
    n_fused = 0
    if fuse_gate_up:
        for layer in layers:
            g, u = layer.packed.get(PackKind.GateProj), layer.packed.get(PackKind.UpProj)
            if g is None or u is None or g.k != u.k or g.n != u.n or g.n % 128 != 0:
                continue
            b_gu, s_gu = marlin_gemm.interleave_gate_up_device(g.b_packed, g.scales, u.b_packed, u.scales, g.groupsize)
            layer.gate_up_fused = MarlinPackedProj(b_gu, s_gu, g.groupsize, g.k, 2 * g.n)
            n_fused += 1
    stats = {"inputs": len(inputs), "packed": n_packed, "kept_bf16": len(inputs) - n_packed, "gate_up_fused": n_fused}
    if fuse_same_input_groups:
        stats["same_input_fused"] = sum(fuse_same_input(layer) for layer in layers)
    return stats
