"""Host mirror of the reference crate `kiln-marlin-gemm` (crates/kiln-marlin-gemm/src/lib.rs).

`marlin_w4a16_gemm` keeps the reference's argument meaning, checks and error
texts (lib.rs:97-166); `pack` keeps `MAX_Q`, `Q_OFFSET` and
`quantize_and_pack` (lib.rs:284-491).  What differs is behind the C ABI: the
activations stay bf16 (no fp16 round trip, lib.rs:169,269), and `b_packed` /
`scales` hold the tile layout instead of the Marlin permutation.  torch only
provides device memory and the stream handle.
"""
from __future__ import annotations

import ctypes
from types import SimpleNamespace

import numpy as np
import torch

from . import _lib


class MarlinGemmError(ValueError):
    """What `candle_core::bail!` is to the reference wrapper."""


def _bail(msg: str):
    raise MarlinGemmError(f"kiln-marlin-gemm: {msg}")


# One workspace per (device, stream): only its counter prefix must be zero on first use and the
# kernels leave it zero on exit, so it is allocated once, grown when a larger call comes, and
# never cleared again.
_workspaces: dict[tuple[int, int], torch.Tensor] = {}


def _workspace(device: torch.device, stream_ptr: int, nbytes: int) -> torch.Tensor:
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_ptr)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        ws[:_lib.load().kiln_w4a16_workspace_zeroed_bytes()].zero_()
        _workspaces[key] = ws
    return ws


def workspace_wait_status(device: torch.device | None = None) -> int:
    """OR of the sticky words of every workspace this module holds on `device` (all devices if None):
    0 unless a bounded wait inside some launch gave up (`_lib.WAIT_*` says which kind).  Synchronises
    the streams involved; meant for a health check once per step or per request, not per GEMM."""
    import ctypes
    lib, bits = _lib.load(), 0
    for (dev_index, stream_ptr), ws in list(_workspaces.items()):
        if device is not None and device.index is not None and device.index != dev_index:
            continue
        word = ctypes.c_uint32(0)
        with torch.cuda.device(dev_index):
            st = lib.kiln_w4a16_workspace_check(ws.data_ptr(), ctypes.byref(word), stream_ptr)
            if st != 0:
                raise MarlinGemmError(f"kiln_w4a16_workspace_check: {_lib.status_string(st)}")
            torch.cuda.synchronize(dev_index)
        bits |= word.value
    return bits


def workspace_reset(device: torch.device | None = None) -> None:
    """Zero the prefix (sticky word included) of every workspace this module holds on `device`: what a
    caller does after `workspace_wait_status` came back non-zero and the device has drained."""
    lib = _lib.load()
    for (dev_index, stream_ptr), ws in list(_workspaces.items()):
        if device is not None and device.index is not None and device.index != dev_index:
            continue
        with torch.cuda.device(dev_index):
            torch.cuda.synchronize(dev_index)
            st = lib.kiln_w4a16_workspace_reset(ws.data_ptr(), stream_ptr)
            if st != 0:
                raise MarlinGemmError(f"kiln_w4a16_workspace_reset: {_lib.status_string(st)}")
            torch.cuda.synchronize(dev_index)


def _check_gemm_args(a, b_packed, scales, groupsize):
    """lib.rs:103-166, same order, same texts."""
    if not a.is_cuda:
        _bail("a must be on CUDA")
    if a.dim() != 2 or b_packed.dim() != 2 or scales.dim() != 2:
        _bail("a, b_packed and scales must be 2-D")
    m, k = a.shape
    b_rows, b_cols = b_packed.shape
    s_rows, n = scales.shape
    if k % 128 != 0:
        _bail(f"k must be a multiple of 128 (got {k})")
    if n % 256 != 0:
        _bail(f"n must be a multiple of 256 (got {n})")
    if b_rows != k // 16 or b_cols != n * 16 // 8:
        _bail(f"b_packed shape [{b_rows}, {b_cols}] does not match expected "
              f"[k/16={k // 16}, n*16/8={n * 16 // 8}] for k={k}, n={n}")
    if not (groupsize == -1 or groupsize == 128):
        _bail(f"groupsize must be -1 or 128 (got {groupsize})")
    g = k if groupsize == -1 else groupsize
    if g > k or k % g != 0:
        _bail(f"k={k} must be divisible by groupsize={groupsize}")
    if s_rows != k // g:
        _bail(f"scales rows {s_rows} != expected {k // g} (k={k}, groupsize={groupsize})")
    if a.dtype != torch.bfloat16:
        _bail(f"a must be bf16 (got {a.dtype})")
    if b_packed.dtype != torch.int32:
        _bail(f"b_packed must be i32 (got {b_packed.dtype})")
    if scales.dtype != torch.float16:
        _bail(f"scales must be f16 (got {scales.dtype})")
    if not b_packed.is_cuda:
        _bail("b_packed must be on CUDA")
    if not scales.is_cuda:
        _bail("scales must be on CUDA")
    return m, k, n


def marlin_w4a16_gemm(a: torch.Tensor, b_packed: torch.Tensor, scales: torch.Tensor,
                      groupsize: int, *, thread_k: int = -1, thread_n: int = -1,
                      out: torch.Tensor | None = None) -> torch.Tensor:
    """`[m, k] bf16 @ dequant([k/16, 2n] i32, [k/g, n] f16) -> [m, n] bf16` (lib.rs:97-102).

    `thread_k` / `thread_n` are the tile overrides of the C entry point
    (the reference wrapper always passes -1, lib.rs:252-253).
    """
    m, k, n = _check_gemm_args(a, b_packed, scales, groupsize)
    lib = _lib.load()
    a = a.contiguous()
    b_packed = b_packed.contiguous()
    scales = scales.contiguous()
    if out is None:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
    if m == 0:
        return out
    with torch.cuda.device(a.device):
        stream = torch.cuda.current_stream(a.device).cuda_stream
        if thread_k > 0 or thread_n > 0:
            nbytes = lib.kiln_w4a16_workspace_bytes_tuned(m, n, k, thread_k, thread_n, -1)
        else:
            nbytes = lib.kiln_w4a16_workspace_bytes(m, n, k)
        ws = _workspace(a.device, stream, nbytes)
        status = lib.kiln_marlin_w4a16_gemm(
            a.data_ptr(), b_packed.data_ptr(), out.data_ptr(), scales.data_ptr(), m, n, k,
            ws.data_ptr(), groupsize, a.device.index or 0, stream, thread_k, thread_n, -1, 16)
    if status != 0:
        raise MarlinGemmError(
            f"kiln_marlin_w4a16_gemm failed with status {status} "
            f"(1=ERR_PROB_SHAPE, 2=ERR_KERN_SHAPE) for m={m}, n={n}, k={k}, groupsize={groupsize}")
    return out


def dequant_f32(b_packed: torch.Tensor, scales: torch.Tensor, groupsize: int) -> torch.Tensor:
    """Device-side `(code - 8) * scale` of a packed weight -> `[k, n]` f32."""
    k, n = b_packed.shape[0] * 16, b_packed.shape[1] // 2
    lib = _lib.load()
    out = torch.empty((k, n), dtype=torch.float32, device=b_packed.device)
    with torch.cuda.device(b_packed.device):
        stream = torch.cuda.current_stream(b_packed.device).cuda_stream
        status = lib.kiln_w4a16_dequant_f32(b_packed.data_ptr(), scales.data_ptr(), k, n, groupsize,
                                            out.data_ptr(), b_packed.device.index or 0, stream)
    if status != 0:
        raise MarlinGemmError(f"kiln_w4a16_dequant_f32 failed: {_lib.status_string(status)}")
    return out


# ---------------------------------------------------------------------------
# pack namespace (lib.rs:284-529)
# ---------------------------------------------------------------------------

MAX_Q = 15     # lib.rs:288
Q_OFFSET = 8   # lib.rs:289


def _vp(arr: np.ndarray | None):
    return None if arr is None else arr.ctypes.data_as(ctypes.c_void_p)


def quantize_and_pack(weight, k: int, n: int, groupsize: int, want_dequant: bool = True):
    """`(&[f32] [k, n], k, n, groupsize) -> (b_packed, scales_f16, dequant)` (lib.rs:370-375).

    Returns numpy arrays shaped as the reference's callers reshape them
    (marlin_proj.rs:163-174): int32 `[k/16, 2n]`, float16 `[k/g, n]`, float32 `[k, n]`.
    """
    weight = np.ascontiguousarray(weight, dtype=np.float32).reshape(-1)
    if weight.size != k * n:
        raise AssertionError(f"weight has {weight.size} elements, expected k*n={k * n}")
    if k % 128 != 0:
        raise AssertionError("k must be %128 == 0")          # lib.rs:377
    if n % 256 != 0:
        raise AssertionError("n must be %256 == 0")          # lib.rs:378
    if not (groupsize == -1 or groupsize == 128):
        raise AssertionError(f"groupsize must be -1 or 128 (got {groupsize})")
    g = k if groupsize == -1 else groupsize
    b_packed = np.empty((k // 16, n * 2), dtype=np.int32)
    scales = np.empty((k // g, n), dtype=np.float16)
    dequant = np.empty((k, n), dtype=np.float32) if want_dequant else None
    st = _lib.load().kiln_w4a16_quantize_and_pack(_vp(weight), k, n, groupsize, _vp(b_packed),
                                                  _vp(scales), _vp(dequant))
    if st != 0:
        raise MarlinGemmError(f"kiln_w4a16_quantize_and_pack: {_lib.status_string(st)}")
    return b_packed, scales, dequant


def quantize_and_pack_device(weight_t: torch.Tensor, groupsize: int):
    """`quantize_and_pack` for a bf16 `[k, n]` weight that is already on the GPU: the same quantiser
    (lib.rs:393-427) run there, the same bits out -- `(b_packed int32 [k/16, 2n], scales f16 [k/g, n])`
    as CUDA tensors -- without the download, host pack and upload of marlin_proj.rs:86-181."""
    if weight_t.dim() != 2 or weight_t.dtype != torch.bfloat16 or not weight_t.is_cuda:
        _bail("weight_t must be a 2D [k, n] bf16 CUDA tensor")
    k, n = weight_t.shape
    if k % 128 != 0 or n % 256 != 0 or not (groupsize == -1 or groupsize == 128):
        _bail(f"unsupported shape k={k} n={n} groupsize={groupsize} (k % 128, n % 256, groupsize -1 or 128)")
    weight_t = weight_t.contiguous()
    g = k if groupsize == -1 else groupsize
    b_packed = torch.empty((k // 16, 2 * n), dtype=torch.int32, device=weight_t.device)
    scales = torch.empty((k // g, n), dtype=torch.float16, device=weight_t.device)
    with torch.cuda.device(weight_t.device):
        stream = torch.cuda.current_stream(weight_t.device).cuda_stream
        st = _lib.load().kiln_w4a16_quantize_and_pack_device(weight_t.data_ptr(), k, n, groupsize, b_packed.data_ptr(),
                                                             scales.data_ptr(), weight_t.device.index or 0, stream)
    if st != 0:
        raise MarlinGemmError(f"kiln_w4a16_quantize_and_pack_device: {_lib.status_string(st)}")
    return b_packed, scales


def repack_gptq(qweight, scales_f16, qzeros=None, groupsize: int = 128):
    """One-time repack of GPTQ-canonical tensors (`qweight [k/8, n]` int32, `scales [k/g, n]`
    f16, optional `qzeros [k/g, n/8]`; quantized.rs:1-14) into the tile layout."""
    qweight = np.ascontiguousarray(qweight).view(np.int32)
    k, n = qweight.shape[0] * 8, qweight.shape[1]
    scales_f16 = np.ascontiguousarray(scales_f16).view(np.float16)
    g = k if groupsize == -1 else groupsize
    if scales_f16.shape != (k // g, n):
        raise MarlinGemmError(f"kiln-marlin-gemm: scales shape {scales_f16.shape} != {(k // g, n)}")
    qz = None if qzeros is None else np.ascontiguousarray(qzeros).view(np.int32)
    b_packed = np.empty((k // 16, n * 2), dtype=np.int32)
    s_tiled = np.empty((k // g, n), dtype=np.float16)
    st = _lib.load().kiln_w4a16_repack_gptq(_vp(qweight), _vp(scales_f16), _vp(qz), k, n, groupsize,
                                            _vp(b_packed), _vp(s_tiled))
    if st != 0:
        raise MarlinGemmError(f"kiln_w4a16_repack_gptq: {_lib.status_string(st)}")
    return b_packed, s_tiled


def unpack_to_gptq(b_packed, scales_tiled, groupsize: int = 128):
    """Inverse of `repack_gptq`."""
    b_packed = np.ascontiguousarray(b_packed).view(np.int32)
    k, n = b_packed.shape[0] * 16, b_packed.shape[1] // 2
    scales_tiled = np.ascontiguousarray(scales_tiled).view(np.float16)
    g = k if groupsize == -1 else groupsize
    qweight = np.empty((k // 8, n), dtype=np.int32)
    scales = np.empty((k // g, n), dtype=np.float16)
    st = _lib.load().kiln_w4a16_unpack_to_gptq(_vp(b_packed), _vp(scales_tiled), k, n, groupsize,
                                               _vp(qweight), _vp(scales))
    if st != 0:
        raise MarlinGemmError(f"kiln_w4a16_unpack_to_gptq: {_lib.status_string(st)}")
    return qweight, scales


def interleave_gate_up(gate_b, gate_s, up_b, up_s, groupsize: int = 128):
    """Two packed projections of equal shape `[k, n_each]` (gate, up) -> the packed `[k, 2 n_each]`
    form `marlin_w4a16_gemm_swiglu` reads: per 16 columns (one column tile), 8 gate columns then
    the 8 matching up columns."""
    gate_b = np.ascontiguousarray(gate_b).view(np.int32)
    up_b = np.ascontiguousarray(up_b).view(np.int32)
    gate_s = np.ascontiguousarray(gate_s).view(np.float16)
    up_s = np.ascontiguousarray(up_s).view(np.float16)
    if gate_b.shape != up_b.shape or gate_s.shape != up_s.shape:
        raise MarlinGemmError("kiln-marlin-gemm: gate and up must have the same packed shapes")
    k, n_each = gate_b.shape[0] * 16, gate_b.shape[1] // 2
    out_b = np.empty((k // 16, 4 * n_each), dtype=np.int32)
    out_s = np.empty((gate_s.shape[0], 2 * n_each), dtype=np.float16)
    st = _lib.load().kiln_w4a16_interleave_gate_up(_vp(gate_b), _vp(gate_s), _vp(up_b), _vp(up_s), k, n_each,
                                                   groupsize, _vp(out_b), _vp(out_s))
    if st != 0:
        raise MarlinGemmError(f"kiln_w4a16_interleave_gate_up: {_lib.status_string(st)}")
    return out_b, out_s


def repack_gptq_device(qweight: torch.Tensor, scales_f16: torch.Tensor, qzeros: torch.Tensor | None = None,
                       groupsize: int = 128):
    """`repack_gptq` for GPTQ tensors that are CUDA tensors (`qweight [k/8, n]` int32, `scales [k/g, n]` f16,
    optional `qzeros [k/g, n/8]` int32): the same packed words and scales, formed on the GPU."""
    if not (qweight.is_cuda and scales_f16.is_cuda) or qweight.dtype != torch.int32 or scales_f16.dtype != torch.float16:
        _bail("repack_gptq_device takes CUDA tensors: int32 qweight, float16 scales")
    k, n = qweight.shape[0] * 8, qweight.shape[1]
    g = k if groupsize == -1 else groupsize
    if tuple(scales_f16.shape) != (k // g, n):
        _bail(f"scales must be [{k // g}, {n}]")
    if qzeros is not None and (not qzeros.is_cuda or qzeros.dtype != torch.int32 or tuple(qzeros.shape) != (k // g, n // 8)):
        _bail(f"qzeros must be a CUDA int32 [{k // g}, {n // 8}] tensor")
    qweight, scales_f16 = qweight.contiguous(), scales_f16.contiguous()
    qzeros = qzeros.contiguous() if qzeros is not None else None
    b_packed = torch.empty((k // 16, 2 * n), dtype=torch.int32, device=qweight.device)
    scales = torch.empty((k // g, n), dtype=torch.float16, device=qweight.device)
    with torch.cuda.device(qweight.device):
        stream = torch.cuda.current_stream(qweight.device).cuda_stream
        st = _lib.load().kiln_w4a16_repack_gptq_device(qweight.data_ptr(), scales_f16.data_ptr(),
                                                       qzeros.data_ptr() if qzeros is not None else None, k, n, groupsize,
                                                       b_packed.data_ptr(), scales.data_ptr(), qweight.device.index or 0, stream)
    if st != 0:
        raise MarlinGemmError(f"kiln_w4a16_repack_gptq_device: {_lib.status_string(st)}")
    return b_packed, scales


def interleave_gate_up_device(gate_b: torch.Tensor, gate_s: torch.Tensor, up_b: torch.Tensor, up_s: torch.Tensor,
                              groupsize: int = 128):
    """`interleave_gate_up` for packed projections that are CUDA tensors: one copy kernel, same bits."""
    for t in (gate_b, gate_s, up_b, up_s):
        if not t.is_cuda:
            _bail("interleave_gate_up_device takes CUDA tensors")
    if gate_b.shape != up_b.shape or gate_s.shape != up_s.shape or gate_b.dtype != torch.int32 or \
            up_b.dtype != torch.int32 or gate_s.dtype != torch.float16 or up_s.dtype != torch.float16:
        _bail("kiln-marlin-gemm: gate and up must have the same packed shapes (int32 words, fp16 scales)")
    k, n_each = gate_b.shape[0] * 16, gate_b.shape[1] // 2
    gate_b, gate_s, up_b, up_s = gate_b.contiguous(), gate_s.contiguous(), up_b.contiguous(), up_s.contiguous()
    out_b = torch.empty((k // 16, 4 * n_each), dtype=torch.int32, device=gate_b.device)
    out_s = torch.empty((gate_s.shape[0], 2 * n_each), dtype=torch.float16, device=gate_b.device)
    with torch.cuda.device(gate_b.device):
        stream = torch.cuda.current_stream(gate_b.device).cuda_stream
        st = _lib.load().kiln_w4a16_interleave_gate_up_device(gate_b.data_ptr(), gate_s.data_ptr(), up_b.data_ptr(),
                                                              up_s.data_ptr(), k, n_each, groupsize, out_b.data_ptr(),
                                                              out_s.data_ptr(), gate_b.device.index or 0, stream)
    if st != 0:
        raise MarlinGemmError(f"kiln_w4a16_interleave_gate_up_device: {_lib.status_string(st)}")
    return out_b, out_s


pack = SimpleNamespace(MAX_Q=MAX_Q, Q_OFFSET=Q_OFFSET, quantize_and_pack=quantize_and_pack,
                       interleave_gate_up_device=interleave_gate_up_device, repack_gptq_device=repack_gptq_device,
                       quantize_and_pack_device=quantize_and_pack_device,
                       repack_gptq=repack_gptq, unpack_to_gptq=unpack_to_gptq,
                       interleave_gate_up=interleave_gate_up)


def marlin_w4a16_gemm_swiglu(a: torch.Tensor, b_packed: torch.Tensor, scales: torch.Tensor, groupsize: int,
                             *, out: torch.Tensor | None = None) -> torch.Tensor:
    """`silu(gate) * up` with `[gate | up] = a @ dequant(b_packed)`: `[m, k]` bf16 -> `[m, n_out]`
    bf16, `b_packed` / `scales` from `pack.interleave_gate_up` (`2 n_out` packed columns).

    Fused form of the gate GEMM, up GEMM, silu and multiply the reference issues separately
    (crates/kiln-model/src/forward.rs:2771-2819).
    """
    m, k, n = _check_gemm_args(a, b_packed, scales, groupsize)
    if n % 256 != 0:
        _bail(f"fused gate+up width {n} must be a multiple of 256")
    n_out = n // 2
    lib = _lib.load()
    a, b_packed, scales = a.contiguous(), b_packed.contiguous(), scales.contiguous()
    if out is None:
        out = torch.empty((m, n_out), dtype=torch.bfloat16, device=a.device)
    if m == 0:
        return out
    with torch.cuda.device(a.device):
        stream = torch.cuda.current_stream(a.device).cuda_stream
        ws = _workspace(a.device, stream, lib.kiln_w4a16_swiglu_workspace_bytes(m, n_out, k))
        status = lib.kiln_w4a16_gemm_swiglu(a.data_ptr(), b_packed.data_ptr(), out.data_ptr(), scales.data_ptr(),
                                            m, n_out, k, ws.data_ptr(), groupsize, a.device.index or 0, stream)
    if status != 0:
        raise MarlinGemmError(f"kiln_w4a16_gemm_swiglu failed with status {status}: "
                              f"{_lib.status_string(status)} (m={m}, n_out={n_out}, k={k})")
    return out


def marlin_w4a16_mlp(x: torch.Tensor, b_gate_up: torch.Tensor, s_gate_up: torch.Tensor, b_down: torch.Tensor,
                     s_down: torch.Tensor, groupsize: int, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """`down(silu(gate(x)) * up(x))`: `[m, hidden]` bf16 -> `[m, n_down]` bf16, the whole MLP of a layer
    (crates/kiln-model/src/forward.rs:2723-2848) as one call: the fused gate+up SwiGLU GEMM, then the down
    GEMM, `silu(gate) * up` kept in the workspace between them.
    `b_gate_up` / `s_gate_up` from `pack.interleave_gate_up`, `b_down` / `s_down` the packed down projection."""
    m, k, n = _check_gemm_args(x, b_gate_up, s_gate_up, groupsize)
    if n % 256 != 0:
        _bail(f"fused gate+up width {n} must be a multiple of 256")
    n_out = n // 2
    if b_down.dim() != 2 or s_down.dim() != 2 or b_down.shape[0] * 16 != n_out:
        _bail(f"down projection must be packed for k = {n_out} (b_down is {tuple(b_down.shape)})")
    n_down = s_down.shape[1]
    groups = 1 if groupsize == -1 else n_out // 128
    if n_down % 256 != 0 or b_down.shape[1] != 2 * n_down or s_down.shape[0] != groups:
        _bail(f"down projection: b_down {tuple(b_down.shape)} / s_down {tuple(s_down.shape)} do not match k = {n_out}")
    if b_down.dtype != torch.int32 or s_down.dtype != torch.float16 or not (b_down.is_cuda and s_down.is_cuda):
        _bail("down projection: b_down must be int32 and s_down float16, both on CUDA")
    lib = _lib.load()
    x, b_gate_up, s_gate_up = x.contiguous(), b_gate_up.contiguous(), s_gate_up.contiguous()
    b_down, s_down = b_down.contiguous(), s_down.contiguous()
    if out is None:
        out = torch.empty((m, n_down), dtype=torch.bfloat16, device=x.device)
    if m == 0:
        return out
    with torch.cuda.device(x.device):
        stream = torch.cuda.current_stream(x.device).cuda_stream
        ws = _workspace(x.device, stream, lib.kiln_w4a16_mlp_workspace_bytes(m, k, n_out, n_down))
        status = lib.kiln_w4a16_mlp(x.data_ptr(), b_gate_up.data_ptr(), s_gate_up.data_ptr(), b_down.data_ptr(),
                                    s_down.data_ptr(), out.data_ptr(), m, k, n_out, n_down, ws.data_ptr(), groupsize,
                                    x.device.index or 0, stream)
    if status != 0:
        raise MarlinGemmError(f"kiln_w4a16_mlp failed with status {status}: {_lib.status_string(status)} "
                              f"(m={m}, hidden={k}, n_out={n_out}, n_down={n_down})")
    return out


def marlin_w4a16_gemm_lora(a: torch.Tensor, b_packed: torch.Tensor, scales: torch.Tensor,
                           groupsize: int, lora_a: torch.Tensor, lora_b: torch.Tensor,
                           ranks, lora_scales, *, out: torch.Tensor | None = None) -> torch.Tensor:
    """`a @ dequant(b_packed) + sum_i s_i * (a @ A_i^T) @ B_i^T`, rounded to bf16 once.

    Fused form of what the reference computes as `base + compute_lora_delta(x, proj, scale)`
    (crates/kiln-model/src/forward.rs:2932-2939, lora_loader.rs:213-232).
    `lora_a` is `[r_total, k]` (adapter A matrices stacked along rows), `lora_b` is
    `[n, r_total]` (B matrices stacked along columns), both bf16; `ranks` / `lora_scales`
    give each adapter's rank and scale.
    """
    m, k, n = _check_gemm_args(a, b_packed, scales, groupsize)
    ranks = [int(r) for r in ranks]
    lora_scales = [float(v) for v in lora_scales]
    r_total = sum(ranks)
    if len(ranks) != len(lora_scales) or not ranks:
        _bail("ranks and lora_scales must be non-empty and of equal length")
    if tuple(lora_a.shape) != (r_total, k) or tuple(lora_b.shape) != (n, r_total):
        _bail(f"LoRA shapes {tuple(lora_a.shape)} / {tuple(lora_b.shape)} do not match "
              f"[r_total={r_total}, k={k}] / [n={n}, r_total={r_total}]")
    if lora_a.dtype != torch.bfloat16 or lora_b.dtype != torch.bfloat16:
        _bail("LoRA matrices must be bf16")
    if not (lora_a.is_cuda and lora_b.is_cuda):
        _bail("LoRA matrices must be on CUDA")
    lib = _lib.load()
    a, b_packed, scales = a.contiguous(), b_packed.contiguous(), scales.contiguous()
    lora_a, lora_b = lora_a.contiguous(), lora_b.contiguous()
    if out is None:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=a.device)
    if m == 0:
        return out
    c_ranks = (ctypes.c_int * len(ranks))(*ranks)
    c_scales = (ctypes.c_float * len(ranks))(*lora_scales)
    with torch.cuda.device(a.device):
        stream = torch.cuda.current_stream(a.device).cuda_stream
        ws = _workspace(a.device, stream, lib.kiln_w4a16_workspace_bytes(m, n, k))
        status = lib.kiln_w4a16_gemm_lora(
            a.data_ptr(), b_packed.data_ptr(), out.data_ptr(), scales.data_ptr(), m, n, k,
            ws.data_ptr(), groupsize, a.device.index or 0, stream, lora_a.data_ptr(),
            lora_b.data_ptr(), r_total, len(ranks), c_ranks, c_scales)
    if status != 0:
        raise MarlinGemmError(f"kiln_w4a16_gemm_lora failed with status {status}: "
                              f"{_lib.status_string(status)} (m={m}, n={n}, k={k}, r_total={r_total})")
    return out


def interleave_gate_up_lora_b(gate_b: torch.Tensor | None, up_b: torch.Tensor | None, n_out: int) -> torch.Tensor:
    """The stacked `lora_b` `marlin_w4a16_gemm_swiglu_lora` reads, from gate's `[n_out, r_gate]` and up's
    `[n_out, r_up]` column-concatenated B matrices (either may be None: no adapter on that projection):
    `[2 n_out, r_gate + r_up]`, rows in the packed column order of `pack.interleave_gate_up` (per 16
    rows 8 gate columns, then the 8 matching up columns); a gate row is `[B_gate row | 0]`, an up row
    `[0 | B_up row]`."""
    ref = gate_b if gate_b is not None else up_b
    if ref is None:
        _bail("at least one of gate's and up's LoRA B matrices is needed")
    if n_out % 8 != 0:
        _bail(f"n_out {n_out} must be a multiple of 8")
    r_gate = 0 if gate_b is None else gate_b.shape[1]
    r_up = 0 if up_b is None else up_b.shape[1]
    for b in (gate_b, up_b):
        if b is not None and (b.dim() != 2 or b.shape[0] != n_out or b.dtype != torch.bfloat16):
            _bail(f"LoRA B matrices must be bf16 [n_out={n_out}, rank]")
    out = torch.zeros((n_out // 8, 2, 8, r_gate + r_up), dtype=torch.bfloat16, device=ref.device)
    if gate_b is not None:
        out[:, 0, :, :r_gate] = gate_b.reshape(n_out // 8, 8, r_gate)
    if up_b is not None:
        out[:, 1, :, r_gate:] = up_b.reshape(n_out // 8, 8, r_up)
    return out.reshape(2 * n_out, r_gate + r_up)


def marlin_w4a16_gemm_swiglu_lora(a: torch.Tensor, b_packed: torch.Tensor, scales: torch.Tensor, groupsize: int,
                                  lora_a: torch.Tensor, lora_b: torch.Tensor, ranks, lora_scales,
                                  *, out: torch.Tensor | None = None) -> torch.Tensor:
    """`silu(gate + d_gate) * (up + d_up)`: `marlin_w4a16_gemm_swiglu` with LoRA adapters on gate_proj and
    up_proj, the deltas added to the f32 sums before the product is formed and rounded once.

    Fused form of the two `mlp_proj_forward` calls with `lora_layer.gate_proj` / `up_proj`, `silu` and the
    multiply (crates/kiln-model/src/forward.rs:2771-2819).  `lora_a` is `[r_total, k]` (gate's adapters,
    then up's, stacked along rows), `lora_b` `[2 n_out, r_total]` from `interleave_gate_up_lora_b`;
    `ranks` / `lora_scales` one entry per stacked adapter.
    """
    m, k, n = _check_gemm_args(a, b_packed, scales, groupsize)
    if n % 256 != 0:
        _bail(f"fused gate+up width {n} must be a multiple of 256")
    n_out = n // 2
    ranks = [int(r) for r in ranks]
    lora_scales = [float(v) for v in lora_scales]
    r_total = sum(ranks)
    if len(ranks) != len(lora_scales) or not ranks:
        _bail("ranks and lora_scales must be non-empty and of equal length")
    if tuple(lora_a.shape) != (r_total, k) or tuple(lora_b.shape) != (n, r_total):
        _bail(f"LoRA shapes {tuple(lora_a.shape)} / {tuple(lora_b.shape)} do not match "
              f"[r_total={r_total}, k={k}] / [2 n_out={n}, r_total={r_total}]")
    if lora_a.dtype != torch.bfloat16 or lora_b.dtype != torch.bfloat16:
        _bail("LoRA matrices must be bf16")
    if not (lora_a.is_cuda and lora_b.is_cuda):
        _bail("LoRA matrices must be on CUDA")
    lib = _lib.load()
    a, b_packed, scales = a.contiguous(), b_packed.contiguous(), scales.contiguous()
    lora_a, lora_b = lora_a.contiguous(), lora_b.contiguous()
    if out is None:
        out = torch.empty((m, n_out), dtype=torch.bfloat16, device=a.device)
    if m == 0:
        return out
    c_ranks = (ctypes.c_int * len(ranks))(*ranks)
    c_scales = (ctypes.c_float * len(ranks))(*lora_scales)
    with torch.cuda.device(a.device):
        stream = torch.cuda.current_stream(a.device).cuda_stream
        ws = _workspace(a.device, stream, lib.kiln_w4a16_swiglu_workspace_bytes(m, n_out, k))
        status = lib.kiln_w4a16_gemm_swiglu_lora(
            a.data_ptr(), b_packed.data_ptr(), out.data_ptr(), scales.data_ptr(), m, n_out, k,
            ws.data_ptr(), groupsize, a.device.index or 0, stream, lora_a.data_ptr(),
            lora_b.data_ptr(), r_total, len(ranks), c_ranks, c_scales)
    if status != 0:
        raise MarlinGemmError(f"kiln_w4a16_gemm_swiglu_lora failed with status {status}: "
                              f"{_lib.status_string(status)} (m={m}, n_out={n_out}, k={k}, r_total={r_total})")
    return out
