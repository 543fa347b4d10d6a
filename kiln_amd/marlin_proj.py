"""Host mirror of crates/kiln-model/src/marlin_proj.rs: packed projections for a
quantised linear layer.

Same names and contracts as the reference module: `MarlinPackedProj`
(marlin_proj.rs:38-50), `shape_is_supported` (:53-55), the three packing
phases `prepare_pack_job` / `pack_host` / `upload_packed` (:87-182),
`pack_from_bf16` (:198-207), `pack_from_bf16_batch` (:229-262), `matmul_bf16`
(:285-319), `env_enabled` (:330-338) and `parallel_pack_disabled` (:346-356).
An unsupported shape or a weight that is not on the GPU yields `None`, which
tells the caller to stay on its bf16 path, exactly as in the reference.

The entry points a model loader and forward pass use (`pack_from_bf16`,
`pack_from_bf16_batch`, `pack_from_gptq`, `matmul_bf16`, `save`, `load`, the
environment switches) run in the library's C++ host layer
(`kiln_marlin_proj_*`, include/kiln_marlin_proj.h); this module binds them and
keeps the reference's three separate phases as Python functions over the same
C quantiser.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np
import torch

import ctypes

from . import _lib, marlin_gemm


class MarlinProjError(ValueError):
    pass


class _NativeOwner:
    """Owns a `kiln_marlin_packed_proj_t`; freed when the last view of its memory is gone."""

    def __init__(self, handle: int):
        self.handle = handle

    def __del__(self):
        if self.handle:
            _lib.load().kiln_marlin_proj_free(self.handle)
            self.handle = 0


class _DeviceView:
    """Device memory of a native projection, exposed through the array interface torch reads."""

    def __init__(self, owner: _NativeOwner, ptr: int, shape, typestr: str):
        self.owner = owner
        self.__cuda_array_interface__ = {"shape": tuple(shape), "typestr": typestr, "data": (ptr, False),
                                         "version": 2, "strides": None}


@dataclass
class MarlinPackedProj:
    """marlin_proj.rs:38-50"""
    b_packed: torch.Tensor   # [k/16, n*16/8] int32, tile layout
    scales: torch.Tensor     # [k/groupsize, n] float16, tile layout
    groupsize: int           # -1 (per column) or 128
    k: int
    n: int
    native: Optional[_NativeOwner] = None   # set when the C++ layer owns the memory


def _raise_last():
    raise MarlinProjError(_lib.load().kiln_marlin_proj_last_error().decode())


def _wrap_native(handle: int, device: torch.device) -> MarlinPackedProj:
    L = _lib.load()
    owner = _NativeOwner(handle)
    k, n, g = L.kiln_marlin_proj_k(handle), L.kiln_marlin_proj_n(handle), L.kiln_marlin_proj_groupsize(handle)
    groups = 1 if g == -1 else k // g
    b = torch.as_tensor(_DeviceView(owner, L.kiln_marlin_proj_b_packed(handle), (k // 16, n * 16 // 8), "<i4"),
                        device=device)
    s = torch.as_tensor(_DeviceView(owner, L.kiln_marlin_proj_scales(handle), (groups, n), "<f2"), device=device)
    return MarlinPackedProj(b, s, g, k, n, owner)


def _device_index(t: torch.Tensor) -> int:
    if not t.is_cuda:
        return -1
    return t.device.index if t.device.index is not None else torch.cuda.current_device()


@dataclass
class PackJobHost:
    """marlin_proj.rs:63-69"""
    host_weight: np.ndarray  # [k, n] row-major f32
    k: int
    n: int
    groupsize: int


@dataclass
class PackedHost:
    """marlin_proj.rs:74-80"""
    b_packed_vec: np.ndarray
    scales_vec: np.ndarray
    k: int
    n: int
    groupsize: int


def shape_is_supported(k: int, n: int) -> bool:
    return bool(_lib.load().kiln_marlin_proj_shape_is_supported(k, n))


def prepare_pack_job(weight_t: torch.Tensor, groupsize: int) -> Optional[PackJobHost]:
    """Phase 1 (marlin_proj.rs:87-124): validate, widen to f32 on the device, download."""
    if not weight_t.is_cuda:
        return None
    if weight_t.dim() != 2:
        raise MarlinProjError("marlin_proj: weight_t must be a 2D [k, n] tensor")
    k, n = weight_t.shape
    if not shape_is_supported(k, n):
        return None
    if not (groupsize == -1 or groupsize == 128):
        raise MarlinProjError(f"marlin_proj: groupsize must be -1 or 128 (got {groupsize})")
    host = weight_t.to(torch.float32).contiguous().cpu().numpy()
    return PackJobHost(host, k, n, groupsize)


def pack_host(job: PackJobHost) -> PackedHost:
    """Phase 2 (marlin_proj.rs:130-144): pure CPU, safe to run from any worker thread."""
    b, s, _ = marlin_gemm.quantize_and_pack(job.host_weight, job.k, job.n, job.groupsize,
                                            want_dequant=False)
    return PackedHost(b, s, job.k, job.n, job.groupsize)


def upload_packed(packed: PackedHost, device: torch.device) -> MarlinPackedProj:
    """Phase 3 (marlin_proj.rs:150-182)."""
    num_groups = 1 if packed.groupsize == -1 else packed.k // packed.groupsize
    b = torch.from_numpy(packed.b_packed_vec).reshape(packed.k // 16, packed.n * 16 // 8).to(device)
    s = torch.from_numpy(packed.scales_vec).reshape(num_groups, packed.n).to(device)
    return MarlinPackedProj(b, s, packed.groupsize, packed.k, packed.n)


def pack_from_bf16(weight_t: torch.Tensor, groupsize: int) -> Optional[MarlinPackedProj]:
    """marlin_proj.rs:198-207: `[k, n] = [in, out]` bf16 weight -> packed projection."""
    if weight_t.dim() != 2:
        raise MarlinProjError("marlin_proj: weight_t must be a 2D [k, n] tensor")
    if weight_t.is_cuda and weight_t.dtype != torch.bfloat16:
        weight_t = weight_t.to(torch.bfloat16)
    w = weight_t.contiguous()
    torch.cuda.synchronize() if w.is_cuda else None
    out = ctypes.c_void_p()
    st = _lib.load().kiln_marlin_proj_pack_from_bf16(w.data_ptr() if w.is_cuda else None, w.shape[0], w.shape[1],
                                                   groupsize, _device_index(w), ctypes.byref(out))
    if st == _lib.PROJ_SKIPPED:
        return None
    if st != _lib.PROJ_OK:
        _raise_last()
    return _wrap_native(out.value, w.device)


def pack_from_bf16_batch(inputs: Sequence[tuple[torch.Tensor, int]]) -> list[Optional[MarlinPackedProj]]:
    """marlin_proj.rs:229-262: serial download, parallel CPU pack, serial upload; order kept."""
    if not inputs:
        return []
    device = inputs[0][0].device
    ws = []
    for t, _ in inputs:
        if t.dim() != 2:
            raise MarlinProjError("marlin_proj: weight_t must be a 2D [k, n] tensor")
        ws.append((t.to(torch.bfloat16) if t.is_cuda else t).contiguous())
    if device.type == "cuda":
        torch.cuda.synchronize()
    count = len(ws)
    ptrs = (ctypes.c_void_p * count)(*[w.data_ptr() if w.is_cuda else None for w in ws])
    ks = (ctypes.c_int64 * count)(*[w.shape[0] for w in ws])
    ns = (ctypes.c_int64 * count)(*[w.shape[1] for w in ws])
    gs = (ctypes.c_int * count)(*[g for _, g in inputs])
    outs = (ctypes.c_void_p * count)()
    st = _lib.load().kiln_marlin_proj_pack_from_bf16_batch(ptrs, ks, ns, gs, count, _device_index(ws[0]), outs)
    if st not in (_lib.PROJ_OK, _lib.PROJ_SKIPPED):
        _raise_last()
    return [None if not h else _wrap_native(h, device) for h in outs]


def pack_from_gptq(qweight: torch.Tensor, scales: torch.Tensor, qzeros: Optional[torch.Tensor],
                   groupsize: int, device: torch.device) -> Optional[MarlinPackedProj]:
    """Offline-repack entry: GPTQ-canonical tensors (quantized.rs:1-14) -> packed projection.
    The reference has no such path (it dequantises GPTQ to bf16 and re-quantises)."""
    k, n = qweight.shape[0] * 8, qweight.shape[1]
    device = torch.device(device)
    q = np.ascontiguousarray(qweight.cpu().numpy().view(np.int32))
    s = np.ascontiguousarray(scales.cpu().numpy().view(np.uint16))
    z = None if qzeros is None else np.ascontiguousarray(qzeros.cpu().numpy().view(np.int32))
    out = ctypes.c_void_p()
    dev = -1 if device.type != "cuda" else (device.index if device.index is not None else torch.cuda.current_device())
    st = _lib.load().kiln_marlin_proj_pack_from_gptq(q.ctypes.data, s.ctypes.data, None if z is None else z.ctypes.data,
                                                   k, n, groupsize, dev, ctypes.byref(out))
    if st == _lib.PROJ_SKIPPED:
        return None
    if st != _lib.PROJ_OK:
        _raise_last()
    return _wrap_native(out.value, device)


def matmul_bf16(x: torch.Tensor, w: MarlinPackedProj) -> torch.Tensor:
    """marlin_proj.rs:285-319: `[m, k]` or `[batch, seq, k]` bf16 -> same rank, last dim n."""
    rank = x.dim()
    if w.native is None or rank not in (2, 3):
        return _matmul_bf16_py(x, w)
    x = x.contiguous()
    dims = (ctypes.c_int64 * rank)(*x.shape)
    m = x.numel() // x.shape[-1] if x.shape[-1] else 0
    y = torch.empty(*x.shape[:-1], w.n, dtype=torch.bfloat16, device=x.device)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    L = _lib.load()
    nbytes = L.kiln_w4a16_workspace_bytes(m, w.n, w.k)
    ws = marlin_gemm._workspace(x.device, stream, nbytes)
    st = L.kiln_marlin_proj_matmul_bf16(w.native.handle, x.data_ptr(), dims, rank, y.data_ptr(), ws.data_ptr(),
                                        ws.numel(), stream)
    if st != _lib.PROJ_OK:
        _raise_last()
    return y


def _matmul_bf16_py(x: torch.Tensor, w: MarlinPackedProj) -> torch.Tensor:
    rank = x.dim()
    if rank == 2:
        m, k = x.shape
        if k != w.k:
            raise MarlinProjError(f"marlin_proj: x last-dim {k} != packed weight k {w.k}")
        return marlin_gemm.marlin_w4a16_gemm(x.contiguous(), w.b_packed, w.scales, w.groupsize)
    if rank == 3:
        batch, seq, k = x.shape
        if k != w.k:
            raise MarlinProjError(f"marlin_proj: x last-dim {k} != packed weight k {w.k}")
        x2 = x.reshape(batch * seq, k).contiguous()
        y2 = marlin_gemm.marlin_w4a16_gemm(x2, w.b_packed, w.scales, w.groupsize)
        return y2.reshape(batch, seq, w.n)
    raise MarlinProjError(f"marlin_proj: unsupported activation rank {rank}")


def save(w: MarlinPackedProj, path: str) -> None:
    """Persist a packed projection (header with k, n, groupsize, layout version, checksum + body)."""
    L = _lib.load()
    if w.native is not None:
        st = L.kiln_marlin_proj_save(w.native.handle, str(path).encode())
    else:
        b = np.ascontiguousarray(w.b_packed.cpu().numpy())
        s = np.ascontiguousarray(w.scales.cpu().numpy().view(np.uint16))
        st = L.kiln_w4a16_artifact_write(str(path).encode(), b.ctypes.data, s.ctypes.data, w.k, w.n, w.groupsize)
    if st != _lib.PROJ_OK:
        _raise_last()


def load(path: str, device: torch.device) -> MarlinPackedProj:
    """Load a persisted packed projection onto `device`; a file of another layout version or with a
    bad checksum is an error."""
    device = torch.device(device)
    out = ctypes.c_void_p()
    dev = device.index if device.index is not None else torch.cuda.current_device()
    st = _lib.load().kiln_marlin_proj_load(str(path).encode(), dev, ctypes.byref(out))
    if st != _lib.PROJ_OK:
        _raise_last()
    return _wrap_native(out.value, device)


def env_enabled() -> bool:
    """`KILN_W4A16` (marlin_proj.rs:330-338)."""
    return bool(_lib.load().kiln_marlin_proj_env_enabled())


def parallel_pack_disabled() -> bool:
    """`KILN_DISABLE_PARALLEL_PACK` (marlin_proj.rs:346-356)."""
    return bool(_lib.load().kiln_marlin_proj_parallel_pack_disabled())


def bf16_drop_disabled() -> bool:
    """`KILN_DISABLE_MARLIN_BF16_DROP` in {1, true, yes} (forward.rs:1565-1580)."""
    return bool(_lib.load().kiln_marlin_proj_bf16_drop_disabled())
