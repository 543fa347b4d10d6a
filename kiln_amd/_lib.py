"""ctypes binding of libkiln_marlin_gemm.so (declared in include/kiln_w4a16.h).

The library is loaded from kiln_amd/lib/ only.  A missing library is an error:
there is no CPU or eager fallback for the GEMM.
"""
from __future__ import annotations

import ctypes
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libkiln_marlin_gemm.so"

# every symbol include/kiln_w4a16.h declares
EXPORTS = (
    "kiln_marlin_w4a16_gemm",
    "kiln_w4a16_workspace_bytes",
    "kiln_w4a16_workspace_bytes_tuned",
    "kiln_w4a16_workspace_zeroed_bytes",
    "kiln_w4a16_workspace_error_offset",
    "kiln_w4a16_workspace_check",
    "kiln_w4a16_workspace_reset",
    "kiln_marlin_w4a16_gemm_static_scratch",
    "kiln_w4a16_gemm_lora",
    "kiln_w4a16_gemm_swiglu",
    "kiln_w4a16_swiglu_workspace_bytes",
    "kiln_w4a16_gemm_swiglu_lora",
    "kiln_w4a16_mlp",
    "kiln_w4a16_mlp_workspace_bytes",
    "kiln_w4a16_quantize_and_pack_device",
    "kiln_w4a16_interleave_gate_up_device",
    "kiln_w4a16_repack_gptq_device",
    "kiln_w4a16_interleave_gate_up",
    "kiln_w4a16_dequant_f32",
    "kiln_w4a16_quantize_and_pack",
    "kiln_w4a16_repack_gptq",
    "kiln_w4a16_unpack_to_gptq",
    "kiln_w4a16_status_string",
    "kiln_w4a16_layout_version",
    "kiln_w4a16_debug_gemm_plan",
    "kiln_w4a16_debug_decode_plan",
    "kiln_w4a16_debug_prefill_rowsum_producers",
)

# every symbol include/kiln_marlin_proj.h declares
PROJ_EXPORTS = (
    "kiln_marlin_proj_shape_is_supported",
    "kiln_marlin_proj_env_enabled",
    "kiln_marlin_proj_parallel_pack_disabled",
    "kiln_marlin_proj_bf16_drop_disabled",
    "kiln_marlin_proj_pack_from_bf16",
    "kiln_marlin_proj_pack_from_bf16_batch",
    "kiln_marlin_proj_pack_from_gptq",
    "kiln_marlin_proj_matmul_bf16",
    "kiln_marlin_proj_k",
    "kiln_marlin_proj_n",
    "kiln_marlin_proj_groupsize",
    "kiln_marlin_proj_b_packed",
    "kiln_marlin_proj_scales",
    "kiln_marlin_proj_free",
    "kiln_marlin_proj_last_error",
    "kiln_w4a16_artifact_write",
    "kiln_w4a16_artifact_info",
    "kiln_w4a16_artifact_read",
    "kiln_marlin_proj_save",
    "kiln_marlin_proj_load",
)

PROJ_OK, PROJ_SKIPPED, PROJ_ERR = 0, 1, -1

STATIC_SCRATCH_BYTES = 8 << 20   # KILN_W4A16_STATIC_SCRATCH_BYTES

OK, ERR_PROB_SHAPE, ERR_KERN_SHAPE, ERR_LAUNCH, ERR_ARGUMENT, ERR_ZERO_POINT, ERR_SCRATCH = range(7)
# bits of the workspace's sticky word (KILN_W4A16_WAIT_*): which bounded wait gave up
WAIT_DECODE_EXCHANGE, WAIT_MID_EXCHANGE, WAIT_DECODE_FOLD, WAIT_MID_FOLD, WAIT_PREFILL_FOLD = 1, 2, 4, 8, 16

# The tuning build: the same sources with -DKILN_W4A16_TUNING_HOOKS, which adds process-wide
# overrides of the automatic plan (kiln_w4a16_debug_*).  Tests and profiling scripts that pin a
# kernel instance load it; the shipped library has no such state.
TUNING_LIB_PATH = LIB_PATH.with_name("libkiln_marlin_gemm_tuning.so")

TUNING_EXPORTS = (
    "kiln_w4a16_debug_prefill_min_m", "kiln_w4a16_debug_prefill_ks", "kiln_w4a16_debug_prefill_bn",
    "kiln_w4a16_debug_prefill_bm", "kiln_w4a16_debug_prefill_nb_full", "kiln_w4a16_debug_decode_direct_max_m",
    "kiln_w4a16_debug_decode_group_major", "kiln_w4a16_debug_decode_runs_per_launch", "kiln_w4a16_debug_tune",
    "kiln_w4a16_debug_mid", "kiln_w4a16_debug_gmp", "kiln_w4a16_debug_flagged", "kiln_w4a16_debug_lora_fold",
    "kiln_w4a16_debug_rowsum_fold", "kiln_w4a16_debug_mid_waves",
)

_libs: dict[bool, ctypes.CDLL] = {}
_active_tuning = False


class LibraryMissing(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """The library the wrappers call: the shipped one unless `load_tuning()` made the tuning build active."""
    return _load(_active_tuning)


def load_tuning() -> ctypes.CDLL:
    """Load the tuning build and make it the library the wrappers call until `use_shipped()`."""
    global _active_tuning
    L = _load(True)
    _active_tuning = True
    return L


def use_shipped() -> None:
    """Back to the shipped library, with every override of the tuning build reset."""
    global _active_tuning
    if _active_tuning:
        L = _libs[True]
        L.kiln_w4a16_debug_tune(0, 0, 0)
        L.kiln_w4a16_debug_prefill_min_m(0)
        L.kiln_w4a16_debug_prefill_ks(0)
        L.kiln_w4a16_debug_prefill_bn(0)
        L.kiln_w4a16_debug_prefill_bm(0)
        L.kiln_w4a16_debug_prefill_nb_full(-1)
        L.kiln_w4a16_debug_decode_direct_max_m(-1)
        L.kiln_w4a16_debug_decode_group_major(-1)
        L.kiln_w4a16_debug_decode_runs_per_launch(0)
        L.kiln_w4a16_debug_mid(-1, 0, 0)
        L.kiln_w4a16_debug_gmp(0, 0, 0)
        L.kiln_w4a16_debug_flagged(-1)
        L.kiln_w4a16_debug_lora_fold(-1)
        L.kiln_w4a16_debug_rowsum_fold(-1)
        L.kiln_w4a16_debug_mid_waves(0)
    _active_tuning = False


def _load(tuning: bool) -> ctypes.CDLL:
    if tuning in _libs:
        return _libs[tuning]
    path = TUNING_LIB_PATH if tuning else LIB_PATH
    if not path.exists():
        raise LibraryMissing(
            f"kiln-marlin-gemm: {path} is not built; run `python -m kiln_amd.build` "
            "(needs hipcc). There is no fallback path.")
    L = ctypes.CDLL(str(path))
    if tuning:
        for name in TUNING_EXPORTS:
            fn = getattr(L, name)
            fn.restype = None
            fn.argtypes = [ctypes.c_int] * (3 if name in ("kiln_w4a16_debug_tune", "kiln_w4a16_debug_mid", "kiln_w4a16_debug_gmp") else 1)

    c = ctypes
    vp, i = c.c_void_p, c.c_int
    L.kiln_marlin_w4a16_gemm.restype = i
    L.kiln_marlin_w4a16_gemm.argtypes = [vp, vp, vp, vp, i, i, i, vp, i, i, vp, i, i, i, i]
    L.kiln_w4a16_workspace_bytes.restype = c.c_size_t
    L.kiln_w4a16_workspace_bytes.argtypes = [i, i, i]
    L.kiln_w4a16_workspace_bytes_tuned.restype = c.c_size_t
    L.kiln_w4a16_workspace_bytes_tuned.argtypes = [i, i, i, i, i, i]
    L.kiln_w4a16_workspace_zeroed_bytes.restype = c.c_size_t
    L.kiln_w4a16_workspace_zeroed_bytes.argtypes = []
    L.kiln_w4a16_workspace_error_offset.restype = c.c_size_t
    L.kiln_w4a16_workspace_error_offset.argtypes = []
    L.kiln_w4a16_workspace_check.restype = i
    L.kiln_w4a16_workspace_check.argtypes = [vp, c.POINTER(c.c_uint32), vp]
    L.kiln_w4a16_workspace_reset.restype = i
    L.kiln_w4a16_workspace_reset.argtypes = [vp, vp]
    L.kiln_marlin_w4a16_gemm_static_scratch.restype = i
    L.kiln_marlin_w4a16_gemm_static_scratch.argtypes = [vp, vp, vp, vp, i, i, i, i, i, vp]
    L.kiln_w4a16_debug_decode_plan.restype = i
    L.kiln_w4a16_debug_decode_plan.argtypes = [i, i, i, i, c.POINTER(c.c_int)]
    L.kiln_w4a16_debug_gemm_plan.restype = i
    L.kiln_w4a16_debug_gemm_plan.argtypes = [i, i, i, i, c.POINTER(c.c_int)]
    L.kiln_w4a16_debug_prefill_rowsum_producers.restype = i
    L.kiln_w4a16_debug_prefill_rowsum_producers.argtypes = [i, i, i, i]
    L.kiln_w4a16_gemm_lora.restype = i
    L.kiln_w4a16_gemm_lora.argtypes = [vp, vp, vp, vp, i, i, i, vp, i, i, vp, vp, vp, i, i,
                                       c.POINTER(c.c_int), c.POINTER(c.c_float)]
    L.kiln_w4a16_gemm_swiglu.restype = i
    L.kiln_w4a16_gemm_swiglu.argtypes = [vp, vp, vp, vp, i, i, i, vp, i, i, vp]
    L.kiln_w4a16_gemm_swiglu_lora.restype = i
    L.kiln_w4a16_gemm_swiglu_lora.argtypes = L.kiln_w4a16_gemm_lora.argtypes
    L.kiln_w4a16_mlp.restype = i
    L.kiln_w4a16_mlp.argtypes = [vp, vp, vp, vp, vp, vp, i, i, i, i, vp, i, i, vp]
    L.kiln_w4a16_mlp_workspace_bytes.restype = c.c_size_t
    L.kiln_w4a16_mlp_workspace_bytes.argtypes = [i, i, i, i]
    L.kiln_w4a16_quantize_and_pack_device.restype = i
    L.kiln_w4a16_quantize_and_pack_device.argtypes = [vp, i, i, i, vp, vp, i, vp]
    L.kiln_w4a16_repack_gptq_device.restype = i
    L.kiln_w4a16_repack_gptq_device.argtypes = [vp, vp, vp, i, i, i, vp, vp, i, vp]
    L.kiln_w4a16_interleave_gate_up_device.restype = i
    L.kiln_w4a16_interleave_gate_up_device.argtypes = [vp, vp, vp, vp, i, i, i, vp, vp, i, vp]
    L.kiln_w4a16_swiglu_workspace_bytes.restype = c.c_size_t
    L.kiln_w4a16_swiglu_workspace_bytes.argtypes = [i, i, i]
    L.kiln_w4a16_interleave_gate_up.restype = i
    L.kiln_w4a16_interleave_gate_up.argtypes = [vp, vp, vp, vp, i, i, i, vp, vp]
    L.kiln_w4a16_dequant_f32.restype = i
    L.kiln_w4a16_dequant_f32.argtypes = [vp, vp, i, i, i, vp, i, vp]
    L.kiln_w4a16_quantize_and_pack.restype = i
    L.kiln_w4a16_quantize_and_pack.argtypes = [vp, i, i, i, vp, vp, vp]
    L.kiln_w4a16_repack_gptq.restype = i
    L.kiln_w4a16_repack_gptq.argtypes = [vp, vp, vp, i, i, i, vp, vp]
    L.kiln_w4a16_unpack_to_gptq.restype = i
    L.kiln_w4a16_unpack_to_gptq.argtypes = [vp, vp, i, i, i, vp, vp]
    L.kiln_w4a16_status_string.restype = c.c_char_p
    L.kiln_w4a16_status_string.argtypes = [i]
    L.kiln_w4a16_layout_version.restype = i
    L.kiln_w4a16_layout_version.argtypes = []
    # include/kiln_marlin_proj.h
    i64, pp = c.c_int64, c.POINTER(c.c_void_p)
    L.kiln_marlin_proj_shape_is_supported.restype = i
    L.kiln_marlin_proj_shape_is_supported.argtypes = [i64, i64]
    L.kiln_marlin_proj_env_enabled.restype = i
    L.kiln_marlin_proj_env_enabled.argtypes = []
    L.kiln_marlin_proj_parallel_pack_disabled.restype = i
    L.kiln_marlin_proj_parallel_pack_disabled.argtypes = []
    L.kiln_marlin_proj_bf16_drop_disabled.restype = i
    L.kiln_marlin_proj_bf16_drop_disabled.argtypes = []
    L.kiln_marlin_proj_pack_from_bf16.restype = i
    L.kiln_marlin_proj_pack_from_bf16.argtypes = [vp, i64, i64, i, i, pp]
    L.kiln_marlin_proj_pack_from_bf16_batch.restype = i
    L.kiln_marlin_proj_pack_from_bf16_batch.argtypes = [c.POINTER(vp), c.POINTER(i64), c.POINTER(i64),
                                                        c.POINTER(i), i, i, pp]
    L.kiln_marlin_proj_pack_from_gptq.restype = i
    L.kiln_marlin_proj_pack_from_gptq.argtypes = [vp, vp, vp, i64, i64, i, i, pp]
    L.kiln_marlin_proj_matmul_bf16.restype = i
    L.kiln_marlin_proj_matmul_bf16.argtypes = [vp, vp, c.POINTER(i64), i, vp, vp, c.c_size_t, vp]
    for name, res in (("k", i64), ("n", i64), ("groupsize", i), ("b_packed", vp), ("scales", vp)):
        fn = getattr(L, f"kiln_marlin_proj_{name}")
        fn.restype = res
        fn.argtypes = [vp]
    L.kiln_marlin_proj_free.restype = None
    L.kiln_marlin_proj_free.argtypes = [vp]
    L.kiln_marlin_proj_last_error.restype = c.c_char_p
    L.kiln_marlin_proj_last_error.argtypes = []
    L.kiln_w4a16_artifact_write.restype = i
    L.kiln_w4a16_artifact_write.argtypes = [c.c_char_p, vp, vp, i64, i64, i]
    L.kiln_w4a16_artifact_info.restype = i
    L.kiln_w4a16_artifact_info.argtypes = [c.c_char_p, c.POINTER(i64), c.POINTER(i64), c.POINTER(i), c.POINTER(i)]
    L.kiln_w4a16_artifact_read.restype = i
    L.kiln_w4a16_artifact_read.argtypes = [c.c_char_p, vp, vp]
    L.kiln_marlin_proj_save.restype = i
    L.kiln_marlin_proj_save.argtypes = [vp, c.c_char_p]
    L.kiln_marlin_proj_load.restype = i
    L.kiln_marlin_proj_load.argtypes = [c.c_char_p, i, pp]
    _libs[tuning] = L
    return L


def status_string(status: int) -> str:
    return load().kiln_w4a16_status_string(status).decode()
