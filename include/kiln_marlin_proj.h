/*
 * Projection-level host glue over the W4A16 GEMM -- C ABI.
 *
 * Mirrors crates/kiln-model/src/marlin_proj.rs of the reference (storage of a
 * packed projection, the three-phase pack at model load, the rank-2 / rank-3
 * activation path, the two environment switches) for hosts that are not Rust,
 * plus the persisted form of a packed projection, which the reference lacks
 * (it re-quantises every projection at every start, marlin_proj.rs:198-262).
 *
 * Functions return 0 on success, KILN_PROJ_SKIPPED where the reference returns
 * Ok(None), and a negative value on error; kiln_marlin_proj_last_error() then
 * holds the message (same texts as the reference's anyhow errors, prefix
 * "marlin_proj:").  Pack and artefact functions allocate and synchronise (they
 * run at load time); kiln_marlin_proj_matmul_bf16 only enqueues work.
 */
#ifndef KILN_MARLIN_PROJ_H
#define KILN_MARLIN_PROJ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KILN_PROJ_OK        0
#define KILN_PROJ_SKIPPED   1   /* shape outside k % 128 == 0, n % 256 == 0, or weight not on a GPU */
#define KILN_PROJ_ERR      (-1) /* see kiln_marlin_proj_last_error() */

/* MarlinPackedProj (marlin_proj.rs:38-50): packed weight + scales on the GPU, k, n, groupsize. */
typedef struct kiln_marlin_packed_proj kiln_marlin_packed_proj_t;

/* shape_is_supported (marlin_proj.rs:53-55). */
int kiln_marlin_proj_shape_is_supported(int64_t k, int64_t n);

/* env_enabled (marlin_proj.rs:330-338): KILN_W4A16 in {1, true, yes}, case-insensitive. */
int kiln_marlin_proj_env_enabled(void);

/* parallel_pack_disabled (marlin_proj.rs:346-356): KILN_DISABLE_PARALLEL_PACK in {1, true, yes}. */
int kiln_marlin_proj_parallel_pack_disabled(void);

/* marlin_bf16_drop_disabled (crates/kiln-model/src/forward.rs:1565-1580): KILN_DISABLE_MARLIN_BF16_DROP in
 * {1, true, yes} keeps the bf16 copy of a projection resident beside its packed weight. */
int kiln_marlin_proj_bf16_drop_disabled(void);

/*
 * pack_from_bf16 (marlin_proj.rs:198-207): quantise and pack a bf16 [k, n] row-major
 * weight that lies on device `dev`.  The reference downloads it, packs on the host and
 * uploads; here two kernels do it where the weight lies (kiln_w4a16_quantize_and_pack_device,
 * the same bits; they run on the device's default stream and the call returns when they are
 * done).  KILN_W4A16_HOST_PACK in {1, true, yes} takes the reference's three-phase host route.
 * `dev` < 0 means "not on a GPU": skipped, as the reference does for non-CUDA
 * tensors (marlin_proj.rs:88-91).  *out is NULL unless the result is KILN_PROJ_OK.
 */
int kiln_marlin_proj_pack_from_bf16(const void *weight_t, int64_t k, int64_t n, int groupsize, int dev,
                                    kiln_marlin_packed_proj_t **out);

/*
 * pack_from_bf16_batch (marlin_proj.rs:230-262): every weight packed on the device in
 * turn; on the host route (KILN_W4A16_HOST_PACK) serial downloads, the host pack of all jobs
 * in parallel (sequential under KILN_DISABLE_PARALLEL_PACK), serial uploads.
 * outs[i] is NULL for skipped entries; order is preserved.
 */
int kiln_marlin_proj_pack_from_bf16_batch(const void *const *weights_t, const int64_t *ks, const int64_t *ns,
                                          const int *groupsizes, int count, int dev,
                                          kiln_marlin_packed_proj_t **outs);

/*
 * Build a packed projection from GPTQ-canonical host tensors (the one-time
 * offline repack; no re-quantisation).  No counterpart in the reference, which
 * dequantises GPTQ weights to bf16 (crates/kiln-model/src/quantized.rs:70-163)
 * and then re-quantises them (marlin_proj.rs:229).  The tensors are uploaded as they are
 * and rearranged on the device (kiln_w4a16_repack_gptq_device); KILN_W4A16_HOST_PACK in
 * {1, true, yes} rearranges on the host and uploads the result (same bits).
 */
int kiln_marlin_proj_pack_from_gptq(const int32_t *qweight, const uint16_t *scales_f16, const int32_t *qzeros,
                                    int64_t k, int64_t n, int groupsize, int dev,
                                    kiln_marlin_packed_proj_t **out);

/*
 * matmul_bf16 (marlin_proj.rs:285-319): x is bf16, rank 2 [m, k] or rank 3
 * [batch, seq, k], contiguous; y receives [.., n] bf16.  `workspace` holds at
 * least kiln_w4a16_workspace_bytes(m, n, k) zero-initialised bytes (m = the
 * product of the leading dims) and is reusable across calls on one stream.
 */
int kiln_marlin_proj_matmul_bf16(const kiln_marlin_packed_proj_t *w, const void *x, const int64_t *dims, int rank,
                                 void *y, void *workspace, size_t workspace_bytes, void *stream);

/* Field access (the struct's public fields in the reference). */
int64_t kiln_marlin_proj_k(const kiln_marlin_packed_proj_t *w);
int64_t kiln_marlin_proj_n(const kiln_marlin_packed_proj_t *w);
int kiln_marlin_proj_groupsize(const kiln_marlin_packed_proj_t *w);
const void *kiln_marlin_proj_b_packed(const kiln_marlin_packed_proj_t *w); /* device, int32 [k/16, 2n] */
const void *kiln_marlin_proj_scales(const kiln_marlin_packed_proj_t *w);   /* device, fp16 [k/g, n] */

void kiln_marlin_proj_free(kiln_marlin_packed_proj_t *w);

/* Message of the calling thread's last error ("" if none). */
const char *kiln_marlin_proj_last_error(void);

/* ---- persisted packed projections ---------------------------------------
 *
 * File = 64-byte header + packed words + scales.  Header (little endian):
 *   0  char[8]  "KW4A16\0\0"
 *   8  u32      layout version (kiln_w4a16_layout_version())
 *   12 i32      groupsize (-1 or 128)
 *   16 u64      k          24 u64  n
 *   32 u64      bytes of packed words (k * n / 2)
 *   40 u64      bytes of scales ((k / g) * n * 2)
 *   48 u64      FNV-1a 64 of the body
 *   56 u64      zero
 * No counterpart in the reference.
 */
int kiln_w4a16_artifact_write(const char *path, const int32_t *b_packed, const uint16_t *scales, int64_t k, int64_t n,
                              int groupsize);
/* Reads and validates the header only. */
int kiln_w4a16_artifact_info(const char *path, int64_t *k, int64_t *n, int *groupsize, int *layout_version);
/* Reads the body into caller buffers of the sizes the header states; verifies the checksum. */
int kiln_w4a16_artifact_read(const char *path, int32_t *b_packed, uint16_t *scales);
/* Write a packed projection (downloads it from the GPU). */
int kiln_marlin_proj_save(const kiln_marlin_packed_proj_t *w, const char *path);
/* Load a packed projection onto device `dev`; rejects other layout versions and corrupt files. */
int kiln_marlin_proj_load(const char *path, int dev, kiln_marlin_packed_proj_t **out);

#ifdef __cplusplus
}
#endif
#endif /* KILN_MARLIN_PROJ_H */
