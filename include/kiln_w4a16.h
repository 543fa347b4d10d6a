/*
 * kiln W4A16 GEMM for AMD Instinct MI355X (gfx950) -- C ABI.
 *
 * Drop-in replacement for the C boundary of the reference crate
 * `kiln-marlin-gemm` (crates/kiln-marlin-gemm/csrc/marlin_kernel.h:39-55 and
 * the Rust `extern "C"` block at crates/kiln-marlin-gemm/src/lib.rs:50-68).
 * Plain pointers and sizes only; no C++ or torch types cross this boundary.
 *
 * Data contract (all device buffers row-major and contiguous):
 *
 *   A   bf16  [m, k]            activations            (reference: fp16 after a cast)
 *   B   int32 [k/16, 2n]        packed int4 weights, k*n/8 words.  Same word
 *                               count and tensor shape as the reference
 *                               (lib.rs:119), different order inside: the
 *                               "tile layout" written by the host functions
 *                               below.  Callers treat it as opaque.
 *   s   fp16  [k/g, n]          scales (g = 128, or one row when groupsize=-1),
 *                               same element count as the reference
 *                               (lib.rs:144-150), tile-ordered by the same host
 *                               functions.  Opaque to callers.
 *   C   bf16  [m, n]            output                 (reference: fp16, cast after)
 *
 * Weight semantics: code in 0..15, zero-point 8, value = (code - 8) * scale
 * (lib.rs:415-425).  Shape constraints are the reference's: k % 128 == 0,
 * n % 256 == 0, groupsize in {-1, 128} (lib.rs:112-130).
 *
 * Every device entry point only enqueues work on `stream`: no allocation, no
 * synchronisation, no host-side memset, safe under stream capture, re-entrant.
 */
#ifndef KILN_W4A16_H
#define KILN_W4A16_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int kiln_marlin_status_t;

/* Status codes.  0..2 are the reference's (marlin_kernel.cu:728-729). */
#define KILN_W4A16_OK               0
#define KILN_W4A16_ERR_PROB_SHAPE   1  /* k % 128, n % 256, groupsize not in {-1,128}, m < 0 */
#define KILN_W4A16_ERR_KERN_SHAPE   2  /* no kernel for this configuration (e.g. LoRA rank too large) */
#define KILN_W4A16_ERR_LAUNCH       3  /* HIP reported an error at launch */
#define KILN_W4A16_ERR_ARGUMENT     4  /* null pointer or inconsistent argument */
#define KILN_W4A16_ERR_ZERO_POINT   5  /* repack: a GPTQ zero-point other than 8 */
#define KILN_W4A16_ERR_SCRATCH      6  /* the call needs more scratch than the library's static array holds */

/*
 * Bits of the workspace's sticky word (kiln_w4a16_workspace_check): which bounded wait gave up.
 * Launches whose blocks wait for other blocks of the same launch (K slices that meet in the zeroed
 * prefix, blocks that wait for a LoRA projection computed by the launch's first blocks) poll a bounded
 * number of times (2^20 polls, tens of milliseconds).  Blocks are dispatched in index order and a
 * waiting block only waits for lower indices, so a launch that has the GPU to itself always gets there.
 */
#define KILN_W4A16_WAIT_DECODE_EXCHANGE 1u   /* K slices of a call of up to 16 rows */
#define KILN_W4A16_WAIT_MID_EXCHANGE    2u   /* K slices of a call the mid-M kernel takes (17 rows up to 1024) */
#define KILN_W4A16_WAIT_DECODE_FOLD     4u   /* LoRA projection inside a launch of up to 16 rows */
#define KILN_W4A16_WAIT_MID_FOLD        8u   /* ... of 17...320 rows on the mid-M kernel */
#define KILN_W4A16_WAIT_PREFILL_FOLD    16u  /* ... on the matrix-core path */

/* Size of the static device array behind kiln_marlin_w4a16_gemm_static_scratch (per GPU). */
#define KILN_W4A16_STATIC_SCRATCH_BYTES (8u << 20)

/*
 * C = A * dequant(B, s).
 * Replaces `kiln_marlin_w4a16_gemm` (marlin_kernel.h:39-55, marlin_kernel.cu:831-860)
 * with the same name and argument order.  Differences, all documented:
 *   - A and C are bf16 (the reference wrapper's two casts, lib.rs:169,269, go away);
 *   - B and s are in the tile layout;
 *   - A, B, C, s and `workspace` must be 16-byte aligned (KILN_W4A16_ERR_ARGUMENT otherwise);
 *   - `workspace` must hold kiln_w4a16_workspace_bytes(m, n, k) bytes (with overrides:
 *     kiln_w4a16_workspace_bytes_tuned), its first kiln_w4a16_workspace_zeroed_bytes()
 *     bytes zero on first use; every call leaves that prefix zero again (the
 *     reference's lock array has the same in/out contract, marlin_kernel.cu:177-180);
 *   - `stream` is a hipStream_t; thread_k (rows of K per block or K slice) and
 *     thread_n (columns per block) keep the reference's meaning as overrides of
 *     the automatic plan, -1 = automatic; sms overrides the compute-unit count;
 *     max_par is accepted and unused (callers pass -1, -1, -1, 16: lib.rs:252-255).
 * m == 0, n == 0 or k == 0 returns 0 without a launch (marlin_kernel.cu:772-773).
 */
kiln_marlin_status_t kiln_marlin_w4a16_gemm(
    const void *A, const void *B, void *C, void *s,
    int prob_m, int prob_n, int prob_k,
    void *workspace, int groupsize, int dev, void *stream,
    int thread_k, int thread_n, int sms, int max_par);

/*
 * Bytes of device workspace the GEMM entry points need for up to prob_m rows of this
 * projection shape with the automatic plan (thread_k = thread_n = sms = -1).  Replaces the
 * reference wrapper's fixed `(n / 128) * max_par` int32 sizing (lib.rs:176-178).
 * The value is the largest need of any row count from 1 to prob_m, so it never decreases
 * with prob_m: one workspace sized for the largest m a caller will issue serves every
 * smaller call, and it is never below kiln_w4a16_workspace_zeroed_bytes().  Only that prefix
 * (arrival counters, and the region in which K slices exchange partial tiles that are their
 * own arrival flags) must be zero before the first call; every call leaves it zero again, and
 * nothing else in the workspace carries state from one call to the next.  A caller that
 * overwrites the prefix between calls must zero it again before the next one.
 */
size_t kiln_w4a16_workspace_bytes(int prob_m, int prob_n, int prob_k);

/* The same for a caller that passes plan overrides to kiln_marlin_w4a16_gemm (<= 0: automatic). */
size_t kiln_w4a16_workspace_bytes_tuned(int prob_m, int prob_n, int prob_k,
                                        int thread_k, int thread_n, int sms);

/*
 * Length of the workspace prefix that must be zero on first use (64 KiB of counters + 4 MiB in
 * which K slices meet without counters; the reference's whole lock array has that contract,
 * marlin_kernel.cu:177-180, lib.rs:176-178).
 */
size_t kiln_w4a16_workspace_zeroed_bytes(void);

/*
 * What a caller can learn about the bounded waits, and how it recovers.  No counterpart in the
 * reference, whose lock waits are unbounded (marlin_kernel.cu:162-175).
 *
 * A wavefront whose wait runs out ORs a KILN_W4A16_WAIT_* bit into one word of the workspace
 * (kiln_w4a16_workspace_error_offset() bytes from its start, inside the zeroed prefix, used by nothing
 * else) and goes on: the call that gave up returns rows with NaN or without their low-rank term, and
 * what it was waiting for may land later and leave the prefix non-zero, which would corrupt every later
 * call on that workspace.  Nothing clears the word but kiln_w4a16_workspace_reset.
 *   kiln_w4a16_workspace_check  enqueues a 4-byte copy of the word to *host_word on `stream`; after the
 *       caller has synchronised the stream, 0 means no wait has given up since the last reset.  (A copy
 *       to host memory: not for use under graph capture.)
 *   kiln_w4a16_workspace_reset  zero-fills the prefix, sticky word included, with a kernel on `stream`
 *       (may be captured); call it after a non-zero check, once the stream has drained.
 * workspace == NULL means the static array of kiln_marlin_w4a16_gemm_static_scratch on the current device.
 * When can a wait run out?  Only when launches from several streams share the GPU in such a way that
 * waiting blocks hold every slot of a die while the blocks they wait for are queued behind other
 * launches' waiting blocks; up to four concurrent streams of the model's shapes cannot get there (a die
 * never fills with waiting blocks alone), more can in principle.  Serving code that overlaps many GEMM
 * streams should check the word once per step.
 */
size_t kiln_w4a16_workspace_error_offset(void);
kiln_marlin_status_t kiln_w4a16_workspace_check(const void *workspace, uint32_t *host_word, void *stream);
kiln_marlin_status_t kiln_w4a16_workspace_reset(void *workspace, void *stream);

/*
 * kiln_marlin_w4a16_gemm without the workspace argument, for callers that cannot allocate
 * device memory or hand a workspace over: code running under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its wrapper
 * allocates and zero-fills a workspace per call, lib.rs:174-178).  The counters and f32 partial
 * tiles live in a device array inside the library, KILN_W4A16_STATIC_SCRATCH_BYTES = 8 MiB per
 * GPU the library runs on, held until the process ends.  The call allocates nothing and frees
 * nothing.  A shape whose plan needs more than that (kiln_w4a16_workspace_bytes says how much a
 * shape needs; every call of the model's projections with m <= 128 fits; large
 * K-sliced prefill calls need tens of MB) is refused with KILN_W4A16_ERR_SCRATCH before anything
 * is launched.  `dev` must be the current device.  All calls on one GPU share that GPU's array:
 * calls that may overlap in time (different streams, or threads launching concurrently) race on
 * it and must be ordered by the caller; calls on one stream are safe back to back.
 */
kiln_marlin_status_t kiln_marlin_w4a16_gemm_static_scratch(
    const void *A, const void *B, void *C, void *s,
    int prob_m, int prob_n, int prob_k,
    int groupsize, int dev, void *stream);

/*
 * C = A * dequant(B, s) + sum_i scale_i * (A * lora_a_i^T) * lora_b_i^T.  Fuses what
 * the reference computes unfused as `base + compute_lora_delta(x, proj, scale)`
 * (crates/kiln-model/src/forward.rs:2932-2939, crates/kiln-model/src/lora_loader.rs:213-232):
 * the scaled projection scale_i * (A * lora_a_i^T) is formed first and rounded to bf16 (as
 * the reference rounds its `hidden`; for m <= 64 in up to 16 slices of K, each rounded on its
 * own), its product with lora_b is accumulated in f32 on top of the base product, and C is
 * rounded to bf16 once.  Any m: few rows take the small-M kernels like the plain GEMM.
 * lora_a and lora_b must be 16-byte aligned.
 *   lora_a  bf16 [r_total, k]   row-concatenated adapter A matrices
 *   lora_b  bf16 [n, r_total]   column-concatenated adapter B matrices
 *           (the stacking of crates/kiln-model/src/adapter_merge.rs:639-712)
 *   ranks, scales: host arrays of length n_adapters; sum(ranks) == r_total <= 64.
 * Workspace as for the plain GEMM.
 */
kiln_marlin_status_t kiln_w4a16_gemm_lora(
    const void *A, const void *B, void *C, const void *s,
    int prob_m, int prob_n, int prob_k,
    void *workspace, int groupsize, int dev, void *stream,
    const void *lora_a, const void *lora_b, int r_total,
    int n_adapters, const int *ranks, const float *scales);

/*
 * C[m, n_out] = silu(gate) * up with [gate | up] = A * dequant(B, s), the fused MLP
 * input projection followed by SwiGLU in one call, at any m.  The reference issues gate and
 * up as two GEMMs and then silu and a multiply as separate kernels on bf16 tensors
 * (crates/kiln-model/src/forward.rs:2771-2819); here every kernel forms the product from its
 * f32 sums where it stores a tile and rounds once: one launch, no intermediate tensor.
 *   B, s   packed for 2 * n_out columns by kiln_w4a16_interleave_gate_up (per 16 packed
 *          columns: 8 gate columns, then the 8 matching up columns); n_out % 128 == 0.
 *   workspace: kiln_w4a16_swiglu_workspace_bytes(m, n_out, k) bytes (= the plain GEMM's for
 *          2 * n_out columns), counter prefix zero on first use.
 */
kiln_marlin_status_t kiln_w4a16_gemm_swiglu(
    const void *A, const void *B, void *C, const void *s,
    int prob_m, int n_out, int prob_k,
    void *workspace, int groupsize, int dev, void *stream);

size_t kiln_w4a16_swiglu_workspace_bytes(int prob_m, int n_out, int prob_k);

/*
 * kiln_w4a16_gemm_swiglu with LoRA adapters on gate_proj and up_proj:
 * C[m, n_out] = silu(gate + d_gate) * (up + d_up), d = the low-rank terms of kiln_w4a16_gemm_lora.
 * The reference adds each projection's delta to its bf16 GEMM result before silu and the multiply
 * (mlp_proj_forward with lora_layer.gate_proj / up_proj, crates/kiln-model/src/forward.rs:2771-2819);
 * here the deltas land on the f32 sums and the product is rounded once.
 *   lora_a  bf16 [r_total, k]           A matrices of gate's adapters, then of up's, row-concatenated
 *   lora_b  bf16 [2 * n_out, r_total]   rows in the packed column order (per 16 rows: 8 gate columns,
 *           then the 8 matching up columns); a gate row holds gate's B entries in the rank columns of
 *           gate's adapters and zeros in up's, an up row the reverse
 *   ranks, scales: one entry per stacked adapter (gate's first), sum(ranks) == r_total <= 64.
 * Workspace: kiln_w4a16_swiglu_workspace_bytes(m, n_out, k).
 */
kiln_marlin_status_t kiln_w4a16_gemm_swiglu_lora(
    const void *A, const void *B, void *C, const void *s,
    int prob_m, int n_out, int prob_k,
    void *workspace, int groupsize, int dev, void *stream,
    const void *lora_a, const void *lora_b, int r_total,
    int n_adapters, const int *ranks, const float *scales);

/*
 * y[m, n_down] = down( silu(gate(x)) * up(x) ): the MLP of a layer as one call, at any m.  The reference's
 * swiglu_ffn_impl (crates/kiln-model/src/forward.rs:2723-2848) issues the gate GEMM, the up GEMM, silu, the
 * multiply and the down GEMM one after the other; this is kiln_w4a16_gemm_swiglu followed by
 * kiln_marlin_w4a16_gemm -- two launches -- with silu(gate) * up kept in the workspace, rounded to bf16 once.
 *   x                    bf16 [m, hidden]
 *   b_gate_up, s_gate_up packed for 2 * n_out columns by kiln_w4a16_interleave_gate_up(_device); n_out % 128 == 0
 *   b_down, s_down       the down projection [n_out, n_down], packed as for kiln_marlin_w4a16_gemm
 *   y                    bf16 [m, n_down]
 *   workspace            kiln_w4a16_mlp_workspace_bytes(m, hidden, n_out, n_down) bytes (never decreases with m),
 *                        zeroed prefix as for every entry point
 */
kiln_marlin_status_t kiln_w4a16_mlp(
    const void *x, const void *b_gate_up, const void *s_gate_up, const void *b_down, const void *s_down,
    void *y, int prob_m, int hidden, int n_out, int n_down,
    void *workspace, int groupsize, int dev, void *stream);

size_t kiln_w4a16_mlp_workspace_bytes(int prob_m, int hidden, int n_out, int n_down);

/*
 * out[k, n] (f32, row-major) = (code - 8) * f32(scale), read from the tile
 * layout on the device.  The device-side statement of lib.rs:425; used to
 * prove the repack bit-exact.  No counterpart entry point in the reference.
 */
kiln_marlin_status_t kiln_w4a16_dequant_f32(
    const void *B, const void *s, int prob_k, int prob_n, int groupsize,
    void *out, int dev, void *stream);

/*
 * Quantise a bf16 [k, n] weight that is already in device memory and pack it there: the same
 * quantiser as kiln_w4a16_quantize_and_pack below (lib.rs:393-427) and the same bits out, without
 * the download, host pack and upload of crates/kiln-model/src/marlin_proj.rs:86-181 (the reference
 * has no device-side counterpart; its host pack costs 17-58 s per model load).  b_packed: k*n/8
 * int32, scales_f16: (k/g)*n fp16, both device memory; the two kernels run on `stream`.
 */
kiln_marlin_status_t kiln_w4a16_quantize_and_pack_device(
    const void *weight_bf16, int k, int n, int groupsize,
    void *b_packed, void *scales_f16, int dev, void *stream);

/*
 * kiln_w4a16_interleave_gate_up (below) for packed projections that are in device memory: one
 * copy kernel on `stream`, same bits.  out_b: k * 2 n_each / 8 int32, out_s: (k/g) * 2 n_each fp16.
 */
kiln_marlin_status_t kiln_w4a16_interleave_gate_up_device(
    const void *gate_b, const void *gate_s, const void *up_b, const void *up_s,
    int k, int n_each, int groupsize, void *out_b, void *out_s, int dev, void *stream);

/*
 * kiln_w4a16_repack_gptq (below) for GPTQ tensors that are in device memory: same bits, no
 * re-quantisation.  With qzeros the call waits for `stream` once (the zero-points must all be 8
 * before anything is written; not for use under graph capture); without, it only launches.
 */
kiln_marlin_status_t kiln_w4a16_repack_gptq_device(
    const void *qweight, const void *scales_f16, const void *qzeros,
    int k, int n, int groupsize, void *b_packed, void *scales_tiled, int dev, void *stream);

/* ---- host-side packing (pure CPU, thread-safe, no GPU state) ------------ */

/*
 * Quantise a row-major f32 [k, n] weight and pack it.  Replaces
 * `pack::quantize_and_pack` (lib.rs:370-491): same quantiser, same output
 * element counts (b_packed k*n/8 int32, scales (k/g)*n fp16, dequant k*n f32
 * or NULL), tile layout instead of the Marlin permutation.
 */
kiln_marlin_status_t kiln_w4a16_quantize_and_pack(
    const float *weight, int k, int n, int groupsize,
    int32_t *b_packed, uint16_t *scales_f16, float *dequant);

/*
 * The one-time offline repack: GPTQ-canonical tensors
 * (qweight int32 [k/8, n], 8 codes per word along k, LSB first; scales fp16
 * [k/g, n]; optional qzeros int32 [k/g, n/8], all of which must be 8:
 * crates/kiln-model/src/quantized.rs:1-14,127-152) -> tile layout.
 */
kiln_marlin_status_t kiln_w4a16_repack_gptq(
    const int32_t *qweight, const uint16_t *scales_f16, const int32_t *qzeros,
    int k, int n, int groupsize, int32_t *b_packed, uint16_t *scales_tiled);

/* Inverse of kiln_w4a16_repack_gptq (tile layout -> GPTQ-canonical). */
kiln_marlin_status_t kiln_w4a16_unpack_to_gptq(
    const int32_t *b_packed, const uint16_t *scales_tiled,
    int k, int n, int groupsize, int32_t *qweight, uint16_t *scales_f16);

/*
 * Interleave two packed projections of equal shape [k, n_each] (gate, up) into the
 * packed form kiln_w4a16_gemm_swiglu reads: [k, 2 * n_each] with, per 16 columns (one
 * column tile), 8 gate columns then the 8 matching up columns.  n_each % 128 == 0.
 * No counterpart in the reference (its gate and up stay separate tensors).
 */
kiln_marlin_status_t kiln_w4a16_interleave_gate_up(
    const int32_t *gate_b, const uint16_t *gate_s, const int32_t *up_b, const uint16_t *up_s,
    int k, int n_each, int groupsize, int32_t *out_b, uint16_t *out_s);

/* Static description of a status code. */
const char *kiln_w4a16_status_string(kiln_marlin_status_t status);

/* Layout revision written into persisted artefacts; bumps when the tile layout changes. */
int kiln_w4a16_layout_version(void);

/*
 * Plan queries: what the library would run for a plain GEMM of these sizes on a part with `cus`
 * compute units.  Pure host functions (no GPU is touched, nothing is launched); they exist for
 * benchmarks, profiles and tests that must name the kernel they measure, and have no counterpart in
 * the reference (whose one kernel picks its tile from a fixed table, marlin_kernel.cu:784-816).
 * The numbers describe this library's kernels and may change with any revision.
 *
 * kiln_w4a16_debug_gemm_plan: out[8] = {matrix-core kernel?, launches of the small-M kernels, block
 *   rows, block columns, whole column blocks, K slices (the last four of the matrix-core kernel),
 *   mid-M kernel?, its tile pairs per block * 16 + K slices}.  Returns 0, or 1 for sizes no kernel takes.
 * kiln_w4a16_debug_decode_plan: the small-M plan for one run of m <= 32 rows, out[8] = {K slices,
 *   groups per slice, chunks per wavefront, blocks per slice, wavefronts per block, fragments straight
 *   from L2?, register-fragment instance?, tiles per block (negative: the private-staging instance)}.
 *   Returns 0, or 1 if no plan fits.
 * kiln_w4a16_debug_prefill_rowsum_producers: where the matrix-core kernel's row sums come from:
 *   > 0 that many blocks of the product's own launch, 0 a launch in front, -2 every block sums its own
 *   rows, -3 another kernel takes the call, -1 bad sizes.
 */
int kiln_w4a16_debug_gemm_plan(int prob_m, int prob_n, int prob_k, int cus, int *out);
int kiln_w4a16_debug_decode_plan(int prob_m, int prob_n, int prob_k, int cus, int *out);
int kiln_w4a16_debug_prefill_rowsum_producers(int prob_m, int prob_n, int prob_k, int cus);

#ifdef __cplusplus
}
#endif
#endif /* KILN_W4A16_H */
