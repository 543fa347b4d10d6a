// Host-side launch descriptors shared between the dispatcher and the kernel files.
#pragma once
#include <atomic>
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace kiln {

// The start of every workspace, zero whenever no launch is running:
//   [0, 64 KiB)          arrival counters of the exchanges that count; the last 64 bytes are not a
//                        counter but one sticky word (kWsErrorOffset): a wavefront whose bounded wait ran
//                        out ORs a bit into it (which wait: the enum below) and nothing ever clears it but
//                        the caller, so that a launch that gave up can be told from one that worked
//   [64 KiB, + 4 MiB)    the region in which K slices exchange partial tiles that are their own arrival
//                        flags; its last 64 KiB hold the flags and counts of a LoRA projection folded
//                        into its GEMM's launch (16 replicas, 4 KiB apart: lora_tail.h)
constexpr size_t kWsCounterBytes = 64 * 1024;
constexpr size_t kWsErrorOffset = kWsCounterBytes - 64;
constexpr size_t kWsCounterCapacity = kWsErrorOffset;  // bytes of the counter region that hold counters
constexpr size_t kWsFlaggedBytes = 4 * 1024 * 1024;
constexpr size_t kWsFoldFlagBytes = 16 * 4096;
constexpr size_t kWsFoldFlagOffset = kWsCounterBytes + kWsFlaggedBytes - kWsFoldFlagBytes;
constexpr size_t kWsZeroedBytes = kWsCounterBytes + kWsFlaggedBytes;
enum WaitGaveUp : unsigned {
    kGaveUpDecodeExchange = 1u,  // K slices of a launch of up to 16 rows
    kGaveUpMidExchange = 2u,     // K slices of a launch of the mid-M kernel (17 rows up to 1024)
    kGaveUpDecodeFold = 4u,      // a block of up to 16 rows waiting for the folded LoRA projection
    kGaveUpMidFold = 8u,         // the same in a launch of the mid-M kernel with adapters (17...320 rows)
    kGaveUpPrefillFold = 16u,    // the same on the matrix-core path
};

// One launch of the decode kernel: M <= 16 rows of A against the whole weight.
constexpr int kDecodeFlaggedMaxSlices = 4;

// Counter-free exchange: blocks go to the eight dies round-robin by linear index (x fastest, then
// the slice), and the slices of a tile should sit on different dies.  Slice ks takes column block
// (x + ks * shift) % column_blocks; consecutive slices of a tile are then column_blocks - shift
// block indices apart, which must be odd to differ modulo 8 for up to eight slices.
inline int exchange_column_shift(int column_blocks) { return column_blocks % 2 == 0 ? 1 : 0; }

struct DecodeArgs {
    const void *A;      // bf16 [M, K]
    const void *B;      // packed weights, tile layout
    const void *S;      // fp16 scales, tile layout
    void *C;            // bf16 [M, N]
    float *partial;     // f32 partial tiles [KS][2][N/16][256]
    int *counters;      // N/16 arrival counters, zero on entry and on exit
    int M, N, K, Gs;
    int rows = 0;       // > M (register-fragment instance, M == 32 only): the launch covers `rows` rows of A and
                        // C, 33...128, in up to four runs of 32 (grid z), run z with counters + z * N/16 and
                        // partial tiles + z * KS * 2 * N/16 * 256
    int KS;             // K slices
    int GS;             // 128-row groups per slice (the last slice may be smaller)
    int U;              // chunks per wavefront, 1..decode_max_run(), <= smallest slice
    int BPS;            // blocks per slice; BPS * waves * U >= (N/16) * GS
    int waves;          // wavefronts per block, 1..16; waves * U >= GS
    bool direct = false;  // operand fragments straight from L2 instead of an LDS-staged slice (few rows)
    bool regs = false;    // the plan is for the register-fragment group-major instance (M <= 32)
    int gm_tiles = 0;     // > 0: the plan is for the LDS-staged group-major instance, this many tiles per block
    bool gmp = false;     // with gm_tiles > 0: the plan is for the private-staging group-major instance instead
    bool flagged = false; // gmp with KS > 1: `partial` is all zero between launches and the parts are their own
                          // arrival flags ((KS - 1) * N/16 * 1 KiB, KS <= kDecodeFlaggedMaxSlices); no counters
    // optional low-rank term (r_total == 0: none): C += lora_t * lora_b^T
    const void *lora_t = nullptr;  // bf16 [lora_slices][lora_rows][r_total rounded up to 16], at this slab's first
                                   // row: scaled projection in K slices, padding columns zero
    const void *lora_b = nullptr;  // bf16 [N, r_total]
    int r_total = 0;               // <= 64
    int lora_slices = 1;
    int lora_rows = 0;             // rows of the whole projection (>= M: the slab may be a part of it)
    // private-staging instance only: the projection computed inside the launch by lora_producers extra blocks
    // (0: lora_t was written by a launch of its own).  lora_t is then written here, [lora_producers][M][rp].
    int lora_producers = 0;        // = lora_slices, <= 16
    int lora_steps_per_slice = 0;  // 32-value steps of K per producer
    const void *lora_a = nullptr;  // bf16 [r_total, K]
    unsigned *lora_flags = nullptr;  // 64 KiB (16 replicas of flags and counts, 4 KiB apart), zero between launches
    int lora_adapters = 0;         // 1...4
    int lora_ends[4] = {};         // exclusive end column of adapter i (r_total past the last adapter)
    float lora_scales[4] = {};     // its scale (0 past the last)
    bool swiglu = false;  // columns are gate/up interleaved by 8 inside every tile; C is [M, N/2] = silu(gate) * up
    int group_major = -1; // tuning: 0 never a group-major instance, 1 only the LDS-staged one, 2 the
                          // register-fragment one wherever a plan fits it; -1: automatic
};

// Raise a kernel's dynamic-LDS limit, once per device and kernel instance (the attribute belongs
// to the device that is current when it is set, and a process may use several).
template <auto Kernel>
inline hipError_t allow_dynamic_lds(int bytes) {
    static std::atomic<unsigned long long> done{0};  // one per kernel instance: bit = device
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return err;
    const unsigned long long bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    err = hipFuncSetAttribute(reinterpret_cast<const void *>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (err == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return err;
}

int decode_max_waves();
int decode_max_run();
int decode_max_lds_bytes();
size_t decode_lds_bytes(int GS, int waves, bool direct);
size_t decode_gm_lds_bytes(int GS, int waves, int tiles);  // group-major instance
bool decode_group_major_ok(const struct DecodeArgs &a);     // does the plan fit the group-major instance?
size_t decode_gmr_lds_bytes(int waves, int tiles, int slabs);
bool decode_group_major_regs_ok(const struct DecodeArgs &a);  // ... and the one that takes up to 32 rows?
int decode_max_tiles_per_block();
hipError_t launch_decode(const DecodeArgs &args, hipStream_t stream);
bool decode_gmp_ok(const DecodeArgs &a);                        // does the plan fit the private-staging instance?
bool decode_gmp_fold_ok(const DecodeArgs &a);                   // ... with the LoRA projection folded into the launch?
hipError_t launch_decode_gmp(const DecodeArgs &a, hipStream_t stream);
hipError_t launch_decode_gmp_lora(const DecodeArgs &a, hipStream_t stream);  // its instances with the low-rank term (checked plan)

// One launch of the mid-M kernel: runs of up to 64 rows (grid z) against the whole weight.
struct MidArgs {
    const void *A;      // bf16 [M, K]
    const void *B;      // packed weights, tile layout
    const void *S;      // fp16 scales, tile layout
    void *C;            // bf16 [M, N]
    float *partial;     // mid_partial_bytes() bytes when KS > 1
    int *counters;      // runs * mid_column_blocks() arrival counters, zero on entry and on exit
    int M, N, K, Gs;
    int KS;             // K slices, all of GS groups
    int GS;             // 128-row groups per slice
    int waves;          // wavefronts per block, <= 8 and <= GS; each owns ceil(GS / waves) groups or one fewer
    int pairs;          // pairs of 16-column tiles per block: 1, 2 or 3
    bool swiglu;        // columns are gate/up interleaved by 8 inside every tile; C is [M, N/2] = silu(gate) * up
    bool flagged = false;  // KS > 1: `partial` is all zero between launches and the parts are their own arrival
                           // flags ((KS - 1) slices of mid_partial_bytes() / KS each); needs mid_flagged_ok()
    // optional low-rank term (r_total == 0: none): C += lora_t * lora_b^T, r_total % 8 == 0
    // (with swiglu the rows of lora_b are in the packed column order)
    const void *lora_t = nullptr;  // bf16 [lora_slices][M][r_total rounded up to 16], written before this launch
    const void *lora_b = nullptr;  // bf16 [N, r_total]
    int r_total = 0;
    int lora_slices = 1;
    // lora_producers > 0: the projection runs in this launch's first blocks (16-row tiles x lora_slices K slices of
    // lora_steps_per_slice steps) and lora_t is written here; needs >= 4 wavefronts per block
    int lora_producers = 0;
    int lora_steps_per_slice = 0;
    const void *lora_a = nullptr;    // bf16 [r_total, K]
    unsigned *lora_words = nullptr;  // 64 KiB that are zero between launches (lora_tail.h)
    int lora_adapters = 0;           // 1...8
    int lora_ends[8] = {};           // exclusive end column of adapter i on the stacked rank axis
    float lora_scales[8] = {};
};
bool mid_flagged_ok(const MidArgs &a);
bool mid_lora_fold_ok(const MidArgs &a);  // the projection onto the adapters inside the launch: do its fields allow it?
int mid_max_waves(int m, int pairs, bool lora);  // wavefronts a block of such a launch may have
int mid_column_blocks(const MidArgs &a);
int mid_max_rows_per_run();
bool mid_plan_ok(const MidArgs &a);
size_t mid_partial_bytes(const MidArgs &a);
hipError_t launch_mid(const MidArgs &a, hipStream_t stream);
hipError_t launch_mid_lora(const MidArgs &a, hipStream_t stream);  // its instances with the low-rank term (checked plan)

// One launch of the prefill path (row-sum pre-pass + MFMA kernel), any M >= 1.
struct PrefillArgs {
    const void *A;   // bf16 [M, K]
    const void *B;   // packed weights, tile layout
    const void *S;   // fp16 scales, tile layout
    void *C;         // bf16 [M, N]
    void *aext;      // prefill_aext_bytes(M, K) bytes of scratch
    int M, N, K, Gs;
    // optional fused LoRA epilogue (r_total == 0: none)
    const void *lora_a = nullptr;   // bf16 [r_total, K], adapters stacked along rows
    const void *lora_b = nullptr;   // bf16 [N, r_total], adapters stacked along columns
    void *lora_t = nullptr;         // prefill_lora_t_bytes(M, few_rows) bytes of scratch
    int r_total = 0;                // <= 64
    int n_adapters = 0;             // <= 8
    const int *ranks = nullptr;     // host arrays of length n_adapters
    const float *scales = nullptr;
    // K split across blocks (1 = none): partial tiles and per-tile arrival counters
    int KS = 1;
    int bn = 128;                   // block columns: 128 or 256
    int bm = 256;                   // block rows: 64, 128 or 256
    bool swiglu = false;            // columns are gate/up interleaved by 8 inside every tile; C is [M, N/2] = silu(gate) * up
    int nb_full = 0;                // leading column blocks computed as whole tiles; the rest is sliced
    int cus = 256;                  // compute units of the device
    float *partial = nullptr;       // prefill_partial_bytes(M, N, KS) bytes
    int *counters = nullptr;        // one per 256 x 128 tile, zero on entry and on exit
    unsigned *lora_words = nullptr; // 64 KiB that are zero between launches (see lora_tail.h): with them the LoRA
                                    // projection may run inside the product's launch; null: always in front of it
};

size_t prefill_aext_bytes(int m, int k);
size_t prefill_lora_t_bytes(int m, bool few_rows);  // scratch of the LoRA projection on either path
int prefill_lora_max_slices(int m);
int lora_project_slices(int m, int k);  // K slices of the few-rows projection (before rounding to whole groups)
struct PrefillPlan {
    int bn = 128;     // block columns
    int bm = 256;     // block rows
    int nb_full = 0;  // leading column blocks computed as whole tiles
    int ks = 1;       // K slices of the remaining column blocks
};
PrefillPlan plan_prefill(int m, int n, int k, int cus, int force_bn = 0, int force_bm = 0);
int prefill_grid(int m, int n, const PrefillPlan &p);
size_t prefill_partial_bytes(int m, int n, const PrefillPlan &p);
int prefill_rowsum_producers(int m, int n, int k, const PrefillPlan &p, int cus);  // blocks of a plain launch that form the row sums inside it (0: a launch in front does, -2: every block its own)
hipError_t launch_prefill(const PrefillArgs &args, hipStream_t stream);
// lora_t = bf16 [*slices][M][r_total rounded up to 16] = per-adapter scale * (A * lora_a^T) in K slices,
// padding columns zero.  few_rows: the small-M kernels will multiply it, in up to
// prefill_lora_max_slices(M) slices; otherwise one slice.
hipError_t launch_lora_project(const PrefillArgs &args, bool few_rows, hipStream_t stream, int *slices,
                               bool with_row_sums = false);  // many rows: also write the extension operand (args.aext)

}  // namespace kiln
