// Large-M (prefill) W4A16 GEMM kernel for gfx950.
//
// Replaces the m > 16 arm of the reference dispatcher and kernel
// (crates/kiln-marlin-gemm/csrc/marlin_kernel.cu:754-763, :784-816, :189-700).
// This regime is a dense contraction bound by the bf16 matrix cores.
//
// Block = 4 wavefronts (2 x 2), block tile 256 rows x 128 columns, wavefront
// tile 128 x 64 = 4 x 2 tiles of v_mfma_f32_32x32x16_bf16 (128 accumulator
// registers, two wavefronts per SIMD).  Per 32 rows of K:
//   * a 256 x 32 bf16 tile of A goes global -> LDS with direct 128-bit loads
//     (no registers, no VALU) into a ring of four stages, three stages ahead
//     of the products, one barrier per stage, stored with an XOR swizzle so
//     that fragment reads are bank-conflict free;
//   * each wavefront reads its 64 columns of packed weights straight from
//     global memory (four 128-bit loads per lane and 128-row group, prefetched
//     one group ahead) and expands the codes in registers: weights never touch
//     LDS, and each expanded fragment feeds four products.
// Group scales are applied in f32 by a running rescale of the accumulator (one
// multiply per accumulator register and group): after group g it holds
// (partial result) / scale(g); the step to the next group multiplies by
// scale(g) / scale(g+1).  No second accumulator set is needed, and scales are
// never rounded into the weights.
// The B operand carries 136 + d (d = code - 8).  The surplus
// 136 * sum_k(a) * scale is removed at the end by a short extra contraction
// over "extension" operands: per (row, group) the value c = -136 * sum_k a,
// split exactly into three bf16 terms by the pre-pass kernel below, times the
// group scale split exactly into two bf16 terms; six exact products per group
// accumulate c * scale into the result (about 5 % extra matrix work).
#include <type_traits>

#include "device_common.h"
#include "launch.h"
#include "lora_tail.h"
#include "lora_project.h"
#include "async_loads.h"

namespace kiln {

namespace {

constexpr int kAStages = 4;

// c[m][g] = -136 * sum_{k in group g} a[m][k], split into bf16 hi/mid/lo and
// stored (group-major, [g][m]) as the 8-slot extension operand
// [hi, hi, mid, mid, lo, lo, 0, 0].
__global__ __launch_bounds__(256) void w4a16_prefill_rowsum_kernel(const uint16_t *__restrict__ A,
                                                                 u32x4 *__restrict__ aext, int M, int K) {
    const int G = K / kGroupK;
    const int item = blockIdx.x * 16 + (threadIdx.x >> 4);  // (row, group), 16 lanes each
    const int sub = threadIdx.x & 15;
    if (item >= M * G) return;
    const int row = item / G, g = item - row * G;
    float sum = sum_bf16x8(*reinterpret_cast<const u32x4 *>(A + (size_t)row * K + (size_t)g * kGroupK + sub * 8));
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, 16);
    if (sub == 0) aext[(size_t)g * M + row] = extension_operand(sum);  // group-major: the 32 rows of a half-wavefront are contiguous
}

template <int RB>
__global__ __launch_bounds__(256) void w4a16_lora_project_kernel(const uint16_t *__restrict__ X,
                                                                const uint16_t *__restrict__ a_cat,
                                                                uint16_t *__restrict__ T, int M, int K, int r_total,
                                                                int RP, int steps_per_slice, LoraScales ls,
                                                                float *partial, int *counters, u32x4 *aext) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    lora_project_block<RB>(lds, X, a_cat, T, M, K, r_total, RP, steps_per_slice, ls, partial, counters, aext,
                           blockIdx.x, blockIdx.y, gridDim.y, nullptr);
}

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// 128-bit direct global -> LDS load: lane i's 16 bytes land at lds_addr + 16 i.
// Written as inline asm on purpose.  Through the compiler's builtin, every
// later LDS read is preceded by a wait for *all* outstanding loads (the
// compiler cannot tell which ring slot a direct load targets), which would
// serialise the pipeline; completion is tracked by the explicit s_waitcnt
// before each barrier instead.  Only addresses enter the asm, never loaded data.
// Plain global loads issued the same way (the compiler counts only the loads it
// knows about, so a compiler-tracked load consumed while asm loads are in
// flight would drain the whole queue).  The results may be used only after an
// explicit s_waitcnt that covers them, followed by pin() on the registers.
__device__ __forceinline__ u32x4 async_load_b128(const u32x4 *p) {
    u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ uint32_t async_load_u16(const uint16_t *p) {
    uint32_t v;
    asm volatile("global_load_ushort %0, %1, off" : "=&v"(v) : "v"(p) : "memory");
    return v;
}
// Orders every later use of v after this point (and hence after the preceding s_waitcnt).
__device__ __forceinline__ void pin(u32x4 &v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin(uint32_t &v) { asm volatile("" : "+v"(v)); }

// immediate of s_waitcnt for vmcnt(n), other counters unconstrained
constexpr int vmcnt_imm(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

__device__ __forceinline__ void direct_load_b128(const void *gptr, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_addr)
                 : "memory", "m0");
}

// Probe builds only (-DKILN_PREFILL_TIMELINE): wall-clock stamps per block.
#ifdef KILN_PREFILL_TIMELINE
__device__ long long *g_timeline;
#define KILN_TL(i)                                                                              \
    do {                                                                                        \
        if (threadIdx.x == 0) {                                                                 \
            g_timeline[(size_t)blockIdx.x * 8 + (i)] = __builtin_amdgcn_s_memrealtime();        \
            if ((i) < 2) g_timeline[(size_t)blockIdx.x * 8 + 6 + (i)] = __builtin_amdgcn_s_memtime(); \
        }                                                                                       \
    } while (0)
#else
#define KILN_TL(i) \
    do {           \
    } while (0)
#endif

// v from the lane selected by a data-parallel-primitive control word (no LDS traffic)
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Block shape: WM x NWN wavefronts, each owning MI x 2 tiles of 32 x 32 (MI * 32 rows x 64
// columns).  WM = 2, MI = 4: 256-row blocks (256 x 128 with 4 wavefronts, 256 x 256 with 8);
// WM = 1: 128-row (MI = 4) and 64-row (MI = 2) blocks for small M.
// SWIGLU: every 16-column tile of the packed weight holds 8 gate columns, then the 8 matching up
// columns; a wavefront's sub-tile 0 gathers the gate columns of its four tiles and sub-tile 1 the
// up columns; the store writes silu(gate) * up, half as wide
// (crates/kiln-model/src/forward.rs:2771-2819 computes gate, up, silu and the product as
// separate bf16 tensors; here the product is formed from the f32 accumulators and rounded once).
// RS: the row sums of A that the offset removal needs are formed inside the kernel from the A
// tiles in LDS (one extra 128-bit LDS read and ~20 VALU instructions per wavefront and stage)
// instead of by the pre-pass kernel: for the small blocks, whose launches are bound by latency,
// this saves a launch and the global reads of the extension operands.
// The LoRA projection (and the extension operand) computed inside the launch that uses them: the
// first `producers` blocks of the grid run lora_project_block (row tiles of 16 rows, K slices one
// after the other) while the others multiply; a block of the product looks at its row tiles' words
// behind its main loop -- long after they were raised -- and reads both operands with ordinary
// loads (no cache on its die has seen those lines since the launch began).  The words live in
// workspace that is all zero between launches (the region lora_tail.h describes: the tile words
// from word kPrefillFoldTileWord of its first replica on); every block counts itself after its
// look, on the replicated counts, and the last one zeroes words and counts.
// A launch without adapters uses the same words for the row sums alone (a_cat == nullptr): its
// producers run rowsum_producer_block.  A block asks for its words a few groups before its main
// loop ends, with a load that lands in LDS by itself (prefill_fold_peek), and waits for them behind
// the loop only if that look came too early.
struct PrefillFold {
    const uint16_t *a_cat;   // bf16 [r_total, K]
    uint16_t *t;             // bf16 [M, RP], behind it the f32 tiles in which K slices meet
    u32x4 *aext;             // the extension operand the producers write
    float *partial;
    int *counters;           // per row tile, zero on entry and exit (not the product's own counters)
    unsigned *words;         // the zeroed region
    int producers;           // row_tiles * kz rounded up to a multiple of 8 (the product's blocks keep their dies)
    int row_tiles, kz, steps_per_slice;
    int consumers;           // blocks of the product (grid padding included)
    int sum_tiles;           // a_cat == nullptr (no adapters): the producers form the row sums only, this many
                             // 16-row tiles each
    LoraScales ls;
};
constexpr int kPrefillFoldTileWord = 32;
constexpr int kPrefillFoldMaxTiles = kLoraFoldReplicaWords - kPrefillFoldTileWord;
constexpr int kPrefillFoldSpinLimit = 1 << 20;
// where a wavefront's early look at its words lands: the last KiB of the LDS every instance that takes part has
// (the projection's blocks need kProjectLdsBytes16), behind the A ring and the row sums a block may keep there
constexpr int kProjectLdsBytes16 = (16 + kProjectMaxRank) * kProjectRowBytes + kProjectMaxRank * (int)sizeof(float);
constexpr int kFoldPeekOffset = kProjectLdsBytes16 - 1024;

// The row sums of a launch without adapters, as the work of one of its first blocks: the extension
// operand of 16-row tiles [t0, t1) -- a contiguous piece of A, streamed with 24 loads per thread in
// flight; 16 lanes per (row, group), the order of additions of w4a16_prefill_rowsum_kernel, whose
// launch this saves -- written through to memory, then the tiles' words.
__device__ __forceinline__ void rowsum_producer_block(const uint16_t *__restrict__ A, u32x4 *__restrict__ aext, int M,
                                                      int K, int t0, int t1, unsigned *done) {
    constexpr int U = 24;
    const int G = K / kGroupK;
    const int r0 = t0 * 16, r1 = min(t1 * 16, M);
    const int items = (r1 - r0) * G;  // item L: the 256 bytes from byte 256 L of the piece on
    const int tid = threadIdx.x, sub = tid & 15, slot = tid >> 4;
    const u32x4 *src = reinterpret_cast<const u32x4 *>(A + (size_t)r0 * K) + sub;
    for (int base = 0; base < items; base += 16 * U) {
        u32x4 v[U];
        float sum[U];
#pragma unroll
        for (int u = 0; u < U; ++u)  // items past the end re-read the last one
            v[u] = async_load_b128(src + (size_t)min(base + u * 16 + slot, items - 1) * 16);
        unrolled<0, U>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            // loads complete in issue order: load u has landed when at most the U - 1 - u later ones are pending
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(U - 1 - u));
            pin(v[u]);
            sum[u] = sum_bf16x8(v[u]);
#pragma unroll
            for (int off = 8; off >= 1; off >>= 1) sum[u] += __shfl_xor(sum[u], off, 16);
        });
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int L = base + u * 16 + slot;
            if (sub == 0 && L < items) {
                const int row = L / G, g = L - row * G;
                store_b128_through(aext + (size_t)g * M + r0 + row, extension_operand(sum[u]));
            }
        }
    }
    // every wavefront's stores acknowledged, then the words
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    for (int t = t0 + tid; t < t1; t += 256) __hip_atomic_store(done + t, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// A look at the words of rows [m0, m0 + rows) that nobody waits for: one device-scope load per lane
// straight into LDS (256 bytes per wavefront at lds_addr), asked for a few groups before the main
// loop ends so that the round trip runs under its products; prefill_fold_seen() reads the answer.
// Every lane must see a raised word: lanes beyond the last tile look at the last one.
__device__ __forceinline__ void prefill_fold_peek(const PrefillFold &pf, int m0, int rows, int lane, unsigned lds_addr) {
    const int t0 = m0 >> 4, nt = min((rows + 15) >> 4, pf.row_tiles - t0);
    const unsigned *p = pf.words + kPrefillFoldTileWord + t0 + min(lane, nt - 1);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off sc1" : : "v"(p), "s"(lds_addr) : "memory", "m0");
}
__device__ __forceinline__ bool prefill_fold_seen(const unsigned char *lds_slot, int lane) {
    const unsigned f = *reinterpret_cast<const volatile unsigned *>(lds_slot + lane * 4);
    return __builtin_amdgcn_ballot_w64(f == 0u) == 0;
}

// rows [m0, m0 + rows) of T and of the extension operand are in memory
__device__ __forceinline__ void prefill_fold_wait(const PrefillFold &pf, int m0, int rows, int lane) {
    const int t0 = m0 >> 4, nt = min((rows + 15) >> 4, pf.row_tiles - t0);
    int spins = 0;
    for (; spins < kPrefillFoldSpinLimit; ++spins) {
        unsigned f = 1u;
        if (lane < nt) f = __hip_atomic_load(pf.words + kPrefillFoldTileWord + t0 + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (__builtin_amdgcn_ballot_w64(f == 0u) == 0) break;
        __builtin_amdgcn_s_sleep(8);
    }
    if (__builtin_expect(spins == kPrefillFoldSpinLimit, 0))
        report_wait_gave_up(error_word_before_fold_words(pf.words), kGaveUpPrefillFold, lane);
}
// one wavefront of block `consumer`, after its look: count the block; the last one zeroes everything
__device__ __forceinline__ void prefill_fold_done(const PrefillFold &pf, int consumer, int lane) {
    const int replica = consumer % kLoraFoldReplicas;
    const unsigned quota = (unsigned)(pf.consumers - replica + kLoraFoldReplicas - 1) / kLoraFoldReplicas;
    const unsigned replicas = (unsigned)min(pf.consumers, kLoraFoldReplicas);
    unsigned before = 0;
    if (lane == 0)
        before = __hip_atomic_fetch_add(pf.words + replica * kLoraFoldReplicaWords + kLoraFoldCountWord, 1u, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
    before = (unsigned)__builtin_amdgcn_readfirstlane((int)before);
    if (before != quota - 1u) return;
    if (lane == 0) before = __hip_atomic_fetch_add(pf.words + kLoraFoldTopWord, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    before = (unsigned)__builtin_amdgcn_readfirstlane((int)before);
    if (before != replicas - 1u) return;
    for (int i = lane; i < pf.row_tiles; i += 64)
        __hip_atomic_store(pf.words + kPrefillFoldTileWord + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (lane <= kLoraFoldTopWord)
        for (int r = 0; r < kLoraFoldReplicas; ++r)
            __hip_atomic_store(pf.words + r * kLoraFoldReplicaWords + lane, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int NWN, int WM, int MI, bool SWIGLU, bool RS, bool FOLD = false>
__global__ __launch_bounds__(64 * WM * NWN, (WM == 2 && NWN == 4) ? 1 : 2) void w4a16_prefill_kernel(
    const uint16_t *__restrict__ A, const u32x4 *__restrict__ B, const uint16_t *__restrict__ S,
    uint16_t *__restrict__ C, const u32x4 *__restrict__ aext, int M, int N, int K, int Gs, int m_blocks,
    const uint16_t *__restrict__ lora_t, const uint16_t *__restrict__ lora_b, int r_total, int RP, int nb_full,
    int KS, int GSb, float *partial, int *counters, int die_rows, PrefillFold pf) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];  // the A ring; reused by the store
    static_assert(!FOLD || WM * NWN == 4, "the projection's blocks have four wavefronts");
    if constexpr (FOLD) {
        if ((int)blockIdx.x < pf.producers) {
            const int unit = blockIdx.x;
            if (pf.a_cat == nullptr) {
                const int t0 = unit * pf.sum_tiles;
                if (t0 < pf.row_tiles)
                    rowsum_producer_block(A, pf.aext, M, K, t0, min(t0 + pf.sum_tiles, pf.row_tiles),
                                          pf.words + kPrefillFoldTileWord);
                return;
            }
            if (unit < pf.row_tiles * pf.kz)
                lora_project_block<16>(lds, A, pf.a_cat, pf.t, M, K, r_total, RP, pf.steps_per_slice, pf.ls, pf.partial,
                                       pf.counters, pf.aext, unit % pf.row_tiles, unit / pf.row_tiles, pf.kz,
                                       pf.words + kPrefillFoldTileWord);
            return;
        }
    }
    constexpr int BM = WM * MI * 32, BN = 64 * NWN;  // block rows and columns
    constexpr int NW = WM * NWN, NT = 64 * NW;       // wavefronts, threads
    constexpr int kAStageBytes = BM * 32 * 2;        // BM rows x 32 columns of bf16 per stage
    constexpr int APW = (BM / 16) / NW;              // A loads (16 rows each) per wavefront and stage
    static_assert(APW * NW * 16 == BM, "A stage must divide evenly over the wavefronts");
    constexpr int RPW = BM / NW;                     // RS: rows of A each wavefront sums
    static_assert(!RS || RPW % 16 == 0, "row sums are taken 16 rows per read");

    KILN_TL(0);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / NWN, wn = wave % NWN;
    const int G = K / kGroupK;
    const int l32 = lane & 31, h = lane >> 5;

    // Work list.  The first nb_full column blocks are whole tiles (all of K in
    // one block); the remaining column blocks are cut into KS slices of K each,
    // so that a last, partly filled round of tiles still spreads over the whole
    // chip.  Blocks are dispatched in id order: whole tiles first, slices last.
    // Consecutive ids go to different dies.  The 8 dies form a die_rows x
    // (8 / die_rows) grid over (row blocks x units), a unit being a column block
    // or a K slice of one; inside its rectangle a die walks unit by unit, all its
    // row blocks of one unit back to back.  Blocks resident on a die at one time
    // therefore share the few row blocks of A the die owns (they stay in its L2,
    // where the loads that feed the matrix cores three stages ahead must hit) and
    // read each unit's weights from memory once.
    int id = blockIdx.x;
    if constexpr (FOLD) id -= pf.producers;
    [[maybe_unused]] const int consumer = id;
    const int n_blocks = N / BN;
    const int die_cols = 8 / die_rows, rows_per_die = (m_blocks + die_rows - 1) / die_rows;
    const int per_die_full = rows_per_die * ((nb_full + die_cols - 1) / die_cols);
    const bool sliced = id >= 8 * per_die_full;
    if (sliced) id -= 8 * per_die_full;
    const int units = sliced ? (n_blocks - nb_full) * KS : nb_full;  // per row block
    const int units_per_die = (units + die_cols - 1) / die_cols;
    const int die = id & 7, seq = id >> 3;
    const int unit = (die / die_rows) * units_per_die + seq / rows_per_die;
    const int mb = (die % die_rows) * rows_per_die + seq % rows_per_die;
    if (seq >= rows_per_die * units_per_die || unit >= units || mb >= m_blocks) {  // grid padding (whole block, before any barrier)
        if constexpr (FOLD) {
            if (wave == 0) prefill_fold_done(pf, consumer, lane);  // counted like the others: it will never look
        }
        return;
    }
    int nb = unit, ks = 0;
    if (sliced) {
        nb = nb_full + unit / KS;
        ks = unit % KS;
    }
    const int m0 = mb * BM, n0 = nb * BN;
    // K slice of this block: groups [g_begin, g_end).  With KS > 1 the slices of
    // a tile are combined through the workspace at the end.
    const int g_begin = sliced ? ks * GSb : 0, g_end = sliced ? min(G, g_begin + GSb) : G;

    // --- A: global -> LDS without passing through registers --------------------
    // A stage is BM rows x 32 columns of bf16 = 64 B per row, 4 units of 16 B;
    // four stages form a ring and loads run three stages ahead of the products
    // (a stage lasts about as long as one L2 round trip, so a shallower
    // pipeline leaves the matrix cores waiting at every barrier).
    // Unit c of row r is stored at unit position c ^ ((r >> 2) & 3): with four units
    // per row, any 16 consecutive rows read at one unit index then touch the 16
    // different 16-byte positions of a 256-byte bank line, so the 128-bit fragment
    // reads are bank-conflict free (with (r >> 1) & 3 rows r and r + 8 collided: four
    // conflict cycles on every fragment read, 13 % of the launch's cycles).  One direct
    // load moves 1 KiB = 16 rows: lane i writes LDS slot i, so it fetches row i / 4,
    // unit (i % 4) ^ ((i / 16) & 3).
    // Wavefront w moves the 16-row blocks w, w + NW, ...
    // Rows past M re-read row M - 1: their products are never stored.
    const uint16_t *a_src[APW];
#pragma unroll
    for (int p = 0; p < APW; ++p) {
        const int blk = wave + NW * p;
        int row = m0 + blk * 16 + (lane >> 2);
        row = row < M ? row : M - 1;
        a_src[p] = A + (size_t)row * K + (size_t)g_begin * kGroupK + (((lane & 3) ^ ((lane >> 4) & 3)) * 8);
    }
    const int n_stages = 4 * (g_end - g_begin);
    const unsigned lds_base = (unsigned)(size_t)(lds_ptr_t)lds;
    auto load_a = [&](int st) {  // stage st (32 columns of K) -> ring slot st & 3
        const unsigned slot = lds_base + (st & 3) * kAStageBytes;
#pragma unroll
        for (int p = 0; p < APW; ++p) direct_load_b128(a_src[p] + (size_t)st * 32, slot + (wave + NW * p) * 1024);
    };

    // --- B: column sub-tile ni (32 columns = chunks 2ni, 2ni+1 of this wavefront);
    // load v (0/1) fetches lane (l32 % 16) + 16 * (2v + h) of chunk (l32 / 16).
    const int nt_base = (n0 + wn * 64) / kTileN;  // first 16-column tile of this wavefront
    const u32x4 *b_src[2][2];
    const uint16_t *s_src[2];
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
        // SWIGLU: every 16-column tile holds 8 gate columns, then the 8 matching up columns; sub-tile 0
        // gathers the gate columns of the wavefront's four tiles, sub-tile 1 their up columns, so a lane
        // holds a gate value and its up value in the same register of the two accumulators
        const int nt = SWIGLU ? nt_base + (l32 >> 3) : nt_base + 2 * ni + (l32 >> 4);
        const int c = SWIGLU ? (l32 & 7) + 8 * ni : (l32 & 15);
#pragma unroll
        for (int v = 0; v < 2; ++v) b_src[ni][v] = B + (size_t)nt * G * 64 + c + 16 * (2 * v + h);
        s_src[ni] = S + (size_t)nt * Gs * kTileN + c;
    }
    const int gs_mask = (Gs == 1) ? 0 : -1;
    // a zero scale would break the running rescale below; it is replaced by a
    // value too small to matter (the same value in the extension contraction)
    auto scale_value = [&](uint32_t raw) {
        const float sv = f16_bits_to_f32((uint16_t)raw);
        return sv == 0.f ? 0x1p-40f : sv;
    };

    const DequantConsts dq = dequant_consts();
    // fragment read offsets inside a stage for the two k16 steps of a stage:
    // row (wm*MI*32 + mi*32 + l32), unit (2*step + h) ^ ((row >> 2) & 3)
    int a_off[2];
#pragma unroll
    for (int sp = 0; sp < 2; ++sp)
        a_off[sp] = (wm * MI * 32 + l32) * 64 + (((2 * sp + h) ^ ((l32 >> 2) & 3)) * 16);

    f32x16 acc[MI][2];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;

    // prologue: three stages of A, the first group's weights
    load_a(0);
    load_a(1);
    load_a(2);
    u32x4 bw[2][2], bw_next[2][2];
    uint32_t sc_raw[2], sc_raw_next[2];
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
        bw[ni][0] = async_load_b128(b_src[ni][0] + (size_t)g_begin * 64);
        bw[ni][1] = async_load_b128(b_src[ni][1] + (size_t)g_begin * 64);
        sc_raw[ni] = async_load_u16(s_src[ni] + (size_t)(g_begin & gs_mask) * kTileN);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    float sc[2];
#pragma unroll
    for (int ni = 0; ni < 2; ++ni) {
        pin(bw[ni][0]);
        pin(bw[ni][1]);
        pin(sc_raw[ni]);
        sc[ni] = scale_value(sc_raw[ni]);
    }

    // RS: c[group][row] = -136 * (row sum of the group), f32, behind the ring
    [[maybe_unused]] float gsum[RS ? RPW / 16 : 1] = {};
    [[maybe_unused]] float *csum = reinterpret_cast<float *>(lds + kAStages * kAStageBytes);
    [[maybe_unused]] const int g_peek = max(g_begin, g_end - 3);
    for (int g = g_begin; g < g_end; ++g) {
        const bool more = g + 1 < g_end;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int st = 4 * (g - g_begin) + q;
            if (st + 3 < n_stages) load_a(st + 3);  // into the slot read one stage ago
            if (q == 0 && more) {
#pragma unroll
                for (int ni = 0; ni < 2; ++ni) {
                    bw_next[ni][0] = async_load_b128(b_src[ni][0] + (size_t)(g + 1) * 64);
                    bw_next[ni][1] = async_load_b128(b_src[ni][1] + (size_t)(g + 1) * 64);
                    sc_raw_next[ni] = async_load_u16(s_src[ni] + (size_t)((g + 1) & gs_mask) * kTileN);
                }
            }
            if constexpr (FOLD) {
                // (one more load in flight only makes the counted waits below stricter)
                if (q == 0 && g == g_peek)
                    prefill_fold_peek(pf, m0, min(BM, M - m0), lane, lds_base + kFoldPeekOffset + wave * 256);
            }
            const unsigned char *slot = lds + (st & 3) * kAStageBytes;
            // Two k16 steps per stage (step u = 2q + sp uses word q of load sp).
            // Fragments of the second step are read while the first step's
            // products run, and each expansion of codes is placed between
            // products: a product occupies the matrix pipe for 32 cycles, enough
            // to issue the 7 VALU instructions of one expansion behind it.
            if constexpr (RS) {
                // this wavefront's rows of the stage: lane -> row lane / 4, unit lane % 4 (8 columns)
#pragma unroll
                for (int rr = 0; rr < RPW / 16; ++rr) {
                    const int row = wave * RPW + rr * 16 + (lane >> 2);
                    const u32x4 v = *reinterpret_cast<const u32x4 *>(slot + row * 64 + (((lane & 3) ^ ((row >> 2) & 3)) * 16));
                    const uint32_t wd[4] = {v.x, v.y, v.z, v.w};
                    float s8 = 0.f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        s8 += __builtin_bit_cast(float, wd[i] << 16);
                        s8 += __builtin_bit_cast(float, wd[i] & 0xFFFF0000u);
                    }
                    s8 += dpp_move<0xB1>(s8);  // quad_perm [1,0,3,2]
                    s8 += dpp_move<0x4E>(s8);  // quad_perm [2,3,0,1]: the row's 32 columns
                    gsum[rr] += s8;
                }
            }
            bf16x8 a0[MI], a1[MI];
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
                a0[mi] = *reinterpret_cast<const bf16x8 *>(slot + a_off[0] + mi * 32 * 64);
            auto word_of = [&](int ni, int sp) {
                return (q == 0) ? bw[ni][sp].x : (q == 1) ? bw[ni][sp].y : (q == 2) ? bw[ni][sp].z : bw[ni][sp].w;
            };
            bf16x8 b00 = codes_to_bf16x8(word_of(0, 0), dq);
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
                a1[mi] = *reinterpret_cast<const bf16x8 *>(slot + a_off[1] + mi * 32 * 64);
            const bf16x8 b10 = codes_to_bf16x8(word_of(1, 0), dq);
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
                acc[mi][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0[mi], b00, acc[mi][0], 0, 0, 0);
            const bf16x8 b01 = codes_to_bf16x8(word_of(0, 1), dq);
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
                acc[mi][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0[mi], b10, acc[mi][1], 0, 0, 0);
            const bf16x8 b11 = codes_to_bf16x8(word_of(1, 1), dq);
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
                acc[mi][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1[mi], b01, acc[mi][0], 0, 0, 0);
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
                acc[mi][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1[mi], b11, acc[mi][1], 0, 0, 0);
            if constexpr (MI == 4) {
                // scheduling hint: 4 x (product, 2 VALU, 1 LDS read), then 12 x (product, 2 VALU)
    #pragma unroll
                for (int i = 0; i < 4; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
    #pragma unroll
                for (int i = 0; i < 12; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
                }
            }
            // Stage st + 1 must have landed.  Loads complete in issue order; still
            // allowed in flight are the loads of stages st + 2 and st + 3 (APW each)
            // and, in three of four steps, the 6 weight/scale loads issued after
            // stage st + 1's.  After step 3 that leaves the next group's weights
            // complete as well.  The last group drains everything.
            if (!more) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
            else if (q == 3) __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * APW));  // vmcnt(2 APW)
            else __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * APW + 6));          // vmcnt(2 APW + 6)
            __syncthreads();
        }
        if constexpr (RS) {
            if ((lane & 3) == 0) {
#pragma unroll
                for (int rr = 0; rr < RPW / 16; ++rr)
                    csum[(g - g_begin) * BM + wave * RPW + rr * 16 + (lane >> 2)] = -kCodeBias * gsum[rr];
            }
#pragma unroll
            for (int rr = 0; rr < RPW / 16; ++rr) gsum[rr] = 0.f;
        }
        // Running rescale: the accumulator holds (sum so far) / scale(g).
        // Switching to the next group's scale multiplies it by
        // scale(g) / scale(g+1); after the last group, by scale(g).  One multiply
        // per accumulator register and group; nothing is ever rounded to bf16.
        float f[2];
        if (more) {
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
                pin(bw_next[ni][0]);
                pin(bw_next[ni][1]);
                pin(sc_raw_next[ni]);
                const float sn = scale_value(sc_raw_next[ni]);
                f[ni] = sc[ni] * __builtin_amdgcn_rcpf(sn);
                bw[ni][0] = bw_next[ni][0];
                bw[ni][1] = bw_next[ni][1];
                sc[ni] = sn;
            }
        } else {
            f[0] = sc[0];
            f[1] = sc[1];
        }
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[mi][ni][r] *= f[ni];
    }

    KILN_TL(1);
    if constexpr (RS) __syncthreads();  // every wavefront's row sums are in LDS
    if constexpr (FOLD) {
        // the rows of this block in the extension operand and in T: written during this launch
        // (the last group's waits have drained every load, the early look included)
        if (!prefill_fold_seen(lds + kFoldPeekOffset + wave * 256, lane)) prefill_fold_wait(pf, m0, min(BM, M - m0), lane);
        if (wave == 0) prefill_fold_done(pf, consumer, lane);
    }
    // --- remove the 136 * sum(a) * scale surplus: extension contraction ------
    // Step e covers groups g_begin + 2e (lanes 0-31) and g_begin + 2e + 1 (lanes
    // 32-63), 8 slots each.  Operands come straight from global memory, loaded
    // several steps ahead: every step issues its loads unconditionally (the group
    // index is clamped, dead slots are zeroed), so the loads of later steps are
    // in flight while the products of this one run.
    {
        int ext_row[MI];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            const int row = m0 + wm * MI * 32 + mi * 32 + l32;
            ext_row[mi] = row < M ? row : M - 1;
        }
        struct ExtOps {
            u32x4 a[MI];
            uint32_t s[2];
        };
        auto ext_load = [&](int e, ExtOps &o) {  // writes the registers of o in place: no copies of pending loads
            int g = g_begin + 2 * e + h;
            g = g < g_end ? g : g_end - 1;
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
                if constexpr (!RS) o.a[mi] = async_load_b128(aext + (size_t)g * M + ext_row[mi]);
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) o.s[ni] = async_load_u16(s_src[ni] + (size_t)(g & gs_mask) * kTileN);
        };
        constexpr int kExtDepth = MI == 4 ? 5 : 6;
        constexpr int kExtLoads = RS ? 2 : MI + 2;  // loads per step
        auto ext_step = [&](int e, ExtOps &o) {
            // this step's operands have landed when at most the later steps' loads are pending
            __builtin_amdgcn_s_waitcnt(vmcnt_imm((kExtDepth - 1) * kExtLoads));
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
                if constexpr (!RS) pin(o.a[mi]);
            pin(o.s[0]);
            pin(o.s[1]);
            const bool live = g_begin + 2 * e + h < g_end;
            if constexpr (RS) {
                // c from LDS, split exactly into three bf16 terms: [hi, hi, mid, mid, lo, lo, 0, 0]
                const int gl = live ? 2 * e + h : 0;  // group inside this block's K range
#pragma unroll
                for (int mi = 0; mi < MI; ++mi) {
                    const float c = csum[gl * BM + wm * MI * 32 + mi * 32 + l32];
                    const uint32_t hi = __builtin_bit_cast(uint32_t, c) & 0xFFFF0000u;
                    const float r1 = c - __builtin_bit_cast(float, hi);                     // exact
                    const uint32_t mid = __builtin_bit_cast(uint32_t, r1) & 0xFFFF0000u;
                    const float r2 = r1 - __builtin_bit_cast(float, mid);                   // exact, <= 8 significant bits
                    const uint32_t lo = __builtin_bit_cast(uint32_t, r2) & 0xFFFF0000u;
                    o.a[mi] = live ? u32x4{(hi >> 16) | hi, (mid >> 16) | mid, (lo >> 16) | lo, 0u} : u32x4{0u, 0u, 0u, 0u};
                }
            }
            bf16x8 bx[2];
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
                const float sv = scale_value(o.s[ni]);
                const uint32_t hi = __builtin_bit_cast(uint32_t, sv) & 0xFFFF0000u;
                const float lo_f = sv - __builtin_bit_cast(float, hi);  // exact: f16 has 11 significant bits
                const uint32_t pair = live ? ((hi >> 16) | (__builtin_bit_cast(uint32_t, lo_f) & 0xFFFF0000u)) : 0u;
                const u32x4 r = {pair, pair, pair, 0u};
                bx[ni] = __builtin_bit_cast(bf16x8, r);
            }
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                const bf16x8 ax = __builtin_bit_cast(bf16x8, o.a[mi]);
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ax, bx[ni], acc[mi][ni], 0, 0, 0);
            }
        };
        // kExtDepth register sets rotate by position, never by copying (a copy of
        // a register whose load is still in flight would wait for it); the step
        // count is rounded up to a multiple of the depth, the extra steps multiply
        // by zero.  The main loop's weight and fragment registers are dead here,
        // which is what pays for the depth.
        const int n_ext = (g_end - g_begin + 1) / 2;
        ExtOps o[kExtDepth];
#pragma unroll
        for (int d = 0; d < kExtDepth; ++d) ext_load(d, o[d]);
        for (int e = 0; e < n_ext; e += kExtDepth) {
#pragma unroll
            for (int d = 0; d < kExtDepth; ++d) {
                ext_step(e + d, o[d]);
                ext_load(e + d + kExtDepth, o[d]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // the look-ahead loads of steps past the end are still in flight; nothing may reuse
        // their registers before they land
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
#pragma unroll
        for (int d = 0; d < kExtDepth; ++d) {
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
                if constexpr (!RS) pin(o[d].a[mi]);
            pin(o[d].s[0]);
            pin(o[d].s[1]);
        }
    }

    // --- fused LoRA epilogue: y += T * B_cat^T with T = scaled x * A_cat^T from the
    // pre-pass (crates/kiln-model/src/lora_loader.rs:213-232, unfused at the call
    // sites forward.rs:2932-2939).  RP / 16 more k16 steps on the same accumulators.
    for (int u = 0; u < (ks == 0 ? RP / 16 : 0); ++u) {  // the LoRA term belongs to one slice only
        const int j8 = 16 * u + 8 * h;  // this lane's 8 rank columns
        bf16x8 lb[2];
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
            // the lane's column of accumulator ni, as the main loop maps it (SWIGLU: gate columns of four
            // tiles in accumulator 0, their up columns in 1; lora_b's rows are in the packed column order)
            const int bcol = SWIGLU ? 16 * (l32 >> 3) + 8 * ni + (l32 & 7) : ni * 32 + l32;
            const uint16_t *bp = lora_b + (size_t)(n0 + wn * 64 + bcol) * r_total + j8;
            if ((r_total & 7) == 0 && j8 + 8 <= r_total) {
                lb[ni] = *reinterpret_cast<const bf16x8 *>(bp);
            } else {
                uint16_t tmp[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) tmp[i] = (j8 + i < r_total) ? bp[i] : (uint16_t)0;
                u32x4 r = {tmp[0] | ((uint32_t)tmp[1] << 16), tmp[2] | ((uint32_t)tmp[3] << 16),
                           tmp[4] | ((uint32_t)tmp[5] << 16), tmp[6] | ((uint32_t)tmp[7] << 16)};
                lb[ni] = __builtin_bit_cast(bf16x8, r);
            }
        }
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            int row = m0 + wm * MI * 32 + mi * 32 + l32;
            row = row < M ? row : M - 1;
            const bf16x8 la = *reinterpret_cast<const bf16x8 *>(lora_t + (size_t)row * RP + j8);
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
                acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(la, lb[ni], acc[mi][ni], 0, 0, 0);
        }
    }

    // --- store.  Register r of a 32x32 tile holds row 8*(r/4) + 4*h + r%4,
    // column l32: a lane owns one column.  Each wavefront transposes its
    // (MI * 32) x 64 tile through its own piece of LDS (the now idle A ring) as bf16, then
    // writes rows with 128-bit stores: 8 lanes cover the 128 contiguous bytes
    // of one row of the tile.
    KILN_TL(2);
    if (sliced && KS > 1) {
        // Combine the K slices of this tile.  Every block writes its f32 partial
        // tile with device-scope accesses (element (mi, ni, r) of thread t at
        // ((mi*2+ni)*16 + r) * NT + t: coalesced both ways); the last block to
        // arrive reads all KS partial tiles back and adds them in slice order,
        // so the result does not depend on arrival order.
        __shared__ int s_last;
        const int tile = (nb - nb_full) * m_blocks + mb;
        float *mine = partial + ((size_t)tile * KS + ks) * (BM * BN);
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    __hip_atomic_store(mine + ((mi * 2 + ni) * 16 + r) * NT + tid, acc[mi][ni][r],
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // each wavefront waits until its own stores have been acknowledged (a barrier alone
        // orders nothing outside the workgroup); after the barrier the arrival is counted
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();
        KILN_TL(3);
        if (tid == 0)
            s_last = (__hip_atomic_fetch_add(counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == KS - 1);
        __syncthreads();
        if (!s_last) return;
        // slice 0 lands straight in the accumulators; the others go through a
        // 64-register staging array, MI / 2 batches per slice
        const float *all = partial + (size_t)tile * KS * (BM * BN) + tid;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[mi][ni][r] = __hip_atomic_load(all + ((mi * 2 + ni) * 16 + r) * NT, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
        for (int s2 = 1; s2 < KS; ++s2) {
            const float *src = all + (size_t)s2 * (BM * BN);
#pragma unroll
            for (int half = 0; half < MI / 2; ++half) {
                float t[64];
#pragma unroll
                for (int i = 0; i < 64; ++i)
                    t[i] = __hip_atomic_load(src + (half * 64 + i) * NT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int i = 0; i < 64; ++i) acc[half * 2 + i / 32][(i / 16) & 1][i & 15] += t[i];
            }
        }
        if (tid == 0) __hip_atomic_store(counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        KILN_TL(4);
    }
    __syncthreads();  // every wavefront is done reading the A ring
    if constexpr (SWIGLU) {
        // acc[mi][0] holds gate, acc[mi][1] the matching up columns: h = gate / (1 + exp(-gate)) * up.
        // The wavefront's tile becomes (MI * 32) x 32: rows of 64 bytes, 4 lanes per row.
        uint16_t *tile = reinterpret_cast<uint16_t *>(lds + wave * (MI * 32 * 32 * 2));  // [MI * 32][32] bf16
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float gate = acc[mi][0][r], up = acc[mi][1][r];
                const float hval = gate * __builtin_amdgcn_rcpf(1.f + __expf(-gate)) * up;
                const int row = mi * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                tile[row * 32 + ((((l32 >> 3) ^ (row & 3)) << 3) | (l32 & 7))] = f32_to_bf16_bits(hval);
            }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
#pragma unroll
        for (int p = 0; p < MI * 2; ++p) {
            const int row = p * 16 + (lane >> 2), unit = lane & 3;
            const u32x4 v = *reinterpret_cast<const u32x4 *>(tile + row * 32 + ((unit ^ (row & 3)) << 3));
            const int grow = m0 + wm * MI * 32 + row;
            if (grow < M)
                *reinterpret_cast<u32x4 *>(C + (size_t)grow * (N / 2) + (n0 + wn * 64) / 2 + unit * 8) = v;
        }
    } else {
        uint16_t *tile = reinterpret_cast<uint16_t *>(lds + wave * (MI * 32 * 64 * 2));  // [MI * 32][64] bf16
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = mi * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                    // 16-byte unit index XOR (row & 7): keeps the row reads below conflict free
                    const int col = ni * 32 + l32;
                    tile[row * 64 + ((((col >> 3) ^ (row & 7)) << 3) | (col & 7))] = f32_to_bf16_bits(acc[mi][ni][r]);
                }
        // same wavefront wrote and reads: only the LDS counter needs to drain
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
#pragma unroll
        for (int p = 0; p < MI * 4; ++p) {
            const int row = p * 8 + (lane >> 3), unit = lane & 7;
            const u32x4 v = *reinterpret_cast<const u32x4 *>(tile + row * 64 + ((unit ^ (row & 7)) << 3));
            const int grow = m0 + wm * MI * 32 + row;
            if (grow < M)
                *reinterpret_cast<u32x4 *>(C + (size_t)grow * N + n0 + wn * 64 + unit * 8) = v;
        }
    }
    KILN_TL(5);
}

}  // namespace

#ifdef KILN_PREFILL_TIMELINE
extern "C" int kiln_w4a16_debug_timeline(long long *buf) {
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(g_timeline), &buf, sizeof(buf));
}
#endif

size_t prefill_aext_bytes(int m, int k) { return (size_t)m * (k / kGroupK) * sizeof(u32x4); }

// Scratch of the projection.  For the small-M kernels (few_rows): up to 16 K slices of T in bf16.
// For the matrix-core kernel: T once and behind it the f32 tiles in which the slices meet (at most
// ceil(256 / row tiles) slices per row tile: fewer than 256 + 2 x row tiles tiles of 64 or 16 rows
// x 64 columns).
constexpr int kProjectMaxCounters = (int)(kWsCounterCapacity / sizeof(int));  // the counter region less its sticky word
constexpr int kProjectFoldCounters = 8192;  // folded into the product's launch: the product's counters first, then the projection's
// measured at 2048 rows: 16-row blocks 9.9 us against 13.1 for K = 2560, 23.5 against 20.2 for K = 9216
int lora_project_rows_per_block(int m, int k) { return m > 1024 && k > 4096 ? 64 : 16; }
int prefill_lora_max_slices(int) { return 16; }
size_t prefill_lora_t_bytes(int m, bool few_rows) {
    if (few_rows) return (size_t)prefill_lora_max_slices(m) * m * 64 * sizeof(uint16_t);
    size_t many = 0;
    for (int rb = 16; rb <= 64; rb *= 4) {  // either block height
        const size_t tiles = 256 + 2 * (size_t)((m + rb - 1) / rb);
        const size_t bytes = (size_t)m * 64 * sizeof(uint16_t) + tiles * rb * 64 * sizeof(float);
        if (bytes > many) many = bytes;
    }
    return many;
}

// Rows of the die grid (a power of two up to 8; the dies form rows x 8 / rows over row blocks x units): the one
// under which the busiest die has the least to do -- ceil(row blocks / rows) row blocks of ceil(units / columns)
// units each, a whole tile counting as `ks` slices -- and of equals the one with the most rows, so that a die
// keeps few row blocks of A in its L2.  Neither count need divide: the grid is padded with blocks that leave at once.
// (Until the row blocks could be padded it was the largest power of two that divides them, i.e. one row of
// eight columns for any odd count, which leaves dies idle wherever the units are fewer than eight or do not
// divide by eight: 1024 -> 1024 at 20000 rows, 313 row blocks of three whole column blocks and one more, ran
// 165 us on three dies and then one, against 58 us at 19968 rows.)
static int prefill_die_rows(int m_blocks, int units_full, int units_sliced, int ks) {
    int best = 1;
    long best_work = -1;
    for (int dr = 8; dr >= 1; dr >>= 1) {
        const int dc = 8 / dr, rows = (m_blocks + dr - 1) / dr;
        const long work = (long)rows * ((long)((units_full + dc - 1) / dc) * ks + (units_sliced + dc - 1) / dc);
        if (best_work < 0 || work < best_work) {
            best = dr;
            best_work = work;
        }
    }
    return best;
}
static int prefill_die_rows(int m_blocks, int n, const PrefillPlan &p) {
    return prefill_die_rows(m_blocks, p.nb_full, (n / p.bn - p.nb_full) * p.ks, p.ks);
}

// blocks launched: whole tiles, then (tile, K slice) units, each part padded to the die grid
int prefill_grid(int m, int n, const PrefillPlan &p) {
    const int m_blocks = (m + p.bm - 1) / p.bm;
    const int dr = prefill_die_rows(m_blocks, n, p), dc = 8 / dr, rows = (m_blocks + dr - 1) / dr;
    const int units_full = p.nb_full, units_sliced = (n / p.bn - p.nb_full) * p.ks;
    return 8 * rows * ((units_full + dc - 1) / dc) + 8 * rows * ((units_sliced + dc - 1) / dc);
}

// Whole-tile part and K slices for a block shape.  Whole rounds of tiles (one tile per
// compute unit and round) run unsliced.  What is left -- everything, for a small problem --
// is cut into as many K slices as still leave one block per compute unit and three groups
// per slice, so the last round is as full as the others instead of leaving most of the chip
// idle.
static PrefillPlan plan_for_shape(int m, int n, int k, int cus, int bn, int bm, int sliced_units = 0) {
    if (sliced_units <= 0) sliced_units = cus;  // (tile, K slice) units the sliced round may have
    PrefillPlan p;
    p.bn = bn;
    p.bm = bm;
    const int G = k / kGroupK, m_blocks = (m + bm - 1) / bm;
    const int n_blocks = n / bn, tiles = m_blocks * n_blocks;
    const int rounds = tiles / cus;
    p.nb_full = (rounds * cus) / m_blocks;  // whole column blocks that fit the whole rounds
    if (p.nb_full > n_blocks) p.nb_full = n_blocks;
    // ... on every die: the dies deal the tiles as a grid (prefill_die_rows), and a die whose rectangle holds more
    // whole tiles than its share of the rounds runs a round of its own behind them (4096 -> 4096 at 1100 rows: 18
    // row blocks x 14 column blocks are 252 tiles, but 36 on each of six dies of 32 units -- 80 us, against 62 us at
    // 1217 rows, whose 20 x 12 are 30 per die)
    for (;; --p.nb_full) {
        const int rest = n_blocks - p.nb_full;
        p.ks = 1;
        for (int ks = 2; ks <= 8 && G / ks >= 3; ++ks) {
            const int gsb = (G + ks - 1) / ks;
            if ((ks - 1) * gsb >= G) continue;  // would leave an empty slice
            const int dr = prefill_die_rows(m_blocks, p.nb_full, rest * ks, ks), dc = 8 / dr;
            if (8 * ((m_blocks + dr - 1) / dr) * ((rest * ks + dc - 1) / dc) <= sliced_units) p.ks = ks;
        }
        if (p.nb_full == 0 || p.nb_full == n_blocks) break;
        const int dr = prefill_die_rows(m_blocks, p.nb_full, rest * p.ks, p.ks), dc = 8 / dr;
        if (((m_blocks + dr - 1) / dr) * ((p.nb_full + dc - 1) / dc) <= rounds * (cus / 8)) break;
    }
    return p;
}

// Relative cost of a plan in units of one 128-column block's group: whole rounds, then the
// sliced round, then the exchange of its partial tiles (wider blocks take about 1.3 times as
// long per group and exchange twice the data).
// A 128-row block takes 1.5 times as long per group as a 64-row one, exchanges at four times the price per
// slice, and its launch carries 6 units more (the row sums from a launch in front, a longer prologue and
// store): fitted to 98 cases -- 14 shapes at 400 ... 4096 rows, each with 64- and 128-row blocks forced --
// and to 72 more -- 12 shapes of other models at 129 ... 512 rows, the three block shapes forced -- on which
// the cheaper plan by this cost is the faster one or within 0.8 % (the former) and 0.6 % (the latter) of it
// on average, 18 % and 5 % at worst.
static float plan_cost(int m, int n, int k, int cus, const PrefillPlan &p) {
    const int G = k / kGroupK, m_blocks = (m + p.bm - 1) / p.bm, n_blocks = n / p.bn;
    const float rows = p.bm == 128 ? 1.5f : 1.0f;
    const float per_group = (p.bn == 256 ? 1.3f : 1.0f) * rows;
    const float per_slice = (p.bm == 128 ? 2.0f : 0.5f) * rows;
    float cost = (float)((m_blocks * n_blocks) / cus) * G * per_group + (p.bm == 128 ? 6.f : 0.f);
    if (n_blocks > p.nb_full) {
        cost += (float)((G + p.ks - 1) / p.ks) * per_group;
        if (p.ks > 1) cost += per_slice * p.ks;
        // 128-row blocks sit two to a unit: behind whole rounds, the blocks of a K-sliced rest run beside the last round's
        // and hold it up by their own length, in proportion to how many of them there are (gate+up at 640
        // rows, 255 whole tiles and 105 in two slices of ten groups: 87.5 us, 73 with every tile whole or in
        // 64-row blocks; at 512 rows, 32 tiles in five slices of four groups: nothing)
        // (0.75 of that, and nothing for a rest of whole tiles, which is a round like the others: fitted with the rest)
        if (p.bm == 128 && p.nb_full > 0 && p.ks > 1)
            cost += 0.75f * (float)((n_blocks - p.nb_full) * m_blocks * p.ks) / cus * ((G + p.ks - 1) / p.ks) * per_group;
    }
    return cost;
}

// Block shape for a problem.  64-row blocks (four wavefronts side by side, three blocks per compute
// unit) for small problems, which are bound by latency and by how evenly the tiles cover the chip,
// not by the matrix cores (rows past M are computed and dropped); 128 x 256 blocks (four wavefronts
// side by side, each 128 x 64) where the chip is saturated: the best measured rate, because every
// wavefront's weights are its own and A is shared by all four.  Which of the two, and which width
// of the 64-row block: the lower modelled cost (plan_cost); up to 128 rows always 64 (until the 129...512-row
// sweep it was 384, and 128 x 256 blocks in K slices were missed where they lead by 15...25 %: 18944 -> 3584 at
// 321 rows 81.5 us against 107, 28672 -> 8192 at 256 rows 150 against 173, 6144 -> 6144 at 321 rows 51 against 68).  (A fixed
// switch at 768 rows was 5 % slower on average over the same 98 cases and 69 % at worst: narrow
// outputs want 64 rows at any row count, large products 128 rows from 400 on.)
// The 256-row shapes stay available through the overrides.
PrefillPlan plan_prefill(int m, int n, int k, int cus, int force_bn, int force_bm) {
    // 128-row tiles for 50...100 % of the compute units: two such blocks fit a unit, and with every tile cut
    // into as many K slices as fill those slots the chip is busier than with 64-row blocks, provided a slice
    // stays long (measured on N = 2560: K = 9216 at M = 2048 / 2560 / 3072, three or two slices of 24 or 36
    // groups, 121 / 148 / 162 us against 124 / 159 / 168; K = 4096 at M = 3072 in two slices of 16 groups
    // 90 against 84)
    int sliced_units = 0;
    {
        const int tiles = ((m + 127) / 128) * (n / 256);
        if (2 * tiles >= cus && tiles < cus) {
            const int ks = 2 * cus / tiles;
            // (shorter slices where the tiles leave a quarter of the units idle or more: 160 tiles of 8192 -> 10240 at
            // 448...512 rows in three slices of 21 / 22 groups 103.5 us against 119 in two and 114...125 in 64-row
            // blocks; 128 tiles of 8192 -> 8192, 14336 -> 8192, 28672 -> 8192 in four slices 3...8 % ahead of two)
            const int min_groups = 4 * tiles <= 3 * cus ? 16 : 24;
            if (ks >= 2 && k / kGroupK / ks >= min_groups) sliced_units = 2 * cus;
        }
    }
    if (force_bm == 64 || force_bm == 128 || force_bm == 256) {
        const int bm = force_bm;
        if (force_bn == 128 || force_bn == 256) return plan_for_shape(m, n, k, cus, force_bn, bm);
        const PrefillPlan wide = plan_for_shape(m, n, k, cus, 256, bm, bm == 128 ? sliced_units : 0);
        if (bm == 128) return wide;
        const PrefillPlan narrow = plan_for_shape(m, n, k, cus, 128, bm);
        if (bm == 64) return plan_cost(m, n, k, cus, narrow) <= plan_cost(m, n, k, cus, wide) ? narrow : wide;
        // 256-row blocks: narrow unless its tiles neither fill a round nor can be sliced
        if (narrow.nb_full == 0 && narrow.ks == 1 && wide.nb_full == 0 && wide.ks >= 2) return wide;
        return narrow;
    }
    // 64-row blocks of either width, and from 385 rows on 128 x 256 blocks: whichever the cost model prices lower
    PrefillPlan best = plan_for_shape(m, n, k, cus, force_bn == 128 ? 128 : 256, 64);
    if (force_bn != 128 && force_bn != 256) {
        const PrefillPlan narrow = plan_for_shape(m, n, k, cus, 128, 64);
        // (not as whole rounds plus a rest in five slices or more: 4096 -> 12288 at 129...192 rows ran 70.7 us as
        // 85 whole column blocks and 11 in seven slices against 47.4 as 64 x 256 blocks, 6144 -> 6144 at 321 rows
        // 103 against 68.5)
        const bool rest_in_many_slices = narrow.nb_full > 0 && narrow.ks >= 5;
        // Two wavefronts a block: for outputs too narrow to give the wider block enough tiles (2560 -> 1024 at
        // 400...4096 rows 17...36 us against 27...43).  On wider outputs the model's 1.0 : 1.3 a group does not hold
        // where a compute unit gets one such block (3584 -> 4608 at 448 rows, 252 tiles: 65 us, 38...44 in the other
        // shapes), and over 170 forced cases it never led by more than 3 % there.
        const bool narrow_output = n <= 2048;
        if (narrow_output && !rest_in_many_slices && plan_cost(m, n, k, cus, narrow) <= plan_cost(m, n, k, cus, best))
            best = narrow;
    }
    if (m > 128 && force_bn != 128) {
        const PrefillPlan tall = plan_for_shape(m, n, k, cus, 256, 128, sliced_units);
        if (plan_cost(m, n, k, cus, tall) < plan_cost(m, n, k, cus, best)) best = tall;
    }
    return best;
}
size_t prefill_partial_bytes(int m, int n, const PrefillPlan &p) {
    if (p.ks <= 1) return 0;
    return (size_t)((m + p.bm - 1) / p.bm) * p.bm * (size_t)(n - p.nb_full * p.bn) * p.ks * sizeof(float);
}

namespace {

// Bytes of LDS for the in-kernel row sums of a 64-row block covering `groups` groups of K.
constexpr int kMaxRowSumBytes = 24 * 1024;
static int row_sum_bytes(int groups) { return groups * 64 * (int)sizeof(float); }


template <int NWN, int WM, int MI, bool SWIGLU, bool RS, bool FOLD = false>
hipError_t launch_shape_as(const PrefillArgs &a, int grid, int m_blocks, int RP, int KS, int GSb, int max_groups,
                           hipStream_t stream, const PrefillFold &pf = PrefillFold{}) {
    constexpr int BM = WM * MI * 32, NW = WM * NWN;
    constexpr int kRing = kAStages * BM * 64;       // the A ring
    constexpr int kStore = NW * MI * 32 * 64 * 2;   // the store's per-wavefront transposes (reuses the ring)
    // RS: the row sums sit behind the ring and are dead by the time the store reuses the space
    constexpr int kLdsMax = RS ? (kRing + kMaxRowSumBytes > kStore ? kRing + kMaxRowSumBytes : kStore)
                               : (kRing > kStore ? kRing : kStore);
    int lds_bytes = kRing > kStore ? kRing : kStore;
    if (RS && kRing + row_sum_bytes(max_groups) > lds_bytes) lds_bytes = kRing + row_sum_bytes(max_groups);
    // The 256 x 128 block fits twice on a compute unit.  A grid of at most one block per unit
    // asks for more LDS than two blocks could share, so the dispatcher cannot stack two blocks
    // on one unit while others idle.
    constexpr int kLdsSolo0 = (WM == 2 && NWN == 2) ? 96 * 1024 : kLdsMax;
    constexpr int kLdsSolo = FOLD && kLdsSolo0 < kProjectLdsBytes16 ? kProjectLdsBytes16 : kLdsSolo0;
    const hipError_t attr = allow_dynamic_lds<&w4a16_prefill_kernel<NWN, WM, MI, SWIGLU, RS, FOLD>>(kLdsSolo);
    if (attr != hipSuccess) return attr;
    if (WM == 2 && NWN == 2 && grid <= a.cus) lds_bytes = kLdsSolo;
    if (FOLD && lds_bytes < kProjectLdsBytes16) lds_bytes = kProjectLdsBytes16;  // the projection's blocks stage more
    w4a16_prefill_kernel<NWN, WM, MI, SWIGLU, RS, FOLD><<<grid + (FOLD ? pf.producers : 0), 64 * NW, lds_bytes, stream>>>(
        (const uint16_t *)a.A, (const u32x4 *)a.B, (const uint16_t *)a.S, (uint16_t *)a.C, (const u32x4 *)a.aext,
        a.M, a.N, a.K, a.Gs, m_blocks, (const uint16_t *)a.lora_t, (const uint16_t *)a.lora_b, a.r_total, RP,
        a.nb_full, KS, GSb, a.partial, a.counters,
        prefill_die_rows(m_blocks, a.nb_full, (a.N / (NWN * 64) - a.nb_full) * KS, KS), pf);
    return hipGetLastError();
}

template <int NWN, int WM, int MI>
hipError_t launch_shape(const PrefillArgs &a, int grid, int m_blocks, int RP, int KS, int GSb, int max_groups,
                        bool rs, hipStream_t stream) {
    if constexpr (MI == 2) {
        if (rs)
            return a.swiglu ? launch_shape_as<NWN, WM, MI, true, true>(a, grid, m_blocks, RP, KS, GSb, max_groups, stream)
                            : launch_shape_as<NWN, WM, MI, false, true>(a, grid, m_blocks, RP, KS, GSb, max_groups, stream);
    }
    return a.swiglu ? launch_shape_as<NWN, WM, MI, true, false>(a, grid, m_blocks, RP, KS, GSb, max_groups, stream)
                    : launch_shape_as<NWN, WM, MI, false, false>(a, grid, m_blocks, RP, KS, GSb, max_groups, stream);
}

}  // namespace

// K slices of the projection for few rows (the small-M kernels multiply T): up to 16, each staging
// two pieces; the consumer runs over them as if they were further rank columns, which costs it
// less than a meeting of the blocks would cost here.
int lora_project_slices(int m, int k) {
    const int pieces = (k + kProjectPieceK - 1) / kProjectPieceK;
    int kz = (pieces + 1) / 2;
    if (kz > prefill_lora_max_slices(m)) kz = prefill_lora_max_slices(m);
    return kz < 1 ? 1 : kz;
}

// Many rows: rows per block, row tiles, K slices (as many as keep about 256 blocks busy) and steps of
// 32 values per slice (whole groups).
static void project_slicing(int m, int k, bool have_counters, int *rb_out, int *row_tiles_out, int *kz_out, int *per_slice_out) {
    const int steps = k / 32;
    const int rb = lora_project_rows_per_block(m, k), row_tiles = (m + rb - 1) / rb;
    const int pieces = (k + kProjectPieceK - 1) / kProjectPieceK;
    int kz = (256 + row_tiles - 1) / row_tiles;
    const int zmax = rb == 16 ? 16 : 8;  // what the kernel's meeting reads in one go
    if (kz > zmax) kz = zmax;
    if (kz > pieces) kz = pieces;
    if (row_tiles > kProjectMaxCounters || !have_counters) kz = 1;
    const int per_slice = ((steps + kz - 1) / kz + 3) / 4 * 4;
    kz = (steps + per_slice - 1) / per_slice;
    *rb_out = rb;
    *row_tiles_out = row_tiles;
    *kz_out = kz;
    *per_slice_out = per_slice;
}

hipError_t launch_lora_project(const PrefillArgs &a, bool few_rows, hipStream_t stream, int *slices, bool with_row_sums) {
    if (a.r_total < 1 || a.r_total > kProjectMaxRank || a.n_adapters < 1 || a.n_adapters > 8 || !a.lora_a ||
        !a.lora_t || !a.ranks || !a.scales || a.M < 1 || a.K < kGroupK)
        return hipErrorInvalidValue;
    const int RP = (a.r_total + 15) / 16 * 16;
    LoraScales ls;
    ls.count = a.n_adapters;
    int end = 0;
    for (int i = 0; i < 8; ++i) {
        if (i < a.n_adapters) end += a.ranks[i];
        ls.ends[i] = end;
        ls.scales[i] = i < a.n_adapters ? a.scales[i] : 0.f;
    }
    *slices = 1;
    const int steps = a.K / 32;
    u32x4 *aext = with_row_sums && !few_rows ? (u32x4 *)a.aext : nullptr;
    if (with_row_sums && !aext) return hipErrorInvalidValue;
    if (!few_rows) {
        // many rows: T whole.  K slices that meet in f32 behind T, as many as keep about 256 blocks busy.
        int rb, row_tiles, kz, per_slice;
        project_slicing(a.M, a.K, a.counters != nullptr, &rb, &row_tiles, &kz, &per_slice);
        float *partial = reinterpret_cast<float *>(reinterpret_cast<char *>(a.lora_t) + (size_t)a.M * 64 * sizeof(uint16_t));
        const int lds_bytes = (rb + kProjectMaxRank) * kProjectRowBytes + kProjectMaxRank * (int)sizeof(float);
        if (rb == 16) {
            w4a16_lora_project_kernel<16><<<dim3(row_tiles, kz), 256, lds_bytes, stream>>>(
                (const uint16_t *)a.A, (const uint16_t *)a.lora_a, (uint16_t *)a.lora_t, a.M, a.K, a.r_total, RP,
                per_slice, ls, partial, a.counters, aext);
        } else {
            const hipError_t attr = allow_dynamic_lds<&w4a16_lora_project_kernel<64>>(lds_bytes);
            if (attr != hipSuccess) return attr;
            w4a16_lora_project_kernel<64><<<dim3(row_tiles, kz), 256, lds_bytes, stream>>>(
                (const uint16_t *)a.A, (const uint16_t *)a.lora_a, (uint16_t *)a.lora_t, a.M, a.K, a.r_total, RP,
                per_slice, ls, partial, a.counters, aext);
        }
        return hipGetLastError();
    }
    int kz = lora_project_slices(a.M, a.K);
    const int per_slice = ((steps + kz - 1) / kz + 3) / 4 * 4;  // whole 128-value groups
    kz = (steps + per_slice - 1) / per_slice;
    *slices = kz;
    const int lds_bytes = (16 + kProjectMaxRank) * kProjectRowBytes + kProjectMaxRank * (int)sizeof(float);
    w4a16_lora_project_kernel<16><<<dim3((a.M + 15) / 16, kz), 256, lds_bytes, stream>>>(
        (const uint16_t *)a.A, (const uint16_t *)a.lora_a, (uint16_t *)a.lora_t, a.M, a.K, a.r_total, RP, per_slice, ls,
        nullptr, nullptr, nullptr);
    return hipGetLastError();
}

// 64-row blocks form the row sums themselves when they fit next to the A ring and the launch is
// bound by latency rather than by work (measured: -2...-10 % up to about 28 GFLOP or on narrow
// outputs, +6...+8 % beyond, where the extra VALU and LDS work in the main loop costs more
// than the saved pre-pass launch)
static bool blocks_sum_their_rows(int M, int N, int K, const PrefillPlan &p) {
    const int G = K / kGroupK, ks = p.ks < 1 ? 1 : p.ks;
    // most groups of K any one block covers: all of them for a whole tile
    const int max_groups = p.nb_full > 0 ? G : (G + ks - 1) / ks;
    const double flops = 2.0 * M * (double)N * K;
    return p.bm == 64 && row_sum_bytes(max_groups) <= kMaxRowSumBytes && (flops <= 28e9 || N <= 4096);
}

// Without adapters a few of the product's own first blocks form the row sums (rowsum_producer_block)
// where the launch is a single round of blocks that leaves block slots free: producers in those
// slots cost the product nothing and save the launch in front (down projection at 2048 rows
// 116 -> 112 us, 2560 -> 8192 at 777 rows 61 -> 59.5).  They must be done before the first block's main
// loop is: at least one per 64 rows (its piece of A then streams in about half that time, whatever
// K), as many as there are free slots up to one per 16-row tile.  In a launch of several rounds the
// producers' slots are taken from the product: measured 2 to 5 us slower than the launch in front
// (gate+up at 2048 and 4096 rows), so those keep it.  0: from the launch in front; -2: the blocks sum
// their rows themselves.
int prefill_rowsum_producers(int M, int N, int K, const PrefillPlan &p, int cus) {
    if (blocks_sum_their_rows(M, N, K, p)) return -2;
    if ( p.bn != 256 || (p.bm != 64 && p.bm != 128) ||
        (M + 15) / 16 > kPrefillFoldMaxTiles || p.nb_full < 0 || p.nb_full > N / p.bn)
        return 0;
    const int grid = prefill_grid(M, N, p), slots = cus * (p.bm == 128 ? 2 : 3);
    const int want = ((M + 63) / 64 + 7) / 8 * 8, tiles8 = ((M + 15) / 16 + 7) / 8 * 8;
    const int free_slots = (slots - grid) / 8 * 8;
    if (free_slots < want) return 0;
    const int producers = free_slots < tiles8 ? free_slots : tiles8;
    return producers < 128 ? producers : 128;
}

hipError_t launch_prefill(const PrefillArgs &a, hipStream_t stream) {
    const int G = a.K / kGroupK;
    if (a.bm != 64 && a.bm != 128 && a.bm != 256) return hipErrorInvalidValue;
    const int KS_ = a.KS < 1 ? 1 : a.KS;
    PrefillPlan shape;
    shape.bn = a.bn;
    shape.bm = a.bm;
    shape.ks = KS_;
    shape.nb_full = a.nb_full;
    const int max_groups = a.nb_full > 0 ? G : (G + KS_ - 1) / KS_;
    const bool rs = blocks_sum_their_rows(a.M, a.N, a.K, shape);
    hipError_t err = hipSuccess;
    // with adapters the projection's launch forms the row sums on its way over x
    const bool sums_with_projection = !rs && a.r_total > 0;
    const int inside = a.r_total == 0 && a.lora_words ? prefill_rowsum_producers(a.M, a.N, a.K, shape, a.cus) : 0;
    const int sum_producers = inside > 0 ? inside : 0;
    if (!rs && !sums_with_projection && sum_producers == 0) {
        const int items = a.M * G;
        w4a16_prefill_rowsum_kernel<<<(items + 15) / 16, 256, 0, stream>>>((const uint16_t *)a.A, (u32x4 *)a.aext,
                                                                          a.M, a.K);
        err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    int RP = 0;
    // The projection inside the product's launch (PrefillFold): four-wavefront blocks, 16-row tiles of T,
    // the extension operand from the projection (unless the blocks sum their rows themselves), and room
    // for its counters behind the product's.
    PrefillFold pf{};
    bool fold = false;
    if (a.r_total > 0) {
        RP = (a.r_total + 15) / 16 * 16;
        int rb = 0, row_tiles = 0, kz = 0, per_slice = 0;
        project_slicing(a.M, a.K, a.counters != nullptr, &rb, &row_tiles, &kz, &per_slice);
        const int sliced_tiles = (a.N / a.bn - a.nb_full) * ((a.M + a.bm - 1) / a.bm);
        // A product that fits the chip's block slots in one go must still fit them with the projection's blocks
        // in front: the blocks that find no slot start when the producers leave, on whichever units the
        // dispatcher picks, and two of them on one unit beside idle units take 1.6 times as long as one (4096 ->
        // 4096 at 1700 rows, 224 blocks of 128 x 256 and 328 producers for 512 slots: 121 us against 86 at 1600
        // rows, 300 + 208 blocks; 97 with the projection in front).  So the projection is cut into fewer K slices
        // there -- its blocks stay far shorter than the product's -- and runs in front if its row tiles alone do
        // not fit.  Launches of several rounds keep all slices (gate+up at 2048 rows 189 us inside, 194 in front), and
        // so do 64-row blocks, three to a unit, which were never seen to suffer (gate+up at 512 rows, 768 blocks and
        // 256 producers for 768 slots: 62 us inside, 68 in front).
        bool room = true;
        if (rb == 16 && a.bm == 128) {
            const int slots = a.cus * 2, product = prefill_grid(a.M, a.N, shape);
            if (product <= slots && product + (row_tiles * kz + 7) / 8 * 8 > slots) {
                const int cap = (slots - product) / 8 * 8 / row_tiles;
                room = cap >= 1;
                if (room) {
                    const int steps = a.K / 32;
                    per_slice = ((steps + cap - 1) / cap + 3) / 4 * 4;
                    kz = (steps + per_slice - 1) / per_slice;
                }
            }
        }
        fold = room && a.lora_words && a.bn == 256 && (a.bm == 64 || a.bm == 128) && rb == 16 &&
               a.counters && row_tiles <= kPrefillFoldMaxTiles && row_tiles <= kProjectMaxCounters - kProjectFoldCounters &&
               sliced_tiles <= kProjectFoldCounters && a.n_adapters >= 1 && a.n_adapters <= 8 && a.lora_a && a.lora_t &&
               a.ranks && a.scales && a.r_total <= kProjectMaxRank;
        if (fold) {
            pf.a_cat = (const uint16_t *)a.lora_a;
            pf.t = (uint16_t *)a.lora_t;
            pf.aext = rs ? nullptr : (u32x4 *)a.aext;  // blocks that sum their rows themselves need no operand
            pf.partial = reinterpret_cast<float *>(reinterpret_cast<char *>(a.lora_t) + (size_t)a.M * 64 * sizeof(uint16_t));
            pf.counters = a.counters + kProjectFoldCounters;
            pf.words = a.lora_words;
            pf.row_tiles = row_tiles;
            pf.kz = kz;
            pf.steps_per_slice = per_slice;
            pf.producers = (row_tiles * kz + 7) / 8 * 8;
            pf.ls.count = a.n_adapters;
            int end = 0;
            for (int i = 0; i < 8; ++i) {
                if (i < a.n_adapters) end += a.ranks[i];
                pf.ls.ends[i] = end;
                pf.ls.scales[i] = i < a.n_adapters ? a.scales[i] : 0.f;
            }
        } else {
            int slices = 1;  // many rows: T is whole
            err = launch_lora_project(a, false, stream, &slices, sums_with_projection);
            if (err != hipSuccess) return err;
            if (slices != 1) return hipErrorInvalidValue;
        }
    }
    if (sum_producers > 0) {
        fold = true;
        pf.aext = (u32x4 *)a.aext;
        pf.words = a.lora_words;
        pf.row_tiles = (a.M + 15) / 16;
        pf.producers = sum_producers;
        pf.sum_tiles = (pf.row_tiles + sum_producers - 1) / sum_producers;
    }
    if (a.bn != 128 && a.bn != 256) return hipErrorInvalidValue;
    const int m_blocks = (a.M + a.bm - 1) / a.bm;
    const int KS = a.KS < 1 ? 1 : a.KS;
    const int GSb = (G + KS - 1) / KS;
    if (KS > 1 && (!a.partial || !a.counters || (KS - 1) * GSb >= G)) return hipErrorInvalidValue;
    if (a.nb_full < 0 || a.nb_full > a.N / a.bn) return hipErrorInvalidValue;
    const int grid = prefill_grid(a.M, a.N, shape);
    if (fold) {
        pf.consumers = grid;
        if (a.swiglu) {
            if (a.bm == 128) return launch_shape_as<4, 1, 4, true, false, true>(a, grid, m_blocks, RP, KS, GSb, max_groups, stream, pf);
            return rs ? launch_shape_as<4, 1, 2, true, true, true>(a, grid, m_blocks, RP, KS, GSb, max_groups, stream, pf)
                      : launch_shape_as<4, 1, 2, true, false, true>(a, grid, m_blocks, RP, KS, GSb, max_groups, stream, pf);
        }
        if (a.bm == 128) return launch_shape_as<4, 1, 4, false, false, true>(a, grid, m_blocks, RP, KS, GSb, max_groups, stream, pf);
        return rs ? launch_shape_as<4, 1, 2, false, true, true>(a, grid, m_blocks, RP, KS, GSb, max_groups, stream, pf)
                  : launch_shape_as<4, 1, 2, false, false, true>(a, grid, m_blocks, RP, KS, GSb, max_groups, stream, pf);
    }
    if (a.bm == 256) {
        return a.bn == 256 ? launch_shape<4, 2, 4>(a, grid, m_blocks, RP, KS, GSb, max_groups, rs, stream)
                           : launch_shape<2, 2, 4>(a, grid, m_blocks, RP, KS, GSb, max_groups, rs, stream);
    } else if (a.bm == 128) {
        return a.bn == 256 ? launch_shape<4, 1, 4>(a, grid, m_blocks, RP, KS, GSb, max_groups, rs, stream)
                           : launch_shape<2, 1, 4>(a, grid, m_blocks, RP, KS, GSb, max_groups, rs, stream);
    }
    return a.bn == 256 ? launch_shape<4, 1, 2>(a, grid, m_blocks, RP, KS, GSb, max_groups, rs, stream)
                       : launch_shape<2, 1, 2>(a, grid, m_blocks, RP, KS, GSb, max_groups, rs, stream);
}

}  // namespace kiln
