// Small-M (decode) W4A16 GEMM kernel for gfx950: group-major split with wavefront-private
// staging of the activations.
//
// Same arm of the reference dispatcher as the other small-M kernels
// (crates/kiln-marlin-gemm/csrc/marlin_kernel.cu:754-763, :189-700) and the same inner step:
// 1 KiB chunks (16 columns x 128 rows) by one 128-bit load per lane, codes expanded to bf16 in
// registers, v_mfma_f32_16x16x32_bf16, scales applied in f32.  What differs is where the
// activations live and what the block waits for:
//   * a block holds T whole column tiles of one K slice and wavefront w owns a run of the
//     slice's groups (as in the group-major instances), but each wavefront stages the rows of A of
//     its own groups into its own piece of LDS with LDS-direct loads (1 KiB per instruction: four
//     rows of one group, fully coalesced) -- nobody else reads them, so there is no barrier before
//     the first product, a wavefront waits for its own loads only, and a slice may be as long as
//     K: the down projection runs unsliced, without the exchange through the workspace;
//   * the weight requests are the first memory instructions of the kernel, ahead of the
//     activations (which come from L2 and land first anyway);
//   * K slices, where a plan still has them, meet tile by tile without a block-wide barrier: up to
//     four slices store their parts as their own arrival flags (complemented f32 words in workspace
//     that is zero between launches) and the last slice's wavefront polls, adds in slice order and
//     writes the zeros back; plans beyond that count arrivals -- the wavefront that summed a tile
//     stores its part, waits for its own stores, counts, and the last one adds.
#include <cstddef>

#include "async_loads.h"
#include "launch.h"
#include "lora_tail.h"

namespace kiln {

namespace {

constexpr int kGmpMaxWaves = 16;
constexpr int kGmpSlotBytes = 16 * 256;  // one group of A: 16 rows x 128 bf16
#ifndef KILN_GMP_HEAD
#define KILN_GMP_HEAD 3
#endif
// This file is compiled twice: as it is for calls without adapters, and with -DKILN_GMP_LORA=1 for
// calls with them (launch_decode_gmp_lora only).  What the low-rank term adds -- one wavefront more,
// its arguments, the signalling between the wavefronts -- then costs calls without adapters
// nothing: as one kernel with run-time branches it cost them 0.1...0.2 us per launch.
#ifndef KILN_GMP_LORA
#define KILN_GMP_LORA 0
#endif
constexpr bool kGmpLora = KILN_GMP_LORA != 0;

// Probe builds only (-DKILN_GMP_TIMELINE): wall-clock stamps (100 MHz) per wavefront.
#ifdef KILN_GMP_TIMELINE
#if KILN_GMP_LORA
#define g_gmp_tl g_gmp_tl_lora
#endif
__device__ long long *g_gmp_tl;
#define KILN_GMP_TL(i, v) tl_[i] = (v)
#define KILN_GMP_NOW() ((long long)__builtin_amdgcn_s_memrealtime())
#else
#define KILN_GMP_TL(i, v) \
    do {                  \
    } while (0)
#define KILN_GMP_NOW() 0ll
#endif

constexpr int kGmpHead = KILN_GMP_HEAD;  // chunks requested ahead of the one being consumed
constexpr int kGmpMaxChunks = 16;        // chunks per wavefront, at most (straight-line code)

// Issue order of a wavefront's loads (chunk j = group j / T, tile j % T: 2 loads each; A(g): AQ
// LDS-direct loads into slot g % 2):
//   before the first step: chunks 0 ... HEAD - 1, then A(0);
//   step j: chunk j + HEAD; at the start of group g = j / T: A(g + 1) (its slot's last reader,
//   group g - 1, is done), [wait for A(g)], fragments to registers; then [wait for chunk j], products.
// The activations of a group are requested one group ahead, not all at once: every block stages
// its own copy of the slice, as many bytes through L2 as the weights at 16 rows, and a burst of
// them at the start keeps the wavefronts in the issue stage while the weight stream runs dry.
struct GmpSchedule {
    int wait_a[kGmpMaxChunks];      // by group
    int wait_chunk[kGmpMaxChunks];  // by chunk
};
constexpr GmpSchedule gmp_schedule(int T, int groups, int AQ) {
    const int U = T * groups;
    int kind[3 * kGmpMaxChunks] = {}, idx[3 * kGmpMaxChunks] = {}, size[3 * kGmpMaxChunks] = {};
    int n = 0;
    auto push = [&](int k, int i, int sz) {
        kind[n] = k;
        idx[n] = i;
        size[n] = sz;
        ++n;
    };
    auto issued_after = [&](int k, int i) {
        int after = 0;
        bool seen = false;
        for (int e = 0; e < n; ++e) {
            if (seen) after += size[e];
            if (kind[e] == k && idx[e] == i) seen = true;
        }
        return after;
    };
    for (int j = 0; j < kGmpHead && j < U; ++j) push(1, j, 2);
    push(0, 0, AQ);
    GmpSchedule s{};
    for (int j = 0; j < U; ++j) {
        if (j + kGmpHead < U) push(1, j + kGmpHead, 2);
        if (j % T == 0) {
            const int g = j / T;
            if (g + 1 < groups) push(0, g + 1, AQ);
            s.wait_a[g] = issued_after(0, g);
        }
        s.wait_chunk[j] = issued_after(1, j);
    }
    return s;
}
template <int T, int GROUPS, int AQ>
struct GmpScheduleOf {
    static constexpr GmpSchedule value = gmp_schedule(T, GROUPS, AQ);
};

constexpr int gmp_slots(int gpw) { return gpw < 2 ? gpw : 2; }
constexpr int kGmpFlaggedSlices = kDecodeFlaggedMaxSlices;  // most K slices the counter-free exchange takes
constexpr int kGmpSpinLimit = 1 << 20;  // polls of the other slices' parts before the adding wavefront gives up

// `units` 16-byte units from global memory (src: the same for the whole wavefront) to LDS at lds_addr
// by one wavefront, 1 KiB per LDS-direct load, all of them in flight at once; done when the
// wavefront's vector loads have landed.  The last load re-reads the last unit in its spare lanes:
// up to 1 KiB - 16 bytes behind the destination are overwritten.
__device__ __forceinline__ void copy_to_lds(unsigned lds_addr, const uint16_t *src, int units, int lane) {
    for (int base = 0; base < units; base += 64)
        load_to_lds_b128(src, (uint32_t)min(base + lane, units - 1) * 16u, lds_addr + (unsigned)base * 16u);
}

// One word of LDS as a signal from the adapter wavefront to the wavefronts that add the low-rank
// term: LDS serves its requests in order, so whoever reads the word set reads the operands that
// were written before it.  The wait is bounded like every other wait here.
__device__ __forceinline__ void lds_signal_store(unsigned lds_addr, uint32_t value) {
    asm volatile("ds_write_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : : "v"(lds_addr), "v"(value) : "memory");
}
__device__ __forceinline__ void lds_signal_wait(unsigned lds_addr, int at_least) {
    for (int spins = 0; spins < kGmpSpinLimit; ++spins) {
        uint32_t seen;
        asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(seen) : "v"(lds_addr) : "memory");
        if (__builtin_amdgcn_readfirstlane((int)seen) >= at_least) break;
        __builtin_amdgcn_s_sleep(1);
    }
}
constexpr uint32_t kGmpLooked = 1, kGmpOperandsReady = 2;  // values of the signal word
// A count in LDS that wavefronts raise (after their own LDS writes, which LDS serves first) and
// others wait for: a barrier that only holds up those who need what the others wrote.
[[maybe_unused]] __device__ __forceinline__ void lds_count_arrival(unsigned lds_addr, int lane) {
    if (lane == 0) asm volatile("ds_add_u32 %0, %1" : : "v"(lds_addr), "v"(1u) : "memory");
}
// Two words at the start of the adapter wavefront's part of LDS: the signal and the arrival count.
constexpr unsigned kGmpSyncBytes = 16;

// The kernel's last argument and where it sits among the arguments: the kernel reads it late, through
// the argument segment's address (see there), so its place is spelled out as a struct with the
// kernel's parameter list.
struct GmpLoraArgs {
    LoraTail lo;
    LoraFold fold;
};
struct GmpKernelArgs {
    const uint16_t *A;
    const u32x4 *B;
    const uint16_t *S;
    uint16_t *C;
    float *partial;
    int *counters;
    int M, N, K, Gs, KS, GS, full_waves, slot_bytes, col_shift, producers, adapter, col_blocks, nw_all, swiglu, flagged;
    GmpLoraArgs la;
};
constexpr int kGmpLoraArgsOffset = (int)offsetof(GmpKernelArgs, la);
static_assert(sizeof(GmpLoraArgs) % 4 == 0, "read word by word");

// What only the end of the kernel needs -- where the result and the partial tiles go, how a tile is
// stored -- waits in vector registers, of which the kernel has plenty, while the main loop uses
// every scalar register there is for its addresses.
struct GmpTailArgs {
    uint16_t *C;
    float *partial;
    int *counters;
    int swiglu, flagged;
};
struct GmpParkedTail {
    uint32_t w[8];
};
[[maybe_unused]] __device__ __forceinline__ GmpParkedTail gmp_park(const GmpTailArgs &t) {
    struct Words {
        uint32_t w[8];
    } in = __builtin_bit_cast(Words, t);
    GmpParkedTail p;
#pragma unroll
    for (int i = 0; i < 8; ++i) asm volatile("v_mov_b32 %0, %1" : "=v"(p.w[i]) : "s"(in.w[i]));
    return p;
}
[[maybe_unused]] __device__ __forceinline__ GmpTailArgs gmp_unpark(const GmpParkedTail &p) {
    struct Words {
        uint32_t w[8];
    } out;
#pragma unroll
    for (int i = 0; i < 8; ++i) out.w[i] = (uint32_t)__builtin_amdgcn_readfirstlane((int)p.w[i]);
    return __builtin_bit_cast(GmpTailArgs, out);
}
static_assert(sizeof(GmpTailArgs) == 32, "eight words");

// T tiles per block, GPW groups per wavefront (the first `full_waves` wavefronts; the others one
// fewer), AQ = LDS-direct loads per group of A: 4 (16 rows), 2 (M <= 8) or 1 (M <= 4: rows 0...3
// only; the other rows of the product are computed from whatever LDS holds and never stored).
template <int T, int GPW, int AQ, bool LORA>
__global__ __launch_bounds__(kGmpMaxWaves * 64) void w4a16_decode_gmp_kernel(
    const uint16_t *__restrict__ A, const u32x4 *__restrict__ B, const uint16_t *__restrict__ S,
    uint16_t *__restrict__ C_arg, float *partial_arg, int *counters_arg, int M, int N, int K, int Gs, int KS, int GS,
    int full_waves, int slot_bytes, int col_shift, int producers_arg, int adapter_arg, int col_blocks, int nw_all,
    int swiglu_arg, int flagged_arg, GmpLoraArgs la) {
    const int producers = LORA ? producers_arg : 0, adapter = LORA ? adapter_arg : 0;
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
#ifdef KILN_GMP_TIMELINE
    long long tl_[8] = {};
#endif
    KILN_GMP_TL(0, KILN_GMP_NOW());
    // Everything the first requests depend on is fetched from the kernel arguments in one go: left to
    // itself the compiler fetches what lies behind the branch below only there, one more scalar
    // round trip (0.2 us) between the launch and the first weight request.
    asm volatile("" : : "s"(A), "s"(B), "s"(S), "s"(M), "s"(N), "s"(K), "s"(Gs), "s"(KS), "s"(GS), "s"(full_waves),
                 "s"(slot_bytes), "s"(col_shift), "s"(producers), "s"(adapter), "s"(col_blocks), "s"(nw_all));
    [[maybe_unused]] GmpParkedTail parked_tail;
    if constexpr (LORA) parked_tail = gmp_park(GmpTailArgs{C_arg, partial_arg, counters_arg, swiglu_arg, flagged_arg});
    constexpr int NS = gmp_slots(GPW);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // With adapters the block has one wavefront more than the main loop uses: it fetches what the
    // low-rank term needs into LDS while the others stream weights.
    const int nw = nw_all - adapter;  // nw_all = wavefronts of the block
    const bool adapter_wave = wave == nw;  // never true without adapters
    const int G = K / kGroupK;
    const int NT = N / kTileN;
    // Calls without a folded projection: grid (column blocks, K slices).  With one, a single row
    // of blocks: the `producers` blocks that compute it first, then the slices one after the other
    // (a second grid dimension would launch the producers' indices once per slice, and the idle
    // ones delay as many working blocks of the last slice by a round).
    int ks = blockIdx.y, bx = blockIdx.x;
    if (__builtin_expect(producers > 0, 0)) {
        if (bx < producers) {
            lora_project_slice(A, la.fold, la.lo, M, K, bx, lds, wave, lane, nw_all);
#ifdef KILN_GMP_TIMELINE
            if (lane == 0 && g_gmp_tl) {
                long long *o = g_gmp_tl + ((size_t)blockIdx.x * 16 + wave) * 8;
                o[0] = tl_[0];
                o[6] = KILN_GMP_NOW();
                o[7] = 100;
            }
#endif
            return;
        }
        bx -= producers;  // at most four slices with a folded projection (decode_gmp_fold_ok)
        ks = (bx >= col_blocks ? 1 : 0) + (bx >= 2 * col_blocks ? 1 : 0) + (bx >= 3 * col_blocks ? 1 : 0);
        bx -= ks * col_blocks;
    }
    // Blocks go to the eight dies round-robin by linear index.  With the counter-free exchange the
    // column block is shifted by col_shift per slice, so that the slices of a tile sit on different
    // dies: a device-scope store and the device-scope load that polls it are slow when they meet
    // in one die's L2 (measured: 2...3 us per poll instead of 0.5).
    const int col_block = (bx + ks * col_shift) % col_blocks;
    const int tf = col_block * T;  // first tile of the block; tiles from NT on do not exist
    const bool full = wave < full_waves;
    const int g_first = full ? wave * GPW : full_waves * GPW + (wave - full_waves) * (GPW - 1);
    const int g0 = ks * GS + g_first;  // all slices have GS groups
    const int gs_mask = (Gs == 1) ? 0 : -1;

    // chunk j of the wavefront = (group j / T, tile j % T); a tile past the end is read as the last
    // tile and never stored.  Four register sets rotate.
    u32x4 w[kGmpHead + 1];
    uint32_t sc[kGmpHead + 1];
    static_assert(2 * kGmpHead + 8 <= 63, "outstanding loads must fit the wait counter");
    const uint32_t b_lane = lane * 16, s_lane = (lane & 15) * 2;
    auto request_chunk = [&](auto jc) {
        constexpr int j = decltype(jc)::value;
        constexpr int gi = j / T, ti = j % T, set = j % (kGmpHead + 1);
        const int tt = min(tf + ti, NT - 1);
        const char *b_ptr = reinterpret_cast<const char *>(B) + ((size_t)tt * G + (g0 + gi)) * 1024;
        const char *s_ptr = reinterpret_cast<const char *>(S) + ((size_t)tt * Gs + ((g0 + gi) & gs_mask)) * (kTileN * 2);
        load_b128_streaming(w[set], b_ptr, b_lane);
        load_u16(sc[set], s_ptr, s_lane);
    };

    // A of one group: AQ loads of 4 rows x 256 bytes; lane i of load p fetches 16-byte unit
    // (i % 16) ^ (row % 16) of row 4 p + i / 16, so unit u of a row sits at position u ^ (row % 16)
    // and the 16 lanes that read one unit index of 16 rows hit 16 different positions.
    unsigned char *mine = lds + wave * slot_bytes;
    const unsigned mine_addr = (unsigned)(size_t)(lds_ptr_t)mine;
    const uint32_t row_pitch = (uint32_t)K * 2;
    auto request_a = [&](int gi, int slot) {
        const char *base = reinterpret_cast<const char *>(A) + (size_t)(g0 + gi) * 256;
        const uint32_t quad_row = (uint32_t)(lane >> 4) + opaque_zero();  // keeps the offsets local to this request
#pragma unroll
        for (int p = 0; p < AQ; ++p) {
            const uint32_t row = 4 * p + quad_row;
            const uint32_t off = min(row, (uint32_t)(M - 1)) * row_pitch + (((uint32_t)(lane & 15) ^ (row & 15)) << 4);
            load_to_lds_b128(base, off, mine_addr + slot * kGmpSlotBytes + p * 1024);
        }
    };

    const bf16x8 minus_bias = bf16x8_splat(0xC308C308u);  // bf16(-136) pairs
    const DequantConsts dq = dequant_consts();
    f32x4 y[T];
#pragma unroll
    for (int ti = 0; ti < T; ++ti) y[ti] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Straight-line code from the first request to the last use, one instance per group count.
    auto run = [&](auto nc) {
        constexpr int NGR = decltype(nc)::value, U = T * NGR;
        using Sch = GmpScheduleOf<T, NGR, AQ>;
        unrolled<0, (kGmpHead < U ? kGmpHead : U)>(request_chunk);
        request_a(0, 0);
        if constexpr (LORA) __syncthreads();  // the adapter wavefront has zeroed the words the block meets on
        u32x4 af[4];
        f32x4 offset_term;
        unrolled<0, U>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            constexpr int gi = j / T, ti = j % T, set = j % (kGmpHead + 1);
            if constexpr (j + kGmpHead < U) request_chunk(std::integral_constant<int, j + kGmpHead>{});
            if constexpr (ti == 0) {  // next group: fragments of its activations and its offset term
                if constexpr (gi + 1 < NGR) {  // one group ahead
                    // Its slot was read by group gi - 1.  Those reads were issued a group ago, but the
                    // compiler may sink the products that wait for them below this request: without a
                    // wait of its own the first rows of the new group can land under the last read.
                    if constexpr (gi + 1 >= NS) wait_lds_reads();
                    request_a(gi + 1, (gi + 1) % NS);
                }
                wait_vector_loads<Sch::value.wait_a[gi]>();
                const unsigned char *ap = mine + (gi % NS) * kGmpSlotBytes + (lane & 15) * 256;
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    af[t] = *reinterpret_cast<const u32x4 *>(ap + (((4 * t + (lane >> 4)) ^ (lane & 15)) << 4));
                offset_term = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    offset_term = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[t]), minus_bias,
                                                                          offset_term, 0, 0, 0);
            }
            wait_vector_loads<Sch::value.wait_chunk[j]>();
            pin_loaded(w[set]);
            pin_loaded(sc[set]);
            f32x4 acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[0]),
                                                                codes_to_bf16x8(w[set].x, dq), offset_term, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[1]), codes_to_bf16x8(w[set].y, dq),
                                                          acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[2]), codes_to_bf16x8(w[set].z, dq),
                                                          acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[3]), codes_to_bf16x8(w[set].w, dq),
                                                          acc, 0, 0, 0);
            y[ti] += acc * f16_bits_to_f32((uint16_t)sc[set]);
        });
    };
    if (__builtin_expect(!adapter_wave, 1)) {
        if (full) run(std::integral_constant<int, GPW>{});
        else if constexpr (GPW > 1) run(std::integral_constant<int, GPW - 1>{});
        // every wavefront's partial tiles into its own piece of LDS, then tile ti = their sum in
        // wavefront (= ascending K) order, one tile per wavefront at a time
        KILN_GMP_TL(1, KILN_GMP_NOW());
        f32x4 *slots = reinterpret_cast<f32x4 *>(mine);
#pragma unroll
        for (int ti = 0; ti < T; ++ti) slots[ti * 64 + lane] = y[ti];
    } else if constexpr (LORA) {
        const unsigned sync_addr = (unsigned)(size_t)(lds_ptr_t)(lds + nw * slot_bytes);
        lds_signal_store(sync_addr, 0u);
        lds_signal_store(sync_addr + 4, 0u);
        __syncthreads();  // pairs with the one behind the main wavefronts' first requests
    }

    // What the low-rank term needs is read from the kernel arguments only now: as ordinary
    // parameters these values would sit in scalar registers through the whole main loop, which
    // already uses nearly all of them.
    GmpLoraArgs late_args{};
    if (__builtin_expect(adapter != 0, 0)) {  // a call without adapters does not wait for these loads
        typedef const char __attribute__((address_space(4))) *kernarg_ptr_t;
        typedef const uint32_t __attribute__((address_space(4))) *kernarg_words_t;
        kernarg_ptr_t kernarg = (kernarg_ptr_t)__builtin_amdgcn_kernarg_segment_ptr();
        asm volatile("" : "+s"(kernarg));  // opaque: nothing read through it moves above this point
        kernarg_words_t src = (kernarg_words_t)(kernarg + kGmpLoraArgsOffset);
        struct Words {
            uint32_t w[sizeof(GmpLoraArgs) / 4];
        } words;
#pragma unroll
        for (int i = 0; i < (int)(sizeof(GmpLoraArgs) / 4); ++i) words.w[i] = src[i];
        late_args = __builtin_bit_cast(GmpLoraArgs, words);
    }
    const LoraTail &lo = late_args.lo;
    const LoraFold &fold = late_args.fold;
    // The low-rank term y += T * B_cat^T is added where a finished tile is stored, by the slice that
    // finishes it.  Its operands come from LDS behind the main wavefronts' slots: the adapter
    // wavefront copies the rows of B_cat that belong to the block's tiles at once, and T -- all of
    // it, [slices][M][rp] -- as soon as it exists: with the projection folded into this launch, when
    // every producer's flag is up.  It holds up nobody with that: the tiles are summed (and exchanged
    // between K slices) while T is on its way, and a word of LDS tells the summing wavefronts when
    // the operands are there.
    unsigned char *lora_b_lds = lds + nw * slot_bytes + kGmpSyncBytes;
    const int lora_b_bytes = (T * kTileN * lo.r_total * 2 + 15) & ~15;
    unsigned char *lora_t_lds = lora_b_lds + lora_b_bytes;
    // (evaluated where they are used: no scalar register held meanwhile)
    auto lora_t_units = [&] { return lo.slices * lo.t_rows * lo.rp / 8; };
    auto lora_ready_addr = [&] { return (unsigned)(size_t)(lds_ptr_t)(lds + nw * slot_bytes); };  // the signal word
    auto arrivals_addr = [&] { return lora_ready_addr() + 4u; };                                   // the arrival count
    const bool adds_term = adapter != 0 && ks == KS - 1;
    // Once the block has looked at the producers' flags it counts itself (the last block to do so
    // zeroes them for the next launch): two atomics in a row across the chip, which the last main
    // wavefront takes on where it has no tile to sum, so that they do not end the launch.
    auto counting_wave_exists = [&] { return nw - 1 >= min(T, NT - tf); };
    // Without adapters the block meets at a barrier.  With them it must not: the adapter wavefront
    // waits for the producers, and the main wavefronts of a fast block would wait with it.  There the
    // main wavefronts count their arrival in LDS, only those that sum a tile wait for the count, and
    // the adapter wavefront runs beside them from the first instruction on.
    if constexpr (!LORA) {
        __syncthreads();  // every wavefront's partial tiles are in LDS
    } else if (!adapter_wave) {
        lds_count_arrival(arrivals_addr(), lane);
    }
    KILN_GMP_TL(2, KILN_GMP_NOW());
    if (__builtin_expect(adapter_wave, 0)) {
        // This one copies the block's rows of B, waits for T (with the projection folded into the
        // launch: for every producer's flag), copies it behind the rows of B -- loads land in
        // issue order, so what the copy of B overwrote behind its end is overwritten again -- and
        // signals.
        if (adds_term) {
            const int live_tiles = min(T, NT - tf);
            copy_to_lds((unsigned)(size_t)(lds_ptr_t)lora_b_lds, lo.b + (size_t)tf * kTileN * lo.r_total,
                        live_tiles * kTileN * lo.r_total / 8, lane);
            if (fold.producers > 0) {
                KILN_GMP_TL(3, KILN_GMP_NOW());
                const int polls = lora_fold_wait(fold, tf / T, lane);
                if (__builtin_expect(polls == kLoraFoldSpinLimit, 0))
                    report_wait_gave_up(error_word_before_fold_words(fold.flags), kGaveUpDecodeFold, lane);
                KILN_GMP_TL(4, KILN_GMP_NOW());
                KILN_GMP_TL(5, (long long)polls + 1);
                lds_signal_store(lora_ready_addr(), kGmpLooked);
            }
            copy_to_lds((unsigned)(size_t)(lds_ptr_t)lora_t_lds, lo.t, lora_t_units(), lane);
            wait_vector_loads<0>();
            lds_signal_store(lora_ready_addr(), kGmpOperandsReady);
            if (fold.producers > 0 && !counting_wave_exists()) lora_fold_done(fold, tf / T, lane);
        }
#ifdef KILN_GMP_TIMELINE
        if (lane == 0 && g_gmp_tl) {
            long long *o = g_gmp_tl + (((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 16 + wave) * 8;
            for (int i = 0; i < 6; ++i) o[i] = tl_[i];
            o[6] = KILN_GMP_NOW();
            o[7] = 200;
        }
#endif
        return;
    }

    if (__builtin_expect(adds_term && fold.producers > 0 && wave == nw - 1 && counting_wave_exists(), 0)) {
        lds_signal_wait(lora_ready_addr(), kGmpLooked);
        lora_fold_done(fold, tf / T, lane);  // tf / T: the column block
        return;
    }

    GmpTailArgs tail{C_arg, partial_arg, counters_arg, swiglu_arg, flagged_arg};
    if constexpr (LORA) tail = gmp_unpark(parked_tail);
    uint16_t *const C = tail.C;
    float *const partial = tail.partial;
    int *const counters = tail.counters;
    const int swiglu = tail.swiglu, flagged = tail.flagged;
    const int q4 = lane >> 4, c = lane & 15;
    const int tiles = min(T, NT - tf);
    if constexpr (LORA) {
        if (wave < tiles) lds_signal_wait(arrivals_addr(), nw);  // every main wavefront's partial tiles are in LDS
    }
    for (int ti = wave; ti < tiles; ti += nw) {
        const int tt = tf + ti;
        // (requesting all wavefronts' parts at once and adding them behind selects measured
        // 0.1...0.3 us slower per launch than this loop)
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int wv = 0; wv < nw; ++wv) sum += reinterpret_cast<const f32x4 *>(lds + wv * slot_bytes)[ti * 64 + lane];
        if (KS > 1 && flagged) {
            // The slices of the tile meet in a part of the workspace that is all zero between
            // launches.  A word there is either zero (not written yet) or the complement of a
            // partial sum's bits (a sum never has all bits set: that is a NaN whose payload no
            // arithmetic here produces), so the data is its own arrival flag: no counter, no
            // wait for the stores.  The last slice adds the parts; its blocks are dispatched after
            // all others (grid y is the slice), so every block it waits for is running or done.
            uint32_t *own = reinterpret_cast<uint32_t *>(partial) + ((size_t)ks * NT + tt) * 256 + lane * 4;
            KILN_GMP_TL(3, KILN_GMP_NOW());
            if (ks != KS - 1) {
                const u32x4 bits = __builtin_bit_cast(u32x4, sum);
                store_b128_device_scope(own, u32x4{~bits.x, ~bits.y, ~bits.z, ~bits.w});
                continue;
            }
            // The other parts, all polled at once, one 128-bit device-scope load each.  Every load of a
            // poll goes to an address of its own -- a second device-scope load of an address the
            // wavefront has just loaded waits for the first (measured: 0.5 us per repeat) -- so a slice
            // index past the last other part reads the same tile in a part nobody writes (zeros).
            u32x4 got[kGmpFlaggedSlices - 1];
            const uint32_t *base = reinterpret_cast<const uint32_t *>(partial) + (size_t)tt * 256 + lane * 4;
            for (int spins = 0;; ++spins) {
#pragma unroll
                for (int s2 = 0; s2 < kGmpFlaggedSlices - 1; ++s2) load_b128_device_scope(got[s2], base + (size_t)s2 * NT * 256);
                wait_vector_loads<0>();
                bool missing = false;
#pragma unroll
                for (int s2 = 0; s2 < kGmpFlaggedSlices - 1; ++s2) {
                    pin_loaded(got[s2]);
                    missing |= s2 < KS - 1 && (got[s2].x == 0 || got[s2].y == 0 || got[s2].z == 0 || got[s2].w == 0);
                }
                // the bound is never reached in a working launch; past it the words still missing read
                // as NaN in the result
                if (__builtin_amdgcn_ballot_w64(missing) == 0) {
                    KILN_GMP_TL(5, (long long)spins + 1);
                    break;
                }
                if (__builtin_expect(spins == kGmpSpinLimit, 0)) {  // the host can see this in the workspace's sticky word
                    report_wait_gave_up(error_word_before_exchange_region(partial), kGaveUpDecodeExchange, lane);
                    break;
                }
                __builtin_amdgcn_s_sleep(2);
            }
            KILN_GMP_TL(4, KILN_GMP_NOW());
            f32x4 total = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s2 = 0; s2 < kGmpFlaggedSlices - 1; ++s2) {
                if (s2 < KS - 1) {  // ascending K order, this slice's own part last
                    const u32x4 g = got[s2];
                    total += __builtin_bit_cast(f32x4, u32x4{~g.x, ~g.y, ~g.z, ~g.w});
                    store_b128_device_scope(const_cast<uint32_t *>(base) + (size_t)s2 * NT * 256,
                                            u32x4{0u, 0u, 0u, 0u});  // zero for the next launch
                }
            }
            sum = total + sum;
        } else if (KS > 1) {
            // the slices of the tile meet in the workspace: store this part with device-scope
            // accesses, wait until the stores are acknowledged, count the arrival; the last to arrive
            // adds all parts in ascending K order (so the result does not depend on arrival order)
            // and leaves the counter zero
            KILN_GMP_TL(3, KILN_GMP_NOW());
            // With adapters the last slice's part carries the low-rank term: whichever slice arrives last finishes the
            // tile here, and only the last slice's blocks hold the term's operands (adds_term).  (Added behind the
            // exchange instead, the term came from LDS that nobody had filled whenever another slice arrived last:
            // always, with the slices of a tile on compute units of one round.)
            if constexpr (LORA) {
                if (adds_term) {
                    lds_signal_wait(lora_ready_addr(), kGmpOperandsReady);  // the term's operands are in LDS
                    lora_add_from_lds(sum, lo, lora_t_lds, lora_b_lds, ti, M, lane);
                }
            }
            float *dst = partial + ((size_t)ks * NT + tt) * 256 + lane * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) __hip_atomic_store(dst + i, sum[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            wait_vector_loads<0>();
            int arrived = 0;
            if (lane == 0) arrived = __hip_atomic_fetch_add(counters + tt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            arrived = __builtin_amdgcn_readfirstlane(arrived);
            if (arrived != KS - 1) continue;
            KILN_GMP_TL(5, KILN_GMP_NOW());
            if (lane == 0) __hip_atomic_store(counters + tt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            sum = f32x4{0.f, 0.f, 0.f, 0.f};
            for (int s2 = 0; s2 < KS; ++s2) {
                const float *src = partial + ((size_t)s2 * NT + tt) * 256 + lane * 4;
                f32x4 v;
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                sum += v;
            }
            KILN_GMP_TL(4, KILN_GMP_NOW());
        }
        if (adapter && (KS == 1 || flagged)) {  // (through counters it is in the last slice's part already)
            lds_signal_wait(lora_ready_addr(), kGmpOperandsReady);  // the term's operands are in LDS
            lora_add_from_lds(sum, lo, lora_t_lds, lora_b_lds, ti, M, lane);
        }
        store_tile_rows(C, N, M, 4 * q4, tt, c, sum, swiglu != 0);
    }
#ifdef KILN_GMP_TIMELINE
    tl_[6] = KILN_GMP_NOW();
    tl_[7] = 1ll + ks;
    if (lane == 0 && g_gmp_tl) {
        long long *o = g_gmp_tl + (((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 16 + wave) * 8;
        for (int i = 0; i < 8; ++i) o[i] = tl_[i];
    }
#endif
}

// LDS behind the main wavefronts' slots for the low-rank term: the rows of B_cat of a block's tiles
// and T whole.
size_t gmp_adapter_lds_bytes(const DecodeArgs &a) {
    if (a.r_total <= 0) return 0;
    const size_t rp = (size_t)(a.r_total + 15) / 16 * 16;
    const size_t b_bytes = ((size_t)a.gm_tiles * kTileN * a.r_total * 2 + 15) & ~(size_t)15;
    // + the KiB that the LDS-direct copy of T may overwrite behind it, + the words the block meets on
    return kGmpSyncBytes + b_bytes + (size_t)a.lora_slices * a.lora_rows * rp * 2 + 1024;
}

int gmp_slot_bytes(int gpw, int tiles) {
    const int a = gmp_slots(gpw) * kGmpSlotBytes, r = tiles * 1024;
    return a > r ? a : r;
}

template <int T, int GPW, int AQ>
hipError_t launch_gmp_tga(const DecodeArgs &a, hipStream_t stream) {
    const hipError_t attr = allow_dynamic_lds<&w4a16_decode_gmp_kernel<T, GPW, AQ, kGmpLora>>(decode_max_lds_bytes());
    if (attr != hipSuccess) return attr;
    const int NT = a.N / kTileN;
    const int full_waves = a.GS - a.waves * (GPW - 1);
    const int slot = gmp_slot_bytes(GPW, T);
    const int col_blocks = (NT + T - 1) / T;
    LoraFold fold{};
    if (a.lora_producers > 0) {
        fold.a_cat = (const uint16_t *)a.lora_a;
        fold.t = (uint16_t *)const_cast<void *>(a.lora_t);
        fold.flags = a.lora_flags;
        fold.producers = a.lora_producers;
        fold.steps_per_slice = a.lora_steps_per_slice;
        fold.consumers = col_blocks;
        const int *e = a.lora_ends;
        const float *sc = a.lora_scales;
        fold.e0 = e[0], fold.e1 = e[1], fold.e2 = e[2], fold.e3 = e[3];
        fold.s0 = sc[0], fold.s1 = sc[1], fold.s2 = sc[2], fold.s3 = sc[3];
    }
    const dim3 grid = fold.producers > 0 ? dim3(fold.producers + col_blocks * a.KS, 1) : dim3(col_blocks, a.KS);
    const int adapter = a.r_total > 0 ? 1 : 0;  // one wavefront more: it fetches the low-rank term's operands
    const size_t lds_bytes = (size_t)a.waves * slot + gmp_adapter_lds_bytes(a);
    w4a16_decode_gmp_kernel<T, GPW, AQ, kGmpLora><<<grid, (a.waves + adapter) * 64, lds_bytes, stream>>>(
        (const uint16_t *)a.A, (const u32x4 *)a.B, (const uint16_t *)a.S, (uint16_t *)a.C, a.partial, a.counters, a.M,
        a.N, a.K, a.Gs, a.KS, a.GS, full_waves, slot, a.flagged ? exchange_column_shift(col_blocks) : 0, fold.producers,
        adapter, col_blocks, a.waves + adapter, a.swiglu ? 1 : 0, a.flagged ? 1 : 0, GmpLoraArgs{lora_tail(a), fold});
    return hipGetLastError();
}

template <int T, int GPW>
hipError_t launch_gmp_tg(const DecodeArgs &a, hipStream_t stream) {
    if (a.M <= 4) return launch_gmp_tga<T, GPW, 1>(a, stream);
    return a.M <= 8 ? launch_gmp_tga<T, GPW, 2>(a, stream) : launch_gmp_tga<T, GPW, 4>(a, stream);
}

template <int T>
hipError_t launch_gmp_t(const DecodeArgs &a, int gpw, hipStream_t stream) {
    switch (gpw) {
        case 1: return launch_gmp_tg<T, 1>(a, stream);
        case 2: return launch_gmp_tg<T, 2>(a, stream);
        case 3:
            if constexpr (T * 3 <= kGmpMaxChunks) return launch_gmp_tg<T, 3>(a, stream);
            break;
        case 4:
            if constexpr (T <= 2) return launch_gmp_tg<T, 4>(a, stream);
            break;
        case 5:
            if constexpr (T <= 2) return launch_gmp_tg<T, 5>(a, stream);
            break;
        case 6:
            if constexpr (T <= 2) return launch_gmp_tg<T, 6>(a, stream);
            break;
    }
    return hipErrorInvalidValue;
}

}  // namespace

#if KILN_GMP_LORA
// The instances with the low-rank term; the caller (launch_decode_gmp) has checked the plan.
hipError_t launch_decode_gmp_lora(const DecodeArgs &a, hipStream_t stream) {
    if (a.r_total <= 0) return hipErrorInvalidValue;  // these instances count on the adapter wavefront
    const int gpw = (a.GS + a.waves - 1) / a.waves;
    switch (a.gm_tiles) {
        case 1: return launch_gmp_t<1>(a, gpw, stream);
        case 2: return launch_gmp_t<2>(a, gpw, stream);
        case 3: return launch_gmp_t<3>(a, gpw, stream);
        case 4: return launch_gmp_t<4>(a, gpw, stream);
        case 5: return launch_gmp_t<5>(a, gpw, stream);
        default: return launch_gmp_t<6>(a, gpw, stream);
    }
}
#else
// The private-staging group-major instance: M <= 16 rows, 1...6 whole tiles per block in equal K
// slices of any length, wavefronts of ceil(GS / waves) groups (or one fewer) with at most 16
// chunks each; a.waves <= 16 and <= GS.
bool decode_gmp_ok(const DecodeArgs &a) {
    const int G = a.K / kGroupK;
    if (a.M < 1 || a.M > 16 || a.gm_tiles < 1 || a.gm_tiles > 6) return false;
    if (a.r_total > 0) {
        // the low-rank term's operands are read from LDS in 16-byte pieces by one wavefront more than the
        // main loop uses; T is whole and belongs to exactly this launch's rows (with the fused gate/up
        // store the rows of lora_b are in the packed column order, so nothing changes here)
        if (a.r_total > 64 || a.r_total % 8 != 0 || a.waves + 1 > kGmpMaxWaves) return false;
        if (a.lora_slices < 1 || a.lora_slices > 16 || a.lora_rows != a.M || !a.lora_t || !a.lora_b) return false;
    }
    if (a.KS < 1 || a.GS < 1 || a.KS * a.GS != G || a.waves < 1 || a.waves > kGmpMaxWaves || a.waves > a.GS) return false;
    const int gpw = (a.GS + a.waves - 1) / a.waves, T = a.gm_tiles;
    if (gpw > (T <= 2 ? 6 : 3) || T * gpw > kGmpMaxChunks) return false;
    const int full_waves = a.GS - a.waves * (gpw - 1);
    if (full_waves < 1 || full_waves > a.waves) return false;
    return (size_t)a.waves * gmp_slot_bytes(gpw, T) + gmp_adapter_lds_bytes(a) <= (size_t)decode_max_lds_bytes();
}

// The projection folded into the launch: one producer block per K slice of it, each with at least
// as many wavefronts as T has rank tiles and a KiB of LDS per wavefront for their meeting.
bool decode_gmp_fold_ok(const DecodeArgs &a) {
    if (a.r_total < 1 || a.r_total > 64 || !a.lora_a || !a.lora_t || !a.lora_flags) return false;
    const int jt = (a.r_total + 15) / 16;
    if (a.lora_producers < 1 || a.lora_producers > kLoraFoldMaxProducers || a.lora_producers != a.lora_slices) return false;
    if (a.lora_steps_per_slice < 1 || (long)a.lora_producers * a.lora_steps_per_slice * 32 < a.K) return false;
    if (a.waves < jt || (a.lora_steps_per_slice + a.waves / jt - 1) / (a.waves / jt) > kLoraFoldStepsPerWave ||
        a.lora_rows != a.M || a.lora_adapters < 1 || a.lora_adapters > kLoraFoldMaxAdapters) return false;
    if (a.KS > 4) return false;  // the kernel finds a block's slice in a one-row grid by three comparisons
    const int gpw = (a.GS + a.waves - 1) / a.waves;
    return gmp_slot_bytes(gpw, a.gm_tiles) >= 1024;
}

hipError_t launch_decode_gmp(const DecodeArgs &a, hipStream_t stream) {
    if (!decode_gmp_ok(a)) return hipErrorInvalidValue;
    if (a.KS > 1 && (!a.partial || !a.counters)) return hipErrorInvalidValue;
    if (a.flagged && a.KS > kGmpFlaggedSlices) return hipErrorInvalidValue;
    if (a.lora_producers > 0 && !decode_gmp_fold_ok(a)) return hipErrorInvalidValue;
    if (a.r_total > 0) return launch_decode_gmp_lora(a, stream);
    const int gpw = (a.GS + a.waves - 1) / a.waves;
    switch (a.gm_tiles) {
        case 1: return launch_gmp_t<1>(a, gpw, stream);
        case 2: return launch_gmp_t<2>(a, gpw, stream);
        case 3: return launch_gmp_t<3>(a, gpw, stream);
        case 4: return launch_gmp_t<4>(a, gpw, stream);
        case 5: return launch_gmp_t<5>(a, gpw, stream);
        default: return launch_gmp_t<6>(a, gpw, stream);
    }
}

#endif  // KILN_GMP_LORA

}  // namespace kiln

#ifdef KILN_GMP_TIMELINE
#if KILN_GMP_LORA
extern "C" int kiln_gmp_timeline_lora(long long *buf) {
#else
extern "C" int kiln_gmp_timeline(long long *buf) {
#endif
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(kiln::g_gmp_tl), &buf, sizeof(buf));
}
#endif
