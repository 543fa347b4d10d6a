// Mid-M W4A16 GEMM kernel for gfx950: runs of up to 64 rows per pass over the weights.
//
// Covers the row counts between the decode kernels (one or two 16-row slabs, 16x16x32
// products) and the prefill kernel (whole-chip tiling, matrix-core bound): the arm of the
// reference dispatcher that pads M to 16 * thread_m_blocks up to 64 rows
// (crates/kiln-marlin-gemm/csrc/marlin_kernel.cu:784-816).  At 17...128 rows (and up to 320 on
// small weights) the problem is still bound by the int4 weight stream, but the products are no
// longer free: a run of 64 rows takes v_mfma_f32_32x32x16_bf16 (the 16-row shape runs at half the
// rate per flop) and one pass over the weights; a run of up to 32 rows computes one of the two row
// blocks only.
//
// Work split (group-major, as in the decode kernels): a block owns TP pairs of neighbouring
// 16-column tiles (32 columns per pair = one 32x32 product tile) and one K slice of GS groups;
// wavefront w owns a contiguous run of those groups and multiplies them with every pair of the
// block, 64 rows each.  So each element of the activations is read once per block, by the one
// wavefront that needs it, and nobody waits at a barrier before the first product:
//   * A: the wavefront's 64 rows x 128 values of one group go from L2 into its private 16 KiB
//     of LDS with 16 LDS-direct loads (4 rows of 256 bytes each, fully coalesced), swizzled on
//     16-byte units so that the fragment reads are free of bank conflicts; the fragments are
//     then held in registers for the whole group, which frees the LDS slot for the next group.
//   * B: 2 x 128-bit per lane, pair and group, straight into the product's operand layout,
//     requested one or two groups ahead (as the registers allow) into rotating register sets.
//   * Scales in f32 by a running rescale of the accumulators (as in the prefill kernel); the
//     B operand carries 136 + d, and the surplus 136 * sum(a) * scale is removed after the
//     wavefront's last group by a short extra contraction (as in the prefill kernel) over the
//     groups' row sums, which the vector unit forms from the fragments (v_dot2c_f32_bf16) while
//     the matrix unit multiplies.
// At the end the wavefronts' f32 tiles are summed through LDS in wavefront (= ascending K)
// order; K slices of a tile meet in the workspace, last arriver adds in slice order.
#include "async_loads.h"
#include "launch.h"
#include "lora_project.h"
#include "lora_tail.h"

namespace kiln {

namespace {

// This file is compiled twice: as it is for calls without adapters, and with -DKILN_MID_LORA=1 for calls
// with them (launch_mid_lora only), so that what the low-rank term adds costs plain calls nothing.
#ifndef KILN_MID_LORA
#define KILN_MID_LORA 0
#endif
constexpr bool kMidLora = KILN_MID_LORA != 0;

// Probe builds only (-DKILN_MID_TIMELINE): wall-clock stamps (100 MHz) per wavefront.
#ifdef KILN_MID_TIMELINE
#if KILN_MID_LORA
#define g_mid_tl g_mid_tl_lora
#endif
__device__ long long *g_mid_tl;
#define KILN_MID_TL(i) tl_[i] = (long long)__builtin_amdgcn_s_memrealtime()
#else
#define KILN_MID_TL(i) \
    do {               \
    } while (0)
#endif

constexpr int kMidWaves = 8;                    // wavefronts per block, at most (and what the counter-free exchange takes)
constexpr int kMidWavesMost = 10;               // ... of a launch of up to 32 rows, or of one pair per block, without adapters
constexpr int kMidRows = 64;                    // rows per run
constexpr int kMidSlotBytes = kMidRows * 256;   // one group of A: 64 rows x 128 bf16
constexpr int kMidALoads = 16;                  // LDS-direct loads per group of A
constexpr int kMidMaxGroups = 4;                // groups per wavefront, at most
constexpr int kMidFlaggedSlices = kDecodeFlaggedMaxSlices;  // most K slices the counter-free exchange takes
constexpr int kMidSpinLimit = 1 << 20;          // polls of the other slices' parts before the adding wavefront gives up

// Issue order of a wavefront's loads -- A(g): NA LDS-direct loads (16, or 8 where a run has at most 32
// rows), B(g): NL register loads, the
// weights D groups ahead in D + 1 register sets --
//   before the first step: A(0), B(0) ... B(D-1) (the weights first measured 0.3...0.5 us slower:
//     loads return in issue order, so A(0) then waits for the weights' trip to memory before the
//     fragments can be read and A(1) asked for), A(1) ... A(DA-1);
//   step g: [wait for A(g)] fragments to registers, A(g+DA), B(g+D), [wait for B(g)], products.
// DA = groups of A in flight: 1 where a group fills the wavefront's slot (64 rows), 2 where it fills half
// (one row block per pass: the halves take turns).
// wait_a[g] / wait_b[g] = loads issued after A(g) / B(g) up to that wait: what may still be
// outstanding when the wait returns.
struct MidSchedule {
    int wait_a[kMidMaxGroups];
    int wait_b[kMidMaxGroups];
};
constexpr MidSchedule mid_schedule(int ng, int nl, int d, int na, int da) {
    int kind[4 * kMidMaxGroups] = {}, grp[4 * kMidMaxGroups] = {}, size[4 * kMidMaxGroups] = {};
    int n = 0;
    auto push = [&](int k, int g, int sz) {
        kind[n] = k;
        grp[n] = g;
        size[n] = sz;
        ++n;
    };
    auto issued_after = [&](int k, int g) {
        int after = 0;
        bool seen = false;
        for (int i = 0; i < n; ++i) {
            if (seen) after += size[i];
            if (kind[i] == k && grp[i] == g) seen = true;
        }
        return after;
    };
    push(0, 0, na);
    for (int g = 0; g < d && g < ng; ++g) push(1, g, nl);
    for (int g = 1; g < da && g < ng; ++g) push(0, g, na);
    MidSchedule s{};
    for (int g = 0; g < ng; ++g) {
        s.wait_a[g] = issued_after(0, g);
        if (g + da < ng) push(0, g + da, na);
        if (g + d < ng) push(1, g + d, nl);
        s.wait_b[g] = issued_after(1, g);
    }
    return s;
}

template <int NG, int NL, int D, int NA, int DA>
struct MidScheduleOf {
    static constexpr MidSchedule value = mid_schedule(NG, NL, D, NA, DA);
};

// The low-rank term of a call with adapters (LORA instances): T = the scaled projection of x onto the
// stacked adapters in `slices` K slices, each rounded on its own, bf16 [slices][rows][rp] (written by
// a launch in front of this one), B_cat bf16 [N][r_total], r_total % 8 == 0.
struct MidLora {
    const uint16_t *t;
    const uint16_t *b;
    int r_total, rp, slices;
    // producers > 0: the projection runs in this launch's first `producers` blocks (row tiles of 16 rows x
    // the K slices, lora_project_block), which raise a word per (slice, row tile) -- in 16 copies, 4 KiB
    // apart, block b looks at copy b % 16: hundreds of readers of one address are served one by one -- in
    // workspace that is zero between launches; the blocks of the first K slice look at the words of their
    // rows behind their main loop, count themselves, and the last one zeroes words and counts.
    const uint16_t *a_cat;
    unsigned *words;
    int producers, row_tiles, steps_per_slice, col_blocks, consumers;
    LoraScales ls;
};
constexpr int kMidFoldTileWord = 32;  // a copy's words start here (the first words are the small-M kernel's)
constexpr int kMidFoldSpinLimit = 1 << 20;

// The work of one block.  RBN: row blocks of 32 its pass computes -- 2, or 1 where the block's run of rows
// has at most 32 (a launch of up to 32 rows, or the last run of a longer one: half the loads of A, fragment
// reads and products; the other row block's accumulators stay zero, and its items take no part in the
// wavefronts' meeting, in the exchange between K slices or in the store).
template <int TP, int GPW, bool LORA, int RBN>
__device__ __forceinline__ void mid_block(
    const uint16_t *__restrict__ A_all, const u32x4 *__restrict__ B, const uint16_t *__restrict__ S,
    uint16_t *__restrict__ C_all, float *partial_all, int *counters_all, int rows, int N, int K, int Gs, int KS,
    int GS, int full_waves, int swiglu, int flagged, int col_shift, const MidLora &lo, int nw) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    int &s_last = *reinterpret_cast<int *>(lds);  // used between two barriers behind the meeting, when nothing else is in LDS
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, h = lane >> 5;
    const int G = K / kGroupK;
#ifdef KILN_MID_TIMELINE
    long long tl_[8] = {};
    struct TimelineWriter {  // on every way out of the kernel
        long long *tl;
        int lane, wave;
        __device__ ~TimelineWriter() {
            tl[7] = (long long)__builtin_amdgcn_s_memrealtime();
            if (lane == 0 && g_mid_tl) {
                long long *o = g_mid_tl + ((((size_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * 8 + wave) * 8;
                for (int i = 0; i < 8; ++i) o[i] = tl[i];
            }
        }
    } timeline_writer{tl_, lane, wave};
#endif
    KILN_MID_TL(0);
    // Grid (column blocks, K slices, runs of 64 rows) -- or, with the projection in this launch, one row
    // of blocks: the producers, then the same order.
    int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z, ncb = gridDim.x;
    if constexpr (LORA) {
        if (lo.producers > 0) {
            int id = blockIdx.x;
            if (id < lo.producers) {
                const int tile = id % lo.row_tiles, slice = id / lo.row_tiles;
                lora_project_block<16>(lds, A_all, lo.a_cat, const_cast<uint16_t *>(lo.t), rows, K, lo.r_total, lo.rp,
                                       lo.steps_per_slice, lo.ls, nullptr, nullptr, nullptr, tile, slice, lo.slices,
                                       lo.words + kMidFoldTileWord + slice * lo.row_tiles, kLoraFoldReplicas,
                                       kLoraFoldReplicaWords);
                return;
            }
            id -= lo.producers;
            ncb = lo.col_blocks;
            bx = id % ncb;
            id /= ncb;
            by = id % KS;
            bz = id / KS;
        }
    }
    // bz: which run of 64 rows (each with its own counters and partial tiles)
    const int zr = bz * kMidRows;
    const int M = min(rows - zr, kMidRows);
    const uint16_t *__restrict__ A = A_all + (size_t)zr * K;
    const int ldc = swiglu ? N >> 1 : N;  // the fused gate/up result is half as wide
    uint16_t *__restrict__ C = C_all + (size_t)zr * ldc;
    const int ks = by;
    // Column block of this block.  Blocks go to the eight dies round-robin by linear index; the
    // counter-free exchange shifts the column block by col_shift per slice so that the slices of a
    // tile sit on different dies (a device-scope store and the device-scope load that polls it
    // are slow when they meet in one die's L2).
    const int cb = (bx + ks * col_shift) % ncb;
    const int tf = cb * (2 * TP);  // first 16-column tile of the block
    // the first `fw` wavefronts own GPW groups each, the others GPW - 1; the last slice may have fewer groups
    // than the others (K in groups not a multiple of the slices) and then fewer wavefronts of GPW: its count
    // rides in the argument's second byte
    const int fw = (ks == KS - 1 ? full_waves >> 8 : full_waves) & 255;
    const bool full = wave < fw;
    const int g_first = full ? wave * GPW : fw * GPW + (wave - fw) * (GPW - 1);
    const int g0 = ks * GS + g_first;  // all slices have GS groups
    const int gs_mask = (Gs == 1) ? 0 : -1;

    // --- A: 16 loads of 4 rows x 256 bytes.  Lane i of load p fetches 16-byte unit
    // (i % 16) ^ (row % 16) of row 4 p + i / 16, so unit u of a row sits at position u ^ (row % 16):
    // the 16 lanes that read one unit index of 16 different rows then hit 16 different positions.
    // Rows from M on read row M - 1 (a valid address); their products are never stored.
    unsigned char *slot = lds + wave * kMidSlotBytes;
    const unsigned slot_addr = (unsigned)(size_t)(lds_ptr_t)slot;
    const uint32_t row_pitch = (uint32_t)K * 2;
    constexpr int kASlots = RBN == 1 ? 2 : 1;  // groups of A a slot holds, and as many are in flight
    auto request_a = [&](int gi) {
        const char *base = reinterpret_cast<const char *>(A) + (size_t)(g0 + gi) * 256;
        const uint32_t quad_row = (uint32_t)(lane >> 4) + opaque_zero();  // keeps the offsets below local to this group
#pragma unroll
        for (int p = 0; p < kMidALoads * RBN / 2; ++p) {
            const uint32_t row = 4 * p + quad_row;
            const uint32_t off = min(row, (uint32_t)(M - 1)) * row_pitch + (((uint32_t)(lane & 15) ^ (row & 15)) << 4);
            load_to_lds_b128(base, off, slot_addr + (uint32_t)(gi % kASlots) * (kMidSlotBytes / 2) + p * 1024);
        }
    };

    // --- B: pair p = tiles tf + 2 p, tf + 2 p + 1.  Lane (l32, h) holds column l32 of the pair and
    // rows 16 s + 8 h ... + 7 of step s: word s / 2 of the 128-bit unit c + 16 (2 (s % 2) + h) of
    // chunk l32 / 16 (c = l32 % 16).  Load v = s % 2 therefore serves steps v, v + 2, v + 4, v + 6.
    constexpr int D = TP == 1 ? 2 : 1;  // groups of look-ahead (more pairs: the registers allow one)
    constexpr int kSets = D + 1;
    u32x4 bw[kSets][TP][2];
    uint32_t sc_raw[kSets][TP];
    const uint32_t b_lane = (uint32_t)(l32 >> 4) * (uint32_t)G * 1024u + (uint32_t)((l32 & 15) + 16 * h) * 16u;
    const uint32_t s_lane = (uint32_t)(l32 >> 4) * (uint32_t)Gs * (kTileN * 2) + (uint32_t)(l32 & 15) * 2u;
    auto request_b = [&](auto gc) {
        constexpr int gi = decltype(gc)::value, set = gi % kSets;
        const int g = g0 + gi;
        unrolled<0, TP>([&](auto pc) {
            constexpr int p = decltype(pc)::value;
            const int tp = min(tf + 2 * p, N / kTileN - 2);  // a pair past the last tile reads the last pair; never stored
            const char *bb = reinterpret_cast<const char *>(B) + ((size_t)tp * G + g) * 1024;
            load_b128_streaming(bw[set][p][0], bb, b_lane);
            load_b128_streaming(bw[set][p][1], bb, b_lane + 512u);
            const char *sb = reinterpret_cast<const char *>(S) + ((size_t)tp * Gs + (g & gs_mask)) * (kTileN * 2);
            load_u16(sc_raw[set][p], sb, s_lane);
        });
    };

    // a zero scale would break the running rescale; it is replaced by a value too small to matter
    // (the exact result for such a group is 0; the stand-in contributes < 1e-12 * |a|)
    auto scale_value = [&](uint32_t raw) {
        const float sv = f16_bits_to_f32((uint16_t)raw);
        return sv == 0.f ? 0x1p-40f : sv;
    };

    const DequantConsts dq = dequant_consts();
    f32x16 acc[TP][2];
#pragma unroll
    for (int p = 0; p < TP; ++p)
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[p][rb][r] = 0.f;

    // The wavefront's groups: straight-line code from the first request to the last use, one
    // instance per group count (a register that an asm load fills must be requested, waited for and
    // used inside one basic block).
    auto run = [&](auto nc) {
        constexpr int NG = decltype(nc)::value;
        constexpr int NL = 3 * TP;
        using Sch = MidScheduleOf<NG, NL, D, kMidALoads * RBN / 2, kASlots>;
        request_a(0);
        unrolled<0, (D < NG ? D : NG)>(request_b);
        if constexpr (kASlots == 2 && NG > 1) request_a(1);
        float s_cur[TP];
        float s_of[NG][TP];   // the scale of every group (this lane's column of each pair)
        float c_of[NG][RBN];  // -136 * (sum of the group's activations) of row 32 rb + l32
        uint32_t ones;
        asm("s_mov_b32 %0, 0x3f803f80" : "=s"(ones));  // bf16 (1, 1)
        unrolled<0, NG>([&](auto gc) {
            constexpr int gi = decltype(gc)::value, set = gi % kSets;
            // this group's rows of A are in LDS; their fragments go to registers: lane (l32, h) holds
            // row 32 rb + l32, values 16 s + 8 h ... + 7 of the group
            if constexpr (gi == 1) KILN_MID_TL(3);  // products of group 0 issued
            wait_vector_loads<Sch::value.wait_a[gi]>();
            if constexpr (gi == 0) KILN_MID_TL(1);  // A(0) has arrived
            if constexpr (gi == 1) KILN_MID_TL(4);  // A(1) has arrived
            u32x4 af[RBN][8];
#pragma unroll
            for (int rb = 0; rb < RBN; ++rb)
#pragma unroll
                for (int s = 0; s < 8; ++s)
                    af[rb][s] = *reinterpret_cast<const u32x4 *>(slot + (gi % kASlots) * (kMidSlotBytes / 2) +
                                                                 (rb * 32 + l32) * 256 + (((2 * s + h) ^ (l32 & 15)) << 4));
            wait_lds_reads();  // the slot (or this half of it) is free again
            if constexpr (gi + kASlots < NG) request_a(gi + kASlots);
            if constexpr (gi + D < NG) request_b(std::integral_constant<int, gi + D>{});
            // Row sums of the group for the offset term, on the vector unit while the matrix unit
            // multiplies: v_dot2c_f32_bf16 adds both halves of a register to an f32 sum (products with
            // 1.0 are exact), two interleaved sums per row block; the lane's half of K here, the other
            // half from lane + 32.
#pragma unroll
            for (int rb = 0; rb < RBN; ++rb) {
                float e0 = 0.f, e1 = 0.f;
#pragma unroll
                for (int s = 0; s < 7; ++s) {
                    asm("v_dot2c_f32_bf16 %0, %2, %1" : "+v"(e0) : "v"(af[rb][s].x), "s"(ones));
                    asm("v_dot2c_f32_bf16 %0, %2, %1" : "+v"(e1) : "v"(af[rb][s].y), "s"(ones));
                    asm("v_dot2c_f32_bf16 %0, %2, %1" : "+v"(e0) : "v"(af[rb][s].z), "s"(ones));
                    asm("v_dot2c_f32_bf16 %0, %2, %1" : "+v"(e1) : "v"(af[rb][s].w), "s"(ones));
                }
                asm("v_dot2c_f32_bf16 %0, %2, %1" : "+v"(e0) : "v"(af[rb][7].x), "s"(ones));
                asm("v_dot2c_f32_bf16 %0, %2, %1" : "+v"(e1) : "v"(af[rb][7].y), "s"(ones));
                // A dot instruction may feed its own kind as the addend back to back, but another
                // vector instruction must wait three states before it reads the result; the compiler
                // does not know what the asm holds, so the last link of each chain carries the wait.
                asm("v_dot2c_f32_bf16 %0, %2, %1\n\ts_nop 3" : "+v"(e0) : "v"(af[rb][7].z), "s"(ones));
                asm("v_dot2c_f32_bf16 %0, %2, %1\n\ts_nop 3" : "+v"(e1) : "v"(af[rb][7].w), "s"(ones));
                const float half_sum = e0 + e1;
                c_of[gi][rb] = -kCodeBias * (half_sum + __shfl_xor(half_sum, 32, 64));
            }
            wait_vector_loads<Sch::value.wait_b[gi]>();
            if constexpr (gi == 0) KILN_MID_TL(2);  // B(0) has arrived
#pragma unroll
            for (int p = 0; p < TP; ++p) {
                pin_loaded(bw[set][p][0]);
                pin_loaded(bw[set][p][1]);
                pin_loaded(sc_raw[set][p]);
                const float sn = scale_value(sc_raw[set][p]);
                s_of[gi][p] = sn;
                if constexpr (gi > 0) {  // into this group's units: accumulator = sum so far / scale of this group
                    const float f = s_cur[p] * __builtin_amdgcn_rcpf(sn);
#pragma unroll
                    for (int rb = 0; rb < RBN; ++rb)
#pragma unroll
                        for (int r = 0; r < 16; ++r) acc[p][rb][r] *= f;
                }
                s_cur[p] = sn;
            }
#pragma unroll
            for (int s = 0; s < 8; ++s)
#pragma unroll
                for (int p = 0; p < TP; ++p) {
                    const u32x4 &w4 = bw[set][p][s & 1];
                    const uint32_t word = (s >> 1) == 0 ? w4.x : (s >> 1) == 1 ? w4.y : (s >> 1) == 2 ? w4.z : w4.w;
                    const bf16x8 bexp = codes_to_bf16x8(word, dq);
#pragma unroll
                    for (int rb = 0; rb < RBN; ++rb)
                        acc[p][rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, af[rb][s]), bexp,
                                                                             acc[p][rb], 0, 0, 0);
                }
        });
        // out of the last group's units
#pragma unroll
        for (int p = 0; p < TP; ++p)
#pragma unroll
            for (int rb = 0; rb < RBN; ++rb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[p][rb][r] *= s_cur[p];
        // The B operand carried 136 + d: remove 136 * sum(a) * scale per group by a short extra
        // contraction.  Step e covers group 2 e in lanes 0-31 and group 2 e + 1 in lanes 32-63 (the
        // two halves of a product's K); c is split exactly into three bf16 terms, the scale into two,
        // and the six exact products per group add up to c * scale in the f32 accumulator.
        unrolled<0, (NG + 1) / 2>([&](auto ec) {
            constexpr int e = decltype(ec)::value;
            constexpr bool has_odd = 2 * e + 1 < NG;
            constexpr int g_odd = has_odd ? 2 * e + 1 : 2 * e;
            bf16x8 ax[RBN];
#pragma unroll
            for (int rb = 0; rb < RBN; ++rb) {
                const float c = h ? (has_odd ? c_of[g_odd][rb] : 0.f) : c_of[2 * e][rb];
                const uint32_t hi = __builtin_bit_cast(uint32_t, c) & 0xFFFF0000u;
                const float r1 = c - __builtin_bit_cast(float, hi);                     // exact
                const uint32_t mid = __builtin_bit_cast(uint32_t, r1) & 0xFFFF0000u;
                const float r2 = r1 - __builtin_bit_cast(float, mid);                   // exact, <= 8 significant bits
                const uint32_t lo = __builtin_bit_cast(uint32_t, r2) & 0xFFFF0000u;
                const u32x4 r = {(hi >> 16) | hi, (mid >> 16) | mid, (lo >> 16) | lo, 0u};
                ax[rb] = __builtin_bit_cast(bf16x8, r);
            }
#pragma unroll
            for (int p = 0; p < TP; ++p) {
                const float sv = h ? (has_odd ? s_of[g_odd][p] : 0.f) : s_of[2 * e][p];
                const uint32_t hi = __builtin_bit_cast(uint32_t, sv) & 0xFFFF0000u;
                const float lo_f = sv - __builtin_bit_cast(float, hi);  // exact: f16 has 11 significant bits
                const uint32_t pair = (hi >> 16) | (__builtin_bit_cast(uint32_t, lo_f) & 0xFFFF0000u);
                const u32x4 r = {pair, pair, pair, 0u};
                const bf16x8 bx = __builtin_bit_cast(bf16x8, r);
#pragma unroll
                for (int rb = 0; rb < RBN; ++rb)
                    acc[p][rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ax[rb], bx, acc[p][rb], 0, 0, 0);
            }
        });
    };
    if (full) run(std::integral_constant<int, GPW>{});
    else if constexpr (GPW > 1) run(std::integral_constant<int, GPW - 1>{});
    if constexpr (LORA) {
        // y += T * B_cat^T (crates/kiln-model/src/lora_loader.rs:213-232, the second product) on the f32
        // accumulators, before the single rounding: (K slice of T, 16 rank columns) pairs are dealt to the
        // wavefronts of the first K slice's blocks, each adds its share to its own partial tiles, and
        // the meeting below sums them with everything else.  Rows from M on read row M - 1 (never stored).
        if (ks == 0 && lo.producers > 0) {
            // T of this run's rows, every slice: one wavefront looks (lane 4 z + i: slice z, i-th row tile
            // of the run), counts the block, and the barrier tells the others
            if (wave == 0) {
                const int t0 = zr >> 4, nt = min((M + 15) >> 4, lo.row_tiles - t0), consumer = bz * ncb + bx;
                const unsigned *mine = lo.words + (consumer % kLoraFoldReplicas) * kLoraFoldReplicaWords + kMidFoldTileWord;
                int spins = 0;
                for (; spins < kMidFoldSpinLimit; ++spins) {
                    unsigned f = 1u;
                    if ((lane >> 2) < lo.slices && (lane & 3) < nt)
                        f = __hip_atomic_load(mine + (lane >> 2) * lo.row_tiles + t0 + (lane & 3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (__builtin_amdgcn_ballot_w64(f == 0u) == 0) break;
                    __builtin_amdgcn_s_sleep(4);
                }
                if (__builtin_expect(spins == kMidFoldSpinLimit, 0))
                    report_wait_gave_up(error_word_before_fold_words(lo.words), kGaveUpMidFold, lane);
                // count: the replica's count, then the top count; the last block zeroes words and counts
                const int replica = consumer % kLoraFoldReplicas;
                const unsigned quota = (unsigned)(lo.consumers - replica + kLoraFoldReplicas - 1) / kLoraFoldReplicas;
                const unsigned replicas = (unsigned)min(lo.consumers, kLoraFoldReplicas);
                unsigned before = 0;
                if (lane == 0)
                    before = __hip_atomic_fetch_add(lo.words + replica * kLoraFoldReplicaWords + kLoraFoldCountWord, 1u,
                                                    __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                bool last = (unsigned)__builtin_amdgcn_readfirstlane((int)before) == quota - 1u;
                if (last) {
                    if (lane == 0)
                        before = __hip_atomic_fetch_add(lo.words + kLoraFoldTopWord, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    last = (unsigned)__builtin_amdgcn_readfirstlane((int)before) == replicas - 1u;
                }
                if (last) {
                    const int n_words = lo.slices * lo.row_tiles;
                    for (int r = 0; r < kLoraFoldReplicas; ++r) {
                        for (int i = lane; i < n_words; i += 64)
                            __hip_atomic_store(lo.words + r * kLoraFoldReplicaWords + kMidFoldTileWord + i, 0u, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT);
                        if (lane <= kLoraFoldTopWord)
                            __hip_atomic_store(lo.words + r * kLoraFoldReplicaWords + lane, 0u, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
            }
            __syncthreads();
        }
        if (ks == 0) {
            const int JS = lo.rp >> 4;
            for (int c = wave; c < lo.slices * JS; c += nw) {
                const int z = c / JS, j8 = (c - z * JS) * 16 + 8 * h;  // this lane's 8 rank columns
                const bool live_rank = j8 + 8 <= lo.r_total;           // r_total % 8 == 0: all or none
                u32x4 ta[RBN], tb[TP];
#pragma unroll
                for (int rb = 0; rb < RBN; ++rb) {
                    const int row = zr + min(32 * rb + l32, M - 1);
                    ta[rb] = *reinterpret_cast<const u32x4 *>(lo.t + ((size_t)z * rows + row) * lo.rp + j8);
                }
#pragma unroll
                for (int p = 0; p < TP; ++p) {
                    const int col = min(tf + 2 * p, N / kTileN - 2) * kTileN + l32;
                    tb[p] = u32x4{0u, 0u, 0u, 0u};
                    if (live_rank) tb[p] = *reinterpret_cast<const u32x4 *>(lo.b + (size_t)col * lo.r_total + j8);
                }
#pragma unroll
                for (int p = 0; p < TP; ++p)
#pragma unroll
                    for (int rb = 0; rb < RBN; ++rb)
                        acc[p][rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ta[rb]),
                                                                             __builtin_bit_cast(bf16x8, tb[p]), acc[p][rb], 0, 0, 0);
            }
        }
    }
    KILN_MID_TL(5);  // main loop done

    // --- the wavefronts' partial tiles meet in LDS, as many pairs at a time as a wavefront's 16 KiB slot
    // holds (two with both row blocks, all of them with one): every wavefront writes its own slot (item =
    // (pair, row block, register quad q): rows 32 rb + 8 q + 4 h ... + 3 of column l32; a pass over one row
    // block has the items of that block only, packed), then every item is summed over the wavefronts, in
    // wavefront (= ascending K) order, by one wavefront.
    constexpr int kItems = TP * 2 * 4;         // ids of items: pair * 8 + row block * 4 + quad (as the partial tiles are laid out)
    constexpr int kPerPair = RBN * 4;          // items of a pair in this pass, = their stride in a slot
    constexpr int kPhasePairs = 16 / kPerPair; // pairs a slot holds
    constexpr int kPhases = (TP + kPhasePairs - 1) / kPhasePairs;
    const int NT = N / kTileN;
    auto store_item = [&](f32x4 v, int item) {
        const int q = item & 3, rb = (item >> 2) & 1, p = item >> 3;
        const int row0 = 32 * rb + 8 * q + 4 * h;
        const bool live = tf + 2 * p < NT;  // false: a pair past the last tile (grid padding)
        if (!swiglu) {
            uint16_t *dst = C + (size_t)row0 * N + (tf + 2 * p) * kTileN + l32;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (live && row0 + i < M) dst[(size_t)i * N] = f32_to_bf16_bits(v[i]);
            return;
        }
        // gate/up interleaved by 8 inside every tile: the lane of gate column c takes up from lane
        // c + 8 of its 16-lane row and stores silu(gate) * up (forward.rs:2789-2819) half as wide
        f32x4 up;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float vi = v[i];  // a scalar copy: bit-casting the vector element in place reads element 0
            up[i] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, vi), 0x128, 0xF, 0xF, true));
            asm volatile("" : "+v"(up[i]));  // exchanged while all lanes are active, not folded into the gate lanes' arithmetic
        }
        if (live && (l32 & 8) == 0) {
            uint16_t *dst = C + (size_t)row0 * ldc + (tf + 2 * p) * (kTileN / 2) + (l32 >> 4) * 8 + (l32 & 7);
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (row0 + i < M) {
                    const float gate = v[i];
                    dst[(size_t)i * ldc] = f32_to_bf16_bits(gate * __builtin_amdgcn_rcpf(1.f + __expf(-gate)) * up[i]);
                }
        }
    };
    float *partial = partial_all + ((size_t)(bz * KS) * ncb + cb) * (kItems * 256);
    const size_t slice_stride = (size_t)ncb * (kItems * 256);  // floats between two K slices of a block
    f32x4 *mine = reinterpret_cast<f32x4 *>(slot);
    // item `local` of the phase, summed over the wavefronts in wavefront (= ascending K) order
    auto sum_over_wavefronts = [&](int local) {
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int wv = 0; wv < nw; ++wv)
            sum += reinterpret_cast<const f32x4 *>(lds + wv * kMidSlotBytes)[local * 64 + lane];
        return sum;
    };
    [[maybe_unused]] f32x4 own[TP];  // counter-free exchange, last slice: this wavefront's sums, one per pair
    unrolled<0, kPhases>([&](auto phc) {
        constexpr int p0 = kPhasePairs * decltype(phc)::value, p1 = p0 + kPhasePairs < TP ? p0 + kPhasePairs : TP;
        if constexpr (p0 > 0) __syncthreads();  // the previous phase's sums have been read
#pragma unroll
        for (int p = p0; p < p1; ++p)
#pragma unroll
            for (int rb = 0; rb < RBN; ++rb)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    mine[(((p - p0) * RBN + rb) * 4 + q) * 64 + lane] =
                        f32x4{acc[p][rb][4 * q], acc[p][rb][4 * q + 1], acc[p][rb][4 * q + 2], acc[p][rb][4 * q + 3]};
        __syncthreads();
        if constexpr (p0 == 0) KILN_MID_TL(6);  // every wavefront's tiles are in LDS
        if (flagged) {  // eight wavefronts: item (p0 + j) * 8 + wave for each pair j of the phase
            if (wave >= kPerPair) return;  // (one row block per pass: four items a pair)
#pragma unroll
            for (int j = 0; j < p1 - p0; ++j) {
                const int item = (p0 + j) * 8 + wave;
                const f32x4 sum = sum_over_wavefronts(j * kPerPair + wave);
                if (ks == KS - 1) {
                    own[p0 + j] = sum;
                } else {  // the complement of a sum's bits is never zero, so the part is its own arrival flag
                    const u32x4 bits = __builtin_bit_cast(u32x4, sum);
                    store_b128_device_scope(partial + ks * slice_stride + item * 256 + lane * 4,
                                            u32x4{~bits.x, ~bits.y, ~bits.z, ~bits.w});
                }
            }
            return;
        }
        for (int c = wave; c < (p1 - p0) * kPerPair; c += nw) {
            const int item = (p0 + c / kPerPair) * 8 + c % kPerPair;
            const f32x4 sum = sum_over_wavefronts(c);
            if (KS == 1) {
                store_item(sum, item);
            } else {
                store_b128_device_scope(partial + ks * slice_stride + item * 256 + lane * 4,
                                        __builtin_bit_cast(u32x4, sum));
            }
        }
    });
    if (KS == 1) return;

    if (flagged) {
        // Counter-free exchange.  The parts live in a region that is all zero between launches; a
        // written word is the complement of a sum's bits and never zero (a sum with all bits set
        // would be a NaN whose payload no arithmetic here produces).  The last slice adds the
        // parts; its blocks are dispatched after all others (grid y is the slice), so every block
        // it waits for is running or done.  Each part is loaded once per poll; the loads are
        // straight-line code up to their wait, so the parts of absent slices (zeros nobody
        // writes, or another run's parts) are loaded too and ignored.
        if (ks != KS - 1 || wave >= kPerPair) return;
        u32x4 got[TP][kMidFlaggedSlices - 1] = {};
        uint32_t *base = reinterpret_cast<uint32_t *>(partial) + wave * 256 + lane * 4;
        for (int spins = 0;; ++spins) {
#pragma unroll
            for (int j = 0; j < TP; ++j)
#pragma unroll
                for (int s2 = 0; s2 < kMidFlaggedSlices - 1; ++s2)
                    load_b128_device_scope(got[j][s2], base + s2 * slice_stride + j * 8 * 256);
            wait_vector_loads<0>();
            bool missing = false;
#pragma unroll
            for (int j = 0; j < TP; ++j)
#pragma unroll
                for (int s2 = 0; s2 < kMidFlaggedSlices - 1; ++s2) {
                    pin_loaded(got[j][s2]);
                    const u32x4 g = got[j][s2];
                    missing |= s2 < KS - 1 && (g.x == 0 || g.y == 0 || g.z == 0 || g.w == 0);
                }
            // the bound is never reached in a working launch; past it the missing words read as NaN
            if (__builtin_amdgcn_ballot_w64(missing) == 0) break;
            if (__builtin_expect(spins == kMidSpinLimit, 0)) {  // the host can see this in the workspace's sticky word
                report_wait_gave_up(error_word_before_exchange_region(partial), kGaveUpMidExchange, lane);
                break;
            }
            __builtin_amdgcn_s_sleep(2);
        }
#pragma unroll
        for (int j = 0; j < TP; ++j) {
            f32x4 total = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s2 = 0; s2 < kMidFlaggedSlices - 1; ++s2)
                if (s2 < KS - 1) {  // ascending K order, this slice's own part last
                    const u32x4 g = got[j][s2];
                    total += __builtin_bit_cast(f32x4, u32x4{~g.x, ~g.y, ~g.z, ~g.w});
                    store_b128_device_scope(base + s2 * slice_stride + j * 8 * 256, u32x4{0, 0, 0, 0});  // zero for the next launch
                }
            store_item(total + own[j], j * 8 + wave);
        }
        return;
    }

    // Exchange between the K slices of the block's tiles: device-scope stores, acknowledged
    // (vmcnt(0)) before the barrier that precedes the arrival count; the last block to arrive
    // adds the slices in ascending K order and leaves the counter zero.
    wait_vector_loads<0>();
    __syncthreads();
    int *counter = counters_all + bz * ncb + bx;
    if (tid == 0) {
        const bool last = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == KS - 1;
        s_last = last;
        if (last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;
    for (int c = wave; c < TP * kPerPair; c += nw) {
        const int item = (c / kPerPair) * 8 + c % kPerPair;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int s2 = 0; s2 < KS; ++s2) {
            u32x4 v;
            load_b128_device_scope(v, partial + s2 * slice_stride + item * 256 + lane * 4);
            wait_vector_loads<0>();
            pin_loaded(v);
            sum += __builtin_bit_cast(f32x4, v);
        }
        store_item(sum, item);
    }
}

// Which row blocks a launch's blocks pass over, a kernel for each so that none carries code or registers it
// does not use (a launch costs more the more registers its wavefronts hold, 0.3 us between the first and
// the second here, and the kernel with both bodies measured 0.5 us above the second at 64 rows):
// kMidOneRowBlock -- at most 32 rows in the launch; kMidTwoRowBlocks -- every run of 64 rows has more
// than 32; kMidRowBlocksByRun -- the last run has 32 or fewer and the runs before it 64, each block looks
// at its own.
constexpr int kMidOneRowBlock = 1, kMidTwoRowBlocks = 2, kMidRowBlocksByRun = 0;

// (one pair per block: 114...153 registers whatever the row blocks, so ten wavefronts there too; with adapters the
// one-row-block instances: 162...166)
template <int TP, int ROW_BLOCKS, bool LORA>
constexpr int kMidWavesOf = ROW_BLOCKS == kMidOneRowBlock || (!LORA && TP == 1) ? kMidWavesMost : kMidWaves;

template <int TP, int GPW, bool LORA, int ROW_BLOCKS>
__global__ __launch_bounds__((kMidWavesOf<TP, ROW_BLOCKS, LORA> * 64)) void w4a16_mid_kernel(
    const uint16_t *__restrict__ A_all, const u32x4 *__restrict__ B, const uint16_t *__restrict__ S,
    uint16_t *__restrict__ C_all, float *partial_all, int *counters_all, int rows, int N, int K, int Gs, int KS,
    int GS, int full_waves, int swiglu, int flagged, int col_shift, MidLora lo) {
    // the block's wavefronts, read here: in the kernel itself the compiler knows every block to be whole
    // and reads the launch's block size, in a device function it first asks whether this block is a partial
    // one (a dependent load at the very start)
    const int nw = blockDim.x >> 6;
    if constexpr (ROW_BLOCKS != kMidRowBlocksByRun) {
        mid_block<TP, GPW, LORA, ROW_BLOCKS>(A_all, B, S, C_all, partial_all, counters_all, rows, N, K, Gs, KS, GS,
                                             full_waves, swiglu, flagged, col_shift, lo, nw);
    } else {
        // the run of 64 rows this block belongs to, as mid_block maps its index (a producer block of a call
        // with adapters belongs to none: either instance runs the projection and returns)
        int bz = blockIdx.z;
        if constexpr (LORA) {
            if (lo.producers > 0) {
                const int id = (int)blockIdx.x - lo.producers;
                bz = id < 0 ? 0 : id / lo.col_blocks / KS;
            }
        }
        if (rows - bz * kMidRows <= 32)
            mid_block<TP, GPW, LORA, 1>(A_all, B, S, C_all, partial_all, counters_all, rows, N, K, Gs, KS, GS, full_waves,
                                        swiglu, flagged, col_shift, lo, nw);
        else
            mid_block<TP, GPW, LORA, 2>(A_all, B, S, C_all, partial_all, counters_all, rows, N, K, Gs, KS, GS, full_waves,
                                        swiglu, flagged, col_shift, lo, nw);
    }
}

template <int TP, int GPW, int ROW_BLOCKS>
hipError_t launch_mid_tgs(const MidArgs &a, hipStream_t stream) {
    const hipError_t attr = allow_dynamic_lds<&w4a16_mid_kernel<TP, GPW, kMidLora, ROW_BLOCKS>>(kMidWavesOf<TP, ROW_BLOCKS, kMidLora> * kMidSlotBytes);
    if (attr != hipSuccess) return attr;
    const int NT = a.N / kTileN;
    const int runs = (a.M + kMidRows - 1) / kMidRows;
    const int last_groups = a.K / kGroupK - (a.KS - 1) * a.GS;  // of the last slice: GS, or fewer
    const int full_waves = (a.GS - a.waves * (GPW - 1)) | ((last_groups - a.waves * (GPW - 1)) << 8);
    MidLora lo{};
    lo.t = (const uint16_t *)a.lora_t;
    lo.b = (const uint16_t *)a.lora_b;
    lo.r_total = a.r_total;
    lo.rp = (a.r_total + 15) / 16 * 16;
    lo.slices = a.lora_slices;
    const int col_blocks = (NT + 2 * TP - 1) / (2 * TP);
    dim3 grid(col_blocks, a.KS, runs);
    if (a.lora_producers > 0) {
        lo.a_cat = (const uint16_t *)a.lora_a;
        lo.words = a.lora_words;
        lo.producers = a.lora_producers;
        lo.row_tiles = (a.M + 15) / 16;
        lo.steps_per_slice = a.lora_steps_per_slice;
        lo.col_blocks = col_blocks;
        lo.consumers = col_blocks * runs;
        lo.ls.count = a.lora_adapters;
        for (int i = 0; i < 8; ++i) {
            lo.ls.ends[i] = a.lora_ends[i];
            lo.ls.scales[i] = a.lora_scales[i];
        }
        grid = dim3(a.lora_producers + col_blocks * a.KS * runs, 1, 1);
    }
    w4a16_mid_kernel<TP, GPW, kMidLora, ROW_BLOCKS><<<grid, a.waves * 64, a.waves * kMidSlotBytes, stream>>>(
        (const uint16_t *)a.A, (const u32x4 *)a.B, (const uint16_t *)a.S, (uint16_t *)a.C, a.partial, a.counters, a.M,
        a.N, a.K, a.Gs, a.KS, a.GS, full_waves, a.swiglu ? 1 : 0, a.flagged ? 1 : 0,
        a.flagged ? exchange_column_shift((NT + 2 * TP - 1) / (2 * TP)) : 0, lo);
    return hipGetLastError();
}

template <int TP, int GPW>
hipError_t launch_mid_tg(const MidArgs &a, hipStream_t stream) {
    if (a.M <= 32) return launch_mid_tgs<TP, GPW, kMidOneRowBlock>(a, stream);
    const int last_run = a.M - (a.M - 1) / kMidRows * kMidRows;
    return last_run <= 32 ? launch_mid_tgs<TP, GPW, kMidRowBlocksByRun>(a, stream)
                          : launch_mid_tgs<TP, GPW, kMidTwoRowBlocks>(a, stream);
}

template <int TP>
hipError_t launch_mid_t(const MidArgs &a, int gpw, hipStream_t stream) {
    switch (gpw) {
        case 1: return launch_mid_tg<TP, 1>(a, stream);
        case 2: return launch_mid_tg<TP, 2>(a, stream);
        case 3: return launch_mid_tg<TP, 3>(a, stream);
        case 4: return launch_mid_tg<TP, 4>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

#if KILN_MID_LORA
// The instances with the low-rank term; the caller (launch_mid) has checked the plan.
hipError_t launch_mid_lora(const MidArgs &a, hipStream_t stream) {
    if (a.r_total < 8 || a.r_total > 64 || a.r_total % 8 != 0 || !a.lora_t || !a.lora_b || a.lora_slices < 1)
        return hipErrorInvalidValue;
    if (a.lora_producers > 0 && !mid_lora_fold_ok(a)) return hipErrorInvalidValue;
    const int gpw = (a.GS + a.waves - 1) / a.waves;
    switch (a.pairs) {
        case 1: return launch_mid_t<1>(a, gpw, stream);
        case 2: return launch_mid_t<2>(a, gpw, stream);
        default: return launch_mid_t<3>(a, gpw, stream);
    }
}
#else
int mid_max_rows_per_run() { return kMidRows; }

// May the projection onto the adapters run in this launch's first blocks?  Those blocks: 256 working threads,
// 16-row tiles, words for (slice, tile) in a copy's 4 KiB; up to four runs of rows.
bool mid_lora_fold_ok(const MidArgs &a) {
    const int row_tiles = (a.M + 15) / 16;
    return a.waves >= 4 && a.lora_slices >= 1 && a.lora_slices <= 16 &&
           row_tiles * a.lora_slices <= kLoraFoldReplicaWords - kMidFoldTileWord &&
           a.lora_producers == row_tiles * a.lora_slices && a.lora_a && a.lora_words && a.lora_adapters >= 1 &&
           a.lora_adapters <= 8 && a.lora_steps_per_slice >= 4 && a.lora_steps_per_slice % 4 == 0 &&
           (long)a.lora_slices * a.lora_steps_per_slice * 32 >= a.K && a.M <= 4 * kMidRows;
}

// What a launch of the mid-M kernel assumes: one to three pairs of tiles per block (N % 256 == 0
// makes the tile count even; a last block may hold fewer pairs), equal K slices, at most eight
// wavefronts of one to four groups each, every wavefront at least one group.
// Ten wavefronts fit a compute unit's LDS (10 x 16 KiB) and, three to a SIMD, hold at most 170 registers each:
// the instances of a pass over one row block do (up to 32 rows; with adapters 162...166
// registers), and those of one pair per block without adapters.
int mid_max_waves(int m, int pairs, bool lora) {
    if (lora) return m <= 32 ? kMidWavesMost : kMidWaves;
    return m <= 32 || pairs == 1 ? kMidWavesMost : kMidWaves;
}

bool mid_plan_ok(const MidArgs &a) {
    if (a.M < 1 || a.N < 256 || a.N % 256 != 0 || a.K < kGroupK || a.K % kGroupK != 0) return false;
    if (a.pairs < 1 || a.pairs > 3) return false;
    const int G = a.K / kGroupK;
    // slices of GS groups; the last one may be shorter (11008 = 86 groups = 29 + 29 + 28)
    if (a.KS < 1 || a.GS < 1 || a.KS * a.GS < G || (a.KS - 1) * a.GS >= G) return false;
    if (a.waves < 1 || a.waves > mid_max_waves(a.M, a.pairs, a.r_total > 0) || a.waves > a.GS) return false;
    const int gpw = (a.GS + a.waves - 1) / a.waves;
    if (gpw > kMidMaxGroups || (a.pairs == 3 && gpw == 4)) return false;  // (3, 4) would spill registers
    const int full_waves = a.GS - a.waves * (gpw - 1);
    // the last slice: every wavefront gpw or gpw - 1 groups there too (none of gpw is fine)
    const int last_full_waves = G - (a.KS - 1) * a.GS - a.waves * (gpw - 1);
    return full_waves >= 1 && full_waves <= a.waves && last_full_waves >= 0 && last_full_waves <= a.waves;
}

// The counter-free exchange deals a pair's items (eight, or four of a pass over one row block) to the block's
// first wavefronts, one each: blocks of eight wavefronts or more.
bool mid_flagged_ok(const MidArgs &a) { return a.KS > 1 && a.KS <= kMidFlaggedSlices && a.waves >= kMidWaves; }

int mid_column_blocks(const MidArgs &a) { return (a.N / kTileN + 2 * a.pairs - 1) / (2 * a.pairs); }

size_t mid_partial_bytes(const MidArgs &a) {
    if (a.KS <= 1) return 0;
    const int runs = (a.M + kMidRows - 1) / kMidRows, col_blocks = mid_column_blocks(a);
    return (size_t)runs * a.KS * col_blocks * (size_t)(a.pairs * 32) * kMidRows * sizeof(float);
}

hipError_t launch_mid(const MidArgs &a, hipStream_t stream) {
    if (!mid_plan_ok(a)) return hipErrorInvalidValue;
    if (a.KS > 1 && (!a.partial || !a.counters)) return hipErrorInvalidValue;
    if (a.flagged && !mid_flagged_ok(a)) return hipErrorInvalidValue;
    if (a.r_total > 0) return launch_mid_lora(a, stream);
    const int gpw = (a.GS + a.waves - 1) / a.waves;
    switch (a.pairs) {
        case 1: return launch_mid_t<1>(a, gpw, stream);
        case 2: return launch_mid_t<2>(a, gpw, stream);
        default: return launch_mid_t<3>(a, gpw, stream);
    }
}
#endif  // KILN_MID_LORA

}  // namespace kiln

#ifdef KILN_MID_TIMELINE
#if KILN_MID_LORA
extern "C" int kiln_mid_timeline_lora(long long *buf) {
#else
extern "C" int kiln_mid_timeline(long long *buf) {
#endif
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(kiln::g_mid_tl), &buf, sizeof(buf));
}
#endif
