// Small-M (decode) W4A16 GEMM kernels for gfx950.
//
// Replace the m <= 16 arm of the reference dispatcher and its persistent
// kernel (crates/kiln-marlin-gemm/csrc/marlin_kernel.cu:754-763, :189-700).
// The problem is bound by the int4 weight stream and, next to it, by fixed
// latencies and the vector instructions that expand the codes.  A wavefront
// reads 1 KiB chunks (16 columns x 128 rows, one scale group) with one 128-bit
// load per lane, expands the codes to bf16 in registers and feeds
// v_mfma_f32_16x16x32_bf16.
//
// Three kernels share that inner step and differ in how a block's chunks are
// dealt to its wavefronts and where the activations live:
//   w4a16_decode_kernel      tile-major runs: any plan, any shape; activations
//                            staged in LDS, or (DIRECT, few rows, short runs)
//                            read from L2 beside each chunk.
//   w4a16_decode_gm_kernel   group-major: a wavefront owns a few groups of K
//                            and multiplies them with every tile of the block;
//                            activations staged in LDS.  For plans of whole
//                            tiles, which the planner prefers.
//   w4a16_decode_gmr_kernel  group-major with the operand fragments in
//                            registers, one or two 16-row slabs (M <= 32) per
//                            pass over the weights.
//
// Work split (tile-major kernel).  K is cut into KS slices (so that a slice of
// the activations fits LDS).  Inside a slice the chunks are numbered tile-major
// (index = tile * gs + group) and cut into runs of exactly U chunks, one run
// per wavefront.  Every wavefront therefore issues the same, compile-time-known
// number of loads, consumes each chunk as it lands, and streams contiguous
// memory; a run touches at most two column tiles.  Tiles that lie inside one
// block are summed through LDS and written directly.  Tiles cut by a block
// boundary or by the K slicing are exchanged as f32 partial tiles through the
// workspace; the last contributor to arrive adds them in ascending K order, so
// the result does not depend on scheduling.
#include <type_traits>

#include "device_common.h"
#include "launch.h"
#include "lora_tail.h"

// This file is compiled twice: as is for the plain kernels, and with -DKILN_DECODE_LORA=1 for the
// instances that add the low-rank term where they store a tile (with the term behind a run-time
// branch the plain launches measured a few hundred nanoseconds slower, and one translation unit
// per set halves the build time).
#ifndef KILN_DECODE_LORA
#define KILN_DECODE_LORA 0
#endif

namespace kiln {

namespace {

constexpr bool kLora = KILN_DECODE_LORA != 0;
constexpr int kMaxWaves = 16;
constexpr int kMaxTouched = 40;  // column tiles one block can touch (16 runs x up to 2, plus slack)
[[maybe_unused]] constexpr int kSlotBytes = 64 * sizeof(f32x4);
constexpr int kOffsetBytes = 32 * 16 * sizeof(float);  // offset terms of up to 32 groups x 16 rows

// f(integral_constant<int, I>) for I = first ... last - 1, unrolled at compile time
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

__device__ __forceinline__ int lds_row_stride(int gs) { return gs * 256 + 16; }  // bytes, padded

typedef __attribute__((address_space(3))) void *lds_ptr_t;

// 16 bytes per lane from global memory straight into LDS at lds_addr + 16 * lane (lds_addr is
// the same for the whole wavefront).  Counts as a vector memory load for s_waitcnt.
__device__ __forceinline__ void stage_b128(const void *gptr, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_addr)
                 : "memory", "m0");
}

// Loads whose completion the kernel tracks itself (explicit s_waitcnt, then pin): the compiler
// neither reorders them nor waits for them.  The destination must stay where it is until pinned.
// Address = wavefront-uniform base (scalar registers) + per-lane byte offset (+ immediate).
__device__ __forceinline__ void request_b128_nt(u32x4 &dst, const void *base, uint32_t lane_off) {
    asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=&v"(dst) : "v"(lane_off), "s"(base) : "memory");
}
template <int IMM>
__device__ __forceinline__ void request_b128(u32x4 &dst, const void *base, uint32_t lane_off) {
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=&v"(dst) : "v"(lane_off), "s"(base), "n"(IMM) : "memory");
}
__device__ __forceinline__ void request_u16(uint32_t &dst, const void *base, uint32_t lane_off) {
    asm volatile("global_load_ushort %0, %1, %2" : "=&v"(dst) : "v"(lane_off), "s"(base) : "memory");
}
// Orders every later use of v after this point (and hence after the preceding s_waitcnt).
__device__ __forceinline__ void pin(u32x4 &v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void pin(uint32_t &v) { asm volatile("" : "+v"(v)); }

// immediate of s_waitcnt for vmcnt(n), other counters unconstrained
constexpr int vmcnt_imm(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

// a / b for 0 <= a < 2^22 and small b > 0, without the integer-division sequence: the float
// quotient is off by at most one.
__device__ __forceinline__ int div_small(int a, int b) {
    int q = (int)((float)a * __builtin_amdgcn_rcpf((float)b));
    const int r = a - q * b;
    q += (r >= b) ? 1 : 0;
    q -= (r < 0) ? 1 : 0;
    return q;
}

// U: chunks per wavefront (register array size); U <= groups per slice.
// DIRECT (M <= 4): the few rows of activations are not staged in LDS; every lane
// reads its own operand fragments (16 bytes per 32 rows of K) from L2 next to the
// chunk they multiply, in the same software pipeline.  Lanes of rows past M read
// row M - 1 (the same cache lines as their neighbours) and zero the value.  This
// removes the wait for the activations and the first barrier from the path
// between launch and the first product; the traffic it adds (64 lanes x 64 bytes
// per chunk, nearly all of it duplicates) only pays off for very few rows.
template <int U, bool DIRECT, bool CROSS, bool LORA>
__global__ __launch_bounds__(kMaxWaves * 64) void w4a16_decode_kernel(
    const uint16_t *__restrict__ A, const u32x4 *__restrict__ B, const uint16_t *__restrict__ S,
    uint16_t *__restrict__ C, float *partial, int *counters, int M, int N, int K, int Gs, int KS,
    int GS, int BPS, int swiglu, LoraTail lo) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    __shared__ int s_last[kMaxTouched];

#ifdef KILN_TIMELINE
    long long tl_t[8]; tl_t[0] = wall_clock64();
#define TL(i) tl_t[i] = wall_clock64()
#else
#define TL(i)
#endif
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw = blockDim.x >> 6;
    const int R = nw * U;  // chunks per block
    const int G = K / kGroupK;
    const int NT = N / kTileN;

    // this block's K slice and position inside the slice
    const int ks = blockIdx.y, bi = blockIdx.x;
    const int g_lo = ks * GS;
    const int gs = min(GS, G - g_lo);
    const int total = NT * gs;  // chunks in the slice
    const int blk0 = bi * R, blk1 = min(total, blk0 + R);

    // this wavefront's run [i0, i0 + U).  A run reaching past the end of the
    // slice still loads U chunks (the U ending at the slice's end, cache hits
    // for all but one wavefront) and skips the first `jskip` of them, so the
    // load sequence is the same straight-line code for every wavefront.
    const int i0 = blk0 + wave * U;
    const int i0s = min(i0, total - U);
    const int jskip = i0 - i0s;
    const int gs_mask = (Gs == 1) ? 0 : -1;
    const int stride = lds_row_stride(gs);

    // Activations first (requesting the first chunks ahead of them measured 0.1-0.2 us slower).
    // Rows < M of the slice go from L2 straight into LDS, one kilobyte per wavefront instruction
    // and no registers in between; the pieces of all rows are dealt round robin to the
    // wavefronts.  Rows from M on are left as LDS holds them: a row of the product
    // depends on its own row of the activations only, and rows from M on are never stored.
    if constexpr (!DIRECT) {
        const unsigned lds_base = (unsigned)(size_t)(lds_ptr_t)lds;
        const int row_bytes = gs * 256;
        const int ppr = (row_bytes + 1023) >> 10;  // pieces per row, the last one possibly short
        const char *a_slice = reinterpret_cast<const char *>(A + (size_t)g_lo * kGroupK) + lane * 16;
        int row = 0, q = wave;
        while (q >= ppr) { q -= ppr; ++row; }
        while (row < M) {
            if (q * 1024 + lane * 16 < row_bytes)
                stage_b128(a_slice + (size_t)row * K * 2 + q * 1024, lds_base + row * stride + q * 1024);
            q += nw;
            while (q >= ppr) { q -= ppr; ++row; }
        }
    }

    // The weight stream: exactly U chunk loads and U scale loads, unconditional, software-
    // pipelined kHead chunks ahead of the chunk being consumed, requested and waited for
    // explicitly (vector memory loads complete in order, so "at most n outstanding" names the
    // chunk that has landed).  A compute unit accepts new loads only as fast as memory delivers,
    // so a wavefront that queued its whole run first would sit in the issue stage (and keep its
    // block from passing the barrier) until most of the data had landed; with a short look-ahead
    // the early chunks are consumed while the later ones stream.  The first kHead chunks are
    // requested before the block waits for its activations.
#ifndef KILN_DEC_HEAD
#define KILN_DEC_HEAD 3
#endif
#ifndef KILN_DEC_OFFS
#define KILN_DEC_OFFS 0
#endif
    constexpr bool kOffs = !DIRECT && KILN_DEC_OFFS;
    constexpr int kHead = DIRECT ? (U < 2 ? U : 2) : (U < KILN_DEC_HEAD ? U : KILN_DEC_HEAD);
    constexpr int kLoads = DIRECT ? 6 : 2;  // loads per chunk
    u32x4 w[U];
    uint32_t sc[U];
    u32x4 af[DIRECT ? U : 1][4];  // DIRECT: this lane's operand fragments of chunk j
    int t = div_small(i0s, gs), g = i0s - t * gs;
    // tile and group of the first consumed chunk (jskip < U <= gs: at most one tile further)
    const bool consumes = jskip < U;
    const int first_wrap = (consumes && g + jskip >= gs) ? 1 : 0;
    const int gA0 = consumes ? g + jskip - first_wrap * gs : 0;
    const int first_tile = consumes ? t + first_wrap : -2;  // -2: this run consumed nothing
    // Running addresses of the window's chunks, their scales and (DIRECT) the activations of
    // their groups: wavefront-uniform, advanced by scalar adds; the per-lane parts are constant.
    const char *b_ptr = reinterpret_cast<const char *>(B) + ((size_t)t * G + (g_lo + g)) * 1024;
    const char *s_ptr = reinterpret_cast<const char *>(S) + ((size_t)t * Gs + ((g_lo + g) & gs_mask)) * (kTileN * 2);
    const int b_wrap = (G - gs) * 1024;                                    // extra step into the next tile
    const int s_step = gs_mask & (kTileN * 2);
    const int s_wrap = (Gs == 1) ? kTileN * 2 : (Gs - gs) * (kTileN * 2);
    const uint32_t b_lane = lane * 16, s_lane = (lane & 15) * 2;
    const int a_row = (lane & 15) < M ? (lane & 15) : M - 1;
    const char *a_ptr = reinterpret_cast<const char *>(A + (size_t)g_lo * kGroupK);
    const uint32_t a_lane_off = (uint32_t)a_row * (uint32_t)K * 2 + (lane >> 4) * 16;
    auto request_chunk = [&](int j) {
        request_b128_nt(w[j], b_ptr, b_lane);
        request_u16(sc[j], s_ptr, s_lane);
        if constexpr (DIRECT) {
            const char *ag = a_ptr + g * 256;
            request_b128<0>(af[j][0], ag, a_lane_off);
            request_b128<64>(af[j][1], ag, a_lane_off);
            request_b128<128>(af[j][2], ag, a_lane_off);
            request_b128<192>(af[j][3], ag, a_lane_off);
        }
        b_ptr += 1024;
        s_ptr += s_step;
        if (++g == gs) {
            g = 0;
            b_ptr += b_wrap;
            s_ptr += s_wrap;
        }
    };
#pragma unroll
    for (int j = 0; j < kHead; ++j) request_chunk(j);

    TL(1);
    // The activations were requested before the kHead chunks: they are in LDS once at most
    // those chunks' loads are outstanding.
    if constexpr (!DIRECT) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoads * kHead));
        __syncthreads();
    }
    TL(2);

    // The B operand carries 136 + d (d = code - 8).  A second product of the
    // same activations with a constant -136 operand removes the offset inside
    // the f32 accumulator exactly: every product is exact and both sums run
    // over the same activations.
    const bf16x8 minus_bias = bf16x8_splat(0xC308C308u);  // bf16(-136) pairs
    const DequantConsts dq = dequant_consts();
    const unsigned char *a_lane = lds + (lane & 15) * stride + (lane >> 4) * 16;
    // LDS behind the activations: offset terms [gs][16 rows] f32 (staged instance), then the
    // wavefronts' partial tiles [wave][2][lane]
    unsigned char *offs = lds + 16 * stride;
    f32x4 *slots = reinterpret_cast<f32x4 *>(DIRECT ? lds : offs + kOffsetBytes);
    const unsigned char *offs_lane = offs + (lane >> 4) * 16;

    // Offset terms, once per block: group g's term, -136 * (sum of the group's activations) per
    // row, is the same for every column tile, so the wavefronts compute the slice's groups
    // between them (four products each, in the accumulator layout: lane 16 q holds rows
    // 4 q ... 4 q + 3) and every chunk's accumulator then starts from its group's term.  The
    // values are the ones four more products per chunk would give.
    if constexpr (kOffs) {
        for (int gq = wave; gq < gs; gq += nw) {
            const unsigned char *ap = a_lane + gq * 256;
            f32x4 o = {0.f, 0.f, 0.f, 0.f};
            o = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8 *>(ap), minus_bias, o, 0, 0, 0);
            o = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8 *>(ap + 64), minus_bias, o, 0, 0, 0);
            o = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8 *>(ap + 128), minus_bias, o, 0, 0, 0);
            o = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8 *>(ap + 192), minus_bias, o, 0, 0, 0);
            if ((lane & 15) == 0) *reinterpret_cast<f32x4 *>(offs + gq * 64 + (lane >> 4) * 16) = o;
        }
        __syncthreads();
    }

    // Straight-line code for all U chunks (no branches, so the compiler can
    // overlap one chunk's LDS reads with the previous chunk's products).  A run
    // touches at most two tiles: y0 collects the chunks of the first, y1 of the
    // second (CROSS; without it the plan guarantees that no run crosses a tile
    // boundary and y0 is the only sum); chunks before `jskip` are multiplied by a
    // zero scale.
    __shared__ int s_first_tile[kMaxWaves];
    f32x4 y0 = {0.f, 0.f, 0.f, 0.f}, y1 = {0.f, 0.f, 0.f, 0.f};
    static_for<0, U>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        if constexpr (j + kHead < U) request_chunk(j + kHead);
        // chunk j has landed once only the chunks requested after it are outstanding
        constexpr int kAhead = (U - 1 - j) < kHead ? (U - 1 - j) : kHead;
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoads * kAhead));
        pin(w[j]);
        pin(sc[j]);
        if constexpr (DIRECT) {
#pragma unroll
            for (int q = 0; q < 4; ++q) pin(af[j][q]);
        }
        const int rel = j - jskip;          // position inside the consumed run
        int gj = gA0 + rel;
        const bool valid = rel >= 0;
        const bool second = CROSS && gj >= gs;
        gj = second ? gj - gs : gj;
        gj = valid ? gj : 0;
        bf16x8 a0, a1, a2, a3;
        if constexpr (DIRECT) {
            // the fragments were loaded for the chunk's own group, whatever `valid` says
            const bool live = (lane & 15) < M;
            const u32x4 z = {0u, 0u, 0u, 0u};
            a0 = __builtin_bit_cast(bf16x8, live ? af[j][0] : z);
            a1 = __builtin_bit_cast(bf16x8, live ? af[j][1] : z);
            a2 = __builtin_bit_cast(bf16x8, live ? af[j][2] : z);
            a3 = __builtin_bit_cast(bf16x8, live ? af[j][3] : z);
        } else {
            const unsigned char *ap = a_lane + gj * 256;
            a0 = *reinterpret_cast<const bf16x8 *>(ap);
            a1 = *reinterpret_cast<const bf16x8 *>(ap + 64);
            a2 = *reinterpret_cast<const bf16x8 *>(ap + 128);
            a3 = *reinterpret_cast<const bf16x8 *>(ap + 192);
        }
        // acc starts from the offset term of this group: -136 * (sum of the group's activations)
        f32x4 acc;
        if constexpr (!kOffs) {
            acc = f32x4{0.f, 0.f, 0.f, 0.f};
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, minus_bias, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, minus_bias, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2, minus_bias, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a3, minus_bias, acc, 0, 0, 0);
        } else {
            acc = *reinterpret_cast<const f32x4 *>(offs_lane + gj * 64);
        }
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, codes_to_bf16x8(w[j].x, dq), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, codes_to_bf16x8(w[j].y, dq), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2, codes_to_bf16x8(w[j].z, dq), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a3, codes_to_bf16x8(w[j].w, dq), acc, 0, 0, 0);
        const float sv = f16_bits_to_f32((uint16_t)sc[j]);
        if constexpr (CROSS) {
            const float m0 = (valid && !second) ? 1.f : 0.f;  // wave-uniform
            const float m1 = (valid && second) ? 1.f : 0.f;
            y0 += acc * (sv * m0);
            y1 += acc * (sv * m1);
        } else {
            y0 += acc * (valid ? sv : 0.f);
        }
    });
    slots[(wave * 2 + 0) * 64 + lane] = y0;
    if constexpr (CROSS) slots[(wave * 2 + 1) * 64 + lane] = y1;
    TL(3);
    if (lane == 0) s_first_tile[wave] = first_tile;
    __syncthreads();
    TL(4);
    if (blk0 >= total) return;  // block past the end of the slice (grid padding)

    // Sum the wavefronts' partial tiles in wavefront (= ascending K) order, one tile per
    // wavefront at a time, every lane on the four elements it would hold of that tile in the
    // accumulator layout: lane c + 16 q has rows 4 q ... 4 q + 3 of column c.
    const int tf = div_small(blk0, gs), tl = div_small(blk1 - 1, gs);  // tiles this block touches
    const int ntouched = tl - tf + 1;
    const int q4 = lane >> 4, c = lane & 15;
    auto store_tile = [&](f32x4 v, int tt) {
        if constexpr (LORA) lora_add(v, lo, 0, M, tt, lane);
        store_tile_rows(C, N, M, 4 * q4, tt, c, v, swiglu != 0);
    };
    for (int ti = wave; ti < ntouched; ti += nw) {
        const int tt = tf + ti;
        const int lo = max(tt * gs, blk0), hi = min((tt + 1) * gs, blk1);  // chunks of tt in this block
        const int w_first = (lo - blk0) / U, w_last = (hi - 1 - blk0) / U;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int wv = w_first; wv <= w_last; ++wv)
            sum += slots[(wv * 2 + ((CROSS && tt != s_first_tile[wv]) ? 1 : 0)) * 64 + lane];
        if (KS == 1 && hi - lo == gs) {
            store_tile(sum, tt);
        } else {
            // device-coherent stores: they reach the other dies without a cache flush.
            // part 0 = the block holding the tile's first chunk of this slice, part 1 = the next block
            const int part = (lo == tt * gs) ? 0 : 1;
            float *dst = partial + ((size_t)(ks * 2 + part) * NT + tt) * 256 + lane * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                __hip_atomic_store(dst + i, sum[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
#ifdef KILN_TIMELINE
    TL(5);
    if (lane == 0) for (int i = 0; i < 8; ++i) ((long long *)partial)[(1 << 20) + ((size_t)(blockIdx.y * BPS + blockIdx.x) * 16 + wave) * 8 + i] = tl_t[i];
#endif
    if (KS == 1 && blk0 == tf * gs && blk1 == (tl + 1) * gs) return;  // nothing was exchanged

    // Exchange of partial tiles.  They are written and read with device-scope
    // atomic accesses (no whole-cache write-back or invalidate).  A barrier by itself
    // orders nothing outside the workgroup, so every wavefront first waits until its own
    // stores have been acknowledged (vmcnt(0)); only then does the barrier let the block's
    // arrivals be counted.  For each tile, the last contributor to arrive adds all parts
    // in ascending K order.
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
    if (tid < ntouched) {
        const int tt = tf + tid;
        const int lo = max(tt * gs, blk0), hi = min((tt + 1) * gs, blk1);
        int last = 0;
        if (!(KS == 1 && hi - lo == gs)) {
            int expected = 0;  // contributors to this tile over all slices
            for (int s2 = 0; s2 < KS; ++s2) {
                const int gs2 = min(GS, G - s2 * GS);
                expected += ((tt * gs2) / R != ((tt + 1) * gs2 - 1) / R) ? 2 : 1;
            }
            last = (__hip_atomic_fetch_add(counters + tt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
                    expected - 1);
        }
        s_last[tid] = last;
    }
    __syncthreads();
    for (int ti = wave; ti < ntouched; ti += nw) {
        if (!s_last[ti]) continue;
        const int tt = tf + ti;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int s2 = 0; s2 < KS; ++s2) {
            const int gs2 = min(GS, G - s2 * GS);
            const int parts = ((tt * gs2) / R != ((tt + 1) * gs2 - 1) / R) ? 2 : 1;
            for (int p = 0; p < parts; ++p) {
                const float *src = partial + ((size_t)(s2 * 2 + p) * NT + tt) * 256 + lane * 4;
                f32x4 v;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    v[i] = __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                sum += v;
            }
        }
        store_tile(sum, tt);
        // leave the counter zero for the next call
        if (lane == 0) __hip_atomic_store(counters + tt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Group-major instance for plans whose blocks hold T whole column tiles of a slice and whose
// wavefronts divide the slice's groups evenly (GPW groups each).  A wavefront multiplies its
// GPW groups with all T tiles: the operand fragments of a group are read from LDS once and the
// offset term (four products with the constant -136 operand) is formed once per group instead
// of once per chunk, so a chunk costs 4 + 4 / T products instead of 8 and a quarter of the LDS
// reads; per chunk the arithmetic is the same sequence as in the kernel above (offset products,
// then code products, on one accumulator).  The price is the reduction: every tile is the sum
// of all wavefronts' partial tiles.
template <int T, int GPW, bool LORA>
__global__ __launch_bounds__(kMaxWaves * 64) void w4a16_decode_gm_kernel(
    const uint16_t *__restrict__ A, const u32x4 *__restrict__ B, const uint16_t *__restrict__ S,
    uint16_t *__restrict__ C, float *partial, int *counters, int M, int N, int K, int Gs, int KS,
    int GS, int full_waves, int swiglu, LoraTail lo) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    __shared__ int s_last[T];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw = blockDim.x >> 6;
    const int G = K / kGroupK;
    const int NT = N / kTileN;
    const int ks = blockIdx.y;
    const int g_lo = ks * GS;       // all slices have GS groups
    const int tf = blockIdx.x * T;  // first tile of the block; tiles from NT on do not exist
    const int gs_mask = (Gs == 1) ? 0 : -1;
    const int stride = lds_row_stride(GS);
    // The first `full_waves` wavefronts own GPW groups each, the others GPW - 1 (GS need not be a
    // multiple of the block size: 20 groups over 12 wavefronts, 2 + 2 + 1 on every SIMD, finish
    // earlier than 10 wavefronts of 2 groups, of which two SIMDs hold three).
    const bool full = wave < full_waves;
    const int g_first = full ? wave * GPW : full_waves * GPW + (wave - full_waves) * (GPW - 1);  // in the slice

    // activations of the slice: as in the kernel above
    {
        const unsigned lds_base = (unsigned)(size_t)(lds_ptr_t)lds;
        const int row_bytes = GS * 256;
        const int ppr = (row_bytes + 1023) >> 10;
        const char *a_slice = reinterpret_cast<const char *>(A + (size_t)g_lo * kGroupK) + lane * 16;
        int row = 0, q = wave;
        while (q >= ppr) { q -= ppr; ++row; }
        while (row < M) {
            if (q * 1024 + lane * 16 < row_bytes)
                stage_b128(a_slice + (size_t)row * K * 2 + q * 1024, lds_base + row * stride + q * 1024);
            q += nw;
            while (q >= ppr) { q -= ppr; ++row; }
        }
    }

    // chunk j of the wavefront = (group j / T, tile j % T); a tile past the end is read as the
    // last tile and never stored
    u32x4 w[T * GPW];
    uint32_t sc[T * GPW];
    const int g0 = g_lo + g_first;
    const uint32_t b_lane = lane * 16, s_lane = (lane & 15) * 2;
    auto request_chunk = [&](auto jc) {
        constexpr int j = decltype(jc)::value;
        constexpr int gi = j / T, ti = j % T;
        const int tt = min(tf + ti, NT - 1);
        const char *b_ptr = reinterpret_cast<const char *>(B) + ((size_t)tt * G + (g0 + gi)) * 1024;
        const char *s_ptr = reinterpret_cast<const char *>(S) + ((size_t)tt * Gs + ((g0 + gi) & gs_mask)) * (kTileN * 2);
        request_b128_nt(w[j], b_ptr, b_lane);
        request_u16(sc[j], s_ptr, s_lane);
    };

    const bf16x8 minus_bias = bf16x8_splat(0xC308C308u);  // bf16(-136) pairs
    const DequantConsts dq = dequant_consts();
    const unsigned char *a_lane = lds + (lane & 15) * stride + (lane >> 4) * 16 + g_first * 256;
    f32x4 *slots = reinterpret_cast<f32x4 *>(lds + 16 * stride);  // [wave][T][lane]
    f32x4 y[T];
#pragma unroll
    for (int ti = 0; ti < T; ++ti) y[ti] = f32x4{0.f, 0.f, 0.f, 0.f};
    bf16x8 a0, a1, a2, a3;
    f32x4 offset_term;
    // The wavefront's chunks, for its number of groups.  Everything from the first request to the
    // last use is straight-line code inside one branch, the block's barrier included (one barrier
    // instruction per branch, every wavefront executes exactly one): a register that is requested
    // in one basic block and used in another may be copied in between -- before its data has
    // arrived, since the compiler does not know that the request is a load.
    auto run = [&](auto nc) {
        constexpr int U = T * decltype(nc)::value, kHead = U < 3 ? U : 3;
        // the first chunks are requested before the block waits for its activations
        static_for<0, kHead>(request_chunk);
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(2 * kHead));
        __syncthreads();
        static_for<0, U>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            constexpr int gi = j / T, ti = j % T;
            if constexpr (j + kHead < U) request_chunk(std::integral_constant<int, j + kHead>{});
            constexpr int kAhead = (U - 1 - j) < kHead ? (U - 1 - j) : kHead;
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(2 * kAhead));
            pin(w[j]);
            pin(sc[j]);
            if constexpr (ti == 0) {  // next group: its operand fragments and its offset term
                const unsigned char *ap = a_lane + gi * 256;
                a0 = *reinterpret_cast<const bf16x8 *>(ap);
                a1 = *reinterpret_cast<const bf16x8 *>(ap + 64);
                a2 = *reinterpret_cast<const bf16x8 *>(ap + 128);
                a3 = *reinterpret_cast<const bf16x8 *>(ap + 192);
                offset_term = f32x4{0.f, 0.f, 0.f, 0.f};
                offset_term = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, minus_bias, offset_term, 0, 0, 0);
                offset_term = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, minus_bias, offset_term, 0, 0, 0);
                offset_term = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2, minus_bias, offset_term, 0, 0, 0);
                offset_term = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a3, minus_bias, offset_term, 0, 0, 0);
            }
            f32x4 acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, codes_to_bf16x8(w[j].x, dq), offset_term, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, codes_to_bf16x8(w[j].y, dq), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2, codes_to_bf16x8(w[j].z, dq), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a3, codes_to_bf16x8(w[j].w, dq), acc, 0, 0, 0);
            y[ti] += acc * f16_bits_to_f32((uint16_t)sc[j]);
        });
    };
    if (full) run(std::integral_constant<int, GPW>{});
    else if constexpr (GPW > 1) run(std::integral_constant<int, GPW - 1>{});
#pragma unroll
    for (int ti = 0; ti < T; ++ti) slots[(wave * T + ti) * 64 + lane] = y[ti];
    __syncthreads();

    // tile ti = the sum of all wavefronts' partial tiles, in wavefront (= ascending K) order
    const int q4 = lane >> 4, c = lane & 15;
    auto store_tile = [&](f32x4 v, int tt) {
        if constexpr (LORA) lora_add(v, lo, 0, M, tt, lane);
        store_tile_rows(C, N, M, 4 * q4, tt, c, v, swiglu != 0);
    };
    const int tiles = min(T, NT - tf);
    for (int ti = wave; ti < tiles; ti += nw) {
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int wv = 0; wv < nw; ++wv) sum += slots[(wv * T + ti) * 64 + lane];
        if (KS == 1) {
            store_tile(sum, tf + ti);
        } else {
            float *dst = partial + ((size_t)(ks * 2) * NT + tf + ti) * 256 + lane * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                __hip_atomic_store(dst + i, sum[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (KS == 1) return;

    // exchange between the slices: as in the kernel above, one part per slice (every
    // wavefront's stores acknowledged, then the barrier, then the arrival is counted)
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
    if (tid < tiles)
        s_last[tid] = __hip_atomic_fetch_add(counters + tf + tid, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == KS - 1;
    __syncthreads();
    for (int ti = wave; ti < tiles; ti += nw) {
        if (!s_last[ti]) continue;
        const int tt = tf + ti;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int s2 = 0; s2 < KS; ++s2) {
            const float *src = partial + ((size_t)(s2 * 2) * NT + tt) * 256 + lane * 4;
            f32x4 v;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            sum += v;
        }
        store_tile(sum, tt);
        if (lane == 0) __hip_atomic_store(counters + tt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Request schedule of the register-fragment instance (chunk j = group j / T, tile j % T;
// fragments are requested AH groups ahead of their use, into AH + 1 register buffers):
//   before the loop: fragments of groups 0 ... AH - 1, then chunks 0 ... HEAD - 1;
//   step j: chunk j + HEAD (if any), then, if j starts group gi and gi + AH < GPW, the fragments
//   of group gi + AH; then the wait; then chunk j is consumed.
// A chunk is 2 loads, a group's fragments 4 * SL.  gmr_outstanding(j) = how many loads may
// still be outstanding at step j's wait: those requested after chunk j and, where step j starts a
// group, after that group's fragments.
constexpr int gmr_groups_ahead(int T, int SL) {
    const int want = (3 + T - 1) / T, most = SL == 2 ? 2 : 3;  // about three chunks of lead
    return want < 1 ? 1 : (want > most ? most : want);
}
template <int T, int GPW, int SL, int HEAD, int AH>
constexpr int gmr_outstanding(int j) {
    constexpr int U = T * GPW;
    // step at which a request is issued; before the loop: -2 for fragments, -1 for chunks (the
    // fragments come first); within a step the chunk request precedes the fragment request
    auto chunk_step = [](int jj) { return jj < HEAD ? -1 : jj - HEAD; };
    auto frag_step = [](int g) { return g < AH ? -2 : (g - AH) * T; };
    int allowed = 0;
    for (int jj = j + 1; jj < U && chunk_step(jj) <= j; ++jj) allowed += 2;
    for (int g = AH; g < GPW; ++g)
        if (frag_step(g) <= j && frag_step(g) >= chunk_step(j)) allowed += 4 * SL;
    if (j % T == 0 && j / T >= 1) {  // the group's fragments must have landed too
        const int g = j / T, fs = frag_step(g);
        int after_frag = 0;
        for (int jj = 0; jj < U; ++jj)
            if (chunk_step(jj) <= j && (chunk_step(jj) > fs || (fs == -2 && chunk_step(jj) == -1))) after_frag += 2;
        for (int g2 = g + 1; g2 < GPW; ++g2)
            if (frag_step(g2) <= j) after_frag += 4 * SL;
        if (after_frag < allowed) allowed = after_frag;
    }
    return allowed;
}

// Group-major instance without LDS staging, for up to 16 * SL rows (SL = 1, 2 slabs of 16).
// In the group-major split a wavefront is the only user of its groups' activations, so it
// reads its operand fragments from L2 straight into registers (each element once per block, as
// the staged instances do) and nothing waits at a barrier before the first product.  With
// SL = 2 one launch multiplies 17...32 rows with weights streamed once; the two slabs of a
// tile go through the exchange as part 0 and part 1 (blocks of whole tiles have no other use
// for part 1).
template <int T, int GPW, int SL, bool LORA>
__global__ __launch_bounds__(12 * 64) void w4a16_decode_gmr_kernel(
    const uint16_t *__restrict__ A_all, const u32x4 *__restrict__ B, const uint16_t *__restrict__ S,
    uint16_t *__restrict__ C_all, float *partial_all, int *counters_all, int rows, int N, int K, int Gs, int KS,
    int GS, int swiglu, LoraTail lo) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    __shared__ int s_last[T];
    constexpr int U = T * GPW;  // chunks per wavefront
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw = blockDim.x >> 6;  // == GS / GPW
    const int G = K / kGroupK;
    const int NT = N / kTileN;
    // blockIdx.z: which run of 16 * SL rows of the launch (each with its own counters and partial
    // tiles; a launch of several runs saves the gap between two launches, nothing else)
    const int zr = blockIdx.z * (16 * SL);
    const uint16_t *__restrict__ A = A_all + (size_t)zr * K;
    uint16_t *__restrict__ C = C_all + (size_t)zr * (swiglu ? N >> 1 : N);  // the fused result is half as wide
    float *partial = partial_all + (size_t)blockIdx.z * KS * 2 * NT * 256;
    int *counters = counters_all + blockIdx.z * NT;
    const int M = min(rows - zr, 16 * SL);
    if constexpr (LORA) lo.t += (size_t)zr * lo.rp;
    const int ks = blockIdx.y;
    const int g_lo = ks * GS;       // all slices have GS groups
    const int tf = blockIdx.x * T;  // first tile of the block; tiles from NT on do not exist
    const int gs_mask = (Gs == 1) ? 0 : -1;
    const int g0 = g_lo + wave * GPW;

    // Operand fragments of this wavefront's groups: lane c + 16 q reads row c (of each slab),
    // k = 32 step + 8 q ... + 7; rows from M on read row M - 1 and are never stored.  AH + 1
    // buffers: group gi + AH is requested when group gi starts.
    constexpr int AH = gmr_groups_ahead(T, SL), NB = AH + 1;
    u32x4 af[NB][SL][4];
    const char *a_ptr = reinterpret_cast<const char *>(A + (size_t)g0 * kGroupK);
    uint32_t a_off[SL];
#pragma unroll
    for (int sl = 0; sl < SL; ++sl)
        a_off[sl] = (uint32_t)min(16 * sl + (lane & 15), M - 1) * (uint32_t)K * 2 + (lane >> 4) * 16;
    auto request_fragments = [&](auto gc) {
        constexpr int gi = decltype(gc)::value;
#pragma unroll
        for (int sl = 0; sl < SL; ++sl) {
            request_b128<0>(af[gi % NB][sl][0], a_ptr + gi * 256, a_off[sl]);
            request_b128<64>(af[gi % NB][sl][1], a_ptr + gi * 256, a_off[sl]);
            request_b128<128>(af[gi % NB][sl][2], a_ptr + gi * 256, a_off[sl]);
            request_b128<192>(af[gi % NB][sl][3], a_ptr + gi * 256, a_off[sl]);
        }
    };
    static_for<0, (AH < GPW ? AH : GPW)>(request_fragments);

    // chunk j of the wavefront = (group j / T, tile j % T); a tile past the end is read as the
    // last tile and never stored
    constexpr int kHead = U < 3 ? U : 3;
    u32x4 w[U];
    uint32_t sc[U];
    const uint32_t b_lane = lane * 16, s_lane = (lane & 15) * 2;
    auto request_chunk = [&](auto jc) {
        constexpr int j = decltype(jc)::value;
        constexpr int gi = j / T, ti = j % T;
        const int tt = min(tf + ti, NT - 1);
        const char *b_ptr = reinterpret_cast<const char *>(B) + ((size_t)tt * G + (g0 + gi)) * 1024;
        const char *s_ptr = reinterpret_cast<const char *>(S) + ((size_t)tt * Gs + ((g0 + gi) & gs_mask)) * (kTileN * 2);
        request_b128_nt(w[j], b_ptr, b_lane);
        request_u16(sc[j], s_ptr, s_lane);
    };
    static_for<0, kHead>(request_chunk);

    const bf16x8 minus_bias = bf16x8_splat(0xC308C308u);  // bf16(-136) pairs
    const DequantConsts dq = dequant_consts();
    f32x4 *slots = reinterpret_cast<f32x4 *>(lds);  // [wave][T][SL][lane]
    f32x4 y[T][SL];
#pragma unroll
    for (int ti = 0; ti < T; ++ti)
#pragma unroll
        for (int sl = 0; sl < SL; ++sl) y[ti][sl] = f32x4{0.f, 0.f, 0.f, 0.f};
    f32x4 offset_term[SL];
    static_for<0, U>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        constexpr int gi = j / T, ti = j % T;
        // requests of step j: chunk j + kHead, then (first tile of a group) the next group's fragments
        if constexpr (j + kHead < U) request_chunk(std::integral_constant<int, j + kHead>{});
        if constexpr (ti == 0 && gi + AH < GPW) request_fragments(std::integral_constant<int, gi + AH>{});
        // loads complete in order: wait until only those requested after chunk j (and, where a
        // group starts, after its fragments) are outstanding
        constexpr int kWait = gmr_outstanding<T, GPW, SL, kHead, AH>(j);
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kWait));
        pin(w[j]);
        pin(sc[j]);
        if constexpr (ti == 0) {  // next group: its offset terms
#pragma unroll
            for (int sl = 0; sl < SL; ++sl) {
#pragma unroll
                for (int q = 0; q < 4; ++q) pin(af[gi % NB][sl][q]);
                f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    o = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[gi % NB][sl][q]), minus_bias, o, 0, 0, 0);
                offset_term[sl] = o;
            }
        }
        const bf16x8 b0 = codes_to_bf16x8(w[j].x, dq), b1 = codes_to_bf16x8(w[j].y, dq);
        const bf16x8 b2 = codes_to_bf16x8(w[j].z, dq), b3 = codes_to_bf16x8(w[j].w, dq);
        const float sv = f16_bits_to_f32((uint16_t)sc[j]);
#pragma unroll
        for (int sl = 0; sl < SL; ++sl) {
            f32x4 acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[gi % NB][sl][0]), b0, offset_term[sl], 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[gi % NB][sl][1]), b1, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[gi % NB][sl][2]), b2, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af[gi % NB][sl][3]), b3, acc, 0, 0, 0);
            y[ti][sl] += acc * sv;
        }
    });
#pragma unroll
    for (int ti = 0; ti < T; ++ti)
#pragma unroll
        for (int sl = 0; sl < SL; ++sl) slots[((wave * T + ti) * SL + sl) * 64 + lane] = y[ti][sl];
    __syncthreads();

    // (tile, slab) = the sum of all wavefronts' partial tiles, in wavefront (= ascending K) order
    const int q4 = lane >> 4, c = lane & 15;
    auto store_tile = [&](f32x4 v, int tt, int sl) {
        if constexpr (LORA) lora_add(v, lo, 16 * sl, M, tt, lane);
        store_tile_rows(C, N, M, 16 * sl + 4 * q4, tt, c, v, swiglu != 0);
    };
    const int tiles = min(T, NT - tf);
    for (int it = wave; it < tiles * SL; it += nw) {
        const int ti = it / SL, sl = it - ti * SL;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int wv = 0; wv < nw; ++wv) sum += slots[((wv * T + ti) * SL + sl) * 64 + lane];
        if (KS == 1) {
            store_tile(sum, tf + ti, sl);
        } else {
            float *dst = partial + ((size_t)(ks * 2 + sl) * NT + tf + ti) * 256 + lane * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                __hip_atomic_store(dst + i, sum[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (KS == 1) return;

    // exchange between the slices: one part per slice and slab (every wavefront's stores
    // acknowledged, then the barrier, then the arrival is counted)
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
    if (tid < tiles) {
        const bool last =
            __hip_atomic_fetch_add(counters + tf + tid, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == KS - 1;
        s_last[tid] = last;
        // every contributor has arrived: leave the counter zero for the next call
        if (last) __hip_atomic_store(counters + tf + tid, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    for (int it = wave; it < tiles * SL; it += nw) {
        const int ti = it / SL, sl = it - ti * SL;
        if (!s_last[ti]) continue;
        const int tt = tf + ti;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int s2 = 0; s2 < KS; ++s2) {
            const float *src = partial + ((size_t)(s2 * 2 + sl) * NT + tt) * 256 + lane * 4;
            f32x4 v;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            sum += v;
        }
        store_tile(sum, tt, sl);
    }
}

template <int T, int GPW, int SL>
hipError_t launch_gmr_tgs(const DecodeArgs &a, hipStream_t stream) {
    const hipError_t attr = allow_dynamic_lds<&w4a16_decode_gmr_kernel<T, GPW, SL, kLora>>(decode_max_lds_bytes());
    if (attr != hipSuccess) return attr;
    const int NT = a.N / kTileN;
    const int runs = a.rows > a.M ? (a.rows + 16 * SL - 1) / (16 * SL) : 1;
    w4a16_decode_gmr_kernel<T, GPW, SL, kLora><<<dim3((NT + T - 1) / T, a.KS, runs), a.waves * 64,
                                                 decode_gmr_lds_bytes(a.waves, T, SL), stream>>>(
        (const uint16_t *)a.A, (const u32x4 *)a.B, (const uint16_t *)a.S, (uint16_t *)a.C, a.partial,
        a.counters, a.rows > a.M ? a.rows : a.M, a.N, a.K, a.Gs, a.KS, a.GS, a.swiglu ? 1 : 0, lora_tail(a));
    return hipGetLastError();
}

template <int T, int SL>
hipError_t launch_gmr_ts(const DecodeArgs &a, int gpw, hipStream_t stream) {
    switch (gpw) {
        case 1: return launch_gmr_tgs<T, 1, SL>(a, stream);
        case 2: return launch_gmr_tgs<T, 2, SL>(a, stream);
        case 3: return launch_gmr_tgs<T, 3, SL>(a, stream);
        case 4: return launch_gmr_tgs<T, 4, SL>(a, stream);
        case 5: return launch_gmr_tgs<T, 5, SL>(a, stream);
        case 6: return launch_gmr_tgs<T, 6, SL>(a, stream);
        case 8: return launch_gmr_tgs<T, 8, SL>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

template <int SL>
hipError_t launch_gmr_s(const DecodeArgs &a, hipStream_t stream) {
    const int gpw = a.GS / a.waves;
    switch (a.waves * a.U / a.GS) {
        case 1:  // one tile per block: only with one slab and one or two groups per wavefront
            if constexpr (SL == 1) {
                if (gpw == 1) return launch_gmr_tgs<1, 1, 1>(a, stream);
                if (gpw == 2) return launch_gmr_tgs<1, 2, 1>(a, stream);
            }
            return hipErrorInvalidValue;
        case 2: return launch_gmr_ts<2, SL>(a, gpw, stream);
        case 3: return launch_gmr_ts<3, SL>(a, gpw, stream);
        case 4: return launch_gmr_ts<4, SL>(a, gpw, stream);
        case 5: return launch_gmr_ts<5, SL>(a, gpw, stream);
        case 6: return launch_gmr_ts<6, SL>(a, gpw, stream);
        default: return hipErrorInvalidValue;
    }
}

template <int T, int GPW>
hipError_t launch_gm_tg(const DecodeArgs &a, hipStream_t stream) {
    const hipError_t attr = allow_dynamic_lds<&w4a16_decode_gm_kernel<T, GPW, kLora>>(decode_max_lds_bytes());
    if (attr != hipSuccess) return attr;
    const int NT = a.N / kTileN;
    const int full_waves = a.GS - a.waves * (GPW - 1);  // wavefronts that own GPW groups; the others GPW - 1
    w4a16_decode_gm_kernel<T, GPW, kLora><<<dim3((NT + T - 1) / T, a.KS), a.waves * 64,
                                            decode_gm_lds_bytes(a.GS, a.waves, T), stream>>>(
        (const uint16_t *)a.A, (const u32x4 *)a.B, (const uint16_t *)a.S, (uint16_t *)a.C, a.partial,
        a.counters, a.M, a.N, a.K, a.Gs, a.KS, a.GS, full_waves, a.swiglu ? 1 : 0, lora_tail(a));
    return hipGetLastError();
}

template <int T>
hipError_t launch_gm_t(const DecodeArgs &a, int gpw, hipStream_t stream) {
    switch (gpw) {
        case 1: return launch_gm_tg<T, 1>(a, stream);
        case 2: return launch_gm_tg<T, 2>(a, stream);
        case 3: return launch_gm_tg<T, 3>(a, stream);
        case 4: return launch_gm_tg<T, 4>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

template <int U, bool DIRECT, bool CROSS>
hipError_t launch_udc(const DecodeArgs &a, hipStream_t stream) {
    const hipError_t attr = allow_dynamic_lds<&w4a16_decode_kernel<U, DIRECT, CROSS, kLora>>(decode_max_lds_bytes());
    if (attr != hipSuccess) return attr;
    const size_t lds = decode_lds_bytes(a.GS, a.waves, DIRECT);
    w4a16_decode_kernel<U, DIRECT, CROSS, kLora><<<dim3(a.BPS, a.KS), a.waves * 64, lds, stream>>>(
        (const uint16_t *)a.A, (const u32x4 *)a.B, (const uint16_t *)a.S, (uint16_t *)a.C, a.partial,
        a.counters, a.M, a.N, a.K, a.Gs, a.KS, a.GS, a.BPS, a.swiglu ? 1 : 0, lora_tail(a));
    return hipGetLastError();
}

template <int U>
hipError_t launch_u(const DecodeArgs &a, hipStream_t stream) {
    // A run can only cross a tile boundary if the boundaries are not multiples of the run length:
    // blocks start at multiples of R = waves * U, runs at multiples of U.
    const int G = a.K / kGroupK, gs_last = G - (a.KS - 1) * a.GS;
    const bool cross = a.GS % U != 0 || gs_last % U != 0;
    if (a.direct) return cross ? launch_udc<U, true, true>(a, stream) : launch_udc<U, true, false>(a, stream);
    return cross ? launch_udc<U, false, true>(a, stream) : launch_udc<U, false, false>(a, stream);
}

}  // namespace

#if !KILN_DECODE_LORA
int decode_max_waves() { return kMaxWaves; }
int decode_max_run() { return 12; }
int decode_max_tiles_per_block() { return kMaxTouched; }
int decode_max_lds_bytes() { return 160 * 1024 - 1024; }
size_t decode_lds_bytes(int GS, int waves, bool direct) {  // the direct instance stages no activations
    return (direct ? 0 : (size_t)16 * (GS * 256 + 16) + kOffsetBytes) + (size_t)waves * 2 * kSlotBytes;
}

size_t decode_gm_lds_bytes(int GS, int waves, int tiles) {
    return (size_t)16 * (GS * 256 + 16) + (size_t)waves * tiles * kSlotBytes;
}
size_t decode_gmr_lds_bytes(int waves, int tiles, int slabs) { return (size_t)waves * tiles * slabs * kSlotBytes; }

// The register-fragment group-major instance: whole tiles (1...6 per block) in equal slices of
// any length whose groups divide evenly among at most 12 wavefronts (its register budget), 1...6
// or 8 groups each; the only instance that takes up to 32 rows.
bool decode_group_major_regs_ok(const DecodeArgs &a) {
    const int G = a.K / kGroupK;
    if (a.direct || a.group_major == 0 || a.group_major == 1 || a.KS * a.GS != G || a.waves > 12) return false;
    const int R = a.waves * a.U;
    if (R % a.GS != 0 || a.GS % a.waves != 0) return false;
    const int T = R / a.GS, gpw = a.GS / a.waves;
    // two slabs: the instances below would spill registers
    if (a.M > 16 && ((T == 2 && gpw >= 5) || (T >= 5 && gpw >= 3))) return false;
    if (T == 1 && (gpw > 2 || a.M > 16)) return false;  // not instantiated: the planner never wants them
    return T >= 1 && T <= 6 && gpw >= 1 && gpw <= 8 && gpw != 7 && a.M <= 32 &&
           decode_gmr_lds_bytes(a.waves, T, a.M > 16 ? 2 : 1) <= (size_t)decode_max_lds_bytes();
}

// The LDS-staged group-major instance runs plans of gm_tiles = 2...6 whole tiles per block in
// equal slices; the slice's groups are dealt to the wavefronts as evenly as they go (at most 4
// each, U = tiles x the most any wavefront gets).
bool decode_group_major_ok(const DecodeArgs &a) {
    const int G = a.K / kGroupK;
    if (a.direct || a.regs || a.group_major == 0 || a.KS * a.GS != G || a.GS > 32 || a.GS < a.waves) return false;
    const int gpw = (a.GS + a.waves - 1) / a.waves, T = a.gm_tiles;
    return T >= 2 && T <= 6 && gpw <= 4 && a.U == T * gpw &&
           decode_gm_lds_bytes(a.GS, a.waves, T) <= (size_t)decode_max_lds_bytes();
}

#endif

#if KILN_DECODE_LORA
hipError_t launch_decode_lora(const DecodeArgs &a, hipStream_t stream) {
    if (a.r_total < 1) return hipErrorInvalidValue;
#else
hipError_t launch_decode_lora(const DecodeArgs &a, hipStream_t stream);  // the other compilation of this file
hipError_t launch_decode(const DecodeArgs &a, hipStream_t stream) {
    if (a.r_total > 0) return launch_decode_lora(a, stream);
#endif
    const int G = a.K / kGroupK, NT = a.N / kTileN;
    const int gs_last = G - (a.KS - 1) * a.GS;  // smallest slice
    const bool sane = a.waves >= 1 && a.waves <= kMaxWaves && a.M >= 1 && a.U >= 1 && a.GS >= 1 && a.KS >= 1;
    if (a.r_total < 0 || a.r_total > 64) return hipErrorInvalidValue;
    if (a.r_total > 0 && (!a.lora_t || !a.lora_b || a.lora_slices < 1 || a.lora_rows < a.M)) return hipErrorInvalidValue;
    if (a.rows > a.M && (!a.regs || a.M != 32 || a.rows > 128)) return hipErrorInvalidValue;  // up to four runs of 32 rows
    if (a.regs) {
        if (!sane || !decode_group_major_regs_ok(a)) return hipErrorInvalidValue;
        return a.M > 16 ? launch_gmr_s<2>(a, stream) : launch_gmr_s<1>(a, stream);
    }
    if (a.gm_tiles > 0) {
        if (!sane || a.M > 16 || !decode_group_major_ok(a)) return hipErrorInvalidValue;
        const int gpw = (a.GS + a.waves - 1) / a.waves;
        switch (a.gm_tiles) {
            case 2: return launch_gm_t<2>(a, gpw, stream);
            case 3: return launch_gm_t<3>(a, gpw, stream);
            case 4: return launch_gm_t<4>(a, gpw, stream);
            case 5: return launch_gm_t<5>(a, gpw, stream);
            case 6: return launch_gm_t<6>(a, gpw, stream);
        }
    }
    if (a.waves < 1 || a.waves > kMaxWaves || a.M < 1 || a.M > 16) return hipErrorInvalidValue;
    if (a.KS < 1 || a.GS < 1 || gs_last < 1 || gs_last > a.GS) return hipErrorInvalidValue;
    if (decode_lds_bytes(a.GS, a.waves, a.direct) > (size_t)decode_max_lds_bytes()) return hipErrorInvalidValue;
    if (!a.direct && a.GS > 32) return hipErrorInvalidValue;  // the staging loop covers 32 groups per row
    // a run must not cover more than two tiles, must fit the smallest slice, and a
    // block must not touch more tiles than its flag array holds
    if (a.U < 1 || a.U > gs_last || a.U > NT * gs_last) return hipErrorInvalidValue;
    if (a.waves * a.U < a.GS) return hipErrorInvalidValue;  // a tile may be cut by one block boundary only
    if ((a.waves * a.U) / gs_last + 2 > kMaxTouched) return hipErrorInvalidValue;
    if ((long)a.BPS * a.waves * a.U < (long)NT * a.GS) return hipErrorInvalidValue;
    switch (a.U) {
        case 1: return launch_u<1>(a, stream);
        case 2: return launch_u<2>(a, stream);
        case 3: return launch_u<3>(a, stream);
        case 4: return launch_u<4>(a, stream);
        case 5: return launch_u<5>(a, stream);
        case 6: return launch_u<6>(a, stream);
        case 7: return launch_u<7>(a, stream);
        case 8: return launch_u<8>(a, stream);
        case 9: return launch_u<9>(a, stream);
        case 10: return launch_u<10>(a, stream);
        case 11: return launch_u<11>(a, stream);
        case 12: return launch_u<12>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace kiln
