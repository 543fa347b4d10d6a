// The low-rank term the small-M kernels add where they store a tile (gfx950 only).
#pragma once
#include "device_common.h"
#include "launch.h"

namespace kiln {

// Optional low-rank term of the result: y += T * B_cat^T, where T = bf16 [M, rp] is the scaled
// projection of the activations onto the stacked adapters (columns r_total ... rp - 1 zero, rp a
// multiple of 16) and B_cat = bf16 [N, r_total] (crates/kiln-model/src/lora_loader.rs:213-232,
// added unfused at forward.rs:2932-2939).  rp == 0: none.
struct LoraTail {
    const uint16_t *t;
    const uint16_t *b;
    int r_total;
    int rp;
    int slices;    // T = [slices][t_rows][rp]: K slices of the projection, each rounded on its own
    int t_rows;
};

// v = rows row0 + 4 (lane / 16) ... + 3 of column lane % 16 of tile tt, in the accumulator layout.
// rp <= 64: two steps of 32 rank columns at most.  Everything a chunk of eight slices needs is
// requested before the first product (one memory round trip instead of one per step: the operands
// come from L2 or beyond, 1...2 us away, and this sits at the very end of the launch).
[[maybe_unused]] __device__ __forceinline__ void lora_add(f32x4 &v, const LoraTail &lo, int row0, int M, int tt,
                                                          int lane) {
    const int kq = lane >> 4, c = lane & 15;
    int row = row0 + c;
    row = row < M ? row : M - 1;  // rows past M: any finite operand, the products are never stored
    const uint16_t *tp = lo.t + (size_t)row * lo.rp;
    const uint16_t *bp = lo.b + (size_t)(tt * kTileN + c) * lo.r_total;
    u32x4 tb[2];
#pragma unroll
    for (int js = 0; js < 2; ++js) {
        const int j8 = 32 * js + 8 * kq;  // this lane's 8 rank columns of step js
        tb[js] = u32x4{0u, 0u, 0u, 0u};
        if ((lo.r_total & 7) == 0) {
            if (j8 < lo.r_total) tb[js] = *reinterpret_cast<const u32x4 *>(bp + j8);
        } else {
            uint32_t e[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) e[i] = (j8 + i < lo.r_total) ? (uint32_t)bp[j8 + i] : 0u;
            tb[js] = u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
        }
    }
    for (int z0 = 0; z0 < lo.slices; z0 += 8) {  // eight slices requested at a time
        u32x4 ta[2][8];
#pragma unroll
        for (int js = 0; js < 2; ++js) {
            const int j8 = 32 * js + 8 * kq;
#pragma unroll
            for (int zi = 0; zi < 8; ++zi) {
                ta[js][zi] = u32x4{0u, 0u, 0u, 0u};
                if (j8 < lo.rp && z0 + zi < lo.slices)
                    ta[js][zi] = *reinterpret_cast<const u32x4 *>(tp + (size_t)(z0 + zi) * lo.t_rows * lo.rp + j8);
            }
        }
#pragma unroll
        for (int js = 0; js < 2; ++js)
#pragma unroll
            for (int zi = 0; zi < 8; ++zi)
                if (32 * js < lo.rp && z0 + zi < lo.slices)
                    v = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ta[js][zi]),
                                                                __builtin_bit_cast(bf16x8, tb[js]), v, 0, 0, 0);
    }
}

// The same term with its operands in LDS: T whole ([slices][t_rows][rp], t_rows = M) and the
// r_total-wide rows of B_cat of the block's columns (tile ti of the block starts at row 16 ti);
// r_total % 8 == 0.  v = rows 4 (lane / 16) ... + 3 of column lane % 16 of the tile.
__device__ __forceinline__ void lora_add_from_lds(f32x4 &v, const LoraTail &lo, const unsigned char *t_lds,
                                                  const unsigned char *b_lds, int ti, int M, int lane) {
    const int kq = lane >> 4, c = lane & 15;
    const int row = c < M ? c : M - 1;  // rows past M: any finite operand, the products are never stored
    for (int j0 = 0; j0 < lo.rp; j0 += 32) {
        const int j8 = j0 + 8 * kq;  // this lane's 8 rank columns
        u32x4 tb = {0u, 0u, 0u, 0u};
        if (j8 < lo.r_total) tb = *reinterpret_cast<const u32x4 *>(b_lds + ((ti * kTileN + c) * lo.r_total + j8) * 2);
        for (int z = 0; z < lo.slices; ++z) {
            u32x4 ta = {0u, 0u, 0u, 0u};
            if (j8 < lo.rp) ta = *reinterpret_cast<const u32x4 *>(t_lds + ((z * lo.t_rows + row) * lo.rp + j8) * 2);
            v = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ta), __builtin_bit_cast(bf16x8, tb), v, 0,
                                                        0, 0);
        }
    }
}

// The projection T computed inside the launch that adds it, by `producers` extra blocks at the
// front of the grid (one K slice each) while the other blocks stream their weights.  A producer
// writes its slice of T with device-scope stores, waits until they are acknowledged and raises
// its flag; the blocks that add the term look at the flags through one wavefront (while the
// others sum their tiles) and read T with ordinary loads once the flags are up (no cache on
// their die has seen those lines since the launch began).  The flag words and the reader counts
// live in workspace that is all zero between launches: every adding block counts itself after
// its look, and the last one to do so zeroes the words.  Hundreds of blocks looking at one
// address, or counting on one, are served one after the other (measured: 231 single polls of one
// 64-byte line, every flag already up, took up to 4 us, and as long again for their 231 atomic
// adds on one counter): the flags therefore exist kLoraFoldReplicas times, 4 KiB apart, block b
// looks at and counts on replica b % kLoraFoldReplicas, and whoever completes a replica's count
// counts once more on a top word.  producers == 0: T comes from a launch of its own.
struct LoraFold {
    const uint16_t *a_cat;   // bf16 [r_total, K]: the adapters' A matrices stacked along rows
    uint16_t *t;             // where the producers write T: [producers][t_rows][rp] bf16
    unsigned *flags;         // kLoraFoldReplicas x kLoraFoldReplicaWords words: per replica one flag per producer,
                             // then the replica's reader count; the top count behind that in replica 0
    int producers;           // K slices of the projection
    int steps_per_slice;     // 32-value steps of K per slice
    int consumers;           // blocks that add the term
    // exclusive end column of adapter i on the stacked rank axis (r_total past the last adapter) and its
    // scale (0 past the last); plain members, not arrays: an indexed kernel argument is copied to scratch memory
    int e0, e1, e2, e3;      // (four adapters at most: every member is a scalar register for the whole kernel)
    float s0, s1, s2, s3;
};
constexpr int kLoraFoldMaxProducers = 16;
constexpr int kLoraFoldMaxAdapters = 4;
constexpr int kLoraFoldStepsPerWave = 12;  // 32-value steps of K one producer wavefront takes, at most
constexpr int kLoraFoldReplicas = 16;
constexpr int kLoraFoldReplicaWords = 1024;                  // 4 KiB from one replica to the next
constexpr int kLoraFoldCountWord = kLoraFoldMaxProducers;    // a replica's reader count
constexpr int kLoraFoldTopWord = kLoraFoldMaxProducers + 1;  // in replica 0: completed replicas
constexpr size_t kLoraFoldFlagBytes = (size_t)kLoraFoldReplicas * kLoraFoldReplicaWords * sizeof(unsigned);
constexpr int kLoraFoldSpinLimit = 1 << 20;

// One producer block: slice `slice` of T = scale(j) * x * a_cat^T for up to 16 rows of x (bf16 [M, K]),
// rounded to bf16 (crates/kiln-model/src/lora_loader.rs:213-232, the first product, with the
// adapter scale folded in before the rounding).  Wavefront w takes rank tile w % JT and every
// Q-th step of the slice from w / JT on (JT = rp / 16 rank tiles, Q = nw / JT; nw >= JT); the Q
// parts of a tile meet in LDS (nw KiB) and are added in ascending order.  Every wavefront of the
// block must call this (two barriers inside).
__device__ __forceinline__ void lora_project_slice(const uint16_t *__restrict__ X, const LoraFold &fold,
                                                   const LoraTail &lo, int M, int K, int slice,
                                                   unsigned char *lds, int wave, int lane, int nw) {
    const int JT = lo.rp >> 4, Q = nw / JT;
    const int steps = K >> 5, s0 = slice * fold.steps_per_slice, s1 = min(steps, s0 + fold.steps_per_slice);
    const int r = lane & 15, kq = lane >> 4;
    const int jt = wave % JT, q = wave / JT;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    if (q < Q) {
        const int rank = jt * 16 + r;
        const uint16_t *xp = X + (size_t)min(r, M - 1) * K + kq * 8;
        const uint16_t *ap = fold.a_cat + (size_t)min(rank, lo.r_total - 1) * K + kq * 8;
        const bool live = rank < lo.r_total;  // padding columns of T are zero
        // four steps requested at a time (more in flight would raise the whole kernel's register count,
        // and with it the launch cost of calls without adapters: measured +0.45 us at 97 instead of 82)
        for (int i0 = 0; i0 < kLoraFoldStepsPerWave; i0 += 4) {
            u32x4 xa[4], aa[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int st = s0 + q + (i0 + i) * Q;
                xa[i] = aa[i] = u32x4{0u, 0u, 0u, 0u};
                if (st < s1) {
                    xa[i] = *reinterpret_cast<const u32x4 *>(xp + (size_t)st * 32);
                    if (live) aa[i] = *reinterpret_cast<const u32x4 *>(ap + (size_t)st * 32);
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[i]),
                                                              __builtin_bit_cast(bf16x8, aa[i]), acc, 0, 0, 0);
            if (s0 + q + (i0 + 4) * Q >= s1) break;
        }
    }
    f32x4 *parts = reinterpret_cast<f32x4 *>(lds);
    parts[wave * 64 + lane] = acc;
    __syncthreads();
    if (wave < JT) {  // rows 4 (lane / 16) ... + 3 of rank column 16 wave + lane % 16
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int q2 = 0; q2 < Q; ++q2) sum += parts[(wave + q2 * JT) * 64 + lane];
        const int j = wave * 16 + r;
        // the scale of the first adapter whose columns end behind j
        float sc = 0.f;
        sc = j < fold.e3 ? fold.s3 : sc;
        sc = j < fold.e2 ? fold.s2 : sc;
        sc = j < fold.e1 ? fold.s1 : sc;
        sc = j < fold.e0 ? fold.s0 : sc;
        uint16_t *tz = fold.t + (size_t)slice * lo.t_rows * lo.rp;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // two neighbouring columns per 32-bit device-scope store (even lanes)
            const uint32_t mine = f32_to_bf16_bits(sum[i] * sc);
            const uint32_t next = (uint32_t)__shfl_xor((int)mine, 1, 64);
            const int row = 4 * kq + i;
            if ((lane & 1) == 0 && row < M)
                __hip_atomic_store(reinterpret_cast<uint32_t *>(tz + (size_t)row * lo.rp + j), mine | (next << 16),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");  // this wavefront's part of T has reached memory
    __syncthreads();
    if (wave == 0 && lane < kLoraFoldReplicas)
        __hip_atomic_store(fold.flags + lane * kLoraFoldReplicaWords + slice, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// A block that adds the term (the `consumer`-th of them), one wavefront of it: wait until every
// producer has raised its flag.  The bound is never reached in a working launch.
__device__ __forceinline__ int lora_fold_wait(const LoraFold &fold, int consumer, int lane) {
    const unsigned *mine = fold.flags + (consumer % kLoraFoldReplicas) * kLoraFoldReplicaWords;
    int spins = 0;
    for (; spins < kLoraFoldSpinLimit; ++spins) {
        unsigned f = 1u;
        if (lane < fold.producers) f = __hip_atomic_load(mine + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (__builtin_amdgcn_ballot_w64(f == 0u) == 0) break;
        __builtin_amdgcn_s_sleep(4);
    }
    return spins;  // polls that came back without every flag
}

// The same wavefront, after its look: count this block on its replica; the block that completes a
// replica counts on the top word, and the one that completes that has seen every other block
// past its look at the flags and zeroes flags and counts for the next launch.
__device__ __forceinline__ void lora_fold_done(const LoraFold &fold, int consumer, int lane) {
    const int replica = consumer % kLoraFoldReplicas;
    const unsigned quota = (unsigned)(fold.consumers - replica + kLoraFoldReplicas - 1) / kLoraFoldReplicas;
    const unsigned replicas = (unsigned)min(fold.consumers, kLoraFoldReplicas);
    unsigned before = 0;
    if (lane == 0)
        before = __hip_atomic_fetch_add(fold.flags + replica * kLoraFoldReplicaWords + kLoraFoldCountWord, 1u,
                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    before = (unsigned)__builtin_amdgcn_readfirstlane((int)before);
    if (before != quota - 1u) return;
    if (lane == 0)
        before = __hip_atomic_fetch_add(fold.flags + kLoraFoldTopWord, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    before = (unsigned)__builtin_amdgcn_readfirstlane((int)before);
    if (before != replicas - 1u) return;
    if (lane <= kLoraFoldTopWord)
        for (int r = 0; r < kLoraFoldReplicas; ++r)
            __hip_atomic_store(fold.flags + r * kLoraFoldReplicaWords + lane, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

inline LoraTail lora_tail(const DecodeArgs &a) {
    LoraTail lo{};
    if (a.r_total > 0) {
        lo.t = (const uint16_t *)a.lora_t;
        lo.b = (const uint16_t *)a.lora_b;
        lo.r_total = a.r_total;
        lo.rp = (a.r_total + 15) / 16 * 16;
        lo.slices = a.lora_slices;
        lo.t_rows = a.lora_rows;
    }
    return lo;
}

}  // namespace kiln
