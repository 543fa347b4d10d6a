// The LoRA projection T = scale * x * A_cat^T as the work of one 256-thread block, shared by the kernel
// that runs it as a launch of its own and by the kernels that run it in their own launch's first blocks.
#pragma once
#include "device_common.h"

namespace kiln {

__device__ __forceinline__ u32x4 extension_operand(float sum) {
    const float c = -kCodeBias * sum;
    const uint32_t hi = __builtin_bit_cast(uint32_t, c) & 0xFFFF0000u;
    const float r1 = c - __builtin_bit_cast(float, hi);                     // exact
    const uint32_t mid = __builtin_bit_cast(uint32_t, r1) & 0xFFFF0000u;
    const float r2 = r1 - __builtin_bit_cast(float, mid);                   // exact, <= 8 significant bits
    const uint32_t lo = __builtin_bit_cast(uint32_t, r2) & 0xFFFF0000u;
    return u32x4{(hi >> 16) | hi, (mid >> 16) | mid, (lo >> 16) | lo, 0u};
}
// the sum of 8 bf16 values in a 128-bit unit, in the order both kernels below use
__device__ __forceinline__ float sum_bf16x8(u32x4 v) {
    const uint32_t wd[4] = {v.x, v.y, v.z, v.w};
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        sum += __builtin_bit_cast(float, wd[i] << 16);
        sum += __builtin_bit_cast(float, wd[i] & 0xFFFF0000u);
    }
    return sum;
}

// T[m][j] = bf16(scale(j) * sum_k x[m][k] * a_cat[j][k]) for the stacked LoRA A matrices (rows j
// of a_cat, adapter boundaries in `ends`); columns r_total..RP-1 of T are written as zero.
// Follows the first product of crates/kiln-model/src/lora_loader.rs:213-232 (hidden = x * A^T),
// with the adapter scale folded in before the rounding.
//
// The product is a few hundred MFLOP over a few MB: its time is memory round trips, so K is cut
// into gridDim.y slices that run side by side.  Without `partial` every slice is rounded to bf16
// on its own, T = [slices][M][RP], and whoever multiplies T with B_cat^T runs over the slices as
// if they were further rank columns (the small-M kernels: a few more loads and products where
// they store a tile cost less than a meeting of the blocks costs here).  With `partial` the
// slices of a row tile meet there as f32 tiles and the last block to arrive writes T whole (the
// matrix-core kernel, for which further rank columns would be real work).
//
// A block takes RB rows, all RP columns and one slice, 256 values of K at a time: the RB x 256
// piece of x and the RP x 256 piece of a_cat go to LDS through registers with fully coalesced
// 128-bit loads (a wavefront reads two 512-byte row pieces per instruction; fragment-shaped loads
// straight from memory would touch 16 rows per instruction and run at a quarter of the rate),
// rows padded by 16 bytes so that the fragment reads are free of bank conflicts; two pieces are
// in flight while a third is multiplied.  The 16 x 16 tiles of T are dealt round-robin to the four
// wavefronts.
struct LoraScales {
    int ends[8];     // exclusive end column of adapter i inside the stacked rank axis
    float scales[8];
    int count;
};

constexpr int kProjectPieceK = 256;                          // values of K per staged piece
constexpr int kProjectRowBytes = kProjectPieceK * 2 + 16;    // padded LDS row
constexpr int kProjectMaxRank = 64;

// A 128-bit store that is written through to memory (device scope).  A store of more than 64 bits
// reads the upper part of its data registers after it has issued; the compiler pads that for its
// own stores, not for one inside inline asm: hence the s_nop.
__device__ __forceinline__ void store_b128_through(void *ptr, u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(ptr), "v"(v) : "memory");
}

// The work of one block (256 threads): row tile `row_tile` (RB rows), K slice `slice` of `KZ`.
// `done` (optional): a word per row tile, raised when the tile's rows of T (and, with `aext`, of the
// extension operand) are in memory -- for a caller that computes the projection inside another
// kernel's launch instead of in front of it.  Both are then written through to memory: an ordinary
// store is complete when this die's cache has it, which a reader on another die does not see
// before the launch ends.
template <int RB>  // rows per block: 16 or 64
__device__ __forceinline__ void lora_project_block(unsigned char *lds, const uint16_t *__restrict__ X,
                                                   const uint16_t *__restrict__ a_cat, uint16_t *__restrict__ T, int M,
                                                   int K, int r_total, int RP, int steps_per_slice, const LoraScales &ls,
                                                   float *partial, int *counters, u32x4 *aext, int row_tile, int slice,
                                                   int KZ, unsigned *done, int done_copies = 1, int done_stride = 0) {
    constexpr int XL = RB * 32 / 256;                // 128-bit loads per thread and piece: x ...
    constexpr int AL = kProjectMaxRank * 32 / 256;   // ... and a_cat (rows from r_total on are not read)
    constexpr int IT = RB / 16;                      // tiles of T per wavefront, at most
    constexpr int ZMAX = RB == 16 ? 16 : 8;          // K slices that may meet in one T
    constexpr int kPieceSteps = kProjectPieceK / 32;
    unsigned char *x_lds = lds, *a_lds = lds + RB * kProjectRowBytes;
    float *sc_lds = reinterpret_cast<float *>(lds + (RB + kProjectMaxRank) * kProjectRowBytes);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = row_tile * RB;
    const int steps = K / 32;                        // steps of 32 values of K
    const int s0 = slice * steps_per_slice, s1 = min(steps, s0 + steps_per_slice);
    const int rows = min(RB, M - m0), row_tiles = (rows + 15) >> 4, JT = RP >> 4;
    // A block may have more than the 256 threads that work here (a kernel that runs this in its own
    // launch's first blocks): the others take part in the barriers only.
    const bool active = tid < 256;
    const int items = active ? row_tiles * JT : 0;

    if (tid < kProjectMaxRank) {
        float sc = 0.f;
        if (tid < r_total) {
            sc = ls.scales[ls.count - 1];
            for (int i = ls.count - 1; i >= 0; --i)
                if (tid < ls.ends[i]) sc = ls.scales[i];
        }
        sc_lds[tid] = sc;
    }

    // thread t holds 16-byte piece t % 32 of rows t / 32, t / 32 + 8, ...; two pieces in flight
    u32x4 xr[2][XL], ar[2][AL];
    const int pc = tid & 31, pr = tid >> 5;
    auto request = [&](auto buf, int c0) {  // the piece that starts at step c0
        constexpr int b = decltype(buf)::value;
        const bool k_ok = c0 + (pc >> 2) < s1;
        const size_t col = (size_t)c0 * 32 + pc * 8;
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int row = pr + 8 * i;
            xr[b][i] = u32x4{0u, 0u, 0u, 0u};
            if (active && k_ok && row < row_tiles * 16)
                xr[b][i] = *reinterpret_cast<const u32x4 *>(X + (size_t)min(m0 + row, M - 1) * K + col);
        }
#pragma unroll
        for (int i = 0; i < AL; ++i) {
            const int row = pr + 8 * i;
            ar[b][i] = u32x4{0u, 0u, 0u, 0u};
            if (active && k_ok && row < r_total) ar[b][i] = *reinterpret_cast<const u32x4 *>(a_cat + (size_t)row * K + col);
        }
    };

    f32x4 acc[IT];
#pragma unroll
    for (int it = 0; it < IT; ++it) acc[it] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int frag = (lane & 15) * kProjectRowBytes + (lane >> 4) * 16;
    auto multiply = [&](auto buf, int c0) {  // piece c0 from its registers through LDS into the products
        constexpr int b = decltype(buf)::value;
        if (c0 != s0) __syncthreads();  // the previous piece has been multiplied
        if (active) {
#pragma unroll
            for (int i = 0; i < XL; ++i)
                *reinterpret_cast<u32x4 *>(x_lds + (pr + 8 * i) * kProjectRowBytes + pc * 16) = xr[b][i];
#pragma unroll
            for (int i = 0; i < AL; ++i)
                if (pr + 8 * i < RP)
                    *reinterpret_cast<u32x4 *>(a_lds + (pr + 8 * i) * kProjectRowBytes + pc * 16) = ar[b][i];
        }
        __syncthreads();
        if (c0 + 2 * kPieceSteps < s1) request(buf, c0 + 2 * kPieceSteps);
        if (aext && active) {
            // The matrix-core kernel's extension operand (see w4a16_prefill_rowsum_kernel, whose launch
            // this saves): the staged piece of x holds two whole groups of every row of the block --
            // slices are whole groups, so each (row, group) is formed exactly once.  16 lanes per item,
            // same order of additions as the kernel above.
            const int sub = tid & 15;
#pragma unroll
            for (int base = 0; base < RB * 2; base += 16) {
                const int it2 = base + (tid >> 4), row = it2 >> 1, half = it2 & 1;
                float sum = sum_bf16x8(*reinterpret_cast<const u32x4 *>(x_lds + row * kProjectRowBytes + half * 256 + sub * 16));
#pragma unroll
                for (int off = 8; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, 16);
                if (sub == 0 && m0 + row < M && c0 + 4 * half < s1) {
                    u32x4 *dst = aext + (size_t)(c0 / 4 + half) * M + m0 + row;
                    if (done) store_b128_through(dst, extension_operand(sum));
                    else *dst = extension_operand(sum);
                }
            }
        }
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int item = wave + 4 * it;
            if (item < items) {
                const int rt = item / JT, jt = item - rt * JT;
                const unsigned char *xp = x_lds + rt * 16 * kProjectRowBytes + frag;
                const unsigned char *ap = a_lds + jt * 16 * kProjectRowBytes + frag;
#pragma unroll
                for (int st = 0; st < kPieceSteps; ++st)
                    acc[it] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8 *>(xp + 64 * st),
                                                                       *reinterpret_cast<const bf16x8 *>(ap + 64 * st),
                                                                       acc[it], 0, 0, 0);
            }
        }
    };
    using buf0 = std::integral_constant<int, 0>;
    using buf1 = std::integral_constant<int, 1>;
    request(buf0{}, s0);
    if (s0 + kPieceSteps < s1) request(buf1{}, s0 + kPieceSteps);
    for (int c0 = s0; c0 < s1; c0 += 2 * kPieceSteps) {
        multiply(buf0{}, c0);
        if (c0 + kPieceSteps < s1) multiply(buf1{}, c0 + kPieceSteps);
    }
    __syncthreads();  // sc_lds (a slice may be empty: then no barrier above)

    uint16_t *Tz = T + (size_t)slice * M * RP;
    if (partial && KZ > 1) {
        // One T for all of K: the slices of a row tile meet in `partial` as f32 tiles (device-scope
        // accesses); the last block to arrive adds them in slice order, so the result does not
        // depend on arrival order, and leaves the counter at zero.
        __shared__ int s_last;
        float *tile0 = partial + (size_t)row_tile * KZ * (IT * 4) * 256 + lane;  // [slice][item][4][64]
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int item = wave + 4 * it;
            if (item < items)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    __hip_atomic_store(tile0 + ((size_t)(slice * (IT * 4) + item) * 4 + i) * 64, acc[it][i],
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // each wavefront waits until its own stores have been acknowledged (a barrier alone
        // orders nothing outside the workgroup); after the barrier the arrival is counted
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();
        if (tid == 0)
            s_last = __hip_atomic_fetch_add(counters + row_tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == KZ - 1;
        __syncthreads();
        if (!s_last) return;
        // every read is requested before the first is used: device-scope reads are slow, and this
        // round trip is hidden by nothing else
        f32x4 part[IT][ZMAX];
#pragma unroll
        for (int it = 0; it < IT; ++it)
#pragma unroll
            for (int z = 0; z < ZMAX; ++z)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    part[it][z][i] = (wave + 4 * it < items && z < KZ)
                                         ? __hip_atomic_load(tile0 + ((size_t)(z * (IT * 4) + wave + 4 * it) * 4 + i) * 64,
                                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                         : 0.f;
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            acc[it] = part[it][0];
#pragma unroll
            for (int z = 1; z < ZMAX; ++z) acc[it] += part[it][z];
        }
        if (tid == 0) __hip_atomic_store(counters + row_tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        Tz = T;
    }
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int item = wave + 4 * it;
        if (item >= items) continue;
        const int rt = item / JT, jt = item - rt * JT;
        const int j = jt * 16 + (lane & 15);
        const float sc = sc_lds[j];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = m0 + rt * 16 + 4 * (lane >> 4) + i;
            const uint32_t mine = f32_to_bf16_bits(acc[it][i] * sc);
            if (done) {  // two neighbouring columns per 32-bit device-scope store (even lanes)
                const uint32_t next = (uint32_t)__shfl_xor((int)mine, 1, 64);
                if ((lane & 1) == 0 && r < M)
                    __hip_atomic_store(reinterpret_cast<uint32_t *>(Tz + (size_t)r * RP + j), mine | (next << 16),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else if (r < M) {
                Tz[(size_t)r * RP + j] = (uint16_t)mine;
            }
        }
    }
    if (done) {
        // whoever gets here wrote the tile's rows of T, after every slice's stores (its own included)
        // had been acknowledged: the extension operand of all slices is in memory too
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();
        // (done_copies copies of the word, done_stride words apart, for readers too many for one address)
        if (tid < done_copies)
            __hip_atomic_store(done + (size_t)tid * done_stride + row_tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

}  // namespace kiln
