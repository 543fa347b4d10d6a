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
//   * K slices, where a plan still has them, meet tile by tile: the wavefront that summed a tile
//     stores its part, waits for its own stores, counts its arrival and, if it is the last,
//     adds the parts in slice order -- no block-wide barrier in the exchange.
#include "async_loads.h"
#include "launch.h"

namespace kiln {

namespace {

constexpr int kGmpMaxWaves = 16;
constexpr int kGmpSlotBytes = 16 * 256;  // one group of A: 16 rows x 128 bf16
#ifndef KILN_GMP_HEAD
#define KILN_GMP_HEAD 3
#endif
// Probe builds only (-DKILN_GMP_TIMELINE): wall-clock stamps (100 MHz) per wavefront.
#ifdef KILN_GMP_TIMELINE
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

// T tiles per block, GPW groups per wavefront (the first `full_waves` wavefronts; the others one
// fewer), AQ = LDS-direct loads per group of A: 4 (16 rows), 2 (M <= 8) or 1 (M <= 4: rows 0...3
// only; the other rows of the product are computed from whatever LDS holds and never stored).
template <int T, int GPW, int AQ>
__global__ __launch_bounds__(kGmpMaxWaves * 64) void w4a16_decode_gmp_kernel(
    const uint16_t *__restrict__ A, const u32x4 *__restrict__ B, const uint16_t *__restrict__ S,
    uint16_t *__restrict__ C, float *partial, int *counters, int M, int N, int K, int Gs, int KS, int GS,
    int full_waves, int slot_bytes, int swiglu, int flagged, int col_shift) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
#ifdef KILN_GMP_TIMELINE
    long long tl_[8] = {};
#endif
    KILN_GMP_TL(0, KILN_GMP_NOW());
    constexpr int NS = gmp_slots(GPW);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nw = blockDim.x >> 6;
    const int G = K / kGroupK;
    const int NT = N / kTileN;
    const int ks = blockIdx.y;
    // Blocks go to the eight dies round-robin by linear index.  With the counter-free exchange the
    // column block is shifted by col_shift per slice, so that the slices of a tile sit on different
    // dies: a device-scope store and the device-scope load that polls it are slow when they meet
    // in one die's L2 (measured: 2...3 us per poll instead of 0.5).
    const int col_block = (int)((blockIdx.x + ks * col_shift) % gridDim.x);
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
    if (full) run(std::integral_constant<int, GPW>{});
    else if constexpr (GPW > 1) run(std::integral_constant<int, GPW - 1>{});

    // every wavefront's partial tiles into its own piece of LDS, then tile ti = their sum in
    // wavefront (= ascending K) order, one tile per wavefront at a time
    KILN_GMP_TL(1, KILN_GMP_NOW());
    f32x4 *slots = reinterpret_cast<f32x4 *>(mine);
#pragma unroll
    for (int ti = 0; ti < T; ++ti) slots[ti * 64 + lane] = y[ti];
    __syncthreads();
    KILN_GMP_TL(2, KILN_GMP_NOW());

    const int q4 = lane >> 4, c = lane & 15;
    const int tiles = min(T, NT - tf);
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
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    __hip_atomic_store(own + i, ~__builtin_bit_cast(uint32_t, (float)sum[i]), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                continue;
            }
            // up to kGmpFlaggedSlices - 1 other parts, all polled at once.  Every part is loaded once per
            // poll: a second device-scope load of an address the wavefront has just loaded waits for
            // the first (measured: 0.5 us per repeat).
            uint32_t got[kGmpFlaggedSlices - 1][4] = {};
            const uint32_t *base = reinterpret_cast<const uint32_t *>(partial) + (size_t)tt * 256 + lane * 4;
            for (int spins = 0;; ++spins) {
                bool missing = false;
#pragma unroll
                for (int s2 = 0; s2 < kGmpFlaggedSlices - 1; ++s2) {
                    if (s2 < KS - 1) {
                        const uint32_t *src = base + (size_t)s2 * NT * 256;
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            got[s2][i] = __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
#pragma unroll
                for (int s2 = 0; s2 < kGmpFlaggedSlices - 1; ++s2)  // after all requests: one round trip per poll
#pragma unroll
                    for (int i = 0; i < 4; ++i) missing |= s2 < KS - 1 && got[s2][i] == 0;
                // the bound is never reached in a working launch; past it the words still missing read
                // as NaN in the result
                if (__builtin_amdgcn_ballot_w64(missing) == 0 || spins == kGmpSpinLimit) {
                    KILN_GMP_TL(5, (long long)spins + 1);
                    break;
                }
                __builtin_amdgcn_s_sleep(2);
            }
            KILN_GMP_TL(4, KILN_GMP_NOW());
            f32x4 total = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s2 = 0; s2 < kGmpFlaggedSlices - 1; ++s2) {
                if (s2 < KS - 1) {  // ascending K order, this slice's own part last
                    uint32_t *src = const_cast<uint32_t *>(base) + (size_t)s2 * NT * 256;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        total[i] += __builtin_bit_cast(float, ~got[s2][i]);
                        __hip_atomic_store(src + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // zero for the next launch
                    }
                }
            }
            sum = total + sum;
        } else if (KS > 1) {
            // the slices of the tile meet in the workspace: store this part with device-scope
            // accesses, wait until the stores are acknowledged, count the arrival; the last to arrive
            // adds all parts in ascending K order (so the result does not depend on arrival order)
            // and leaves the counter zero
            KILN_GMP_TL(3, KILN_GMP_NOW());
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
        store_tile_rows(C, N, M, 4 * q4, tt, c, sum, swiglu != 0);
    }
#ifdef KILN_GMP_TIMELINE
    tl_[6] = KILN_GMP_NOW();
    tl_[7] = 1ll + blockIdx.y;
    if (lane == 0 && g_gmp_tl) {
        long long *o = g_gmp_tl + (((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 16 + wave) * 8;
        for (int i = 0; i < 8; ++i) o[i] = tl_[i];
    }
#endif
}

int gmp_slot_bytes(int gpw, int tiles) {
    const int a = gmp_slots(gpw) * kGmpSlotBytes, r = tiles * 1024;
    return a > r ? a : r;
}

template <int T, int GPW, int AQ>
hipError_t launch_gmp_tga(const DecodeArgs &a, hipStream_t stream) {
    const hipError_t attr = allow_dynamic_lds<&w4a16_decode_gmp_kernel<T, GPW, AQ>>(decode_max_lds_bytes());
    if (attr != hipSuccess) return attr;
    const int NT = a.N / kTileN;
    const int full_waves = a.GS - a.waves * (GPW - 1);
    const int slot = gmp_slot_bytes(GPW, T);
    w4a16_decode_gmp_kernel<T, GPW, AQ><<<dim3((NT + T - 1) / T, a.KS), a.waves * 64, a.waves * slot, stream>>>(
        (const uint16_t *)a.A, (const u32x4 *)a.B, (const uint16_t *)a.S, (uint16_t *)a.C, a.partial, a.counters, a.M,
        a.N, a.K, a.Gs, a.KS, a.GS, full_waves, slot, a.swiglu ? 1 : 0, a.flagged ? 1 : 0,
        a.flagged ? exchange_column_shift((NT + T - 1) / T) : 0);
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

// The private-staging group-major instance: M <= 16 rows, 1...6 whole tiles per block in equal K
// slices of any length, wavefronts of ceil(GS / waves) groups (or one fewer) with at most 16
// chunks each; a.waves <= 16 and <= GS.
bool decode_gmp_ok(const DecodeArgs &a) {
    const int G = a.K / kGroupK;
    if (a.M < 1 || a.M > 16 || a.r_total > 0 || a.gm_tiles < 1 || a.gm_tiles > 6) return false;
    if (a.KS < 1 || a.GS < 1 || a.KS * a.GS != G || a.waves < 1 || a.waves > kGmpMaxWaves || a.waves > a.GS) return false;
    const int gpw = (a.GS + a.waves - 1) / a.waves, T = a.gm_tiles;
    if (gpw > (T <= 2 ? 6 : 3) || T * gpw > kGmpMaxChunks) return false;
    const int full_waves = a.GS - a.waves * (gpw - 1);
    if (full_waves < 1 || full_waves > a.waves) return false;
    return (size_t)a.waves * gmp_slot_bytes(gpw, T) <= (size_t)decode_max_lds_bytes();
}

hipError_t launch_decode_gmp(const DecodeArgs &a, hipStream_t stream) {
    if (!decode_gmp_ok(a)) return hipErrorInvalidValue;
    if (a.KS > 1 && (!a.partial || !a.counters)) return hipErrorInvalidValue;
    if (a.flagged && a.KS > kGmpFlaggedSlices) return hipErrorInvalidValue;
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

}  // namespace kiln

#ifdef KILN_GMP_TIMELINE
extern "C" int kiln_gmp_timeline(long long *buf) {
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(kiln::g_gmp_tl), &buf, sizeof(buf));
}
#endif
