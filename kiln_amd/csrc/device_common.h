// Device-side helpers shared by the W4A16 kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "launch.h"
#include "layout.h"

namespace kiln {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// bf16 bit pattern 0x4300 | code is exactly 128 + code (bf16 has ulp 1 in
// [128, 256)), so a packed pair of codes becomes a packed pair of bf16 values
// with one and-or.  The kernels multiply with (136 + d), d = code - 8, and
// remove the 136 * sum(x) term separately; see kCodeBias.
constexpr uint32_t kNibbleMask = 0x000F000Fu;
constexpr uint32_t kBf16Magic = 0x43004300u;
constexpr float kCodeBias = 136.0f;  // 128 (magic) + 8 (zero-point)

// The two constants of the code -> bf16 expansion, held in registers the
// compiler cannot see through.  With literal constants it emits an AND and an
// OR per register pair (a VOP3 instruction on this target cannot carry two
// literals); with one scalar and one vector register operand it selects
// v_and_or_b32.  The asm statements only define constants: no loaded data
// passes through inline asm.
struct DequantConsts {
    uint32_t mask;   // scalar register
    uint32_t magic;  // vector register
};

__device__ __forceinline__ DequantConsts dequant_consts() {
    DequantConsts c;
    asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(c.mask));
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(c.magic));
    return c;
}

// One packed word (8 codes, nibble order of layout.h) -> the 8 bf16 values
// 128 + code, in row order j = 0..7: the B operand of one MFMA k-step.
__device__ __forceinline__ bf16x8 codes_to_bf16x8(uint32_t w, const DequantConsts &c) {
    u32x4 r;
    r.x = (w & c.mask) | c.magic;
    r.y = ((w >> 4) & c.mask) | c.magic;
    r.z = ((w >> 8) & c.mask) | c.magic;
    r.w = ((w >> 12) & c.mask) | c.magic;
    return __builtin_bit_cast(bf16x8, r);
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}

// f32 -> bf16 bits, round to nearest even.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float v) {
    return __builtin_bit_cast(uint16_t, (__bf16)v);
}

__device__ __forceinline__ bf16x8 bf16x8_splat_one() {
    u32x4 r = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    return __builtin_bit_cast(bf16x8, r);
}

// all eight lanes of the operand = the bf16 pair given as one 32-bit pattern
__device__ __forceinline__ bf16x8 bf16x8_splat(uint32_t pair) {
    u32x4 r = {pair, pair, pair, pair};
    return __builtin_bit_cast(bf16x8, r);
}

// Store four rows (row0 ... row0 + 3, those below M) of column c of 16-column tile tt from a lane
// of the 16x16 accumulator layout (lane = c + 16 q holds rows 4 q ... 4 q + 3 of column c).
// swiglu: the tile holds 8 gate columns, then the 8 matching up columns (the packing of
// kiln_w4a16_interleave_gate_up); the lane of gate column c takes up from lane c + 8 of its
// 16-lane row and stores silu(gate) * up = gate / (1 + exp(-gate)) * up into a result half as wide
// (crates/kiln-model/src/forward.rs:2789-2819 forms it from bf16 tensors; here from the f32 sums,
// rounded once).  Every lane of the wavefront must be active.
__device__ __forceinline__ void store_tile_rows(uint16_t *__restrict__ C, int N, int M, int row0, int tt, int c,
                                                f32x4 v, bool swiglu) {
    if (!swiglu) {
        uint16_t *dst = C + (size_t)row0 * N + tt * kTileN + c;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (row0 + i < M) dst[(size_t)i * N] = f32_to_bf16_bits(v[i]);
        return;
    }
    const int n_out = N >> 1;
    f32x4 up;
#pragma unroll
    for (int i = 0; i < 4; ++i) {  // row_ror:8 inside each row of 16 lanes
        const float vi = v[i];  // a scalar copy: bit-casting the vector element in place reads element 0
            up[i] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, vi), 0x128, 0xF, 0xF, true));
        // the exchange must run while all lanes are active: keep it from being folded into the
        // arithmetic below, which runs for the gate lanes only (a disabled source lane reads as zero)
        asm volatile("" : "+v"(up[i]));
    }
    if ((c & 8) == 0) {
        uint16_t *dst = C + (size_t)row0 * n_out + tt * (kTileN / 2) + c;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (row0 + i < M) {
                const float gate = v[i];
                dst[(size_t)i * n_out] = f32_to_bf16_bits(gate * __builtin_amdgcn_rcpf(1.f + __expf(-gate)) * up[i]);
            }
    }
}

// A bounded wait ran out: leave a mark the host can find (launch.h describes the word).  `exchange_region`
// is the start of the region in which K slices meet without counters, `fold_words` the LoRA fold's flags;
// both sit at fixed distances from the sticky word.  One lane; the wavefront goes on with what it has.
__device__ __forceinline__ void report_wait_gave_up(unsigned *error_word, unsigned which, int lane) {
    if (lane == 0) __hip_atomic_fetch_or(error_word, which, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned *error_word_before_exchange_region(const void *exchange_region) {
    return reinterpret_cast<unsigned *>(reinterpret_cast<uintptr_t>(exchange_region) - (kWsCounterBytes - kWsErrorOffset));
}
__device__ __forceinline__ unsigned *error_word_before_fold_words(const unsigned *fold_words) {
    return reinterpret_cast<unsigned *>(reinterpret_cast<uintptr_t>(fold_words) - (kWsFoldFlagOffset - kWsErrorOffset));
}

__device__ __forceinline__ bf16x8 bf16x8_zero() {
    u32x4 r = {0u, 0u, 0u, 0u};
    return __builtin_bit_cast(bf16x8, r);
}

}  // namespace kiln
