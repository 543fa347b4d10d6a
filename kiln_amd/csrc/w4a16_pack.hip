// Quantise-and-pack on the device: bf16 weights [k, n] in device memory -> the tile layout of
// layout.h and its fp16 scales, without leaving the GPU.
//
// The arithmetic is the reference quantiser's (crates/kiln-marlin-gemm/src/lib.rs:393-427), as
// pack_host.cpp states it on the host, and the results are the same bits: per scale group and
// column s = f16(2 * max|w| / 15) (max == 0 -> 1.0), code = clamp(round(w / f32(s)) + 8, 0, 15) with
// ties away from zero and Rust's saturating float-to-int cast.  The reference has no device-side
// counterpart: marlin_proj.rs:86-181 downloads every weight, quantises on the host (17-58 s per
// model load for its 104 projections, ARCHITECTURE.md:570) and uploads the result.  Both kernels
// are bound by memory traffic that is small next to a single GEMM's (read the weight twice, write
// an eighth of it), so they are written for exactness and simple indexing, not tuned.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kiln_w4a16.h"
#include "device_common.h"
#include "layout.h"

namespace kiln {
namespace {

// IEEE binary32 -> binary16, round to nearest even, in integer arithmetic (the host quantiser's
// f32_to_f16, half::f16::from_f32 at lib.rs:411): independent of the device's rounding and
// denormal modes.
__device__ uint16_t pack_f32_to_f16(float v) {
    const uint32_t x = __builtin_bit_cast(uint32_t, v);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t ex = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (ex == 0xFF) {
        if (!man) return sign | 0x7C00u;
        const uint16_t m = (uint16_t)(man >> 13);
        return sign | 0x7C00u | m | (m ? 0 : 0x0200u);
    }
    const int e = (int)ex - 112;
    if (e >= 31) return sign | 0x7C00u;
    if (e <= 0) {
        if (e < -10) return sign;
        man |= 0x800000u;
        const int shift = 14 - e;
        uint32_t h = man >> shift;
        const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1u))) ++h;
        return sign | (uint16_t)h;
    }
    uint32_t out = ((uint32_t)e << 10) | (man >> 13);
    const uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (out & 1u))) ++out;
    return sign | (uint16_t)out;
}

__device__ float pack_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t ex = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    if (ex == 0) {
        if (!man) return __builtin_bit_cast(float, sign);
        int sh = 0;
        while (!(man & 0x400u)) {
            man <<= 1;
            ++sh;
        }
        return __builtin_bit_cast(float, sign | ((uint32_t)(113 - sh) << 23) | ((man & 0x3FFu) << 13));
    }
    if (ex == 31) return __builtin_bit_cast(float, sign | 0x7F800000u | (man << 13));
    return __builtin_bit_cast(float, sign | ((ex + 112) << 23) | (man << 13));
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }

// max of |w| as the host forms it: std::max(acc, fabs(w)) starting from 0 keeps acc when w is NaN
__device__ __forceinline__ float max_abs_step(float acc, float w) {
    const float a = __builtin_fabsf(w);
    return acc < a ? a : acc;
}

// Scales: block = 256 threads = 64 columns x 4 row lanes; grid (n / 64, scale groups).
// lib.rs:394-412.
__global__ __launch_bounds__(256) void w4a16_pack_scales_kernel(const uint16_t *__restrict__ w, int n, int g_rows,
                                                                int Gs, uint16_t *__restrict__ scales) {
    __shared__ float part[4][64];
    const int c = threadIdx.x & 63, rl = threadIdx.x >> 6;
    const int col = blockIdx.x * 64 + c, gs = blockIdx.y;
    const uint16_t *src = w + (size_t)gs * g_rows * n + col;
    float mx = 0.f;
    for (int r = rl; r < g_rows; r += 4) mx = max_abs_step(mx, bf16_bits_to_f32(src[(size_t)r * n]));
    part[rl][c] = mx;
    __syncthreads();
    if (rl != 0) return;
    // rows in ascending order of their row lane: max is exact, so the order only matters for NaN,
    // which max_abs_step never keeps
    for (int i = 1; i < 4; ++i) mx = max_abs_step(mx, part[i][c]);
    if (mx == 0.f) mx = 1.f;
    scales[scale_index(gs, col, Gs)] = pack_f32_to_f16(__fdiv_rn(2.0f * mx, 15.0f));
}

// Codes: one wavefront per chunk (column tile nt, group g); lane = c + 16 kq writes its four words
// (t = 0...3: rows 128 g + 32 t + 8 kq + j, j = 0...7, row j in nibble nibble_pos(j)) as one 16-byte store.
// Block = 4 wavefronts = 4 neighbouring column tiles of one group.  lib.rs:416-427.
__global__ __launch_bounds__(256) void w4a16_pack_codes_kernel(const uint16_t *__restrict__ w, int n, int G, int Gs,
                                                               const uint16_t *__restrict__ scales,
                                                               u32x4 *__restrict__ b_packed) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nt = blockIdx.x * 4 + wave, g = blockIdx.y;
    const int c = lane & 15, kq = lane >> 4;
    const int col = nt * kTileN + c;
    const int gs = Gs == 1 ? 0 : g;
    const float s = pack_f16_to_f32(scales[scale_index(gs, col, Gs)]);
    uint32_t words[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int row = g * kGroupK + 32 * t + 8 * kq + j;
            const float q = roundf(__fdiv_rn(bf16_bits_to_f32(w[(size_t)row * n + col]), s));
            long long raw;  // Rust `as i32`: saturating, NaN -> 0
            if (q != q) raw = 0;
            else if (q >= 2147483647.0f) raw = 2147483647LL;
            else if (q <= -2147483648.0f) raw = -2147483648LL;
            else raw = (long long)q;
            long long code = raw + 8;  // an i32 sum in the reference (lib.rs:423): wraps from a saturated raw
            if (code > 2147483647LL) code -= 4294967296LL;
            code = code < 0 ? 0 : (code > 15 ? 15 : code);
            word |= (uint32_t)code << (4 * nibble_pos(j));
        }
        words[t] = word;
    }
    b_packed[((size_t)nt * G + g) * (kChunkWords / 4) + lane] = u32x4{words[0], words[1], words[2], words[3]};
}

// Gate and up of equal shape into the pack the fused SwiGLU entry point reads (output tile j = gate
// columns 8 j ... 8 j + 7, then the same up columns: kiln_w4a16_interleave_gate_up on the host).  One
// wavefront per output chunk: lane c + 16 kq copies the 16 bytes of its source lane.
__global__ __launch_bounds__(256) void w4a16_interleave_kernel(const u32x4 *__restrict__ gate_b,
                                                               const uint16_t *__restrict__ gate_s,
                                                               const u32x4 *__restrict__ up_b,
                                                               const uint16_t *__restrict__ up_s, int G, int Gs,
                                                               u32x4 *__restrict__ out_b, uint16_t *__restrict__ out_s) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = blockIdx.x * 4 + wave, g = blockIdx.y;
    const int c = lane & 15, kq = lane >> 4;
    const int src_tile = j >> 1, src_c = 8 * (j & 1) + (c & 7);
    const bool up = (c & 8) != 0;
    const u32x4 *src_b = up ? up_b : gate_b;
    out_b[((size_t)j * G + g) * (kChunkWords / 4) + lane] = src_b[((size_t)src_tile * G + g) * (kChunkWords / 4) + src_c + 16 * kq];
    if (g < Gs && kq == 0) {
        const uint16_t *src_s = up ? up_s : gate_s;
        out_s[((size_t)j * Gs + g) * kTileN + c] = src_s[((size_t)src_tile * Gs + g) * kTileN + src_c];
    }
}

// GPTQ-canonical tensors (qweight [k/8, n] int32 with row j of eight in bits 4 j, scales [k/g, n] fp16;
// crates/kiln-model/src/quantized.rs:1-14, :127-152) into the tile layout: kiln_w4a16_repack_gptq on the
// host.  One wavefront per chunk; lane c + 16 kq gathers its four source words and moves each nibble to
// its place in the layout's word.  No re-quantisation: the codes are the checkpoint's.
__device__ __forceinline__ uint32_t pack_shuffle_nibbles(uint32_t w) {
    uint32_t out = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) out |= ((w >> (4 * j)) & 0xFu) << (4 * nibble_pos(j));
    return out;
}

__global__ __launch_bounds__(256) void w4a16_repack_gptq_kernel(const uint32_t *__restrict__ qweight,
                                                                const uint16_t *__restrict__ scales, int n, int G, int Gs,
                                                                u32x4 *__restrict__ b_packed,
                                                                uint16_t *__restrict__ scales_tiled) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nt = blockIdx.x * 4 + wave, g = blockIdx.y;
    const int c = lane & 15, kq = lane >> 4;
    const int col = nt * kTileN + c;
    uint32_t words[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
        words[t] = pack_shuffle_nibbles(qweight[(size_t)((g * kGroupK + 32 * t + 8 * kq) / 8) * n + col]);
    b_packed[((size_t)nt * G + g) * (kChunkWords / 4) + lane] = u32x4{words[0], words[1], words[2], words[3]};
    if (g < Gs && kq == 0) scales_tiled[scale_index(g, col, Gs)] = scales[(size_t)g * n + col];
}

// 1 in *bad if any packed zero-point word differs from 0x88888888 (zero-point 8 in all eight nibbles)
__global__ void w4a16_check_qzeros_kernel(const uint32_t *__restrict__ qzeros, size_t count, int *bad) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
        if (qzeros[i] != 0x88888888u) *bad = 1;
}
__global__ void w4a16_clear_flag_kernel(int *flag) { *flag = 0; }

}  // namespace
}  // namespace kiln

extern "C" kiln_marlin_status_t kiln_w4a16_repack_gptq_device(const void *qweight, const void *scales, const void *qzeros,
                                                              int k, int n, int groupsize, void *b_packed,
                                                              void *scales_tiled, int dev, void *stream) {
    using namespace kiln;
    (void)dev;
    if (!qweight || !scales || !b_packed || !scales_tiled) return KILN_W4A16_ERR_ARGUMENT;
    if (k <= 0 || n <= 0 || k % 128 != 0 || n % 256 != 0 || !(groupsize == -1 || groupsize == 128))
        return KILN_W4A16_ERR_PROB_SHAPE;
    const int G = k / kGroupK, Gs = groupsize == -1 ? 1 : G;
    if (G > 65535) return KILN_W4A16_ERR_PROB_SHAPE;  // grid y
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (qzeros) {
        // the zero-points must all be 8, as on the host route; the answer is needed before anything is written, so
        // this one check waits for the stream.  The flag lives at the start of the output and is overwritten below.
        int *flag = reinterpret_cast<int *>(b_packed);
        int bad = 0;
        w4a16_clear_flag_kernel<<<1, 1, 0, st>>>(flag);
        w4a16_check_qzeros_kernel<<<64, 256, 0, st>>>((const uint32_t *)qzeros, (size_t)Gs * (n / 8), flag);
        if (hipGetLastError() != hipSuccess ||
            hipMemcpyAsync(&bad, flag, sizeof(int), hipMemcpyDeviceToHost, st) != hipSuccess ||
            hipStreamSynchronize(st) != hipSuccess)
            return KILN_W4A16_ERR_LAUNCH;
        if (bad) return KILN_W4A16_ERR_ZERO_POINT;
    }
    w4a16_repack_gptq_kernel<<<dim3(n / 64, G), 256, 0, st>>>((const uint32_t *)qweight, (const uint16_t *)scales, n, G, Gs,
                                                               (u32x4 *)b_packed, (uint16_t *)scales_tiled);
    return hipGetLastError() == hipSuccess ? KILN_W4A16_OK : KILN_W4A16_ERR_LAUNCH;
}

extern "C" kiln_marlin_status_t kiln_w4a16_interleave_gate_up_device(const void *gate_b, const void *gate_s,
                                                                     const void *up_b, const void *up_s, int k,
                                                                     int n_each, int groupsize, void *out_b,
                                                                     void *out_s, int dev, void *stream) {
    using namespace kiln;
    (void)dev;
    if (!gate_b || !gate_s || !up_b || !up_s || !out_b || !out_s) return KILN_W4A16_ERR_ARGUMENT;
    if (k <= 0 || k % 128 != 0 || n_each <= 0 || n_each % 128 != 0 || !(groupsize == -1 || groupsize == 128))
        return KILN_W4A16_ERR_PROB_SHAPE;
    const int G = k / kGroupK, Gs = groupsize == -1 ? 1 : G;
    if (G > 65535) return KILN_W4A16_ERR_PROB_SHAPE;  // grid y
    w4a16_interleave_kernel<<<dim3(n_each / 8 / 4, G), 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        (const u32x4 *)gate_b, (const uint16_t *)gate_s, (const u32x4 *)up_b, (const uint16_t *)up_s, G, Gs,
        (u32x4 *)out_b, (uint16_t *)out_s);
    return hipGetLastError() == hipSuccess ? KILN_W4A16_OK : KILN_W4A16_ERR_LAUNCH;
}

extern "C" kiln_marlin_status_t kiln_w4a16_quantize_and_pack_device(const void *weight_bf16, int k, int n, int groupsize,
                                                                    void *b_packed, void *scales_f16, int dev,
                                                                    void *stream) {
    using namespace kiln;
    (void)dev;
    if (k <= 0 || n <= 0 || k % 128 != 0 || n % 256 != 0 || !(groupsize == -1 || groupsize == 128))
        return KILN_W4A16_ERR_PROB_SHAPE;
    if (!weight_bf16 || !b_packed || !scales_f16) return KILN_W4A16_ERR_ARGUMENT;
    const int G = k / kGroupK, Gs = groupsize == -1 ? 1 : G, g_rows = groupsize == -1 ? k : kGroupK;
    if (Gs > 65535 || G > 65535) return KILN_W4A16_ERR_PROB_SHAPE;  // grid y
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    w4a16_pack_scales_kernel<<<dim3(n / 64, Gs), 256, 0, st>>>((const uint16_t *)weight_bf16, n, g_rows, Gs,
                                                                (uint16_t *)scales_f16);
    if (hipGetLastError() != hipSuccess) return KILN_W4A16_ERR_LAUNCH;
    w4a16_pack_codes_kernel<<<dim3(n / 64, G), 256, 0, st>>>((const uint16_t *)weight_bf16, n, G, Gs,
                                                              (const uint16_t *)scales_f16, (u32x4 *)b_packed);
    return hipGetLastError() == hipSuccess ? KILN_W4A16_OK : KILN_W4A16_ERR_LAUNCH;
}
