// Host-side quantiser and layout conversion (pure CPU, no GPU state).
//
// kiln_w4a16_quantize_and_pack follows the arithmetic of the reference
// quantiser (crates/kiln-marlin-gemm/src/lib.rs:393-427) and writes the tile
// layout described in layout.h instead of the Marlin permutation
// (lib.rs:429-479).  kiln_w4a16_repack_gptq is the one-time offline repack
// from GPTQ-canonical tensors (crates/kiln-model/src/quantized.rs:127-152).
#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

#include "kiln_w4a16.h"
#include "layout.h"

namespace {

using namespace kiln;

inline uint32_t f32_bits(float f) { uint32_t b; std::memcpy(&b, &f, 4); return b; }
inline float bits_f32(uint32_t b) { float f; std::memcpy(&f, &b, 4); return f; }

// IEEE binary32 -> binary16, round to nearest even (half::f16::from_f32, lib.rs:411).
uint16_t f32_to_f16(float v) {
    const uint32_t x = f32_bits(v);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t ex = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (ex == 0xFF) {
        if (!man) return sign | 0x7C00u;
        uint16_t m = (uint16_t)(man >> 13);
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

float f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t ex = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    if (ex == 0) {
        if (!man) return bits_f32(sign);
        int sh = 0;
        while (!(man & 0x400u)) { man <<= 1; ++sh; }
        return bits_f32(sign | ((uint32_t)(113 - sh) << 23) | ((man & 0x3FFu) << 13));
    }
    if (ex == 31) return bits_f32(sign | 0x7F800000u | (man << 13));
    return bits_f32(sign | ((ex + 112) << 23) | (man << 13));
}

// Spread 8 nibbles (row j at bits 4j) to the in-word order of layout.h.
inline uint32_t shuffle_nibbles(uint32_t w) {
    uint32_t out = 0;
    for (int j = 0; j < 8; ++j) out |= ((w >> (4 * j)) & 0xFu) << (4 * nibble_pos(j));
    return out;
}
inline uint32_t unshuffle_nibbles(uint32_t w) {
    uint32_t out = 0;
    for (int j = 0; j < 8; ++j) out |= ((w >> (4 * nibble_pos(j))) & 0xFu) << (4 * j);
    return out;
}

template <typename F>
void parallel_for(int count, F &&body) {
    unsigned hw = std::thread::hardware_concurrency();
    int nthreads = (int)std::min<unsigned>(hw ? hw : 1, 16);
    nthreads = std::min(nthreads, count);
    if (nthreads <= 1) {
        for (int i = 0; i < count; ++i) body(i);
        return;
    }
    std::vector<std::thread> pool;
    pool.reserve(nthreads);
    for (int t = 0; t < nthreads; ++t)
        pool.emplace_back([=, &body]() {
            for (int i = t; i < count; i += nthreads) body(i);
        });
    for (auto &th : pool) th.join();
}

bool shape_ok(int k, int n, int groupsize) {
    return k > 0 && n > 0 && k % 128 == 0 && n % 256 == 0 && (groupsize == -1 || groupsize == 128);
}

}  // namespace

extern "C" {

int kiln_w4a16_layout_version(void) { return kLayoutVersion; }

const char *kiln_w4a16_status_string(kiln_marlin_status_t st) {
    switch (st) {
        case KILN_W4A16_OK: return "ok";
        case KILN_W4A16_ERR_PROB_SHAPE:
            return "unsupported problem shape (need k % 128 == 0, n % 256 == 0, groupsize -1 or 128)";
        case KILN_W4A16_ERR_KERN_SHAPE: return "no kernel for this configuration";
        case KILN_W4A16_ERR_LAUNCH: return "HIP launch error";
        case KILN_W4A16_ERR_ARGUMENT: return "null or inconsistent argument";
        case KILN_W4A16_ERR_ZERO_POINT: return "GPTQ zero-point other than 8 is not supported";
        case KILN_W4A16_ERR_SCRATCH:
            return "the call needs more scratch than the library's static device array holds; use the entry point "
                   "that takes a workspace";
        default: return "unknown status";
    }
}

kiln_marlin_status_t kiln_w4a16_quantize_and_pack(const float *weight, int k, int n,
                                                  int groupsize, int32_t *b_packed,
                                                  uint16_t *scales_f16, float *dequant) {
    if (!weight || !b_packed || !scales_f16) return KILN_W4A16_ERR_ARGUMENT;
    if (!shape_ok(k, n, groupsize)) return KILN_W4A16_ERR_PROB_SHAPE;
    const int G = k / kGroupK;
    const int Gs = (groupsize == -1) ? 1 : G;
    const int g_rows = (groupsize == -1) ? k : 128;
    uint32_t *out = reinterpret_cast<uint32_t *>(b_packed);

    parallel_for(n / kTileN, [&](int nt) {
        float s_f32[16];
        for (int gs = 0; gs < Gs; ++gs) {
            // lib.rs:394-412: s = f16(2 * max|w| / 15), max == 0 -> 1.0
            float max_abs[16];
            for (int c = 0; c < 16; ++c) max_abs[c] = 0.0f;
            for (int r = 0; r < g_rows; ++r) {
                const float *row = weight + (size_t)(gs * g_rows + r) * n + nt * 16;
                for (int c = 0; c < 16; ++c) max_abs[c] = std::max(max_abs[c], std::fabs(row[c]));
            }
            for (int c = 0; c < 16; ++c) {
                const float mx = (max_abs[c] == 0.0f) ? 1.0f : max_abs[c];
                const uint16_t h = f32_to_f16((2.0f * mx) / 15.0f);
                scales_f16[scale_index(gs, nt * 16 + c, Gs)] = h;
                s_f32[c] = f16_to_f32(h);
            }
            // lib.rs:416-427: code = clamp(round(w / s) + 8, 0, 15), ties away from zero
            for (int gi = 0; gi < g_rows / kGroupK; ++gi) {
                const int g = gs * (g_rows / kGroupK) + gi;
                uint32_t *chunk = out + ((size_t)nt * G + g) * kChunkWords;
                for (int t = 0; t < 4; ++t)
                    for (int kq = 0; kq < 4; ++kq) {
                        uint32_t words[16] = {0};
                        for (int j = 0; j < 8; ++j) {
                            const int kk = g * kGroupK + 32 * t + 8 * kq + j;
                            const float *row = weight + (size_t)kk * n + nt * 16;
                            float *drow = dequant ? dequant + (size_t)kk * n + nt * 16 : nullptr;
                            for (int c = 0; c < 16; ++c) {
                                const float q = std::round(row[c] / s_f32[c]);
                                long long raw;           // Rust `as i32`: saturating, NaN -> 0
                                if (q != q) raw = 0;
                                else if (q >= 2147483647.0f) raw = 2147483647LL;
                                else if (q <= -2147483648.0f) raw = -2147483648LL;
                                else raw = (long long)q;
                                // the reference adds the offset in i32 (lib.rs:423): from a saturated raw a
                                // release build wraps to a negative sum, which the clamp makes code 0
                                long long shifted = raw + 8;
                                if (shifted > 2147483647LL) shifted -= 4294967296LL;
                                const int code = (int)std::min<long long>(15, std::max<long long>(0, shifted));
                                words[c] |= (uint32_t)code << (4 * nibble_pos(j));
                                if (drow) drow[c] = (float)(code - 8) * s_f32[c];
                            }
                        }
                        for (int c = 0; c < 16; ++c) chunk[(c + 16 * kq) * 4 + t] = words[c];
                    }
            }
        }
    });
    return KILN_W4A16_OK;
}

kiln_marlin_status_t kiln_w4a16_repack_gptq(const int32_t *qweight, const uint16_t *scales,
                                            const int32_t *qzeros, int k, int n, int groupsize,
                                            int32_t *b_packed, uint16_t *scales_tiled) {
    if (!qweight || !scales || !b_packed || !scales_tiled) return KILN_W4A16_ERR_ARGUMENT;
    if (!shape_ok(k, n, groupsize)) return KILN_W4A16_ERR_PROB_SHAPE;
    const int G = k / kGroupK;
    const int Gs = (groupsize == -1) ? 1 : G;
    if (qzeros) {
        const size_t count = (size_t)Gs * (n / 8);
        for (size_t i = 0; i < count; ++i)
            if ((uint32_t)qzeros[i] != 0x88888888u) return KILN_W4A16_ERR_ZERO_POINT;
    }
    const uint32_t *qw = reinterpret_cast<const uint32_t *>(qweight);
    uint32_t *out = reinterpret_cast<uint32_t *>(b_packed);
    parallel_for(n / kTileN, [&](int nt) {
        for (int g = 0; g < G; ++g) {
            uint32_t *chunk = out + ((size_t)nt * G + g) * kChunkWords;
            for (int t = 0; t < 4; ++t)
                for (int kq = 0; kq < 4; ++kq) {
                    const uint32_t *src = qw + (size_t)((g * kGroupK + 32 * t + 8 * kq) / 8) * n + nt * 16;
                    for (int c = 0; c < 16; ++c)
                        chunk[(c + 16 * kq) * 4 + t] = shuffle_nibbles(src[c]);
                }
        }
        for (int gs = 0; gs < Gs; ++gs)
            for (int c = 0; c < 16; ++c)
                scales_tiled[scale_index(gs, nt * 16 + c, Gs)] = scales[(size_t)gs * n + nt * 16 + c];
    });
    return KILN_W4A16_OK;
}

kiln_marlin_status_t kiln_w4a16_unpack_to_gptq(const int32_t *b_packed, const uint16_t *scales_tiled,
                                               int k, int n, int groupsize, int32_t *qweight,
                                               uint16_t *scales) {
    if (!qweight || !scales || !b_packed || !scales_tiled) return KILN_W4A16_ERR_ARGUMENT;
    if (!shape_ok(k, n, groupsize)) return KILN_W4A16_ERR_PROB_SHAPE;
    const int G = k / kGroupK;
    const int Gs = (groupsize == -1) ? 1 : G;
    const uint32_t *in = reinterpret_cast<const uint32_t *>(b_packed);
    uint32_t *qw = reinterpret_cast<uint32_t *>(qweight);
    parallel_for(n / kTileN, [&](int nt) {
        for (int g = 0; g < G; ++g) {
            const uint32_t *chunk = in + ((size_t)nt * G + g) * kChunkWords;
            for (int t = 0; t < 4; ++t)
                for (int kq = 0; kq < 4; ++kq) {
                    uint32_t *dst = qw + (size_t)((g * kGroupK + 32 * t + 8 * kq) / 8) * n + nt * 16;
                    for (int c = 0; c < 16; ++c)
                        dst[c] = unshuffle_nibbles(chunk[(c + 16 * kq) * 4 + t]);
                }
        }
        for (int gs = 0; gs < Gs; ++gs)
            for (int c = 0; c < 16; ++c)
                scales[(size_t)gs * n + nt * 16 + c] = scales_tiled[scale_index(gs, nt * 16 + c, Gs)];
    });
    return KILN_W4A16_OK;
}

kiln_marlin_status_t kiln_w4a16_interleave_gate_up(const int32_t *gate_b, const uint16_t *gate_s,
                                                   const int32_t *up_b, const uint16_t *up_s, int k, int n_each,
                                                   int groupsize, int32_t *out_b, uint16_t *out_s) {
    if (!gate_b || !gate_s || !up_b || !up_s || !out_b || !out_s) return KILN_W4A16_ERR_ARGUMENT;
    // the fused width 2 * n_each must itself be a legal width
    if (n_each <= 0 || n_each % 128 != 0 || !shape_ok(k, 2 * n_each, groupsize)) return KILN_W4A16_ERR_PROB_SHAPE;
    const int G = k / kGroupK;
    const int Gs = (groupsize == -1) ? 1 : G;
    const size_t tile_words = (size_t)G * kChunkWords, tile_scales = (size_t)Gs * kTileN;
    // Output tile j = gate columns 8 j ... 8 j + 7, then up columns 8 j ... 8 j + 7: half of source
    // tile j / 2.  In a chunk, lane c + 16 kq owns four words, so the eight lanes of a half tile and
    // one kq are 128 contiguous bytes on both sides.
    parallel_for(n_each / 8, [&](int j) {
        const size_t src_tile = (size_t)j / 2;
        const int c0 = 8 * (j & 1);  // first source column inside its tile
        for (int half = 0; half < 2; ++half) {  // gate, then up
            const int32_t *src_b = (half ? up_b : gate_b) + src_tile * tile_words;
            const uint16_t *src_s = (half ? up_s : gate_s) + src_tile * tile_scales;
            int32_t *dst_b = out_b + (size_t)j * tile_words;
            uint16_t *dst_s = out_s + (size_t)j * tile_scales;
            for (int g = 0; g < G; ++g)
                for (int kq = 0; kq < 4; ++kq)
                    std::memcpy(dst_b + (size_t)g * kChunkWords + (size_t)(8 * half + 16 * kq) * 4,
                                src_b + (size_t)g * kChunkWords + (size_t)(c0 + 16 * kq) * 4, 8 * 4 * sizeof(int32_t));
            for (int gs = 0; gs < Gs; ++gs)
                std::memcpy(dst_s + (size_t)gs * kTileN + 8 * half, src_s + (size_t)gs * kTileN + c0, 8 * sizeof(uint16_t));
        }
    });
    return KILN_W4A16_OK;
}

}  // extern "C"
