/*
 * CPU oracle for the W4A16 GEMM path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 * See w4a16_oracle.h for what each function restates and what pins it.
 * Built by oracle/Makefile with gcc; OpenMP is used for the matmul loops only.
 */
#include "w4a16_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------ */
/* scalar conversions                                                        */
/* ------------------------------------------------------------------------ */

static inline float bits_to_f32(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}

static inline uint32_t f32_to_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

/* quantized.rs:223-252 -- sign / exponent / fraction split, subnormals are
 * normalised by shifting until the hidden bit appears. */
float ko_f16_to_f32(uint16_t bits) {
    uint32_t sign = (bits >> 15) & 1u;
    uint32_t exp = (bits >> 10) & 0x1Fu;
    uint32_t frac = bits & 0x3FFu;
    if (exp == 0) {
        if (frac == 0) return bits_to_f32(sign << 31);
        uint32_t e = 0;
        while ((frac & 0x400u) == 0) {
            frac <<= 1;
            e += 1;
        }
        frac &= 0x3FFu;
        uint32_t exp32 = 127 - 15 + 1 - e;
        return bits_to_f32((sign << 31) | (exp32 << 23) | (frac << 13));
    }
    if (exp == 31) return bits_to_f32((sign << 31) | (0xFFu << 23) | (frac << 13));
    return bits_to_f32((sign << 31) | ((exp + 127 - 15) << 23) | (frac << 13));
}

/* IEEE binary32 -> binary16, round to nearest even (what half::f16::from_f32
 * computes, lib.rs:411). */
uint16_t ko_f32_to_f16(float v) {
    uint32_t x = f32_to_bits(v);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (exp == 0xFF) { /* inf / nan */
        if (man == 0) return (uint16_t)(sign | 0x7C00u);
        uint16_t m = (uint16_t)(man >> 13);
        return (uint16_t)(sign | 0x7C00u | m | (m == 0 ? 0x0200u : 0u));
    }
    int e = (int)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u); /* overflow -> inf */
    if (e <= 0) {
        if (e < -10) return sign; /* below half the smallest subnormal */
        man |= 0x800000u;
        int shift = 14 - e; /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man += 1;
        return (uint16_t)(sign | half_man);
    }
    uint32_t out = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (out & 1u))) out += 1; /* may carry into exp */
    return (uint16_t)(sign | out);
}

/* quantized.rs:254-257 */
float ko_bf16_to_f32(uint16_t bits) { return bits_to_f32((uint32_t)bits << 16); }

/* quantized.rs:260-265 */
uint16_t ko_f32_to_bf16(float v) {
    uint32_t bits = f32_to_bits(v);
    uint32_t round = bits + (0x7FFFu + ((bits >> 16) & 1u));
    return (uint16_t)(round >> 16);
}

/* ------------------------------------------------------------------------ */
/* deterministic inputs                                                      */
/* ------------------------------------------------------------------------ */

/* parity.rs:22-31: 64-bit LCG, top bits -> [0, 2^31) -> f32 / 2^31 - 0.5 */
uint64_t ko_lcg_fill(float *out, size_t count, uint64_t seed, float mul) {
    uint64_t state = seed;
    for (size_t i = 0; i < count; ++i) {
        state = state * 6364136223846793005ULL + 1442695040888963407ULL;
        uint32_t bits = (uint32_t)(state >> 33) & 0x7FFFFFFFu;
        float v = ((float)bits / (float)2147483647) - 0.5f; /* i32::MAX as f32 */
        out[i] = v * mul;
    }
    return state;
}

/* ------------------------------------------------------------------------ */
/* quantiser                                                                 */
/* ------------------------------------------------------------------------ */

/* lib.rs:393-427 */
void ko_quantize(const float *weight, int k, int n, int groupsize, int32_t *codes,
                 uint16_t *scales_f16, float *dequant) {
    const int g = (groupsize == -1) ? k : groupsize;
    const int num_groups = k / g;
    float *scales = (float *)malloc(sizeof(float) * (size_t)num_groups * n);
    for (int grp = 0; grp < num_groups; ++grp) {
        for (int col = 0; col < n; ++col) {
            float max_abs = 0.0f;
            for (int r = 0; r < g; ++r) {
                float v = fabsf(weight[(size_t)(grp * g + r) * n + col]);
                if (v > max_abs) max_abs = v;
            }
            if (max_abs == 0.0f) max_abs = 1.0f; /* lib.rs:405-407 */
            float s_f32 = (2.0f * max_abs) / 15.0f;
            uint16_t h = ko_f32_to_f16(s_f32);
            scales_f16[(size_t)grp * n + col] = h;
            scales[(size_t)grp * n + col] = ko_f16_to_f32(h);
        }
    }
    for (int r = 0; r < k; ++r) {
        const int grp = r / g;
        for (int col = 0; col < n; ++col) {
            const float s = scales[(size_t)grp * n + col];
            /* Rust f32::round = half away from zero = roundf; `as i32`
             * saturates and maps NaN to 0.  `raw + Q_OFFSET` is an i32 sum
             * (lib.rs:423): where `raw` saturated at i32::MAX -- w / s = +inf, a
             * tiny non-zero group whose f16 scale rounded to 0 -- a release
             * build wraps to a negative value, which the clamp turns into code
             * 0 (a debug build panics there).  The release behaviour is
             * restated: the sum is formed in 64 bits and wrapped by hand. */
            float q = roundf(weight[(size_t)r * n + col] / s);
            long long raw;
            if (q != q) raw = 0;
            else if (q >= 2147483647.0f) raw = 2147483647LL;
            else if (q <= -2147483648.0f) raw = -2147483648LL;
            else raw = (long long)q;
            long long shifted = raw + 8;
            if (shifted > 2147483647LL) shifted -= 4294967296LL;
            if (shifted < 0) shifted = 0;
            if (shifted > 15) shifted = 15;
            codes[(size_t)r * n + col] = (int32_t)shifted;
            if (dequant) dequant[(size_t)r * n + col] = (float)((int)shifted - 8) * s;
        }
    }
    free(scales);
}

/* ------------------------------------------------------------------------ */
/* GPTQ-canonical layout                                                     */
/* ------------------------------------------------------------------------ */

void ko_pack_gptq(const int32_t *codes, int k, int n, uint32_t *qweight) {
    memset(qweight, 0, sizeof(uint32_t) * (size_t)(k / 8) * n);
    for (int r = 0; r < k; ++r)
        for (int c = 0; c < n; ++c)
            qweight[(size_t)(r / 8) * n + c] |= ((uint32_t)codes[(size_t)r * n + c] & 0xFu)
                                                << (4 * (r % 8));
}

/* quantized.rs:127-152 */
void ko_gptq_dequant_bf16(const uint32_t *qweight, const uint16_t *scales_f16,
                          const uint32_t *qzeros, int k, int n, int groupsize,
                          uint16_t *out_bf16) {
    const int g = (groupsize == -1) ? k : groupsize;
    const int n_packed = n / 8;
    for (int out_idx = 0; out_idx < n; ++out_idx) {
        for (int in_idx = 0; in_idx < k; ++in_idx) {
            int group = in_idx / g;
            uint32_t packed = qweight[(size_t)(in_idx / 8) * n + out_idx];
            int weight_int = (int)((packed >> ((in_idx % 8) * 4)) & 0xFu);
            int zero_int = 8;
            if (qzeros) {
                uint32_t zp = qzeros[(size_t)group * n_packed + out_idx / 8];
                zero_int = (int)((zp >> ((out_idx % 8) * 4)) & 0xFu);
            }
            float scale = ko_f16_to_f32(scales_f16[(size_t)group * n + out_idx]);
            float deq = (float)(weight_int - zero_int) * scale;
            out_bf16[(size_t)out_idx * k + in_idx] = ko_f32_to_bf16(deq);
        }
    }
}

/* lib.rs:425 applied to the GPTQ-canonical words */
void ko_dequant_f32(const uint32_t *qweight, const uint16_t *scales_f16, int k, int n,
                    int groupsize, float *out) {
    const int g = (groupsize == -1) ? k : groupsize;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < k; ++r) {
        const int group = r / g;
        const uint32_t *qrow = qweight + (size_t)(r / 8) * n;
        const int sh = (r % 8) * 4;
        for (int c = 0; c < n; ++c) {
            int code = (int)((qrow[c] >> sh) & 0xFu);
            out[(size_t)r * n + c] =
                (float)(code - 8) * ko_f16_to_f32(scales_f16[(size_t)group * n + c]);
        }
    }
}

/* ------------------------------------------------------------------------ */
/* matmul                                                                    */
/* ------------------------------------------------------------------------ */

int ko_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* lora_loader.rs:290-300.  Each output keeps one f32 accumulator that sees
 * k = 0, 1, 2, ... in order; columns are independent so the loop over column
 * blocks is what gets threaded. */
void ko_gemm_f32(const uint16_t *x_bf16, const float *w, int m, int k, int n, float *y) {
    const int NB = 256;
#pragma omp parallel for schedule(static)
    for (int n0 = 0; n0 < n; n0 += NB) {
        const int nb = (n - n0 < NB) ? (n - n0) : NB;
        for (int i = 0; i < m; ++i) {
            float acc[256];
            for (int j = 0; j < nb; ++j) acc[j] = 0.0f;
            for (int kk = 0; kk < k; ++kk) {
                const float xv = ko_bf16_to_f32(x_bf16[(size_t)i * k + kk]);
                const float *wrow = w + (size_t)kk * n + n0;
                for (int j = 0; j < nb; ++j) acc[j] += xv * wrow[j];
            }
            for (int j = 0; j < nb; ++j) y[(size_t)i * n + n0 + j] = acc[j];
        }
    }
}

void ko_gemm_f64(const uint16_t *x_bf16, const float *w, int m, int k, int n, double *y) {
    const int NB = 256;
#pragma omp parallel for schedule(static)
    for (int n0 = 0; n0 < n; n0 += NB) {
        const int nb = (n - n0 < NB) ? (n - n0) : NB;
        for (int i = 0; i < m; ++i) {
            double acc[256];
            for (int j = 0; j < nb; ++j) acc[j] = 0.0;
            for (int kk = 0; kk < k; ++kk) {
                const double xv = (double)ko_bf16_to_f32(x_bf16[(size_t)i * k + kk]);
                const float *wrow = w + (size_t)kk * n + n0;
                for (int j = 0; j < nb; ++j) acc[j] += xv * (double)wrow[j];
            }
            for (int j = 0; j < nb; ++j) y[(size_t)i * n + n0 + j] = acc[j];
        }
    }
}

void ko_w4a16_cpu_path(const uint16_t *x_bf16, const uint32_t *qweight,
                       const uint16_t *scales_f16, int m, int k, int n, int groupsize,
                       float *scratch, float *y) {
    ko_dequant_f32(qweight, scales_f16, k, n, groupsize, scratch);
    ko_gemm_f32(x_bf16, scratch, m, k, n, y);
}

/* lora_loader.rs:213-232 on the CPU/f32 branch: hidden = x * A^T [m, r],
 * delta = hidden * B^T [m, n], then * scale. */
void ko_lora_delta_add_f32(const uint16_t *x_bf16, const uint16_t *a_bf16,
                           const uint16_t *b_bf16, float scale, int m, int k, int n, int r,
                           float *y) {
    float *hidden = (float *)malloc(sizeof(float) * (size_t)m * r);
    for (int i = 0; i < m; ++i) {
        for (int j = 0; j < r; ++j) {
            float acc = 0.0f;
            for (int kk = 0; kk < k; ++kk)
                acc += ko_bf16_to_f32(x_bf16[(size_t)i * k + kk]) *
                       ko_bf16_to_f32(a_bf16[(size_t)j * k + kk]);
            hidden[(size_t)i * r + j] = acc;
        }
    }
#pragma omp parallel for schedule(static)
    for (int c = 0; c < n; ++c) {
        for (int i = 0; i < m; ++i) {
            float acc = 0.0f;
            for (int j = 0; j < r; ++j)
                acc += hidden[(size_t)i * r + j] * ko_bf16_to_f32(b_bf16[(size_t)c * r + j]);
            y[(size_t)i * n + c] += acc * scale;
        }
    }
    free(hidden);
}

/* forward.rs:110-114, 2789-2819: silu(gate) * up */
void ko_swiglu_f32(const float *gate, const float *up, size_t count, float *out) {
#pragma omp parallel for
    for (size_t i = 0; i < count; ++i) {
        const double g = gate[i];
        out[i] = (float)(g / (1.0 + exp(-g)) * (double)up[i]);
    }
}

/* adapter_merge.rs:639-712 */
void ko_merge_concat(const float *const *a_list, const float *const *b_list, const int *ranks,
                     const float *weights, int count, int k, int n, float *a_cat,
                     float *b_cat) {
    int r_total = 0;
    for (int i = 0; i < count; ++i) r_total += ranks[i];
    int row = 0;
    for (int i = 0; i < count; ++i) {
        memcpy(a_cat + (size_t)row * k, a_list[i], sizeof(float) * (size_t)ranks[i] * k);
        row += ranks[i];
    }
    int col = 0;
    for (int i = 0; i < count; ++i) {
        for (int j = 0; j < n; ++j)
            for (int c = 0; c < ranks[i]; ++c)
                b_cat[(size_t)j * r_total + col + c] =
                    weights[i] * b_list[i][(size_t)j * ranks[i] + c];
        col += ranks[i];
    }
}
