// Tile layout of packed int4 weights and fp16 scales (layout version 1).
//
// The unit is a "chunk": 16 output columns x 128 input rows (one scale group)
// = 2048 codes = 256 words = 1 KiB.  Chunks are ordered [column tile][group]:
//
//     chunk(nt, g) starts at word ((nt * G + g) * 256),  nt = n/16, g = k/128, G = K/128
//
// Inside a chunk, word index = lane * 4 + t with lane in 0..63, t in 0..3:
//
//     lane = c + 16 * kq      c  = column within the tile (0..15)
//                             kq = which 8-row slice of a 32-row step (0..3)
//     word (lane, t) holds rows  k = 128 g + 32 t + 8 kq + j,  j = 0..7
//     row j sits in nibble  p(j) = j/2 + 4 * (j & 1)
//
// Why: one wavefront reads a chunk with a single 128-bit load per lane (1 KiB,
// fully coalesced).  Word t of a lane is exactly that lane's B operand for the
// t-th v_mfma_f32_16x16x32_bf16 step (lane = column c, k-slice kq, 8 rows), and
// `(w >> 4r) & 0x000F000F` leaves rows 2r (low half) and 2r+1 (high half) in
// place for a packed bf16 pair, so register r of the operand needs one
// shift and one and-or.  Two such loads also feed v_mfma_f32_32x32x16_bf16
// (lanes 0-31 / 32-63 take the kq pairs of two neighbouring column tiles).
//
// Scales: [column tile][scale group][16] fp16, scale group = g when
// groupsize == 128 and 0 when groupsize == -1.
#pragma once
#include <stddef.h>
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define KILN_HD __host__ __device__
#else
#define KILN_HD
#endif

namespace kiln {

// Revision of the layout written into artefacts.
//   1: the chunk layout of this file; fused gate/up packs carried 32 gate then 32 up columns per 64.
//   2: fused gate/up packs carry 8 gate then the 8 matching up columns per 16-column tile, which is
//      what every kernel's SwiGLU store pairs up.  The chunk layout itself did not change, but a
//      revision-1 fused pack read by these kernels would pair the wrong columns without any error,
//      so revision-1 artefacts are refused and must be repacked.
constexpr int kLayoutVersion = 2;
constexpr int kTileN = 16;        // columns per chunk
constexpr int kGroupK = 128;      // rows per chunk (= quantisation group)
constexpr int kChunkWords = 256;  // 1 KiB

// nibble position of row j (0..7) inside a word
KILN_HD constexpr int nibble_pos(int j) { return (j >> 1) + 4 * (j & 1); }

// word index of (k, n) in the packed buffer, and the nibble inside it
KILN_HD inline size_t packed_word_index(int k, int n, int G) {
    const int nt = n / kTileN, c = n % kTileN;
    const int g = k / kGroupK, kr = k % kGroupK;
    const int t = kr / 32, kq = (kr % 32) / 8;
    return ((size_t)nt * G + g) * kChunkWords + (size_t)(c + 16 * kq) * 4 + t;
}

// index of the scale of (scale group gs, column n); Gs = number of scale groups
KILN_HD inline size_t scale_index(int gs, int n, int Gs) {
    return ((size_t)(n / kTileN) * Gs + gs) * kTileN + (n % kTileN);
}

}  // namespace kiln
