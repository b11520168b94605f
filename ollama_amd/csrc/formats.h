// GGUF block formats on the quantized-matmul path, and the device-private layouts the kernels read.
//
// Block byte layouts follow the size formulas in /root/reference/fs/ggml/ggml.go:450-473:
//   Q4_0  2 + 32/2             = 18   fp16 d; u8 qs[16]  (low nibbles = elements 0..15, high = 16..31; value q-8)
//   Q8_0  2 + 32               = 34   fp16 d; i8 qs[32]
//   Q4_K  2 + 2 + 12 + 256/2   = 144  fp16 d, dmin; u8 scales[12] (8 x 6-bit scale + 8 x 6-bit min); u8 qs[128]
//   Q5_K  2 + 2 + 12 + 32 + 128 = 176 fp16 d, dmin; u8 scales[12]; u8 qh[32] (bit j of qh[l]: fifth bit of element l of
//                                     sub-block j); u8 qs[128]
//   Q6_K  256/2 + 256/4 + 16+2 = 210  u8 ql[128]; u8 qh[64]; i8 scales[16]; fp16 d   (value q-32)
//   Q8_K  4 + 256 + 2*16       = 292  f32 d; i8 qs[256]; i16 bsums[16]
#pragma once

#include <stdint.h>

namespace miqmm {

enum : int { T_F32 = 0, T_F16 = 1, T_BF16 = 30, T_Q4_0 = 2, T_Q5_0 = 6, T_Q8_0 = 8, T_Q4_K = 12, T_Q5_K = 13, T_Q6_K = 14, T_Q8_K = 15, T_MXFP4 = 39 };

constexpr int QK = 32;    // elements per Q4_0 / Q8_0 block
constexpr int QKK = 256;  // elements per K-quant super-block
constexpr int Q4_0_BYTES = 18, Q8_0_BYTES = 34, Q4_K_BYTES = 144, Q5_K_BYTES = 176, Q6_K_BYTES = 210, Q8_K_BYTES = 292;

// Weight tensor as the kernels see it.  Device-private "plane" layout chosen so that every
// wavefront load is a run of aligned 16-byte pieces:
//   Q4_K : p0 = the GGUF blocks unchanged (144 B is already 16-B aligned: header 16 B + qs 128 B)
//   Q4_0 : p0 = qs plane, 16 B per block, [M][K/32][16];           d = fp16 plane [M][K/32]
//   Q8_0 : p0 = qs plane, 32 B per block, [M][K];                  d = fp16 plane [M][K/32]
//   Q6_K : p0 = ql plane [M][K/2]; p1 = qh plane [M][K/4]; p2 = scales plane [M][K/16] (i8);
//          d = fp16 plane [M][K/256]
//   Q5_K : stored as a Q4_K tensor of rows twice as long (type = T_Q4_K, K = 2 K'): blocks 0 .. K'/256 - 1 of a row are
//          the Q5_K blocks without their fifth bits, blocks K'/256 .. are the fifth bits alone -- same scales, no mins,
//          nibble 8 where the bit is set, block scale 2 d -- so that against the activations repeated, [x | x], every
//          Q4_K kernel computes sum sc (q4 + 16 h) y exactly (see relayout.hip)
//   Q5_0 : stored as the Q8_0 planes with the same dot products (type = T_Q8_0): the 5-bit values minus 16 as int8, d as it is
//   MXFP4: stored as the Q8_0 planes with the same dot products (type = T_Q8_0): the doubled E2M1 values as int8, the scale
//          2^(e - 128) as the fp16 block scale (see relayout.hip) -- what the matrix-core kernels multiply -- and once more as
//          it is (type = T_MXFP4: p0 = nibble plane [M][K/32][16], d = the scale bytes, 16 bits each) for the streaming kernels
//   F32, F16, BF16 : p0 = the rows unchanged, [M][K] elements
// Byte order inside each plane is the GGUF order; only the interleaving of fields is undone.
struct DevWeight {
    const uint8_t *p0;
    const uint8_t *p1;
    const uint8_t *p2;
    const uint16_t *d;
    int64_t K, M;
    int type;
};

// Quantized activations as the kernels see them (structure of arrays, one row per activation row):
//   qs    [N][K]      int8 quants
//   d     [N][K/B]    fp32 block scale (B = 32 for Q8_0 where the value is the fp16-rounded scale
//                     widened exactly; B = 256 for Q8_K)
//   bsums [N][K/S]    int16 partial sums of quants (S = 32 for Q8_0: one per block; S = 16 for Q8_K)
// Q8_K only, for the MFMA GEMM (block sums as two int8 digits, S = 64*S_h + S_l, S_l in 0..63):
//   sd8   [N][K/256][16]   S_j = bsums[2j] + bsums[2j+1], j = 0..7:  bytes [S_l(0..7) | S_h(0..7)]
//   sd16  [N][K/256][32]   S_g = bsums[g], g = 0..15:                bytes [S_l(0..15) | S_h(0..15)]
// Q8_K only, for the fp16-MFMA GEMM (null when not planned):
//   qf    [N][K]           the quants as fp16 numbers; inside every group of 32, element 16h + 8u + j sits at
//                          16u + 8h + p(j), p = 0 2 1 3 4 6 5 7 (the order the GEMM expands weight nibbles in)
//   bsf   [N][K/256][16]   bsums as fp16 numbers (|sum of 16 quants| <= 2048: exact)
struct DevAct {
    const int8_t *qs;
    const float *d;
    const int16_t *bsums;
    const uint8_t *sd8;
    const uint8_t *sd16;
    int64_t K;
    int N;
    int type;  // T_Q8_0 or T_Q8_K
    const uint16_t *qf = nullptr;
    const uint16_t *bsf = nullptr;
};

}  // namespace miqmm
