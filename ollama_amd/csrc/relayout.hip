// Upload-time re-layout: GGUF block bytes -> the device-private planes described in formats.h.
//
// GGUF rows are arrays of packed blocks (/root/reference/fs/ggml/gguf.go:281-308 hands them out
// unchanged).  18-, 34- and 210-byte blocks are only 2-byte aligned, so a wavefront cannot read them
// with aligned 16-byte loads; splitting each block's fields into separate planes restores that.
// Runs once per tensor at load; every field offset and size is even, so the copy moves 16-bit units.
#include <algorithm>

#include "internal.h"

namespace miqmm {

namespace {

// one thread per 16-bit unit of the source
template <int TYPE>
__global__ void relayout_kernel(const uint16_t *__restrict__ src, int64_t nblocks, uint16_t *__restrict__ p0,
                                uint16_t *__restrict__ p1, uint16_t *__restrict__ p2,
                                uint16_t *__restrict__ d) {
    constexpr int UNITS = (TYPE == T_Q4_0 ? Q4_0_BYTES : TYPE == T_Q8_0 ? Q8_0_BYTES : Q6_K_BYTES) / 2;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nblocks * UNITS) return;
    const int64_t blk = i / UNITS;
    const int u = (int)(i - blk * UNITS);
    const uint16_t v = src[i];
    if (TYPE == T_Q4_0) {  // d(1 unit) qs(8 units)
        if (u == 0) d[blk] = v; else p0[blk * 8 + (u - 1)] = v;
    } else if (TYPE == T_Q8_0) {  // d(1) qs(16)
        if (u == 0) d[blk] = v; else p0[blk * 16 + (u - 1)] = v;
    } else {  // Q6_K: ql(64) qh(32) scales(8) d(1)
        if (u < 64) p0[blk * 64 + u] = v;
        else if (u < 96) p1[blk * 32 + (u - 64)] = v;
        else if (u < 104) p2[blk * 8 + (u - 96)] = v;
        else d[blk] = v;
    }
}

// Q5_K -> a Q4_K tensor of rows twice as long.  w = d sc (q4 + 16 h) - dmin m with h the fifth bit, so a row's dot
// product is the Q4_K dot product of its low parts plus 16 d yd sum_j sc_j sum_l h_jl y_jl: the same shape of sum with
// nibble 8 h, block scale 2 d (exact in fp16 unless |d| > 32752) and no mins.  Block b of a row goes to block b (d, dmin,
// scales, nibbles as they are) and to block nsb + b (2 d, dmin = 0, the same scale bytes, nibble 8 for a set bit).
// One thread per 16-bit unit of the 144-byte destination blocks of both halves.
__global__ void relayout_q5k_kernel(const uint8_t *__restrict__ src, int64_t M, int nsb, uint8_t *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = M * nsb * 2 * (Q4_K_BYTES / 2);
    if (i >= total) return;
    const int u = (int)(i % (Q4_K_BYTES / 2));       // 16-bit unit inside the destination block
    const int64_t db = i / (Q4_K_BYTES / 2);         // destination block: row * 2 nsb + (half * nsb + b)
    const int64_t row = db / (2 * nsb);
    const int within = (int)(db - row * 2 * nsb), half = within / nsb, b = within - half * nsb;
    const uint8_t *blk = src + (row * nsb + b) * Q5_K_BYTES;
    uint16_t v;
    if (u < 8) {  // d, dmin, scales[12]
        v = (uint16_t)(blk[2 * u] | (blk[2 * u + 1] << 8));
        if (half == 1) {
            if (u == 0) v = __builtin_bit_cast(uint16_t, (_Float16)((_Float16)2.0f * __builtin_bit_cast(_Float16, v)));
            else if (u == 1) v = 0;
        }
    } else {      // nibble bytes 2 (u - 8), 2 (u - 8) + 1 of the 128
        const int q0 = 2 * (u - 8);
        if (half == 0) v = (uint16_t)(blk[48 + q0] | (blk[48 + q0 + 1] << 8));
        else {
            uint16_t r = 0;
            for (int t = 0; t < 2; t++) {
                const int q = q0 + t, c = q >> 5, l = q & 31;  // byte q holds elements l of sub-blocks 2c (low) and 2c + 1 (high)
                const unsigned h = blk[16 + l];
                const unsigned byte = (((h >> (2 * c)) & 1u) << 3) | (((h >> (2 * c + 1)) & 1u) << 7);
                r |= (uint16_t)(byte << (8 * t));
            }
            v = r;
        }
    }
    reinterpret_cast<uint16_t *>(out)[i] = v;
}

// MXFP4 -> Q8_0 planes.  An MXFP4 block (/root/reference/convert/convert_gptoss.go:216-238: an E8M0 scale byte, then 16
// bytes whose low nibbles are elements 0..15 and whose high nibbles are elements 16..31) is 32 small integers -- the E2M1
// values doubled: 0 1 2 3 4 6 8 12 and their negatives -- under the scale 2^(e - 128), and ggml multiplies it with Q8_0
// activations as sum_i q_i y_i * (scale * d_y): the Q8_0 dot product of a block with those integers and that scale.  The
// scale is a half for e in 104 .. 143; up to e = 146 the integers are shifted left instead (12 * 8 = 96 fits); below 104
// (weights under 7.2e-7) the block is zero; above 146 *bad is set.  One thread per nibble byte.
// Rows are padded with zero blocks from nb_in to nb_out blocks (rows of a whole number of 256-element steps, which the
// matrix-core kernels for the 32-element formats want).
__global__ void relayout_mxfp4_kernel(const uint8_t *__restrict__ src, int64_t M, int nb_in, int nb_out, int8_t *__restrict__ qs,
                                      uint16_t *__restrict__ d, int *__restrict__ bad) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= M * nb_out * 16) return;
    const int64_t blk = i >> 4, row = blk / nb_out;
    const int bi = (int)(blk - row * nb_out), j = (int)(i & 15);
    if (bi >= nb_in) {
        qs[blk * 32 + j] = 0;
        qs[blk * 32 + j + 16] = 0;
        if (j == 0) d[blk] = 0;
        return;
    }
    const uint8_t *b = src + (row * nb_in + bi) * 17;
    const int e = b[0];
    int shift = 0, he = e - 128 + 15;  // biased fp16 exponent of 2^(e - 128)
    if (e > 143) { shift = e - 143; he = 30; }
    if (e > 146) { shift = 0; he = 0; if (j == 0) atomicOr(bad, 1); }
    const bool zero = e < 104 || e > 146;
    const int lo = b[1 + j] & 15, hi = b[1 + j] >> 4;
    const int mag_lo = (lo & 7) < 5 ? (lo & 7) : (lo & 7) == 5 ? 6 : (lo & 7) == 6 ? 8 : 12;
    const int mag_hi = (hi & 7) < 5 ? (hi & 7) : (hi & 7) == 5 ? 6 : (hi & 7) == 6 ? 8 : 12;
    qs[blk * 32 + j] = zero ? 0 : (int8_t)(((lo & 8) ? -mag_lo : mag_lo) << shift);
    qs[blk * 32 + j + 16] = zero ? 0 : (int8_t)(((hi & 8) ? -mag_hi : mag_hi) << shift);
    if (j == 0) {
        // 2^(e - 128) as a half: normal from 2^-14 (e = 114), subnormal 2^-24 .. 2^-15 below
        uint16_t h;
        if (zero) h = 0;
        else if (he >= 1) h = (uint16_t)(he << 10);
        else h = (uint16_t)(1u << (e - 104));
        d[blk] = h;
    }
}

// Q5_0 -> Q8_0 planes.  w = d (q - 16) with q the nibble plus 16 times bit i of the 32-bit word qh: 32 integers in -16..15
// under the block's fp16 scale, and ggml multiplies them with Q8_0 activations as sum_i (q_i - 16) y_i * (d d_y) -- the Q8_0 dot
// product of those integers, term for term.  Rows padded with zero blocks from nb_in to nb_out blocks.  One thread per nibble byte.
__global__ void relayout_q5_0_kernel(const uint8_t *__restrict__ src, int64_t M, int nb_in, int nb_out, int8_t *__restrict__ qs,
                                     uint16_t *__restrict__ d) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= M * nb_out * 16) return;
    const int64_t blk = i >> 4, row = blk / nb_out;
    const int bi = (int)(blk - row * nb_out), j = (int)(i & 15);
    if (bi >= nb_in) {
        qs[blk * 32 + j] = 0;
        qs[blk * 32 + j + 16] = 0;
        if (j == 0) d[blk] = 0;
        return;
    }
    const uint8_t *b = src + (row * nb_in + bi) * 22;
    const unsigned qh = b[2] | (b[3] << 8) | (b[4] << 16) | ((unsigned)b[5] << 24);
    const int q = b[6 + j];
    qs[blk * 32 + j] = (int8_t)(((q & 15) | (((qh >> j) & 1u) << 4)) - 16);
    qs[blk * 32 + j + 16] = (int8_t)(((q >> 4) | (((qh >> (j + 16)) & 1u) << 4)) - 16);
    if (j == 0) d[blk] = (uint16_t)(b[0] | (b[1] << 8));
}

// MXFP4 as it is, for the streaming kernels: the 16 nibble bytes of every block in one plane, its scale byte (widened to 16
// bits) in another; rows padded with zero blocks (scale byte 0, codes 0) from nb_in to nb_out blocks.
__global__ void relayout_mxfp4_native_kernel(const uint8_t *__restrict__ src, int64_t M, int nb_in, int nb_out, uint8_t *__restrict__ qs,
                                             uint16_t *__restrict__ e) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= M * nb_out * 16) return;
    const int64_t blk = i >> 4, row = blk / nb_out;
    const int bi = (int)(blk - row * nb_out), j = (int)(i & 15);
    const bool pad = bi >= nb_in;
    const uint8_t *b = src + (row * nb_in + (pad ? 0 : bi)) * 17;
    qs[blk * 16 + j] = pad ? 0 : b[1 + j];
    if (j == 0) e[blk] = pad ? 0 : b[0];
}

// out [n][k_out] from x [n][k_in] (in float4 units): the row, then -- repeat (k_out = 2 k_in): the row once more; else zeros
__global__ void expand_rows_kernel(const float4 *__restrict__ x, float4 *__restrict__ out, int64_t k4_in, int64_t k4_out, int64_t n, bool repeat) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < k4_out * n; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / k4_out, c = i - r * k4_out;
        float4 v = {0.f, 0.f, 0.f, 0.f};
        if (c < k4_in) v = x[r * k4_in + c];
        else if (repeat) v = x[r * k4_in + (c - k4_in)];
        out[i] = v;
    }
}

}  // namespace

hipError_t launch_relayout_q5k(const uint8_t *gguf, int64_t K, int64_t M, uint8_t *out, hipStream_t s) {
    if (K * M == 0) return hipSuccess;
    const int64_t n = M * (K / QKK) * 2 * (Q4_K_BYTES / 2);
    if ((n + 255) / 256 > 0x7fffffff) return hipErrorInvalidValue;
    relayout_q5k_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(gguf, M, (int)(K / QKK), out);
    return hipGetLastError();
}

hipError_t launch_relayout_mxfp4(const uint8_t *gguf, int64_t K, int64_t K_out, int64_t M, uint8_t *qs, uint16_t *d, int *bad, hipStream_t s) {
    if (K * M == 0) return hipSuccess;
    if (K % QK || K_out % QK || K_out < K) return hipErrorInvalidValue;
    const int64_t n = M * (K_out / QK) * 16;
    if ((n + 255) / 256 > 0x7fffffff) return hipErrorInvalidValue;
    relayout_mxfp4_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(gguf, M, (int)(K / QK), (int)(K_out / QK), (int8_t *)qs, d, bad);
    return hipGetLastError();
}

hipError_t launch_relayout_q5_0(const uint8_t *gguf, int64_t K, int64_t K_out, int64_t M, uint8_t *qs, uint16_t *d, hipStream_t s) {
    if (K * M == 0) return hipSuccess;
    if (K % QK || K_out % QK || K_out < K) return hipErrorInvalidValue;
    const int64_t n = M * (K_out / QK) * 16;
    if ((n + 255) / 256 > 0x7fffffff) return hipErrorInvalidValue;
    relayout_q5_0_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(gguf, M, (int)(K / QK), (int)(K_out / QK), (int8_t *)qs, d);
    return hipGetLastError();
}

hipError_t launch_relayout_mxfp4_native(const uint8_t *gguf, int64_t K, int64_t K_out, int64_t M, uint8_t *qs, uint16_t *e, hipStream_t s) {
    if (K * M == 0) return hipSuccess;
    if (K % QK || K_out % QK || K_out < K) return hipErrorInvalidValue;
    const int64_t n = M * (K_out / QK) * 16;
    if ((n + 255) / 256 > 0x7fffffff) return hipErrorInvalidValue;
    relayout_mxfp4_native_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(gguf, M, (int)(K / QK), (int)(K_out / QK), qs, e);
    return hipGetLastError();
}

hipError_t launch_expand_rows(const float *x, int64_t K, int64_t K_out, int64_t n, bool repeat, float *out, hipStream_t s) {
    if (K * n == 0) return hipSuccess;
    if (K % 4 || K_out % 4 || K_out < K || (repeat && K_out != 2 * K)) return hipErrorInvalidValue;
    const int64_t work = K_out / 4 * n;
    expand_rows_kernel<<<(unsigned)std::min<int64_t>((work + 255) / 256, 4096), 256, 0, s>>>((const float4 *)x, (float4 *)out, K / 4, K_out / 4, n,
                                                                                             repeat);
    return hipGetLastError();
}

hipError_t launch_relayout(int type, const uint8_t *gguf, int64_t K, int64_t M, uint8_t *p0, uint8_t *p1,
                           uint8_t *p2, uint16_t *d, hipStream_t s) {
    if (K * M == 0) return hipSuccess;
    const uint16_t *src = (const uint16_t *)gguf;
    if (type == T_Q4_K) {
        return hipMemcpyAsync(p0, gguf, (size_t)(M * (K / QKK) * Q4_K_BYTES), hipMemcpyDeviceToDevice, s);
    } else if (type == T_Q4_0) {
        const int64_t nb = M * (K / QK), n = nb * (Q4_0_BYTES / 2);
        relayout_kernel<T_Q4_0><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(src, nb, (uint16_t *)p0, nullptr, nullptr, d);
    } else if (type == T_Q8_0) {
        const int64_t nb = M * (K / QK), n = nb * (Q8_0_BYTES / 2);
        relayout_kernel<T_Q8_0><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(src, nb, (uint16_t *)p0, nullptr, nullptr, d);
    } else if (type == T_Q6_K) {
        const int64_t nb = M * (K / QKK), n = nb * (Q6_K_BYTES / 2);
        relayout_kernel<T_Q6_K><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(src, nb, (uint16_t *)p0, (uint16_t *)p1,
                                                                            (uint16_t *)p2, d);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace miqmm
