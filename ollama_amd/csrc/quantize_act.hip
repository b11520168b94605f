// Kernel 1: on-GPU activation quantization to ggml's Q8_0 / Q8_K block formats.
//
// The block quantizers themselves (and the CPU semantics they reproduce bit for bit) are in
// quant_dev.h; this file holds the stand-alone kernels that write the structure-of-arrays planes the
// GEMV / GEMM kernels read, and the repacking of those planes into GGUF block bytes.
//
// HBM-bound and tiny next to the weight stream (N*K*4 bytes in, ~N*K*1.14 out); one float4 per lane,
// cross-lane max / sums over the 8 (Q8_0) or 64 (Q8_K) lanes that share a block.
#include "internal.h"
#include "quant_dev.h"

namespace miqmm {

namespace {

// 8 lanes per block of 32; 8 blocks per wave.  nblk = N*K/32 blocks in total.
__global__ __launch_bounds__(256) void quantize_q8_0_kernel(const float4 *__restrict__ x,
                                                            int *__restrict__ qs, float *__restrict__ d,
                                                            int16_t *__restrict__ bsums, int64_t nblk) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t blk = t >> 3;
    const bool live = blk < nblk;
    const float4 v = live ? x[t] : make_float4(0.f, 0.f, 0.f, 0.f);
    float dd;
    int sum;
    const int packed = q8_0_quantize_lane(v, dd, sum);
    if (live) {
        qs[t] = packed;
        if ((t & 7) == 0) {
            d[blk] = dd;
            bsums[blk] = (int16_t)sum;
        }
    }
}

// one wave per super-block of 256; 4 waves per workgroup.  nblk = N*K/256.
__global__ __launch_bounds__(256) void quantize_q8_K_kernel(const float4 *__restrict__ x,
                                                            int *__restrict__ qs, float *__restrict__ d,
                                                            int16_t *__restrict__ bsums, uint8_t *__restrict__ sd8,
                                                            uint8_t *__restrict__ sd16, int64_t nblk) {
    const int lane = threadIdx.x & 63;
    const int64_t blk = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (blk >= nblk) return;  // whole wave leaves together
    float dd;
    int sum, pair;
    const int packed = q8_K_quantize_lane(x[blk * 64 + lane], lane, dd, sum, pair);
    qs[blk * 64 + lane] = packed;
    if ((lane & 3) == 0) bsums[blk * 16 + (lane >> 2)] = (int16_t)sum;
    if (lane == 0) d[blk] = dd;
    // block sums as two int8 digits (s = 64*(s >> 6) + (s & 63)) for the int8-MFMA GEMM
    if (sd16 && (lane & 3) == 0) {
        sd16[blk * 32 + (lane >> 2)] = (uint8_t)(sum & 63);
        sd16[blk * 32 + 16 + (lane >> 2)] = (uint8_t)(sum >> 6);
    }
    if (sd8 && (lane & 7) == 0) {
        sd8[blk * 16 + (lane >> 3)] = (uint8_t)(pair & 63);
        sd8[blk * 16 + 8 + (lane >> 3)] = (uint8_t)(pair >> 6);
    }
}

// planes -> GGUF bytes; one thread per output byte (a convenience path, not on the hot path)
__global__ void pack_q8_0_kernel(const int8_t *__restrict__ qs, const float *__restrict__ d,
                                 uint8_t *__restrict__ out, int64_t nbytes) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nbytes) return;
    const int64_t blk = i / Q8_0_BYTES;
    const int off = (int)(i - blk * Q8_0_BYTES);
    if (off < 2) {
        const unsigned short h = __half_as_ushort(__float2half_rn(d[blk]));
        out[i] = (uint8_t)(h >> (8 * off));
    } else {
        out[i] = (uint8_t)qs[blk * QK + off - 2];
    }
}

__global__ void pack_q8_K_kernel(const int8_t *__restrict__ qs, const float *__restrict__ d,
                                 const int16_t *__restrict__ bsums, uint8_t *__restrict__ out,
                                 int64_t nbytes) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nbytes) return;
    const int64_t blk = i / Q8_K_BYTES;
    const int off = (int)(i - blk * Q8_K_BYTES);
    if (off < 4) {
        out[i] = (uint8_t)(__float_as_uint(d[blk]) >> (8 * off));
    } else if (off < 4 + QKK) {
        out[i] = (uint8_t)qs[blk * QKK + off - 4];
    } else {
        const int b = off - 4 - QKK;
        const unsigned short s = (unsigned short)bsums[blk * 16 + (b >> 1)];
        out[i] = (uint8_t)(s >> (8 * (b & 1)));
    }
}

}  // namespace

hipError_t launch_quantize_act(int q8_type, const float *x, int64_t K, int64_t N, int8_t *qs, float *d,
                               int16_t *bsums, uint8_t *sd8, uint8_t *sd16, hipStream_t s) {
    if (N * K == 0) return hipSuccess;
    if (q8_type == T_Q8_0) {
        const int64_t nblk = N * K / QK;
        const int64_t threads = nblk * 8;
        const unsigned grid = (unsigned)((threads + 255) / 256);
        quantize_q8_0_kernel<<<grid, 256, 0, s>>>((const float4 *)x, (int *)qs, d, bsums, nblk);
    } else if (q8_type == T_Q8_K) {
        const int64_t nblk = N * K / QKK;
        const unsigned grid = (unsigned)((nblk + 3) / 4);
        quantize_q8_K_kernel<<<grid, 256, 0, s>>>((const float4 *)x, (int *)qs, d, bsums, sd8, sd16, nblk);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_pack_act_gguf(int q8_type, const int8_t *qs, const float *d, const int16_t *bsums,
                                int64_t K, int64_t N, uint8_t *out, hipStream_t s) {
    if (N * K == 0) return hipSuccess;
    if (q8_type == T_Q8_0) {
        const int64_t nbytes = N * K / QK * Q8_0_BYTES;
        pack_q8_0_kernel<<<(unsigned)((nbytes + 255) / 256), 256, 0, s>>>(qs, d, out, nbytes);
    } else if (q8_type == T_Q8_K) {
        const int64_t nbytes = N * K / QKK * Q8_K_BYTES;
        pack_q8_K_kernel<<<(unsigned)((nbytes + 255) / 256), 256, 0, s>>>(qs, d, bsums, out, nbytes);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace miqmm
