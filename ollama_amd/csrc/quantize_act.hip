// Kernel 1: on-GPU activation quantization to ggml's Q8_0 / Q8_K block formats.
//
// Semantics are the scalar CPU quantizers' (quantize_row_q8_0_ref / quantize_row_q8_K_ref of ggml,
// the from_float step of the CPU mul_mat that Tensor.Mulmat -- /root/reference/ml/backend.go:151 --
// ends in); the bytes produced are identical to the CPU's:
//   Q8_0: amax over 32; d = amax/127 (IEEE fp32 divide); id = d ? 1/d : 0; q = roundf(x*id)
//         (half away from zero); stored scale = fp16_rne(d).
//   Q8_K: first element of largest |x| over 256, with its sign: max; iscale = -127/max;
//         q = min(127, rne(iscale*x)) on the fp32-rounded product; bsums = sums of 16; d = 1/iscale.
//         An all-zero block is all zero bytes.
// This file is compiled with -ffp-contract=off: none of the expressions above may be fused.
//
// HBM-bound and tiny next to the weight stream (N*K*4 bytes in, ~N*K*1.14 out); one float4 per lane,
// cross-lane max / sums over the 8 (Q8_0) or 64 (Q8_K) lanes that share a block.
#include <hip/hip_fp16.h>

#include "internal.h"

namespace miqmm {

namespace {

__device__ __forceinline__ int pack4(int a, int b, int c, int d) {
    return (a & 0xff) | ((b & 0xff) << 8) | ((c & 0xff) << 16) | ((d & 0xff) << 24);
}

// 8 lanes per block of 32; 8 blocks per wave.  nblk = N*K/32 blocks in total.
__global__ __launch_bounds__(256) void quantize_q8_0_kernel(const float4 *__restrict__ x,
                                                            int *__restrict__ qs, float *__restrict__ d,
                                                            int16_t *__restrict__ bsums, int64_t nblk) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t blk = t >> 3;
    const bool live = blk < nblk;
    float4 v = live ? x[t] : make_float4(0.f, 0.f, 0.f, 0.f);
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    amax = fmaxf(amax, __shfl_xor(amax, 2));
    amax = fmaxf(amax, __shfl_xor(amax, 4));
    const float dd = amax / 127.0f;
    const float id = dd != 0.0f ? 1.0f / dd : 0.0f;
    const int q0 = (int)roundf(v.x * id), q1 = (int)roundf(v.y * id);
    const int q2 = (int)roundf(v.z * id), q3 = (int)roundf(v.w * id);
    int sum = q0 + q1 + q2 + q3;
    sum += __shfl_xor(sum, 1);
    sum += __shfl_xor(sum, 2);
    sum += __shfl_xor(sum, 4);
    if (live) {
        qs[t] = pack4(q0, q1, q2, q3);
        if ((t & 7) == 0) {
            d[blk] = __half2float(__float2half_rn(dd));  // the scale the CPU stores and later reads
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
    const float4 v = x[blk * 64 + lane];
    // first strictly-greater scan, ascending index
    float amax = 0.0f, mx = 0.0f;
    int idx = 0;
    const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float ax = fabsf(e[i]);
        if (ax > amax) { amax = ax; mx = e[i]; idx = lane * 4 + i; }
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float oa = __shfl_xor(amax, off), om = __shfl_xor(mx, off);
        const int oi = __shfl_xor(idx, off);
        if (oa > amax || (oa == amax && oi < idx)) { amax = oa; mx = om; idx = oi; }
    }
    int q[4] = {0, 0, 0, 0};
    float dd = 0.0f;
    if (amax != 0.0f) {
        const float iscale = -127.0f / mx;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float p = iscale * e[i];
            q[i] = min(127, (int)rintf(p));
        }
        dd = 1.0f / iscale;
    }
    int sum = q[0] + q[1] + q[2] + q[3];
    sum += __shfl_xor(sum, 1);
    sum += __shfl_xor(sum, 2);
    const int pair = sum + __shfl_xor(sum, 4);  // bsums[2j] + bsums[2j+1] in lanes 8j .. 8j+7
    qs[blk * 64 + lane] = pack4(q[0], q[1], q[2], q[3]);
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
