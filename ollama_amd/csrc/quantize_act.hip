// Kernel 1: on-GPU activation quantization to ggml's Q8_0 / Q8_K block formats.
//
// The block quantizers themselves (and the CPU semantics they reproduce bit for bit) are in
// quant_dev.h; this file holds the stand-alone kernels that write the structure-of-arrays planes the
// GEMV / GEMM kernels read, and the repacking of those planes into GGUF block bytes.
//
// With a producer (RMSNorm, SwiGLU: produce_dev.h) the quantizers apply it to x on the fly, so the
// normalized / gated activations exist only as Q8 planes; the same producers are also here as plain
// f32 kernels for graph nodes whose result something other than a product reads.
//
// HBM-bound and tiny next to the weight stream (N*K*4 bytes in, ~N*K*1.14 out); one float4 per lane,
// cross-lane max / sums over the 8 (Q8_0) or 64 (Q8_K) lanes that share a block.
#include "internal.h"
#include "produce_dev.h"
#include "quant_dev.h"

namespace miqmm {

namespace {

// float4 number t of x [N][K] after the producer
template <int KIND>
__device__ __forceinline__ float4 produced(const float4 *__restrict__ x, int64_t t, const Produce &pr, int64_t k4) {
    const float4 v = x[t];
    if (KIND == PRODUCE_RMSNORM) {
        const int64_t row = t / k4;
        const float4 *g4 = reinterpret_cast<const float4 *>(pr.aux);
        return rms_apply(v, pr.row_scale[row], g4 ? g4[t - row * k4] : v, g4 != nullptr);
    }
    if (KIND == PRODUCE_SWIGLU) return swiglu_apply(v, reinterpret_cast<const float4 *>(pr.aux)[t]);
    return v;
}

// 8 lanes per block of 32; 8 blocks per wave.  nblk = N*K/32 blocks in total.
template <int KIND>
__global__ __launch_bounds__(256) void quantize_q8_0_kernel(const float4 *__restrict__ x,
                                                            int *__restrict__ qs, float *__restrict__ d,
                                                            int16_t *__restrict__ bsums, int64_t nblk, Produce pr,
                                                            int64_t k4) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;  // 256 threads per workgroup (launch_quantize_act)
    const int64_t blk = t >> 3;
    const bool live = blk < nblk;
    // unconditional load (threads past the end read the last piece again and drop it): a conditional one
    // fetches its pointer only after the branch
    const float4 vl = produced<KIND>(x, live ? t : nblk * 8 - 1, pr, k4);
    const float4 v = live ? vl : make_float4(0.f, 0.f, 0.f, 0.f);
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
template <int KIND>
__global__ __launch_bounds__(256) void quantize_q8_K_kernel(const float4 *__restrict__ x,
                                                            int *__restrict__ qs, float *__restrict__ d,
                                                            int16_t *__restrict__ bsums, uint8_t *__restrict__ sd8,
                                                            uint8_t *__restrict__ sd16, uint16_t *__restrict__ qf,
                                                            uint16_t *__restrict__ bsf, int64_t nblk, Produce pr,
                                                            int64_t k4) {
    const int lane = threadIdx.x & 63;
    const int64_t blk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // 256 threads per workgroup (launch_quantize_act)
    // the load goes out before the range check (a wave past the end reads the last block again and leaves):
    // with the check first, the pointer is fetched only after the branch, a second round of scalar loads
    const float4 v = produced<KIND>(x, (blk < nblk ? blk : nblk - 1) * 64 + lane, pr, k4);
    if (blk >= nblk) return;  // whole wave leaves together
    float dd;
    int sum, pair;
    const int packed = q8_K_quantize_lane(v, lane, dd, sum, pair);
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
    // the quants and block sums as fp16 numbers for the fp16-MFMA GEMM.  This lane holds elements 4 (lane & 7) + i of
    // group lane >> 3; element 16h + 8u + j of a group goes to 16u + 8h + p(j), p = 0 2 1 3 4 6 5 7.
    if (qf) {
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        const h4 v4 = {(_Float16)(float)(int8_t)packed, (_Float16)(float)(int8_t)(packed >> 16),
                       (_Float16)(float)(int8_t)(packed >> 8), (_Float16)(float)(packed >> 24)};
        const int at = 32 * (lane >> 3) + 16 * ((lane >> 1) & 1) + 8 * ((lane >> 2) & 1) + 4 * (lane & 1);
        *reinterpret_cast<h4 *>(qf + blk * QKK + at) = v4;
        if ((lane & 3) == 0) bsf[blk * 16 + (lane >> 2)] = __half_as_ushort(__float2half_rn((float)sum));
    }
}

// The same planes with a quarter of a wave per super-block (q8_K_quantize_row16: lane l of a 16-lane row holds
// elements 16l.. of its block): a wave takes four consecutive blocks, 4 KiB of x in flight per wave instead of one, and
// about 45 vector instructions per block instead of 75.  Used for batches: with 28672 blocks (512 rows of 14336) the
// wave-per-block kernel is bound by how many of its small waves fit the machine, not by HBM.  Same bytes.
template <int KIND>
__global__ __launch_bounds__(256) void quantize_q8_K_row16_kernel(const float4 *__restrict__ x, uint4 *__restrict__ qs, float *__restrict__ d,
                                                                  int16_t *__restrict__ bsums, uint8_t *__restrict__ sd8,
                                                                  uint8_t *__restrict__ sd16, uint16_t *__restrict__ qf,
                                                                  uint16_t *__restrict__ bsf, int64_t nblk, Produce pr, int64_t k4) {
    const int lane = threadIdx.x & 63, sub = lane & 15;
    const int64_t b0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 4;  // 256 threads per workgroup: four waves of four blocks
    const int64_t blk = b0 + (lane >> 4), src = blk < nblk ? blk : nblk - 1;  // past the end: the last block again, not stored
    float4 v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) v[j] = produced<KIND>(x, src * 64 + 4 * sub + j, pr, k4);
    if (b0 >= nblk) return;  // whole wave leaves together
    float dd, qfl[16];
    int sum, pair;
    const uint4 packed = q8_K_quantize_row16(v, lane, dd, sum, pair, qf ? qfl : nullptr);
    if (blk >= nblk) return;  // whole 16-lane rows drop out; no cross-lane step follows
    qs[blk * 16 + sub] = packed;
    bsums[blk * 16 + sub] = (int16_t)sum;
    if (sub == 0) d[blk] = dd;
    if (sd16) {
        sd16[blk * 32 + sub] = (uint8_t)(sum & 63);
        sd16[blk * 32 + 16 + sub] = (uint8_t)(sum >> 6);
    }
    if (sd8 && (sub & 1) == 0) {
        sd8[blk * 16 + (sub >> 1)] = (uint8_t)(pair & 63);
        sd8[blk * 16 + 8 + (sub >> 1)] = (uint8_t)(pair >> 6);
    }
    if (qf) {
        // element 16h + 8u + j of a group of 32 goes to 16u + 8h + p(j), p = 0 2 1 3 4 6 5 7; this lane holds the half h = sub & 1
        // of group sub >> 1: its elements 8u + j, two runs of eight halves
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        uint16_t *base = qf + blk * QKK + 32 * (sub >> 1) + 8 * (sub & 1);
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const float *q8 = qfl + 8 * u;
            const h8 o = {(_Float16)q8[0], (_Float16)q8[2], (_Float16)q8[1], (_Float16)q8[3],
                          (_Float16)q8[4], (_Float16)q8[6], (_Float16)q8[5], (_Float16)q8[7]};
            *reinterpret_cast<h8 *>(base + 16 * u) = o;
        }
        bsf[blk * 16 + sub] = __half_as_ushort(__float2half_rn((float)sum));
    }
}

// RMSNorm, one workgroup per row of K floats: the row's scale (scale_out, optional) and the normalized row
// times the weight g (y, optional; g may be null).  Piece sums go through LDS 512 at a time and are added
// in piece order by every thread.
__global__ __launch_bounds__(256) void rms_norm_kernel(const float4 *__restrict__ x, const float4 *__restrict__ g,
                                                       float eps, int64_t K, float *__restrict__ scale_out,
                                                       float4 *__restrict__ y) {
    __shared__ double psum[512];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t n4 = K / 4, npieces = (n4 + 63) / 64;
    const float4 *xr = x + (int64_t)blockIdx.x * n4;
    double tot = 0.0;
    for (int64_t base = 0; base < npieces; base += 512) {
        const int64_t end = base + 512 < npieces ? base + 512 : npieces;
        for (int64_t c = base + wave; c < end; c += 4) {
            const int64_t i4 = c * 64 + lane;
            const double s = piece_sumsq(i4 < n4 ? xr[i4] : make_float4(0.f, 0.f, 0.f, 0.f));
            if (lane == 0) psum[c - base] = s;
        }
        __syncthreads();
        for (int64_t c = base; c < end; c++) tot += psum[c - base];
        __syncthreads();
    }
    const float scale = rms_scale_of(tot, K, eps);
    if (scale_out && threadIdx.x == 0) scale_out[blockIdx.x] = scale;
    if (y) {
        float4 *yr = y + (int64_t)blockIdx.x * n4;
        for (int64_t i4 = threadIdx.x; i4 < n4; i4 += 256) yr[i4] = rms_apply(xr[i4], scale, g ? g[i4] : xr[i4], g != nullptr);
    }
}

// count floats: float4 pieces where the pointers allow (vec), the rest one by one.  up == nullptr: the bare silu.
__global__ __launch_bounds__(256) void swiglu_kernel(const float *__restrict__ gate, const float *__restrict__ up,
                                                     float *__restrict__ y, int64_t count, bool vec) {
    const int64_t n4 = vec ? count / 4 : 0, first = (int64_t)blockIdx.x * 256 + threadIdx.x, step = (int64_t)gridDim.x * 256;
    if (!up) {
        for (int64_t i = first; i < n4; i += step) {
            const float4 v = reinterpret_cast<const float4 *>(gate)[i];
            reinterpret_cast<float4 *>(y)[i] = make_float4(silu(v.x), silu(v.y), silu(v.z), silu(v.w));
        }
        for (int64_t i = 4 * n4 + first; i < count; i += step) y[i] = silu(gate[i]);
        return;
    }
    for (int64_t i = first; i < n4; i += step)
        reinterpret_cast<float4 *>(y)[i] = swiglu_apply(reinterpret_cast<const float4 *>(gate)[i], reinterpret_cast<const float4 *>(up)[i]);
    for (int64_t i = 4 * n4 + first; i < count; i += step) y[i] = silu_mul(gate[i], up[i]);
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
                               int16_t *bsums, uint8_t *sd8, uint8_t *sd16, hipStream_t s, const Produce *produce,
                               uint16_t *qf, uint16_t *bsf) {
    if (N * K == 0) return hipSuccess;
    if ((qf != nullptr) != (bsf != nullptr)) return hipErrorInvalidValue;
    Produce pr{PRODUCE_NONE, nullptr, 0.f, nullptr};
    if (produce) pr = *produce;
    if ((pr.kind == PRODUCE_RMSNORM && !pr.row_scale) || (pr.kind == PRODUCE_SWIGLU && !pr.aux) ||
        pr.kind < PRODUCE_NONE || pr.kind > PRODUCE_SWIGLU || K % 4)
        return hipErrorInvalidValue;
    const int64_t k4 = K / 4;
    const float4 *x4 = (const float4 *)x;
    if (q8_type == T_Q8_0) {
        const int64_t nblk = N * K / QK;
        const int64_t threads = nblk * 8;
        const unsigned grid = (unsigned)((threads + 255) / 256);
        if (pr.kind == PRODUCE_RMSNORM) quantize_q8_0_kernel<PRODUCE_RMSNORM><<<grid, 256, 0, s>>>(x4, (int *)qs, d, bsums, nblk, pr, k4);
        else if (pr.kind == PRODUCE_SWIGLU) quantize_q8_0_kernel<PRODUCE_SWIGLU><<<grid, 256, 0, s>>>(x4, (int *)qs, d, bsums, nblk, pr, k4);
        else quantize_q8_0_kernel<PRODUCE_NONE><<<grid, 256, 0, s>>>(x4, (int *)qs, d, bsums, nblk, pr, k4);
    } else if (q8_type == T_Q8_K) {
        const int64_t nblk = N * K / QKK;
        if (nblk >= 4096) {  // batches: four blocks per wave (the same bytes)
            const unsigned grid16 = (unsigned)((nblk + 15) / 16);
            uint4 *q4 = reinterpret_cast<uint4 *>(qs);
            if (pr.kind == PRODUCE_RMSNORM) quantize_q8_K_row16_kernel<PRODUCE_RMSNORM><<<grid16, 256, 0, s>>>(x4, q4, d, bsums, sd8, sd16, qf, bsf, nblk, pr, k4);
            else if (pr.kind == PRODUCE_SWIGLU) quantize_q8_K_row16_kernel<PRODUCE_SWIGLU><<<grid16, 256, 0, s>>>(x4, q4, d, bsums, sd8, sd16, qf, bsf, nblk, pr, k4);
            else quantize_q8_K_row16_kernel<PRODUCE_NONE><<<grid16, 256, 0, s>>>(x4, q4, d, bsums, sd8, sd16, qf, bsf, nblk, pr, k4);
            return hipGetLastError();
        }
        const unsigned grid = (unsigned)((nblk + 3) / 4);
        if (pr.kind == PRODUCE_RMSNORM) quantize_q8_K_kernel<PRODUCE_RMSNORM><<<grid, 256, 0, s>>>(x4, (int *)qs, d, bsums, sd8, sd16, qf, bsf, nblk, pr, k4);
        else if (pr.kind == PRODUCE_SWIGLU) quantize_q8_K_kernel<PRODUCE_SWIGLU><<<grid, 256, 0, s>>>(x4, (int *)qs, d, bsums, sd8, sd16, qf, bsf, nblk, pr, k4);
        else quantize_q8_K_kernel<PRODUCE_NONE><<<grid, 256, 0, s>>>(x4, (int *)qs, d, bsums, sd8, sd16, qf, bsf, nblk, pr, k4);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_rms_norm(const float *x, const float *g, float eps, int64_t K, int64_t N, float *scale_out, float *y,
                           hipStream_t s) {
    if (N * K == 0) return hipSuccess;
    if (!x || K % 4 || N > 0x7fffffff || (!scale_out && !y)) return hipErrorInvalidValue;
    rms_norm_kernel<<<(unsigned)N, 256, 0, s>>>((const float4 *)x, (const float4 *)g, eps, K, scale_out, (float4 *)y);
    return hipGetLastError();
}

hipError_t launch_swiglu(const float *gate, const float *up, int64_t count, float *y, hipStream_t s) {
    if (count == 0) return hipSuccess;
    if (!gate || !y) return hipErrorInvalidValue;
    const bool vec = (((uintptr_t)gate | (uintptr_t)up | (uintptr_t)y) & 15) == 0;
    const int64_t work = vec ? count / 4 + 3 : count, blocks = (work + 255) / 256;
    swiglu_kernel<<<(unsigned)(blocks < 8192 ? blocks : 8192), 256, 0, s>>>(gate, up, y, count, vec);
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
