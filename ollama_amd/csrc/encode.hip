// Weight encoders on the GPU: f32 rows -> GGUF blocks of Q4_0, Q8_0, Q4_K and Q6_K, the step the reference
// hands to llama-quantize (/root/reference/server/quantization.go:125-181), which runs ggml's scalar
// quantize_row_*_ref once per row for these four types when there is no importance matrix.  The encoders are
// defined by sequential fp32 loops (running sums in element order, a first-maximum rule, a 21- or 18-step grid
// search with "strictly better" updates); the kernels keep every one of those orders, so the bytes are those of
// the scalar code: no fused multiply-adds (the library is compiled with -ffp-contract=off), correctly rounded
// division and square root, round-to-nearest-even through the 1.5 * 2^23 add.
//
// Mapping: one lane per sub-block (the unit of the searches: 32 elements for Q4_K, 16 for Q6_K) with the
// sub-block's elements in registers; the 8 (16) lanes of a super-block then agree on the super-block scales with
// a few cross-lane reads and pack the block through LDS.  Q4_0 / Q8_0: one lane per 32-element block.  This is a
// one-off conversion, bound by the searches' arithmetic (about 10^4 operations per sub-block), not by memory.
#include <hip/hip_fp16.h>

#include "internal.h"

namespace miqmm {

namespace {

__device__ __forceinline__ int nearest_int(float f) {
    const float v = f + 12582912.f;
    return (__float_as_int(v) & 0x007fffff) - 0x00400000;
}
// (the value is pinned in a register first: left alone the compiler folds a preceding multiply into a mixed-precision
// fma with a +0 addend, which turns the -0.0 scale of an all-zero Q4_0 block into +0.0)
__device__ __forceinline__ unsigned short f2h_bits(float f) {
    asm volatile("" : "+v"(f));
    return __half_as_ushort(__float2half_rn(f));
}
__device__ __forceinline__ float h2f_bits(unsigned short h) { return __half2float(__ushort_as_half(h)); }
__device__ __forceinline__ void store_u16(uint8_t *p, unsigned v) { *reinterpret_cast<unsigned short *>(p) = (unsigned short)v; }

// ---- Q4_0 / Q8_0: one lane per block -----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void encode_q4_0_kernel(const float *__restrict__ x, uint8_t *__restrict__ out, int64_t nblocks) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float4 *x4 = reinterpret_cast<const float4 *>(x + b * QK);
    float v[QK];
#pragma unroll
    for (int j = 0; j < QK / 4; j++) {
        const float4 t = x4[j];
        v[4 * j] = t.x; v[4 * j + 1] = t.y; v[4 * j + 2] = t.z; v[4 * j + 3] = t.w;
    }
    float amax = 0.0f, vmax = 0.0f;  // the first element of largest magnitude, with its sign
#pragma unroll
    for (int j = 0; j < QK; j++)
        if (amax < fabsf(v[j])) { amax = fabsf(v[j]); vmax = v[j]; }
    const float d = vmax / -8;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint8_t *y = out + b * Q4_0_BYTES;
    store_u16(y, f2h_bits(d));
#pragma unroll
    for (int j = 0; j < QK / 2; j += 2) {
        unsigned pair = 0;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const float x0 = v[j + u] * id, x1 = v[QK / 2 + j + u] * id;
            const int xi0 = min(15, (int)(int8_t)(x0 + 8.5f)), xi1 = min(15, (int)(int8_t)(x1 + 8.5f));
            pair |= (unsigned)((xi0 | (xi1 << 4)) & 0xff) << (8 * u);
        }
        store_u16(y + 2 + j, pair);
    }
}

__global__ __launch_bounds__(256) void encode_q8_0_kernel(const float *__restrict__ x, uint8_t *__restrict__ out, int64_t nblocks) {
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float4 *x4 = reinterpret_cast<const float4 *>(x + b * QK);
    float v[QK];
#pragma unroll
    for (int j = 0; j < QK / 4; j++) {
        const float4 t = x4[j];
        v[4 * j] = t.x; v[4 * j + 1] = t.y; v[4 * j + 2] = t.z; v[4 * j + 3] = t.w;
    }
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < QK; j++) amax = fmaxf(amax, fabsf(v[j]));
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint8_t *y = out + b * Q8_0_BYTES;
    store_u16(y, f2h_bits(d));
#pragma unroll
    for (int j = 0; j < QK; j += 2) {
        const int q0 = (int)roundf(v[j] * id), q1 = (int)roundf(v[j + 1] * id);
        store_u16(y + 2 + j, (unsigned)(q0 & 0xff) | ((unsigned)(q1 & 0xff) << 8));
    }
}

// ---- Q4_K ---------------------------------------------------------------------------------------------------------
// The weighted (scale, min) search over a 16-level grid for one sub-block of 32: returns the scale, *the_min
// receives -min, L the levels.  Weights av_x + |x|; grid steps (-1 + 0.1 is + 15) / (max - min), is = 0 .. 20.
__device__ __forceinline__ float search_scale_min_32(const float (&x)[32], float av_x, uint8_t (&L)[32], float &the_min) {
    constexpr int nmax = 15, nstep = 20;
    const float rmin = -1.f, rdelta = 0.1f;
    float vmin = x[0], vmax = x[0];
    float sum_w = av_x + fabsf(x[0]);
    float sum_x = sum_w * x[0];
#pragma unroll
    for (int i = 1; i < 32; i++) {
        if (x[i] < vmin) vmin = x[i];
        if (x[i] > vmax) vmax = x[i];
        const float w = av_x + fabsf(x[i]);
        sum_w += w;
        sum_x += w * x[i];
    }
    if (vmin > 0) vmin = 0;
    if (vmax == vmin) {
#pragma unroll
        for (int i = 0; i < 32; i++) L[i] = 0;
        the_min = -vmin;
        return 0.f;
    }
    float iscale = nmax / (vmax - vmin);
    float scale = 1 / iscale;
    float best = 0;
#pragma unroll
    for (int i = 0; i < 32; i++) {
        const int l = nearest_int(iscale * (x[i] - vmin));
        L[i] = (uint8_t)max(0, min(nmax, l));
        float diff = scale * L[i] + vmin - x[i];
        diff = diff * diff;
        best += (av_x + fabsf(x[i])) * diff;
    }
#pragma unroll 1
    for (int is = 0; is <= nstep; is++) {
        iscale = (rmin + rdelta * is + nmax) / (vmax - vmin);  // (vmin: the best candidate's so far, as in the scalar loop)
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        uint8_t Laux[32];
#pragma unroll
        for (int i = 0; i < 32; i++) {
            int l = nearest_int(iscale * (x[i] - vmin));
            l = max(0, min(nmax, l));
            Laux[i] = (uint8_t)l;
            const float w = av_x + fabsf(x[i]);
            sum_l += w * l;
            sum_l2 += w * l * l;
            sum_xl += w * l * x[i];
        }
        const float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0) {
                this_min = 0;
                this_scale = sum_xl / sum_l2;
            }
            float err = 0;
#pragma unroll
            for (int i = 0; i < 32; i++) {
                float diff = this_scale * Laux[i] + this_min - x[i];
                diff = diff * diff;
                err += (av_x + fabsf(x[i])) * diff;
            }
            if (err < best) {
#pragma unroll
                for (int i = 0; i < 32; i++) L[i] = Laux[i];
                best = err;
                scale = this_scale;
                vmin = this_min;
            }
        }
    }
    the_min = -vmin;
    return scale;
}

// 8 lanes per super-block (lane j = sub-block j), 8 super-blocks per wave, 256 threads per workgroup.
__global__ __launch_bounds__(256) void encode_q4_K_kernel(const float *__restrict__ x, uint8_t *__restrict__ out, int64_t nsuper) {
    __shared__ uint8_t lds_L[32][QKK];  // the levels of the workgroup's 32 super-blocks
    const int tid = threadIdx.x, lane = tid & 63, j = tid & 7, sbl = tid >> 3;
    const int64_t sb = (int64_t)blockIdx.x * 32 + sbl;
    const bool live = sb < nsuper;
    const int64_t sbc = live ? sb : nsuper - 1;  // dead lanes redo the last super-block and store nothing
    float v[32];
    {
        const float4 *x4 = reinterpret_cast<const float4 *>(x + sbc * QKK + 32 * j);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float4 t = x4[i];
            v[4 * i] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
        }
    }
    float sum_x2 = 0;
#pragma unroll
    for (int l = 0; l < 32; l++) sum_x2 += v[l] * v[l];
    const float av_x = sqrtf(sum_x2 / 32);
    uint8_t L[32];
    float mn;
    const float sc = search_scale_min_32(v, av_x, L, mn);
    // the super-block's largest scale and min: a maximum over eight values, whatever the order
    float max_scale = 0, max_min = 0;
#pragma unroll
    for (int t = 0; t < 8; t++) {
        const float s = __shfl(sc, (lane & ~7) + t, 64), m = __shfl(mn, (lane & ~7) + t, 64);
        if (s > max_scale) max_scale = s;
        if (m > max_min) max_min = m;
    }
    const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
    const float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
    const int ls = min(63, (int)(uint8_t)nearest_int(inv_scale * sc));
    const int lm = min(63, (int)(uint8_t)nearest_int(inv_min * mn));
    const unsigned short dh = f2h_bits(max_scale / 63.f), dmh = f2h_bits(max_min / 63.f);
    const float d = h2f_bits(dh) * ls;
    if (d != 0.0f) {  // (otherwise the levels of the search stay)
        const float dm = h2f_bits(dmh) * lm;
#pragma unroll
        for (int i = 0; i < 32; i++) {
            const int l = nearest_int((v[i] + dm) / d);
            L[i] = (uint8_t)max(0, min(15, l));
        }
    }
#pragma unroll
    for (int i = 0; i < 32; i += 4)
        *reinterpret_cast<unsigned *>(&lds_L[sbl][32 * j + i]) = L[i] | (L[i + 1] << 8) | (L[i + 2] << 16) | ((unsigned)L[i + 3] << 24);
    // the 12 scale bytes: lanes gather all eight (ls, lm)
    unsigned lsv[8], lmv[8];
#pragma unroll
    for (int t = 0; t < 8; t++) {
        lsv[t] = (unsigned)__shfl(ls, (lane & ~7) + t, 64);
        lmv[t] = (unsigned)__shfl(lm, (lane & ~7) + t, 64);
    }
    __syncthreads();
    if (!live) return;
    uint8_t *y = out + sb * Q4_K_BYTES;
    if (j == 0) {
        unsigned w[3] = {0, 0, 0};  // scales[0..3], scales[4..7], scales[8..11]
#pragma unroll
        for (int t = 0; t < 4; t++) {
            w[0] |= (lsv[t] | ((lsv[t + 4] >> 4) << 6)) << (8 * t);
            w[1] |= (lmv[t] | ((lmv[t + 4] >> 4) << 6)) << (8 * t);
            w[2] |= ((lsv[t + 4] & 0xF) | ((lmv[t + 4] & 0xF) << 4)) << (8 * t);
        }
        unsigned *y32 = reinterpret_cast<unsigned *>(y);
        y32[0] = (unsigned)dh | ((unsigned)dmh << 16);
        y32[1] = w[0]; y32[2] = w[1]; y32[3] = w[2];
    }
    // qs: 64 elements -> 32 bytes (low nibble: the first 32, high nibble: the next 32); lane j writes 16 bytes
    {
        const int grp = j >> 1, half = j & 1;  // bytes [32 grp + 16 half, +16)
        unsigned *y32 = reinterpret_cast<unsigned *>(y + 16 + 32 * grp + 16 * half);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const unsigned lo = *reinterpret_cast<const unsigned *>(&lds_L[sbl][64 * grp + 16 * half + 4 * i]);
            const unsigned hi = *reinterpret_cast<const unsigned *>(&lds_L[sbl][64 * grp + 32 + 16 * half + 4 * i]);
            y32[i] = lo | (hi << 4);
        }
    }
}

// ---- Q6_K ---------------------------------------------------------------------------------------------------------
// The symmetric search over a 64-level grid for one sub-block of 16 (weights x^2): returns the scale, L the levels + 32.
__device__ __forceinline__ float search_scale_16(const float (&x)[16], int8_t (&L)[16]) {
    constexpr int nmax = 32;
    float vmax = 0, amax = 0;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; vmax = x[i]; }
    }
    if (amax < 1e-15f) {
#pragma unroll
        for (int i = 0; i < 16; i++) L[i] = 0;
        return 0.f;
    }
    float iscale = -nmax / vmax;
    float sumlx = 0, suml2 = 0;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        int l = nearest_int(iscale * x[i]);
        l = max(-nmax, min(nmax - 1, l));
        L[i] = (int8_t)(l + nmax);
        const float w = x[i] * x[i];
        sumlx += w * x[i] * l;
        suml2 += w * l * l;
    }
    float scale = suml2 != 0.0f ? sumlx / suml2 : 0.0f;
    float best = scale * sumlx;
#pragma unroll 1
    for (int is = -9; is <= 9; is++) {
        if (is == 0) continue;
        iscale = -(nmax + 0.1f * is) / vmax;
        sumlx = suml2 = 0;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            int l = nearest_int(iscale * x[i]);
            l = max(-nmax, min(nmax - 1, l));
            const float w = x[i] * x[i];
            sumlx += w * x[i] * l;
            suml2 += w * l * l;
        }
        if (suml2 > 0 && sumlx * sumlx > best * suml2) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int l = nearest_int(iscale * x[i]);
                L[i] = (int8_t)(nmax + max(-nmax, min(nmax - 1, l)));
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

// 16 lanes per super-block (lane j = sub-block j), 4 super-blocks per wave, 256 threads per workgroup.
__global__ __launch_bounds__(256) void encode_q6_K_kernel(const float *__restrict__ x, uint8_t *__restrict__ out, int64_t nsuper) {
    __shared__ int8_t lds_L[16][QKK];
    const int tid = threadIdx.x, lane = tid & 63, j = tid & 15, sbl = tid >> 4;
    const int64_t sb = (int64_t)blockIdx.x * 16 + sbl;
    const bool live = sb < nsuper;
    const int64_t sbc = live ? sb : nsuper - 1;
    float v[16];
    {
        const float4 *x4 = reinterpret_cast<const float4 *>(x + sbc * QKK + 16 * j);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float4 t = x4[i];
            v[4 * i] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
        }
    }
    int8_t L[16];
    const float scale = search_scale_16(v, L);
    // the first sub-block scale of largest magnitude, with its sign
    float max_scale = 0, max_abs_scale = 0;
#pragma unroll
    for (int t = 0; t < 16; t++) {
        const float s = __shfl(scale, (lane & ~15) + t, 64);
        const float as = fabsf(s);
        if (as > max_abs_scale) { max_abs_scale = as; max_scale = s; }
    }
    const bool empty = max_abs_scale < 1e-15f;  // the whole block is zero bytes
    const float iscale = -128.f / max_scale;
    const unsigned short dh = f2h_bits(1 / iscale);
    const int sc8 = min(127, nearest_int(iscale * scale));
    const float d = h2f_bits(dh) * (float)(int8_t)sc8;
    if (!empty && d != 0.0f) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            int l = nearest_int(v[i] / d);
            l = max(-32, min(31, l));
            L[i] = (int8_t)(l + 32);
        }
    }
#pragma unroll
    for (int i = 0; i < 16; i += 4)
        *reinterpret_cast<unsigned *>(&lds_L[sbl][16 * j + i]) =
            (unsigned)(uint8_t)L[i] | ((unsigned)(uint8_t)L[i + 1] << 8) | ((unsigned)(uint8_t)L[i + 2] << 16) | ((unsigned)(uint8_t)L[i + 3] << 24);
    const int sc_next = __shfl(sc8, (lane & ~15) + ((j + 1) & 15), 64);  // (for the 16-bit stores of the scale bytes)
    __syncthreads();
    if (!live) return;
    uint8_t *y = out + sb * Q6_K_BYTES;  // ql 128, qh 64, scales 16, d 2: two-byte aligned
    // lane j packs elements l = 2 (j & 15) .. +1 of both 128-element halves: 2 x (ql[l], ql[l + 32], qh[l]) byte pairs
    const uint8_t *Ls = reinterpret_cast<const uint8_t *>(lds_L[sbl]);
#pragma unroll
    for (int h = 0; h < 2; h++) {
        unsigned qa = 0, qb = 0, qq = 0;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int l = 2 * j + u, base = 128 * h + l;
            const unsigned L1 = empty ? 0 : Ls[base], L2 = empty ? 0 : Ls[base + 32], L3 = empty ? 0 : Ls[base + 64], L4 = empty ? 0 : Ls[base + 96];
            qa |= ((L1 & 0xF) | ((L3 & 0xF) << 4)) << (8 * u);
            qb |= ((L2 & 0xF) | ((L4 & 0xF) << 4)) << (8 * u);
            qq |= ((L1 >> 4) | ((L2 >> 4) << 2) | ((L3 >> 4) << 4) | ((L4 >> 4) << 6)) << (8 * u);
        }
        store_u16(y + 64 * h + 2 * j, qa);
        store_u16(y + 64 * h + 32 + 2 * j, qb);
        store_u16(y + 128 + 32 * h + 2 * j, qq);
    }
    if ((j & 1) == 0) store_u16(y + 192 + j, empty ? 0 : ((unsigned)(sc8 & 0xff) | ((unsigned)(sc_next & 0xff) << 8)));
    if (j == 0) store_u16(y + 208, empty ? 0 : dh);
}

}  // namespace

bool encode_supported(int type, int64_t K) {
    switch (type) {
    case T_Q4_0: case T_Q8_0: return K > 0 && K % QK == 0;
    case T_Q4_K: case T_Q6_K: return K > 0 && K % QKK == 0;
    default: return false;
    }
}

hipError_t launch_encode_weights(int type, const float *x, int64_t K, int64_t M, uint8_t *out, hipStream_t s) {
    if (!encode_supported(type, K) || M < 0) return hipErrorInvalidValue;
    if (M == 0) return hipSuccess;
    const int64_t units = M * (K / (type == T_Q4_0 || type == T_Q8_0 ? QK : QKK));
    const int64_t per_wg = type == T_Q4_K ? 32 : type == T_Q6_K ? 16 : 256;
    const int64_t grid = (units + per_wg - 1) / per_wg;
    if (grid > 0x7fffffff) return hipErrorInvalidValue;
    switch (type) {
    case T_Q4_0: encode_q4_0_kernel<<<(unsigned)grid, 256, 0, s>>>(x, out, units); break;
    case T_Q8_0: encode_q8_0_kernel<<<(unsigned)grid, 256, 0, s>>>(x, out, units); break;
    case T_Q4_K: encode_q4_K_kernel<<<(unsigned)grid, 256, 0, s>>>(x, out, units); break;
    default: encode_q6_K_kernel<<<(unsigned)grid, 256, 0, s>>>(x, out, units); break;
    }
    return hipGetLastError();
}

}  // namespace miqmm
