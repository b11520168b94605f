// Device-side block quantizers shared by the stand-alone activation-quantization kernel and the
// decode GEMV that quantizes its f32 activations in its own prologue.
//
// Semantics are the scalar CPU quantizers' (quantize_row_q8_0_ref / quantize_row_q8_K_ref of ggml,
// the from_float step of the CPU mul_mat that Tensor.Mulmat -- /root/reference/ml/backend.go:151 --
// ends in); the values produced are identical to the CPU's:
//   Q8_0: amax over 32; d = amax/127 (IEEE fp32 divide); id = d ? 1/d : 0; q = roundf(x*id)
//         (half away from zero); stored scale = fp16_rne(d).
//   Q8_K: first element of largest |x| over 256, with its sign: max; iscale = -127/max;
//         q = min(127, rne(iscale*x)) on the fp32-rounded product; bsums = sums of 16; d = 1/iscale.
//         An all-zero block is all zero bytes.
// Every file that includes this is compiled with -ffp-contract=off: none of the expressions above may
// be fused.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

namespace miqmm {

__device__ __forceinline__ int pack4_i8(int a, int b, int c, int d) {
    return (a & 0xff) | ((b & 0xff) << 8) | ((c & 0xff) << 16) | ((d & 0xff) << 24);
}

// Cross-lane exchanges on the data-parallel-primitive path (no LDS round trip, a few cycles each).
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ int dpp_i(int old, int v) {
    return __builtin_amdgcn_update_dpp(old, v, CTRL, ROW_MASK, 0xf, false);
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_f(float old, float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
constexpr int DPP_XOR1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int DPP_XOR2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int DPP_HALF_MIRROR = 0x141; // lane i <-> 7-i inside each group of 8
constexpr int DPP_MIRROR = 0x140;      // lane i <-> 15-i inside each row of 16
constexpr int DPP_BCAST15 = 0x142;     // lane 15 of each row into the next row
constexpr int DPP_BCAST31 = 0x143;     // lane 31 into rows 2 and 3

// Q8_0: eight consecutive lanes (aligned group of 8) hold the 32 elements of a block, four each.
// Every lane calls this (dead lanes with zeros).  Returns the lane's four quants packed; d is the
// fp16-rounded scale widened to fp32 and sum the block's quant sum, both valid in all eight lanes.
__device__ __forceinline__ int q8_0_quantize_lane(const float4 v, float &d, int &sum) {
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = fmaxf(amax, dpp_f<DPP_XOR1>(amax, amax));
    amax = fmaxf(amax, dpp_f<DPP_XOR2>(amax, amax));
    amax = fmaxf(amax, dpp_f<DPP_HALF_MIRROR>(amax, amax));  // the quads now hold one value each
    const float dd = amax / 127.0f;
    const float id = dd != 0.0f ? 1.0f / dd : 0.0f;
    const int q0 = (int)roundf(v.x * id), q1 = (int)roundf(v.y * id);
    const int q2 = (int)roundf(v.z * id), q3 = (int)roundf(v.w * id);
    int s = q0 + q1 + q2 + q3;
    s += dpp_i<DPP_XOR1>(0, s);
    s += dpp_i<DPP_XOR2>(0, s);
    s += dpp_i<DPP_HALF_MIRROR>(0, s);
    sum = s;
    d = __half2float(__float2half_rn(dd));  // the scale the CPU stores and later reads
    return pack4_i8(q0, q1, q2, q3);
}

// Q8_K: the 64 lanes of a wave hold the 256 elements of a super-block, four each (lane l has
// elements 4l .. 4l+3).  Returns the lane's four quants packed; d is valid in every lane;
// sum16 is bsums[l/4] in every lane (the sum over the lane's group of 16 elements) and
// pair32 = bsums[2j] + bsums[2j+1] for j = l/8.
// "First element of largest magnitude": the wave maximum of |x| is exact whatever the order of the
// reduction; the lowest lane that holds it (ballot + find-first) holds the lowest such index, and that
// lane's own scan kept its first such element.
__device__ __forceinline__ int q8_K_quantize_lane(const float4 v, int lane, float &d, int &sum16, int &pair32) {
    float amax = 0.0f, mx = 0.0f;
    const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float ax = fabsf(e[i]);
        if (ax > amax) { amax = ax; mx = e[i]; }
    }
    float wmax = fmaxf(amax, dpp_f<DPP_XOR1>(amax, amax));
    wmax = fmaxf(wmax, dpp_f<DPP_XOR2>(wmax, wmax));
    wmax = fmaxf(wmax, dpp_f<DPP_HALF_MIRROR>(wmax, wmax));
    wmax = fmaxf(wmax, dpp_f<DPP_MIRROR>(wmax, wmax));            // every lane of a row: the row's maximum
    wmax = fmaxf(wmax, dpp_f<DPP_BCAST15, 0xa>(wmax, wmax));      // rows 1 and 3: max with the row before
    wmax = fmaxf(wmax, dpp_f<DPP_BCAST31, 0xc>(wmax, wmax));      // row 3: the wave's maximum
    wmax = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wmax), 63));
    int q[4] = {0, 0, 0, 0};
    float dd = 0.0f;
    if (wmax != 0.0f) {  // wave-uniform
        const unsigned long long holders = __ballot(amax == wmax);
        const int first = __ffsll((long long)holders) - 1;
        const float wmx = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(mx), first));
        const float iscale = -127.0f / wmx;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float p = iscale * e[i];
            q[i] = min(127, (int)rintf(p));
        }
        dd = 1.0f / iscale;
    }
    int s = q[0] + q[1] + q[2] + q[3];
    s += dpp_i<DPP_XOR1>(0, s);
    s += dpp_i<DPP_XOR2>(0, s);
    sum16 = s;
    pair32 = s + dpp_i<DPP_HALF_MIRROR>(0, s);
    d = dd;
    return pack4_i8(q[0], q[1], q[2], q[3]);
}

// Q8_K with a quarter of a wave per super-block: the 16 lanes of a DPP row hold the 256 elements of a block, sixteen
// consecutive ones each (lane l of the row has elements 16l .. 16l+15), so a wave quantizes four blocks at once and
// the cross-lane steps are four row exchanges instead of eight over the wave: about 45 vector instructions per block
// against 75 -- what the decode GEMV's prologue is made of.  The same values as q8_K_quantize_lane (the maximum is
// exact whatever the order; the first element that holds it is the lowest such index of the lowest such lane).
// Returns the lane's sixteen quants; d is valid in every lane of the row; sum16 = bsums[l] is the lane's own sum and
// pair32 = bsums[2j] + bsums[2j+1] for j = l/2.
// qfl (optional): the sixteen quants as floats (exact), for callers that also write them out as fp16.
__device__ __forceinline__ uint4 q8_K_quantize_row16(const float4 (&v)[4], int lane, float &d, int &sum16, int &pair32,
                                                     float *qfl = nullptr) {
    const float e[16] = {v[0].x, v[0].y, v[0].z, v[0].w, v[1].x, v[1].y, v[1].z, v[1].w,
                         v[2].x, v[2].y, v[2].z, v[2].w, v[3].x, v[3].y, v[3].z, v[3].w};
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i++) amax = fmaxf(amax, fabsf(e[i]));
    float wmax = fmaxf(amax, dpp_f<DPP_XOR1>(amax, amax));
    wmax = fmaxf(wmax, dpp_f<DPP_XOR2>(wmax, wmax));
    wmax = fmaxf(wmax, dpp_f<DPP_HALF_MIRROR>(wmax, wmax));
    wmax = fmaxf(wmax, dpp_f<DPP_MIRROR>(wmax, wmax));  // every lane of the row: the block's maximum
    float mine = 0.0f;  // this lane's first element of that magnitude, if it has one
#pragma unroll
    for (int i = 15; i >= 0; i--) mine = fabsf(e[i]) == wmax ? e[i] : mine;
    const unsigned long long holders = __ballot(amax == wmax);
    const unsigned in_row = (unsigned)(holders >> (lane & 48)) & 0xffffu;  // never empty: some lane of the row holds its maximum
    const int first = (lane & 48) + __ffs((int)in_row) - 1;
    const float wmx = __int_as_float(__builtin_amdgcn_ds_bpermute(4 * first, __float_as_int(mine)));
    const bool any = wmax != 0.0f;
    const float iscale = any ? -127.0f / wmx : 0.0f;  // an all-zero block: every product is (signed) zero, every quant 0
    // q = min(127, rne(p)), p = the fp32-rounded product iscale * e.  |p| <= fl(fl(127 / |max|) * |max|), which is 127
    // or the next float above it, so the min never acts; and for |p| < 2^22 adding 1.5 * 2^23 rounds p to the nearest
    // integer, ties to even, and leaves it in the low mantissa bits: t = p + magic, q = bits(t) - bits(magic), the
    // low byte of bits(t) is the quant's byte.  (The product is rounded before the add: no contraction in this file.)
    const float magic = 12582912.0f;
    unsigned t[16], us = 0;  // (unsigned: the sum of sixteen bit patterns wraps before bits(magic) comes off again)
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float r = iscale * e[i] + magic;
        t[i] = __float_as_uint(r);
        us += t[i];
        if (qfl) qfl[i] = r - magic;  // exact: both are integers below 2^24
    }
    const int s = (int)(us - 16u * 0x4B400000u);  // bits(magic) = 0x4B400000
    sum16 = s;
    pair32 = s + dpp_i<DPP_XOR1>(0, s);
    d = any ? 1.0f / iscale : 0.0f;
    uint4 out;
    unsigned *o = &out.x;
#pragma unroll
    for (int j = 0; j < 4; j++) {  // the low bytes of four words
        const unsigned lo = __builtin_amdgcn_perm(t[4 * j + 1], t[4 * j], 0x0c0c0400u);      // [t0.b0, t1.b0, 0, 0]
        const unsigned hi = __builtin_amdgcn_perm(t[4 * j + 3], t[4 * j + 2], 0x04000c0cu);  // [0, 0, t2.b0, t3.b0]
        o[j] = lo | hi;
    }
    return out;
}

}  // namespace miqmm
