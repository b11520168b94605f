// Producers of the activations: the two steps that sit in front of a quantized product in a transformer
// block, computed on the fly by whoever quantizes x so that their f32 result never goes through HBM.
//   RMSNorm (Tensor.RMSNorm, /root/reference/ml/backend.go:159; ggml's rms_norm followed by the broadcast
//            multiply with the norm weight):  x' = (x * scale) * g,  scale = 1 / sqrtf(mean(x^2) + eps)
//   SwiGLU  (Tensor.SILU with an "up" operand, /root/reference/ml/backend.go:180; ggml's swiglu):
//            x' = silu(x) * up,  silu(v) = v / (1 + expf(-v))
// CPU semantics restated: squares formed in fp32 and accumulated in double, the mean rounded to fp32,
// sqrtf and the divisions correctly rounded, the two multiplies of RMSNorm rounded separately.  The sum of
// squares is taken in one fixed order whatever the launch geometry -- element order inside a lane, a
// butterfly over the 64 lanes of a 256-element piece, then piece after piece -- so every kernel that
// produces a row gives the same bits.  Files that include this are compiled with -ffp-contract=off.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace miqmm {

enum { PRODUCE_NONE = 0, PRODUCE_RMSNORM = 1, PRODUCE_SWIGLU = 2 };

// what a quantizer applies to x before it quantizes
struct Produce {
    int kind;                // PRODUCE_*
    const float *aux;        // RMSNORM: the norm weight g [K] or null; SWIGLU: up, same shape as x
    float eps;               // RMSNORM
    const float *row_scale;  // RMSNORM in the stand-alone quantizers: scale per row, from launch_rms_scale
};

// v from the lane the DPP control names, 0.0 in lanes whose row is masked out
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ double dpp_d(double v) {
    const long long b = __double_as_longlong(v);
    const unsigned lo = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)b, CTRL, ROW_MASK, 0xf, false);
    const unsigned hi = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)((unsigned long long)b >> 32), CTRL, ROW_MASK, 0xf, false);
    return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

// Sum of the squares of the 256 elements a wave holds four per lane; every lane returns the total.
// Data-parallel-primitive exchanges (a few cycles each, no LDS round trip): pairs, quads, groups of 8, rows of
// 16, then row 0 into row 1 and row 2 into row 3, rows 0+1 into row 3; lane 63 holds the total.
__device__ __forceinline__ double piece_sumsq(const float4 v) {
    double s = (double)(v.x * v.x);
    s += (double)(v.y * v.y);
    s += (double)(v.z * v.z);
    s += (double)(v.w * v.w);
    s += dpp_d<0xB1>(s);         // quad_perm [1,0,3,2]
    s += dpp_d<0x4E>(s);         // quad_perm [2,3,0,1]
    s += dpp_d<0x141>(s);        // lane i <-> 7-i inside each group of 8
    s += dpp_d<0x140>(s);        // lane i <-> 15-i inside each row of 16
    s += dpp_d<0x142, 0xa>(s);   // lane 15 of rows 0 and 2 into rows 1 and 3
    s += dpp_d<0x143, 0xc>(s);   // lane 31 into rows 2 and 3
    const long long b = __double_as_longlong(s);
    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)b, 63);
    const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)((unsigned long long)b >> 32), 63);
    return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

__device__ __forceinline__ float rms_scale_of(double sumsq, int64_t K, float eps) {
    const float mean = (float)(sumsq / (double)K);
    return 1.0f / sqrtf(mean + eps);
}

__device__ __forceinline__ float4 rms_apply(const float4 v, float scale, const float4 g, bool has_g) {
    float4 r = make_float4(v.x * scale, v.y * scale, v.z * scale, v.w * scale);
    if (has_g) { r.x *= g.x; r.y *= g.y; r.z *= g.z; r.w *= g.w; }
    return r;
}

__device__ __forceinline__ float silu(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float silu_mul(float v, float up) { return silu(v) * up; }

__device__ __forceinline__ float4 swiglu_apply(const float4 v, const float4 up) {
    return make_float4(silu_mul(v.x, up.x), silu_mul(v.y, up.y), silu_mul(v.z, up.z), silu_mul(v.w, up.w));
}

}  // namespace miqmm
