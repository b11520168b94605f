// Measurement aid for bench.py, not part of the product library: what rate do the matrix cores of this machine
// sustain when they do nothing else?  Every wave runs a loop of independent MFMAs (four accumulators, so one can
// issue every 32 cycles) on operands that differ from lane to lane and from one MFMA to the next -- random bits, or
// values distributed like the prefill kernels' operands; with constant operands the same loop runs close to the
// nominal peak.  Two
// waves per SIMD on every CU, a few milliseconds per launch: long enough for power management to settle the clock.
// bench.py shows the prefill GEMM's figures next to this rate: it is the practical ceiling of an MFMA-bound kernel
// here, as the pure-read launch is for the HBM-bound ones.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

__device__ __forceinline__ unsigned lcg(unsigned &st) {
    st = st * 1664525u + 1013904223u;
    return st;
}
// roughly normal, mean 0 and deviation 1: the sum of four uniform bytes
__device__ __forceinline__ float normalish(unsigned &st) {
    const unsigned x = lcg(st);
    const int sum = (int)(x & 255) + (int)((x >> 8) & 255) + (int)((x >> 16) & 255) + (int)(x >> 24);
    return (float)(sum - 510) * (1.0f / 147.8f);
}
// an activation as the Q8_K quantizer leaves it (127 at about three deviations) and a Q4_K weight: nibble around
// the middle of its range, times a six-bit block scale
__device__ __forceinline__ int real_act(unsigned &st) { return max(-127, min(127, (int)rintf(42.f * normalish(st)))); }
__device__ __forceinline__ int real_nibble(unsigned &st) { return max(0, min(15, (int)rintf(7.5f + 2.7f * normalish(st)))); }
__device__ __forceinline__ unsigned half_bits(float v) { return (unsigned)__builtin_bit_cast(unsigned short, (_Float16)v); }

// KIND 0: v_mfma_f32_32x32x16_f16 (32768 flop) on random bits, 1: v_mfma_i32_32x32x32_i8 (65536 op) on random bits;
// 2 and 3: the same two instructions on operands drawn like the prefill kernels' -- activations quantized from a
// normal distribution against (block scale * nibble) * 2^-14 as fp16, or against bare nibbles for int8.  Fewer bits
// toggle per operand than with random ones, which is what the power-limited clock responds to.
template <int KIND>
__global__ __launch_bounds__(256, 2) void mfma_rate_kernel(float *__restrict__ out, long long *__restrict__ clk, int iters, int seed) {
    v4i ra[8], rb[8];
    unsigned st = seed * 2654435761u + threadIdx.x * 40503u + blockIdx.x * 69069u;
    for (int j = 0; j < 8; j++)
        for (int i = 0; i < 4; i++) {
            if (KIND == 0) {  // fp16 values in [64, 128) and +-[0.125, 0.25): no overflow however long the loop
                const unsigned x1 = lcg(st), x2 = lcg(st);
                ra[j][i] = (int)((x1 & 0x03ff03ffu) | 0x54005400u);
                rb[j][i] = (int)((x2 & 0x83ff83ffu) | 0x30003000u);
            } else if (KIND == 1) {
                const unsigned x1 = lcg(st), x2 = lcg(st);
                ra[j][i] = (int)x1;
                rb[j][i] = (int)(x2 & 0x0f0f0f0fu);
            } else if (KIND == 2) {
                const unsigned sc = 20u + (lcg(st) >> 27);  // one block scale for the pair: 20..51
                const unsigned a0 = half_bits((float)real_act(st)), a1 = half_bits((float)real_act(st));
                const unsigned b0 = half_bits((float)(sc * real_nibble(st)) * (1.f / 16384.f));
                const unsigned b1 = half_bits((float)(sc * real_nibble(st)) * (1.f / 16384.f));
                ra[j][i] = (int)(a0 | (a1 << 16));
                rb[j][i] = (int)(b0 | (b1 << 16));
            } else {
                unsigned a = 0, b = 0;
                for (int k = 0; k < 4; k++) {
                    a |= (unsigned)(real_act(st) & 255) << (8 * k);
                    b |= (unsigned)real_nibble(st) << (8 * k);
                }
                ra[j][i] = (int)a;
                rb[j][i] = (int)b;
            }
        }
    v16f c[4];
    v16i d[4];
    for (int x = 0; x < 4; x++)
        for (int i = 0; i < 16; i++) { c[x][i] = 0.f; d[x][i] = 0; }
    const long long c0 = clock64(), r0 = wall_clock64();
#pragma unroll 2
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int x = 0; x < 4; x++) {
            const int ia = (2 * x + (it & 1)) & 7, ib = (2 * x + 1 + (it & 1)) & 7;
            if (KIND == 0 || KIND == 2) c[x] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, ra[ia]), __builtin_bit_cast(v8h, rb[ib]), c[x], 0, 0, 0);
            else d[x] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ra[ia], rb[ib], d[x], 0, 0, 0);
        }
    }
    const long long c1 = clock64(), r1 = wall_clock64();
    float s = 0;
    for (int x = 0; x < 4; x++)
        for (int i = 0; i < 16; i++) s += c[x][i] + (float)d[x][i];
    if (s == 12345.678f) out[threadIdx.x] = s;  // keeps the loop alive
    if (threadIdx.x == 0 && blockIdx.x == 0) {  // shader cycles and 100 MHz ticks of workgroup 0: the clock it ran at
        clk[0] = c1 - c0;
        clk[1] = r1 - r0;
    }
}

}  // namespace

// Queues one launch of `blocks` workgroups (4 waves each) that issue 4 * iters MFMAs per wave.  kind 0: fp16
// 32x32x16 on random bits, 1: int8 32x32x32 on random bits, 2 / 3: the same on operands distributed like the prefill
// kernels'.  out: device scratch of 256 floats; clk: device, two int64 (shader cycles and 100 MHz ticks that
// workgroup 0 spent in its loop).
extern "C" int mi_mfma_rate(int kind, int iters, int blocks, float *out, long long *clk, void *stream) {
    if (!out || !clk || iters < 1 || blocks < 1 || kind < 0 || kind > 3) return -1;
    hipStream_t s = (hipStream_t)stream;
    if (kind == 0) mfma_rate_kernel<0><<<blocks, 256, 0, s>>>(out, clk, iters, 1);
    else if (kind == 1) mfma_rate_kernel<1><<<blocks, 256, 0, s>>>(out, clk, iters, 1);
    else if (kind == 2) mfma_rate_kernel<2><<<blocks, 256, 0, s>>>(out, clk, iters, 1);
    else mfma_rate_kernel<3><<<blocks, 256, 0, s>>>(out, clk, iters, 1);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}
