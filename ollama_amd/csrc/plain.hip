// Mulmat on the unquantized weight types of a GGUF file: F32, F16 and BF16 (the file types F32 / F16 / BF16 of
// /root/reference/fs/ggml/type.go:55-88, the tensors a K-quant file keeps unquantized, and the ones the reference keeps
// at f16 on purpose: /root/reference/server/quantization.go:296-333).
//
// Semantics: the ggml CPU backend's.  The f32 activations are converted to the weight's own type (F16: IEEE round to
// nearest even; BF16: round to nearest even on the upper 16 bits; F32: as they are), both operands are widened to fp32
// and multiplied there; a product of two halves or two bfloat16 is exact in fp32.  The CPU adds the products in double,
// the kernels here in fp32 (lane partial sums, then a tree over the lanes; the matrix cores' own order in the GEMM):
// the difference is rounding of fp32 sums, orders of magnitude inside the path's 1e-3 tolerance.
//
// Four kernels:
//   plain_skinny_kernel 1..16 activation columns whose converted form fits the LDS, bound by HBM: weights straight from
//                       HBM into the operands of 16 x 16 MFMAs, a ring of eight 16-byte loads in flight per lane.
//   plain_gemv_kernel   1..8 columns of anything else with rows of whole 16-byte pieces: a wave streams two weight rows
//                       at a time, vector ALU, the converted activations in LDS chunk by chunk.
//   plain_gemm_kernel   more columns: 128 x 128 (or 128 x 32) output tiles on v_mfma_f32_32x32x16_{f16,bf16} /
//                       v_mfma_f32_32x32x2_f32, operands staged through LDS in two buffers, from activations converted
//                       once by plain_convert_kernel.
//   plain_naive_kernel  rows whose byte length is no multiple of 16 (K odd ...): a wave per output, element loads.
#include <algorithm>
#include <type_traits>

#include "internal.h"

namespace miqmm {

namespace {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ unsigned f32_bits(float f) { return __builtin_bit_cast(unsigned, f); }
__device__ __forceinline__ float bits_f32(unsigned u) { return __builtin_bit_cast(float, u); }

// f32 -> the 16-bit pattern of the weight's type
template <int TYPE>
__device__ __forceinline__ unsigned short narrow16(float f) {
    if (TYPE == T_F16) return __builtin_bit_cast(unsigned short, (_Float16)f);
    const unsigned u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 64);
    return (unsigned short)((u + (0x7fffu + ((u >> 16) & 1u))) >> 16);
}
// the two 16-bit values of a dword, widened
template <int TYPE>
__device__ __forceinline__ void widen2(unsigned u, float &lo, float &hi) {
    if (TYPE == T_F16) {
        lo = (float)__builtin_bit_cast(_Float16, (unsigned short)(u & 0xffffu));
        hi = (float)__builtin_bit_cast(_Float16, (unsigned short)(u >> 16));
    } else {
        lo = bits_f32(u << 16);
        hi = bits_f32(u & 0xffff0000u);
    }
}
// a 16-byte piece of a row as floats: E = 8 (16-bit types) or 4 (F32)
template <int TYPE>
__device__ __forceinline__ void widen_piece(const v4u &p, float *f) {
    if (TYPE == T_F32) {
        f[0] = bits_f32(p.x); f[1] = bits_f32(p.y); f[2] = bits_f32(p.z); f[3] = bits_f32(p.w);
    } else {
        widen2<TYPE>(p.x, f[0], f[1]); widen2<TYPE>(p.y, f[2], f[3]);
        widen2<TYPE>(p.z, f[4], f[5]); widen2<TYPE>(p.w, f[6], f[7]);
    }
}

template <int TYPE>
__global__ __launch_bounds__(256) void plain_convert_kernel(const float *__restrict__ x, unsigned short *__restrict__ out, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) out[i] = narrow16<TYPE>(x[i]);
}

// ---- 1..8 columns -------------------------------------------------------------------------------------------------
// Workgroup of 16 waves; a round is 32 consecutive rows, two per wave.  K is walked in chunks of KC elements (KC a
// multiple of 128 * E; one chunk where all of K fits, and then the activations are staged once for the whole launch).
// Requires (K * ES) % 16 == 0.  LDS: NC * min(K, KC) elements of the weight's type.
constexpr int GEMV_WAVES = 16;
template <int TYPE, int NC>
__global__ __launch_bounds__(64 * GEMV_WAVES) void plain_gemv_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x,
                                                                     float *__restrict__ y, int K, int64_t M, int KC) {
    constexpr int ES = TYPE == T_F32 ? 4 : 2, E = 16 / ES;
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nchunks = (K + KC - 1) / KC;
    const int64_t rounds = (M + 31) / 32;
    const int64_t row_bytes = (int64_t)K * ES;
    bool staged = false;
    for (int64_t round = blockIdx.x; round < rounds; round += gridDim.x) {
        const int64_t r0 = round * 32 + 2 * wave;
        const bool live = r0 < M;
        const int64_t r1 = r0 + 1 < M ? r0 + 1 : (live ? r0 : 0);
        const uint8_t *w0 = w + (live ? r0 : 0) * row_bytes, *w1 = w + r1 * row_bytes;
        float acc0[NC], acc1[NC];
#pragma unroll
        for (int c = 0; c < NC; c++) acc0[c] = acc1[c] = 0.0f;
        for (int ch = 0; ch < nchunks; ch++) {
            const int k0 = ch * KC, len = K - k0 < KC ? K - k0 : KC;
            if (nchunks > 1 || !staged) {
                if (staged) __syncthreads();  // every wave is through with the chunk that is about to be replaced
                for (int c = 0; c < NC; c++)
                    for (int i = tid; i < len; i += 64 * GEMV_WAVES) {
                        const float v = x[(int64_t)c * K + k0 + i];
                        if (TYPE == T_F32) reinterpret_cast<float *>(xs)[c * KC + i] = v;
                        else reinterpret_cast<unsigned short *>(xs)[c * KC + i] = narrow16<TYPE>(v);
                    }
                staged = true;
                __syncthreads();
            }
            if (!live) continue;
            const uint8_t *p0 = w0 + (int64_t)k0 * ES, *p1 = w1 + (int64_t)k0 * ES;
            for (int e = lane * E; e < len; e += 128 * E) {
                const int e2 = e + 64 * E;
                const bool two = e2 < len;
                const v4u a0 = *reinterpret_cast<const v4u *>(p0 + (int64_t)e * ES);
                const v4u b0 = *reinterpret_cast<const v4u *>(p1 + (int64_t)e * ES);
                v4u a1 = {0, 0, 0, 0}, b1 = {0, 0, 0, 0};
                if (two) {
                    a1 = *reinterpret_cast<const v4u *>(p0 + (int64_t)e2 * ES);
                    b1 = *reinterpret_cast<const v4u *>(p1 + (int64_t)e2 * ES);
                }
                float fa[E], fb[E], fx[E];
                widen_piece<TYPE>(a0, fa);
                widen_piece<TYPE>(b0, fb);
#pragma unroll
                for (int c = 0; c < NC; c++) {
                    widen_piece<TYPE>(*reinterpret_cast<const v4u *>(xs + ((int64_t)c * KC + e) * ES), fx);
#pragma unroll
                    for (int j = 0; j < E; j++) {
                        acc0[c] = __builtin_fmaf(fa[j], fx[j], acc0[c]);
                        acc1[c] = __builtin_fmaf(fb[j], fx[j], acc1[c]);
                    }
                }
                if (two) {
                    widen_piece<TYPE>(a1, fa);
                    widen_piece<TYPE>(b1, fb);
#pragma unroll
                    for (int c = 0; c < NC; c++) {
                        widen_piece<TYPE>(*reinterpret_cast<const v4u *>(xs + ((int64_t)c * KC + e2) * ES), fx);
#pragma unroll
                        for (int j = 0; j < E; j++) {
                            acc0[c] = __builtin_fmaf(fa[j], fx[j], acc0[c]);
                            acc1[c] = __builtin_fmaf(fb[j], fx[j], acc1[c]);
                        }
                    }
                }
            }
        }
        if (!live) continue;
#pragma unroll
        for (int c = 0; c < NC; c++) {
            float s0 = acc0[c], s1 = acc1[c];
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) {
                s0 += __shfl_xor(s0, o, 64);
                s1 += __shfl_xor(s1, o, 64);
            }
            if (lane == 0) {
                y[(int64_t)c * M + r0] = s0;
                if (r0 + 1 < M) y[(int64_t)c * M + r0 + 1] = s1;
            }
        }
    }
}

// ---- 1..16 columns on the matrix cores ------------------------------------------------------------------------------
// The weights go from HBM straight into the A operand of a 16 x 16 MFMA: lane (r, g) of a wave holds bytes 16 g .. 16 g + 15
// of a 64-byte step of row r of the wave's group of 16 rows (v_mfma_f32_16x16x32_f16 / _bf16: 8 elements of K group g;
// v_mfma_f32_16x16x4_f32: four MFMAs, one per float), a ring of SK_RING steps in flight per lane.  The B operand is the
// converted activations, resident in LDS for the whole launch: column c at XOFF + c * (row bytes + 16) -- the 16 bytes
// shift neighbouring columns to other banks -- and the lanes of columns that do not exist read a block of zeros.
// A workgroup of 16 waves is RG row groups x S segments of K (S a power of two); the segments' partial tiles are added in
// segment order through LDS, so a result does not depend on the launch geometry beyond S.
// Accumulator q of lane (c, g) is weight row 4 g + q of the group and activation column c.
// Requires (K * ES) % 64 == 0 and 256 + N * (K * ES + 16) + 16 KiB of LDS.
constexpr int SK_WAVES = 16, SK_RING = 8, SK_XOFF = 256;
typedef float v4f __attribute__((ext_vector_type(4)));

template <int TYPE>
__device__ __forceinline__ void skinny_step(const v4u &a, const v4u &b, v4f *acc, int which) {
    if (TYPE == T_F32) {
        acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(bits_f32(a.x), bits_f32(b.x), acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(bits_f32(a.y), bits_f32(b.y), acc[1], 0, 0, 0);
        acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(bits_f32(a.z), bits_f32(b.z), acc[2], 0, 0, 0);
        acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(bits_f32(a.w), bits_f32(b.w), acc[3], 0, 0, 0);
    } else if (TYPE == T_F16) {
        acc[which] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), acc[which], 0, 0, 0);
    } else {
        acc[which] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), acc[which], 0, 0, 0);
    }
}

template <int TYPE>
__global__ __launch_bounds__(64 * SK_WAVES) void plain_skinny_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x,
                                                                     float *__restrict__ y, int K, int64_t M, int N, int S, int sps) {
    constexpr int ES = TYPE == T_F32 ? 4 : 2;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, g = lane >> 4;
    const int RG = SK_WAVES / S, rg = wave / S, seg = wave - rg * S;
    const int64_t groups = (M + 15) / 16, group = (int64_t)blockIdx.x * RG + rg;
    const bool live = group < groups;
    const int row_bytes = K * ES, k64 = row_bytes / 64, cs = row_bytes + 16;
    const int64_t row = live ? (group * 16 + r < M ? group * 16 + r : M - 1) : 0;
    const int t0 = seg * sps, t1 = t0 + sps < k64 ? t0 + sps : k64;  // this wave's steps (none when t0 >= k64)
    const uint8_t *wp = w + row * (int64_t)row_bytes + g * 16;
    auto fetch = [&](int t) { return *reinterpret_cast<const v4u *>(wp + (int64_t)(t < k64 ? t : k64 - 1) * 64); };

    v4u ring[SK_RING];
#pragma unroll
    for (int j = 0; j < SK_RING; j++) ring[j] = fetch(t0 + j);

    // the activations, converted to the weight's type
    if (tid < 64) reinterpret_cast<unsigned *>(lds)[tid] = 0u;
    for (int c = 0; c < N; c++) {
        const float4 *xc = reinterpret_cast<const float4 *>(x + (int64_t)c * K);
        uint8_t *dst = lds + SK_XOFF + c * cs;
        for (int i = tid; i < K / 4; i += 64 * SK_WAVES) {
            const float4 v = xc[i];
            if (TYPE == T_F32) *reinterpret_cast<float4 *>(dst + i * 16) = v;
            else {
                uint2 p;
                p.x = (unsigned)narrow16<TYPE>(v.x) | ((unsigned)narrow16<TYPE>(v.y) << 16);
                p.y = (unsigned)narrow16<TYPE>(v.z) | ((unsigned)narrow16<TYPE>(v.w) << 16);
                *reinterpret_cast<uint2 *>(dst + i * 8) = p;
            }
        }
    }
    __syncthreads();

    const uint8_t *xp = r < N ? lds + SK_XOFF + r * cs + g * 16 : lds;
    const int xstep = r < N ? 64 : 0;
    v4f acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i] = (v4f){0.f, 0.f, 0.f, 0.f};

    int t = t0;
    // full turns of the ring: every slot is multiplied and asked for again
    for (; t + 2 * SK_RING <= t1; t += SK_RING) {
#pragma unroll
        for (int j = 0; j < SK_RING; j++) {
            const v4u b = *reinterpret_cast<const v4u *>(xp + (int64_t)(t + j) * xstep);
            skinny_step<TYPE>(ring[j], b, acc, j & 1);
            ring[j] = fetch(t + j + SK_RING);
        }
    }
    // the last one or two turns
    if (t + SK_RING < t1) {
#pragma unroll
        for (int j = 0; j < SK_RING; j++) {
            const v4u b = *reinterpret_cast<const v4u *>(xp + (int64_t)(t + j) * xstep);
            skinny_step<TYPE>(ring[j], b, acc, j & 1);
            ring[j] = fetch(t + j + SK_RING);
        }
        t += SK_RING;
    }
#pragma unroll
    for (int j = 0; j < SK_RING; j++)
        if (t + j < t1) {
            const v4u b = *reinterpret_cast<const v4u *>(xp + (int64_t)(t + j) * xstep);
            skinny_step<TYPE>(ring[j], b, acc, j & 1);
        }

    v4f sum = TYPE == T_F32 ? (acc[0] + acc[1]) + (acc[2] + acc[3]) : acc[0] + acc[1];
    if (S > 1) {
        v4f *part = reinterpret_cast<v4f *>(lds + (SK_XOFF + N * cs + 15) / 16 * 16);
        part[wave * 64 + lane] = sum;
        __syncthreads();
        if (seg != 0) return;
        for (int sgm = 1; sgm < S; sgm++) sum += part[(wave + sgm) * 64 + lane];
    }
    if (!live || r >= N) return;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int64_t m = group * 16 + 4 * g + q;
        if (m < M) y[(int64_t)r * M + m] = sum[q];
    }
}

// ---- any K: a wave per output, element loads -------------------------------------------------------------------------
template <int TYPE>
__global__ __launch_bounds__(256) void plain_naive_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ y,
                                                          int64_t K, int64_t M, int64_t N) {
    const int lane = threadIdx.x & 63;
    const int64_t waves = (int64_t)gridDim.x * 4, total = M * N;
    for (int64_t o = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); o < total; o += waves) {
        const int64_t n = o / M, m = o - n * M;
        float s = 0.0f;
        for (int64_t k = lane; k < K; k += 64) {
            float wv, xv = x[n * K + k];
            if (TYPE == T_F32) wv = reinterpret_cast<const float *>(w)[m * K + k];
            else {
                float dummy;
                widen2<TYPE>(reinterpret_cast<const unsigned short *>(w)[m * K + k], wv, dummy);
                widen2<TYPE>(narrow16<TYPE>(xv), xv, dummy);
            }
            s = __builtin_fmaf(wv, xv, s);
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
        if (lane == 0) y[o] = s;
    }
}

// Which output tile a workgroup takes.  Workgroups go to the eight XCDs round robin by their id, and each XCD has an L2
// of its own: the workgroups that share a weight tile (all activation tiles of one tile of weight rows) must sit on one
// XCD, or every XCD fetches that tile from HBM for itself (14336 x 4096 halves at 512 columns: eight activation tiles,
// 940 MB of weight reads for 117 MB of weights).  XCD k takes the weight tiles k, k + 8, ..., an activation tile after
// the other.  The grid is tiles_n * (tiles_m rounded up to a multiple of 8); false: no such tile.
__device__ __forceinline__ bool tile_of(unsigned id, int tiles_n, int64_t tiles_m, int64_t &mt, int &nt) {
    const unsigned xcd = id & 7, slot = id >> 3;
    nt = (int)(slot % (unsigned)tiles_n);
    mt = (int64_t)(slot / (unsigned)tiles_n) * 8 + xcd;
    return mt < tiles_m;
}

// ---- 9 columns and more: tiles on the matrix cores ---------------------------------------------------------------------
// Workgroup of WM x WN waves; a wave owns TN x TM accumulator tiles of 32 (activation rows) x 32 (weight rows).  The
// A operand of an MFMA is the activations, the B operand the weights: accumulator i of lane l is activation row
// 8 (i / 4) + 4 (l / 32) + i % 4 and weight row l % 32, so a store instruction writes runs of 32 consecutive floats of y.
// A stage is 64 bytes of every row of the tile (32 halves or 16 floats), rows padded to 80 bytes in LDS; two stages.
// Requires (K * ES) % 64 == 0.  xc: the activations in the weight's type, [N][K].
template <int TYPE, int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(64 * WM * WN) void plain_gemm_kernel(const uint8_t *__restrict__ w, const uint8_t *__restrict__ xc,
                                                                  float *__restrict__ y, int64_t K, int64_t M, int64_t N) {
    constexpr int ES = TYPE == T_F32 ? 4 : 2;
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32, NT = 64 * WM * WN;
    constexpr int LDR = 80, ROWS = BM + BN, PIECES = ROWS * 4, PP = (PIECES + NT - 1) / NT;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2][ROWS * LDR];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave / WN, wn = wave % WN;
    int64_t mt;
    int nt;
    if (!tile_of(blockIdx.x, (int)((N + BN - 1) / BN), (M + BM - 1) / BM, mt, nt)) return;
    const int64_t n0 = (int64_t)nt * BN, m0 = mt * BM;
    const int64_t row_bytes = K * ES;
    const int nk = (int)(row_bytes / 64);

    // the pieces this thread copies per stage: tile row r (weights first, then activations), 16-byte piece q
    const uint8_t *src[PP];
    int dst[PP];
#pragma unroll
    for (int i = 0; i < PP; i++) {
        const int idx = tid + i * NT, r = idx >> 2, q = idx & 3;
        dst[i] = idx < PIECES ? r * LDR + q * 16 : -1;
        if (r < BM) {
            const int64_t m = m0 + r < M ? m0 + r : M - 1;
            src[i] = w + m * row_bytes + q * 16;
        } else {
            const int64_t n = n0 + (r - BM) < N ? n0 + (r - BM) : N - 1;
            src[i] = xc + n * row_bytes + q * 16;
        }
    }
    // two stages on their way in registers while a third is multiplied out of LDS: stage kt + 1 sits in set (kt + 1) & 1,
    // stage kt + 2 in set kt & 1 (stages past the last are the last one again: no load under a condition)
    v4u regs[2][PP];
    auto fetch = [&](int set, int kt) {
        const int64_t off = (int64_t)(kt < nk ? kt : nk - 1) * 64;
#pragma unroll
        for (int i = 0; i < PP; i++)
            if (dst[i] >= 0) regs[set][i] = *reinterpret_cast<const v4u *>(src[i] + off);
    };
    auto park = [&](int set, int buf) {
#pragma unroll
        for (int i = 0; i < PP; i++)
            if (dst[i] >= 0) *reinterpret_cast<v4u *>(&lds[buf][dst[i]]) = regs[set][i];
    };

    v16f acc[TN][TM];
#pragma unroll
    for (int a = 0; a < TN; a++)
#pragma unroll
        for (int b = 0; b < TM; b++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[a][b][i] = 0.0f;

    const int row_in = lane & 31, kg = lane >> 5;
    const int wrow = (wm * TM * 32 + row_in) * LDR, xrow = (BM + wn * TN * 32 + row_in) * LDR;

    fetch(0, 0);
    park(0, 0);
    fetch(1, 1);
    fetch(0, 2);
    __syncthreads();
    auto stage = [&](int kt, auto parity) {
        constexpr int P = decltype(parity)::value;  // kt & 1
        const uint8_t *L = lds[P];
        if (TYPE == T_F32) {
            // the 16 products of a stage are added up from zero and their sum joins the running total: K / 16 roundings
            // of the total instead of K / 2 (a row of 14336 floats: 896 instead of 7168)
            v16f part[TN][TM];
#pragma unroll
            for (int a = 0; a < TN; a++)
#pragma unroll
                for (int b = 0; b < TM; b++)
#pragma unroll
                    for (int i = 0; i < 16; i++) part[a][b][i] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < 8; ks++) {
                float fa[TN], fb[TM];
#pragma unroll
                for (int a = 0; a < TN; a++) fa[a] = *reinterpret_cast<const float *>(L + xrow + a * 32 * LDR + ks * 8 + kg * 4);
#pragma unroll
                for (int b = 0; b < TM; b++) fb[b] = *reinterpret_cast<const float *>(L + wrow + b * 32 * LDR + ks * 8 + kg * 4);
#pragma unroll
                for (int a = 0; a < TN; a++)
#pragma unroll
                    for (int b = 0; b < TM; b++) part[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[a], fb[b], part[a][b], 0, 0, 0);
            }
#pragma unroll
            for (int a = 0; a < TN; a++)
#pragma unroll
                for (int b = 0; b < TM; b++)
#pragma unroll
                    for (int i = 0; i < 16; i++) acc[a][b][i] += part[a][b][i];
        } else {
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                v4u fa[TN], fb[TM];
#pragma unroll
                for (int a = 0; a < TN; a++) fa[a] = *reinterpret_cast<const v4u *>(L + xrow + a * 32 * LDR + ks * 32 + kg * 16);
#pragma unroll
                for (int b = 0; b < TM; b++) fb[b] = *reinterpret_cast<const v4u *>(L + wrow + b * 32 * LDR + ks * 32 + kg * 16);
#pragma unroll
                for (int a = 0; a < TN; a++)
#pragma unroll
                    for (int b = 0; b < TM; b++) {
                        if (TYPE == T_F16)
                            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, fa[a]), __builtin_bit_cast(v8h, fb[b]),
                                                                               acc[a][b], 0, 0, 0);
                        else
                            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, fa[a]), __builtin_bit_cast(v8bf, fb[b]),
                                                                                acc[a][b], 0, 0, 0);
                    }
            }
        }
        park(P ^ 1, P ^ 1);   // stage kt + 1 into the other buffer (its last readers passed the barrier below one stage ago)
        fetch(P ^ 1, kt + 3);
        __syncthreads();
    };
    for (int kt = 0; kt < nk; kt += 2) {
        stage(kt, std::integral_constant<int, 0>());
        if (kt + 1 < nk) stage(kt + 1, std::integral_constant<int, 1>());
    }

#pragma unroll
    for (int b = 0; b < TM; b++) {
        const int64_t m = m0 + wm * TM * 32 + b * 32 + row_in;
        if (m >= M) continue;
#pragma unroll
        for (int a = 0; a < TN; a++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int64_t n = n0 + wn * TN * 32 + a * 32 + 8 * (i >> 2) + 4 * kg + (i & 3);
                if (n < N) y[n * M + m] = acc[a][b][i];
            }
    }
}

// ---- the tiles for F16 / BF16 with the weights kept out of LDS --------------------------------------------------------
// The tiled kernel above reads one 1 KiB operand fragment from LDS per MFMA, and at the 16-bit types' MFMA rate that
// read is what bounds it.  Here only the activations go through LDS: a wave owns 64 weight rows, four groups of 16, whose
// fragments it loads from global memory straight into the B operand of v_mfma_f32_16x16x32 -- lane (c, kg) holds bytes
// 16 kg .. 16 kg + 15 of a 64-byte K step of row c, so an instruction reads runs of 64 bytes of 16 rows (the 32 x 32
// shape would read 16-byte pieces of 64 different lines per instruction: measured, 164 against 133 us on 14336 x 4096 at
// 512 columns) -- and multiplies each against a 64-row activation tile: four LDS reads per sixteen MFMAs.  Workgroup:
// two waves, 128 weight rows x 64 activation rows; a stage is two K steps (128 bytes of every row); two stages of
// weights in registers, the activation stage after next in registers, the next one in LDS.
// Accumulator q of lane (c, kg) in tile (a, b) is activation row 16 a + 4 kg + q and weight row 16 b + c.
// Requires (K * 2) % 128 == 0.
constexpr int G2_WAVES = 2, G2_TM = 4, G2_TN = 4, G2_BM = G2_WAVES * G2_TM * 16, G2_BN = G2_TN * 16, G2_LDR = 144;
template <int TYPE>
__global__ __launch_bounds__(64 * G2_WAVES, 2) void plain_gemm2_kernel(const uint8_t *__restrict__ w, const uint8_t *__restrict__ xc,
                                                                    float *__restrict__ y, int64_t K, int64_t M, int64_t N) {
    constexpr int NT = 64 * G2_WAVES, PP = G2_BN * 8 / NT;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2][G2_BN * G2_LDR];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, kg = lane >> 4;
    int64_t mt;
    int nt;
    if (!tile_of(blockIdx.x, (int)((N + G2_BN - 1) / G2_BN), (M + G2_BM - 1) / G2_BM, mt, nt)) return;
    const int64_t n0 = (int64_t)nt * G2_BN, m0 = mt * G2_BM;
    const int64_t row_bytes = K * 2;
    const int nk = (int)(row_bytes / 128);

    const uint8_t *wsrc[G2_TM];
#pragma unroll
    for (int b = 0; b < G2_TM; b++) {
        const int64_t m = m0 + wave * (G2_TM * 16) + b * 16 + c;
        wsrc[b] = w + (m < M ? m : M - 1) * row_bytes + kg * 16;
    }
    const uint8_t *asrc[PP];
    int adst[PP];
#pragma unroll
    for (int i = 0; i < PP; i++) {
        const int idx = tid + i * NT, r = idx >> 3, q = idx & 7;
        const int64_t n = n0 + r < N ? n0 + r : N - 1;
        asrc[i] = xc + n * row_bytes + q * 16;
        adst[i] = r * G2_LDR + q * 16;
    }
    v4u wr[2][G2_TM][2], ar[PP];
    auto fetch_w = [&](int set, int kt) {
        const int64_t off = (int64_t)(kt < nk ? kt : nk - 1) * 128;
#pragma unroll
        for (int b = 0; b < G2_TM; b++)
#pragma unroll
            for (int k = 0; k < 2; k++) wr[set][b][k] = *reinterpret_cast<const v4u *>(wsrc[b] + off + k * 64);
    };
    auto fetch_a = [&](int kt) {
        const int64_t off = (int64_t)(kt < nk ? kt : nk - 1) * 128;
#pragma unroll
        for (int i = 0; i < PP; i++) ar[i] = *reinterpret_cast<const v4u *>(asrc[i] + off);
    };
    auto park_a = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PP; i++) *reinterpret_cast<v4u *>(&lds[buf][adst[i]]) = ar[i];
    };

    v4f acc[G2_TN][G2_TM];
#pragma unroll
    for (int a = 0; a < G2_TN; a++)
#pragma unroll
        for (int b = 0; b < G2_TM; b++) acc[a][b] = (v4f){0.f, 0.f, 0.f, 0.f};

    fetch_w(0, 0);
    fetch_a(0);
    park_a(0);
    fetch_w(1, 1);
    fetch_a(1);
    __syncthreads();
    const int arow = c * G2_LDR + kg * 16;
    auto stage = [&](int kt, auto parity) {
        constexpr int P = decltype(parity)::value;  // kt & 1
        const uint8_t *L = lds[P];
#pragma unroll
        for (int k = 0; k < 2; k++) {
            v4u fa[G2_TN];
#pragma unroll
            for (int a = 0; a < G2_TN; a++) fa[a] = *reinterpret_cast<const v4u *>(L + arow + a * 16 * G2_LDR + k * 64);
#pragma unroll
            for (int a = 0; a < G2_TN; a++)
#pragma unroll
                for (int b = 0; b < G2_TM; b++) {
                    if (TYPE == T_F16)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, fa[a]), __builtin_bit_cast(v8h, wr[P][b][k]),
                                                                           acc[a][b], 0, 0, 0);
                    else
                        acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, fa[a]), __builtin_bit_cast(v8bf, wr[P][b][k]),
                                                                            acc[a][b], 0, 0, 0);
                }
        }
        park_a(P ^ 1);       // activation stage kt + 1 into the other buffer
        fetch_a(kt + 2);
        fetch_w(P, kt + 2);  // the weight set just multiplied
        __syncthreads();
    };
    for (int kt = 0; kt < nk; kt += 2) {
        stage(kt, std::integral_constant<int, 0>());
        if (kt + 1 < nk) stage(kt + 1, std::integral_constant<int, 1>());
    }

#pragma unroll
    for (int b = 0; b < G2_TM; b++) {
        const int64_t m = m0 + wave * (G2_TM * 16) + b * 16 + c;
        if (m >= M) continue;
#pragma unroll
        for (int a = 0; a < G2_TN; a++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int64_t n = n0 + a * 16 + 4 * kg + q;
                if (n < N) y[n * M + m] = acc[a][b][q];
            }
    }
}

int elem_size(int type) { return type == T_F32 ? 4 : 2; }

template <int TYPE>
hipError_t gemv_typed(const DevWeight &w, const float *x, int ncols, float *y, int num_cus, hipStream_t s) {
    constexpr int ES = TYPE == T_F32 ? 4 : 2, E = 16 / ES;
    // the chunk: what 64 KiB of LDS holds for ncols columns, a multiple of the 128 pieces a wave takes per turn
    int kc = 65536 / (ncols * ES);
    kc -= kc % (128 * E);
    const int K = (int)w.K;
    if (kc > K) kc = (K + 128 * E - 1) / (128 * E) * (128 * E);
    const size_t lds = (size_t)ncols * kc * ES;
    const int64_t rounds = (w.M + 31) / 32;
    const dim3 grid((unsigned)std::min<int64_t>(rounds, 2 * (int64_t)num_cus)), block(64 * GEMV_WAVES);
#define PLAIN_GEMV(NC) case NC: plain_gemv_kernel<TYPE, NC><<<grid, block, lds, s>>>(w.p0, x, y, K, w.M, kc); break;
    switch (ncols) {
        PLAIN_GEMV(1) PLAIN_GEMV(2) PLAIN_GEMV(3) PLAIN_GEMV(4) PLAIN_GEMV(5) PLAIN_GEMV(6) PLAIN_GEMV(7) PLAIN_GEMV(8)
    default: return hipErrorInvalidValue;
    }
#undef PLAIN_GEMV
    return hipGetLastError();
}

size_t skinny_lds(int type, int64_t K, int N) {
    return (size_t)(SK_XOFF + N * (K * elem_size(type) + 16) + 15) / 16 * 16 + SK_WAVES * 1024;
}

template <int TYPE>
hipError_t skinny_typed(const DevWeight &w, const float *x, int N, float *y, int num_cus, hipStream_t s) {
    static bool allowed[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 && !allowed[dev]) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(plain_skinny_kernel<TYPE>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        allowed[dev] = true;
    }
    const int k64 = (int)(w.K * elem_size(TYPE) / 64);
    const int64_t groups = (w.M + 15) / 16;
    // segments of K per row group: as many as keep the launch within one workgroup per CU (the registers leave room for
    // one; a second round of workgroups that fills part of the CUs costs a whole round: 14336 x 4096 halves at one column
    // 28.3 us with 448 workgroups), while a segment keeps a ring of steps
    int S = 1;
    while (S < SK_WAVES && groups * (2 * S) <= (int64_t)num_cus * SK_WAVES && k64 / (2 * S) >= SK_RING) S *= 2;
    const int sps = (k64 + S - 1) / S, RG = SK_WAVES / S;
    const int64_t grid = (groups + RG - 1) / RG;
    if (grid > 0x7fffffff) return hipErrorInvalidValue;
    plain_skinny_kernel<TYPE><<<dim3((unsigned)grid), dim3(64 * SK_WAVES), skinny_lds(TYPE, w.K, N), s>>>(w.p0, x, y, (int)w.K, w.M, N, S, sps);
    return hipGetLastError();
}

template <int TYPE>
hipError_t gemm_typed(const DevWeight &w, const void *xc, int64_t N, float *y, int num_cus, hipStream_t s) {
    const uint8_t *xb = (const uint8_t *)xc;
    // one-dimensional grids: tiles_n x (tiles_m rounded up to a multiple of 8), see tile_of
    auto grid_of = [&](int bm, int bn, unsigned &g) {
        const int64_t tn = (N + bn - 1) / bn, tm8 = ((w.M + bm - 1) / bm + 7) / 8 * 8;
        if (tn * tm8 > 0x7fffffff) return false;
        g = (unsigned)(tn * tm8);
        return true;
    };
    unsigned g = 0;
    const int64_t mt = (w.M + 127) / 128;
    // F16 / BF16 products with too few 128 x 128 tiles for the CUs: 128 x 64 tiles with the weights kept out of LDS (4096 x
    // 4096 at 512 columns 72 -> 56 us; with tiles enough the 128 x 128 kernel is ahead: 14336 x 4096 at 512 columns 151
    // against 133 us -- a 128 x 64 tile moves 1.5 times the bytes per flop into the CU)
    if (TYPE != T_F32 && N > 32 && (w.K * 2) % 128 == 0 && mt * ((N + 127) / 128) < num_cus) {
        if (!grid_of(G2_BM, G2_BN, g)) return hipErrorInvalidValue;
        plain_gemm2_kernel<TYPE == T_F32 ? T_F16 : TYPE><<<g, 64 * G2_WAVES, 0, s>>>(w.p0, xb, y, w.K, w.M, N);
        return hipGetLastError();
    }
    if (N <= 32) {
        if (!grid_of(128, 32, g)) return hipErrorInvalidValue;
        plain_gemm_kernel<TYPE, 4, 1, 1, 1><<<g, 256, 0, s>>>(w.p0, xb, y, w.K, w.M, N);
    } else if (TYPE == T_F32 && mt * ((N + 127) / 128) < num_cus) {
        // too few 128 x 128 tiles for the CUs: 128 x 64 (4096 x 4096 at 512 columns 370 -> 230 us; the 16-bit types, whose
        // MFMAs are eight times as fast, are bound by the LDS reads and lose there: 72 -> 95 us)
        if (!grid_of(128, 64, g)) return hipErrorInvalidValue;
        plain_gemm_kernel<TYPE, 2, 2, 2, 1><<<g, 256, 0, s>>>(w.p0, xb, y, w.K, w.M, N);
    } else {
        // (256 x 128 tiles of four waves of 64 x 128 -- six LDS fragment reads per eight MFMAs instead of eight -- measured
        // 133 us where these take 122: 14336 x 4096 at 512 columns is 224 such tiles for 256 CUs)
        if (!grid_of(128, 128, g)) return hipErrorInvalidValue;
        plain_gemm_kernel<TYPE, 2, 2, 2, 2><<<g, 256, 0, s>>>(w.p0, xb, y, w.K, w.M, N);
    }
    return hipGetLastError();
}

}  // namespace

bool plain_type(int type) { return type == T_F32 || type == T_F16 || type == T_BF16; }

int plain_kind(int type, int64_t K, int64_t M, int64_t N, int force) {
    if (!plain_type(type) || K < 1 || M < 1 || N < 1 || K > 0x7fffffff / 4) return 0;
    const int64_t row_bytes = K * elem_size(type);
    const bool tiles = row_bytes % 64 == 0;
    if (force == 2) return tiles ? 2 : 0;
    if (N <= 16 && row_bytes % 64 == 0 && skinny_lds(type, K, (int)N) <= 160 * 1024) return 5;
    if (N <= 8 && row_bytes % 16 == 0) return 1;
    if (tiles && force != 1) return 2;
    return row_bytes % 16 == 0 ? 4 : 3;
}

size_t plain_convert_bytes(int type, int64_t K, int64_t N) { return type == T_F32 ? 0 : (size_t)(K * N) * 2; }

hipError_t launch_plain(const DevWeight &w, const float *x, int64_t N, float *y, void *xc, int num_cus, hipStream_t s, int force) {
    const int kind = plain_kind(w.type, w.K, w.M, N, force);
    if (kind == 0 || N > 0x7fffffff) return hipErrorInvalidValue;
    if (kind == 1 || kind == 4) {
        for (int64_t c0 = 0; c0 < N; c0 += 8) {
            const int nc = (int)(N - c0 < 8 ? N - c0 : 8);
            const float *xg = x + c0 * w.K;
            float *yg = y + c0 * w.M;
            hipError_t e;
            switch (w.type) {
            case T_F32: e = gemv_typed<T_F32>(w, xg, nc, yg, num_cus, s); break;
            case T_F16: e = gemv_typed<T_F16>(w, xg, nc, yg, num_cus, s); break;
            default: e = gemv_typed<T_BF16>(w, xg, nc, yg, num_cus, s); break;
            }
            if (e != hipSuccess) return e;
        }
        return hipSuccess;
    }
    if (kind == 5) {
        switch (w.type) {
        case T_F32: return skinny_typed<T_F32>(w, x, (int)N, y, num_cus, s);
        case T_F16: return skinny_typed<T_F16>(w, x, (int)N, y, num_cus, s);
        default: return skinny_typed<T_BF16>(w, x, (int)N, y, num_cus, s);
        }
    }
    if (kind == 2) {
        if (w.type == T_F32) return gemm_typed<T_F32>(w, x, N, y, num_cus, s);
        if (!xc) return hipErrorInvalidValue;
        const int64_t count = w.K * N;
        const unsigned blocks = (unsigned)std::min<int64_t>((count + 255) / 256, 8 * (int64_t)num_cus);
        if (w.type == T_F16) plain_convert_kernel<T_F16><<<blocks, 256, 0, s>>>(x, (unsigned short *)xc, count);
        else plain_convert_kernel<T_BF16><<<blocks, 256, 0, s>>>(x, (unsigned short *)xc, count);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        return w.type == T_F16 ? gemm_typed<T_F16>(w, xc, N, y, num_cus, s) : gemm_typed<T_BF16>(w, xc, N, y, num_cus, s);
    }
    const int64_t outs = w.M * N;
    const unsigned blocks = (unsigned)std::min<int64_t>((outs + 3) / 4, 16 * (int64_t)num_cus);
    switch (w.type) {
    case T_F32: plain_naive_kernel<T_F32><<<blocks, 256, 0, s>>>(w.p0, x, y, w.K, w.M, N); break;
    case T_F16: plain_naive_kernel<T_F16><<<blocks, 256, 0, s>>>(w.p0, x, y, w.K, w.M, N); break;
    default: plain_naive_kernel<T_BF16><<<blocks, 256, 0, s>>>(w.p0, x, y, w.K, w.M, N); break;
    }
    return hipGetLastError();
}

}  // namespace miqmm
