// Prefill GEMM (batch >= 32) on the int8 matrix cores for Q4_0 and Q8_0 weights against Q8_0
// activations -- y[n][m] = vec_dot(W row m, Q8_0(x row n)), the work behind Tensor.Mulmat
// (/root/reference/ml/backend.go:151) for a prompt batch on the 32-element block formats.
//
// Both sides carry an fp16 scale per 32 elements, so the integer sum is only homogeneous over one
// block: one v_mfma_i32_32x32x32_i8 (K = 32) is exactly one block of a 32 x 32 output tile, and every
// MFMA is followed by an fp32 step  y += float(I) * (d_w * d_x)  on its 16 accumulators -- 48 vector
// instructions per MFMA, which is what bounds the kernel (one MFMA costs about 6 vector instructions
// of issue time), not the matrix cores and not memory.  What is left to design is keeping that vector
// work fed:
//   * A wave owns 32 weight rows x 64 activation columns and a run of blocks of K; the weights are the
//     A operand (a lane supplies 16 consecutive K values of one row: one 16-byte load for Q8_0, the
//     low or the high nibbles of the block's 16 bytes for Q4_0, minus 8, for Q4_0), shared by the
//     two MFMAs of a block; the activations are the B operand straight from the Q8_0 quants plane.
//   * Operands go global -> registers, one block ahead; waves are independent (no barriers in the
//     loop).  The only LDS traffic is the transposition of the weight scales: a lane's 16 accumulators
//     are 16 different weight rows, so each block's 32 scales go through a per-wave LDS line.
//   * The waves of a workgroup cut K between them and sum their tiles through LDS at the end, in a
//     fixed order: enough waves to fill the machine even when M/32 x N/64 is small.
#include <hip/hip_fp16.h>

#include "internal.h"

namespace miqmm {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float h2f(unsigned bits16) { return __half2float(__ushort_as_half((unsigned short)bits16)); }

// One block of a wave's operands as loaded: raw weight bytes of the lane's row, the quants of its two
// activation columns, and the scales that go with them.
template <bool Q4>
struct Blk {
    v4i w;        // Q8_0: the lane's 16 quants; Q4_0: the block's 16 packed bytes
    v4i x[2];     // 16 activation quants of column n0 + 32t + lane%32
    float dx[2];  // their block scales
    unsigned dw;  // fp16 scale of weight row lane%32 (lanes 0..31 use it)
};

template <bool Q4>
__device__ __forceinline__ void load_blk(Blk<Q4> &b, const uint8_t *wq, const uint16_t *wd, const int8_t *const (&xq)[2],
                                         const float *const (&xd)[2], int64_t blk, int half) {
    if (Q4) b.w = *reinterpret_cast<const v4i *>(wq + blk * 16);
    else b.w = *reinterpret_cast<const v4i *>(wq + blk * 32 + 16 * half);
    b.dw = wd[blk];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        b.x[t] = *reinterpret_cast<const v4i *>(xq[t] + blk * 32 + 16 * half);
        b.dx[t] = xd[t][blk];
    }
}

// Q4_0: elements 0..15 of a block are the low nibbles of its 16 bytes, 16..31 the high ones; value q - 8.
// (q | 0x80) - 8 never borrows across bytes; flipping the top bit back leaves q - 8 as a signed byte.
__device__ __forceinline__ v4i unpack_q4_0(v4i raw, int half) {
    v4i r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const unsigned nib = ((unsigned)raw[i] >> (4 * half)) & 0x0f0f0f0fu;
        r[i] = (int)((((nib | 0x80808080u) - 0x08080808u)) ^ 0x80808080u);
    }
    return r;
}

// Sum of the waves' tiles over the K cuts (through LDS, fixed order, wave 0 keeps its own and does the
// adding), then the stores: accumulator v of a lane is weight row 8*(v/4) + 4*(lane/32) + v%4, column
// lane%32 of MFMA t.  part: [waves - 1][2][16][64] floats.
__device__ __forceinline__ void store_tile(float (&acc)[2][16], float *part, int waves, int wave, int lane, int64_t m0,
                                           int64_t n0, int64_t M, int64_t N, float *__restrict__ y) {
    const int c = lane & 31, half = lane >> 5;
    if (waves > 1) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int v = 0; v < 16; v++)
                if (wave > 0) part[(((wave - 1) * 2 + t) * 16 + v) * 64 + lane] = acc[t][v];
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                float s = acc[t][v];
                for (int k = 1; k < waves; k++) s += part[(((k - 1) * 2 + t) * 16 + v) * 64 + lane];
                acc[t][v] = s;
            }
    }
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int64_t col = n0 + 32 * t + c;
        if (col >= N) continue;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int64_t r = m0 + 8 * q + 4 * half;
            float *out = y + col * M + r;
            if (r + 3 < M && (M & 3) == 0) {
                *reinterpret_cast<float4 *>(out) = make_float4(acc[t][4 * q], acc[t][4 * q + 1], acc[t][4 * q + 2], acc[t][4 * q + 3]);
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (r + j < M) out[j] = acc[t][4 * q + j];
            }
        }
    }
}

// blockDim.x / 64 waves cut K; blockIdx.x = n-tile * tiles_m + m-tile (consecutive workgroups share
// their activation columns).
template <bool Q4>
__global__ __launch_bounds__(512, 2) void gemm_blk32_kernel(DevWeight w, DevAct a, float *__restrict__ y, int tiles_m) {
    extern __shared__ __align__(16) uint8_t smem[];  // per wave: 2 x 32 floats of weight scales; then the K-cut partials
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = blockDim.x >> 6;
    const int c = lane & 31, half = lane >> 5;
    const int tn = blockIdx.x / tiles_m, tm = blockIdx.x - tn * tiles_m;
    const int64_t m0 = (int64_t)tm * 32, n0 = (int64_t)tn * 64;
    const int64_t nblk = w.K / QK;
    const int64_t b0 = nblk * wave / waves, b1 = nblk * (wave + 1) / waves;

    // rows / columns past the edge: the last one again, results dropped
    const int64_t row = min(m0 + c, w.M - 1);
    const uint8_t *wq = w.p0 + row * (Q4 ? nblk * 16 : w.K);
    const uint16_t *wd = w.d + row * nblk;
    const int8_t *xq[2];
    const float *xd[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int64_t col = min(n0 + 32 * t + c, (int64_t)a.N - 1);
        xq[t] = a.qs + col * a.K;
        xd[t] = a.d + col * nblk;
    }
    float *dsm = reinterpret_cast<float *>(smem) + wave * 64;  // [2][32]

    float acc[2][16];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][v] = 0.f;

    if (b0 < b1) {
        Blk<Q4> cur, nxt;
        load_blk<Q4>(cur, wq, wd, xq, xd, b0, half);
#pragma unroll 1
        for (int64_t b = b0; b < b1; b++) {
            float *line = dsm + ((b - b0) & 1) * 32;
            if (half == 0) line[c] = h2f(cur.dw);
            load_blk<Q4>(nxt, wq, wd, xq, xd, min(b + 1, b1 - 1), half);
            const v4i aop = Q4 ? unpack_q4_0(cur.w, half) : cur.w;
            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const v16i i0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, cur.x[0], zero, 0, 0, 0);
            const v16i i1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, cur.x[1], zero, 0, 0, 0);
            // accumulator v of a lane is weight row 8*(v/4) + 4*half + v%4 of the tile
            float dwv[16];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 f = *reinterpret_cast<const float4 *>(line + 8 * q + 4 * half);
                dwv[4 * q] = f.x; dwv[4 * q + 1] = f.y; dwv[4 * q + 2] = f.z; dwv[4 * q + 3] = f.w;
            }
#pragma unroll
            for (int v = 0; v < 16; v++) {
                acc[0][v] = __builtin_fmaf((float)i0[v], dwv[v] * cur.dx[0], acc[0][v]);
                acc[1][v] = __builtin_fmaf((float)i1[v], dwv[v] * cur.dx[1], acc[1][v]);
            }
            cur = nxt;
        }
    }

    store_tile(acc, reinterpret_cast<float *>(smem) + waves * 64, waves, wave, lane, m0, n0, w.M, a.N, y);
}

// The same product four blocks (128 elements of K) at a time, for K a multiple of 128: the four
// blocks of a chunk share a cache line per row, their scales are one 8-byte (weights) and one 16-byte
// (activations) load, and the whole next chunk is in flight while the current one is multiplied --
// four times the bytes in flight per wave and about half the load instructions of the block-wise loop.
template <bool Q4>
struct Chunk {
    v4i w[4];
    v4i x[2][4];
    float4 dx[2];
    uint2 dw;  // four fp16 scales of weight row lane%32
};

template <bool Q4>
__device__ __forceinline__ void load_chunk(Chunk<Q4> &ch, const uint8_t *wq, const uint16_t *wd, const int8_t *const (&xq)[2],
                                           const float *const (&xd)[2], int64_t blk, int half) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
        if (Q4) ch.w[j] = *reinterpret_cast<const v4i *>(wq + (blk + j) * 16);
        else ch.w[j] = *reinterpret_cast<const v4i *>(wq + (blk + j) * 32 + 16 * half);
    }
    ch.dw = *reinterpret_cast<const uint2 *>(wd + blk);
#pragma unroll
    for (int t = 0; t < 2; t++) {
#pragma unroll
        for (int j = 0; j < 4; j++) ch.x[t][j] = *reinterpret_cast<const v4i *>(xq[t] + (blk + j) * 32 + 16 * half);
        ch.dx[t] = *reinterpret_cast<const float4 *>(xd[t] + blk);
    }
}

template <bool Q4>
__global__ __launch_bounds__(512, 1) void gemm_blk32_chunk_kernel(DevWeight w, DevAct a, float *__restrict__ y, int tiles_m) {
    extern __shared__ __align__(16) uint8_t smem[];  // per wave: 2 x 4 x 32 floats of weight scales; then the K-cut partials
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = blockDim.x >> 6;
    const int c = lane & 31, half = lane >> 5;
    const int tn = blockIdx.x / tiles_m, tm = blockIdx.x - tn * tiles_m;
    const int64_t m0 = (int64_t)tm * 32, n0 = (int64_t)tn * 64;
    const int64_t nblk = w.K / QK, nch = nblk / 4;
    const int64_t c0 = nch * wave / waves, c1 = nch * (wave + 1) / waves;  // this wave's chunks

    const int64_t row = min(m0 + c, w.M - 1);
    const uint8_t *wq = w.p0 + row * (Q4 ? nblk * 16 : w.K);
    const uint16_t *wd = w.d + row * nblk;
    const int8_t *xq[2];
    const float *xd[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int64_t col = min(n0 + 32 * t + c, (int64_t)a.N - 1);
        xq[t] = a.qs + col * a.K;
        xd[t] = a.d + col * nblk;
    }
    float *dsm = reinterpret_cast<float *>(smem) + wave * 256;  // [2][4][32]

    float acc[2][16];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][v] = 0.f;

    if (c0 < c1) {
        Chunk<Q4> cur, nxt;
        load_chunk<Q4>(cur, wq, wd, xq, xd, c0 * 4, half);
#pragma unroll 1
        for (int64_t ch = c0; ch < c1; ch++) {
            float *lines = dsm + ((ch - c0) & 1) * 128;
            if (half == 0) {
                lines[c] = h2f(cur.dw.x & 0xffff);
                lines[32 + c] = h2f(cur.dw.x >> 16);
                lines[64 + c] = h2f(cur.dw.y & 0xffff);
                lines[96 + c] = h2f(cur.dw.y >> 16);
            }
            load_chunk<Q4>(nxt, wq, wd, xq, xd, min(ch + 1, c1 - 1) * 4, half);
            const float dx0[4] = {cur.dx[0].x, cur.dx[0].y, cur.dx[0].z, cur.dx[0].w};
            const float dx1[4] = {cur.dx[1].x, cur.dx[1].y, cur.dx[1].z, cur.dx[1].w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const v4i aop = Q4 ? unpack_q4_0(cur.w[j], half) : cur.w[j];
                const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                const v16i i0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, cur.x[0][j], zero, 0, 0, 0);
                const v16i i1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, cur.x[1][j], zero, 0, 0, 0);
                float dwv[16];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float4 f = *reinterpret_cast<const float4 *>(lines + 32 * j + 8 * q + 4 * half);
                    dwv[4 * q] = f.x; dwv[4 * q + 1] = f.y; dwv[4 * q + 2] = f.z; dwv[4 * q + 3] = f.w;
                }
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    acc[0][v] = __builtin_fmaf((float)i0[v], dwv[v] * dx0[j], acc[0][v]);
                    acc[1][v] = __builtin_fmaf((float)i1[v], dwv[v] * dx1[j], acc[1][v]);
                }
            }
            cur = nxt;
        }
    }
    store_tile(acc, reinterpret_cast<float *>(smem) + waves * 256, waves, wave, lane, m0, n0, w.M, a.N, y);
}

}  // namespace

bool gemm_blk32_supports(int type, int64_t K, int64_t M) {
    return (type == T_Q4_0 || type == T_Q8_0) && K >= QK && K % QK == 0 && M >= 1;
}

hipError_t launch_gemm_blk32(const DevWeight &w, const DevAct &a, float *y, int num_cus, hipStream_t s) {
    if (!gemm_blk32_supports(w.type, w.K, w.M) || a.type != T_Q8_0 || a.K != w.K || a.N < 1 || !y) return hipErrorInvalidValue;
    const int64_t tiles_m = (w.M + 31) / 32, tiles_n = ((int64_t)a.N + 63) / 64, tiles = tiles_m * tiles_n;
    if (tiles > 0x7fffffff) return hipErrorInvalidValue;
    // waves per workgroup = cuts of K: about four waves per SIMD over the whole grid, at least eight
    // blocks per wave
    // waves per workgroup = cuts of K: enough waves over the whole grid to keep every SIMD busy, at
    // least eight blocks per wave
    const int64_t nblk = w.K / QK;
    const bool chunked = w.K % 128 == 0;
    const int64_t want = ((int64_t)num_cus * (chunked ? 12 : 16) + tiles - 1) / tiles;  // 3 / 4 waves fit a SIMD
    int waves = (int)(want < 1 ? 1 : want > 8 ? 8 : want);
    while (waves > 1 && nblk / waves < 8) waves--;
    const size_t part = (size_t)(waves - 1) * 2 * 16 * 64 * sizeof(float);  // <= 56 KiB
    if (chunked) {
        const size_t lds = (size_t)waves * 256 * sizeof(float) + part;
        if (w.type == T_Q4_0) gemm_blk32_chunk_kernel<true><<<(unsigned)tiles, 64 * waves, lds, s>>>(w, a, y, (int)tiles_m);
        else gemm_blk32_chunk_kernel<false><<<(unsigned)tiles, 64 * waves, lds, s>>>(w, a, y, (int)tiles_m);
    } else {
        const size_t lds = (size_t)waves * 64 * sizeof(float) + part;
        if (w.type == T_Q4_0) gemm_blk32_kernel<true><<<(unsigned)tiles, 64 * waves, lds, s>>>(w, a, y, (int)tiles_m);
        else gemm_blk32_kernel<false><<<(unsigned)tiles, 64 * waves, lds, s>>>(w, a, y, (int)tiles_m);
    }
    return hipGetLastError();
}

}  // namespace miqmm
