// Prefill GEMM (batch >= 32) on the int8 matrix cores for Q4_0 and Q8_0 weights against Q8_0
// activations -- y[n][m] = vec_dot(W row m, Q8_0(x row n)), the work behind Tensor.Mulmat
// (/root/reference/ml/backend.go:151) for a prompt batch on the 32-element block formats.
//
// Both sides carry an fp16 scale per 32 elements, so the integer sum is only homogeneous over one
// block: one v_mfma_i32_32x32x32_i8 (K = 32) is exactly one block of a 32 x 32 output tile, and every
// MFMA is followed by an fp32 step  y += float(I) * (d_w * d_x)  on its 16 accumulators -- at least 48
// vector instructions per MFMA, which is what bounds the kernels (one MFMA costs about 6 vector
// instructions of issue time), not the matrix cores and not memory.
//   * A wave owns 32 weight rows x 64 activation columns and a run of blocks of K; the weights are the
//     A operand (a lane supplies 16 consecutive K values of one row: 16 bytes of a Q8_0 block, or the
//     low / high nibbles of a Q4_0 block's 16 bytes minus 8), shared by the two MFMAs of a block; the
//     activations are the B operand straight from the Q8_0 quants plane.
//   * Waves are independent (no barriers in the loop).  A lane's 16 accumulators are 16 different
//     weight rows, so the weight scales of a block reach the lanes through LDS.
//   * The waves of a workgroup cut K between them and sum their tiles through LDS at the end, in a
//     fixed order.
//   * gemm_blk32_dma_kernel (K a multiple of 64) stages all operands through per-wave LDS rings with
//     direct-to-LDS loads; gemm_blk32_kernel (any K) loads them into registers one block ahead.
#include <hip/hip_fp16.h>

#include "internal.h"

namespace miqmm {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void lds_ptr_t;
typedef const __attribute__((address_space(1))) void glb_ptr_t;

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

// The same product with the operands staged through LDS by direct-to-LDS loads, for K a multiple of
// 64.  A register load in MFMA operand layout touches 32 rows with 16 bytes each -- 32 cache lines
// per instruction, and the L1's line rate, not its bandwidth, bounds the kernels above.  Here
// consecutive lanes copy consecutive 16-byte pieces of a row (four lanes per 64-byte run of two
// blocks), the copies need no registers, and a wave keeps two stages of two blocks in flight in its
// own LDS region: no barriers in the loop, each wave waits on its own memory counter (every wave
// issues exactly NDMA copies per stage, so "at most NDMA outstanding" means the older stage landed).
// Pieces are XOR-swizzled with row bits so that the operand reads spread over the banks.
template <bool Q4>
struct DmaGeo {
    static constexpr int W_BYTES = Q4 ? 1024 : 2048;  // 32 rows x 2 blocks
    static constexpr int W_INSTRS = W_BYTES / 1024;
    static constexpr int X_BYTES = 4096;              // 64 columns x 2 blocks of quants
    static constexpr int DW_OFF = W_BYTES + X_BYTES;  // 32 rows x 2 fp16
    static constexpr int DX_OFF = DW_OFF + 256;       // 2 blocks x 64 floats
    static constexpr int STAGE = DX_OFF + 512;
    static constexpr int NDMA = W_INSTRS + 4 + 1 + 2;
    static constexpr int WAVE_BYTES = (2 * STAGE > 8192 ? 2 * STAGE : 8192);  // the K-cut partials reuse the region
};

template <bool Q4>
__global__ __launch_bounds__(512, 1) void gemm_blk32_dma_kernel(DevWeight w, DevAct a, float *__restrict__ y, int tiles_m) {
    typedef DmaGeo<Q4> Geo;
    extern __shared__ __align__(256) uint8_t smem[];  // waves x WAVE_BYTES
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = blockDim.x >> 6;
    const int c = lane & 31, half = lane >> 5;
    const int tn = blockIdx.x / tiles_m, tm = blockIdx.x - tn * tiles_m;
    const int64_t m0 = (int64_t)tm * 32, n0 = (int64_t)tn * 64;
    const int64_t nblk = w.K / QK, nch = nblk / 2;
    const int64_t c0 = nch * wave / waves, c1 = nch * (wave + 1) / waves;  // this wave's chunks of two blocks
    uint8_t *wsm = smem + wave * Geo::WAVE_BYTES;
    const int rows_left = (int)min((int64_t)32, w.M - m0), cols_left = (int)min((int64_t)64, (int64_t)a.N - n0);

    // ---- copy plan: per-lane offsets from uniform bases; rows / columns past the edge copy the last one
    unsigned woff[Geo::W_INSTRS], xoff[4];
#pragma unroll
    for (int i = 0; i < Geo::W_INSTRS; i++) {
        if (Q4) {
            const int r = lane >> 1, pos = lane & 1, piece = pos ^ ((r >> 3) & 1);  // piece = block of the chunk
            woff[i] = (unsigned)min(r, rows_left - 1) * (unsigned)(nblk * 16) + 16u * piece;
        } else {
            const int s_ = 64 * i + lane, r = s_ >> 2, pos = s_ & 3, piece = pos ^ ((r >> 2) & 3);  // piece = 2*block + half
            woff[i] = (unsigned)min(r, rows_left - 1) * (unsigned)w.K + 16u * piece;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int s_ = 64 * i + lane, col = s_ >> 2, pos = s_ & 3, piece = pos ^ ((col >> 2) & 3);
        xoff[i] = (unsigned)min(col, cols_left - 1) * (unsigned)a.K + 16u * piece;
    }
    const unsigned dwoff = (unsigned)min(c, rows_left - 1) * (unsigned)nblk * 2u;      // bytes into the fp16 plane
    const unsigned dxoff = (unsigned)min(lane, cols_left - 1) * (unsigned)nblk * 4u;  // bytes into the f32 plane
    const uint8_t *wbase = w.p0 + m0 * (Q4 ? nblk * 16 : w.K);
    const uint8_t *xbase = reinterpret_cast<const uint8_t *>(a.qs) + n0 * a.K;
    const uint8_t *dwbase = reinterpret_cast<const uint8_t *>(w.d + m0 * nblk);
    const uint8_t *dxbase = reinterpret_cast<const uint8_t *>(a.d + n0 * nblk);

    auto stage_copy = [&](uint8_t *st, int64_t ch) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < Geo::W_INSTRS; i++) {
            const uint8_t *gp = wbase + ch * (Q4 ? 32 : 64) + woff[i];
            __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + 1024 * i), 16, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint8_t *gp = xbase + ch * 64 + xoff[i];
            __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + Geo::W_BYTES + 1024 * i), 16, 0, 0);
        }
        {
            const uint8_t *gp = dwbase + ch * 4 + dwoff;
            if (lane < 32) __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + Geo::DW_OFF), 4, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint8_t *gp = dxbase + (ch * 2 + j) * 4 + dxoff;
            __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + Geo::DX_OFF + 256 * j), 4, 0, 0);
        }
    };

    float acc[2][16];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][v] = 0.f;

    if (c0 < c1) {
        stage_copy(wsm, c0);
        stage_copy(wsm + Geo::STAGE, min(c0 + 1, c1 - 1));
#pragma unroll 1
        for (int64_t ch = c0; ch < c1; ch++) {
            uint8_t *st = wsm + ((ch - c0) & 1) * Geo::STAGE;
            __builtin_amdgcn_s_waitcnt((Geo::NDMA & 15) | (7 << 4) | (15 << 8) | ((Geo::NDMA >> 4) << 14));
            v4i aw[2], bx[2][2];
            uint4 dwq[4];
            float dxv[2][2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                if (Q4) aw[j] = *reinterpret_cast<const v4i *>(st + c * 32 + 16 * (j ^ ((c >> 3) & 1)));
                else aw[j] = *reinterpret_cast<const v4i *>(st + c * 64 + 16 * ((2 * j + half) ^ ((c >> 2) & 3)));
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    const int col = 32 * t + c;
                    bx[t][j] = *reinterpret_cast<const v4i *>(st + Geo::W_BYTES + col * 64 + 16 * ((2 * j + half) ^ ((col >> 2) & 3)));
                    dxv[t][j] = *reinterpret_cast<const float *>(st + Geo::DX_OFF + 256 * j + 4 * col);
                }
            }
#pragma unroll
            for (int q = 0; q < 4; q++) dwq[q] = *reinterpret_cast<const uint4 *>(st + Geo::DW_OFF + 4 * (8 * q + 4 * half));
            // operands are in registers: the stage can take the copies of chunk ch + 2
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            stage_copy(st, min(ch + 2, c1 - 1));
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const v4i aop = Q4 ? unpack_q4_0(aw[j], half) : aw[j];
                const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                const v16i i0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, bx[0][j], zero, 0, 0, 0);
                const v16i i1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, bx[1][j], zero, 0, 0, 0);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const unsigned pr[4] = {dwq[q].x, dwq[q].y, dwq[q].z, dwq[q].w};  // rows 8q + 4*half + i: (block 0, block 1) fp16
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float dwf = h2f(j ? pr[i] >> 16 : pr[i] & 0xffff);
                        const int v = 4 * q + i;
                        acc[0][v] = __builtin_fmaf((float)i0[v], dwf * dxv[0][j], acc[0][v]);
                        acc[1][v] = __builtin_fmaf((float)i1[v], dwf * dxv[1][j], acc[1][v]);
                    }
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0);  // the redundant copies of the last iterations must land before the region is reused
    }
    // K-cut partials: wave k > 0 parks its tile in its own (now idle) stage region
    float *mine = reinterpret_cast<float *>(wsm);
    if (waves > 1) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int v = 0; v < 16; v++)
                if (wave > 0) mine[(t * 16 + v) * 64 + lane] = acc[t][v];
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                float s_ = acc[t][v];
                for (int k = 1; k < waves; k++)
                    s_ += reinterpret_cast<const float *>(smem + k * Geo::WAVE_BYTES)[(t * 16 + v) * 64 + lane];
                acc[t][v] = s_;
            }
    }
    store_tile(acc, nullptr, 1, 0, lane, m0, n0, w.M, a.N, y);
}

// ---------------------------------------------------------------------------------------------
// Skinny product (a few activation columns: small-batch decode) for Q4_0 / Q8_0 on the matrix cores.
// The streaming GEMV pays one v_dot4 pass per column; here the columns share one
// v_mfma_i32_16x16x64_i8 per 16 weight rows and 64 elements.  A 64-wide step is two blocks (K groups
// 0,1 and 2,3), so the 16 rows of the A operand are 8 columns x the 2 blocks of the step: row r is
// column r>>1 restricted to the K groups of block r&1, zeros elsewhere (those lanes read a zero slot).
// Lane l then holds, for weight row l%16, the integer block sums of columns 2(l>>4), 2(l>>4)+1 with both
// blocks of the step, and scales each with d_w * d_x in fp32 -- ggml's order of operations.  Q4_0 quants
// stay unsigned nibbles; the -8 goes through the activations' block sums.
// Same shape as the K-quant skinny kernel: a workgroup owns 16 weight rows, its waves cut K in runs
// of 256 elements and stream weights, activations and both sides' scales through private two-stage LDS
// rings with direct-to-LDS loads; one barrier at the end for the sum over the K cuts.  (Q8_0 at up to eight columns with
// waves of at most two steps takes the weights straight into registers instead: DW below, 9.9 -> 9.4 us and 10.2 -> 9.5 us
// for 4096 x 4096 at four and eight columns, quantization launch included.)
// ---------------------------------------------------------------------------------------------
typedef int v4acc __attribute__((ext_vector_type(4)));

template <bool Q4, int NCT>
struct Sk32Geo {
    static constexpr int W_BYTES = Q4 ? 2048 : 4096, W_INSTRS = W_BYTES / 1024;  // 16 rows x 256 elements
    static constexpr int DW_OFF = W_BYTES;                 // 16 rows x 8 fp16
    static constexpr int A_OFF = DW_OFF + 256;             // NCT columns x 256 quants
    static constexpr int A_INSTRS = NCT / 4;
    static constexpr int DX_OFF = A_OFF + NCT * 256;       // NCT columns x 8 f32
    static constexpr int BS_OFF = DX_OFF + NCT * 32;       // NCT columns x 8 i16 (Q4_0)
    static constexpr int Z_OFF = BS_OFF + (Q4 ? NCT * 16 : 0);
    static constexpr int STAGE = (Z_OFF + 16 + 63) / 64 * 64;
    static constexpr int NDMA = W_INSTRS + 1 + A_INSTRS + 1 + (Q4 ? 1 : 0);
    static constexpr int WAVE_BYTES = (2 * STAGE + 255) / 256 * 256;
    static constexpr int PART_BYTES = 16 * 16 * 4;
    static constexpr int SETS = NCT / 8;
};

// Expert-indexed launches (Tensor.MulmatID, /root/reference/ml/backend.go:153): w is a stack of expert
// matrices, a workgroup belongs to one group of up to 16 (token, slot) pairs of one expert (bucketed by
// group_pairs_kernel) and to 16 rows of that expert; the group's pairs are its activation columns.
struct Sk32Ids {
    const int *groups;  // groups[0] = number of groups, then records {expert or -1, count, pair[16]}
    int64_t M;          // rows per expert
    int wgs_per_group, n_used, b_cols;
};
constexpr int SK32_ID_REC = 2 + 16;

// Several matrices of one type and K against the same activations in one launch (q, k, v; gate, up): their
// 16-row groups are numbered through, matrix 0 is the kernel's w and y, the others come in this block.
struct Sk32Multi {
    const uint8_t *p0[3];
    const uint16_t *d[3];
    float *y[3];
    int64_t M[3];
    int grp_end[3];  // exclusive ends of the runs of matrices 0, 1, 2; INT_MAX past the last matrix
};

// DW ("direct weights", Q8_0, one set of columns, waves of at most two steps): the weights and their scales go from
// memory straight into registers -- a quad of lanes on 64 contiguous bytes of a row, as in the deep kernels of
// skinny_deep.hip -- and ds_bpermute puts them into the MFMA operand order; only the activations still pass through the
// wave's LDS stages.  Same K cut, same expressions in the same order: the bits of the staged form.
template <bool Q4, int NCT, bool ID, bool MULTI = false, bool DW = false>
__global__ __launch_bounds__(512, (NCT > 8 ? 2 : 4)) void skinny32_kernel(DevWeight w_in, DevAct a_in, int col0, int nc, float *__restrict__ y_in,
                                                                          Sk32Ids si_in, int WAVES, Sk32Multi mt) {
    static_assert(!(ID && MULTI), "expert-indexed launches take one stack");
    static_assert(!DW || (!Q4 && NCT == 8 && !ID && !MULTI), "direct weights: Q8_0, up to eight columns, one matrix");
    typedef Sk32Geo<Q4, NCT> Geo;
    constexpr int STAGE = Geo::STAGE, NDMA = Geo::NDMA, SETS = Geo::SETS;
    // The argument block in one batch of scalar loads: everything is named here and pinned by an empty asm
    // (otherwise each branch below is followed by a round of loads of its own), pointers as
    // global-address-space pointers so that they stay known to be global, the block size as an argument.
    typedef const __attribute__((address_space(1))) uint8_t *gbytes_t;
    typedef const __attribute__((address_space(1))) uint16_t *ghalves_t;
    typedef const __attribute__((address_space(1))) int8_t *gi8_t;
    typedef const __attribute__((address_space(1))) int16_t *gi16_t;
    typedef const __attribute__((address_space(1))) float *gcfloats_t;
    typedef const __attribute__((address_space(1))) int *gcints_t;
    typedef __attribute__((address_space(1))) float *gfloats_t;
    typedef int ints4_t __attribute__((ext_vector_type(4)));
    typedef long longs2_t __attribute__((ext_vector_type(2)));
    gbytes_t p0 = (gbytes_t)w_in.p0;
    ghalves_t wd = (ghalves_t)w_in.d;
    gi8_t aqs = (gi8_t)a_in.qs;
    gcfloats_t ad = (gcfloats_t)a_in.d;
    gi16_t ab = (gi16_t)a_in.bsums;
    gcints_t groups = (gcints_t)si_in.groups;
    gfloats_t yg = (gfloats_t)y_in;
    longs2_t km = {(long)w_in.K, (long)w_in.M}, km2 = {(long)a_in.K, (long)si_in.M};
    ints4_t i0 = {col0, nc, WAVES, a_in.N}, i1 = {si_in.wgs_per_group, si_in.n_used, si_in.b_cols, 0};
    asm volatile("" : "+s"(p0), "+s"(wd), "+s"(aqs), "+s"(ad), "+s"(ab), "+s"(groups), "+s"(yg), "+s"(km), "+s"(km2), "+s"(i0),
                      "+s"(i1));
    DevWeight w{(const uint8_t *)p0, w_in.p1, w_in.p2, (const uint16_t *)wd, km[0], km[1], w_in.type};
    const DevAct a{(const int8_t *)aqs, (const float *)ad, (const int16_t *)ab, a_in.sd8, a_in.sd16, km2[0], i0[3], a_in.type};
    const Sk32Ids si{(const int *)groups, km2[1], i1[0], i1[1], i1[2]};
    float *__restrict__ y = (float *)yg;
    int first_group = 0;  // where the workgroup's matrix starts in the numbered-through groups
    if (MULTI) {
#pragma unroll
        for (int t = 0; t < 3; t++)
            if ((int)blockIdx.x >= mt.grp_end[t]) {
                w.p0 = mt.p0[t]; w.d = mt.d[t]; w.M = mt.M[t];
                y = mt.y[t];
                first_group = mt.grp_end[t];
            }
    }
    col0 = i0[0]; nc = i0[1]; WAVES = i0[2];
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];  // WAVES x (WAVE_BYTES + PART_BYTES)
    float (*part)[16][16] = reinterpret_cast<float (*)[16][16]>(smem + WAVES * Geo::WAVE_BYTES);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, g = lane >> 4;
    int64_t m0 = (int64_t)((int)blockIdx.x - first_group) * 16, yrow0 = m0, ldy = w.M;  // first weight row in w; first row and pitch of y
    int rows_left = (int)min((int64_t)16, w.M - m0);
    const int *rec = nullptr;
    if (ID) {
        const int group = blockIdx.x / si.wgs_per_group, wg = blockIdx.x - group * si.wgs_per_group;
        if (group >= si.groups[0]) return;
        rec = si.groups + 1 + (size_t)group * SK32_ID_REC;
        const int expert = rec[0];
        nc = rec[1];
        yrow0 = (int64_t)wg * 16;
        ldy = si.M;
        rows_left = (int)min((int64_t)16, si.M - yrow0);
        if (expert < 0) {  // ids outside the stack: the outputs of these pairs are all NaN
            for (int o = tid; o < 16 * nc; o += (64 * WAVES))
                if ((o & 15) < rows_left) y[(int64_t)rec[2 + (o >> 4)] * ldy + yrow0 + (o & 15)] = __int_as_float(0x7fc00000);
            return;
        }
        m0 = (int64_t)expert * si.M + yrow0;
    }
    // activation row behind column i of the launch (i clamped to the live columns)
    auto col_of = [&](int i) -> unsigned {
        i = min(i, nc - 1);
        if (!ID) return (unsigned)(col0 + i);
        const int pair = rec[2 + i], tok = pair / si.n_used, slot = pair - tok * si.n_used;
        return (unsigned)(tok * si.b_cols + slot % si.b_cols);
    };
    const int64_t nblk = w.K / QK, nst = w.K / 256;
    const int64_t s0 = nst * wave / WAVES, s1 = nst * (wave + 1) / WAVES;  // this wave's run of 256-element steps
    uint8_t *wsm = smem + wave * Geo::WAVE_BYTES;

    // ---- copy plan
    unsigned woff[Geo::W_INSTRS], aoff[Geo::A_INSTRS];
#pragma unroll
    for (int i = 0; i < Geo::W_INSTRS; i++) {
        const int idx = 64 * i + lane;
        if (Q4) {
            const int r = idx >> 3, slot = idx & 7, piece = slot ^ ((r >> 1) & 7);  // piece = block of the step
            woff[i] = (unsigned)min(r, rows_left - 1) * (unsigned)(nblk * 16) + 16u * piece;
        } else {
            const int r = idx >> 4, slot = idx & 15, piece = slot ^ r;  // piece = 16 quants
            woff[i] = (unsigned)min(r, rows_left - 1) * (unsigned)w.K + 16u * piece;
        }
    }
#pragma unroll
    for (int j = 0; j < Geo::A_INSTRS; j++) {
        const int col = 4 * j + (lane >> 4), slot = lane & 15;  // stage slot [col][slot] holds piece slot ^ col
        aoff[j] = col_of(col) * (unsigned)a.K + 16u * (slot ^ col);
    }
    const unsigned dwoff = (unsigned)min(c, rows_left - 1) * (unsigned)nblk * 2u;
    const unsigned dxoff = col_of(lane >> 1) * (unsigned)nblk * 4u + 16u * (lane & 1);
    const unsigned bsoff = col_of(lane) * (unsigned)nblk * 2u;
    const uint8_t *wbase = w.p0 + m0 * (Q4 ? nblk * 16 : w.K);
    const uint8_t *dwbase = reinterpret_cast<const uint8_t *>(w.d + m0 * nblk);
    const uint8_t *aq = reinterpret_cast<const uint8_t *>(a.qs);
    const uint8_t *adx = reinterpret_cast<const uint8_t *>(a.d);
    const uint8_t *abs_ = reinterpret_cast<const uint8_t *>(a.bsums);

    auto stage_copy = [&](uint8_t *st, int64_t sp) __attribute__((always_inline)) {
        if (!DW) {
#pragma unroll
            for (int i = 0; i < Geo::W_INSTRS; i++) {
                const uint8_t *gp = wbase + sp * (Q4 ? 128 : 256) + woff[i];
                __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + 1024 * i), 16, 0, 0);
            }
            const uint8_t *gp = dwbase + sp * 16 + dwoff;
            if (lane < 16) __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + Geo::DW_OFF), 16, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < Geo::A_INSTRS; j++) {
            const uint8_t *gp = aq + sp * 256 + aoff[j];
            __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + Geo::A_OFF + 1024 * j), 16, 0, 0);
        }
        {
            const uint8_t *gp = adx + sp * 32 + dxoff;
            if (lane < 2 * NCT) __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + Geo::DX_OFF), 16, 0, 0);
        }
        if (Q4) {
            const uint8_t *gp = abs_ + sp * 16 + bsoff;
            if (lane < NCT) __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + Geo::BS_OFF), 16, 0, 0);
        }
    };

    // ---- operand reads.  A row r = lane & 15 of column set cs is column 8 cs + (r >> 1), block r & 1 of
    // the step; lanes of the other block's K groups, and columns past nc, read the zero slot.
    if (lane < 8) *reinterpret_cast<int *>(wsm + (lane >> 2) * STAGE + Geo::Z_OFF + 4 * (lane & 3)) = 0;
    int aro[SETS][4], lcol[SETS][2];
#pragma unroll
    for (int cs = 0; cs < SETS; cs++) {
        const int col = 8 * cs + (c >> 1);
        const bool on = col < nc && (g >> 1) == (c & 1);
#pragma unroll
        for (int t = 0; t < 4; t++) aro[cs][t] = on ? Geo::A_OFF + col * 256 + 16 * ((4 * t + g) ^ col) : Geo::Z_OFF;
#pragma unroll
        for (int u = 0; u < 2; u++) lcol[cs][u] = min(8 * cs + 2 * g + u, NCT - 1);  // the lane's output columns
    }

    float acc[SETS][2];
#pragma unroll
    for (int cs = 0; cs < SETS; cs++) acc[cs][0] = acc[cs][1] = 0.f;
    if (DW) {
        if (s0 < s1) {
            typedef unsigned u4v __attribute__((ext_vector_type(4)));
            typedef const __attribute__((address_space(1))) u4v *gu4_t;
            typedef const __attribute__((address_space(1))) unsigned *gu_t;
            // loading lane: its row and which 16 bytes of the quad's 64 (rows 8..15 in the order 2 3 0 1: sources of
            // rows r and r + 8 must not share a bank of the ds_bpermute crossbar)
            const int lrow = min(lane >> 2, rows_left - 1), lq = (lane & 3) ^ ((lane >> 4) & 2);
            const unsigned qoff = (unsigned)lrow * (unsigned)w.K + 16u * lq, doff = (unsigned)lrow * (unsigned)nblk * 2u + 4u * lq;
            const int rsw = (c >> 3) << 1, bidx = 4 * (4 * c + (g ^ rsw));
            u4v wq[2][4];
            unsigned wdr[2];
            // requests: the activations of a step, then its weights; both steps at once (a wave has at most two)
#pragma unroll
            for (int st = 0; st < 2; st++) {
                const int64_t sp = min(s0 + st, s1 - 1);
                stage_copy(wsm + st * STAGE, sp);
                __builtin_amdgcn_sched_barrier(0);
                const __attribute__((address_space(1))) uint8_t *wp = (const __attribute__((address_space(1))) uint8_t *)(wbase + sp * 256);
                const __attribute__((address_space(1))) uint8_t *dp = (const __attribute__((address_space(1))) uint8_t *)(dwbase + sp * 16);
#pragma unroll
                for (int t = 0; t < 4; t++) wq[st][t] = *(gu4_t)(wp + (qoff + 64u * t));
                wdr[st] = *(gu_t)(dp + doff);
                __builtin_amdgcn_sched_barrier(0);
            }
            constexpr int PER_STEP = Geo::A_INSTRS + 1 + 5;  // copies and loads of one step
            const v4acc zero = {0, 0, 0, 0};
#pragma unroll
            for (int st = 0; st < 2; st++) {
                if (s0 + st < s1) {  // wave-uniform
                    const uint8_t *stg = wsm + st * STAGE;
                    if (st == 0) __builtin_amdgcn_s_waitcnt((PER_STEP & 15) | (7 << 4) | (15 << 8) | ((PER_STEP >> 4) << 14));
                    else __builtin_amdgcn_s_waitcnt((0 & 15) | (7 << 4) | (15 << 8));
                    v4i bq[4], av[4];
                    uint4 dxr[2][2];
#pragma unroll
                    for (int t = 0; t < 4; t++) {
#pragma unroll
                        for (int i = 0; i < 4; i++) bq[t][i] = __builtin_amdgcn_ds_bpermute(bidx, (int)wq[st][t][i]);
                        av[t] = *reinterpret_cast<const v4i *>(stg + aro[0][t]);
                    }
                    unsigned dwp[4];
#pragma unroll
                    for (int j = 0; j < 4; j++) dwp[j] = (unsigned)__builtin_amdgcn_ds_bpermute(4 * (4 * c) + 4 * (j ^ rsw), (int)wdr[st]);
#pragma unroll
                    for (int u = 0; u < 2; u++) {
                        dxr[u][0] = *reinterpret_cast<const uint4 *>(stg + Geo::DX_OFF + 32 * lcol[0][u]);
                        dxr[u][1] = *reinterpret_cast<const uint4 *>(stg + Geo::DX_OFF + 32 * lcol[0][u] + 16);
                    }
                    float dwf[8];
#pragma unroll
                    for (int b = 0; b < 8; b++) dwf[b] = h2f(b & 1 ? dwp[b >> 1] >> 16 : dwp[b >> 1] & 0xffff);
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        const v4acc dv = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[t], bq[t], zero, 0, 0, 0);
#pragma unroll
                        for (int u = 0; u < 2; u++) {
                            const unsigned dxp[8] = {dxr[u][0].x, dxr[u][0].y, dxr[u][0].z, dxr[u][0].w,
                                                     dxr[u][1].x, dxr[u][1].y, dxr[u][1].z, dxr[u][1].w};
#pragma unroll
                            for (int sblk = 0; sblk < 2; sblk++) {
                                const int b = 2 * t + sblk;
                                acc[0][u] = __builtin_fmaf((float)dv[2 * u + sblk], dwf[b] * __uint_as_float(dxp[b]), acc[0][u]);
                            }
                        }
                    }
                }
            }
            __builtin_amdgcn_s_waitcnt(0);
        }
    } else
    if (s0 < s1) {
        stage_copy(wsm, s0);
        stage_copy(wsm + STAGE, min(s0 + 1, s1 - 1));
        const v4acc zero = {0, 0, 0, 0};
#pragma unroll 1
        for (int64_t sp = s0; sp < s1; sp++) {
            uint8_t *st = wsm + ((sp - s0) & 1) * STAGE;
            __builtin_amdgcn_s_waitcnt((NDMA & 15) | (7 << 4) | (15 << 8) | ((NDMA >> 4) << 14));
            v4i bq[4], av[SETS][4];
            uint4 dxr[SETS][2][2], bsr[SETS][2];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                if (Q4) bq[t] = *reinterpret_cast<const v4i *>(st + c * 128 + 16 * ((2 * t + (g >> 1)) ^ ((c >> 1) & 7)));
                else bq[t] = *reinterpret_cast<const v4i *>(st + c * 256 + 16 * ((4 * t + g) ^ c));
            }
            const uint4 dwr = *reinterpret_cast<const uint4 *>(st + Geo::DW_OFF + 16 * c);
#pragma unroll
            for (int cs = 0; cs < SETS; cs++) {
#pragma unroll
                for (int t = 0; t < 4; t++) av[cs][t] = *reinterpret_cast<const v4i *>(st + aro[cs][t]);
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    dxr[cs][u][0] = *reinterpret_cast<const uint4 *>(st + Geo::DX_OFF + 32 * lcol[cs][u]);
                    dxr[cs][u][1] = *reinterpret_cast<const uint4 *>(st + Geo::DX_OFF + 32 * lcol[cs][u] + 16);
                    if (Q4) bsr[cs][u] = *reinterpret_cast<const uint4 *>(st + Geo::BS_OFF + 16 * lcol[cs][u]);
                }
            }
            // operands are in registers: the stage can take the copies of step sp + 2
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            stage_copy(st, min(sp + 2, s1 - 1));
            if (Q4) {
#pragma unroll
                for (int t = 0; t < 4; t++)
#pragma unroll
                    for (int i = 0; i < 4; i++) bq[t][i] = (int)(((unsigned)bq[t][i] >> (4 * (g & 1))) & 0x0f0f0f0fu);
            }
            const unsigned dwp[4] = {dwr.x, dwr.y, dwr.z, dwr.w};
            float dwf[8];
#pragma unroll
            for (int b = 0; b < 8; b++) dwf[b] = h2f(b & 1 ? dwp[b >> 1] >> 16 : dwp[b >> 1] & 0xffff);
#pragma unroll
            for (int cs = 0; cs < SETS; cs++) {
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const v4acc dv = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[cs][t], bq[t], zero, 0, 0, 0);
#pragma unroll
                    for (int u = 0; u < 2; u++) {
                        const unsigned dxp[8] = {dxr[cs][u][0].x, dxr[cs][u][0].y, dxr[cs][u][0].z, dxr[cs][u][0].w,
                                                 dxr[cs][u][1].x, dxr[cs][u][1].y, dxr[cs][u][1].z, dxr[cs][u][1].w};
                        const unsigned bsp[4] = {bsr[cs][u].x, bsr[cs][u].y, bsr[cs][u].z, bsr[cs][u].w};
#pragma unroll
                        for (int sblk = 0; sblk < 2; sblk++) {
                            const int b = 2 * t + sblk;
                            int iv = dv[2 * u + sblk];
                            if (Q4) {
                                const int bs = (int)(short)(b & 1 ? bsp[b >> 1] >> 16 : bsp[b >> 1] & 0xffff);
                                iv -= 8 * bs;  // sum (q - 8) x = sum q x - 8 sum x
                            }
                            acc[cs][u] = __builtin_fmaf((float)iv, dwf[b] * __uint_as_float(dxp[b]), acc[cs][u]);
                        }
                    }
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0);  // the repeated copies of the last iterations must not outlive the kernel's LDS
    }
#pragma unroll
    for (int cs = 0; cs < SETS; cs++)
#pragma unroll
        for (int u = 0; u < 2; u++) part[wave][8 * cs + 2 * g + u][c] = acc[cs][u];
    __syncthreads();
    for (int o = tid; o < 16 * NCT; o += (64 * WAVES)) {
        const int i = o >> 4, j = o & 15;  // activation column, weight row of the tile
        float sum = 0.f;
        for (int k = 0; k < WAVES; k++) sum += part[k][i][j];
        if (i < nc && j < rows_left) y[(int64_t)(ID ? rec[2 + i] : col0 + i) * ldy + yrow0 + j] = sum;
    }
}

template <bool Q4, int NCT, bool ID = false>
void launch_skinny32_as(const DevWeight &w, const DevAct &a, int col0, int ncols, float *y, int num_cus, hipStream_t s,
                        const Sk32Ids &si = Sk32Ids{nullptr, 0, 0, 0, 0}, int64_t id_grid = 0) {
    typedef Sk32Geo<Q4, NCT> Geo;
    const int64_t groups = ID ? id_grid : (w.M + 15) / 16, nst = w.K / 256;
    // about eight waves per CU over the whole grid (see the K-quant skinny kernel), every wave at least one step
    const int64_t want = ((int64_t)num_cus * 8 + groups / 2) / groups;
    int waves = want >= 8 ? 8 : want >= 6 ? 6 : want >= 4 ? 4 : want >= 3 ? 3 : want >= 2 ? 2 : 1;
    while (waves > 1 && nst / waves < 1) waves = waves > 4 ? waves - 2 : waves - 1;
    const size_t lds = (size_t)waves * (Geo::WAVE_BYTES + Geo::PART_BYTES);
    static bool allowed[64] = {false};  // more than 64 KiB of dynamic LDS has to be allowed once per device
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 && !allowed[dev]) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(skinny32_kernel<Q4, NCT, ID>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        allowed[dev] = true;
    }
    if constexpr (!Q4 && NCT == 8 && !ID) {
        // waves of at most two steps: the weights straight into registers (the bits are those of the staged form)
        if (nst <= 2 * waves && w.M * w.K < ((int64_t)1 << 32)) {
            static bool allowed_dw[64] = {false};
            if (dev >= 0 && dev < 64 && !allowed_dw[dev]) {
                (void)hipFuncSetAttribute(reinterpret_cast<const void *>(skinny32_kernel<false, 8, false, false, true>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                allowed_dw[dev] = true;
            }
            skinny32_kernel<false, 8, false, false, true><<<(unsigned)groups, 64 * waves, lds, s>>>(w, a, col0, ncols, y, si, waves, Sk32Multi{});
            return;
        }
    }
    skinny32_kernel<Q4, NCT, ID><<<(unsigned)groups, 64 * waves, lds, s>>>(w, a, col0, ncols, y, si, waves, Sk32Multi{});
}

// the K cut a matrix gets in a launch of its own
int skinny32_waves(int64_t M, int64_t K, int num_cus) {
    const int64_t groups = (M + 15) / 16, nst = K / 256;
    const int64_t want = ((int64_t)num_cus * 8 + groups / 2) / groups;
    int waves = want >= 8 ? 8 : want >= 6 ? 6 : want >= 4 ? 4 : want >= 3 ? 3 : want >= 2 ? 2 : 1;
    while (waves > 1 && nst / waves < 1) waves = waves > 4 ? waves - 2 : waves - 1;
    return waves;
}

template <bool Q4, int NCT>
void launch_skinny32_multi_as(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int ncols, int waves,
                              hipStream_t s) {
    typedef Sk32Geo<Q4, NCT> Geo;
    Sk32Multi mt;
    int64_t rg = (ws[0].M + 15) / 16;
    for (int t = 0; t < 3; t++) {
        const int j = t + 1 < count ? t + 1 : count - 1;
        mt.p0[t] = ws[j].p0; mt.d[t] = ws[j].d; mt.y[t] = ys[j]; mt.M[t] = ws[j].M;
        mt.grp_end[t] = t + 1 < count ? (int)rg : 0x7fffffff;
        if (t + 1 < count) rg += (ws[j].M + 15) / 16;
    }
    const size_t lds = (size_t)waves * (Geo::WAVE_BYTES + Geo::PART_BYTES);
    static bool allowed[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 && !allowed[dev]) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(skinny32_kernel<Q4, NCT, false, true>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        allowed[dev] = true;
    }
    skinny32_kernel<Q4, NCT, false, true><<<(unsigned)rg, 64 * waves, lds, s>>>(ws[0], a, 0, ncols, ys[0], Sk32Ids{nullptr, 0, 0, 0, 0},
                                                                                waves, mt);
}

}  // namespace

bool skinny32_supports(int type, int64_t K, int64_t M) {
    return (type == T_Q4_0 || type == T_Q8_0) && K >= 256 && K % 256 == 0 && M >= 1 && (M + 15) / 16 <= 0x7fffffff;
}

hipError_t launch_skinny32(const DevWeight &w, const DevAct &a, int col0, int ncols, float *y, int num_cus, hipStream_t s) {
    if (!skinny32_supports(w.type, w.K, w.M) || a.type != T_Q8_0 || a.K != w.K || !y) return hipErrorInvalidValue;
    if (ncols < 1 || ncols > 16 || col0 < 0 || col0 + ncols > a.N) return hipErrorInvalidValue;
    if ((int64_t)(col0 + ncols) * a.K >= ((int64_t)1 << 32) || (w.type == T_Q4_0 && !a.bsums)) return hipErrorInvalidValue;
    if (w.type == T_Q4_0) {
        if (ncols <= 8) launch_skinny32_as<true, 8>(w, a, col0, ncols, y, num_cus, s);
        else launch_skinny32_as<true, 16>(w, a, col0, ncols, y, num_cus, s);
    } else {
        if (ncols <= 8) launch_skinny32_as<false, 8>(w, a, col0, ncols, y, num_cus, s);
        else launch_skinny32_as<false, 16>(w, a, col0, ncols, y, num_cus, s);
    }
    return hipGetLastError();
}

// Several Q4_0 or Q8_0 matrices of one K in one launch, taken when each keeps the K cut of a launch of its own
// (the results are then the same bits) and the joint grid stays within about 16 waves per CU.
bool skinny32_multi_supports(const DevWeight *ws, int count, int ncols, int num_cus) {
    if (count < 2 || count > 4 || ncols < 1 || ncols > 16) return false;
    const int waves0 = skinny32_waves(ws[0].M, ws[0].K, num_cus);
    int64_t groups = 0;
    for (int i = 0; i < count; i++) {
        if (ws[i].type != ws[0].type || ws[i].K != ws[0].K || !skinny32_supports(ws[i].type, ws[i].K, ws[i].M)) return false;
        if (skinny32_waves(ws[i].M, ws[i].K, num_cus) != waves0) return false;
        groups += (ws[i].M + 15) / 16;
    }
    return groups < 0x7fffffff && groups * waves0 <= 16 * (int64_t)num_cus;
}

hipError_t launch_skinny32_multi(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int ncols, int num_cus,
                                 hipStream_t s) {
    if (!skinny32_multi_supports(ws, count, ncols, num_cus) || a.type != T_Q8_0 || a.K != ws[0].K) return hipErrorInvalidValue;
    if (ncols > a.N || (int64_t)ncols * a.K >= ((int64_t)1 << 32) || (ws[0].type == T_Q4_0 && !a.bsums)) return hipErrorInvalidValue;
    const int waves = skinny32_waves(ws[0].M, ws[0].K, num_cus);
    if (ws[0].type == T_Q4_0) {
        if (ncols <= 8) launch_skinny32_multi_as<true, 8>(ws, ys, count, a, ncols, waves, s);
        else launch_skinny32_multi_as<true, 16>(ws, ys, count, a, ncols, waves, s);
    } else {
        if (ncols <= 8) launch_skinny32_multi_as<false, 8>(ws, ys, count, a, ncols, waves, s);
        else launch_skinny32_multi_as<false, 16>(ws, ys, count, a, ncols, waves, s);
    }
    return hipGetLastError();
}

bool skinny32_id_supports(int type, int64_t K, int64_t M, int64_t pairs, int n_expert) {
    // from about four pairs per expert the buckets fill well enough to pay for the matrix cores
    return skinny32_supports(type, K, M) && pairs >= 4 * (int64_t)n_expert;
}

hipError_t launch_skinny32_id(const DevWeight &w, int n_expert, const DevAct &a, const int *ids, int n_used, int n_tokens,
                              int b_cols, float *y, int *groups, int num_cus, hipStream_t s) {
    if (n_expert < 1 || w.M % n_expert || !skinny32_supports(w.type, w.K, w.M / n_expert) || a.type != T_Q8_0 || a.K != w.K ||
        !ids || !y || !groups || n_used < 1 || n_tokens < 1 || b_cols < 1 || a.N != (int64_t)b_cols * n_tokens ||
        (int64_t)a.N * a.K >= ((int64_t)1 << 32) || (w.type == T_Q4_0 && !a.bsums))
        return hipErrorInvalidValue;
    const int64_t pairs = (int64_t)n_used * n_tokens, M = w.M / n_expert;
    if (pairs > 0x7fffffff / 16) return hipErrorInvalidValue;
    if (hipError_t e = launch_group_pairs(ids, (int)pairs, n_expert, 16, groups, s)) return e;
    const int64_t max_groups = min(pairs, (int64_t)n_expert + 1 + pairs / 16), wgs_per_group = (M + 15) / 16;
    if (max_groups * wgs_per_group > 0x7fffffff) return hipErrorInvalidValue;
    const Sk32Ids si{groups, M, (int)wgs_per_group, n_used, b_cols};
    if (w.type == T_Q4_0) launch_skinny32_as<true, 16, true>(w, a, 0, 16, y, num_cus, s, si, max_groups * wgs_per_group);
    else launch_skinny32_as<false, 16, true>(w, a, 0, 16, y, num_cus, s, si, max_groups * wgs_per_group);
    return hipGetLastError();
}

bool gemm_blk32_supports(int type, int64_t K, int64_t M) {
    return (type == T_Q4_0 || type == T_Q8_0) && K >= QK && K % QK == 0 && M >= 1;
}

hipError_t launch_gemm_blk32(const DevWeight &w, const DevAct &a, float *y, int num_cus, hipStream_t s) {
    if (!gemm_blk32_supports(w.type, w.K, w.M) || a.type != T_Q8_0 || a.K != w.K || a.N < 1 || !y) return hipErrorInvalidValue;
    const int64_t tiles_m = (w.M + 31) / 32, tiles_n = ((int64_t)a.N + 63) / 64, tiles = tiles_m * tiles_n;
    if (tiles > 0x7fffffff) return hipErrorInvalidValue;
    // Waves per workgroup = cuts of K.  The kernels are bound by the vector ALU and run best with about
    // one wave per SIMD over the whole grid (measured: more waves only add K-cut sums); at least eight
    // blocks per wave.
    const int64_t nblk = w.K / QK, want = ((int64_t)num_cus * 4 + tiles - 1) / tiles;
    int waves = (int)(want < 1 ? 1 : want > 8 ? 8 : want);
    while (waves > 1 && nblk / waves < 8) waves--;
    if (w.K % 64 == 0 && (uint64_t)w.K * 64 < (1ull << 31)) {
        const size_t lds = (size_t)waves * (w.type == T_Q4_0 ? DmaGeo<true>::WAVE_BYTES : DmaGeo<false>::WAVE_BYTES);
        static bool allowed_dev[64] = {false};  // more than 64 KiB of dynamic LDS has to be allowed once per device
        int dev = 0;
        (void)hipGetDevice(&dev);
        bool &allowed = allowed_dev[dev >= 0 && dev < 64 ? dev : 0];
        if (!allowed) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_blk32_dma_kernel<true>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_blk32_dma_kernel<false>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            allowed = true;
        }
        if (w.type == T_Q4_0) gemm_blk32_dma_kernel<true><<<(unsigned)tiles, 64 * waves, lds, s>>>(w, a, y, (int)tiles_m);
        else gemm_blk32_dma_kernel<false><<<(unsigned)tiles, 64 * waves, lds, s>>>(w, a, y, (int)tiles_m);
    } else {
        // K an odd number of blocks: operands by register loads, one block ahead
        const size_t lds = (size_t)waves * 64 * sizeof(float) + (size_t)(waves - 1) * 2 * 16 * 64 * sizeof(float);  // <= 58 KiB
        if (w.type == T_Q4_0) gemm_blk32_kernel<true><<<(unsigned)tiles, 64 * waves, lds, s>>>(w, a, y, (int)tiles_m);
        else gemm_blk32_kernel<false><<<(unsigned)tiles, 64 * waves, lds, s>>>(w, a, y, (int)tiles_m);
    }
    return hipGetLastError();
}

}  // namespace miqmm
