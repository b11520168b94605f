// Kernel 3c: prefill GEMM for Q6_K weights on the int8 matrix cores (v_mfma_i32_32x32x32_i8), for products with
// enough output tiles -- after cutting K into slices if need be -- to fill the machine (ffn_down at batch 512,
// the output head at prefill).  Same numbers as the other kernels behind Tensor.Mulmat
// (/root/reference/ml/backend.go:151): y[n][m] = sum over super-blocks of yd[n] * d[m] * sum_k sc_g (e_k - 32) y_k,
// every integer sum exact.
//
// As in the 128-row kernel of gemm_mfma.hip the 8-bit scale of a 16-element group is folded into the weights and
// the 13-bit product p = sc * (e - 32) is split into two int8 digits, p = 256 p_h + p_l (p_l the low byte read as
// int8, p_h the high byte of p + 128), which are multiplied separately.  What is different:
//   * The digits come from r = sc * e + (128 - 32 sc), one packed 16-bit multiply-add per two weights: p_h is the high
//     byte of r, p_l its low byte with the top bit flipped.
//   * One accumulator, not two.  All high-digit MFMAs of a super-block come first, the accumulator is shifted left
//     by eight, and the low-digit MFMAs add on top of it: sum = 256 * sum_h + sum_l with 16 registers per 32x32
//     tile instead of 32.  That halves the accumulators and lets a wave cover 128 activation rows (four tiles), so
//     the expansion of a weight row -- by far the largest part of the vector-ALU work -- is shared by four tiles
//     instead of two.  The low digits wait in registers (32 per lane) for their pass; the activations stay in LDS
//     for the whole super-block and are read twice.
//   * The -32 goes into the product itself (one packed subtract), so there are no block-sum MFMAs and no block-sum
//     digit planes.
//   * 256 x 128 tiles, eight waves of 32 x 128, as in the fp16 kernel (gemm_f16.hip): the activations of a
//     super-block (128 x 256 B) double-buffered, the packed weights of half a super-block (ql 256 x 64 B, qh
//     256 x 32 B) in a ring of three, scales / row scales / activation scales per super-block, all by
//     direct-to-LDS copies issued from inline assembly with hand-counted waits; one raw barrier per half
//     super-block.  LDS reads of 16 bytes are laid out for the lanes the hardware serves together.
// Per 32x32 tile and super-block: 16 MFMAs and about 176 vector instructions (370 in the 128-row kernel).
//
// A product whose tiles alone would leave most CUs idle (4096 x 14336 at batch 512: 64 tiles) is cut along K into
// slices, each writing its partial sums to its own [N][M] plane of a workspace; a second kernel adds the planes
// in slice order (deterministic).
#include <hip/hip_fp16.h>

#include "internal.h"

namespace miqmm {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef short s2 __attribute__((ext_vector_type(2)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
__device__ __forceinline__ s2 as_s2(unsigned v) { return __builtin_bit_cast(s2, v); }
__device__ __forceinline__ unsigned as_u(s2 v) { return __builtin_bit_cast(unsigned, v); }
__device__ __forceinline__ float h2f(unsigned bits16) { return __half2float(__ushort_as_half((unsigned short)bits16)); }

constexpr int TM = 256, TN = 128;  // eight waves per workgroup, 32 weight rows each
constexpr int A_BUF = TN * 256;                 // one super-block of activation quants
constexpr int W_QL = TM * 64, W_QH = TM * 32, W_STAGE = W_QL + W_QH;  // one half super-block of packed weights
constexpr int OFF_A = 0, OFF_W = OFF_A + 2 * A_BUF, OFF_SC = OFF_W + 3 * W_STAGE, OFF_D = OFF_SC + 2 * TM * 16,
              OFF_YD = OFF_D + 2 * TM * 4, OFF_DUMMY = OFF_YD + 2 * TN * 4, LDS_BYTES = OFF_DUMMY + 1024;

__device__ __forceinline__ const uint8_t* uniform_ptr(const uint8_t* p) {
    const unsigned long long v = (unsigned long long)p;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    return (const uint8_t*)(((unsigned long long)hi << 32) | lo);
}
__device__ __forceinline__ void dma16(const uint8_t* base, unsigned off, unsigned lds_addr) {
    base = uniform_ptr(base);
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(lds_addr) : "memory");
}
__device__ __forceinline__ void dma4(const uint8_t* base, unsigned off, unsigned lds_addr) {
    base = uniform_ptr(base);
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" ::"v"(off), "s"(base), "s"(lds_addr) : "memory");
}
template <int N> __device__ __forceinline__ void wait_vm() {
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

__global__ __launch_bounds__(512, 2) void gemm_q6k_kernel(const uint8_t *__restrict__ Wql, const uint8_t *__restrict__ Wqh,
                                                          const uint8_t *__restrict__ Wsc, const uint8_t *__restrict__ Wd,
                                                          const uint8_t *__restrict__ A, const float *__restrict__ YD,
                                                          float *__restrict__ Y, int M, int N, int K, int tiles_m, int tiles_n) {
    __shared__ __attribute__((aligned(1024))) uint8_t lds[LDS_BYTES];
    const unsigned lbase = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, h = lane >> 5;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int tile_n = slot % tiles_n, tile_m = xcd + 8 * (slot / tiles_n);
    if (tile_m >= tiles_m) return;
    const int nsb = K / QKK;
    // K slice of this workgroup
    const int sb0 = nsb * blockIdx.y / gridDim.y, sb1 = nsb * (blockIdx.y + 1) / gridDim.y, S = sb1 - sb0;
    const int64_t m0 = (int64_t)tile_m * TM, n0 = (int64_t)tile_n * TN;
    const int rows_left = (int)min((int64_t)TM, (int64_t)M - m0);
    float* __restrict__ Yout = Y + (int64_t)blockIdx.y * N * M;

    // ---- copy plan
    // A (per super-block 128 rows x 256 B = 32 instrs of 1 KiB: 4 per wave): instr j = 4*wave + i covers rows 4j..4j+3, 16 pieces each
    unsigned aoff[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int j = 4 * wave + i, row = 4 * j + (lane >> 4), pos = lane & 15;
        aoff[i] = (unsigned)row * (unsigned)K + 16u * (pos ^ (row & 15));
    }
    // ql (per half 256 rows x 64 B = 16 instrs: 2 per wave): instr j = 2*wave + i covers rows 16j.., 4 pieces each
    unsigned qloff[2], qhoff;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int j = 2 * wave + i, row = 16 * j + (lane >> 2), pos = lane & 3;
        qloff[i] = (unsigned)min(row, rows_left - 1) * (unsigned)(K / 2) + 16u * (pos ^ ((row >> 2) & 3));
    }
    {   // qh (per half 256 rows x 32 B = 8 instrs: 1 per wave): rows 32*wave.., 2 pieces each
        const int row = 32 * wave + (lane >> 1), pos = lane & 1;
        qhoff = (unsigned)min(row, rows_left - 1) * (unsigned)(K / 4) + 16u * (pos ^ ((row >> 3) & 1));
    }
    // per super-block: scales (256 rows x 16 B: waves 0..3, 64 rows each), d (256 rows, the aligned dword: waves 4..7), yd (128 rows: waves 0, 1)
    const int srow = min((wave & 3) * 64 + lane, rows_left - 1);
    const unsigned scoff = (unsigned)srow * (unsigned)(K / 16);
    const int64_t drow = (int64_t)(m0 + srow) * nsb * 2;  // byte offset of the row in the plane of fp16 scales
    const unsigned ydoff = (unsigned)((wave & 1) * 64 + lane) * (unsigned)(nsb * 4);
    const uint8_t *qlbase = Wql + m0 * (K / 2);
    const uint8_t *qhbase = Wqh + m0 * (K / 4);
    const uint8_t *scbase = Wsc + m0 * (K / 16);
    const uint8_t *dbase = Wd;
    const uint8_t* abase = A + n0 * (int64_t)K;
    const uint8_t* ydbase = reinterpret_cast<const uint8_t*>(YD + n0 * nsb);

    auto copy_a = [&](int sb, int part) __attribute__((always_inline)) {  // part 0, 1: two instrs each
        sb = min(sb, sb1 - 1);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int ii = 2 * part + i;
            dma16(abase + (int64_t)sb * 256, aoff[ii], lbase + OFF_A + (sb & 1) * A_BUF + (4 * wave + ii) * 1024);
        }
    };
    auto copy_sb = [&](int sb) __attribute__((always_inline)) {  // two instrs
        sb = min(sb, sb1 - 1);
        const int p = sb & 1;
        if (wave < 4) dma16(scbase + (int64_t)sb * 16, scoff, lbase + OFF_SC + p * 4096 + wave * 1024);
        else {
            // the aligned dword that holds the row's fp16 scale of this super-block
            const unsigned off = (unsigned)((drow + 2 * sb) & ~(int64_t)3);
            dma4(dbase, off, lbase + OFF_D + p * 1024 + (wave - 4) * 256);
        }
        dma4(ydbase + (int64_t)sb * 4, ydoff, lbase + (wave < 2 ? OFF_YD + p * 512 + wave * 256 : OFF_DUMMY));
    };
    auto copy_w = [&](int g) __attribute__((always_inline)) {  // global half index g (relative to sb0): three instrs
        g = min(g, 2 * S - 1);
        const int sb = sb0 + (g >> 1), H = g & 1, st = g % 3;
#pragma unroll
        for (int i = 0; i < 2; i++)
            dma16(qlbase + (int64_t)sb * 128 + 64 * H, qloff[i], lbase + OFF_W + st * W_STAGE + (2 * wave + i) * 1024);
        dma16(qhbase + (int64_t)sb * 64 + 32 * H, qhoff, lbase + OFF_W + st * W_STAGE + W_QL + wave * 1024);
    };

    // ---- read plan
    const int wrow = 32 * wave + col;
    const int rd_ql = OFF_W + wrow * 64, qlsw = (wrow >> 2) & 3;
    const int rd_qh = OFF_W + W_QL + wrow * 32 + 16 * (h ^ ((wrow >> 3) & 1));
    const int rd_sc = OFF_SC + wrow * 16;
    const int rd_d = OFF_D + wrow * 4;
    const int rd_a = OFF_A + col * 256, asw = col & 15;
    const int rd_yd = OFF_YD + 16 * h;
    const int64_t dpar = (m0 + min(wrow, rows_left - 1)) * nsb;  // parity of (dpar + sb) picks the half of the dword

    v16i T[4];
    float yacc[4][16];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int i = 0; i < 16; i++) { yacc[a][i] = 0.f; T[a][i] = 0; }
    v4i BL[8];

    // prologue
    copy_sb(sb0);
    copy_a(sb0, 0); copy_a(sb0, 1);
    copy_w(0);
    copy_w(1);

    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 1
    for (int sbi = 0; sbi < S; sbi++) {
        const int sb = sb0 + sbi, p = sb & 1;
        v4u scv;
#pragma unroll
        for (int H = 0; H < 2; H++) {
            const int g = 2 * sbi + H;
            // W(g) (and at H = 0 this super-block's activations and scales) landed in every wave; the stages copied into below are free
            if (H == 0) wait_vm<3>(); else wait_vm<7>();
            __builtin_amdgcn_s_barrier();
            // copies: next super-block's activations (half of them), its scales at H = 0, the weights two halves ahead
            copy_a(sb + 1, H);
            if (H == 0) copy_sb(sb + 1);
            copy_w(g + 2);
            const int st = g % 3;
            if (H == 0) scv = *reinterpret_cast<const v4u*>(lds + rd_sc + p * 4096);
            const v4u hq = *reinterpret_cast<const v4u*>(lds + rd_qh + st * W_STAGE);
            v4u lq[2];
#pragma unroll
            for (int e = 0; e < 2; e++) lq[e] = *reinterpret_cast<const v4u*>(lds + rd_ql + st * W_STAGE + 16 * ((2 * e + h) ^ qlsw));
#pragma unroll
            for (int rr = 0; rr < 4; rr++) {
                const int s = 4 * H + rr;      // K step of the super-block: elements 32s + 16h .. = scale group 2s + h
                v4i av[4];
#pragma unroll
                for (int ns = 0; ns < 4; ns++)
                    av[ns] = *reinterpret_cast<const v4i*>(lds + rd_a + p * A_BUF + ns * 8192 + 16 * ((2 * s + h) ^ asw));
                // scale of group 2s + h, in both 16-bit lanes
                const unsigned scw = s < 2 ? scv.x : s < 4 ? scv.y : s < 6 ? scv.z : scv.w;
                const int sc = (int)(int8_t)(scw >> (8 * (2 * (s & 1) + h)));
                const s2 sc2 = {(short)sc, (short)sc};
                const short cc = (short)(128 - 32 * sc);
                const s2 c2 = {cc, cc};
                v4i bh, bl;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const unsigned l = lq[rr & 1][i], hh = hq[i];
                    const unsigned nib = (rr >> 1) ? (l >> 4) & 0x0f0f0f0fu : l & 0x0f0f0f0fu;
                    const unsigned hs = rr == 0 ? hh << 4 : rr == 1 ? hh << 2 : rr == 2 ? hh : hh >> 2;
                    const unsigned e = (hs & 0x30303030u) | nib;  // 0..63 per byte
                    // r = sc * (e - 32) + 128 per 16-bit lane (one packed multiply-add): its high byte is the high digit,
                    // its low byte with the top bit flipped the low digit
                    const s2 re = as_s2(e & 0x00ff00ffu) * sc2 + c2;                             // elements 0 and 2
                    const s2 ro = as_s2(__builtin_amdgcn_perm(0u, e, 0x0c030c01u)) * sc2 + c2;   // elements 1 and 3
                    bl[i] = (int)(__builtin_amdgcn_perm(as_u(ro), as_u(re), 0x06020400u) ^ 0x80808080u);
                    bh[i] = (int)__builtin_amdgcn_perm(as_u(ro), as_u(re), 0x07030501u);
                }
                BL[s] = bl;
#pragma unroll
                for (int ns = 0; ns < 4; ns++)
                    T[ns] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[ns], bh, s == 0 ? zero : T[ns], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // all high digits are in: T = 256 * (sum of high-digit products), then the low digits on top
#pragma unroll
        for (int ns = 0; ns < 4; ns++)
#pragma unroll
            for (int i = 0; i < 16; i++) T[ns][i] <<= 8;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            v4i av[4];
#pragma unroll
            for (int ns = 0; ns < 4; ns++)
                av[ns] = *reinterpret_cast<const v4i*>(lds + rd_a + p * A_BUF + ns * 8192 + 16 * ((2 * s + h) ^ asw));
#pragma unroll
            for (int ns = 0; ns < 4; ns++)
                T[ns] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[ns], BL[s], T[ns], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        // epilogue
        const unsigned dpair = *reinterpret_cast<const unsigned*>(lds + rd_d + p * 1024);
        const float dd = h2f(((dpar + sb) & 1) ? dpair >> 16 : dpair & 0xffff);
#pragma unroll
        for (int ns = 0; ns < 4; ns++) {
            float4 yd4[4];
#pragma unroll
            for (int gq = 0; gq < 4; gq++) yd4[gq] = *reinterpret_cast<const float4*>(lds + rd_yd + p * 512 + (32 * ns + 8 * gq) * 4);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float4 y4 = yd4[i >> 2];
                const float ydv = (i & 3) == 0 ? y4.x : (i & 3) == 1 ? y4.y : (i & 3) == 2 ? y4.z : y4.w;
                yacc[ns][i] = __builtin_fmaf(ydv, dd * (float)T[ns][i], yacc[ns][i]);
            }
        }
    }
    wait_vm<0>();
    const int64_t m = m0 + 32 * wave + col;
    if (m < M) {
#pragma unroll
        for (int ns = 0; ns < 4; ns++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int64_t n = n0 + 32 * ns + 8 * (i >> 2) + 4 * h + (i & 3);
                if (n < N) Yout[n * M + m] = yacc[ns][i];
            }
    }
}

// y[i] = sum over slices of part[slice][i], in slice order; V = float4, or float for a y that is not 16-byte aligned
// (a caller's offset into a larger tensor): the same sums in the same order either way
__device__ __forceinline__ void add_to(float4 &a, const float4 &v) { a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w; }
__device__ __forceinline__ void add_to(float &a, const float &v) { a += v; }
template <class V>
__global__ __launch_bounds__(256) void sum_planes_kernel(const V *__restrict__ part, V *__restrict__ y, int64_t n, int slices) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        V acc = part[i];
        for (int sl = 1; sl < slices; sl++) add_to(acc, part[sl * n + i]);
        y[i] = acc;
    }
}

}  // namespace

// 0: this kernel is not the one for the product; otherwise the number of K slices (1: none).  Depends on the
// weight's shape and the batch only.  The kernel pays where its 256 x 128 tiles, times the slices, give at least
// three quarters of the CUs a workgroup, every slice keeping four super-blocks or more.
int gemm_q6k_slices(int type, int64_t K, int64_t M, int64_t N, int num_cus) {
    if (type != T_Q6_K || K < QKK || K % QKK || N <= 64 || M < 1) return 0;  // up to 64 rows: the 128 x 64 tiles of the other kernel
    if (N * K >= ((int64_t)1 << 31) || M * (K / QKK) * 2 >= ((int64_t)1 << 32) || M > 0x7fffffff) return 0;  // 32-bit lane offsets
    const int64_t tiles = (M + TM - 1) / TM * ((N + TN - 1) / TN), nsb = K / QKK;
    int64_t ks = 1;
    if (4 * tiles < 3 * (int64_t)num_cus) {
        ks = num_cus / tiles;
        if (ks > 8) ks = 8;
        if (ks > nsb / 4) ks = nsb / 4;
        if (ks < 1 || (N * M) % 4 != 0) ks = 1;
    }
    return 4 * tiles * ks >= 3 * (int64_t)num_cus ? (int)ks : 0;
}

size_t gemm_q6k_workspace_floats(int type, int64_t K, int64_t M, int64_t N, int num_cus) {
    const int ks = gemm_q6k_slices(type, K, M, N, num_cus);
    return ks > 1 ? (size_t)ks * N * M : 0;
}

hipError_t launch_gemm_q6k(const DevWeight &w, const DevAct &a, float *y, float *workspace, size_t workspace_floats, int num_cus,
                           hipStream_t s) {
    const int ks = gemm_q6k_slices(w.type, w.K, w.M, a.N, num_cus);
    if (!ks || a.type != T_Q8_K || a.K != w.K || !y || !w.p0 || !w.p1 || !w.p2 || !w.d) return hipErrorInvalidValue;
    if (ks > 1 && (!workspace || workspace_floats < (size_t)ks * a.N * w.M)) return hipErrorInvalidValue;
    const int64_t tiles_m = (w.M + TM - 1) / TM, tiles_n = (a.N + TN - 1) / TN;
    const int64_t gx = tiles_n * ((tiles_m + 7) / 8 * 8);  // whole rounds of the 8 XCDs
    if (gx > 0x7fffffff) return hipErrorInvalidValue;
    const dim3 grid((unsigned)gx, (unsigned)ks);
    gemm_q6k_kernel<<<grid, 512, 0, s>>>(w.p0, w.p1, w.p2, reinterpret_cast<const uint8_t *>(w.d), reinterpret_cast<const uint8_t *>(a.qs),
                                         a.d, ks > 1 ? workspace : y, (int)w.M, a.N, (int)w.K, (int)tiles_m, (int)tiles_n);
    if (ks > 1) {
        const bool vec = ((uintptr_t)y & 15) == 0;  // (the slice count itself depends on the shape alone; (N * M) % 4 == 0 here)
        const int64_t n = (int64_t)a.N * w.M / (vec ? 4 : 1);
        const unsigned blocks = (unsigned)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048);
        if (vec) sum_planes_kernel<float4><<<blocks, 256, 0, s>>>(reinterpret_cast<const float4 *>(workspace), reinterpret_cast<float4 *>(y), n, ks);
        else sum_planes_kernel<float><<<blocks, 256, 0, s>>>(workspace, y, n, ks);
    }
    return hipGetLastError();
}

}  // namespace miqmm
