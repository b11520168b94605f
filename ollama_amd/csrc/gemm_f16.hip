// Kernel 3b: prefill GEMM for Q4_K weights on the fp16 matrix cores (v_mfma_f32_32x32x16_f16), for products
// with enough output tiles to fill the machine (the feed-forward matrices at batch 512, every matrix at larger
// batches).  Same numbers as the other kernels behind Tensor.Mulmat (/root/reference/ml/backend.go:151):
// y[n][m] = sum over super-blocks of yd[n] * (d[m] * sum_j sc_j sum_i q_i y_i  -  dmin[m] * sum_j m_j S_j),
// with every integer sum exact.
//
// Why fp16 operands: the 6-bit sub-block scale times the 4-bit quant is a 10-bit integer.  An int8 MFMA needs it
// in two digit planes (two MFMAs per 32 K values and a recombination on the vector ALU); as an fp16 number it is
// exact in one operand, the int8 activations are exact in fp16 too, and the fp32 accumulator holds the sum of a
// whole super-block as an integer scaled by a power of two: exactly while it stays below 2^24 in magnitude (the
// bound 256 * 63 * 15 * 127 is 1.8 times that; a sum that large needs nearly every product at its maximum with
// one sign, and is then rounded to 24 bits once per addition).  16 MFMAs of K = 16 per 32x32 tile
// and super-block, one more for the mins against the activations' block sums, and an epilogue of three vector
// instructions per output and super-block -- against 18 MFMAs and seven in the digit-plane kernel.
//
// Expansion (vector ALU, per weight row and 32 K values: 9 instructions per 8 elements): a nibble left in the low
// mantissa bits of an fp16 word is the subnormal n * 2^-24; one packed multiply by sc * 2^10 (low nibbles) or
// sc * 2^6 (the nibble four bits up) gives sc * n * 2^-14, a normal number with at most ten significant bits.
// The factor 2^14 goes into d.  The mins take the same route (m * 2^-24 times 2^15, 2^9 into dmin).
//
// Activations arrive as fp16 planes written by the quantizer (a.qf: the int8 quants as halves, 32-element
// groups stored [K-step u][lane half h][8 values in the order 0 2 1 3 4 6 5 7], which is the order the
// expansion produces its B operand in; a.bsf: the sixteen block sums of 16 as halves).
//
// Shape: a workgroup of eight waves owns 256 weight rows x 128 activation rows; wave w owns rows 32w.. and all
// 128 activation rows (four 32x32 accumulators), so a row is expanded once per workgroup and its B operand feeds
// four MFMAs.  K advances in chunks of 64 (the 32 quant bytes of a row that hold two sub-blocks): per chunk the
// workgroup stages 128 x 128 B of activations and 256 x 32 B of weights in a ring of four LDS stages, filled by
// direct-to-LDS copies three chunks ahead.  The copies are issued from inline assembly: left to the compiler's
// builtin, every later LDS read would wait for all copies in flight (it cannot tell which stage a read touches);
// here the waits are counted by hand.  One raw s_barrier per chunk, placed in the middle of the chunk so that the
// operands of the next chunk's first K-step can be fetched ahead; LDS reads are pinned one K-step ahead of their
// MFMAs with scheduling barriers (the compiler otherwise sinks them to their use).  The two waves of a SIMD lower
// their priority as they advance past the barrier, so the one behind goes first and both reach the next barrier
// together.
#include <hip/hip_fp16.h>

#include "internal.h"

namespace miqmm {

namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ h2 as_h2(unsigned v) { return __builtin_bit_cast(h2, v); }
__device__ __forceinline__ unsigned as_u(h2 v) { return __builtin_bit_cast(unsigned, v); }
__device__ __forceinline__ float h2f(unsigned bits16) { return __half2float(__ushort_as_half((unsigned short)bits16)); }

// Tile shapes: 256 x 128 (eight waves) where that gives nearly every CU a workgroup; 128 x 64 (four waves) for products
// with fewer outputs -- the 4096-row attention projections at batch 512 are 64 tiles of the first kind and 256 of the
// second.  A wave owns 32 weight rows and all TN activation rows either way; per chunk every wave issues one weight copy
// and two activation copies in both shapes (TN * 128 B over TM / 32 waves), so the hand-counted waits are the same.
constexpr int NST = 4;
template <int TM_, int TN_>
struct F16Tile {
    static constexpr int TM = TM_, TN = TN_, WAVES = TM / 32, NS = TN / 32;
    static_assert(TN * 128 == 2 * WAVES * 1024, "two activation copies per wave and chunk");
    static constexpr int A_STAGE = TN * 128, W_STAGE = TM * 32;
    static constexpr int OFF_A = 0, OFF_W = OFF_A + NST * A_STAGE, OFF_H = OFF_W + NST * W_STAGE, OFF_BS = OFF_H + 2 * TM * 16,
                         OFF_YD = OFF_BS + 2 * TN * 32, OFF_DUMMY = OFF_YD + 2 * TN * 4, LDS_BYTES = OFF_DUMMY + 256;
};

__device__ __forceinline__ const uint8_t *uniform_ptr(const uint8_t *p) {
    const unsigned long long v = (unsigned long long)p;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    return (const uint8_t *)(((unsigned long long)hi << 32) | lo);
}
// direct-to-LDS copy of 64 x 16 (64 x 4) bytes: lane l's piece of base + off lands at lds_addr + 16 l (4 l)
__device__ __forceinline__ void dma16(const uint8_t *base, unsigned off, unsigned lds_addr) {
    base = uniform_ptr(base);
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(lds_addr) : "memory");
}
__device__ __forceinline__ void dma4(const uint8_t *base, unsigned off, unsigned lds_addr) {
    base = uniform_ptr(base);
    lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" ::"v"(off), "s"(base), "s"(lds_addr) : "memory");
}
// wait until at most N vector-memory operations of this wave are outstanding (they retire in order)
template <int N>
__device__ __forceinline__ void wait_vm() {
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// Up to F16_MULTI matrices of one K in a launch (q, k and v of an attention block: too few tiles each, enough
// together): the row tiles of the matrices are numbered through, tile_end[i] is the first tile past matrix i.
constexpr int F16_MULTI = 4;
struct F16Args {
    const uint8_t *W[F16_MULTI];
    float *Y[F16_MULTI];
    int M[F16_MULTI];
    int tile_end[F16_MULTI];
};

template <class T>
__global__ __launch_bounds__(64 * T::WAVES, 2) void gemm_f16_q4k_kernel(F16Args fa, const uint8_t *__restrict__ A,
                                                                        const float *__restrict__ YD, const uint8_t *__restrict__ BS,
                                                                        int N, int K, int tiles_m, int tiles_n) {
    constexpr int TM = T::TM, TN = T::TN, WAVES = T::WAVES, NS = T::NS, A_STAGE = T::A_STAGE, W_STAGE = T::W_STAGE, OFF_A = T::OFF_A,
                  OFF_W = T::OFF_W, OFF_H = T::OFF_H, OFF_BS = T::OFF_BS, OFF_YD = T::OFF_YD, OFF_DUMMY = T::OFF_DUMMY;
    constexpr int HW = WAVES / 2;  // waves that copy weight headers; the other half copies block sums
    __shared__ __attribute__((aligned(1024))) uint8_t lds[T::LDS_BYTES];
    const unsigned lbase = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, h = lane >> 5;
    // row blocks that share activation tiles sit on one XCD (workgroup ids 8 apart share an L2)
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int tile_n = slot % tiles_n, tile_all = xcd + 8 * (slot / tiles_n);
    if (tile_all >= tiles_m) return;  // the grid is rounded up to whole rounds of the 8 XCDs
    const int e0 = fa.tile_end[0], e1 = fa.tile_end[1], e2 = fa.tile_end[2];
    const int t = (tile_all >= e0) + (tile_all >= e1) + (tile_all >= e2);
    const int tile_m = tile_all - (t == 0 ? 0 : t == 1 ? e0 : t == 2 ? e1 : e2);
    const uint8_t *__restrict__ W = t == 0 ? fa.W[0] : t == 1 ? fa.W[1] : t == 2 ? fa.W[2] : fa.W[3];
    float *__restrict__ Y = t == 0 ? fa.Y[0] : t == 1 ? fa.Y[1] : t == 2 ? fa.Y[2] : fa.Y[3];
    const int M = t == 0 ? fa.M[0] : t == 1 ? fa.M[1] : t == 2 ? fa.M[2] : fa.M[3];
    const int nsb = K / QKK;
    const int64_t pitch = (int64_t)nsb * Q4_K_BYTES;
    const int64_t m0 = (int64_t)tile_m * TM, n0 = (int64_t)tile_n * TN;
    const int rows_left = (int)min((int64_t)TM, (int64_t)M - m0);  // rows past M: the last row again, results dropped

    // ---- copy plan: per wave and chunk two activation copies and one weight copy; per super-block one copy of
    // weight headers (the first half of the waves) or block sums (the second half) and one of block scales (the first
    // TN / 64 waves; the others copy to a dummy slot so that every wave counts the same number of operations)
    unsigned aoff[2], woff, soff;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int s = (i * WAVES + wave) * 64 + lane;
        const int row = s >> 3, pp = s & 7;
        aoff[i] = (unsigned)row * (unsigned)(K * 2) + 16u * (pp ^ ((row >> 1) & 7));
    }
    {
        const int s = wave * 64 + lane, wr = s >> 1, hh = s & 1;
        woff = (unsigned)min(wr, rows_left - 1) * (unsigned)pitch + 16u + 16u * (hh ^ ((wr >> 3) & 1));
        const int s4 = (wave % HW) * 64 + lane, brow = s4 >> 1, bh = s4 & 1;
        soff = wave < HW ? (unsigned)min(s4, rows_left - 1) * (unsigned)pitch
                         : (unsigned)brow * (unsigned)(nsb * 32) + 16u * (bh ^ ((brow >> 3) & 1));
    }
    const unsigned ydoff = (unsigned)((wave % (TN / 64)) * 64 + lane) * (unsigned)(nsb * 4);
    const uint8_t *wbase = W + m0 * pitch;
    const uint8_t *abase = A + n0 * (int64_t)K * 2;
    const uint8_t *bsbase = BS + n0 * nsb * 32;
    const uint8_t *ydbase = reinterpret_cast<const uint8_t *>(YD + n0 * nsb);

    auto copy_sb = [&](int sb, int sbslot) __attribute__((always_inline)) {
        if (wave < HW) dma16(wbase + (int64_t)sb * Q4_K_BYTES, soff, lbase + OFF_H + sbslot * (TM * 16) + wave * 1024);
        else dma16(bsbase + (int64_t)sb * 32, soff, lbase + OFF_BS + sbslot * (TN * 32) + (wave - HW) * 1024);
        dma4(ydbase + (int64_t)sb * 4, ydoff, lbase + (wave < TN / 64 ? OFF_YD + sbslot * (TN * 4) + wave * 256 : OFF_DUMMY));
    };
    // a chunk's three copies go out one at a time (part 0: weights, 1 and 2: activations): eight waves issuing all of
    // theirs right behind a barrier queue up at the texture addresser
    auto copy_part = [&](int sb, int c, int part) __attribute__((always_inline)) {
        if (part == 0) dma16(wbase + (int64_t)sb * Q4_K_BYTES + 32 * c, woff, lbase + OFF_W + c * W_STAGE + wave * 1024);
        else dma16(abase + (int64_t)sb * 512 + 128 * c, aoff[part - 1], lbase + OFF_A + c * A_STAGE + ((part - 1) * WAVES + wave) * 1024);
    };

    // ---- read plan (byte offsets into lds).  Reads of 16 bytes are served 16 lanes at a time from 64 banks: the 16
    // lanes must hit 16 different 16-byte slots modulo 256 bytes, hence the XOR of the piece number with row bits.
    const int wrow = 32 * wave + col;
    const int rd_h = OFF_H + wrow * 16;
    const int rd_w = OFF_W + wrow * 32 + 16 * (h ^ ((col >> 3) & 1));
    const int rd_a = OFF_A + col * 128;
    const int asw = (col >> 1) & 7;
    const int rd_bs = OFF_BS + col * 32 + 16 * (h ^ ((col >> 3) & 1));
    const int rd_yd = OFF_YD + 16 * h;

    v16f acc[NS];
    float yacc[NS][16];
#pragma unroll
    for (int a = 0; a < NS; a++)
#pragma unroll
        for (int i = 0; i < 16; i++) { yacc[a][i] = 0.f; acc[a][i] = 0.f; }

    auto load_a = [&](int stage, int t, v8h (&a)[NS]) __attribute__((always_inline)) {
#pragma unroll
        for (int ns = 0; ns < NS; ns++)
            a[ns] = *reinterpret_cast<const v8h *>(lds + rd_a + stage * A_STAGE + ns * 4096 + 16 * ((2 * t + h) ^ asw));
    };

    // prologue: the groups of chunks 0..2 in flight, group 0 landed, first operands in registers
    copy_sb(0, 0);
#pragma unroll
    for (int c = 0; c < 3; c++) { copy_part(0, c, 0); copy_part(0, c, 1); copy_part(0, c, 2); }
    wait_vm<6>();
    __syncthreads();

    float dd = 0.f, dmin = 0.f;
    unsigned sc03 = 0, sc47 = 0;
    v8h bmin;
    v8h a_cur[NS], a_nxt[NS];
    v4u raw_nxt;
    load_a(0, 0, a_nxt);
    raw_nxt = *reinterpret_cast<const v4u *>(lds + rd_w);

    const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 1
    for (int sb = 0; sb < nsb; sb++) {
        const int sbslot = sb & 1;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            if (c == 0) {
                const v4u hd = *reinterpret_cast<const v4u *>(lds + rd_h + sbslot * (TM * 16));
                dd = h2f(hd.x & 0xffff) * 16384.f;
                dmin = h2f(hd.x >> 16) * 512.f;
                // 8 six-bit scales and mins as bytes
                sc03 = hd.y & 0x3f3f3f3fu;
                sc47 = (hd.w & 0x0f0f0f0fu) | (((hd.y >> 6) & 0x03030303u) << 4);
                const unsigned mn03 = hd.z & 0x3f3f3f3fu, mn47 = ((hd.w >> 4) & 0x0f0f0f0fu) | (((hd.z >> 6) & 0x03030303u) << 4);
                // B operand of the block-sum MFMA: K slot s of lane half h is block sum 8h + s, i.e. min 4h + s/2
                const unsigned mw = h ? mn47 : mn03;
                const h2 k15 = {(_Float16)32768.f, (_Float16)32768.f};
                v4u bm;
                bm.x = as_u(as_h2(__builtin_amdgcn_perm(0u, mw, 0x0c000c00u)) * k15);
                bm.y = as_u(as_h2(__builtin_amdgcn_perm(0u, mw, 0x0c010c01u)) * k15);
                bm.z = as_u(as_h2(__builtin_amdgcn_perm(0u, mw, 0x0c020c02u)) * k15);
                bm.w = as_u(as_h2(__builtin_amdgcn_perm(0u, mw, 0x0c030c03u)) * k15);
                bmin = __builtin_bit_cast(v8h, bm);
            }
            const v4u raw = raw_nxt;
            unsigned cpair;  // (sc of sub-block 2c) * 2^10 in the low half, (sc of sub-block 2c+1) * 2^6 in the high half
            {
                const unsigned sw = c < 2 ? sc03 : sc47;
                const unsigned pb = __builtin_amdgcn_perm(0u, sw, (c & 1) ? 0x0c030c02u : 0x0c010c00u);
                const h2 k15 = {(_Float16)32768.f, (_Float16)32768.f}, k16_1 = {(_Float16)16.f, (_Float16)1.f};
                cpair = as_u(((as_h2(pb) * k15) * k15) * k16_1);
            }
            const unsigned sh[4] = {raw.x >> 8, raw.y >> 8, raw.z >> 8, raw.w >> 8};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int u = t & 1, lohi = t >> 1;
#pragma unroll
                for (int ns = 0; ns < NS; ns++) a_cur[ns] = a_nxt[ns];
                if (t == 2) {
                    // The next chunk (group q+1) must have landed in every wave before its operands are fetched below;
                    // one later group (q+2) stays in flight.  After the barrier every wave is past chunk q-1, whose stage
                    // the copies of group q+3 overwrite.  No fence: the LDS reads of that stage fed MFMAs issued long ago.
                    if (((c + 2) & 3) == 0) wait_vm<5>(); else wait_vm<3>();
                    __builtin_amdgcn_s_barrier();
                }
                {   // group q+3 goes out in three parts: at t = 2 (behind the barrier), t = 3 and t = 0 of the next chunk
                    const int part = t == 2 ? 0 : t == 3 ? 1 : t == 0 ? 2 : -1;
                    const int cq = part == 2 ? c + 2 : c + 3;  // chunk the part belongs to, counted from this super-block
                    if (part >= 0 && (sb > 0 || c > 0 || t >= 2)) {
                        const int cn = cq & 3, sbn = min(sb + (cq >> 2), nsb - 1);  // past the end: the last chunk again
                        if (part == 0 && cn == 0) copy_sb(sbn, (sb + 1) & 1);
                        copy_part(sbn, cn, part);
                    }
                }
                // the wave that is behind since the last barrier goes first
                if (t == 2) __builtin_amdgcn_s_setprio(3);
                else if (t == 3) __builtin_amdgcn_s_setprio(2);
                else if (t == 0) __builtin_amdgcn_s_setprio(1);
                else __builtin_amdgcn_s_setprio(0);
                // operands of the next K-step
                if (t < 3) load_a(c, t + 1, a_nxt);
                else {
                    load_a((c + 1) & 3, 0, a_nxt);
                    raw_nxt = *reinterpret_cast<const v4u *>(lds + rd_w + ((c + 1) & 3) * W_STAGE);
                }
                __builtin_amdgcn_sched_barrier(0);
                v8h b;
                {
                    const unsigned mask = lohi ? 0x00f000f0u : 0x000f000fu;
                    const h2 cc = as_h2(cpair);
                    const h2 cs = lohi ? (h2){cc.y, cc.y} : (h2){cc.x, cc.x};
                    const unsigned q0 = u ? raw.z : raw.x, q1 = u ? raw.w : raw.y;
                    v4u bb;
                    bb.x = as_u(as_h2(q0 & mask) * cs);
                    bb.y = as_u(as_h2(sh[2 * u] & mask) * cs);
                    bb.z = as_u(as_h2(q1 & mask) * cs);
                    bb.w = as_u(as_h2(sh[2 * u + 1] & mask) * cs);
                    b = __builtin_bit_cast(v8h, bb);
                }
#pragma unroll
                for (int ns = 0; ns < NS; ns++)
                    acc[ns] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_cur[ns], b, (c == 0 && t == 0) ? zero : acc[ns], 0, 0, 0);
            }
            if (c == 3) {
                // per-super-block epilogue: accumulator i of a lane is activation row 8(i/4) + 4h + i%4, weight row col
#pragma unroll
                for (int ns = 0; ns < NS; ns++) {
                    const v8h am = *reinterpret_cast<const v8h *>(lds + rd_bs + sbslot * (TN * 32) + ns * 1024);
                    float4 yd4[4];
#pragma unroll
                    for (int g = 0; g < 4; g++) yd4[g] = *reinterpret_cast<const float4 *>(lds + rd_yd + sbslot * (TN * 4) + (32 * ns + 8 * g) * 4);
                    const v16f mac = __builtin_amdgcn_mfma_f32_32x32x16_f16(am, bmin, zero, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const float4 y4 = yd4[i >> 2];
                        const float ydv = (i & 3) == 0 ? y4.x : (i & 3) == 1 ? y4.y : (i & 3) == 2 ? y4.z : y4.w;
                        const float tmin = dmin * mac[i];
                        const float uu = __builtin_fmaf(dd, acc[ns][i], -tmin);
                        yacc[ns][i] = __builtin_fmaf(ydv, uu, yacc[ns][i]);
                    }
                }
            }
        }
    }
    __builtin_amdgcn_s_setprio(0);
    wait_vm<0>();  // the copies still in flight target this workgroup's LDS
    const int64_t m = m0 + 32 * wave + col;
    if (m < M) {
#pragma unroll
        for (int ns = 0; ns < NS; ns++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int64_t n = n0 + 32 * ns + 8 * (i >> 2) + 4 * h + (i & 3);
                if (n < N) Y[n * M + m] = yacc[ns][i];
            }
    }
}

}  // namespace

typedef F16Tile<256, 128> TileBig;
typedef F16Tile<128, 64> TileSmall;

namespace {

// which tile shape a launch over these matrices takes: 2 = 256 x 128 when that gives at least three quarters of the CUs a
// workgroup, else 1 = 128 x 64 on the same condition, else 0 (the launch stays on the int8 kernel)
int f16_tile_kind(const DevWeight *ws, int count, int64_t n, int num_cus) {
    int64_t big = 0, small = 0;
    for (int i = 0; i < count; i++) {
        big += (ws[i].M + TileBig::TM - 1) / TileBig::TM * ((n + TileBig::TN - 1) / TileBig::TN);
        small += (ws[i].M + TileSmall::TM - 1) / TileSmall::TM * ((n + TileSmall::TN - 1) / TileSmall::TN);
    }
    if (4 * big >= 3 * (int64_t)num_cus) return 2;
    if (4 * small >= 3 * (int64_t)num_cus) return 1;
    return 0;
}

bool f16_shape_ok(const DevWeight &w, const DevAct &a) {
    if (w.type != T_Q4_K || !a.qf || !a.bsf || w.K < QKK || w.K % QKK || w.M < 1 || a.N <= 64) return false;  // up to 64 rows: the 128 x 64 tiles of the int8 kernel
    return (int64_t)a.N * w.K < ((int64_t)1 << 31) && w.M * (w.K / QKK * Q4_K_BYTES) < ((int64_t)1 << 32);  // 32-bit lane offsets
}

template <class T>
hipError_t launch_tiles(const DevWeight *ws, float *const *ys, int count, const DevAct &a, hipStream_t s) {
    F16Args fa;
    int64_t tiles_m = 0;
    for (int i = 0; i < F16_MULTI; i++) {
        const int j = i < count ? i : count - 1;
        fa.W[i] = ws[j].p0; fa.Y[i] = ys[j]; fa.M[i] = (int)ws[j].M;
        if (i < count) tiles_m += (ws[i].M + T::TM - 1) / T::TM;
        fa.tile_end[i] = i < count ? (int)tiles_m : 0x7fffffff;
    }
    const int64_t tiles_n = (a.N + T::TN - 1) / T::TN;
    const int64_t grid = tiles_n * ((tiles_m + 7) / 8 * 8);  // whole rounds of the 8 XCDs
    if (grid > 0x7fffffff || a.K > 0x7fffffff) return hipErrorInvalidValue;
    gemm_f16_q4k_kernel<T><<<(unsigned)grid, 64 * T::WAVES, 0, s>>>(fa, reinterpret_cast<const uint8_t *>(a.qf), a.d,
                                                                    reinterpret_cast<const uint8_t *>(a.bsf), a.N, (int)a.K, (int)tiles_m,
                                                                    (int)tiles_n);
    return hipGetLastError();
}

}  // namespace

// The kernel pays where its tiles -- 256 x 128, or 128 x 64 for products with fewer outputs -- give (nearly) every CU a
// workgroup; smaller products stay on the int8 kernel.  The choice depends on the weight and the batch only, never on
// what else a call multiplies, so a product's bits do not depend on how it was asked for (both tile shapes and the
// int8 kernel add a row's super-blocks in the same order with the same fp32 expressions).
bool gemm_f16_wanted(const DevWeight &w, const DevAct &a, int num_cus) {
    if (!f16_shape_ok(w, a)) return false;
    const int kind = f16_tile_kind(&w, 1, a.N, num_cus);
    // The small tiles only where the int8 kernel would not cut K: a long K with few tiles (4096 x 14336 at batch 512) is
    // faster there in two K slices (96.6 against 101.3 us); without slices the small tiles win (5120 x 5120 at batch 512:
    // 49.0 against 59.2 us, 8192 x 8192 at 384: 80.8 against 95.1, 4096 x 4096 at 1024: 54.4 against 59.7).
    return kind == 2 || (kind == 1 && gemm_workspace_floats(w.type, w.K, w.M, a.N, num_cus) == 0);
}

// Several matrices in one launch: every matrix Q4_K of one K within the kernel's offset limits, together at least three
// quarters of a tile per CU.  That takes in matrices too small for a launch of their own on this kernel (k and v beside
// q: the int8 kernel such a matrix takes alone computes the same exact integer sums and combines them with the same
// fp32 expressions, so the bits are those of the single launches) and it pays for large ones too: gate + up in one
// launch measured 137.5 against 143.7 us at batch 512 and 527 against 573 at batch 2048 (one launch gap less, and the
// second matrix's tiles fill the CUs the first one's last round leaves idle).
bool gemm_f16_multi_wanted(const DevWeight *ws, int count, const DevAct &a, int num_cus) {
    if (count < 2 || count > F16_MULTI) return false;
    for (int i = 0; i < count; i++)
        if (!f16_shape_ok(ws[i], a) || ws[i].K != ws[0].K) return false;
    const int kind = f16_tile_kind(ws, count, a.N, num_cus);
    for (int i = 0; kind == 1 && i < count; i++)
        if (gemm_workspace_floats(ws[i].type, ws[i].K, ws[i].M, a.N, num_cus) != 0) return false;
    return kind != 0;
}

hipError_t launch_gemm_f16_multi(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int num_cus, hipStream_t s) {
    if (count < 1 || count > F16_MULTI || a.type != T_Q8_K || !a.qf || !a.bsf || a.N < 1) return hipErrorInvalidValue;
    for (int i = 0; i < count; i++)
        if (ws[i].type != T_Q4_K || ws[i].K != a.K || !ys[i] || ws[i].M > 0x7fffffff || ws[i].M < 1) return hipErrorInvalidValue;
    // (a caller that asks for this kernel on a product it is not wanted for gets the large tiles)
    if (f16_tile_kind(ws, count, a.N, num_cus) == 1) return launch_tiles<TileSmall>(ws, ys, count, a, s);
    return launch_tiles<TileBig>(ws, ys, count, a, s);
}

hipError_t launch_gemm_f16(const DevWeight &w, const DevAct &a, float *y, int num_cus, hipStream_t s) {
    if (!y) return hipErrorInvalidValue;
    float *ys[1] = {y};
    return launch_gemm_f16_multi(&w, ys, 1, a, num_cus, s);
}

}  // namespace miqmm
