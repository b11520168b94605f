// Kernel 3: prefill GEMM (batch >= 32) on the int8 matrix cores for Q4_K and Q6_K weights.
//
// Computes the same numbers as the GEMV -- y[n][m] = vec_dot(W row m, Q8_K(x row n)), the work behind
// Tensor.Mulmat (/root/reference/ml/backend.go:151) for a prompt batch -- with every integer sum done
// by v_mfma_i32_32x32x32_i8 and exact:
//
//   * The 6-bit (Q4_K) / 8-bit (Q6_K) sub-block scale is folded into the weights, which makes the
//     integer accumulation homogeneous over a whole 256-element super-block instead of over 32 or 16
//     elements, so there is no per-sub-block fix-up on the vector ALU.  The scaled weight does not fit
//     int8, so it is split into two int8 "digit" planes and multiplied twice:
//       Q4_K:  sc = 8*sh + sl  (sh, sl <= 7):  q*sh and q*sl <= 105;   sum sc*q*y = 8*A_h + A_l
//       Q6_K:  p = sc*e (e = 0..63 unsigned 6-bit value, |p| <= 8064) = 256*p_h + p_l in signed digits:
//              p_l = the low byte of p read as int8, p_h = (p + 128) >> 8 in -31..31 -- bytes of the
//              16-bit products, picked by byte permutes;            sum p*y    = 256*A_h + A_l
//   * The terms that multiply sums of activations (Q4_K mins; the -32 offset of Q6_K) use the Q8_K
//     block sums, also on the matrix cores: sum_j m_j * S_j with S split into two int8 digits
//     (S = 64*S_h + S_l) costs two more MFMAs per 32x32 tile and super-block.
//   * Per super-block and output there remains one fp32 epilogue: y += yd_n * (d_m * I - dmin_m * Imin).
//
// Data flow: everything a workgroup multiplies in one super-block step -- 128 rows of packed weights,
// 64 or 128 rows of activation quants, their block scales and block-sum digits -- goes HBM/L2 -> LDS by
// direct-to-LDS loads (global_load_lds: no registers, no vector-ALU work, consecutive lanes fetch
// consecutive 16-byte pieces), two LDS stages, the copy of step sb+1 running under the math of step sb.
// A wave reads the packed blocks of its 32 weight rows from LDS, expands them to digit planes IN
// REGISTERS as the MFMA B operand (a lane needs 16 consecutive K values of one row -- exactly a 16-byte
// piece of the GGUF block) and reuses them for its 32-row activation sub-tiles, which come from LDS as
// the A operand; rows are XOR-swizzled or odd-pitched so that operand reads are conflict-free.  W on
// the B side puts one weight row in each lane's 16 accumulators (one d/dmin per lane) and makes the
// output stores contiguous in m.
#include <hip/hip_fp16.h>


#include <type_traits>

#include "internal.h"

namespace miqmm {

int skinny_waves(int64_t row_groups, int64_t nsb, int num_cus);  // how many waves cut K in a workgroup of the general skinny kernel

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef short s2 __attribute__((ext_vector_type(2)));


__device__ __forceinline__ float h2f(unsigned bits16) { return __half2float(__ushort_as_half((unsigned short)bits16)); }
__device__ __forceinline__ uint4 ld16(const uint8_t *p) { return *reinterpret_cast<const uint4 *>(p); }
__device__ __forceinline__ s2 as_s2(unsigned v) { return __builtin_bit_cast(s2, v); }
__device__ __forceinline__ unsigned as_u(s2 v) { return __builtin_bit_cast(unsigned, v); }
__device__ __forceinline__ v16i mfma(v4i a, v4i b, v16i c) { return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0); }

// The B operand of one wave for one super-block: 8 k-steps of 32, two digit planes, plus the operands
// of the two block-sum MFMAs and the fp32 scales of the lane's weight row.
struct BOperand {
    v4i hi[8], lo[8];
    v4i min_lo, min_hi;
    float d, dmin;
};

// ---- Q4_K --------------------------------------------------------------------------------------
struct GemmQ4K {
    static constexpr int SD = 16;  // bytes of block-sum digits per activation row and super-block
    static __device__ __forceinline__ const uint8_t *digits(const DevAct &a) { return a.sd8; }
    // lane (r = lane%32, h = lane/32): elements 32s+16h.. of k-step s = sub-block s.  Sub-blocks 2c and
    // 2c+1 are the low / high nibbles of qs bytes [32c+16h, +16).
    struct Raw { uint4 hdr, q[4]; };
    // LDS weight stage: the rows' 144-byte blocks back to back, [row][9 pieces of 16 bytes]; copy slot
    // p (16 bytes, consecutive in LDS) holds piece p%9 of row p/9.
    static constexpr int W_PIECES = 9;
    static constexpr int OCC_SMALL = 4;  // waves per SIMD with the 128 x 64 tile: two workgroups share a CU
    static constexpr int W_INSTRS = 3;  // copy instructions per wave: 128 rows x 9 pieces / (8 waves x 64 lanes)
    static __device__ __forceinline__ unsigned w_lane_off(const DevWeight &w, int p, int rows_left) {
        const int rowi = min(p / 9, rows_left - 1), pc = p % 9;
        return (unsigned)rowi * (unsigned)(w.K / QKK * Q4_K_BYTES) + 16u * pc;
    }
    static __device__ __forceinline__ const uint8_t *w_base(const DevWeight &w, int, int64_t m0, int64_t sb) {
        return w.p0 + m0 * (w.K / QKK * Q4_K_BYTES) + sb * Q4_K_BYTES;
    }
    static __device__ __forceinline__ void read_raw(const uint8_t *wt, int rowi, int h, const DevWeight &, int64_t, int64_t,
                                                    Raw &raw) {
        const uint8_t *p = wt + rowi * 144;
        raw.hdr = ld16(p);
#pragma unroll
        for (int c = 0; c < 4; c++) raw.q[c] = ld16(p + 16 + 32 * c + 16 * h);
    }
    static __device__ __forceinline__ void expand(const Raw &raw, int h, BOperand &b) {
        const uint4 hdr = raw.hdr;
        const uint4 *q = raw.q;
        b.d = h2f(hdr.x & 0xffff);
        b.dmin = h2f(hdr.x >> 16);
        // 8 six-bit scales and mins as bytes
        const unsigned sc03 = hdr.y & 0x3f3f3f3fu, sc47 = (hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4);
        const unsigned mn03 = hdr.z & 0x3f3f3f3fu, mn47 = ((hdr.w >> 4) & 0x0f0f0f0fu) | (((hdr.z >> 6) & 0x03030303u) << 4);
        const unsigned shw[2] = {(sc03 >> 3) & 0x07070707u, (sc47 >> 3) & 0x07070707u};
        const unsigned slw[2] = {sc03 & 0x07070707u, sc47 & 0x07070707u};
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const unsigned v[4] = {q[c].x, q[c].y, q[c].z, q[c].w};
#pragma unroll
            for (int half = 0; half < 2; half++) {  // low nibbles: sub-block 2c, high nibbles: 2c+1
                const int j = 2 * c + half;
                const unsigned sh = (shw[j >> 2] >> (8 * (j & 3))) & 0xff, sl = (slw[j >> 2] >> (8 * (j & 3))) & 0xff;
                v4i bh, bl;
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const unsigned nib = half ? (v[t] >> 4) & 0x0f0f0f0fu : v[t] & 0x0f0f0f0fu;
                    bh[t] = (int)(nib * sh);  // four byte products <= 105: no carries between bytes
                    bl[t] = (int)(nib * sl);
                }
                b.hi[j] = bh;
                b.lo[j] = bl;
            }
        }
        // block-sum MFMAs: A rows carry [S_l(0..7) | S_h(0..7)] in the h=0 half and zeros in the h=1 half
        const int mz = h == 0 ? -1 : 0;
        b.min_lo = (v4i){(int)mn03 & mz, (int)mn47 & mz, 0, 0};
        b.min_hi = (v4i){0, 0, (int)mn03 & mz, (int)mn47 & mz};
    }
    // block-sum term of one output, folded right after its two MFMAs so only 16 registers stay live
    static __device__ __forceinline__ float fold_min(float dmin, int xh, int xl) {
        return dmin * (float)((xh << 6) + xl);
    }
    static __device__ __forceinline__ float combine(float d, int ah, int al, float fm) {
        return __builtin_fmaf(d, (float)((ah << 3) + al), -fm);
    }
};

// ---- Q6_K --------------------------------------------------------------------------------------
struct GemmQ6K {
    static constexpr int SD = 32;
    static __device__ __forceinline__ const uint8_t *digits(const DevAct &a) { return a.sd16; }
    // lane (r, h), k-step s: elements 32s+16h.. = scale group 2s+h; half H = s>>2, run rr = s&3:
    // ql bytes [64H + 32(rr&1) + 16h, +16) (low nibble for rr<2, high for rr>=2), qh bytes [32H+16h, +16) >> 2rr.
    struct Raw { uint4 L[2][2], Hq[2], scv; unsigned dh; };
    // LDS weight stage, one region per plane so that every copy instruction reads one plane:
    //   ql [128 rows][8 pieces] at 0, qh [128][4] at 16 KiB, scales [128][1] at 24 KiB.
    // Rows are 128 / 64 bytes apart, which would put a column of 16 rows on two / four bank groups;
    // the piece positions inside a row are XOR-ed with row bits so a 16-row read is conflict-free.
    static constexpr int W_PIECES = 13;
    static constexpr int OCC_SMALL = 2;  // 90 KiB of LDS per workgroup: one per CU whatever the tile
    static constexpr int W_INSTRS = 4;  // 26 KiB of copy slots over 8 waves
    static __device__ __forceinline__ unsigned w_lane_off(const DevWeight &w, int p, int rows_left) {
        if (p < 1024) {
            const int slot_row = p >> 3, pos = p & 7, piece = pos ^ ((slot_row >> 1) & 7);
            return (unsigned)min(slot_row, rows_left - 1) * (unsigned)(w.K / 2) + 16u * piece;
        } else if (p < 1536) {
            const int q = p - 1024, slot_row = q >> 2, pos = q & 3, piece = pos ^ ((slot_row >> 2) & 3);
            return (unsigned)min(slot_row, rows_left - 1) * (unsigned)(w.K / 4) + 16u * piece;
        }
        return (unsigned)min(p - 1536, rows_left - 1) * (unsigned)(w.K / 16);
    }
    static __device__ __forceinline__ const uint8_t *w_base(const DevWeight &w, int blk, int64_t m0, int64_t sb) {
        if (blk < 16) return w.p0 + m0 * (w.K / 2) + sb * 128;
        if (blk < 24) return w.p1 + m0 * (w.K / 4) + sb * 64;
        return w.p2 + m0 * (w.K / 16) + sb * 16;
    }
    static __device__ __forceinline__ void read_raw(const uint8_t *wt, int rowi, int h, const DevWeight &w, int64_t row,
                                                    int64_t sb, Raw &raw) {
        raw.dh = w.d[row * (w.K / QKK) + sb];
        const uint8_t *pl = wt + rowi * 128, *ph = wt + 16384 + rowi * 64;
        const int xl = (rowi >> 1) & 7, xh = (rowi >> 2) & 3;
#pragma unroll
        for (int H = 0; H < 2; H++) {
            raw.L[H][0] = ld16(pl + 16 * ((4 * H + h) ^ xl));
            raw.L[H][1] = ld16(pl + 16 * ((4 * H + 2 + h) ^ xl));
            raw.Hq[H] = ld16(ph + 16 * ((2 * H + h) ^ xh));
        }
        raw.scv = ld16(wt + 24576 + rowi * 16);
    }
    static __device__ __forceinline__ void expand(const Raw &raw, int h, BOperand &b) {
        const uint4 scv = raw.scv;
        const unsigned scw[4] = {scv.x, scv.y, scv.z, scv.w};
        b.d = h2f(raw.dh);
        b.dmin = 0.f;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const int H = s >> 2, rr = s & 3;
            const uint4 lv = raw.L[H][rr & 1], hv = raw.Hq[H];
            const unsigned l[4] = {lv.x, lv.y, lv.z, lv.w}, hq[4] = {hv.x, hv.y, hv.z, hv.w};
            // scale of group g = 2s + h, sign-extended into both 16-bit lanes
            const int g0 = 2 * s, g1 = 2 * s + 1;
            const int sc0 = (int)(int8_t)(scw[g0 >> 2] >> (8 * (g0 & 3))), sc1 = (int)(int8_t)(scw[g1 >> 2] >> (8 * (g1 & 3)));
            const int sc = h ? sc1 : sc0;
            const s2 scv2 = {(short)sc, (short)sc};
            v4i bh, bl;
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const unsigned nib = rr < 2 ? l[t] & 0x0f0f0f0fu : (l[t] >> 4) & 0x0f0f0f0fu;
                const unsigned e = nib | (((hq[t] >> (2 * rr)) & 0x03030303u) << 4);  // 0..63 per byte
                const s2 pe = as_s2(e & 0x00ff00ffu) * scv2;                                 // elements 0 and 2, 16-bit products
                const s2 po = as_s2(__builtin_amdgcn_perm(0u, e, 0x0c030c01u)) * scv2;       // elements 1 and 3
                // signed digits to base 256: the low byte of the product read as int8, and what is left,
                // (product + 128) >> 8 -- the high byte after adding 128.  Digits are bytes: two permutes.
                const s2 half = {128, 128};
                const unsigned re = as_u(pe + half), ro = as_u(po + half);
                bl[t] = (int)__builtin_amdgcn_perm(as_u(po), as_u(pe), 0x06020400u);  // bytes: pe.b0, po.b0, pe.b2, po.b2
                bh[t] = (int)__builtin_amdgcn_perm(ro, re, 0x07030501u);              // bytes: re.b1, ro.b1, re.b3, ro.b3
            }
            b.hi[s] = bh;
            b.lo[s] = bl;
        }
        // block-sum MFMAs: A rows carry S_l(0..15) in the h=0 half and S_h(0..15) in the h=1 half
        const int z0 = h == 0 ? -1 : 0, z1 = ~z0;
        b.min_lo = (v4i){(int)scw[0] & z0, (int)scw[1] & z0, (int)scw[2] & z0, (int)scw[3] & z0};
        b.min_hi = (v4i){(int)scw[0] & z1, (int)scw[1] & z1, (int)scw[2] & z1, (int)scw[3] & z1};
    }
    // sum sc*(e-32)*y = sum sc*e*y - 32 * sum_g sc_g*S_g, all in exact integers
    static __device__ __forceinline__ float fold_min(float, int xh, int xl) {
        return __int_as_float(32 * ((xh << 6) + xl));  // kept as an integer: it joins the main sum exactly
    }
    static __device__ __forceinline__ float combine(float d, int ah, int al, float fm) {
        return d * (float)((ah << 8) + al - __float_as_int(fm));
    }
};

typedef __attribute__((address_space(3))) void lds_ptr_t;
typedef const __attribute__((address_space(1))) void glb_ptr_t;

// Direct-to-LDS copies issued from inline assembly, for kernels that keep several stages in flight and count
// their waits by hand (after the compiler's builtin every later LDS read waits for all copies in flight: it
// cannot tell which stage a read touches).  Lane l's BYTES (16 or 4) at base + off land at lds_address +
// BYTES * l; base and lds_address are wave-uniform.
__device__ __forceinline__ unsigned lds_addr(const void *p) {
    return (unsigned)(uintptr_t)(const __attribute__((address_space(3))) uint8_t *)p;
}
template <int BYTES>
__device__ __forceinline__ void dma_lds(const uint8_t *base, unsigned off, unsigned lds_address) {
    const unsigned long long v = (unsigned long long)base;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    base = (const uint8_t *)(((unsigned long long)hi << 32) | lo);
    lds_address = __builtin_amdgcn_readfirstlane(lds_address);
    if (BYTES == 16)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(lds_address) : "memory");
    else
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(off), "s"(base), "s"(lds_address) : "memory");
}
// LDS reads through a 32-bit LDS address plus a compile-time offset (the offset goes into the instruction)
template <class T>
__device__ __forceinline__ T lds_at(unsigned address, int imm) {
    return *(const __attribute__((address_space(3))) T *)(uintptr_t)(address + (unsigned)imm);
}
__device__ __forceinline__ uint4 lds_u4(unsigned address, int imm) {
    typedef unsigned u4_t __attribute__((ext_vector_type(4)));
    const u4_t v = lds_at<u4_t>(address, imm);
    return make_uint4(v[0], v[1], v[2], v[3]);
}
// wait until at most N vector-memory operations of this wave are outstanding (they retire in order)
template <int N>
__device__ __forceinline__ void wait_vm() {
    static_assert(N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// ---------------------------------------------------------------------------------------------
// Everything through LDS.  Loading the packed weights straight into the lanes that expand them costs a
// wave one memory instruction per 16-byte piece and row -- 32 cache lines per instruction -- and that
// latency sits on the critical path of every super-block.  Here the 128 x 128 tile's packed weights
// travel like the activations: coalesced direct-to-LDS copies (consecutive lanes fetch consecutive
// 16-byte pieces of a row), two LDS stages, the copy of super-block sb+1 running under the math of sb.
// Eight waves (two per SIMD, 256 registers each, MFMA results in ordinary VGPRs): wave (mb, nh) owns
// weight rows 32*mb.. and activation rows 64*nh.. of the tile.
// ---------------------------------------------------------------------------------------------
template <class G, int TN>
struct Stage3 {
    uint8_t q[TN * 256];
    uint8_t s[TN * G::SD];
    float yd[TN < 256 ? 256 : TN];  // keeps the members that follow 1 KiB aligned
    uint8_t wt[128 * 16 * G::W_PIECES];
};

// Up to GEMM_MULTI weight tensors of one type and K against the same activations in one launch (q, k
// and v; gate and up): the grid walks the concatenated 128-row blocks of all of them, which fills the
// machine where a 1024-row k or v projection alone would occupy 32 of 256 CUs.
constexpr int GEMM_MULTI = 4;
struct GemmArgs {
    const uint8_t *p0[GEMM_MULTI], *p1[GEMM_MULTI], *p2[GEMM_MULTI];
    const uint16_t *d[GEMM_MULTI];
    float *y[GEMM_MULTI];
    int64_t M[GEMM_MULTI];
    int tile_end[GEMM_MULTI];  // exclusive end of each tensor's 128-row block range; INT_MAX past the last
    int64_t K;
    int type;
};

// TNT = 32-row activation sub-tiles per wave: the workgroup tile is 128 weight rows x 64*TNT activation rows.
// Expert GEMM (Tensor.MulmatID on a batch, /root/reference/ml/backend.go:153): ga holds one stack of
// expert matrices of expert_rows rows each; the (token, slot) pairs are sorted by expert into runs of whole
// 64- or 128-row tiles (sort_pairs_kernel), tile_n picks a run's tile from the table and with it the expert.  The
// activation planes stay in their own order: every copy gathers its rows through src_rows, and out_rows
// maps a sorted row to the pair whose output row it is.
struct GemmIds {
    const int *tiles;     // null: an ordinary launch
    const int *src_rows;  // sorted row -> row of the activation planes (-1: padding)
    const int *out_rows;  // sorted row -> pair (-1: padding)
    int64_t expert_rows;
};

template <class G, int TNT>
__global__ __launch_bounds__(512, TNT == 1 ? G::OCC_SMALL : 2) void gemm3_kernel(GemmArgs ga, DevAct a, int tiles_m, int tiles_n,
                                                                             float *__restrict__ part, GemmIds gi) {
    constexpr int WAVES = 8, TN = 64 * TNT, TM = 128;
    typedef Stage3<G, TN> StageT;
    __shared__ __attribute__((aligned(1024))) StageT lds[2];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, h = lane >> 5;
    const int mb = wave & 3, nh = wave >> 2;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int tile_n = slot % tiles_n, gtile_m = xcd + 8 * (slot / tiles_n);
    if (gtile_m >= tiles_m) return;  // the grid is rounded up to 8 row blocks
    const int e0 = ga.tile_end[0], e1 = ga.tile_end[1], e2 = ga.tile_end[2];
    const int ti = (gtile_m >= e0) + (gtile_m >= e1) + (gtile_m >= e2);
    const int tile_m = gtile_m - (ti == 0 ? 0 : ti == 1 ? e0 : ti == 2 ? e1 : e2);
#define GEMM_SEL(f) (ti == 0 ? ga.f[0] : ti == 1 ? ga.f[1] : ti == 2 ? ga.f[2] : ga.f[3])
    const DevWeight w{GEMM_SEL(p0), GEMM_SEL(p1), GEMM_SEL(p2), GEMM_SEL(d), ga.K, GEMM_SEL(M), ga.type};
    float *__restrict__ y = GEMM_SEL(y);
#undef GEMM_SEL
    int64_t ldy = w.M, m_rows = w.M, m_stack = 0;  // output pitch, rows of the matrix the tile is in, its first row in w
    int64_t n0 = (int64_t)tile_n * (64 * TNT);
    if (gi.tiles) {
        if (tile_n >= gi.tiles[0]) return;
        const int expert = gi.tiles[1 + 2 * tile_n];
        n0 = gi.tiles[2 + 2 * tile_n];
        ldy = m_rows = gi.expert_rows;
        if (expert < 0) {
            // ids outside the stack: the outputs of these pairs are all NaN
            for (int o = tid; o < 128 * 64 * TNT; o += 512) {
                const int64_t m = (int64_t)tile_m * 128 + (o & 127);
                const int pr = gi.out_rows[n0 + (o >> 7)];
                if (m < m_rows && pr >= 0) y[(int64_t)pr * ldy + m] = __int_as_float(0x7fc00000);
            }
            return;
        }
        m_stack = (int64_t)expert * gi.expert_rows;
    }
    // split K: slice blockIdx.y of gridDim.y covers a contiguous run of super-blocks and writes its
    // partial sums to its own [N][M] plane of part; a second kernel adds the planes up in slice order
    // (deterministic, unlike floating-point atomics).  Single-tensor launches only.
    if (part) y = part + (int64_t)blockIdx.y * a.N * w.M;
    const int64_t m0 = m_stack + (int64_t)tile_m * TM;  // first weight row of the tile
    const int rows_left = (int)min((int64_t)TM, m_rows - (int64_t)tile_m * TM);  // rows past the end: the last row again, results dropped
    const int rowi = min(32 * mb + r, rows_left - 1);
    const int64_t nsb = w.K / QKK;  // row pitch of the planes, in super-blocks
    const int64_t sb_begin = nsb * blockIdx.y / gridDim.y, sb_end = nsb * (blockIdx.y + 1) / gridDim.y;
    const uint8_t *aq = reinterpret_cast<const uint8_t *>(a.qs);
    const uint8_t *asd = G::digits(a);

    float acc[TNT][16];
#pragma unroll
    for (int t = 0; t < TNT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[t][i] = 0.f;

    // ---- copy plan: per-lane 32-bit offsets, uniform bases per super-block
    constexpr int QI = TN / 4 / WAVES;  // quant copies per wave: rows 4*wave + lane/16 + 32*i
    constexpr int RPI = 1024 / G::SD;   // activation rows per digit copy (64 or 32)
    // Row of the activation planes behind tile row t, relative to nbase: the tile's own rows n0 + t, or rows
    // gathered through src_rows (padding: row 0; the host checked that 32-bit byte offsets reach every row).
    const int64_t nbase = gi.tiles ? 0 : n0;
    auto arow_of = [&](int t) -> unsigned {
        if (!gi.tiles) return (unsigned)t;
        const int src = gi.src_rows[n0 + min(t, TN - 1)];
        return src < 0 ? 0u : (unsigned)src;
    };
    unsigned qoff[QI];
#pragma unroll
    for (int i = 0; i < QI; i++) {
        const int R = 4 * wave + (lane >> 4) + 32 * i;
        qoff[i] = arow_of(R) * (unsigned)a.K + 16u * ((lane & 15) ^ (R & 15));
    }
    const unsigned soff = arow_of(RPI * wave + lane / (G::SD / 16)) * (unsigned)(nsb * G::SD) + 16u * (lane % (G::SD / 16));
    unsigned doff[TN / 64];
#pragma unroll
    for (int b = 0; b < TN / 64; b++) doff[b] = arow_of(64 * b + lane) * (unsigned)nsb * 4u;
    unsigned woff[G::W_INSTRS];
#pragma unroll
    for (int j = 0; j < G::W_INSTRS; j++) woff[j] = G::w_lane_off(w, (j * WAVES + wave) * 64 + lane, rows_left);

    auto stage_copy = [&](StageT &st, int64_t sb) __attribute__((always_inline)) {
        // weights
#pragma unroll
        for (int j = 0; j < G::W_INSTRS; j++) {
            const int blk = j * WAVES + wave;  // uniform: which KiB of the weight stage
            if (blk * 64 < 128 * G::W_PIECES) {
                const uint8_t *g = G::w_base(w, blk, m0, sb) + woff[j];
                __builtin_amdgcn_global_load_lds((glb_ptr_t *)g, (lds_ptr_t *)(st.wt + 1024 * blk), 16, 0, 0);
            }
        }
        // block-sum digits: TN / RPI copies, one per wave from wave 0 up
        if (wave < TN / RPI) {
            const uint8_t *g = asd + (nbase * nsb + sb) * G::SD + soff;
            __builtin_amdgcn_global_load_lds((glb_ptr_t *)g, (lds_ptr_t *)(st.s + 1024 * wave), 16, 0, 0);
        }
        // block scales: copies of 64 rows each, by the last waves
        if (wave >= WAVES - TN / 64) {
            const int blk = wave - (WAVES - TN / 64);
            const uint8_t *g = reinterpret_cast<const uint8_t *>(a.d + nbase * nsb + sb) + doff[blk];
            __builtin_amdgcn_global_load_lds((glb_ptr_t *)g, (lds_ptr_t *)(st.yd + 64 * blk), 4, 0, 0);
        }
        // quants
        const uint8_t *qb = aq + nbase * a.K + sb * QKK;
#pragma unroll
        for (int i = 0; i < QI; i++) {
            const uint8_t *g = qb + qoff[i];
            __builtin_amdgcn_global_load_lds((glb_ptr_t *)g, (lds_ptr_t *)(st.q + 1024 * (wave + WAVES * i)), 16, 0, 0);
        }
    };
    const int swz = 16 * (h ^ (r & 15));

    stage_copy(lds[0], sb_begin);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll 1
    for (int64_t sb = sb_begin; sb < sb_end; sb++) {
        StageT &cur = lds[(sb - sb_begin) & 1];
        // the other stage was last read in iteration sb-1 and every wave has passed that barrier
        // (a Q6_K row's fp16 scale is a plain global load: it goes out ahead of the copies, so waiting
        // for it does not mean waiting for them)
        typename G::Raw raw;
        G::read_raw(cur.wt, rowi, h, w, m0 + rowi, sb, raw);
        stage_copy(lds[(sb + 1 - sb_begin) & 1], min(sb + 1, sb_end - 1));
        BOperand b;
        G::expand(raw, h, b);
#pragma unroll
        for (int tt = 0; tt < TNT; tt++) {
            const int t = TNT * nh + tt;  // 32-row activation sub-tile of the stage
            const uint8_t *arow = cur.q + (32 * t + r) * 256;
            const v4i sv = *reinterpret_cast<const v4i *>(cur.s + (32 * t + r) * G::SD + (G::SD == 32 ? 16 * h : 0));
            v4i abuf[3];
            abuf[0] = *reinterpret_cast<const v4i *>(arow + (0 ^ swz));
            abuf[1] = *reinterpret_cast<const v4i *>(arow + (32 ^ swz));
            float4 yd[4];  // block scales of the 32 activation rows: accumulator i is row 8(i/4) + 4h + i%4
#pragma unroll
            for (int gq = 0; gq < 4; gq++) yd[gq] = *reinterpret_cast<const float4 *>(cur.yd + 32 * t + 8 * gq + 4 * h);
            const v16i xl = mfma(sv, b.min_lo, zero);
            const v16i xh = mfma(sv, b.min_hi, zero);
            v16i ah, al;
#pragma unroll
            for (int s = 0; s < 8; s++) {
                if (s + 2 < 8) abuf[(s + 2) % 3] = *reinterpret_cast<const v4i *>(arow + ((32 * (s + 2)) ^ swz));
                const v4i av = abuf[s % 3];
                ah = mfma(av, b.hi[s], s == 0 ? zero : ah);
                al = mfma(av, b.lo[s], s == 0 ? zero : al);
            }
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float4 y4 = yd[i >> 2];
                const float ydv = (i & 3) == 0 ? y4.x : (i & 3) == 1 ? y4.y : (i & 3) == 2 ? y4.z : y4.w;
                const float fm = G::fold_min(b.dmin, xh[i], xl[i]);
                acc[tt][i] = __builtin_fmaf(ydv, G::combine(b.d, ah[i], al[i], fm), acc[tt][i]);
            }
        }
        // this wave's copies have landed; after the barrier so have everybody else's, and nobody still
        // reads the stage that the next iteration overwrites
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
    }

    const int64_t m = (int64_t)tile_m * TM + 32 * mb + r;  // row inside its matrix
    if (m < m_rows) {
#pragma unroll
        for (int tt = 0; tt < TNT; tt++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                int64_t n = n0 + 32 * (TNT * nh + tt) + 8 * (i >> 2) + 4 * h + (i & 3);
                if (gi.tiles) n = gi.out_rows[n];  // sorted row -> pair
                if (n >= 0 && (gi.tiles || n < a.N)) y[n * ldy + m] = acc[tt][i];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Skinny product on the matrix cores: 3..16 activation columns (speculative / small-batch decode).
// The streaming GEMV multiplies every column with its own pass of v_dot4 (about 450 vector
// instructions per row and lane at eight columns) and is vector-ALU bound from three columns up.
//
// v_mfma_i32_16x16x64_i8: the B operand is the weights (lane l: weight row l%16, the 16 K values
// 16*(l/16).. of a 64-wide step -- one K group), unscaled.  A sub-block of the K-quants is one
// (Q6_K) or two (Q4_K) K groups, so the 16 rows of the A operand are spent on columns x sub-blocks:
// row r carries one activation column restricted to the K groups of one sub-block and zeros elsewhere
// (lanes that hold zeros read a zero slot of the stage).  An MFMA then leaves every lane with the
// partial dot products of its column(s) with each sub-block of the step in its four accumulators,
// the sub-block scale is applied there by v_mad_i32_i24, and the min / -32 terms come from one more
// MFMA per column set (block-sum digits x mins or scales).
//
// HBM-bound like the GEMV, so the shape is the GEMV's: many small independent waves.  A workgroup owns
// 16 weight rows, its waves a run of K each (combined through LDS at the very end -- the only
// barrier).  Every wave streams its own packed weights and activation operands through its own two LDS
// stages with direct-to-LDS loads (coalesced: consecutive lanes fetch consecutive 16-byte pieces of a
// row; loading 16-byte pieces of 16 different rows per instruction straight into registers touched 16
// cache lines per instruction and ran at half the speed) and waits on its own memory counter.
// ---------------------------------------------------------------------------------------------
typedef int v4acc __attribute__((ext_vector_type(4)));
__device__ __forceinline__ int mad24(int a, int b, int c) { return __mul24(a, b) + c; }  // v_mad_i32_i24
__device__ __forceinline__ v4acc mfma16(v4i a, v4i b, v4acc c) { return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0); }

// One super-block of a lane's weight row as MFMA operands: the quants of the four 64-wide K steps as they
// are (no scale folded in), the sub-block scales for the vector ALU, the operand of the block-sum MFMA.
template <int NSC>
struct B16 {
    v4i q[4];
    int sc[NSC];  // sub-block scales of the lane's weight row
    v4i bsum;     // B operand of the block-sum MFMA: mins (Q4_K) / scales (Q6_K) in K group 0, zeros elsewhere
    float d, dmin;
};

// ds_read_b128 serves 16 lanes per cycle: lanes 0-3, 12-15, 20-23, 24-27 together, lanes 4-11, 16-19, 28-31
// together, and the same in the upper half of the wave.  With lane = 16g + c the rows c>>2 in {0, 3} of K group g
// therefore share a cycle with the rows c>>2 in {1, 2} of group g ^ 1.  quad_swz maps c>>2 = 0, 1, 2, 3 to 0, 2,
// 3, 1: x ^ quad_swz(j) for j in {0, 3} and (x ^ 1) ^ quad_swz(j) for j in {1, 2} are four different values.
__device__ __forceinline__ int quad_swz(int j) { return (((j >> 1) ^ j) & 1) << 1 | ((j >> 1) & 1); }

struct Sk16Q4K {
    typedef GemmQ4K G;
    static constexpr int W_BYTES = 16 * 144;  // 16 rows x 144 B: two full copy instructions and a quarter of a third
    static constexpr bool SCALES_OUTSIDE = false;  // d and dmin sit in the block header
    static constexpr int W_INSTRS = 3;
    static constexpr int D_LANES_PER_COL = 1;  // 16 digit bytes per activation column and super-block
    // copy slot p (16 bytes) of the weight stage holds piece p%9 of row p/9 -- with the two halves of every 32-byte
    // run of quants swapped in the rows p/9 = 4..11 (half_swz): the lanes that one LDS cycle serves are rows 0-3 and
    // 12-15 of K group g and rows 4-11 of group g ^ 1, which want opposite halves of their rows' runs; after the
    // swap they all read the same position of sixteen different rows, and rows are 9 pieces (an odd number) apart.
    static __device__ __forceinline__ int half_swz(int row) { return ((row >> 2) ^ (row >> 3)) & 1; }
    static __device__ __forceinline__ void w_plan(const DevWeight &w, int j, int lane, int rows_left, unsigned &off, bool &on) {
        const int p = 64 * j + lane;
        on = p < 16 * 9;
        const int pp = on ? p : 0, row = pp / 9, pc = pp % 9;
        const int src = pc == 0 ? 0 : 1 + ((pc - 1) ^ half_swz(row));
        off = (unsigned)min(row, rows_left - 1) * (unsigned)(w.K / QKK * Q4_K_BYTES) + 16u * src;
    }
    static __device__ __forceinline__ const uint8_t *w_base(const DevWeight &w, int, int64_t m0, int64_t sb) {
        return w.p0 + m0 * (w.K / QKK * Q4_K_BYTES) + sb * Q4_K_BYTES;
    }
    // step t covers sub-blocks 2t (low nibbles of qs bytes [32t, 32t+32)) and 2t+1 (high nibbles); K group
    // g of the step is elements 16(g&1).. of sub-block 2t + (g>>1): bytes [32t + 16(g&1), +16), nibble g>>1
    struct Raw { uint4 hdr, q[4]; };
    // the lane's read offsets into a weight stage (header; first run of quants), then the reads of one super-block
    // from absolute LDS addresses plus a compile-time offset
    static constexpr int NRO = 2;
    static __device__ __forceinline__ void read_plan(int c, int g, unsigned (&ro)[NRO]) {
        ro[0] = c * 144;
        ro[1] = c * 144 + 16 + 16 * ((g & 1) ^ half_swz(c));
    }
    static __device__ __forceinline__ void read(const unsigned (&wa)[NRO], int imm, Raw &raw) {
        raw.hdr = lds_u4(wa[0], imm);
#pragma unroll
        for (int t = 0; t < 4; t++) raw.q[t] = lds_u4(wa[1], imm + 32 * t);
    }
    static __device__ __forceinline__ void read(const uint8_t *wt, int c, int g, Raw &raw) {
        const uint8_t *p = wt + c * 144;
        raw.hdr = ld16(p);
#pragma unroll
        for (int t = 0; t < 4; t++) raw.q[t] = ld16(p + 16 + 32 * t + 16 * ((g & 1) ^ half_swz(c)));
    }
    // A sub-block is 32 elements = two K groups of a step, so the 16 rows of the A operand are 8 columns x
    // the two sub-blocks of the step: row r is column r>>1 restricted to sub-block r&1 (K groups 2(r&1),
    // 2(r&1)+1; the other two are zero).  The outputs of lane l are then rows 4(l>>4) + v = columns
    // 2(l>>4), 2(l>>4)+1 x sub-blocks 2t, 2t+1: four partial dot products that take their 6-bit scale
    // on the vector ALU.
    static constexpr int SET_COLS = 8, LANE_COLS = 2, NSC = 8;
    typedef B16<NSC> Ops;
    static __device__ __forceinline__ int a_col(int r) { return r >> 1; }
    static __device__ __forceinline__ bool a_on(int r, int g) { return (g >> 1) == (r & 1); }
    // A stage: piece p of column col sits at position p ^ a_swz(col).  The lanes of one LDS cycle that read real
    // pieces hold the eight columns of a set, pieces 4t + g and 4t + (g ^ 1): eight slots of one half of the 256
    // bytes; the lanes that read zeros go to the other half.
    static __device__ __forceinline__ int a_swz(int col) { return col & 15; }
    static __device__ __forceinline__ int a_zero(int cs, int t) { return 128 * (((t >> 1) ^ cs ^ 1) & 1); }
    static __device__ __forceinline__ int lane_col(int lg, int u) { return 2 * lg + u; }
    static __device__ __forceinline__ void expand(const Raw &raw, int g, unsigned, Ops &b) {
        const uint4 hdr = raw.hdr;
        b.d = h2f(hdr.x & 0xffff);
        b.dmin = h2f(hdr.x >> 16);
        const unsigned sc03 = hdr.y & 0x3f3f3f3fu, sc47 = (hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4);
        const unsigned mn03 = hdr.z & 0x3f3f3f3fu, mn47 = ((hdr.w >> 4) & 0x0f0f0f0fu) | (((hdr.z >> 6) & 0x03030303u) << 4);
#pragma unroll
        for (int j = 0; j < 8; j++) b.sc[j] = (int)(((j < 4 ? sc03 : sc47) >> (8 * (j & 3))) & 0xff);
        const int hiN = g >> 1;  // 0: low nibbles (sub-block 2t), 1: high nibbles (sub-block 2t+1)
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const unsigned v[4] = {raw.q[t].x, raw.q[t].y, raw.q[t].z, raw.q[t].w};
#pragma unroll
            for (int i = 0; i < 4; i++) b.q[t][i] = (int)((v[i] >> (4 * hiN)) & 0x0f0f0f0fu);
        }
        // block-sum MFMA: mins 0..7 in the first eight K slots, against the digits of the eight 32-element sums
        // in the same slots of the A rows (K group 0 only: in the other groups the A operand is zero, so what
        // the B operand holds there does not matter)
        b.bsum = (v4i){(int)mn03, (int)mn47, 0, 0};
    }
    // outputs v of a step's MFMA -> the lane's two columns
    static __device__ __forceinline__ void scale_step(const v4acc &dv, int t, const Ops &b, int (&isum)[LANE_COLS]) {
        isum[0] = mad24(b.sc[2 * t], dv[0], mad24(b.sc[2 * t + 1], dv[1], isum[0]));
        isum[1] = mad24(b.sc[2 * t], dv[2], mad24(b.sc[2 * t + 1], dv[3], isum[1]));
    }
    // Block-sum operand: row r carries, in K group 0, the low (r even) or high (r odd) digits of column
    // r>>1's eight sums; the stage holds [S_l(0..7) | S_h(0..7)] per column.
    static __device__ __forceinline__ bool d_on(int r, int g) { return g == 0; }
    static __device__ __forceinline__ int d_off(int r) { return 0; }
    static __device__ __forceinline__ v4i d_fix(v4i raw, int r) {
        return (r & 1) ? (v4i){raw[2], raw[3], 0, 0} : (v4i){raw[0], raw[1], 0, 0};
    }
    // y contribution of one column and super-block, without the activation scale
    static __device__ __forceinline__ float finish(const Ops &b, int isum, const v4acc &x, int u) {
        const float fm = G::fold_min(b.dmin, x[2 * u + 1], x[2 * u]);
        return __builtin_fmaf(b.d, (float)isum, -fm);
    }
};

struct Sk16Q6K {
    typedef GemmQ6K G;
    static constexpr int W_BYTES = 3 * 1024 + 256;  // ql 2 KiB, qh 1 KiB, scales 256 B
    static constexpr bool SCALES_OUTSIDE = true;  // the row's fp16 scale is a plane of its own
    static constexpr int W_INSTRS = 4;
    static constexpr int D_LANES_PER_COL = 2;  // 32 digit bytes per activation column and super-block
    // stage regions: ql [16 rows][8 pieces] at 0, qh [16][4] at 2 KiB, scales [16][1] at 3 KiB; piece
    // positions XOR-ed with row bits so that the 16 rows of a read fall on distinct banks
    static __device__ __forceinline__ void w_plan(const DevWeight &w, int j, int lane, int rows_left, unsigned &off, bool &on) {
        on = true;
        if (j < 2) {
            const int q = 64 * j + lane, slot_row = q >> 3, pos = q & 7, piece = pos ^ ((slot_row >> 1) & 7);
            off = (unsigned)min(slot_row, rows_left - 1) * (unsigned)(w.K / 2) + 16u * piece;
        } else if (j == 2) {
            const int slot_row = lane >> 2, pos = lane & 3, piece = pos ^ quad_swz(slot_row >> 2);
            off = (unsigned)min(slot_row, rows_left - 1) * (unsigned)(w.K / 4) + 16u * piece;
        } else {
            on = lane < 16;
            off = (unsigned)min(on ? lane : 0, rows_left - 1) * (unsigned)(w.K / 16);
        }
    }
    static __device__ __forceinline__ const uint8_t *w_base(const DevWeight &w, int j, int64_t m0, int64_t sb) {
        if (j < 2) return w.p0 + m0 * (w.K / 2) + sb * 128;
        if (j == 2) return w.p1 + m0 * (w.K / 4) + sb * 64;
        return w.p2 + m0 * (w.K / 16) + sb * 16;
    }
    // step t, K group g = scale group 4t + g (16 elements).  With H = t>>1, rr = 2(t&1) + (g>>1):
    // ql bytes [64H + 32(g>>1) + 16(g&1), +16) = piece 4H + g, nibble t&1; qh bytes [32H + 16(g&1), +16) >> 2rr.
    struct Raw { uint4 L[2], Hq[2], scv; };
    // the lane's read offsets into a weight stage: ql of half H at ro[H], qh at ro[2 + H], scales at ro[4]
    static constexpr int NRO = 5;
    static __device__ __forceinline__ void read_plan(int c, int g, unsigned (&ro)[NRO]) {
        const int xl = (c >> 1) & 7, xh = quad_swz(c >> 2);
#pragma unroll
        for (int H = 0; H < 2; H++) {
            ro[H] = c * 128 + 16 * ((4 * H + g) ^ xl);
            ro[2 + H] = 2048 + c * 64 + 16 * ((2 * H + (g & 1)) ^ xh);
        }
        ro[4] = 3072 + c * 16;
    }
    static __device__ __forceinline__ void read(const uint8_t *wt, int c, int g, Raw &raw) {
        const int xl = (c >> 1) & 7, xh = quad_swz(c >> 2);
#pragma unroll
        for (int H = 0; H < 2; H++) {
            raw.L[H] = ld16(wt + c * 128 + 16 * ((4 * H + g) ^ xl));
            raw.Hq[H] = ld16(wt + 2048 + c * 64 + 16 * ((2 * H + (g & 1)) ^ xh));
        }
        raw.scv = ld16(wt + 3072 + c * 16);
    }
    // A stage: piece p of column col sits at position p ^ a_swz(col).  The lanes of one LDS cycle that read real
    // pieces are rows {0, 12} of K group g and rows {5, 9} of group g ^ 1 (or the other way round): columns 4cs +
    // {0, 3} with piece 4t + g and 4cs + {1, 2} with piece 4t + (g ^ 1); quad_swz puts them on four different slots
    // of the block 4(t ^ cs), and the lanes that read zeros go to the block next to it.
    static __device__ __forceinline__ int a_swz(int col) { return (col & 12) | quad_swz(col); }
    static __device__ __forceinline__ int a_zero(int cs, int t) { return 64 * ((t ^ cs ^ 1) & 3); }
    // A sub-block is 16 elements = one K group of a step, so the 16 rows of the A operand are 4 columns x
    // the four sub-blocks of the step: row r is column r>>2 restricted to K group r&3.  The outputs of
    // lane l are rows 4(l>>4) + v = column l>>4 x sub-blocks 4t + v.
    static constexpr int SET_COLS = 4, LANE_COLS = 1, NSC = 16;
    typedef B16<NSC> Ops;
    static __device__ __forceinline__ int a_col(int r) { return r >> 2; }
    static __device__ __forceinline__ bool a_on(int r, int g) { return g == (r & 3); }
    static __device__ __forceinline__ int lane_col(int lg, int) { return lg; }
    static __device__ __forceinline__ void expand(const Raw &raw, int g, unsigned dh, Ops &b) {
        const unsigned scw[4] = {raw.scv.x, raw.scv.y, raw.scv.z, raw.scv.w};
        b.d = h2f(dh);
        b.dmin = 0.f;
#pragma unroll
        for (int j = 0; j < 16; j++) b.sc[j] = (int)(int8_t)(scw[j >> 2] >> (8 * (j & 3)));
        // Per pair of words (ql word l; qh word hq shifted so that the lane's two bit pairs sit at bits 0-1 and
        // 4-5 of every byte): step 2H takes the low nibbles and the pair at bits 0-1, step 2H+1 the high nibbles
        // and the pair at bits 4-5 -- seven instructions for eight bytes of operand.  0..63 per byte; the -32
        // goes through the block sums.
        const unsigned sh = 2 * (g >> 1);
#pragma unroll
        for (int H = 0; H < 2; H++) {
            const unsigned l[4] = {raw.L[H].x, raw.L[H].y, raw.L[H].z, raw.L[H].w};
            const unsigned hq[4] = {raw.Hq[H].x, raw.Hq[H].y, raw.Hq[H].z, raw.Hq[H].w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const unsigned hs = hq[i] >> sh;
                b.q[2 * H][i] = (int)(((hs & 0x03030303u) << 4) | (l[i] & 0x0f0f0f0fu));
                b.q[2 * H + 1][i] = (int)((hs & 0x30303030u) | ((l[i] >> 4) & 0x0f0f0f0fu));
            }
        }
        // block-sum MFMA: the 16 scales against the digits of the sixteen 16-element sums (K group 0 only: in
        // the other groups the A operand is zero, so what the B operand holds there does not matter)
        b.bsum = (v4i){(int)scw[0], (int)scw[1], (int)scw[2], (int)scw[3]};
    }
    static __device__ __forceinline__ void scale_step(const v4acc &dv, int t, const Ops &b, int (&isum)[LANE_COLS]) {
        isum[0] = mad24(b.sc[4 * t], dv[0], mad24(b.sc[4 * t + 1], dv[1], mad24(b.sc[4 * t + 2], dv[2],
                  mad24(b.sc[4 * t + 3], dv[3], isum[0]))));
    }
    // Block-sum operand: row r carries, in K group 0, the low (r&3 == 0) or high (r&3 == 1) digits of
    // column r>>2's sixteen sums; the stage holds [S_l(0..15) | S_h(0..15)] per column.
    static __device__ __forceinline__ bool d_on(int r, int g) { return g == 0 && (r & 3) < 2; }
    static __device__ __forceinline__ int d_off(int r) { return 16 * (r & 1); }
    static __device__ __forceinline__ v4i d_fix(v4i raw, int) { return raw; }
    static __device__ __forceinline__ float finish(const Ops &b, int isum, const v4acc &x, int) {
        return b.d * (float)(isum - 32 * ((x[1] << 6) + x[0]));  // sum sc*(e-32)*y = sum sc*e*y - 32 sum_g sc_g*S_g
    }
};


// NCT = activation columns the stages are laid out for (8 or 16)
template <class S, int NCT, int NST = 2>
struct SkinnyGeo {
    static constexpr int A_BYTES = NCT * 256, A_INSTRS = NCT / 4;
    static constexpr int D_BYTES = 16 * NCT * S::D_LANES_PER_COL, Y_BYTES = 4 * NCT;
    // A stage starts with 256 zero bytes that no copy ever writes (the lanes of an operand read that carry zeros
    // pick the 16 of them that share no bank with the lanes that carry data), then weights, activation quants,
    // block-sum digits, activation scales, and (Q6_K) per row the aligned dword that holds its fp16 super-block scale.
    static constexpr int Z_BYTES = 256;
    static constexpr int W_OFF = Z_BYTES, A_OFF = W_OFF + S::W_BYTES, D_OFF = A_OFF + A_BYTES, Y_OFF = D_OFF + D_BYTES;
    static constexpr int DH_OFF = Y_OFF + Y_BYTES;
    static constexpr int STAGE = (DH_OFF + (S::SCALES_OUTSIDE ? 64 : 0) + 255) / 256 * 256;  // stages keep the 256-byte phase
    static constexpr int SETS = NCT / S::SET_COLS, LANE_ACC = SETS * S::LANE_COLS;  // column sets; outputs per lane
    static constexpr int NDMA = S::W_INSTRS + A_INSTRS + 2 + (S::SCALES_OUTSIDE ? 1 : 0);  // copy instructions per stage
    static constexpr int NSTAGE = NST;  // stages in a wave's ring: NSTAGE - 1 super-blocks in flight behind the one being multiplied
    static constexpr int WAVE_BYTES = (NSTAGE * STAGE + 255) / 256 * 256;
    static constexpr int PART_BYTES = 16 * 16 * 4;  // per wave: its partial sums
};

// Expert-indexed launches (Tensor.MulmatID, /root/reference/ml/backend.go:153): w is a stack of expert
// matrices of M rows each, a workgroup belongs to one group of up to 16 (token, slot) pairs that all
// name the same expert, takes its activation columns from the pairs and writes y[pair][row].
struct SkinnyIds {
    const int *groups;  // groups[0] = number of groups, then records {expert or -1, count, pair[16]}
    int64_t M;          // rows per expert
    int wgs_per_group, n_used, b_cols;
};
constexpr int SKINNY_ID_REC = 2 + 16;

// Several matrices of one type and K against the same activations in one launch (q, k, v; gate, up): their
// 16-row groups are numbered through, matrix 0 is the kernel's w and y, the others come in this block, and
// a work item finds its matrix by comparing its group number with the ends of the runs.
struct SkinnyMulti {
    const uint8_t *p0[3], *p1[3], *p2[3];
    const uint16_t *d[3];
    float *y[3];
    int64_t M[3];
    int grp_end[3];  // exclusive ends of the runs of matrices 0, 1, 2; INT_MAX past the last matrix
    int groups_total;
};
struct SkinnyWhere { DevWeight w; float *y; int first; };
template <bool MULTI>
__device__ __forceinline__ SkinnyWhere skinny_where(const DevWeight &w0, float *y0, const SkinnyMulti &mt, int group) {
    SkinnyWhere x{w0, y0, 0};
    if (!MULTI) return x;
#pragma unroll
    for (int t = 0; t < 3; t++)
        if (group >= mt.grp_end[t]) {
            x.w.p0 = mt.p0[t]; x.w.p1 = mt.p1[t]; x.w.p2 = mt.p2[t]; x.w.d = mt.d[t]; x.w.M = mt.M[t];
            x.y = mt.y[t];
            x.first = mt.grp_end[t];
        }
    return x;
}

// The number of waves per workgroup (how many ways K is cut) is the launch's block size / 64.
template <class S, int NCT, bool ID, int NST, bool MULTI = false>
__global__ __launch_bounds__(512, (NCT / S::SET_COLS >= 4 ? 2 : 4)) void skinny_kernel(DevWeight w_in, DevAct a_in, int col0, int nc, float *__restrict__ y_in,
                                                        SkinnyIds si_in, int WAVES, int grid_size, SkinnyMulti mt) {
    static_assert(!(ID && MULTI), "expert-indexed launches take one stack");
    typedef typename S::G G;
    typedef SkinnyGeo<S, NCT, NST> Geo;
    constexpr int A_INSTRS = Geo::A_INSTRS;
    constexpr int STAGE = Geo::STAGE, NDMA = Geo::NDMA, WAVE_BYTES = Geo::WAVE_BYTES;
    // The whole argument block in one batch of scalar loads: every value is named here and pinned by an
    // empty asm (left alone the compiler fetches them where each branch first needs them, four or five
    // dependent rounds before the first copy is issued).  Pointers go through as global-address-space
    // pointers so that they stay known to be global; the block and grid sizes are arguments (WAVES,
    // grid_size) rather than reads of the hidden arguments.
    typedef const __attribute__((address_space(1))) uint8_t *gbytes_t;
    typedef const __attribute__((address_space(1))) uint16_t *ghalves_t;
    typedef const __attribute__((address_space(1))) int8_t *gi8_t;
    typedef const __attribute__((address_space(1))) int16_t *gi16_t;
    typedef const __attribute__((address_space(1))) float *gcfloats_t;
    typedef const __attribute__((address_space(1))) int *gcints_t;
    typedef __attribute__((address_space(1))) float *gfloats_t;
    typedef int ints4_t __attribute__((ext_vector_type(4)));
    typedef long longs2_t __attribute__((ext_vector_type(2)));
    gbytes_t p0 = (gbytes_t)w_in.p0, p1 = (gbytes_t)w_in.p1, p2 = (gbytes_t)w_in.p2, sd8 = (gbytes_t)a_in.sd8, sd16 = (gbytes_t)a_in.sd16;
    ghalves_t wd = (ghalves_t)w_in.d;
    gi8_t aqs = (gi8_t)a_in.qs;
    gcfloats_t ad = (gcfloats_t)a_in.d;
    gi16_t ab = (gi16_t)a_in.bsums;
    gcints_t groups = (gcints_t)si_in.groups;
    gfloats_t yg = (gfloats_t)y_in;
    longs2_t km = {(long)w_in.K, (long)w_in.M}, km2 = {(long)a_in.K, (long)si_in.M};
    ints4_t i0 = {col0, nc, WAVES, grid_size}, i1 = {si_in.wgs_per_group, si_in.n_used, si_in.b_cols, a_in.N};
    asm volatile("" : "+s"(p0), "+s"(p1), "+s"(p2), "+s"(sd8), "+s"(sd16), "+s"(wd), "+s"(aqs), "+s"(ad), "+s"(ab), "+s"(groups),
                      "+s"(yg), "+s"(km), "+s"(km2), "+s"(i0), "+s"(i1));
    const DevWeight w0{(const uint8_t *)p0, (const uint8_t *)p1, (const uint8_t *)p2, (const uint16_t *)wd, km[0], km[1], w_in.type};
    const DevAct a{(const int8_t *)aqs, (const float *)ad, (const int16_t *)ab, (const uint8_t *)sd8, (const uint8_t *)sd16, km2[0],
                   i1[3], a_in.type};
    const SkinnyIds si{(const int *)groups, km2[1], i1[0], i1[1], i1[2]};
    float *const y0 = (float *)yg;
    col0 = i0[0]; nc = i0[1]; WAVES = i0[2]; grid_size = i0[3];
    // the matrix of the item being multiplied (w, y) and of the item being copied (cw)
    const SkinnyWhere at0 = skinny_where<MULTI>(w0, y0, mt, (int)blockIdx.x);
    DevWeight w = at0.w, cw = at0.w;
    float *y = at0.y;
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];  // WAVES x (WAVE_BYTES + PART_BYTES)
    float (*part)[16][16] = reinterpret_cast<float (*)[16][16]>(smem + WAVES * WAVE_BYTES);

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, g = lane >> 4;
    int64_t m0 = (int64_t)((int)blockIdx.x - at0.first) * 16, yrow0 = m0, ldy = w.M;
    int rows_left = (int)min((int64_t)16, w.M - m0);  // rows past M: the last row again, results dropped
    const int *rec = nullptr;
    if (ID) {
        const int group = blockIdx.x / si.wgs_per_group;
        if (group >= si.groups[0]) return;
        rec = si.groups + 1 + (size_t)group * SKINNY_ID_REC;
        const int expert = rec[0];
        nc = rec[1];
        yrow0 = (int64_t)(blockIdx.x - group * si.wgs_per_group) * 16;  // row inside the expert
        rows_left = (int)min((int64_t)16, si.M - yrow0);
        ldy = si.M;
        if (expert < 0) {
            // ids outside the stack: these pairs' outputs are all NaN
            for (int o = tid; o < 16 * nc; o += (64 * WAVES))
                if ((o & 15) < rows_left) y[(int64_t)rec[2 + (o >> 4)] * ldy + yrow0 + (o & 15)] = __int_as_float(0x7fc00000);
            return;
        }
        m0 = (int64_t)expert * si.M + yrow0;
    }
    // activation column (row of a) behind the launch's column i
    auto acol = [&](int i) {
        i = min(i, nc - 1);
        if (!ID) return col0 + i;
        const int pair = rec[2 + i], tok = pair / si.n_used;
        return tok * si.b_cols + (pair - tok * si.n_used) % si.b_cols;
    };
    const int64_t nsb = w.K / QKK;
    const int64_t sb0 = nsb * wave / WAVES, sb1 = nsb * (wave + 1) / WAVES;  // this wave's run of super-blocks
    uint8_t *wsm = smem + wave * WAVE_BYTES;
    // Work items: the 16-row groups this workgroup goes through, blockIdx.x + k * grid_size (an
    // expert-indexed launch has exactly one per workgroup).  The copy stream runs two stages ahead of
    // the math and simply continues into the next item, so only the first item pays the pipeline fill.
    const int64_t total_items = ID ? 0 : MULTI ? mt.groups_total : (w.M + 15) / 16;
    const int64_t items = ID ? 1 : (total_items - blockIdx.x + grid_size - 1) / grid_size;

    // ---- copy plan: per-lane 32-bit offsets, uniform bases per super-block
    unsigned woff[S::W_INSTRS];
    int64_t dhrow = 0;  // byte offset of the lane's row in the plane of fp16 super-block scales
    bool won[S::W_INSTRS];
    int64_t cp_m0 = m0, cp_k = 0, cp_sb = sb0;  // the copy cursor: item (its first row) and super-block
    auto plan_item = [&](int64_t first_row, int rows) __attribute__((always_inline)) {
        cp_m0 = first_row;
#pragma unroll
        for (int j = 0; j < S::W_INSTRS; j++) S::w_plan(cw, j, lane, rows, woff[j], won[j]);
        dhrow = (first_row + min(c, rows - 1)) * nsb * 2;
    };
    plan_item(m0, rows_left);
    unsigned aoff[A_INSTRS];
#pragma unroll
    for (int j = 0; j < A_INSTRS; j++) {
        const int col = 4 * j + (lane >> 4), slot = lane & 15;  // stage slot [col][slot] holds piece slot ^ a_swz(col)
        aoff[j] = (unsigned)acol(col) * (unsigned)a.K + 16u * (slot ^ S::a_swz(col));
    }
    const int dcol = lane / S::D_LANES_PER_COL;
    const bool don = lane < NCT * S::D_LANES_PER_COL, yon = lane < NCT;
    const unsigned doff = (unsigned)acol(dcol) * (unsigned)(nsb * G::SD) + 16u * (lane % S::D_LANES_PER_COL);
    const unsigned yoff = (unsigned)acol(lane) * (unsigned)nsb * 4u;
    const uint8_t *aq = reinterpret_cast<const uint8_t *>(a.qs);
    const uint8_t *asd = G::digits(a);

    // one stage = everything the wave multiplies in one super-block; then the cursor moves on (past the
    // last super-block of the last item it stays put: the copy is repeated so that every iteration
    // issues the same number of copies)
    auto stage_copy = [&](uint8_t *st) __attribute__((always_inline)) {
        const int64_t sb = cp_sb;
#pragma unroll
        for (int j = 0; j < S::W_INSTRS; j++) {
            const uint8_t *gp = S::w_base(cw, j, cp_m0, sb) + woff[j];
            if (won[j]) __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + Geo::W_OFF + 1024 * j), 16, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < A_INSTRS; j++) {
            const uint8_t *gp = aq + sb * QKK + aoff[j];
            __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + Geo::A_OFF + 1024 * j), 16, 0, 0);
        }
        {
            const uint8_t *gp = asd + sb * G::SD + doff;
            if (don) __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + Geo::D_OFF), 16, 0, 0);
        }
        {
            const uint8_t *gp = reinterpret_cast<const uint8_t *>(a.d) + sb * 4 + yoff;
            if (yon) __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + Geo::Y_OFF), 4, 0, 0);
        }
        if (S::SCALES_OUTSIDE) {  // the rows' fp16 super-block scales are a plane of their own (Q6_K)
            const uint8_t *gp = reinterpret_cast<const uint8_t *>(cw.d) + ((dhrow + 2 * sb) & ~(int64_t)3);
            if (lane < 16) __builtin_amdgcn_global_load_lds((glb_ptr_t *)gp, (lds_ptr_t *)(st + Geo::DH_OFF), 4, 0, 0);
        }
        if (cp_sb + 1 < sb1) {
            cp_sb++;
        } else if (cp_k + 1 < items) {
            cp_k++;
            cp_sb = sb0;
            const int group = (int)((int64_t)blockIdx.x + cp_k * grid_size);  // never taken by expert-indexed launches
            const SkinnyWhere at = skinny_where<MULTI>(w0, y0, mt, group);
            cw = at.w;
            const int64_t first = (int64_t)(group - at.first) * 16;
            plan_item(first, (int)min((int64_t)16, cw.M - first));
        }
    };

    // ---- operand reads: per-lane offsets into a stage.  A row r = lane & 15 of column set cs is column
    // SET_COLS*cs + a_col(r) restricted to the K groups of one sub-block (a_on); every other lane, and every
    // column past nc, reads the stage's 16 zero bytes instead.
    constexpr int SETS = Geo::SETS, LANE_ACC = Geo::LANE_ACC;
#pragma unroll
    for (int i = 0; i < Geo::NSTAGE; i++) *reinterpret_cast<int *>(wsm + i * STAGE + 4 * lane) = 0;  // the stages' zero bytes
    int aro[SETS][4], dro[SETS], yro[LANE_ACC];
#pragma unroll
    for (int cs = 0; cs < SETS; cs++) {
        const int col = S::SET_COLS * cs + S::a_col(c);
        const bool on = col < nc;
#pragma unroll
        for (int t = 0; t < 4; t++)
            aro[cs][t] = on && S::a_on(c, g) ? Geo::A_OFF + col * 256 + 16 * ((4 * t + g) ^ S::a_swz(col)) : S::a_zero(cs, t);
        // (the digits of a column set lie in the half of the 256 bytes that its parity picks: zeros from the other)
        dro[cs] = on && S::d_on(c, g) ? Geo::D_OFF + col * (16 * S::D_LANES_PER_COL) + S::d_off(c) : 128 * ((cs & 1) ^ 1);
#pragma unroll
        for (int u = 0; u < S::LANE_COLS; u++)  // columns past nc: any staged scale (their sums are zero)
            yro[cs * S::LANE_COLS + u] = Geo::Y_OFF + 4 * min(S::SET_COLS * cs + S::lane_col(g, u), NCT - 1);
    }

    const bool has_k = sb0 < sb1;  // (the launcher gives every wave at least two super-blocks)
    if (has_k) {
        stage_copy(wsm);
#pragma unroll
        for (int i = 1; i < Geo::NSTAGE; i++) stage_copy(wsm + i * STAGE);
    }
    const v4acc zero = {0, 0, 0, 0};
    unsigned parity = 0;  // which stage the next super-block is in
#pragma unroll 1
    for (int64_t k = 0; k < items; k++) {
        if (!ID) {
            const int group = (int)((int64_t)blockIdx.x + k * grid_size);
            const SkinnyWhere at = skinny_where<MULTI>(w0, y0, mt, group);
            w = at.w;
            y = at.y;
            m0 = (int64_t)(group - at.first) * 16;
            yrow0 = m0;
            ldy = w.M;
            rows_left = (int)min((int64_t)16, w.M - m0);
        }
        float acc[LANE_ACC];
#pragma unroll
        for (int i = 0; i < LANE_ACC; i++) acc[i] = 0.f;
#pragma unroll 1
        for (int64_t sb = sb0; sb < sb1; sb++) {
            uint8_t *st = wsm + parity * STAGE;
            parity = parity + 1 == Geo::NSTAGE ? 0 : parity + 1;
            // Every wave issues exactly NDMA copy instructions per stage, in order: once at most NDMA
            // are outstanding, this stage has landed and the next one may still be in flight.
            constexpr int INFLIGHT = (Geo::NSTAGE - 1) * NDMA;
            static_assert(INFLIGHT < 64, "vmcnt is a 6-bit counter");
            __builtin_amdgcn_s_waitcnt((INFLIGHT & 15) | (7 << 4) | (15 << 8) | ((INFLIGHT >> 4) << 14));
            typename S::Raw raw;
            S::read(st + Geo::W_OFF, c, g, raw);
            v4i av[SETS][4], sv[SETS];
            float ydv[LANE_ACC];
#pragma unroll
            for (int cs = 0; cs < SETS; cs++) {
#pragma unroll
                for (int t = 0; t < 4; t++) av[cs][t] = *reinterpret_cast<const v4i *>(st + aro[cs][t]);
                sv[cs] = *reinterpret_cast<const v4i *>(st + dro[cs]);
            }
#pragma unroll
            for (int i = 0; i < LANE_ACC; i++) ydv[i] = *reinterpret_cast<const float *>(st + yro[i]);
            unsigned dh = 0;
            if (S::SCALES_OUTSIDE) {
                const unsigned pair = *reinterpret_cast<const unsigned *>(st + Geo::DH_OFF + 4 * c);
                const bool odd = (((m0 + min(c, rows_left - 1)) * nsb + sb) & 1) != 0;  // which half of the aligned dword
                dh = odd ? pair >> 16 : pair & 0xffff;
            }
            // operands are in registers: the stage can take the copies of the super-block after next
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            stage_copy(st);
            typename S::Ops b;
            S::expand(raw, g, dh, b);
#pragma unroll
            for (int cs = 0; cs < SETS; cs++) {
                const v4acc x = mfma16(S::d_fix(sv[cs], c), b.bsum, zero);
                int isum[S::LANE_COLS];
#pragma unroll
                for (int u = 0; u < S::LANE_COLS; u++) isum[u] = 0;
#pragma unroll
                for (int t = 0; t < 4; t++) S::scale_step(mfma16(av[cs][t], b.q[t], zero), t, b, isum);
#pragma unroll
                for (int u = 0; u < S::LANE_COLS; u++) {
                    const int i = cs * S::LANE_COLS + u;
                    acc[i] = __builtin_fmaf(ydv[i], S::finish(b, isum[u], x, u), acc[i]);
                }
            }
        }
        // lane l holds weight row l & 15 of columns SET_COLS*cs + lane_col(l >> 4, u)
#pragma unroll
        for (int cs = 0; cs < SETS; cs++)
#pragma unroll
            for (int u = 0; u < S::LANE_COLS; u++)
                part[wave][S::SET_COLS * cs + S::lane_col(g, u)][c] = acc[cs * S::LANE_COLS + u];
        __syncthreads();
        for (int o = tid; o < 16 * NCT; o += (64 * WAVES)) {
            const int i = o >> 4, j = o & 15;  // activation column, weight row of the tile
            float sum = 0.f;
            for (int kk = 0; kk < WAVES; kk++) sum += part[kk][i][j];
            if (i < nc && j < rows_left) y[(int64_t)(ID ? rec[2 + i] : col0 + i) * ldy + yrow0 + j] = sum;
        }
        if (k + 1 < items) __syncthreads();  // the partial sums are read before the next item overwrites them
    }
    if (has_k) __builtin_amdgcn_s_waitcnt(0);  // the repeated copies at the end must not outlive the kernel's LDS
}

// ---------------------------------------------------------------------------------------------
// Q6_K products with very many rows, few columns and a short K (the output head at 3..8 tokens).
//
// What bounds the kernel above on this shape is neither its arithmetic nor HBM bandwidth but the number of
// copy instructions and of cache lines they name: per 16 rows and super-block it issues nine direct-to-LDS
// copies that touch 96 lines -- among them 16 bytes of sub-block scales out of each of 16 lines, 2 bytes of
// super-block scale out of 16 more, and the activations' quants, digits and scales again for every row group.
// With everything but the copies taken out it ran no faster; without the small copies it ran at HBM speed.
//
// So this kernel copies per super-block only what is new (ql: 16 x 128 B, qh: 16 x 64 B; three instructions)
// and fetches the rest in whole lines: the sub-block scales of eight super-blocks at once (16 lines, two
// instructions per eight super-blocks), the super-block scales of all of a row group's super-blocks (one
// instruction per row group), and the activations -- which are the same for every row group -- once per
// workgroup into LDS, where they stay.  A workgroup is eight waves on one CU; a wave owns whole row groups
// (all of K, so no partial sums) and streams its weights through its own ring of three stages.
//
// Copy order and waits: a wave issues, for the super-block its copy cursor stands on, first the whole-line
// copies that start there (super-block scales at a row group's first super-block, sub-block scales at every
// eighth), then the three weight copies.  Waiting until at most six copies are outstanding therefore means
// that the stage about to be multiplied has landed together with every whole-line copy issued before it.
// ---------------------------------------------------------------------------------------------
template <int NCT>
struct RowsGeo {
    // resident activations, per super-block: 256 zero bytes (operand lanes that carry zeros read here), quants
    // [column][16 pieces, swizzled], block-sum digits [column][32 B], scales [column] (padded to 256 B)
    static constexpr int Z_OFF = 0, A_OFF = 256, D_OFF = A_OFF + NCT * 256, Y_OFF = D_OFF + NCT * 32, RB = Y_OFF + 256;
    // per wave: three weight stages (ql [16 rows][8 pieces] at 0, qh [16][4] at 2 KiB), two buffers of sub-block
    // scales (16 lines of 128 B = eight super-blocks), two of super-block scales (16 rows x up to 16 halves)
    static constexpr int NST = 3, W_STAGE = 3072, SC_BYTES = 2048, DH_BYTES = 512;
    static constexpr int SC_OFF = NST * W_STAGE, DH_OFF = SC_OFF + 2 * SC_BYTES, WAVE_BYTES = DH_OFF + 2 * DH_BYTES;
    static constexpr int WAVES = 8;
    static constexpr size_t lds_bytes(int64_t nsb) { return (size_t)nsb * RB + (size_t)WAVES * WAVE_BYTES; }
};

template <int NCT>
__global__ __launch_bounds__(512, 2) void skinny_rows_q6k_kernel(DevWeight w, DevAct a, int col0, int nc, float *__restrict__ y, int grid_size) {
    typedef Sk16Q6K S;
    typedef GemmQ6K G;
    typedef RowsGeo<NCT> Geo;
    constexpr int SETS = NCT / S::SET_COLS, A_INSTRS = NCT / 4;
    static_assert(S::LANE_COLS == 1, "one output column per lane and column set");
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int nsb = (int)(w.K / QKK);  // 8 or 16
    const unsigned res_a = lds_addr(smem), wv_a = res_a + (unsigned)nsb * Geo::RB + (unsigned)wave * Geo::WAVE_BYTES;

    // ---- the activations, once per workgroup: wave v copies super-blocks v, v + 8
    for (int i = tid; i < nsb * 64; i += 64 * Geo::WAVES) *reinterpret_cast<int *>(smem + (i >> 6) * Geo::RB + 4 * (i & 63)) = 0;
    {
        auto acol = [&](int i) { return col0 + min(i, nc - 1); };
        const uint8_t *aq = reinterpret_cast<const uint8_t *>(a.qs);
        unsigned aoff[A_INSTRS];
#pragma unroll
        for (int j = 0; j < A_INSTRS; j++) {
            const int col = 4 * j + (lane >> 4), slot = lane & 15;  // slot [col][slot] holds piece slot ^ a_swz(col)
            aoff[j] = (unsigned)acol(col) * (unsigned)a.K + 16u * (slot ^ S::a_swz(col));
        }
        const bool don = lane < 2 * NCT, yon = lane < NCT;
        const unsigned doff = (unsigned)acol(lane >> 1) * (unsigned)(nsb * G::SD) + 16u * (lane & 1);
        const unsigned yoff = (unsigned)acol(lane) * (unsigned)nsb * 4u;
        for (int sb = wave; sb < nsb; sb += Geo::WAVES) {
            const unsigned sa = res_a + (unsigned)sb * Geo::RB;
#pragma unroll
            for (int j = 0; j < A_INSTRS; j++) dma_lds<16>(aq + (int64_t)sb * QKK, aoff[j], sa + Geo::A_OFF + 1024 * j);
            if (don) dma_lds<16>(a.sd16 + (int64_t)sb * G::SD, doff, sa + Geo::D_OFF);
            if (yon) dma_lds<4>(reinterpret_cast<const uint8_t *>(a.d) + (int64_t)sb * 4, yoff, sa + Geo::Y_OFF);
        }
    }

    // ---- the wave's row groups: ((k * grid + workgroup) * 8 + wave), k = 0, 1, ...: the eight waves of a workgroup
    // stream 128 consecutive rows at a time
    const int64_t groups = (w.M + 15) / 16;
    auto item_group = [&](int64_t k) { return (k * grid_size + (int64_t)blockIdx.x) * Geo::WAVES + wave; };
    int64_t items = 0;
    if (item_group(0) < groups) items = (groups - 1 - item_group(0)) / ((int64_t)grid_size * Geo::WAVES) + 1;

    // ---- copy plan: per-lane 32-bit offsets from uniform bases
    unsigned woff[3], scoff[2], dhoff = 0;
    const bool dhon = lane < 2 * nsb;
    int64_t cp_m0 = 0, cp_k = 0;
    int cp_sb = 0;
    unsigned cp_half = 0;  // eight-super-block runs copied so far: run h goes to scale buffer h & 1
    auto plan_item = [&](int64_t k) __attribute__((always_inline)) {
        cp_m0 = item_group(k) * 16;
        const int rows = (int)min((int64_t)16, w.M - cp_m0);  // rows past M: the last row again, results dropped
#pragma unroll
        for (int j = 0; j < 3; j++) {
            bool on;
            S::w_plan(w, j, lane, rows, woff[j], on);
        }
#pragma unroll
        for (int i = 0; i < 2; i++) {
            // scale buffer slot P = 64 i + lane (16 B each): line P >> 3 holds row L ^ (L >> 3), and inside the line
            // piece p of row r sits at position p ^ (r & 7) -- the sixteen rows of a read then fall on sixteen
            // different slots of the LDS's 256-byte bank period
            const int P = 64 * i + lane, L = P >> 3, r = L ^ (L >> 3), p = (P & 7) ^ (r & 7);
            scoff[i] = (unsigned)min(r, rows - 1) * (unsigned)(nsb * 16) + 16u * p;
        }
        {
            const int row = (16 * lane) / (2 * nsb), within = (16 * lane) % (2 * nsb);
            dhoff = (unsigned)min(row, rows - 1) * (unsigned)(2 * nsb) + within;
        }
    };
    auto stage_copy = [&](unsigned st) __attribute__((always_inline)) {
        const int sb = cp_sb;
        if (sb == 0 && dhon)
            dma_lds<16>(reinterpret_cast<const uint8_t *>(w.d) + cp_m0 * nsb * 2, dhoff, wv_a + Geo::DH_OFF + (unsigned)(cp_k & 1) * Geo::DH_BYTES);
        if ((sb & 7) == 0) {
            const uint8_t *base = w.p2 + cp_m0 * (w.K / 16) + (sb >> 3) * 128;
            const unsigned dst = wv_a + Geo::SC_OFF + (cp_half & 1) * Geo::SC_BYTES;
            dma_lds<16>(base, scoff[0], dst);
            dma_lds<16>(base, scoff[1], dst + 1024);
            cp_half++;
        }
#pragma unroll
        for (int j = 0; j < 3; j++) dma_lds<16>(S::w_base(w, j, cp_m0, sb), woff[j], st + 1024 * j);
        if (cp_sb + 1 < nsb) {
            cp_sb++;
        } else if (cp_k + 1 < items) {
            cp_k++;
            cp_sb = 0;
            plan_item(cp_k);
        }  // past the last super-block of the last row group the cursor stays put: the copy is repeated
    };

    // ---- operand reads: absolute LDS addresses, pinned in registers
    unsigned wro[S::NRO];
    S::read_plan(c, g, wro);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        wro[i] += wv_a;
        asm volatile("" : "+v"(wro[i]));
    }
    const unsigned scro = wv_a + Geo::SC_OFF + (unsigned)(c ^ (c >> 3)) * 128u;  // the lane's row in a scale buffer
    const unsigned dhro = wv_a + Geo::DH_OFF + (unsigned)c * (unsigned)(2 * nsb);
    unsigned aro[SETS][4], dro[SETS], yro[SETS];
#pragma unroll
    for (int cs = 0; cs < SETS; cs++) {
        const int col = S::SET_COLS * cs + S::a_col(c);
        const bool on = col < nc;
#pragma unroll
        for (int t = 0; t < 4; t++)
            aro[cs][t] = res_a + (on && S::a_on(c, g) ? Geo::A_OFF + col * 256 + 16 * ((4 * t + g) ^ S::a_swz(col)) : S::a_zero(cs, t));
        dro[cs] = res_a + (on && S::d_on(c, g) ? Geo::D_OFF + col * 32 + S::d_off(c) : 128 * ((cs & 1) ^ 1));
        yro[cs] = res_a + Geo::Y_OFF + 4 * min(S::SET_COLS * cs + S::lane_col(g, 0), NCT - 1);  // columns past nc: any staged scale
    }

    if (items > 0) {
        plan_item(0);
#pragma unroll
        for (int i = 0; i < Geo::NST; i++) stage_copy(wv_a + i * Geo::W_STAGE);
    }
    // the activations have landed (a wave's own copies: all but the nine just issued; everybody's: the barrier)
    if (items > 0) wait_vm<3 * Geo::NST + 3>();
    else wait_vm<0>();
    __syncthreads();

    const v4acc zero = {0, 0, 0, 0};
    unsigned parity = 0, half_run = 0;
#pragma unroll 1
    for (int64_t k = 0; k < items; k++) {
        const int64_t m0 = item_group(k) * 16;
        const int rows_left = (int)min((int64_t)16, w.M - m0);
        float acc[SETS];
#pragma unroll
        for (int i = 0; i < SETS; i++) acc[i] = 0.f;
        const unsigned dh_a = dhro + (unsigned)(k & 1) * Geo::DH_BYTES;
        auto step = [&](auto stg, int sb) __attribute__((always_inline)) {
            constexpr int STG = decltype(stg)::value;
            wait_vm<3 * (Geo::NST - 1)>();
            typename S::Raw raw;
#pragma unroll
            for (int H = 0; H < 2; H++) {
                raw.L[H] = lds_u4(wro[H], STG * Geo::W_STAGE);
                raw.Hq[H] = lds_u4(wro[2 + H], STG * Geo::W_STAGE);
            }
            raw.scv = lds_u4(scro + ((half_run + (unsigned)(sb >> 3)) & 1) * Geo::SC_BYTES + 16u * ((sb & 7) ^ (c & 7)), 0);
            const unsigned dh = lds_at<unsigned short>(dh_a + 2u * (unsigned)sb, 0);
            const unsigned ro = (unsigned)sb * Geo::RB;
            v4i av[SETS][4], sv[SETS];
            float ydv[SETS];
#pragma unroll
            for (int cs = 0; cs < SETS; cs++) {
#pragma unroll
                for (int t = 0; t < 4; t++) av[cs][t] = lds_at<v4i>(aro[cs][t] + ro, 0);
                sv[cs] = lds_at<v4i>(dro[cs] + ro, 0);
                ydv[cs] = lds_at<float>(yro[cs] + ro, 0);
            }
            // operands are in registers: the stage can take the copies of the super-block after next
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            stage_copy(wv_a + STG * Geo::W_STAGE);
            typename S::Ops b;
            S::expand(raw, g, dh, b);
#pragma unroll
            for (int cs = 0; cs < SETS; cs++) {
                const v4acc x = mfma16(S::d_fix(sv[cs], c), b.bsum, zero);
                int isum[1] = {0};
#pragma unroll
                for (int t = 0; t < 4; t++) S::scale_step(mfma16(av[cs][t], b.q[t], zero), t, b, isum);
                acc[cs] = __builtin_fmaf(ydv[cs], S::finish(b, isum[0], x, 0), acc[cs]);
            }
        };
#pragma unroll 1
        for (int sb = 0; sb < nsb; sb++) {
            if (parity == 0) step(std::integral_constant<int, 0>{}, sb);
            else if (parity == 1) step(std::integral_constant<int, 1>{}, sb);
            else step(std::integral_constant<int, 2>{}, sb);
            parity = parity == Geo::NST - 1 ? 0 : parity + 1;
        }
        half_run += (unsigned)(nsb >> 3);
        // lane l holds weight row l & 15 of column 4 cs + (l >> 4)
#pragma unroll
        for (int cs = 0; cs < SETS; cs++) {
            const int col = S::SET_COLS * cs + g;
            if (col < nc && c < rows_left) y[(int64_t)(col0 + col) * w.M + m0 + c] = acc[cs];
        }
    }
    wait_vm<0>();  // the repeated copies at the end must not outlive the kernel's LDS
}

bool rows_wanted(const DevWeight &w, int ncols, int num_cus) {
    const int64_t nsb = w.K / QKK;
    return w.type == T_Q6_K && ncols >= 1 && ncols <= 8 && (nsb == 8 || nsb == 16) &&
           (w.M + 15) / 16 >= (int64_t)16 * num_cus;  // two row groups and more for every wave of a full grid
}

void launch_skinny_rows(const DevWeight &w, const DevAct &a, int col0, int ncols, float *y, int num_cus, hipStream_t s) {
    typedef RowsGeo<8> Geo;
    const size_t lds = Geo::lds_bytes(w.K / QKK);
    static bool allowed[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 && !allowed[dev]) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(skinny_rows_q6k_kernel<8>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  160 * 1024);
        allowed[dev] = true;
    }
    skinny_rows_q6k_kernel<8><<<(unsigned)num_cus, 64 * Geo::WAVES, lds, s>>>(w, a, col0, ncols, y, num_cus);
}

// ---------------------------------------------------------------------------------------------
// The same for Q4_K at 3..16 columns on matrices with many rows and K up to 8192 (the feed-forward gate and up
// projections at a few tokens, alone or both in one launch): of the seven copies the general kernel issues per 16
// rows and super-block, four bring activations.  Here the activations are resident (per super-block: zero block,
// quants, block-sum digits, scales), a wave owns whole row groups -- all of K, no partial sums -- and streams
// only weights: three copies per super-block through a ring of four stages.  A workgroup has as many waves (up
// to eight) as it takes to give every CU about the same number of row groups.
//
// Same bits as the general kernel: that one cuts a matrix's K between the waves of a workgroup (skinny_waves) and
// adds the partial sums in order; a wave here restarts its fp32 accumulator at the same super-blocks and adds the
// pieces in the same order, so a matrix gives the same result alone (either kernel) and in a joint launch.
// ---------------------------------------------------------------------------------------------
constexpr int ROWS_MULTI = 4;
struct RowsArgs {
    const uint8_t *p0[ROWS_MULTI];
    float *y[ROWS_MULTI];
    int64_t M[ROWS_MULTI];
    int grp_end[ROWS_MULTI];  // exclusive end of each matrix's run of 16-row groups; INT_MAX past the last matrix
    int kcut[ROWS_MULTI];     // how many ways the general kernel would cut K for this matrix alone (see below)
    int64_t K;
    int groups_total;
};
struct RowsWhere { const uint8_t *p0; float *y; int64_t M; int first, kcut; };
__device__ __forceinline__ RowsWhere rows_where(const RowsArgs &g, int group) {
    RowsWhere w{g.p0[0], g.y[0], g.M[0], 0, g.kcut[0]};
#pragma unroll
    for (int t = 1; t < ROWS_MULTI; t++)
        if (group >= g.grp_end[t - 1]) w = RowsWhere{g.p0[t], g.y[t], g.M[t], g.grp_end[t - 1], g.kcut[t]};
    return w;
}

template <int NCT>
struct RowsGeoQ4K {
    static constexpr int Z_OFF = 0, A_OFF = 256, D_OFF = A_OFF + NCT * 256, Y_OFF = D_OFF + NCT * 16;
    static constexpr int RB = (Y_OFF + NCT * 4 + 255) / 256 * 256;
    static constexpr int NST = 4, W_STAGE = 2560;  // 16 rows x 144 B, padded to the 256-byte bank period
    static constexpr size_t lds_bytes(int64_t nsb, int waves) { return (size_t)nsb * RB + (size_t)waves * NST * W_STAGE; }
};

template <int NCT>
__global__ __launch_bounds__(512, 2) void skinny_rows_q4k_kernel(RowsArgs ra, DevAct a, int col0, int nc, int grid_size, int waves) {
    typedef Sk16Q4K S;
    typedef GemmQ4K G;
    typedef RowsGeoQ4K<NCT> Geo;
    constexpr int SETS = NCT / S::SET_COLS, LANE_ACC = SETS * S::LANE_COLS, A_INSTRS = NCT / 4;
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int nsb = (int)(ra.K / QKK);
    const unsigned res_a = lds_addr(smem), wv_a = res_a + (unsigned)nsb * Geo::RB + (unsigned)wave * (Geo::NST * Geo::W_STAGE);

    // ---- the wave's row groups: ((k * waves + wave) * grid + workgroup), k = 0, 1, ...: consecutive row groups go to
    // consecutive workgroups, so a count that is no multiple of the grid still loads every CU alike
    auto item_group = [&](int64_t k) { return (k * waves + wave) * grid_size + (int64_t)blockIdx.x; };
    int64_t items = 0;
    if (item_group(0) < ra.groups_total) items = (ra.groups_total - 1 - item_group(0)) / ((int64_t)grid_size * waves) + 1;

    // ---- weight copies: per-lane offsets from a uniform base per row group and super-block
    unsigned woff[3];
    bool won[3];
    const uint8_t *cp_base = nullptr;
    int64_t cp_k = 0;
    int cp_sb = 0;
    auto plan_item = [&](int64_t k) __attribute__((always_inline)) {
        const int group = (int)item_group(k);
        const RowsWhere at = rows_where(ra, group);
        const int64_t first = (int64_t)(group - at.first) * 16;
        const int rows = (int)min((int64_t)16, at.M - first);  // rows past M: the last row again, results dropped
        const DevWeight w{at.p0, nullptr, nullptr, nullptr, ra.K, at.M, T_Q4_K};
#pragma unroll
        for (int j = 0; j < 3; j++) S::w_plan(w, j, lane, rows, woff[j], won[j]);
        cp_base = S::w_base(w, 0, first, 0);
    };
    auto stage_copy = [&](unsigned st) __attribute__((always_inline)) {
        const uint8_t *base = cp_base + (int64_t)cp_sb * Q4_K_BYTES;
#pragma unroll
        for (int j = 0; j < 3; j++)
            if (won[j]) dma_lds<16>(base, woff[j], st + 1024 * j);
        if (cp_sb + 1 < nsb) {
            cp_sb++;
        } else if (cp_k + 1 < items) {
            cp_k++;
            cp_sb = 0;
            plan_item(cp_k);
        }  // past the last super-block of the last row group the cursor stays put: the copy is repeated
    };
    if (items > 0) {
        plan_item(0);
#pragma unroll
        for (int i = 0; i < Geo::NST; i++) stage_copy(wv_a + i * Geo::W_STAGE);
    }

    // ---- the activations, once per workgroup, behind the first weight copies: wave v copies super-blocks v, v + waves, ...
    for (int i = tid; i < nsb * 64; i += 64 * waves) *reinterpret_cast<int *>(smem + (i >> 6) * Geo::RB + 4 * (i & 63)) = 0;
    {
        auto acol = [&](int i) { return col0 + min(i, nc - 1); };
        const uint8_t *aq = reinterpret_cast<const uint8_t *>(a.qs);
        unsigned aoff[A_INSTRS];
#pragma unroll
        for (int j = 0; j < A_INSTRS; j++) {
            const int col = 4 * j + (lane >> 4), slot = lane & 15;  // slot [col][slot] holds piece slot ^ a_swz(col)
            aoff[j] = (unsigned)acol(col) * (unsigned)a.K + 16u * (slot ^ S::a_swz(col));
        }
        const bool don = lane < NCT, yon = lane < NCT;
        const unsigned doff = (unsigned)acol(lane) * (unsigned)(nsb * G::SD);
        const unsigned yoff = (unsigned)acol(lane) * (unsigned)nsb * 4u;
        for (int sb = wave; sb < nsb; sb += waves) {
            const unsigned sa = res_a + (unsigned)sb * Geo::RB;
#pragma unroll
            for (int j = 0; j < A_INSTRS; j++) dma_lds<16>(aq + (int64_t)sb * QKK, aoff[j], sa + Geo::A_OFF + 1024 * j);
            if (don) dma_lds<16>(a.sd8 + (int64_t)sb * G::SD, doff, sa + Geo::D_OFF);
            if (yon) dma_lds<4>(reinterpret_cast<const uint8_t *>(a.d) + (int64_t)sb * 4, yoff, sa + Geo::Y_OFF);
        }
    }
    wait_vm<0>();  // (once: the weight copies issued above wait with it)
    __syncthreads();

    // ---- operand reads: absolute LDS addresses
    unsigned wro[S::NRO];
    S::read_plan(c, g, wro);
#pragma unroll
    for (int i = 0; i < S::NRO; i++) {
        wro[i] += wv_a;
        asm volatile("" : "+v"(wro[i]));
    }
    unsigned aro[SETS][4], dro[SETS], yro[LANE_ACC];
#pragma unroll
    for (int cs = 0; cs < SETS; cs++) {
        const int col = S::SET_COLS * cs + S::a_col(c);
        const bool on = col < nc;
#pragma unroll
        for (int t = 0; t < 4; t++)
            aro[cs][t] = res_a + (on && S::a_on(c, g) ? Geo::A_OFF + col * 256 + 16 * ((4 * t + g) ^ S::a_swz(col)) : S::a_zero(cs, t));
        dro[cs] = res_a + (on && S::d_on(c, g) ? Geo::D_OFF + col * 16 + S::d_off(c) : 128 * ((cs & 1) ^ 1));
#pragma unroll
        for (int u = 0; u < S::LANE_COLS; u++)  // columns past nc: any staged scale (their sums are zero)
            yro[cs * S::LANE_COLS + u] = res_a + Geo::Y_OFF + 4 * min(S::SET_COLS * cs + S::lane_col(g, u), NCT - 1);
    }

    const v4acc zero = {0, 0, 0, 0};
    unsigned parity = 0;
#pragma unroll 1
    for (int64_t k = 0; k < items; k++) {
        const int group = (int)item_group(k);
        const RowsWhere at = rows_where(ra, group);
        const int64_t m0 = (int64_t)(group - at.first) * 16;
        const int rows_left = (int)min((int64_t)16, at.M - m0);
        float acc[LANE_ACC], total[LANE_ACC];
#pragma unroll
        for (int i = 0; i < LANE_ACC; i++) acc[i] = total[i] = 0.f;
        int cut = 1, next_cut = nsb / at.kcut;  // pieces of K as the general kernel cuts them: [nsb j / kcut, nsb (j + 1) / kcut)
        auto step = [&](auto stg, int sb) __attribute__((always_inline)) {
            constexpr int STG = decltype(stg)::value;
            wait_vm<3 * (Geo::NST - 1)>();  // three copies per stage: this stage has landed, the next three may be in flight
            typename S::Raw raw;
            S::read(wro, STG * Geo::W_STAGE, raw);
            const unsigned ro = (unsigned)sb * Geo::RB;
            v4i av[SETS][4], sv[SETS];
            float ydv[LANE_ACC];
#pragma unroll
            for (int cs = 0; cs < SETS; cs++) {
#pragma unroll
                for (int t = 0; t < 4; t++) av[cs][t] = lds_at<v4i>(aro[cs][t] + ro, 0);
                sv[cs] = lds_at<v4i>(dro[cs] + ro, 0);
            }
#pragma unroll
            for (int i = 0; i < LANE_ACC; i++) ydv[i] = lds_at<float>(yro[i] + ro, 0);
            // operands are in registers: the stage can take the copies of the super-block three ahead
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            stage_copy(wv_a + STG * Geo::W_STAGE);
            typename S::Ops b;
            S::expand(raw, g, 0, b);
#pragma unroll
            for (int cs = 0; cs < SETS; cs++) {
                const v4acc x = mfma16(S::d_fix(sv[cs], c), b.bsum, zero);
                int isum[S::LANE_COLS];
#pragma unroll
                for (int u = 0; u < S::LANE_COLS; u++) isum[u] = 0;
#pragma unroll
                for (int t = 0; t < 4; t++) S::scale_step(mfma16(av[cs][t], b.q[t], zero), t, b, isum);
#pragma unroll
                for (int u = 0; u < S::LANE_COLS; u++) {
                    const int i = cs * S::LANE_COLS + u;
                    acc[i] = __builtin_fmaf(ydv[i], S::finish(b, isum[u], x, u), acc[i]);
                }
            }
        };
#pragma unroll 1
        for (int sb = 0; sb < nsb; sb++) {
            if (sb == next_cut) {
#pragma unroll
                for (int i = 0; i < LANE_ACC; i++) {
                    total[i] += acc[i];
                    acc[i] = 0.f;
                }
                cut++;
                next_cut = nsb * cut / at.kcut;
            }
            if (parity == 0) step(std::integral_constant<int, 0>{}, sb);
            else if (parity == 1) step(std::integral_constant<int, 1>{}, sb);
            else if (parity == 2) step(std::integral_constant<int, 2>{}, sb);
            else step(std::integral_constant<int, 3>{}, sb);
            parity = (parity + 1) & 3;
        }
        // lane l holds weight row l & 15 of columns SET_COLS*cs + lane_col(l >> 4, u)
#pragma unroll
        for (int cs = 0; cs < SETS; cs++)
#pragma unroll
            for (int u = 0; u < S::LANE_COLS; u++) {
                const int col = S::SET_COLS * cs + S::lane_col(g, u), i = cs * S::LANE_COLS + u;
                if (col < nc && c < rows_left) at.y[(int64_t)(col0 + col) * at.M + m0 + c] = total[i] + acc[i];
            }
    }
    wait_vm<0>();  // the repeated copies at the end must not outlive the kernel's LDS
}

// waves per workgroup and grid for `groups` row groups: every CU about the same number of groups, up to eight waves
void rows_q4k_shape(int64_t groups, int num_cus, int &waves, int &grid) {
    grid = (int)min((int64_t)num_cus, groups);
    waves = (int)min((int64_t)8, (groups + grid - 1) / grid);
}
bool rows_q4k_wanted(int type, int64_t K, int64_t total_m, int ncols, int num_cus) {
    if (type != T_Q4_K || ncols < 3 || ncols > 16 || K % QKK) return false;
    const int64_t nsb = K / QKK, groups = (total_m + 15) / 16;
    int waves, grid;
    rows_q4k_shape(groups, num_cus, waves, grid);
    const size_t lds = ncols <= 8 ? RowsGeoQ4K<8>::lds_bytes(nsb, waves) : RowsGeoQ4K<16>::lds_bytes(nsb, waves);
    // from six row groups per CU: a wave runs a row group's whole K, and with fewer waves than that the general
    // kernel's K cut keeps more of the memory system busy (gate 14336 x 4096 alone, 3.5 groups per CU: 12.2 us here
    // against 11.3 at three columns; gate + up in one launch, 7 per CU: 19.6 against 22.1)
    return lds <= 160 * 1024 && groups >= 6 * (int64_t)num_cus;
}

template <int NCT>
void launch_rows_q4k_as(const RowsArgs &ra, const DevAct &a, int col0, int ncols, int num_cus, hipStream_t s) {
    int waves, grid;
    rows_q4k_shape(ra.groups_total, num_cus, waves, grid);
    const size_t lds = RowsGeoQ4K<NCT>::lds_bytes(ra.K / QKK, waves);
    static bool allowed[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 && !allowed[dev]) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(skinny_rows_q4k_kernel<NCT>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  160 * 1024);
        allowed[dev] = true;
    }
    skinny_rows_q4k_kernel<NCT><<<(unsigned)grid, 64 * waves, lds, s>>>(ra, a, col0, ncols, grid, waves);
}
void launch_rows_q4k(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int col0, int ncols, int num_cus, hipStream_t s) {
    RowsArgs ra;
    int64_t rg = 0;
    for (int t = 0; t < ROWS_MULTI; t++) {
        const int j = t < count ? t : count - 1;
        ra.p0[t] = ws[j].p0; ra.y[t] = ys[j]; ra.M[t] = ws[j].M;
        ra.kcut[t] = skinny_waves((ws[j].M + 15) / 16, ws[j].K / QKK, num_cus);
        if (t < count) rg += (ws[j].M + 15) / 16;
        ra.grp_end[t] = t + 1 < count ? (int)rg : 0x7fffffff;
    }
    ra.K = ws[0].K;
    ra.groups_total = (int)rg;
    if (ncols <= 8) launch_rows_q4k_as<8>(ra, a, col0, ncols, num_cus, s);
    else launch_rows_q4k_as<16>(ra, a, col0, ncols, num_cus, s);
}

// ---------------------------------------------------------------------------------------------
// Q4_K at up to four activation columns with the weights loaded straight into the MFMA operand
// registers: the faster of the two skinny kernels while the matrix is small enough that latency, not
// HBM time, decides (launch_skinny picks).  A 16-row group is cut kcut ways along K, one wave per cut;
// a workgroup holds one or more groups.  Lane l = (row r = l%16, chunk q = l/16) loads the 32 quant
// bytes of chunk q of its row's super-block -- elements [64q, 64q+64): low nibbles sub-block 2q, high
// nibbles sub-block 2q+1 -- and the row's 16-byte header: three 16-byte loads per lane and super-block,
// every byte of the 16 rows fetched once, nothing staged in LDS, no copy pipeline to fill.  Four MFMAs
// cover the super-block: low nibbles of the first / second 16 bytes, then the high nibbles, so K group q
// of MFMA j is elements 64q + 16j.. of the super-block and belongs to sub-block 2q + (j>>1).  The 16 rows
// of the A operand are 4 columns x 4 K groups (row i = column i>>2 restricted to K group i&3, zero
// elsewhere): the lane that holds a non-zero piece reads 64 consecutive activation bytes.  Lane (r, c)
// then holds, for weight row r and column c, the sums of the four even sub-blocks (MFMAs 0, 1 chained)
// and of the four odd ones (MFMAs 2, 3), scales them with v_mad_i32_i24, and takes the mins term from
// one more MFMA (block-sum digits x mins) exactly as the staged kernel above does.
//
// Up to DIRECT16_MULTI matrices that share K and the activations go out in one launch: their 16-row groups
// are numbered through, and a wave finds its matrix by comparing its group number with the ends of the runs.
constexpr int DIRECT16_MULTI = 4;
struct Direct16Args {
    const uint8_t *p0[DIRECT16_MULTI];
    float *y[DIRECT16_MULTI];
    int64_t M[DIRECT16_MULTI];
    int grp_end[DIRECT16_MULTI];  // exclusive end of each matrix's run of groups; INT_MAX past the last matrix
    int64_t K;
    int groups_total;
};

struct Direct16Where { const uint8_t *p0; float *y; int64_t M; int first; };
template <bool MULTI>
__device__ __forceinline__ Direct16Where direct16_where(const Direct16Args &g, int group) {
    Direct16Where w{g.p0[0], g.y[0], g.M[0], 0};
    if (!MULTI) return w;
#pragma unroll
    for (int t = 1; t < DIRECT16_MULTI; t++)
        if (group >= g.grp_end[t - 1]) w = Direct16Where{g.p0[t], g.y[t], g.M[t], g.grp_end[t - 1]};
    return w;
}

template <bool MULTI>
__global__ __launch_bounds__(1024, 8) void direct16_q4k_kernel(Direct16Args g, DevAct a, int col0, int nc, int kcut, int threads) {
    __shared__ float part[16][4][16];  // [wave][column][row]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int GROUPS = (threads >> 6) / kcut;  // row groups of this workgroup (threads = the block size, as an argument:
                                               // one batch of scalar loads fetches everything the prologue needs)
    const int r = lane & 15, q = lane >> 4;
    const int grp = wave / kcut, kw = wave - grp * kcut;
    const int group = min((int)blockIdx.x * GROUPS + grp, g.groups_total - 1);  // groups past the last: the last one again, not stored
    const Direct16Where w = direct16_where<MULTI>(g, group);
    const int64_t m0 = (int64_t)(group - w.first) * 16;
    const int rows_left = (int)min((int64_t)16, w.M - m0);
    const int nsb = (int)(g.K / QKK);
    const int sb0 = nsb * kw / kcut, sb1 = nsb * (kw + 1) / kcut;
    const uint8_t *hp = w.p0 + (m0 + min(r, rows_left - 1)) * ((int64_t)nsb * Q4_K_BYTES);  // rows past M: the last row again
    const uint8_t *wp = hp + 16 + 32 * q;
    const int col = r >> 2, colc = col0 + min(col, nc - 1);
    const bool a_on = col < nc && q == (r & 3);
    const bool d_on = col < nc && q == 0 && (r & 3) < 2;  // low digits in row 4c, high digits in row 4c + 1
    const int8_t *ap = a.qs + (int64_t)colc * a.K + 64 * q;
    const uint8_t *dp = a.sd8 + (int64_t)colc * nsb * 16 + 8 * (r & 1);
    const float *ydp = a.d + (int64_t)(col0 + min(q, nc - 1)) * nsb;  // the column this lane's outputs belong to
    const v4acc zero = {0, 0, 0, 0};
    const v4i none = {0, 0, 0, 0};
    float acc = 0.f;
#pragma unroll 2
    for (int sb = sb0; sb < sb1; sb++) {
        const uint4 hdr = ld16(hp + sb * Q4_K_BYTES);
        const uint4 qa = ld16(wp + sb * Q4_K_BYTES), qb = ld16(wp + sb * Q4_K_BYTES + 16);
        v4i av[4];
#pragma unroll
        for (int j = 0; j < 4; j++) av[j] = a_on ? *reinterpret_cast<const v4i *>(ap + sb * QKK + 16 * j) : none;
        const int2 dg = d_on ? *reinterpret_cast<const int2 *>(dp + sb * 16) : make_int2(0, 0);
        const float yd = ydp[sb];
        const float d = h2f(hdr.x & 0xffff), dmin = h2f(hdr.x >> 16);
        const unsigned sc03 = hdr.y & 0x3f3f3f3fu, sc47 = (hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4);
        const unsigned mn03 = hdr.z & 0x3f3f3f3fu, mn47 = ((hdr.w >> 4) & 0x0f0f0f0fu) | (((hdr.z >> 6) & 0x03030303u) << 4);
        int sc[8];
#pragma unroll
        for (int j = 0; j < 8; j++) sc[j] = (int)(((j < 4 ? sc03 : sc47) >> (8 * (j & 3))) & 0xff);
        const v4i b0 = {(int)(qa.x & 0x0f0f0f0fu), (int)(qa.y & 0x0f0f0f0fu), (int)(qa.z & 0x0f0f0f0fu), (int)(qa.w & 0x0f0f0f0fu)};
        const v4i b1 = {(int)(qb.x & 0x0f0f0f0fu), (int)(qb.y & 0x0f0f0f0fu), (int)(qb.z & 0x0f0f0f0fu), (int)(qb.w & 0x0f0f0f0fu)};
        const v4i b2 = {(int)((qa.x >> 4) & 0x0f0f0f0fu), (int)((qa.y >> 4) & 0x0f0f0f0fu), (int)((qa.z >> 4) & 0x0f0f0f0fu),
                        (int)((qa.w >> 4) & 0x0f0f0f0fu)};
        const v4i b3 = {(int)((qb.x >> 4) & 0x0f0f0f0fu), (int)((qb.y >> 4) & 0x0f0f0f0fu), (int)((qb.z >> 4) & 0x0f0f0f0fu),
                        (int)((qb.w >> 4) & 0x0f0f0f0fu)};
        const int mz = q == 0 ? -1 : 0;
        const v4i bm = {(int)mn03 & mz, (int)mn47 & mz, 0, 0};
        const v4acc even = mfma16(av[1], b1, mfma16(av[0], b0, zero));
        const v4acc odd = mfma16(av[3], b3, mfma16(av[2], b2, zero));
        const v4acc x = mfma16((v4i){dg.x, dg.y, 0, 0}, bm, zero);
        int isum = 0;
#pragma unroll
        for (int v = 0; v < 4; v++) isum = mad24(sc[2 * v], even[v], mad24(sc[2 * v + 1], odd[v], isum));
        const float fm = GemmQ4K::fold_min(dmin, x[1], x[0]);
        acc = __builtin_fmaf(yd, __builtin_fmaf(d, (float)isum, -fm), acc);
    }
    part[wave][q][r] = acc;
    __syncthreads();
    for (int o = tid; o < GROUPS * 64; o += threads) {
        const int og = o >> 6, i = (o >> 4) & 3, j = o & 15;  // group, activation column, weight row
        const int out_group = (int)blockIdx.x * GROUPS + og;
        const Direct16Where ow = direct16_where<MULTI>(g, min(out_group, g.groups_total - 1));
        const int64_t row = (int64_t)(out_group - ow.first) * 16 + j;
        float sum = 0.f;
        for (int kk = 0; kk < kcut; kk++) sum += part[og * kcut + kk][i][j];
        if (i < nc && out_group < g.groups_total && row < ow.M) ow.y[(int64_t)(col0 + i) * ow.M + row] = sum;
    }
}

// The direct kernel wins (5..19 %, measured over projection shapes from 512 x 2048 to 4096 x 11008 at three
// and four columns) while M x K stays under about 40 M elements; from the 14336 x 4096 FFN matrices up the
// staged kernel's coalesced copies are ahead (11.7 against 12.4 us), and so they are from five columns up,
// where a second column set doubles the direct kernel's activation loads.
bool direct16_wanted(int type, int64_t K, int64_t total_m, int ncols) {
    return type == T_Q4_K && ncols <= 4 && total_m * K <= (int64_t)40 << 20;
}

// K is always cut 16 ways (fewer when it has fewer super-blocks), whatever the number of rows: the order of
// the floating-point sums then does not depend on which matrices share a launch, and measured over the same
// shapes it is as fast as cutting by the size of the grid.  16-wave workgroups: one row group each, or
// several when K is short, as long as that leaves about two workgroups per CU.
void launch_direct16(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int col0, int ncols, int num_cus,
                     hipStream_t s) {
    Direct16Args g;
    int64_t rg = 0;
    for (int i = 0; i < DIRECT16_MULTI; i++) {
        const int j = i < count ? i : count - 1;
        g.p0[i] = ws[j].p0; g.y[i] = ys[j]; g.M[i] = ws[j].M;
        if (i < count) rg += (ws[i].M + 15) / 16;
        g.grp_end[i] = i < count ? (int)rg : 0x7fffffff;
    }
    g.K = ws[0].K;
    g.groups_total = (int)rg;
    const int nsb = (int)(g.K / QKK);
    int kcut = 16;
    while (kcut > nsb) kcut >>= 1;
    int groups = 16 / kcut;
    while (groups > 1 && (rg + groups - 1) / groups < 2 * (int64_t)num_cus) groups >>= 1;
    const unsigned grid = (unsigned)((rg + groups - 1) / groups);
    const int threads = 64 * kcut * groups;
    if (count > 1) direct16_q4k_kernel<true><<<grid, threads, 0, s>>>(g, a, col0, ncols, kcut, threads);
    else direct16_q4k_kernel<false><<<grid, threads, 0, s>>>(g, a, col0, ncols, kcut, threads);
}

// y[i] = sum over slices of part[slice][i], in slice order; V = float4, or float for a y that is not 16-byte aligned
// (a caller's offset into a larger tensor): the same sums in the same order either way
__device__ __forceinline__ void add_to(float4 &a, const float4 &v) { a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w; }
__device__ __forceinline__ void add_to(float &a, const float &v) { a += v; }
template <class V>
__global__ __launch_bounds__(256) void sum_slices_kernel(const V *__restrict__ part, V *__restrict__ y, int64_t n, int slices) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        V acc = part[i];
        for (int sl = 1; sl < slices; sl++) add_to(acc, part[sl * n + i]);
        y[i] = acc;
    }
}

// K slices for a single tensor: when 128 x 128 tiles alone would leave CUs idle, cut K so that the
// large tile (half the vector-ALU work per MFMA of the small one) still fills the machine.
int pick_ksplit(int64_t K, int64_t M, int64_t N, int num_cus) {
    const int64_t tiles = (M + 127) / 128 * ((N + 127) / 128), nsb = K / QKK;
    if ((N * M) % 4 != 0) return 1;
    int ks = 1;
    while (ks < 4 && tiles * ks * 2 <= num_cus && nsb / (ks * 2) >= 16) ks *= 2;
    return ks;
}

}  // namespace

bool gemm_supports(int type, int64_t K, int64_t M) {
    return (type == T_Q4_K || type == T_Q6_K) && K >= QKK && K % QKK == 0 && M >= 1;
}

size_t gemm_workspace_floats(int type, int64_t K, int64_t M, int64_t N, int num_cus) {
    if (!gemm_supports(type, K, M)) return 0;
    const int ks = pick_ksplit(K, M, N, num_cus);
    return ks > 1 ? (size_t)ks * N * M : 0;
}

template <class G>
hipError_t launch3(const DevWeight *ws, float *const *ys, int count, const DevAct &a, float *workspace,
                   size_t workspace_floats, int num_cus, hipStream_t s) {
    GemmArgs ga;
    int64_t tiles_m = 0;
    for (int i = 0; i < GEMM_MULTI; i++) {
        const int j = i < count ? i : count - 1;
        ga.p0[i] = ws[j].p0; ga.p1[i] = ws[j].p1; ga.p2[i] = ws[j].p2; ga.d[i] = ws[j].d;
        ga.y[i] = ys[j]; ga.M[i] = ws[j].M;
        if (i < count) tiles_m += (ws[i].M + 127) / 128;
        ga.tile_end[i] = i < count ? (int)tiles_m : 0x7fffffff;
    }
    ga.K = ws[0].K; ga.type = ws[0].type;
    int ksplit = count == 1 ? pick_ksplit(ws[0].K, ws[0].M, a.N, num_cus) : 1;
    if (ksplit > 1 && (!workspace || workspace_floats < (size_t)ksplit * a.N * ws[0].M)) ksplit = 1;
    // Q6_K: 128 x 128 tiles when they still give every CU work for most of the run, else 128 x 64.  Q4_K
    // unpacks with less vector work, and two resident 128 x 64 workgroups per CU (each covering the other's
    // waits) measure 3..8 % faster than one 128 x 128 at every batch size from 512 to 8192.
    const int64_t big = tiles_m * ((a.N + 127) / 128) * ksplit;
    const bool tnt2 = ksplit > 1 || (ga.type == T_Q6_K && 2 * big >= 3 * (int64_t)num_cus);
    const int64_t tn = tnt2 ? 128 : 64, tiles_n = (a.N + tn - 1) / tn;
    const int64_t gx = tiles_n * ((tiles_m + 7) / 8 * 8);  // whole rounds of the 8 XCDs
    if (tiles_m > 0x7ffffff0 || gx > 0x7fffffff) return hipErrorInvalidValue;
    const dim3 grid((unsigned)gx, (unsigned)ksplit);
    float *part = ksplit > 1 ? workspace : nullptr;
    const GemmIds none{nullptr, nullptr, nullptr, 0};
    if (tnt2) gemm3_kernel<G, 2><<<grid, 512, 0, s>>>(ga, a, (int)tiles_m, (int)tiles_n, part, none);
    else gemm3_kernel<G, 1><<<grid, 512, 0, s>>>(ga, a, (int)tiles_m, (int)tiles_n, part, none);
    if (ksplit > 1) {
        const bool vec = ((uintptr_t)ys[0] & 15) == 0 && (a.N * ws[0].M) % 4 == 0;
        const int64_t n = a.N * ws[0].M / (vec ? 4 : 1);
        const unsigned blocks = (unsigned)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048);
        if (vec) sum_slices_kernel<float4><<<blocks, 256, 0, s>>>(reinterpret_cast<const float4 *>(part), reinterpret_cast<float4 *>(ys[0]), n, ksplit);
        else sum_slices_kernel<float><<<blocks, 256, 0, s>>>(part, ys[0], n, ksplit);
    }
    return hipGetLastError();
}

int gemm_max_multi() { return GEMM_MULTI; }

bool skinny_supports(int type, int64_t K, int64_t M) {
    return gemm_supports(type, K, M);
}

// How many waves cut K in a workgroup.  Measured over decode shapes (gate 14336 x 4096, down 4096 x 14336,
// q 4096 x 4096, the 128256-row head): the kernel runs best with about eight waves per CU over the whole
// grid -- fewer leave the memory system idle, more only add pipeline fills and K-cut sums -- and with
// every wave having at least two super-blocks.
int skinny_waves(int64_t row_groups, int64_t nsb, int num_cus) {
    const int64_t want = ((int64_t)num_cus * 8 + row_groups / 2) / row_groups;  // nearest
    int waves = want >= 8 ? 8 : want >= 6 ? 6 : want >= 4 ? 4 : want >= 3 ? 3 : want >= 2 ? 2 : 1;
    while (waves > 1 && nsb / waves < 2) waves = waves > 4 ? waves - 2 : waves - 1;
    return waves;
}

template <class S, int NCT, bool ID, int NST>
void launch_skinny_grid(const DevWeight &w, const DevAct &a, int col0, int ncols, float *y, const SkinnyIds &si,
                        int64_t grid, int waves, hipStream_t s) {
    typedef SkinnyGeo<S, NCT, NST> Geo;
    const size_t lds = (size_t)waves * (Geo::WAVE_BYTES + Geo::PART_BYTES);
    // more than 64 KiB of dynamic LDS has to be allowed once per device
    static bool allowed[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 && !allowed[dev]) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(skinny_kernel<S, NCT, ID, NST>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        allowed[dev] = true;
    }
    skinny_kernel<S, NCT, ID, NST><<<(unsigned)grid, 64 * waves, lds, s>>>(w, a, col0, ncols, y, si, waves, (int)grid, SkinnyMulti{});
}

// several matrices in one launch: their row groups numbered through (see SkinnyMulti)
template <class S, int NCT>
void launch_skinny_grid_multi(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int ncols, int waves,
                              int num_cus, hipStream_t s) {
    typedef SkinnyGeo<S, NCT, 2> Geo;
    SkinnyMulti mt;
    int64_t rg = (ws[0].M + 15) / 16;
    for (int t = 0; t < 3; t++) {
        const int j = t + 1 < count ? t + 1 : count - 1;
        mt.p0[t] = ws[j].p0; mt.p1[t] = ws[j].p1; mt.p2[t] = ws[j].p2; mt.d[t] = ws[j].d; mt.y[t] = ys[j]; mt.M[t] = ws[j].M;
        mt.grp_end[t] = t + 1 < count ? (int)rg : 0x7fffffff;
        if (t + 1 < count) rg += (ws[j].M + 15) / 16;
    }
    mt.groups_total = (int)rg;
    int64_t grid = rg;
    if (waves == 1) {
        const int64_t items = (rg + (int64_t)num_cus * 4) / ((int64_t)num_cus * 8);
        if (items > 1) grid = (rg + items - 1) / items;
    }
    const size_t lds = (size_t)waves * (Geo::WAVE_BYTES + Geo::PART_BYTES);
    static bool allowed[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 && !allowed[dev]) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(skinny_kernel<S, NCT, false, 2, true>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        allowed[dev] = true;
    }
    skinny_kernel<S, NCT, false, 2, true><<<(unsigned)grid, 64 * waves, lds, s>>>(ws[0], a, 0, ncols, ys[0], SkinnyIds{}, waves,
                                                                                  (int)grid, mt);
}

template <class S, int NCT, bool ID>
void launch_skinny_as(const DevWeight &w, const DevAct &a, int col0, int ncols, float *y, const SkinnyIds &si,
                      int64_t row_groups, int num_cus, hipStream_t s) {
    const int waves = skinny_waves(row_groups, w.K / QKK, num_cus);
    // More row groups than eight waves per CU: each workgroup walks through several of them, its copy
    // stream continuing from one into the next.  Expert-indexed launches keep one item per workgroup:
    // their columns change from group to group.
    int64_t grid = row_groups;
    if (!ID && waves == 1) {
        const int64_t items = (row_groups + (int64_t)num_cus * 4) / ((int64_t)num_cus * 8);  // nearest, at least 1
        if (items > 1) grid = (row_groups + items - 1) / items;
    }
    // One-wave workgroups (many row groups: the output head) are latency-bound with one super-block in flight per
    // wave; a third stage doubles that where eight waves with three stages still fit a CU's LDS.
    typedef SkinnyGeo<S, NCT, 3> Geo3;
    if (!ID && waves == 1 && 8 * (Geo3::WAVE_BYTES + Geo3::PART_BYTES) <= 160 * 1024)
        launch_skinny_grid<S, NCT, ID, 3>(w, a, col0, ncols, y, si, grid, waves, s);
    else
        launch_skinny_grid<S, NCT, ID, 2>(w, a, col0, ncols, y, si, grid, waves, s);
}

bool skinny_rows_wanted(const DevWeight &w, int ncols, int num_cus) { return rows_wanted(w, ncols, num_cus); }

// Which skinny kernel a single K-quant product of ncols columns takes: 1 deep direct-load (skinny_deep.hip), 2 the
// many-small-waves direct-load kernel, 3 the Q4_K rows kernel, 4 the staged kernel, 5 the Q6_K rows kernel.
int skinny_kind(const DevWeight &w, int ncols, int num_cus) {
    if (w.type == T_Q4_K) {
        if (deep16_wanted(w.type, w.K, w.M, ncols, num_cus)) return 1;
        if (direct16_wanted(w.type, w.K, w.M, ncols)) return 2;
        if (rows_q4k_wanted(w.type, w.K, w.M, ncols, num_cus)) return 3;
        return 4;
    }
    // (on the 128256-row head the rows kernel stays ahead of the deep one: 82-85 against 88-94 us at 2..8 columns)
    const bool rows = rows_wanted(w, ncols, num_cus);
    if (!rows && deep6_wanted(w.type, w.K, w.M, ncols, num_cus)) return 1;
    return rows ? 5 : 4;
}

hipError_t launch_skinny(const DevWeight &w, const DevAct &a, int col0, int ncols, float *y, int num_cus, hipStream_t s) {
    if (!skinny_supports(w.type, w.K, w.M) || a.type != T_Q8_K || a.K != w.K || !a.sd8 || !a.sd16) return hipErrorInvalidValue;
    if (ncols < 1 || ncols > 16 || col0 < 0 || col0 + ncols > a.N) return hipErrorInvalidValue;
    if ((int64_t)(col0 + ncols) * a.K >= ((int64_t)1 << 32)) return hipErrorInvalidValue;  // 32-bit activation offsets
    if ((w.M + 15) / 16 > 0x7fffffff) return hipErrorInvalidValue;
    const SkinnyIds none{};
    const int64_t rg = (w.M + 15) / 16;
    const int kind = skinny_kind(w, ncols, num_cus);
    if (kind == 1 && w.type == T_Q6_K) return launch_deep6(w, y, a, col0, ncols, num_cus, s);
    if (kind == 1) return launch_deep16(&w, &y, 1, a, col0, ncols, num_cus, s);
    if (w.type == T_Q4_K) {
        if (kind == 2) launch_direct16(&w, &y, 1, a, col0, ncols, num_cus, s);
        else if (kind == 3) launch_rows_q4k(&w, &y, 1, a, col0, ncols, num_cus, s);
        else if (ncols <= 8) launch_skinny_as<Sk16Q4K, 8, false>(w, a, col0, ncols, y, none, rg, num_cus, s);
        else launch_skinny_as<Sk16Q4K, 16, false>(w, a, col0, ncols, y, none, rg, num_cus, s);
    } else {
        if (kind == 5) launch_skinny_rows(w, a, col0, ncols, y, num_cus, s);
        else if (ncols <= 8) launch_skinny_as<Sk16Q6K, 8, false>(w, a, col0, ncols, y, none, rg, num_cus, s);
        else launch_skinny_as<Sk16Q6K, 16, false>(w, a, col0, ncols, y, none, rg, num_cus, s);
    }
    return hipGetLastError();
}

// Several Q4_K matrices that share K against the same three or four activation columns: one launch of
// the direct-load kernel over their numbered-through row groups when together they are small enough for it.
// 1: one launch of the direct-load kernel; 2: one launch of the staged kernel; 3: one launch of the rows kernel;
// 4: one launch of the deep direct-load kernel; 0: no.  Either way every matrix takes the kernel and the K cut it would take in a launch of its own, so the
// results are the same bits as those of separate launches.
int skinny_multi_kind(const DevWeight *ws, int count, int ncols, int num_cus) {
    if (count < 2 || count > DIRECT16_MULTI || ncols < 1 || ncols > 16) return 0;
    int64_t total_m = 0;
    bool each_direct = true, none_direct = true, same_waves = true, each_deep = true, none_deep = true;
    const int waves0 = skinny_waves((ws[0].M + 15) / 16, ws[0].K / QKK, num_cus);
    for (int i = 0; i < count; i++) {
        if (ws[i].type != ws[0].type || ws[i].K != ws[0].K || !skinny_supports(ws[i].type, ws[i].K, ws[i].M)) return 0;
        total_m += ws[i].M;
        const bool dir = direct16_wanted(ws[i].type, ws[i].K, ws[i].M, ncols);
        const bool deep = deep16_wanted(ws[i].type, ws[i].K, ws[i].M, ncols, num_cus) || deep6_wanted(ws[i].type, ws[i].K, ws[i].M, ncols, num_cus);
        each_deep = each_deep && deep;
        none_deep = none_deep && !deep;
        each_direct = each_direct && dir;
        none_direct = none_direct && !dir;
        same_waves = same_waves && skinny_waves((ws[i].M + 15) / 16, ws[i].K / QKK, num_cus) == waves0;
    }
    if ((total_m + 15 * count) / 16 >= 0x7fffffff) return 0;
    // the deep direct-load kernel: its order of sums does not depend on the launch
    if (each_deep && ws[0].type == T_Q4_K && deep16_wanted(ws[0].type, ws[0].K, total_m, ncols, num_cus)) return 4;
    if (!none_deep) return 0;  // (a matrix that takes the deep kernel alone joins no launch of another kernel)
    if (each_direct && direct16_wanted(ws[0].type, ws[0].K, total_m, ncols)) return 1;
    // the rows kernel (it reproduces the K cut each matrix would get alone, see skinny_rows_q4k_kernel)
    if (count <= ROWS_MULTI && none_direct && rows_q4k_wanted(ws[0].type, ws[0].K, total_m, ncols, num_cus)) return 3;
    // staged: the common K cut must still leave at most about 16 waves per CU over the joint grid.  Q4_K only:
    // measured, q + k + v at 6 / 8 / 16 columns take 9.4 / 9.8 / 13.3 us in one launch against 17.0 / 17.6 / 21.2 in
    // three, gate + up at 4..8 columns 19.6..20.9 against 23.0..23.6; the Q6_K kernel (more registers and LDS per
    // wave) comes out 3..7 % slower joined than apart.
    if (ws[0].type == T_Q4_K && none_direct && same_waves && (total_m + 15) / 16 * waves0 <= 16 * (int64_t)num_cus) return 2;
    return 0;
}
bool skinny_multi_supports(const DevWeight *ws, int count, int ncols, int num_cus) {
    return skinny_multi_kind(ws, count, ncols, num_cus) != 0;
}

hipError_t launch_skinny_multi(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int ncols, int num_cus,
                               hipStream_t s) {
    const int kind = skinny_multi_kind(ws, count, ncols, num_cus);
    if (!kind || a.type != T_Q8_K || a.K != ws[0].K || !a.sd8 || !a.sd16) return hipErrorInvalidValue;
    if (ncols < 1 || ncols > a.N || (int64_t)ncols * a.K >= ((int64_t)1 << 32)) return hipErrorInvalidValue;
    if (kind == 4) {
        return launch_deep16(ws, ys, count, a, 0, ncols, num_cus, s);
    } else if (kind == 1) {
        launch_direct16(ws, ys, count, a, 0, ncols, num_cus, s);
    } else if (kind == 3) {
        launch_rows_q4k(ws, ys, count, a, 0, ncols, num_cus, s);
    } else {
        const int waves = skinny_waves((ws[0].M + 15) / 16, ws[0].K / QKK, num_cus);
        if (ws[0].type == T_Q4_K) {
            if (ncols <= 8) launch_skinny_grid_multi<Sk16Q4K, 8>(ws, ys, count, a, ncols, waves, num_cus, s);
            else launch_skinny_grid_multi<Sk16Q4K, 16>(ws, ys, count, a, ncols, waves, num_cus, s);
        } else {
            if (ncols <= 8) launch_skinny_grid_multi<Sk16Q6K, 8>(ws, ys, count, a, ncols, waves, num_cus, s);
            else launch_skinny_grid_multi<Sk16Q6K, 16>(ws, ys, count, a, ncols, waves, num_cus, s);
        }
    }
    return hipGetLastError();
}

bool skinny_id_supports(int type, int64_t K, int64_t M, int64_t pairs, int n_expert) {
    // from about two pairs per expert the experts' weights are worth sharing between pairs
    return pairs >= 2 * (int64_t)n_expert && skinny_supports(type, K, M);
}

hipError_t launch_skinny_id(const DevWeight &w, int n_expert, const DevAct &a, const int *ids, int n_used, int n_tokens,
                            int b_cols, float *y, int *groups, int num_cus, hipStream_t s) {
    if (n_expert < 1 || w.M % n_expert || !skinny_supports(w.type, w.K, w.M / n_expert) || a.type != T_Q8_K ||
        a.K != w.K || !a.sd8 || !a.sd16 || !ids || !y || !groups || n_used < 1 || n_tokens < 1 || b_cols < 1 ||
        a.N != (int64_t)b_cols * n_tokens || (int64_t)a.N * a.K >= ((int64_t)1 << 32))
        return hipErrorInvalidValue;
    const int64_t pairs = (int64_t)n_used * n_tokens;
    if (hipError_t e = launch_group_pairs(ids, (int)pairs, n_expert, 16, groups, s)) return e;
    SkinnyIds si;
    si.groups = groups; si.M = w.M / n_expert; si.n_used = n_used; si.b_cols = b_cols;
    si.wgs_per_group = (int)((si.M + 15) / 16);
    // every expert (and the bucket of bad ids) ends with at most one partly filled group
    const int64_t max_groups = min(pairs, (int64_t)n_expert + 1 + pairs / 16);
    const int64_t wgs = max_groups * si.wgs_per_group;
    if (wgs > 0x7fffffff) return hipErrorInvalidValue;
    if (w.type == T_Q4_K) launch_skinny_as<Sk16Q4K, 16, true>(w, a, 0, 16, y, si, wgs, num_cus, s);
    else launch_skinny_as<Sk16Q6K, 16, true>(w, a, 0, 16, y, si, wgs, num_cus, s);
    return hipGetLastError();
}

bool gemm_id_supports(int type, int64_t K, int64_t M, int64_t pairs, int n_expert) {
    // worth sorting the pairs and padding every expert to 64-row tiles from about sixteen pairs per expert
    return gemm_supports(type, K, M) && pairs >= 16 * (int64_t)n_expert;
}

// Pairs per tile: 64, and for Q6_K 128 once the experts see 128 pairs each on average (measured on 8 experts of
// 14336 x 4096 at 2 of 8: Q6_K 351 against 290 TOPS at 1024 pairs per expert, even at 128; Q4_K is faster
// with 64 at every count, as in the dense product).
int gemm_id_tile_width(int type, int64_t pairs, int n_expert) {
    return type == T_Q6_K && pairs >= 128 * (int64_t)n_expert ? 128 : 64;
}

hipError_t launch_gemm_id(const DevWeight &w, int n_expert, const DevAct &a, const int *tiles, const int *src_rows,
                          const int *out_rows, int64_t max_tiles, int tile_width, float *y, hipStream_t s) {
    if (tile_width != 64 && !(tile_width == 128 && w.type == T_Q6_K)) return hipErrorInvalidValue;
    if (n_expert < 1 || w.M % n_expert || !gemm_supports(w.type, w.K, w.M / n_expert) || a.type != T_Q8_K || a.K != w.K ||
        !a.sd8 || !a.sd16 || !tiles || !src_rows || !out_rows || !y || max_tiles < 1 ||
        (int64_t)a.N * a.K >= ((int64_t)1 << 32))  // the copies address activation bytes with 32-bit offsets
        return hipErrorInvalidValue;
    GemmArgs ga;
    for (int i = 0; i < GEMM_MULTI; i++) {
        ga.p0[i] = w.p0; ga.p1[i] = w.p1; ga.p2[i] = w.p2; ga.d[i] = w.d; ga.y[i] = y; ga.M[i] = w.M;
        ga.tile_end[i] = 0x7fffffff;
    }
    ga.K = w.K; ga.type = w.type;
    const GemmIds gi{tiles, src_rows, out_rows, w.M / n_expert};
    const int64_t tiles_m = (gi.expert_rows + 127) / 128;
    const int64_t gx = max_tiles * ((tiles_m + 7) / 8 * 8);  // whole rounds of the 8 XCDs
    if (gx > 0x7fffffff) return hipErrorInvalidValue;
    if (w.type == T_Q4_K) gemm3_kernel<GemmQ4K, 1><<<(unsigned)gx, 512, 0, s>>>(ga, a, (int)tiles_m, (int)max_tiles, nullptr, gi);
    else if (tile_width == 128) gemm3_kernel<GemmQ6K, 2><<<(unsigned)gx, 512, 0, s>>>(ga, a, (int)tiles_m, (int)max_tiles, nullptr, gi);
    else gemm3_kernel<GemmQ6K, 1><<<(unsigned)gx, 512, 0, s>>>(ga, a, (int)tiles_m, (int)max_tiles, nullptr, gi);
    return hipGetLastError();
}

hipError_t launch_gemm_multi(const DevWeight *ws, float *const *ys, int count, const DevAct &a, float *workspace,
                             size_t workspace_floats, int num_cus, hipStream_t s) {
    if (count < 1 || count > GEMM_MULTI) return hipErrorInvalidValue;
    for (int i = 0; i < count; i++)
        if (ws[i].type != ws[0].type || ws[i].K != ws[0].K || !gemm_supports(ws[i].type, ws[i].K, ws[i].M) || !ys[i])
            return hipErrorInvalidValue;
    if (a.type != T_Q8_K || a.K != ws[0].K || a.N < 1 || !a.sd8 || !a.sd16) return hipErrorInvalidValue;
    return ws[0].type == T_Q4_K ? launch3<GemmQ4K>(ws, ys, count, a, workspace, workspace_floats, num_cus, s)
                                : launch3<GemmQ6K>(ws, ys, count, a, workspace, workspace_floats, num_cus, s);
}

hipError_t launch_gemm(const DevWeight &w, const DevAct &a, float *y, int64_t ldy, float *workspace,
                       size_t workspace_floats, int num_cus, hipStream_t s) {
    if (ldy != w.M) return hipErrorInvalidValue;
    float *ys[1] = {y};
    return launch_gemm_multi(&w, ys, 1, a, workspace, workspace_floats, num_cus, s);
}

}  // namespace miqmm
