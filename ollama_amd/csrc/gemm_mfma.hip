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
//       Q6_K:  p = sc*e (e = 0..63 unsigned 6-bit value, |p| <= 8064) = 64*p_h + p_l, p_l in 0..63,
//              p_h in -126..126;                                      sum p*y    = 64*A_h + A_l
//   * The terms that multiply sums of activations (Q4_K mins; the -32 offset of Q6_K) use the Q8_K
//     block sums, also on the matrix cores: sum_j m_j * S_j with S split into two int8 digits
//     (S = 64*S_h + S_l) costs two more MFMAs per 32x32 tile and super-block.
//   * Per super-block and output there remains one fp32 epilogue: y += yd_n * (d_m * I - dmin_m * Imin).
//
// Data flow: the activation tile of a super-block (128 rows x 256 int8, their block scale and block-sum
// digits) goes HBM/L2 -> LDS by direct-to-LDS loads (global_load_lds_dwordx4: no registers, no vector
// ALU work, two LDS buffers so the copy of the next tile runs under the current tile's MFMAs) and is
// read as the MFMA A operand; the 16-byte pieces of a row are XOR-swizzled with the row number so the
// 32 rows x 16 bytes of an operand read fall on distinct banks.  Each wave owns 32 weight rows, loads their packed
// blocks straight from HBM, expands them to digit planes IN REGISTERS as the MFMA B operand (each lane
// needs 16 consecutive K values of one row -- exactly a 16-byte piece of the GGUF block) and reuses them
// for all four 32-row activation sub-tiles.  W on the B side puts one weight row in each lane's 16
// accumulators (one d/dmin per lane) and makes the output stores contiguous in m.
#include <hip/hip_fp16.h>

#include "internal.h"

namespace miqmm {

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
    static constexpr int RAW_LOADS = 5;  // memory instructions of load_raw
    static __device__ __forceinline__ void load_raw(const DevWeight &w, int64_t row, int64_t sb, int h, Raw &raw) {
        const uint8_t *p = w.p0 + row * (w.K / QKK * Q4_K_BYTES) + sb * Q4_K_BYTES;
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
    static constexpr int RAW_LOADS = 8;
    static __device__ __forceinline__ void load_raw(const DevWeight &w, int64_t row, int64_t sb, int h, Raw &raw) {
        const uint8_t *pl = w.p0 + row * (w.K / 2) + sb * 128 + 16 * h;
        const uint8_t *ph = w.p1 + row * (w.K / 4) + sb * 64 + 16 * h;
#pragma unroll
        for (int H = 0; H < 2; H++) {
            raw.L[H][0] = ld16(pl + 64 * H);
            raw.L[H][1] = ld16(pl + 64 * H + 32);
            raw.Hq[H] = ld16(ph + 32 * H);
        }
        raw.scv = ld16(w.p2 + row * (w.K / 16) + sb * 16);
        raw.dh = w.d[row * (w.K / QKK) + sb];
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
                const s2 pe = as_s2(e & 0x00ff00ffu) * scv2;         // elements 0 and 2, 16-bit products
                const s2 po = as_s2((e >> 8) & 0x00ff00ffu) * scv2;  // elements 1 and 3
                const unsigned le = as_u(pe) & 0x003f003fu, lo_ = as_u(po) & 0x003f003fu;
                const unsigned he = as_u(pe >> 6), ho = as_u(po >> 6);  // arithmetic shift per 16-bit lane
                bl[t] = (int)(le | (lo_ << 8));
                bh[t] = (int)__builtin_amdgcn_perm(ho, he, 0x06020400u);  // bytes: he.b0, ho.b0, he.b2, ho.b2
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
        return d * (float)((ah << 6) + al - __float_as_int(fm));
    }
};

typedef __attribute__((address_space(3))) void lds_ptr_t;
typedef const __attribute__((address_space(1))) void glb_ptr_t;

// One LDS stage: the activation tile of one super-block.  q rows are 256 bytes, unpadded; the 16-byte
// piece p of row R is stored at piece position p ^ (R & 15).
template <int TN>
struct Stage {
    uint8_t q[TN * 256];
    uint8_t s[TN * 32];
    float yd[TN < 256 ? 256 : TN];  // keeps the stage a multiple of 1 KiB
};

// Workgroup = WAVES waves x 32 weight rows, against TN = 32*TNT activation rows.  Per super-block:
//   start the direct-to-LDS copy of the next activation stage; expand the prefetched packed weights
//   into the B operand; start the loads of the next super-block's packed weights; run the four 32-row
//   activation sub-tiles (18 MFMAs + fp32 epilogue each); wait for the copies; one barrier.
template <class G, int WAVES, int TNT>
__global__ __launch_bounds__(64 * WAVES, 1) void gemm_kernel(DevWeight w, DevAct a, float *__restrict__ y,
                                                             int64_t ldy, int tiles_n) {
    constexpr int TN = 32 * TNT;  // activation rows per workgroup
    typedef Stage<TN> StageT;
    __shared__ __attribute__((aligned(1024))) StageT lds[3];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, h = lane >> 5;
    // Workgroup i runs on XCD i % 8 and every XCD has its own L2: the tiles_n workgroups that share a
    // block of weight rows are given ids that are 8 apart, so they meet in one L2.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int tile_n = slot % tiles_n, tile_m = xcd + 8 * (slot / tiles_n);
    if ((int64_t)tile_m * (32 * WAVES) >= w.M) return;  // the grid is rounded up to 8 row blocks
    const int64_t n0 = (int64_t)tile_n * TN, m0 = (int64_t)tile_m * (32 * WAVES);
    const int64_t row = min(m0 + 32 * wave + r, w.M - 1);  // rows past M are computed and dropped
    const int64_t nsb = w.K / QKK;
    const uint8_t *aq = reinterpret_cast<const uint8_t *>(a.qs);
    const uint8_t *asd = G::digits(a);

    float acc[TNT][16];
#pragma unroll
    for (int t = 0; t < TNT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[t][i] = 0.f;

    // direct-to-LDS copy of the stage of super-block sb: every wave instruction moves 64 x 16 bytes to
    // 1 KiB of consecutive LDS; which global piece a lane fetches implements the swizzle.  Activation
    // rows past N are read too (the planes are allocated in whole tiles) and their results dropped, so
    // all addresses of a lane are one base plus a uniform stride.
    constexpr int QI = TN / 4 / WAVES;     // quant copy instructions per wave and stage
    constexpr int QSTEP = 4 * WAVES;       // rows between consecutive instructions of a wave (16 or 8)
    constexpr int NB = 16 / QSTEP < 1 ? 1 : 16 / QSTEP;  // distinct (row & 15) values per lane (1 or 2)
    const uint8_t *qbase[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) {
        const int R = 4 * wave + (lane >> 4) + QSTEP * j;
        qbase[j] = aq + (n0 + R) * a.K + 16 * ((lane & 15) ^ (R & 15));
    }
    constexpr int RPI = 1024 / G::SD;      // rows per instruction for the digit plane (64 or 32)
    const uint8_t *sbase = asd + (n0 + lane / (G::SD / 16)) * nsb * G::SD + 16 * (lane % (G::SD / 16));
    const float *dbase = a.d + (n0 + lane) * nsb;
    auto stage_copy = [&](StageT &st, int64_t sb) __attribute__((always_inline)) {  // quants last: the in-order wait at the end of an iteration counts on it
#pragma unroll
        for (int i = 0; i < (TN / RPI + WAVES - 1) / WAVES; i++) {
            const int blk = wave + WAVES * i;  // uniform
            if (blk < TN / RPI) {
                const uint8_t *g = sbase + ((int64_t)RPI * blk * nsb + sb) * G::SD;
                __builtin_amdgcn_global_load_lds((glb_ptr_t *)g, (lds_ptr_t *)(st.s + 1024 * blk), 16, 0, 0);
            }
        }
        if (wave < (TN + 63) / 64) {  // block scales: 64 rows per instruction
            const float *g = dbase + (int64_t)64 * wave * nsb + sb;
            __builtin_amdgcn_global_load_lds((glb_ptr_t *)g, (lds_ptr_t *)(st.yd + 64 * wave), 4, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < QI; i++) {
            const uint8_t *g = qbase[i % NB] + (int64_t)(QSTEP * (i - i % NB)) * a.K + sb * QKK;
            __builtin_amdgcn_global_load_lds((glb_ptr_t *)g, (lds_ptr_t *)(st.q + 1024 * (wave + WAVES * i)), 16, 0, 0);
        }
    };

    // A-operand piece offsets inside a row, swizzled: piece 2s+h of row R sits at (2s+h) ^ (R & 15)
    const int swz = 16 * (h ^ (r & 15));

    // One super-block: expand the packed weights fetched two iterations ago, start the copies and the
    // weight loads for two super-blocks ahead (three LDS stages, two packed-weight register sets: a
    // load has two whole iterations to arrive), run the MFMAs of this stage, then wait for everything
    // except what was just issued.
    auto body = [&](typename G::Raw &raw, int64_t sb) __attribute__((always_inline)) {
        StageT &cur = lds[sb % 3];
        // the last two iterations fetch the final super-block again (into a stage nobody reads): the
        // loop body stays free of branches and the wait below can always leave the same number of
        // memory instructions in flight
        const int64_t sbn = min(sb + 2, nsb - 1);
        BOperand b;
#if defined(GEMV_VARIANT) && GEMV_VARIANT == 15
        __builtin_memset(&b, 1, sizeof(b)); b.d = __int_as_float(raw.hdr.x);
#else
        G::expand(raw, h, b);
#endif
#if !(defined(GEMV_VARIANT) && (GEMV_VARIANT == 16 || GEMV_VARIANT == 18))
        stage_copy(lds[(sb + 2) % 3], sbn);  // that stage was last read in iteration sb-1: every wave has passed its barrier
#endif
#if !(defined(GEMV_VARIANT) && (GEMV_VARIANT == 17 || GEMV_VARIANT == 18))
        G::load_raw(w, row, sbn, h, raw);
#endif
        // The matrix cores and the vector ALU are fed from one in-order instruction stream per wave, and
        // there is one wave per SIMD: to keep both busy the fp32 epilogue of sub-tile t-1 is interleaved
        // by hand with the MFMAs of sub-tile t -- per k-step two MFMAs (64 matrix-core cycles), then
        // the epilogue of two outputs -- with scheduling barriers pinning that order.
        const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        v16i ah[2], al[2], xl[2], xh[2];
#pragma unroll
        for (int t = 0; t <= TNT; t++) {
            const int p = t & 1, q = p ^ 1;  // accumulator set being produced / consumed
            const uint8_t *arow = cur.q + (32 * (t < TNT ? t : 0) + r) * 256;
            v4i abuf[3];
            if (t < TNT) {
                const v4i sv = *reinterpret_cast<const v4i *>(cur.s + (32 * t + r) * G::SD + (G::SD == 32 ? 16 * h : 0));
                abuf[0] = *reinterpret_cast<const v4i *>(arow + (0 ^ swz));
                abuf[1] = *reinterpret_cast<const v4i *>(arow + (32 ^ swz));
                xl[p] = mfma(sv, b.min_lo, zero);
                xh[p] = mfma(sv, b.min_hi, zero);
                ah[p] = zero;
                al[p] = zero;
            }
#pragma unroll
            for (int s = 0; s < 8; s++) {
                if (t < TNT) {
                    if (s + 2 < 8) abuf[(s + 2) % 3] = *reinterpret_cast<const v4i *>(arow + ((32 * (s + 2)) ^ swz));
                    const v4i av = abuf[s % 3];
#if defined(GEMV_VARIANT) && (GEMV_VARIANT == 12 || GEMV_VARIANT == 14)
                    ah[p][s] ^= av[0] ^ b.hi[s][1]; al[p][s] ^= av[2] ^ b.lo[s][3];   // MFMAs removed
#else
                    ah[p] = mfma(av, b.hi[s], ah[p]);
                    al[p] = mfma(av, b.lo[s], al[p]);
#endif
                }
                __builtin_amdgcn_sched_barrier(0);
                if (t > 0) {  // outputs 2s and 2s+1 of sub-tile t-1; accumulator i is activation row 8(i/4) + 4h + i%4
#pragma unroll
                    for (int i = 2 * s; i < 2 * s + 2; i++) {
                        const float yd = cur.yd[32 * (t - 1) + 8 * (i >> 2) + 4 * h + (i & 3)];
                        const float fm = G::fold_min(b.dmin, xh[q][i], xl[q][i]);
#if defined(GEMV_VARIANT) && (GEMV_VARIANT == 11 || GEMV_VARIANT == 14)
                        acc[t - 1][i] += __int_as_float(ah[q][i] ^ al[q][i]) + yd + fm * 0.f;
#else
                        acc[t - 1][i] = __builtin_fmaf(yd, G::combine(b.d, ah[q][i], al[q][i], fm), acc[t - 1][i]);
#endif
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // the youngest QI + RAW_LOADS memory instructions are the quant copies and packed-weight loads
        // for super-block sb+2; everything older (stage sb+1, weights sb+1) must have landed
        constexpr int KEEP = QI + G::RAW_LOADS;
#if defined(GEMV_VARIANT) && GEMV_VARIANT >= 16 && GEMV_VARIANT <= 18
        __builtin_amdgcn_s_waitcnt(0);
#else
        __builtin_amdgcn_s_waitcnt((KEEP & 15) | (7 << 4) | (15 << 8) | ((KEEP >> 4) << 14));
#endif
        // a bare barrier: __syncthreads() carries a fence that drains every outstanding load, i.e. it
        // would wait for the copies issued a moment ago.  What must be ordered here is LDS only: the
        // copies of the next stage are complete (the wait above, in every wave) and this wave's reads
        // of the current stage have returned (they fed the MFMAs above).
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };

    // ---- prologue: stages 0 and 1, packed weights 0 and 1
    typename G::Raw raw0, raw1;
    G::load_raw(w, row, 0, h, raw0);
    stage_copy(lds[0], 0);
    if (nsb > 1) {
        G::load_raw(w, row, 1, h, raw1);
        stage_copy(lds[1], 1);
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    for (int64_t sb = 0; sb < nsb; sb += 2) {
        body(raw0, sb);
        if (sb + 1 < nsb) body(raw1, sb + 1);
    }

    // ---- store: lanes r = 0..31 hold consecutive m
    const int64_t m = m0 + 32 * wave + r;
    if (m < w.M) {
#pragma unroll
        for (int t = 0; t < TNT; t++) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int64_t n = n0 + 32 * t + 8 * (i >> 2) + 4 * h + (i & 3);
                if (n < a.N) y[n * ldy + m] = acc[t][i];
            }
        }
    }
}

}  // namespace

bool gemm_supports(int type, int64_t K, int64_t M) {
    return (type == T_Q4_K || type == T_Q6_K) && K >= QKK && K % QKK == 0 && M >= 1;
}

template <class G>
hipError_t launch_cfg(const DevWeight &w, const DevAct &a, float *y, int64_t ldy, int num_cus, hipStream_t s) {
    // One workgroup per CU (three LDS stages, one wave per SIMD with the full register file).  Prefer
    // the largest tile that still gives about one workgroup per CU; smaller tiles re-expand the weights
    // more often but keep all CUs (and all four SIMDs) busy on the smaller matrices.
    struct Cfg { int waves, tn; } cfgs[3] = {{4, 128}, {4, 64}, {2, 64}};
    int pick = 2;
    for (int i = 0; i < 3; i++) {
        const int64_t t = ((w.M + 32 * cfgs[i].waves - 1) / (32 * cfgs[i].waves)) * ((a.N + cfgs[i].tn - 1) / cfgs[i].tn);
        if (4 * t >= 3 * (int64_t)num_cus) { pick = i; break; }
    }
    const int64_t tm = 32 * cfgs[pick].waves, tn = cfgs[pick].tn;
    const int64_t tiles_n = (a.N + tn - 1) / tn, tiles_m = ((w.M + tm - 1) / tm + 7) / 8 * 8;  // whole rounds of 8 XCDs
    if (tiles_n * tiles_m > 0x7fffffff) return hipErrorInvalidValue;
    const unsigned grid = (unsigned)(tiles_n * tiles_m);
    switch (pick) {
    case 0: gemm_kernel<G, 4, 4><<<grid, 256, 0, s>>>(w, a, y, ldy, (int)tiles_n); break;
    case 1: gemm_kernel<G, 4, 2><<<grid, 256, 0, s>>>(w, a, y, ldy, (int)tiles_n); break;
    default: gemm_kernel<G, 2, 2><<<grid, 128, 0, s>>>(w, a, y, ldy, (int)tiles_n); break;
    }
    return hipGetLastError();
}

hipError_t launch_gemm(const DevWeight &w, const DevAct &a, float *y, int64_t ldy, int num_cus, hipStream_t s) {
    if (!gemm_supports(w.type, w.K, w.M) || a.type != T_Q8_K || a.K != w.K || a.N < 1 || !a.sd8 || !a.sd16)
        return hipErrorInvalidValue;
    return w.type == T_Q4_K ? launch_cfg<GemmQ4K>(w, a, y, ldy, num_cus, s) : launch_cfg<GemmQ6K>(w, a, y, ldy, num_cus, s);
}

}  // namespace miqmm
