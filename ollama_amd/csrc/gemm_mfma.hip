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
// Data flow: the activation tile (128 rows x 256 int8, their block scale and block-sum digits) is
// staged in LDS and read as the MFMA A operand; each wave owns 32 weight rows, loads their packed
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

constexpr int TM = 128;       // weight rows per workgroup (4 waves x 32)
constexpr int TN = 128;       // activation rows per workgroup (4 sub-tiles of 32)
constexpr int QROW = 272;     // LDS bytes per activation row: 256 quants + 16 pad (conflict-free b128 reads)
constexpr int SDIG = 32;      // LDS bytes of block-sum digits per activation row

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
    static constexpr int MAIN_SHIFT = 3;   // I = (A_h << 3) + A_l
    static constexpr int NSUM = 8;         // block sums per super-block (one per sub-block of 32)
    // lane (r = lane%32, h = lane/32): elements 32s+16h.. of k-step s = sub-block s.  Sub-blocks 2c and
    // 2c+1 are the low / high nibbles of qs bytes [32c+16h, +16).
    static __device__ __forceinline__ void expand(const DevWeight &w, int64_t row, int64_t sb, int h, BOperand &b) {
        const uint8_t *p = w.p0 + row * (w.K / QKK * Q4_K_BYTES) + sb * Q4_K_BYTES;
        const uint4 hdr = ld16(p);
        uint4 q[4];
#pragma unroll
        for (int c = 0; c < 4; c++) q[c] = ld16(p + 16 + 32 * c + 16 * h);
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
    // block-sum digits of one activation row: S_j = bsums[2j] + bsums[2j+1]; out = [S_l 0..7 | S_h 0..7 | 0 x16]
    static __device__ __forceinline__ void sum_digits(const int16_t *bs, uint4 &d0, uint4 &d1) {
        unsigned lo[2] = {0, 0}, hi[2] = {0, 0};
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int s = (int)bs[2 * j] + (int)bs[2 * j + 1];
            lo[j >> 2] |= (unsigned)(s & 63) << (8 * (j & 3));
            hi[j >> 2] |= (unsigned)((s >> 6) & 0xff) << (8 * (j & 3));
        }
        d0 = make_uint4(lo[0], lo[1], hi[0], hi[1]);
        d1 = make_uint4(0, 0, 0, 0);
    }
    static __device__ __forceinline__ float combine(float d, float dmin, int ah, int al, int xh, int xl) {
        const int I = (ah << 3) + al, Im = (xh << 6) + xl;
        return __builtin_fmaf(-dmin, (float)Im, d * (float)I);
    }
};

// ---- Q6_K --------------------------------------------------------------------------------------
struct GemmQ6K {
    static constexpr int MAIN_SHIFT = 6;
    static constexpr int NSUM = 16;  // block sums per super-block (one per scale group of 16)
    // lane (r, h), k-step s: elements 32s+16h.. = scale group 2s+h; half H = s>>2, run rr = s&3:
    // ql bytes [64H + 32(rr&1) + 16h, +16) (low nibble for rr<2, high for rr>=2), qh bytes [32H+16h, +16) >> 2rr.
    static __device__ __forceinline__ void expand(const DevWeight &w, int64_t row, int64_t sb, int h, BOperand &b) {
        const uint8_t *pl = w.p0 + row * (w.K / 2) + sb * 128 + 16 * h;
        const uint8_t *ph = w.p1 + row * (w.K / 4) + sb * 64 + 16 * h;
        uint4 L[2][2], Hq[2];
#pragma unroll
        for (int H = 0; H < 2; H++) {
            L[H][0] = ld16(pl + 64 * H);
            L[H][1] = ld16(pl + 64 * H + 32);
            Hq[H] = ld16(ph + 32 * H);
        }
        const uint4 scv = ld16(w.p2 + row * (w.K / 16) + sb * 16);
        const unsigned scw[4] = {scv.x, scv.y, scv.z, scv.w};
        b.d = h2f(w.d[row * (w.K / QKK) + sb]);
        b.dmin = 0.f;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const int H = s >> 2, rr = s & 3;
            const uint4 lv = L[H][rr & 1], hv = Hq[H];
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
    // out = [S_l 0..15 | S_h 0..15] with S_g = bsums[g]
    static __device__ __forceinline__ void sum_digits(const int16_t *bs, uint4 &d0, uint4 &d1) {
        unsigned lo[4] = {0, 0, 0, 0}, hi[4] = {0, 0, 0, 0};
#pragma unroll
        for (int g = 0; g < 16; g++) {
            const int s = bs[g];
            lo[g >> 2] |= (unsigned)(s & 63) << (8 * (g & 3));
            hi[g >> 2] |= (unsigned)((s >> 6) & 0xff) << (8 * (g & 3));
        }
        d0 = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        d1 = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    }
    // sum sc*(e-32)*y = sum sc*e*y - 32 * sum_g sc_g*S_g, all in exact integers
    static __device__ __forceinline__ float combine(float d, float, int ah, int al, int xh, int xl) {
        const int I = (ah << 6) + al - 32 * ((xh << 6) + xl);
        return d * (float)I;
    }
};

template <class G>
__global__ __launch_bounds__(256, 2) void gemm_kernel(DevWeight w, DevAct a, float *__restrict__ y, int64_t ldy,
                                                      int tiles_n) {
    __shared__ __attribute__((aligned(16))) uint8_t lds_q[TN * QROW];
    __shared__ __attribute__((aligned(16))) uint8_t lds_s[TN * SDIG];
    __shared__ float lds_yd[TN];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, h = lane >> 5;
    // consecutive workgroups share the weight rows (their tiles differ in n): the second reader hits L2
    const int tile_n = blockIdx.x % tiles_n, tile_m = blockIdx.x / tiles_n;
    const int64_t n0 = (int64_t)tile_n * TN, m0 = (int64_t)tile_m * TM;
    const int64_t row = min(m0 + 32 * wave + r, w.M - 1);  // rows past M are computed and dropped
    const int64_t nsb = w.K / QKK;

    float acc[TN / 32][16];
#pragma unroll
    for (int t = 0; t < TN / 32; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[t][i] = 0.f;

    for (int64_t sb = 0; sb < nsb; sb++) {
        // ---- weights of this wave: HBM -> registers, expanded to digit planes
        BOperand b;
        G::expand(w, row, sb, h, b);

        // ---- activations: HBM/L2 -> LDS (quants, block scale, block-sum digits)
        __syncthreads();  // everyone is done reading the previous stage
#pragma unroll
        for (int i = 0; i < TN * 16 / 256; i++) {
            const int piece = tid + 256 * i, tok = piece >> 4, off = (piece & 15) * 16;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (n0 + tok < a.N) v = ld16(reinterpret_cast<const uint8_t *>(a.qs) + (n0 + tok) * a.K + sb * QKK + off);
            *reinterpret_cast<uint4 *>(lds_q + tok * QROW + off) = v;
        }
        if (tid < TN) {
            uint4 d0 = make_uint4(0, 0, 0, 0), d1 = d0;
            float yd = 0.f;
            if (n0 + tid < a.N) {
                yd = a.d[(n0 + tid) * nsb + sb];
                G::sum_digits(a.bsums + (n0 + tid) * (a.K / 16) + sb * 16, d0, d1);
            }
            lds_yd[tid] = yd;
            *reinterpret_cast<uint4 *>(lds_s + tid * SDIG) = d0;
            *reinterpret_cast<uint4 *>(lds_s + tid * SDIG + 16) = d1;
        }
        __syncthreads();

        // ---- matrix cores: 4 activation sub-tiles of 32 rows against this wave's 32 weight rows
#pragma unroll
        for (int t = 0; t < TN / 32; t++) {
            v16i ah, al, xh, xl;
#pragma unroll
            for (int i = 0; i < 16; i++) ah[i] = al[i] = xh[i] = xl[i] = 0;
            const uint8_t *arow = lds_q + (32 * t + r) * QROW + 16 * h;
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const v4i av = *reinterpret_cast<const v4i *>(arow + 32 * s);
                ah = mfma(av, b.hi[s], ah);
                al = mfma(av, b.lo[s], al);
            }
            const v4i sv = *reinterpret_cast<const v4i *>(lds_s + (32 * t + r) * SDIG + 16 * h);
            xl = mfma(sv, b.min_lo, xl);
            xh = mfma(sv, b.min_hi, xh);
            // ---- fp32 epilogue of the super-block: accumulator i is activation row 8(i/4) + 4h + i%4
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float yd = lds_yd[32 * t + 8 * (i >> 2) + 4 * h + (i & 3)];
                acc[t][i] = __builtin_fmaf(yd, G::combine(b.d, b.dmin, ah[i], al[i], xh[i], xl[i]), acc[t][i]);
            }
        }
    }

    // ---- store: lanes r = 0..31 hold consecutive m
    const int64_t m = m0 + 32 * wave + r;
    if (m < w.M) {
#pragma unroll
        for (int t = 0; t < TN / 32; t++) {
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

hipError_t launch_gemm(const DevWeight &w, const DevAct &a, float *y, int64_t ldy, int, hipStream_t s) {
    if (!gemm_supports(w.type, w.K, w.M) || a.type != T_Q8_K || a.K != w.K || a.N < 1) return hipErrorInvalidValue;
    const int64_t tiles_n = ((int64_t)a.N + TN - 1) / TN, tiles_m = (w.M + TM - 1) / TM;
    if (tiles_n * tiles_m > 0x7fffffff) return hipErrorInvalidValue;
    const unsigned grid = (unsigned)(tiles_n * tiles_m);
    if (w.type == T_Q4_K) gemm_kernel<GemmQ4K><<<grid, 256, 0, s>>>(w, a, y, ldy, (int)tiles_n);
    else gemm_kernel<GemmQ6K><<<grid, 256, 0, s>>>(w, a, y, ldy, (int)tiles_n);
    return hipGetLastError();
}

}  // namespace miqmm
