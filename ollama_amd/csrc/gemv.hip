// Kernels 2 and 4: streaming decode GEMV / skinny GEMM (1..8 activation columns) for GGUF
// Q4_0, Q8_0, Q4_K and the Q6_K output head.
//
// Computes y[n][m] = vec_dot(W row m, Q8(x row n)) with ggml's CPU-backend semantics (integer block
// dot products, scales applied in fp32) -- the work behind Tensor.Mulmat,
// /root/reference/ml/backend.go:151, for batch <= 8.
//
// Shape of the computation (HBM-bound: every weight byte is read exactly once):
//   * A wavefront owns a fixed slice of K (a "segment": 4096 elements for the K-quants, 2048 for
//     Q4_0, 1024 for Q8_0) and a few consecutive rows.  A lane's piece of a row is one or two aligned
//     16-byte loads and the wave as a whole reads a contiguous run of the row.
//   * Because the lane's K positions never change, its Q8 activation quants (and the block scale and
//     partial sums that go with them) are loaded ONCE into registers and reused for every row: the
//     inner loop reads nothing but weights.
//   * Nibbles / 6-bit values are unpacked in registers, multiplied with v_dot4_i32_i8, the sub-block
//     scales applied in-lane, each row reduced across the wave with cross-lane moves; waves that own
//     different K segments of the same rows combine through LDS at the end of the workgroup.
//   * Two kernels.  gemv_thin_kernel (everything up to eight K segments per row): many small waves,
//     a rolled loop of about 1 KiB, one row in registers and the next in flight, the latency hidden
//     by occupancy; optionally quantizes f32 activations itself in its prologue.  gemv_kernel (longer
//     rows only): few waves, each K segment list in registers, rows in double-buffered passes.
#include <hip/hip_fp16.h>

#include "internal.h"
#include "produce_dev.h"
#include "quant_dev.h"

namespace miqmm {

namespace {

constexpr int MAXC = 8;       // activation columns per launch
constexpr int MAX_MULTI = 4;  // weight tensors per launch

__device__ __forceinline__ int dot4(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }

__device__ __forceinline__ float h2f(unsigned int bits16) {
    return __half2float(__ushort_as_half((unsigned short)bits16));
}

__device__ __forceinline__ uint4 ld16(const uint8_t *p) { return *reinterpret_cast<const uint4 *>(p); }

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

// Reduce U per-lane values over the 64 lanes at once.  On return every lane whose (lane & (U-1))
// equals u holds the total of v[u].  The xor-1 / xor-2 exchange steps double as the transposition:
// a lane keeps the value of "its" row and hands the other one to its partner.
template <int U>
__device__ __forceinline__ float reduce_rows(const float (&v)[U], int lane) {
    float w;
    if (U == 4) {
        const bool b0 = lane & 1, b1 = lane & 2;
        const float k01 = b0 ? v[1] : v[0], g01 = b0 ? v[0] : v[1];
        const float k23 = b0 ? v[3] : v[2], g23 = b0 ? v[2] : v[3];
        const float s01 = k01 + dpp_mov<0xB1>(g01);  // quad_perm [1,0,3,2]: lane ^ 1
        const float s23 = k23 + dpp_mov<0xB1>(g23);
        const float k = b1 ? s23 : s01, g = b1 ? s01 : s23;
        w = k + dpp_mov<0x4E>(g);                    // quad_perm [2,3,0,1]: lane ^ 2
    } else if (U == 2) {
        const bool b0 = lane & 1;
        const float k = b0 ? v[1] : v[0], g = b0 ? v[0] : v[1];
        w = k + dpp_mov<0xB1>(g);
        w += dpp_mov<0x4E>(w);
    } else {
        w = v[0] + dpp_mov<0xB1>(v[0]);
        w += dpp_mov<0x4E>(w);
    }
    w += dpp_mov<0x124>(w);  // row_ror:4  -- the other quads of the row of 16; keeps lane & 3
    w += dpp_mov<0x128>(w);  // row_ror:8
    w += __shfl_xor(w, 16);
    w += __shfl_xor(w, 32);
    return w;
}

// ---------------------------------------------------------------------------------------------
// Per-type policies.  Each provides
//   SEG                      elements of K one wave covers per row
//   Geo                      per-lane constants (offsets into the row, shifts, validity)
//   Act                      per-lane, per-column activation registers
//   Raw                      the lane's loaded weight bytes for one row
//   geo(), load_act(), load(), dot()
// A lane whose K slice lies beyond K (ragged last segment) is "dead": its loads are redirected to the
// start of the row / activation row (branch-free, so all loads of a pass stay in one basic block and
// the compiler can wait for exactly the loads it needs) and its activation registers are forced to
// zero, so it contributes exactly 0.
// ---------------------------------------------------------------------------------------------

struct PolQ4K {
    static constexpr int PLANES = 1;  // planes of the device layout a row is read from
    static constexpr int F32_WAVES_ONE_SEG = 16;  // waves per workgroup when it quantizes one column of one-segment rows
    static constexpr int SEG = 4096;  // 16 super-blocks, 4 lanes each
    static constexpr int ACT_BLK = QKK, ACT_BSUM = 16;  // Q8_K: one scale per 256, one sum per 16
    static constexpr bool USES_BSUMS = true;
    static constexpr bool HEAVY = true;
    // lane c (0..3) of a super-block owns qs bytes [32c, 32c+32): low nibbles are sub-block 2c,
    // high nibbles sub-block 2c+1 (32 elements each), and with them scales/mins 2c and 2c+1.
    struct Geo {
        int64_t row_bytes;
        int off;    // byte offset of the lane's super-block in the row
        int qoff;   // byte offset of the lane's 32 qs bytes in the row
        int sh;     // 16*(c&1): where the (2c, 2c+1) byte pair sits inside a scales word
        bool hi;    // c >= 2: sub-blocks 4..7 use the split 4+2 bit packing
        bool live;
    };
    struct Act { int lo[8], hi[8]; float d; int s_lo, s_hi; };
    struct Raw { uint4 hdr, q0, q1; };

    static __device__ __forceinline__ Geo geo(const DevWeight &w, int seg, int lane) {
        Geo g;
        const int sb = seg * 16 + (lane >> 2), c = lane & 3;
        g.row_bytes = w.K / QKK * Q4_K_BYTES;
        g.live = (int64_t)sb * QKK < w.K;
        g.off = g.live ? sb * Q4_K_BYTES : 0;
        g.qoff = g.off + 16 + 32 * c;
        g.sh = 16 * (c & 1);
        g.hi = c >= 2;
        return g;
    }
    template <class AV>
    static __device__ __forceinline__ void load_act(const AV &a, int n, int seg, int lane, const Geo &g, Act &r) {
        const int sb = g.live ? seg * 16 + (lane >> 2) : 0, c = lane & 3;
        const int keep = g.live ? -1 : 0;
        const int4 *q = reinterpret_cast<const int4 *>(a.qs + (int64_t)n * a.K + (int64_t)sb * QKK + 64 * c);
        const int4 v0 = q[0], v1 = q[1], v2 = q[2], v3 = q[3];
        const float dd = a.d[(int64_t)n * (a.K / QKK) + sb];
        const int2 bs = *reinterpret_cast<const int2 *>(a.bsums + (int64_t)n * (a.K / 16) + (int64_t)sb * 16 + 4 * c);
        r.lo[0] = v0.x & keep; r.lo[1] = v0.y & keep; r.lo[2] = v0.z & keep; r.lo[3] = v0.w & keep;
        r.lo[4] = v1.x & keep; r.lo[5] = v1.y & keep; r.lo[6] = v1.z & keep; r.lo[7] = v1.w & keep;
        r.hi[0] = v2.x & keep; r.hi[1] = v2.y & keep; r.hi[2] = v2.z & keep; r.hi[3] = v2.w & keep;
        r.hi[4] = v3.x & keep; r.hi[5] = v3.y & keep; r.hi[6] = v3.z & keep; r.hi[7] = v3.w & keep;
        r.d = g.live ? dd : 0.f;
        r.s_lo = (((short)bs.x) + (bs.x >> 16)) & keep;  // sum of q8 over sub-block 2c
        r.s_hi = (((short)bs.y) + (bs.y >> 16)) & keep;  // ... and 2c+1
    }
    static __device__ __forceinline__ Raw load(const DevWeight &w, const Geo &g, int64_t row) {
        Raw r;
        const uint8_t *p = w.p0 + row * g.row_bytes;
        r.hdr = ld16(p + g.off);
        r.q0 = ld16(p + g.qoff);
        r.q1 = ld16(p + g.qoff + 16);
        return r;
    }
    template <int NC>
    static __device__ __forceinline__ void dot(const Raw &r, const Geo &g, const Act (&a)[NC], float (&acc)[NC]) {
        // hdr.x = d | dmin<<16 ; hdr.y = scales[0..3] ; hdr.z = scales[4..7] ; hdr.w = scales[8..11]
        const float dw = h2f(r.hdr.x & 0xffff), dminw = h2f(r.hdr.x >> 16);
        const unsigned ty = r.hdr.y >> g.sh, tz = r.hdr.z >> g.sh, tw = r.hdr.w >> g.sh;
        // byte pairs (sc[2c], sc[2c+1]) and (m[2c], m[2c+1])
        const unsigned scA = ty & 0x3f3fu, mA = tz & 0x3f3fu;
        const unsigned scB = (tw & 0x0f0fu) | ((ty >> 2) & 0x3030u);
        const unsigned mB = ((tw >> 4) & 0x0f0fu) | ((tz >> 2) & 0x3030u);
        const unsigned scp = g.hi ? scB : scA, mp = g.hi ? mB : mA;
        const int sc_lo = scp & 0xff, sc_hi = scp >> 8, m_lo = mp & 0xff, m_hi = mp >> 8;
        const unsigned v[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
        int lo[8], hi[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            lo[i] = (int)(v[i] & 0x0f0f0f0fu);
            hi[i] = (int)((v[i] >> 4) & 0x0f0f0f0fu);
        }
#pragma unroll
        for (int n = 0; n < NC; n++) {
            int dl = 0, dh = 0;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                dl = dot4(lo[i], a[n].lo[i], dl);
                dh = dot4(hi[i], a[n].hi[i], dh);
            }
            const int isum = __mul24(sc_lo, dl) + __mul24(sc_hi, dh);
            const int msum = __mul24(m_lo, a[n].s_lo) + __mul24(m_hi, a[n].s_hi);
            acc[n] = __builtin_fmaf(dw * a[n].d, (float)isum, acc[n]);
            acc[n] = __builtin_fmaf(-(dminw * a[n].d), (float)msum, acc[n]);
        }
    }
};

// Q5_K in its own 176-byte blocks (16 bytes of header, 32 of fifth bits, 128 of nibbles: every field 16-byte aligned).
// As PolQ4K, plus the fifth bits: bit j of qh[l] belongs to element l of sub-block j, so lane c -- which owns sub-blocks 2c
// and 2c + 1 -- takes bits 2c and 2c + 1 of all 32 bytes and adds 16 to the nibbles whose bit is set.
struct PolQ5K {
    static constexpr int PLANES = 1;
    static constexpr int F32_WAVES_ONE_SEG = 16;
    static constexpr int SEG = 4096;
    static constexpr int ACT_BLK = QKK, ACT_BSUM = 16;
    static constexpr bool USES_BSUMS = true;
    static constexpr bool HEAVY = true;
    struct Geo {
        int64_t row_bytes;
        int off, qoff, sh, hb;  // hb = 2c: the lane's first bit in the bytes of fifth bits
        bool hi, live;
    };
    typedef PolQ4K::Act Act;
    struct Raw { uint4 hdr, h0, h1, q0, q1; };

    static __device__ __forceinline__ Geo geo(const DevWeight &w, int seg, int lane) {
        Geo g;
        const int sb = seg * 16 + (lane >> 2), c = lane & 3;
        g.row_bytes = w.K / QKK * Q5_K_BYTES;
        g.live = (int64_t)sb * QKK < w.K;
        g.off = g.live ? sb * Q5_K_BYTES : 0;
        g.qoff = g.off + 48 + 32 * c;
        g.sh = 16 * (c & 1);
        g.hb = 2 * c;
        g.hi = c >= 2;
        return g;
    }
    template <class AV>
    static __device__ __forceinline__ void load_act(const AV &a, int n, int seg, int lane, const Geo &g, Act &r) {
        PolQ4K::Geo g4;
        g4.live = g.live;
        PolQ4K::load_act(a, n, seg, lane, g4, r);
    }
    static __device__ __forceinline__ Raw load(const DevWeight &w, const Geo &g, int64_t row) {
        Raw r;
        const uint8_t *p = w.p0 + row * g.row_bytes;
        r.hdr = ld16(p + g.off);
        r.h0 = ld16(p + g.off + 16);
        r.h1 = ld16(p + g.off + 32);
        r.q0 = ld16(p + g.qoff);
        r.q1 = ld16(p + g.qoff + 16);
        return r;
    }
    template <int NC>
    static __device__ __forceinline__ void dot(const Raw &r, const Geo &g, const Act (&a)[NC], float (&acc)[NC]) {
        const float dw = h2f(r.hdr.x & 0xffff), dminw = h2f(r.hdr.x >> 16);
        const unsigned ty = r.hdr.y >> g.sh, tz = r.hdr.z >> g.sh, tw = r.hdr.w >> g.sh;
        const unsigned scA = ty & 0x3f3fu, mA = tz & 0x3f3fu;
        const unsigned scB = (tw & 0x0f0fu) | ((ty >> 2) & 0x3030u);
        const unsigned mB = ((tw >> 4) & 0x0f0fu) | ((tz >> 2) & 0x3030u);
        const unsigned scp = g.hi ? scB : scA, mp = g.hi ? mB : mA;
        const int sc_lo = scp & 0xff, sc_hi = scp >> 8, m_lo = mp & 0xff, m_hi = mp >> 8;
        const unsigned v[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
        const unsigned hb[8] = {r.h0.x, r.h0.y, r.h0.z, r.h0.w, r.h1.x, r.h1.y, r.h1.z, r.h1.w};
        int lo[8], hi[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const unsigned t = hb[i] >> g.hb;
            lo[i] = (int)((v[i] & 0x0f0f0f0fu) | ((t & 0x01010101u) << 4));
            hi[i] = (int)(((v[i] >> 4) & 0x0f0f0f0fu) | (((t >> 1) & 0x01010101u) << 4));
        }
#pragma unroll
        for (int n = 0; n < NC; n++) {
            int dl = 0, dh = 0;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                dl = dot4(lo[i], a[n].lo[i], dl);
                dh = dot4(hi[i], a[n].hi[i], dh);
            }
            const int isum = __mul24(sc_lo, dl) + __mul24(sc_hi, dh);
            const int msum = __mul24(m_lo, a[n].s_lo) + __mul24(m_hi, a[n].s_hi);
            acc[n] = __builtin_fmaf(dw * a[n].d, (float)isum, acc[n]);
            acc[n] = __builtin_fmaf(-(dminw * a[n].d), (float)msum, acc[n]);
        }
    }
};

struct PolQ4_0 {
    static constexpr int PLANES = 2;  // planes of the device layout a row is read from
    static constexpr int F32_WAVES_ONE_SEG = 16;  // waves per workgroup when it quantizes one column of one-segment rows
    static constexpr int SEG = 2048;  // 64 blocks, one per lane
    static constexpr int ACT_BLK = QK, ACT_BSUM = QK;  // Q8_0: one scale and one sum per 32
    static constexpr bool USES_BSUMS = true;
    static constexpr bool HEAVY = false;
    struct Geo { int64_t qrow, drow; int blk; bool live; };
    struct Act { int q[8]; float d; int s8; };
    struct Raw { uint4 qv; unsigned dh; };

    static __device__ __forceinline__ Geo geo(const DevWeight &w, int seg, int lane) {
        Geo g;
        g.blk = seg * 64 + lane;
        g.live = (int64_t)g.blk * QK < w.K;
        if (!g.live) g.blk = 0;
        g.qrow = w.K / 2;
        g.drow = w.K / QK;
        return g;
    }
    template <class AV>
    static __device__ __forceinline__ void load_act(const AV &a, int n, int seg, int lane, const Geo &g, Act &r) {
        const int keep = g.live ? -1 : 0;
        const int4 *q = reinterpret_cast<const int4 *>(a.qs + (int64_t)n * a.K + (int64_t)g.blk * QK);
        const int4 lo = q[0], hi = q[1];
        const float dd = a.d[(int64_t)n * (a.K / QK) + g.blk];
        const int s = a.bsums[(int64_t)n * (a.K / QK) + g.blk];
        r.q[0] = lo.x & keep; r.q[1] = lo.y & keep; r.q[2] = lo.z & keep; r.q[3] = lo.w & keep;
        r.q[4] = hi.x & keep; r.q[5] = hi.y & keep; r.q[6] = hi.z & keep; r.q[7] = hi.w & keep;
        r.d = g.live ? dd : 0.f;
        r.s8 = (8 * s) & keep;
    }
    static __device__ __forceinline__ Raw load(const DevWeight &w, const Geo &g, int64_t row) {
        Raw r;
        r.qv = ld16(w.p0 + row * g.qrow + (int64_t)g.blk * 16);
        r.dh = w.d[row * g.drow + g.blk];
        return r;
    }
    template <int NC>
    static __device__ __forceinline__ void dot(const Raw &r, const Geo &, const Act (&a)[NC], float (&acc)[NC]) {
        const float dw = h2f(r.dh);
        const unsigned v[4] = {r.qv.x, r.qv.y, r.qv.z, r.qv.w};
        int lo[4], hi[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            lo[i] = (int)(v[i] & 0x0f0f0f0fu);
            hi[i] = (int)((v[i] >> 4) & 0x0f0f0f0fu);
        }
#pragma unroll
        for (int n = 0; n < NC; n++) {
            int s = -a[n].s8;  // sum (q-8)*y = sum q*y - 8*sum y
#pragma unroll
            for (int i = 0; i < 4; i++) {
                s = dot4(lo[i], a[n].q[i], s);
                s = dot4(hi[i], a[n].q[4 + i], s);
            }
            acc[n] += (float)s * dw * a[n].d;
        }
    }
};

// MXFP4 in its own 17 bytes per block (18 on the device: the layout of Q4_0, nibble plane + a 16-bit plane that holds the
// E8M0 scale byte).  A nibble is an E2M1 code: magnitude index in the low three bits, sign in the fourth; ggml multiplies
// the doubled values 0 1 2 3 4 6 8 12 as integers and scales the block sum by 2^(e - 128) d_y.  The eight magnitudes are a
// byte table in two registers (v_perm_b32 looks up four codes per instruction), the signs split every dword into the bytes
// that count positively and those that count negatively.  No scale byte is out of range here.
struct PolMXFP4 {
    static constexpr int PLANES = 2;
    static constexpr int F32_WAVES_ONE_SEG = 16;
    static constexpr int SEG = 2048;  // 64 blocks, one per lane
    static constexpr int ACT_BLK = QK, ACT_BSUM = QK;
    static constexpr bool USES_BSUMS = false;
    static constexpr bool HEAVY = false;
    struct Geo { int64_t qrow, drow; int blk; bool live; };
    struct Act { int q[8]; float d; };
    struct Raw { uint4 qv; unsigned e; };

    static __device__ __forceinline__ Geo geo(const DevWeight &w, int seg, int lane) {
        Geo g;
        g.blk = seg * 64 + lane;
        g.live = (int64_t)g.blk * QK < w.K;
        if (!g.live) g.blk = 0;
        g.qrow = w.K / 2;
        g.drow = w.K / QK;
        return g;
    }
    template <class AV>
    static __device__ __forceinline__ void load_act(const AV &a, int n, int seg, int lane, const Geo &g, Act &r) {
        const int keep = g.live ? -1 : 0;
        const int4 *q = reinterpret_cast<const int4 *>(a.qs + (int64_t)n * a.K + (int64_t)g.blk * QK);
        const int4 lo = q[0], hi = q[1];
        const float dd = a.d[(int64_t)n * (a.K / QK) + g.blk];
        r.q[0] = lo.x & keep; r.q[1] = lo.y & keep; r.q[2] = lo.z & keep; r.q[3] = lo.w & keep;
        r.q[4] = hi.x & keep; r.q[5] = hi.y & keep; r.q[6] = hi.z & keep; r.q[7] = hi.w & keep;
        r.d = g.live ? dd : 0.f;
    }
    static __device__ __forceinline__ Raw load(const DevWeight &w, const Geo &g, int64_t row) {
        Raw r;
        r.qv = ld16(w.p0 + row * g.qrow + (int64_t)g.blk * 16);
        r.e = w.d[row * g.drow + g.blk];
        return r;
    }
    // Four codes (bit 3 the sign, bits 0..2 the magnitude index; one per byte at bit `shift` of raw) as four int8 values
    // 2 * kvalue: the magnitude and its negation from two byte tables, then a byte-wise choice between them by the sign
    // (a third byte permute whose selector is 0x03020100 + 4 * sign).  Bits of raw outside the codes are masked here.
    template <int SHIFT>
    static __device__ __forceinline__ int decode4(unsigned raw) {
        const unsigned sel = (SHIFT ? raw >> SHIFT : raw) & 0x07070707u;
        const unsigned pos = __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, sel);
        const unsigned neg = __builtin_amdgcn_perm(0xF4F8FAFCu, 0xFDFEFF00u, sel);
        const unsigned sign = (raw >> (SHIFT + 3)) & 0x01010101u;
        return (int)__builtin_amdgcn_perm(neg, pos, (sign << 2) + 0x03020100u);
    }
    template <int NC>
    static __device__ __forceinline__ void dot(const Raw &r, const Geo &, const Act (&a)[NC], float (&acc)[NC]) {
        // 2^(e - 128): the exponent field e - 1, or a subnormal for the two smallest scale bytes
        const float dw = __builtin_bit_cast(float, r.e < 2 ? 0x00200000u << r.e : (r.e - 1) << 23);
        const unsigned v[4] = {r.qv.x, r.qv.y, r.qv.z, r.qv.w};
        int w8[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w8[i] = decode4<0>(v[i]);
            w8[4 + i] = decode4<4>(v[i]);
        }
#pragma unroll
        for (int n = 0; n < NC; n++) {
            int s = 0;
#pragma unroll
            for (int i = 0; i < 8; i++) s = dot4(w8[i], a[n].q[i], s);
            acc[n] += (float)s * (a[n].d * dw);
        }
    }
};

struct PolQ8_0 {
    static constexpr int PLANES = 2;  // planes of the device layout a row is read from
    static constexpr int F32_WAVES_ONE_SEG = 16;  // waves per workgroup when it quantizes one column of one-segment rows
    static constexpr int SEG = 1024;  // 32 blocks, two lanes (16 quants each) per block
    static constexpr int ACT_BLK = QK, ACT_BSUM = QK;
    static constexpr bool USES_BSUMS = false;
    static constexpr bool HEAVY = false;
    struct Geo { int64_t qrow, drow; int hb; bool live; };
    struct Act { int q[4]; float d; };
    struct Raw { uint4 qv; unsigned dh; };

    static __device__ __forceinline__ Geo geo(const DevWeight &w, int seg, int lane) {
        Geo g;
        g.hb = seg * 64 + lane;  // half-block index along the row
        g.live = (int64_t)g.hb * 16 < w.K;
        if (!g.live) g.hb = 0;
        g.qrow = w.K;
        g.drow = w.K / QK;
        return g;
    }
    template <class AV>
    static __device__ __forceinline__ void load_act(const AV &a, int n, int seg, int lane, const Geo &g, Act &r) {
        const int keep = g.live ? -1 : 0;
        const int4 v = *reinterpret_cast<const int4 *>(a.qs + (int64_t)n * a.K + (int64_t)g.hb * 16);
        const float dd = a.d[(int64_t)n * (a.K / QK) + (g.hb >> 1)];
        r.q[0] = v.x & keep; r.q[1] = v.y & keep; r.q[2] = v.z & keep; r.q[3] = v.w & keep;
        r.d = g.live ? dd : 0.f;
    }
    static __device__ __forceinline__ Raw load(const DevWeight &w, const Geo &g, int64_t row) {
        Raw r;
        r.qv = ld16(w.p0 + row * g.qrow + (int64_t)g.hb * 16);
        r.dh = w.d[row * g.drow + (g.hb >> 1)];
        return r;
    }
    template <int NC>
    static __device__ __forceinline__ void dot(const Raw &r, const Geo &, const Act (&a)[NC], float (&acc)[NC]) {
        const float dw = h2f(r.dh);
#pragma unroll
        for (int n = 0; n < NC; n++) {
            int s = dot4((int)r.qv.x, a[n].q[0], 0);
            s = dot4((int)r.qv.y, a[n].q[1], s);
            s = dot4((int)r.qv.z, a[n].q[2], s);
            s = dot4((int)r.qv.w, a[n].q[3], s);
            acc[n] += (float)s * (dw * a[n].d);
        }
    }
};

struct PolQ6K {
    static constexpr int PLANES = 4;  // planes of the device layout a row is read from
    static constexpr int F32_WAVES_ONE_SEG = 8;  // waves per workgroup when it quantizes one column of one-segment rows
    static constexpr int SEG = 4096;  // 16 super-blocks, 4 lanes each
    static constexpr int ACT_BLK = QKK, ACT_BSUM = 16;  // Q8_K: one scale per 256, one sum per 16
    static constexpr bool USES_BSUMS = true;
    static constexpr bool HEAVY = true;
    // lane (h = l4>>1, t = l4&1) of a super-block owns, in half h (128 elements):
    //   ql bytes [64h+16t, +16) and [64h+32+16t, +16), qh bytes [32h+16t, +16)
    // which hold four runs of 16 elements e = 128h + 16t + 32r + i (r = 0..3):
    //   r=0: low nibbles of the first ql piece,  high bits qh>>0
    //   r=1: low nibbles of the second ql piece, high bits qh>>2
    //   r=2: high nibbles of the first piece,    high bits qh>>4
    //   r=3: high nibbles of the second piece,   high bits qh>>6
    // each run is one 16-element scale group: scales[8h + t + 2r].
    struct Geo { int64_t lrow, hrow, srow, drow; int sb, loff, hoff, soff, e0, sh; bool live; };
    struct Act { int q[4][4]; float d; int s32[4]; };
    struct Raw { uint4 l0, l1, qh; uint2 sc8; unsigned dh; };

    static __device__ __forceinline__ Geo geo(const DevWeight &w, int seg, int lane) {
        Geo g;
        const int l4 = lane & 3, h = l4 >> 1, t = l4 & 1;
        g.sb = seg * 16 + (lane >> 2);
        g.live = (int64_t)g.sb * QKK < w.K;
        if (!g.live) g.sb = 0;
        g.lrow = w.K / 2; g.hrow = w.K / 4; g.srow = w.K / 16; g.drow = w.K / QKK;
        g.loff = g.sb * 128 + 64 * h + 16 * t;
        g.hoff = g.sb * 64 + 32 * h + 16 * t;
        g.soff = g.sb * 16 + 8 * h;  // the half's 8 scale bytes; the lane uses bytes t, t+2, t+4, t+6
        g.sh = 8 * t;
        g.e0 = 128 * h + 16 * t;
        return g;
    }
    template <class AV>
    static __device__ __forceinline__ void load_act(const AV &a, int n, int seg, int lane, const Geo &g, Act &r) {
        const int keep = g.live ? -1 : 0;
        const int8_t *q = a.qs + (int64_t)n * a.K + (int64_t)g.sb * QKK + g.e0;
        const int16_t *bs = a.bsums + (int64_t)n * (a.K / 16) + (int64_t)g.sb * 16 + (g.e0 >> 4);
        int4 v[4];
        int b[4];
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            v[rr] = *reinterpret_cast<const int4 *>(q + 32 * rr);
            b[rr] = bs[2 * rr];
        }
        const float dd = a.d[(int64_t)n * (a.K / QKK) + g.sb];
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            r.q[rr][0] = v[rr].x & keep; r.q[rr][1] = v[rr].y & keep;
            r.q[rr][2] = v[rr].z & keep; r.q[rr][3] = v[rr].w & keep;
            r.s32[rr] = (32 * b[rr]) & keep;
        }
        r.d = g.live ? dd : 0.f;
    }
    static __device__ __forceinline__ Raw load(const DevWeight &w, const Geo &g, int64_t row) {
        Raw r;
        const uint8_t *pl = w.p0 + row * g.lrow + g.loff;
        r.l0 = ld16(pl);
        r.l1 = ld16(pl + 32);
        r.qh = ld16(w.p1 + row * g.hrow + g.hoff);
        r.sc8 = *reinterpret_cast<const uint2 *>(w.p2 + row * g.srow + g.soff);
        r.dh = w.d[row * g.drow + g.sb];
        return r;
    }
    template <int NC>
    static __device__ __forceinline__ void dot(const Raw &r, const Geo &g, const Act (&a)[NC], float (&acc)[NC]) {
        const float dw = h2f(r.dh);
        const int sc[4] = {(int)(int8_t)(r.sc8.x >> g.sh), (int)(int8_t)(r.sc8.x >> (g.sh + 16)),
                           (int)(int8_t)(r.sc8.y >> g.sh), (int)(int8_t)(r.sc8.y >> (g.sh + 16))};
        const unsigned l0[4] = {r.l0.x, r.l0.y, r.l0.z, r.l0.w}, l1[4] = {r.l1.x, r.l1.y, r.l1.z, r.l1.w};
        const unsigned hq[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
        int e[4][4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            e[0][i] = (int)((l0[i] & 0x0f0f0f0fu) | ((hq[i] << 4) & 0x30303030u));
            e[1][i] = (int)((l1[i] & 0x0f0f0f0fu) | ((hq[i] << 2) & 0x30303030u));
            e[2][i] = (int)(((l0[i] >> 4) & 0x0f0f0f0fu) | (hq[i] & 0x30303030u));
            e[3][i] = (int)(((l1[i] >> 4) & 0x0f0f0f0fu) | ((hq[i] >> 2) & 0x30303030u));
        }
#pragma unroll
        for (int n = 0; n < NC; n++) {
            int isum = 0;
#pragma unroll
            for (int rr = 0; rr < 4; rr++) {
                int s = -a[n].s32[rr];  // sum (q-32)*y = sum q*y - 32*sum y
#pragma unroll
                for (int i = 0; i < 4; i++) s = dot4(e[rr][i], a[n].q[rr][i], s);
                isum += __mul24(sc[rr], s);
            }
            acc[n] = __builtin_fmaf(dw * a[n].d, (float)isum, acc[n]);
        }
    }
};

// ---------------------------------------------------------------------------------------------
// The kernel.  Workgroup = KW x RW waves: wave (kseg, rg) owns K segments kseg, kseg+KW, ...
// (SPW of them, held in registers) and rows r0+rg, r0+rg+RW, r0+rg+2RW, ... of the workgroup's row
// range.  With KW == 1 a wave's totals are final and go straight to y; otherwise part[] (LDS)
// receives one partial per (row, column, kseg) and after a barrier the workgroup sums over kseg.
// ---------------------------------------------------------------------------------------------
template <class P, int SPW, int U>
__device__ __forceinline__ void load_pass(const DevWeight &w, const typename P::Geo (&g)[SPW],
                                          typename P::Raw (&raw)[U][SPW], int64_t rbase, int rw, int i0,
                                          int nrw) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int i = min(i0 + u, nrw - 1);  // past the wave's last row: re-read it (dropped later)
#pragma unroll
        for (int s = 0; s < SPW; s++) raw[u][s] = P::load(w, g[s], rbase + (int64_t)i * rw);
    }
}

template <class P, int NC, int SPW, int U, bool DIRECT>
__device__ __forceinline__ void compute_pass(const typename P::Geo (&g)[SPW],
                                             const typename P::Act (&act)[SPW][NC],
                                             const typename P::Raw (&raw)[U][SPW], int rl0, int rw, int i0,
                                             int nrw, int lane, int kseg, int kw, float *part, float *yrow0,
                                             int64_t ldy) {
    float acc[NC][U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        float a1[NC];
#pragma unroll
        for (int n = 0; n < NC; n++) a1[n] = 0.f;
#pragma unroll
        for (int s = 0; s < SPW; s++) P::template dot<NC>(raw[u][s], g[s], act[s], a1);
#pragma unroll
        for (int n = 0; n < NC; n++) acc[n][u] = a1[n];
    }
    const int u = lane & (U - 1);  // the row of the pass this lane ends up holding
    const bool writer = lane < U && i0 + u < nrw;
    const int rl = rl0 + (i0 + u) * rw;  // row index inside the workgroup's range
#pragma unroll
    for (int n = 0; n < NC; n++) {
        const float tot = reduce_rows<U>(acc[n], lane);
        if (writer) {
            if (DIRECT) yrow0[(int64_t)n * ldy + rl] = tot;
            else part[(rl * NC + n) * kw + kseg] = tot;
        }
    }
}

// Up to MAX_MULTI weight tensors that share K, type and the activations (gate and up, or q/k/v) go
// through one launch: the grid is the concatenation of the tensors' workgroup ranges.
struct MultiArgs {
    DevWeight w[MAX_MULTI];
    float *y[MAX_MULTI];
    int64_t ldy[MAX_MULTI];
    int wg_end[MAX_MULTI];  // exclusive prefix end of each tensor's workgroup range
    int count;
};

template <class P, int NC, int SPW, int U, bool DIRECT>
__global__ __launch_bounds__(512, 2) void gemv_kernel(MultiArgs ma, DevAct a, int col0, int rows_per_wg, int kw,
                                                   int rw_log2) {
    extern __shared__ float part[];  // [rows_per_wg][NC][kw], unused when DIRECT
    int t = 0, wg = blockIdx.x;
#pragma unroll
    for (int i = 0; i < MAX_MULTI - 1; i++)
        if (i + 1 < ma.count && (int)blockIdx.x >= ma.wg_end[i]) { t = i + 1; wg = blockIdx.x - ma.wg_end[i]; }
    const DevWeight &w = ma.w[t];
    float *__restrict__ y = ma.y[t];
    const int64_t ldy = ma.ldy[t];
    // the wave index is uniform across the wave: keep it (and all row arithmetic that follows from it)
    // in scalar registers
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rw = 1 << rw_log2;
    const int rg = wave & (rw - 1), kseg = wave >> rw_log2;  // rw is a power of two: no divisions here
    const int64_t r0 = (int64_t)wg * rows_per_wg;
    const int64_t r1 = min(w.M, r0 + (int64_t)rows_per_wg);
    const int nrows = (int)(r1 - r0);
    const int nrw = (nrows - rg + rw - 1) >> rw_log2;  // rows of this wave: r0 + rg + i*rw, i < nrw
    float *yrow0 = y + (int64_t)col0 * ldy + r0;

    if (nrw > 0) {
        // The first pass of weight loads goes out before anything else: every instruction ahead of it
        // delays the moment the wave starts pulling on HBM.  The activation loads follow, then the
        // second pass; the memory counter retires in order, so the first compute pass waits for
        // weights(A) + activations only, while weights(B) stay in flight.
        typename P::Geo g[SPW];
#pragma unroll
        for (int s = 0; s < SPW; s++) g[s] = P::geo(w, kseg + s * kw, lane);
        typename P::Raw bufA[U][SPW], bufB[U][SPW];
        const int64_t rbase = r0 + rg;
        load_pass<P, SPW, U>(w, g, bufA, rbase, rw, 0, nrw);
        typename P::Act act[SPW][NC];
#pragma unroll
        for (int s = 0; s < SPW; s++)
#pragma unroll
            for (int n = 0; n < NC; n++) P::load_act(a, col0 + n, kseg + s * kw, lane, g[s], act[s][n]);
        load_pass<P, SPW, U>(w, g, bufB, rbase, rw, U, nrw);  // clamped to the last row if nrw <= U
        // Steady state: no branches around the loads, so the compiler can make each compute pass wait
        // for exactly its own loads while the next pass stays in flight.  The loop runs as long as rows
        // remain beyond the two loaded passes; loads that reach past the wave's last row re-read that
        // row (at most 2U-1 redundant row loads per wave, served by the caches).
        int i0 = 0;
        for (; i0 + 2 * U < nrw; i0 += 2 * U) {
            compute_pass<P, NC, SPW, U, DIRECT>(g, act, bufA, rg, rw, i0, nrw, lane, kseg, kw, part, yrow0, ldy);
            load_pass<P, SPW, U>(w, g, bufA, rbase, rw, i0 + 2 * U, nrw);
            compute_pass<P, NC, SPW, U, DIRECT>(g, act, bufB, rg, rw, i0 + U, nrw, lane, kseg, kw, part, yrow0, ldy);
            load_pass<P, SPW, U>(w, g, bufB, rbase, rw, i0 + 3 * U, nrw);
        }
        compute_pass<P, NC, SPW, U, DIRECT>(g, act, bufA, rg, rw, i0, nrw, lane, kseg, kw, part, yrow0, ldy);
        if (i0 + U < nrw)
            compute_pass<P, NC, SPW, U, DIRECT>(g, act, bufB, rg, rw, i0 + U, nrw, lane, kseg, kw, part, yrow0, ldy);
    }
    if (DIRECT) return;

    __syncthreads();
    for (int i = threadIdx.x; i < nrows * NC; i += blockDim.x) {
        const int n = i / nrows, rl = i - n * nrows;  // consecutive threads -> consecutive rows
        float s = 0.f;
        for (int k = 0; k < kw; k++) s += part[(rl * NC + n) * kw + k];
        yrow0[(int64_t)n * ldy + rl] = s;
    }
}

// Sum over the 64 lanes; the total is valid in lanes 48..63.  Cross-lane moves only (quad swaps,
// rotations inside rows of 16, then the row broadcasts), no LDS round trip.
template <int CTRL, int ROWS>
__device__ __forceinline__ float dpp_row(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROWS, 0xf, false));
}
__device__ __forceinline__ float wave_total(float w) {
    w += dpp_mov<0xB1>(w);
    w += dpp_mov<0x4E>(w);
    w += dpp_mov<0x124>(w);
    w += dpp_mov<0x128>(w);
    w += dpp_row<0x142, 0xa>(w);  // row_bcast:15 -- lane 15 of rows 0 and 2 into rows 1 and 3
    w += dpp_row<0x143, 0xc>(w);  // row_bcast:31 -- lane 31 into rows 2 and 3
    return w;
}

// Sums over runs of 64/RPL lanes (RPL = 1, 2, 4 rows side by side in a wave); a run's total is
// taken from its last lane.  RPL = 1 is wave_total.
template <int RPL>
__device__ __forceinline__ float run_total(float w) {
    w += dpp_mov<0xB1>(w);
    w += dpp_mov<0x4E>(w);
    w += dpp_mov<0x124>(w);
    w += dpp_mov<0x128>(w);
    if (RPL <= 2) w += dpp_row<0x142, 0xa>(w);
    if (RPL == 1) w += dpp_row<0x143, 0xc>(w);
    return w;
}

// How many rows a wave takes side by side: a row shorter than half (a quarter) of a wave's K segment
// leaves half (three quarters) of the lanes without work, so the lanes are split into 2 (4) runs that
// each hold a row of their own.  Only for rows inside one segment.
template <class P>
constexpr int rows_per_load(int64_t K) { return K * 4 <= P::SEG ? 4 : K * 2 <= P::SEG ? 2 : 1; }

// The row loop of the thin kernels: rows wrow0 .. wrow0+nrw-1 of w against the activation registers,
// one load of RPL rows in registers and the next in flight.  cur holds the first load (issued by the
// caller ahead of its prologue: rows wrow0 + min(run, nrw-1)).  DIRECT: on return lane 63-i of keep[n]
// holds the total of the wave's row i; otherwise the totals go to part[(rl0+i)*NC + n][kseg] (rows side by side there:
// the waves of a mostly empty last K segment).
template <class P, int NC, bool DIRECT, int RPL>
__device__ __forceinline__ void thin_rows(const DevWeight &w, const typename P::Geo &g, typename P::Raw cur,
                                          const typename P::Act (&act)[NC], int64_t wrow0, int nrw, int lane,
                                          float (&keep)[NC], float *part, int rl0, int kw, int kseg) {
    const int run = RPL == 1 ? 0 : lane / (64 / RPL);
#pragma unroll
    for (int n = 0; n < NC; n++) keep[n] = 0.f;
#pragma unroll 1
    for (int i = 0; i < nrw; i += RPL) {
        float acc[NC];
#pragma unroll
        for (int n = 0; n < NC; n++) acc[n] = 0.f;
        P::template dot<NC>(cur, g, act, acc);
        if (i + RPL < nrw) cur = P::load(w, g, wrow0 + min(i + RPL + run, nrw - 1));  // wave-uniform branch
#pragma unroll
        for (int n = 0; n < NC; n++) {
            // Every lane of a run's last quad row holds the total, but each quad added the quads of its
            // row in its own order: take the run's last lane, so a row's result does not depend on which
            // lane parks it (i.e. not on how many rows a wave was given).
            const int tot_all = __float_as_int(run_total<RPL>(acc[n]));
#pragma unroll
            for (int r = 0; r < RPL; r++) {
                const float tot = __int_as_float(__builtin_amdgcn_readlane(tot_all, 64 / RPL * (r + 1) - 1));
                if (DIRECT) keep[n] = lane == 63 - (i + r) ? tot : keep[n];
                else if (lane == 63 && i + r < nrw) part[((rl0 + i + r) * NC + n) * kw + kseg] = tot;
            }
        }
    }
}

// The row loop for a wave whose second row was requested while the workgroup was still quantizing (next = row
// wrow0 + min(1, nrw-1)): otherwise thin_rows for one column and one row per load.
template <class P, bool DIRECT>
__device__ __forceinline__ void thin_rows_ahead(const DevWeight &w, const typename P::Geo &g, typename P::Raw cur, typename P::Raw next,
                                                const typename P::Act (&act)[1], int64_t wrow0, int nrw, int lane, float (&keep)[1],
                                                float *part, int rl0, int kw, int kseg) {
    keep[0] = 0.f;
#pragma unroll 1
    for (int i = 0; i < nrw; i++) {
        float acc[1] = {0.f};
        P::template dot<1>(cur, g, act, acc);
        cur = next;
        if (i + 2 < nrw) next = P::load(w, g, wrow0 + i + 2);  // wave-uniform
        const float tot = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(run_total<1>(acc[0])), 63));
        if (DIRECT) keep[0] = lane == 63 - i ? tot : keep[0];
        else if (lane == 63) part[(rl0 + i) * kw + kseg] = tot;
    }
}

// The row loop with two loads in flight and nothing in the way of the compiler's count of them: the loads alternate
// between two named sets of registers (no copy from "next" to "current", which would have to wait for the next row before
// the current one is multiplied), every load inside the loop is unconditional (the last iteration is peeled off instead;
// a wave with an odd number of loads re-reads its last rows once), so each multiply waits for its own row only.
// a, b: the first two loads (rows wrow0 + min(run, nrw-1) and wrow0 + min(RPL + run, nrw-1)), requested by the caller.
// Totals go to part[(rl0+i)][kseg] (one column).  For rows cut into K segments; for rows of one segment (two workgroups
// per CU, every wave asking at once) a second load in flight measured slower: gate + up 13.1-13.4 against 12.9 us.
template <class P, int RPL>
__device__ __forceinline__ void thin_rows_two(const DevWeight &w, const typename P::Geo &g, typename P::Raw a, typename P::Raw b,
                                              const typename P::Act (&act)[1], int64_t wrow0, int nrw, int lane, float *part, int rl0,
                                              int kw, int kseg) {
    const int run = RPL == 1 ? 0 : lane / (64 / RPL);
    auto finish = [&](const typename P::Raw &raw, int i) __attribute__((always_inline)) {
        float acc[1] = {0.f};
        P::template dot<1>(raw, g, act, acc);
        const int tot_all = __float_as_int(run_total<RPL>(acc[0]));
#pragma unroll
        for (int r = 0; r < RPL; r++) {
            const float tot = __int_as_float(__builtin_amdgcn_readlane(tot_all, 64 / RPL * (r + 1) - 1));
            if (lane == 63 && i + r < nrw) part[(rl0 + i + r) * kw + kseg] = tot;
        }
    };
    int i = 0;
#pragma unroll 1
    for (; i + 2 * RPL < nrw; i += 2 * RPL) {
        finish(a, i);
        a = P::load(w, g, wrow0 + min(i + 2 * RPL + run, nrw - 1));
        finish(b, i + RPL);
        b = P::load(w, g, wrow0 + min(i + 3 * RPL + run, nrw - 1));
    }
    finish(a, i);
    if (i + RPL < nrw) finish(b, i + RPL);  // wave-uniform
}

// ---------------------------------------------------------------------------------------------
// The thin-wave kernel: many small waves instead of a few unrolled ones.
//
// A dispatch starts with a cold instruction cache, and straight-line code is fetched at roughly
// 0.2 us per KiB -- an unrolled, double-buffered 8 KiB kernel spends a fifth of a 33 MB launch
// fetching itself.  Here a wave runs a rolled loop over a handful of rows (one row of weights in
// registers, the next one in flight), the body is about 1 KiB, and the memory-level parallelism
// comes from occupancy: 6-8 waves per SIMD, each with a row in flight.
// ---------------------------------------------------------------------------------------------
// The activations as the kernel sees them once staged in LDS: same layout as DevAct, columns
// col0 .. col0+NC-1 only.
struct LdsAct {
    const int8_t *qs;
    const float *d;
    const int16_t *bsums;
    int64_t K;
};

// The f32 prologue shared by the kernels that quantize their own activations: a wave takes 256
// consecutive elements ("pieces" of 64 float4) at a time, the same lane-to-element mapping as the
// stand-alone quantization kernel, so the values are the same bits.  The first XPRE pieces of a wave
// are requested by prefetch_x (before the wave's first weight load), the rest inside quantize_x_to_lds.
constexpr int XPRE = 4;

template <int XP>
__device__ __forceinline__ void prefetch_x(const float4 *__restrict__ x4, int total4, int wave, int nwaves, int lane,
                                           float4 (&xpre)[XP]) {
#pragma unroll
    for (int j = 0; j < XP; j++) {
        const int i4 = (wave + j * nwaves) * 64 + lane;
        xpre[j] = x4[min(i4, total4 - 1)];  // clamped: the loads stay unconditional
    }
}

template <class P, int XP>
__device__ __forceinline__ void quantize_x_to_lds(const float4 *__restrict__ x4, int total4, int wave, int nwaves,
                                                  int lane, const float4 (&xpre)[XP], int8_t *lqs, float *ld_,
                                                  int16_t *lbs) {
    auto quantize_piece = [&](int c, float4 v) {
        const int i4 = c * 64 + lane;
        const bool live = i4 < total4;  // Q8_0 only: the element count need not be a multiple of 256
        if (!live) v = make_float4(0.f, 0.f, 0.f, 0.f);
        float dd;
        if (P::ACT_BLK == QKK) {
            int sum16, pair;
            const int packed = q8_K_quantize_lane(v, lane, dd, sum16, pair);
            reinterpret_cast<int *>(lqs)[i4] = packed;
            if (lane == 0) ld_[c] = dd;
            if (P::USES_BSUMS && (lane & 3) == 0) lbs[c * 16 + (lane >> 2)] = (int16_t)sum16;
        } else {
            int sum;
            const int packed = q8_0_quantize_lane(v, dd, sum);
            if (live) {
                reinterpret_cast<int *>(lqs)[i4] = packed;
                if ((lane & 7) == 0) {
                    ld_[i4 >> 3] = dd;
                    if (P::USES_BSUMS) lbs[i4 >> 3] = (int16_t)sum;
                }
            }
        }
    };
#pragma unroll
    for (int j = 0; j < XP; j++) {
        const int c = wave + j * nwaves;
        if (c * 64 < total4) quantize_piece(c, xpre[j]);  // wave-uniform
    }
    // (XP == 1 is launched only where a piece per wave covers all of x: no further pieces, and no loop with loads in
    // it for the compiler to lose its count of the outstanding ones over)
    if constexpr (XP > 1)
        for (int c = wave + XP * nwaves; c * 64 < total4; c += nwaves)
            quantize_piece(c, x4[min(c * 64 + lane, total4 - 1)]);
}

// The same for Q8_K activations with a quarter of a wave per block (q8_K_quantize_row16: lane l of a 16-lane row holds
// elements 16l.. of its block, a wave quantizes four consecutive blocks at a time): fewer cross-lane steps per block,
// and the plain decode prologue is made of little else.  Same bits.  A wave's first four blocks are requested by
// prefetch_x16 ahead of its first weight load.
__device__ __forceinline__ void prefetch_x16(const float4 *__restrict__ x4, int nblk_all, int wave, int lane, float4 (&xq)[4]) {
    const int b = min(4 * wave + (lane >> 4), nblk_all - 1);  // clamped: the loads stay unconditional
#pragma unroll
    for (int j = 0; j < 4; j++) xq[j] = x4[b * 64 + 4 * (lane & 15) + j];
}
template <class P>
__device__ __forceinline__ void quantize_x_to_lds16(const float4 *__restrict__ x4, int nblk_all, int wave, int nwaves, int lane,
                                                    const float4 (&xq)[4], int8_t *lqs, float *ld_, int16_t *lbs) {
    auto quantize_four = [&](int b0, const float4 (&v)[4]) {
        const int b = b0 + (lane >> 4), sub = lane & 15;
        float dd;
        int sum16, pair;
        const uint4 packed = q8_K_quantize_row16(v, lane, dd, sum16, pair);
        if (b < nblk_all) {  // the last four may end early: whole rows of 16 lanes drop out
            *reinterpret_cast<uint4 *>(lqs + (size_t)b * QKK + 16 * sub) = packed;
            if (sub == 0) ld_[b] = dd;
            if (P::USES_BSUMS) lbs[b * 16 + sub] = (int16_t)sum16;
        }
    };
    if (4 * wave < nblk_all) quantize_four(4 * wave, xq);  // wave-uniform
    for (int b0 = 4 * (wave + nwaves); b0 < nblk_all; b0 += 4 * nwaves) {
        float4 v[4];
        const int b = min(b0 + (lane >> 4), nblk_all - 1);
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = x4[b * 64 + 4 * (lane & 15) + j];
        quantize_four(b0, v);
    }
}

// Global-address-space pointer types: what a kernel's pointer arguments are cast to before an empty asm pins
// them in scalar registers (see gemv_thin_kernel), so that they come out of it still known to be global.
typedef const __attribute__((address_space(1))) uint8_t *gbytes_t;
typedef __attribute__((address_space(1))) float *gfloats_t;
typedef const __attribute__((address_space(1))) float *gcfloats_t;
typedef const __attribute__((address_space(1))) int *gcints_t;

// Kernel arguments of the thin kernel, arranged so that the tensor a workgroup belongs to is picked
// with compares and selects on values that are all fetched by one batch of scalar loads: a select
// chain that indexes the argument block with a computed index makes each pointer load wait for the
// previous one, a microsecond of latency before the first HBM request.
struct ThinArgs {
    const uint8_t *p0[MAX_MULTI], *p1[MAX_MULTI], *p2[MAX_MULTI];
    const uint16_t *d[MAX_MULTI];
    float *y[MAX_MULTI];
    int64_t M[MAX_MULTI];
    int wg_end[MAX_MULTI];  // exclusive end of each tensor's workgroup range; INT_MAX past the last tensor
    int64_t K;
    int type;
};

// workgroup size limit: 16 waves leave a wave 128 VGPRs, enough for up to three activation columns
constexpr int thin_max_waves(int nc, bool f32) { return f32 ? (nc <= 3 ? 16 : 8) : 4; }

// XMODE: where the activations come from -- 0: quantized planes (a); 1: f32 x, quantized here; 2 / 3: f32 x
// that first goes through RMSNorm / SwiGLU (pr; one column, all of x in the waves' XP prefetch registers: XP is
// 1 when a piece per wave covers the row, which keeps the kernel at two workgroups per CU).
// AHEAD (one f32 column, long rows, one workgroup per CU anyway): a wave requests its second row as soon as it has
// quantized its share of x -- not before, where the request would queue in front of other waves' x -- so that two
// rows per wave stream while the workgroup waits at the barrier and reads its activations back.
// TAILR (2 or 4; rows cut into segments, one or two columns): the waves of the last K segment, which is at most half
// (a quarter) full, take TAILR rows side by side per load -- as RPL does for short rows -- instead of running with
// most of their lanes dead.  Same bits: a dead lane adds an exact zero to its row's sum.
template <class P, int NC, bool DIRECT, int XMODE, int RPL, int XP = XPRE, bool AHEAD = false, int TAILR = 1>
__global__ __launch_bounds__(XMODE && NC <= 3 ? 1024 : 512) void gemv_thin_kernel(ThinArgs ta, DevAct a, const float *__restrict__ xf,
                                                         int col0, int rows_per_wave, int kw, int rw_log2, Produce pr) {
    constexpr bool F32 = XMODE != 0;
    // LDS: the NC activation columns (quants, block scales, block sums), then, unless DIRECT, the
    // partial sums [rows_per_wg][NC][kw].
    extern __shared__ __align__(16) uint8_t smem[];
    const int bid = blockIdx.x;
    // Everything the prologue needs from the argument block is named here and pinned by an empty asm, so
    // that the scalar loads go out as one batch at the top: left alone the compiler turns the selects
    // below into branches and fetches each side's pointers only after the branch, three dependent rounds
    // of scalar loads before the first vector load.
    // (The pointers go through the asm as global-address-space pointers: as plain ones they would come out
    // with their address space unknown and every load through them would become a flat load.)
    typedef const __attribute__((address_space(1))) uint16_t *ghalves_t;
    typedef const __attribute__((address_space(1))) int8_t *gi8_t;
    typedef const __attribute__((address_space(1))) int16_t *gi16_t;
    typedef int ints4_t __attribute__((ext_vector_type(4)));
    typedef long longs2_t __attribute__((ext_vector_type(2)));
    gbytes_t p0a = (gbytes_t)ta.p0[0], p0b = (gbytes_t)ta.p0[1], p0c = (gbytes_t)ta.p0[2], p0d = (gbytes_t)ta.p0[3];
    gbytes_t p1a = (gbytes_t)ta.p1[0], p1b = (gbytes_t)ta.p1[1], p1c = (gbytes_t)ta.p1[2], p1d = (gbytes_t)ta.p1[3];
    gbytes_t p2a = (gbytes_t)ta.p2[0], p2b = (gbytes_t)ta.p2[1], p2c = (gbytes_t)ta.p2[2], p2d = (gbytes_t)ta.p2[3];
    ghalves_t da = (ghalves_t)ta.d[0], db = (ghalves_t)ta.d[1], dc = (ghalves_t)ta.d[2], dd = (ghalves_t)ta.d[3];
    gfloats_t ya = (gfloats_t)ta.y[0], yb = (gfloats_t)ta.y[1], yc = (gfloats_t)ta.y[2], yd = (gfloats_t)ta.y[3];
    gcfloats_t xg = (gcfloats_t)xf;
    gi8_t aq = (gi8_t)a.qs;
    gcfloats_t ad = (gcfloats_t)a.d;
    gi16_t ab = (gi16_t)a.bsums;
    ints4_t ends = {ta.wg_end[0], ta.wg_end[1], ta.wg_end[2], ta.wg_end[3]};
    ints4_t dims = {col0, rows_per_wave, kw, rw_log2};
    longs2_t Mab = {(long)ta.M[0], (long)ta.M[1]}, Mcd = {(long)ta.M[2], (long)ta.M[3]}, Ks = {(long)ta.K, (long)a.K};
    if (F32 && P::PLANES > 1) {
        // (f32 x with a format of several planes: the first loads are the wave's pieces of x, which need only
        // the first few arguments, and the rest arrives while those are in flight -- pinning all 29 values up
        // front measured 3..5 % slower for Q4_0 / Q8_0.  Q4_K, one plane and 17 values, gains about 1 %.)
    } else if (P::PLANES > 1)
        asm volatile("" : "+s"(p0a), "+s"(p0b), "+s"(p0c), "+s"(p0d), "+s"(p1a), "+s"(p1b), "+s"(p1c), "+s"(p1d), "+s"(p2a), "+s"(p2b),
                          "+s"(p2c), "+s"(p2d), "+s"(da), "+s"(db), "+s"(dc), "+s"(dd), "+s"(ya), "+s"(yb), "+s"(yc), "+s"(yd),
                          "+s"(xg), "+s"(aq), "+s"(ad), "+s"(ab), "+s"(ends), "+s"(dims), "+s"(Mab), "+s"(Mcd), "+s"(Ks));
    else
        asm volatile("" : "+s"(p0a), "+s"(p0b), "+s"(p0c), "+s"(p0d), "+s"(ya), "+s"(yb), "+s"(yc), "+s"(yd), "+s"(xg), "+s"(aq),
                          "+s"(ad), "+s"(ab), "+s"(ends), "+s"(dims), "+s"(Mab), "+s"(Mcd), "+s"(Ks));
    xf = (const float *)xg;
    a.qs = (const int8_t *)aq;
    a.d = (const float *)ad;
    a.bsums = (const int16_t *)ab;
    a.K = Ks[1];
    col0 = dims[0]; rows_per_wave = dims[1]; kw = dims[2]; rw_log2 = dims[3];
    const int e0 = ends[0], e1 = ends[1], e2 = ends[2];
    const int64_t Ma = Mab[0], Mb = Mab[1], Mc = Mcd[0], Md = Mcd[1], Kall = Ks[0];
    const int t = (bid >= e0) + (bid >= e1) + (bid >= e2);
    const int wg = bid - (t == 0 ? 0 : t == 1 ? e0 : t == 2 ? e1 : e2);
#define THIN_SEL4(a, b, c, d) (t == 0 ? a : t == 1 ? b : t == 2 ? c : d)
    const DevWeight w{(const uint8_t *)THIN_SEL4(p0a, p0b, p0c, p0d), (const uint8_t *)THIN_SEL4(p1a, p1b, p1c, p1d),
                      (const uint8_t *)THIN_SEL4(p2a, p2b, p2c, p2d), (const uint16_t *)THIN_SEL4(da, db, dc, dd), Kall,
                      THIN_SEL4(Ma, Mb, Mc, Md), ta.type};
    float *__restrict__ y = (float *)THIN_SEL4(ya, yb, yc, yd);
#undef THIN_SEL4
    const int64_t ldy = w.M;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rw = 1 << rw_log2;
    const int rg = wave & (rw - 1), kseg = wave >> rw_log2;
    // rows_per_wave: the low half is the rows of every wave, the high half how many of the workgroup's first row groups
    // take one more (a workgroup's rows need not divide by its row groups: 28672 rows are 512 workgroups of 56)
    const int rpw_base = rows_per_wave & 0xffff, rpw_extra = rows_per_wave >> 16;
    const int rows_per_wg = (rpw_base << rw_log2) + rpw_extra;
    const int64_t r0 = (int64_t)wg * rows_per_wg;
    const int nrows = (int)min((int64_t)rows_per_wg, w.M - r0);
    const int rl0 = rg * rpw_base + min(rg, rpw_extra);    // the wave's rows: r0 + rl0 + i, i < nrw
    const int nrw = max(0, min(rpw_base + (rg < rpw_extra ? 1 : 0), nrows - rl0));
    float *yrow0 = y + (int64_t)col0 * ldy + r0;

    // rows side by side in this wave: RPL for short rows, TAILR in the waves of a mostly empty last segment
    static_assert(TAILR == 1 || (!DIRECT && RPL == 1 && NC <= 2 && XMODE <= 1), "side-by-side tail rows: plain products of rows cut into segments");
    const bool tail = TAILR > 1 && kseg == kw - 1;  // wave-uniform
    const int vlane = tail ? lane & (64 / TAILR - 1) : lane & (64 / RPL - 1);  // position inside the lane's run
    const int run = tail ? lane / (64 / TAILR) : RPL == 1 ? 0 : lane / (64 / RPL);
    const typename P::Geo g = P::geo(w, kseg, vlane);

    // With f32 activations the workgroup quantizes them itself, into LDS, in the layout of DevAct
    // (columns col0 .. col0+NC-1 only): a wave takes 256 consecutive elements at a time, the same
    // lane-to-element mapping as the stand-alone quantization kernel, so the values are the same bits.
    const int64_t K = ta.K;
    const int nblk = (int)(K / P::ACT_BLK);
    const int nbs = P::USES_BSUMS ? (int)(K / P::ACT_BSUM) : 0;
    const size_t act_bytes = F32 ? (((size_t)NC * (K + nblk * 4 + nbs * 2)) + 15) / 16 * 16 : 0;
    int8_t *lqs = reinterpret_cast<int8_t *>(smem);
    float *ld_ = reinterpret_cast<float *>(smem + (size_t)NC * K);
    int16_t *lbs = reinterpret_cast<int16_t *>(smem + (size_t)NC * K + (size_t)NC * nblk * 4);
    // Order of the memory requests: the wave's pieces of x (L2 hits, they come back first), then its
    // first row of weights (HBM).  The memory counter retires in order, so the quantization can start
    // as soon as x is there while the weights are still in flight.
    const float4 *x4 = reinterpret_cast<const float4 *>(xf + (int64_t)col0 * K);
    const int total4 = (int)((int64_t)NC * K / 4);  // float4 pieces over all NC columns
    const int nwaves = kw << rw_log2 /* = (kw << rw_log2) * 64 / 64, without the hidden-argument load */;
    // plain Q8_K activations with several blocks per wave (long rows): four blocks per wave at a time.  Where a block
    // per wave covers the row (XP = 1) sixteen waves quantizing one block each finish sooner than four waves
    // quantizing four (measured: the gate+up launch 13.2 against 13.4 us).
    // SwiGLU in front (XMODE 3) is elementwise and takes the same route; RMSNorm's sum of squares is tied to the
    // wave-per-block order and does not.
    constexpr bool ROW16 = (XMODE == 1 || XMODE == 3) && P::ACT_BLK == QKK && XP > 1;
    float4 xpre[XP], apre[XP], xq[4], apre16[4];
    if (ROW16) prefetch_x16(x4, NC * nblk, wave, lane, xq);
    else if (F32) prefetch_x(x4, total4, wave, nwaves, lane, xpre);
    // the producer's operand, requested unconditionally (RMSNorm without a weight reads x again and ignores
    // it) so that the number of loads in flight stays known to the waits below
    const bool has_aux = XMODE == 3 || (XMODE == 2 && pr.aux != nullptr);
    if (ROW16 && XMODE == 3) prefetch_x16(reinterpret_cast<const float4 *>(pr.aux), NC * nblk, wave, lane, apre16);
    else if (XMODE >= 2) prefetch_x(has_aux ? reinterpret_cast<const float4 *>(pr.aux) : x4, total4, wave, nwaves, lane, apre);
    static_assert(!AHEAD || (!DIRECT && RPL == 1 && NC == 1 && XMODE == 1), "a second row ahead: one plain f32 column, rows cut into K segments");
    typename P::Raw cur, nxt;
    // The first row of weights is requested whether or not the wave has rows (a wave past the matrix' last row re-reads
    // that row and drops it): behind a condition the compiler no longer knows how many loads are in flight where the two
    // paths meet, and waits for all of them -- the weights from HBM included -- before it lets the quantization touch x.
    // (The scheduling barriers keep the requests in this order -- x first: loads return in the order they were made.)
    // (Q4_0 / Q8_0 keep the request under its condition: on their short launches, 5-7 us, the order the compiler then
    // chooses measured 3 % faster.)
    if constexpr (P::ACT_BLK == QKK) {
        __builtin_amdgcn_sched_barrier(0);
        cur = P::load(w, g, min(r0 + rl0 + min(run, max(nrw, 1) - 1), w.M - 1));
        __builtin_amdgcn_sched_barrier(0);
    } else {
        if (nrw > 0) cur = P::load(w, g, r0 + rl0 + min(run, nrw - 1));
    }
    constexpr size_t PSUM_BYTES = XMODE == 2 ? XPRE * 16 * sizeof(double) : 0;  // one sum per 256-element piece
    // AHEAD kernels (one plain f32 column, rows cut into K segments): where the four waves of a K segment are also the
    // four that quantize that segment's sixteen blocks (four row groups per workgroup, segments of 4096, one round of
    // four blocks per wave), a wave waits for those three others only -- a count in LDS -- instead of for all sixteen
    // at a barrier, and the waves that share a row group hand their partial sums to whichever of them finishes last
    // instead of meeting at a second barrier.  The counters are cleared here, behind a barrier that costs nothing: every
    // wave has its requests out and nothing to do until x arrives.
    const int part_floats = rows_per_wg * NC * kw;
    int *seg_cnt = reinterpret_cast<int *>(smem + act_bytes + PSUM_BYTES) + part_floats;  // [8] segments, [8] row groups
    const bool seg_sync = AHEAD && ROW16 && rw_log2 == 2 && P::SEG == 4096 && NC * nblk <= 4 * nwaves && kw <= 8;
    if (AHEAD && seg_sync) {
        if (threadIdx.x < 16) seg_cnt[threadIdx.x] = 0;
        __syncthreads();
    }
    if (XMODE == 2) {
        // RMSNorm: piece sums of squares through LDS, added in piece order by every thread
        double *psum = reinterpret_cast<double *>(smem + act_bytes);
#pragma unroll
        for (int j = 0; j < XP; j++) {
            const int c = wave + j * nwaves;
            if (c * 64 < total4) {  // wave-uniform
                const double sq = piece_sumsq(c * 64 + lane < total4 ? xpre[j] : make_float4(0.f, 0.f, 0.f, 0.f));
                if (lane == 0) psum[c] = sq;
            }
        }
        __syncthreads();
        double tot = 0.0;
        for (int c = 0; c * 64 < total4; c++) tot += psum[c];
        const float scale = rms_scale_of(tot, K, pr.eps);
#pragma unroll
        for (int j = 0; j < XP; j++) xpre[j] = rms_apply(xpre[j], scale, apre[j], has_aux);
    }
    if (XMODE == 3 && ROW16) {  // (the plan keeps such rows within one group of four blocks per wave)
#pragma unroll
        for (int j = 0; j < 4; j++) xq[j] = swiglu_apply(xq[j], apre16[j]);
    } else if (XMODE == 3) {
#pragma unroll
        for (int j = 0; j < XP; j++) xpre[j] = swiglu_apply(xpre[j], apre[j]);
    }
    if (F32) {
        if (ROW16) quantize_x_to_lds16<P>(x4, NC * nblk, wave, nwaves, lane, xq, lqs, ld_, lbs);
        else quantize_x_to_lds<P, XP>(x4, total4, wave, nwaves, lane, xpre, lqs, ld_, lbs);
        if constexpr (AHEAD && ROW16) {  // the wave's second load: unconditional, like the first
            const int step = tail ? TAILR : 1;
            nxt = P::load(w, g, min(r0 + rl0 + min(step + run, max(nrw, 1) - 1), w.M - 1));
            __builtin_amdgcn_sched_barrier(0);
        } else if constexpr (AHEAD) {
            // (Q4_0 / Q8_0: short launches on which the two-load loop below measured 4-6 % slower; they keep the second
            // row under its condition and the loop that copies it down)
            if (nrw > 0 && !tail) nxt = P::load(w, g, r0 + rl0 + min(1, nrw - 1));
        }
        if (AHEAD && seg_sync) {
            // this wave's blocks are in LDS (it waits for its own writes), then it counts itself in and waits for the
            // other quantizing waves of its segment: blocks 16 kseg .. of the row come from waves 4 kseg ..
            const int quantizers = min(4, (nblk - 16 * kseg + 3) / 4);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (lane == 0 && 4 * wave < nblk) __hip_atomic_fetch_add(&seg_cnt[kseg], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            while (__hip_atomic_load(&seg_cnt[kseg], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < quantizers) __builtin_amdgcn_s_sleep(1);
            asm volatile("" ::: "memory");
        } else {
            __syncthreads();
        }
    }
    float *part = reinterpret_cast<float *>(smem + act_bytes + PSUM_BYTES);

    if (nrw > 0) {
        typename P::Act act[NC];
        if (F32) {
            const LdsAct la{lqs, ld_, lbs, K};
#pragma unroll
            for (int n = 0; n < NC; n++) P::load_act(la, n, kseg, vlane, g, act[n]);
        } else {
#pragma unroll
            for (int n = 0; n < NC; n++) P::load_act(a, col0 + n, kseg, vlane, g, act[n]);
        }
        float keep[NC];  // lane 63-i ends up holding the total of the wave's row i
        if constexpr (AHEAD && ROW16) {
            if (tail) thin_rows_two<P, TAILR>(w, g, cur, nxt, act, r0 + rl0, nrw, lane, part, rl0, kw, kseg);
            else thin_rows_two<P, 1>(w, g, cur, nxt, act, r0 + rl0, nrw, lane, part, rl0, kw, kseg);
        } else if constexpr (AHEAD) {
            if (tail) thin_rows<P, NC, DIRECT, TAILR>(w, g, cur, act, r0 + rl0, nrw, lane, keep, part, rl0, kw, kseg);
            else thin_rows_ahead<P, DIRECT>(w, g, cur, nxt, act, r0 + rl0, nrw, lane, keep, part, rl0, kw, kseg);
        } else if (tail) thin_rows<P, NC, DIRECT, TAILR>(w, g, cur, act, r0 + rl0, nrw, lane, keep, part, rl0, kw, kseg);
        else thin_rows<P, NC, DIRECT, RPL>(w, g, cur, act, r0 + rl0, nrw, lane, keep, part, rl0, kw, kseg);
        if (DIRECT && lane > 63 - nrw) {
#pragma unroll
            for (int n = 0; n < NC; n++) yrow0[(int64_t)n * ldy + rl0 + (63 - lane)] = keep[n];
        }
    }
    if (DIRECT) return;

    if (AHEAD && seg_sync) {
        // the kw waves of a row group count themselves in when their partial sums are in LDS; the last one adds them, in
        // segment order as always, and stores the rows
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        int arrived = 0;
        if (lane == 0) arrived = __hip_atomic_fetch_add(&seg_cnt[8 + rg], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        arrived = __builtin_amdgcn_readfirstlane(arrived);
        if (arrived == kw - 1 && lane < nrw) {
            float sum = 0.f;
            for (int k = 0; k < kw; k++) sum += part[(rl0 + lane) * kw + k];
            yrow0[rl0 + lane] = sum;
        }
        return;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nrows * NC; i += (kw << rw_log2) * 64) {
        const int n = i / nrows, rl = i - n * nrows;
        float sum = 0.f;
        for (int k = 0; k < kw; k++) sum += part[(rl * NC + n) * kw + k];
        yrow0[(int64_t)n * ldy + rl] = sum;
    }
}

// ---------------------------------------------------------------------------------------------
// Gate and up of a feed-forward block in one pass with the gating in the epilogue: h = silu(Wg x) * (Wu x).
// A wave walks "virtual rows" 2j (row j of the gate matrix) and 2j+1 (row j of the up matrix) with the
// thin kernel's loop, so both totals of a row meet in one wave (neighbouring lanes) or in one
// workgroup's LDS, and silu(gate) * up is computed once per element, by whoever produced it -- instead
// of by every workgroup of the down projection in its prologue.  One column, f32 x (optionally through
// RMSNorm first).  The two totals are the numbers the separate products give, so h has the bits of
// mi_qmm_swiglu on their outputs.
// ---------------------------------------------------------------------------------------------
template <class P, bool DIRECT, int RPL>
__device__ __forceinline__ void thin_rows_pair(const DevWeight &wa, const DevWeight &wb, const typename P::Geo &g,
                                               typename P::Raw cur, const typename P::Act (&act)[1], int64_t wrow0, int nv,
                                               int lane, float &keep, float *part, int rl0v, int kw, int kseg) {
    static_assert(RPL == 1 || DIRECT, "rows side by side only when a row lies inside one K segment");
    const int run = RPL == 1 ? 0 : lane / (64 / RPL);
    keep = 0.f;
#pragma unroll 1
    for (int i = 0; i < nv; i += RPL) {
        float acc[1] = {0.f};
        P::template dot<1>(cur, g, act, acc);
        if (i + RPL < nv) {  // wave-uniform branch
            const int v = min(i + RPL + run, nv - 1);
            cur = P::load(v & 1 ? wb : wa, g, wrow0 + (v >> 1));
        }
        const int tot_all = __float_as_int(run_total<RPL>(acc[0]));
#pragma unroll
        for (int r = 0; r < RPL; r++) {
            const float tot = __int_as_float(__builtin_amdgcn_readlane(tot_all, 64 / RPL * (r + 1) - 1));
            if (DIRECT) keep = lane == 63 - (i + r) ? tot : keep;
            else if (lane == 63) part[(rl0v + i) * kw + kseg] = tot;
        }
    }
}

template <class P, bool DIRECT, int XMODE, int RPL, int XP>
__global__ __launch_bounds__(1024) void gemv_pair_kernel(ThinArgs ta, const float *__restrict__ xf, int rows_per_wave, int kw,
                                                         int rw_log2, Produce pr) {
    static_assert(XMODE == 1 || XMODE == 2, "f32 x, plain or through RMSNorm");
    extern __shared__ __align__(16) uint8_t smem[];
    const DevWeight wa{ta.p0[0], ta.p1[0], ta.p2[0], ta.d[0], ta.K, ta.M[0], ta.type};
    const DevWeight wb{ta.p0[1], ta.p1[1], ta.p2[1], ta.d[1], ta.K, ta.M[0], ta.type};
    float *__restrict__ hout = ta.y[0];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rw = 1 << rw_log2;
    const int rg = wave & (rw - 1), kseg = wave >> rw_log2;
    // rows_per_wave as in gemv_thin_kernel: rows of h of every wave, and in the high half how many of the first row groups
    // take one more
    const int rpw_base = rows_per_wave & 0xffff, rpw_extra = rows_per_wave >> 16;
    const int rows_per_wg = (rpw_base << rw_log2) + rpw_extra;  // rows of h per workgroup
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_wg;
    const int nrows = (int)min((int64_t)rows_per_wg, wa.M - r0);
    const int rl0 = rg * rpw_base + min(rg, rpw_extra);
    const int nrw = max(0, min(rpw_base + (rg < rpw_extra ? 1 : 0), nrows - rl0));   // rows of h of this wave; 2 * nrw virtual rows
    const int vlane = lane & (64 / RPL - 1), run = RPL == 1 ? 0 : lane / (64 / RPL);
    const typename P::Geo g = P::geo(wa, kseg, vlane);

    const int64_t K = ta.K;
    const int nblk = (int)(K / P::ACT_BLK);
    const int nbs = P::USES_BSUMS ? (int)(K / P::ACT_BSUM) : 0;
    const size_t act_bytes = (((size_t)(K + nblk * 4 + nbs * 2)) + 15) / 16 * 16;
    int8_t *lqs = reinterpret_cast<int8_t *>(smem);
    float *ld_ = reinterpret_cast<float *>(smem + (size_t)K);
    int16_t *lbs = reinterpret_cast<int16_t *>(smem + (size_t)K + (size_t)nblk * 4);
    const float4 *x4 = reinterpret_cast<const float4 *>(xf);
    const int total4 = (int)(K / 4);
    const int nwaves = kw << rw_log2 /* = (kw << rw_log2) * 64 / 64, without the hidden-argument load */;
    float4 xpre[XP], apre[XP];
    prefetch_x(x4, total4, wave, nwaves, lane, xpre);
    const bool has_aux = XMODE == 2 && pr.aux != nullptr;
    if (XMODE == 2) prefetch_x(has_aux ? reinterpret_cast<const float4 *>(pr.aux) : x4, total4, wave, nwaves, lane, apre);
    typename P::Raw cur;
    {   // unconditional and behind the x loads, as in gemv_thin_kernel: the quantization then waits for x only
        const int v = min(run, 2 * max(nrw, 1) - 1);
        __builtin_amdgcn_sched_barrier(0);
        cur = P::load(v & 1 ? wb : wa, g, min(r0 + rl0 + (v >> 1), wa.M - 1));
        __builtin_amdgcn_sched_barrier(0);
    }
    constexpr size_t PSUM_BYTES = XMODE == 2 ? XPRE * 16 * sizeof(double) : 0;
    if (XMODE == 2) {
        double *psum = reinterpret_cast<double *>(smem + act_bytes);
#pragma unroll
        for (int j = 0; j < XP; j++) {
            const int c = wave + j * nwaves;
            if (c * 64 < total4) {  // wave-uniform
                const double sq = piece_sumsq(c * 64 + lane < total4 ? xpre[j] : make_float4(0.f, 0.f, 0.f, 0.f));
                if (lane == 0) psum[c] = sq;
            }
        }
        __syncthreads();
        double tot = 0.0;
        for (int c = 0; c * 64 < total4; c++) tot += psum[c];
        const float scale = rms_scale_of(tot, K, pr.eps);
#pragma unroll
        for (int j = 0; j < XP; j++) xpre[j] = rms_apply(xpre[j], scale, apre[j], has_aux);
    }
    quantize_x_to_lds<P, XP>(x4, total4, wave, nwaves, lane, xpre, lqs, ld_, lbs);
    __syncthreads();
    float *part = reinterpret_cast<float *>(smem + act_bytes + PSUM_BYTES);

    if (nrw > 0) {
        typename P::Act act[1];
        const LdsAct la{lqs, ld_, lbs, K};
        P::load_act(la, 0, kseg, vlane, g, act[0]);
        float keep;  // lane 63-v ends up holding the total of the wave's virtual row v
        thin_rows_pair<P, DIRECT, RPL>(wa, wb, g, cur, act, r0 + rl0, 2 * nrw, lane, keep, part, 2 * rl0, kw, kseg);
        if (DIRECT) {
            const float up = dpp_mov<0xB1>(keep);  // lane ^ 1: the odd lane 63-2j takes the up total from lane 62-2j
            if ((lane & 1) && lane > 63 - 2 * nrw) hout[r0 + rl0 + ((63 - lane) >> 1)] = silu_mul(keep, up);
        }
    }
    if (DIRECT) return;

    __syncthreads();
    for (int i = threadIdx.x; i < nrows; i += (kw << rw_log2) * 64) {
        float gsum = 0.f, usum = 0.f;
        for (int k = 0; k < kw; k++) gsum += part[(2 * i) * kw + k];
        for (int k = 0; k < kw; k++) usum += part[(2 * i + 1) * kw + k];
        hout[r0 + i] = silu_mul(gsum, usum);
    }
}

struct Plan { int kw, rw, rw_log2, spw, rows_per_wg, rpl, tail_log2 = 0; unsigned grid; size_t lds; int even_wgs = 0; };

// 8 waves per workgroup (two per SIMD, so a wave may use up to 256 VGPRs), one or two workgroups per CU.
// total_m is the number of rows over all tensors of the launch.
template <class P>
bool make_plan(int64_t K, int64_t total_m, int nc, int num_cus, Plan &p) {
    const int nseg = (int)((K + P::SEG - 1) / P::SEG);
    if (nseg < 1) return false;
    p.spw = nseg <= 8 ? 1 : nseg <= 16 ? 2 : nseg <= 32 ? 4 : 0;
    if (!p.spw) return false;
    p.kw = (nseg + p.spw - 1) / p.spw;
    p.rw_log2 = p.kw >= 5 ? 0 : p.kw >= 3 ? 1 : p.kw == 2 ? 2 : 3;  // largest power of two with kw*rw <= 8
    p.rw = 1 << p.rw_log2;
    const int64_t target_wgs = (int64_t)num_cus * (P::HEAVY ? 1 : 2);
    int64_t rows = (total_m + target_wgs - 1) / target_wgs;
    const int64_t lds_cap_rows = 8192 / (nc * p.kw);  // <= 32 KiB of partials
    if (rows > lds_cap_rows) rows = lds_cap_rows;
    if (rows < 1) rows = 1;
    p.rows_per_wg = (int)rows;
    p.lds = p.kw == 1 ? 0 : (size_t)rows * nc * p.kw * sizeof(float);
    return true;
}

// Thin plan: kw waves side by side along K (one segment each) times rw row groups, a few consecutive
// rows per wave.  Four waves per workgroup (kw of them when K has more than four segments); with f32
// activations the workgroup also quantizes all of x into LDS first, so it is made larger (up to 16
// waves) to spread that work and to keep the number of times x is read from L2 down.
constexpr size_t THIN_LDS_MAX = 64 * 1024;

template <class P>
size_t thin_act_lds(int64_t K, int nc) {
    const size_t b = (size_t)nc * (K + K / P::ACT_BLK * 4 + (P::USES_BSUMS ? K / P::ACT_BSUM * 2 : 0));
    return (b + 15) / 16 * 16;
}

// produce: the f32 activations go through a producer first (one column; room for RMSNorm's piece sums, and
// every piece of x must sit in a prefetch register of some wave)
// uneven: the caller's kernel takes workgroups whose rows do not divide by their row groups (gemv_thin_kernel)
template <class P>
bool make_thin_plan(int64_t K, int64_t total_m, int nc, bool f32, Plan &p, bool produce = false, bool uneven = false) {
    const int nseg = (int)((K + P::SEG - 1) / P::SEG);
    if (nseg < 1 || nseg > 8) return false;
    p.spw = 1;
    p.kw = nseg;
    // Q6_K needs 70-75 registers: a 16-wave workgroup then has a CU to itself (four waves per SIMD), three
    // 8-wave ones share it (six per SIMD).  Measured with rows of one segment: 14336 x 4096 12.2 against
    // 15.6 us; with several segments per row the larger workgroup wins (4096 x 14336: 13.5 against 18.0 us).
    const int mwt = f32 && p.kw == 1 && nc == 1 ? P::F32_WAVES_ONE_SEG : thin_max_waves(nc, f32);
    const int max_waves = p.kw > mwt ? p.kw : mwt;
    p.rw_log2 = 0;
    while (p.kw << (p.rw_log2 + 1) <= max_waves) p.rw_log2++;
    p.rw = 1 << p.rw_log2;
    int rows_per_wave;
    {
        if (f32) {
            // every workgroup re-quantizes x: keep them to one resident round (at most 1.75 per CU),
            // an even number of rows per wave
            const int64_t rows_per_rw = (total_m + (int64_t)448 * p.rw - 1) / ((int64_t)448 * p.rw);
            rows_per_wave = (int)((rows_per_rw + 1) / 2 * 2);
            if (rows_per_wave < 2) rows_per_wave = 2;
            // ... and among the larger even counts the one that loads the 256 CUs most evenly: the busiest CU runs
            // ceil(workgroups / 256) workgroups of rw * rows each (4096 rows in workgroups of 12 are 342 workgroups,
            // two on every third CU; in workgroups of 16 they are one per CU: Q4_0 4096 x 14336 13.0 -> 11.0 us)
            auto busiest = [&](int rows) {
                const int64_t wgs = (total_m + (int64_t)p.rw * rows - 1) / ((int64_t)p.rw * rows);
                return (wgs + 255) / 256 * rows;
            };
            for (int rows = rows_per_wave + 2; rows <= 16; rows += 2)
                if (busiest(rows) < busiest(rows_per_wave)) rows_per_wave = rows;
        } else {
            rows_per_wave = (nc >= 4 || total_m > 65536) ? 4 : 2;
        }
    }
    // Rows of several segments whose last segment is at most half (a quarter) full -- K = 14336 = 3.5 segments of
    // 4096, K = 5120 = 1.25: the waves of that segment take 2 (4) rows side by side per load, as the waves of short
    // rows do, instead of running with half (three quarters) of their lanes dead.  One and two columns.
    p.tail_log2 = 0;
    if (p.kw > 1 && nc <= 2 && !produce) {
        const int tail = rows_per_load<P>(K - (int64_t)(p.kw - 1) * P::SEG);
        p.tail_log2 = tail == 4 ? 2 : tail == 2 ? 1 : 0;
        rows_per_wave = (rows_per_wave + tail - 1) / tail * tail;
    }
    // short rows: 2 or 4 side by side per load, and at least two loads per wave (one in flight)
    p.rpl = p.kw == 1 ? rows_per_load<P>(K) : 1;
    if (p.rpl > 1) rows_per_wave = max(2 * p.rpl, (rows_per_wave + p.rpl - 1) / p.rpl * p.rpl);
    if (rows_per_wave > 16) rows_per_wave = 16;  // a wave parks its row totals in lanes 63, 62, ...
    p.rows_per_wg = p.rw * rows_per_wave;
    if (uneven && f32 && p.kw == 1 && p.rpl == 1 && nc <= 2) {
        // The same number of workgroups on every CU: their count rounded up to a multiple of the CUs and the rows dealt
        // out evenly, some row groups taking one row more than the others.  28672 rows in workgroups of 64 are 448
        // workgroups, two on 192 CUs and one on 64; the lone ones are through at 7.9 us, the second workgroups of the
        // others at 11.2-11.8 (stamps per wave).  In 512 workgroups of 56 rows: gate + up 12.91 -> 12.61 us, Q6_K
        // 14336 x 4096 11.5 -> 10.4.  It pays where CUs hold two workgroups and it adds few (at most a fifth more; with one
        // workgroup per CU, 230 -> 256 workgroups, 22016 rows measured 11.2 -> 12.0 us, Q6_K 11008 rows 9.5 -> 10.5, and the
        // gate / up pair kernel at 11008 rows 11.4 -> 12.0) or where a wave has only two rows
        // anyway and the launch is all start-up (Q4_K 4096 / 6144 / 11008 / 13824 rows: 2-6 % faster with every CU at work;
        // at two columns Q4_K 4096 x 4096 5.6 -> 5.0 us, Q6_K 14336 x 4096 14.7 -> 13.2).
        const int64_t wgs = (total_m + p.rows_per_wg - 1) / p.rows_per_wg;
        const int64_t target = (wgs + 255) / 256 * 256;
        const int64_t even = (total_m + target - 1) / target;
        const bool few_more = target >= 512 && 5 * target <= 6 * wgs, short_waves = rows_per_wave == 2 && p.rw == 16;
        if (target != wgs && (few_more || short_waves) && even >= p.rw && even <= 16 * p.rw) {
            p.rows_per_wg = (int)even;
            p.even_wgs = (int)target;  // (several matrices: the caller makes sure their workgroups together do not exceed it)
        }
    }
    p.lds = (f32 ? thin_act_lds<P>(K, nc) : 0) + (p.kw == 1 ? 0 : (size_t)p.rows_per_wg * nc * p.kw * sizeof(float) + 64);  // + 16 counters
    if (produce) {
        if (!f32 || nc != 1 || K > (int64_t)XPRE * p.kw * p.rw * 256) return false;
        p.lds += XPRE * 16 * sizeof(double);
    }
    return p.lds <= THIN_LDS_MAX;
}

template <class P, int NC, int XMODE, int XP = XPRE>
void launch_thin_mode(const Plan &p, const ThinArgs &ma, const DevAct &a, const float *xf, int col0, const Produce &pr,
                      hipStream_t s) {
    const dim3 block(64 * p.kw * p.rw);
    const int rpw = (p.rows_per_wg >> p.rw_log2) | ((p.rows_per_wg & (p.rw - 1)) << 16);
#define THIN_LAUNCH(DIRECT, RPL) \
    gemv_thin_kernel<P, NC, DIRECT, XMODE, RPL, XP><<<p.grid, block, p.lds, s>>>(ma, a, xf, col0, rpw, p.kw, p.rw_log2, pr)
#define THIN_LAUNCH_SEGMENTS(AHEAD, TAILR) \
    gemv_thin_kernel<P, NC, false, XMODE, 1, XP, AHEAD, TAILR><<<p.grid, block, p.lds, s>>>(ma, a, xf, col0, rpw, p.kw, p.rw_log2, pr)
    if constexpr (XMODE <= 1 && NC <= 2) {
        if (p.kw > 1) {
            // one plain f32 column (the down projection's shape): the second row ahead, +1.4 % on the whole decode step
            constexpr bool AH = XMODE == 1 && NC == 1 && XP > 1;
            if (p.tail_log2 == 2) THIN_LAUNCH_SEGMENTS(AH, 4);
            else if (p.tail_log2 == 1) THIN_LAUNCH_SEGMENTS(AH, 2);
            else THIN_LAUNCH_SEGMENTS(AH, 1);
            return;
        }
    }
    if (p.kw > 1) THIN_LAUNCH(false, 1);
    else if (p.rpl == 4) THIN_LAUNCH(true, 4);
    else if (p.rpl == 2) THIN_LAUNCH(true, 2);
    else THIN_LAUNCH(true, 1);
#undef THIN_LAUNCH
#undef THIN_LAUNCH_SEGMENTS
}

template <class P, int NC>
void launch_thin(const Plan &p, const ThinArgs &ma, const DevAct &a, const float *xf, int col0, const Produce &pr,
                 hipStream_t s) {
    const bool one_piece = ma.K <= (int64_t)256 * p.kw * p.rw;  // a piece per wave covers the row
    if (!xf) launch_thin_mode<P, NC, 0>(p, ma, a, xf, col0, pr, s);
    else if (NC == 1 && pr.kind == PRODUCE_RMSNORM && one_piece) launch_thin_mode<P, 1, 2, 1>(p, ma, a, xf, col0, pr, s);
    else if (NC == 1 && pr.kind == PRODUCE_RMSNORM) launch_thin_mode<P, 1, 2>(p, ma, a, xf, col0, pr, s);
    else if (NC == 1 && pr.kind == PRODUCE_SWIGLU && one_piece) launch_thin_mode<P, 1, 3, 1>(p, ma, a, xf, col0, pr, s);
    else if (NC == 1 && pr.kind == PRODUCE_SWIGLU) launch_thin_mode<P, 1, 3>(p, ma, a, xf, col0, pr, s);
    else if (NC == 1 && one_piece) launch_thin_mode<P, 1, 1, 1>(p, ma, a, xf, col0, pr, s);
    else launch_thin_mode<P, NC, 1>(p, ma, a, xf, col0, pr, s);
}

template <class P, int NC, int SPW, int U>
void launch_one(const Plan &p, const MultiArgs &ma, const DevAct &a, int col0, hipStream_t s) {
    const dim3 block(64 * p.kw * p.rw);
    if (p.kw == 1)
        gemv_kernel<P, NC, SPW, U, true><<<p.grid, block, 0, s>>>(ma, a, col0, p.rows_per_wg, p.kw, p.rw_log2);
    else
        gemv_kernel<P, NC, SPW, U, false><<<p.grid, block, p.lds, s>>>(ma, a, col0, p.rows_per_wg, p.kw, p.rw_log2);
}

template <class P>
hipError_t launch_type(const DevWeight *ws, float *const *ys, int count, const DevAct &a, const float *xf, int col0,
                       int nc, int num_cus, const Produce &pr, hipStream_t s) {
    int64_t total_m = 0;
    for (int i = 0; i < count; i++) total_m += ws[i].M;
    Plan p;
    const bool thin = make_thin_plan<P>(ws[0].K, total_m, nc, xf != nullptr, p, pr.kind != PRODUCE_NONE, true);
    if (pr.kind != PRODUCE_NONE && !thin) return hipErrorInvalidValue;  // callers ask gemv_produce_supported() first
    if (xf && !thin) return hipErrorInvalidValue;  // callers ask gemv_f32_supported() first
    if (!thin) {
        if (!make_plan<P>(ws[0].K, total_m, nc, num_cus, p)) return hipErrorInvalidValue;
        if (p.spw > 1 && !make_plan<P>(ws[0].K, total_m, 1, num_cus, p)) return hipErrorInvalidValue;
    }
    if (thin && p.even_wgs && count > 1) {
        // an even plan was made for the rows of all matrices together; every matrix rounds its workgroups up by itself, and
        // one workgroup too many is a CU with three where the others have two
        auto wgs_at = [&](int rows) {
            int64_t n = 0;
            for (int i = 0; i < count; i++) n += (ws[i].M + rows - 1) / rows;
            return n;
        };
        while (wgs_at(p.rows_per_wg) > p.even_wgs && p.rows_per_wg < 16 * p.rw) p.rows_per_wg++;
    }
    MultiArgs ma;
    ma.count = count;
    int64_t wgs = 0;
    for (int i = 0; i < MAX_MULTI; i++) {
        const int j = i < count ? i : count - 1;
        ma.w[i] = ws[j]; ma.y[i] = ys[j]; ma.ldy[i] = ws[j].M;
        if (i < count) wgs += (ws[i].M + p.rows_per_wg - 1) / p.rows_per_wg;
        ma.wg_end[i] = (int)wgs;
    }
    if (wgs > 0x7fffffff) return hipErrorInvalidValue;
    p.grid = (unsigned)wgs;
    if (thin) {
        ThinArgs ta;
        for (int i = 0; i < MAX_MULTI; i++) {
            const int j = i < count ? i : count - 1;
            ta.p0[i] = ws[j].p0; ta.p1[i] = ws[j].p1; ta.p2[i] = ws[j].p2; ta.d[i] = ws[j].d;
            ta.y[i] = ys[j]; ta.M[i] = ws[j].M;
            ta.wg_end[i] = i < count ? ma.wg_end[i] : 0x7fffffff;
        }
        ta.K = ws[0].K; ta.type = ws[0].type;
        switch (nc) {
        case 1: launch_thin<P, 1>(p, ta, a, xf, col0, pr, s); break;
        case 2: launch_thin<P, 2>(p, ta, a, xf, col0, pr, s); break;
        case 3: launch_thin<P, 3>(p, ta, a, xf, col0, pr, s); break;
        case 4: launch_thin<P, 4>(p, ta, a, xf, col0, pr, s); break;
        case 5: launch_thin<P, 5>(p, ta, a, xf, col0, pr, s); break;
        case 6: launch_thin<P, 6>(p, ta, a, xf, col0, pr, s); break;
        case 7: launch_thin<P, 7>(p, ta, a, xf, col0, pr, s); break;
        case 8: launch_thin<P, 8>(p, ta, a, xf, col0, pr, s); break;
        default: return hipErrorInvalidValue;
        }
        return hipGetLastError();
    }
    if (p.spw > 1) {
        // long rows: several segments per wave, one column per launch
        for (int c = col0; c < col0 + nc; c++) {
            if (p.spw == 2) launch_one<P, 1, 2, (P::HEAVY ? 1 : 2)>(p, ma, a, c, s);
            else launch_one<P, 1, 4, 1>(p, ma, a, c, s);
        }
        return hipGetLastError();
    }
    return hipErrorInvalidValue;  // not reached: K within eight segments always takes the thin plan
}

}  // namespace

int64_t gemv_max_k(int type) {
    switch (type) {
    case T_Q8_0: return 32 * (int64_t)PolQ8_0::SEG;
    case T_Q4_0: return 32 * (int64_t)PolQ4_0::SEG;
    case T_MXFP4: return 32 * (int64_t)PolMXFP4::SEG;
    case T_Q4_K: return 32 * (int64_t)PolQ4K::SEG;
    case T_Q5_K: return 32 * (int64_t)PolQ5K::SEG;
    case T_Q6_K: return 32 * (int64_t)PolQ6K::SEG;
    default: return 0;
    }
}

int gemv_max_multi() { return MAX_MULTI; }

namespace {

hipError_t dispatch(const DevWeight *ws, float *const *ys, int count, const DevAct &a, const float *xf, int col0,
                    int ncols, int num_cus, hipStream_t s, const Produce &pr = Produce{PRODUCE_NONE, nullptr, 0.f, nullptr}) {
    if (count < 1 || count > MAX_MULTI || ncols < 1 || ncols > MAXC || col0 < 0 || col0 + ncols > a.N)
        return hipErrorInvalidValue;
    for (int i = 0; i < count; i++)
        if (ws[i].type != ws[0].type || ws[i].K != ws[0].K || ws[i].M < 1 || !ys[i]) return hipErrorInvalidValue;
    if (ws[0].K < 1 || ws[0].K > gemv_max_k(ws[0].type) || a.K != ws[0].K) return hipErrorInvalidValue;
    switch (ws[0].type) {
    case T_Q4_K: return a.type == T_Q8_K ? launch_type<PolQ4K>(ws, ys, count, a, xf, col0, ncols, num_cus, pr, s) : hipErrorInvalidValue;
    case T_Q5_K: return a.type == T_Q8_K ? launch_type<PolQ5K>(ws, ys, count, a, xf, col0, ncols, num_cus, pr, s) : hipErrorInvalidValue;
    case T_Q6_K: return a.type == T_Q8_K ? launch_type<PolQ6K>(ws, ys, count, a, xf, col0, ncols, num_cus, pr, s) : hipErrorInvalidValue;
    case T_Q4_0: return a.type == T_Q8_0 ? launch_type<PolQ4_0>(ws, ys, count, a, xf, col0, ncols, num_cus, pr, s) : hipErrorInvalidValue;
    case T_MXFP4: return a.type == T_Q8_0 ? launch_type<PolMXFP4>(ws, ys, count, a, xf, col0, ncols, num_cus, pr, s) : hipErrorInvalidValue;
    case T_Q8_0: return a.type == T_Q8_0 ? launch_type<PolQ8_0>(ws, ys, count, a, xf, col0, ncols, num_cus, pr, s) : hipErrorInvalidValue;
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

hipError_t launch_gemv_multi(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int col0, int ncols,
                             int num_cus, hipStream_t s) {
    return dispatch(ws, ys, count, a, nullptr, col0, ncols, num_cus, s);
}

hipError_t launch_gemv(const DevWeight &w, const DevAct &a, int col0, int ncols, float *y, int64_t ldy,
                       int num_cus, hipStream_t s) {
    if (ldy != w.M) return hipErrorInvalidValue;
    float *ys[1] = {y};
    return launch_gemv_multi(&w, ys, 1, a, col0, ncols, num_cus, s);
}

bool gemv_f32_supported(int type, int64_t K, int64_t total_m, int ncols) {
    // Beyond 64 Ki rows (an output head) the redundant per-workgroup quantization costs more than the
    // launch it saves.  Several columns (every workgroup quantizes all of them), measured against
    // quantize-then-multiply on matrices from 2 MB to 97 MB: two columns of the K-quants always win (gate 14336 x 4096
    // 12.9 -> 12.0 us, down 4096 x 14336 14.9 -> 12.9, Q6_K 4096 x 14336 18.4 -> 14.3, gate + up in one launch 20.3 ->
    // 18.9); three columns of Q6_K (which the matrix-core kernel takes from four) win from about 32 MB (22.2 -> 17.8 us
    // at 48 MB) and lose below (6.6 -> 7.8 at 3 MB); two and three columns of Q4_0 / Q8_0 win at every size while rows
    // are short (Q8_0 14336 x 4096: 17.6 -> 14.0 and 20.1 -> 17.9) and lose on long rows (Q4_0 4096 x 14336: 14.9 ->
    // 19.5), which take the matrix-core kernel from two columns instead (wants_skinny in capi.hip).
    if (ncols < 1 || ncols > MAXC || K < 1 || total_m < 1 || total_m > 65536) return false;
    if (ncols > 1) {
        const bool kquant = type == T_Q4_K || type == T_Q5_K || type == T_Q6_K;
        const int64_t approx_bytes = total_m * K * (type == T_Q8_0 ? 34 : type == T_Q6_K ? 26 : 18) / 32;
        if (kquant) {
            if (ncols > 3 || (ncols == 3 && (type != T_Q6_K || approx_bytes < (32 << 20)))) return false;
        } else {
            if (ncols > 3 || K > 8192) return false;
        }
    }
    Plan p;
    switch (type) {
    case T_Q4_K: return make_thin_plan<PolQ4K>(K, total_m, ncols, true, p);
    case T_Q5_K: return make_thin_plan<PolQ5K>(K, total_m, ncols, true, p);
    case T_Q6_K: return make_thin_plan<PolQ6K>(K, total_m, ncols, true, p);
    case T_Q4_0: return make_thin_plan<PolQ4_0>(K, total_m, ncols, true, p);
    case T_MXFP4: return make_thin_plan<PolMXFP4>(K, total_m, ncols, true, p);
    case T_Q8_0: return make_thin_plan<PolQ8_0>(K, total_m, ncols, true, p);
    default: return false;
    }
}

hipError_t launch_gemv_f32_multi(const DevWeight *ws, float *const *ys, int count, const float *x, int ncols,
                                 int num_cus, hipStream_t s, const Produce *produce) {
    if (!x || count < 1) return hipErrorInvalidValue;
    Produce pr{PRODUCE_NONE, nullptr, 0.f, nullptr};
    if (produce) pr = *produce;
    if (pr.kind < PRODUCE_NONE || pr.kind > PRODUCE_SWIGLU || (pr.kind == PRODUCE_SWIGLU && !pr.aux) ||
        (pr.kind != PRODUCE_NONE && ncols != 1))
        return hipErrorInvalidValue;
    DevAct a{};  // only the geometry is read: the kernel quantizes x itself
    a.K = ws[0].K;
    a.N = ncols;
    a.type = (ws[0].type == T_Q4_K || ws[0].type == T_Q5_K || ws[0].type == T_Q6_K) ? T_Q8_K : T_Q8_0;
    return dispatch(ws, ys, count, a, x, 0, ncols, num_cus, s, pr);
}

namespace {

template <class P, int XMODE, int XP>
void launch_pair_mode(const Plan &p, const ThinArgs &ta, const float *xf, const Produce &pr, unsigned grid, int rows_h, hipStream_t s) {
    const dim3 block(64 * p.kw * p.rw);
    const int rpw = (rows_h >> p.rw_log2) | ((rows_h & (p.rw - 1)) << 16);  // rows of h per wave (+ row groups with one more)
#define PAIR_LAUNCH(DIRECT, RPL) \
    gemv_pair_kernel<P, DIRECT, XMODE, RPL, XP><<<grid, block, p.lds, s>>>(ta, xf, rpw, p.kw, p.rw_log2, pr)
    if (p.kw > 1) PAIR_LAUNCH(false, 1);
    else if (p.rpl == 4) PAIR_LAUNCH(true, 4);
    else if (p.rpl == 2) PAIR_LAUNCH(true, 2);
    else PAIR_LAUNCH(true, 1);
#undef PAIR_LAUNCH
}

template <class P>
bool pair_plan(int64_t K, int64_t M, bool rms, Plan &p) {
    // planned like the two matrices in one launch: the virtual rows of a wave are an even number
    if (M < 1 || 2 * M > 65536 || !make_thin_plan<P>(K, 2 * M, 1, true, p, rms)) return false;
    return ((p.rows_per_wg >> p.rw_log2) & 1) == 0;
}

template <class P>
hipError_t launch_pair_type(const DevWeight &wg, const DevWeight &wu, const float *xf, float *h, const Produce &pr,
                            hipStream_t s) {
    Plan p;
    const bool rms = pr.kind == PRODUCE_RMSNORM;
    if (!pair_plan<P>(wg.K, wg.M, rms, p)) return hipErrorInvalidValue;
    ThinArgs ta;
    for (int i = 0; i < MAX_MULTI; i++) {
        const DevWeight &w = i == 1 ? wu : wg;
        ta.p0[i] = w.p0; ta.p1[i] = w.p1; ta.p2[i] = w.p2; ta.d[i] = w.d; ta.y[i] = h; ta.M[i] = wg.M;
        ta.wg_end[i] = 0x7fffffff;
    }
    ta.K = wg.K; ta.type = wg.type;
    int rows_per_wg = p.rows_per_wg / 2;  // rows of h
    if (p.kw == 1 && p.rpl == 1) {
        // the same number of workgroups on every CU where they hold two and that adds at most a fifth (as in
        // make_thin_plan): 14336 rows of h in 512 workgroups of 28 instead of 448 of 32, 13.1 -> 12.8 us
        const int64_t wgs = (wg.M + rows_per_wg - 1) / rows_per_wg, target = (wgs + 255) / 256 * 256;
        const int64_t even = (wg.M + target - 1) / target;
        if (target != wgs && target >= 512 && 5 * target <= 6 * wgs && even >= p.rw && even <= 8 * p.rw) rows_per_wg = (int)even;
    }
    const unsigned grid = (unsigned)((wg.M + rows_per_wg - 1) / rows_per_wg);
    const bool one_piece = wg.K <= (int64_t)256 * p.kw * p.rw;
    if (rms && one_piece) launch_pair_mode<P, 2, 1>(p, ta, xf, pr, grid, rows_per_wg, s);
    else if (rms) launch_pair_mode<P, 2, XPRE>(p, ta, xf, pr, grid, rows_per_wg, s);
    else if (one_piece) launch_pair_mode<P, 1, 1>(p, ta, xf, pr, grid, rows_per_wg, s);
    else launch_pair_mode<P, 1, XPRE>(p, ta, xf, pr, grid, rows_per_wg, s);
    return hipGetLastError();
}

}  // namespace

bool gemv_pair_supported(int type, int64_t K, int64_t M, bool rms) {
    Plan p;
    switch (type) {
    case T_Q4_K: return pair_plan<PolQ4K>(K, M, rms, p);
    case T_Q5_K: return pair_plan<PolQ5K>(K, M, rms, p);
    case T_Q6_K: return pair_plan<PolQ6K>(K, M, rms, p);
    case T_Q4_0: return pair_plan<PolQ4_0>(K, M, rms, p);
    case T_MXFP4: return pair_plan<PolMXFP4>(K, M, rms, p);
    case T_Q8_0: return pair_plan<PolQ8_0>(K, M, rms, p);
    default: return false;
    }
}

hipError_t launch_gemv_pair_f32(const DevWeight &wg, const DevWeight &wu, const float *x, float *h, hipStream_t s,
                                const Produce *produce) {
    if (!x || !h || wg.type != wu.type || wg.K != wu.K || wg.M != wu.M || wg.K < 1 || wg.K > gemv_max_k(wg.type))
        return hipErrorInvalidValue;
    Produce pr{PRODUCE_NONE, nullptr, 0.f, nullptr};
    if (produce) pr = *produce;
    if (pr.kind != PRODUCE_NONE && pr.kind != PRODUCE_RMSNORM) return hipErrorInvalidValue;
    switch (wg.type) {
    case T_Q4_K: return launch_pair_type<PolQ4K>(wg, wu, x, h, pr, s);
    case T_Q5_K: return launch_pair_type<PolQ5K>(wg, wu, x, h, pr, s);
    case T_Q6_K: return launch_pair_type<PolQ6K>(wg, wu, x, h, pr, s);
    case T_Q4_0: return launch_pair_type<PolQ4_0>(wg, wu, x, h, pr, s);
    case T_MXFP4: return launch_pair_type<PolMXFP4>(wg, wu, x, h, pr, s);
    case T_Q8_0: return launch_pair_type<PolQ8_0>(wg, wu, x, h, pr, s);
    default: return hipErrorInvalidValue;
    }
}

bool gemv_produce_supported(int type, int64_t K, int64_t total_m) {
    if (!gemv_f32_supported(type, K, total_m, 1)) return false;
    Plan p;
    switch (type) {
    case T_Q4_K: return make_thin_plan<PolQ4K>(K, total_m, 1, true, p, true);
    case T_Q5_K: return make_thin_plan<PolQ5K>(K, total_m, 1, true, p, true);
    case T_Q6_K: return make_thin_plan<PolQ6K>(K, total_m, 1, true, p, true);
    case T_Q4_0: return make_thin_plan<PolQ4_0>(K, total_m, 1, true, p, true);
    case T_MXFP4: return make_thin_plan<PolMXFP4>(K, total_m, 1, true, p, true);
    case T_Q8_0: return make_thin_plan<PolQ8_0>(K, total_m, 1, true, p, true);
    default: return false;
    }
}


// ---------------------------------------------------------------------------------------------
// Expert-indexed product (Tensor.MulmatID, /root/reference/ml/backend.go:153): the weight is a stack
// of n_expert matrices [K, M] (GGUF ne = [in, out, experts], /root/reference/convert/convert_gemma4.go:274-275),
// ids[t][i] names the expert that slot i of token t goes through, and
//   y[t][i][:] = W[ids[t][i]] . Q8(b[t][i mod b_cols][:])
// The (token, slot) pairs are independent GEMVs that happen to share weights when two pairs name
// the same expert.  A "group" is up to NC pairs of one expert; a workgroup belongs to one group and
// runs the thin kernel's loop over a few rows of that expert with the group's pairs as its
// activation columns.  Decode (a handful of pairs, experts all different) takes one pair per group
// straight from ids; larger batches are bucketed by expert first (group_pairs_kernel).
// A pair's result does not depend on what else is in its group: every column has its own
// accumulators and the same reduction order.
// ---------------------------------------------------------------------------------------------
namespace {

constexpr int ID_MAX_EXPERTS = 4096;

struct IdArgs {
    DevWeight w;           // the stack: rows e*M .. e*M+M-1 are expert e (w.M = M * n_expert)
    const int *ids;        // [pairs], pair = token * n_used + slot
    const int *groups;     // grouped launches: n_groups, then per group {expert, count, pair[NC]}; else null
    float *y;              // [pairs][M]
    int64_t M;             // rows per expert
    int n_expert, pairs, n_used, b_cols, wgs_per_group;
    // a second stack of the same type and shape against the same activations and ids (gate and up of an
    // expert FFN): the workgroups from wgs_first on belong to it.  wgs_first = INT_MAX: one stack.
    const uint8_t *p0b, *p1b, *p2b;
    const uint16_t *db;
    float *yb;
    int wgs_first;
};

// One workgroup of 1024 threads buckets the pairs by expert: counts in LDS, group ranges from a
// running sum over the experts, then every pair takes the next free place of its expert.  Pairs with
// an id outside 0..n_expert-1 go to a bucket of their own whose groups carry expert = -1.
template <int NC>
__global__ __launch_bounds__(1024) void group_pairs_kernel(const int *__restrict__ ids, int pairs, int n_expert,
                                                            int *__restrict__ groups) {
    __shared__ int count[ID_MAX_EXPERTS + 1], start[ID_MAX_EXPERTS + 1];
    constexpr int REC = 2 + NC;
    const int nb = n_expert + 1;
    for (int e = threadIdx.x; e < nb; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        const int e = ids[p];
        atomicAdd(&count[(e < 0 || e >= n_expert) ? n_expert : e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int g = 0;
        for (int e = 0; e < nb; e++) {
            start[e] = g;
            g += (count[e] + NC - 1) / NC;
        }
        groups[0] = g;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < nb; e += blockDim.x) {
        const int c = count[e];
        for (int g = 0; g * NC < c; g++) {
            int *rec = groups + 1 + (size_t)(start[e] + g) * REC;
            rec[0] = e < n_expert ? e : -1;
            rec[1] = min(NC, c - g * NC);
        }
        count[e] = 0;  // reused as the fill cursor
    }
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        const int e0 = ids[p];
        const int e = (e0 < 0 || e0 >= n_expert) ? n_expert : e0;
        const int pos = atomicAdd(&count[e], 1);
        groups[1 + (size_t)(start[e] + pos / NC) * REC + 2 + pos % NC] = p;
    }
}

// F32 (one pair per group only): xf is b itself, [tokens][b_cols][K] floats, and the workgroup quantizes
// its pair's activation row into LDS first, like the thin kernel does -- decode is one launch.
// For the expert GEMM: the pairs sorted by expert, every expert's run padded to whole 64-row tiles.
//   out[0]                       number of tiles
//   out[1 + 2t], out[2 + 2t]     tile t: expert (-1: ids outside the stack), first sorted row
//   src_col[row]                 activation row (token * b_cols + slot mod b_cols) behind sorted row, -1: padding
//   out_pair[row]                pair (token * n_used + slot) behind sorted row, -1: padding
// Which place a pair gets inside its expert's run depends on the order of the atomics; the product of a
// row does not depend on its place.
__global__ __launch_bounds__(1024) void sort_pairs_kernel(const int *__restrict__ ids, int pairs, int n_expert, int n_used,
                                                           int b_cols, int max_tiles, int tw, int *__restrict__ out,
                                                           int *__restrict__ src_col, int *__restrict__ out_pair) {
    __shared__ int count[ID_MAX_EXPERTS + 1], start[ID_MAX_EXPERTS + 1], scan[2][1024];
    const int nb = n_expert + 1, tid = threadIdx.x;
    // eight independent loads at a time: one workgroup has to hide the latency of ids by itself.  The first
    // 8192 ids are requested before anything else and stay in registers for both passes.
    int first[8];
#pragma unroll
    for (int j = 0; j < 8; j++) first[j] = tid + 1024 * j < pairs ? ids[tid + 1024 * j] : -1;
    for (int e = tid; e < nb; e += 1024) count[e] = 0;
    for (int r = tid; r < tw * max_tiles; r += 1024) { src_col[r] = -1; out_pair[r] = -1; }
    __syncthreads();
    for (int p0 = tid; p0 < pairs; p0 += 8 * 1024) {
        int e[8];
#pragma unroll
        for (int j = 0; j < 8; j++) e[j] = p0 == tid ? first[j] : p0 + 1024 * j < pairs ? ids[p0 + 1024 * j] : -1;
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (p0 + 1024 * j < pairs) atomicAdd(&count[(e[j] < 0 || e[j] >= n_expert) ? n_expert : e[j]], 1);
    }
    __syncthreads();
    // tiles per expert, then a running sum over the experts: thread t owns experts PER*t .. PER*t + PER-1
    constexpr int PER = (ID_MAX_EXPERTS + 1 + 1023) / 1024;
    int mine = 0;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int e = PER * tid + j;
        mine += e < nb ? (count[e] + tw - 1) / tw : 0;
    }
    scan[0][tid] = mine;
    __syncthreads();
    int cur = 0;
    const int owners = (nb + PER - 1) / PER;  // threads past these own no expert and never use their sums
    for (int step = 1; step < owners; step <<= 1, cur ^= 1) {
        scan[cur ^ 1][tid] = scan[cur][tid] + (tid >= step ? scan[cur][tid - step] : 0);
        __syncthreads();
    }
    int t = scan[cur][tid] - mine;  // tiles of all experts before this thread's
    if (tid == owners - 1) out[0] = scan[cur][tid];
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int e = PER * tid + j;
        if (e >= nb) break;
        start[e] = tw * t;
        for (int c = 0; c < count[e]; c += tw, t++) {
            out[1 + 2 * t] = e < n_expert ? e : -1;
            out[2 + 2 * t] = tw * t;
        }
        count[e] = 0;  // reused as the fill cursor
    }
    __syncthreads();
    for (int p0 = tid; p0 < pairs; p0 += 8 * 1024) {
        int e[8];
#pragma unroll
        for (int j = 0; j < 8; j++) e[j] = p0 == tid ? first[j] : p0 + 1024 * j < pairs ? ids[p0 + 1024 * j] : -1;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int p = p0 + 1024 * j;
            if (p >= pairs) break;
            const int eb = (e[j] < 0 || e[j] >= n_expert) ? n_expert : e[j];
            const int row = start[eb] + atomicAdd(&count[eb], 1);
            const int tok = p / n_used, slot = p - tok * n_used;
            src_col[row] = tok * b_cols + slot % b_cols;
            out_pair[row] = p;
        }
    }
}

// The same sort for many pairs, spread over workgroups of SORT_CHUNK pairs each:
//   count: every workgroup histograms its chunk (and clears its share of the row tables);
//   plan:  one workgroup turns the histograms into the tile table and, per chunk and expert, the first
//          sorted row that chunk's pairs of that expert go to;
//   place: every workgroup hands its pairs their rows.
constexpr int SORT_CHUNK = 2048, SORT_MAX_CHUNKS = 256;

__global__ __launch_bounds__(1024) void sort_count_kernel(const int *__restrict__ ids, int pairs, int n_expert, int table_rows,
                                                           int *__restrict__ hist, int *__restrict__ src_col,
                                                           int *__restrict__ out_pair) {
    __shared__ int count[ID_MAX_EXPERTS + 1];
    const int nb = n_expert + 1, tid = threadIdx.x;
    for (int e = tid; e < nb; e += 1024) count[e] = 0;
    for (int r = blockIdx.x * 1024 + tid; r < table_rows; r += gridDim.x * 1024) { src_col[r] = -1; out_pair[r] = -1; }
    __syncthreads();
    const int p0 = blockIdx.x * SORT_CHUNK + tid;
    int e[SORT_CHUNK / 1024];
#pragma unroll
    for (int j = 0; j < SORT_CHUNK / 1024; j++) e[j] = p0 + 1024 * j < pairs ? ids[p0 + 1024 * j] : -1;
#pragma unroll
    for (int j = 0; j < SORT_CHUNK / 1024; j++)
        if (p0 + 1024 * j < pairs) atomicAdd(&count[(e[j] < 0 || e[j] >= n_expert) ? n_expert : e[j]], 1);
    __syncthreads();
    for (int x = tid; x < nb; x += 1024) hist[(size_t)blockIdx.x * nb + x] = count[x];
}

__global__ __launch_bounds__(1024) void sort_plan_kernel(int n_expert, int chunks, int tw, int *__restrict__ hist, int *__restrict__ out) {
    __shared__ int scan[2][1024];
    const int nb = n_expert + 1, tid = threadIdx.x;
    constexpr int PER = (ID_MAX_EXPERTS + 1 + 1023) / 1024;
    int total[PER], mine = 0;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int e = PER * tid + j;
        total[j] = 0;
        if (e < nb)
            for (int c = 0; c < chunks; c++) total[j] += hist[(size_t)c * nb + e];
        mine += (total[j] + tw - 1) / tw;
    }
    scan[0][tid] = mine;
    __syncthreads();
    int cur = 0;
    for (int step = 1; step < 1024; step <<= 1, cur ^= 1) {
        scan[cur ^ 1][tid] = scan[cur][tid] + (tid >= step ? scan[cur][tid - step] : 0);
        __syncthreads();
    }
    int t = scan[cur][tid] - mine;
    if (tid == 1023) out[0] = scan[cur][tid];
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int e = PER * tid + j;
        if (e >= nb) break;
        int row = tw * t;  // first sorted row of the expert; the chunks' pairs follow one another
        for (int c = 0; c < chunks; c++) {
            const int n = hist[(size_t)c * nb + e];
            hist[(size_t)c * nb + e] = row;
            row += n;
        }
        for (int c = 0; c < total[j]; c += tw, t++) {
            out[1 + 2 * t] = e < n_expert ? e : -1;
            out[2 + 2 * t] = tw * t;
        }
    }
}

__global__ __launch_bounds__(1024) void sort_place_kernel(const int *__restrict__ ids, int pairs, int n_expert, int n_used,
                                                           int b_cols, const int *__restrict__ base, int *__restrict__ src_col,
                                                           int *__restrict__ out_pair) {
    __shared__ int next[ID_MAX_EXPERTS + 1];
    const int nb = n_expert + 1, tid = threadIdx.x;
    for (int e = tid; e < nb; e += 1024) next[e] = base[(size_t)blockIdx.x * nb + e];
    __syncthreads();
    const int p0 = blockIdx.x * SORT_CHUNK + tid;
    int e[SORT_CHUNK / 1024];
#pragma unroll
    for (int j = 0; j < SORT_CHUNK / 1024; j++) e[j] = p0 + 1024 * j < pairs ? ids[p0 + 1024 * j] : -1;
#pragma unroll
    for (int j = 0; j < SORT_CHUNK / 1024; j++) {
        const int p = p0 + 1024 * j;
        if (p >= pairs) break;
        const int row = atomicAdd(&next[(e[j] < 0 || e[j] >= n_expert) ? n_expert : e[j]], 1);
        const int tok = p / n_used, slot = p - tok * n_used;
        src_col[row] = tok * b_cols + slot % b_cols;
        out_pair[row] = p;
    }
}

// XMODE as in gemv_thin_kernel: 0 quantized planes, 1 f32 rows quantized here, 3 f32 rows through SwiGLU first
// (up: the second operand, laid out like xf).
template <class P, int NC, bool DIRECT, int XMODE, int RPL>
__global__ __launch_bounds__(XMODE ? 1024 : 512) void gemv_id_kernel(IdArgs ia, DevAct a, const float *__restrict__ xf,
                                                      const float *__restrict__ up, int rows_per_wave, int kw, int rw_log2) {
    constexpr bool F32 = XMODE != 0;
    static_assert(XMODE == 0 || XMODE == 1 || XMODE == 3, "RMSNorm is not produced here");
    static_assert(!F32 || NC == 1, "the f32 prologue quantizes one activation row");
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int REC = 2 + NC;
    // the argument block in one batch of scalar loads, as in gemv_thin_kernel: the branches below would
    // otherwise each be followed by a round of their own
    gbytes_t p0a = (gbytes_t)ia.w.p0, p0b = (gbytes_t)ia.p0b;
    gfloats_t ya = (gfloats_t)ia.y, yb = (gfloats_t)ia.yb;
    gcints_t ids = (gcints_t)ia.ids, groups = (gcints_t)ia.groups;
    gcfloats_t xg = (gcfloats_t)xf, upg = (gcfloats_t)up;
    int64_t M = ia.M, Kall = ia.w.K;
    int n_expert = ia.n_expert, n_used = ia.n_used, b_cols = ia.b_cols, wgs_per_group = ia.wgs_per_group, wgs_first = ia.wgs_first;
    asm volatile("" : "+s"(p0a), "+s"(p0b), "+s"(ya), "+s"(yb), "+s"(ids), "+s"(groups), "+s"(xg), "+s"(upg), "+s"(M), "+s"(Kall),
                      "+s"(n_expert), "+s"(n_used), "+s"(b_cols), "+s"(wgs_per_group), "+s"(wgs_first), "+s"(rows_per_wave), "+s"(kw),
                      "+s"(rw_log2));
    xf = (const float *)xg;
    up = (const float *)upg;
    const bool second = (int)blockIdx.x >= wgs_first;
    const int bid = (int)blockIdx.x - (second ? wgs_first : 0);
    const DevWeight w{(const uint8_t *)(second ? p0b : p0a), second ? ia.p1b : ia.w.p1, second ? ia.p2b : ia.w.p2,
                      second ? ia.db : ia.w.d, Kall, ia.w.M, ia.w.type};
    float *__restrict__ y = (float *)(second ? yb : ya);
    const int group = bid / wgs_per_group, wg = bid - group * wgs_per_group;
    int expert, count, pair[NC];
    if (groups) {
        if (group >= groups[0]) return;
        gcints_t rec = groups + 1 + (size_t)group * REC;
        expert = rec[0];
        count = rec[1];
#pragma unroll
        for (int n = 0; n < NC; n++) pair[n] = rec[2 + min(n, count - 1)];
    } else {
        expert = ids[group];
        if (expert < 0 || expert >= n_expert) expert = -1;
        count = 1;
#pragma unroll
        for (int n = 0; n < NC; n++) pair[n] = group;
    }
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rw = 1 << rw_log2;
    const int rg = wave & (rw - 1), kseg = wave >> rw_log2;
    const int rows_per_wg = rows_per_wave << rw_log2;
    const int64_t r0 = (int64_t)wg * rows_per_wg;  // row inside the expert
    const int nrows = (int)min((int64_t)rows_per_wg, M - r0);
    if (expert < 0) {
        // an id outside the stack: the pair's output is all NaN
        for (int i = threadIdx.x; i < nrows * count; i += (kw << rw_log2) * 64) {
            const int n = i / nrows, rl = i - n * nrows;
            y[(int64_t)pair[n] * M + r0 + rl] = __int_as_float(0x7fc00000);
        }
        return;
    }
    const int rl0 = rg * rows_per_wave;
    const int nrw = max(0, min(rows_per_wave, nrows - rl0));
    const int64_t wrow0 = (int64_t)expert * M + r0 + rl0;  // row inside the stack

    const int vlane = lane & (64 / RPL - 1), run = RPL == 1 ? 0 : lane / (64 / RPL);
    const typename P::Geo g = P::geo(w, kseg, vlane);
    int col[NC];  // activation row of each pair: token * b_cols + slot mod b_cols
#pragma unroll
    for (int n = 0; n < NC; n++) {
        const int tok = pair[n] / n_used, slot = pair[n] - tok * n_used;
        col[n] = tok * b_cols + slot % b_cols;
    }
    const int64_t K = w.K;
    const int nblk = (int)(K / P::ACT_BLK);
    const size_t act_bytes = F32 ? ((size_t)(K + nblk * 4 + (P::USES_BSUMS ? K / P::ACT_BSUM * 2 : 0)) + 15) / 16 * 16 : 0;
    int8_t *lqs = reinterpret_cast<int8_t *>(smem);
    float *ld_ = reinterpret_cast<float *>(smem + K);
    int16_t *lbs = reinterpret_cast<int16_t *>(smem + K + (size_t)nblk * 4);
    const float4 *x4 = reinterpret_cast<const float4 *>(xf + (int64_t)col[0] * K);
    const int total4 = (int)(K / 4), nwaves = kw << rw_log2 /* = (kw << rw_log2) * 64 / 64, without the hidden-argument load */;
    float4 xpre[XPRE], apre[XPRE];
    if (F32) prefetch_x(x4, total4, wave, nwaves, lane, xpre);
    if (XMODE == 3) prefetch_x(reinterpret_cast<const float4 *>(up + (int64_t)col[0] * K), total4, wave, nwaves, lane, apre);
    typename P::Raw cur;
    if (nrw > 0) cur = P::load(w, g, wrow0 + min(run, nrw - 1));
    if (XMODE == 3) {  // the whole row sits in the prefetch registers (the launcher checked)
#pragma unroll
        for (int j = 0; j < XPRE; j++) xpre[j] = swiglu_apply(xpre[j], apre[j]);
    }
    if (F32) {
        quantize_x_to_lds<P, XPRE>(x4, total4, wave, nwaves, lane, xpre, lqs, ld_, lbs);
        __syncthreads();
    }
    float *part = reinterpret_cast<float *>(smem + act_bytes);
    if (nrw > 0) {
        typename P::Act act[NC];
        if (F32) {
            const LdsAct la{lqs, ld_, lbs, K};
            P::load_act(la, 0, kseg, vlane, g, act[0]);
        } else {
#pragma unroll
            for (int n = 0; n < NC; n++) P::load_act(a, col[n], kseg, vlane, g, act[n]);
        }
        float keep[NC];
        thin_rows<P, NC, DIRECT, RPL>(w, g, cur, act, wrow0, nrw, lane, keep, part, rl0, kw, kseg);
        if (DIRECT && lane > 63 - nrw) {
#pragma unroll
            for (int n = 0; n < NC; n++)
                if (n < count) y[(int64_t)pair[n] * M + r0 + rl0 + (63 - lane)] = keep[n];
        }
    }
    if (DIRECT) return;
    __syncthreads();
    for (int i = threadIdx.x; i < nrows * count; i += (kw << rw_log2) * 64) {
        const int n = i / nrows, rl = i - n * nrows;
        float sum = 0.f;
        for (int k = 0; k < kw; k++) sum += part[(rl * NC + n) * kw + k];
        y[(int64_t)pair[n] * M + r0 + rl] = sum;
    }
}

// Gate and up of an expert feed-forward block at decode size with the gating in the epilogue (see
// gemv_pair_kernel): one (token, slot) pair per group of workgroups, the wave walks row j of the pair's expert
// in both stacks, h[pair][j] = silu(gate total) * up total.  ia.w / ia.p0b.. are the gate / up stacks, ia.y is h.
template <class P, bool DIRECT, int RPL>
__global__ __launch_bounds__(512) void gemv_id_pair_kernel(IdArgs ia, const float *__restrict__ xf, int rows_per_wave, int kw,
                                                           int rw_log2) {
    extern __shared__ __align__(16) uint8_t smem[];
    // the argument block in one batch of scalar loads, as in gemv_thin_kernel
    gbytes_t p0a = (gbytes_t)ia.w.p0, p0b = (gbytes_t)ia.p0b;
    gfloats_t ya = (gfloats_t)ia.y;
    gcints_t ids = (gcints_t)ia.ids;
    gcfloats_t xg = (gcfloats_t)xf;
    int64_t M = ia.M, Kall = ia.w.K;
    int n_expert = ia.n_expert, n_used = ia.n_used, b_cols = ia.b_cols, wgs_per_group = ia.wgs_per_group;
    asm volatile("" : "+s"(p0a), "+s"(p0b), "+s"(ya), "+s"(ids), "+s"(xg), "+s"(M), "+s"(Kall), "+s"(n_expert), "+s"(n_used),
                      "+s"(b_cols), "+s"(wgs_per_group), "+s"(rows_per_wave), "+s"(kw), "+s"(rw_log2));
    xf = (const float *)xg;
    const DevWeight wa{(const uint8_t *)p0a, ia.w.p1, ia.w.p2, ia.w.d, Kall, ia.w.M, ia.w.type};
    const DevWeight wb{(const uint8_t *)p0b, ia.p1b, ia.p2b, ia.db, Kall, ia.w.M, ia.w.type};
    float *__restrict__ hout = (float *)ya;
    const int pair = (int)blockIdx.x / wgs_per_group, wg = (int)blockIdx.x - pair * wgs_per_group;
    int expert = ids[pair];
    if (expert < 0 || expert >= n_expert) expert = -1;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rw = 1 << rw_log2;
    const int rg = wave & (rw - 1), kseg = wave >> rw_log2;
    const int rows_per_wg = rows_per_wave << rw_log2;  // rows of h per workgroup
    const int64_t r0 = (int64_t)wg * rows_per_wg;
    const int nrows = (int)min((int64_t)rows_per_wg, M - r0);
    if (expert < 0) {
        for (int i = threadIdx.x; i < nrows; i += (kw << rw_log2) * 64) hout[(int64_t)pair * M + r0 + i] = __int_as_float(0x7fc00000);
        return;
    }
    const int rl0 = rg * rows_per_wave;
    const int nrw = max(0, min(rows_per_wave, nrows - rl0));
    const int64_t wrow0 = (int64_t)expert * M + r0 + rl0;
    const int vlane = lane & (64 / RPL - 1), run = RPL == 1 ? 0 : lane / (64 / RPL);
    const typename P::Geo g = P::geo(wa, kseg, vlane);
    const int tok = pair / n_used, slot = pair - tok * n_used;
    const int col = tok * b_cols + slot % b_cols;

    const int64_t K = wa.K;
    const int nblk = (int)(K / P::ACT_BLK);
    const size_t act_bytes = ((size_t)(K + nblk * 4 + (P::USES_BSUMS ? K / P::ACT_BSUM * 2 : 0)) + 15) / 16 * 16;
    int8_t *lqs = reinterpret_cast<int8_t *>(smem);
    float *ld_ = reinterpret_cast<float *>(smem + K);
    int16_t *lbs = reinterpret_cast<int16_t *>(smem + K + (size_t)nblk * 4);
    const float4 *x4 = reinterpret_cast<const float4 *>(xf + (int64_t)col * K);
    const int total4 = (int)(K / 4), nwaves = kw << rw_log2 /* = (kw << rw_log2) * 64 / 64, without the hidden-argument load */;
    float4 xpre[XPRE];
    prefetch_x(x4, total4, wave, nwaves, lane, xpre);
    typename P::Raw cur;
    if (nrw > 0) {
        const int v = min(run, 2 * nrw - 1);
        cur = P::load(v & 1 ? wb : wa, g, wrow0 + (v >> 1));
    }
    quantize_x_to_lds<P, XPRE>(x4, total4, wave, nwaves, lane, xpre, lqs, ld_, lbs);
    __syncthreads();
    float *part = reinterpret_cast<float *>(smem + act_bytes);
    if (nrw > 0) {
        typename P::Act act[1];
        const LdsAct la{lqs, ld_, lbs, K};
        P::load_act(la, 0, kseg, vlane, g, act[0]);
        float keep;
        thin_rows_pair<P, DIRECT, RPL>(wa, wb, g, cur, act, wrow0, 2 * nrw, lane, keep, part, 2 * rl0, kw, kseg);
        if (DIRECT) {
            const float up = dpp_mov<0xB1>(keep);
            if ((lane & 1) && lane > 63 - 2 * nrw) hout[(int64_t)pair * M + r0 + rl0 + ((63 - lane) >> 1)] = silu_mul(keep, up);
        }
    }
    if (DIRECT) return;
    __syncthreads();
    for (int i = threadIdx.x; i < nrows; i += (kw << rw_log2) * 64) {
        float gsum = 0.f, usum = 0.f;
        for (int k = 0; k < kw; k++) gsum += part[(2 * i) * kw + k];
        for (int k = 0; k < kw; k++) usum += part[(2 * i + 1) * kw + k];
        hout[(int64_t)pair * M + r0 + i] = silu_mul(gsum, usum);
    }
}

// The plan of an expert-indexed launch whose workgroups quantize x themselves (decode: a group of workgroups per pair).
// Every workgroup reads and quantizes a whole activation row before its first weights, so a workgroup of four waves with
// two rows each (the plan for quantized planes) reads more activation bytes than weight bytes.  Instead, as for the plain
// product on f32 rows: sixteen waves (max_waves) and one workgroup per CU, rows per wave to match, at least four -- where
// that leaves fewer than 160 workgroups, eight waves and about three workgroups per CU (one where rows are cut into four
// or more segments).  Measured, one token, us: MXFP4 32 x (2880 x 2880) top-4 17.0 -> 11.3, (5760 x 2880) 27.5 -> 16.1
// (14.8 with the cheaper decoding of the codes); Q8_0 (2880 x 2880) 17.6 -> 8.5; Q4_K (2880 x 4096) top-4 10.2 -> 7.8,
// 8 x (14336 x 4096) top-2 20.0 -> 12.6, 8 x (4096 x 14336) top-2 50.1 -> 15.1; 128 x (768 x 2048) top-8 5.0 -> 4.7.
// A row's sum does not depend on the plan.
template <class P>
void retune_id_plan(Plan &p, int64_t total_rows, int nc, int max_waves) {
    auto shape = [&](int waves, int64_t wgs) {
        p.rw_log2 = 0;
        while (p.kw << (p.rw_log2 + 1) <= waves) p.rw_log2++;
        p.rw = 1 << p.rw_log2;
        int64_t rows = (total_rows + wgs * p.rw - 1) / (wgs * p.rw);
        rows = (rows + 1) / 2 * 2;
        if (rows < 4) rows = 4;
        if (p.rpl > 1) rows = max((int64_t)2 * p.rpl, (rows + p.rpl - 1) / p.rpl * p.rpl);
        if (rows > 16) rows = 16;  // a wave parks its row totals in lanes 63, 62, ...
        p.rows_per_wg = p.rw * (int)rows;
    };
    shape(max_waves, 256);
    if (max_waves <= 8 || p.kw > max_waves || total_rows / p.rows_per_wg < 160) shape(p.kw > 8 ? p.kw : 8, p.kw >= 4 ? 256 : 768);
    p.lds = p.kw == 1 ? 0 : (size_t)p.rows_per_wg * nc * p.kw * sizeof(float) + 64;
}

template <class P>
hipError_t launch_id_pair(IdArgs ia, const float *xf, hipStream_t s) {
    Plan p;
    if (!make_thin_plan<P>(ia.w.K, (int64_t)ia.pairs * ia.M * 2, 1, false, p)) return hipErrorInvalidValue;
    retune_id_plan<P>(p, (int64_t)ia.pairs * ia.M * 2, 1, 8);
    const size_t act_lds = thin_act_lds<P>(ia.w.K, 1);
    const int rpw_v = p.rows_per_wg >> p.rw_log2;  // virtual rows per wave: row j of gate and of up alternate
    if (act_lds + p.lds > THIN_LDS_MAX || (rpw_v & 1)) return hipErrorInvalidValue;
    const int rows_per_wg = p.rows_per_wg / 2;
    const int64_t wgs_per_group = (ia.M + rows_per_wg - 1) / rows_per_wg;
    if (wgs_per_group * ia.pairs > 0x7fffffff) return hipErrorInvalidValue;
    ia.wgs_per_group = (int)wgs_per_group;
    ia.groups = nullptr;
    const dim3 grid((unsigned)(wgs_per_group * ia.pairs)), block(64 * p.kw * p.rw);
    const size_t lds = act_lds + p.lds;
#define IDP_LAUNCH(DIRECT, RPL) gemv_id_pair_kernel<P, DIRECT, RPL><<<grid, block, lds, s>>>(ia, xf, rpw_v / 2, p.kw, p.rw_log2)
    if (p.kw > 1) IDP_LAUNCH(false, 1);
    else if (p.rpl == 4) IDP_LAUNCH(true, 4);
    else if (p.rpl == 2) IDP_LAUNCH(true, 2);
    else IDP_LAUNCH(true, 1);
#undef IDP_LAUNCH
    return hipGetLastError();
}

template <class P, int NC>
hipError_t launch_id_as(IdArgs ia, const DevAct &a, const float *xf, const float *up, int *groups, hipStream_t s) {
    Plan p;
    if (!make_thin_plan<P>(ia.w.K, (int64_t)ia.pairs * ia.M * (ia.yb ? 2 : 1), NC, false, p)) return hipErrorInvalidValue;
    if (xf) retune_id_plan<P>(p, (int64_t)ia.pairs * ia.M * (ia.yb ? 2 : 1), NC, 16);
    const size_t act_lds = xf ? thin_act_lds<P>(ia.w.K, 1) : 0;
    if (xf && (NC != 1 || act_lds + p.lds > THIN_LDS_MAX)) return hipErrorInvalidValue;
    if (up && (!xf || ia.w.K > (int64_t)XPRE * p.kw * p.rw * 256)) return hipErrorInvalidValue;
    const int64_t wgs_per_group = (ia.M + p.rows_per_wg - 1) / p.rows_per_wg;
    int64_t max_groups = ia.pairs;
    if (NC > 1) {
        // every expert (and the bucket of bad ids) ends with at most one partly filled group
        max_groups = min((int64_t)ia.pairs, (int64_t)ia.n_expert + 1 + ia.pairs / NC);
        if (hipError_t e = launch_group_pairs(ia.ids, ia.pairs, ia.n_expert, NC, groups, s)) return e;
        ia.groups = groups;
    } else {
        ia.groups = nullptr;
    }
    const int stacks = ia.yb ? 2 : 1;
    if (wgs_per_group * max_groups * stacks > 0x7fffffff) return hipErrorInvalidValue;
    ia.wgs_per_group = (int)wgs_per_group;
    ia.wgs_first = stacks == 2 ? (int)(wgs_per_group * max_groups) : 0x7fffffff;
    const dim3 grid((unsigned)(wgs_per_group * max_groups * stacks)), block(64 * p.kw * p.rw);
    const int rpw = p.rows_per_wg >> p.rw_log2;
    const size_t lds = act_lds + p.lds;
#define ID_LAUNCH(N, DIRECT, XMODE, RPL) \
    gemv_id_kernel<P, N, DIRECT, XMODE, RPL><<<grid, block, lds, s>>>(ia, a, xf, up, rpw, p.kw, p.rw_log2)
    if (xf && up) {
        if (p.kw > 1) ID_LAUNCH(1, false, 3, 1);
        else if (p.rpl == 4) ID_LAUNCH(1, true, 3, 4);
        else if (p.rpl == 2) ID_LAUNCH(1, true, 3, 2);
        else ID_LAUNCH(1, true, 3, 1);
    } else if (xf) {
        if (p.kw > 1) ID_LAUNCH(1, false, 1, 1);
        else if (p.rpl == 4) ID_LAUNCH(1, true, 1, 4);
        else if (p.rpl == 2) ID_LAUNCH(1, true, 1, 2);
        else ID_LAUNCH(1, true, 1, 1);
    } else {
        if (p.kw > 1) ID_LAUNCH(NC, false, 0, 1);
        else if (p.rpl == 4) ID_LAUNCH(NC, true, 0, 4);
        else if (p.rpl == 2) ID_LAUNCH(NC, true, 0, 2);
        else ID_LAUNCH(NC, true, 0, 1);
    }
#undef ID_LAUNCH
    return hipGetLastError();
}

template <class P>
hipError_t launch_id_type(const IdArgs &ia, const DevAct &a, const float *xf, const float *up, int *groups, hipStream_t s) {
    // few pairs per expert (decode: the experts of a token are all different): nothing to share, one
    // pair per group; otherwise up to eight pairs of an expert per pass over it
    if (xf || !gemv_id_groups(ia.pairs, ia.n_expert)) return launch_id_as<P, 1>(ia, a, xf, up, groups, s);
    return launch_id_as<P, 8>(ia, a, xf, nullptr, groups, s);
}

}  // namespace

size_t gemv_id_scratch_ints(int64_t pairs) { return 1 + (size_t)pairs * (2 + 16); }

hipError_t launch_group_pairs(const int *ids, int pairs, int n_expert, int nc, int *groups, hipStream_t s) {
    if (!ids || !groups || pairs < 1 || n_expert < 1 || n_expert > ID_MAX_EXPERTS) return hipErrorInvalidValue;
    if (nc == 8) group_pairs_kernel<8><<<1, 1024, 0, s>>>(ids, pairs, n_expert, groups);
    else if (nc == 16) group_pairs_kernel<16><<<1, 1024, 0, s>>>(ids, pairs, n_expert, groups);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

// most tiles the sort can emit for tiles of tile_width pairs (every expert's run, and that of the pairs with
// ids outside the stack, ends in one partly filled tile)
int64_t sort_pairs_max_tiles(int64_t pairs, int n_expert, int tile_width) { return pairs / tile_width + n_expert + 2; }

// ints of device scratch behind the row tables for the chunked sort's histograms (0: one workgroup does it all)
size_t sort_pairs_hist_ints(int64_t pairs, int n_expert) {
    const int64_t chunks = (pairs + SORT_CHUNK - 1) / SORT_CHUNK;
    return chunks >= 3 && chunks <= SORT_MAX_CHUNKS ? (size_t)chunks * (n_expert + 1) : 0;
}

hipError_t launch_sort_pairs(const int *ids, int pairs, int n_expert, int n_used, int b_cols, int tile_width, int *tiles,
                             int *src_col, int *out_pair, int *hist, hipStream_t s) {
    if (!ids || !tiles || !src_col || !out_pair || pairs < 1 || n_expert < 1 || n_expert > ID_MAX_EXPERTS || n_used < 1 ||
        b_cols < 1 || tile_width < 1)
        return hipErrorInvalidValue;
    const int tw = tile_width, max_tiles = (int)sort_pairs_max_tiles(pairs, n_expert, tw);
    if (hist && sort_pairs_hist_ints(pairs, n_expert)) {
        const int chunks = (pairs + SORT_CHUNK - 1) / SORT_CHUNK;
        sort_count_kernel<<<chunks, 1024, 0, s>>>(ids, pairs, n_expert, tw * max_tiles, hist, src_col, out_pair);
        sort_plan_kernel<<<1, 1024, 0, s>>>(n_expert, chunks, tw, hist, tiles);
        sort_place_kernel<<<chunks, 1024, 0, s>>>(ids, pairs, n_expert, n_used, b_cols, hist, src_col, out_pair);
    } else {
        sort_pairs_kernel<<<1, 1024, 0, s>>>(ids, pairs, n_expert, n_used, b_cols, max_tiles, tw, tiles, src_col, out_pair);
    }
    return hipGetLastError();
}

bool gemv_id_groups(int64_t pairs, int n_expert) { return pairs >= 4 * (int64_t)n_expert; }

bool gemv_id_f32_supported(int type, int64_t K, int64_t M, int64_t pairs, int n_expert, bool swiglu) {
    // every workgroup quantizes its pair's activation row again: worth it while the launch is small
    if (gemv_id_groups(pairs, n_expert) || pairs > 64 || K < 1 || K > gemv_max_k(type)) return false;
    Plan p;
    bool ok = false;
    size_t act = 0;
    switch (type) {  // the plan of the launch: activation row plus the partial sums must fit in LDS
    case T_Q4_K: ok = make_thin_plan<PolQ4K>(K, pairs * M, 1, false, p); if (ok) retune_id_plan<PolQ4K>(p, pairs * M, 1, 16); act = thin_act_lds<PolQ4K>(K, 1); break;
    case T_Q5_K: ok = make_thin_plan<PolQ5K>(K, pairs * M, 1, false, p); if (ok) retune_id_plan<PolQ5K>(p, pairs * M, 1, 16); act = thin_act_lds<PolQ5K>(K, 1); break;
    case T_Q6_K: ok = make_thin_plan<PolQ6K>(K, pairs * M, 1, false, p); if (ok) retune_id_plan<PolQ6K>(p, pairs * M, 1, 16); act = thin_act_lds<PolQ6K>(K, 1); break;
    case T_Q4_0: ok = make_thin_plan<PolQ4_0>(K, pairs * M, 1, false, p); if (ok) retune_id_plan<PolQ4_0>(p, pairs * M, 1, 16); act = thin_act_lds<PolQ4_0>(K, 1); break;
    case T_MXFP4: ok = make_thin_plan<PolMXFP4>(K, pairs * M, 1, false, p); if (ok) retune_id_plan<PolMXFP4>(p, pairs * M, 1, 16); act = thin_act_lds<PolMXFP4>(K, 1); break;
    case T_Q8_0: ok = make_thin_plan<PolQ8_0>(K, pairs * M, 1, false, p); if (ok) retune_id_plan<PolQ8_0>(p, pairs * M, 1, 16); act = thin_act_lds<PolQ8_0>(K, 1); break;
    default: break;
    }
    // gated rows must sit in the waves' prefetch registers whole
    if (ok && swiglu && K > (int64_t)XPRE * p.kw * p.rw * 256) return false;
    return ok && act + p.lds <= THIN_LDS_MAX;
}

hipError_t launch_gemv_id_pair(const DevWeight &wg, const DevWeight &wu, int n_expert, const float *xf, const int *ids,
                               int n_used, int n_tokens, int b_cols, float *h, hipStream_t s) {
    if (wg.type != wu.type || wg.K != wu.K || wg.M != wu.M || n_expert < 1 || n_expert > ID_MAX_EXPERTS || wg.M % n_expert ||
        n_used < 1 || n_tokens < 1 || b_cols < 1 || !ids || !h || !xf || (int64_t)n_used * n_tokens > 0x7fffffff / 16 ||
        wg.K < 1 || wg.K > gemv_max_k(wg.type))
        return hipErrorInvalidValue;
    IdArgs ia{};
    ia.w = wg; ia.ids = ids; ia.y = h; ia.M = wg.M / n_expert;
    ia.n_expert = n_expert; ia.pairs = n_used * n_tokens; ia.n_used = n_used; ia.b_cols = b_cols;
    ia.p0b = wu.p0; ia.p1b = wu.p1; ia.p2b = wu.p2; ia.db = wu.d; ia.yb = nullptr; ia.wgs_first = 0x7fffffff;
    switch (wg.type) {
    case T_Q4_K: return launch_id_pair<PolQ4K>(ia, xf, s);
    case T_Q5_K: return launch_id_pair<PolQ5K>(ia, xf, s);
    case T_Q6_K: return launch_id_pair<PolQ6K>(ia, xf, s);
    case T_Q4_0: return launch_id_pair<PolQ4_0>(ia, xf, s);
    case T_MXFP4: return launch_id_pair<PolMXFP4>(ia, xf, s);
    case T_Q8_0: return launch_id_pair<PolQ8_0>(ia, xf, s);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_gemv_id(const DevWeight &w, int n_expert, const DevAct &a, const float *xf, const int *ids,
                          int n_used, int n_tokens, int b_cols, float *y, int *groups, hipStream_t s,
                          const DevWeight *w2, float *y2, const float *up) {
    if ((w2 != nullptr) != (y2 != nullptr) || (w2 && (w2->type != w.type || w2->K != w.K || w2->M != w.M)))
        return hipErrorInvalidValue;
    if (n_expert < 1 || n_expert > ID_MAX_EXPERTS || w.M % n_expert || n_used < 1 || n_tokens < 1 || b_cols < 1 || !ids || !y || !groups || a.K != w.K || a.N != (int64_t)b_cols * n_tokens ||
        (int64_t)n_used * n_tokens > 0x7fffffff / 16)
        return hipErrorInvalidValue;
    if (w.K < 1 || w.K > gemv_max_k(w.type)) return hipErrorInvalidValue;
    IdArgs ia{};
    ia.w = w; ia.ids = ids; ia.y = y; ia.M = w.M / n_expert;
    ia.n_expert = n_expert; ia.pairs = n_used * n_tokens; ia.n_used = n_used; ia.b_cols = b_cols;
    if (w2) { ia.p0b = w2->p0; ia.p1b = w2->p1; ia.p2b = w2->p2; ia.db = w2->d; ia.yb = y2; }
    switch (w.type) {
    case T_Q4_K: return a.type == T_Q8_K ? launch_id_type<PolQ4K>(ia, a, xf, up, groups, s) : hipErrorInvalidValue;
    case T_Q5_K: return a.type == T_Q8_K ? launch_id_type<PolQ5K>(ia, a, xf, up, groups, s) : hipErrorInvalidValue;
    case T_Q6_K: return a.type == T_Q8_K ? launch_id_type<PolQ6K>(ia, a, xf, up, groups, s) : hipErrorInvalidValue;
    case T_Q4_0: return a.type == T_Q8_0 ? launch_id_type<PolQ4_0>(ia, a, xf, up, groups, s) : hipErrorInvalidValue;
    case T_MXFP4: return a.type == T_Q8_0 ? launch_id_type<PolMXFP4>(ia, a, xf, up, groups, s) : hipErrorInvalidValue;
    case T_Q8_0: return a.type == T_Q8_0 ? launch_id_type<PolQ8_0>(ia, a, xf, up, groups, s) : hipErrorInvalidValue;
    default: return hipErrorInvalidValue;
    }
}

}  // namespace miqmm
