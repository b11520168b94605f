// Kernels 2 and 4: streaming decode GEMV / skinny GEMM (1..8 activation columns) for GGUF
// Q4_0, Q8_0, Q4_K and the Q6_K output head.
//
// Computes y[n][m] = vec_dot(W row m, Q8(x row n)) with ggml's CPU-backend semantics (integer block
// dot products, scales applied in fp32) -- the work behind Tensor.Mulmat,
// /root/reference/ml/backend.go:151, for batch <= 8.
//
// Shape of the computation (HBM-bound: every weight byte is read exactly once):
//   * A wavefront owns a fixed slice of K ("segment": 2048 elements, 1024 for Q8_0) and walks down
//     the rows.  Each lane's piece of every row is one aligned 16-byte load, consecutive lanes read
//     consecutive 16-byte pieces, so a wave reads 1 KiB runs of the row.
//   * Because the lane's K positions never change, its Q8 activation quants (and the block scale and
//     partial sums that go with them) are loaded ONCE into registers and reused for every row: the
//     inner loop reads nothing but weights.
//   * Nibbles / 6-bit values are unpacked in registers, multiplied with v_dot4_i32_i8, the sub-block
//     scales applied in-lane, and the lane partials reduced across the wave; waves that own different
//     K segments of the same rows combine through LDS at the end of the workgroup.
//   * U rows are in flight per wave (all loads issued before the first use) to cover HBM latency.
#include <hip/hip_fp16.h>

#include "internal.h"

namespace miqmm {

namespace {

constexpr int MAXC = 8;  // activation columns per launch

__device__ __forceinline__ int dot4(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }

__device__ __forceinline__ float h2f(unsigned int bits16) {
    return __half2float(__ushort_as_half((unsigned short)bits16));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

__device__ __forceinline__ uint4 ld16(const uint8_t *p) { return *reinterpret_cast<const uint4 *>(p); }

// ---------------------------------------------------------------------------------------------
// Per-type policies.  Each provides
//   SEG                      elements of K one wave covers per row
//   Geo                      per-lane constants (offsets into the row, shifts, validity)
//   Act                      per-lane, per-column activation registers
//   Raw                      the lane's loaded weight bytes for one row
//   geo(), load_act(), load(), dot()
// A lane whose K slice lies beyond K (ragged last segment) is "dead": its activation registers are
// zero and its weight loads are redirected to the start of the row, so it contributes exactly 0.
// ---------------------------------------------------------------------------------------------

struct PolQ4K {
    static constexpr int SEG = 2048;  // 8 super-blocks, 8 lanes each
    struct Geo {
        int64_t row_bytes;
        int off;      // byte offset of the lane's super-block in the row
        int l8;       // lane within the super-block: chunk c = l8>>1 (32 qs bytes), half = l8&1
        int sh16;     // 16*(c&1): position of the (sc[2c], sc[2c+1]) pair inside a scales word
        int sh8;      // 8*(l8&3): position of m[l8] inside a scales word
        bool live;
    };
    struct Act { int q[8]; float d; int s; };
    struct Raw { uint4 hdr, qv; };

    static __device__ __forceinline__ Geo geo(const DevWeight &w, int seg, int lane) {
        Geo g;
        const int sb = seg * 8 + (lane >> 3);
        g.row_bytes = w.K / QKK * Q4_K_BYTES;
        g.live = (int64_t)sb * QKK < w.K;
        g.off = g.live ? sb * Q4_K_BYTES : 0;
        g.l8 = lane & 7;
        g.sh16 = 16 * ((g.l8 >> 1) & 1);
        g.sh8 = 8 * (g.l8 & 3);
        return g;
    }
    static __device__ __forceinline__ void load_act(const DevAct &a, int n, int seg, int lane, const Geo &g, Act &r) {
        const int sb = seg * 8 + (lane >> 3);
        const int c = g.l8 >> 1, half = g.l8 & 1;
        if (!g.live) {
#pragma unroll
            for (int i = 0; i < 8; i++) r.q[i] = 0;
            r.d = 0.f; r.s = 0;
            return;
        }
        // low nibbles of the lane's 16 qs bytes are elements 64c+16*half.. of sub-block 2c,
        // high nibbles the same offsets of sub-block 2c+1 (32 elements further)
        const int8_t *q = a.qs + (int64_t)n * a.K + (int64_t)sb * QKK + 64 * c + 16 * half;
        const int4 lo = *reinterpret_cast<const int4 *>(q), hi = *reinterpret_cast<const int4 *>(q + 32);
        r.q[0] = lo.x; r.q[1] = lo.y; r.q[2] = lo.z; r.q[3] = lo.w;
        r.q[4] = hi.x; r.q[5] = hi.y; r.q[6] = hi.z; r.q[7] = hi.w;
        r.d = a.d[(int64_t)n * (a.K / QKK) + sb];
        const int16_t *bs = a.bsums + (int64_t)n * (a.K / 16) + (int64_t)sb * 16 + 2 * g.l8;
        r.s = (int)bs[0] + (int)bs[1];  // sum of q8 over sub-block l8 (the lane owns min l8)
    }
    static __device__ __forceinline__ Raw load(const DevWeight &w, const Geo &g, int64_t row) {
        const uint8_t *p = w.p0 + row * g.row_bytes + g.off;
        Raw r;
        r.hdr = ld16(p);
        r.qv = ld16(p + 16 + 16 * g.l8);
        return r;
    }
    template <int NC>
    static __device__ __forceinline__ void dot(const Raw &r, const Geo &g, const Act (&a)[NC], float (&acc)[NC]) {
        // hdr.x = d | dmin<<16 ; hdr.y = scales[0..3] ; hdr.z = scales[4..7] ; hdr.w = scales[8..11]
        const float dw = h2f(r.hdr.x & 0xffff), dminw = h2f(r.hdr.x >> 16);
        // (sc[2c], sc[2c+1]) as two bytes
        const unsigned t0 = r.hdr.y >> g.sh16, t2 = r.hdr.w >> g.sh16;
        const unsigned pairA = t0 & 0x3f3fu;
        const unsigned pairB = (t2 & 0x0f0fu) | ((t0 >> 2) & 0x3030u);
        const unsigned pair = (g.l8 < 4) ? pairA : pairB;
        const int sc_lo = pair & 0xff, sc_hi = pair >> 8;
        // m[l8]
        const unsigned ma = r.hdr.z >> g.sh8, mb = r.hdr.w >> g.sh8;
        const int mA = ma & 63, mB = ((mb >> 4) & 0xf) | ((ma >> 2) & 0x30);
        const int mn = (g.l8 < 4) ? mA : mB;
        const unsigned v[4] = {r.qv.x, r.qv.y, r.qv.z, r.qv.w};
        int lo[4], hi[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            lo[i] = (int)(v[i] & 0x0f0f0f0fu);
            hi[i] = (int)((v[i] >> 4) & 0x0f0f0f0fu);
        }
#pragma unroll
        for (int n = 0; n < NC; n++) {
            int dl = 0, dh = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                dl = dot4(lo[i], a[n].q[i], dl);
                dh = dot4(hi[i], a[n].q[4 + i], dh);
            }
            const int isum = __mul24(sc_lo, dl) + __mul24(sc_hi, dh);
            acc[n] += (dw * a[n].d) * (float)isum - (dminw * a[n].d) * (float)__mul24(mn, a[n].s);
        }
    }
};

struct PolQ4_0 {
    static constexpr int SEG = 2048;  // 64 blocks, one per lane
    struct Geo { int64_t qrow, drow; int blk; bool live; };
    struct Act { int q[8]; float d; int s8; };
    struct Raw { uint4 qv; unsigned short dh; };

    static __device__ __forceinline__ Geo geo(const DevWeight &w, int seg, int lane) {
        Geo g;
        const int blk = seg * 64 + lane;
        g.live = (int64_t)blk * QK < w.K;
        g.blk = g.live ? blk : 0;
        g.qrow = w.K / 2;
        g.drow = w.K / QK;
        return g;
    }
    static __device__ __forceinline__ void load_act(const DevAct &a, int n, int seg, int lane, const Geo &g, Act &r) {
        if (!g.live) {
#pragma unroll
            for (int i = 0; i < 8; i++) r.q[i] = 0;
            r.d = 0.f; r.s8 = 0;
            return;
        }
        const int8_t *q = a.qs + (int64_t)n * a.K + (int64_t)g.blk * QK;
        const int4 lo = *reinterpret_cast<const int4 *>(q), hi = *reinterpret_cast<const int4 *>(q + 16);
        r.q[0] = lo.x; r.q[1] = lo.y; r.q[2] = lo.z; r.q[3] = lo.w;
        r.q[4] = hi.x; r.q[5] = hi.y; r.q[6] = hi.z; r.q[7] = hi.w;
        r.d = a.d[(int64_t)n * (a.K / QK) + g.blk];
        r.s8 = 8 * (int)a.bsums[(int64_t)n * (a.K / QK) + g.blk];
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

struct PolQ8_0 {
    static constexpr int SEG = 1024;  // 32 blocks, two lanes (16 quants each) per block
    struct Geo { int64_t qrow, drow; int hb; bool live; };
    struct Act { int q[4]; float d; };
    struct Raw { uint4 qv; unsigned short dh; };

    static __device__ __forceinline__ Geo geo(const DevWeight &w, int seg, int lane) {
        Geo g;
        const int hb = seg * 64 + lane;  // half-block index along the row
        g.live = (int64_t)hb * 16 < w.K;
        g.hb = g.live ? hb : 0;
        g.qrow = w.K;
        g.drow = w.K / QK;
        return g;
    }
    static __device__ __forceinline__ void load_act(const DevAct &a, int n, int seg, int lane, const Geo &g, Act &r) {
        if (!g.live) {
            r.q[0] = r.q[1] = r.q[2] = r.q[3] = 0; r.d = 0.f;
            return;
        }
        const int4 v = *reinterpret_cast<const int4 *>(a.qs + (int64_t)n * a.K + (int64_t)g.hb * 16);
        r.q[0] = v.x; r.q[1] = v.y; r.q[2] = v.z; r.q[3] = v.w;
        r.d = a.d[(int64_t)n * (a.K / QK) + (g.hb >> 1)];
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
    static constexpr int SEG = 2048;  // 8 super-blocks, 8 lanes each
    // lane (h = l8>>2, t = l8&3) of a super-block reads ql bytes [64h+16t, +16): their low nibbles are
    // elements 128h + eo + i, their high nibbles elements 128h + eo + 64 + i, eo = 16(t&1) + 32(t>>1);
    // the two high bits come from qh bytes [32h + 16(t&1), +16) at bit 2(t>>1) (low) and +4 (high).
    struct Geo {
        int64_t lrow, hrow, srow, drow;
        int sb, loff, hoff, soff;
        int shl;  // 4 - 2(t>>1): left shift that brings the low element's 2 bits to bit 4
        int shr;  // 2(t>>1):     right shift that brings the high element's 2 bits to bit 4
        bool live;
    };
    struct Act { int q[8]; float d; int s_lo, s_hi; };
    struct Raw { uint4 ql, qh; int sc_lo, sc_hi; unsigned short dh; };

    static __device__ __forceinline__ Geo geo(const DevWeight &w, int seg, int lane) {
        Geo g;
        const int sb = seg * 8 + (lane >> 3), l8 = lane & 7, h = l8 >> 2, t = l8 & 3;
        g.live = (int64_t)sb * QKK < w.K;
        g.sb = g.live ? sb : 0;
        g.lrow = w.K / 2; g.hrow = w.K / 4; g.srow = w.K / 16; g.drow = w.K / QKK;
        g.loff = g.sb * 128 + 64 * h + 16 * t;
        g.hoff = g.sb * 64 + 32 * h + 16 * (t & 1);
        g.soff = g.sb * 16 + 8 * h + t;
        g.shl = 4 - 2 * (t >> 1);
        g.shr = 2 * (t >> 1);
        return g;
    }
    static __device__ __forceinline__ void load_act(const DevAct &a, int n, int seg, int lane, const Geo &g, Act &r) {
        // dead lanes read super-block 0 (always present) and zero what they read
        const int l8 = lane & 7, h = l8 >> 2, t = l8 & 3;
        const int e0 = 128 * h + 16 * (t & 1) + 32 * (t >> 1);
        const int8_t *q = a.qs + (int64_t)n * a.K + (int64_t)g.sb * QKK + e0;
        const int4 lo = *reinterpret_cast<const int4 *>(q), hi = *reinterpret_cast<const int4 *>(q + 64);
        const int keep = g.live ? -1 : 0;
        r.q[0] = lo.x & keep; r.q[1] = lo.y & keep; r.q[2] = lo.z & keep; r.q[3] = lo.w & keep;
        r.q[4] = hi.x & keep; r.q[5] = hi.y & keep; r.q[6] = hi.z & keep; r.q[7] = hi.w & keep;
        const float dd = a.d[(int64_t)n * (a.K / QKK) + g.sb];
        r.d = g.live ? dd : 0.f;
        const int16_t *bs = a.bsums + (int64_t)n * (a.K / 16) + (int64_t)g.sb * 16 + (e0 >> 4);
        const int b0 = bs[0], b4 = bs[4];
        r.s_lo = (32 * b0) & keep;
        r.s_hi = (32 * b4) & keep;
    }
    static __device__ __forceinline__ Raw load(const DevWeight &w, const Geo &g, int64_t row) {
        Raw r;
        r.ql = ld16(w.p0 + row * g.lrow + g.loff);
        r.qh = ld16(w.p1 + row * g.hrow + g.hoff);
        const int8_t *sc = reinterpret_cast<const int8_t *>(w.p2) + row * g.srow + g.soff;
        r.sc_lo = sc[0];
        r.sc_hi = sc[4];
        r.dh = w.d[row * g.drow + g.sb];
        return r;
    }
    template <int NC>
    static __device__ __forceinline__ void dot(const Raw &r, const Geo &g, const Act (&a)[NC], float (&acc)[NC]) {
        const float dw = h2f(r.dh);
        const unsigned l[4] = {r.ql.x, r.ql.y, r.ql.z, r.ql.w};
        const unsigned hq[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
        int lo[4], hi[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            lo[i] = (int)((l[i] & 0x0f0f0f0fu) | ((hq[i] << g.shl) & 0x30303030u));
            hi[i] = (int)(((l[i] >> 4) & 0x0f0f0f0fu) | ((hq[i] >> g.shr) & 0x30303030u));
        }
#pragma unroll
        for (int n = 0; n < NC; n++) {
            int dl = -a[n].s_lo, dh = -a[n].s_hi;  // sum (q-32)*y = sum q*y - 32*sum y
#pragma unroll
            for (int i = 0; i < 4; i++) {
                dl = dot4(lo[i], a[n].q[i], dl);
                dh = dot4(hi[i], a[n].q[4 + i], dh);
            }
            const int isum = __mul24(r.sc_lo, dl) + __mul24(r.sc_hi, dh);
            acc[n] += (dw * a[n].d) * (float)isum;
        }
    }
};

// ---------------------------------------------------------------------------------------------
// The kernel.  Workgroup = KW x RW waves: wave (kseg, rg) owns K segments kseg, kseg+KW, ...
// (SPW of them, held in registers) and rows r0+rg, r0+rg+RW, r0+rg+2RW, ... of the workgroup's row
// range, U of them in flight at a time.  part[] (LDS) receives one partial per (row, column, kseg);
// after a barrier the workgroup sums over kseg and stores y.
// ---------------------------------------------------------------------------------------------
template <class P, int NC, int SPW, int U>
__device__ __forceinline__ void rows_step(const DevWeight &w, const typename P::Geo (&g)[SPW],
                                          const typename P::Act (&act)[SPW][NC], int64_t r, int rw,
                                          int64_t r0, int lane, int kseg, int kw, float *part) {
    typename P::Raw raw[U][SPW];
#pragma unroll
    for (int u = 0; u < U; u++)
#pragma unroll
        for (int s = 0; s < SPW; s++) raw[u][s] = P::load(w, g[s], r + (int64_t)u * rw);
#pragma unroll
    for (int u = 0; u < U; u++) {
        float acc[NC];
#pragma unroll
        for (int n = 0; n < NC; n++) acc[n] = 0.f;
#pragma unroll
        for (int s = 0; s < SPW; s++) P::template dot<NC>(raw[u][s], g[s], act[s], acc);
#pragma unroll
        for (int n = 0; n < NC; n++) acc[n] = wave_sum(acc[n]);
        if (lane == 0) {
            const int rl = (int)(r + (int64_t)u * rw - r0);
#pragma unroll
            for (int n = 0; n < NC; n++) part[(rl * NC + n) * kw + kseg] = acc[n];
        }
    }
}

template <class P, int NC, int SPW, int U>
__global__ __launch_bounds__(512) void gemv_kernel(DevWeight w, DevAct a, int col0, float *__restrict__ y,
                                                    int64_t ldy, int rows_per_wg, int kw, int rw) {
    extern __shared__ float part[];  // [rows_per_wg][NC][kw]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int kseg = wave % kw, rg = wave / kw;
    const int64_t r0 = (int64_t)blockIdx.x * rows_per_wg;
    const int64_t r1 = min(w.M, r0 + (int64_t)rows_per_wg);

    typename P::Geo g[SPW];
    typename P::Act act[SPW][NC];
#pragma unroll
    for (int s = 0; s < SPW; s++) {
        g[s] = P::geo(w, kseg + s * kw, lane);
#pragma unroll
        for (int n = 0; n < NC; n++) P::load_act(a, col0 + n, kseg + s * kw, lane, g[s], act[s][n]);
    }

    int64_t r = r0 + rg;
    for (; r + (int64_t)(U - 1) * rw < r1; r += (int64_t)U * rw)
        rows_step<P, NC, SPW, U>(w, g, act, r, rw, r0, lane, kseg, kw, part);
    for (; r < r1; r += rw)  // fewer than U rows left for this wave
        rows_step<P, NC, SPW, 1>(w, g, act, r, rw, r0, lane, kseg, kw, part);

    __syncthreads();
    const int nrows = (int)(r1 - r0);
    for (int i = threadIdx.x; i < nrows * NC; i += blockDim.x) {
        const int n = i / nrows, rl = i - n * nrows;  // consecutive threads -> consecutive rows
        float s = 0.f;
        for (int k = 0; k < kw; k++) s += part[(rl * NC + n) * kw + k];
        y[(int64_t)(col0 + n) * ldy + r0 + rl] = s;
    }
}

struct Plan { int kw, rw, spw, rows_per_wg; unsigned grid; size_t lds; };

// At most 8 waves per workgroup (two per SIMD, so a wave may use up to 256 VGPRs).
template <class P>
bool make_plan(const DevWeight &w, int nc, int num_cus, Plan &p) {
    const int nseg = (int)((w.K + P::SEG - 1) / P::SEG);
    if (nseg < 1) return false;
    p.spw = nseg <= 8 ? 1 : nseg <= 16 ? 2 : nseg <= 32 ? 4 : nseg <= 64 ? 8 : 0;
    if (!p.spw) return false;
    p.kw = (nseg + p.spw - 1) / p.spw;
    p.rw = 8 / p.kw;
    const int wg_per_cu = 2;  // 16 waves per CU when the kernel fits 128 VGPRs, else 8
    const int64_t target_wgs = (int64_t)num_cus * wg_per_cu;
    int64_t rows = (w.M + target_wgs - 1) / target_wgs;
    const int64_t lds_cap_rows = 8192 / (nc * p.kw);  // <= 32 KiB of partials
    if (rows > lds_cap_rows) rows = lds_cap_rows;
    if (rows < 1) rows = 1;
    p.rows_per_wg = (int)rows;
    p.grid = (unsigned)((w.M + rows - 1) / rows);
    p.lds = (size_t)rows * nc * p.kw * sizeof(float);
    return true;
}

template <class P, int NC, int U>
hipError_t launch_nc(const DevWeight &w, const DevAct &a, int col0, float *y, int64_t ldy, int num_cus,
                     hipStream_t s) {
    Plan p;
    if (!make_plan<P>(w, NC, num_cus, p) || p.spw != 1) return hipErrorInvalidValue;
    const dim3 block(64 * p.kw * p.rw);
    gemv_kernel<P, NC, 1, U><<<p.grid, block, p.lds, s>>>(w, a, col0, y, ldy, p.rows_per_wg, p.kw, p.rw);
    return hipGetLastError();
}

// long rows (more than 8 segments): several segments per wave, one column per launch
template <class P>
hipError_t launch_long(const DevWeight &w, const DevAct &a, int col0, int nc, float *y, int64_t ldy,
                       int num_cus, hipStream_t s) {
    Plan p;
    if (!make_plan<P>(w, 1, num_cus, p)) return hipErrorInvalidValue;
    const dim3 block(64 * p.kw * p.rw);
    for (int c = col0; c < col0 + nc; c++) {
        if (p.spw == 2)
            gemv_kernel<P, 1, 2, 2><<<p.grid, block, p.lds, s>>>(w, a, c, y, ldy, p.rows_per_wg, p.kw, p.rw);
        else if (p.spw == 4)
            gemv_kernel<P, 1, 4, 2><<<p.grid, block, p.lds, s>>>(w, a, c, y, ldy, p.rows_per_wg, p.kw, p.rw);
        else
            gemv_kernel<P, 1, 8, 1><<<p.grid, block, p.lds, s>>>(w, a, c, y, ldy, p.rows_per_wg, p.kw, p.rw);
    }
    return hipGetLastError();
}

template <class P>
hipError_t launch_type(const DevWeight &w, const DevAct &a, int col0, int nc, float *y, int64_t ldy,
                       int num_cus, hipStream_t s) {
    if (w.K > 8 * (int64_t)P::SEG) return launch_long<P>(w, a, col0, nc, y, ldy, num_cus, s);
    switch (nc) {
    case 1: return launch_nc<P, 1, 4>(w, a, col0, y, ldy, num_cus, s);
    case 2: return launch_nc<P, 2, 4>(w, a, col0, y, ldy, num_cus, s);
    case 3: return launch_nc<P, 3, 2>(w, a, col0, y, ldy, num_cus, s);
    case 4: return launch_nc<P, 4, 2>(w, a, col0, y, ldy, num_cus, s);
    case 5: return launch_nc<P, 5, 2>(w, a, col0, y, ldy, num_cus, s);
    case 6: return launch_nc<P, 6, 2>(w, a, col0, y, ldy, num_cus, s);
    case 7: return launch_nc<P, 7, 2>(w, a, col0, y, ldy, num_cus, s);
    case 8: return launch_nc<P, 8, 2>(w, a, col0, y, ldy, num_cus, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

int64_t gemv_max_k(int type) {
    switch (type) {
    case T_Q8_0: return 64 * (int64_t)PolQ8_0::SEG;
    case T_Q4_0: case T_Q4_K: case T_Q6_K: return 64 * (int64_t)2048;
    default: return 0;
    }
}

hipError_t launch_gemv(const DevWeight &w, const DevAct &a, int col0, int ncols, float *y, int64_t ldy,
                       int num_cus, hipStream_t s) {
    if (ncols < 1 || ncols > MAXC || w.M < 1 || w.K < 1 || w.K > gemv_max_k(w.type) || a.K != w.K ||
        col0 < 0 || col0 + ncols > a.N)
        return hipErrorInvalidValue;
    switch (w.type) {
    case T_Q4_K: return a.type == T_Q8_K ? launch_type<PolQ4K>(w, a, col0, ncols, y, ldy, num_cus, s) : hipErrorInvalidValue;
    case T_Q6_K: return a.type == T_Q8_K ? launch_type<PolQ6K>(w, a, col0, ncols, y, ldy, num_cus, s) : hipErrorInvalidValue;
    case T_Q4_0: return a.type == T_Q8_0 ? launch_type<PolQ4_0>(w, a, col0, ncols, y, ldy, num_cus, s) : hipErrorInvalidValue;
    case T_Q8_0: return a.type == T_Q8_0 ? launch_type<PolQ8_0>(w, a, col0, ncols, y, ldy, num_cus, s) : hipErrorInvalidValue;
    default: return hipErrorInvalidValue;
    }
}

}  // namespace miqmm
