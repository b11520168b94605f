// Q4_K and (second half of the file) Q6_K products at a few activation columns (2..8) on large matrices: the bandwidth-bound shape of
// several sequences decoding together -- Tensor.Mulmat (/root/reference/ml/backend.go:151) on the
// feed-forward matrices of a layer with a handful of tokens in flight.
//
// Shape of the kernel: one workgroup of up to sixteen waves per CU, each wave with a lot in flight.
//   * Weights go HBM -> registers directly.  A wave works on a 16-row group; per super-block (16 x 144 bytes) it
//     issues a 4-byte and two 16-byte loads per lane, laid out so that the four lanes of a quad read contiguous
//     bytes of one row (lane = 4 * row + j: dword j of the row's header, its quant bytes [16j, +16) and [64 + 16j, +16)): the memory
//     pipeline is handed whole runs of a row, which matters -- the same bytes requested in the matrix cores'
//     own operand order (consecutive lanes on consecutive rows) stream a quarter slower.  A wave requests a
//     "piece" of four super-blocks at once (twelve loads per lane) and requests a slot of the ring again, for its
//     next piece, as soon as that slot has been multiplied.
//   * One ds_bpermute per register then moves the loaded values to the lanes of the MFMA operand order
//     (lane = 16 * j + row): the crossbar of the LDS does the transposition, no LDS memory is touched.
//   * Activations are the same for every row group, so they live in LDS for the whole launch: copied from the
//     quantized planes by direct-to-LDS copies, or -- f32 input -- quantized to Q8_K by the workgroup itself (the block
//     quantizer of the stand-alone kernel: the same bits), which saves the separate quantization launch.  Either way
//     they are requested before the weights: the memory system serves requests roughly in the order they were made,
//     and a wave of this kernel can queue kilobytes per lane.
//   * Arithmetic: v_mfma_i32_16x16x64_i8 with the weights as B operand, quants unscaled.  Lane (row, j) holds the
//     quant bytes [16j, +16) and [64 + 16j, +16) of its row's super-block; four MFMAs take their low and high
//     nibbles.  In each of them K groups {0, 1} are the two halves of one 32-element sub-block and K groups {2, 3}
//     of another, so the 16 rows of the A operand are 8 columns x those two sub-blocks (row 2c + w is column c
//     restricted to the K groups of sub-block w, zero elsewhere -- the lanes that hold zeros read a zero block of
//     LDS, which costs no instruction).  A lane is left with the partial dot products of two columns with the
//     eight sub-blocks, applies the 6-bit scales with v_mad_i32_i24 and takes the mins term from a fifth MFMA on
//     the block-sum digits.  All integer sums are exact.
//
// Order of the floating-point sums (what makes a result independent of the launch geometry): a row's K is cut
// into pieces of four super-blocks; inside a piece the super-blocks are accumulated in order from zero; the
// piece sums are added in order.  Whichever wave computes a piece, and however many matrices share the launch,
// the bits are the same.
#include <hip/hip_fp16.h>

#include <algorithm>
#include <type_traits>

#include "internal.h"
#include "quant_dev.h"

namespace miqmm {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned u4v __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(1))) uint8_t *gbytes_t;
typedef const __attribute__((address_space(1))) u4v *gu4_t;

__device__ __forceinline__ float h2f(unsigned bits16) { return __half2float(__ushort_as_half((unsigned short)bits16)); }
__device__ __forceinline__ int mad24(int a, int b, int c) { return __mul24(a, b) + c; }
__device__ __forceinline__ v4i mfma16(v4i a, v4i b, v4i c) { return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0); }
__device__ __forceinline__ unsigned lds_addr(const void *p) {
    return (unsigned)(uintptr_t)(const __attribute__((address_space(3))) uint8_t *)p;
}
template <class T>
__device__ __forceinline__ T lds_at(unsigned address, int imm) {
    return *(const __attribute__((address_space(3))) T *)(uintptr_t)(address + (unsigned)imm);
}
// direct-to-LDS copy issued from inline assembly: lane l's BYTES at base + off land at lds_address + BYTES * l
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
__device__ __forceinline__ u4v bperm(int idx, u4v v) {
    u4v o;
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = (unsigned)__builtin_amdgcn_ds_bpermute(idx, (int)v[i]);
    return o;
}

constexpr int DEEP_MULTI = 4;    // matrices per launch
constexpr int PIECE = 4;         // super-blocks per piece
constexpr int MAX_WAVES = 16;    // waves per workgroup (one workgroup per CU)
constexpr int NCT = 8;           // activation columns the LDS layout and the A operand are made for
struct DeepArgs {
    const uint8_t *p0[DEEP_MULTI];
    float *y[DEEP_MULTI];
    int64_t M[DEEP_MULTI];
    int grp_end[DEEP_MULTI];  // exclusive end of each matrix's run of 16-row groups; INT_MAX past the last matrix
    int groups_total, nsb;
};
// how the launch is cut (computed on the host: the kernel's prologue has no division)
struct DeepCut {
    int W, wpg, inv_wpg;  // waves per workgroup; waves that share a row group; ceil(256 / wpg): wave / wpg = wave * inv >> 8
    int Wact;             // waves that stream weights (slots * wpg); waves Wact .. W-1 only help to quantize f32 x and leave
    int inv_nsb;          // ceil(2^20 / nsb): b / nsb = b * inv >> 20 for the block numbers of up to eight columns
    int slots, ppw;       // row groups a workgroup holds at a time; pieces per wave
    int iters, grid;      // row groups per slot; workgroups
};
struct DeepWhere { const uint8_t *p0; float *y; int64_t M; int first; };
__device__ __forceinline__ DeepWhere deep_where(const DeepArgs &g, int group) {
    DeepWhere w{g.p0[0], g.y[0], g.M[0], 0};
#pragma unroll
    for (int t = 1; t < DEEP_MULTI; t++)
        if (group >= g.grp_end[t - 1]) w = DeepWhere{g.p0[t], g.y[t], g.M[t], g.grp_end[t - 1]};
    return w;
}

// LDS map.  512 zero bytes (operand lanes that carry zeros read there); per super-block and column 256 bytes of
// quants in 16-byte pieces, piece p of column c at slot p ^ a_swz(c); per (super-block, column) 16 bytes of block-sum
// digits and the fp32 block scale; then the piece sums [slot][piece][column][row] of workgroups whose waves share
// row groups.
//
// a_swz: ds_read_b128 serves 16 lanes per cycle, lanes 0-3, 12-15 and 20-27 together and lanes 4-11, 16-19 and 28-31
// together (the same in the upper half of the wave).  Of the first group the lanes that read real data are rows
// {0, 2, 12, 14} of K group 0 -- columns 0, 1, 6, 7, piece p -- and rows {4, 6, 8, 10} of K group 1 -- columns 2, 3, 4,
// 5, piece p ^ 1 (of the second group: the same with the column sets exchanged).  With a_swz = 0, 2, 4, 6 inside each
// column set the eight lanes fall on the eight slots of p's aligned block of eight; the lanes that read zeros all read
// one address in the other block.
__device__ __host__ constexpr int a_swz(int col) { return 2 * ((col & 1) + 2 * (col >> 2)) & 6; }
static_assert(a_swz(0) == 0 && a_swz(1) == 2 && a_swz(6) == 4 && a_swz(7) == 6 && a_swz(2) == 0 && a_swz(3) == 2 &&
              a_swz(4) == 4 && a_swz(5) == 6, "column swizzle");
// ncs: the columns the layout holds per super-block, 4 (launches of up to four columns) or 8.
struct DeepGeo {
    static constexpr int A_OFF = 512;
    static __host__ __device__ constexpr int dg_off(int nsb, int ncs) { return A_OFF + nsb * ncs * 256; }
    static __host__ __device__ constexpr int y_off(int nsb, int ncs) { return dg_off(nsb, ncs) + nsb * ncs * 16; }
    static __host__ __device__ constexpr int part_off(int nsb, int ncs) { return (y_off(nsb, ncs) + nsb * ncs * 4 + 255) / 256 * 256; }
    static __host__ __device__ constexpr size_t lds_bytes(int nsb, int ncs, int slots, int npieces, bool shared_groups) {
        return (size_t)part_off(nsb, ncs) + (shared_groups ? (size_t)slots * npieces * NCT * 16 * 4 : 0);
    }
};

// One piece of a lane's weights in flight: a dword of the header (the quad holds all four) and two 16-byte runs of
// quants for four super-blocks.
struct PieceRegs { unsigned hdr[PIECE]; u4v qa[PIECE], qb[PIECE]; };

// SHARED: several waves share a row group (wpg > 1) and add their piece sums through LDS.
// XF32: the activations come as f32 rows xf [nc][K] and the workgroup quantizes them to Q8_K itself, straight into its LDS
// (the same block quantizer as the stand-alone kernel: the same bits), instead of copying quantized planes.
// HELP (with XF32): the workgroup is filled up to sixteen waves with helper waves (below).
template <bool SHARED, bool XF32, bool HELP = false>
__global__ __launch_bounds__(64 * MAX_WAVES) void deep16_q4k_kernel(DeepArgs g, DevAct a, const float *__restrict__ xf, int col0, int nc,
                                                                    DeepCut cut) {
    typedef DeepGeo Geo;
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nsb = g.nsb, npieces = (nsb + PIECE - 1) / PIECE;
    const int slot = (wave * cut.inv_wpg) >> 8, sub = wave - slot * cut.wpg;
    const int p_begin = sub * cut.ppw, p_end = min(npieces, p_begin + cut.ppw);
    const unsigned row_bytes = (unsigned)nsb * Q4_K_BYTES;
    const unsigned sm = lds_addr(smem);
    const int bid = blockIdx.x;
    // this wave's row groups: (k * slots + slot) * grid + workgroup, k = 0, 1, ...
    const int group_step = cut.slots * cut.grid;
    const int group0 = slot * cut.grid + bid;

    // ---- 1. the activations, requested first: quants, block-sum digits, block scales -> LDS
    const int nblk = nc * nsb;  // Q8_K blocks of the launch's columns; block b = column b / nsb, super-block b % nsb
    const int ncs_log2 = nc > 4 ? 3 : 2, ncs = 1 << ncs_log2;  // columns of the LDS layout
    const float4 *x4 = reinterpret_cast<const float4 *>(xf) + (int64_t)col0 * nsb * 64;
    // f32 input: four blocks per wave and round (block 4 (wave + round * W) + lane / 16), sixteen lanes a block, sixteen
    // consecutive elements a lane; the first XR rounds are requested here, ahead of the weights
    constexpr int XR = 3;
    float4 xq[XR][4];
    if (XF32) {
#pragma unroll
        for (int t = 0; t < XR; t++) {
            if (4 * (wave + t * cut.W) < nblk) {  // wave-uniform
                const int b = min(4 * (wave + t * cut.W) + (lane >> 4), nblk - 1);
#pragma unroll
                for (int j = 0; j < 4; j++) xq[t][j] = x4[b * 64 + 4 * (lane & 15) + j];
            }
        }
    } else {
        auto acol = [&](int i) { return col0 + min(i, nc - 1); };
        const uint8_t *aq = reinterpret_cast<const uint8_t *>(a.qs);
        // copy instructions are dealt out to the waves in turn: first the quants (two instructions per super-block:
        // columns 0..3 and 4..7), then the digits and the scales (64 (super-block, column) cells per instruction)
        // (columns past nc are not copied: the lanes of the A operand that stand for them read zeros)
        const int sets = nc > 4 ? 2 : 1;
        const int cells = nsb * ncs, n_q = nsb * sets, n_c = (cells + 63) / 64;
        for (int n = wave; n < n_q + 2 * n_c; n += cut.W) {
            if (n < n_q) {
                const int sb = sets == 2 ? n >> 1 : n, j = sets == 2 ? n & 1 : 0;
                const int col = 4 * j + (lane >> 4), pc = (lane & 15) ^ a_swz(col);
                if (col < nc)
                    dma_lds<16>(aq + (int64_t)sb * QKK, (unsigned)acol(col) * (unsigned)a.K + 16u * pc,
                                sm + Geo::A_OFF + (unsigned)(sb * ncs + 4 * j) * 256u);
            } else {
                const bool digits = n < n_q + n_c;
                const int c0 = 64 * (digits ? n - n_q : n - n_q - n_c);
                const int cell = min(c0 + lane, cells - 1), sb = cell >> ncs_log2, col = cell & (ncs - 1);
                const unsigned at = (unsigned)acol(col) * (unsigned)nsb + (unsigned)sb;
                if (c0 + lane < cells) {
                    if (digits) dma_lds<16>(a.sd8, at * 16u, sm + Geo::dg_off(nsb, ncs) + 16u * c0);
                    else dma_lds<4>(reinterpret_cast<const uint8_t *>(a.d), at * 4u, sm + Geo::y_off(nsb, ncs) + 4u * c0);
                }
            }
        }
    }
    if (tid < 64) *reinterpret_cast<int2 *>(smem + 8 * tid) = make_int2(0, 0);  // the zero block (a workgroup can be one wave)

    // ---- 2. the weight stream: a ring of four super-blocks per lane; a slot is requested again (for the same slot of
    // the wave's next piece) as soon as its super-block has been multiplied
    // loading: the lane's row and which 16-byte piece of the quad's 64 bytes it takes.  Rows 8..15 take the pieces in the
    // order 2 3 0 1: ds_bpermute moves 32 lanes per cycle through 32 banks (bank = source lane mod 32), a half-wave reads
    // pieces {0, 1} (or {2, 3}) of all 16 rows, and with the same order in every row the sources 4 r + p of rows r and
    // r + 8 would share a bank.
    const int lrow = lane >> 2, lq = (lane & 3) ^ ((lane >> 4) & 2);
    struct ItemAt { gbytes_t base; unsigned roff; };
    auto item_at = [&](int group) __attribute__((always_inline)) {
        const DeepWhere at = deep_where(g, group);
        const int64_t m0 = (int64_t)(group - at.first) * 16;
        const int rows_left = (int)min((int64_t)16, at.M - m0);  // rows past M: the last row again, results dropped
        ItemAt ia;
        ia.base = (gbytes_t)at.p0 + m0 * row_bytes;
        ia.roff = (unsigned)min(lrow, rows_left - 1) * row_bytes;
        return ia;
    };
    PieceRegs R;
    auto load_slot = [&](const ItemAt &ia, int piece, int i) __attribute__((always_inline)) {
        const int sb = min(piece * PIECE + i, nsb - 1);  // past the row's end: the last super-block again
        // (the base through readfirstlane: known to be uniform, the loads then take it from scalar registers and a 32-bit
        // lane offset instead of a 64-bit address per lane)
        const unsigned long long bv = (unsigned long long)(ia.base + (unsigned)(sb * Q4_K_BYTES));
        gbytes_t p = (gbytes_t)(((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(bv >> 32)) << 32) |
                                (unsigned)__builtin_amdgcn_readfirstlane((int)bv));
        R.hdr[i] = *(const __attribute__((address_space(1))) unsigned *)(p + (ia.roff + 4u * lq));
        R.qa[i] = *(gu4_t)(p + (ia.roff + 16u + 16u * lq));
        R.qb[i] = *(gu4_t)(p + (ia.roff + 80u + 16u * lq));
    };
    // load cursor: the piece the ring is being filled with
    int lgroup = min(group0, g.groups_total - 1), lp = p_begin;
    ItemAt L = item_at(lgroup);
    // Order of the first requests.  The memory system serves requests roughly in the order they were made, machine-wide,
    // and the waves of this launch can have tens of megabytes of weights queued within the first microsecond: activations
    // requested behind that queue arrive when it has drained, microseconds later, and nothing can be multiplied until
    // they are there.  So: the copies first; one super-block of weights per wave behind them (enough to start the
    // stream); the rest of the ring only when the activations have landed.
    if (XF32) {
        auto quantize_four = [&](int b0, const float4 (&v)[4]) __attribute__((always_inline)) {
            const int b = b0 + (lane >> 4), sub = lane & 15;
            float dd;
            int sum16, pair;
            const uint4 packed = q8_K_quantize_row16(v, lane, dd, sum16, pair);
            if (b < nblk) {  // the last four may end early: whole rows of 16 lanes drop out
                const int col = (b * cut.inv_nsb) >> 20, sb = b - col * nsb, cell = sb * ncs + col;
                *reinterpret_cast<uint4 *>(smem + Geo::A_OFF + cell * 256 + 16 * (sub ^ a_swz(col))) = packed;
                if ((sub & 1) == 0) {  // the sum of a sub-block of 32 as two digits, S = 64 * (S >> 6) + (S & 63)
                    smem[Geo::dg_off(nsb, ncs) + cell * 16 + (sub >> 1)] = (uint8_t)(pair & 63);
                    smem[Geo::dg_off(nsb, ncs) + cell * 16 + 8 + (sub >> 1)] = (uint8_t)(pair >> 6);
                }
                if (sub == 0) *reinterpret_cast<float *>(smem + Geo::y_off(nsb, ncs) + cell * 4) = dd;
            }
        };
        auto quantize_share = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int t = 0; t < XR; t++)
                if (4 * (wave + t * cut.W) < nblk) quantize_four(4 * (wave + t * cut.W), xq[t]);
            for (int b0 = 4 * (wave + XR * cut.W); b0 < nblk; b0 += 4 * cut.W) {  // (more rounds than were requested ahead)
                float4 v[4];
                const int bc = min(b0 + (lane >> 4), nblk - 1);
#pragma unroll
                for (int j = 0; j < 4; j++) v[j] = x4[bc * 64 + 4 * (lane & 15) + j];
                quantize_four(b0, v);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the LDS writes, before the barrier
        };
        // Helper waves: a workgroup that streams with fewer than sixteen waves (few row groups per CU, a short K) has too
        // few to quantize x in two or three rounds; the launch fills the workgroup up to sixteen, the extra waves take
        // their share of the blocks and leave.  (A barrier waits for the waves that have not ended.)
        // (A variant of its own: with the early exit in the code the full workgroups of the large products measured 0.15 to
        // 0.5 us slower.)
        const bool helper = HELP && wave >= cut.Wact;
        // x is on its way (cache hits for all but the first workgroups to ask); one super-block of weights per wave goes
        // out behind it, the rest of the ring after the quantization: a wave that requests more than the memory
        // pipeline takes at once is held at the request, and could not quantize meanwhile
        if (!helper) load_slot(L, lp, 0);
        __builtin_amdgcn_sched_barrier(0);
        quantize_share();
        __builtin_amdgcn_s_barrier();
        if (HELP && helper) return;
#pragma unroll
        for (int i = 1; i < PIECE; i++) {
            load_slot(L, lp, i);
            __builtin_amdgcn_sched_barrier(0);  // slot after slot, the order the loop refills them in
        }
    } else {
        // Order of the first requests.  The memory system serves requests roughly in the order they were made,
        // machine-wide, and the waves of this launch can have tens of megabytes of weights queued within the first
        // microsecond: copies requested behind that queue arrive when it has drained, microseconds later, and nothing
        // can be multiplied until they are there.  So: the copies first; one super-block of weights per wave behind them
        // (enough to start the stream); the rest of the ring only when the activations have landed.
        load_slot(L, lp, 0);
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory");  // (loads retire in order: all but the three weight loads)
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int i = 1; i < PIECE; i++) {
            load_slot(L, lp, i);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- 3. operand reads: per-lane LDS addresses and per-super-block strides (0 for lanes that read zeros)
    const int r = lane & 15, kg = lane >> 4;  // MFMA order: the lane's weight row (= A row) and K group
    const int rsw = (r >> 3) << 1;            // (rows 8..15 were loaded with their pieces in the order 2 3 0 1)
    const int bidx = 4 * (4 * r + (kg ^ rsw));  // ds_bpermute: the lane that loaded what this lane multiplies
    unsigned a0_at, a_st, d_at, d_st, y_at;
    const unsigned y_st = (unsigned)ncs * 4;
    {
        const int col = r >> 1, w = r & 1;  // A row r: column, which of the MFMA's two sub-blocks
        const bool a_on = col < nc && (kg >> 1) == w;
        const bool d_on = col < nc && kg == 0;  // low digits in A row 2c, high digits in row 2c + 1
        const int s0 = (4 * (kg >> 1) + (kg & 1)) ^ a_swz(col);  // slot of the lane's first piece; the others: ^2, ^8, ^10
        a0_at = sm + (a_on ? Geo::A_OFF + col * 256 + 16 * s0 : 128);
        a_st = a_on ? ncs * 256 : 0;
        d_at = sm + (d_on ? Geo::dg_off(nsb, ncs) + col * 16 + 8 * w : 0);
        d_st = d_on ? ncs * 16 : 0;
        // the two columns this lane's outputs belong to (a layout of four columns: K groups 2, 3 read those of columns 2, 3,
        // their outputs are dropped)
        y_at = sm + Geo::y_off(nsb, ncs) + 4 * min(2 * kg, ncs - 2);
    }
    float *part = reinterpret_cast<float *>(smem + Geo::part_off(nsb, ncs));  // [slot][piece][NCT][16]

    const v4i zero = {0, 0, 0, 0};
    // one super-block (ring slot i) into the piece's accumulators; aa0 / da: the lane's LDS addresses of its first operand
    // piece and of its digits for this super-block (kept running: lanes that read zeros have stride 0)
    auto mul_slot = [&](int i, int sb, unsigned aa0, unsigned da, float (&acc)[2]) __attribute__((always_inline)) {
        const unsigned aa1 = aa0 ^ 32u;  // (slots s0 and s0 ^ 2; every base is a multiple of 64)
        const v2i dg = lds_at<v2i>(da, 0);
        const v2f yd = lds_at<v2f>(y_at + (unsigned)sb * y_st, 0);
        u4v hdr;  // the four dwords of the row's header, from the four lanes of the quad that loaded it
#pragma unroll
        for (int j = 0; j < 4; j++) hdr[j] = (unsigned)__builtin_amdgcn_ds_bpermute(4 * (4 * r) + 4 * (j ^ rsw), (int)R.hdr[i]);
        const v4i av0 = lds_at<v4i>(aa0, 0), av1 = lds_at<v4i>(aa1, 0);
        const u4v qa = bperm(bidx, R.qa[i]);
        const float d = h2f(hdr.x & 0xffff), dmin = h2f(hdr.x >> 16);
        const unsigned sc03 = hdr.y & 0x3f3f3f3fu, sc47 = (hdr.w & 0x0f0f0f0fu) | (((hdr.y >> 6) & 0x03030303u) << 4);
        const unsigned mn03 = hdr.z & 0x3f3f3f3fu, mn47 = ((hdr.w >> 4) & 0x0f0f0f0fu) | (((hdr.z >> 6) & 0x03030303u) << 4);
        int sc[8];
#pragma unroll
        for (int j = 0; j < 8; j++) sc[j] = (int)(((j < 4 ? sc03 : sc47) >> (8 * (j & 3))) & 0xff);
        // The mins against the block-sum digits.  Only K group 0 of the A operand is not zero, and of it only the first
        // eight bytes: whatever else the B operand holds is multiplied by zeros, so the mins go in unmasked and the
        // operand's other two registers are left as they are.
        v4i bm;
        bm[0] = (int)mn03;
        bm[1] = (int)mn47;
        const v4i x = mfma16((v4i){dg.x, dg.y, 0, 0}, bm, zero);
        // MFMA j: K groups {0, 1} = sub-block 4 (j >> 1) + (j & 1), K groups {2, 3} = that + 2; output v of a lane:
        // column 2 kg + (v >> 1), the MFMA's sub-block v & 1
        auto nib_lo = [](u4v q) { return (v4i){(int)(q.x & 0x0f0f0f0fu), (int)(q.y & 0x0f0f0f0fu), (int)(q.z & 0x0f0f0f0fu), (int)(q.w & 0x0f0f0f0fu)}; };
        auto nib_hi = [](u4v q) {
            return (v4i){(int)((q.x >> 4) & 0x0f0f0f0fu), (int)((q.y >> 4) & 0x0f0f0f0fu), (int)((q.z >> 4) & 0x0f0f0f0fu),
                         (int)((q.w >> 4) & 0x0f0f0f0fu)};
        };
        // one v_mad_i32_i24 per product: the empty asm keeps the compiler from regrouping the sum into multiplies and
        // three-operand adds, half again as many instructions
        auto mad = [](int a_, int b_, int c_) {
            int o = __mul24(a_, b_) + c_;
            asm("" : "+v"(o));
            return o;
        };
        const v4i D0 = mfma16(av0, nib_lo(qa), zero), D1 = mfma16(av1, nib_hi(qa), zero);
        const v4i av2 = lds_at<v4i>(aa0, 128), av3 = lds_at<v4i>(aa1, 128);
        const u4v qb = bperm(bidx, R.qb[i]);
        const v4i D2 = mfma16(av2, nib_lo(qb), zero), D3 = mfma16(av3, nib_hi(qb), zero);
#pragma unroll
        for (int u = 0; u < 2; u++) {
            int isum = __mul24(sc[0], D0[2 * u]);
            isum = mad(sc[2], D0[2 * u + 1], isum);
            isum = mad(sc[1], D1[2 * u], mad(sc[3], D1[2 * u + 1], isum));
            isum = mad(sc[4], D2[2 * u], mad(sc[6], D2[2 * u + 1], isum));
            isum = mad(sc[5], D3[2 * u], mad(sc[7], D3[2 * u + 1], isum));
            const float fm = dmin * (float)((x[2 * u + 1] << 6) + x[2 * u]);
            acc[u] = __builtin_fmaf(yd[u], __builtin_fmaf(d, (float)isum, -fm), acc[u]);
        }
    };

    // ---- 4. the pieces in order.  Every piece but the wave's last refills the ring for the piece after it (of the same
    // row group, or the first of the wave's next one); the last piece is a copy of the loop's body without the requests,
    // so that no request in the loop is conditional (the compiler counts the outstanding loads in front of every use, and
    // a conditional request makes it assume the worst).
    const int np = max(p_end - p_begin, 0);
    int items = 0;  // row groups of this wave
    if (np > 0 && group0 < g.groups_total) items = group0 + (cut.iters - 1) * group_step < g.groups_total ? cut.iters : cut.iters - 1;
    const int n_total = items * np;
    int ck = 0, cp = p_begin;  // compute cursor: item, piece
    float total[2] = {0.f, 0.f};
    // the piece sums of each output of row group k of this slot are added in piece order, by the first wave of the row group
    auto sum_shared = [&](int k) __attribute__((always_inline)) {
        __syncthreads();
        const int group = group0 + k * group_step;
        if (sub == 0 && group < g.groups_total) {
            const DeepWhere at = deep_where(g, group);
            const int64_t m0 = (int64_t)(group - at.first) * 16;
            for (int o = lane; o < NCT * 16; o += 64) {
                const int col = o >> 4, row = o & 15;
                float sum = 0.f;
                for (int p = 0; p < npieces; p++) sum += part[((slot * npieces + p) * NCT + col) * 16 + row];
                if (col < nc && m0 + row < at.M) at.y[(int64_t)(col0 + col) * at.M + m0 + row] = sum;
            }
        }
        if (k + 1 < cut.iters) __syncthreads();
    };
    auto one_piece = [&](auto refill_tag) __attribute__((always_inline)) {
        constexpr bool REFILL = decltype(refill_tag)::value;
        if (REFILL) {
            if (lp + 1 < p_end) lp++;
            else {
                lp = p_begin;
                lgroup += group_step;
                L = item_at(lgroup);
            }
        }
        float acc[2] = {0.f, 0.f};
        unsigned aa = a0_at + (unsigned)(cp * PIECE) * a_st, da = d_at + (unsigned)(cp * PIECE) * d_st;
#pragma unroll
        for (int i = 0; i < PIECE; i++) {
            if (cp * PIECE + i < nsb) mul_slot(i, cp * PIECE + i, aa, da, acc);  // wave-uniform
            aa += a_st;
            da += d_st;
            if (REFILL) load_slot(L, lp, i);
        }
        const bool item_done = cp + 1 == p_end;
        if (!SHARED) {
            total[0] += acc[0];
            total[1] += acc[1];
            if (item_done) {  // the row group is complete: lane (r, kg) holds row r of columns 2 kg, 2 kg + 1
                const int group = group0 + ck * group_step;
                const DeepWhere at = deep_where(g, group);
                const int64_t m0 = (int64_t)(group - at.first) * 16;
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const int col = 2 * kg + u;
                    if (col < nc && m0 + r < at.M) at.y[(int64_t)(col0 + col) * at.M + m0 + r] = total[u];
                    total[u] = 0.f;
                }
            }
        } else {
#pragma unroll
            for (int u = 0; u < 2; u++) part[((slot * npieces + cp) * NCT + 2 * kg + u) * 16 + r] = acc[u];
            if (item_done) sum_shared(ck);
        }
        if (item_done) {
            ck++;
            cp = p_begin;
        } else {
            cp++;
        }
    };
#pragma unroll 1
    for (int f = 0; f + 1 < n_total; f++) one_piece(std::true_type{});
    if (n_total > 0) one_piece(std::false_type{});
    if (SHARED) {  // (waves with fewer row groups than the workgroup's first slot still take part in its barriers)
#pragma unroll 1
        for (int k = items; k < cut.iters; k++) sum_shared(k);
    }
}

// Waves the f32 form launches per workgroup.  Each wave quantizes four blocks of x per round.  A workgroup that streams
// with fewer than sixteen waves (few row groups per CU, a short K) is filled up to sixteen with helper waves -- they
// take their share of the blocks and leave -- where that saves two rounds or more: 4096 x 4096 (four working waves) at
// three / eight columns 8.3 / 8.4 -> 5.5 / 7.4 us, 8192 x 4096 (eight waves) at eight columns 9.2 -> 9.0; where it
// saves one round or none the filled workgroup is 0.3 to 0.7 us slower (8192 x 4096 at three columns 6.5 -> 7.2,
// 12288 x 4096 8.6 -> 9.3, 28672 x 4096 at eight 16.0 -> 16.1).
int deep16_f32_waves(int ncols, int nsb, int working) {
    auto rounds = [&](int waves) { return (ncols * nsb + 4 * waves - 1) / (4 * waves); };
    return working < MAX_WAVES && rounds(working) - rounds(MAX_WAVES) >= 2 ? MAX_WAVES : working;
}

bool deep16_cut(int64_t K, int64_t groups, int ncols, int num_cus, DeepCut &c, size_t &lds) {
    if (K % QKK || ncols < 1 || ncols > NCT || groups < 1 || groups > 0x7fffffff || num_cus < 1) return false;
    const int nsb = (int)(K / QKK), npieces = (nsb + PIECE - 1) / PIECE;
    const int64_t per_cu = (groups + num_cus - 1) / num_cus;
    int wpg = per_cu >= MAX_WAVES ? 1 : (int)(MAX_WAVES / per_cu);
    if (wpg > npieces) wpg = npieces;
    c.ppw = (npieces + wpg - 1) / wpg;
    c.wpg = (npieces + c.ppw - 1) / c.ppw;
    c.inv_wpg = (256 + c.wpg - 1) / c.wpg;
    c.slots = MAX_WAVES / c.wpg;
    if (c.slots > per_cu) c.slots = (int)per_cu;
    c.W = c.Wact = c.slots * c.wpg;
    c.grid = (int)std::min<int64_t>(num_cus, (groups + c.slots - 1) / c.slots);
    c.iters = (int)((groups + (int64_t)c.slots * c.grid - 1) / ((int64_t)c.slots * c.grid));
    for (int wv = 0; wv < c.W; wv++)
        if (((wv * c.inv_wpg) >> 8) != wv / c.wpg) return false;  // (never: checked for every wpg up to 16)
    c.inv_nsb = ((1 << 20) + nsb - 1) / nsb;
    for (int b = 0; b < NCT * nsb; b++)
        if (((b * c.inv_nsb) >> 20) != b / nsb) return false;  // (exact while 8 nsb^2 < 2^20: every K whose activations fit the LDS)
    lds = DeepGeo::lds_bytes(nsb, ncols > 4 ? 8 : 4, c.slots, npieces, c.wpg > 1);
    return lds <= 160 * 1024;
}

}  // namespace

bool deep16_wanted(int type, int64_t K, int64_t total_m, int ncols, int num_cus) {
    // two columns only on rows of one K segment: on longer rows the streaming kernel with its in-kernel quantization is
    // ahead -- where it applies (rows of 28672 are beyond it: 8192 x 28672 at two columns 44.9 us through quantization +
    // GEMV, 32 here)
    if (type != T_Q4_K || ncols < 2 || (ncols == 2 && K > 4096 && gemv_f32_supported(type, K, total_m, 2))) return false;
    DeepCut c;
    size_t lds;
    if (!deep16_cut(K, (total_m + 15) / 16, ncols, num_cus, c, lds)) return false;
    if (total_m * K > ((int64_t)40 << 20)) return true;  // (below that the many-small-waves direct kernel is ahead at 3..4 columns)
    // Five to eight columns, where the alternative is the staged kernel: from 20 Mi weights (below 24576 rows: beyond, the
    // rows kernel).  6144 x 4096 7.5 against 9.1 us at five columns (9.4 / 9.5 at eight), 8192 x 4096 8.2 / 10.1 against
    // 10.5 / 11.0; on 4096 x 4096 this kernel is 5 % behind (8.4 against 8.0 us: its four waves per CU cannot quantize x
    // themselves).  (q + k + v of 4096 + 1024 + 1024 rows in one launch would take 7.8 / 10.5 us here against 12.7 / 13.0
    // staged, but a joint launch takes a kernel only when every matrix takes it alone, and alone they are too small.)
    if (ncols >= 5 && total_m * K >= ((int64_t)20 << 20) && (total_m + 15) / 16 < 6 * (int64_t)num_cus) return true;
    // Three to eight columns of anything smaller, where the workgroups can quantize f32 x themselves in three rounds (K up
    // to 4096 at eight columns, 12288 at four): one launch instead of quantization + product, and that launch is what
    // such a small product costs -- 4096 x 4096 at three / eight columns 7.2 / 8.0 -> 5.5 / 7.4 us, 1024 x 4096 7.2 / 7.8
    // -> 5.4 / 7.2, 4096 x 1024 6.7 / 7.2 -> 4.5 / 4.5 against the direct-load and the staged kernel.  (From quantized
    // planes this kernel is 0.2 to 0.7 us behind them on these shapes: 4096 x 4096 4.9 -> 5.4 us at three columns.)
    return ncols >= 3 && (int64_t)ncols * (K / QKK) <= 3 * 4 * deep16_f32_waves(ncols, (int)(K / QKK), c.Wact) &&
           (total_m + 15) / 16 < 6 * (int64_t)num_cus;
}

namespace {

hipError_t launch_deep16_any(const DevWeight *ws, float *const *ys, int count, const DevAct *a, const float *xf, int col0, int ncols,
                             int num_cus, hipStream_t s) {
    if (count < 1 || count > DEEP_MULTI) return hipErrorInvalidValue;
    DeepArgs g;
    int64_t rg = 0;
    for (int i = 0; i < DEEP_MULTI; i++) {
        const int j = i < count ? i : count - 1;
        g.p0[i] = ws[j].p0; g.y[i] = ys[j]; g.M[i] = ws[j].M;
        if (i < count) rg += (ws[i].M + 15) / 16;
        g.grp_end[i] = i < count ? (int)rg : 0x7fffffff;
    }
    g.groups_total = (int)rg;
    g.nsb = (int)(ws[0].K / QKK);
    DeepCut c;
    size_t lds;
    if (!deep16_cut(ws[0].K, rg, ncols, num_cus, c, lds)) return hipErrorInvalidValue;
    static bool allowed[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 && !allowed[dev]) {
#define DEEP_ALLOW(...) \
    (void)hipFuncSetAttribute(reinterpret_cast<const void *>(deep16_q4k_kernel<__VA_ARGS__>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024)
        DEEP_ALLOW(false, false); DEEP_ALLOW(true, false); DEEP_ALLOW(false, true); DEEP_ALLOW(true, true);
        DEEP_ALLOW(false, true, true); DEEP_ALLOW(true, true, true);
#undef DEEP_ALLOW
        allowed[dev] = true;
    }
    const DevAct none{};
    const bool help = xf && deep16_f32_waves(ncols, g.nsb, c.Wact) > c.Wact;
    if (help) c.W = MAX_WAVES;  // (waves beyond the working ones help to quantize x and leave)
    const dim3 grid((unsigned)c.grid), block(64 * c.W);
    if (help) {
        if (c.wpg == 1) deep16_q4k_kernel<false, true, true><<<grid, block, lds, s>>>(g, none, xf, col0, ncols, c);
        else deep16_q4k_kernel<true, true, true><<<grid, block, lds, s>>>(g, none, xf, col0, ncols, c);
    } else if (xf) {
        if (c.wpg == 1) deep16_q4k_kernel<false, true><<<grid, block, lds, s>>>(g, none, xf, col0, ncols, c);
        else deep16_q4k_kernel<true, true><<<grid, block, lds, s>>>(g, none, xf, col0, ncols, c);
    } else {
        if (c.wpg == 1) deep16_q4k_kernel<false, false><<<grid, block, lds, s>>>(g, *a, nullptr, col0, ncols, c);
        else deep16_q4k_kernel<true, false><<<grid, block, lds, s>>>(g, *a, nullptr, col0, ncols, c);
    }
    return hipGetLastError();
}

}  // namespace

namespace {

// ---------------------------------------------------------------------------------------------------------------------
// The same kernel shape for Q6_K (the down projection and the value projection of the common mixed files).
//
//   * Weights: the planes of formats.h.  Per super-block a lane (row, j) of a 16-row group loads the 16-byte pieces j
//     and 4 + j of the row's 128 low-nibble bytes, piece j of its 64 bytes of high bit pairs and dword j of its 16
//     scales -- the quad reads runs of its row -- and, in the matrix cores' lane order, the row's fp16 scale.
//   * Arithmetic: the 6-bit quants go into v_mfma_i32_16x16x64_i8 as they are stored, 0..63; the offset of 32 is
//     taken out with the block sums: sum (q - 32) y = sum q y - 32 sum y.  A chunk of 64 elements is one MFMA whose
//     four K groups are four scale groups of 16, so the 16 rows of the A operand are 4 columns x 4 K groups (row
//     4 c + w is column c restricted to K group w) and one MFMA serves four activation columns; five to eight columns
//     take a second set of MFMAs on the same weight operand.  In chunk ch lane (row, kg) multiplies elements
//     64 ch + 16 kg ..: low (ch even) or high nibbles of piece 4 (ch / 2) + kg of the low-nibble bytes, and of piece
//     2 (ch / 2) + (kg & 1) of the bit pairs the pair at bit 4 (ch & 1) + 2 (kg / 2).  A lane is left with the
//     partial sums of column kg (and 4 + kg) with the 16 scale groups and applies the int8 scales with
//     v_mad_i32_i24; sum scale x block sum comes from one more MFMA on the block-sum digits.  All integer sums exact.
//   * One matrix per launch, activations from the quantized planes.
//
// Order of the floating-point sums: as above (pieces of four super-blocks in order, piece sums in order).
constexpr int Q6_QL = 128, Q6_QH = 64, Q6_SC = 16;
constexpr int DEEP6_FROM = 3;  // activation columns from which the kernel is taken (at two the streaming kernel is ahead: 14.1 / 14.9 against 15.6 / 15.1 us)
struct Deep6Args {
    const uint8_t *ql, *qh, *sc;
    const uint16_t *d;
    float *y;
    int64_t M;
    int groups_total, nsb;
};
// LDS map for 4 * SETS activation columns.  512 zero bytes; per super-block and column 256 bytes of quants in
// 16-byte pieces, piece p of column c at slot p ^ (c & 2); per (super-block, column) 32 bytes of block-sum digits (the
// low digits of the 16 sums, then the high digits) and the fp32 block scale; then the piece sums.
//
// The slot swizzle: ds_read_b128 serves 16 lanes per cycle, and the lanes of one such group that read real data
// are A rows (c, w) = (0, w0) (3, w0) (1, w0 + 1) (2, w0 + 1) or (1, w0) (2, w0) (0, w0 + 1) (3, w0 + 1), w0 = 0 or 2:
// with slots w ^ (c & 2) the four fall on the four slots of the chunk's aligned block of four; the lanes that read
// zeros read one address in the next block of four.
template <int SETS>
struct Deep6Geo {
    static constexpr int NC = 4 * SETS;
    static constexpr int A_OFF = 512;
    static __host__ __device__ constexpr int dg_off(int nsb) { return A_OFF + nsb * NC * 256; }
    static __host__ __device__ constexpr int y_off(int nsb) { return dg_off(nsb) + nsb * NC * 32; }
    static __host__ __device__ constexpr int part_off(int nsb) { return (y_off(nsb) + nsb * NC * 4 + 255) / 256 * 256; }
    static __host__ __device__ constexpr size_t lds_bytes(int nsb, int slots, int npieces, bool shared_groups) {
        return (size_t)part_off(nsb) + (shared_groups ? (size_t)slots * npieces * NC * 16 * 4 : 0);
    }
};
struct Piece6Regs { unsigned sc[PIECE], d[PIECE]; u4v qa[PIECE], qb[PIECE], qh[PIECE]; };

// XF32: f32 activations xf [nc][K], quantized by the workgroup itself (as in the Q4_K kernel above).
// HELP (with XF32): helper waves fill the workgroup up to sixteen, as above.
template <bool SHARED, int SETS, bool XF32, bool HELP = false>
__global__ __launch_bounds__(64 * MAX_WAVES) void deep16_q6k_kernel(Deep6Args g, DevAct a, const float *__restrict__ xf, int col0, int nc,
                                                                    DeepCut cut) {
    typedef Deep6Geo<SETS> Geo;
    constexpr int NC = Geo::NC;
    extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nsb = g.nsb, npieces = (nsb + PIECE - 1) / PIECE;
    const int slot = (wave * cut.inv_wpg) >> 8, sub = wave - slot * cut.wpg;
    const int p_begin = sub * cut.ppw, p_end = min(npieces, p_begin + cut.ppw);
    const unsigned sm = lds_addr(smem);
    const int bid = blockIdx.x;
    const int group_step = cut.slots * cut.grid;
    const int group0 = slot * cut.grid + bid;

    // ---- 1. the activations, requested first: quants, block-sum digits, block scales -> LDS
    const int nblk = nc * nsb;  // Q8_K blocks of the launch's columns; block b = column b / nsb, super-block b % nsb
    const float4 *x4 = reinterpret_cast<const float4 *>(xf) + (int64_t)col0 * nsb * 64;
    constexpr int XR = 3;  // rounds of four blocks per wave requested here, ahead of the weights
    float4 xq[XR][4];
    if (XF32) {
#pragma unroll
        for (int t = 0; t < XR; t++) {
            if (4 * (wave + t * cut.W) < nblk) {  // wave-uniform
                const int b = min(4 * (wave + t * cut.W) + (lane >> 4), nblk - 1);
#pragma unroll
                for (int j = 0; j < 4; j++) xq[t][j] = x4[b * 64 + 4 * (lane & 15) + j];
            }
        }
    } else {
        auto acol = [&](int i) { return col0 + min(i, nc - 1); };
        const uint8_t *aq = reinterpret_cast<const uint8_t *>(a.qs);
        // copy instructions are dealt out to the waves in turn: the quants (one instruction per super-block and set of
        // four columns), the digits (32 (super-block, column) cells per instruction), the scales (64 cells)
        const int cells = nsb * NC, n_q = nsb * SETS, n_g = (cells + 31) / 32, n_c = (cells + 63) / 64;
        for (int n = wave; n < n_q + n_g + n_c; n += cut.W) {
            if (n < n_q) {
                const int sb = n / SETS, j = n % SETS;
                const int col = 4 * j + (lane >> 4), pc = (lane & 15) ^ (col & 2);
                if (col < nc)  // (columns past nc keep what the LDS held: they are multiplied and dropped)
                    dma_lds<16>(aq + (int64_t)sb * QKK, (unsigned)acol(col) * (unsigned)a.K + 16u * pc,
                                sm + Geo::A_OFF + (unsigned)(sb * NC + 4 * j) * 256u);
            } else if (n < n_q + n_g) {
                const int c0 = 32 * (n - n_q);
                const int cell = min(c0 + (lane >> 1), cells - 1), sb = cell / NC, col = cell % NC;
                const unsigned at = (unsigned)acol(col) * (unsigned)nsb + (unsigned)sb;
                if (c0 + (lane >> 1) < cells) dma_lds<16>(a.sd16, at * 32u + 16u * (lane & 1), sm + Geo::dg_off(nsb) + 32u * c0);
            } else {
                const int c0 = 64 * (n - n_q - n_g);
                const int cell = min(c0 + lane, cells - 1), sb = cell / NC, col = cell % NC;
                const unsigned at = (unsigned)acol(col) * (unsigned)nsb + (unsigned)sb;
                if (c0 + lane < cells) dma_lds<4>(reinterpret_cast<const uint8_t *>(a.d), at * 4u, sm + Geo::y_off(nsb) + 4u * c0);
            }
        }
    }
    if (tid < 64) *reinterpret_cast<int2 *>(smem + 8 * tid) = make_int2(0, 0);  // the zero block (a workgroup can be one wave)

    // ---- 2. the weight stream: a ring of four super-blocks per lane
    // loading lane: its row and which piece of the quad's run it takes (rows 8..15 in the order 2 3 0 1, so that the
    // sources 4 r + p of rows r and r + 8 do not share a bank of the ds_bpermute crossbar)
    const int lrow = lane >> 2, lq = (lane & 3) ^ ((lane >> 4) & 2);
    const int r = lane & 15, kg = lane >> 4;  // MFMA order: the lane's weight row (= A row) and K group
    struct ItemAt { int64_t blk0; unsigned o_ql, o_qh, o_sc, o_d; };  // first block of the group's first row; lane offsets
    auto item_at = [&](int group) __attribute__((always_inline)) {
        const int64_t m0 = (int64_t)group * 16;
        const int rows_left = (int)min((int64_t)16, g.M - m0);  // rows past M: the last row again, results dropped
        ItemAt ia;
        ia.blk0 = m0 * nsb;
        const unsigned lb = (unsigned)(min(lrow, rows_left - 1) * nsb);
        ia.o_ql = lb * Q6_QL + 16u * lq;
        ia.o_qh = lb * Q6_QH + 16u * lq;
        ia.o_sc = lb * Q6_SC + 4u * lq;
        ia.o_d = (unsigned)(min(r, rows_left - 1) * nsb) * 2u;
        return ia;
    };
    auto uniform = [](const void *p) __attribute__((always_inline)) {
        const unsigned long long v = (unsigned long long)p;
        return (gbytes_t)(((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(v >> 32)) << 32) |
                          (unsigned)__builtin_amdgcn_readfirstlane((int)v));
    };
    Piece6Regs R;
    auto load_slot = [&](const ItemAt &ia, int piece, int i) __attribute__((always_inline)) {
        const int64_t blk = ia.blk0 + min(piece * PIECE + i, nsb - 1);  // past the row's end: the last super-block again
        gbytes_t pl = uniform(g.ql + blk * Q6_QL), ph = uniform(g.qh + blk * Q6_QH), ps = uniform(g.sc + blk * Q6_SC),
                 pd = uniform(g.d + blk);
        R.sc[i] = *(const __attribute__((address_space(1))) unsigned *)(ps + ia.o_sc);
        R.d[i] = *(const __attribute__((address_space(1))) unsigned short *)(pd + ia.o_d);
        R.qa[i] = *(gu4_t)(pl + ia.o_ql);
        R.qh[i] = *(gu4_t)(ph + ia.o_qh);
        R.qb[i] = *(gu4_t)(pl + (ia.o_ql + 64u));
    };
    int lgroup = min(group0, g.groups_total - 1), lp = p_begin;
    ItemAt L = item_at(lgroup);
    // the copies first; one super-block of weights per wave behind them; the rest of the ring when the activations
    // have landed (requests are served roughly in the order they were made)
    const bool helper = HELP && wave >= cut.Wact;  // (quantizes its share of x and leaves)
    if (!helper) load_slot(L, lp, 0);
    __builtin_amdgcn_sched_barrier(0);
    if (XF32) {
        auto quantize_four = [&](int b0, const float4 (&v)[4]) __attribute__((always_inline)) {
            const int b = b0 + (lane >> 4), sub16 = lane & 15;
            float dd;
            int sum16, pair;
            const uint4 packed = q8_K_quantize_row16(v, lane, dd, sum16, pair);
            if (b < nblk) {  // the last four may end early: whole rows of 16 lanes drop out
                const int col = (b * cut.inv_nsb) >> 20, sb = b - col * nsb, cell = sb * NC + col;
                *reinterpret_cast<uint4 *>(smem + Geo::A_OFF + cell * 256 + 16 * (sub16 ^ (col & 2))) = packed;
                // the sum of the lane's 16 quants as two digits, S = 64 * (S >> 6) + (S & 63)
                smem[Geo::dg_off(nsb) + cell * 32 + sub16] = (uint8_t)(sum16 & 63);
                smem[Geo::dg_off(nsb) + cell * 32 + 16 + sub16] = (uint8_t)(sum16 >> 6);
                if (sub16 == 0) *reinterpret_cast<float *>(smem + Geo::y_off(nsb) + cell * 4) = dd;
            }
        };
#pragma unroll
        for (int t = 0; t < XR; t++)
            if (4 * (wave + t * cut.W) < nblk) quantize_four(4 * (wave + t * cut.W), xq[t]);
        for (int b0 = 4 * (wave + XR * cut.W); b0 < nblk; b0 += 4 * cut.W) {  // (more rounds than were requested ahead)
            float4 v[4];
            const int bc = min(b0 + (lane >> 4), nblk - 1);
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = x4[bc * 64 + 4 * (lane & 15) + j];
            quantize_four(b0, v);
        }
        // columns past nc of the last set keep what the LDS held: they are multiplied and dropped
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the LDS writes, before the barrier
    } else {
        asm volatile("s_waitcnt vmcnt(5) lgkmcnt(0)" ::: "memory");  // (loads retire in order: all but the five weight loads)
    }
    __builtin_amdgcn_s_barrier();
    if (HELP && helper) return;
#pragma unroll
    for (int i = 1; i < PIECE; i++) {
        load_slot(L, lp, i);
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- 3. operand reads: per-lane LDS addresses and per-super-block strides (0 for lanes that read zeros)
    const int rsw = (r >> 3) << 1;
    const int bidx = 4 * (4 * r + (kg ^ rsw));              // low-nibble pieces: piece kg of either half
    const int bidx_h0 = 4 * (4 * r + ((kg & 1) ^ rsw));     // bit pairs of the first half: piece kg & 1
    const int bidx_h1 = 4 * (4 * r + ((2 + (kg & 1)) ^ rsw));  // of the second half: piece 2 + (kg & 1)
    const unsigned lsh = 2 * (kg >> 1);
    unsigned a_at[SETS], a_st, d_at, d_st, y_at;
    {
        const int c = r >> 2, w = r & 3;  // A row r: column c of a set, K group w
        const bool a_on = kg == w;
#pragma unroll
        for (int s = 0; s < SETS; s++) a_at[s] = sm + (a_on ? Geo::A_OFF + (4 * s + c) * 256 + 16 * (w ^ (c & 2)) : 64);
        a_st = a_on ? NC * 256 : 0;
        // block-sum digits: A row 4 c' + 2 s + digit is column 4 s + c' (so that a lane's outputs belong to its columns)
        const int dc = 4 * ((r >> 1) & 1) + (r >> 2), dig = r & 1;
        const bool d_on = kg == 0 && dc < NC;
        d_at = sm + (d_on ? Geo::dg_off(nsb) + dc * 32 + 16 * dig : 0);
        d_st = d_on ? NC * 32 : 0;
        y_at = sm + Geo::y_off(nsb) + 4 * kg;  // columns kg (and 4 + kg)
    }
    float *part = reinterpret_cast<float *>(smem + Geo::part_off(nsb));  // [slot][piece][NC][16]

    const v4i zero = {0, 0, 0, 0};
    auto mul_slot = [&](int i, int sb, const unsigned (&aa)[SETS], unsigned da, float (&acc)[SETS]) __attribute__((always_inline)) {
        const v4i dg = lds_at<v4i>(da, 0);
        float yd[SETS];
#pragma unroll
        for (int s = 0; s < SETS; s++) yd[s] = lds_at<float>(y_at + (unsigned)sb * (NC * 4), 16 * s);
        v4i scv;  // the row's 16 scales, from the four lanes of the quad that loaded them
#pragma unroll
        for (int j = 0; j < 4; j++) scv[j] = __builtin_amdgcn_ds_bpermute(4 * (4 * r) + 4 * (j ^ rsw), (int)R.sc[i]);
        const float d = h2f(R.d[i]);
        auto mad = [](int a_, int b_, int c_) {
            int o = __mul24(a_, b_) + c_;
            asm("" : "+v"(o));
            return o;
        };
        int isum[SETS];
        // scale x block sum: K group 0 of the A operand holds a digit of the 16 sums, the B operand the 16 scales (what
        // the other K groups of B hold is multiplied by zeros)
        const v4i x = mfma16(dg, scv, zero);
        // one chunk: the weight operand from low-nibble bytes lo4 (already shifted and masked) and bit pairs hi (in place)
        auto chunk = [&](int ch, u4v lo4, u4v hi, bool first) __attribute__((always_inline)) {
            v4i b;
#pragma unroll
            for (int k = 0; k < 4; k++) b[k] = (int)(lo4[k] | (hi[k] & 0x30303030u));
#pragma unroll
            for (int s = 0; s < SETS; s++) {
                const v4i av = lds_at<v4i>(aa[s], 64 * ch);
                const v4i D = mfma16(av, b, zero);
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    const int g16 = 4 * ch + w;
                    const int scale = __builtin_amdgcn_sbfe(scv[g16 >> 2], 8 * (g16 & 3), 8);
                    isum[s] = first && w == 0 ? __mul24(scale, D[w]) : mad(scale, D[w], isum[s]);
                }
            }
        };
        auto lo_nib = [](u4v q) { return (u4v){q.x & 0x0f0f0f0fu, q.y & 0x0f0f0f0fu, q.z & 0x0f0f0f0fu, q.w & 0x0f0f0f0fu}; };
        auto hi_nib = [](u4v q) { return (u4v){(q.x >> 4) & 0x0f0f0f0fu, (q.y >> 4) & 0x0f0f0f0fu, (q.z >> 4) & 0x0f0f0f0fu, (q.w >> 4) & 0x0f0f0f0fu}; };
        {
            const u4v qa = bperm(bidx, R.qa[i]);
            u4v t = bperm(bidx_h0, R.qh[i]);
#pragma unroll
            for (int k = 0; k < 4; k++) t[k] >>= lsh;
            chunk(0, lo_nib(qa), (u4v){t.x << 4, t.y << 4, t.z << 4, t.w << 4}, true);
            chunk(1, hi_nib(qa), t, false);
        }
        {
            const u4v qb = bperm(bidx, R.qb[i]);
            u4v t = bperm(bidx_h1, R.qh[i]);
#pragma unroll
            for (int k = 0; k < 4; k++) t[k] >>= lsh;
            chunk(2, lo_nib(qb), (u4v){t.x << 4, t.y << 4, t.z << 4, t.w << 4}, false);
            chunk(3, hi_nib(qb), t, false);
        }
#pragma unroll
        for (int s = 0; s < SETS; s++) {
            const int corr = (x[2 * s + 1] << 6) + x[2 * s];  // sum over the 16 groups of scale x block sum
            acc[s] = __builtin_fmaf(d * yd[s], (float)(isum[s] - (corr << 5)), acc[s]);
        }
    };

    // ---- 4. the pieces in order (the last piece apart, without requests: no request in the loop is conditional)
    const int np = max(p_end - p_begin, 0);
    int items = 0;
    if (np > 0 && group0 < g.groups_total) items = group0 + (cut.iters - 1) * group_step < g.groups_total ? cut.iters : cut.iters - 1;
    const int n_total = items * np;
    int ck = 0, cp = p_begin;
    float total[SETS];
#pragma unroll
    for (int s = 0; s < SETS; s++) total[s] = 0.f;
    auto sum_shared = [&](int k) __attribute__((always_inline)) {
        __syncthreads();
        const int group = group0 + k * group_step;
        if (sub == 0 && group < g.groups_total) {
            const int64_t m0 = (int64_t)group * 16;
            for (int o = lane; o < NC * 16; o += 64) {
                const int col = o >> 4, row = o & 15;
                float sum = 0.f;
                for (int p = 0; p < npieces; p++) sum += part[((slot * npieces + p) * NC + col) * 16 + row];
                if (col < nc && m0 + row < g.M) g.y[(int64_t)(col0 + col) * g.M + m0 + row] = sum;
            }
        }
        if (k + 1 < cut.iters) __syncthreads();
    };
    auto one_piece = [&](auto refill_tag) __attribute__((always_inline)) {
        constexpr bool REFILL = decltype(refill_tag)::value;
        if (REFILL) {
            if (lp + 1 < p_end) lp++;
            else {
                lp = p_begin;
                lgroup += group_step;
                L = item_at(min(lgroup, g.groups_total - 1));
            }
        }
        float acc[SETS];
        unsigned aa[SETS], da = d_at + (unsigned)(cp * PIECE) * d_st;
#pragma unroll
        for (int s = 0; s < SETS; s++) {
            acc[s] = 0.f;
            aa[s] = a_at[s] + (unsigned)(cp * PIECE) * a_st;
        }
#pragma unroll
        for (int i = 0; i < PIECE; i++) {
            if (cp * PIECE + i < nsb) mul_slot(i, cp * PIECE + i, aa, da, acc);  // wave-uniform
#pragma unroll
            for (int s = 0; s < SETS; s++) aa[s] += a_st;
            da += d_st;
            if (REFILL) load_slot(L, lp, i);
        }
        const bool item_done = cp + 1 == p_end;
        if (!SHARED) {
#pragma unroll
            for (int s = 0; s < SETS; s++) total[s] += acc[s];
            if (item_done) {  // the row group is complete: lane (r, kg) holds row r of columns kg and 4 + kg
                const int64_t m0 = (int64_t)(group0 + ck * group_step) * 16;
#pragma unroll
                for (int s = 0; s < SETS; s++) {
                    const int col = 4 * s + kg;
                    if (col < nc && m0 + r < g.M) g.y[(int64_t)(col0 + col) * g.M + m0 + r] = total[s];
                    total[s] = 0.f;
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < SETS; s++) part[((slot * npieces + cp) * NC + 4 * s + kg) * 16 + r] = acc[s];
            if (item_done) sum_shared(ck);
        }
        if (item_done) {
            ck++;
            cp = p_begin;
        } else {
            cp++;
        }
    };
#pragma unroll 1
    for (int f = 0; f + 1 < n_total; f++) one_piece(std::true_type{});
    if (n_total > 0) one_piece(std::false_type{});
    if (SHARED) {
#pragma unroll 1
        for (int k = items; k < cut.iters; k++) sum_shared(k);
    }
}

bool deep6_cut(int64_t K, int64_t groups, int ncols, int num_cus, DeepCut &c, size_t &lds) {
    if (K % QKK || ncols < 1 || ncols > 8 || groups < 1 || groups > 0x7fffffff || num_cus < 1) return false;
    const int nsb = (int)(K / QKK), npieces = (nsb + PIECE - 1) / PIECE;
    const int64_t per_cu = (groups + num_cus - 1) / num_cus;
    int wpg = per_cu >= MAX_WAVES ? 1 : (int)(MAX_WAVES / per_cu);
    if (wpg > npieces) wpg = npieces;
    c.ppw = (npieces + wpg - 1) / wpg;
    c.wpg = (npieces + c.ppw - 1) / c.ppw;
    c.inv_wpg = (256 + c.wpg - 1) / c.wpg;
    c.slots = MAX_WAVES / c.wpg;
    if (c.slots > per_cu) c.slots = (int)per_cu;
    c.W = c.Wact = c.slots * c.wpg;
    c.grid = (int)std::min<int64_t>(num_cus, (groups + c.slots - 1) / c.slots);
    c.iters = (int)((groups + (int64_t)c.slots * c.grid - 1) / ((int64_t)c.slots * c.grid));
    for (int wv = 0; wv < c.W; wv++)
        if (((wv * c.inv_wpg) >> 8) != wv / c.wpg) return false;
    c.inv_nsb = ((1 << 20) + nsb - 1) / nsb;
    for (int b = 0; b < 8 * nsb; b++)
        if (((b * c.inv_nsb) >> 20) != b / nsb) return false;
    lds = ncols <= 4 ? Deep6Geo<1>::lds_bytes(nsb, c.slots, npieces, c.wpg > 1) : Deep6Geo<2>::lds_bytes(nsb, c.slots, npieces, c.wpg > 1);
    return lds <= 160 * 1024;
}

}  // namespace

bool deep6_wanted(int type, int64_t K, int64_t M, int ncols, int num_cus) {
    // (two columns only where the streaming kernel cannot quantize x itself: rows of 28672)
    if (type != T_Q6_K || ncols > 8 || ncols < (gemv_f32_supported(type, K, M, 2) ? DEEP6_FROM : 2)) return false;
    DeepCut c;
    size_t lds;
    if (!deep6_cut(K, (M + 15) / 16, ncols, num_cus, c, lds)) return false;
    if (M * (K / QKK) * (int64_t)Q6_QL >= ((int64_t)1 << 32)) return false;  // 32-bit lane offsets into the planes
    // from 4096 x 4096 at four columns and more, from 20 Mi weights at three (where the streaming kernel is the alternative):
    // 6144 x 4096 at 3 / 4 / 8 columns 11.8 / 12.5 / 13.4 -> 7.6 / 8.7 / 11.5 us, 5120 x 5120 14.5 / 15.3 / 16.1 -> 9.8 / 10.4 / 13.0
    if (M * K >= ((int64_t)(ncols == 3 ? 20 : 16) << 20)) return true;
    // anything smaller (below 24576 rows) where the workgroups can quantize f32 x themselves in two rounds, with helper
    // waves where they stream with few: one launch instead of quantization + product.  f32 x in, 3 / 4 / 8 columns:
    // 4096 x 4096 8.9 / 8.7 / 9.4 -> 6.4 / 6.4 / 8.5 us, 1024 x 4096 7.3 / 8.2 / 8.4 -> 5.9 / 6.0 / 7.9, 4096 x 1024 7.0 / 7.1 / 7.3 ->
    // 5.0 / 5.2 / 5.5.  (From quantized planes: within 0.3 us of the streaming kernel at three columns, 0.9 us ahead of
    // the staged kernel at four on K = 4096, 0.8 to 1.0 us behind it at five to eight columns of K up to 2048.)
    const int nsb = (int)(K / QKK);
    return (int64_t)ncols * nsb <= 2 * 4 * deep16_f32_waves(ncols, nsb, c.Wact) && (M + 15) / 16 < 6 * (int64_t)num_cus;
}

namespace {

hipError_t launch_deep6_any(const DevWeight &w, float *y, const DevAct *a, const float *xf, int col0, int ncols, int num_cus, hipStream_t s) {
    if (w.type != T_Q6_K || ncols < 1 || ncols > 8) return hipErrorInvalidValue;
    Deep6Args g{w.p0, w.p1, w.p2, w.d, y, w.M, 0, (int)(w.K / QKK)};
    const int64_t rg = (w.M + 15) / 16;
    g.groups_total = (int)rg;
    DeepCut c;
    size_t lds;
    if (!deep6_cut(w.K, rg, ncols, num_cus, c, lds)) return hipErrorInvalidValue;
    static bool allowed[64] = {false};
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 && !allowed[dev]) {
#define DEEP_ALLOW(...) \
    (void)hipFuncSetAttribute(reinterpret_cast<const void *>(deep16_q6k_kernel<__VA_ARGS__>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024)
        DEEP_ALLOW(false, 1, false); DEEP_ALLOW(true, 1, false); DEEP_ALLOW(false, 2, false); DEEP_ALLOW(true, 2, false);
        DEEP_ALLOW(false, 1, true); DEEP_ALLOW(true, 1, true); DEEP_ALLOW(false, 2, true); DEEP_ALLOW(true, 2, true);
        DEEP_ALLOW(false, 1, true, true); DEEP_ALLOW(true, 1, true, true); DEEP_ALLOW(false, 2, true, true); DEEP_ALLOW(true, 2, true, true);
#undef DEEP_ALLOW
        allowed[dev] = true;
    }
    const DevAct none{};
    const DevAct &da = a ? *a : none;
    const bool help = xf && deep16_f32_waves(ncols, g.nsb, c.Wact) > c.Wact;
    if (help) c.W = MAX_WAVES;  // (waves beyond the working ones help to quantize x and leave)
    const dim3 grid((unsigned)c.grid), block(64 * c.W);
#define DEEP_GO(SHARED, SETS) \
    do { \
        if (help) deep16_q6k_kernel<SHARED, SETS, true, true><<<grid, block, lds, s>>>(g, da, xf, col0, ncols, c); \
        else if (xf) deep16_q6k_kernel<SHARED, SETS, true><<<grid, block, lds, s>>>(g, da, xf, col0, ncols, c); \
        else deep16_q6k_kernel<SHARED, SETS, false><<<grid, block, lds, s>>>(g, da, nullptr, col0, ncols, c); \
    } while (0)
    if (ncols <= 4) {
        if (c.wpg == 1) DEEP_GO(false, 1); else DEEP_GO(true, 1);
    } else {
        if (c.wpg == 1) DEEP_GO(false, 2); else DEEP_GO(true, 2);
    }
#undef DEEP_GO
    return hipGetLastError();
}

}  // namespace

hipError_t launch_deep6(const DevWeight &w, float *y, const DevAct &a, int col0, int ncols, int num_cus, hipStream_t s) {
    if (a.type != T_Q8_K || a.K != w.K || !a.sd16) return hipErrorInvalidValue;
    return launch_deep6_any(w, y, &a, nullptr, col0, ncols, num_cus, s);
}

hipError_t launch_deep16(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int col0, int ncols, int num_cus,
                         hipStream_t s) {
    return launch_deep16_any(ws, ys, count, &a, nullptr, col0, ncols, num_cus, s);
}

// The same from f32 activations x [ncols][K] (device): the workgroups quantize x themselves.  Every workgroup reads all of
// x again (as f32: 3.5 times the bytes of its quantized planes) and repeats the quantization, so this is for few columns
// of a short K: up to three rounds of four blocks per wave, the rounds a wave requests ahead of its first weights.  (A
// fourth round -- four columns of K = 14336 -- measured 14.7 us against 13.5 for quantize-then-multiply.)
bool deep16_f32_wanted(int type, int64_t K, int64_t total_m, int ncols, int num_cus) {
    if (type == T_Q6_K) {
        // one matrix per launch (total_m is that matrix's rows) and up to two rounds: three columns of K = 14336 measured
        // 15.8 us in three rounds against 15.4 for quantize-then-multiply
        DeepCut c;
        size_t lds;
        return deep6_wanted(type, K, total_m, ncols, num_cus) && deep6_cut(K, (total_m + 15) / 16, ncols, num_cus, c, lds) &&
               (int64_t)ncols * (K / QKK) <= 2 * 4 * deep16_f32_waves(ncols, (int)(K / QKK), c.Wact);
    }
    if (!deep16_wanted(type, K, total_m, ncols, num_cus)) return false;
    DeepCut c;
    size_t lds;
    if (!deep16_cut(K, (total_m + 15) / 16, ncols, num_cus, c, lds)) return false;
    return (int64_t)ncols * (K / QKK) <= 3 * 4 * deep16_f32_waves(ncols, (int)(K / QKK), c.Wact);
}
hipError_t launch_deep16_f32(const DevWeight *ws, float *const *ys, int count, const float *x, int ncols, int num_cus, hipStream_t s) {
    if (!x) return hipErrorInvalidValue;
    if (ws[0].type == T_Q6_K) return count == 1 ? launch_deep6_any(ws[0], ys[0], nullptr, x, 0, ncols, num_cus, s) : hipErrorInvalidValue;
    return launch_deep16_any(ws, ys, count, nullptr, x, 0, ncols, num_cus, s);
}

}  // namespace miqmm
