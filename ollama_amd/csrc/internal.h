// Launchers shared between the C ABI (capi.hip) and the kernel translation units.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "formats.h"
#include "produce_dev.h"

namespace miqmm {

// Weight encoders (encode.hip): f32 rows [M][K] -> GGUF blocks [M][row_size], the bytes of ggml's scalar
// quantize_row_{q4_0,q8_0,q4_K,q6_K}_ref.  x and out are device pointers.
bool encode_supported(int type, int64_t K);
hipError_t launch_encode_weights(int type, const float *x, int64_t K, int64_t M, uint8_t *out, hipStream_t s);

// kernel 1: f32 rows -> Q8_0 / Q8_K planes (bit-exact with the scalar CPU quantizers)
// sd8 / sd16: block-sum digit planes for the GEMM (Q8_K only; may be null)
// produce (optional): applied to x on the fly (RMSNORM needs row_scale from launch_rms_norm first)
// qf / bsf: quants and block sums as fp16 planes for the fp16-MFMA GEMM (Q8_K only; both or neither)
hipError_t launch_quantize_act(int q8_type, const float *x, int64_t K, int64_t N, int8_t *qs,
                               float *d, int16_t *bsums, uint8_t *sd8, uint8_t *sd16, hipStream_t s,
                               const Produce *produce = nullptr, uint16_t *qf = nullptr, uint16_t *bsf = nullptr);
// RMSNorm over rows of K floats: scale_out [N] (optional) = 1/sqrtf(mean(x^2)+eps) per row; y (optional) =
// (x * scale) * g with g [K] or null.  SwiGLU: y = silu(gate) * up over count floats (up null: y = silu(gate)).
hipError_t launch_rms_norm(const float *x, const float *g, float eps, int64_t K, int64_t N, float *scale_out, float *y,
                           hipStream_t s);
hipError_t launch_swiglu(const float *gate, const float *up, int64_t count, float *y, hipStream_t s);
// planes -> GGUF block bytes (34 B / 292 B blocks), for callers that want the bytes
hipError_t launch_pack_act_gguf(int q8_type, const int8_t *qs, const float *d, const int16_t *bsums,
                                int64_t K, int64_t N, uint8_t *out, hipStream_t s);

// upload-time re-layout GGUF blocks -> planes (Q4_0, Q8_0, Q6_K); Q4_K is copied unchanged
hipError_t launch_relayout(int type, const uint8_t *gguf, int64_t K, int64_t M, uint8_t *p0,
                           uint8_t *p1, uint8_t *p2, uint16_t *d, hipStream_t s);

// Q5_K blocks [M][K/256][176] -> the Q4_K tensor of rows of 2 K that stands for them (formats.h): out [M][2 K/256][144]
hipError_t launch_relayout_q5k(const uint8_t *gguf, int64_t K, int64_t M, uint8_t *out, hipStream_t s);
// MXFP4 blocks [M][K/32][17] -> Q8_0 planes (qs [M][K_out], d [M][K_out/32], rows padded with zero blocks) with the same dot products; *bad (device int, zeroed
// by the caller) is set when a block's scale is beyond what the planes can hold (e > 146: weights of 2^18 and more)
hipError_t launch_relayout_mxfp4(const uint8_t *gguf, int64_t K, int64_t K_out, int64_t M, uint8_t *qs, uint16_t *d, int *bad, hipStream_t s);
// Q5_0 blocks [M][K/32][22] -> Q8_0 planes with the same dot products, rows padded with zero blocks to K_out
hipError_t launch_relayout_q5_0(const uint8_t *gguf, int64_t K, int64_t K_out, int64_t M, uint8_t *qs, uint16_t *d, hipStream_t s);
// MXFP4 blocks -> their own planes for the streaming kernels (type T_MXFP4: p0 = nibble plane [M][K_out/32][16], d = the scale
// bytes as 16-bit values [M][K_out/32]), rows padded with zero blocks
hipError_t launch_relayout_mxfp4_native(const uint8_t *gguf, int64_t K, int64_t K_out, int64_t M, uint8_t *qs, uint16_t *e, hipStream_t s);
// out [n][K_out] for x [n][K] (both multiples of 4, K <= K_out): the row followed by itself (repeat, K_out = 2 K: the
// activations a Q5_K tensor kept as Q4_K is multiplied with) or by zeros (rows padded to the length the weight was padded to)
hipError_t launch_expand_rows(const float *x, int64_t K, int64_t K_out, int64_t n, bool repeat, float *out, hipStream_t s);

// kernels 2 and 4: streaming GEMV / skinny GEMM, ncols in 1..8.  y[n*ldy + m].
// returns hipErrorInvalidValue if the shape is outside the kernel's limits (caller reports it).
hipError_t launch_gemv(const DevWeight &w, const DevAct &a, int col0, int ncols, float *y,
                       int64_t ldy, int num_cus, hipStream_t s);
// several weight tensors of one type and K against the same activations in one launch
hipError_t launch_gemv_multi(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int col0, int ncols,
                             int num_cus, hipStream_t s);
int gemv_max_multi();
// The same products from f32 activations x [ncols][K] (device): the kernel quantizes x in its own
// prologue, saving the separate quantization launch.  Ask gemv_f32_supported() first.
bool gemv_f32_supported(int type, int64_t K, int64_t total_m, int ncols);
// produce (optional; one column; ask gemv_produce_supported() first): x goes through RMSNorm / SwiGLU in
// the same prologue, before it is quantized.
hipError_t launch_gemv_f32_multi(const DevWeight *ws, float *const *ys, int count, const float *x, int ncols,
                                 int num_cus, hipStream_t s, const Produce *produce = nullptr);
bool gemv_produce_supported(int type, int64_t K, int64_t total_m);
// Gate and up of a feed-forward block at one column with the gating in the epilogue: h [M] =
// silu(wg . Q8(x')) * (wu . Q8(x')), x' = x or RMSNorm(x) (produce: NONE or RMSNORM).  Same bits as the
// two products followed by launch_swiglu.
bool gemv_pair_supported(int type, int64_t K, int64_t M, bool rms);
hipError_t launch_gemv_pair_f32(const DevWeight &wg, const DevWeight &wu, const float *x, float *h, hipStream_t s,
                                const Produce *produce = nullptr);
// largest K the GEMV handles for a weight type
int64_t gemv_max_k(int type);
// Expert-indexed GEMV: w is a stack of n_expert matrices (w.M = rows per expert * n_expert), a holds
// the quantized activations of b [n_tokens][b_cols][K], ids [n_tokens][n_used] (device) picks the
// expert of every (token, slot) pair, y [n_tokens][n_used][M].  An id outside the stack gives NaNs.
// groups: device scratch of gemv_id_scratch_ints(n_used * n_tokens) ints.
// xf (optional, device): b itself in f32 -- the kernel then quantizes each pair's row in its prologue
// and a only carries the geometry; ask gemv_id_f32_supported() first.
size_t gemv_id_scratch_ints(int64_t pairs);
bool gemv_id_groups(int64_t pairs, int n_expert);  // enough pairs per expert to bucket them by expert
bool gemv_id_f32_supported(int type, int64_t K, int64_t M, int64_t pairs, int n_expert, bool swiglu = false);
// w2 / y2 (optional): a second stack of the same type and shape against the same activations and ids,
// in the same launch (gate and up of an expert FFN).
// up (optional, with xf; ask gemv_id_f32_supported(..., true)): the rows are silu(xf) * up, produced in the
// prologue (the down projection of an expert FFN).
hipError_t launch_gemv_id(const DevWeight &w, int n_expert, const DevAct &a, const float *xf, const int *ids,
                          int n_used, int n_tokens, int b_cols, float *y, int *groups, hipStream_t s,
                          const DevWeight *w2 = nullptr, float *y2 = nullptr, const float *up = nullptr);
// Gate and up stacks of an expert feed-forward block at decode size (ask gemv_id_f32_supported with twice the
// rows) with the gating in the epilogue: h [n_tokens][n_used][M] = silu(gate product) * up product.
hipError_t launch_gemv_id_pair(const DevWeight &wg, const DevWeight &wu, int n_expert, const float *xf, const int *ids,
                               int n_used, int n_tokens, int b_cols, float *h, hipStream_t s);
// buckets the pairs by expert into groups of at most nc (1..16) pairs: groups[0] = number of groups,
// then records {expert or -1 for ids outside the stack, count, pair[nc]}
hipError_t launch_group_pairs(const int *ids, int pairs, int n_expert, int nc, int *groups, hipStream_t s);

// kernel 3: int8-MFMA GEMM, any N >= 1.  y[n*ldy + m].  workspace (device, may be null) lets the
// launcher cut K into slices when the output alone has too few tiles to fill the GPU;
// gemm_workspace_floats() says how much that takes (0: no split).
hipError_t launch_gemm(const DevWeight &w, const DevAct &a, float *y, int64_t ldy, float *workspace,
                       size_t workspace_floats, int num_cus, hipStream_t s);
bool gemm_supports(int type, int64_t K, int64_t M);
size_t gemm_workspace_floats(int type, int64_t K, int64_t M, int64_t N, int num_cus);
// several weight tensors of one type and K against the same activations in one launch
hipError_t launch_gemm_multi(const DevWeight *ws, float *const *ys, int count, const DevAct &a, float *workspace,
                             size_t workspace_floats, int num_cus, hipStream_t s);
int gemm_max_multi();
// kernel 3b: fp16-MFMA GEMM for Q4_K weights on products with enough 256 x 128 output tiles to fill the GPU;
// a needs the fp16 planes (qf, bsf).  y[n*M + m].  gemm_f16_wanted() depends on the weight and the batch only.
bool gemm_f16_wanted(const DevWeight &w, const DevAct &a, int num_cus);
hipError_t launch_gemm_f16(const DevWeight &w, const DevAct &a, float *y, int num_cus, hipStream_t s);
// Up to four Q4_K matrices of one K in one launch of that kernel (q, k, v; gate, up): wanted when together they fill the
// machine; the bits are those of the single launches.
bool gemm_f16_multi_wanted(const DevWeight *ws, int count, const DevAct &a, int num_cus);
hipError_t launch_gemm_f16_multi(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int num_cus, hipStream_t s);
// kernel 3c: int8-MFMA GEMM for Q6_K weights with 256 x 128 tiles and one accumulator per tile; y[n*M + m].
// gemm_q6k_slices(): 0 = not the kernel for this product (too few tiles), else the K slices it is cut into;
// more than one slice needs gemm_q6k_workspace_floats() floats of device workspace.
int gemm_q6k_slices(int type, int64_t K, int64_t M, int64_t N, int num_cus);
size_t gemm_q6k_workspace_floats(int type, int64_t K, int64_t M, int64_t N, int num_cus);
hipError_t launch_gemm_q6k(const DevWeight &w, const DevAct &a, float *y, float *workspace, size_t workspace_floats,
                           int num_cus, hipStream_t s);
// 1..16 activation columns (col0 .. col0+ncols-1 of a) on the matrix cores, K-quants; y[n*M + m]
bool skinny_supports(int type, int64_t K, int64_t M);
// Q6_K with very many rows, K of 2048 or 4096 and up to 8 columns: launch_skinny then takes a kernel of its own
bool skinny_rows_wanted(const DevWeight &w, int ncols, int num_cus);
hipError_t launch_skinny(const DevWeight &w, const DevAct &a, int col0, int ncols, float *y, int num_cus,
                         hipStream_t s);
// which kernel launch_skinny takes for ncols columns: 1 deep direct-load, 2 many-small-waves direct-load, 3 Q4_K rows
// kernel, 4 staged, 5 Q6_K rows kernel
int skinny_kind(const DevWeight &w, int ncols, int num_cus);
// several K-quant matrices of one type and K in one launch of a skinny kernel (up to 16 columns), when every
// one of them keeps the kernel and K cut of a launch of its own
bool skinny_multi_supports(const DevWeight *ws, int count, int ncols, int num_cus);
hipError_t launch_skinny_multi(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int ncols, int num_cus,
                               hipStream_t s);

// Q4_K at 3..8 columns on large matrices (skinny_deep.hip): weights straight into MFMA operand registers, two
// pieces of four super-blocks in flight per wave, activations resident in LDS.  Up to four matrices of one K per
// launch; the order of the floating-point sums does not depend on the launch geometry.
bool deep16_wanted(int type, int64_t K, int64_t total_m, int ncols, int num_cus);
// The same kernel shape for one Q6_K matrix at 3..8 columns (quantized planes with sd16; launch_deep16_f32 takes a
// single Q6_K matrix too, where deep16_f32_wanted says so).
bool deep6_wanted(int type, int64_t K, int64_t M, int ncols, int num_cus);
hipError_t launch_deep6(const DevWeight &w, float *y, const DevAct &a, int col0, int ncols, int num_cus, hipStream_t s);
hipError_t launch_deep16(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int col0, int ncols, int num_cus,
                         hipStream_t s);
// the same from f32 activations x [ncols][K] (device), quantized by the kernel's workgroups themselves: one launch per
// product group.  Ask deep16_f32_wanted() first (few columns of a short K).
bool deep16_f32_wanted(int type, int64_t K, int64_t total_m, int ncols, int num_cus);
hipError_t launch_deep16_f32(const DevWeight *ws, float *const *ys, int count, const float *x, int ncols, int num_cus, hipStream_t s);

// int8-MFMA GEMM for the 32-element block formats (Q4_0, Q8_0 weights; Q8_0 activations), any N >= 1.
// y[n*M + m].
bool gemm_blk32_supports(int type, int64_t K, int64_t M);
hipError_t launch_gemm_blk32(const DevWeight &w, const DevAct &a, float *y, int num_cus, hipStream_t s);

// 1..16 activation columns on the matrix cores for Q4_0 / Q8_0 (K a multiple of 256); y[n*M + m]
bool skinny32_supports(int type, int64_t K, int64_t M);
hipError_t launch_skinny32(const DevWeight &w, const DevAct &a, int col0, int ncols, float *y, int num_cus,
                           hipStream_t s);
// the same kernel on expert stacks (see launch_gemv_id for the arguments): pairs bucketed 16 to a group
// several Q4_0 / Q8_0 matrices of one K in one launch, when each keeps the K cut of a launch of its own
bool skinny32_multi_supports(const DevWeight *ws, int count, int ncols, int num_cus);
hipError_t launch_skinny32_multi(const DevWeight *ws, float *const *ys, int count, const DevAct &a, int ncols, int num_cus,
                                 hipStream_t s);
bool skinny32_id_supports(int type, int64_t K, int64_t M, int64_t pairs, int n_expert);
hipError_t launch_skinny32_id(const DevWeight &w, int n_expert, const DevAct &a, const int *ids, int n_used, int n_tokens,
                              int b_cols, float *y, int *groups, int num_cus, hipStream_t s);

// Expert GEMM (K-quants, batches with many pairs per expert): sort_pairs sorts the (token, slot) pairs by
// expert into runs of whole 64- or 128-row tiles; the tiled GEMM multiplies every run by its expert's matrix,
// gathering the run's activation rows from the planes (which stay in their own order) and writing each
// result row to its pair's place in y.
//   tiles: 1 + 2 * max_tiles ints; src_col, out_pair: tile_width * max_tiles ints each; hist:
//   sort_pairs_hist_ints() ints (device scratch; with many pairs the sort runs as three launches over chunks)
int64_t sort_pairs_max_tiles(int64_t pairs, int n_expert, int tile_width);
size_t sort_pairs_hist_ints(int64_t pairs, int n_expert);
hipError_t launch_sort_pairs(const int *ids, int pairs, int n_expert, int n_used, int b_cols, int tile_width, int *tiles,
                             int *src_col, int *out_pair, int *hist, hipStream_t s);
bool gemm_id_supports(int type, int64_t K, int64_t M, int64_t pairs, int n_expert);
int gemm_id_tile_width(int type, int64_t pairs, int n_expert);  // pairs per tile the GEMM wants: 64 or 128
hipError_t launch_gemm_id(const DevWeight &w, int n_expert, const DevAct &a, const int *tiles, const int *src_rows,
                          const int *out_rows, int64_t max_tiles, int tile_width, float *y, hipStream_t s);

// Expert-indexed product on the matrix cores (K-quants): the pairs are bucketed by expert, 16 per group;
// a needs the block-sum digit planes.  groups: device scratch of gemv_id_scratch_ints(pairs) ints.
bool skinny_id_supports(int type, int64_t K, int64_t M, int64_t pairs, int n_expert);
hipError_t launch_skinny_id(const DevWeight &w, int n_expert, const DevAct &a, const int *ids, int n_used, int n_tokens,
                            int b_cols, float *y, int *groups, int num_cus, hipStream_t s);

// Unquantized weights (F32, F16, BF16; plain.hip): x f32 [N][K] on the device, y[n*M + m].
//   plain_kind: 0 = not such a product, 1 = streaming kernel (N <= 8, rows a multiple of 16 bytes), 2 = matrix-core tiles
//   (rows a multiple of 64 bytes), 3 = a wave per output (any K), 4 = the streaming kernel, 8 columns per launch,
//   5 = the matrix-core streaming kernel (N <= 16, rows a multiple of 64 bytes, the converted x fits the LDS).
//   force: 0 = as plain_kind says, 1 = never the tiles, 2 = the tiles or an error.
//   xc: device scratch of plain_convert_bytes() bytes for the converted activations of kind 2 (F16 / BF16).
bool plain_type(int type);
int plain_kind(int type, int64_t K, int64_t M, int64_t N, int force = 0);
size_t plain_convert_bytes(int type, int64_t K, int64_t N);
hipError_t launch_plain(const DevWeight &w, const float *x, int64_t N, float *y, void *xc, int num_cus, hipStream_t s, int force = 0);

}  // namespace miqmm
