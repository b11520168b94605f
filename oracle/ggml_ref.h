/*
 * CPU oracle for the GGUF block-quantized matmul path  --  TEST INFRASTRUCTURE ONLY.
 *
 * A scalar C restatement of the ggml CPU backend's semantics for
 *   mul_mat(W quantized {Q4_0,Q8_0,Q4_K,Q5_K,Q6_K} or plain {F32,F16,BF16}, X f32) -> Y f32
 * i.e. activation quantization to Q8_0 / Q8_K followed by the per-type integer dot products.
 * Nothing in the shipped library links or calls this file: it is the checker the GPU path is
 * compared against, and the timed "port" CPU baseline.
 *
 * The arithmetic lives in llama.cpp (ggml) at the tag the reference pins in
 * /root/reference/LLAMA_CPP_VERSION:1 (b10488); that source is fetched at configure time
 * (/root/reference/llama/server/CMakeLists.txt:112-188) and is not present offline, so this
 * file restates the published algorithms (ggml-quants.c *_ref quantizers, ggml-cpu/quants.c
 * generic vec_dot loops, ggml-cpu.c mul_mat driver).  What the reference itself pins:
 *   block/type sizes      /root/reference/fs/ggml/ggml.go:407-513, ggml_test.go:163-213
 *   ggml_type ids         /root/reference/fs/ggml/type.go:250-293
 *   call shape            /root/reference/ml/backend.go:151 (Tensor.Mulmat)
 *
 * Parity status per function (what pins it is in tests/test_oracle_*.py):
 *   fp16<->fp32, q8_0/q8_K quantizers, 6-bit scale unpack, five vec_dots (Q5_K among them), dequantizers,
 *   mul_mat driver:  pinned (numpy float16, closed forms, fp64 brute force, KATs).
 *   F32 / F16 / BF16 weights (activations converted to the weight's type, products in fp32, sum in double):
 *   pinned as mathematics (numpy float16 casts, bfloat16 rounding against an integer statement of
 *   round-to-nearest-even over every 16-bit pattern and its neighbours, fp64 dot products of the converted
 *   operands).  Upstream's SIMD variants sum in fp32 lanes: PARITY UNPINNED below 1e-6 relative.
 *   mul_mat_id driver: the per-pair arithmetic is the pinned vec_dots; the indexing is pinned by
 *   its reduction to mul_mat (one expert; a pair's result equals mul_mat on that expert alone) and
 *   fp64 brute force.  The rule "slot i reads activation row i mod ne11" is upstream ggml's and the
 *   reference holds no test of it: PARITY UNPINNED for b_cols other than 1 and n_used.
 *   rms_norm / swiglu (the producers in front of the path): pinned as mathematics (closed forms for
 *   constant and one-hot rows, scale invariance, silu(v) - silu(-v) = v, fp64 evaluation with numpy
 *   to 1e-6); the fp32 rounding of upstream's SIMD variants (vectorized expf, reduction order of the
 *   sum of squares) is not fixed by anything in the reference: PARITY UNPINNED below 1e-6 relative.
 *   weight encoders q4_K / q6_K (make_qkx2_quants / make_qx_quants searches):
 *   PARITY UNPINNED bit-for-bit against llama-quantize.  What mathematics fixes is checked in fp64: the
 *   returned (scale, min) is the weighted least-squares optimum for the returned levels, no candidate of
 *   the search grid fits better, the result never fits worse than the min/max start, the stored levels
 *   are the nearest ones for the stored scales.  That catches slips of transcription, not of recall.
 *   q4_0 / q8_0 encoders are closed forms and pinned.
 */
#ifndef GGML_REF_H
#define GGML_REF_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml_type ids, /root/reference/fs/ggml/type.go:250-268 */
enum { REF_TYPE_F32 = 0, REF_TYPE_F16 = 1, REF_TYPE_BF16 = 30, REF_TYPE_MXFP4 = 39, REF_TYPE_Q4_0 = 2, REF_TYPE_Q5_0 = 6, REF_TYPE_Q8_0 = 8, REF_TYPE_Q4_K = 12, REF_TYPE_Q5_K = 13,
       REF_TYPE_Q6_K = 14, REF_TYPE_Q8_K = 15 };

int64_t ref_block_size(int type);               /* elements per block, 0 if unknown */
int64_t ref_type_size(int type);                /* bytes per block                 */
int64_t ref_row_size(int type, int64_t k);      /* bytes of a row of k elements, -1 if k % block */

uint16_t ref_fp32_to_fp16(float f);
float    ref_fp16_to_fp32(uint16_t h);
uint16_t ref_fp32_to_bf16(float f);             /* round to nearest even, NaNs made quiet */
float    ref_bf16_to_fp32(uint16_t h);

/* activation quantizers (canonical scalar *_ref semantics) */
void ref_quantize_row_q8_0(const float *x, void *y, int64_t k);
void ref_quantize_row_q8_K(const float *x, void *y, int64_t k);

/* weight encoders */
void ref_quantize_row_q4_0(const float *x, void *y, int64_t k);
void ref_quantize_row_q4_K(const float *x, void *y, int64_t k);
void ref_quantize_row_q6_K(const float *x, void *y, int64_t k);
/* dispatch on type (2, 8, 12, 14, 15; 0, 1, 30: conversion of the row to f32 / f16 / bf16); rows are independent.
 * returns 0 or -1 */
int  ref_quantize(int type, const float *x, void *y, int64_t k, int64_t rows, int nthreads);

/* The two searches inside the K-quant encoders, callable on one group of values so that tests can check what they
 * return against what least squares fixes.  q4_K calls the first with (32, 15, x, av_x + |x|, ..., -1, 0.1, 20) per
 * 32 values, q6_K the second with (16, 32, x) per 16 values (weights x^2). */
float ref_qkx2_search(int n, int nmax, const float *x, const float *weights, uint8_t *levels, float *neg_min,
                      float rmin, float rdelta, int nstep);
float ref_qx_search(int n, int nmax, const float *x, int8_t *levels);

/* dequantizers */
int  ref_dequantize_row(int type, const void *x, float *y, int64_t k);

/* 6-bit scale/min unpack of a Q4_K block header (both published formulations) */
void ref_get_scale_min_k4(int j, const uint8_t *s12, uint8_t *sc, uint8_t *m);
void ref_unpack_scales_kmask(const uint8_t *s12, uint8_t sc[8], uint8_t m[8]);

/* dot products: n elements, x = weight row blocks, y = activation row blocks */
float ref_vec_dot_q4_0_q8_0(int64_t n, const void *x, const void *y);
float ref_vec_dot_q8_0_q8_0(int64_t n, const void *x, const void *y);
float ref_vec_dot_q5_0_q8_0(int64_t n, const void *x, const void *y);
float ref_vec_dot_mxfp4_q8_0(int64_t n, const void *x, const void *y);
float ref_e8m0_to_fp32_half(uint8_t e);   /* 2^(e - 128): half the E8M0 scale (ggml keeps the E2M1 values doubled) */
float ref_vec_dot_q4_K_q8_K(int64_t n, const void *x, const void *y);
float ref_vec_dot_q5_K_q8_K(int64_t n, const void *x, const void *y);
float ref_vec_dot_q6_K_q8_K(int64_t n, const void *x, const void *y);
/* the unquantized types: both rows in the weight's type, products in fp32, sum in double in element order */
float ref_vec_dot_f32(int64_t n, const void *x, const void *y);
float ref_vec_dot_f16(int64_t n, const void *x, const void *y);
float ref_vec_dot_bf16(int64_t n, const void *x, const void *y);

/* the activation type the CPU path converts to for a given weight type (8 or 15; 0, 1, 30 for the weight types
 * F32, F16, BF16 themselves), -1 unknown */
int  ref_vec_dot_type(int wtype);

/*
 * mul_mat driver: W is M rows of K elements in GGUF block layout, X is N rows of K floats,
 * Y[n*M + m] = vec_dot(W row m, Q(X row n)).  xq_out (optional) receives the quantized
 * activation rows (N * row_size(vec_dot_type, K) bytes).  returns 0 or -1 on bad arguments.
 */
int  ref_mul_mat(int wtype, const void *w, int64_t k, int64_t m,
                 const float *x, int64_t n, float *y, void *xq_out, int nthreads);

/*
 * mul_mat_id: as = n_expert matrices of M rows of K elements, one after the other; b = f32
 * [n_tokens][b_cols][K]; ids = int32 [n_tokens][n_used];
 * y[(t*n_used + i)*M + m] = vec_dot(as[ids[t][i]] row m, Q(b[t][i % b_cols])).
 * returns 0, -1 on bad arguments, -2 when an id is outside 0..n_expert-1.
 */
int  ref_mul_mat_id(int wtype, const void *as, int64_t k, int64_t m, int64_t n_expert, const float *b,
                    int64_t b_cols, const int32_t *ids, int64_t n_used, int64_t n_tokens, float *y);

/*
 * Producers of the activations (Tensor.RMSNorm, Tensor.SILU(up): /root/reference/ml/backend.go:159, :180).
 * rms_norm: x [n][k]; g [k] or NULL; y[r][i] = (x[r][i] * scale_r) * g[i], scale_r = 1/sqrtf(mean(x_r^2) + eps).
 * swiglu:   y[i] = silu(gate[i]) * up[i] over count elements.
 */
void ref_rms_norm(const float *x, const float *g, float eps, int64_t k, int64_t n, float *y);
void ref_swiglu(const float *gate, const float *up, int64_t count, float *y);

#ifdef __cplusplus
}
#endif
#endif
