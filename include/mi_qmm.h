/*
 * mi_qmm -- MI355X (gfx950) GGUF block-quantized matmul, C ABI.
 *
 * The drop-in boundary for the one hot path of Ollama's tensor backend:
 *     y = W.Mulmat(ctx, x)       /root/reference/ml/backend.go:151  (ml.Tensor.Mulmat)
 * with W a GGUF block-quantized weight (Q4_0, Q8_0, Q4_K, Q6_K) loaded by fs/ggml and x f32
 * activations, i.e. ggml's mul_mat(W, x): W.Shape() = [K, M], x.Shape() = [K, N] (dim 0
 * contiguous) -> f32 [M, N].  The arithmetic is ggml's CPU-backend semantics: x is quantized to
 * Q8_0 (for Q4_0/Q8_0 weights) or Q8_K (for Q4_K/Q6_K weights) and every output is the integer
 * block dot product scaled in fp32.
 *
 * Plain C: opaque handles, plain pointers and sizes, int status returns (0 = ok, negative =
 * error, text via mi_qmm_last_error(), which is thread-local).  No callbacks, nothing retains a
 * caller pointer after the call returns (the cgo pointer-passing rule), no call depends on
 * thread-affine state: the device is re-asserted from the handle on every call, so calls may come
 * from any OS thread.  Calls on one ctx must not overlap in time; use one ctx per goroutine/thread
 * that drives the GPU.
 *
 * There is no CPU fallback: without a usable gfx950 device mi_qmm_init fails and every compute
 * entry point needs a ctx.
 */
#ifndef MI_QMM_H
#define MI_QMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mi_qmm_ctx mi_qmm_ctx;       /* one device + one stream + scratch workspace      */
typedef struct mi_qmm_weight mi_qmm_weight; /* one weight tensor resident in HBM (device layout) */

/* status codes */
enum {
    MI_QMM_OK = 0,
    MI_QMM_ERR_INVALID = -1,     /* bad argument (null pointer, negative size, K not a block multiple) */
    MI_QMM_ERR_UNSUPPORTED = -2, /* ggml type or shape outside what the kernels cover               */
    MI_QMM_ERR_HIP = -3,         /* a HIP runtime call failed; message carries hipGetErrorString    */
    MI_QMM_ERR_NOMEM = -4,       /* device or host allocation failed                                */
    MI_QMM_ERR_NODEVICE = -5     /* no gfx950 device at that ordinal                                */
};

/* ggml_type ids this path uses -- /root/reference/fs/ggml/type.go:250-268 */
enum {
    MI_QMM_TYPE_F32 = 0,
    MI_QMM_TYPE_F16 = 1,
    MI_QMM_TYPE_Q4_0 = 2,
    MI_QMM_TYPE_Q5_0 = 6,
    MI_QMM_TYPE_Q8_0 = 8,
    MI_QMM_TYPE_Q4_K = 12,
    MI_QMM_TYPE_Q5_K = 13,
    MI_QMM_TYPE_Q6_K = 14,
    MI_QMM_TYPE_Q8_K = 15,
    MI_QMM_TYPE_BF16 = 30,
    MI_QMM_TYPE_MXFP4 = 39
};

/* where x / y / weight bytes live */
enum { MI_QMM_HOST = 0, MI_QMM_DEVICE = 1 };

/* kernel selection for mi_qmm_mulmat_path */
enum {
    MI_QMM_PATH_AUTO = 0, /* decode kernels below N = 32, tiled int8-MFMA GEMM from N = 32             */
    MI_QMM_PATH_GEMV = 1, /* the decode kernels at any N: streaming GEMV, 8 columns at a time; from
                             3 (Q4_K) / 4 (Q6_K, Q4_0, Q8_0) columns the skinny matrix-core kernels,
                             16 columns at a time                                                    */
    MI_QMM_PATH_GEMM = 2, /* force the tiled int8-MFMA GEMM (any N >= 1, padded to the tile)          */
    MI_QMM_PATH_QUERY = 3 /* launch nothing: return the MI_QMM_ROUTE_* value of the kernel that
                             MI_QMM_PATH_AUTO would take for this weight and n (x and y may be NULL).
                             No counterpart in the reference; for tests that pin the routing table.  */
};

/* what MI_QMM_PATH_QUERY returns: the kernel a product takes.  It depends on the weight's type and shape, on n and
 * on the form the activations come in (f32 for mi_qmm_mulmat_path, quantized planes for mi_qmm_mulmat_q8) only. */
enum {
    MI_QMM_ROUTE_GEMV_F32 = 1,         /* streaming GEMV, x quantized in its prologue (one launch)               */
    MI_QMM_ROUTE_DEEP_F32 = 2,         /* Q4_K deep direct-load kernel, x quantized by its workgroups (one launch) */
    MI_QMM_ROUTE_GEMM_BLK32 = 3,       /* Q4_0 / Q8_0 int8-MFMA GEMM                                              */
    MI_QMM_ROUTE_GEMM_F16 = 4,         /* Q4_K fp16-MFMA GEMM, 256 x 128 tiles                                    */
    MI_QMM_ROUTE_GEMM_Q6K = 5,         /* Q6_K int8-MFMA GEMM, 256 x 128 tiles, K slices                          */
    MI_QMM_ROUTE_GEMM_INT8 = 6,        /* K-quant int8-MFMA GEMM, 128-row tiles                                   */
    MI_QMM_ROUTE_SKINNY32 = 7,         /* Q4_0 / Q8_0 matrix-core kernel for 2..31 columns                        */
    MI_QMM_ROUTE_SKINNY_DEEP = 8,      /* Q4_K deep direct-load kernel on quantized planes                        */
    MI_QMM_ROUTE_SKINNY_DIRECT = 9,    /* Q4_K direct-load kernel of many small waves (small matrices, <= 4 columns) */
    MI_QMM_ROUTE_SKINNY_ROWS_Q4K = 10, /* Q4_K rows kernel (activations resident in LDS, a wave per row group)    */
    MI_QMM_ROUTE_SKINNY_STAGED = 11,   /* K-quant staged matrix-core kernel for 3..31 columns                     */
    MI_QMM_ROUTE_SKINNY_ROWS_Q6K = 12, /* Q6_K rows kernel (the output head at 2..8 columns)                      */
    MI_QMM_ROUTE_GEMV = 13,            /* streaming GEMV on quantized planes                                      */
    MI_QMM_ROUTE_PLAIN_GEMV = 14,      /* F32 / F16 / BF16 weights: vector-ALU streaming kernel, 1..8 columns      */
    MI_QMM_ROUTE_PLAIN_GEMM = 15,      /* F32 / F16 / BF16 weights: tiles on the f32 / f16 / bf16 matrix cores     */
    MI_QMM_ROUTE_PLAIN_NAIVE = 16,     /* F32 / F16 / BF16 weights whose rows are no multiple of 16 bytes          */
    MI_QMM_ROUTE_PLAIN_SKINNY = 17     /* F32 / F16 / BF16 weights at 1..16 columns: weights straight into MFMA operands */
};

/* ---- size tables: replace TensorType.BlockSize / TypeSize and Tensor.Size's row rule
 *      /root/reference/fs/ggml/ggml.go:407-436 (BlockSize), :442-513 (TypeSize), :550-556 (row rule).
 *      Cover every ggml_type id of that table, not only the four weight types. 0 = unknown id. */
int64_t mi_qmm_block_size(int ggml_type);
int64_t mi_qmm_type_size(int ggml_type);
/* bytes of one row of k elements; -1 when the id is unknown or k is not a multiple of the block */
int64_t mi_qmm_row_size(int ggml_type, int64_t k);
/* activation type the path converts x to for a weight type: 8 (Q8_0), 15 (Q8_K); the unquantized weight types
 * 0 (F32), 1 (F16) and 30 (BF16) are multiplied in their own type; -1 if the weight type is not supported --
 * ggml type_traits_cpu[type].vec_dot_type */
int mi_qmm_vec_dot_type(int weight_type);

/* ---- lifetime: replaces Backend construction / Close, /root/reference/ml/backend.go:16-18, 78-92.
 *      device_ordinal indexes the HIP device list the process sees (already filtered by
 *      ROCR_VISIBLE_DEVICES, /root/reference/ml/device.go:688-735); 0 is the normal value. */
int mi_qmm_init(int device_ordinal, mi_qmm_ctx **out);
void mi_qmm_destroy(mi_qmm_ctx *ctx);
/* run on a caller-owned hipStream_t (e.g. the framework's current stream); NULL restores the
 * ctx's own stream.  The ctx never destroys a caller stream.  The call waits for the work queued on
 * the previous stream.  With device pointers the product entry points only queue kernels once the
 * ctx's scratch buffers have reached their size (first call of a shape), so such calls may be
 * captured into a HIP graph on the caller's stream after one eager call. */
int mi_qmm_set_stream(mi_qmm_ctx *ctx, void *hip_stream);
/* Scratch and captured graphs.  The product entry points keep quantized activations, K-split partial sums
 * and host staging in scratch buffers that belong to the ctx and GROW on demand: a call that needs more
 * than any earlier call frees the old buffer and allocates a larger one.  A HIP graph captured earlier
 * still holds the old addresses, and replaying it after such a call would touch freed memory.  So:
 * run every shape the graph's lifetime will see once (largest first is enough), then freeze.  While
 * frozen (frozen != 0) a call that would have to grow any scratch returns MI_QMM_ERR_INVALID and leaves
 * the buffers alone; frozen = 0 allows growth again (re-capture afterwards). */
int mi_qmm_scratch_freeze(mi_qmm_ctx *ctx, int frozen);
/* block until everything queued on the ctx's stream has finished */
int mi_qmm_sync(mi_qmm_ctx *ctx);

/* Page-locked host memory for x / y buffers of MI_QMM_HOST calls: the copies to and from the device
 * then run at full PCIe rate and without a staging copy inside the driver.  A cgo caller keeps Go
 * pointers out of C this way too (the buffer is C memory; cf. the static trampolines of
 * /root/reference/discover/native_probe_linux.go:26-54).  Plain pointers: any entry point accepts
 * them wherever it accepts host memory.  NULL (and an error message) when the allocation fails.
 * mi_qmm_host_free does not use its ctx argument (it may be NULL or already destroyed). */
void *mi_qmm_host_alloc(mi_qmm_ctx *ctx, size_t bytes);
void mi_qmm_host_free(mi_qmm_ctx *ctx, void *p);

/* ---- weights: replaces Backend.Load + Backend.Get(name), /root/reference/ml/backend.go:20, 26,
 *      fed with the tensor bytes fs/ggml hands out (/root/reference/fs/ggml/gguf.go:281-308;
 *      fs/gguf/gguf.go:388-430): M rows of K elements in GGUF block layout, rows contiguous.
 *      The bytes are copied (and re-laid-out for the device) before the call returns.
 *      ggml_type: the block-quantized types 2 (Q4_0), 8 (Q8_0), 12 (Q4_K), 14 (Q6_K); 13 (Q5_K), which the
 *      Q4_K_S mixture of the reference's file types gives some tensors; and the unquantized ones a GGUF file
 *      holds beside them or instead of them, 0 (F32), 1 (F16), 30 (BF16): together every tensor type of the file
 *      types /root/reference/fs/ggml/type.go:55-88 accepts, the tensors a K-quant file keeps unquantized and the
 *      ones /root/reference/server/quantization.go:296-333 keeps at f16.  Q5_K and the unquantized types go
 *      through mi_qmm_mulmat, mi_qmm_mulmat_path, mi_qmm_mulmat_noalloc and mi_qmm_mulmat_multi (one product
 *      after the other there); the produced, expert-indexed and pre-quantized entry points take Q4_0 / Q8_0 /
 *      Q4_K / Q6_K weights only and return MI_QMM_ERR_UNSUPPORTED otherwise.  A Q5_K tensor is kept as the Q4_K
 *      tensor of rows twice as long that gives the same integer sums against [x | x] (1.64 times the bytes of
 *      the file: its products cost what a Q4_K product of twice the K costs) and, for up to six activation rows
 *      (eight on tensors of up to 8 Mi weights), as the blocks themselves, which the streaming kernel reads at their own
 *      176 bytes (from three rows on, and at two on long rows, against x quantized once by a launch in front of it).  39 (MXFP4, the expert tensors of
 *      /root/reference/convert/convert_gptoss.go:124-150; DTypeMXFP4, /root/reference/ml/backend.go:404-412) is kept
 *      as the Q8_0 planes that give the same dot products -- the doubled E2M1 values as int8, the scale 2^(e - 128)
 *      as the block scale, twice the bytes of the file -- and goes through every entry point a Q8_0 weight goes
 *      through, the expert-indexed ones included, when k is a multiple of 256.  Otherwise (k = 2880) its rows are
 *      kept padded with zero blocks to the next multiple of 256 and the library pads the activation rows likewise
 *      inside mi_qmm_mulmat, _path, _noalloc, _multi and mi_qmm_mulmat_id; the other entry points then return
 *      MI_QMM_ERR_UNSUPPORTED.  The tensor is also kept in its own layout, which the streaming kernels (one or
 *      two activation rows, a few pairs per expert) read at half the bytes.  A scale byte above 146 is
 *      MI_QMM_ERR_UNSUPPORTED; blocks with a scale byte below 104 (weights under 7.2e-7) are zeros in the Q8_0
 *      planes (the matrix-core kernels) and exact in the streaming kernels.  6 (Q5_0) is kept as Q8_0 planes in the
 *      same way (its 5-bit values minus 16 as int8 under the block's own scale: the same dot products, term for
 *      term) with the same rule for rows that are no multiple of 256.
 *      src_location: MI_QMM_HOST or MI_QMM_DEVICE. */
int mi_qmm_weight_upload(mi_qmm_ctx *ctx, int ggml_type, const void *gguf_bytes, int64_t k,
                         int64_t m, int src_location, mi_qmm_weight **out);
void mi_qmm_weight_free(mi_qmm_weight *w);
int mi_qmm_weight_info(const mi_qmm_weight *w, int *ggml_type, int64_t *k, int64_t *m,
                       int64_t *device_bytes);

/* ---- weight encoders on the GPU: f32 rows -> GGUF blocks of Q4_0, Q8_0, Q4_K or Q6_K.  Replaces what the
 *      reference obtains by running llama-quantize (/root/reference/server/quantization.go:125-181,
 *      /root/reference/server/create.go:931-944): for these four types and no importance matrix that tool
 *      encodes every row with ggml's scalar quantize_row_*_ref.  The kernels follow the order of operations of
 *      this repository's C restatement of those routines (oracle/ggml_ref.c) and produce its bytes, which the GPU
 *      tests check; for Q4_K and Q6_K the restatement itself could not be compared offline with the bytes a
 *      compiled llama-quantize writes, so parity with that tool is not pinned for the two K-quant encoders
 *      (Q4_0 and Q8_0 are pinned by closed forms).  (Which tensor gets which type -- the Q4_K_M mixture --
 *      stays with the caller.)  x: f32 [m][k]; out_blocks receives m * row_size(ggml_type, k) bytes, ready for
 *      mi_qmm_weight_upload or a GGUF file.  location applies to both x and out_blocks; device pointers: x
 *      16-byte aligned, out_blocks 4-byte aligned (queued on the ctx stream, returns without waiting). */
int mi_qmm_quantize_weights(mi_qmm_ctx *ctx, int ggml_type, const float *x, int64_t k, int64_t m,
                            void *out_blocks, int location);

/* ---- activation quantization on the GPU: replaces ggml's from_float step of mul_mat
 *      (quantize_row_q8_0 / quantize_row_q8_K, canonical scalar semantics).
 *      x: f32 [n][k]; out_blocks receives n * row_size(q8_type, k) bytes in GGUF block layout,
 *      bit-identical to the CPU path.  location applies to both x and out_blocks. */
int mi_qmm_quantize_act(mi_qmm_ctx *ctx, int q8_type, const float *x, int64_t k, int64_t n,
                        void *out_blocks, int location);

/* ---- the product: replaces Tensor.Mulmat + Context.Compute + Tensor.Floats,
 *      /root/reference/ml/backend.go:151, 110, 140.
 *      x: f32 [n][k], y: f32 [n][m] with y[i*m + r] = dot(W row r, Q8(x row i)); for F32 / F16 / BF16
 *      weights Q8 is the conversion of x to the weight's own type (round to nearest even) and the products
 *      are formed and added in fp32 (ggml_vec_dot_f32 / _f16 / _bf16 add them in double: the difference is
 *      far inside the path's 1e-3 tolerance).
 *      location = MI_QMM_HOST: copies in, computes, copies out and returns when y is complete.
 *      location = MI_QMM_DEVICE: x and y are device pointers; the work is queued on the ctx's
 *      stream and the call returns without waiting (mi_qmm_sync or stream order to consume). */
int mi_qmm_mulmat(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const float *x, int64_t n, float *y,
                  int location);
int mi_qmm_mulmat_path(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const float *x, int64_t n,
                       float *y, int location, int path);
/* mi_qmm_mulmat for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): x and y are DEVICE pointers, the work is queued on
 * the ctx's stream, and the call never allocates or frees -- neither device memory nor the ctx's growable
 * scratch.  It has no counterpart in the reference (ggml's CPU mul_mat gets its work buffer from the
 * caller's graph plan); it exists for those callers.  The quantized activations go to a static device
 * array of MI_QMM_NOALLOC_SCRATCH_BYTES that each GPU the library runs on holds until the process ends;
 * a call whose quantized activations do not fit (about n * k * 1.4 bytes for Q4_K / Q6_K weights from
 * three or four rows up -- n * k * 3.4 for Q4_K weights from 65 rows up, where the planes of the fp16 GEMM
 * are written too; n is rounded up to a multiple of 128 for these types -- and n * k * 1.2 for Q4_0 / Q8_0;
 * one to a few rows need no scratch at all) returns MI_QMM_ERR_UNSUPPORTED.  Every call on a GPU shares that GPU's array: calls that overlap in time on
 * one GPU (two streams, two ctxs) race.  Results are those of mi_qmm_mulmat (bit-identical, except that
 * the tiled GEMM never cuts K into slices here, which changes the order of its fp32 sums). */
#define MI_QMM_NOALLOC_SCRATCH_BYTES (16u << 20)
int mi_qmm_mulmat_noalloc(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const float *x, int64_t n, float *y);
/* several weights of the same k against the same f32 activations x [n][k]: ys[i] receives
 * f32 [n][m_i].  These are the mul_mat nodes of one graph that share src1 (gate and up, or q/k/v),
 * which Context.Compute (/root/reference/ml/backend.go:110) sees together.  For weights of one
 * type, one or two columns (three for some formats and sizes) and count <= 4 this is ONE kernel
 * launch: the decode GEMV quantizes x in its prologue and walks the concatenated rows of all weights.
 * Otherwise x is quantized once per activation format in use and the products follow, weights of one
 * type sharing launches four at a time while n <= 16 where a kernel takes them together (the GEMV; the
 * matrix-core kernels for Q4_K).  Results are those of mi_qmm_mulmat per weight. */
int mi_qmm_mulmat_multi(mi_qmm_ctx *ctx, const mi_qmm_weight *const *ws, int count, const float *x,
                        int64_t n, float *const *ys, int location);

/* Producers of the activations: the two graph nodes that feed the quantized products of a transformer
 * block, fused into the quantization so that their f32 result never goes through memory.
 *   MI_QMM_PRODUCE_RMSNORM  Tensor.RMSNorm(ctx, weight, eps)  (/root/reference/ml/backend.go:159):
 *       x' = (x * scale) * aux,  scale = 1 / sqrtf(mean(x^2) + eps) per row;  aux = the norm weight
 *       f32 [k], or NULL for the bare normalization
 *   MI_QMM_PRODUCE_SWIGLU   Tensor.SILU(ctx, up)  (/root/reference/ml/backend.go:180):
 *       x' = silu(x) * aux,  silu(v) = v / (1 + expf(-v));  aux = up, f32 [n][k] like x
 * ggml's scalar arithmetic: squares in fp32 accumulated in double, the mean rounded to fp32, the two
 * multiplies of RMSNorm rounded separately.  expf is the device library's (within 1 ulp). */
enum {
    MI_QMM_PRODUCE_NONE = 0,
    MI_QMM_PRODUCE_RMSNORM = 1,
    MI_QMM_PRODUCE_SWIGLU = 2,
};
/* mi_qmm_mulmat_multi on x' = producer(x): ys[i] = ws[i] * Q8(x').  With one activation row (decode)
 * and weights of one type this is ONE kernel launch: every workgroup of the GEMV normalizes / gates x,
 * quantizes it and walks its rows.  Otherwise x' is quantized once per activation format by a fused
 * quantizer (RMSNorm: after one launch for the row scales) and the products follow.  aux lives where x
 * does (location).  Results are bit-identical to mi_qmm_rms_norm / mi_qmm_swiglu followed by
 * mi_qmm_mulmat_multi. */
int mi_qmm_mulmat_produced(mi_qmm_ctx *ctx, const mi_qmm_weight *const *ws, int count, int producer,
                           const float *aux, float eps, const float *x, int64_t n, float *const *ys,
                           int location);
/* Gate and up of a feed-forward block together with their gating -- the graph pattern
 * gate.SILU(ctx, up) with gate = w_gate.Mulmat(x') and up = w_up.Mulmat(x'), x' = x or RMSNorm(x)
 * (producer MI_QMM_PRODUCE_NONE or _RMSNORM with aux = norm weight [k] or NULL):
 *     h[i][r] = silu(w_gate row r . Q8(x'[i])) * (w_up row r . Q8(x'[i])),  h f32 [n][m].
 * With one activation row this is ONE launch: a wave walks row r of both matrices, and whoever holds
 * the two totals of a row gates them, so neither product goes through memory and silu is evaluated
 * once per element.  Larger n: the two products (mi_qmm_mulmat_produced) and mi_qmm_swiglu.
 * Bit-identical to those either way. */
int mi_qmm_mulmat_swiglu(mi_qmm_ctx *ctx, const mi_qmm_weight *w_gate, const mi_qmm_weight *w_up, int producer,
                         const float *aux, float eps, const float *x, int64_t n, float *h, int location);
/* The same producers as plain f32 operations, for graph nodes that something other than a product
 * reads: x, y f32 [n][k] (k a multiple of 4), g f32 [k] or NULL; gate, up, y f32 [n][k] (any k).
 * up == NULL: the bare activation y = silu(gate), Tensor.SILU(ctx) without an operand
 * (/root/reference/ml/backend.go:180 is variadic). */
int mi_qmm_rms_norm(mi_qmm_ctx *ctx, const float *x, const float *g, float eps, int64_t k, int64_t n,
                    float *y, int location);
int mi_qmm_swiglu(mi_qmm_ctx *ctx, const float *gate, const float *up, int64_t k, int64_t n, float *y,
                  int location);

/* Expert-indexed product, Tensor.MulmatID (/root/reference/ml/backend.go:153).  w is a stack of
 * n_expert matrices uploaded as ONE weight of m = rows_per_expert * n_expert rows: GGUF stores expert
 * tensors with ne = [in, out, experts] (/root/reference/convert/convert_gemma4.go:274-275), so the
 * bytes of the 3-D tensor are that 2-D weight unchanged.  x is f32 [n_tokens][b_cols][k], ids is
 * int32 [n_tokens][n_used], y receives f32 [n_tokens][n_used][rows_per_expert]:
 *     y[t][i][:] = W[ids[t][i]] * Q8(x[t][i % b_cols][:])
 * (b_cols = 1: all slots of a token share one activation row, as for gate/up; b_cols = n_used: every
 * slot has its own, as for the down projection.)  location covers x, ids and y alike.  With ids in
 * host memory an id outside 0..n_expert-1 is MI_QMM_ERR_INVALID (ggml aborts there); with ids in
 * device memory the call cannot see them and the rows of such a pair come back as NaN.
 * The kernel follows n_tokens * n_used / n_expert: one streaming product per pair (decode), pairs
 * bucketed by expert on the device for the 16-column matrix-core kernel, and from 16 pairs per expert
 * (Q4_K / Q6_K) pairs sorted by expert and multiplied tile by tile on the matrix cores.  Scratch for
 * the buckets comes from the ctx's workspace, which grows on demand (a device allocation on the
 * first call of a new size). */
int mi_qmm_mulmat_id(mi_qmm_ctx *ctx, const mi_qmm_weight *w, int n_expert, const float *x, int b_cols,
                     const int32_t *ids, int n_used, int64_t n_tokens, float *y, int location);

/* several expert stacks against the same x and ids (gate and up of an expert FFN): ys[i] receives
 * f32 [n_tokens][n_used][rows_per_expert_i].  Stacks of one type and shape go out two at a time with x
 * quantized once; for decode-sized calls such a pair is ONE kernel launch.  Results are those of
 * mi_qmm_mulmat_id per stack. */
int mi_qmm_mulmat_id_multi(mi_qmm_ctx *ctx, const mi_qmm_weight *const *ws, int count, int n_expert,
                           const float *x, int b_cols, const int32_t *ids, int n_used, int64_t n_tokens,
                           float *const *ys, int location);
/* Gate and up of an EXPERT feed-forward block with their gating: mi_qmm_mulmat_swiglu for expert stacks,
 *     h[t][i][:] = silu(Wg[ids[t][i]] * Q8(x[t][i % b_cols])) * (Wu[ids[t][i]] * Q8(x[t][i % b_cols])),
 * h f32 [n_tokens][n_used][rows_per_expert]; arguments as for mi_qmm_mulmat_id.  Decode-sized calls are one
 * launch (a wave walks row j of the pair's expert in both stacks and gates the two totals); larger ones
 * the two products and mi_qmm_swiglu.  Bit-identical to those either way. */
int mi_qmm_mulmat_id_swiglu(mi_qmm_ctx *ctx, const mi_qmm_weight *w_gate, const mi_qmm_weight *w_up, int n_expert,
                            const float *x, int b_cols, const int32_t *ids, int n_used, int64_t n_tokens, float *h,
                            int location);

/* mi_qmm_mulmat_id on x' = producer(x) (the producers of mi_qmm_mulmat_produced): the down projection of
 * an expert feed-forward block reads silu(gate) * up, x = gate and aux = up being the two
 * [n_tokens][b_cols][k] results of the gate / up stacks.  Decode-sized calls gate and quantize each
 * pair's row in the prologue of its product (one launch); larger ones quantize x' once with the fused
 * quantizer.  RMSNorm: aux = the norm weight [k] or NULL.  Bit-identical to mi_qmm_swiglu /
 * mi_qmm_rms_norm followed by mi_qmm_mulmat_id. */
int mi_qmm_mulmat_id_produced(mi_qmm_ctx *ctx, const mi_qmm_weight *w, int n_expert, int producer,
                              const float *aux, float eps, const float *x, int b_cols, const int32_t *ids,
                              int n_used, int64_t n_tokens, float *y, int location);

/* ---- two-phase form: quantize once, multiply by several weights (gate and up, or q/k/v, share
 *      one x).  In ggml's graph the from_float step belongs to each mul_mat node; a backend that
 *      sees the whole graph at Context.Compute (/root/reference/ml/backend.go:110) may hoist it,
 *      which is what these entry points are for.  An mi_qmm_act owns device storage for up to
 *      n_max rows of k elements in the ctx's device; it is reusable across calls. */
typedef struct mi_qmm_act mi_qmm_act;
int mi_qmm_act_create(mi_qmm_ctx *ctx, int q8_type, int64_t k, int64_t n_max, mi_qmm_act **out);
void mi_qmm_act_free(mi_qmm_act *act);
/* x: f32 [n][k] (n <= n_max), quantized on the ctx's stream into act */
int mi_qmm_act_quantize(mi_qmm_ctx *ctx, mi_qmm_act *act, const float *x, int64_t n, int location);
/* y: f32 [n][m] from the rows last quantized into act; act's type must be
 * mi_qmm_vec_dot_type(weight type) and its k the weight's k */
int mi_qmm_mulmat_q8(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const mi_qmm_act *act, float *y,
                     int location, int path);

/* several weights of one type and k against the same activations: ys[i] receives f32 [n][m_i].
 * For count <= 4 and n <= 8 (decode GEMV) or n >= 32 with Q4_K / Q6_K weights (prefill GEMM) this
 * is ONE kernel launch over the concatenated rows (gate+up, q+k+v); otherwise it is the same as
 * calling mi_qmm_mulmat_q8 per weight. */
int mi_qmm_mulmat_q8_multi(mi_qmm_ctx *ctx, const mi_qmm_weight *const *ws, int count,
                           const mi_qmm_act *act, float *const *ys, int location);

/* ---- GGUF files: replaces gguf.Open / File.KeyValue / File.TensorInfo / File.TensorReader,
 *      /root/reference/fs/gguf/gguf.go:54-110, 332-351, 361-378, 390-430 (and the loader loop of
 *      Backend.Load, /root/reference/ml/backend.go:20).  The file is mapped read-only; header,
 *      key-values and tensor infos are parsed by open (the reference parses lazily: same values,
 *      errors surface at open instead of later).  No GPU is needed except for gguf_upload. */
typedef struct mi_qmm_gguf mi_qmm_gguf;
int mi_qmm_gguf_open(const char *path, mi_qmm_gguf **out);
void mi_qmm_gguf_close(mi_qmm_gguf *f);
/* version, general.alignment (default 32), file offset of the tensor data, counts */
int mi_qmm_gguf_info(const mi_qmm_gguf *f, int *version, int64_t *alignment, int64_t *data_offset,
                     int64_t *num_kv, int64_t *num_tensors);
/* tensor by index: name (valid until close), ggml type id, dims (dims[0] contiguous; unused = 1),
 * offset inside the data section, byte size by the block rule of fs/gguf/tensor.go:47-76 */
int mi_qmm_gguf_tensor(const mi_qmm_gguf *f, int64_t index, const char **name, int *type, int *n_dims,
                       int64_t dims[4], int64_t *offset, int64_t *nbytes);
int64_t mi_qmm_gguf_find_tensor(const mi_qmm_gguf *f, const char *name); /* index, or -1 */
const void *mi_qmm_gguf_tensor_data(const mi_qmm_gguf *f, int64_t index); /* into the mapping; NULL if out of range */
/* key-value lookup with the reference's rule: a key outside "general." / "tokenizer." is looked
 * up as "<general.architecture>.<key>".  Returns the index or -1. */
int64_t mi_qmm_gguf_find_kv(const mi_qmm_gguf *f, const char *key);
/* key (valid until close), value type (0..12 = u8,i8,u16,i16,u32,i32,f32,bool,string,array,u64,i64,f64),
 * and for arrays the element type and length */
int mi_qmm_gguf_kv(const mi_qmm_gguf *f, int64_t index, const char **key, int *type, int *elem_type,
                   int64_t *count);
/* Scalar accessors; elem < 0 reads the value itself, elem >= 0 that element of an array.  As in
 * the reference (fs/gguf/keyvalue.go:42-91) a kind mismatch is not an error: the result is 0 / "". */
int mi_qmm_gguf_kv_int(const mi_qmm_gguf *f, int64_t index, int64_t elem, int64_t *out);
int mi_qmm_gguf_kv_uint(const mi_qmm_gguf *f, int64_t index, int64_t elem, uint64_t *out);
int mi_qmm_gguf_kv_float(const mi_qmm_gguf *f, int64_t index, int64_t elem, double *out);
int mi_qmm_gguf_kv_bool(const mi_qmm_gguf *f, int64_t index, int64_t elem, int *out);
/* string bytes are not NUL-terminated: *str points into the mapping, *len is the length */
int mi_qmm_gguf_kv_string(const mi_qmm_gguf *f, int64_t index, int64_t elem, const char **str, int64_t *len);
/* upload tensor `index` (a type this library multiplies: 2, 8, 12, 14) as a resident weight; the bytes
 * go from the mapping to the device.  2-D: K = dims[0], M = dims[1].  3-D (an expert stack for
 * mi_qmm_mulmat_id): K = dims[0], M = dims[1] * dims[2], n_expert = dims[2]. */
int mi_qmm_gguf_upload(mi_qmm_ctx *ctx, const mi_qmm_gguf *f, int64_t index, mi_qmm_weight **out);

/* ---- diagnostics */
const char *mi_qmm_last_error(void); /* thread-local, never NULL */
const char *mi_qmm_version(void);
/* number of compute units and device name of the ctx's device (for bench reports) */
int mi_qmm_device_info(mi_qmm_ctx *ctx, int *compute_units, int *clock_mhz, char *name, int name_len);

#ifdef __cplusplus
}
#endif
#endif /* MI_QMM_H */
