// C ABI of the library (include/mi_qmm.h): argument checking, device memory, kernel dispatch.
// Everything that computes runs on the GPU; there is no CPU fallback in this file.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>

#include "../../include/mi_qmm.h"
#include "gguf_file.h"
#include <vector>

#include "internal.h"

using namespace miqmm;

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

#define HIP_TRY(expr)                                                                       \
    do {                                                                                    \
        hipError_t e_ = (expr);                                                             \
        if (e_ != hipSuccess)                                                               \
            return fail(e_ == hipErrorOutOfMemory ? MI_QMM_ERR_NOMEM : MI_QMM_ERR_HIP,      \
                        "%s: %s", #expr, hipGetErrorString(e_));                            \
    } while (0)

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

// Scratch of the entry point that allocates nothing (mi_qmm_mulmat_noalloc): quantized activation planes live
// here instead of in memory from hipMalloc.  Every GPU the library runs on holds its own copy of the array
// until the process ends.  In host code the name is only a stand-in: mi_qmm_init asks for the device
// address once per ctx (hipGetSymbolAddress, with the ctx's device current) and everything else uses that.
static __device__ __align__(256) unsigned char scratch[MI_QMM_NOALLOC_SCRATCH_BYTES];

struct mi_qmm_ctx {
    int device = 0;
    int num_cus = 0;
    int clock_mhz = 0;
    char name[128] = {0};
    hipStream_t own_stream = nullptr;
    hipStream_t stream = nullptr;
    // growable scratch: quantized activation planes and host<->device staging
    void *act_buf = nullptr;  size_t act_cap = 0;
    void *io_buf = nullptr;   size_t io_cap = 0;
    void *ws_buf = nullptr;   size_t ws_cap = 0;   // partial sums of a K-split GEMM
    void *pair_buf = nullptr; size_t pair_cap = 0; // the two products of a gated pair when they are not one launch
    void *dup_buf = nullptr;  size_t dup_cap = 0;  // [x | x] for Q5_K weights (and host staging of such a call)
    bool scratch_frozen = false;                   // mi_qmm_scratch_freeze: growth is an error, not a reallocation
    void *static_scratch = nullptr;                // this device's copy of the file-scope array `scratch` below
};

struct mi_qmm_weight {
    int device = 0;
    void *base = nullptr;
    size_t bytes = 0;
    DevWeight dev{};
    // expand: the caller's activation rows must be expanded before the product, from k_user to dev.K floats --
    // a Q5_K tensor (dev is the Q4_K tensor of rows of 2 k_user that stands for it, formats.h: multiplied with [x | x]) or an
    // MXFP4 tensor whose rows were padded with zero blocks to whole 256-element steps (multiplied with [x | 0])
    bool expand = false;
    bool repeat = false;  // [x | x] rather than [x | 0]
    int64_t k_user = 0;
    int file_type = -1;  // the ggml type the tensor had in the file, where dev.type is another (Q5_K, MXFP4); -1: dev.type
    // MXFP4: the tensor once more in its own layout (type T_MXFP4, same K and M as dev), which the streaming kernels read at
    // half the bytes of the Q8_0 planes the matrix-core kernels multiply.  Q5_K: the blocks as they are (type T_Q5_K, K = k_user),
    // for the streaming kernel at one or two activation rows -- against x itself, not [x | x]
    bool has_native = false;
    DevWeight native{};
};

struct mi_qmm_gguf {
    GgufFile file;
};

struct mi_qmm_act {
    int device = 0;
    int type = 0;
    int64_t k = 0, n_max = 0, n = 0;
    void *base = nullptr;
    bool f16 = false;  // carries the fp16 planes of the fp16-MFMA GEMM
};

namespace {

int reserve(mi_qmm_ctx *ctx, void **buf, size_t *cap, size_t need) {
    if (need <= *cap) return MI_QMM_OK;
    hipStream_t s = ctx->stream;
    // A captured HIP graph keeps the raw addresses of the scratch its kernels used: growing (= freeing) it
    // afterwards would leave the graph pointing at freed memory.  Frozen scratch refuses to grow instead.
    if (ctx->scratch_frozen)
        return fail(MI_QMM_ERR_INVALID,
                    "the call needs %zu bytes of scratch, the ctx holds %zu and its scratch is frozen "
                    "(mi_qmm_scratch_freeze): run the largest shapes once before freezing", need, *cap);
    if (*buf) {
        HIP_TRY(hipStreamSynchronize(s));  // queued kernels may still read the old buffer
        HIP_TRY(hipFree(*buf));
        *buf = nullptr;
        *cap = 0;
    }
    need = align_up(need + need / 4, 1 << 20);
    HIP_TRY(hipMalloc(buf, need));
    *cap = need;
    return MI_QMM_OK;
}

struct ActPlanes { int8_t *qs; float *d; int16_t *bsums; uint8_t *sd8; uint8_t *sd16; uint16_t *qf; uint16_t *bsf; size_t total; };

// fp16 planes for the fp16-MFMA GEMM: wanted where a Q4_K weight may meet a batch that kernel takes
bool wants_f16_planes(int weight_type, int64_t n) { return weight_type == T_Q4_K && n > 64; }

// carve the activation scratch into planes for N rows of K elements
ActPlanes plan_act(void *base, int q8_type, int64_t K, int64_t N, bool f16 = false) {
    // the GEMM reads Q8_K activation rows in tiles of 128 without bounds checks (results of rows past
    // N are dropped), so the planes are sized in whole tiles
    if (q8_type == T_Q8_K) N = (N + 127) / 128 * 128;
    const int64_t blk = q8_type == T_Q8_0 ? QK : QKK;
    const int64_t sums = q8_type == T_Q8_0 ? QK : 16;
    ActPlanes p;
    size_t off = 0;
    p.qs = (int8_t *)((char *)base + off);     off = align_up(off + (size_t)(N * K), 256);
    p.d = (float *)((char *)base + off);       off = align_up(off + (size_t)(N * (K / blk)) * 4, 256);
    p.bsums = (int16_t *)((char *)base + off); off = align_up(off + (size_t)(N * (K / sums)) * 2, 256);
    p.sd8 = p.sd16 = nullptr;
    if (q8_type == T_Q8_K) {  // block-sum digit planes read by the MFMA GEMM
        p.sd8 = (uint8_t *)base + off;  off = align_up(off + (size_t)(N * (K / QKK)) * 16, 256);
        p.sd16 = (uint8_t *)base + off; off = align_up(off + (size_t)(N * (K / QKK)) * 32, 256);
    }
    p.qf = p.bsf = nullptr;
    if (q8_type == T_Q8_K && f16) {
        p.qf = (uint16_t *)((char *)base + off);  off = align_up(off + (size_t)(N * K) * 2, 256);
        p.bsf = (uint16_t *)((char *)base + off); off = align_up(off + (size_t)(N * (K / QKK)) * 32, 256);
    }
    p.total = off;
    return p;
}

int check_ctx(mi_qmm_ctx *ctx) {
    if (!ctx) return fail(MI_QMM_ERR_INVALID, "ctx is NULL");
    HIP_TRY(hipSetDevice(ctx->device));  // calls may arrive on any OS thread
    return MI_QMM_OK;
}

}  // namespace

extern "C" {

const char *mi_qmm_last_error(void) { return g_err; }
const char *mi_qmm_version(void) { return "mi_qmm 0.1 (gfx950)"; }

// ---- size tables, every id of /root/reference/fs/ggml/ggml.go:407-513 ------------------------
int64_t mi_qmm_block_size(int t) {
    switch (t) {
    case 0: case 1: case 24: case 25: case 26: case 27: case 28: case 30: return 1;  // F32 F16 I8..F64 BF16
    case 2: case 3: case 6: case 7: case 8: case 9: case 20: case 39: return 32;     // Q4_0..Q8_1 IQ4_NL MXFP4
    case 40: return 64;                                                              // NVFP4
    case 41: return 128;                                                             // Q1_0
    case 10: case 11: case 12: case 13: case 14: case 15: case 16: case 17: case 18: case 19: case 21:
    case 22: case 23: case 29: case 34: case 35: return 256;                         // K-quants, IQ*, TQ*
    default: return 0;
    }
}

int64_t mi_qmm_type_size(int t) {
    const int64_t b = mi_qmm_block_size(t);
    switch (t) {
    case 0: return 4;
    case 1: return 2;
    case 2: return 2 + b / 2;
    case 3: return 2 + 2 + b / 2;
    case 6: return 2 + 4 + b / 2;
    case 7: return 2 + 2 + 4 + b / 2;
    case 8: return 2 + b;
    case 9: return 2 + 2 + b;
    case 10: return b / 16 + b / 4 + 2 + 2;
    case 11: return b / 8 + b / 4 + 12 + 2;
    case 12: return 2 + 2 + 12 + b / 2;
    case 13: return 2 + 2 + 12 + b / 8 + b / 2;
    case 14: return b / 2 + b / 4 + b / 16 + 2;
    case 15: return 4 + b + 2 * b / 16;
    case 16: return 2 + 2 * b / 8;
    case 17: return 2 + 2 * b / 8 + b / 32;
    case 18: return 2 + b / 4 + b / 8;
    case 19: return 2 + b / 8 + b / 16;
    case 20: return 2 + b / 2;
    case 21: return 2 + b / 4 + b / 8 + b / 32 + 4;
    case 22: return 2 + b / 4 + b / 16;
    case 23: return 2 + 2 + b / 2 + b / 64;
    case 24: return 1;
    case 25: return 2;
    case 26: return 4;
    case 27: return 8;
    case 28: return 8;
    case 29: return b / 8 + b / 16 + b / 32;
    case 30: return 2;
    case 39: return 1 + b / 2;
    case 40: return 4 + b / 2;
    case 41: return 2 + b / 8;
    default: return 0;  // includes TQ1_0/TQ2_0 (34, 35), which the reference's TypeSize leaves at 0
    }
}

int64_t mi_qmm_row_size(int t, int64_t k) {
    const int64_t b = mi_qmm_block_size(t), s = mi_qmm_type_size(t);
    if (b == 0 || s == 0 || k < 0 || k % b != 0) return -1;
    return k / b * s;
}

int mi_qmm_vec_dot_type(int wt) {
    switch (wt) {
    case T_Q4_0: case T_Q5_0: case T_Q8_0: case T_MXFP4: return T_Q8_0;
    case T_Q4_K: case T_Q5_K: case T_Q6_K: return T_Q8_K;
    case T_F32: case T_F16: case T_BF16: return wt;  // multiplied in their own type: x is converted to it
    default: return -1;
    }
}

// ---- lifetime -----------------------------------------------------------------------------------
int mi_qmm_init(int device_ordinal, mi_qmm_ctx **out) {
    if (!out) return fail(MI_QMM_ERR_INVALID, "out is NULL");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return fail(MI_QMM_ERR_NODEVICE, "no HIP device visible (%s); this library has no CPU path",
                    e == hipSuccess ? "device count 0" : hipGetErrorString(e));
    if (device_ordinal < 0 || device_ordinal >= count)
        return fail(MI_QMM_ERR_NODEVICE, "device ordinal %d out of range (0..%d)", device_ordinal, count - 1);
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device_ordinal));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(MI_QMM_ERR_NODEVICE, "device %d is %s; the kernels are built for gfx950 only",
                    device_ordinal, prop.gcnArchName);
    HIP_TRY(hipSetDevice(device_ordinal));
    mi_qmm_ctx *c = new (std::nothrow) mi_qmm_ctx();
    if (!c) return fail(MI_QMM_ERR_NOMEM, "host allocation failed");
    c->device = device_ordinal;
    c->num_cus = prop.multiProcessorCount;
    c->clock_mhz = prop.clockRate / 1000;
    snprintf(c->name, sizeof(c->name), "%s (%s)", prop.name, prop.gcnArchName);
    e = hipStreamCreateWithFlags(&c->own_stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete c;
        return fail(MI_QMM_ERR_HIP, "hipStreamCreate: %s", hipGetErrorString(e));
    }
    c->stream = c->own_stream;
    e = hipGetSymbolAddress(&c->static_scratch, HIP_SYMBOL(scratch));  // device_ordinal is current (hipSetDevice above)
    if (e != hipSuccess || !c->static_scratch) {
        (void)hipStreamDestroy(c->own_stream);
        delete c;
        return fail(MI_QMM_ERR_HIP, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    }
    *out = c;
    return MI_QMM_OK;
}

void mi_qmm_destroy(mi_qmm_ctx *ctx) {
    if (!ctx) return;
    if (hipSetDevice(ctx->device) == hipSuccess) {
        (void)hipStreamSynchronize(ctx->stream);
        if (ctx->act_buf) (void)hipFree(ctx->act_buf);
        if (ctx->io_buf) (void)hipFree(ctx->io_buf);
        if (ctx->ws_buf) (void)hipFree(ctx->ws_buf);
        if (ctx->pair_buf) (void)hipFree(ctx->pair_buf);
        if (ctx->dup_buf) (void)hipFree(ctx->dup_buf);
        if (ctx->own_stream) (void)hipStreamDestroy(ctx->own_stream);
    }
    delete ctx;
}

int mi_qmm_set_stream(mi_qmm_ctx *ctx, void *hip_stream) {
    int rc = check_ctx(ctx);
    if (rc) return rc;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    ctx->stream = hip_stream ? (hipStream_t)hip_stream : ctx->own_stream;
    return MI_QMM_OK;
}

int mi_qmm_sync(mi_qmm_ctx *ctx) {
    int rc = check_ctx(ctx);
    if (rc) return rc;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return MI_QMM_OK;
}

void *mi_qmm_host_alloc(mi_qmm_ctx *ctx, size_t bytes) {
    if (check_ctx(ctx)) return nullptr;
    void *p = nullptr;
    hipError_t e = hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocDefault);
    if (e != hipSuccess) {
        fail(MI_QMM_ERR_NOMEM, "hipHostMalloc(%zu): %s", bytes, hipGetErrorString(e));
        return nullptr;
    }
    return p;
}

void mi_qmm_host_free(mi_qmm_ctx *, void *p) {
    if (p) (void)hipHostFree(p);  // page-locked memory is not tied to the current device: the ctx may be gone already
}

int mi_qmm_device_info(mi_qmm_ctx *ctx, int *compute_units, int *clock_mhz, char *name, int name_len) {
    if (!ctx) return fail(MI_QMM_ERR_INVALID, "ctx is NULL");
    if (compute_units) *compute_units = ctx->num_cus;
    if (clock_mhz) *clock_mhz = ctx->clock_mhz;
    if (name && name_len > 0) snprintf(name, (size_t)name_len, "%s", ctx->name);
    return MI_QMM_OK;
}

// ---- weights --------------------------------------------------------------------------------------
int mi_qmm_weight_upload(mi_qmm_ctx *ctx, int type, const void *bytes, int64_t k, int64_t m, int src_location,
                         mi_qmm_weight **out) {
    if (!out) return fail(MI_QMM_ERR_INVALID, "out is NULL");
    *out = nullptr;
    if (mi_qmm_vec_dot_type(type) < 0)
        return fail(MI_QMM_ERR_UNSUPPORTED, "ggml type %d is not a supported weight type (0, 1, 2, 6, 8, 12, 13, 14, 30, 39)", type);
    if (k <= 0 || m <= 0) return fail(MI_QMM_ERR_INVALID, "k=%lld m=%lld must be positive", (long long)k, (long long)m);
    const int64_t row = mi_qmm_row_size(type, k);
    if (row < 0)
        return fail(MI_QMM_ERR_INVALID, "k=%lld is not a multiple of the block size %lld of type %d",
                    (long long)k, (long long)mi_qmm_block_size(type), type);
    if (type == T_Q4_0 || type == T_Q5_0 || type == T_Q8_0 || type == T_MXFP4) {
        // the activation quantizer pairs these with Q8_0 planes read as 16-byte pieces
        if (k % QK != 0) return fail(MI_QMM_ERR_INVALID, "k not a multiple of 32");
    }
    if (!bytes) return fail(MI_QMM_ERR_INVALID, "gguf_bytes is NULL");
    if (src_location != MI_QMM_HOST && src_location != MI_QMM_DEVICE)
        return fail(MI_QMM_ERR_INVALID, "src_location must be MI_QMM_HOST or MI_QMM_DEVICE");
    int rc = check_ctx(ctx);
    if (rc) return rc;

    const size_t total = (size_t)(row * m);
    // plane sizes (bytes), each plane 256-byte aligned inside one allocation
    size_t s0 = 0, s1 = 0, s2 = 0, sd = 0;
    switch (type) {
    case T_Q4_K: case T_F32: case T_F16: case T_BF16: s0 = total; break;
    case T_Q5_K: s0 = (size_t)(m * (k / QKK)) * 2 * Q4_K_BYTES; s1 = total; break;  // a Q4_K tensor of rows twice as long; the blocks as they are
    case T_Q4_0: s0 = (size_t)(m * (k / 2)); sd = (size_t)(m * (k / QK)) * 2; break;
    case T_Q8_0: s0 = (size_t)(m * k); sd = (size_t)(m * (k / QK)) * 2; break;
    case T_Q5_0: {   // kept as Q8_0 planes, rows of whole 256-element steps
        const size_t kp = align_up((size_t)k, 256);
        s0 = (size_t)m * kp; sd = (size_t)m * (kp / QK) * 2;
        break;
    }
    case T_MXFP4: {  // Q8_0 planes (p0, d), and the tensor as it is (p1: nibbles, p2: scale bytes)
        const size_t kp = align_up((size_t)k, 256);
        s0 = (size_t)m * kp; sd = (size_t)m * (kp / QK) * 2; s1 = (size_t)m * (kp / QK) * 16; s2 = (size_t)m * (kp / QK) * 2;
        break;
    }
    case T_Q6_K: s0 = (size_t)(m * (k / 2)); s1 = (size_t)(m * (k / 4)); s2 = (size_t)(m * (k / 16));
                 sd = (size_t)(m * (k / QKK)) * 2; break;
    }
    const size_t o0 = 0, o1 = align_up(o0 + s0, 256), o2 = align_up(o1 + s1, 256), od = align_up(o2 + s2, 256);
    const size_t dev_bytes = align_up(od + sd, 256) + 256;  // tail slack: 16-byte loads never leave the allocation

    mi_qmm_weight *w = new (std::nothrow) mi_qmm_weight();
    if (!w) return fail(MI_QMM_ERR_NOMEM, "host allocation failed");
    w->device = ctx->device;
    hipError_t e = hipMalloc(&w->base, dev_bytes);
    if (e != hipSuccess) {
        delete w;
        return fail(MI_QMM_ERR_NOMEM, "hipMalloc(%zu) for weight: %s", dev_bytes, hipGetErrorString(e));
    }
    w->bytes = dev_bytes;
    uint8_t *b = (uint8_t *)w->base;
    w->dev.p0 = b + o0;
    w->dev.p1 = s1 ? b + o1 : nullptr;
    w->dev.p2 = s2 ? b + o2 : nullptr;
    w->dev.d = sd ? (const uint16_t *)(b + od) : nullptr;
    w->dev.K = k; w->dev.M = m; w->dev.type = type;
    if (type == T_Q5_K) {
        w->expand = w->repeat = true; w->k_user = k; w->dev.K = 2 * k; w->dev.type = T_Q4_K; w->file_type = T_Q5_K;
        // ... and the blocks as they are, which the streaming kernel reads at one or two activation rows (176 instead of 288 B)
        w->has_native = true;
        w->native = w->dev;
        w->native.type = T_Q5_K; w->native.K = k; w->native.p0 = b + o1; w->native.p1 = nullptr;
        w->dev.p1 = nullptr;
    }
    if (type == T_Q5_0) {
        w->dev.type = T_Q8_0; w->file_type = T_Q5_0; w->dev.K = (int64_t)align_up((size_t)k, 256);
        if (w->dev.K != k) { w->expand = true; w->k_user = k; }
    }
    if (type == T_MXFP4) {
        // rows of a whole number of 256-element steps (2880 -> 3072): the matrix-core kernels of the 32-element formats want that
        w->dev.type = T_Q8_0; w->file_type = T_MXFP4; w->dev.K = (int64_t)align_up((size_t)k, 256);
        if (w->dev.K != k) { w->expand = true; w->k_user = k; }
        w->has_native = true;
        w->native = w->dev;
        w->native.type = T_MXFP4; w->native.p0 = b + o1; w->native.d = (const uint16_t *)(b + o2); w->native.p1 = w->native.p2 = nullptr;
        w->dev.p1 = w->dev.p2 = nullptr;
    }

    void *staging = nullptr;
    const uint8_t *src = (const uint8_t *)bytes;
    auto cleanup = [&](int code, const char *what, hipError_t err) {
        if (staging) (void)hipFree(staging);
        (void)hipFree(w->base);
        delete w;
        return fail(code, "%s: %s", what, hipGetErrorString(err));
    };
    if (type == T_Q4_K || plain_type(type)) {
        e = hipMemcpyAsync(b + o0, bytes, total,
                           src_location == MI_QMM_HOST ? hipMemcpyHostToDevice : hipMemcpyDeviceToDevice, ctx->stream);
        if (e != hipSuccess) return cleanup(MI_QMM_ERR_HIP, "hipMemcpy(weight)", e);
    } else {
        if (src_location == MI_QMM_HOST) {
            e = hipMalloc(&staging, total);
            if (e != hipSuccess) return cleanup(MI_QMM_ERR_NOMEM, "hipMalloc(staging)", e);
            e = hipMemcpyAsync(staging, bytes, total, hipMemcpyHostToDevice, ctx->stream);
            if (e != hipSuccess) return cleanup(MI_QMM_ERR_HIP, "hipMemcpy(staging)", e);
            src = (const uint8_t *)staging;
        }
        int *bad = nullptr;
        if (type == T_MXFP4) {  // the tail slack of the allocation holds the flag of scales the planes cannot hold
            bad = (int *)(b + dev_bytes - 256);
            e = hipMemsetAsync(bad, 0, sizeof(int), ctx->stream);
            if (e != hipSuccess) return cleanup(MI_QMM_ERR_HIP, "hipMemset(flag)", e);
        }
        e = type == T_Q5_K ? launch_relayout_q5k(src, k, m, b + o0, ctx->stream)
            : type == T_Q5_0 ? launch_relayout_q5_0(src, k, w->dev.K, m, b + o0, (uint16_t *)(b + od), ctx->stream)
            : type == T_MXFP4 ? launch_relayout_mxfp4(src, k, w->dev.K, m, b + o0, (uint16_t *)(b + od), bad, ctx->stream)
                              : launch_relayout(type, src, k, m, b + o0, b + o1, b + o2, (uint16_t *)(b + od), ctx->stream);
        if (e != hipSuccess) return cleanup(MI_QMM_ERR_HIP, "relayout kernel", e);
        if (type == T_MXFP4) {
            e = launch_relayout_mxfp4_native(src, k, w->dev.K, m, b + o1, (uint16_t *)(b + o2), ctx->stream);
            if (e != hipSuccess) return cleanup(MI_QMM_ERR_HIP, "relayout kernel", e);
        }
        if (type == T_Q5_K) {
            e = hipMemcpyAsync(b + o1, src, total, hipMemcpyDeviceToDevice, ctx->stream);
            if (e != hipSuccess) return cleanup(MI_QMM_ERR_HIP, "hipMemcpy(weight)", e);
        }
        if (bad) {
            int flag = 0;
            e = hipMemcpyAsync(&flag, bad, sizeof(int), hipMemcpyDeviceToHost, ctx->stream);
            if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
            if (e != hipSuccess) return cleanup(MI_QMM_ERR_HIP, "hipMemcpy(flag)", e);
            if (flag) {
                if (staging) (void)hipFree(staging);
                (void)hipFree(w->base);
                delete w;
                return fail(MI_QMM_ERR_UNSUPPORTED, "an MXFP4 block has a scale byte above 146 (weights of 2^18 and more): beyond the fp16 block scales it is kept with");
            }
        }
    }
    e = hipStreamSynchronize(ctx->stream);  // the caller's bytes must not be needed after return
    if (e != hipSuccess) return cleanup(MI_QMM_ERR_HIP, "hipStreamSynchronize(upload)", e);
    if (staging) (void)hipFree(staging);
    *out = w;
    return MI_QMM_OK;
}

void mi_qmm_weight_free(mi_qmm_weight *w) {
    if (!w) return;
    if (hipSetDevice(w->device) == hipSuccess && w->base) {
        (void)hipDeviceSynchronize();
        (void)hipFree(w->base);
    }
    delete w;
}

int mi_qmm_weight_info(const mi_qmm_weight *w, int *type, int64_t *k, int64_t *m, int64_t *device_bytes) {
    if (!w) return fail(MI_QMM_ERR_INVALID, "weight is NULL");
    if (type) *type = w->file_type >= 0 ? w->file_type : w->dev.type;
    if (k) *k = w->expand ? w->k_user : w->dev.K;  // (the caller's K)
    if (m) *m = w->dev.M;
    if (device_bytes) *device_bytes = (int64_t)w->bytes;
    return MI_QMM_OK;
}

// ---- activation quantization ---------------------------------------------------------------------
int mi_qmm_quantize_act(mi_qmm_ctx *ctx, int q8_type, const float *x, int64_t k, int64_t n, void *out_blocks,
                        int location) {
    if (q8_type != T_Q8_0 && q8_type != T_Q8_K)
        return fail(MI_QMM_ERR_UNSUPPORTED, "activation type %d is not Q8_0 (8) or Q8_K (15)", q8_type);
    if (k < 0 || n < 0) return fail(MI_QMM_ERR_INVALID, "k=%lld n=%lld must be non-negative", (long long)k, (long long)n);
    const int64_t row = mi_qmm_row_size(q8_type, k);
    if (row < 0)
        return fail(MI_QMM_ERR_INVALID, "k=%lld is not a multiple of the block size %lld of type %d",
                    (long long)k, (long long)mi_qmm_block_size(q8_type), q8_type);
    if (location != MI_QMM_HOST && location != MI_QMM_DEVICE)
        return fail(MI_QMM_ERR_INVALID, "location must be MI_QMM_HOST or MI_QMM_DEVICE");
    int rc = check_ctx(ctx);
    if (rc) return rc;
    if (k * n == 0) return MI_QMM_OK;
    if (!x || !out_blocks) return fail(MI_QMM_ERR_INVALID, "x or out_blocks is NULL");

    const ActPlanes probe = plan_act(nullptr, q8_type, k, n);
    if ((rc = reserve(ctx, &ctx->act_buf, &ctx->act_cap, probe.total))) return rc;
    const ActPlanes p = plan_act(ctx->act_buf, q8_type, k, n);
    const size_t xbytes = (size_t)(n * k) * 4, obytes = (size_t)(n * row);
    const float *dx = x;
    uint8_t *dout = (uint8_t *)out_blocks;
    if (location == MI_QMM_HOST) {
        const size_t xoff = align_up(obytes, 256);
        if ((rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, xoff + xbytes))) return rc;
        dout = (uint8_t *)ctx->io_buf;
        dx = (const float *)((char *)ctx->io_buf + xoff);
        HIP_TRY(hipMemcpyAsync((void *)dx, x, xbytes, hipMemcpyHostToDevice, ctx->stream));
    }
    HIP_TRY(launch_quantize_act(q8_type, dx, k, n, p.qs, p.d, p.bsums, p.sd8, p.sd16, ctx->stream));
    HIP_TRY(launch_pack_act_gguf(q8_type, p.qs, p.d, p.bsums, k, n, dout, ctx->stream));
    if (location == MI_QMM_HOST) {
        HIP_TRY(hipMemcpyAsync(out_blocks, dout, obytes, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
    }
    return MI_QMM_OK;
}

int mi_qmm_quantize_weights(mi_qmm_ctx *ctx, int ggml_type, const float *x, int64_t k, int64_t m, void *out_blocks,
                            int location) {
    if (ggml_type != T_Q4_0 && ggml_type != T_Q8_0 && ggml_type != T_Q4_K && ggml_type != T_Q6_K)
        return fail(MI_QMM_ERR_UNSUPPORTED, "weight type %d is not Q4_0 (2), Q8_0 (8), Q4_K (12) or Q6_K (14)", ggml_type);
    if (k < 0 || m < 0) return fail(MI_QMM_ERR_INVALID, "k=%lld m=%lld must be non-negative", (long long)k, (long long)m);
    const int64_t row = mi_qmm_row_size(ggml_type, k);
    if (row < 0)
        return fail(MI_QMM_ERR_INVALID, "k=%lld is not a multiple of the block size %lld of type %d",
                    (long long)k, (long long)mi_qmm_block_size(ggml_type), ggml_type);
    if (location != MI_QMM_HOST && location != MI_QMM_DEVICE)
        return fail(MI_QMM_ERR_INVALID, "location must be MI_QMM_HOST or MI_QMM_DEVICE");
    int rc = check_ctx(ctx);
    if (rc) return rc;
    if (k * m == 0) return MI_QMM_OK;
    if (!x || !out_blocks) return fail(MI_QMM_ERR_INVALID, "x or out_blocks is NULL");
    if (location == MI_QMM_DEVICE) {
        // (the kernels read x in 16-byte pieces and write Q4_K blocks in 4-byte words)
        if (((uintptr_t)x & 15) || ((uintptr_t)out_blocks & 3))
            return fail(MI_QMM_ERR_INVALID, "device x must be 16-byte aligned and out_blocks 4-byte aligned");
        HIP_TRY(launch_encode_weights(ggml_type, x, k, m, (uint8_t *)out_blocks, ctx->stream));
        return MI_QMM_OK;
    }
    // host buffers: slabs of rows through the ctx's staging buffer (at most 64 MiB of f32 at a time)
    const int64_t slab_rows = std::max<int64_t>(1, std::min<int64_t>(m, ((int64_t)64 << 20) / (k * 4)));
    const size_t xoff = align_up((size_t)(slab_rows * row), 256);
    if ((rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, xoff + (size_t)(slab_rows * k) * 4))) return rc;
    uint8_t *dout = (uint8_t *)ctx->io_buf;
    float *dx = (float *)((char *)ctx->io_buf + xoff);
    for (int64_t r0 = 0; r0 < m; r0 += slab_rows) {
        const int64_t rows = std::min(slab_rows, m - r0);
        HIP_TRY(hipMemcpyAsync(dx, x + r0 * k, (size_t)(rows * k) * 4, hipMemcpyHostToDevice, ctx->stream));
        HIP_TRY(launch_encode_weights(ggml_type, dx, k, rows, dout, ctx->stream));
        HIP_TRY(hipMemcpyAsync((char *)out_blocks + r0 * row, dout, (size_t)(rows * row), hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));  // the slab buffers are reused
    }
    return MI_QMM_OK;
}

}  // extern "C"

// ---- the product ------------------------------------------------------------------------------------
namespace {

// The tensor the streaming GEMV reads for a weight: an MXFP4 weight's own layout (half the bytes of its Q8_0 planes)
// where the kernel takes that type at this shape too.
const DevWeight &gemv_dev(const mi_qmm_weight *w, int ncols, bool f32_x) {
    if (!w->has_native || w->native.type != T_MXFP4 || w->native.K > gemv_max_k(T_MXFP4)) return w->dev;
    if (f32_x && !gemv_f32_supported(T_MXFP4, w->native.K, w->native.M, ncols)) return w->dev;
    return w->native;
}

// From this many activation columns up a product below the GEMM's batch goes to a matrix-core skinny
// kernel instead of the streaming GEMV (measured crossovers on MI355X: the GEMV pays one v_dot4 pass
// per column).
bool wants_skinny(int type, int64_t K, int64_t M, int64_t n, int num_cus) {
    // (long rows of Q4_0 / Q8_0 from two columns: the GEMV at 4096 x 14336 takes 27 / 39 us at two / three columns of
    // Q8_0 where the matrix-core kernel takes 17.5)
    if (type == T_Q4_0 || type == T_Q8_0) return n >= (K > 8192 ? 2 : 4) && skinny32_supports(type, K, M);
    // (two columns of a large Q4_K matrix with rows of one K segment: the deep direct-load kernel, 16.4 against 17.1 us
    // for gate + up)
    if (type == T_Q4_K && n == 2 && skinny_supports(type, K, M) && deep16_wanted(type, K, M, 2, num_cus)) return true;
    if (type == T_Q6_K && n < 4 && skinny_supports(type, K, M) && deep6_wanted(type, K, M, (int)n, num_cus)) return true;
    const int64_t from = type == T_Q4_K ? 3 : 4;
    return n >= from && skinny_supports(type, K, M);
}

// One matrix at a few f32 columns on the deep direct-load kernel that quantizes x itself (Q6_K: unless the rows kernel is
// the one for this matrix).
bool deep_f32_one(const mi_qmm_ctx *ctx, const mi_qmm_weight *w, int64_t n) {
    if (n > 8 || !deep16_f32_wanted(w->dev.type, w->dev.K, w->dev.M, (int)n, ctx->num_cus)) return false;
    return !(w->dev.type == T_Q6_K && skinny_rows_wanted(w->dev, (int)n, ctx->num_cus));
}

// Which kernel a product takes (the values of the MI_QMM_ROUTE_* enum of mi_qmm.h).  Decided from the weight's type and
// shape, the number of activation columns and the planes at hand -- never from what else a call multiplies.
// a: the quantized activations (only N, sd8 and qf are looked at).  err (optional): why there is no route.
int route_planes(const mi_qmm_ctx *ctx, const mi_qmm_weight *w, const DevAct &a, int path, bool may_alloc, const char **err) {
    const int64_t K = w->dev.K, M = w->dev.M, n = a.N;
    const bool blk32 = gemm_blk32_supports(w->dev.type, K, M);  // Q4_0 / Q8_0: their own MFMA kernel
    bool use_gemm;
    if (path == MI_QMM_PATH_GEMM) use_gemm = true;
    else if (path == MI_QMM_PATH_GEMV) use_gemm = false;
    else use_gemm = n >= 32 && (blk32 || gemm_supports(w->dev.type, K, M));
    if (use_gemm && !blk32 && !gemm_supports(w->dev.type, K, M)) {
        if (err) *err = "the MFMA GEMM does not cover this type and shape";
        return 0;
    }
    if (!use_gemm && K > gemv_max_k(w->dev.type)) {
        if (err) *err = "K exceeds the GEMV limit for this type";
        return 0;
    }
    const bool auto_path = path != MI_QMM_PATH_GEMM && path != MI_QMM_PATH_GEMV;
    if (use_gemm) {
        if (blk32) return MI_QMM_ROUTE_GEMM_BLK32;
        if (auto_path && gemm_f16_wanted(w->dev, a, ctx->num_cus)) return MI_QMM_ROUTE_GEMM_F16;
        const int slices = auto_path ? gemm_q6k_slices(w->dev.type, K, M, n, ctx->num_cus) : 0;
        // (a caller that may not allocate gets the 256-row Q6_K kernel only where it needs no K-slice workspace)
        if (slices >= 1 && (may_alloc || slices == 1)) return MI_QMM_ROUTE_GEMM_Q6K;
        return MI_QMM_ROUTE_GEMM_INT8;
    }
    if (blk32 && wants_skinny(w->dev.type, K, M, n, ctx->num_cus)) return MI_QMM_ROUTE_SKINNY32;
    if (a.sd8 && (wants_skinny(w->dev.type, K, M, n, ctx->num_cus) || (n >= 2 && n <= 8 && skinny_rows_wanted(w->dev, (int)n, ctx->num_cus)))) {
        // from a few columns up the K-quants go to the matrix cores, 16 columns per launch: the streaming GEMV pays one
        // v_dot4 pass per column
        switch (skinny_kind(w->dev, (int)(n < 16 ? n : 16), ctx->num_cus)) {
        case 1: return MI_QMM_ROUTE_SKINNY_DEEP;
        case 2: return MI_QMM_ROUTE_SKINNY_DIRECT;
        case 3: return MI_QMM_ROUTE_SKINNY_ROWS_Q4K;
        case 5: return MI_QMM_ROUTE_SKINNY_ROWS_Q6K;
        default: return MI_QMM_ROUTE_SKINNY_STAGED;
        }
    }
    return MI_QMM_ROUTE_GEMV;
}

// dy: device output [n][M].  Picks the kernel and queues it on the ctx's stream.
// may_alloc = false: never touches the ctx's growable buffers (the tiled GEMM then runs without its K-split workspace).
int run_product(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const DevAct &a, float *dy, int path, bool may_alloc = true) {
    const int64_t K = w->dev.K, M = w->dev.M, n = a.N;
    const char *why = nullptr;
    const int route = route_planes(ctx, w, a, path, may_alloc, &why);
    switch (route) {
    case 0:
        return fail(MI_QMM_ERR_UNSUPPORTED, "%s (type %d, K=%lld, M=%lld)", why, w->dev.type, (long long)K, (long long)M);
    case MI_QMM_ROUTE_GEMM_BLK32:
        HIP_TRY(launch_gemm_blk32(w->dev, a, dy, ctx->num_cus, ctx->stream));
        break;
    case MI_QMM_ROUTE_GEMM_F16:
        HIP_TRY(launch_gemm_f16(w->dev, a, dy, ctx->num_cus, ctx->stream));
        break;
    case MI_QMM_ROUTE_GEMM_Q6K: {
        const size_t wsf = gemm_q6k_workspace_floats(w->dev.type, K, M, n, ctx->num_cus);
        if (wsf) {
            int rc = reserve(ctx, &ctx->ws_buf, &ctx->ws_cap, wsf * sizeof(float));
            if (rc) return rc;
        }
        HIP_TRY(launch_gemm_q6k(w->dev, a, dy, wsf ? (float *)ctx->ws_buf : nullptr, wsf, ctx->num_cus, ctx->stream));
        break;
    }
    case MI_QMM_ROUTE_GEMM_INT8: {
        const size_t wsf = may_alloc ? gemm_workspace_floats(w->dev.type, K, M, n, ctx->num_cus) : 0;
        if (wsf) {
            int rc = reserve(ctx, &ctx->ws_buf, &ctx->ws_cap, wsf * sizeof(float));
            if (rc) return rc;
        }
        HIP_TRY(launch_gemm(w->dev, a, dy, M, wsf ? (float *)ctx->ws_buf : nullptr, wsf, ctx->num_cus, ctx->stream));
        break;
    }
    case MI_QMM_ROUTE_SKINNY32:
        for (int64_t c0 = 0; c0 < n; c0 += 16)
            HIP_TRY(launch_skinny32(w->dev, a, (int)c0, (int)(n - c0 < 16 ? n - c0 : 16), dy, ctx->num_cus, ctx->stream));
        break;
    case MI_QMM_ROUTE_SKINNY_DEEP:
    case MI_QMM_ROUTE_SKINNY_DIRECT:
    case MI_QMM_ROUTE_SKINNY_ROWS_Q4K:
    case MI_QMM_ROUTE_SKINNY_ROWS_Q6K:
    case MI_QMM_ROUTE_SKINNY_STAGED:
        for (int64_t c0 = 0; c0 < n; c0 += 16)
            HIP_TRY(launch_skinny(w->dev, a, (int)c0, (int)(n - c0 < 16 ? n - c0 : 16), dy, ctx->num_cus, ctx->stream));
        break;
    default:
        for (int64_t c0 = 0; c0 < n; c0 += 8) {
            const int nc = (int)(n - c0 < 8 ? n - c0 : 8);
            HIP_TRY(launch_gemv(gemv_dev(w, nc, false), a, (int)c0, nc, dy, M, ctx->num_cus, ctx->stream));
        }
    }
    return MI_QMM_OK;
}

// The route of mi_qmm_mulmat on f32 activations: the kernels that quantize x themselves where they apply, else the
// route of the planes the call would make.
int route_f32(const mi_qmm_ctx *ctx, const mi_qmm_weight *w, int64_t n, int path, const char **err) {
    const int64_t K = w->dev.K, M = w->dev.M;
    if (path != MI_QMM_PATH_GEMM && n <= 8 && !wants_skinny(w->dev.type, K, M, n, ctx->num_cus) && gemv_f32_supported(w->dev.type, K, M, (int)n))
        return MI_QMM_ROUTE_GEMV_F32;
    if (path == MI_QMM_PATH_AUTO && deep_f32_one(ctx, w, n)) return MI_QMM_ROUTE_DEEP_F32;
    static const uint8_t some_plane = 0;  // (stands for "the planes are there": route_planes only asks whether)
    DevAct a;
    a.sd8 = mi_qmm_vec_dot_type(w->dev.type) == T_Q8_K ? &some_plane : nullptr;
    a.sd16 = a.sd8;
    a.qf = wants_f16_planes(w->dev.type, n) ? reinterpret_cast<const uint16_t *>(&some_plane) : nullptr;
    a.bsf = a.qf;
    a.K = K;
    a.N = (int)n;
    a.type = mi_qmm_vec_dot_type(w->dev.type);
    return route_planes(ctx, w, a, path, /*may_alloc=*/true, err);
}

// allow_plain: the entry point also multiplies by F32 / F16 / BF16 weights (mi_qmm_mulmat and its variants do; the
// joint, produced, expert-indexed and pre-quantized forms are for the block-quantized types)
int check_product_args(mi_qmm_ctx *ctx, const mi_qmm_weight *w, int location, int path, bool allow_plain = false) {
    if (!w) return fail(MI_QMM_ERR_INVALID, "weight is NULL");
    if (!allow_plain && (plain_type(w->dev.type) || w->expand))
        return fail(MI_QMM_ERR_UNSUPPORTED, "this entry point takes Q4_0 / Q8_0 / Q4_K / Q6_K weights; type %d goes through mi_qmm_mulmat",
                    w->file_type >= 0 ? w->file_type : w->dev.type);
    if (location != MI_QMM_HOST && location != MI_QMM_DEVICE)
        return fail(MI_QMM_ERR_INVALID, "location must be MI_QMM_HOST or MI_QMM_DEVICE");
    if (path != MI_QMM_PATH_AUTO && path != MI_QMM_PATH_GEMV && path != MI_QMM_PATH_GEMM && path != MI_QMM_PATH_QUERY)
        return fail(MI_QMM_ERR_INVALID, "unknown path %d", path);
    int rc = check_ctx(ctx);
    if (rc) return rc;
    if (w->device != ctx->device)
        return fail(MI_QMM_ERR_INVALID, "weight lives on device %d, ctx on device %d", w->device, ctx->device);
    return MI_QMM_OK;
}

// mi_qmm_mulmat on an F32 / F16 / BF16 weight.  scratch: where the converted activations of the tiled kernel go -- NULL:
// the ctx's growable buffer; else a buffer of scratch_bytes the call must fit (mi_qmm_mulmat_noalloc).
int plain_mulmat(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const float *x, int64_t n, float *y, int location, int path,
                 void *scratch, size_t scratch_bytes) {
    const int64_t K = w->dev.K, M = w->dev.M;
    const int force = path == MI_QMM_PATH_GEMV ? 1 : path == MI_QMM_PATH_GEMM ? 2 : 0;
    const int kind = plain_kind(w->dev.type, K, M, n, force);
    if (!kind)
        return fail(MI_QMM_ERR_UNSUPPORTED, "no kernel for type %d, K=%lld, M=%lld, n=%lld on this path", w->dev.type, (long long)K,
                    (long long)M, (long long)n);
    int rc;
    void *xc = nullptr;
    const size_t need = kind == 2 ? plain_convert_bytes(w->dev.type, K, n) : 0;
    if (need && scratch) {
        if (need > scratch_bytes)
            return fail(MI_QMM_ERR_UNSUPPORTED, "n=%lld rows of k=%lld need %zu bytes of converted activations; the static scratch of "
                        "mi_qmm_mulmat_noalloc holds %zu (use mi_qmm_mulmat)", (long long)n, (long long)K, need, scratch_bytes);
        xc = scratch;
    } else if (need) {
        if ((rc = reserve(ctx, &ctx->act_buf, &ctx->act_cap, need))) return rc;
        xc = ctx->act_buf;
    }
    const size_t xbytes = (size_t)(n * K) * 4, ybytes = (size_t)(n * M) * 4;
    const float *dx = x;
    float *dy = y;
    if (location == MI_QMM_HOST) {
        const size_t yoff = align_up(xbytes, 256);
        if ((rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, yoff + ybytes))) return rc;
        dx = (const float *)ctx->io_buf;
        dy = (float *)((char *)ctx->io_buf + yoff);
        HIP_TRY(hipMemcpyAsync((void *)dx, x, xbytes, hipMemcpyHostToDevice, ctx->stream));
    }
    HIP_TRY(launch_plain(w->dev, dx, n, dy, xc, ctx->num_cus, ctx->stream, force));
    if (location == MI_QMM_HOST) {
        HIP_TRY(hipMemcpyAsync(y, dy, ybytes, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
    }
    return MI_QMM_OK;
}

int plain_route(const mi_qmm_weight *w, int64_t n) {
    switch (plain_kind(w->dev.type, w->dev.K, w->dev.M, n)) {
    case 1: case 4: return MI_QMM_ROUTE_PLAIN_GEMV;
    case 5: return MI_QMM_ROUTE_PLAIN_SKINNY;
    case 2: return MI_QMM_ROUTE_PLAIN_GEMM;
    case 3: return MI_QMM_ROUTE_PLAIN_NAIVE;
    default: return 0;
    }
}

// Q5_K at three to eight activation rows on device pointers: whether the streaming kernel multiplies the blocks as they
// are by quantized planes of x (a rule of the shape alone), and the two launches of that product.
bool q5k_native_planes(const mi_qmm_weight *w, int64_t n, int path) {
    // measured against the doubled rows (us): 1024 x 4096 at 3 / 4 / 5 / 8 rows 10.5 / 10.9 / 11.6 / 13.0 -> 8.4 / 9.0 / 9.5 / 11.5;
    // 4096 x 14336 at 2 / 3 / 4 / 5 / 6 / 7 / 8: 22.8 / 22.6 / 22.7 / 25.2 / 25.8 / 26.7 / 27.2 -> 17.3 / 18.9 / 18.9 / 20.8 / 22.6 / 26.2 / 28.3;
    // 14336 x 4096 at 3 / 4 / 5 / 6 / 7 / 8: 20.0 / 20.5 / 21.0 / 22.2 / 22.2 / 22.2 -> 16.7 / 17.5 / 18.3 / 22.1 / 23.9 / 25.4
    const int64_t limit = w->k_user * w->dev.M <= (8 << 20) ? 8 : 6;
    return w->repeat && w->has_native && n >= 2 && n <= limit && path != MI_QMM_PATH_GEMM && w->k_user % QKK == 0 &&
           w->k_user <= gemv_max_k(T_Q5_K);
}

int q5k_planes_product(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const float *dx, int64_t n, float *dy, void *planes) {
    const int64_t K = w->k_user;
    const ActPlanes p = plan_act(planes, T_Q8_K, K, n, false);
    HIP_TRY(launch_quantize_act(T_Q8_K, dx, K, n, p.qs, p.d, p.bsums, p.sd8, p.sd16, ctx->stream, nullptr, p.qf, p.bsf));
    DevAct a;
    a.qs = p.qs; a.d = p.d; a.bsums = p.bsums; a.sd8 = p.sd8; a.sd16 = p.sd16; a.qf = p.qf; a.bsf = p.bsf; a.K = K; a.N = (int)n; a.type = T_Q8_K;
    HIP_TRY(launch_gemv(w->native, a, 0, (int)n, dy, w->dev.M, ctx->num_cus, ctx->stream));
    return MI_QMM_OK;
}

}  // namespace

extern "C" {

int mi_qmm_mulmat_path(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const float *x, int64_t n, float *y, int location,
                       int path) {
    if (n < 0) return fail(MI_QMM_ERR_INVALID, "n=%lld must be non-negative", (long long)n);
    int rc = check_product_args(ctx, w, location, path, /*allow_plain=*/true);
    if (rc) return rc;
    if (n > INT32_MAX) return fail(MI_QMM_ERR_UNSUPPORTED, "n too large");
    if (w->expand) {
        // the tensor of longer rows that stands for this one, against the expanded activations ([x | x] or [x | 0])
        mi_qmm_weight lo = *w;
        lo.expand = false;
        // Q5_K at one or two activation rows: the streaming kernel on the blocks as they are, x quantized in its prologue
        const bool q5_gemv = w->repeat && w->has_native && n >= 1 && n <= 2 && path != MI_QMM_PATH_GEMM &&
                             gemv_f32_supported(T_Q5_K, w->k_user, w->dev.M, (int)n);
        // Q5_K at three to eight activation rows: x quantized once at its own length, then the streaming kernel on the
        // blocks as they are (176 bytes a super-block read instead of the 288 of the doubled rows, no [x | x] copy)
        const bool q5_planes = !q5_gemv && q5k_native_planes(w, n, path);
        if (path == MI_QMM_PATH_QUERY && q5_gemv) return MI_QMM_ROUTE_GEMV_F32;
        if (path == MI_QMM_PATH_QUERY && q5_planes) return MI_QMM_ROUTE_GEMV;
        if (path == MI_QMM_PATH_QUERY || n == 0) return mi_qmm_mulmat_path(ctx, &lo, x, n, y, location, path);
        if (!x || !y) return fail(MI_QMM_ERR_INVALID, "x or y is NULL");
        if (q5_gemv) {
            const size_t xb5 = (size_t)(n * w->k_user) * 4, yb5 = (size_t)(n * w->dev.M) * 4;
            const float *dx5 = x;
            float *dy5 = y;
            if (location == MI_QMM_HOST) {
                const size_t yoff = align_up(xb5, 256);
                if ((rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, yoff + yb5))) return rc;
                dx5 = (const float *)ctx->io_buf;
                dy5 = (float *)((char *)ctx->io_buf + yoff);
                HIP_TRY(hipMemcpyAsync((void *)dx5, x, xb5, hipMemcpyHostToDevice, ctx->stream));
            }
            float *ys5[1] = {dy5};
            HIP_TRY(launch_gemv_f32_multi(&w->native, ys5, 1, dx5, (int)n, ctx->num_cus, ctx->stream));
            if (location == MI_QMM_HOST) {
                HIP_TRY(hipMemcpyAsync(y, dy5, yb5, hipMemcpyDeviceToHost, ctx->stream));
                HIP_TRY(hipStreamSynchronize(ctx->stream));
            }
            return MI_QMM_OK;
        }
        if (q5_planes) {
            const int64_t K5 = w->k_user, M5 = w->dev.M;
            const size_t xb5 = (size_t)(n * K5) * 4, yb5 = (size_t)(n * M5) * 4;
            const ActPlanes probe5 = plan_act(nullptr, T_Q8_K, K5, n, false);
            if ((rc = reserve(ctx, &ctx->act_buf, &ctx->act_cap, probe5.total))) return rc;
            const float *dx5 = x;
            float *dy5 = y;
            if (location == MI_QMM_HOST) {
                const size_t yoff = align_up(xb5, 256);
                if ((rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, yoff + yb5))) return rc;
                dx5 = (const float *)ctx->io_buf;
                dy5 = (float *)((char *)ctx->io_buf + yoff);
                HIP_TRY(hipMemcpyAsync((void *)dx5, x, xb5, hipMemcpyHostToDevice, ctx->stream));
            }
            if ((rc = q5k_planes_product(ctx, w, dx5, n, dy5, ctx->act_buf))) return rc;
            if (location == MI_QMM_HOST) {
                HIP_TRY(hipMemcpyAsync(y, dy5, yb5, hipMemcpyDeviceToHost, ctx->stream));
                HIP_TRY(hipStreamSynchronize(ctx->stream));
            }
            return MI_QMM_OK;
        }
        const size_t xb = (size_t)(n * w->k_user) * 4, xxb = (size_t)(n * w->dev.K) * 4, yb = (size_t)(n * w->dev.M) * 4;
        const size_t o_raw = align_up(xxb, 256), o_y = o_raw + align_up(xb, 256);
        if ((rc = reserve(ctx, &ctx->dup_buf, &ctx->dup_cap, location == MI_QMM_HOST ? o_y + yb : xxb))) return rc;
        float *xx = (float *)ctx->dup_buf;
        const float *dx = x;
        float *dy = y;
        if (location == MI_QMM_HOST) {
            dx = (const float *)((char *)ctx->dup_buf + o_raw);
            dy = (float *)((char *)ctx->dup_buf + o_y);
            HIP_TRY(hipMemcpyAsync((void *)dx, x, xb, hipMemcpyHostToDevice, ctx->stream));
        }
        HIP_TRY(launch_expand_rows(dx, w->k_user, w->dev.K, n, w->repeat, xx, ctx->stream));
        if ((rc = mi_qmm_mulmat_path(ctx, &lo, xx, n, dy, MI_QMM_DEVICE, path))) return rc;
        if (location == MI_QMM_HOST) {
            HIP_TRY(hipMemcpyAsync(y, dy, yb, hipMemcpyDeviceToHost, ctx->stream));
            HIP_TRY(hipStreamSynchronize(ctx->stream));
        }
        return MI_QMM_OK;
    }
    if (path == MI_QMM_PATH_QUERY) {  // which kernel mi_qmm_mulmat would take; nothing is launched, x and y may be NULL
        if (n == 0) return fail(MI_QMM_ERR_INVALID, "a product of no columns has no route");
        if (plain_type(w->dev.type)) {
            const int route = plain_route(w, n);
            return route ? route : fail(MI_QMM_ERR_UNSUPPORTED, "no kernel for this shape");
        }
        const char *why = nullptr;
        const int route = route_f32(ctx, w, n, MI_QMM_PATH_AUTO, &why);
        return route ? route : fail(MI_QMM_ERR_UNSUPPORTED, "%s", why);
    }
    if (n == 0) return MI_QMM_OK;
    if (!x || !y) return fail(MI_QMM_ERR_INVALID, "x or y is NULL");
    if (plain_type(w->dev.type)) return plain_mulmat(ctx, w, x, n, y, location, path, nullptr, 0);

    const int64_t K = w->dev.K, M = w->dev.M;
    const int q8 = mi_qmm_vec_dot_type(w->dev.type);
    const bool f16 = wants_f16_planes(w->dev.type, n);
    const ActPlanes probe = plan_act(nullptr, q8, K, n, f16);
    if ((rc = reserve(ctx, &ctx->act_buf, &ctx->act_cap, probe.total))) return rc;
    const ActPlanes p = plan_act(ctx->act_buf, q8, K, n, f16);

    const size_t xbytes = (size_t)(n * K) * 4, ybytes = (size_t)(n * M) * 4;
    const float *dx = x;
    float *dy = y;
    if (location == MI_QMM_HOST) {
        const size_t yoff = align_up(xbytes, 256);
        if ((rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, yoff + ybytes))) return rc;
        dx = (const float *)ctx->io_buf;
        dy = (float *)((char *)ctx->io_buf + yoff);
        HIP_TRY(hipMemcpyAsync((void *)dx, x, xbytes, hipMemcpyHostToDevice, ctx->stream));
    }
    const int route = route_f32(ctx, w, n, path, nullptr);
    if (route == MI_QMM_ROUTE_GEMV_F32) {
        // decode: one launch, the GEMV quantizes x in its prologue
        float *ys[1] = {dy};
        HIP_TRY(launch_gemv_f32_multi(&gemv_dev(w, (int)n, true), ys, 1, dx, (int)n, ctx->num_cus, ctx->stream));
    } else if (route == MI_QMM_ROUTE_DEEP_F32) {
        // a few columns on a large Q4_K matrix: one launch, the workgroups quantize x themselves
        float *ys[1] = {dy};
        HIP_TRY(launch_deep16_f32(&w->dev, ys, 1, dx, (int)n, ctx->num_cus, ctx->stream));
    } else {
        HIP_TRY(launch_quantize_act(q8, dx, K, n, p.qs, p.d, p.bsums, p.sd8, p.sd16, ctx->stream, nullptr, p.qf, p.bsf));
        DevAct a;
        a.qs = p.qs; a.d = p.d; a.bsums = p.bsums; a.sd8 = p.sd8; a.sd16 = p.sd16; a.qf = p.qf; a.bsf = p.bsf; a.K = K; a.N = (int)n; a.type = q8;
        if ((rc = run_product(ctx, w, a, dy, path))) return rc;
    }
    if (location == MI_QMM_HOST) {
        HIP_TRY(hipMemcpyAsync(y, dy, ybytes, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
    }
    return MI_QMM_OK;
}

int mi_qmm_mulmat(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const float *x, int64_t n, float *y, int location) {
    return mi_qmm_mulmat_path(ctx, w, x, n, y, location, MI_QMM_PATH_AUTO);
}

// mi_qmm_mulmat on device pointers without any allocation: the quantized activation planes go to this
// device's copy of the static array `scratch` (ctx->static_scratch), never to the ctx's growable buffers,
// and the tiled GEMM runs without its K-split workspace.  Same kernels as mi_qmm_mulmat otherwise.
static int noalloc_core(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const float *x, int64_t n, float *y, void *sbase, size_t sbytes) {
    if (n < 0) return fail(MI_QMM_ERR_INVALID, "n=%lld must be non-negative", (long long)n);
    int rc = check_product_args(ctx, w, MI_QMM_DEVICE, MI_QMM_PATH_AUTO, /*allow_plain=*/true);
    if (rc) return rc;
    if (n == 0) return MI_QMM_OK;
    if (!x || !y) return fail(MI_QMM_ERR_INVALID, "x or y is NULL");
    if (n > INT32_MAX) return fail(MI_QMM_ERR_UNSUPPORTED, "n too large");
    if (w->expand) {
        if (w->repeat && w->has_native && n <= 2 && gemv_f32_supported(T_Q5_K, w->k_user, w->dev.M, (int)n)) {
            float *ys5[1] = {y};  // Q5_K at one or two rows: the streaming kernel on the blocks as they are, no scratch
            HIP_TRY(launch_gemv_f32_multi(&w->native, ys5, 1, x, (int)n, ctx->num_cus, ctx->stream));
            return MI_QMM_OK;
        }
        if (q5k_native_planes(w, n, MI_QMM_PATH_AUTO)) {
            const ActPlanes probe5 = plan_act(nullptr, T_Q8_K, w->k_user, n, false);
            if (probe5.total > sbytes)
                return fail(MI_QMM_ERR_UNSUPPORTED, "n=%lld rows of k=%lld need %zu bytes of quantized activations; the static scratch of "
                            "mi_qmm_mulmat_noalloc holds %zu (use mi_qmm_mulmat)", (long long)n, (long long)w->k_user, probe5.total, sbytes);
            return q5k_planes_product(ctx, w, x, n, y, sbase);
        }
        // the expanded activations at the end of the scratch, the quantized planes of the product in front of them
        mi_qmm_weight lo = *w;
        lo.expand = false;
        const size_t xx_bytes = align_up((size_t)(n * w->dev.K) * 4, 256);
        if (xx_bytes + 256 > sbytes)
            return fail(MI_QMM_ERR_UNSUPPORTED, "n=%lld rows of k=%lld of this product need %zu bytes for the expanded activations alone; the "
                        "static scratch of mi_qmm_mulmat_noalloc holds %zu (use mi_qmm_mulmat)", (long long)n, (long long)w->k_user, xx_bytes, sbytes);
        float *xx = (float *)((char *)sbase + (sbytes - xx_bytes) / 256 * 256);
        HIP_TRY(launch_expand_rows(x, w->k_user, w->dev.K, n, w->repeat, xx, ctx->stream));
        return noalloc_core(ctx, &lo, xx, n, y, sbase, (sbytes - xx_bytes) / 256 * 256);
    }
    if (plain_type(w->dev.type))
        return plain_mulmat(ctx, w, x, n, y, MI_QMM_DEVICE, MI_QMM_PATH_AUTO, sbase, sbytes);
    const int64_t K = w->dev.K, M = w->dev.M;
    const int q8 = mi_qmm_vec_dot_type(w->dev.type);
    if (n <= 8 && !wants_skinny(w->dev.type, K, M, n, ctx->num_cus) && gemv_f32_supported(w->dev.type, K, M, (int)n)) {
        // decode: the GEMV quantizes x in its own prologue, into LDS -- no scratch at all
        float *ys[1] = {y};
        HIP_TRY(launch_gemv_f32_multi(&gemv_dev(w, (int)n, true), ys, 1, x, (int)n, ctx->num_cus, ctx->stream));
        return MI_QMM_OK;
    }
    if (deep_f32_one(ctx, w, n)) {
        float *ys[1] = {y};
        HIP_TRY(launch_deep16_f32(&w->dev, ys, 1, x, (int)n, ctx->num_cus, ctx->stream));
        return MI_QMM_OK;
    }
    const bool f16 = wants_f16_planes(w->dev.type, n);
    const ActPlanes probe = plan_act(nullptr, q8, K, n, f16);
    if (probe.total > sbytes)
        return fail(MI_QMM_ERR_UNSUPPORTED,
                    "n=%lld rows of k=%lld need %zu bytes of quantized activations; the static scratch of "
                    "mi_qmm_mulmat_noalloc holds %zu (use mi_qmm_mulmat)", (long long)n, (long long)K, probe.total,
                    sbytes);
    const ActPlanes p = plan_act(sbase, q8, K, n, f16);
    // every plane row below n is rewritten by the quantizer; rows n.. of the last 128-row tile keep what an
    // earlier call left there, and the GEMM drops the results of those rows
    HIP_TRY(launch_quantize_act(q8, x, K, n, p.qs, p.d, p.bsums, p.sd8, p.sd16, ctx->stream, nullptr, p.qf, p.bsf));
    DevAct a;
    a.qs = p.qs; a.d = p.d; a.bsums = p.bsums; a.sd8 = p.sd8; a.sd16 = p.sd16; a.qf = p.qf; a.bsf = p.bsf; a.K = K; a.N = (int)n; a.type = q8;
    return run_product(ctx, w, a, y, MI_QMM_PATH_AUTO, /*may_alloc=*/false);
}

int mi_qmm_mulmat_noalloc(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const float *x, int64_t n, float *y) {
    if (!ctx) return fail(MI_QMM_ERR_INVALID, "ctx is NULL");
    return noalloc_core(ctx, w, x, n, y, ctx->static_scratch, (size_t)MI_QMM_NOALLOC_SCRATCH_BYTES);
}

int mi_qmm_scratch_freeze(mi_qmm_ctx *ctx, int frozen) {
    int rc = check_ctx(ctx);
    if (rc) return rc;
    ctx->scratch_frozen = frozen != 0;
    return MI_QMM_OK;
}

}  // extern "C"

namespace {

// mi_qmm_mulmat_multi and mi_qmm_mulmat_produced: several weights of one K against the same activations,
// which may first go through a producer (prod: kind, aux and eps as the caller gave them, aux in `location`).
// q, k and v of an attention block, or gate and up of a feed-forward block, at prefill batch sizes: one launch of the
// fp16 GEMM when together they fill the machine.  A matrix that a launch of its own would cut into K slices keeps that cut
// (the order of its fp32 sums must not depend on how the product was asked for), so it rules the joint launch out.
// Of a only the type, K, N and the presence of the fp16 planes are read.
bool f16_multi_ok(const mi_qmm_ctx *ctx, const mi_qmm_weight *const *ws, int count, const DevAct &a) {
    if (count < 2 || count > 4 || a.type != T_Q8_K) return false;
    DevWeight dw[4];
    for (int i = 0; i < count; i++) dw[i] = ws[i]->dev;
    if (!gemm_f16_multi_wanted(dw, count, a, ctx->num_cus)) return false;
    for (int i = 0; i < count; i++)
        if (!gemm_f16_wanted(dw[i], a, ctx->num_cus) && gemm_workspace_floats(dw[i].type, dw[i].K, dw[i].M, a.N, ctx->num_cus) != 0)
            return false;
    return true;
}

int mulmat_multi_impl(mi_qmm_ctx *ctx, const mi_qmm_weight *const *ws, int count, const Produce *prod, const float *x,
                      int64_t n, float *const *ys, int location) {
    if (!ws || !ys || count < 1) return fail(MI_QMM_ERR_INVALID, "ws/ys is NULL or count < 1");
    for (int i = 0; i < count; i++)
        if (!ws[i] || !ys[i]) return fail(MI_QMM_ERR_INVALID, "ws[%d] or ys[%d] is NULL", i, i);
    if (n < 0) return fail(MI_QMM_ERR_INVALID, "n=%lld must be non-negative", (long long)n);
    bool same_type = true;
    for (int i = 1; i < count; i++) {
        if (ws[i]->dev.K != ws[0]->dev.K)
            return fail(MI_QMM_ERR_INVALID, "ws[%d] has k=%lld, ws[0] has k=%lld: one x cannot serve both", i,
                        (long long)ws[i]->dev.K, (long long)ws[0]->dev.K);
        same_type = same_type && ws[i]->dev.type == ws[0]->dev.type;
    }
    int rc = check_product_args(ctx, ws[0], location, MI_QMM_PATH_AUTO);
    if (rc) return rc;
    for (int i = 0; i < count; i++) {
        if (ws[i]->device != ctx->device) return fail(MI_QMM_ERR_INVALID, "ws[%d] is on another device", i);
        if (plain_type(ws[i]->dev.type) || ws[i]->expand)
            return fail(MI_QMM_ERR_UNSUPPORTED, "ws[%d] is of a type that only mi_qmm_mulmat multiplies (F32 / F16 / BF16 / Q5_K)", i);
    }
    Produce pr{PRODUCE_NONE, nullptr, 0.f, nullptr};
    if (prod) pr = *prod;
    if (pr.kind == PRODUCE_SWIGLU && !pr.aux && n > 0) return fail(MI_QMM_ERR_INVALID, "SwiGLU needs the up operand");
    if (pr.kind == PRODUCE_RMSNORM && !(pr.eps >= 0.f)) return fail(MI_QMM_ERR_INVALID, "eps must be non-negative");
    if (n == 0) return MI_QMM_OK;
    if (!x) return fail(MI_QMM_ERR_INVALID, "x is NULL");
    if (n > INT32_MAX) return fail(MI_QMM_ERR_UNSUPPORTED, "n too large");
    const int64_t K = ws[0]->dev.K;
    int64_t total_m = 0;
    for (int i = 0; i < count; i++) total_m += ws[i]->dev.M;

    // x, the producer's operand and the outputs on the device
    const size_t xbytes = (size_t)(n * K) * 4;
    const size_t auxbytes = !pr.aux ? 0 : pr.kind == PRODUCE_SWIGLU ? xbytes : (size_t)K * 4;
    const float *dx = x;
    std::vector<float *> dys(ys, ys + count);
    if (location == MI_QMM_HOST) {
        std::vector<size_t> offs(count + 1);
        const size_t auxoff = align_up(xbytes, 256);
        offs[0] = auxoff + align_up(auxbytes, 256);
        for (int i = 0; i < count; i++) offs[i + 1] = offs[i] + align_up((size_t)(n * ws[i]->dev.M) * 4, 256);
        if ((rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, offs[count]))) return rc;
        dx = (const float *)ctx->io_buf;
        for (int i = 0; i < count; i++) dys[i] = (float *)((char *)ctx->io_buf + offs[i]);
        HIP_TRY(hipMemcpyAsync((void *)dx, x, xbytes, hipMemcpyHostToDevice, ctx->stream));
        if (auxbytes) {
            float *daux = (float *)((char *)ctx->io_buf + auxoff);
            HIP_TRY(hipMemcpyAsync(daux, pr.aux, auxbytes, hipMemcpyHostToDevice, ctx->stream));
            pr.aux = daux;
        }
    }

    bool skinny = false;
    for (int i = 0; i < count; i++) skinny = skinny || wants_skinny(ws[i]->dev.type, K, ws[i]->dev.M, n, ctx->num_cus);
    const bool in_kernel = same_type && !skinny && count <= gemv_max_multi() && n <= 8 &&
                           (pr.kind == PRODUCE_NONE ? gemv_f32_supported(ws[0]->dev.type, K, total_m, (int)n)
                                                    : n == 1 && gemv_produce_supported(ws[0]->dev.type, K, total_m));
    // a few columns on large Q4_K matrices: one launch of the deep kernel, whose workgroups quantize x themselves --
    // when every matrix would take that kernel alone too (its sums do not depend on what shares the launch)
    bool deep_f32 = same_type && !in_kernel && pr.kind == PRODUCE_NONE && n <= 8 && count <= 4 &&
                    deep16_f32_wanted(ws[0]->dev.type, K, total_m, (int)n, ctx->num_cus);
    for (int i = 0; deep_f32 && i < count; i++) deep_f32 = deep16_wanted(ws[i]->dev.type, K, ws[i]->dev.M, (int)n, ctx->num_cus);
    if (in_kernel) {
        // decode: one launch over the concatenated rows, the kernel produces and quantizes x in its prologue
        DevWeight dw[8];
        for (int i = 0; i < count; i++) dw[i] = ws[i]->dev;
        HIP_TRY(launch_gemv_f32_multi(dw, dys.data(), count, dx, (int)n, ctx->num_cus, ctx->stream,
                                      pr.kind == PRODUCE_NONE ? nullptr : &pr));
    } else if (deep_f32) {
        DevWeight dw[4];
        for (int i = 0; i < count; i++) dw[i] = ws[i]->dev;
        HIP_TRY(launch_deep16_f32(dw, dys.data(), count, dx, (int)n, ctx->num_cus, ctx->stream));
    } else {
        // x is produced and quantized once per activation format (Q8_0 / Q8_K) in use; weights of one type
        // then share GEMV launches four at a time, everything else goes out one product at a time
        size_t act_need = 0;
        bool f16 = false;
        for (int i = 0; i < count; i++) f16 = f16 || wants_f16_planes(ws[i]->dev.type, n);
        for (int i = 0; i < count; i++) {
            const size_t t = plan_act(nullptr, mi_qmm_vec_dot_type(ws[i]->dev.type), K, n, f16).total;
            act_need = t > act_need ? t : act_need;
        }
        if ((rc = reserve(ctx, &ctx->act_buf, &ctx->act_cap, act_need + align_up((size_t)n * 4, 256)))) return rc;
        if (pr.kind == PRODUCE_RMSNORM) {
            float *scales = (float *)((char *)ctx->act_buf + act_need);
            HIP_TRY(launch_rms_norm(dx, nullptr, pr.eps, K, n, scales, nullptr, ctx->stream));
            pr.row_scale = scales;
        }
        for (int q8 : {(int)T_Q8_0, (int)T_Q8_K}) {
            std::vector<int> idx;
            for (int i = 0; i < count; i++)
                if (mi_qmm_vec_dot_type(ws[i]->dev.type) == q8) idx.push_back(i);
            if (idx.empty()) continue;
            const ActPlanes p = plan_act(ctx->act_buf, q8, K, n, f16);
            HIP_TRY(launch_quantize_act(q8, dx, K, n, p.qs, p.d, p.bsums, p.sd8, p.sd16, ctx->stream,
                                        pr.kind == PRODUCE_NONE ? nullptr : &pr, p.qf, p.bsf));
            DevAct a;
            a.qs = p.qs; a.d = p.d; a.bsums = p.bsums; a.sd8 = p.sd8; a.sd16 = p.sd16; a.qf = p.qf; a.bsf = p.bsf; a.K = K; a.N = (int)n; a.type = q8;
            size_t j = 0;
            if (q8 == T_Q8_K && idx.size() == (size_t)count && f16_multi_ok(ctx, ws, count, a)) {
                DevWeight dw[4];
                for (int i = 0; i < count; i++) dw[i] = ws[i]->dev;
                HIP_TRY(launch_gemm_f16_multi(dw, dys.data(), count, a, ctx->num_cus, ctx->stream));
                j = idx.size();
            }
            while (j < idx.size()) {
                const mi_qmm_weight *w0 = ws[idx[j]];
                size_t e = j + 1;
                if (n <= 8 && !wants_skinny(w0->dev.type, K, w0->dev.M, n, ctx->num_cus) && K <= gemv_max_k(w0->dev.type))
                    while (e < idx.size() && e - j < (size_t)gemv_max_multi() && ws[idx[e]]->dev.type == w0->dev.type &&
                           !wants_skinny(w0->dev.type, K, ws[idx[e]]->dev.M, n, ctx->num_cus))
                        e++;
                // matrices on the skinny MFMA kernels (q, k and v of a layer at 3..16 columns): one launch
                // over as many of them as keep the kernel and K cut of a launch of their own
                size_t es = j + 1;
                {
                    DevWeight dw[8];
                    dw[0] = w0->dev;
                    while (es < idx.size() && es - j < 8) {
                        dw[es - j] = ws[idx[es]]->dev;
                        const bool ok = q8 == T_Q8_0 ? skinny32_multi_supports(dw, (int)(es - j + 1), (int)n, ctx->num_cus)
                                                     : skinny_multi_supports(dw, (int)(es - j + 1), (int)n, ctx->num_cus);
                        if (!ok) break;
                        es++;
                    }
                }
                if (e - j == 1 && es - j > 1 && (q8 == T_Q8_0 || (a.sd8 && a.sd16)) && wants_skinny(w0->dev.type, K, w0->dev.M, n, ctx->num_cus)) {
                    DevWeight dw[8];
                    float *out[8];
                    for (size_t t = j; t < es; t++) { dw[t - j] = ws[idx[t]]->dev; out[t - j] = dys[idx[t]]; }
                    if (q8 == T_Q8_0) HIP_TRY(launch_skinny32_multi(dw, out, (int)(es - j), a, (int)n, ctx->num_cus, ctx->stream));
                    else HIP_TRY(launch_skinny_multi(dw, out, (int)(es - j), a, (int)n, ctx->num_cus, ctx->stream));
                    e = es;
                } else if (e - j > 1) {
                    DevWeight dw[8];
                    float *out[8];
                    for (size_t t = j; t < e; t++) { dw[t - j] = ws[idx[t]]->dev; out[t - j] = dys[idx[t]]; }
                    HIP_TRY(launch_gemv_multi(dw, out, (int)(e - j), a, 0, (int)n, ctx->num_cus, ctx->stream));
                } else if ((rc = run_product(ctx, w0, a, dys[idx[j]], MI_QMM_PATH_AUTO))) {
                    return rc;
                }
                j = e;
            }
        }
    }
    if (location == MI_QMM_HOST) {
        for (int i = 0; i < count; i++)
            HIP_TRY(hipMemcpyAsync(ys[i], dys[i], (size_t)(n * ws[i]->dev.M) * 4, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
    }
    return MI_QMM_OK;
}

// x, y (and more) of `bytes` each between the caller's location and the device: staged through io_buf for
// host callers.  Returns device pointers in dptr[]; the first n_in are copied in.
int stage_in(mi_qmm_ctx *ctx, int location, const void *const *src, const size_t *bytes, int n_in, int n_total,
             void **dptr) {
    if (location == MI_QMM_DEVICE) {
        for (int i = 0; i < n_total; i++) dptr[i] = const_cast<void *>(src[i]);
        return MI_QMM_OK;
    }
    size_t off = 0, offs[8];
    for (int i = 0; i < n_total; i++) { offs[i] = off; off += align_up(bytes[i], 256); }
    int rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, off);
    if (rc) return rc;
    for (int i = 0; i < n_total; i++) {
        dptr[i] = (char *)ctx->io_buf + offs[i];
        if (i < n_in && src[i] && bytes[i])
            HIP_TRY(hipMemcpyAsync(dptr[i], src[i], bytes[i], hipMemcpyHostToDevice, ctx->stream));
    }
    return MI_QMM_OK;
}

int check_elementwise_args(mi_qmm_ctx *ctx, int64_t k, int64_t n, int location) {
    if (location != MI_QMM_HOST && location != MI_QMM_DEVICE)
        return fail(MI_QMM_ERR_INVALID, "location must be MI_QMM_HOST or MI_QMM_DEVICE");
    if (k < 0 || n < 0) return fail(MI_QMM_ERR_INVALID, "k=%lld n=%lld must be non-negative", (long long)k, (long long)n);
    if (k % 4) return fail(MI_QMM_ERR_UNSUPPORTED, "k=%lld must be a multiple of 4", (long long)k);
    if (n > INT32_MAX) return fail(MI_QMM_ERR_UNSUPPORTED, "n too large");
    return check_ctx(ctx);
}

}  // namespace

extern "C" {

int mi_qmm_mulmat_multi(mi_qmm_ctx *ctx, const mi_qmm_weight *const *ws, int count, const float *x, int64_t n,
                        float *const *ys, int location) {
    bool plain = false;
    for (int i = 0; ws && ys && i < count; i++) plain = plain || (ws[i] && (plain_type(ws[i]->dev.type) || ws[i]->expand));
    if (plain) {
        // unquantized and Q5_K weights have no joint kernels: one product after the other, each as mi_qmm_mulmat gives it
        auto user_k = [](const mi_qmm_weight *w) { return w->expand ? w->k_user : w->dev.K; };
        for (int i = 0; i < count; i++) {
            if (!ws[i] || !ys[i]) return fail(MI_QMM_ERR_INVALID, "ws[%d] or ys[%d] is NULL", i, i);
            if (user_k(ws[i]) != user_k(ws[0]))
                return fail(MI_QMM_ERR_INVALID, "ws[%d] has k=%lld, ws[0] has k=%lld: one x cannot serve both", i,
                            (long long)user_k(ws[i]), (long long)user_k(ws[0]));
        }
        for (int i = 0; i < count; i++) {
            const int rc = mi_qmm_mulmat(ctx, ws[i], x, n, ys[i], location);
            if (rc) return rc;
        }
        return MI_QMM_OK;
    }
    return mulmat_multi_impl(ctx, ws, count, nullptr, x, n, ys, location);
}

int mi_qmm_mulmat_produced(mi_qmm_ctx *ctx, const mi_qmm_weight *const *ws, int count, int producer, const float *aux,
                           float eps, const float *x, int64_t n, float *const *ys, int location) {
    if (producer != MI_QMM_PRODUCE_NONE && producer != MI_QMM_PRODUCE_RMSNORM && producer != MI_QMM_PRODUCE_SWIGLU)
        return fail(MI_QMM_ERR_INVALID, "unknown producer %d", producer);
    const Produce pr{producer, producer == MI_QMM_PRODUCE_NONE ? nullptr : aux, eps, nullptr};
    return mulmat_multi_impl(ctx, ws, count, &pr, x, n, ys, location);
}

int mi_qmm_mulmat_swiglu(mi_qmm_ctx *ctx, const mi_qmm_weight *w_gate, const mi_qmm_weight *w_up, int producer,
                         const float *aux, float eps, const float *x, int64_t n, float *h, int location) {
    if (!w_gate || !w_up) return fail(MI_QMM_ERR_INVALID, "w_gate or w_up is NULL");
    if (producer != MI_QMM_PRODUCE_NONE && producer != MI_QMM_PRODUCE_RMSNORM)
        return fail(MI_QMM_ERR_INVALID, "the producer in front of gate and up is none or RMSNorm, not %d", producer);
    if (w_gate->dev.K != w_up->dev.K || w_gate->dev.M != w_up->dev.M)
        return fail(MI_QMM_ERR_INVALID, "gate is %lld x %lld, up is %lld x %lld: the gating needs equal shapes",
                    (long long)w_gate->dev.M, (long long)w_gate->dev.K, (long long)w_up->dev.M, (long long)w_up->dev.K);
    if (n < 0) return fail(MI_QMM_ERR_INVALID, "n=%lld must be non-negative", (long long)n);
    int rc = check_product_args(ctx, w_gate, location, MI_QMM_PATH_AUTO);
    if (rc) return rc;
    if (w_up->device != ctx->device) return fail(MI_QMM_ERR_INVALID, "w_up is on another device");
    if (plain_type(w_up->dev.type) || w_up->expand) return fail(MI_QMM_ERR_UNSUPPORTED, "w_up is of a type that only mi_qmm_mulmat multiplies");
    if (producer == MI_QMM_PRODUCE_RMSNORM && !(eps >= 0.f)) return fail(MI_QMM_ERR_INVALID, "eps must be non-negative");
    if (n == 0) return MI_QMM_OK;
    if (!x || !h) return fail(MI_QMM_ERR_INVALID, "x or h is NULL");
    if (n > INT32_MAX) return fail(MI_QMM_ERR_UNSUPPORTED, "n too large");
    const int64_t K = w_gate->dev.K, M = w_gate->dev.M;
    const bool rms = producer == MI_QMM_PRODUCE_RMSNORM;
    const bool paired = n == 1 && w_gate->dev.type == w_up->dev.type && gemv_pair_supported(w_gate->dev.type, K, M, rms);
    // x, the norm weight, h and (unless both products and the gating are one launch) the two products
    const size_t ybytes = (size_t)(n * M) * 4;
    const size_t bytes[5] = {(size_t)(n * K) * 4, rms && aux ? (size_t)K * 4 : 0, ybytes, paired ? 0 : ybytes, paired ? 0 : ybytes};
    const void *src[5] = {x, aux, h, nullptr, nullptr};
    void *d[5];
    if (location == MI_QMM_HOST || paired) {
        if ((rc = stage_in(ctx, location, src, bytes, 2, 5, d))) return rc;
    } else {
        // device caller: only the two intermediate products need room
        d[0] = const_cast<float *>(x); d[1] = const_cast<float *>(aux); d[2] = h;
        if ((rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, 2 * align_up(ybytes, 256)))) return rc;
        d[3] = ctx->io_buf;
        d[4] = (char *)ctx->io_buf + align_up(ybytes, 256);
    }
    const Produce pr{producer, rms && aux ? (const float *)d[1] : nullptr, eps, nullptr};
    if (paired) {
        HIP_TRY(launch_gemv_pair_f32(w_gate->dev, w_up->dev, (const float *)d[0], (float *)d[2], ctx->stream, &pr));
    } else {
        const mi_qmm_weight *ws[2] = {w_gate, w_up};
        float *ys[2] = {(float *)d[3], (float *)d[4]};
        if ((rc = mulmat_multi_impl(ctx, ws, 2, &pr, (const float *)d[0], n, ys, MI_QMM_DEVICE))) return rc;
        HIP_TRY(launch_swiglu(ys[0], ys[1], n * M, (float *)d[2], ctx->stream));
    }
    if (location == MI_QMM_HOST) {
        HIP_TRY(hipMemcpyAsync(h, d[2], ybytes, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
    }
    return MI_QMM_OK;
}

int mi_qmm_rms_norm(mi_qmm_ctx *ctx, const float *x, const float *g, float eps, int64_t k, int64_t n, float *y,
                    int location) {
    int rc = check_elementwise_args(ctx, k, n, location);
    if (rc) return rc;
    if (!(eps >= 0.f)) return fail(MI_QMM_ERR_INVALID, "eps must be non-negative");
    if (k * n == 0) return MI_QMM_OK;
    if (!x || !y) return fail(MI_QMM_ERR_INVALID, "x or y is NULL");
    const size_t bytes[3] = {(size_t)(n * k) * 4, g ? (size_t)k * 4 : 0, (size_t)(n * k) * 4};
    const void *src[3] = {x, g, y};
    void *d[3];
    if ((rc = stage_in(ctx, location, src, bytes, 2, 3, d))) return rc;
    HIP_TRY(launch_rms_norm((const float *)d[0], g ? (const float *)d[1] : nullptr, eps, k, n, nullptr, (float *)d[2],
                            ctx->stream));
    if (location == MI_QMM_HOST) {
        HIP_TRY(hipMemcpyAsync(y, d[2], bytes[2], hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
    }
    return MI_QMM_OK;
}

int mi_qmm_swiglu(mi_qmm_ctx *ctx, const float *gate, const float *up, int64_t k, int64_t n, float *y, int location) {
    int rc = check_elementwise_args(ctx, k % 4 ? 4 * k : k, n, location);  // any k: the operation is elementwise
    if (rc) return rc;
    if (k < 0) return fail(MI_QMM_ERR_INVALID, "k=%lld must be non-negative", (long long)k);
    if (k * n == 0) return MI_QMM_OK;
    if (!gate || !y) return fail(MI_QMM_ERR_INVALID, "gate or y is NULL");
    const size_t b = (size_t)(n * k) * 4, bytes[3] = {b, up ? b : 0, b};
    const void *src[3] = {gate, up, y};
    void *d[3];
    if ((rc = stage_in(ctx, location, src, bytes, 2, 3, d))) return rc;
    HIP_TRY(launch_swiglu((const float *)d[0], up ? (const float *)d[1] : nullptr, n * k, (float *)d[2], ctx->stream));
    if (location == MI_QMM_HOST) {
        HIP_TRY(hipMemcpyAsync(y, d[2], b, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
    }
    return MI_QMM_OK;
}

}  // extern "C"

namespace {

// w2 / y2 (optional): a second stack of w's type and shape multiplied by the same activations and ids;
// x is quantized once for both and the decode launch covers both.
int mulmat_id_impl(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const mi_qmm_weight *w2, int n_expert, const float *x,
                   int b_cols, const int32_t *ids, int n_used, int64_t n_tokens, float *y, float *y2, int location,
                   const Produce *prod = nullptr) {
    int rc = check_product_args(ctx, w, location, MI_QMM_PATH_AUTO);
    if (rc) return rc;
    Produce pr{PRODUCE_NONE, nullptr, 0.f, nullptr};
    if (prod) pr = *prod;
    if (pr.kind == PRODUCE_SWIGLU && !pr.aux && n_tokens > 0) return fail(MI_QMM_ERR_INVALID, "SwiGLU needs the up operand");
    if (pr.kind == PRODUCE_RMSNORM && !(pr.eps >= 0.f)) return fail(MI_QMM_ERR_INVALID, "eps must be non-negative");
    if (w2 && w2->expand) return fail(MI_QMM_ERR_UNSUPPORTED, "the second expert stack is of a type that only mi_qmm_mulmat multiplies");
    if (w2 && (w2->device != ctx->device || w2->dev.type != w->dev.type || w2->dev.K != w->dev.K || w2->dev.M != w->dev.M))
        return fail(MI_QMM_ERR_INVALID, "the two expert stacks differ in device, type or shape");
    if (n_expert < 1 || n_used < 1 || b_cols < 1 || n_tokens < 0)
        return fail(MI_QMM_ERR_INVALID, "n_expert=%d n_used=%d b_cols=%d n_tokens=%lld: all must be positive", n_expert,
                    n_used, b_cols, (long long)n_tokens);
    const int64_t K = w->dev.K;
    if (w->dev.M % n_expert)
        return fail(MI_QMM_ERR_INVALID, "the weight has %lld rows, not a multiple of n_expert=%d", (long long)w->dev.M,
                    n_expert);
    const int64_t M = w->dev.M / n_expert;
    if (n_tokens == 0) return MI_QMM_OK;
    if (!x || !ids || !y || (w2 && !y2)) return fail(MI_QMM_ERR_INVALID, "x, ids or y is NULL");
    const int64_t pairs = (int64_t)n_used * n_tokens, ncols = (int64_t)b_cols * n_tokens;
    if (n_expert > 4096 || pairs > (1 << 24) || ncols > (1 << 24))
        return fail(MI_QMM_ERR_UNSUPPORTED, "mulmat_id covers up to 4096 experts and 2^24 pairs");
    if (location == MI_QMM_HOST)
        for (int64_t p = 0; p < pairs; p++)
            if (ids[p] < 0 || ids[p] >= n_expert)
                return fail(MI_QMM_ERR_INVALID, "ids[%lld] = %d is outside 0..%d", (long long)p, ids[p], n_expert - 1);

    const int q8 = mi_qmm_vec_dot_type(w->dev.type);
    // batches with many pairs per expert: sort the pairs by expert and run the tiled GEMM per expert
    const bool gemm = gemm_id_supports(w->dev.type, K, M, pairs, n_expert) && ncols * K < ((int64_t)1 << 32);
    const int tile_w = gemm_id_tile_width(w->dev.type, pairs, n_expert);
    const int64_t max_tiles = gemm ? sort_pairs_max_tiles(pairs, n_expert, tile_w) : 0, sorted_rows = tile_w * max_tiles;
    const ActPlanes probe = plan_act(nullptr, q8, K, ncols);
    if ((rc = reserve(ctx, &ctx->act_buf, &ctx->act_cap, probe.total + align_up((size_t)ncols * 4, 256)))) return rc;
    const ActPlanes p = plan_act(ctx->act_buf, q8, K, ncols);
    float *row_scales = (float *)((char *)ctx->act_buf + probe.total);  // RMSNorm: one scale per activation row
    const size_t hist_ints = gemm ? sort_pairs_hist_ints(pairs, n_expert) : 0;
    const size_t scratch_ints = gemm ? (size_t)(1 + 2 * max_tiles + 2 * sorted_rows) + hist_ints : gemv_id_scratch_ints(pairs);
    if ((rc = reserve(ctx, &ctx->ws_buf, &ctx->ws_cap, scratch_ints * sizeof(int)))) return rc;

    const size_t xbytes = (size_t)(ncols * K) * 4, ibytes = (size_t)pairs * 4, ybytes = (size_t)(pairs * M) * 4;
    const size_t auxbytes = !pr.aux ? 0 : pr.kind == PRODUCE_SWIGLU ? xbytes : (size_t)K * 4;
    const float *dx = x;
    const int32_t *dids = ids;
    float *dy = y, *dy2 = y2;
    if (location == MI_QMM_HOST) {
        const size_t ioff = align_up(xbytes, 256), yoff = ioff + align_up(ibytes, 256), yoff2 = yoff + align_up(ybytes, 256);
        const size_t auxoff = yoff2 + align_up(w2 ? ybytes : 0, 256);
        if ((rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, auxoff + auxbytes))) return rc;
        if (auxbytes) {
            float *daux = (float *)((char *)ctx->io_buf + auxoff);
            HIP_TRY(hipMemcpyAsync(daux, pr.aux, auxbytes, hipMemcpyHostToDevice, ctx->stream));
            pr.aux = daux;
        }
        dx = (const float *)ctx->io_buf;
        dids = (const int32_t *)((char *)ctx->io_buf + ioff);
        dy = (float *)((char *)ctx->io_buf + yoff);
        if (w2) dy2 = (float *)((char *)ctx->io_buf + yoff2);
        HIP_TRY(hipMemcpyAsync((void *)dx, x, xbytes, hipMemcpyHostToDevice, ctx->stream));
        HIP_TRY(hipMemcpyAsync((void *)dids, ids, ibytes, hipMemcpyHostToDevice, ctx->stream));
    }
    // the quantization of x, through the producer if there is one
    auto quantize = [&]() -> hipError_t {
        if (pr.kind == PRODUCE_RMSNORM) {
            if (hipError_t e = launch_rms_norm(dx, nullptr, pr.eps, K, ncols, row_scales, nullptr, ctx->stream)) return e;
            pr.row_scale = row_scales;
        }
        return launch_quantize_act(q8, dx, K, ncols, p.qs, p.d, p.bsums, p.sd8, p.sd16, ctx->stream,
                                   pr.kind == PRODUCE_NONE ? nullptr : &pr);
    };
    if (gemm) {
        int *tiles = (int *)ctx->ws_buf, *src_col = tiles + 1 + 2 * max_tiles, *out_pair = src_col + sorted_rows;
        HIP_TRY(launch_sort_pairs(dids, (int)pairs, n_expert, n_used, b_cols, tile_w, tiles, src_col, out_pair,
                                  hist_ints ? out_pair + sorted_rows : nullptr, ctx->stream));
        HIP_TRY(quantize());
        DevAct as;
        as.qs = p.qs; as.d = p.d; as.bsums = p.bsums; as.sd8 = p.sd8; as.sd16 = p.sd16; as.qf = p.qf; as.bsf = p.bsf; as.K = K; as.N = (int)ncols; as.type = q8;
        HIP_TRY(launch_gemm_id(w->dev, n_expert, as, tiles, src_col, out_pair, max_tiles, tile_w, dy, ctx->stream));
        if (w2) HIP_TRY(launch_gemm_id(w2->dev, n_expert, as, tiles, src_col, out_pair, max_tiles, tile_w, dy2, ctx->stream));
        if (location == MI_QMM_HOST) {
            HIP_TRY(hipMemcpyAsync(y, dy, ybytes, hipMemcpyDeviceToHost, ctx->stream));
            if (w2) HIP_TRY(hipMemcpyAsync(y2, dy2, ybytes, hipMemcpyDeviceToHost, ctx->stream));
            HIP_TRY(hipStreamSynchronize(ctx->stream));
        }
        return MI_QMM_OK;
    }
    DevAct a{};
    a.K = K; a.N = (int)ncols; a.type = q8;
    // the matrix-core kernel addresses activation bytes with 32-bit offsets
    const bool skinny32 = skinny32_id_supports(w->dev.type, K, M, pairs, n_expert) && ncols * K < ((int64_t)1 << 32);
    const bool skinny = skinny32 || (skinny_id_supports(w->dev.type, K, M, pairs, n_expert) && ncols * K < ((int64_t)1 << 32));
    // only the streaming kernels have a row-length limit (the sorted GEMM and the matrix-core kernels walk any K)
    if (!skinny && K > gemv_max_k(w->dev.type))
        return fail(MI_QMM_ERR_UNSUPPORTED, "mulmat_id with this few pairs per expert streams the rows: k <= %lld for type %d",
                    (long long)gemv_max_k(w->dev.type), w->dev.type);
    const bool fused = !skinny && pr.kind != PRODUCE_RMSNORM &&
                       gemv_id_f32_supported(w->dev.type, K, M, pairs, n_expert, pr.kind == PRODUCE_SWIGLU);
    if (!fused) {
        HIP_TRY(quantize());
        a.qs = p.qs; a.d = p.d; a.bsums = p.bsums; a.sd8 = p.sd8; a.sd16 = p.sd16; a.qf = p.qf; a.bsf = p.bsf;
    }
    if (skinny32) {
        HIP_TRY(launch_skinny32_id(w->dev, n_expert, a, dids, n_used, (int)n_tokens, b_cols, dy, (int *)ctx->ws_buf,
                                   ctx->num_cus, ctx->stream));
        if (w2)
            HIP_TRY(launch_skinny32_id(w2->dev, n_expert, a, dids, n_used, (int)n_tokens, b_cols, dy2, (int *)ctx->ws_buf,
                                       ctx->num_cus, ctx->stream));
    } else if (skinny) {
        // a few pairs per expert and more: on the matrix cores, the experts' weights read once per 16 pairs
        HIP_TRY(launch_skinny_id(w->dev, n_expert, a, dids, n_used, (int)n_tokens, b_cols, dy, (int *)ctx->ws_buf,
                                 ctx->num_cus, ctx->stream));
        if (w2)
            HIP_TRY(launch_skinny_id(w2->dev, n_expert, a, dids, n_used, (int)n_tokens, b_cols, dy2, (int *)ctx->ws_buf,
                                     ctx->num_cus, ctx->stream));
    } else {
        // MXFP4 stacks: the streaming kernel reads them in their own layout where it takes that type at this shape
        const bool native = w->has_native && w->native.type == T_MXFP4 && (!w2 || w2->has_native) && K <= gemv_max_k(T_MXFP4) &&
                            (!fused || gemv_id_f32_supported(T_MXFP4, K, M, pairs, n_expert, pr.kind == PRODUCE_SWIGLU));
        HIP_TRY(launch_gemv_id(native ? w->native : w->dev, n_expert, a, fused ? dx : nullptr, dids, n_used, (int)n_tokens, b_cols, dy,
                               (int *)ctx->ws_buf, ctx->stream, w2 ? (native ? &w2->native : &w2->dev) : nullptr, dy2,
                               fused && pr.kind == PRODUCE_SWIGLU ? pr.aux : nullptr));
    }
    if (location == MI_QMM_HOST) {
        HIP_TRY(hipMemcpyAsync(y, dy, ybytes, hipMemcpyDeviceToHost, ctx->stream));
        if (w2) HIP_TRY(hipMemcpyAsync(y2, dy2, ybytes, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
    }
    return MI_QMM_OK;
}

}  // namespace

extern "C" {

int mi_qmm_mulmat_id(mi_qmm_ctx *ctx, const mi_qmm_weight *w, int n_expert, const float *x, int b_cols,
                     const int32_t *ids, int n_used, int64_t n_tokens, float *y, int location) {
    if (w && w->expand && !w->repeat && ctx && x && y && ids && n_tokens > 0 && n_used > 0 && b_cols > 0 && n_expert > 0 &&
        (location == MI_QMM_HOST || location == MI_QMM_DEVICE) && n_tokens * (int64_t)b_cols <= INT32_MAX) {
        // an expert stack whose rows were padded to whole 256-element steps (MXFP4 experts of K = 2880): the activation
        // rows are padded likewise, on the device, and the product runs on device pointers
        int rc = check_ctx(ctx);
        if (rc) return rc;
        mi_qmm_weight lo = *w;
        lo.expand = false;
        const int64_t rows = n_tokens * b_cols, pairs = n_tokens * n_used;
        const size_t xb = (size_t)(rows * w->k_user) * 4, xxb = (size_t)(rows * w->dev.K) * 4;
        const size_t yb = (size_t)(pairs * (w->dev.M / n_expert)) * 4, ib = (size_t)pairs * 4;
        const size_t o_raw = align_up(xxb, 256), o_y = o_raw + align_up(xb, 256), o_ids = o_y + align_up(yb, 256);
        if ((rc = reserve(ctx, &ctx->dup_buf, &ctx->dup_cap, location == MI_QMM_HOST ? o_ids + ib : xxb))) return rc;
        float *xx = (float *)ctx->dup_buf;
        const float *dx = x;
        float *dy = y;
        const int32_t *dids = ids;
        if (location == MI_QMM_HOST) {
            for (int64_t p = 0; p < pairs; p++)
                if (ids[p] < 0 || ids[p] >= n_expert)
                    return fail(MI_QMM_ERR_INVALID, "ids[%lld] = %d is outside 0..%d", (long long)p, ids[p], n_expert - 1);
            dx = (const float *)((char *)ctx->dup_buf + o_raw);
            dy = (float *)((char *)ctx->dup_buf + o_y);
            dids = (const int32_t *)((char *)ctx->dup_buf + o_ids);
            HIP_TRY(hipMemcpyAsync((void *)dx, x, xb, hipMemcpyHostToDevice, ctx->stream));
            HIP_TRY(hipMemcpyAsync((void *)dids, ids, ib, hipMemcpyHostToDevice, ctx->stream));
        }
        HIP_TRY(launch_expand_rows(dx, w->k_user, w->dev.K, rows, false, xx, ctx->stream));
        if ((rc = mulmat_id_impl(ctx, &lo, nullptr, n_expert, xx, b_cols, dids, n_used, n_tokens, dy, nullptr, MI_QMM_DEVICE))) return rc;
        if (location == MI_QMM_HOST) {
            HIP_TRY(hipMemcpyAsync(y, dy, yb, hipMemcpyDeviceToHost, ctx->stream));
            HIP_TRY(hipStreamSynchronize(ctx->stream));
        }
        return MI_QMM_OK;
    }
    return mulmat_id_impl(ctx, w, nullptr, n_expert, x, b_cols, ids, n_used, n_tokens, y, nullptr, location);
}

int mi_qmm_mulmat_id_multi(mi_qmm_ctx *ctx, const mi_qmm_weight *const *ws, int count, int n_expert, const float *x,
                           int b_cols, const int32_t *ids, int n_used, int64_t n_tokens, float *const *ys, int location) {
    if (!ws || !ys || count < 1) return fail(MI_QMM_ERR_INVALID, "ws/ys is NULL or count < 1");
    for (int i = 0; i < count; i++)
        if (!ws[i] || !ys[i]) return fail(MI_QMM_ERR_INVALID, "ws[%d] or ys[%d] is NULL", i, i);
    for (int i = 0; i < count;) {
        // stacks of one type and shape go out two at a time
        const bool pair = i + 1 < count && ws[i + 1]->dev.type == ws[i]->dev.type && ws[i + 1]->dev.K == ws[i]->dev.K &&
                          ws[i + 1]->dev.M == ws[i]->dev.M;
        int rc = mulmat_id_impl(ctx, ws[i], pair ? ws[i + 1] : nullptr, n_expert, x, b_cols, ids, n_used, n_tokens, ys[i],
                                pair ? ys[i + 1] : nullptr, location);
        if (rc) return rc;
        i += pair ? 2 : 1;
    }
    return MI_QMM_OK;
}

int mi_qmm_mulmat_id_produced(mi_qmm_ctx *ctx, const mi_qmm_weight *w, int n_expert, int producer, const float *aux,
                              float eps, const float *x, int b_cols, const int32_t *ids, int n_used, int64_t n_tokens,
                              float *y, int location) {
    if (producer != MI_QMM_PRODUCE_NONE && producer != MI_QMM_PRODUCE_RMSNORM && producer != MI_QMM_PRODUCE_SWIGLU)
        return fail(MI_QMM_ERR_INVALID, "unknown producer %d", producer);
    const Produce pr{producer, producer == MI_QMM_PRODUCE_NONE ? nullptr : aux, eps, nullptr};
    return mulmat_id_impl(ctx, w, nullptr, n_expert, x, b_cols, ids, n_used, n_tokens, y, nullptr, location, &pr);
}

int mi_qmm_mulmat_id_swiglu(mi_qmm_ctx *ctx, const mi_qmm_weight *w_gate, const mi_qmm_weight *w_up, int n_expert,
                            const float *x, int b_cols, const int32_t *ids, int n_used, int64_t n_tokens, float *h,
                            int location) {
    if (!w_gate || !w_up) return fail(MI_QMM_ERR_INVALID, "w_gate or w_up is NULL");
    int rc = check_product_args(ctx, w_gate, location, MI_QMM_PATH_AUTO);
    if (rc) return rc;
    if (w_up->device != ctx->device || w_up->dev.K != w_gate->dev.K || w_up->dev.M != w_gate->dev.M)
        return fail(MI_QMM_ERR_INVALID, "the gate and up stacks differ in device or shape");
    if (plain_type(w_up->dev.type) || w_up->expand) return fail(MI_QMM_ERR_UNSUPPORTED, "w_up is of a type that only mi_qmm_mulmat multiplies");
    if (n_expert < 1 || n_used < 1 || b_cols < 1 || n_tokens < 0)
        return fail(MI_QMM_ERR_INVALID, "n_expert=%d n_used=%d b_cols=%d n_tokens=%lld: all must be positive", n_expert,
                    n_used, b_cols, (long long)n_tokens);
    const int64_t K = w_gate->dev.K;
    if (w_gate->dev.M % n_expert)
        return fail(MI_QMM_ERR_INVALID, "the weight has %lld rows, not a multiple of n_expert=%d", (long long)w_gate->dev.M,
                    n_expert);
    const int64_t M = w_gate->dev.M / n_expert;
    if (n_tokens == 0) return MI_QMM_OK;
    if (!x || !ids || !h) return fail(MI_QMM_ERR_INVALID, "x, ids or h is NULL");
    const int64_t pairs = (int64_t)n_used * n_tokens, ncols = (int64_t)b_cols * n_tokens;
    if (n_expert > 4096 || pairs > (1 << 24) || ncols > (1 << 24))
        return fail(MI_QMM_ERR_UNSUPPORTED, "mulmat_id covers up to 4096 experts and 2^24 pairs");
    if (location == MI_QMM_HOST)
        for (int64_t p = 0; p < pairs; p++)
            if (ids[p] < 0 || ids[p] >= n_expert)
                return fail(MI_QMM_ERR_INVALID, "ids[%lld] = %d is outside 0..%d", (long long)p, ids[p], n_expert - 1);
    // decode-sized and both stacks of one type: one launch with the gating in its epilogue; else the two products
    // (which share their quantization and, at decode size, their launch) and the gating kernel
    const bool paired = w_gate->dev.type == w_up->dev.type && K <= gemv_max_k(w_gate->dev.type) &&
                        gemv_id_f32_supported(w_gate->dev.type, K, 2 * M, pairs, n_expert);
    const size_t hbytes = (size_t)(pairs * M) * 4;
    const size_t bytes[5] = {(size_t)(ncols * K) * 4, (size_t)pairs * 4, hbytes, paired ? 0 : hbytes, paired ? 0 : hbytes};
    const void *src[5] = {x, ids, h, nullptr, nullptr};
    void *d[5];
    if (paired) {
        if ((rc = stage_in(ctx, location, src, bytes, 2, 5, d))) return rc;
        HIP_TRY(launch_gemv_id_pair(w_gate->dev, w_up->dev, n_expert, (const float *)d[0], (const int *)d[1], n_used,
                                    (int)n_tokens, b_cols, (float *)d[2], ctx->stream));
        if (location == MI_QMM_HOST) {
            HIP_TRY(hipMemcpyAsync(h, d[2], hbytes, hipMemcpyDeviceToHost, ctx->stream));
            HIP_TRY(hipStreamSynchronize(ctx->stream));
        }
        return MI_QMM_OK;
    }
    // the two products into scratch of their own (mulmat_id_impl stages host operands through io_buf itself)
    if ((rc = reserve(ctx, &ctx->pair_buf, &ctx->pair_cap, 3 * align_up(hbytes, 256)))) return rc;
    float *yg = (float *)ctx->pair_buf, *yu = (float *)((char *)ctx->pair_buf + align_up(hbytes, 256));
    float *dh = location == MI_QMM_HOST ? (float *)((char *)ctx->pair_buf + 2 * align_up(hbytes, 256)) : h;
    const bool same = w_gate->dev.type == w_up->dev.type;
    if (location == MI_QMM_HOST) {
        // host operands: the products return host arrays; keep them on the device instead by staging here
        if ((rc = stage_in(ctx, location, src, bytes, 2, 2, d))) return rc;
        // io_buf now holds x and ids; mulmat_id_impl with device pointers does not touch io_buf
    } else {
        d[0] = const_cast<float *>(x); d[1] = const_cast<int32_t *>(ids);
    }
    if (same) {
        if ((rc = mulmat_id_impl(ctx, w_gate, w_up, n_expert, (const float *)d[0], b_cols, (const int32_t *)d[1], n_used, n_tokens,
                                 yg, yu, MI_QMM_DEVICE)))
            return rc;
    } else {
        if ((rc = mulmat_id_impl(ctx, w_gate, nullptr, n_expert, (const float *)d[0], b_cols, (const int32_t *)d[1], n_used,
                                 n_tokens, yg, nullptr, MI_QMM_DEVICE)))
            return rc;
        if ((rc = mulmat_id_impl(ctx, w_up, nullptr, n_expert, (const float *)d[0], b_cols, (const int32_t *)d[1], n_used,
                                 n_tokens, yu, nullptr, MI_QMM_DEVICE)))
            return rc;
    }
    HIP_TRY(launch_swiglu(yg, yu, pairs * M, dh, ctx->stream));
    if (location == MI_QMM_HOST) {
        HIP_TRY(hipMemcpyAsync(h, dh, hbytes, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
    }
    return MI_QMM_OK;
}

// ---- two-phase form ----------------------------------------------------------------------------------
int mi_qmm_act_create(mi_qmm_ctx *ctx, int q8_type, int64_t k, int64_t n_max, mi_qmm_act **out) {
    if (!out) return fail(MI_QMM_ERR_INVALID, "out is NULL");
    *out = nullptr;
    if (q8_type != T_Q8_0 && q8_type != T_Q8_K)
        return fail(MI_QMM_ERR_UNSUPPORTED, "activation type %d is not Q8_0 (8) or Q8_K (15)", q8_type);
    if (k <= 0 || n_max <= 0 || n_max > INT32_MAX)
        return fail(MI_QMM_ERR_INVALID, "k=%lld n_max=%lld must be positive", (long long)k, (long long)n_max);
    if (mi_qmm_row_size(q8_type, k) < 0)
        return fail(MI_QMM_ERR_INVALID, "k=%lld is not a multiple of the block size %lld of type %d",
                    (long long)k, (long long)mi_qmm_block_size(q8_type), q8_type);
    int rc = check_ctx(ctx);
    if (rc) return rc;
    mi_qmm_act *a = new (std::nothrow) mi_qmm_act();
    if (!a) return fail(MI_QMM_ERR_NOMEM, "host allocation failed");
    a->device = ctx->device; a->type = q8_type; a->k = k; a->n_max = n_max;
    a->f16 = q8_type == T_Q8_K && n_max > 64;  // any Q4_K weight may meet these rows: keep the fp16 planes too
    const ActPlanes probe = plan_act(nullptr, q8_type, k, n_max, a->f16);
    hipError_t e = hipMalloc(&a->base, probe.total + 256);
    if (e != hipSuccess) {
        delete a;
        return fail(MI_QMM_ERR_NOMEM, "hipMalloc(%zu) for activations: %s", probe.total, hipGetErrorString(e));
    }
    *out = a;
    return MI_QMM_OK;
}

void mi_qmm_act_free(mi_qmm_act *act) {
    if (!act) return;
    if (hipSetDevice(act->device) == hipSuccess && act->base) {
        (void)hipDeviceSynchronize();
        (void)hipFree(act->base);
    }
    delete act;
}

int mi_qmm_act_quantize(mi_qmm_ctx *ctx, mi_qmm_act *act, const float *x, int64_t n, int location) {
    if (!act) return fail(MI_QMM_ERR_INVALID, "act is NULL");
    if (n < 0 || n > act->n_max)
        return fail(MI_QMM_ERR_INVALID, "n=%lld outside 0..n_max=%lld", (long long)n, (long long)act->n_max);
    if (location != MI_QMM_HOST && location != MI_QMM_DEVICE)
        return fail(MI_QMM_ERR_INVALID, "location must be MI_QMM_HOST or MI_QMM_DEVICE");
    int rc = check_ctx(ctx);
    if (rc) return rc;
    if (act->device != ctx->device) return fail(MI_QMM_ERR_INVALID, "act and ctx are on different devices");
    act->n = n;
    if (n == 0) return MI_QMM_OK;
    if (!x) return fail(MI_QMM_ERR_INVALID, "x is NULL");
    // planes are carved for n_max so their addresses do not move between calls
    const ActPlanes p = plan_act(act->base, act->type, act->k, act->n_max, act->f16);
    const float *dx = x;
    if (location == MI_QMM_HOST) {
        const size_t xbytes = (size_t)(n * act->k) * 4;
        if ((rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, xbytes))) return rc;
        dx = (const float *)ctx->io_buf;
        HIP_TRY(hipMemcpyAsync((void *)dx, x, xbytes, hipMemcpyHostToDevice, ctx->stream));
    }
    HIP_TRY(launch_quantize_act(act->type, dx, act->k, n, p.qs, p.d, p.bsums, p.sd8, p.sd16, ctx->stream, nullptr, p.qf, p.bsf));
    if (location == MI_QMM_HOST) HIP_TRY(hipStreamSynchronize(ctx->stream));  // x may be reused by the caller
    return MI_QMM_OK;
}

int mi_qmm_mulmat_q8(mi_qmm_ctx *ctx, const mi_qmm_weight *w, const mi_qmm_act *act, float *y, int location,
                     int path) {
    if (!act) return fail(MI_QMM_ERR_INVALID, "act is NULL");
    int rc = check_product_args(ctx, w, location, path);
    if (rc) return rc;
    if (act->device != ctx->device) return fail(MI_QMM_ERR_INVALID, "act and ctx are on different devices");
    if (act->type != mi_qmm_vec_dot_type(w->dev.type) || act->k != w->dev.K)
        return fail(MI_QMM_ERR_INVALID, "act (type %d, k=%lld) does not match weight (type %d needs %d, k=%lld)",
                    act->type, (long long)act->k, w->dev.type, mi_qmm_vec_dot_type(w->dev.type), (long long)w->dev.K);
    const int64_t n = act->n, M = w->dev.M;
    if (n == 0) return path == MI_QMM_PATH_QUERY ? fail(MI_QMM_ERR_INVALID, "a product of no columns has no route") : MI_QMM_OK;
    const ActPlanes p = plan_act(act->base, act->type, act->k, act->n_max, act->f16);
    DevAct a;
    a.qs = p.qs; a.d = p.d; a.bsums = p.bsums; a.sd8 = p.sd8; a.sd16 = p.sd16; a.qf = p.qf; a.bsf = p.bsf; a.K = act->k; a.N = (int)n; a.type = act->type;
    if (path == MI_QMM_PATH_QUERY) {  // which kernel the product of these planes would take; nothing is launched
        const char *why = nullptr;
        const int route = route_planes(ctx, w, a, MI_QMM_PATH_AUTO, /*may_alloc=*/true, &why);
        return route ? route : fail(MI_QMM_ERR_UNSUPPORTED, "%s", why);
    }
    if (!y) return fail(MI_QMM_ERR_INVALID, "y is NULL");
    float *dy = y;
    const size_t ybytes = (size_t)(n * M) * 4;
    if (location == MI_QMM_HOST) {
        if ((rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, ybytes))) return rc;
        dy = (float *)ctx->io_buf;
    }
    if ((rc = run_product(ctx, w, a, dy, path))) return rc;
    if (location == MI_QMM_HOST) {
        HIP_TRY(hipMemcpyAsync(y, dy, ybytes, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
    }
    return MI_QMM_OK;
}

int mi_qmm_mulmat_q8_multi(mi_qmm_ctx *ctx, const mi_qmm_weight *const *ws, int count, const mi_qmm_act *act,
                           float *const *ys, int location) {
    if (!ctx) return fail(MI_QMM_ERR_INVALID, "ctx is NULL");  // ctx->num_cus is read before check_product_args below
    if (!ws || !ys || count < 1) return fail(MI_QMM_ERR_INVALID, "ws/ys is NULL or count < 1");
    if (!act) return fail(MI_QMM_ERR_INVALID, "act is NULL");
    for (int i = 0; i < count; i++)
        if (!ws[i] || !ys[i]) return fail(MI_QMM_ERR_INVALID, "ws[%d] or ys[%d] is NULL", i, i);
    bool same = true;
    for (int i = 1; i < count; i++)
        same = same && ws[i]->dev.type == ws[0]->dev.type && ws[i]->dev.K == ws[0]->dev.K;
    bool gemm_ok = same && count <= gemm_max_multi() && act->n >= 32;
    int64_t tiles = 0;
    for (int i = 0; gemm_ok && i < count; i++) {
        // a weight that would be cut into K slices in a launch of its own (long rows, few tiles) keeps that cut:
        // the joint launch never slices, and the order of the fp32 sums must not depend on how a product was asked for
        gemm_ok = gemm_supports(ws[i]->dev.type, ws[i]->dev.K, ws[i]->dev.M) &&
                  gemm_workspace_floats(ws[i]->dev.type, ws[i]->dev.K, ws[i]->dev.M, act->n, ctx->num_cus) == 0;
        tiles += (ws[i]->dev.M + 127) / 128 * ((act->n + 127) / 128);
    }
    // one launch pays when the tensors are too small to fill the machine one by one (q, k, v); large
    // ones (gate, up) run slightly faster back to back
    gemm_ok = gemm_ok && 2 * tiles < 3 * (int64_t)ctx->num_cus;
    for (int i = 0; gemm_ok && i < count; i++)  // so does a Q6_K weight that the 256-row kernel takes
        gemm_ok = gemm_q6k_slices(ws[i]->dev.type, ws[i]->dev.K, ws[i]->dev.M, act->n, ctx->num_cus) == 0;
    if (gemm_ok && act->f16) {  // a weight that the fp16 GEMM takes in a launch of its own keeps that kernel
        DevAct probe;
        probe.qs = nullptr; probe.d = nullptr; probe.bsums = nullptr; probe.sd8 = probe.sd16 = nullptr;
        probe.K = act->k; probe.N = (int)act->n; probe.type = act->type;
        probe.qf = probe.bsf = reinterpret_cast<const uint16_t *>(act->base);  // presence is all that is read
        for (int i = 0; gemm_ok && i < count; i++) gemm_ok = !gemm_f16_wanted(ws[i]->dev, probe, ctx->num_cus);
    }
    bool f16_ok = false;
    if (!gemm_ok && same && act->f16 && act->n >= 32) {
        DevAct probe;
        probe.qs = nullptr; probe.d = nullptr; probe.bsums = nullptr; probe.sd8 = probe.sd16 = nullptr;
        probe.K = act->k; probe.N = (int)act->n; probe.type = act->type;
        probe.qf = probe.bsf = reinterpret_cast<const uint16_t *>(act->base);  // presence is all that is read
        f16_ok = f16_multi_ok(ctx, ws, count, probe);
    }
    bool gemv_ok = !f16_ok && same && count <= gemv_max_multi() && act->n <= 8 && ws[0]->dev.K <= gemv_max_k(ws[0]->dev.type);
    for (int i = 0; gemv_ok && i < count; i++)  // from five or six columns up each weight goes to the skinny kernel
        gemv_ok = !wants_skinny(ws[i]->dev.type, ws[i]->dev.K, ws[i]->dev.M, act->n, ctx->num_cus);
    // K-quant matrices at 3..16 columns: one launch of a skinny MFMA kernel when it gives the same bits
    bool skinny_ok = false;
    if (!gemm_ok && !gemv_ok && same && count >= 2 && count <= 8 && act->n >= 1 && act->n <= 16 &&
        wants_skinny(ws[0]->dev.type, ws[0]->dev.K, ws[0]->dev.M, act->n, ctx->num_cus)) {
        DevWeight probe[8];
        for (int i = 0; i < count; i++) probe[i] = ws[i]->dev;
        skinny_ok = act->type == T_Q8_0 ? skinny32_multi_supports(probe, count, (int)act->n, ctx->num_cus)
                                        : skinny_multi_supports(probe, count, (int)act->n, ctx->num_cus);
    }
    if (!gemm_ok && !f16_ok && !gemv_ok && !skinny_ok) {
        for (int i = 0; i < count; i++) {
            int rc = mi_qmm_mulmat_q8(ctx, ws[i], act, ys[i], location, MI_QMM_PATH_AUTO);
            if (rc) return rc;
        }
        return MI_QMM_OK;
    }
    int rc = check_product_args(ctx, ws[0], location, MI_QMM_PATH_AUTO);
    if (rc) return rc;
    if (act->device != ctx->device) return fail(MI_QMM_ERR_INVALID, "act and ctx are on different devices");
    if (act->type != mi_qmm_vec_dot_type(ws[0]->dev.type) || act->k != ws[0]->dev.K)
        return fail(MI_QMM_ERR_INVALID, "act (type %d, k=%lld) does not match the weights (type %d, k=%lld)",
                    act->type, (long long)act->k, ws[0]->dev.type, (long long)ws[0]->dev.K);
    if (act->n == 0) return MI_QMM_OK;
    const ActPlanes p = plan_act(act->base, act->type, act->k, act->n_max, act->f16);
    DevAct a;
    a.qs = p.qs; a.d = p.d; a.bsums = p.bsums; a.sd8 = p.sd8; a.sd16 = p.sd16; a.qf = p.qf; a.bsf = p.bsf; a.K = act->k; a.N = (int)act->n; a.type = act->type;
    DevWeight dw[8];
    for (int i = 0; i < count; i++) {
        if (ws[i]->device != ctx->device) return fail(MI_QMM_ERR_INVALID, "ws[%d] is on another device", i);
        if (plain_type(ws[i]->dev.type) || ws[i]->expand)
            return fail(MI_QMM_ERR_UNSUPPORTED, "ws[%d] is of a type that only mi_qmm_mulmat multiplies (F32 / F16 / BF16 / Q5_K)", i);
        dw[i] = ws[i]->dev;
    }
    float *dys[8];
    size_t offs[9] = {0};
    for (int i = 0; i < count; i++) {
        dys[i] = ys[i];
        offs[i + 1] = offs[i] + align_up((size_t)(act->n * dw[i].M) * 4, 256);
    }
    if (location == MI_QMM_HOST) {
        if ((rc = reserve(ctx, &ctx->io_buf, &ctx->io_cap, offs[count]))) return rc;
        for (int i = 0; i < count; i++) dys[i] = (float *)((char *)ctx->io_buf + offs[i]);
    }
    if (f16_ok) HIP_TRY(launch_gemm_f16_multi(dw, dys, count, a, ctx->num_cus, ctx->stream));
    else if (gemm_ok) HIP_TRY(launch_gemm_multi(dw, dys, count, a, nullptr, 0, ctx->num_cus, ctx->stream));
    else if (skinny_ok && a.type == T_Q8_0) HIP_TRY(launch_skinny32_multi(dw, dys, count, a, (int)act->n, ctx->num_cus, ctx->stream));
    else if (skinny_ok) HIP_TRY(launch_skinny_multi(dw, dys, count, a, (int)act->n, ctx->num_cus, ctx->stream));
    else HIP_TRY(launch_gemv_multi(dw, dys, count, a, 0, (int)act->n, ctx->num_cus, ctx->stream));
    if (location == MI_QMM_HOST) {
        for (int i = 0; i < count; i++)
            HIP_TRY(hipMemcpyAsync(ys[i], dys[i], (size_t)(act->n * dw[i].M) * 4, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
    }
    return MI_QMM_OK;
}

}  // extern "C"

// ---- GGUF files ----------------------------------------------------------------------------------------
extern "C" {

int mi_qmm_gguf_open(const char *path, mi_qmm_gguf **out) {
    if (!out) return fail(MI_QMM_ERR_INVALID, "out is NULL");
    *out = nullptr;
    if (!path) return fail(MI_QMM_ERR_INVALID, "path is NULL");
    mi_qmm_gguf *g = new (std::nothrow) mi_qmm_gguf();
    if (!g) return fail(MI_QMM_ERR_NOMEM, "host allocation failed");
    const std::string err = g->file.open(path);
    if (!err.empty()) {
        delete g;
        const bool unsupported = err.find("unsupported") != std::string::npos;
        return fail(unsupported ? MI_QMM_ERR_UNSUPPORTED : MI_QMM_ERR_INVALID, "%s", err.c_str());
    }
    *out = g;
    return MI_QMM_OK;
}

void mi_qmm_gguf_close(mi_qmm_gguf *f) { delete f; }

int mi_qmm_gguf_info(const mi_qmm_gguf *f, int *version, int64_t *alignment, int64_t *data_offset, int64_t *num_kv,
                     int64_t *num_tensors) {
    if (!f) return fail(MI_QMM_ERR_INVALID, "gguf is NULL");
    if (version) *version = (int)f->file.version;
    if (alignment) *alignment = f->file.alignment;
    if (data_offset) *data_offset = (int64_t)f->file.data_offset;
    if (num_kv) *num_kv = (int64_t)f->file.kvs.size();
    if (num_tensors) *num_tensors = (int64_t)f->file.tensors.size();
    return MI_QMM_OK;
}

int mi_qmm_gguf_tensor(const mi_qmm_gguf *f, int64_t index, const char **name, int *type, int *n_dims,
                       int64_t dims[4], int64_t *offset, int64_t *nbytes) {
    if (!f) return fail(MI_QMM_ERR_INVALID, "gguf is NULL");
    if (index < 0 || index >= (int64_t)f->file.tensors.size())
        return fail(MI_QMM_ERR_INVALID, "tensor index %lld outside 0..%zu", (long long)index, f->file.tensors.size());
    const GgufTensor &t = f->file.tensors[index];
    if (name) *name = t.name.c_str();
    if (type) *type = (int)t.type;
    if (n_dims) *n_dims = (int)t.n_dims;
    if (dims)
        for (int i = 0; i < 4; i++) dims[i] = (int64_t)t.dims[i];
    if (offset) *offset = (int64_t)t.offset;
    if (nbytes) *nbytes = t.nbytes;
    return MI_QMM_OK;
}

int64_t mi_qmm_gguf_find_tensor(const mi_qmm_gguf *f, const char *name) {
    return f && name ? f->file.find_tensor(name) : -1;
}

const void *mi_qmm_gguf_tensor_data(const mi_qmm_gguf *f, int64_t index) {
    if (!f || index < 0 || index >= (int64_t)f->file.tensors.size()) return nullptr;
    return f->file.tensor_data(f->file.tensors[index]);
}

int64_t mi_qmm_gguf_find_kv(const mi_qmm_gguf *f, const char *key) { return f && key ? f->file.find_kv(key) : -1; }

int mi_qmm_gguf_kv(const mi_qmm_gguf *f, int64_t index, const char **key, int *type, int *elem_type, int64_t *count) {
    if (!f) return fail(MI_QMM_ERR_INVALID, "gguf is NULL");
    if (index < 0 || index >= (int64_t)f->file.kvs.size())
        return fail(MI_QMM_ERR_INVALID, "key-value index %lld outside 0..%zu", (long long)index, f->file.kvs.size());
    const GgufKV &kv = f->file.kvs[index];
    if (key) *key = kv.key.c_str();
    if (type) *type = (int)kv.value.type;
    if (elem_type) *elem_type = kv.value.type == GGUF_ARRAY ? (int)kv.value.elem_type : -1;
    if (count) *count = kv.value.type == GGUF_ARRAY ? (int64_t)kv.value.count : 0;
    return MI_QMM_OK;
}

}  // extern "C"

namespace {

// the scalar a (key-value index, element) pair denotes; rc != 0 with the error set if there is none
int kv_scalar(const mi_qmm_gguf *f, int64_t index, int64_t elem, GgufValue &out) {
    if (!f) return fail(MI_QMM_ERR_INVALID, "gguf is NULL");
    if (index < 0 || index >= (int64_t)f->file.kvs.size())
        return fail(MI_QMM_ERR_INVALID, "key-value index %lld outside 0..%zu", (long long)index, f->file.kvs.size());
    const GgufValue &v = f->file.kvs[index].value;
    if (elem < 0) {
        out = v;
        if (v.type == GGUF_ARRAY) out.type = 0xffffffffu;  // an array is no scalar: every accessor yields its zero
        return MI_QMM_OK;
    }
    if (v.type != GGUF_ARRAY || (uint64_t)elem >= v.count)
        return fail(MI_QMM_ERR_INVALID, "element %lld outside the value (array length %llu)", (long long)elem,
                    (unsigned long long)(v.type == GGUF_ARRAY ? v.count : 0));
    out = GgufFile::array_elem(v, (uint64_t)elem);
    return MI_QMM_OK;
}

}  // namespace

extern "C" {

int mi_qmm_gguf_kv_int(const mi_qmm_gguf *f, int64_t index, int64_t elem, int64_t *out) {
    GgufValue v;
    int rc = kv_scalar(f, index, elem, v);
    if (rc) return rc;
    if (out) *out = GgufFile::as_int(v);
    return MI_QMM_OK;
}

int mi_qmm_gguf_kv_uint(const mi_qmm_gguf *f, int64_t index, int64_t elem, uint64_t *out) {
    GgufValue v;
    int rc = kv_scalar(f, index, elem, v);
    if (rc) return rc;
    if (out) *out = GgufFile::as_uint(v);
    return MI_QMM_OK;
}

int mi_qmm_gguf_kv_float(const mi_qmm_gguf *f, int64_t index, int64_t elem, double *out) {
    GgufValue v;
    int rc = kv_scalar(f, index, elem, v);
    if (rc) return rc;
    if (out) *out = GgufFile::as_float(v);
    return MI_QMM_OK;
}

int mi_qmm_gguf_kv_bool(const mi_qmm_gguf *f, int64_t index, int64_t elem, int *out) {
    GgufValue v;
    int rc = kv_scalar(f, index, elem, v);
    if (rc) return rc;
    if (out) *out = GgufFile::as_bool(v) ? 1 : 0;
    return MI_QMM_OK;
}

int mi_qmm_gguf_kv_string(const mi_qmm_gguf *f, int64_t index, int64_t elem, const char **str, int64_t *len) {
    GgufValue v;
    int rc = kv_scalar(f, index, elem, v);
    if (rc) return rc;
    const bool is_str = v.type == GGUF_STRING;
    if (str) *str = is_str ? reinterpret_cast<const char *>(v.data) : "";
    if (len) *len = is_str ? (int64_t)v.len : 0;
    return MI_QMM_OK;
}

int mi_qmm_gguf_upload(mi_qmm_ctx *ctx, const mi_qmm_gguf *f, int64_t index, mi_qmm_weight **out) {
    if (!out) return fail(MI_QMM_ERR_INVALID, "out is NULL");
    *out = nullptr;
    if (!f) return fail(MI_QMM_ERR_INVALID, "gguf is NULL");
    if (index < 0 || index >= (int64_t)f->file.tensors.size())
        return fail(MI_QMM_ERR_INVALID, "tensor index %lld outside 0..%zu", (long long)index, f->file.tensors.size());
    const GgufTensor &t = f->file.tensors[index];
    if (t.n_dims != 2 && t.n_dims != 3)
        return fail(MI_QMM_ERR_UNSUPPORTED,
                    "tensor \"%s\" has %u dimensions: Mulmat takes 2-D weights, MulmatID 3-D expert stacks",
                    t.name.c_str(), t.n_dims);
    // an expert stack [K, M, E] is E matrices of M rows one after the other: the same bytes as [K, M*E]
    const int64_t m = (int64_t)t.dims[1] * (t.n_dims == 3 ? (int64_t)t.dims[2] : 1);
    return mi_qmm_weight_upload(ctx, (int)t.type, f->file.tensor_data(t), (int64_t)t.dims[0], m, MI_QMM_HOST, out);
}

}  // extern "C"
