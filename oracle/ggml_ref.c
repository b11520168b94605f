/*
 * CPU oracle for the GGUF block-quantized matmul path  --  TEST INFRASTRUCTURE ONLY.
 * See ggml_ref.h for scope, provenance and the parity status of every function.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math (no FMA contraction: the quantizers are
 * defined by the unfused C expressions below).
 */
#include "ggml_ref.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define QK 32    /* elements per Q4_0 / Q8_0 block   */
#define QKK 256  /* elements per K-quant super-block */

/* ---- block layouts: byte sizes follow /root/reference/fs/ggml/ggml.go:450-473 ------------- */
#pragma pack(push, 1)
typedef struct { uint16_t d; uint8_t qs[QK / 2]; } blk_q4_0;                                /* 2+16      */
typedef struct { uint16_t d; uint8_t qh[4]; uint8_t qs[QK / 2]; } blk_q5_0;                 /* 2+4+16    */
typedef struct { uint16_t d; int8_t qs[QK]; } blk_q8_0;                                     /* 2+32      */
typedef struct { uint8_t e; uint8_t qs[QK / 2]; } blk_mxfp4;                                /* 1+16      */
typedef struct { uint16_t d; uint16_t dmin; uint8_t scales[12]; uint8_t qs[QKK / 2]; } blk_q4_K; /* 2+2+12+128 */
typedef struct { uint16_t d; uint16_t dmin; uint8_t scales[12]; uint8_t qh[QKK / 8]; uint8_t qs[QKK / 2]; } blk_q5_K; /* 2+2+12+32+128 */
typedef struct { uint8_t ql[QKK / 2]; uint8_t qh[QKK / 4]; int8_t scales[QKK / 16]; uint16_t d; } blk_q6_K; /* 128+64+16+2 */
typedef struct { float d; int8_t qs[QKK]; int16_t bsums[QKK / 16]; } blk_q8_K;              /* 4+256+32  */
#pragma pack(pop)

_Static_assert(sizeof(blk_q4_0) == 18, "Q4_0 block is 18 bytes");
_Static_assert(sizeof(blk_q5_0) == 22, "Q5_0 block is 22 bytes");
_Static_assert(sizeof(blk_q8_0) == 34, "Q8_0 block is 34 bytes");
_Static_assert(sizeof(blk_mxfp4) == 17, "MXFP4 block is 17 bytes");
_Static_assert(sizeof(blk_q4_K) == 144, "Q4_K block is 144 bytes");
_Static_assert(sizeof(blk_q5_K) == 176, "Q5_K block is 176 bytes");
_Static_assert(sizeof(blk_q6_K) == 210, "Q6_K block is 210 bytes");
_Static_assert(sizeof(blk_q8_K) == 292, "Q8_K block is 292 bytes");

int64_t ref_block_size(int type) {
    switch (type) {
    case REF_TYPE_F32: case REF_TYPE_F16: case REF_TYPE_BF16: return 1;
    case REF_TYPE_Q4_0: case REF_TYPE_Q5_0: case REF_TYPE_Q8_0: case REF_TYPE_MXFP4: return QK;
    case REF_TYPE_Q4_K: case REF_TYPE_Q5_K: case REF_TYPE_Q6_K: case REF_TYPE_Q8_K: return QKK;
    default: return 0;
    }
}

int64_t ref_type_size(int type) {
    switch (type) {
    case REF_TYPE_F32: return 4;
    case REF_TYPE_F16: case REF_TYPE_BF16: return 2;
    case REF_TYPE_Q4_0: return sizeof(blk_q4_0);
    case REF_TYPE_Q5_0: return sizeof(blk_q5_0);
    case REF_TYPE_Q8_0: return sizeof(blk_q8_0);
    case REF_TYPE_MXFP4: return sizeof(blk_mxfp4);
    case REF_TYPE_Q4_K: return sizeof(blk_q4_K);
    case REF_TYPE_Q5_K: return sizeof(blk_q5_K);
    case REF_TYPE_Q6_K: return sizeof(blk_q6_K);
    case REF_TYPE_Q8_K: return sizeof(blk_q8_K);
    default: return 0;
    }
}

int64_t ref_row_size(int type, int64_t k) {
    int64_t bs = ref_block_size(type);
    if (bs == 0 || k < 0 || k % bs != 0) return -1;
    return k / bs * ref_type_size(type);
}

int ref_vec_dot_type(int wtype) {
    switch (wtype) {
    case REF_TYPE_Q4_0: case REF_TYPE_Q5_0: case REF_TYPE_Q8_0: case REF_TYPE_MXFP4: return REF_TYPE_Q8_0;
    case REF_TYPE_Q4_K: case REF_TYPE_Q5_K: case REF_TYPE_Q6_K: return REF_TYPE_Q8_K;
    /* the unquantized weight types are multiplied in their own type: the activations are converted to it */
    case REF_TYPE_F32: case REF_TYPE_F16: case REF_TYPE_BF16: return wtype;
    default: return -1;
    }
}

static float bf16_widen(uint16_t h) {
    const uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* ---- IEEE binary16 <-> binary32, round to nearest even, subnormals kept ------------------- */
uint16_t ref_fp32_to_fp16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t mag = u & 0x7fffffffu;
    if (mag >= 0x7f800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | (mag > 0x7f800000u ? 0x0200u | ((mag >> 13) & 0x3ffu) : 0));
    if (mag >= 0x477ff000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    if (mag < 0x33000001u) /* < 2^-25 (or exactly 2^-25, tie to even 0) */
        return (uint16_t)sign;
    int32_t e = (int32_t)(mag >> 23) - 127;
    uint32_t man = (mag & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int shift;                                      /* bits dropped from the significand */
    uint32_t base;
    if (e < -14) { /* subnormal half */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7fffffu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) q++;
    return (uint16_t)(sign | (base + q)); /* carry into the exponent is the correct result */
}

float ref_fp16_to_fp32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    uint32_t u;
    if (e == 0) {
        if (man == 0) {
            u = sign;
        } else { /* subnormal: value = man * 2^-24 */
            float v = (float)man * 0x1p-24f;
            memcpy(&u, &v, 4);
            u |= sign;
        }
    } else if (e == 31) {
        u = sign | 0x7f800000u | (man << 13);
    } else {
        u = sign | ((e + 112) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even of an fp32 value via the 1.5*2^23 magic add; valid for |v| <= 2^22 */
static inline int nearest_int(float fval) {
    float val = fval + 12582912.f;
    int i;
    memcpy(&i, &val, sizeof(int));
    return (i & 0x007fffff) - 0x00400000;
}

#define MAXI(a, b) ((a) > (b) ? (a) : (b))
#define MINI(a, b) ((a) < (b) ? (a) : (b))

/* ---- activation quantizers ----------------------------------------------------------------- */
void ref_quantize_row_q8_0(const float *x, void *vy, int64_t k) {
    blk_q8_0 *y = (blk_q8_0 *)vy;
    const int64_t nb = k / QK;
    for (int64_t i = 0; i < nb; i++) {
        float amax = 0.0f;
        for (int j = 0; j < QK; j++) {
            const float v = fabsf(x[i * QK + j]);
            if (v > amax) amax = v;
        }
        const float d = amax / 127.0f;
        const float id = d ? 1.0f / d : 0.0f;
        y[i].d = ref_fp32_to_fp16(d);
        for (int j = 0; j < QK; j++) {
            const float x0 = x[i * QK + j] * id;
            y[i].qs[j] = (int8_t)roundf(x0);
        }
    }
}

void ref_quantize_row_q8_K(const float *x, void *vy, int64_t k) {
    blk_q8_K *y = (blk_q8_K *)vy;
    const int64_t nb = k / QKK;
    for (int64_t i = 0; i < nb; i++) {
        float max = 0, amax = 0;
        for (int j = 0; j < QKK; j++) {
            const float ax = fabsf(x[j]);
            if (ax > amax) { amax = ax; max = x[j]; }
        }
        if (!amax) {
            /* upstream leaves bsums untouched here; the canonical form used by this build
             * writes zeros so the block is fully defined */
            memset(&y[i], 0, sizeof(blk_q8_K));
            x += QKK;
            continue;
        }
        const float iscale = -127.f / max;
        for (int j = 0; j < QKK; j++) {
            int v = nearest_int(iscale * x[j]);
            y[i].qs[j] = (int8_t)MINI(127, v);
        }
        for (int j = 0; j < QKK / 16; j++) {
            int sum = 0;
            for (int ii = 0; ii < 16; ii++) sum += y[i].qs[j * 16 + ii];
            y[i].bsums[j] = (int16_t)sum;
        }
        y[i].d = 1 / iscale;
        x += QKK;
    }
}

/* ---- weight encoders ------------------------------------------------------------------------ */
void ref_quantize_row_q4_0(const float *x, void *vy, int64_t k) {
    blk_q4_0 *y = (blk_q4_0 *)vy;
    const int64_t nb = k / QK;
    for (int64_t i = 0; i < nb; i++) {
        float amax = 0.0f, max = 0.0f;
        for (int j = 0; j < QK; j++) {
            const float v = x[i * QK + j];
            if (amax < fabsf(v)) { amax = fabsf(v); max = v; }
        }
        const float d = max / -8;
        const float id = d ? 1.0f / d : 0.0f;
        y[i].d = ref_fp32_to_fp16(d);
        for (int j = 0; j < QK / 2; j++) {
            const float x0 = x[i * QK + 0 + j] * id;
            const float x1 = x[i * QK + QK / 2 + j] * id;
            const uint8_t xi0 = (uint8_t)MINI(15, (int8_t)(x0 + 8.5f));
            const uint8_t xi1 = (uint8_t)MINI(15, (int8_t)(x1 + 8.5f));
            y[i].qs[j] = (uint8_t)(xi0 | (xi1 << 4));
        }
    }
}

/* weighted (scale, min) search for an asymmetric nmax-level grid over n values */
static float make_qkx2_quants(int n, int nmax, const float *x, const float *weights, uint8_t *L,
                              float *the_min, uint8_t *Laux, float rmin, float rdelta, int nstep) {
    float min = x[0], max = x[0];
    float sum_w = weights[0];
    float sum_x = sum_w * x[0];
    for (int i = 1; i < n; i++) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
        const float w = weights[i];
        sum_w += w;
        sum_x += w * x[i];
    }
    if (min > 0) min = 0;
    if (max == min) {
        for (int i = 0; i < n; i++) L[i] = 0;
        *the_min = -min;
        return 0.f;
    }
    float iscale = nmax / (max - min);
    float scale = 1 / iscale;
    float best = 0;
    for (int i = 0; i < n; i++) {
        int l = nearest_int(iscale * (x[i] - min));
        L[i] = (uint8_t)MAXI(0, MINI(nmax, l));
        float diff = scale * L[i] + min - x[i];
        diff = diff * diff;
        best += weights[i] * diff;
    }
    if (nstep < 1) {
        *the_min = -min;
        return scale;
    }
    for (int is = 0; is <= nstep; is++) {
        iscale = (rmin + rdelta * is + nmax) / (max - min);
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        for (int i = 0; i < n; i++) {
            int l = nearest_int(iscale * (x[i] - min));
            l = MAXI(0, MINI(nmax, l));
            Laux[i] = (uint8_t)l;
            const float w = weights[i];
            sum_l += w * l;
            sum_l2 += w * l * l;
            sum_xl += w * l * x[i];
        }
        const float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0) {
                this_min = 0;
                this_scale = sum_xl / sum_l2;
            }
            float err = 0;
            for (int i = 0; i < n; i++) {
                float diff = this_scale * Laux[i] + this_min - x[i];
                diff = diff * diff;
                err += weights[i] * diff;
            }
            if (err < best) {
                for (int i = 0; i < n; i++) L[i] = Laux[i];
                best = err;
                scale = this_scale;
                min = this_min;
            }
        }
    }
    *the_min = -min;
    return scale;
}

/* the search on its own, for tests of what it returns: levels[n], *neg_min = -min, returns the scale */
float ref_qkx2_search(int n, int nmax, const float *x, const float *weights, uint8_t *levels, float *neg_min,
                      float rmin, float rdelta, int nstep) {
    uint8_t laux[QKK];
    if (n < 1 || n > QKK) return -1.f;
    return make_qkx2_quants(n, nmax, x, weights, levels, neg_min, laux, rmin, rdelta, nstep);
}

void ref_get_scale_min_k4(int j, const uint8_t *q, uint8_t *d, uint8_t *m) {
    if (j < 4) {
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j - 0] >> 6) << 4));
    }
}

void ref_unpack_scales_kmask(const uint8_t *s12, uint8_t sc[8], uint8_t m[8]) {
    static const uint32_t kmask1 = 0x3f3f3f3f, kmask2 = 0x0f0f0f0f, kmask3 = 0x03030303;
    uint32_t utmp[4];
    memcpy(utmp, s12, 12);
    utmp[3] = ((utmp[2] >> 4) & kmask2) | (((utmp[1] >> 6) & kmask3) << 4);
    const uint32_t uaux = utmp[1] & kmask1;
    utmp[1] = (utmp[2] & kmask2) | (((utmp[0] >> 6) & kmask3) << 4);
    utmp[2] = uaux;
    utmp[0] &= kmask1;
    memcpy(sc, &utmp[0], 8);
    memcpy(m, &utmp[2], 8);
}

void ref_quantize_row_q4_K(const float *x, void *vy, int64_t k) {
    blk_q4_K *y = (blk_q4_K *)vy;
    const int64_t nb = k / QKK;
    uint8_t L[QKK], Laux[32];
    float weights[32], mins[QKK / 32], scales[QKK / 32];
    for (int64_t i = 0; i < nb; i++) {
        float max_scale = 0, max_min = 0;
        for (int j = 0; j < QKK / 32; j++) {
            float sum_x2 = 0;
            for (int l = 0; l < 32; l++) sum_x2 += x[32 * j + l] * x[32 * j + l];
            const float av_x = sqrtf(sum_x2 / 32);
            for (int l = 0; l < 32; l++) weights[l] = av_x + fabsf(x[32 * j + l]);
            scales[j] = make_qkx2_quants(32, 15, x + 32 * j, weights, L + 32 * j, &mins[j], Laux,
                                         -1.f, 0.1f, 20);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
        const float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
        memset(y[i].scales, 0, 12);
        for (int j = 0; j < QKK / 32; j++) {
            uint8_t ls = (uint8_t)nearest_int(inv_scale * scales[j]);
            uint8_t lm = (uint8_t)nearest_int(inv_min * mins[j]);
            ls = MINI(63, ls);
            lm = MINI(63, lm);
            if (j < 4) {
                y[i].scales[j] |= ls;     /* low 6 bits; the top 2 are filled by j+4 below */
                y[i].scales[j + 4] |= lm;
            } else {
                y[i].scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                y[i].scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                y[i].scales[j - 0] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        y[i].d = ref_fp32_to_fp16(max_scale / 63.f);
        y[i].dmin = ref_fp32_to_fp16(max_min / 63.f);
        for (int j = 0; j < QKK / 32; j++) {
            uint8_t sc, m;
            ref_get_scale_min_k4(j, y[i].scales, &sc, &m);
            const float d = ref_fp16_to_fp32(y[i].d) * sc;
            if (!d) continue;
            const float dm = ref_fp16_to_fp32(y[i].dmin) * m;
            for (int ii = 0; ii < 32; ii++) {
                int l = nearest_int((x[32 * j + ii] + dm) / d);
                L[32 * j + ii] = (uint8_t)MAXI(0, MINI(15, l));
            }
        }
        uint8_t *q = y[i].qs;
        for (int j = 0; j < QKK; j += 64) {
            for (int l = 0; l < 32; l++) q[l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
            q += 32;
        }
        x += QKK;
    }
}

#define GROUP_MAX_EPS 1e-15f

/* symmetric grid search, weights x^2 (the rmse_type == 1 variant used by Q6_K) */
static float make_qx_quants(int n, int nmax, const float *x, int8_t *L) {
    float max = 0, amax = 0;
    for (int i = 0; i < n; i++) {
        const float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; max = x[i]; }
    }
    if (amax < GROUP_MAX_EPS) {
        for (int i = 0; i < n; i++) L[i] = 0;
        return 0.f;
    }
    float iscale = -nmax / max;
    float sumlx = 0, suml2 = 0;
    for (int i = 0; i < n; i++) {
        int l = nearest_int(iscale * x[i]);
        l = MAXI(-nmax, MINI(nmax - 1, l));
        L[i] = (int8_t)(l + nmax);
        const float w = x[i] * x[i];
        sumlx += w * x[i] * l;
        suml2 += w * l * l;
    }
    float scale = suml2 ? sumlx / suml2 : 0.0f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; is++) {
        if (is == 0) continue;
        iscale = -(nmax + 0.1f * is) / max;
        sumlx = suml2 = 0;
        for (int i = 0; i < n; i++) {
            int l = nearest_int(iscale * x[i]);
            l = MAXI(-nmax, MINI(nmax - 1, l));
            const float w = x[i] * x[i];
            sumlx += w * x[i] * l;
            suml2 += w * l * l;
        }
        if (suml2 > 0 && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; i++) {
                int l = nearest_int(iscale * x[i]);
                L[i] = (int8_t)(nmax + MAXI(-nmax, MINI(nmax - 1, l)));
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

/* the search on its own, for tests of what it returns: levels[n] hold l + nmax, returns the scale */
float ref_qx_search(int n, int nmax, const float *x, int8_t *levels) {
    return make_qx_quants(n, nmax, x, levels);
}

void ref_quantize_row_q6_K(const float *x, void *vy, int64_t k) {
    blk_q6_K *y = (blk_q6_K *)vy;
    const int64_t nb = k / QKK;
    int8_t L[QKK];
    float scales[QKK / 16];
    for (int64_t i = 0; i < nb; i++) {
        float max_scale = 0, max_abs_scale = 0;
        for (int ib = 0; ib < QKK / 16; ib++) {
            const float scale = make_qx_quants(16, 32, x + 16 * ib, L + 16 * ib);
            scales[ib] = scale;
            const float abs_scale = fabsf(scale);
            if (abs_scale > max_abs_scale) { max_abs_scale = abs_scale; max_scale = scale; }
        }
        if (max_abs_scale < GROUP_MAX_EPS) {
            memset(&y[i], 0, sizeof(blk_q6_K));
            x += QKK;
            continue;
        }
        const float iscale = -128.f / max_scale;
        y[i].d = ref_fp32_to_fp16(1 / iscale);
        for (int ib = 0; ib < QKK / 16; ib++)
            y[i].scales[ib] = (int8_t)MINI(127, nearest_int(iscale * scales[ib]));
        for (int j = 0; j < QKK / 16; j++) {
            const float d = ref_fp16_to_fp32(y[i].d) * y[i].scales[j];
            if (!d) continue;
            for (int ii = 0; ii < 16; ii++) {
                int l = nearest_int(x[16 * j + ii] / d);
                l = MAXI(-32, MINI(31, l));
                L[16 * j + ii] = (int8_t)(l + 32);
            }
        }
        uint8_t *ql = y[i].ql, *qh = y[i].qh;
        for (int j = 0; j < QKK; j += 128) {
            for (int l = 0; l < 32; l++) {
                const uint8_t q1 = L[j + l + 0] & 0xF, q2 = L[j + l + 32] & 0xF;
                const uint8_t q3 = L[j + l + 64] & 0xF, q4 = L[j + l + 96] & 0xF;
                ql[l + 0] = (uint8_t)(q1 | (q3 << 4));
                ql[l + 32] = (uint8_t)(q2 | (q4 << 4));
                qh[l] = (uint8_t)((L[j + l] >> 4) | ((L[j + l + 32] >> 4) << 2) |
                                  ((L[j + l + 64] >> 4) << 4) | ((L[j + l + 96] >> 4) << 6));
            }
            ql += 64;
            qh += 32;
        }
        x += QKK;
    }
}

/* ---- dequantizers ---------------------------------------------------------------------------- */
static void dequant_q4_0(const blk_q4_0 *x, float *y, int64_t k) {
    for (int64_t i = 0; i < k / QK; i++) {
        const float d = ref_fp16_to_fp32(x[i].d);
        for (int j = 0; j < QK / 2; j++) {
            y[i * QK + j] = ((x[i].qs[j] & 0x0F) - 8) * d;
            y[i * QK + j + QK / 2] = ((x[i].qs[j] >> 4) - 8) * d;
        }
    }
}

static void dequant_q8_0(const blk_q8_0 *x, float *y, int64_t k) {
    for (int64_t i = 0; i < k / QK; i++) {
        const float d = ref_fp16_to_fp32(x[i].d);
        for (int j = 0; j < QK; j++) y[i * QK + j] = x[i].qs[j] * d;
    }
}

static void dequant_q4_K(const blk_q4_K *x, float *y, int64_t k) {
    for (int64_t i = 0; i < k / QKK; i++) {
        const uint8_t *q = x[i].qs;
        const float d = ref_fp16_to_fp32(x[i].d), min = ref_fp16_to_fp32(x[i].dmin);
        int is = 0;
        for (int j = 0; j < QKK; j += 64) {
            uint8_t sc, m;
            ref_get_scale_min_k4(is + 0, x[i].scales, &sc, &m);
            const float d1 = d * sc, m1 = min * m;
            ref_get_scale_min_k4(is + 1, x[i].scales, &sc, &m);
            const float d2 = d * sc, m2 = min * m;
            for (int l = 0; l < 32; l++) *y++ = d1 * (q[l] & 0xF) - m1;
            for (int l = 0; l < 32; l++) *y++ = d2 * (q[l] >> 4) - m2;
            q += 32;
            is += 2;
        }
    }
}

/* Q5_0: the Q4_0 layout with a fifth bit per weight in a 32-bit word: bit j of qh belongs to element j; w = d (q - 16) */
static void dequant_q5_0(const blk_q5_0 *x, float *y, int64_t k) {
    for (int64_t i = 0; i < k / QK; i++) {
        const float d = ref_fp16_to_fp32(x[i].d);
        uint32_t qh;
        memcpy(&qh, x[i].qh, 4);
        for (int j = 0; j < QK / 2; j++) {
            const uint8_t xh_0 = (uint8_t)(((qh >> (j + 0)) << 4) & 0x10);
            const uint8_t xh_1 = (uint8_t)((qh >> (j + 12)) & 0x10);
            y[i * QK + j] = (float)(((x[i].qs[j] & 0x0F) | xh_0) - 16) * d;
            y[i * QK + j + QK / 2] = (float)(((x[i].qs[j] >> 4) | xh_1) - 16) * d;
        }
    }
}

/* MXFP4 (OCP microscaling: 32 four-bit floats E2M1 under one power-of-two scale E8M0; the block layout is the one
 * /root/reference/convert/convert_gptoss.go:216-238 writes: the scale byte, then 16 bytes whose low nibbles are elements
 * 0..15 and whose high nibbles are elements 16..31).  ggml keeps the E2M1 values doubled as integers and halves the
 * scale instead: element = kvalue[nibble] * 2^(e - 128). */
static const int8_t mxfp4_kvalues[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};

float ref_e8m0_to_fp32_half(uint8_t e) {
    uint32_t bits = e < 2 ? 0x00200000u << e : (uint32_t)(e - 1) << 23;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static void dequant_mxfp4(const blk_mxfp4 *x, float *y, int64_t k) {
    for (int64_t i = 0; i < k / QK; i++) {
        const float d = ref_e8m0_to_fp32_half(x[i].e);
        for (int j = 0; j < QK / 2; j++) {
            y[i * QK + j] = d * mxfp4_kvalues[x[i].qs[j] & 0x0F];
            y[i * QK + j + QK / 2] = d * mxfp4_kvalues[x[i].qs[j] >> 4];
        }
    }
}

/* Q5_K: the Q4_K layout with a fifth bit per weight.  Bit j of qh[l] belongs to element l of sub-block j (the low
 * nibbles of chunk c are sub-block 2c, the high nibbles sub-block 2c + 1); w = d * sc * (nibble + 16 * bit) - dmin * m. */
static void dequant_q5_K(const blk_q5_K *x, float *y, int64_t k) {
    for (int64_t i = 0; i < k / QKK; i++) {
        const uint8_t *ql = x[i].qs, *qh = x[i].qh;
        const float d = ref_fp16_to_fp32(x[i].d), min = ref_fp16_to_fp32(x[i].dmin);
        int is = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int j = 0; j < QKK; j += 64) {
            uint8_t sc, m;
            ref_get_scale_min_k4(is + 0, x[i].scales, &sc, &m);
            const float d1 = d * sc, m1 = min * m;
            ref_get_scale_min_k4(is + 1, x[i].scales, &sc, &m);
            const float d2 = d * sc, m2 = min * m;
            for (int l = 0; l < 32; l++) *y++ = d1 * ((ql[l] & 0xF) + (qh[l] & u1 ? 16 : 0)) - m1;
            for (int l = 0; l < 32; l++) *y++ = d2 * ((ql[l] >> 4) + (qh[l] & u2 ? 16 : 0)) - m2;
            ql += 32;
            is += 2;
            u1 <<= 2;
            u2 <<= 2;
        }
    }
}

static void dequant_q6_K(const blk_q6_K *x, float *y, int64_t k) {
    for (int64_t i = 0; i < k / QKK; i++) {
        const float d = ref_fp16_to_fp32(x[i].d);
        const uint8_t *ql = x[i].ql, *qh = x[i].qh;
        const int8_t *sc = x[i].scales;
        for (int n = 0; n < QKK; n += 128) {
            for (int l = 0; l < 32; l++) {
                const int is = l / 16;
                const int8_t q1 = (int8_t)((ql[l + 0] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                const int8_t q2 = (int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                const int8_t q3 = (int8_t)((ql[l + 0] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                const int8_t q4 = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                y[l + 0] = d * sc[is + 0] * q1;
                y[l + 32] = d * sc[is + 2] * q2;
                y[l + 64] = d * sc[is + 4] * q3;
                y[l + 96] = d * sc[is + 6] * q4;
            }
            y += 128;
            ql += 64;
            qh += 32;
            sc += 8;
        }
    }
}

static void dequant_q8_K(const blk_q8_K *x, float *y, int64_t k) {
    for (int64_t i = 0; i < k / QKK; i++)
        for (int j = 0; j < QKK; j++) *y++ = x[i].d * x[i].qs[j];
}

int ref_dequantize_row(int type, const void *x, float *y, int64_t k) {
    if (ref_row_size(type, k) < 0) return -1;
    switch (type) {
    case REF_TYPE_Q4_0: dequant_q4_0((const blk_q4_0 *)x, y, k); return 0;
    case REF_TYPE_Q5_0: dequant_q5_0((const blk_q5_0 *)x, y, k); return 0;
    case REF_TYPE_Q8_0: dequant_q8_0((const blk_q8_0 *)x, y, k); return 0;
    case REF_TYPE_MXFP4: dequant_mxfp4((const blk_mxfp4 *)x, y, k); return 0;
    case REF_TYPE_Q4_K: dequant_q4_K((const blk_q4_K *)x, y, k); return 0;
    case REF_TYPE_Q5_K: dequant_q5_K((const blk_q5_K *)x, y, k); return 0;
    case REF_TYPE_Q6_K: dequant_q6_K((const blk_q6_K *)x, y, k); return 0;
    case REF_TYPE_Q8_K: dequant_q8_K((const blk_q8_K *)x, y, k); return 0;
    case REF_TYPE_F32: memcpy(y, x, (size_t)k * 4); return 0;
    case REF_TYPE_F16: for (int64_t i = 0; i < k; i++) y[i] = ref_fp16_to_fp32(((const uint16_t *)x)[i]); return 0;
    case REF_TYPE_BF16: for (int64_t i = 0; i < k; i++) y[i] = bf16_widen(((const uint16_t *)x)[i]); return 0;
    default: return -1;
    }
}

/* ---- dot products (generic scalar path; integer parts exact, fp32 order as written) -------- */
float ref_vec_dot_q4_0_q8_0(int64_t n, const void *vx, const void *vy) {
    const blk_q4_0 *x = (const blk_q4_0 *)vx;
    const blk_q8_0 *y = (const blk_q8_0 *)vy;
    float sumf = 0;
    for (int64_t ib = 0; ib < n / QK; ib++) {
        int sumi0 = 0, sumi1 = 0;
        for (int j = 0; j < QK / 2; j++) {
            const int v0 = (x[ib].qs[j] & 0x0F) - 8;
            const int v1 = (x[ib].qs[j] >> 4) - 8;
            sumi0 += v0 * y[ib].qs[j];
            sumi1 += v1 * y[ib].qs[j + QK / 2];
        }
        const int sumi = sumi0 + sumi1;
        sumf += sumi * ref_fp16_to_fp32(x[ib].d) * ref_fp16_to_fp32(y[ib].d);
    }
    return sumf;
}

float ref_vec_dot_q8_0_q8_0(int64_t n, const void *vx, const void *vy) {
    const blk_q8_0 *x = (const blk_q8_0 *)vx;
    const blk_q8_0 *y = (const blk_q8_0 *)vy;
    float sumf = 0;
    for (int64_t ib = 0; ib < n / QK; ib++) {
        int sumi = 0;
        for (int j = 0; j < QK; j++) sumi += x[ib].qs[j] * y[ib].qs[j];
        sumf += sumi * (ref_fp16_to_fp32(x[ib].d) * ref_fp16_to_fp32(y[ib].d));
    }
    return sumf;
}

/* ggml_vec_dot_q5_0_q8_0, generic path */
float ref_vec_dot_q5_0_q8_0(int64_t n, const void *vx, const void *vy) {
    const blk_q5_0 *x = (const blk_q5_0 *)vx;
    const blk_q8_0 *y = (const blk_q8_0 *)vy;
    float sumf = 0;
    for (int64_t ib = 0; ib < n / QK; ib++) {
        uint32_t qh;
        memcpy(&qh, x[ib].qh, 4);
        int sumi0 = 0, sumi1 = 0;
        for (int j = 0; j < QK / 2; j++) {
            const uint8_t xh_0 = (uint8_t)(((qh & (1u << (j + 0))) >> (j + 0)) << 4);
            const uint8_t xh_1 = (uint8_t)((qh & (1u << (j + 16))) >> (j + 12));
            const int32_t x0 = (int8_t)(((x[ib].qs[j] & 0x0F) | xh_0) - 16);
            const int32_t x1 = (int8_t)(((x[ib].qs[j] >> 4) | xh_1) - 16);
            sumi0 += x0 * y[ib].qs[j];
            sumi1 += x1 * y[ib].qs[j + QK / 2];
        }
        const int sumi = sumi0 + sumi1;
        sumf += (ref_fp16_to_fp32(x[ib].d) * ref_fp16_to_fp32(y[ib].d)) * sumi;
    }
    return sumf;
}

/* ggml_vec_dot_mxfp4_q8_0, generic path */
float ref_vec_dot_mxfp4_q8_0(int64_t n, const void *vx, const void *vy) {
    const blk_mxfp4 *x = (const blk_mxfp4 *)vx;
    const blk_q8_0 *y = (const blk_q8_0 *)vy;
    float sumf = 0;
    for (int64_t ib = 0; ib < n / QK; ib++) {
        const float d = ref_fp16_to_fp32(y[ib].d) * ref_e8m0_to_fp32_half(x[ib].e);
        int sumi1 = 0, sumi2 = 0;
        for (int j = 0; j < QK / 2; j++) {
            sumi1 += y[ib].qs[j] * mxfp4_kvalues[x[ib].qs[j] & 0x0F];
            sumi2 += y[ib].qs[j + QK / 2] * mxfp4_kvalues[x[ib].qs[j] >> 4];
        }
        sumf += d * (sumi1 + sumi2);
    }
    return sumf;
}

float ref_vec_dot_q4_K_q8_K(int64_t n, const void *vx, const void *vy) {
    const blk_q4_K *x = (const blk_q4_K *)vx;
    const blk_q8_K *y = (const blk_q8_K *)vy;
    int8_t aux8[QKK];
    int16_t aux16[8];
    int32_t aux32[8];
    float sums[8];
    uint8_t scales[8], mins[8];
    memset(sums, 0, sizeof(sums));
    float sumf = 0;
    for (int64_t i = 0; i < n / QKK; i++) {
        const uint8_t *q4 = x[i].qs;
        const int8_t *q8 = y[i].qs;
        memset(aux32, 0, sizeof(aux32));
        int8_t *a = aux8;
        for (int j = 0; j < QKK / 64; j++) {
            for (int l = 0; l < 32; l++) a[l] = (int8_t)(q4[l] & 0xF);
            a += 32;
            for (int l = 0; l < 32; l++) a[l] = (int8_t)(q4[l] >> 4);
            a += 32;
            q4 += 32;
        }
        ref_unpack_scales_kmask(x[i].scales, scales, mins);
        int sumi = 0;
        for (int j = 0; j < QKK / 16; j++) sumi += y[i].bsums[j] * mins[j / 2];
        a = aux8;
        for (int j = 0; j < QKK / 32; j++) {
            const int32_t scale = scales[j];
            for (int rep = 0; rep < 4; rep++) {
                for (int l = 0; l < 8; l++) aux16[l] = (int16_t)(q8[l] * a[l]);
                for (int l = 0; l < 8; l++) aux32[l] += scale * aux16[l];
                q8 += 8;
                a += 8;
            }
        }
        const float d = ref_fp16_to_fp32(x[i].d) * y[i].d;
        for (int l = 0; l < 8; l++) sums[l] += d * aux32[l];
        const float dmin = ref_fp16_to_fp32(x[i].dmin) * y[i].d;
        sumf -= dmin * sumi;
    }
    for (int l = 0; l < 8; l++) sumf += sums[l];
    return sumf;
}

/* ggml_vec_dot_q5_K_q8_K, generic path: the 5-bit values in element order, then as for Q4_K */
float ref_vec_dot_q5_K_q8_K(int64_t n, const void *vx, const void *vy) {
    const blk_q5_K *x = (const blk_q5_K *)vx;
    const blk_q8_K *y = (const blk_q8_K *)vy;
    int8_t aux8[QKK];
    int16_t aux16[8];
    int32_t aux32[8];
    float sums[8];
    uint8_t scales[8], mins[8];
    memset(sums, 0, sizeof(sums));
    float sumf = 0;
    for (int64_t i = 0; i < n / QKK; i++) {
        const uint8_t *q4 = x[i].qs, *hm = x[i].qh;
        const int8_t *q8 = y[i].qs;
        memset(aux32, 0, sizeof(aux32));
        int8_t *a = aux8;
        uint8_t m = 1;
        for (int j = 0; j < QKK / 64; j++) {
            for (int l = 0; l < 32; l++) a[l] = (int8_t)(q4[l] & 0xF);
            for (int l = 0; l < 32; l++) a[l] += (hm[l] & m ? 16 : 0);
            a += 32;
            m <<= 1;
            for (int l = 0; l < 32; l++) a[l] = (int8_t)(q4[l] >> 4);
            for (int l = 0; l < 32; l++) a[l] += (hm[l] & m ? 16 : 0);
            a += 32;
            m <<= 1;
            q4 += 32;
        }
        ref_unpack_scales_kmask(x[i].scales, scales, mins);
        int sumi = 0;
        for (int j = 0; j < QKK / 16; j++) sumi += y[i].bsums[j] * mins[j / 2];
        a = aux8;
        for (int j = 0; j < QKK / 32; j++) {
            const int32_t scale = scales[j];
            for (int rep = 0; rep < 4; rep++) {
                for (int l = 0; l < 8; l++) aux16[l] = (int16_t)(q8[l] * a[l]);
                for (int l = 0; l < 8; l++) aux32[l] += scale * aux16[l];
                q8 += 8;
                a += 8;
            }
        }
        const float d = ref_fp16_to_fp32(x[i].d) * y[i].d;
        for (int l = 0; l < 8; l++) sums[l] += d * aux32[l];
        const float dmin = ref_fp16_to_fp32(x[i].dmin) * y[i].d;
        sumf -= dmin * sumi;
    }
    for (int l = 0; l < 8; l++) sumf += sums[l];
    return sumf;
}

float ref_vec_dot_q6_K_q8_K(int64_t n, const void *vx, const void *vy) {
    const blk_q6_K *x = (const blk_q6_K *)vx;
    const blk_q8_K *y = (const blk_q8_K *)vy;
    int8_t aux8[QKK];
    int16_t aux16[8];
    int32_t aux32[8];
    float sums[8];
    memset(sums, 0, sizeof(sums));
    float sumf = 0;
    for (int64_t i = 0; i < n / QKK; i++) {
        const uint8_t *q4 = x[i].ql, *qh = x[i].qh;
        const int8_t *q8 = y[i].qs;
        memset(aux32, 0, sizeof(aux32));
        int8_t *a = aux8;
        for (int j = 0; j < QKK; j += 128) {
            for (int l = 0; l < 32; l++) {
                a[l + 0] = (int8_t)((q4[l + 0] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                a[l + 32] = (int8_t)((q4[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                a[l + 64] = (int8_t)((q4[l + 0] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                a[l + 96] = (int8_t)((q4[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
            }
            a += 128;
            q4 += 64;
            qh += 32;
        }
        a = aux8;
        for (int j = 0; j < QKK / 16; j++) {
            const int scale = x[i].scales[j];
            for (int rep = 0; rep < 2; rep++) {
                for (int l = 0; l < 8; l++) aux16[l] = (int16_t)(q8[l] * a[l]);
                for (int l = 0; l < 8; l++) aux32[l] += scale * aux16[l];
                q8 += 8;
                a += 8;
            }
        }
        const float d = ref_fp16_to_fp32(x[i].d) * y[i].d;
        for (int l = 0; l < 8; l++) sums[l] += d * aux32[l];
    }
    for (int l = 0; l < 8; l++) sumf += sums[l];
    return sumf;
}

/* ---- drivers ------------------------------------------------------------------------------------ */
/* ---- the unquantized weight types (F32, F16, BF16) ------------------------------------------------
 * ggml's CPU mul_mat converts the f32 activations to the weight's own type (type_traits_cpu:
 * vec_dot_type F32 / F16 / BF16, from_float = the row converters) and calls ggml_vec_dot_f32 / _f16 /
 * _bf16.  Their scalar loops widen both operands to fp32, form the product in fp32 and accumulate in
 * ggml_float (double) in element order; the sum is narrowed to fp32 once at the end.  A product of two
 * halves or two bfloat16 is exact in fp32; a product of two floats is rounded to fp32 first.
 *
 * bfloat16 <- fp32 (ggml_compute_fp32_to_bf16): NaNs keep their top mantissa bits and are made quiet,
 * everything else is rounded to nearest even on the upper 16 bits, subnormals included. */
uint16_t ref_fp32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 64);
    return (uint16_t)((u + (0x7fffu + ((u >> 16) & 1u))) >> 16);
}

float ref_bf16_to_fp32(uint16_t h) { return bf16_widen(h); }

static void convert_row_f32(const float *x, void *y, int64_t k) { memcpy(y, x, (size_t)k * 4); }
static void convert_row_f16(const float *x, void *y, int64_t k) {
    uint16_t *o = (uint16_t *)y;
    for (int64_t i = 0; i < k; i++) o[i] = ref_fp32_to_fp16(x[i]);
}
static void convert_row_bf16(const float *x, void *y, int64_t k) {
    uint16_t *o = (uint16_t *)y;
    for (int64_t i = 0; i < k; i++) o[i] = ref_fp32_to_bf16(x[i]);
}

float ref_vec_dot_f32(int64_t n, const void *vx, const void *vy) {
    const float *x = (const float *)vx, *y = (const float *)vy;
    double sum = 0.0;
    for (int64_t i = 0; i < n; i++) sum += (double)(x[i] * y[i]);
    return (float)sum;
}

float ref_vec_dot_f16(int64_t n, const void *vx, const void *vy) {
    const uint16_t *x = (const uint16_t *)vx, *y = (const uint16_t *)vy;
    double sum = 0.0;
    for (int64_t i = 0; i < n; i++) sum += (double)(ref_fp16_to_fp32(x[i]) * ref_fp16_to_fp32(y[i]));
    return (float)sum;
}

float ref_vec_dot_bf16(int64_t n, const void *vx, const void *vy) {
    const uint16_t *x = (const uint16_t *)vx, *y = (const uint16_t *)vy;
    double sum = 0.0;
    for (int64_t i = 0; i < n; i++) sum += (double)(ref_bf16_to_fp32(x[i]) * ref_bf16_to_fp32(y[i]));
    return (float)sum;
}


typedef void (*quant_fn)(const float *, void *, int64_t);
typedef float (*dot_fn)(int64_t, const void *, const void *);

static quant_fn quantizer_for(int type) {
    switch (type) {
    case REF_TYPE_Q4_0: return ref_quantize_row_q4_0;
    case REF_TYPE_Q8_0: return ref_quantize_row_q8_0;
    case REF_TYPE_Q4_K: return ref_quantize_row_q4_K;
    case REF_TYPE_Q6_K: return ref_quantize_row_q6_K;
    case REF_TYPE_Q8_K: return ref_quantize_row_q8_K;
    case REF_TYPE_F32: return convert_row_f32;
    case REF_TYPE_F16: return convert_row_f16;
    case REF_TYPE_BF16: return convert_row_bf16;
    default: return NULL;
    }
}

static dot_fn dot_for(int wtype) {
    switch (wtype) {
    case REF_TYPE_Q4_0: return ref_vec_dot_q4_0_q8_0;
    case REF_TYPE_Q5_0: return ref_vec_dot_q5_0_q8_0;
    case REF_TYPE_Q8_0: return ref_vec_dot_q8_0_q8_0;
    case REF_TYPE_MXFP4: return ref_vec_dot_mxfp4_q8_0;
    case REF_TYPE_Q4_K: return ref_vec_dot_q4_K_q8_K;
    case REF_TYPE_Q5_K: return ref_vec_dot_q5_K_q8_K;
    case REF_TYPE_Q6_K: return ref_vec_dot_q6_K_q8_K;
    case REF_TYPE_F32: return ref_vec_dot_f32;
    case REF_TYPE_F16: return ref_vec_dot_f16;
    case REF_TYPE_BF16: return ref_vec_dot_bf16;
    default: return NULL;
    }
}

typedef struct {
    int tid, nth;
    /* quantize job */
    quant_fn qf; const float *x; char *y; int64_t k, rows, row_bytes;
    /* mul_mat job */
    dot_fn df; const char *w; int64_t w_row_bytes, m, n; const char *xq; int64_t xq_row_bytes; float *out;
} job_t;

static void *quant_worker(void *arg) {
    job_t *j = (job_t *)arg;
    for (int64_t r = j->tid; r < j->rows; r += j->nth)
        j->qf(j->x + r * j->k, j->y + r * j->row_bytes, j->k);
    return NULL;
}

static void *mulmat_worker(void *arg) {
    job_t *j = (job_t *)arg;
    /* contiguous slabs of weight rows per thread; each weight row is streamed once and dotted
     * with every activation row */
    const int64_t per = (j->m + j->nth - 1) / j->nth;
    const int64_t m0 = per * j->tid, m1 = MINI(j->m, m0 + per);
    for (int64_t mi = m0; mi < m1; mi++)
        for (int64_t ni = 0; ni < j->n; ni++)
            j->out[ni * j->m + mi] = j->df(j->k, j->w + mi * j->w_row_bytes, j->xq + ni * j->xq_row_bytes);
    return NULL;
}

static void run_threads(void *(*fn)(void *), job_t *proto, int nthreads) {
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 256) nthreads = 256;
    pthread_t th[256];
    job_t jobs[256];
    for (int t = 0; t < nthreads; t++) {
        jobs[t] = *proto;
        jobs[t].tid = t;
        jobs[t].nth = nthreads;
    }
    for (int t = 1; t < nthreads; t++) pthread_create(&th[t], NULL, fn, &jobs[t]);
    fn(&jobs[0]);
    for (int t = 1; t < nthreads; t++) pthread_join(th[t], NULL);
}

int ref_quantize(int type, const float *x, void *y, int64_t k, int64_t rows, int nthreads) {
    quant_fn qf = quantizer_for(type);
    const int64_t rb = ref_row_size(type, k);
    if (!qf || rb < 0 || rows < 0 || (!x && rows * k != 0) || (!y && rows * k != 0)) return -1;
    job_t j;
    memset(&j, 0, sizeof(j));
    j.qf = qf; j.x = x; j.y = (char *)y; j.k = k; j.rows = rows; j.row_bytes = rb;
    run_threads(quant_worker, &j, nthreads);
    return 0;
}

int ref_mul_mat(int wtype, const void *w, int64_t k, int64_t m, const float *x, int64_t n,
                float *y, void *xq_out, int nthreads) {
    dot_fn df = dot_for(wtype);
    const int qt = ref_vec_dot_type(wtype);
    if (!df || qt < 0 || m < 0 || n < 0) return -1;
    const int64_t wrb = ref_row_size(wtype, k), xrb = ref_row_size(qt, k);
    if (wrb < 0 || xrb < 0) return -1;
    if (m * n == 0) return 0;
    if (!w || !x || !y) return -1;
    char *xq = (char *)xq_out;
    if (!xq) {
        xq = (char *)malloc((size_t)(n * xrb) + 1);
        if (!xq) return -1;
    }
    ref_quantize(qt, x, xq, k, n, nthreads);
    job_t j;
    memset(&j, 0, sizeof(j));
    j.df = df; j.w = (const char *)w; j.w_row_bytes = wrb; j.m = m; j.n = n; j.k = k;
    j.xq = xq; j.xq_row_bytes = xrb; j.out = y;
    run_threads(mulmat_worker, &j, nthreads);
    if (!xq_out) free(xq);
    return 0;
}

/*
 * mul_mat_id (ggml-cpu.c ggml_compute_forward_mul_mat_id, upstream): src1 is quantized row by row
 * to the weight's vec_dot_type, then for every (token t, slot i) pair
 *     dst[t][i][m] = vec_dot(as[ids[t][i]] row m, Q(src1[t][i % ne11]))
 * -- the expert comes from ids, the activation row of slot i is i modulo src1's second dimension
 * (ne11 = 1: one row per token shared by all slots; ne11 = n_used: a row per slot).  upstream
 * asserts 0 <= id < n_as; here that is return value -2.
 */
int ref_mul_mat_id(int wtype, const void *as, int64_t k, int64_t m, int64_t n_expert, const float *b,
                   int64_t b_cols, const int32_t *ids, int64_t n_used, int64_t n_tokens, float *y) {
    dot_fn df = dot_for(wtype);
    const int qt = ref_vec_dot_type(wtype);
    if (!df || qt < 0 || m < 0 || n_expert < 1 || b_cols < 1 || n_used < 1 || n_tokens < 0) return -1;
    const int64_t wrb = ref_row_size(wtype, k), xrb = ref_row_size(qt, k);
    if (wrb < 0 || xrb < 0) return -1;
    if (m * n_tokens == 0) return 0;
    if (!as || !b || !ids || !y) return -1;
    for (int64_t p = 0; p < n_used * n_tokens; p++)
        if (ids[p] < 0 || ids[p] >= n_expert) return -2;
    char *xq = (char *)malloc((size_t)(n_tokens * b_cols * xrb) + 1);
    if (!xq) return -1;
    ref_quantize(qt, b, xq, k, n_tokens * b_cols, 1);
    for (int64_t t = 0; t < n_tokens; t++)
        for (int64_t i = 0; i < n_used; i++) {
            const char *w = (const char *)as + (int64_t)ids[t * n_used + i] * m * wrb;
            const char *x = xq + (t * b_cols + i % b_cols) * xrb;
            float *out = y + (t * n_used + i) * m;
            for (int64_t r = 0; r < m; r++) out[r] = df(k, w + r * wrb, x);
        }
    free(xq);
    return 0;
}

/*
 * Producers of the activations, the steps in front of the path (Tensor.RMSNorm and Tensor.SILU with an
 * "up" operand, /root/reference/ml/backend.go:159 and :180; the arithmetic is upstream ggml's
 * ggml_compute_forward_rms_norm_f32, ggml_compute_forward_mul and ggml_vec_swiglu_f32, restated from
 * their published scalar loops).
 *
 * rms_norm, per row of k floats: the squares are formed in fp32 and accumulated in double in element
 * order; mean = (float)(sum / k); scale = 1.0f / sqrtf(mean + eps); y = x * scale.  The weight g, when
 * given, is the separate broadcast multiply that follows in the graph: y = (x * scale) * g, two
 * roundings.
 */
void ref_rms_norm(const float *x, const float *g, float eps, int64_t k, int64_t n, float *y) {
    for (int64_t r = 0; r < n; r++) {
        const float *xr = x + r * k;
        float *yr = y + r * k;
        double sum = 0.0;
        for (int64_t i = 0; i < k; i++) sum += (double)(xr[i] * xr[i]);
        const float mean = (float)(sum / (double)k);
        const float scale = 1.0f / sqrtf(mean + eps);
        for (int64_t i = 0; i < k; i++) {
            const float v = xr[i] * scale;
            yr[i] = g ? v * g[i] : v;
        }
    }
}

/* swiglu, elementwise over count floats: y = silu(gate) * up with silu(v) = v / (1.0f + expf(-v)). */
void ref_swiglu(const float *gate, const float *up, int64_t count, float *y) {
    for (int64_t i = 0; i < count; i++) y[i] = gate[i] / (1.0f + expf(-gate[i])) * up[i];
}
