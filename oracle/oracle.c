/*
 * CPU oracle for the quantized-inference hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * Plain scalar C restatement of the reference algorithms (ggerganov/llama.cpp).
 * Paths below are relative to the reference root.  Compile with
 * -ffp-contract=off -fno-fast-math so float expressions evaluate exactly as written.
 *
 * What pins each function (see tests/test_oracle_*.py):
 *   - orc_f32_to_f16 / orc_f16_to_f32: exhaustive over all 65536 halves and a seeded
 *     float sweep against the reference build's ggml_fp32_to_fp16_row.
 *   - quantizers / dequantizers: bytewise against the reference build on seeded rows,
 *     closed-form special cases (zero block, single +-amax, .5 ties), round-trip error.
 *   - integer sub-block dots: brute force against dequantized integer levels.
 *   - orc_mul_mat_*: against the reference CPU backend's MUL_MAT (NMSE) and against
 *     dequantize . x in double.
 *   - orc_flash_attn_*: against the reference CPU backend (NMSE) and the textbook
 *     softmax form; GQA pinned by repeating K/V heads.
 *   - glue ops: closed forms and the reference CPU backend.
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define QK   32   /* elements per Q4_0/Q4_1/Q5_0/Q5_1/Q8_0/Q8_1/IQ4_NL block  (ggml/src/ggml-common.h:161-210, 399) */
#define QKK 256   /* elements per K-quant super-block   (ggml/src/ggml-common.h:85) */

#define MAXI(a, b) ((a) > (b) ? (a) : (b))
#define MINI(a, b) ((a) < (b) ? (a) : (b))

/* ------------------------------------------------------------------ block layouts
 * ggml/src/ggml-common.h:161-166 (q4_0), 203-208 (q8_0), 210-221 (q8_1),
 * 279-290 (q4_K), 296-308 (q5_K), 314-320 (q6_K), 322-328 (q8_K), 168-179 (q4_1), 181-187 (q5_0), 189-201 (q5_1),
 * 399-404 (iq4_nl), 406-412 (iq4_xs).  All packed, no padding. */
#pragma pack(push, 1)
typedef struct { uint16_t d; uint8_t qs[16]; } blk_q4_0;                       /* 18 B  */
typedef struct { uint16_t d; uint16_t m; uint8_t qs[16]; } blk_q4_1;           /* 20 B  */
typedef struct { uint16_t d; uint8_t qh[4]; uint8_t qs[16]; } blk_q5_0;        /* 22 B  */
typedef struct { uint16_t d; uint16_t m; uint8_t qh[4]; uint8_t qs[16]; } blk_q5_1; /* 24 B */
typedef struct { uint16_t d; uint8_t qs[16]; } blk_iq4_nl;                     /* 18 B  */
typedef struct { uint16_t d; uint16_t scales_h; uint8_t scales_l[4]; uint8_t qs[128]; } blk_iq4_xs; /* 136 B */
typedef struct { uint16_t d; int8_t qs[32]; } blk_q8_0;                        /* 34 B  */
typedef struct { uint16_t d; uint16_t s; int8_t qs[32]; } blk_q8_1;            /* 36 B  */
typedef struct { uint16_t d; uint16_t dmin; uint8_t scales[12]; uint8_t qs[128]; } blk_q4_K; /* 144 B */
typedef struct { uint16_t d; uint16_t dmin; uint8_t scales[12]; uint8_t qh[32]; uint8_t qs[128]; } blk_q5_K; /* 176 B */
typedef struct { uint8_t ql[128]; uint8_t qh[64]; int8_t scales[16]; uint16_t d; } blk_q6_K; /* 210 B */
typedef struct { float d; int8_t qs[256]; int16_t bsums[16]; } blk_q8_K;       /* 292 B */
#pragma pack(pop)

/* ------------------------------------------------------------------ fp16
 * Behaviour of GGML_FP32_TO_FP16 / GGML_FP16_TO_FP32 (ggml/src/ggml-impl.h:323-357,
 * 380-455): IEEE binary16, round to nearest even, overflow to inf, NaN kept NaN. */
uint16_t orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t absx = x & 0x7fffffffu;
    if (absx > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);      /* NaN */
    if (absx >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);     /* >= 65520 -> inf */
    if (absx < 0x33000001u) return (uint16_t)sign;                  /* <= 2^-25 -> 0 (tie to even) */
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7fffffu) | 0x800000u;                    /* 24-bit significand */
    uint32_t shift;
    uint32_t base;
    if (e < -14) { shift = (uint32_t)(13 + (-14 - e)); base = 0; }  /* subnormal half */
    else { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7fffffu; }
    uint32_t q = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | (base + q));                           /* carry propagates into exponent */
}

float orc_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    uint32_t x;
    if (e == 0) {
        if (m == 0) x = sign;
        else {
            int sh = 0;
            while (!(m & 0x400u)) { m <<= 1; sh++; }
            m &= 0x3ffu;
            x = sign | ((uint32_t)(127 - 15 - sh + 1) << 23) | (m << 13);
        }
    } else if (e == 31) x = sign | 0x7f800000u | (m << 13) | (m ? 0x00400000u : 0u);   /* NaNs come out quiet */
    else x = sign | ((e + 112u) << 23) | (m << 13);
    float f;
    memcpy(&f, &x, 4);
    return f;
}

void orc_f32_to_f16_row(const float *x, uint16_t *y, int64_t n) { for (int64_t i = 0; i < n; i++) y[i] = orc_f32_to_f16(x[i]); }
void orc_f16_to_f32_row(const uint16_t *x, float *y, int64_t n) { for (int64_t i = 0; i < n; i++) y[i] = orc_f16_to_f32(x[i]); }

/* ------------------------------------------------------------------ geometry
 * type table ggml/src/ggml.c:613 (q4_0), 657 (q8_0), 665 (q8_1), 688 (q4_K), 704 (q6_K) */
int orc_block_elems(int type) {
    switch (type) {
        case ORC_F32: case ORC_F16: return 1;
        case ORC_Q4_0: case ORC_Q4_1: case ORC_Q5_0: case ORC_Q5_1: case ORC_IQ4_NL: case ORC_Q8_0: case ORC_Q8_1: return QK;
        case ORC_Q4_K: case ORC_Q5_K: case ORC_Q6_K: case ORC_Q8_K: case ORC_IQ4_XS: return QKK;
        default: return 0;
    }
}
size_t orc_block_bytes(int type) {
    switch (type) {
        case ORC_F32: return 4;
        case ORC_F16: return 2;
        case ORC_Q4_0: return sizeof(blk_q4_0);
        case ORC_Q4_1: return sizeof(blk_q4_1);
        case ORC_Q5_0: return sizeof(blk_q5_0);
        case ORC_Q5_1: return sizeof(blk_q5_1);
        case ORC_IQ4_NL: return sizeof(blk_iq4_nl);
        case ORC_IQ4_XS: return sizeof(blk_iq4_xs);
        case ORC_Q8_0: return sizeof(blk_q8_0);
        case ORC_Q8_1: return sizeof(blk_q8_1);
        case ORC_Q4_K: return sizeof(blk_q4_K);
        case ORC_Q5_K: return sizeof(blk_q5_K);
        case ORC_Q6_K: return sizeof(blk_q6_K);
        case ORC_Q8_K: return sizeof(blk_q8_K);
        default: return 0;
    }
}
size_t orc_row_bytes(int type, int64_t k) {
    const int be = orc_block_elems(type);
    return be ? (size_t)(k / be) * orc_block_bytes(type) : 0;
}

/* ------------------------------------------------------------------ helpers
 * nearest_int: ggml/src/ggml-quants.c:372-377 (magic-number round to nearest even) */
static int near_int(float v) {
    float t = v + 12582912.f;
    int i;
    memcpy(&i, &t, sizeof(int));
    return (i & 0x007fffff) - 0x00400000;
}

/* 6-bit (scale, min) pair j of a Q4_K super-block: ggml/src/ggml-quants.c:631-638 */
static void q4k_scale_min(int j, const uint8_t *p, uint8_t *sc, uint8_t *mn) {
    if (j < 4) {
        *sc = p[j] & 63;
        *mn = p[j + 4] & 63;
    } else {
        *sc = (uint8_t)((p[j + 4] & 0x0F) | ((p[j - 4] >> 6) << 4));
        *mn = (uint8_t)((p[j + 4] >> 4) | ((p[j] >> 6) << 4));
    }
}

/* integer level (0..63) of element e (0..255) of a Q6_K super-block,
 * layout from dequantize_row_q6_K, ggml/src/ggml-quants.c:1690-1719 */
static int q6k_level(const blk_q6_K *b, int e) {
    const int half = e >> 7, r = e & 127, quad = r >> 5, l = r & 31;
    const uint8_t lo = b->ql[64 * half + 32 * (quad & 1) + l];
    const int nib = (quad < 2) ? (lo & 0x0F) : (lo >> 4);
    const int hi = (b->qh[32 * half + l] >> (2 * quad)) & 3;
    return nib | (hi << 4);
}
/* integer level (0..15) of element e of a Q4_K super-block, ggml-quants.c:1280-1302 */
static int q4k_level(const blk_q4_K *b, int e) {
    const int grp = e >> 6, r = e & 63;
    const uint8_t byte = b->qs[32 * grp + (r & 31)];
    return (r < 32) ? (byte & 0x0F) : (byte >> 4);
}
/* level 0..31 of element e of a Q5_K super-block: low nibble as in Q4_K, bit 4 from qh (dequantize_row_q5_K, ggml-quants.c:1482-1507:
 * sub-block j = e / 32 takes bit j of qh[e % 32]) */
static int q5k_level(const blk_q5_K *b, int e) {
    const int j = e / 32, l = e % 32;
    const uint8_t q = b->qs[(j / 2) * 32 + l];
    return ((j & 1) ? (q >> 4) : (q & 0x0F)) + (((b->qh[l] >> j) & 1) ? 16 : 0);
}

/* ------------------------------------------------------------------ Q4_0
 * quantize_row_q4_0_ref, ggml/src/ggml-quants.c:31-66 */
static void quant_q4_0(const float *x, blk_q4_0 *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float *xb = x + b * QK;
        float amax = 0.0f, vmax = 0.0f;
        for (int j = 0; j < QK; j++) {
            if (amax < fabsf(xb[j])) { amax = fabsf(xb[j]); vmax = xb[j]; }
        }
        const float d = vmax / -8;
        const float id = d ? 1.0f / d : 0.0f;
        y[b].d = orc_f32_to_f16(d);
        for (int j = 0; j < QK / 2; j++) {
            const float a0 = xb[j] * id, a1 = xb[j + QK / 2] * id;
            const uint8_t lo = (uint8_t)MINI(15, (int8_t)(a0 + 8.5f));
            const uint8_t hi = (uint8_t)MINI(15, (int8_t)(a1 + 8.5f));
            y[b].qs[j] = (uint8_t)(lo | (hi << 4));
        }
    }
}
/* dequantize_row_q4_0, ggml/src/ggml-quants.c:255-273 */
static void dequant_q4_0(const blk_q4_0 *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float d = orc_f16_to_f32(x[b].d);
        for (int j = 0; j < QK / 2; j++) {
            y[b * QK + j] = ((x[b].qs[j] & 0x0F) - 8) * d;
            y[b * QK + j + QK / 2] = ((x[b].qs[j] >> 4) - 8) * d;
        }
    }
}

/* ------------------------------------------------------------------ Q4_1, Q5_0, Q5_1
 * quantize_row_q4_1_ref / q5_0_ref / q5_1_ref, ggml/src/ggml-quants.c:68-103, 105-147, 149-192;
 * dequantize_row_q4_1 / q5_0 / q5_1, ggml/src/ggml-quants.c:275-294, 296-320, 322-347.
 * Bit j of qh is the fifth bit of element j of the block (elements 0..15 sit in the low nibbles, 16..31 in the high ones). */
static uint32_t q5_qh(const uint8_t *qh) { return (uint32_t)qh[0] | ((uint32_t)qh[1] << 8) | ((uint32_t)qh[2] << 16) | ((uint32_t)qh[3] << 24); }
static int q5_level(const uint8_t *qs, const uint8_t *qh, int j) {
    const int n = j < 16 ? (qs[j] & 0x0F) : (qs[j - 16] >> 4);
    return n | (int)(((q5_qh(qh) >> j) & 1u) << 4);
}
static void quant_q4_1(const float *x, blk_q4_1 *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float *xb = x + b * QK;
        float vmin = 3.402823466e+38f, vmax = -3.402823466e+38f;
        for (int j = 0; j < QK; j++) {
            if (xb[j] < vmin) vmin = xb[j];
            if (xb[j] > vmax) vmax = xb[j];
        }
        const float d = (vmax - vmin) / 15;
        const float id = d ? 1.0f / d : 0.0f;
        y[b].d = orc_f32_to_f16(d);
        y[b].m = orc_f32_to_f16(vmin);
        for (int j = 0; j < QK / 2; j++) {
            const float a0 = (xb[j] - vmin) * id, a1 = (xb[j + QK / 2] - vmin) * id;
            const uint8_t lo = (uint8_t)MINI(15, (int8_t)(a0 + 0.5f));
            const uint8_t hi = (uint8_t)MINI(15, (int8_t)(a1 + 0.5f));
            y[b].qs[j] = (uint8_t)(lo | (hi << 4));
        }
    }
}
static void dequant_q4_1(const blk_q4_1 *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float d = orc_f16_to_f32(x[b].d), m = orc_f16_to_f32(x[b].m);
        for (int j = 0; j < QK / 2; j++) {
            y[b * QK + j] = (x[b].qs[j] & 0x0F) * d + m;
            y[b * QK + j + QK / 2] = (x[b].qs[j] >> 4) * d + m;
        }
    }
}
static void q5_store(uint8_t *qs, uint8_t *qh, const uint8_t *lv) {   /* 32 levels 0..31 -> nibbles + fifth bits */
    uint32_t h = 0;
    for (int j = 0; j < QK / 2; j++) {
        qs[j] = (uint8_t)((lv[j] & 0x0F) | ((lv[j + QK / 2] & 0x0F) << 4));
        h |= (uint32_t)((lv[j] & 0x10) >> 4) << j;
        h |= (uint32_t)((lv[j + QK / 2] & 0x10) >> 4) << (j + QK / 2);
    }
    for (int i = 0; i < 4; i++) qh[i] = (uint8_t)(h >> (8 * i));
}
static void quant_q5_0(const float *x, blk_q5_0 *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float *xb = x + b * QK;
        float amax = 0.0f, vmax = 0.0f;
        for (int j = 0; j < QK; j++) {
            if (amax < fabsf(xb[j])) { amax = fabsf(xb[j]); vmax = xb[j]; }
        }
        const float d = vmax / -16;
        const float id = d ? 1.0f / d : 0.0f;
        y[b].d = orc_f32_to_f16(d);
        uint8_t lv[QK];
        for (int j = 0; j < QK; j++) lv[j] = (uint8_t)MINI(31, (int8_t)(xb[j] * id + 16.5f));
        q5_store(y[b].qs, y[b].qh, lv);
    }
}
static void dequant_q5_0(const blk_q5_0 *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float d = orc_f16_to_f32(x[b].d);
        for (int j = 0; j < QK; j++) y[b * QK + j] = (q5_level(x[b].qs, x[b].qh, j) - 16) * d;
    }
}
static void quant_q5_1(const float *x, blk_q5_1 *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float *xb = x + b * QK;
        float vmin = 3.402823466e+38f, vmax = -3.402823466e+38f;
        for (int j = 0; j < QK; j++) {
            if (xb[j] < vmin) vmin = xb[j];
            if (xb[j] > vmax) vmax = xb[j];
        }
        const float d = (vmax - vmin) / 31;
        const float id = d ? 1.0f / d : 0.0f;
        y[b].d = orc_f32_to_f16(d);
        y[b].m = orc_f32_to_f16(vmin);
        uint8_t lv[QK];
        for (int j = 0; j < QK; j++) lv[j] = (uint8_t)((xb[j] - vmin) * id + 0.5f);   /* no clamp in the reference: bits above the fifth are dropped */
        q5_store(y[b].qs, y[b].qh, lv);
    }
}
static void dequant_q5_1(const blk_q5_1 *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float d = orc_f16_to_f32(x[b].d), m = orc_f16_to_f32(x[b].m);
        for (int j = 0; j < QK; j++) y[b * QK + j] = q5_level(x[b].qs, x[b].qh, j) * d + m;
    }
}

/* ------------------------------------------------------------------ IQ4_NL
 * sixteen non-uniform levels (kvalues_iq4nl, ggml/src/ggml-cpu/ggml-cpu-quants.c:1672); dequantize_row_iq4_nl,
 * ggml/src/ggml-quants.c:2436-2452.  The quantizer is quantize_iq4_nl without importance weights (ggml/src/ggml-quants.c:
 * 4684-4704: what ggml_quantize_chunk and the quantize tool run), i.e. quantize_row_iq4_nl_impl (:4573-4682) on one
 * 32-element block with ntry = 7: a first scale max / -127, then 15 candidate scales, each scored by the weighted
 * least-squares fit with weights x^2, and the levels re-chosen for the winning scale. */
static const int8_t iq4nl_values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
static int iq4nl_best_index(float x) {   /* best_index_int8, ggml/src/ggml-quants.c:4562-4571 */
    const int8_t *val = iq4nl_values;
    if (x <= val[0]) return 0;
    if (x >= val[15]) return 15;
    int ml = 0, mu = 15;
    while (mu - ml > 1) {
        const int mav = (ml + mu) / 2;
        if (x < val[mav]) mu = mav; else ml = mav;
    }
    return x - val[mu - 1] < val[mu] - x ? mu - 1 : mu;
}
/* the scale of one 32-element block: the first guess max / -127, then the 15 candidates (itry - 127) / max, each scored by the
 * weighted least-squares fit with weights x^2 (quantize_row_iq4_nl_impl :4588-4640 with quant_weights == NULL, ntry = 7);
 * 0 for a block whose largest magnitude is below GROUP_MAX_EPS */
static float iq4nl_block_scale(const float *xb) {
    const int ntry = 7;
    float amax = 0, max = 0;
    for (int j = 0; j < QK; j++) {
        const float ax = fabsf(xb[j]);
        if (ax > amax) { amax = ax; max = xb[j]; }
    }
    if (amax < 1e-15f) return 0;
    float d = -max / iq4nl_values[0];
    float id = 1 / d;
    float sumqx = 0, sumq2 = 0;
    for (int j = 0; j < QK; j++) {
        const float q = iq4nl_values[iq4nl_best_index(id * xb[j])];
        const float w = xb[j] * xb[j];
        sumqx += w * q * xb[j];
        sumq2 += w * q * q;
    }
    d = sumqx / sumq2;
    float best = d * sumqx;
    for (int itry = -ntry; itry <= ntry; itry++) {
        id = (itry + iq4nl_values[0]) / max;
        sumqx = sumq2 = 0;
        for (int j = 0; j < QK; j++) {
            const float q = iq4nl_values[iq4nl_best_index(id * xb[j])];
            const float w = xb[j] * xb[j];
            sumqx += w * q * xb[j];
            sumq2 += w * q * q;
        }
        if (sumq2 > 0 && sumqx * sumqx > best * sumq2) { d = sumqx / sumq2; best = d * sumqx; }
    }
    return d;
}
static void iq4nl_pack_block(const float *xb, float id, uint8_t *qs) {   /* element j low, element 16 + j high in byte j */
    uint8_t L[QK];
    for (int j = 0; j < QK; j++) L[j] = (uint8_t)iq4nl_best_index(id * xb[j]);
    for (int j = 0; j < 16; j++) qs[j] = (uint8_t)(L[j] | (L[16 + j] << 4));
}
static void quant_iq4_nl(const float *x, blk_iq4_nl *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float *xb = x + b * QK;
        const float scale = iq4nl_block_scale(xb);
        y[b].d = orc_f32_to_f16(scale);
        iq4nl_pack_block(xb, scale ? 1 / scale : 0, y[b].qs);
    }
}
static void dequant_iq4_nl(const blk_iq4_nl *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float d = orc_f16_to_f32(x[b].d);
        for (int j = 0; j < QK / 2; j++) {
            y[b * QK + j] = d * iq4nl_values[x[b].qs[j] & 0x0F];
            y[b * QK + j + QK / 2] = d * iq4nl_values[x[b].qs[j] >> 4];
        }
    }
}

/* ------------------------------------------------------------------ IQ4_XS
 * super-blocks of 256: eight 32-element blocks of IQ4_NL levels whose scales are d * (ls - 32), ls six bits (low four in scales_l,
 * high two in scales_h).  quantize_iq4_xs without importance weights (ggml/src/ggml-quants.c:4722-4745) = quantize_row_iq4_nl_impl
 * on the super-block (:4573-4682): the block scales as for IQ4_NL, d = -(the block scale of largest magnitude) / 32, ls = the block
 * scale over d rounded and clamped to [-32, 31], the levels chosen again for d * ls.  dequantize_row_iq4_xs :2454-2475. */
static int iq4xs_ls(const blk_iq4_xs *b, int ib) {
    return ((b->scales_l[ib / 2] >> 4 * (ib % 2)) & 0xF) | (((b->scales_h >> 2 * ib) & 3) << 4);
}
static void quant_iq4_xs(const float *x, blk_iq4_xs *y, int64_t k) {
    for (int64_t sb = 0; sb < k / QKK; sb++) {
        const float *xs = x + sb * QKK;
        float scales[8];
        float max_scale = 0, amax_scale = 0;
        memset(&y[sb], 0, sizeof(blk_iq4_xs));
        for (int ib = 0; ib < 8; ib++) {
            scales[ib] = iq4nl_block_scale(xs + ib * QK);
            const float a = fabsf(scales[ib]);
            if (a > amax_scale) { amax_scale = a; max_scale = scales[ib]; }
        }
        const float d = -max_scale / 32;
        y[sb].d = orc_f32_to_f16(d);
        const float id = d ? 1 / d : 0.f;
        for (int ib = 0; ib < 8; ib++) {
            int l = near_int(id * scales[ib]);
            l = MAXI(-32, MINI(31, l));
            const float dl = d * l;
            iq4nl_pack_block(xs + ib * QK, dl ? 1 / dl : 0.f, y[sb].qs + 16 * ib);
            l += 32;
            y[sb].scales_l[ib / 2] |= (uint8_t)((l & 0xF) << 4 * (ib % 2));
            y[sb].scales_h |= (uint16_t)((l >> 4) << 2 * ib);
        }
    }
}
static void dequant_iq4_xs(const blk_iq4_xs *x, float *y, int64_t k) {
    for (int64_t sb = 0; sb < k / QKK; sb++) {
        const float d = orc_f16_to_f32(x[sb].d);
        for (int ib = 0; ib < 8; ib++) {
            const float dl = d * (iq4xs_ls(&x[sb], ib) - 32);
            const uint8_t *qs = x[sb].qs + 16 * ib;
            for (int j = 0; j < 16; j++) {
                y[sb * QKK + ib * QK + j] = dl * iq4nl_values[qs[j] & 0x0F];
                y[sb * QKK + ib * QK + j + 16] = dl * iq4nl_values[qs[j] >> 4];
            }
        }
    }
}

/* ------------------------------------------------------------------ Q8_0
 * quantize_row_q8_0_ref, ggml/src/ggml-quants.c:194-217 */
static void quant_q8_0(const float *x, blk_q8_0 *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float *xb = x + b * QK;
        float amax = 0.0f;
        for (int j = 0; j < QK; j++) amax = fabsf(xb[j]) > amax ? fabsf(xb[j]) : amax;
        const float d = amax / 127;
        const float id = d ? 1.0f / d : 0.0f;
        y[b].d = orc_f32_to_f16(d);
        for (int j = 0; j < QK; j++) y[b].qs[j] = (int8_t)roundf(xb[j] * id);
    }
}
/* dequantize_row_q8_0, ggml/src/ggml-quants.c:349-363 */
static void dequant_q8_0(const blk_q8_0 *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float d = orc_f16_to_f32(x[b].d);
        for (int j = 0; j < QK; j++) y[b * QK + j] = x[b].qs[j] * d;
    }
}

/* ------------------------------------------------------------------ Q8_1
 * quantize_row_q8_1_ref, ggml/src/ggml-quants.c:220-253: the bit-exact target of the
 * on-device activation quantizer. */
static void quant_q8_1(const float *x, blk_q8_1 *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float *xb = x + b * QK;
        float amax = 0.0f;
        for (int j = 0; j < QK; j++) amax = fabsf(xb[j]) > amax ? fabsf(xb[j]) : amax;
        const float d = amax / 127;
        const float id = d ? 1.0f / d : 0.0f;
        y[b].d = orc_f32_to_f16(d);
        int sum = 0;
        for (int j = 0; j < QK; j++) {
            y[b].qs[j] = (int8_t)roundf(xb[j] * id);
            sum += y[b].qs[j];
        }
        y[b].s = orc_f32_to_f16(sum * d);
    }
}
static void dequant_q8_1(const blk_q8_1 *x, float *y, int64_t k) {
    for (int64_t b = 0; b < k / QK; b++) {
        const float d = orc_f16_to_f32(x[b].d);
        for (int j = 0; j < QK; j++) y[b * QK + j] = x[b].qs[j] * d;
    }
}

/* ------------------------------------------------------------------ Q4_K
 * make_qkx2_quants, ggml/src/ggml-quants.c:550-629: weighted least-squares search for
 * the (scale, min) of one 32-element sub-block quantized to levels 0..nmax. */
static float fit_scale_min(int n, int nmax, const float *x, const float *w, uint8_t *L, float *the_min,
                           uint8_t *Laux, float rmin, float rdelta, int nstep) {
    float lo = x[0], hi = x[0];
    float sum_w = w[0];
    float sum_x = sum_w * x[0];
    for (int i = 1; i < n; i++) {
        if (x[i] < lo) lo = x[i];
        if (x[i] > hi) hi = x[i];
        sum_w += w[i];
        sum_x += w[i] * x[i];
    }
    if (lo > 0) lo = 0;
    if (hi == lo) {
        for (int i = 0; i < n; i++) L[i] = 0;
        *the_min = -lo;
        return 0.f;
    }
    float iscale = nmax / (hi - lo);
    float scale = 1 / iscale;
    float best = 0;
    for (int i = 0; i < n; i++) {
        int l = near_int(iscale * (x[i] - lo));
        L[i] = (uint8_t)MAXI(0, MINI(nmax, l));
        float diff = scale * L[i] + lo - x[i];
        diff = diff * diff;
        best += w[i] * diff;
    }
    if (nstep < 1) {
        *the_min = -lo;
        return scale;
    }
    for (int is = 0; is <= nstep; is++) {
        iscale = (rmin + rdelta * is + nmax) / (hi - lo);
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        for (int i = 0; i < n; i++) {
            int l = near_int(iscale * (x[i] - lo));
            l = MAXI(0, MINI(nmax, l));
            Laux[i] = (uint8_t)l;
            sum_l += w[i] * l;
            sum_l2 += w[i] * l * l;
            sum_xl += w[i] * l * x[i];
        }
        const float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float sc = (sum_w * sum_xl - sum_x * sum_l) / D;
            float mn = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (mn > 0) {
                mn = 0;
                sc = sum_xl / sum_l2;
            }
            float err = 0;
            for (int i = 0; i < n; i++) {
                float diff = sc * Laux[i] + mn - x[i];
                diff = diff * diff;
                err += w[i] * diff;
            }
            if (err < best) {
                for (int i = 0; i < n; i++) L[i] = Laux[i];
                best = err;
                scale = sc;
                lo = mn;
            }
        }
    }
    *the_min = -lo;
    return scale;
}

/* quantize_row_q4_K_ref, ggml/src/ggml-quants.c:1208-1278 */
static void quant_q4_K(const float *x, blk_q4_K *y, int64_t k) {
    uint8_t L[QKK], Laux[32];
    float wts[32], mins[8], scales[8];
    for (int64_t sb = 0; sb < k / QKK; sb++, x += QKK) {
        float max_scale = 0, max_min = 0;
        for (int j = 0; j < 8; j++) {
            float sum_x2 = 0;
            for (int l = 0; l < 32; l++) sum_x2 += x[32 * j + l] * x[32 * j + l];
            const float av_x = sqrtf(sum_x2 / 32);
            for (int l = 0; l < 32; l++) wts[l] = av_x + fabsf(x[32 * j + l]);
            scales[j] = fit_scale_min(32, 15, x + 32 * j, wts, L + 32 * j, &mins[j], Laux, -1.f, 0.1f, 20);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
        const float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
        memset(y[sb].scales, 0, 12);
        for (int j = 0; j < 8; j++) {
            uint8_t ls = (uint8_t)near_int(inv_scale * scales[j]);
            uint8_t lm = (uint8_t)near_int(inv_min * mins[j]);
            ls = (uint8_t)MINI(63, ls);
            lm = (uint8_t)MINI(63, lm);
            if (j < 4) {
                y[sb].scales[j] = ls;
                y[sb].scales[j + 4] = lm;
            } else {
                y[sb].scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                y[sb].scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                y[sb].scales[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        y[sb].d = orc_f32_to_f16(max_scale / 63.f);
        y[sb].dmin = orc_f32_to_f16(max_min / 63.f);
        for (int j = 0; j < 8; j++) {
            uint8_t sc, mn;
            q4k_scale_min(j, y[sb].scales, &sc, &mn);
            const float d = orc_f16_to_f32(y[sb].d) * sc;
            if (!d) continue;
            const float dm = orc_f16_to_f32(y[sb].dmin) * mn;
            for (int i = 0; i < 32; i++) {
                int l = near_int((x[32 * j + i] + dm) / d);
                L[32 * j + i] = (uint8_t)MAXI(0, MINI(15, l));
            }
        }
        uint8_t *q = y[sb].qs;
        for (int j = 0; j < QKK; j += 64, q += 32)
            for (int l = 0; l < 32; l++) q[l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
    }
}
/* dequantize_row_q4_K, ggml/src/ggml-quants.c:1280-1302 */
static void dequant_q4_K(const blk_q4_K *x, float *y, int64_t k) {
    for (int64_t sb = 0; sb < k / QKK; sb++) {
        const float d = orc_f16_to_f32(x[sb].d), dmin = orc_f16_to_f32(x[sb].dmin);
        for (int j = 0; j < 8; j++) {
            uint8_t sc, mn;
            q4k_scale_min(j, x[sb].scales, &sc, &mn);
            const float dj = d * sc, mj = dmin * mn;
            for (int l = 0; l < 32; l++) y[sb * QKK + 32 * j + l] = dj * q4k_level(&x[sb], 32 * j + l) - mj;
        }
    }
}

/* ------------------------------------------------------------------ Q5_K
 * quantize_row_q5_K_ref, ggml/src/ggml-quants.c:1395-1480: the Q4_K scheme with 32 levels (search parameters -0.5, 0.1, 15) and the
 * fifth bit of sub-block j in bit j of qh */
static void quant_q5_K(const float *x, blk_q5_K *y, int64_t k) {
    uint8_t L[QKK], Laux[32];
    float wts[32], mins[8], scales[8];
    for (int64_t sb = 0; sb < k / QKK; sb++, x += QKK) {
        float max_scale = 0, max_min = 0;
        for (int j = 0; j < 8; j++) {
            float sum_x2 = 0;
            for (int l = 0; l < 32; l++) sum_x2 += x[32 * j + l] * x[32 * j + l];
            const float av_x = sqrtf(sum_x2 / 32);
            for (int l = 0; l < 32; l++) wts[l] = av_x + fabsf(x[32 * j + l]);
            scales[j] = fit_scale_min(32, 31, x + 32 * j, wts, L + 32 * j, &mins[j], Laux, -0.5f, 0.1f, 15);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
        const float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
        memset(y[sb].scales, 0, 12);
        for (int j = 0; j < 8; j++) {
            uint8_t ls = (uint8_t)near_int(inv_scale * scales[j]);
            uint8_t lm = (uint8_t)near_int(inv_min * mins[j]);
            ls = (uint8_t)MINI(63, ls);
            lm = (uint8_t)MINI(63, lm);
            if (j < 4) {
                y[sb].scales[j] = ls;
                y[sb].scales[j + 4] = lm;
            } else {
                y[sb].scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                y[sb].scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                y[sb].scales[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        y[sb].d = orc_f32_to_f16(max_scale / 63.f);
        y[sb].dmin = orc_f32_to_f16(max_min / 63.f);
        for (int j = 0; j < 8; j++) {
            uint8_t sc, mn;
            q4k_scale_min(j, y[sb].scales, &sc, &mn);
            const float d = orc_f16_to_f32(y[sb].d) * sc;
            if (!d) continue;
            const float dm = orc_f16_to_f32(y[sb].dmin) * mn;
            for (int i = 0; i < 32; i++) {
                int l = near_int((x[32 * j + i] + dm) / d);
                L[32 * j + i] = (uint8_t)MAXI(0, MINI(31, l));
            }
        }
        memset(y[sb].qh, 0, 32);
        for (int j = 0; j < 8; j++)
            for (int l = 0; l < 32; l++) {
                const int v = L[32 * j + l];
                uint8_t *q = &y[sb].qs[(j / 2) * 32 + l];
                if (j & 1) *q = (uint8_t)((*q & 0x0F) | ((v & 15) << 4));
                else *q = (uint8_t)(v & 15);
                if (v > 15) y[sb].qh[l] |= (uint8_t)(1u << j);
            }
    }
}
/* dequantize_row_q5_K, ggml/src/ggml-quants.c:1482-1507 */
static void dequant_q5_K(const blk_q5_K *x, float *y, int64_t k) {
    for (int64_t sb = 0; sb < k / QKK; sb++) {
        const float d = orc_f16_to_f32(x[sb].d), dmin = orc_f16_to_f32(x[sb].dmin);
        for (int j = 0; j < 8; j++) {
            uint8_t sc, mn;
            q4k_scale_min(j, x[sb].scales, &sc, &mn);
            const float dj = d * sc, mj = dmin * mn;
            for (int l = 0; l < 32; l++) y[sb * QKK + 32 * j + l] = dj * q5k_level(&x[sb], 32 * j + l) - mj;
        }
    }
}

/* ------------------------------------------------------------------ Q6_K
 * make_qx_quants with rmse_type 1 and no weights, ggml/src/ggml-quants.c:379-446 */
static float fit_scale_sym(int n, int nmax, const float *x, int8_t *L) {
    float vmax = 0, amax = 0;
    for (int i = 0; i < n; i++) {
        const float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; vmax = x[i]; }
    }
    if (amax < 1e-15f) {                       /* GROUP_MAX_EPS, ggml-quants.c:22 */
        for (int i = 0; i < n; i++) L[i] = 0;
        return 0.f;
    }
    float iscale = -nmax / vmax;
    float sumlx = 0, suml2 = 0;
    for (int i = 0; i < n; i++) {
        int l = near_int(iscale * x[i]);
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
        iscale = -(nmax + 0.1f * is) / vmax;
        sumlx = suml2 = 0;
        for (int i = 0; i < n; i++) {
            int l = near_int(iscale * x[i]);
            l = MAXI(-nmax, MINI(nmax - 1, l));
            const float w = x[i] * x[i];
            sumlx += w * x[i] * l;
            suml2 += w * l * l;
        }
        if (suml2 > 0 && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; i++) {
                int l = near_int(iscale * x[i]);
                L[i] = (int8_t)(nmax + MAXI(-nmax, MINI(nmax - 1, l)));
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

/* quantize_row_q6_K_ref, ggml/src/ggml-quants.c:1620-1688 */
static void quant_q6_K(const float *x, blk_q6_K *y, int64_t k) {
    int8_t L[QKK];
    float scales[16];
    for (int64_t sb = 0; sb < k / QKK; sb++, x += QKK) {
        float max_scale = 0, max_abs = 0;
        for (int g = 0; g < 16; g++) {
            scales[g] = fit_scale_sym(16, 32, x + 16 * g, L + 16 * g);
            if (fabsf(scales[g]) > max_abs) { max_abs = fabsf(scales[g]); max_scale = scales[g]; }
        }
        if (max_abs < 1e-15f) {
            memset(&y[sb], 0, sizeof(blk_q6_K));
            continue;
        }
        const float iscale = -128.f / max_scale;
        y[sb].d = orc_f32_to_f16(1 / iscale);
        for (int g = 0; g < 16; g++) y[sb].scales[g] = (int8_t)MINI(127, near_int(iscale * scales[g]));
        for (int g = 0; g < 16; g++) {
            const float d = orc_f16_to_f32(y[sb].d) * y[sb].scales[g];
            if (!d) continue;
            for (int i = 0; i < 16; i++) {
                int l = near_int(x[16 * g + i] / d);
                L[16 * g + i] = (int8_t)(MAXI(-32, MINI(31, l)) + 32);
            }
        }
        uint8_t *ql = y[sb].ql, *qh = y[sb].qh;
        for (int j = 0; j < QKK; j += 128, ql += 64, qh += 32) {
            for (int l = 0; l < 32; l++) {
                ql[l] = (uint8_t)((L[j + l] & 0xF) | ((L[j + l + 64] & 0xF) << 4));
                ql[l + 32] = (uint8_t)((L[j + l + 32] & 0xF) | ((L[j + l + 96] & 0xF) << 4));
                qh[l] = (uint8_t)((L[j + l] >> 4) | ((L[j + l + 32] >> 4) << 2) | ((L[j + l + 64] >> 4) << 4) |
                                  ((L[j + l + 96] >> 4) << 6));
            }
        }
    }
}
/* dequantize_row_q6_K, ggml/src/ggml-quants.c:1690-1719 */
static void dequant_q6_K(const blk_q6_K *x, float *y, int64_t k) {
    for (int64_t sb = 0; sb < k / QKK; sb++) {
        const float d = orc_f16_to_f32(x[sb].d);
        for (int e = 0; e < QKK; e++) {
            const int8_t q = (int8_t)(q6k_level(&x[sb], e) - 32);
            y[sb * QKK + e] = d * x[sb].scales[e / 16] * q;
        }
    }
}

/* ------------------------------------------------------------------ Q8_K
 * quantize_row_q8_K_ref, ggml/src/ggml-quants.c:2479-2516 */
static void quant_q8_K(const float *x, blk_q8_K *y, int64_t k) {
    for (int64_t sb = 0; sb < k / QKK; sb++, x += QKK) {
        float vmax = 0, amax = 0;
        for (int j = 0; j < QKK; j++) {
            const float ax = fabsf(x[j]);
            if (ax > amax) { amax = ax; vmax = x[j]; }
        }
        if (!amax) {
            y[sb].d = 0;
            memset(y[sb].qs, 0, QKK);
            memset(y[sb].bsums, 0, sizeof(y[sb].bsums));   /* the reference leaves bsums untouched here */
            continue;
        }
        const float iscale = -127.f / vmax;
        for (int j = 0; j < QKK; j++) y[sb].qs[j] = (int8_t)MINI(127, near_int(iscale * x[j]));
        for (int g = 0; g < 16; g++) {
            int sum = 0;
            for (int i = 0; i < 16; i++) sum += y[sb].qs[16 * g + i];
            y[sb].bsums[g] = (int16_t)sum;
        }
        y[sb].d = 1 / iscale;
    }
}
static void dequant_q8_K(const blk_q8_K *x, float *y, int64_t k) {
    for (int64_t sb = 0; sb < k / QKK; sb++)
        for (int j = 0; j < QKK; j++) y[sb * QKK + j] = x[sb].d * x[sb].qs[j];
}

/* ------------------------------------------------------------------ type dispatch */
static int quantize_row(int type, const float *x, void *y, int64_t k) {
    switch (type) {
        case ORC_F32: memcpy(y, x, (size_t)k * 4); return 0;
        case ORC_F16: orc_f32_to_f16_row(x, (uint16_t *)y, k); return 0;
        case ORC_Q4_0: quant_q4_0(x, (blk_q4_0 *)y, k); return 0;
        case ORC_Q4_1: quant_q4_1(x, (blk_q4_1 *)y, k); return 0;
        case ORC_Q5_0: quant_q5_0(x, (blk_q5_0 *)y, k); return 0;
        case ORC_Q5_1: quant_q5_1(x, (blk_q5_1 *)y, k); return 0;
        case ORC_IQ4_NL: quant_iq4_nl(x, (blk_iq4_nl *)y, k); return 0;
        case ORC_IQ4_XS: quant_iq4_xs(x, (blk_iq4_xs *)y, k); return 0;
        case ORC_Q8_0: quant_q8_0(x, (blk_q8_0 *)y, k); return 0;
        case ORC_Q8_1: quant_q8_1(x, (blk_q8_1 *)y, k); return 0;
        case ORC_Q4_K: quant_q4_K(x, (blk_q4_K *)y, k); return 0;
        case ORC_Q5_K: quant_q5_K(x, (blk_q5_K *)y, k); return 0;
        case ORC_Q6_K: quant_q6_K(x, (blk_q6_K *)y, k); return 0;
        case ORC_Q8_K: quant_q8_K(x, (blk_q8_K *)y, k); return 0;
        default: return -1;
    }
}
static int dequantize_row(int type, const void *x, float *y, int64_t k) {
    switch (type) {
        case ORC_F32: memcpy(y, x, (size_t)k * 4); return 0;
        case ORC_F16: orc_f16_to_f32_row((const uint16_t *)x, y, k); return 0;
        case ORC_Q4_0: dequant_q4_0((const blk_q4_0 *)x, y, k); return 0;
        case ORC_Q4_1: dequant_q4_1((const blk_q4_1 *)x, y, k); return 0;
        case ORC_Q5_0: dequant_q5_0((const blk_q5_0 *)x, y, k); return 0;
        case ORC_Q5_1: dequant_q5_1((const blk_q5_1 *)x, y, k); return 0;
        case ORC_IQ4_NL: dequant_iq4_nl((const blk_iq4_nl *)x, y, k); return 0;
        case ORC_IQ4_XS: dequant_iq4_xs((const blk_iq4_xs *)x, y, k); return 0;
        case ORC_Q8_0: dequant_q8_0((const blk_q8_0 *)x, y, k); return 0;
        case ORC_Q8_1: dequant_q8_1((const blk_q8_1 *)x, y, k); return 0;
        case ORC_Q4_K: dequant_q4_K((const blk_q4_K *)x, y, k); return 0;
        case ORC_Q5_K: dequant_q5_K((const blk_q5_K *)x, y, k); return 0;
        case ORC_Q6_K: dequant_q6_K((const blk_q6_K *)x, y, k); return 0;
        case ORC_Q8_K: dequant_q8_K((const blk_q8_K *)x, y, k); return 0;
        default: return -1;
    }
}
int orc_quantize(int type, const float *x, void *y, int64_t nrows, int64_t k) {
    const int be = orc_block_elems(type);
    if (!be || k % be) return -1;
    const size_t rb = orc_row_bytes(type, k);
    for (int64_t r = 0; r < nrows; r++)
        if (quantize_row(type, x + r * k, (char *)y + r * rb, k)) return -1;
    return 0;
}
int orc_dequantize(int type, const void *x, float *y, int64_t nrows, int64_t k) {
    const int be = orc_block_elems(type);
    if (!be || k % be) return -1;
    const size_t rb = orc_row_bytes(type, k);
    for (int64_t r = 0; r < nrows; r++)
        if (dequantize_row(type, (const char *)x + r * rb, y + r * k, k)) return -1;
    return 0;
}

/* ------------------------------------------------------------------ integer sub-block dots vs Q8_1
 * The integer parts of ggml_vec_dot_q4_0_q8_0 (ggml/src/ggml-cpu/ggml-cpu-quants.c:2492-2506),
 * ggml_vec_dot_q8_0_q8_0 (:3919-3927), ggml_vec_dot_q4_K_q8_K (:6817-6848) and
 * ggml_vec_dot_q6_K_q8_K (:8262-8283), taken per 32-element (16 for Q6_K) granule. */
static int weight_level(int type, const void *row, int64_t e) {
    switch (type) {
        case ORC_Q4_0: {
            const blk_q4_0 *b = (const blk_q4_0 *)row + e / QK;
            const int j = (int)(e % QK);
            return (j < 16 ? (b->qs[j] & 0x0F) : (b->qs[j - 16] >> 4)) - 8;
        }
        case ORC_Q4_1: {   /* unsigned levels; the block minimum enters through the sum of the activation levels */
            const blk_q4_1 *b = (const blk_q4_1 *)row + e / QK;
            const int j = (int)(e % QK);
            return j < 16 ? (b->qs[j] & 0x0F) : (b->qs[j - 16] >> 4);
        }
        case ORC_Q5_0: { const blk_q5_0 *b = (const blk_q5_0 *)row + e / QK; return q5_level(b->qs, b->qh, (int)(e % QK)) - 16; }
        case ORC_Q5_1: { const blk_q5_1 *b = (const blk_q5_1 *)row + e / QK; return q5_level(b->qs, b->qh, (int)(e % QK)); }
        case ORC_IQ4_NL: {
            const blk_iq4_nl *b = (const blk_iq4_nl *)row + e / QK;
            const int j = (int)(e % QK);
            return iq4nl_values[j < 16 ? (b->qs[j] & 0x0F) : (b->qs[j - 16] >> 4)];
        }
        case ORC_IQ4_XS: {
            const blk_iq4_xs *b = (const blk_iq4_xs *)row + e / QKK;
            const int ib = (int)(e % QKK) / QK, j = (int)(e % QK);
            return iq4nl_values[j < 16 ? (b->qs[16 * ib + j] & 0x0F) : (b->qs[16 * ib + j - 16] >> 4)];
        }
        case ORC_Q8_0: return ((const blk_q8_0 *)row + e / QK)->qs[e % QK];
        case ORC_Q4_K: return q4k_level((const blk_q4_K *)row + e / QKK, (int)(e % QKK));
        case ORC_Q5_K: return q5k_level((const blk_q5_K *)row + e / QKK, (int)(e % QKK));
        case ORC_Q6_K: return q6k_level((const blk_q6_K *)row + e / QKK, (int)(e % QKK)) - 32;
        default: return 0;
    }
}
static int granule(int type) { return type == ORC_Q6_K ? 16 : 32; }
static int is_weight_type(int type) {
    switch (type) {
        case ORC_Q4_0: case ORC_Q4_1: case ORC_Q5_0: case ORC_Q5_1: case ORC_IQ4_NL: case ORC_Q8_0:
        case ORC_Q4_K: case ORC_Q5_K: case ORC_Q6_K: case ORC_IQ4_XS: return 1;
        default: return 0;
    }
}

int orc_block_dots_q8_1(int type, const void *W, const void *a, int64_t nrows, int64_t k, int32_t *out) {
    if (!is_weight_type(type)) return -1;
    if (k % orc_block_elems(type)) return -1;
    const int g = granule(type);
    const size_t rb = orc_row_bytes(type, k);
    const blk_q8_1 *act = (const blk_q8_1 *)a;
    for (int64_t r = 0; r < nrows; r++) {
        const char *row = (const char *)W + r * rb;
        for (int64_t j = 0; j < k / g; j++) {
            int32_t acc = 0;
            for (int i = 0; i < g; i++) {
                const int64_t e = j * g + i;
                acc += weight_level(type, row, e) * act[e / QK].qs[e % QK];
            }
            out[r * (k / g) + j] = acc;
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ MUL_MAT
 * ggml_compute_forward_mul_mat, ggml/src/ggml-cpu/ggml-cpu.c:7443-7635: src1 rows are
 * quantized to the weight type's vec_dot_type (type_traits_cpu, :252-417), then
 * dst[n,b] = vec_dot(W row n, quantized x row b). */
static float dot_q4_0_q8_0(const blk_q4_0 *w, const blk_q8_0 *a, int64_t k) {   /* ggml-cpu-quants.c:2492-2506 */
    float sumf = 0;
    for (int64_t b = 0; b < k / QK; b++) {
        int sumi0 = 0, sumi1 = 0;
        for (int j = 0; j < 16; j++) {
            sumi0 += ((w[b].qs[j] & 0x0F) - 8) * a[b].qs[j];
            sumi1 += ((w[b].qs[j] >> 4) - 8) * a[b].qs[j + 16];
        }
        sumf += (sumi0 + sumi1) * orc_f16_to_f32(w[b].d) * orc_f16_to_f32(a[b].d);
    }
    return sumf;
}
/* the per-32 types share one form: sum over blocks of (d_w * d_a) * sumi [+ m_w * s_a]
 * (ggml_vec_dot_q4_1_q8_1 ggml-cpu-quants.c:2511 ff., scalar tail :2784-2799; q5_0_q8_0 :2804 ff., tail :3131-3153;
 * q5_1_q8_1 :3159 ff., tail :3504-3526; iq4_nl_q8_0 :11188 ff., tail :11368-11377) */
static float dot_q4_1_q8_1(const blk_q4_1 *w, const blk_q8_1 *a, int64_t k) {
    float sumf = 0;
    for (int64_t b = 0; b < k / QK; b++) {
        int sumi0 = 0, sumi1 = 0;
        for (int j = 0; j < 16; j++) {
            sumi0 += (w[b].qs[j] & 0x0F) * a[b].qs[j];
            sumi1 += (w[b].qs[j] >> 4) * a[b].qs[j + 16];
        }
        sumf += (orc_f16_to_f32(w[b].d) * orc_f16_to_f32(a[b].d)) * (sumi0 + sumi1) + orc_f16_to_f32(w[b].m) * orc_f16_to_f32(a[b].s);
    }
    return sumf;
}
static float dot_q5_0_q8_0(const blk_q5_0 *w, const blk_q8_0 *a, int64_t k) {
    float sumf = 0;
    for (int64_t b = 0; b < k / QK; b++) {
        int sumi0 = 0, sumi1 = 0;
        for (int j = 0; j < 16; j++) {
            sumi0 += (q5_level(w[b].qs, w[b].qh, j) - 16) * a[b].qs[j];
            sumi1 += (q5_level(w[b].qs, w[b].qh, j + 16) - 16) * a[b].qs[j + 16];
        }
        sumf += (orc_f16_to_f32(w[b].d) * orc_f16_to_f32(a[b].d)) * (sumi0 + sumi1);
    }
    return sumf;
}
static float dot_q5_1_q8_1(const blk_q5_1 *w, const blk_q8_1 *a, int64_t k) {
    float sumf = 0;
    for (int64_t b = 0; b < k / QK; b++) {
        int sumi0 = 0, sumi1 = 0;
        for (int j = 0; j < 16; j++) {
            sumi0 += q5_level(w[b].qs, w[b].qh, j) * a[b].qs[j];
            sumi1 += q5_level(w[b].qs, w[b].qh, j + 16) * a[b].qs[j + 16];
        }
        sumf += (orc_f16_to_f32(w[b].d) * orc_f16_to_f32(a[b].d)) * (sumi0 + sumi1) + orc_f16_to_f32(w[b].m) * orc_f16_to_f32(a[b].s);
    }
    return sumf;
}
static float dot_iq4_nl_q8_0(const blk_iq4_nl *w, const blk_q8_0 *a, int64_t k) {
    float sumf = 0;
    for (int64_t b = 0; b < k / QK; b++) {
        const float d = orc_f16_to_f32(a[b].d) * orc_f16_to_f32(w[b].d);
        int sumi1 = 0, sumi2 = 0;
        for (int j = 0; j < 16; j++) {
            sumi1 += a[b].qs[j] * iq4nl_values[w[b].qs[j] & 0x0F];
            sumi2 += a[b].qs[j + 16] * iq4nl_values[w[b].qs[j] >> 4];
        }
        sumf += d * (sumi1 + sumi2);
    }
    return sumf;
}
static float dot_q8_0_q8_0(const blk_q8_0 *w, const blk_q8_0 *a, int64_t k) {   /* ggml-cpu-quants.c:3919-3927 */
    float sumf = 0;
    for (int64_t b = 0; b < k / QK; b++) {
        int sumi = 0;
        for (int j = 0; j < QK; j++) sumi += w[b].qs[j] * a[b].qs[j];
        sumf += sumi * (orc_f16_to_f32(w[b].d) * orc_f16_to_f32(a[b].d));
    }
    return sumf;
}
static float dot_q4_K_q8_K(const blk_q4_K *w, const blk_q8_K *a, int64_t k) {   /* ggml-cpu-quants.c:6800-6856 */
    float sums[8] = {0};
    float sumf = 0;
    for (int64_t sb = 0; sb < k / QKK; sb++) {
        int32_t lane[8] = {0};
        int summ = 0;
        for (int j = 0; j < 8; j++) {
            uint8_t sc, mn;
            q4k_scale_min(j, w[sb].scales, &sc, &mn);
            summ += (a[sb].bsums[2 * j] + a[sb].bsums[2 * j + 1]) * mn;
            for (int l = 0; l < 32; l++) lane[l & 7] += sc * (q4k_level(&w[sb], 32 * j + l) * a[sb].qs[32 * j + l]);
        }
        const float d = orc_f16_to_f32(w[sb].d) * a[sb].d;
        for (int l = 0; l < 8; l++) sums[l] += d * lane[l];
        const float dmin = orc_f16_to_f32(w[sb].dmin) * a[sb].d;
        sumf -= dmin * summ;
    }
    for (int l = 0; l < 8; l++) sumf += sums[l];
    return sumf;
}
static float dot_q5_K_q8_K(const blk_q5_K *w, const blk_q8_K *a, int64_t k) {   /* ggml-cpu-quants.c:7539-7592: the Q4_K form on 5-bit levels */
    float sums[8] = {0};
    float sumf = 0;
    for (int64_t sb = 0; sb < k / QKK; sb++) {
        int32_t lane[8] = {0};
        int summ = 0;
        for (int j = 0; j < 8; j++) {
            uint8_t sc, mn;
            q4k_scale_min(j, w[sb].scales, &sc, &mn);
            summ += (a[sb].bsums[2 * j] + a[sb].bsums[2 * j + 1]) * mn;
            for (int l = 0; l < 32; l++) lane[l & 7] += sc * (q5k_level(&w[sb], 32 * j + l) * a[sb].qs[32 * j + l]);
        }
        const float d = orc_f16_to_f32(w[sb].d) * a[sb].d;
        for (int l = 0; l < 8; l++) sums[l] += d * lane[l];
        const float dmin = orc_f16_to_f32(w[sb].dmin) * a[sb].d;
        sumf -= dmin * summ;
    }
    for (int l = 0; l < 8; l++) sumf += sums[l];
    return sumf;
}
static float dot_q6_K_q8_K(const blk_q6_K *w, const blk_q8_K *a, int64_t k) {   /* ggml-cpu-quants.c:8247-8289 */
    float sums[8] = {0};
    float sumf = 0;
    for (int64_t sb = 0; sb < k / QKK; sb++) {
        int32_t lane[8] = {0};
        for (int e = 0; e < QKK; e++)
            lane[e & 7] += w[sb].scales[e / 16] * ((q6k_level(&w[sb], e) - 32) * a[sb].qs[e]);
        const float d = orc_f16_to_f32(w[sb].d) * a[sb].d;
        for (int l = 0; l < 8; l++) sums[l] += d * lane[l];
    }
    for (int l = 0; l < 8; l++) sumf += sums[l];
    return sumf;
}

static float dot_iq4_xs_q8_K(const blk_iq4_xs *w, const blk_q8_K *a, int64_t k) {   /* ggml-cpu-quants.c:11381 ff., scalar tail :11647-11676 */
    float sumf = 0;
    for (int64_t sb = 0; sb < k / QKK; sb++) {
        const float d4d8 = orc_f16_to_f32(w[sb].d) * a[sb].d;
        for (int ib = 0; ib < 8; ib++) {
            const float dl = d4d8 * (iq4xs_ls(&w[sb], ib) - 32);
            const uint8_t *qs = w[sb].qs + 16 * ib;
            const int8_t *q8 = a[sb].qs + 32 * ib;
            int sumi1 = 0, sumi2 = 0;
            for (int j = 0; j < 16; j++) {
                sumi1 += q8[j] * iq4nl_values[qs[j] & 0x0F];
                sumi2 += q8[j + 16] * iq4nl_values[qs[j] >> 4];
            }
            sumf += dl * (sumi1 + sumi2);
        }
    }
    return sumf;
}

int orc_mul_mat_cpu(int type, const void *W, const float *x, float *dst, int64_t N, int64_t K, int64_t B) {
    int atype;
    switch (type) {
        case ORC_Q4_0: case ORC_Q5_0: case ORC_IQ4_NL: case ORC_Q8_0: atype = ORC_Q8_0; break;
        case ORC_Q4_1: case ORC_Q5_1: atype = ORC_Q8_1; break;    /* vec_dot_type, ggml-cpu.c:274-296, 384-389 */
        case ORC_Q4_K: case ORC_Q5_K: case ORC_Q6_K: case ORC_IQ4_XS: atype = ORC_Q8_K; break;   /* :390-395 for IQ4_XS */
        default: return -1;
    }
    if (K % orc_block_elems(type)) return -1;
    const size_t wrb = orc_row_bytes(type, K), arb = orc_row_bytes(atype, K);
    void *act = malloc(arb);
    if (!act) return -1;
    for (int64_t b = 0; b < B; b++) {
        quantize_row(atype, x + b * K, act, K);
        for (int64_t n = 0; n < N; n++) {
            const void *row = (const char *)W + n * wrb;
            float r;
            switch (type) {
                case ORC_Q4_0: r = dot_q4_0_q8_0((const blk_q4_0 *)row, (const blk_q8_0 *)act, K); break;
                case ORC_Q4_1: r = dot_q4_1_q8_1((const blk_q4_1 *)row, (const blk_q8_1 *)act, K); break;
                case ORC_Q5_0: r = dot_q5_0_q8_0((const blk_q5_0 *)row, (const blk_q8_0 *)act, K); break;
                case ORC_Q5_1: r = dot_q5_1_q8_1((const blk_q5_1 *)row, (const blk_q8_1 *)act, K); break;
                case ORC_IQ4_NL: r = dot_iq4_nl_q8_0((const blk_iq4_nl *)row, (const blk_q8_0 *)act, K); break;
                case ORC_Q8_0: r = dot_q8_0_q8_0((const blk_q8_0 *)row, (const blk_q8_0 *)act, K); break;
                case ORC_Q4_K: r = dot_q4_K_q8_K((const blk_q4_K *)row, (const blk_q8_K *)act, K); break;
                case ORC_Q5_K: r = dot_q5_K_q8_K((const blk_q5_K *)row, (const blk_q8_K *)act, K); break;
                case ORC_IQ4_XS: r = dot_iq4_xs_q8_K((const blk_iq4_xs *)row, (const blk_q8_K *)act, K); break;
                default:       r = dot_q6_K_q8_K((const blk_q6_K *)row, (const blk_q8_K *)act, K); break;
            }
            dst[b * N + n] = r;
        }
    }
    free(act);
    return 0;
}

/* Device formulation: activations as Q8_1 (quantize_row_q8_1_ref), exact integer granule
 * dots, then the scale algebra of the dequantizers (ggml-quants.c:255-273, 349-363,
 * 1280-1302, 1690-1719) applied in double.  The sum of the activation levels is taken
 * in integers (not from the fp16 `s` field). */
static double row_dot_q8_1(int type, const void *row, const blk_q8_1 *act, int64_t K) {
    double acc = 0;
    for (int64_t b = 0; b < K / QK; b++) {
        const double dx = orc_f16_to_f32(act[b].d);
        int isum = 0, sumq = 0, isum2 = 0;
        for (int j = 0; j < QK; j++) sumq += act[b].qs[j];
        switch (type) {
            case ORC_Q4_0: {
                for (int j = 0; j < QK; j++) isum += weight_level(type, row, b * QK + j) * act[b].qs[j];
                acc += (double)orc_f16_to_f32(((const blk_q4_0 *)row)[b].d) * dx * isum;
            } break;
            case ORC_Q8_0: {
                for (int j = 0; j < QK; j++) isum += weight_level(type, row, b * QK + j) * act[b].qs[j];
                acc += (double)orc_f16_to_f32(((const blk_q8_0 *)row)[b].d) * dx * isum;
            } break;
            case ORC_Q5_0: case ORC_IQ4_NL: {   /* d sits first in both blocks */
                for (int j = 0; j < QK; j++) isum += weight_level(type, row, b * QK + j) * act[b].qs[j];
                const uint16_t dh = type == ORC_Q5_0 ? ((const blk_q5_0 *)row)[b].d : ((const blk_iq4_nl *)row)[b].d;
                acc += (double)orc_f16_to_f32(dh) * dx * isum;
            } break;
            case ORC_IQ4_XS: {
                const blk_iq4_xs *w = (const blk_iq4_xs *)row + b / 8;
                for (int j = 0; j < QK; j++) isum += weight_level(type, row, b * QK + j) * act[b].qs[j];
                acc += (double)orc_f16_to_f32(w->d) * (iq4xs_ls(w, (int)(b % 8)) - 32) * dx * isum;
            } break;
            case ORC_Q4_1: case ORC_Q5_1: {     /* value = d * level + m */
                for (int j = 0; j < QK; j++) isum += weight_level(type, row, b * QK + j) * act[b].qs[j];
                const uint16_t dh = type == ORC_Q4_1 ? ((const blk_q4_1 *)row)[b].d : ((const blk_q5_1 *)row)[b].d;
                const uint16_t mh = type == ORC_Q4_1 ? ((const blk_q4_1 *)row)[b].m : ((const blk_q5_1 *)row)[b].m;
                acc += dx * ((double)orc_f16_to_f32(dh) * isum + (double)orc_f16_to_f32(mh) * sumq);
            } break;
            case ORC_Q4_K: {
                const blk_q4_K *w = (const blk_q4_K *)row + b / 8;
                uint8_t sc, mn;
                q4k_scale_min((int)(b % 8), w->scales, &sc, &mn);
                for (int j = 0; j < QK; j++) isum += weight_level(type, row, b * QK + j) * act[b].qs[j];
                acc += dx * ((double)orc_f16_to_f32(w->d) * sc * isum - (double)orc_f16_to_f32(w->dmin) * mn * sumq);
            } break;
            case ORC_Q5_K: {
                const blk_q5_K *w = (const blk_q5_K *)row + b / 8;
                uint8_t sc, mn;
                q4k_scale_min((int)(b % 8), w->scales, &sc, &mn);
                for (int j = 0; j < QK; j++) isum += weight_level(type, row, b * QK + j) * act[b].qs[j];
                acc += dx * ((double)orc_f16_to_f32(w->d) * sc * isum - (double)orc_f16_to_f32(w->dmin) * mn * sumq);
            } break;
            default: { /* Q6_K: two 16-element groups per activation block */
                const blk_q6_K *w = (const blk_q6_K *)row + b / 8;
                for (int j = 0; j < 16; j++) isum += weight_level(type, row, b * QK + j) * act[b].qs[j];
                for (int j = 16; j < 32; j++) isum2 += weight_level(type, row, b * QK + j) * act[b].qs[j];
                const int g = (int)(b % 8) * 2;
                acc += (double)orc_f16_to_f32(w->d) * dx * ((double)w->scales[g] * isum + (double)w->scales[g + 1] * isum2);
            } break;
        }
    }
    return acc;
}

int orc_mul_mat_q8_1(int type, const void *W, const float *x, float *dst, int64_t N, int64_t K, int64_t B) {
    if (!is_weight_type(type)) return -1;
    if (K % orc_block_elems(type)) return -1;
    const size_t wrb = orc_row_bytes(type, K);
    blk_q8_1 *act = (blk_q8_1 *)malloc(orc_row_bytes(ORC_Q8_1, K));
    if (!act) return -1;
    for (int64_t b = 0; b < B; b++) {
        quant_q8_1(x + b * K, act, K);
        for (int64_t n = 0; n < N; n++) dst[b * N + n] = (float)row_dot_q8_1(type, (const char *)W + n * wrb, act, K);
    }
    free(act);
    return 0;
}

int orc_mul_mat_f64(int type, const void *W, const float *x, float *dst, int64_t N, int64_t K, int64_t B) {
    if (K % MAXI(1, orc_block_elems(type))) return -1;
    const size_t wrb = orc_row_bytes(type, K);
    float *row = (float *)malloc((size_t)K * sizeof(float));
    if (!row) return -1;
    for (int64_t n = 0; n < N; n++) {
        if (dequantize_row(type, (const char *)W + n * wrb, row, K)) { free(row); return -1; }
        for (int64_t b = 0; b < B; b++) {
            double acc = 0;
            for (int64_t i = 0; i < K; i++) acc += (double)row[i] * (double)x[b * K + i];
            dst[b * N + n] = (float)acc;
        }
    }
    free(row);
    return 0;
}

/* ------------------------------------------------------------------ MUL_MAT_ID
 * ggml_mul_mat_id semantics, ggml/src/ggml.c:2723-2759 and
 * ggml_compute_forward_mul_mat_id, ggml/src/ggml-cpu/ggml-cpu.c:7717-7895 */
int orc_mul_mat_id_q8_1(int type, const void *as, const float *b, const int32_t *ids, int64_t ids_stride, float *dst,
                        int64_t N, int64_t K, int64_t n_expert, int64_t n_used, int64_t nb1, int64_t T) {
    if (!is_weight_type(type)) return -1;
    const size_t wrb = orc_row_bytes(type, K);
    blk_q8_1 *act = (blk_q8_1 *)malloc(orc_row_bytes(ORC_Q8_1, K));
    if (!act) return -1;
    for (int64_t t = 0; t < T; t++) {
        for (int64_t e = 0; e < n_used; e++) {
            const int32_t ex = ids[t * ids_stride + e];
            if (ex < 0 || ex >= n_expert) { free(act); return -1; }
            quant_q8_1(b + (t * nb1 + e % nb1) * K, act, K);
            const char *mat = (const char *)as + (size_t)ex * N * wrb;
            for (int64_t n = 0; n < N; n++)
                dst[(t * n_used + e) * N + n] = (float)row_dot_q8_1(type, mat + n * wrb, act, K);
        }
    }
    free(act);
    return 0;
}

/* ------------------------------------------------------------------ FLASH_ATTN_EXT
 * ggml_compute_forward_flash_attn_ext_f16, ggml/src/ggml-cpu/ggml-cpu.c:10916-11129.
 * K is f16 so q is rounded to f16 and the dot is taken over f16 values in float
 * (ggml_vec_dot_f16); V is f16 so the accumulator is kept in f16 (ggml_vec_mad_f16 /
 * ggml_vec_scale_f16 round after every update). */
static float alibi_slope(float max_bias, uint32_t h, uint32_t n_head) {
    if (!(max_bias > 0.0f)) return 1.0f;
    const uint32_t n2 = 1u << (uint32_t)floor(log2(n_head));
    const float m0 = powf(2.0f, -(max_bias) / n2);
    const float m1 = powf(2.0f, -(max_bias / 2.0f) / n2);
    return h < n2 ? powf(m0, h + 1) : powf(m1, 2 * (h - n2) + 1);
}

void orc_flash_attn_cpu(const float *q, const uint16_t *k, const uint16_t *v, const uint16_t *mask, float *dst,
                        int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, float scale, float max_bias,
                        float softcap) {
    if (softcap != 0) scale /= softcap;
    uint16_t *acc16 = (uint16_t *)malloc((size_t)D * 2);
    float *q16 = (float *)malloc((size_t)D * 4);
    const int64_t rep = Hq / Hkv;
    for (int64_t h = 0; h < Hq; h++) {
        const float slope = alibi_slope(max_bias, (uint32_t)h, (uint32_t)Hq);
        const int64_t hk = h / rep;
        for (int64_t i = 0; i < Nq; i++) {
            const float *qr = q + (h * Nq + i) * D;
            for (int64_t d = 0; d < D; d++) q16[d] = orc_f16_to_f32(orc_f32_to_f16(qr[d]));
            memset(acc16, 0, (size_t)D * 2);
            float S = 0.0f, M = -INFINITY;
            for (int64_t c = 0; c < Nkv; c++) {
                const float mv = mask ? slope * orc_f16_to_f32(mask[i * Nkv + c]) : 0.0f;
                if (mv == -INFINITY) continue;
                const uint16_t *kr = k + (hk * Nkv + c) * D;
                double dotacc = 0;    /* the reference sums f16 products in float SIMD lanes; order-free stand-in */
                for (int64_t d = 0; d < D; d++) dotacc += (double)orc_f16_to_f32(kr[d]) * (double)q16[d];
                float s = (float)dotacc * scale;
                if (softcap != 0.0f) s = softcap * tanhf(s);
                s += mv;
                const float Mold = M;
                float ms = 1.0f, vs = 1.0f;
                const uint16_t *vr = v + (hk * Nkv + c) * D;
                if (s > M) {
                    M = s;
                    ms = expf(Mold - M);
                    for (int64_t d = 0; d < D; d++) acc16[d] = orc_f32_to_f16(orc_f16_to_f32(acc16[d]) * ms);
                } else {
                    vs = expf(s - M);
                }
                for (int64_t d = 0; d < D; d++)
                    acc16[d] = orc_f32_to_f16(orc_f16_to_f32(acc16[d]) + orc_f16_to_f32(vr[d]) * vs);
                S = S * ms + vs;
            }
            const float S_inv = 1.0f / S;
            float *o = dst + (i * Hq + h) * D;     /* dst is [D, Hq, Nq]: the permute at :11126-11127 */
            for (int64_t d = 0; d < D; d++) o[d] = orc_f16_to_f32(acc16[d]) * S_inv;
        }
    }
    free(acc16);
    free(q16);
}

/* The same kernel with a quantized KV cache (type_k, type_v each ORC_F16, ORC_Q8_0 or ORC_Q4_0; k, v are [Hkv][Nkv] rows of
 * D elements in the type's block layout).  ggml-cpu.c:10997-11003: q is converted to K's vec_dot_type - f16 for f16 K, Q8_0
 * blocks for Q8_0 and Q4_0 K - and the score is the type's vec_dot (ggml-cpu-quants.c:2492-2506 q4_0 x q8_0, :3919-3927
 * q8_0 x q8_0: per block the integer dot times both scales, summed in float).  :11040-11099: a V of another type than f16 is
 * dequantized row by row (to_float) into f32 and accumulated with ggml_vec_mad_f32 in an f32 accumulator. */
int orc_flash_attn_kv_cpu(const float *q, const void *k, int type_k, const void *v, int type_v, const uint16_t *mask, float *dst,
                          int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, float scale, float max_bias, float softcap) {
    if ((type_k != ORC_F16 && type_k != ORC_Q8_0 && type_k != ORC_Q4_0) || (type_v != ORC_F16 && type_v != ORC_Q8_0 && type_v != ORC_Q4_0)) return -1;
    if (D % QK) return -1;
    if (softcap != 0) scale /= softcap;
    const size_t krb = type_k == ORC_F16 ? (size_t)D * 2 : orc_row_bytes(type_k, D);
    const size_t vrb = type_v == ORC_F16 ? (size_t)D * 2 : orc_row_bytes(type_v, D);
    uint16_t *acc16 = (uint16_t *)malloc((size_t)D * 2);
    float *acc32 = (float *)malloc((size_t)D * 4);
    float *v32 = (float *)malloc((size_t)D * 4);
    float *q16 = (float *)malloc((size_t)D * 4);
    blk_q8_0 *qq = (blk_q8_0 *)malloc((size_t)(D / QK) * sizeof(blk_q8_0));
    const int64_t rep = Hq / Hkv;
    for (int64_t h = 0; h < Hq; h++) {
        const float slope = alibi_slope(max_bias, (uint32_t)h, (uint32_t)Hq);
        const int64_t hk = h / rep;
        for (int64_t i = 0; i < Nq; i++) {
            const float *qr = q + (h * Nq + i) * D;
            if (type_k == ORC_F16) for (int64_t d = 0; d < D; d++) q16[d] = orc_f16_to_f32(orc_f32_to_f16(qr[d]));
            else quantize_row(ORC_Q8_0, qr, qq, D);
            memset(acc16, 0, (size_t)D * 2);
            memset(acc32, 0, (size_t)D * 4);
            float S = 0.0f, M = -INFINITY;
            for (int64_t c = 0; c < Nkv; c++) {
                const float mv = mask ? slope * orc_f16_to_f32(mask[i * Nkv + c]) : 0.0f;
                if (mv == -INFINITY) continue;
                const char *kr = (const char *)k + (size_t)(hk * Nkv + c) * krb;
                double dotacc = 0;    /* the reference sums per-block products in float SIMD lanes; order-free stand-in */
                if (type_k == ORC_F16) {
                    const uint16_t *kh = (const uint16_t *)kr;
                    for (int64_t d = 0; d < D; d++) dotacc += (double)orc_f16_to_f32(kh[d]) * (double)q16[d];
                } else {
                    for (int64_t b = 0; b < D / QK; b++) {
                        int sumi = 0;
                        float dk;
                        if (type_k == ORC_Q8_0) {
                            const blk_q8_0 *kb = (const blk_q8_0 *)kr + b;
                            for (int j = 0; j < QK; j++) sumi += (int)kb->qs[j] * (int)qq[b].qs[j];
                            dk = orc_f16_to_f32(kb->d);
                        } else {
                            const blk_q4_0 *kb = (const blk_q4_0 *)kr + b;
                            for (int j = 0; j < QK / 2; j++) {
                                sumi += ((int)(kb->qs[j] & 0x0F) - 8) * (int)qq[b].qs[j];
                                sumi += ((int)(kb->qs[j] >> 4) - 8) * (int)qq[b].qs[j + QK / 2];
                            }
                            dk = orc_f16_to_f32(kb->d);
                        }
                        dotacc += (double)((float)sumi * (dk * orc_f16_to_f32(qq[b].d)));
                    }
                }
                float s = (float)dotacc * scale;
                if (softcap != 0.0f) s = softcap * tanhf(s);
                s += mv;
                const float Mold = M;
                float ms = 1.0f, vs = 1.0f;
                const char *vr = (const char *)v + (size_t)(hk * Nkv + c) * vrb;
                if (s > M) {
                    M = s;
                    ms = expf(Mold - M);
                    if (type_v == ORC_F16) for (int64_t d = 0; d < D; d++) acc16[d] = orc_f32_to_f16(orc_f16_to_f32(acc16[d]) * ms);
                    else for (int64_t d = 0; d < D; d++) acc32[d] *= ms;
                } else {
                    vs = expf(s - M);
                }
                if (type_v == ORC_F16) {
                    const uint16_t *vh = (const uint16_t *)vr;
                    for (int64_t d = 0; d < D; d++) acc16[d] = orc_f32_to_f16(orc_f16_to_f32(acc16[d]) + orc_f16_to_f32(vh[d]) * vs);
                } else {
                    dequantize_row(type_v, vr, v32, D);
                    for (int64_t d = 0; d < D; d++) acc32[d] = fmaf(v32[d], vs, acc32[d]);
                }
                S = S * ms + vs;
            }
            const float S_inv = 1.0f / S;
            float *o = dst + (i * Hq + h) * D;
            for (int64_t d = 0; d < D; d++) o[d] = (type_v == ORC_F16 ? orc_f16_to_f32(acc16[d]) : acc32[d]) * S_inv;
        }
    }
    free(acc16); free(acc32); free(v32); free(q16); free(qq);
    return 0;
}

void orc_flash_attn_f64(const float *q, const uint16_t *k, const uint16_t *v, const uint16_t *mask, float *dst,
                        int64_t D, int64_t Nq, int64_t Nkv, int64_t Hq, int64_t Hkv, float scale, float max_bias,
                        float softcap) {
    double *p = (double *)malloc((size_t)Nkv * sizeof(double));
    const int64_t rep = Hq / Hkv;
    const double sc = softcap != 0 ? (double)scale / softcap : scale;
    for (int64_t h = 0; h < Hq; h++) {
        const double slope = alibi_slope(max_bias, (uint32_t)h, (uint32_t)Hq);
        const int64_t hk = h / rep;
        for (int64_t i = 0; i < Nq; i++) {
            const float *qr = q + (h * Nq + i) * D;
            double mx = -INFINITY;
            for (int64_t c = 0; c < Nkv; c++) {
                const uint16_t *kr = k + (hk * Nkv + c) * D;
                double s = 0;
                for (int64_t d = 0; d < D; d++) s += (double)qr[d] * (double)orc_f16_to_f32(kr[d]);
                s *= sc;
                if (softcap != 0) s = softcap * tanh(s);
                if (mask) s += slope * (double)orc_f16_to_f32(mask[i * Nkv + c]);
                p[c] = s;
                if (s > mx) mx = s;
            }
            double den = 0;
            for (int64_t c = 0; c < Nkv; c++) {
                p[c] = (p[c] == -INFINITY) ? 0.0 : exp(p[c] - mx);
                den += p[c];
            }
            float *o = dst + (i * Hq + h) * D;
            for (int64_t d = 0; d < D; d++) {
                double acc = 0;
                for (int64_t c = 0; c < Nkv; c++) acc += p[c] * (double)orc_f16_to_f32(v[(hk * Nkv + c) * D + d]);
                o[d] = (float)(acc / den);
            }
        }
    }
    free(p);
}

/* ------------------------------------------------------------------ glue ops
 * ggml_compute_forward_rms_norm_f32, ggml/src/ggml-cpu/ggml-cpu.c:7015-7061 */
void orc_rms_norm(const float *x, float *y, int64_t ncols, int64_t nrows, float eps) {
    for (int64_t r = 0; r < nrows; r++) {
        double sum = 0.0;
        for (int64_t i = 0; i < ncols; i++) sum += (double)(x[r * ncols + i] * x[r * ncols + i]);
        const float mean = (float)(sum / ncols);
        const float scale = 1.0f / sqrtf(mean + eps);
        for (int64_t i = 0; i < ncols; i++) y[r * ncols + i] = x[r * ncols + i] * scale;
    }
}

/* ggml_silu_f32, ggml/src/ggml-cpu/ggml-cpu.c:1814 */
void orc_silu(const float *x, float *y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = x[i] / (1.0f + expf(-x[i]));
}

/* ggml_compute_forward_soft_max_f32, ggml/src/ggml-cpu/ggml-cpu.c:8959-9055 (max_bias 0) */
void orc_soft_max(const float *x, const float *mask, float *y, int64_t ncols, int64_t nrows, float scale) {
    for (int64_t r = 0; r < nrows; r++) {
        float mx = -INFINITY;
        for (int64_t i = 0; i < ncols; i++) {
            const float v = x[r * ncols + i] * scale + (mask ? mask[r * ncols + i] : 0.0f);
            y[r * ncols + i] = v;
            if (v > mx) mx = v;
        }
        double sum = 0.0;
        for (int64_t i = 0; i < ncols; i++) {
            const float e = expf(y[r * ncols + i] - mx);
            y[r * ncols + i] = e;
            sum += (double)e;
        }
        const float inv = (float)(1.0 / sum);
        for (int64_t i = 0; i < ncols; i++) y[r * ncols + i] *= inv;
    }
}

/* ggml_compute_forward_rope_f32 + ggml_rope_cache_init + rope_yarn,
 * ggml/src/ggml-cpu/ggml-cpu.c:9366-9549, 9292-9306, 9275-9290;
 * ggml_rope_yarn_corr_dims, ggml/src/ggml.c:3695-3707.  x is [ne0, n_heads, n_tokens]. */
void orc_rope(const float *x, const int32_t *pos, const float *freq_factors, float *y, int64_t ne0, int64_t n_heads,
              int64_t n_tokens, int n_dims, int mode, float freq_base, float freq_scale, float ext_factor,
              float attn_factor, float beta_fast, float beta_slow, int n_ctx_orig) {
    const float theta_scale = powf(freq_base, -2.0f / n_dims);
    const float pi = 3.14159265358979323846f;
    float c0 = floorf(n_dims * logf(n_ctx_orig / (beta_fast * 2 * pi)) / (2 * logf(freq_base)));
    float c1 = ceilf(n_dims * logf(n_ctx_orig / (beta_slow * 2 * pi)) / (2 * logf(freq_base)));
    const float lo = c0 > 0 ? c0 : 0, hi = c1 < n_dims - 1 ? c1 : (float)(n_dims - 1);
    float *cs = (float *)malloc((size_t)ne0 * sizeof(float));
    for (int64_t t = 0; t < n_tokens; t++) {
        float theta = (float)pos[t];
        for (int64_t i0 = 0; i0 < ne0; i0 += 2) {
            const float ff = freq_factors ? freq_factors[i0 / 2] : 1.0f;
            const float extrap = theta / ff;
            const float interp = freq_scale * extrap;
            float th = interp, ms = attn_factor;
            if (ext_factor != 0.0f) {
                const float yv = (i0 / 2 - lo) / (0.001f > hi - lo ? 0.001f : hi - lo);
                const float ramp = (1 - (yv < 0 ? 0 : (yv > 1 ? 1 : yv))) * ext_factor;
                th = interp * (1 - ramp) + extrap * ramp;
                ms *= 1.0f + 0.1f * logf(1.0f / freq_scale);
            }
            cs[i0] = cosf(th) * ms;
            cs[i0 + 1] = sinf(th) * ms;
            theta *= theta_scale;
        }
        for (int64_t h = 0; h < n_heads; h++) {
            const float *src = x + (t * n_heads + h) * ne0;
            float *dst = y + (t * n_heads + h) * ne0;
            for (int64_t i0 = 0; i0 < n_dims; i0 += 2) {
                const float c = cs[i0], s = cs[i0 + 1];
                const int64_t a = (mode & 2) ? i0 / 2 : i0;
                const int64_t b = (mode & 2) ? i0 / 2 + n_dims / 2 : i0 + 1;
                const float x0 = src[a], x1 = src[b];
                dst[a] = x0 * c - x1 * s;
                dst[b] = x0 * s + x1 * c;
            }
            for (int64_t i0 = n_dims; i0 < ne0; i0++) dst[i0] = src[i0];
        }
    }
    free(cs);
}

/* ggml_compute_forward_argsort_f32, ggml/src/ggml-cpu/ggml-cpu.c:10857: a stable-free
 * exchange sort; ties keep the order this loop produces. */
void orc_argsort(const float *x, int32_t *idx, int64_t ncols, int64_t nrows, int descending) {
    for (int64_t r = 0; r < nrows; r++) {
        int32_t *d = idx + r * ncols;
        const float *s = x + r * ncols;
        for (int64_t j = 0; j < ncols; j++) d[j] = (int32_t)j;
        for (int64_t j = 0; j < ncols; j++)
            for (int64_t kk = j + 1; kk < ncols; kk++)
                if ((!descending && s[d[j]] > s[d[kk]]) || (descending && s[d[j]] < s[d[kk]])) {
                    int32_t t = d[j]; d[j] = d[kk]; d[kk] = t;
                }
    }
}
