/*
 * qoracle.c - CPU oracle for the GGML block-quantized linear path (see qoracle.h).
 *
 * TEST INFRASTRUCTURE ONLY: checker and reported CPU baseline, never the product path.
 *
 * Parity status (what pins each function; tests/test_oracle_*.py hold the checks):
 *   qo_fp16_to_fp32        pinned: exhaustive 65536-input golden from the compiled reference
 *                          + IEEE closed form (numpy float16).
 *   qo_dequantize_row_*    pinned: golden blocks decoded by the compiled reference (random
 *                          bytes, random finite/subnormal/inf/nan fp16 scales, bit-exact),
 *                          + an independent element-indexed double-precision formula rounded
 *                          once to fp32, + one-hot/hand-built blocks.
 *   qo_k4_*_scales         pinned: pack/unpack round trip over all 6-bit values + goldens.
 *   codebooks              pinned: SHA-256 of the memory image; sign table by closed form.
 *   qo_gemv_f64/_f32       pinned: all-ones x == row sums of the decoded row, one-hot x ==
 *                          single decoded element, numpy float64 matmul on decoded rows,
 *                          and the compiled reference's tf_qmatvec on the same inputs.
 *   qo_gemm_tokmajor_*     pinned: equals per-token gemv (brute force) and numpy matmul.
 *   qo_moe_route           pinned: weights sum to 1, index set == argsort top-k, weights ==
 *                          softmax over the selected logits; and ids (in order) and weights against the
 *                          fixture of the MoE block below, whose selection ran on the compiled reference's
 *                          tf_softmax (the heap itself is inline in the reference's forward pass and is
 *                          restated beside that fixture's generator, independently of this file).
 *   qo_moe_ffn_token_*     pinned: numpy float64 restatement on decoded expert slices, and the fixture
 *                          of one token's whole block composed from the compiled reference's tf_softmax,
 *                          tf_qmatvec_expert (x3) and tf_silu_mul_avx2 (tests/golden/make_golden.py), to
 *                          5e-6: that SiLU uses a polynomial exp, this file expf.
 */
#include "qoracle.h"
#include "qoracle_tables.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ helpers */

static inline uint16_t rd_u16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static inline uint32_t rd_u32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

/* IEEE binary16 -> binary32, exact for every input (follows common/ggml_dequant.h:206-229:
 * zero keeps its sign, subnormals are normalised, Inf/NaN keep their payload shifted left 13). */
float qo_fp16_to_fp32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h >> 15) << 31;
    const uint32_t e = (h >> 10) & 31u;
    const uint32_t m = h & 1023u;
    uint32_t bits;
    if (e == 31u) {
        bits = sign | 0x7F800000u | (m << 13);
    } else if (e != 0u) {
        bits = sign | ((e + 112u) << 23) | (m << 13);
    } else {
        /* value = m * 2^-24: an integer below 2^10 times a power of two is exact in fp32 */
        float mag = (float)m * 0x1p-24f;
        memcpy(&bits, &mag, 4);
        bits |= sign;
    }
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

/* all 65536 inputs at once (returning a float through a foreign-function interface would
 * quiet signalling NaNs on the way; writing to memory keeps every bit) */
void qo_fp16_table(float *out) {
    for (uint32_t h = 0; h < 65536u; h++) out[h] = qo_fp16_to_fp32((uint16_t)h);
}

typedef struct { uint32_t type; int elems; int bytes; } qo_type_info;
static const qo_type_info k_types[] = {
    {QO_TYPE_F32, 1, 4},       {QO_TYPE_F16, 1, 2},      {QO_TYPE_BF16, 1, 2},
    {QO_TYPE_Q8_0, 32, 34},    {QO_TYPE_Q4_K, 256, 144}, {QO_TYPE_Q5_K, 256, 176},
    {QO_TYPE_Q6_K, 256, 210},  {QO_TYPE_IQ2_XXS, 256, 66}, {QO_TYPE_IQ4_NL, 32, 18},
    {QO_TYPE_IQ3_S, 256, 110},
    {QO_TYPE_Q4_0, 32, 18},    {QO_TYPE_Q4_1, 32, 20},   {QO_TYPE_Q5_0, 32, 22},
    {QO_TYPE_Q5_1, 32, 24},    {QO_TYPE_Q2_K, 256, 84},  {QO_TYPE_Q3_K, 256, 110},
    {QO_TYPE_IQ2_XS, 256, 74}, {QO_TYPE_IQ3_XXS, 256, 98}, {QO_TYPE_IQ1_S, 256, 50},
    {QO_TYPE_IQ2_S, 256, 82},  {QO_TYPE_IQ4_XS, 256, 136}, {QO_TYPE_IQ1_M, 256, 56},
    {QO_TYPE_TQ1_0, 256, 54},  {QO_TYPE_TQ2_0, 256, 66}, {QO_TYPE_MXFP4, 32, 17},
    {QO_TYPE_NVFP4, 64, 36},   {QO_TYPE_Q1_0, 128, 18},
};
static const qo_type_info *find_type(uint32_t type) {
    for (size_t i = 0; i < sizeof(k_types) / sizeof(k_types[0]); i++)
        if (k_types[i].type == type) return &k_types[i];
    return NULL;
}
int qo_block_elems(uint32_t type) { const qo_type_info *t = find_type(type); return t ? t->elems : 0; }
int qo_block_bytes(uint32_t type) { const qo_type_info *t = find_type(type); return t ? t->bytes : 0; }

/* ceil(n / block) * block_bytes, 0 if unknown (common/ggml_dequant.h:261-294) */
size_t qo_row_size(uint32_t type, int n) {
    const qo_type_info *t = find_type(type);
    if (!t) return 0;
    return (size_t)((n + t->elems - 1) / t->elems) * (size_t)t->bytes;
}

/* sign table of the 2-bit/3-bit i-quants: entry i (7 bits) gets bit 7 = parity of i, so that
 * every byte has an even number of set bits (data at common/ggml_dequant.h:1765-1774). */
static inline uint8_t iq_sign_byte(uint32_t i7) {
    uint32_t p = i7 ^ (i7 >> 4);
    p ^= p >> 2;
    p ^= p >> 1;
    return (uint8_t)(i7 | ((p & 1u) << 7));
}

static uint8_t g_sign_table[128];
const void *qo_table(const char *name, size_t *bytes) {
    if (!strcmp(name, "iq2xxs_grid")) { *bytes = sizeof(qo_iq2xxs_grid); return qo_iq2xxs_grid; }
    if (!strcmp(name, "iq3s_grid")) { *bytes = sizeof(qo_iq3s_grid); return qo_iq3s_grid; }
    if (!strcmp(name, "iq4nl_values")) { *bytes = sizeof(qo_iq4nl_values); return qo_iq4nl_values; }
    if (!strcmp(name, "ksigns")) {
        for (uint32_t i = 0; i < 128; i++) g_sign_table[i] = iq_sign_byte(i);
        *bytes = 128;
        return g_sign_table;
    }
    return qo_table_ext(name, bytes);
}

/* ------------------------------------------------------------------ decoders
 * Every decoder drops a ragged tail: it decodes n / block_elems whole blocks, like the
 * reference's integer division. */

/* Q8_0: [d f16][32 x int8]; y = d * q (common/ggml_dequant.h:1479-1489) */
void qo_dequantize_row_q8_0(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 32; b++, p += 34, dst += 32) {
        const float d = qo_fp16_to_fp32(rd_u16(p));
        const int8_t *q = (const int8_t *)(p + 2);
        for (int k = 0; k < 32; k++) dst[k] = d * (float)q[k];
    }
}

/* 6-bit scale/min unpack shared by Q4_K and Q5_K (get_scale_min_k4,
 * common/ggml_dequant.h:1582-1590): fields 0..3 sit in the low 6 bits of bytes 0..3 (scales)
 * and 4..7 (mins); fields 4..7 take their low 4 bits from bytes 8..11 and their high 2 bits
 * from the top of bytes 0..3 (scales) / 4..7 (mins). */
void qo_k4_unpack_scales(const uint8_t s[12], uint8_t sc[8], uint8_t mn[8]) {
    for (int j = 0; j < 4; j++) {
        sc[j] = s[j] & 63;
        mn[j] = s[j + 4] & 63;
        sc[j + 4] = (uint8_t)((s[j + 8] & 15) | ((s[j] >> 6) << 4));
        mn[j + 4] = (uint8_t)((s[j + 8] >> 4) | ((s[j + 4] >> 6) << 4));
    }
}
void qo_k4_pack_scales(const uint8_t sc[8], const uint8_t mn[8], uint8_t s[12]) {
    for (int j = 0; j < 4; j++) {
        s[j] = (uint8_t)((sc[j] & 63) | ((sc[j + 4] >> 4) << 6));
        s[j + 4] = (uint8_t)((mn[j] & 63) | ((mn[j + 4] >> 4) << 6));
        s[j + 8] = (uint8_t)((sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4));
    }
}

/* Q4_K: [d][dmin][12 scale bytes][128 nibble bytes]; sub-block g (32 elements) uses the low
 * nibbles of qs[32*(g/2) ..] when g is even, the high nibbles when odd;
 * y = (d*sc_g)*q - (dmin*m_g)  (common/ggml_dequant.h:1592-1618) */
void qo_dequantize_row_q4_K(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 144, dst += 256) {
        const float d = qo_fp16_to_fp32(rd_u16(p));
        const float dmin = qo_fp16_to_fp32(rd_u16(p + 2));
        uint8_t sc[8], mn[8];
        qo_k4_unpack_scales(p + 4, sc, mn);
        const uint8_t *qs = p + 16;
        for (int g = 0; g < 8; g++) {
            const float dl = d * (float)sc[g];
            const float ml = dmin * (float)mn[g];
            const uint8_t *q = qs + 32 * (g >> 1);
            const int sh = (g & 1) * 4;
            for (int l = 0; l < 32; l++) dst[32 * g + l] = dl * (float)((q[l] >> sh) & 15) - ml;
        }
    }
}

/* Q5_K: as Q4_K plus a fifth bit: bit g of qh[l] adds 16 to element l of sub-block g
 * (common/ggml_dequant.h:1620-1651) */
void qo_dequantize_row_q5_K(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 176, dst += 256) {
        const float d = qo_fp16_to_fp32(rd_u16(p));
        const float dmin = qo_fp16_to_fp32(rd_u16(p + 2));
        uint8_t sc[8], mn[8];
        qo_k4_unpack_scales(p + 4, sc, mn);
        const uint8_t *qh = p + 16;
        const uint8_t *qs = p + 48;
        for (int g = 0; g < 8; g++) {
            const float dl = d * (float)sc[g];
            const float ml = dmin * (float)mn[g];
            const uint8_t *q = qs + 32 * (g >> 1);
            const int sh = (g & 1) * 4;
            for (int l = 0; l < 32; l++) {
                const int v = ((q[l] >> sh) & 15) + (((qh[l] >> g) & 1) << 4);
                dst[32 * g + l] = dl * (float)v - ml;
            }
        }
    }
}

/* Q6_K: [ql 128][qh 64][16 x int8 scales][d]. Two halves of 128 elements; inside a half,
 * segment s (32 elements) reads ql[64*half + 32*(s&1) + l], low nibble for s<2 else high, and
 * bits 2s..2s+1 of qh[32*half + l]; scale index 8*half + 2*s + l/16;
 * y = (d*sc)*(q-32)  (common/ggml_dequant.h:1653-1687) */
void qo_dequantize_row_q6_K(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 210, dst += 256) {
        const uint8_t *ql = p, *qh = p + 128;
        const int8_t *sc = (const int8_t *)(p + 192);
        const float d = qo_fp16_to_fp32(rd_u16(p + 208));
        for (int half = 0; half < 2; half++) {
            for (int s = 0; s < 4; s++) {
                for (int l = 0; l < 32; l++) {
                    const uint8_t lo = ql[64 * half + 32 * (s & 1) + l];
                    const int nib = (s < 2) ? (lo & 15) : (lo >> 4);
                    const int hi2 = (qh[32 * half + l] >> (2 * s)) & 3;
                    const int q = (nib | (hi2 << 4)) - 32;
                    const float scale = d * (float)sc[8 * half + 2 * s + (l >> 4)];
                    dst[128 * half + 32 * s + l] = scale * (float)q;
                }
            }
        }
    }
}

/* IQ2_XXS: [d][8 groups of 8 bytes]. Group: u32 a0 = four grid indices (one byte each),
 * u32 a1 = four 7-bit sign indices + 4-bit scale in the top nibble.
 * db = (d*(0.5+scale))*0.25; y = (db*grid_byte)*(+-1)  (common/ggml_dequant.h:2793-2816) */
void qo_dequantize_row_iq2_xxs(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 66, dst += 256) {
        const float d = qo_fp16_to_fp32(rd_u16(p));
        for (int g = 0; g < 8; g++) {
            const uint32_t a0 = rd_u32(p + 2 + 8 * g);
            const uint32_t a1 = rd_u32(p + 6 + 8 * g);
            const float db = d * (0.5f + (float)(a1 >> 28)) * 0.25f;
            for (int l = 0; l < 4; l++) {
                const uint64_t cell = qo_iq2xxs_grid[(a0 >> (8 * l)) & 255u];
                const uint8_t sg = iq_sign_byte((a1 >> (7 * l)) & 127u);
                for (int j = 0; j < 8; j++) {
                    const float mag = db * (float)((cell >> (8 * j)) & 255u);
                    dst[32 * g + 8 * l + j] = mag * (((sg >> j) & 1) ? -1.0f : 1.0f);
                }
            }
        }
    }
}

/* IQ4_NL: [d][16 nibble bytes]; element j<16 = low nibble of qs[j], j>=16 = high nibble of
 * qs[j-16]; y = d * codebook[nibble]  (common/ggml_dequant.h:2942-2954) */
void qo_dequantize_row_iq4_nl(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 32; b++, p += 18, dst += 32) {
        const float d = qo_fp16_to_fp32(rd_u16(p));
        for (int j = 0; j < 16; j++) {
            dst[j] = d * (float)qo_iq4nl_values[p[2 + j] & 15];
            dst[j + 16] = d * (float)qo_iq4nl_values[p[2 + j] >> 4];
        }
    }
}

/* IQ3_S: [d][qs 64][qh 8][signs 32][scales 4]. Group g of 32 elements: scale nibble g of the
 * scale bytes, db = d*(1+2*nib). Eight elements at a time (l=0..3): two 9-bit grid indices
 * qs[8g+2l], qs[8g+2l+1] whose ninth bits are bits 2l and 2l+1 of qh[g]; each grid entry holds
 * four magnitudes; sign bits from signs[4g+l].  (common/ggml_dequant.h:3022-3058) */
void qo_dequantize_row_iq3_s(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 110, dst += 256) {
        const float d = qo_fp16_to_fp32(rd_u16(p));
        const uint8_t *qs = p + 2, *qh = p + 66, *sg = p + 74, *scales = p + 106;
        for (int g = 0; g < 8; g++) {
            const int nib = (scales[g >> 1] >> (4 * (g & 1))) & 15;
            const float db = d * (float)(1 + 2 * nib);
            for (int l = 0; l < 4; l++) {
                const uint32_t i0 = qs[8 * g + 2 * l] | (((uint32_t)(qh[g] >> (2 * l)) & 1u) << 8);
                const uint32_t i1 = qs[8 * g + 2 * l + 1] | (((uint32_t)(qh[g] >> (2 * l + 1)) & 1u) << 8);
                const uint32_t c0 = qo_iq3s_grid[i0], c1 = qo_iq3s_grid[i1];
                const uint8_t sb = sg[4 * g + l];
                for (int j = 0; j < 4; j++) {
                    const float m0 = db * (float)((c0 >> (8 * j)) & 255u);
                    const float m1 = db * (float)((c1 >> (8 * j)) & 255u);
                    dst[32 * g + 8 * l + j] = m0 * (((sb >> j) & 1) ? -1.0f : 1.0f);
                    dst[32 * g + 8 * l + 4 + j] = m1 * (((sb >> (j + 4)) & 1) ? -1.0f : 1.0f);
                }
            }
        }
    }
}

/* type switch (common/ggml_dequant.h:3177-3265); F32 copy, F16 convert, BF16 shift */
int qo_dequant_row(uint32_t type, const void *src, float *dst, int n) {
    switch (type) {
    case QO_TYPE_Q8_0: qo_dequantize_row_q8_0(src, dst, n); return 0;
    case QO_TYPE_Q4_K: qo_dequantize_row_q4_K(src, dst, n); return 0;
    case QO_TYPE_Q5_K: qo_dequantize_row_q5_K(src, dst, n); return 0;
    case QO_TYPE_Q6_K: qo_dequantize_row_q6_K(src, dst, n); return 0;
    case QO_TYPE_IQ2_XXS: qo_dequantize_row_iq2_xxs(src, dst, n); return 0;
    case QO_TYPE_IQ4_NL: qo_dequantize_row_iq4_nl(src, dst, n); return 0;
    case QO_TYPE_IQ3_S: qo_dequantize_row_iq3_s(src, dst, n); return 0;
    case QO_TYPE_Q4_0: qo_dequantize_row_q4_0(src, dst, n); return 0;
    case QO_TYPE_Q4_1: qo_dequantize_row_q4_1(src, dst, n); return 0;
    case QO_TYPE_Q5_0: qo_dequantize_row_q5_0(src, dst, n); return 0;
    case QO_TYPE_Q5_1: qo_dequantize_row_q5_1(src, dst, n); return 0;
    case QO_TYPE_Q2_K: qo_dequantize_row_q2_K(src, dst, n); return 0;
    case QO_TYPE_Q3_K: qo_dequantize_row_q3_K(src, dst, n); return 0;
    case QO_TYPE_Q1_0: qo_dequantize_row_q1_0(src, dst, n); return 0;
    case QO_TYPE_MXFP4: qo_dequantize_row_mxfp4(src, dst, n); return 0;
    case QO_TYPE_NVFP4: qo_dequantize_row_nvfp4(src, dst, n); return 0;
    case QO_TYPE_IQ3_XXS: qo_dequantize_row_iq3_xxs(src, dst, n); return 0;
    case QO_TYPE_IQ4_XS: qo_dequantize_row_iq4_xs(src, dst, n); return 0;
    case QO_TYPE_IQ2_XS: qo_dequantize_row_iq2_xs(src, dst, n); return 0;
    case QO_TYPE_IQ2_S: qo_dequantize_row_iq2_s(src, dst, n); return 0;
    case QO_TYPE_IQ1_S: qo_dequantize_row_iq1_s(src, dst, n); return 0;
    case QO_TYPE_IQ1_M: qo_dequantize_row_iq1_m(src, dst, n); return 0;
    case QO_TYPE_TQ1_0: qo_dequantize_row_tq1_0(src, dst, n); return 0;
    case QO_TYPE_TQ2_0: qo_dequantize_row_tq2_0(src, dst, n); return 0;
    case QO_TYPE_F32: memcpy(dst, src, (size_t)n * 4); return 0;
    case QO_TYPE_F16: {
        const uint8_t *p = (const uint8_t *)src;
        for (int i = 0; i < n; i++) dst[i] = qo_fp16_to_fp32(rd_u16(p + 2 * i));
        return 0;
    }
    case QO_TYPE_BF16: {
        const uint8_t *p = (const uint8_t *)src;
        for (int i = 0; i < n; i++) {
            uint32_t bits = (uint32_t)rd_u16(p + 2 * i) << 16;
            memcpy(&dst[i], &bits, 4);
        }
        return 0;
    }
    default: return -1;
    }
}

/* ------------------------------------------------------------------ dots */

typedef float v8f __attribute__((vector_size(32)));
static inline v8f ld8(const float *p) { v8f v; memcpy(&v, p, 32); return v; }
static inline float hsum8(v8f v) {
    /* (lanes 0-3 + lanes 4-7), then pairs, then the last two: the usual 256->128->64->32 tree */
    float a = v[0] + v[4], b = v[1] + v[5], c = v[2] + v[6], d = v[3] + v[7];
    return (a + c) + (b + d);
}

/* fp32 dot of a decoded row with x: four independent 8-lane FMA accumulators over 32-element
 * strides, an 8-lane tail, then a scalar tail (shape of common/transformer.h:1086-1113) */
static float dot_f32(const float *w, const float *x, int n) {
    v8f a0 = {0}, a1 = {0}, a2 = {0}, a3 = {0};
    int j = 0;
    for (; j + 31 < n; j += 32) {
        a0 += ld8(w + j) * ld8(x + j);
        a1 += ld8(w + j + 8) * ld8(x + j + 8);
        a2 += ld8(w + j + 16) * ld8(x + j + 16);
        a3 += ld8(w + j + 24) * ld8(x + j + 24);
    }
    for (; j + 7 < n; j += 8) a0 += ld8(w + j) * ld8(x + j);
    float sum = hsum8((a0 + a1) + (a2 + a3));
    for (; j < n; j++) sum += w[j] * x[j];
    return sum;
}

/* Q8_0 fused dequant-dot: per block, each group of eight int8 is converted, scaled by d and
 * FMA'd with x into two alternating accumulators (shape of common/ggml_dequant.h:953-998) */
static float dot_q8_0_f32(const uint8_t *row, const float *x, int n) {
    v8f a0 = {0}, a1 = {0};
    for (int b = 0; b < n / 32; b++, row += 34, x += 32) {
        const float d = qo_fp16_to_fp32(rd_u16(row));
        const int8_t *q = (const int8_t *)(row + 2);
        for (int g = 0; g < 4; g++) {
            v8f f;
            for (int k = 0; k < 8; k++) f[k] = (float)q[8 * g + k] * d;
            if (g & 1) a1 += f * ld8(x + 8 * g);
            else a0 += f * ld8(x + 8 * g);
        }
    }
    return hsum8(a0 + a1);
}

static double dot_f64(const float *w, const float *x, int n) {
    double s = 0.0;
    for (int j = 0; j < n; j++) s += (double)w[j] * (double)x[j];
    return s;
}

int qo_gemv_f64(uint32_t type, const void *W, const float *x, float *y, int n_rows, int n_cols) {
    const size_t rb = qo_row_size(type, n_cols);
    if (!rb) return -1;
    float *tmp = (float *)calloc((size_t)n_cols, sizeof(float));
    if (!tmp) return -2;
    for (int r = 0; r < n_rows; r++) {
        qo_dequant_row(type, (const uint8_t *)W + (size_t)r * rb, tmp, n_cols);
        y[r] = (float)dot_f64(tmp, x, n_cols);
    }
    free(tmp);
    return 0;
}

typedef struct {
    uint32_t type;
    const uint8_t *W;
    const float *x;
    float *y;
    int n_cols, row_lo, row_hi, iters;
    size_t rb;
    float *tmp;
    pthread_barrier_t *bar;
} gemv_task;

static void gemv_rows_f32(const gemv_task *t) {
    if (t->type == QO_TYPE_Q8_0) {
        for (int r = t->row_lo; r < t->row_hi; r++)
            t->y[r] = dot_q8_0_f32(t->W + (size_t)r * t->rb, t->x, t->n_cols);
        return;
    }
    for (int r = t->row_lo; r < t->row_hi; r++) {
        qo_dequant_row(t->type, t->W + (size_t)r * t->rb, t->tmp, t->n_cols);
        t->y[r] = dot_f32(t->tmp, t->x, t->n_cols);
    }
}

static void *gemv_thread(void *arg) {
    gemv_task *t = (gemv_task *)arg;
    for (int it = 0; it < t->iters; it++) {
        if (t->bar) pthread_barrier_wait(t->bar); /* stands in for the pool wake-up */
        gemv_rows_f32(t);
        if (t->bar) pthread_barrier_wait(t->bar); /* ... and the completion wait */
    }
    return NULL;
}

/* rows_per = n_rows / nt, the first n_rows % nt threads take one more
 * (common/transformer.h:1124-1131); serial when n_rows < 4*nt (:1119) */
static int run_gemv_f32(uint32_t type, const void *W, const float *x, float *y, int n_rows,
                        int n_cols, int nt, int iters) {
    const size_t rb = qo_row_size(type, n_cols);
    if (!rb) return -1;
    if (nt < 1) nt = 1;
    if (n_rows < 4 * nt) nt = 1;
    gemv_task *tasks = (gemv_task *)calloc((size_t)nt, sizeof(gemv_task));
    pthread_t *th = (pthread_t *)calloc((size_t)nt, sizeof(pthread_t));
    pthread_barrier_t bar;
    if (nt > 1) pthread_barrier_init(&bar, NULL, (unsigned)nt);
    const int per = n_rows / nt, extra = n_rows % nt;
    int lo = 0;
    for (int t = 0; t < nt; t++) {
        const int cnt = per + (t < extra ? 1 : 0);
        tasks[t] = (gemv_task){type, (const uint8_t *)W, x, y, n_cols, lo, lo + cnt, iters, rb,
                               (float *)calloc((size_t)n_cols, sizeof(float)),
                               nt > 1 ? &bar : NULL};
        lo += cnt;
    }
    for (int t = 1; t < nt; t++) pthread_create(&th[t], NULL, gemv_thread, &tasks[t]);
    gemv_thread(&tasks[0]); /* the calling thread runs partition 0 */
    for (int t = 1; t < nt; t++) pthread_join(th[t], NULL);
    for (int t = 0; t < nt; t++) free(tasks[t].tmp);
    if (nt > 1) pthread_barrier_destroy(&bar);
    free(tasks);
    free(th);
    return 0;
}

int qo_gemv_f32(uint32_t type, const void *W, const float *x, float *y, int n_rows, int n_cols,
                int n_threads) {
    return run_gemv_f32(type, W, x, y, n_rows, n_cols, n_threads, 1);
}

#include <time.h>
static double now_s(void) {
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

double qo_gemv_f32_time(uint32_t type, const void *W, const float *x, float *y, int n_rows,
                        int n_cols, int n_threads, int iters) {
    if (iters < 1) iters = 1;
    if (run_gemv_f32(type, W, x, y, n_rows, n_cols, n_threads, 1) != 0) return -1.0; /* warm */
    const double t0 = now_s();
    run_gemv_f32(type, W, x, y, n_rows, n_cols, n_threads, iters);
    return (now_s() - t0) / (double)iters;
}

/* ------------------------------------------------------------------ prefill GEMM */

int qo_gemm_tokmajor_f64(uint32_t type, const void *W, const float *X, float *Y, int n_rows,
                         int n_cols, int n_tok, int out_stride, int x_stride) {
    const size_t rb = qo_row_size(type, n_cols);
    if (!rb) return -1;
    float *tmp = (float *)calloc((size_t)n_cols, sizeof(float));
    if (!tmp) return -2;
    for (int r = 0; r < n_rows; r++) {
        qo_dequant_row(type, (const uint8_t *)W + (size_t)r * rb, tmp, n_cols);
        for (int t = 0; t < n_tok; t++)
            Y[(size_t)t * out_stride + r] = (float)dot_f64(tmp, X + (size_t)t * x_stride, n_cols);
    }
    free(tmp);
    return 0;
}

/* the reference's generic prefill path: for every token, for every row, decode the row again
 * and dot it in fp32, single-threaded (common/transformer.h:4535-4572) */
int qo_gemm_tokmajor_f32(uint32_t type, const void *W, const float *X, float *Y, int n_rows,
                         int n_cols, int n_tok, int out_stride, int x_stride) {
    const size_t rb = qo_row_size(type, n_cols);
    if (!rb) return -1;
    float *tmp = (float *)calloc((size_t)n_cols, sizeof(float));
    if (!tmp) return -2;
    for (int t = 0; t < n_tok; t++) {
        const float *xt = X + (size_t)t * x_stride;
        for (int r = 0; r < n_rows; r++) {
            qo_dequant_row(type, (const uint8_t *)W + (size_t)r * rb, tmp, n_cols);
            Y[(size_t)t * out_stride + r] = dot_f32(tmp, xt, n_cols);
        }
    }
    free(tmp);
    return 0;
}

/* ------------------------------------------------------------------ MoE */

static void heap_swap(float *w, int *idx, int a, int b) {
    float tw = w[a]; w[a] = w[b]; w[b] = tw;
    int ti = idx[a]; idx[a] = idx[b]; idx[b] = ti;
}

/* common/transformer.h:4054-4091: softmax over every expert (plain expf here; the
 * reference's AVX2 build substitutes a 1e-4 polynomial exp, which is not followed), then a
 * k-entry min-heap keyed on the weight: fill the first k, afterwards replace the root only
 * when the candidate is strictly larger; finally divide by the sum of the survivors. */
void qo_moe_route(const float *logits, int n_expert, int top_k, int *idx, float *w) {
    float *p = (float *)malloc((size_t)n_expert * sizeof(float));
    float mx = logits[0];
    for (int e = 1; e < n_expert; e++) if (logits[e] > mx) mx = logits[e];
    float sum = 0.0f;
    for (int e = 0; e < n_expert; e++) { p[e] = expf(logits[e] - mx); sum += p[e]; }
    for (int e = 0; e < n_expert; e++) p[e] /= sum;

    int k = 0;
    for (int e = 0; e < n_expert; e++) {
        if (k < top_k) {
            idx[k] = e; w[k] = p[e];
            for (int j = k; j > 0;) { /* sift up */
                const int parent = (j - 1) / 2;
                if (w[j] < w[parent]) { heap_swap(w, idx, j, parent); j = parent; }
                else break;
            }
            k++;
        } else if (p[e] > w[0]) {
            w[0] = p[e]; idx[0] = e;
            for (int j = 0;;) { /* sift down */
                int s = j;
                const int l = 2 * j + 1, r = 2 * j + 2;
                if (l < top_k && w[l] < w[s]) s = l;
                if (r < top_k && w[r] < w[s]) s = r;
                if (s == j) break;
                heap_swap(w, idx, j, s);
                j = s;
            }
        }
    }
    float wsum = 0.0f;
    for (int i = 0; i < top_k; i++) wsum += w[i];
    if (wsum > 0.0f) for (int i = 0; i < top_k; i++) w[i] /= wsum;
    free(p);
}

static int moe_token(uint32_t type_gate, uint32_t type_up, uint32_t type_down, const void *gate, const void *up,
                     const void *down, int n_embd, int n_ff, const float *x, const int *idx, const float *w, int top_k,
                     float *out, int use_f64) {
    const size_t rb_g = qo_row_size(type_gate, n_embd); /* gate/up rows have n_embd columns */
    const size_t rb_u = qo_row_size(type_up, n_embd);
    const size_t rb_dn = qo_row_size(type_down, n_ff);  /* down rows have n_ff columns */
    if (!rb_g || !rb_u || !rb_dn) return -1;
    const int mx = n_embd > n_ff ? n_embd : n_ff;
    float *tmp = (float *)calloc((size_t)mx, sizeof(float));
    float *g = (float *)calloc((size_t)n_ff, sizeof(float));
    float *u = (float *)calloc((size_t)n_ff, sizeof(float));
    float *q = (float *)calloc((size_t)n_embd, sizeof(float));
    double *acc = (double *)calloc((size_t)n_embd, sizeof(double));
    for (int i = 0; i < n_embd; i++) out[i] = 0.0f;
    for (int k = 0; k < top_k; k++) {
        /* expert slice = base + expert * rows_per_expert * row_bytes (common/transformer.h:525) */
        const uint8_t *ge = (const uint8_t *)gate + (size_t)idx[k] * n_ff * rb_g;
        const uint8_t *ue = (const uint8_t *)up + (size_t)idx[k] * n_ff * rb_u;
        const uint8_t *de = (const uint8_t *)down + (size_t)idx[k] * n_embd * rb_dn;
        for (int r = 0; r < n_ff; r++) {
            qo_dequant_row(type_up, ue + (size_t)r * rb_u, tmp, n_embd);
            u[r] = use_f64 ? (float)dot_f64(tmp, x, n_embd) : dot_f32(tmp, x, n_embd);
            qo_dequant_row(type_gate, ge + (size_t)r * rb_g, tmp, n_embd);
            g[r] = use_f64 ? (float)dot_f64(tmp, x, n_embd) : dot_f32(tmp, x, n_embd);
        }
        /* h = silu(gate) * up, written over gate (common/transformer.h:4108, scalar form :4690) */
        for (int r = 0; r < n_ff; r++) {
            if (use_f64) g[r] = (float)((double)g[r] / (1.0 + exp(-(double)g[r])) * (double)u[r]);
            else g[r] = g[r] / (1.0f + expf(-g[r])) * u[r];
        }
        for (int r = 0; r < n_embd; r++) {
            qo_dequant_row(type_down, de + (size_t)r * rb_dn, tmp, n_ff);
            q[r] = use_f64 ? (float)dot_f64(tmp, g, n_ff) : dot_f32(tmp, g, n_ff);
        }
        if (use_f64) for (int i = 0; i < n_embd; i++) acc[i] += (double)w[k] * (double)q[i];
        else for (int i = 0; i < n_embd; i++) out[i] += w[k] * q[i];
    }
    if (use_f64) for (int i = 0; i < n_embd; i++) out[i] = (float)acc[i];
    free(tmp); free(g); free(u); free(q); free(acc);
    return 0;
}

int qo_moe_ffn_token_f64(uint32_t type, const void *gate, const void *up, const void *down,
                         int n_embd, int n_ff, const float *x, const int *idx, const float *w,
                         int top_k, float *out) {
    return moe_token(type, type, type, gate, up, down, n_embd, n_ff, x, idx, w, top_k, out, 1);
}
int qo_moe_ffn_token_f32(uint32_t type, const void *gate, const void *up, const void *down,
                         int n_embd, int n_ff, const float *x, const int *idx, const float *w,
                         int top_k, float *out) {
    return moe_token(type, type, type, gate, up, down, n_embd, n_ff, x, idx, w, top_k, out, 0);
}
int qo_moe_ffn_token_types(uint32_t type_gate, uint32_t type_up, uint32_t type_down, const void *gate, const void *up,
                           const void *down, int n_embd, int n_ff, const float *x, const int *idx, const float *w,
                           int top_k, float *out, int use_f64) {
    return moe_token(type_gate, type_up, type_down, gate, up, down, n_embd, n_ff, x, idx, w, top_k, out, use_f64);
}
