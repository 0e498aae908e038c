/*
 * qoracle_ext.c - CPU oracle, decoders of the further GGML block formats (see qoracle.h).
 *
 * TEST INFRASTRUCTURE ONLY: checker, never the product path.
 *
 * Each decoder is written per output element (which bytes and bits element k reads), not as
 * the reference's running-pointer loops; the fp32 operation order of the reference is kept so
 * that results are bit-identical. Parity status: every function here is pinned by golden
 * blocks decoded by the compiled reference (random bytes including NaN/Inf/subnormal scale
 * patterns, bit-exact), by a SHA-256 over a larger sweep, and by an independent float64
 * closed form rounded once to fp32 (tests/formulas.py).
 */
#include "qoracle.h"
#include "qoracle_tables_ext.h"

#include <string.h>

static inline uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static inline uint32_t rd32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}
static inline float bits_to_float(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }

/* 7 stored sign bits + their parity as bit 7 (table at common/ggml_dequant.h:1765-1774) */
static inline uint32_t sign_byte(uint32_t i7) {
    uint32_t p = i7 ^ (i7 >> 4);
    p ^= p >> 2;
    p ^= p >> 1;
    return i7 | ((p & 1u) << 7);
}
static inline float pm1(uint32_t bit) { return bit ? -1.0f : 1.0f; }

/* E8M0 exponent byte -> HALF of 2^(e-127) (common/ggml_dequant.h:1464-1469): 2^(e-128), the two
 * smallest as fp32 subnormals */
float qo_e8m0_half_to_fp32(uint8_t e) {
    return bits_to_float(e < 2 ? (0x00200000u << e) : ((uint32_t)(e - 1) << 23));
}

/* unsigned E4M3 (bit 7 ignored), halved (common/ggml_dequant.h:1471-1477): 0 for 0x00 and 0x7f,
 * man * 2^-10 for exponent 0, else (8 + man) * 2^(exp - 11) */
float qo_ue4m3_half_to_fp32(uint8_t x) {
    if (x == 0 || x == 0x7f) return 0.0f;
    const int e = (x >> 3) & 15, man = x & 7;
    if (e == 0) return (float)man * 0x1p-10f;
    return (float)(8 + man) * bits_to_float((uint32_t)(e - 11 + 127) << 23);
}

const void *qo_table_ext(const char *name, size_t *bytes) {
    if (!strcmp(name, "mxfp4_values")) { *bytes = sizeof(qo_mxfp4_values); return qo_mxfp4_values; }
    if (!strcmp(name, "iq3xxs_grid")) { *bytes = sizeof(qo_iq3xxs_grid); return qo_iq3xxs_grid; }
    if (!strcmp(name, "iq2xs_grid")) { *bytes = sizeof(qo_iq2xs_grid); return qo_iq2xs_grid; }
    if (!strcmp(name, "iq2s_grid")) { *bytes = sizeof(qo_iq2s_grid); return qo_iq2s_grid; }
    if (!strcmp(name, "iq1s_grid")) { *bytes = sizeof(qo_iq1s_grid); return qo_iq1s_grid; }
    *bytes = 0;
    return NULL;
}

/* ---- 32-element blocks with one fp16 scale: element k < 16 is the low nibble of qs[k],
 * element k >= 16 the high nibble of qs[k-16] ---- */

/* Q4_0: [d][qs 16]; y = (nibble - 8) * d (common/ggml_dequant.h:2850-2862) */
void qo_dequantize_row_q4_0(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 32; b++, p += 18, dst += 32) {
        const float d = qo_fp16_to_fp32(rd16(p));
        for (int k = 0; k < 32; k++) dst[k] = (float)(((p[2 + (k & 15)] >> (4 * (k >> 4))) & 15) - 8) * d;
    }
}

/* Q4_1: [d][m][qs 16]; y = nibble * d + m (:2864-2877) */
void qo_dequantize_row_q4_1(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 32; b++, p += 20, dst += 32) {
        const float d = qo_fp16_to_fp32(rd16(p)), m = qo_fp16_to_fp32(rd16(p + 2));
        for (int k = 0; k < 32; k++) dst[k] = (float)((p[4 + (k & 15)] >> (4 * (k >> 4))) & 15) * d + m;
    }
}

/* Q5_0: [d][qh 4][qs 16]; bit k of qh is the fifth bit of element k; y = (q5 - 16) * d (:2879-2895) */
void qo_dequantize_row_q5_0(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 32; b++, p += 22, dst += 32) {
        const float d = qo_fp16_to_fp32(rd16(p));
        const uint32_t qh = rd32(p + 2);
        for (int k = 0; k < 32; k++) {
            const int q = (int)(((p[6 + (k & 15)] >> (4 * (k >> 4))) & 15) | (((qh >> k) & 1u) << 4));
            dst[k] = (float)(q - 16) * d;
        }
    }
}

/* Q5_1: [d][m][qh 4][qs 16]; y = q5 * d + m (:2897-2914) */
void qo_dequantize_row_q5_1(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 32; b++, p += 24, dst += 32) {
        const float d = qo_fp16_to_fp32(rd16(p)), m = qo_fp16_to_fp32(rd16(p + 2));
        const uint32_t qh = rd32(p + 4);
        for (int k = 0; k < 32; k++) {
            const int q = (int)(((p[8 + (k & 15)] >> (4 * (k >> 4))) & 15) | (((qh >> k) & 1u) << 4));
            dst[k] = (float)q * d + m;
        }
    }
}

/* MXFP4: [e][qs 16]; y = E2M1x2[nibble] * 2^(e-128) (:2818-2830) */
void qo_dequantize_row_mxfp4(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 32; b++, p += 17, dst += 32) {
        const float d = qo_e8m0_half_to_fp32(p[0]);
        for (int k = 0; k < 32; k++) dst[k] = (float)qo_mxfp4_values[(p[1 + (k & 15)] >> (4 * (k >> 4))) & 15] * d;
    }
}

/* NVFP4: [d 4 x ue4m3][qs 32], four sub-blocks of 16: inside sub-block s, element j < 8 is the
 * low nibble of qs[8s+j], j >= 8 the high nibble of qs[8s+j-8] (:2832-2848) */
void qo_dequantize_row_nvfp4(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 64; b++, p += 36, dst += 64) {
        for (int k = 0; k < 64; k++) {
            const int s = k >> 4, j = k & 15;
            const float d = qo_ue4m3_half_to_fp32(p[s]);
            dst[k] = (float)qo_mxfp4_values[(p[4 + 8 * s + (j & 7)] >> (4 * (j >> 3))) & 15] * d;
        }
    }
}

/* Q1_0: [d][128 bits]; bit k set -> +d, clear -> -d (:1491-1503) */
void qo_dequantize_row_q1_0(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 128; b++, p += 18, dst += 128) {
        const float d = qo_fp16_to_fp32(rd16(p));
        const float nd = -d;
        for (int k = 0; k < 128; k++) dst[k] = ((p[2 + (k >> 3)] >> (k & 7)) & 1) ? d : nd;
    }
}

/* ---- K-quants with 2-bit planes. Element k of a 256-block: half = k/128, plane j = (k%128)/32
 * (bit pair 2j of the byte), sixteen-group sub = (k%32)/16, l = k%16; its byte is
 * qs[32*half + 16*sub + l] and its scale index 8*half + 2*j + sub. ---- */

/* Q2_K: [scales 16][qs 64][d][dmin]; y = (d*(sc&15))*q2 - dmin*(sc>>4) (:1505-1534) */
void qo_dequantize_row_q2_K(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 84, dst += 256) {
        const float d = qo_fp16_to_fp32(rd16(p + 80)), dmin = qo_fp16_to_fp32(rd16(p + 82));
        for (int k = 0; k < 256; k++) {
            const int half = k >> 7, j = (k >> 5) & 3, sub = (k >> 4) & 1, l = k & 15;
            const uint8_t sc = p[8 * half + 2 * j + sub];
            const float dl = d * (float)(sc & 15), ml = dmin * (float)(sc >> 4);
            const int q = (p[16 + 32 * half + 16 * sub + l] >> (2 * j)) & 3;
            dst[k] = dl * (float)q - ml;
        }
    }
}

/* 6-bit scale i (0..15) of a Q3_K block from its 12 packed bytes: low nibble from byte i (i<8:
 * low half of byte i, i>=8: high half of byte i-8), two more bits from byte 8 + i%4 at bit
 * position 2*(i/4)  (the word shuffle at common/ggml_dequant.h:1549-1557) */
int qo_q3k_scale(const uint8_t s[12], int i) {
    const int lo = i < 8 ? (s[i] & 15) : (s[i - 8] >> 4);
    const int hi = (s[8 + (i & 3)] >> (2 * (i >> 2))) & 3;
    return lo | (hi << 4);
}

/* Q3_K: [hmask 32][qs 64][scales 12][d]; q = 2 low bits, minus 4 when bit (4*half + j) of
 * hmask[16*sub + l] is CLEAR; y = (d*(sc-32))*q (:1536-1580) */
void qo_dequantize_row_q3_K(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 110, dst += 256) {
        const float d = qo_fp16_to_fp32(rd16(p + 108));
        for (int k = 0; k < 256; k++) {
            const int half = k >> 7, j = (k >> 5) & 3, sub = (k >> 4) & 1, l = k & 15;
            const float dl = d * (float)(qo_q3k_scale(p + 96, 8 * half + 2 * j + sub) - 32);
            const int lo = (p[32 + 32 * half + 16 * sub + l] >> (2 * j)) & 3;
            const int hbit = (p[16 * sub + l] >> (4 * half + j)) & 1;
            dst[k] = dl * (float)(lo - (hbit ? 0 : 4));
        }
    }
}

/* ---- i-quants: groups of 32 elements (g), eight elements (l = 0..3) per grid lookup ---- */

/* IQ3_XXS: [d][qs 64][8 x u32]; word g: bits 28..31 scale s, four 7-bit sign indices;
 * db = d*(0.5+s)*0.5; elements 8l..8l+3 from grid[qs[8g+2l]], 8l+4..8l+7 from grid[qs[8g+2l+1]]
 * (:2916-2940) */
void qo_dequantize_row_iq3_xxs(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 98, dst += 256) {
        const float d = qo_fp16_to_fp32(rd16(p));
        for (int g = 0; g < 8; g++) {
            const uint32_t w = rd32(p + 66 + 4 * g);
            const float db = d * (0.5f + (float)(w >> 28)) * 0.5f;
            for (int l = 0; l < 4; l++) {
                const uint32_t sg = sign_byte((w >> (7 * l)) & 127u);
                const uint32_t c0 = qo_iq3xxs_grid[p[2 + 8 * g + 2 * l]], c1 = qo_iq3xxs_grid[p[2 + 8 * g + 2 * l + 1]];
                for (int j = 0; j < 4; j++) {
                    dst[32 * g + 8 * l + j] = db * (float)((c0 >> (8 * j)) & 255u) * pm1((sg >> j) & 1u);
                    dst[32 * g + 8 * l + 4 + j] = db * (float)((c1 >> (8 * j)) & 255u) * pm1((sg >> (j + 4)) & 1u);
                }
            }
        }
    }
}

/* IQ4_XS: [d][scales_h u16][scales_l 4][qs 128]; 6-bit scale of group g = nibble g of scales_l
 * plus bits 2g,2g+1 of scales_h; y = (d*(ls-32)) * iq4nl[nibble], nibble order as Q4_0 inside
 * each group's 16 bytes (:2956-2973) */
void qo_dequantize_row_iq4_xs(const void *src, float *dst, int n) {
    size_t tb;
    const int8_t *nl = (const int8_t *)qo_table("iq4nl_values", &tb);
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 136, dst += 256) {
        const float d = qo_fp16_to_fp32(rd16(p));
        const uint32_t sh = rd16(p + 2);
        for (int g = 0; g < 8; g++) {
            const int ls = (int)(((p[4 + (g >> 1)] >> (4 * (g & 1))) & 15) | (((sh >> (2 * g)) & 3u) << 4));
            const float dl = d * (float)(ls - 32);
            for (int k = 0; k < 32; k++)
                dst[32 * g + k] = dl * (float)nl[(p[8 + 16 * g + (k & 15)] >> (4 * (k >> 4))) & 15];
        }
    }
}

/* IQ2_XS: [d][qs 32 x u16][scales 8]; word 4g+l: bits 0..8 grid index, 9..15 sign index;
 * db = d*(0.5+nibble)*0.25 with the low nibble of scales[g] for l<2, the high one for l>=2
 * (:2975-2994) */
void qo_dequantize_row_iq2_xs(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 74, dst += 256) {
        const float d = qo_fp16_to_fp32(rd16(p));
        for (int g = 0; g < 8; g++) {
            for (int l = 0; l < 4; l++) {
                const int nib = (p[66 + g] >> (4 * (l >> 1))) & 15;
                const float db = d * (0.5f + (float)nib) * 0.25f;
                const uint32_t w = rd16(p + 2 + 2 * (4 * g + l));
                const uint64_t cell = qo_iq2xs_grid[w & 511u];
                const uint32_t sg = sign_byte(w >> 9);
                for (int j = 0; j < 8; j++)
                    dst[32 * g + 8 * l + j] = db * (float)(uint32_t)((cell >> (8 * j)) & 255u) * pm1((sg >> j) & 1u);
            }
        }
    }
}

/* IQ2_S: [d][qs 64][qh 8][scales 8]; grid index = qs[4g+l] + 256 * (bit pair l of qh[g]); the
 * sign byte is stored as is in qs[32 + 4g + l]; db as IQ2_XS (:2996-3020) */
void qo_dequantize_row_iq2_s(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 82, dst += 256) {
        const float d = qo_fp16_to_fp32(rd16(p));
        for (int g = 0; g < 8; g++) {
            for (int l = 0; l < 4; l++) {
                const int nib = (p[74 + g] >> (4 * (l >> 1))) & 15;
                const float db = d * (0.5f + (float)nib) * 0.25f;
                const uint32_t idx = p[2 + 4 * g + l] | ((((uint32_t)p[66 + g] >> (2 * l)) & 3u) << 8);
                const uint64_t cell = qo_iq2s_grid[idx];
                const uint32_t sg = p[34 + 4 * g + l];
                for (int j = 0; j < 8; j++)
                    dst[32 * g + 8 * l + j] = db * (float)(uint32_t)((cell >> (8 * j)) & 255u) * pm1((sg >> j) & 1u);
            }
        }
    }
}

/* IQ1_S: [d][qs 32][qh 8 x u16]; word g: 3-bit index extensions at bits 3l, scale at 12..14,
 * sign of the shift at bit 15; y = (d*(2s+1)) * (t + (+-0.125)), t in {-1,0,1} from the grid
 * (:3062-3082) */
void qo_dequantize_row_iq1_s(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 50, dst += 256) {
        const float d = qo_fp16_to_fp32(rd16(p));
        for (int g = 0; g < 8; g++) {
            const uint32_t h = rd16(p + 34 + 2 * g);
            const float dl = d * (float)(2 * (int)((h >> 12) & 7u) + 1);
            const float delta = (h & 0x8000u) ? -0.125f : 0.125f;
            for (int l = 0; l < 4; l++) {
                const uint64_t cell = qo_iq1s_grid[p[2 + 4 * g + l] | (((h >> (3 * l)) & 7u) << 8)];
                for (int j = 0; j < 8; j++)
                    dst[32 * g + 8 * l + j] = dl * ((float)(int8_t)((cell >> (8 * j)) & 255u) + delta);
            }
        }
    }
}

/* IQ1_M: [qs 32][qh 16][scales 4 x u16]; the fp16 super-scale is spread over the top nibbles of
 * the four scale words; group g uses word g/2, 3-bit scales at bit 6*(g%2) (l<2) and
 * 6*(g%2)+3 (l>=2); nibble (l%2) of qh[2g + l/2]: low 3 bits extend the grid index, bit 3 picks
 * the sign of the shift (:3084-3125) */
void qo_dequantize_row_iq1_m(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 56, dst += 256) {
        const uint32_t s0 = rd16(p + 48), s1 = rd16(p + 50), s2 = rd16(p + 52), s3 = rd16(p + 54);
        const uint32_t sw[4] = {s0, s1, s2, s3};
        const float d = qo_fp16_to_fp32((uint16_t)((s0 >> 12) | ((s1 >> 8) & 0x00f0u) | ((s2 >> 4) & 0x0f00u) | (s3 & 0xf000u)));
        for (int g = 0; g < 8; g++) {
            for (int l = 0; l < 4; l++) {
                const int s = (int)((sw[g >> 1] >> (6 * (g & 1) + 3 * (l >> 1))) & 7u);
                const float dl = d * (float)(2 * s + 1);
                const uint32_t nib = ((uint32_t)p[32 + 2 * g + (l >> 1)] >> (4 * (l & 1))) & 15u;
                const float delta = (nib & 8u) ? -0.125f : 0.125f;
                const uint64_t cell = qo_iq1s_grid[p[4 * g + l] | ((nib & 7u) << 8)];
                for (int j = 0; j < 8; j++)
                    dst[32 * g + 8 * l + j] = dl * ((float)(int8_t)((cell >> (8 * j)) & 255u) + delta);
            }
        }
    }
}

/* ---- ternary formats ---- */

/* digit n of a base-3 fixed-point byte: multiply by 3^n modulo 256, then the top "trit" of the
 * result is (v*3) >> 8 (common/ggml_dequant.h:3127-3159) */
static inline int trit(uint8_t byte, int n) {
    static const uint8_t pow3[5] = {1, 3, 9, 27, 81};
    const uint8_t v = (uint8_t)(byte * pow3[n]);
    return ((int)v * 3) >> 8;
}

/* TQ1_0: [qs 48][qh 4][d]. Elements 0..159: digit k/32 of qs[k%32]; 160..239: digit (k-160)/16
 * of qs[32 + (k-160)%16]; 240..255: digit (k-240)/4 of qh[(k-240)%4]; y = (trit-1)*d */
void qo_dequantize_row_tq1_0(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 54, dst += 256) {
        const float d = qo_fp16_to_fp32(rd16(p + 52));
        for (int k = 0; k < 256; k++) {
            int t;
            if (k < 160) t = trit(p[k & 31], k >> 5);
            else if (k < 240) t = trit(p[32 + ((k - 160) & 15)], (k - 160) >> 4);
            else t = trit(p[48 + ((k - 240) & 3)], (k - 240) >> 2);
            dst[k] = (float)(t - 1) * d;
        }
    }
}

/* TQ2_0: [qs 64][d]; element k: bit pair (k%128)/32 of qs[32*(k/128) + k%32]; y = (q-1)*d
 * (:3161-3175) */
void qo_dequantize_row_tq2_0(const void *src, float *dst, int n) {
    const uint8_t *p = (const uint8_t *)src;
    for (int b = 0; b < n / 256; b++, p += 66, dst += 256) {
        const float d = qo_fp16_to_fp32(rd16(p + 64));
        for (int k = 0; k < 256; k++) {
            const int q = (p[32 * (k >> 7) + (k & 31)] >> (2 * ((k >> 5) & 3))) & 3;
            dst[k] = (float)(q - 1) * d;
        }
    }
}
