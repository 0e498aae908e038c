/*
 * qlin_codecs_ext.h - device decoders of the further GGML block formats (gfx950).
 *
 * Included by qlin_device.h. Same contract as the decoders there: decode8(blk, k0, y) yields
 * elements k0..k0+7 (k0 a multiple of 8) of one block with the reference's fp32 operation
 * order, so results are bit-identical to common/ggml_dequant.h. Every product below is exact in
 * fp32 (an 11-bit fp16 significand times integers of a few bits), so a fused multiply-add
 * rounds like the separate multiply and add of the scalar code.
 */
#ifndef QLIN_CODECS_EXT_H
#define QLIN_CODECS_EXT_H

namespace qlin {

template <> struct Geom<T_Q4_0>    { static constexpr int BE = 32,  BB = 18;  };
template <> struct Geom<T_Q4_1>    { static constexpr int BE = 32,  BB = 20;  };
template <> struct Geom<T_Q5_0>    { static constexpr int BE = 32,  BB = 22;  };
template <> struct Geom<T_Q5_1>    { static constexpr int BE = 32,  BB = 24;  };
template <> struct Geom<T_Q2_K>    { static constexpr int BE = 256, BB = 84;  };
template <> struct Geom<T_Q3_K>    { static constexpr int BE = 256, BB = 110; };
template <> struct Geom<T_IQ2_XS>  { static constexpr int BE = 256, BB = 74;  };
template <> struct Geom<T_IQ3_XXS> { static constexpr int BE = 256, BB = 98;  };
template <> struct Geom<T_IQ1_S>   { static constexpr int BE = 256, BB = 50;  };
template <> struct Geom<T_IQ2_S>   { static constexpr int BE = 256, BB = 82;  };
template <> struct Geom<T_IQ4_XS>  { static constexpr int BE = 256, BB = 136; };
template <> struct Geom<T_IQ1_M>   { static constexpr int BE = 256, BB = 56;  };
template <> struct Geom<T_TQ1_0>   { static constexpr int BE = 256, BB = 54;  };
template <> struct Geom<T_TQ2_0>   { static constexpr int BE = 256, BB = 66;  };
template <> struct Geom<T_MXFP4>   { static constexpr int BE = 32,  BB = 17;  };
template <> struct Geom<T_NVFP4>   { static constexpr int BE = 64,  BB = 36;  };
template <> struct Geom<T_Q1_0>    { static constexpr int BE = 128, BB = 18;  };

__device__ __forceinline__ float sign_pm1(uint32_t bit) { return bit ? -1.0f : 1.0f; }

/* ---- 32-element blocks: element k < 16 is the low nibble of qs[k], k >= 16 the high nibble
 * of qs[k-16]; eight consecutive elements share the nibble position ---- */

/* Q4_0 [d][qs 16]: (nibble - 8) * d   (common/ggml_dequant.h:2850-2862) */
template <> struct Codec<T_Q4_0> : Geom<T_Q4_0> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const uint8_t *q = blk + 2 + (k0 & 15);
        const int sh = (k0 >> 4) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = (float)((int)((q[i] >> sh) & 15) - 8) * d;
    }
};

/* Q4_1 [d][m][qs 16]: nibble * d + m   (:2864-2877) */
template <> struct Codec<T_Q4_1> : Geom<T_Q4_1> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk)), m = half_bits_exact(ld_u16(blk + 2));
        const uint8_t *q = blk + 4 + (k0 & 15);
        const int sh = (k0 >> 4) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = (float)((q[i] >> sh) & 15) * d + m;
    }
};

/* Q5_0 [d][qh 4][qs 16]: bit k of qh is the fifth bit of element k; (q5 - 16) * d   (:2879-2895) */
template <> struct Codec<T_Q5_0> : Geom<T_Q5_0> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const uint32_t hb = blk[2 + (k0 >> 3)]; /* the eight fifth bits of this group */
        const uint8_t *q = blk + 6 + (k0 & 15);
        const int sh = (k0 >> 4) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int v = (int)(((q[i] >> sh) & 15) | (((hb >> i) & 1u) << 4));
            y[i] = (float)(v - 16) * d;
        }
    }
};

/* Q5_1 [d][m][qh 4][qs 16]: q5 * d + m   (:2897-2914) */
template <> struct Codec<T_Q5_1> : Geom<T_Q5_1> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk)), m = half_bits_exact(ld_u16(blk + 2));
        const uint32_t hb = blk[4 + (k0 >> 3)];
        const uint8_t *q = blk + 8 + (k0 & 15);
        const int sh = (k0 >> 4) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int v = (int)(((q[i] >> sh) & 15) | (((hb >> i) & 1u) << 4));
            y[i] = (float)v * d + m;
        }
    }
};

/* E8M0 scale byte, halved: 2^(e-128), the two smallest as fp32 subnormals (:1464-1469) */
__device__ __forceinline__ float e8m0_half(uint32_t e) {
    return __uint_as_float(e < 2u ? (0x00200000u << e) : ((e - 1u) << 23));
}

/* unsigned E4M3 scale byte (bit 7 ignored), halved (:1471-1477) */
__device__ __forceinline__ float ue4m3_half(uint32_t x) {
    if (x == 0u || x == 0x7Fu) return 0.0f;
    const uint32_t e = (x >> 3) & 15u, man = x & 7u;
    if (e == 0u) return (float)man * 0x1p-10f;
    return (float)(8u + man) * __uint_as_float((e + 116u) << 23); /* (8+man) * 2^(e-11) */
}

/* MXFP4 [e][qs 16]: E2M1x2[nibble] * 2^(e-128); blocks are 17 bytes, so only byte loads (:2818-2830) */
template <> struct Codec<T_MXFP4> : Geom<T_MXFP4> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = e8m0_half(blk[0]);
        const uint8_t *q = blk + 1 + (k0 & 15);
        const int sh = (k0 >> 4) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = (float)qlin_mxfp4_values[(q[i] >> sh) & 15] * d;
    }
};

/* NVFP4 [d 4 x ue4m3][qs 32]: four sub-blocks of 16 with the Q4_0 nibble order over 8 bytes (:2832-2848) */
template <> struct Codec<T_NVFP4> : Geom<T_NVFP4> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const int s = k0 >> 4;
        const float d = ue4m3_half(blk[s]);
        const uint8_t *q = blk + 4 + 8 * s;
        const int sh = ((k0 >> 3) & 1) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = (float)qlin_mxfp4_values[(q[i] >> sh) & 15] * d;
    }
};

/* Q1_0 [d][128 bits]: bit set -> d, clear -> -d   (:1491-1503) */
template <> struct Codec<T_Q1_0> : Geom<T_Q1_0> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const uint32_t db = __float_as_uint(half_bits_exact(ld_u16(blk)));
        const uint32_t bits = blk[2 + (k0 >> 3)];
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = __uint_as_float(db ^ ((((bits >> i) & 1u) ^ 1u) << 31));
    }
};

/* ---- K-quants with 2-bit planes: element k: half = k/128, plane j = (k%128)/32, sixteen-group
 * sub = (k%32)/16, l = k%16; byte qs[32*half + 16*sub + l], scale index 8*half + 2*j + sub ---- */

/* Q2_K [scales 16][qs 64][d][dmin]: (d*(sc&15))*q2 - dmin*(sc>>4)   (:1505-1534) */
template <> struct Codec<T_Q2_K> : Geom<T_Q2_K> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk + 80)), dmin = half_bits_exact(ld_u16(blk + 82));
        const int half = k0 >> 7, j = (k0 >> 5) & 3, sub = (k0 >> 4) & 1, l0 = k0 & 15;
        const uint32_t sc = blk[8 * half + 2 * j + sub];
        const float dl = d * (float)(sc & 15u), ml = dmin * (float)(sc >> 4);
        const uint8_t *q = blk + 16 + 32 * half + 16 * sub + l0;
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = dl * (float)((q[i] >> (2 * j)) & 3) - ml;
    }
};

/* Q3_K [hmask 32][qs 64][scales 12][d]: 6-bit scale i = low nibble (byte i, or high half of
 * byte i-8) + two bits of byte 8 + i%4 at position 2*(i/4); q = 2 low bits, minus 4 when bit
 * (4*half + j) of hmask[16*sub + l] is clear; (d*(sc-32))*q   (:1536-1580) */
template <> struct Codec<T_Q3_K> : Geom<T_Q3_K> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk + 108));
        const int half = k0 >> 7, j = (k0 >> 5) & 3, sub = (k0 >> 4) & 1, l0 = k0 & 15;
        const int is = 8 * half + 2 * j + sub;
        const uint8_t *s = blk + 96;
        const int lo4 = is < 8 ? (s[is] & 15) : (s[is - 8] >> 4);
        const int hi2 = (s[8 + (is & 3)] >> (2 * (is >> 2))) & 3;
        const float dl = d * (float)((lo4 | (hi2 << 4)) - 32);
        const uint8_t *q = blk + 32 + 32 * half + 16 * sub + l0;
        const uint8_t *hm = blk + 16 * sub + l0;
        const int hsh = 4 * half + j;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int v = (int)((q[i] >> (2 * j)) & 3) - (((hm[i] >> hsh) & 1) ? 0 : 4);
            y[i] = dl * (float)v;
        }
    }
};

/* ---- i-quants: group g = k/32, l = (k%32)/8 picks the grid lookup ---- */

/* IQ3_XXS [d][qs 64][8 x u32]: word g holds the scale (bits 28..31) and four 7-bit sign indices;
 * db = d*(0.5+s)*0.5; two four-magnitude grid entries per eight elements   (:2916-2940) */
template <> struct Codec<T_IQ3_XXS> : Geom<T_IQ3_XXS> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const uint32_t w = ld_u32_a2(blk + 66 + 4 * g);
        const float db = d * (0.5f + (float)(w >> 28)) * 0.5f;
        const uint32_t sg = iq_sign_byte((w >> (7 * l)) & 127u);
        const uint32_t c0 = qlin_iq3xxs_grid[blk[2 + 8 * g + 2 * l]], c1 = qlin_iq3xxs_grid[blk[2 + 8 * g + 2 * l + 1]];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            y[i] = db * (float)((c0 >> (8 * i)) & 255u) * sign_pm1((sg >> i) & 1u);
            y[i + 4] = db * (float)((c1 >> (8 * i)) & 255u) * sign_pm1((sg >> (i + 4)) & 1u);
        }
    }
};

/* IQ4_XS [d][scales_h u16][scales_l 4][qs 128]: 6-bit scale of group g = nibble g of scales_l +
 * bits 2g,2g+1 of scales_h; (d*(ls-32)) * iq4nl[nibble]   (:2956-2973) */
template <> struct Codec<T_IQ4_XS> : Geom<T_IQ4_XS> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const int g = k0 >> 5, r = k0 & 31;
        const int ls = (int)(((blk[4 + (g >> 1)] >> (4 * (g & 1))) & 15) | (((ld_u16(blk + 2) >> (2 * g)) & 3u) << 4));
        const float dl = d * (float)(ls - 32);
        const uint8_t *q = blk + 8 + 16 * g + (r & 15);
        const int sh = (r >> 4) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = dl * (float)qlin_iq4nl_values[(q[i] >> sh) & 15];
    }
};

/* eight magnitudes of a 64-bit grid cell times a scale, signs from a byte */
__device__ __forceinline__ void cell_times(uint64_t cell, float db, uint32_t sg, float (&y)[8]) {
#pragma unroll
    for (int i = 0; i < 8; i++)
        y[i] = db * (float)(uint32_t)((cell >> (8 * i)) & 255u) * sign_pm1((sg >> i) & 1u);
}

/* IQ2_XS [d][qs 32 x u16][scales 8]: word 4g+l = 9-bit grid index + 7-bit sign index;
 * db = d*(0.5+nibble)*0.25, low nibble of scales[g] for l<2, high for l>=2   (:2975-2994) */
template <> struct Codec<T_IQ2_XS> : Geom<T_IQ2_XS> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const float db = d * (0.5f + (float)((blk[66 + g] >> (4 * (l >> 1))) & 15)) * 0.25f;
        const uint32_t w = ld_u16(blk + 2 + 2 * (4 * g + l));
        cell_times(qlin_iq2xs_grid[w & 511u], db, iq_sign_byte(w >> 9), y);
    }
};

/* IQ2_S [d][qs 64][qh 8][scales 8]: grid index = qs[4g+l] + 256 * bit pair l of qh[g]; sign byte
 * stored as is in qs[32+4g+l]; db as IQ2_XS   (:2996-3020) */
template <> struct Codec<T_IQ2_S> : Geom<T_IQ2_S> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const float db = d * (0.5f + (float)((blk[74 + g] >> (4 * (l >> 1))) & 15)) * 0.25f;
        const uint32_t idx = blk[2 + 4 * g + l] | ((((uint32_t)blk[66 + g] >> (2 * l)) & 3u) << 8);
        cell_times(qlin_iq2s_grid[idx], db, blk[34 + 4 * g + l], y);
    }
};

/* eight ternary values {-1,0,1} of a grid cell, shifted by +-1/8 and scaled */
__device__ __forceinline__ void ternary_cell(uint64_t cell, float dl, float delta, float (&y)[8]) {
#pragma unroll
    for (int i = 0; i < 8; i++) y[i] = dl * ((float)(int)(int8_t)((cell >> (8 * i)) & 255u) + delta);
}

/* IQ1_S [d][qs 32][qh 8 x u16]: word g = four 3-bit index extensions, scale at bits 12..14, sign
 * of the shift at bit 15; (d*(2s+1)) * (t +- 0.125)   (:3062-3082) */
template <> struct Codec<T_IQ1_S> : Geom<T_IQ1_S> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const uint32_t h = ld_u16(blk + 34 + 2 * g);
        const float dl = d * (float)(2 * (int)((h >> 12) & 7u) + 1);
        const float delta = (h & 0x8000u) ? -0.125f : 0.125f;
        ternary_cell(qlin_iq1s_grid[blk[2 + 4 * g + l] | (((h >> (3 * l)) & 7u) << 8)], dl, delta, y);
    }
};

/* IQ1_M [qs 32][qh 16][scales 4 x u16]: the fp16 super-scale sits in the top nibbles of the four
 * scale words; group g: word g/2, 3-bit scale at bit 6*(g%2) + 3*(l/2); nibble l%2 of
 * qh[2g + l/2]: 3 index bits + the sign of the shift   (:3084-3125) */
template <> struct Codec<T_IQ1_M> : Geom<T_IQ1_M> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const uint32_t s0 = ld_u16(blk + 48), s1 = ld_u16(blk + 50), s2 = ld_u16(blk + 52), s3 = ld_u16(blk + 54);
        const float d = half_bits_exact((s0 >> 12) | ((s1 >> 8) & 0x00F0u) | ((s2 >> 4) & 0x0F00u) | (s3 & 0xF000u));
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const uint32_t sw = ld_u16(blk + 48 + 2 * (g >> 1));
        const float dl = d * (float)(2 * (int)((sw >> (6 * (g & 1) + 3 * (l >> 1))) & 7u) + 1);
        const uint32_t nib = ((uint32_t)blk[32 + 2 * g + (l >> 1)] >> (4 * (l & 1))) & 15u;
        const float delta = (nib & 8u) ? -0.125f : 0.125f;
        ternary_cell(qlin_iq1s_grid[blk[4 * g + l] | ((nib & 7u) << 8)], dl, delta, y);
    }
};

/* ---- ternary formats ---- */

/* base-3 digit n (0..4) of a fixed-point byte: (byte * 3^n mod 256) * 3 >> 8   (:3127-3159) */
__device__ __forceinline__ int trit_of(uint32_t byte, int n) {
    const uint32_t pow3 = (uint32_t)(0x511B090301ull >> (8 * n)) & 255u; /* 1, 3, 9, 27, 81 */
    return (int)((((byte * pow3) & 255u) * 3u) >> 8);
}

/* TQ1_0 [qs 48][qh 4][d]: elements 0..159 digit k/32 of qs[k%32]; 160..239 digit (k-160)/16 of
 * qs[32+(k-160)%16]; 240..255 digit (k-240)/4 of qh[(k-240)%4]; (trit-1)*d */
template <> struct Codec<T_TQ1_0> : Geom<T_TQ1_0> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk + 52));
        if (k0 < 240) {
            const int r = k0 < 160 ? k0 : k0 - 160;
            const int n = k0 < 160 ? (r >> 5) : (r >> 4);
            const uint8_t *q = k0 < 160 ? blk + (r & 31) : blk + 32 + (r & 15);
#pragma unroll
            for (int i = 0; i < 8; i++) y[i] = (float)(trit_of(q[i], n) - 1) * d;
        } else {
            const int r = k0 - 240;
#pragma unroll
            for (int i = 0; i < 8; i++) y[i] = (float)(trit_of(blk[48 + (i & 3)], (r + i) >> 2) - 1) * d;
        }
    }
};

/* TQ2_0 [qs 64][d]: element k = bit pair (k%128)/32 of qs[32*(k/128) + k%32]; (q-1)*d   (:3161-3175) */
template <> struct Codec<T_TQ2_0> : Geom<T_TQ2_0> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk + 64));
        const uint8_t *q = blk + 32 * (k0 >> 7) + (k0 & 31);
        const int sh = 2 * ((k0 >> 5) & 3);
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = (float)((int)((q[i] >> sh) & 3) - 1) * d;
    }
};

}  // namespace qlin
#endif /* QLIN_CODECS_EXT_H */
