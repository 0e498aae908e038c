/*
 * gemv_int.hip - batch-1 matvec y = W.x on 8-bit integer dot products, for the block formats whose
 * codes are small integers under a per-group scale (what tf_qmatvec computes,
 * common/transformer.h:1049-1114; the summation order differs).
 *
 * The scheme of the tuned Q4_K kernel, made generic over the format:
 *   - x is converted once per workgroup to fixed point per 32 elements, X = rint(x * 2^(22-e)),
 *     and stored in LDS as three byte planes (top byte signed, the lower two unsigned) with
 *     2^(e-22), the fp32 sums of the two halves of the group, and (for signed codes) the constant
 *     128 * (256 * sum(mid bytes) + sum(low bytes));
 *   - rows travel HBM -> LDS images as flat byte streams, one in flight per image;
 *   - a lane takes one 32-element group per step: the format's extractor turns the group's bits
 *     into 8 dwords of 4 codes in element order plus the scale (and the offset that multiplies
 *     sum(x)) of each 16-element half; 24 four-way integer dot instructions give the exact
 *     integer sums, and  sum (s*q - o) x = s * 2^(e-22) * S - o * sum(x)  is evaluated in fp32.
 *     Signed codes (Q8_0, the 4-bit codebooks) use signed*signed on the top plane and
 *     (code ^ 0x80) = code + 128 against the unsigned planes, minus the stored constant.
 * That is 1 to 2.5 vector instructions per weight where the float path of gemv_stream.hip needs
 * 2 to 5. Quantisation error is 2^-23 of the group's largest |x| (about 1e-6 relative end to end).
 * A non-finite x makes every output NaN.
 *
 * Shape rules as in gemv_stream.hip (the launcher returns false otherwise): whole blocks, n_cols a
 * multiple of 32 and <= 16384, row bytes a multiple of 16 and <= 8 KB, W and x 16-byte aligned.
 */
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

namespace {

constexpr int kGroupDw = 28; /* dwords per x group in LDS: 8 top | 8 mid | 8 low | inv, C, sum_lo, sum_hi; 7 x 16 B
                                (an odd number of 16-byte slots: consecutive lanes read distinct banks) */

template <int CTRL> __device__ __forceinline__ float dppf(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL> __device__ __forceinline__ uint32_t dppu(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) { return __builtin_amdgcn_sdot4((int)a, (int)b, c, false); }
__device__ __forceinline__ uint32_t udot4(uint32_t a, uint32_t b, uint32_t c) { return __builtin_amdgcn_udot4(a, b, c, false); }

/* n dwords starting at any byte of an LDS image (img itself may sit at any byte too), read as aligned dwords
 * and funnel-shifted (misaligned LDS reads stall the LDS pipeline); touches up to 4 bytes past the end */
template <int N> __device__ __forceinline__ void ld_dwords_at(const uint8_t *img, int off, uint32_t (&out)[N]) {
    const uint8_t *p = img + off;
    const uint32_t mis = (uint32_t)(uintptr_t)p & 3u;
    const uint32_t *q = reinterpret_cast<const uint32_t *>(p - mis);
    const uint32_t sh = mis * 8u;
    uint32_t prev = q[0];
#pragma unroll
    for (int i = 0; i < N; i++) {
        const uint32_t next = q[i + 1];
        out[i] = __builtin_amdgcn_alignbit(next, prev, sh);
        prev = next;
    }
}

/* bits 0..3 of v spread to bit 0 of bytes 0..3 */
__device__ __forceinline__ uint32_t spread4(uint32_t v) { return ((v & 15u) * 0x00204081u) & 0x01010101u; }

/* 16-entry byte table lookup of four nibbles (bytes 0..15 in t0..t3): two byte permutes + select */
struct Table16 {
    uint32_t t0, t1, t2, t3;
    /* the grid formats: their codebook in LDS, and byte masks of the eight signs of a group of eight
     * elements (0xFF where the element is negative), by sign byte and by the 7-bit index of the 2/3-bit
     * i-quants (eighth sign = parity) */
    const uint32_t *grid;
    const uint2 *sign256, *sign128;
};
__device__ __forceinline__ uint32_t look4(uint32_t n, const Table16 &t) {
    const uint32_t sel = n & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(t.t1, t.t0, sel), hi = __builtin_amdgcn_perm(t.t3, t.t2, sel);
    const uint32_t m = ((n >> 3) & 0x01010101u) * 0xFFu;
    return (hi & m) | (lo & ~m);
}

/* one 32-element group of a row: codes in element order, scale and offset per 16-element half */
struct Codes {
    uint32_t c[8];
    float s_lo, s_hi, o_lo, o_hi;
};

/* Per format: kSigned (codes are int8), kPer16 (the halves have their own scale/offset), and
 * get(img, g, table): group g (elements 32g..32g+31) of the row image. */
template <uint32_t T> struct IntFmt;

/* Q8_0 [d][32 x int8] (common/ggml_dequant.h:1479-1489) */
template <> struct IntFmt<T_Q8_0> {
    static constexpr bool kSigned = true, kPer16 = false;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &) {
        Codes r;
        const int off = g * 34;
        r.s_lo = half_bits_fast(ld_u16(img + off));
        ld_dwords_at<8>(img, off + 2, r.c);
        r.o_lo = 0.0f;
        return r;
    }
};

/* low nibbles of 16 bytes = elements 0..15, high nibbles = elements 16..31 */
__device__ __forceinline__ void nibbles32(const uint32_t (&q)[4], uint32_t (&c)[8]) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        c[i] = q[i] & 0x0F0F0F0Fu;
        c[4 + i] = (q[i] >> 4) & 0x0F0F0F0Fu;
    }
}

/* Q4_0 [d][qs 16]: d * (nibble - 8) (:2850-2862) */
template <> struct IntFmt<T_Q4_0> {
    static constexpr bool kSigned = false, kPer16 = false;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &) {
        Codes r;
        const int off = g * 18;
        uint32_t q[4];
        ld_dwords_at<4>(img, off + 2, q);
        nibbles32(q, r.c);
        r.s_lo = half_bits_fast(ld_u16(img + off));
        r.o_lo = 8.0f * r.s_lo;
        return r;
    }
};

/* Q4_1 [d][m][qs 16]: d * nibble + m (:2864-2877); 20-byte blocks are dword aligned */
template <> struct IntFmt<T_Q4_1> {
    static constexpr bool kSigned = false, kPer16 = false;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &) {
        Codes r;
        const uint32_t *b = reinterpret_cast<const uint32_t *>(img + g * 20);
        const uint32_t q[4] = {b[1], b[2], b[3], b[4]};
        nibbles32(q, r.c);
        r.s_lo = half_bits_fast(b[0] & 0xFFFFu);
        r.o_lo = -half_bits_fast(b[0] >> 16);
        return r;
    }
};

/* fifth bits: bit e of qh belongs to element e */
__device__ __forceinline__ void add_fifth_bits(uint32_t qh, uint32_t (&c)[8]) {
#pragma unroll
    for (int i = 0; i < 8; i++) c[i] |= spread4(qh >> (4 * i)) << 4;
}

/* Q5_0 [d][qh 4][qs 16]: d * (q5 - 16) (:2879-2895) */
template <> struct IntFmt<T_Q5_0> {
    static constexpr bool kSigned = false, kPer16 = false;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &) {
        Codes r;
        const int off = g * 22;
        uint32_t w[5]; /* qh, then the 16 nibble bytes */
        ld_dwords_at<5>(img, off + 2, w);
        const uint32_t q[4] = {w[1], w[2], w[3], w[4]};
        nibbles32(q, r.c);
        add_fifth_bits(w[0], r.c);
        r.s_lo = half_bits_fast(ld_u16(img + off));
        r.o_lo = 16.0f * r.s_lo;
        return r;
    }
};

/* Q5_1 [d][m][qh 4][qs 16]: d * q5 + m (:2897-2914); 24-byte blocks are dword aligned */
template <> struct IntFmt<T_Q5_1> {
    static constexpr bool kSigned = false, kPer16 = false;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &) {
        Codes r;
        const uint32_t *b = reinterpret_cast<const uint32_t *>(img + g * 24);
        const uint32_t q[4] = {b[2], b[3], b[4], b[5]};
        nibbles32(q, r.c);
        add_fifth_bits(b[1], r.c);
        r.s_lo = half_bits_fast(b[0] & 0xFFFFu);
        r.o_lo = -half_bits_fast(b[0] >> 16);
        return r;
    }
};

/* Q5_K (:1620-1651): sub-block `sub` of a 176-byte super-block (16-byte aligned in the image) */
template <> struct IntFmt<T_Q5_K> {
    static constexpr bool kSigned = false, kPer16 = false;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &) {
        Codes r;
        const uint8_t *blk = img + (g >> 3) * 176;
        const int sub = g & 7;
        const uint4 h = *reinterpret_cast<const uint4 *>(blk);
        /* get_scale_min_k4 (:1582-1590), four fields at a time */
        const uint32_t scw = sub < 4 ? (h.y & 0x3F3F3F3Fu) : ((h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u));
        const uint32_t mnw = sub < 4 ? (h.z & 0x3F3F3F3Fu) : (((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u));
        const int sh8 = 8 * (sub & 3);
        r.s_lo = half_bits_fast(h.x & 0xFFFFu) * (float)((scw >> sh8) & 0xFFu);
        r.o_lo = half_bits_fast(h.x >> 16) * (float)((mnw >> sh8) & 0xFFu);
        const uint4 *q = reinterpret_cast<const uint4 *>(blk + 48 + (sub >> 1) * 32);
        const uint4 *qh = reinterpret_cast<const uint4 *>(blk + 16);
        const uint4 qa = q[0], qb = q[1], ha = qh[0], hb = qh[1];
        const uint32_t qs[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        const uint32_t hs[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
        const int nsh = (sub & 1) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) r.c[i] = ((qs[i] >> nsh) & 0x0F0F0F0Fu) | (((hs[i] >> sub) & 0x01010101u) << 4);
        return r;
    }
};

/* Q6_K (:1653-1687): 32 elements = segment `seg` of half `half`; two int8 scales; codes - 32 */
template <> struct IntFmt<T_Q6_K> {
    static constexpr bool kSigned = false, kPer16 = true;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &) {
        Codes r;
        const int boff = (g >> 3) * 210, sub = g & 7, half = sub >> 2, seg = sub & 3;
        uint32_t ql[8], qh[8];
        ld_dwords_at<8>(img, boff + 64 * half + 32 * (seg & 1), ql);
        ld_dwords_at<8>(img, boff + 128 + 32 * half, qh);
        const int nsh = (seg >> 1) * 4, hsh = 2 * seg;
#pragma unroll
        for (int i = 0; i < 8; i++) r.c[i] = ((ql[i] >> nsh) & 0x0F0F0F0Fu) | (((qh[i] >> hsh) & 0x03030303u) << 4);
        const uint32_t sc = ld_u16(img + boff + 192 + 8 * half + 2 * seg); /* two int8 scales */
        const float d = half_bits_fast(ld_u16(img + boff + 208));
        r.s_lo = d * (float)(int)(int8_t)(sc & 0xFFu);
        r.s_hi = d * (float)(int)(int8_t)(sc >> 8);
        r.o_lo = 32.0f * r.s_lo;
        r.o_hi = 32.0f * r.s_hi;
        return r;
    }
};

/* Q2_K (:1505-1534): plane j of half `half`; 84-byte blocks are dword aligned */
template <> struct IntFmt<T_Q2_K> {
    static constexpr bool kSigned = false, kPer16 = true;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &) {
        Codes r;
        const uint8_t *blk = img + (g >> 3) * 84;
        const int sub = g & 7, half = sub >> 2, j = sub & 3;
        const uint32_t *q = reinterpret_cast<const uint32_t *>(blk + 16 + 32 * half);
#pragma unroll
        for (int i = 0; i < 8; i++) r.c[i] = (q[i] >> (2 * j)) & 0x03030303u;
        const uint32_t h = *reinterpret_cast<const uint32_t *>(blk + 80);
        const float d = half_bits_fast(h & 0xFFFFu), dmin = half_bits_fast(h >> 16);
        const uint32_t sc = ld_u16(blk + 8 * half + 2 * j);
        r.s_lo = d * (float)(sc & 15u);
        r.o_lo = dmin * (float)((sc >> 4) & 15u);
        r.s_hi = d * (float)((sc >> 8) & 15u);
        r.o_hi = dmin * (float)(sc >> 12);
        return r;
    }
};

/* Q3_K (:1536-1580): 2 low bits + high bit from hmask; code + 4*hbit - 4; 6-bit scales - 32 */
template <> struct IntFmt<T_Q3_K> {
    static constexpr bool kSigned = false, kPer16 = true;
    __device__ static float scale6(const uint8_t *sp, int is) {
        const int lo4 = is < 8 ? (sp[is] & 15) : (sp[is - 8] >> 4);
        const int hi2 = (sp[8 + (is & 3)] >> (2 * (is >> 2))) & 3;
        return (float)((lo4 | (hi2 << 4)) - 32);
    }
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &) {
        Codes r;
        const int boff = (g >> 3) * 110, sub = g & 7, half = sub >> 2, j = sub & 3;
        uint32_t q[8], hm[8];
        ld_dwords_at<8>(img, boff + 32 + 32 * half, q);
        ld_dwords_at<8>(img, boff, hm);
        const int hsh = 4 * half + j;
#pragma unroll
        for (int i = 0; i < 8; i++) r.c[i] = ((q[i] >> (2 * j)) & 0x03030303u) | (((hm[i] >> hsh) & 0x01010101u) << 2);
        const float d = half_bits_fast(ld_u16(img + boff + 108));
        const int is = 8 * half + 2 * j;
        r.s_lo = d * scale6(img + boff + 96, is);
        r.s_hi = d * scale6(img + boff + 96, is + 1);
        r.o_lo = 4.0f * r.s_lo;
        r.o_hi = 4.0f * r.s_hi;
        return r;
    }
};

/* IQ4_NL [d][qs 16]: d * table[nibble], table values are signed bytes (:2942-2954) */
template <> struct IntFmt<T_IQ4_NL> {
    static constexpr bool kSigned = true, kPer16 = false;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &t) {
        Codes r;
        const int off = g * 18;
        uint32_t q[4];
        ld_dwords_at<4>(img, off + 2, q);
        nibbles32(q, r.c);
#pragma unroll
        for (int i = 0; i < 8; i++) r.c[i] = look4(r.c[i], t);
        r.s_lo = half_bits_fast(ld_u16(img + off));
        r.o_lo = 0.0f;
        return r;
    }
};

/* IQ4_XS (:2956-2973): 136-byte blocks (8-byte aligned), 6-bit scale - 32 per 32 elements */
template <> struct IntFmt<T_IQ4_XS> {
    static constexpr bool kSigned = true, kPer16 = false;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &t) {
        Codes r;
        const uint8_t *blk = img + (g >> 3) * 136;
        const int sub = g & 7;
        const uint2 h = *reinterpret_cast<const uint2 *>(blk);
        const int ls = (int)(((h.y >> (4 * sub)) & 15u) | ((((h.x >> 16) >> (2 * sub)) & 3u) << 4));
        r.s_lo = half_bits_fast(h.x & 0xFFFFu) * (float)(ls - 32);
        r.o_lo = 0.0f;
        const uint2 *qp = reinterpret_cast<const uint2 *>(blk + 8 + 16 * sub);
        const uint2 qa = qp[0], qb = qp[1];
        const uint32_t q[4] = {qa.x, qa.y, qb.x, qb.y};
        nibbles32(q, r.c);
#pragma unroll
        for (int i = 0; i < 8; i++) r.c[i] = look4(r.c[i], t);
        return r;
    }
};

/* MXFP4 [e][qs 16]: 2^(e-128) * E2M1x2[nibble] (:2818-2830); 17-byte blocks */
template <> struct IntFmt<T_MXFP4> {
    static constexpr bool kSigned = true, kPer16 = false;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &t) {
        Codes r;
        const int off = g * 17;
        uint32_t q[4];
        ld_dwords_at<4>(img, off + 1, q);
        nibbles32(q, r.c);
#pragma unroll
        for (int i = 0; i < 8; i++) r.c[i] = look4(r.c[i], t);
        r.s_lo = e8m0_half(img[off]);
        r.o_lo = 0.0f;
        return r;
    }
};

/* magnitudes m (four bytes, each 1..127: no grid of these formats holds a zero) with the signs of mask s
 * (0xFF = negative) -> signed bytes: (m ^ s) + (s & 1) per byte; a nonzero m keeps the +1 inside its byte */
__device__ __forceinline__ uint32_t apply_signs(uint32_t m, uint32_t s) { return (m ^ s) + (s & 0x01010101u); }

/* IQ2_XXS [d][8 x (4 grid indices, 4 x 7 sign bits + 4-bit scale)]: d*(0.5+s)*0.25 * grid byte * sign
 * (common/ggml_dequant.h:2793-2816); 66-byte blocks */
template <> struct IntFmt<T_IQ2_XXS> {
    static constexpr bool kSigned = true, kPer16 = false;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &t) {
        Codes r;
        const int off = (g >> 3) * 66;
        uint32_t a[2];
        ld_dwords_at<2>(img, off + 2 + 8 * (g & 7), a);
        const uint2 *grid = reinterpret_cast<const uint2 *>(t.grid);
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint2 m = grid[(a[0] >> (8 * l)) & 255u];
            const uint2 sg = t.sign128[(a[1] >> (7 * l)) & 127u];
            r.c[2 * l] = apply_signs(m.x, sg.x);
            r.c[2 * l + 1] = apply_signs(m.y, sg.y);
        }
        r.s_lo = half_bits_fast(ld_u16(img + off)) * (0.5f + (float)(a[1] >> 28)) * 0.25f;
        r.o_lo = 0.0f;
        return r;
    }
};

/* IQ3_XXS [d][qs 64][8 x (4 x 7 sign bits + 4-bit scale)]: d*(0.5+s)*0.5 * grid byte * sign, a four-byte
 * grid entry per index byte (:2916-2940); 98-byte blocks */
template <> struct IntFmt<T_IQ3_XXS> {
    static constexpr bool kSigned = true, kPer16 = false;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &t) {
        Codes r;
        const int off = (g >> 3) * 98, gi = g & 7;
        uint32_t q[2], w[1];
        ld_dwords_at<2>(img, off + 2 + 8 * gi, q);
        ld_dwords_at<1>(img, off + 66 + 4 * gi, w);
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint32_t pair = (l < 2 ? q[0] : q[1]) >> (16 * (l & 1));
            const uint2 sg = t.sign128[(w[0] >> (7 * l)) & 127u];
            r.c[2 * l] = apply_signs(t.grid[pair & 255u], sg.x);
            r.c[2 * l + 1] = apply_signs(t.grid[(pair >> 8) & 255u], sg.y);
        }
        r.s_lo = half_bits_fast(ld_u16(img + off)) * (0.5f + (float)(w[0] >> 28)) * 0.5f;
        r.o_lo = 0.0f;
        return r;
    }
};

/* IQ3_S [d][qs 64][qh 8][signs 32][scales 4]: d*(1+2s) * grid byte * sign, 9-bit grid indices (:3022-3058);
 * 110-byte blocks */
template <> struct IntFmt<T_IQ3_S> {
    static constexpr bool kSigned = true, kPer16 = false;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &t) {
        Codes r;
        const int off = (g >> 3) * 110, gi = g & 7;
        uint32_t q[2], sb[1];
        ld_dwords_at<2>(img, off + 2 + 8 * gi, q);
        ld_dwords_at<1>(img, off + 74 + 4 * gi, sb);
        const uint32_t qh = img[off + 66 + gi];
        const uint32_t nib = (img[off + 106 + (gi >> 1)] >> (4 * (gi & 1))) & 15u;
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint32_t pair = (l < 2 ? q[0] : q[1]) >> (16 * (l & 1));
            const uint32_t i0 = (pair & 255u) | (((qh >> (2 * l)) & 1u) << 8);
            const uint32_t i1 = ((pair >> 8) & 255u) | (((qh >> (2 * l + 1)) & 1u) << 8);
            const uint2 sg = t.sign256[(sb[0] >> (8 * l)) & 255u];
            r.c[2 * l] = apply_signs(t.grid[i0], sg.x);
            r.c[2 * l + 1] = apply_signs(t.grid[i1], sg.y);
        }
        r.s_lo = half_bits_fast(ld_u16(img + off)) * (float)(1u + 2u * nib);
        r.o_lo = 0.0f;
        return r;
    }
};

/* IQ2_XS [d][32 x (9-bit grid index, 7 sign bits)][scales 8]: d*(0.5+s)*0.25 * grid byte * sign with one
 * 4-bit scale per 16 elements (common/ggml_dequant.h:2966-2994); 74-byte blocks */
template <> struct IntFmt<T_IQ2_XS> {
    static constexpr bool kSigned = true, kPer16 = true;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &t) {
        Codes r;
        const int off = (g >> 3) * 74, gi = g & 7;
        uint32_t q[2];
        ld_dwords_at<2>(img, off + 2 + 8 * gi, q);
        const uint32_t sc = img[off + 66 + gi];
        const uint2 *grid = reinterpret_cast<const uint2 *>(t.grid);
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint32_t w = ((l < 2 ? q[0] : q[1]) >> (16 * (l & 1))) & 0xFFFFu;
            const uint2 m = grid[w & 511u];
            const uint2 sg = t.sign128[w >> 9];
            r.c[2 * l] = apply_signs(m.x, sg.x);
            r.c[2 * l + 1] = apply_signs(m.y, sg.y);
        }
        const float d = half_bits_fast(ld_u16(img + off));
        r.s_lo = d * (0.5f + (float)(sc & 15u)) * 0.25f;
        r.s_hi = d * (0.5f + (float)(sc >> 4)) * 0.25f;
        r.o_lo = r.o_hi = 0.0f;
        return r;
    }
};

/* IQ2_S [d][qs 32][signs 32][qh 8][scales 8]: 10-bit grid indices (two more bits per index from qh), sign
 * bytes stored as they are, scales as IQ2_XS (:2996-3020); 82-byte blocks */
template <> struct IntFmt<T_IQ2_S> {
    static constexpr bool kSigned = true, kPer16 = true;
    __device__ static Codes get(const uint8_t *img, int g, const Table16 &t) {
        Codes r;
        const int off = (g >> 3) * 82, gi = g & 7;
        uint32_t q[1], sb[1];
        ld_dwords_at<1>(img, off + 2 + 4 * gi, q);
        ld_dwords_at<1>(img, off + 34 + 4 * gi, sb);
        const uint32_t qh = img[off + 66 + gi], sc = img[off + 74 + gi];
        const uint2 *grid = reinterpret_cast<const uint2 *>(t.grid);
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint2 m = grid[((q[0] >> (8 * l)) & 255u) | (((qh >> (2 * l)) & 3u) << 8)];
            const uint2 sg = t.sign256[(sb[0] >> (8 * l)) & 255u];
            r.c[2 * l] = apply_signs(m.x, sg.x);
            r.c[2 * l + 1] = apply_signs(m.y, sg.y);
        }
        const float d = half_bits_fast(ld_u16(img + off));
        r.s_lo = d * (0.5f + (float)(sc & 15u)) * 0.25f;
        r.s_hi = d * (0.5f + (float)(sc >> 4)) * 0.25f;
        r.o_lo = r.o_hi = 0.0f;
        return r;
    }
};

template <uint32_t T> constexpr bool kUsesTable = (T == T_IQ4_NL || T == T_IQ4_XS || T == T_MXFP4);
/* codebook of the grid formats: bytes staged in LDS and their source */
template <uint32_t T> struct IntGrid { static constexpr int kBytes = 0; __device__ static const uint32_t *src() { return nullptr; } };
template <> struct IntGrid<T_IQ2_XXS> { static constexpr int kBytes = 2048; __device__ static const uint32_t *src() { return reinterpret_cast<const uint32_t *>(qlin_iq2xxs_grid); } };
template <> struct IntGrid<T_IQ3_XXS> { static constexpr int kBytes = 1024; __device__ static const uint32_t *src() { return qlin_iq3xxs_grid; } };
template <> struct IntGrid<T_IQ2_XS> { static constexpr int kBytes = 4096; __device__ static const uint32_t *src() { return reinterpret_cast<const uint32_t *>(qlin_iq2xs_grid); } };
template <> struct IntGrid<T_IQ2_S> { static constexpr int kBytes = 8192; __device__ static const uint32_t *src() { return reinterpret_cast<const uint32_t *>(qlin_iq2s_grid); } };
template <> struct IntGrid<T_IQ3_S> { static constexpr int kBytes = 2048; __device__ static const uint32_t *src() { return qlin_iq3s_grid; } };
constexpr int kSignTableBytes = (256 + 128) * 8;
template <uint32_t T> constexpr int kAuxBytes = IntGrid<T>::kBytes > 0 ? IntGrid<T>::kBytes + kSignTableBytes : 0;

/* planes and constants of one x group, as read from LDS */
struct XGroup {
    uint32_t xt[8], xm[8], xl[8];
    float inv, sum_lo, sum_hi; /* signed codes with a scale per half: the halves' own cneg, as bit patterns */
    int cneg; /* 128 * (256 * sum of mid bytes + sum of low bytes) */
};
__device__ __forceinline__ XGroup load_xgroup(const uint32_t *planes, int g) {
    const uint4 *pp = reinterpret_cast<const uint4 *>(planes + g * kGroupDw);
    const uint4 t0 = pp[0], t1 = pp[1], m0 = pp[2], m1 = pp[3], l0 = pp[4], l1 = pp[5], meta = pp[6];
    XGroup x = {{t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w},
                {m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w},
                {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w},
                __uint_as_float(meta.x), __uint_as_float(meta.z), __uint_as_float(meta.w), (int)meta.y};
    return x;
}

/* one group of codes against one group of x: the group's contribution to the row's dot product */
template <typename F> __device__ __forceinline__ float group_dot(const Codes &cd, const XGroup &x) {
    if (F::kSigned && F::kPer16) {
        int at0 = 0, at1 = 0;
        uint32_t am0 = 0, al0 = 0, am1 = 0, al1 = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t u0 = cd.c[k] ^ 0x80808080u, u1 = cd.c[4 + k] ^ 0x80808080u; /* code + 128 */
            at0 = sdot4(cd.c[k], x.xt[k], at0);
            am0 = udot4(u0, x.xm[k], am0);
            al0 = udot4(u0, x.xl[k], al0);
            at1 = sdot4(cd.c[4 + k], x.xt[4 + k], at1);
            am1 = udot4(u1, x.xm[4 + k], am1);
            al1 = udot4(u1, x.xl[4 + k], al1);
        }
        const float f0 = fmaf((float)at0, 65536.0f, (float)((int)((am0 << 8) + al0) - __float_as_int(x.sum_lo)));
        const float f1 = fmaf((float)at1, 65536.0f, (float)((int)((am1 << 8) + al1) - __float_as_int(x.sum_hi)));
        return (cd.s_lo * f0 + cd.s_hi * f1) * x.inv;
    } else if (F::kSigned) {
        int at = 0;
        uint32_t am = 0, al = 0;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const uint32_t u = cd.c[k] ^ 0x80808080u; /* code + 128 */
            at = sdot4(cd.c[k], x.xt[k], at);
            am = udot4(u, x.xm[k], am);
            al = udot4(u, x.xl[k], al);
        }
        /* none of the signed formats has an offset */
        return cd.s_lo * (fmaf((float)at, 65536.0f, (float)((int)((am << 8) + al) - x.cneg)) * x.inv);
    } else if (F::kPer16) {
        int at0 = 0, at1 = 0;
        uint32_t am0 = 0, al0 = 0, am1 = 0, al1 = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            at0 = sdot4(cd.c[k], x.xt[k], at0);
            am0 = udot4(cd.c[k], x.xm[k], am0);
            al0 = udot4(cd.c[k], x.xl[k], al0);
            at1 = sdot4(cd.c[4 + k], x.xt[4 + k], at1);
            am1 = udot4(cd.c[4 + k], x.xm[4 + k], am1);
            al1 = udot4(cd.c[4 + k], x.xl[4 + k], al1);
        }
        const float f0 = fmaf((float)at0, 65536.0f, (float)((am0 << 8) + al0)) * x.inv;
        const float f1 = fmaf((float)at1, 65536.0f, (float)((am1 << 8) + al1)) * x.inv;
        return (cd.s_lo * f0 - cd.o_lo * x.sum_lo) + (cd.s_hi * f1 - cd.o_hi * x.sum_hi);
    } else {
        int at = 0;
        uint32_t am = 0, al = 0;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            at = sdot4(cd.c[k], x.xt[k], at);
            am = udot4(cd.c[k], x.xm[k], am);
            al = udot4(cd.c[k], x.xl[k], al);
        }
        const float f = fmaf((float)at, 65536.0f, (float)((am << 8) + al)) * x.inv;
        return cd.s_lo * f - cd.o_lo * (x.sum_lo + x.sum_hi);
    }
}

/* NG > 0: a lane's groups (lane, lane + 64, ... : at most NG of them) keep their x planes in registers
 * for all rows; NG == 0: any row length, the planes are read from LDS for every row */
template <uint32_t T, int NG>
__global__ void __launch_bounds__(NG > 2 ? 512 : 1024)
gemv_int_kernel(const JobView job, const float *__restrict__ x, int n_cols, int row_bytes, int n_chunks, size_t row_stride,
                int depth, int rows_per_wg) {
    using F = IntFmt<T>;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    /* LDS map: x groups [n_cols/32][28 dwords] | raw x [n_cols] floats | codebook and sign masks of the grid
     * formats | row images [waves][depth][16 n_chunks]. A row (row_bytes bytes from any even address) is copied as
     * the n_chunks aligned 16-byte pieces from the one that holds its first byte on; its image starts that many
     * bytes into the copy */
    const int n_groups = n_cols >> 5;
    uint32_t *planes = reinterpret_cast<uint32_t *>(lds);
    const float4 *xraw = reinterpret_cast<const float4 *>(planes + n_groups * kGroupDw);
    uint8_t *aux = lds + (size_t)n_groups * kGroupDw * 4 + (size_t)n_cols * 4;
    uint8_t *images = aux + kAuxBytes<T>;

    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = blockDim.x >> 6, n_threads = blockDim.x;
    const bool paired = job.mode == 2;
    const int n_rows = paired ? job.n0 : job.n0 + job.n1 + job.n2;
    const int row0 = blockIdx.x * rows_per_wg;
    int rows_here = n_rows - row0;
    if (rows_here > rows_per_wg) rows_here = rows_per_wg;
    const int my_rows = (wv < rows_here ? (rows_here - wv + n_waves - 1) / n_waves : 0) * (paired ? 2 : 1);
    auto locate = [&](int i, const uint8_t *&Wm, float *&ym, int &r) {
        if (paired) {
            Wm = (i & 1) ? job.W1 : job.W0;
            ym = job.y0;
            r = row0 + wv + (i >> 1) * n_waves;
        } else {
            job_locate(job, row0 + wv + i * n_waves, Wm, ym, r);
        }
    };
    const int image_bytes = n_chunks << 4;
    const int loads_per_row = (n_chunks + 63) >> 6;
    uint8_t *my_images = images + (size_t)wv * depth * image_bytes;
    const uint32_t my_images_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)my_images;
    auto row_address = [&](int i) {
        const uint8_t *Wm;
        float *ym;
        int r;
        locate(i, Wm, ym, r);
        return Wm + (size_t)r * row_stride;
    };
    /* Row i of this wave -> image i % depth; data goes HBM -> LDS at M0 + 16*lane. The loads are
     * written as instructions and waited for by hand (the compiler would wait for all of them
     * before any LDS access). Nothing else in this kernel uses M0. Every row takes the same number of
     * instructions: lanes past the row's last piece fetch that piece again (their LDS slots lie behind the row). */
    auto issue = [&](int i) {
        const uint8_t *row = row_address(i);
        const uint32_t delta = (uint32_t)(uintptr_t)row & 15u;
        const uint4 *gp = reinterpret_cast<const uint4 *>(row - delta);
        const int last_piece = (int)((delta + (uint32_t)row_bytes + 15u) >> 4) - 1;
        const uint32_t img = my_images_lds + (uint32_t)((i % depth) * image_bytes);
        for (int c0 = 0; c0 < n_chunks; c0 += 64) {
            const uint32_t m0v = __builtin_amdgcn_readfirstlane(img + 16u * (uint32_t)c0);
            const int piece = c0 + lane < last_piece ? c0 + lane : last_piece;
            if (c0 + lane < n_chunks)
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt"
                             : : "v"(gp + piece), "s"(m0v) : "memory");
        }
    };

    /* x first (raw copy to LDS), a barrier so that every wave's x request precedes every row
     * request, then the first rows; loads retire in order, so once at most the row loads are
     * outstanding this wave's part of x has landed */
    const int n4 = n_cols >> 2;
    const float4 *xg = reinterpret_cast<const float4 *>(x);
    const uint32_t xraw_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)xraw;
    for (int base = wv * 64; base < n4; base += n_threads) {
        const uint32_t m0v = __builtin_amdgcn_readfirstlane(xraw_lds + 16u * (uint32_t)base);
        if (base + lane < n4)
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                         : : "v"(xg + base + lane), "s"(m0v) : "memory");
    }
    asm volatile("s_barrier" ::: "memory");
    int issued = 0;
    for (; issued < depth && issued < my_rows; issued++) issue(issued);
    wait_vm_at_most(issued * loads_per_row);

    /* x -> fixed-point byte planes: 4 elements per thread, 8 consecutive threads share a group; each
     * thread converts exactly the elements its own wave fetched */
    for (int base = wv * 64; base < n4; base += n_threads) {
        const int idx = base + lane;
        const bool mine = idx < n4;
        const float4 v = mine ? xraw[idx] : make_float4(0.f, 0.f, 0.f, 0.f);
        float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        amax = fmaxf(amax, dppf<0xB1>(amax));
        amax = fmaxf(amax, dppf<0x4E>(amax));
        amax = fmaxf(amax, dppf<0x141>(amax));
        float sum = (v.x + v.y) + (v.z + v.w);
        sum += dppf<0xB1>(sum);
        sum += dppf<0x4E>(sum); /* sum over this thread's 16-element half */
        int e = (int)(__float_as_uint(amax) >> 23) - 126; /* amax in [2^(e-1), 2^e) */
        if (e < -100) e = -100;
        const float scale = __uint_as_float((uint32_t)(127 + 22 - e) << 23);
        float inv = __uint_as_float((uint32_t)(127 - 22 + e) << 23);
        /* Inf or NaN in x poisons every row (the maximum above drops NaNs, the sum does not) */
        const float sum32 = sum + dppf<0x141>(sum);
        if (!(amax <= 3.0e38f) || !(fabsf(sum32) <= 3.0e38f)) inv = __uint_as_float(0x7FC00000u);
        const uint32_t X0 = (uint32_t)__float2int_rn(v.x * scale), X1 = (uint32_t)__float2int_rn(v.y * scale);
        const uint32_t X2 = (uint32_t)__float2int_rn(v.z * scale), X3 = (uint32_t)__float2int_rn(v.w * scale);
        /* byte transpose: plane k = byte k of X0..X3 */
        const uint32_t lo01 = __builtin_amdgcn_perm(X1, X0, 0x05010400u), lo23 = __builtin_amdgcn_perm(X3, X2, 0x05010400u);
        const uint32_t hi01 = __builtin_amdgcn_perm(X1, X0, 0x07030602u), hi23 = __builtin_amdgcn_perm(X3, X2, 0x07030602u);
        const uint32_t pl_low = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
        const uint32_t pl_mid = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
        const uint32_t pl_top = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
        /* 128 * (256 * sum of mid bytes + sum of low bytes) over the group */
        uint32_t cs = (udot4(pl_mid, 0x01010101u, 0u) << 8) + udot4(pl_low, 0x01010101u, 0u);
        cs += dppu<0xB1>(cs);
        cs += dppu<0x4E>(cs);
        const uint32_t cs_half = cs; /* over this thread's 16-element half */
        cs += dppu<0x141>(cs);
        const int grp = idx >> 3, j = idx & 7;
        uint32_t *dst = planes + grp * kGroupDw;
        if (mine) {
            dst[j] = pl_top;
            dst[8 + j] = pl_mid;
            dst[16 + j] = pl_low;
            if (j == 0) {
                dst[24] = __float_as_uint(inv);
                dst[25] = cs << 7;
                dst[26] = (F::kSigned && F::kPer16) ? cs_half << 7 : __float_as_uint(sum);
            }
            if (j == 4) dst[27] = (F::kSigned && F::kPer16) ? cs_half << 7 : __float_as_uint(sum);
        }
    }
    Table16 tab = {0, 0, 0, 0, nullptr, nullptr, nullptr};
    if (IntGrid<T>::kBytes > 0) {
        uint32_t *grid = reinterpret_cast<uint32_t *>(aux);
        uint2 *sign256 = reinterpret_cast<uint2 *>(aux + IntGrid<T>::kBytes), *sign128 = sign256 + 256;
        for (int t = threadIdx.x; t < IntGrid<T>::kBytes / 4; t += n_threads) grid[t] = IntGrid<T>::src()[t];
        if (threadIdx.x < 384) {
            const uint32_t i = threadIdx.x, sb = i < 256 ? i : iq_sign_byte(i - 256);
            sign256[i] = make_uint2(spread4(sb) * 0xFFu, spread4(sb >> 4) * 0xFFu);
        }
        tab.grid = grid;
        tab.sign256 = sign256;
        tab.sign128 = sign128;
    }
    if (kUsesTable<T>) {
        const uint4 v = *reinterpret_cast<const uint4 *>(T == T_MXFP4 ? qlin_mxfp4_values : qlin_iq4nl_values);
        tab.t0 = v.x; tab.t1 = v.y; tab.t2 = v.z; tab.t3 = v.w;
    }
    __syncthreads();

    XGroup xr[NG > 0 ? NG : 1];
    if (NG > 0) {
#pragma unroll
        for (int jj = 0; jj < NG; jj++) {
            const int g = lane + 64 * jj;
            xr[jj] = load_xgroup(planes, g < n_groups ? g : 0);
        }
    }
    float gate_value = 0.0f;
    for (int i = 0; i < my_rows; i++) {
        wait_vm_at_most((issued - i - 1) * loads_per_row);
        const uint8_t *img = my_images + (size_t)(i % depth) * image_bytes + ((uint32_t)(uintptr_t)row_address(i) & 15u);
        float acc = 0.0f;
        if (NG > 0) {
#pragma unroll
            for (int jj = 0; jj < NG; jj++) {
                const int g = lane + 64 * jj;
                if (g < n_groups) acc += group_dot<F>(F::get(img, g, tab), xr[jj]);
            }
        } else {
            for (int g = lane; g < n_groups; g += 64) acc += group_dot<F>(F::get(img, g, tab), load_xgroup(planes, g));
        }
        /* the image may be refilled once its reads have returned */
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (issued < my_rows) {
            issue(issued);
            issued++;
        }
        const float s = wave_sum_dpp(acc);
        const uint8_t *Wm;
        float *ym;
        int r;
        locate(i, Wm, ym, r);
        if (paired) {
            if (i & 1) {
                if (lane == 0) ym[r] = silu_times(gate_value, s);
            } else {
                gate_value = s;
            }
        } else if (lane == 0) {
            if (job.mode == 1) unsafeAtomicAdd(ym + r, s); /* no read of y: the wave has row loads in flight */
            else ym[r] = s;
        }
    }
}

template <uint32_t T>
bool int_typed(const GemvJob &job, const float *x, int n_cols, int n_cu, hipStream_t stream, hipError_t *err, size_t row_stride) {
    int be, bb;
    type_geometry(T, &be, &bb);
    const size_t row_bytes = (size_t)(n_cols / be) * bb;
    if (n_cols > 16384 || (n_cols & 31) || (n_cols % be) || row_bytes > 8192) return false;
    if (row_stride == 0) row_stride = row_bytes; /* rows that are a column range of longer ones keep those rows' pitch */
    /* rows on 16-byte boundaries are copied as they are; rows at other (even) addresses with the 16-byte piece
     * that holds their first byte and the one that holds their last */
    bool on16 = (row_stride & 15) == 0 && (row_bytes & 15) == 0;
    for (int m = 0; m < job.n_mat; m++) on16 = on16 && ((uintptr_t)job.W[m] & 15) == 0;
    if (!on16) {
        if ((bb & 1) || (row_stride & 1)) return false; /* the 16-bit fields want even addresses */
        for (int m = 0; m < job.n_mat; m++)
            if ((uintptr_t)job.W[m] & 1) return false;
    }
    const int n_chunks = (int)((row_bytes + (on16 ? 0 : 14) + 15) >> 4);
    const size_t image_bytes = (size_t)n_chunks * 16;
    if ((uintptr_t)x & 15) return false;
    const int n_rows = job.mode == kSiluMul ? job.n_rows[0] : job.total_rows();
    const size_t x_bytes = (size_t)(n_cols >> 5) * kGroupDw * 4 + (size_t)n_cols * 4 + (size_t)kAuxBytes<T>;
    const size_t lds_cap = 160 * 1024 - 16;
    const int n_groups = n_cols >> 5;
    /* long rows of the grid formats: eight waves of 256 registers, so that a lane keeps the x planes of its
     * seven groups for all its rows (read from LDS for every row they are what the kernel waits for) */
    const bool wide = IntGrid<T>::kBytes > 0 && n_groups > 128 && n_groups <= 448;
    int waves = wide ? 8 : 16, depth = 2;
    if (x_bytes + (size_t)waves * depth * image_bytes > lds_cap) depth = 1;
    if (x_bytes + (size_t)waves * depth * image_bytes > lds_cap) { waves = 8; depth = 2; }
    if (x_bytes + (size_t)waves * depth * image_bytes > lds_cap) depth = 1;
    if (x_bytes + (size_t)waves * depth * image_bytes > lds_cap) return false;
    if ((size_t)(n_chunks + 63) / 64 * depth > 15) return false; /* the hand-placed waits count to 15 */
    int rows_per_wg = (n_rows + n_cu - 1) / n_cu;
    if (rows_per_wg < 1) rows_per_wg = 1;
    const int grid = (n_rows + rows_per_wg - 1) / rows_per_wg;
    const size_t lds_bytes = x_bytes + (size_t)waves * depth * image_bytes + 16; /* + slack for the funnel-shift reads */
    auto launch = [&](auto kernel, OnceFlag &raised) {
        if (!raised.is_set()) {
            *err = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (*err != hipSuccess) return;
            raised.set();
        }
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(waves * 64), lds_bytes, stream, job_view(job), x, n_cols,
                           (int)row_bytes, n_chunks, row_stride, depth, rows_per_wg);
        *err = hipGetLastError();
    };
    static OnceFlag raised[4];
    if (n_groups <= 64) launch(gemv_int_kernel<T, 1>, raised[1]);
    else if (n_groups <= 128) launch(gemv_int_kernel<T, 2>, raised[2]);
    else if (wide && waves == 8) launch(gemv_int_kernel<T, (IntGrid<T>::kBytes > 0) ? 7 : 0>, raised[3]);
    else launch(gemv_int_kernel<T, 0>, raised[0]);
    return true;
}

}  // namespace

bool gemv_int_takes_any_even_address(uint32_t type) {
    switch (type) {
    case T_Q8_0: case T_Q4_0: case T_Q4_1: case T_Q5_0: case T_Q5_1: case T_Q5_K: case T_Q6_K: case T_Q2_K: case T_Q3_K:
    case T_IQ4_NL: case T_IQ4_XS: case T_IQ2_XXS: case T_IQ3_XXS: case T_IQ3_S: case T_IQ2_XS: case T_IQ2_S:
        return true;
    default: return false; /* MXFP4 (17-byte blocks) and the formats of the other kernels */
    }
}

bool launch_gemv_int(uint32_t type, const GemvJob &job, const float *x, int n_cols, int n_cu, hipStream_t stream,
                     hipError_t *err, size_t row_stride) {
    *err = hipSuccess;
    switch (type) {
    case T_Q8_0: return int_typed<T_Q8_0>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q4_0: return int_typed<T_Q4_0>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q4_1: return int_typed<T_Q4_1>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q5_0: return int_typed<T_Q5_0>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q5_1: return int_typed<T_Q5_1>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q5_K: return int_typed<T_Q5_K>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q6_K: return int_typed<T_Q6_K>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q2_K: return int_typed<T_Q2_K>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q3_K: return int_typed<T_Q3_K>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ4_NL: return int_typed<T_IQ4_NL>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ4_XS: return int_typed<T_IQ4_XS>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_MXFP4: return int_typed<T_MXFP4>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ2_XXS: return int_typed<T_IQ2_XXS>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ3_XXS: return int_typed<T_IQ3_XXS>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ3_S: return int_typed<T_IQ3_S>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ2_XS: return int_typed<T_IQ2_XS>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ2_S: return int_typed<T_IQ2_S>(job, x, n_cols, n_cu, stream, err, row_stride);
    default: return false;
    }
}

}  // namespace qlin
