/*
 * gemv_stream.hip - batch-1 matvec y = W.x for every supported block type, organised for HBM
 * streaming (what tf_qmatvec computes, common/transformer.h:1049-1114; the summation order
 * differs).
 *
 * One workgroup per block of rows, about one per compute unit. x is copied once per workgroup
 * into LDS as fp32. Every wavefront then walks its rows: a row travels from HBM into a private
 * LDS image as one flat byte stream (fully contiguous 16-byte-per-lane loads that write LDS
 * directly, global_load_lds_dwordx4), the next row is requested while the current one is
 * decoded. A lane takes eight consecutive elements per step: the codes are unpacked four bytes
 * at a time with byte-parallel masks, converted byte-to-float and FMA'd with x; the block scale
 * goes on once per eight elements, and constant offsets (-128 of Q8_0, -32 of Q6_K, the mins of
 * Q5_K) are applied to the precomputed sum of the eight x instead of to every element:
 *     sum (s*q_i - o) x_i = s * sum q_i x_i - o * sum x_i.
 * The i-quant grids sit in LDS; their sign bits are OR'ed into the converted magnitudes. Results
 * differ from the decoders' only in rounding (the matvec tolerance is 1e-5, it is not bit-exact
 * work); fp32 accumulate, one wave reduction per row.
 *
 * Shape rules (the launcher returns false and the caller falls back to the plain kernel
 * otherwise): whole blocks, n_cols <= 16384, row bytes a multiple of 16 and at most 8 KB, W and
 * x 16-byte aligned.
 */
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

namespace {


/* ---- eight elements of one block against eight x, per type ---- */

__device__ __forceinline__ float ub0(uint32_t v) { float f; asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ub1(uint32_t v) { float f; asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ub2(uint32_t v) { float f; asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(v)); return f; }
__device__ __forceinline__ float ub3(uint32_t v) { float f; asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(v)); return f; }

/* acc + sum of (unsigned byte i of b) * x_i */
__device__ __forceinline__ float dot_u4(uint32_t b, const float4 x, float acc) {
    acc = fmaf(ub0(b), x.x, acc);
    acc = fmaf(ub1(b), x.y, acc);
    acc = fmaf(ub2(b), x.z, acc);
    return fmaf(ub3(b), x.w, acc);
}
/* same with sign bit i of `signs` (bits 0..3) applied to term i; magnitudes are non-negative, so
 * the sign can simply be OR'ed into the converted float */
__device__ __forceinline__ float dot_u4_signed(uint32_t b, uint32_t signs, const float4 x, float acc) {
    const uint32_t t = signs << 28; /* bit 3 -> bit 31 */
    acc = fmaf(__uint_as_float(__float_as_uint(ub0(b)) | ((t << 3) & 0x80000000u)), x.x, acc);
    acc = fmaf(__uint_as_float(__float_as_uint(ub1(b)) | ((t << 2) & 0x80000000u)), x.y, acc);
    acc = fmaf(__uint_as_float(__float_as_uint(ub2(b)) | ((t << 1) & 0x80000000u)), x.z, acc);
    return fmaf(__uint_as_float(__float_as_uint(ub3(b)) | (t & 0x80000000u)), x.w, acc);
}
/* 8 (4) bytes at any byte offset `off` of a 16-byte aligned LDS image. Misaligned LDS reads
 * stall the LDS pipeline on this part (they were 3/4 of its busy time in the first version of
 * this kernel), so the bytes are fetched as aligned dwords and funnel-shifted into place. May
 * touch up to 4 bytes past the last one asked for. */
__device__ __forceinline__ uint2 ld8_at(const uint8_t *img, int off) {
    const uint32_t *q = reinterpret_cast<const uint32_t *>(img + (off & ~3));
    const uint32_t sh = (uint32_t)(off & 3) * 8u;
    const uint32_t w0 = q[0], w1 = q[1], w2 = q[2];
    return make_uint2(__builtin_amdgcn_alignbit(w1, w0, sh), __builtin_amdgcn_alignbit(w2, w1, sh));
}
__device__ __forceinline__ uint32_t ld4_at(const uint8_t *img, int off) {
    const uint32_t *q = reinterpret_cast<const uint32_t *>(img + (off & ~3));
    return __builtin_amdgcn_alignbit(q[1], q[0], (uint32_t)(off & 3) * 8u);
}

struct Tables {
    const uint64_t *grid2; /* iq2xxs grid in LDS */
    const uint32_t *grid3; /* iq3s grid in LDS */
    uint32_t nl0, nl1, nl2, nl3; /* the 16 values of a 4-bit codebook (iq4nl or E2M1) + 128, as bytes */
};

/* default: the bit-exact decoder (Q4_K reaches this kernel only when the tuned one declines) */
template <uint32_t T> struct Lean {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float, const Tables &) {
        const uint8_t *blk = img + boff;
        float w[8];
        Codec<T>::decode8(blk, k0, w);
        return w[0] * xa.x + w[1] * xa.y + w[2] * xa.z + w[3] * xa.w + w[4] * xb.x + w[5] * xb.y + w[6] * xb.z +
               w[7] * xb.w;
    }
};

/* dense fp16 rows: the hardware conversion (the decoder's hand-rebuilt NaN payloads cost six instructions per
 * element and mean nothing inside a sum) */
template <> struct Lean<T_F16> {
    __device__ static float dot8(const uint8_t *img, int boff, int, const float4 xa, const float4 xb, float, const Tables &) {
        typedef _Float16 half2v __attribute__((ext_vector_type(2)));
        const uint4 v = *reinterpret_cast<const uint4 *>(img + boff);
        const half2v a = __builtin_bit_cast(half2v, v.x), b = __builtin_bit_cast(half2v, v.y);
        const half2v c = __builtin_bit_cast(half2v, v.z), d = __builtin_bit_cast(half2v, v.w);
        float acc = (float)a[0] * xa.x;
        acc = fmaf((float)a[1], xa.y, acc);
        acc = fmaf((float)b[0], xa.z, acc);
        acc = fmaf((float)b[1], xa.w, acc);
        acc = fmaf((float)c[0], xb.x, acc);
        acc = fmaf((float)c[1], xb.y, acc);
        acc = fmaf((float)d[0], xb.z, acc);
        return fmaf((float)d[1], xb.w, acc);
    }
};

/* Q8_0 (common/ggml_dequant.h:1479-1489): d * q, q int8 = (q ^ 0x80 as unsigned) - 128 */
template <> struct Lean<T_Q8_0> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &) {
        const uint8_t *blk = img + boff;
        const float d = half_bits_fast(ld_u16(blk));
        const uint2 q = ld8_at(img, boff + 2 + k0);
        const float s = dot_u4(q.y ^ 0x80808080u, xb, dot_u4(q.x ^ 0x80808080u, xa, 0.0f));
        return d * fmaf(-128.0f, xs8, s);
    }
};

/* Q5_K (:1620-1651): (d*sc)*(nibble + 16*highbit) - dmin*m */
template <> struct Lean<T_Q5_K> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &) {
        const uint8_t *blk = img + boff;
        const uint4 h = *reinterpret_cast<const uint4 *>(blk);
        const int g = k0 >> 5, l0 = k0 & 31;
        /* get_scale_min_k4 (:1582-1590), four fields at a time */
        const uint32_t scw = g < 4 ? (h.y & 0x3F3F3F3Fu) : ((h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u));
        const uint32_t mnw = g < 4 ? (h.z & 0x3F3F3F3Fu) : (((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u));
        const int sh8 = 8 * (g & 3);
        const float dl = half_bits_fast(h.x & 0xFFFFu) * (float)((scw >> sh8) & 0xFFu);
        const float ml = half_bits_fast(h.x >> 16) * (float)((mnw >> sh8) & 0xFFu);
        const uint2 q = *reinterpret_cast<const uint2 *>(blk + 48 + (g >> 1) * 32 + l0);
        const uint2 qh = *reinterpret_cast<const uint2 *>(blk + 16 + l0);
        const int sh = (g & 1) * 4;
        const uint32_t v0 = ((q.x >> sh) & 0x0F0F0F0Fu) | (((qh.x >> g) & 0x01010101u) << 4);
        const uint32_t v1 = ((q.y >> sh) & 0x0F0F0F0Fu) | (((qh.y >> g) & 0x01010101u) << 4);
        const float s = dot_u4(v1, xb, dot_u4(v0, xa, 0.0f));
        return fmaf(dl, s, -ml * xs8);
    }
};

/* Q6_K (:1653-1687): (d*sc)*(q - 32), q = low nibble | two high bits << 4 */
template <> struct Lean<T_Q6_K> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &) {
        const uint8_t *blk = img + boff;
        const int half = k0 >> 7, r = k0 & 127, seg = r >> 5, l0 = r & 31;
        const uint2 ql = ld8_at(img, boff + 64 * half + 32 * (seg & 1) + l0);
        const uint2 qh = ld8_at(img, boff + 128 + 32 * half + l0);
        const int nsh = (seg >> 1) * 4, hsh = 2 * seg;
        const uint32_t v0 = ((ql.x >> nsh) & 0x0F0F0F0Fu) | (((qh.x >> hsh) & 0x03030303u) << 4);
        const uint32_t v1 = ((ql.y >> nsh) & 0x0F0F0F0Fu) | (((qh.y >> hsh) & 0x03030303u) << 4);
        const float sc = (float)reinterpret_cast<const int8_t *>(blk + 192)[8 * half + 2 * seg + (l0 >> 4)];
        const float dl = half_bits_fast(ld_u16(blk + 208)) * sc;
        const float s = dot_u4(v1, xb, dot_u4(v0, xa, 0.0f));
        return dl * fmaf(-32.0f, xs8, s);
    }
};

/* IQ4_NL (:2942-2954): d * table[nibble]; the 16-entry table lookup is two byte permutes (entries
 * 0-7 and 8-15) and a select on bit 3 of the nibble; table entries are stored + 128 */
template <> struct Lean<T_IQ4_NL> {
    __device__ static uint32_t look4(uint32_t n, const Tables &t) {
        const uint32_t sel = n & 0x07070707u;
        const uint32_t lo = __builtin_amdgcn_perm(t.nl1, t.nl0, sel), hi = __builtin_amdgcn_perm(t.nl3, t.nl2, sel);
        const uint32_t m = ((n >> 3) & 0x01010101u) * 0xFFu;
        return (hi & m) | (lo & ~m);
    }
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &t) {
        const uint8_t *blk = img + boff;
        const float d = half_bits_fast(ld_u16(blk));
        const uint2 q = ld8_at(img, boff + 2 + (k0 & 15));
        const int sh = (k0 >> 4) * 4;
        const uint32_t v0 = look4((q.x >> sh) & 0x0F0F0F0Fu, t), v1 = look4((q.y >> sh) & 0x0F0F0F0Fu, t);
        const float s = dot_u4(v1, xb, dot_u4(v0, xa, 0.0f));
        return d * fmaf(-128.0f, xs8, s);
    }
};

/* IQ2_XXS (:2793-2816): d*(0.5+s)*0.25 * grid byte * sign */
template <> struct Lean<T_IQ2_XXS> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float, const Tables &t) {
        const uint8_t *blk = img + boff;
        const float d = half_bits_fast(ld_u16(blk));
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const uint2 a = ld8_at(img, boff + 2 + 8 * g);
        const uint32_t a0 = a.x, a1 = a.y;
        const float db = d * (0.5f + (float)(a1 >> 28)) * 0.25f;
        const uint2 cell = *reinterpret_cast<const uint2 *>(t.grid2 + ((a0 >> (8 * l)) & 255u));
        const uint32_t sg = iq_sign_byte((a1 >> (7 * l)) & 127u);
        const float s = dot_u4_signed(cell.y, sg >> 4, xb, dot_u4_signed(cell.x, sg & 15u, xa, 0.0f));
        return db * s;
    }
};

/* IQ3_S (:3022-3058): d*(1+2s) * grid byte * sign; two 4-byte grid entries per eight elements */
template <> struct Lean<T_IQ3_S> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float, const Tables &t) {
        const uint8_t *blk = img + boff;
        const float d = half_bits_fast(ld_u16(blk));
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const uint32_t nib = (blk[106 + (g >> 1)] >> (4 * (g & 1))) & 15u;
        const float db = d * (float)(1u + 2u * nib);
        const uint32_t qh = blk[66 + g];
        const uint32_t pair = ld_u16(blk + 2 + 8 * g + 2 * l);
        const uint32_t i0 = (pair & 255u) | (((qh >> (2 * l)) & 1u) << 8);
        const uint32_t i1 = (pair >> 8) | (((qh >> (2 * l + 1)) & 1u) << 8);
        const uint32_t sb = blk[74 + 4 * g + l];
        const float s = dot_u4_signed(t.grid3[i1], sb >> 4, xb, dot_u4_signed(t.grid3[i0], sb & 15u, xa, 0.0f));
        return db * s;
    }
};


/* bits 0..3 of v spread to bit 0 of bytes 0..3 (the shifted copies of the multiply do not overlap) */
__device__ __forceinline__ uint32_t spread4(uint32_t v) { return ((v & 15u) * 0x00204081u) & 0x01010101u; }

/* Q4_0 (:2850-2862): d * (nibble - 8) */
template <> struct Lean<T_Q4_0> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &) {
        const float d = half_bits_fast(ld_u16(img + boff));
        const uint2 q = ld8_at(img, boff + 2 + (k0 & 15));
        const int sh = (k0 >> 4) * 4;
        const float s = dot_u4((q.y >> sh) & 0x0F0F0F0Fu, xb, dot_u4((q.x >> sh) & 0x0F0F0F0Fu, xa, 0.0f));
        return d * fmaf(-8.0f, xs8, s);
    }
};

/* Q4_1 (:2864-2877): d * nibble + m */
template <> struct Lean<T_Q4_1> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &) {
        const uint32_t h = *reinterpret_cast<const uint32_t *>(img + boff); /* 20-byte blocks: dword aligned */
        const uint2 q = ld8_at(img, boff + 4 + (k0 & 15));
        const int sh = (k0 >> 4) * 4;
        const float s = dot_u4((q.y >> sh) & 0x0F0F0F0Fu, xb, dot_u4((q.x >> sh) & 0x0F0F0F0Fu, xa, 0.0f));
        return fmaf(half_bits_fast(h & 0xFFFFu), s, half_bits_fast(h >> 16) * xs8);
    }
};

/* Q5_0 (:2879-2895): d * (nibble + 16*bit - 16); the eight fifth bits of a group are one byte of qh */
template <> struct Lean<T_Q5_0> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &) {
        const uint8_t *blk = img + boff;
        const float d = half_bits_fast(ld_u16(blk));
        const uint32_t hb = blk[2 + (k0 >> 3)];
        const uint2 q = ld8_at(img, boff + 6 + (k0 & 15));
        const int sh = (k0 >> 4) * 4;
        const uint32_t v0 = ((q.x >> sh) & 0x0F0F0F0Fu) | (spread4(hb) << 4);
        const uint32_t v1 = ((q.y >> sh) & 0x0F0F0F0Fu) | (spread4(hb >> 4) << 4);
        return d * fmaf(-16.0f, xs8, dot_u4(v1, xb, dot_u4(v0, xa, 0.0f)));
    }
};

/* Q5_1 (:2897-2914): d * (nibble + 16*bit) + m */
template <> struct Lean<T_Q5_1> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &) {
        const uint8_t *blk = img + boff;
        const uint32_t h = *reinterpret_cast<const uint32_t *>(blk); /* 24-byte blocks: dword aligned */
        const uint32_t hb = blk[4 + (k0 >> 3)];
        const uint2 q = *reinterpret_cast<const uint2 *>(blk + 8 + (k0 & 15));
        const int sh = (k0 >> 4) * 4;
        const uint32_t v0 = ((q.x >> sh) & 0x0F0F0F0Fu) | (spread4(hb) << 4);
        const uint32_t v1 = ((q.y >> sh) & 0x0F0F0F0Fu) | (spread4(hb >> 4) << 4);
        return fmaf(half_bits_fast(h & 0xFFFFu), dot_u4(v1, xb, dot_u4(v0, xa, 0.0f)), half_bits_fast(h >> 16) * xs8);
    }
};

/* Q2_K (:1505-1534): (d*(sc&15)) * q2 - dmin*(sc>>4); 84-byte blocks are dword aligned */
template <> struct Lean<T_Q2_K> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &) {
        const uint8_t *blk = img + boff;
        const uint32_t h = *reinterpret_cast<const uint32_t *>(blk + 80);
        const int half = k0 >> 7, j = (k0 >> 5) & 3, sub = (k0 >> 4) & 1, l0 = k0 & 15;
        const uint32_t sc = blk[8 * half + 2 * j + sub];
        const uint2 q = ld8_at(img, boff + 16 + 32 * half + 16 * sub + l0);
        const float s = dot_u4((q.y >> (2 * j)) & 0x03030303u, xb, dot_u4((q.x >> (2 * j)) & 0x03030303u, xa, 0.0f));
        return fmaf(half_bits_fast(h & 0xFFFFu) * (float)(sc & 15u), s, -(half_bits_fast(h >> 16) * (float)(sc >> 4)) * xs8);
    }
};

/* Q3_K (:1536-1580): (d*(sc-32)) * (q2 + 4*hbit - 4) */
template <> struct Lean<T_Q3_K> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &) {
        const uint8_t *blk = img + boff;
        const int half = k0 >> 7, j = (k0 >> 5) & 3, sub = (k0 >> 4) & 1, l0 = k0 & 15;
        const int is = 8 * half + 2 * j + sub;
        const uint8_t *sp = blk + 96;
        const int lo4 = is < 8 ? (sp[is] & 15) : (sp[is - 8] >> 4);
        const int hi2 = (sp[8 + (is & 3)] >> (2 * (is >> 2))) & 3;
        const float dl = half_bits_fast(ld_u16(blk + 108)) * (float)((lo4 | (hi2 << 4)) - 32);
        const uint2 q = ld8_at(img, boff + 32 + 32 * half + 16 * sub + l0);
        const uint2 hm = ld8_at(img, boff + 16 * sub + l0);
        const int hsh = 4 * half + j;
        const uint32_t v0 = ((q.x >> (2 * j)) & 0x03030303u) | (((hm.x >> hsh) & 0x01010101u) << 2);
        const uint32_t v1 = ((q.y >> (2 * j)) & 0x03030303u) | (((hm.y >> hsh) & 0x01010101u) << 2);
        return dl * fmaf(-4.0f, xs8, dot_u4(v1, xb, dot_u4(v0, xa, 0.0f)));
    }
};

/* IQ4_XS (:2956-2973): (d*(ls-32)) * table[nibble]; 136-byte blocks are dword aligned */
template <> struct Lean<T_IQ4_XS> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &t) {
        const uint8_t *blk = img + boff;
        const uint2 h = *reinterpret_cast<const uint2 *>(blk); /* d, scales_h | scales_l */
        const int g = k0 >> 5, r = k0 & 31;
        const int ls = (int)(((h.y >> (4 * g)) & 15u) | ((((h.x >> 16) >> (2 * g)) & 3u) << 4));
        const float dl = half_bits_fast(h.x & 0xFFFFu) * (float)(ls - 32);
        const uint2 q = *reinterpret_cast<const uint2 *>(blk + 8 + 16 * g + (r & 15));
        const int sh = (r >> 4) * 4;
        const uint32_t v0 = Lean<T_IQ4_NL>::look4((q.x >> sh) & 0x0F0F0F0Fu, t), v1 = Lean<T_IQ4_NL>::look4((q.y >> sh) & 0x0F0F0F0Fu, t);
        return dl * fmaf(-128.0f, xs8, dot_u4(v1, xb, dot_u4(v0, xa, 0.0f)));
    }
};

/* IQ2_XS (:2975-2994): d*(0.5+nibble)*0.25 * grid byte * sign */
template <> struct Lean<T_IQ2_XS> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float, const Tables &t) {
        const uint8_t *blk = img + boff;
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const float db = half_bits_fast(ld_u16(blk)) * (0.5f + (float)((blk[66 + g] >> (4 * (l >> 1))) & 15)) * 0.25f;
        const uint32_t w = ld_u16(blk + 2 + 2 * (4 * g + l));
        const uint2 cell = *reinterpret_cast<const uint2 *>(t.grid2 + (w & 511u));
        const uint32_t sg = iq_sign_byte(w >> 9);
        return db * dot_u4_signed(cell.y, sg >> 4, xb, dot_u4_signed(cell.x, sg & 15u, xa, 0.0f));
    }
};

/* IQ2_S (:2996-3020): as IQ2_XS with a 10-bit grid index and the sign byte stored as is */
template <> struct Lean<T_IQ2_S> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float, const Tables &t) {
        const uint8_t *blk = img + boff;
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const float db = half_bits_fast(ld_u16(blk)) * (0.5f + (float)((blk[74 + g] >> (4 * (l >> 1))) & 15)) * 0.25f;
        const uint32_t idx = blk[2 + 4 * g + l] | ((((uint32_t)blk[66 + g] >> (2 * l)) & 3u) << 8);
        const uint2 cell = *reinterpret_cast<const uint2 *>(t.grid2 + idx);
        const uint32_t sg = blk[34 + 4 * g + l];
        return db * dot_u4_signed(cell.y, sg >> 4, xb, dot_u4_signed(cell.x, sg & 15u, xa, 0.0f));
    }
};

/* IQ3_XXS (:2916-2940): d*(0.5+s)*0.5 * grid byte * sign, two 4-byte grid entries per eight elements */
template <> struct Lean<T_IQ3_XXS> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float, const Tables &t) {
        const uint8_t *blk = img + boff;
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const uint32_t w = ld4_at(img, boff + 66 + 4 * g);
        const float db = half_bits_fast(ld_u16(blk)) * (0.5f + (float)(w >> 28)) * 0.5f;
        const uint32_t sg = iq_sign_byte((w >> (7 * l)) & 127u);
        const uint32_t pair = ld_u16(blk + 2 + 8 * g + 2 * l);
        return db * dot_u4_signed(t.grid3[pair >> 8], sg >> 4, xb, dot_u4_signed(t.grid3[pair & 255u], sg & 15u, xa, 0.0f));
    }
};

/* IQ1_S (:3062-3082): (d*(2s+1)) * (t + delta); the grid is staged as t+1 in {0,1,2}, so
 * sum (t + delta) x = sum (t+1) x + (delta - 1) sum x */
template <> struct Lean<T_IQ1_S> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &t) {
        const uint8_t *blk = img + boff;
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const uint32_t h = ld_u16(blk + 34 + 2 * g);
        const float dl = half_bits_fast(ld_u16(blk)) * (float)(2 * (int)((h >> 12) & 7u) + 1);
        const float dm1 = (h & 0x8000u) ? -1.125f : -0.875f;
        const uint2 cell = *reinterpret_cast<const uint2 *>(t.grid2 + (blk[2 + 4 * g + l] | (((h >> (3 * l)) & 7u) << 8)));
        return dl * fmaf(dm1, xs8, dot_u4(cell.y, xb, dot_u4(cell.x, xa, 0.0f)));
    }
};

/* IQ1_M (:3084-3125): as IQ1_S with the super-scale in the top nibbles of the four scale words
 * and per-eight index extension and shift sign in the nibbles of qh; 56-byte blocks are 8-byte aligned */
template <> struct Lean<T_IQ1_M> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &t) {
        const uint8_t *blk = img + boff;
        const uint2 sw = *reinterpret_cast<const uint2 *>(blk + 48);
        const uint32_t dbits = ((sw.x >> 12) & 0x000Fu) | ((sw.x >> 24) & 0x00F0u) | ((sw.y >> 4) & 0x0F00u) | ((sw.y >> 16) & 0xF000u);
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const uint32_t word = ((g & 4) ? sw.y : sw.x) >> (16 * ((g >> 1) & 1));
        const float dl = half_bits_fast(dbits) * (float)(2 * (int)((word >> (6 * (g & 1) + 3 * (l >> 1))) & 7u) + 1);
        const uint32_t nib = ((uint32_t)blk[32 + 2 * g + (l >> 1)] >> (4 * (l & 1))) & 15u;
        const float dm1 = (nib & 8u) ? -1.125f : -0.875f;
        const uint2 cell = *reinterpret_cast<const uint2 *>(t.grid2 + (blk[4 * g + l] | ((nib & 7u) << 8)));
        return dl * fmaf(dm1, xs8, dot_u4(cell.y, xb, dot_u4(cell.x, xa, 0.0f)));
    }
};

/* TQ2_0 (:3161-3175): d * (q2 - 1) */
template <> struct Lean<T_TQ2_0> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &) {
        const float d = half_bits_fast(ld_u16(img + boff + 64));
        const uint2 q = ld8_at(img, boff + 32 * (k0 >> 7) + (k0 & 31));
        const int sh = 2 * ((k0 >> 5) & 3);
        return d * (dot_u4((q.y >> sh) & 0x03030303u, xb, dot_u4((q.x >> sh) & 0x03030303u, xa, 0.0f)) - xs8);
    }
};

/* Q1_0 (:1491-1503): +d where the bit is set, -d where it is clear: d * (2 * sum_{set} x - sum x) */
template <> struct Lean<T_Q1_0> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &) {
        const uint8_t *blk = img + boff;
        const float d = half_bits_fast(ld_u16(blk));
        const uint32_t bits = blk[2 + (k0 >> 3)];
        return d * fmaf(2.0f, dot_u4(spread4(bits >> 4), xb, dot_u4(spread4(bits), xa, 0.0f)), -xs8);
    }
};

/* MXFP4 (:2818-2830): 2^(e-128) * E2M1x2[nibble], the 16 values looked up like IQ4_NL's (stored + 128) */
template <> struct Lean<T_MXFP4> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &t) {
        const float d = e8m0_half(img[boff]);
        const uint2 q = ld8_at(img, boff + 1 + (k0 & 15));
        const int sh = (k0 >> 4) * 4;
        const uint32_t v0 = Lean<T_IQ4_NL>::look4((q.x >> sh) & 0x0F0F0F0Fu, t), v1 = Lean<T_IQ4_NL>::look4((q.y >> sh) & 0x0F0F0F0Fu, t);
        return d * fmaf(-128.0f, xs8, dot_u4(v1, xb, dot_u4(v0, xa, 0.0f)));
    }
};

/* NVFP4 (:2832-2848): ue4m3 scale per 16 elements, same value table */
template <> struct Lean<T_NVFP4> {
    __device__ static float dot8(const uint8_t *img, int boff, int k0, const float4 xa, const float4 xb, float xs8, const Tables &t) {
        const int sb = k0 >> 4;
        const float d = ue4m3_half(img[boff + sb]);
        const uint2 q = ld8_at(img, boff + 4 + 8 * sb);
        const int sh = ((k0 >> 3) & 1) * 4;
        const uint32_t v0 = Lean<T_IQ4_NL>::look4((q.x >> sh) & 0x0F0F0F0Fu, t), v1 = Lean<T_IQ4_NL>::look4((q.y >> sh) & 0x0F0F0F0Fu, t);
        return d * fmaf(-128.0f, xs8, dot_u4(v1, xb, dot_u4(v0, xa, 0.0f)));
    }
};

/* codebook a type's dot8 reads from LDS: its source in device memory and its size; the ternary
 * grid of IQ1_S/IQ1_M is staged with 1 added to every byte */
template <uint32_t T> struct Grid { static constexpr int kBytes = 0; static constexpr bool kPlusOne = false; __device__ static const uint32_t *src() { return nullptr; } };
#define QLIN_GRID(TT, TABLE, PLUS)                                                                \
    template <> struct Grid<TT> {                                                                 \
        static constexpr int kBytes = (int)sizeof(TABLE);                                          \
        static constexpr bool kPlusOne = PLUS;                                                     \
        __device__ static const uint32_t *src() { return reinterpret_cast<const uint32_t *>(TABLE); } \
    };
QLIN_GRID(T_IQ2_XXS, qlin_iq2xxs_grid, false)
QLIN_GRID(T_IQ3_S, qlin_iq3s_grid, false)
QLIN_GRID(T_IQ2_XS, qlin_iq2xs_grid, false)
QLIN_GRID(T_IQ2_S, qlin_iq2s_grid, false)
QLIN_GRID(T_IQ3_XXS, qlin_iq3xxs_grid, false)
QLIN_GRID(T_IQ1_S, qlin_iq1s_grid, true)
QLIN_GRID(T_IQ1_M, qlin_iq1s_grid, true)
#undef QLIN_GRID


template <uint32_t T>
__global__ void __launch_bounds__(1024)
gemv_stream_kernel(const JobView job, const float *__restrict__ x, int n_cols, int row_bytes, int image_bytes,
                   size_t row_stride, int depth, int rows_per_wg) {
    using C = Codec<T>;
    constexpr int GPB = C::BE / 8;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    /* LDS map: x [n_cols] | sums of eight x [n_cols/8] | i-quant grid (1..16 KB) where the type has one |
     * row images [waves][depth][image_bytes] */
    float *xs = reinterpret_cast<float *>(lds);
    float *xs8 = xs + n_cols;
    uint8_t *grid = reinterpret_cast<uint8_t *>(xs8 + (n_cols >> 3));
    uint8_t *images = grid + Grid<T>::kBytes;

    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); /* wave-uniform, and the compiler is told so */
    const int n_waves = blockDim.x >> 6, n_threads = blockDim.x;
    /* a workgroup owns rows_per_wg rows of the concatenated matrices; where two results are
     * combined (mode 2) a wave takes row r of the first matrix, then row r of the second */
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
    const int n_chunks = row_bytes >> 4;
    const int loads_per_row = (n_chunks + 63) >> 6;

    uint8_t *my_images = images + (size_t)wv * depth * image_bytes;
    const uint32_t my_images_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)my_images;
    /* Row i of this wave -> image i % depth. The loads are written as instructions: the data goes
     * to LDS at M0 + 16*lane, no register is held while it is in flight, and the compiler (which
     * would wait for every outstanding one of them before any LDS access) does not see them; the
     * waits are placed by hand below. Nothing else in this kernel uses M0. */
    auto issue = [&](int i) {
        const uint8_t *Wm;
        float *ym;
        int r;
        locate(i, Wm, ym, r);
        const uint4 *g = reinterpret_cast<const uint4 *>(Wm + (size_t)r * row_stride);
        const uint32_t img = my_images_lds + (uint32_t)((i % depth) * image_bytes);
        for (int c0 = 0; c0 < n_chunks; c0 += 64) {
            const uint32_t m0v = __builtin_amdgcn_readfirstlane(img + 16u * (uint32_t)c0);
            if (c0 + lane < n_chunks)
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt"
                             : : "v"(g + c0 + lane), "s"(m0v) : "memory");
        }
    };

    /* x first: it goes to LDS the same way, 1 KB per instruction and wave, so no register holds
     * data that is still in flight. A barrier makes every wave's x request precede every row
     * request, then the first rows are requested. */
    const int n4 = n_cols >> 2;
    const float4 *xg = reinterpret_cast<const float4 *>(x);
    const uint32_t xs_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)xs;
    for (int base = wv * 64; base < n4; base += n_threads) { /* uniform per wave */
        const uint32_t m0v = __builtin_amdgcn_readfirstlane(xs_lds + 16u * (uint32_t)base);
        if (base + lane < n4)
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                         : : "v"(xg + base + lane), "s"(m0v) : "memory");
    }
    asm volatile("s_barrier" ::: "memory");
    int issued = 0;
    for (; issued < depth && issued < my_rows; issued++) issue(issued);
    /* loads retire in order: at most the row loads outstanding means this wave's part of x has landed */
    wait_vm_at_most(issued * loads_per_row);
    Tables tab;
    tab.grid2 = reinterpret_cast<const uint64_t *>(grid);
    tab.grid3 = reinterpret_cast<const uint32_t *>(grid);
    tab.nl0 = tab.nl1 = tab.nl2 = tab.nl3 = 0;
    if (T == T_IQ4_NL || T == T_IQ4_XS || T == T_MXFP4 || T == T_NVFP4) {
        const uint4 v = *reinterpret_cast<const uint4 *>((T == T_MXFP4 || T == T_NVFP4) ? qlin_mxfp4_values : qlin_iq4nl_values);
        tab.nl0 = v.x ^ 0x80808080u; tab.nl1 = v.y ^ 0x80808080u; tab.nl2 = v.z ^ 0x80808080u; tab.nl3 = v.w ^ 0x80808080u;
    }
    if (Grid<T>::kBytes > 0)
        for (int t = threadIdx.x; t < Grid<T>::kBytes / 4; t += n_threads) {
            uint32_t v = Grid<T>::src()[t];
            if (Grid<T>::kPlusOne) /* bytes 0xFF, 0, 1 -> 0, 1, 2: add 1 per byte, no carry between bytes */
                v = ((v & 0x7F7F7F7Fu) + 0x01010101u) ^ (v & 0x80808080u);
            reinterpret_cast<uint32_t *>(grid)[t] = v;
        }
    __syncthreads();
    for (int t = threadIdx.x; t < (n_cols >> 3); t += n_threads) {
        const float4 a = *reinterpret_cast<const float4 *>(xs + 8 * t), b = *reinterpret_cast<const float4 *>(xs + 8 * t + 4);
        xs8[t] = ((a.x + a.y) + (a.z + a.w)) + ((b.x + b.y) + (b.z + b.w));
    }
    __syncthreads();

    static_assert(64 % GPB == 0, "a wave covers whole blocks");
    const int n_blocks = n_cols / C::BE;
    const int k0 = (lane % GPB) * 8, blk_first = lane / GPB;
    float gate_value = 0.0f;
    for (int i = 0; i < my_rows; i++) {
        /* rows i .. issued-1 are in flight, row i the oldest */
        wait_vm_at_most((issued - i - 1) * loads_per_row);
        const uint8_t *img = my_images + (size_t)(i % depth) * image_bytes;
        float acc = 0.0f;
        /* 64 is a multiple of the groups per block, so a lane keeps its position k0 inside the
         * block for the whole row and everything derived from k0 is loop-invariant */
        for (int blk = blk_first; blk < n_blocks; blk += 64 / GPB) {
            const float4 xa = *reinterpret_cast<const float4 *>(xs + blk * C::BE + k0);
            const float4 xb = *reinterpret_cast<const float4 *>(xs + blk * C::BE + k0 + 4);
            acc += Lean<T>::dot8(img, blk * C::BB, k0, xa, xb, xs8[blk * GPB + (k0 >> 3)], tab);
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
            /* the add is sent as a memory-side atomic: a read of y here would make the wave wait for
             * the row loads it has in flight */
            if (job.mode == 1) unsafeAtomicAdd(ym + r, s);
            else ym[r] = s;
        }
    }
}

template <uint32_t T>
bool stream_typed(const GemvJob &job, const float *x, int n_cols, int n_cu, hipStream_t stream, hipError_t *err,
                  size_t row_stride) {
    const size_t row_bytes = (size_t)(n_cols / Codec<T>::BE) * Codec<T>::BB;
    if (n_cols > 16384 || (n_cols & 31) || (row_bytes & 15) || row_bytes > 8192) return false;
    if (row_stride == 0) row_stride = row_bytes; /* rows that are a column range of longer ones keep those rows' pitch */
    if (row_stride & 15) return false;
    for (int m = 0; m < job.n_mat; m++)
        if ((uintptr_t)job.W[m] & 15) return false;
    if ((uintptr_t)x & 15) return false;
    const int n_rows = job.mode == kSiluMul ? job.n_rows[0] : job.total_rows();
    const size_t x_bytes = (size_t)n_cols * 4 + (size_t)(n_cols >> 3) * 4 + (size_t)Grid<T>::kBytes;
    const size_t lds_cap = 160 * 1024 - 16;
    /* 16 waves with two images each if that fits, else one image, else 8 waves */
    int waves = 16, depth = 2;
    if (x_bytes + (size_t)waves * depth * row_bytes > lds_cap) depth = 1;
    if (x_bytes + (size_t)waves * depth * row_bytes > lds_cap) { waves = 8; depth = 2; }
    if (x_bytes + (size_t)waves * depth * row_bytes > lds_cap) depth = 1;
    if (x_bytes + (size_t)waves * depth * row_bytes > lds_cap) return false;
    if ((size_t)((row_bytes >> 4) + 63) / 64 * depth > 15) return false; /* the hand-placed waits count to 15 */
    int rows_per_wg = (n_rows + n_cu - 1) / n_cu;
    if (rows_per_wg < 1) rows_per_wg = 1;
    const int grid = (n_rows + rows_per_wg - 1) / rows_per_wg;
    const size_t lds_bytes = x_bytes + (size_t)waves * depth * row_bytes + 16; /* + slack for ld8_at */
    static OnceFlag raised;
    if (!raised.is_set()) {
        *err = hipFuncSetAttribute((const void *)gemv_stream_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   160 * 1024);
        if (*err != hipSuccess) return true;
        raised.set();
    }
    const JobView view = job_view(job);
    hipLaunchKernelGGL((gemv_stream_kernel<T>), dim3(grid), dim3(waves * 64), lds_bytes, stream, view, x, n_cols,
                       (int)row_bytes, (int)row_bytes, row_stride, depth, rows_per_wg);
    *err = hipGetLastError();
    return true;
}

}  // namespace

bool launch_gemv_stream(uint32_t type, const GemvJob &job, const float *x, int n_cols, int n_cu,
                        hipStream_t stream, hipError_t *err, size_t row_stride) {
    *err = hipSuccess;
    switch (type) {
#define QLIN_CASE(TT) case TT: return stream_typed<TT>(job, x, n_cols, n_cu, stream, err, row_stride);
    QLIN_FOR_EACH_BLOCK_TYPE(QLIN_CASE)
    QLIN_FOR_EACH_DENSE_TYPE(QLIN_CASE)
#undef QLIN_CASE
    default: return false;
    }
}

}  // namespace qlin
