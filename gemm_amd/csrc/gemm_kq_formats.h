/*
 * gemm_kq_formats.h - what the fused prefill GEMM kernels (gemm_kq_wave4.hip, gemm_kq_wave4s.hip) share: the format
 * descriptions (what a lane takes from its row's block and the arithmetic that turns it into bf16 matrix operands) and
 * a few device helpers. A kernel hands a format description its context `c`: the members it reads and writes are
 * wa[2][4] (decoded operands), t (scratch), sc (the super-block's scales), kg (lane half), unit (the fp8 reading's
 * factor), w_rsrc and w_own (the lane's own row in memory, for formats with kExtraLoads).
 */
#ifndef QLIN_GEMM_KQ_FORMATS_H
#define QLIN_GEMM_KQ_FORMATS_H

#include "qlin_device.h"

namespace qlin {
namespace kq {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef float float2v __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void;

#define QLIN_INL __device__ __forceinline__ __attribute__((always_inline))

/* chunk-position swizzle of token row `row` */
QLIN_INL int fsw(int row) {
    const int j = (row >> 1) & 7;
    return (j & 1) | ((j & 2) << 1) | ((j & 4) >> 1);
}

/* two bytes 0x0q read as E4M3 are q times one fixed power of two (subnormal and first normal
 * binade form one linear ramp over q = 0..15) */
QLIN_INL float2v fp8_pair_lo(uint32_t v) { return __builtin_amdgcn_cvt_pk_f32_fp8((int)v, false); }
QLIN_INL float2v fp8_pair_hi(uint32_t v) { return __builtin_amdgcn_cvt_pk_f32_fp8((int)v, true); }

QLIN_INL uint32_t pack_bf16(float a, float b) {
    typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
    bf16x2 r;
    r[0] = (__bf16)a; /* round to nearest even */
    r[1] = (__bf16)b;
    return __builtin_bit_cast(uint32_t, r);
}

/* byte B of v as a float (v_cvt_f32_ubyteB) */
template <int B> QLIN_INL float ubyte_f32(uint32_t v) {
    float f;
    if (B == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(v));
    else if (B == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(v));
    else if (B == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(v));
    else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(v));
    return f;
}

/* s_waitcnt vmcnt(N) and nothing else (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8) */
template <int N> QLIN_INL void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

/* where a lane finds vector J of its raw data in its row's image: byte offset, and what the upper lane half adds */
struct VecAt { int off; int by_half; };

/* scratch of the decode that all formats share */
struct Temps {
    uint32_t cm, hb, lo, hi;
    float2v cp0, cp1;
    float f0, f1, f2, f3, w0, w1, w2, w3;
    float s_a, s_b, m_a, m_b, dl_a, dl_b, nml_a, nml_b; /* of the two sub-blocks (scale groups) of the tile in work */
};

/* four bytes cm -> four weights f * dl + off as two bf16 pairs of `out` (HALF 0: x, y; 1: z, w), in the pieces 2..6 of
 * a code word's seven */
template <int PH, int HALF, class C> QLIN_INL void bytes4_piece(C &c, float dl, float off, u32x4 &out) {
    Temps &t = c.t;
    if constexpr (PH == 2) { t.f0 = ubyte_f32<0>(t.cm); t.f1 = ubyte_f32<1>(t.cm); }
    else if constexpr (PH == 3) { t.f2 = ubyte_f32<2>(t.cm); t.f3 = ubyte_f32<3>(t.cm); }
    else if constexpr (PH == 4) { t.w0 = fmaf(t.f0, dl, off); t.w1 = fmaf(t.f1, dl, off); }
    else if constexpr (PH == 5) { t.w2 = fmaf(t.f2, dl, off); t.w3 = fmaf(t.f3, dl, off); }
    else if constexpr (HALF == 0) { out.x = pack_bf16(t.w0, t.w1); out.y = pack_bf16(t.w2, t.w3); }
    else { out.z = pack_bf16(t.w0, t.w1); out.w = pack_bf16(t.w2, t.w3); }
}

/* d, dmin and the 6-bit scales and mins of a Q4_K / Q5_K super-block from its 16-byte header (get_scale_min_k4,
 * common/ggml_dequant.h:1582-1590, four fields at a time) */
struct K4Scales { float d, dmin; uint32_t sc_lo, sc_hi, mn_lo, mn_hi; }; /* bytes 0..3 of lo = sub-blocks 0..3, of hi = 4..7 */
template <int P, class C> QLIN_INL void k4_unpack(C &c, const u32x4 &h, float d_factor) {
    if constexpr (P == 0) { c.sc.d = half_bits_fast(h.x & 0xFFFFu) * d_factor; c.sc.dmin = half_bits_fast(h.x >> 16); }
    else if constexpr (P == 1) { c.sc.sc_lo = h.y & 0x3F3F3F3Fu; c.sc.mn_lo = h.z & 0x3F3F3F3Fu; }
    else if constexpr (P == 2) c.sc.sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
    else c.sc.mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
}
/* pieces 0..3 of a tile: d*sc and -(dmin*m) of sub-blocks 2 TC (a) and 2 TC + 1 (b) */
template <int TC, int P, class C> QLIN_INL void k4_tile_scales(C &c) {
    Temps &t = c.t;
    if constexpr (P == 0) {
        t.s_a = ubyte_f32<2 * (TC & 1)>(TC & 2 ? c.sc.sc_hi : c.sc.sc_lo);
        t.s_b = ubyte_f32<2 * (TC & 1) + 1>(TC & 2 ? c.sc.sc_hi : c.sc.sc_lo);
    } else if constexpr (P == 1) {
        t.m_a = ubyte_f32<2 * (TC & 1)>(TC & 2 ? c.sc.mn_hi : c.sc.mn_lo);
        t.m_b = ubyte_f32<2 * (TC & 1) + 1>(TC & 2 ? c.sc.mn_hi : c.sc.mn_lo);
    } else if constexpr (P == 2) {
        t.dl_a = c.sc.d * t.s_a; t.dl_b = c.sc.d * t.s_b;
    } else {
        t.nml_a = -(c.sc.dmin * t.m_a); t.nml_b = -(c.sc.dmin * t.m_b);
    }
}

/* ---- Q4_K: 144-byte blocks = header | 4 x 32 code bytes (quarter c: low nibbles sub-block 2c, high 2c + 1). A lane
 * takes the header and code bytes 16 kg .. + 15 of every quarter. k-step s of a tile: low (s < 2) or high nibbles of
 * the lane's bytes 8 (s & 1) .. + 7. */
struct FQ4K {
    static constexpr int kBlockBytes = 144, kPieces = 9, kReq = 5, kLaneVec = 5, kPrepPieces = 4, kTilePieces = 44;
    static constexpr int kExtraVec = 0, kExtraLoads = 0, kKgChunk = 2;
    static constexpr bool kSwizzle = false;
    static constexpr int frag_xor(int s) { return ((s & 1) << 4) | ((s >> 1) << 6); }
    /* which k-step of a tile (0..3) tile piece P serves; 4, 5: both k-steps of half 0, 1; -1: all four */
    static constexpr int piece_step(int P) { return P < 4 ? -1 : ((P - 4) / 5) >> 1; }
    template <int J, class C> static QLIN_INL void extra_load(C &, u32x4 (&)[kLaneVec + kExtraVec], int) {}
    typedef K4Scales Scales;
    static QLIN_INL uint32_t piece_src(int part) { return 16u * part; }
    static constexpr VecAt vec_at(int j) { return j == 0 ? VecAt{0, 0} : VecAt{16 + 32 * (j - 1), 16}; }
    template <int P, class C> static QLIN_INL void prep(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) { k4_unpack<P>(c, raw[0], c.unit); }
    template <int TC, int WB, int P, class C> static QLIN_INL void tile_piece(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) {
        Temps &t = c.t;
        if constexpr (P < 4) k4_tile_scales<TC, P>(c);
        else {
            constexpr int dw = (P - 4) / 5, ph = (P - 4) % 5; /* code word 0..3: low nibbles of the lane's dwords, 4..7: high */
            const uint32_t word = raw[1 + TC][dw & 3];
            const float dl = dw < 4 ? t.dl_a : t.dl_b, nml = dw < 4 ? t.nml_a : t.nml_b;
            if constexpr (ph == 0) t.cm = (dw < 4 ? word : word >> 4) & 0x0F0F0F0Fu;
            else if constexpr (ph == 1) { t.cp0 = fp8_pair_lo(t.cm); t.cp1 = fp8_pair_hi(t.cm); }
            else if constexpr (ph == 2) { t.w0 = fmaf(t.cp0.x, dl, nml); t.w1 = fmaf(t.cp0.y, dl, nml); }
            else if constexpr (ph == 3) { t.w2 = fmaf(t.cp1.x, dl, nml); t.w3 = fmaf(t.cp1.y, dl, nml); }
            else if constexpr ((dw & 1) == 0) { c.wa[WB][dw >> 1].x = pack_bf16(t.w0, t.w1); c.wa[WB][dw >> 1].y = pack_bf16(t.w2, t.w3); }
            else { c.wa[WB][dw >> 1].z = pack_bf16(t.w0, t.w1); c.wa[WB][dw >> 1].w = pack_bf16(t.w2, t.w3); }
        }
    }
};

/* ---- Q5_K: 176-byte blocks = header | 32 bytes of fifth bits (bit g of byte l: element l of sub-block g) | 4 x 32 code
 * bytes as Q4_K. A lane takes the header, fifth-bit bytes 16 kg .. + 15 and its code bytes of every quarter; the 5-bit
 * code goes through the byte-to-float conversion (the fp8 reading is linear up to 15 only). */
struct FQ5K {
    static constexpr int kBlockBytes = 176, kPieces = 11, kReq = 6, kLaneVec = 6, kPrepPieces = 4, kTilePieces = 60;
    static constexpr int kExtraVec = 0, kExtraLoads = 0, kKgChunk = 2;
    static constexpr bool kSwizzle = false;
    static constexpr int frag_xor(int s) { return ((s & 1) << 4) | ((s >> 1) << 6); }
    /* which k-step of a tile (0..3) tile piece P serves; 4, 5: both k-steps of half 0, 1; -1: all four */
    static constexpr int piece_step(int P) { return P < 4 ? -1 : ((P - 4) / 7) >> 1; }
    template <int J, class C> static QLIN_INL void extra_load(C &, u32x4 (&)[kLaneVec + kExtraVec], int) {}
    typedef K4Scales Scales;
    static QLIN_INL uint32_t piece_src(int part) { return 16u * part; }
    static constexpr VecAt vec_at(int j) { return j == 0 ? VecAt{0, 0} : j == 1 ? VecAt{16, 16} : VecAt{48 + 32 * (j - 2), 16}; }
    template <int P, class C> static QLIN_INL void prep(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) { k4_unpack<P>(c, raw[0], 1.0f); }
    template <int TC, int WB, int P, class C> static QLIN_INL void tile_piece(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) {
        Temps &t = c.t;
        if constexpr (P < 4) k4_tile_scales<TC, P>(c);
        else {
            constexpr int dw = (P - 4) / 7, ph = (P - 4) % 7, hi = dw >> 2;
            const float dl = hi ? t.dl_b : t.dl_a, nml = hi ? t.nml_b : t.nml_a;
            if constexpr (ph == 0) t.cm = (hi ? raw[2 + TC][dw & 3] >> 4 : raw[2 + TC][dw & 3]) & 0x0F0F0F0Fu;
            else if constexpr (ph == 1) { t.hb = (raw[1][dw & 3] >> (2 * TC + hi)) & 0x01010101u; t.cm |= t.hb << 4; }
            else bytes4_piece<ph, dw & 1>(c, dl, nml, c.wa[WB][dw >> 1]);
        }
    }
};

/* ---- Q6_K: 210-byte blocks = 128 nibble bytes | 64 bytes of bit pairs | 16 int8 scales (one per 16 elements) | d.
 * Half h of a super-block, element 32 seg + l: nibble seg >> 1 of byte 64 h + 32 (seg & 1) + l, bits 2 seg of byte
 * 128 + 32 h + l; tile c = half c >> 1, segments 2 (c & 1) and 2 (c & 1) + 1. A lane takes l = 16 kg .. + 15: per half two
 * runs of nibble bytes and one of bit pairs, and the scales and d. In LDS a row's image is 13 pieces of the block as
 * they come, bytes 194..209 (d in its last two) as the 14th, and one of padding (15: an odd stride). */
struct Q6Scales { float d; };
struct FQ6K {
    static constexpr int kBlockBytes = 210, kPieces = 15, kReq = 8, kLaneVec = 8, kPrepPieces = 1, kTilePieces = 60;
    static constexpr int kExtraVec = 0, kExtraLoads = 0, kKgChunk = 2;
    static constexpr bool kSwizzle = false;
    static constexpr int frag_xor(int s) { return ((s & 1) << 4) | ((s >> 1) << 6); }
    /* which k-step of a tile (0..3) tile piece P serves; 4, 5: both k-steps of half 0, 1; -1: all four */
    static constexpr int piece_step(int P) { return P < 4 ? 4 + (P >> 1) : ((P - 4) / 7) >> 1; }
    template <int J, class C> static QLIN_INL void extra_load(C &, u32x4 (&)[kLaneVec + kExtraVec], int) {}
    typedef Q6Scales Scales;
    static QLIN_INL uint32_t piece_src(int part) { return part < 13 ? 16u * part : part == 13 ? 194u : 0u; }
    static constexpr VecAt vec_at(int j) {
        return j < 4 ? VecAt{64 * (j >> 1) + 32 * (j & 1), 16} : j < 6 ? VecAt{128 + 32 * (j - 4), 16} : j == 6 ? VecAt{192, 0} : VecAt{208, 0};
    }
    template <int P, class C> static QLIN_INL void prep(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) { c.sc.d = half_bits_fast(raw[7].w >> 16); }
    template <int TC, int WB, int P, class C> static QLIN_INL void tile_piece(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) {
        Temps &t = c.t;
        constexpr int half = TC >> 1, p = TC & 1;
        if constexpr (P < 4) {
            /* scale 8 half + 4 p + 2 jj + kg: byte 2 jj + kg of dword 2 half + p of the sixteen */
            constexpr int jj = P >> 1;
            if constexpr ((P & 1) == 0) {
                const int sv = __builtin_amdgcn_sbfe((int)raw[6][2 * half + p], 8 * (2 * jj + c.kg), 8);
                (jj ? t.s_b : t.s_a) = (float)sv;
            } else if constexpr (jj == 0) { t.dl_a = c.sc.d * t.s_a; t.nml_a = -32.0f * t.dl_a; }
            else { t.dl_b = c.sc.d * t.s_b; t.nml_b = -32.0f * t.dl_b; }
        } else {
            constexpr int dw = (P - 4) / 7, ph = (P - 4) % 7, jj = dw >> 2;
            const float dl = jj ? t.dl_b : t.dl_a, off = jj ? t.nml_b : t.nml_a;
            if constexpr (ph == 0) t.cm = (p ? raw[2 * half + jj][dw & 3] >> 4 : raw[2 * half + jj][dw & 3]) & 0x0F0F0F0Fu;
            else if constexpr (ph == 1) { t.hb = (raw[4 + half][dw & 3] >> (4 * p + 2 * jj)) & 0x03030303u; t.cm |= t.hb << 4; }
            else bytes4_piece<ph, dw & 1>(c, dl, off, c.wa[WB][dw >> 1]);
        }
    }
};

/* ---- Q8_0: 34-byte blocks = d | 32 int8 codes; eight of them are the unit of the pipeline. Only the codes go through
 * LDS (two 16-byte pieces per block, fetched from 34 b + 2 and 34 b + 18: the load-to-LDS path takes any source
 * alignment, and the image's vectors come out aligned), 512 bytes per row: with the four activation stages that is all
 * of the 160 KB. The scales come straight from memory into registers, four two-byte loads per lane and unit. So that
 * four suffice, the k order inside a tile differs from the K-quants': lane half kg takes ALL codes of block 2 c + kg of
 * tile c, k-step s its codes 8 s .. 8 s + 7, and the activation fragment of that lane half is chunk 4 kg + s. */
struct FQ8_0 {
    static constexpr int kBlockBytes = 272, kPieces = 16, kReq = 8, kLaneVec = 8, kPrepPieces = 0, kTilePieces = 49;
    static constexpr int kExtraVec = 1, kExtraLoads = 4, kKgChunk = 4;
    /* a row's image is 256 bytes, a whole turn of the LDS banks: piece p of row r sits at position p ^ (r % 16) of the
     * row, so that 16 rows reading the same piece hit 16 different bank groups */
    static constexpr bool kSwizzle = true;
    struct Scales {};
    static constexpr int frag_xor(int s) { return s << 4; }
    /* which k-step of a tile (0..3) tile piece P serves; 4, 5: both k-steps of half 0, 1; -1: all four */
    static constexpr int piece_step(int P) { return P < 1 ? -1 : ((P - 1) / 6) >> 1; }
    static QLIN_INL uint32_t piece_src(int part) { return 34u * (part >> 1) + 2u + 16u * (part & 1); }
    /* vector j: half j & 1 of the codes of block 2 (j >> 1) + kg */
    static constexpr VecAt vec_at(int j) { return VecAt{64 * (j >> 1) + 16 * (j & 1), 32}; }
    /* scale J (0..3) of super-block `sb`: d of block 2 J + kg of the lane's own row, kept as the 16 bits that came */
    template <int J, class C> static QLIN_INL void extra_load(C &c, u32x4 (&raw)[kLaneVec + kExtraVec], int sb) {
        raw[kLaneVec][J] = __builtin_amdgcn_raw_buffer_load_b16(c.w_rsrc, c.w_own + 34u * c.kg + 68u * J, sb * kBlockBytes, 0);
    }
    template <int P, class C> static QLIN_INL void prep(C &, const u32x4 (&)[kLaneVec + kExtraVec]) {}
    template <int TC, int WB, int P, class C> static QLIN_INL void tile_piece(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) {
        Temps &t = c.t;
        if constexpr (P == 0) { t.dl_a = half_bits_fast(raw[kLaneVec][TC] & 0xFFFFu); t.nml_a = -128.0f * t.dl_a; }
        else {
            /* the int8 code with its sign bit flipped is code + 128 as an unsigned byte */
            constexpr int dw = (P - 1) / 6, ph = (P - 1) % 6;
            if constexpr (ph == 0) t.cm = raw[2 * TC + (dw >> 2)][dw & 3] ^ 0x80808080u;
            else bytes4_piece<ph + 1, dw & 1>(c, t.dl_a, t.nml_a, c.wa[WB][dw >> 1]);
        }
    }
};

/* ---- IQ4_NL: 18-byte blocks = d | 16 bytes whose low nibbles are elements 0..15 and high nibbles 16..31, each nibble an
 * index into a table of 16 int8 values (common/ggml_dequant.h:2942-2954); eight blocks (144 bytes, like a Q4_K
 * super-block) are the unit. Both lane halves take the same bytes - half kg their nibble kg - so a lane keeps the whole
 * 144-byte image of its row in nine vectors and cuts a block's four code dwords out of them at offsets known at
 * compile time (blocks with an even index start two bytes into a dword: one v_alignbyte per dword). The table lookup
 * is two byte permutes (entries 0..7, 8..15, stored with 128 added so that they are unsigned bytes) and a select on
 * bit 3 of the index: about 5 vector instructions per weight, more than one wave per SIMD can issue beside the matrix
 * instructions, but far fewer than the decode to bf16 in memory costs. */
struct FIQ4NL {
    static constexpr int kBlockBytes = 144, kPieces = 9, kReq = 5, kLaneVec = 9, kPrepPieces = 0, kTilePieces = 82;
    static constexpr int kExtraVec = 0, kExtraLoads = 0, kKgChunk = 2;
    static constexpr bool kSwizzle = false;
    struct Scales {};
    static constexpr int frag_xor(int s) { return ((s & 1) << 4) | ((s >> 1) << 6); }
    /* which k-step of a tile (0..3) tile piece P serves; 4, 5: both k-steps of half 0, 1; -1: all four */
    static constexpr int piece_step(int P) { return P < 2 ? 4 + P : ((P - 2) / 10) >> 1; }
    static QLIN_INL uint32_t piece_src(int part) { return 16u * part; }
    static constexpr VecAt vec_at(int j) { return VecAt{16 * j, 0}; }
    template <int J, class C> static QLIN_INL void extra_load(C &, u32x4 (&)[kLaneVec + kExtraVec], int) {}
    template <int P, class C> static QLIN_INL void prep(C &, const u32x4 (&)[kLaneVec + kExtraVec]) {}
    /* dword I of the row image */
    template <int I> static QLIN_INL uint32_t image_dword(const u32x4 (&raw)[kLaneVec + kExtraVec]) { return raw[I >> 2][I & 3]; }
    template <int TC, int WB, int P, class C> static QLIN_INL void tile_piece(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) {
        Temps &t = c.t;
        if constexpr (P < 2) {
            /* d of block 2 TC + P: bytes 18 b, 18 b + 1 of the image */
            constexpr int b = 2 * TC + P, at = 18 * b;
            const float d = half_bits_fast((image_dword<(at >> 2)>(raw) >> (8 * (at & 3))) & 0xFFFFu);
            if constexpr (P == 0) { t.dl_a = d; t.nml_a = -128.0f * d; }
            else { t.dl_b = d; t.nml_b = -128.0f * d; }
        } else {
            constexpr int dw = (P - 2) / 10, ph = (P - 2) % 10, b = 2 * TC + (dw >> 2), at = 18 * b + 2 + 4 * (dw & 3);
            const float dl = (dw >> 2) ? t.dl_b : t.dl_a, off = (dw >> 2) ? t.nml_b : t.nml_a;
            if constexpr (ph == 0) {
                uint32_t src;
                if constexpr ((at & 3) == 0) src = image_dword<(at >> 2)>(raw);
                else src = __builtin_amdgcn_alignbyte(image_dword<(at >> 2) + 1>(raw), image_dword<(at >> 2)>(raw), at & 3);
                t.hb = src >> (4u * (uint32_t)c.kg); /* the lane half's nibble of every byte */
            } else if constexpr (ph == 1) {
                t.cm = t.hb & 0x0F0F0F0Fu;
                t.hb = t.cm & 0x07070707u;
            } else if constexpr (ph == 2) {
                t.lo = __builtin_amdgcn_perm(0x766A5D4Fu, 0x3F2D1801u, t.hb); /* table entries 0..7, + 128 */
                t.hi = __builtin_amdgcn_perm(0xF1D9C5B5u, 0xA6998D81u, t.hb); /* entries 8..15 */
            } else if constexpr (ph == 3) {
                t.hb = (t.cm >> 3) & 0x01010101u;
            } else if constexpr (ph == 4) {
                t.hb *= 255u; /* 0xFF in the bytes whose index is 8 or more */
                t.cm = (t.hb & t.hi) | (~t.hb & t.lo);
            } else {
                bytes4_piece<ph - 3, dw & 1>(c, dl, off, c.wa[WB][dw >> 1]);
            }
        }
    }
};

/* ---- Q4_0: 18-byte blocks = d | 16 bytes, elements 0..15 in the low nibbles, 16..31 in the high ones, value d (q - 8)
 * (common/ggml_dequant.h:2850-2862). The layout and the lane roles of IQ4_NL with the arithmetic of Q4_K: the nibbles
 * go through the fp8 reading. */
struct FQ4_0 {
    static constexpr int kBlockBytes = 144, kPieces = 9, kReq = 5, kLaneVec = 9, kPrepPieces = 0, kTilePieces = 50;
    static constexpr int kExtraVec = 0, kExtraLoads = 0, kKgChunk = 2;
    static constexpr bool kSwizzle = false;
    struct Scales {};
    static constexpr int frag_xor(int s) { return ((s & 1) << 4) | ((s >> 1) << 6); }
    /* which k-step of a tile (0..3) tile piece P serves; 4, 5: both k-steps of half 0, 1; -1: all four */
    static constexpr int piece_step(int P) { return P < 2 ? 4 + P : ((P - 2) / 6) >> 1; }
    static QLIN_INL uint32_t piece_src(int part) { return 16u * part; }
    static constexpr VecAt vec_at(int j) { return VecAt{16 * j, 0}; }
    template <int J, class C> static QLIN_INL void extra_load(C &, u32x4 (&)[kLaneVec + kExtraVec], int) {}
    template <int P, class C> static QLIN_INL void prep(C &, const u32x4 (&)[kLaneVec + kExtraVec]) {}
    template <int TC, int WB, int P, class C> static QLIN_INL void tile_piece(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) {
        Temps &t = c.t;
        if constexpr (P < 2) {
            constexpr int b = 2 * TC + P, at = 18 * b;
            const float d = half_bits_fast((FIQ4NL::image_dword<(at >> 2)>(raw) >> (8 * (at & 3))) & 0xFFFFu);
            if constexpr (P == 0) { t.dl_a = d * c.unit; t.nml_a = -8.0f * d; }
            else { t.dl_b = d * c.unit; t.nml_b = -8.0f * d; }
        } else {
            constexpr int dw = (P - 2) / 6, ph = (P - 2) % 6, b = 2 * TC + (dw >> 2), at = 18 * b + 2 + 4 * (dw & 3);
            const float dl = (dw >> 2) ? t.dl_b : t.dl_a, off = (dw >> 2) ? t.nml_b : t.nml_a;
            if constexpr (ph == 0) {
                uint32_t src;
                if constexpr ((at & 3) == 0) src = FIQ4NL::image_dword<(at >> 2)>(raw);
                else src = __builtin_amdgcn_alignbyte(FIQ4NL::image_dword<(at >> 2) + 1>(raw), FIQ4NL::image_dword<(at >> 2)>(raw), at & 3);
                t.hb = src >> (4u * (uint32_t)c.kg);
            } else if constexpr (ph == 1) t.cm = t.hb & 0x0F0F0F0Fu;
            else if constexpr (ph == 2) { t.cp0 = fp8_pair_lo(t.cm); t.cp1 = fp8_pair_hi(t.cm); }
            else if constexpr (ph == 3) { t.w0 = fmaf(t.cp0.x, dl, off); t.w1 = fmaf(t.cp0.y, dl, off); }
            else if constexpr (ph == 4) { t.w2 = fmaf(t.cp1.x, dl, off); t.w3 = fmaf(t.cp1.y, dl, off); }
            else if constexpr ((dw & 1) == 0) { c.wa[WB][dw >> 1].x = pack_bf16(t.w0, t.w1); c.wa[WB][dw >> 1].y = pack_bf16(t.w2, t.w3); }
            else { c.wa[WB][dw >> 1].z = pack_bf16(t.w0, t.w1); c.wa[WB][dw >> 1].w = pack_bf16(t.w2, t.w3); }
        }
    }
};

/* ---- IQ4_XS: 136-byte super-blocks = d | 8 x 2 high scale bits | 8 x 4 low scale bits | 8 x 16 code bytes; sub-block g
 * (32 elements) = the nibbles of bytes 8 + 16 g .. + 15 as in IQ4_NL, through the same table, times d (ls_g - 32)
 * (common/ggml_dequant.h:2956-2973). A row's image is nine 16-byte pieces (the last one half belongs to the next
 * super-block); the code dwords are aligned. */
struct XsScales { float d; };
struct FIQ4XS {
    static constexpr int kBlockBytes = 136, kPieces = 9, kReq = 5, kLaneVec = 9, kPrepPieces = 1, kTilePieces = 88;
    static constexpr int kExtraVec = 0, kExtraLoads = 0, kKgChunk = 2;
    static constexpr bool kSwizzle = false;
    typedef XsScales Scales;
    static constexpr int frag_xor(int s) { return ((s & 1) << 4) | ((s >> 1) << 6); }
    /* which k-step of a tile (0..3) tile piece P serves; 4, 5: both k-steps of half 0, 1; -1: all four */
    static constexpr int piece_step(int P) { return P < 8 ? 4 + (P >> 2) : ((P - 8) / 10) >> 1; }
    static QLIN_INL uint32_t piece_src(int part) { return 16u * part; }
    static constexpr VecAt vec_at(int j) { return VecAt{16 * j, 0}; }
    template <int J, class C> static QLIN_INL void extra_load(C &, u32x4 (&)[kLaneVec + kExtraVec], int) {}
    template <int P, class C> static QLIN_INL void prep(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) {
        c.sc.d = half_bits_fast(raw[0].x & 0xFFFFu);
    }
    template <int TC, int WB, int P, class C> static QLIN_INL void tile_piece(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) {
        Temps &t = c.t;
        if constexpr (P < 8) {
            /* four pieces per sub-block g = 2 TC + P / 4: the 6-bit scale, then d (ls - 32) and -128 times that */
            constexpr int g = 2 * TC + (P >> 2), q = P & 3;
            float &dl = (P >> 2) ? t.dl_b : t.dl_a, &nml = (P >> 2) ? t.nml_b : t.nml_a;
            if constexpr (q == 0) { t.lo = (raw[0].y >> (8 * (g >> 1) + 4 * (g & 1))) & 15u; t.hi = (raw[0].x >> (16 + 2 * g)) & 3u; }
            else if constexpr (q == 1) t.lo = (t.lo | (t.hi << 4)) - 32u;
            else if constexpr (q == 2) dl = c.sc.d * (float)(int)t.lo;
            else nml = -128.0f * dl;
        } else {
            constexpr int dw = (P - 8) / 10, ph = (P - 8) % 10, g = 2 * TC + (dw >> 2);
            const float dl = (dw >> 2) ? t.dl_b : t.dl_a, off = (dw >> 2) ? t.nml_b : t.nml_a;
            if constexpr (ph == 0) {
                t.hb = FIQ4NL::image_dword<2 + 4 * g + (dw & 3)>(raw) >> (4u * (uint32_t)c.kg);
            } else if constexpr (ph == 1) {
                t.cm = t.hb & 0x0F0F0F0Fu;
                t.hb = t.cm & 0x07070707u;
            } else if constexpr (ph == 2) {
                t.lo = __builtin_amdgcn_perm(0x766A5D4Fu, 0x3F2D1801u, t.hb);
                t.hi = __builtin_amdgcn_perm(0xF1D9C5B5u, 0xA6998D81u, t.hb);
            } else if constexpr (ph == 3) {
                t.hb = (t.cm >> 3) & 0x01010101u;
            } else if constexpr (ph == 4) {
                t.hb *= 255u;
                t.cm = (t.hb & t.hi) | (~t.hb & t.lo);
            } else {
                bytes4_piece<ph - 3, dw & 1>(c, dl, off, c.wa[WB][dw >> 1]);
            }
        }
    }
};

/* ---- Q2_K and Q3_K share their element order: half h (128 elements) of a super-block, shift j (0..3), 16-element group
 * sub, element l: bits 2 j of code byte 32 h + 16 sub + l, scale 8 h + 2 j + sub (common/ggml_dequant.h:1505-1580). Tile c
 * is half c >> 1, shifts 2 (c & 1) and 2 (c & 1) + 1; lane half kg takes sub = kg, so its 16 code bytes per half serve
 * both tiles of the half, and its two scales of a tile are bytes kg and kg + 2 of dword 2 h + (c & 1) of the sixteen.
 * k-step s: shift 2 (c & 1) + (s >> 1), the lane's bytes 8 (s & 1) .. + 7. The codes (0..3, with Q3_K's third bit 0..7) go
 * through the fp8 reading. */
template <int TC, int DW> struct K23 { static constexpr int half = TC >> 1, j = 2 * (TC & 1) + (DW >> 2), sdw = 2 * half + (TC & 1); };

/* Q2_K: 84-byte blocks = 16 scale bytes (low nibble scale, high nibble min) | 64 code bytes | d | dmin; (d sc) q - dmin m.
 * A row's image is the first five 16-byte pieces and bytes 68..83 as the sixth (d and dmin in its last dword; a fetch of
 * bytes 80..95 would leave the row, and the buffer at its last row). */
struct Q2Scales { float d, dmin; };
struct FQ2K {
    static constexpr int kBlockBytes = 84, kPieces = 6, kReq = 3, kLaneVec = 4, kPrepPieces = 1, kTilePieces = 44;
    static constexpr int kExtraVec = 0, kExtraLoads = 0, kKgChunk = 2;
    static constexpr bool kSwizzle = false;
    typedef Q2Scales Scales;
    static constexpr int frag_xor(int s) { return ((s & 1) << 4) | ((s >> 1) << 6); }
    /* which k-step of a tile (0..3) tile piece P serves; 4, 5: both k-steps of half 0, 1; -1: all four */
    static constexpr int piece_step(int P) { return P < 4 ? -1 : ((P - 4) / 5) >> 1; }
    static QLIN_INL uint32_t piece_src(int part) { return part < 5 ? 16u * part : 68u; }
    /* vector 0: the scales; 1, 2: the lane's code bytes of half 0, 1; 3: the piece with d and dmin */
    static constexpr VecAt vec_at(int j) { return j == 0 ? VecAt{0, 0} : j < 3 ? VecAt{16 + 32 * (j - 1), 16} : VecAt{80, 0}; }
    template <int J, class C> static QLIN_INL void extra_load(C &, u32x4 (&)[kLaneVec + kExtraVec], int) {}
    template <int P, class C> static QLIN_INL void prep(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) {
        c.sc.d = half_bits_fast(raw[3].w & 0xFFFFu) * c.unit;
        c.sc.dmin = half_bits_fast(raw[3].w >> 16);
    }
    template <int TC, int WB, int P, class C> static QLIN_INL void tile_piece(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) {
        Temps &t = c.t;
        if constexpr (P < 4) {
            const uint32_t word = raw[0][K23<TC, 0>::sdw], at = 8u * (uint32_t)c.kg;
            if constexpr (P == 0) { t.s_a = (float)__builtin_amdgcn_ubfe(word, at, 4); t.s_b = (float)__builtin_amdgcn_ubfe(word, at + 16, 4); }
            else if constexpr (P == 1) { t.m_a = (float)__builtin_amdgcn_ubfe(word, at + 4, 4); t.m_b = (float)__builtin_amdgcn_ubfe(word, at + 20, 4); }
            else if constexpr (P == 2) { t.dl_a = c.sc.d * t.s_a; t.dl_b = c.sc.d * t.s_b; }
            else { t.nml_a = -(c.sc.dmin * t.m_a); t.nml_b = -(c.sc.dmin * t.m_b); }
        } else {
            constexpr int dw = (P - 4) / 5, ph = (P - 4) % 5;
            typedef K23<TC, dw> G;
            const float dl = dw < 4 ? t.dl_a : t.dl_b, nml = dw < 4 ? t.nml_a : t.nml_b;
            if constexpr (ph == 0) t.cm = (raw[1 + G::half][dw & 3] >> (2 * G::j)) & 0x03030303u;
            else if constexpr (ph == 1) { t.cp0 = fp8_pair_lo(t.cm); t.cp1 = fp8_pair_hi(t.cm); }
            else if constexpr (ph == 2) { t.w0 = fmaf(t.cp0.x, dl, nml); t.w1 = fmaf(t.cp0.y, dl, nml); }
            else if constexpr (ph == 3) { t.w2 = fmaf(t.cp1.x, dl, nml); t.w3 = fmaf(t.cp1.y, dl, nml); }
            else if constexpr ((dw & 1) == 0) { c.wa[WB][dw >> 1].x = pack_bf16(t.w0, t.w1); c.wa[WB][dw >> 1].y = pack_bf16(t.w2, t.w3); }
            else { c.wa[WB][dw >> 1].z = pack_bf16(t.w0, t.w1); c.wa[WB][dw >> 1].w = pack_bf16(t.w2, t.w3); }
        }
    }
};

/* Q3_K: 110-byte blocks = 32 bytes of third bits (bit 4 h + j of byte 16 sub + l) | 64 code bytes | 12 bytes of sixteen
 * 6-bit scales | d; (d (sc - 32)) (q - 4) with q the three bits. A row's image is the first six pieces and bytes 94..109
 * as the seventh (ending with the block, as Q2_K's last), 112 bytes: a stride that spreads 16 rows over all banks. The
 * packed scales start two bytes into that piece; once per super-block they are cut out and spread to sixteen bytes. */
struct Q3Scales { float d, dm4; uint32_t a0, a1, hi, sc[4]; }; /* d with the fp8 reading's factor, dm4 = -4 d without */
struct FQ3K {
    static constexpr int kBlockBytes = 110, kPieces = 7, kReq = 4, kLaneVec = 4, kPrepPieces = 4, kTilePieces = 52;
    static constexpr int kExtraVec = 0, kExtraLoads = 0, kKgChunk = 2;
    static constexpr bool kSwizzle = false;
    typedef Q3Scales Scales;
    static constexpr int frag_xor(int s) { return ((s & 1) << 4) | ((s >> 1) << 6); }
    /* which k-step of a tile (0..3) tile piece P serves; 4, 5: both k-steps of half 0, 1; -1: all four */
    static constexpr int piece_step(int P) { return P < 4 ? -1 : ((P - 4) / 6) >> 1; }
    static QLIN_INL uint32_t piece_src(int part) { return part < 6 ? 16u * part : 94u; }
    /* vector 0: the lane's third-bit bytes; 1, 2: its code bytes of half 0, 1; 3: the piece with scales and d */
    static constexpr VecAt vec_at(int j) { return j == 0 ? VecAt{0, 16} : j < 3 ? VecAt{32 + 32 * (j - 1), 16} : VecAt{96, 0}; }
    template <int J, class C> static QLIN_INL void extra_load(C &, u32x4 (&)[kLaneVec + kExtraVec], int) {}
    template <int P, class C> static QLIN_INL void prep(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) {
        const u32x4 &v = raw[3]; /* block bytes 94..109: scale bytes 0..11 at 2..13, d at 14 */
        if constexpr (P == 0) { c.sc.a0 = __builtin_amdgcn_alignbyte(v.y, v.x, 2); c.sc.a1 = __builtin_amdgcn_alignbyte(v.z, v.y, 2); }
        else if constexpr (P == 1) {
            c.sc.hi = __builtin_amdgcn_alignbyte(v.w, v.z, 2);
            c.sc.dm4 = -4.0f * half_bits_fast(v.w >> 16);
            c.sc.d = c.sc.dm4 * (-0.25f * c.unit);
        }
        else if constexpr (P == 2) {
            c.sc.sc[0] = (c.sc.a0 & 0x0F0F0F0Fu) | ((c.sc.hi & 0x03030303u) << 4);
            c.sc.sc[1] = (c.sc.a1 & 0x0F0F0F0Fu) | (((c.sc.hi >> 2) & 0x03030303u) << 4);
        } else {
            c.sc.sc[2] = ((c.sc.a0 >> 4) & 0x0F0F0F0Fu) | (((c.sc.hi >> 4) & 0x03030303u) << 4);
            c.sc.sc[3] = ((c.sc.a1 >> 4) & 0x0F0F0F0Fu) | (((c.sc.hi >> 6) & 0x03030303u) << 4);
        }
    }
    template <int TC, int WB, int P, class C> static QLIN_INL void tile_piece(C &c, const u32x4 (&raw)[kLaneVec + kExtraVec]) {
        Temps &t = c.t;
        if constexpr (P < 4) {
            const uint32_t word = c.sc.sc[K23<TC, 0>::sdw], at = 8u * (uint32_t)c.kg;
            if constexpr (P == 0) t.s_a = (float)((int)__builtin_amdgcn_ubfe(word, at, 8) - 32);
            else if constexpr (P == 1) t.s_b = (float)((int)__builtin_amdgcn_ubfe(word, at + 16, 8) - 32);
            else if constexpr (P == 2) { t.dl_a = c.sc.d * t.s_a; t.dl_b = c.sc.d * t.s_b; }
            else { t.nml_a = c.sc.dm4 * t.s_a; t.nml_b = c.sc.dm4 * t.s_b; }
        } else {
            constexpr int dw = (P - 4) / 6, ph = (P - 4) % 6;
            typedef K23<TC, dw> G;
            const float dl = dw < 4 ? t.dl_a : t.dl_b, nml = dw < 4 ? t.nml_a : t.nml_b;
            if constexpr (ph == 0) t.cm = (raw[1 + G::half][dw & 3] >> (2 * G::j)) & 0x03030303u;
            else if constexpr (ph == 1) { t.hb = (raw[0][dw & 3] >> (4 * G::half + G::j)) & 0x01010101u; t.cm |= t.hb << 2; }
            else if constexpr (ph == 2) { t.cp0 = fp8_pair_lo(t.cm); t.cp1 = fp8_pair_hi(t.cm); }
            else if constexpr (ph == 3) { t.w0 = fmaf(t.cp0.x, dl, nml); t.w1 = fmaf(t.cp0.y, dl, nml); }
            else if constexpr (ph == 4) { t.w2 = fmaf(t.cp1.x, dl, nml); t.w3 = fmaf(t.cp1.y, dl, nml); }
            else if constexpr ((dw & 1) == 0) { c.wa[WB][dw >> 1].x = pack_bf16(t.w0, t.w1); c.wa[WB][dw >> 1].y = pack_bf16(t.w2, t.w3); }
            else { c.wa[WB][dw >> 1].z = pack_bf16(t.w0, t.w1); c.wa[WB][dw >> 1].w = pack_bf16(t.w2, t.w3); }
        }
    }
};

/* Does a wave that takes half WK of a tile's k-steps (2 WK and 2 WK + 1) run tile piece q of format F? */
template <class F, int WK> constexpr bool owns_piece(int q) {
    const int st = F::piece_step(q);
    return st < 0 || (st < 4 ? st >> 1 : st - 4) == WK;
}
/* The decode pieces of a tile that such a wave runs: the NPREP pieces of the next super-block's scales (last tile of
 * a super-block), then its tile pieces, in their order. */
template <class F, int WK, int NPREP> struct Owned {
    static constexpr int count() {
        int n = NPREP;
        for (int q = 0; q < F::kTilePieces; q++) n += owns_piece<F, WK>(q) ? 1 : 0;
        return n;
    }
    /* the i-th of them: below NPREP a prep piece, else NPREP + the tile piece's number */
    static constexpr int nth(int i) {
        if (i < NPREP) return i;
        int n = NPREP;
        for (int q = 0; q < F::kTilePieces; q++)
            if (owns_piece<F, WK>(q)) {
                if (n == i) return NPREP + q;
                n++;
            }
        return -1;
    }
};

/* Up to three weight tensors of one format and one K against the same activations in one launch (the Q, K and V
 * projections of a prefill chunk: a 1024-row tensor alone is 64 small tiles at 512 tokens; gate and up). Row tiles are
 * numbered through the tensors: tensor i owns tiles end[i - 1] .. end[i] - 1. */
struct TileSet { /* named members, not arrays: the kernels pick by comparisons on scalar registers, never by an index */
    const uint8_t *W0, *W1, *W2;
    float *Y0, *Y1, *Y2;
    int n_rows0, n_rows1, n_rows2, ldy0, ldy1, ldy2, end0, end1, end2;
};
/* host: entries past n_mat repeat the last tensor and own no tile -> the number of row tiles */
inline int fill_tile_set(TileSet &set, int n_mat, const void *const *W, float *const *Y, const int *n_rows, const int *ldy,
                         int rows_per_tile) {
    int n_tiles = 0, end[3];
    for (int i = 0; i < 3; i++) {
        if (i < n_mat) n_tiles += (n_rows[i] + rows_per_tile - 1) / rows_per_tile;
        end[i] = n_tiles;
    }
    const int j1 = n_mat > 1 ? 1 : 0, j2 = n_mat > 2 ? 2 : j1;
    set.W0 = (const uint8_t *)W[0]; set.W1 = (const uint8_t *)W[j1]; set.W2 = (const uint8_t *)W[j2];
    set.Y0 = Y[0]; set.Y1 = Y[j1]; set.Y2 = Y[j2];
    set.n_rows0 = n_rows[0]; set.n_rows1 = n_rows[j1]; set.n_rows2 = n_rows[j2];
    set.ldy0 = ldy[0]; set.ldy1 = ldy[j1]; set.ldy2 = ldy[j2];
    set.end0 = end[0]; set.end1 = end[1]; set.end2 = end[2];
    return n_tiles;
}
/* device: the tensor of row tile `tile_all` (below end2) and the tile's number inside it */
struct TileOf { const uint8_t *W; float *Y; int n_rows, ldy, tile; };
QLIN_INL TileOf tile_of(const TileSet &set, int tile_all) {
    TileOf t;
    if (tile_all < set.end0) { t.W = set.W0; t.Y = set.Y0; t.n_rows = set.n_rows0; t.ldy = set.ldy0; t.tile = tile_all; }
    else if (tile_all < set.end1) { t.W = set.W1; t.Y = set.Y1; t.n_rows = set.n_rows1; t.ldy = set.ldy1; t.tile = tile_all - set.end0; }
    else { t.W = set.W2; t.Y = set.Y2; t.n_rows = set.n_rows2; t.ldy = set.ldy2; t.tile = tile_all - set.end1; }
    return t;
}

/* one load-to-LDS request: lane l's 16 bytes from voff + soff of the buffer land at lds + 16 l */
QLIN_INL void dma16(__amdgpu_buffer_rsrc_t rsrc, uint8_t *lds, uint32_t voff, uint32_t soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void *)lds, 16, voff, soff, 0, 0);
}

}  // namespace kq
}  // namespace qlin
#endif
