/*
 * gemm_kq_wave4.hip - Q4_K, Q5_K, Q6_K and Q8_0 x bf16 prefill GEMM for more than 128 tokens: four waves per workgroup,
 * one per SIMD.
 *
 *   Y[t*ldy + r] = sum_k X[t*ldx + k] * decode(W)[r][k]      X bf16, Y fp32, fp32 accumulate
 *
 * The contraction of tf_gemm_f16_mt_tokenmajor (common/transformer.h:4487, generic branch :4535-4572) with the
 * weights decoded as dequantize_row_q4_K / _q5_K / _q6_K / _q8_0 do (common/ggml_dequant.h:1592-1618, :1620-1660,
 * :1662-1700, :1479-1489; y = (d*sc)*q - dmin*m, resp. d*sc*(q - 32), resp. d*q, in fp32) and rounded once to bf16,
 * nearest even. What the reference's
 * fused kernel does per tile for every type (rdna4/dequant/bench_dequant.c:359-459), on this part's terms.
 *
 * What the shape follows from, measured on MI355X with one wave per SIMD (cycles that the matrix pipe waits for
 * an instruction issued between two v_mfma_f32_32x32x16_bf16 of 32 cycles each):
 *     up to 4 vector-ALU instructions      ~0      (v_cvt_pk_f32_fp8 counts as two)
 *     ds_read_b128                         ~7      (16 alone: 1 KB at 64 B per clock and SIMD)
 *     ds_write_b128                        ~46     (1 KB at about 20 B per clock and SIMD; not hidden by anything)
 *     buffer_load_dwordx4 to registers     64 per KB and SIMD once the compute unit's 64 B per clock are in use, and
 *                                          four times that when every lane reads its own row (as an operand layout
 *                                          would need)
 *     buffer_load_dwordx4 ... lds          the same 64 B per clock, no register or LDS-store cost
 * So nothing is stored to LDS by a wave:
 *   - activations go from global memory to LDS by the load-to-LDS path, 256 tokens x 64 k per tile, whole 128-byte
 *     row segments per 8 lanes, four stages deep;
 *   - decoded weights never touch LDS: wave w owns rows 32 w .. 32 w + 31 of the workgroup's 128 and all 256 tokens,
 *     its lane (row i, half kg) takes 16 of the 32 code bytes of a quarter super-block of its row and decodes them
 *     straight into the matrix instruction's first-operand layout (8 consecutive k of one row per lane): no decode
 *     is done twice in the workgroup, and there is nothing to exchange. The raw blocks of a wave's rows come the same
 *     way as the activations (whole 144-byte blocks, consecutive lanes consecutive bytes; a lane reading its own
 *     row from global memory costs the memory pipe four times as much) and are read back by the wave itself;
 *   - per matrix instruction one ds_read_b128 (a 32-token x 16-k activation fragment) and about three vector
 *     instructions of decode.
 *
 * The formats differ in what a lane takes from its row's block (Q4_K: 16 code bytes per quarter; Q5_K: those
 * and 16 bytes of fifth bits per super-block; Q6_K: two runs of 16 nibble bytes and 16 bytes of bit pairs per half
 * super-block; Q8_0: the 32 codes of one block per tile, scales straight from memory) and in the arithmetic of a
 * piece; the tile loop is one template over a format description.
 *
 * k inside a tile is permuted so that a lane's 16 code bytes serve its four k-steps (Q4_K; the others alike): k-step s of lane half kg covers
 * the low (s < 2) or high nibbles of code bytes 16 kg + 8 (s & 1) .. + 7, i.e. tile k 32 (s >> 1) + 16 kg + 8 (s & 1) ..;
 * the activation fragment of that lane half is chunk 4 (s >> 1) + 2 kg + (s & 1) of the token's 128-byte row segment.
 *
 * LDS: four stages of [256 tokens][64 k] bf16 = 32 KB; 16-byte chunk c of token row r sits at chunk position
 * c ^ f(r), f = bits 1 and 2 of (r >> 1) & 7 swapped, so that the 16 rows of a fragment fetch hit 16 different
 * 16-byte bank groups. One tile = 32 slots of [matrix instruction, fragment fetch for the next k-step, side work],
 * nothing moves between slots; side work = the load-to-LDS requests of the tile three ahead and of the raw blocks
 * two super-blocks ahead, and the decode of the next tile in 44 pieces of at most two vector instructions. Before the last
 * k-step: wait for this wave's requests of the next tile, barrier (the next tile is complete; nobody reads the
 * stage that is requested next, its last fragments were fetched a k-step earlier).
 */
#include <climits>
#include <utility>

#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef float float2v __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void;

constexpr int kBM = 256, kBN = 128;
constexpr int kXStage = kBM * 128; /* bytes of one stage */

/* the four stages are separate objects: a fetch from one stage then never has to wait for a request into another */
__shared__ __attribute__((aligned(1024))) uint8_t w4_stage0[kXStage];
__shared__ __attribute__((aligned(1024))) uint8_t w4_stage1[kXStage];
__shared__ __attribute__((aligned(1024))) uint8_t w4_stage2[kXStage];
__shared__ __attribute__((aligned(1024))) uint8_t w4_stage3[kXStage];

#define QLIN_INL __device__ __forceinline__ __attribute__((always_inline))

template <int ST> QLIN_INL uint8_t *stage_ptr() {
    if constexpr (ST == 0) return w4_stage0;
    else if constexpr (ST == 1) return w4_stage1;
    else if constexpr (ST == 2) return w4_stage2;
    else return w4_stage3;
}

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
    uint32_t cm, hb;
    float2v cp0, cp1;
    float f0, f1, f2, f3, w0, w1, w2, w3;
    float s_a, s_b, m_a, m_b, dl_a, dl_b, nml_a, nml_b; /* of the two sub-blocks (scale groups) of the tile in work */
};

/* everything a slot touches; every member ends up in registers (all indices are constants after inlining) */
template <class F> struct Ctx {
    floatx16 acc[8];         /* [token block]: 32 rows x 32 tokens each */
    bf16x8 xf[2][8];         /* activation fragments of the k-step in use and of the next: [k-step & 1][token block] */
    u32x4 wa[2][4];          /* decoded weights of the tile in use and of the next: [tile & 1][k-step] */
    u32x4 cur[F::kLaneVec + F::kExtraVec], nxt[F::kLaneVec + F::kExtraVec]; /* raw data of the super-block of the tile being
                                decoded, and of the next: kLaneVec vectors out of the LDS image, kExtraVec straight from memory */
    typename F::Scales sc;   /* of the super-block being decoded */
    Temps t;
    uint32_t xrd;            /* byte offset of this lane's fragment fetches in a stage: k-step 0, token block 0 */
    __amdgpu_buffer_rsrc_t w_rsrc, x_rsrc;
    uint32_t w_off[F::kReq], w_rd, w_swz, w_own, x_off[8]; /* w_swz: see kSwizzle; w_own: byte offset of the lane's own
                                                               row in the weight tile */
    uint8_t *raw;            /* the workgroup's raw-block area in LDS */
    int wv, kg;              /* wave of the workgroup; lane half */
    int sb, n_sb;            /* super-block of the tile in use */
    float unit;
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

/* one load-to-LDS request: lane l's 16 bytes from voff + soff of the buffer land at lds + 16 l */
QLIN_INL void dma16(__amdgpu_buffer_rsrc_t rsrc, uint8_t *lds, uint32_t voff, uint32_t soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void *)lds, 16, voff, soff, 0, 0);
}

/* request Q (0 .. kReq - 1) of this wave for the raw blocks of super-block `sb` of its 32 rows (past the end of K: a
 * harmless re-read) */
template <class F, int Q> QLIN_INL void request_w(Ctx<F> &c, int sb) {
    dma16(c.w_rsrc, c.raw + (c.wv * F::kReq + Q) * 1024, c.w_off[Q], min(sb, c.n_sb - 1) * F::kBlockBytes);
}
/* vector J of this lane's raw data out of its row's image */
template <class F, int J> QLIN_INL u32x4 load_raw(Ctx<F> &c) {
    constexpr VecAt at = F::vec_at(J);
    return *reinterpret_cast<const u32x4 *>(c.raw + c.w_rd + ((uint32_t)(at.off + at.by_half * c.kg) ^ c.w_swz));
}

/* request I (0..7) of this wave for 64-k tile `tile` into stage ST: token rows 64 wv + 8 I .. + 7, 128 bytes each */
template <class F, int ST, int I> QLIN_INL void request_x(Ctx<F> &c, int tile) {
    dma16(c.x_rsrc, stage_ptr<ST>() + (8 * c.wv + I) * 1024, c.x_off[I], min(tile, 4 * c.n_sb - 1) * 128);
}

/* activation fragment of token block BJ, k-step S of stage ST */
template <class F, int ST, int S, int BJ> QLIN_INL bf16x8 load_frag(Ctx<F> &c) {
    return *reinterpret_cast<const bf16x8 *>(stage_ptr<ST>() + (c.xrd ^ (uint32_t)F::frag_xor(S)) + BJ * 4096);
}

/* slot T (0..31) of tile 4 sb + U */
template <class F, int U, int T> QLIN_INL void slot(Ctx<F> &c) {
    constexpr int s = T / 8, bj = T % 8;
    if constexpr (T == 24) {
        /* this wave's requests of the next tile have landed: younger are the 8 of the tile after it, 6 of the one
         * after that, the weight requests of a tile with U = 1 and the scale loads of one with U = 0 (all of them if
         * that was the tile before, those of its first 24 slots if it is this one) */
        constexpr int w_now = F::kReq < 6 ? F::kReq : 6, x_now = F::kExtraLoads < 6 ? F::kExtraLoads : 6;
        wait_vmcnt<14 + (U == 0 ? x_now : 0) + (U == 1 ? w_now + F::kExtraLoads : 0) + (U == 2 ? F::kReq : 0)>();
        __builtin_amdgcn_s_barrier();
    }
    c.acc[bj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, c.wa[U & 1][s]), c.xf[s & 1][bj], c.acc[bj], 0, 0, 0);
    c.xf[(s + 1) & 1][bj] = load_frag<F, (s == 3 ? (U + 1) & 3 : U), (s + 1) & 3, bj>(c);
    if constexpr (T % 4 == 2) request_x<F, (U + 3) & 3, T / 4>(c, 4 * c.sb + U + 3);
    /* U = 0: the raw data of the next super-block (requested three tiles ago) into registers; U = 1: request the
     * one after it into the same place; U = 3: the tile being decoded is the first of the next super-block, which
     * then becomes the one in work */
    if constexpr (U == 0 && T % 4 == 1 && T / 4 < F::kLaneVec) c.nxt[T / 4] = load_raw<F, T / 4>(c);
    if constexpr (U == 0 && T % 4 == 1 && T / 4 < F::kExtraLoads) F::template extra_load<T / 4>(c, c.nxt, min(c.sb + 1, c.n_sb - 1));
    if constexpr (U == 1 && T % 4 == 1 && T / 4 < F::kReq) request_w<F, T / 4>(c, c.sb + 2);
    if constexpr (U == 3 && T % 3 == 2 && T / 3 < F::kLaneVec + F::kExtraVec) c.cur[T / 3] = c.nxt[T / 3];
    constexpr int n_pieces = F::kTilePieces + (U == 3 ? F::kPrepPieces : 0);
    constexpr int p0 = (T * n_pieces + 31) / 32, p1 = ((T + 1) * n_pieces + 31) / 32; /* pieces p with p * 32 / n_pieces == T */
    auto piece = [&](auto pc) {
        constexpr int p = decltype(pc)::value;
        if constexpr (p < p1) {
            if constexpr (U == 3) {
                if constexpr (p < F::kPrepPieces) F::template prep<p>(c, c.nxt);
                else F::template tile_piece<0, 0, p - F::kPrepPieces>(c, c.nxt);
            } else {
                F::template tile_piece<U + 1, (U + 1) & 1, p>(c, c.cur);
            }
        }
    };
    piece(std::integral_constant<int, p0>{});
    piece(std::integral_constant<int, p0 + 1>{});
    static_assert(p1 - p0 <= 2, "at most two pieces per slot");
    __builtin_amdgcn_sched_barrier(0);
}

template <class F, int U, int... T> QLIN_INL void run_tile(Ctx<F> &c, std::integer_sequence<int, T...>) { (slot<F, U, T>(c), ...); }
template <class F, int... P> QLIN_INL void prep_first(Ctx<F> &c, std::integer_sequence<int, P...>) { (F::template prep<P>(c, c.cur), ...); }
template <class F, int... P> QLIN_INL void decode_first(Ctx<F> &c, std::integer_sequence<int, P...>) { (F::template tile_piece<0, 0, P>(c, c.cur), ...); }
template <class F, int ST, int... I> QLIN_INL void request_tile(Ctx<F> &c, int tile, std::integer_sequence<int, I...>) { (request_x<F, ST, I>(c, tile), ...); }
template <class F, int... Q> QLIN_INL void request_raw(Ctx<F> &c, int sb, std::integer_sequence<int, Q...>) { (request_w<F, Q>(c, sb), ...); }
template <class F, int... J> QLIN_INL void load_cur(Ctx<F> &c, std::integer_sequence<int, J...>) { ((c.cur[J] = load_raw<F, J>(c)), ...); }
template <class F, int... J> QLIN_INL void load_cur_extra(Ctx<F> &c, std::integer_sequence<int, J...>) { (F::template extra_load<J>(c, c.cur, 0), ...); }

}  // namespace

template <class F>
__global__ void __launch_bounds__(256)
gemm_kq_bf16_wave4_kernel(const uint8_t *__restrict__ W, const uint16_t *__restrict__ X, float *__restrict__ Y,
                          int n_rows, int n_sb, int n_tok, int ldx, int ldy, int m_tiles) {
    /* raw blocks of one super-block of each wave's 32 weight rows (32 x kPieces pieces, rounded up to whole requests) */
    __shared__ __attribute__((aligned(1024))) uint8_t w4_raw[4 * F::kReq * 1024];
    const int tid = threadIdx.x, lane = tid & 63;

    /* consecutive workgroup ids land on different XCDs (id % 8), each with its own L2; the token tiles
     * that share one weight tile get ids 8 apart and meet in the same L2 */
    const int xcd = blockIdx.x & 7, slot_id = blockIdx.x >> 3;
    const int tile_m = slot_id % m_tiles;
    const int tile_n = (slot_id / m_tiles) * 8 + xcd;
    if (tile_n * kBN >= n_rows) return;

    Ctx<F> c;
    c.raw = w4_raw;
    c.wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    c.n_sb = n_sb;
    c.unit = 1.0f / fp8_pair_lo(1u).x;
    const uint32_t row_bytes = (uint32_t)n_sb * F::kBlockBytes;
    /* Global loads are buffer loads: a descriptor of this workgroup's weight rows / token rows in scalar
     * registers, a 32-bit offset per lane that never changes, and a scalar offset that moves along K.
     * Weight role: lane (i = lane % 32, kg = lane / 32) owns row 32 wv + i; rows past the end re-read the last one
     * (decoded, never stored). Request q of a wave fills pieces 64 q .. 64 q + 63 of its 32 x kPieces. */
    const int li = lane & 31, kg = lane >> 5;
    const int w_rows = min(kBN, n_rows - tile_n * kBN);
    c.w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(W) + (size_t)tile_n * kBN * row_bytes, 0,
                                                 w_rows * row_bytes, 0x00020000);
    c.kg = kg;
#pragma unroll
    for (int q = 0; q < F::kReq; q++) {
        const int id = min(64 * q + lane, 32 * F::kPieces - 1); /* past the last piece: padding */
        const int part = F::kSwizzle ? (id % F::kPieces) ^ ((id / F::kPieces) & 15) : id % F::kPieces;
        c.w_off[q] = (uint32_t)min(32 * c.wv + id / F::kPieces, w_rows - 1) * row_bytes + F::piece_src(part);
    }
    c.w_rd = (uint32_t)(c.wv * F::kReq * 1024 + li * F::kPieces * 16);
    c.w_swz = F::kSwizzle ? (uint32_t)(li & 15) << 4 : 0u;
    c.w_own = (uint32_t)min(32 * c.wv + li, w_rows - 1) * row_bytes;
    /* Activation requests: request I of this wave fills 1 KB of a stage, lane l the 16 bytes at chunk position l % 8 of
     * token row 64 wv + 8 I + l / 8, i.e. chunk (l % 8) ^ f(row) of that token's 128 bytes; tokens past the end
     * re-read the last one (never stored) */
    const int x_rows = min(kBM, n_tok - tile_m * kBM);
    c.x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(X) + (size_t)tile_m * kBM * ldx, 0,
                                                 ((x_rows - 1) * ldx + n_sb * 256) * 2, 0x00020000);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int row = 64 * c.wv + 8 * i + (lane >> 3);
        c.x_off[i] = (uint32_t)min(row, x_rows - 1) * (uint32_t)(2 * ldx) + (uint32_t)((((lane & 7) ^ fsw(row))) << 4);
    }
    /* fragment fetches: token li of each block of 32; chunk 4 (s >> 1) + 2 kg + (s & 1) for the K-quants */
    c.xrd = (uint32_t)(li * 128 + (((F::kKgChunk * kg) ^ fsw(li)) << 4));

#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) c.acc[i][v] = 0.0f;

    /* ---- prologue: raw blocks of super-block 0 fetched and read back, those of super-block 1 and tiles 0..2
     * requested; tile 0 decoded; fragments of its k-step 0 fetched */
    c.sb = 0;
    load_cur_extra<F>(c, std::make_integer_sequence<int, F::kExtraLoads>{});
    request_raw<F>(c, 0, std::make_integer_sequence<int, F::kReq>{});
    request_tile<F, 0>(c, 0, std::make_integer_sequence<int, 8>{});
    wait_vmcnt<8>();
    load_cur<F>(c, std::make_integer_sequence<int, F::kLaneVec>{});
    __builtin_amdgcn_s_waitcnt(0xC07F); /* lgkmcnt(0): the registers hold super-block 0 before its place is requested again */
    request_raw<F>(c, 1, std::make_integer_sequence<int, F::kReq>{});
    request_tile<F, 1>(c, 1, std::make_integer_sequence<int, 8>{});
    request_tile<F, 2>(c, 2, std::make_integer_sequence<int, 8>{});
    prep_first<F>(c, std::make_integer_sequence<int, F::kPrepPieces>{});
    decode_first<F>(c, std::make_integer_sequence<int, F::kTilePieces>{});
    wait_vmcnt<16>(); /* tile 0 and the raw blocks of super-block 1 are in LDS as far as this wave's requests go */
    __builtin_amdgcn_s_barrier();
    c.xf[0][0] = load_frag<F, 0, 0, 0>(c); c.xf[0][1] = load_frag<F, 0, 0, 1>(c); c.xf[0][2] = load_frag<F, 0, 0, 2>(c);
    c.xf[0][3] = load_frag<F, 0, 0, 3>(c); c.xf[0][4] = load_frag<F, 0, 0, 4>(c); c.xf[0][5] = load_frag<F, 0, 0, 5>(c);
    c.xf[0][6] = load_frag<F, 0, 0, 6>(c); c.xf[0][7] = load_frag<F, 0, 0, 7>(c);

#pragma unroll 1
    for (int sb = 0; sb < n_sb; sb++) { /* one super-block of K = four tiles per pass */
        c.sb = sb;
        run_tile<F, 0>(c, std::make_integer_sequence<int, 32>{});
        run_tile<F, 1>(c, std::make_integer_sequence<int, 32>{});
        run_tile<F, 2>(c, std::make_integer_sequence<int, 32>{});
        run_tile<F, 3>(c, std::make_integer_sequence<int, 32>{});
    }
    wait_vmcnt<0>(); /* requests past the end of K are still on their way into LDS */

    /* C layout of the 32x32 MFMA: register v of lane l holds row 8 (v / 4) + 4 (l / 32) + v % 4 (a weight row), column
     * l % 32 (a token): four runs of four consecutive floats of one token's output row per lane */
    const bool vec_ok = (ldy & 3) == 0 && (reinterpret_cast<uintptr_t>(Y) & 15) == 0;
#pragma unroll
    for (int bj = 0; bj < 8; bj++) {
        const int m = tile_m * kBM + 32 * bj + li;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int n = tile_n * kBN + 32 * c.wv + 8 * g + 4 * kg;
            if (m >= n_tok) continue;
            float *y = Y + (size_t)m * ldy + n;
            const floatx4 a = {c.acc[bj][4 * g], c.acc[bj][4 * g + 1], c.acc[bj][4 * g + 2], c.acc[bj][4 * g + 3]};
            if (vec_ok && n + 3 < n_rows) {
                *reinterpret_cast<floatx4 *>(y) = a;
            } else {
#pragma unroll
                for (int v = 0; v < 4; v++)
                    if (n + v < n_rows) y[v] = a[v];
            }
        }
    }
}

namespace {
template <class F>
hipError_t launch_wave4(const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok, int ldx, int ldy,
                        hipStream_t stream) {
    const int n_sb = n_cols / 256;
    const int m_tiles = (n_tok + kBM - 1) / kBM;
    const int n_tiles = (n_rows + kBN - 1) / kBN;
    /* ids are dealt to 8 XCDs; pad the n-tile count to a multiple of 8 (surplus groups exit) */
    const int n_tiles_pad = (n_tiles + 7) / 8 * 8;
    hipLaunchKernelGGL(gemm_kq_bf16_wave4_kernel<F>, dim3(n_tiles_pad * m_tiles), dim3(256), 0, stream,
                       (const uint8_t *)W, X, Y, n_rows, n_sb, n_tok, ldx, ldy, m_tiles);
    return hipGetLastError();
}
}  // namespace

bool gemm_kq_wave4_covers(uint32_t type) { return type == T_Q4_K || type == T_Q5_K || type == T_Q6_K || type == T_Q8_0; }

/* Every 256 tokens decode the weights again, which costs more the more there is to decode, while decoding once into
 * a workspace costs 27 - 38 us whatever the token count. 14336 x 4096, this kernel against decode + the vendor library's
 * product, us: at 512 tokens Q4_K 61 / 86, Q5_K 62 / 92, Q6_K 66 / 84, Q8_0 71 / 83; at 1024 118 / 125, 121 / 135,
 * 131 / 126, 139 / 121; at 1536 181 / 190, 185 / 195, 206 / 184, 216 / 177; at 2048 267 / 244, 262 / 260, 273 / 240,
 * 311 / 224 (Q8_0's extra is mostly its scale loads). Above these token counts the decode + dense route is taken
 * where a workspace is at hand. */
int gemm_kq_wave4_max_tokens(uint32_t type) {
    switch (type) {
    case T_Q4_K: case T_Q5_K: return 1536;
    case T_Q6_K: case T_Q8_0: return 512;
    default: return INT_MAX;
    }
}

hipError_t launch_gemm_kq_bf16_wave4(uint32_t type, const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols,
                                     int n_tok, int ldx, int ldy, hipStream_t stream) {
    switch (type) {
    case T_Q4_K: return launch_wave4<FQ4K>(W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q5_K: return launch_wave4<FQ5K>(W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q6_K: return launch_wave4<FQ6K>(W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q8_0: return launch_wave4<FQ8_0>(W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_gemm_q4k_bf16_wave4(const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok,
                                      int ldx, int ldy, hipStream_t stream) {
    return launch_wave4<FQ4K>(W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
}

}  // namespace qlin
