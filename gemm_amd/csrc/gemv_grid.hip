/*
 * gemv_grid.hip - batch-1 matvec for rows of more than 4096 elements (and, where it measured faster, of 2048 to
 * 4096) on gfx950, for the codebook ("grid") formats
 * IQ1_S, IQ1_M, IQ2_XXS, IQ2_XS, IQ2_S, IQ3_XXS and IQ3_S and for Q6_K, Q5_K, Q8_0, Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, IQ4_XS, MXFP4, NVFP4, TQ1_0, TQ2_0, Q1_0, Q2_K and Q3_K: the inner products run on the 8-bit
 * integer matrix instruction; the grid formats look their codebook and sign masks up in LDS, the others build their
 * codes in registers and read the x operand from LDS for every item.
 *
 * y[r] = sum over 16- or 32-element groups of scale(r, group) * (codes . x_group) (- offset * sum of x_group), with
 * the codes of common/ggml_dequant.h:2793-2816, :2916-2940, :3022-3058 (grid formats), :1653-1687 (Q6_K),
 * :1620-1651 (Q5_K), :1479-1489 (Q8_0), :2850-2862 (Q4_0), :2942-2954 (IQ4_NL), :2956-2973 (IQ4_XS),
 * :1505-1534 (Q2_K), :1536-1580 (Q3_K), :2864-2915 (Q4_1, Q5_0, Q5_1), :2818-2830 (MXFP4) and
 * :2832-2848 (NVFP4), :3161-3176 (TQ2_0), :2975-3020 (IQ2_XS, IQ2_S), :1491-1503 (Q1_0),
 * :3062-3126 (IQ1_S, IQ1_M), :3127-3160 (TQ1_0).
 *
 *  1. x -> fixed point per 32-element group, three signed base-256 digits (the Q4_K matvec, gemv_q4k.hip,
 *     keeps four): X = rint(x * 2^(22-e)), e the exponent of the group's largest |x|; the error is at most
 *     2^-23 of that largest |x| per element.
 *  2. v_mfma_i32_16x16x64_i8: 16 weight rows (B operand: one code byte per element) against 16 "x rows"
 *     (A operand). Lane group g = lane/16 of a wave owns 64 elements of the wave's super-block, 16 per
 *     instruction s = 0..3 (F::elem0(g, s): elements [64 g + 16 s, +16) for most formats; Q6_K takes the 16
 *     elements of one scale). The A operand is block-diagonal to match: x row 4g + digit (digit 0..2; row 4g+3
 *     stays zero) holds that digit plane of lane group g's 16 elements at lane group g's k positions and zeros
 *     elsewhere, so result register v of lane (n, g) is digit plane v of lane group g's elements for weight
 *     row n. Which k position carries which element is free as long as both operands agree.
 *  3. Wave w of the 16-wave workgroup owns super-block w (w+16, ...) of every row of the workgroup, prepares
 *     only its own 256 elements of x, and reads its bytes of a block straight from HBM: lane (n, g) takes
 *     the bytes of its 64 elements of row n (blocks of the grid formats and Q6_K are 2-byte aligned:
 *     dword-aligned loads, a 16-bit tail and a funnel shift). The waves' shares of a row meet in LDS at the end.
 *
 * What a lane of a grid format spends per element is one table lookup per 4-8 elements for the grid, one per 8
 * for the sign mask, two vector instructions per 4 elements to apply the signs and a sixteenth of a matrix
 * instruction; the v_dot4 formulation (gemv_int.hip) spends an instruction per element on the products alone.
 *
 * A non-finite x makes every output NaN (the fixed-point form cannot carry Inf).
 */
#include "qlin_codebooks.h"
#include "qlin_codebooks_ext.h"
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));

constexpr int kWaves = 16;        /* wavefronts per workgroup */
constexpr int kMaxKc = 4;         /* super-blocks per wave: K <= 16384 */
constexpr int kMaxRowsPerWg = 640; /* local rows (both matrices of a gate+up pair): 40 KB of partial sums, 63 KB in all */
constexpr int kXScratch = 1152;   /* per wave: 3 digit planes x 256 B, 128 zero bytes, (at 1024) 8 x 2^(e-22), (at 1056) 16 sums of 16 x */

/* x operand of one super-block: A[s] for instruction s. The other two things an item needs stay in the wave's
 * scratch until the next super-block is prepared: meta[G] = 2^(e-22) of 32-element group G, meta[8 + S] = the sum
 * of x over 16-element group S (formats with a constant offset per code). */
struct XOperand {
    v4i A[4];             /* formats whose items keep LDS busy with table lookups hold the operand in registers */
    const uint8_t *arows; /* the others read it per item: instruction s at arows + F::kStep * s (zeros for a dead lane) */
    const float *meta;
};

template <int CTRL> __device__ __forceinline__ uint32_t dpp_movu(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, false);
}

/* sixteen bytes at p (2-byte aligned, inside a block that starts at least two bytes before p): the aligned
 * dwords around them and, where p sits in the middle of a dword, the two bytes behind the last full one */
struct Raw16 {
    u32x4_a4 q;
    uint32_t tail;
};
__device__ __forceinline__ Raw16 load16(const uint8_t *p) {
    Raw16 r;
    const uint32_t odd = (uint32_t)(uintptr_t)p & 2u;
    r.q = *reinterpret_cast<const u32x4_a4 *>(p - odd);
    r.tail = 0;
    if (odd) r.tail = *reinterpret_cast<const uint16_t *>(p + 14);
    return r;
}
__device__ __forceinline__ void bytes16(const Raw16 &r, uint32_t sh, uint32_t (&w)[4]) { /* sh = 0 or 16 */
    w[0] = __builtin_amdgcn_alignbit(r.q.y, r.q.x, sh);
    w[1] = __builtin_amdgcn_alignbit(r.q.z, r.q.y, sh);
    w[2] = __builtin_amdgcn_alignbit(r.q.w, r.q.z, sh);
    w[3] = __builtin_amdgcn_alignbit(r.tail, r.q.w, sh);
}
struct Raw8 {
    u32x2_a4 q;
    uint32_t tail;
};
__device__ __forceinline__ Raw8 load8(const uint8_t *p) {
    Raw8 r;
    const uint32_t odd = (uint32_t)(uintptr_t)p & 2u;
    r.q = *reinterpret_cast<const u32x2_a4 *>(p - odd);
    r.tail = 0;
    if (odd) r.tail = *reinterpret_cast<const uint16_t *>(p + 6);
    return r;
}
__device__ __forceinline__ void bytes8(const Raw8 &r, uint32_t sh, uint32_t (&w)[2]) {
    w[0] = __builtin_amdgcn_alignbit(r.q.y, r.q.x, sh);
    w[1] = __builtin_amdgcn_alignbit(r.tail, r.q.y, sh);
}

/* the tables in LDS: the format's grid, and the sign masks (0xFF per negative element, two dwords per sign
 * byte): 256 entries by sign byte, then 128 by the seven stored bits of the formats that keep a parity bit */
struct Tables {
    const uint32_t *grid;
    const uint2 *sign256, *sign128;
};

/* magnitudes m (four bytes, each 1..127: no grid of these formats holds a zero) with the signs of mask s
 * (0xFF = negative) -> signed bytes: (m ^ s) + (s & 1) per byte; a nonzero m keeps the +1 inside its byte */
__device__ __forceinline__ int apply_signs(uint32_t m, uint32_t s) { return (int)((m ^ s) + (s & 0x01010101u)); }
__device__ __forceinline__ uint32_t spread4(uint32_t v) { return ((v & 15u) * 0x00204081u) & 0x01010101u; }

/* digit sums of one group (top, middle, low) -> the group's integer inner product as a float */
__device__ __forceinline__ float join_digits(v4i c) {
    return fmaf((float)c.x, 65536.0f, (float)((c.y << 8) + c.z));
}

template <uint32_t T> struct GridFmt;

/* IQ2_XXS [d][8 x (4 grid indices, 4 x 7 sign bits + 4-bit scale)]: d*(0.5+s)*0.25 * grid byte * sign, an
 * eight-byte grid entry per index (common/ggml_dequant.h:2793-2816); 66-byte blocks */
template <> struct GridFmt<T_IQ2_XXS> {
    static constexpr int kBlock = 66, kGridBytes = 2048;
    static constexpr int kAlign = 2; /* what the loads want of the matrix address and the row pitch */
    static constexpr int kStep = 16; /* bytes between the x rows of consecutive instructions */
    static constexpr bool kAInRegs = true;
    static constexpr int kPiece = 2; /* every piece a lane reads starts 2 (mod 4) bytes into the block */
    static constexpr bool kSums = false;
    /* lane group g takes elements [64 g, 64 g + 64) in order, 16 per instruction */
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    __device__ static const uint32_t *grid_src() { return reinterpret_cast<const uint32_t *>(qlin_iq2xxs_grid); }
    struct Raw {
        Raw16 a; /* groups 2g, 2g+1: [indices, signs + scale] each */
        uint32_t d;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        r.a = load16(blk + 2 + 16 * g);
        r.d = *reinterpret_cast<const uint16_t *>(blk);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t sh, const Tables &t, int g) {
        uint32_t w[4];
        bytes16(r.a, sh, w);
        const uint2 *grid = reinterpret_cast<const uint2 *>(t.grid);
        const float d = half_bits_fast(r.d) * 0.25f;
        float acc = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t a0 = w[2 * h], a1 = w[2 * h + 1];
            v4i c = {0, 0, 0, 0};
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const uint2 m0 = grid[(a0 >> (16 * q)) & 255u], m1 = grid[(a0 >> (16 * q + 8)) & 255u];
                const uint2 s0 = t.sign128[(a1 >> (14 * q)) & 127u], s1 = t.sign128[(a1 >> (14 * q + 7)) & 127u];
                const v4i b = {apply_signs(m0.x, s0.x), apply_signs(m0.y, s0.y), apply_signs(m1.x, s1.x), apply_signs(m1.y, s1.y)};
                c = __builtin_amdgcn_mfma_i32_16x16x64_i8(xo.A[2 * h + q], b, c, 0, 0, 0);
            }
            acc = fmaf(join_digits(c) * xo.meta[2 * g + h], 0.5f + (float)(a1 >> 28), acc);
        }
        return d * acc;
    }
};

/* IQ3_XXS [d][qs 64][8 x (4 x 7 sign bits + 4-bit scale)]: d*(0.5+s)*0.5 * grid byte * sign, a four-byte
 * grid entry per index byte (:2916-2940); 98-byte blocks */
template <> struct GridFmt<T_IQ3_XXS> {
    static constexpr int kBlock = 98, kGridBytes = 1024;
    static constexpr int kAlign = 2; /* what the loads want of the matrix address and the row pitch */
    static constexpr int kStep = 16; /* bytes between the x rows of consecutive instructions */
    static constexpr bool kAInRegs = true;
    static constexpr int kPiece = 2; /* every piece a lane reads starts 2 (mod 4) bytes into the block */
    static constexpr bool kSums = false;
    /* lane group g takes elements [64 g, 64 g + 64) in order, 16 per instruction */
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    __device__ static const uint32_t *grid_src() { return qlin_iq3xxs_grid; }
    struct Raw {
        Raw16 qs; /* index bytes of groups 2g, 2g+1 */
        Raw8 sc;  /* their sign + scale words */
        uint32_t d;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        r.qs = load16(blk + 2 + 16 * g);
        r.sc = load8(blk + 66 + 8 * g);
        r.d = *reinterpret_cast<const uint16_t *>(blk);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t sh, const Tables &t, int g) {
        uint32_t qs[4], sc[2];
        bytes16(r.qs, sh, qs);
        bytes8(r.sc, sh, sc);
        const float d = half_bits_fast(r.d) * 0.5f;
        float acc = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t a1 = sc[h];
            v4i c = {0, 0, 0, 0};
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const uint32_t ix = qs[2 * h + q];
                const uint2 s0 = t.sign128[(a1 >> (14 * q)) & 127u], s1 = t.sign128[(a1 >> (14 * q + 7)) & 127u];
                const v4i b = {apply_signs(t.grid[ix & 255u], s0.x), apply_signs(t.grid[(ix >> 8) & 255u], s0.y),
                               apply_signs(t.grid[(ix >> 16) & 255u], s1.x), apply_signs(t.grid[ix >> 24], s1.y)};
                c = __builtin_amdgcn_mfma_i32_16x16x64_i8(xo.A[2 * h + q], b, c, 0, 0, 0);
            }
            acc = fmaf(join_digits(c) * xo.meta[2 * g + h], 0.5f + (float)(a1 >> 28), acc);
        }
        return d * acc;
    }
};

/* IQ3_S [d][qs 64][qh 8][signs 32][scales 4]: d*(1+2s) * grid byte * sign, 9-bit grid indices (:3022-3058);
 * 110-byte blocks */
template <> struct GridFmt<T_IQ3_S> {
    static constexpr int kBlock = 110, kGridBytes = 2048;
    static constexpr int kAlign = 2; /* what the loads want of the matrix address and the row pitch */
    static constexpr int kStep = 16; /* bytes between the x rows of consecutive instructions */
    static constexpr bool kAInRegs = true;
    static constexpr int kPiece = 2; /* every piece a lane reads starts 2 (mod 4) bytes into the block */
    static constexpr bool kSums = false;
    /* lane group g takes elements [64 g, 64 g + 64) in order, 16 per instruction */
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    __device__ static const uint32_t *grid_src() { return qlin_iq3s_grid; }
    struct Raw {
        Raw16 qs;  /* low index bytes of groups 2g, 2g+1 */
        Raw8 sg;   /* their sign bytes */
        uint32_t qh, scales, d; /* the ninth index bits (a byte per group), the byte with both 4-bit scales */
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        r.qs = load16(blk + 2 + 16 * g);
        r.sg = load8(blk + 74 + 8 * g);
        r.qh = *reinterpret_cast<const uint16_t *>(blk + 66 + 2 * g);
        r.scales = blk[106 + g];
        r.d = *reinterpret_cast<const uint16_t *>(blk);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t sh, const Tables &t, int g) {
        uint32_t qs[4], sg[2];
        bytes16(r.qs, sh, qs);
        bytes8(r.sg, sh, sg);
        const float d = half_bits_fast(r.d);
        float acc = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            v4i c = {0, 0, 0, 0};
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const uint32_t ix = qs[2 * h + q];
                const uint32_t hb = r.qh >> (8 * h + 4 * q); /* bits 0..3: the ninth bits of these four indices */
                const uint2 s0 = t.sign256[(sg[h] >> (16 * q)) & 255u], s1 = t.sign256[(sg[h] >> (16 * q + 8)) & 255u];
                const uint32_t i0 = (ix & 255u) | ((hb & 1u) << 8), i1 = ((ix >> 8) & 255u) | ((hb & 2u) << 7);
                const uint32_t i2 = ((ix >> 16) & 255u) | ((hb & 4u) << 6), i3 = (ix >> 24) | ((hb & 8u) << 5);
                const v4i b = {apply_signs(t.grid[i0], s0.x), apply_signs(t.grid[i1], s0.y),
                               apply_signs(t.grid[i2], s1.x), apply_signs(t.grid[i3], s1.y)};
                c = __builtin_amdgcn_mfma_i32_16x16x64_i8(xo.A[2 * h + q], b, c, 0, 0, 0);
            }
            const uint32_t nib = (r.scales >> (4 * h)) & 15u;
            acc = fmaf(join_digits(c) * xo.meta[2 * g + h], (float)(1u + 2u * nib), acc);
        }
        return d * acc;
    }
};

/* IQ2_XS [d][32 x (9-bit grid index | 7 sign bits << 9)][8 scale bytes] (common/ggml_dequant.h:2975-2994), 74 bytes:
 * d * (0.5 + nibble) * 0.25 * grid byte * sign, an eight-byte grid entry per 16-bit code, one scale nibble per 16
 * elements. Lane group g takes groups 2g, 2g + 1: eight codes; an instruction is the two codes of one nibble. */
template <> struct GridFmt<T_IQ2_XS> {
    static constexpr int kBlock = 74, kGridBytes = 4096;
    static constexpr int kAlign = 2, kPiece = 2;
    static constexpr int kStep = 16;
    static constexpr bool kAInRegs = true, kSums = false;
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    __device__ static const uint32_t *grid_src() { return reinterpret_cast<const uint32_t *>(qlin_iq2xs_grid); }
    struct Raw {
        Raw16 qs;
        uint32_t sc, d;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        r.qs = load16(blk + 2 + 16 * g);
        r.sc = *reinterpret_cast<const uint16_t *>(blk + 66 + 2 * g);
        r.d = *reinterpret_cast<const uint16_t *>(blk);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t sh, const Tables &t, int g) {
        uint32_t w[4];
        bytes16(r.qs, sh, w);
        const uint2 *grid = reinterpret_cast<const uint2 *>(t.grid);
        float acc = 0.0f;
#pragma unroll
        for (int st = 0; st < 4; st++) {
            const uint32_t u0 = w[st] & 0xFFFFu, u1 = w[st] >> 16;
            const uint2 m0 = grid[u0 & 511u], m1 = grid[u1 & 511u];
            const uint2 s0 = t.sign128[u0 >> 9], s1 = t.sign128[u1 >> 9];
            const v4i b = {apply_signs(m0.x, s0.x), apply_signs(m0.y, s0.y), apply_signs(m1.x, s1.x), apply_signs(m1.y, s1.y)};
            const v4i zero = {0, 0, 0, 0};
            const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(xo.A[st], b, zero, 0, 0, 0);
            const uint32_t nib = (r.sc >> (8 * (st >> 1) + 4 * (st & 1))) & 15u;
            acc = fmaf(join_digits(c) * xo.meta[2 * g + (st >> 1)], 0.5f + (float)nib, acc);
        }
        return half_bits_fast(r.d) * 0.25f * acc;
    }
};

/* IQ2_S [d][32 index bytes][32 sign bytes][qh 8][8 scale bytes] (:2996-3020), 82 bytes: as IQ2_XS with a 10-bit
 * index (two high bits per code in qh) into a 1024-entry grid and explicit sign bytes. */
template <> struct GridFmt<T_IQ2_S> {
    static constexpr int kBlock = 82, kGridBytes = 8192;
    static constexpr int kAlign = 2, kPiece = 2;
    static constexpr int kStep = 16;
    static constexpr bool kAInRegs = true, kSums = false;
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    __device__ static const uint32_t *grid_src() { return reinterpret_cast<const uint32_t *>(qlin_iq2s_grid); }
    struct Raw {
        Raw8 qs, sg;
        uint32_t qh, sc, d;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        r.qs = load8(blk + 2 + 8 * g);
        r.sg = load8(blk + 34 + 8 * g);
        r.qh = *reinterpret_cast<const uint16_t *>(blk + 66 + 2 * g);
        r.sc = *reinterpret_cast<const uint16_t *>(blk + 74 + 2 * g);
        r.d = *reinterpret_cast<const uint16_t *>(blk);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t sh, const Tables &t, int g) {
        uint32_t q[2], sg[2];
        bytes8(r.qs, sh, q);
        bytes8(r.sg, sh, sg);
        const uint2 *grid = reinterpret_cast<const uint2 *>(t.grid);
        float acc = 0.0f;
#pragma unroll
        for (int st = 0; st < 4; st++) {
            const int h = st >> 1, l0 = 2 * (st & 1);
            const uint32_t qhb = (r.qh >> (8 * h)) & 0xFFu;
            const uint32_t i0 = ((q[h] >> (8 * l0)) & 0xFFu) | ((qhb << (8 - 2 * l0)) & 0x300u);
            const uint32_t i1 = ((q[h] >> (8 * l0 + 8)) & 0xFFu) | ((qhb << (6 - 2 * l0)) & 0x300u);
            const uint2 m0 = grid[i0], m1 = grid[i1];
            const uint2 s0 = t.sign256[(sg[h] >> (8 * l0)) & 0xFFu], s1 = t.sign256[(sg[h] >> (8 * l0 + 8)) & 0xFFu];
            const v4i b = {apply_signs(m0.x, s0.x), apply_signs(m0.y, s0.y), apply_signs(m1.x, s1.x), apply_signs(m1.y, s1.y)};
            const v4i zero = {0, 0, 0, 0};
            const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(xo.A[st], b, zero, 0, 0, 0);
            const uint32_t nib = (r.sc >> (8 * h + 4 * (st & 1))) & 15u;
            acc = fmaf(join_digits(c) * xo.meta[2 * g + h], 0.5f + (float)nib, acc);
        }
        return half_bits_fast(r.d) * 0.25f * acc;
    }
};

/* IQ1_S [d][32 index bytes][8 x u16: 4 x 3 high index bits, 3-bit scale, shift sign] (common/ggml_dequant.h:3062-3083),
 * 50 bytes: d * (2 s + 1) * (t + delta), t in {-1, 0, 1} from an eight-byte entry of a 2048-entry grid, delta = +-1/8
 * per 32 elements. The grid bytes are the signed codes; delta goes onto the sum of x. */
template <> struct GridFmt<T_IQ1_S> {
    static constexpr int kBlock = 50, kGridBytes = 16384;
    static constexpr int kAlign = 2, kPiece = 2;
    static constexpr int kStep = 16;
    static constexpr bool kAInRegs = true, kSums = true;
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    __device__ static const uint32_t *grid_src() { return reinterpret_cast<const uint32_t *>(qlin_iq1s_grid); }
    struct Raw {
        Raw8 qs;
        uint32_t qh_q, qh_tail, d; /* the two u16 of groups 2g, 2g + 1: aligned dword and, off the grid, the tail */
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        r.qs = load8(blk + 2 + 8 * g);
        const uint8_t *p = blk + 34 + 4 * g;
        const uint32_t odd = (uint32_t)(uintptr_t)p & 2u;
        r.qh_q = *reinterpret_cast<const uint32_t *>(p - odd);
        r.qh_tail = 0;
        if (odd) r.qh_tail = *reinterpret_cast<const uint16_t *>(p + 2);
        r.d = *reinterpret_cast<const uint16_t *>(blk);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t sh, const Tables &t, int g) {
        uint32_t q[2];
        bytes8(r.qs, sh, q);
        const uint32_t qh2 = __builtin_amdgcn_alignbit(r.qh_tail, r.qh_q, sh);
        const uint2 *grid = reinterpret_cast<const uint2 *>(t.grid);
        float acc = 0.0f;
#pragma unroll
        for (int st = 0; st < 4; st++) {
            const int h = st >> 1, l0 = 2 * (st & 1);
            const uint32_t qh = (qh2 >> (16 * h)) & 0xFFFFu;
            const uint32_t i0 = ((q[h] >> (8 * l0)) & 0xFFu) | (((qh >> (3 * l0)) & 7u) << 8);
            const uint32_t i1 = ((q[h] >> (8 * l0 + 8)) & 0xFFu) | (((qh >> (3 * l0 + 3)) & 7u) << 8);
            const uint2 m0 = grid[i0], m1 = grid[i1];
            const v4i b = {(int)m0.x, (int)m0.y, (int)m1.x, (int)m1.y};
            const v4i zero = {0, 0, 0, 0};
            const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(xo.A[st], b, zero, 0, 0, 0);
            const float dl = (float)(2u * ((qh >> 12) & 7u) + 1u);
            const float delta = (qh & 0x8000u) ? -0.125f : 0.125f;
            const int e0 = elem0(g, st);
            acc = fmaf(dl, fmaf(join_digits(c), xo.meta[e0 >> 5], delta * xo.meta[8 + (e0 >> 4)]), acc);
        }
        return half_bits_fast(r.d) * acc;
    }
};

/* IQ1_M [32 index bytes][qh 16][8 scale bytes] (common/ggml_dequant.h:3084-3126), 56 bytes and no d field (its
 * four nibbles sit on top of the four scale words): d * (2 s + 1) * (t + delta) with the IQ1_S grid, a 3-bit scale
 * per 16 elements and delta = +-1/8 per 8. The codes are 8 t + (+-1), signed bytes picked from a four-byte table by
 * the grid byte's two low bits (t = -1, 0, 1 are 0xFF, 0, 1), and the scale carries the 1/8. */
template <> struct GridFmt<T_IQ1_M> {
    static constexpr int kBlock = 56, kGridBytes = 16384;
    static constexpr int kAlign = 4, kPiece = 0;
    static constexpr int kStep = 16;
    static constexpr bool kAInRegs = true, kSums = false;
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    __device__ static const uint32_t *grid_src() { return reinterpret_cast<const uint32_t *>(qlin_iq1s_grid); }
    struct Raw {
        u32x2_a4 qs, sc;
        uint32_t qh;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        r.qs = *reinterpret_cast<const u32x2_a4 *>(blk + 8 * g);
        r.qh = *reinterpret_cast<const uint32_t *>(blk + 32 + 4 * g);
        r.sc = *reinterpret_cast<const u32x2_a4 *>(blk + 48);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t, const Tables &t, int g) {
        const uint32_t q[2] = {r.qs.x, r.qs.y};
        const uint2 *grid = reinterpret_cast<const uint2 *>(t.grid);
        const uint32_t dbits = ((r.sc.x >> 12) & 0x000Fu) | ((r.sc.x >> 24) & 0x00F0u) | ((r.sc.y >> 4) & 0x0F00u) | ((r.sc.y >> 16) & 0xF000u);
        const uint32_t scg = ((g & 2) ? r.sc.y : r.sc.x) >> (16 * (g & 1)); /* scale word g: groups 2g and 2g + 1 */
        /* codes of t = 0, 1, (unused), -1 for delta = +1/8 and -1/8, as 8 t + (+-1) */
        constexpr uint32_t kPlus = 0xF9000901u, kMinus = 0xF70007FFu;
        float acc = 0.0f;
#pragma unroll
        for (int st = 0; st < 4; st++) {
            const int h = st >> 1, l0 = 2 * (st & 1);
            const uint32_t qb = (r.qh >> (8 * (2 * h + (st & 1)))) & 0xFFu;
            const uint32_t i0 = ((q[h] >> (8 * l0)) & 0xFFu) | ((qb << 8) & 0x700u);
            const uint32_t i1 = ((q[h] >> (8 * l0 + 8)) & 0xFFu) | ((qb << 4) & 0x700u);
            const uint2 m0 = grid[i0], m1 = grid[i1];
            const uint32_t t0 = (qb & 0x08u) ? kMinus : kPlus, t1 = (qb & 0x80u) ? kMinus : kPlus;
            const v4i b = {(int)__builtin_amdgcn_perm(0u, t0, m0.x & 0x03030303u), (int)__builtin_amdgcn_perm(0u, t0, m0.y & 0x03030303u),
                           (int)__builtin_amdgcn_perm(0u, t1, m1.x & 0x03030303u), (int)__builtin_amdgcn_perm(0u, t1, m1.y & 0x03030303u)};
            const v4i zero = {0, 0, 0, 0};
            const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(xo.A[st], b, zero, 0, 0, 0);
            const uint32_t s3 = (scg >> (6 * h + 3 * (st & 1))) & 7u;
            acc = fmaf((float)(2u * s3 + 1u), join_digits(c) * xo.meta[2 * g + h], acc);
        }
        return half_bits_fast(dbits) * 0.125f * acc;
    }
};

/* Q6_K [ql 128][qh 64][16 int8 scales][d]: d * sc * (q - 32), q = low nibble | two high bits << 4, one scale per
 * 16 elements (common/ggml_dequant.h:1653-1687); 210-byte blocks. Element 128 h + 32 q + l (h = half, q = 0..3,
 * l < 32) has its nibble in ql[64 h + 32 (q & 1) + l] (the high one for q >= 2) and its high bits in
 * qh[32 h + l] >> 2 q. Lane group g = (h, p) takes l in [16 p, 16 p + 16) of all four q: instruction q, sixteen
 * elements of one scale. The codes stay unsigned (0..63); the -32 goes onto the sum of x. */
template <> struct GridFmt<T_Q6_K> {
    static constexpr int kBlock = 210, kGridBytes = 0;
    static constexpr int kAlign = 2; /* what the loads want of the matrix address and the row pitch */
    static constexpr int kStep = 32;
    static constexpr bool kAInRegs = false; /* no table lookups: LDS has time to deliver the x operand per item */
    static constexpr int kPiece = 0;
    static constexpr bool kSums = true;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 128 * (g >> 1) + 32 * st + 16 * (g & 1); }
    struct Raw {
        Raw16 qa, qb, qh; /* ql[64 h + 16 p ..], ql[64 h + 32 + 16 p ..], qh[32 h + 16 p ..] */
        Raw8 sc;          /* the eight scales of the half */
        uint32_t d;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        const int h = g >> 1, p = g & 1;
        r.qa = load16(blk + 64 * h + 16 * p);
        r.qb = load16(blk + 64 * h + 32 + 16 * p);
        r.qh = load16(blk + 128 + 32 * h + 16 * p);
        r.sc = load8(blk + 192 + 8 * h);
        r.d = *reinterpret_cast<const uint16_t *>(blk + 208);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t sh, const Tables &, int g) {
        uint32_t qa[4], qb[4], qh[4], sc[2];
        bytes16(r.qa, sh, qa);
        bytes16(r.qb, sh, qb);
        bytes16(r.qh, sh, qh);
        bytes8(r.sc, sh, sc);
        const uint32_t scp = (g & 1) ? (sc[0] >> 8) | (sc[1] << 24) : sc[0]; /* byte 2 q (q < 2): scale of (q, p) */
        const uint32_t scq = (g & 1) ? sc[1] >> 8 : sc[1];                  /* byte 2 (q - 2) for q >= 2 */
        float acc = 0.0f;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t(&ql)[4] = (q & 1) ? qb : qa;
            v4i b;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t lo = (ql[i] >> (4 * (q >> 1))) & 0x0F0F0F0Fu;
                const uint32_t hi = ((qh[i] >> (2 * q)) & 0x03030303u) << 4;
                b[i] = (int)(lo | hi);
            }
            const v4i zero = {0, 0, 0, 0};
            const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * q);
            const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
            const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, zero, 0, 0, 0);
            const uint32_t w = q < 2 ? scp >> (16 * q) : scq >> (16 * (q - 2));
            const float scale = (float)(int)(int8_t)(w & 0xFFu);
            const int e0 = elem0(g, q);
            acc = fmaf(scale, fmaf(join_digits(c), xo.meta[e0 >> 5], -32.0f * xo.meta[8 + (e0 >> 4)]), acc);
        }
        return half_bits_fast(r.d) * acc;
    }
};

/* Q8_0 [d][32 x int8] x 8 per 256 elements (common/ggml_dequant.h:1479-1489): 272 bytes, so a row of whole
 * 256-element groups keeps the alignment of the matrix. Lane group g takes blocks 2g, 2g+1: 68 bytes, 17 dwords. */
template <> struct GridFmt<T_Q8_0> {
    static constexpr int kBlock = 272, kGridBytes = 0;
    static constexpr int kPiece = 0, kAlign = 4;
    static constexpr int kStep = 16;
    static constexpr bool kSums = false, kAInRegs = false;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    struct Raw {
        u32x4_a4 a, b, c, d;
        uint32_t e;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        const uint8_t *p = blk + 68 * g;
        r.a = *reinterpret_cast<const u32x4_a4 *>(p);
        r.b = *reinterpret_cast<const u32x4_a4 *>(p + 16);
        r.c = *reinterpret_cast<const u32x4_a4 *>(p + 32);
        r.d = *reinterpret_cast<const u32x4_a4 *>(p + 48);
        r.e = *reinterpret_cast<const uint32_t *>(p + 64);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t, const Tables &, int g) {
        const uint32_t w[17] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w, r.c.x,
                                r.c.y, r.c.z, r.c.w, r.d.x, r.d.y, r.d.z, r.d.w, r.e};
        float acc = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            v4i c = {0, 0, 0, 0};
#pragma unroll
            for (int q = 0; q < 2; q++) {
                v4i b;
#pragma unroll
                for (int i = 0; i < 4; i++) /* block 0: the codes start 2 bytes into dword 0; block 1: at dword 9 */
                    b[i] = h == 0 ? (int)__builtin_amdgcn_alignbit(w[4 * q + i + 1], w[4 * q + i], 16) : (int)w[9 + 4 * q + i];
                const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * (2 * h + q));
                const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
                c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
            }
            const float d = half_bits_fast(h == 0 ? w[0] & 0xFFFFu : w[8] >> 16);
            acc = fmaf(join_digits(c) * xo.meta[2 * g + h], d, acc);
        }
        return acc;
    }
};

/* Q5_K [d][dmin][12 bytes of 6-bit scales and mins][qh 32][qs 128] (:1620-1651), 176 bytes: element 64 j + 32 u + l
 * has its nibble in qs[32 j + l] (the high one for u = 1) and its fifth bit in qh[l] >> (2 j + u); (d sc) q - dmin m
 * with one scale and min per 32 elements. Lane group g takes j = g: low nibbles, then high nibbles. */
template <> struct GridFmt<T_Q5_K> {
    static constexpr int kBlock = 176, kGridBytes = 0;
    static constexpr int kPiece = 0, kAlign = 16;
    static constexpr int kStep = 16;
    static constexpr bool kSums = true, kAInRegs = false;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    struct Raw {
        uint4 hd, qh0, qh1, qs0, qs1;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        r.hd = *reinterpret_cast<const uint4 *>(blk);
        r.qh0 = *reinterpret_cast<const uint4 *>(blk + 16);
        r.qh1 = *reinterpret_cast<const uint4 *>(blk + 32);
        r.qs0 = *reinterpret_cast<const uint4 *>(blk + 48 + 32 * g);
        r.qs1 = *reinterpret_cast<const uint4 *>(blk + 64 + 32 * g);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t, const Tables &, int g) {
        const uint32_t qs[8] = {r.qs0.x, r.qs0.y, r.qs0.z, r.qs0.w, r.qs1.x, r.qs1.y, r.qs1.z, r.qs1.w};
        const uint32_t qh[8] = {r.qh0.x, r.qh0.y, r.qh0.z, r.qh0.w, r.qh1.x, r.qh1.y, r.qh1.z, r.qh1.w};
        float dots = 0.0f, mins = 0.0f;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            v4i c = {0, 0, 0, 0};
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {
                v4i b;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t lo = (qs[4 * hf + i] >> (4 * u)) & 0x0F0F0F0Fu;
                    const uint32_t hi = ((qh[4 * hf + i] >> (2 * g + u)) & 0x01010101u) << 4;
                    b[i] = (int)(lo | hi);
                }
                const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * (2 * u + hf));
                const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
                c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
            }
            /* get_scale_min_k4 (:1582-1590) for sub-block j = 2g + u, from the header's registers */
            const int j = 2 * g + u;
            const uint32_t at = 8u * (uint32_t)(j & 3);
            const uint32_t yb = __builtin_amdgcn_ubfe(r.hd.y, at, 8), zb = __builtin_amdgcn_ubfe(r.hd.z, at, 8);
            const uint32_t wb = __builtin_amdgcn_ubfe(r.hd.w, at, 8);
            const uint32_t sc = j < 4 ? yb & 63u : (wb & 15u) | ((yb >> 6) << 4);
            const uint32_t mn = j < 4 ? zb & 63u : (wb >> 4) | ((zb >> 6) << 4);
            dots = fmaf((float)sc, join_digits(c) * xo.meta[j], dots);
            mins = fmaf((float)mn, xo.meta[8 + 2 * j] + xo.meta[8 + 2 * j + 1], mins);
        }
        return half_bits_fast(r.hd.x & 0xFFFFu) * dots - half_bits_fast(r.hd.x >> 16) * mins;
    }
};

/* Q2_K [16 scale bytes][qs 64][d][dmin] (common/ggml_dequant.h:1505-1534), 84 bytes: element 128 h + 32 j + l
 * (l < 32) is bits 2j, 2j+1 of qs[32 h + l], scaled by d * (low nibble) and offset by -dmin * (high nibble) of
 * scale byte 8 h + 2 j + l / 16. Lane group g = (h, p) takes l in [16 p, 16 p + 16) of all four j, as Q6_K. */
template <> struct GridFmt<T_Q2_K> {
    static constexpr int kBlock = 84, kGridBytes = 0;
    static constexpr int kPiece = 0, kAlign = 4;
    static constexpr int kStep = 32;
    static constexpr bool kSums = true, kAInRegs = false;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 128 * (g >> 1) + 32 * st + 16 * (g & 1); }
    struct Raw {
        u32x4_a4 qs;
        u32x2_a4 sc; /* the eight scale bytes of the half */
        uint32_t dd;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        r.qs = *reinterpret_cast<const u32x4_a4 *>(blk + 16 + 16 * g);
        r.sc = *reinterpret_cast<const u32x2_a4 *>(blk + 8 * (g >> 1));
        r.dd = *reinterpret_cast<const uint32_t *>(blk + 80);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t, const Tables &, int g) {
        const uint32_t qs[4] = {r.qs.x, r.qs.y, r.qs.z, r.qs.w};
        const uint32_t scp = (g & 1) ? (r.sc.x >> 8) | (r.sc.y << 24) : r.sc.x; /* byte 2 j (j < 2): scale of (j, p) */
        const uint32_t scq = (g & 1) ? r.sc.y >> 8 : r.sc.y;                    /* byte 2 (j - 2) for j >= 2 */
        float dots = 0.0f, mins = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v4i b;
#pragma unroll
            for (int i = 0; i < 4; i++) b[i] = (int)((qs[i] >> (2 * j)) & 0x03030303u);
            const v4i zero = {0, 0, 0, 0};
            const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * j);
            const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
            const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, zero, 0, 0, 0);
            const uint32_t w = (j < 2 ? scp >> (16 * j) : scq >> (16 * (j - 2))) & 0xFFu;
            const int e0 = elem0(g, j);
            dots = fmaf((float)(w & 15u), join_digits(c) * xo.meta[e0 >> 5], dots);
            mins = fmaf((float)(w >> 4), xo.meta[8 + (e0 >> 4)], mins);
        }
        return half_bits_fast(r.dd & 0xFFFFu) * dots - half_bits_fast(r.dd >> 16) * mins;
    }
};

/* TQ2_0 [qs 64][d] (common/ggml_dequant.h:3161-3176), 66 bytes: element 128 h + 32 l + m (m < 32) is bits 2l, 2l+1
 * of qs[32 h + m], minus 1, times d. Lane group g = (h, p) takes m in [16 p, 16 p + 16) of all four l, as Q6_K; the
 * codes stay unsigned (0..2) and the -1 goes onto the sum of x. */
template <> struct GridFmt<T_TQ2_0> {
    static constexpr int kBlock = 66, kGridBytes = 0;
    static constexpr int kPiece = 0, kAlign = 2;
    static constexpr int kStep = 32;
    static constexpr bool kSums = true, kAInRegs = false;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 128 * (g >> 1) + 32 * st + 16 * (g & 1); }
    struct Raw {
        Raw16 qs;
        uint32_t d;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        r.qs = load16(blk + 16 * g);
        r.d = *reinterpret_cast<const uint16_t *>(blk + 64);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t sh, const Tables &, int g) {
        uint32_t qs[4];
        bytes16(r.qs, sh, qs);
        float acc = 0.0f;
#pragma unroll
        for (int l = 0; l < 4; l++) {
            v4i b;
#pragma unroll
            for (int i = 0; i < 4; i++) b[i] = (int)((qs[i] >> (2 * l)) & 0x03030303u);
            const v4i zero = {0, 0, 0, 0};
            const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * l);
            const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
            const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, zero, 0, 0, 0);
            const int e0 = elem0(g, l);
            acc += fmaf(join_digits(c), xo.meta[e0 >> 5], -xo.meta[8 + (e0 >> 4)]);
        }
        return half_bits_fast(r.d) * acc;
    }
};

/* Q1_0 [d][128 bits] per 128 elements (common/ggml_dequant.h:1491-1503), 18 bytes: bit set -> +d, clear -> -d; 36
 * bytes per 256 elements. Lane group g takes 64 bits of block g / 2, which start 2 (mod 4) bytes into the 36 for the
 * first block: aligned dwords and a funnel shift there. The codes are the bits; 2 * (bits . x) - sum of x. */
template <> struct GridFmt<T_Q1_0> {
    static constexpr int kBlock = 36, kGridBytes = 0;
    static constexpr int kPiece = 0, kAlign = 4;
    static constexpr int kStep = 16;
    static constexpr bool kSums = true, kAInRegs = false;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    struct Raw {
        u32x2_a4 q;
        uint32_t tail, d;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        const int off = 18 * (g >> 1) + 2 + 8 * (g & 1); /* 2, 10, 20, 28 */
        const uint8_t *p = blk + (off & ~3);
        r.q = *reinterpret_cast<const u32x2_a4 *>(p);
        r.tail = 0;
        if (g < 2) r.tail = *reinterpret_cast<const uint32_t *>(p + 8); /* the second block's bits start on a dword */
        r.d = *reinterpret_cast<const uint16_t *>(blk + 18 * (g >> 1));
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t, const Tables &, int g) {
        const uint32_t sh = g < 2 ? 16u : 0u;
        const uint32_t bits[2] = {__builtin_amdgcn_alignbit(r.q.y, r.q.x, sh), __builtin_amdgcn_alignbit(r.tail, r.q.y, sh)};
        float acc = 0.0f;
#pragma unroll
        for (int st = 0; st < 4; st++) {
            const uint32_t b16 = bits[st >> 1] >> (16 * (st & 1));
            const v4i b = {(int)spread4(b16), (int)spread4(b16 >> 4), (int)spread4(b16 >> 8), (int)spread4(b16 >> 12)};
            const v4i zero = {0, 0, 0, 0};
            const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * st);
            const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
            const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, zero, 0, 0, 0);
            const int e0 = elem0(g, st);
            acc += fmaf(2.0f * join_digits(c), xo.meta[e0 >> 5], -xo.meta[8 + (e0 >> 4)]);
        }
        return half_bits_fast(r.d) * acc;
    }
};

/* four bytes at p (2-byte aligned, at least two bytes into a block) */
struct Raw4 {
    uint32_t q, tail;
};
__device__ __forceinline__ Raw4 load4(const uint8_t *p) {
    Raw4 r;
    const uint32_t odd = (uint32_t)(uintptr_t)p & 2u;
    r.q = *reinterpret_cast<const uint32_t *>(p - odd);
    r.tail = 0;
    if (odd) r.tail = *reinterpret_cast<const uint16_t *>(p + 2);
    return r;
}

/* TQ1_0 [qs 48][qh 4][d] (common/ggml_dequant.h:3127-3160), 54 bytes: base-3 digits, five to a byte of qs and four to
 * a byte of qh; digit n of byte b is ((uint8)(b * 3^n) * 3) >> 8, the value (digit - 1) * d. Elements in runs of 16:
 * runs 0..9 are digit n = run / 2 of qs[16 (run % 2) ..], runs 10..14 digit run - 10 of qs[32..48), run 15 the digits
 * 0..3 of qh[0..4) (element 4 n + j = digit n of qh[j]). Lane group g takes runs 4g..4g + 3; every lane reads the
 * three 16-byte pieces of qs and qh and picks. The codes stay unsigned (0..2); the -1 goes onto the sum of x. */
template <> struct GridFmt<T_TQ1_0> {
    static constexpr int kBlock = 54, kGridBytes = 0;
    static constexpr int kPiece = 0, kAlign = 2;
    static constexpr int kStep = 16;
    static constexpr bool kSums = true, kAInRegs = false;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    struct Raw {
        Raw16 a, b, c;
        Raw4 qh;
        uint32_t d;
    };
    __device__ static Raw load(const uint8_t *blk, int) {
        Raw r;
        r.a = load16(blk);
        r.b = load16(blk + 16);
        r.c = load16(blk + 32);
        r.qh = load4(blk + 48);
        r.d = *reinterpret_cast<const uint16_t *>(blk + 52);
        return r;
    }
    /* digit of four bytes: ((b * pw) mod 256) * 3 >> 8, two bytes at a time in the halves of a dword */
    __device__ static uint32_t digits4(uint32_t w, uint32_t pw) {
        const uint32_t lo = (((w & 0x00FF00FFu) * pw) & 0x00FF00FFu) * 3u, hi = ((((w >> 8) & 0x00FF00FFu) * pw) & 0x00FF00FFu) * 3u;
        return ((lo >> 8) & 0x00030003u) | (hi & 0x03000300u);
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t sh, const Tables &, int g) {
        uint32_t a[4], b[4], c[4];
        bytes16(r.a, sh, a);
        bytes16(r.b, sh, b);
        bytes16(r.c, sh, c);
        const uint32_t qh = __builtin_amdgcn_alignbit(r.qh.tail, r.qh.q, sh);
        /* power of 3 of run 4g + st: runs 0..9 -> run / 2, runs 10..14 -> run - 10 */
        float acc = 0.0f;
#pragma unroll
        for (int st = 0; st < 4; st++) {
            const int run = 4 * g + st;
            const bool from_c = run >= 10, special = run == 15;
            const int n = from_c ? run - 10 : run >> 1;
            const uint32_t pw = n == 0 ? 1u : n == 1 ? 3u : n == 2 ? 9u : n == 3 ? 27u : 81u;
            v4i code;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t src = special ? qh : from_c ? c[i] : (run & 1) ? b[i] : a[i];
                const uint32_t p = special ? (i == 0 ? 1u : i == 1 ? 3u : i == 2 ? 9u : 27u) : pw;
                code[i] = (int)digits4(src, p);
            }
            const v4i zero = {0, 0, 0, 0};
            const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * st);
            const v4i av4 = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
            const v4i cc = __builtin_amdgcn_mfma_i32_16x16x64_i8(av4, code, zero, 0, 0, 0);
            const int e0 = elem0(g, st);
            acc += fmaf(join_digits(cc), xo.meta[e0 >> 5], -xo.meta[8 + (e0 >> 4)]);
        }
        return half_bits_fast(r.d) * acc;
    }
};

/* Q3_K [hmask 32][qs 64][12 packed scale bytes][d] (:1536-1580), 110 bytes: element 128 h + 32 j + l (l < 32) is
 * bits 2j, 2j+1 of qs[32 h + l], minus 4 unless bit 4 h + j of hmask[l] is set, times d * (6-bit scale - 32) of
 * index 8 h + 2 j + l / 16: low nibbles in bytes 0..7 (index & 7, the high nibble for indices 8..15), the two high
 * bits of index i in byte 8 + (i & 3) at bit 2 (i >> 2). Lane group g = (h, p) as Q6_K; the codes stay unsigned
 * (0..7) and the -4 goes onto the sum of x. */
template <> struct GridFmt<T_Q3_K> {
    static constexpr int kBlock = 110, kGridBytes = 0;
    static constexpr int kPiece = 0, kAlign = 2;
    static constexpr int kStep = 32;
    static constexpr bool kSums = true, kAInRegs = false;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 128 * (g >> 1) + 32 * st + 16 * (g & 1); }
    struct Raw {
        Raw16 qs, hm;
        Raw8 lo; /* scale bytes 0..7 */
        Raw4 hi; /* scale bytes 8..11 */
        uint32_t d;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        r.qs = load16(blk + 32 + 16 * g);
        r.hm = load16(blk + 16 * (g & 1));
        r.lo = load8(blk + 96);
        r.hi = load4(blk + 104);
        r.d = *reinterpret_cast<const uint16_t *>(blk + 108);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t sh, const Tables &, int g) {
        uint32_t qs[4], hm[4], lo[2];
        bytes16(r.qs, sh, qs);
        bytes16(r.hm, sh, hm);
        bytes8(r.lo, sh, lo);
        const uint32_t hi = __builtin_amdgcn_alignbit(r.hi.tail, r.hi.q, sh);
        const int h = g >> 1, p = g & 1;
        const uint32_t scp = p ? (lo[0] >> 8) | (lo[1] << 24) : lo[0]; /* byte 2 j (j < 2) */
        const uint32_t scq = p ? lo[1] >> 8 : lo[1];                   /* byte 2 (j - 2) for j >= 2 */
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v4i b;
#pragma unroll
            for (int i = 0; i < 4; i++)
                b[i] = (int)(((qs[i] >> (2 * j)) & 0x03030303u) | (((hm[i] >> (4 * h + j)) & 0x01010101u) << 2));
            const v4i zero = {0, 0, 0, 0};
            const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * j);
            const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
            const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, zero, 0, 0, 0);
            const uint32_t w = j < 2 ? scp >> (16 * j) : scq >> (16 * (j - 2));
            const uint32_t low = (w >> (4 * h)) & 15u;
            const uint32_t high = (hi >> (8 * (2 * (j & 1) + p) + 2 * (2 * h + (j >> 1)))) & 3u;
            const float scale = (float)((int)(low | (high << 4)) - 32);
            const int e0 = elem0(g, j);
            acc = fmaf(scale, fmaf(join_digits(c), xo.meta[e0 >> 5], -4.0f * xo.meta[8 + (e0 >> 4)]), acc);
        }
        return half_bits_fast(r.d) * acc;
    }
};

/* the sixteen signed bytes of the IQ4 codebook (common/ggml_dequant.h:2942-2954) in four registers, and its
 * lookup for four nibbles at once: two byte permutes and a select by the nibbles' top bits */
struct Table16 {
    uint32_t t0, t1, t2, t3;
};
__device__ __forceinline__ Table16 table16(const int8_t *values) {
    const uint4 v = *reinterpret_cast<const uint4 *>(values);
    const Table16 t = {v.x, v.y, v.z, v.w};
    return t;
}
__device__ __forceinline__ int look4(uint32_t n, const Table16 &t) {
    const uint32_t sel = n & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(t.t1, t.t0, sel), hi = __builtin_amdgcn_perm(t.t3, t.t2, sel);
    const uint32_t m = ((n >> 3) & 0x01010101u) * 0xFFu;
    return (int)((hi & m) | (lo & ~m));
}

/* IQ4_NL [d][16 bytes of nibbles] x 8 per 256 elements (:2942-2954): d * table[nibble]; element l of a block is the
 * low nibble of byte l, element 16 + l the high one. 144 bytes per 256 elements; lane group g takes blocks 2g, 2g+1:
 * 36 bytes, nine dwords. Q4_0 (:2850-2862) has the same layout with d * (nibble - 8): its codes stay unsigned and
 * the -8 goes onto the sum of x. */
template <uint32_t T> struct Nibble18 {
    static constexpr int kBlock = 144, kGridBytes = 0;
    static constexpr int kPiece = 0, kAlign = 4;
    static constexpr int kStep = 16;
    static constexpr bool kSums = T == T_Q4_0, kAInRegs = false;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    struct Raw {
        u32x4_a4 a, b;
        uint32_t c;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        const uint8_t *p = blk + 36 * g;
        r.a = *reinterpret_cast<const u32x4_a4 *>(p);
        r.b = *reinterpret_cast<const u32x4_a4 *>(p + 16);
        r.c = *reinterpret_cast<const uint32_t *>(p + 32);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t, const Tables &, int g) {
        const uint32_t w[9] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w, r.c};
        const Table16 tab = table16(qlin_iq4nl_values);
        float acc = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint32_t qs[4]; /* block 0: the nibble bytes start 2 bytes into dword 0; block 1: at dword 5 */
#pragma unroll
            for (int i = 0; i < 4; i++) qs[i] = h == 0 ? __builtin_amdgcn_alignbit(w[i + 1], w[i], 16) : w[5 + i];
            v4i c = {0, 0, 0, 0};
#pragma unroll
            for (int u = 0; u < 2; u++) {
                v4i b;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t nib = (qs[i] >> (4 * u)) & 0x0F0F0F0Fu;
                    b[i] = T == T_Q4_0 ? (int)nib : look4(nib, tab);
                }
                const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * (2 * h + u));
                const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
                c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
            }
            const float d = half_bits_fast(h == 0 ? w[0] & 0xFFFFu : w[4] >> 16);
            const int G = 2 * g + h;
            float dot = join_digits(c) * xo.meta[G];
            if (T == T_Q4_0) dot = fmaf(-8.0f, xo.meta[8 + 2 * G] + xo.meta[8 + 2 * G + 1], dot);
            acc = fmaf(dot, d, acc);
        }
        return acc;
    }
};
template <> struct GridFmt<T_IQ4_NL> : Nibble18<T_IQ4_NL> {};
template <> struct GridFmt<T_Q4_0> : Nibble18<T_Q4_0> {};

/* MXFP4 [e][16 nibble bytes] (common/ggml_dequant.h:2818-2830), 17 bytes: table[nibble] * 2^(e - 127) / 2, low
 * nibbles first as in IQ4_NL; 136 bytes per 256 elements. Lane group g takes blocks 2g and 2g + 1, the 34 bytes from
 * byte 34 g - which is 2 (mod 4) for odd g: nine aligned dwords from two bytes earlier there, and byte shifts. */
template <> struct GridFmt<T_MXFP4> {
    static constexpr int kBlock = 136, kGridBytes = 0;
    static constexpr int kPiece = 0, kAlign = 4;
    static constexpr int kStep = 16;
    static constexpr bool kSums = false, kAInRegs = false;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    struct Raw {
        u32x4_a4 a, b;
        uint32_t c;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        const uint8_t *p = blk + 34 * g - 2 * (g & 1);
        r.a = *reinterpret_cast<const u32x4_a4 *>(p);
        r.b = *reinterpret_cast<const u32x4_a4 *>(p + 16);
        r.c = *reinterpret_cast<const uint32_t *>(p + 32);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t, const Tables &, int g) {
        const uint32_t w[9] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w, r.c};
        const Table16 tab = table16(qlin_mxfp4_values);
        const uint32_t odd = (uint32_t)g & 1u; /* the piece starts two bytes into w */
        float acc = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint32_t qs[4]; /* block 0: the nibble bytes start 1 (3) bytes into dword 0; block 1: 2 bytes into dword 4 (at dword 5) */
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if (h == 0) qs[i] = __builtin_amdgcn_alignbit(w[i + 1], w[i], 8u + 16u * odd);
                else qs[i] = odd ? w[5 + i] : __builtin_amdgcn_alignbit(w[5 + i], w[4 + i], 16);
            }
            v4i c = {0, 0, 0, 0};
#pragma unroll
            for (int u = 0; u < 2; u++) {
                v4i b;
#pragma unroll
                for (int i = 0; i < 4; i++) b[i] = look4((qs[i] >> (4 * u)) & 0x0F0F0F0Fu, tab);
                const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * (2 * h + u));
                const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
                c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
            }
            const uint32_t e = (h == 0 ? w[0] >> (16u * odd) : w[4] >> (8u + 16u * odd)) & 0xFFu;
            acc = fmaf(join_digits(c) * xo.meta[2 * g + h], e8m0_half(e), acc);
        }
        return acc;
    }
};

/* NVFP4 [4 x ue4m3 scale][32 nibble bytes] per 64 elements (common/ggml_dequant.h:2832-2848), 36 bytes: sub-block s
 * of 16 elements is table[nibble] * scale_s over bytes 8 s .. 8 s + 7, low nibbles first. Lane group g takes block g
 * of the 256 elements, nine dwords; an instruction is one sub-block. */
template <> struct GridFmt<T_NVFP4> {
    static constexpr int kBlock = 144, kGridBytes = 0;
    static constexpr int kPiece = 0, kAlign = 4;
    static constexpr int kStep = 16;
    static constexpr bool kSums = false, kAInRegs = false;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    struct Raw {
        u32x4_a4 a, b;
        uint32_t c;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        const uint8_t *p = blk + 36 * g;
        r.a = *reinterpret_cast<const u32x4_a4 *>(p);
        r.b = *reinterpret_cast<const u32x4_a4 *>(p + 16);
        r.c = *reinterpret_cast<const uint32_t *>(p + 32);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t, const Tables &, int g) {
        const uint32_t w[9] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w, r.c};
        const Table16 tab = table16(qlin_mxfp4_values);
        float acc = 0.0f;
#pragma unroll
        for (int st = 0; st < 4; st++) {
            const uint32_t q0 = w[1 + 2 * st], q1 = w[2 + 2 * st];
            const v4i b = {look4(q0 & 0x0F0F0F0Fu, tab), look4(q1 & 0x0F0F0F0Fu, tab), look4((q0 >> 4) & 0x0F0F0F0Fu, tab),
                           look4((q1 >> 4) & 0x0F0F0F0Fu, tab)};
            const v4i zero = {0, 0, 0, 0};
            const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * st);
            const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
            const v4i c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, zero, 0, 0, 0);
            acc = fmaf(join_digits(c) * xo.meta[2 * g + (st >> 1)], ue4m3_half((w[0] >> (8 * st)) & 0xFFu), acc);
        }
        return acc;
    }
};

/* Q4_1 [d][m][16 nibble bytes] (common/ggml_dequant.h:2864-2877), Q5_0 [d][qh 4][16] (:2879-2895) and Q5_1
 * [d][m][qh 4][16] (:2897-2915): blocks of 32 elements in 20, 22 and 24 bytes; element l < 16 is the low nibble of
 * byte l (+ 16 x bit l of qh), element 16 + l the high nibble (+ 16 x bit 16 + l); Q4_1 and Q5_1 add m, Q5_0
 * subtracts 16. Lane group g takes blocks 2g and 2g + 1 as 10, 11 or 12 dwords; the codes stay unsigned and m or
 * -16 d goes onto the sum of x. */
template <uint32_t T> struct Legacy32 {
    static constexpr int kBytes = T == T_Q4_1 ? 20 : T == T_Q5_0 ? 22 : 24;
    static constexpr int kDw = kBytes / 2; /* dwords of two blocks */
    static constexpr bool kHigh = T != T_Q4_1, kMin = T != T_Q5_0;
    static constexpr int kBlock = 8 * kBytes, kGridBytes = 0;
    static constexpr int kPiece = 0, kAlign = 4;
    static constexpr int kStep = 16;
    static constexpr bool kSums = true, kAInRegs = false;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    struct Raw {
        uint32_t w[kDw];
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        const uint8_t *p = blk + 2 * kBytes * g;
#pragma unroll
        for (int i = 0; i + 4 <= kDw; i += 4) {
            const u32x4_a4 v = *reinterpret_cast<const u32x4_a4 *>(p + 4 * i);
            r.w[i] = v.x; r.w[i + 1] = v.y; r.w[i + 2] = v.z; r.w[i + 3] = v.w;
        }
        if (kDw % 4 >= 2) {
            const u32x2_a4 v = *reinterpret_cast<const u32x2_a4 *>(p + 4 * (kDw & ~3));
            r.w[kDw & ~3] = v.x; r.w[(kDw & ~3) + 1] = v.y;
        }
        if (kDw % 2) r.w[kDw - 1] = *reinterpret_cast<const uint32_t *>(p + 4 * (kDw - 1));
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t, const Tables &, int g) {
        const uint32_t(&w)[kDw] = r.w;
        float acc = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint32_t dm, qh = 0, qs[4];
            if (T == T_Q5_0) { /* the second block starts in the middle of dword 5 */
                dm = h == 0 ? w[0] & 0xFFFFu : w[5] >> 16;
                qh = h == 0 ? __builtin_amdgcn_alignbit(w[1], w[0], 16) : w[6];
#pragma unroll
                for (int i = 0; i < 4; i++) qs[i] = h == 0 ? __builtin_amdgcn_alignbit(w[i + 2], w[i + 1], 16) : w[7 + i];
            } else {
                constexpr int kHead = kHigh ? 2 : 1;
                const int b = (kDw / 2) * h;
                dm = w[b];
                if (kHigh) qh = w[b + 1];
#pragma unroll
                for (int i = 0; i < 4; i++) qs[i] = w[b + kHead + i];
            }
            v4i c = {0, 0, 0, 0};
#pragma unroll
            for (int u = 0; u < 2; u++) {
                v4i b;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    uint32_t code = (qs[i] >> (4 * u)) & 0x0F0F0F0Fu;
                    if (kHigh) code |= spread4(qh >> (16 * u + 4 * i)) << 4;
                    b[i] = (int)code;
                }
                const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * (2 * h + u));
                const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
                c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
            }
            const int G = 2 * g + h;
            const float sum = xo.meta[8 + 2 * G] + xo.meta[8 + 2 * G + 1];
            const float d = half_bits_fast(dm & 0xFFFFu);
            float dot = join_digits(c) * xo.meta[G];
            if (!kMin) dot = fmaf(-16.0f, sum, dot);
            acc = fmaf(dot, d, acc);
            if (kMin) acc = fmaf(half_bits_fast(dm >> 16), sum, acc);
        }
        return acc;
    }
};
template <> struct GridFmt<T_Q4_1> : Legacy32<T_Q4_1> {};
template <> struct GridFmt<T_Q5_0> : Legacy32<T_Q5_0> {};
template <> struct GridFmt<T_Q5_1> : Legacy32<T_Q5_1> {};

/* IQ4_XS [d][scales_h 2][scales_l 4][qs 128] (:2956-2973), 136 bytes: group j of 32 elements has its nibbles in
 * qs[16 j ..] (low nibbles first, as IQ4_NL) and a 6-bit scale - 32. Lane group g takes groups 2g, 2g+1. */
template <> struct GridFmt<T_IQ4_XS> {
    static constexpr int kBlock = 136, kGridBytes = 0;
    static constexpr int kPiece = 0, kAlign = 4;
    static constexpr int kStep = 16;
    static constexpr bool kSums = false, kAInRegs = false;
    __device__ static const uint32_t *grid_src() { return nullptr; }
    __device__ static int elem0(int g, int st) { return 64 * g + 16 * st; }
    struct Raw {
        u32x4_a4 a, b;
        u32x2_a4 hd;
    };
    __device__ static Raw load(const uint8_t *blk, int g) {
        Raw r;
        r.hd = *reinterpret_cast<const u32x2_a4 *>(blk);
        r.a = *reinterpret_cast<const u32x4_a4 *>(blk + 8 + 32 * g);
        r.b = *reinterpret_cast<const u32x4_a4 *>(blk + 24 + 32 * g);
        return r;
    }
    __device__ static float item(const XOperand &xo, const Raw &r, uint32_t, const Tables &, int g) {
        const uint32_t qs[8] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w};
        const Table16 tab = table16(qlin_iq4nl_values);
        float acc = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            v4i c = {0, 0, 0, 0};
#pragma unroll
            for (int u = 0; u < 2; u++) {
                v4i b;
#pragma unroll
                for (int i = 0; i < 4; i++) b[i] = look4((qs[4 * h + i] >> (4 * u)) & 0x0F0F0F0Fu, tab);
                const uint4 av = *reinterpret_cast<const uint4 *>(xo.arows + kStep * (2 * h + u));
                const v4i a = {(int)av.x, (int)av.y, (int)av.z, (int)av.w};
                c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
            }
            const int j = 2 * g + h;
            const uint32_t ls = ((r.hd.y >> (4 * j)) & 15u) | ((((r.hd.x >> 16) >> (2 * j)) & 3u) << 4);
            acc = fmaf(join_digits(c) * xo.meta[j], (float)((int)ls - 32), acc);
        }
        return half_bits_fast(r.hd.x & 0xFFFFu) * acc;
    }
};

}  // namespace

/* MOE = 0: the matvec. MOE = 1, 2: a token's routed experts (the reference's MoE block for a token,
 * common/transformer.h:4045-4131) on the same kernel, as moe1_q4k_kernel (gemv_q4k.hip) does for Q4_K:
 *   1  gate + up + SiLU of pair blockIdx.y = token * top_k + k: the job's two matrices moved to expert idx[pair], the
 *      result to h[pair], x the token's bf16 activations;
 *   2  down of token blockIdx.y: one matvec over a row of top_k * n_ff elements whose super-blocks sit in different
 *      experts, x = h scaled by the routing weight of the super-block's expert (nothing for an index out of range). */
struct MoeArgs {
    const int32_t *idx;
    const float *wts;
    int top_k, n_expert, sb_per_expert;
    int ldx; /* elements between two tokens' activations (MOE = 1) or rows of h (MOE = 2) */
    size_t expert_bytes;
    int sb0; /* MOE = 2: the launch covers super-blocks sb0, sb0 + 1, ... of the token's row (x points at sb0's) */
};

template <uint32_t T, int NKC, int MOE = 0>
__global__ void __launch_bounds__(kWaves * 64)
gemv_grid_kernel(const JobView job_in, const float *__restrict__ x, int n_sb, int rows_per_wg, size_t row_bytes, const MoeArgs moe,
                 int lone_ahead) {
    using F = GridFmt<T>;
    JobView job = job_in;
    const int32_t *idx = moe.idx;
    const float *wts = moe.wts;
    if (MOE == 1) {
        const int pair = blockIdx.y, e = idx[pair];
        if (e < 0 || e >= moe.n_expert) return; /* uniform over the workgroup */
        job.W0 += (size_t)e * moe.expert_bytes;
        job.W1 += (size_t)e * moe.expert_bytes;
        job.y0 += (size_t)pair * job.n0;
        x = reinterpret_cast<const float *>(reinterpret_cast<const uint16_t *>(x) + (size_t)(pair / moe.top_k) * moe.ldx);
    } else if (MOE == 2) {
        idx += (size_t)blockIdx.y * moe.top_k;
        wts += (size_t)blockIdx.y * moe.top_k;
        x += (size_t)blockIdx.y * moe.ldx;
        job.y0 += (size_t)blockIdx.y * job.n0;
    }
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 15, g = lane >> 4;

    /* a workgroup owns rows_per_wg rows: of the concatenated matrices, or, where two results are
     * combined (mode 2), the same rows of both matrices (local rows: first matrix, then second) */
    const bool paired = job.mode == 2;
    const int n_mats_here = paired ? 2 : 1;
    const int n_rows = paired ? job.n0 : job.n0 + job.n1 + job.n2;
    const int row0 = blockIdx.x * rows_per_wg;
    int rows_here = n_rows - row0;
    if (rows_here > rows_per_wg) rows_here = rows_per_wg;
    const int n_lrows = rows_here * n_mats_here;
    const int n_rg = (n_lrows + 15) >> 4;
    const int n_kc = wv < n_sb ? ((n_sb - wv + 15) >> 4) : 0; /* this wave's super-blocks: wv, wv+16, ... */

    /* LDS: x scratch per wave, the grid and the sign masks at addresses the compiler knows (a lookup is then a
     * shift, a mask and a read with a constant offset); the partial sums [rows][kWaves] behind them */
    __shared__ __attribute__((aligned(16))) uint8_t xs_all[kWaves * kXScratch];
    __shared__ __attribute__((aligned(16))) uint32_t grid_lds[F::kGridBytes > 0 ? F::kGridBytes / 4 : 4];
    __shared__ __attribute__((aligned(16))) uint2 sign_lds[F::kGridBytes > 0 ? 256 + 128 : 2];
    uint8_t *xs = xs_all + wv * kXScratch;
    float *partial = reinterpret_cast<float *>(lds);
    const Tables tab = {grid_lds, sign_lds, sign_lds + (F::kGridBytes > 0 ? 256 : 0)};

    const bool one_matrix = !paired && job.n1 == 0 && job.n2 == 0; /* a scalar test: no search by row then */
    auto locate = [&](int lr, const uint8_t *&Wm, float *&ym, int &r) {
        if (one_matrix) {
            Wm = job.W0;
            ym = job.y0;
            r = row0 + lr;
        } else if (paired) {
            const bool second = lr >= rows_here;
            Wm = second ? job.W1 : job.W0;
            ym = job.y0;
            r = row0 + (second ? lr - rows_here : lr);
        } else {
            job_locate(job, row0 + lr, Wm, ym, r);
        }
    };
    auto row_pointer = [&](int rg) { /* this lane's row of row group rg (rows past the end: the last one, never stored) */
        int lr = 16 * rg + n;
        if (lr >= n_lrows) lr = n_lrows - 1;
        /* by branches: a choice between the three matrix arguments by selects becomes a load from the argument
         * block, with a full wait, in front of every weight request */
        const uint8_t *Wm;
        float *ym;
        int r;
        locate(lr, Wm, ym, r);
        return Wm + (size_t)r * row_bytes;
    };
    /* where in its row the wave's super-block kc sits (MOE = 2: in which expert's copy of the row, too; an index
     * out of range reads expert 0 and gets zeros for x) */
    auto sb_off = [&](int kc) {
        const int s = wv + 16 * kc;
        if (MOE == 2) {
            const int v = moe.sb0 + s, j = v / moe.sb_per_expert, e = idx[j];
            const bool valid = e >= 0 && e < moe.n_expert;
            return (size_t)(valid ? e : 0) * moe.expert_bytes + (size_t)(v - j * moe.sb_per_expert) * F::kBlock;
        }
        return (size_t)s * F::kBlock;
    };
    auto moe_x = [&](v4f v, int kc) { /* MOE = 2: the routing weight of the super-block's expert goes onto x */
        if (MOE == 2) {
            const int j = (moe.sb0 + wv + 16 * kc) / moe.sb_per_expert, e = idx[j];
            const float wj = wts[j];
            const v4f zero = {0.0f, 0.0f, 0.0f, 0.0f};
            v = (e >= 0 && e < moe.n_expert) ? v * wj : zero;
        }
        return v;
    };

    /* the wave's first super-block of x; later ones are fetched where they are used */
    auto load_x = [&](int kc) {
        if (MOE == 1) { /* bf16 activations */
            const uint2 b = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(x) + (size_t)(16 * kc + wv) * 256 + 4 * lane);
            const v4f v = {__uint_as_float(b.x << 16), __uint_as_float(b.x & 0xFFFF0000u), __uint_as_float(b.y << 16),
                           __uint_as_float(b.y & 0xFFFF0000u)};
            return v;
        }
        return *reinterpret_cast<const v4f *>(x + (size_t)(16 * kc + wv) * 256 + 4 * lane);
    };
    v4f xq = {0.0f, 0.0f, 0.0f, 0.0f};
    if (n_kc > 0) xq = load_x(0);

    /* x -> signed digit planes -> A operands, wave-private */
    auto prepare = [&](v4f v, XOperand &xo) {
        /* the largest |x| of the group as a bit pattern: an integer maximum keeps a NaN or an Inf on top */
        constexpr uint32_t kAbs = 0x7FFFFFFFu;
        uint32_t amax = max(max(__float_as_uint(v.x) & kAbs, __float_as_uint(v.y) & kAbs),
                            max(__float_as_uint(v.z) & kAbs, __float_as_uint(v.w) & kAbs));
        /* 8 consecutive lanes share one 32-element group */
        amax = max(amax, dpp_movu<0xB1>(amax));
        amax = max(amax, dpp_movu<0x4E>(amax));
        amax = max(amax, dpp_movu<0x141>(amax));
        int e = (int)(amax >> 23) - 126; /* amax in [2^(e-1), 2^e) */
        if (e < -96) e = -96;            /* zero and tiny groups */
        const float up = __uint_as_float((uint32_t)(127 + 22 - e) << 23);
        float down = __uint_as_float((uint32_t)(127 - 22 + e) << 23);
        if (amax >= 0x7F800000u) down = __uint_as_float(0x7FC00000u); /* Inf/NaN in x: poison every row */
        const int X[4] = {__float2int_rn(v.x * up), __float2int_rn(v.y * up), __float2int_rn(v.z * up),
                          __float2int_rn(v.w * up)};
        /* The three signed base-256 digits of X (X = 256*X1 + d0 with d0 = (int8)X, X1 = 256*X2 + d1, X2 in
         * [-64, 64]) are bytes 0..2 of (X + 0x8080) ^ 0x8080: adding 128 at a byte makes its digit unsigned and
         * carries exactly when the digit is negative, the xor takes the 128 off again. */
        uint32_t Z[4];
#pragma unroll
        for (int k = 0; k < 4; k++) Z[k] = ((uint32_t)X[k] + 0x00008080u) ^ 0x00008080u;
        /* byte transpose: plane j = byte j of Z[0..3] (selector 0-3: second operand, 4-7: first) */
        const uint32_t lo01 = __builtin_amdgcn_perm(Z[1], Z[0], 0x05010400u), lo23 = __builtin_amdgcn_perm(Z[3], Z[2], 0x05010400u);
        const uint32_t hi01 = __builtin_amdgcn_perm(Z[1], Z[0], 0x07030602u), hi23 = __builtin_amdgcn_perm(Z[3], Z[2], 0x07030602u);
        uint32_t *pl = reinterpret_cast<uint32_t *>(xs);
        pl[lane] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);       /* digit 2 (top) */
        pl[64 + lane] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);  /* digit 1 */
        pl[128 + lane] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u); /* digit 0 */
        if ((lane & 7) == 0) reinterpret_cast<float *>(xs + 1024)[lane >> 3] = down;
        if (F::kSums) { /* the sum of x over each 16 elements: four lanes */
            float sum = (v.x + v.y) + (v.z + v.w);
            sum += dpp_mov<0xB1>(sum);
            sum += dpp_mov<0x4E>(sum);
            if ((lane & 3) == 0) reinterpret_cast<float *>(xs + 1056)[lane >> 2] = sum;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        /* A operand: x row i = lane%16 = 4*g' + plane (plane 3 unused) is live in lane group g' only and holds,
         * for instruction s, the digits of the 16 elements from F::elem0(g', s) on. Every other lane reads zeros. */
        const int plane = n & 3;
        const bool live = (n >> 2) == g && plane < 3;
        xo.arows = xs + (live ? plane * 256 + F::elem0(g, 0) : 768);
        if (F::kAInRegs) {
#pragma unroll
            for (int st = 0; st < 4; st++) {
                const uint4 d = *reinterpret_cast<const uint4 *>(xo.arows + F::kStep * st);
                const v4i a = {(int)d.x, (int)d.y, (int)d.z, (int)d.w};
                xo.A[st] = a;
            }
        }
        xo.meta = reinterpret_cast<const float *>(xs + 1024);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

    auto store_partial = [&](int rg, float v, bool add) { /* the four lane groups hold four shares of the same row */
        v = sum_lane_groups(v);
        const int lr = 16 * rg + n;
        if (lane < 16 && lr < n_lrows) {
            float *p = partial + lr * kWaves + wv;
            *p = add ? *p + v : v;
        }
    };

    /* every piece of a block that a lane reads starts F::kPiece (mod 4) bytes into the block: the funnel shift of its bytes */
    auto shift_of = [](const uint8_t *blk) { return (((uint32_t)(uintptr_t)blk + (uint32_t)F::kPiece) & 2u) * 8u; };

    /* the first blocks are requested before the tables are built and x is prepared: the wave's first two
     * super-blocks of a lone row group (long rows), else its first super-block of the first row groups */
    const bool long_rows = NKC > 1 && n_rg < 2 && lone_ahead;
    /* row groups of a super-block column in flight per wave: with sixteen waves per compute unit one is enough, and
     * two or four measured slower for every format (IQ2_XXS 8192 x 28672: 38.8 us with four, 29.6 with one) */
    constexpr int D = 1;
    constexpr int NF = (NKC > 1 && D < 2) ? 2 : D; /* the long-rows path keeps two */
    typename F::Raw first[NF];
    uint32_t first_sh[NF];
    if (n_kc > 0) {
#pragma unroll
        for (int q = 0; q < NF; q++) {
            if (long_rows ? q >= 2 : q >= D) break;
            const uint8_t *blk = long_rows ? row_pointer(0) + sb_off(q < n_kc ? q : 0) : row_pointer(q < n_rg ? q : 0) + sb_off(0);
            first[q] = F::load(blk, g);
            first_sh[q] = shift_of(blk);
        }
    }
    if (lane < 32) reinterpret_cast<uint32_t *>(xs + 768)[lane] = 0u; /* what the dead lanes of the x operand read */
    for (int t = threadIdx.x; t < F::kGridBytes / 4; t += kWaves * 64) grid_lds[t] = F::grid_src()[t];
    if (F::kGridBytes > 0 && threadIdx.x < 384) {
        const uint32_t i = threadIdx.x, sb = i < 256 ? i : iq_sign_byte(i - 256);
        sign_lds[i] = make_uint2(spread4(sb) * 0xFFu, spread4(sb >> 4) * 0xFFu);
    }
    __syncthreads();

    XOperand xo;
    if (n_kc == 0) { /* a wave without a super-block (K < 4096) contributes zeros */
        for (int rg = 0; rg < n_rg; rg++) store_partial(rg, 0.0f, false);
    } else if (long_rows) {
        /* one row group: the wave's super-blocks of it, two requested ahead of the one being multiplied */
        float acc = 0.0f;
        const uint8_t *blk0 = row_pointer(0);
#pragma unroll
        for (int kc = 0; kc < NKC; kc++) {
            if (kc < n_kc) {
                prepare(moe_x(xq, kc), xo);
                if (kc + 1 < n_kc) xq = load_x(kc + 1); /* on its way while this super-block is multiplied */
                acc += F::item(xo, first[kc & 1], first_sh[kc & 1], tab, g);
            }
            if (kc + 2 < n_kc) { /* into the registers just used */
                const uint8_t *blk = blk0 + sb_off(kc + 2);
                first[kc & 1] = F::load(blk, g);
                first_sh[kc & 1] = shift_of(blk);
            }
            __builtin_amdgcn_sched_barrier(0); /* one super-block at a time: interleaving them costs registers */
        }
        store_partial(0, acc, false);
    } else {
        for (int kc = 0; kc < n_kc; kc++) {
            v4f v = xq;
            if (kc > 0) v = load_x(kc);
            prepare(moe_x(v, kc), xo);
            /* D row groups in flight: a group's registers are refilled as soon as it has been multiplied */
            if (kc > 0) {
#pragma unroll
                for (int q = 0; q < D; q++) {
                    const uint8_t *blk = row_pointer(q < n_rg ? q : 0) + sb_off(kc);
                    first[q] = F::load(blk, g);
                    first_sh[q] = shift_of(blk);
                }
            }
            for (int rg = 0; rg < n_rg; rg += D) {
#pragma unroll
                for (int q = 0; q < D; q++) {
                    if (rg + q < n_rg) store_partial(rg + q, F::item(xo, first[q], first_sh[q], tab, g), kc > 0);
                    if (rg + q + D < n_rg) {
                        const uint8_t *blk = row_pointer(rg + q + D) + sb_off(kc);
                        first[q] = F::load(blk, g);
                        first_sh[q] = shift_of(blk);
                    }
                }
            }
        }
    }
    __syncthreads();

    /* sum the waves' shares of each row and store */
    auto row_total = [&](int lr) {
        const float4 *p = reinterpret_cast<const float4 *>(partial + lr * kWaves);
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < kWaves / 4; k++) {
            const float4 v = p[k];
            s += (v.x + v.y) + (v.z + v.w);
        }
        return s;
    };
    if (paired) {
        for (int lr = threadIdx.x; lr < rows_here; lr += kWaves * 64)
            job.y0[row0 + lr] = silu_times(row_total(lr), row_total(rows_here + lr));
    } else {
        for (int lr = threadIdx.x; lr < n_lrows; lr += kWaves * 64) {
            const uint8_t *Wm;
            float *ym;
            int r;
            locate(lr, Wm, ym, r);
            const float s = row_total(lr);
            ym[r] = job.mode == 1 ? ym[r] + s : s;
        }
    }
}

namespace {

/* Rows of up to 4096 elements, one super-block per wave and one row group per wave in flight (two and four measured
 * slower for every format): where this kernel measured faster than the v_dot4 kernel (gemv_int.hip) over 1024 to
 * 151936 rows of 2048 to 4096 elements. 14336 x 4096, us: IQ4_NL 13.3 -> 10.3, IQ4_XS 12.8 -> 10.6, Q4_0 10.4 -> 8.7,
 * Q2_K 10.0 -> 8.0, IQ2_XXS 11.0 -> 9.0, Q3_K 13.8 -> 12.8, IQ3_S 13.3 -> 12.5, Q5_K 12.8 -> 12.5; 151936 x 4096:
 * IQ2_XXS 82 -> 51, Q2_K 74 -> 54, IQ4_NL 100 -> 79, but Q5_K 90 -> 112, Q6_K 103 -> 141, Q8_0 103 -> 132 (and
 * Q6_K, Q8_0 no faster at 14336 rows or below 4096: they come here for 4096 to 8192 rows only, 4096 x 4096:
 * Q8_0 6.9 -> 6.0, Q6_K 7.1 -> 6.8; 8192 x 4096: 9.3 -> 8.7, 11.1 -> 10.0). With fewer than eight super-blocks more
 * than half of the waves would have nothing to do. Two workgroups per compute unit (the instances of 64 registers
 * or fewer would fit) measured slower for every format. */
bool short_rows_pay(uint32_t type, int n_sb, int n_rows) {
    if (n_sb < 8) return false;
    switch (type) {
    case T_IQ4_NL: case T_IQ4_XS: case T_Q4_0: case T_Q2_K: case T_IQ2_XXS: case T_IQ3_XXS: case T_IQ3_S: return true;
    case T_IQ2_XS: return true; /* 14336: 12.0 -> 10.3, 151936: 90 -> 64; IQ2_S (12.7 against 13.0, 95 against 101) stays */
    case T_TQ1_0: return true; /* 14336: 31.7 -> 15.7, 151936: 306 -> 107 */
    case T_Q1_0: case T_IQ1_S: case T_IQ1_M: return true; /* 14336: 10.9 -> 7.5, 13.9 -> 10.5, 16.0 -> 10.7; 151936: 89 -> 44, 111 -> 75, 135 -> 67 */
    case T_MXFP4: case T_NVFP4: case T_TQ2_0: return true; /* 14336: 13.4 -> 11.2, 17.9 -> 12.5, 11.7 -> 7.4; 151936: 98 -> 74, 162 -> 88, 93 -> 43 */
    case T_Q3_K: return n_rows >= 4096;
    case T_Q5_K: return n_rows <= 16384;
    case T_Q4_1: case T_Q5_0: case T_Q5_1: return n_rows <= 32768; /* 14336: 10.5 -> 9.3, 12.1 -> 10.0, 12.0 -> 10.3; 151936: 67 -> 88 */
    case T_Q6_K: case T_Q8_0: return n_rows >= 4096 && n_rows <= 8192;
    default: return false;
    }
}

template <uint32_t T>
bool grid_typed(const GemvJob &job, const float *x, int n_cols, int n_cu, hipStream_t stream, hipError_t *err,
                size_t row_stride) {
    const int n_sb = n_cols / 256;
    const bool short_rows = n_sb <= 16;
    if (n_cols % 256 != 0 || n_sb > 16 * kMaxKc || ((uintptr_t)x & 15)) return false;
    /* what the format's loads want of the addresses (block sizes are even; the formats whose 256 elements fill a
     * multiple of 4 or 16 bytes read whole dwords or 16-byte groups) */
    for (int m = 0; m < job.n_mat; m++)
        if ((uintptr_t)job.W[m] % GridFmt<T>::kAlign) return false;
    if (row_stride % GridFmt<T>::kAlign) return false;
    const int n_mats_here = job.mode == kSiluMul ? 2 : 1;
    const int n_rows = job.mode == kSiluMul ? job.n_rows[0] : job.total_rows();
    if (n_rows == 0) return false;
    if (short_rows && !short_rows_pay(T, n_sb, n_rows * n_mats_here)) return false;
    /* one workgroup per compute unit where its partial sums fit in LDS (with the lookup tables: in 128 rows' worth,
     * more measured slower for those formats), else so many equal rounds of workgroups that they do (Q2_K 151936 x
     * 4096: 55 -> 48 us, 49152 rows 22.3 -> 17.4) */
    constexpr int max_rows = GridFmt<T>::kGridBytes > 0 ? 128 : kMaxRowsPerWg;
    const int rows_per_cu = (n_rows + n_cu - 1) / n_cu;
    const int rounds = (rows_per_cu * n_mats_here + max_rows - 1) / max_rows;
    int rows_per_wg = (n_rows + n_cu * rounds - 1) / (n_cu * rounds);
    /* long rows: whole row groups, a matrix instruction wants 16 rows anyway; short ones: a workgroup on every
     * compute unit counts for more (14336 rows: 56 each) */
    if (!short_rows) rows_per_wg = (rows_per_wg + 15) & ~15;
    if (rows_per_wg * n_mats_here > max_rows) rows_per_wg = max_rows / n_mats_here;
    const int grid = (n_rows + rows_per_wg - 1) / rows_per_wg;
    const size_t lds_bytes = (size_t)rows_per_wg * n_mats_here * kWaves * 4; /* the partial sums; the rest is static */
    const JobView view = job_view(job);
    const size_t pitch = row_stride ? row_stride : (size_t)n_sb * GridFmt<T>::kBlock;
    const MoeArgs none = {nullptr, nullptr, 0, 0, 0, 0, 0, 0};
    if (short_rows)
        hipLaunchKernelGGL((gemv_grid_kernel<T, 1>), dim3(grid), dim3(kWaves * 64), lds_bytes, stream, view, x, n_sb, rows_per_wg, pitch, none, 1);
    else
        {
        /* a lone row group per workgroup: two super-blocks requested ahead, except for the two formats with the most
         * loads per item where every compute unit has a workgroup - there one super-block at a time measured faster
         * (Q6_K 4096 x 8192: 11.3 -> 9.9 us, 4096 x 14336: 14.9 -> 14.6; IQ3_S 10.7 -> 9.9, 13.5 -> 13.0) */
        const bool one_at_a_time = (T == T_Q6_K || T == T_IQ3_S) && grid >= n_cu;
        hipLaunchKernelGGL((gemv_grid_kernel<T, kMaxKc>), dim3(grid), dim3(kWaves * 64), lds_bytes, stream, view, x, n_sb, rows_per_wg, pitch, none,
                           one_at_a_time ? 0 : 1);
    }
    *err = hipGetLastError();
    return true;
}

}  // namespace

namespace {

template <uint32_t T>
bool moe1_up_typed(const void *gate, const void *up, const uint16_t *X, const int32_t *idx, float *h, int n_tok, int top_k,
                   int n_embd, int n_ff, int n_expert, int n_cu, hipStream_t stream, bool dry, hipError_t *err) {
    using F = GridFmt<T>;
    const int n_sb = n_embd / 256;
    const size_t row_bytes = (size_t)n_sb * F::kBlock, expert_bytes = (size_t)n_ff * row_bytes;
    if (n_embd % 256 != 0 || n_sb > 16 * kMaxKc || n_ff < 1 || top_k < 1 || n_tok < 1) return false;
    if (((uintptr_t)gate | (uintptr_t)up | expert_bytes) % F::kAlign || ((uintptr_t)X & 7) || ((uintptr_t)h & 15)) return false;
    if (dry) return true;
    constexpr int max_rows = F::kGridBytes > 0 ? 128 : kMaxRowsPerWg;
    const int n_pairs = n_tok * top_k;
    const int tiles = n_cu / n_pairs > 0 ? n_cu / n_pairs : 1;
    int rows_per_wg = (n_ff + tiles - 1) / tiles;
    if (2 * rows_per_wg > max_rows) rows_per_wg = max_rows / 2;
    GemvJob job = {};
    job.W[0] = gate; job.W[1] = up; job.y[0] = h;
    job.n_rows[0] = job.n_rows[1] = n_ff;
    job.n_mat = 2;
    job.mode = kSiluMul;
    const MoeArgs moe = {idx, nullptr, top_k, n_expert, n_sb, n_embd, expert_bytes, 0};
    const dim3 grid((n_ff + rows_per_wg - 1) / rows_per_wg, n_pairs);
    const size_t lds_bytes = (size_t)2 * rows_per_wg * kWaves * 4;
    const float *x = reinterpret_cast<const float *>(X);
    if (n_sb <= 16)
        hipLaunchKernelGGL((gemv_grid_kernel<T, 1, 1>), grid, dim3(kWaves * 64), lds_bytes, stream, job_view(job), x, n_sb, rows_per_wg, row_bytes, moe, 1);
    else
        hipLaunchKernelGGL((gemv_grid_kernel<T, kMaxKc, 1>), grid, dim3(kWaves * 64), lds_bytes, stream, job_view(job), x, n_sb, rows_per_wg, row_bytes, moe, 1);
    *err = hipGetLastError();
    return true;
}

template <uint32_t T>
bool moe1_down_typed(const void *down, const float *h, const int32_t *idx, const float *w, float *out, int n_tok, int top_k,
                     int n_embd, int n_ff, int n_expert, int n_cu, hipStream_t stream, bool dry, hipError_t *err) {
    using F = GridFmt<T>;
    const int sbpe = n_ff / 256, n_sb = top_k * sbpe; /* the row of a token: top_k experts' rows side by side */
    const size_t row_bytes = (size_t)sbpe * F::kBlock, expert_bytes = (size_t)n_embd * row_bytes;
    if (n_ff % 256 != 0 || n_embd < 1 || top_k < 1 || n_tok < 1) return false;
    if (((uintptr_t)down | row_bytes) % F::kAlign || ((uintptr_t)h & 15)) return false;
    if (dry) return true;
    constexpr int max_rows = F::kGridBytes > 0 ? 128 : kMaxRowsPerWg;
    const int tiles = n_cu / n_tok > 0 ? n_cu / n_tok : 1;
    int rows_per_wg = (n_embd + tiles - 1) / tiles;
    if (rows_per_wg > max_rows) rows_per_wg = max_rows;
    const dim3 grid((n_embd + rows_per_wg - 1) / rows_per_wg, n_tok);
    const size_t lds_bytes = (size_t)rows_per_wg * kWaves * 4;
    /* a launch takes 64 super-blocks of the row; a longer row (wide experts) goes in ranges, the later ones adding */
    for (int sb0 = 0; sb0 < n_sb; sb0 += 16 * kMaxKc) {
        const int n_here = n_sb - sb0 < 16 * kMaxKc ? n_sb - sb0 : 16 * kMaxKc;
        GemvJob job = single_job(down, out, n_embd, sb0 == 0 ? kStore : kAdd);
        const MoeArgs moe = {idx, w, top_k, n_expert, sbpe, n_sb * 256, expert_bytes, sb0};
        const float *x = h + (size_t)sb0 * 256;
        if (n_here <= 16)
            hipLaunchKernelGGL((gemv_grid_kernel<T, 1, 2>), grid, dim3(kWaves * 64), lds_bytes, stream, job_view(job), x, n_here, rows_per_wg, row_bytes, moe, 1);
        else
            hipLaunchKernelGGL((gemv_grid_kernel<T, kMaxKc, 2>), grid, dim3(kWaves * 64), lds_bytes, stream, job_view(job), x, n_here, rows_per_wg, row_bytes, moe, 1);
    }
    *err = hipGetLastError();
    return true;
}

}  // namespace

/* every format of this kernel (Q4_K experts take moe1_q4k_kernel, gemv_q4k.hip) */
#define QLIN_MOE1_TYPES(X)                                                                                           \
    X(T_Q6_K) X(T_Q5_K) X(T_Q8_0) X(T_Q4_0) X(T_Q4_1) X(T_Q5_0) X(T_Q5_1) X(T_IQ4_NL) X(T_IQ4_XS) X(T_Q2_K) X(T_Q3_K)  \
    X(T_MXFP4) X(T_NVFP4) X(T_TQ2_0) X(T_Q1_0) X(T_IQ2_XXS) X(T_IQ2_XS) X(T_IQ2_S) X(T_IQ3_XXS) X(T_IQ3_S) X(T_IQ1_S) X(T_IQ1_M) X(T_TQ1_0)

bool launch_moe1_grid_up(uint32_t type, const void *gate, const void *up, const uint16_t *X, const int32_t *idx, float *h,
                         int n_tok, int top_k, int n_embd, int n_ff, int n_expert, int n_cu, hipStream_t stream, bool dry,
                         hipError_t *err) {
    *err = hipSuccess;
    switch (type) {
#define QLIN_CASE(TT) case TT: return moe1_up_typed<TT>(gate, up, X, idx, h, n_tok, top_k, n_embd, n_ff, n_expert, n_cu, stream, dry, err);
    QLIN_MOE1_TYPES(QLIN_CASE)
#undef QLIN_CASE
    default: return false;
    }
}

bool launch_moe1_grid_down(uint32_t type, const void *down, const float *h, const int32_t *idx, const float *w, float *out,
                           int n_tok, int top_k, int n_embd, int n_ff, int n_expert, int n_cu, hipStream_t stream, bool dry,
                           hipError_t *err) {
    *err = hipSuccess;
    switch (type) {
#define QLIN_CASE(TT) case TT: return moe1_down_typed<TT>(down, h, idx, w, out, n_tok, top_k, n_embd, n_ff, n_expert, n_cu, stream, dry, err);
    QLIN_MOE1_TYPES(QLIN_CASE)
#undef QLIN_CASE
    default: return false;
    }
}

bool gemv_grid_covers(uint32_t type) {
    return type == T_IQ2_XXS || type == T_IQ3_XXS || type == T_IQ3_S || type == T_Q6_K || type == T_Q5_K || type == T_Q8_0 ||
           type == T_IQ4_NL || type == T_IQ4_XS || type == T_Q4_0 || type == T_Q2_K || type == T_Q3_K ||
           type == T_Q4_1 || type == T_Q5_0 || type == T_Q5_1 || type == T_MXFP4 || type == T_NVFP4 || type == T_TQ2_0 || type == T_IQ2_XS || type == T_IQ2_S || type == T_Q1_0 || type == T_IQ1_S || type == T_IQ1_M || type == T_TQ1_0;
}

bool launch_gemv_grid(uint32_t type, const GemvJob &job, const float *x, int n_cols, int n_cu, hipStream_t stream,
                      hipError_t *err, size_t row_stride) {
    *err = hipSuccess;
    switch (type) {
    case T_IQ2_XXS: return grid_typed<T_IQ2_XXS>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ3_XXS: return grid_typed<T_IQ3_XXS>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ3_S: return grid_typed<T_IQ3_S>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q6_K: return grid_typed<T_Q6_K>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q5_K: return grid_typed<T_Q5_K>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q8_0: return grid_typed<T_Q8_0>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ4_NL: return grid_typed<T_IQ4_NL>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ4_XS: return grid_typed<T_IQ4_XS>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q4_0: return grid_typed<T_Q4_0>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q2_K: return grid_typed<T_Q2_K>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q3_K: return grid_typed<T_Q3_K>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q4_1: return grid_typed<T_Q4_1>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q5_0: return grid_typed<T_Q5_0>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q5_1: return grid_typed<T_Q5_1>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_MXFP4: return grid_typed<T_MXFP4>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_NVFP4: return grid_typed<T_NVFP4>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_TQ2_0: return grid_typed<T_TQ2_0>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ2_XS: return grid_typed<T_IQ2_XS>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ2_S: return grid_typed<T_IQ2_S>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_Q1_0: return grid_typed<T_Q1_0>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ1_S: return grid_typed<T_IQ1_S>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_IQ1_M: return grid_typed<T_IQ1_M>(job, x, n_cols, n_cu, stream, err, row_stride);
    case T_TQ1_0: return grid_typed<T_TQ1_0>(job, x, n_cols, n_cu, stream, err, row_stride);
    default: return false;
    }
}

}  // namespace qlin
