/*
 * gemm_q4k_wave4.hip - Q4_K x bf16 prefill GEMM for more than 128 tokens: four waves per workgroup, one per SIMD.
 *
 *   Y[t*ldy + r] = sum_k X[t*ldx + k] * decode(W)[r][k]      X bf16, Y fp32, fp32 accumulate
 *
 * The contraction of tf_gemm_f16_mt_tokenmajor for a Q4_K tensor (common/transformer.h:4487, generic
 * branch :4535-4572) with the weights decoded as dequantize_row_q4_K does (common/ggml_dequant.h:1592-1618,
 * y = (d*sc)*q - dmin*m in fp32) and rounded once to bf16, nearest even.
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
 * k inside a tile is permuted so that a lane's 16 code bytes serve its four k-steps: k-step s of lane half kg covers
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
/* raw blocks of one super-block of a wave's 32 weight rows (32 x 144 bytes, rounded up to five requests of 1 KB) */
constexpr int kWRaw = 5 * 1024;
__shared__ __attribute__((aligned(1024))) uint8_t w4_wraw[4 * kWRaw];

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

/* header and codes of one super-block of a lane's weight row: 16 of the 32 code bytes of each quarter */
struct SbRegs { u32x4 hdr; u32x4 q[4]; };

/* everything a slot touches; every member ends up in registers (all indices are constants after inlining) */
struct Ctx {
    floatx16 acc[8];         /* [token block]: 32 rows x 32 tokens each */
    bf16x8 xf[2][8];         /* activation fragments of the k-step in use and of the next: [k-step & 1][token block] */
    u32x4 wa[2][4];          /* decoded weights of the tile in use and of the next: [tile & 1][k-step] */
    SbRegs cur, nxt;         /* raw codes of the super-block of the tile being decoded, and of the one after */
    float d, dmin;           /* of the super-block being decoded; d carries the factor that undoes the fp8 reading */
    uint32_t sc_lo, sc_hi, mn_lo, mn_hi; /* its 6-bit scales / mins: bytes 0..3 = sub-blocks 0..3 (lo), 4..7 (hi) */
    float s_a, s_b, m_a, m_b, dl_a, dl_b, nml_a, nml_b; /* sub-blocks 2q (a) and 2q + 1 (b) of the quarter in work */
    uint32_t cm;
    float2v cp0, cp1;
    float w0, w1, w2, w3;
    uint32_t xrd;            /* byte offset of this lane's fragment fetches in a stage: k-step 0, token block 0 */
    __amdgpu_buffer_rsrc_t w_rsrc, x_rsrc;
    uint32_t w_off[5], w_rd, x_off[8];
    int wv, kg;              /* wave of the workgroup; lane half */
    int sb, n_sb;            /* super-block of the tile in use */
    float unit;
};

QLIN_INL void unpack0(Ctx &c, const u32x4 &h) {
    c.d = half_bits_fast(h.x & 0xFFFFu) * c.unit;
    c.dmin = half_bits_fast(h.x >> 16);
}
/* the 6-bit scales and mins of a super-block from its header (get_scale_min_k4, common/ggml_dequant.h:1582-1590,
 * four fields at a time) */
QLIN_INL void unpack1(Ctx &c, const u32x4 &h) { c.sc_lo = h.y & 0x3F3F3F3Fu; c.mn_lo = h.z & 0x3F3F3F3Fu; }
QLIN_INL void unpack2(Ctx &c, const u32x4 &h) { c.sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u); }
QLIN_INL void unpack3(Ctx &c, const u32x4 &h) { c.mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u); }

/* piece PP (0..43) of the decode of quarter CQ (codes `q`, scales unpacked) into c.wa[WB] */
template <int CQ, int WB, int PP> QLIN_INL void decode_piece(Ctx &c, const u32x4 &q) {
    if constexpr (PP == 0) {
        c.s_a = ubyte_f32<2 * (CQ & 1)>(CQ & 2 ? c.sc_hi : c.sc_lo);
        c.s_b = ubyte_f32<2 * (CQ & 1) + 1>(CQ & 2 ? c.sc_hi : c.sc_lo);
    } else if constexpr (PP == 1) {
        c.m_a = ubyte_f32<2 * (CQ & 1)>(CQ & 2 ? c.mn_hi : c.mn_lo);
        c.m_b = ubyte_f32<2 * (CQ & 1) + 1>(CQ & 2 ? c.mn_hi : c.mn_lo);
    } else if constexpr (PP == 2) {
        c.dl_a = c.d * c.s_a; c.dl_b = c.d * c.s_b;
    } else if constexpr (PP == 3) {
        c.nml_a = -(c.dmin * c.m_a); c.nml_b = -(c.dmin * c.m_b);
    } else {
        constexpr int dw = (PP - 4) / 5, ph = (PP - 4) % 5; /* code word 0..3: low nibbles of q.x..q.w, 4..7: high nibbles */
        const uint32_t word = q[dw & 3];
        const float dl = dw < 4 ? c.dl_a : c.dl_b, nml = dw < 4 ? c.nml_a : c.nml_b;
        if constexpr (ph == 0) c.cm = (dw < 4 ? word : word >> 4) & 0x0F0F0F0Fu;
        else if constexpr (ph == 1) { c.cp0 = fp8_pair_lo(c.cm); c.cp1 = fp8_pair_hi(c.cm); }
        else if constexpr (ph == 2) { c.w0 = fmaf(c.cp0.x, dl, nml); c.w1 = fmaf(c.cp0.y, dl, nml); }
        else if constexpr (ph == 3) { c.w2 = fmaf(c.cp1.x, dl, nml); c.w3 = fmaf(c.cp1.y, dl, nml); }
        else if constexpr ((dw & 1) == 0) { c.wa[WB][dw >> 1].x = pack_bf16(c.w0, c.w1); c.wa[WB][dw >> 1].y = pack_bf16(c.w2, c.w3); }
        else { c.wa[WB][dw >> 1].z = pack_bf16(c.w0, c.w1); c.wa[WB][dw >> 1].w = pack_bf16(c.w2, c.w3); }
    }
}

/* request Q (0..4) of this wave for the raw blocks of super-block `sb` of its 32 rows: 64 consecutive 16-byte
 * pieces of the 32 x 9 (past the end of K: a harmless re-read) */
template <int Q> QLIN_INL void request_w(Ctx &c, int sb) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(c.w_rsrc, (lds_void *)(w4_wraw + c.wv * kWRaw + Q * 1024), 16, c.w_off[Q],
                                             min(sb, c.n_sb - 1) * 144, 0, 0);
}
/* this lane's part WHICH (0: header, 1..4: its 16 code bytes of quarter WHICH - 1) of the raw blocks in LDS */
template <int WHICH> QLIN_INL void load_sb(Ctx &c, SbRegs &r) {
    if constexpr (WHICH == 0) r.hdr = *reinterpret_cast<const u32x4 *>(w4_wraw + c.w_rd);
    else r.q[WHICH - 1] = *reinterpret_cast<const u32x4 *>(w4_wraw + c.w_rd + 16 + 32 * (WHICH - 1) + 16 * c.kg);
}

/* request I (0..7) of this wave for 64-k tile `tile` into stage ST: token rows 64 wv + 8 I .. + 7, 128 bytes each */
template <int ST, int I> QLIN_INL void request_x(Ctx &c, int tile) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(c.x_rsrc, (lds_void *)(stage_ptr<ST>() + (8 * c.wv + I) * 1024), 16,
                                             c.x_off[I], min(tile, 4 * c.n_sb - 1) * 128, 0, 0);
}

/* activation fragment of token block BJ, k-step S of stage ST */
template <int ST, int S, int BJ> QLIN_INL bf16x8 load_frag(Ctx &c) {
    return *reinterpret_cast<const bf16x8 *>(stage_ptr<ST>() + (c.xrd ^ (uint32_t)(((S & 1) << 4) | ((S >> 1) << 6))) + BJ * 4096);
}

/* slot T (0..31) of tile 4 sb + U */
template <int U, int T> QLIN_INL void slot(Ctx &c) {
    constexpr int s = T / 8, bj = T % 8;
    if constexpr (T == 24) {
        /* this wave's requests of the next tile have landed: younger are the 8 of the tile after it, 6 of the one
         * after that, and the five weight requests of the tiles with U = 1 */
        wait_vmcnt<14 + (U == 1 || U == 2 ? 5 : 0)>();
        __builtin_amdgcn_s_barrier();
    }
    c.acc[bj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, c.wa[U & 1][s]), c.xf[s & 1][bj], c.acc[bj], 0, 0, 0);
    c.xf[(s + 1) & 1][bj] = load_frag<(s == 3 ? (U + 1) & 3 : U), (s + 1) & 3, bj>(c);
    if constexpr (T % 4 == 2) request_x<(U + 3) & 3, T / 4>(c, 4 * c.sb + U + 3);
    /* U = 0: the raw blocks of the next super-block (requested three tiles ago) into registers; U = 1: request the
     * ones after it into the same place */
    if constexpr (U == 0 && T % 4 == 1 && T / 4 < 5) load_sb<T / 4>(c, c.nxt);
    if constexpr (U == 1 && T % 4 == 1 && T / 4 < 5) request_w<T / 4>(c, c.sb + 2);
    if constexpr (U == 3 && T % 8 == 4 && T / 8 < 3) c.cur.q[T / 8 + 1] = c.nxt.q[T / 8 + 1];
    /* decode of the next tile: quarter (U + 1) & 3, for U = 3 of the next super-block, whose header is unpacked first */
    constexpr int n_pieces = U == 3 ? 48 : 44;
    constexpr int p0 = (T * n_pieces + 31) / 32, p1 = ((T + 1) * n_pieces + 31) / 32; /* pieces p with p * 32 / n_pieces == T */
    auto piece = [&](auto pc) {
        constexpr int p = decltype(pc)::value;
        if constexpr (p < p1) {
            if constexpr (U == 3) {
                if constexpr (p == 0) unpack0(c, c.nxt.hdr);
                else if constexpr (p == 1) unpack1(c, c.nxt.hdr);
                else if constexpr (p == 2) unpack2(c, c.nxt.hdr);
                else if constexpr (p == 3) unpack3(c, c.nxt.hdr);
                else decode_piece<0, 0, p - 4>(c, c.nxt.q[0]);
            } else {
                decode_piece<U + 1, (U + 1) & 1, p>(c, c.cur.q[U + 1]);
            }
        }
    };
    piece(std::integral_constant<int, p0>{});
    piece(std::integral_constant<int, p0 + 1>{});
    static_assert(p1 - p0 <= 2, "at most two pieces per slot");
    __builtin_amdgcn_sched_barrier(0);
}

template <int U, int... T> QLIN_INL void run_tile(Ctx &c, std::integer_sequence<int, T...>) { (slot<U, T>(c), ...); }
template <int... P> QLIN_INL void decode_first(Ctx &c, std::integer_sequence<int, P...>) { (decode_piece<0, 0, P>(c, c.cur.q[0]), ...); }
template <int ST, int... I> QLIN_INL void request_tile(Ctx &c, int tile, std::integer_sequence<int, I...>) { (request_x<ST, I>(c, tile), ...); }

}  // namespace

__global__ void __launch_bounds__(256)
gemm_q4k_bf16_wave4_kernel(const uint8_t *__restrict__ W, const uint16_t *__restrict__ X, float *__restrict__ Y,
                           int n_rows, int n_sb, int n_tok, int ldx, int ldy, int m_tiles) {
    const int tid = threadIdx.x, lane = tid & 63;

    /* consecutive workgroup ids land on different XCDs (id % 8), each with its own L2; the token tiles
     * that share one weight tile get ids 8 apart and meet in the same L2 */
    const int xcd = blockIdx.x & 7, slot_id = blockIdx.x >> 3;
    const int tile_m = slot_id % m_tiles;
    const int tile_n = (slot_id / m_tiles) * 8 + xcd;
    if (tile_n * kBN >= n_rows) return;

    Ctx c;
    c.wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    c.n_sb = n_sb;
    c.unit = 1.0f / fp8_pair_lo(1u).x;
    const uint32_t row_bytes = (uint32_t)n_sb * 144u;
    /* Global loads are buffer loads: a descriptor of this workgroup's weight rows / token rows in scalar
     * registers, a 32-bit offset per lane that never changes, and a scalar offset that moves along K.
     * Weight role: lane (i = lane % 32, kg = lane / 32) owns row 32 wv + i and code bytes 16 kg .. 16 kg + 15 of every
     * quarter; rows past the end re-read the last one (decoded, never stored) */
    const int li = lane & 31, kg = lane >> 5;
    const int w_rows = min(kBN, n_rows - tile_n * kBN);
    c.w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(W) + (size_t)tile_n * kBN * row_bytes, 0,
                                                 w_rows * row_bytes, 0x00020000);
    c.kg = kg;
#pragma unroll
    for (int q = 0; q < 5; q++) {
        const int id = min(64 * q + lane, 32 * 9 - 1); /* piece id % 9 of row id / 9; the fifth request is half padding */
        c.w_off[q] = (uint32_t)min(32 * c.wv + id / 9, w_rows - 1) * row_bytes + 16 * (id % 9);
    }
    c.w_rd = (uint32_t)(c.wv * kWRaw + li * 144);
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
    /* fragment fetches: token li of each block of 32, chunk 4 (s >> 1) + 2 kg + (s & 1) */
    c.xrd = (uint32_t)(li * 128 + (((2 * kg) ^ fsw(li)) << 4));

#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) c.acc[i][v] = 0.0f;

    /* ---- prologue: codes of super-block 0, tiles 0..2 requested; tile 0 decoded; fragments of its k-step 0 fetched */
    c.sb = 0;
    request_w<0>(c, 0); request_w<1>(c, 0); request_w<2>(c, 0); request_w<3>(c, 0); request_w<4>(c, 0);
    request_tile<0>(c, 0, std::make_integer_sequence<int, 8>{});
    wait_vmcnt<8>();
    load_sb<0>(c, c.cur); load_sb<1>(c, c.cur); load_sb<2>(c, c.cur); load_sb<3>(c, c.cur); load_sb<4>(c, c.cur);
    __builtin_amdgcn_s_waitcnt(0xC07F); /* lgkmcnt(0): the registers hold super-block 0 before its place is requested again */
    request_w<0>(c, 1); request_w<1>(c, 1); request_w<2>(c, 1); request_w<3>(c, 1); request_w<4>(c, 1);
    request_tile<1>(c, 1, std::make_integer_sequence<int, 8>{});
    request_tile<2>(c, 2, std::make_integer_sequence<int, 8>{});
    unpack0(c, c.cur.hdr); unpack1(c, c.cur.hdr); unpack2(c, c.cur.hdr); unpack3(c, c.cur.hdr);
    decode_first(c, std::make_integer_sequence<int, 44>{});
    wait_vmcnt<21>(); /* tile 0 is in LDS as far as this wave's requests go */
    __builtin_amdgcn_s_barrier();
    c.xf[0][0] = load_frag<0, 0, 0>(c); c.xf[0][1] = load_frag<0, 0, 1>(c); c.xf[0][2] = load_frag<0, 0, 2>(c);
    c.xf[0][3] = load_frag<0, 0, 3>(c); c.xf[0][4] = load_frag<0, 0, 4>(c); c.xf[0][5] = load_frag<0, 0, 5>(c);
    c.xf[0][6] = load_frag<0, 0, 6>(c); c.xf[0][7] = load_frag<0, 0, 7>(c);

#pragma unroll 1
    for (int sb = 0; sb < n_sb; sb++) { /* one super-block of K = four tiles per pass */
        c.sb = sb;
        run_tile<0>(c, std::make_integer_sequence<int, 32>{});
        run_tile<1>(c, std::make_integer_sequence<int, 32>{});
        run_tile<2>(c, std::make_integer_sequence<int, 32>{});
        run_tile<3>(c, std::make_integer_sequence<int, 32>{});
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

hipError_t launch_gemm_q4k_bf16_wave4(const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok,
                                      int ldx, int ldy, hipStream_t stream) {
    const int n_sb = n_cols / 256;
    const int m_tiles = (n_tok + kBM - 1) / kBM;
    const int n_tiles = (n_rows + kBN - 1) / kBN;
    /* ids are dealt to 8 XCDs; pad the n-tile count to a multiple of 8 (surplus groups exit) */
    const int n_tiles_pad = (n_tiles + 7) / 8 * 8;
    hipLaunchKernelGGL(gemm_q4k_bf16_wave4_kernel, dim3(n_tiles_pad * m_tiles), dim3(256), 0, stream,
                       (const uint8_t *)W, X, Y, n_rows, n_sb, n_tok, ldx, ldy, m_tiles);
    return hipGetLastError();
}

}  // namespace qlin
