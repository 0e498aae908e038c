/*
 * gemm_kq_wave4.hip - the fused block-format x bf16 prefill GEMM (Q2_K ... Q6_K, Q8_0, IQ4_NL, IQ4_XS, Q4_0: the formats of
 * gemm_kq_formats.h) in 256-token x 128-row tiles: four waves per workgroup, one per SIMD.
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

#include "gemm_kq_formats.h"
#include "qlin_internal.h"

namespace qlin {

using namespace kq;

namespace {

constexpr int kBM = 256, kBN = 128;
constexpr int kXStage = kBM * 128; /* bytes of one stage */

/* the four stages are separate objects: a fetch from one stage then never has to wait for a request into another */
__shared__ __attribute__((aligned(1024))) uint8_t w4_stage0[kXStage];
__shared__ __attribute__((aligned(1024))) uint8_t w4_stage1[kXStage];
__shared__ __attribute__((aligned(1024))) uint8_t w4_stage2[kXStage];
__shared__ __attribute__((aligned(1024))) uint8_t w4_stage3[kXStage];


template <int ST> QLIN_INL uint8_t *stage_ptr() {
    if constexpr (ST == 0) return w4_stage0;
    else if constexpr (ST == 1) return w4_stage1;
    else if constexpr (ST == 2) return w4_stage2;
    else return w4_stage3;
}

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
    if constexpr (U == 0 && T % 3 == 1 && T / 3 < F::kLaneVec) c.nxt[T / 3] = load_raw<F, T / 3>(c);
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
    piece(std::integral_constant<int, p0 + 2>{});
    static_assert(p1 - p0 <= 3, "at most three pieces per slot");
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
gemm_kq_bf16_wave4_kernel(TileSet set, const uint16_t *__restrict__ X, int n_sb, int n_tok, int ldx, int m_tiles) {
    /* raw blocks of one super-block of each wave's 32 weight rows (32 x kPieces pieces, rounded up to whole requests) */
    __shared__ __attribute__((aligned(1024))) uint8_t w4_raw[4 * F::kReq * 1024];
    const int tid = threadIdx.x, lane = tid & 63;

    /* consecutive workgroup ids land on different XCDs (id % 8), each with its own L2; the token tiles
     * that share one weight tile get ids 8 apart and meet in the same L2 */
    const int xcd = blockIdx.x & 7, slot_id = blockIdx.x >> 3;
    const int tile_m = slot_id % m_tiles;
    const int tile_all = (slot_id / m_tiles) * 8 + xcd;
    if (tile_all >= set.end2) return;
    const TileOf t = tile_of(set, tile_all);
    const uint8_t *W = t.W;
    float *Y = t.Y;
    const int n_rows = t.n_rows, ldy = t.ldy, tile_n = t.tile;

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
hipError_t launch_wave4(int n_mat, const void *const *W, const uint16_t *X, float *const *Y, const int *n_rows, int n_cols,
                        int n_tok, int ldx, const int *ldy, hipStream_t stream) {
    const int n_sb = n_cols / 256;
    const int m_tiles = (n_tok + kBM - 1) / kBM;
    TileSet set;
    const int n_tiles = fill_tile_set(set, n_mat, W, Y, n_rows, ldy, kBN);
    /* ids are dealt to 8 XCDs; pad the n-tile count to a multiple of 8 (surplus groups exit) */
    const int n_tiles_pad = (n_tiles + 7) / 8 * 8;
    hipLaunchKernelGGL(gemm_kq_bf16_wave4_kernel<F>, dim3(n_tiles_pad * m_tiles), dim3(256), 0, stream, set, X, n_sb,
                       n_tok, ldx, m_tiles);
    return hipGetLastError();
}
template <class F>
hipError_t launch_wave4(const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok, int ldx, int ldy,
                        hipStream_t stream) {
    return launch_wave4<F>(1, &W, X, &Y, &n_rows, n_cols, n_tok, ldx, &ldy, stream);
}
}  // namespace

bool gemm_kq_wave4_covers(uint32_t type) {
    return type == T_Q4_K || type == T_Q5_K || type == T_Q6_K || type == T_Q8_0 || type == T_IQ4_NL || type == T_IQ4_XS ||
           type == T_Q4_0 || type == T_Q2_K || type == T_Q3_K;
}

/* Which kernel takes a prefill GEMM of a format with a fused kernel, beyond the token counts of the few-token kernels.
 * 200 or more 256-token x 128-row tiles fill the chip: the large-tile kernel - up to a token count, because it decodes
 * the weights again every 256 tokens, which costs more the more there is to decode, while decoding once into a workspace
 * costs 27 - 38 us whatever the token count (14336 x 4096, large tiles against decode + the vendor library's product, us:
 * at 512 tokens Q4_K 61 / 86, Q5_K 62 / 92, Q6_K 66 / 84, Q8_0 71 / 83, IQ4_NL 62 / 95, IQ4_XS 68 / 99, Q4_0 62 / 81,
 * Q2_K 59 / 82, Q3_K 62 / 91; at 1024 118 / 125, 121 / 135, 131 / 126, 139 / 121, 123 / 132, 133 / 139, 122 / 120,
 * 117 / 120, 127 / 128; at 1536 Q4_K 181 / 190, Q5_K 185 / 195, Q6_K 206 / 184, Q8_0 216 / 177; at 2048 267 / 244,
 * 262 / 260, 273 / 240, 311 / 224, 279 / 254, 305 / 270, 272 / 241, 251 / 222, 261 / 253).
 * Fewer large tiles: the small-tile kernel, up to a token count per format (small tiles / decode + library, us, at
 * 4096 x 4096 and 4096 x 14336 with 512 tokens, the same two with 1024, 6144 x 4096 with 768, 14336 x 4096 with 256:
 * Q4_K 24 / 43, 72 / 97, 42 / 52, 133 / 153, 57 / 59, 39 / 75; Q5_K 25 / 44, 74 / 104, 43 / 54, 139 / 158, 59 / 61, 41 / 80;
 * Q6_K 29 / 40, 85 / 96, 49 / 51, 163 / 154, 68 / 57, 47 / 71; Q8_0 35 / 38, 109 / 97, 64 / 49, 216 / 152, 91 / 55, 62 / 75;
 * IQ4_NL 27 / 45, 80 / 108, 46 / 55, 148 / 161, 63 / 63, 44 / 88; IQ4_XS 27 / 45, 82 / 110, 47 / 55, 154 / 162, 64 / 63,
 * 45 / 80; Q4_0 24 / 41, 72 / 91, 41 / 50, 133 / 144, 57 / 56, 39 / 72; Q2_K 24 / 42, 70 / 94, 41 / 52, 132 / 149, 55 / 58,
 * 38 / 74; Q3_K 26 / 45, 75 / 102, 44 / 54, 144 / 160, 61 / 61, 42 / 82).
 * Without a workspace there is no decode + dense route to prefer. */
FusedTile choose_fused_tile(uint32_t type, int n_rows, int n_cols, int n_tok, int ldx, bool have_workspace) {
    if (!gemm_kq_wave4_covers(type) || n_cols % 256 != 0 || ldx >= (1 << 22)) return kFusedNone;
    const long long large_tiles = (long long)((n_rows + 127) / 128) * ((n_tok + 255) / 256);
    /* token counts up to which the large-tile and the small-tile kernel measured faster than decode + dense */
    int large_max = 512, small_max = 256; /* Q8_0 */
    switch (type) {
    case T_Q4_K: case T_Q5_K: large_max = 1536; small_max = INT_MAX; break;
    case T_Q4_0: case T_Q2_K: case T_Q3_K: large_max = 1024; small_max = INT_MAX; break;
    case T_IQ4_NL: large_max = 1536; small_max = 1024; break;
    case T_IQ4_XS: large_max = 1024; small_max = 1024; break;
    case T_Q6_K: small_max = 512; break;
    default: break;
    }
    if (large_tiles >= 200) return (n_tok <= large_max || !have_workspace) ? kFusedLarge : kFusedNone;
    return (n_tok <= small_max || !have_workspace) ? kFusedSmall : kFusedNone;
}

hipError_t launch_fused_tile(FusedTile tile, uint32_t type, const void *W, const uint16_t *X, float *Y, int n_rows,
                             int n_cols, int n_tok, int ldx, int ldy, hipStream_t stream) {
    if (tile == kFusedLarge) return launch_gemm_kq_bf16_wave4(type, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    if (tile == kFusedSmall) return launch_gemm_kq_bf16_wave4s(type, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    return hipErrorInvalidValue;
}

hipError_t launch_gemm_kq_bf16_wave4_multi(uint32_t type, int n_mat, const void *const *W, const uint16_t *X,
                                           float *const *Y, const int *n_rows, int n_cols, int n_tok, int ldx,
                                           const int *ldy, hipStream_t stream) {
    if (n_mat < 1 || n_mat > 3) return hipErrorInvalidValue;
    switch (type) {
    case T_Q4_K: return launch_wave4<FQ4K>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q5_K: return launch_wave4<FQ5K>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q6_K: return launch_wave4<FQ6K>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q8_0: return launch_wave4<FQ8_0>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_IQ4_NL: return launch_wave4<FIQ4NL>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_IQ4_XS: return launch_wave4<FIQ4XS>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q4_0: return launch_wave4<FQ4_0>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q2_K: return launch_wave4<FQ2K>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q3_K: return launch_wave4<FQ3K>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_gemm_kq_bf16_wave4(uint32_t type, const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols,
                                     int n_tok, int ldx, int ldy, hipStream_t stream) {
    return launch_gemm_kq_bf16_wave4_multi(type, 1, &W, X, &Y, &n_rows, n_cols, n_tok, ldx, &ldy, stream);
}

hipError_t launch_gemm_q4k_bf16_wave4(const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok,
                                      int ldx, int ldy, hipStream_t stream) {
    return launch_wave4<FQ4K>(W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
}

}  // namespace qlin
