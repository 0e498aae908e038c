/*
 * gemm_kq_wave4s.hip - the fused block-format x bf16 prefill GEMM (the formats of gemm_kq_formats.h) in 128-token x 64-row
 * tiles, for the shapes whose 256-token x 128-row tiles (gemm_kq_wave4.hip) would leave most of the chip idle: 4096-row projections
 * at 512 tokens (64 large tiles, 256 small ones), 14336 rows at 129..256 tokens.
 *
 *   Y[t*ldy + r] = sum_k X[t*ldx + k] * decode(W)[r][k]      X bf16, Y fp32, fp32 accumulate
 *
 * Same contraction, same decode and the same single rounding of the weights to bf16 as the large-tile kernel (the
 * format descriptions are shared, gemm_kq_formats.h); what the reference does per tile in
 * rdna4/dequant/bench_dequant.c:359-459.
 *
 * Four waves as 2 row halves x 2 halves of K: wave (wr, wk) owns rows 32 wr .. + 31 and all 128 tokens of the tile
 * (four 32 x 32 accumulators) and, of every 64-k tile, the k-steps 2 wk and 2 wk + 1 - the 32 elements of one
 * sub-block of the K-quants. It decodes only those: every weight is decoded once per workgroup, about 6 vector
 * instructions beside every matrix instruction (with the waves split over the tokens instead, both waves of a row
 * half decoded the same weights, 12 beside every matrix instruction, and the vector ALU bound the kernel). The two
 * waves of a row half share one raw-block image in LDS, each requesting every other KB of it; their partial sums meet
 * in LDS at the end (wave wk adds and stores the token blocks 2 wk and 2 wk + 1). 64 KB of activation stages and
 * 10-16 KB of raw blocks per workgroup: two workgroups per compute unit, whose waves fill each other's gaps.
 *
 * One tile = 8 slots of [matrix instruction, fragment fetch for the wave's next k-step, side work]: slots 0..3 are
 * the wave's first k-step over the four token blocks, 4..7 its second. Side work: the load-to-LDS requests of the
 * tile three ahead (4 per wave and tile), in the first tile of a super-block the raw data of the next super-block
 * out of the shared image into registers, in the second the requests that refill the image (after the barrier of
 * the first tile: every wave has read it), in the fourth the move of those registers into the ones in work; and
 * the wave's share of the decode of the next tile. Before the second k-step (whose slots fetch fragments of the
 * next tile): wait for this wave's requests of the next tile, barrier.
 */
#include <utility>

#include "gemm_kq_formats.h"
#include "qlin_internal.h"

namespace qlin {

using namespace kq;

namespace {

constexpr int kBM = 128, kBN = 64;
constexpr int kXStage = kBM * 128; /* bytes of one stage: 128 tokens x 64 k */

__shared__ __attribute__((aligned(1024))) uint8_t w4s_stage0[kXStage];
__shared__ __attribute__((aligned(1024))) uint8_t w4s_stage1[kXStage];
__shared__ __attribute__((aligned(1024))) uint8_t w4s_stage2[kXStage];
__shared__ __attribute__((aligned(1024))) uint8_t w4s_stage3[kXStage];

template <int ST> QLIN_INL uint8_t *stage_ptr() {
    if constexpr (ST == 0) return w4s_stage0;
    else if constexpr (ST == 1) return w4s_stage1;
    else if constexpr (ST == 2) return w4s_stage2;
    else return w4s_stage3;
}

template <class F> struct Ctx {
    static constexpr int kMyReq = (F::kReq + 1) / 2; /* weight requests of one wave per super-block */
    floatx16 acc[4];         /* [token block]: 32 rows x 32 tokens each, over the wave's half of K */
    bf16x8 xf[2][4];         /* activation fragments: [the wave's k-step 0 / 1][token block] */
    u32x4 wa[2][4];          /* decoded weights of the tile in use and of the next: [tile & 1][k-step] */
    u32x4 cur[F::kLaneVec + F::kExtraVec], nxt[F::kLaneVec + F::kExtraVec];
    typename F::Scales sc;
    Temps t;
    uint32_t xrd;
    __amdgpu_buffer_rsrc_t w_rsrc, x_rsrc;
    uint32_t w_off[kMyReq], w_dst[kMyReq], w_rd, w_swz, w_own, x_off[4];
    uint8_t *raw;            /* the workgroup's two raw-block images */
    int wv, kg;
    int sb, n_sb;
    float unit;
};

template <class F, int Q> QLIN_INL void request_w(Ctx<F> &c, int sb) {
    dma16(c.w_rsrc, c.raw + c.w_dst[Q], c.w_off[Q], min(sb, c.n_sb - 1) * F::kBlockBytes);
}
template <class F, int J> QLIN_INL u32x4 load_raw(Ctx<F> &c) {
    constexpr VecAt at = F::vec_at(J);
    return *reinterpret_cast<const u32x4 *>(c.raw + c.w_rd + ((uint32_t)(at.off + at.by_half * c.kg) ^ c.w_swz));
}
/* request I (0..3) of this wave for 64-k tile `tile` into stage ST: token rows 32 wv + 8 I .. + 7, 128 bytes each */
template <class F, int ST, int I> QLIN_INL void request_x(Ctx<F> &c, int tile) {
    dma16(c.x_rsrc, stage_ptr<ST>() + (4 * c.wv + I) * 1024, c.x_off[I], min(tile, 4 * c.n_sb - 1) * 128);
}
template <class F, int ST, int S, int BJ> QLIN_INL bf16x8 load_frag(Ctx<F> &c) {
    return *reinterpret_cast<const bf16x8 *>(stage_ptr<ST>() + (c.xrd ^ (uint32_t)F::frag_xor(S)) + BJ * 4096);
}

/* owned pieces I0 + I of a slot, as far as they are below I1 */
template <class F, int WK, int U, int I0, int I1, int... I> QLIN_INL void pieces(Ctx<F> &c, std::integer_sequence<int, I...>) {
    constexpr int n_prep = U == 3 ? F::kPrepPieces : 0;
    auto piece = [&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (i < I1) {
            constexpr int p = Owned<F, WK, n_prep>::nth(i);
            static_assert(p >= 0, "piece index past the wave's list");
            if constexpr (U == 3) {
                if constexpr (p < n_prep) F::template prep<p>(c, c.nxt);
                else F::template tile_piece<0, 0, p - n_prep>(c, c.nxt);
            } else {
                F::template tile_piece<U + 1, (U + 1) & 1, p>(c, c.cur);
            }
        }
    };
    (piece(std::integral_constant<int, I0 + I>{}), ...);
}

/* slot T (0..7) of tile 4 sb + U for wave half WK: its k-step T / 4 (k-step 2 WK + T / 4 of the tile), token block T % 4 */
template <class F, int WK, int U, int T> QLIN_INL void slot(Ctx<F> &c) {
    constexpr int sl = T / 4, s = 2 * WK + sl, bj = T % 4, nW = Ctx<F>::kMyReq, nE = F::kExtraLoads, nV = F::kLaneVec + F::kExtraVec;
    static_assert(nE <= 4 && nW <= 4 && F::kLaneVec <= 12 && nV <= 10, "side work is laid out over the first slots of a tile");
    if constexpr (T == 4) {
        /* this wave's requests of the next tile have landed: younger are the 4 of the tile after it, 2 of the one
         * after that, the weight requests of a tile with U = 1 and the scale loads of one with U = 0 */
        wait_vmcnt<6 + (U == 0 ? nE : 0) + (U == 1 ? nW + nE : 0) + (U == 2 ? nW : 0)>();
        /* U = 0: this wave's reads of the raw image are done before anybody refills it */
        if constexpr (U == 0) __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_s_barrier();
    }
    c.acc[bj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, c.wa[U & 1][s]), c.xf[sl][bj], c.acc[bj], 0, 0, 0);
    c.xf[sl ^ 1][bj] = load_frag<F, (sl == 1 ? (U + 1) & 3 : U), 2 * WK + (sl ^ 1), bj>(c);
    if constexpr (T % 2 == 1) request_x<F, (U + 3) & 3, T / 2>(c, 4 * c.sb + U + 3);
    if constexpr (U == 0 && T < 4) { /* all before the barrier of this tile */
        if constexpr (3 * T < F::kLaneVec) c.nxt[3 * T] = load_raw<F, 3 * T>(c);
        if constexpr (3 * T + 1 < F::kLaneVec) c.nxt[3 * T + 1] = load_raw<F, 3 * T + 1>(c);
        if constexpr (3 * T + 2 < F::kLaneVec) c.nxt[3 * T + 2] = load_raw<F, 3 * T + 2>(c);
        if constexpr (T < nE) F::template extra_load<T>(c, c.nxt, min(c.sb + 1, c.n_sb - 1));
    }
    if constexpr (U == 1 && T < nW) request_w<F, T>(c, c.sb + 2);
    if constexpr (U == 3 && T < 5) {
        if constexpr (2 * T < nV) c.cur[2 * T] = c.nxt[2 * T];
        if constexpr (2 * T + 1 < nV) c.cur[2 * T + 1] = c.nxt[2 * T + 1];
    }
    constexpr int n_own = Owned<F, WK, (U == 3 ? F::kPrepPieces : 0)>::count();
    constexpr int i0 = (T * n_own + 7) / 8, i1 = ((T + 1) * n_own + 7) / 8; /* owned pieces i with i * 8 / n_own == T */
    static_assert(i1 - i0 <= 8, "at most eight pieces per slot");
    pieces<F, WK, U, i0, i1>(c, std::make_integer_sequence<int, 8>{});
    __builtin_amdgcn_sched_barrier(0);
}

template <class F, int WK, int U, int... T> QLIN_INL void run_tile(Ctx<F> &c, std::integer_sequence<int, T...>) { (slot<F, WK, U, T>(c), ...); }
template <class F, int... P> QLIN_INL void prep_first(Ctx<F> &c, std::integer_sequence<int, P...>) { (F::template prep<P>(c, c.cur), ...); }
template <class F, int... P> QLIN_INL void decode_first(Ctx<F> &c, std::integer_sequence<int, P...>) { (F::template tile_piece<0, 0, P>(c, c.cur), ...); }
template <class F, int ST, int... I> QLIN_INL void request_tile(Ctx<F> &c, int tile, std::integer_sequence<int, I...>) { (request_x<F, ST, I>(c, tile), ...); }
template <class F, int... Q> QLIN_INL void request_raw(Ctx<F> &c, int sb, std::integer_sequence<int, Q...>) { (request_w<F, Q>(c, sb), ...); }
template <class F, int... J> QLIN_INL void load_cur(Ctx<F> &c, std::integer_sequence<int, J...>) { ((c.cur[J] = load_raw<F, J>(c)), ...); }
template <class F, int... J> QLIN_INL void load_cur_extra(Ctx<F> &c, std::integer_sequence<int, J...>) { (F::template extra_load<J>(c, c.cur, 0), ...); }

QLIN_INL uint8_t *stage_of(int i) { return i == 0 ? w4s_stage0 : i == 1 ? w4s_stage1 : i == 2 ? w4s_stage2 : w4s_stage3; }

/* main loop and result of a wave of K half WK; on entry tile 0 is decoded and in LDS */
template <class F, int WK>
QLIN_INL void run_half(Ctx<F> &c, float *__restrict__ Y, int n_rows, int n_tok, int ldy, int tile_m, int tile_n, int wr,
                       int li, int lane) {
    c.xf[0][0] = load_frag<F, 0, 2 * WK, 0>(c);
    c.xf[0][1] = load_frag<F, 0, 2 * WK, 1>(c);
    c.xf[0][2] = load_frag<F, 0, 2 * WK, 2>(c);
    c.xf[0][3] = load_frag<F, 0, 2 * WK, 3>(c);

#pragma unroll 1
    for (int sb = 0; sb < c.n_sb; sb++) { /* one super-block of K = four tiles per pass */
        c.sb = sb;
        run_tile<F, WK, 0>(c, std::make_integer_sequence<int, 8>{});
        run_tile<F, WK, 1>(c, std::make_integer_sequence<int, 8>{});
        run_tile<F, WK, 2>(c, std::make_integer_sequence<int, 8>{});
        run_tile<F, WK, 3>(c, std::make_integer_sequence<int, 8>{});
    }
    /* requests past the end of K are still on their way into LDS, and fragment fetches of the tile past the end may
     * be too: both have to be over in every wave before the stages are used for the exchange below */
    wait_vmcnt<0>();
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();

    /* The two K halves of a row half add up: wave WK hands the partner the two token blocks the partner stores
     * (2 (1 - WK) + b, b = 0, 1: 8 KB at the start of the stage with the wave's number) and adds the partner's share
     * to its own two. Both waves hold element (row, token) of a block in the same register of the same lane. */
    floatx4 *mine = reinterpret_cast<floatx4 *>(stage_of(c.wv));
    const floatx4 *theirs = reinterpret_cast<const floatx4 *>(stage_of(c.wv ^ 2));
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const floatx16 &a = c.acc[2 * (1 - WK) + b];
            mine[(b * 4 + g) * 64 + lane] = floatx4{a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
        }
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();

    /* C layout of the 32x32 MFMA: register v of lane l holds row 8 (v / 4) + 4 (l / 32) + v % 4 (a weight row), column
     * l % 32 (a token): four runs of four consecutive floats of one token's output row per lane */
    const bool vec_ok = (ldy & 3) == 0 && (reinterpret_cast<uintptr_t>(Y) & 15) == 0;
    const int kg = lane >> 5;
#pragma unroll
    for (int b = 0; b < 2; b++) {
        const int bj = 2 * WK + b;
        const int m = tile_m * kBM + 32 * bj + li;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int n = tile_n * kBN + 32 * wr + 8 * g + 4 * kg;
            const floatx4 other = theirs[(b * 4 + g) * 64 + lane];
            /* the sum over the first half of K plus the sum over the second */
            floatx4 a = {c.acc[bj][4 * g], c.acc[bj][4 * g + 1], c.acc[bj][4 * g + 2], c.acc[bj][4 * g + 3]};
            a = WK == 0 ? a + other : other + a;
            if (m >= n_tok) continue;
            float *y = Y + (size_t)m * ldy + n;
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

}  // namespace

template <class F>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
gemm_kq_bf16_wave4s_kernel(TileSet set, const uint16_t *__restrict__ X, int n_sb, int n_tok, int ldx, int m_tiles) {
    /* raw blocks of one super-block of the two row halves (32 x kPieces pieces each, rounded up to whole requests) */
    __shared__ __attribute__((aligned(1024))) uint8_t w4s_raw[2 * F::kReq * 1024];
    constexpr int nW = Ctx<F>::kMyReq;
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
    c.raw = w4s_raw;
    c.wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = c.wv & 1, wk = c.wv >> 1;
    c.n_sb = n_sb;
    c.unit = 1.0f / fp8_pair_lo(1u).x;
    const uint32_t row_bytes = (uint32_t)n_sb * F::kBlockBytes;
    const int li = lane & 31, kg = lane >> 5;
    c.kg = kg;
    /* weights: lane (li, kg) owns row 32 wr + li of the tile; rows past the end re-read the last one (decoded, never
     * stored). Request Q of a row half fills pieces 64 Q .. 64 Q + 63 of its 32 x kPieces; the wave with K half wk
     * issues Q = wk, wk + 2, ... (one past the last: the last again, into the same place) */
    const int w_rows = min(kBN, n_rows - tile_n * kBN);
    c.w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(W) + (size_t)tile_n * kBN * row_bytes, 0,
                                                 w_rows * row_bytes, 0x00020000);
#pragma unroll
    for (int q = 0; q < nW; q++) {
        const int Q = min(2 * q + wk, F::kReq - 1);
        const int id = min(64 * Q + lane, 32 * F::kPieces - 1); /* past the last piece: padding */
        const int part = F::kSwizzle ? (id % F::kPieces) ^ ((id / F::kPieces) & 15) : id % F::kPieces;
        c.w_off[q] = (uint32_t)min(32 * wr + id / F::kPieces, w_rows - 1) * row_bytes + F::piece_src(part);
        c.w_dst[q] = (uint32_t)((wr * F::kReq + Q) * 1024);
    }
    c.w_rd = (uint32_t)(wr * F::kReq * 1024 + li * F::kPieces * 16);
    c.w_swz = F::kSwizzle ? (uint32_t)(li & 15) << 4 : 0u;
    c.w_own = (uint32_t)min(32 * wr + li, w_rows - 1) * row_bytes;
    /* activations: request I of this wave fills 1 KB of a stage, lane l the 16 bytes at chunk position l % 8 of token
     * row 32 wv + 8 I + l / 8, i.e. chunk (l % 8) ^ f(row) of that token's 128 bytes; tokens past the end re-read the
     * last one (never stored) */
    const int x_rows = min(kBM, n_tok - tile_m * kBM);
    c.x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(X) + (size_t)tile_m * kBM * ldx, 0,
                                                 ((x_rows - 1) * ldx + n_sb * 256) * 2, 0x00020000);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int row = 32 * c.wv + 8 * i + (lane >> 3);
        c.x_off[i] = (uint32_t)min(row, x_rows - 1) * (uint32_t)(2 * ldx) + (uint32_t)((((lane & 7) ^ fsw(row))) << 4);
    }
    /* fragment fetches: token li of each block of 32 */
    c.xrd = (uint32_t)(li * 128 + (((F::kKgChunk * kg) ^ fsw(li)) << 4));

#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) c.acc[i][v] = 0.0f;

    /* ---- prologue: raw blocks of super-block 0 fetched and read back by both waves of a row half, those of
     * super-block 1 and tiles 0..2 requested; tile 0 decoded; fragments of its k-step 0 fetched */
    c.sb = 0;
    load_cur_extra<F>(c, std::make_integer_sequence<int, F::kExtraLoads>{});
    request_raw<F>(c, 0, std::make_integer_sequence<int, nW>{});
    request_tile<F, 0>(c, 0, std::make_integer_sequence<int, 4>{});
    wait_vmcnt<4>();
    __builtin_amdgcn_s_barrier(); /* both shares of the image are in */
    load_cur<F>(c, std::make_integer_sequence<int, F::kLaneVec>{});
    __builtin_amdgcn_s_waitcnt(0xC07F); /* lgkmcnt(0): the registers hold super-block 0 ... */
    __builtin_amdgcn_s_barrier();       /* ... in every wave, before its place is requested again */
    request_raw<F>(c, 1, std::make_integer_sequence<int, nW>{});
    request_tile<F, 1>(c, 1, std::make_integer_sequence<int, 4>{});
    request_tile<F, 2>(c, 2, std::make_integer_sequence<int, 4>{});
    prep_first<F>(c, std::make_integer_sequence<int, F::kPrepPieces>{});
    decode_first<F>(c, std::make_integer_sequence<int, F::kTilePieces>{});
    wait_vmcnt<8>(); /* tile 0 and the raw blocks of super-block 1 are in LDS as far as this wave's requests go */
    __builtin_amdgcn_s_barrier();
    /* from here on the two K halves run their own instruction streams (what a wave decodes and which fragments it
     * fetches is fixed at compile time); they meet at the same barriers */
    if (wk == 0) run_half<F, 0>(c, Y, n_rows, n_tok, ldy, tile_m, tile_n, wr, li, lane);
    else run_half<F, 1>(c, Y, n_rows, n_tok, ldy, tile_m, tile_n, wr, li, lane);
}

namespace {
template <class F>
hipError_t launch_wave4s(int n_mat, const void *const *W, const uint16_t *X, float *const *Y, const int *n_rows, int n_cols,
                         int n_tok, int ldx, const int *ldy, hipStream_t stream) {
    const int n_sb = n_cols / 256;
    const int m_tiles = (n_tok + kBM - 1) / kBM;
    TileSet set;
    const int n_tiles = fill_tile_set(set, n_mat, W, Y, n_rows, ldy, kBN);
    const int n_tiles_pad = (n_tiles + 7) / 8 * 8; /* ids are dealt to 8 XCDs; surplus groups exit */
    hipLaunchKernelGGL(gemm_kq_bf16_wave4s_kernel<F>, dim3(n_tiles_pad * m_tiles), dim3(256), 0, stream, set, X, n_sb,
                       n_tok, ldx, m_tiles);
    return hipGetLastError();
}
}  // namespace

hipError_t launch_gemm_kq_bf16_wave4s_multi(uint32_t type, int n_mat, const void *const *W, const uint16_t *X,
                                            float *const *Y, const int *n_rows, int n_cols, int n_tok, int ldx,
                                            const int *ldy, hipStream_t stream) {
    if (n_mat < 1 || n_mat > 3) return hipErrorInvalidValue;
    switch (type) {
    case T_Q4_K: return launch_wave4s<FQ4K>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q5_K: return launch_wave4s<FQ5K>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q6_K: return launch_wave4s<FQ6K>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q8_0: return launch_wave4s<FQ8_0>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_IQ4_NL: return launch_wave4s<FIQ4NL>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_IQ4_XS: return launch_wave4s<FIQ4XS>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q4_0: return launch_wave4s<FQ4_0>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q2_K: return launch_wave4s<FQ2K>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    case T_Q3_K: return launch_wave4s<FQ3K>(n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_gemm_kq_bf16_wave4s(uint32_t type, const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols,
                                      int n_tok, int ldx, int ldy, hipStream_t stream) {
    return launch_gemm_kq_bf16_wave4s_multi(type, 1, &W, X, &Y, &n_rows, n_cols, n_tok, ldx, &ldy, stream);
}

}  // namespace qlin
