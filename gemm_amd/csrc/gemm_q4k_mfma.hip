/*
 * gemm_q4k_mfma.hip - prefill GEMM with Q4_K weights on the gfx950 matrix cores.
 *
 *   Y[t*ldy + r] = sum_k X[t*ldx + k] * decode(W)[r][k]      X bf16, Y fp32, fp32 accumulate
 *
 * The contraction tf_gemm_f16_mt_tokenmajor computes for a Q4_K tensor (common/transformer.h:4487,
 * generic branch :4535-4572: decode a row, dot it with every token), restated as a tiled GEMM:
 * weights are decoded exactly as dequantize_row_q4_K does (common/ggml_dequant.h:1592-1618,
 * y = (d*sc)*q - dmin*m in fp32), rounded ONCE to bf16 (nearest even) and fed to
 * v_mfma_f32_32x32x16_bf16 against the bf16 activations. Rounding the weights to bf16 costs
 * about 1.7e-3 relative L2 against an exact-weight reference (budget 2e-3); truncation would
 * not fit.
 *
 * Tiling. A workgroup (512 threads) owns BM = 256 tokens x BN = 128 weight rows and walks K in
 * tiles of 64 = one pair of Q4_K sub-blocks (the low and high nibbles of 32 quant bytes). Its 8
 * waves form a 4 x 2 grid of 64x64 sub-tiles (2x2 MFMA tiles of 32x32, 64 accumulator
 * registers). Per tile every thread decodes 16 weights (8 nibble bytes of one row) to bf16 and
 * copies 4 x 16 bytes of activations into an LDS ring of three stages; the MFMA operands of a
 * tile are fetched from LDS half a tile ahead of the MFMAs that use them, the decode of tile
 * i+2 is issued in the shadow of the MFMAs of tile i, and global loads run four tiles ahead
 * (two register sets). One barrier per tile. The loop is unrolled by the four tiles of a
 * super-block: d, dmin and the packed scales of the thread's row are unpacked once per super-block.
 * When 128-row tiles would leave compute units
 * without a workgroup (few tokens, or few rows) the same kernel runs with BN = 64: 4 x 2 waves
 * of 64 tokens x 32 rows, eight 4-byte weight parts per row. When even those
 * tiles number 128 or fewer (4096 rows at 512 tokens), K is cut in two halves that add their results to
 * a zeroed Y (4096 x 14336 at 512 tokens: 166 -> 108 us; two addends onto zero commute, so the result
 * does not depend on which half arrives first). Up to 128 tokens the tile is 128 tokens x 64 rows on four waves
 * (2 x 2 of 64 x 32, four 8-byte weight parts per row), two workgroups to a compute unit, K cut in two while the
 * tiles number a chip's worth or fewer (M = 128 at 14336 x 4096: 51.7 -> 39.5 us).
 *
 * Measured on MI355X at M=512, N=14336, K=4096: 76-77 us, 0.79 PFLOP/s on 224 of 256 compute
 * units. Cycle stamps (s_memtime) around the parts of one tile show a tile of about 1920 cycles
 * at a shader clock of 1.75-1.9 GHz under this load (2.0-2.1 GHz in a light kernel), against
 * 1024 cycles of matrix-pipe work per SIMD: the eight operand fetches that follow the barrier
 * take 350-450 cycles to issue for the first wave of each SIMD and 650-750 for the second
 * (about 45 cycles per ds_read_b128 and SIMD, twice what the same access pattern costs in a loop
 * of nothing but reads), the second wave stays that far behind through the tile, and the first
 * wave waits 600-700 cycles at the barrier. Matrix pipe, vector ALU and LDS are each busy about
 * half of the time (SQ counters). Orders that were measured and were not faster: MFMAs ahead of
 * the fetches, one fetch per MFMA, four MFMAs then the fetches then the rest.
 *
 * Both MFMA operands are read from LDS with the same [row][k] indexing, so the result does
 * not depend on which k a given lane/element position feeds inside the instruction.
 */
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef float float2v __attribute__((ext_vector_type(2)));

constexpr int kBK = 64;         /* k per step */
constexpr int kRow = 136;       /* average bytes per LDS tile row: pairs of 128-byte rows + 16 bytes */
constexpr int kStages = 3;      /* LDS ring depth */

/* byte offset of 16-byte chunk `chunk` (0..7) of tile row `row`: rows are stored in pairs of
 * 2 x 128 bytes followed by 16 bytes of padding. With 64 banks of 4 bytes, the 16-byte slot of
 * (row, chunk) is ((row>>1) + 8*(row&1) + chunk) mod 16, so the 16 rows that one LDS cycle
 * serves for an MFMA operand fetch (16 lanes x 16 bytes, consecutive rows, same chunk) use 16
 * distinct slots, and a row written as 8 consecutive chunks stays clear of its pair row.
 * (Padding every row to 144 bytes would do the same but three ring stages would not fit.) */
__device__ __forceinline__ int swz(int row, int chunk) { return (row >> 1) * 272 + (row & 1) * 128 + (chunk << 4); }

struct StepRegs {
    uint4 x[4];   /* 4 x 8 bf16 of activations */
    uint4 hdr;    /* d, dmin, 12 packed scale bytes of this thread's weight row / super-block */
    uint2 qs;     /* 8 nibble bytes */
};

/* two bytes 0x0q read as E4M3 are q times one fixed power of two (subnormal and first normal
 * binade form one linear ramp over q = 0..15) */
__device__ __forceinline__ float2v fp8_pair_lo(uint32_t v) { return __builtin_amdgcn_cvt_pk_f32_fp8((int)v, false); }
__device__ __forceinline__ float2v fp8_pair_hi(uint32_t v) { return __builtin_amdgcn_cvt_pk_f32_fp8((int)v, true); }

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
    bf16x2 r;
    r[0] = (__bf16)a; /* round to nearest even */
    r[1] = (__bf16)b;
    return __builtin_bit_cast(uint32_t, r);
}

/* 8 nibbles of one dword pair position -> 8 decoded weights (dl*q - ml), as 4 bf16 pairs */
__device__ __forceinline__ uint4 decode8(uint32_t n0, uint32_t n1, float dl, float ml) {
    const float2v a = fp8_pair_lo(n0), b = fp8_pair_hi(n0), c = fp8_pair_lo(n1), d = fp8_pair_hi(n1);
    uint4 r;
    r.x = pack_bf16(fmaf(a.x, dl, -ml), fmaf(a.y, dl, -ml));
    r.y = pack_bf16(fmaf(b.x, dl, -ml), fmaf(b.y, dl, -ml));
    r.z = pack_bf16(fmaf(c.x, dl, -ml), fmaf(c.y, dl, -ml));
    r.w = pack_bf16(fmaf(d.x, dl, -ml), fmaf(d.y, dl, -ml));
    return r;
}

/* 4 nibbles of one dword -> 4 decoded weights as 2 bf16 pairs */
__device__ __forceinline__ uint2 decode4(uint32_t n0, float dl, float ml) {
    const float2v a = fp8_pair_lo(n0), b = fp8_pair_hi(n0);
    return make_uint2(pack_bf16(fmaf(a.x, dl, -ml), fmaf(a.y, dl, -ml)), pack_bf16(fmaf(b.x, dl, -ml), fmaf(b.y, dl, -ml)));
}

}  // namespace

/* NB = 2: 128 weight rows per workgroup (wave tile 64 tokens x 64 rows); NB = 1: 64 weight rows (wave
 * tile 64 x 32) and twice as many workgroups, for shapes whose grid would not fill the chip. WM = 4: 256 tokens
 * per workgroup, eight waves; WM = 2: 128 tokens, four waves (with NB = 1 only) */
template <int WM, int NB>
__global__ void __launch_bounds__(128 * WM)
gemm_q4k_bf16_kernel(const uint8_t *__restrict__ W, const uint16_t *__restrict__ X, float *__restrict__ Y,
                     int n_rows, int n_sb, int n_tok, int ldx, int ldy, int m_tiles, int k_split) {
    constexpr int BM = 64 * WM, NT = 128 * WM;
    constexpr int BN = 64 * NB;
    /* one part of a weight row's 32 nibble bytes per thread: four parts of 8 bytes or eight of 4 */
    constexpr bool kPart8 = BN * 4 == NT;
    static_assert(kPart8 || BN * 8 == NT, "one weight-row part per thread");
    constexpr int kARows = NT / 8; /* token rows that one pass of the threads' 16-byte activation chunks covers */
    constexpr int kATile = BM * kRow, kBTile = BN * kRow;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    uint8_t *As = lds;                      /* [kStages][BM][kRow]  */
    uint8_t *Bs = lds + kStages * kATile;   /* [kStages][BN][kRow]  */

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int wm = wv >> 1, wn = wv & 1;

    /* XCD-aware tile order: consecutive workgroup ids land on different XCDs (id % 8), each
     * with its own L2; the m-tiles that share one weight tile are given ids 8 apart so that
     * they meet in the same L2 */
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int tile_m = slot % m_tiles;
    const int tile_n = (slot / m_tiles) * 8 + xcd;
    if (tile_n * BN >= n_rows) return;

    const size_t row_bytes = (size_t)n_sb * 144;
    /* B-tile role: weight row br, part bp of the 32 nibble bytes of a sub-block pair (NB = 2: four
     * 8-byte parts per row, NB = 1: eight 4-byte parts) */
    const int br = kPart8 ? tid >> 2 : tid >> 3, bp = kPart8 ? tid & 3 : tid & 7;
    int w_row = tile_n * BN + br;
    if (w_row >= n_rows) w_row = n_rows - 1;
    const uint8_t *w_ptr = W + (size_t)w_row * row_bytes;
    /* A-tile role: chunks (token row ar + kARows j, 16-byte column ac), j = 0..3 */
    const int ar = tid >> 3, ac = tid & 7;
    /* blockIdx.y = which part of K (k_split parts of equal, even length); with more than one part the
     * results are added to a zeroed Y */
    const int n_steps = (int)(blockIdx.y + 1) * (n_sb * 4 / k_split);
    const int step0 = (int)blockIdx.y * (n_sb * 4 / k_split);

    /* register set of one tile in flight from global memory; named members only (a set that
     * lives across the tile loop stays in registers only when nothing indexes it) */
    struct StepRegs { uint4 x0, x1, x2, x3; uint2 qs; };
    /* d, dmin and the 6-bit scales and mins of one super-block of this thread's weight row, unpacked once
     * per super-block (four tiles): bytes 0..3 of sc_lo / mn_lo belong to sub-blocks 0..3, of sc_hi / mn_hi
     * to sub-blocks 4..7 */
    struct SbScales { float d, dmin; uint32_t sc_lo, sc_hi, mn_lo, mn_hi; };
    auto x_chunk = [&](int j, int step) {
        /* token rows past the end re-read row 0: their products land in accumulator rows that
         * are never stored */
        const int m = tile_m * BM + ar + kARows * j;
        return *reinterpret_cast<const uint4 *>(X + (size_t)(m < n_tok ? m : 0) * ldx + (size_t)step * kBK + 8 * ac);
    };
    auto fetch = [&](StepRegs &r, int step) {
        if (step >= n_steps) step = n_steps - 1; /* harmless re-read past the end */
        const int sb = step >> 2, c = step & 3;
        const uint8_t *blk = w_ptr + (size_t)sb * 144;
        if (kPart8) r.qs = *reinterpret_cast<const uint2 *>(blk + 16 + 32 * c + 8 * bp);
        else r.qs = make_uint2(*reinterpret_cast<const uint32_t *>(blk + 16 + 32 * c + 4 * bp), 0u);
        r.x0 = x_chunk(0, step); r.x1 = x_chunk(1, step); r.x2 = x_chunk(2, step); r.x3 = x_chunk(3, step);
    };

    const float unit = 1.0f / fp8_pair_lo(1u).x;
    auto load_hdr = [&](int sb) {
        if (sb * 4 >= n_steps) sb = n_steps / 4 - 1; /* harmless re-read past the end */
        return *reinterpret_cast<const uint4 *>(w_ptr + (size_t)sb * 144);
    };
    auto unpack_hdr = [&](const uint4 &h, SbScales &sc) {
        sc.d = half_bits_fast(h.x & 0xFFFFu) * unit;
        sc.dmin = half_bits_fast(h.x >> 16);
        sc.sc_lo = h.y & 0x3F3F3F3Fu;
        sc.mn_lo = h.z & 0x3F3F3F3Fu;
        sc.sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
        sc.mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
    };
    /* the two halves of the work that puts one tile into LDS stage `st`; c = which quarter of the
     * super-block, a constant at every call site */
    auto stage_weights = [&](const StepRegs &r, const SbScales &sc, int c, int st) {
        const uint32_t sc2 = ((c & 2) ? sc.sc_hi : sc.sc_lo) >> ((c & 1) * 16);
        const uint32_t mn2 = ((c & 2) ? sc.mn_hi : sc.mn_lo) >> ((c & 1) * 16);
        const float dl_a = sc.d * (float)(sc2 & 0xFFu), dl_b = sc.d * (float)((sc2 >> 8) & 0xFFu);
        const float ml_a = sc.dmin * (float)(mn2 & 0xFFu), ml_b = sc.dmin * (float)((mn2 >> 8) & 0xFFu);
        uint8_t *bt = Bs + st * kBTile;
        /* sub-block 2c (low nibbles) -> k 0..31 = chunks 0..3, sub-block 2c+1 -> chunks 4..7 */
        if (kPart8) {
            *reinterpret_cast<uint4 *>(bt + swz(br, bp)) = decode8(r.qs.x & 0x0F0F0F0Fu, r.qs.y & 0x0F0F0F0Fu, dl_a, ml_a);
            *reinterpret_cast<uint4 *>(bt + swz(br, 4 + bp)) =
                decode8((r.qs.x >> 4) & 0x0F0F0F0Fu, (r.qs.y >> 4) & 0x0F0F0F0Fu, dl_b, ml_b);
        } else { /* four codes per nibble position: half a 16-byte chunk each */
            *reinterpret_cast<uint2 *>(bt + swz(br, bp >> 1) + 8 * (bp & 1)) = decode4(r.qs.x & 0x0F0F0F0Fu, dl_a, ml_a);
            *reinterpret_cast<uint2 *>(bt + swz(br, 4 + (bp >> 1)) + 8 * (bp & 1)) =
                decode4((r.qs.x >> 4) & 0x0F0F0F0Fu, dl_b, ml_b);
        }
    };
    auto stage_acts = [&](const StepRegs &r, int st) {
        uint8_t *at = As + st * kATile;
        *reinterpret_cast<uint4 *>(at + swz(ar, ac)) = r.x0;
        *reinterpret_cast<uint4 *>(at + swz(ar + kARows, ac)) = r.x1;
        *reinterpret_cast<uint4 *>(at + swz(ar + 2 * kARows, ac)) = r.x2;
        *reinterpret_cast<uint4 *>(at + swz(ar + 3 * kARows, ac)) = r.x3;
    };

    floatx16 acc00, acc01, acc10, acc11;
#pragma unroll
    for (int v = 0; v < 16; v++) { acc00[v] = 0.0f; acc01[v] = 0.0f; acc10[v] = 0.0f; acc11[v] = 0.0f; }

    /* operand fragments of two k-steps (half a tile): 2 x (2 A + 2 B) x 8 bf16 */
    struct Frags { bf16x8 a0, a1, b0, b1, c0, c1, d0, d1; };
    const int frag_row = lane & 31, kg = lane >> 5;
    const int a_row = wm * 64 + frag_row, b_row = wn * (32 * NB) + frag_row;
    auto load_frags = [&](Frags &f, int st, int half) {
        const uint8_t *at = As + st * kATile, *bt = Bs + st * kBTile;
        const int ch0 = 4 * half + kg, ch1 = ch0 + 2; /* logical chunks of k-steps 2*half, 2*half+1 */
        f.a0 = *reinterpret_cast<const bf16x8 *>(at + swz(a_row, ch0));
        f.a1 = *reinterpret_cast<const bf16x8 *>(at + swz(a_row + 32, ch0));
        f.b0 = *reinterpret_cast<const bf16x8 *>(bt + swz(b_row, ch0));
        if (NB == 2) f.b1 = *reinterpret_cast<const bf16x8 *>(bt + swz(b_row + 32, ch0));
        f.c0 = *reinterpret_cast<const bf16x8 *>(at + swz(a_row, ch1));
        f.c1 = *reinterpret_cast<const bf16x8 *>(at + swz(a_row + 32, ch1));
        f.d0 = *reinterpret_cast<const bf16x8 *>(bt + swz(b_row, ch1));
        if (NB == 2) f.d1 = *reinterpret_cast<const bf16x8 *>(bt + swz(b_row + 32, ch1));
    };
    auto mma_half = [&](const Frags &f) {
        acc00 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a0, f.b0, acc00, 0, 0, 0);
        if (NB == 2) acc01 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a0, f.b1, acc01, 0, 0, 0);
        acc10 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a1, f.b0, acc10, 0, 0, 0);
        if (NB == 2) acc11 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a1, f.b1, acc11, 0, 0, 0);
        acc00 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.c0, f.d0, acc00, 0, 0, 0);
        if (NB == 2) acc01 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.c0, f.d1, acc01, 0, 0, 0);
        acc10 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.c1, f.d0, acc10, 0, 0, 0);
        if (NB == 2) acc11 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.c1, f.d1, acc11, 0, 0, 0);
    };

    /* ask the instruction scheduler for "one MFMA, then a few vector-ALU instructions" eight
     * times over, so that the decode arithmetic is issued in the shadow of the MFMAs of the same
     * wave instead of in front of them */
#define QLIN_INTERLEAVE_8(VALU_PER_MFMA)                                  \
    _Pragma("unroll") for (int q_ = 0; q_ < 4 * NB; q_++) {               \
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                \
        __builtin_amdgcn_sched_group_barrier(0x002, VALU_PER_MFMA, 0);    \
    }

    /* Pipeline, per tile i (LDS stage i % 3), all in one basic block between two barriers:
     *   matrix pipe : 16 MFMAs on tile i from fragment registers
     *   LDS reads   : second half of tile i, then first half of tile i+1 (half a tile ahead)
     *   vector ALU  : decode tile i+2 from registers into stage (i+2) % 3
     *   global loads: tile i+4 into the registers just freed
     * Stage (i+2) % 3 held tile i-1, whose last fragments were read before the barrier that
     * opens tile i; tile i+1 was completed before that same barrier. */
    StepRegs r0, r1;
    SbScales sbs;
    uint4 hdr_next;
    fetch(r0, step0);
    fetch(r1, step0 + 1);
    unpack_hdr(load_hdr(step0 >> 2), sbs);
    hdr_next = load_hdr((step0 >> 2) + 1);
    stage_weights(r0, sbs, 0, 0);
    stage_acts(r0, 0);
    fetch(r0, step0 + 2);
    stage_weights(r1, sbs, 1, 1);
    stage_acts(r1, 1);
    fetch(r1, step0 + 3);
    __syncthreads();
    Frags f0, f1;
    load_frags(f0, 0, 0);
    int st = 0; /* stage of the current tile */
    /* tile STEP + U of a super-block (U = 0..3, a constant); registers R hold tile STEP + U + 2, quarter
     * (U + 2) % 4 of its super-block, which for U >= 2 is the next one: its header was requested four
     * tiles ago and is unpacked here, and the one after it is requested */
#define QLIN_GEMM_TILE(R, STEP, U)                                                                     \
    {                                                                                                  \
        const int st1 = st == 2 ? 0 : st + 1, st2 = st1 == 2 ? 0 : st1 + 1;                            \
        load_frags(f1, st, 1);                                                                         \
        __builtin_amdgcn_sched_barrier(0); /* keep the operand fetch ahead of the MFMAs it hides behind */ \
        if ((U) == 2) {                                                                                \
            unpack_hdr(hdr_next, sbs);                                                                 \
            hdr_next = load_hdr(((STEP) >> 2) + 2);                                                    \
        }                                                                                              \
        stage_weights(R, sbs, ((U) + 2) & 3, st2);                                                     \
        mma_half(f0);                                                                                  \
        QLIN_INTERLEAVE_8(8)                                                                           \
        __builtin_amdgcn_sched_barrier(0);                                                             \
        load_frags(f0, st1, 0);                                                                        \
        __builtin_amdgcn_sched_barrier(0);                                                             \
        stage_acts(R, st2);                                                                            \
        fetch(R, (STEP) + (U) + 4);                                                                    \
        mma_half(f1);                                                                                  \
        QLIN_INTERLEAVE_8(5)                                                                           \
        __builtin_amdgcn_sched_barrier(0);                                                             \
        st = st1;                                                                                      \
    }                                                                                                  \
    __syncthreads();

    for (int step = step0; step < n_steps; step += 4) { /* one super-block of K per pass */
        QLIN_GEMM_TILE(r0, step, 0)
        QLIN_GEMM_TILE(r1, step, 1)
        QLIN_GEMM_TILE(r0, step, 2)
        QLIN_GEMM_TILE(r1, step, 3)
    }
#undef QLIN_GEMM_TILE

    /* C layout of the 32x32 MFMA: register v of lane l holds row 8*(v/4) + 4*(l/32) + v%4,
     * column l%32. Columns are weight rows, contiguous in the token-major output. */
    auto store_tile = [&](const floatx16 &acc, int mi, int ni) {
        const int n = tile_n * BN + wn * (32 * NB) + ni * 32 + (lane & 31);
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int m = tile_m * BM + wm * 64 + mi * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
            if (m < n_tok && n < n_rows) {
                if (k_split == 1) Y[(size_t)m * ldy + n] = acc[v];
                else unsafeAtomicAdd(&Y[(size_t)m * ldy + n], acc[v]); /* two addends onto zero: the order cannot matter */
            }
        }
    };
    store_tile(acc00, 0, 0);
    store_tile(acc10, 1, 0);
    if (NB == 2) {
        store_tile(acc01, 0, 1);
        store_tile(acc11, 1, 1);
    }
}

namespace {

__global__ void __launch_bounds__(256) zero_rows_kernel(float *__restrict__ Y, int n_rows, int ldy) {
    const int n = blockIdx.x * 256 + threadIdx.x;
    if (n < n_rows) Y[(size_t)blockIdx.y * ldy + n] = 0.0f;
}

template <int WM, int NB>
hipError_t launch_tiled(const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok, int ldx,
                        int ldy, hipStream_t stream) {
    static OnceFlag lds_raised;
    constexpr int BM = 64 * WM, BN = 64 * NB;
    const int n_sb = n_cols / 256;
    const int m_tiles = (n_tok + BM - 1) / BM;
    const int n_tiles = (n_rows + BN - 1) / BN;
    /* ids are dealt to 8 XCDs; pad the n-tile count to a multiple of 8 (surplus groups exit) */
    const int n_tiles_pad = (n_tiles + 7) / 8 * 8;
    const int grid = n_tiles_pad * m_tiles;
    const size_t lds_bytes = (size_t)kStages * (BM + BN) * kRow;
    /* half a chip's worth of tiles or less (4096 rows at 512 tokens: 128): each tile's K range is cut in
     * two halves that add their results to a zeroed Y; a + b onto zero is the same in either order, so
     * the result stays deterministic (three or more parts would not) */
    /* (128-token tiles: two workgroups fit a compute unit, so up to a chip's worth of tiles is cut) */
    const int k_split = (NB == 1 && n_tiles * m_tiles <= (WM == 2 ? 256 : 128) && n_sb >= 4 && n_sb % 2 == 0) ? 2 : 1;
    if (k_split > 1) {
        hipLaunchKernelGGL(zero_rows_kernel, dim3((n_rows + 255) / 256, n_tok), dim3(256), 0, stream, Y, n_rows, ldy);
    }
    if (!lds_raised.is_set()) {
        hipError_t e = hipFuncSetAttribute((const void *)gemm_q4k_bf16_kernel<WM, NB>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        lds_raised.set();
    }
    hipLaunchKernelGGL((gemm_q4k_bf16_kernel<WM, NB>), dim3(grid, k_split), dim3(128 * WM), lds_bytes, stream,
                       (const uint8_t *)W, X, Y, n_rows, n_sb, n_tok, ldx, ldy, m_tiles, k_split);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_gemm_q4k_bf16(const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols,
                                int n_tok, int ldx, int ldy, hipStream_t stream) {
    /* up to 48 tokens the weights are better streamed once per 16 tokens with exact codes (13-39 us at
     * 14336 x 4096) than pushed through a 256-token tile (54 us whatever the count) */
    if (n_tok <= kFewTokens) return launch_gemm_q4k_fewtok(W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    /* the four-wave kernels, large or small tiles by how many there are (their 32-bit offsets hold 256 rows of X) */
    const FusedTile tile = choose_fused_tile(T_Q4_K, n_rows, n_cols, n_tok, ldx, false);
    if (tile != kFusedNone) return launch_fused_tile(tile, T_Q4_K, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    /* a row pitch of 4 M elements or more: the eight-wave kernel of this file, which addresses with 64 bits.
     * 128-row tiles unless they would leave compute units without a workgroup */
    const int m_tiles = (n_tok + 255) / 256, n_tiles_128 = (n_rows + 127) / 128;
    if (n_tok <= 128) return launch_tiled<2, 1>(W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    if (m_tiles * n_tiles_128 < 200) return launch_tiled<4, 1>(W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    return launch_tiled<4, 2>(W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
}

}  // namespace qlin
