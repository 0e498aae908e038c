/*
 * gemm_dense_mfma.hip - prefill GEMM with dense bf16 weights on the gfx950 matrix cores.
 *
 *   Y[t*ldy + r] = sum_k X[t*ldx + k] * Wd[r*n_cols + k]      X, Wd bf16, Y fp32, fp32 accumulate
 *
 * The contraction of tf_gemm_f16_mt_tokenmajor (common/transformer.h:4487-4595; BF16 rows: the dense
 * branch of common/ggml_dequant.h:1201-1456) for weights that are bf16 already: BF16 tensors as they are,
 * every other format after one decode pass into a bf16 workspace (dequant.hip). The tile loop is the one
 * of the fused Q4_K kernel (gemm_q4k_mfma.hip) with the weight tile copied instead of decoded:
 * a workgroup of 512 threads owns 256 tokens x 128 weight rows (64 where the grid would not fill the chip)
 * and walks K in tiles of 64; 8 waves as 4 x 2 sub-tiles of 64 x 64 (2 x 2 v_mfma_f32_32x32x16_bf16);
 * LDS ring of three stages with the paired-row padding that keeps 16-byte operand reads conflict-free;
 * operands fetched half a tile ahead of the MFMAs, tile i+2 staged in their shadow, global loads four
 * tiles ahead in two register sets; one barrier per tile; workgroup ids dealt so that the token tiles of
 * one weight tile share an XCD's L2.
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

}  // namespace

/* NB = 2: 128 weight rows per workgroup (wave tile 64 tokens x 64 rows); NB = 1: 64 weight rows (wave
 * tile 64 x 32) and twice as many workgroups, for shapes whose grid would not fill the chip */
template <int WM, int NB>
__global__ void __launch_bounds__(128 * WM)
gemm_dense_bf16_kernel(const uint16_t *__restrict__ Wd, const uint16_t *__restrict__ X, float *__restrict__ Y,
                       int n_rows, int n_cols, int n_tok, int ldx, int ldy, int m_tiles, int k_split) {
    constexpr int BM = 64 * WM, NT = 128 * WM;
    static_assert(NT == 512, "one weight-row part per thread: 512 threads");
    constexpr int BN = 64 * NB;
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

    /* tile roles: chunk (row ar + 64j, 16-byte column ac) of the token tile (j = 0..3) and of the weight
     * tile (j = 0..NB-1) */
    const int ar = tid >> 3, ac = tid & 7;
    /* blockIdx.y = which part of K (k_split parts of equal length, each a multiple of four tiles); with
     * more than one part the results are added to a zeroed Y */
    const int k_tiles = n_cols / kBK;
    const int n_steps = (int)(blockIdx.y + 1) * (k_tiles / k_split);
    const int step0 = (int)blockIdx.y * (k_tiles / k_split);

    /* register set of one tile in flight from global memory; named members only (a set that
     * lives across the tile loop stays in registers only when nothing indexes it) */
    struct StepRegs { uint4 x0, x1, x2, x3, w0, w1; };
    auto x_chunk = [&](int j, int step) {
        /* token rows past the end re-read row 0: their products land in accumulator rows that
         * are never stored */
        const int m = tile_m * BM + ar + 64 * j;
        return *reinterpret_cast<const uint4 *>(X + (size_t)(m < n_tok ? m : 0) * ldx + (size_t)step * kBK + 8 * ac);
    };
    auto w_chunk = [&](int j, int step) { /* weight rows past the end re-read the last row; never stored */
        const int n = tile_n * BN + ar + 64 * j;
        return *reinterpret_cast<const uint4 *>(Wd + (size_t)(n < n_rows ? n : n_rows - 1) * n_cols + (size_t)step * kBK + 8 * ac);
    };
    auto fetch = [&](StepRegs &r, int step) {
        if (step >= n_steps) step = n_steps - 1; /* harmless re-read past the end */
        r.w0 = w_chunk(0, step);
        if (NB == 2) r.w1 = w_chunk(1, step);
        r.x0 = x_chunk(0, step); r.x1 = x_chunk(1, step); r.x2 = x_chunk(2, step); r.x3 = x_chunk(3, step);
    };
    /* the two halves of the work that puts one tile into LDS stage `st` */
    auto stage_weights = [&](const StepRegs &r, int st) {
        uint8_t *bt = Bs + st * kBTile;
        *reinterpret_cast<uint4 *>(bt + swz(ar, ac)) = r.w0;
        if (NB == 2) *reinterpret_cast<uint4 *>(bt + swz(ar + 64, ac)) = r.w1;
    };
    auto stage_acts = [&](const StepRegs &r, int st) {
        uint8_t *at = As + st * kATile;
        *reinterpret_cast<uint4 *>(at + swz(ar, ac)) = r.x0;
        *reinterpret_cast<uint4 *>(at + swz(ar + 64, ac)) = r.x1;
        *reinterpret_cast<uint4 *>(at + swz(ar + 128, ac)) = r.x2;
        *reinterpret_cast<uint4 *>(at + swz(ar + 192, ac)) = r.x3;
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
     *   LDS writes  : tile i+2 from registers into stage (i+2) % 3
     *   global loads: tile i+4 into the registers just freed
     * Stage (i+2) % 3 held tile i-1, whose last fragments were read before the barrier that
     * opens tile i; tile i+1 was completed before that same barrier. */
    StepRegs r0, r1;
    fetch(r0, step0);
    fetch(r1, step0 + 1);
    stage_weights(r0, 0);
    stage_acts(r0, 0);
    fetch(r0, step0 + 2);
    stage_weights(r1, 1);
    stage_acts(r1, 1);
    fetch(r1, step0 + 3);
    __syncthreads();
    Frags f0, f1;
    load_frags(f0, 0, 0);
    int st = 0; /* stage of the current tile */
    /* tile STEP + U (U = 0..3); registers R hold tile STEP + U + 2 */
#define QLIN_GEMM_TILE(R, STEP, U)                                                                     \
    {                                                                                                  \
        const int st1 = st == 2 ? 0 : st + 1, st2 = st1 == 2 ? 0 : st1 + 1;                            \
        load_frags(f1, st, 1);                                                                         \
        __builtin_amdgcn_sched_barrier(0); /* keep the operand fetch ahead of the MFMAs it hides behind */ \
        stage_weights(R, st2);                                                                         \
        mma_half(f0);                                                                                  \
        QLIN_INTERLEAVE_8(2)                                                                           \
        __builtin_amdgcn_sched_barrier(0);                                                             \
        load_frags(f0, st1, 0);                                                                        \
        __builtin_amdgcn_sched_barrier(0);                                                             \
        stage_acts(R, st2);                                                                            \
        fetch(R, (STEP) + (U) + 4);                                                                    \
        mma_half(f1);                                                                                  \
        QLIN_INTERLEAVE_8(3)                                                                           \
        __builtin_amdgcn_sched_barrier(0);                                                             \
        st = st1;                                                                                      \
    }                                                                                                  \
    __syncthreads();

    for (int step = step0; step < n_steps; step += 4) {
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

template <int NB>
hipError_t launch_tiled(const uint16_t *Wd, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok, int ldx,
                        int ldy, hipStream_t stream) {
    static OnceFlag lds_raised;
    constexpr int WM = 4, BM = 64 * WM, BN = 64 * NB;
    const int k_tiles = n_cols / kBK;
    const int m_tiles = (n_tok + BM - 1) / BM;
    const int n_tiles = (n_rows + BN - 1) / BN;
    /* ids are dealt to 8 XCDs; pad the n-tile count to a multiple of 8 (surplus groups exit) */
    const int n_tiles_pad = (n_tiles + 7) / 8 * 8;
    const int grid = n_tiles_pad * m_tiles;
    const size_t lds_bytes = (size_t)kStages * (BM + BN) * kRow;
    /* half a chip's worth of tiles or less: each tile's K range is cut in two halves that add their results
     * to a zeroed Y; a + b onto zero is the same in either order, so the result stays deterministic */
    const int k_split = (NB == 1 && n_tiles * m_tiles <= 128 && k_tiles >= 16 && k_tiles % 8 == 0) ? 2 : 1;
    if (k_split > 1) {
        hipLaunchKernelGGL(zero_rows_kernel, dim3((n_rows + 255) / 256, n_tok), dim3(256), 0, stream, Y, n_rows, ldy);
    }
    if (!lds_raised.is_set()) {
        hipError_t e = hipFuncSetAttribute((const void *)gemm_dense_bf16_kernel<WM, NB>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        lds_raised.set();
    }
    hipLaunchKernelGGL((gemm_dense_bf16_kernel<WM, NB>), dim3(grid, k_split), dim3(128 * WM), lds_bytes, stream,
                       Wd, X, Y, n_rows, n_cols, n_tok, ldx, ldy, m_tiles, k_split);
    return hipGetLastError();
}

}  // namespace

/* n_cols a multiple of 256, Wd and X 16-byte aligned, ldx a multiple of 8 */
hipError_t launch_gemm_dense_own(const uint16_t *Wd, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok,
                                 int ldx, int ldy, hipStream_t stream) {
    /* 128-row tiles unless they would leave compute units without a workgroup */
    const int m_tiles = (n_tok + 255) / 256, n_tiles_128 = (n_rows + 127) / 128;
    if (m_tiles * n_tiles_128 < 200) return launch_tiled<1>(Wd, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    return launch_tiled<2>(Wd, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
}

}  // namespace qlin
