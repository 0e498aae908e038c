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
 * Tiling. A workgroup owns BM = 64*WM tokens x BN = 128 weight rows and walks K in steps of
 * 64 = one pair of Q4_K sub-blocks (the low and high nibbles of 32 quant bytes). Its waves
 * form a WM x 2 grid of 64x64 sub-tiles (2x2 MFMA tiles of 32x32, 64 accumulator registers).
 * Per step every thread
 *   - decodes 16 weights (8 nibble bytes of one row) into registers and stores them as bf16
 *     into the LDS B tile,
 *   - copies 4 x 16 bytes of activations into the LDS A tile,
 * and after one barrier the waves run 4 k-steps x 4 MFMAs from LDS. Global loads for step
 * i+2 are issued into a second register set before the MFMAs of step i (two LDS buffers, two
 * register sets). LDS rows are padded from 128 to 144 bytes so that the 32 rows read by one
 * MFMA operand fetch fall on distinct bank groups.
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

constexpr int kBN = 128;        /* weight rows per workgroup */
constexpr int kBK = 64;         /* k per step */
constexpr int kLdsRow = 144;    /* bytes per LDS tile row: 64 bf16 + 16 bytes of padding */

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

}  // namespace

template <int WM>
__global__ void __launch_bounds__(128 * WM)
gemm_q4k_bf16_kernel(const uint8_t *__restrict__ W, const uint16_t *__restrict__ X, float *__restrict__ Y,
                     int n_rows, int n_sb, int n_tok, int ldx, int ldy, int m_tiles) {
    constexpr int BM = 64 * WM, NT = 128 * WM;
    constexpr int PP = 512 / NT; /* (row, part) pairs of the B tile per thread */
    static_assert(PP == 1, "one weight-row part per thread: 512 threads");
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    uint8_t *As = lds;                          /* [2][BM][kLdsRow] */
    uint8_t *Bs = lds + 2 * BM * kLdsRow;       /* [2][kBN][kLdsRow] */

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int wm = wv >> 1, wn = wv & 1;

    /* XCD-aware tile order: consecutive workgroup ids land on different XCDs (id % 8), each
     * with its own L2; the m-tiles that share one weight tile are given ids 8 apart so that
     * they meet in the same L2 */
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int tile_m = slot % m_tiles;
    const int tile_n = (slot / m_tiles) * 8 + xcd;
    if (tile_n * kBN >= n_rows) return;

    const size_t row_bytes = (size_t)n_sb * 144;
    /* B-tile role: weight row br, 8-byte part bp of the 32 nibble bytes of a sub-block pair */
    const int br = tid >> 2, bp = tid & 3;
    int w_row = tile_n * kBN + br;
    if (w_row >= n_rows) w_row = n_rows - 1;
    const uint8_t *w_ptr = W + (size_t)w_row * row_bytes;
    /* A-tile role: chunk q = tid + j*NT -> token row q/8, 16-byte column q%8 */
    const int n_steps = n_sb * 4;

    auto fetch = [&](int step) {
        StepRegs r;
        if (step >= n_steps) step = n_steps - 1; /* harmless re-read past the end */
        const int sb = step >> 2, c = step & 3;
        const uint8_t *blk = w_ptr + (size_t)sb * 144;
        r.hdr = *reinterpret_cast<const uint4 *>(blk);
        r.qs = *reinterpret_cast<const uint2 *>(blk + 16 + 32 * c + 8 * bp);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int q = tid + j * NT;
            const int m = tile_m * BM + (q >> 3);
            const uint16_t *xp = X + (size_t)(m < n_tok ? m : 0) * ldx + (size_t)step * kBK + 8 * (q & 7);
            uint4 v = *reinterpret_cast<const uint4 *>(xp);
            if (m >= n_tok) v = make_uint4(0, 0, 0, 0);
            r.x[j] = v;
        }
        return r;
    };

    const float unit = 1.0f / fp8_pair_lo(1u).x;

    auto stage = [&](const StepRegs &r, int step, int buf) {
        /* activations */
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int q = tid + j * NT;
            *reinterpret_cast<uint4 *>(As + (size_t)buf * BM * kLdsRow + (q >> 3) * kLdsRow + 16 * (q & 7)) = r.x[j];
        }
        /* weights: sub-blocks 2c (low nibbles) and 2c+1 (high nibbles) */
        const int c = step & 3;
        const uint4 h = r.hdr;
        const float d = half_bits_fast(h.x & 0xFFFFu) * unit, dmin = half_bits_fast(h.x >> 16);
        const uint32_t sc_lo = h.y & 0x3F3F3F3Fu, mn_lo = h.z & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
        const uint32_t sc2 = ((c & 2) ? sc_hi : sc_lo) >> ((c & 1) * 16);
        const uint32_t mn2 = ((c & 2) ? mn_hi : mn_lo) >> ((c & 1) * 16);
        const float dl_a = d * (float)(sc2 & 0xFFu), dl_b = d * (float)((sc2 >> 8) & 0xFFu);
        const float ml_a = dmin * (float)(mn2 & 0xFFu), ml_b = dmin * (float)((mn2 >> 8) & 0xFFu);
        const uint32_t lo0 = r.qs.x & 0x0F0F0F0Fu, lo1 = r.qs.y & 0x0F0F0F0Fu;
        const uint32_t hi0 = (r.qs.x >> 4) & 0x0F0F0F0Fu, hi1 = (r.qs.y >> 4) & 0x0F0F0F0Fu;
        uint8_t *brow = Bs + (size_t)buf * kBN * kLdsRow + br * kLdsRow;
        *reinterpret_cast<uint4 *>(brow + 16 * bp) = decode8(lo0, lo1, dl_a, ml_a);
        *reinterpret_cast<uint4 *>(brow + 64 + 16 * bp) = decode8(hi0, hi1, dl_b, ml_b);
    };

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    const int frag_row = lane & 31, frag_k = (lane >> 5) * 16; /* byte offset of this lane's 8 k */
    auto compute = [&](int buf) {
        const uint8_t *a_base = As + (size_t)buf * BM * kLdsRow + (wm * 64 + frag_row) * kLdsRow + frag_k;
        const uint8_t *b_base = Bs + (size_t)buf * kBN * kLdsRow + (wn * 64 + frag_row) * kLdsRow + frag_k;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const bf16x8 a0 = *reinterpret_cast<const bf16x8 *>(a_base + 32 * s);
            const bf16x8 a1 = *reinterpret_cast<const bf16x8 *>(a_base + 32 * kLdsRow + 32 * s);
            const bf16x8 b0 = *reinterpret_cast<const bf16x8 *>(b_base + 32 * s);
            const bf16x8 b1 = *reinterpret_cast<const bf16x8 *>(b_base + 32 * kLdsRow + 32 * s);
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b1, acc[1][1], 0, 0, 0);
        }
    };

    StepRegs r0 = fetch(0), r1 = fetch(1);
    for (int step = 0; step < n_steps; step += 2) {
        stage(r0, step, 0);
        __syncthreads();
        r0 = fetch(step + 2);
        compute(0);
        stage(r1, step + 1, 1);
        __syncthreads();
        r1 = fetch(step + 3);
        compute(1);
    }

    /* C layout of the 32x32 MFMA: register v of lane l holds row 8*(v/4) + 4*(l/32) + v%4,
     * column l%32. Columns are weight rows, contiguous in the token-major output. */
#pragma unroll
    for (int mi = 0; mi < 2; mi++) {
#pragma unroll
        for (int ni = 0; ni < 2; ni++) {
            const int n = tile_n * kBN + wn * 64 + ni * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = tile_m * BM + wm * 64 + mi * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (m < n_tok && n < n_rows) Y[(size_t)m * ldy + n] = acc[mi][ni][v];
            }
        }
    }
}

hipError_t launch_gemm_q4k_bf16(const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols,
                                int n_tok, int ldx, int ldy, hipStream_t stream) {
    static bool lds_raised = false;
    constexpr int WM = 4, BM = 64 * WM;
    const int n_sb = n_cols / 256;
    const int m_tiles = (n_tok + BM - 1) / BM;
    const int n_tiles = (n_rows + kBN - 1) / kBN;
    /* ids are dealt to 8 XCDs; pad the n-tile count to a multiple of 8 (surplus groups exit) */
    const int n_tiles_pad = (n_tiles + 7) / 8 * 8;
    const int grid = n_tiles_pad * m_tiles;
    const size_t lds_bytes = (size_t)2 * (BM + kBN) * kLdsRow;
    if (!lds_raised) {
        hipError_t e = hipFuncSetAttribute((const void *)gemm_q4k_bf16_kernel<WM>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        lds_raised = true;
    }
    hipLaunchKernelGGL((gemm_q4k_bf16_kernel<WM>), dim3(grid), dim3(128 * WM), lds_bytes, stream,
                       (const uint8_t *)W, X, Y, n_rows, n_sb, n_tok, ldx, ldy, m_tiles);
    return hipGetLastError();
}

/* grouped MoE expert FFN: not built yet */
size_t moe_workspace_bytes(int, int, int, int, int) { return 256; }
hipError_t launch_moe_ffn_q4k(const void *, const void *, const void *, const uint16_t *, const int32_t *,
                              const float *, float *, int, int, int, int, int, void *, hipStream_t) {
    return hipErrorNotSupported;
}

}  // namespace qlin
