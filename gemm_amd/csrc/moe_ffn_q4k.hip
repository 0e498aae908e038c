/*
 * moe_ffn_q4k.hip - grouped MoE expert FFN for Q4_K experts and bf16 activations:
 *
 *     out[t] = sum_k w[t,k] * down_e( silu(gate_e x_t) * (up_e x_t) ),  e = idx[t,k]
 *
 * the batched form of the per-token loop of common/transformer.h:4093-4128. With a few dozen
 * tokens spread over a hundred experts every expert sees a handful of tokens, so the job is
 * to stream each routed expert's blocks from HBM exactly once; the arithmetic is small.
 *
 * Four launches:
 *   1. group:   counting sort of the (token, k) pairs by expert (one workgroup).
 *   2. gate_up: one workgroup per (expert, 16 rows of gate and of up), its waves splitting K. For
 *               every 32-element sub-block a wave issues v_mfma_f32_16x16x32_bf16 with
 *                   A = 16 of the expert's tokens x 32 activations (bf16, as given),
 *                   B = 32 raw 4-bit codes x 16 rows, the codes 0..15 converted to bf16
 *                       (exact), two per instruction, by the scaled fp8 conversion,
 *               which yields S = sum_k q*x per (token, row) without any rounding of the
 *               weights; the block scales go on in fp32: acc += (d*sc)*S - (dmin*m)*SX, where
 *               SX = sum_k x comes from one more MFMA against a B of ones and lands in the
 *               same lanes as S. silu(g)*u is then split into a bf16 head and a bf16 tail
 *               (h = hi + lo up to 2^-17 relative), so the second GEMM sees h to ~fp32.
 *   3. down:    same scheme over K = n_ff with A = hi and A = lo accumulated in one
 *               accumulator; writes w[t,k] * result per pair. A workgroup walks four groups of 32
 *               rows with the next group's weights in flight (one group per workgroup when K
 *               exceeds 2048 or the rows are not a multiple of 128).
 *   4. combine: out[t] = the token's top_k partial rows added in k order (deterministic).
 *
 * Lane layout of the 16x16x32 MFMA (A: tokens i, B: rows j): lane l feeds A[i = l%16]
 * [k = 8*(l/16) .. +7] and B[k = 8*(l/16) .. +7][j = l%16]; it receives C[i = 4*(l/16)+v][j = l%16],
 * v = 0..3. So a lane owns one weight row (one scale pair per sub-block) and four tokens.
 * Sub-block 2c of a super-block is the low nibbles of qs[32c..32c+31], 2c+1 the high nibbles
 * (common/ggml_dequant.h:1592-1618): one 8-byte load per lane serves two MFMAs.
 */
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr int kQ4KBlock = 144;
constexpr int kHeadInts = 32, kHeadTokens = 16; /* an expert's record: one 128-byte line */
constexpr int kHeadLive = 2; /* record i, this entry: the i-th expert that has tokens (-1 behind the last) */

struct Workspace {
    int32_t *offsets;  /* [n_expert + 1] first slot of each expert */
    int32_t *head;     /* [n_expert][32] per expert: first slot, count, 14 unused, tokens of its first 16 slots */
    int32_t *order;    /* [n_pairs] slot -> pair (t*top_k + k), grouped by expert */
    int32_t *slot_of;  /* [n_pairs] pair -> slot, -1 for an expert index out of range */
    uint16_t *h_hi;    /* [n_pairs, n_ff] bf16 head of silu(g)*u, by slot */
    uint16_t *h_lo;    /* [n_pairs, n_ff] bf16 tail */
    float *part;       /* [n_pairs, n_embd] down(h), by slot */
    float *g32, *u32;  /* [n_pairs, n_ff] each: gate and up results of the any-format kernels, by slot */
    size_t bytes;
};

size_t round256(size_t n) { return (n + 255) & ~(size_t)255; }

Workspace carve(void *base, int n_tok, int top_k, int n_embd, int n_ff, int n_expert) {
    const size_t n_pairs = (size_t)n_tok * top_k;
    char *p = (char *)base;
    size_t off = 0;
    Workspace w;
    w.offsets = (int32_t *)(p + off); off += round256(((size_t)n_expert + 1) * 4);
    w.head = (int32_t *)(p + off);    off += round256((size_t)n_expert * kHeadInts * 4);
    w.order = (int32_t *)(p + off);   off += round256(n_pairs * 4);
    w.slot_of = (int32_t *)(p + off); off += round256(n_pairs * 4);
    w.h_hi = (uint16_t *)(p + off);   off += round256(n_pairs * n_ff * 2);
    w.h_lo = (uint16_t *)(p + off);   off += round256(n_pairs * n_ff * 2);
    w.part = (float *)(p + off);      off += round256(n_pairs * n_embd * 4);
    w.g32 = (float *)(p + off);       off += round256(n_pairs * n_ff * 4);
    w.u32 = (float *)(p + off);       off += round256(n_pairs * n_ff * 4);
    w.bytes = off;
    return w;
}

/* The expert of a workgroup of the matrix kernels: blockIdx.y itself, or - where a call has fewer (token, choice)
 * pairs than experts and the launch covers that many experts only - entry blockIdx.y of the list of experts that
 * have tokens (routed = the records; negative: no such expert, the workgroup ends). A launch over all experts
 * would start thousands of workgroups that only find their expert unused, and the gate/up kernels request
 * their first weight image before they know. */
__device__ __forceinline__ int block_expert(const int32_t *routed) {
    return routed ? __builtin_amdgcn_readfirstlane(routed[blockIdx.y * kHeadInts + kHeadLive]) : (int)blockIdx.y;
}

/* ---- 1. counting sort of pairs by expert; cnt[] and cur[] live in LDS ---- */
__global__ void __launch_bounds__(1024)
moe_group_kernel(const int32_t *__restrict__ idx, int n_pairs, int n_expert, int32_t *__restrict__ offsets,
                 int32_t *__restrict__ order, int32_t *__restrict__ slot_of, int32_t *__restrict__ head, int top_k) {
    extern __shared__ int32_t lds[]; /* cnt[n_expert], cur[n_expert], wave_total[16], wave_live[16] */
    int32_t *cnt = lds, *cur = lds + n_expert;
    for (int e = threadIdx.x; e < n_expert; e += blockDim.x) cnt[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const int e = idx[p];
        if (e >= 0 && e < n_expert) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    /* exclusive prefix sums over the workgroup, of cnt[] and of "has tokens": a thread owns `per` consecutive
     * experts, the threads' sums are scanned inside each wave by shuffles and the 16 wave totals by every thread */
    {
        const int per = (n_expert + (int)blockDim.x - 1) / (int)blockDim.x;
        const int e0 = threadIdx.x * per;
        int mine = 0, mine_live = 0;
        for (int q = 0; q < per; q++) {
            const int c = (e0 + q < n_expert) ? cnt[e0 + q] : 0;
            mine += c;
            mine_live += c > 0;
        }
        const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
        int incl = mine, incl_live = mine_live;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d, 64), up_live = __shfl_up(incl_live, d, 64);
            if (lane >= d) {
                incl += up;
                incl_live += up_live;
            }
        }
        int32_t *wave_total = lds + 2 * n_expert, *wave_live = wave_total + 16; /* [16] each */
        if (lane == 63) {
            wave_total[wv] = incl;
            wave_live[wv] = incl_live;
        }
        __syncthreads();
        int run = incl - mine, rank = incl_live - mine_live, n_live = 0;
        for (int w = 0; w < (int)(blockDim.x >> 6); w++) {
            if (w < wv) {
                run += wave_total[w];
                rank += wave_live[w];
            }
            n_live += wave_live[w];
        }
        for (int q = 0; q < per; q++) {
            if (e0 + q < n_expert) {
                offsets[e0 + q] = run;
                head[(e0 + q) * kHeadInts] = run;
                head[(e0 + q) * kHeadInts + 1] = cnt[e0 + q];
                cur[e0 + q] = run;
                run += cnt[e0 + q];
                /* the list of experts that have tokens, in expert order, one entry per record (record i holds
                 * the i-th such expert, -1 behind the last): a launch over fewer workgroups than experts reads it */
                if (cnt[e0 + q] > 0) head[(rank++) * kHeadInts + kHeadLive] = e0 + q;
            }
        }
        if (threadIdx.x == blockDim.x - 1) offsets[n_expert] = run;
        for (int i = n_live + threadIdx.x; i < n_expert; i += blockDim.x) head[i * kHeadInts + kHeadLive] = -1;
    }
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const int e = idx[p];
        int slot = -1;
        if (e >= 0 && e < n_expert) {
            slot = atomicAdd(&cur[e], 1);
            order[slot] = p;
            /* the tokens of an expert's first slots sit beside its count: the matrix kernels find them with
             * one load instead of offsets -> order -> token */
            const int rank = slot - offsets[e];
            if (rank < kHeadTokens) head[e * kHeadInts + kHeadInts - kHeadTokens + rank] = p / top_k;
        }
        slot_of[p] = slot;
    }
}

/* ---- shared pieces of the two matrix kernels ---- */

/* the sixteen 6-bit fields of a super-block as bytes: sc_lo = scales of sub-blocks 0..3,
 * sc_hi = 4..7, likewise the mins (get_scale_min_k4, common/ggml_dequant.h:1582-1590) */
struct Scales {
    float d, dmin;
    uint32_t sc_lo, sc_hi, mn_lo, mn_hi;
};

__device__ __forceinline__ Scales unpack_header(u32x4 h) {
    Scales s;
    s.d = half_bits_fast(h.x & 0xFFFFu);
    s.dmin = half_bits_fast(h.x >> 16);
    const uint32_t y = h.y, z = h.z, w = h.w;
    s.sc_lo = y & 0x3F3F3F3Fu;
    s.mn_lo = z & 0x3F3F3F3Fu;
    s.sc_hi = (w & 0x0F0F0F0Fu) | ((y >> 2) & 0x30303030u);
    s.mn_hi = ((w >> 4) & 0x0F0F0F0Fu) | ((z >> 2) & 0x30303030u);
    return s;
}

template <int SUB>
__device__ __forceinline__ void sub_scales(const Scales &s, float &dsc, float &dm) {
    const uint32_t sc = (SUB < 4) ? s.sc_lo : s.sc_hi;
    const uint32_t mn = (SUB < 4) ? s.mn_lo : s.mn_hi;
    constexpr int sh = 8 * (SUB & 3);
    dsc = s.d * (float)((sc >> sh) & 0xFFu);
    dm = s.dmin * (float)((mn >> sh) & 0xFFu);
}

/* 8 bytes 0x0q -> 8 bf16 holding q exactly: an E4M3 byte 0x0q is q * 2^-9, the scale 2^9 undoes that */
__device__ __forceinline__ bf16x8 codes_to_bf16(uint32_t a, uint32_t b) {
    const bf16x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(a, 512.0f, false);
    const bf16x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(a, 512.0f, true);
    const bf16x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(b, 512.0f, false);
    const bf16x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(b, 512.0f, true);
    bf16x8 r;
    r[0] = p0[0]; r[1] = p0[1]; r[2] = p1[0]; r[3] = p1[1];
    r[4] = p2[0]; r[5] = p2[1]; r[6] = p3[0]; r[7] = p3[1];
    return r;
}

__device__ __forceinline__ bf16x8 ones_bf16() {
    const u32x4 v = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    return __builtin_bit_cast(bf16x8, v);
}

__device__ __forceinline__ f32x4 mma(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 load_a(const uint16_t *p, bool live) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (live) v = *(const u32x4 *)p;
    return __builtin_bit_cast(bf16x8, v);
}

/* acc[v] += dsc0*S0[v] - dm0*X0[v] + dsc1*S1[v] - dm1*X1[v] */
__device__ __forceinline__ void apply_scales(f32x4 &acc, f32x4 S0, f32x4 S1, f32x4 X0, f32x4 X1, float dsc0,
                                             float dm0, float dsc1, float dm1) {
#pragma unroll
    for (int v = 0; v < 4; v++) {
        float a = acc[v];
        a = fmaf(dsc0, S0[v], a);
        a = fmaf(-dm0, X0[v], a);
        a = fmaf(dsc1, S1[v], a);
        a = fmaf(-dm1, X1[v], a);
        acc[v] = a;
    }
}

/* The lane's activation operands of one super-block: for each of the NA operands eight 16-byte
 * pieces, [2*c + half] = elements 64c + 32*half + 8*kg .. +7 of the super-block */
template <int NA>
struct Acts {
    u32x4 a[NA][8];
};

template <int NA>
__device__ __forceinline__ void load_acts(Acts<NA> &s, const uint16_t *const (&arow)[NA], int sb, int kg, bool live) {
#pragma unroll
    for (int v = 0; v < NA; v++) {
        const uint16_t *xk = arow[v] + sb * 256 + 8 * kg;
#pragma unroll
        for (int p = 0; p < 8; p++) {
            u32x4 t = {0u, 0u, 0u, 0u};
            if (live) t = *(const u32x4 *)(xk + 32 * p);
            s.a[v][p] = t;
        }
    }
}

/* One super-block of NW * 16 rows goes from global memory to a wave-private LDS image
 * [NW * 16 rows][144 bytes] as a flat stream of 16-byte chunks: chunk t = 64 i + lane of
 * instruction i is chunk t % 9 of image row t / 9, so nine consecutive lanes read one row piece of
 * 144 contiguous bytes. (Reading the pieces in the layout the matrix instruction wants, 8 bytes per
 * lane from 16 rows at once, costs one cache access per lane: 63 accesses per load instruction
 * measured, and the kernels were bound by exactly that.) The loads write LDS directly
 * (global_load_lds_dwordx4); they are written as instructions and waited for by hand because the
 * compiler would otherwise serialise every LDS access behind all of them. Image row R is row
 * R % rows_per_matrix of matrix R / rows_per_matrix (gate then up; one matrix for down).
 * Nothing else in these kernels uses M0. The loads carry no non-temporal mark, unlike the rows of
 * the matvec kernels: a 144-byte piece ends 16 bytes into a cache line whose rest belongs to the next
 * super-block, fetched a moment later by a neighbouring wave, and a second token tile of 16 walks
 * the same weights again (few-token GEMM 13.8 -> 12.9 us at 8 tokens, 26.6 -> 24.4 us at 32). */
/* The per-lane part of those addresses does not depend on the super-block: byte offset of the lane's chunk
 * inside its matrix tile, computed once per kernel. The loads then take the tile's address plus the
 * super-block's 144 * sb as a scalar base, so fetching an image costs no vector instruction beyond the
 * loads (the 64-bit address arithmetic per chunk was a sixth of the vector instructions of these kernels).
 * NM = 2: the first half of the image rows comes from one matrix, the second half from another (gate, up). */
template <int NW, int NM>
struct ImagePlan {
    static constexpr int kRows = NW * 16 / NM, kChunks = kRows * 9, kInstr = (kChunks + 63) / 64;
    uint32_t off[kInstr];
};

template <int NW, int NM>
__device__ __forceinline__ void plan_image(ImagePlan<NW, NM> &p, size_t row_bytes, int lane, int last_row = 0x7fffffff) {
#pragma unroll
    for (int i = 0; i < ImagePlan<NW, NM>::kInstr; i++) {
        const int t = 64 * i + lane;
        int R = t / 9;
        const int c9 = t - 9 * R;
        R = R < ImagePlan<NW, NM>::kRows ? R : ImagePlan<NW, NM>::kRows - 1; /* lanes past the last chunk issue nothing */
        R = R < last_row ? R : last_row; /* a ragged last tile re-reads its last row; those results are not stored */
        p.off[i] = (uint32_t)R * (uint32_t)row_bytes + 16u * (uint32_t)c9;
    }
}

__device__ __forceinline__ const uint8_t *uniform_ptr(const uint8_t *p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return (const uint8_t *)(uintptr_t)(((uint64_t)hi << 32) | (uint64_t)lo);
}

template <int NW, int NM>
__device__ __forceinline__ void image_from_global(uint8_t *img, const uint8_t *m0_rows, const uint8_t *m1_rows,
                                                  const ImagePlan<NW, NM> &p, int sb, int lane) {
    using Plan = ImagePlan<NW, NM>;
    const uint32_t img_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)img;
#pragma unroll
    for (int m = 0; m < NM; m++) {
        const uint8_t *base = uniform_ptr((m == 0 ? m0_rows : m1_rows) + (size_t)sb * kQ4KBlock);
#pragma unroll
        for (int i = 0; i < Plan::kInstr; i++) {
            const uint32_t m0v =
                __builtin_amdgcn_readfirstlane(img_lds + (uint32_t)(m * Plan::kRows * kQ4KBlock) + 1024u * (uint32_t)i);
            if (64 * i + lane < Plan::kChunks)
                asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                             :
                             : "v"(p.off[i]), "s"(base), "s"(m0v)
                             : "memory");
        }
    }
}

template <int C, int NW, int NA>
__device__ __forceinline__ void slice_math(const uint8_t *img_row, const Acts<NA> &s, const Scales (&sc)[NW],
                                           f32x4 (&acc)[NW]) {
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    bf16x8 a0[NA], a1[NA];
    f32x4 X0 = zero, X1 = zero;
#pragma unroll
    for (int v = 0; v < NA; v++) {
        a0[v] = __builtin_bit_cast(bf16x8, s.a[v][2 * C]);
        a1[v] = __builtin_bit_cast(bf16x8, s.a[v][2 * C + 1]);
        X0 = mma(a0[v], ones_bf16(), X0);
        X1 = mma(a1[v], ones_bf16(), X1);
    }
#pragma unroll
    for (int w = 0; w < NW; w++) {
        /* the lane's 8 bytes hold its 8 codes of sub-block 2c (low nibbles) and of 2c+1 (high nibbles) */
        const u32x2 q = *(const u32x2 *)(img_row + w * 16 * kQ4KBlock + 16 + 32 * C);
        const bf16x8 lo = codes_to_bf16(q.x & 0x0F0F0F0Fu, q.y & 0x0F0F0F0Fu);
        const bf16x8 hi = codes_to_bf16((q.x >> 4) & 0x0F0F0F0Fu, (q.y >> 4) & 0x0F0F0F0Fu);
        f32x4 S0 = zero, S1 = zero;
#pragma unroll
        for (int v = 0; v < NA; v++) {
            S0 = mma(a0[v], lo, S0);
            S1 = mma(a1[v], hi, S1);
        }
        float dsc0, dm0, dsc1, dm1;
        sub_scales<2 * C>(sc[w], dsc0, dm0);
        sub_scales<2 * C + 1>(sc[w], dsc1, dm1);
        apply_scales(acc[w], S0, S1, X0, X1, dsc0, dm0, dsc1, dm1);
    }
}

/* img_row: the lane's row j of stream 0 in the image, plus 8 * kg (its code bytes inside a slice) */
template <int NW, int NA>
__device__ __forceinline__ void step_math(const uint8_t *img, int j, int kg, const Acts<NA> &s, f32x4 (&acc)[NW]) {
    Scales sc[NW];
#pragma unroll
    for (int w = 0; w < NW; w++) sc[w] = unpack_header(*(const u32x4 *)(img + (w * 16 + j) * kQ4KBlock));
    const uint8_t *img_row = img + j * kQ4KBlock + 8 * kg;
    slice_math<0>(img_row, s, sc, acc);
    slice_math<1>(img_row, s, sc, acc);
    slice_math<2>(img_row, s, sc, acc);
    slice_math<3>(img_row, s, sc, acc);
}

/* A workgroup owns (expert, 32 rows); its waves split K: wave w takes super-blocks w, w + waves, ...
 * (exactly one each up to K = 256 * waves), so every wave issues all of its loads at once and the
 * chip has thousands of independent requests in flight instead of a few waves walking K. The
 * partial sums of the waves meet in LDS: red[wave][stream][lane][4]. After the call and a barrier,
 * element (stream s, lane l, v) of the tile is the sum over waves of
 * red[(w * NW + s) * 256 + l * 4 + v], taken in wave order. */
template <int NW, int NM, int NA>
__device__ __forceinline__ void ksplit_tile(uint8_t *img, const uint8_t *m0_rows, const uint8_t *m1_rows,
                                            const ImagePlan<NW, NM> &plan,
                                            const uint16_t *const (&arow)[NA], int n_sb, int wv, int n_waves,
                                            int lane, bool live, int fetched_sb, float *red) {
    const int j = lane & 15, kg = lane >> 4;
    f32x4 acc[NW];
#pragma unroll
    for (int w = 0; w < NW; w++) acc[w] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    for (int sb = wv; sb < n_sb; sb += n_waves) {
        Acts<NA> s;
        if (sb != fetched_sb) { /* else the image of this super-block has been requested already */
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* reads of the previous image have returned */
            image_from_global(img, m0_rows, m1_rows, plan, sb, lane);
        }
        load_acts(s, arow, sb, kg, live);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* image (and activations) have landed */
        step_math<NW, NA>(img, j, kg, s, acc);
    }
#pragma unroll
    for (int w = 0; w < NW; w++) *reinterpret_cast<f32x4 *>(red + ((wv * NW + w) * 64 + lane) * 4) = acc[w];
}

/* ---- the same sums for an expert with at most four tokens: block-diagonal activation operand ----
 * An expert of a routed batch sees about four tokens, so twelve of the sixteen token rows of the matrix
 * instruction above are padding, and the fp32 scale step (16 multiply-adds per lane for every two
 * sub-blocks) is spent on them. Here the sixteen A rows are 4 sub-blocks x 4 tokens instead: row
 * i = 4 * s + t holds token t's activations in k group s and zeros in the other three groups, and the
 * B lanes of k group s carry codes of a sub-block of their own (2s: low nibbles, 2s + 1: high nibbles of
 * qs[32s .. 32s + 31]). C[4s + t][j] is then the sum over that one sub-block, it lands in lane (j, s), and
 * four instructions chained into one accumulator cover the sub-block's 32 elements: a lane applies ONE
 * scale pair per super-block half to four token values, 16 multiply-adds per super-block instead of 128.
 * The sums over the four k groups and over the waves are taken afterwards.
 *
 * The four tokens' activations of a super-block (2 KB) come into a wave-private LDS buffer by two
 * direct-to-LDS loads (xoff[i]: the byte offset of the lane's 16-byte chunk, token row included) instead
 * of eight register loads of which three quarters of the lanes would be idle; the operand lanes read
 * their 16 bytes from there. K is split over the waves as in ksplit_tile. After the call and a barrier,
 * the value for (stream s, token t, row j) is the sum over waves w of qred[((w * NW + s) * 16 + j) * 4 + t]. */
template <int NW, int NM>
__device__ __forceinline__ void ksplit_quad(uint8_t *img, const uint8_t *m0_rows, const uint8_t *m1_rows,
                                            const ImagePlan<NW, NM> &plan, uint8_t *actbuf, const uint8_t *x_base,
                                            const uint32_t (&xoff)[2], int n_sb, int wv, int n_waves, int lane,
                                            int fetched_sb, float *qred) {
    const int j = lane & 15, kg = lane >> 4;
    const bool diag = (j >> 2) == kg;
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    const uint32_t act_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)actbuf;
    const uint8_t *arow = actbuf + (j & 3) * 512 + 128 * kg; /* token j & 3, sub-blocks 2 * kg and 2 * kg + 1 */
    const uint8_t *codes = img + j * kQ4KBlock + 16 + 32 * kg;
    f32x4 acc[NW];
#pragma unroll
    for (int w = 0; w < NW; w++) acc[w] = zero;
    for (int sb = wv; sb < n_sb; sb += n_waves) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* reads of the previous image and activations have returned */
        if (sb != fetched_sb) image_from_global(img, m0_rows, m1_rows, plan, sb, lane);
        const uint8_t *xb = uniform_ptr(x_base + (size_t)sb * 512);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint32_t m0v = __builtin_amdgcn_readfirstlane(act_lds + 1024u * (uint32_t)i);
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(xoff[i]), "s"(xb), "s"(m0v) : "memory");
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* image and activations have landed */
        f32x4 S[NW][2], X0 = zero, X1 = zero;
#pragma unroll
        for (int w = 0; w < NW; w++) S[w][0] = S[w][1] = zero;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            u32x4 r0 = {0u, 0u, 0u, 0u}, r1 = {0u, 0u, 0u, 0u};
            if (diag) {
                r0 = *(const u32x4 *)(arow + 16 * c);
                r1 = *(const u32x4 *)(arow + 64 + 16 * c);
            }
            const bf16x8 a0 = __builtin_bit_cast(bf16x8, r0), a1 = __builtin_bit_cast(bf16x8, r1);
            X0 = mma(a0, ones_bf16(), X0);
            X1 = mma(a1, ones_bf16(), X1);
#pragma unroll
            for (int w = 0; w < NW; w++) {
                const u32x2 qv = *(const u32x2 *)(codes + w * 16 * kQ4KBlock + 8 * c);
                const bf16x8 lo = codes_to_bf16(qv.x & 0x0F0F0F0Fu, qv.y & 0x0F0F0F0Fu);
                const bf16x8 hi = codes_to_bf16((qv.x >> 4) & 0x0F0F0F0Fu, (qv.y >> 4) & 0x0F0F0F0Fu);
                S[w][0] = mma(a0, lo, S[w][0]);
                S[w][1] = mma(a1, hi, S[w][1]);
            }
        }
#pragma unroll
        for (int w = 0; w < NW; w++) {
            const Scales sc = unpack_header(*(const u32x4 *)(img + (w * 16 + j) * kQ4KBlock));
            /* the lane's two sub-blocks 2 * kg and 2 * kg + 1: bytes 2 * (kg & 1) and + 1 of the low or high word */
            const uint32_t sh = 16u * (uint32_t)(kg & 1);
            const uint32_t sp = (kg < 2 ? sc.sc_lo : sc.sc_hi) >> sh, mp = (kg < 2 ? sc.mn_lo : sc.mn_hi) >> sh;
            const float dsc0 = sc.d * (float)(sp & 0xFFu), dsc1 = sc.d * (float)((sp >> 8) & 0xFFu);
            const float dm0 = sc.dmin * (float)(mp & 0xFFu), dm1 = sc.dmin * (float)((mp >> 8) & 0xFFu);
            apply_scales(acc[w], S[w][0], S[w][1], X0, X1, dsc0, dm0, dsc1, dm1);
        }
    }
    /* a lane holds the share of its k group: add the four groups (lanes j, j + 16, j + 32, j + 48) */
#pragma unroll
    for (int w = 0; w < NW; w++) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
            float a = acc[w][v];
            a = sum_lane_groups(a);
            acc[w][v] = a;
        }
        if (kg == 0) *reinterpret_cast<f32x4 *>(qred + ((wv * NW + w) * 16 + j) * 4) = acc[w];
    }
}

/* thread -> element of the (16 * RT)-row x 16-slot result tile, token slot by token slot with consecutive
 * threads on consecutive rows: idx = (slot * RT + r) * 16 + j, so that a tile with n live slots is the
 * first n * 16 * RT elements (an expert sees about four tokens; summing the empty slots' shares as well
 * took a fifth of the down projection's time). Slot 4 * kg + v of row j is register v of lane (j, kg). */
struct TileElem { int r, lane, v, slot, row; };
template <int RT>
__device__ __forceinline__ TileElem tile_elem(int idx) {
    TileElem t;
    const int j = idx & 15, q = idx >> 4;
    t.r = q % RT;
    t.slot = q / RT;
    t.v = t.slot & 3;
    t.lane = (t.slot >> 2) * 16 + j;
    t.row = 16 * t.r + j;        /* row inside the group */
    return t;
}
__device__ __forceinline__ int live_slots(int cnt, int t0) { return cnt - t0 < 16 ? cnt - t0 : 16; }

/* ---- 2. gate and up for RT * 16 rows of one expert, all of its tokens ---- */
/* launch shape of the grouped kernels, as measured best at 128 experts of 768 x 2048, 64 tokens, top-8 */
constexpr int kGuWavesPerSimd = 2; /* gate+up kernel: waves per SIMD the registers are budgeted for */
constexpr int kDnWavesPerSimd = 2; /* down kernels: the same */
constexpr int kGuWgWaves = 4;      /* gate+up kernel: waves of a workgroup (each takes a share of K) */
constexpr int kGuRowTiles = 1;     /* gate+up kernel: 16-row tiles per workgroup */
template <int RT>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(kGuWavesPerSimd)))
moe_gate_up_kernel(const uint8_t *__restrict__ gate, const uint8_t *__restrict__ up,
                   const uint16_t *__restrict__ X, const int32_t *__restrict__ head,
                   const int32_t *__restrict__ order, uint16_t *__restrict__ h_hi, uint16_t *__restrict__ h_lo,
                   int n_embd, int n_ff, int top_k, const int32_t *__restrict__ routed) {
    constexpr int NW = 2 * RT, kRows = 16 * RT; /* streams: RT gate tiles, then RT up tiles */
    extern __shared__ __attribute__((aligned(16))) float red[];
    const int e = block_expert(routed);
    if (e < 0) return;
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n_waves = blockDim.x >> 6;
    const int row0 = blockIdx.x * kRows;
    const int j = lane & 15;
    const int n_sb = n_embd >> 8;
    const size_t row_bytes = (size_t)n_sb * kQ4KBlock;
    const size_t ebase = ((size_t)e * n_ff + row0) * row_bytes;
    /* LDS: red [waves][NW][64][4] floats | images [waves][NW * 16 rows][144 bytes] | qred [waves][NW][16][4] floats.
     * The four-token form keeps a wave's activations (2 KB) in the wave's part of red and reduces through qred. */
    uint8_t *img = reinterpret_cast<uint8_t *>(red + n_waves * NW * 256) + wv * (NW * 16 * kQ4KBlock);
    float *qred = reinterpret_cast<float *>(reinterpret_cast<uint8_t *>(red + n_waves * NW * 256) + n_waves * (NW * 16 * kQ4KBlock));
    const bool one_sb = n_sb <= n_waves; /* then a wave's image is fetched once for all token tiles */
    ImagePlan<NW, 2> plan;
    plan_image(plan, row_bytes, lane);
    /* The expert's record and the wave's first image are requested together: the lane's token for the
     * sixteen-token form and for the four-token form, then the image; the wait for the tokens leaves the
     * image's loads outstanding, and the activation loads follow while the image is still on its way.
     * (Waiting for the record first and for the token list after it cost a workgroup a quarter of its life.) */
    const int32_t *hd = head + (size_t)e * kHeadInts;
    const int32_t *tok_at = hd + (kHeadInts - kHeadTokens);
    int tok16, tok_a, tok_b; /* the token of slot j; of slots lane / 32 and 2 + lane / 32 */
    u32x2 first_cnt; /* loaded here as well: a load the compiler issues would be waited for with everything before it */
    asm volatile("global_load_dword %0, %4, off\n\tglobal_load_dword %1, %5, off\n\tglobal_load_dword %2, %5, off offset:8\n\t"
                 "global_load_dwordx2 %3, %6, off"
                 : "=&v"(tok16), "=&v"(tok_a), "=&v"(tok_b), "=&v"(first_cnt)
                 : "v"(tok_at + j), "v"(tok_at + (lane >> 5)), "v"(hd)
                 : "memory");
    image_from_global(img, gate + ebase, up + ebase, plan, wv, lane); /* wv < n_sb: the launch starts min(n_sb, 4) waves */
    constexpr int kImageLoads = 2 * ImagePlan<NW, 2>::kInstr;
    static_assert(kImageLoads <= 15, "the wait below counts outstanding loads up to 15");
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(tok16), "+v"(tok_a), "+v"(tok_b), "+v"(first_cnt) : "n"(kImageLoads) : "memory");
    const int first = __builtin_amdgcn_readfirstlane((int)first_cnt.x), cnt = __builtin_amdgcn_readfirstlane((int)first_cnt.y);
    if (cnt == 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* nothing may arrive in LDS after the wave has ended */
        return;
    }
    auto store_h = [&](float g, float u, int slot, int row) {
        const float h = g / (1.0f + expf(-g)) * u; /* tf_silu_mul, common/transformer.h:4679-4694 */
        const __bf16 hi = (__bf16)h;
        const __bf16 lo = (__bf16)(h - (float)hi);
        const size_t at = (size_t)slot * n_ff + row0 + row;
        h_hi[at] = __builtin_bit_cast(uint16_t, hi);
        h_lo[at] = __builtin_bit_cast(uint16_t, lo);
    };

    if (cnt <= 4) {
        /* by the expert's count, not a tile's: the rounding of a token's result must not depend on its slot */
        const int tok0 = __builtin_amdgcn_readfirstlane(tok_a); /* slot 0 exists; it stands in for the empty slots */
        const int sa = lane >> 5, sb2 = 2 + (lane >> 5);
        const uint32_t xoff[2] = {(uint32_t)(sa < cnt ? tok_a : tok0) * (uint32_t)n_embd * 2u + 16u * (uint32_t)(lane & 31),
                                  (uint32_t)(sb2 < cnt ? tok_b : tok0) * (uint32_t)n_embd * 2u + 16u * (uint32_t)(lane & 31)};
        ksplit_quad<NW, 2>(img, gate + ebase, up + ebase, plan, reinterpret_cast<uint8_t *>(red + wv * NW * 256),
                           reinterpret_cast<const uint8_t *>(X), xoff, n_sb, wv, n_waves, lane, wv, qred);
        __syncthreads();
        for (int idx = threadIdx.x; idx < 64 * RT; idx += blockDim.x) {
            /* consecutive threads: consecutive rows of one token */
            const int jj = idx & 15, r = (idx >> 4) % RT, t = idx / (16 * RT);
            float g = 0.0f, u = 0.0f;
            for (int w = 0; w < n_waves; w++) {
                g += qred[((w * NW + r) * 16 + jj) * 4 + t];
                u += qred[((w * NW + RT + r) * 16 + jj) * 4 + t];
            }
            if (t < cnt) store_h(g, u, first + t, 16 * r + jj);
        }
        return;
    }
    for (int t0 = 0; t0 < cnt; t0 += 16) {
        const int fetched_sb = (t0 == 0 || one_sb) ? wv : -1;
        const bool live = t0 + j < cnt; /* as an A lane, j is the token slot */
        const int tok = !live ? 0 : t0 == 0 ? tok16 : order[first + t0 + j] / top_k;
        const uint16_t *const arow[1] = {X + (size_t)tok * n_embd};
        ksplit_tile<NW, 2, 1>(img, gate + ebase, up + ebase, plan, arow, n_sb, wv, n_waves, lane, live, fetched_sb, red);
        __syncthreads();
        for (int idx = threadIdx.x; idx < live_slots(cnt, t0) * 16 * RT; idx += blockDim.x) {
            const TileElem t = tile_elem<RT>(idx);
            float g = 0.0f, u = 0.0f;
            for (int w = 0; w < n_waves; w++) {
                g += red[((w * NW + t.r) * 64 + t.lane) * 4 + t.v];
                u += red[((w * NW + RT + t.r) * 64 + t.lane) * 4 + t.v];
            }
            store_h(g, u, first + t0 + t.slot, t.row);
        }
        __syncthreads();
    }
}

/* ---- 3. down for RT * 16 rows of one expert ---- */
constexpr int kDnRowTiles = 2; /* down kernels: 16-row tiles per workgroup */
template <int RT>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(kDnWavesPerSimd)))
moe_down_kernel(const uint8_t *__restrict__ down, const uint16_t *__restrict__ h_hi,
                const uint16_t *__restrict__ h_lo, const int32_t *__restrict__ offsets, float *__restrict__ part,
                int n_embd, int n_ff, const int32_t *__restrict__ routed) {
    constexpr int kRows = 16 * RT;
    extern __shared__ __attribute__((aligned(16))) float red[];
    const int e = block_expert(routed);
    if (e < 0) return;
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n_waves = blockDim.x >> 6;
    const int row0 = blockIdx.x * kRows;
    const int first = offsets[e], cnt = offsets[e + 1] - first;
    if (cnt == 0) return;
    const int j = lane & 15;
    const int n_sb = n_ff >> 8;
    const size_t row_bytes = (size_t)n_sb * kQ4KBlock;
    const uint8_t *d0 = down + ((size_t)e * n_embd + row0) * row_bytes;
    /* LDS: red [waves][RT][64][4] floats | images [waves][RT * 16 rows][144 bytes] */
    uint8_t *img = reinterpret_cast<uint8_t *>(red + n_waves * RT * 256) + wv * (kRows * kQ4KBlock);
    const bool one_sb = n_sb <= n_waves;
    ImagePlan<RT, 1> plan;
    plan_image(plan, row_bytes, lane);
    if (one_sb && wv < n_sb) image_from_global(img, d0, d0, plan, wv, lane);

    for (int t0 = 0; t0 < cnt; t0 += 16) {
        const bool live = t0 + j < cnt;
        const size_t at_a = (size_t)(first + (live ? t0 + j : 0)) * n_ff;
        const uint16_t *const arow[2] = {h_hi + at_a, h_lo + at_a};
        ksplit_tile<RT, 1, 2>(img, d0, d0, plan, arow, n_sb, wv, n_waves, lane, live, one_sb ? wv : -1, red);
        __syncthreads();
        for (int idx = threadIdx.x; idx < live_slots(cnt, t0) * 16 * RT; idx += blockDim.x) {
            const TileElem t = tile_elem<RT>(idx);
            float d = 0.0f;
            for (int w = 0; w < n_waves; w++) d += red[((w * RT + t.r) * 64 + t.lane) * 4 + t.v];
            part[(size_t)(first + t0 + t.slot) * n_embd + row0 + t.row] = d; /* the routing weight goes on in the combine */
        }
        __syncthreads();
    }
}

/* ---- 3b. down for NT consecutive groups of RT * 16 rows of one expert, K <= 256 * waves ----
 * The same arithmetic as moe_down_kernel, with the workgroup walking NT row groups: the weight image of
 * group r + 1 is in flight while group r is multiplied, reduced over the waves and stored, and the
 * expert's activations and routing weights are fetched once for all NT groups. A (expert, 32 rows)
 * workgroup lives for four or five memory round trips and moves 14 KB of weights; with a handful of them
 * on a compute unit that bounded the kernel at a quarter of HBM speed. */
constexpr int kDnColTiles = 4; /* wide down kernel: row-tile groups that share one workgroup's activations */
template <int RT, int NT>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(kDnWavesPerSimd)))
moe_down_walk_kernel(const uint8_t *__restrict__ down, const uint16_t *__restrict__ h_hi,
                     const uint16_t *__restrict__ h_lo, const int32_t *__restrict__ offsets,
                     float *__restrict__ part, int n_embd, int n_ff, const int32_t *__restrict__ routed) {
    constexpr int kRows = 16 * RT, kImage = kRows * kQ4KBlock;
    constexpr int kImageLoads = (kRows * 9 + 63) / 64; /* direct-to-LDS instructions per image and wave */
    constexpr int kElems = 256 * RT;                   /* results of one row group and token tile */
    static_assert(kImageLoads <= 15, "the wait below counts outstanding loads up to 15");
    extern __shared__ __attribute__((aligned(16))) float red[];
    const int e = block_expert(routed);
    if (e < 0) return;
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n_waves = blockDim.x >> 6;
    const int row0 = blockIdx.x * (kRows * NT);
    const int first = offsets[e], cnt = offsets[e + 1] - first;
    if (cnt == 0) return;
    const int j = lane & 15, kg = lane >> 4;
    const int n_sb = n_ff >> 8; /* <= n_waves: wave wv owns super-block wv */
    const size_t row_bytes = (size_t)n_sb * kQ4KBlock;
    const uint8_t *d0 = down + ((size_t)e * n_embd + row0) * row_bytes;
    /* LDS: red [waves][RT][64][4] floats | images [waves][2][RT * 16 rows][144 bytes] */
    uint8_t *img = reinterpret_cast<uint8_t *>(red + n_waves * kElems) + wv * (2 * kImage);
    const bool has_k = wv < n_sb;
    ImagePlan<RT, 1> plan;
    plan_image(plan, row_bytes, lane);

    for (int t0 = 0; t0 < cnt; t0 += 16) {
        const bool live = t0 + j < cnt;
        const size_t at_a = (size_t)(first + (live ? t0 + j : 0)) * n_ff;
        const uint16_t *const arow[2] = {h_hi + at_a, h_lo + at_a};
        Acts<2> s;
        if (has_k) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* reads of the previous token tile's images have returned */
            image_from_global(img, d0, d0, plan, wv, lane);
            load_acts(s, arow, wv, kg, live);
        }
        /* no other global load inside the walk: the compiler would wait for the image in flight with it
         * (the pairs' routing weights are applied by the combine) */
        for (int rt = 0; rt < NT; rt++) {
            f32x4 acc[RT];
#pragma unroll
            for (int w = 0; w < RT; w++) acc[w] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            if (has_k) {
                if (rt + 1 < NT) {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* the other image has been read */
                    const uint8_t *dn = d0 + (size_t)(rt + 1) * kRows * row_bytes;
                    image_from_global(img + ((rt + 1) & 1) * kImage, dn, dn, plan, wv, lane);
                    wait_vm_at_most(kImageLoads); /* everything older than those: this group's image, the activations */
                } else {
                    wait_vm_at_most(0);
                }
                step_math<RT, 2>(img + (rt & 1) * kImage, j, kg, s, acc);
            }
#pragma unroll
            for (int w = 0; w < RT; w++) *reinterpret_cast<f32x4 *>(red + ((wv * RT + w) * 64 + lane) * 4) = acc[w];
            __syncthreads();
            for (int idx = threadIdx.x; idx < live_slots(cnt, t0) * 16 * RT; idx += blockDim.x) {
                const TileElem t = tile_elem<RT>(idx);
                float d = 0.0f;
                for (int w = 0; w < n_waves; w++) d += red[((w * RT + t.r) * 64 + t.lane) * 4 + t.v];
                part[(size_t)(first + t0 + t.slot) * n_embd + row0 + rt * kRows + t.row] = d;
            }
            __syncthreads();
        }
    }
}

/* ---- 3c. down for Q6_K and Q5_K experts (what K-quant mixes store beside or instead of Q4_K) ----
 * The same walk as moe_down_walk_kernel over NT groups of 16 rows, a wave per super-block of K, the next
 * group's image in flight while this one is multiplied. What differs:
 *   * A Q6_K block is 210 bytes, so rows and blocks start on 2-byte boundaries. A wave's image row is the 14
 *     aligned 16-byte chunks that cover its block (the block starts `o` = 0..14 bytes into the first); LDS is
 *     read as aligned dwords and funnel-shifted.
 *   * A code is q = nibble + 16 * two high bits - 32 with one int8 scale per 16 elements
 *     (common/ggml_dequant.h:1653-1686). Nibble and high bits go through the matrix instruction as two exact
 *     bf16 operands (both below 16, so the scaled fp8 conversion applies): sum q x = S_lo + 16 S_hi - 32 X.
 *   * One instruction spans 32 elements = two scale groups, so the token operand is block-diagonal: A row
 *     8 s + t holds token t's activations in the k groups of scale group s (2s, 2s + 1) and zeros in the
 *     others; C[8 s + t][j] lands in lane (j, kg) with s = kg >> 1, t = 4 (kg & 1) + v. Eight tokens per pass.
 * The weights stay exact as in the Q4_K kernels; the intermediate arrives as bf16 head + tail. */
constexpr int kQ6KBlock = 210, kKqWalkGroups = 8;
constexpr uint32_t kNoChunk = 0xFFFFFFFFu;

/* n dwords from byte offset off (even) of an LDS area whose base is 16-byte aligned: aligned dword reads,
 * funnel-shifted by the two odd bytes if any */
template <int N>
__device__ __forceinline__ void lds_dwords_at(const uint8_t *base, int off, uint32_t (&out)[N]) {
    const uint32_t *q = reinterpret_cast<const uint32_t *>(base + (off & ~3));
    const uint32_t sh = (uint32_t)(off & 3) * 8u;
    uint32_t prev = q[0];
#pragma unroll
    for (int i = 0; i < N; i++) {
        const uint32_t next = q[i + 1];
        out[i] = __builtin_amdgcn_alignbit(next, prev, sh);
        prev = next;
    }
}

/* One Q6_K block of this lane's weight row (at byte blk_at of the image im) against NA activation operands
 * (a[p][u]: elements 32 u + 8 kg .. + 7 of the block, block-diagonal as described above): adds, for the
 * lane's scale groups kg >> 1 of the eight runs, d * sc * (S_lo + 16 S_hi - 32 X) to acc[v], token 4 (kg & 1) + v */
template <int NA>
__device__ __forceinline__ void q6k_block_math(const uint8_t *im, int blk_at, int kg, const u32x4 *const (&a)[NA], f32x4 &acc) {
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    uint32_t scw[5];
    lds_dwords_at<5>(im, blk_at + 192, scw); /* 16 int8 scales, then d */
    const float d = half_bits_fast(scw[4] & 0xFFFFu);
#pragma unroll
    for (int n = 0; n < 2; n++) {
        uint32_t qa[2], qb[2], qh[2]; /* ql[64n + 8kg ..], ql[64n + 32 + 8kg ..], qh[32n + 8kg ..] */
        lds_dwords_at<2>(im, blk_at + 64 * n + 8 * kg, qa);
        lds_dwords_at<2>(im, blk_at + 64 * n + 32 + 8 * kg, qb);
        lds_dwords_at<2>(im, blk_at + 128 + 32 * n + 8 * kg, qh);
#pragma unroll
        for (int qd = 0; qd < 4; qd++) {
            const int u = 4 * n + qd;
            const uint32_t l0 = ((qd & 1) ? qb[0] : qa[0]) >> (4 * (qd >> 1)), l1 = ((qd & 1) ? qb[1] : qa[1]) >> (4 * (qd >> 1));
            const bf16x8 lo = codes_to_bf16(l0 & 0x0F0F0F0Fu, l1 & 0x0F0F0F0Fu);
            const bf16x8 hi = codes_to_bf16((qh[0] >> (2 * qd)) & 0x03030303u, (qh[1] >> (2 * qd)) & 0x03030303u);
            f32x4 S_lo = zero, S_hi = zero, X = zero;
#pragma unroll
            for (int p = 0; p < NA; p++) {
                const bf16x8 av = __builtin_bit_cast(bf16x8, a[p][u]);
                S_lo = mma(av, lo, S_lo);
                S_hi = mma(av, hi, S_hi);
                X = mma(av, ones_bf16(), X);
            }
            /* this lane's scale group of the run: byte 8n + 2qd + (kg >> 1) of the 16 scales */
            const int sidx = 8 * n + 2 * qd;
            const uint32_t w = scw[sidx >> 2] >> (8 * (sidx & 3)); /* bytes sidx, sidx + 1 at bits 0..15 */
            const int sc = (int)(int8_t)((kg >> 1) ? (w >> 8) : w);
            const float dsc = d * (float)sc;
#pragma unroll
            for (int v = 0; v < 4; v++) acc[v] = fmaf(dsc, fmaf(16.0f, S_hi[v], S_lo[v]) - 32.0f * X[v], acc[v]);
        }
    }
}

/* The same for a Q5_K block (176 bytes, 16-byte aligned): code = nibble + 16 * high bit, one 6-bit scale and min
 * per 32 elements (common/ggml_dequant.h:1620-1651): (d sc) (S_lo + 16 S_hi) - (dmin m) X. Both scale groups
 * of a run share the sub-block's scale, so the block-diagonal operand only costs its eight-token passes. */
template <int NA>
__device__ __forceinline__ void q5k_block_math(const uint8_t *im, int blk_at, int kg, const u32x4 *const (&a)[NA], f32x4 &acc) {
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    const Scales sc = unpack_header(*(const u32x4 *)(im + blk_at));
    const u32x2 qh = *(const u32x2 *)(im + blk_at + 16 + 8 * kg); /* bit s of byte l: high bit of element l of sub-block s */
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const u32x2 qs = *(const u32x2 *)(im + blk_at + 48 + 32 * c + 8 * kg); /* sub-blocks 2c (low nibbles), 2c + 1 */
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int u = 2 * c + h;
            const bf16x8 lo = codes_to_bf16((qs.x >> (4 * h)) & 0x0F0F0F0Fu, (qs.y >> (4 * h)) & 0x0F0F0F0Fu);
            const bf16x8 hi = codes_to_bf16((qh.x >> u) & 0x01010101u, (qh.y >> u) & 0x01010101u);
            f32x4 S_lo = zero, S_hi = zero, X = zero;
#pragma unroll
            for (int p = 0; p < NA; p++) {
                const bf16x8 av = __builtin_bit_cast(bf16x8, a[p][u]);
                S_lo = mma(av, lo, S_lo);
                S_hi = mma(av, hi, S_hi);
                X = mma(av, ones_bf16(), X);
            }
            const uint32_t scw = (u < 4 ? sc.sc_lo : sc.sc_hi) >> (8 * (u & 3)), mnw = (u < 4 ? sc.mn_lo : sc.mn_hi) >> (8 * (u & 3));
            const float dsc = sc.d * (float)(scw & 0xFFu), dm = sc.dmin * (float)(mnw & 0xFFu);
#pragma unroll
            for (int v = 0; v < 4; v++) acc[v] = fmaf(dsc, fmaf(16.0f, S_hi[v], S_lo[v]), fmaf(-dm, X[v], acc[v]));
        }
    }
}

/* The same for eight Q8_0 blocks (256 elements, 8 x 34 = 272 bytes: a 16-byte multiple, but the codes of a
 * block start 2 bytes in): an int8 code is low nibble + 16 * (high nibble ^ 8) - 128 (the high nibble read as
 * signed, shifted to 0..15), one fp16 scale per 32 elements (common/ggml_dequant.h:1479-1489). */
template <int NA>
__device__ __forceinline__ void q8_0_block_math(const uint8_t *im, int blk_at, int kg, const u32x4 *const (&a)[NA], f32x4 &acc) {
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int u = 0; u < 8; u++) {
        uint32_t q[2];
        lds_dwords_at<2>(im, blk_at + 34 * u + 2 + 8 * kg, q);
        const float d = half_bits_fast(*reinterpret_cast<const uint16_t *>(im + blk_at + 34 * u));
        const bf16x8 lo = codes_to_bf16(q[0] & 0x0F0F0F0Fu, q[1] & 0x0F0F0F0Fu);
        const bf16x8 hi = codes_to_bf16(((q[0] >> 4) & 0x0F0F0F0Fu) ^ 0x08080808u, ((q[1] >> 4) & 0x0F0F0F0Fu) ^ 0x08080808u);
        f32x4 S_lo = zero, S_hi = zero, X = zero;
#pragma unroll
        for (int p = 0; p < NA; p++) {
            const bf16x8 av = __builtin_bit_cast(bf16x8, a[p][u]);
            S_lo = mma(av, lo, S_lo);
            S_hi = mma(av, hi, S_hi);
            X = mma(av, ones_bf16(), X);
        }
#pragma unroll
        for (int v = 0; v < 4; v++) acc[v] = fmaf(d, fmaf(16.0f, S_hi[v], S_lo[v]) - 128.0f * X[v], acc[v]);
    }
}

/* byte `i` (lane-variable, 0..11) of three dwords */
__device__ __forceinline__ uint32_t byte_of3(const uint32_t (&w)[3], int i) {
    const uint32_t d = i < 4 ? w[0] : i < 8 ? w[1] : w[2];
    return (d >> (8 * (i & 3))) & 255u;
}

/* Q2_K (84 bytes, 4-byte aligned): 2-bit codes, per 16 elements a 4-bit scale and a 4-bit min in one byte:
 * (d sc) q - dmin m (common/ggml_dequant.h:1495-1534) */
template <int NA>
__device__ __forceinline__ void q2k_block_math(const uint8_t *im, int blk_at, int kg, const u32x4 *const (&a)[NA], f32x4 &acc) {
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    uint32_t scw[4], dd[1];
    lds_dwords_at<4>(im, blk_at, scw);       /* 16 scale/min bytes */
    lds_dwords_at<1>(im, blk_at + 80, dd);   /* d, dmin */
    const float d = half_bits_fast(dd[0] & 0xFFFFu), dmin = half_bits_fast(dd[0] >> 16);
#pragma unroll
    for (int n = 0; n < 2; n++) {
        uint32_t q[2]; /* qs[32 n + 8 kg ..]: two bits per run j of the half */
        lds_dwords_at<2>(im, blk_at + 16 + 32 * n + 8 * kg, q);
#pragma unroll
        for (int jr = 0; jr < 4; jr++) {
            const int u = 4 * n + jr;
            const bf16x8 lo = codes_to_bf16((q[0] >> (2 * jr)) & 0x03030303u, (q[1] >> (2 * jr)) & 0x03030303u);
            f32x4 S = zero, X = zero;
#pragma unroll
            for (int p = 0; p < NA; p++) {
                const bf16x8 av = __builtin_bit_cast(bf16x8, a[p][u]);
                S = mma(av, lo, S);
                X = mma(av, ones_bf16(), X);
            }
            const int sidx = 8 * n + 2 * jr; /* + (kg >> 1): bytes sidx, sidx + 1 of the dword sidx / 4 */
            const uint32_t w = scw[sidx >> 2] >> (8 * (sidx & 3));
            const uint32_t sb = ((kg >> 1) ? (w >> 8) : w) & 255u;
            const float dl = d * (float)(sb & 15u), ml = dmin * (float)(sb >> 4);
#pragma unroll
            for (int v = 0; v < 4; v++) acc[v] = fmaf(dl, S[v], fmaf(-ml, X[v], acc[v]));
        }
    }
}

/* Q3_K (110 bytes): q = 2 low bits + 4 * mask bit - 4, a 6-bit scale (minus 32) per 16 elements packed into
 * 12 bytes (common/ggml_dequant.h:1536-1580): (d (sc - 32)) (S_lo + 4 S_hb - 4 X) */
template <int NA>
__device__ __forceinline__ void q3k_block_math(const uint8_t *im, int blk_at, int kg, const u32x4 *const (&a)[NA], f32x4 &acc) {
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    uint32_t scw4[4], hm[2];
    lds_dwords_at<4>(im, blk_at + 96, scw4); /* 12 scale bytes, d, two bytes beyond the block */
    const uint32_t scw[3] = {scw4[0], scw4[1], scw4[2]};
    const float d = half_bits_fast(scw4[3] & 0xFFFFu);
    lds_dwords_at<2>(im, blk_at + 8 * kg, hm); /* bit u of byte l: mask bit of element l of run u */
#pragma unroll
    for (int n = 0; n < 2; n++) {
        uint32_t q[2];
        lds_dwords_at<2>(im, blk_at + 32 + 32 * n + 8 * kg, q);
#pragma unroll
        for (int jr = 0; jr < 4; jr++) {
            const int u = 4 * n + jr;
            const bf16x8 lo = codes_to_bf16((q[0] >> (2 * jr)) & 0x03030303u, (q[1] >> (2 * jr)) & 0x03030303u);
            const bf16x8 hb = codes_to_bf16((hm[0] >> u) & 0x01010101u, (hm[1] >> u) & 0x01010101u);
            f32x4 S_lo = zero, S_hb = zero, X = zero;
#pragma unroll
            for (int p = 0; p < NA; p++) {
                const bf16x8 av = __builtin_bit_cast(bf16x8, a[p][u]);
                S_lo = mma(av, lo, S_lo);
                S_hb = mma(av, hb, S_hb);
                X = mma(av, ones_bf16(), X);
            }
            const int is = 2 * u + (kg >> 1);
            const uint32_t lo4 = (byte_of3(scw, is & 7) >> (4 * (is >> 3))) & 15u;
            const uint32_t hi2 = (byte_of3(scw, 8 + (is & 3)) >> (2 * (is >> 2))) & 3u;
            const float dl = d * (float)((int)(lo4 | (hi2 << 4)) - 32);
#pragma unroll
            for (int v = 0; v < 4; v++) acc[v] = fmaf(dl, fmaf(4.0f, S_hb[v], S_lo[v]) - 4.0f * X[v], acc[v]);
        }
    }
}

/* what the two kernels below need to know about a format */
struct KqQ6K {
    static constexpr int kBlock = kQ6KBlock, kRowChunks = 14;
    template <int NA> __device__ static void math(const uint8_t *im, int blk_at, int kg, const u32x4 *const (&a)[NA], f32x4 &acc) {
        q6k_block_math<NA>(im, blk_at, kg, a, acc);
    }
};
struct KqQ2K {
    static constexpr int kBlock = 84, kRowChunks = 6;
    template <int NA> __device__ static void math(const uint8_t *im, int blk_at, int kg, const u32x4 *const (&a)[NA], f32x4 &acc) {
        q2k_block_math<NA>(im, blk_at, kg, a, acc);
    }
};
struct KqQ3K {
    static constexpr int kBlock = 110, kRowChunks = 8;
    template <int NA> __device__ static void math(const uint8_t *im, int blk_at, int kg, const u32x4 *const (&a)[NA], f32x4 &acc) {
        q3k_block_math<NA>(im, blk_at, kg, a, acc);
    }
};
struct KqQ8_0 {
    static constexpr int kBlock = 272, kRowChunks = 17;
    template <int NA> __device__ static void math(const uint8_t *im, int blk_at, int kg, const u32x4 *const (&a)[NA], f32x4 &acc) {
        q8_0_block_math<NA>(im, blk_at, kg, a, acc);
    }
};
struct KqQ5K {
    static constexpr int kBlock = 176, kRowChunks = 11;
    template <int NA> __device__ static void math(const uint8_t *im, int blk_at, int kg, const u32x4 *const (&a)[NA], f32x4 &acc) {
        q5k_block_math<NA>(im, blk_at, kg, a, acc);
    }
};

template <typename F, int NT>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(3)))
moe_down_kq_walk_kernel(const uint8_t *__restrict__ down, const uint16_t *__restrict__ h_hi,
                         const uint16_t *__restrict__ h_lo, const int32_t *__restrict__ offsets,
                         float *__restrict__ part, int n_embd, int n_ff, const int32_t *__restrict__ routed) {
    constexpr int kImageRow = 16 * F::kRowChunks;
    constexpr int kImage = 16 * kImageRow + 16; /* + slack for the funnel-shift read past the last row */
    constexpr int kChunks = 16 * F::kRowChunks, kImageLoads = (kChunks + 63) / 64;
    extern __shared__ __attribute__((aligned(16))) float red[];
    const int e = block_expert(routed);
    if (e < 0) return;
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n_waves = blockDim.x >> 6;
    const int row0 = blockIdx.x * (16 * NT);
    const int first = offsets[e], cnt = offsets[e + 1] - first;
    if (cnt == 0) return;
    const int j = lane & 15, kg = lane >> 4;
    const int n_sb = n_ff >> 8; /* == n_waves: wave wv owns super-block wv */
    const int row_bytes = n_sb * F::kBlock;
    /* 16 * row_bytes is a multiple of 16, so every row group starts on a 16-byte boundary like the tensor */
    const uint8_t *d0 = down + ((size_t)e * n_embd + row0) * row_bytes;
    /* LDS: red [waves][8 tokens][16 rows] floats | images [waves][2][16 rows][224 bytes + slack] */
    uint8_t *img = reinterpret_cast<uint8_t *>(red + n_waves * 128) + wv * (2 * kImage);
    const uint32_t img_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)img;
    uint32_t off[kImageLoads];
#pragma unroll
    for (int i = 0; i < kImageLoads; i++) {
        const int t = 64 * i + lane;
        int R = t / F::kRowChunks;
        const int c = t - F::kRowChunks * R;
        R = R < 16 ? R : 15;
        const int at = R * row_bytes + wv * F::kBlock;
        /* a chunk that lies wholly behind the block is not read: behind the tensor's last block there may be nothing */
        off[i] = (t < kChunks && 16 * c < (at & 15) + F::kBlock) ? (uint32_t)(at & ~15) + 16u * (uint32_t)c : kNoChunk;
    }
    auto request = [&](int rt, int buf) {
        const uint8_t *base = uniform_ptr(d0 + (size_t)rt * 16 * row_bytes);
#pragma unroll
        for (int i = 0; i < kImageLoads; i++) {
            const uint32_t m0v = __builtin_amdgcn_readfirstlane(img_lds + (uint32_t)(buf * kImage) + 1024u * (uint32_t)i);
            if (off[i] != kNoChunk)
                asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(off[i]), "s"(base), "s"(m0v) : "memory");
        }
    };
    /* this lane's row j as a B lane: where its block starts inside its image row */
    const int blk_at = j * kImageRow + ((j * row_bytes + wv * F::kBlock) & 15);
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};

    for (int t0 = 0; t0 < cnt; t0 += 8) {
        const int n_live = cnt - t0 < 8 ? cnt - t0 : 8;
        /* A lane (i, kg): token i & 7 in the k groups of scale group i >> 3 */
        const int tok = j & 7;
        const bool live = (kg >> 1) == (j >> 3) && tok < n_live;
        const size_t at_a = (size_t)(first + t0 + (tok < n_live ? tok : 0)) * n_ff + (size_t)wv * 256 + 8 * kg;
        u32x4 a_hi[8], a_lo[8]; /* [run u]: elements 32 u + 8 kg .. + 7 of the wave's super-block */
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* reads of the previous pass's images have returned */
        request(0, 0);
#pragma unroll
        for (int u = 0; u < 8; u++) {
            u32x4 vh = {0u, 0u, 0u, 0u}, vl = {0u, 0u, 0u, 0u};
            if (live) {
                vh = *(const u32x4 *)(h_hi + at_a + 32 * u);
                vl = *(const u32x4 *)(h_lo + at_a + 32 * u);
            }
            a_hi[u] = vh;
            a_lo[u] = vl;
        }
#pragma unroll 1
        for (int rt = 0; rt < NT; rt++) {
            if (rt + 1 < NT) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* the other image has been read */
                request(rt + 1, (rt + 1) & 1);
                wait_vm_at_most(kImageLoads);
            } else {
                wait_vm_at_most(0);
            }
            const uint8_t *im = img + (rt & 1) * kImage;
            f32x4 acc = zero;
            const u32x4 *const aa[2] = {a_hi, a_lo};
            F::template math<2>(im, blk_at, kg, aa, acc);
            /* the two scale groups of every run sit in lanes kg and kg ^ 2 */
#pragma unroll
            for (int v = 0; v < 4; v++) acc[v] = add_lane32(acc[v]);
            if (kg < 2) {
#pragma unroll
                for (int v = 0; v < 4; v++) red[(wv * 8 + 4 * kg + v) * 16 + j] = acc[v];
            }
            __syncthreads();
            for (int idx = threadIdx.x; idx < n_live * 16; idx += blockDim.x) {
                const int jj = idx & 15, t = idx >> 4;
                float dsum = 0.0f;
                for (int w = 0; w < n_waves; w++) dsum += red[(w * 8 + t) * 16 + jj];
                part[(size_t)(first + t0 + t) * n_embd + row0 + rt * 16 + jj] = dsum;
            }
            __syncthreads();
        }
    }
}

/* ---- 3c. down for experts in those formats when K is longer than the walk's eight super-blocks (n_ff above 2048):
 * 16 rows per workgroup, K split over at most four waves (a wave takes super-blocks wv, wv + 4, ...), eight tokens
 * per pass, one image per wave ---- */
template <typename F>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3)))
moe_down_kq_long_kernel(const uint8_t *__restrict__ down, const uint16_t *__restrict__ h_hi,
                        const uint16_t *__restrict__ h_lo, const int32_t *__restrict__ offsets,
                        float *__restrict__ part, int n_embd, int n_ff, const int32_t *__restrict__ routed) {
    constexpr int kImageRow = 16 * F::kRowChunks;
    constexpr int kImage = 16 * kImageRow + 16;
    constexpr int kChunks = 16 * F::kRowChunks, kImageLoads = (kChunks + 63) / 64;
    extern __shared__ __attribute__((aligned(16))) float red[];
    const int e = block_expert(routed);
    if (e < 0) return;
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n_waves = blockDim.x >> 6;
    const int row0 = blockIdx.x * 16;
    const int first = offsets[e], cnt = offsets[e + 1] - first;
    if (cnt == 0) return;
    const int j = lane & 15, kg = lane >> 4;
    const int n_sb = n_ff >> 8;
    const int row_bytes = n_sb * F::kBlock;
    /* 16 * row_bytes is a multiple of 16, so every row group starts on a 16-byte boundary like the tensor */
    const uint8_t *w0 = uniform_ptr(down + ((size_t)e * n_embd + row0) * row_bytes);
    /* LDS: red [waves][8 tokens][16 rows] floats | images [waves][16 rows][chunks + slack] */
    uint8_t *img = reinterpret_cast<uint8_t *>(red + n_waves * 128) + wv * kImage;
    const uint32_t img_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)img;
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};

    for (int t0 = 0; t0 < cnt; t0 += 8) {
        const int n_live = cnt - t0 < 8 ? cnt - t0 : 8;
        const int tok = j & 7;
        const bool live = (kg >> 1) == (j >> 3) && tok < n_live;
        const size_t at_a = (size_t)(first + t0 + (tok < n_live ? tok : 0)) * n_ff + 8 * kg;
        f32x4 acc = zero;
        for (int sb = wv; sb < n_sb; sb += n_waves) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* reads of the previous image have returned */
#pragma unroll
            for (int i = 0; i < kImageLoads; i++) {
                const int t = 64 * i + lane;
                int R = t / F::kRowChunks;
                const int c = t - F::kRowChunks * R;
                R = R < 16 ? R : 15;
                const int at = R * row_bytes + sb * F::kBlock;
                const uint32_t off = (uint32_t)(at & ~15) + 16u * (uint32_t)c;
                /* a chunk that lies wholly behind the block is not read: behind the tensor's last block there may be nothing */
                const bool wanted = t < kChunks && 16 * c < (at & 15) + F::kBlock;
                const uint32_t m0v = __builtin_amdgcn_readfirstlane(img_lds + 1024u * (uint32_t)i);
                if (wanted)
                    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(off), "s"(w0), "s"(m0v) : "memory");
            }
            u32x4 a_hi[8], a_lo[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                u32x4 vh = {0u, 0u, 0u, 0u}, vl = {0u, 0u, 0u, 0u};
                if (live) {
                    vh = *(const u32x4 *)(h_hi + at_a + (size_t)sb * 256 + 32 * u);
                    vl = *(const u32x4 *)(h_lo + at_a + (size_t)sb * 256 + 32 * u);
                }
                a_hi[u] = vh;
                a_lo[u] = vl;
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* image and activations have landed */
            const int blk_at = j * kImageRow + ((j * row_bytes + sb * F::kBlock) & 15);
            const u32x4 *const aa[2] = {a_hi, a_lo};
            F::template math<2>(img, blk_at, kg, aa, acc);
        }
#pragma unroll
        for (int v = 0; v < 4; v++) acc[v] = add_lane32(acc[v]);
        if (kg < 2) {
#pragma unroll
            for (int v = 0; v < 4; v++) red[(wv * 8 + 4 * kg + v) * 16 + j] = acc[v];
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < n_live * 16; idx += blockDim.x) {
            const int jj = idx & 15, t = idx >> 4;
            float dsum = 0.0f;
            for (int w = 0; w < n_waves; w++) dsum += red[(w * 8 + t) * 16 + jj];
            part[(size_t)(first + t0 + t) * n_embd + row0 + jj] = dsum;
        }
        __syncthreads();
    }
}

/* ---- 2c. gate and up for Q6_K experts: 16 rows of each per workgroup, K split over at most four waves (a wave
 * takes super-blocks wv, wv + 4, ...), eight tokens per pass, the arithmetic of the Q6_K down kernel ---- */
template <typename F>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4)))
moe_gate_up_kq_kernel(const uint8_t *__restrict__ gate, const uint8_t *__restrict__ up,
                       const uint16_t *__restrict__ X, const int32_t *__restrict__ head,
                       const int32_t *__restrict__ order, uint16_t *__restrict__ h_hi, uint16_t *__restrict__ h_lo,
                       int n_embd, int n_ff, int top_k, const int32_t *__restrict__ routed) {
    constexpr int kImageRow = 16 * F::kRowChunks;
    constexpr int kImage = 16 * kImageRow + 16;
    constexpr int kChunks = 16 * F::kRowChunks, kImageLoads = (kChunks + 63) / 64;
    extern __shared__ __attribute__((aligned(16))) float red[];
    const int e = block_expert(routed);
    if (e < 0) return;
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n_waves = blockDim.x >> 6;
    const int row0 = blockIdx.x * 16;
    const int32_t *hd = head + (size_t)e * kHeadInts; /* first slot, count and the first 16 tokens in one line */
    const int first = hd[0], cnt = hd[1];
    if (cnt == 0) return;
    const int j = lane & 15, kg = lane >> 4;
    const int n_sb = n_embd >> 8;
    const int row_bytes = n_sb * F::kBlock;
    const size_t ebase = ((size_t)e * n_ff + row0) * row_bytes; /* a multiple of 16: row0 is */
    /* LDS: red [waves][gate, up][8 tokens][16 rows] floats | images [waves][gate, up][16 rows][224 bytes + slack] */
    uint8_t *img = reinterpret_cast<uint8_t *>(red + n_waves * 256) + wv * (2 * kImage);
    const uint32_t img_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)img;
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};

    for (int t0 = 0; t0 < cnt; t0 += 8) {
        const int n_live = cnt - t0 < 8 ? cnt - t0 : 8;
        const int tslot = j & 7;
        const bool live = (kg >> 1) == (j >> 3) && tslot < n_live;
        const int ts = t0 + (tslot < n_live ? tslot : 0);
        const int tok = ts < kHeadTokens ? hd[kHeadInts - kHeadTokens + ts] : order[first + ts] / top_k;
        const uint16_t *xrow = X + (size_t)tok * n_embd + 8 * kg;
        f32x4 acc_g = zero, acc_u = zero;
        for (int sb = wv; sb < n_sb; sb += n_waves) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* reads of the previous images have returned */
            const uint8_t *gb = uniform_ptr(gate + ebase), *ub = uniform_ptr(up + ebase);
#pragma unroll
            for (int i = 0; i < kImageLoads; i++) {
                const int t = 64 * i + lane;
                int R = t / F::kRowChunks;
                const int c = t - F::kRowChunks * R;
                R = R < 16 ? R : 15;
                const int at = R * row_bytes + sb * F::kBlock;
                const uint32_t off = (uint32_t)(at & ~15) + 16u * (uint32_t)c;
                const bool wanted = t < kChunks && 16 * c < (at & 15) + F::kBlock; /* not the chunk behind the block */
                const uint32_t m0g = __builtin_amdgcn_readfirstlane(img_lds + 1024u * (uint32_t)i);
                const uint32_t m0u = __builtin_amdgcn_readfirstlane(img_lds + (uint32_t)kImage + 1024u * (uint32_t)i);
                if (wanted) {
                    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(off), "s"(gb), "s"(m0g) : "memory");
                    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(off), "s"(ub), "s"(m0u) : "memory");
                }
            }
            u32x4 a[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                u32x4 v = {0u, 0u, 0u, 0u};
                if (live) v = *(const u32x4 *)(xrow + sb * 256 + 32 * u);
                a[u] = v;
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* images and activations have landed */
            const int blk_at = j * kImageRow + ((j * row_bytes + sb * F::kBlock) & 15);
            const u32x4 *const aa[1] = {a};
            F::template math<1>(img, blk_at, kg, aa, acc_g);
            F::template math<1>(img + kImage, blk_at, kg, aa, acc_u);
        }
#pragma unroll
        for (int v = 0; v < 4; v++) {
            acc_g[v] = add_lane32(acc_g[v]);
            acc_u[v] = add_lane32(acc_u[v]);
        }
        if (kg < 2) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                red[(wv * 2 + 0) * 128 + (4 * kg + v) * 16 + j] = acc_g[v];
                red[(wv * 2 + 1) * 128 + (4 * kg + v) * 16 + j] = acc_u[v];
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < n_live * 16; idx += blockDim.x) {
            const int jj = idx & 15, t = idx >> 4;
            float g = 0.0f, u = 0.0f;
            for (int w = 0; w < n_waves; w++) {
                g += red[(w * 2 + 0) * 128 + t * 16 + jj];
                u += red[(w * 2 + 1) * 128 + t * 16 + jj];
            }
            const float h = g / (1.0f + expf(-g)) * u; /* tf_silu_mul, common/transformer.h:4679-4694 */
            const __bf16 hh = (__bf16)h;
            const __bf16 hl = (__bf16)(h - (float)hh);
            const size_t at = (size_t)(first + t0 + t) * n_ff + row0 + jj;
            h_hi[at] = __builtin_bit_cast(uint16_t, hh);
            h_lo[at] = __builtin_bit_cast(uint16_t, hl);
        }
        __syncthreads();
    }
}

/* ---- 5b. dense GEMM for a handful of tokens in the formats of the kernels above ----
 * Y[t*ldy + r] = sum_k X[t*ldx + k] * decode(W)[r][k] for 16 rows per workgroup, K split over at most four waves,
 * eight tokens per pass, the weights exact: what a small batch of decode steps needs for a Q6_K, Q5_K, Q3_K, Q2_K
 * or Q8_0 tensor (decoding the whole tensor to bf16 for the library's GEMM costs more than streaming it a few
 * times). Rows past n_rows repeat the last row and are not stored. */
template <typename F, int NQ>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(NQ == 1 ? 4 : 2)))
gemm_kq_fewtok_kernel(const uint8_t *__restrict__ W, const uint16_t *__restrict__ X, float *__restrict__ Y, int n_rows,
                      int n_sb, int n_tok, int ldx, int ldy) {
    constexpr int kImageRow = 16 * F::kRowChunks;
    constexpr int kImage = 16 * kImageRow + 16;
    constexpr int kChunks = 16 * F::kRowChunks, kImageLoads = (kChunks + 63) / 64;
    constexpr int kPass = 8 * NQ; /* tokens per pass over the weights */
    extern __shared__ __attribute__((aligned(16))) float red[];
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n_waves = blockDim.x >> 6;
    const int row0 = blockIdx.x * 16;
    const int j = lane & 15, kg = lane >> 4;
    const int row_bytes = n_sb * F::kBlock;
    const int last = n_rows - 1 - row0; /* >= 0: the grid covers n_rows */
    /* LDS: red [waves][8 NQ tokens][16 rows] floats | images [waves][16 rows][chunks + slack] */
    uint8_t *img = reinterpret_cast<uint8_t *>(red + n_waves * (16 * kPass)) + wv * kImage;
    const uint32_t img_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)img;
    const uint8_t *w0 = uniform_ptr(W + (size_t)row0 * row_bytes); /* 16-byte aligned: row0 is a multiple of 16 */
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    const int jrow = j < last ? j : last;
    const int tslot = j & 7;
    const bool mine = (kg >> 1) == (j >> 3); /* the block-diagonal operand: scale group kg >> 1 in rows 8 (kg >> 1) .. + 7 */

    for (int t0 = 0; t0 < n_tok; t0 += kPass) {
        const int n_live = n_tok - t0 < kPass ? n_tok - t0 : kPass;
        const uint16_t *xrow[NQ];
        bool live[NQ];
        f32x4 acc[NQ];
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            live[q] = mine && 8 * q + tslot < n_live;
            xrow[q] = X + (size_t)(t0 + (8 * q + tslot < n_live ? 8 * q + tslot : 0)) * ldx + 8 * kg;
            acc[q] = zero;
        }
        for (int sb = wv; sb < n_sb; sb += n_waves) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* reads of the previous image have returned */
#pragma unroll
            for (int i = 0; i < kImageLoads; i++) {
                const int t = 64 * i + lane;
                int R = t / F::kRowChunks;
                const int c = t - F::kRowChunks * R;
                R = R < 16 ? R : 15;
                R = R < last ? R : last;
                const int at = R * row_bytes + sb * F::kBlock;
                const uint32_t off = (uint32_t)(at & ~15) + 16u * (uint32_t)c;
                const bool wanted = t < kChunks && 16 * c < (at & 15) + F::kBlock;
                const uint32_t m0v = __builtin_amdgcn_readfirstlane(img_lds + 1024u * (uint32_t)i);
                if (wanted)
                    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(off), "s"(w0), "s"(m0v) : "memory");
            }
            u32x4 a[NQ][8];
#pragma unroll
            for (int q = 0; q < NQ; q++) {
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    u32x4 v = {0u, 0u, 0u, 0u};
                    if (live[q]) v = *(const u32x4 *)(xrow[q] + sb * 256 + 32 * u);
                    a[q][u] = v;
                }
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* image and activations have landed */
            const int blk_at = j * kImageRow + ((jrow * row_bytes + sb * F::kBlock) & 15);
            /* one call per token group: the decode of the block is common to them */
#pragma unroll
            for (int q = 0; q < NQ; q++) {
                const u32x4 *const aa[1] = {a[q]};
                F::template math<1>(img, blk_at, kg, aa, acc[q]);
            }
        }
#pragma unroll
        for (int q = 0; q < NQ; q++) {
#pragma unroll
            for (int v = 0; v < 4; v++) acc[q][v] = add_lane32(acc[q][v]);
            if (kg < 2) {
#pragma unroll
                for (int v = 0; v < 4; v++) red[(wv * kPass + 8 * q + 4 * kg + v) * 16 + j] = acc[q][v];
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < n_live * 16; idx += blockDim.x) {
            const int jj = idx & 15, t = idx >> 4;
            float d = 0.0f;
            for (int w = 0; w < n_waves; w++) d += red[(w * kPass + t) * 16 + jj];
            if (row0 + jj < n_rows) Y[(size_t)(t0 + t) * ldy + row0 + jj] = d;
        }
        __syncthreads();
    }
}

/* ---- 4. out[t] = sum over k, in k order ---- */
__global__ void __launch_bounds__(256)
moe_combine_kernel(const float *__restrict__ part, const int32_t *__restrict__ slot_of,
                   const float *__restrict__ expert_w, float *__restrict__ out, int n_embd, int top_k) {
    const int t = blockIdx.x;
    const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 4;
    if (c >= n_embd) return;
    float4 s = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    /* eight experts at a time: their slots, then their rows, are requested together; the additions stay in k order */
    for (int k0 = 0; k0 < top_k; k0 += 8) {
        int slot[8];
        float wq[8];
        float4 p[8];
#pragma unroll
        for (int q = 0; q < 8; q++) {
            slot[q] = k0 + q < top_k ? slot_of[t * top_k + k0 + q] : -1;
            wq[q] = k0 + q < top_k ? expert_w[t * top_k + k0 + q] : 0.0f;
        }
#pragma unroll
        for (int q = 0; q < 8; q++)
            p[q] = slot[q] >= 0 ? *(const float4 *)(part + (size_t)slot[q] * n_embd + c) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
        for (int q = 0; q < 8; q++) {
            if (slot[q] >= 0) {
                /* out[i] += w * q (common/transformer.h:4116-4127): product rounded, then added */
                float4 m = make_float4(wq[q] * p[q].x, wq[q] * p[q].y, wq[q] * p[q].z, wq[q] * p[q].w);
                asm volatile("" : "+v"(m.x), "+v"(m.y), "+v"(m.z), "+v"(m.w)); /* keeps the products out of a fused multiply-add */
                s.x += m.x; s.y += m.y; s.z += m.z; s.w += m.w;
            }
        }
    }
    *(float4 *)(out + (size_t)t * n_embd + c) = s;
}

/* ---- 6. the expert matrices of any format: rows of one matrix for all tokens of an expert ----
 * A workgroup of four waves owns 16 rows of one expert. The activations of 8 of the expert's tokens
 * are staged in LDS as fp32, 1024 elements of K at a time; a wave then walks its 4 rows, decodes each
 * with the bit-exact codec (8 elements per lane and step) and dots it with the staged rows: what
 * tf_qmatvec_expert computes per token (common/transformer.h:517-548), grouped by expert so that a
 * row is decoded once per 8 tokens.
 * NX = 1: activations are the tokens' bf16 rows X[token] (gate, up); NX = 2: the bf16 head and tail
 * of the intermediate, by slot (down), and the result is scaled by the pair's routing weight. */
constexpr int kAnyRows = 16, kAnyTok = 8, kAnyChunk = 1024;

template <uint32_t T, int NX>
__global__ void __launch_bounds__(256)
moe_rows_any_kernel(const uint8_t *__restrict__ W, int rows_per_expert, int n_cols, size_t row_bytes,
                    const int32_t *__restrict__ offsets, const int32_t *__restrict__ order, int top_k,
                    const uint16_t *__restrict__ X0, const uint16_t *__restrict__ X1,
                    const float *__restrict__ w_slot, float *__restrict__ out) {
    using C = Codec<T>;
    constexpr int GPB = C::BE / 8, RW = kAnyRows / 4; /* rows per wave */
    static_assert(kAnyChunk % 256 == 0, "a chunk is a whole number of blocks of every format");
    extern __shared__ __attribute__((aligned(16))) float xs[]; /* [kAnyTok][chunk] */
    const int e = blockIdx.y;
    const int first = offsets[e], cnt = offsets[e + 1] - first;
    if (cnt == 0) return;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int row0 = blockIdx.x * kAnyRows + wv * RW;
    const int chunk = n_cols < kAnyChunk ? n_cols : kAnyChunk;
    const uint8_t *wrow[RW];
#pragma unroll
    for (int r = 0; r < RW; r++) {
        const int row = row0 + r < rows_per_expert ? row0 + r : rows_per_expert - 1;
        wrow[r] = W + ((size_t)e * rows_per_expert + row) * row_bytes;
    }
    for (int t0 = 0; t0 < cnt; t0 += kAnyTok) {
        const int n_live = cnt - t0 < kAnyTok ? cnt - t0 : kAnyTok;
        float acc[RW][kAnyTok];
#pragma unroll
        for (int r = 0; r < RW; r++)
#pragma unroll
            for (int t = 0; t < kAnyTok; t++) acc[r][t] = 0.0f;
        for (int c0 = 0; c0 < n_cols; c0 += chunk) {
            const int c_len = n_cols - c0 < chunk ? n_cols - c0 : chunk;
            __syncthreads(); /* the previous chunk has been consumed */
            /* stage: 8 elements per thread and step */
            for (int i = threadIdx.x; i < n_live * (c_len / 8); i += 256) {
                const int t = i / (c_len / 8), k8 = i - t * (c_len / 8);
                const int slot = first + t0 + t;
                const size_t src = (NX == 1 ? (size_t)(order[slot] / top_k) : (size_t)slot) * n_cols + c0 + 8 * k8;
                const uint4 a = *reinterpret_cast<const uint4 *>(X0 + src);
                const uint32_t av[4] = {a.x, a.y, a.z, a.w};
                float x[8];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    x[2 * q] = __uint_as_float(av[q] << 16);
                    x[2 * q + 1] = __uint_as_float(av[q] & 0xFFFF0000u);
                }
                if (NX == 2) {
                    const uint4 b = *reinterpret_cast<const uint4 *>(X1 + src);
                    const uint32_t bv[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        x[2 * q] += __uint_as_float(bv[q] << 16);
                        x[2 * q + 1] += __uint_as_float(bv[q] & 0xFFFF0000u);
                    }
                }
                float4 *dst = reinterpret_cast<float4 *>(xs + (size_t)t * chunk + 8 * k8);
                dst[0] = make_float4(x[0], x[1], x[2], x[3]);
                dst[1] = make_float4(x[4], x[5], x[6], x[7]);
            }
            __syncthreads();
            const int groups = c_len / 8, g0 = c0 / 8;
            for (int g = lane; g < groups; g += 64) {
                const int gg = g0 + g, blk = gg / GPB, k0 = (gg - blk * GPB) * 8;
                float w[RW][8];
#pragma unroll
                for (int r = 0; r < RW; r++) {
                    C::decode8(wrow[r] + (size_t)blk * C::BB, k0, w[r]);
                }
#pragma unroll
                for (int t = 0; t < kAnyTok; t++) {
                    if (t < n_live) { /* one read of the token's 8 activations serves the 4 rows */
                        const float4 xa = *reinterpret_cast<const float4 *>(xs + (size_t)t * chunk + 8 * g);
                        const float4 xb = *reinterpret_cast<const float4 *>(xs + (size_t)t * chunk + 8 * g + 4);
#pragma unroll
                        for (int r = 0; r < RW; r++) {
                            float a = acc[r][t];
                            a = fmaf(w[r][0], xa.x, a); a = fmaf(w[r][1], xa.y, a); a = fmaf(w[r][2], xa.z, a);
                            a = fmaf(w[r][3], xa.w, a); a = fmaf(w[r][4], xb.x, a); a = fmaf(w[r][5], xb.y, a);
                            a = fmaf(w[r][6], xb.z, a); a = fmaf(w[r][7], xb.w, a);
                            acc[r][t] = a;
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < RW; r++) {
#pragma unroll
            for (int t = 0; t < kAnyTok; t++) {
                if (t < n_live) { /* uniform over the wave: the reduction runs with all lanes */
                    const float sum = wave_sum_dpp(acc[r][t]);
                    if (lane == 0 && row0 + r < rows_per_expert) {
                        const int slot = first + t0 + t;
                        out[(size_t)slot * rows_per_expert + row0 + r] = w_slot ? w_slot[slot] * sum : sum;
                    }
                }
            }
        }
    }
}

/* h = silu(g) * u (tf_silu_mul, common/transformer.h:4679-4694) as a bf16 head and tail, by slot */
__global__ void __launch_bounds__(256)
moe_silu_split_kernel(const float *__restrict__ g32, const float *__restrict__ u32, uint16_t *__restrict__ h_hi,
                      uint16_t *__restrict__ h_lo, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float g = g32[i];
    const float h = g / (1.0f + expf(-g)) * u32[i];
    const __bf16 hi = (__bf16)h;
    const __bf16 lo = (__bf16)(h - (float)hi);
    h_hi[i] = __builtin_bit_cast(uint16_t, hi);
    h_lo[i] = __builtin_bit_cast(uint16_t, lo);
}

template <uint32_t T, int NX>
hipError_t launch_rows_any_typed(const void *W, int rows_per_expert, int n_cols, int n_expert, const Workspace &ws,
                                 int top_k, const uint16_t *X0, const uint16_t *X1, const float *w_slot, float *out,
                                 hipStream_t stream) {
    static OnceFlag lds_raised;
    const size_t lds = (size_t)kAnyTok * (n_cols < kAnyChunk ? n_cols : kAnyChunk) * sizeof(float);
    if (!lds_raised.is_set()) { /* 8 x 1024 floats = 32 KB: several workgroups per compute unit */
        hipError_t e = hipFuncSetAttribute((const void *)moe_rows_any_kernel<T, NX>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)((size_t)kAnyTok * kAnyChunk * sizeof(float)));
        if (e != hipSuccess) return e;
        lds_raised.set();
    }
    hipLaunchKernelGGL((moe_rows_any_kernel<T, NX>), dim3((rows_per_expert + kAnyRows - 1) / kAnyRows, n_expert), dim3(256),
                       lds, stream, (const uint8_t *)W, rows_per_expert, n_cols,
                       (size_t)(n_cols / Codec<T>::BE) * Codec<T>::BB, ws.offsets, ws.order, top_k, X0, X1, w_slot, out);
    return hipGetLastError();
}

template <int NX>
hipError_t launch_rows_any(uint32_t type, const void *W, int rows_per_expert, int n_cols, int n_expert,
                           const Workspace &ws, int top_k, const uint16_t *X0, const uint16_t *X1,
                           const float *w_slot, float *out, hipStream_t stream) {
    switch (type) {
#define QLIN_CASE(TT) \
    case TT: return launch_rows_any_typed<TT, NX>(W, rows_per_expert, n_cols, n_expert, ws, top_k, X0, X1, w_slot, out, stream);
    QLIN_FOR_EACH_BLOCK_TYPE(QLIN_CASE)
    QLIN_FOR_EACH_DENSE_TYPE(QLIN_CASE)
#undef QLIN_CASE
    default: return hipErrorInvalidValue;
    }
}

/* ---- 5. dense GEMM for a handful of tokens on the same machinery ----
 * Y[t*ldy + r] = sum_k X[t*ldx + k] * decode(W)[r][k] for RT * 16 rows per workgroup and 16 tokens at a
 * time: one "expert" with every token routed to it. The weights stay exact (4-bit codes through the
 * matrix instruction, block scales applied in fp32), so this path is closer to the oracle than the
 * bf16-weights tile kernel; it streams the weights once per 16 tokens, which is what a few tokens need
 * (common/transformer.h:4535-4572 decodes a row and dots it with every token). */
template <int RT>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2)))
gemm_q4k_fewtok_kernel(const uint8_t *__restrict__ W, const uint16_t *__restrict__ X, float *__restrict__ Y,
                       int n_rows, int n_sb, int n_tok, int ldx, int ldy) {
    constexpr int kRows = 16 * RT;
    extern __shared__ __attribute__((aligned(16))) float red[];
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n_waves = blockDim.x >> 6;
    const int row0 = blockIdx.x * kRows;
    const int j = lane & 15;
    const size_t row_bytes = (size_t)n_sb * kQ4KBlock;
    const uint8_t *w0 = W + (size_t)row0 * row_bytes;
    const int last_row = n_rows - 1 - row0; /* >= 0: the grid covers n_rows */
    /* LDS: red [waves][RT][64][4] floats | images [waves][RT * 16 rows][144 bytes] */
    uint8_t *img = reinterpret_cast<uint8_t *>(red + n_waves * RT * 256) + wv * (kRows * kQ4KBlock);
    const bool one_sb = n_sb <= n_waves;
    ImagePlan<RT, 1> plan;
    plan_image(plan, row_bytes, lane, last_row);
    if (one_sb && wv < n_sb) image_from_global(img, w0, w0, plan, wv, lane);

    for (int t0 = 0; t0 < n_tok; t0 += 16) {
        const bool live = t0 + j < n_tok;
        const uint16_t *const arow[1] = {X + (size_t)(live ? t0 + j : 0) * ldx};
        ksplit_tile<RT, 1, 1>(img, w0, w0, plan, arow, n_sb, wv, n_waves, lane, live, one_sb ? wv : -1, red);
        __syncthreads();
        for (int idx = threadIdx.x; idx < live_slots(n_tok, t0) * 16 * RT; idx += blockDim.x) {
            const TileElem t = tile_elem<RT>(idx);
            float d = 0.0f;
            for (int w = 0; w < n_waves; w++) d += red[((w * RT + t.r) * 64 + t.lane) * 4 + t.v];
            if (row0 + t.row < n_rows) Y[(size_t)(t0 + t.slot) * ldy + row0 + t.row] = d;
        }
        __syncthreads();
    }
}

}  // namespace

hipError_t launch_gemm_q4k_fewtok(const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok,
                                  int ldx, int ldy, hipStream_t stream) {
    /* 32 rows and 4 waves per workgroup measured best at 14336 x 4096 (12.8 us for one token, 14.8 for
     * 16, 27 for 32); 16 rows: 21 us at 16 tokens, 64 rows: 15.5 us at one, 8 waves: +1 us from 16 tokens on */
    constexpr int RT = 2;
    const int n_sb = n_cols / 256;
    const int waves = n_sb < 4 ? n_sb : 4;
    const int grid = (n_rows + 16 * RT - 1) / (16 * RT);
    hipLaunchKernelGGL(gemm_q4k_fewtok_kernel<RT>, dim3(grid), dim3(64 * waves),
                       (size_t)waves * RT * (1024 + 16 * kQ4KBlock), stream, (const uint8_t *)W, X, Y, n_rows, n_sb,
                       n_tok, ldx, ldy);
    return hipGetLastError();
}

/* formats whose experts run on the matrix cores through moe_gate_up_kq_kernel / moe_down_kq_walk_kernel */
static bool kq_type(uint32_t t) { return t == T_Q6_K || t == T_Q5_K || t == T_Q3_K || t == T_Q2_K || t == T_Q8_0; }

bool launch_gemm_kq_fewtok(uint32_t type, const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok,
                           int ldx, int ldy, hipStream_t stream, hipError_t *err) {
    *err = hipSuccess;
    if (!kq_type(type) || n_cols % 256 != 0 || n_tok > kKqFewTokens || ((uintptr_t)W & 15) || ((uintptr_t)X & 15) || (ldx & 7))
        return false;
    const int n_sb = n_cols / 256;
    const int waves = n_sb < 4 ? n_sb : 4;
    auto go = [&](auto tag) {
        using F = decltype(tag);
        /* the tensor has to end on a 16-byte boundary: the image of its last block is whole chunks */
        if (((size_t)n_rows * n_sb * F::kBlock) & 15) return false;
        const dim3 grid((n_rows + 15) / 16), block(64 * waves);
        const size_t image = (size_t)waves * (16 * 16 * F::kRowChunks + 16);
        const uint8_t *Wb = (const uint8_t *)W;
        /* 8, 16 or 24 tokens per pass over the weights */
        if (n_tok <= 8)
            hipLaunchKernelGGL((gemm_kq_fewtok_kernel<F, 1>), grid, block, waves * 512 + image, stream, Wb, X, Y, n_rows, n_sb, n_tok, ldx, ldy);
        else if (n_tok <= 16)
            hipLaunchKernelGGL((gemm_kq_fewtok_kernel<F, 2>), grid, block, waves * 1024 + image, stream, Wb, X, Y, n_rows, n_sb, n_tok, ldx, ldy);
        else
            hipLaunchKernelGGL((gemm_kq_fewtok_kernel<F, 3>), grid, block, waves * 1536 + image, stream, Wb, X, Y, n_rows, n_sb, n_tok, ldx, ldy);
        *err = hipGetLastError();
        return true;
    };
    switch (type) {
    case T_Q6_K: return go(KqQ6K());
    case T_Q5_K: return go(KqQ5K());
    case T_Q3_K: return go(KqQ3K());
    case T_Q2_K: return go(KqQ2K());
    default: return go(KqQ8_0());
    }
}

size_t moe_workspace_bytes(int n_tok, int top_k, int n_embd, int n_ff, int n_expert) {
    return carve(nullptr, n_tok, top_k, n_embd, n_ff, n_expert).bytes;
}

hipError_t launch_moe_ffn(uint32_t type_gate, uint32_t type_up, uint32_t type_down, const void *gate, const void *up,
                          const void *down, const uint16_t *X, const int32_t *idx, const float *w, float *out, int n_tok,
                          int top_k, int n_embd, int n_ff, int n_expert, int n_cu, void *workspace, hipStream_t stream) {
    const Workspace ws = carve(workspace, n_tok, top_k, n_embd, n_ff, n_expert);
    const int n_pairs = n_tok * top_k;
    /* One token (the reference's own case), or up to eight that will mostly meet different experts (two pairs or
     * fewer per four experts): each token on its own through two launches of the Q4_K matvec, no grouping and no
     * combine. 128 experts of 768 x 2048, top-8, us: 1 token 19.9 -> 10.6, 2: 24.3 -> 13.5, 4: 33.5 -> 19.2,
     * 8: 49.1 -> 37.6; at 12 tokens (76.9 against 61.0) the experts that tokens share are read once per token too often.
     * Q4_K experts on the Q4_K matvec, the other common expert formats on the matrix-instruction matvec (gate and up of
     * one type; 1 token: Q4_K/Q4_K/Q6_K 21.6 -> 13.5, Q6_K 25.9 -> 15.7, Q8_0 26.0 -> 13.2, IQ4_XS 62.7 -> 12.4). */
    if (n_tok == 1 || (n_tok <= 8 && 2 * n_pairs <= n_expert)) {
        hipError_t e1 = hipSuccess;
        auto up_step = [&](bool dry) {
            if (type_gate == T_Q4_K && type_up == T_Q4_K)
                return launch_moe1_q4k_up(gate, up, X, idx, ws.g32, n_tok, top_k, n_embd, n_ff, n_expert, n_cu, stream, dry, &e1);
            return type_gate == type_up &&
                   launch_moe1_grid_up(type_gate, gate, up, X, idx, ws.g32, n_tok, top_k, n_embd, n_ff, n_expert, n_cu, stream, dry, &e1);
        };
        auto down_step = [&](bool dry) {
            if (type_down == T_Q4_K)
                return launch_moe1_q4k_down(down, ws.g32, idx, w, out, n_tok, top_k, n_embd, n_ff, n_expert, n_cu, stream, dry, &e1);
            return launch_moe1_grid_down(type_down, down, ws.g32, idx, w, out, n_tok, top_k, n_embd, n_ff, n_expert, n_cu, stream, dry, &e1);
        };
        if (up_step(true) && down_step(true)) {
            up_step(false);
            if (e1 != hipSuccess) return e1;
            down_step(false);
            return e1;
        }
    }
    /* few pairs per expert: the matrix kernels look their expert up in the list of those that have tokens, and
     * the launch covers no more experts than there are pairs */
    /* up to two pairs per expert (a third or more of the experts unused at random routing): measured faster or equal
     * up to there (128 experts, top-8: 1 token 39.9 -> 22.7 us, 8 tokens 59.8 -> 48.6, 32 tokens 92.9 -> 90.7) */
    const bool compact = n_pairs <= 2 * n_expert;
    const int32_t *routed = compact ? ws.head : nullptr;
    const int grid_y = routed && n_pairs < n_expert ? n_pairs : n_expert;
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), ((size_t)n_expert * 2 + 32) * sizeof(int32_t), stream, idx,
                       n_pairs, n_expert, ws.offsets, ws.order, ws.slot_of, ws.head, top_k);
    static OnceFlag lds_raised;
    if (!lds_raised.is_set()) {
        hipError_t e1 = hipFuncSetAttribute((const void *)moe_gate_up_kernel<kGuRowTiles>,
                                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e1 != hipSuccess) return e1;
        lds_raised.set();
    }
    /* Q4_K matrices take the matrix-core kernels; any other format (or a shape their tiles do not divide)
     * the any-format kernel, matrix by matrix: gate and up -> fp32 by slot -> silu(g)*u as head + tail */
    const bool fast_gu = type_gate == T_Q4_K && type_up == T_Q4_K && n_embd % 256 == 0 && n_ff % (16 * kGuRowTiles) == 0;
    const bool fast_dn = type_down == T_Q4_K && n_ff % 256 == 0 && n_embd % (16 * kDnRowTiles) == 0;
    /* waves per workgroup = super-blocks of K, at most 4 for gate/up (a wave then walks several
     * super-blocks one after the other) and 8 for down. The gate/up kernel needs 138 registers, so a
     * compute unit holds 12 of its waves: three 4-wave workgroups in different phases instead of one
     * 8-wave workgroup that loads, computes and reduces with nothing beside it (75 -> 65 us). */
    const int gu_waves = n_embd / 256 < kGuWgWaves ? n_embd / 256 : kGuWgWaves, dn_waves = n_ff / 256 < 8 ? n_ff / 256 : 8;
    if (fast_gu) {
        constexpr int RT = kGuRowTiles;
        hipLaunchKernelGGL(moe_gate_up_kernel<RT>, dim3(n_ff / (16 * RT), grid_y), dim3(64 * gu_waves),
                           (size_t)gu_waves * 2 * RT * (1024 + 16 * kQ4KBlock + 256), stream,
                           (const uint8_t *)gate, (const uint8_t *)up, X, ws.head, ws.order, ws.h_hi, ws.h_lo, n_embd,
                           n_ff, top_k, routed);
    } else if (type_gate == type_up && kq_type(type_gate) && n_embd % 256 == 0 && n_ff % 16 == 0 &&
               (((uintptr_t)gate | (uintptr_t)up) & 15) == 0) {
        const int waves = n_embd / 256 < 4 ? n_embd / 256 : 4;
        auto go = [&](auto tag) {
            using F = decltype(tag);
            hipLaunchKernelGGL(moe_gate_up_kq_kernel<F>, dim3(n_ff / 16, grid_y), dim3(64 * waves),
                               (size_t)waves * (256 * 4 + 2 * (16 * 16 * F::kRowChunks + 16)), stream, (const uint8_t *)gate,
                               (const uint8_t *)up, X, ws.head, ws.order, ws.h_hi, ws.h_lo, n_embd, n_ff, top_k, routed);
        };
        switch (type_gate) {
        case T_Q6_K: go(KqQ6K()); break;
        case T_Q5_K: go(KqQ5K()); break;
        case T_Q3_K: go(KqQ3K()); break;
        case T_Q2_K: go(KqQ2K()); break;
        default: go(KqQ8_0()); break;
        }
    } else {
        hipError_t e1 = launch_rows_any<1>(type_gate, gate, n_ff, n_embd, n_expert, ws, top_k, X, nullptr, nullptr, ws.g32, stream);
        if (e1 != hipSuccess) return e1;
        e1 = launch_rows_any<1>(type_up, up, n_ff, n_embd, n_expert, ws, top_k, X, nullptr, nullptr, ws.u32, stream);
        if (e1 != hipSuccess) return e1;
        const size_t n = (size_t)n_pairs * n_ff;
        hipLaunchKernelGGL(moe_silu_split_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, ws.g32, ws.u32,
                           ws.h_hi, ws.h_lo, n);
    }
    /* a handful of routed experts: the walk's 128-row workgroups would leave most compute units idle */
    const bool few_tiles = routed && (long long)grid_y * (n_embd / (16 * kDnRowTiles * kDnColTiles)) < 512;
    if (fast_dn && n_ff / 256 <= dn_waves && n_embd % (16 * kDnRowTiles * kDnColTiles) == 0 && !few_tiles) {
        constexpr int DRT = kDnRowTiles, DNT = kDnColTiles;
        static OnceFlag walk_lds_raised;
        if (!walk_lds_raised.is_set()) { /* 8 waves: 90 KB */
            hipError_t e1 = hipFuncSetAttribute((const void *)moe_down_walk_kernel<DRT, DNT>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e1 != hipSuccess) return e1;
            walk_lds_raised.set();
        }
        hipLaunchKernelGGL((moe_down_walk_kernel<DRT, DNT>), dim3(n_embd / (16 * DRT * DNT), grid_y), dim3(64 * dn_waves),
                           (size_t)dn_waves * DRT * (1024 + 2 * 16 * kQ4KBlock), stream,
                           (const uint8_t *)down, ws.h_hi, ws.h_lo, ws.offsets, ws.part, n_embd, n_ff, routed);
    } else if (!fast_dn && !few_tiles && kq_type(type_down) && n_ff % 256 == 0 && n_ff / 256 <= 8 &&
               n_embd % (16 * kKqWalkGroups) == 0 && ((uintptr_t)down & 15) == 0) {
        const int waves = n_ff / 256;
        auto go = [&](auto tag) {
            using F = decltype(tag);
            hipLaunchKernelGGL((moe_down_kq_walk_kernel<F, kKqWalkGroups>), dim3(n_embd / (16 * kKqWalkGroups), grid_y),
                               dim3(64 * waves), (size_t)waves * (128 * 4 + 2 * (16 * 16 * F::kRowChunks + 16)), stream,
                               (const uint8_t *)down, ws.h_hi, ws.h_lo, ws.offsets, ws.part, n_embd, n_ff, routed);
        };
        switch (type_down) {
        case T_Q6_K: go(KqQ6K()); break;
        case T_Q5_K: go(KqQ5K()); break;
        case T_Q3_K: go(KqQ3K()); break;
        case T_Q2_K: go(KqQ2K()); break;
        default: go(KqQ8_0()); break;
        }
    } else if (!fast_dn && kq_type(type_down) && n_ff % 256 == 0 && n_embd % 16 == 0 && ((uintptr_t)down & 15) == 0) {
        const int waves = n_ff / 256 < 4 ? n_ff / 256 : 4;
        auto go = [&](auto tag) {
            using F = decltype(tag);
            hipLaunchKernelGGL((moe_down_kq_long_kernel<F>), dim3(n_embd / 16, grid_y), dim3(64 * waves),
                               (size_t)waves * (128 * 4 + 16 * 16 * F::kRowChunks + 16), stream, (const uint8_t *)down, ws.h_hi,
                               ws.h_lo, ws.offsets, ws.part, n_embd, n_ff, routed);
        };
        switch (type_down) {
        case T_Q6_K: go(KqQ6K()); break;
        case T_Q5_K: go(KqQ5K()); break;
        case T_Q3_K: go(KqQ3K()); break;
        case T_Q2_K: go(KqQ2K()); break;
        default: go(KqQ8_0()); break;
        }
    } else if (fast_dn) {
        constexpr int DRT = kDnRowTiles;
        hipLaunchKernelGGL(moe_down_kernel<DRT>, dim3(n_embd / (16 * DRT), grid_y), dim3(64 * dn_waves),
                           (size_t)dn_waves * DRT * (1024 + 16 * kQ4KBlock), stream,
                           (const uint8_t *)down, ws.h_hi, ws.h_lo, ws.offsets, ws.part, n_embd, n_ff, routed);
    } else {
        hipError_t e1 = launch_rows_any<2>(type_down, down, n_embd, n_ff, n_expert, ws, top_k, ws.h_hi, ws.h_lo, nullptr,
                                           ws.part, stream);
        if (e1 != hipSuccess) return e1;
    }
    hipLaunchKernelGGL(moe_combine_kernel, dim3(n_tok, (n_embd / 4 + 63) / 64), dim3(64), 0, stream, ws.part,
                       ws.slot_of, w, out, n_embd, top_k);
    return hipGetLastError();
}

/* ---- scratch of the entry point that allocates nothing (qlin_moe_ffn_static_dev): the workspace of
 * launch_moe_ffn as a file-scope device array. Every GPU the library's code object is loaded on holds its
 * own copy at its own address until the process ends; host code never uses the array's name as an address,
 * only what hipGetSymbolAddress returned for the device that was current. */
static __device__ __align__(256) unsigned char scratch[kMoeStaticScratchBytes];
static void *g_scratch_ptr[kMaxScratchDevices]; /* written under the caller's lock, once per device */

hipError_t moe_static_scratch_setup(int device) {
    if (device < 0 || device >= kMaxScratchDevices) return hipErrorInvalidDevice;
    if (g_scratch_ptr[device]) return hipSuccess;
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_scratch_ptr[device] = p;
    return hipSuccess;
}

hipError_t launch_moe_ffn_static(uint32_t type_gate, uint32_t type_up, uint32_t type_down, const void *gate,
                                 const void *up, const void *down, const uint16_t *X, const int32_t *idx, const float *w,
                                 float *out, int n_tok, int top_k, int n_embd, int n_ff, int n_expert, int device,
                                 int n_cu, hipStream_t stream) {
    if (device < 0 || device >= kMaxScratchDevices || !g_scratch_ptr[device]) return hipErrorNotInitialized;
    if (moe_workspace_bytes(n_tok, top_k, n_embd, n_ff, n_expert) > kMoeStaticScratchBytes) return hipErrorInvalidValue;
    /* nothing in the workspace has to start at zero: the grouping kernel writes every offset, slot and weight
     * it later reads, and the expert kernels write every slot row the combine step reads */
    return launch_moe_ffn(type_gate, type_up, type_down, gate, up, down, X, idx, w, out, n_tok, top_k, n_embd, n_ff,
                          n_expert, n_cu, g_scratch_ptr[device], stream);
}

}  // namespace qlin
