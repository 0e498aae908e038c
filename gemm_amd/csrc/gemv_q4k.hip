/*
 * gemv_q4k.hip - batch-1 Q4_K matvec for gfx950: inner products on the 8-bit integer matrix
 * instruction, weights read straight from HBM in the operand layout (no LDS staging).
 *
 * y[r] = sum over super-blocks of d*sum_s sc_s*(q_s . x_s) - dmin*sum_s m_s*sum(x_s)
 * (the factored form of common/ggml_dequant.h:1592-1618 dotted with x; sub-block s = 32 elements,
 * 6-bit sc/m from get_scale_min_k4, :1582-1590).
 *
 *  1. x -> fixed point per 32-element sub-block: X = rint(x * 2^(30-e)), e the exponent of the
 *     sub-block's largest |x|, written as four SIGNED base-256 digits (top in [-64,64], the others in
 *     [-128,127]). q_s . x_s = 2^(e-30) * sum_k 256^k * D_k with D_k the exact integer inner products of
 *     the 4-bit codes with the digit planes. An element keeps all 24 bits of its significand unless it
 *     is more than 2^7 times smaller than the largest of its sub-block; the error is at most 2^-31 of
 *     that largest |x| per element, so an outlier 10^5 times the bulk still leaves its 31 neighbours
 *     14 bits.
 *  2. The inner products run on v_mfma_i32_16x16x64_i8: 16 weight rows (B operand: the codes, one
 *     byte each) against 16 "x rows" (A operand). Wave w of a 16-wave workgroup owns super-block w
 *     (w+16, w+32, w+48 for longer rows) of every row, so it prepares only ITS 256 elements of x - one
 *     16-byte load per lane, no workgroup-wide x pass, no barrier before the weights are requested.
 *     Per super-block two chains of two instructions: chain p covers the 64 code bytes [64p, 64p+64)
 *     = sub-blocks 4p..4p+3; lane group g = lane/16 supplies 16 of those bytes, low nibbles in operand
 *     registers 0-1, high nibbles in 2-3. The A operand is block-diagonal to match: x-row 4*s'+digit
 *     (s' = 0..3, digit 3..0) holds the digits of sub-block 4p+s' at exactly the k positions
 *     that carry that sub-block's codes and zeros elsewhere, so result register r of lane group s' is
 *     digit plane r of sub-block 4p+s' for weight row lane%16: all 16 x-rows and all 64 lanes are used
 *     (2 shift-adds, 2 converts, 4 multiply-adds per sub-block and row). About 60 vector instructions per
 *     (16 rows x super-block) instead of the ~150 per row of a v_dot4 formulation.
 *  3. Lane (n, g) loads the header and its two 16-byte code chunks of row 16*rg + n directly from HBM:
 *     per instruction 16 rows x 64 contiguous bytes. One row group (3 loads) is in flight per wave - the
 *     sixteen waves of a compute unit keep the requests coming, and a wave that requested several row groups
 *     together measured slower; waves never wait for each other until the final sum over the 16
 *     super-block shares of a row, which meets in LDS. A workgroup takes up to 640 rows (one workgroup per
 *     compute unit up to 163840 rows, equal rounds of them beyond).
 *
 * Measured alternatives on this part (14336x4096, period per launch; a bare read of the same bytes with
 * contiguous 1 KB-per-instruction loads is 6.2 us, with this kernel's access pattern 7.3 us): rows copied
 * to LDS by global_load_lds as contiguous streams with 16-row tiles handed over by workgroup barriers
 * 10.3-11.2 us (waves stuck in issue reach the barrier late, and LDS instructions of other waves slow
 * the incoming copy stream); dedicated copying waves that publish their progress in LDS 10.4 us; each
 * wave gathering its own 144-byte blocks into LDS 16 us (a gather of short runs costs one access per
 * lane); a v_dot4 kernel with one row per wave in LDS 8.3-8.6 us, against 7.9-8.4 us for this one, which needs a
 * third of the vector instructions and no LDS for the weights.
 *
 * A non-finite x makes every output NaN (the fixed-point form cannot carry Inf).
 */
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWaves = 16;             /* wavefronts per workgroup */
constexpr int kMaxKc = 4;               /* 16-super-block column chunks: K <= 16384 */
constexpr int kMaxRowsPerWg = 640;      /* local rows (both matrices of a gate+up pair): 40 KB of partial sums */
constexpr int kXScratch = 1088;         /* per wave: 4 digit planes x 256 B + 8 x (2^(e-30), sum) */
/* x operand of one super-block: A[2p+h] for chain p, instruction h; scale[p] = 2^(e-30) and
 * sum[p] = sum of x for sub-block 4p + lane/16 */
struct XOperand {
    v4i A[4];
    float scale[2], sum[2];
};

/* x -> signed digit planes -> A operands, wave-private (xs: the wave's kXScratch bytes of LDS) */
__device__ __forceinline__ void q4k_prepare(v4f v, XOperand &xo, uint8_t *xs, int lane) {
    const int n = lane & 15, g = lane >> 4;
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    float sum = (v.x + v.y) + (v.z + v.w);
    /* 8 consecutive lanes share one 32-element sub-block */
    amax = fmaxf(amax, dpp_mov<0xB1>(amax));
    amax = fmaxf(amax, dpp_mov<0x4E>(amax));
    amax = fmaxf(amax, dpp_mov<0x141>(amax));
    sum += dpp_mov<0xB1>(sum);
    sum += dpp_mov<0x4E>(sum);
    sum += dpp_mov<0x141>(sum);
    int e = (int)(__float_as_uint(amax) >> 23) - 126; /* amax in [2^(e-1), 2^e) */
    if (e < -96) e = -96;                              /* zero and tiny sub-blocks */
    const float up = __uint_as_float((uint32_t)(127 + 30 - e) << 23);
    float down = __uint_as_float((uint32_t)(127 - 30 + e) << 23);
    if (!(amax <= 3.0e38f)) down = __uint_as_float(0x7FC00000u); /* Inf/NaN in x: poison every row */
    const int X[4] = {__float2int_rn(v.x * up), __float2int_rn(v.y * up), __float2int_rn(v.z * up),
                      __float2int_rn(v.w * up)};
    /* The four signed base-256 digits of X (X = 256*X1 + d0 with d0 = (int8)X, X1 = 256*X2 + d1, ...;
     * the top one in [-64, 64]) are the bytes of (X + 0x00808080) ^ 0x00808080: adding 128 at a byte makes its
     * digit unsigned and carries exactly when the digit is negative, the xor takes the 128 off again. */
    uint32_t Z[4];
#pragma unroll
    for (int k = 0; k < 4; k++) Z[k] = ((uint32_t)X[k] + 0x00808080u) ^ 0x00808080u;
    /* byte transpose: plane j = byte j of Z[0..3] (selector 0-3: second operand, 4-7: first) */
    const uint32_t lo01 = __builtin_amdgcn_perm(Z[1], Z[0], 0x05010400u), lo23 = __builtin_amdgcn_perm(Z[3], Z[2], 0x05010400u);
    const uint32_t hi01 = __builtin_amdgcn_perm(Z[1], Z[0], 0x07030602u), hi23 = __builtin_amdgcn_perm(Z[3], Z[2], 0x07030602u);
    uint32_t *pl = reinterpret_cast<uint32_t *>(xs);
    pl[lane] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);       /* digit 3 (top) */
    pl[64 + lane] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);  /* digit 2 */
    pl[128 + lane] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u); /* digit 1 */
    pl[192 + lane] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u); /* digit 0 */
    if ((lane & 7) == 0) reinterpret_cast<float2 *>(xs + 1024)[lane >> 3] = make_float2(down, sum);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    /* A operand: x-row i = lane%16 = 4*s' + plane; k group lane/16 carries sub-blocks 2*(g>>1)
     * (registers 0-1) and 2*(g>>1)+1 (registers 2-3) of the chain, elements 16*(g&1) + 8h .. +7 */
    const int sq = n >> 2, plane = n & 3;
    const bool live = (g >> 1) == (sq >> 1);
    const uint8_t *src = xs + plane * 256 + 32 * sq + 16 * (g & 1);
#pragma unroll
    for (int p = 0; p < 2; p++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint2 d = *reinterpret_cast<const uint2 *>(src + 128 * p + 8 * h);
            const bool lo = live && !(sq & 1), hi = live && (sq & 1);
            v4i a;
            a.x = lo ? (int)d.x : 0;
            a.y = lo ? (int)d.y : 0;
            a.z = hi ? (int)d.x : 0;
            a.w = hi ? (int)d.y : 0;
            xo.A[2 * p + h] = a;
        }
#pragma unroll
    for (int p = 0; p < 2; p++) {
        const float2 m = reinterpret_cast<const float2 *>(xs + 1024)[4 * p + g];
        xo.scale[p] = m.x;
        xo.sum[p] = m.y;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

/* one super-block of 16 rows: header hh, code bytes qa (chain 0) and qb (chain 1) of this lane; g = lane / 16 */
__device__ __forceinline__ float q4k_item(const XOperand &xo, const uint4 hh, const uint4 qa, const uint4 qb, int g) {
    constexpr uint32_t M = 0x0F0F0F0Fu;
    v4i c0 = {0, 0, 0, 0}, c1 = {0, 0, 0, 0};
    v4i b;
    b.x = (int)(qa.x & M); b.y = (int)(qa.y & M); b.z = (int)((qa.x >> 4) & M); b.w = (int)((qa.y >> 4) & M);
    c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(xo.A[0], b, c0, 0, 0, 0);
    b.x = (int)(qb.x & M); b.y = (int)(qb.y & M); b.z = (int)((qb.x >> 4) & M); b.w = (int)((qb.y >> 4) & M);
    c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(xo.A[2], b, c1, 0, 0, 0);
    b.x = (int)(qa.z & M); b.y = (int)(qa.w & M); b.z = (int)((qa.z >> 4) & M); b.w = (int)((qa.w >> 4) & M);
    c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(xo.A[1], b, c0, 0, 0, 0);
    b.x = (int)(qb.z & M); b.y = (int)(qb.w & M); b.z = (int)((qb.z >> 4) & M); b.w = (int)((qb.w >> 4) & M);
    c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(xo.A[3], b, c1, 0, 0, 0);
    /* 6-bit scale and min of sub-blocks g (chain 0) and 4+g (chain 1) */
    const uint32_t sh = 8u * (uint32_t)g;
    const uint32_t sc0 = __builtin_amdgcn_ubfe(hh.y, sh, 6), mn0 = __builtin_amdgcn_ubfe(hh.z, sh, 6);
    const uint32_t sc1 = __builtin_amdgcn_ubfe(hh.w, sh, 4) | (__builtin_amdgcn_ubfe(hh.y, sh + 6, 2) << 4);
    const uint32_t mn1 = __builtin_amdgcn_ubfe(hh.w, sh + 4, 4) | (__builtin_amdgcn_ubfe(hh.z, sh + 6, 2) << 4);
    const float d = half_bits_fast(hh.x & 0xFFFFu), dmin = half_bits_fast(hh.x >> 16);
    /* digit sums: |top| <= 32*15*64, the others <= 32*15*128, so each pair below is an integer of less
     * than 24 bits and its conversion is exact; one rounding in the multiply-add that joins them */
    const float s0 = fmaf((float)((c0.x << 8) + c0.y), 65536.0f, (float)((c0.z << 8) + c0.w));
    const float s1 = fmaf((float)((c1.x << 8) + c1.y), 65536.0f, (float)((c1.z << 8) + c1.w));
    const float z0 = s0 * xo.scale[0], z1 = s1 * xo.scale[1];
    const float dots = (float)sc0 * z0 + (float)sc1 * z1;
    const float mins = (float)mn0 * xo.sum[0] + (float)mn1 * xo.sum[1];
    return d * dots - dmin * mins;
}

}  // namespace

/* ONE: the job is one matrix, stored or added to y (the matrix and row of a local row then need no searching:
 * found by branches, they cost each weight request some forty instructions before it could go out) */
template <int NKC, bool ONE>
__global__ void __launch_bounds__(kWaves * 64)
gemv_q4k_kernel(const JobView job, const float *__restrict__ x, int n_sb, int rows_per_wg, size_t row_bytes, int lone_ahead) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 15, g = lane >> 4;

    /* a workgroup owns rows_per_wg rows: of the concatenated matrices, or, where two results are
     * combined (mode 2), the same rows of both matrices (local rows: first matrix, then second) */
    const bool paired = !ONE && job.mode == 2;
    const int n_mats_here = paired ? 2 : 1;
    const int n_rows = ONE ? job.n0 : paired ? job.n0 : job.n0 + job.n1 + job.n2;
    const int row0 = blockIdx.x * rows_per_wg;
    int rows_here = n_rows - row0;
    if (rows_here > rows_per_wg) rows_here = rows_per_wg;
    const int n_lrows = rows_here * n_mats_here;
    const int n_rg = (n_lrows + 15) >> 4;
    const int n_kc = wv < n_sb ? ((n_sb - wv + 15) >> 4) : 0; /* this wave's super-blocks: wv, wv+16, ... */

    /* LDS map: x scratch [kWaves][kXScratch] | partial sums [rows][kWaves] */
    uint8_t *xs = lds + wv * kXScratch;
    float *partial = reinterpret_cast<float *>(lds + kWaves * kXScratch);

    auto locate = [&](int lr, const uint8_t *&Wm, float *&ym, int &r) {
        if (ONE) {
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

    v4f xr[NKC];
#pragma unroll
    for (int kc = 0; kc < NKC; kc++) {
        v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (kc < n_kc) v = *reinterpret_cast<const v4f *>(x + (16 * kc + wv) * 256 + 4 * lane);
        xr[kc] = v;
    }
    auto prepare = [&](v4f v, XOperand &xo) { q4k_prepare(v, xo, xs, lane); };
    auto item = [&](const XOperand &xo, const uint4 hh, const uint4 qa, const uint4 qb) { return q4k_item(xo, hh, qa, qb, g); };
    auto row_pointer = [&](int rg) { /* this lane's row of row group rg (rows past the end: the last one, never stored) */
        int lr = 16 * rg + n;
        if (lr >= n_lrows) lr = n_lrows - 1;
        const uint8_t *Wm;
        float *ym;
        int r;
        locate(lr, Wm, ym, r);
        return Wm + (size_t)r * row_bytes + (size_t)wv * 144;
    };
    auto store_partial = [&](int rg, float v, bool add) { /* the four lane groups hold four sub-blocks' shares of the same row */
        v = sum_lane_groups(v);
        const int lr = 16 * rg + n;
        if (lane < 16 && lr < n_lrows) {
            float *p = partial + lr * kWaves + wv;
            *p = add ? *p + v : v;
        }
    };
    XOperand xo;
    /* one row group of column chunk kc at a time: the sixteen waves of a compute unit keep enough requests going
     * between them, and a wave that requested two to four row groups together before using the first measured slower
     * wherever a workgroup has more than one (14336 x 4096: 9.1 -> 8.7 us, gate+up+SiLU of that shape 15.6 -> 13.5,
     * 151936 x 4096: 80 -> 68, 8192 x 28672: 37 -> 32) */
    auto run_group = [&](int rg, int kc) {
        const uint8_t *blk = row_pointer(rg) + (size_t)kc * (16 * 144);
        const uint4 h = *reinterpret_cast<const uint4 *>(blk);
        const uint4 q0 = *reinterpret_cast<const uint4 *>(blk + 16 + 16 * g);
        const uint4 q1 = *reinterpret_cast<const uint4 *>(blk + 80 + 16 * g);
        if (rg == 0) { /* x is prepared while the first blocks are on their way */
            v4f v = xr[0];
            if (NKC > 1 && kc > 0) v = *reinterpret_cast<const v4f *>(x + (size_t)(16 * kc + wv) * 256 + 4 * lane);
            /* x is not looked at before this point: left alone, the compiler moves the first steps of the
             * preparation (they do not change from one pass of the loops to the next) in front of the loops, and
             * every wave then waits for x before it requests its first weights */
            asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w) : : "memory");
            prepare(v, xo);
        }
        store_partial(rg, item(xo, h, q0, q1), kc > 0);
    };
    if (n_kc == 0) { /* a wave without a super-block (K < 4096) contributes zeros */
        for (int rg = 0; rg < n_rg; rg++) store_partial(rg, 0.0f, false);
    } else if (NKC == 1 || n_rg >= 2 || !lone_ahead) {
        for (int kc = 0; kc < n_kc; kc++)
            for (int rg = 0; rg < n_rg; rg++) run_group(rg, kc);
    } else {
        /* long rows, one row group, workgroups for part of the compute units only: two of the wave's super-blocks
         * of the row are requested ahead of the one being multiplied (2048 x 16384: 7.9 us, 9.1 one at a time, 8.5
         * with all four requested together). With a workgroup on every compute unit the loop above, one super-block
         * at a time, is the faster one (4096 x 14336: 9.5 against 9.9 us, 4096 x 11008: 7.6 against 7.9). */
        const uint8_t *blk0 = row_pointer(0);
        uint4 h[2], q0[2], q1[2];
        auto request = [&](int slot, int kc) {
            const uint8_t *blk = blk0 + (size_t)kc * (16 * 144);
            h[slot] = *reinterpret_cast<const uint4 *>(blk);
            q0[slot] = *reinterpret_cast<const uint4 *>(blk + 16 + 16 * g);
            q1[slot] = *reinterpret_cast<const uint4 *>(blk + 80 + 16 * g);
        };
        request(0, 0);
        request(1, n_kc > 1 ? 1 : 0);
        float acc = 0.0f;
#pragma unroll
        for (int kc = 0; kc < NKC; kc++) {
            if (kc < n_kc) {
                prepare(xr[kc], xo);
                acc += item(xo, h[kc & 1], q0[kc & 1], q1[kc & 1]);
            }
            if (kc + 2 < n_kc) request(kc & 1, kc + 2);
            __builtin_amdgcn_sched_barrier(0);
        }
        store_partial(0, acc, false);
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

/* The same matvec for one matrix of rows of at most 4096 elements and at most kDmaRows rows per workgroup, with the
 * blocks fetched by the load-to-LDS path: wave w copies super-block w of all the workgroup's rows (runs of 144
 * contiguous bytes, consecutive lanes consecutive 16-byte pieces) into its own LDS image with eight requests
 * issued at once, and takes the matrix operands of a row group from there as soon as the requests that cover it
 * have landed (requests complete in order: three cover the first 16 rows, five the first 32, seven the first 48).
 * What the memory pipe sees is then 64 contiguous bytes per four lanes instead of four rows per four lanes.
 * All vector-memory instructions of the loop are written out with their own waits: the compiler's counters
 * would make the first wait cover every request. */
/* s_waitcnt vmcnt(N) that the compiler moves no memory access across (and, with an argument, no use of it) */
template <int N> __device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory"); }
template <int N> __device__ __forceinline__ void wait_vm(v4f &v) { asm volatile("s_waitcnt vmcnt(%1)" : "+v"(v) : "n"(N) : "memory"); }
constexpr int kDmaRows = 56;
constexpr int kDmaImage = 8192; /* 56 x 144 B = 8064 */

/* NQ: requests per wave = ceil(rows per workgroup x 9 / 64) */
template <int NQ>
__global__ void __launch_bounds__(kWaves * 64)
gemv_q4k_dma_kernel(const uint8_t *__restrict__ W, float *__restrict__ y, const float *__restrict__ x, int n_rows,
                    int n_sb, int add, int rows_per_wg, size_t row_bytes) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 15, g = lane >> 4;
    const int row0 = blockIdx.x * rows_per_wg;
    int rows_here = n_rows - row0;
    if (rows_here > rows_per_wg) rows_here = rows_per_wg;
    const int n_rg = (rows_here + 15) >> 4;
    /* LDS map: images [kWaves][kDmaImage] | x scratch [kWaves][kXScratch] | partial sums [rows][kWaves] */
    uint8_t *img = lds + wv * kDmaImage;
    uint8_t *xs = lds + kWaves * kDmaImage + wv * kXScratch;
    float *partial = reinterpret_cast<float *>(lds + kWaves * (kDmaImage + kXScratch));

    auto store_partial = [&](int rg, float v) { /* the four lane groups hold four sub-blocks' shares of the same row */
        v = sum_lane_groups(v);
        const int lr = 16 * rg + n;
        if (lane < 16 && lr < rows_here) partial[lr * kWaves + wv] = v;
    };
    if (wv >= n_sb) { /* a wave without a super-block (K < 4096) contributes zeros */
        for (int rg = 0; rg < n_rg; rg++) store_partial(rg, 0.0f);
    } else {
        /* x first, then the eight requests: piece id = 64 q + lane is part id % 9 of row id / 9 */
        v4f xv;
        const uint32_t x_off = (uint32_t)(wv * 256 + 4 * lane) * 4u;
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(xv) : "v"(x_off), "s"(x) : "memory");
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint8_t *>(W) + (size_t)row0 * row_bytes + (size_t)wv * 144, 0,
            (int)((size_t)(rows_here - 1) * row_bytes + 144), 0x00020000);
        const uint32_t img_base = (uint32_t)(uintptr_t)img; /* LDS addresses are the low 32 bits of the flat ones */
        /* 64 = 7 x 9 + 1: from one request to the next a lane moves on seven rows and one part (eight rows when the
         * part wraps). Pieces past the last row lie outside the descriptor and arrive as zeros. */
        uint32_t part = (uint32_t)lane % 9u, voff = ((uint32_t)lane / 9u) * (uint32_t)row_bytes + 16u * part;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                         :
                         : "s"(img_base + 1024u * q), "v"(voff), "s"(rsrc)
                         : "memory");
            const bool wrap = part == 8u;
            part = wrap ? 0u : part + 1u;
            voff += 7u * (uint32_t)row_bytes + (wrap ? (uint32_t)row_bytes - 128u : 16u);
        }
        /* xv is written by the load above without the compiler knowing when: this wait is its first use, in the
         * registers the load wrote (the compiled code is checked for a copy ahead of it whenever this kernel changes) */
        wait_vm<NQ>(xv);
        XOperand xo;
        q4k_prepare(xv, xo, xs, lane);
        auto run = [&](int rg) {
            int lr = 16 * rg + n;
            if (lr >= rows_here) lr = rows_here - 1; /* rows past the end: the last one, never stored */
            const uint8_t *blk = img + lr * 144;
            const uint4 h = *reinterpret_cast<const uint4 *>(blk);
            const uint4 q0 = *reinterpret_cast<const uint4 *>(blk + 16 + 16 * g);
            const uint4 q1 = *reinterpret_cast<const uint4 *>(blk + 80 + 16 * g);
            store_partial(rg, q4k_item(xo, h, q0, q1, g));
        };
        /* row group rg is covered by requests 0 .. (144 (rg + 1) - 1) / 64 */
        wait_vm<(NQ - 3 > 0 ? NQ - 3 : 0)>();
        run(0);
        if (n_rg > 1) {
            wait_vm<(NQ - 5 > 0 ? NQ - 5 : 0)>();
            run(1);
        }
        if (n_rg > 2) {
            wait_vm<(NQ - 7 > 0 ? NQ - 7 : 0)>();
            run(2);
        }
        if (n_rg > 3) {
            wait_vm<0>();
            run(3);
        }
        wait_vm<0>(); /* nothing on its way into LDS when the wave ends */
    }
    __syncthreads();
    for (int lr = threadIdx.x; lr < rows_here; lr += kWaves * 64) {
        const float4 *p = reinterpret_cast<const float4 *>(partial + lr * kWaves);
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < kWaves / 4; k++) {
            const float4 v = p[k];
            s += (v.x + v.y) + (v.z + v.w);
        }
        y[row0 + lr] = add ? y[row0 + lr] + s : s;
    }
}

/* The load-to-LDS matvec for one matrix of longer rows (17 to 64 super-blocks) and at most kDmaLongRows rows per
 * workgroup - the down projection, 4096 x 14336: 16 rows per compute unit. Wave w takes super-blocks w, w + 16, ... of
 * the workgroup's rows, one pass each; the image of a pass is rows x 144 bytes (NQ requests), two image slots per wave:
 * the pass after next is requested as soon as a pass has been multiplied, so a wave has two passes in flight or in
 * work instead of one round trip after the other. A pass's 256 activations come by the same path into the last KB of
 * its slot (a register load would have to be waited for by a counter the compiler cannot see). A row's shares of
 * all passes are added in registers. */
constexpr int kDmaLongRows = 21;   /* 21 x 144 B = 3024: a 4 KB slot holds the image (3 requests) and 1 KB of activations */
constexpr int kDmaLongPasses = 4;

template <int NQ>
__global__ void __launch_bounds__(kWaves * 64)
gemv_q4k_dma_long_kernel(const uint8_t *__restrict__ W, float *__restrict__ y, const float *__restrict__ x, int n_rows,
                         int n_sb, int add, int rows_per_wg, size_t row_bytes) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 15, g = lane >> 4;
    const int row0 = blockIdx.x * rows_per_wg;
    int rows_here = n_rows - row0;
    if (rows_here > rows_per_wg) rows_here = rows_per_wg;
    const int n_rg = (rows_here + 15) >> 4; /* 1 or 2 */
    const int n_kc = (n_sb - wv + 15) >> 4; /* this wave's passes: 1 .. 4 (n_sb > 16) */
    /* LDS map: image slots [kWaves][2][4 KB] | x scratch [kWaves][kXScratch] | partial sums [rows][kWaves] */
    uint8_t *img = lds + wv * kDmaImage;
    uint8_t *xs = lds + kWaves * kDmaImage + wv * kXScratch;
    float *partial = reinterpret_cast<float *>(lds + kWaves * (kDmaImage + kXScratch));

    static_assert(NQ <= 3, "a slot is three requests of weights and one of activations");
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(x), 0, n_sb * 1024, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(W) + (size_t)row0 * row_bytes, 0, (int)((size_t)(rows_here - 1) * row_bytes + (size_t)n_sb * 144),
        0x00020000);
    const uint32_t img_base = (uint32_t)(uintptr_t)img;
    /* piece id = 64 q + lane is part id % 9 of row id / 9; pieces past the last row arrive as zeros */
    uint32_t voff0[NQ];
    {
        uint32_t part = (uint32_t)lane % 9u, row = (uint32_t)lane / 9u;
#pragma unroll
        for (int q = 0; q < NQ; q++) {
            voff0[q] = row < (uint32_t)rows_here ? row * (uint32_t)row_bytes + 16u * part : 0xFFFFFFF0u;
            const bool wrap = part == 8u;
            part = wrap ? 0u : part + 1u;
            row += wrap ? 8u : 7u;
        }
    }
    const uint32_t x_voff = 16u * (uint32_t)lane;
    auto request = [&](int kc) { /* pass kc into slot kc & 1: its activations, then its blocks */
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :
                     : "s"(img_base + 4096u * (kc & 1) + 3072u), "v"(x_voff), "s"(x_rsrc), "s"((uint32_t)(16 * kc + wv) * 1024u)
                     : "memory");
        const uint32_t soff = (uint32_t)(16 * kc + wv) * 144u;
#pragma unroll
        for (int q = 0; q < NQ; q++)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :
                         : "s"(img_base + 4096u * (kc & 1) + 1024u * q), "v"(voff0[q]), "s"(rsrc), "s"(soff)
                         : "memory");
    };
    request(0);
    if (n_kc > 1) request(1);
    float acc[2] = {0.0f, 0.0f};
    XOperand xo;
#pragma unroll
    for (int kc = 0; kc < kDmaLongPasses; kc++) {
        if (kc < n_kc) {
            /* the requests of this pass are in when at most those of the next one are outstanding */
            if (kc + 1 < n_kc) wait_vm<NQ + 1>();
            else wait_vm<0>();
            const uint8_t *slot = img + 4096 * (kc & 1);
            q4k_prepare(*reinterpret_cast<const v4f *>(slot + 3072 + 16 * lane), xo, xs, lane);
#pragma unroll
            for (int rg = 0; rg < 2; rg++) {
                if (rg < n_rg) {
                    int lr = 16 * rg + n;
                    if (lr >= rows_here) lr = rows_here - 1; /* rows past the end: the last one, never stored */
                    const uint8_t *blk = slot + lr * 144;
                    const uint4 h = *reinterpret_cast<const uint4 *>(blk);
                    const uint4 q0 = *reinterpret_cast<const uint4 *>(blk + 16 + 16 * g);
                    const uint4 q1 = *reinterpret_cast<const uint4 *>(blk + 80 + 16 * g);
                    acc[rg] += q4k_item(xo, h, q0, q1, g);
                }
            }
            if (kc + 2 < n_kc) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* the slot has been read before it is refilled */
                request(kc + 2);
            }
        }
    }
#pragma unroll
    for (int rg = 0; rg < 2; rg++) {
        if (rg < n_rg) {
            const float v = sum_lane_groups(acc[rg]);
            const int lr = 16 * rg + n;
            if (lane < 16 && lr < rows_here) partial[lr * kWaves + wv] = v;
        }
    }
    __syncthreads();
    for (int lr = threadIdx.x; lr < rows_here; lr += kWaves * 64) {
        const float4 *p = reinterpret_cast<const float4 *>(partial + lr * kWaves);
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < kWaves / 4; k++) {
            const float4 v = p[k];
            s += (v.x + v.y) + (v.z + v.w);
        }
        y[row0 + lr] = add ? y[row0 + lr] + s : s;
    }
}

/* A token (or a few, each on its own) through its top_k routed experts, Q4_K expert tensors (the reference's MoE block for a token,
 * common/transformer.h:4045-4131: sum_j w_j * down_e(silu(gate_e x) * up_e x), e = idx[j]), as two launches of the
 * matvec above:
 *   DOWN = false  h[j][r] = silu(gate_e[r,:] . x) * (up_e[r,:] . x), r < rows_per_expert (n_ff); grid (row tiles, tokens x top_k);
 *                 x is the token's bf16 activations, sb_per_expert = n_embd / 256
 *   DOWN = true   y[r] = sum_j w_j * (down_e[r,:] . h[j]), r < rows_per_expert (n_embd), grid (row tiles, tokens): ONE matvec over a row of
 *                 top_k * n_ff elements whose super-blocks sit in different experts, the routing weight folded into
 *                 its x; sb_per_expert = n_ff / 256. The sum runs in a fixed order.
 * An expert index outside [0, n_expert) contributes nothing. Wave w owns super-blocks w, w + waves, ... */
template <bool DOWN>
__global__ void __launch_bounds__(kWaves * 64)
moe1_q4k_kernel(const uint8_t *__restrict__ Wa, const uint8_t *__restrict__ Wb, const void *xin,
                const int32_t *idx, const float *wts, float *y, int top_k,
                int n_expert, int rows_per_expert, int sb_per_expert, int rows_per_wg, int ldx) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n_waves = blockDim.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int row0 = blockIdx.x * rows_per_wg;
    int rows_here = rows_per_expert - row0;
    if (rows_here > rows_per_wg) rows_here = rows_per_wg;
    const int n_lrows = DOWN ? rows_here : 2 * rows_here; /* gate rows, then up rows */
    const int n_rg = (n_lrows + 15) >> 4;
    const size_t row_bytes = (size_t)sb_per_expert * 144, expert_bytes = (size_t)rows_per_expert * row_bytes;
    const int n_sb = DOWN ? top_k * sb_per_expert : sb_per_expert;
    const int pair = DOWN ? 0 : (int)blockIdx.y; /* token * top_k + k */
    if (DOWN) { /* blockIdx.y = token */
        idx += (size_t)blockIdx.y * top_k;
        wts += (size_t)blockIdx.y * top_k;
        xin = static_cast<const float *>(xin) + (size_t)blockIdx.y * top_k * (sb_per_expert * 256);
        y += (size_t)blockIdx.y * rows_per_expert;
    } else {
        xin = static_cast<const uint16_t *>(xin) + (size_t)(pair / top_k) * ldx;
    }
    int e_up = 0;
    if (!DOWN) {
        e_up = idx[pair];
        if (e_up < 0 || e_up >= n_expert) return; /* uniform over the workgroup */
    }
    uint8_t *xs = lds + wv * kXScratch;
    float *partial = reinterpret_cast<float *>(lds + n_waves * kXScratch); /* [local row][wave] */
    for (int lr = lane; lr < n_lrows; lr += 64) partial[lr * n_waves + wv] = 0.0f;

    XOperand xo;
    for (int sb = wv; sb < n_sb; sb += n_waves) {
        /* the expert and the super-block inside its rows that this (virtual) super-block is, and its x */
        int e = e_up, sbi = sb, j = pair;
        if (DOWN) {
            j = sb / sb_per_expert;
            sbi = sb - j * sb_per_expert;
            e = idx[j];
            if (e < 0 || e >= n_expert) continue; /* uniform over the wave */
        }
        const uint8_t *base_a = Wa + (size_t)e * expert_bytes + (size_t)sbi * 144;
        const uint8_t *base_b = DOWN ? base_a : Wb + (size_t)e * expert_bytes + (size_t)sbi * 144;
        for (int rg = 0; rg < n_rg; rg++) {
            int lr = 16 * rg + n;
            if (lr >= n_lrows) lr = n_lrows - 1; /* rows past the end: the last one, never stored */
            const bool second = !DOWN && lr >= rows_here;
            const uint8_t *blk = (second ? base_b : base_a) + (size_t)(row0 + (second ? lr - rows_here : lr)) * row_bytes;
            const uint4 h = *reinterpret_cast<const uint4 *>(blk);
            const uint4 q0 = *reinterpret_cast<const uint4 *>(blk + 16 + 16 * g);
            const uint4 q1 = *reinterpret_cast<const uint4 *>(blk + 80 + 16 * g);
            if (rg == 0) { /* x is prepared while the first blocks are on their way */
                v4f v;
                if (DOWN) {
                    const float wj = wts[j];
                    v = *reinterpret_cast<const v4f *>(static_cast<const float *>(xin) + (size_t)j * (sb_per_expert * 256) + sbi * 256 + 4 * lane);
                    v.x *= wj; v.y *= wj; v.z *= wj; v.w *= wj;
                } else {
                    const uint2 b = *reinterpret_cast<const uint2 *>(static_cast<const uint16_t *>(xin) + sbi * 256 + 4 * lane);
                    v.x = __uint_as_float(b.x << 16); v.y = __uint_as_float(b.x & 0xFFFF0000u);
                    v.z = __uint_as_float(b.y << 16); v.w = __uint_as_float(b.y & 0xFFFF0000u);
                }
                asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w) : : "memory");
                q4k_prepare(v, xo, xs, lane);
            }
            const float part = sum_lane_groups(q4k_item(xo, h, q0, q1, g));
            const int slr = 16 * rg + n;
            if (lane < 16 && slr < n_lrows) partial[slr * n_waves + wv] += part;
        }
    }
    __syncthreads();
    auto row_total = [&](int lr) {
        const float4 *p = reinterpret_cast<const float4 *>(partial + lr * n_waves);
        float s = 0.0f;
        for (int k = 0; k < n_waves / 4; k++) {
            const float4 v = p[k];
            s += (v.x + v.y) + (v.z + v.w);
        }
        return s;
    };
    for (int lr = threadIdx.x; lr < rows_here; lr += blockDim.x) {
        if (DOWN) y[row0 + lr] = row_total(lr);
        else y[(size_t)pair * rows_per_expert + row0 + lr] = silu_times(row_total(lr), row_total(rows_here + lr));
    }
}

/* The two launches above, one function each; false: not a shape for it (the caller takes its general path).
 * dry: only say whether it would be taken. h: n_tok * top_k * n_ff floats of scratch. */
bool launch_moe1_q4k_up(const void *gate, const void *up, const uint16_t *X, const int32_t *idx, float *h, int n_tok,
                        int top_k, int n_embd, int n_ff, int n_expert, int n_cu, hipStream_t stream, bool dry, hipError_t *err) {
    *err = hipSuccess;
    if (n_embd % 256 != 0 || n_ff < 1 || top_k < 1 || n_tok < 1 || n_cu < 1) return false;
    if ((((uintptr_t)gate | (uintptr_t)up | (uintptr_t)h) & 15) || ((uintptr_t)X & 7)) return false;
    if (dry) return true;
    /* n_tok * top_k experts x n_ff row pairs over the compute units */
    const int n_pairs = n_tok * top_k;
    const int tiles = n_cu / n_pairs > 0 ? n_cu / n_pairs : 1;
    int rows_per_wg = (n_ff + tiles - 1) / tiles;
    if (2 * rows_per_wg > kMaxRowsPerWg) rows_per_wg = kMaxRowsPerWg / 2;
    const int waves = n_embd / 256 <= 8 ? 8 : kWaves;
    hipLaunchKernelGGL(moe1_q4k_kernel<false>, dim3((n_ff + rows_per_wg - 1) / rows_per_wg, n_pairs), dim3(waves * 64),
                       (size_t)waves * kXScratch + (size_t)2 * rows_per_wg * waves * 4, stream, (const uint8_t *)gate,
                       (const uint8_t *)up, (const void *)X, idx, (const float *)nullptr, h, top_k, n_expert, n_ff, n_embd / 256,
                       rows_per_wg, n_embd);
    *err = hipGetLastError();
    return true;
}

bool launch_moe1_q4k_down(const void *down, const float *h, const int32_t *idx, const float *w, float *out, int n_tok, int top_k,
                          int n_embd, int n_ff, int n_expert, int n_cu, hipStream_t stream, bool dry, hipError_t *err) {
    *err = hipSuccess;
    if (n_ff % 256 != 0 || n_embd < 1 || top_k < 1 || n_tok < 1 || n_cu < 1) return false;
    if (((uintptr_t)down | (uintptr_t)h) & 15) return false;
    if (dry) return true;
    const int tiles = n_cu / n_tok > 0 ? n_cu / n_tok : 1;
    int rows_per_wg = (n_embd + tiles - 1) / tiles;
    if (rows_per_wg > kMaxRowsPerWg) rows_per_wg = kMaxRowsPerWg;
    hipLaunchKernelGGL(moe1_q4k_kernel<true>, dim3((n_embd + rows_per_wg - 1) / rows_per_wg, n_tok), dim3(kWaves * 64),
                       (size_t)kWaves * kXScratch + (size_t)rows_per_wg * kWaves * 4, stream, (const uint8_t *)down,
                       (const uint8_t *)down, (const void *)h, idx, w, out, top_k, n_expert, n_embd, n_ff / 256, rows_per_wg, 0);
    *err = hipGetLastError();
    return true;
}

hipError_t launch_gemv_q4k(const GemvJob &job, const float *x, int n_cols, hipStream_t stream, int n_cu, size_t row_stride) {
    const int n_sb = n_cols / 256;
    if (n_sb > 16 * kMaxKc || n_sb < 1) return hipErrorInvalidValue;
    const int n_mats_here = job.mode == kSiluMul ? 2 : 1;
    const int n_rows = job.mode == kSiluMul ? job.n_rows[0] : job.total_rows();
    if (n_rows == 0) return hipSuccess;
    /* one workgroup per compute unit where its partial sums fit in LDS, else so many equal rounds of workgroups
     * that they do (151936 rows: 594 each; with 128-row workgroups the 1187 of them left a fifth round a third full:
     * 66.5 -> 60.5 us, 49152 rows 26.8 -> 21.3) */
    const int rows_per_cu = (n_rows + n_cu - 1) / n_cu;
    const int rounds = (rows_per_cu * n_mats_here + kMaxRowsPerWg - 1) / kMaxRowsPerWg;
    int rows_per_wg = (n_rows + n_cu * rounds - 1) / (n_cu * rounds);
    if (rows_per_wg < 1) rows_per_wg = 1;
    if (rows_per_wg * n_mats_here > kMaxRowsPerWg) rows_per_wg = kMaxRowsPerWg / n_mats_here;
    const int grid = (n_rows + rows_per_wg - 1) / rows_per_wg;
    const size_t lds_bytes = (size_t)kWaves * kXScratch + (size_t)rows_per_wg * n_mats_here * kWaves * 4;
    const JobView view = job_view(job);
    if (row_stride == 0) row_stride = (size_t)n_sb * 144; /* rows that are a column range of longer ones keep those rows' pitch */
    const bool one = job.n_mat == 1 && job.mode != kSiluMul;
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(kWaves * 64), lds_bytes, stream, view, x, n_sb, rows_per_wg, row_stride,
                           grid < n_cu ? 1 : 0);
    };
    /* one matrix, rows of up to 4096 elements, at most 56 rows per workgroup: the load-to-LDS kernel */
    if (one && n_sb <= 16 && rows_per_wg <= kDmaRows && (size_t)kDmaRows * row_stride < ((size_t)1 << 31)) {
        auto launch_dma = [&](auto kernel, OnceFlag &lds_raised) {
            if (!lds_raised.is_set()) {
                hipError_t e = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return e;
                lds_raised.set();
            }
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(kWaves * 64),
                               (size_t)kWaves * (kDmaImage + kXScratch) + (size_t)rows_per_wg * kWaves * 4, stream,
                               (const uint8_t *)job.W[0], job.y[0], x, n_rows, n_sb, job.mode == kAdd ? 1 : 0, rows_per_wg, row_stride);
            return hipGetLastError();
        };
        static OnceFlag raised[8];
        switch ((rows_per_wg * 9 + 63) / 64) {
        case 1: return launch_dma(gemv_q4k_dma_kernel<1>, raised[0]);
        case 2: return launch_dma(gemv_q4k_dma_kernel<2>, raised[1]);
        case 3: return launch_dma(gemv_q4k_dma_kernel<3>, raised[2]);
        case 4: return launch_dma(gemv_q4k_dma_kernel<4>, raised[3]);
        case 5: return launch_dma(gemv_q4k_dma_kernel<5>, raised[4]);
        case 6: return launch_dma(gemv_q4k_dma_kernel<6>, raised[5]);
        case 7: return launch_dma(gemv_q4k_dma_kernel<7>, raised[6]);
        default: return launch_dma(gemv_q4k_dma_kernel<8>, raised[7]);
        }
    }
    /* one matrix, rows of 17 to 64 super-blocks, at most 21 rows per workgroup: the load-to-LDS kernel for long rows */
    /* (1 GiB rotation, this kernel / the register-load kernel below, us: 4096 x 14336 9.1 / 9.8, 2048 x 16384 8.2 / 9.5,
     * 4096 x 8192 6.3 / 7.1, 1024 x 14336 6.6 / 7.7, 4096 x 5120 5.0 / 5.2; with three passes for most waves and two for
     * the rest, 4096 x 11008, it measured 8.3 / 7.7, so rows of 33 to 48 super-blocks stay with the other kernel) */
    if (one && n_sb > 16 && n_sb <= 16 * kDmaLongPasses && (n_sb <= 32 || n_sb > 48) && rows_per_wg <= kDmaLongRows &&
        (size_t)kDmaLongRows * row_stride < ((size_t)1 << 31)) {
        auto launch_long = [&](auto kernel, OnceFlag &lds_raised) {
            if (!lds_raised.is_set()) {
                hipError_t e = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return e;
                lds_raised.set();
            }
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(kWaves * 64),
                               (size_t)kWaves * (kDmaImage + kXScratch) + (size_t)rows_per_wg * kWaves * 4, stream,
                               (const uint8_t *)job.W[0], job.y[0], x, n_rows, n_sb, job.mode == kAdd ? 1 : 0, rows_per_wg, row_stride);
            return hipGetLastError();
        };
        static OnceFlag raised_long[3];
        switch ((rows_per_wg * 9 + 63) / 64) {
        case 1: return launch_long(gemv_q4k_dma_long_kernel<1>, raised_long[0]);
        case 2: return launch_long(gemv_q4k_dma_long_kernel<2>, raised_long[1]);
        default: return launch_long(gemv_q4k_dma_long_kernel<3>, raised_long[2]);
        }
    }
    if (n_sb <= 16) {
        if (one) launch(gemv_q4k_kernel<1, true>);
        else launch(gemv_q4k_kernel<1, false>);
    } else {
        if (one) launch(gemv_q4k_kernel<kMaxKc, true>);
        else launch(gemv_q4k_kernel<kMaxKc, false>);
    }
    return hipGetLastError();
}

}  // namespace qlin
