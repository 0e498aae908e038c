/*
 * gemv_q4k.hip - batch-1 Q4_K matvec tuned for HBM streaming on gfx950.
 *
 * Structure (one workgroup of 16 wavefronts per block of rows, about one per compute unit):
 *
 *  1. x -> fixed point, once per workgroup. Each 32-element sub-block of x (the Q4_K scale
 *     granularity, common/ggml_dequant.h:71-76) is scaled by a power of two so that
 *     X = rint(x * 2^(22-e)) fits 23 bits, and the three bytes of X are stored as three
 *     "digit planes" in LDS (top byte signed, lower two unsigned) together with 2^(e-22) and
 *     the fp32 sum of the sub-block. Quantisation error is 2^-23 of the sub-block's largest
 *     |x|; measured end-to-end error is ~7e-7 relative L2 against the double-precision oracle.
 *  2. Weights are streamed as a FLAT byte stream: a wavefront moves a row (or a slice of at
 *     most 16 super-blocks = 2304 bytes of it) with up to three fully contiguous
 *     16-byte-per-lane loads that write straight into a private LDS row image
 *     (global_load_lds_dwordx4: no registers are held while the data is in flight). Only the
 *     flat pattern reaches the streaming rate of a plain copy kernel; lane-owned strided
 *     16-byte loads cost 40 % more time on this part. One row per wavefront in flight (16
 *     per compute unit, 9.4 MB over the chip) already runs HBM at the rate it gives a burst of
 *     this size; deeper rings (the code takes up to four images) measured slower, because
 *     they only lengthen the queue in front of the x loads and of each wave's last row.
 *     The x loads of all 16 waves are issued before any row load (a barrier separates them),
 *     so the x preparation overlaps the first rows instead of waiting behind them.
 *  3. Arithmetic re-reads the row image in the layout it wants: four lanes per super-block,
 *     lane c takes nibble bytes qs[32c..32c+31] = sub-blocks 2c (low nibbles) and 2c+1 (high
 *     nibbles). The nibbles are masked into bytes and multiplied with the digit planes by
 *     4-way integer dot instructions: 48 per row and lane instead of 128 converts and FMAs.
 *     Per sub-block: S = top*65536 + mid*256 + low, y += d*sc*2^(e-22)*S - dmin*m*sum(x)
 *     (the factored form of common/ggml_dequant.h:1592-1618 dotted with x; scales unpacked
 *     four at a time from the 12 packed bytes, get_scale_min_k4, :1582-1590).
 *  4. Rows longer than 16 super-blocks are cut into S = 2 or 4 slices; slice s of a row is
 *     handled by a wave with (wave % S) == s, so every wave keeps ONE slice of the digit
 *     planes in registers for all its rows. Partial sums meet in LDS at the end.
 *
 * A non-finite x makes every output NaN (the fixed-point form cannot carry Inf).
 */
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

namespace {

#ifndef Q4K_WAVES
#define Q4K_WAVES 16
#endif
constexpr int kWaves = Q4K_WAVES;   /* wavefronts per workgroup: 16 or 8 (a multiple of 4, the most slices) */
constexpr int kThreads = kWaves * 64;
constexpr int kChunk = 52;          /* dwords per 64-element x chunk: 3 planes x 16, padded so that
                                       consecutive lanes' 16-byte reads fall on distinct banks */
constexpr int kRowImage = 2304;     /* bytes per LDS row image: 16 super-blocks */
#ifndef Q4K_MAX_DEPTH
#define Q4K_MAX_DEPTH 1
#endif
constexpr int kMaxDepth = Q4K_MAX_DEPTH; /* row images per wavefront */
constexpr int kMaxRowsPerWg = 128;

__device__ __forceinline__ int sdot4(uint32_t a, uint32_t b, int c) { return __builtin_amdgcn_sdot4((int)a, (int)b, c, false); }
__device__ __forceinline__ uint32_t udot4(uint32_t a, uint32_t b, uint32_t c) { return __builtin_amdgcn_udot4(a, b, c, false); }

}  // namespace

__global__ void __launch_bounds__(kThreads)
gemv_q4k_kernel(const JobView job, const float *__restrict__ x, int n_sb, int n_slices, int slice_sb,
                int rows_per_wg, int depth) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    /* LDS map: planes [n_sb*4][kChunk] dwords | meta [n_sb*4] float4 | row images [16][depth][kRowImage] |
     * partial sums [rows_per_wg * n_slices] floats (padded to 16 bytes) | raw x [n_sb*256] floats */
    uint32_t *planes = reinterpret_cast<uint32_t *>(lds);
    float4 *meta = reinterpret_cast<float4 *>(planes + n_sb * 4 * kChunk);
    uint8_t *images = reinterpret_cast<uint8_t *>(meta + n_sb * 4);
    float *partial = reinterpret_cast<float *>(images + kWaves * depth * kRowImage);
    /* a workgroup owns rows_per_wg rows: of the concatenated matrices, or, where two results are
     * combined (mode 2), the same rows of both matrices (local rows: first matrix, then second) */
    const bool paired = job.mode == 2;
    const int n_mats_here = paired ? 2 : 1;
    const float4 *xraw = reinterpret_cast<const float4 *>(partial + ((rows_per_wg * n_mats_here * n_slices + 3) & ~3));

    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); /* wave-uniform, and the compiler is told so */
    const int c = lane & 3;
    const int slice = wv % n_slices;
    const int sb0 = slice * slice_sb;
    int sb_cnt = n_sb - sb0;
    if (sb_cnt > slice_sb) sb_cnt = slice_sb;
    const bool active = (lane >> 2) < sb_cnt;
    const int sb_local = active ? (lane >> 2) : 0;
    const size_t row_bytes = (size_t)n_sb * 144;
    const int n_chunks = sb_cnt * 9;                  /* 16-byte chunks in this wave's slice of a row */
    const int loads_per_row = (n_chunks + 63) >> 6;   /* wave-uniform: 1, 2 or 3 */

    const int n_rows = paired ? job.n0 : job.n0 + job.n1 + job.n2;
    const int row0 = blockIdx.x * rows_per_wg; /* first row of this workgroup */
    int rows_here = n_rows - row0;
    if (rows_here > rows_per_wg) rows_here = rows_per_wg;
    const int n_lrows = rows_here * n_mats_here;  /* local rows */
    const int n_vrows = n_lrows * n_slices;       /* (local row, slice) pairs of this workgroup */

    /* this wave's virtual rows: wv, wv + 16, ... ; virtual row j = (row j / S, slice j % S), and
     * 16 % S == 0 keeps the slice of a wave fixed. my_rows of them, numbered i = 0.. */
    const int my_rows = wv < n_vrows ? (n_vrows - wv + kWaves - 1) / kWaves : 0;
    /* where local row lr lives: matrix and row */
    auto locate = [&](int lr, const uint8_t *&Wm, float *&ym, int &r) {
        if (paired) {
            const bool second = lr >= rows_here;
            Wm = second ? job.W1 : job.W0;
            ym = job.y0;
            r = row0 + (second ? lr - rows_here : lr);
        } else {
            job_locate(job, row0 + lr, Wm, ym, r);
        }
    };
    uint8_t *my_images = images + wv * (depth * kRowImage);
    const uint32_t my_images_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)my_images;
    /* Row i of this wave -> image slot i % depth; exactly loads_per_row instructions are issued.
     * Each is a 16-byte-per-lane load whose data goes to LDS at M0 + 16*lane instead of to
     * registers. They are written as instructions: for the builtin form the compiler, which
     * cannot tell the images apart, waits for every outstanding one before any LDS access, and
     * that would serialise the ring. The waits this kernel needs are placed by hand
     * (wait_vm_at_most before an image is read, lgkmcnt(0) before its slot is refilled).
     * Nothing else in this kernel uses M0. The rows are marked non-temporal: every weight byte is
     * read once, and without the mark a launch pushes x, the kernel arguments and its own code out
     * of the L2 for the next launch (measured: 0.6 us per launch). */
    auto issue = [&](int i) {
        const int j = wv + i * kWaves;
        const uint8_t *Wm;
        float *ym;
        int r;
        locate(j / n_slices, Wm, ym, r);
        const uint4 *g = reinterpret_cast<const uint4 *>(Wm + (size_t)r * row_bytes + (size_t)sb0 * 144);
        const uint32_t img = __builtin_amdgcn_readfirstlane(my_images_lds + (uint32_t)((i % depth) * kRowImage));
#define QLIN_LOAD_TO_LDS(chunk0)                                                                          \
        if ((chunk0) + lane < n_chunks)                                                                   \
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt"                 \
                         : : "v"(g + (chunk0) + lane), "s"(img + 16u * (chunk0)) : "memory")
        QLIN_LOAD_TO_LDS(0);
        QLIN_LOAD_TO_LDS(64);
        QLIN_LOAD_TO_LDS(128);
#undef QLIN_LOAD_TO_LDS
    };

    /* x is requested first, so that it does not queue behind the weight stream: like the rows it
     * goes straight to LDS (a raw fp32 copy, 1 KB per instruction and wave), so no register holds
     * data that is still in flight. A barrier makes every wave's x request precede every row
     * request; then up to `depth` rows per wave are put in flight while x is being prepared.
     * Loads retire in order, so "at most the row loads outstanding" means that this wave's part
     * of x has landed; each thread then prepares exactly the elements its own wave fetched. */
    const int n4 = n_sb * 64;
    const float4 *xg = reinterpret_cast<const float4 *>(x);
    const uint32_t xraw_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)xraw;
    for (int base = wv * 64; base < n4; base += kThreads) { /* uniform per wave */
        const uint32_t m0v = __builtin_amdgcn_readfirstlane(xraw_lds + 16u * (uint32_t)base);
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                     : : "v"(xg + base + lane), "s"(m0v) : "memory");
    }
    asm volatile("s_barrier" ::: "memory");
    int issued = 0;
    for (; issued < depth && issued < my_rows; issued++) issue(issued);
    wait_vm_at_most(issued * loads_per_row);

    /* ---- x -> digit planes (whole workgroup, 4 elements per thread and step); no loads in here,
     * so nothing in it waits for the weights */
    auto quantize = [&](int idx, const float4 v) {
            const bool mine = idx < n4;
            float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
            float sum = (v.x + v.y) + (v.z + v.w);
            /* 8 consecutive threads share one 32-element sub-block */
            amax = fmaxf(amax, dpp_mov<0xB1>(amax));
            amax = fmaxf(amax, dpp_mov<0x4E>(amax));
            amax = fmaxf(amax, dpp_mov<0x141>(amax));
            sum += dpp_mov<0xB1>(sum);
            sum += dpp_mov<0x4E>(sum);
            sum += dpp_mov<0x141>(sum);
            int e = (int)(__float_as_uint(amax) >> 23) - 126; /* amax in [2^(e-1), 2^e) */
            if (e < -100) e = -100;                            /* zero and tiny blocks */
            const float scale = __uint_as_float((uint32_t)(127 + 22 - e) << 23);
            float inv = __uint_as_float((uint32_t)(127 - 22 + e) << 23);
            if (!(amax <= 3.0e38f)) inv = __uint_as_float(0x7FC00000u); /* Inf/NaN in x: poison every row */
            const uint32_t X0 = (uint32_t)__float2int_rn(v.x * scale), X1 = (uint32_t)__float2int_rn(v.y * scale);
            const uint32_t X2 = (uint32_t)__float2int_rn(v.z * scale), X3 = (uint32_t)__float2int_rn(v.w * scale);
            /* byte transpose: plane k = byte k of X0..X3 (selector 0-3: second operand, 4-7: first) */
            const uint32_t lo01 = __builtin_amdgcn_perm(X1, X0, 0x05010400u); /* X0.b0 X1.b0 X0.b1 X1.b1 */
            const uint32_t lo23 = __builtin_amdgcn_perm(X3, X2, 0x05010400u);
            const uint32_t hi01 = __builtin_amdgcn_perm(X1, X0, 0x07030602u); /* X0.b2 X1.b2 X0.b3 X1.b3 */
            const uint32_t hi23 = __builtin_amdgcn_perm(X3, X2, 0x07030602u);
            const uint32_t pl_low = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u); /* bytes 0 of X0..X3 */
            const uint32_t pl_mid = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u); /* bytes 1 */
            const uint32_t pl_top = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u); /* bytes 2 */
            const int sub = idx >> 3, j = idx & 7;
            const int chunk = sub >> 1, is_b = sub & 1;
            uint32_t *dst = planes + chunk * kChunk + is_b * 8 + j;
            if (mine) {
                dst[0] = pl_top;
                dst[16] = pl_mid;
                dst[32] = pl_low;
            }
            if (mine && j == 0) {
                float *m = reinterpret_cast<float *>(meta + chunk);
                m[is_b] = inv;
                m[2 + is_b] = sum;
            }
    };
    for (int idx = threadIdx.x; idx < n4; idx += kThreads) quantize(idx, xraw[idx]);
    __syncthreads();

    /* this lane's x: 16 dwords per plane (8 for sub-block 2c, 8 for 2c+1) */
    uint32_t xt[16], xm[16], xl[16];
    {
        const uint4 *pp = reinterpret_cast<const uint4 *>(planes + ((sb0 + sb_local) * 4 + c) * kChunk);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint4 t = pp[i], m = pp[4 + i], l = pp[8 + i];
            xt[4 * i] = t.x; xt[4 * i + 1] = t.y; xt[4 * i + 2] = t.z; xt[4 * i + 3] = t.w;
            xm[4 * i] = m.x; xm[4 * i + 1] = m.y; xm[4 * i + 2] = m.z; xm[4 * i + 3] = m.w;
            xl[4 * i] = l.x; xl[4 * i + 1] = l.y; xl[4 * i + 2] = l.z; xl[4 * i + 3] = l.w;
        }
    }
    const float4 mt = meta[(sb0 + sb_local) * 4 + c];
    const float inv_a = mt.x, inv_b = mt.y, sum_a = mt.z, sum_b = mt.w;

    for (int i = 0; i < my_rows; i++) {
        /* rows i .. issued-1 are in flight; row i is the oldest */
        wait_vm_at_most((issued - i - 1) * loads_per_row);
        const uint8_t *blk = my_images + (i % depth) * kRowImage + sb_local * 144;
        const uint4 h = *reinterpret_cast<const uint4 *>(blk);
        const uint4 qa = *reinterpret_cast<const uint4 *>(blk + 16 + 32 * c);
        const uint4 qb = *reinterpret_cast<const uint4 *>(blk + 32 + 32 * c);
        /* the image may be overwritten once these reads have returned */
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (issued < my_rows) {
            issue(issued);
            issued++;
        }
        const float d = half_bits_fast(h.x & 0xFFFFu), dmin = half_bits_fast(h.x >> 16);
        /* bytes of sc_lo: scales 0..3, mn_lo: mins 0..3, sc_hi: scales 4..7, mn_hi: mins 4..7 */
        const uint32_t sc_lo = h.y & 0x3F3F3F3Fu, mn_lo = h.z & 0x3F3F3F3Fu;
        const uint32_t sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
        const uint32_t mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
        const uint32_t sc2 = ((c & 2) ? sc_hi : sc_lo) >> ((c & 1) * 16);
        const uint32_t mn2 = ((c & 2) ? mn_hi : mn_lo) >> ((c & 1) * 16);
        const uint32_t w[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        int at = 0, bt = 0;
        uint32_t am = 0, al = 0, bm = 0, bl = 0;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const uint32_t lo = w[k] & 0x0F0F0F0Fu, hi = (w[k] >> 4) & 0x0F0F0F0Fu;
            at = sdot4(lo, xt[k], at);
            am = udot4(lo, xm[k], am);
            al = udot4(lo, xl[k], al);
            bt = sdot4(hi, xt[8 + k], bt);
            bm = udot4(hi, xm[8 + k], bm);
            bl = udot4(hi, xl[8 + k], bl);
        }
        /* |top| <= 32*15*64, mid/low <= 32*15*255: the low part fits an int exactly */
        const float fa = fmaf((float)at, 65536.0f, (float)((am << 8) + al)) * inv_a;
        const float fb = fmaf((float)bt, 65536.0f, (float)((bm << 8) + bl)) * inv_b;
        const float da = d * (float)(sc2 & 0xFFu), db = d * (float)((sc2 >> 8) & 0xFFu);
        const float ma = dmin * (float)(mn2 & 0xFFu), mb = dmin * (float)((mn2 >> 8) & 0xFFu);
        float v = active ? (da * fa + db * fb - (ma * sum_a + mb * sum_b)) : 0.0f;
        v = wave_sum_dpp(v);
        if (lane == 0) partial[wv + i * kWaves] = v;
    }
    __syncthreads();

    /* combine the slices of each row and store */
    auto row_total = [&](int lr) {
        float s = 0.0f;
        for (int k = 0; k < n_slices; k++) s += partial[lr * n_slices + k];
        return s;
    };
    if (paired) {
        for (int lr = threadIdx.x; lr < rows_here; lr += kThreads)
            job.y0[row0 + lr] = silu_times(row_total(lr), row_total(rows_here + lr));
    } else {
        for (int lr = threadIdx.x; lr < n_lrows; lr += kThreads) {
            const uint8_t *Wm;
            float *ym;
            int r;
            locate(lr, Wm, ym, r);
            const float s = row_total(lr);
            ym[r] = job.mode == 1 ? ym[r] + s : s;
        }
    }

}

/* Launch geometry: one 16-wave workgroup per block of rows, sized so that the grid covers the
 * compute units once (more workgroups only when a block would exceed kMaxRowsPerWg rows). */
hipError_t launch_gemv_q4k(const GemvJob &job, const float *x, int n_cols, hipStream_t stream, int n_cu) {
    static OnceFlag lds_raised;
    const int n_sb = n_cols / 256;
    if (n_sb > 64 || n_sb < 1) return hipErrorInvalidValue;
    const int n_slices = n_sb <= 16 ? 1 : n_sb <= 32 ? 2 : 4;
    const int slice_sb = (n_sb + n_slices - 1) / n_slices;
    const int n_mats_here = job.mode == kSiluMul ? 2 : 1;
    const int n_rows = job.mode == kSiluMul ? job.n_rows[0] : job.total_rows();
    if (n_rows == 0) return hipSuccess;
    int rows_per_wg = (n_rows + n_cu - 1) / n_cu;
    if (rows_per_wg < 1) rows_per_wg = 1;
    if (rows_per_wg * n_mats_here > kMaxRowsPerWg) rows_per_wg = kMaxRowsPerWg / n_mats_here;
    const int grid = (n_rows + rows_per_wg - 1) / rows_per_wg;
    const size_t fixed_bytes = (size_t)n_sb * 4 * kChunk * 4 + (size_t)n_sb * 4 * 16 +
                               (size_t)((rows_per_wg * n_mats_here * n_slices + 3) & ~3) * 4 + (size_t)n_sb * 256 * 4;
    if (fixed_bytes + (size_t)kWaves * kRowImage > 160 * 1024) return hipErrorInvalidValue;
    int depth = (int)((160 * 1024 - fixed_bytes) / ((size_t)kWaves * kRowImage));
    if (depth > kMaxDepth) depth = kMaxDepth;
    const size_t lds_bytes = fixed_bytes + (size_t)kWaves * depth * kRowImage;
    if (!lds_raised.is_set()) {
        hipError_t e = hipFuncSetAttribute((const void *)gemv_q4k_kernel,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        lds_raised.set();
    }
    const JobView view = job_view(job);
    hipLaunchKernelGGL(gemv_q4k_kernel, dim3(grid), dim3(kThreads), lds_bytes, stream, view, x, n_sb, n_slices,
                       slice_sb, rows_per_wg, depth);
    return hipGetLastError();
}

}  // namespace qlin
