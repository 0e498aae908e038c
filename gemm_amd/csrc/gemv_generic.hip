/*
 * gemv_generic.hip - y = W.x and Y = X.W^T in fp32 for every supported block type.
 *
 * The plain path: correct for any shape made of whole blocks, used for types and shapes the
 * tuned kernels do not take. A wavefront owns R consecutive rows; its lanes stride over
 * 8-element groups of the row, decode them in registers and FMA them with x (read as two
 * float4 per group, contiguous across the lanes). fp32 accumulate, wave64 shuffle reduction.
 * Computes what tf_qmatvec computes (common/transformer.h:1049-1114): the dot of each
 * decoded row with x; only the summation order differs.
 */
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

template <uint32_t T>
__global__ void __launch_bounds__(256)
gemv_generic_kernel(const JobView job, const float *__restrict__ x, int n_cols, size_t row_bytes) {
    using C = Codec<T>;
    constexpr int GPB = C::BE / 8;
    constexpr int R = 2;
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    /* the wave's two rows: consecutive rows of the concatenated matrices, or (mode 2) row `wave` of
     * the first and of the second matrix */
    const bool paired = job.mode == 2;
    const int n_rows = paired ? job.n0 : job.n0 + job.n1 + job.n2;
    const uint8_t *Wr[R];
    float *yr[R];
    int rr[R];
    bool live[R];
    if (paired) {
        if (wave >= n_rows) return;
        Wr[0] = job.W0; Wr[1] = job.W1; yr[0] = yr[1] = job.y0; rr[0] = rr[1] = wave; live[0] = live[1] = true;
    } else {
        if (wave * R >= n_rows) return;
#pragma unroll
        for (int r = 0; r < R; r++) {
            live[r] = wave * R + r < n_rows;
            job_locate(job, live[r] ? wave * R + r : 0, Wr[r], yr[r], rr[r]);
        }
    }
    const int groups = (n_cols / C::BE) * GPB;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;
    for (int g = lane; g < groups; g += 64) {
        const int blk = g / GPB, k0 = (g - blk * GPB) * 8;
        const float4 xa = *reinterpret_cast<const float4 *>(x + (size_t)blk * C::BE + k0);
        const float4 xb = *reinterpret_cast<const float4 *>(x + (size_t)blk * C::BE + k0 + 4);
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (live[r]) {
                float w[8];
                C::decode8(Wr[r] + (size_t)rr[r] * row_bytes + (size_t)blk * C::BB, k0, w);
                acc[r] += w[0] * xa.x + w[1] * xa.y + w[2] * xa.z + w[3] * xa.w +
                          w[4] * xb.x + w[5] * xb.y + w[6] * xb.z + w[7] * xb.w;
            }
        }
    }
    float s[R];
#pragma unroll
    for (int r = 0; r < R; r++) s[r] = wave_sum(acc[r]);
    if (lane != 0) return;
    if (paired) {
        yr[0][rr[0]] = silu_times(s[0], s[1]);
    } else {
#pragma unroll
        for (int r = 0; r < R; r++)
            if (live[r]) yr[r][rr[r]] = job.mode == 1 ? yr[r][rr[r]] + s[r] : s[r];
    }
}

/* dense rows whose length is not a multiple of eight elements, or that start off a 16-byte boundary: one
 * wave per row (mode 2: per row pair), one element per lane and step, scalar loads. tf_qmatvec takes such
 * rows (common/transformer.h:1049-1114: F32/F16/BF16 rows are dotted element by element). */
template <uint32_t T>
__global__ void __launch_bounds__(256)
gemv_dense_ragged_kernel(const JobView job, const float *__restrict__ x, int n_cols) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const bool paired = job.mode == 2;
    const int n_rows = paired ? job.n0 : job.n0 + job.n1 + job.n2;
    if (wave >= n_rows) return;
    auto dot = [&](const uint8_t *W, int r) {
        float acc = 0.0f;
        if (T == T_F32) {
            const float *row = reinterpret_cast<const float *>(W) + (size_t)r * n_cols;
            for (int k = lane; k < n_cols; k += 64) acc += row[k] * x[k];
        } else {
            const uint16_t *row = reinterpret_cast<const uint16_t *>(W) + (size_t)r * n_cols;
            for (int k = lane; k < n_cols; k += 64) {
                const uint32_t h = row[k];
                acc += (T == T_F16 ? half_bits_exact(h) : __uint_as_float(h << 16)) * x[k];
            }
        }
        return wave_sum(acc);
    };
    if (paired) {
        const float g = dot(job.W0, wave), u = dot(job.W1, wave);
        if (lane == 0) job.y0[wave] = silu_times(g, u);
    } else {
        const uint8_t *Wm;
        float *ym;
        int r;
        job_locate(job, wave, Wm, ym, r);
        const float s = dot(Wm, r);
        if (lane == 0) ym[r] = job.mode == 1 ? ym[r] + s : s;
    }
}

hipError_t launch_gemv_dense_ragged(uint32_t type, const GemvJob &job, const float *x, int n_cols, hipStream_t s) {
    const int waves = job.mode == kSiluMul ? job.n_rows[0] : job.total_rows();
    if (waves == 0) return hipSuccess;
    const JobView view = job_view(job);
    const dim3 grid((waves + 3) / 4), block(256);
    switch (type) {
    case T_F32: hipLaunchKernelGGL((gemv_dense_ragged_kernel<T_F32>), grid, block, 0, s, view, x, n_cols); break;
    case T_F16: hipLaunchKernelGGL((gemv_dense_ragged_kernel<T_F16>), grid, block, 0, s, view, x, n_cols); break;
    case T_BF16: hipLaunchKernelGGL((gemv_dense_ragged_kernel<T_BF16>), grid, block, 0, s, view, x, n_cols); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

/* Dense F32 / F16 / BF16 rows of more than 4096 elements (whole groups of eight, 16-byte aligned): x in LDS as
 * fp32, a wave per row, eight elements per lane and step straight from HBM into registers. The streaming kernel
 * (gemv_stream.hip) keeps whole rows in LDS and would take such rows as column ranges, a launch each
 * (BF16 4096 x 14336: 30.8 us in four launches, 22.6 us here; F32 54.6 -> 41.5). Stores or adds; no gate+up
 * pairing. Rows of more than 16384 elements come as column ranges of this kernel. */
template <uint32_t T>
__global__ void __launch_bounds__(1024)
gemv_dense_long_kernel(const JobView job, const float *__restrict__ x, int n_cols, int rows_per_wg, size_t row_bytes) {
    using C = Codec<T>;
    constexpr int kChunk = T == T_F32 ? 32 : 16; /* bytes of eight elements */
    extern __shared__ __attribute__((aligned(16))) float xs_long[];
    for (int i = threadIdx.x * 4; i < n_cols; i += blockDim.x * 4)
        *reinterpret_cast<float4 *>(xs_long + i) = *reinterpret_cast<const float4 *>(x + i);
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n_waves = blockDim.x >> 6;
    const int n_rows = job.n0 + job.n1 + job.n2;
    const int row0 = blockIdx.x * rows_per_wg;
    int rows_here = n_rows - row0;
    if (rows_here > rows_per_wg) rows_here = rows_per_wg;
    const int n8 = n_cols >> 3;
    for (int lr = wv; lr < rows_here; lr += n_waves) {
        const uint8_t *Wm;
        float *ym;
        int r;
        job_locate(job, row0 + lr, Wm, ym, r);
        const uint8_t *row = Wm + (size_t)r * row_bytes;
        float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll 4
        for (int c = lane; c < n8; c += 64) {
            float w[8];
            if (T == T_F16) { /* the conversion instruction: exact for every finite half (a signalling NaN comes out quiet) */
                const uint4 v = *reinterpret_cast<const uint4 *>(row + (size_t)c * kChunk);
                const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    w[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(d[i] & 0xFFFFu));
                    w[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(d[i] >> 16));
                }
            } else {
                C::decode8(row + (size_t)c * kChunk, 0, w);
            }
            const float4 xa = *reinterpret_cast<const float4 *>(xs_long + 8 * c);
            const float4 xb = *reinterpret_cast<const float4 *>(xs_long + 8 * c + 4);
            acc0 = fmaf(w[0], xa.x, fmaf(w[1], xa.y, fmaf(w[2], xa.z, fmaf(w[3], xa.w, acc0))));
            acc1 = fmaf(w[4], xb.x, fmaf(w[5], xb.y, fmaf(w[6], xb.z, fmaf(w[7], xb.w, acc1))));
        }
        const float s = wave_sum(acc0 + acc1);
        if (lane == 0) ym[r] = job.mode == 1 ? ym[r] + s : s;
    }
}

bool launch_gemv_dense_long(uint32_t type, const GemvJob &job, const float *x, int n_cols, int n_cu, hipStream_t stream,
                            hipError_t *err, size_t row_stride) {
    *err = hipSuccess;
    if (type != T_F32 && type != T_F16 && type != T_BF16) return false;
    if (job.mode == kSiluMul || n_cols <= 4096 || n_cols > 16384 || n_cols % 8 != 0 || ((uintptr_t)x & 15)) return false;
    for (int m = 0; m < job.n_mat; m++)
        if ((uintptr_t)job.W[m] & 15) return false;
    const int n_rows = job.total_rows();
    if (n_rows == 0) return false;
    int rows_per_wg = (n_rows + n_cu - 1) / n_cu;
    if (rows_per_wg < 1) rows_per_wg = 1;
    const int grid = (n_rows + rows_per_wg - 1) / rows_per_wg;
    const int waves = rows_per_wg >= 16 ? 16 : rows_per_wg >= 4 ? rows_per_wg : 4; /* a wave per row where they are few */
    const size_t lds_bytes = (size_t)n_cols * 4;
    /* rows that are a column range of longer ones keep those rows' pitch */
    const size_t row_bytes = row_stride ? row_stride : (size_t)n_cols * (type == T_F32 ? 4 : 2);
    if (row_bytes & 15) return false;
    const JobView view = job_view(job);
    switch (type) {
    case T_F32: hipLaunchKernelGGL((gemv_dense_long_kernel<T_F32>), dim3(grid), dim3(waves * 64), lds_bytes, stream, view, x, n_cols, rows_per_wg, row_bytes); break;
    case T_F16: hipLaunchKernelGGL((gemv_dense_long_kernel<T_F16>), dim3(grid), dim3(waves * 64), lds_bytes, stream, view, x, n_cols, rows_per_wg, row_bytes); break;
    default: hipLaunchKernelGGL((gemv_dense_long_kernel<T_BF16>), dim3(grid), dim3(waves * 64), lds_bytes, stream, view, x, n_cols, rows_per_wg, row_bytes); break;
    }
    *err = hipGetLastError();
    return true;
}

/* prefill in fp32: a wavefront owns one weight row and TT tokens at a time; the row is
 * decoded once per token tile. Y is token-major. (Semantics of the reference's generic
 * prefill path, common/transformer.h:4535-4572.) */
template <uint32_t T, int TT>
__global__ void __launch_bounds__(256)
gemm_f32_generic_kernel(const uint8_t *__restrict__ W, const float *__restrict__ X, float *__restrict__ Y,
                        int n_rows, int n_cols, int n_tok, int ldx, int ldy, size_t row_bytes) {
    using C = Codec<T>;
    constexpr int GPB = C::BE / 8;
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const int t0 = blockIdx.y * TT;
    const int groups = (n_cols / C::BE) * GPB;
    float acc[TT];
#pragma unroll
    for (int t = 0; t < TT; t++) acc[t] = 0.0f;
    for (int g = lane; g < groups; g += 64) {
        const int blk = g / GPB, k0 = (g - blk * GPB) * 8;
        float w[8];
        C::decode8(W + (size_t)row * row_bytes + (size_t)blk * C::BB, k0, w);
#pragma unroll
        for (int t = 0; t < TT; t++) {
            if (t0 + t < n_tok) {
                const float *xp = X + (size_t)(t0 + t) * ldx + (size_t)blk * C::BE + k0;
#pragma unroll
                for (int i = 0; i < 8; i++) acc[t] += w[i] * xp[i];
            }
        }
    }
#pragma unroll
    for (int t = 0; t < TT; t++) {
        const float s = wave_sum(acc[t]);
        if (lane == 0 && t0 + t < n_tok) Y[(size_t)(t0 + t) * ldy + row] = s;
    }
}

template <uint32_t T>
static hipError_t gemv_typed(const GemvJob &job, const float *x, int n_cols, hipStream_t s) {
    const size_t rb = (size_t)(n_cols / Codec<T>::BE) * Codec<T>::BB;
    const int waves = job.mode == kSiluMul ? job.n_rows[0] : (job.total_rows() + 1) / 2;
    if (waves == 0) return hipSuccess;
    const JobView view = job_view(job);
    hipLaunchKernelGGL((gemv_generic_kernel<T>), dim3((waves + 3) / 4), dim3(256), 0, s, view, x, n_cols, rb);
    return hipGetLastError();
}

hipError_t launch_gemv_generic(uint32_t type, const GemvJob &job, const float *x, int n_cols, hipStream_t s) {
    switch (type) {
#define QLIN_CASE(TT) case TT: return gemv_typed<TT>(job, x, n_cols, s);
    QLIN_FOR_EACH_BLOCK_TYPE(QLIN_CASE)
    QLIN_FOR_EACH_DENSE_TYPE(QLIN_CASE)
#undef QLIN_CASE
    default: return hipErrorInvalidValue;
    }
}

template <uint32_t T>
static hipError_t gemm_typed(const void *W, const float *X, float *Y, int n_rows, int n_cols, int n_tok,
                             int ldx, int ldy, hipStream_t s) {
    constexpr int TT = 8;
    const size_t rb = (size_t)(n_cols / Codec<T>::BE) * Codec<T>::BB;
    dim3 grid((n_rows + 3) / 4, (n_tok + TT - 1) / TT);
    hipLaunchKernelGGL((gemm_f32_generic_kernel<T, TT>), grid, dim3(256), 0, s, (const uint8_t *)W, X, Y,
                       n_rows, n_cols, n_tok, ldx, ldy, rb);
    return hipGetLastError();
}

hipError_t launch_gemm_f32(uint32_t type, const void *W, const float *X, float *Y, int n_rows,
                           int n_cols, int n_tok, int ldx, int ldy, hipStream_t s) {
    if (n_rows == 0 || n_tok == 0) return hipSuccess;
    switch (type) {
#define QLIN_CASE(TT) case TT: return gemm_typed<TT>(W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, s);
    QLIN_FOR_EACH_BLOCK_TYPE(QLIN_CASE)
    QLIN_FOR_EACH_DENSE_TYPE(QLIN_CASE)
#undef QLIN_CASE
    default: return hipErrorInvalidValue;
    }
}

}  // namespace qlin
