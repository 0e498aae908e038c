/*
 * dequant.hip - block decoders: raw GGML blocks -> fp32, bit-identical to the reference's
 * scalar decoders (common/ggml_dequant.h:1479-1687, :2793-3058, type switch :3177-3265).
 *
 * One thread decodes eight consecutive elements and writes 32 contiguous bytes, so a
 * wavefront writes 2 KiB of contiguous fp32 per store pair. The kernel is bound by that
 * write stream (4 B out per 0.26..1.06 B in).
 */
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

template <uint32_t T, bool VEC>
__global__ void __launch_bounds__(256)
dequant_kernel(const uint8_t *__restrict__ W, const int32_t *__restrict__ row_ids, int n_src_rows,
               float *__restrict__ out, int n_rows, int n_cols, size_t row_bytes, int blocks_per_row) {
    using C = Codec<T>;
    constexpr int GPB = C::BE / 8; /* 8-element groups per block */
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long groups_per_row = (long long)blocks_per_row * GPB;
    if (gid >= groups_per_row * n_rows) return;
    const int row = (int)(gid / groups_per_row);
    const int g = (int)(gid - (long long)row * groups_per_row);
    const int blk = g / GPB, k0 = (g - blk * GPB) * 8;
    float y[8];
    /* output row `row` is source row row_ids[row] when a list is given (embedding lookup); an id
     * outside the table yields a row of zeros */
    const int src_row = row_ids ? row_ids[row] : row;
    if (src_row >= 0 && src_row < n_src_rows) {
        C::decode8(W + (size_t)src_row * row_bytes + (size_t)blk * C::BB, k0, y);
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = 0.0f;
    }
    float *o = out + (size_t)row * n_cols + (size_t)blk * C::BE + k0;
    if (VEC) {
        reinterpret_cast<float4 *>(o)[0] = make_float4(y[0], y[1], y[2], y[3]);
        reinterpret_cast<float4 *>(o)[1] = make_float4(y[4], y[5], y[6], y[7]);
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) o[i] = y[i];
    }
}

/* F16 / BF16 / F32 rows (common/ggml_dequant.h:3251-3261); output row r = source row row_ids[r]
 * when a list is given */
__global__ void __launch_bounds__(256)
convert_plain_kernel(uint32_t type, const uint8_t *__restrict__ src, const int32_t *__restrict__ row_ids,
                     int n_src_rows, float *__restrict__ out, long long n, int n_cols) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    long long s = i;
    if (row_ids) {
        const long long r = i / n_cols;
        const int id = row_ids[r];
        if (id < 0 || id >= n_src_rows) {
            out[i] = 0.0f;
            return;
        }
        s = (long long)id * n_cols + (i - r * n_cols);
    }
    if (type == T_F32) {
        reinterpret_cast<uint32_t *>(out)[i] = reinterpret_cast<const uint32_t *>(src)[s];
    } else {
        const uint32_t h = reinterpret_cast<const uint16_t *>(src)[s];
        out[i] = (type == T_F16) ? half_bits_exact(h) : __uint_as_float(h << 16);
    }
}

/* the same decode with the result rounded once to bf16 (nearest even) and stored 8 values = 16 bytes per
 * thread: the weight operand of the dense matrix-core GEMM */
template <uint32_t T>
__global__ void __launch_bounds__(256)
dequant_bf16_kernel(const uint8_t *__restrict__ W, uint16_t *__restrict__ out, int n_rows, int n_cols,
                    size_t row_bytes, int blocks_per_row) {
    using C = Codec<T>;
    constexpr int GPB = C::BE / 8;
    /* a thread decodes two 8-element groups half a workgroup's span apart, so that each of its two
     * 16-byte stores is part of a contiguous 4 KB of the workgroup */
    const long long groups_per_row = (long long)blocks_per_row * GPB;
    const long long n_groups = groups_per_row * n_rows;
    const long long base = (long long)blockIdx.x * 512 + threadIdx.x;
    typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const long long gid = base + 256 * h;
        if (gid >= n_groups) return;
        const int row = (int)(gid / groups_per_row);
        const int g = (int)(gid - (long long)row * groups_per_row);
        const int blk = g / GPB, k0 = (g - blk * GPB) * 8;
        float y[8];
        C::decode8(W + (size_t)row * row_bytes + (size_t)blk * C::BB, k0, y);
        uint4 v;
        uint32_t *vp = &v.x;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            bf16x2 r;
            r[0] = (__bf16)y[2 * i];
            r[1] = (__bf16)y[2 * i + 1];
            vp[i] = __builtin_bit_cast(uint32_t, r);
        }
        *reinterpret_cast<uint4 *>(out + (size_t)row * n_cols + (size_t)blk * C::BE + k0) = v;
    }
}

template <uint32_t T>
static hipError_t launch_bf16_typed(const void *W, uint16_t *out, int n_rows, int n_cols, size_t row_bytes,
                                    hipStream_t stream) {
    const int bpr = n_cols / Codec<T>::BE;
    const long long groups = (long long)bpr * (Codec<T>::BE / 8) * n_rows;
    if (groups == 0) return hipSuccess;
    hipLaunchKernelGGL((dequant_bf16_kernel<T>), dim3((unsigned)((groups + 511) / 512)), dim3(256), 0, stream,
                       (const uint8_t *)W, out, n_rows, n_cols, row_bytes, bpr);
    return hipGetLastError();
}

template <uint32_t T>
static hipError_t launch_typed(const void *W, const int32_t *row_ids, int n_src_rows, float *out, int n_rows,
                               int n_cols, size_t row_bytes, hipStream_t stream) {
    const int bpr = n_cols / Codec<T>::BE;
    const long long groups = (long long)bpr * (Codec<T>::BE / 8) * n_rows;
    if (groups == 0) return hipSuccess;
    const unsigned grid = (unsigned)((groups + 255) / 256);
    const bool vec = (n_cols % 4 == 0) && ((reinterpret_cast<uintptr_t>(out) & 15u) == 0);
    if (vec)
        hipLaunchKernelGGL((dequant_kernel<T, true>), dim3(grid), dim3(256), 0, stream,
                           (const uint8_t *)W, row_ids, n_src_rows, out, n_rows, n_cols, row_bytes, bpr);
    else
        hipLaunchKernelGGL((dequant_kernel<T, false>), dim3(grid), dim3(256), 0, stream,
                           (const uint8_t *)W, row_ids, n_src_rows, out, n_rows, n_cols, row_bytes, bpr);
    return hipGetLastError();
}

hipError_t launch_dequant(uint32_t type, const void *W, const int32_t *row_ids, int n_src_rows, float *out,
                          int n_rows, int n_cols, size_t row_bytes, hipStream_t stream) {
    if (!row_ids) n_src_rows = n_rows;
    switch (type) {
#define QLIN_CASE(TT) case TT: return launch_typed<TT>(W, row_ids, n_src_rows, out, n_rows, n_cols, row_bytes, stream);
    QLIN_FOR_EACH_BLOCK_TYPE(QLIN_CASE)
#undef QLIN_CASE
    case T_F32: case T_F16: case T_BF16: {
        const long long n = (long long)n_rows * n_cols;
        if (n == 0) return hipSuccess;
        hipLaunchKernelGGL(convert_plain_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream,
                           type, (const uint8_t *)W, row_ids, n_src_rows, out, n, n_cols);
        return hipGetLastError();
    }
    default: return hipErrorInvalidValue;
    }
}

/* out[r * n_cols + k] = bf16(decode(W)[r][k]); out 16-byte aligned, n_cols a multiple of the block size */
hipError_t launch_dequant_bf16(uint32_t type, const void *W, uint16_t *out, int n_rows, int n_cols, size_t row_bytes,
                               hipStream_t stream) {
    switch (type) {
#define QLIN_CASE(TT) case TT: return launch_bf16_typed<TT>(W, out, n_rows, n_cols, row_bytes, stream);
    QLIN_FOR_EACH_BLOCK_TYPE(QLIN_CASE)
    QLIN_FOR_EACH_DENSE_TYPE(QLIN_CASE)
#undef QLIN_CASE
    default: return hipErrorInvalidValue;
    }
}

}  // namespace qlin
