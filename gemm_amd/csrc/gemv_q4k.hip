/*
 * gemv_q4k.hip - batch-1 Q4_K matvec tuned for HBM streaming on gfx950.
 *
 * Work split. A row of K columns is K/256 super-blocks of 144 bytes (common/ggml_dequant.h:71-76).
 * Four lanes own one super-block: lane c (0..3) takes the 32 nibble bytes qs[32c..32c+31], i.e.
 * the 64 elements of sub-blocks 2c (low nibbles) and 2c+1 (high nibbles). A wavefront therefore
 * covers a slice of up to 16 super-blocks (4096 columns) of one row per pass. The slice of x a
 * wavefront needs (64 floats per lane) is loaded ONCE and stays in registers while the
 * wavefront streams R rows per pass: the raw 32 nibble bytes and the 16-byte block header
 * (d, dmin, 12 packed scale bytes) of all R rows are requested before any arithmetic starts,
 * so each wave keeps R*48 bytes per lane in flight.
 * Rows longer than 16 super-blocks are cut into S slices handled by the S waves of a
 * workgroup, whose partial sums meet in LDS.
 *
 * Arithmetic, per row and lane (factored form of common/ggml_dequant.h:1592-1618 dotted with x):
 *   y += d*sc_a*sum(q_lo*x_a) + d*sc_b*sum(q_hi*x_b) - dmin*(m_a*sum(x_a) + m_b*sum(x_b))
 * sum(x_a), sum(x_b) do not depend on the row and are formed once per wave. The eight 6-bit
 * scales and mins of a super-block are unpacked four at a time with byte-parallel mask ops.
 * High nibbles are used as 16*q (masked in place, no shift); the 1/16 goes into the scale.
 * fp32 accumulate throughout; result within ~1e-6 relative L2 of the double-precision oracle.
 */
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

__device__ __forceinline__ float ub0(uint32_t v) { return (float)(v & 0xFFu); }
__device__ __forceinline__ float ub1(uint32_t v) { return (float)((v >> 8) & 0xFFu); }
__device__ __forceinline__ float ub2(uint32_t v) { return (float)((v >> 16) & 0xFFu); }
__device__ __forceinline__ float ub3(uint32_t v) { return (float)(v >> 24); }

/* Per-lane scale terms for sub-blocks 2c and 2c+1 from the block header.
 * hdr.x = d | dmin << 16 (two halves), hdr.y/z/w = the 12 packed scale bytes.
 * Bytes 0..3 of (y & 0x3F..) are scales 0..3, of (z & 0x3F..) mins 0..3; scales 4..7 are
 * (w & 0x0F..) | ((y >> 2) & 0x30..), mins 4..7 are ((w >> 4) & 0x0F..) | ((z >> 2) & 0x30..)
 * (get_scale_min_k4, common/ggml_dequant.h:1582-1590, four fields per operation). */
__device__ __forceinline__ void q4k_lane_scales(const uint4 hdr, int c, float &da, float &db16,
                                                float &ma, float &mb) {
    const float d = half_bits_fast(hdr.x & 0xFFFFu);
    const float dmin = half_bits_fast(hdr.x >> 16);
    const uint32_t sc_lo = hdr.y & 0x3F3F3F3Fu;
    const uint32_t mn_lo = hdr.z & 0x3F3F3F3Fu;
    const uint32_t sc_hi = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
    const uint32_t mn_hi = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
    const uint32_t sc4 = (c & 2) ? sc_hi : sc_lo;
    const uint32_t mn4 = (c & 2) ? mn_hi : mn_lo;
    const uint32_t sh = (c & 1) * 16;
    const uint32_t sc2 = sc4 >> sh, mn2 = mn4 >> sh;
    da = d * ub0(sc2);
    db16 = d * ub1(sc2) * 0.0625f;
    ma = dmin * ub0(mn2);
    mb = dmin * ub1(mn2);
}

template <int R>
__global__ void __launch_bounds__(256)
gemv_q4k_kernel(const uint8_t *__restrict__ W, const float *__restrict__ x, float *__restrict__ y,
                int n_rows, int n_sb, int slice_sb, int n_slices, int rows_per_wave) {
    __shared__ float partial[4][8];
    const int lane = threadIdx.x & 63;
    const int wv = threadIdx.x >> 6;
    const int waves_per_wg = blockDim.x >> 6;
    const int slice = (n_slices == 1) ? 0 : wv;
    const int rowset = (n_slices == 1) ? blockIdx.x * waves_per_wg + wv : blockIdx.x;
    const int sb0 = slice * slice_sb;
    int sb_cnt = n_sb - sb0;
    if (sb_cnt > slice_sb) sb_cnt = slice_sb;
    const int c = lane & 3;
    const bool active = (lane >> 2) < sb_cnt;
    const int sb = sb0 + (active ? (lane >> 2) : 0); /* idle lanes re-read block sb0, scaled by 0 */
    const size_t row_bytes = (size_t)n_sb * 144;

    /* this lane's 64 x values: xa = elements of sub-block 2c, xb = of sub-block 2c+1 */
    float xa[32], xb[32];
    {
        const float4 *xp = reinterpret_cast<const float4 *>(x + (size_t)sb * 256 + 64 * c);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float4 v = xp[i], u = xp[8 + i];
            xa[4 * i] = v.x; xa[4 * i + 1] = v.y; xa[4 * i + 2] = v.z; xa[4 * i + 3] = v.w;
            xb[4 * i] = u.x; xb[4 * i + 1] = u.y; xb[4 * i + 2] = u.z; xb[4 * i + 3] = u.w;
        }
    }
    float sxa = 0.0f, sxb = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) { sxa += xa[i]; sxb += xb[i]; }

    const int row_begin = rowset * rows_per_wave;
    for (int p = 0; p < rows_per_wave; p += R) {
        uint4 hdr[R], q0[R], q1[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            int row = row_begin + p + r;
            if (row >= n_rows) row = n_rows - 1; /* keep the load in bounds; result discarded */
            const uint8_t *blk = W + (size_t)row * row_bytes + (size_t)sb * 144;
            hdr[r] = *reinterpret_cast<const uint4 *>(blk);
            q0[r] = *reinterpret_cast<const uint4 *>(blk + 16 + 32 * c);
            q1[r] = *reinterpret_cast<const uint4 *>(blk + 32 + 32 * c);
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            float da, db16, ma, mb;
            q4k_lane_scales(hdr[r], c, da, db16, ma, mb);
            const uint32_t w[8] = {q0[r].x, q0[r].y, q0[r].z, q0[r].w, q1[r].x, q1[r].y, q1[r].z, q1[r].w};
            float sa = 0.0f, sb_ = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const uint32_t lo = w[i] & 0x0F0F0F0Fu;
                const uint32_t hi = w[i] & 0xF0F0F0F0u;
                sa += ub0(lo) * xa[4 * i] + ub1(lo) * xa[4 * i + 1] + ub2(lo) * xa[4 * i + 2] + ub3(lo) * xa[4 * i + 3];
                sb_ += ub0(hi) * xb[4 * i] + ub1(hi) * xb[4 * i + 1] + ub2(hi) * xb[4 * i + 2] + ub3(hi) * xb[4 * i + 3];
            }
            float v = active ? (da * sa + db16 * sb_ - (ma * sxa + mb * sxb)) : 0.0f;
            v = wave_sum(v);
            const int row = row_begin + p + r;
            if (n_slices == 1) {
                if (lane == 0 && row < n_rows && p + r < rows_per_wave) y[row] = v;
            } else {
                if (lane == 0) partial[wv][r] = v;
            }
        }
        if (n_slices > 1) {
            __syncthreads();
            if (threadIdx.x < R) {
                const int row = row_begin + p + threadIdx.x;
                float s = 0.0f;
                for (int k = 0; k < n_slices; k++) s += partial[k][threadIdx.x];
                if (row < n_rows && p + (int)threadIdx.x < rows_per_wave) y[row] = s;
            }
            __syncthreads();
        }
    }
}

/* Launch geometry: slices of at most 16 super-blocks; rows per wave chosen so that the grid
 * fills the 256 compute units evenly with about `target_waves_per_cu` waves each. */
hipError_t launch_gemv_q4k(const void *W, const float *x, float *y, int n_rows, int n_cols,
                           hipStream_t stream, int n_cu, int rows_per_pass, int target_waves_per_cu) {
    const int n_sb = n_cols / 256;
    const int n_slices = (n_sb + 15) / 16;
    if (n_slices > 4) return hipErrorInvalidValue;
    const int slice_sb = (n_sb + n_slices - 1) / n_slices;
    const int waves_per_wg = (n_slices == 1) ? 4 : n_slices;
    /* row sets = groups of rows handled by one wave (or one workgroup of slice-waves) */
    const int wave_groups_target = n_cu * target_waves_per_cu / n_slices;
    int rpw = (n_rows + wave_groups_target - 1) / wave_groups_target;
    if (rpw < 1) rpw = 1;
    const int rowsets = (n_rows + rpw - 1) / rpw;
    const int grid = (n_slices == 1) ? (rowsets + waves_per_wg - 1) / waves_per_wg : rowsets;
    const dim3 block(64 * waves_per_wg);
#define QLIN_Q4K_LAUNCH(RR)                                                                     \
    hipLaunchKernelGGL((gemv_q4k_kernel<RR>), dim3(grid), block, 0, stream, (const uint8_t *)W, \
                       x, y, n_rows, n_sb, slice_sb, n_slices, rpw)
    switch (rows_per_pass) {
    case 1: QLIN_Q4K_LAUNCH(1); break;
    case 2: QLIN_Q4K_LAUNCH(2); break;
    case 4: QLIN_Q4K_LAUNCH(4); break;
    case 7: QLIN_Q4K_LAUNCH(7); break;
    case 8: QLIN_Q4K_LAUNCH(8); break;
    default: return hipErrorInvalidValue;
    }
#undef QLIN_Q4K_LAUNCH
    return hipGetLastError();
}

}  // namespace qlin
