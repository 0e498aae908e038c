/*
 * qlinear_ggml.h - the codec and Q8_0 helpers of common/ggml_dequant.h under the reference's own names, over
 * libqlinear.so, for C code that was written against that header:
 *
 *   dequant_row, dequant_row_size          common/ggml_dequant.h:258, :261-294
 *   dequantize_row_<type> (24 + bf16)      :231-255
 *   ggml_fp16_to_fp32                      :206-229   (host inline, no GPU involved)
 *   vec_dot_q8_0_f32, matvec_q8_0_f32      :326-329   (one-row matvec on the GPU)
 *   gemm_q8_0_f32_tokmajor                 :331-334   (qlin_gemm_tokenmajor)
 *
 * The functions are always available with a qlin_ggml_ prefix; define QLINEAR_GGML_REFERENCE_NAMES before
 * including this header to also get the reference's names as macros. The decoders are bit-exact with the
 * reference's; the Q8_0 products accumulate in fp32 in another order than the CPU loop does (~1e-6 relative).
 * Where the reference cannot fail and the GPU can (no device, out of memory), the message goes to stderr and the
 * result is NaN (vec_dot) or left as qlin_matvec / qlin_gemm_tokenmajor leave it on failure.
 */
#ifndef QLINEAR_GGML_H
#define QLINEAR_GGML_H

#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "qlinear.h"

#ifdef __cplusplus
extern "C" {
#endif

#define QLIN_GGML_TYPE_Q8_0 8u

/* IEEE half -> float. The 15 magnitude bits are placed where a float keeps exponent and mantissa, which leaves the
 * exponent 112 short; one multiplication by 2^112 repairs that for normal and subnormal halves alike (exactly: the
 * product has at most 11 significant bits). Halves with all exponent bits set (infinities, NaNs) come out of the
 * product at 2^16 or more and get the float's all-ones exponent; their mantissa bits are already in place. */
static inline float qlin_ggml_fp16_to_fp32(uint16_t h) {
    uint32_t bits = (uint32_t)(h & 0x7FFFu) << 13;
    const uint32_t two_pow_112 = (uint32_t)(127 + 112) << 23;
    float mag, scale;
    memcpy(&mag, &bits, 4);
    memcpy(&scale, &two_pow_112, 4);
    mag *= scale;
    memcpy(&bits, &mag, 4);
    if (mag >= 65536.0f || mag != mag) bits |= 0x7F800000u;
    bits |= (uint32_t)(h & 0x8000u) << 16;
    memcpy(&mag, &bits, 4);
    return mag;
}

/* 0 on success, -1 if the type has no decoder (the reference's return values) */
static inline int qlin_ggml_dequant_row(uint32_t ggml_type, const void *src, float *dst, int n) {
    const int rc = qlin_dequant_row(ggml_type, src, dst, n);
    if (rc != QLIN_OK && rc != QLIN_ERR_TYPE) fprintf(stderr, "dequant_row: %s\n", qlin_last_error());
    return rc == QLIN_OK ? 0 : -1;
}

/* sum_i decode(q8_row)[i] * x[i], K a multiple of 32 */
static inline float qlin_ggml_vec_dot_q8_0_f32(const void *q8_row, const float *x, int K) {
    float r = 0.0f;
    if (qlin_matvec(&r, q8_row, QLIN_GGML_TYPE_Q8_0, K, x, 1) != QLIN_OK) {
        fprintf(stderr, "vec_dot_q8_0_f32: %s\n", qlin_last_error());
        return NAN;
    }
    return r;
}

static inline void qlin_ggml_matvec_q8_0_f32(float *dst, const void *q8_row, const float *x, int K) {
    *dst = qlin_ggml_vec_dot_q8_0_f32(q8_row, x, K);
}

/* Y[tok * Y_stride + row] = dot(W[row, :], X[tok * X_stride ...]); W Q8_0, rows of K / 32 blocks */
static inline void qlin_ggml_gemm_q8_0_f32_tokmajor(float *Y, const void *W, const float *X, int n_rows, int K, int N,
                                                    int Y_stride, int X_stride) {
    if (qlin_gemm_tokenmajor(Y, W, QLIN_GGML_TYPE_Q8_0, K, X, n_rows, N, Y_stride, X_stride) != QLIN_OK)
        fprintf(stderr, "gemm_q8_0_f32_tokmajor: %s\n", qlin_last_error());
}

#ifdef QLINEAR_GGML_REFERENCE_NAMES
#define ggml_fp16_to_fp32       qlin_ggml_fp16_to_fp32
#define dequant_row             qlin_ggml_dequant_row
#define dequant_row_size        qlin_dequant_row_size
#define vec_dot_q8_0_f32        qlin_ggml_vec_dot_q8_0_f32
#define matvec_q8_0_f32         qlin_ggml_matvec_q8_0_f32
#define gemm_q8_0_f32_tokmajor  qlin_ggml_gemm_q8_0_f32_tokmajor
#define dequantize_row_q2_K     qlin_dequantize_row_q2_K
#define dequantize_row_q3_K     qlin_dequantize_row_q3_K
#define dequantize_row_q8_0     qlin_dequantize_row_q8_0
#define dequantize_row_q1_0     qlin_dequantize_row_q1_0
#define dequantize_row_mxfp4    qlin_dequantize_row_mxfp4
#define dequantize_row_nvfp4    qlin_dequantize_row_nvfp4
#define dequantize_row_q4_K     qlin_dequantize_row_q4_K
#define dequantize_row_q5_K     qlin_dequantize_row_q5_K
#define dequantize_row_q6_K     qlin_dequantize_row_q6_K
#define dequantize_row_iq2_xxs  qlin_dequantize_row_iq2_xxs
#define dequantize_row_q4_0     qlin_dequantize_row_q4_0
#define dequantize_row_q4_1     qlin_dequantize_row_q4_1
#define dequantize_row_q5_0     qlin_dequantize_row_q5_0
#define dequantize_row_q5_1     qlin_dequantize_row_q5_1
#define dequantize_row_iq2_xs   qlin_dequantize_row_iq2_xs
#define dequantize_row_iq2_s    qlin_dequantize_row_iq2_s
#define dequantize_row_iq3_xxs  qlin_dequantize_row_iq3_xxs
#define dequantize_row_iq3_s    qlin_dequantize_row_iq3_s
#define dequantize_row_iq4_nl   qlin_dequantize_row_iq4_nl
#define dequantize_row_iq4_xs   qlin_dequantize_row_iq4_xs
#define dequantize_row_iq1_s    qlin_dequantize_row_iq1_s
#define dequantize_row_iq1_m    qlin_dequantize_row_iq1_m
#define dequantize_row_tq1_0    qlin_dequantize_row_tq1_0
#define dequantize_row_tq2_0    qlin_dequantize_row_tq2_0
#define dequantize_row_bf16     qlin_dequantize_row_bf16
#endif

#ifdef __cplusplus
}
#endif
#endif /* QLINEAR_GGML_H */
