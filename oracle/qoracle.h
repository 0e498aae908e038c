/*
 * qoracle.h - CPU oracle for the GGML block-quantized linear path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing here is part of the shipped library: only the test
 * suite, the smoke check and the benchmark's cpu_baseline leg may build, load or call it,
 * and there only as the checker / the reported CPU baseline - never as the product path.
 *
 * It restates, in plain C, the algorithm of the reference's CPU path:
 *   codec      common/ggml_dequant.h:206-229 (fp16), :261-294 (row size), :1479-1489 (Q8_0),
 *              :1582-1687 (Q4_K/Q5_K/Q6_K), :2793-2816 (IQ2_XXS), :2942-2954 (IQ4_NL),
 *              :3022-3058 (IQ3_S), :3177-3265 (type switch); the other seventeen block
 *              formats of that switch are in qoracle_ext.c, cited per function there
 *   matvec     common/transformer.h:651-660 (double-accumulate oracle mode),
 *              :1049-1114 (fp32 path: dequantize row to scratch, 4x8-lane FMA dot),
 *              common/ggml_dequant.h:953-998 (Q8_0 fused dequant-dot), :1117-1133 of
 *              transformer.h (static row partition over threads)
 *   prefill    common/transformer.h:4535-4572 (per-token re-dequant fallback, token-major Y)
 *   MoE FFN    common/transformer.h:4045-4131 (softmax, top-k min-heap, renormalise,
 *              per-expert up/gate/SiLU/down, weighted sum), :517-548 (expert slice addressing)
 *
 * Parity status of each function is listed in the header comment of qoracle.c.
 */
#ifndef QORACLE_H
#define QORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids, values of enum ggml_dtype (common/gguf_loader.h:45-85) */
enum {
    QO_TYPE_F32 = 0, QO_TYPE_F16 = 1, QO_TYPE_Q8_0 = 8, QO_TYPE_Q4_K = 12, QO_TYPE_Q5_K = 13,
    QO_TYPE_Q6_K = 14, QO_TYPE_IQ2_XXS = 16, QO_TYPE_IQ4_NL = 20, QO_TYPE_IQ3_S = 21,
    QO_TYPE_BF16 = 30,
    /* the further block formats of the type switch (decoders in qoracle_ext.c) */
    QO_TYPE_Q4_0 = 2, QO_TYPE_Q4_1 = 3, QO_TYPE_Q5_0 = 6, QO_TYPE_Q5_1 = 7, QO_TYPE_Q2_K = 10,
    QO_TYPE_Q3_K = 11, QO_TYPE_IQ2_XS = 17, QO_TYPE_IQ3_XXS = 18, QO_TYPE_IQ1_S = 19,
    QO_TYPE_IQ2_S = 22, QO_TYPE_IQ4_XS = 23, QO_TYPE_IQ1_M = 29, QO_TYPE_TQ1_0 = 34,
    QO_TYPE_TQ2_0 = 35, QO_TYPE_MXFP4 = 39, QO_TYPE_NVFP4 = 40, QO_TYPE_Q1_0 = 41
};

/* ---- codec ---- */
float  qo_fp16_to_fp32(uint16_t h);
/* out[65536]: every half-precision bit pattern converted */
void   qo_fp16_table(float *out);
/* bytes of one row of n elements; 0 for an unknown type */
size_t qo_row_size(uint32_t type, int n);
/* elements per block / bytes per block; 0 for an unknown type */
int    qo_block_elems(uint32_t type);
int    qo_block_bytes(uint32_t type);

void qo_dequantize_row_q8_0(const void *src, float *dst, int n);
void qo_dequantize_row_q4_K(const void *src, float *dst, int n);
void qo_dequantize_row_q5_K(const void *src, float *dst, int n);
void qo_dequantize_row_q6_K(const void *src, float *dst, int n);
void qo_dequantize_row_iq2_xxs(const void *src, float *dst, int n);
void qo_dequantize_row_iq4_nl(const void *src, float *dst, int n);
void qo_dequantize_row_iq3_s(const void *src, float *dst, int n);
/* further formats (common/ggml_dequant.h:1491-1580 q1_0/q2_K/q3_K, :2818-2914 mxfp4/nvfp4/q4_0/
 * q4_1/q5_0/q5_1, :2916-3020 iq3_xxs/iq4_xs/iq2_xs/iq2_s, :3062-3175 iq1_s/iq1_m/tq1_0/tq2_0) */
void qo_dequantize_row_q4_0(const void *src, float *dst, int n);
void qo_dequantize_row_q4_1(const void *src, float *dst, int n);
void qo_dequantize_row_q5_0(const void *src, float *dst, int n);
void qo_dequantize_row_q5_1(const void *src, float *dst, int n);
void qo_dequantize_row_q2_K(const void *src, float *dst, int n);
void qo_dequantize_row_q3_K(const void *src, float *dst, int n);
void qo_dequantize_row_q1_0(const void *src, float *dst, int n);
void qo_dequantize_row_mxfp4(const void *src, float *dst, int n);
void qo_dequantize_row_nvfp4(const void *src, float *dst, int n);
void qo_dequantize_row_iq3_xxs(const void *src, float *dst, int n);
void qo_dequantize_row_iq4_xs(const void *src, float *dst, int n);
void qo_dequantize_row_iq2_xs(const void *src, float *dst, int n);
void qo_dequantize_row_iq2_s(const void *src, float *dst, int n);
void qo_dequantize_row_iq1_s(const void *src, float *dst, int n);
void qo_dequantize_row_iq1_m(const void *src, float *dst, int n);
void qo_dequantize_row_tq1_0(const void *src, float *dst, int n);
void qo_dequantize_row_tq2_0(const void *src, float *dst, int n);
/* scale bytes of MXFP4 (E8M0, halved) and NVFP4 (unsigned E4M3, halved) */
float qo_e8m0_half_to_fp32(uint8_t e);
float qo_ue4m3_half_to_fp32(uint8_t x);
/* 6-bit scale i (0..15) of a Q3_K block's 12 packed scale bytes, before the -32 offset */
int  qo_q3k_scale(const uint8_t packed[12], int i);
/* 0 on success, -1 for an unsupported type (dst untouched) */
int  qo_dequant_row(uint32_t type, const void *src, float *dst, int n);

/* unpack the 12 packed bytes of a Q4_K/Q5_K super-block into 8 scales and 8 mins */
void qo_k4_unpack_scales(const uint8_t packed[12], uint8_t sc[8], uint8_t mn[8]);
/* inverse: pack 8 six-bit scales and 8 six-bit mins into 12 bytes */
void qo_k4_pack_scales(const uint8_t sc[8], const uint8_t mn[8], uint8_t packed[12]);

/* raw access to the codebooks, for checksum tests */
const void *qo_table(const char *name, size_t *bytes);
const void *qo_table_ext(const char *name, size_t *bytes);

/* ---- matvec y[n_rows] = W . x ---- */
/* dequantize each row to fp32, dot in double, round once to fp32 */
int qo_gemv_f64(uint32_t type, const void *W, const float *x, float *y, int n_rows, int n_cols);
/* fp32 path in the reference's shape; rows statically partitioned over n_threads */
int qo_gemv_f32(uint32_t type, const void *W, const float *x, float *y, int n_rows, int n_cols,
                int n_threads);
/* times `iters` back-to-back calls on persistent threads; returns seconds per call, <0 on error */
double qo_gemv_f32_time(uint32_t type, const void *W, const float *x, float *y, int n_rows,
                        int n_cols, int n_threads, int iters);

/* ---- prefill GEMM, token-major: Y[t*out_stride + r] = dot(W[r,:], X[t*x_stride ..]) ---- */
int qo_gemm_tokmajor_f64(uint32_t type, const void *W, const float *X, float *Y, int n_rows,
                         int n_cols, int n_tok, int out_stride, int x_stride);
int qo_gemm_tokmajor_f32(uint32_t type, const void *W, const float *X, float *Y, int n_rows,
                         int n_cols, int n_tok, int out_stride, int x_stride);

/* ---- MoE FFN ---- */
/* softmax over all experts, top-k by single-pass min-heap with strict '>', renormalise by the
 * sum of the selected weights. idx/w come out in heap order, like the reference. */
void qo_moe_route(const float *logits, int n_expert, int top_k, int *idx, float *w);
/* one token: out[n_embd] = sum_k w_k * down_{e_k}( silu(gate_{e_k} x) * up_{e_k} x ).
 * Expert tensors are [n_expert][rows][cols] slices of one ggml type; accumulation in double. */
int qo_moe_ffn_token_f64(uint32_t type, const void *gate, const void *up, const void *down,
                         int n_embd, int n_ff, const float *x, const int *idx, const float *w,
                         int top_k, float *out);
/* same, all arithmetic in fp32 in the reference's order (the timed CPU baseline) */
int qo_moe_ffn_token_f32(uint32_t type, const void *gate, const void *up, const void *down,
                         int n_embd, int n_ff, const float *x, const int *idx, const float *w,
                         int top_k, float *out);
/* the three matrices in a format each; use_f64 as the two above */
int qo_moe_ffn_token_types(uint32_t type_gate, uint32_t type_up, uint32_t type_down, const void *gate, const void *up,
                           const void *down, int n_embd, int n_ff, const float *x, const int *idx, const float *w,
                           int top_k, float *out, int use_f64);

#ifdef __cplusplus
}
#endif
#endif /* QORACLE_H */
