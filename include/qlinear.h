/*
 * qlinear.h - C ABI of the MI355X (gfx950) quantized-linear engine.
 *
 * GGML block dequantization and quantized matvec / matmul / MoE expert FFN on one GPU, behind
 * plain-C entry points (pointers and sizes only). The first two groups below have the shapes
 * of the reference's own C functions so that a C engine built like common/transformer.h can
 * call them where it calls its CPU path today; the third group works on device-resident
 * buffers (no copies per call) for engines that keep activations on the GPU.
 *
 * Supported ggml types (ids are enum ggml_dtype, common/gguf_loader.h:45-85): all 24 block formats with
 * a decoder in common/ggml_dequant.h - Q4_0 = 2, Q4_1 = 3, Q5_0 = 6, Q5_1 = 7, Q8_0 = 8, Q2_K = 10,
 * Q3_K = 11, Q4_K = 12, Q5_K = 13, Q6_K = 14, IQ2_XXS = 16, IQ2_XS = 17, IQ3_XXS = 18, IQ1_S = 19,
 * IQ4_NL = 20, IQ3_S = 21, IQ2_S = 22, IQ4_XS = 23, IQ1_M = 29, TQ1_0 = 34, TQ2_0 = 35, MXFP4 = 39,
 * NVFP4 = 40, Q1_0 = 41 - and the dense F32 = 0 / F16 = 1 / BF16 = 30 rows.
 *
 * Every function returns a status (0 = ok, negative = error) unless it mirrors a `void`
 * reference function, in which case it reports on stderr and zero-fills its output the way
 * the reference does for an unsupported type (common/transformer.h:451-454, :520-523).
 * There is no CPU fallback anywhere: without a usable GPU every call fails with
 * QLIN_ERR_DEVICE.
 *
 * Threading: host-pointer entry points are serialised on one internal mutex, run on the library's
 * own stream and return after the result is in host memory. Device-resident calls may be made from
 * several threads at once; they are asynchronous on the stream they are given. qlin_timer_begin/end
 * keep their events per calling thread.
 *
 * First call and stream capture: the first call of a device-resident entry point for a given kernel
 * variant raises that kernel's LDS limit (hipFuncSetAttribute), and the routes through the vendor's
 * dense GEMM create its handle and a plan per shape. Neither may happen while a stream is being
 * captured into a graph: run every call shape once before hipStreamBeginCapture.
 */
#ifndef QLINEAR_H
#define QLINEAR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QLIN_OK            0
#define QLIN_ERR_TYPE     (-1) /* unsupported ggml type; same value dequant_row returns */
#define QLIN_ERR_ARG      (-2) /* null pointer, negative size, shape the kernels cannot take */
#define QLIN_ERR_DEVICE   (-3) /* no GPU / HIP failure; text in qlin_last_error() */
#define QLIN_ERR_NOMEM    (-4)

enum qlin_type {
    QLIN_TYPE_F32 = 0, QLIN_TYPE_F16 = 1, QLIN_TYPE_Q8_0 = 8, QLIN_TYPE_Q4_K = 12,
    QLIN_TYPE_Q5_K = 13, QLIN_TYPE_Q6_K = 14, QLIN_TYPE_IQ2_XXS = 16, QLIN_TYPE_IQ4_NL = 20,
    QLIN_TYPE_IQ3_S = 21, QLIN_TYPE_BF16 = 30,
    QLIN_TYPE_Q4_0 = 2, QLIN_TYPE_Q4_1 = 3, QLIN_TYPE_Q5_0 = 6, QLIN_TYPE_Q5_1 = 7,
    QLIN_TYPE_Q2_K = 10, QLIN_TYPE_Q3_K = 11, QLIN_TYPE_IQ2_XS = 17, QLIN_TYPE_IQ3_XXS = 18,
    QLIN_TYPE_IQ1_S = 19, QLIN_TYPE_IQ2_S = 22, QLIN_TYPE_IQ4_XS = 23, QLIN_TYPE_IQ1_M = 29,
    QLIN_TYPE_TQ1_0 = 34, QLIN_TYPE_TQ2_0 = 35, QLIN_TYPE_MXFP4 = 39, QLIN_TYPE_NVFP4 = 40,
    QLIN_TYPE_Q1_0 = 41
};

/* ------------------------------------------------------------------ lifecycle */

/* Select the GPU, create the library stream, upload the codebooks. Idempotent. Called
 * implicitly (device 0) by the first entry point that needs the GPU.
 * Stands where transformer_load sets a model up (common/transformer.h:225). */
int  qlin_init(int device);
void qlin_shutdown(void);
/* Text of the most recent error on this thread's last failing call ("" if none). */
const char *qlin_last_error(void);
/* Device name (truncated to cap-1 chars), compute units, total memory in bytes. */
int  qlin_device_info(char *name, size_t cap, int *compute_units, size_t *mem_bytes);

/* ------------------------------------------------------------------ codec (host pointers)
 * Same signatures and meaning as common/ggml_dequant.h:231-294: n = element count, whole
 * blocks are decoded (n / block_elems of them), a ragged tail is left untouched; src needs
 * 2-byte alignment at most. Decoding runs on the GPU; results are bit-identical to the
 * reference's scalar decoders. */
size_t qlin_dequant_row_size(uint32_t ggml_type, int n);               /* :261-294, 0 if unknown */
int    qlin_dequant_row(uint32_t ggml_type, const void *src, float *dst, int n); /* :258, :3177 */
void   qlin_dequantize_row_q8_0(const void *src, float *dst, int n);    /* :233, :1479 */
void   qlin_dequantize_row_q4_K(const void *src, float *dst, int n);    /* :237, :1592 */
void   qlin_dequantize_row_q5_K(const void *src, float *dst, int n);    /* :238, :1620 */
void   qlin_dequantize_row_q6_K(const void *src, float *dst, int n);    /* :239, :1653 */
void   qlin_dequantize_row_iq2_xxs(const void *src, float *dst, int n); /* :240, :2793 */
void   qlin_dequantize_row_iq3_s(const void *src, float *dst, int n);   /* :248, :3022 */
void   qlin_dequantize_row_iq4_nl(const void *src, float *dst, int n);  /* :249, :2942 */
void   qlin_dequantize_row_q4_0(const void *src, float *dst, int n); /* :241, :2850 */
void   qlin_dequantize_row_q4_1(const void *src, float *dst, int n); /* :242, :2864 */
void   qlin_dequantize_row_q5_0(const void *src, float *dst, int n); /* :243, :2879 */
void   qlin_dequantize_row_q5_1(const void *src, float *dst, int n); /* :244, :2897 */
void   qlin_dequantize_row_q2_K(const void *src, float *dst, int n); /* :231, :1505 */
void   qlin_dequantize_row_q3_K(const void *src, float *dst, int n); /* :232, :1536 */
void   qlin_dequantize_row_q1_0(const void *src, float *dst, int n); /* :234, :1491 */
void   qlin_dequantize_row_mxfp4(const void *src, float *dst, int n); /* :235, :2818 */
void   qlin_dequantize_row_nvfp4(const void *src, float *dst, int n); /* :236, :2832 */
void   qlin_dequantize_row_iq2_xs(const void *src, float *dst, int n); /* :245, :2975 */
void   qlin_dequantize_row_iq2_s(const void *src, float *dst, int n); /* :246, :2996 */
void   qlin_dequantize_row_iq3_xxs(const void *src, float *dst, int n); /* :247, :2916 */
void   qlin_dequantize_row_iq4_xs(const void *src, float *dst, int n); /* :250, :2956 */
void   qlin_dequantize_row_iq1_s(const void *src, float *dst, int n); /* :251, :3062 */
void   qlin_dequantize_row_iq1_m(const void *src, float *dst, int n); /* :252, :3084 */
void   qlin_dequantize_row_tq1_0(const void *src, float *dst, int n); /* :253, :3127 */
void   qlin_dequantize_row_tq2_0(const void *src, float *dst, int n); /* :254, :3161 */
void   qlin_dequantize_row_bf16(const void *src, float *dst, int n); /* :255, :1689 */
/* Many rows at once: src holds n_rows rows of qlin_dequant_row_size(type, n_cols) bytes,
 * dst is [n_rows, n_cols] fp32. Shape of the per-row loop in tf_dequant_row callers
 * (common/transformer.h:425-460). */
int    qlin_dequant_rows(uint32_t ggml_type, const void *src, float *dst, int n_rows, int n_cols);

/* ------------------------------------------------------------------ weights
 * The reference's tensors are borrowed pointers into the GGUF mapping, immutable for the
 * life of the model (tf_load_tensor, common/transformer.h:363-381). Registering such a
 * pointer uploads its bytes to HBM once; later host-pointer calls that name the same pointer
 * (or a pointer inside the registered range, e.g. an expert slice) use the device copy.
 * Calls with an unregistered pointer still work: the bytes are staged for that call only. */
int  qlin_weight_register(const void *host_data, size_t n_bytes);
int  qlin_weight_unregister(const void *host_data);
/* Same registration for a host range whose device copy already exists (n_bytes at dev_copy, from
 * hipMalloc): nothing is copied, the library takes ownership and frees it on unregister. */
int  qlin_weight_adopt(const void *host_data, size_t n_bytes, void *dev_copy);
/* Device address that mirrors host_ptr, or NULL if host_ptr is in no registered range. */
const void *qlin_weight_device_ptr(const void *host_ptr);

/* ------------------------------------------------------------------ linear (host pointers)
 * W: raw ggml blocks, n_rows rows of n_cols elements; x, dst: host fp32. */

/* dst[n_rows] = W . x        tf_qmatvec / tf_qmatvec_pool, common/transformer.h:1049, :1117 */
int qlin_matvec(float *dst, const void *W, uint32_t ggml_type, int n_cols, const float *x, int n_rows);
/* two matrices, one x        tf_qmatvec_fused2_pool, common/transformer.h:897 */
int qlin_matvec_fused2(float *dst1, const void *W1, uint32_t type1, float *dst2, const void *W2,
                       uint32_t type2, int n_cols, const float *x, int n_rows);
/* Q/K/V in one call, each with its own type; K and V share n_kv
 *                            tf_qmatvec_fused_qkv_pool, common/transformer.h:1021 */
int qlin_matvec_qkv(float *q, const void *Wq, uint32_t type_q, int n_q, float *k, const void *Wk,
                    uint32_t type_k, float *v, const void *Wv, uint32_t type_v, int n_kv,
                    int n_cols, const float *x);
/* dst[r] = silu(Wgate[r,:].x) * (Wup[r,:].x), silu(g) = g / (1 + exp(-g)): gate and up projection
 * with the activation applied before anything is written
 *                            tf_qmatvec_fused2_silu_pool, common/transformer.h:953 */
int qlin_matvec_silu_mul(float *dst, const void *Wgate, uint32_t type_gate, const void *Wup,
                         uint32_t type_up, int n_cols, const float *x, int n_rows);
/* dst[r] += W[r,:].x: a projection followed by the residual add
 *                            tf_qmatvec_pool + tf_vadd, common/transformer.h:4037, :551 */
int qlin_matvec_add(float *dst, const void *W, uint32_t ggml_type, int n_cols, const float *x, int n_rows);
/* output projection and greedy pick: *index = first largest of W.x (the loop of
 * server/server_llm.c:224-228 over transformer_compute_logits, common/transformer.h:4302-4307),
 * *value = that logit (may be NULL), logits[n_rows] = all of them (may be NULL: then only 8 bytes
 * come back from the GPU) */
int qlin_matvec_argmax(int *index, float *value, float *logits, const void *W, uint32_t ggml_type,
                       int n_cols, const float *x, int n_rows);
/* one expert of a [n_cols, rows_per_expert, n_expert] tensor: rows start at
 * W + expert * rows_per_expert * row_bytes
 *                            tf_qmatvec_expert(_pool), common/transformer.h:517, :1136 */
int qlin_matvec_expert(float *dst, const void *W, uint32_t ggml_type, int n_cols, int expert,
                       const float *x, int rows_per_expert);
/* prefill: Y[t*out_stride + r] = dot(W[r,:], X[t*x_stride ...]), r < n_rows, t < n_tok; X fp32.
 * Computed in fp32 (no bf16 rounding) so that it can stand in for the CPU path exactly: with 8 tokens or
 * more the weights are decoded to fp32 device scratch (bands of at most 512 MiB) and multiplied by the
 * vendor library's dense fp32 GEMM on the matrix cores; fewer tokens run a vector-ALU kernel.
 *                            tf_gemm_f16_mt_tokenmajor, common/transformer.h:4487
 * qlin_set_prefill_matrix_cores(1), or QLIN_PREFILL_MATRIX_CORES=1 in the environment when the library
 * initialises, sends calls with 8 tokens or more through the bf16 matrix-core route instead (activations
 * and decoded weights rounded to bf16: relative L2 <= 3e-3 instead of 1e-6; 5x less kernel time again). */
int qlin_set_prefill_matrix_cores(int enable);
int qlin_gemm_tokenmajor(float *Y, const void *W, uint32_t ggml_type, int n_cols, const float *X,
                         int n_rows, int n_tok, int out_stride, int x_stride);
/* one token of the MoE FFN block (common/transformer.h:4045-4131) without the router matvec:
 * logits[n_expert] -> softmax -> top_k -> renormalise -> sum_k w_k down_k(silu(gate_k x)*up_k x).
 * out[n_embd] is overwritten (the caller adds it to the residual, :4130). */
int qlin_moe_ffn_token(float *out, const void *gate_exps, const void *up_exps, const void *down_exps,
                       uint32_t ggml_type, int n_embd, int n_ff_expert, int n_expert, int top_k,
                       const float *router_logits, const float *x);
/* the same with one format per tensor (the down projections of K-quant mixes are partly Q6_K) */
int qlin_moe_ffn_token_types(float *out, const void *gate_exps, const void *up_exps, const void *down_exps,
                             uint32_t type_gate, uint32_t type_up, uint32_t type_down, int n_embd, int n_ff,
                             int n_expert, int top_k, const float *router_logits, const float *x);

/* ------------------------------------------------------------------ device-resident
 * All pointers are device addresses; `stream` is a hipStream_t passed as void* (NULL = the
 * null stream). Calls only enqueue work. No counterpart in the reference's CPU API; the
 * arithmetic is the same as the group above. */
void *qlin_dev_alloc(size_t n_bytes);
void  qlin_dev_free(void *p);
int   qlin_dev_upload(void *dst_dev, const void *src_host, size_t n_bytes);
int   qlin_dev_download(void *dst_host, const void *src_dev, size_t n_bytes);
int   qlin_dev_sync(void *stream);

/* out[n_rows, n_cols] fp32 = decode(W); whole blocks only */
int qlin_dequant_dev(uint32_t ggml_type, const void *W, float *out, int n_rows, int n_cols, void *stream);
/* out[n_rows, n_cols] bf16 (bit patterns) = decode(W) rounded to nearest even: the weight operand of
 * qlin_gemm_bf16_any_dev. An engine with HBM to spare decodes the tensors its prefill uses most once and
 * passes the copy as GGML_TYPE_BF16 (the decode is 35-45 us of a 90 us call at 14336 x 4096 x 512 tokens).
 * W and out 16-byte aligned, n_cols a whole number of blocks (dense types: a multiple of 8). */
int qlin_dequant_bf16_dev(uint32_t ggml_type, const void *W, uint16_t *out, int n_rows, int n_cols, void *stream);
/* out[i, :] = decode(table row row_ids[i]) for i < n_ids: the token-embedding lookup
 * (tf_dequant_row on token_embd, common/transformer.h:3509) for a list of device-resident ids.
 * An id outside [0, n_table_rows) gives a row of zeros (the reference refuses such a token, :3501). */
int qlin_embed_rows_dev(uint32_t ggml_type, const void *table, int n_table_rows, const int32_t *row_ids,
                        int n_ids, float *out, int n_cols, void *stream);
/* y[n_rows] = W . x, x fp32 (16-byte aligned), W 2-byte aligned (F32: 4-byte). Besides the block formats W may be
 * dense F16, BF16 or F32 rows of any length: the fp32 dot of the widened row with x, as tf_qmatvec does for these
 * types (common/transformer.h:1051-1075); dense rows whose length is not a multiple of 8, or that do not start on
 * 16-byte addresses, take a one-element-per-lane kernel. Rows of any length in whole blocks: rows
 * of more than 16384 elements run as several launches over column ranges, the later ones adding to y (still one
 * call, ordered on `stream`). */
int qlin_gemv_dev(uint32_t ggml_type, const void *W, const float *x, float *y, int n_rows,
                  int n_cols, void *stream);
/* The fused call shapes of the decode loop, one launch each (all matrices of one ggml type):
 *   add       y[r] += W[r,:].x                                   (projection + residual)
 *   silu_mul  out[r] = silu(Wgate[r,:].x) * (Wup[r,:].x)         (common/transformer.h:953)
 *   multi     y_m = W_m . x for m < n_mat <= 3 matrices sharing x (gate+up :897, Q/K/V :1021)
 *   argmax    logits = W.x (written, n_rows floats), then result = {int32 index of the first
 *             largest logit, float value} in the first 8 bytes of `result`, which must hold
 *             QLIN_ARGMAX_RESULT_BYTES bytes, 8-byte aligned (the rest is scratch for the pick) */
#define QLIN_ARGMAX_RESULT_BYTES 2056
int qlin_gemv_add_dev(uint32_t ggml_type, const void *W, const float *x, float *y, int n_rows,
                      int n_cols, void *stream);
int qlin_gemv_silu_mul_dev(uint32_t ggml_type, const void *Wgate, const void *Wup, const float *x,
                           float *out, int n_rows, int n_cols, void *stream);
int qlin_gemv_multi_dev(uint32_t ggml_type, int n_mat, const void *const *W, float *const *y,
                        const int *n_rows, const float *x, int n_cols, void *stream);
int qlin_gemv_argmax_dev(uint32_t ggml_type, const void *W, const float *x, float *logits,
                         void *result, int n_rows, int n_cols, void *stream);
/* Y[t*ldy + r] = dot(W[r,:], X[t*ldx ...]); X bf16 (uint16 bit patterns), fp32 accumulate on
 * the matrix cores, Y fp32 token-major. Q4_K only; n_cols % 256 == 0. From 33 tokens on the
 * decoded weights are rounded to bf16 once (relative L2 of Y <= 2e-3 against exact weights); up to
 * 32 tokens the 4-bit codes go through the matrix instruction unrounded and the block scales are
 * applied in fp32 (~1e-6). */
int qlin_gemm_bf16_dev(uint32_t ggml_type, const void *W, const uint16_t *X, float *Y, int n_rows,
                       int n_cols, int n_tok, int ldx, int ldy, void *stream);
/* The same contraction for EVERY weight format (block-quantized and dense F16/BF16/F32), the role of
 * tf_gemm_f16_mt_tokenmajor for the formats it re-decodes once per token (common/transformer.h:4535-4572):
 * W is decoded once to bf16 (nearest even) into `workspace` and multiplied by the dense matrix-core GEMM of
 * the vendor library. Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, Q8_0, IQ4_NL, IQ4_XS and Q4_0 tensors (n_cols % 256 == 0) are instead
 * decoded inside the product by this library's tile kernels, with the same single rounding to bf16, and leave the workspace alone (it may be NULL
 * for them): 256-token x 128-row tiles where 200 or more of them fill the chip (12800 rows at 257..512 tokens, 6400 at
 * 513..1024, ...), 128-token x 64-row tiles for smaller shapes (4096-row projections at 512 tokens, any row count at
 * 33..256 tokens). Given a workspace, the decode + dense route still takes the shapes where decoding once measured
 * faster: large-tile shapes above 1536 tokens (Q4_K, Q5_K, IQ4_NL), 1024 (Q2_K, Q3_K, IQ4_XS, Q4_0) or 512 (Q6_K, Q8_0), small-tile
 * shapes of Q8_0 above 256 tokens, of Q6_K above 512, of IQ4_NL and IQ4_XS above 1024. Q4_K up to 32 tokens: the few-token kernel of qlin_gemm_bf16_dev.
 * Up to 24 tokens of a Q6_K, Q5_K, Q3_K, Q2_K or
 * Q8_0 tensor (n_cols % 256 == 0, the tensor's bytes a multiple of 16) also run in one fused kernel with
 * unrounded weights (~1e-6) and leave the workspace alone (it may be NULL then). Up to 4 tokens of any other
 * block format go one by one through the matvec kernels (exact weights, ~1e-6; the workspace holds their
 * activations as fp32, and when ldx is so wide that (n_tok - 1) * ldx + n_cols floats do not fit it they take the
 * decode + dense route). workspace: device memory, 256-byte aligned, at least
 * qlin_gemm_bf16_any_workspace_bytes(n_rows, n_cols) bytes (2 bytes per weight + 32 MiB for the library);
 * calls that share a workspace must be ordered on one stream. Relative L2 of Y against exact weights
 * <= 2e-3.
 * qlin_set_dense_gemm_own(1), or QLIN_DENSE_GEMM=own in the environment when the library initialises,
 * replaces the vendor library's dense GEMM by this library's own bf16 tile kernel (rows of a multiple of
 * 256 elements; about 0.8x the vendor kernel's speed at 512 tokens, 0.6x at 2048); the own kernel also
 * takes over whenever the vendor library offers no kernel for a shape, and where neither takes it the
 * vector-ALU kernel of qlin_gemm_f32_dev does (exact weights, activations widened to fp32 a band of tokens at a
 * time in the workspace) - qlin_set_dense_gemm_own(2) sends every dense product there (a test switch: slow). */
int qlin_set_dense_gemm_own(int enable);
size_t qlin_gemm_bf16_any_workspace_bytes(int n_rows, int n_cols);
int qlin_gemm_bf16_any_dev(uint32_t ggml_type, const void *W, const uint16_t *X, float *Y, int n_rows,
                           int n_cols, int n_tok, int ldx, int ldy, void *workspace, size_t workspace_bytes,
                           void *stream);
/* qlin_gemm_bf16_any_dev for one to three weight tensors of ONE format and row length against the same activations:
 * the Q, K and V projections of a prefill chunk, which the reference multiplies tensor by tensor
 * (tf_gemm_f16_mt_tokenmajor per projection, common/transformer.h:5256-5258). Y[i][t * ldy[i] + r] is tensor i's
 * product. Where every tensor on its own would take the same tile kernel (more than 32 tokens of a format with one)
 * they share one launch, their row tiles numbered through, with the results of one call per tensor bit for bit: a
 * 1024-row K or V projection alone is 64 workgroups of 128 tokens x 64 rows at 512 tokens on 256 compute units (Q4_K
 * 4096 + 1024 + 1024 rows x 4096 at 512 tokens: 36 us in one launch against 24 + 22 + 22). Every other case is one
 * qlin_gemm_bf16_any_dev call per tensor, with its argument checks and its use of the workspace (sized for the
 * largest tensor). The arrays W, Y, n_rows and ldy are host memory and are read before the call returns. */
int qlin_gemm_bf16_multi_dev(uint32_t ggml_type, int n_mat, const void *const *W, const uint16_t *X, float *const *Y,
                             const int *n_rows, int n_cols, int n_tok, int ldx, const int *ldy, void *workspace,
                             size_t workspace_bytes, void *stream);
/* Same contraction in fp32 (X fp32, no rounding of weights or activations); any supported type.
 * Vector-ALU kernel, no workspace: the choice for a few tokens. */
int qlin_gemm_f32_dev(uint32_t ggml_type, const void *W, const float *X, float *Y, int n_rows,
                      int n_cols, int n_tok, int ldx, int ldy, void *stream);
/* The fp32 contraction for many tokens, any supported type: W is decoded once to fp32 (bit-exact, as
 * qlin_dequant_dev) into `workspace` and multiplied by the vendor library's dense fp32 GEMM (fp32 operands,
 * fp32 accumulation on the matrix cores) -- what tf_gemm_f16_mt_tokenmajor (common/transformer.h:4487)
 * computes for fp32 activations, without the 16-bit rounding of its fast paths. Relative L2 against a
 * double-precision reference <= 1e-5. Fewer than 8 tokens run the kernel of qlin_gemm_f32_dev and leave the
 * workspace alone (it may then be NULL). workspace: device memory, 256-byte aligned, at least
 * qlin_gemm_f32_any_workspace_bytes(n_rows, n_cols) bytes (4 bytes per weight + 32 MiB for the library);
 * calls that share a workspace must be ordered on one stream. */
size_t qlin_gemm_f32_any_workspace_bytes(int n_rows, int n_cols);
int qlin_gemm_f32_any_dev(uint32_t ggml_type, const void *W, const float *X, float *Y, int n_rows,
                          int n_cols, int n_tok, int ldx, int ldy, void *workspace, size_t workspace_bytes,
                          void *stream);
/* Grouped MoE expert FFN over n_tok tokens (the block of common/transformer.h:4045-4131 after the router):
 *   X bf16 [n_tok, n_embd]; expert_idx int32 [n_tok, top_k]; expert_w fp32 [n_tok, top_k];
 *   gate/up: [n_expert][n_ff][n_embd] blocks, down: [n_expert][n_embd][n_ff] blocks;
 *   out fp32 [n_tok, n_embd] (overwritten). workspace: qlin_moe_workspace_bytes() bytes.
 * Q4_K, Q5_K, Q6_K, Q3_K, Q2_K and Q8_0 matrices run on the matrix cores with unrounded codes; every other format
 * (block-quantized or dense) runs through the bit-exact decoder in fp32, several times slower. qlin_moe_ffn_types_dev takes one format
 * per tensor: K-quant mixes store part of the down projections as Q6_K beside Q4_K gate and up.
 * One token - the reference's own call - and up to eight tokens when there are at most two (token, choice) pairs per
 * four experts go token by token through two launches of the matvec kernels instead, for every block format (gate and
 * up of one format): no rounding of activations or weights, the sum over a token's experts in a fixed order. */
size_t qlin_moe_workspace_bytes(int n_tok, int top_k, int n_embd, int n_ff, int n_expert);
int qlin_moe_route_dev(const float *router_logits, int n_tok, int n_expert, int top_k,
                       int32_t *expert_idx, float *expert_w, void *stream);
int qlin_moe_ffn_dev(uint32_t ggml_type, const void *gate_exps, const void *up_exps,
                     const void *down_exps, const uint16_t *X, const int32_t *expert_idx,
                     const float *expert_w, float *out, int n_tok, int top_k, int n_embd,
                     int n_ff, int n_expert, void *workspace, void *stream);
int qlin_moe_ffn_types_dev(uint32_t type_gate, uint32_t type_up, uint32_t type_down, const void *gate_exps,
                           const void *up_exps, const void *down_exps, const uint16_t *X,
                           const int32_t *expert_idx, const float *expert_w, float *out, int n_tok, int top_k,
                           int n_embd, int n_ff, int n_expert, void *workspace, void *stream);
/* qlin_moe_ffn_types_dev without the workspace argument and without any allocation: the scratch its kernels
 * need (slot tables, the intermediate activations by slot, the per-slot down projections) lives in a device
 * array inside the library, QLIN_MOE_STATIC_SCRATCH_BYTES per GPU, held until the process ends. No counterpart
 * in the reference; it is for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc. Same arguments, results and error codes as qlin_moe_ffn_types_dev, plus:
 *   - QLIN_ERR_ARG if qlin_moe_workspace_bytes(n_tok, top_k, n_embd, n_ff, n_expert) exceeds
 *     QLIN_MOE_STATIC_SCRATCH_BYTES (64 tokens x top-8 x 2048/768 x 128 experts needs 8.7 MB);
 *   - QLIN_ERR_DEVICE if qlin_init() has not run (initialising creates a stream and events, which this call
 *     must not do); the scratch address of the device is looked up there, once.
 * The call enqueues kernels on `stream` and returns. Every call on a GPU shares that GPU's scratch and leaves
 * its contents behind: calls whose kernels could overlap (different streams, different host threads) race -
 * order them on one stream. */
#define QLIN_MOE_STATIC_SCRATCH_BYTES (16u << 20)
int qlin_moe_ffn_static_dev(uint32_t type_gate, uint32_t type_up, uint32_t type_down, const void *gate_exps,
                            const void *up_exps, const void *down_exps, const uint16_t *X,
                            const int32_t *expert_idx, const float *expert_w, float *out, int n_tok, int top_k,
                            int n_embd, int n_ff, int n_expert, void *stream);

/* ------------------------------------------------------------------ GGUF file -> HBM
 * The tensor table and key/value pairs of a GGUF model file (versions 2 and 3, as read by
 * gguf_open, common/gguf_loader.h:343-411) and its tensor bytes in device memory.
 * qlin_gguf_open parses the header (no GPU needed, no tensor data read); qlin_gguf_upload streams
 * the data section into ONE device allocation through pinned staging buffers and registers the
 * host range of the (lazily) mapped file, so that qlin_gguf_tensor_host(i) pointers work with the
 * host-pointer entry points above without further copies (the place of tf_load_tensor's
 * `gguf_tensor_data` pointers, common/transformer.h:363-381) and qlin_gguf_tensor_dev(i) with the
 * device-resident ones. Tensor sizes follow gguf_tensor_size (:520-532). */
typedef struct qlin_gguf qlin_gguf;
int  qlin_gguf_open(const char *path, qlin_gguf **out);
void qlin_gguf_close(qlin_gguf *g);       /* also releases the device copy */
uint32_t qlin_gguf_version(const qlin_gguf *g);
uint32_t qlin_gguf_alignment(const qlin_gguf *g);
size_t qlin_gguf_data_offset(const qlin_gguf *g);   /* file offset of the data section */
size_t qlin_gguf_data_size(const qlin_gguf *g);     /* end of the last tensor */
int  qlin_gguf_n_tensors(const qlin_gguf *g);
int  qlin_gguf_find_tensor(const qlin_gguf *g, const char *name); /* index or -1 (tf_find_tensor, :355) */
int  qlin_gguf_tensor_info(const qlin_gguf *g, int i, const char **name, uint32_t *ggml_type, int *n_dims,
                           uint64_t dims[4], uint64_t *offset, size_t *n_bytes);
const void *qlin_gguf_tensor_host(const qlin_gguf *g, int i);  /* address in the mapped file */
const void *qlin_gguf_tensor_dev(const qlin_gguf *g, int i);   /* NULL before qlin_gguf_upload */
int  qlin_gguf_upload(qlin_gguf *g);
/* key/value pairs: index of a key or -1; value type = enum gguf_value_type (:26-41) */
int  qlin_gguf_n_kv(const qlin_gguf *g);
int  qlin_gguf_find_key(const qlin_gguf *g, const char *key);
const char *qlin_gguf_key(const qlin_gguf *g, int i);
int  qlin_gguf_value_type(const qlin_gguf *g, int i);
int  qlin_gguf_get_i64(const qlin_gguf *g, int i, int64_t *out);   /* any integer width, bool */
int  qlin_gguf_get_f64(const qlin_gguf *g, int i, double *out);    /* any number */
const char *qlin_gguf_get_str(const qlin_gguf *g, int i);           /* NULL unless a string */
/* arrays: element type, count and the address of the first element in the mapped file (strings:
 * u64 length + bytes each, not terminated) */
int  qlin_gguf_get_array(const qlin_gguf *g, int i, uint32_t *elem_type, uint64_t *n, const void **first);

/* Elapsed milliseconds of work enqueued on `stream` between the two calls, by HIP events
 * recorded on that stream (the role of elapsed_kernel_ms in rdna4/dequant/bench_dequant.c:764-780). */
int qlin_timer_begin(void *stream);
int qlin_timer_end(void *stream, float *ms);

#ifdef __cplusplus
}
#endif
#endif /* QLINEAR_H */
