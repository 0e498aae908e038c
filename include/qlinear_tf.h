/*
 * qlinear_tf.h - the reference's quantized-linear call shapes on top of the C ABI of qlinear.h.
 *
 * The reference keeps this path as `static` functions of a header-only library
 * (common/transformer.h). The functions below take the same arguments and behave the same on
 * failure (a message on stderr and a zero-filled output; they return void). The single-thread
 * forms keep the reference's argument order; the `_pool` forms take the activation first instead of
 * the model pointer, and the QLINEAR_TF_REFERENCE_NAMES macros at the end of this header restore
 * the reference's names AND argument order for all of them, so a C engine written against
 * transformer.h compiles against this header unchanged:
 *
 *   qtensor                      common/transformer.h:34-43 (same fields, same order)
 *   qtf_row_bytes                tf_row_bytes                  :489-514
 *   qtf_is_supported_weight_type tf_is_supported_weight_type   :462-487
 *   qtf_dequant_row              tf_dequant_row                :425-460
 *   qtf_qmatvec                  tf_qmatvec                    :1049-1114
 *   qtf_qmatvec_pool             tf_qmatvec_pool               :1117-1133
 *   qtf_qmatvec_fused2_pool      tf_qmatvec_fused2_pool        :897-914
 *   qtf_qmatvec_fused2_silu_pool tf_qmatvec_fused2_silu_pool   :953-970
 *   qtf_qmatvec_fused_qkv_pool   tf_qmatvec_fused_qkv_pool     :1021-1047
 *   qtf_qmatvec_add              tf_qmatvec_pool + tf_vadd     :4037, :551 (projection + residual)
 *   qtf_logits_argmax            transformer_compute_logits + the greedy loop of
 *                                server/server_llm.c:224-228   :4302-4307
 *   qtf_qmatvec_expert           tf_qmatvec_expert             :517-548
 *   qtf_qmatvec_expert_pool      tf_qmatvec_expert_pool        :1136-1158
 *   qtf_gemm_tokenmajor          tf_gemm_f16_mt_tokenmajor     :4487-4595
 *   qtf_moe_ffn                  the MoE FFN block             :4045-4131
 *   qtf_load_tensor              tf_load_tensor                :363-381
 *   qtf_get_int / qtf_get_float  tf_get_int / tf_get_float     :383-396
 *   qtf_register_tensor          (upload once; the reference maps the file and never copies)
 *
 * Differences, all on the caller's side of the boundary:
 *   - the `transformer_model *m` of the pool variants is replaced by the activation pointer the
 *     reference reads from it (m->xb); thread counts and scratch rows (`tmp`) are accepted and
 *     ignored: the GPU needs neither.
 *   - supported weight types are the sixteen block formats plus F32/F16/BF16 that the reference's model
 *     path accepts (tf_is_supported_weight_type, :462-487); any other type reports "unsupported"
 *     exactly as an unknown type does in the reference.
 * Define QLINEAR_TF_REFERENCE_NAMES before including this header to also get the reference's own
 * names (tf_qmatvec, ...) as macros.
 */
#ifndef QLINEAR_TF_H
#define QLINEAR_TF_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    void    *data;       /* raw ggml blocks, rows contiguous */
    uint32_t type;       /* enum ggml_dtype value */
    int      n_rows;
    int      n_cols;     /* elements per row */
    int      n_dims;
    uint64_t dims[4];
    float    scale;      /* carried, never applied (the reference's CPU path does not read it either) */
    int      has_scale;
} qtensor;

/* an open model file (include/qlinear.h: qlin_gguf_open / qlin_gguf_upload) */
struct qlin_gguf;
/* the qtensor of a named tensor: data = its address in the mapped file (registered with the GPU copy
 * once qlin_gguf_upload has run), n_cols = dims[0], n_rows = product of the other dims; data == NULL
 * if the tensor is missing (with a message on stderr when `required`)
 *                                tf_load_tensor, common/transformer.h:363-381 */
qtensor qtf_load_tensor(const struct qlin_gguf *gguf, const char *name, int required);
/* u32/i32 and f32 values with a default   tf_get_int, tf_get_float, common/transformer.h:383-396 */
int    qtf_get_int(const struct qlin_gguf *gguf, const char *key, int default_val);
float  qtf_get_float(const struct qlin_gguf *gguf, const char *key, float default_val);

size_t qtf_row_bytes(uint32_t type, int n_cols);
int    qtf_is_supported_weight_type(uint32_t type);
/* Uploads the tensor's bytes to the GPU once; later calls that pass this tensor (or an expert
 * slice of it) use the device copy. 0 on success. Unregistered tensors still work, slowly. */
int    qtf_register_tensor(const qtensor *t);
int    qtf_unregister_tensor(const qtensor *t);

void qtf_dequant_row(const qtensor *t, int row, float *dst);
void qtf_qmatvec(float *dst, const qtensor *mat, const float *x, int n_rows, float *tmp);
void qtf_qmatvec_pool(const float *x, float *dst, const qtensor *mat, int n_rows);
void qtf_qmatvec_fused2_pool(const float *x, float *dst1, const qtensor *mat1, float *dst2,
                             const qtensor *mat2, int n_rows);
/* dst = silu(gate_mat . x) * (up_mat . x) */
void qtf_qmatvec_fused2_silu_pool(const float *x, float *dst, const qtensor *gate_mat, const qtensor *up_mat,
                                  int n_rows);
/* dst += mat . x */
void qtf_qmatvec_add(const float *x, float *dst, const qtensor *mat, int n_rows);
/* index of the first largest of output . x (-1 on failure); logits may be NULL */
int  qtf_logits_argmax(const float *x, const qtensor *output, int n_vocab, float *logits);
void qtf_qmatvec_fused_qkv_pool(const float *x, float *q, const qtensor *mat_q, int n_q, float *k,
                                const qtensor *mat_k, float *v, const qtensor *mat_v, int n_kv);
void qtf_qmatvec_expert(float *dst, const qtensor *mat, int expert, const float *x,
                        int rows_per_expert, float *tmp);
void qtf_qmatvec_expert_pool(const float *x, float *dst, const qtensor *mat, int expert,
                             int rows_per_expert);
void qtf_gemm_tokenmajor(float *Y_out, const qtensor *mat, const float *X, int n_rows, int N,
                         int out_stride, int X_stride, int n_threads);
/* out[n_embd] = sum over the top_k routed experts of w_e * down_e(silu(gate_e x) * up_e x);
 * router_logits[n_expert] are the router matvec's outputs (:4048-4052). */
void qtf_moe_ffn(float *out, const qtensor *gate_exps, const qtensor *up_exps,
                 const qtensor *down_exps, int n_expert, int top_k, int n_ff_expert,
                 const float *router_logits, const float *x);

#ifdef QLINEAR_TF_REFERENCE_NAMES
#define tf_row_bytes                 qtf_row_bytes
#define tf_is_supported_weight_type  qtf_is_supported_weight_type
#define tf_qmatvec_fused2_silu_pool(m, dst, gate_mat, up_mat, x, n_rows) qtf_qmatvec_fused2_silu_pool(x, dst, gate_mat, up_mat, n_rows)
#define tf_dequant_row               qtf_dequant_row
#define tf_qmatvec                   qtf_qmatvec
#define tf_qmatvec_expert            qtf_qmatvec_expert
#define tf_gemm_f16_mt_tokenmajor    qtf_gemm_tokenmajor
/* the pool variants, in the reference's argument order (common/transformer.h:1117, :897, :1021, :1136): the
 * model pointer is dropped, except that the fused Q/K/V call reads its activation from it (m->xb, as the
 * reference does, :1027-1029), so `m` must point to a struct with a `const float *xb` member there */
#define tf_qmatvec_pool(m, dst, mat, x, n_rows) qtf_qmatvec_pool(x, dst, mat, n_rows)
#define tf_qmatvec_fused2_pool(m, dst1, mat1, dst2, mat2, x, n_rows) qtf_qmatvec_fused2_pool(x, dst1, mat1, dst2, mat2, n_rows)
#define tf_qmatvec_fused_qkv_pool(m, q, mat_q, n_q, k, mat_k, v, mat_v, n_kv) \
    qtf_qmatvec_fused_qkv_pool((m)->xb, q, mat_q, n_q, k, mat_k, v, mat_v, n_kv)
#define tf_qmatvec_expert_pool(m, dst, mat, expert, x, rows_per_expert) qtf_qmatvec_expert_pool(x, dst, mat, expert, rows_per_expert)
#endif

#ifdef __cplusplus
}
#endif
#endif /* QLINEAR_TF_H */
