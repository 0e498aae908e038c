/*
 * qlinear_tf.c - the reference's call shapes (common/transformer.h) over the C ABI of
 * libqlinear. Plain C, no GPU code: every function forwards to one qlin_* entry point and
 * turns a failure into what the reference does at the same place: a line on stderr and a
 * zero-filled destination (common/transformer.h:451-454, :520-523).
 */
#include "qlinear_tf.h"

#include <stdio.h>
#include <string.h>

#include "qlinear.h"

static void zero_fill(float *dst, size_t n) {
    if (dst && n) memset(dst, 0, n * sizeof(float));
}

static void complain(const char *where) {
    fprintf(stderr, "qlinear: %s failed: %s\n", where, qlin_last_error());
}

/* the weight types the reference's model path takes (common/transformer.h:462-487): sixteen
 * block formats and the three plain ones; the decoders know more formats than this */
int qtf_is_supported_weight_type(uint32_t type) {
    switch (type) {
    case QLIN_TYPE_Q2_K: case QLIN_TYPE_Q3_K: case QLIN_TYPE_Q4_0: case QLIN_TYPE_Q8_0:
    case QLIN_TYPE_Q4_K: case QLIN_TYPE_Q5_K: case QLIN_TYPE_Q6_K: case QLIN_TYPE_IQ2_XXS:
    case QLIN_TYPE_IQ2_XS: case QLIN_TYPE_IQ3_XXS: case QLIN_TYPE_IQ1_S: case QLIN_TYPE_IQ4_NL:
    case QLIN_TYPE_IQ3_S: case QLIN_TYPE_IQ2_S: case QLIN_TYPE_IQ4_XS: case QLIN_TYPE_IQ1_M:
    case QLIN_TYPE_F32: case QLIN_TYPE_F16: case QLIN_TYPE_BF16:
        return 1;
    default:
        return 0;
    }
}

/* 0 for a type outside that list, like the reference (common/transformer.h:489-514) */
size_t qtf_row_bytes(uint32_t type, int n_cols) {
    return qtf_is_supported_weight_type(type) ? qlin_dequant_row_size(type, n_cols) : 0;
}

qtensor qtf_load_tensor(const struct qlin_gguf *gguf, const char *name, int required) {
    qtensor t;
    memset(&t, 0, sizeof(t));
    const int idx = qlin_gguf_find_tensor(gguf, name);
    if (idx < 0) {
        if (required) fprintf(stderr, "qlinear: missing tensor '%s'\n", name);
        return t;
    }
    uint32_t type = 0;
    int n_dims = 0;
    uint64_t dims[4] = {0, 0, 0, 0};
    if (qlin_gguf_tensor_info(gguf, idx, NULL, &type, &n_dims, dims, NULL, NULL) != QLIN_OK) return t;
    t.data = (void *)qlin_gguf_tensor_host(gguf, idx);
    t.type = type;
    t.n_dims = n_dims;
    uint64_t n_rows = 1;
    for (int d = 0; d < n_dims; d++) {
        t.dims[d] = dims[d];
        if (d > 0) n_rows *= dims[d];
    }
    t.n_cols = (int)dims[0];
    t.n_rows = (int)n_rows;
    return t;
}

int qtf_get_int(const struct qlin_gguf *gguf, const char *key, int default_val) {
    const int i = qlin_gguf_find_key(gguf, key);
    const int type = i < 0 ? -1 : qlin_gguf_value_type(gguf, i);
    int64_t v;
    if ((type != 4 && type != 5) || qlin_gguf_get_i64(gguf, i, &v) != QLIN_OK) return default_val; /* u32, i32 only */
    return (int)v;
}

float qtf_get_float(const struct qlin_gguf *gguf, const char *key, float default_val) {
    const int i = qlin_gguf_find_key(gguf, key);
    double v;
    if (i < 0 || qlin_gguf_value_type(gguf, i) != 6 || qlin_gguf_get_f64(gguf, i, &v) != QLIN_OK) return default_val;
    return (float)v;
}

static size_t tensor_bytes(const qtensor *t) {
    return (size_t)t->n_rows * qtf_row_bytes(t->type, t->n_cols);
}

int qtf_register_tensor(const qtensor *t) {
    if (!t || !t->data || !qtf_is_supported_weight_type(t->type)) return -1;
    return qlin_weight_register(t->data, tensor_bytes(t));
}

int qtf_unregister_tensor(const qtensor *t) { return t ? qlin_weight_unregister(t->data) : -1; }

void qtf_dequant_row(const qtensor *t, int row, float *dst) {
    const size_t rb = qtf_row_bytes(t->type, t->n_cols);
    if (rb == 0 || qlin_dequant_row(t->type, (const uint8_t *)t->data + (size_t)row * rb, dst, t->n_cols) != 0) {
        complain("dequant_row");
        zero_fill(dst, (size_t)t->n_cols);
    }
}

void qtf_qmatvec(float *dst, const qtensor *mat, const float *x, int n_rows, float *tmp) {
    (void)tmp;
    if (qlin_matvec(dst, mat->data, mat->type, mat->n_cols, x, n_rows) != QLIN_OK) {
        complain("qmatvec");
        zero_fill(dst, (size_t)n_rows);
    }
}

void qtf_qmatvec_pool(const float *x, float *dst, const qtensor *mat, int n_rows) {
    qtf_qmatvec(dst, mat, x, n_rows, NULL);
}

void qtf_qmatvec_fused2_pool(const float *x, float *dst1, const qtensor *mat1, float *dst2, const qtensor *mat2,
                             int n_rows) {
    if (qlin_matvec_fused2(dst1, mat1->data, mat1->type, dst2, mat2->data, mat2->type, mat1->n_cols, x, n_rows) !=
        QLIN_OK) {
        complain("qmatvec_fused2");
        zero_fill(dst1, (size_t)n_rows);
        zero_fill(dst2, (size_t)n_rows);
    }
}

void qtf_qmatvec_fused2_silu_pool(const float *x, float *dst, const qtensor *gate_mat, const qtensor *up_mat,
                                  int n_rows) {
    if (qlin_matvec_silu_mul(dst, gate_mat->data, gate_mat->type, up_mat->data, up_mat->type, gate_mat->n_cols, x,
                             n_rows) != QLIN_OK) {
        complain("qmatvec_fused2_silu");
        zero_fill(dst, (size_t)n_rows);
    }
}

void qtf_qmatvec_add(const float *x, float *dst, const qtensor *mat, int n_rows) {
    /* on failure the residual stream is left as it was */
    if (qlin_matvec_add(dst, mat->data, mat->type, mat->n_cols, x, n_rows) != QLIN_OK) complain("qmatvec_add");
}

int qtf_logits_argmax(const float *x, const qtensor *output, int n_vocab, float *logits) {
    int index = -1;
    if (qlin_matvec_argmax(&index, NULL, logits, output->data, output->type, output->n_cols, x, n_vocab) != QLIN_OK) {
        complain("logits_argmax");
        return -1;
    }
    return index;
}

void qtf_qmatvec_fused_qkv_pool(const float *x, float *q, const qtensor *mat_q, int n_q, float *k,
                                const qtensor *mat_k, float *v, const qtensor *mat_v, int n_kv) {
    if (qlin_matvec_qkv(q, mat_q->data, mat_q->type, n_q, k, mat_k->data, mat_k->type, v, mat_v->data, mat_v->type,
                        n_kv, mat_q->n_cols, x) != QLIN_OK) {
        complain("qmatvec_fused_qkv");
        zero_fill(q, (size_t)n_q);
        zero_fill(k, (size_t)n_kv);
        zero_fill(v, (size_t)n_kv);
    }
}

void qtf_qmatvec_expert(float *dst, const qtensor *mat, int expert, const float *x, int rows_per_expert,
                        float *tmp) {
    (void)tmp;
    if (qlin_matvec_expert(dst, mat->data, mat->type, mat->n_cols, expert, x, rows_per_expert) != QLIN_OK) {
        complain("qmatvec_expert");
        zero_fill(dst, (size_t)rows_per_expert);
    }
}

void qtf_qmatvec_expert_pool(const float *x, float *dst, const qtensor *mat, int expert, int rows_per_expert) {
    qtf_qmatvec_expert(dst, mat, expert, x, rows_per_expert, NULL);
}

void qtf_gemm_tokenmajor(float *Y_out, const qtensor *mat, const float *X, int n_rows, int N, int out_stride,
                         int X_stride, int n_threads) {
    (void)n_threads;
    if (qlin_gemm_tokenmajor(Y_out, mat->data, mat->type, mat->n_cols, X, n_rows, N, out_stride, X_stride) !=
        QLIN_OK) {
        complain("gemm_tokenmajor");
        for (int t = 0; t < N; t++) zero_fill(Y_out + (size_t)t * out_stride, (size_t)n_rows);
    }
}

void qtf_moe_ffn(float *out, const qtensor *gate_exps, const qtensor *up_exps, const qtensor *down_exps,
                 int n_expert, int top_k, int n_ff_expert, const float *router_logits, const float *x) {
    const int n_embd = gate_exps->n_cols;
    if (qlin_moe_ffn_token_types(out, gate_exps->data, up_exps->data, down_exps->data, gate_exps->type, up_exps->type,
                                 down_exps->type, n_embd, n_ff_expert, n_expert, top_k, router_logits, x) != QLIN_OK) {
        complain("moe_ffn");
        zero_fill(out, (size_t)n_embd);
    }
}
