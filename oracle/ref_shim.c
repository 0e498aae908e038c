/*
 * ref_shim.c - exports a few of the reference's own static functions as a shared library.
 *
 * TEST INFRASTRUCTURE ONLY. This translation unit includes the reference's header-only C
 * sources where they lie (the include path points at the read-only reference checkout); no
 * reference source is copied into this repository. The library it builds (oracle/_ref/) is
 * used to (1) write the golden fixtures under tests/golden/, (2) cross-check the oracle, and
 * (3) serve as the "reference" CPU baseline timed by the benchmark. It is never linked into or
 * loaded by the shipped library.
 */
#include <string.h>
#include <stdlib.h>
#include <time.h>

#define GGUF_LOADER_IMPLEMENTATION
#include "common/gguf_loader.h"
#define GGML_DEQUANT_IMPLEMENTATION
#include "common/ggml_dequant.h"
#define BPE_TOKENIZER_IMPLEMENTATION
#include "common/bpe_tokenizer.h"
#define TRANSFORMER_IMPLEMENTATION
#include "common/transformer.h"

float ref_fp16_to_fp32(uint16_t h) { return ggml_fp16_to_fp32(h); }
void ref_fp16_table(float *out) { for (uint32_t h = 0; h < 65536u; h++) out[h] = ggml_fp16_to_fp32((uint16_t)h); }
int ref_dequant_row(uint32_t type, const void *src, float *dst, int n) { return dequant_row(type, src, dst, n); }
size_t ref_dequant_row_size(uint32_t type, int n) { return dequant_row_size(type, n); }
size_t ref_tf_row_bytes(uint32_t type, int n_cols) { return tf_row_bytes(type, n_cols); }

static qtensor make_qt(const void *data, uint32_t type, int n_rows, int n_cols) {
    qtensor t;
    memset(&t, 0, sizeof(t));
    t.data = (void *)data;
    t.type = type;
    t.n_rows = n_rows;
    t.n_cols = n_cols;
    t.n_dims = 2;
    t.dims[0] = (uint64_t)n_cols;
    t.dims[1] = (uint64_t)n_rows;
    return t;
}

/* tf_qmatvec on a 2-D tensor; f64_accum selects the reference's double-accumulate oracle mode
 * (which only exists in the worker, so it is reached through a 1-thread pool call). */
void ref_tf_qmatvec(float *dst, const void *W, uint32_t type, const float *x, int n_rows, int n_cols) {
    qtensor t = make_qt(W, type, n_rows, n_cols);
    float *tmp = (float *)malloc((size_t)n_cols * sizeof(float));
    tf_qmatvec(dst, &t, x, n_rows, tmp);
    free(tmp);
}

void ref_tf_qmatvec_f64(float *dst, const void *W, uint32_t type, const float *x, int n_rows, int n_cols) {
    qtensor t = make_qt(W, type, n_rows, n_cols);
    float *tmp = (float *)malloc((size_t)n_cols * sizeof(float));
    tf_matvec_task task = {dst, &t, x, 0, n_rows, tmp};
    int saved = tf_g_f64_accum;
    tf_g_f64_accum = 1;
    tf_qmatvec_worker(&task);
    tf_g_f64_accum = saved;
    free(tmp);
}

void ref_tf_qmatvec_expert(float *dst, const void *W, uint32_t type, int expert, const float *x,
                           int rows_per_expert, int n_cols) {
    qtensor t = make_qt(W, type, rows_per_expert, n_cols);
    float *tmp = (float *)malloc((size_t)n_cols * sizeof(float));
    tf_qmatvec_expert(dst, &t, expert, x, rows_per_expert, tmp);
    free(tmp);
}

void ref_tf_gemm_tokenmajor(float *Y, const void *W, uint32_t type, const float *X, int n_rows,
                            int n_cols, int N, int out_stride, int X_stride, int n_threads) {
    qtensor t = make_qt(W, type, n_rows, n_cols);
    tf_gemm_f16_mt_tokenmajor(Y, &t, X, n_rows, N, out_stride, X_stride, n_threads);
}

void ref_tf_softmax(float *x, int n) { tf_softmax(x, n); }
void ref_tf_silu_mul(float *out, const float *gate, const float *up, int n) { tf_silu_mul_avx2(out, gate, up, n); }

/* tf_qmatvec_pool on a stand-in model that only carries what the pool path reads: thread
 * count, per-thread scratch and the pool itself. Returns seconds per call over `iters` calls. */
double ref_tf_qmatvec_pool_time(float *dst, const void *W, uint32_t type, const float *x,
                                int n_rows, int n_cols, int n_threads, int iters) {
    transformer_model *m = (transformer_model *)calloc(1, sizeof(transformer_model));
    qtensor t = make_qt(W, type, n_rows, n_cols);
    if (n_threads < 1) n_threads = 1;
    m->n_threads = n_threads;
    m->thread_tmp = (float **)calloc((size_t)n_threads, sizeof(float *));
    for (int i = 0; i < n_threads; i++) m->thread_tmp[i] = (float *)calloc((size_t)n_cols, sizeof(float));
    if (n_threads > 1) tf_pool_start(m);
    tf_qmatvec_pool(m, dst, &t, x, n_rows); /* warm-up */
    struct timespec a, b;
    clock_gettime(CLOCK_MONOTONIC, &a);
    for (int i = 0; i < iters; i++) tf_qmatvec_pool(m, dst, &t, x, n_rows);
    clock_gettime(CLOCK_MONOTONIC, &b);
    if (n_threads > 1) tf_pool_shutdown(m);
    for (int i = 0; i < n_threads; i++) free(m->thread_tmp[i]);
    free(m->thread_tmp);
    free(m);
    return ((double)(b.tv_sec - a.tv_sec) + 1e-9 * (double)(b.tv_nsec - a.tv_nsec)) / (double)(iters > 0 ? iters : 1);
}

const void *ref_table(const char *name, size_t *bytes) {
    if (!strcmp(name, "iq2xxs_grid")) { *bytes = sizeof(iq2xxs_grid); return iq2xxs_grid; }
    if (!strcmp(name, "iq3s_grid")) { *bytes = sizeof(iq3s_grid); return iq3s_grid; }
    if (!strcmp(name, "iq4nl_values")) { *bytes = sizeof(kvalues_iq4nl); return kvalues_iq4nl; }
    if (!strcmp(name, "ksigns")) { *bytes = sizeof(ksigns_iq2xs); return ksigns_iq2xs; }
    if (!strcmp(name, "mxfp4_values")) { *bytes = sizeof(kvalues_mxfp4); return kvalues_mxfp4; }
    if (!strcmp(name, "iq3xxs_grid")) { *bytes = sizeof(iq3xxs_grid); return iq3xxs_grid; }
    if (!strcmp(name, "iq2xs_grid")) { *bytes = sizeof(iq2xs_grid); return iq2xs_grid; }
    if (!strcmp(name, "iq2s_grid")) { *bytes = sizeof(iq2s_grid); return iq2s_grid; }
    if (!strcmp(name, "iq1s_grid")) { *bytes = sizeof(iq1s_grid); return iq1s_grid; }
    *bytes = 0;
    return NULL;
}

/* ---- GGUF loader of the reference, for the fixture of the file parser ---- */
void *ref_gguf_open(const char *path) { return gguf_open(path, 0); }
void ref_gguf_close(void *c) { gguf_close((gguf_context *)c); }
uint64_t ref_gguf_n_tensors(const void *c) { return ((const gguf_context *)c)->n_tensors; }
uint64_t ref_gguf_n_kv(const void *c) { return ((const gguf_context *)c)->n_kv; }
uint32_t ref_gguf_version(const void *c) { return ((const gguf_context *)c)->version; }
uint32_t ref_gguf_alignment(const void *c) { return ((const gguf_context *)c)->alignment; }
uint64_t ref_gguf_data_offset(const void *c) { return ((const gguf_context *)c)->data_offset; }
uint64_t ref_gguf_data_size(const void *c) { return ((const gguf_context *)c)->data_size; }
const char *ref_gguf_tensor_name(const void *c, int i) { return gguf_tensor_name((const gguf_context *)c, i); }
uint64_t ref_gguf_tensor_size(const void *c, int i) { return gguf_tensor_size((const gguf_context *)c, i); }
const void *ref_gguf_tensor_data(const void *c, int i) { return gguf_tensor_data((const gguf_context *)c, i); }
/* out: type, n_dims, dims[4], offset */
void ref_gguf_tensor_info(const void *c, int i, uint64_t out[7]) {
    const gguf_tensor_info *t = &((const gguf_context *)c)->tensors[i];
    out[0] = t->type; out[1] = t->n_dims;
    for (int d = 0; d < 4; d++) out[2 + d] = t->dims[d];
    out[6] = t->offset;
}
/* the qtensor tf_load_tensor builds for a name: out = type, n_rows, n_cols, n_dims; returns the data
 * offset from the start of the data section, or -1 if the tensor is missing */
int64_t ref_tf_load_tensor(const void *c, const char *name, int64_t out[4]) {
    const gguf_context *g = (const gguf_context *)c;
    qtensor t = tf_load_tensor(g, name, 0);
    if (!t.data) return -1;
    out[0] = t.type; out[1] = t.n_rows; out[2] = t.n_cols; out[3] = t.n_dims;
    return (int64_t)((const uint8_t *)t.data - g->data);
}
int ref_gguf_find_key(const void *c, const char *key) { return gguf_find_key((const gguf_context *)c, key); }
uint32_t ref_gguf_kv_type(const void *c, int i) { return ((const gguf_context *)c)->kv[i].type; }
uint64_t ref_gguf_kv_u64(const void *c, int i) { return ((const gguf_context *)c)->kv[i].value.u64; }
const char *ref_gguf_kv_str(const void *c, int i) { return ((const gguf_context *)c)->kv[i].value.str.str; }
uint64_t ref_gguf_kv_arr_n(const void *c, int i) { return ((const gguf_context *)c)->kv[i].value.arr.n; }
int ref_tf_get_int(const void *c, const char *key, int dflt) { return tf_get_int((const gguf_context *)c, key, dflt); }
