/*
 * test_tf_mirror.c - exercises the reference-shaped C wrappers (include/qlinear_tf.h) the way a C
 * engine written against common/transformer.h would: qtensor structs over host memory, void calls.
 * Needs a GPU. Checks each linear call against a double-precision dot over rows decoded with
 * qtf_dequant_row (whose bit-exactness the Python parity tests establish separately).
 * Exit code 0 = all checks passed.
 */
#define QLINEAR_TF_REFERENCE_NAMES
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "qlinear.h"
#include "qlinear_tf.h"

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint32_t rnd(void) {
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 7;
    rng_state ^= rng_state << 17;
    return (uint32_t)(rng_state >> 32);
}
static float rndf(void) { return (float)(rnd() >> 8) * (1.0f / 8388608.0f) - 1.0f; }

/* random blocks with a small positive fp16 in every fp16 slot of the block header */
static qtensor make_tensor(uint32_t type, int n_rows, int n_cols) {
    qtensor t;
    memset(&t, 0, sizeof t);
    const size_t rb = tf_row_bytes(type, n_cols);
    uint8_t *p = (uint8_t *)malloc(rb * (size_t)n_rows);
    for (size_t i = 0; i < rb * (size_t)n_rows; i++) p[i] = (uint8_t)rnd();
    const int bb = type == 8 ? 34 : type == 12 ? 144 : type == 17 ? 74 : 210;
    for (size_t off = 0; off + bb <= rb * (size_t)n_rows; off += bb) {
        const uint16_t h = (uint16_t)(0x1C00 + (rnd() & 0x3FF)); /* 2^-8 .. 2^-7 */
        if (type == 14) memcpy(p + off + 208, &h, 2);
        else {
            memcpy(p + off, &h, 2);
            if (type == 12) memcpy(p + off + 2, &h, 2);
        }
    }
    t.data = p; t.type = type; t.n_rows = n_rows; t.n_cols = n_cols; t.n_dims = 2;
    t.dims[0] = (uint64_t)n_cols; t.dims[1] = (uint64_t)n_rows;
    return t;
}

static int failures = 0;
static void check_rows(const char *what, const qtensor *t, int row0, int n_rows, const float *x, const float *got) {
    float *dec = (float *)malloc(sizeof(float) * (size_t)t->n_cols);
    double num = 0, den = 0;
    for (int r = 0; r < n_rows; r++) {
        tf_dequant_row(t, row0 + r, dec);
        double s = 0;
        for (int c = 0; c < t->n_cols; c++) s += (double)dec[c] * (double)x[c];
        num += (s - got[r]) * (s - got[r]);
        den += s * s;
    }
    free(dec);
    const double rel = sqrt(num / (den > 0 ? den : 1));
    printf("%-28s rel-L2 %.3e %s\n", what, rel, rel <= 1e-5 ? "ok" : "FAIL");
    if (!(rel <= 1e-5)) failures++;
}

int main(void) {
    if (qlin_init(0) != QLIN_OK) { fprintf(stderr, "init: %s\n", qlin_last_error()); return 2; }
    const int K = 1024;
    float *x = (float *)malloc(sizeof(float) * K * 3);
    for (int i = 0; i < K * 3; i++) x[i] = rndf();
    float y[512], y2[512], y3[512];

    qtensor a = make_tensor(12, 256, K), b = make_tensor(12, 256, K), c8 = make_tensor(8, 96, K),
            c6 = make_tensor(14, 96, K);
    /* 17 = IQ2_XS is a model weight type; 3 = Q4_1 has a decoder but is not one (common/transformer.h:462-487) */
    if (tf_is_supported_weight_type(12) != 1 || tf_is_supported_weight_type(17) != 1 || tf_is_supported_weight_type(3) != 0) { printf("type check FAIL\n"); failures++; }
    if (tf_row_bytes(12, 4096) != 2304 || tf_row_bytes(17, 4096) != 1184 || tf_row_bytes(3, 4096) != 0 || tf_row_bytes(99, 4096) != 0) { printf("row bytes FAIL\n"); failures++; }
    qtensor c17 = make_tensor(17, 96, K);
    tf_qmatvec(y, &c17, x, 96, NULL);
    check_rows("tf_qmatvec iq2_xs", &c17, 0, 96, x, y);

    tf_qmatvec(y, &a, x, 256, NULL);
    check_rows("tf_qmatvec q4_K", &a, 0, 256, x, y);
    if (qtf_register_tensor(&a) != 0) { printf("register FAIL\n"); failures++; }
    struct { const float *xb; } model = {x}, *m = &model; /* what the reference's pool calls read from the model */
    tf_qmatvec_pool(m, y, &a, x, 200); /* fewer rows than the tensor holds */
    check_rows("qmatvec_pool registered", &a, 0, 200, x, y);

    tf_qmatvec_fused2_pool(m, y, &a, y2, &b, x, 256);
    check_rows("fused2 first", &a, 0, 256, x, y);
    check_rows("fused2 second", &b, 0, 256, x, y2);

    tf_qmatvec_fused_qkv_pool(m, y, &a, 256, y2, &c8, y3, &c6, 96);
    check_rows("fused qkv q (q4_K)", &a, 0, 256, x, y);
    check_rows("fused qkv k (q8_0)", &c8, 0, 96, x, y2);
    check_rows("fused qkv v (q6_K)", &c6, 0, 96, x, y3);

    /* gate+up+SiLU, projection+residual, output projection + greedy pick */
    {
        float g[256], u[256], want[256];
        tf_qmatvec(g, &a, x, 256, NULL);
        tf_qmatvec(u, &b, x, 256, NULL);
        tf_qmatvec_fused2_silu_pool(NULL, y, &a, &b, x, 256);
        double num = 0, den = 0;
        for (int i = 0; i < 256; i++) {
            want[i] = (float)((double)g[i] / (1.0 + exp(-(double)g[i])) * (double)u[i]);
            num += ((double)y[i] - want[i]) * ((double)y[i] - want[i]);
            den += (double)want[i] * want[i];
        }
        printf("%-28s rel-L2 %.3e %s\n", "fused2 silu", sqrt(num / den), sqrt(num / den) <= 1e-5 ? "ok" : "FAIL");
        if (!(sqrt(num / den) <= 1e-5)) failures++;
        for (int i = 0; i < 256; i++) y2[i] = 0.25f * (float)i;
        qtf_qmatvec_add(x, y2, &a, 256);
        num = den = 0;
        for (int i = 0; i < 256; i++) {
            const double w = 0.25 * i + (double)g[i];
            num += ((double)y2[i] - w) * ((double)y2[i] - w);
            den += w * w;
        }
        printf("%-28s rel-L2 %.3e %s\n", "projection + residual", sqrt(num / den), sqrt(num / den) <= 1e-5 ? "ok" : "FAIL");
        if (!(sqrt(num / den) <= 1e-5)) failures++;
        int best = 0;
        for (int i = 1; i < 256; i++) if (g[i] > g[best]) best = i;
        const int got = qtf_logits_argmax(x, &a, 256, y3);
        printf("%-28s %d vs %d %s\n", "logits argmax", got, best, got == best ? "ok" : "FAIL");
        if (got != best) failures++;
    }

    tf_qmatvec_expert(y, &a, 3, x, 64, NULL); /* 4 experts of 64 rows */
    check_rows("tf_qmatvec_expert", &a, 192, 64, x, y);
    tf_qmatvec_expert_pool(m, y, &a, 2, x, 64);
    check_rows("tf_qmatvec_expert_pool", &a, 128, 64, x, y);

    /* prefill, token-major with strides wider than the data */
    float *Y = (float *)malloc(sizeof(float) * 3 * 300);
    for (int i = 0; i < 900; i++) Y[i] = -5.0f;
    tf_gemm_f16_mt_tokenmajor(Y, &b, x, 256, 3, 300, K, 8);
    for (int t = 0; t < 3; t++) check_rows("gemm tokenmajor token", &b, 0, 256, x + (size_t)t * K, Y + (size_t)t * 300);
    if (Y[256] != -5.0f || Y[299] != -5.0f) { printf("gemm wrote outside its rows FAIL\n"); failures++; }

    /* failure behaviour: unsupported type -> message on stderr, zero-filled output, no crash */
    qtensor bad = a;
    bad.type = 9; /* Q8_1: an activation format, no weight decoder */
    for (int i = 0; i < 256; i++) y[i] = 1.0f;
    tf_qmatvec(y, &bad, x, 256, NULL);
    int zeros = 1;
    for (int i = 0; i < 256; i++) zeros &= (y[i] == 0.0f);
    printf("%-28s %s\n", "unsupported type zero-fill", zeros ? "ok" : "FAIL");
    if (!zeros) failures++;

    qtf_unregister_tensor(&a);
    qlin_shutdown();
    printf("%s\n", failures ? "FAILED" : "all C-mirror checks passed");
    return failures ? 1 : 0;
}
