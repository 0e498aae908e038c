/*
 * test_tf_mirror.c - exercises the reference-shaped C wrappers (include/qlinear_tf.h) the way a C
 * engine written against common/transformer.h would: qtensor structs over host memory, void calls.
 * Needs a GPU. Checks each linear call against a double-precision dot over rows decoded with
 * qtf_dequant_row (whose bit-exactness the Python parity tests establish separately).
 * Exit code 0 = all checks passed.
 */
#define QLINEAR_TF_REFERENCE_NAMES
#define QLINEAR_GGML_REFERENCE_NAMES
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "qlinear.h"
#include "qlinear_tf.h"
#include "qlinear_ggml.h"

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

/* the codec under the names of common/ggml_dequant.h: every per-type decoder once against dequant_row of its type
 * (bit for bit), the row sizes, the half conversion over all 65536 patterns, and the Q8_0 products */
typedef void (*row_decoder)(const void *, float *, int);
static void check_ggml_names(void) {
    static const struct { const char *name; uint32_t type; int block_elems, block_bytes; row_decoder fn; } dec[] = {
        {"q2_K", 10, 256, 84, dequantize_row_q2_K},       {"q3_K", 11, 256, 110, dequantize_row_q3_K},
        {"q8_0", 8, 32, 34, dequantize_row_q8_0},         {"q1_0", 41, 128, 18, dequantize_row_q1_0},
        {"mxfp4", 39, 32, 17, dequantize_row_mxfp4},      {"nvfp4", 40, 64, 36, dequantize_row_nvfp4},
        {"q4_K", 12, 256, 144, dequantize_row_q4_K},      {"q5_K", 13, 256, 176, dequantize_row_q5_K},
        {"q6_K", 14, 256, 210, dequantize_row_q6_K},      {"iq2_xxs", 16, 256, 66, dequantize_row_iq2_xxs},
        {"q4_0", 2, 32, 18, dequantize_row_q4_0},         {"q4_1", 3, 32, 20, dequantize_row_q4_1},
        {"q5_0", 6, 32, 22, dequantize_row_q5_0},         {"q5_1", 7, 32, 24, dequantize_row_q5_1},
        {"iq2_xs", 17, 256, 74, dequantize_row_iq2_xs},   {"iq2_s", 22, 256, 82, dequantize_row_iq2_s},
        {"iq3_xxs", 18, 256, 98, dequantize_row_iq3_xxs}, {"iq3_s", 21, 256, 110, dequantize_row_iq3_s},
        {"iq4_nl", 20, 32, 18, dequantize_row_iq4_nl},    {"iq4_xs", 23, 256, 136, dequantize_row_iq4_xs},
        {"iq1_s", 19, 256, 50, dequantize_row_iq1_s},     {"iq1_m", 29, 256, 56, dequantize_row_iq1_m},
        {"tq1_0", 34, 256, 54, dequantize_row_tq1_0},     {"tq2_0", 35, 256, 66, dequantize_row_tq2_0},
        {"bf16", 30, 1, 2, dequantize_row_bf16},
    };
    const int n = 512;
    uint8_t *src = (uint8_t *)malloc(2 * n + 4096);
    float *a = (float *)malloc(sizeof(float) * n), *b = (float *)malloc(sizeof(float) * n);
    int bad = 0;
    for (size_t i = 0; i < sizeof dec / sizeof dec[0]; i++) {
        const size_t bytes = (size_t)(n / dec[i].block_elems) * dec[i].block_bytes;
        if (dequant_row_size(dec[i].type, n) != bytes) { printf("dequant_row_size %s FAIL\n", dec[i].name); bad++; }
        for (size_t j = 0; j < bytes; j++) src[j] = (uint8_t)rnd();
        memset(a, 0xAA, sizeof(float) * n);
        memset(b, 0x55, sizeof(float) * n);
        dec[i].fn(src, a, n);
        if (dequant_row(dec[i].type, src, b, n) != 0 || memcmp(a, b, sizeof(float) * n) != 0) {
            printf("dequantize_row_%s vs dequant_row FAIL\n", dec[i].name);
            bad++;
        }
    }
    if (dequant_row(9, src, a, n) != -1 || dequant_row_size(9, n) != 0) { printf("unsupported type FAIL\n"); bad++; }
    printf("%-28s %s\n", "ggml decoder names (25)", bad ? "FAIL" : "ok");
    failures += bad;

    /* ggml_fp16_to_fp32 against the library's F16 decoder, all patterns, bit for bit */
    uint16_t *h = (uint16_t *)malloc(2 * 65536);
    float *f = (float *)malloc(4 * 65536);
    for (int i = 0; i < 65536; i++) h[i] = (uint16_t)i;
    bad = dequant_row(1, h, f, 65536) != 0;
    for (int i = 0; i < 65536 && !bad; i++) {
        const float g = ggml_fp16_to_fp32((uint16_t)i);
        if (memcmp(&g, &f[i], 4) != 0 && !(g != g && f[i] != f[i])) { printf("fp16 0x%04x FAIL\n", i); bad = 1; }
    }
    printf("%-28s %s\n", "ggml_fp16_to_fp32 (65536)", bad ? "FAIL" : "ok");
    failures += bad;
    free(h); free(f); free(src); free(a); free(b);

    /* Q8_0 row dot, one-row matvec, token-major GEMM */
    const int K = 1024, R = 40, N = 3;
    qtensor w = make_tensor(8, R, K);
    float *x = (float *)malloc(sizeof(float) * K * N), *Y = (float *)malloc(sizeof(float) * N * 64);
    for (int i = 0; i < K * N; i++) x[i] = rndf();
    float one[1], two[1];
    one[0] = vec_dot_q8_0_f32((const uint8_t *)w.data + 5 * dequant_row_size(8, K), x, K);
    check_rows("vec_dot_q8_0_f32", &w, 5, 1, x, one);
    matvec_q8_0_f32(two, (const uint8_t *)w.data + 7 * dequant_row_size(8, K), x, K);
    check_rows("matvec_q8_0_f32", &w, 7, 1, x, two);
    for (int i = 0; i < N * 64; i++) Y[i] = -5.0f;
    gemm_q8_0_f32_tokmajor(Y, w.data, x, R, K, N, 64, K);
    for (int t = 0; t < N; t++) check_rows("gemm_q8_0_f32_tokmajor", &w, 0, R, x + (size_t)t * K, Y + (size_t)t * 64);
    if (Y[R] != -5.0f || Y[63] != -5.0f) { printf("gemm_q8_0 wrote outside its rows FAIL\n"); failures++; }
    free(x); free(Y); free(w.data);
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

    check_ggml_names();

    qtf_unregister_tensor(&a);
    qlin_shutdown();
    printf("%s\n", failures ? "FAILED" : "all C-mirror checks passed");
    return failures ? 1 : 0;
}
