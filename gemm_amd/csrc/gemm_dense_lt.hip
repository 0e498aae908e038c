/*
 * gemm_dense_lt.hip - prefill GEMM for every weight format: decode W once in a caller-provided
 * workspace (dequant kernels, one pass at HBM speed), then a plain dense GEMM with fp32 accumulation,
 * which is the vendor library's job (hipBLASLt; transposed-A form). Two operand types:
 *
 *   bf16:  Y[t*ldy + r] = sum_k X[t*ldx + k] * bf16(decode(W)[r][k])      X bf16
 *   fp32:  Y[t*ldy + r] = sum_k X[t*ldx + k] * decode(W)[r][k]            X fp32, weights exact
 *
 * This is the shape of tf_gemm_f16_mt_tokenmajor (common/transformer.h:4487-4595), which converts a
 * weight row to a 16-bit float row and multiplies it with every token; its fast paths cover Q8_0, F16
 * and BF16 only and every other format falls back to one re-decode per token (:4535-4572). Rounding the
 * decoded weights to bf16 costs 1.8e-3 relative L2 on Y against exact weights, as in the fused Q4_K
 * tile kernel.
 *
 * In column-major terms (what the library speaks): C (n_rows x n_tok, ld ldy) = A^T * B with
 * A = the bf16 weights (n_cols x n_rows, ld n_cols) and B = X (n_cols x n_tok, ld ldx).
 */
#include <hipblaslt/hipblaslt.h>

#include <array>
#include <map>
#include <mutex>

#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

namespace {

struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t ws_bytes = 0; /* workspace the algorithm was chosen for */
};

std::mutex g_mu;
hipblasLtHandle_t g_handle = nullptr;
std::map<std::array<long long, 6>, Plan> g_plans; /* (fp32?, n_rows, n_cols, n_tok, ldx, ldy) -> plan; at most kMaxPlans */

constexpr size_t kMaxPlans = 512;

void destroy_plan(Plan &p) {
    if (p.a) hipblasLtMatrixLayoutDestroy(p.a);
    if (p.b) hipblasLtMatrixLayoutDestroy(p.b);
    if (p.c) hipblasLtMatrixLayoutDestroy(p.c);
    if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
    p = Plan();
}

const char *make_plan(Plan &p, bool fp32, long long n_rows, long long n_cols, long long n_tok, long long ldx,
                      long long ldy, size_t lib_ws_bytes) {
    const hipDataType in = fp32 ? HIP_R_32F : HIP_R_16BF;
    if (hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS)
        return "hipblasLtMatmulDescCreate failed";
    const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
    if (hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)) != HIPBLAS_STATUS_SUCCESS)
        return "hipblasLtMatmulDescSetAttribute failed";
    if (hipblasLtMatrixLayoutCreate(&p.a, in, n_cols, n_rows, n_cols) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatrixLayoutCreate(&p.b, in, n_cols, n_tok, ldx) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatrixLayoutCreate(&p.c, HIP_R_32F, n_rows, n_tok, ldy) != HIPBLAS_STATUS_SUCCESS)
        return "hipblasLtMatrixLayoutCreate failed";
    hipblasLtMatmulPreference_t pref = nullptr;
    if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return "hipblasLtMatmulPreferenceCreate failed";
    /* The library's kernels that split K over workgroups and reduce through the workspace write a padded
     * output (ldy > n_rows) as if it were dense (measured: K = 8192 and up with few output tiles, relative
     * error 1.4). Offering no workspace leaves only kernels that write Y themselves. */
    if (ldy != n_rows) lib_ws_bytes = 0;
    hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &lib_ws_bytes, sizeof(lib_ws_bytes));
    hipblasLtMatmulHeuristicResult_t res[1];
    int n = 0;
    const hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.a, p.b, p.c, p.c, pref, 1, res, &n);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (st != HIPBLAS_STATUS_SUCCESS || n == 0) return "the library offers no algorithm for this shape";
    p.algo = res[0].algo;
    p.ws_bytes = lib_ws_bytes;
    return nullptr;
}

}  // namespace

size_t dense_gemm_weight_bytes(int n_rows, int n_cols) {
    return ((size_t)n_rows * n_cols * 2 + 255) & ~(size_t)255;
}
size_t dense_gemm_weight_bytes_f32(int n_rows, int n_cols) {
    return ((size_t)n_rows * n_cols * 4 + 255) & ~(size_t)255;
}

/* Wd and X are both bf16 (fp32_operands == false) or both fp32; nullptr on success, else what failed */
const char *launch_gemm_dense(bool fp32_operands, const void *Wd, const void *X, float *Y, int n_rows, int n_cols,
                              int n_tok, int ldx, int ldy, void *lib_ws, size_t lib_ws_bytes, hipStream_t stream) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_handle && hipblasLtCreate(&g_handle) != HIPBLAS_STATUS_SUCCESS) {
        g_handle = nullptr;
        return "hipblasLtCreate failed";
    }
    const std::array<long long, 6> key = {fp32_operands ? 1 : 0, n_rows, n_cols, n_tok, ldx, ldy};
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
        if (g_plans.size() >= kMaxPlans) { /* a caller with ever-changing token counts: start over */
            for (auto &kv : g_plans) destroy_plan(kv.second);
            g_plans.clear();
        }
        Plan p;
        if (const char *err = make_plan(p, fp32_operands, n_rows, n_cols, n_tok, ldx, ldy, lib_ws_bytes)) {
            destroy_plan(p);
            return err;
        }
        it = g_plans.emplace(key, p).first;
    }
    const Plan &p = it->second;
    const float alpha = 1.0f, beta = 0.0f;
    if (hipblasLtMatmul(g_handle, p.desc, &alpha, Wd, p.a, X, p.b, &beta, Y, p.c, Y, p.c, &p.algo, p.ws_bytes ? lib_ws : nullptr,
                        p.ws_bytes, stream) != HIPBLAS_STATUS_SUCCESS)
        return "hipblasLtMatmul failed";
    return nullptr;
}

const char *launch_gemm_dense_bf16(const uint16_t *Wd, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok,
                                   int ldx, int ldy, void *lib_ws, size_t lib_ws_bytes, hipStream_t stream) {
    return launch_gemm_dense(false, Wd, X, Y, n_rows, n_cols, n_tok, ldx, ldy, lib_ws, lib_ws_bytes, stream);
}

}  // namespace qlin
