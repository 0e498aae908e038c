/*
 * qlin_internal.h - host-side launchers shared between the translation units of libqlinear.
 * Every launcher validates nothing: the C-ABI layer (qlin_api.hip) checks shapes, alignment
 * and types before it calls in here. All return the hipError_t of the launch.
 */
#ifndef QLIN_INTERNAL_H
#define QLIN_INTERNAL_H

#include <hip/hip_runtime.h>

#include <atomic>
#include <stddef.h>
#include <stdint.h>

#include "qlin_device.h"

namespace qlin {

/* "this kernel's dynamic LDS limit has been raised": set after hipFuncSetAttribute succeeded. Device entry
 * points may be called from several threads; raising the limit twice is harmless, a torn flag is not. */
struct OnceFlag {
    std::atomic<bool> done{false};
    bool is_set() const { return done.load(std::memory_order_acquire); }
    void set() { done.store(true, std::memory_order_release); }
};

/* out[n_rows, n_cols] = decode(W); n_cols may be ragged: only n_cols / block_elems blocks per
 * row are decoded, row r of W starts at r * row_bytes, row r of out at r * n_cols. With row_ids
 * (device, n_rows entries) output row r is decoded from source row row_ids[r] of a table of
 * n_src_rows rows (zeros for an id outside it); without, n_src_rows is ignored. */
hipError_t launch_dequant(uint32_t type, const void *W, const int32_t *row_ids, int n_src_rows, float *out,
                          int n_rows, int n_cols, size_t row_bytes, hipStream_t stream);

/* One matvec launch over up to three matrices of ONE block type that share x and n_cols: the
 * fused call shapes of the reference's decode loop.
 *   kStore    y_m[r] = W_m[r,:] . x for every matrix m (rows of the matrices are concatenated:
 *             tf_qmatvec_fused2_pool, tf_qmatvec_fused_qkv_pool, common/transformer.h:897, :1021)
 *   kAdd      y_m[r] += W_m[r,:] . x   (projection followed by the residual add, :4037)
 *   kSiluMul  two matrices of equal row count: y_0[r] = silu(W_0[r,:].x) * (W_1[r,:].x)
 *             (tf_qmatvec_fused2_silu_pool, :953; silu(g) = g / (1 + exp(-g))) */
enum GemvMode : int { kStore = 0, kAdd = 1, kSiluMul = 2 };
struct GemvJob {
    const void *W[3];
    float *y[3];
    int n_rows[3];
    int n_mat;   /* 1..3; kSiluMul: 2 */
    int mode;    /* GemvMode */
    int total_rows() const { return n_rows[0] + (n_mat > 1 ? n_rows[1] : 0) + (n_mat > 2 ? n_rows[2] : 0); }
};
inline GemvJob single_job(const void *W, float *y, int n_rows, int mode = kStore) {
    GemvJob j = {{W, nullptr, nullptr}, {y, nullptr, nullptr}, {n_rows, 0, 0}, 1, mode};
    return j;
}

inline JobView job_view(const GemvJob &job) {
    const JobView v = {(const uint8_t *)job.W[0], (const uint8_t *)job.W[1], (const uint8_t *)job.W[2],
                       job.y[0], job.y[1], job.y[2],
                       job.n_rows[0], job.n_mat > 1 ? job.n_rows[1] : 0, job.n_mat > 2 ? job.n_rows[2] : 0, job.mode};
    return v;
}

/* one job: y[n_rows] = W . x (or the fused forms above), any supported type and any whole-block shape */
hipError_t launch_gemv_generic(uint32_t type, const GemvJob &job, const float *x, int n_cols, hipStream_t stream);
/* dense F32/F16/BF16 rows of any length and element alignment, one element per lane and step */
hipError_t launch_gemv_dense_ragged(uint32_t type, const GemvJob &job, const float *x, int n_cols, hipStream_t stream);
/* dense rows of 4097..16384 elements in one launch; false: not this kernel's shape */
bool launch_gemv_dense_long(uint32_t type, const GemvJob &job, const float *x, int n_cols, int n_cu, hipStream_t stream,
                            hipError_t *err, size_t row_stride = 0);
/* streaming matvec for every type; returns false if the shape rules of gemv_stream.hip do not
 * hold (nothing was launched), else true with the launch status in *err */
/* row_stride (all four kernels below): bytes between the rows of a matrix; 0 = the rows are packed. Anything else
 * runs the kernel over a column range of longer rows (W then points at the range's first block of row 0). */
bool launch_gemv_stream(uint32_t type, const GemvJob &job, const float *x, int n_cols, int n_cu,
                        hipStream_t stream, hipError_t *err, size_t row_stride = 0);
/* integer-dot matvec (gemv_int.hip) for the formats it covers; same contract as launch_gemv_stream */
bool launch_gemv_int(uint32_t type, const GemvJob &job, const float *x, int n_cols, int n_cu,
                     hipStream_t stream, hipError_t *err, size_t row_stride = 0);
/* the formats whose rows launch_gemv_int reads from any even address (the others want 16-byte boundaries) */
bool gemv_int_takes_any_even_address(uint32_t type);
/* matrix-instruction matvec for the formats of gemv_grid_covers (gemv_grid.hip): n_cols % 256 == 0, n_cols <= 16384,
 * rows of up to 4096 elements only where it measured faster; same contract as launch_gemv_stream */
bool launch_gemv_grid(uint32_t type, const GemvJob &job, const float *x, int n_cols, int n_cu,
                      hipStream_t stream, hipError_t *err, size_t row_stride = 0);
bool gemv_grid_covers(uint32_t type); /* the formats it has an item for */
/* A few tokens, each on its own, through their top_k experts as two matvec launches: gate + up + SiLU into h
 * (n_tok * top_k * n_ff floats, X [n_tok, n_embd] bf16), then down with the routing weights folded into h. Q4_K experts
 * and the formats of the matrix-instruction matvec (gate and up of one type). false: not a shape for it; dry: only say so. */
bool launch_moe1_q4k_up(const void *gate, const void *up, const uint16_t *X, const int32_t *idx, float *h, int n_tok,
                        int top_k, int n_embd, int n_ff, int n_expert, int n_cu, hipStream_t stream, bool dry, hipError_t *err);
bool launch_moe1_q4k_down(const void *down, const float *h, const int32_t *idx, const float *w, float *out, int n_tok, int top_k,
                          int n_embd, int n_ff, int n_expert, int n_cu, hipStream_t stream, bool dry, hipError_t *err);
bool launch_moe1_grid_up(uint32_t type, const void *gate, const void *up, const uint16_t *X, const int32_t *idx, float *h,
                         int n_tok, int top_k, int n_embd, int n_ff, int n_expert, int n_cu, hipStream_t stream, bool dry,
                         hipError_t *err);
bool launch_moe1_grid_down(uint32_t type, const void *down, const float *h, const int32_t *idx, const float *w, float *out,
                           int n_tok, int top_k, int n_embd, int n_ff, int n_expert, int n_cu, hipStream_t stream, bool dry,
                           hipError_t *err);
/* tuned Q4_K matvec: n_cols % 256 == 0, n_cols <= 16384, W and x 16-byte aligned */
hipError_t launch_gemv_q4k(const GemvJob &job, const float *x, int n_cols, hipStream_t stream, int n_cu,
                           size_t row_stride = 0);

/* Y[t*ldy + r] = dot(W[r,:], X[t*ldx..]) in fp32 */
hipError_t launch_gemm_f32(uint32_t type, const void *W, const float *X, float *Y, int n_rows,
                           int n_cols, int n_tok, int ldx, int ldy, hipStream_t stream);

/* Q4_K x bf16 on the matrix cores */
/* the same contraction for a handful of tokens: exact 4-bit codes through the matrix instruction, block
 * scales in fp32, weights streamed once per 16 tokens (moe_ffn_q4k.hip) */
/* any format: decode to bf16 (dequant.hip), then the dense library GEMM (gemm_dense_lt.hip) */
hipError_t launch_dequant_bf16(uint32_t type, const void *W, uint16_t *out, int n_rows, int n_cols, size_t row_bytes,
                               hipStream_t stream);
size_t dense_gemm_weight_bytes(int n_rows, int n_cols);
size_t dense_gemm_weight_bytes_f32(int n_rows, int n_cols);
const char *launch_gemm_dense(bool fp32_operands, const void *Wd, const void *X, float *Y, int n_rows, int n_cols,
                              int n_tok, int ldx, int ldy, void *lib_ws, size_t lib_ws_bytes, hipStream_t stream);
const char *launch_gemm_dense_bf16(const uint16_t *Wd, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok,
                                   int ldx, int ldy, void *lib_ws, size_t lib_ws_bytes, hipStream_t stream);
/* this library's dense bf16 x bf16 tile kernel (gemm_dense_mfma.hip): n_cols % 256 == 0, Wd and X 16-byte
 * aligned, ldx % 8 == 0 */
hipError_t launch_gemm_dense_own(const uint16_t *Wd, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok,
                                 int ldx, int ldy, hipStream_t stream);
constexpr int kKqFewTokens = 24; /* up to this many tokens Q6_K, Q5_K, Q3_K, Q2_K and Q8_0 tensors are streamed once per
                                    eight tokens with exact codes instead of decoded to bf16 for the library's GEMM */
/* false: not a shape for this kernel (the caller takes another route); true: launched, *err says how it went */
bool launch_gemm_kq_fewtok(uint32_t type, const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok,
                           int ldx, int ldy, hipStream_t stream, hipError_t *err);
constexpr int kMatvecTokens = 4; /* qlin_gemm_bf16_any_dev: up to this many tokens of a format without a few-token kernel go through the matvec */
constexpr int kFewTokens = 32; /* launch_gemm_q4k_bf16 hands token counts up to this to the few-token kernel (14336 x 4096:
                                  24 us at 32 tokens, 34 at 48; the small-tile kernel 26 for up to 128) */
hipError_t launch_gemm_q4k_fewtok(const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok,
                                  int ldx, int ldy, hipStream_t stream);
/* 256-token x 128-row tiles on four waves, one per SIMD, weights decoded from their blocks into the matrix operand
 * (gemm_kq_wave4.hip): the formats of gemm_kq_wave4_covers, n_cols % 256 == 0, ldx < 2^22 */
bool gemm_kq_wave4_covers(uint32_t type);
/* the same in 128-token x 64-row tiles, two workgroups per compute unit (gemm_kq_wave4s.hip) */
hipError_t launch_gemm_kq_bf16_wave4s(uint32_t type, const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols,
                                      int n_tok, int ldx, int ldy, hipStream_t stream);
/* the same kernel over up to three tensors of one format and K in one launch (row tiles numbered through the tensors) */
hipError_t launch_gemm_kq_bf16_wave4_multi(uint32_t type, int n_mat, const void *const *W, const uint16_t *X,
                                           float *const *Y, const int *n_rows, int n_cols, int n_tok, int ldx,
                                           const int *ldy, hipStream_t stream);
hipError_t launch_gemm_kq_bf16_wave4s_multi(uint32_t type, int n_mat, const void *const *W, const uint16_t *X,
                                            float *const *Y, const int *n_rows, int n_cols, int n_tok, int ldx,
                                            const int *ldy, hipStream_t stream);
/* the fused kernel for a shape (kFusedNone: decode + dense product, or the format has none) and its launch */
enum FusedTile { kFusedNone = 0, kFusedLarge, kFusedSmall };
FusedTile choose_fused_tile(uint32_t type, int n_rows, int n_cols, int n_tok, int ldx, bool have_workspace);
hipError_t launch_fused_tile(FusedTile tile, uint32_t type, const void *W, const uint16_t *X, float *Y, int n_rows,
                             int n_cols, int n_tok, int ldx, int ldy, hipStream_t stream);
hipError_t launch_gemm_kq_bf16_wave4(uint32_t type, const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols,
                                     int n_tok, int ldx, int ldy, hipStream_t stream);
hipError_t launch_gemm_q4k_bf16_wave4(const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols, int n_tok,
                                      int ldx, int ldy, hipStream_t stream);
hipError_t launch_gemm_q4k_bf16(const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols,
                                int n_tok, int ldx, int ldy, hipStream_t stream);

/* grouped MoE expert FFN (bf16 activations): Q4_K matrices on the matrix cores, any other format through
 * the bit-exact codec in fp32; the three matrices may have different formats */
size_t moe_workspace_bytes(int n_tok, int top_k, int n_embd, int n_ff, int n_expert);
hipError_t launch_moe_ffn(uint32_t type_gate, uint32_t type_up, uint32_t type_down, const void *gate, const void *up,
                          const void *down, const uint16_t *X, const int32_t *idx, const float *w, float *out, int n_tok,
                          int top_k, int n_embd, int n_ff, int n_expert, int n_cu, void *workspace, hipStream_t stream);

/* the same with the workspace in a device array of the library (at most kMoeStaticScratchBytes); setup once per
 * device with that device current, before the first launch there */
constexpr size_t kMoeStaticScratchBytes = (size_t)16 << 20; /* = QLIN_MOE_STATIC_SCRATCH_BYTES of the public header */
constexpr int kMaxScratchDevices = 64;
hipError_t moe_static_scratch_setup(int device);
hipError_t launch_moe_ffn_static(uint32_t type_gate, uint32_t type_up, uint32_t type_down, const void *gate,
                                 const void *up, const void *down, const uint16_t *X, const int32_t *idx, const float *w,
                                 float *out, int n_tok, int top_k, int n_embd, int n_ff, int n_expert, int device,
                                 int n_cu, hipStream_t stream);

/* MoE pieces */
hipError_t launch_moe_route(const float *logits, int n_tok, int n_expert, int top_k, int32_t *idx,
                            float *w, hipStream_t stream);
hipError_t launch_silu_mul(float *h, const float *gate, const float *up, int n, hipStream_t stream);
/* result[0] = index (as int32 bits) of the first largest of v[0..n), result[1] = that value: the
 * loop `if (v[j] > v[best]) best = j` (server/server_llm.c:224-228). result holds
 * QLIN_ARGMAX_RESULT_BYTES bytes: the rest is scratch for the first stage. */
hipError_t launch_argmax(const float *v, int n, float *result, hipStream_t stream);
/* measurement probes (probe.hip): a register-only MFMA loop (flops issued come back in *flops) with the
 * cycle and 100 MHz counters around it, and a streaming read of a device buffer */
hipError_t launch_probe_mfma(int iters, int n_cu, hipStream_t stream, double *flops);
hipError_t launch_probe_read(const void *buf, size_t n_bytes, hipStream_t stream);
hipError_t read_probe_clocks(uint64_t out[2]);
hipError_t launch_axpy_dev_weight(float *out, const float *q, const float *w, int widx, int n,
                                  int overwrite, hipStream_t stream);

}  // namespace qlin
#endif
