/*
 * qlinear_bench.h - measurement probes of libqlinear.so. Not part of the engine's interface: bench.py uses
 * them to print what the GPU at hand sustains beside every measured rate.
 */
#ifndef QLINEAR_BENCH_H
#define QLINEAR_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* What this GPU sustains on the two resources the kernels are priced against (the
 * reference prints a peak beside every measured rate, rdna4/dequant/bench_dequant.c:1043-1110). All three
 * only enqueue; time them with qlin_timer_begin/end.
 *   qlin_probe_mfma_bf16: register-only loop of the prefill GEMM's matrix instruction on every compute
 *     unit, `iters` x 4 instructions per wave; *flops receives the flops of the launch.
 *   qlin_probe_clocks: waits for the stream, then returns the shader clock (MHz) that the last
 *     qlin_probe_mfma_bf16 launch ran at (cycle counter against the 100 MHz counter).
 *   qlin_probe_hbm_read: streaming read of n_bytes (16-byte aligned) of device memory. */
int qlin_probe_mfma_bf16(int iters, void *stream, double *flops);
int qlin_probe_clocks(void *stream, double *shader_mhz);
int qlin_probe_hbm_read(const void *buf, size_t n_bytes, void *stream);

/* One tile kernel of the fused prefill GEMM by name, whatever the shape-based choice of qlin_gemm_bf16_any_dev would be:
 * tile 0 = 256 tokens x 128 rows, 1 = 128 tokens x 64 rows. Arguments and result as qlin_gemm_bf16_any_dev without a
 * workspace; Q4_K, Q5_K, Q6_K, Q8_0, IQ4_NL, IQ4_XS, Q4_0; n_cols % 256 == 0. For timing one against the other and for the parity tests of
 * each on small shapes. */
/* which of them qlin_gemm_bf16_any_dev picks for a shape above the few-token kernels' token counts: 1 = the 256 x 128
 * tile kernel, 2 = the 128 x 64 one, 0 = neither (decode to bf16 + dense product) */
int qlin_probe_gemm_route(uint32_t ggml_type, int n_rows, int n_cols, int n_tok, int ldx, int have_workspace);
int qlin_probe_gemm_tile(int tile, uint32_t ggml_type, const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols,
                         int n_tok, int ldx, int ldy, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* QLINEAR_BENCH_H */
