/*
 * qlinear_bench.h - measurement probes of libqlinear.so. Not part of the engine's interface: bench.py uses
 * them to print what the GPU at hand sustains beside every measured rate.
 */
#ifndef QLINEAR_BENCH_H
#define QLINEAR_BENCH_H

#include <stddef.h>

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

#ifdef __cplusplus
}
#endif
#endif /* QLINEAR_BENCH_H */
