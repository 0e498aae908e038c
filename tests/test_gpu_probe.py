"""The measurement probes of the C ABI: a register-only loop of the prefill GEMM's matrix instruction and a
streaming read. They produce no result to check against the oracle; the tests pin what the benchmark
relies on: the flop count handed back, plausible rates and clock, and the argument checks."""
import ctypes as C

import pytest

from gemm_amd import qlinear

pytestmark = pytest.mark.gpu


def test_mfma_probe_reports_its_flops_and_a_plausible_rate():
    _, n_cu, _ = qlinear.device_info()
    iters = 4000
    qlinear.probe_mfma_bf16(200)
    qlinear.sync()
    qlinear.timer_begin()
    flops = qlinear.probe_mfma_bf16(iters)
    ms = qlinear.timer_end()
    # 4 workgroups x 4 waves per compute unit, 4 MFMAs of 32x32x16 per iteration
    assert flops == n_cu * 4 * 4 * iters * 4 * 2.0 * 32 * 32 * 16
    tflops = flops / (ms * 1e-3) / 1e12
    assert 200.0 < tflops < 2600.0, tflops       # below the published dense bf16 figure, far above the vector ALUs
    mhz = qlinear.probe_clocks()
    assert 500.0 < mhz < 3000.0, mhz


def test_read_probe_runs_and_checks_its_arguments():
    buf = qlinear.DevBuf(64 << 20)
    qlinear.probe_hbm_read(buf)
    qlinear.sync()
    qlinear.timer_begin()
    for _ in range(4):
        qlinear.probe_hbm_read(buf)
    ms = qlinear.timer_end() / 4
    gbps = buf.nbytes / (ms * 1e-3) / 1e9
    assert 500.0 < gbps < 20000.0, gbps          # 64 MiB may sit in the last-level cache: only a sanity band
    lib = qlinear.load()
    assert lib.qlin_probe_hbm_read(C.c_void_p(buf.ptr + 4), 1024, None) == qlinear.ERR_ARG
    assert lib.qlin_probe_hbm_read(None, 1024, None) == qlinear.ERR_ARG
    flops = C.c_double(0)
    assert lib.qlin_probe_mfma_bf16(0, None, C.byref(flops)) == qlinear.ERR_ARG
    assert lib.qlin_probe_mfma_bf16(10, None, None) == qlinear.ERR_ARG
    buf.free()
