"""Edge cases of the matvec kernels that a standard-normal x never reaches, through the C ABI:
outliers (the integer-dot kernels share one exponent per 32 elements of x), all-zero and denormal
chunks, |x| near the ends of the fp32 range, non-finite x, and concurrent callers."""
import threading

import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests.conftest import rel_l2

pytestmark = pytest.mark.gpu
NAMES = list(synth.TYPE_NAMES.items()) + list(synth.DENSE_TYPES.items())
TOL = 1e-5
# formats whose matvec runs on integer dot products with x in per-32-element fixed point
FIXED_POINT = {synth.GGML_Q4_K, synth.GGML_Q8_0, synth.GGML_Q4_0, synth.GGML_Q4_1, synth.GGML_Q5_0, synth.GGML_Q5_1,
               synth.GGML_Q5_K, synth.GGML_Q6_K, synth.GGML_Q2_K, synth.GGML_Q3_K, synth.GGML_IQ4_NL, synth.GGML_IQ4_XS,
               synth.GGML_MXFP4, synth.GGML_IQ2_XXS, synth.GGML_IQ3_XXS, synth.GGML_IQ3_S, synth.GGML_IQ2_XS, synth.GGML_IQ2_S,
               synth.GGML_NVFP4, synth.GGML_TQ1_0, synth.GGML_TQ2_0, synth.GGML_Q1_0, synth.GGML_IQ1_S, synth.GGML_IQ1_M}


def x_step(tid):
    """largest error of one element of x in units of the largest |x| of its 32-element chunk: the Q4_K kernel
    keeps 31-bit fixed point per chunk, the other integer-dot formats 23-bit, the float kernels use x as it is"""
    if tid == synth.GGML_Q4_K:
        return 2.0 ** -30
    return 2.0 ** -22 if tid in FIXED_POINT else 0.0


def check(oracle, tid, name, W, x, n_cols, what, fp32_factor):
    """relative L2 <= 1e-5 over the outputs, and every single output within
    fp32_factor * sum|w||x| (rounding of an fp32 dot product: at most K * 2^-24 of that sum in any order)
    + x_step * sum over chunks of max|x| * sum|w| (the fixed-point form of x, exact integer sums after it)"""
    y = qlinear.matvec(tid, W, x, n_cols)
    want = oracle.gemv_f64(tid, W, x, n_cols)
    assert rel_l2(y, want) <= TOL, (name, what, rel_l2(y, want))
    dec = np.abs(oracle.dequant_matrix(tid, W, n_cols)).astype(np.float64)
    ax = np.abs(x).astype(np.float64)
    bound = fp32_factor * (dec @ ax)
    bound += x_step(tid) * (dec.reshape(dec.shape[0], -1, 32).sum(axis=2) @ ax.reshape(-1, 32).max(axis=1))
    worst = np.max(np.abs(y.astype(np.float64) - want) / (bound + 1e-300))
    assert worst <= 1.0, (name, what, worst)


@pytest.mark.parametrize("tid,name", NAMES)
@pytest.mark.parametrize("n_rows,n_cols", [(64, 4096), (48, 14336)])
def test_outliers_in_x(oracle, tid, name, n_rows, n_cols):
    """a few activations 10^3..10^5 times the bulk, inside a chunk and on both sides of a chunk border"""
    W = synth.make_weights(tid, n_rows, n_cols, seed=1000 + tid)
    x = synth.make_activation(n_cols, seed=1001 + tid)
    x[5] *= 1e3
    x[300] = 1e4
    x[1023] = -1e5
    x[1024] = 3e4
    x[n_cols - 1] = -2e3
    check(oracle, tid, name, W, x, n_cols, "outliers", 1e-4)
    # one huge value only: everything else in its chunk must still count
    x = synth.make_activation(n_cols, seed=1002 + tid)
    x[777] = 1e5
    check(oracle, tid, name, W, x, n_cols, "single outlier", 1e-4)


@pytest.mark.parametrize("tid,name", NAMES)
def test_zero_and_denormal_chunks(oracle, tid, name):
    n_rows, n_cols = 64, 4096
    W = synth.make_weights(tid, n_rows, n_cols, seed=1100 + tid)
    x = synth.make_activation(n_cols, seed=1101 + tid)
    x[64:128] = 0.0
    x[256:512] = 0.0
    x[512:544] *= np.float32(1e-40)  # fp32 denormals
    x[1000:1032] = np.float32(1e-44)
    check(oracle, tid, name, W, x, n_cols, "zero and denormal chunks", 1e-6)
    y = qlinear.matvec(tid, W, np.zeros(n_cols, np.float32), n_cols)
    assert np.all(y == 0.0), name


@pytest.mark.parametrize("tid,name", NAMES)
@pytest.mark.parametrize("scale", [1e30, 1e-30])
def test_x_near_the_ends_of_the_fp32_range(oracle, tid, name, scale):
    n_rows, n_cols = 64, 4096
    W = synth.make_weights(tid, n_rows, n_cols, seed=1200 + tid)
    x = (synth.make_activation(n_cols, seed=1201 + tid).astype(np.float64) * scale).astype(np.float32)
    y = qlinear.matvec(tid, W, x, n_cols)
    want = oracle.gemv_f64(tid, W, x, n_cols)
    assert np.all(np.isfinite(y)), name
    assert rel_l2(y, want) <= TOL, (name, scale, rel_l2(y, want))


@pytest.mark.parametrize("tid,name", NAMES)
def test_non_finite_x(oracle, tid, name):
    """The reference's fp32 loop gives +-Inf where every product with the infinite element has one sign and
    NaN otherwise. Here no row that sees the infinity is finite either, and an infinite output has the
    reference's sign, but more rows are NaN: the fixed-point kernels cannot carry an infinity and return NaN
    for EVERY row, and the float kernels of the formats with a constant offset per block multiply that
    offset with a sum of x that is itself infinite. A NaN in x gives NaN in every row that sees it."""
    n_rows, n_cols = 32, 4096
    W = synth.make_weights(tid, n_rows, n_cols, seed=1300 + tid)
    dec = oracle.dequant_matrix(tid, W, n_cols)
    x = synth.make_activation(n_cols, seed=1301 + tid)
    x[100] = np.inf
    y = qlinear.matvec(tid, W, x, n_cols)
    hit = dec[:, 100] != 0  # rows that see the infinity at all
    assert not np.any(np.isfinite(y[hit])), name
    if tid in FIXED_POINT:
        assert np.all(np.isnan(y)), name
    else:
        with np.errstate(invalid="ignore", over="ignore"):
            want = (dec.astype(np.float64) * x.astype(np.float64)[None, :]).sum(axis=1)
        inf = np.isinf(y)
        assert np.array_equal(y[inf], want[inf].astype(np.float32)), name
    x[100] = np.nan
    y = qlinear.matvec(tid, W, x, n_cols)
    assert np.all(np.isnan(y[hit])), name


def test_concurrent_host_threads(oracle):
    """tf_thread_matvec's calling pattern (common/transformer.h:3252-3269): several host threads inside the
    library at once, each with its own tensors; results equal the serial ones bit for bit"""
    lib = qlinear.load()
    jobs = []
    for k, (tid, n_rows, n_cols) in enumerate([(synth.GGML_Q4_K, 512, 4096), (synth.GGML_Q6_K, 300, 2048),
                                               (synth.GGML_Q8_0, 257, 4096), (synth.GGML_IQ2_XXS, 128, 4096)]):
        W = synth.make_weights(tid, n_rows, n_cols, seed=1400 + k)
        x = synth.make_activation(n_cols, seed=1410 + k)
        jobs.append((tid, n_rows, n_cols, W, x, qlinear.matvec(tid, W, x, n_cols)))
    assert lib.qlin_weight_register(jobs[0][3].ctypes.data, jobs[0][3].nbytes) == 0  # one job on a device copy
    errors = []

    def worker(job, dev):
        tid, n_rows, n_cols, W, x, serial = job
        y = np.zeros(n_rows, np.float32)
        dW = dx = dy = None
        if dev:
            dW, dx, dy = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(x), qlinear.DevBuf(n_rows * 4)
        for it in range(200):
            if dev and it % 2:
                qlinear.gemv_dev(tid, dW, dx, dy, n_rows, n_cols)
                qlinear.sync()
                got = dy.to_numpy(np.float32, (n_rows,))
            else:
                rc = lib.qlin_matvec(y.ctypes.data, W.ctypes.data, tid, n_cols, x.ctypes.data, n_rows)
                if rc != 0:
                    errors.append((tid, it, "rc %d" % rc))
                    return
                got = y
            if not np.array_equal(got, serial):
                errors.append((tid, it, "differs from the serial result"))
                return

    threads = [threading.Thread(target=worker, args=(job, k % 2 == 1)) for k, job in enumerate(jobs)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert lib.qlin_weight_unregister(jobs[0][3].ctypes.data) == 0
    assert not errors, errors
    for tid, n_rows, n_cols, W, x, serial in jobs:
        assert rel_l2(serial, oracle.gemv_f64(tid, W, x, n_cols)) <= TOL


@pytest.mark.parametrize("tid,name", list(synth.DENSE_TYPES.items()))
@pytest.mark.parametrize("n_cols", [1, 7, 1001, 4100])
def test_dense_rows_of_any_length(tid, name, n_cols):
    """tf_qmatvec dots F32/F16/BF16 rows element by element, whatever their length
    (common/transformer.h:1049-1114); so does the matvec here, on host and on device pointers, also when a
    matrix starts off a 16-byte boundary."""
    n_rows = 37
    W = synth.make_weights(tid, n_rows, n_cols, seed=900 + tid)
    x = synth.make_activation(n_cols, seed=901)
    if tid == synth.GGML_F32:
        dec = W.view(np.float32).reshape(n_rows, n_cols)
    elif tid == synth.GGML_F16:
        dec = W.view(np.float16).reshape(n_rows, n_cols).astype(np.float32)
    else:
        dec = synth.bf16_bits_to_f32(W.view(np.uint16).reshape(n_rows, n_cols))
    want = dec.astype(np.float64) @ x.astype(np.float64)
    got = qlinear.matvec(tid, W, x, n_cols)
    assert rel_l2(got, want) <= TOL, (name, n_cols, rel_l2(got, want))
    # device pointers, the matrix one element past a 16-byte boundary
    elem = 4 if tid == synth.GGML_F32 else 2
    raw = np.concatenate([np.zeros(elem, np.uint8), W.reshape(-1)])
    dW, dx, dy = qlinear.DevBuf.from_numpy(raw), qlinear.DevBuf.from_numpy(x), qlinear.DevBuf(n_rows * 4)
    lib = qlinear.load()
    assert lib.qlin_gemv_dev(tid, dW.ptr + elem, dx.ptr, dy.ptr, n_rows, n_cols, None) == 0
    qlinear.sync()
    got = dy.to_numpy(np.float32, (n_rows,))
    assert rel_l2(got, want) <= TOL, (name, n_cols, "offset", rel_l2(got, want))
    for b in (dW, dx, dy):
        b.free()
