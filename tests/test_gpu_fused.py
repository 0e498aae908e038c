"""GPU parity of the fused matvec call shapes (gate+up+SiLU, projection+residual, several matrices
in one launch, output projection + greedy pick) against the CPU oracle, through the C ABI.
Tolerance: relative L2 <= 1e-5 like every fp32 matvec path."""
import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests.conftest import rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-5
Q4K, Q6K, Q80, IQ2XS = synth.GGML_Q4_K, synth.GGML_Q6_K, synth.GGML_Q8_0, synth.GGML_IQ2_XS


def silu_mul64(g, u):
    g, u = g.astype(np.float64), u.astype(np.float64)
    return g / (1.0 + np.exp(-g)) * u


# (type of gate, type of up, rows, cols): tuned Q4_K kernel with 1, 2 and 4 row slices, the streaming
# kernel, the plain kernel (cols above the streaming limit), and two types (one launch per matrix)
SILU_CASES = [(Q4K, Q4K, 1, 256), (Q4K, Q4K, 13, 4096), (Q4K, Q4K, 257, 2048), (Q4K, Q4K, 700, 8192),
              (Q4K, Q4K, 96, 14336), (Q6K, Q6K, 300, 4096), (IQ2XS, IQ2XS, 65, 1024), (Q80, Q80, 33, 20480),
              (Q4K, Q6K, 48, 1024)]


@pytest.mark.parametrize("tg,tu,n_rows,n_cols", SILU_CASES)
def test_gate_up_silu_host(oracle, tg, tu, n_rows, n_cols):
    Wg = synth.make_weights(tg, n_rows, n_cols, seed=11 + n_rows)
    Wu = synth.make_weights(tu, n_rows, n_cols, seed=12 + n_rows)
    # activations scaled so that gate values spread over the curved part of SiLU
    x = synth.make_activation(n_cols, seed=13) * np.float32(0.05)
    got = qlinear.matvec_silu_mul(tg, Wg, tu, Wu, x, n_cols)
    want = silu_mul64(oracle.gemv_f64(tg, Wg, x, n_cols), oracle.gemv_f64(tu, Wu, x, n_cols))
    if n_rows >= 13:
        assert rel_l2(got, want) <= TOL
    assert np.allclose(got, want, rtol=2e-4, atol=1e-6 * np.abs(want).max())


def test_gate_up_silu_full_size_device_resident(oracle):
    """14336 x 4096 Q4_K (the decode FFN shape): one launch; sampled rows against the oracle"""
    n_rows, n_cols = 14336, 4096
    Wg = synth.make_weights(Q4K, n_rows, n_cols, seed=21)
    Wu = synth.make_weights(Q4K, n_rows, n_cols, seed=22)
    x = synth.make_activation(n_cols, seed=23) * np.float32(0.05)
    dg, du, dx = (qlinear.DevBuf.from_numpy(a) for a in (Wg, Wu, x))
    dout = qlinear.DevBuf(n_rows * 4)
    qlinear.gemv_silu_mul_dev(Q4K, dg, du, dx, dout, n_rows, n_cols)
    qlinear.sync()
    got = dout.to_numpy(np.float32, (n_rows,))
    rows = np.r_[0:40, 7000:7040, n_rows - 40:n_rows]
    want = silu_mul64(oracle.gemv_f64(Q4K, Wg[rows], x, n_cols), oracle.gemv_f64(Q4K, Wu[rows], x, n_cols))
    assert rel_l2(got[rows], want) <= TOL
    # the same numbers as two plain launches followed by the activation on the host
    dyg, dyu = qlinear.DevBuf(n_rows * 4), qlinear.DevBuf(n_rows * 4)
    qlinear.gemv_dev(Q4K, dg, dx, dyg, n_rows, n_cols)
    qlinear.gemv_dev(Q4K, du, dx, dyu, n_rows, n_cols)
    qlinear.sync()
    two = silu_mul64(dyg.to_numpy(np.float32, (n_rows,)), dyu.to_numpy(np.float32, (n_rows,)))
    assert rel_l2(got, two) <= 1e-6


@pytest.mark.parametrize("tid,n_rows,n_cols", [(Q4K, 4096, 14336), (Q4K, 57, 512), (Q6K, 130, 4096),
                                               (IQ2XS, 9, 768), (Q80, 21, 20480)])
def test_projection_plus_residual(oracle, tid, n_rows, n_cols):
    W = synth.make_weights(tid, n_rows, n_cols, seed=31)
    x = synth.make_activation(n_cols, seed=32)
    res = synth.make_activation(n_rows, seed=33)
    got = qlinear.matvec_add(tid, W, x, n_cols, res)
    want = res.astype(np.float64) + oracle.gemv_f64(tid, W, x, n_cols)
    assert rel_l2(got, want) <= TOL
    # device-resident form, applied twice: y + 2 W.x
    dW, dx, dy = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(x), qlinear.DevBuf.from_numpy(res)
    qlinear.gemv_add_dev(tid, dW, dx, dy, n_rows, n_cols)
    qlinear.gemv_add_dev(tid, dW, dx, dy, n_rows, n_cols)
    qlinear.sync()
    want2 = res.astype(np.float64) + 2.0 * oracle.gemv_f64(tid, W, x, n_cols)
    assert rel_l2(dy.to_numpy(np.float32, (n_rows,)), want2) <= TOL


@pytest.mark.parametrize("tid,rows,n_cols", [(Q4K, (4096, 1024, 1024), 4096), (Q4K, (33, 7, 7), 8192),
                                             (Q6K, (64, 16, 16), 2048), (Q80, (5, 0, 3), 512),
                                             (IQ2XS, (10, 11, 0), 20480), (Q4K, (300, 300), 14336)])
def test_several_matrices_one_launch(oracle, tid, rows, n_cols):
    Ws = [synth.make_weights(tid, max(r, 1), n_cols, seed=41 + i) for i, r in enumerate(rows)]
    x = synth.make_activation(n_cols, seed=44)
    dWs = [qlinear.DevBuf.from_numpy(W) for W in Ws]
    dys = [qlinear.DevBuf(max(r, 1) * 4) for r in rows]
    dx = qlinear.DevBuf.from_numpy(x)
    qlinear.gemv_multi_dev(tid, dWs, dys, list(rows), dx, n_cols)
    qlinear.sync()
    for W, dy, r in zip(Ws, dys, rows):
        if r:
            assert rel_l2(dy.to_numpy(np.float32, (r,)), oracle.gemv_f64(tid, W[:r], x, n_cols)) <= TOL


def test_qkv_same_type_host(oracle):
    n_cols, n_q, n_kv = 2048, 512, 128
    lib = qlinear.load()
    Wq, Wk, Wv = (synth.make_weights(Q4K, r, n_cols, seed=50 + i) for i, r in enumerate((n_q, n_kv, n_kv)))
    x = synth.make_activation(n_cols, seed=53)
    q, k, v = np.zeros(n_q, np.float32), np.zeros(n_kv, np.float32), np.zeros(n_kv, np.float32)
    assert lib.qlin_matvec_qkv(q.ctypes.data, Wq.ctypes.data, Q4K, n_q, k.ctypes.data, Wk.ctypes.data, Q4K,
                               v.ctypes.data, Wv.ctypes.data, Q4K, n_kv, n_cols, x.ctypes.data) == 0
    for got, W in ((q, Wq), (k, Wk), (v, Wv)):
        assert rel_l2(got, oracle.gemv_f64(Q4K, W, x, n_cols)) <= TOL


@pytest.mark.parametrize("tid,n_rows,n_cols", [(Q6K, 5000, 1024), (Q4K, 3001, 2048), (Q80, 17, 256)])
def test_output_projection_and_greedy_pick(oracle, tid, n_rows, n_cols):
    W = synth.make_weights(tid, n_rows, n_cols, seed=61)
    x = synth.make_activation(n_cols, seed=62)
    idx, val, logits = qlinear.matvec_argmax(tid, W, x, n_cols, want_logits=True)
    assert rel_l2(logits, oracle.gemv_f64(tid, W, x, n_cols)) <= TOL
    assert idx == int(np.argmax(logits)) and val == logits[idx]  # numpy's argmax is the first largest too
    idx2, val2, none = qlinear.matvec_argmax(tid, W, x, n_cols)
    assert (idx2, val2, none) == (idx, val, None)
    # every row twice: the largest logit appears twice, the first occurrence wins
    idx3, _, _ = qlinear.matvec_argmax(tid, np.concatenate([W, W]), x, n_cols)
    assert idx3 == idx
    # a NaN in x makes every logit NaN: nothing is greater than element 0
    xn = x.copy()
    xn[3] = np.nan
    assert qlinear.matvec_argmax(tid, W, xn, n_cols)[0] == 0


def test_greedy_pick_skips_nan_and_keeps_first():
    """hand-made logits: Q8_0 rows [q_r, 0, ...] with d = 1 against x = e_0 give logit_r = q_r exactly;
    a NaN scale gives a NaN logit. NaNs after index 0 never win, ties go to the lowest index."""
    lib = qlinear.load()
    n = 5000
    rng = np.random.default_rng(5)
    q = rng.integers(-127, 101, n).astype(np.int8)
    q[[77, 1234, 4999]] = 127
    W = np.zeros((n, 34), np.uint8)
    W[:, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    W[:, 2] = q.view(np.uint8)
    W[[10, 4000], 0:2] = np.frombuffer(np.uint16(0x7E00).tobytes(), np.uint8)  # NaN scale
    x = np.zeros(32, np.float32)
    x[0] = 1.0
    idx, val, logits = qlinear.matvec_argmax(Q80, W, x, 32, want_logits=True)
    assert np.isnan(logits[10]) and np.isnan(logits[4000])
    assert (idx, val) == (77, 127.0)
    # NaN at index 0: the sequential loop never moves off it
    W[0, 0:2] = np.frombuffer(np.uint16(0x7E00).tobytes(), np.uint8)
    assert qlinear.matvec_argmax(Q80, W, x, 32)[0] == 0
    # device-resident form
    dW, dx = qlinear.DevBuf.from_numpy(W[1:]), qlinear.DevBuf.from_numpy(x)
    dl, dr = qlinear.DevBuf((n - 1) * 4), qlinear.DevBuf(qlinear.ARGMAX_RESULT_BYTES)
    qlinear.gemv_argmax_dev(Q80, dW, dx, dl, dr, n - 1, 32)
    qlinear.sync()
    assert dr.to_numpy(np.int32, (2,))[0] == 76 and dr.to_numpy(np.float32, (2,))[1] == 127.0
    assert lib.qlin_matvec_argmax(None, None, None, W.ctypes.data, Q80, 32, x.ctypes.data, n) == qlinear.ERR_ARG


@pytest.mark.parametrize("offset_floats", [0, 1])
@pytest.mark.parametrize("n", [1, 5, 1023, 1024, 1025, 151936])
def test_greedy_pick_sizes_and_logit_alignment(n, offset_floats):
    """the pick reads the logits four at a time when their address allows it and one at a time otherwise;
    slices of the vector end inside a group of four for most n"""
    lib = qlinear.load()
    rng = np.random.default_rng(n)
    q = rng.integers(-127, 120, n).astype(np.int8)
    hot = sorted({n - 1, n // 2, (n * 3) // 4})
    q[hot] = 127  # ties: the first of them wins
    W = np.zeros((n, 34), np.uint8)
    W[:, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    W[:, 2] = q.view(np.uint8)
    x = np.zeros(32, np.float32)
    x[0] = 1.0
    dW, dx = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(x)
    dl, dr = qlinear.DevBuf((n + 4) * 4), qlinear.DevBuf(qlinear.ARGMAX_RESULT_BYTES)
    assert lib.qlin_gemv_argmax_dev(Q80, dW.ptr, dx.ptr, dl.ptr + 4 * offset_floats, dr.ptr, n, 32, None) == 0
    qlinear.sync()
    assert dr.to_numpy(np.int32, (2,))[0] == hot[0] and dr.to_numpy(np.float32, (2,))[1] == 127.0
    for b in (dW, dx, dl, dr):
        b.free()


def test_fused_errors():
    lib = qlinear.load()
    W = synth.make_weights(Q4K, 4, 512, seed=1)
    x = synth.make_activation(512, seed=2)
    y = np.zeros(4, np.float32)
    assert lib.qlin_matvec_silu_mul(y.ctypes.data, W.ctypes.data, Q4K, W.ctypes.data, 99, 512, x.ctypes.data, 4) == qlinear.ERR_TYPE
    assert lib.qlin_matvec_silu_mul(y.ctypes.data, W.ctypes.data, Q4K, None, Q4K, 512, x.ctypes.data, 4) == qlinear.ERR_ARG
    assert lib.qlin_matvec_add(y.ctypes.data, W.ctypes.data, Q4K, 500, x.ctypes.data, 4) == qlinear.ERR_ARG
    assert lib.qlin_matvec_add(y.ctypes.data, W.ctypes.data, Q4K, 512, x.ctypes.data, 0) == 0
    assert lib.qlin_gemv_multi_dev(Q4K, 4, None, None, None, None, 512, None) == qlinear.ERR_ARG
