"""GPU parity of the matvec on rows that the tuned kernels cannot take whole: rows of more than 16384 elements
or 8 KB (run as column ranges, one launch each, the later ones adding to y) and rows whose byte count is not a
multiple of 16 (every row then starts at a different offset inside a 16-byte piece). Every format, through the
C ABI, against the CPU oracle; relative L2 <= 1e-5. The row lengths are the FFN widths of common models."""
import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests.conftest import rel_l2

pytestmark = pytest.mark.gpu
NAMES = list(synth.TYPE_NAMES.items()) + list(synth.DENSE_TYPES.items())
TOL = 1e-5


# 11008 = 43 x 256 and 13824 = 54 x 256 (rows of 210-, 110-, 84-, 66-byte blocks end off a 16-byte boundary),
# 14336 (Q6_K, Q5_K, Q8_0 rows above 8 KB), 18944 and 28672 (above 16384 elements)
@pytest.mark.parametrize("n_rows,n_cols", [(37, 11008), (16, 13824), (21, 14336), (9, 18944), (18, 28672)])
@pytest.mark.parametrize("tid,name", NAMES)
def test_matvec(oracle, tid, name, n_rows, n_cols):
    W = synth.make_weights(tid, n_rows, n_cols, seed=n_rows + tid)
    x = synth.make_activation(n_cols, seed=n_cols + tid)
    dW, dx, dy = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(x), qlinear.DevBuf(n_rows * 4)
    qlinear.gemv_dev(tid, dW, dx, dy, n_rows, n_cols)
    qlinear.sync()
    got = dy.to_numpy(np.float32, (n_rows,))
    want = oracle.gemv_f64(tid, W, x, n_cols)
    assert rel_l2(got, want) <= TOL, (name, n_rows, n_cols, rel_l2(got, want))
    assert np.allclose(got, want, rtol=3e-4, atol=3e-6 * np.abs(want).max()), (name, n_rows, n_cols)


@pytest.mark.parametrize("tid,name", NAMES)
def test_residual_add_and_several_matrices(oracle, tid, name):
    """the ranges after the first add to y: a residual already there must survive, twice over; three matrices
    of different row counts share the launches"""
    n_cols, rows = 18944, (19, 5, 16)
    Ws = [synth.make_weights(tid, r, n_cols, seed=41 + i + tid) for i, r in enumerate(rows)]
    x = synth.make_activation(n_cols, seed=44)
    res = synth.make_activation(rows[0], seed=45)
    dW, dx, dy = qlinear.DevBuf.from_numpy(Ws[0]), qlinear.DevBuf.from_numpy(x), qlinear.DevBuf.from_numpy(res)
    qlinear.gemv_add_dev(tid, dW, dx, dy, rows[0], n_cols)
    qlinear.gemv_add_dev(tid, dW, dx, dy, rows[0], n_cols)
    qlinear.sync()
    want = res.astype(np.float64) + 2.0 * oracle.gemv_f64(tid, Ws[0], x, n_cols)
    assert rel_l2(dy.to_numpy(np.float32, (rows[0],)), want) <= TOL, name
    dWs = [qlinear.DevBuf.from_numpy(W) for W in Ws]
    dys = [qlinear.DevBuf.from_numpy(np.full(r, 7.0, np.float32)) for r in rows]
    qlinear.gemv_multi_dev(tid, dWs, dys, list(rows), dx, n_cols)
    qlinear.sync()
    for W, d, r in zip(Ws, dys, rows):
        assert rel_l2(d.to_numpy(np.float32, (r,)), oracle.gemv_f64(tid, W, x, n_cols)) <= TOL, name


# dense rows of 4097..16384 elements take one launch of their own kernel: the longest it takes (64 KB of x in LDS), the
# shortest, many rows per workgroup; then a residual add and three matrices in one launch
@pytest.mark.parametrize("n_rows,n_cols", [(130, 16384), (70, 4104), (5000, 8192), (3, 6000)])
@pytest.mark.parametrize("tid,name", list(synth.DENSE_TYPES.items()))
def test_dense_long_rows(oracle, tid, name, n_rows, n_cols):
    W = synth.make_weights(tid, n_rows, n_cols, seed=n_rows + tid)
    x = synth.make_activation(n_cols, seed=n_cols + tid)
    res = synth.make_activation(n_rows, seed=3)
    dW, dx, dy = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(x), qlinear.DevBuf.from_numpy(res)
    qlinear.gemv_add_dev(tid, dW, dx, dy, n_rows, n_cols)
    qlinear.sync()
    rows = np.arange(n_rows) if n_rows <= 400 else np.r_[0:50, n_rows - 50:n_rows]
    want = res[rows].astype(np.float64) + oracle.gemv_f64(tid, np.ascontiguousarray(W[rows]), x, n_cols)
    assert rel_l2(dy.to_numpy(np.float32, (n_rows,))[rows], want) <= TOL, (name, n_rows, n_cols)
    if n_rows == 130:
        parts = (60, 1, 69)
        dys = [qlinear.DevBuf(r * 4) for r in parts]
        offs = np.cumsum((0,) + parts)
        dWs = [qlinear.DevBuf.from_numpy(np.ascontiguousarray(W[offs[i]:offs[i + 1]])) for i in range(3)]
        qlinear.gemv_multi_dev(tid, dWs, dys, list(parts), dx, n_cols)
        qlinear.sync()
        got = np.concatenate([d.to_numpy(np.float32, (r,)) for d, r in zip(dys, parts)])
        assert rel_l2(got, oracle.gemv_f64(tid, W, x, n_cols)) <= TOL, name


@pytest.mark.parametrize("tid", [synth.GGML_Q6_K, synth.GGML_Q3_K, synth.GGML_IQ2_XXS, synth.GGML_Q8_0])
def test_gate_up_silu_on_rows_off_the_16_byte_grid(oracle, tid):
    n_rows, n_cols = 45, 11008
    Wg = synth.make_weights(tid, n_rows, n_cols, seed=11)
    Wu = synth.make_weights(tid, n_rows, n_cols, seed=12)
    x = synth.make_activation(n_cols, seed=13) * np.float32(0.02)
    got = qlinear.matvec_silu_mul(tid, Wg, tid, Wu, x, n_cols)
    g, u = oracle.gemv_f64(tid, Wg, x, n_cols), oracle.gemv_f64(tid, Wu, x, n_cols)
    assert rel_l2(got, g / (1.0 + np.exp(-g)) * u) <= TOL


@pytest.mark.parametrize("tid", [synth.GGML_Q6_K, synth.GGML_Q4_K, synth.GGML_IQ4_XS])
def test_full_size_down_projection(oracle, tid):
    """4096 x 14336 and 3584 x 18944 on the device, sampled rows against the oracle, repeatable bits"""
    for n_rows, n_cols in ((4096, 14336), (3584, 18944)):
        W = synth.make_weights(tid, n_rows, n_cols, seed=5)
        x = synth.make_activation(n_cols, seed=6)
        dW, dx, dy = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(x), qlinear.DevBuf(n_rows * 4)
        outs = []
        for _ in range(2):
            qlinear.gemv_dev(tid, dW, dx, dy, n_rows, n_cols)
            qlinear.sync()
            outs.append(dy.to_numpy(np.float32, (n_rows,)).copy())
        assert np.array_equal(outs[0], outs[1])
        rows = np.r_[0:24, n_rows // 2:n_rows // 2 + 24, n_rows - 24:n_rows]
        assert rel_l2(outs[0][rows], oracle.gemv_f64(tid, W[rows], x, n_cols)) <= TOL
        for b in (dW, dx, dy):
            b.free()
