"""GPU parity of the matrix-instruction matvec for the codebook formats IQ1_S, IQ1_M, IQ2_XXS, IQ2_XS, IQ2_S, IQ3_XXS, IQ3_S and for Q6_K, Q5_K,
Q8_0, Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, IQ4_XS, MXFP4, NVFP4, TQ1_0, TQ2_0, Q1_0, Q2_K, Q3_K (rows longer than 4096 elements take it, and most of these formats' rows from 2048 elements) against the CPU oracle, through the C ABI: plain, ragged row counts, several
matrices in one launch, gate+up+SiLU, projection+residual, non-finite x. Relative L2 <= 1e-5."""
import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests.conftest import rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-5
GRID = {synth.GGML_IQ2_XXS: "iq2_xxs", synth.GGML_IQ3_XXS: "iq3_xxs", synth.GGML_IQ3_S: "iq3_s",
        synth.GGML_Q6_K: "q6_K", synth.GGML_Q5_K: "q5_K", synth.GGML_Q8_0: "q8_0", synth.GGML_IQ4_NL: "iq4_nl",
        synth.GGML_IQ4_XS: "iq4_xs", synth.GGML_Q4_0: "q4_0", synth.GGML_Q2_K: "q2_K", synth.GGML_Q3_K: "q3_K",
        synth.GGML_Q4_1: "q4_1", synth.GGML_Q5_0: "q5_0", synth.GGML_Q5_1: "q5_1", synth.GGML_MXFP4: "mxfp4", synth.GGML_NVFP4: "nvfp4", synth.GGML_TQ2_0: "tq2_0",
        synth.GGML_IQ2_XS: "iq2_xs", synth.GGML_IQ2_S: "iq2_s", synth.GGML_Q1_0: "q1_0", synth.GGML_IQ1_S: "iq1_s", synth.GGML_IQ1_M: "iq1_m", synth.GGML_TQ1_0: "tq1_0"}


# 17 super-blocks (one wave with two), 43 (ragged over the 16 waves), 56 and 64 (the most a wave takes);
# one row, a ragged last row group, several row groups per workgroup, more rows than compute units x 16; rows of
# 2048 to 4096 elements (one super-block or none per wave): 56 rows per workgroup, ragged row counts, many row groups
@pytest.mark.parametrize("n_rows,n_cols", [(1, 4352), (16, 4352), (37, 11008), (300, 8192), (4096, 14336), (130, 16384),
                                           (5000, 4608), (14336, 4096), (4113, 2048), (9, 4096), (40001, 3072)])
@pytest.mark.parametrize("tid", sorted(GRID), ids=lambda t: GRID[t])
def test_matvec(oracle, tid, n_rows, n_cols):
    W = synth.make_weights(tid, n_rows, n_cols, seed=n_rows + tid)
    x = synth.make_activation(n_cols, seed=n_cols + tid)
    dW, dx, dy = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(x), qlinear.DevBuf(n_rows * 4)
    qlinear.gemv_dev(tid, dW, dx, dy, n_rows, n_cols)
    qlinear.sync()
    got = dy.to_numpy(np.float32, (n_rows,))
    rows = np.arange(n_rows) if n_rows <= 400 else np.r_[0:60, n_rows // 2:n_rows // 2 + 60, n_rows - 60:n_rows]
    want = oracle.gemv_f64(tid, W[rows], x, n_cols)
    if n_rows >= 16:
        assert rel_l2(got[rows], want) <= TOL
    assert np.allclose(got[rows], want, rtol=2e-4, atol=2e-6 * np.abs(want).max())


@pytest.mark.parametrize("tid", sorted(GRID), ids=lambda t: GRID[t])
def test_outlier_and_tiny_activations(oracle, tid):
    """an element 1e5 times its neighbours, a group of zeros and a group of denormal-sized values"""
    n_rows, n_cols = 48, 8192
    W = synth.make_weights(tid, n_rows, n_cols, seed=7)
    x = synth.make_activation(n_cols, seed=8)
    x[1000] = 1.0e5
    x[2048:2080] = 0.0
    x[4096:4128] = 1.0e-39
    dW, dx, dy = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(x), qlinear.DevBuf(n_rows * 4)
    qlinear.gemv_dev(tid, dW, dx, dy, n_rows, n_cols)
    qlinear.sync()
    assert rel_l2(dy.to_numpy(np.float32, (n_rows,)), oracle.gemv_f64(tid, W, x, n_cols)) <= TOL


@pytest.mark.parametrize("n_rows,n_cols", [(203, 8192), (203, 4096), (9000, 2048)])
@pytest.mark.parametrize("tid", sorted(GRID), ids=lambda t: GRID[t])
def test_gate_up_silu(oracle, tid, n_rows, n_cols):
    Wg = synth.make_weights(tid, n_rows, n_cols, seed=11)
    Wu = synth.make_weights(tid, n_rows, n_cols, seed=12)
    x = synth.make_activation(n_cols, seed=13) * np.float32(0.02)
    got = qlinear.matvec_silu_mul(tid, Wg, tid, Wu, x, n_cols)
    g, u = oracle.gemv_f64(tid, Wg, x, n_cols), oracle.gemv_f64(tid, Wu, x, n_cols)
    with np.errstate(over="ignore"):  # exp(-g) of a very negative g is inf, the quotient 0: what SiLU gives
        want = g / (1.0 + np.exp(-g)) * u
    assert rel_l2(got, want) <= TOL


@pytest.mark.parametrize("tid", sorted(GRID), ids=lambda t: GRID[t])
def test_projection_plus_residual_twice(oracle, tid):
    n_rows, n_cols = 77, 14336
    W = synth.make_weights(tid, n_rows, n_cols, seed=31)
    x = synth.make_activation(n_cols, seed=32)
    res = synth.make_activation(n_rows, seed=33)
    dW, dx, dy = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(x), qlinear.DevBuf.from_numpy(res)
    qlinear.gemv_add_dev(tid, dW, dx, dy, n_rows, n_cols)
    qlinear.gemv_add_dev(tid, dW, dx, dy, n_rows, n_cols)
    qlinear.sync()
    want = res.astype(np.float64) + 2.0 * oracle.gemv_f64(tid, W, x, n_cols)
    assert rel_l2(dy.to_numpy(np.float32, (n_rows,)), want) <= TOL


# row counts that put the matrices' borders inside a row group and inside a workgroup
@pytest.mark.parametrize("rows,n_cols", [((40, 9, 9), 5120), ((16, 16, 0), 5120), ((300, 7, 100), 5120),
                                         ((4096, 1024, 1024), 4096), ((5000, 3, 700), 3072)])
@pytest.mark.parametrize("tid", sorted(GRID), ids=lambda t: GRID[t])
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


@pytest.mark.parametrize("bad", [np.nan, np.inf, -np.inf])
@pytest.mark.parametrize("tid", sorted(GRID), ids=lambda t: GRID[t])
def test_non_finite_x_poisons_every_row(tid, bad):
    n_rows, n_cols = 33, 8192
    W = synth.make_weights(tid, n_rows, n_cols, seed=3)
    x = synth.make_activation(n_cols, seed=4)
    x[5000] = bad
    y = qlinear.matvec(tid, W, x, n_cols)
    assert np.all(np.isnan(y))


@pytest.mark.parametrize("tid", sorted(GRID), ids=lambda t: GRID[t])
def test_repeatable_bits(tid):
    n_rows, n_cols = 512, 14336
    W = synth.make_weights(tid, n_rows, n_cols, seed=5)
    x = synth.make_activation(n_cols, seed=6)
    dW, dx, dy = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(x), qlinear.DevBuf(n_rows * 4)
    outs = []
    for _ in range(3):
        qlinear.gemv_dev(tid, dW, dx, dy, n_rows, n_cols)
        qlinear.sync()
        outs.append(dy.to_numpy(np.float32, (n_rows,)).copy())
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
