"""GPU parity of the exact prefill GEMM for every weight format (decode once to fp32, bit-exact, then the
vendor library's dense fp32 GEMM with fp32 accumulation), through the C ABI: what
tf_gemm_f16_mt_tokenmajor (common/transformer.h:4487) computes for fp32 activations. Nothing is rounded
to 16 bits, so the bar is the matvec's: relative L2 <= 1e-5 against a double-precision contraction of the
oracle's decoded weights with the same activations."""
import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests.conftest import rel_l2

pytestmark = pytest.mark.gpu
ALL = dict(synth.TYPE_NAMES)
ALL.update(synth.DENSE_TYPES)
TOL = 1e-5


def run(tid, W, X, n_rows, n_cols, ldx=None, ldy=None, ws="own"):
    n_tok = X.shape[0]
    ldx, ldy = ldx or n_cols, ldy or n_rows
    Xpad = np.zeros((n_tok, ldx), np.float32)
    Xpad[:, :n_cols] = X
    dW, dX = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(Xpad)
    dY = qlinear.DevBuf.from_numpy(np.full((n_tok, ldy), -3.0, np.float32))
    dws = qlinear.DevBuf(qlinear.gemm_f32_any_workspace_bytes(n_rows, n_cols)) if ws == "own" else ws
    qlinear.gemm_f32_any_dev(tid, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy, dws)
    qlinear.sync()
    Y = dY.to_numpy(np.float32, (n_tok, ldy))
    for b in (dW, dX, dY) + ((dws,) if ws == "own" else ()):
        b.free()
    return Y


def reference(oracle, tid, W, X, n_cols):
    return X.astype(np.float64) @ oracle.dequant_matrix(tid, W, n_cols).astype(np.float64).T


@pytest.mark.parametrize("tid", sorted(ALL), ids=lambda t: ALL[t])
def test_every_format(oracle, tid):
    n_tok, n_rows, n_cols = 72, 160, 512
    W = synth.make_weights(tid, n_rows, n_cols, seed=300 + tid)
    X = synth.make_activation(n_cols, seed=400 + tid, tokens=n_tok)
    Y = run(tid, W, X, n_rows, n_cols)
    assert rel_l2(Y, reference(oracle, tid, W, X, n_cols)) <= TOL, ALL[tid]


@pytest.mark.parametrize("tid,n_tok,n_rows,n_cols", [
    (synth.GGML_Q4_K, 8, 16, 256), (synth.GGML_Q6_K, 515, 1000, 1024), (synth.GGML_Q8_0, 130, 257, 96),
    (synth.GGML_Q5_K, 64, 2048, 768), (synth.GGML_IQ4_NL, 200, 130, 4096), (synth.GGML_Q4_K, 1100, 300, 256),
    (synth.GGML_F32, 33, 100, 264), (synth.GGML_F16, 300, 64, 1000), (synth.GGML_Q4_K, 9, 1, 256),
])
def test_shapes(oracle, tid, n_tok, n_rows, n_cols):
    W = synth.make_weights(tid, n_rows, n_cols, seed=n_rows + n_tok)
    X = synth.make_activation(n_cols, seed=n_cols + n_tok, tokens=n_tok)
    Y = run(tid, W, X, n_rows, n_cols)
    assert rel_l2(Y, reference(oracle, tid, W, X, n_cols)) <= TOL, (ALL[tid], n_tok, n_rows, n_cols)


def test_one_hot_activations_return_the_codec_values_exactly(oracle):
    """a one-hot fp32 activation picks out single decoded weights; products with 1.0 and sums with 0.0 are
    exact, so the fp32 route must return the oracle's decoded values bit for bit"""
    tid, n_rows, n_cols = synth.GGML_Q6_K, 96, 512
    W = synth.make_weights(tid, n_rows, n_cols, seed=5)
    ks = [0, 1, 15, 16, 127, 128, 255, 256, 300, 511, 7, 8]
    X = np.zeros((len(ks), n_cols), np.float32)
    for i, k in enumerate(ks):
        X[i, k] = 1.0
    Y = run(tid, W, X, n_rows, n_cols)
    dec = oracle.dequant_matrix(tid, W, n_cols)
    assert np.array_equal(Y, dec[:, ks].T)


def test_few_tokens_need_no_workspace(oracle):
    tid, n_rows, n_cols = synth.GGML_Q5_K, 70, 512
    W = synth.make_weights(tid, n_rows, n_cols, seed=6)
    X = synth.make_activation(n_cols, seed=7, tokens=7)
    Y = run(tid, W, X, n_rows, n_cols, ws=None)
    assert rel_l2(Y, reference(oracle, tid, W, X, n_cols)) <= TOL


def test_strides_padding_and_workspace_reuse(oracle):
    n_rows, n_cols, n_tok = 200, 1024, 40
    ws = qlinear.DevBuf(qlinear.gemm_f32_any_workspace_bytes(n_rows, n_cols))
    for tid in (synth.GGML_Q6_K, synth.GGML_IQ3_S):
        W = synth.make_weights(tid, n_rows, n_cols, seed=3 + tid)
        X = synth.make_activation(n_cols, seed=4, tokens=n_tok)
        Y = run(tid, W, X, n_rows, n_cols, ldx=n_cols + 64, ldy=n_rows + 12, ws=ws)
        assert rel_l2(Y[:, :n_rows], reference(oracle, tid, W, X, n_cols)) <= TOL
        assert np.all(Y[:, n_rows:] == -3.0)
    ws.free()


@pytest.mark.parametrize("pad", [0, 12])
@pytest.mark.parametrize("n_tok,n_rows,n_cols", [(9, 300, 8192), (512, 300, 8192), (64, 4096, 16384)])
def test_padded_output_with_long_rows(oracle, n_tok, n_rows, n_cols, pad):
    """few output tiles and a long K: the library's kernels that split K and reduce through a workspace wrote
    a padded Y (ldy > n_rows) as if it were dense; the plan for such a call offers them no workspace
    (pad = 0: the same shapes with a dense Y, where those kernels are used)"""
    rng = np.random.default_rng(n_tok + n_cols)
    W = rng.standard_normal((n_rows, n_cols)).astype(np.float32)
    X = rng.standard_normal((n_tok, n_cols)).astype(np.float32)
    Y = run(synth.GGML_F32, W.view(np.uint8), X, n_rows, n_cols, ldx=n_cols + 64, ldy=n_rows + pad)
    assert rel_l2(Y[:, :n_rows], X.astype(np.float64) @ W.astype(np.float64).T) <= TOL
    assert np.all(Y[:, n_rows:] == -3.0)


def test_argument_checks():
    lib = qlinear.load()
    d = qlinear.DevBuf(1 << 20)
    Q6K = synth.GGML_Q6_K
    big = qlinear.gemm_f32_any_workspace_bytes(128, 256)
    assert big == 128 * 256 * 4 + (32 << 20)
    assert qlinear.gemm_f32_any_workspace_bytes(0, 256) == 0
    args = (128, 256, 16, 256, 128)
    assert lib.qlin_gemm_f32_any_dev(Q6K, d.ptr, d.ptr, d.ptr, *args, None, 0, None) == qlinear.ERR_ARG          # no workspace
    assert lib.qlin_gemm_f32_any_dev(Q6K, d.ptr, d.ptr, d.ptr, *args, d.ptr, 1 << 20, None) == qlinear.ERR_ARG  # too small
    assert lib.qlin_gemm_f32_any_dev(99, d.ptr, d.ptr, d.ptr, *args, d.ptr, big, None) == qlinear.ERR_TYPE
    assert lib.qlin_gemm_f32_any_dev(Q6K, d.ptr, d.ptr, d.ptr, 128, 300, 16, 300, 128, d.ptr, big, None) == qlinear.ERR_ARG
    assert lib.qlin_gemm_f32_any_dev(Q6K, d.ptr, d.ptr, d.ptr, 128, 256, 16, 200, 128, d.ptr, big, None) == qlinear.ERR_ARG  # ldx < cols
    assert lib.qlin_gemm_f32_any_dev(Q6K, d.ptr, d.ptr, d.ptr, 0, 256, 16, 256, 128, None, 0, None) == 0
    d.free()


def test_host_pointer_prefill_takes_this_route_in_row_bands(oracle):
    """qlin_gemm_tokenmajor with 8 tokens or more: decode + dense fp32 GEMM, here with more rows than one
    512 MiB band of fp32 weights holds (K = 16384: 8192 rows per band), so two bands write one Y"""
    tid, n_rows, n_cols, n_tok = synth.GGML_Q4_K, 8192 + 300, 16384, 9
    W = synth.make_weights(tid, n_rows, n_cols, seed=11)
    X = synth.make_activation(n_cols, seed=12, tokens=n_tok)
    Y = qlinear.gemm_tokenmajor(tid, W, X, n_cols)
    rows = np.r_[0:40, 8170:8230, n_rows - 40:n_rows]
    want = reference(oracle, tid, W[rows], X, n_cols)
    assert rel_l2(Y[:, rows], want) <= TOL
    few = qlinear.gemm_tokenmajor(tid, W[:64], X[:3], n_cols)  # fewer than 8 tokens: the vector-ALU kernel
    assert rel_l2(few, reference(oracle, tid, W[:64], X[:3], n_cols)) <= TOL
