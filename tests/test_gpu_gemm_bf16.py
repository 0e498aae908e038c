"""GPU parity of the Q4_K x bf16 matrix-core prefill GEMM, through the C ABI.

Two bars per case:
  * the contract: relative L2 <= 2e-3 against a double-precision-accumulated reference that
    uses the EXACT fp32 decoded weights (the CPU oracle) and the same bf16-rounded activations;
  * the arithmetic: relative L2 <= 2e-5 against a double-precision reference of what the kernel
    is designed to compute, so that only fp32 accumulation order is left: from 49 tokens on
    the decoded weights rounded to bf16 (nearest even), up to FEW_TOKENS = 32 tokens the exact
    weights (the few-token kernel does not round them).
"""
import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests.conftest import rel_l2

pytestmark = pytest.mark.gpu
Q4K = synth.GGML_Q4_K
FEW_TOKENS = 32  # kFewTokens of the library: up to here the weights stay exact


def run_gemm(W, Xb, n_rows, n_cols, n_tok, ldx=None, ldy=None):
    ldx = ldx or n_cols
    ldy = ldy or n_rows
    Xpad = np.zeros((n_tok, ldx), np.uint16)
    Xpad[:, :n_cols] = Xb
    dW, dX = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(Xpad)
    Yh = np.full((n_tok, ldy), -3.0, np.float32)
    dY = qlinear.DevBuf.from_numpy(Yh)
    qlinear.gemm_bf16_dev(Q4K, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy)
    qlinear.sync()
    return dY.to_numpy(np.float32, (n_tok, ldy))


def references(oracle, W, Xb, n_cols):
    dec = oracle.dequant_matrix(Q4K, W, n_cols)
    Xf = synth.bf16_bits_to_f32(Xb).astype(np.float64)
    exact = Xf @ dec.astype(np.float64).T
    dec_bf16 = synth.bf16_bits_to_f32(synth.to_bf16_bits(dec)).astype(np.float64)
    designed = Xf @ dec_bf16.T
    return exact, (exact if Xb.shape[0] <= FEW_TOKENS else designed)


@pytest.mark.parametrize("n_tok,n_rows,n_cols", [
    (1, 128, 256), (7, 130, 512), (64, 256, 1024), (128, 384, 4096), (256, 128, 4096),
    (300, 257, 2048), (512, 1024, 4096), (33, 1000, 768), (16, 14336, 256), (17, 48, 512), (48, 100, 256),
    (49, 100, 256), (3, 16, 2560),
    (260, 12805, 256), (1030, 5130, 512),  # enough tiles for the 128-row variant of the kernel
    # 49..128 tokens: 128-token tiles; more than a chip's worth of them (K stays whole), an odd super-block count
    (128, 16500, 1024), (100, 20000, 512), (90, 130, 768), (65, 70, 2048),
])
def test_gemm_bf16_shapes(oracle, n_tok, n_rows, n_cols):
    W = synth.make_weights(Q4K, n_rows, n_cols, seed=n_rows + n_tok)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=n_cols + n_tok, tokens=n_tok))
    Y = run_gemm(W, Xb, n_rows, n_cols, n_tok)
    exact, designed = references(oracle, W, Xb, n_cols)
    assert rel_l2(Y, designed) <= 2e-5, (n_tok, n_rows, n_cols)
    assert rel_l2(Y, exact) <= 2e-3, (n_tok, n_rows, n_cols)


@pytest.mark.parametrize("n_tok", [30, 72])  # few-token kernel, tile kernel
def test_gemm_bf16_strides_and_untouched_padding(oracle, n_tok):
    n_rows, n_cols = 200, 1024
    W = synth.make_weights(Q4K, n_rows, n_cols, seed=3)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=4, tokens=n_tok))
    Y = run_gemm(W, Xb, n_rows, n_cols, n_tok, ldx=n_cols + 64, ldy=n_rows + 12)
    exact, designed = references(oracle, W, Xb, n_cols)
    assert rel_l2(Y[:, :n_rows], designed) <= 2e-5
    assert np.all(Y[:, n_rows:] == -3.0)


def test_gemm_bf16_equals_per_token_matvec(oracle):
    """one-hot activations pick out single decoded weights: the kernel must return exactly the
    bf16 rounding of the oracle's decoded value (ties the GEMM to the bit-exact codec)."""
    n_rows, n_cols = 256, 512
    W = synth.make_weights(Q4K, n_rows, n_cols, seed=8)
    ks = [0, 1, 31, 32, 63, 64, 255, 256, 300, 511]
    X = np.zeros((len(ks), n_cols), np.float32)
    for i, k in enumerate(ks):
        X[i, k] = 1.0
    Y = run_gemm(W, synth.to_bf16_bits(X), n_rows, n_cols, len(ks))
    dec = oracle.dequant_matrix(Q4K, W, n_cols)
    assert np.array_equal(Y, dec[:, ks].T)  # ten tokens: exact weights, bit for bit the codec's values
    # the same probes inside a batch that takes the tile kernel: the bf16 rounding of those values
    Xbig = np.zeros((FEW_TOKENS + 16, n_cols), np.float32)
    Xbig[:len(ks)] = X
    Ybig = run_gemm(W, synth.to_bf16_bits(Xbig), n_rows, n_cols, Xbig.shape[0])
    want = synth.bf16_bits_to_f32(synth.to_bf16_bits(dec[:, ks].T.copy()))
    assert np.array_equal(Ybig[:len(ks)], want)
    assert not Ybig[len(ks):].any()


def test_gemm_bf16_argument_checks():
    lib = qlinear.load()
    d = qlinear.DevBuf(1 << 20)
    assert lib.qlin_gemm_bf16_dev(synth.GGML_Q6_K, d.ptr, d.ptr, d.ptr, 128, 256, 4, 256, 128, None) == qlinear.ERR_TYPE
    assert lib.qlin_gemm_bf16_dev(Q4K, d.ptr, d.ptr, d.ptr, 128, 300, 4, 304, 128, None) == qlinear.ERR_ARG
    assert lib.qlin_gemm_bf16_dev(Q4K, d.ptr, d.ptr, d.ptr, 128, 256, 4, 260, 128, None) == qlinear.ERR_ARG  # ldx % 8
    assert lib.qlin_gemm_bf16_dev(Q4K, d.ptr, d.ptr, d.ptr, 128, 256, 4, 256, 100, None) == qlinear.ERR_ARG  # ldy < rows
    assert lib.qlin_gemm_bf16_dev(Q4K, d.ptr, d.ptr, d.ptr, 0, 256, 4, 256, 128, None) == 0


@pytest.mark.parametrize("n_tok", [128, 512, 2048])
def test_gemm_bf16_full_size_config(oracle, n_tok):
    """Y[n_tok x 14336] = X[n_tok x 4096] . W^T at the benchmark shapes. The oracle is applied to
    a sample of weight rows (all tokens); linearity in X is checked over the whole output."""
    n_rows, n_cols = 14336, 4096
    W = synth.make_weights(Q4K, n_rows, n_cols, seed=41)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=42, tokens=n_tok))
    Y = run_gemm(W, Xb, n_rows, n_cols, n_tok)
    rows = np.random.default_rng(1).choice(n_rows, 192, replace=False)
    exact, designed = references(oracle, W[rows], Xb, n_cols)
    assert rel_l2(Y[:, rows], designed) <= 2e-5
    assert rel_l2(Y[:, rows], exact) <= 2e-3
    # exact scaling by two commutes with every rounding step
    X2 = synth.to_bf16_bits(2.0 * synth.bf16_bits_to_f32(Xb))
    Y2 = run_gemm(W, X2, n_rows, n_cols, n_tok)
    assert np.array_equal(Y2, 2.0 * Y)
