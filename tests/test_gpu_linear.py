"""GPU parity of the quantized matvec / prefill / MoE-token paths against the CPU oracle
(double-precision accumulate) and the reference's golden outputs, through the C ABI.
Tolerance: relative L2 <= 1e-5 for every fp32 path."""
import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests.conftest import rel_l2

pytestmark = pytest.mark.gpu
# every block format, plus dense F32/F16/BF16 rows
NAMES = list(synth.TYPE_NAMES.items()) + list(synth.DENSE_TYPES.items())
# the types the reference golden outputs exist for: the model path's block formats and dense rows
LINEAR = list(synth.LINEAR_TYPES.items()) + list(synth.DENSE_TYPES.items())
TOL = 1e-5


@pytest.mark.parametrize("tid,name", LINEAR)
def test_matvec_matches_reference_golden(linear_golden, tid, name):
    W, x = linear_golden[name + "_W"], linear_golden["x"]
    y = qlinear.matvec(tid, W, x, x.shape[0])
    assert rel_l2(y, linear_golden[name + "_y_f64"]) <= TOL
    assert rel_l2(y, linear_golden[name + "_y_f32"]) <= TOL


@pytest.mark.parametrize("tid,name", NAMES)
@pytest.mark.parametrize("n_rows,n_cols", [(1, 256), (13, 512), (64, 4096), (257, 2048), (33, 14336), (5, 20480)])
def test_matvec_shapes(oracle, tid, name, n_rows, n_cols):
    W = synth.make_weights(tid, n_rows, n_cols, seed=n_rows * 7 + tid)
    x = synth.make_activation(n_cols, seed=n_cols + tid)
    y = qlinear.matvec(tid, W, x, n_cols)
    want = oracle.gemv_f64(tid, W, x, n_cols)
    if n_rows >= 13:
        assert rel_l2(y, want) <= TOL, (name, n_rows, n_cols)
    # a relative-L2 figure over one or a few outputs only measures cancellation in those dot
    # products, so every output is also held to the fp32 dot-product error bound
    # |err| <= 1e-6 * sum|w||x| (about 10 ulp of the un-cancelled magnitude)
    bound = np.abs(oracle.dequant_matrix(tid, W, n_cols)).astype(np.float64) @ np.abs(x).astype(np.float64)
    assert np.all(np.abs(y.astype(np.float64) - want) <= 1e-6 * bound + 1e-30), (name, n_rows, n_cols)


@pytest.mark.parametrize("tid,name", NAMES)
def test_matvec_one_hot_and_ones(oracle, tid, name):
    n_rows, n_cols = 40, 4096
    W = synth.make_weights(tid, n_rows, n_cols, seed=90 + tid)
    dec = oracle.dequant_matrix(tid, W, n_cols)
    for k in (0, 17, 255, 256, 4095):
        e = np.zeros(n_cols, np.float32)
        e[k] = 1.0
        y = qlinear.matvec(tid, W, e, n_cols)
        assert np.allclose(y, dec[:, k], rtol=1e-6, atol=1e-9), (name, k)
    y = qlinear.matvec(tid, W, np.ones(n_cols, np.float32), n_cols)
    assert rel_l2(y, dec.astype(np.float64).sum(axis=1)) <= TOL


def test_matvec_empty_and_errors():
    lib = qlinear.load()
    W = synth.make_weights(synth.GGML_Q4_K, 4, 512, seed=1)
    x = synth.make_activation(512, seed=2)
    y = np.zeros(4, np.float32)
    assert lib.qlin_matvec(y.ctypes.data, W.ctypes.data, synth.GGML_Q4_K, 512, x.ctypes.data, 0) == 0
    assert lib.qlin_matvec(y.ctypes.data, W.ctypes.data, 99, 512, x.ctypes.data, 4) == qlinear.ERR_TYPE
    assert lib.qlin_matvec(y.ctypes.data, W.ctypes.data, 9, 512, x.ctypes.data, 4) == qlinear.ERR_TYPE  # Q8_1
    assert lib.qlin_matvec(y.ctypes.data, W.ctypes.data, synth.GGML_F16, 500, x.ctypes.data, 4) == 0  # dense rows: any length
    assert lib.qlin_matvec(y.ctypes.data, W.ctypes.data, synth.GGML_Q4_K, 500, x.ctypes.data, 4) == qlinear.ERR_ARG
    assert lib.qlin_matvec(None, W.ctypes.data, synth.GGML_Q4_K, 512, x.ctypes.data, 4) == qlinear.ERR_ARG
    assert lib.qlin_matvec(y.ctypes.data, W.ctypes.data, synth.GGML_Q4_K, 512, x.ctypes.data, -1) == qlinear.ERR_ARG


# (type, rows, cols) of the benchmark configurations, at full size
FULL = [
    (synth.GGML_Q8_0, 4096, 4096), (synth.GGML_Q4_K, 4096, 4096), (synth.GGML_Q4_K, 14336, 4096),
    (synth.GGML_Q4_K, 4096, 14336), (synth.GGML_Q5_K, 4096, 4096), (synth.GGML_IQ4_NL, 14336, 4096),
    (synth.GGML_IQ2_XXS, 4096, 14336), (synth.GGML_IQ3_S, 4096, 14336), (synth.GGML_Q6_K, 151936, 4096),
    # vocabulary-sized projections in the formats of the matrix-instruction kernels: one workgroup of several hundred
    # rows per compute unit, or several equal rounds of them
    (synth.GGML_Q4_K, 151936, 4096), (synth.GGML_Q4_K, 200003, 2048), (synth.GGML_IQ4_NL, 151936, 4096),
    (synth.GGML_Q2_K, 170001, 2048), (synth.GGML_IQ2_XXS, 151936, 4096), (synth.GGML_Q4_0, 49152, 4096),
]


@pytest.mark.parametrize("tid,n_rows,n_cols", FULL)
def test_device_gemv_full_size_configs(oracle, tid, n_rows, n_cols):
    W = synth.make_weights(tid, n_rows, n_cols, seed=tid * 3 + 1)
    x = synth.make_activation(n_cols, seed=tid * 3 + 2)
    dW, dx = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(x)
    dy = qlinear.DevBuf(n_rows * 4)
    qlinear.gemv_dev(tid, dW, dx, dy, n_rows, n_cols)
    qlinear.sync()
    y = dy.to_numpy(np.float32, (n_rows,))
    # oracle on a strided sample of rows when the matrix is huge (keeps the CPU side to seconds)
    step = 1 if n_rows <= 16384 else 16
    want = oracle.gemv_f64(tid, W[::step], x, n_cols)
    assert rel_l2(y[::step], want) <= TOL
    # linearity over the whole output: W.(2x) == 2 W.x exactly, W.(x+e0) - W.x == column 0
    dx2 = qlinear.DevBuf.from_numpy(2 * x)
    qlinear.gemv_dev(tid, dW, dx2, dy, n_rows, n_cols)
    qlinear.sync()
    assert np.array_equal(dy.to_numpy(np.float32, (n_rows,)), 2 * y)


def test_fused_entry_points(oracle, linear_golden):
    lib = qlinear.load()
    x = linear_golden["x"]
    n_cols = x.shape[0]
    Wa, Wb, Wc = linear_golden["q4_K_W"], linear_golden["q6_K_W"], linear_golden["q8_0_W"]
    ya, yb = np.zeros(24, np.float32), np.zeros(24, np.float32)
    assert lib.qlin_matvec_fused2(ya.ctypes.data, Wa.ctypes.data, synth.GGML_Q4_K, yb.ctypes.data, Wb.ctypes.data,
                                  synth.GGML_Q6_K, n_cols, x.ctypes.data, 24) == 0
    assert rel_l2(ya, linear_golden["q4_K_y_f64"]) <= TOL and rel_l2(yb, linear_golden["q6_K_y_f64"]) <= TOL
    q, k, v = np.zeros(24, np.float32), np.zeros(16, np.float32), np.zeros(16, np.float32)
    assert lib.qlin_matvec_qkv(q.ctypes.data, Wa.ctypes.data, synth.GGML_Q4_K, 24, k.ctypes.data, Wb.ctypes.data,
                               synth.GGML_Q6_K, v.ctypes.data, Wc.ctypes.data, synth.GGML_Q8_0, 16, n_cols,
                               x.ctypes.data) == 0
    assert rel_l2(q, linear_golden["q4_K_y_f64"]) <= TOL
    assert rel_l2(k, linear_golden["q6_K_y_f64"][:16]) <= TOL
    assert rel_l2(v, linear_golden["q8_0_y_f64"][:16]) <= TOL


@pytest.mark.parametrize("tid,name", LINEAR)
def test_expert_slice_and_prefill_match_reference_golden(linear_golden, tid, name):
    lib = qlinear.load()
    W, x, X = linear_golden[name + "_W"], linear_golden["x"], linear_golden["X"]
    n_cols = x.shape[0]
    y = np.zeros(8, np.float32)
    assert lib.qlin_matvec_expert(y.ctypes.data, W.ctypes.data, tid, n_cols, 1, x.ctypes.data, 8) == 0
    assert rel_l2(y, linear_golden[name + "_y_expert1"]) <= TOL
    Y = qlinear.gemm_tokenmajor(tid, W, X, n_cols)
    assert rel_l2(Y, linear_golden[name + "_Y_tokmajor"]) <= TOL


def test_prefill_strides(oracle):
    tid, n_rows, n_cols, n_tok = synth.GGML_Q5_K, 37, 768, 11
    lib = qlinear.load()
    W = synth.make_weights(tid, n_rows, n_cols, seed=5)
    X = np.zeros((n_tok, n_cols + 24), np.float32)
    X[:, :n_cols] = synth.make_activation(n_cols, seed=6, tokens=n_tok)
    X[:, n_cols:] = np.nan  # padding must never be read into the result
    Y = np.full((n_tok, n_rows + 5), -7.0, np.float32)
    assert lib.qlin_gemm_tokenmajor(Y.ctypes.data, W.ctypes.data, tid, n_cols, X.ctypes.data, n_rows, n_tok,
                                    n_rows + 5, n_cols + 24) == 0
    want = oracle.gemm_tokmajor(tid, W, np.ascontiguousarray(X[:, :n_cols]), n_cols)
    assert rel_l2(Y[:, :n_rows], want) <= TOL
    assert np.all(Y[:, n_rows:] == -7.0)


def test_weight_registry(oracle):
    lib = qlinear.load()
    tid, n_rows, n_cols = synth.GGML_Q4_K, 128, 4096
    W = synth.make_weights(tid, n_rows, n_cols, seed=21)
    keep = W.copy()
    x = synth.make_activation(n_cols, seed=22)
    want = oracle.gemv_f64(tid, keep, x, n_cols)
    assert lib.qlin_weight_register(W.ctypes.data, W.nbytes) == 0
    assert lib.qlin_weight_register(W.ctypes.data + 100, 10) == qlinear.ERR_ARG  # overlap
    assert lib.qlin_weight_device_ptr(W.ctypes.data + 2304)
    W[:] = 0  # the device copy, not the (now zeroed) host bytes, must be what the matvec reads
    assert rel_l2(qlinear.matvec(tid, W, x, n_cols), want) <= TOL
    y = np.zeros(32, np.float32)  # an expert slice inside the registered range
    assert lib.qlin_matvec_expert(y.ctypes.data, W.ctypes.data, tid, n_cols, 2, x.ctypes.data, 32) == 0
    assert rel_l2(y, want[64:96]) <= TOL
    assert lib.qlin_weight_unregister(W.ctypes.data) == 0
    assert lib.qlin_weight_unregister(W.ctypes.data) == qlinear.ERR_ARG
    assert np.all(qlinear.matvec(tid, W, x, n_cols) == 0)


@pytest.mark.parametrize("label", ["q4k", "q4k_down_q6k"])
def test_moe_token_ffn_against_the_compiled_reference(manifest, linear_golden, label):
    """qlin_moe_ffn_token_types from router logits to output against the fixture of the reference's own block
    (tf_softmax, heap selection, tf_qmatvec_expert x3, tf_silu_mul_avx2, weighted sum). Bar 2e-4: the reference's
    softmax and SiLU use a polynomial exp that moves the expert weights by up to 5e-5."""
    from tests.conftest import moe_block_case
    c = moe_block_case(manifest, linear_golden, label)
    lib = qlinear.load()
    for t in range(c["logits"].shape[0]):
        out = np.zeros(c["n_embd"], np.float32)
        logits, x = np.ascontiguousarray(c["logits"][t]), np.ascontiguousarray(c["x"][t])
        assert lib.qlin_moe_ffn_token_types(out.ctypes.data, c["gate"].ctypes.data, c["up"].ctypes.data, c["down"].ctypes.data,
                                            c["types"][0], c["types"][1], c["types"][2], c["n_embd"], c["n_ff"],
                                            c["n_expert"], c["top_k"], logits.ctypes.data, x.ctypes.data) == 0
        assert rel_l2(out, c["out"][t]) <= 2e-4, (label, t)
        # the device routing picks the reference's experts with the reference's weights (the order of the k is the
        # device's own: it only decides the order of an fp32 sum)
        dl = qlinear.DevBuf.from_numpy(logits)
        di, dw = qlinear.DevBuf(c["top_k"] * 4), qlinear.DevBuf(c["top_k"] * 4)
        assert lib.qlin_moe_route_dev(dl.ptr, 1, c["n_expert"], c["top_k"], di.ptr, dw.ptr, None) == 0
        qlinear.sync()
        gi, gw = di.to_numpy(np.int32, (c["top_k"],)), dw.to_numpy(np.float32, (c["top_k"],))
        assert np.array_equal(np.sort(gi), np.sort(c["idx"][t]))
        assert np.allclose(gw[np.argsort(gi)], c["w"][t][np.argsort(c["idx"][t])], rtol=5e-5, atol=0)
        for b in (dl, di, dw):
            b.free()


def test_moe_route_and_token_ffn(oracle):
    lib = qlinear.load()
    tid, n_expert, n_embd, n_ff, k = synth.GGML_Q4_K, 16, 512, 256, 4
    gate = synth.make_weights(tid, n_expert * n_ff, n_embd, seed=31)
    up = synth.make_weights(tid, n_expert * n_ff, n_embd, seed=32)
    down = synth.make_weights(tid, n_expert * n_embd, n_ff, seed=33)
    x = synth.make_activation(n_embd, seed=34)
    logits = synth.make_router_logits(1, n_expert, seed=35)[0]
    idx, w = oracle.moe_route(logits, k)
    want = oracle.moe_ffn_token(tid, gate, up, down, n_embd, n_ff, x, idx, w, f64=True)
    out = np.zeros(n_embd, np.float32)
    assert lib.qlin_moe_ffn_token(out.ctypes.data, gate.ctypes.data, up.ctypes.data, down.ctypes.data, tid, n_embd,
                                  n_ff, n_expert, k, logits.ctypes.data, x.ctypes.data) == 0
    assert rel_l2(out, want) <= TOL
    # routing on its own, many tokens: same expert set and weights as the oracle
    n_tok, n_expert, k = 64, 128, 8
    lg = synth.make_router_logits(n_tok, n_expert, seed=36)
    dl = qlinear.DevBuf.from_numpy(lg)
    di, dw = qlinear.DevBuf(n_tok * k * 4), qlinear.DevBuf(n_tok * k * 4)
    assert lib.qlin_moe_route_dev(dl.ptr, n_tok, n_expert, k, di.ptr, dw.ptr, None) == 0
    qlinear.sync()
    gi, gw = di.to_numpy(np.int32, (n_tok, k)), dw.to_numpy(np.float32, (n_tok, k))
    for t in range(n_tok):
        oi, ow = oracle.moe_route(lg[t], k)
        order_o, order_g = np.argsort(oi), np.argsort(gi[t])
        assert np.array_equal(oi[order_o], gi[t][order_g])
        assert np.allclose(ow[order_o], gw[t][order_g], rtol=1e-5, atol=1e-8)
        assert np.all(np.diff(gw[t]) <= 0)  # descending weight order


@pytest.mark.parametrize("types", [(synth.GGML_Q4_K, synth.GGML_Q4_K, synth.GGML_Q6_K),
                                   (synth.GGML_Q4_K, synth.GGML_Q6_K, synth.GGML_Q8_0),
                                   (synth.GGML_IQ4_NL, synth.GGML_IQ4_NL, synth.GGML_F16)])
def test_token_ffn_with_one_format_per_tensor(oracle, types):
    """the down projections of K-quant mixes are partly Q6_K beside Q4_K gate and up"""
    lib = qlinear.load()
    n_expert, n_embd, n_ff, k = 8, 512, 256, 3
    gate = synth.make_weights(types[0], n_expert * n_ff, n_embd, seed=41)
    up = synth.make_weights(types[1], n_expert * n_ff, n_embd, seed=42)
    down = synth.make_weights(types[2], n_expert * n_embd, n_ff, seed=43)
    x = synth.make_activation(n_embd, seed=44)
    logits = synth.make_router_logits(1, n_expert, seed=45)[0]
    idx, w = oracle.moe_route(logits, k)
    want = np.zeros(n_embd, np.float64)
    for e, we in zip(idx, w):
        G = oracle.dequant_matrix(types[0], gate[e * n_ff:(e + 1) * n_ff], n_embd).astype(np.float64)
        U = oracle.dequant_matrix(types[1], up[e * n_ff:(e + 1) * n_ff], n_embd).astype(np.float64)
        D = oracle.dequant_matrix(types[2], down[e * n_embd:(e + 1) * n_embd], n_ff).astype(np.float64)
        g, u = G @ x.astype(np.float64), U @ x.astype(np.float64)
        want += float(we) * (D @ (g / (1.0 + np.exp(-g)) * u))
    out = np.zeros(n_embd, np.float32)
    assert lib.qlin_moe_ffn_token_types(out.ctypes.data, gate.ctypes.data, up.ctypes.data, down.ctypes.data, types[0],
                                        types[1], types[2], n_embd, n_ff, n_expert, k, logits.ctypes.data,
                                        x.ctypes.data) == 0
    assert rel_l2(out, want) <= TOL


@pytest.mark.parametrize("n_expert,k", [(5, 1), (5, 5), (64, 8), (65, 8), (128, 8), (200, 64), (300, 4), (512, 8),
                                        (513, 8), (1000, 2), (128, 100)])
def test_routing_over_expert_counts(oracle, n_expert, k):
    """register-resident form up to 512 experts and 64 picks, LDS form beyond; same experts and weights as
    the oracle, in descending weight order"""
    lib = qlinear.load()
    n_tok = 9
    lg = synth.make_router_logits(n_tok, n_expert, seed=n_expert + k)
    dl = qlinear.DevBuf.from_numpy(lg)
    di, dw = qlinear.DevBuf(n_tok * k * 4), qlinear.DevBuf(n_tok * k * 4)
    assert lib.qlin_moe_route_dev(dl.ptr, n_tok, n_expert, k, di.ptr, dw.ptr, None) == 0
    qlinear.sync()
    gi, gw = di.to_numpy(np.int32, (n_tok, k)), dw.to_numpy(np.float32, (n_tok, k))
    for t in range(n_tok):
        oi, ow = oracle.moe_route(lg[t], k)
        order_o, order_g = np.argsort(oi), np.argsort(gi[t])
        assert np.array_equal(oi[order_o], gi[t][order_g]), (t, n_expert, k)
        assert np.allclose(ow[order_o], gw[t][order_g], rtol=1e-5, atol=1e-8)
        assert np.all(np.diff(gw[t]) <= 0)
    for b in (dl, di, dw):
        b.free()


def _route_on_device(lg, k):
    n_tok, n_expert = lg.shape
    dl = qlinear.DevBuf.from_numpy(lg)
    di, dw = qlinear.DevBuf(n_tok * k * 4), qlinear.DevBuf(n_tok * k * 4)
    assert qlinear.load().qlin_moe_route_dev(dl.ptr, n_tok, n_expert, k, di.ptr, dw.ptr, None) == 0
    qlinear.sync()
    idx, w = di.to_numpy(np.int32, (n_tok, k)), dw.to_numpy(np.float32, (n_tok, k))
    for b in (dl, di, dw):
        b.free()
    return idx, w


@pytest.mark.parametrize("n_expert", [100, 600])  # probabilities in registers / in LDS
def test_routing_ties_choose_the_experts_the_reference_heap_keeps(oracle, n_expert):
    """Equal probabilities around the k-th place: which of them survive is decided by the reference's
    min-heap (common/transformer.h:4057-4086), not by the index. The device must keep the same experts
    with the same weights; where the heap decides it also emits them in heap order."""
    rng = np.random.default_rng(77 + n_expert)
    k = 6
    lg = rng.integers(0, 3, size=(40, n_expert)).astype(np.float32) * np.float32(0.5)  # three levels: ties everywhere
    lg[0] = 0.0
    lg[0, 70] = 1.0                       # one winner, everything else equal
    lg[1] = 0.25                          # all equal
    idx, w = _route_on_device(lg, k)
    for t in range(lg.shape[0]):
        oi, ow = oracle.moe_route(lg[t], k)
        got = dict(zip(idx[t].tolist(), w[t].tolist()))
        want = dict(zip(oi.tolist(), ow.tolist()))
        assert set(got) == set(want), (t, sorted(got), sorted(want))
        for e in want:
            assert abs(got[e] - want[e]) <= 1e-6 * want[e], (t, e)
    # all equal: the heap keeps the first k experts it saw, root first
    assert idx[1].tolist() == oracle.moe_route(lg[1], k)[0].tolist()


@pytest.mark.parametrize("n_expert", [100, 600])
def test_routing_with_non_finite_logits_follows_the_reference(oracle, n_expert):
    """A NaN or +Inf logit makes every probability NaN (softmax divides by a NaN sum); the reference's heap
    then keeps the first k experts with NaN weights (every comparison is false). Same here."""
    k = 4
    lg = np.random.default_rng(5).standard_normal((3, n_expert)).astype(np.float32)
    lg[0, 17] = np.nan
    lg[1, 3] = np.inf
    idx, w = _route_on_device(lg, k)
    for t in (0, 1):
        oi, ow = oracle.moe_route(lg[t], k)
        assert idx[t].tolist() == oi.tolist() == list(range(k))
        assert np.all(np.isnan(w[t])) and np.all(np.isnan(ow))
    oi, ow = oracle.moe_route(lg[2], k)  # the finite token beside them is untouched
    assert set(idx[2].tolist()) == set(oi.tolist()) and abs(float(w[2].sum()) - 1.0) < 1e-6
