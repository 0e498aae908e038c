"""The device-resident entry points only enqueue kernels (no allocation, no synchronisation, no
memset), so a decode-style sequence of them can be captured into a HIP graph and replayed.
The graph is replayed several times with eager work and synchronisations in between, and every
replay is checked against the eager result."""
import ctypes as C

import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests.conftest import rel_l2

pytestmark = pytest.mark.gpu
Q4K, Q6K = synth.GGML_Q4_K, synth.GGML_Q6_K


def test_decode_style_sequence_in_a_graph(oracle):
    hip = C.CDLL("libamdhip64.so")
    K, FF, KV, V = 1024, 2048, 256, 3000
    host = {"q": synth.make_weights(Q4K, K, K, seed=1), "k": synth.make_weights(Q4K, KV, K, seed=2),
            "v": synth.make_weights(Q4K, KV, K, seed=3), "o": synth.make_weights(Q4K, K, K, seed=4),
            "g": synth.make_weights(Q4K, FF, K, seed=5), "u": synth.make_weights(Q4K, FF, K, seed=6),
            "d": synth.make_weights(Q4K, K, FF, seed=7), "out": synth.make_weights(Q6K, V, K, seed=8)}
    W = {n: qlinear.DevBuf.from_numpy(a) for n, a in host.items()}
    x0 = synth.make_activation(K, seed=9) * np.float32(0.05)
    x = qlinear.DevBuf.from_numpy(x0)
    q, k, v, h = (qlinear.DevBuf(n * 4) for n in (K, KV, KV, FF))
    logits, pick = qlinear.DevBuf(V * 4), qlinear.DevBuf(qlinear.ARGMAX_RESULT_BYTES)

    def enqueue(stream):
        qlinear.gemv_multi_dev(Q4K, [W["q"], W["k"], W["v"]], [q, k, v], [K, KV, KV], x, K, stream)
        qlinear.gemv_add_dev(Q4K, W["o"], q, x, K, K, stream)
        qlinear.gemv_silu_mul_dev(Q4K, W["g"], W["u"], x, h, FF, K, stream)
        qlinear.gemv_add_dev(Q4K, W["d"], h, x, K, FF, stream)
        qlinear.gemv_argmax_dev(Q6K, W["out"], x, logits, pick, V, K, stream)

    def reset_x():
        assert qlinear.load().qlin_dev_upload(x.ptr, x0.ctypes.data, x0.nbytes) == 0

    # eager reference run (also the warm-up: one-time kernel attributes are set outside the capture)
    enqueue(None)
    qlinear.sync()
    want_x = x.to_numpy(np.float32, (K,))
    want_logits = logits.to_numpy(np.float32, (V,))
    want_pick = int(pick.to_numpy(np.int32, (2,))[0])
    # the eager result itself against the oracle, step by step in float64
    g64 = lambda name, vec: oracle.gemv_f64(Q4K if name != "out" else Q6K, host[name], vec.astype(np.float32), vec.shape[0]).astype(np.float64)
    x1 = x0.astype(np.float64) + g64("o", g64("q", x0))
    gg, uu = g64("g", x1), g64("u", x1)
    x2 = x1 + g64("d", gg / (1 + np.exp(-gg)) * uu)
    assert rel_l2(want_x, x2) <= 2e-5
    assert want_pick == int(np.argmax(want_logits))

    stream, graph, gexec = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert hip.hipStreamCreate(C.byref(stream)) == 0
    reset_x()
    assert hip.hipStreamBeginCapture(stream, 0) == 0  # hipStreamCaptureModeGlobal
    enqueue(stream)
    assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
    n_nodes = C.c_size_t(0)
    assert hip.hipGraphGetNodes(graph, None, C.byref(n_nodes)) == 0
    assert n_nodes.value == 7  # five matvec launches + the two kernels of the pick: nothing but kernels
    for replay in range(4):
        reset_x()
        assert hip.hipGraphLaunch(gexec, stream) == 0
        assert hip.hipStreamSynchronize(stream) == 0
        assert np.array_equal(x.to_numpy(np.float32, (K,)), want_x), replay
        assert np.array_equal(logits.to_numpy(np.float32, (V,)), want_logits), replay
        assert int(pick.to_numpy(np.int32, (2,))[0]) == want_pick, replay
        # eager work of the program between replays
        qlinear.gemv_dev(Q4K, W["q"], x, q, K, K)
        qlinear.sync()
    assert hip.hipGraphExecDestroy(gexec) == 0 and hip.hipGraphDestroy(graph) == 0
    assert hip.hipStreamDestroy(stream) == 0


def test_prefill_sequence_in_a_graph(oracle):
    """The fused prefill GEMMs take no workspace and only enqueue: a chunk's projections (large tiles, small tiles and
    the few-token kernel, three formats, and three tensors in one launch of qlin_gemm_bf16_multi_dev) are captured with a
    NULL workspace and replayed bit-identically."""
    hip = C.CDLL("libamdhip64.so")
    Q5K, NL = synth.GGML_Q5_K, synth.GGML_IQ4_NL
    K, n_tok = 512, 300
    shapes = [(Q4K, 12900, n_tok), (Q5K, 640, n_tok), (NL, 300, n_tok), (Q6K, 200, 20)]  # large tiles, small, small, few tokens
    host = [synth.make_weights(t, r, K, seed=20 + i) for i, (t, r, _) in enumerate(shapes)]
    W = [qlinear.DevBuf.from_numpy(a) for a in host]
    Xb = synth.to_bf16_bits(synth.make_activation(K, seed=30, tokens=n_tok))
    dX = qlinear.DevBuf.from_numpy(Xb)
    Y = [qlinear.DevBuf(m * r * 4) for (_, r, m) in shapes]
    lib = qlinear.load()
    # three Q5_K tensors that share one launch (the shape of a chunk's Q, K and V projections)
    qkv_rows = [640, 130, 70]
    qkv_host = [synth.make_weights(Q5K, r, K, seed=40 + i) for i, r in enumerate(qkv_rows)]
    qkv_W = [qlinear.DevBuf.from_numpy(a) for a in qkv_host]
    qkv_Y = [qlinear.DevBuf(n_tok * r * 4) for r in qkv_rows]
    Wp = (C.c_void_p * 3)(*[b.ptr for b in qkv_W])
    Yp = (C.c_void_p * 3)(*[b.ptr for b in qkv_Y])
    rows3 = (C.c_int * 3)(*qkv_rows)

    def enqueue(stream):
        for (t, r, m), w, y in zip(shapes, W, Y):
            assert lib.qlin_gemm_bf16_any_dev(t, w.ptr, dX.ptr, y.ptr, r, K, m, K, r, None, 0, stream) == 0, lib.qlin_last_error()
        assert lib.qlin_gemm_bf16_multi_dev(Q5K, 3, Wp, dX.ptr, Yp, rows3, K, n_tok, K, rows3, None, 0, stream) == 0, lib.qlin_last_error()

    def clear():
        for r, m, y in [(r, m, y) for (_, r, m), y in zip(shapes, Y)] + [(r, n_tok, y) for r, y in zip(qkv_rows, qkv_Y)]:
            z = np.full(m * r, -3.0, np.float32)
            assert lib.qlin_dev_upload(y.ptr, z.ctypes.data, z.nbytes) == 0

    enqueue(None)  # eager run: the reference for the replays, itself checked against the oracle
    qlinear.sync()
    want = [y.to_numpy(np.float32, (m, r)) for (_, r, m), y in zip(shapes, Y)]
    Xf = synth.bf16_bits_to_f32(Xb).astype(np.float64)
    for (t, r, m), h, got in zip(shapes, host, want):
        dec = oracle.dequant_matrix(t, h, K)
        if m > 24:
            dec = synth.bf16_bits_to_f32(synth.to_bf16_bits(dec))
        assert rel_l2(got, Xf[:m] @ dec.astype(np.float64).T) <= 2e-5, (t, r, m)
    qkv_want = [y.to_numpy(np.float32, (n_tok, r)) for r, y in zip(qkv_rows, qkv_Y)]
    for r, h, got in zip(qkv_rows, qkv_host, qkv_want):
        dec = synth.bf16_bits_to_f32(synth.to_bf16_bits(oracle.dequant_matrix(Q5K, h, K)))
        assert rel_l2(got, Xf @ dec.astype(np.float64).T) <= 2e-5, r

    stream, graph, gexec = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert hip.hipStreamCreate(C.byref(stream)) == 0
    assert hip.hipStreamBeginCapture(stream, 0) == 0  # hipStreamCaptureModeGlobal
    enqueue(stream)
    assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
    n_nodes = C.c_size_t(0)
    assert hip.hipGraphGetNodes(graph, None, C.byref(n_nodes)) == 0
    assert n_nodes.value == len(shapes) + 1  # one kernel per product and one for the three tensors together, nothing else
    for replay in range(3):
        clear()
        assert hip.hipGraphLaunch(gexec, stream) == 0
        assert hip.hipStreamSynchronize(stream) == 0
        for (_, r, m), y, w_ in zip(shapes, Y, want):
            assert np.array_equal(y.to_numpy(np.float32, (m, r)), w_), replay
        for r, y, w_ in zip(qkv_rows, qkv_Y, qkv_want):
            assert np.array_equal(y.to_numpy(np.float32, (n_tok, r)), w_), (replay, r)
        qlinear.gemm_bf16_any_dev(Q5K, W[1], dX, Y[1], 640, K, 100, K, 640, None)  # eager work between replays
        qlinear.sync()
    assert hip.hipGraphExecDestroy(gexec) == 0 and hip.hipGraphDestroy(graph) == 0
    assert hip.hipStreamDestroy(stream) == 0
    for b in W + Y + [dX] + qkv_W + qkv_Y:
        b.free()
