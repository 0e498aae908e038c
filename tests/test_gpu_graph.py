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
