"""The entry point that allocates nothing, qlin_moe_ffn_static_dev (scratch in a device array of the library),
against qlin_moe_ffn_types_dev with a caller's workspace: bit-identical outputs on two calls in a row, the
second with a smaller input, so that whatever the first call left in the scratch does not leak into the second.
Collected last: it must pass alone in a fresh process and after every other test."""
import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests.conftest import rel_l2

pytestmark = pytest.mark.gpu
Q4K, Q6K = synth.GGML_Q4_K, synth.GGML_Q6_K


def both(types, gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert):
    n_tok, top_k = idx.shape
    bufs = [qlinear.DevBuf.from_numpy(a) for a in (gate, up, down, Xb, idx.astype(np.int32), w.astype(np.float32))]
    outs = []
    for static in (False, True):
        dout = qlinear.DevBuf.from_numpy(np.full((n_tok, n_embd), -7.0, np.float32))
        if static:
            qlinear.moe_ffn_static_dev(types, *bufs, dout, n_tok, top_k, n_embd, n_ff, n_expert)
            dws = None
        else:
            dws = qlinear.DevBuf(max(qlinear.moe_workspace_bytes(n_tok, top_k, n_embd, n_ff, n_expert), 256))
            qlinear.moe_ffn_types_dev(types, *bufs, dout, n_tok, top_k, n_embd, n_ff, n_expert, dws)
        qlinear.sync()
        outs.append(dout.to_numpy(np.float32, (n_tok, n_embd)))
        dout.free()
        if dws:
            dws.free()
    for b in bufs:
        b.free()
    return outs


@pytest.mark.parametrize("types", [(Q4K, Q4K, Q4K), (Q4K, Q4K, Q6K)])
def test_static_scratch_matches_workspace_variant_on_two_calls(oracle, types):
    assert qlinear.load().qlin_init(0) == 0
    n_expert, n_embd, n_ff = 16, 1024, 512
    gate = synth.make_weights(types[0], n_expert * n_ff, n_embd, seed=71)
    up = synth.make_weights(types[1], n_expert * n_ff, n_embd, seed=72)
    down = synth.make_weights(types[2], n_expert * n_embd, n_ff, seed=73)
    for n_tok, top_k, seed in ((48, 4, 1), (7, 2, 2)):  # the second call is smaller than the first
        Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=80 + seed, tokens=n_tok))
        logits = synth.make_router_logits(n_tok, n_expert, seed=90 + seed)
        idx = np.zeros((n_tok, top_k), np.int32)
        w = np.zeros((n_tok, top_k), np.float32)
        for t in range(n_tok):
            idx[t], w[t] = oracle.moe_route(logits[t], top_k)
        with_ws, static = both(types, gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert)
        assert np.array_equal(with_ws.view(np.uint32), static.view(np.uint32)), (types, n_tok)
        if types[2] == Q4K:  # and both are right (the mixed case is checked against the oracle in test_gpu_moe.py)
            X = synth.bf16_bits_to_f32(Xb)
            want = np.stack([oracle.moe_ffn_token(Q4K, gate, up, down, n_embd, n_ff, X[t], idx[t], w[t], f64=True)
                             for t in range(n_tok)])
            assert rel_l2(static, want) <= 2e-5


def test_static_scratch_rejects_what_does_not_fit():
    lib = qlinear.load()
    assert lib.qlin_init(0) == 0
    n_tok, top_k, n_embd, n_ff, n_expert = 512, 8, 2048, 768, 128
    assert qlinear.moe_workspace_bytes(n_tok, top_k, n_embd, n_ff, n_expert) > 16 << 20
    d = qlinear.DevBuf(4096)
    rc = lib.qlin_moe_ffn_static_dev(Q4K, Q4K, Q4K, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, n_tok, top_k, n_embd,
                                     n_ff, n_expert, None)
    assert rc == qlinear.ERR_ARG
    assert b"scratch" in lib.qlin_last_error()
    # the benchmark's shape fits
    assert qlinear.moe_workspace_bytes(64, 8, 2048, 768, 128) <= 16 << 20
    d.free()


def test_static_entry_records_into_a_graph_and_replays_bit_identically(oracle):
    """Stream capture refuses a call that allocates or synchronises, so recording qlin_moe_ffn_static_dev (after one
    eager call has done its once-only kernel set-up) shows that it does neither. The graph is replayed three times
    with eager work of the same entry point on another shape between the replays; every replay reproduces the eager
    result bit for bit."""
    import ctypes as C
    lib = qlinear.load()
    assert lib.qlin_init(0) == 0
    hip = C.CDLL("libamdhip64.so")
    vp = C.c_void_p
    hip.hipStreamCreate.argtypes = [C.POINTER(vp)]
    hip.hipStreamBeginCapture.argtypes = [vp, C.c_int]
    hip.hipStreamEndCapture.argtypes = [vp, C.POINTER(vp)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(vp), vp, vp, vp, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [vp, vp]
    hip.hipStreamSynchronize.argtypes = [vp]
    hip.hipGraphExecDestroy.argtypes = [vp]
    hip.hipGraphDestroy.argtypes = [vp]
    hip.hipStreamDestroy.argtypes = [vp]

    types = (Q4K, Q4K, Q6K)
    n_expert, n_embd, n_ff, n_tok, top_k = 16, 1024, 512, 40, 4
    gate = synth.make_weights(types[0], n_expert * n_ff, n_embd, seed=171)
    up = synth.make_weights(types[1], n_expert * n_ff, n_embd, seed=172)
    down = synth.make_weights(types[2], n_expert * n_embd, n_ff, seed=173)

    def inputs(n, k, seed):
        Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=seed, tokens=n))
        logits = synth.make_router_logits(n, n_expert, seed=seed + 1)
        idx, w = np.zeros((n, k), np.int32), np.zeros((n, k), np.float32)
        for t in range(n):
            idx[t], w[t] = oracle.moe_route(logits[t], k)
        return [qlinear.DevBuf.from_numpy(a) for a in (Xb, idx, w)]

    wbufs = [qlinear.DevBuf.from_numpy(a) for a in (gate, up, down)]
    main_in, other_in = inputs(n_tok, top_k, 300), inputs(9, 2, 310)
    dout = qlinear.DevBuf.from_numpy(np.full((n_tok, n_embd), -7.0, np.float32))
    dother = qlinear.DevBuf(9 * n_embd * 4)

    stream = vp()
    assert hip.hipStreamCreate(C.byref(stream)) == 0
    qlinear.moe_ffn_static_dev(types, *wbufs, *main_in, dout, n_tok, top_k, n_embd, n_ff, n_expert, stream)
    qlinear.sync(stream)
    eager = dout.to_numpy(np.float32, (n_tok, n_embd))

    graph, gexec = vp(), vp()
    assert hip.hipStreamBeginCapture(stream, 0) == 0  # hipStreamCaptureModeGlobal
    rc = lib.qlin_moe_ffn_static_dev(types[0], types[1], types[2], *[b.ptr for b in wbufs], *[b.ptr for b in main_in],
                                     dout.ptr, n_tok, top_k, n_embd, n_ff, n_expert, stream)
    end = hip.hipStreamEndCapture(stream, C.byref(graph))
    assert rc == 0, lib.qlin_last_error()
    assert end == 0 and graph.value
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
    for replay in range(3):
        fill = np.full((n_tok, n_embd), -7.0, np.float32)  # the output starts from a known value each time
        assert lib.qlin_dev_upload(dout.ptr, fill.ctypes.data_as(vp), fill.nbytes) == 0
        assert hip.hipGraphLaunch(gexec, stream) == 0
        assert hip.hipStreamSynchronize(stream) == 0
        got = dout.to_numpy(np.float32, (n_tok, n_embd))
        assert np.array_equal(got.view(np.uint32), eager.view(np.uint32)), replay
        # eager work of the same entry point on another shape overwrites the shared scratch between replays
        qlinear.moe_ffn_static_dev(types, *wbufs, *other_in, dother, 9, 2, n_embd, n_ff, n_expert, stream)
        qlinear.sync(stream)
    assert hip.hipGraphExecDestroy(gexec) == 0
    assert hip.hipGraphDestroy(graph) == 0
    assert hip.hipStreamDestroy(stream) == 0
    for b in wbufs + main_in + other_in + [dout, dother]:
        b.free()
