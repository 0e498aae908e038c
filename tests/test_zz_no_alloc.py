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
