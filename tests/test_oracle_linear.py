"""Pins the CPU oracle's matvec / prefill / MoE functions. CPU only."""
import numpy as np
import pytest

import synth
from tests.conftest import rel_l2

NAMES = list(synth.TYPE_NAMES.items())
# the types the reference golden outputs exist for: the model path's block formats and dense rows
LINEAR = list(synth.LINEAR_TYPES.items()) + list(synth.DENSE_TYPES.items())


@pytest.mark.parametrize("tid,name", NAMES)
def test_gemv_special_vectors(oracle, tid, name):
    n_rows, n_cols = 12, 1024
    W = synth.make_weights(tid, n_rows, n_cols, seed=40 + tid)
    dec = oracle.dequant_matrix(tid, W, n_cols)
    ones = np.ones(n_cols, np.float32)
    y = oracle.gemv_f64(tid, W, ones, n_cols)
    assert np.array_equal(y, dec.astype(np.float64).sum(axis=1).astype(np.float32)) or \
        rel_l2(y, dec.astype(np.float64).sum(axis=1)) < 1e-7
    for k in (0, 1, 31, 32, 255, 256, 700, n_cols - 1):
        e = np.zeros(n_cols, np.float32)
        e[k] = 1.0
        assert np.array_equal(oracle.gemv_f64(tid, W, e, n_cols), dec[:, k]), (name, k)
        assert np.array_equal(oracle.gemv_f32(tid, W, e, n_cols), dec[:, k]), (name, k)


@pytest.mark.parametrize("tid,name", LINEAR)
def test_gemv_against_numpy_and_reference_golden(oracle, linear_golden, tid, name):
    W, x = linear_golden[name + "_W"], linear_golden["x"]
    n_cols = x.shape[0]
    dec = oracle.dequant_matrix(tid, W, n_cols).astype(np.float64)
    exact = dec @ x.astype(np.float64)
    y64 = oracle.gemv_f64(tid, W, x, n_cols)
    y32 = oracle.gemv_f32(tid, W, x, n_cols)
    assert rel_l2(y64, exact) < 1e-7
    assert rel_l2(y32, exact) < 1e-5
    # same sequential double sum as the reference's oracle mode -> identical bits
    assert np.array_equal(y64.view(np.uint32), linear_golden[name + "_y_f64"].view(np.uint32))
    assert rel_l2(y32, linear_golden[name + "_y_f32"]) < 2e-6
    for nt in (2, 3, 8):
        assert np.array_equal(oracle.gemv_f32(tid, W, x, n_cols, n_threads=nt), y32)


@pytest.mark.parametrize("tid,name", LINEAR)
def test_gemm_tokmajor_equals_per_token_gemv(oracle, linear_golden, tid, name):
    W, X = linear_golden[name + "_W"], linear_golden["X"]
    n_cols = X.shape[1]
    Y64 = oracle.gemm_tokmajor(tid, W, X, n_cols, f64=True)
    Y32 = oracle.gemm_tokmajor(tid, W, X, n_cols, f64=False)
    for t in range(X.shape[0]):
        assert np.array_equal(Y64[t], oracle.gemv_f64(tid, W, X[t], n_cols))
    dec = oracle.dequant_matrix(tid, W, n_cols).astype(np.float64)
    assert rel_l2(Y64, X.astype(np.float64) @ dec.T) < 1e-7
    assert rel_l2(Y32, linear_golden[name + "_Y_tokmajor"]) < 2e-6


@pytest.mark.parametrize("tid,name", LINEAR)
def test_expert_slice_addressing(oracle, linear_golden, tid, name):
    W, x = linear_golden[name + "_W"], linear_golden["x"]
    y = oracle.gemv_f32(tid, W[8:16], x, x.shape[0])
    assert rel_l2(y, linear_golden[name + "_y_expert1"]) < 2e-6


def test_moe_route_invariants(oracle):
    rng = np.random.default_rng(11)
    for trial in range(50):
        n_expert, k = 128, 8
        logits = rng.random(n_expert, dtype=np.float32) * (1 + trial % 5)
        idx, w = oracle.moe_route(logits, k)
        assert abs(float(w.sum()) - 1.0) < 1e-6
        assert set(idx.tolist()) == set(np.argsort(-logits, kind="stable")[:k].tolist())
        sel = logits[idx].astype(np.float64)
        sm = np.exp(sel - sel.max())
        sm /= sm.sum()
        assert np.allclose(w, sm, rtol=2e-6, atol=1e-8)
        assert w[0] == w.min()  # heap order: the root is the smallest survivor


def test_moe_route_ties_follow_the_heap(oracle):
    """Worked by hand from common/transformer.h:4057-4086 with probabilities (0.2, 0.2, 0.6), k = 2: experts 0
    and 1 fill the heap (root 0), expert 2 replaces the root and sinks below expert 1 -> heap (1, 2). A
    selection by index order would keep expert 0."""
    idx, w = oracle.moe_route(np.log(np.array([0.2, 0.2, 0.6], np.float32)), 2)
    assert idx.tolist() == [1, 2]
    assert np.allclose(w, [0.25, 0.75], rtol=1e-6)
    # all equal: nothing ever beats the root, the first k stay, in fill order
    idx, w = oracle.moe_route(np.zeros(10, np.float32), 4)
    assert idx.tolist() == [0, 1, 2, 3] and np.allclose(w, 0.25)
    # four experts (0.1, 0.4, 0.1, 0.4), k = 2: fill (0, 1); expert 2 ties with the root and stays out;
    # expert 3 replaces the root (0.1) and stays on top of the equal 0.4 -> heap (3, 1)
    idx, w = oracle.moe_route(np.log(np.array([0.1, 0.4, 0.1, 0.4], np.float32)), 2)
    assert idx.tolist() == [3, 1] and np.allclose(w, [0.5, 0.5], rtol=1e-6)


def test_moe_ffn_token_against_numpy(oracle):
    tid = synth.GGML_Q4_K
    n_expert, n_embd, n_ff, k = 6, 512, 256, 3
    gate = synth.make_weights(tid, n_expert * n_ff, n_embd, seed=1)
    up = synth.make_weights(tid, n_expert * n_ff, n_embd, seed=2)
    down = synth.make_weights(tid, n_expert * n_embd, n_ff, seed=3)
    x = synth.bf16_bits_to_f32(synth.to_bf16_bits(synth.make_activation(n_embd, seed=4)))
    logits = synth.make_router_logits(1, n_expert, seed=5)[0]
    idx, w = oracle.moe_route(logits, k)
    G = oracle.dequant_matrix(tid, gate, n_embd).astype(np.float64).reshape(n_expert, n_ff, n_embd)
    U = oracle.dequant_matrix(tid, up, n_embd).astype(np.float64).reshape(n_expert, n_ff, n_embd)
    D = oracle.dequant_matrix(tid, down, n_ff).astype(np.float64).reshape(n_expert, n_embd, n_ff)
    want = np.zeros(n_embd)
    for e, we in zip(idx, w):
        g = G[e] @ x.astype(np.float64)
        u = U[e] @ x.astype(np.float64)
        want += float(we) * (D[e] @ (g / (1 + np.exp(-g)) * u))
    got64 = oracle.moe_ffn_token(tid, gate, up, down, n_embd, n_ff, x, idx, w, f64=True)
    got32 = oracle.moe_ffn_token(tid, gate, up, down, n_embd, n_ff, x, idx, w, f64=False)
    assert rel_l2(got64, want) < 1e-6
    assert rel_l2(got32, want) < 1e-5


@pytest.mark.parametrize("label", ["q4k", "q4k_down_q6k"])
def test_moe_block_against_the_compiled_reference(oracle, manifest, linear_golden, label):
    """One token's MoE FFN block as the reference's own compiled pieces compute it (tf_softmax, the heap selection,
    tf_qmatvec_expert three times per expert, tf_silu_mul_avx2, the weighted sum): the oracle's routing gives the same
    experts in the same order, the same weights up to the polynomial exp of the reference's softmax (5e-5; the oracle
    calls expf), and its fp32 and double-precision blocks the same output to 5e-6 (measured 2e-7 .. 8e-7: the exp
    inside the reference's SiLU is a polynomial too)."""
    from tests.conftest import moe_block_case
    c = moe_block_case(manifest, linear_golden, label)
    for t in range(c["logits"].shape[0]):
        idx, w = oracle.moe_route(c["logits"][t], c["top_k"])
        assert np.array_equal(idx, c["idx"][t])
        assert np.allclose(w, c["w"][t], rtol=5e-5, atol=0)
        for f64 in (False, True):
            got = oracle.moe_ffn_token_types(c["types"], c["gate"], c["up"], c["down"], c["n_embd"], c["n_ff"], c["x"][t],
                                             c["idx"][t], c["w"][t], f64=f64)
            assert rel_l2(got, c["out"][t]) <= 5e-6, (label, t, f64)
