"""GPU parity of the grouped MoE expert FFN (Q4_K experts, bf16 activations), through the C ABI.

The reference computes, per token, sum_k w_k * down_e(silu(gate_e x) * up_e x) with fp32 matvecs
over decoded rows (common/transformer.h:4093-4128). The checks here use
  * the CPU oracle's per-token function with double accumulation on the same bf16-rounded x and
    the same (idx, w), and
  * for the full-size case, a numpy float64 restatement over oracle-decoded expert matrices.
Contract: relative L2 <= 2e-3. The kernel keeps the weights exact and carries the intermediate
activation as a bf16 head + tail, so it is held to 2e-5 here.
"""
import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests.conftest import rel_l2

pytestmark = pytest.mark.gpu
Q4K = synth.GGML_Q4_K
CONTRACT, DESIGNED = 2e-3, 2e-5
ALL_NAMES = dict(synth.TYPE_NAMES)
ALL_NAMES.update(synth.DENSE_TYPES)


def make_experts(n_expert, n_embd, n_ff, seed, types=(Q4K, Q4K, Q4K)):
    gate = synth.make_weights(types[0], n_expert * n_ff, n_embd, seed=seed)
    up = synth.make_weights(types[1], n_expert * n_ff, n_embd, seed=seed + 1)
    down = synth.make_weights(types[2], n_expert * n_embd, n_ff, seed=seed + 2)
    return gate, up, down


def run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert, fill=-7.0, types=None):
    n_tok, top_k = idx.shape
    bufs = [qlinear.DevBuf.from_numpy(a) for a in (gate, up, down, Xb, idx.astype(np.int32), w.astype(np.float32))]
    out0 = np.full((max(n_tok, 1), n_embd), fill, np.float32)
    dout = qlinear.DevBuf.from_numpy(out0)
    nws = qlinear.moe_workspace_bytes(n_tok, top_k, n_embd, n_ff, n_expert)
    dws = qlinear.DevBuf(max(nws, 256))
    if types is None:
        qlinear.moe_ffn_dev(Q4K, *bufs, dout, n_tok, top_k, n_embd, n_ff, n_expert, dws)
    else:
        qlinear.moe_ffn_types_dev(types, *bufs, dout, n_tok, top_k, n_embd, n_ff, n_expert, dws)
    qlinear.sync()
    out = dout.to_numpy(np.float32, out0.shape)[:n_tok]
    for b in bufs + [dout, dws]:
        b.free()
    return out


def route(oracle, logits, top_k):
    idx = np.zeros((logits.shape[0], top_k), np.int32)
    w = np.zeros((logits.shape[0], top_k), np.float32)
    for t in range(logits.shape[0]):
        idx[t], w[t] = oracle.moe_route(logits[t], top_k)
    return idx, w


def oracle_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff):
    X = synth.bf16_bits_to_f32(Xb)
    return np.stack([oracle.moe_ffn_token(Q4K, gate, up, down, n_embd, n_ff, X[t], idx[t], w[t], f64=True)
                     for t in range(X.shape[0])])


def numpy_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff, types=(Q4K, Q4K, Q4K)):
    """float64 restatement grouped by expert: decode each routed expert once."""
    X = synth.bf16_bits_to_f32(Xb).astype(np.float64)
    out = np.zeros((X.shape[0], n_embd), np.float64)
    gb, ub, db = synth.row_bytes(types[0], n_embd), synth.row_bytes(types[1], n_embd), synth.row_bytes(types[2], n_ff)
    for e in np.unique(idx):
        if e < 0:
            continue
        G = oracle.dequant_matrix(types[0], gate[e * n_ff:(e + 1) * n_ff].reshape(n_ff, gb), n_embd).astype(np.float64)
        U = oracle.dequant_matrix(types[1], up[e * n_ff:(e + 1) * n_ff].reshape(n_ff, ub), n_embd).astype(np.float64)
        D = oracle.dequant_matrix(types[2], down[e * n_embd:(e + 1) * n_embd].reshape(n_embd, db), n_ff).astype(np.float64)
        toks, ks = np.nonzero(idx == e)
        g, u = X[toks] @ G.T, X[toks] @ U.T
        with np.errstate(over="ignore"):  # exp(-g) -> inf gives h -> 0, as in fp32
            h = g / (1.0 + np.exp(-g)) * u
        np.add.at(out, toks, w[toks, ks].astype(np.float64)[:, None] * (h @ D.T))  # a token may name an expert twice
    return out


@pytest.mark.parametrize("n_tok", [1, 5, 40, 100])
def test_grouped_ffn_small(oracle, n_tok):
    n_expert, n_embd, n_ff, k = 16, 512, 256, 4
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=300)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=310 + n_tok, tokens=n_tok))
    idx, w = route(oracle, synth.make_router_logits(n_tok, n_expert, seed=320 + n_tok), k)
    got = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert)
    want = oracle_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff)
    err = rel_l2(got, want)
    assert err <= DESIGNED, err
    assert err <= CONTRACT
    # per-token as well: no token may hide behind the others
    for t in range(n_tok):
        assert rel_l2(got[t], want[t]) <= 10 * DESIGNED, t
    assert rel_l2(numpy_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff), want) <= 1e-6


@pytest.mark.parametrize("n_tok", [1, 2, 3, 8, 9])
def test_few_tokens_many_experts(oracle, n_tok):
    """one to eight tokens over 64 experts, top-4: each token goes through the matvec kernels on its own (nine tokens:
    the grouped kernels); one expert twice in a token, an index out of range, and the same bits on a second run"""
    n_expert, n_embd, n_ff, k = 64, 512, 768, 4
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=900)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=910 + n_tok, tokens=n_tok))
    idx, w = route(oracle, synth.make_router_logits(n_tok, n_expert, seed=920 + n_tok), k)
    got = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert)
    want = oracle_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff)
    for t in range(n_tok):
        assert rel_l2(got[t], want[t]) <= DESIGNED, t
    assert np.array_equal(run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert), got)
    idx2, w2 = idx.copy(), w.copy()
    idx2[0, 1] = idx2[0, 0]  # the same expert twice: its output counts with both weights
    idx2[-1, 2] = n_expert + 5  # out of range: contributes nothing
    got2 = run_ffn(gate, up, down, Xb, idx2, w2, n_embd, n_ff, n_expert)
    w3 = w2.copy()
    w3[-1, 2] = 0.0
    idx3 = idx2.copy()
    idx3[-1, 2] = 0
    want2 = oracle_ffn(oracle, gate, up, down, Xb, idx3, w3, n_embd, n_ff)
    for t in range(n_tok):
        assert rel_l2(got2[t], want2[t]) <= DESIGNED, t


Q6K, Q5K = synth.GGML_Q6_K, synth.GGML_Q5_K
FEW_TOKEN_TYPES = [(Q4K, Q4K, Q6K), (Q6K, Q6K, Q6K), (Q5K, Q5K, Q6K), (synth.GGML_Q8_0,) * 3, (synth.GGML_IQ4_XS,) * 3,
                   (synth.GGML_MXFP4,) * 3, (synth.GGML_Q3_K, synth.GGML_Q3_K, Q4K), (synth.GGML_Q2_K,) * 3,
                   (synth.GGML_IQ4_NL, synth.GGML_IQ4_NL, synth.GGML_Q4_0), (synth.GGML_IQ2_XXS,) * 3,
                   (synth.GGML_IQ2_XS, synth.GGML_IQ2_XS, synth.GGML_IQ3_S), (synth.GGML_IQ3_XXS, synth.GGML_IQ3_XXS, synth.GGML_IQ2_S),
                   (synth.GGML_TQ2_0, synth.GGML_TQ2_0, synth.GGML_Q1_0), (synth.GGML_Q5_0, synth.GGML_Q5_0, synth.GGML_Q5_1),
                   (synth.GGML_NVFP4, synth.GGML_NVFP4, synth.GGML_Q4_1), (synth.GGML_IQ1_S, synth.GGML_IQ1_S, synth.GGML_IQ1_M), (Q4K, Q6K, Q4K)]


@pytest.mark.parametrize("n_tok", [1, 3, 8])
@pytest.mark.parametrize("types", FEW_TOKEN_TYPES, ids=lambda t: "-".join(ALL_NAMES[x] for x in t))
def test_few_tokens_other_expert_formats(oracle, types, n_tok):
    """the same route with the experts in the formats of the matrix-instruction matvec, gate/up and down of different
    types (the last case, gate and up of different types, keeps the grouped kernels); a repeated expert and an index
    out of range as above"""
    n_expert, n_embd, n_ff, k = 64, 512, 768, 4
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=950, types=types)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=960 + n_tok, tokens=n_tok))
    idx, w = route(oracle, synth.make_router_logits(n_tok, n_expert, seed=970 + n_tok), k)
    idx[0, 1] = idx[0, 0]
    got = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert, types=types)
    want = numpy_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff, types=types)
    for t in range(n_tok):
        assert rel_l2(got[t], want[t]) <= DESIGNED, t
    idx2 = idx.copy()
    idx2[-1, 2] = -3
    w0 = w.copy()
    w0[-1, 2] = 0.0
    dropped = run_ffn(gate, up, down, Xb, idx2, w, n_embd, n_ff, n_expert, types=types)
    zeroed = run_ffn(gate, up, down, Xb, idx, w0, n_embd, n_ff, n_expert, types=types)
    assert rel_l2(dropped, zeroed) <= 1e-7
    assert np.array_equal(run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert, types=types), got)


@pytest.mark.parametrize("types", [(Q4K, Q4K, Q4K), (Q4K, Q4K, Q6K), (Q6K, Q6K, Q4K)], ids=["q4k", "q4k_q4k_q6k", "q6k_q6k_q4k"])
def test_one_token_wide_experts(oracle, types):
    """one token, top-2 of 8 experts with 8704-column down projections (a Mixtral-like shape, scaled): the down step
    is a row of 68 super-blocks - more than the matrix-instruction kernel takes per launch, so a Q6_K down runs as
    two ranges of that row, the second adding; a Q4_K down walks the row in one launch"""
    n_expert, n_embd, n_ff, k, n_tok = 8, 1024, 8704, 2, 1
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=980, types=types)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=981, tokens=n_tok) * np.float32(0.05))
    idx, w = route(oracle, synth.make_router_logits(n_tok, n_expert, seed=982), k)
    got = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert, types=types)
    want = numpy_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff, types=types)
    assert rel_l2(got, want) <= DESIGNED


def test_grouped_ffn_all_tokens_one_expert(oracle):
    """37 tokens on one expert: three passes of 16 token slots, the last one ragged."""
    n_expert, n_embd, n_ff, k, n_tok = 8, 256, 256, 2, 37
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=400)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=401, tokens=n_tok))
    idx = np.tile(np.array([[5, 2]], np.int32), (n_tok, 1))
    w = np.tile(np.array([[0.75, 0.25]], np.float32), (n_tok, 1))
    got = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert)
    want = oracle_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff)
    assert rel_l2(got, want) <= DESIGNED


def test_grouped_ffn_linearity_and_bad_index(oracle):
    """A pair whose expert index is out of range contributes nothing; weights enter linearly."""
    n_expert, n_embd, n_ff, k, n_tok = 8, 256, 256, 3, 9
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=500)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=501, tokens=n_tok))
    idx, w = route(oracle, synth.make_router_logits(n_tok, n_expert, seed=502), k)
    full = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert)
    idx2 = idx.copy()
    idx2[:, 1] = np.where(np.arange(n_tok) % 2 == 0, -1, n_expert + 3)
    w0 = w.copy()
    w0[:, 1] = 0.0
    dropped = run_ffn(gate, up, down, Xb, idx2, w, n_embd, n_ff, n_expert)
    zeroed = run_ffn(gate, up, down, Xb, idx, w0, n_embd, n_ff, n_expert)
    assert np.array_equal(dropped, zeroed + 0.0) or rel_l2(dropped, zeroed) <= 1e-7
    assert rel_l2(run_ffn(gate, up, down, Xb, idx, 2.0 * w, n_embd, n_ff, n_expert), 2.0 * full) <= 1e-7
    assert np.array_equal(run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert), full)  # deterministic


def test_grouped_ffn_zero_tokens():
    n_expert, n_embd, n_ff, k = 4, 256, 256, 2
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=600)
    out = run_ffn(gate, up, down, np.zeros((1, n_embd), np.uint16), np.zeros((0, k), np.int32),
                  np.zeros((0, k), np.float32), n_embd, n_ff, n_expert)
    assert out.shape == (0, n_embd)


def test_grouped_ffn_rejects_other_types_and_shapes():
    lib = qlinear.load()
    d = qlinear.DevBuf(4096)
    p = d.ptr
    assert lib.qlin_moe_ffn_dev(9, p, p, p, p, p, p, p, 1, 1, 256, 256, 2, p, None) == qlinear.ERR_TYPE
    assert lib.qlin_moe_ffn_types_dev(Q4K, Q4K, 9, p, p, p, p, p, p, p, 1, 1, 256, 256, 2, p, None) == qlinear.ERR_TYPE
    assert lib.qlin_moe_ffn_types_dev(Q4K, Q4K, synth.GGML_Q8_0, p, p, p, p, p, p, p, 1, 1, 256, 250, 2, p, None) == qlinear.ERR_ARG
    assert lib.qlin_moe_ffn_dev(Q4K, p, p, p, p, p, p, p, 1, 1, 250, 256, 2, p, None) == qlinear.ERR_ARG
    assert lib.qlin_moe_ffn_dev(Q4K, p, p, p, p, p, p, p, 1, 3, 256, 256, 2, p, None) == qlinear.ERR_ARG
    assert lib.qlin_moe_ffn_dev(Q4K, p, p, p, p, p, p, p, 1, 1, 256, 256, 2, None, None) == qlinear.ERR_ARG
    d.free()


def test_grouped_ffn_full_size(oracle):
    """128 experts of gate/up 768x2048 and down 2048x768, 64 tokens, top-8 (the MoE benchmark shape)."""
    n_expert, n_embd, n_ff, k, n_tok = 128, 2048, 768, 8, 64
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=700)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=701, tokens=n_tok))
    logits = synth.make_router_logits(n_tok, n_expert, seed=702)
    # route on the device, as a caller would, and check it against the oracle's routing
    dl = qlinear.DevBuf.from_numpy(logits)
    di, dw = qlinear.DevBuf(n_tok * k * 4), qlinear.DevBuf(n_tok * k * 4)
    qlinear.moe_route_dev(dl, n_tok, n_expert, k, di, dw)
    qlinear.sync()
    idx, w = di.to_numpy(np.int32, (n_tok, k)), dw.to_numpy(np.float32, (n_tok, k))
    oi, ow = route(oracle, logits, k)
    assert np.array_equal(np.sort(idx, axis=1), np.sort(oi, axis=1))
    assert np.allclose(np.sort(w, axis=1), np.sort(ow, axis=1), rtol=1e-5)
    got = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert)
    want = numpy_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff)
    err = rel_l2(got, want)
    assert err <= DESIGNED, err
    for t in (0, 17, 63):  # the per-token oracle on a few tokens ties the numpy restatement to it
        one = oracle.moe_ffn_token(Q4K, gate, up, down, n_embd, n_ff, synth.bf16_bits_to_f32(Xb[t]), idx[t], w[t], f64=True)
        assert rel_l2(want[t], one) <= 1e-6
        assert rel_l2(got[t], one) <= 10 * DESIGNED


Q6K, Q8_0 = synth.GGML_Q6_K, synth.GGML_Q8_0


@pytest.mark.parametrize("types", [
    (Q4K, Q4K, Q6K),                                    # what K-quant mixes store for part of the layers
    (Q6K, Q6K, Q6K), (Q8_0, Q8_0, Q8_0), (Q4K, Q6K, Q4K),
    (synth.GGML_IQ4_NL, synth.GGML_IQ4_NL, synth.GGML_Q5_K), (synth.GGML_BF16, synth.GGML_F16, synth.GGML_F32),
    (synth.GGML_IQ2_XXS, synth.GGML_IQ3_S, synth.GGML_Q4_0),
], ids=lambda t: "-".join(ALL_NAMES[x] for x in t))
@pytest.mark.parametrize("n_tok", [3, 40])
def test_grouped_ffn_other_and_mixed_formats(oracle, types, n_tok):
    n_expert, n_embd, n_ff, k = 8, 512, 256, 3
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=700, types=types)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=710 + n_tok, tokens=n_tok))
    idx, w = route(oracle, synth.make_router_logits(n_tok, n_expert, seed=720 + n_tok), k)
    got = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert, types=types)
    want = numpy_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff, types=types)
    err = rel_l2(got, want)
    assert err <= DESIGNED, (err, types)
    for t in range(n_tok):
        assert rel_l2(got[t], want[t]) <= 10 * DESIGNED, t


@pytest.mark.parametrize("type_id", sorted(synth.TYPE_NAMES), ids=lambda t: ALL_NAMES[t])
def test_grouped_ffn_every_block_format(oracle, type_id):
    """all three expert tensors in each of the 24 block formats (Q4_K: the matrix-core kernels; every other
    format: the any-format kernel with that format's codec)"""
    types = (type_id, type_id, type_id)
    n_expert, n_embd, n_ff, k, n_tok = 4, 512, 256, 2, 11
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=900 + type_id, types=types)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=901, tokens=n_tok))
    idx, w = route(oracle, synth.make_router_logits(n_tok, n_expert, seed=902), k)
    got = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert, types=types)
    want = numpy_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff, types=types)
    assert rel_l2(got, want) <= DESIGNED, ALL_NAMES[type_id]


@pytest.mark.parametrize("types,n_embd,n_ff", [
    ((Q4K, Q4K, Q4K), 256, 2304),      # 9 super-blocks of K for down: more than its 8 waves, one row group per workgroup
    ((Q8_0, Q8_0, Q4K), 160, 256),     # 160 rows of down: not a whole number of the four-group walks
    ((Q4K, Q4K, Q4K), 1024, 512),      # the walk: 8 groups of 4 x 32 rows, two super-blocks of K
    ((Q4K, Q4K, Q6K), 256, 768),       # Q6_K down on the matrix cores: 630-byte rows, three waves, blocks at every even offset
    ((Q4K, Q4K, Q6K), 1024, 512),      # 420-byte rows, two waves, eight walks per expert
    ((Q8_0, Q8_0, Q6K), 160, 256),     # rows not a multiple of 128: the any-format kernel
    ((Q6K, Q6K, Q6K), 2048, 256),      # Q6_K gate and up: four waves, two super-blocks each, 1680-byte rows
    ((Q6K, Q6K, Q4K), 768, 512),       # three waves, 630-byte rows; 48 rows of gate/up per expert... and Q4_K down
    ((synth.GGML_Q5_K, synth.GGML_Q5_K, Q6K), 1024, 768),   # what the 5-bit K-quant mixes store
    ((synth.GGML_Q5_K, synth.GGML_Q5_K, synth.GGML_Q5_K), 2048, 512),
    ((Q8_0, Q8_0, Q8_0), 1024, 768),
    ((synth.GGML_Q3_K, synth.GGML_Q3_K, Q4K), 1024, 512),   # the 3-bit mixes
    ((synth.GGML_Q3_K, synth.GGML_Q3_K, synth.GGML_Q3_K), 768, 768),
    ((synth.GGML_Q2_K, synth.GGML_Q2_K, synth.GGML_Q3_K), 1024, 512),
    ((synth.GGML_Q2_K, synth.GGML_Q2_K, synth.GGML_Q2_K), 768, 768),
    ((Q4K, Q4K, Q6K), 256, 2304),      # Q6_K down with nine super-blocks of K: the 16-row kernel that loops over K
    ((Q8_0, Q8_0, Q8_0), 256, 4096),   # sixteen super-blocks over four waves
    ((synth.GGML_Q5_K, synth.GGML_Q5_K, synth.GGML_Q5_K), 512, 2560),
    ((synth.GGML_Q3_K, synth.GGML_Q3_K, synth.GGML_Q3_K), 256, 2304),
    ((synth.GGML_Q2_K, synth.GGML_Q2_K, synth.GGML_Q2_K), 256, 2816),
], ids=["long_k", "rows_not_multiple_of_128", "walk", "q6k_down_3_waves", "q6k_down_2_waves", "q6k_down_fallback",
        "q6k_gate_up_4_waves", "q6k_gate_up_3_waves", "q5k_q5k_q6k", "q5k", "q8_0", "q3k_q3k_q4k", "q3k", "q2k_q2k_q3k", "q2k",
        "q6k_down_long_k", "q8_0_long_k", "q5k_long_k", "q3k_long_k", "q2k_long_k"])
def test_grouped_ffn_down_kernel_variants(oracle, types, n_embd, n_ff):
    """the Q4_K down projection has two kernels: one row group of 32 per workgroup, and a walk over four
    groups with the next weight image in flight (K up to 2048, rows a multiple of 128); Q6_K down has a walk of
    its own (eight tokens per pass: 21 tokens over 3 experts give it several) and the any-format kernel"""
    n_expert, k, n_tok = 3, 2, 21
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=950, types=types)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=951, tokens=n_tok))
    idx, w = route(oracle, synth.make_router_logits(n_tok, n_expert, seed=952), k)
    got = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert, types=types)
    want = numpy_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff, types=types)
    assert rel_l2(got, want) <= DESIGNED
    for t in range(n_tok):
        assert rel_l2(got[t], want[t]) <= 10 * DESIGNED, t


@pytest.mark.parametrize("types", [(Q4K, Q4K, Q4K), (Q4K, Q4K, Q6K), (Q6K, Q6K, Q6K), (Q8_0, Q8_0, Q8_0)],
                         ids=["q4k", "q4k_q4k_q6k", "q6k", "q8_0"])
@pytest.mark.parametrize("n_tok", [1, 2, 7, 8, 9, 17])
def test_grouped_ffn_fewer_pairs_than_experts(oracle, types, n_tok):
    """32 experts, top-4: up to two pairs per expert (16 tokens) the expert kernels look their expert up in the list
    of routed ones and the launch covers no more experts than pairs; 17 tokens take the launch over all experts.
    One and two tokens also take the 32-row down kernel instead of the walk."""
    n_expert, n_embd, n_ff, k = 32, 512, 256, 4
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=970, types=types)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=971 + n_tok, tokens=n_tok))
    idx, w = route(oracle, synth.make_router_logits(n_tok, n_expert, seed=972 + n_tok), k)
    got = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert, types=types)
    want = numpy_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff, types=types)
    assert rel_l2(got, want) <= DESIGNED
    for t in range(n_tok):
        assert rel_l2(got[t], want[t]) <= 10 * DESIGNED, t
    # the highest and the lowest expert routed, everything between unused
    idx2 = np.tile(np.array([[n_expert - 1, 0, 5, 6]], np.int32), (n_tok, 1))
    got2 = run_ffn(gate, up, down, Xb, idx2, w, n_embd, n_ff, n_expert, types=types)
    assert rel_l2(got2, numpy_ffn(oracle, gate, up, down, Xb, idx2, w, n_embd, n_ff, types=types)) <= DESIGNED


def test_grouped_ffn_mixed_formats_many_tokens_per_expert_and_ragged_shapes(oracle):
    """two experts, 50 tokens: 8-token passes of the any-format kernel with a ragged tail; n_ff = 96 is not a
    multiple of the matrix-core tiles, so Q4_K gate/up cannot be used and Q8_0 (32-element blocks) is"""
    types = (Q8_0, Q8_0, Q8_0)
    n_expert, n_embd, n_ff, k, n_tok = 2, 160, 96, 2, 50
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=800, types=types)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=801, tokens=n_tok))
    idx = np.tile(np.array([[1, 0]], np.int32), (n_tok, 1))
    w = np.tile(np.array([[0.6, 0.4]], np.float32), (n_tok, 1))
    got = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert, types=types)
    want = numpy_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff, types=types)
    assert rel_l2(got, want) <= DESIGNED


def test_experts_with_chosen_token_counts_and_repeatability(oracle):
    """Experts that see exactly 1, 4, 5, 16, 17 and 33 tokens (and some that see none): the kernels switch form
    at four tokens, walk tiles of sixteen, and find the first sixteen tokens of an expert in its record and the rest
    in the sorted list. The slots inside an expert are handed out by atomics, so the call is also repeated: the
    result may not depend on the order they came in."""
    n_expert, n_embd, n_ff, top_k = 12, 512, 256, 2
    counts = {0: 1, 2: 4, 3: 5, 5: 16, 6: 17, 9: 33}
    pairs = [e for e, c in counts.items() for _ in range(c)]  # sorted by expert; no expert holds half of them
    rng = np.random.default_rng(7)
    n_tok = len(pairs) // top_k
    assert n_tok * top_k == len(pairs)
    # token t gets entries t and t + n_tok of the sorted list: two different experts, as a router would give
    idx = np.stack([np.array(pairs[:n_tok], np.int32), np.array(pairs[n_tok:], np.int32)], axis=1)
    idx = idx[rng.permutation(n_tok)]
    assert np.all(idx[:, 0] != idx[:, 1])
    w = rng.random((n_tok, top_k), dtype=np.float32) + 0.25
    gate, up, down = make_experts(n_expert, n_embd, n_ff, seed=300)
    Xb = synth.to_bf16_bits(synth.make_activation(n_embd, seed=303, tokens=n_tok))
    want = numpy_ffn(oracle, gate, up, down, Xb, idx, w, n_embd, n_ff)
    first = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert)
    assert rel_l2(first, want) <= DESIGNED
    for _ in range(3):
        again = run_ffn(gate, up, down, Xb, idx, w, n_embd, n_ff, n_expert)
        assert np.array_equal(first.view(np.uint32), again.view(np.uint32))
