"""GPU parity of the block decoders: bit-exact against the CPU oracle and the reference's
golden vectors, through the C ABI. NaN outputs (only reachable from NaN/Inf fp16 scales in the
all-random-bytes cases) are compared bit for bit as well, payload included, for the formats with one
scale per block; for the five formats with two fp16 scales per block the payload of NaN * x - NaN * y
depends on the operand order the compiler picks, so those are compared by position."""
import numpy as np
import pytest

from gemm_amd import qlinear
import synth

pytestmark = pytest.mark.gpu
NAMES = list(synth.TYPE_NAMES.items())


TWO_SCALES = {"q4_K", "q5_K", "q2_K", "q4_1", "q5_1"}


def assert_same_bits(got, want, what=""):
    got = np.ascontiguousarray(got, np.float32)
    want = np.ascontiguousarray(want, np.float32)
    assert got.shape == want.shape
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan), what + ": NaN positions differ"
    if what.split(" ")[0] not in TWO_SCALES:
        nan = np.zeros_like(nan)  # payloads count too
    g, w = got.view(np.uint32)[~nan], want.view(np.uint32)[~nan]
    bad = np.flatnonzero(g != w)
    assert bad.size == 0, "%s: %d of %d values differ, first at %d: %08x vs %08x" % (
        what, bad.size, g.size, bad[0], g[bad[0]], w[bad[0]])


def test_device_is_gfx950():
    name, cu, mem = qlinear.device_info()
    print("device:", name, cu, "CUs", mem >> 30, "GiB")
    assert "gfx950" in name
    assert cu >= 200


def test_fp16_exhaustive_bit_exact(oracle):
    halves = np.arange(65536, dtype=np.uint16)
    rc, got = qlinear.dequant_row(synth.GGML_F16, halves.view(np.uint8), 65536)
    assert rc == 0
    want = oracle.fp16_table()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))  # every bit, NaN payloads included


@pytest.mark.parametrize("tid,name", NAMES)
def test_decoder_matches_reference_golden(codec_golden, tid, name):
    src = codec_golden[name + "_src"]
    want = codec_golden[name + "_f32bits"].view(np.float32)
    for r in range(src.shape[0]):
        rc, got = qlinear.dequant_row(tid, src[r], want.shape[1])
        assert rc == 0
        assert_same_bits(got, want[r], "%s row %d" % (name, r))
    # the void entry points that mirror dequantize_row_<type>
    lib = qlinear.load()
    dst = np.zeros(want.shape[1], np.float32)
    getattr(lib, "qlin_dequantize_row_" + name)(src[0].ctypes.data, dst.ctypes.data, want.shape[1])
    assert_same_bits(dst, want[0], name + " void entry")


@pytest.mark.parametrize("tid,name", NAMES)
@pytest.mark.parametrize("wild", [False, True])
def test_decoder_matches_oracle_sweep(oracle, tid, name, wild):
    n_rows, n_cols = 96, 4096
    W = synth.make_weights(tid, n_rows, n_cols, seed=600 + tid, wild=wild)
    got = qlinear.dequant_rows(tid, W, n_rows, n_cols)
    assert_same_bits(got, oracle.dequant_matrix(tid, W, n_cols), name)


@pytest.mark.parametrize("tid,name", NAMES)
def test_ragged_tail_and_empty(oracle, tid, name):
    be, bb = synth.BLOCK_GEOMETRY[tid]
    W = synth.make_weights(tid, 1, 3 * be, seed=9)[0]
    sentinel = np.full(3 * be - 1, -123.0, np.float32)
    rc, got = qlinear.dequant_row(tid, W, 3 * be - 1, dst=sentinel.copy())
    assert rc == 0
    _, want = oracle.dequant_row(tid, W, 2 * be)
    assert_same_bits(got[:2 * be], want, name)
    assert np.all(got[2 * be:] == -123.0)  # the undecoded tail is left untouched
    rc, got = qlinear.dequant_row(tid, W, 0)
    assert rc == 0 and got.size == 0
    rc, got = qlinear.dequant_row(tid, W, be - 1, dst=np.full(be - 1, 7.0, np.float32))
    assert rc == 0 and np.all(got == 7.0)


def test_unknown_type_and_plain_types(oracle):
    rc, _ = qlinear.dequant_row(99, np.zeros(64, np.uint8), 32)
    assert rc == qlinear.ERR_TYPE == -1
    assert "99" in qlinear.load().qlin_last_error().decode()
    f = synth.make_activation(1000, seed=1)
    rc, y = qlinear.dequant_row(synth.GGML_F32, f.view(np.uint8), 1000)
    assert rc == 0 and np.array_equal(y, f)
    b = synth.to_bf16_bits(f)
    rc, y = qlinear.dequant_row(synth.GGML_BF16, b.view(np.uint8), 1000)
    assert rc == 0 and np.array_equal(y, synth.bf16_bits_to_f32(b))


@pytest.mark.parametrize("tid,name", NAMES)
def test_device_resident_decode(oracle, tid, name):
    n_rows, n_cols = 257, 2048
    W = synth.make_weights(tid, n_rows, n_cols, seed=700 + tid)
    dW = qlinear.DevBuf.from_numpy(W)
    dO = qlinear.DevBuf(n_rows * n_cols * 4)
    qlinear.dequant_dev(tid, dW, dO, n_rows, n_cols)
    qlinear.sync()
    assert_same_bits(dO.to_numpy(np.float32, (n_rows, n_cols)), oracle.dequant_matrix(tid, W, n_cols), name)


def test_full_size_q4k_decode_properties(oracle):
    """14336 x 4096 (the decode-shape weight): every sub-block's decoded range must sit inside
    [-dmin*m, d*sc*15 - dmin*m], and a random sample of rows must match the oracle bit for bit."""
    n_rows, n_cols = 14336, 4096
    W = synth.make_weights(synth.GGML_Q4_K, n_rows, n_cols, seed=12)
    dW = qlinear.DevBuf.from_numpy(W)
    dO = qlinear.DevBuf(n_rows * n_cols * 4)
    qlinear.dequant_dev(synth.GGML_Q4_K, dW, dO, n_rows, n_cols)
    qlinear.sync()
    out = dO.to_numpy(np.float32, (n_rows, n_cols))
    rows = np.random.default_rng(0).choice(n_rows, 64, replace=False)
    assert_same_bits(out[rows], oracle.dequant_matrix(synth.GGML_Q4_K, W[rows], n_cols), "q4_K sampled rows")
    blocks = W.reshape(n_rows, n_cols // 256, 144)
    d = blocks[..., 0:2].copy().view(np.float16)[..., 0].astype(np.float32)
    dmin = blocks[..., 2:4].copy().view(np.float16)[..., 0].astype(np.float32)
    hi = (d * 63 * 15)[..., None]
    lo = (-dmin * 63)[..., None]
    o = out.reshape(n_rows, n_cols // 256, 256)
    assert np.all(o <= hi + 1e-6) and np.all(o >= lo - 1e-6)


@pytest.mark.parametrize("tid,name", NAMES + list(synth.DENSE_TYPES.items()))
def test_embedding_lookup_by_device_resident_ids(oracle, tid, name):
    """rows picked by a list of ids, decoded bit-exactly; an id outside the table gives zeros"""
    n_vocab, n_cols = 300, 1024
    W = synth.make_weights(tid, n_vocab, n_cols, seed=800 + tid)
    ids = np.array([5, 299, 0, 5, -1, 300, 123], np.int32)
    dW, dI = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(ids)
    dO = qlinear.DevBuf(ids.size * n_cols * 4)
    qlinear.embed_rows_dev(tid, dW, n_vocab, dI, ids.size, dO, n_cols)
    qlinear.sync()
    got = dO.to_numpy(np.float32, (ids.size, n_cols))
    dec = oracle.dequant_matrix(tid, W, n_cols)
    for i, t in enumerate(ids):
        want = dec[t] if 0 <= t < n_vocab else np.zeros(n_cols, np.float32)
        assert_same_bits(got[i], want, "%s id %d" % (name, t))
