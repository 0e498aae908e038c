"""GPU parity of the prefill GEMM for every weight format (decode once to bf16, then the dense
matrix-core GEMM), through the C ABI. Two bars, as for the fused Q4_K kernel: relative L2 <= 2e-3 against
the oracle's exact decoded weights, and <= 2e-5 against the same weights rounded to bf16 (nearest even),
which is what the path is designed to compute."""
import ctypes as C

import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests.conftest import rel_l2

pytestmark = pytest.mark.gpu
Q4K = synth.GGML_Q4_K
ALL = dict(synth.TYPE_NAMES)
ALL.update(synth.DENSE_TYPES)


def run(tid, W, Xb, n_rows, n_cols, n_tok, ldx=None, ldy=None, ws=None):
    ldx, ldy = ldx or n_cols, ldy or n_rows
    Xpad = np.zeros((n_tok, ldx), np.uint16)
    Xpad[:, :n_cols] = Xb
    dW, dX = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(Xpad)
    dY = qlinear.DevBuf.from_numpy(np.full((n_tok, ldy), -3.0, np.float32))
    dws = ws or qlinear.DevBuf(qlinear.gemm_bf16_any_workspace_bytes(n_rows, n_cols))
    qlinear.gemm_bf16_any_dev(tid, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy, dws)
    qlinear.sync()
    Y = dY.to_numpy(np.float32, (n_tok, ldy))
    for b in (dW, dX, dY) + (() if ws else (dws,)):
        b.free()
    return Y


@pytest.fixture(params=["vendor", "own"])
def dense_kernel(request):
    """both dense bf16 products behind qlin_gemm_bf16_any_dev: the vendor library's (default) and this
    library's own tile kernel"""
    qlinear.check(qlinear.load().qlin_set_dense_gemm_own(1 if request.param == "own" else 0))
    yield request.param
    qlinear.check(qlinear.load().qlin_set_dense_gemm_own(0))


FUSED = [Q4K, synth.GGML_Q5_K, synth.GGML_Q6_K, synth.GGML_Q8_0, synth.GGML_IQ4_NL, synth.GGML_IQ4_XS,
         synth.GGML_Q4_0, synth.GGML_Q2_K, synth.GGML_Q3_K]  # decoded inside the tile kernels
FEW = 32  # tokens up to which Q4_K takes its few-token kernel
KQ = {synth.GGML_Q6_K, synth.GGML_Q5_K, synth.GGML_Q3_K, synth.GGML_Q2_K, synth.GGML_Q8_0}


def streams_exact_weights(tid, n_tok, n_rows, n_cols):
    """few tokens of these formats go through a kernel that multiplies the unrounded weights; up to four tokens of any
    other block format (Q4_K has its own route) go through the matvec"""
    if tid in KQ and n_tok <= 24 and n_cols % 256 == 0 and n_rows * synth.row_bytes(tid, n_cols) % 16 == 0:
        return True
    return n_tok <= 4 and tid not in synth.DENSE_TYPES and tid != synth.GGML_Q4_K


def references(oracle, tid, W, Xb, n_cols):
    dec = oracle.dequant_matrix(tid, W, n_cols)
    Xf = synth.bf16_bits_to_f32(Xb).astype(np.float64)
    exact = Xf @ dec.astype(np.float64).T
    designed = Xf @ synth.bf16_bits_to_f32(synth.to_bf16_bits(dec)).astype(np.float64).T
    return exact, designed


@pytest.mark.parametrize("tid", sorted(ALL), ids=lambda t: ALL[t])
def test_every_format(oracle, tid, dense_kernel):
    n_tok, n_rows, n_cols = 72, 160, 512
    W = synth.make_weights(tid, n_rows, n_cols, seed=500 + tid)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=600 + tid, tokens=n_tok))
    Y = run(tid, W, Xb, n_rows, n_cols, n_tok)
    exact, designed = references(oracle, tid, W, Xb, n_cols)
    assert rel_l2(Y, designed) <= 2e-5, ALL[tid]
    # F32 weights carry 24 significant bits, everything else at most 11 + a few: rounding to bf16 is 2^-9 each
    assert rel_l2(Y, exact) <= 3e-3, ALL[tid]


@pytest.mark.parametrize("tid,n_tok,n_rows,n_cols", [
    (synth.GGML_Q6_K, 1, 16, 256), (synth.GGML_Q6_K, 515, 1000, 1024), (synth.GGML_Q8_0, 130, 257, 96),
    (synth.GGML_Q5_K, 64, 2048, 768), (synth.GGML_IQ4_NL, 200, 130, 4096), (Q4K, 513, 384, 512),
    # enough tiles for the fused kernel, but more tokens than it keeps when there is a workspace to decode into
    (synth.GGML_Q6_K, 1030, 5130, 512), (synth.GGML_Q8_0, 770, 8200, 256),
    (Q4K, 1100, 300, 256), (Q4K, 300, 25700, 256), (synth.GGML_BF16, 33, 100, 264), (synth.GGML_F16, 300, 64, 1000),
    (synth.GGML_BF16, 700, 3000, 1024), (synth.GGML_Q6_K, 257, 129, 2048), (synth.GGML_Q8_0, 100, 4100, 512),
])
def test_shapes(oracle, tid, n_tok, n_rows, n_cols, dense_kernel):
    W = synth.make_weights(tid, n_rows, n_cols, seed=n_rows + n_tok)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=n_cols + n_tok, tokens=n_tok))
    Y = run(tid, W, Xb, n_rows, n_cols, n_tok)
    exact, designed = references(oracle, tid, W, Xb, n_cols)
    assert rel_l2(Y, exact if streams_exact_weights(tid, n_tok, n_rows, n_cols) else designed) <= 2e-5, (ALL[tid], n_tok, n_rows, n_cols)
    assert rel_l2(Y, exact) <= 3e-3


@pytest.mark.parametrize("tid", FUSED, ids=lambda t: ALL[t])
@pytest.mark.parametrize("n_tok,n_rows,n_cols", [
    (260, 12805, 256),   # 101 x 2 tiles: one super-block, ragged rows and tokens
    (1030, 5130, 768),   # 41 x 5 tiles, an odd super-block count
    (513, 8500, 1024),
])
def test_fused_tile_kernel_shapes(oracle, tid, n_tok, n_rows, n_cols):
    """200 or more 256-token x 128-row tiles: Q4_K, Q5_K, Q6_K and Q8_0 are decoded inside the product (no workspace is
    read: none is passed); weights rounded once to bf16, as the decode + dense route rounds them"""
    W = synth.make_weights(tid, n_rows, n_cols, seed=n_rows + tid)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=n_tok + tid, tokens=n_tok))
    ldx, ldy = n_cols + 8, n_rows + 3
    Xpad = np.zeros((n_tok, ldx), np.uint16)
    Xpad[:, :n_cols] = Xb
    dW, dX = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(Xpad)
    dY = qlinear.DevBuf.from_numpy(np.full((n_tok, ldy), -3.0, np.float32))
    qlinear.check(qlinear.load().qlin_gemm_bf16_any_dev(tid, dW.ptr, dX.ptr, dY.ptr, n_rows, n_cols, n_tok, ldx, ldy,
                                                        None, 0, None))
    qlinear.sync()
    Y = dY.to_numpy(np.float32, (n_tok, ldy))
    for buf in (dW, dX, dY):
        buf.free()
    assert np.all(Y[:, n_rows:] == -3.0)
    rows = np.unique(np.concatenate([np.random.default_rng(n_tok).choice(n_rows, 300, replace=False),
                                     np.arange(n_rows - 140, n_rows)]))  # a sample, and the ragged last tiles whole
    exact, designed = references(oracle, tid, W[rows], Xb, n_cols)
    assert rel_l2(Y[:, rows], designed) <= 2e-5, (ALL[tid], n_tok, n_rows, n_cols)
    assert rel_l2(Y[:, rows], exact) <= 3e-3


@pytest.mark.parametrize("tile", [0, 1], ids=["256x128", "128x64"])
@pytest.mark.parametrize("tid", FUSED, ids=lambda t: ALL[t])
@pytest.mark.parametrize("n_tok,n_rows,n_cols", [
    (5, 7, 256), (130, 70, 512), (300, 200, 1280), (64, 129, 2048), (513, 65, 256),
])
def test_each_tile_kernel_on_small_and_ragged_shapes(oracle, tile, tid, n_tok, n_rows, n_cols):
    """both tile kernels called by name, on shapes the shape-based choice would give to other kernels: one super-block,
    an odd count of them, single rows and tokens, ragged last tiles, padded leading dimensions"""
    W = synth.make_weights(tid, n_rows, n_cols, seed=3 * n_rows + tid + tile)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=n_tok + tid, tokens=n_tok))
    ldx, ldy = n_cols + 16, n_rows + 1
    Xpad = np.zeros((n_tok, ldx), np.uint16)
    Xpad[:, :n_cols] = Xb
    dW, dX = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(Xpad)
    dY = qlinear.DevBuf.from_numpy(np.full((n_tok, ldy), -3.0, np.float32))
    qlinear.probe_gemm_tile(tile, tid, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy)
    qlinear.sync()
    Y = dY.to_numpy(np.float32, (n_tok, ldy))
    for buf in (dW, dX, dY):
        buf.free()
    assert np.all(Y[:, n_rows:] == -3.0)
    exact, designed = references(oracle, tid, W, Xb, n_cols)
    assert rel_l2(Y[:, :n_rows], designed) <= 2e-5, (ALL[tid], tile, n_tok, n_rows, n_cols)
    if n_tok * n_rows >= 1000:  # the bar on the bf16 rounding of the weights is a statistical one
        assert rel_l2(Y[:, :n_rows], exact) <= 3e-3


def multi_case(tid, rows, n_cols, n_tok, seed):
    Ws = [synth.make_weights(tid, r, n_cols, seed=seed + i) for i, r in enumerate(rows)]
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=seed + 9, tokens=n_tok))
    ldx = n_cols + 8
    Xpad = np.zeros((n_tok, ldx), np.uint16)
    Xpad[:, :n_cols] = Xb
    ldys = [r + 1 + i for i, r in enumerate(rows)]
    return Ws, Xb, Xpad, ldx, ldys


def run_multi(tid, Ws, Xpad, rows, n_cols, n_tok, ldx, ldys, together, ws_bytes=0):
    dWs = [qlinear.DevBuf.from_numpy(W) for W in Ws]
    dX = qlinear.DevBuf.from_numpy(Xpad)
    dYs = [qlinear.DevBuf.from_numpy(np.full((n_tok, ld), -3.0, np.float32)) for ld in ldys]
    dws = qlinear.DevBuf(ws_bytes) if ws_bytes else None
    if together:
        qlinear.gemm_bf16_multi_dev(tid, dWs, dX, dYs, rows, n_cols, n_tok, ldx, ldys, dws)
    else:
        for dW, dY, r, ld in zip(dWs, dYs, rows, ldys):
            qlinear.gemm_bf16_any_dev(tid, dW, dX, dY, r, n_cols, n_tok, ldx, ld, dws)
    qlinear.sync()
    Ys = [dY.to_numpy(np.float32, (n_tok, ld)) for dY, ld in zip(dYs, ldys)]
    for b in dWs + dYs + [dX] + ([dws] if dws else []):
        b.free()
    return Ys


@pytest.mark.parametrize("tid", FUSED, ids=lambda t: ALL[t])
@pytest.mark.parametrize("rows,n_cols,n_tok", [
    ((256, 64, 70), 512, 130),   # ragged last tiles of the second and third tensor, two token tiles
    ((130, 129), 1280, 64),      # two tensors, neither a whole number of tiles
    ((64, 64, 64), 256, 33),     # one tile each, one super-block
    ((6400, 6500), 256, 1024),   # 200 and more 256-token x 128-row tiles each: the large-tile kernel
])
def test_several_tensors_in_one_launch_equal_one_call_each(oracle, tid, rows, n_cols, n_tok):
    """qlin_gemm_bf16_multi_dev on shapes where every tensor takes the same tile kernel: bit for bit what one call per
    tensor gives (the same workgroups run, numbered through the tensors), right against the oracle, and nothing written
    past a tensor's rows"""
    rows = list(rows)
    Ws, Xb, Xpad, ldx, ldys = multi_case(tid, rows, n_cols, n_tok, seed=500 + tid)
    one_by_one = run_multi(tid, Ws, Xpad, rows, n_cols, n_tok, ldx, ldys, together=False)
    together = run_multi(tid, Ws, Xpad, rows, n_cols, n_tok, ldx, ldys, together=True)
    for W, r, a, b in zip(Ws, rows, one_by_one, together):
        if tid == Q4K and n_tok <= FEW:  # the single call takes the few-token kernel (exact codes): compare by value
            assert rel_l2(b[:, :r], a[:, :r]) <= 3e-3
        else:
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (ALL[tid], r)
        assert np.all(b[:, r:] == -3.0)
        exact, designed = references(oracle, tid, W, Xb, n_cols)
        assert rel_l2(b[:, :r], designed) <= 2e-5, (ALL[tid], r)


def test_several_tensors_fall_back_to_one_call_each(oracle):
    """a format without a tile kernel, a few tokens, and a single tensor: the per-tensor route, same results and same errors"""
    lib = qlinear.load()
    for tid, n_tok in ((synth.GGML_Q5_1, 40), (synth.GGML_Q6_K, 8), (Q4K, 16)):
        rows, n_cols = [96, 33], 512
        Ws, Xb, Xpad, ldx, ldys = multi_case(tid, rows, n_cols, n_tok, seed=700 + tid)
        ws_bytes = qlinear.gemm_bf16_any_workspace_bytes(max(rows), n_cols)
        a = run_multi(tid, Ws, Xpad, rows, n_cols, n_tok, ldx, ldys, together=False, ws_bytes=ws_bytes)
        b = run_multi(tid, Ws, Xpad, rows, n_cols, n_tok, ldx, ldys, together=True, ws_bytes=ws_bytes)
        for x, y in zip(a, b):
            assert np.array_equal(x.view(np.uint32), y.view(np.uint32)), ALL[tid]
    # the formats without a tile kernel need the workspace here as well
    rows, n_cols, n_tok = [96, 33], 512, 40
    Ws, Xb, Xpad, ldx, ldys = multi_case(synth.GGML_Q5_1, rows, n_cols, n_tok, seed=3)
    with pytest.raises(qlinear.QlinError):
        run_multi(synth.GGML_Q5_1, Ws, Xpad, rows, n_cols, n_tok, ldx, ldys, together=True)
    d = qlinear.DevBuf(4096)
    import ctypes as C
    one = (C.c_void_p * 1)(d.ptr)
    n1 = (C.c_int * 1)(16)
    f = lib.qlin_gemm_bf16_multi_dev
    assert f(Q4K, 0, one, d.ptr, one, n1, 256, 4, 256, n1, None, 0, None) == qlinear.ERR_ARG   # no tensor
    assert f(Q4K, 4, one, d.ptr, one, n1, 256, 4, 256, n1, None, 0, None) == qlinear.ERR_ARG   # more than three
    assert f(Q4K, 1, None, d.ptr, one, n1, 256, 4, 256, n1, None, 0, None) == qlinear.ERR_ARG  # no array
    d.free()


@pytest.mark.parametrize("tid", [t for t in FUSED if t != Q4K], ids=lambda t: ALL[t])  # Q4_K: test_gpu_gemm_bf16.py
def test_fused_tile_kernel_full_size_config(oracle, tid):
    """14336 x 4096 at 512 tokens; the oracle on a sample of rows, and scaling X by two scales Y exactly"""
    n_rows, n_cols, n_tok = 14336, 4096, 512
    W = synth.make_weights(tid, n_rows, n_cols, seed=43)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=44, tokens=n_tok))
    Y = run(tid, W, Xb, n_rows, n_cols, n_tok)
    rows = np.random.default_rng(2).choice(n_rows, 160, replace=False)
    exact, designed = references(oracle, tid, W[rows], Xb, n_cols)
    assert rel_l2(Y[:, rows], designed) <= 2e-5
    assert rel_l2(Y[:, rows], exact) <= 3e-3
    Y2 = run(tid, W, synth.to_bf16_bits(2.0 * synth.bf16_bits_to_f32(Xb)), n_rows, n_cols, n_tok)
    assert np.array_equal(Y2, 2.0 * Y)


@pytest.mark.parametrize("tid,n_tok,n_rows,n_cols", [
    (synth.GGML_IQ3_S, 70, 130, 512), (synth.GGML_Q8_0, 33, 257, 96), (synth.GGML_BF16, 40, 64, 1024),
    (synth.GGML_Q4_1, 9000, 16, 1024),  # more tokens than one band of the workspace holds as fp32
])
def test_neither_dense_kernel_takes_the_shape(oracle, tid, n_tok, n_rows, n_cols):
    """with both dense products switched off the call still answers: the vector-ALU kernel on the exact weights"""
    W = synth.make_weights(tid, n_rows, n_cols, seed=5 + tid)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=6 + tid, tokens=n_tok))
    qlinear.check(qlinear.load().qlin_set_dense_gemm_own(2))
    try:
        Y = run(tid, W, Xb, n_rows, n_cols, n_tok, ldx=n_cols + 16, ldy=n_rows + 5)
    finally:
        qlinear.check(qlinear.load().qlin_set_dense_gemm_own(0))
    assert np.all(Y[:, n_rows:] == -3.0)
    exact, _ = references(oracle, tid, W, Xb, n_cols)
    assert rel_l2(Y[:, :n_rows], exact) <= 2e-5
    assert qlinear.load().qlin_set_dense_gemm_own(3) == qlinear.ERR_ARG


BLOCK_NOT_KQ = sorted(t for t in ALL if t not in KQ and t not in synth.DENSE_TYPES and t != Q4K)


@pytest.mark.parametrize("n_tok", [1, 4, 5])
@pytest.mark.parametrize("tid", BLOCK_NOT_KQ, ids=lambda t: ALL[t])
def test_up_to_four_tokens_take_the_matvec(oracle, tid, n_tok):
    """formats without a few-token kernel: up to four tokens go one by one through the matvec (exact weights, padded
    X and Y rows left alone), five through decode + dense product"""
    n_rows, n_cols = 203, 4608
    W = synth.make_weights(tid, n_rows, n_cols, seed=70 + tid)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=71 + n_tok, tokens=n_tok))
    ldx, ldy = n_cols + 24, n_rows + 5
    Y = run(tid, W, Xb, n_rows, n_cols, n_tok, ldx=ldx, ldy=ldy)
    exact, designed = references(oracle, tid, W, Xb, n_cols)
    assert rel_l2(Y[:, :n_rows], exact if n_tok <= 4 else designed) <= 2e-5, (ALL[tid], n_tok)
    assert np.all(Y[:, n_rows:] == -3.0)


def test_few_tokens_whose_rows_lie_far_apart(oracle):
    """three tokens of X with a leading dimension so wide that their fp32 copy would not fit the workspace: the call
    must not write past it (it takes the decode + dense route instead)"""
    tid = synth.GGML_IQ4_XS
    n_rows, n_cols, n_tok = 16, 256, 3
    ws_bytes = qlinear.gemm_bf16_any_workspace_bytes(n_rows, n_cols)
    ldx = (ws_bytes // 4 // (n_tok - 1) + 8) // 8 * 8  # (n_tok - 1) * ldx * 4 bytes > the workspace
    W = synth.make_weights(tid, n_rows, n_cols, seed=91)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=92, tokens=n_tok))
    Xpad = np.zeros((n_tok - 1) * ldx + n_cols, np.uint16)
    for t in range(n_tok):
        Xpad[t * ldx:t * ldx + n_cols] = Xb[t]
    dW, dX = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(Xpad)
    dY = qlinear.DevBuf.from_numpy(np.full((n_tok, n_rows), -3.0, np.float32))
    guard = 1 << 20
    ws = qlinear.DevBuf.from_numpy(np.full(ws_bytes + guard, 0x5A, np.uint8))
    # the workspace is declared without its guard megabyte, which has to come back untouched
    qlinear.check(qlinear.load().qlin_gemm_bf16_any_dev(tid, dW.ptr, dX.ptr, dY.ptr, n_rows, n_cols, n_tok, ldx, n_rows,
                                                        ws.ptr, ws_bytes, None))
    qlinear.sync()
    exact, designed = references(oracle, tid, W, Xb, n_cols)
    assert rel_l2(dY.to_numpy(np.float32, (n_tok, n_rows)), designed) <= 2e-5
    assert np.all(ws.to_numpy(np.uint8, (ws_bytes + guard,))[ws_bytes:] == 0x5A)


@pytest.mark.parametrize("n_tok", [1, 8, 9, 24, 25])
@pytest.mark.parametrize("tid", sorted(KQ), ids=lambda t: ALL[t])
def test_few_tokens_of_a_k_quant_or_q8_0_tensor(oracle, tid, n_tok):
    """up to 24 tokens: one kernel, unrounded weights, no workspace, rows and padding of any count; 25 tokens: weights
    rounded to bf16 - inside the tile kernel for the formats that has (no workspace either), else by the decode + dense
    route, which needs the workspace"""
    # 5 super-blocks over 4 waves, a last row tile of 8 rows; the kernel wants the tensor to end on a 16-byte
    # boundary (210-, 110- and 84-byte blocks: a row count that is a multiple of 8)
    n_rows, n_cols = 296, 1280
    W = synth.make_weights(tid, n_rows, n_cols, seed=40 + tid)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=41 + n_tok, tokens=n_tok))
    ldx, ldy = n_cols + 8, n_rows + 3
    Xpad = np.zeros((n_tok, ldx), np.uint16)
    Xpad[:, :n_cols] = Xb
    dW, dX = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(Xpad)
    dY = qlinear.DevBuf.from_numpy(np.full((n_tok, ldy), -3.0, np.float32))
    exact, designed = references(oracle, tid, W, Xb, n_cols)
    if n_tok <= 24:
        qlinear.gemm_bf16_any_dev(tid, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy, None)
        want = exact
    elif tid in FUSED:
        qlinear.gemm_bf16_any_dev(tid, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy, None)
        want = designed
    else:
        with pytest.raises(qlinear.QlinError):
            qlinear.gemm_bf16_any_dev(tid, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy, None)
        ws = qlinear.DevBuf(qlinear.gemm_bf16_any_workspace_bytes(n_rows, n_cols))
        qlinear.gemm_bf16_any_dev(tid, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy, ws)
        want = designed
    qlinear.sync()
    Y = dY.to_numpy(np.float32, (n_tok, ldy))
    assert rel_l2(Y[:, :n_rows], want) <= 2e-5, (ALL[tid], n_tok)
    assert np.all(Y[:, n_rows:] == -3.0)


def test_q4k_few_tokens_is_the_fused_path_and_needs_no_workspace(oracle):
    n_tok, n_rows, n_cols = 30, 96, 512
    W = synth.make_weights(Q4K, n_rows, n_cols, seed=1)
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=2, tokens=n_tok))
    dW, dX, dY = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf.from_numpy(Xb), qlinear.DevBuf(n_tok * n_rows * 4)
    qlinear.gemm_bf16_any_dev(Q4K, dW, dX, dY, n_rows, n_cols, n_tok, n_cols, n_rows, None)
    qlinear.sync()
    exact, _ = references(oracle, Q4K, W, Xb, n_cols)
    assert rel_l2(dY.to_numpy(np.float32, (n_tok, n_rows)), exact) <= 2e-5  # few-token kernel: exact weights


def test_strides_padding_and_workspace_reuse(oracle):
    tid, n_tok, n_rows, n_cols = synth.GGML_Q6_K, 90, 200, 1024
    ws = qlinear.DevBuf(qlinear.gemm_bf16_any_workspace_bytes(n_rows, n_cols))
    for seed in (3, 4):  # two different tensors through one workspace, back to back
        W = synth.make_weights(tid, n_rows, n_cols, seed=seed)
        Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=seed + 10, tokens=n_tok))
        Y = run(tid, W, Xb, n_rows, n_cols, n_tok, ldx=n_cols + 64, ldy=n_rows + 12, ws=ws)
        _, designed = references(oracle, tid, W, Xb, n_cols)
        assert rel_l2(Y[:, :n_rows], designed) <= 2e-5
        assert np.all(Y[:, n_rows:] == -3.0)
    ws.free()


@pytest.mark.parametrize("pad", [0, 12])
@pytest.mark.parametrize("n_tok,n_rows,n_cols", [(9, 300, 8192), (512, 300, 8192), (64, 4096, 16384)])
def test_padded_output_with_long_rows(n_tok, n_rows, n_cols, pad):
    """few output tiles and a long K: the library's kernels that split K and reduce through a workspace wrote
    a padded Y (ldy > n_rows) as if it were dense; the plan for such a call offers them no workspace
    (pad = 0: the same shapes with a dense Y, where those kernels are used)"""
    rng = np.random.default_rng(n_tok + n_cols)
    Wb = synth.to_bf16_bits(rng.standard_normal((n_rows, n_cols)).astype(np.float32))
    Xb = synth.to_bf16_bits(rng.standard_normal((n_tok, n_cols)).astype(np.float32))
    Y = run(synth.GGML_BF16, Wb.view(np.uint8), Xb, n_rows, n_cols, n_tok, ldx=n_cols + 64, ldy=n_rows + pad)
    want = synth.bf16_bits_to_f32(Xb).astype(np.float64) @ synth.bf16_bits_to_f32(Wb).astype(np.float64).T
    assert rel_l2(Y[:, :n_rows], want) <= 2e-5
    assert np.all(Y[:, n_rows:] == -3.0)


def test_argument_checks():
    lib = qlinear.load()
    d = qlinear.DevBuf(1 << 20)
    need = qlinear.gemm_bf16_any_workspace_bytes(128, 256)
    assert need == 128 * 256 * 2 + (32 << 20)
    ws = qlinear.DevBuf(need)
    f = lib.qlin_gemm_bf16_any_dev
    Q6K = synth.GGML_Q6_K
    assert f(9, d.ptr, d.ptr, d.ptr, 128, 256, 4, 256, 128, ws.ptr, need, None) == qlinear.ERR_TYPE
    assert f(Q6K, d.ptr, d.ptr, d.ptr, 128, 300, 4, 304, 128, ws.ptr, need, None) == qlinear.ERR_ARG      # ragged K
    assert f(Q6K, d.ptr, d.ptr, d.ptr, 128, 256, 4, 260, 128, ws.ptr, need, None) == qlinear.ERR_ARG      # ldx % 8
    assert f(Q6K, d.ptr, d.ptr, d.ptr, 128, 256, 4, 256, 100, ws.ptr, need, None) == qlinear.ERR_ARG      # ldy < rows
    NL = synth.GGML_Q5_1  # a format that always takes the decode + dense route above 24 tokens
    assert f(NL, d.ptr, d.ptr, d.ptr, 128, 256, 32, 256, 128, ws.ptr, need - 1, None) == qlinear.ERR_ARG  # small workspace
    assert f(NL, d.ptr, d.ptr, d.ptr, 128, 256, 32, 256, 128, None, 0, None) == qlinear.ERR_ARG           # no workspace
    assert f(NL, d.ptr, d.ptr, d.ptr, 128, 256, 32, 256, 128, C.c_void_p(ws.ptr + 16), need, None) == qlinear.ERR_ARG
    assert f(Q6K, d.ptr, d.ptr, d.ptr, 128, 256, 4, 256, 128, None, 0, None) == 0   # few tokens: no workspace needed
    assert f(Q6K, d.ptr, d.ptr, d.ptr, 128, 256, 32, 256, 128, None, 0, None) == 0  # nor by the tile kernels
    assert f(Q6K, d.ptr, d.ptr, d.ptr, 0, 256, 4, 256, 128, None, 0, None) == 0
    assert f(Q6K, d.ptr, d.ptr, d.ptr, 128, 256, 0, 256, 128, None, 0, None) == 0
    assert lib.qlin_gemm_bf16_any_workspace_bytes(0, 256) == 0


@pytest.mark.parametrize("tid", sorted(ALL), ids=lambda t: ALL[t])
def test_decode_to_bf16_is_the_codec_rounded_once(oracle, tid):
    n_rows, n_cols = 37, 1024
    W = synth.make_weights(tid, n_rows, n_cols, seed=40 + tid)
    dW, dout = qlinear.DevBuf.from_numpy(W), qlinear.DevBuf(n_rows * n_cols * 2)
    qlinear.dequant_bf16_dev(tid, dW, dout, n_rows, n_cols)
    qlinear.sync()
    got = dout.to_numpy(np.uint16, (n_rows, n_cols))
    want = synth.to_bf16_bits(oracle.dequant_matrix(tid, W, n_cols))
    assert np.array_equal(got, want), ALL[tid]
    # a cached bf16 copy is a weight tensor of its own
    n_tok = 70
    Xb = synth.to_bf16_bits(synth.make_activation(n_cols, seed=7, tokens=n_tok))
    Y_cached = run(synth.GGML_BF16, got.view(np.uint8).reshape(n_rows, -1), Xb, n_rows, n_cols, n_tok)
    Y_direct = run(tid, W, Xb, n_rows, n_cols, n_tok)
    if tid in FUSED:  # the same rounded weights inside the tile kernel, summed in another order
        assert rel_l2(Y_direct, Y_cached) <= 2e-6
    else:
        assert np.array_equal(Y_cached, Y_direct)
    dW.free()
    dout.free()


@pytest.mark.parametrize("tid", [Q4K, synth.GGML_Q6_K, synth.GGML_Q8_0, synth.GGML_IQ3_S, synth.GGML_F16, synth.GGML_F32,
                                 synth.GGML_BF16], ids=lambda t: ALL[t])
def test_host_pointer_prefill_on_the_matrix_cores_when_opted_in(oracle, tid):
    lib = qlinear.load()
    n_tok, n_rows, n_cols = 60, 300, 1024
    W = synth.make_weights(tid, n_rows, n_cols, seed=77 + tid)
    X = synth.make_activation(n_cols, seed=78, tokens=n_tok)
    want = X.astype(np.float64) @ oracle.dequant_matrix(tid, W, n_cols).astype(np.float64).T
    exact = qlinear.gemm_tokenmajor(tid, W, X, n_cols)
    assert rel_l2(exact, want) <= 1e-5
    assert lib.qlin_set_prefill_matrix_cores(1) == 0
    try:
        fast = qlinear.gemm_tokenmajor(tid, W, X, n_cols)
        few = qlinear.gemm_tokenmajor(tid, W, X[:5], n_cols)  # fewer than 8 tokens stay on the fp32 path
    finally:
        assert lib.qlin_set_prefill_matrix_cores(0) == 0
    err = rel_l2(fast, want)
    assert 1e-5 < err <= 3e-3, err  # the bf16 route really ran, and inside its contract
    assert rel_l2(few, want[:5]) <= 1e-5
    assert rel_l2(qlinear.gemm_tokenmajor(tid, W, X, n_cols), want) <= 1e-5  # and the switch is off again


def test_more_shapes_than_the_plan_cache_holds():
    """the dense GEMM keeps one library plan per shape, at most 512: a caller with ever-changing token counts
    makes it start over, and results stay right on both sides of that"""
    n_rows, n_cols = 64, 64
    rng = np.random.default_rng(5)
    Wf = rng.standard_normal((n_rows, n_cols)).astype(np.float32)
    Wb = synth.to_bf16_bits(Wf)
    Wd = synth.bf16_bits_to_f32(Wb).astype(np.float64)
    dW = qlinear.DevBuf.from_numpy(Wb.view(np.uint8))
    ws = qlinear.DevBuf(qlinear.gemm_bf16_any_workspace_bytes(n_rows, n_cols))
    n_max = 530
    Xb = synth.to_bf16_bits(rng.standard_normal((n_max, n_cols)).astype(np.float32))
    dX, dY = qlinear.DevBuf.from_numpy(Xb), qlinear.DevBuf(n_max * n_rows * 4)
    want = synth.bf16_bits_to_f32(Xb).astype(np.float64) @ Wd.T
    for n_tok in range(1, n_max + 1):
        qlinear.gemm_bf16_any_dev(synth.GGML_BF16, dW, dX, dY, n_rows, n_cols, n_tok, n_cols, n_rows, ws)
        if n_tok in (1, 2, 511, 512, 513, 514, n_max):
            qlinear.sync()
            got = dY.to_numpy(np.float32, (n_max, n_rows))[:n_tok]
            assert rel_l2(got, want[:n_tok]) <= 2e-5, n_tok
    qlinear.sync()
    for b in (dW, ws, dX, dY):
        b.free()
