"""GGUF file -> HBM: the data section streamed into one device block, tensors usable through the
device-resident and the host-pointer entry points without another upload."""
import ctypes as C
import os

import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests import gguf_writer as gw
from tests.conftest import GOLDEN, rel_l2
from tests.test_gguf_parse import Gguf

pytestmark = pytest.mark.gpu


def test_fixture_upload_and_matvec(oracle):
    g = Gguf(os.path.join(GOLDEN, "tiny.gguf"))
    L = g.lib
    assert g.rc == 0 and L.qlin_gguf_upload(g.h) == 0 and L.qlin_gguf_upload(g.h) == 0  # idempotent
    x = synth.make_activation(256, seed=9)
    for i in range(L.qlin_gguf_n_tensors(g.h)):
        t = g.tensor(i)
        host, dev = L.qlin_gguf_tensor_host(g.h, i), L.qlin_gguf_tensor_dev(g.h, i)
        assert dev and L.qlin_weight_device_ptr(host) == dev  # the mapped file's range is registered
        back = np.zeros(t["size"], np.uint8)
        assert L.qlin_dev_download(back.ctypes.data, dev, t["size"]) == 0
        assert back.tobytes() == C.string_at(host, t["size"])
        if t["n_dims"] < 2 or t["dims"][0] != 256:
            continue
        n_rows = int(np.prod(t["dims"][1:t["n_dims"]]))
        W = np.frombuffer(C.string_at(host, t["size"]), np.uint8).reshape(n_rows, -1)
        want = oracle.gemv_f64(t["type"], W, x, 256)
        y = np.zeros(n_rows, np.float32)
        assert L.qlin_matvec(y.ctypes.data, host, t["type"], 256, x.ctypes.data, n_rows) == 0  # host pointer
        assert rel_l2(y, want) <= 1e-5, t["name"]
        dx, dy = qlinear.DevBuf.from_numpy(x), qlinear.DevBuf(n_rows * 4)
        assert L.qlin_gemv_dev(t["type"], dev, dx.ptr, dy.ptr, n_rows, 256, None) == 0      # device pointer
        qlinear.sync()
        assert rel_l2(dy.to_numpy(np.float32, (n_rows,)), want) <= 1e-5, t["name"]
    host0 = L.qlin_gguf_tensor_host(g.h, 0)
    g.close()
    assert L.qlin_weight_device_ptr(host0) is None  # closing releases the registration and the block


def test_large_file_goes_through_the_staging_ring(oracle, tmp_path):
    """about 180 MB: three 64 MB staging turns, the last one partial"""
    rng = np.random.default_rng(1)
    shapes = [("w%d" % i, synth.GGML_Q4_K, 4096, 12000 + 2000 * i) for i in range(5)]
    tensors = [(name, tid, (n_cols, n_rows), synth.make_weights(tid, n_rows, n_cols, seed=i))
               for i, (name, tid, n_cols, n_rows) in enumerate(shapes)]
    tensors.append(("tail", synth.GGML_F32, (1001,), rng.integers(0, 256, 4004, dtype=np.uint8)))
    path = tmp_path / "big.gguf"
    gw.write(path, [("general.architecture", gw.STR, "test")], tensors)
    g = Gguf(path)
    L = g.lib
    assert g.rc == 0 and L.qlin_gguf_data_size(g.h) > 2 * (64 << 20)
    assert L.qlin_gguf_upload(g.h) == 0, L.qlin_last_error()
    x = synth.make_activation(4096, seed=2)
    dx = qlinear.DevBuf.from_numpy(x)
    for i, (name, tid, dims, data) in enumerate(tensors[:-1]):
        n_rows = dims[1]
        dy = qlinear.DevBuf(n_rows * 4)
        assert L.qlin_gemv_dev(tid, L.qlin_gguf_tensor_dev(g.h, i), dx.ptr, dy.ptr, n_rows, 4096, None) == 0
        qlinear.sync()
        rows = np.r_[0:8, n_rows - 8:n_rows]
        assert rel_l2(dy.to_numpy(np.float32, (n_rows,))[rows], oracle.gemv_f64(tid, data[rows], x, 4096)) <= 1e-5
    t = g.tensor(len(tensors) - 1)
    back = np.zeros(4004, np.uint8)
    assert L.qlin_dev_download(back.ctypes.data, L.qlin_gguf_tensor_dev(g.h, len(tensors) - 1), 4004) == 0
    assert np.array_equal(back, tensors[-1][3])
    g.close()
