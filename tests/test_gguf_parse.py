"""The GGUF header parser of the C-ABI library (no GPU needed): against what the reference's own
loader read from the committed fixture file, against files written here, and against damaged files."""
import ctypes as C
import hashlib
import os
import struct

import numpy as np
import pytest

from gemm_amd import qlinear
import synth
from tests import gguf_writer as gw
from tests.conftest import GOLDEN


class Gguf:
    def __init__(self, path):
        self.lib = qlinear.load()
        h = C.c_void_p()
        self.rc = self.lib.qlin_gguf_open(str(path).encode(), C.byref(h))
        self.h = h if self.rc == 0 else None

    def close(self):
        if self.h:
            self.lib.qlin_gguf_close(self.h)
            self.h = None

    def tensor(self, i):
        name, ttype, nd = C.c_char_p(), C.c_uint32(), C.c_int()
        dims, off, size = (C.c_uint64 * 4)(), C.c_uint64(), C.c_size_t()
        rc = self.lib.qlin_gguf_tensor_info(self.h, i, C.byref(name), C.byref(ttype), C.byref(nd), dims, C.byref(off),
                                            C.byref(size))
        assert rc == 0
        return {"name": name.value.decode(), "type": ttype.value, "n_dims": nd.value, "dims": list(dims),
                "offset": off.value, "size": size.value}

    def i64(self, key):
        v = C.c_int64()
        rc = self.lib.qlin_gguf_get_i64(self.h, self.lib.qlin_gguf_find_key(self.h, key.encode()), C.byref(v))
        return rc, v.value

    def f64(self, key):
        v = C.c_double()
        rc = self.lib.qlin_gguf_get_f64(self.h, self.lib.qlin_gguf_find_key(self.h, key.encode()), C.byref(v))
        return rc, v.value


@pytest.fixture()
def tiny():
    g = Gguf(os.path.join(GOLDEN, "tiny.gguf"))
    assert g.rc == 0, qlinear.load().qlin_last_error()
    yield g
    g.close()


def test_fixture_file_is_the_one_the_reference_read(manifest):
    raw = open(os.path.join(GOLDEN, "tiny.gguf"), "rb").read()
    assert hashlib.sha256(raw).hexdigest() == manifest["gguf_fixture"]["file_sha256"]


def test_header_matches_reference(tiny, manifest):
    ref, L = manifest["gguf_fixture"], tiny.lib
    assert L.qlin_gguf_version(tiny.h) == ref["version"]
    assert L.qlin_gguf_alignment(tiny.h) == ref["alignment"]
    assert L.qlin_gguf_data_offset(tiny.h) == ref["data_offset"]
    assert L.qlin_gguf_data_size(tiny.h) == ref["data_size"]
    assert L.qlin_gguf_n_kv(tiny.h) == ref["n_kv"]
    assert L.qlin_gguf_n_tensors(tiny.h) == len(ref["tensors"])


def test_tensor_table_and_bytes_match_reference(tiny, manifest):
    ref, L = manifest["gguf_fixture"], tiny.lib
    for i, want in enumerate(ref["tensors"]):
        got = tiny.tensor(i)
        for k in ("name", "type", "n_dims", "dims", "offset", "size"):
            assert got[k] == want[k], (i, k)
        assert L.qlin_gguf_find_tensor(tiny.h, want["name"].encode()) == i
        raw = C.string_at(L.qlin_gguf_tensor_host(tiny.h, i), got["size"])
        assert hashlib.sha256(raw).hexdigest() == want["data_sha256"]
        # the qtensor the reference builds from this entry (tf_load_tensor): cols = dims[0], rows = the rest
        qt = want["qtensor"]
        assert qt["n_cols"] == got["dims"][0] and qt["data_offset"] == got["offset"] and qt["type"] == got["type"]
        assert qt["n_rows"] == int(np.prod(got["dims"][1:got["n_dims"]], dtype=np.int64)) if got["n_dims"] > 1 else qt["n_rows"] == 1
        assert got["size"] == qt["n_rows"] * L.qlin_dequant_row_size(got["type"], qt["n_cols"]) or got["n_dims"] == 1
        assert L.qlin_gguf_tensor_dev(tiny.h, i) is None  # nothing uploaded
    assert L.qlin_gguf_find_tensor(tiny.h, b"no.such.tensor") == -1


def test_key_values_match_reference(tiny, manifest):
    ref, L = manifest["gguf_fixture"], tiny.lib
    width = {0: 1, 1: 1, 7: 1, 2: 2, 3: 2, 4: 4, 5: 4, 6: 4, 10: 8, 11: 8, 12: 8}
    for key, e in ref["kv"].items():
        i = L.qlin_gguf_find_key(tiny.h, key.encode())
        assert i == e["index"] and L.qlin_gguf_key(tiny.h, i).decode() == key
        assert L.qlin_gguf_value_type(tiny.h, i) == e["type"]
        if "str" in e:
            assert L.qlin_gguf_get_str(tiny.h, i).decode() == e["str"]
        elif "n" in e:
            et, n, first = C.c_uint32(), C.c_uint64(), C.c_void_p()
            assert L.qlin_gguf_get_array(tiny.h, i, C.byref(et), C.byref(n), C.byref(first)) == 0
            assert n.value == e["n"]
        elif e["type"] in (6, 12):  # floats: same bits
            rc, v = tiny.f64(key)
            packed = struct.pack("<f" if e["type"] == 6 else "<d", v)
            assert rc == 0 and int.from_bytes(packed, "little") == e["raw_u64"]
        else:
            rc, v = tiny.i64(key)
            assert rc == 0 and v & ((1 << (8 * width[e["type"]])) - 1) == e["raw_u64"]
    assert tiny.i64("some.i8") == (0, -100) and tiny.i64("some.u8") == (0, 200)
    assert tiny.i64("some.i16") == (0, -30000) and tiny.i64("some.i64") == (0, -2 ** 62)
    assert tiny.f64("some.u16") == (0, 60000.0) and tiny.f64("qwen3.rope.freq_base") == (0, 1000000.0)
    assert tiny.i64("general.architecture")[0] == qlinear.ERR_TYPE
    assert L.qlin_gguf_get_str(tiny.h, L.qlin_gguf_find_key(tiny.h, b"some.u8")) is None
    assert L.qlin_gguf_find_key(tiny.h, b"missing.key") == -1
    # tf_get_int (common/transformer.h:383-389) takes u32 and i32 only
    for key, want in ref["tf_get_int"].items():
        i = L.qlin_gguf_find_key(tiny.h, key.encode())
        got = tiny.i64(key)[1] if i >= 0 and L.qlin_gguf_value_type(tiny.h, i) in (4, 5) else -7
        assert got == want, key
    # array payloads
    et, n, first = C.c_uint32(), C.c_uint64(), C.c_void_p()
    i = L.qlin_gguf_find_key(tiny.h, b"tokenizer.ggml.scores")
    L.qlin_gguf_get_array(tiny.h, i, C.byref(et), C.byref(n), C.byref(first))
    assert et.value == gw.F32 and list(np.frombuffer(C.string_at(first, 12), np.float32)) == [0.0, -1.5, 2.25]
    i = L.qlin_gguf_find_key(tiny.h, b"tokenizer.ggml.tokens")
    L.qlin_gguf_get_array(tiny.h, i, C.byref(et), C.byref(n), C.byref(first))
    assert et.value == gw.STR and C.string_at(first, 8 + 3) == struct.pack("<Q", 3) + b"<s>"


def test_written_files_round_trip(tmp_path):
    """version 2 and 3, default and custom alignment, no tensors, no key/values, 1-D and 4-D tensors"""
    rng = np.random.default_rng(3)
    for version in (2, 3):
        for alignment in (None, 8, 256):
            tensors = [("a", synth.GGML_Q4_K, (256, 2, 3, 2), rng.integers(0, 256, 12 * 144, dtype=np.uint8)),
                       ("b", synth.GGML_F32, (5,), rng.integers(0, 256, 20, dtype=np.uint8)),
                       ("c", 26, (3, 3), rng.integers(0, 256, 36, dtype=np.uint8)),       # I32: size known, no decoder
                       ("d", synth.GGML_MXFP4, (64, 3), rng.integers(0, 256, 6 * 17, dtype=np.uint8))]
            path = tmp_path / ("v%d_%s.gguf" % (version, alignment))
            offsets, data_offset = gw.write(path, [("k", gw.U32, 7)], tensors, version=version, alignment=alignment)
            g = Gguf(path)
            assert g.rc == 0
            assert g.lib.qlin_gguf_version(g.h) == version and g.lib.qlin_gguf_data_offset(g.h) == data_offset
            assert g.lib.qlin_gguf_alignment(g.h) == (alignment or 32)
            for i, ((name, ttype, dims, data), off) in enumerate(zip(tensors, offsets)):
                t = g.tensor(i)
                assert (t["name"], t["type"], t["offset"], t["size"]) == (name, ttype, off, len(data))
                assert t["dims"][:len(dims)] == list(dims)
                assert C.string_at(g.lib.qlin_gguf_tensor_host(g.h, i), len(data)) == data.tobytes()
            assert g.lib.qlin_gguf_data_size(g.h) == offsets[-1] + len(tensors[-1][3])
            g.close()
    path = tmp_path / "empty.gguf"
    gw.write(path, [], [])
    g = Gguf(path)
    assert g.rc == 0 and g.lib.qlin_gguf_n_tensors(g.h) == 0 and g.lib.qlin_gguf_n_kv(g.h) == 0
    assert g.lib.qlin_gguf_data_size(g.h) == 0
    g.close()


def test_every_truncation_is_refused_or_consistent(tmp_path):
    """cut the fixture at every length: the parser never reads past the end; a prefix is accepted only
    if the whole header and every tensor's bytes are inside it"""
    raw = open(os.path.join(GOLDEN, "tiny.gguf"), "rb").read()
    ref_data_offset = 1152
    lengths = list(range(0, ref_data_offset + 40)) + list(range(ref_data_offset + 40, len(raw), 997)) + [len(raw) - 1]
    path = tmp_path / "cut.gguf"
    accepted = 0
    for n in lengths:
        with open(path, "wb") as f:
            f.write(raw[:n])
        g = Gguf(path)
        if g.rc == 0:
            accepted += 1
            assert n >= g.lib.qlin_gguf_data_offset(g.h) + g.lib.qlin_gguf_data_size(g.h)
        else:
            assert g.rc in (qlinear.ERR_ARG, qlinear.ERR_TYPE) and qlinear.load().qlin_last_error().startswith(b"gguf:")
        g.close()
    assert accepted == 0  # the last tensor ends at the end of the file


def _patched(raw, at, fmt, value):
    b = bytearray(raw)
    b[at:at + struct.calcsize(fmt)] = struct.pack(fmt, value)
    return bytes(b)


def test_damaged_headers_are_refused(tmp_path):
    raw = open(os.path.join(GOLDEN, "tiny.gguf"), "rb").read()
    cases = {
        "magic": _patched(raw, 0, "<I", 0x46554746),
        "version": _patched(raw, 4, "<I", 1),
        "version4": _patched(raw, 4, "<I", 4),
        "tensor count": _patched(raw, 8, "<Q", 2 ** 60),
        "kv count": _patched(raw, 16, "<Q", 2 ** 40),
        "first key length": _patched(raw, 24, "<Q", 2 ** 63),
        "first value type": _patched(raw, 24 + 8 + len("general.architecture"), "<I", 13),
    }
    # a tensor entry that points outside the file / has 5 dims / an unknown type
    name = b"token_embd.weight"
    at = raw.index(name) + len(name)
    cases["five dims"] = _patched(raw, at, "<I", 5)
    cases["unknown tensor type"] = _patched(raw, at + 4 + 16, "<I", 36)
    cases["offset outside"] = _patched(raw, at + 4 + 16 + 4, "<Q", 2 ** 40)
    cases["huge dims"] = _patched(raw, at + 4, "<Q", 2 ** 62)
    path = tmp_path / "bad.gguf"
    for what, data in cases.items():
        with open(path, "wb") as f:
            f.write(data)
        g = Gguf(path)
        assert g.rc != 0, what
        g.close()
    assert Gguf(tmp_path / "does_not_exist.gguf").rc == qlinear.ERR_ARG


def test_reference_shaped_loader_calls(tiny, manifest):
    """qtf_load_tensor / qtf_get_int / qtf_get_float of the reference-named layer against what
    tf_load_tensor / tf_get_int read from the same file"""
    from gemm_amd import build

    class QTensor(C.Structure):
        _fields_ = [("data", C.c_void_p), ("type", C.c_uint32), ("n_rows", C.c_int), ("n_cols", C.c_int),
                    ("n_dims", C.c_int), ("dims", C.c_uint64 * 4), ("scale", C.c_float), ("has_scale", C.c_int)]
    if not os.path.exists(build.TF_LIB):
        build.build_host(verbose=False)
    tf = C.CDLL(build.TF_LIB)
    tf.qtf_load_tensor.restype = QTensor
    tf.qtf_load_tensor.argtypes = [C.c_void_p, C.c_char_p, C.c_int]
    tf.qtf_get_int.argtypes = [C.c_void_p, C.c_char_p, C.c_int]
    tf.qtf_get_float.restype = C.c_float
    tf.qtf_get_float.argtypes = [C.c_void_p, C.c_char_p, C.c_float]
    ref = manifest["gguf_fixture"]
    base = tiny.lib.qlin_gguf_tensor_host(tiny.h, 0) - ref["tensors"][0]["offset"]
    for want in ref["tensors"]:
        t = tf.qtf_load_tensor(tiny.h, want["name"].encode(), 1)
        q = want["qtensor"]
        assert (t.type, t.n_rows, t.n_cols, t.n_dims) == (q["type"], q["n_rows"], q["n_cols"], q["n_dims"])
        assert t.data - base == q["data_offset"] and list(t.dims) == want["dims"]
    assert tf.qtf_load_tensor(tiny.h, b"missing", 0).data is None
    for key, want in ref["tf_get_int"].items():
        assert tf.qtf_get_int(tiny.h, key.encode(), -7) == want, key
    assert tf.qtf_get_float(tiny.h, b"qwen3.rope.freq_base", 0.0) == 1000000.0
    assert tf.qtf_get_float(tiny.h, b"some.f64", 3.0) == 3.0  # f32 only, like the reference
