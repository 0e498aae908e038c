"""The C-ABI library loads and exports every symbol include/qlinear.h declares. CPU only:
no entry point that needs the GPU is called."""
import os
import re

import pytest

from gemm_amd import qlinear

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    """every function of the engine's header and of the bench-only probe header"""
    names = set()
    for header in ("qlinear.h", "qlinear_bench.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(qlin_[a-z0-9_A-Z]+)\s*\(", text))
    return sorted(names)


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(qlinear.LIB_PATH):
        from gemm_amd import build
        build.build(verbose=False)
    return qlinear.load()


def test_header_and_binding_agree():
    assert set(declared_symbols()) == set(qlinear.SIGNATURES)


def test_every_declared_symbol_is_exported(lib):
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_row_size_needs_no_gpu(lib):
    # pure arithmetic entry point: ceil(n / block) * block_bytes, 0 for unknown types
    assert lib.qlin_dequant_row_size(12, 4096) == 2304
    assert lib.qlin_dequant_row_size(8, 4096) == 4352
    assert lib.qlin_dequant_row_size(14, 4096) == 3360
    assert lib.qlin_dequant_row_size(16, 14336) == 3696
    assert lib.qlin_dequant_row_size(21, 14336) == 6160
    assert lib.qlin_dequant_row_size(20, 4096) == 2304
    assert lib.qlin_dequant_row_size(13, 257) == 352
    assert lib.qlin_dequant_row_size(99, 4096) == 0


def test_row_size_matches_reference_manifest(lib, manifest):
    for t, per_n in manifest["row_size"].items():
        for n, want in per_n.items():
            assert lib.qlin_dequant_row_size(int(t), int(n)) == want, (t, n)


def test_reference_shaped_layer_exports_its_header():
    """libqlinear_tf.so (plain C over the ABI) exports every function include/qlinear_tf.h declares."""
    import ctypes
    from gemm_amd import build
    if not os.path.exists(build.TF_LIB):
        build.build_host(verbose=False)
    text = open(os.path.join(ROOT, "include", "qlinear_tf.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^#.*$", "", text, flags=re.M)
    names = sorted(set(re.findall(r"\b(qtf_[a-z0-9_]+)\s*\(", text)))
    assert len(names) >= 13
    tf = ctypes.CDLL(build.TF_LIB)
    for name in names:
        assert hasattr(tf, name), name
    tf.qtf_row_bytes.restype = ctypes.c_size_t
    assert tf.qtf_row_bytes(12, 4096) == 2304
    assert tf.qtf_is_supported_weight_type(14) == 1 and tf.qtf_is_supported_weight_type(3) == 0
