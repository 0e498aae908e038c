"""The C-ABI library loads and exports every symbol include/qlinear.h declares. CPU only:
no entry point that needs the GPU is called."""
import os
import re

import pytest

from gemm_amd import qlinear

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "qlinear.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(qlin_[a-z0-9_A-Z]+)\s*\(", text)))


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
