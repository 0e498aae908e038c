"""Pins the CPU oracle's codec: golden vectors decoded by the compiled reference, independent
closed forms, table checksums. CPU only."""
import hashlib

import numpy as np
import pytest

from gemm_amd import synth
from tests import formulas

NAMES = list(synth.TYPE_NAMES.items())

# SHA-256 of each codebook's little-endian memory image, computed from the reference's tables
TABLE_SHA = {
    "iq2xxs_grid": "05826b5d3e472a3a78f196be62ac78acf81df0f909626e12ab9fa2a5d490dd54",
    "ksigns": "a76742a603f8beca5212ecce0f1f02f11a4887fd2f7c8b15aca0ea3eb3380c31",
    "iq4nl_values": "61aa47540aa024b5d6ddaa839b84ffe59f3d5a349af5c6c7ffcb5e0474b46163",
    "iq3s_grid": "bd1af4945a1717c65610b0284e4628b9a1ba3b306fae3a06f6e5f597356e349f",
}


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def test_fp16_exhaustive_matches_reference_hash(oracle, manifest):
    table = oracle.fp16_table()
    assert sha(table.view(np.uint32)) == manifest["fp16_table_sha256"]
    for h, bits in manifest["fp16_probe_bits"].items():
        assert "%08x" % int(table.view(np.uint32)[int(h, 16)]) == bits


def test_fp16_exhaustive_matches_ieee(oracle):
    table = oracle.fp16_table()
    ieee = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    finite = np.isfinite(ieee)
    assert np.array_equal(table.view(np.uint32)[finite], ieee.view(np.uint32)[finite])
    assert np.array_equal(np.isnan(table), np.isnan(ieee))
    assert np.array_equal(np.isinf(table), np.isinf(ieee))
    # NaN payload: sign | 0x7F800000 | mantissa << 13, never quieted
    h = np.arange(65536, dtype=np.uint32)
    nan = np.isnan(ieee)
    want = ((h >> 15) << 31) | 0x7F800000 | ((h & 1023) << 13)
    assert np.array_equal(table.view(np.uint32)[nan], want[nan].astype(np.uint32))


def test_tables_match_published_checksums(oracle, manifest):
    for name, digest in TABLE_SHA.items():
        assert hashlib.sha256(oracle.table(name)).hexdigest() == digest, name
        assert manifest["tables_sha256"][name] == digest, name


def test_sign_table_closed_form(oracle):
    t = np.frombuffer(oracle.table("ksigns"), np.uint8)
    for i in range(128):
        assert t[i] == i | ((bin(i).count("1") & 1) << 7)
        assert bin(int(t[i])).count("1") % 2 == 0


@pytest.mark.parametrize("tid,name", NAMES)
def test_decoder_matches_reference_golden_bits(oracle, codec_golden, tid, name):
    src = codec_golden[name + "_src"]
    want = codec_golden[name + "_f32bits"]
    n = want.shape[1]
    for r in range(src.shape[0]):
        rc, got = oracle.dequant_row(tid, src[r], n)
        assert rc == 0
        assert np.array_equal(got.view(np.uint32), want[r]), (name, r)
        got2 = oracle.dequantize_named(name, src[r], n)
        assert np.array_equal(got2.view(np.uint32), want[r]), (name, r)


@pytest.mark.parametrize("tid,name", NAMES)
def test_decoder_matches_reference_sweep_hash(oracle, manifest, tid, name):
    info = manifest["codec_sweep"][name]
    W = synth.make_weights(tid, info["rows"], info["cols"], seed=info["seed"], wild=info["wild"])
    if sha(W) != info["input_sha256"]:
        pytest.skip("numpy's random stream differs from the one the fixture was drawn with")
    dec = oracle.dequant_matrix(tid, W, info["cols"])
    assert sha(dec.view(np.uint32)) == info["output_sha256"]


@pytest.mark.parametrize("tid,name", NAMES)
def test_decoder_matches_independent_closed_form(oracle, tid, name):
    """float64 formula rounded once to fp32 == decoder, bit for bit (finite scales)."""
    n = 1024
    W = synth.make_weights(tid, 8, n, seed=500 + tid)
    for r in range(W.shape[0]):
        if name == "iq2_xxs":
            f = formulas.iq2_xxs(W[r], oracle.table("iq2xxs_grid"))
        elif name == "iq3_s":
            f = formulas.iq3_s(W[r], oracle.table("iq3s_grid"))
        else:
            f = getattr(formulas, name)(W[r])
        rc, got = oracle.dequant_row(tid, W[r], n)
        assert np.array_equal(got.view(np.uint32), f.astype(np.float32).view(np.uint32)), (name, r)


def test_q4k_hand_built_block(oracle):
    """d=1, dmin=0, all scales 1 -> the decoded row is the nibbles themselves."""
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    sc = np.ones(8, np.uint8)
    blk[4:16] = oracle.k4_pack(sc, np.zeros(8, np.uint8))
    blk[16:] = np.arange(128, dtype=np.uint8) * 37 + 11
    rc, y = oracle.dequant_row(synth.GGML_Q4_K, blk, 256)
    q = blk[16:]
    for c in range(4):
        assert np.array_equal(y[64 * c:64 * c + 32], (q[32 * c:32 * c + 32] & 15).astype(np.float32))
        assert np.array_equal(y[64 * c + 32:64 * c + 64], (q[32 * c:32 * c + 32] >> 4).astype(np.float32))


def test_k4_scale_pack_unpack_round_trip(oracle):
    rng = np.random.default_rng(3)
    for _ in range(200):
        sc = rng.integers(0, 64, 8).astype(np.uint8)
        mn = rng.integers(0, 64, 8).astype(np.uint8)
        sc2, mn2 = oracle.k4_unpack(oracle.k4_pack(sc, mn))
        assert np.array_equal(sc, sc2) and np.array_equal(mn, mn2)
    for v in range(64):  # every 6-bit value in every slot
        for slot in range(8):
            sc = np.zeros(8, np.uint8)
            sc[slot] = v
            sc2, mn2 = oracle.k4_unpack(oracle.k4_pack(sc, sc[::-1].copy()))
            assert np.array_equal(sc, sc2) and np.array_equal(sc[::-1], mn2)


def test_row_size_and_unknown_type(oracle, manifest):
    for t, per_n in manifest["row_size"].items():
        if int(t) not in list(synth.TYPE_NAMES) + [0, 1, 30, 9, 15, 99]:
            continue
        for n, want in per_n.items():
            if int(t) in (9, 15, 99):
                assert oracle.row_size(int(t), int(n)) == 0 == want
            else:
                assert oracle.row_size(int(t), int(n)) == want, (t, n)
    rc, _ = oracle.dequant_row(99, np.zeros(64, np.uint8), 32)
    assert rc == -1 == manifest["dequant_row_unknown_type_rc"]


@pytest.mark.parametrize("tid,name", NAMES)
def test_ragged_tail_is_dropped(oracle, tid, name):
    be, bb = synth.BLOCK_GEOMETRY[tid]
    W = synth.make_weights(tid, 1, 2 * be, seed=9)[0]
    rc, full = oracle.dequant_row(tid, W, 2 * be)
    rc, part = oracle.dequant_row(tid, W, 2 * be - 1)  # one whole block, the second is dropped
    assert np.array_equal(part[:be], full[:be])
    assert not part[be:].any()
    rc, none = oracle.dequant_row(tid, W, 0)
    assert none.size == 0


def test_plain_float_types(oracle):
    rng = np.random.default_rng(5)
    f = rng.standard_normal(64).astype(np.float32)
    rc, y = oracle.dequant_row(synth.GGML_F32, f.view(np.uint8), 64)
    assert rc == 0 and np.array_equal(y, f)
    h = f.astype(np.float16)
    rc, y = oracle.dequant_row(synth.GGML_F16, h.view(np.uint8), 64)
    assert np.array_equal(y, h.astype(np.float32))
    b = synth.to_bf16_bits(f)
    rc, y = oracle.dequant_row(synth.GGML_BF16, b.view(np.uint8), 64)
    assert np.array_equal(y, synth.bf16_bits_to_f32(b))
