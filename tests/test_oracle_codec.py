"""Pins the CPU oracle's codec: golden vectors decoded by the compiled reference, independent
closed forms, table checksums. CPU only."""
import hashlib

import numpy as np
import pytest

import synth
from tests import formulas

NAMES = list(synth.TYPE_NAMES.items())

# SHA-256 of each codebook's little-endian memory image, computed from the reference's tables
TABLE_SHA = {
    "iq2xxs_grid": "05826b5d3e472a3a78f196be62ac78acf81df0f909626e12ab9fa2a5d490dd54",
    "ksigns": "a76742a603f8beca5212ecce0f1f02f11a4887fd2f7c8b15aca0ea3eb3380c31",
    "iq4nl_values": "61aa47540aa024b5d6ddaa839b84ffe59f3d5a349af5c6c7ffcb5e0474b46163",
    "iq3s_grid": "bd1af4945a1717c65610b0284e4628b9a1ba3b306fae3a06f6e5f597356e349f",
    "mxfp4_values": "adf76b672d47eb7fc0afd4db132d548d59d3190aa0ad118fdbf569d5fd478f97",
    "iq3xxs_grid": "46e35f5a997efdee6c99ce57854c8a0d4f0ff8ca57e5e8a60c0793ea580acf5d",
    "iq2xs_grid": "06e47aaca60b4dc1d9b5a3f34540437058a6b142b4d7a59d5ded769b4d1bf1de",
    "iq2s_grid": "e1aa1473412b0552c2174c30ef22ab4073f6a181b85a17056e8249bd2932fd88",
    "iq1s_grid": "07540ffc1aeaf6ad4d97e96b0fcc765aae39671d4ae4a27bbd0e796fde167c6a",
}


# formats with two fp16 scales per block: where both are NaN, which payload the result carries
# depends on the compiler's operand order, so NaNs are compared by position for these
TWO_SCALES = {"q4_K", "q5_K", "q2_K", "q4_1", "q5_1"}


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def canonical_nan(bits):
    bits = np.array(bits, dtype=np.uint32, copy=True)
    bits[(bits & 0x7FFFFFFF) > 0x7F800000] = 0x7FC00000
    return bits


def same_bits(got, want_bits, name):
    got_bits = np.ascontiguousarray(got, np.float32).view(np.uint32)
    if name in TWO_SCALES:
        return np.array_equal(canonical_nan(got_bits), canonical_nan(want_bits))
    return np.array_equal(got_bits, want_bits)


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
        assert same_bits(got, want[r], name), (name, r)
        got2 = oracle.dequantize_named(name, src[r], n)
        assert same_bits(got2, want[r], name), (name, r)


@pytest.mark.parametrize("tid,name", NAMES)
def test_decoder_matches_reference_sweep_hash(oracle, manifest, tid, name):
    info = manifest["codec_sweep"][name]
    W = synth.make_weights(tid, info["rows"], info["cols"], seed=info["seed"], wild=info["wild"])
    if sha(W) != info["input_sha256"]:
        pytest.skip("numpy's random stream differs from the one the fixture was drawn with")
    dec = oracle.dequant_matrix(tid, W, info["cols"])
    assert sha(canonical_nan(dec.view(np.uint32))) == info["output_sha256"]


@pytest.mark.parametrize("tid,name", NAMES)
def test_decoder_matches_independent_closed_form(oracle, tid, name):
    """float64 formula rounded once to fp32 == decoder, bit for bit (finite scales)."""
    n = 1024
    W = synth.make_weights(tid, 8, n, seed=500 + tid)
    for r in range(W.shape[0]):
        f = getattr(formulas, name)(W[r], *[oracle.table(t) for t in formulas.TABLE_ARGS.get(name, ())])
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


def test_scale_byte_formats_exhaustive(oracle):
    """E8M0 and unsigned E4M3 scale bytes (halved, as the MXFP4/NVFP4 decoders use them) against
    their definitions, all 256 inputs each."""
    L = oracle.lib
    import ctypes as C
    L.qo_e8m0_half_to_fp32.restype = L.qo_ue4m3_half_to_fp32.restype = C.c_float
    L.qo_e8m0_half_to_fp32.argtypes = L.qo_ue4m3_half_to_fp32.argtypes = [C.c_uint8]
    for e in range(256):
        assert L.qo_e8m0_half_to_fp32(e) == float(np.ldexp(np.float32(1), e - 128)), e
    for x in range(256):
        ex, man = (x >> 3) & 15, x & 7
        want = 0.0 if x in (0, 0x7F) else (man * 2.0 ** -9 if ex == 0 else (1 + man / 8) * 2.0 ** (ex - 7)) * 0.5
        assert L.qo_ue4m3_half_to_fp32(x) == want, x


def test_q3k_scale_unpack_one_hot(oracle):
    """each of the 16 six-bit scale fields of a Q3_K block, set alone to every value, must come
    back at its own index and leave the other fifteen at zero"""
    import ctypes as C
    L = oracle.lib
    L.qo_q3k_scale.argtypes = [C.c_void_p, C.c_int]

    def pack(fields):  # the layout stated bit by bit: low nibbles in bytes 0..7, top bit pairs in 8..11
        s = np.zeros(12, np.uint8)
        for i, v in enumerate(fields):
            s[i % 8] |= (v & 15) << (4 * (i // 8))
            s[8 + i % 4] |= (v >> 4) << (2 * (i // 4))
        return s
    for i in range(16):
        for v in (1, 15, 16, 32, 63):
            fields = [0] * 16
            fields[i] = v
            s = pack(fields)
            got = [L.qo_q3k_scale(s.ctypes.data, j) for j in range(16)]
            assert got == fields, (i, v)


def test_one_hot_blocks_of_the_small_formats(oracle):
    """a single set code in an otherwise neutral block lands on the element the layout says"""
    one = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    for k in range(32):  # Q4_0: d = 1, all nibbles 8 (-> 0) but one
        blk = np.full(18, 0x88, np.uint8)
        blk[0:2] = one
        byte, hi = k % 16, k // 16
        blk[2 + byte] = (0x88 & ~(15 << (4 * hi))) | (15 << (4 * hi))
        _, y = oracle.dequant_row(synth.GGML_Q4_0, blk, 32)
        want = np.zeros(32, np.float32)
        want[k] = 7.0
        assert np.array_equal(y, want), k
    for k in range(128):  # Q1_0: all -1 but one +1
        blk = np.zeros(18, np.uint8)
        blk[0:2] = one
        blk[2 + k // 8] = 1 << (k % 8)
        _, y = oracle.dequant_row(synth.GGML_Q1_0, blk, 128)
        want = -np.ones(128, np.float32)
        want[k] = 1.0
        assert np.array_equal(y, want), k
    for k in range(256):  # TQ2_0: all codes 1 (-> 0) but one code 2 (-> +1)
        blk = np.full(66, 0x55, np.uint8)
        blk[64:66] = one
        byte, pair = 32 * (k // 128) + k % 32, (k % 128) // 32
        blk[byte] = (0x55 & ~(3 << (2 * pair))) | (2 << (2 * pair))
        _, y = oracle.dequant_row(synth.GGML_TQ2_0, blk, 256)
        want = np.zeros(256, np.float32)
        want[k] = 1.0
        assert np.array_equal(y, want), k


def test_tq1_0_digits_round_trip(oracle):
    """pack known trits the way the format defines (base 3, most significant digit first, scaled
    to a byte by ceil(v*256/243)) and read them back"""
    rng = np.random.default_rng(8)
    trits = rng.integers(0, 3, 256)
    blk = np.zeros(54, np.uint8)
    blk[52:54] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)

    def pack(digits):  # digits[0] is read first (n = 0)
        v = 0
        for t in digits:
            v = v * 3 + int(t)
        v *= 3 ** (5 - len(digits))
        return (v * 256 + 242) // 243
    for m in range(32):
        blk[m] = pack([trits[32 * n + m] for n in range(5)])
    for m in range(16):
        blk[32 + m] = pack([trits[160 + 16 * n + m] for n in range(5)])
    for j in range(4):
        blk[48 + j] = pack([trits[240 + 4 * n + j] for n in range(4)])
    _, y = oracle.dequant_row(synth.GGML_TQ1_0, blk, 256)
    assert np.array_equal(y, (trits - 1).astype(np.float32))


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
