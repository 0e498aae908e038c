"""Element-indexed closed forms of the seven block formats, in numpy float64.

An independent statement of the arithmetic (one formula per output element instead of the
reference's nested loops), used to pin the oracle: every product of an fp16 scale, a 6..8-bit
integer scale and a <=6-bit quant is exact in fp32, so evaluating the formula in float64 and
rounding ONCE to fp32 must reproduce the decoder bit for bit on finite inputs. Only block
layouts (byte offsets) are shared with the code under test; the index algebra is restated here.
"""
import numpy as np

IQ4NL = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float64)


def f16(lo, hi):
    """two uint8 arrays -> float64 value of the IEEE half they spell"""
    bits = (lo.astype(np.uint16) | (hi.astype(np.uint16) << 8))
    return bits.view(np.float16).astype(np.float64)


def _blocks(row, bb):
    row = np.asarray(row, np.uint8)
    return row.reshape(-1, bb)


def q8_0(row):
    b = _blocks(row, 34)
    d = f16(b[:, 0], b[:, 1])
    return (d[:, None] * b[:, 2:].view(np.int8).astype(np.float64)).ravel()


def _k4_fields(s):
    """s: [nb,12] -> sc[nb,8], mn[nb,8] for sub-block g of element k (g = k >> 5)"""
    s = s.astype(np.int64)
    sc = np.zeros((s.shape[0], 8), np.int64)
    mn = np.zeros((s.shape[0], 8), np.int64)
    for g in range(8):
        if g < 4:
            sc[:, g] = s[:, g] & 63
            mn[:, g] = s[:, g + 4] & 63
        else:
            sc[:, g] = (s[:, g + 4] & 15) | ((s[:, g - 4] >> 6) << 4)
            mn[:, g] = (s[:, g + 4] >> 4) | ((s[:, g] >> 6) << 4)
    return sc, mn


def q4_K(row):
    b = _blocks(row, 144)
    d, dmin = f16(b[:, 0], b[:, 1]), f16(b[:, 2], b[:, 3])
    sc, mn = _k4_fields(b[:, 4:16])
    k = np.arange(256)
    g, l = k >> 5, k & 31
    byte = b[:, 16 + (g >> 1) * 32 + l].astype(np.int64)
    q = np.where(g & 1, byte >> 4, byte & 15)
    return (d[:, None] * sc[:, g] * q - dmin[:, None] * mn[:, g]).ravel()


def q5_K(row):
    b = _blocks(row, 176)
    d, dmin = f16(b[:, 0], b[:, 1]), f16(b[:, 2], b[:, 3])
    sc, mn = _k4_fields(b[:, 4:16])
    k = np.arange(256)
    g, l = k >> 5, k & 31
    byte = b[:, 48 + (g >> 1) * 32 + l].astype(np.int64)
    q = np.where(g & 1, byte >> 4, byte & 15) + 16 * ((b[:, 16 + l].astype(np.int64) >> g) & 1)
    return (d[:, None] * sc[:, g] * q - dmin[:, None] * mn[:, g]).ravel()


def q6_K(row):
    b = _blocks(row, 210)
    d = f16(b[:, 208], b[:, 209])
    k = np.arange(256)
    half, r = k >> 7, k & 127
    seg, l = r >> 5, r & 31
    qlb = b[:, half * 64 + l + (seg & 1) * 32].astype(np.int64)
    nib = np.where(seg >= 2, qlb >> 4, qlb & 15)
    hi2 = (b[:, 128 + half * 32 + l].astype(np.int64) >> (2 * seg)) & 3
    q = (nib | (hi2 << 4)) - 32
    sc = b[:, 192 + half * 8 + (l >> 4) + 2 * seg].view(np.int8).astype(np.float64)
    return (d[:, None] * sc * q).ravel()


def iq4_nl(row):
    b = _blocks(row, 18)
    d = f16(b[:, 0], b[:, 1])
    k = np.arange(32)
    byte = b[:, 2 + (k & 15)].astype(np.int64)
    nib = np.where(k < 16, byte & 15, byte >> 4)
    return (d[:, None] * IQ4NL[nib]).ravel()


def _parity(v):
    v = v ^ (v >> 4)
    v = v ^ (v >> 2)
    v = v ^ (v >> 1)
    return v & 1


def iq2_xxs(row, grid_bytes):
    """grid_bytes: the 2048-byte memory image of the 256 x u64 grid"""
    grid = np.frombuffer(grid_bytes, np.uint8).reshape(256, 8).astype(np.float64)
    b = _blocks(row, 66)
    d = f16(b[:, 0], b[:, 1])
    q = b[:, 2:].astype(np.uint64)
    k = np.arange(256)
    ib, l, j = k >> 5, (k & 31) >> 3, k & 7
    a0 = q[:, 8 * ib] | (q[:, 8 * ib + 1] << 8) | (q[:, 8 * ib + 2] << 16) | (q[:, 8 * ib + 3] << 24)
    a1 = q[:, 8 * ib + 4] | (q[:, 8 * ib + 5] << 8) | (q[:, 8 * ib + 6] << 16) | (q[:, 8 * ib + 7] << 24)
    db = d[:, None] * (0.5 + (a1 >> 28).astype(np.float64)) * 0.25
    gidx = ((a0 >> (8 * l).astype(np.uint64)) & 255).astype(np.int64)
    mag = grid[gidx, j]
    s7 = ((a1 >> (7 * l).astype(np.uint64)) & 127).astype(np.int64)
    sbyte = s7 | (_parity(s7) << 7)
    sign = np.where((sbyte >> j) & 1, -1.0, 1.0)
    return (db * mag * sign).ravel()


def iq3_s(row, grid_bytes):
    """grid_bytes: the 2048-byte memory image of the 512 x u32 grid"""
    grid = np.frombuffer(grid_bytes, np.uint8).reshape(512, 4).astype(np.float64)
    b = _blocks(row, 110).astype(np.int64)
    d = f16(b[:, 0].astype(np.uint8), b[:, 1].astype(np.uint8))
    k = np.arange(256)
    ib, l, j = k >> 5, (k & 31) >> 3, k & 7
    sbyte = b[:, 106 + (ib >> 1)]
    nib = np.where(ib & 1, sbyte >> 4, sbyte & 15)
    db = d[:, None] * (1 + 2 * nib)
    qs = b[:, 2 + 8 * ib + 2 * l + (j >> 2)]
    ninth = (b[:, 66 + ib] >> (2 * l + (j >> 2))) & 1
    mag = grid[qs | (ninth << 8), j & 3]
    sign = np.where((b[:, 74 + 4 * ib + l] >> j) & 1, -1.0, 1.0)
    return (db * mag * sign).ravel()


# ---- the further block formats ----
# names of the codebooks (memory images) a formula takes after the row, in order
TABLE_ARGS = {"iq2_xxs": ("iq2xxs_grid",), "iq3_s": ("iq3s_grid",), "iq3_xxs": ("iq3xxs_grid",),
              "iq2_xs": ("iq2xs_grid",), "iq2_s": ("iq2s_grid",), "iq1_s": ("iq1s_grid",),
              "iq1_m": ("iq1s_grid",)}

E2M1X2 = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.float64)


def _nibble32(b, off):
    """[nb,32] 4-bit codes of a 32-element block: element k<16 low nibble of byte off+k, else high of off+k-16"""
    k = np.arange(32)
    byte = b[:, off + (k & 15)].astype(np.int64)
    return np.where(k < 16, byte & 15, byte >> 4)


def _fifth_bits(b, off):
    k = np.arange(32)
    return (b[:, off + (k >> 3)].astype(np.int64) >> (k & 7)) & 1


def q4_0(row):
    b = _blocks(row, 18)
    return (f16(b[:, 0], b[:, 1])[:, None] * (_nibble32(b, 2) - 8)).ravel()


def q4_1(row):
    b = _blocks(row, 20)
    return (f16(b[:, 0], b[:, 1])[:, None] * _nibble32(b, 4) + f16(b[:, 2], b[:, 3])[:, None]).ravel()


def q5_0(row):
    b = _blocks(row, 22)
    return (f16(b[:, 0], b[:, 1])[:, None] * (_nibble32(b, 6) + 16 * _fifth_bits(b, 2) - 16)).ravel()


def q5_1(row):
    b = _blocks(row, 24)
    q = _nibble32(b, 8) + 16 * _fifth_bits(b, 4)
    return (f16(b[:, 0], b[:, 1])[:, None] * q + f16(b[:, 2], b[:, 3])[:, None]).ravel()


def mxfp4(row):
    b = _blocks(row, 17)
    d = np.ldexp(1.0, b[:, 0].astype(np.int64) - 128)  # half of 2^(e-127)
    return (d[:, None] * E2M1X2[_nibble32(b, 1)]).ravel()


def _ue4m3_half(x):
    x = x.astype(np.int64)
    e, m = (x >> 3) & 15, x & 7
    v = np.where(e == 0, np.ldexp(m.astype(np.float64), -10), np.ldexp(8.0 + m, e - 11))
    return np.where((x == 0) | (x == 0x7F), 0.0, v)


def nvfp4(row):
    b = _blocks(row, 36)
    k = np.arange(64)
    s, j = k >> 4, k & 15
    byte = b[:, 4 + 8 * s + (j & 7)].astype(np.int64)
    code = np.where(j < 8, byte & 15, byte >> 4)
    return (_ue4m3_half(b[:, s]) * E2M1X2[code]).ravel()


def q1_0(row):
    b = _blocks(row, 18)
    k = np.arange(128)
    bit = (b[:, 2 + (k >> 3)].astype(np.int64) >> (k & 7)) & 1
    return (f16(b[:, 0], b[:, 1])[:, None] * (2 * bit - 1)).ravel()


def _k2_index():
    k = np.arange(256)
    half, j, sub, l = k >> 7, (k >> 5) & 3, (k >> 4) & 1, k & 15
    return half, j, sub, l


def q2_K(row):
    b = _blocks(row, 84)
    d, dmin = f16(b[:, 80], b[:, 81]), f16(b[:, 82], b[:, 83])
    half, j, sub, l = _k2_index()
    sc = b[:, 8 * half + 2 * j + sub].astype(np.int64)
    q = (b[:, 16 + 32 * half + 16 * sub + l].astype(np.int64) >> (2 * j)) & 3
    return (d[:, None] * (sc & 15) * q - dmin[:, None] * (sc >> 4)).ravel()


def q3_K(row):
    b = _blocks(row, 110)
    d = f16(b[:, 108], b[:, 109])
    half, j, sub, l = _k2_index()
    i = 8 * half + 2 * j + sub  # scale index
    s = b[:, 96:108].astype(np.int64)
    lo = np.where(i < 8, s[:, i % 8] & 15, s[:, i % 8] >> 4)
    hi = (s[:, 8 + (i & 3)] >> (2 * (i >> 2))) & 3
    sc = (lo | (hi << 4)) - 32
    low2 = (b[:, 32 + 32 * half + 16 * sub + l].astype(np.int64) >> (2 * j)) & 3
    hbit = (b[:, 16 * sub + l].astype(np.int64) >> (4 * half + j)) & 1
    return (d[:, None] * sc * (low2 - 4 * (1 - hbit))).ravel()


def _group_index():
    k = np.arange(256)
    return k >> 5, (k & 31) >> 3, k & 7


def _u16_at(b, off):
    return b[:, off].astype(np.int64) | (b[:, off + 1].astype(np.int64) << 8)


def _signs(byte, j):
    return np.where((byte >> j) & 1, -1.0, 1.0)


def iq3_xxs(row, grid_bytes):
    grid = np.frombuffer(grid_bytes, np.uint8).reshape(256, 4).astype(np.float64)
    b = _blocks(row, 98)
    d = f16(b[:, 0], b[:, 1])
    g, l, j = _group_index()
    w = _u16_at(b, 66 + 4 * g) | (_u16_at(b, 68 + 4 * g) << 16)
    db = d[:, None] * (0.5 + (w >> 28)) * 0.5
    s7 = (w >> (7 * l)) & 127
    mag = grid[b[:, 2 + 8 * g + 2 * l + (j >> 2)].astype(np.int64), j & 3]
    return (db * mag * _signs(s7 | (_parity(s7) << 7), j)).ravel()


def iq4_xs(row):
    b = _blocks(row, 136)
    d = f16(b[:, 0], b[:, 1])
    k = np.arange(256)
    g, r = k >> 5, k & 31
    sl = b[:, 4 + (g >> 1)].astype(np.int64)
    ls = np.where(g & 1, sl >> 4, sl & 15) | (((_u16_at(b, 2)[:, None] >> (2 * g)) & 3) << 4)
    byte = b[:, 8 + 16 * g + (r & 15)].astype(np.int64)
    code = np.where(r < 16, byte & 15, byte >> 4)
    return (d[:, None] * (ls - 32) * IQ4NL[code]).ravel()


def _scale_nibble(b, off, g, l):
    sb = b[:, off + g].astype(np.int64)
    return np.where(l >= 2, sb >> 4, sb & 15)


def iq2_xs(row, grid_bytes):
    grid = np.frombuffer(grid_bytes, np.uint8).reshape(512, 8).astype(np.float64)
    b = _blocks(row, 74)
    d = f16(b[:, 0], b[:, 1])
    g, l, j = _group_index()
    db = d[:, None] * (0.5 + _scale_nibble(b, 66, g, l)) * 0.25
    w = _u16_at(b, 2 + 2 * (4 * g + l))
    s7 = w >> 9
    return (db * grid[w & 511, j] * _signs(s7 | (_parity(s7) << 7), j)).ravel()


def iq2_s(row, grid_bytes):
    grid = np.frombuffer(grid_bytes, np.uint8).reshape(1024, 8).astype(np.float64)
    b = _blocks(row, 82)
    d = f16(b[:, 0], b[:, 1])
    g, l, j = _group_index()
    db = d[:, None] * (0.5 + _scale_nibble(b, 74, g, l)) * 0.25
    idx = b[:, 2 + 4 * g + l].astype(np.int64) | (((b[:, 66 + g].astype(np.int64) >> (2 * l)) & 3) << 8)
    return (db * grid[idx, j] * _signs(b[:, 34 + 4 * g + l].astype(np.int64), j)).ravel()


def iq1_s(row, grid_bytes):
    grid = np.frombuffer(grid_bytes, np.int8).reshape(2048, 8).astype(np.float64)
    b = _blocks(row, 50)
    d = f16(b[:, 0], b[:, 1])
    g, l, j = _group_index()
    h = _u16_at(b, 34 + 2 * g)
    dl = d[:, None] * (2 * ((h >> 12) & 7) + 1)
    delta = np.where(h & 0x8000, -0.125, 0.125)
    idx = b[:, 2 + 4 * g + l].astype(np.int64) | (((h >> (3 * l)) & 7) << 8)
    return (dl * (grid[idx, j] + delta)).ravel()


def iq1_m(row, grid_bytes):
    grid = np.frombuffer(grid_bytes, np.int8).reshape(2048, 8).astype(np.float64)
    b = _blocks(row, 56)
    sw = [_u16_at(b, 48 + 2 * w) for w in range(4)]
    dbits = (sw[0] >> 12) | ((sw[1] >> 12) << 4) | ((sw[2] >> 12) << 8) | ((sw[3] >> 12) << 12)
    d = dbits.astype(np.uint16).view(np.float16).astype(np.float64)
    g, l, j = _group_index()
    word = np.stack(sw, axis=1)[:, g >> 1]
    dl = d[:, None] * (2 * ((word >> (6 * (g & 1) + 3 * (l >> 1))) & 7) + 1)
    nib = (b[:, 32 + 2 * g + (l >> 1)].astype(np.int64) >> (4 * (l & 1))) & 15
    delta = np.where(nib & 8, -0.125, 0.125)
    idx = b[:, 4 * g + l].astype(np.int64) | ((nib & 7) << 8)
    return (dl * (grid[idx, j] + delta)).ravel()


def _trit(byte, n):
    return ((((byte.astype(np.int64) * 3 ** n) & 255) * 3) >> 8) - 1


def tq1_0(row):
    b = _blocks(row, 54)
    d = f16(b[:, 52], b[:, 53])
    k = np.arange(256)
    byte_at = np.where(k < 160, k & 31, np.where(k < 240, 32 + ((k - 160) & 15), 48 + ((k - 240) & 3)))
    digit = np.where(k < 160, k >> 5, np.where(k < 240, (k - 160) >> 4, (k - 240) >> 2))
    return (d[:, None] * _trit(b[:, byte_at], digit)).ravel()


def tq2_0(row):
    b = _blocks(row, 66)
    d = f16(b[:, 64], b[:, 65])
    k = np.arange(256)
    q = (b[:, 32 * (k >> 7) + (k & 31)].astype(np.int64) >> (2 * ((k >> 5) & 3))) & 3
    return (d[:, None] * (q - 1)).ravel()
