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
