"""ctypes front end of the CPU oracle (oracle/liboracle.so) and, where it was built, of the
compiled reference (oracle/_ref/libref.so).

TEST INFRASTRUCTURE ONLY: the checker and the reported CPU baseline, never the product path.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_SO = os.path.join(_HERE, "liboracle.so")
_REF_SO = os.path.join(_HERE, "_ref", "libref.so")

# enum ggml_dtype values (common/gguf_loader.h:45-85)
F32, F16, Q8_0, Q4_K, Q5_K, Q6_K, IQ2_XXS, IQ4_NL, IQ3_S, BF16 = 0, 1, 8, 12, 13, 14, 16, 20, 21, 30
BLOCK_TYPES = {"q8_0": Q8_0, "q4_K": Q4_K, "q5_K": Q5_K, "q6_K": Q6_K,
               "iq2_xxs": IQ2_XXS, "iq4_nl": IQ4_NL, "iq3_s": IQ3_S,
               "q4_0": 2, "q4_1": 3, "q5_0": 6, "q5_1": 7, "q2_K": 10, "q3_K": 11, "iq2_xs": 17,
               "iq3_xxs": 18, "iq1_s": 19, "iq2_s": 22, "iq4_xs": 23, "iq1_m": 29, "tq1_0": 34,
               "tq2_0": 35, "mxfp4": 39, "nvfp4": 40, "q1_0": 41}

_vp, _fp, _ip = C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_int)


def build(force=False):
    """Compile liboracle.so (and _ref/libref.so when the reference checkout is present)."""
    if force or not os.path.exists(_ORACLE_SO):
        subprocess.check_call(["make", "-C", _HERE, "-s", "all"])


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_fp)


def _u8(a):
    a = np.ascontiguousarray(a, dtype=np.uint8)
    return a, a.ctypes.data_as(_vp)


class Oracle:
    """The oracle's C functions on numpy arrays. Weight matrices are uint8 [n_rows, row_bytes]."""

    def __init__(self):
        build()
        L = self.lib = C.CDLL(_ORACLE_SO)
        L.qo_fp16_to_fp32.restype = C.c_float
        L.qo_fp16_to_fp32.argtypes = [C.c_uint16]
        L.qo_row_size.restype = C.c_size_t
        L.qo_row_size.argtypes = [C.c_uint32, C.c_int]
        L.qo_block_elems.argtypes = L.qo_block_bytes.argtypes = [C.c_uint32]
        L.qo_dequant_row.argtypes = [C.c_uint32, _vp, _fp, C.c_int]
        for name in BLOCK_TYPES:
            getattr(L, "qo_dequantize_row_" + name).argtypes = [_vp, _fp, C.c_int]
            getattr(L, "qo_dequantize_row_" + name).restype = None
        L.qo_k4_unpack_scales.argtypes = L.qo_k4_pack_scales.argtypes = [_vp, _vp, _vp]
        L.qo_table.restype = _vp
        L.qo_table.argtypes = [C.c_char_p, C.POINTER(C.c_size_t)]
        L.qo_gemv_f64.argtypes = [C.c_uint32, _vp, _fp, _fp, C.c_int, C.c_int]
        L.qo_gemv_f32.argtypes = [C.c_uint32, _vp, _fp, _fp, C.c_int, C.c_int, C.c_int]
        L.qo_gemv_f32_time.restype = C.c_double
        L.qo_gemv_f32_time.argtypes = [C.c_uint32, _vp, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_int]
        for f in (L.qo_gemm_tokmajor_f64, L.qo_gemm_tokmajor_f32):
            f.argtypes = [C.c_uint32, _vp, _fp, _fp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
        L.qo_moe_route.restype = None
        L.qo_moe_route.argtypes = [_fp, C.c_int, C.c_int, _ip, _fp]
        for f in (L.qo_moe_ffn_token_f64, L.qo_moe_ffn_token_f32):
            f.argtypes = [C.c_uint32, _vp, _vp, _vp, C.c_int, C.c_int, _fp, _ip, _fp, C.c_int, _fp]
        L.qo_moe_ffn_token_types.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, _vp, _vp, _vp, C.c_int, C.c_int, _fp, _ip,
                                             _fp, C.c_int, _fp, C.c_int]

    # ---- codec
    def fp16_table(self):
        out = np.zeros(65536, np.float32)
        self.lib.qo_fp16_table.restype = None
        self.lib.qo_fp16_table.argtypes = [_fp]
        self.lib.qo_fp16_table(out.ctypes.data_as(_fp))
        return out

    def row_size(self, type_id, n):
        return int(self.lib.qo_row_size(type_id, n))

    def block_elems(self, type_id):
        return int(self.lib.qo_block_elems(type_id))

    def block_bytes(self, type_id):
        return int(self.lib.qo_block_bytes(type_id))

    def dequant_row(self, type_id, src, n):
        src, ps = _u8(src)
        dst = np.zeros(n, dtype=np.float32)
        rc = self.lib.qo_dequant_row(type_id, ps, dst.ctypes.data_as(_fp), n)
        return rc, dst

    def dequantize_named(self, name, src, n):
        src, ps = _u8(src)
        dst = np.zeros(n, dtype=np.float32)
        getattr(self.lib, "qo_dequantize_row_" + name)(ps, dst.ctypes.data_as(_fp), n)
        return dst

    def dequant_matrix(self, type_id, W, n_cols):
        W = np.ascontiguousarray(W, dtype=np.uint8)
        out = np.zeros((W.shape[0], n_cols), dtype=np.float32)
        for r in range(W.shape[0]):
            rc = self.lib.qo_dequant_row(type_id, W[r].ctypes.data_as(_vp), out[r].ctypes.data_as(_fp), n_cols)
            assert rc == 0
        return out

    def k4_unpack(self, packed):
        packed, pp = _u8(packed)
        sc, mn = np.zeros(8, np.uint8), np.zeros(8, np.uint8)
        self.lib.qo_k4_unpack_scales(pp, sc.ctypes.data_as(_vp), mn.ctypes.data_as(_vp))
        return sc, mn

    def k4_pack(self, sc, mn):
        sc, ps = _u8(sc)
        mn, pm = _u8(mn)
        out = np.zeros(12, np.uint8)
        self.lib.qo_k4_pack_scales(ps, pm, out.ctypes.data_as(_vp))
        return out

    def table(self, name):
        n = C.c_size_t(0)
        p = self.lib.qo_table(name.encode(), C.byref(n))
        return bytes(C.string_at(p, n.value)) if p else None

    # ---- linear
    def gemv_f64(self, type_id, W, x, n_cols):
        W, pw = _u8(W)
        x, px = _f32(x)
        y = np.zeros(W.shape[0], np.float32)
        rc = self.lib.qo_gemv_f64(type_id, pw, px, y.ctypes.data_as(_fp), W.shape[0], n_cols)
        assert rc == 0, rc
        return y

    def gemv_f32(self, type_id, W, x, n_cols, n_threads=1):
        W, pw = _u8(W)
        x, px = _f32(x)
        y = np.zeros(W.shape[0], np.float32)
        rc = self.lib.qo_gemv_f32(type_id, pw, px, y.ctypes.data_as(_fp), W.shape[0], n_cols, n_threads)
        assert rc == 0, rc
        return y

    def gemv_f32_time(self, type_id, W, x, n_cols, n_threads, iters):
        W, pw = _u8(W)
        x, px = _f32(x)
        y = np.zeros(W.shape[0], np.float32)
        return float(self.lib.qo_gemv_f32_time(type_id, pw, px, y.ctypes.data_as(_fp), W.shape[0], n_cols,
                                               n_threads, iters))

    def gemm_tokmajor(self, type_id, W, X, n_cols, f64=True):
        """X float32 [n_tok, n_cols] -> Y float32 [n_tok, n_rows]"""
        W, pw = _u8(W)
        X, px = _f32(X)
        n_tok, n_rows = X.shape[0], W.shape[0]
        Y = np.zeros((n_tok, n_rows), np.float32)
        fn = self.lib.qo_gemm_tokmajor_f64 if f64 else self.lib.qo_gemm_tokmajor_f32
        rc = fn(type_id, pw, px, Y.ctypes.data_as(_fp), n_rows, n_cols, n_tok, n_rows, X.shape[1])
        assert rc == 0, rc
        return Y

    def moe_route(self, logits, top_k):
        logits, pl = _f32(logits)
        idx = np.zeros(top_k, np.int32)
        w = np.zeros(top_k, np.float32)
        self.lib.qo_moe_route(pl, logits.shape[0], top_k, idx.ctypes.data_as(_ip), w.ctypes.data_as(_fp))
        return idx, w

    def moe_ffn_token(self, type_id, gate, up, down, n_embd, n_ff, x, idx, w, f64=True):
        gate, pg = _u8(gate)
        up, pu = _u8(up)
        down, pd = _u8(down)
        x, px = _f32(x)
        idx = np.ascontiguousarray(idx, np.int32)
        w, pw = _f32(w)
        out = np.zeros(n_embd, np.float32)
        fn = self.lib.qo_moe_ffn_token_f64 if f64 else self.lib.qo_moe_ffn_token_f32
        rc = fn(type_id, pg, pu, pd, n_embd, n_ff, px, idx.ctypes.data_as(_ip), pw, len(idx),
                out.ctypes.data_as(_fp))
        assert rc == 0, rc
        return out

    def moe_ffn_token_types(self, types, gate, up, down, n_embd, n_ff, x, idx, w, f64=True):
        """the three expert tensors in a format each (gate, up, down)"""
        gate, pg = _u8(gate)
        up, pu = _u8(up)
        down, pd = _u8(down)
        x, px = _f32(x)
        idx = np.ascontiguousarray(idx, np.int32)
        w, pw = _f32(w)
        out = np.zeros(n_embd, np.float32)
        rc = self.lib.qo_moe_ffn_token_types(types[0], types[1], types[2], pg, pu, pd, n_embd, n_ff, px,
                                             idx.ctypes.data_as(_ip), pw, len(idx), out.ctypes.data_as(_fp), 1 if f64 else 0)
        assert rc == 0, rc
        return out


class Reference:
    """The reference's own functions, compiled from its sources (oracle/_ref/libref.so).
    `available()` is False where that library was not built (e.g. no reference checkout)."""

    @staticmethod
    def available():
        return os.path.exists(_REF_SO)

    def __init__(self):
        L = self.lib = C.CDLL(_REF_SO)
        L.ref_fp16_to_fp32.restype = C.c_float
        L.ref_fp16_to_fp32.argtypes = [C.c_uint16]
        L.ref_dequant_row.argtypes = [C.c_uint32, _vp, _fp, C.c_int]
        L.ref_dequant_row_size.restype = C.c_size_t
        L.ref_dequant_row_size.argtypes = [C.c_uint32, C.c_int]
        L.ref_tf_row_bytes.restype = C.c_size_t
        L.ref_tf_row_bytes.argtypes = [C.c_uint32, C.c_int]
        L.ref_tf_qmatvec.restype = L.ref_tf_qmatvec_f64.restype = None
        L.ref_tf_qmatvec.argtypes = L.ref_tf_qmatvec_f64.argtypes = [_fp, _vp, C.c_uint32, _fp, C.c_int, C.c_int]
        L.ref_tf_qmatvec_expert.restype = None
        L.ref_tf_qmatvec_expert.argtypes = [_fp, _vp, C.c_uint32, C.c_int, _fp, C.c_int, C.c_int]
        L.ref_tf_gemm_tokenmajor.restype = None
        L.ref_tf_gemm_tokenmajor.argtypes = [_fp, _vp, C.c_uint32, _fp, C.c_int, C.c_int, C.c_int, C.c_int,
                                             C.c_int, C.c_int]
        L.ref_tf_softmax.restype = None
        L.ref_tf_softmax.argtypes = [_fp, C.c_int]
        L.ref_tf_silu_mul.restype = None
        L.ref_tf_silu_mul.argtypes = [_fp, _fp, _fp, C.c_int]
        L.ref_tf_qmatvec_pool_time.restype = C.c_double
        L.ref_tf_qmatvec_pool_time.argtypes = [_fp, _vp, C.c_uint32, _fp, C.c_int, C.c_int, C.c_int, C.c_int]
        L.ref_table.restype = _vp
        L.ref_table.argtypes = [C.c_char_p, C.POINTER(C.c_size_t)]

    def fp16_table(self):
        out = np.zeros(65536, np.float32)
        self.lib.ref_fp16_table.restype = None
        self.lib.ref_fp16_table.argtypes = [_fp]
        self.lib.ref_fp16_table(out.ctypes.data_as(_fp))
        return out

    def row_size(self, type_id, n):
        return int(self.lib.ref_dequant_row_size(type_id, n))

    def tf_row_bytes(self, type_id, n_cols):
        return int(self.lib.ref_tf_row_bytes(type_id, n_cols))

    def dequant_row(self, type_id, src, n):
        src, ps = _u8(src)
        dst = np.zeros(n, dtype=np.float32)
        rc = self.lib.ref_dequant_row(type_id, ps, dst.ctypes.data_as(_fp), n)
        return rc, dst

    def qmatvec(self, type_id, W, x, n_cols, f64=False):
        W, pw = _u8(W)
        x, px = _f32(x)
        y = np.zeros(W.shape[0], np.float32)
        fn = self.lib.ref_tf_qmatvec_f64 if f64 else self.lib.ref_tf_qmatvec
        fn(y.ctypes.data_as(_fp), pw, type_id, px, W.shape[0], n_cols)
        return y

    def qmatvec_expert(self, type_id, W, expert, x, rows_per_expert, n_cols):
        W, pw = _u8(W)
        x, px = _f32(x)
        y = np.zeros(rows_per_expert, np.float32)
        self.lib.ref_tf_qmatvec_expert(y.ctypes.data_as(_fp), pw, type_id, expert, px, rows_per_expert, n_cols)
        return y

    def gemm_tokenmajor(self, type_id, W, X, n_cols, n_threads=1):
        W, pw = _u8(W)
        X, px = _f32(X)
        n_tok, n_rows = X.shape[0], W.shape[0]
        Y = np.zeros((n_tok, n_rows), np.float32)
        self.lib.ref_tf_gemm_tokenmajor(Y.ctypes.data_as(_fp), pw, type_id, px, n_rows, n_cols, n_tok, n_rows,
                                        X.shape[1], n_threads)
        return Y

    def softmax(self, x):
        """tf_softmax (common/transformer.h:1537-1586), on a copy"""
        x = np.array(x, np.float32, copy=True)
        self.lib.ref_tf_softmax(x.ctypes.data_as(_fp), x.shape[0])
        return x

    def silu_mul(self, gate, up):
        """tf_silu_mul_avx2 (common/transformer.h:4679-4694): silu(gate) * up"""
        gate, pg = _f32(gate)
        up, pu = _f32(up)
        out = np.zeros(gate.shape[0], np.float32)
        self.lib.ref_tf_silu_mul(out.ctypes.data_as(_fp), pg, pu, gate.shape[0])
        return out

    def qmatvec_pool_time(self, type_id, W, x, n_cols, n_threads, iters):
        W, pw = _u8(W)
        x, px = _f32(x)
        y = np.zeros(W.shape[0], np.float32)
        return float(self.lib.ref_tf_qmatvec_pool_time(y.ctypes.data_as(_fp), pw, type_id, px, W.shape[0], n_cols,
                                                       n_threads, iters))

    def table(self, name):
        n = C.c_size_t(0)
        p = self.lib.ref_table(name.encode(), C.byref(n))
        return bytes(C.string_at(p, n.value)) if p else None
