"""ctypes binding of libqlinear.so (the C ABI declared in include/qlinear.h).

The library is the product; this module only marshals numpy arrays and device pointers into
it. There is no fallback: if the shared library is missing or no GPU is usable, calls raise.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# QLINEAR_LIB names another build of the same library (e.g. an experimental one); default: the in-tree build
LIB_PATH = os.environ.get("QLINEAR_LIB") or os.path.join(_HERE, "libqlinear.so")

OK, ERR_TYPE, ERR_ARG, ERR_DEVICE, ERR_NOMEM = 0, -1, -2, -3, -4

_vp, _fp, _ip, _u16p = C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_int32), C.POINTER(C.c_uint16)

# name -> (restype, argtypes); every symbol include/qlinear.h declares
SIGNATURES = {
    "qlin_init": (C.c_int, [C.c_int]),
    "qlin_shutdown": (None, []),
    "qlin_last_error": (C.c_char_p, []),
    "qlin_device_info": (C.c_int, [C.c_char_p, C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_size_t)]),
    "qlin_dequant_row_size": (C.c_size_t, [C.c_uint32, C.c_int]),
    "qlin_dequant_row": (C.c_int, [C.c_uint32, _vp, _vp, C.c_int]),
    "qlin_dequantize_row_q8_0": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_q4_K": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_q5_K": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_q6_K": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_iq2_xxs": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_iq3_s": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_iq4_nl": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_q4_0": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_q4_1": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_q5_0": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_q5_1": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_q2_K": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_q3_K": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_q1_0": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_mxfp4": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_nvfp4": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_iq2_xs": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_iq2_s": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_iq3_xxs": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_iq4_xs": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_iq1_s": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_iq1_m": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_tq1_0": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_tq2_0": (None, [_vp, _vp, C.c_int]),
    "qlin_dequantize_row_bf16": (None, [_vp, _vp, C.c_int]),
    "qlin_dequant_rows": (C.c_int, [C.c_uint32, _vp, _vp, C.c_int, C.c_int]),
    "qlin_weight_register": (C.c_int, [_vp, C.c_size_t]),
    "qlin_weight_adopt": (C.c_int, [_vp, C.c_size_t, _vp]),
    "qlin_weight_unregister": (C.c_int, [_vp]),
    "qlin_weight_device_ptr": (_vp, [_vp]),
    "qlin_matvec": (C.c_int, [_vp, _vp, C.c_uint32, C.c_int, _vp, C.c_int]),
    "qlin_matvec_fused2": (C.c_int, [_vp, _vp, C.c_uint32, _vp, _vp, C.c_uint32, C.c_int, _vp, C.c_int]),
    "qlin_matvec_qkv": (C.c_int, [_vp, _vp, C.c_uint32, C.c_int, _vp, _vp, C.c_uint32, _vp, _vp, C.c_uint32,
                                  C.c_int, C.c_int, _vp]),
    "qlin_matvec_expert": (C.c_int, [_vp, _vp, C.c_uint32, C.c_int, C.c_int, _vp, C.c_int]),
    "qlin_matvec_silu_mul": (C.c_int, [_vp, _vp, C.c_uint32, _vp, C.c_uint32, C.c_int, _vp, C.c_int]),
    "qlin_matvec_add": (C.c_int, [_vp, _vp, C.c_uint32, C.c_int, _vp, C.c_int]),
    "qlin_matvec_argmax": (C.c_int, [_vp, _vp, _vp, _vp, C.c_uint32, C.c_int, _vp, C.c_int]),
    "qlin_gemm_tokenmajor": (C.c_int, [_vp, _vp, C.c_uint32, C.c_int, _vp, C.c_int, C.c_int, C.c_int, C.c_int]),
    "qlin_moe_ffn_token": (C.c_int, [_vp, _vp, _vp, _vp, C.c_uint32, C.c_int, C.c_int, C.c_int, C.c_int, _vp, _vp]),
    "qlin_moe_ffn_token_types": (C.c_int, [_vp, _vp, _vp, _vp, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int, C.c_int, C.c_int,
                                           C.c_int, _vp, _vp]),
    "qlin_dev_alloc": (_vp, [C.c_size_t]),
    "qlin_dev_free": (None, [_vp]),
    "qlin_dev_upload": (C.c_int, [_vp, _vp, C.c_size_t]),
    "qlin_dev_download": (C.c_int, [_vp, _vp, C.c_size_t]),
    "qlin_dev_sync": (C.c_int, [_vp]),
    "qlin_dequant_dev": (C.c_int, [C.c_uint32, _vp, _vp, C.c_int, C.c_int, _vp]),
    "qlin_gemv_dev": (C.c_int, [C.c_uint32, _vp, _vp, _vp, C.c_int, C.c_int, _vp]),
    "qlin_embed_rows_dev": (C.c_int, [C.c_uint32, _vp, C.c_int, _vp, C.c_int, _vp, C.c_int, _vp]),
    "qlin_gemv_add_dev": (C.c_int, [C.c_uint32, _vp, _vp, _vp, C.c_int, C.c_int, _vp]),
    "qlin_gemv_silu_mul_dev": (C.c_int, [C.c_uint32, _vp, _vp, _vp, _vp, C.c_int, C.c_int, _vp]),
    "qlin_gemv_multi_dev": (C.c_int, [C.c_uint32, C.c_int, _vp, _vp, _vp, _vp, C.c_int, _vp]),
    "qlin_gemv_argmax_dev": (C.c_int, [C.c_uint32, _vp, _vp, _vp, _vp, C.c_int, C.c_int, _vp]),
    "qlin_gemm_bf16_dev": (C.c_int, [C.c_uint32, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp]),
    "qlin_gemm_f32_dev": (C.c_int, [C.c_uint32, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp]),
    "qlin_moe_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "qlin_moe_route_dev": (C.c_int, [_vp, C.c_int, C.c_int, C.c_int, _vp, _vp, _vp]),
    "qlin_moe_ffn_dev": (C.c_int, [C.c_uint32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int,
                                   C.c_int, C.c_int, _vp, _vp]),
    "qlin_moe_ffn_types_dev": (C.c_int, [C.c_uint32, C.c_uint32, C.c_uint32, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                         C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp, _vp]),
    "qlin_moe_ffn_static_dev": (C.c_int, [C.c_uint32, C.c_uint32, C.c_uint32, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                          C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp]),
    "qlin_gguf_open": (C.c_int, [C.c_char_p, _vp]),
    "qlin_gguf_close": (None, [_vp]),
    "qlin_gguf_version": (C.c_uint32, [_vp]),
    "qlin_gguf_alignment": (C.c_uint32, [_vp]),
    "qlin_gguf_data_offset": (C.c_size_t, [_vp]),
    "qlin_gguf_data_size": (C.c_size_t, [_vp]),
    "qlin_gguf_n_tensors": (C.c_int, [_vp]),
    "qlin_gguf_find_tensor": (C.c_int, [_vp, C.c_char_p]),
    "qlin_gguf_tensor_info": (C.c_int, [_vp, C.c_int, _vp, _vp, _vp, _vp, _vp, _vp]),
    "qlin_gguf_tensor_host": (_vp, [_vp, C.c_int]),
    "qlin_gguf_tensor_dev": (_vp, [_vp, C.c_int]),
    "qlin_gguf_upload": (C.c_int, [_vp]),
    "qlin_gguf_n_kv": (C.c_int, [_vp]),
    "qlin_gguf_find_key": (C.c_int, [_vp, C.c_char_p]),
    "qlin_gguf_key": (C.c_char_p, [_vp, C.c_int]),
    "qlin_gguf_value_type": (C.c_int, [_vp, C.c_int]),
    "qlin_gguf_get_i64": (C.c_int, [_vp, C.c_int, _vp]),
    "qlin_gguf_get_f64": (C.c_int, [_vp, C.c_int, _vp]),
    "qlin_gguf_get_str": (C.c_char_p, [_vp, C.c_int]),
    "qlin_gguf_get_array": (C.c_int, [_vp, C.c_int, _vp, _vp, _vp]),
    "qlin_set_prefill_matrix_cores": (C.c_int, [C.c_int]),
    "qlin_set_dense_gemm_own": (C.c_int, [C.c_int]),
    "qlin_dequant_bf16_dev": (C.c_int, [C.c_uint32, _vp, _vp, C.c_int, C.c_int, _vp]),
    "qlin_gemm_bf16_any_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int]),
    "qlin_gemm_bf16_any_dev": (C.c_int, [C.c_uint32, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp, C.c_size_t, _vp]),
    "qlin_gemm_bf16_multi_dev": (C.c_int, [C.c_uint32, C.c_int, _vp, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int, _vp, _vp, C.c_size_t, _vp]),
    "qlin_gemm_f32_any_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int]),
    "qlin_gemm_f32_any_dev": (C.c_int, [C.c_uint32, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp, C.c_size_t, _vp]),
    "qlin_probe_mfma_bf16": (C.c_int, [C.c_int, _vp, C.POINTER(C.c_double)]),
    "qlin_probe_clocks": (C.c_int, [_vp, C.POINTER(C.c_double)]),
    "qlin_probe_hbm_read": (C.c_int, [_vp, C.c_size_t, _vp]),
    "qlin_probe_gemm_route": (C.c_int, [C.c_uint32, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "qlin_probe_gemm_tile": (C.c_int, [C.c_int, C.c_uint32, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _vp]),
    "qlin_timer_begin": (C.c_int, [_vp]),
    "qlin_timer_end": (C.c_int, [_vp, _fp]),
}

_lib = None


class QlinError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("qlinear error %d: %s" % (code, text))
        self.code = code


def load():
    """dlopen libqlinear.so and declare every entry point. Raises if the library is absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(LIB_PATH + " is missing: run `python -m gemm_amd.build` (there is no fallback)")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(rc):
    if rc != OK:
        raise QlinError(rc, load().qlin_last_error().decode(errors="replace"))


def _ptr(a):
    return a.ctypes.data_as(_vp)


def device_info():
    lib = load()
    name = C.create_string_buffer(256)
    cu, mem = C.c_int(0), C.c_size_t(0)
    check(lib.qlin_device_info(name, 256, C.byref(cu), C.byref(mem)))
    return name.value.decode(), cu.value, mem.value


class DevBuf:
    """A device allocation owned through the library (hipMalloc / hipFree)."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        self.ptr = load().qlin_dev_alloc(max(self.nbytes, 1))
        if not self.ptr:
            raise QlinError(ERR_NOMEM, load().qlin_last_error().decode())

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        if a.nbytes:
            check(load().qlin_dev_upload(b.ptr, _ptr(a), a.nbytes))
        return b

    def to_numpy(self, dtype, shape):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        if out.nbytes:
            check(load().qlin_dev_download(_ptr(out), self.ptr, out.nbytes))
        return out

    def free(self):
        if self.ptr:
            load().qlin_dev_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


# ---------------------------------------------------------------- host-pointer calls (numpy in, numpy out)

def dequant_row(type_id, src, n, dst=None):
    src = np.ascontiguousarray(src, np.uint8)
    if dst is None:
        dst = np.zeros(n, np.float32)
    rc = load().qlin_dequant_row(type_id, _ptr(src), _ptr(dst), n)
    return rc, dst


def dequant_rows(type_id, src, n_rows, n_cols):
    src = np.ascontiguousarray(src, np.uint8)
    dst = np.zeros((n_rows, n_cols), np.float32)
    check(load().qlin_dequant_rows(type_id, _ptr(src), _ptr(dst), n_rows, n_cols))
    return dst


def matvec(type_id, W, x, n_cols):
    W = np.ascontiguousarray(W, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    y = np.zeros(W.shape[0], np.float32)
    check(load().qlin_matvec(_ptr(y), _ptr(W), type_id, n_cols, _ptr(x), W.shape[0]))
    return y


def gemm_tokenmajor(type_id, W, X, n_cols):
    W = np.ascontiguousarray(W, np.uint8)
    X = np.ascontiguousarray(X, np.float32)
    Y = np.zeros((X.shape[0], W.shape[0]), np.float32)
    check(load().qlin_gemm_tokenmajor(_ptr(Y), _ptr(W), type_id, n_cols, _ptr(X), W.shape[0], X.shape[0],
                                      W.shape[0], X.shape[1]))
    return Y


# ---------------------------------------------------------------- device-resident calls

def gemv_dev(type_id, dW, dx, dy, n_rows, n_cols, stream=None):
    check(load().qlin_gemv_dev(type_id, dW.ptr, dx.ptr, dy.ptr, n_rows, n_cols, stream))


def embed_rows_dev(type_id, dtable, n_table_rows, dids, n_ids, dout, n_cols, stream=None):
    check(load().qlin_embed_rows_dev(type_id, dtable.ptr, n_table_rows, dids.ptr, n_ids, dout.ptr, n_cols, stream))


def gemv_add_dev(type_id, dW, dx, dy, n_rows, n_cols, stream=None):
    check(load().qlin_gemv_add_dev(type_id, dW.ptr, dx.ptr, dy.ptr, n_rows, n_cols, stream))


def gemv_silu_mul_dev(type_id, dWgate, dWup, dx, dout, n_rows, n_cols, stream=None):
    check(load().qlin_gemv_silu_mul_dev(type_id, dWgate.ptr, dWup.ptr, dx.ptr, dout.ptr, n_rows, n_cols, stream))


def gemv_multi_dev(type_id, dWs, dys, n_rows, dx, n_cols, stream=None):
    """dWs, dys: lists of 1..3 DevBuf; n_rows: list of ints"""
    n = len(dWs)
    Wp = (C.c_void_p * n)(*[d.ptr for d in dWs])
    yp = (C.c_void_p * n)(*[d.ptr for d in dys])
    rows = (C.c_int * n)(*n_rows)
    check(load().qlin_gemv_multi_dev(type_id, n, C.addressof(Wp), C.addressof(yp), C.addressof(rows), dx.ptr, n_cols,
                                     stream))


ARGMAX_RESULT_BYTES = 2056  # QLIN_ARGMAX_RESULT_BYTES of include/qlinear.h


def gemv_argmax_dev(type_id, dW, dx, dlogits, dresult, n_rows, n_cols, stream=None):
    check(load().qlin_gemv_argmax_dev(type_id, dW.ptr, dx.ptr, dlogits.ptr, dresult.ptr, n_rows, n_cols, stream))


def matvec_silu_mul(type_gate, Wgate, type_up, Wup, x, n_cols):
    Wgate, Wup = np.ascontiguousarray(Wgate, np.uint8), np.ascontiguousarray(Wup, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    y = np.zeros(Wgate.shape[0], np.float32)
    check(load().qlin_matvec_silu_mul(_ptr(y), _ptr(Wgate), type_gate, _ptr(Wup), type_up, n_cols, _ptr(x),
                                      Wgate.shape[0]))
    return y


def matvec_add(type_id, W, x, n_cols, residual):
    W = np.ascontiguousarray(W, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    y = np.array(residual, dtype=np.float32, copy=True)
    check(load().qlin_matvec_add(_ptr(y), _ptr(W), type_id, n_cols, _ptr(x), W.shape[0]))
    return y


def matvec_argmax(type_id, W, x, n_cols, want_logits=False):
    """-> (index, value, logits or None)"""
    W = np.ascontiguousarray(W, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    idx = np.zeros(1, np.int32)
    val = np.zeros(1, np.float32)
    logits = np.zeros(W.shape[0], np.float32) if want_logits else None
    check(load().qlin_matvec_argmax(_ptr(idx), _ptr(val), _ptr(logits) if want_logits else None, _ptr(W), type_id,
                                    n_cols, _ptr(x), W.shape[0]))
    return int(idx[0]), float(val[0]), logits


def dequant_dev(type_id, dW, dout, n_rows, n_cols, stream=None):
    check(load().qlin_dequant_dev(type_id, dW.ptr, dout.ptr, n_rows, n_cols, stream))


def gemm_bf16_dev(type_id, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy, stream=None):
    check(load().qlin_gemm_bf16_dev(type_id, dW.ptr, dX.ptr, dY.ptr, n_rows, n_cols, n_tok, ldx, ldy, stream))


def gemm_f32_dev(type_id, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy, stream=None):
    check(load().qlin_gemm_f32_dev(type_id, dW.ptr, dX.ptr, dY.ptr, n_rows, n_cols, n_tok, ldx, ldy, stream))


def dequant_bf16_dev(type_id, dW, dout, n_rows, n_cols, stream=None):
    check(load().qlin_dequant_bf16_dev(type_id, dW.ptr, dout.ptr, n_rows, n_cols, stream))


def gemm_bf16_any_workspace_bytes(n_rows, n_cols):
    return load().qlin_gemm_bf16_any_workspace_bytes(n_rows, n_cols)


def gemm_bf16_any_dev(type_id, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy, dws, stream=None):
    check(load().qlin_gemm_bf16_any_dev(type_id, dW.ptr, dX.ptr, dY.ptr, n_rows, n_cols, n_tok, ldx, ldy,
                                        dws.ptr if dws is not None else None, dws.nbytes if dws is not None else 0, stream))


def gemm_bf16_multi_dev(type_id, dWs, dX, dYs, n_rows, n_cols, n_tok, ldx, ldys, dws, stream=None):
    """dWs, dYs: lists of DevBuf; n_rows, ldys: lists of int (one entry per tensor)"""
    n = len(dWs)
    Wp = (C.c_void_p * n)(*[b.ptr for b in dWs])
    Yp = (C.c_void_p * n)(*[b.ptr for b in dYs])
    rows = (C.c_int * n)(*n_rows)
    ld = (C.c_int * n)(*ldys)
    check(load().qlin_gemm_bf16_multi_dev(type_id, n, Wp, dX.ptr, Yp, rows, n_cols, n_tok, ldx, ld,
                                          dws.ptr if dws is not None else None, dws.nbytes if dws is not None else 0, stream))


def gemm_f32_any_workspace_bytes(n_rows, n_cols):
    return load().qlin_gemm_f32_any_workspace_bytes(n_rows, n_cols)


def gemm_f32_any_dev(type_id, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy, dws, stream=None):
    check(load().qlin_gemm_f32_any_dev(type_id, dW.ptr, dX.ptr, dY.ptr, n_rows, n_cols, n_tok, ldx, ldy,
                                       dws.ptr if dws is not None else None, dws.nbytes if dws is not None else 0, stream))


def moe_workspace_bytes(n_tok, top_k, n_embd, n_ff, n_expert):
    return load().qlin_moe_workspace_bytes(n_tok, top_k, n_embd, n_ff, n_expert)


def moe_route_dev(dlogits, n_tok, n_expert, top_k, didx, dw, stream=None):
    check(load().qlin_moe_route_dev(dlogits.ptr, n_tok, n_expert, top_k, didx.ptr, dw.ptr, stream))


def moe_ffn_dev(type_id, dgate, dup, ddown, dX, didx, dw, dout, n_tok, top_k, n_embd, n_ff, n_expert, dws,
                stream=None):
    check(load().qlin_moe_ffn_dev(type_id, dgate.ptr, dup.ptr, ddown.ptr, dX.ptr, didx.ptr, dw.ptr, dout.ptr,
                                  n_tok, top_k, n_embd, n_ff, n_expert, dws.ptr, stream))


def moe_ffn_types_dev(types, dgate, dup, ddown, dX, didx, dw, dout, n_tok, top_k, n_embd, n_ff, n_expert, dws, stream=None):
    check(load().qlin_moe_ffn_types_dev(types[0], types[1], types[2], dgate.ptr, dup.ptr, ddown.ptr, dX.ptr, didx.ptr,
                                        dw.ptr, dout.ptr, n_tok, top_k, n_embd, n_ff, n_expert, dws.ptr, stream))


def moe_ffn_static_dev(types, dgate, dup, ddown, dX, didx, dw, dout, n_tok, top_k, n_embd, n_ff, n_expert, stream=None):
    check(load().qlin_moe_ffn_static_dev(types[0], types[1], types[2], dgate.ptr, dup.ptr, ddown.ptr, dX.ptr, didx.ptr,
                                         dw.ptr, dout.ptr, n_tok, top_k, n_embd, n_ff, n_expert, stream))


def sync(stream=None):
    check(load().qlin_dev_sync(stream))


def probe_mfma_bf16(iters, stream=None):
    """Enqueue the register-only MFMA loop; returns the flops of the launch."""
    flops = C.c_double(0)
    check(load().qlin_probe_mfma_bf16(iters, stream, C.byref(flops)))
    return flops.value


def probe_clocks(stream=None):
    """Shader clock (MHz) of the last probe_mfma_bf16 launch."""
    mhz = C.c_double(0)
    check(load().qlin_probe_clocks(stream, C.byref(mhz)))
    return mhz.value


def probe_gemm_tile(tile, type_id, dW, dX, dY, n_rows, n_cols, n_tok, ldx, ldy, stream=None):
    check(load().qlin_probe_gemm_tile(tile, type_id, dW.ptr, dX.ptr, dY.ptr, n_rows, n_cols, n_tok, ldx, ldy, stream))


def probe_hbm_read(buf, n_bytes=None, stream=None):
    check(load().qlin_probe_hbm_read(buf.ptr, buf.nbytes if n_bytes is None else n_bytes, stream))


def timer_begin(stream=None):
    check(load().qlin_timer_begin(stream))


def timer_end(stream=None):
    ms = C.c_float(0)
    check(load().qlin_timer_end(stream, C.byref(ms)))
    return ms.value
