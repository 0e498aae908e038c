"""Writes GGUF files for the parser tests (test helper, not part of the product).

Layout as read by common/gguf_loader.h:343-411: "GGUF", version u32, n_tensors u64, n_kv u64,
key/value pairs, tensor infos, padding to general.alignment (default 32), tensor data at their
offsets from the start of the data section."""
import struct

import numpy as np

U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q",
        I64: "<q", F64: "<d"}


def _s(text):
    b = text.encode() if isinstance(text, str) else bytes(text)
    return struct.pack("<Q", len(b)) + b


def _value(vtype, v):
    if vtype == STR:
        return _s(v)
    if vtype == ARR:
        etype, items = v
        out = struct.pack("<IQ", etype, len(items))
        return out + b"".join(_value(etype, it) for it in items)
    return struct.pack(_FMT[vtype], v)


def write(path, kvs, tensors, version=3, alignment=None, pad_data_to=None):
    """kvs: list of (key, vtype, value); tensors: list of (name, ggml_type, dims (inner first), raw uint8 data).
    Tensor data are placed one after the other, each start rounded up to the alignment.
    -> list of data-section offsets, data section file offset"""
    align = 32
    kvs = list(kvs)
    if alignment is not None:
        kvs.append(("general.alignment", U32, alignment))
        align = alignment
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(kvs))
    for key, vtype, v in kvs:
        head += _s(key) + struct.pack("<I", vtype) + _value(vtype, v)
    offsets, off = [], 0
    for _, _, _, data in tensors:
        off = (off + align - 1) // align * align
        offsets.append(off)
        off += len(np.asarray(data, np.uint8).ravel())
    for (name, ttype, dims, _), o in zip(tensors, offsets):
        head += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", ttype, o)
    data_offset = (len(head) + align - 1) // align * align
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * (data_offset - len(head)))
        pos = 0
        for (_, _, _, data), o in zip(tensors, offsets):
            f.write(b"\0" * (o - pos))
            raw = np.asarray(data, np.uint8).ravel().tobytes()
            f.write(raw)
            pos = o + len(raw)
        if pad_data_to and pos < pad_data_to:
            f.write(b"\0" * (pad_data_to - pos))
    return offsets, data_offset
