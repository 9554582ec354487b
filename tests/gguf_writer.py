"""Minimal GGUF writer for the reader's tests: the container layout of the published specification
(header, key/value metadata, tensor-info table, aligned tensor data), written independently of the reader."""
import struct

import numpy as np

T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STR, T_ARR, T_U64, T_I64, T_F64 = range(13)
_FMT = {T_U8: "<B", T_I8: "<b", T_U16: "<H", T_I16: "<h", T_U32: "<I", T_I32: "<i", T_F32: "<f", T_BOOL: "<?",
        T_U64: "<Q", T_I64: "<q", T_F64: "<d"}


def _s(text):
    b = text.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _value(vtype, v):
    if vtype == T_STR:
        return _s(v)
    if vtype == T_ARR:
        etype, items = v
        return struct.pack("<IQ", etype, len(items)) + b"".join(_value(etype, x) for x in items)
    return struct.pack(_FMT[vtype], v)


def write_gguf(path, metadata, tensors, version=3, alignment=None, misalign=None):
    """metadata: list of (key, type, value); tensors: list of (name, dims_innermost_first, ggml_type_code, bytes)."""
    kv = list(metadata)
    if alignment is not None:
        kv.append(("general.alignment", T_U32, alignment))
    align = alignment or 32
    out = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(kv))
    for key, vtype, v in kv:
        out += _s(key) + struct.pack("<I", vtype) + _value(vtype, v)
    rel, infos, blobs = 0, b"", []
    for name, dims, tcode, data in tensors:
        data = bytes(data)
        off = rel + (1 if misalign == name else 0)
        infos += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        infos += struct.pack("<IQ", tcode, off)
        blobs.append((off, data))
        rel = (off + len(data) + align - 1) // align * align
    out += infos
    out += b"\0" * ((len(out) + align - 1) // align * align - len(out))
    body = bytearray(rel)
    for off, data in blobs:
        body[off:off + len(data)] = data
    with open(path, "wb") as f:
        f.write(out + bytes(body))
    return path
