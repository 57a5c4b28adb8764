"""A GGUF file writer for the tests: lays the container out field by field from the format's definition (magic,
version, counts, typed key/values, tensor infos, aligned data section). Independent of both readers under test."""
import struct

import numpy as np

_NUM = {"u8": (0, "B"), "i8": (1, "b"), "u16": (2, "H"), "i16": (3, "h"), "u32": (4, "I"), "i32": (5, "i"), "f32": (6, "f"),
        "bool": (7, "B"), "u64": (10, "Q"), "i64": (11, "q"), "f64": (12, "d")}


def _s(text):
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def _val(kind, v):
    if kind == "str":
        return _s(v)
    if kind.startswith("arr:"):
        et = kind[4:]
        code = 8 if et == "str" else _NUM[et][0]
        return struct.pack("<IQ", code, len(v)) + b"".join(_val(et, e) for e in v)
    return struct.pack("<" + _NUM[kind][1], v)


def write_gguf(meta, tensors, align=None, version=3, pad_data_to=None):
    """meta: list of (key, kind, value) with kind in u8..f64, bool, str, arr:<kind>. tensors: list of
    (name, dims, ggml_type, bytes[, forced_offset]). Returns (file bytes, data_start, {name: offset})."""
    meta = list(meta)
    if align is not None:
        meta.append(("general.alignment", "u32", align))
    a = align or 32
    offs, data, cur = {}, bytearray(), 0
    for t in tensors:
        name, dims, ty, raw = t[:4]
        off = t[4] if len(t) > 4 else -(-cur // a) * a
        offs[name] = off
        if len(data) < off:
            data.extend(b"\0" * (off - len(data)))
        raw = bytes(np.asarray(raw, np.uint8).tobytes())
        data[off:off + len(raw)] = raw
        cur = max(cur, off + len(raw))
    head = bytearray(b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(meta)))
    for key, kind, v in meta:
        code = 8 if kind == "str" else 9 if kind.startswith("arr:") else _NUM[kind][0]
        head += _s(key) + struct.pack("<I", code) + _val(kind, v)
    for t in tensors:
        name, dims, ty = t[:3]
        head += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", ty, offs[name])
    data_start = -(-len(head) // a) * a
    head.extend(b"\0" * (data_start - len(head)))
    if pad_data_to is not None and len(data) < pad_data_to:
        data.extend(b"\0" * (pad_data_to - len(data)))
    return bytes(head + data), data_start, offs
