"""Pure-Python restatement of the reference's GGUF header reader, for checking the native one.

TEST INFRASTRUCTURE ONLY (imported by tests/). Follows crates/ferric-gguf/src/lib.rs: the bounds-safe cursor
(:56-104), parse (:105-132, without resolve_ambiguous_types :330-385), check_declared_strides (:387-431) and
type_size (:460-484). Pinned in tests/test_gguf.py against the numbers of the reference's own stride test
(lib.rs:1425-1458) and against files written field by field by an independent writer (tests/gguf_writer.py).
"""
import struct

TYPE_SIZE = {0: (1, 4), 1: (1, 2), 30: (1, 2), 8: (32, 34), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 12: (256, 144),
             13: (256, 176), 14: (256, 210), 20: (32, 18), 23: (256, 136), 35: (256, 66), 39: (32, 17), 41: (128, 18), 42: (128, 34),
             1042: (128, 129)}


def type_size(ty, n):
    if ty not in TYPE_SIZE:
        raise ValueError(f"unsupported ggml type {ty}")
    v, b = TYPE_SIZE[ty]
    return n // v * b


class _Cur:
    def __init__(self, b):
        self.b, self.p, self.ok = b, 0, True

    def take(self, k):
        if not self.ok or self.p + k > len(self.b):
            self.ok = False
            return None
        s = self.b[self.p:self.p + k]
        self.p += k
        return s

    def num(self, fmt, k, default=0):
        s = self.take(k)
        return struct.unpack("<" + fmt, s)[0] if s is not None else default

    def str(self):
        n = self.num("Q", 8)
        if n > len(self.b) - self.p:
            self.ok = False
            return ""
        s = self.take(n)
        return s.decode("utf-8", "replace") if s is not None else ""

    def val(self, ty):
        if ty == 0: return ("U", self.num("B", 1))
        if ty == 1: return ("I", self.num("b", 1))
        if ty == 2: return ("U", self.num("H", 2))
        if ty == 3: return ("I", self.num("h", 2))
        if ty == 4: return ("U", self.num("I", 4))
        if ty == 5: return ("I", self.num("i", 4))
        if ty == 6: return ("F", float(self.num("f", 4, 0.0)))
        if ty == 7: return ("Bool", self.num("B", 1) != 0)
        if ty == 8: return ("Str", self.str())
        if ty == 9:
            et, n = self.num("I", 4), self.num("Q", 8)
            if n > len(self.b) - self.p:
                self.ok = False
                return ("Arr", [])
            v = []
            for _ in range(n):
                if not self.ok:
                    break
                v.append(self.val(et))
            return ("Arr", v)
        if ty == 10: return ("U", self.num("Q", 8))
        if ty == 11: return ("I", self.num("q", 8))
        if ty == 12: return ("F", self.num("d", 8, 0.0))
        self.ok = False
        return ("U", 0)


def check_declared_strides(tensors, data_len, align):
    """tensors: list of (name, dims, ggml_type, offset). Returns None or the refusal message."""
    by = sorted(tensors, key=lambda t: t[3])
    have_full = (not by) or data_len >= by[-1][3]
    for i, (name, dims, ty, off) in enumerate(by):
        n = 1
        for d in dims:
            n *= d
        if ty not in TYPE_SIZE:
            continue
        sz = type_size(ty, n)
        if i + 1 < len(by):
            limit = by[i + 1][3]
        elif have_full:
            limit = data_len
        else:
            continue
        avail = max(0, limit - off)
        if sz > avail:
            return f"tensor '{name}' (ggml type {ty}, {n} elements) needs {sz} bytes by this reader's block layout, but the file leaves only {avail} before the next tensor."
        if i + 1 < len(by) and avail > sz + max(align, 64) * 4 and avail > sz * 2:
            return f"tensor '{name}' (ggml type {ty}, {n} elements) is {sz} bytes by this reader's block layout, but the file reserves {avail} for it"
    return None


def parse(data):
    """Returns dict(metadata={key: (kind, value)}, tensors=[(name, dims, type, offset)], data_start=int); raises ValueError."""
    c = _Cur(bytes(data))
    if c.num("I", 4) != struct.unpack("<I", b"GGUF")[0]:
        raise ValueError("not a GGUF file")
    version = c.num("I", 4)
    n_tensors, n_meta = c.num("Q", 8), c.num("Q", 8)
    meta = {}
    for _ in range(n_meta):
        if not c.ok:
            break
        key = c.str()
        ty = c.num("I", 4)
        meta[key] = c.val(ty)
    tensors = []
    for _ in range(n_tensors):
        if not c.ok:
            break
        name = c.str()
        nd = c.num("I", 4)
        if nd * 8 > len(c.b) - c.p:
            c.ok = False
            break
        dims = [c.num("Q", 8) for _ in range(nd)]
        ty = c.num("I", 4)
        off = c.num("Q", 8)
        tensors.append((name, dims, ty, off))
    if not c.ok:
        raise ValueError("GGUF header truncated or malformed")
    a = meta.get("general.alignment")
    align = a[1] if a is not None and a[0] == "U" else 32
    if align == 0:
        raise ValueError("GGUF general.alignment is 0")
    data_start = -(-c.p // align) * align
    why = check_declared_strides(tensors, max(0, len(c.b) - data_start), align)
    if why:
        raise ValueError(why)
    return {"version": version, "metadata": meta, "tensors": tensors, "data_start": data_start}
