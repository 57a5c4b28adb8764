"""GGUF ingest: the host-side mirror of crates/ferric-gguf's reader over the C ABI (fhip_gguf_*).

    g = GgufFile.open(path)            # maps the file, parses header + metadata + tensor table
    g.metadata["general.architecture"] # Meta values as Python int / float / bool / str / list
    g.tensor("blk.0.ffn_down.weight")  # TensorInfo(name, dims, ggml_type, offset) or None
    g.raw(name)                        # the packed bytes as stored (a view into the mapping)
    g.qmatrix(name)                    # file -> HBM, no host copy: a QMatrix ready for matmul_q

Parsing touches no device; only qmatrix() does.
"""
import ctypes as C
from collections import namedtuple

import numpy as np

from . import _lib
from .qmatrix import QMatrix

TensorInfo = namedtuple("TensorInfo", "name dims ggml_type offset")   # crates/ferric-gguf/src/lib.rs:41-47
_SELF = C.c_size_t(-1).value


class Gguf:
    """crates/ferric-gguf/src/lib.rs:49 Gguf / :520 GgufFile behind one handle."""

    def __init__(self, handle, keepalive=None):
        self._h, self._keep = handle, keepalive
        lib = _lib.load()
        self.version = lib.fhip_gguf_version(handle)
        self.data_start = lib.fhip_gguf_data_start(handle)
        self.tensors = []
        for i in range(lib.fhip_gguf_n_tensors(handle)):
            name, nd, dims, ty, off = C.c_char_p(), C.c_uint32(), C.POINTER(C.c_uint64)(), C.c_uint32(), C.c_uint64()
            _lib.check(lib.fhip_gguf_tensor(handle, i, C.byref(name), C.byref(nd), C.byref(dims), C.byref(ty), C.byref(off)))
            self.tensors.append(TensorInfo(name.value.decode("utf-8", "replace"), [int(dims[d]) for d in range(nd.value)],
                                           ty.value, off.value))
        self.metadata = {}
        for i in range(lib.fhip_gguf_n_meta(handle)):
            key = lib.fhip_gguf_meta_key(handle, i)
            self.metadata[key.decode("utf-8", "replace")] = self._meta(key, _SELF)

    def _meta(self, key, j, kind=None):
        lib = _lib.load()
        if kind is None:
            n = C.c_size_t()
            kind = lib.fhip_gguf_meta_kind(self._h, key, C.byref(n))
            if kind == 5:
                return [self._elem(key, e) for e in range(n.value)]
        return self._scalar(key, j, kind)

    def _elem(self, key, j):
        # arrays are homogeneous in practice but each element carries its own kind: try the getters in turn
        lib = _lib.load()
        for kind in (0, 1, 2, 4):
            try:
                return self._scalar(key, j, kind)
            except ValueError:
                continue
        return None   # a nested array: not produced by any writer this path meets

    def _scalar(self, key, j, kind):
        lib = _lib.load()
        if kind in (0, 3):
            v = C.c_uint64()
            _lib.check(lib.fhip_gguf_meta_u64(self._h, key, j, C.byref(v)))
            return bool(v.value) if kind == 3 else v.value
        if kind == 1:
            v = C.c_int64()
            _lib.check(lib.fhip_gguf_meta_i64(self._h, key, j, C.byref(v)))
            return v.value
        if kind == 2:
            v = C.c_double()
            _lib.check(lib.fhip_gguf_meta_f64(self._h, key, j, C.byref(v)))
            return v.value
        s, n = C.c_char_p(), C.c_size_t()
        p = C.c_void_p()
        _lib.check(lib.fhip_gguf_meta_str(self._h, key, j, C.byref(p), C.byref(n)))
        return C.string_at(p, n.value).decode("utf-8", "replace")

    @staticmethod
    def parse(data):
        """lib.rs:105 parse(bytes): raises ValueError with the reference's message on a bad file."""
        buf = np.frombuffer(bytes(data), dtype=np.uint8) if not isinstance(data, np.ndarray) else np.ascontiguousarray(data, np.uint8)
        h = C.c_void_p()
        _lib.check(_lib.load().fhip_gguf_parse(buf.ctypes.data_as(C.c_void_p), buf.size, C.byref(h)))
        return Gguf(h, keepalive=buf)

    @staticmethod
    def open(path):
        """The file-backed reader (lib.rs:520 GgufFile::open): the file is mapped, nothing is read eagerly."""
        h = C.c_void_p()
        _lib.check(_lib.load().fhip_gguf_open(str(path).encode(), C.byref(h)))
        return Gguf(h)

    def tensor(self, name):
        i = _lib.load().fhip_gguf_find(self._h, name.encode())
        return self.tensors[i] if i >= 0 else None

    def raw(self, name):
        """The tensor's packed bytes exactly as stored -- lib.rs:443 / :566. A read-only view; keep `self` alive."""
        p, n = C.c_void_p(), C.c_size_t()
        _lib.check(_lib.load().fhip_gguf_raw(self._h, name.encode(), C.byref(p), C.byref(n)))
        if n.value == 0:
            return np.zeros(0, np.uint8)
        a = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(n.value,))
        a.flags.writeable = False
        return a

    def dequant(self, name):
        """The tensor as f32, row-major, whatever its type -- lib.rs:456 / :575 (deq_raw over the tensor's bytes, on the GPU)."""
        from .qmatrix import deq_raw
        t = self.tensor(name)
        if t is None:
            raise ValueError(f"no tensor '{name}'")
        n = 1
        for d in t.dims:
            n *= int(d)
        return deq_raw(self.raw(name), n, t.ggml_type)

    def qmatrix(self, name):
        """Upload the tensor straight from the mapping: dims [in, out] (or [in, rows per expert, n_expert])."""
        t = self.tensor(name)
        h = C.c_void_p()
        _lib.init()
        _lib.check(_lib.load().fhip_weight_from_gguf(self._h, name.encode(), C.byref(h)))
        return QMatrix(h, t.ggml_type)

    def qm(self, name):
        """crates/ferric-llama/src/qwen35.rs:366 qm(ctx, g, name): the tensor as a packed weight [out = dims[1], in = dims[0]]. (The
        reference's dense fallback for formats without a packed kernel is not part of this path: ValueError.)"""
        if self.tensor(name) is None:
            raise ValueError(f"no tensor '{name}'")
        return self.qmatrix(name)

    def qm_cat(self, names):
        """qwen35.rs:379 qm_cat(ctx, g, names): same-format tensors of one input width stacked along the output dim into one
        weight (fused QKV, fused gate|up), each uploaded straight from the mapping to its place in HBM."""
        names = list(names)
        arr = (C.c_char_p * len(names))(*[n.encode() for n in names])
        h = C.c_void_p()
        _lib.init()
        _lib.check(_lib.load().fhip_weight_from_gguf_cat(self._h, arr, len(names), C.byref(h)))
        return QMatrix(h, self.tensor(names[0]).ggml_type)

    def close(self):
        if self._h:
            _lib.load().fhip_gguf_close(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


GgufFile = Gguf


class Proj:
    """crates/ferric-llama/src/qwen3.rs:192-228: a projection made of one or several GGUF tensors. Tensors of one format are fused into
    one weight (`Fused`); mixed formats (V is often Q6_K beside Q4_K Q and K) stay apart and their outputs are concatenated (`Split`)."""

    def __init__(self, fused=None, split=None):
        self.fused, self.split = fused, split

    @staticmethod
    def load(g, names):
        names = list(names)
        types = [(g.tensor(n).ggml_type if g.tensor(n) is not None else 0) for n in names]
        if len(names) > 1 and all(a == b for a, b in zip(types, types[1:])):
            return Proj(fused=g.qm_cat(names))
        if len(names) == 1:
            return Proj(fused=g.qm(names[0]))
        return Proj(split=[g.qm(n) for n in names])

    def matmul(self, x, stream=None):
        if self.fused is not None:
            return x.matmul_q(self.fused, stream)
        out = x.matmul_q(self.split[0], stream)
        for w in self.split[1:]:
            out = out.cat(x.matmul_q(w, stream), 1, stream)
        return out

    def gate_up_swiglu(self, x, n_ff, stream=None):
        """One fused kernel when gate|up is one K-quant weight, else the plain matmul and SwiGLU: the same result either way."""
        if self.fused is not None:
            o = x.try_matmul_swiglu(self.fused, stream)
            if o is not None:
                return o
        return self.matmul(x, stream).swiglu(n_ff, stream)
