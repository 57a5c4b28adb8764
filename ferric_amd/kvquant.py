"""Host mirror of the reference's block-quantized KV cache, `ferric_tensor::kvquant::QKvCache`
(crates/ferric-tensor/src/kvquant.rs:118-133, 411-668): preallocate, append rows, double when full; the stored rows are
llama.cpp-layout blocks of 32 along the row (Q8_0 8.5, Q4_0 4.5, Q4_1 5.0 bits per value) in two device arrays, `codes` and
`scales`, byte for byte the reference's. Everything runs through libferric_hip; there is no CPU path.
"""
import ctypes as C

import numpy as np

from . import _lib
from .qmatrix import DeviceBuffer, Tensor, _stream_handle, _vp

QK = 32                                            # kvquant.rs:54
Q8_0, Q4_0, Q4_1 = 0, 1, 2                         # FHIP_KVQ_*; KvqFmt, kvquant.rs:57-64
ALL = (Q8_0, Q4_0, Q4_1)                           # KvqFmt::ALL, :101
NAMES = {Q8_0: "q8_0", Q4_0: "q4_0", Q4_1: "q4_1"}  # KvqFmt::name, :94-100
BLOCK_BYTES = {Q8_0: 34, Q4_0: 18, Q4_1: 20}       # KvqFmt::block_bytes, :83-89


def bits_per_value(fmt):
    """KvqFmt::bits_per_value, kvquant.rs:91-93."""
    return BLOCK_BYTES[fmt] * 8 / QK


def sizes(fmt, rows, width):
    """(code words, scale words) of rows x width -- KvqFmt::code_words / scale_words, kvquant.rs:66-81."""
    cw, sw = C.c_size_t(), C.c_size_t()
    _lib.check(_lib.load().fhip_kvq_sizes(fmt, rows, width, C.byref(cw), C.byref(sw)))
    return cw.value, sw.value


class QKvCache:
    """kvquant.rs:118 -- a grow-in-place quantized K or V cache. `cap` rows may be reserved up front (with the width), which a
    captured decode step needs: growth reallocates."""

    def __init__(self, fmt, cap=0, width=0):
        assert fmt in ALL, f"unknown KV format {fmt}"
        self.fmt, self.len, self.cap, self.width = fmt, 0, 0, 0
        self.codes = self.scales = None
        if cap and width:
            assert width % QK == 0, f"QKvCache row width {width} must be a multiple of {QK}"
            self.width = width
            self._grow(cap)

    @staticmethod
    def from_tensor(src, fmt, stream=None):
        """kvquant.rs:417: quantize a whole [t, width] tensor into a fresh cache."""
        return QKvCache(fmt).append(src, stream)

    def is_empty(self):
        return self.len == 0

    def nblk_per_row(self):
        return self.width // QK

    def bytes(self):
        """kvquant.rs:429: what is allocated."""
        cw, sw = sizes(self.fmt, self.cap, self.width) if self.width else (0, 0)
        return (cw + sw) * 4

    def live_bytes(self):
        """kvquant.rs:445: what the filled rows cost."""
        cw, sw = sizes(self.fmt, self.len, self.width) if self.width else (0, 0)
        return (cw + sw) * 4

    def f32_bytes(self):
        """kvquant.rs:451."""
        return self.len * self.width * 4

    def _alloc(self, cap):
        cw, sw = sizes(self.fmt, cap, self.width)
        return DeviceBuffer(max(cw * 4, 4)), DeviceBuffer(max(sw * 4, 4))

    def _copy_live(self, codes, scales, rows, stream):
        cw, sw = sizes(self.fmt, rows, self.width)
        lib, s = _lib.load(), _stream_handle(stream)
        if cw:
            _lib.check(lib.fhip_memcpy_d2d(codes.ptr, self.codes.ptr, cw * 4, s))
            _lib.check(lib.fhip_memcpy_d2d(scales.ptr, self.scales.ptr, sw * 4, s))

    def _grow(self, new_cap, stream=None):
        """kvquant.rs:519-533: larger arrays, the live words copied over."""
        codes, scales = self._alloc(new_cap)
        if self.len:
            self._copy_live(codes, scales, self.len, stream)
            _lib.check(_lib.load().fhip_stream_sync(_stream_handle(stream)))     # the old arrays are freed on return
        self.codes, self.scales, self.cap = codes, scales, new_cap

    def append(self, src, stream=None, cols=None):
        """kvquant.rs:464: quantize exactly the rows of src [t, width] behind the filled ones. cols = (first, width): a window
        of wider rows read in place, as the reference reads a strided view (:486-495)."""
        assert len(src.shape) == 2, "QKvCache::append expects a 2D [t, width] tensor"
        t = src.shape[0]
        offset, width = (0, src.shape[1]) if cols is None else cols
        row_stride = src.shape[1]
        assert offset + width <= row_stride, "QKvCache::append: the window leaves the source rows"
        if t == 0:
            return self
        assert width % QK == 0, f"QKvCache row width {width} must be a multiple of {QK}"
        if self.width == 0:
            self.width = width
        assert width == self.width, "QKvCache width changed"
        need = self.len + t
        if self.cap < need:
            self._grow(max(need, self.cap * 2, 64), stream)
        src_ptr = C.c_void_p(src.buf.ptr.value + 4 * offset)
        _lib.check(_lib.load().fhip_kvq_append(self.fmt, src_ptr, row_stride, t, width, None, self.len, 0, self.cap, self.codes.ptr,
                                               self.scales.ptr, _stream_handle(stream)))
        self.len = need
        return self

    def dequantize_rows(self, row0, rows, stream=None):
        """kvquant.rs:621."""
        assert row0 + rows <= self.len, f"dequantize_rows({row0}, {rows}) past len {self.len}"
        out = Tensor.empty((rows, self.width))
        if rows * self.width:
            _lib.check(_lib.load().fhip_kvq_dequantize_rows(self.fmt, self.codes.ptr, self.scales.ptr, row0, rows, self.width, None,
                                                            out.buf.ptr, _stream_handle(stream)))
        return out

    def dequantize(self, stream=None):
        """kvquant.rs:617: the whole cache as [len, width] f32."""
        return self.dequantize_rows(0, self.len, stream)

    def deep_clone(self, stream=None):
        """kvquant.rs:556: a copy that shares no device memory (the live region only)."""
        out = QKvCache(self.fmt)
        out.len, out.cap, out.width = self.len, self.cap, self.width
        if self.codes is not None:
            out.codes, out.scales = self._alloc(self.cap)
            self._copy_live(out.codes, out.scales, self.len, stream)
        return out

    def clone_prefix(self, rows, stream=None):
        """kvquant.rs:595: the first `rows` rows in arrays of their own, capacity max(rows, 64)."""
        rows = min(rows, self.len)
        out = QKvCache(self.fmt)
        if rows == 0 or self.width == 0:
            return out
        out.width, out.len, out.cap = self.width, rows, max(rows, 64)
        out.codes, out.scales = out._alloc(out.cap)
        self._copy_live(out.codes, out.scales, rows, stream)
        return out

    def to_host(self, stream=None):
        """kvquant.rs:654: (codes, scales) of the live rows as u32 words."""
        cw, sw = sizes(self.fmt, self.len, self.width) if self.width else (0, 0)
        c, s = np.zeros(cw, np.uint32), np.zeros(sw, np.uint32)
        lib, st = _lib.load(), _stream_handle(stream)
        if cw:
            _lib.check(lib.fhip_memcpy_d2h(_vp(c), self.codes.ptr, cw * 4, st))
            _lib.check(lib.fhip_memcpy_d2h(_vp(s), self.scales.ptr, sw * 4, st))
        return c, s
