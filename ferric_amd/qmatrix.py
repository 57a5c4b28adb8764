"""Host-side mirror of the reference's quantized-linear interface, over the C ABI.

Names, argument meaning and error behaviour follow the reference (paths relative to its checkout):

    type_size / deq_raw                       crates/ferric-gguf/src/lib.rs:471 / :497
    QMatrix.block_bytes / from_bytes / ...    crates/ferric-tensor/src/dtype.rs:873-931
    Q8_0Weights / Q4_KWeights / Q6_KWeights   crates/ferric-tensor/src/dtype.rs:1261 / 1374 / 1138
    Tensor.matmul_q / try_matmul_swiglu / ... crates/ferric-tensor/src/dtype.rs:935-959
    Tensor.swiglu                             crates/ferric-tensor/src/lib.rs:728
    matvec_q8_0 / _threaded / _span           crates/ferric-tensor/src/cpu_simd.rs:79-122

`Err(String)` becomes ValueError, an `assert!` panic becomes AssertionError. Everything computes on
the GPU through libferric_hip.so; nothing here does arithmetic on the host.
"""
import ctypes as C

import numpy as np

from . import _lib

Q8_0, Q4_K, Q6_K = 8, 12, 14
Q4_0, Q4_1, Q5_0, Q5_1, Q5_K = 2, 3, 6, 7, 13   # further formats: unpackers, mat-vec / small batch, "_id" variants
IQ4_NL, IQ4_XS, MXFP4 = 20, 23, 39             # codebook / microscaling formats, same coverage
BATCH_AUTO, BATCH_F32_MATVEC, BATCH_ORDERED = 0, 1, 2   # QMatrix.batch_policy
F32, F16, BF16 = 0, 1, 30                      # unquantized tensor types: type_size and deq_raw only (lib.rs:473-475, 499-501)


def _vp(a):
    return a.ctypes.data_as(C.c_void_p)


class Stream:
    """One HIP stream; ops enqueue on it and return (ordering = submission order, as on the
    reference's single wgpu queue). None means the default stream."""

    def __init__(self):
        lib = _lib.init()
        h = C.c_void_p()
        _lib.check(lib.fhip_stream_create(C.byref(h)))
        self.handle = h

    def synchronize(self):
        _lib.check(_lib.load().fhip_stream_sync(self.handle))

    def __del__(self):
        try:
            if self.handle:
                _lib.load().fhip_stream_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


class Graph:
    """Calls recorded on a stream between Graph.begin(stream) and .end(), replayed with launch():
    the counterpart of the reference's batch(ctx, ..) single-submission recorder (lib.rs:1802)."""

    def __init__(self, stream):
        self.stream, self.handle = stream, None

    @staticmethod
    def begin(stream):
        g = Graph(stream)
        _lib.check(_lib.load().fhip_graph_capture_begin(stream.handle))
        return g

    def end(self):
        h = C.c_void_p()
        _lib.check(_lib.load().fhip_graph_capture_end(self.stream.handle, C.byref(h)))
        self.handle = h
        return self

    def launch(self, stream=None):
        _lib.check(_lib.load().fhip_graph_launch(self.handle, (stream or self.stream).handle))

    def __del__(self):
        try:
            if self.handle:
                _lib.load().fhip_graph_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


def _stream_handle(stream):
    return stream.handle if stream is not None else None


class DeviceBuffer:
    """nbytes of device memory, freed with the object."""

    def __init__(self, nbytes):
        lib = _lib.init()
        p = C.c_void_p()
        _lib.check(lib.fhip_malloc(C.byref(p), nbytes))
        self.ptr, self.nbytes = p, nbytes

    def __del__(self):
        try:
            if self.ptr:
                _lib.load().fhip_free(self.ptr)
                self.ptr = None
        except Exception:
            pass


class Tensor:
    """A contiguous row-major device tensor (f32 unless made with from_bf16_bits)."""

    def __init__(self, buf, shape, dtype=np.float32):
        self.buf, self.shape, self.dtype = buf, tuple(int(s) for s in shape), np.dtype(dtype)

    # -- construction / readback (crates/ferric-tensor/src/lib.rs: Tensor::from_vec, to_vec) --
    @staticmethod
    def from_vec(data, shape, stream=None):
        a = np.ascontiguousarray(data, dtype=np.float32)
        assert a.size == int(np.prod(shape)), "from_vec: data does not match shape"
        t = Tensor(DeviceBuffer(a.nbytes), shape)
        _lib.check(_lib.load().fhip_memcpy_h2d(t.buf.ptr, _vp(a), a.nbytes, _stream_handle(stream)))
        if stream is None:
            _lib.check(_lib.load().fhip_stream_sync(None))
        else:
            stream.synchronize()  # the host array may go away
        return t

    @staticmethod
    def from_bf16_bits(bits, shape):
        a = np.ascontiguousarray(bits, dtype=np.uint16)
        assert a.size == int(np.prod(shape))
        t = Tensor(DeviceBuffer(a.nbytes), shape, np.uint16)
        _lib.check(_lib.load().fhip_memcpy_h2d(t.buf.ptr, _vp(a), a.nbytes, None))
        _lib.check(_lib.load().fhip_stream_sync(None))
        return t

    @staticmethod
    def empty(shape, dtype=np.float32):
        n = int(np.prod(shape))
        return Tensor(DeviceBuffer(n * np.dtype(dtype).itemsize), shape, dtype)

    def numel(self):
        return int(np.prod(self.shape))

    def to_vec(self, stream=None):
        """Device -> host; the only synchronising call (the reference's readback)."""
        out = np.empty(self.numel(), dtype=self.dtype)
        _lib.check(_lib.load().fhip_memcpy_d2h(_vp(out), self.buf.ptr, out.nbytes, _stream_handle(stream)))
        return out

    def cat(self, other, dim, stream=None):
        """Concatenation of two tensors of the same dtype along `dim` -- lib.rs:201 (the reference's asserts; here for the vectors and
        matrices this path handles: each side is copied into its rows or columns of the result)."""
        assert len(self.shape) == len(other.shape), "cat: rank mismatch"
        assert len(self.shape) in (1, 2) and 0 <= dim < len(self.shape), "cat: vectors and matrices only"
        for d in range(len(self.shape)):
            if d != dim:
                assert self.shape[d] == other.shape[d], f"cat: dim {d} mismatch {list(self.shape)} vs {list(other.shape)}"
        assert self.dtype == other.dtype, "cat: dtype mismatch"
        shape = list(self.shape)
        shape[dim] += other.shape[dim]
        out = Tensor.empty(shape, self.dtype)
        lib, sh, it = _lib.load(), _stream_handle(stream), self.dtype.itemsize
        if dim == 0:
            na = self.numel() * it
            _lib.check(lib.fhip_memcpy_d2d(out.buf.ptr, self.buf.ptr, na, sh))
            _lib.check(lib.fhip_memcpy_d2d(C.c_void_p(out.buf.ptr.value + na), other.buf.ptr, other.numel() * it, sh))
        else:
            rows, wa, wb = self.shape[0], self.shape[1] * it, other.shape[1] * it
            _lib.check(lib.fhip_memcpy_2d_d2d(out.buf.ptr, wa + wb, self.buf.ptr, wa, wa, rows, sh))
            _lib.check(lib.fhip_memcpy_2d_d2d(C.c_void_p(out.buf.ptr.value + wa), wa + wb, other.buf.ptr, wb, wb, rows, sh))
        return out

    # -- quantized matmuls --------------------------------------------------------------------
    def _rows_inner(self):
        assert len(self.shape) == 2, "matmul_q expects a [rows, in] tensor"
        return self.shape

    def matmul_q(self, w, stream=None):
        """y = x . W^T for a packed weight of any supported format -- dtype.rs:935."""
        rows, inn = self._rows_inner()
        assert inn == w.cols(), f"inner dim mismatch: x[..,{inn}] vs W[..,{w.cols()}]"
        out = Tensor.empty((rows, w.rows()))
        _lib.check(_lib.load().fhip_matmul_q(w.handle, self.buf.ptr, rows, out.buf.ptr, _stream_handle(stream)))
        return out

    def _matmul_typed(self, w, ty, stream):
        assert w.ggml_type == ty, f"weight is ggml type {w.ggml_type}, not {ty}"
        return self.matmul_q(w, stream)

    def matmul_q8_0(self, w, stream=None):  # dtype.rs:1292
        return self._matmul_typed(w, Q8_0, stream)

    def matmul_q4_k(self, w, stream=None):  # dtype.rs:1426
        return self._matmul_typed(w, Q4_K, stream)

    def matmul_q6_k(self, w, stream=None):  # dtype.rs:1172
        return self._matmul_typed(w, Q6_K, stream)

    def matmul_q5_k(self, w, stream=None):  # dtype.rs:1049
        return self._matmul_typed(w, Q5_K, stream)

    def matmul_q4_0(self, w, stream=None):  # dtype.rs:1838
        return self._matmul_typed(w, Q4_0, stream)

    def matmul_q4_1(self, w, stream=None):  # dtype.rs:1860
        return self._matmul_typed(w, Q4_1, stream)

    def matmul_q5_0(self, w, stream=None):  # dtype.rs:1882
        return self._matmul_typed(w, Q5_0, stream)

    def matmul_q5_1(self, w, stream=None):  # dtype.rs:1904
        return self._matmul_typed(w, Q5_1, stream)

    def matmul_iq4_nl(self, w, stream=None):  # dtype.rs:3259
        return self._matmul_typed(w, IQ4_NL, stream)

    def matmul_iq4_xs(self, w, stream=None):  # dtype.rs:3185
        return self._matmul_typed(w, IQ4_XS, stream)

    def matmul_mxfp4(self, w, stream=None):  # dtype.rs:3396
        return self._matmul_typed(w, MXFP4, stream)

    def try_matmul_swiglu(self, w, stream=None):
        """Fused gate/up + SwiGLU -- dtype.rs:949. None when the format has no fused kernel
        (Q8_0 and the 32-value formats); the caller then runs matmul_q(w).swiglu(n_ff)."""
        if w.ggml_type not in (Q4_K, Q6_K, Q5_K):
            return None
        rows, inn = self._rows_inner()
        assert inn == w.cols(), f"inner dim mismatch: x[..,{inn}] vs W[..,{w.cols()}]"
        out = Tensor.empty((rows, w.rows() // 2))
        _lib.check(_lib.load().fhip_matmul_q_swiglu(w.handle, self.buf.ptr, rows, out.buf.ptr, _stream_handle(stream)))
        return out

    def matmul_q4_k_swiglu(self, w, stream=None):  # dtype.rs:1551
        assert w.ggml_type == Q4_K
        return self.try_matmul_swiglu(w, stream)

    def matmul_q6_k_swiglu(self, w, stream=None):  # dtype.rs:1802
        assert w.ggml_type == Q6_K
        return self.try_matmul_swiglu(w, stream)

    def matmul_q5_k_swiglu(self, w, stream=None):  # dtype.rs:1784
        assert w.ggml_type == Q5_K
        return self.try_matmul_swiglu(w, stream)

    def swiglu(self, d, stream=None):
        """self is [t, 2d] = [gate | up]; returns silu(gate) * up as [t, d] -- lib.rs:728."""
        t = self.numel() // (2 * d)
        out = Tensor.empty((t, d))
        _lib.check(_lib.load().fhip_swiglu(self.buf.ptr, t, d, out.buf.ptr, _stream_handle(stream)))
        return out

    def ffn(self, gate_up, down, stream=None):
        """down(swiglu(gate_up(x))) -- the FFN of crates/ferric-llama/src/qwen3.rs:944-964."""
        rows, inn = self._rows_inner()
        assert inn == gate_up.cols(), "gate_up in dim mismatch"
        n_ff = gate_up.rows() // 2
        ws = Tensor.empty((rows, n_ff))
        out = Tensor.empty((rows, down.rows()))
        _lib.check(_lib.load().fhip_ffn(gate_up.handle, down.handle, self.buf.ptr, rows, out.buf.ptr, ws.buf.ptr,
                                        _stream_handle(stream)))
        out._keepalive = ws  # scratch must outlive the enqueued work
        return out

    # -- mixture-of-experts decode (dtype.rs:1582-1780) -----------------------------------------
    def moe_topk(self, bias, k, sigmoid, scale, stream=None):
        """Router top-k on the device -- dtype.rs:1582. self = logits [T, n_expert]; returns [T, 2k] = [w | idx]."""
        return self.moe_topk_ex(bias, k, sigmoid, scale, True, stream)

    def moe_topk_ex(self, bias, k, sigmoid, scale, norm, stream=None):
        """moe_topk with explicit control over renormalisation -- dtype.rs:1596."""
        t, ne = (self.shape[0], self.shape[1]) if len(self.shape) == 2 else (1, self.numel())
        assert 1 <= k <= 8, "k must be 1..=8"
        assert ne <= 1024, "moe_topk: n_expert <= 1024 (single-thread scan)"
        out = Tensor.empty((t, 2 * k))
        _lib.check(_lib.load().fhip_moe_topk(self.buf.ptr, bias.buf.ptr if bias is not None else None, t, ne, k, int(bool(sigmoid)),
                                             float(scale), int(bool(norm)), out.buf.ptr, _stream_handle(stream)))
        return out

    def matmul_q_swiglu_id(self, w, selw, k, eff, stream=None):
        """Any format's selected-expert gate|up + SwiGLU (the typed methods below assert the format and call this)."""
        t, inn = self._rows_inner()
        assert inn == w.cols(), f"inner dim mismatch: x[..,{inn}] vs W[..,{w.cols()}]"
        assert 1 <= k <= 8, "k must be 1..=8"
        out = Tensor.empty((t, k, eff))
        _lib.check(_lib.load().fhip_matmul_q_swiglu_id(w.handle, self.buf.ptr, t, selw.buf.ptr, k, eff, out.buf.ptr, _stream_handle(stream)))
        return out

    def matmul_q4_k_swiglu_id(self, w, selw, k, eff, stream=None):
        """Selected experts' gate|up + SwiGLU for every (token, slot): [T, in] -> [T, k, eff] -- dtype.rs:1620."""
        assert w.ggml_type == Q4_K
        return self.matmul_q_swiglu_id(w, selw, k, eff, stream)

    def matmul_q8_0_swiglu_id(self, w, selw, k, eff, stream=None):
        """dtype.rs:1731."""
        assert w.ggml_type == Q8_0
        return self.matmul_q_swiglu_id(w, selw, k, eff, stream)

    def matmul_q_relu2_id(self, w, selw, k, eff, stream=None):
        """Any format's selected-expert up projection with max(v, 0)^2 applied: [T, in] -> [T, k, eff]."""
        t, inn = self._rows_inner()
        assert 1 <= k <= 8, "k must be 1..=8"
        assert inn == w.cols(), f"inner dim mismatch: x[..,{inn}] vs W[..,{w.cols()}]"
        out = Tensor.empty((t, k, eff))
        _lib.check(_lib.load().fhip_matmul_q_relu2_id(w.handle, self.buf.ptr, t, selw.buf.ptr, k, eff, out.buf.ptr, _stream_handle(stream)))
        return out

    def matmul_q5_0_relu2_id(self, w, selw, k, eff, stream=None):
        """The squared-ReLU expert MLP's up projection on a Q5_0 slab -- dtype.rs:1711."""
        assert w.ggml_type == Q5_0
        assert self._rows_inner()[1] % 32 == 0, "Q5_0 inner dim must be a multiple of 32"
        return self.matmul_q_relu2_id(w, selw, k, eff, stream)

    def matmul_q6_k_id(self, w, selw, out_pe, stream=None):
        """Selected experts' down projection, one row per slot: [k, in] -> [k, out_pe] -- dtype.rs:1640."""
        k, inn = self._rows_inner()
        assert 1 <= k <= 8, "k must be 1..=8"
        assert inn == w.cols(), f"inner dim mismatch: x[..,{inn}] vs W[..,{w.cols()}]"
        out = Tensor.empty((k, out_pe))
        _lib.check(_lib.load().fhip_matmul_q_id(w.handle, self.buf.ptr, selw.buf.ptr, k, out_pe, out.buf.ptr, _stream_handle(stream)))
        return out

    def matmul_q_id_wsum(self, w, selw, out_pe, stream=None):
        """Any format's selected-expert down projection with the weighted sum over slots fused."""
        t, k, inn = self.shape if len(self.shape) == 3 else (1, self.shape[0], self.shape[1])
        assert 1 <= k <= 8, "k must be 1..=8"
        assert inn == w.cols(), f"inner dim mismatch: x[..,{inn}] vs W[..,{w.cols()}]"
        out = Tensor.empty((t, out_pe))
        ws = Tensor.empty((t * k, out_pe))
        _lib.check(_lib.load().fhip_matmul_q_id_wsum(w.handle, self.buf.ptr, t, selw.buf.ptr, k, out_pe, out.buf.ptr, ws.buf.ptr,
                                                     _stream_handle(stream)))
        if stream is not None:
            stream.synchronize()      # ws is freed on return
        else:
            _lib.check(_lib.load().fhip_stream_sync(None))
        return out

    def matmul_q6_k_id_wsum(self, w, selw, out_pe, stream=None):
        """Down projection with the weighted sum over slots fused: [T, k, in] -> [T, out_pe] -- dtype.rs:1662."""
        assert w.ggml_type == Q6_K
        return self.matmul_q_id_wsum(w, selw, out_pe, stream)

    def matmul_q4_k_id_wsum(self, w, selw, out_pe, stream=None):
        """dtype.rs:1765."""
        assert w.ggml_type == Q4_K
        return self.matmul_q_id_wsum(w, selw, out_pe, stream)

    def matmul_q8_0_id_wsum(self, w, selw, out_pe, stream=None):
        """dtype.rs:1748."""
        assert w.ggml_type == Q8_0
        return self.matmul_q_id_wsum(w, selw, out_pe, stream)

    def matmul_q5_0_id_wsum(self, w, selw, out_pe, stream=None):
        """dtype.rs:1686 (the expert down slab of a mixed-precision checkpoint)."""
        assert w.ggml_type == Q5_0
        return self.matmul_q_id_wsum(w, selw, out_pe, stream)

    def cvt_bf16(self, stream=None):
        """f32 -> bf16 bit patterns (round to nearest even), same shape."""
        assert self.dtype == np.float32
        n = self.numel()
        out = Tensor(DeviceBuffer(max(16, 2 * n)), self.shape, np.uint16)
        _lib.check(_lib.load().fhip_cvt_f32_bf16(self.buf.ptr, n, out.buf.ptr, _stream_handle(stream)))
        return out

    def matmul_q_coop(self, w, stream=None):
        """f32 x [rows, in] @ W^T on the matrix cores -- dtype.rs:1818 matmul_q4_k_coop / :1199 / :1316 / :1074 (Q5_K)."""
        assert self.dtype == np.float32, "matmul_q_coop expects f32 activations"
        rows, inn = self._rows_inner()
        assert inn == w.cols(), "inner dim mismatch"
        assert w.rows() % 8 == 0, "matmul_q_coop needs N (out) a multiple of 8"   # dtype.rs:1822
        out = Tensor.empty((rows, w.rows()))
        ws = DeviceBuffer(max(16, rows * inn * 2))
        _lib.check(_lib.load().fhip_matmul_q_coop(w.handle, self.buf.ptr, rows, out.buf.ptr, ws.ptr, _stream_handle(stream)))
        if stream is not None:
            stream.synchronize()      # ws is freed on return
        else:
            _lib.check(_lib.load().fhip_stream_sync(None))
        return out

    def matmul_q4_k_coop(self, w, stream=None):
        assert w.ggml_type == 12
        return self.matmul_q_coop(w, stream)

    def matmul_q6_k_coop(self, w, stream=None):
        assert w.ggml_type == 14
        return self.matmul_q_coop(w, stream)

    def matmul_q8_0_coop(self, w, stream=None):
        assert w.ggml_type == 8
        return self.matmul_q_coop(w, stream)

    def matmul_q5_k_coop(self, w, stream=None):  # dtype.rs:1074
        assert w.ggml_type == 13
        return self.matmul_q_coop(w, stream)

    def matmul_q_f16x2(self, w, stream=None):
        """x [rows <= 32, in] @ W^T in one pass over the weights, f32-grade results -- dtype.rs:935-944 for small batches."""
        assert self.dtype == np.float32, "matmul_q_f16x2 expects f32 activations"
        rows, inn = self._rows_inner()
        assert inn == w.cols(), "inner dim mismatch"
        lib = _lib.load()
        ws = DeviceBuffer(max(256, lib.fhip_matmul_q_f16x2_ws_bytes(w.handle, rows)))
        out = Tensor.empty((rows, w.rows()))
        _lib.check(lib.fhip_matmul_q_f16x2(w.handle, self.buf.ptr, rows, out.buf.ptr, ws.ptr, _stream_handle(stream)))
        if stream is not None:
            stream.synchronize()      # ws is freed on return
        else:
            _lib.check(lib.fhip_stream_sync(None))
        return out

    def ffn_f16x2(self, gate_up, down, stream=None):
        """down(swiglu(gate_up(x))) for a batch of rows <= 32 in one pass over each weight -- qwen3.rs:944-964."""
        rows, inn = self._rows_inner()
        assert inn == gate_up.cols(), "inner dim mismatch"
        lib = _lib.load()
        ws = DeviceBuffer(max(256, lib.fhip_ffn_f16x2_ws_bytes(gate_up.handle, down.handle, rows)))
        out = Tensor.empty((rows, down.rows()))
        _lib.check(lib.fhip_ffn_f16x2(gate_up.handle, down.handle, self.buf.ptr, rows, out.buf.ptr, ws.ptr, _stream_handle(stream)))
        if stream is not None:
            stream.synchronize()      # ws is freed on return
        else:
            _lib.check(lib.fhip_stream_sync(None))
        return out

    def ffn_coop(self, gate_up, down, stream=None):
        """down(swiglu(gate_up(x))) on the matrix cores, for a batch of rows -- qwen3.rs:944-964 over dtype.rs:1818."""
        rows, inn = self._rows_inner()
        assert inn == gate_up.cols(), "inner dim mismatch"
        lib = _lib.load()
        ws = DeviceBuffer(max(256, lib.fhip_ffn_coop_ws_bytes(gate_up.handle, down.handle, rows)))
        out = Tensor.empty((rows, down.rows()))
        _lib.check(lib.fhip_ffn_coop(gate_up.handle, down.handle, self.buf.ptr, rows, out.buf.ptr, ws.ptr, _stream_handle(stream)))
        if stream is not None:
            stream.synchronize()      # ws is freed on return
        else:
            _lib.check(lib.fhip_stream_sync(None))
        return out

    def gemm_q_bf16(self, w, stream=None):
        """Prefill: self holds bf16 bit patterns [t, in]; y f32 [t, out] via the matrix cores -- dtype.rs:1818."""
        assert self.dtype == np.uint16, "gemm_q_bf16 expects bf16 bit patterns"
        t, inn = self._rows_inner()
        assert inn == w.cols(), f"inner dim mismatch: x[..,{inn}] vs W[..,{w.cols()}]"
        out = Tensor.empty((t, w.rows()))
        _lib.check(_lib.load().fhip_gemm_q_bf16(w.handle, self.buf.ptr, t, out.buf.ptr, _stream_handle(stream)))
        return out


class QMatrix:
    """A packed-quant weight [rows = out, cols = in] resident in HBM as the raw GGUF block stream."""

    def __init__(self, handle, ggml_type, keepalive=None):
        self.handle, self.ggml_type, self._keepalive = handle, ggml_type, keepalive

    @staticmethod
    def block_bytes(ggml_type):
        """(values per block, bytes per block) or None -- dtype.rs:873."""
        v, b = C.c_size_t(), C.c_size_t()
        rc = _lib.load().fhip_block_bytes(ggml_type, C.byref(v), C.byref(b))
        return (v.value, b.value) if rc == _lib.OK else None

    @staticmethod
    def from_bytes(data, ggml_type, rows, cols):
        """dtype.rs:893. Unknown type -> ValueError; cols not a block multiple or a wrong byte
        length -> AssertionError (the per-format constructors' asserts)."""
        lib = _lib.init()
        a = np.ascontiguousarray(np.frombuffer(data, dtype=np.uint8) if isinstance(data, (bytes, bytearray, memoryview)) else data,
                                 dtype=np.uint8)
        h = C.c_void_p()
        _lib.check(lib.fhip_weight_create(ggml_type, _vp(a), a.size, rows, cols, C.byref(h)))
        return QMatrix(h, ggml_type)

    @staticmethod
    def from_parts(parts, ggml_type, rows, cols):
        """One weight from several byte arrays stacked along the output dim (the fused QKV / gate|up of qwen35.rs:379-402):
        every part is uploaded to its place, nothing is concatenated on the host. Errors as from_bytes."""
        lib = _lib.init()
        arrs = [np.ascontiguousarray(np.frombuffer(p, dtype=np.uint8) if isinstance(p, (bytes, bytearray, memoryview)) else p, dtype=np.uint8)
                for p in parts]
        ptrs = (C.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])
        sizes = (C.c_size_t * len(arrs))(*[a.size for a in arrs])
        h = C.c_void_p()
        _lib.check(lib.fhip_weight_create_parts(ggml_type, ptrs, sizes, len(arrs), rows, cols, C.byref(h)))
        return QMatrix(h, ggml_type)

    @staticmethod
    def wrap_device(buf, nbytes, ggml_type, rows, cols, offset=0):
        """Adopt block bytes already in HBM (buf: DeviceBuffer), no copy."""
        lib = _lib.init()
        h = C.c_void_p()
        _lib.check(lib.fhip_weight_wrap_device(ggml_type, C.c_void_p(buf.ptr.value + offset), nbytes, rows, cols, C.byref(h)))
        return QMatrix(h, ggml_type, keepalive=buf)

    def rows(self):
        return _lib.load().fhip_weight_rows(self.handle)

    def cols(self):
        return _lib.load().fhip_weight_cols(self.handle)

    def nbytes(self):
        return _lib.load().fhip_weight_nbytes(self.handle)

    def n_shards(self):
        return 1  # one HBM allocation holds any size; the reference shards only for WebGPU binding limits

    def matvec_precision(self, bits=0):
        """Activation bits of this weight's streaming mat-vec: 24 (what a new weight has: the f32 significand, the reference
        examples' 1e-5 bar) or 16 (faster, about 1e-4); 0 only queries. Returns the setting before the call."""
        rc = _lib.load().fhip_weight_matvec_precision(self.handle, bits)
        if rc < 0:
            _lib.check(rc)
        return rc

    def batch_policy(self, policy=-1):
        """Which kernels this weight's batches of three rows and more take (BATCH_ORDERED, what a new weight has, BATCH_AUTO or
        BATCH_F32_MATVEC); any other value only queries. Returns the policy before the call."""
        return _lib.load().fhip_weight_batch_policy(self.handle, policy)

    def dequant_rows(self, row0, nrows, stream=None):
        """Rows [row0, row0+nrows) dequantized on the GPU, bit-exact with deq_raw."""
        out = Tensor.empty((nrows, self.cols()))
        _lib.check(_lib.load().fhip_dequant_rows(self.handle, row0, nrows, out.buf.ptr, _stream_handle(stream)))
        return out

    def dequant(self, stream=None):
        return self.dequant_rows(0, self.rows(), stream)

    def __del__(self):
        try:
            if self.handle:
                _lib.load().fhip_weight_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


def _typed(ty, name):
    class _W:
        """Per-format constructor, same asserts as the reference's `from_bytes`."""

        @staticmethod
        def from_bytes(data, rows, cols):
            return QMatrix.from_bytes(data, ty, rows, cols)

    _W.__name__ = name
    return _W


Q8_0Weights = _typed(Q8_0, "Q8_0Weights")
Q4_KWeights = _typed(Q4_K, "Q4_KWeights")
Q6_KWeights = _typed(Q6_K, "Q6_KWeights")
Q5_KWeights = _typed(Q5_K, "Q5_KWeights")
Q4_0Weights = _typed(Q4_0, "Q4_0Weights")
Q4_1Weights = _typed(Q4_1, "Q4_1Weights")
Q5_0Weights = _typed(Q5_0, "Q5_0Weights")
Q5_1Weights = _typed(Q5_1, "Q5_1Weights")
Iq4NlWeights = _typed(IQ4_NL, "Iq4NlWeights")
Iq4XsWeights = _typed(IQ4_XS, "Iq4XsWeights")
Mxfp4Weights = _typed(MXFP4, "Mxfp4Weights")


def type_size(ty, n):
    """Bytes of n elements of ggml type ty -- lib.rs:471; unknown type -> ValueError."""
    if QMatrix.block_bytes(ty) is None and ty not in (F32, F16, BF16):
        raise ValueError(f"unsupported ggml type {ty}")
    return int(_lib.load().fhip_type_size(ty, n))


def deq_raw(raw, n, ty):
    """Dequantize n elements out of raw block bytes on the GPU -- lib.rs:497. Same edge behaviour:
    every format returns n values with a ragged tail left 0.0, except Q8_0, which returns whole blocks only; the
    unquantized types F32 / F16 / BF16 need all n elements' bytes (fewer: AssertionError, the reference's slice panic)."""
    lib = _lib.init()
    a = np.ascontiguousarray(raw, dtype=np.uint8)
    out = np.empty(n, dtype=np.float32)
    got = C.c_size_t()
    _lib.check(lib.fhip_deq_raw(_vp(a), a.size, n, ty, _vp(out), C.byref(got)))
    return out[: got.value]


def f16_to_f32(bits):
    """IEEE binary16 patterns -> f32 on the GPU -- lib.rs:605 rd_f16."""
    lib = _lib.init()
    a = np.ascontiguousarray(bits, dtype=np.uint16)
    din, dout = DeviceBuffer(a.nbytes), DeviceBuffer(a.size * 4)
    _lib.check(lib.fhip_memcpy_h2d(din.ptr, _vp(a), a.nbytes, None))
    _lib.check(lib.fhip_f16_to_f32(din.ptr, a.size, dout.ptr, None))
    out = np.empty(a.size, dtype=np.float32)
    _lib.check(lib.fhip_memcpy_d2h(_vp(out), dout.ptr, out.nbytes, None))
    return out


def matvec_q8_0(x, w, rows, cols):
    """y = x . W^T, W raw Q8_0 bytes [rows, cols], host arrays in and out -- cpu_simd.rs:79."""
    lib = _lib.init()
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.uint8)
    assert cols % 32 == 0, "Q8_0 cols must be a multiple of 32"
    assert x.size == cols, "activation length must equal cols"
    y = np.empty(rows, dtype=np.float32)
    _lib.check(lib.fhip_matvec_q8_0_host(_vp(x), _vp(w), w.size, rows, cols, _vp(y)))
    return y


def matvec_q8_0_threaded(x, w, rows, cols, threads):
    """cpu_simd.rs:92. The thread count only partitions rows on the CPU; on the GPU every
    partition gives the same result, so it is accepted and ignored."""
    del threads
    return matvec_q8_0(x, w, rows, cols)


def matvec_q8_0_span(x, w, cols, lo, hi, threads=1):
    """Rows [lo, hi) only -- cpu_simd.rs:118."""
    assert lo <= hi, "empty or inverted span"
    row_bytes = cols // 32 * 34
    w = np.ascontiguousarray(w, dtype=np.uint8)
    return matvec_q8_0_threaded(x, w[lo * row_bytes: hi * row_bytes], hi - lo, cols, threads)


class Pool:
    """cpu_simd.rs:238 Pool: set up once, reused by every matvec_q8_0_pooled call. On the GPU what it keeps is the weight
    of the last call resident in HBM (and staging buffers, and a stream), so a repeated call uploads the activations only."""

    def __init__(self, n):
        lib = _lib.init()
        self.handle = C.c_void_p()
        _lib.check(lib.fhip_pool_create(int(n), C.byref(self.handle)))
        self._w = None      # keeps the keyed array alive: its address is the pool's key

    def threads(self):
        return int(_lib.load().fhip_pool_threads(self.handle))

    def uploads(self):
        return int(_lib.load().fhip_pool_uploads(self.handle))

    def forget(self):
        _lib.load().fhip_pool_forget(self.handle)
        self._w = None

    def close(self):
        if self.handle:
            _lib.load().fhip_pool_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def matvec_q8_0_pooled(pool, x, w, cols, lo, hi):
    """Rows [lo, hi) of y = x . W^T on a pool -- cpu_simd.rs:303. `w` must be a contiguous uint8 array (its address keys the
    pool's resident copy, as the Arc does in the reference); anything else is copied and uploaded on every call."""
    lib = _lib.load()
    x = np.ascontiguousarray(x, dtype=np.float32)
    if not (isinstance(w, np.ndarray) and w.dtype == np.uint8 and w.flags.c_contiguous):
        w = np.ascontiguousarray(w, dtype=np.uint8)
    pool._w = w
    y = np.empty(max(0, hi - lo), dtype=np.float32)
    _lib.check(lib.fhip_matvec_q8_0_pooled(pool.handle, _vp(x), x.size, _vp(w), w.size, cols, lo, hi, _vp(y)))
    return y
