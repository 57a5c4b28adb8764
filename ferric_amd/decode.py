"""Host mirror of the reference's decode-layer ops and of `Qwen3::apply_layer` for one new token.

The ops are the reference's `Tensor::rmsnorm / add_rmsnorm / add / rope*` (crates/ferric-tensor/src/lib.rs:279-520),
`append2` (lib.rs:1379) and `nn::decode_attention` (crates/ferric-tensor/src/nn.rs:140); `Qwen3Decoder` is
`Qwen3::attn / ffn / apply_layer` (crates/ferric-llama/src/qwen3.rs:861-966, 979-1052) for one new token on an f32 cache:
the default pre-norm arm, and per layer or configuration a sliding window, a score softcap, no rotation (NoPE), a rope
base of the layer's own, a sigmoid gate on the attention output, post-norms on both branch outputs, GEGLU.
Everything runs through libferric_hip; there is no CPU path.
"""
import ctypes as C

import numpy as np

from . import _lib
from .qmatrix import DeviceBuffer, Graph, Tensor, _stream_handle, _vp


def _check(rc):
    _lib.check(rc)


def _u32_tensor(values):
    a = np.ascontiguousarray(values, dtype=np.uint32)
    t = Tensor(DeviceBuffer(max(a.nbytes, 4)), a.shape, np.uint32)
    _check(_lib.load().fhip_memcpy_h2d(t.buf.ptr, _vp(a), a.nbytes, None))
    _check(_lib.load().fhip_stream_sync(None))
    return t


def rmsnorm(x, weight, eps, stream=None):
    """lib.rs:346: x [.., d] normalised over the last dim, times weight [d]."""
    d = x.shape[-1]
    assert weight.numel() == d, f"rmsnorm: weight has {weight.numel()} elements, rows have {d}"
    out = Tensor.empty(x.shape)
    _check(_lib.load().fhip_rmsnorm(x.buf.ptr, weight.buf.ptr, x.numel() // d, d, eps, out.buf.ptr, _stream_handle(stream)))
    return out


def add_rmsnorm(a, b, weight, eps, stream=None):
    """lib.rs:372: (a + b, rmsnorm(a + b, weight))."""
    assert a.shape == b.shape, f"add_rmsnorm: shape mismatch {list(a.shape)} vs {list(b.shape)}"
    d = a.shape[-1]
    assert weight.numel() == d
    s, n = Tensor.empty(a.shape), Tensor.empty(a.shape)
    _check(_lib.load().fhip_add_rmsnorm(a.buf.ptr, b.buf.ptr, weight.buf.ptr, a.numel() // d, d, eps, s.buf.ptr, n.buf.ptr,
                                        _stream_handle(stream)))
    return s, n


def add(a, b, stream=None):
    """lib.rs:279 for equal shapes."""
    assert a.shape == b.shape, "add: shapes differ (no broadcasting on this path)"
    out = Tensor.empty(a.shape)
    _check(_lib.load().fhip_add(a.buf.ptr, b.buf.ptr, a.numel(), out.buf.ptr, _stream_handle(stream)))
    return out


def mul_sigmoid(a, g, stream=None):
    """a * sigmoid(g), equal shapes -- the attention gate of qwen3.rs:936-938."""
    assert a.shape == g.shape, "mul_sigmoid: shapes differ"
    out = Tensor.empty(a.shape)
    _check(_lib.load().fhip_mul_sigmoid(a.buf.ptr, g.buf.ptr, a.numel(), out.buf.ptr, _stream_handle(stream)))
    return out


def geglu(gu, stream=None):
    """gelu_tanh(gate) * up for rows [gate | up] -- qwen3.rs:953-958 with lib.rs:304."""
    assert gu.shape[-1] % 2 == 0, "geglu: rows hold gate | up"
    d = gu.shape[-1] // 2
    out = Tensor.empty(tuple(gu.shape[:-1]) + (d,))
    _check(_lib.load().fhip_geglu(gu.buf.ptr, gu.numel() // (2 * d), d, out.buf.ptr, _stream_handle(stream)))
    return out


def rope(x, n_heads, head_dim, base, offset=0, positions=None, freq_scale=None, interleaved=False, n_rot=None, stream=None):
    """lib.rs:417 rope (split-half pairs), :409 rope_interleaved, :429 rope_partial (n_rot), :465 rope_at / :489 rope_at_ex
    (positions: one absolute position per row, host values or a device u32 Tensor)."""
    n_rot = head_dim if n_rot is None else n_rot
    assert n_rot <= head_dim and n_rot % 2 == 0, "n_rot must be even and <= head_dim"
    t = x.numel() // (n_heads * head_dim)
    pos_t = None
    if positions is not None:
        pos_t = positions if isinstance(positions, Tensor) else _u32_tensor(positions)
        assert pos_t.numel() == t, f"rope_at needs one position per row: {t} rows, {pos_t.numel()} given"
    out = Tensor.empty(x.shape)
    _check(_lib.load().fhip_rope(x.buf.ptr, 0, t, n_heads, head_dim, n_rot, base, pos_t.buf.ptr if pos_t is not None else None, offset,
                                 freq_scale.buf.ptr if freq_scale is not None else None, int(interleaved), out.buf.ptr,
                                 _stream_handle(stream)))
    if pos_t is not None and not isinstance(positions, Tensor):
        _check(_lib.load().fhip_stream_sync(_stream_handle(stream)))     # the temporary position buffer is freed on return
    return out


class KvCache:
    """One layer's K and V history, [cap, width] f32 each, filled to `len` rows (the reference's pair of KvBuf, lib.rs:1287,
    with a fixed capacity: a captured step cannot reallocate)."""

    def __init__(self, cap, width):
        self.cap, self.width, self.len = int(cap), int(width), 0
        self.k, self.v = Tensor.empty((cap, width)), Tensor.empty((cap, width))

    def append2(self, k, v, stream=None):
        """lib.rs:1379: rows of k and v [t, width] appended to both caches in one launch."""
        assert len(k.shape) == 2 and len(v.shape) == 2, "append2 expects 2D [t, width] tensors"
        assert k.shape[0] == v.shape[0], "K and V must append the same number of rows"
        assert k.shape[1] == self.width and v.shape[1] == self.width, "KvBuf width changed"
        t = k.shape[0]
        assert self.len + t <= self.cap, f"KvCache: {self.len} + {t} rows exceed the capacity {self.cap}"
        _check(_lib.load().fhip_kv_append2(k.buf.ptr, v.buf.ptr, t, self.width, None, self.len, self.k.buf.ptr, self.v.buf.ptr, self.cap,
                                           _stream_handle(stream)))
        self.len += t
        return self


def decode_attention(q, cache, n_heads, n_kv_heads, length=None, last_pos=None, ws=None, stream=None, window=0, softcap=0.0):
    """nn.rs:140 (window / softcap: nn.rs:92 decode_attention_win and the softcapped scores of nn.rs:61): q [1, n_heads * dh] against the first `length` rows of the cache (default: all filled rows). last_pos: a
    device u32 Tensor holding the newest row's index, read at run time instead (for a captured step)."""
    assert len(q.shape) == 2 and q.shape[0] == 1, "decode_attention takes one query row"
    dh = q.shape[1] // n_heads
    length = cache.len if length is None else length
    assert 1 <= length <= cache.cap, f"decode_attention: length {length} outside the cache's 1..={cache.cap} rows"
    assert cache.width == n_kv_heads * dh
    lib = _lib.load()
    need = lib.fhip_decode_attention_ws_bytes(n_heads, n_kv_heads, dh, length)
    own = None
    if need and ws is None:
        own = ws = DeviceBuffer(need)
    out = Tensor.empty((1, n_heads * dh))
    _check(lib.fhip_decode_attention_ex(q.buf.ptr, cache.k.buf.ptr, cache.v.buf.ptr, n_heads, n_kv_heads, dh, length,
                                        last_pos.buf.ptr if last_pos is not None else None, window, softcap,
                                        ws.ptr if ws is not None else None, out.buf.ptr, _stream_handle(stream)))
    if own is not None:
        _check(lib.fhip_stream_sync(_stream_handle(stream)))   # the scratch is freed on return
    return out


def causal_attention(q, k, v, n_heads, n_kv_heads, window=0, softcap=0.0, stream=None):
    """nn.rs:40 causal_attention / :66 causal_attention_win / :239 chunked_attention: q [t, n_heads * dh] against k, v
    [s, n_kv_heads * dh] with s >= t; query i at position s - t + i."""
    t, s = q.shape[0], k.shape[0]
    assert s >= t, f"cache ({s}) cannot be shorter than the query block ({t})"
    assert k.shape == v.shape and k.shape[1] * n_heads == q.shape[1] * n_kv_heads
    out = Tensor.empty(q.shape)
    _check(_lib.load().fhip_causal_attention(q.buf.ptr, k.buf.ptr, v.buf.ptr, t, s, n_heads, n_kv_heads, q.shape[1] // n_heads, window, softcap,
                                             out.buf.ptr, _stream_handle(stream)))
    return out


def decode_attention_kvq(q, kcache, vcache, n_heads, n_kv_heads, length=None, last_pos=None, ws=None, stream=None, window=0, softcap=0.0):
    """decode_attention over a pair of block-quantized caches (kvquant.QKvCache) read in place -- the quantized arm of
    qwen3.rs:906-924 without the dequantized copy of the history."""
    assert len(q.shape) == 2 and q.shape[0] == 1, "decode_attention takes one query row"
    dh = q.shape[1] // n_heads
    length = kcache.len if length is None else length
    assert kcache.fmt == vcache.fmt and kcache.width == vcache.width == n_kv_heads * dh
    assert 1 <= length <= min(kcache.cap, vcache.cap), f"decode_attention: length {length} outside the caches"
    lib = _lib.load()
    need = lib.fhip_decode_attention_ws_bytes(n_heads, n_kv_heads, dh, length)
    own = None
    if need and ws is None:
        own = ws = DeviceBuffer(need)
    out = Tensor.empty((1, n_heads * dh))
    _check(lib.fhip_decode_attention_kvq(kcache.fmt, q.buf.ptr, kcache.codes.ptr, kcache.scales.ptr, vcache.codes.ptr, vcache.scales.ptr,
                                         n_heads, n_kv_heads, dh, length, last_pos.buf.ptr if last_pos is not None else None, window, softcap,
                                         ws.ptr if ws is not None else None, out.buf.ptr, _stream_handle(stream)))
    if own is not None:
        _check(lib.fhip_stream_sync(_stream_handle(stream)))   # the scratch is freed on return
    return out


class Qwen3Cfg:
    """The fields of the reference's Cfg this path reads (qwen3.rs:60-100: n_head, n_head_kv, head_dim, eps, rope pairing,
    attn_softcap, post_norm_eps; geglu stands for is_gemma's FFN activation, qwen3.rs:953)."""

    def __init__(self, d_model, n_head, n_head_kv, head_dim, n_ff, eps=1e-6, rope_base=1e6, rope_interleaved=False, attn_softcap=0.0,
                 post_norm_eps=None, geglu=False):
        self.d_model, self.n_head, self.n_head_kv, self.head_dim, self.n_ff = d_model, n_head, n_head_kv, head_dim, n_ff
        self.eps, self.rope_base, self.rope_interleaved = float(eps), float(rope_base), bool(rope_interleaved)
        self.attn_softcap = float(attn_softcap)
        self.post_norm_eps = float(eps if post_norm_eps is None else post_norm_eps)
        self.geglu = bool(geglu)


class Qwen3Layer:
    """qwen3.rs:230-253: norms as f32 Tensors, projections as QMatrix (wqkv = q|k|v stacked, ffn_gate_up = gate|up stacked).
    Beyond the default arm: window (> 0: a local layer attends to that many newest keys), rope (False: a NoPE layer, QK-norm
    only), rope_base (None: the configuration's), attn_gate (QMatrix [n_head * head_dim, d_model]), post_attn_norm and
    post_ffn_norm (both or neither)."""

    def __init__(self, attn_norm, wqkv, wo, ffn_norm, ffn_gate_up, ffn_down, q_norm=None, k_norm=None, qkv_bias=None, window=0,
                 rope=True, rope_base=None, attn_gate=None, post_attn_norm=None, post_ffn_norm=None):
        self.attn_norm, self.wqkv, self.wo, self.ffn_norm = attn_norm, wqkv, wo, ffn_norm
        self.ffn_gate_up, self.ffn_down, self.q_norm, self.k_norm, self.qkv_bias = ffn_gate_up, ffn_down, q_norm, k_norm, qkv_bias
        self.window, self.rope, self.rope_base, self.attn_gate = int(window), bool(rope), rope_base, attn_gate
        assert (post_attn_norm is None) == (post_ffn_norm is None), "the two post-norms come together (qwen3.rs:567-568)"
        self.post_attn_norm, self.post_ffn_norm = post_attn_norm, post_ffn_norm


class Qwen3Decoder:
    """One-token decode through a stack of layers with preallocated activations, so that a whole step is a fixed sequence
    of launches (capturable as one graph). Per layer, 7 launches (6 with the second and third in one):
        qkv = rmsnorm(x [+ previous FFN output]) Wqkv^T   [norm and residual add formed inside the mat-vec]
        q/k norm + rope + cache append;  attention;  combine of its splits;  o = a Wo^T
        f = swiglu(rmsnorm(x + o) Wgu^T)                  [again inside the mat-vec];  y = f Wdown^T
    With fuse_norm=False the norms run as their own launches (9 per layer), as the reference issues them. With fuse_attn=True
    (also what None, the default, means) the q/k norm + rope + cache append happen inside the attention launch, 6 launches per layer.
    A gated layer adds two launches (the gate's mat-vec on the same normed input, the sigmoid product), post-norms two (the
    RMSNorm of each branch output; the add happens inside the next mat-vec as before), GEGLU one (the activation on its own).
    kv_fmt: the caches are block-quantized (kvquant.QKvCache pairs of fixed capacity): the token's K and V rows are quantized by
    one launch and attention reads the blocks in place, 8 launches per layer; no f32 copy of the history exists.
    """

    def __init__(self, cfg, layers, max_len, stream=None, output_norm=None, lm_head=None, fuse_norm=True, fuse_attn=None, kv_fmt=None):
        self.cfg, self.layers, self.max_len, self.stream, self.fuse_norm = cfg, layers, int(max_len), stream, bool(fuse_norm)
        self.fuse_attn = fuse_attn
        self.kv_fmt = kv_fmt                              # None: f32 caches; else kvquant.Q8_0 / Q4_0 / Q4_1 (Cache::with_kvq, qwen3.rs:303)
        self.output_norm, self.lm_head = output_norm, lm_head          # final norm + LM head: hidden -> logits in the same step
        assert (output_norm is None) == (lm_head is None), "output_norm and lm_head come together"
        self.logits = Tensor.empty((1, lm_head.rows())) if lm_head is not None else None
        c = cfg
        self.q_out, self.kv_out = c.n_head * c.head_dim, c.n_head_kv * c.head_dim
        if kv_fmt is None:
            self.caches = [KvCache(max_len, self.kv_out) for _ in layers]
        else:
            from .kvquant import QKvCache
            self.caches = [(QKvCache(kv_fmt, max_len, self.kv_out), QKvCache(kv_fmt, max_len, self.kv_out)) for _ in layers]
            self.k1, self.v1 = Tensor.empty((1, self.kv_out)), Tensor.empty((1, self.kv_out))     # the new token's rows before they are stored
            fuse_attn = self.fuse_attn = False            # the rows are quantized by a launch of their own
        self.pos = _u32_tensor([0])                       # device word: the position of the token being decoded
        self.xa = Tensor.empty((1, c.d_model))            # residual stream: the step's input is written here ...
        self.xb = Tensor.empty((1, c.d_model))            # ... and the residual alternates between the two buffers
        self.x = self.xa                                  # where the last step left the hidden state
        self.h = Tensor.empty((1, c.d_model))             # normed input of the current block (unfused path / scratch)
        self.qkv = Tensor.empty((1, self.q_out + 2 * self.kv_out))
        self.q = Tensor.empty((1, self.q_out))
        self.att = Tensor.empty((1, self.q_out))
        self.o = Tensor.empty((1, c.d_model))
        self.f = Tensor.empty((1, c.n_ff))
        self.y = Tensor.empty((1, c.d_model))
        self.gate = Tensor.empty((1, self.q_out)) if any(l.attn_gate is not None for l in layers) else None
        self.gu = Tensor.empty((1, 2 * c.n_ff)) if c.geglu else None
        post = any(l.post_attn_norm is not None for l in layers)
        self.on = Tensor.empty((1, c.d_model)) if post else None      # post-normed attention branch
        self.yn = Tensor.empty((1, c.d_model)) if post else None      # post-normed FFN branch
        lib = _lib.load()
        need = lib.fhip_decode_attention_ws_bytes(c.n_head, c.n_head_kv, c.head_dim, self.max_len)
        self.ws = DeviceBuffer(need) if need else None
        if self.fuse_attn is None:
            # Every attention workgroup repeats the query post-processing in front of its keys; that stays cheaper than a launch
            # of its own up to 2048 keys (5.12 -> 5.06 ms/token there, 4.92 -> 4.84 at 128) and is level with it from 4096 on.
            self.fuse_attn = True
        self.fuse_attn = bool(self.fuse_attn)
        # a default-arm layer; caches of up to 256 rows under grouped query heads need no combine launch behind the attention
        short = self.max_len <= 256 and c.n_head > c.n_head_kv
        self.launches_per_layer = ((7 if self.fuse_norm else 9) - (1 if self.fuse_attn else 0) + (1 if kv_fmt is not None else 0)
                                   - (1 if short else 0))
        # per token beside the layers: the position word's increment and the head (final norm inside the head's mat-vec; a head of
        # 128 MB and more takes the norm as a launch of its own, which costs less than the wider workgroups the fused norm needs)
        big_head = lm_head is not None and lm_head.nbytes() >= (128 << 20)
        self.launches_per_token_extra = 1 + ((1 if self.fuse_norm and not big_head else 2) if lm_head is not None else 0)
        self._graph = None

    # -- state ------------------------------------------------------------------------------------
    def set_pos(self, pos):
        a = np.array([pos], np.uint32)
        _check(_lib.load().fhip_memcpy_h2d(self.pos.buf.ptr, _vp(a), 4, _stream_handle(self.stream)))
        _check(_lib.load().fhip_stream_sync(_stream_handle(self.stream)))
        for c in self._all_caches():
            c.len = pos

    def _all_caches(self):
        return self.caches if self.kv_fmt is None else [c for pair in self.caches for c in pair]

    def set_input(self, x_host):
        a = np.ascontiguousarray(x_host, dtype=np.float32).reshape(-1)
        assert a.size == self.cfg.d_model
        _check(_lib.load().fhip_memcpy_h2d(self.xa.buf.ptr, _vp(a), a.nbytes, _stream_handle(self.stream)))
        _check(_lib.load().fhip_stream_sync(_stream_handle(self.stream)))

    # -- one step ---------------------------------------------------------------------------------
    def _norm_matmul(self, w, cur, alt, resid, norm_w, y, swiglu):
        """y = [swiglu] rmsnorm(cur [+ resid]) W^T; returns the buffer that holds cur + resid afterwards."""
        lib, c, s = _lib.load(), self.cfg, _stream_handle(self.stream)
        if self.fuse_norm:
            _check(lib.fhip_norm_matmul_q(w.handle, cur.buf.ptr, resid.buf.ptr if resid is not None else None, norm_w.buf.ptr, c.eps,
                                          alt.buf.ptr if resid is not None else None, self.h.buf.ptr, int(swiglu), y.buf.ptr, s))
            return alt if resid is not None else cur
        if resid is None:
            _check(lib.fhip_rmsnorm(cur.buf.ptr, norm_w.buf.ptr, 1, c.d_model, c.eps, self.h.buf.ptr, s))
        else:   # the residual updated in place, and its norm, in one launch
            _check(lib.fhip_add_rmsnorm(cur.buf.ptr, resid.buf.ptr, norm_w.buf.ptr, 1, c.d_model, c.eps, cur.buf.ptr, self.h.buf.ptr, s))
        fn = lib.fhip_matmul_q_swiglu if swiglu else lib.fhip_matmul_q
        _check(fn(w.handle, self.h.buf.ptr, 1, y.buf.ptr, s))
        return cur

    def _enqueue_step(self):
        """All layers on the input in xa at position *pos; leaves the final hidden state in self.x and advances *pos."""
        lib, c, s = _lib.load(), self.cfg, _stream_handle(self.stream)
        cur, alt = self.xa, self.xb
        other = lambda t: self.xb if t is self.xa else self.xa
        pending = None                                   # the previous layer's FFN branch, not yet added to the residual
        for il, (l, kv) in enumerate(zip(self.layers, self.caches)):
            cur = self._norm_matmul(l.wqkv, cur, alt, pending, l.attn_norm, self.qkv, False)
            alt = other(cur)
            if l.attn_gate is not None:                  # the gate projects the same normed input (qwen3.rs:936-938)
                if self.fuse_norm:
                    self._norm_matmul(l.attn_gate, cur, alt, None, l.attn_norm, self.gate, False)
                else:                                    # self.h still holds the normed input
                    _check(lib.fhip_matmul_q(l.attn_gate.handle, self.h.buf.ptr, 1, self.gate.buf.ptr, s))
            n_rot = c.head_dim if l.rope else 0          # NoPE: q/k norm only (qwen3.rs:857-863)
            base = c.rope_base if l.rope_base is None else float(l.rope_base)
            bias = l.qkv_bias.buf.ptr if l.qkv_bias is not None else None
            qn = l.q_norm.buf.ptr if l.q_norm is not None else None
            kn = l.k_norm.buf.ptr if l.k_norm is not None else None
            ws = self.ws.ptr if self.ws is not None else None
            if self.kv_fmt is not None:
                # the quantized arm (qwen3.rs:906-912): post-process, store the token's rows as blocks, attend over the blocks
                kq, vq = kv
                _check(lib.fhip_qkv_post_packed(self.qkv.buf.ptr, bias, qn, kn, self.pos.buf.ptr, None, 1, c.n_head, c.n_head_kv, c.head_dim, n_rot,
                                                int(c.rope_interleaved), c.eps, base, self.q.buf.ptr, self.k1.buf.ptr, self.v1.buf.ptr, s))
                _check(lib.fhip_kvq_append2(self.kv_fmt, self.k1.buf.ptr, self.v1.buf.ptr, 0, 1, self.kv_out, self.pos.buf.ptr, 0, kq.cap,
                                            kq.codes.ptr, kq.scales.ptr, vq.codes.ptr, vq.scales.ptr, s))
                _check(lib.fhip_decode_attention_kvq(self.kv_fmt, self.q.buf.ptr, kq.codes.ptr, kq.scales.ptr, vq.codes.ptr, vq.scales.ptr, c.n_head,
                                                     c.n_head_kv, c.head_dim, self.max_len, self.pos.buf.ptr, l.window, c.attn_softcap, ws,
                                                     self.att.buf.ptr, s))
            elif self.fuse_attn:
                _check(lib.fhip_qkv_post_attention(self.qkv.buf.ptr, bias, qn, kn, self.pos.buf.ptr, None, c.n_head, c.n_head_kv, c.head_dim,
                                                   n_rot, int(c.rope_interleaved), c.eps, base, kv.k.buf.ptr, kv.v.buf.ptr, kv.cap,
                                                   self.max_len, l.window, c.attn_softcap, ws, self.att.buf.ptr, s))
            else:
                _check(lib.fhip_qkv_post(self.qkv.buf.ptr, bias, qn, kn, self.pos.buf.ptr, None, 1, c.n_head, c.n_head_kv, c.head_dim, n_rot,
                                         int(c.rope_interleaved), c.eps, base, self.q.buf.ptr, kv.k.buf.ptr, kv.v.buf.ptr, kv.cap, s))
                _check(lib.fhip_decode_attention_ex(self.q.buf.ptr, kv.k.buf.ptr, kv.v.buf.ptr, c.n_head, c.n_head_kv, c.head_dim, self.max_len,
                                                    self.pos.buf.ptr, l.window, c.attn_softcap, ws, self.att.buf.ptr, s))
            if l.attn_gate is not None:
                _check(lib.fhip_mul_sigmoid(self.att.buf.ptr, self.gate.buf.ptr, self.q_out, self.att.buf.ptr, s))
            _check(lib.fhip_matmul_q(l.wo.handle, self.att.buf.ptr, 1, self.o.buf.ptr, s))
            branch = self.o
            if l.post_attn_norm is not None:             # x + post_attn_norm(attn(..)), its own epsilon (qwen3.rs:1015-1018)
                _check(lib.fhip_rmsnorm(self.o.buf.ptr, l.post_attn_norm.buf.ptr, 1, c.d_model, c.post_norm_eps, self.on.buf.ptr, s))
                branch = self.on
            if c.geglu:                                  # Gemma: gate|up unfused, gelu_tanh(gate) * up (qwen3.rs:953-958)
                cur = self._norm_matmul(l.ffn_gate_up, cur, alt, branch, l.ffn_norm, self.gu, False)
                _check(lib.fhip_geglu(self.gu.buf.ptr, 1, c.n_ff, self.f.buf.ptr, s))
            else:
                cur = self._norm_matmul(l.ffn_gate_up, cur, alt, branch, l.ffn_norm, self.f, True)
            alt = other(cur)
            _check(lib.fhip_matmul_q(l.ffn_down.handle, self.f.buf.ptr, 1, self.y.buf.ptr, s))
            pending = self.y
            if l.post_ffn_norm is not None:              # x1 + post_ffn_norm(ffn(..)) (qwen3.rs:1019-1020)
                _check(lib.fhip_rmsnorm(self.y.buf.ptr, l.post_ffn_norm.buf.ptr, 1, c.d_model, c.post_norm_eps, self.yn.buf.ptr, s))
                pending = self.yn
        if self.lm_head is not None:   # last residual add fused with the output norm, then the LM head
            cur = self._norm_matmul(self.lm_head, cur, alt, pending, self.output_norm, self.logits, False)
        else:
            _check(lib.fhip_add(cur.buf.ptr, pending.buf.ptr, c.d_model, cur.buf.ptr, s))
        self.x = cur
        _check(lib.fhip_u32_add(self.pos.buf.ptr, 1, 1, s))

    # -- a block of prompt rows -------------------------------------------------------------------
    def prefill(self, x_host, precise=False):
        """`forward_cached` for t > 1 rows (qwen3.rs:979-1052 with the attention arms of :917-930): hidden rows x [t, d_model] at
        the positions behind what the caches hold; appends their K and V rows, leaves the position word behind them and returns
        the rows' final hidden states [t, d_model] (host). Eager, with buffers of its own. The projections run on the bf16
        matrix cores (fhip_matmul_q_coop / fhip_ffn_coop, the reference's coop route for prompt rows, dtype.rs:1818); precise=True
        takes fhip_matmul_q / fhip_ffn instead, whose results have the f32 grade of the decode step. Attention is
        fhip_causal_attention over the cache; on a quantized cache the rows are stored as blocks first and attention reads
        what they dequantize to, as the reference does (qwen3.rs:906-912)."""
        lib, c, s = _lib.load(), self.cfg, _stream_handle(self.stream)
        x = np.ascontiguousarray(x_host, dtype=np.float32).reshape(-1, c.d_model)
        t = x.shape[0]
        pos0 = self._all_caches()[0].len
        assert pos0 + t <= self.max_len, f"prefill: {pos0} + {t} rows exceed the capacity {self.max_len}"
        E = Tensor.empty
        X = Tensor.from_vec(x, x.shape, self.stream)
        positions = _u32_tensor(np.arange(pos0, pos0 + t))
        h, qkv, q, att = E((t, c.d_model)), E((t, self.q_out + 2 * self.kv_out)), E((t, self.q_out)), E((t, self.q_out))
        o, x1, y = E((t, c.d_model)), E((t, c.d_model)), E((t, c.d_model))
        normed = E((t, c.d_model)) if self.on is not None else None                   # a post-normed branch output
        f, gu = E((t, c.n_ff)), (E((t, 2 * c.n_ff)) if c.geglu else None)
        gate = E((t, self.q_out)) if self.gate is not None else None
        ws16 = DeviceBuffer(2 * t * max(c.d_model, self.q_out, c.n_ff) + 256)          # bf16 copies of the coop matmuls' inputs
        k1 = v1 = kd = vd = None
        if self.kv_fmt is not None:
            k1, v1 = E((t, self.kv_out)), E((t, self.kv_out))
            kd, vd = E((pos0 + t, self.kv_out)), E((pos0 + t, self.kv_out))          # what the stored blocks dequantize to
        wsf = [None]

        def matmul(w, a, out):
            if precise:
                _check(lib.fhip_matmul_q(w.handle, a.buf.ptr, t, out.buf.ptr, s))
            else:
                _check(lib.fhip_matmul_q_coop(w.handle, a.buf.ptr, t, out.buf.ptr, ws16.ptr, s))

        def ffn(l, a, out):
            if c.geglu:
                matmul(l.ffn_gate_up, a, gu)
                _check(lib.fhip_geglu(gu.buf.ptr, t, c.n_ff, f.buf.ptr, s))
                matmul(l.ffn_down, f, out)
            elif precise:
                _check(lib.fhip_ffn(l.ffn_gate_up.handle, l.ffn_down.handle, a.buf.ptr, t, out.buf.ptr, f.buf.ptr, s))
            else:
                need = lib.fhip_ffn_coop_ws_bytes(l.ffn_gate_up.handle, l.ffn_down.handle, t)
                if wsf[0] is None or wsf[0].nbytes < need:
                    wsf[0] = DeviceBuffer(max(need, 256))
                _check(lib.fhip_ffn_coop(l.ffn_gate_up.handle, l.ffn_down.handle, a.buf.ptr, t, out.buf.ptr, wsf[0].ptr, s))

        for l, kv in zip(self.layers, self.caches):
            _check(lib.fhip_rmsnorm(X.buf.ptr, l.attn_norm.buf.ptr, t, c.d_model, c.eps, h.buf.ptr, s))
            matmul(l.wqkv, h, qkv)
            bias = l.qkv_bias.buf.ptr if l.qkv_bias is not None else None
            qn = l.q_norm.buf.ptr if l.q_norm is not None else None
            kn = l.k_norm.buf.ptr if l.k_norm is not None else None
            n_rot = c.head_dim if l.rope else 0
            base = c.rope_base if l.rope_base is None else float(l.rope_base)
            if self.kv_fmt is None:
                _check(lib.fhip_qkv_post(qkv.buf.ptr, bias, qn, kn, positions.buf.ptr, None, t, c.n_head, c.n_head_kv, c.head_dim, n_rot,
                                         int(c.rope_interleaved), c.eps, base, q.buf.ptr, kv.k.buf.ptr, kv.v.buf.ptr, kv.cap, s))
                kp, vp = kv.k.buf.ptr, kv.v.buf.ptr
            else:
                kq, vq = kv
                _check(lib.fhip_qkv_post_packed(qkv.buf.ptr, bias, qn, kn, positions.buf.ptr, None, t, c.n_head, c.n_head_kv, c.head_dim, n_rot,
                                                int(c.rope_interleaved), c.eps, base, q.buf.ptr, k1.buf.ptr, v1.buf.ptr, s))
                _check(lib.fhip_kvq_append2(self.kv_fmt, k1.buf.ptr, v1.buf.ptr, 0, t, self.kv_out, positions.buf.ptr, 0, kq.cap, kq.codes.ptr,
                                            kq.scales.ptr, vq.codes.ptr, vq.scales.ptr, s))
                for cache, dst in ((kq, kd), (vq, vd)):
                    _check(lib.fhip_kvq_dequantize_rows(self.kv_fmt, cache.codes.ptr, cache.scales.ptr, 0, pos0 + t, self.kv_out, None,
                                                        dst.buf.ptr, s))
                kp, vp = kd.buf.ptr, vd.buf.ptr
            _check(lib.fhip_causal_attention(q.buf.ptr, kp, vp, t, pos0 + t, c.n_head, c.n_head_kv, c.head_dim, l.window, c.attn_softcap,
                                             att.buf.ptr, s))
            if l.attn_gate is not None:
                matmul(l.attn_gate, h, gate)
                _check(lib.fhip_mul_sigmoid(att.buf.ptr, gate.buf.ptr, t * self.q_out, att.buf.ptr, s))
            matmul(l.wo, att, o)
            branch = o
            if l.post_attn_norm is not None:
                _check(lib.fhip_rmsnorm(o.buf.ptr, l.post_attn_norm.buf.ptr, t, c.d_model, c.post_norm_eps, normed.buf.ptr, s))
                branch = normed
            _check(lib.fhip_add_rmsnorm(X.buf.ptr, branch.buf.ptr, l.ffn_norm.buf.ptr, t, c.d_model, c.eps, x1.buf.ptr, h.buf.ptr, s))
            ffn(l, h, y)
            branch = y
            if l.post_ffn_norm is not None:
                _check(lib.fhip_rmsnorm(y.buf.ptr, l.post_ffn_norm.buf.ptr, t, c.d_model, c.post_norm_eps, normed.buf.ptr, s))
                branch = normed
            _check(lib.fhip_add(x1.buf.ptr, branch.buf.ptr, t * c.d_model, X.buf.ptr, s))
        _check(lib.fhip_u32_add(self.pos.buf.ptr, 1, t, s))
        out = X.to_vec(self.stream).reshape(t, c.d_model)      # synchronises: the temporaries may go
        for cache in self._all_caches():
            cache.len += t
        return out

    def step(self):
        """Eager: enqueue one step and account for the appended row."""
        self._enqueue_step()
        for c in self._all_caches():
            c.len += 1

    def capture(self):
        """The same step as one graph; replay with step_graph()."""
        assert self.stream is not None, "capture needs a stream from Stream()"
        g = Graph.begin(self.stream)
        self._enqueue_step()
        self._graph = g.end()
        return self._graph

    def step_graph(self):
        self._graph.launch()
        for c in self._all_caches():
            c.len += 1

    def hidden(self):
        return self.x.to_vec(self.stream)
