"""CPU restatement (numpy, f64 arithmetic on the f32 inputs) of the decode-layer steps around the quantized matmuls.

TEST INFRASTRUCTURE ONLY: imported by tests/ and the smoke check, never by the shipped package.

Each function follows the reference code it cites (paths under the reference checkout) but evaluates in float64, so that
it is the mathematical value the f32 kernels on either side approximate; the tests compare within stated tolerances.
Pinned in tests/test_oracle_decode.py by closed forms and invariants (constant rows, scale invariance, rotation norms and
angle additivity, one-key and uniform-key attention, brute-force loops over heads), not against reference outputs: the
reference's kernels are WGSL whose exp / log / sin / cos precision is implementation-defined, so bit-level answers do not
exist for them.
"""
import numpy as np


def rmsnorm(x, weight, eps):
    """crates/ferric-tensor/src/lib.rs:2018-2033: x * (1 / sqrt(mean(x^2) + eps)) * weight over the last dim."""
    x = np.asarray(x, np.float64)
    inv = 1.0 / np.sqrt((x * x).mean(axis=-1, keepdims=True) + np.float64(np.float32(eps)))
    return x * inv * np.asarray(weight, np.float64)


def add_rmsnorm(a, b, weight, eps):
    """lib.rs:2057-2074: (sum, rmsnorm(sum)); the sum is the f32 sum (one rounding), as the kernel stores it."""
    s = (np.asarray(a, np.float32) + np.asarray(b, np.float32)).astype(np.float32)
    return s, rmsnorm(s, weight, eps)


def rope_inv_freq(n_rot, base, freq_scale=None):
    """lib.rs:2145 `exp(-2 c / n_rot * ln base)`: the exact value, rounded to f32 once (times freq_scale[c], lib.rs:2106)."""
    c = np.arange(n_rot // 2, dtype=np.float64)
    inv = np.exp(-2.0 * c / n_rot * np.log(np.float64(np.float32(base)))).astype(np.float32)
    if freq_scale is not None:
        inv = (inv * np.asarray(freq_scale, np.float32)).astype(np.float32)
    return inv


def rope(x, n_heads, head_dim, base, positions, interleaved=False, n_rot=None, freq_scale=None):
    """lib.rs:2118-2162: x [t, n_heads * head_dim]; row i at positions[i]. The angle is the f32 product f32(pos) * inv the
    reference forms; its cos / sin and the rotation are evaluated in f64."""
    n_rot = head_dim if n_rot is None else n_rot
    x = np.asarray(x, np.float64)
    t = x.size // (n_heads * head_dim)
    x = x.reshape(t, n_heads, head_dim)
    out = x.copy()
    half = n_rot // 2
    inv = rope_inv_freq(n_rot, base, freq_scale)
    c = np.arange(half)
    p0, p1 = (2 * c, 2 * c + 1) if interleaved else (c, c + half)
    for i in range(t):
        ang = (np.float32(positions[i]) * inv).astype(np.float32).astype(np.float64)
        cs, sn = np.cos(ang), np.sin(ang)
        x1, x2 = x[i][:, p0], x[i][:, p1]
        out[i][:, p0] = x1 * cs - x2 * sn
        out[i][:, p1] = x2 * cs + x1 * sn
    return out.reshape(t, n_heads * head_dim)


def decode_attention(q, k, v, n_heads, n_kv_heads, window=0, softcap=0.0):
    """crates/ferric-tensor/src/nn.rs:153-166 (the composed form the fused kernel is defined by): q [n_heads * dh], k / v
    [S, n_kv_heads * dh]; head h uses KV head h // (n_heads / n_kv_heads); softmax(q.k / sqrt(dh)) @ v. softcap > 0: scaled
    scores x become cap * tanh(x / cap) (nn.rs:61, lib.rs:308); 0 < window < S: keys older than the last `window` are masked
    out (nn.rs:92-111; the reference adds -1e30 to them, which exp() turns into exactly 0)."""
    q = np.asarray(q, np.float64).reshape(n_heads, -1)
    dh = q.shape[1]
    s = np.asarray(k).shape[0]
    k = np.asarray(k, np.float64).reshape(s, n_kv_heads, dh)
    v = np.asarray(v, np.float64).reshape(s, n_kv_heads, dh)
    g = n_heads // n_kv_heads
    scale = np.float64(np.float32(1.0) / np.sqrt(np.float32(dh)))
    out = np.zeros((n_heads, dh))
    for h in range(n_heads):
        sc = k[:, h // g, :] @ q[h] * scale
        if softcap > 0:
            sc = np.float64(np.float32(softcap)) * np.tanh(sc / np.float64(np.float32(softcap)))
        if 0 < window < s:
            sc[: s - window] = -np.inf
        p = np.exp(sc - sc.max())
        out[h] = (p / p.sum()) @ v[:, h // g, :]
    return out.reshape(1, n_heads * dh)


def causal_attention(q, k, v, n_heads, n_kv_heads, window=0, softcap=0.0):
    """nn.rs:40-57, :66-88, :239-265: q [t, n_heads * dh] against k, v [s, n_kv_heads * dh], s >= t; query i sits at position
    off + i, off = s - t, sees keys 0 ..= off + i and, with a window, only those with (off + i) - j < window (:128-133): row by
    row the single-query attention over the keys up to the row's position."""
    q = np.asarray(q, np.float64)
    t, s = q.shape[0], np.asarray(k).shape[0]
    assert s >= t
    off = s - t
    return np.concatenate([decode_attention(q[i], np.asarray(k)[:off + i + 1], np.asarray(v)[:off + i + 1], n_heads, n_kv_heads, window, softcap)
                           for i in range(t)], axis=0)


def qkv_post(qkv, bias, q_norm, k_norm, positions, n_head, n_kv, hd, eps, base, interleaved=False, n_rot=None, freq_scale=None):
    """crates/ferric-llama/src/qwen3.rs:848-905: + bias, per-head RMSNorm of q and k (when the norms exist), rope of both at
    the rows' positions; returns (q [t, n_head*hd], k [t, n_kv*hd], v [t, n_kv*hd])."""
    qkv = np.asarray(qkv, np.float64)
    t = qkv.shape[0]
    if bias is not None:
        qkv = (np.asarray(qkv, np.float32) + np.asarray(bias, np.float32)).astype(np.float32).astype(np.float64)
    qo, ko = n_head * hd, n_kv * hd
    q, k, v = qkv[:, :qo], qkv[:, qo:qo + ko], qkv[:, qo + ko:]
    if q_norm is not None:
        q = rmsnorm(q.reshape(t, n_head, hd), q_norm, eps).reshape(t, qo)
    if k_norm is not None:
        k = rmsnorm(k.reshape(t, n_kv, hd), k_norm, eps).reshape(t, ko)
    q = rope(q, n_head, hd, base, positions, interleaved, n_rot, freq_scale)
    k = rope(k, n_kv, hd, base, positions, interleaved, n_rot, freq_scale)
    return q, k, v


def silu_mul(gu, n_ff):
    g, u = gu[..., :n_ff], gu[..., n_ff:]
    return g / (1.0 + np.exp(-g)) * u


def sigmoid(x):
    """crates/ferric-tensor/src/lib.rs:1915: 1 / (1 + exp(-v))."""
    return 1.0 / (1.0 + np.exp(-np.asarray(x, np.float64)))


def gelu_tanh(x):
    """lib.rs:1926: 0.5 v (1 + tanh(clamp(0.7978845608028654 (v + 0.044715 v^3), -15, 15)))."""
    v = np.asarray(x, np.float64)
    a = np.clip(0.7978845608028654 * (v + 0.044715 * v * v * v), -15.0, 15.0)
    return 0.5 * v * (1.0 + np.tanh(a))


def gelu_mul(gu, n_ff):
    """crates/ferric-llama/src/qwen3.rs:953-958: gelu_tanh(gate) * up of rows [gate | up]."""
    return gelu_tanh(gu[..., :n_ff]) * gu[..., n_ff:]


class Layer:
    """Dequantized (f64) weights of one layer: attn_norm, wqkv [q+2kv, d], wo, ffn_norm, gate_up [2 n_ff, d], down, norms.
    Optional, for the other arms of the reference's layer: window (keys a local layer attends to), rope (False: a NoPE layer),
    rope_base, attn_gate [q, d], post_attn_norm / post_ffn_norm [d]."""

    def __init__(self, **kw):
        self.__dict__.update(kw)


def apply_layer(x, l, kc, vc, pos, cfg):
    """qwen3.rs:979-1047 for one token at position pos; kc / vc are lists of earlier K / V rows (appended to). The default
    arm (:1041-1047) unless the layer or the configuration carries one of: a sliding window and a score softcap (:917-924),
    no rotation (:857-863: QK-norm still applies), its own rope base, a sigmoid gate on the attention output projected from
    the normed input (:936-938), post-norms on both branch outputs with their own epsilon (:1015-1020), GEGLU (:953-958), a
    block-quantized cache (cfg.kv_fmt, :906-912)."""
    opt = lambda o, name, default: getattr(o, name, default) if getattr(o, name, None) is not None else default
    h = rmsnorm(x, l.attn_norm, cfg.eps)
    qkv = h @ l.wqkv.T
    n_rot = cfg.head_dim if opt(l, "rope", True) else 0
    q, k, v = qkv_post(qkv.reshape(1, -1), getattr(l, "qkv_bias", None), getattr(l, "q_norm", None), getattr(l, "k_norm", None), [pos],
                       cfg.n_head, cfg.n_head_kv, cfg.head_dim, cfg.eps, opt(l, "rope_base", cfg.rope_base), cfg.rope_interleaved, n_rot)
    kv_fmt = getattr(cfg, "kv_fmt", None)
    if kv_fmt is not None:
        # the quantized arm (:906-912): the rows are stored as blocks and attention reads what dequantize() gives back
        from . import kvquant_oracle as KQ
        k = KQ.roundtrip(k.astype(np.float32), 1, k.shape[1], kv_fmt).astype(np.float64)
        v = KQ.roundtrip(v.astype(np.float32), 1, v.shape[1], kv_fmt).astype(np.float64)
    kc.append(k[0]); vc.append(v[0])
    a = decode_attention(q[0], np.stack(kc), np.stack(vc), cfg.n_head, cfg.n_head_kv, opt(l, "window", 0), opt(cfg, "attn_softcap", 0.0))
    if getattr(l, "attn_gate", None) is not None:
        a = a * sigmoid(h @ l.attn_gate.T)
    y = a[0] @ l.wo.T
    post = getattr(l, "post_attn_norm", None) is not None
    pe = opt(cfg, "post_norm_eps", cfg.eps)
    xy = x + (rmsnorm(y, l.post_attn_norm, pe) if post else y)
    gu = rmsnorm(xy, l.ffn_norm, cfg.eps) @ l.gate_up.T
    f = (gelu_mul(gu, cfg.n_ff) if opt(cfg, "geglu", False) else silu_mul(gu, cfg.n_ff)) @ l.down.T
    return xy + (rmsnorm(f, l.post_ffn_norm, pe) if post else f)
