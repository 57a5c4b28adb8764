"""Pins the numpy restatement of the decode-layer steps (oracle/decode_oracle.py) with closed forms, invariants and
brute-force loops: a dropped eps, a wrong pairing, a transposed GQA map or a missing 1/sqrt(dh) fails one of them."""
import math

import numpy as np
import pytest

from oracle import decode_oracle as D


def test_rmsnorm_closed_forms():
    w = np.array([1.0, 2.0, -1.0, 0.5])
    out = D.rmsnorm(np.full((1, 4), 3.0, np.float32), w, 0.25)
    assert np.allclose(out, 3.0 / math.sqrt(9.0 + 0.25) * w, rtol=1e-14)              # constant row: mean square = c^2
    x = np.random.default_rng(0).standard_normal((5, 64)).astype(np.float32)
    y = D.rmsnorm(x, np.ones(64), 0.0)
    assert np.allclose((y * y).mean(axis=1), 1.0, rtol=1e-12)                            # unit mean square when eps = 0
    assert np.allclose(D.rmsnorm(x * np.float32(8.0), np.ones(64), 0.0), y, rtol=1e-12)  # scale invariant without eps
    assert np.allclose(D.rmsnorm(np.zeros((1, 4), np.float32), w, 1e-6), 0.0)            # eps keeps the zero row finite
    one = np.zeros((1, 4), np.float32); one[0, 2] = 2.0                                  # mean square 1: x / sqrt(1 + eps) * w
    assert np.allclose(D.rmsnorm(one, w, 3.0), [0, 0, 2.0 / 2.0 * -1.0, 0], rtol=1e-14)


def test_add_rmsnorm_is_add_then_rmsnorm_with_an_f32_sum():
    rng = np.random.default_rng(1)
    a, b = rng.standard_normal((3, 32)).astype(np.float32), rng.standard_normal((3, 32)).astype(np.float32)
    w = rng.standard_normal(32).astype(np.float32)
    s, n = D.add_rmsnorm(a, b, w, 1e-5)
    assert s.dtype == np.float32 and np.array_equal(s, a + b)
    assert np.array_equal(n, D.rmsnorm(a + b, w, 1e-5))


def test_rope_closed_forms():
    assert np.allclose(D.rope_inv_freq(8, 10000.0), [1.0, 0.1, 0.01, 0.001], rtol=1e-7)   # base^(-2c / n_rot)
    assert np.allclose(D.rope_inv_freq(8, 10000.0, [1, 2, 4, 8]), [1.0, 0.2, 0.04, 0.008], rtol=1e-7)
    x = np.random.default_rng(2).standard_normal((3, 2 * 8)).astype(np.float32)
    assert np.array_equal(D.rope(x, 2, 8, 1e4, [0, 0, 0]), x.astype(np.float64))           # position 0 is the identity
    # pair 0 turns by exactly `pos` radians; split-half partners are (0, 4), interleaved (0, 1)
    e = np.zeros((1, 8), np.float32); e[0, 0] = 1.0
    r = D.rope(e, 1, 8, 1e4, [3])
    assert np.allclose(r[0, [0, 4]], [math.cos(3.0), math.sin(3.0)], rtol=1e-12) and not r[0, [1, 2, 3, 5, 6, 7]].any()
    r = D.rope(e, 1, 8, 1e4, [3], interleaved=True)
    assert np.allclose(r[0, [0, 1]], [math.cos(3.0), math.sin(3.0)], rtol=1e-12) and not r[0, 2:].any()
    e = np.zeros((1, 8), np.float32); e[0, 5] = 1.0          # second element of pair 1 (split-half): angle 3 * 0.1, turns towards -x
    r = D.rope(e, 1, 8, 1e4, [3])
    a = float(np.float32(3.0) * np.float32(0.1))
    assert np.allclose(r[0, [1, 5]], [-math.sin(a), math.cos(a)], rtol=1e-12)
    # rotations: norms of pairs are kept, angles add
    y = D.rope(x, 2, 8, 1e4, [5, 9, 200])
    xs, ys = x.reshape(3, 2, 2, 4).astype(np.float64), y.reshape(3, 2, 2, 4)
    assert np.allclose((xs ** 2).sum(axis=2), (ys ** 2).sum(axis=2), rtol=1e-12)
    assert np.allclose(D.rope(D.rope(x, 2, 8, 1e4, [2, 4, 8]), 2, 8, 1e4, [3, 5, 8]), D.rope(x, 2, 8, 1e4, [5, 9, 16]), atol=2e-6)
    # partial rotation leaves the tail alone and equals a full rotation of the leading n_rot dims
    part = D.rope(x, 2, 8, 1e4, [5, 9, 200], n_rot=4)
    assert np.array_equal(part.reshape(3, 2, 8)[:, :, 4:], x.reshape(3, 2, 8)[:, :, 4:].astype(np.float64))
    lead = np.ascontiguousarray(x.reshape(3, 2, 8)[:, :, :4]).reshape(3, 8)
    assert np.array_equal(part.reshape(3, 2, 8)[:, :, :4], D.rope(lead, 2, 4, 1e4, [5, 9, 200]).reshape(3, 2, 4))
    # every head turns by the same angles (the reference ropes q|k as one span for that reason, qwen3.rs:839-846)
    both = D.rope(np.concatenate([x, x], axis=1), 4, 8, 1e4, [5, 9, 200])
    assert np.array_equal(both[:, :16], y) and np.array_equal(both[:, 16:], y)


def brute_attention(q, k, v, nh, nkv):
    dh = q.size // nh
    s = k.shape[0]
    out = np.zeros(nh * dh)
    for h in range(nh):
        kvh = h // (nh // nkv)
        scale = float(np.float32(1.0) / np.sqrt(np.float32(dh)))      # the reference's f32 `1.0 / (dh as f32).sqrt()`
        sc = [sum(float(q[h * dh + d]) * float(k[j, kvh * dh + d]) for d in range(dh)) * scale for j in range(s)]
        mx = max(sc)
        e = [math.exp(x - mx) for x in sc]
        z = sum(e)
        for d in range(dh):
            out[h * dh + d] = sum(e[j] / z * float(v[j, kvh * dh + d]) for j in range(s))
    return out


def test_decode_attention_against_loops_and_special_cases():
    rng = np.random.default_rng(3)
    for nh, nkv, dh, s in [(4, 2, 8, 5), (6, 1, 4, 9), (3, 3, 16, 1), (8, 2, 8, 33)]:
        q = rng.standard_normal(nh * dh).astype(np.float32)
        k = rng.standard_normal((s, nkv * dh)).astype(np.float32)
        v = rng.standard_normal((s, nkv * dh)).astype(np.float32)
        assert np.allclose(D.decode_attention(q, k, v, nh, nkv)[0], brute_attention(q, k, v, nh, nkv), rtol=1e-9, atol=1e-12)
    nh, nkv, dh = 6, 2, 8
    q = rng.standard_normal(nh * dh).astype(np.float32)
    v = rng.standard_normal((7, nkv * dh)).astype(np.float32)
    one = D.decode_attention(q, v[:1], v[:1], nh, nkv).reshape(nh, dh)          # one key: the output is its value row,
    for h in range(nh):                                                          # of KV head h // 3
        assert np.array_equal(one[h], v[0, (h // 3) * dh:(h // 3 + 1) * dh].astype(np.float64))
    same = np.tile(rng.standard_normal((1, nkv * dh)).astype(np.float32), (7, 1))
    uni = D.decode_attention(q, same, v, nh, nkv).reshape(nh, dh)                # equal keys: the mean of the values
    assert np.allclose(uni[4], v[:, dh:2 * dh].astype(np.float64).mean(axis=0), rtol=1e-12)
    k = np.zeros((7, nkv * dh), np.float32); k[3, :dh] = q[:dh] * 50             # one key dominates head 0
    assert np.allclose(D.decode_attention(q, k, v, nh, nkv).reshape(nh, dh)[0], v[3, :dh], atol=1e-9)
    # the 1 / sqrt(dh): two keys with scores a, 0 -> weights sigmoid(a / sqrt(dh))
    q1 = np.zeros(dh, np.float32); q1[0] = 4.0
    k2 = np.zeros((2, dh), np.float32); k2[0, 0] = 1.0
    v2 = np.array([[1.0] * dh, [0.0] * dh], np.float32)
    assert np.allclose(D.decode_attention(q1, k2, v2, 1, 1), 1.0 / (1.0 + math.exp(-4.0 / math.sqrt(dh))), rtol=1e-7)


def test_window_and_softcap_in_the_attention_oracle():
    rng = np.random.default_rng(6)
    nh, nkv, dh, s = 4, 2, 8, 11
    q = rng.standard_normal(nh * dh).astype(np.float32)
    k = rng.standard_normal((s, nkv * dh)).astype(np.float32)
    v = rng.standard_normal((s, nkv * dh)).astype(np.float32)
    full = D.decode_attention(q, k, v, nh, nkv)
    assert np.array_equal(D.decode_attention(q, k, v, nh, nkv, window=0), full)
    assert np.array_equal(D.decode_attention(q, k, v, nh, nkv, window=s), full) and np.array_equal(D.decode_attention(q, k, v, nh, nkv, window=s + 5), full)
    # the last w keys only == attention over the truncated cache (nn.rs:92-111)
    for w in (1, 3, 10):
        assert np.allclose(D.decode_attention(q, k, v, nh, nkv, window=w), D.decode_attention(q, k[s - w:], v[s - w:], nh, nkv), rtol=1e-13)
    # softcap: cap * tanh(x / cap); a huge cap is the identity, a tiny one flattens the scores to +-cap
    assert np.allclose(D.decode_attention(q, k, v, nh, nkv, softcap=1e6), full, rtol=1e-9)
    flat = D.decode_attention(q * np.float32(1e4), k, v, nh, nkv, softcap=1e-3)     # every score is +-1e-3: nearly the mean
    assert np.allclose(flat.reshape(nh, dh)[0], v[:, :dh].astype(np.float64).mean(axis=0), atol=2e-3)
    q1 = np.zeros(dh, np.float32); q1[0] = 6.0
    k2 = np.zeros((2, dh), np.float32); k2[0, 0] = 1.0
    v2 = np.array([[1.0] * dh, [0.0] * dh], np.float32)
    x = 6.0 / math.sqrt(dh)
    assert np.allclose(D.decode_attention(q1, k2, v2, 1, 1, softcap=1.5), 1.0 / (1.0 + math.exp(-1.5 * math.tanh(x / 1.5))), rtol=1e-7)


def test_qkv_post_composes_bias_norm_and_rope():
    rng = np.random.default_rng(4)
    nh, nkv, hd = 4, 2, 8
    qkv = rng.standard_normal((2, (nh + 2 * nkv) * hd)).astype(np.float32)
    bias = rng.standard_normal((nh + 2 * nkv) * hd).astype(np.float32)
    qn, kn = rng.standard_normal(hd).astype(np.float32), rng.standard_normal(hd).astype(np.float32)
    q, k, v = D.qkv_post(qkv, bias, qn, kn, [3, 11], nh, nkv, hd, 1e-6, 1e6)
    xb = qkv + bias
    assert np.array_equal(v, xb[:, (nh + nkv) * hd:].astype(np.float64))
    want_q = D.rope(D.rmsnorm(xb[:, :nh * hd].reshape(2, nh, hd), qn, 1e-6).reshape(2, -1), nh, hd, 1e6, [3, 11])
    assert np.array_equal(q, want_q)
    q0, k0, _ = D.qkv_post(qkv, None, None, None, [3, 11], nh, nkv, hd, 1e-6, 1e6)       # no norms: rope of the raw span
    span = D.rope(qkv[:, :(nh + nkv) * hd], nh + nkv, hd, 1e6, [3, 11])
    assert np.array_equal(np.concatenate([q0, k0], axis=1), span)


def test_apply_layer_reduces_to_the_residual_when_the_output_projections_vanish():
    rng = np.random.default_rng(5)

    class Cfg:
        n_head, n_head_kv, head_dim, n_ff, eps, rope_base, rope_interleaved = 2, 1, 4, 6, 1e-6, 1e4, False
    d = 8
    l = D.Layer(attn_norm=np.ones(d), wqkv=rng.standard_normal((16, d)), wo=np.zeros((d, 8)), ffn_norm=np.ones(d),
                gate_up=rng.standard_normal((12, d)), down=np.zeros((d, 6)))
    x = rng.standard_normal(d)
    kc, vc = [], []
    assert np.array_equal(D.apply_layer(x, l, kc, vc, 0, Cfg), x) and len(kc) == 1 and kc[0].shape == (4,)
    l.wo = rng.standard_normal((d, 8)); l.down = rng.standard_normal((d, 6))
    y = D.apply_layer(x, l, kc, vc, 1, Cfg)
    # by hand: the same chain written out
    h = D.rmsnorm(x, l.attn_norm, 1e-6)
    q, k, v = D.qkv_post((h @ l.wqkv.T).reshape(1, -1), None, None, None, [1], 2, 1, 4, 1e-6, 1e4)
    a = D.decode_attention(q[0], np.stack([kc[0], k[0]]), np.stack([vc[0], v[0]]), 2, 1)
    xy = x + a[0] @ l.wo.T
    f = D.silu_mul(D.rmsnorm(xy, l.ffn_norm, 1e-6) @ l.gate_up.T, 6)
    assert np.allclose(y, xy + f @ l.down.T, rtol=1e-13)
