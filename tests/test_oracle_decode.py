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


def test_sigmoid_and_gelu_tanh_against_library_routines():
    from scipy.special import expit
    import torch
    x = np.concatenate([np.linspace(-30, 30, 2001), [0.0, 1e-8, -1e-8, 88.0, -88.0]])
    assert np.allclose(D.sigmoid(x), expit(x), rtol=1e-14, atol=0)
    assert D.sigmoid(0.0) == 0.5 and np.allclose(D.sigmoid(x) + D.sigmoid(-x), 1.0, rtol=1e-15)
    g = torch.nn.functional.gelu(torch.from_numpy(x), approximate="tanh").numpy()      # f64 on the CPU
    inside = np.abs(0.7978845608028654 * (x + 0.044715 * x ** 3)) < 15                  # where the reference's clamp is idle
    # (1 + tanh(a) cancels for a << 0: an absolute 1e-14 on values of 1e-12)
    assert np.allclose(D.gelu_tanh(x)[inside], g[inside], rtol=1e-13, atol=1e-14)
    # beyond the clamp tanh(15) = 1 - 1.9e-13: the value is x (or 0) to that relative error, as the unclamped form's
    assert np.allclose(D.gelu_tanh(x)[~inside], g[~inside], rtol=1e-12, atol=1e-10)
    assert np.allclose(D.gelu_tanh(x) - D.gelu_tanh(-x), x, rtol=1e-13, atol=1e-15)    # odd part of x Phi(x) is x / 2 twice
    gu = np.array([[1.0, -2.0, 0.5, 3.0]])
    assert np.array_equal(D.gelu_mul(gu, 2), D.gelu_tanh(gu[:, :2]) * gu[:, 2:])


def _arm_layer(rng, d, nh, nkv, hd, n_ff):
    return D.Layer(attn_norm=rng.random(d) + 0.5, wqkv=rng.standard_normal(((nh + 2 * nkv) * hd, d)), wo=rng.standard_normal((d, nh * hd)),
                   ffn_norm=rng.random(d) + 0.5, gate_up=rng.standard_normal((2 * n_ff, d)), down=rng.standard_normal((d, n_ff)))


def test_the_other_arms_of_apply_layer_by_their_invariants():
    rng = np.random.default_rng(6)

    class Cfg:
        n_head, n_head_kv, head_dim, n_ff, eps, rope_base, rope_interleaved = 4, 2, 8, 12, 1e-6, 1e4, False
    d = 16
    l = _arm_layer(rng, d, 4, 2, 8, 12)
    xs = rng.standard_normal((4, d))

    def run(layer, cfg, positions=(0, 1, 2, 3)):
        kc, vc, out = [], [], []
        for x, pos in zip(xs, positions):
            out.append(D.apply_layer(x, layer, kc, vc, pos, cfg))
        return np.stack(out)
    base = run(l, Cfg)
    # gate: a zero gate projection is sigmoid(0) = 1/2 on every attention output, i.e. the output projection halved; a gate
    # saturated at +40 is the ungated layer
    lg = D.Layer(**l.__dict__); lg.attn_gate = np.zeros((32, d))
    lh = D.Layer(**l.__dict__); lh.wo = l.wo * 0.5
    assert np.allclose(run(lg, Cfg), run(lh, Cfg), rtol=1e-13)
    big = D.Layer(**l.__dict__); big.attn_norm = np.ones(d); big.attn_gate = np.ones((32, d)) * 1e3
    ref = D.Layer(**l.__dict__); ref.attn_norm = np.ones(d)
    xs_pos = np.abs(xs)                                          # a normed input of positive entries: every gate logit >> 40
    kc1, vc1, kc2, vc2 = [], [], [], []
    assert np.allclose(D.apply_layer(xs_pos[0], big, kc1, vc1, 0, Cfg), D.apply_layer(xs_pos[0], ref, kc2, vc2, 0, Cfg), rtol=1e-13)
    # window: at least the history is no window; a window of 1 attends to the newest key only, whose softmax weight is 1:
    # the attention output is the token's own value row, whatever the history
    lw = D.Layer(**l.__dict__); lw.window = 4
    assert np.array_equal(run(lw, Cfg), base)
    l1 = D.Layer(**l.__dict__); l1.window = 1
    w1 = run(l1, Cfg)
    assert np.allclose(w1[0], base[0], rtol=1e-13) and not np.allclose(w1[3], base[3], rtol=1e-3)
    kc, vc = [rng.standard_normal(16)] * 3, [rng.standard_normal(16)] * 3      # another history, same result under window 1
    assert np.allclose(D.apply_layer(xs[3], l1, kc, vc, 3, Cfg), w1[3], rtol=1e-13)
    # NoPE: no rotation, so the positions do not matter; a rotating layer agrees with it at position 0 only
    ln = D.Layer(**l.__dict__); ln.rope = False
    assert np.allclose(run(ln, Cfg), run(ln, Cfg, positions=(7, 3, 11, 2)), rtol=1e-13)
    assert np.allclose(run(ln, Cfg)[0], base[0], rtol=1e-13) and not np.allclose(run(ln, Cfg)[2], base[2], rtol=1e-3)
    # the layer's own rope base replaces the configuration's
    lb = D.Layer(**l.__dict__); lb.rope_base = 5e5

    class Cfg5(Cfg):
        rope_base = 5e5
    assert np.array_equal(run(lb, Cfg), run(l, Cfg5)) and not np.allclose(run(lb, Cfg)[3], base[3], rtol=1e-6)
    # softcap: a huge cap is the identity on the scores
    class CfgCap(Cfg):
        attn_softcap = 1e9
    assert np.allclose(run(l, CfgCap), base, rtol=1e-9)
    # post-norms: each branch output is normalised before the add, so (with a negligible epsilon) scaling an output projection
    # leaves the layer unchanged, and unit post-norm weights give the branch at RMS 1
    class CfgPost(Cfg):
        post_norm_eps = 1e-30
    lp = D.Layer(**l.__dict__); lp.post_attn_norm = rng.random(d) + 0.5; lp.post_ffn_norm = rng.random(d) + 0.5
    ls = D.Layer(**lp.__dict__); ls.wo = lp.wo * 7.0; ls.down = lp.down * 0.125
    assert np.allclose(run(lp, CfgPost), run(ls, CfgPost), rtol=1e-12) and not np.allclose(run(lp, CfgPost), base, rtol=1e-3)
    lu = D.Layer(**l.__dict__); lu.post_attn_norm = np.ones(d); lu.post_ffn_norm = np.ones(d); lu.down = np.zeros((d, 12))
    kc, vc = [], []
    y = D.apply_layer(xs[0], lu, kc, vc, 0, CfgPost)             # down = 0: the FFN branch is rmsnorm(0) = 0
    assert math.isclose(np.sqrt(np.mean((y - xs[0]) ** 2)), 1.0, rel_tol=1e-12)
    # the post-norm epsilon is the configuration's own: with a large one the branch shrinks
    class CfgPostBig(Cfg):
        post_norm_eps = 1e6
    kc, vc = [], []
    yb = D.apply_layer(xs[0], lu, kc, vc, 0, CfgPostBig)
    assert np.sqrt(np.mean((yb - xs[0]) ** 2)) < 0.1
    # GEGLU: the same chain with the gate through the library's tanh GELU
    import torch

    class CfgGe(Cfg):
        geglu = True
    kc, vc = [], []
    yg = D.apply_layer(xs[0], l, kc, vc, 0, CfgGe)
    kc2, vc2 = [], []
    h = D.rmsnorm(xs[0], l.attn_norm, 1e-6)
    q, k, v = D.qkv_post((h @ l.wqkv.T).reshape(1, -1), None, None, None, [0], 4, 2, 8, 1e-6, 1e4)
    xy = xs[0] + D.decode_attention(q[0], k, v, 4, 2)[0] @ l.wo.T
    gu = D.rmsnorm(xy, l.ffn_norm, 1e-6) @ l.gate_up.T
    act = torch.nn.functional.gelu(torch.from_numpy(gu[:12]), approximate="tanh").numpy() * gu[12:]
    assert np.allclose(yg, xy + act @ l.down.T, rtol=1e-12)


def test_causal_attention_against_the_masked_matrix_form():
    """The reference's own formulation (nn.rs:40-57, :66-88, :239-265): all scores at once, an additive mask of -1e30 where
    j > off + i or (off + i) - j >= window, softmax over the keys, times V -- against the row-by-row oracle."""
    rng = np.random.default_rng(12)
    for t, s, nh, nkv, dh, window, cap in [(5, 5, 4, 2, 8, 0, 0.0), (7, 19, 6, 2, 4, 0, 0.0), (9, 9, 2, 2, 8, 3, 0.0), (6, 14, 4, 1, 8, 5, 20.0),
                                           (1, 11, 4, 2, 8, 0, 0.0)]:
        q, k, v = rng.standard_normal((t, nh * dh)), rng.standard_normal((s, nkv * dh)), rng.standard_normal((s, nkv * dh))
        got = D.causal_attention(q, k, v, nh, nkv, window, cap)
        off, g = s - t, nh // nkv
        qh = q.reshape(t, nh, dh).transpose(1, 0, 2)
        kh = np.repeat(k.reshape(s, nkv, dh).transpose(1, 0, 2), g, axis=0)
        vh = np.repeat(v.reshape(s, nkv, dh).transpose(1, 0, 2), g, axis=0)
        sc = qh @ kh.transpose(0, 2, 1) * float(np.float32(1.0) / np.sqrt(np.float32(dh)))
        if cap > 0:
            sc = cap * np.tanh(sc / cap)
        ii, jj = np.arange(t)[:, None] + off, np.arange(s)[None, :]
        mask = np.where((jj > ii) | ((window > 0) & (ii - jj >= window)), -1e30, 0.0)
        sc = sc + mask
        p = np.exp(sc - sc.max(axis=2, keepdims=True))
        want = ((p / p.sum(axis=2, keepdims=True)) @ vh).transpose(1, 0, 2).reshape(t, nh * dh)
        assert np.allclose(got, want, rtol=1e-12, atol=1e-14), (t, s)
    # one query row against the whole cache is the decode op; the first row of a stateless prefill returns its own value row
    q, k, v = rng.standard_normal((1, 32)), rng.standard_normal((6, 16)), rng.standard_normal((6, 16))
    assert np.array_equal(D.causal_attention(q, k, v, 4, 2), D.decode_attention(q[0], k, v, 4, 2))
    q = rng.standard_normal((6, 32))
    assert np.allclose(D.causal_attention(q, k, v, 4, 2)[0].reshape(4, 8), np.repeat(v[0].reshape(2, 8), 2, axis=0), rtol=1e-14)
