"""Pins the numpy restatement of the reference's router top-k (oracle.moe_topk) against what the mathematics
fixes: the reference tree holds no vectors for it (crates/ferric-tensor/src/dtype.rs:2415-2461 is only ever
run on a GPU there), so each check below is chosen to fail for one plausible mistake."""
import numpy as np
import pytest


def brute(logits, bias, k, sigmoid, scale, norm):
    """Independent formulation: scores in f64, one stable argsort (ties -> lower index), no scan."""
    l = np.asarray(logits, np.float64)
    sc = 1 / (1 + np.exp(-l)) if sigmoid else np.exp(l - l.max()) / np.exp(l - l.max()).sum()
    key = sc + (0 if bias is None else np.asarray(bias, np.float64))
    idx = np.argsort(-key, kind="stable")[:k]
    w = sc[idx]
    return w / (w.sum() if norm else 1.0) * scale, idx


@pytest.mark.parametrize("sigmoid", [False, True])
@pytest.mark.parametrize("norm", [False, True])
def test_matches_sort_based_formulation(O, sigmoid, norm):
    rng = np.random.default_rng(3)
    for ne, k, has_bias in [(8, 1, False), (8, 8, True), (60, 4, True), (128, 8, False), (257, 6, True), (1024, 8, True)]:
        logits = (rng.standard_normal((3, ne)) * 3).astype(np.float32)
        bias = (rng.standard_normal(ne) * 0.3).astype(np.float32) if has_bias else None
        got = O.moe_topk(logits, bias, k, sigmoid, 2.5, norm)
        for ti in range(3):
            w, idx = brute(logits[ti], bias, k, sigmoid, 2.5, norm)
            assert np.array_equal(got[ti, k:], idx.astype(np.float32))
            assert np.allclose(got[ti, :k], w, rtol=2e-6, atol=0)


def test_invariants(O):
    rng = np.random.default_rng(4)
    logits = rng.standard_normal((5, 64)).astype(np.float32)
    out = O.moe_topk(logits, None, 8, False, 1.0, True)
    assert np.allclose(out[:, :8].sum(axis=1), 1.0, atol=1e-6)            # renormalised weights sum to scale
    assert all(len(set(r)) == 8 for r in out[:, 8:])                      # an expert is picked once
    assert (np.diff(out[:, :8], axis=1) <= 0).all()                       # without bias, picked in descending score
    raw = O.moe_topk(logits, None, 8, False, 1.0, False)
    assert (raw[:, :8].sum(axis=1) < 1.0).all()                           # raw top-k softmax mass is below 1
    assert np.allclose(raw[:, :8] / raw[:, :8].sum(axis=1, keepdims=True), out[:, :8], rtol=1e-6)
    # k = n_expert with softmax: every expert, and the raw weights are the whole distribution
    full = O.moe_topk(logits[:1, :8], None, 8, False, 1.0, False)
    assert sorted(full[0, 8:]) == list(range(8)) and abs(full[0, :8].sum() - 1) < 1e-6
    # softmax is shift invariant, sigmoid weights are not renormalised across experts
    assert np.array_equal(O.moe_topk(logits + 7.0, None, 4, False, 1.0, True)[:, 4:], O.moe_topk(logits, None, 4, False, 1.0, True)[:, 4:])
    sg = O.moe_topk(logits, None, 2, True, 1.0, False)
    assert np.allclose(sg[:, :2], np.sort(1 / (1 + np.exp(-logits.astype(np.float64))), axis=1)[:, ::-1][:, :2], rtol=1e-6)


def test_bias_steers_selection_but_never_enters_the_weights(O):
    logits = np.array([[0.0, 1.0, 2.0, 3.0]], np.float32)
    bias = np.array([10.0, 0.0, 0.0, 0.0], np.float32)
    out = O.moe_topk(logits, bias, 2, False, 1.0, False)
    assert list(out[0, 2:]) == [0.0, 3.0]                                 # expert 0 wins on bias, then the best score
    p = np.exp(logits[0] - 3) / np.exp(logits[0] - 3).sum()
    assert np.allclose(out[0, :2], [p[0], p[3]], rtol=1e-6)               # weights are the unbiased scores


def test_ties_go_to_the_lowest_index_and_scale_is_applied_last(O):
    out = O.moe_topk(np.zeros((1, 6), np.float32), None, 3, False, 3.0, True)
    assert list(out[0, 3:]) == [0.0, 1.0, 2.0]
    assert np.allclose(out[0, :3], 1.0)                                   # (1/6) / (3/6) * 3
    out = O.moe_topk(np.array([[1, 5, 5, 2]], np.float32), None, 2, True, 1.0, True)
    assert list(out[0, 2:]) == [1.0, 2.0]


def test_asserts(O):
    with pytest.raises(AssertionError, match="k must be"):
        O.moe_topk(np.zeros((1, 16), np.float32), None, 9, False, 1.0)
    with pytest.raises(AssertionError, match="n_expert"):
        O.moe_topk(np.zeros((1, 1025), np.float32), None, 2, False, 1.0)


def test_relu2_id_against_the_reference_kernel_s_element_formulation(O):
    # oracle.matmul_relu2_id_f64 (dequantize the slab, dot, max(v, 0)^2) against the kernel's own arithmetic restated word by
    # word (crates/ferric-tensor/src/dtype.rs:3735-3756: nibble | fifth bit from qh, minus 16, times d; expert ids from the
    # second half of the moe_topk row), and against what one-hot activations fix: out = max(c * w, 0)^2, 0 for a negative dot.
    from ferric_amd.synth import synth_weights
    Q5_0 = 6
    n_expert, eff, cols, t, k = 5, 7, 96, 3, 2
    raw = synth_weights(Q5_0, n_expert * eff, cols, 31)
    rng = np.random.default_rng(32)
    x = rng.standard_normal((t, cols)).astype(np.float32)
    sel = np.zeros((t, 2 * k), np.float32)
    for ti in range(t):
        sel[ti, :k] = rng.random(k)
        sel[ti, k:] = rng.choice(n_expert, size=k, replace=False)
    got, acc, wn = O.matmul_relu2_id_f64(x, raw, Q5_0, sel, k, eff, cols)
    blocks = raw.reshape(n_expert * eff, cols // 32, 22)
    for ti in range(t):
        for s in range(k):
            e = int(sel[ti, k + s])
            for o in range(eff):
                a = 0.0
                for b in range(cols // 32):
                    blk = blocks[e * eff + o, b]
                    d = float(blk[0:2].view(np.float16)[0])
                    qh = int(blk[2:6].view(np.uint32)[0])
                    for j in range(16):
                        lo = ((int(blk[6 + j]) & 15) | (((qh >> j) & 1) << 4)) - 16
                        hi = ((int(blk[6 + j]) >> 4) | (((qh >> (j + 16)) & 1) << 4)) - 16
                        a += (float(x[ti, 32 * b + j]) * lo + float(x[ti, 32 * b + 16 + j]) * hi) * d
                assert abs(a - acc[ti, s, o]) <= 1e-9 * (1 + abs(a))
                assert abs(max(a, 0.0) ** 2 - got[ti, s, o]) <= 1e-9 * (1 + a * a)
    assert (got >= 0).all() and (got[acc < 0] == 0).all() and (acc < 0).any() and (acc > 0).any()
    wd = O.deq_raw(raw, n_expert * eff * cols, Q5_0).reshape(n_expert * eff, cols)
    hot = np.zeros((1, cols), np.float32)
    hot[0, 37] = 3.0
    one = np.array([[1.0, 4.0]], np.float32)                              # k = 1: weight, expert 4
    g1, _, _ = O.matmul_relu2_id_f64(hot, raw, Q5_0, one, 1, eff, cols)
    assert np.allclose(g1[0, 0], np.maximum(3.0 * wd[4 * eff:5 * eff, 37].astype(np.float64), 0) ** 2, rtol=1e-12)
