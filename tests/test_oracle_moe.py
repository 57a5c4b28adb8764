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
