"""Mixture-of-experts decode ops through the C ABI: router top-k and the selected-expert ("_id") matmuls.

Bars: top-k indices exactly the oracle's, weights to 1e-5 relative (device exp vs numpy exp); the matmuls
against f64 on oracle-dequantized weights to the north-star bound 1e-3 * ||w_row|| * ||x|| per dot (and 1e-5 of
the largest output), and bit for bit against the plain matmul entry points run on the selected expert's slice
of the slab -- the "_id" kernels are the same kernels behind an indexed row base."""
import numpy as np
import pytest

from conftest import dot_bar

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("precision")]
Q8_0, Q4_K, Q6_K = 8, 12, 14
BLOCK = {Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210)}


def slab(F, ty, n_expert, rows_pe, cols, seed):
    from ferric_amd.synth import synth_weights
    raw = synth_weights(ty, n_expert * rows_pe, cols, seed)
    return raw, F.QMatrix.from_bytes(raw, ty, n_expert * rows_pe, cols)


def expert_slice(F, raw, ty, e, rows_pe, cols):
    rb = cols // BLOCK[ty][0] * BLOCK[ty][1]
    return F.QMatrix.from_bytes(raw[e * rows_pe * rb:(e + 1) * rows_pe * rb], ty, rows_pe, cols)


def selection(rng, t, k, n_expert):
    sel = np.zeros((t, 2 * k), np.float32)
    for ti in range(t):
        sel[ti, :k] = rng.random(k).astype(np.float32) + 0.1
        sel[ti, k:] = rng.choice(n_expert, size=k, replace=False)
    return sel


@pytest.mark.parametrize("sigmoid", [False, True])
def test_moe_topk_matches_oracle(F, O, sigmoid):
    rng = np.random.default_rng(11)
    for t, ne, k, has_bias, norm in [(1, 8, 1, False, True), (3, 8, 8, True, True), (5, 60, 4, True, False), (2, 128, 8, False, True),
                                     (4, 257, 6, True, True), (8, 1024, 8, True, False), (1, 1, 1, False, True)]:
        logits = (rng.standard_normal((t, ne)) * 3).astype(np.float32)
        bias = (rng.standard_normal(ne) * 0.3).astype(np.float32) if has_bias else None
        want = O.moe_topk(logits, bias, k, sigmoid, 2.5, norm)
        bt = F.Tensor.from_vec(bias, (ne,)) if has_bias else None
        got = F.Tensor.from_vec(logits.reshape(-1), (t, ne)).moe_topk_ex(bt, k, sigmoid, 2.5, norm).to_vec().reshape(t, 2 * k)
        assert np.array_equal(got[:, k:], want[:, k:]), (t, ne, k)
        assert np.allclose(got[:, :k], want[:, :k], rtol=1e-5, atol=0), (t, ne, k)


def test_moe_topk_ties_bias_and_default_norm(F, O):
    z = F.Tensor.from_vec(np.zeros(6, np.float32), (1, 6)).moe_topk(None, 3, False, 3.0).to_vec()
    assert list(z[3:]) == [0.0, 1.0, 2.0] and np.allclose(z[:3], 1.0)
    logits = np.array([[0.0, 1.0, 2.0, 3.0]], np.float32)
    bias = F.Tensor.from_vec(np.array([10.0, 0, 0, 0], np.float32), (4,))
    out = F.Tensor.from_vec(logits.reshape(-1), (1, 4)).moe_topk_ex(bias, 2, False, 1.0, False).to_vec()
    assert list(out[2:]) == [0.0, 3.0]
    p = np.exp(logits[0] - 3) / np.exp(logits[0] - 3).sum()
    assert np.allclose(out[:2], [p[0], p[3]], rtol=1e-5)
    with pytest.raises(AssertionError, match="k must be"):
        F.Tensor.from_vec(np.zeros(16, np.float32), (1, 16)).moe_topk(None, 9, False, 1.0)
    with pytest.raises(AssertionError, match="n_expert"):
        F.Tensor.from_vec(np.zeros(1025, np.float32), (1, 1025)).moe_topk(None, 2, False, 1.0)


# (format, method, in, eff): in = 2048 runs the streaming kernel, 768 / 1280 the shape-complete one
@pytest.mark.parametrize("ty,name,cols,eff", [(Q4_K, "matmul_q4_k_swiglu_id", 2048, 96), (Q4_K, "matmul_q4_k_swiglu_id", 768, 40),
                                               (Q8_0, "matmul_q8_0_swiglu_id", 1024, 64), (Q8_0, "matmul_q8_0_swiglu_id", 160, 24)])
def test_swiglu_id(F, O, ty, name, cols, eff):
    rng = np.random.default_rng(21)
    n_expert, t, k = 6, 3, 4
    raw, w = slab(F, ty, n_expert, 2 * eff, cols, 5)
    x = rng.standard_normal((t, cols)).astype(np.float32)
    sel = selection(rng, t, k, n_expert)
    st = F.Tensor.from_vec(sel.reshape(-1), (t, 2 * k))
    got = getattr(F.Tensor.from_vec(x.reshape(-1), (t, cols)), name)(w, st, k, eff).to_vec().reshape(t, k, eff)
    want = O.matmul_swiglu_id_f64(x, raw, ty, sel, k, eff, cols)
    assert np.abs(got - want).max() <= dot_bar() * np.abs(want).max()
    if ty != Q8_0:   # the plain fused entry point exists for the K-quants only (try_matmul_swiglu is None for Q8_0)
        for ti in range(t):
            for s in range(k):
                one = F.Tensor.from_vec(x[ti], (1, cols)).try_matmul_swiglu(expert_slice(F, raw, ty, int(sel[ti, k + s]), 2 * eff, cols))
                assert np.array_equal(one.to_vec().view(np.uint32), got[ti, s].view(np.uint32)), (ti, s)


# the squared-ReLU expert MLP's up projection (dtype.rs:1703-1729): Q5_0 as in the reference, streaming (cols a multiple of
# 512) and shape-complete kernels, and two other formats through the type-generic entry point
@pytest.mark.parametrize("ty,cols,eff", [(6, 1024, 72), (6, 160, 24), (6, 2688, 58), (Q4_K, 2048, 40), (Q8_0, 512, 33)])
def test_relu2_id(F, O, ty, cols, eff):
    from ferric_amd.synth import synth_weights
    rng = np.random.default_rng(25)
    n_expert, t, k = 6, 3, 4
    raw = synth_weights(ty, n_expert * eff, cols, 9)
    w = F.QMatrix.from_bytes(raw, ty, n_expert * eff, cols)
    x = rng.standard_normal((t, cols)).astype(np.float32)
    sel = selection(rng, t, k, n_expert)
    st = F.Tensor.from_vec(sel.reshape(-1), (t, 2 * k))
    xt = F.Tensor.from_vec(x.reshape(-1), (t, cols))
    got = (xt.matmul_q5_0_relu2_id(w, st, k, eff) if ty == 6 else xt.matmul_q_relu2_id(w, st, k, eff)).to_vec().reshape(t, k, eff)
    want, acc, wn = O.matmul_relu2_id_f64(x, raw, ty, sel, k, eff, cols)
    # the dot to the north-star bound, carried through v -> max(v, 0)^2 (slope 2|v|), and to the bar of the scalar kernels
    bound = 1e-3 * wn * np.linalg.norm(x.astype(np.float64), axis=1)[:, None, None]
    assert (np.abs(got - want) <= 2 * np.abs(acc) * bound + bound ** 2 + 1e-30).all()
    assert np.abs(got - want).max() <= 3 * dot_bar() * np.abs(want).max()
    assert (got >= 0).all() and (got[acc < -1e-3 * np.abs(acc).max()] == 0).all()
    rb = raw.size // (n_expert * eff)
    for ti in range(t):          # the plain mat-vec on the selected expert's slice, then the activation: the same bits
        for s in range(k):
            e = int(sel[ti, k + s])
            one = F.Tensor.from_vec(x[ti], (1, cols)).matmul_q(F.QMatrix.from_bytes(raw[e * eff * rb:(e + 1) * eff * rb], ty, eff, cols)).to_vec()
            a = np.maximum(one, np.float32(0))
            assert np.array_equal((a * a).view(np.uint32), got[ti, s].view(np.uint32)), (ti, s)
    with pytest.raises(AssertionError, match="k must be"):
        xt.matmul_q_relu2_id(w, st, 9, eff)


def test_matmul_q6_k_id(F, O):
    rng = np.random.default_rng(22)
    for cols, out_pe in [(1024, 72), (768, 130)]:
        n_expert, k = 5, 4
        raw, w = slab(F, Q6_K, n_expert, out_pe, cols, 6)
        x = rng.standard_normal((k, cols)).astype(np.float32)
        sel = selection(rng, 1, k, n_expert)
        got = F.Tensor.from_vec(x.reshape(-1), (k, cols)).matmul_q6_k_id(w, F.Tensor.from_vec(sel.reshape(-1), (2 * k,)), out_pe)
        got = got.to_vec().reshape(k, out_pe)
        want, wn = O.matmul_id_f64(x, raw, Q6_K, sel, k, out_pe, cols)
        assert (np.abs(got - want) <= 1e-3 * wn * np.linalg.norm(x.astype(np.float64), axis=1)[:, None]).all()
        assert np.abs(got - want).max() <= dot_bar() * np.abs(want).max()
        for s in range(k):
            one = F.Tensor.from_vec(x[s], (1, cols)).matmul_q(expert_slice(F, raw, Q6_K, int(sel[0, k + s]), out_pe, cols))
            assert np.array_equal(one.to_vec().view(np.uint32), got[s].view(np.uint32))


@pytest.mark.parametrize("ty,name,cols", [(Q6_K, "matmul_q6_k_id_wsum", 1024), (Q6_K, "matmul_q6_k_id_wsum", 768),
                                          (Q4_K, "matmul_q4_k_id_wsum", 2048), (Q4_K, "matmul_q4_k_id_wsum", 256),
                                          (Q8_0, "matmul_q8_0_id_wsum", 512), (Q8_0, "matmul_q8_0_id_wsum", 96)])
def test_id_wsum(F, O, ty, name, cols):
    rng = np.random.default_rng(23)
    n_expert, t, k, out_pe = 7, 3, 5, 136
    raw, w = slab(F, ty, n_expert, out_pe, cols, 7)
    x = rng.standard_normal((t, k, cols)).astype(np.float32)
    sel = selection(rng, t, k, n_expert)
    st = F.Tensor.from_vec(sel.reshape(-1), (t, 2 * k))
    got = getattr(F.Tensor.from_vec(x.reshape(-1), (t, k, cols)), name)(w, st, out_pe).to_vec().reshape(t, out_pe)
    want, bound = O.matmul_id_wsum_f64(x, raw, ty, sel, k, out_pe, cols)
    assert (np.abs(got - want) <= 1e-3 * bound).all()
    assert np.abs(got - want).max() <= dot_bar() * np.abs(want).max()
    # T = 1 given as a 2-D [k, in] tensor (dtype.rs:1664)
    one = getattr(F.Tensor.from_vec(x[1].reshape(-1), (k, cols)), name)(w, F.Tensor.from_vec(sel[1], (1, 2 * k)), out_pe).to_vec()
    assert np.array_equal(one.view(np.uint32), got[1].view(np.uint32))


def test_indices_outside_the_slab_are_clamped_and_shapes_are_checked(F, O):
    rng = np.random.default_rng(24)
    cols, out_pe, n_expert, k = 256, 32, 3, 2
    raw, w = slab(F, Q4_K, n_expert, out_pe, cols, 8)
    x = rng.standard_normal((k, cols)).astype(np.float32)
    xt = F.Tensor.from_vec(x.reshape(-1), (k, cols))
    wild = np.array([[0.5, 0.5, 1e9, -7.0]], np.float32)       # read as expert 2 (the last) and expert 0
    tame = np.array([[0.5, 0.5, 2.0, 0.0]], np.float32)
    a = xt.matmul_q4_k_id_wsum(w, F.Tensor.from_vec(wild.reshape(-1), (1, 4)), out_pe).to_vec()
    b = xt.matmul_q4_k_id_wsum(w, F.Tensor.from_vec(tame.reshape(-1), (1, 4)), out_pe).to_vec()
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    st = F.Tensor.from_vec(tame.reshape(-1), (1, 4))
    with pytest.raises(AssertionError, match="inner dim mismatch"):
        F.Tensor.from_vec(np.zeros(2 * 512, np.float32), (2, 512)).matmul_q4_k_id_wsum(w, st, out_pe)
    with pytest.raises(AssertionError, match="whole number of experts"):
        xt.matmul_q4_k_id_wsum(w, st, 36)
    with pytest.raises(AssertionError, match="k must be"):
        F.Tensor.from_vec(np.zeros(9 * cols, np.float32), (9, cols)).matmul_q4_k_id_wsum(w, st, out_pe)
