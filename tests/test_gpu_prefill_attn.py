"""fhip_causal_attention (prefill / chunked prefill / windowed / softcapped causal attention on the f32 matrix instructions)
through the C ABI against the f64 oracle. Floating point: the bar is 1e-5 of the largest expected output, the bar of the
single-query attention tests; a row that sees one key only must return that key's value row exactly."""
import numpy as np
import pytest

from conftest import bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def D():
    from oracle import decode_oracle
    return decode_oracle


@pytest.fixture(scope="module")
def X(F):
    from ferric_amd import decode
    return decode


def run(F, X, D, t, s, nh, nkv, hd, window=0, cap=0.0, seed=0, scale=1.0):
    rng = np.random.default_rng(seed)
    q = (rng.standard_normal((t, nh * hd)) * scale).astype(np.float32)
    k = rng.standard_normal((s, nkv * hd)).astype(np.float32)
    v = rng.standard_t(3, (s, nkv * hd)).astype(np.float32)
    T = lambda a: F.Tensor.from_vec(a, a.shape)
    got = X.causal_attention(T(q), T(k), T(v), nh, nkv, window, cap).to_vec().reshape(t, nh * hd)
    want = D.causal_attention(q, k, v, nh, nkv, window, cap)
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err <= 1e-5, (t, s, nh, nkv, hd, window, cap, err)
    return got, q, k, v


def test_shapes_groups_and_ragged_ends(F, X, D):
    # stateless prefill (s == t): one row, less than a tile, exactly one, ragged, several query blocks; both head sizes;
    # group sizes 1, 2, 5, 8; then t rows against a longer cache (chunked prefill / a prefix-cached suffix), off inside a tile
    for i, (t, s, nh, nkv, hd) in enumerate([(1, 1, 4, 2, 64), (7, 7, 4, 4, 128), (32, 32, 8, 4, 64), (33, 33, 10, 2, 128), (100, 100, 8, 1, 64),
                                             (130, 130, 5, 1, 128), (257, 257, 16, 2, 128), (300, 300, 6, 3, 64),
                                             (1, 40, 8, 2, 128), (5, 70, 8, 2, 64), (64, 200, 10, 2, 128), (90, 91, 4, 2, 128), (31, 160, 8, 8, 64)]):
        got, q, k, v = run(F, X, D, t, s, nh, nkv, hd, seed=i)
        if s == t:          # the first row sees its own key only
            g = nh // nkv
            assert np.array_equal(bits(got[0].reshape(nh, hd)), bits(np.repeat(v[0].reshape(nkv, hd), g, axis=0)))


def test_window_and_softcap(F, X, D):
    for i, (t, s, nh, nkv, hd, w, cap) in enumerate([(70, 70, 4, 2, 64, 16, 0.0), (70, 70, 4, 2, 128, 1, 0.0), (150, 150, 8, 2, 128, 33, 0.0),
                                                     (40, 300, 8, 2, 64, 100, 0.0), (150, 150, 8, 2, 128, 0, 30.0), (96, 130, 5, 1, 128, 40, 50.0),
                                                     (50, 50, 4, 2, 64, 1000, 0.0)]):
        got, q, k, v = run(F, X, D, t, s, nh, nkv, hd, w, cap, seed=20 + i, scale=3.0)
        if w == 1:          # a window of one key: every row returns its own value row
            g = nh // nkv
            assert np.array_equal(bits(got.reshape(t, nh, hd)), bits(np.repeat(v[s - t:].reshape(t, nkv, hd), g, axis=1)))


def test_a_prefill_sized_block_on_sampled_rows(F, X, D):
    """2048 tokens of the 40 / 8-head x 128 model in one launch; the oracle on a sample of rows (first, tile edges, last)."""
    t, nh, nkv, hd = 2048, 40, 8, 128
    rng = np.random.default_rng(5)
    q = rng.standard_normal((t, nh * hd)).astype(np.float32)
    k = rng.standard_normal((t, nkv * hd)).astype(np.float32)
    v = rng.standard_normal((t, nkv * hd)).astype(np.float32)
    T = lambda a: F.Tensor.from_vec(a, a.shape)
    qt, kt, vt = T(q), T(k), T(v)
    got = X.causal_attention(qt, kt, vt, nh, nkv).to_vec().reshape(t, nh * hd)
    for r in (0, 1, 31, 32, 127, 128, 1000, 1023, 1024, 2047):
        want = D.decode_attention(q[r], k[:r + 1], v[:r + 1], nh, nkv)[0]
        assert np.abs(got[r] - want).max() <= 1e-5 * np.abs(want).max(), r
    again = X.causal_attention(qt, kt, vt, nh, nkv).to_vec().reshape(t, nh * hd)
    assert np.array_equal(bits(got), bits(again))                 # no atomics, a fixed order: the same bits every run
    # a row of the block equals the single-query op on the same cache prefix to the two kernels' rounding
    r = 777
    cache = type("C", (), {})()
    cache.k, cache.v, cache.cap, cache.width, cache.len = kt, vt, t, nkv * hd, r + 1
    one = X.decode_attention(T(q[r:r + 1]), cache, nh, nkv, length=r + 1).to_vec()
    assert np.abs(one - got[r]).max() <= 2e-6 * np.abs(got[r]).max()


def test_argument_checks(F, X):
    lib = F._lib.load()
    a = F.Tensor.from_vec(np.zeros((4, 256), np.float32), (4, 256))
    assert lib.fhip_causal_attention(a.buf.ptr, a.buf.ptr, a.buf.ptr, 4, 3, 4, 4, 64, 0, 0.0, a.buf.ptr, None) != 0
    assert b"cannot be shorter than the query block" in lib.fhip_last_error()          # nn.rs:73
    assert lib.fhip_causal_attention(a.buf.ptr, a.buf.ptr, a.buf.ptr, 4, 4, 4, 3, 64, 0, 0.0, a.buf.ptr, None) != 0
    assert lib.fhip_causal_attention(a.buf.ptr, a.buf.ptr, a.buf.ptr, 4, 4, 8, 8, 32, 0, 0.0, a.buf.ptr, None) != 0
    assert b"head_dim must be 64 or 128" in lib.fhip_last_error()
    assert lib.fhip_causal_attention(None, a.buf.ptr, a.buf.ptr, 4, 4, 4, 4, 64, 0, 0.0, a.buf.ptr, None) != 0
    assert lib.fhip_causal_attention(None, None, None, 0, 0, 4, 4, 64, 0, 0.0, None, None) == 0       # nothing to do
