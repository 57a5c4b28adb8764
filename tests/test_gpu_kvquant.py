"""The block-quantized KV cache through the C ABI against the oracle (oracle/kvquant_oracle.py): codes, scale bits and
dequantized values are integer / single-rounding work and must be bit-identical. Mirrors the reference's own tests of this
module (crates/ferric-tensor/src/kvquant.rs:1620-2130)."""
import ctypes as C

import numpy as np
import pytest

from conftest import bits
from test_oracle_kvquant import exact_case

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from oracle import kvquant_oracle
    return kvquant_oracle


@pytest.fixture(scope="module")
def Q(F):
    from ferric_amd import kvquant
    return kvquant


def packed(Q, K, cache):
    """(codes [nblk, words], scale halves) of the live rows, in the oracle's shapes."""
    c, s = cache.to_host()
    nblk = cache.len * cache.nblk_per_row()
    h = s.view(np.uint16)
    return c.reshape(nblk, K.CODE_WORDS[cache.fmt]), (h.reshape(nblk, 2) if cache.fmt == K.Q4_1 else h[:nblk])


def same_as_oracle(Q, K, cache, x):
    want = K.quantize(x, x.shape[0], x.shape[1], cache.fmt)
    c, s = packed(Q, K, cache)
    assert np.array_equal(c, want.codes), "codes"
    assert np.array_equal(s, want.scales), "scales"
    got = cache.dequantize().to_vec().reshape(x.shape)
    assert np.array_equal(bits(got), bits(want.dequantize_rows(0, x.shape[0]))), "dequantized values"


@pytest.mark.parametrize("fmt", [0, 1, 2])
def test_codes_fixed_by_construction_and_ties(F, Q, K, fmt):
    # kvquant.rs:1620 gpu_quantize_matches_the_exact_codes; :1559 ties away from zero
    x, want = exact_case(7, 96, fmt, 7)
    cache = Q.QKvCache.from_tensor(F.Tensor.from_vec(x, x.shape), fmt)
    ref = K.Cache(fmt, 7, 96)
    ref.codes, ref.scales = packed(Q, K, cache)
    for b in range(21):
        assert np.array_equal(K.codes_of(ref, b), want[b]), b
    assert np.array_equal(cache.dequantize().to_vec().reshape(7, 96), x)          # exactly representable data comes back exactly
    if fmt == K.Q8_0:
        t = np.zeros((1, 32), np.float32)
        t[0, 0] = 127.0
        t[0, 1:7] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5]
        cache = Q.QKvCache.from_tensor(F.Tensor.from_vec(t, t.shape), fmt)
        ref = K.Cache(fmt, 1, 32)
        ref.codes, ref.scales = packed(Q, K, cache)
        assert list(K.codes_of(ref, 0)[1:7]) == [1, 2, 3, -1, -2, -3]


@pytest.mark.parametrize("fmt", [0, 1, 2])
def test_heavy_tailed_and_special_values_bit_for_bit(F, Q, K, fmt):
    # kvquant.rs:1821 gpu_quantize_matches_the_cpu_reference_on_heavy_tailed_data, :1689 dequantize bit for bit
    rng = np.random.default_rng(40 + fmt)
    rows, width = 53, 160                                    # five blocks a row: scale pairs straddle rows
    x = (rng.standard_t(2, (rows, width)) * 10.0 ** rng.integers(-4, 4, (rows, 1))).astype(np.float32)
    x[3, 32:64] = 0.0                                        # d = 0
    x[4, 0:32] = -0.0
    x[5, 64:96] = 2.5                                        # a constant block (Q4_1: d = 0, min = 2.5)
    x[6, 7] = x[6, 20] = -np.abs(x[6, :32]).max() * 2        # equal extremes: the first wins
    x[7, 0:32] *= 1e-7                                       # scales in f16's subnormal range
    x[8, 0:32] *= 1e-10                                      # ... and below it: the scale rounds to zero
    x[9, 96:128] *= 1e7                                      # a scale beyond f16: infinity
    x[10, 3] = np.nan
    x[11, 40] = np.inf
    x[12, 70] = -np.inf
    x[13, 128:160] = np.nan
    x[14, 0:32] = np.float32(1e-42)                          # f32 subnormals
    cache = Q.QKvCache.from_tensor(F.Tensor.from_vec(x, x.shape), fmt)
    with np.errstate(all="ignore"):
        same_as_oracle(Q, K, cache, x)
    assert cache.len == rows and cache.width == width and cache.cap == 64


@pytest.mark.parametrize("fmt", [0, 1, 2])
def test_appends_growth_windows_and_copies(F, Q, K, fmt):
    rng = np.random.default_rng(50 + fmt)
    rows, width = 150, 96
    x = (rng.standard_normal((rows, width)) * 3).astype(np.float32)
    one_shot = Q.QKvCache.from_tensor(F.Tensor.from_vec(x, x.shape), fmt)
    same_as_oracle(Q, K, one_shot, x)
    # one row at a time (kvquant.rs:1908), through two doublings of the capacity (:2052): every earlier row survives
    grown = Q.QKvCache(fmt)
    for r in range(rows):
        grown.append(F.Tensor.from_vec(x[r:r + 1], (1, width)))
    assert grown.cap == 256 and grown.len == rows
    same_as_oracle(Q, K, grown, x)
    # rows in uneven batches, read as a window of wider rows (the key span of a fused qkv row, :2083)
    wide = rng.standard_normal((rows, 40 + width + 24)).astype(np.float32)
    wide[:, 40:40 + width] = x
    wt = F.Tensor.from_vec(wide, wide.shape)
    win = Q.QKvCache(fmt)
    at = 0
    for n in (1, 2, 60, 3, 84):
        part = F.Tensor.from_vec(wide[at:at + n], (n, wide.shape[1]))
        win.append(part, cols=(40, width))
        at += n
    same_as_oracle(Q, K, win, x)
    assert np.array_equal(bits(one_shot.dequantize_rows(17, 9).to_vec()), bits(K.quantize(x, rows, width, fmt).dequantize_rows(17, 9).reshape(-1)))
    # clone_prefix (:1861) and deep_clone (:2008): exactly those rows, and no shared memory
    pre = one_shot.clone_prefix(70)
    assert pre.len == 70 and pre.cap == 70 and pre.width == width
    same_as_oracle(Q, K, pre, x[:70])
    twin = one_shot.deep_clone()
    extra = (rng.standard_normal((5, width)) * 9).astype(np.float32)
    pre.append(F.Tensor.from_vec(extra, extra.shape))
    twin.append(F.Tensor.from_vec(-extra, extra.shape))
    same_as_oracle(Q, K, one_shot, x)                                      # untouched by either
    same_as_oracle(Q, K, pre, np.concatenate([x[:70], extra]))
    same_as_oracle(Q, K, twin, np.concatenate([x, -extra]))
    assert Q.QKvCache(fmt).clone_prefix(3).len == 0 and one_shot.clone_prefix(0).width == 0
    # what it costs (:2110): the advertised bits per value, up to the one shared scale word
    full = Q.QKvCache.from_tensor(F.Tensor.from_vec(x[:64], (64, width)), fmt)
    assert full.bytes() == full.live_bytes() == 64 * 3 * Q.BLOCK_BYTES[fmt] and full.f32_bytes() == 64 * width * 4
    assert Q.bits_per_value(fmt) == {0: 8.5, 1: 4.5, 2: 5.0}[fmt]


def test_positions_on_the_device_and_argument_checks(F, Q, K):
    """What a captured decode step uses: the row index read from a device word on both sides, the source row at that index of a
    full-length f32 staging cache, and a dequantize sized for the capacity that stops at the newest row."""
    lib = F._lib.load()
    rng = np.random.default_rng(60)
    cap, width, fmt = 12, 64, 0
    staging = (rng.standard_normal((cap, width)) * 2).astype(np.float32)
    st = F.Tensor.from_vec(staging, staging.shape)
    cache = Q.QKvCache(fmt, cap, width)
    pos = F.Tensor(F.DeviceBuffer(4), (1,), np.uint32)
    ref = K.Cache(fmt, cap, width)
    out = F.Tensor.from_vec(np.full((cap, width), 777.0, np.float32), (cap, width))
    for p in (0, 1, 2, 7):
        word = np.array([p], np.uint32)
        F._lib.check(lib.fhip_memcpy_h2d(pos.buf.ptr, word.ctypes.data, 4, None))
        F._lib.check(lib.fhip_kvq_append(fmt, st.buf.ptr, width, 1, width, pos.buf.ptr, 0, 1, cap, cache.codes.ptr, cache.scales.ptr, None))
        ref.quantize_into(staging[p], p)
        F._lib.check(lib.fhip_kvq_dequantize_rows(fmt, cache.codes.ptr, cache.scales.ptr, 0, cap, width, pos.buf.ptr, out.buf.ptr, None))
        got = out.to_vec().reshape(cap, width)
        assert np.array_equal(bits(got[p]), bits(ref.dequantize_rows(p, 1)[0])), p
        assert (got[p + 1:] == 777.0).all(), p                                  # rows past the position are not written
    # a position beyond the capacity is dropped, as fhip_kv_append2 drops it
    word = np.array([cap + 3], np.uint32)
    F._lib.check(lib.fhip_memcpy_h2d(pos.buf.ptr, word.ctypes.data, 4, None))
    before = cache.codes
    F._lib.check(lib.fhip_kvq_append(fmt, st.buf.ptr, width, 1, width, pos.buf.ptr, 0, 0, cap, cache.codes.ptr, cache.scales.ptr, None))
    F._lib.check(lib.fhip_stream_sync(None))
    # errors: the reference's width assert (kvquant.rs:470), unknown formats, rows past the capacity, NULL pointers
    assert lib.fhip_kvq_append(fmt, st.buf.ptr, 0, 1, 48, None, 0, 0, cap, cache.codes.ptr, cache.scales.ptr, None) != 0
    assert b"must be a multiple of 32" in lib.fhip_last_error()
    assert lib.fhip_kvq_append(9, st.buf.ptr, 0, 1, 64, None, 0, 0, cap, cache.codes.ptr, cache.scales.ptr, None) != 0
    assert lib.fhip_kvq_append(fmt, st.buf.ptr, 0, 5, 64, None, 10, 0, cap, cache.codes.ptr, cache.scales.ptr, None) != 0
    assert b"exceed the capacity" in lib.fhip_last_error()
    assert lib.fhip_kvq_append(fmt, None, 0, 1, 64, None, 0, 0, cap, cache.codes.ptr, cache.scales.ptr, None) != 0
    assert lib.fhip_kvq_dequantize_rows(fmt, cache.codes.ptr, cache.scales.ptr, 0, 1, 64, None, None, None) != 0
    assert lib.fhip_kvq_append(fmt, None, 0, 0, 64, None, 0, 0, cap, None, None, None) == 0              # nothing to do
    cw, sw = C.c_size_t(), C.c_size_t()
    for f in (0, 1, 2):
        assert lib.fhip_kvq_sizes(f, 7, 96, C.byref(cw), C.byref(sw)) == 0 and (cw.value, sw.value) == K.sizes(7, 96, f)
    with pytest.raises(AssertionError, match="past len"):
        cache.dequantize_rows(0, 1)


@pytest.mark.parametrize("fmt", [0, 1, 2])
def test_attention_over_the_blocks_is_attention_over_the_dequantized_rows(F, Q, K, fmt):
    """fhip_decode_attention_kvq dequantizes rows in registers by the dequantize kernel's own operations, so its output has the
    bits of fhip_decode_attention_ex over dequantize(); and it is the oracle's attention over the oracle's dequantized rows to the
    f32 attention's tolerance (1e-5 of the largest output)."""
    from types import SimpleNamespace
    from ferric_amd import decode as X
    from oracle import decode_oracle as D
    rng = np.random.default_rng(70 + fmt)
    # (heads, kv heads, head dim, rows, window, softcap): one split and many, both head sizes, every group size class, a
    # length that leaves the last split ragged, a window, a softcap
    cases = [(8, 2, 128, 7, 0, 0.0), (40, 8, 128, 300, 0, 0.0), (8, 8, 64, 129, 0, 0.0), (6, 2, 64, 1000, 0, 0.0), (16, 2, 128, 2100, 512, 0.0),
             (5, 1, 128, 260, 0, 30.0), (14, 2, 64, 33, 8, 50.0)]
    for nh, nkv, hd, rows, window, cap in cases:
        width = nkv * hd
        k = (rng.standard_normal((rows, width)) * 2).astype(np.float32)
        v = (rng.standard_t(3, (rows, width))).astype(np.float32)
        q = rng.standard_normal((1, nh * hd)).astype(np.float32)
        kq = Q.QKvCache.from_tensor(F.Tensor.from_vec(k, k.shape), fmt)
        vq = Q.QKvCache.from_tensor(F.Tensor.from_vec(v, v.shape), fmt)
        qt = F.Tensor.from_vec(q, q.shape)
        got = X.decode_attention_kvq(qt, kq, vq, nh, nkv, window=window, softcap=cap).to_vec()
        plain = SimpleNamespace(k=kq.dequantize(), v=vq.dequantize(), cap=rows, width=width, len=rows)
        same = X.decode_attention(qt, plain, nh, nkv, window=window, softcap=cap).to_vec()
        assert np.array_equal(bits(got), bits(same)), (nh, nkv, hd, rows)
        want = D.decode_attention(q[0], K.roundtrip(k, rows, width, fmt), K.roundtrip(v, rows, width, fmt), nh, nkv, window, cap)
        assert np.abs(got - want.reshape(-1)).max() <= 1e-5 * np.abs(want).max(), (nh, nkv, hd, rows)
        # a shorter length, and the length read from a device word (what a captured step does)
        n = max(1, rows // 3)
        word = F.Tensor(F.DeviceBuffer(4), (1,), np.uint32)
        last = np.array([n - 1], np.uint32)
        F._lib.check(F._lib.load().fhip_memcpy_h2d(word.buf.ptr, last.ctypes.data, 4, None))
        a = X.decode_attention_kvq(qt, kq, vq, nh, nkv, length=n, window=window, softcap=cap).to_vec()
        b = X.decode_attention_kvq(qt, kq, vq, nh, nkv, length=rows, last_pos=word, window=window, softcap=cap).to_vec()
        want = D.decode_attention(q[0], K.roundtrip(k[:n], n, width, fmt), K.roundtrip(v[:n], n, width, fmt), nh, nkv, window, cap).reshape(-1)
        assert np.abs(a - want).max() <= 1e-5 * np.abs(want).max() and np.abs(b - want).max() <= 1e-5 * np.abs(want).max()
    lib = F._lib.load()
    assert lib.fhip_decode_attention_kvq(fmt, qt.buf.ptr, kq.codes.ptr, kq.scales.ptr, vq.codes.ptr, vq.scales.ptr, 14, 2, 48, 5, None, 0, 0.0, None,
                                         qt.buf.ptr, None) != 0                      # 2 x 48 is a multiple of 32, the head size is not one the kernel takes
    assert b"head_dim must be 64 or 128" in lib.fhip_last_error()


def test_k_and_v_rows_stored_by_one_launch(F, Q, K):
    rng = np.random.default_rng(80)
    t, width, cap = 5, 256, 16
    k, v = rng.standard_normal((t, width)).astype(np.float32), (rng.standard_normal((t, width)) * 7).astype(np.float32)
    lib = F._lib.load()
    for fmt in (0, 1, 2):
        kq, vq = Q.QKvCache(fmt, cap, width), Q.QKvCache(fmt, cap, width)
        pos = F.Tensor(F.DeviceBuffer(4 * t), (t,), np.uint32)
        where = np.array([3, 0, 9, 15, 4], np.uint32)
        F._lib.check(lib.fhip_memcpy_h2d(pos.buf.ptr, where.ctypes.data, 4 * t, None))
        kt, vt = F.Tensor.from_vec(k, k.shape), F.Tensor.from_vec(v, v.shape)
        F._lib.check(lib.fhip_kvq_append2(fmt, kt.buf.ptr, vt.buf.ptr, 0, t, width, pos.buf.ptr, 0, cap, kq.codes.ptr, kq.scales.ptr, vq.codes.ptr,
                                          vq.scales.ptr, None))
        kq.len = vq.len = cap
        for cache, x in ((kq, k), (vq, v)):
            got = cache.dequantize().to_vec().reshape(cap, width)
            for i, r in enumerate(where):
                assert np.array_equal(bits(got[r]), bits(K.roundtrip(x[i], 1, width, fmt)[0])), (fmt, i)
