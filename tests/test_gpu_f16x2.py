"""Small-batch matmul on the f16 matrix cores (fhip_matmul_q_f16x2 / fhip_ffn_f16x2) vs the CPU oracle, through the C ABI.

The path claims f32-grade results: weights enter the matrix cores as exact integers, activations as a hi/lo pair of f16
scaled chunk by chunk (22 significant bits at a 256-column chunk's largest magnitude). Bars, against the oracle's dequantized weights in f64:
  * |y - y64| <= 2.5e-7 * ||w_row|| * ||x_t||  (measured <= 6e-8; the exact-f32 mat-vec path measures <= 5e-8 on the same
    inputs), 4000x inside the north-star bound 1e-3 * ||w_row|| * ||x_t||;
  * max|d| / max|ref| < 1e-5, the bar the f32 mat-vec tests use;
  * Q8_0 (quants are exact in f16, one f32 scale per 32-wide slice) keeps the same 2.5e-7 bar; at most 16 activation rows;
  * Q6_K only, blocks whose |scale * (q - 32)| exceeds 2048: such a product is rounded to an even integer on its way
    into f16, a relative 2^-12 on that weight, so the bar there is 2.5e-4 * ||w_row|| * ||x_t|| (still 4x inside the
    north-star bound) -- the test builds such blocks on purpose and also checks that ordinary ones stay at 2.5e-7.
"""
import numpy as np
import pytest

# the f32 mat-vec path is the other side of most comparisons here: it runs with 24-bit activations
pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("precision24")]
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
TIGHT = 2.5e-7


def run_case(F, O, ty, t, n, k, seed, x=None, w=None, tol=TIGHT):
    from ferric_amd.synth import synth_weights
    w = synth_weights(ty, n, k, seed) if w is None else w
    x = np.random.default_rng(seed + 1).standard_normal((t, k)).astype(np.float32) if x is None else x
    qm = F.QMatrix.from_bytes(w, ty, n, k)
    y = F.Tensor.from_vec(x, x.shape).matmul_q_f16x2(qm).to_vec().reshape(t, n)
    y64, wn = O.matmul_f64(x, w, ty, n, k)
    err = np.abs(y - y64)
    bound = tol * wn[None, :] * np.linalg.norm(x.astype(np.float64), axis=1)[:, None]
    assert (err <= bound + 1e-300).all(), (ty, t, n, k, float(np.max(err / (bound + 1e-300))))
    assert err.max() / max(1e-30, np.abs(y64).max()) < 1e-5 * max(1.0, tol / TIGHT)
    return y, y64


@pytest.mark.parametrize("ty", [Q4_K, Q5_K, Q6_K, Q8_0])
def test_small_and_ragged_shapes(F, O, ty):
    # every activation-row count class (1..8 -> one group of operand rows, 9..16 -> two, 17..32 -> four), weight rows that
    # do not fill a 16-row set, a 128-row group or a workgroup's share, one chunk and many
    shapes = [(1, 32, 256), (2, 100, 512), (3, 128, 256), (5, 300, 1024), (8, 256, 2048), (9, 130, 768), (16, 257, 1024),
              (17, 64, 512), (31, 15, 256), (32, 200, 1536), (4, 1, 256), (7, 1000, 5120)]
    if ty == Q8_0:
        # at most 16 rows; rows of any whole number of 32-column blocks: shorter than a chunk, ending inside the last one
        shapes = [s for s in shapes if s[0] <= 16] + [(3, 40, 32), (8, 64, 96), (9, 130, 288), (16, 70, 480), (5, 257, 1184),
                                                      (1, 4096, 4096)]
    for i, (t, n, k) in enumerate(shapes):
        run_case(F, O, ty, t, n, k, 100 + i)


@pytest.mark.parametrize("ty", [Q4_K, Q5_K, Q6_K])
def test_a_chunk_of_small_values_keeps_its_bits_beside_a_large_one(F, O, ty):
    # The scale is per 256-column chunk. Weights whose first super-block has scale 0 ignore the first chunk of x, so a
    # first chunk 2^60 times larger than the rest must not cost the rest its precision: the outputs are held to the bound
    # taken over the other chunks' activations only (with one scale per row their 22 bits would all lie above those values).
    from ferric_amd.synth import synth_weights
    t, n, k = 6, 160, 1280
    blk = {Q4_K: 144, Q5_K: 176, Q6_K: 210}[ty]
    w = synth_weights(ty, n, k, 61).copy().reshape(n, k // 256, blk)
    if ty in (Q4_K, Q5_K):
        w[:, 0, 0:4] = 0          # d and dmin of the first super-block of every row
    else:
        w[:, 0, 208:210] = 0      # d
    w = w.reshape(-1)
    x = np.random.default_rng(62).standard_normal((t, k)).astype(np.float32)
    x[:, :256] *= np.float32(2.0 ** 60)
    qm = F.QMatrix.from_bytes(w, ty, n, k)
    y = F.Tensor.from_vec(x, x.shape).matmul_q_f16x2(qm).to_vec().reshape(t, n)
    y64, _ = O.matmul_f64(x, w, ty, n, k)
    wd = O.deq_raw(w, n * k, ty).reshape(n, k).astype(np.float64)
    assert not wd[:, :256].any()
    bound = TIGHT * np.linalg.norm(wd[:, 256:], axis=1)[None, :] * np.linalg.norm(x[:, 256:].astype(np.float64), axis=1)[:, None]
    assert (np.abs(y - y64) <= bound).all(), float(np.max(np.abs(y - y64) / bound))


@pytest.mark.parametrize("ty", [Q4_K, Q5_K, Q6_K, Q8_0])
def test_rows_of_very_different_magnitude(F, O, ty):
    # each chunk of a row is scaled by its own power of two: tiny, huge, zero and outlier rows side by side keep the per-row bound
    t, n, k = 8, 96, 1024
    x = np.random.default_rng(7).standard_normal((t, k)).astype(np.float32)
    x[0] *= np.float32(1e-30)
    x[1] *= np.float32(1e30)
    x[2] = 0.0
    x[3, 17] = np.float32(3e6)            # one outlier sets the scale; the rest of the row is 2^-21 of it
    x[4] *= np.float32(65504.0 * 4)       # beyond the f16 range before scaling
    x[5] *= np.float32(2.0 ** -118)       # near the bottom of the f32 normal range: the scale is capped at 2^126
    y, y64 = run_case(F, O, ty, t, n, k, 8, x=x)
    assert not y[2].any()


def test_nonfinite_values_stay_in_their_row(F, O):
    t, n, k = 6, 64, 512
    x = np.random.default_rng(9).standard_normal((t, k)).astype(np.float32)
    x[1, 5] = np.inf
    x[4, 300] = np.nan
    from ferric_amd.synth import synth_weights
    w = synth_weights(Q4_K, n, k, 10)
    qm = F.QMatrix.from_bytes(w, Q4_K, n, k)
    y = F.Tensor.from_vec(x, x.shape).matmul_q_f16x2(qm).to_vec().reshape(t, n)
    assert not np.isfinite(y[1]).any() and np.isnan(y[4]).all()      # as a dot product with inf / nan in it comes out
    good = [0, 2, 3, 5]
    y64, wn = O.matmul_f64(x[good], w, Q4_K, n, k)
    bound = TIGHT * wn[None, :] * np.linalg.norm(x[good].astype(np.float64), axis=1)[:, None]
    assert (np.abs(y[good] - y64) <= bound).all()


def test_q6_k_products_beyond_the_exact_f16_range(F, O):
    # scales of +-127 / -128 with quants at the ends of their range: |sc * (q - 32)| up to 4096
    from ferric_amd.synth import synth_weights
    n, k, t = 64, 1024, 8
    w = synth_weights(Q6_K, n, k, 11).reshape(n, k // 256, 210).copy()
    rng = np.random.default_rng(12)
    w[:, :, 192:208] = rng.choice(np.array([127, 125, -127, -128], np.int8).view(np.uint8), size=(n, k // 256, 16))
    w[:, :, 0:128] = rng.choice(np.array([0x00, 0xFF, 0x0F, 0xF0, 0x1E], np.uint8), size=(n, k // 256, 128))
    w[:, :, 128:192] = rng.choice(np.array([0x00, 0xFF, 0xCC, 0x33], np.uint8), size=(n, k // 256, 64))
    y, y64 = run_case(F, O, Q6_K, t, n, k, 13, w=w.reshape(-1), tol=2.5e-4)
    # the same blocks with small scales are exact again
    w[:, :, 192:208] = rng.choice(np.array([31, -32, 17, -5], np.int8).view(np.uint8), size=(n, k // 256, 16))
    run_case(F, O, Q6_K, t, n, k, 13, w=w.reshape(-1))


def test_q5_k_every_code_and_the_largest_scales(F, O):
    # all 32 codes (both nibbles, the fifth bit set and clear) under 6-bit scales and minima at their ends: the largest
    # product, 63 * 31 = 1953, is still an exact f16 integer
    n, k, t = 64, 1024, 8
    rng = np.random.default_rng(16)
    w = np.zeros((n, k // 256, 176), np.uint8)
    d = rng.choice(np.array([0.01, -0.02, 0.5, 3e-4], np.float16), size=(n, k // 256, 2))
    w[:, :, 0:4] = d.view(np.uint8).reshape(n, k // 256, 4)
    w[:, :, 4:16] = rng.choice(np.array([0xFF, 0x3F, 0xC0, 0x00, 0x7E, 0xA5], np.uint8), size=(n, k // 256, 12))
    w[:, :, 16:48] = rng.choice(np.array([0x00, 0xFF, 0xAA, 0x55, 0x81], np.uint8), size=(n, k // 256, 32))
    w[:, :, 48:] = rng.choice(np.array([0x00, 0xFF, 0x0F, 0xF0, 0x1E, 0xE1], np.uint8), size=(n, k // 256, 128))
    w[0, 0, 16:48] = np.arange(32, dtype=np.uint8) * 8 + 1
    w[0, 0, 48:] = np.arange(128, dtype=np.uint8) * 2 + 1
    run_case(F, O, Q5_K, t, n, k, 17, w=w.reshape(-1))
    run_case(F, O, Q5_K, 20, n, k, 18, w=w.reshape(-1))


def test_q8_0_every_int8_value_and_scale_signs(F, O):
    # quants over all 256 byte values (-128 included), scales of both signs, zero and the largest finite f16 magnitude class
    n, k, t = 48, 512, 4
    rng = np.random.default_rng(14)
    w = np.zeros((n, k // 32, 34), np.uint8)
    w[:, :, 2:] = rng.integers(0, 256, (n, k // 32, 32), dtype=np.uint8)
    w[0, 0, 2:] = np.arange(32, dtype=np.uint8) * 8          # 0, 8, .., 248: both halves of the int8 range in one block
    w[1, 1, 2:] = 0x80
    d = rng.choice(np.array([0.0, -0.03, 0.5, 1e-4, -2048.0, 6e-8], np.float16), size=(n, k // 32))
    w[:, :, 0:2] = d.view(np.uint8).reshape(n, k // 32, 2)
    run_case(F, O, Q8_0, t, n, k, 15, w=w.reshape(-1))


@pytest.mark.parametrize("ty,n,k", [(Q4_K, 512, 2048), (Q5_K, 400, 1536), (Q6_K, 384, 1024), (Q8_0, 640, 1120)])
def test_agrees_with_the_f32_matvec_path_and_rows_are_independent(F, O, ty, n, k):
    from ferric_amd.synth import synth_weights
    w = synth_weights(ty, n, k, 20)
    qm = F.QMatrix.from_bytes(w, ty, n, k)
    x = np.random.default_rng(21).standard_normal((12, k)).astype(np.float32)
    y = F.Tensor.from_vec(x, x.shape).matmul_q_f16x2(qm).to_vec().reshape(12, n)
    f32 = F.Tensor.from_vec(x, x.shape).matmul_q(qm).to_vec().reshape(12, n)
    assert np.abs(y - f32).max() <= 2e-6 * np.abs(f32).max()
    # a row computed in a batch of 12 (two operand-row groups) and alone (one group): same value up to the order of the
    # f32 additions of K slices
    one = F.Tensor.from_vec(x[9:10], (1, k)).matmul_q_f16x2(qm).to_vec()
    assert np.abs(one - y[9]).max() <= 2e-6 * np.abs(y[9]).max()


@pytest.mark.parametrize("batch", [4, 8])
def test_config3_ffn_block(F, O, batch):
    # gate|up 2 x (5120 -> 17408) Q4_K stacked gate-first, down 17408 -> 5120 Q6_K, SwiGLU between, one call
    from ferric_amd.synth import synth_weights
    n_embd, n_ff = 5120, 17408
    gu = synth_weights(Q4_K, 2 * n_ff, n_embd, 3)
    dn = synth_weights(Q6_K, n_embd, n_ff, 4)
    x = np.random.default_rng(5).standard_normal((batch, n_embd)).astype(np.float32)
    wgu = F.QMatrix.from_bytes(gu, Q4_K, 2 * n_ff, n_embd)
    wdn = F.QMatrix.from_bytes(dn, Q6_K, n_embd, n_ff)
    xt = F.Tensor.from_vec(x, x.shape)
    y = xt.ffn_f16x2(wgu, wdn).to_vec().reshape(batch, n_embd)
    g64, _ = O.matmul_f64(x, gu, Q4_K, 2 * n_ff, n_embd)
    g, u = g64[:, :n_ff], g64[:, n_ff:]
    h64 = g / (1.0 + np.exp(-g)) * u
    # the down projection of the f64 SwiGLU (matmul_f64 takes f32 activations: its rounding of h is 6e-8 relative)
    y64, wn = O.matmul_f64(h64.astype(np.float32), dn, Q6_K, n_embd, n_ff)
    err = np.abs(y - y64)
    assert (err <= 1e-6 * wn[None, :] * np.linalg.norm(h64, axis=1)[:, None]).all()
    assert err.max() / np.abs(y64).max() < 1e-5
    # and the exact-f32 block gives the same answer to f32 rounding
    y32 = xt.ffn(wgu, wdn).to_vec().reshape(batch, n_embd)
    assert np.abs(y - y32).max() / np.abs(y32).max() < 2e-6


@pytest.mark.parametrize("tg,td", [(Q8_0, Q8_0), (Q4_K, Q8_0), (Q8_0, Q6_K)])
def test_ffn_block_with_q8_0_weights(F, O, tg, td):
    # the block with Q8_0 on either side, a hidden width that ends inside a chunk for the Q8_0 down projection
    from ferric_amd.synth import synth_weights
    n_embd, n_ff, batch = 768, (1120 if td == Q8_0 else 1280), 7
    gu = synth_weights(tg, 2 * n_ff, n_embd, 40)
    dn = synth_weights(td, n_embd, n_ff, 41)
    x = np.random.default_rng(42).standard_normal((batch, n_embd)).astype(np.float32)
    wgu, wdn = F.QMatrix.from_bytes(gu, tg, 2 * n_ff, n_embd), F.QMatrix.from_bytes(dn, td, n_embd, n_ff)
    xt = F.Tensor.from_vec(x, x.shape)
    y = xt.ffn_f16x2(wgu, wdn).to_vec().reshape(batch, n_embd)
    g64, _ = O.matmul_f64(x, gu, tg, 2 * n_ff, n_embd)
    h64 = g64[:, :n_ff] / (1.0 + np.exp(-g64[:, :n_ff])) * g64[:, n_ff:]
    y64, wn = O.matmul_f64(h64.astype(np.float32), dn, td, n_embd, n_ff)
    assert (np.abs(y - y64) <= 1e-6 * wn[None, :] * np.linalg.norm(h64, axis=1)[:, None]).all()
    if tg != Q8_0:      # the exact-f32 block takes K-quant gate|up weights only
        y32 = xt.ffn(wgu, wdn).to_vec().reshape(batch, n_embd)
        assert np.abs(y - y32).max() / np.abs(y32).max() < 2e-6


@pytest.mark.parametrize("ty", [Q4_K, Q5_K, Q6_K, Q8_0])
def test_random_shapes_against_the_f32_path(F, O, ty):
    # 24 seeded random (rows of x, rows of W, columns) triples: every branch of the launch plan (whole groups, dealt runs,
    # runs that cross group boundaries, weights shorter than a workgroup's share) against the exact f32 mat-vec path
    from ferric_amd.synth import synth_weights
    rng = np.random.default_rng(1234 + ty)
    for _ in range(24):
        t = int(rng.integers(1, 17 if ty == Q8_0 else 33))
        n = int(rng.choice([1, 7, 16, 31, 33, 127, 128, 129, 255, 300, 511, 777, 1500, 4100]))
        k = 256 * int(rng.choice([1, 2, 3, 5, 8, 13, 20, 31]))
        if ty == Q8_0:
            k = max(32, k - 32 * int(rng.integers(0, 8)))     # rows that end anywhere inside their last chunk
        w = synth_weights(ty, n, k, int(rng.integers(1 << 30)))
        x = (rng.standard_normal((t, k)) * 10.0 ** rng.uniform(-3, 3, size=(t, 1))).astype(np.float32)
        qm = F.QMatrix.from_bytes(w, ty, n, k)
        y = F.Tensor.from_vec(x, x.shape).matmul_q_f16x2(qm).to_vec().reshape(t, n)
        f32 = F.Tensor.from_vec(x, x.shape).matmul_q(qm).to_vec().reshape(t, n)
        wn = np.linalg.norm(O.deq_raw(w, n * k, ty).reshape(n, k).astype(np.float64), axis=1)
        bound = 2 * TIGHT * wn[None, :] * np.linalg.norm(x.astype(np.float64), axis=1)[:, None]   # two paths, each within TIGHT
        assert (np.abs(y - f32) <= bound + 1e-300).all(), (ty, t, n, k)


def test_replays_in_a_graph(F, O):
    # the six launches of the block captured once and replayed with new inputs in the same buffers: every replay must
    # match an eager call on the same input (up to the order of the K-split additions)
    import ctypes as C
    from ferric_amd import _lib
    from ferric_amd.synth import synth_weights
    lib = _lib.load()
    n_embd, n_ff, t = 512, 1280, 5
    gu = F.QMatrix.from_bytes(synth_weights(Q4_K, 2 * n_ff, n_embd, 30), Q4_K, 2 * n_ff, n_embd)
    dn = F.QMatrix.from_bytes(synth_weights(Q6_K, n_embd, n_ff, 31), Q6_K, n_embd, n_ff)
    st = F.Stream()
    x = F.Tensor.from_vec(np.zeros((t, n_embd), np.float32), (t, n_embd))
    y = F.Tensor.empty((t, n_embd))
    ws = F.DeviceBuffer(lib.fhip_ffn_f16x2_ws_bytes(gu.handle, dn.handle, t))
    g = F.Graph.begin(st)
    _lib.check(lib.fhip_ffn_f16x2(gu.handle, dn.handle, x.buf.ptr, t, y.buf.ptr, ws.ptr, st.handle))
    g.end()
    rng = np.random.default_rng(32)
    for rep in range(4):
        xin = (rng.standard_normal((t, n_embd)) * (10.0 ** rep)).astype(np.float32)
        _lib.check(lib.fhip_memcpy_h2d(x.buf.ptr, xin.ctypes.data_as(C.c_void_p), xin.nbytes, st.handle))
        g.launch()
        st.synchronize()
        got = y.to_vec().reshape(t, n_embd)
        want = F.Tensor.from_vec(xin, xin.shape).ffn_f16x2(gu, dn).to_vec().reshape(t, n_embd)
        assert np.abs(got - want).max() <= 2e-6 * np.abs(want).max(), rep


def test_argument_checks(F):
    from ferric_amd import _lib
    import ctypes as C
    lib = _lib.load()
    from ferric_amd.synth import synth_weights
    q4 = F.QMatrix.from_bytes(synth_weights(Q4_K, 32, 256, 1), Q4_K, 32, 256)
    q8 = F.QMatrix.from_bytes(synth_weights(Q8_0, 32, 256, 1), Q8_0, 32, 256)
    q40 = F.QMatrix.from_bytes(synth_weights(2, 32, 256, 1), 2, 32, 256)     # Q4_0: served by the mat-vec path only
    assert lib.fhip_matmul_q_f16x2_ws_bytes(q4.handle, 8) > 0 and lib.fhip_matmul_q_f16x2_ws_bytes(q8.handle, 16) > 0
    assert lib.fhip_matmul_q_f16x2_ws_bytes(q4.handle, 33) == 0 and lib.fhip_matmul_q_f16x2_ws_bytes(q40.handle, 8) == 0
    assert lib.fhip_matmul_q_f16x2_ws_bytes(q8.handle, 17) == 0
    with pytest.raises(AssertionError, match="at most 32 activation rows"):
        F.Tensor.from_vec(np.zeros((33, 256), np.float32), (33, 256)).matmul_q_f16x2(q4)
    with pytest.raises(AssertionError, match="at most 16 activation rows for Q8_0"):
        F.Tensor.from_vec(np.zeros((17, 256), np.float32), (17, 256)).matmul_q_f16x2(q8)
    with pytest.raises(ValueError, match="Q4_K, Q5_K, Q6_K and Q8_0 only"):
        F.Tensor.from_vec(np.zeros((2, 256), np.float32), (2, 256)).matmul_q_f16x2(q40)
    with pytest.raises(AssertionError, match="inner dim mismatch"):
        F.Tensor.from_vec(np.zeros((2, 512), np.float32), (2, 512)).matmul_q_f16x2(q4)
    x = F.Tensor.from_vec(np.zeros((2, 256), np.float32), (2, 256))
    y = F.Tensor.empty((2, 32))
    ws = F.DeviceBuffer(lib.fhip_matmul_q_f16x2_ws_bytes(q4.handle, 2) + 256)
    with pytest.raises(_lib.FerricHipError, match="256-byte aligned"):
        _lib.check(lib.fhip_matmul_q_f16x2(q4.handle, x.buf.ptr, 2, y.buf.ptr, C.c_void_p(ws.ptr.value + 16), None))
    with pytest.raises(_lib.FerricHipError, match="NULL pointer"):
        _lib.check(lib.fhip_matmul_q_f16x2(q4.handle, x.buf.ptr, 2, y.buf.ptr, None, None))
    # no rows: nothing to do, nothing touched
    assert F.Tensor.from_vec(np.zeros(0, np.float32), (0, 256)).matmul_q_f16x2(q4).to_vec().size == 0
    dn = F.QMatrix.from_bytes(synth_weights(Q6_K, 32, 256, 2), Q6_K, 32, 256)
    with pytest.raises(AssertionError, match="down in dim must equal n_ff"):
        F.Tensor.from_vec(np.zeros((2, 256), np.float32), (2, 256)).ffn_f16x2(q4, dn)


# ---------------------------------------------------------------- FHIP_BATCH_ORDERED: the same kernels, partial sums added in order

def test_ordered_policy_gives_the_same_bits_on_every_run(F, O):
    # Under FHIP_BATCH_ORDERED (2, what a new weight has) the drop-in calls keep the one-pass kernels, but a launch that cuts a group's K between
    # workgroups writes the pieces to the library's workspace and adds them in a fixed order: run after run the same bits,
    # and the same bars against the oracle as the default policy. Shapes: cut along K (few groups, long rows), not cut
    # (one chunk), ragged rows, each activation-row class, Q8_0's ragged K; then the FFN block at the model's size, where
    # the down projection (40 groups of 68 chunks) is cut many ways.
    from ferric_amd.synth import synth_weights
    lib = F._lib.load()
    before = lib.fhip_batch_policy(2)
    try:
        assert lib.fhip_batch_policy(-1) == 2
        cases = [(Q4_K, 4, 512, 8192), (Q4_K, 8, 5120, 5120), (Q6_K, 3, 130, 4096), (Q6_K, 12, 1000, 17408), (Q4_K, 20, 257, 2048),
                 (Q4_K, 32, 64, 256), (Q8_0, 5, 300, 4128), (Q8_0, 16, 1024, 4096), (Q4_K, 40, 384, 6144),
                 (Q5_K, 6, 256, 8192), (Q5_K, 24, 1000, 2048)]
        for i, (ty, t, n, k) in enumerate(cases):
            w = synth_weights(ty, n, k, 700 + i)
            x = np.random.default_rng(800 + i).standard_normal((t, k)).astype(np.float32)
            qm = F.QMatrix.from_bytes(w, ty, n, k)
            xt = F.Tensor.from_vec(x, x.shape)
            y = xt.matmul_q(qm).to_vec().reshape(t, n)
            y64, wn = O.matmul_f64(x, w, ty, n, k)
            bound = TIGHT * wn[None, :] * np.linalg.norm(x.astype(np.float64), axis=1)[:, None]
            assert (np.abs(y - y64) <= bound + 1e-300).all(), (ty, t, n, k)
            for _ in range(3):
                assert np.array_equal(xt.matmul_q(qm).to_vec().reshape(t, n), y), (ty, t, n, k)
        n_embd, n_ff, batch = 5120, 17408, 8
        gu = synth_weights(Q4_K, 2 * n_ff, n_embd, 3)
        dn = synth_weights(Q6_K, n_embd, n_ff, 4)
        x = np.random.default_rng(5).standard_normal((batch, n_embd)).astype(np.float32)
        wgu = F.QMatrix.from_bytes(gu, Q4_K, 2 * n_ff, n_embd)
        wdn = F.QMatrix.from_bytes(dn, Q6_K, n_embd, n_ff)
        xt = F.Tensor.from_vec(x, x.shape)
        y = xt.ffn(wgu, wdn).to_vec()
        for _ in range(3):
            assert np.array_equal(xt.ffn(wgu, wdn).to_vec(), y)
        # the block leaves gate|up's partial sums to the launch that prepares the down projection's activations; the three
        # calls it stands for add them in a launch of their own, in the same order: the same bits
        steps = xt.try_matmul_swiglu(wgu).matmul_q(wdn).to_vec()
        assert np.array_equal(steps, y)
        wgu.batch_policy(0), wdn.batch_policy(0)
        y0 = xt.ffn(wgu, wdn).to_vec()                 # FHIP_BATCH_AUTO: atomic adds, the same sums in another order
        assert np.abs(y - y0).max() <= 2e-6 * np.abs(y0).max()
        # a ragged block (hidden width not a multiple of 128, three rows) in one call and in three
        n_embd, n_ff, batch = 768, 1280 + 256, 3
        wgu = F.QMatrix.from_bytes(synth_weights(Q4_K, 2 * n_ff, n_embd, 33), Q4_K, 2 * n_ff, n_embd)
        wdn = F.QMatrix.from_bytes(synth_weights(Q6_K, n_embd - 1, n_ff, 34), Q6_K, n_embd - 1, n_ff)
        xt = F.Tensor.from_vec(np.random.default_rng(35).standard_normal((batch, n_embd)).astype(np.float32), (batch, n_embd))
        assert np.array_equal(xt.try_matmul_swiglu(wgu).matmul_q(wdn).to_vec(), xt.ffn(wgu, wdn).to_vec())
    finally:
        lib.fhip_batch_policy(before)
