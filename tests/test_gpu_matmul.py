"""GPU mat-vec / small-batch matmul / fused SwiGLU / FFN vs the CPU oracle, through the C ABI.

Tolerances (written where used):
  * north-star bound: |y - y64| <= 1e-3 * ||w_row||_2 * ||x||_2 against the f64-accumulated product of
    the oracle-dequantized weights;
  * the reference examples' own bar for scalar kernels: max|y - ref| / max(|ref|, 1e-3) < 1e-5
    (crates/ferric-tensor/examples/q4_k.rs:54, q6_k.rs:33, q8_0.rs:21, ffn_fuse.rs:106).
"""
import numpy as np
import pytest

from conftest import bits, dot_bar

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("precision")]
Q8_0, Q4_K, Q6_K = 8, 12, 14


def check_matmul(F, O, w, ty, rows, cols, x, what=""):
    """Run y = x W^T on the GPU and hold it to both tolerances; returns the GPU result [m, rows]."""
    x = np.ascontiguousarray(x, np.float32).reshape(-1, cols)
    qm = F.QMatrix.from_bytes(w, ty, rows, cols)
    assert (qm.rows(), qm.cols(), qm.nbytes(), qm.n_shards()) == (rows, cols, w.size, 1)
    y = F.Tensor.from_vec(x, x.shape).matmul_q(qm).to_vec().reshape(x.shape[0], rows)
    y64, wn = O.matmul_f64(x, w, ty, rows, cols)
    err = np.abs(y - y64)
    bound = 1e-3 * wn[None, :] * np.linalg.norm(x.astype(np.float64), axis=1)[:, None]
    assert (err <= bound + 1e-30).all(), f"{what}: north-star bound violated by {np.max(err / (bound + 1e-30)):.3g}x"
    rel = err.max() / max(1e-3, np.abs(y64).max())
    assert rel < dot_bar(), f"{what}: max|d|/max|ref| = {rel:.2e}"
    return y


def cosx(m, cols):
    return np.cos(np.arange(m * cols, dtype=np.float32) * np.float32(0.013)).astype(np.float32).reshape(m, cols)


# ---------------------------------------------------------------- the reference examples, same inputs

@pytest.mark.parametrize("rows,cols,m", [(8, 256, 4), (13, 512, 1), (4096, 2048, 1)])
def test_q4_k_example(F, O, rows, cols, m):          # crates/ferric-tensor/examples/q4_k.rs:43-56
    check_matmul(F, O, O.gen_kquant_matrix(Q4_K, rows, cols), Q4_K, rows, cols, cosx(m, cols), "q4_k.rs")


@pytest.mark.parametrize("rows,cols,m", [(8, 256, 4), (7, 512, 1), (2048, 1024, 1)])
def test_q6_k_example(F, O, rows, cols, m):          # crates/ferric-tensor/examples/q6_k.rs:22-35
    check_matmul(F, O, O.gen_kquant_matrix(Q6_K, rows, cols), Q6_K, rows, cols, cosx(m, cols), "q6_k.rs")


@pytest.mark.parametrize("rows,cols,m", [(8, 256, 4), (13, 128, 1), (4096, 2048, 1)])
def test_q8_0_example(F, O, rows, cols, m):          # crates/ferric-tensor/examples/q8_0.rs:10-23
    wf = (np.sin(np.arange(rows * cols, dtype=np.float32) * np.float32(0.021)) * np.float32(0.7)).astype(np.float32)
    check_matmul(F, O, O.quant_q8_0(wf), Q8_0, rows, cols, cosx(m, cols), "q8_0.rs")


def test_golden_gemv_vectors(F, golden):
    x = golden["gemv_x"]
    for name, ty in (("q4k", Q4_K), ("q6k", Q6_K), ("q8_0", Q8_0)):
        qm = F.QMatrix.from_bytes(golden[f"gemv_{name}_w"], ty, 8, 256)
        y = F.Tensor.from_vec(x, (1, 256)).matmul_q(qm).to_vec()
        want = golden[f"gemv_{name}_y64"]
        assert np.abs(y - want).max() / max(1e-3, np.abs(want).max()) < dot_bar(), name
        assert (np.abs(y - want) <= 1e-3 * golden[f"gemv_{name}_wnorm"] * np.linalg.norm(x.astype(np.float64))).all(), name


# ---------------------------------------------------------------- cpu_simd.rs tests against the drop-in host entry

def test_matvec_matches_the_dequantised_reference(F, O):      # cpu_simd.rs:162-173
    for rows, cols in [(1, 32), (8, 64), (17, 256), (64, 512)]:
        raw, vals = O.gen_q8_0_synth(rows, cols, rows * 13 + cols)
        x = ((np.arange(cols) * 37 % 101).astype(np.float32) - 50.0) / np.float32(50.0)
        got = F.matvec_q8_0(x, raw, rows, cols)
        want = (vals.reshape(rows, cols).astype(np.float64) * x).sum(1)
        assert np.abs(got - want).max() / max(1e-6, np.abs(want).max()) < dot_bar()
        cpu = O.matvec_q8_0(x, raw, rows, cols)                # GPU vs the CPU mat-vec itself: fabric_split.rs:54 bar
        assert np.abs(got - cpu).max() / max(1e-6, np.abs(cpu).max()) < max(1e-4, dot_bar())


def test_partitioning_changes_nothing_about_the_answer(F, O):  # cpu_simd.rs:175-200
    raw, _ = O.gen_q8_0_synth(64, 256, 7)
    x = np.sin(np.arange(256, dtype=np.float32) * np.float32(0.01))
    one = F.matvec_q8_0(x, raw, 64, 256)
    for t in (2, 3, 8, 64, 128):
        assert np.array_equal(bits(one), bits(F.matvec_q8_0_threaded(x, raw, 64, 256, t)))
    raw, _ = O.gen_q8_0_synth(40, 128, 3)
    x = (np.arange(128) % 7).astype(np.float32) - 3.0
    whole = F.matvec_q8_0(x, raw, 40, 128)
    for cut in (0, 1, 17, 39, 40):
        joined = np.concatenate([F.matvec_q8_0_span(x, raw, 128, 0, cut), F.matvec_q8_0_span(x, raw, 128, cut, 40)])
        assert np.array_equal(bits(whole), bits(joined)), cut


# ---------------------------------------------------------------- cpu_simd.rs pool_tests (:333-410) against the pooled entry

def test_pooled_matches_the_plain_answer_for_any_pool_size(F, O):     # cpu_simd.rs:349-360, :362-373
    rows, cols = 256, 128
    raw, _ = O.gen_q8_0_synth(rows, cols, 5)
    x = ((np.arange(cols) * 31 % 97).astype(np.float32) - 48.0) / np.float32(48.0)
    want = F.matvec_q8_0(x, raw, rows, cols)
    cpu = O.matvec_q8_0(x, raw, rows, cols)
    assert np.abs(want - cpu).max() / max(1e-6, np.abs(cpu).max()) < 1e-4
    for n in (1, 2, 5, 16):
        pool = F.Pool(n)
        assert pool.threads() == n
        assert np.array_equal(bits(F.matvec_q8_0_pooled(pool, x, raw, cols, 0, rows)), bits(want)), n
    assert F.Pool(0).threads() == 1                                     # Pool::new: n.max(1)


def test_spans_compose_through_the_pool_and_the_weight_is_uploaded_once(F, O):   # cpu_simd.rs:375-387, :389-401
    rows, cols = 128, 64
    raw, _ = O.gen_q8_0_synth(rows, cols, 2)
    x = np.full(cols, -1.25, np.float32)
    pool = F.Pool(4)
    whole = F.matvec_q8_0(x, raw, rows, cols)
    for cut in (0, 1, 63, 127, 128):
        j = np.concatenate([F.matvec_q8_0_pooled(pool, x, raw, cols, 0, cut), F.matvec_q8_0_pooled(pool, x, raw, cols, cut, rows)])
        assert np.array_equal(bits(j), bits(whole)), cut
    first = F.matvec_q8_0_pooled(pool, x, raw, cols, 0, rows)
    for _ in range(20):                                                 # a reused pool does not drift ...
        assert np.array_equal(bits(F.matvec_q8_0_pooled(pool, x, raw, cols, 0, rows)), bits(first))
    assert pool.uploads() == 1                                          # ... and sets up once: the point of a pool
    other, _ = O.gen_q8_0_synth(40, 96, 9)                              # another weight replaces the resident one
    x2 = np.linspace(-1, 1, 96, dtype=np.float32)
    assert np.array_equal(bits(F.matvec_q8_0_pooled(pool, x2, other, 96, 3, 29)), bits(F.matvec_q8_0_span(x2, other, 96, 3, 29)))
    assert pool.uploads() == 2
    changed = raw.copy()
    changed[2:34] ^= 0x55                                               # same shape, new array: keyed by address, so uploaded
    got = F.matvec_q8_0_pooled(pool, x, changed, cols, 0, rows)
    assert pool.uploads() == 3 and np.array_equal(bits(got), bits(F.matvec_q8_0(x, changed, rows, cols)))
    changed[36:68] ^= 0x33                                              # rewritten in place: the caller says so
    pool.forget()
    got = F.matvec_q8_0_pooled(pool, x, changed, cols, 0, rows)
    assert pool.uploads() == 4 and np.array_equal(bits(got), bits(F.matvec_q8_0(x, changed, rows, cols)))
    pool.close()                                                        # cpu_simd.rs:403-409: dropping the pool must not hang


def test_pool_notices_a_weight_rewritten_in_place(F, O):
    # the pool's key is the host pointer, the length and a fingerprint of the bytes: the same buffer with other contents is
    # uploaded again (crates/ferric-tensor/src/cpu_simd.rs:238-331 holds an immutable Arc, so the reference cannot meet this)
    rows, cols = 64, 1024
    w = O.gen_q8_0_synth(rows, cols, 5)[0].copy()
    x = np.cos(np.arange(cols, dtype=np.float32) * np.float32(0.01)).astype(np.float32)
    pool = F.Pool(4)
    y1 = F.matvec_q8_0_pooled(pool, x, w, cols, 0, rows)
    assert pool.uploads() == 1 and np.array_equal(bits(y1), bits(F.matvec_q8_0(x, w, rows, cols)))
    w[:] = O.gen_q8_0_synth(rows, cols, 6)[0]                    # same address, same length, new bytes
    y2 = F.matvec_q8_0_pooled(pool, x, w, cols, 0, rows)
    assert pool.uploads() == 2 and np.array_equal(bits(y2), bits(F.matvec_q8_0(x, w, rows, cols)))
    assert not np.array_equal(bits(y1), bits(y2))
    y3 = F.matvec_q8_0_pooled(pool, x, w, cols, 0, rows)         # unchanged: resident
    assert pool.uploads() == 2 and np.array_equal(bits(y3), bits(y2))


def test_pooled_edge_cases(F, O):
    raw, _ = O.gen_q8_0_synth(8, 64, 1)
    x = np.ones(64, np.float32)
    pool = F.Pool(2)
    assert F.matvec_q8_0_pooled(pool, x, raw, 64, 5, 5).size == 0       # cpu_simd.rs:313
    with pytest.raises(AssertionError, match="empty or inverted span"):  # :311
        F.matvec_q8_0_pooled(pool, x, raw, 64, 6, 5)
    with pytest.raises(AssertionError, match="out of range"):            # the row slice of :321 past the weight
        F.matvec_q8_0_pooled(pool, x, raw, 64, 0, 9)
    with pytest.raises(AssertionError, match="out of range"):            # row_q8_0's activation slice
        F.matvec_q8_0_pooled(pool, x[:40], raw, 64, 0, 8)
    # a longer activation array is fine (only the first cols values are read), and cols / 32 truncates as in row_q8_0
    long_x = np.concatenate([x, np.full(7, 9.0, np.float32)])
    assert np.array_equal(bits(F.matvec_q8_0_pooled(pool, long_x, raw, 64, 0, 8)), bits(F.matvec_q8_0(x, raw, 8, 64)))
    assert not F.matvec_q8_0_pooled(pool, x, raw, 0, 0, 3).any()        # no block: every sum is 0.0


# ---------------------------------------------------------------- benchmark configurations at full size

def test_config1_q8_0_4096(F, O):
    from ferric_amd.synth import synth_weights
    w = synth_weights(Q8_0, 4096, 4096, 0)
    x = np.random.default_rng(0).standard_normal(4096).astype(np.float32)       # seed 0, as the config says
    y = check_matmul(F, O, w, Q8_0, 4096, 4096, x, "C1")
    cpu = O.matmul_cpu(x, w, Q8_0, 4096, 4096, threads=8, direct_q8=True)        # the repo's CPU reference dequant-dot
    assert np.abs(y - cpu).max() / np.abs(cpu).max() < 1e-4


def test_config2_q4_k_5120(F, O):
    from ferric_amd.synth import synth_weights
    w = synth_weights(Q4_K, 5120, 5120, 1)
    x = np.random.default_rng(2).standard_normal(5120).astype(np.float32)
    y = check_matmul(F, O, w, Q4_K, 5120, 5120, x, "C2")
    cpu = O.matmul_cpu(x, w, Q4_K, 5120, 5120, threads=8)
    assert np.abs(y - cpu).max() / np.abs(cpu).max() < 1e-4


@pytest.mark.parametrize("batch", [1, 4, 8])
def test_config3_ffn_block(F, O, batch):
    # gate|up 2 x (5120 -> 17408) Q4_K stacked gate-first, down 17408 -> 5120 Q6_K, SwiGLU between
    from ferric_amd.synth import synth_weights
    n_embd, n_ff = 5120, 17408
    gu = synth_weights(Q4_K, 2 * n_ff, n_embd, 3)
    dn = synth_weights(Q6_K, n_embd, n_ff, 4)
    x = np.random.default_rng(5).standard_normal((batch, n_embd)).astype(np.float32)
    wgu = F.QMatrix.from_bytes(gu, Q4_K, 2 * n_ff, n_embd)
    wdn = F.QMatrix.from_bytes(dn, Q6_K, n_embd, n_ff)
    xt = F.Tensor.from_vec(x, x.shape)
    # stage 1: fused gate/up + SwiGLU vs f64
    h = xt.try_matmul_swiglu(wgu).to_vec().reshape(batch, n_ff)
    g64, wn = O.matmul_f64(x, gu, Q4_K, 2 * n_ff, n_embd)
    g, u = g64[:, :n_ff], g64[:, n_ff:]
    h64 = g / (1.0 + np.exp(-g)) * u
    assert np.abs(h - h64).max() / np.abs(h64).max() < dot_bar()
    # stage 2: down projection of the GPU's own h (so the check isolates the Q6_K matmul)
    y = F.Tensor.from_vec(h, h.shape).matmul_q(wdn).to_vec().reshape(batch, n_embd)
    y64, wn = O.matmul_f64(h, dn, Q6_K, n_embd, n_ff)
    err = np.abs(y - y64)
    assert (err <= 1e-3 * wn[None, :] * np.linalg.norm(h.astype(np.float64), axis=1)[:, None]).all()
    assert err.max() / np.abs(y64).max() < dot_bar()
    # the one-call FFN: the same bits as the two stages on the mat-vec kernel (one or two rows); on the one-pass kernels of
    # wider batches SwiGLU is formed inside the preparation of the down projection's rows, another exp, so the same value
    # to f32 rounding
    y2 = xt.ffn(wgu, wdn).to_vec().reshape(batch, n_embd)
    if batch <= 2:
        assert np.array_equal(bits(y2), bits(y))
    else:
        assert np.abs(y2 - y).max() <= 2e-6 * np.abs(y).max()
        # the one-pass kernels add a cut row's pieces in a fixed order (what a new weight does): the same bits on every run
        assert np.array_equal(bits(xt.ffn(wgu, wdn).to_vec().reshape(batch, n_embd)), bits(y2))
        assert wgu.batch_policy(F.BATCH_F32_MATVEC) == F.BATCH_ORDERED and wdn.batch_policy(F.BATCH_F32_MATVEC) == F.BATCH_ORDERED
        h1 = xt.try_matmul_swiglu(wgu)               # every batch on the mat-vec kernel
        y1 = h1.matmul_q(wdn).to_vec().reshape(batch, n_embd)
        assert np.array_equal(bits(xt.ffn(wgu, wdn).to_vec().reshape(batch, n_embd)), bits(y1))
        assert np.abs(y1 - y64).max() / np.abs(y64).max() < 2 * dot_bar()


# ---------------------------------------------------------------- invariants

@pytest.mark.parametrize("ty,rows,cols", [(Q4_K, 96, 5120), (Q6_K, 70, 2048), (Q8_0, 130, 1024), (Q6_K, 40, 17408)])
def test_batch_rows_are_independent(F, O, ty, rows, cols):
    # On the mat-vec kernel row r of a batch-m result is bit-identical to the batch-1 result for x_r: always when the weight's
    # policy is FHIP_BATCH_F32_MATVEC, and for the one- and two-row batches that take that kernel anyway. Wider batches go to the
    # one-pass matrix-core kernels unless told otherwise: the same values to the accuracy of the two paths, and (the policy a
    # new weight has adds a cut row's pieces in a fixed order) the same bits on every run.
    from ferric_amd.synth import synth_weights
    lib = F._lib.load()
    w = synth_weights(ty, rows, cols, 7)
    qm = F.QMatrix.from_bytes(w, ty, rows, cols)
    x = np.random.default_rng(8).standard_normal((40, cols)).astype(np.float32)
    singles = np.stack([F.Tensor.from_vec(x[i], (1, cols)).matmul_q(qm).to_vec() for i in range(40)])
    wide = 5 if ty == Q8_0 else 3
    for m in (2, 3, 4, 5, 8, 11, 33, 40):          # 33 and 40: more than one group of 32 (Q8_0: 16) rows
        y = check_matmul(F, O, w, ty, rows, cols, x[:m], f"batch {m}")
        if m < wide:
            assert np.array_equal(bits(y), bits(singles[:m])), m
        else:
            assert np.abs(y - singles[:m]).max() <= dot_bar() * np.abs(singles).max(), m
    for m in (3, 8, 33):                            # run to run: the same bits
        xt = F.Tensor.from_vec(x[:m], (m, cols))
        assert np.array_equal(bits(xt.matmul_q(qm).to_vec()), bits(xt.matmul_q(qm).to_vec())), m
    # the policy is the handle's own: another handle on the same bytes keeps what it was made with
    other = F.QMatrix.from_bytes(w, ty, rows, cols)
    assert qm.batch_policy(F.BATCH_F32_MATVEC) == F.BATCH_ORDERED and qm.batch_policy(7) == F.BATCH_F32_MATVEC   # an unknown value only queries
    assert other.batch_policy() == F.BATCH_ORDERED
    for m in (3, 8, 11):
        xt = F.Tensor.from_vec(x[:m], (m, cols))
        assert np.array_equal(bits(xt.matmul_q(qm).to_vec().reshape(m, rows)), bits(singles[:m])), m
    # and what new handles start with can be set for the process; existing handles do not follow
    before = lib.fhip_batch_policy(F.BATCH_F32_MATVEC)
    try:
        assert before == F.BATCH_ORDERED and other.batch_policy() == F.BATCH_ORDERED
        assert F.QMatrix.from_bytes(w, ty, rows, cols).batch_policy() == F.BATCH_F32_MATVEC
    finally:
        lib.fhip_batch_policy(before)


@pytest.mark.parametrize("ty", [Q4_K, Q6_K, Q8_0])
def test_row_partition_invariance_and_odd_shapes(F, O, ty):
    # any split of the output rows gives identical bits (the property QMatrix sharding and the
    # CPU/GPU fabric split rely on: dtype.rs:936-943, cpu_simd.rs:114-122); shapes that do not fill
    # a wave, a workgroup or the grid evenly
    from ferric_amd.synth import synth_weights
    vals, nbytes = O.BLOCK[ty]
    for rows, cols in [(1, 256), (3, 256), (257, 768), (1000, 2304), (33, 8192), (5, 32768 if ty != Q8_0 else 4096)]:
        w = synth_weights(ty, rows, cols, rows)
        x = np.random.default_rng(rows).standard_normal(cols).astype(np.float32)
        whole = check_matmul(F, O, w, ty, rows, cols, x, f"{rows}x{cols}")[0]
        rb = cols // vals * nbytes
        cut = rows // 3
        parts = []
        for lo, hi in ((0, cut), (cut, rows)):
            if hi > lo:
                qm = F.QMatrix.from_bytes(w[lo * rb: hi * rb], ty, hi - lo, cols)
                parts.append(F.Tensor.from_vec(x, (1, cols)).matmul_q(qm).to_vec())
        assert np.array_equal(bits(np.concatenate(parts)), bits(whole))


def test_q8_0_cols_multiple_of_32_only(F, O):
    from ferric_amd.synth import synth_weights
    for rows, cols in [(9, 32), (4, 96), (17, 1056)]:
        w = synth_weights(Q8_0, rows, cols, 3)
        check_matmul(F, O, w, Q8_0, rows, cols, np.random.default_rng(1).standard_normal((3, cols)), f"{rows}x{cols}")


def test_zero_inputs_give_exact_zeros(F, O):
    from ferric_amd.synth import synth_weights
    for ty in (Q4_K, Q6_K, Q8_0):
        w = synth_weights(ty, 64, 1024, 1)
        qm = F.QMatrix.from_bytes(w, ty, 64, 1024)
        y = F.Tensor.from_vec(np.zeros((2, 1024), np.float32), (2, 1024)).matmul_q(qm).to_vec()
        assert not y.any()
        vals, nbytes = O.BLOCK[ty]
        qz = F.QMatrix.from_bytes(np.zeros(64 * 1024 // vals * nbytes, np.uint8), ty, 64, 1024)
        y = F.Tensor.from_vec(np.random.default_rng(0).standard_normal((2, 1024)).astype(np.float32), (2, 1024)).matmul_q(qz).to_vec()
        assert not y.any()


# ---------------------------------------------------------------- fused SwiGLU

@pytest.mark.parametrize("ty", [Q4_K, Q6_K])
@pytest.mark.parametrize("t", [1, 8])
def test_fused_swiglu_matches_unfused(F, O, ty, t):
    # crates/ferric-tensor/examples/ffn_fuse.rs:66-108: n_ff 3072, n_embd 1024, h = cos(0.017 i) * 0.3
    n_ff, n_embd = 3072, 1024
    w = O.gen_kquant_matrix(ty, 2 * n_ff, n_embd)
    qm = F.QMatrix.from_bytes(w, ty, 2 * n_ff, n_embd)
    h = (np.cos(np.arange(t * n_embd, dtype=np.float32) * np.float32(0.017)) * np.float32(0.3)).astype(np.float32).reshape(t, n_embd)
    ht = F.Tensor.from_vec(h, h.shape)
    fused = ht.try_matmul_swiglu(qm).to_vec()
    unfused = ht.matmul_q(qm).swiglu(n_ff).to_vec()
    scale = max(1e-3, np.abs(unfused).max())
    assert np.abs(fused - unfused).max() / scale < 1e-5   # the same dot products, fused or not
    g64, _ = O.matmul_f64(h, w, ty, 2 * n_ff, n_embd)
    want = (g64[:, :n_ff] / (1 + np.exp(-g64[:, :n_ff])) * g64[:, n_ff:]).reshape(-1)
    assert np.abs(fused - want).max() / max(1e-3, np.abs(want).max()) < dot_bar()
    assert np.abs(O.swiglu(ht.matmul_q(qm).to_vec().reshape(t, -1), n_ff).reshape(-1) - unfused).max() / scale < 1e-6


def test_swiglu_unsupported_for_q8_0(F, O):
    from ferric_amd.synth import synth_weights
    qm = F.QMatrix.from_bytes(synth_weights(Q8_0, 64, 256, 1), Q8_0, 64, 256)
    x = F.Tensor.from_vec(np.ones((1, 256), np.float32), (1, 256))
    assert x.try_matmul_swiglu(qm) is None                                  # dtype.rs:949-959 returns None -> caller un-fuses
    y = x.matmul_q(qm).swiglu(32).to_vec()
    assert y.shape == (32,)


# ---------------------------------------------------------------- error behaviour of the boundary

def test_constructor_errors_match_the_reference(F):
    z = np.zeros(144 * 4, np.uint8)
    with pytest.raises(ValueError, match="no native matmul for ggml type 10"):         # dtype.rs:855 (Q2_K)
        F.QMatrix.from_bytes(z, 10, 1, 256)
    with pytest.raises(AssertionError, match="Q4_K cols must be a multiple of 256"):    # dtype.rs:1389
        F.Q4_KWeights.from_bytes(z, 1, 300)
    with pytest.raises(AssertionError, match="unexpected Q4_K byte length"):            # dtype.rs:1390
        F.Q4_KWeights.from_bytes(z, 5, 256)
    with pytest.raises(AssertionError, match="Q6_K cols must be a multiple of 256"):    # dtype.rs:1148
        F.Q6_KWeights.from_bytes(z, 1, 128)
    with pytest.raises(AssertionError, match="unexpected Q8_0 byte length"):            # dtype.rs:1272
        F.Q8_0Weights.from_bytes(z, 2, 64)
    qm = F.Q4_KWeights.from_bytes(z, 4, 256)
    with pytest.raises(AssertionError, match="inner dim mismatch"):                     # dtype.rs:1429
        F.Tensor.from_vec(np.zeros(512, np.float32), (1, 512)).matmul_q(qm)
    with pytest.raises(AssertionError):                                                 # cpu_simd.rs:80-83
        F.matvec_q8_0(np.zeros(33, np.float32), np.zeros(34, np.uint8), 1, 33)
    with pytest.raises(AssertionError, match="unexpected Q8_0 byte length"):
        F.matvec_q8_0(np.zeros(32, np.float32), np.zeros(35, np.uint8), 1, 32)


def test_empty_shapes(F):
    qm = F.QMatrix.from_bytes(np.zeros(0, np.uint8), Q4_K, 0, 256)
    assert F.Tensor.from_vec(np.zeros(256, np.float32), (1, 256)).matmul_q(qm).to_vec().size == 0
    qm = F.QMatrix.from_bytes(np.zeros(144 * 3, np.uint8), Q4_K, 3, 256)
    assert F.Tensor.from_vec(np.zeros(0, np.float32), (0, 256)).matmul_q(qm).to_vec().size == 0
    assert F.matvec_q8_0(np.zeros(0, np.float32), np.zeros(0, np.uint8), 0, 0).size == 0
    y = F.matvec_q8_0(np.zeros(0, np.float32), np.zeros(0, np.uint8), 5, 0)
    assert y.shape == (5,) and not y.any()
    # a weight without columns: every dot product is the empty sum, on every entry point that takes the weight
    lib, check = F._lib.load(), F._lib.check
    qm = F.QMatrix.from_bytes(np.zeros(0, np.uint8), Q4_K, 7, 0)
    yt = F.Tensor.from_vec(np.full((3, 7), 5.0, np.float32), (3, 7))
    dummy = F.Tensor.empty((1, 64))
    for call in (lambda: lib.fhip_matmul_q(qm.handle, dummy.buf.ptr, 3, yt.buf.ptr, None),
                 lambda: lib.fhip_gemm_q_bf16(qm.handle, dummy.buf.ptr, 3, yt.buf.ptr, None),
                 lambda: lib.fhip_matmul_q_coop(qm.handle, dummy.buf.ptr, 3, yt.buf.ptr, dummy.buf.ptr, None)):
        check(lib.fhip_memset(yt.buf.ptr, 0x41, 3 * 7 * 4, None))
        check(call())
        assert not yt.to_vec().any()


# ---------------------------------------------------------------- activations block fixed point cannot hold

@pytest.mark.parametrize("ty", [Q8_0, Q4_K, Q6_K, 13, 2, 3, 6, 7, 20, 23, 39],
                         ids=["q8_0", "q4_k", "q6_k", "q5_k", "q4_0", "q4_1", "q5_0", "q5_1", "iq4_nl", "iq4_xs", "mxfp4"])
def test_non_finite_and_tiny_activations_give_what_the_f32_dot_gives(F, O, ty):
    """crates/ferric-tensor/src/cpu_simd.rs:57-72 and the dequantize-then-dot path sum x[k] * w[k] in f32: a NaN activation
    makes the row NaN, an infinite one +-inf by the weight's sign (NaN against a zero weight, NaN when both signs meet), and
    neither leaks into the other rows of a batch. Runs of activations far below the f32 normal range's middle still count."""
    from ferric_amd.synth import synth_weights
    rows, cols = 96, 2048
    raw = synth_weights(ty, rows, cols, 21).copy()
    if ty == Q4_K:                                    # dmin = 0: no min term to carry the NaN by accident
        raw.reshape(-1, 144)[:, 2:4] = 0
        raw.reshape(-1, 144)[::3, 16:24] = 0          # and some exactly-zero weights under the infinite activation
    rng = np.random.default_rng(22)
    x = rng.standard_normal((6, cols)).astype(np.float32)
    x[0, 1000] = np.nan
    x[1, 37] = np.inf
    x[2, 37] = -np.inf
    x[2, 1999] = np.inf
    x[3, 512:640] *= np.float32(1e-36)                # four runs near the bottom of the normal range
    x[4, 0:32] = np.float32(1e30)                     # a run above 2^96: 128 times its sum is near the end of the f32 range
    # row 5 stays ordinary
    qm = F.QMatrix.from_bytes(raw, ty, rows, cols)
    with np.errstate(all="ignore"):
        want = O.matmul_cpu(x, raw, ty, rows, cols)
        y64, wn = O.matmul_f64(x, raw, ty, rows, cols)
    lib = F._lib.load()
    wide = 5 if ty == Q8_0 else 3                      # from this many rows on a batch takes the one-pass matrix-core kernels
    for policy in (0, 1):
        before = qm.batch_policy(policy)
        try:
            for sl in (slice(0, 6), slice(0, 1), slice(1, 3), slice(2, 6)):      # batches of 6, 1, 2, 4 rows: every pass width
                xs = x[sl]
                y = F.Tensor.from_vec(xs, xs.shape).matmul_q(qm).to_vec().reshape(xs.shape[0], rows)
                w_, y_ = want[sl], y64[sl]
                with np.errstate(all="ignore"):
                    bound = 1e-3 * wn[None, :] * np.linalg.norm(xs.astype(np.float64), axis=1)[:, None]
                one_pass = policy == 0 and xs.shape[0] >= wide and ty in (Q8_0, Q4_K, Q6_K, 13)
                for i, r in enumerate(range(sl.start, sl.stop)):
                    fin = np.isfinite(w_[i])
                    if one_pass and not np.isfinite(xs[i]).all():
                        # the matrix-core kernels scale a row's chunks by their largest magnitudes, and a non-finite operand
                        # meets every weight row: the whole output row is non-finite
                        assert not np.isfinite(y[i]).any(), (ty, r)
                        continue
                    assert np.array_equal(np.isnan(y[i]), np.isnan(w_[i])), (ty, r)
                    assert np.array_equal(np.isposinf(y[i]), np.isposinf(w_[i])) and np.array_equal(np.isneginf(y[i]), np.isneginf(w_[i])), (ty, r)
                    assert (np.abs(y[i] - y_[i])[fin] <= bound[i][fin] + 1e-30).all(), (ty, r)
        finally:
            qm.batch_policy(before)
    assert np.isnan(want[0]).all() and not np.isfinite(want[1]).any() and np.isfinite(want[3:6]).all()


# ---------------------------------------------------------------- the library's workspace behind the batched drop-in calls

def test_batched_calls_inside_a_graph_need_the_workspace_reserved(F, O):
    """A batch of three rows or more keeps its prepared activations in a workspace the library owns per stream; a capturing
    stream cannot allocate, so the call says how much to reserve, and after fhip_workspace_reserve the captured FFN block
    replays to the eager result."""
    import ctypes as C
    from ferric_amd.synth import synth_weights
    lib, check = F._lib.load(), F._lib.check
    n_embd, n_ff, batch = 1024, 3072, 8
    gu = F.QMatrix.from_bytes(synth_weights(Q4_K, 2 * n_ff, n_embd, 31), Q4_K, 2 * n_ff, n_embd)
    dn = F.QMatrix.from_bytes(synth_weights(Q6_K, n_embd, n_ff, 32), Q6_K, n_embd, n_ff)
    x = np.random.default_rng(33).standard_normal((batch, n_embd)).astype(np.float32)
    xt = F.Tensor.from_vec(x, x.shape)
    y, ws = F.Tensor.empty((batch, n_embd)), F.Tensor.empty((batch, n_ff))
    need = lib.fhip_workspace_bytes(gu.handle, dn.handle, batch)
    assert need > 0 and lib.fhip_workspace_bytes(gu.handle, dn.handle, 2) == 0      # two rows: the mat-vec kernel, no workspace
    stream = F.Stream()
    g = F.Graph.begin(stream)
    rc = lib.fhip_ffn(gu.handle, dn.handle, xt.buf.ptr, batch, y.buf.ptr, ws.buf.ptr, stream.handle)
    msg = F._lib.last_error()
    g.end()                                                                           # an empty graph; nothing was enqueued
    assert rc == F._lib.ERR_ARG and "fhip_workspace_reserve" in msg and str(need) in msg
    check(lib.fhip_workspace_reserve(stream.handle, need))
    check(lib.fhip_ffn(gu.handle, dn.handle, xt.buf.ptr, batch, y.buf.ptr, ws.buf.ptr, stream.handle))
    eager = y.to_vec(stream).copy()
    g = F.Graph.begin(stream)
    check(lib.fhip_ffn(gu.handle, dn.handle, xt.buf.ptr, batch, y.buf.ptr, ws.buf.ptr, stream.handle))
    g.end()
    for _ in range(3):
        check(lib.fhip_memset(y.buf.ptr, 0xFF, batch * n_embd * 4, stream.handle))
        g.launch()
        # (a weight row whose columns are shared out over several workgroups is summed with f32 atomic adds: the order, and
        # so the last bits, vary from run to run)
        assert np.abs(y.to_vec(stream) - eager).max() <= 2e-6 * np.abs(eager).max()
    # the result is the FFN block (held to the oracle through the two stages)
    g64, _ = O.matmul_f64(x, synth_weights(Q4_K, 2 * n_ff, n_embd, 31), Q4_K, 2 * n_ff, n_embd)
    h64 = g64[:, :n_ff] / (1.0 + np.exp(-g64[:, :n_ff])) * g64[:, n_ff:]
    y64, _ = O.matmul_f64(h64.astype(np.float32), synth_weights(Q6_K, n_embd, n_ff, 32), Q6_K, n_embd, n_ff)
    assert np.abs(eager.reshape(batch, n_embd) - y64).max() <= 2e-5 * np.abs(y64).max()
    lib.fhip_workspace_release(stream.handle)                                         # and a released workspace comes back on demand
    check(lib.fhip_ffn(gu.handle, dn.handle, xt.buf.ptr, batch, y.buf.ptr, ws.buf.ptr, stream.handle))
    assert np.abs(y.to_vec(stream) - eager).max() <= 2e-6 * np.abs(eager).max()
