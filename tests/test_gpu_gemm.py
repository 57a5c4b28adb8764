"""Prefill dequant-GEMM (bf16 activations, matrix cores) vs the CPU oracle, through the C ABI.

Three bars:
  * against the SAME arithmetic model evaluated in f64 -- activations as given (bf16), weights =
    oracle-dequantized f32 rounded to bf16 (RNE) -- the GPU may differ only by f32 accumulation order:
    max|d| / max|ref| < 2e-5. This is the check that catches a wrong lane/column mapping.
  * the north-star bound |y - y64| <= 1e-3 * ||w_row|| * ||x_t|| against unrounded oracle weights;
  * the reference's own bar for its matrix-unit prefill: max|d| / max|ref| < 6e-2
    (crates/ferric-tensor/examples/coop_q4_k.rs:38).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q6_K, Q5_K = 8, 12, 14, 13


def bf16_round(a):
    """f32 -> nearest bf16 (ties to even), returned as (bits uint16, value f32)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32)
    return r.astype(np.uint16), (r << 16).astype(np.uint32).view(np.float32)


def run_case(F, O, ty, t, n, k, seed, gen=None):
    from ferric_amd.synth import synth_weights
    w = gen(ty, n, k) if gen else synth_weights(ty, n, k, seed)
    x = np.random.default_rng(seed + 1).standard_normal((t, k)).astype(np.float32)
    xb, xv = bf16_round(x)
    qm = F.QMatrix.from_bytes(w, ty, n, k)
    y = F.Tensor.from_bf16_bits(xb, (t, k)).gemm_q_bf16(qm).to_vec().reshape(t, n)
    wd = O.deq_raw(w, n * k, ty).reshape(n, k)
    _, wb = bf16_round(wd)
    x64 = xv.astype(np.float64)
    model = x64 @ wb.astype(np.float64).T
    scale = max(1e-3, np.abs(model).max())
    assert np.abs(y - model).max() / scale < 2e-5, (ty, t, n, k)
    exact = x64 @ wd.astype(np.float64).T
    bound = 1e-3 * np.linalg.norm(wd.astype(np.float64), axis=1)[None, :] * np.linalg.norm(x64, axis=1)[:, None]
    assert (np.abs(y - exact) <= bound).all(), (ty, t, n, k)
    assert np.abs(y - exact).max() / max(1e-3, np.abs(exact).max()) < 6e-2
    return y


@pytest.mark.parametrize("ty", [Q4_K, Q6_K, Q8_0, Q5_K])
def test_small_and_ragged_shapes(F, O, ty):
    for i, (t, n, k) in enumerate([(1, 32, 256), (8, 256, 256), (33, 100, 512), (64, 96, 768), (100, 300, 1024), (130, 257, 2048)]):
        run_case(F, O, ty, t, n, k, 10 + i)


def test_seeded_random_shapes(F, O):
    # 48 shapes drawn with a fixed seed: any row count on either side of the 32-row kernel switch, output widths that are
    # no multiple of a tile (or of 4: the ordered sum of K-split tiles then stores element by element), 1 to 9 chunks of
    # K -- whatever way the launch is cut, every output meets the oracle
    rng = np.random.default_rng(20240607)
    for i in range(48):
        ty = (Q4_K, Q6_K, Q8_0, Q5_K)[i % 4] if i >= 36 else (Q4_K, Q6_K, Q8_0)[i % 3]
        t = int(rng.integers(1, 300)) if i % 4 else int(rng.integers(1, 33))
        n = int(rng.integers(1, 700))
        k = int(rng.integers(1, 10)) * 256 if ty != Q8_0 else int(rng.integers(1, 73)) * 32
        run_case(F, O, ty, t, n, k, 1000 + i)


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5, 6])
def test_every_tile_on_ragged_shapes(F, O, tile):
    # The launcher picks one of seven workgroup tiles by estimate; here each is pinned in turn (64 / 128 / 256 rows x 256
    # outputs, 256 x 160, 128 / 64 rows x 128, 128 x 160) and run on shapes that fill no tile: rows and outputs that end inside a tile, outputs that are no
    # multiple of 4, launches with whole rounds of tiles and a cut remainder, launches where every tile is cut along K.
    lib = F._lib.load()
    before = lib.fhip_debug_gemm_tile(tile)
    try:
        shapes = [(Q4_K, 33, 100, 512), (Q4_K, 300, 4001, 1024), (Q6_K, 130, 257, 2048), (Q8_0, 70, 1283, 1184), (Q4_K, 520, 7000, 768),
                  (Q6_K, 257, 161, 256), (Q8_0, 1025, 330, 96), (Q5_K, 300, 1283, 1024), (Q5_K, 70, 161, 2048)]
        for i, (ty, t, n, k) in enumerate(shapes):
            run_case(F, O, ty, t, n, k, 300 + 10 * tile + i)
    finally:
        lib.fhip_debug_gemm_tile(before)


def test_reference_coop_example_shapes(F, O):
    # crates/ferric-tensor/examples/coop_q4_k.rs: reference-generator weights, M a multiple of 8 and not
    run_case(F, O, Q4_K, 16, 64, 512, 3, gen=O.gen_kquant_matrix)
    run_case(F, O, Q4_K, 13, 128, 1024, 4, gen=O.gen_kquant_matrix)
    run_case(F, O, Q6_K, 24, 64, 512, 5, gen=O.gen_kquant_matrix)


@pytest.mark.parametrize("t", [128, 512, 2048])
def test_config4_prefill_5120(F, O, t):
    # W 5120x5120 Q4_K, X [t, 5120] bf16 ~ N(0,1), f32 out
    run_case(F, O, Q4_K, t, 5120, 5120, 21)


@pytest.mark.parametrize("ty,t,n,k", [(Q4_K, 2048, 34816, 5120), (Q6_K, 512, 5120, 17408), (Q8_0, 2048, 4096, 4096)])
def test_the_layer_s_large_projections_on_sampled_outputs(F, O, ty, t, n, k):
    # The fused gate|up weight at 2048 rows is four whole rounds of 256 x 256 tiles and a remainder cut in four, the down
    # projection at 512 rows 256 x 160 tiles each cut in four, Q8_0 4096 x 4096 a grid of 208 whole 256 x 160 tiles. Too large for
    # the f64 model in full: 384 weight rows spread over the first, the last and random tiles, every activation row.
    from ferric_amd.synth import synth_weights
    w = synth_weights(ty, n, k, 71)
    x = np.random.default_rng(72).standard_normal((t, k)).astype(np.float32)
    xb, xv = bf16_round(x)
    qm = F.QMatrix.from_bytes(w, ty, n, k)
    y = F.Tensor.from_bf16_bits(xb, (t, k)).gemm_q_bf16(qm).to_vec().reshape(t, n)
    rows = np.unique(np.concatenate([np.arange(64), np.arange(n - 64, n), np.random.default_rng(73).integers(0, n, 256)]))
    rb = len(w) // n
    wd = O.deq_raw(np.ascontiguousarray(w.reshape(n, rb)[rows]).reshape(-1), len(rows) * k, ty).reshape(len(rows), k)
    _, wb = bf16_round(wd)
    model = xv.astype(np.float64) @ wb.astype(np.float64).T
    got = y[:, rows]
    assert np.abs(got - model).max() / np.abs(model).max() < 2e-5
    exact = xv.astype(np.float64) @ wd.astype(np.float64).T
    bound = 1e-3 * np.linalg.norm(wd.astype(np.float64), axis=1)[None, :] * np.linalg.norm(xv.astype(np.float64), axis=1)[:, None]
    assert (np.abs(got - exact) <= bound).all()


def test_prefill_other_formats_at_size(F, O):
    run_case(F, O, Q5_K, 512, 5120, 5120, 24)
    run_case(F, O, Q6_K, 256, 5120, 5120, 22)
    run_case(F, O, Q8_0, 256, 4096, 4096, 23)


def test_rows_are_independent_of_the_batch(F, O):
    # A row of a T-row prefill is bit-identical to the same row computed in a smaller batch, as long as
    # both launches have enough output tiles to run without splitting K (a K split changes where the sum over K is cut,
    # so across batch sizes only the tolerance holds there, not bit equality).
    from ferric_amd.synth import synth_weights
    w = synth_weights(Q4_K, 5120, 512, 5)
    qm = F.QMatrix.from_bytes(w, Q4_K, 5120, 512)
    x = np.random.default_rng(1).standard_normal((1536, 512)).astype(np.float32)
    xb, _ = bf16_round(x)
    # 1536 and 1280 rows: 240 and 200 tiles of 128 x 256, each computed whole by one workgroup
    big = F.Tensor.from_bf16_bits(xb, (1536, 512)).gemm_q_bf16(qm).to_vec().reshape(1536, 5120)
    part = F.Tensor.from_bf16_bits(xb[256:], (1280, 512)).gemm_q_bf16(qm).to_vec().reshape(1280, 5120)
    assert np.array_equal(big[256:].view(np.uint32), part.view(np.uint32))
    again = F.Tensor.from_bf16_bits(xb, (1536, 512)).gemm_q_bf16(qm).to_vec().reshape(1536, 5120)
    assert np.array_equal(big.view(np.uint32), again.view(np.uint32))


@pytest.mark.parametrize("ty,t,n,k", [(Q4_K, 128, 5120, 5120), (Q4_K, 512, 5120, 5120), (Q4_K, 2048, 9216, 5120),
                                      (Q6_K, 300, 1000, 4096), (Q8_0, 200, 1300, 2080), (Q4_K, 70, 3000, 8192),
                                      (Q4_K, 8, 5120, 5120), (Q6_K, 20, 1000, 4096), (Q8_0, 3, 1300, 2080), (Q4_K, 32, 1024, 5120),
                                      (Q5_K, 256, 5120, 5120), (Q5_K, 9, 3000, 2048)])
def test_two_runs_give_identical_bits(F, O, ty, t, n, k):
    # Launches with fewer whole tiles than the chip has workgroups cut tiles along K (every shape here does; 2048 x 9216
    # has a cut remainder behind whole tiles; up to 32 rows it is groups of 128 outputs that are cut). The partial tiles are
    # summed in a fixed order, so the bits may not depend on which workgroup finishes first: five runs, with other work on
    # the device in between, one result.
    from ferric_amd.synth import synth_weights
    lib = F._lib.load()
    w = synth_weights(ty, n, k, 31)
    qm = F.QMatrix.from_bytes(w, ty, n, k)
    assert lib.fhip_workspace_bytes_coop(qm.handle, None, t) > 0, "the case is meant to cut tiles along K"
    xb, _ = bf16_round(np.random.default_rng(32).standard_normal((t, k)).astype(np.float32))
    x = F.Tensor.from_bf16_bits(xb, (t, k))
    first = x.gemm_q_bf16(qm).to_vec().view(np.uint32)
    other = F.QMatrix.from_bytes(synth_weights(Q4_K, 512, 1024, 33), Q4_K, 512, 1024)
    xo = F.Tensor.from_bf16_bits(bf16_round(np.ones((40, 1024), np.float32))[0], (40, 1024))
    for _ in range(4):
        xo.gemm_q_bf16(other)              # another launch that uses the same workspace
        assert np.array_equal(first, x.gemm_q_bf16(qm).to_vec().view(np.uint32))


def test_q8_0_rows_ending_inside_a_chunk(F, O):
    # Q8_0 rows are any multiple of 32 long; the kernel walks 256-column chunks, so 32..224 trailing columns
    # exercise the zero-scale / zero-activation padding of the last chunk (and K < 256 has no full chunk at all)
    for i, (t, n, k) in enumerate([(3, 40, 32), (9, 64, 96), (40, 130, 288), (130, 70, 480), (70, 257, 1184)]):
        run_case(F, O, Q8_0, t, n, k, 40 + i)


def test_coop_entry_takes_f32_activations(F, O):
    # dtype.rs:1818 matmul_q4_k_coop reads f32 x; here x is rounded to bf16 (RNE) on the device first. The
    # rounding is checked bit for bit, the product against the bf16 entry point fed host-rounded activations
    # (equal up to the order in which K slices are added when the launch splits K).
    from ferric_amd.synth import synth_weights
    for ty, name, (t, n, k) in [(Q4_K, "matmul_q4_k_coop", (8, 512, 1024)), (Q6_K, "matmul_q6_k_coop", (4, 256, 512)),
                                (Q8_0, "matmul_q8_0_coop", (21, 264, 416)), (Q4_K, "matmul_q4_k_coop", (150, 384, 768)),
                                (Q5_K, "matmul_q5_k_coop", (12, 256, 1024)), (Q5_K, "matmul_q5_k_coop", (150, 384, 768))]:
        w = synth_weights(ty, n, k, 60)
        qm = F.QMatrix.from_bytes(w, ty, n, k)
        x = (np.random.default_rng(61).standard_normal((t, k)) * 3).astype(np.float32)
        x[0, :4] = [0.0, -0.0, 1.00390625, 1.01171875]   # exact ties, to even both ways
        xb, _ = bf16_round(x)
        xt = F.Tensor.from_vec(x.reshape(-1), (t, k))
        assert np.array_equal(xt.cvt_bf16().to_vec().reshape(t, k), xb)
        want = F.Tensor.from_bf16_bits(xb, (t, k)).gemm_q_bf16(qm).to_vec()
        got = getattr(xt, name)(qm).to_vec()
        assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max(), name
    odd = np.arange(13, dtype=np.float32) * 1.001      # a length that is not a multiple of 8: the scalar tail
    odd[:5] = [3.0e38, -3.3895314e38, 1e-40, -65280.0, np.inf]   # near and past the largest bf16, a denormal
    assert np.array_equal(F.Tensor.from_vec(odd, (1, 13)).cvt_bf16().to_vec(), bf16_round(odd)[0])
    with pytest.raises(AssertionError, match="multiple of 8"):
        qm = F.QMatrix.from_bytes(synth_weights(Q4_K, 12, 256, 1), Q4_K, 12, 256)
        F.Tensor.from_vec(np.zeros(256, np.float32), (1, 256)).matmul_q4_k_coop(qm)


def test_batched_decode_ffn_on_the_matrix_cores(F, O):
    # FFN block at batch 4 and 8 through the coop entry points: gate_up -> swiglu -> down, against f64 on
    # oracle-dequantized weights, to the north-star bound applied to each matmul
    from ferric_amd.synth import synth_weights
    d, n_ff = 1024, 2816
    gu = synth_weights(Q4_K, 2 * n_ff, d, 70)
    dn = synth_weights(Q6_K, d, n_ff, 71)
    qgu, qdn = F.QMatrix.from_bytes(gu, Q4_K, 2 * n_ff, d), F.QMatrix.from_bytes(dn, Q6_K, d, n_ff)
    wgu = O.deq_raw(gu, 2 * n_ff * d, Q4_K).reshape(2 * n_ff, d).astype(np.float64)
    wdn = O.deq_raw(dn, d * n_ff, Q6_K).reshape(d, n_ff).astype(np.float64)
    for b in (4, 8):
        x = np.random.default_rng(72 + b).standard_normal((b, d)).astype(np.float32)
        g = F.Tensor.from_vec(x.reshape(-1), (b, d)).matmul_q4_k_coop(qgu)
        g64 = x.astype(np.float64) @ wgu.T
        bound = 1e-3 * np.linalg.norm(wgu, axis=1)[None, :] * np.linalg.norm(x.astype(np.float64), axis=1)[:, None]
        assert (np.abs(g.to_vec().reshape(b, -1) - g64) <= bound).all()
        hid = g.swiglu(n_ff)
        hv = hid.to_vec().reshape(b, n_ff)
        y = hid.matmul_q6_k_coop(qdn).to_vec().reshape(b, d)
        y64 = hv.astype(np.float64) @ wdn.T
        bound = 1e-3 * np.linalg.norm(wdn, axis=1)[None, :] * np.linalg.norm(hv.astype(np.float64), axis=1)[:, None]
        assert (np.abs(y - y64) <= bound).all()
        # the one-call block does the same steps (the SwiGLU output is rounded to bf16 either way)
        y1 = F.Tensor.from_vec(x.reshape(-1), (b, d)).ffn_coop(qgu, qdn).to_vec().reshape(b, d)
        assert np.abs(y1 - y).max() <= 2e-5 * np.abs(y).max()


def test_gemm_errors(F):
    qm = F.QMatrix.from_bytes(np.zeros(144, np.uint8), Q4_K, 1, 256)
    with pytest.raises(AssertionError, match="inner dim mismatch"):
        F.Tensor.from_bf16_bits(np.zeros(512, np.uint16), (1, 512)).gemm_q_bf16(qm)
    assert F.Tensor.from_bf16_bits(np.zeros(0, np.uint16), (0, 256)).gemm_q_bf16(qm).to_vec().size == 0
