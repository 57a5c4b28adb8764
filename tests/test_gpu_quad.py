"""Batches of three and four rows on the kernel that multiplies through the 4 x 4 x 4 int8 matrix instruction
(gemv_quad.hip) against the dot-product mat-vec it restates: the two must give the same bits for every row, whatever the
batch a row sits in (the reference's CPU rows do not depend on their neighbours, crates/ferric-tensor/src/cpu_simd.rs:175-200),
and both are held to the oracle by the tests of the entry points they sit behind."""
import numpy as np
import pytest

from conftest import bits, dot_bar

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("precision")]
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14


def both(F, fn):
    """fn() with the quad kernel on, then off (every batch on the dot-product kernel, two rows a pass)."""
    lib = F._lib.load()
    on = fn()
    before = lib.fhip_debug_quad_matvec(0)
    try:
        off = fn()
    finally:
        lib.fhip_debug_quad_matvec(before)
    return on, off


# rows x cols: one group of units and several, a last group that is partly filled (2304 = 36 units), rows that end inside a
# quad and inside a workgroup's share, fewer rows than the chip has workgroups, rows long enough for a second pass (17408 columns),
# for three and four passes (28672, 31488 with a partly filled last group, 32768: the longest rows the mat-vec entry points take)
SHAPES = [(Q4_K, 96, 5120), (Q4_K, 1023, 256), (Q4_K, 7, 2304), (Q4_K, 2050, 1024), (Q4_K, 300, 17408), (Q4_K, 5120, 5120),
          (Q6_K, 70, 2048), (Q6_K, 40, 17408), (Q6_K, 1, 256), (Q6_K, 1500, 2304), (Q6_K, 5120, 5120), (Q6_K, 515, 11264),
          (Q4_K, 37, 28672), (Q4_K, 12, 31488), (Q6_K, 9, 32768), (Q6_K, 261, 28672),
          (Q5_K, 96, 5120), (Q5_K, 7, 2304), (Q5_K, 5120, 5120), (Q5_K, 130, 17408), (Q5_K, 1023, 256),
          (Q8_0, 4096, 4096), (Q8_0, 130, 1024), (Q8_0, 33, 96), (Q8_0, 12288, 4096), (Q8_0, 1000, 5120), (Q8_0, 77, 32)]


@pytest.mark.parametrize("ty,rows,cols", SHAPES)
def test_same_bits_as_the_dot_product_kernel(F, O, ty, rows, cols):
    from ferric_amd.synth import synth_weights
    w = synth_weights(ty, rows, cols, rows + cols)
    qm = F.QMatrix.from_bytes(w, ty, rows, cols)
    qm.batch_policy(F.BATCH_F32_MATVEC)
    x = np.random.default_rng(cols).standard_normal((9, cols)).astype(np.float32)
    x[1] *= np.float32(300.0)
    x[2, ::7] = 0
    singles = np.stack([F.Tensor.from_vec(x[i], (1, cols)).matmul_q(qm).to_vec() for i in range(9)])
    for m in (3, 4, 7, 8, 9):
        xt = F.Tensor.from_vec(x[:m], (m, cols))
        on, off = both(F, lambda: xt.matmul_q(qm).to_vec().reshape(m, rows))
        assert np.array_equal(bits(on), bits(singles[:m])), (m, "quad against single rows")
        if cols <= 17408:       # (two rows of longer columns do not fit the streaming kernel's LDS: pairs then take the f32 kernel)
            assert np.array_equal(bits(on), bits(off)), (m, "quad against pairs")
    # against f64 on the exactly dequantised weights: the north-star bound everywhere, the bar of the precision under test
    # where a row is long enough for it to be about sums (a single 256-column row at 16 bits is about one run's rounding)
    y64, wn = O.matmul_f64(x[:4], w, ty, rows, cols)
    y = F.Tensor.from_vec(x[:4], (4, cols)).matmul_q(qm).to_vec().reshape(4, rows)
    assert (np.abs(y - y64) <= 1e-3 * wn[None, :] * np.linalg.norm(x[:4].astype(np.float64), axis=1)[:, None] + 1e-30).all()
    if rows >= 64 and cols >= 1024:
        assert np.abs(y - y64).max() / max(1e-3, np.abs(y64).max()) < dot_bar()


@pytest.mark.parametrize("ty,n_ff,cols", [(Q4_K, 1024, 1024), (Q4_K, 333, 2304), (Q6_K, 96, 512), (Q4_K, 17408, 5120), (Q5_K, 500, 1536)])
def test_fused_swiglu_same_bits(F, O, ty, n_ff, cols):
    from ferric_amd.synth import synth_weights
    gu = synth_weights(ty, 2 * n_ff, cols, 5)
    qm = F.QMatrix.from_bytes(gu, ty, 2 * n_ff, cols)
    qm.batch_policy(F.BATCH_F32_MATVEC)
    x = np.random.default_rng(6).standard_normal((4, cols)).astype(np.float32)
    singles = np.stack([F.Tensor.from_vec(x[i], (1, cols)).try_matmul_swiglu(qm).to_vec() for i in range(4)])
    for m in (3, 4):
        xt = F.Tensor.from_vec(x[:m], (m, cols))
        on, off = both(F, lambda: xt.try_matmul_swiglu(qm).to_vec().reshape(m, n_ff))
        assert np.array_equal(bits(on), bits(off)) and np.array_equal(bits(on), bits(singles[:m])), m


@pytest.mark.parametrize("ty", [Q8_0, Q4_K, Q5_K, Q6_K])
def test_runs_block_fixed_point_cannot_hold(F, O, ty):
    """Non-finite activations and runs at the ends of the f32 range take the element-by-element pass: the same bits as on
    the dot-product kernel there too, NaN for NaN."""
    from ferric_amd.synth import synth_weights
    rows, cols = 96, 2048
    w = synth_weights(ty, rows, cols, 21)
    qm = F.QMatrix.from_bytes(w, ty, rows, cols)
    qm.batch_policy(F.BATCH_F32_MATVEC)
    x = np.random.default_rng(22).standard_normal((4, cols)).astype(np.float32)
    x[0, 1000] = np.nan
    x[1, 37] = np.inf
    x[1, 1999] = -np.inf
    x[2, 512:640] *= np.float32(1e-36)
    x[3, 0:32] = np.float32(1e30)
    xt = F.Tensor.from_vec(x, x.shape)
    on = xt.matmul_q(qm).to_vec().reshape(4, rows)
    # (row by row: in a two-row pass of the dot-product kernel a unit goes element by element for both rows when either needs it)
    singles = np.stack([F.Tensor.from_vec(x[i], (1, cols)).matmul_q(qm).to_vec() for i in range(4)])
    assert np.array_equal(np.isnan(on), np.isnan(singles))
    ok = ~np.isnan(on)
    assert np.array_equal(bits(on)[ok], bits(singles)[ok])
    assert np.isnan(on[0]).all() and np.isfinite(on[2:]).all()
