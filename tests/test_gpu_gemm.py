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
Q8_0, Q4_K, Q6_K = 8, 12, 14


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


@pytest.mark.parametrize("ty", [Q4_K, Q6_K, Q8_0])
def test_small_and_ragged_shapes(F, O, ty):
    for i, (t, n, k) in enumerate([(1, 32, 256), (8, 256, 256), (33, 100, 512), (64, 96, 768), (100, 300, 1024), (130, 257, 2048)]):
        run_case(F, O, ty, t, n, k, 10 + i)


def test_reference_coop_example_shapes(F, O):
    # crates/ferric-tensor/examples/coop_q4_k.rs: reference-generator weights, M a multiple of 8 and not
    run_case(F, O, Q4_K, 16, 64, 512, 3, gen=O.gen_kquant_matrix)
    run_case(F, O, Q4_K, 13, 128, 1024, 4, gen=O.gen_kquant_matrix)
    run_case(F, O, Q6_K, 24, 64, 512, 5, gen=O.gen_kquant_matrix)


@pytest.mark.parametrize("t", [128, 512, 2048])
def test_config4_prefill_5120(F, O, t):
    # W 5120x5120 Q4_K, X [t, 5120] bf16 ~ N(0,1), f32 out
    run_case(F, O, Q4_K, t, 5120, 5120, 21)


def test_prefill_other_formats_at_size(F, O):
    run_case(F, O, Q6_K, 256, 5120, 5120, 22)
    run_case(F, O, Q8_0, 256, 4096, 4096, 23)


def test_rows_are_independent_of_the_batch(F, O):
    # A row of a T-row prefill is bit-identical to the same row computed in a smaller batch, as long as
    # both launches have enough output tiles to run without splitting K (with a K split the slices are
    # added atomically, so only the tolerance holds there, not bit equality).
    from ferric_amd.synth import synth_weights
    w = synth_weights(Q4_K, 5120, 512, 5)
    qm = F.QMatrix.from_bytes(w, Q4_K, 5120, 512)
    x = np.random.default_rng(1).standard_normal((2048, 512)).astype(np.float32)
    xb, _ = bf16_round(x)
    big = F.Tensor.from_bf16_bits(xb, (2048, 512)).gemm_q_bf16(qm).to_vec().reshape(2048, 5120)
    part = F.Tensor.from_bf16_bits(xb[256:], (1792, 512)).gemm_q_bf16(qm).to_vec().reshape(1792, 5120)
    assert np.array_equal(big[256:].view(np.uint32), part.view(np.uint32))
    again = F.Tensor.from_bf16_bits(xb, (2048, 512)).gemm_q_bf16(qm).to_vec().reshape(2048, 5120)
    assert np.array_equal(big.view(np.uint32), again.view(np.uint32))


def test_q8_0_rows_ending_inside_a_chunk(F, O):
    # Q8_0 rows are any multiple of 32 long; the kernel walks 256-column chunks, so 32..224 trailing columns
    # exercise the zero-scale / zero-activation padding of the last chunk (and K < 256 has no full chunk at all)
    for i, (t, n, k) in enumerate([(3, 40, 32), (9, 64, 96), (40, 130, 288), (130, 70, 480), (70, 257, 1184)]):
        run_case(F, O, Q8_0, t, n, k, 40 + i)


def test_gemm_errors(F):
    qm = F.QMatrix.from_bytes(np.zeros(144, np.uint8), Q4_K, 1, 256)
    with pytest.raises(AssertionError, match="inner dim mismatch"):
        F.Tensor.from_bf16_bits(np.zeros(512, np.uint16), (1, 512)).gemm_q_bf16(qm)
    assert F.Tensor.from_bf16_bits(np.zeros(0, np.uint16), (0, 256)).gemm_q_bf16(qm).to_vec().size == 0
