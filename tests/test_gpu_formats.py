"""The further block formats (Q4_0, Q4_1, Q5_0, Q5_1, Q5_K) through the C ABI: unpackers bit-exact against the
oracle, mat-vec / small batch against f64 on oracle-dequantized weights (north-star bound per dot and 1e-5 of the
largest output, the reference's bar for its scalar kernels), fused SwiGLU for Q5_K, and the "_id" variants."""
import numpy as np
import pytest

from conftest import bits

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q6_K, Q4_0, Q4_1, Q5_0, Q5_1, Q5_K = 8, 12, 14, 2, 3, 6, 7, 13
NEW = [Q4_0, Q4_1, Q5_0, Q5_1, Q5_K]
GEOM = {Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q5_K: (256, 176)}


@pytest.mark.parametrize("ty", NEW)
def test_unpackers_are_bit_exact(F, O, ty):
    from ferric_amd.synth import synth_weights
    vals, nbytes = GEOM[ty]
    assert F.type_size(ty, vals * 5 + 3) == 5 * nbytes and F.QMatrix.block_bytes(ty) == (vals, nbytes)
    raw = synth_weights(ty, 37, vals * 3, 4)
    n = 37 * vals * 3
    assert np.array_equal(bits(F.deq_raw(raw, n, ty)), bits(O.deq_raw(raw, n, ty)))
    w = F.QMatrix.from_bytes(raw, ty, 37, vals * 3)
    assert np.array_equal(bits(w.dequant().to_vec()), bits(O.deq_raw(raw, n, ty)))
    assert np.array_equal(bits(w.dequant_rows(5, 3).to_vec()), bits(O.deq_raw(raw, n, ty).reshape(37, -1)[5:8].reshape(-1)))
    # every byte value in every field, including non-finite f16 scales
    rng = np.random.default_rng(3)
    blk = rng.integers(0, 256, (512, nbytes), dtype=np.uint8)
    blk[:256, :] = np.arange(256, dtype=np.uint8).reshape(256, 1)
    got, want = F.deq_raw(blk.reshape(-1), 512 * vals, ty), O.deq_raw(blk.reshape(-1), 512 * vals, ty)
    ok = ~np.isnan(want)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(bits(got)[ok], bits(want)[ok])
    # ragged: n past the bytes present and n not a multiple of the block leave zeros, as the reference's vec![0.0; n]
    short = F.deq_raw(raw[: 2 * nbytes + 1], vals * 4, ty)
    assert short.size == vals * 4 and np.array_equal(bits(short), bits(O.deq_raw(raw[: 2 * nbytes + 1], vals * 4, ty)))
    part = F.deq_raw(raw, vals * 2 + 7, ty)
    assert part.size == vals * 2 + 7 and not part[2 * vals:].any()


@pytest.mark.parametrize("ty", NEW)
def test_matmul_small_batch(F, O, ty):
    from ferric_amd.synth import synth_weights
    vals, _ = GEOM[ty]
    rng = np.random.default_rng(7)
    for rows, cols, b in [(1, vals, 1), (70, vals * 3, 1), (257, 1024, 1), (96, 2048, 3), (40, 4096, 8), (33, 5120, 2)]:
        if cols % vals:
            continue
        raw = synth_weights(ty, rows, cols, rows + b)
        w = F.QMatrix.from_bytes(raw, ty, rows, cols)
        x = rng.standard_normal((b, cols)).astype(np.float32)
        y = F.Tensor.from_vec(x.reshape(-1), (b, cols)).matmul_q(w).to_vec().reshape(b, rows)
        y64, wn = O.matmul_f64(x, raw, ty, rows, cols)
        assert (np.abs(y - y64) <= 1e-3 * wn[None, :] * np.linalg.norm(x.astype(np.float64), axis=1)[:, None]).all(), (rows, cols, b)
        assert np.abs(y - y64).max() <= 1e-5 * max(1e-3, np.abs(y64).max()), (rows, cols, b)
        # a row of a batch is bit-identical to the same row alone
        y1 = F.Tensor.from_vec(x[b - 1], (1, cols)).matmul_q(w).to_vec()
        assert np.array_equal(bits(y1), bits(y[b - 1]))
    name = {Q4_0: "matmul_q4_0", Q4_1: "matmul_q4_1", Q5_0: "matmul_q5_0", Q5_1: "matmul_q5_1", Q5_K: "matmul_q5_k"}[ty]
    assert np.array_equal(bits(getattr(F.Tensor.from_vec(x[0], (1, cols)), name)(w).to_vec()), bits(y[0]))
    with pytest.raises(AssertionError, match="inner dim mismatch"):
        F.Tensor.from_vec(np.zeros(cols + vals, np.float32), (1, cols + vals)).matmul_q(w)
    with pytest.raises(AssertionError, match="multiple of"):
        F.QMatrix.from_bytes(raw, ty, rows, cols + 1)


def test_q5_k_fused_swiglu_and_the_others_have_none(F, O):
    from ferric_amd.synth import synth_weights
    n_ff, cols = 136, 1024
    raw = synth_weights(Q5_K, 2 * n_ff, cols, 11)
    w = F.QMatrix.from_bytes(raw, Q5_K, 2 * n_ff, cols)
    x = np.random.default_rng(8).standard_normal((3, cols)).astype(np.float32)
    xt = F.Tensor.from_vec(x.reshape(-1), (3, cols))
    got = xt.matmul_q5_k_swiglu(w).to_vec().reshape(3, n_ff)
    g64, _ = O.matmul_f64(x, raw, Q5_K, 2 * n_ff, cols)
    want = g64[:, :n_ff] / (1 + np.exp(-g64[:, :n_ff])) * g64[:, n_ff:]
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    unfused = xt.matmul_q(w).swiglu(n_ff).to_vec().reshape(3, n_ff)       # same dots, same SwiGLU arithmetic
    assert np.array_equal(bits(unfused), bits(got))
    w40 = F.QMatrix.from_bytes(synth_weights(Q4_0, 2 * n_ff, cols, 12), Q4_0, 2 * n_ff, cols)
    assert xt.try_matmul_swiglu(w40) is None


def test_id_variants_on_the_other_formats(F, O):
    from ferric_amd.synth import synth_weights
    rng = np.random.default_rng(9)
    n_expert, t, k, cols, out_pe = 5, 2, 3, 512, 72
    sel = np.zeros((t, 2 * k), np.float32)
    for ti in range(t):
        sel[ti, :k] = rng.random(k) + 0.1
        sel[ti, k:] = rng.choice(n_expert, size=k, replace=False)
    st = F.Tensor.from_vec(sel.reshape(-1), (t, 2 * k))
    x = rng.standard_normal((t, k, cols)).astype(np.float32)
    for ty in (Q5_0, Q5_K, Q4_1):
        raw = synth_weights(ty, n_expert * out_pe, cols, 13 + ty)
        w = F.QMatrix.from_bytes(raw, ty, n_expert * out_pe, cols)
        got = F.Tensor.from_vec(x.reshape(-1), (t, k, cols)).matmul_q_id_wsum(w, st, out_pe).to_vec().reshape(t, out_pe)
        want, bound = O.matmul_id_wsum_f64(x, raw, ty, sel, k, out_pe, cols)
        assert (np.abs(got - want) <= 1e-3 * bound).all() and np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    raw = synth_weights(Q5_0, n_expert * out_pe, cols, 30)
    w = F.QMatrix.from_bytes(raw, Q5_0, n_expert * out_pe, cols)
    a = F.Tensor.from_vec(x.reshape(-1), (t, k, cols)).matmul_q5_0_id_wsum(w, st, out_pe).to_vec()
    assert np.array_equal(bits(a), bits(F.Tensor.from_vec(x.reshape(-1), (t, k, cols)).matmul_q_id_wsum(w, st, out_pe).to_vec()))
    # gate|up + SwiGLU on a Q5_K expert slab
    eff = 40
    raw = synth_weights(Q5_K, n_expert * 2 * eff, cols, 31)
    w = F.QMatrix.from_bytes(raw, Q5_K, n_expert * 2 * eff, cols)
    got = F.Tensor.from_vec(x[:, 0].reshape(-1), (t, cols)).matmul_q_swiglu_id(w, st, k, eff).to_vec().reshape(t, k, eff)
    want = O.matmul_swiglu_id_f64(x[:, 0], raw, Q5_K, sel, k, eff, cols)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()


def test_matrix_core_entry_points_refuse_the_other_formats(F):
    from ferric_amd.synth import synth_weights
    w = F.QMatrix.from_bytes(synth_weights(Q5_K, 32, 256, 1), Q5_K, 32, 256)
    with pytest.raises(ValueError, match="no native matmul for ggml type 13"):
        F.Tensor.from_bf16_bits(np.zeros(256, np.uint16), (1, 256)).gemm_q_bf16(w)


def test_these_formats_load_from_a_gguf_file(F, O, tmp_path):
    import os
    import sys
    sys.path.insert(0, os.path.dirname(__file__))
    from gguf_writer import write_gguf
    from ferric_amd.synth import synth_weights
    shapes = {f"blk.{i}.w.weight": (ty, 9 + i, GEOM[ty][0] * 4) for i, ty in enumerate(NEW)}
    raw = {n: synth_weights(ty, r, c, 40 + i) for i, (n, (ty, r, c)) in enumerate(shapes.items())}
    data = write_gguf([("general.architecture", "str", "llama")], [(n, [c, r], ty, raw[n]) for n, (ty, r, c) in shapes.items()])[0]
    path = tmp_path / "formats.gguf"
    path.write_bytes(data)
    g = F.GgufFile.open(path)
    for name, (ty, r, c) in shapes.items():
        w = g.qmatrix(name)
        assert (w.rows(), w.cols(), w.ggml_type, w.nbytes()) == (r, c, ty, raw[name].size)
        assert np.array_equal(bits(w.dequant().to_vec()), bits(O.deq_raw(raw[name], r * c, ty)))
