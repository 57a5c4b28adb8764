"""The further block formats (Q4_0, Q4_1, Q5_0, Q5_1, Q5_K, IQ4_NL, IQ4_XS, MXFP4) through the C ABI: unpackers bit-exact against the
oracle, mat-vec / small batch against f64 on oracle-dequantized weights (north-star bound per dot and 1e-5 of the
largest output, the reference's bar for its scalar kernels), fused SwiGLU for Q5_K, and the "_id" variants."""
import numpy as np
import pytest

from conftest import bits, dot_bar

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("precision")]
Q8_0, Q4_K, Q6_K, Q4_0, Q4_1, Q5_0, Q5_1, Q5_K = 8, 12, 14, 2, 3, 6, 7, 13
IQ4_NL, IQ4_XS, MXFP4 = 20, 23, 39
NEW = [Q4_0, Q4_1, Q5_0, Q5_1, Q5_K, IQ4_NL, IQ4_XS, MXFP4]
GEOM = {Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q5_K: (256, 176), IQ4_NL: (32, 18), IQ4_XS: (256, 136),
        MXFP4: (32, 17)}


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
        assert np.abs(y - y64).max() <= dot_bar() * max(1e-3, np.abs(y64).max()), (rows, cols, b)
        # a row of a batch is bit-identical to the same row alone; Q5_K batches of three rows and more take the one-pass
        # matrix-core kernels, as Q4_K's do, and agree with the mat-vec to the bar both are held to
        y1 = F.Tensor.from_vec(x[b - 1], (1, cols)).matmul_q(w).to_vec()
        if ty == Q5_K and b >= 3:
            assert np.abs(y1 - y[b - 1]).max() <= 2 * dot_bar() * np.abs(y64).max()
        else:
            assert np.array_equal(bits(y1), bits(y[b - 1]))
    name = {Q4_0: "matmul_q4_0", Q4_1: "matmul_q4_1", Q5_0: "matmul_q5_0", Q5_1: "matmul_q5_1", Q5_K: "matmul_q5_k",
            IQ4_NL: "matmul_iq4_nl", IQ4_XS: "matmul_iq4_xs", MXFP4: "matmul_mxfp4"}[ty]
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
    assert np.abs(got - want).max() <= dot_bar() * np.abs(want).max()
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
    for ty in (Q5_0, Q5_K, Q4_1, IQ4_NL, IQ4_XS, MXFP4):
        raw = synth_weights(ty, n_expert * out_pe, cols, 13 + ty)
        w = F.QMatrix.from_bytes(raw, ty, n_expert * out_pe, cols)
        got = F.Tensor.from_vec(x.reshape(-1), (t, k, cols)).matmul_q_id_wsum(w, st, out_pe).to_vec().reshape(t, out_pe)
        want, bound = O.matmul_id_wsum_f64(x, raw, ty, sel, k, out_pe, cols)
        assert (np.abs(got - want) <= 1e-3 * bound).all() and np.abs(got - want).max() <= dot_bar() * np.abs(want).max()
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
    assert np.abs(got - want).max() <= dot_bar() * np.abs(want).max()


def test_matrix_core_entry_points_refuse_the_other_formats(F):
    # the matrix-core prefill takes the formats the reference has coop kernels for (Q4_K, Q5_K, Q6_K, Q8_0), no other
    from ferric_amd.synth import synth_weights
    for ty in (Q4_0, Q4_1, Q5_0, Q5_1, IQ4_NL, IQ4_XS, MXFP4):
        cols = GEOM[ty][0] * (8 if GEOM[ty][0] == 32 else 1)
        w = F.QMatrix.from_bytes(synth_weights(ty, 32, cols, 1), ty, 32, cols)
        with pytest.raises(ValueError, match=f"no native matmul for ggml type {ty}"):
            F.Tensor.from_bf16_bits(np.zeros(cols, np.uint16), (1, cols)).gemm_q_bf16(w)


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


def _mxfp4_golden():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "mxfp4_ggml.json")) as f:
        return json.load(f)


def test_mxfp4_unpacker_against_the_ggml_captured_answers(F):
    # the reference's own known answers (crates/ferric-gguf/src/lib.rs:1099-1222), which include subnormal scales (e = 0, 1)
    # and both saturating ends (e = 254, 255): the device must neither flush the former nor overflow early on the latter
    g = _mxfp4_golden()
    blocks, want = [], []
    for ei, e in enumerate(g["e"]):
        for code in range(16):
            lo = np.zeros(17, np.uint8); lo[0] = e; lo[1] = code
            hi = np.zeros(17, np.uint8); hi[0] = e; hi[1] = code << 4
            blocks += [lo, hi]
            w = g["grid_bits"][ei * 16 + code]
            a = np.zeros(32, np.uint32); a[0] = w
            b = np.zeros(32, np.uint32); b[16] = w
            want += [a, b]
    raw = np.concatenate(blocks)
    assert np.array_equal(bits(F.deq_raw(raw, 32 * len(blocks), MXFP4)), np.concatenate(want))
    real = np.array(g["real_raw"], np.uint8)
    assert np.array_equal(bits(F.deq_raw(real, 256, MXFP4)), np.array(g["real_bits"], np.uint32))
    w = F.Mxfp4Weights.from_bytes(real, 1, 256)
    assert np.array_equal(bits(w.dequant().to_vec()), np.array(g["real_bits"], np.uint32))


def test_mxfp4_matvec_forms_the_weight_before_it_meets_the_activation(F, O):
    # crates/ferric-tensor/src/dtype.rs:3331-3335: a block whose weights saturate contributes inf (not a finite x*d*k), a
    # subnormal scale is not flushed, and every (scale, code) pair gives x * w with the oracle's w
    blk = np.zeros((256, 17), np.uint8)
    blk[:, 0] = np.arange(256)
    blk[:, 1:9] = np.arange(16, dtype=np.uint8).reshape(8, 2)[:, 0] | (np.arange(16, dtype=np.uint8).reshape(8, 2)[:, 1] << 4)
    w = F.QMatrix.from_bytes(blk.reshape(-1), MXFP4, 256, 32)            # row e: one block under scale byte e
    wd = O.deq_raw(blk.reshape(-1), 256 * 32, MXFP4).reshape(256, 32)
    for j in (0, 1, 16, 7, 23):                                           # x = 0.5 * unit vector j picks out 0.5 * w[e, j]
        x = np.zeros(32, np.float32); x[j] = 0.5
        y = F.Tensor.from_vec(x, (1, 32)).matmul_q(w).to_vec()
        with np.errstate(over="ignore", invalid="ignore"):
            want = (x[None, :] * wd).sum(axis=1, dtype=np.float32)       # one non-zero product per row; 0 * inf = NaN stays NaN
        # the same NaN / inf pattern; finite products to the rounding of the run scale (the activation 0.5 is the run's
        # maximum, held as 0.5 / QMAX * QMAX)
        assert np.array_equal(np.isnan(y), np.isnan(want)) and np.array_equal(np.isinf(y), np.isinf(want)), j
        fin = np.isfinite(want)
        assert np.array_equal(np.sign(y[fin]), np.sign(want[fin])) and (np.abs(y[fin] - want[fin]) <= 1e-6 * np.abs(want[fin])).all(), j
        assert np.isnan(want[255]) and np.isfinite(want[:250]).all()
    assert np.isinf(wd[255, 1]) and wd[0, 16] == np.float32(2.0 ** -128) and wd[255, 16] == np.float32(2.0 ** 127)
    x = np.zeros(32, np.float32); x[16] = 0.5
    one = F.QMatrix.from_bytes(np.concatenate([blk[255, :1], np.array([0x10], np.uint8), np.zeros(15, np.uint8)]), MXFP4, 1, 32)
    top = F.Tensor.from_vec(x, (1, 32)).matmul_q(one).to_vec()[0]
    assert np.isfinite(top) and abs(float(top) / 2.0 ** 126 - 1.0) <= 1e-6                     # finite at the top scale


def test_mxfp4_saturating_blocks_through_the_streaming_kernel(F, O):
    # a row long enough for the integer-plane kernel (512 columns): blocks whose scale byte can overflow the weight (e >= 252)
    # must still give the reference's x * (k * scale) per element -- inf where a product overflows, NaN where inf meets a zero
    # activation -- and ordinary blocks beside them must not be disturbed
    rng = np.random.default_rng(21)
    rows, cols = 24, 512
    blk = rng.integers(0, 256, (rows, cols // 32, 17), dtype=np.uint8)
    blk[:, :, 0] = rng.integers(0x70, 0x80, (rows, cols // 32), dtype=np.uint8)
    blk[3, 5, 0], blk[7, 0, 0], blk[7, 9, 0], blk[11, 15, 0], blk[12, 2, 0] = 255, 254, 253, 252, 251
    raw = blk.reshape(-1)
    w = F.QMatrix.from_bytes(raw, MXFP4, rows, cols)
    wd = O.deq_raw(raw, rows * cols, MXFP4).reshape(rows, cols)
    x = rng.standard_normal(cols).astype(np.float32)
    x[5 * 32: 5 * 32 + 8] = 0.0                                           # zeros under the e = 255 block of row 3
    y = F.Tensor.from_vec(x, (1, cols)).matmul_q(w).to_vec()
    with np.errstate(over="ignore", invalid="ignore"):
        want = (wd.astype(np.float64) * x.astype(np.float64)).sum(axis=1)
    plain = [r for r in range(rows) if r not in (3, 7, 11, 12)]
    assert np.abs(y[plain] - want[plain]).max() <= dot_bar() * np.abs(want[plain]).max()     # ordinary rows, beside the special blocks
    assert np.isnan(y[3])                                                 # inf weights over zero activations
    assert not np.isfinite(y[7])                                          # e = 254 / 253: weights of both signs overflow
    for r in (11, 12):                                                    # e = 252 / 251: finite weights near the top of f32; the f32
        assert np.isinf(y[r]) or abs(y[r] - want[r]) <= dot_bar() * abs(want[r])   # sum may overflow, but it may not be NaN or wrong


def test_iq4_xs_packed_kernel_matches_the_dense_reference(F, O):
    # crates/ferric-tensor/examples/iq4_xs.rs restated: its block generator, its activation ramp, its shapes and its bar
    # (max |got - want| / max |want| < 1e-5 against the dense product of the dequantized weight)
    def half_bits(x):
        b = int(np.array([x], np.float32).view(np.uint32)[0])
        exp = ((b >> 23) & 0xFF) - 127 + 15
        return ((b >> 16) & 0x8000) if exp <= 0 else (((b >> 16) & 0x8000) | (exp << 10) | ((b >> 13) & 0x3FF))

    def blocks(nblk, seed):
        s = (seed * 2654435761 + 1) & 0xFFFFFFFF
        out = bytearray()

        def rnd():
            nonlocal s
            s = (s * 1664525 + 1013904223) & 0xFFFFFFFF
            return (s >> 16) & 0xFFFF
        for _ in range(nblk):
            out += int(half_bits(np.float32(0.005) + np.float32(rnd() % 40) * np.float32(0.0007))).to_bytes(2, "little")
            out += rnd().to_bytes(2, "little")
            out += bytes(rnd() & 0xFF for _ in range(4))
            out += bytes(rnd() & 0xFF for _ in range(128))
        return np.frombuffer(bytes(out), np.uint8)
    for rows, cols in [(8, 256), (32, 512), (7, 1024), (64, 256)]:
        raw = blocks(rows * (cols // 256), rows * 31 + cols)
        deq = O.deq_raw(raw, rows * cols, IQ4_XS).reshape(rows, cols)
        xv = ((np.arange(cols) * 37 % 101).astype(np.float32) - np.float32(50.0)) / np.float32(50.0)
        want = deq.astype(np.float64) @ xv.astype(np.float64)
        got = F.Tensor.from_vec(xv, (1, cols)).matmul_iq4_xs(F.Iq4XsWeights.from_bytes(raw, rows, cols)).to_vec()
        assert np.abs(got - want).max() / max(1e-6, np.abs(want).max()) < dot_bar(), (rows, cols)


def test_the_shape_complete_f32_kernel_still_agrees(F, O):
    """Every legal row length now runs the streaming kernel; the f32 kernel behind it stays the fallback for rows too long
    for one workgroup. Forced on here so that it keeps its own parity check, for every format."""
    from ferric_amd.synth import synth_weights
    lib = F._lib.load()
    rng = np.random.default_rng(31)
    geom = dict(GEOM); geom.update({Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210)})
    F._lib.check(lib.fhip_debug_generic_matvec(1))
    try:
        for ty, (vals, _) in geom.items():
            for rows, cols, b in [(70, vals * 3, 1), (33, 5120, 2), (40, 1024, 3)]:
                raw = synth_weights(ty, rows, cols, rows + ty)
                w = F.QMatrix.from_bytes(raw, ty, rows, cols)
                x = rng.standard_normal((b, cols)).astype(np.float32)
                y = F.Tensor.from_vec(x.reshape(-1), (b, cols)).matmul_q(w).to_vec().reshape(b, rows)
                y64, wn = O.matmul_f64(x, raw, ty, rows, cols)
                assert (np.abs(y - y64) <= 1e-3 * wn[None, :] * np.linalg.norm(x.astype(np.float64), axis=1)[:, None]).all(), (ty, rows, cols)
                assert np.abs(y - y64).max() <= dot_bar() * max(1e-3, np.abs(y64).max()), (ty, rows, cols)
        n_ff = 96
        for ty in (Q4_K, Q6_K, Q5_K):
            raw = synth_weights(ty, 2 * n_ff, 768, 5)
            w = F.QMatrix.from_bytes(raw, ty, 2 * n_ff, 768)
            x = rng.standard_normal((2, 768)).astype(np.float32)
            got = F.Tensor.from_vec(x.reshape(-1), (2, 768)).try_matmul_swiglu(w).to_vec().reshape(2, n_ff)
            g64, _ = O.matmul_f64(x, raw, ty, 2 * n_ff, 768)
            want = g64[:, :n_ff] / (1 + np.exp(-g64[:, :n_ff])) * g64[:, n_ff:]
            assert np.abs(got - want).max() <= dot_bar() * np.abs(want).max(), ty
    finally:
        F._lib.check(lib.fhip_debug_generic_matvec(0))
