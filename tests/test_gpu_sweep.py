"""The decode weight sweep's own shapes and launch chain against the CPU oracle, through the C ABI: the vocabulary head
(151936 x 5120 Q6_K, the largest single launch), a weight with more rows than one round of workgroups takes, and layers of
the four per-layer projections chained in one captured graph the way the benchmark's sweep issues them.

Bars as in test_gpu_matmul.py: the north-star bound 1e-3 * ||w_row|| * ||x|| per dot product and conftest.dot_bar() of the
largest output; row-partition invariance (a slice of the rows computed alone gives the same bits) replaces the oracle where
the oracle would take minutes.
"""
import ctypes as C

import numpy as np
import pytest

from conftest import bits, dot_bar

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("precision")]
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
BLOCK = {Q8_0: (32, 34), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210)}


def row_bytes(ty, cols):
    vals, b = BLOCK[ty]
    return cols // vals * b


def upload(F, raw):
    lib = F._lib.load()
    buf = F.DeviceBuffer(raw.size)
    F._lib.check(lib.fhip_memcpy_h2d(buf.ptr, raw.ctypes.data_as(C.c_void_p), raw.size, None))
    F._lib.check(lib.fhip_stream_sync(None))
    return buf


def check_rows(O, y, x, raw, ty, cols, row_slices, what):
    """y[rows] against the f64 product over the oracle-dequantized weights, on the given row ranges."""
    rb = row_bytes(ty, cols)
    for r0, r1 in row_slices:
        y64, wn = O.matmul_f64(x, raw[r0 * rb:r1 * rb], ty, r1 - r0, cols)
        err = np.abs(y[r0:r1] - y64[0])
        assert (err <= 1e-3 * wn * np.linalg.norm(x.astype(np.float64))).all(), (what, r0)
        assert err.max() <= dot_bar() * np.abs(y64).max(), (what, r0, err.max() / np.abs(y64).max())


def test_vocabulary_head_151936_x_5120_q6_k(F, O):
    """crates/ferric-llama/src/qwen3.rs:803: logits = hidden . lm_head^T, 638 MB of Q6_K in one launch."""
    from ferric_amd.synth import synth_weights
    rows, cols = 151936, 5120
    raw = synth_weights(Q6_K, rows, cols, 50)
    buf = upload(F, raw)
    w = F.QMatrix.wrap_device(buf, raw.size, Q6_K, rows, cols)
    x = np.random.default_rng(51).standard_normal(cols).astype(np.float32)
    xt = F.Tensor.from_vec(x, (1, cols))
    y = xt.matmul_q(w).to_vec()
    mid = rows // 2
    check_rows(O, y, x, raw, Q6_K, cols, [(0, 768), (mid - 384, mid + 384), (rows - 768, rows), (75000, 75256), (151000, 151300)], "lm_head")
    assert np.isfinite(y).all()
    # row-partition invariance (crates/ferric-tensor/src/cpu_simd.rs:175-200): any span of rows computed alone gives the same
    # bits, here three spans that do not line up with the launch's row groups (a wrapped device pointer has to be 16-byte
    # aligned and a row is 4200 bytes, so the spans start at even rows)
    rb = row_bytes(Q6_K, cols)
    for r0, n in ((0, 1000), (70002, 4099), (rows - 334, 334)):
        part = F.QMatrix.wrap_device(buf, n * rb, Q6_K, n, cols, offset=r0 * rb)
        assert np.array_equal(bits(xt.matmul_q(part).to_vec()), bits(y[r0:r0 + n])), r0


@pytest.mark.parametrize("ty,cols,period", [(Q4_K, 5120, 4096), (Q5_K, 5120, 4096), (Q8_0, 1024, 3000)])
def test_more_rows_than_one_round_of_workgroups(F, O, ty, cols, period):
    """A vocabulary of 262144 rows (the Gemma-class callers of the same matmul_q, crates/ferric-llama/src/gemma4.rs:274-280)
    is more than one workgroup per CU takes at 256 rows per row group: the launch goes over the rows in several rounds (Q5_K:
    two rounds of three row groups per workgroup; Q4_K, with two row groups per workgroup for a weight this large, takes up
    to 1024 rows per row group and stays at one round; Q8_0 rows this short fill one round of sixteen row groups). The
    weight repeats a block of `period` random rows, so every output has an oracle value and equal rows must give equal bits."""
    from ferric_amd.synth import synth_weights
    rows = 262144
    one = synth_weights(ty, period, cols, 60)
    rb = row_bytes(ty, cols)
    reps = -(-rows // period)
    raw = np.tile(one, reps)[: rows * rb]
    w = F.QMatrix.from_bytes(raw, ty, rows, cols)
    x = np.random.default_rng(61).standard_normal(cols).astype(np.float32)
    y = F.Tensor.from_vec(x, (1, cols)).matmul_q(w).to_vec()
    check_rows(O, y, x, one, ty, cols, [(0, period)], "first period")
    pad = np.full(reps * period - rows, np.float32(0))
    tiled = np.concatenate([y, pad]).reshape(reps, period)
    for k in range(1, reps - 1):
        assert np.array_equal(bits(tiled[k]), bits(tiled[0])), k
    last = rows - (reps - 1) * period
    assert np.array_equal(bits(tiled[reps - 1][:last]), bits(tiled[0][:last]))


def test_layers_of_the_sweep_chained_in_one_graph(F, O):
    """Three layers of the sweep's four projections (fused QKV 5120 -> 7168, O 5120 -> 5120, fused gate|up 5120 -> 34816 with
    SwiGLU, all Q4_K; down 17408 -> 5120 Q6_K) and a head, recorded into one graph on one stream in the order the benchmark
    issues them, every launch writing its own output; after the replay each output is held to the oracle. The activations
    are fixed per op (random weights chained through would leave the f32 range within a few layers)."""
    from ferric_amd.synth import synth_weights
    lib = F._lib.load()
    check = F._lib.check
    shapes = [("qkv", Q4_K, 7168, 5120, False), ("o", Q4_K, 5120, 5120, False), ("gate_up", Q4_K, 34816, 5120, True),
              ("down", Q6_K, 5120, 17408, False)]
    layers = 3
    rng = np.random.default_rng(70)
    x = rng.standard_normal(5120).astype(np.float32)
    h = (rng.standard_normal(17408) * 0.1).astype(np.float32)
    xt, ht = F.Tensor.from_vec(x, (1, 5120)), F.Tensor.from_vec(h, (1, 17408))
    raws, ws, outs = {}, {}, {}
    for l in range(layers):
        for i, (name, ty, r, c, sw) in enumerate(shapes):
            raws[l, name] = synth_weights(ty, r, c, 100 + 10 * l + i)
            ws[l, name] = F.QMatrix.from_bytes(raws[l, name], ty, r, c)
            outs[l, name] = F.Tensor.empty((1, r // 2 if sw else r))
    head_raw = synth_weights(Q6_K, 3001, 5120, 99)
    head, logits = F.QMatrix.from_bytes(head_raw, Q6_K, 3001, 5120), F.Tensor.empty((1, 3001))
    stream = F.Stream()
    g = F.Graph.begin(stream)
    for l in range(layers):
        for name, ty, r, c, sw in shapes:
            xin = ht if name == "down" else xt
            fn = lib.fhip_matmul_q_swiglu if sw else lib.fhip_matmul_q
            check(fn(ws[l, name].handle, xin.buf.ptr, 1, outs[l, name].buf.ptr, stream.handle))
    check(lib.fhip_matmul_q(head.handle, xt.buf.ptr, 1, logits.buf.ptr, stream.handle))
    g.end()
    for replay in range(2):
        g.launch()
        stream.synchronize()
    for l in range(layers):
        for name, ty, r, c, sw in shapes:
            xin = h if name == "down" else x
            got = outs[l, name].to_vec(stream)
            y64, wn = O.matmul_f64(xin, raws[l, name], ty, r, c)
            if sw:
                n_ff = r // 2
                gate, up = y64[0, :n_ff], y64[0, n_ff:]
                want = gate / (1.0 + np.exp(-gate)) * up
                assert np.abs(got - want).max() <= dot_bar() * np.abs(want).max(), (l, name)
            else:
                err = np.abs(got - y64[0])
                assert (err <= 1e-3 * wn * np.linalg.norm(xin.astype(np.float64))).all(), (l, name)
                assert err.max() <= dot_bar() * np.abs(y64).max(), (l, name)
    check_rows(O, logits.to_vec(stream), x, head_raw, Q6_K, 5120, [(0, 3001)], "head")


def test_layers_chained_output_to_input_in_one_graph(F, O):
    """Two layers of the same four projections with every launch reading the launch before it, as the benchmark's chained
    sweep does: x -> rmsnorm + QKV -> O (on the first 5120 of the QKV row) -> rmsnorm + gate|up + SwiGLU -> down -> next layer,
    the norms fused into the mat-vecs that consume them (fhip_norm_matmul_q), one captured graph replayed twice. The oracle
    walks the same chain in f64 from the device's own input of each step, so every step is held to the mat-vec's bar by itself,
    and the end of the chain to the product of the steps."""
    from ferric_amd.synth import synth_weights
    lib = F._lib.load()
    check = F._lib.check
    shapes = [("qkv", Q4_K, 7168, 5120, 0), ("o", Q4_K, 5120, 5120, 0), ("gate_up", Q4_K, 34816, 5120, 1), ("down", Q6_K, 5120, 17408, 0)]
    layers, eps = 2, 1e-6
    rng = np.random.default_rng(71)
    x0 = rng.standard_normal(5120).astype(np.float32)
    nw = ((rng.random(5120) + 0.5) * 0.01).astype(np.float32)      # small norm weights keep the chain inside the f32 range
    raws, ws = {}, {}
    for l in range(layers):
        for i, (name, ty, r, c, sw) in enumerate(shapes):
            raws[l, name] = synth_weights(ty, r, c, 300 + 10 * l + i)
            ws[l, name] = F.QMatrix.from_bytes(raws[l, name], ty, r, c)
    T = lambda n: F.Tensor.empty((1, n))
    xt, nwt, scratch = F.Tensor.from_vec(x0, (1, 5120)), F.Tensor.from_vec(nw, (1, 5120)), T(5120)
    bufs = {(l, name): T(r // 2 if sw else r) for l in range(layers) for name, ty, r, c, sw in shapes}
    stream = F.Stream()
    g = F.Graph.begin(stream)
    cur = xt
    for l in range(layers):
        check(lib.fhip_norm_matmul_q(ws[l, "qkv"].handle, cur.buf.ptr, None, nwt.buf.ptr, eps, None, scratch.buf.ptr, 0, bufs[l, "qkv"].buf.ptr, stream.handle))
        check(lib.fhip_matmul_q(ws[l, "o"].handle, bufs[l, "qkv"].buf.ptr, 1, bufs[l, "o"].buf.ptr, stream.handle))
        check(lib.fhip_norm_matmul_q(ws[l, "gate_up"].handle, bufs[l, "o"].buf.ptr, None, nwt.buf.ptr, eps, None, scratch.buf.ptr, 1, bufs[l, "gate_up"].buf.ptr, stream.handle))
        check(lib.fhip_matmul_q(ws[l, "down"].handle, bufs[l, "gate_up"].buf.ptr, 1, bufs[l, "down"].buf.ptr, stream.handle))
        cur = bufs[l, "down"]
    g.end()
    for replay in range(2):
        g.launch()
        stream.synchronize()

    def norm64(v):
        v = v.astype(np.float64)
        return v / np.sqrt((v * v).mean() + eps) * nw.astype(np.float64)

    got = {k: b.to_vec(stream).astype(np.float32) for k, b in bufs.items()}
    prev = x0
    for l in range(layers):
        for name, ty, r, c, sw in shapes:
            xin = norm64(prev) if name in ("qkv", "gate_up") else prev[:c].astype(np.float64)
            y64, wn = O.matmul_f64(xin.astype(np.float32)[None, :], raws[l, name], ty, r, c)
            # the oracle's input is rounded to f32 where the device's staged row is f32 too; the bound covers the difference
            if sw:
                gate, up = y64[0, :r // 2], y64[0, r // 2:]
                want = gate / (1.0 + np.exp(-gate)) * up
            else:
                want = y64[0]
            err = np.abs(got[l, name] - want)
            assert err.max() <= 2 * dot_bar() * np.abs(want).max(), (l, name, float(err.max() / np.abs(want).max()))
            prev = got[l, name]            # the next step starts from what the device produced
    assert np.isfinite(got[layers - 1, "down"]).all() and np.abs(got[layers - 1, "down"]).max() > 0


@pytest.mark.parametrize("ty,rows,cols,swiglu", [(Q4_K, 12301, 5120, False), (Q4_K, 2 * 12303, 5120, True), (Q6_K, 4099, 17408, False),
                                                 (Q8_0, 33001, 1024, False)])
def test_large_weights_whose_rows_are_dealt_in_chunks_of_four(F, O, ty, rows, cols, swiglu):
    """From 16 rows per row group on, the launch deals the rows to the row groups round-robin in chunks of 4 instead of giving
    each a contiguous span. Row counts that leave the last round of chunks, and the last chunk, partly filled; every output
    against the oracle, and a span of the rows computed alone (which takes the other dealing) gives the same bits."""
    from ferric_amd.synth import synth_weights
    raw = synth_weights(ty, rows, cols, 80)
    w = F.QMatrix.from_bytes(raw, ty, rows, cols)
    x = (np.random.default_rng(81).standard_normal(cols) * (0.1 if swiglu else 1.0)).astype(np.float32)
    xt = F.Tensor.from_vec(x, (1, cols))
    y64, wn = O.matmul_f64(x, raw, ty, rows, cols)
    if swiglu:
        n_ff = rows // 2
        got = xt.try_matmul_swiglu(w).to_vec()
        gate, up = y64[0, :n_ff], y64[0, n_ff:]
        want = gate / (1.0 + np.exp(-gate)) * up
        assert got.shape == (n_ff,) and np.abs(got - want).max() <= dot_bar() * np.abs(want).max()
        return
    got = xt.matmul_q(w).to_vec()
    err = np.abs(got - y64[0])
    assert (err <= 1e-3 * wn * np.linalg.norm(x.astype(np.float64))).all()
    assert err.max() <= dot_bar() * np.abs(y64).max()
    rb = row_bytes(ty, cols)
    for r0, n in ((0, 37), (rows - 50, 50), (rows // 2 & ~7, 1001)):
        if (r0 * rb) % 16:
            continue
        part = F.QMatrix.from_bytes(raw[r0 * rb:(r0 + n) * rb], ty, n, cols)
        assert np.array_equal(bits(xt.matmul_q(part).to_vec()), bits(got[r0:r0 + n])), r0
