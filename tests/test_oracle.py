"""Pins the CPU oracle (oracle/ferric_oracle.c) before anything is compared against it.

Evidence used, in order: vectors the reference's own tests hold (Q4_K known-answer block, f16
landmarks, the Q8_0 ground-truth generator and the three cpu_simd tests restated), a library routine
(numpy.float16 over all 65536 patterns), the two formulations the reference itself contains
(sequential dequantizer vs per-element random access), an independent numpy restatement, and
closed forms under single-field perturbations chosen so that a swapped nibble, a wrong scale index,
a dropped min term or a transposed operand fails.
"""
import numpy as np
import pytest

from conftest import bits

Q8_0, Q4_K, Q6_K = 8, 12, 14


def f16b(x):
    return int(np.array([x], dtype=np.float32).astype(np.float16).view(np.uint16)[0])


# ---------------------------------------------------------------- f16

def test_f16_exhaustive_against_numpy(O):
    got = O.f16_table()
    want = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(bits(got)[~nan], bits(want)[~nan])


def test_deq_raw_unquantized_types(O):
    # crates/ferric-gguf/src/lib.rs:499-501. F16 against numpy over every pattern; BF16 against torch's own bfloat16 -> float32
    # conversion over every pattern; F32 is the bytes as they are, NaN payloads included.
    import torch
    F32, F16, BF16 = 0, 1, 30
    pats = np.arange(65536, dtype=np.uint16)
    got = O.deq_raw(pats.view(np.uint8), 65536, F16)
    want = pats.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan) and np.array_equal(bits(got)[~nan], bits(want)[~nan])
    got = O.deq_raw(pats.view(np.uint8), 65536, BF16)
    want = torch.from_numpy(pats.view(np.int16).copy()).view(torch.bfloat16).to(torch.float32).numpy()
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan) and np.array_equal(bits(got)[~nan], bits(want)[~nan])
    assert bits(O.deq_raw(np.array([0x80, 0x3F], np.uint8), 1, BF16))[0] == 0x3F800000        # 1.0
    assert float(O.deq_raw(np.array([0x49, 0x40], np.uint8), 1, BF16)[0]) == 3.140625        # bf16(pi)
    raw32 = np.random.default_rng(0).integers(0, 1 << 32, 4096, dtype=np.uint64).astype(np.uint32)
    raw32[:4] = [0x7FC00001, 0xFF800000, 0x00000001, 0x80000000]
    assert np.array_equal(bits(O.deq_raw(raw32.view(np.uint8), 4096, F32)), raw32)
    assert O.deq_raw(raw32.view(np.uint8), 100, F32).size == 100 and O.deq_raw(np.zeros(0, np.uint8), 0, BF16).size == 0
    assert O.type_size(F32, 7) == 28 and O.type_size(F16, 7) == 14 and O.type_size(BF16, 7) == 14
    for ty, short in ((F32, 15), (F16, 7), (BF16, 7)):      # four elements asked for, bytes for three and a half
        with pytest.raises(AssertionError, match="out of range"):
            O.deq_raw(np.zeros(short, np.uint8), 4, ty)


def test_f16_reference_landmarks(O, golden):
    # crates/ferric-tensor/src/cpu_simd.rs:203-213
    t = O.f16_table()
    for b, v in zip(golden["f16_landmark_bits"], golden["f16_landmark_f32"]):
        assert bits(t[int(b)]) == bits(np.float32(v)), hex(int(b))
    assert abs(float(t[0x0001]) - 5.9604645e-8) < 1e-14
    assert np.isnan(t[0x7E00])


def test_f32_to_f16_matches_numpy_rne(O):
    rng = np.random.default_rng(0)
    xs = np.concatenate([rng.standard_normal(4000).astype(np.float32) * np.float32(s) for s in (1e-7, 1e-4, 1, 1e3, 1e5)])
    xs = np.concatenate([xs, np.array([0.0, -0.0, 65504.0, 65520.0, 1e-8, 6.1e-5, 0.05, 0.11], dtype=np.float32)])
    want = xs.astype(np.float16).view(np.uint16)
    got = np.array([O.f32_to_f16_bits(x) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- sizes / dispatch

def test_type_size_and_unknown_type(O):
    # crates/ferric-gguf/src/lib.rs:471-494; crates/ferric-tensor/src/dtype.rs:4204-4306 keeps these tables in step
    assert O.type_size(Q8_0, 4096 * 4096) == 17825792
    assert O.type_size(Q4_K, 5120 * 5120) == 14745600
    assert O.type_size(Q6_K, 5120 * 17408) == 73113600
    assert O.type_size(Q4_K, 300) == 144 and O.type_size(Q8_0, 31) == 0  # integer division truncates
    with pytest.raises(ValueError, match="unsupported ggml type 99"):
        O.type_size(99, 32)
    with pytest.raises(ValueError, match="unsupported ggml type 99"):
        O.deq_raw(np.zeros(34, np.uint8), 32, 99)


# ---------------------------------------------------------------- Q4_K

def test_q4k_reference_known_answer(O, golden):
    # crates/ferric-gguf/examples/roundtrip.rs:54-87 (its tolerance is 1e-3; the values are exact)
    got = O.deq_raw(golden["q4k_known_block"], 256, Q4_K)
    assert np.array_equal(bits(got), bits(golden["q4k_known_expected"]))
    assert np.array_equal(got[:8], np.arange(8, dtype=np.float32))          # low nibbles of qs[0..8]
    assert np.array_equal(got[32:40], (np.arange(8) + 3) % 8)               # then the high nibbles
    assert not got[128:].any()                                              # sub-blocks 4..7 have scale 0


def test_q4k_scale_pack_unpack_identity_exhaustive(O):
    # every (sub-block j, sc, m) survives the packing of q4_k.rs:23-33 and get_sc_min (lib.rs:795-804)
    from ferric_amd.synth import q4k_pack_scales
    sc, m = np.meshgrid(np.arange(64, dtype=np.uint8), np.arange(64, dtype=np.uint8), indexing="ij")
    sc, m = sc.reshape(-1), m.reshape(-1)
    for j in range(8):
        scs = np.zeros((4096, 8), np.uint8); ms = np.zeros((4096, 8), np.uint8)
        scs[:, j], ms[:, j] = sc, m
        # other sub-blocks carry the complement so cross-talk between fields would show
        for o in range(8):
            if o != j:
                scs[:, o], ms[:, o] = 63 - sc, 63 - m
        packed = q4k_pack_scales(scs, ms)
        nsc, nm = O.np_q4k_scales(packed)
        assert np.array_equal(nsc, scs) and np.array_equal(nm, ms)
        for k in range(0, 4096, 97):  # the C closure on a sample
            assert O.q4k_get_sc_min(packed[k], j) == (int(sc[k]), int(m[k]))


def _q4k_block(d=1.0, dmin=0.0, sc=None, m=None, qs=None):
    from ferric_amd.synth import q4k_pack_scales
    b = np.zeros(144, np.uint8)
    b[0:2] = np.frombuffer(f16b(d).to_bytes(2, "little"), np.uint8)
    b[2:4] = np.frombuffer(f16b(dmin).to_bytes(2, "little"), np.uint8)
    sc = np.zeros(8, np.uint8) if sc is None else np.asarray(sc, np.uint8)
    m = np.zeros(8, np.uint8) if m is None else np.asarray(m, np.uint8)
    b[4:16] = q4k_pack_scales(sc[None], m[None])[0]
    if qs is not None:
        b[16:] = qs
    return b


def test_q4k_single_field_perturbations(O):
    # one nibble set: exactly one output is d*sc*nib, at the position the layout dictates
    for byte, hi in ((0, 0), (0, 1), (31, 0), (37, 1), (100, 0), (127, 1)):
        qs = np.zeros(128, np.uint8)
        qs[byte] = (9 << 4) if hi else 9
        sc = np.arange(1, 9)
        y = O.deq_raw(_q4k_block(d=0.5, sc=sc, qs=qs), 256, Q4_K)
        g, l = byte // 32, byte % 32
        pos = 64 * g + 32 * hi + l
        assert np.count_nonzero(y) == 1 and y[pos] == np.float32(0.5) * sc[2 * g + hi] * 9
    # only mins: y = -(dmin*m_j) on all 32 values of sub-block j, nothing from the quants
    m = np.array([3, 60, 7, 33, 63, 1, 47, 16])
    y = O.deq_raw(_q4k_block(d=1.0, dmin=0.25, m=m, qs=np.full(128, 0xFF, np.uint8)), 256, Q4_K)
    assert np.array_equal(y, np.repeat(-(np.float32(0.25) * m.astype(np.float32)), 32))
    # d and dmin are not swapped, and the subtraction is y = d*sc*q - dmin*m (not +)
    y = O.deq_raw(_q4k_block(d=2.0, dmin=0.5, sc=np.full(8, 3), m=np.full(8, 5), qs=np.full(128, 0x11, np.uint8)), 256, Q4_K)
    assert np.all(y == np.float32(2 * 3 * 1 - 0.5 * 5))


def test_q4k_rounding_is_two_products_then_subtract(O):
    # (d*sc)*q - (dmin*m) with every operation rounded to f32, compared with the same expression in
    # numpy float32. d has 11 significant bits, sc 6 and q 4, so both products are EXACT in f32 and
    # the subtraction is the only rounding: a fused multiply-add cannot change the result either.
    from ferric_amd.synth import synth_weights
    w = synth_weights(Q4_K, 4, 2048, 11)
    y = O.deq_raw(w, 4 * 2048, Q4_K)
    b = w.reshape(-1, 144)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32); dmin = b[:, 2:4].copy().view(np.float16).astype(np.float32)
    sc, m = O.np_q4k_scales(b[:, 4:16])
    qs = b[:, 16:].reshape(-1, 4, 32)
    nib = np.stack([qs & 15, qs >> 4], 2).reshape(-1, 8, 32).astype(np.float32)
    d1 = (d * sc.astype(np.float32))[:, :, None]; mm = (dmin * m.astype(np.float32))[:, :, None]
    assert np.array_equal(bits(y), bits((d1 * nib - mm).reshape(-1)))
    assert np.array_equal((d1 * nib).astype(np.float64), d1.astype(np.float64) * nib)      # exact product
    exact = d.astype(np.float64)[:, :, None] * sc[:, :, None] * nib - dmin.astype(np.float64)[:, :, None] * m[:, :, None]
    assert np.array_equal(bits(y), bits(exact.astype(np.float32).reshape(-1)))              # = correctly rounded true value


# ---------------------------------------------------------------- Q6_K

def _q6k_block(d=1.0, sc=None, ql=None, qh=None):
    b = np.zeros(210, np.uint8)
    if ql is not None: b[0:128] = ql
    if qh is not None: b[128:192] = qh
    b[192:208] = (np.zeros(16, np.int8) if sc is None else np.asarray(sc, np.int8)).view(np.uint8)
    b[208:210] = np.frombuffer(f16b(d).to_bytes(2, "little"), np.uint8)
    return b


def test_q6k_single_field_perturbations(O):
    sc = np.array([1, -2, 3, -4, 5, -6, 7, -8, 9, -10, 11, -12, 13, -14, 15, -16])
    # all-zero quants: every q = -32, y = d*sc*(-32) with scale index 8*half + l/16 + 2*group
    y = O.deq_raw(_q6k_block(d=0.5, sc=sc), 256, Q6_K)
    idx = np.arange(256)
    want_sc = sc[8 * (idx // 128) + (idx % 32) // 16 + 2 * ((idx % 128) // 32)]
    assert np.array_equal(y, np.float32(0.5) * want_sc.astype(np.float32) * np.float32(-32))
    # a single ql nibble / a single qh pair moves exactly one output, to the textbook position
    ones = np.ones(16)
    base = O.deq_raw(_q6k_block(sc=ones), 256, Q6_K)
    for byte, hi, pos in ((0, 0, 0), (0, 1, 64), (32, 0, 32), (45, 1, 96 + 13), (64, 0, 128), (100, 1, 128 + 96 + 4)):
        ql = np.zeros(128, np.uint8); ql[byte] = (5 << 4) if hi else 5
        y = O.deq_raw(_q6k_block(sc=ones, ql=ql), 256, Q6_K)
        diff = np.nonzero(y != base)[0]
        assert list(diff) == [pos] and y[pos] == -32 + 5
    for byte, shift, pos in ((0, 0, 0), (0, 2, 32), (7, 4, 64 + 7), (31, 6, 96 + 31), (32, 0, 128), (40, 6, 128 + 96 + 8)):
        qh = np.zeros(64, np.uint8); qh[byte] = 3 << shift
        y = O.deq_raw(_q6k_block(sc=ones, qh=qh), 256, Q6_K)
        diff = np.nonzero(y != base)[0]
        assert list(diff) == [pos] and y[pos] == -32 + 48
    # d (11 bits) * sc (7 bits) * q (6 bits) is exact in f32 whatever the association, so the
    # result is the exactly representable true product
    from ferric_amd.synth import synth_weights
    w = synth_weights(Q6_K, 4, 1024, 5)
    y = O.deq_raw(w, 4096, Q6_K)
    assert np.array_equal(bits(y), bits(O.np_deq_q6_k(w, 4096)))
    blk = w.reshape(-1, 210)
    d = blk[:, 208:210].copy().view(np.float16).astype(np.float64)
    scb = blk[:, 192:208].view(np.int8).astype(np.float64)
    idx = np.arange(256)
    scl = scb[:, 8 * (idx // 128) + (idx % 32) // 16 + 2 * ((idx % 128) // 32)]
    ok = (d * scl) != 0
    q = y.reshape(-1, 256).astype(np.float64)[ok] / (d * scl)[ok]
    assert np.array_equal(q, np.rint(q)) and q.min() >= -32 and q.max() <= 31
    assert not y.reshape(-1, 256)[~ok].any()


# ---------------------------------------------------------------- all formats: formulations agree

@pytest.mark.parametrize("ty", [Q8_0, Q4_K, Q6_K])
def test_sequential_elementwise_and_numpy_agree(O, ty):
    from ferric_amd.synth import synth_weights
    for seed, (rows, cols) in enumerate([(3, 256), (16, 1024), (5, 5120)]):
        w = synth_weights(ty, rows, cols, 100 + seed)
        n = rows * cols
        a = O.deq_raw(w, n, ty)
        assert np.array_equal(bits(a), bits(O.deq_elemwise(w, n, ty)))   # dtype.rs:2078-2086 / :1236-1246 / :1351-1356
        assert np.array_equal(bits(a), bits(O.np_deq_raw(w, n, ty)))
    # every byte value in every position (uniform random bytes), finite scales
    rng = np.random.default_rng(9)
    vals, nbytes = O.BLOCK[ty]
    raw = rng.integers(0, 256, 64 * nbytes, dtype=np.uint8).reshape(64, nbytes)
    for off in {Q8_0: (0,), Q4_K: (0, 2), Q6_K: (208,)}[ty]:
        raw[:, off + 1] &= 0x3B  # clear exponent top bit -> finite f16
    a = O.deq_raw(raw, 64 * vals, ty)
    assert np.array_equal(bits(a), bits(O.deq_elemwise(raw, 64 * vals, ty)))
    assert np.array_equal(bits(a), bits(O.np_deq_raw(raw.reshape(-1), 64 * vals, ty)))


def test_golden_generator_blocks(O, golden):
    # the reference's deterministic generators, re-derived in Python integers by tests/golden/make_golden.py
    for s in (1, 2, 3, 4):
        assert np.array_equal(O.gen_q4k_block(s), golden["q4k_gen_blocks"][(s - 1) * 144: s * 144])
        assert np.array_equal(O.gen_q6k_block(s), golden["q6k_gen_blocks"][(s - 1) * 210: s * 210])
    assert np.array_equal(bits(O.deq_raw(golden["q4k_gen_blocks"], 1024, Q4_K)), bits(golden["q4k_gen_deq"]))
    assert np.array_equal(bits(O.deq_raw(golden["q6k_gen_blocks"], 1024, Q6_K)), bits(golden["q6k_gen_deq"]))
    # q4_k.rs:17-18: d = f16(0.05 + 0.01*(seed%7)) etc. decode to the expected scales
    b = golden["q4k_gen_blocks"][:144]
    assert abs(O.f16_to_f32(int(b[0]) | int(b[1]) << 8) - 0.06) < 1e-4 and abs(O.f16_to_f32(int(b[2]) | int(b[3]) << 8) - 0.025) < 1e-4


def test_ragged_tails(O):
    from ferric_amd.synth import synth_weights
    # K-quants: output pre-sized to n, ragged tail stays 0.0 (lib.rs:794, :722); Q8_0 returns whole blocks only (lib.rs:609-614)
    w = synth_weights(Q4_K, 1, 512, 1)
    y = O.deq_raw(w, 700, Q4_K)
    assert y.size == 700 and np.array_equal(y[:512], O.deq_raw(w, 512, Q4_K)) and not y[512:].any()
    y = O.deq_raw(w[:144 + 50], 512, Q4_K)       # bytes run out first: chunks_exact drops the partial block
    assert y.size == 512 and not y[256:].any() and y[:256].any()
    w = synth_weights(Q6_K, 1, 256, 1)
    assert O.deq_raw(w, 300, Q6_K).size == 300
    w = synth_weights(Q8_0, 1, 64, 1)
    assert O.deq_raw(w, 70, Q8_0).size == 64 and O.deq_raw(w[:40], 64, Q8_0).size == 32 and O.deq_raw(w, 0, Q8_0).size == 0


# ---------------------------------------------------------------- Q8_0 CPU mat-vec: the reference's own tests restated

def test_q8_dequant_matches_ground_truth_built_beside_the_bytes(O, golden):
    # cpu_simd.rs:136-156: values built while the bytes are written, not through the dequantizer
    assert np.array_equal(bits(O.deq_raw(golden["q8_synth_raw"], 512, Q8_0)), bits(golden["q8_synth_vals"]))
    raw, vals = O.gen_q8_0_synth(8, 64, 8 * 13 + 64)
    assert np.array_equal(raw, golden["q8_synth_raw"]) and np.array_equal(bits(vals), bits(golden["q8_synth_vals"]))


def test_matvec_matches_the_dequantised_reference(O):
    # cpu_simd.rs:162-173
    for rows, cols in [(1, 32), (8, 64), (17, 256), (64, 512)]:
        raw, vals = O.gen_q8_0_synth(rows, cols, rows * 13 + cols)
        x = ((np.arange(cols) * 37 % 101).astype(np.float32) - 50.0) / np.float32(50.0)
        got = O.matvec_q8_0(x, raw, rows, cols)
        want = (vals.reshape(rows, cols).astype(np.float64) * x).sum(1)
        scale = max(1e-6, np.abs(want).max())
        assert np.abs(got - want).max() / scale < 1e-5


def test_threading_changes_nothing_about_the_answer(O):
    # cpu_simd.rs:175-186
    raw, _ = O.gen_q8_0_synth(64, 256, 7)
    x = np.sin(np.arange(256, dtype=np.float32) * np.float32(0.01))
    one = O.matvec_q8_0(x, raw, 64, 256)
    for t in (2, 3, 8, 64, 128):
        assert np.array_equal(bits(one), bits(O.matvec_q8_0_threaded(x, raw, 64, 256, t))), t


def test_spans_concatenate_to_the_whole(O):
    # cpu_simd.rs:188-200
    raw, _ = O.gen_q8_0_synth(40, 128, 3)
    x = (np.arange(128) % 7).astype(np.float32) - 3.0
    whole = O.matvec_q8_0(x, raw, 40, 128)
    for cut in (0, 1, 17, 39, 40):
        joined = np.concatenate([O.matvec_q8_0_span(x, raw, 128, 0, cut, 2), O.matvec_q8_0_span(x, raw, 128, cut, 40, 2)])
        assert np.array_equal(bits(whole), bits(joined)), cut


def test_row_q8_0_accumulation_order(O):
    # per block: part = sum_j x_j*q_j sequentially in f32, then acc += part*d (cpu_simd.rs:64-70)
    raw, _ = O.gen_q8_0_synth(3, 96, 5)
    x = np.random.default_rng(1).standard_normal(96).astype(np.float32)
    got = O.matvec_q8_0(x, raw, 3, 96)
    b = raw.reshape(3, 3, 34)
    for r in range(3):
        acc = np.float32(0)
        for k in range(3):
            d = b[r, k, 0:2].copy().view(np.float16).astype(np.float32)[0]
            part = np.float32(0)
            for j in range(32):
                part = np.float32(part + x[k * 32 + j] * np.float32(np.int8(b[r, k, 2 + j].view(np.int8))))
            acc = np.float32(acc + np.float32(part * d))
        assert bits(acc) == bits(got[r])
    with pytest.raises(AssertionError):
        O.matvec_q8_0(x[:33], raw[:34], 1, 33)            # cols % 32 (cpu_simd.rs:80)
    with pytest.raises(AssertionError):
        O.matvec_q8_0(x, raw[:-1], 3, 96)                 # byte length (cpu_simd.rs:83)


def test_kquant_cpu_matmul_is_dequant_then_sequential_dot(O):
    from ferric_amd.synth import synth_weights
    for ty in (Q4_K, Q6_K, Q8_0):
        w = synth_weights(ty, 6, 512, 2)
        x = np.random.default_rng(2).standard_normal((2, 512)).astype(np.float32)
        got = O.matmul_cpu(x, w, ty, 6, 512, threads=3)
        deq = O.deq_raw(w, 6 * 512, ty).reshape(6, 512)
        for t in range(2):
            for r in range(6):
                s = np.float32(0)
                for l in range(512):
                    s = np.float32(s + np.float32(x[t, l] * deq[r, l]))
                assert bits(s) == bits(got[t, r])
        y64, wn = O.matmul_f64(x, w, ty, 6, 512)
        assert np.allclose(y64, x.astype(np.float64) @ deq.astype(np.float64).T, rtol=1e-12, atol=1e-12)
        assert np.allclose(wn, np.linalg.norm(deq.astype(np.float64), axis=1))


def test_golden_gemv_vectors(O, golden):
    x = golden["gemv_x"]
    assert np.array_equal(bits(x), bits(np.cos(np.arange(256, dtype=np.float32) * np.float32(0.013)).astype(np.float32)))
    for name, ty in (("q4k", Q4_K), ("q6k", Q6_K), ("q8_0", Q8_0)):
        w = golden[f"gemv_{name}_w"]
        y = O.matmul_cpu(x, w, ty, 8, 256)[0]
        want = golden[f"gemv_{name}_y64"]
        assert np.abs(y - want).max() / max(1e-3, np.abs(want).max()) < 1e-5     # the reference examples' bar (q4_k.rs:54)


def test_quant_q8_0_roundtrip(O):
    # crates/ferric-gguf/src/lib.rs:985-997 and examples/roundtrip.rs:47-52 (relative error < 0.02)
    w = (np.sin(np.arange(13 * 128, dtype=np.float32) * np.float32(0.021)) * np.float32(0.7)).astype(np.float32)
    q = O.quant_q8_0(w)
    back = O.deq_raw(q, w.size, Q8_0)
    assert np.abs(back - w).max() / np.abs(w).max() < 0.02
    blk = q[:34]
    amax = np.abs(w[:32]).max()
    assert int(blk[0]) | int(blk[1]) << 8 == f16b(amax / np.float32(127.0))
    assert np.abs(blk[2:].view(np.int8)).max() == 127


def test_swiglu_formula(O):
    # crates/ferric-tensor/src/dtype.rs:2408 and lib.rs:2616: (g / (1 + exp(-g))) * u, [gate | up] per row
    rng = np.random.default_rng(4)
    gu = rng.standard_normal((3, 2 * 40)).astype(np.float32) * 3
    out = O.swiglu(gu, 40)
    g, u = gu[:, :40].astype(np.float64), gu[:, 40:].astype(np.float64)
    assert np.allclose(out, g / (1 + np.exp(-g)) * u, rtol=1e-6, atol=1e-7)
    assert O.swiglu(np.zeros((1, 8), np.float32), 4).tolist() == [[0.0] * 4]
