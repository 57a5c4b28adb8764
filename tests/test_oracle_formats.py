"""Pins the oracle's dequantizers for the further block formats (Q4_0, Q4_1, Q5_0, Q5_1, Q5_K, IQ4_NL, IQ4_XS, MXFP4).
MXFP4 has known-answer data captured from ggml in the reference's own tests (tests/golden/mxfp4_ggml.json); for the
others the reference tree holds no known-answer vectors, so each sequential restatement (crates/ferric-gguf/src/lib.rs:618-716)
must agree bit for bit with (i) the element formula of the reference's own GPU kernels, restated separately
(crates/ferric-tensor/src/dtype.rs:3548-3555, 3613-3620, 3778-3792, 3858-3874, 1108-1121), (ii) a numpy twin written
from the block layout, and satisfy (iii) closed-form relations to the formats pinned in test_oracle.py and (iv)
single-field perturbations with known answers."""
import numpy as np
import pytest

from conftest import bits

Q8_0, Q4_K, Q6_K, Q4_0, Q4_1, Q5_0, Q5_1, Q5_K = 8, 12, 14, 2, 3, 6, 7, 13
IQ4_NL, IQ4_XS, MXFP4 = 20, 23, 39
NEW = [Q4_0, Q4_1, Q5_0, Q5_1, Q5_K, IQ4_NL, IQ4_XS, MXFP4]
GEOM = {Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q5_K: (256, 176), IQ4_NL: (32, 18), IQ4_XS: (256, 136),
        MXFP4: (32, 17)}
KV = [-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113]


def f16b(v):
    return np.array([v], np.float16).view(np.uint8)


@pytest.mark.parametrize("ty", NEW)
def test_three_formulations_agree_bit_for_bit(O, ty):
    from ferric_amd.synth import synth_weights
    vals, nbytes = GEOM[ty]
    assert O.type_size(ty, vals * 7 + 5) == 7 * nbytes
    for seed in range(3):
        raw = synth_weights(ty, 24, vals * 3, seed)
        n = 24 * vals * 3
        a = O.deq_raw(raw, n, ty)
        assert np.array_equal(bits(a), bits(O.deq_elemwise(raw, n, ty)))
        assert np.array_equal(bits(a), bits(O.np_deq_raw(raw, n, ty)))
    # every byte value in every position of one block, scales included (f16 specials: inf/nan propagate identically)
    rng = np.random.default_rng(9)
    blk = rng.integers(0, 256, (512, nbytes), dtype=np.uint8)
    blk[:256, :] = np.arange(256, dtype=np.uint8).reshape(256, 1)
    raw = blk.reshape(-1)
    a, b, c = O.deq_raw(raw, 512 * vals, ty), O.deq_elemwise(raw, 512 * vals, ty), O.np_deq_raw(raw, 512 * vals, ty)
    ok = ~np.isnan(a)
    assert np.array_equal(np.isnan(a), np.isnan(b)) and np.array_equal(np.isnan(a), np.isnan(c))
    assert np.array_equal(bits(a)[ok], bits(b)[ok]) and np.array_equal(bits(a)[ok], bits(c)[ok])


def test_closed_forms_q4_0_q4_1(O):
    blk = np.zeros(18, np.uint8); blk[0:2] = f16b(0.5); blk[2:] = np.arange(16) | ((15 - np.arange(16)) << 4)
    want = np.concatenate([np.arange(16) - 8, (15 - np.arange(16)) - 8]) * 0.5
    assert np.array_equal(O.deq_raw(blk, 32, Q4_0), want.astype(np.float32))
    b1 = np.zeros(20, np.uint8); b1[0:2] = f16b(0.5); b1[2:4] = f16b(-4.0); b1[4:] = blk[2:]
    assert np.array_equal(O.deq_raw(b1, 32, Q4_1), O.deq_raw(blk, 32, Q4_0))          # m = -8d: the affine form is Q4_0
    b1[2:4] = f16b(3.0)
    assert np.array_equal(O.deq_raw(b1, 32, Q4_1), ((want / 0.5 + 8) * 0.5 + 3.0).astype(np.float32))


def test_closed_forms_q5_0_q5_1_and_the_fifth_bit(O):
    rng = np.random.default_rng(5)
    qs = rng.integers(0, 256, 16, dtype=np.uint8)
    b40 = np.zeros(18, np.uint8); b40[0:2] = f16b(0.25); b40[2:] = qs
    b50 = np.zeros(22, np.uint8); b50[0:2] = f16b(0.25); b50[6:] = qs
    assert np.array_equal(O.deq_raw(b50, 32, Q5_0), O.deq_raw(b40, 32, Q4_0) - np.float32(2.0))   # qh = 0: (n-16)d = (n-8)d - 8d
    for v in range(32):                                                                            # bit v of qh adds 16d to value v only
        one = b50.copy(); one[2:6] = np.array([1 << v], "<u4").view(np.uint8)
        diff = O.deq_raw(one, 32, Q5_0) - O.deq_raw(b50, 32, Q5_0)
        want = np.zeros(32, np.float32); want[v] = 4.0
        assert np.array_equal(diff, want), v
    b41 = np.zeros(20, np.uint8); b41[0:2] = f16b(0.25); b41[2:4] = f16b(1.5); b41[4:] = qs
    b51 = np.zeros(24, np.uint8); b51[0:2] = f16b(0.25); b51[2:4] = f16b(1.5); b51[8:] = qs
    assert np.array_equal(O.deq_raw(b51, 32, Q5_1), O.deq_raw(b41, 32, Q4_1))                     # qh = 0: Q5_1 is Q4_1
    b51[4:8] = 0xFF
    assert np.array_equal(O.deq_raw(b51, 32, Q5_1), O.deq_raw(b41, 32, Q4_1) + np.float32(4.0))   # all fifth bits: + 16d


def test_q5_k_reduces_to_q4_k_and_its_high_bits_are_where_the_layout_says(O):
    from ferric_amd.synth import synth_weights
    k4 = synth_weights(Q4_K, 3, 256, 2).reshape(3, 144)
    k5 = np.zeros((3, 176), np.uint8)
    k5[:, :16] = k4[:, :16]; k5[:, 48:] = k4[:, 16:]
    assert np.array_equal(O.deq_raw(k5.reshape(-1), 768, Q5_K), O.deq_raw(k4.reshape(-1), 768, Q4_K))   # qh = 0
    # bit s of qh[l] adds 16 * d * sc_s to element 32 s + l and to nothing else
    blk = k5[0].copy()
    base = O.deq_raw(blk, 256, Q5_K)
    d = np.frombuffer(blk[0:2].tobytes(), np.float16)[0].astype(np.float32)
    for s in range(8):
        for l in (0, 5, 31):
            one = blk.copy(); one[16 + l] = 1 << s
            sc, _ = O.q4k_get_sc_min(blk[4:16], s)
            got = O.deq_raw(one, 256, Q5_K)
            changed = np.nonzero(got != base)[0]
            if sc == 0 or d == 0:
                assert changed.size == 0
                continue
            assert list(changed) == [32 * s + l]
            # y = (d*sc)*(n+16) - mm versus (d*sc)*n - mm, each rounded once: compare through the oracle's own products
            ds = np.float32(d * np.float32(sc))
            n = (blk[48 + 32 * (s >> 1) + l] >> (4 * (s & 1))) & 15
            _, m = O.q4k_get_sc_min(blk[4:16], s)
            mm = np.float32(np.frombuffer(blk[2:4].tobytes(), np.float16)[0].astype(np.float32) * np.float32(m))
            assert got[32 * s + l] == np.float32(np.float32(ds * np.float32(n + 16)) - mm)


@pytest.mark.parametrize("ty", NEW)
def test_ragged_inputs_follow_the_reference(O, ty):
    from ferric_amd.synth import synth_weights
    vals, nbytes = GEOM[ty]
    raw = synth_weights(ty, 1, vals * 4, 1)
    full = O.deq_raw(raw, vals * 4, ty)
    # n beyond the bytes present: whole blocks present are filled, the rest of the n-long output stays zero (vec![0.0; n])
    short = O.deq_raw(raw[: 2 * nbytes + 3], vals * 4, ty)
    assert short.size == vals * 4 and np.array_equal(short[: 2 * vals], full[: 2 * vals]) and not short[2 * vals:].any()
    # n not a multiple of the block: the trailing partial block is left zero
    part = O.deq_raw(raw, vals * 2 + 7, ty)
    assert part.size == vals * 2 + 7 and np.array_equal(part[: 2 * vals], full[: 2 * vals]) and not part[2 * vals:].any()


# ---------------------------------------------------------------- MXFP4: ggml-captured known answers

def _mxfp4_golden():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "mxfp4_ggml.json")) as f:
        return json.load(f)


def test_mxfp4_grid_is_bit_identical_to_ggml(O):
    # crates/ferric-gguf/src/lib.rs:1173-1200: each code in the low nibble of qs[0] (element 0) and in the high nibble
    # (element 16), under ten scale bytes that include both subnormal and both saturating ends
    g = _mxfp4_golden()
    for form in (O.deq_raw, O.deq_elemwise, O.np_deq_raw):
        for ei, e in enumerate(g["e"]):
            for code in range(16):
                want = g["grid_bits"][ei * 16 + code]
                blk = np.zeros(17, np.uint8); blk[0] = e; blk[1] = code
                assert bits(form(blk, 32, MXFP4))[0] == want, (form.__name__, e, code)
                blk[1] = code << 4
                hi = bits(form(blk, 32, MXFP4))
                assert hi[16] == want and hi[0] == 0, (form.__name__, e, code)


def test_mxfp4_real_blocks_are_bit_identical_to_ggml(O):
    # crates/ferric-gguf/src/lib.rs:1205-1222: 8 blocks of a released checkpoint, three distinct exponents, 17-byte stride
    g = _mxfp4_golden()
    raw = np.array(g["real_raw"], np.uint8)
    want = np.array(g["real_bits"], np.uint32)
    for form in (O.deq_raw, O.deq_elemwise, O.np_deq_raw):
        assert np.array_equal(bits(form(raw, 256, MXFP4)), want), form.__name__
    assert O.type_size(MXFP4, 802816) == 426496            # lib.rs:1224-1229, the measured on-disk length of an 896x896 tensor


def test_mxfp4_every_scale_and_code_against_ldexp(O):
    # all 256 x 16 (scale, code) pairs: table[code] / 2 * 2^(e - 127) through f64 ldexp, rounded once to f32
    blk = np.zeros((256, 17), np.uint8)
    blk[:, 0] = np.arange(256)
    blk[:, 1:9] = np.arange(16, dtype=np.uint8).reshape(8, 2)[:, 0] | (np.arange(16, dtype=np.uint8).reshape(8, 2)[:, 1] << 4)
    mag = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, 0, -.5, -1, -1.5, -2, -3, -4, -6])
    got = O.deq_raw(blk.reshape(-1), 256 * 32, MXFP4).reshape(256, 32)
    codes = np.concatenate([blk[:, 1:] & 15, blk[:, 1:] >> 4], axis=1)
    with np.errstate(over="ignore"):
        want = np.ldexp(mag[codes], np.arange(256).reshape(256, 1) - 127).astype(np.float32)
    assert np.array_equal(bits(got), bits(want))
    # e = 255: code 1 (element 16) is the finite 2^127, code 2 (element 1) saturates, code 0 stays +0.0
    assert got[255, 16] == np.float32(2.0 ** 127) and np.isinf(got[255, 1]) and bits(got[255])[0] == 0


# ---------------------------------------------------------------- IQ4_NL / IQ4_XS: closed forms

def test_iq4_nl_codebook_and_nibble_order(O):
    blk = np.zeros(18, np.uint8); blk[0:2] = f16b(1.0)
    blk[2:] = np.arange(16) | ((15 - np.arange(16)) << 4)
    want = np.array(KV + KV[::-1], np.float32)             # element j: index j; element 16 + j: index 15 - j
    assert np.array_equal(O.deq_raw(blk, 32, IQ4_NL), want)
    blk[0:2] = f16b(-0.375)
    assert np.array_equal(O.deq_raw(blk, 32, IQ4_NL), want * np.float32(-0.375))
    assert KV == sorted(KV) and KV[0] == -127 and KV[8] == 1 and sum(KV) == -94   # 16 increasing int8 levels, denser near 0


def test_iq4_xs_sub_scales_sit_where_the_layout_says(O):
    rng = np.random.default_rng(4)
    qs = rng.integers(0, 256, 128, dtype=np.uint8)
    nl = np.zeros((8, 18), np.uint8); nl[:, 0:2] = f16b(0.5); nl[:, 2:] = qs.reshape(8, 16)
    as_nl = O.deq_raw(nl.reshape(-1), 256, IQ4_NL)         # the same indices under a plain scale of 0.5

    def xs(ls):                                             # ls[ib] in 0..63 -> one super-block with d = 0.5
        b = np.zeros(136, np.uint8); b[0:2] = f16b(0.5)
        sh = 0
        for ib, v in enumerate(ls):
            b[4 + ib // 2] |= (v & 15) << (4 * (ib % 2))
            sh |= (v >> 4) << (2 * ib)
        b[2], b[3] = sh & 255, sh >> 8
        b[8:] = qs
        return b
    assert np.array_equal(O.deq_raw(xs([33] * 8), 256, IQ4_XS), as_nl)             # ls - 32 = 1: exactly IQ4_NL
    assert not O.deq_raw(xs([32] * 8), 256, IQ4_XS).any()                           # ls - 32 = 0
    for ib in range(8):
        for v in (0, 15, 16, 48, 63):                       # low nibble only, each high bit alone, everything
            ls = [33] * 8; ls[ib] = v
            want = as_nl.copy(); want[32 * ib: 32 * ib + 32] *= np.float32(v - 32)
            assert np.array_equal(O.deq_raw(xs(ls), 256, IQ4_XS), want), (ib, v)
