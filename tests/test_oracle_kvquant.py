"""Pins the numpy restatement of the block-quantized KV cache (oracle/kvquant_oracle.py): the reference's own known-answer
constructions (crates/ferric-tensor/src/kvquant.rs:1451-1580: blocks whose codes are fixed by construction, exactly
representable data, ties, the all-zero block), a scalar formulation in pure Python with every operation rounded to f32
through `struct`, f16 conversion against `struct`'s, and the error bounds the formats imply."""
import math
import struct

import numpy as np
import pytest

from oracle import kvquant_oracle as K

FMTS = [K.Q8_0, K.Q4_0, K.Q4_1]


def f32(x):
    return struct.unpack("<f", struct.pack("<f", x))[0]


def exact_case(rows, width, fmt, seed):
    """kvquant.rs:1458-1503 with numpy's generator in place of the reference's Lcg: every value an integer code times a power of
    two, each block pinning its own scale by holding the extreme code(s); one block in eight all zero."""
    r = np.random.default_rng(seed)
    nblk = rows * (width // 32)
    x = np.zeros((nblk, 32), np.float32)
    want = np.zeros((nblk, 32), np.int64)
    for b in range(nblk):
        s = 2.0 ** (-3 + b % 5)
        pin = int(r.integers(32))
        if fmt == K.Q8_0:
            c = r.integers(255, size=32) - 127
            c[pin] = -127
            v = c * s
        elif fmt == K.Q4_0:
            c = r.integers(16, size=32)
            c[pin] = 0                         # the -8 end: the value of largest magnitude is negative and d = s
            v = (c - 8) * s
        else:
            c = r.integers(16, size=32)
            c[pin], c[(pin + 1) % 32] = 0, 15  # min and max are exactly -4 s and 11 s
            v = (c - 4) * s
        if b % 8 == 3:
            v = np.zeros(32)
            c = np.full(32, {K.Q8_0: 0, K.Q4_0: 8, K.Q4_1: 0}[fmt])      # floor(0 + 8.5) = 8, floor(0.5) = 0
        x[b], want[b] = v, c
    # blocks run along the row: [rows, width] holds block b at row b // nblk_per_row
    return x.reshape(rows, width), want


@pytest.mark.parametrize("fmt", FMTS)
def test_codes_fixed_by_construction_and_exact_round_trips(fmt):
    rows, width = 7, 96                          # three blocks per row: an odd count, scale pairs straddle rows
    x, want = exact_case(rows, width, fmt, 7)
    c = K.quantize(x, rows, width, fmt)
    for b in range(rows * 3):
        assert np.array_equal(K.codes_of(c, b), want[b]), (fmt, b)
    x, _ = exact_case(5, 64, fmt, 11)
    assert np.array_equal(K.roundtrip(x, 5, 64, fmt), x)


def test_ties_round_away_from_zero():
    x = np.zeros(32, np.float32)                 # kvquant.rs:1559-1575
    x[0] = 127.0
    x[1:7] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5]
    assert list(K.codes_of(K.quantize(x, 1, 32, K.Q8_0), 0)[1:7]) == [1, 2, 3, -1, -2, -3]


def test_sizes_and_layout():
    assert [K.BLOCK_BYTES[f] * 8 / 32 for f in FMTS] == [8.5, 4.5, 5.0]              # kvquant.rs:1-7, :91-93
    assert K.sizes(7, 96, K.Q8_0) == (21 * 8, 11) and K.sizes(7, 96, K.Q4_0) == (21 * 4, 11) and K.sizes(7, 96, K.Q4_1) == (21 * 4, 21)
    for fmt in FMTS:                             # bytes of the packed arrays = the llama.cpp block size, up to the shared last word
        c = K.Cache(fmt, 4, 64)
        assert c.codes.nbytes + c.scales.nbytes == 8 * K.BLOCK_BYTES[fmt]
    # block b = row * nblk + col / 32; byte i of a 4-bit block holds value i (low nibble) and i + 16 (high)
    x = np.zeros((2, 64), np.float32)
    x[1, 32:48] = np.arange(16) - 8              # Q4_0: the largest magnitude is -8 -> d = 1, codes 0..15, then 16 values at the top code
    x[1, 48:] = 7
    c = K.quantize(x, 2, 64, K.Q4_0)
    assert list(K.codes_of(c, 3)) == list(range(16)) + [15] * 16
    assert int(c.codes[3, 0]) == (0 | 15 << 4) | (1 | 15 << 4) << 8 | (2 | 15 << 4) << 16 | (3 | 15 << 4) << 24
    assert np.array_equal(K.codes_of(c, 0), np.full(32, 8)) and c.scales[0] == 0x8000      # 0.0 / -8.0 = -0.0 in the scale


def test_f16_conversion_against_struct():
    rng = np.random.default_rng(3)
    vals = np.concatenate([rng.standard_normal(4000) * 10.0 ** rng.integers(-9, 5, 4000), [0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9,
                           -1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 6.1e-5, 5.96e-8, np.inf, -np.inf]]).astype(np.float32)
    # ties on the f16 grid: halfway between neighbours, to even
    grid = np.arange(0x3C00, 0x3C10, dtype=np.uint16).view(np.float16).astype(np.float32)
    vals = np.concatenate([vals, (grid[:-1] + grid[1:]) / 2]).astype(np.float32)
    got = K.f32_to_f16_bits(vals)
    for v, g in zip(vals, got):
        try:
            w = struct.unpack("<H", struct.pack("<e", float(v)))[0]
        except OverflowError:
            w = 0x7C00 | (0x8000 if v < 0 else 0)
        assert g == w, (v, hex(g), hex(w))
    nan = np.array([0x7FC12345, 0xFF800001], np.uint32).view(np.float32)
    assert list(K.f32_to_f16_bits(nan)) == [0x7C00 | 0x0200 | (0x412345 >> 13), 0x8000 | 0x7C00 | 0x0200]
    every = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    back = K.f16_bits_to_f32(every)
    fin = np.isfinite(back)
    assert np.array_equal(K.f32_to_f16_bits(back[fin]), every[fin])


def scalar_quantize(blk, fmt):
    """One block, operation by operation in f32 (kvquant.rs:1053-1105 read as scalar code)."""
    def f16(x):
        try:
            return struct.unpack("<H", struct.pack("<e", x))[0]
        except OverflowError:
            return 0x7C00 | (0x8000 if x < 0 else 0)
    q = []
    if fmt == K.Q8_0:
        amax = 0.0
        for v in blk:
            amax = max(amax, abs(v))
        d = f32(amax / 127.0)
        inv = f32(1.0 / d) if d > 0 else 0.0
        for v in blk:
            t = f32(v * inv)
            r = math.copysign(math.floor(f32(abs(t) + 0.5)), t)
            q.append(int(min(max(r, -127.0), 127.0)))
        return q, [f16(d)]
    if fmt == K.Q4_0:
        amax, mx = 0.0, 0.0
        for v in blk:
            if amax < abs(v):
                amax, mx = abs(v), v
        d = f32(mx / -8.0)
        inv = f32(1.0 / d) if d != 0 else 0.0
        for v in blk:
            q.append(int(min(max(math.floor(f32(f32(v * inv) + 8.5)), 0.0), 15.0)))
        return q, [f16(d)]
    mn, mx = min(blk), max(blk)
    d = f32(f32(mx - mn) / 15.0)
    inv = f32(1.0 / d) if d != 0 else 0.0
    for v in blk:
        q.append(int(min(max(math.floor(f32(f32(f32(v - mn) * inv) + 0.5)), 0.0), 15.0)))
    return q, [f16(d), f16(mn)]


@pytest.mark.parametrize("fmt", FMTS)
def test_against_the_scalar_formulation(fmt):
    rng = np.random.default_rng(17 + fmt)
    rows, width = 6, 96
    x = (rng.standard_t(2, (rows, width)) * 10.0 ** rng.integers(-3, 3, (rows, 1))).astype(np.float32)      # heavy tails
    x[2, 32:64] = 0.0
    x[3, :32] = -x[3, :32].max()                  # a constant block: Q4_1's d = 0
    x[4, 5] = x[4, 9] = -np.abs(x[4, :32]).max() * 2      # two equal extremes: the first wins
    c = K.quantize(x, rows, width, fmt)
    for b in range(rows * 3):
        blk = [float(v) for v in x.reshape(-1, 32)[b]]
        q, sc = scalar_quantize(blk, fmt)
        assert list(K.codes_of(c, b)) == q, (fmt, b)
        assert list(np.atleast_1d(c.scales[b])) == sc, (fmt, b)
    y = c.dequantize_rows(0, rows).reshape(-1, 32)
    for b in range(rows * 3):
        q = K.codes_of(c, b)
        sc = K.f16_bits_to_f32(np.atleast_1d(c.scales[b]))
        for j in range(32):
            w = f32(q[j] * float(sc[0])) if fmt == K.Q8_0 else f32((q[j] - 8) * float(sc[0])) if fmt == K.Q4_0 else \
                f32(f32(q[j] * float(sc[0])) + float(sc[1]))
            assert y[b, j] == np.float32(w), (fmt, b, j)


@pytest.mark.parametrize("fmt", FMTS)
def test_error_bounds_and_append_in_place(fmt):
    rng = np.random.default_rng(23)
    rows, width = 40, 128
    x = rng.standard_normal((rows, width)).astype(np.float32) * 3
    c = K.quantize(x, rows, width, fmt)
    y = c.dequantize_rows(0, rows)
    blk, yb = x.reshape(-1, 32).astype(np.float64), y.reshape(-1, 32).astype(np.float64)
    if fmt == K.Q8_0:
        d = np.abs(blk).max(axis=1) / 127
        bound = d * (0.5 + 127 / 2048)            # half a step, plus the f16 rounding of d on the largest code
    elif fmt == K.Q4_0:
        d = np.abs(blk).max(axis=1) / 8
        bound = d * (1 + 8 / 2048)                # the end opposite the extreme is clamped at 7 steps: up to a whole step there
    else:
        d = (blk.max(axis=1) - blk.min(axis=1)) / 15
        bound = d * (0.5 + 15 / 2048) + np.abs(blk.min(axis=1)) / 2048
    assert (np.abs(blk - yb).max(axis=1) <= bound * (1 + 1e-6)).all()
    assert (np.abs(blk - yb).max(axis=1) >= bound * 0.2).any()          # and the bound is not vacuous
    # row by row into a larger cache = one shot (kvquant.rs:1908), rows outside the append untouched
    big = K.Cache(fmt, rows + 3, width)
    big.codes[:] = 0xDEADBEEF
    big.scales[:] = 0xABCD
    for r in range(rows):
        big.quantize_into(x[r], r + 1)
    nb = rows * 4
    assert np.array_equal(big.codes[4:4 + nb], c.codes) and np.array_equal(big.scales[4:4 + nb], c.scales)
    assert (big.codes[:4] == 0xDEADBEEF).all() and (big.codes[4 + nb:] == 0xDEADBEEF).all() and (big.scales[:4] == 0xABCD).all()
    assert np.array_equal(big.dequantize_rows(3, 5), y[2:7])
