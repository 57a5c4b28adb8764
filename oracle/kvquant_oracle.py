"""CPU restatement (numpy, every operation a single IEEE f32 operation as in the reference) of the block-quantized KV cache.

TEST INFRASTRUCTURE ONLY: imported by tests/ and the smoke check, never by the shipped package.

Follows crates/ferric-tensor/src/kvquant.rs `mod reference` (:943-1186), which the reference declares the bit-for-bit twin of
its kernels: blocks of QK = 32 consecutive values of a row, block b = row * (width / 32) + col / 32;
  Q8_0  d = amax / 127, q = roundf(v * (1 / d)) clamped to +-127, eight code words of four int8 (:1053-1066);
  Q4_0  d = (the value of largest magnitude, first one wins) / -8, q = floor(v * (1 / d) + 8.5) clamped to 0..15, byte i of a
        block = q[i] | q[i + 16] << 4 (:1067-1088);
  Q4_1  d = (max - min) / 15, q = floor((v - min) * (1 / d) + 0.5) clamped to 0..15, same packing, scale word = f16(d) |
        f16(min) << 16 (:1089-1105).
Q8_0 / Q4_0 scales are f16 bit patterns, two per u32 word, block b in half b % 2 of word b / 2 (:1110-1118). Here the scale
array is addressed as uint16 [block] (Q4_1: [block][2] = d, min), which is the same bytes on a little-endian machine.
Pinned in tests/test_oracle_kvquant.py.
"""
import numpy as np

QK = 32
Q8_0, Q4_0, Q4_1 = 0, 1, 2
CODE_WORDS = {Q8_0: 8, Q4_0: 4, Q4_1: 4}          # kvquant.rs:68-73
BLOCK_BYTES = {Q8_0: 34, Q4_0: 18, Q4_1: 20}      # kvquant.rs:83-89
F32 = np.float32


def scale_words(fmt, nblk):
    """kvquant.rs:76-81."""
    return nblk if fmt == Q4_1 else (nblk + 1) // 2


def sizes(rows, width, fmt):
    """kvquant.rs:1027-1030: (code words, scale words) for rows x width."""
    nblk = rows * (width // QK)
    return nblk * CODE_WORDS[fmt], scale_words(fmt, nblk)


def f32_to_f16_bits(x):
    """kvquant.rs:956-995: round to nearest even; overflow to infinity; a NaN stays a quiet NaN with its top payload bits."""
    x = np.asarray(x, F32)
    b = x.view(np.uint32)
    with np.errstate(over="ignore", invalid="ignore"):
        h = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    nan_bits = (((b >> 16) & 0x8000) | 0x7C00 | 0x0200 | ((b & 0x007FFFFF) >> 13)).astype(np.uint16)
    return np.where(nan, nan_bits, h).astype(np.uint16)


def f16_bits_to_f32(h):
    """kvquant.rs:998-1018."""
    return np.asarray(h, np.uint16).view(np.float16).astype(F32)


def _to_u32(v):
    """Rust `f32 as u32` / `as i32` after a clamp: NaN becomes 0."""
    return np.where(np.isnan(v), 0, v).astype(np.int64)


def _recip(d, nonzero_only):
    """`if d > 0 { 1 / d } else { 0 }` (Q8_0) or `if d != 0` (Q4_0, Q4_1), in f32."""
    ok = (d != 0) if nonzero_only else (d > 0)
    with np.errstate(divide="ignore", invalid="ignore"):
        return np.where(ok, F32(1.0) / np.where(ok, d, F32(1.0)), F32(0.0)).astype(F32)


def quantize_blocks(blk, fmt):
    """blk [n, 32] f32 -> (codes uint32 [n, CODE_WORDS], scale halves uint16 [n] or [n, 2])."""
    blk = np.ascontiguousarray(blk, F32)
    n = blk.shape[0]
    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        if fmt == Q8_0:
            amax = np.fmax.reduce(np.abs(blk), axis=1, initial=F32(0.0)).astype(F32)     # f32::max drops NaNs
            d = (amax / F32(127.0)).astype(F32)
            inv = _recip(d, False)
            t = (blk * inv[:, None]).astype(F32)
            r = np.copysign(np.floor((np.abs(t) + F32(0.5)).astype(F32)), t)            # signum(x) * floor(|x| + 0.5)
            q = _to_u32(np.clip(r, F32(-127.0), F32(127.0))) & 255
            codes = (q.reshape(n, 8, 4) << (8 * np.arange(4))).sum(axis=2).astype(np.uint32)
            return codes, f32_to_f16_bits(d)
        if fmt == Q4_0:
            a = np.abs(blk)
            key = np.where(np.isnan(a), F32(-1.0), a)                                    # `amax < |v|` is false for a NaN
            first = key.argmax(axis=1)                                                   # the first of equal magnitudes wins
            amax = key[np.arange(n), first]
            mx = np.where(amax > 0, blk[np.arange(n), first], F32(0.0)).astype(F32)      # nothing above 0: max stays +0.0
            d = (mx / F32(-8.0)).astype(F32)
            inv = _recip(d, True)
            t = np.floor(((blk * inv[:, None]).astype(F32) + F32(8.5)).astype(F32))
            q = _to_u32(np.clip(t, F32(0.0), F32(15.0)))
            scales = f32_to_f16_bits(d)
        else:
            mn = np.fmin.reduce(blk, axis=1, initial=F32(np.inf)).astype(F32)
            mx = np.fmax.reduce(blk, axis=1, initial=F32(-np.inf)).astype(F32)
            d = ((mx - mn).astype(F32) / F32(15.0)).astype(F32)
            inv = _recip(d, True)
            t = np.floor((((blk - mn[:, None]).astype(F32) * inv[:, None]).astype(F32) + F32(0.5)).astype(F32))
            q = _to_u32(np.clip(t, F32(0.0), F32(15.0)))
            scales = np.stack([f32_to_f16_bits(d), f32_to_f16_bits(mn)], axis=1)
        byte = q[:, :16] | (q[:, 16:] << 4)
        codes = (byte.reshape(n, 4, 4) << (8 * np.arange(4))).sum(axis=2).astype(np.uint32)
        return codes, scales


class Cache:
    """The packed arrays of a cache of `cap` rows: codes uint32 [cap * nblk, CODE_WORDS], scales uint16 [cap * nblk (, 2)]."""

    def __init__(self, fmt, cap, width):
        assert width % QK == 0, f"width {width} must be a multiple of {QK}"
        self.fmt, self.cap, self.width, self.nblk = fmt, cap, width, width // QK
        self.codes = np.zeros((cap * self.nblk, CODE_WORDS[fmt]), np.uint32)
        self.scales = np.zeros((cap * self.nblk, 2) if fmt == Q4_1 else (cap * self.nblk,), np.uint16)

    def quantize_into(self, x, row0):
        """kvquant.rs:1036-1108: rows of x [rows, width] into cache rows row0 .. row0 + rows; nothing else is touched."""
        x = np.asarray(x, F32).reshape(-1, self.width)
        c, s = quantize_blocks(x.reshape(-1, QK), self.fmt)
        b0 = row0 * self.nblk
        self.codes[b0:b0 + c.shape[0]] = c
        self.scales[b0:b0 + c.shape[0]] = s
        return self

    def dequantize_rows(self, row0, rows):
        """kvquant.rs:1130-1176."""
        b0, nb = row0 * self.nblk, rows * self.nblk
        return dequantize_blocks(self.codes[b0:b0 + nb], self.scales[b0:b0 + nb], self.fmt).reshape(rows, self.width)


def dequantize_blocks(codes, scales, fmt):
    """codes [n, CODE_WORDS], scales [n] or [n, 2] -> [n, 32] f32: q * d, (q - 8) * d, q * d + m (two roundings)."""
    n = codes.shape[0]
    by = ((codes[:, :, None] >> (8 * np.arange(4, dtype=np.uint32))) & 255).reshape(n, -1)
    if fmt == Q8_0:
        return (by.astype(np.uint8).view(np.int8).astype(F32) * f16_bits_to_f32(scales)[:, None]).astype(F32)
    nib = np.concatenate([by & 15, by >> 4], axis=1).astype(F32)
    if fmt == Q4_0:
        return ((nib - F32(8.0)).astype(F32) * f16_bits_to_f32(scales)[:, None]).astype(F32)
    d, m = f16_bits_to_f32(scales[:, 0]), f16_bits_to_f32(scales[:, 1])
    return ((nib * d[:, None]).astype(F32) + m[:, None]).astype(F32)


def quantize(x, rows, width, fmt):
    """kvquant.rs:1121-1127: a standalone slab."""
    return Cache(fmt, rows, width).quantize_into(np.asarray(x, F32).reshape(rows, width), 0)


def roundtrip(x, rows, width, fmt):
    """kvquant.rs:1182-1185: what a runtime attends over."""
    return quantize(x, rows, width, fmt).dequantize_rows(0, rows)


def codes_of(cache, b):
    """The 32 codes of block b as integers (signed for Q8_0) -- the reading of kvquant.rs:1505-1522."""
    by = ((cache.codes[b][:, None] >> (8 * np.arange(4, dtype=np.uint32))) & 255).reshape(-1)
    if cache.fmt == Q8_0:
        return by.astype(np.uint8).view(np.int8).astype(np.int64)
    return np.concatenate([by & 15, by >> 4]).astype(np.int64)
