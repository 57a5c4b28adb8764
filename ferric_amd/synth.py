"""Seeded synthetic quantized weights with the field distributions the benchmark configs name.

Pure data generation (numpy); no arithmetic of the matmul path lives here.
"""
import numpy as np

Q8_0, Q4_K, Q6_K = 8, 12, 14
Q4_0, Q4_1, Q5_0, Q5_1, Q5_K = 2, 3, 6, 7, 13
IQ4_NL, IQ4_XS, MXFP4 = 20, 23, 39
BLOCK = {Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210), Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24),
         Q5_K: (256, 176), IQ4_NL: (32, 18), IQ4_XS: (256, 136), MXFP4: (32, 17)}


def q4k_pack_scales(sc, m):
    """Inverse of get_sc_min: sc, m [nb, 8] in 0..63 -> 12 packed bytes per block
    (the packing used by crates/ferric-tensor/examples/q4_k.rs:23-33)."""
    sc = sc.astype(np.uint8); m = m.astype(np.uint8)
    s = np.zeros((sc.shape[0], 12), np.uint8)
    s[:, 0:4] = (sc[:, 0:4] & 63) | ((sc[:, 4:8] >> 4) << 6)
    s[:, 4:8] = (m[:, 0:4] & 63) | ((m[:, 4:8] >> 4) << 6)
    s[:, 8:12] = (sc[:, 4:8] & 0x0F) | ((m[:, 4:8] & 0x0F) << 4)
    return s


def synth_weights(ty, rows, cols, seed):
    """Random blocks with the field distributions the benchmark configs name: fp16 scales
    |N(0,1)|*{0.02 Q8_0, 0.01 K-quants}, int8 uniform [-127,127], 6-bit scales/mins uniform 0..63,
    nibbles/bytes uniform, Q6_K sub-scales uniform [-32,31]."""
    rng = np.random.default_rng(seed)
    vals, bytes_ = BLOCK[ty]
    nb = rows * cols // vals
    b = np.zeros((nb, bytes_), np.uint8)
    if ty == Q8_0:
        b[:, 0:2] = (np.abs(rng.standard_normal(nb)) * 0.02).astype(np.float16).view(np.uint8).reshape(nb, 2)
        b[:, 2:] = rng.integers(-127, 128, (nb, 32), dtype=np.int8).view(np.uint8)
    elif ty == Q4_K:
        b[:, 0:2] = (np.abs(rng.standard_normal(nb)) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 2)
        b[:, 2:4] = (np.abs(rng.standard_normal(nb)) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 2)
        b[:, 4:16] = q4k_pack_scales(rng.integers(0, 64, (nb, 8), dtype=np.uint8), rng.integers(0, 64, (nb, 8), dtype=np.uint8))
        b[:, 16:] = rng.integers(0, 256, (nb, 128), dtype=np.uint8)
    elif ty in (Q4_0, Q4_1, Q5_0, Q5_1):
        # f16 scale (and a signed f16 offset for the affine formats), every other byte uniform
        f16 = lambda v: v.astype(np.float16).view(np.uint8).reshape(nb, 2)
        b[:, 2:] = rng.integers(0, 256, (nb, bytes_ - 2), dtype=np.uint8)
        b[:, 0:2] = f16(np.abs(rng.standard_normal(nb)) * 0.02)
        if ty in (Q4_1, Q5_1):
            b[:, 2:4] = f16(rng.standard_normal(nb) * 0.1)
    elif ty == Q5_K:
        b[:, 0:2] = (np.abs(rng.standard_normal(nb)) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 2)
        b[:, 2:4] = (np.abs(rng.standard_normal(nb)) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 2)
        b[:, 4:16] = q4k_pack_scales(rng.integers(0, 64, (nb, 8), dtype=np.uint8), rng.integers(0, 64, (nb, 8), dtype=np.uint8))
        b[:, 16:] = rng.integers(0, 256, (nb, 160), dtype=np.uint8)
    elif ty in (IQ4_NL, IQ4_XS):
        # f16 super-scale; the 6-bit sub-scales of IQ4_XS (offset by 32 when used) and all codebook indices uniform
        b[:, 2:] = rng.integers(0, 256, (nb, bytes_ - 2), dtype=np.uint8)
        b[:, 0:2] = (np.abs(rng.standard_normal(nb)) * (0.0005 if ty == IQ4_XS else 0.002)).astype(np.float16).view(np.uint8).reshape(nb, 2)
    elif ty == MXFP4:
        # shared exponents around 2^-9 .. 2^-6 (the range a released checkpoint's blocks use), codes uniform
        b[:, 0] = rng.integers(0x75, 0x7A, nb, dtype=np.uint8)
        b[:, 1:] = rng.integers(0, 256, (nb, 16), dtype=np.uint8)
    else:
        assert ty == Q6_K, f"no generator for ggml type {ty}"
        b[:, 0:192] = rng.integers(0, 256, (nb, 192), dtype=np.uint8)
        b[:, 192:208] = rng.integers(-32, 32, (nb, 16), dtype=np.int8).view(np.uint8)
        b[:, 208:210] = (np.abs(rng.standard_normal(nb)) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 2)
    return b.reshape(-1)
