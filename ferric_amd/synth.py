"""Seeded synthetic quantized weights with the field distributions the benchmark configs name.

Pure data generation (numpy); no arithmetic of the matmul path lives here.
"""
import numpy as np

Q8_0, Q4_K, Q6_K = 8, 12, 14
BLOCK = {Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210)}


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
    else:
        b[:, 0:192] = rng.integers(0, 256, (nb, 192), dtype=np.uint8)
        b[:, 192:208] = rng.integers(-32, 32, (nb, 16), dtype=np.int8).view(np.uint8)
        b[:, 208:210] = (np.abs(rng.standard_normal(nb)) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 2)
    return b.reshape(-1)
