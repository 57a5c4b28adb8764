"""Writes tests/golden/vectors.npz: small input/expected-output vectors for the quantized matmul path.

    python tests/golden/make_golden.py

The reference is Rust and cannot be built or run in this environment, so nothing here comes from
executing it. Each vector is either
  * a known answer the reference's own tests state in closed form (the Q4_K block of
    crates/ferric-gguf/examples/roundtrip.rs:54-87, the f16 landmarks of
    crates/ferric-tensor/src/cpu_simd.rs:203-213), rebuilt here from that closed form without any
    dequantizer, or
  * blocks from the reference's deterministic generators (crates/ferric-tensor/examples/q4_k.rs:13-37,
    q6_k.rs:9-17, cpu_simd.rs:136-156) re-derived in pure Python integers below, with the values the
    CPU oracle produces for them (those are regression vectors for the oracle and targets for the GPU).
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as O  # noqa: E402

M32 = 0xFFFFFFFF


def f16_bits(x):
    return int(np.array([x], dtype=np.float32).astype(np.float16).view(np.uint16)[0])


def py_q4k_block(seed):
    """q4_k.rs:13-37 in Python integers (u32 wrapping)."""
    b = bytearray(144)
    d = np.float32(0.05) + np.float32(0.01) * np.float32(seed % 7)
    dmin = np.float32(0.02) + np.float32(0.005) * np.float32(seed % 5)
    b[0:2] = f16_bits(d).to_bytes(2, "little")
    b[2:4] = f16_bits(dmin).to_bytes(2, "little")
    s = [0] * 12
    for j in range(8):
        sc = ((seed * 2654435761 & M32) + j * 40503 & M32) % 64
        mn = ((seed * 40503 & M32) + (j * 2654435761 & M32) & M32) % 64
        if j < 4:
            s[j] |= sc & 63
            s[j + 4] |= mn & 63
        else:
            s[j + 4] |= (sc & 0x0F) | ((mn & 0x0F) << 4)
            s[j - 4] |= (sc >> 4) << 6
            s[j] |= (mn >> 4) << 6
    b[4:16] = bytes(s)
    for i in range(128):
        b[16 + i] = ((seed + (i * 2246822519 & M32)) & M32) % 256
    return np.frombuffer(bytes(b), dtype=np.uint8)


def py_q6k_block(seed):
    """q6_k.rs:9-17 in Python integers."""
    b = bytearray(210)
    for i in range(128):
        b[i] = ((seed + (i * 2246822519 & M32)) & M32) % 256
    for i in range(64):
        b[128 + i] = ((seed * 40503 & M32) + i * 97 & M32) % 256
    for i in range(16):
        b[192 + i] = ((((seed + i * 7) & M32) % 64) - 32) & 0xFF
    b[208:210] = f16_bits(np.float32(0.04) + np.float32(0.01) * np.float32(seed % 6)).to_bytes(2, "little")
    return np.frombuffer(bytes(b), dtype=np.uint8)


def py_q8_synth(rows, cols, seed):
    """cpu_simd.rs:136-156 in Python integers: raw bytes and the exact values built beside them."""
    s = (seed * 2654435761 + 1) & M32
    raw = bytearray()
    vals = np.zeros(rows * cols, dtype=np.float32)
    for r in range(rows):
        for blk in range(cols // 32):
            s = (s * 1664525 + 1013904223) & M32
            dbits = 0x1C00 | ((s >> 16) & 0x3F)
            raw += dbits.to_bytes(2, "little")
            d = np.array([dbits], dtype=np.uint16).view(np.float16).astype(np.float32)[0]
            for j in range(32):
                s = (s * 1664525 + 1013904223) & M32
                c = (s >> 16) & 0xFF
                raw.append(c)
                vals[r * cols + blk * 32 + j] = np.float32(c - 256 if c >= 128 else c) * d
    return np.frombuffer(bytes(raw), dtype=np.uint8), vals


def roundtrip_q4k_known_answer():
    """roundtrip.rs:54-87: d = 1, dmin = 0, scales[0..8] = 1, scales[8..12] = 0,
    qs[i] = (i % 8) | (((i + 3) % 8) << 4); expected values from the test's own closed form."""
    blk = bytearray(144)
    blk[0:2] = f16_bits(1.0).to_bytes(2, "little")
    blk[2:4] = f16_bits(0.0).to_bytes(2, "little")
    scales = [1] * 8 + [0] * 4
    blk[4:16] = bytes(scales)
    qs = [((i % 256) % 8 & 0x0F) | ((((i % 256) + 3) % 8) << 4) for i in range(128)]
    blk[16:144] = bytes(qs)

    def get(j):
        return scales[j] & 63 if j < 4 else (scales[j + 4] & 0x0F) | ((scales[j - 4] >> 6) << 4)

    exp = np.zeros(256, dtype=np.float32)
    y = q = isb = 0
    for _ in range(4):
        s1, s2 = float(get(isb)), float(get(isb + 1))
        for l in range(32):
            exp[y + l] = s1 * float(qs[q + l] & 0x0F)
            exp[y + l + 32] = s2 * float(qs[q + l] >> 4)
        y += 64; q += 32; isb += 2
    return np.frombuffer(bytes(blk), dtype=np.uint8), exp


def main():
    out = {}
    out["f16_landmark_bits"] = np.array([0x0000, 0x3C00, 0xBC00, 0x0001, 0x7C00, 0xFC00, 0x8000, 0x03FF, 0x0400, 0x7BFF],
                                        dtype=np.uint16)
    out["f16_landmark_f32"] = np.array([0.0, 1.0, -1.0, 5.9604645e-8, np.inf, -np.inf, -0.0, 6.097555e-05, 6.1035156e-05,
                                        65504.0], dtype=np.float32)
    blk, exp = roundtrip_q4k_known_answer()
    out["q4k_known_block"], out["q4k_known_expected"] = blk, exp

    q4 = np.concatenate([py_q4k_block(s) for s in (1, 2, 3, 4)])
    q6 = np.concatenate([py_q6k_block(s) for s in (1, 2, 3, 4)])
    q8raw, q8vals = py_q8_synth(8, 64, 8 * 13 + 64)
    out["q4k_gen_blocks"], out["q4k_gen_deq"] = q4, O.deq_raw(q4, 1024, O.Q4_K)
    out["q6k_gen_blocks"], out["q6k_gen_deq"] = q6, O.deq_raw(q6, 1024, O.Q6_K)
    out["q8_synth_raw"], out["q8_synth_vals"] = q8raw, q8vals

    # one 8 x 256 GEMV per format, x = cos(0.013 i) as in the reference examples, f64 expected
    x = np.cos(np.arange(256, dtype=np.float32) * np.float32(0.013)).astype(np.float32)
    out["gemv_x"] = x
    w4 = np.concatenate([py_q4k_block(r + 1) for r in range(8)])
    w6 = np.concatenate([py_q6k_block(r + 1) for r in range(8)])
    w8, _ = py_q8_synth(8, 256, 7)
    for name, ty, w in (("q4k", O.Q4_K, w4), ("q6k", O.Q6_K, w6), ("q8_0", O.Q8_0, w8)):
        y64, wn = O.matmul_f64(x, w, ty, 8, 256)
        out[f"gemv_{name}_w"], out[f"gemv_{name}_y64"], out[f"gemv_{name}_wnorm"] = w, y64.reshape(-1), wn
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
