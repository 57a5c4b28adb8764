"""ctypes front end of the CPU oracle (oracle/ferric_oracle.c) plus an independent numpy twin.

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the CPU-baseline leg of
the benchmark. The shipped package never imports it.

The C functions restate the reference's Rust (citations are in the C file). The ``np_*``
functions below are a second, vectorised restatement written from the block layouts, using
numpy's own float16 conversion; tests demand bit-equality between the two.
"""
import ctypes as C
import os
import subprocess

import numpy as np

Q8_0, Q4_K, Q6_K = 8, 12, 14
Q4_0, Q4_1, Q5_0, Q5_1, Q5_K = 2, 3, 6, 7, 13
IQ4_NL, IQ4_XS, MXFP4 = 20, 23, 39
BLOCK = {Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210), Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24),
         Q5_K: (256, 176), IQ4_NL: (32, 18), IQ4_XS: (256, 136), MXFP4: (32, 17)}

F32, F16, BF16 = 0, 1, 30
DENSE = {F32: 4, F16: 2, BF16: 2}          # unquantized tensor types: bytes per element

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libferric_oracle.so")


def build(force=False):
    """Compile the oracle with the committed Makefile (gcc, -ffp-contract=off)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []), stdout=subprocess.DEVNULL)
    return _SO


_lib = None
_u8p = C.POINTER(C.c_uint8)
_f32p = C.POINTER(C.c_float)
_f64p = C.POINTER(C.c_double)


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_SO)
        L.fo_f16_to_f32.restype = C.c_float
        L.fo_f16_to_f32.argtypes = [C.c_uint16]
        L.fo_f16_table_bits.restype = None
        L.fo_f16_table_bits.argtypes = [C.POINTER(C.c_uint32)]
        L.fo_f32_to_f16.restype = C.c_uint16
        L.fo_f32_to_f16.argtypes = [C.c_float]
        L.fo_type_size.restype = C.c_size_t
        L.fo_type_size.argtypes = [C.c_uint32, C.c_size_t]
        L.fo_deq_raw.restype = C.c_size_t
        L.fo_deq_raw.argtypes = [_u8p, C.c_size_t, C.c_size_t, C.c_uint32, _f32p]
        L.fo_deq_elemwise.restype = None
        L.fo_deq_elemwise.argtypes = [_u8p, C.c_size_t, C.c_uint32, _f32p]
        L.fo_q4k_get_sc_min.restype = None
        L.fo_q4k_get_sc_min.argtypes = [_u8p, C.c_int, _u8p, _u8p]
        L.fo_matvec_q8_0.restype = C.c_int
        L.fo_matvec_q8_0.argtypes = [_f32p, _u8p, C.c_size_t, C.c_size_t, C.c_size_t, _f32p]
        L.fo_matvec_q8_0_threaded.restype = C.c_int
        L.fo_matvec_q8_0_threaded.argtypes = [_f32p, _u8p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, _f32p]
        L.fo_matvec_q8_0_span.restype = C.c_int
        L.fo_matvec_q8_0_span.argtypes = [_f32p, _u8p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, _f32p]
        L.fo_matmul_threaded.restype = C.c_int
        L.fo_matmul_threaded.argtypes = [_f32p, C.c_size_t, _u8p, C.c_size_t, C.c_uint32, C.c_size_t, C.c_size_t,
                                         C.c_int, C.c_size_t, _f32p]
        L.fo_matmul_f64.restype = C.c_int
        L.fo_matmul_f64.argtypes = [_f32p, C.c_size_t, _u8p, C.c_size_t, C.c_uint32, C.c_size_t, C.c_size_t, _f64p, _f64p]
        L.fo_swiglu.restype = None
        L.fo_swiglu.argtypes = [_f32p, C.c_size_t, C.c_size_t, _f32p]
        L.fo_gen_q4k_block.restype = None
        L.fo_gen_q4k_block.argtypes = [C.c_uint32, _u8p]
        L.fo_gen_q6k_block.restype = None
        L.fo_gen_q6k_block.argtypes = [C.c_uint32, _u8p]
        L.fo_gen_kquant_matrix.restype = None
        L.fo_gen_kquant_matrix.argtypes = [C.c_uint32, C.c_size_t, C.c_size_t, _u8p]
        L.fo_quant_q8_0.restype = None
        L.fo_quant_q8_0.argtypes = [_f32p, C.c_size_t, _u8p]
        L.fo_gen_q8_0_synth.restype = None
        L.fo_gen_q8_0_synth.argtypes = [C.c_size_t, C.c_size_t, C.c_uint32, _u8p, _f32p]
        _lib = L
    return _lib


def _u8(a):
    a = np.ascontiguousarray(a, dtype=np.uint8)
    return a, a.ctypes.data_as(_u8p)


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_f32p)


# ---------------------------------------------------------------- C oracle wrappers

def f16_to_f32(bits):
    return float(lib().fo_f16_to_f32(int(bits)))


def f16_table():
    """All 65536 binary16 patterns decoded by the C oracle, as f32 (bit-exact, NaN payloads kept)."""
    out = np.zeros(65536, dtype=np.uint32)
    lib().fo_f16_table_bits(out.ctypes.data_as(C.POINTER(C.c_uint32)))
    return out.view(np.float32)


def f32_to_f16_bits(x):
    return int(lib().fo_f32_to_f16(float(np.float32(x))))


def type_size(ty, n):
    """Bytes of n elements of ggml type ty; raises ValueError('unsupported ggml type N') like the
    reference's Err(String)."""
    if ty not in BLOCK and ty not in DENSE:
        raise ValueError(f"unsupported ggml type {ty}")
    return int(lib().fo_type_size(ty, n))


def deq_raw(raw, n, ty):
    """Reference-order dequantization of n elements (Q8_0 returns a shorter array on a ragged tail; the unquantized
    types slice the bytes first and so panic -- AssertionError here -- when there are fewer than n elements)."""
    if ty not in BLOCK and ty not in DENSE:
        raise ValueError(f"unsupported ggml type {ty}")
    raw, rp = _u8(raw)
    out = np.zeros(n, dtype=np.float32)
    got = lib().fo_deq_raw(rp, raw.size, n, ty, out.ctypes.data_as(_f32p))
    if got == C.c_size_t(-2).value:
        raise AssertionError(f"range end index {n * DENSE[ty]} out of range for slice of length {raw.size}")
    return out[:got]


def deq_elemwise(raw, n, ty):
    """Second formulation (per-element random access)."""
    raw, rp = _u8(raw)
    out = np.zeros(n, dtype=np.float32)
    lib().fo_deq_elemwise(rp, n, ty, out.ctypes.data_as(_f32p))
    return out


def q4k_get_sc_min(scales12, j):
    s, sp = _u8(scales12)
    sc, m = C.c_uint8(), C.c_uint8()
    lib().fo_q4k_get_sc_min(sp, j, C.byref(sc), C.byref(m))
    return sc.value, m.value


def matvec_q8_0(x, w, rows, cols):
    x, xp = _f32(x); w, wp = _u8(w)
    y = np.zeros(rows, dtype=np.float32)
    if not lib().fo_matvec_q8_0(xp, wp, w.size, rows, cols, y.ctypes.data_as(_f32p)):
        raise AssertionError("matvec_q8_0: shape assertion failed")
    return y


def matvec_q8_0_threaded(x, w, rows, cols, threads):
    x, xp = _f32(x); w, wp = _u8(w)
    y = np.zeros(rows, dtype=np.float32)
    if not lib().fo_matvec_q8_0_threaded(xp, wp, w.size, rows, cols, threads, y.ctypes.data_as(_f32p)):
        raise AssertionError("matvec_q8_0_threaded: shape assertion failed")
    return y


def matvec_q8_0_span(x, w, cols, lo, hi, threads):
    x, xp = _f32(x); w, wp = _u8(w)
    y = np.zeros(hi - lo, dtype=np.float32)
    if not lib().fo_matvec_q8_0_span(xp, wp, cols, lo, hi, threads, y.ctypes.data_as(_f32p)):
        raise AssertionError("matvec_q8_0_span: empty or inverted span")
    return y


def matmul_cpu(x, w, ty, rows, cols, threads=1, direct_q8=False):
    """y[xrows, rows] = x[xrows, cols] * W^T in f32, the reference CPU way: Q8_0 direct mat-vec
    (direct_q8) or dequantize-then-sequential-dot, rows split in contiguous spans over threads."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, cols)
    w, wp = _u8(w)
    y = np.zeros((x.shape[0], rows), dtype=np.float32)
    ok = lib().fo_matmul_threaded(x.ctypes.data_as(_f32p), x.shape[0], wp, w.size, ty, rows, cols,
                                  1 if direct_q8 else 0, threads, y.ctypes.data_as(_f32p))
    if not ok:
        raise AssertionError("matmul_cpu: shape assertion failed")
    return y


def matmul_f64(x, w, ty, rows, cols):
    """(y64[xrows, rows], wnorm[rows]): f64-accumulated products and per-row weight norms for the
    tolerance bound |dy| <= 1e-3 * ||w_row|| * ||x||."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, cols)
    w, wp = _u8(w)
    y = np.zeros((x.shape[0], rows), dtype=np.float64)
    wn = np.zeros(rows, dtype=np.float64)
    ok = lib().fo_matmul_f64(x.ctypes.data_as(_f32p), x.shape[0], wp, w.size, ty, rows, cols,
                             y.ctypes.data_as(_f64p), wn.ctypes.data_as(_f64p))
    if not ok:
        raise AssertionError("matmul_f64: shape assertion failed")
    return y, wn


def swiglu(gu, n_ff):
    gu = np.ascontiguousarray(gu, dtype=np.float32).reshape(-1, 2 * n_ff)
    out = np.zeros((gu.shape[0], n_ff), dtype=np.float32)
    lib().fo_swiglu(gu.ctypes.data_as(_f32p), gu.shape[0], n_ff, out.ctypes.data_as(_f32p))
    return out


# ---------------------------------------------------------------- mixture-of-experts ops (numpy restatements)
def moe_topk(logits, bias, k, sigmoid, scale, norm=True):
    """MOE_TOPK_WGSL, crates/ferric-tensor/src/dtype.rs:2415-2461, statement by statement in f32: per token the
    scores (softmax with a sequential f32 sum, or sigmoid), k rounds of a first-maximum scan over the not yet
    picked experts on score + bias, weights = picked scores / (their sequential sum if norm) * scale.
    Returns [T, 2k] f32 = [w | idx]."""
    f = np.float32
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    logits = logits.reshape(1, -1) if logits.ndim == 1 else logits
    t, ne = logits.shape
    assert 1 <= k <= 8, "k must be 1..=8"
    assert ne <= 1024, "moe_topk: n_expert <= 1024 (single-thread scan)"
    out = np.zeros((t, 2 * k), dtype=np.float32)
    for ti in range(t):
        l = logits[ti]
        maxl, ssum = f(-3.4e38), f(0.0)
        if not sigmoid:
            for i in range(ne):
                maxl = max(maxl, l[i])
            for i in range(ne):
                ssum = f(ssum + np.exp(f(l[i] - maxl), dtype=np.float32))

        def score(i):
            if sigmoid:
                return f(f(1.0) / f(f(1.0) + np.exp(f(-l[i]), dtype=np.float32)))
            return f(np.exp(f(l[i] - maxl), dtype=np.float32) / ssum)

        picked, wsum = set(), f(0.0)
        with np.errstate(all="ignore"):
            for s in range(k):
                bi, bv = 0, f(-3.4e38)
                for i in range(ne):
                    if i in picked:
                        continue
                    m = score(i)
                    if bias is not None:
                        m = f(m + f(bias[i]))
                    if m > bv:
                        bv, bi = m, i
                picked.add(bi)
                sc = score(bi)
                out[ti, s], out[ti, k + s] = sc, f(bi)
                wsum = f(wsum + sc)
            den = wsum if norm else f(1.0)
            for s in range(k):
                out[ti, s] = f(f(out[ti, s] / den) * f(scale))
    return out


def matmul_swiglu_id_f64(x, w, ty, selw, k, eff, cols):
    """MATMUL_Q4_K_SWIGLU_ID_WGSL / MATMUL_Q8_0_SWIGLU_ID_WGSL (dtype.rs:2463-2507, :2618-2652) in f64 on the
    dequantized expert slab: out[ti, s, o] = silu(g) * u with g, u the dots of token ti's row with rows
    e*2eff + o and e*2eff + eff + o, e = selw[ti, k + s]. Also returns (|g| bound terms) the per-row weight norms."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, cols)
    w, _ = _u8(w)
    rows = w.size // (cols // BLOCK[ty][0] * BLOCK[ty][1])
    wd = deq_raw(w, rows * cols, ty).reshape(rows, cols).astype(np.float64)
    selw = np.asarray(selw, dtype=np.float32).reshape(x.shape[0], 2 * k)
    out = np.zeros((x.shape[0], k, eff))
    for ti in range(x.shape[0]):
        for s in range(k):
            base = int(selw[ti, k + s]) * 2 * eff
            g = wd[base:base + eff] @ x[ti].astype(np.float64)
            u = wd[base + eff:base + 2 * eff] @ x[ti].astype(np.float64)
            out[ti, s] = g / (1.0 + np.exp(-g)) * u
    return out


def matmul_relu2_id_f64(x, w, ty, selw, k, eff, cols):
    """MATMUL_Q5_0_RELU2_ID_WGSL (crates/ferric-tensor/src/dtype.rs:3714-3758) in f64 on the dequantized expert slab
    [n_expert * eff, cols]: out[ti, s, o] = max(acc, 0)^2 with acc the dot of token ti's row with row e * eff + o,
    e = selw[ti, k + s] (the index half of the moe_topk row). Also returns the rows' norms for the tolerance bound."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, cols)
    w, _ = _u8(w)
    rows = w.size // (cols // BLOCK[ty][0] * BLOCK[ty][1])
    wd = deq_raw(w, rows * cols, ty).reshape(rows, cols).astype(np.float64)
    selw = np.asarray(selw, dtype=np.float32).reshape(x.shape[0], 2 * k)
    out = np.zeros((x.shape[0], k, eff))
    acc = np.zeros((x.shape[0], k, eff))
    wn = np.zeros((x.shape[0], k, eff))
    for ti in range(x.shape[0]):
        for s in range(k):
            blk = wd[int(selw[ti, k + s]) * eff:][:eff]
            acc[ti, s] = blk @ x[ti].astype(np.float64)
            wn[ti, s] = np.linalg.norm(blk, axis=1)
            a = np.maximum(acc[ti, s], 0.0)
            out[ti, s] = a * a
    return out, acc, wn


def matmul_id_f64(x, w, ty, selw, k, out_pe, cols):
    """MATMUL_Q6_K_ID_WGSL (dtype.rs:2509-2536) in f64: out[s, o] = x[s] . W[e_s*out_pe + o], plus the weight norms."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(k, cols)
    w, _ = _u8(w)
    rows = w.size // (cols // BLOCK[ty][0] * BLOCK[ty][1])
    wd = deq_raw(w, rows * cols, ty).reshape(rows, cols).astype(np.float64)
    selw = np.asarray(selw, dtype=np.float32).reshape(-1)
    out = np.zeros((k, out_pe))
    wn = np.zeros((k, out_pe))
    for s in range(k):
        blk = wd[int(selw[k + s]) * out_pe:][:out_pe]
        out[s] = blk @ x[s].astype(np.float64)
        wn[s] = np.linalg.norm(blk, axis=1)
    return out, wn


def matmul_id_wsum_f64(x, w, ty, selw, k, out_pe, cols):
    """MATMUL_{Q6_K,Q4_K,Q8_0}_ID_WSUM_WGSL (dtype.rs:2538-2700) in f64: out[ti, o] = sum_s w[ti, s] * x[ti, s] .
    W[e*out_pe + o]; also returns sum_s |w| * ||W row|| * ||x[ti, s]||, the scale of the tolerance bound."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, k, cols)
    w, _ = _u8(w)
    rows = w.size // (cols // BLOCK[ty][0] * BLOCK[ty][1])
    wd = deq_raw(w, rows * cols, ty).reshape(rows, cols).astype(np.float64)
    selw = np.asarray(selw, dtype=np.float32).reshape(x.shape[0], 2 * k)
    out = np.zeros((x.shape[0], out_pe))
    bound = np.zeros((x.shape[0], out_pe))
    for ti in range(x.shape[0]):
        for s in range(k):
            blk = wd[int(selw[ti, k + s]) * out_pe:][:out_pe]
            xv = x[ti, s].astype(np.float64)
            out[ti] += float(selw[ti, s]) * (blk @ xv)
            bound[ti] += abs(float(selw[ti, s])) * np.linalg.norm(blk, axis=1) * np.linalg.norm(xv)
    return out, bound


# ---------------------------------------------------------------- reference test-data generators

def gen_q4k_block(seed):
    b = np.zeros(144, dtype=np.uint8)
    lib().fo_gen_q4k_block(seed & 0xFFFFFFFF, b.ctypes.data_as(_u8p))
    return b


def gen_q6k_block(seed):
    b = np.zeros(210, dtype=np.uint8)
    lib().fo_gen_q6k_block(seed & 0xFFFFFFFF, b.ctypes.data_as(_u8p))
    return b


def gen_kquant_matrix(ty, rows, cols):
    """Weight as the reference examples build it: block (r, b) uses seed r*nblk + b + 1."""
    out = np.zeros(rows * (cols // 256) * BLOCK[ty][1], dtype=np.uint8)
    lib().fo_gen_kquant_matrix(ty, rows, cols, out.ctypes.data_as(_u8p))
    return out


def quant_q8_0(x):
    x, xp = _f32(x)
    assert x.size % 32 == 0
    out = np.zeros(x.size // 32 * 34, dtype=np.uint8)
    lib().fo_quant_q8_0(xp, x.size, out.ctypes.data_as(_u8p))
    return out


def gen_q8_0_synth(rows, cols, seed):
    raw = np.zeros(rows * cols // 32 * 34, dtype=np.uint8)
    vals = np.zeros(rows * cols, dtype=np.float32)
    lib().fo_gen_q8_0_synth(rows, cols, seed & 0xFFFFFFFF, raw.ctypes.data_as(_u8p), vals.ctypes.data_as(_f32p))
    return raw, vals


# ---------------------------------------------------------------- numpy twin (independent restatement)
# Written from the byte layouts; f16 decoding is numpy's. float32 numpy arithmetic is one rounding
# per ufunc and never fused, like the reference.

def _np_f16(two_bytes):
    return np.ascontiguousarray(two_bytes).view("<f2").astype(np.float32)


def np_deq_q8_0(raw, n):
    nb = min(n // 32, len(raw) // 34)
    b = np.asarray(raw[: nb * 34], dtype=np.uint8).reshape(nb, 34)
    d = _np_f16(b[:, 0:2]).reshape(nb, 1)
    q = b[:, 2:].view(np.int8).astype(np.float32)
    return (q * d).reshape(-1)


def np_q4k_scales(scales):
    """scales: [nb, 12] uint8 -> (sc[nb, 8], m[nb, 8]) uint8, ggml get_scale_min_k4."""
    s = scales.astype(np.uint8)
    sc = np.empty((s.shape[0], 8), np.uint8); m = np.empty_like(sc)
    sc[:, :4] = s[:, 0:4] & 63
    m[:, :4] = s[:, 4:8] & 63
    sc[:, 4:] = (s[:, 8:12] & 0x0F) | ((s[:, 0:4] >> 6) << 4)
    m[:, 4:] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    return sc, m


def np_deq_q4_k(raw, n):
    out = np.zeros(n, np.float32)
    nb = min(n // 256, len(raw) // 144)
    b = np.asarray(raw[: nb * 144], dtype=np.uint8).reshape(nb, 144)
    d = _np_f16(b[:, 0:2]).reshape(nb, 1); dmin = _np_f16(b[:, 2:4]).reshape(nb, 1)
    sc, m = np_q4k_scales(b[:, 4:16])
    qs = b[:, 16:].reshape(nb, 4, 32)
    nib = np.stack([qs & 0x0F, qs >> 4], axis=2).reshape(nb, 8, 32).astype(np.float32)  # sub-block 2g, 2g+1
    d1 = (d * sc.astype(np.float32)).reshape(nb, 8, 1)
    mm = (dmin * m.astype(np.float32)).reshape(nb, 8, 1)
    out[: nb * 256] = (d1 * nib - mm).reshape(-1)
    return out


def np_deq_q6_k(raw, n):
    out = np.zeros(n, np.float32)
    nb = min(n // 256, len(raw) // 210)
    b = np.asarray(raw[: nb * 210], dtype=np.uint8).reshape(nb, 210)
    ql = b[:, 0:128].reshape(nb, 2, 2, 32)     # [half][lo32/hi32][l]
    qh = b[:, 128:192].reshape(nb, 2, 32)      # [half][l]
    sc = b[:, 192:208].view(np.int8).reshape(nb, 2, 8).astype(np.float32)
    d = _np_f16(b[:, 208:210]).reshape(nb, 1, 1)
    q = np.empty((nb, 2, 4, 32), np.int32)     # [half][group g][l] -> element 128*half + 32*g + l
    for g in range(4):
        lo = ql[:, :, g & 1, :]
        nibble = (lo >> 4) if g >= 2 else (lo & 0x0F)
        q[:, :, g, :] = (nibble | (((qh >> (2 * g)) & 3) << 4)).astype(np.int32) - 32
    # scale index within the half: is + 2g with is = l // 16
    sidx = (np.arange(32) // 16)[None, :] + 2 * np.arange(4)[:, None]          # [g][l]
    scl = sc[:, :, sidx]                                                        # [nb][half][g][l]
    dsc = (d.reshape(nb, 1, 1, 1) * scl).astype(np.float32)
    out[: nb * 256] = (dsc * q.astype(np.float32)).reshape(-1)
    return out


def _np_legacy(raw, n, bytes_, has_m, has_qh, off):
    """The four 32-value formats from their layout: [f16 d][f16 m]?[u32 qh]?[16 bytes of nibbles]; value i takes the
    low nibble of byte i, value 16+i the high one; the fifth bit of value v is bit v of qh."""
    out = np.zeros(n, np.float32)
    nb = min(n // 32, len(raw) // bytes_)
    b = np.asarray(raw[: nb * bytes_], dtype=np.uint8).reshape(nb, bytes_)
    d = _np_f16(b[:, 0:2]).reshape(nb, 1)
    p = 2
    m = None
    if has_m:
        m = _np_f16(b[:, 2:4]).reshape(nb, 1)
        p = 4
    q = np.concatenate([b[:, p + 4 * has_qh:] & 0x0F, b[:, p + 4 * has_qh:] >> 4], axis=1).astype(np.int32)   # [nb, 32]
    if has_qh:
        qh = b[:, p:p + 4].copy().view("<u4").reshape(nb, 1)
        q = q | (((qh >> np.arange(32, dtype=np.uint32)) & 1).astype(np.int32) << 4)
    v = (q - off).astype(np.float32) * d
    if has_m:
        v = v + m
    out[: nb * 32] = v.reshape(-1)
    return out


def np_deq_q4_0(raw, n): return _np_legacy(raw, n, 18, False, False, 8)
def np_deq_q4_1(raw, n): return _np_legacy(raw, n, 20, True, False, 0)
def np_deq_q5_0(raw, n): return _np_legacy(raw, n, 22, False, True, 16)
def np_deq_q5_1(raw, n): return _np_legacy(raw, n, 24, True, True, 0)


def np_deq_q5_k(raw, n):
    out = np.zeros(n, np.float32)
    nb = min(n // 256, len(raw) // 176)
    b = np.asarray(raw[: nb * 176], dtype=np.uint8).reshape(nb, 176)
    d = _np_f16(b[:, 0:2]).reshape(nb, 1); dmin = _np_f16(b[:, 2:4]).reshape(nb, 1)
    sc, m = np_q4k_scales(b[:, 4:16])
    qh = b[:, 16:48].reshape(nb, 1, 32)
    qs = b[:, 48:].reshape(nb, 4, 32)
    nib = np.stack([qs & 0x0F, qs >> 4], axis=2).reshape(nb, 8, 32).astype(np.int32)       # sub-block 2g, 2g+1
    bit = ((qh >> np.arange(8, dtype=np.uint8).reshape(1, 8, 1)) & 1).astype(np.int32)        # bit s of qh[l]
    d1 = (d * sc.astype(np.float32)).reshape(nb, 8, 1)
    mm = (dmin * m.astype(np.float32)).reshape(nb, 8, 1)
    out[: nb * 256] = (d1 * (nib + 16 * bit).astype(np.float32) - mm).reshape(-1)
    return out


_KV_IQ4NL = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float32)  # lib.rs:751


def np_deq_iq4_nl(raw, n):
    out = np.zeros(n, np.float32)
    nb = min(n // 32, len(raw) // 18)
    b = np.asarray(raw[: nb * 18], dtype=np.uint8).reshape(nb, 18)
    d = _np_f16(b[:, 0:2]).reshape(nb, 1)
    idx = np.concatenate([b[:, 2:] & 0x0F, b[:, 2:] >> 4], axis=1)
    out[: nb * 32] = (d * _KV_IQ4NL[idx]).reshape(-1)
    return out


def np_deq_iq4_xs(raw, n):
    out = np.zeros(n, np.float32)
    nb = min(n // 256, len(raw) // 136)
    b = np.asarray(raw[: nb * 136], dtype=np.uint8).reshape(nb, 136)
    d = _np_f16(b[:, 0:2]).reshape(nb, 1)
    sh = b[:, 2].astype(np.int32) | (b[:, 3].astype(np.int32) << 8)
    ib = np.arange(8)
    lo = (b[:, 4:8][:, ib // 2].astype(np.int32) >> (4 * (ib % 2))) & 0x0F
    hi = (sh.reshape(nb, 1) >> (2 * ib)) & 3
    dl = (d * ((lo | (hi << 4)) - 32).astype(np.float32)).reshape(nb, 8, 1)
    q = b[:, 8:].reshape(nb, 8, 16)
    idx = np.concatenate([q & 0x0F, q >> 4], axis=2)
    out[: nb * 256] = (dl * _KV_IQ4NL[idx]).reshape(-1)
    return out


def np_deq_mxfp4(raw, n):
    """lib.rs:896-908 through numpy.ldexp: table[code] / 2 * 2^(e - 127) formed in f64 and rounded once to f32, which is
    what a single correctly-rounded f32 multiply by 2^(e - 128) gives (subnormals and overflow included)."""
    out = np.zeros(n, np.float32)
    nb = min(n // 32, len(raw) // 17)
    b = np.asarray(raw[: nb * 17], dtype=np.uint8).reshape(nb, 17)
    mag = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.float64)
    idx = np.concatenate([b[:, 1:] & 0x0F, b[:, 1:] >> 4], axis=1)
    with np.errstate(over="ignore"):
        out[: nb * 32] = np.ldexp(mag[idx], b[:, 0:1].astype(np.int64) - 128).astype(np.float32).reshape(-1)
    return out


def np_deq_raw(raw, n, ty):
    return {Q8_0: np_deq_q8_0, Q4_K: np_deq_q4_k, Q6_K: np_deq_q6_k, Q4_0: np_deq_q4_0, Q4_1: np_deq_q4_1, Q5_0: np_deq_q5_0,
            Q5_1: np_deq_q5_1, Q5_K: np_deq_q5_k, IQ4_NL: np_deq_iq4_nl, IQ4_XS: np_deq_iq4_xs, MXFP4: np_deq_mxfp4}[ty](np.asarray(raw, dtype=np.uint8), n)
