"""GGUF tensor -> HBM weight straight from the mapped file, then the ordinary entry points on it."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(__file__))
from conftest import dot_bar  # noqa: E402
from gguf_writer import write_gguf  # noqa: E402

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q6_K = 8, 12, 14


def test_weights_from_a_gguf_file(F, O, tmp_path):
    from ferric_amd.synth import synth_weights
    shapes = {"blk.0.attn_q.weight": (Q4_K, 48, 1024), "blk.0.ffn_down.weight": (Q6_K, 40, 512), "output.weight": (Q8_0, 33, 96)}
    raw = {n: synth_weights(ty, r, c, 5 + i) for i, (n, (ty, r, c)) in enumerate(shapes.items())}
    n_expert, rows_pe, cols = 4, 24, 256
    raw["blk.0.ffn_down_exps.weight"] = synth_weights(Q4_K, n_expert * rows_pe, cols, 9)
    tensors = [(n, [c, r], ty, raw[n]) for n, (ty, r, c) in shapes.items()]
    tensors.append(("blk.0.ffn_down_exps.weight", [cols, rows_pe, n_expert], Q4_K, raw["blk.0.ffn_down_exps.weight"]))
    norm = np.random.default_rng(3).standard_normal(1024).astype(np.float32)
    embd = np.random.default_rng(4).standard_normal(512).astype(np.float16)
    tensors.append(("blk.0.attn_norm.weight", [1024], 0, norm.view(np.uint8)))
    tensors.append(("token_embd.weight", [64, 8], 1, embd.view(np.uint8)))
    data = write_gguf([("general.architecture", "str", "qwen3")], tensors)[0]
    path = tmp_path / "tiny.gguf"
    path.write_bytes(data)
    g = F.GgufFile.open(path)
    rng = np.random.default_rng(2)
    for name, (ty, r, c) in shapes.items():
        w = g.qmatrix(name)
        assert (w.rows(), w.cols(), w.ggml_type, w.nbytes()) == (r, c, ty, raw[name].size)
        assert np.array_equal(w.dequant().to_vec().view(np.uint32), O.deq_raw(raw[name], r * c, ty).view(np.uint32))
        x = rng.standard_normal((2, c)).astype(np.float32)
        y = F.Tensor.from_vec(x.reshape(-1), (2, c)).matmul_q(w).to_vec()
        y0 = F.Tensor.from_vec(x.reshape(-1), (2, c)).matmul_q(F.QMatrix.from_bytes(raw[name], ty, r, c)).to_vec()
        assert np.array_equal(y.view(np.uint32), y0.view(np.uint32))
    # an expert slab [in, rows per expert, n_expert] becomes one weight of n_expert * rows_pe rows, expert-major
    slab = g.qmatrix("blk.0.ffn_down_exps.weight")
    assert (slab.rows(), slab.cols()) == (n_expert * rows_pe, cols)
    k = 2
    x = rng.standard_normal((k, cols)).astype(np.float32)
    sel = np.array([[0.25, 0.75, 3.0, 1.0]], np.float32)
    got = F.Tensor.from_vec(x.reshape(-1), (k, cols)).matmul_q4_k_id_wsum(slab, F.Tensor.from_vec(sel.reshape(-1), (1, 4)), rows_pe).to_vec()
    want, bound = O.matmul_id_wsum_f64(x, raw["blk.0.ffn_down_exps.weight"], Q4_K, sel, k, rows_pe, cols)
    assert (np.abs(got - want[0]) <= 1e-3 * bound[0]).all()
    with pytest.raises(AssertionError, match="has 1 dims"):
        g.qmatrix("blk.0.attn_norm.weight")          # F32 [1024]: listed, readable, but not a matrix
    with pytest.raises(ValueError, match="no native matmul for ggml type 1"):
        g.qmatrix("token_embd.weight")               # F16 [64, 8]: not one of the quantized formats of this path
    assert g.raw("token_embd.weight").size == 1024
    # lib.rs:575 dequant(name): any tensor of the file as f32, the unquantized ones included
    assert np.array_equal(g.dequant("blk.0.attn_norm.weight").view(np.uint32), norm.view(np.uint32))
    assert np.array_equal(g.dequant("token_embd.weight").view(np.uint32), embd.astype(np.float32).view(np.uint32))
    assert np.array_equal(g.dequant("blk.0.ffn_down.weight").view(np.uint32), O.deq_raw(raw["blk.0.ffn_down.weight"], 40 * 512, Q6_K).view(np.uint32))
    with pytest.raises(ValueError, match="no tensor"):
        g.dequant("missing")
    with pytest.raises(ValueError, match="no tensor"):
        g.qmatrix("missing")


def test_fused_projections_from_a_gguf_file(F, O, tmp_path, precision):
    # qwen35.rs:379-402 qm_cat and qwen3.rs:192-228 Proj: Q, K, V of one format fuse into one weight (bit-identical to the
    # weight made from the concatenated bytes); a V of another format keeps the projection split, outputs concatenated
    from ferric_amd.synth import synth_weights
    d = 512
    spec = {"blk.0.attn_q.weight": (Q4_K, 96), "blk.0.attn_k.weight": (Q4_K, 32), "blk.0.attn_v.weight": (Q4_K, 32),
            "blk.1.attn_v.weight": (Q6_K, 32), "blk.0.ffn_gate.weight": (Q4_K, 160), "blk.0.ffn_up.weight": (Q4_K, 160),
            "blk.0.ffn_gate8.weight": (Q8_0, 64), "blk.0.ffn_up8.weight": (Q8_0, 64), "narrow.weight": (Q4_K, 16)}
    raw = {n: synth_weights(ty, r, 256 if n == "narrow.weight" else d, 20 + i) for i, (n, (ty, r)) in enumerate(spec.items())}
    tensors = [(n, [256 if n == "narrow.weight" else d, r], ty, raw[n]) for n, (ty, r) in spec.items()]
    path = tmp_path / "proj.gguf"
    path.write_bytes(write_gguf([("general.architecture", "str", "qwen3")], tensors)[0])
    g = F.GgufFile.open(path)
    x = np.random.default_rng(6).standard_normal((3, d)).astype(np.float32)
    xt = F.Tensor.from_vec(x, x.shape)

    qkv = ["blk.0.attn_q.weight", "blk.0.attn_k.weight", "blk.0.attn_v.weight"]
    w = g.qm_cat(qkv)
    assert (w.rows(), w.cols(), w.ggml_type) == (160, d, Q4_K)
    cat_bytes = np.concatenate([raw[n] for n in qkv])
    assert np.array_equal(w.dequant().to_vec().view(np.uint32), O.deq_raw(cat_bytes, 160 * d, Q4_K).view(np.uint32))
    want = xt.matmul_q(F.QMatrix.from_bytes(cat_bytes, Q4_K, 160, d)).to_vec()
    p = F.Proj.load(g, qkv)
    assert p.fused is not None and np.array_equal(p.matmul(xt).to_vec().view(np.uint32), want.view(np.uint32))
    same = F.QMatrix.from_parts([raw[n] for n in qkv], Q4_K, 160, d)         # the same stacking from separate host arrays
    assert np.array_equal(xt.matmul_q(same).to_vec().view(np.uint32), want.view(np.uint32))

    mixed = ["blk.0.attn_q.weight", "blk.0.attn_k.weight", "blk.1.attn_v.weight"]
    p = F.Proj.load(g, mixed)
    assert p.fused is None and len(p.split) == 3
    y = p.matmul(xt).to_vec().reshape(3, 160)
    parts = [xt.matmul_q(F.QMatrix.from_bytes(raw[n], spec[n][0], spec[n][1], d)).to_vec().reshape(3, -1) for n in mixed]
    assert np.array_equal(y.view(np.uint32), np.concatenate(parts, axis=1).view(np.uint32))
    with pytest.raises(ValueError, match="blk.1.attn_v.weight: mixed quant formats in one fused matmul"):
        g.qm_cat(mixed)
    with pytest.raises(ValueError, match="narrow.weight: input dim differs"):
        g.qm_cat(["blk.0.attn_q.weight", "narrow.weight"])
    with pytest.raises(ValueError, match="no tensor 'nope'"):
        g.qm_cat(["blk.0.attn_q.weight", "nope"])
    with pytest.raises(ValueError, match="no tensor 'nope'"):
        g.qm("nope")
    assert F.Proj.load(g, ["blk.0.attn_q.weight"]).fused.rows() == 96

    # gate|up: one fused kernel for the K-quant pair, matmul + SwiGLU for the Q8_0 pair; both equal the unfused steps
    for names, n_ff in ((["blk.0.ffn_gate.weight", "blk.0.ffn_up.weight"], 160), (["blk.0.ffn_gate8.weight", "blk.0.ffn_up8.weight"], 64)):
        p = F.Proj.load(g, names)
        got = p.gate_up_swiglu(xt, n_ff).to_vec().reshape(3, n_ff)
        ty = spec[names[0]][0]
        g64, _ = O.matmul_f64(x, np.concatenate([raw[n] for n in names]), ty, 2 * n_ff, d)
        want = g64[:, :n_ff] / (1.0 + np.exp(-g64[:, :n_ff])) * g64[:, n_ff:]
        assert np.abs(got - want).max() <= dot_bar() * np.abs(want).max()
        unfused = p.matmul(xt).swiglu(n_ff).to_vec().reshape(3, n_ff)
        # (three rows: the fused K-quant kernel is the mat-vec, block fixed point activations at the precision under test; the plain
        # matmul of the unfused steps takes the one-pass f16 kernels. The Q8_0 pair runs the same kernel both ways.)
        assert np.abs(got - unfused).max() <= (2e-6 if ty == Q8_0 else dot_bar()) * np.abs(unfused).max()


def test_cat_of_tensors(F):
    # lib.rs:201 Tensor::cat for the vectors and matrices of this path
    a = np.arange(12, dtype=np.float32).reshape(3, 4)
    b = -np.arange(6, dtype=np.float32).reshape(3, 2)
    ta, tb = F.Tensor.from_vec(a, a.shape), F.Tensor.from_vec(b, b.shape)
    assert np.array_equal(ta.cat(tb, 1).to_vec().reshape(3, 6), np.concatenate([a, b], axis=1))
    c = np.ones((2, 4), np.float32)
    assert np.array_equal(ta.cat(F.Tensor.from_vec(c, c.shape), 0).to_vec().reshape(5, 4), np.concatenate([a, c], axis=0))
    with pytest.raises(AssertionError, match="cat: dim 0 mismatch"):
        ta.cat(F.Tensor.from_vec(c, c.shape), 1)
    with pytest.raises(AssertionError, match="cat: rank mismatch"):
        ta.cat(F.Tensor.from_vec(np.zeros(4, np.float32), (4,)), 0)
