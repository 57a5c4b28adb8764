"""GGUF tensor -> HBM weight straight from the mapped file, then the ordinary entry points on it."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(__file__))
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
