"""GGUF ingest (host side, no device): the native reader behind fhip_gguf_* against the Python restatement of
the reference's parser, against files laid out by an independent writer, and against the numbers of the
reference's own stride test (crates/ferric-gguf/src/lib.rs:1425-1458)."""
import os
import struct
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(__file__))
from gguf_writer import write_gguf  # noqa: E402

Q8_0, Q4_K, Q6_K = 8, 12, 14


@pytest.fixture(scope="module")
def G():
    from ferric_amd import _lib
    _lib.load()
    from ferric_amd import gguf
    return gguf


@pytest.fixture(scope="module")
def GO():
    from oracle import gguf_oracle
    return gguf_oracle


def sample_file(align=None):
    rng = np.random.default_rng(1)
    raw = {"a.weight": rng.integers(0, 256, 4 * 144 * 3, dtype=np.uint8),      # Q4_K [1024, 3]
           "b.weight": rng.integers(0, 256, 2 * 210 * 5, dtype=np.uint8),      # Q6_K [512, 5]
           "c.weight": rng.integers(0, 256, 3 * 34 * 7, dtype=np.uint8),       # Q8_0 [96, 7]
           "exps": rng.integers(0, 256, 144 * 2 * 4, dtype=np.uint8),          # Q4_K [256, 2, 4] expert slab
           "norm": rng.integers(0, 256, 4 * 16, dtype=np.uint8)}               # F32 [16]
    tensors = [("a.weight", [1024, 3], Q4_K, raw["a.weight"]), ("b.weight", [512, 5], Q6_K, raw["b.weight"]),
               ("c.weight", [96, 7], Q8_0, raw["c.weight"]), ("exps", [256, 2, 4], Q4_K, raw["exps"]), ("norm", [16], 0, raw["norm"])]
    meta = [("general.architecture", "str", "qwen3"), ("qwen3.block_count", "u32", 64), ("t.u8", "u8", 250), ("t.i8", "i8", -3),
            ("t.u16", "u16", 65000), ("t.i16", "i16", -12345), ("t.i32", "i32", -2**31), ("t.f32", "f32", 1.5), ("t.bool", "bool", 1),
            ("t.u64", "u64", 2**63 + 5), ("t.i64", "i64", -2**62), ("t.f64", "f64", 1e-300), ("tokenizer.tokens", "arr:str", ["a", "bc", ""]),
            ("t.arr_i32", "arr:i32", [1, -2, 3]), ("t.arr_f32", "arr:f32", [0.25, -8.0]), ("t.empty", "arr:u8", []), ("utf8", "str", "naïve ✓")]
    data, data_start, offs = write_gguf(meta, tensors, align=align)
    return data, data_start, offs, raw, meta, tensors


@pytest.mark.parametrize("align", [None, 64, 4096])
def test_header_metadata_tensor_table_and_raw_bytes(G, GO, align, tmp_path):
    data, data_start, offs, raw, meta, tensors = sample_file(align)
    want = GO.parse(data)
    assert want["data_start"] == data_start                                     # the oracle agrees with the writer's layout
    path = tmp_path / "m.gguf"
    path.write_bytes(data)
    for g in (G.Gguf.parse(data), G.GgufFile.open(path)):
        assert g.version == 3 and g.data_start == data_start
        assert [(t.name, t.dims, t.ggml_type, t.offset) for t in g.tensors] == want["tensors"]
        assert [(t.name, t.dims, t.ggml_type, t.offset) for t in g.tensors] == [(t[0], t[1], t[2], offs[t[0]]) for t in tensors]
        pm = {k: v[1] if v[0] != "Arr" else [e[1] for e in v[1]] for k, v in want["metadata"].items()}
        assert g.metadata == pm
        assert g.metadata["t.u64"] == 2**63 + 5 and g.metadata["t.i32"] == -2**31 and g.metadata["t.bool"] is True
        assert g.metadata["tokenizer.tokens"] == ["a", "bc", ""] and g.metadata["utf8"] == "naïve ✓"
        for name, r in raw.items():
            assert np.array_equal(g.raw(name), r), name
        assert g.tensor("a.weight").dims == [1024, 3] and g.tensor("nope") is None
        with pytest.raises(ValueError, match="no tensor 'nope'"):
            g.raw("nope")
        g.close()


def test_not_gguf_and_every_truncation_is_refused_not_crashed(G, GO):
    data = sample_file()[0]
    with pytest.raises(ValueError, match="not a GGUF file"):
        G.Gguf.parse(b"GGML" + data[4:])
    with pytest.raises(ValueError, match="not a GGUF file"):
        G.Gguf.parse(b"")
    header_end = GO.parse(data)["data_start"]
    outcomes = set()
    for n in list(range(0, header_end + 8)) + [len(data) - 1]:
        cut = data[:n]
        try:
            GO.parse(cut)
            want = "ok"
        except ValueError as e:
            want = str(e)[:24]
        try:
            G.Gguf.parse(cut).close()
            got = "ok"
        except ValueError as e:
            got = str(e)[:24]
        assert got == want, n
        outcomes.add(got)
    assert {"not a GGUF file", "GGUF header truncated or", "ok"} <= outcomes
    # garbage counts and lengths: a string longer than the file, an array longer than the file, an unknown value type
    head = b"GGUF" + struct.pack("<IQQ", 3, 0, 1)
    for tail in (struct.pack("<Q", 1 << 60) + b"k", struct.pack("<Q", 1) + b"k" + struct.pack("<IIQ", 9, 4, 1 << 50),
                 struct.pack("<Q", 1) + b"k" + struct.pack("<I", 13) + b"\0" * 64,
                 ):
        with pytest.raises(ValueError, match="truncated or malformed"):
            G.Gguf.parse(head + tail)
    with pytest.raises(ValueError, match="truncated or malformed"):            # tensor with 2^31 dims
        G.Gguf.parse(b"GGUF" + struct.pack("<IQQ", 3, 1, 0) + struct.pack("<Q", 1) + b"t" + struct.pack("<I", 1 << 31) + b"\0" * 64)


def test_stride_refusals_with_the_references_own_numbers(G, GO):
    # lib.rs:1425-1458: two 1024-element Q8_0 tensors, 1088 bytes each
    blob = np.zeros(1088, np.uint8)
    ok = write_gguf([], [("a", [1024], Q8_0, blob, 0), ("b", [1024], Q8_0, blob, 1088)])[0]
    G.Gguf.parse(ok).close()
    assert GO.check_declared_strides([("a", [1024], Q8_0, 0), ("b", [1024], Q8_0, 1088)], 2176, 32) is None
    over = write_gguf([], [("a", [1024], Q8_0, blob, 0), ("b", [1024], Q8_0, blob, 700)], pad_data_to=2176)[0]
    for fn in (G.Gguf.parse, GO.parse):
        with pytest.raises(ValueError) as e:
            fn(over)
        assert "needs 1088 bytes" in str(e.value) and "only 700" in str(e.value)
    under = write_gguf([], [("a", [1024], Q8_0, blob, 0), ("b", [1024], Q8_0, blob, 40000)])[0]
    for fn in (G.Gguf.parse, GO.parse):
        with pytest.raises(ValueError) as e:
            fn(under)
        assert "is 1088 bytes" in str(e.value) and "reserves 40000" in str(e.value)
    # a header probe (a prefix that ends before the tensors begin) must still parse: the last bound is skipped
    start = GO.parse(ok)["data_start"]
    G.Gguf.parse(ok[:start + 16]).close()
    assert GO.check_declared_strides([("a", [1024], Q8_0, 0), ("b", [1024], Q8_0, 1088)], 16, 32) is None
    # the last tensor overrunning a complete file is refused
    short = write_gguf([], [("a", [1024], Q8_0, blob, 0), ("b", [1024], Q8_0, blob[:500], 1088)])[0]
    for fn in (G.Gguf.parse, GO.parse):
        with pytest.raises(ValueError, match="needs 1088 bytes"):
            fn(short)
    # alignment padding between tensors is legal, and an unknown type id is skipped by the check
    G.Gguf.parse(write_gguf([], [("a", [1024], Q8_0, blob), ("x", [7], 99, blob[:10]), ("b", [1024], Q8_0, blob)], align=256)[0]).close()


def test_native_type_table_agrees_with_the_oracles_for_every_id(G, GO):
    # two tensors of each type back to back at exactly the oracle's size load; one byte less is refused with that size
    for ty, (vals, _) in GO.TYPE_SIZE.items():
        n = vals * 6
        sz = GO.type_size(ty, n)
        blob = np.zeros(sz, np.uint8)
        G.Gguf.parse(write_gguf([], [("a", [n], ty, blob, 0), ("b", [n], ty, blob, sz)])[0]).close()
        with pytest.raises(ValueError, match=f"needs {sz} bytes"):
            G.Gguf.parse(write_gguf([], [("a", [n], ty, blob, 0), ("b", [n], ty, blob, sz - 1)], pad_data_to=2 * sz)[0])


def test_type_sizes_of_the_whole_table(GO):
    # lib.rs:460-484, the block geometry of every id the stride check may meet
    for ty, n, want in [(0, 10, 40), (1, 10, 20), (30, 10, 20), (8, 64, 68), (2, 64, 36), (3, 64, 40), (6, 64, 44), (7, 64, 48),
                        (12, 512, 288), (13, 512, 352), (14, 512, 420), (20, 64, 36), (23, 512, 272), (35, 512, 132), (39, 64, 34),
                        (41, 256, 36), (42, 256, 68), (1042, 256, 258)]:
        assert GO.type_size(ty, n) == want
    with pytest.raises(ValueError, match="unsupported ggml type 99"):
        GO.type_size(99, 32)
