"""GPU unpackers vs the CPU oracle: bit-exact, through the C ABI (ferric_amd is a ctypes shim)."""
import numpy as np
import pytest

from conftest import bits

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q6_K = 8, 12, 14


def assert_bits_equal(got, want, what=""):
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    bad = np.nonzero(bits(got) != bits(want))[0]
    assert bad.size == 0, f"{what}: {bad.size} of {got.size} differ, first at {bad[:5]}: {got[bad[:5]]} vs {want[bad[:5]]}"


def test_f16_all_65536_patterns(F, O):
    # crates/ferric-gguf/src/lib.rs:605 rd_f16; crates/ferric-tensor/src/cpu_simd.rs:203-213
    got = F.f16_to_f32(np.arange(65536, dtype=np.uint16))
    want = O.f16_table()
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)          # NaN payloads are not part of the contract
    assert np.array_equal(bits(got)[~nan], bits(want)[~nan])
    assert got[0x0001] == np.float32(5.9604645e-8) and got[0x3C00] == 1.0 and np.isinf(got[0xFC00]) and got[0xFC00] < 0


def test_q4k_reference_known_answer(F, golden):
    # crates/ferric-gguf/examples/roundtrip.rs:54-87
    got = F.deq_raw(golden["q4k_known_block"], 256, Q4_K)
    assert_bits_equal(got, golden["q4k_known_expected"], "roundtrip.rs Q4_K block")


def test_golden_generator_blocks(F, golden):
    assert_bits_equal(F.deq_raw(golden["q4k_gen_blocks"], 1024, Q4_K), golden["q4k_gen_deq"], "q4k_block(1..4)")
    assert_bits_equal(F.deq_raw(golden["q6k_gen_blocks"], 1024, Q6_K), golden["q6k_gen_deq"], "q6k_block(1..4)")
    assert_bits_equal(F.deq_raw(golden["q8_synth_raw"], 512, Q8_0), golden["q8_synth_vals"], "cpu_simd synth ground truth")


@pytest.mark.parametrize("ty", [Q8_0, Q4_K, Q6_K])
def test_random_blocks_bit_exact(F, O, ty):
    from ferric_amd.synth import synth_weights
    for seed, (rows, cols) in enumerate([(1, 256), (3, 512), (16, 1024), (5, 5120), (7, 17408)]):
        w = synth_weights(ty, rows, cols, 200 + seed)
        assert_bits_equal(F.deq_raw(w, rows * cols, ty), O.deq_raw(w, rows * cols, ty), f"ty {ty} {rows}x{cols}")


@pytest.mark.parametrize("ty", [Q8_0, Q4_K, Q6_K])
def test_every_byte_value_and_subnormal_scales(F, O, ty):
    # uniform random bytes in every field (all 6-bit scale/min splits, all nibbles, int8 -128), with
    # the f16 scales forced finite; then the same blocks with subnormal / zero / negative scales
    rng = np.random.default_rng(17)
    vals, nbytes = O.BLOCK[ty]
    raw = rng.integers(0, 256, 4096 * nbytes, dtype=np.uint8).reshape(4096, nbytes)
    offs = {Q8_0: (0,), Q4_K: (0, 2), Q6_K: (208,)}[ty]
    for off in offs:
        raw[:, off + 1] &= 0xBB      # exponent top bit clear -> finite
    assert_bits_equal(F.deq_raw(raw, 4096 * vals, ty), O.deq_raw(raw, 4096 * vals, ty), "random bytes")
    special = np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x0400, 0x0155, 0x7BFF, 0xFBFF, 0x3C00], dtype=np.uint16)
    for off in offs:
        raw[:, off:off + 2] = np.resize(special, 4096).view(np.uint8).reshape(4096, 2)
    assert_bits_equal(F.deq_raw(raw, 4096 * vals, ty), O.deq_raw(raw, 4096 * vals, ty), "special scales")


def test_reference_generator_matrices(F, O):
    # the weights the reference examples validate with (q4_k.rs:43-47, q6_k.rs:22-26)
    for ty, shapes in ((Q4_K, [(8, 256), (13, 512)]), (Q6_K, [(8, 256), (7, 512)])):
        for rows, cols in shapes:
            w = O.gen_kquant_matrix(ty, rows, cols)
            assert_bits_equal(F.deq_raw(w, rows * cols, ty), O.deq_raw(w, rows * cols, ty))
    wf = (np.sin(np.arange(13 * 128, dtype=np.float32) * np.float32(0.021)) * np.float32(0.7)).astype(np.float32)
    w = O.quant_q8_0(wf)                                                  # q8_0.rs:11-13
    assert_bits_equal(F.deq_raw(w, 13 * 128, Q8_0), O.deq_raw(w, 13 * 128, Q8_0))


def test_deq_raw_edge_semantics(F, O):
    from ferric_amd.synth import synth_weights
    w = synth_weights(Q4_K, 1, 512, 1)
    for n in (0, 255, 256, 300, 512, 700):                                # ragged tail stays 0.0 (lib.rs:794)
        assert_bits_equal(F.deq_raw(w, n, Q4_K), O.deq_raw(w, n, Q4_K), f"Q4_K n={n}")
    assert_bits_equal(F.deq_raw(w[:194], 512, Q4_K), O.deq_raw(w[:194], 512, Q4_K))   # bytes run out first
    w = synth_weights(Q6_K, 1, 512, 1)
    for n in (0, 100, 300, 512, 600):
        assert_bits_equal(F.deq_raw(w, n, Q6_K), O.deq_raw(w, n, Q6_K), f"Q6_K n={n}")
    w = synth_weights(Q8_0, 1, 128, 1)
    for n in (0, 31, 32, 70, 128, 200):                                   # Q8_0 returns whole blocks only (lib.rs:609-614)
        got = F.deq_raw(w, n, Q8_0)
        assert got.size == min(n // 32, 4) * 32
        assert_bits_equal(got, O.deq_raw(w, n, Q8_0), f"Q8_0 n={n}")
    with pytest.raises(ValueError, match="unsupported ggml type 10"):     # lib.rs:518 (Q2_K)
        F.deq_raw(np.zeros(84, np.uint8), 256, 10)


def test_deq_raw_unquantized_types(F, O):
    # lib.rs:499-501: F32 / F16 / BF16 tensors through the same entry point, every 16-bit pattern, bit for bit
    pats = np.arange(65536, dtype=np.uint16).view(np.uint8)
    for ty in (F.F16, F.BF16):
        got, want = F.deq_raw(pats, 65536, ty), O.deq_raw(pats, 65536, ty)
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan)
        assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
        assert_bits_equal(F.deq_raw(pats[:2000], 1000, ty), O.deq_raw(pats[:2000], 1000, ty))
        assert F.deq_raw(pats, 0, ty).size == 0
        with pytest.raises(AssertionError, match="out of range"):
            F.deq_raw(pats[:7], 4, ty)
    raw32 = np.random.default_rng(0).integers(0, 1 << 32, 5000, dtype=np.uint64).astype(np.uint32)
    raw32[:4] = [0x7FC00001, 0xFF800000, 0x00000001, 0x80000000]
    assert np.array_equal(F.deq_raw(raw32.view(np.uint8), 5000, F.F32).view(np.uint32), raw32)
    assert F.deq_raw(raw32.view(np.uint8), 17, F.F32).size == 17
    with pytest.raises(AssertionError, match="out of range"):
        F.deq_raw(raw32.view(np.uint8)[:15], 4, F.F32)
    assert F.type_size(F.F32, 5120) == 20480 and F.type_size(F.F16, 5120) == 10240 and F.type_size(F.BF16, 3) == 6


@pytest.mark.parametrize("ty,rows,cols", [(Q4_K, 64, 5120), (Q6_K, 33, 5120), (Q8_0, 40, 4096)])
def test_resident_weight_row_dequant(F, O, ty, rows, cols):
    # embedding-row dequant out of a weight already in HBM (crates/ferric-llama/src/qwen3.rs:749)
    from ferric_amd.synth import synth_weights
    w = synth_weights(ty, rows, cols, 31)
    qm = F.QMatrix.from_bytes(w, ty, rows, cols)
    want = O.deq_raw(w, rows * cols, ty).reshape(rows, cols)
    assert_bits_equal(qm.dequant().to_vec().reshape(rows, cols), want)
    for r0, n in ((0, 1), (rows - 1, 1), (5, 7), (0, 0)):
        assert_bits_equal(qm.dequant_rows(r0, n).to_vec().reshape(n, cols), want[r0:r0 + n])
    with pytest.raises(AssertionError):
        qm.dequant_rows(rows - 1, 2)


def test_full_size_matrices_bit_exact(F, O):
    # the benchmark matrices themselves: Q8_0 4096x4096, Q4_K 5120x5120, and 1024 rows of the Q6_K 5120x17408 down projection
    from ferric_amd.synth import synth_weights
    for ty, rows, cols, seed in ((Q8_0, 4096, 4096, 0), (Q4_K, 5120, 5120, 1), (Q6_K, 1024, 17408, 2)):
        w = synth_weights(ty, rows, cols, seed)
        got = F.deq_raw(w, rows * cols, ty)
        want = O.deq_raw(w, rows * cols, ty)
        assert np.array_equal(bits(got), bits(want)), (ty, rows, cols)
