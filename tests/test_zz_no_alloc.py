"""The FFN entry point that allocates nothing (its intermediate is an array built into the library) against fhip_ffn, through
the C ABI: two calls in a row, the second with a smaller input, bit for bit; and the size limit."""
import numpy as np
import pytest

from conftest import bits

pytestmark = pytest.mark.gpu
Q4_K, Q6_K = 12, 14


def test_ffn_noalloc_matches_fhip_ffn_on_two_calls_in_a_row(F, O):
    from ferric_amd.synth import synth_weights
    lib, check = F._lib.load(), F._lib.check
    n_embd, n_ff = 2048, 5120
    gu_raw, dn_raw = synth_weights(Q4_K, 2 * n_ff, n_embd, 41), synth_weights(Q6_K, n_embd, n_ff, 42)
    gu = F.QMatrix.from_bytes(gu_raw, Q4_K, 2 * n_ff, n_embd)
    dn = F.QMatrix.from_bytes(dn_raw, Q6_K, n_embd, n_ff)
    gu.batch_policy(F.BATCH_F32_MATVEC), dn.batch_policy(F.BATCH_F32_MATVEC)   # fhip_ffn on the mat-vec kernels too, so that the bits can be compared
    if True:
        for rows in (7, 2):                        # the second call is smaller: what the first left in the array must not show
            x = np.random.default_rng(43 + rows).standard_normal((rows, n_embd)).astype(np.float32)
            xt = F.Tensor.from_vec(x, x.shape)
            want = xt.ffn(gu, dn).to_vec().reshape(rows, n_embd)
            y = F.Tensor.empty((rows, n_embd))
            check(lib.fhip_memset(y.buf.ptr, 0xFF, rows * n_embd * 4, None))
            check(lib.fhip_ffn_noalloc(gu.handle, dn.handle, xt.buf.ptr, rows, y.buf.ptr, None))
            got = y.to_vec().reshape(rows, n_embd)
            assert np.array_equal(bits(got), bits(want)), rows
            # and the block itself against the oracle
            g64, _ = O.matmul_f64(x, gu_raw, Q4_K, 2 * n_ff, n_embd)
            h64 = g64[:, :n_ff] / (1.0 + np.exp(-g64[:, :n_ff])) * g64[:, n_ff:]
            y64, _ = O.matmul_f64(h64.astype(np.float32), dn_raw, Q6_K, n_embd, n_ff)
            assert np.abs(got - y64).max() <= 4e-4 * np.abs(y64).max(), rows
    # beyond the built-in array: refused, nothing launched
    rows = 131072 // n_ff + 1
    xt = F.Tensor.from_vec(np.zeros((rows, n_embd), np.float32), (rows, n_embd))
    y = F.Tensor.empty((rows, n_embd))
    rc = lib.fhip_ffn_noalloc(gu.handle, dn.handle, xt.buf.ptr, rows, y.buf.ptr, None)
    assert rc == F._lib.ERR_SHAPE and "131072" in F._lib.last_error()
