import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950); run with -m gpu")


@pytest.fixture(scope="session")
def O():
    """The CPU oracle (test infrastructure)."""
    from oracle import oracle
    oracle.build()
    return oracle


@pytest.fixture(scope="session")
def F():
    """The product package with the device initialised; fails loudly without the library or a GPU."""
    import ferric_amd
    from ferric_amd import _lib
    _lib.init(0)
    return ferric_amd


@pytest.fixture(scope="session")
def golden():
    return np.load(os.path.join(ROOT, "tests", "golden", "vectors.npz"))


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


# ---- precision of the streaming mat-vec's activations (a property of the weight handle; fhip_matvec_precision sets what new
# handles start with): the tests of the mat-vec entry points run once per setting, making their weights under it. At 24
# bits (what a handle has unless told otherwise) the dot products are held to the bar the reference's examples use for its
# scalar kernels (1e-5 of the largest output, crates/ferric-tensor/examples/q4_k.rs:54); at 16 bits (opt-in) to 2e-4: a
# 16-bit significand at the run maximum is 1.5e-5 of that maximum per activation, and the sum over a row measures 2e-5 ..
# 7e-5 of the largest output on these inputs. The north-star bound 1e-3 * ||w_row|| * ||x|| is asserted at both.
_PRECISION = {"bits": 24}


def dot_bar(scale=1.0):
    return scale * (1e-5 if _PRECISION["bits"] == 24 else 2e-4)


@pytest.fixture(params=[16, 24], ids=["x16", "x24"])
def precision(request, F):
    lib = F._lib.load()
    before = lib.fhip_matvec_precision(request.param)
    assert before in (16, 24)
    _PRECISION["bits"] = request.param
    yield request.param
    lib.fhip_matvec_precision(before)
    _PRECISION["bits"] = before


@pytest.fixture
def precision24(F):
    """For tests that use the streaming mat-vec as the f32-grade side of a comparison: the weights they make have 24-bit
    activations, and every batch on that kernel (otherwise a batch of three rows or more goes to the one-pass matrix-core
    kernels)."""
    lib = F._lib.load()
    before = lib.fhip_matvec_precision(24)
    policy = lib.fhip_batch_policy(1)
    _PRECISION["bits"] = 24
    yield
    lib.fhip_matvec_precision(before)
    lib.fhip_batch_policy(policy)
    _PRECISION["bits"] = before
