"""CPU-side checks of the C-ABI boundary: the library loads without a GPU and exports exactly the
symbols include/ferric_hip.h declares; no compute entry point is called here."""
import ctypes
import os
import re

import pytest

from conftest import ROOT


HEADERS = ("ferric_hip.h", "ferric_hip_debug.h")   # the interface a caller binds, and the measurement / test aids of the same library


def _header_text(names=HEADERS):
    text = "".join(open(os.path.join(ROOT, "include", n)).read() for n in names)
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def _declared(names=HEADERS):
    return sorted(set(re.findall(r"\b(fhip_[a-z0-9_]+)\s*\(", _header_text(names))))


def test_debug_entry_points_stay_out_of_the_product_header():
    product, aids = _declared(("ferric_hip.h",)), _declared(("ferric_hip_debug.h",))
    assert not [n for n in product if n.startswith("fhip_debug_")]
    assert aids and all(n.startswith("fhip_debug_") for n in aids)


def test_library_exports_every_declared_symbol():
    from ferric_amd import _lib
    names = _declared()
    assert len(names) >= 30
    assert sorted(_lib.SYMBOLS) == names, "ctypes table and header disagree"
    lib = ctypes.CDLL(_lib.SO_PATH)
    for n in names:
        assert hasattr(lib, n), n


def test_no_undeclared_fhip_exports():
    from ferric_amd import _lib
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.SO_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(set(re.findall(r"\bT (fhip_[a-z0-9_]+)$", out, flags=re.M)))
    assert exported == _declared()


def test_the_rust_binding_declares_the_same_entry_points():
    # crates/ferric-hip/src/ffi.rs is the binding a maintainer links: one `pub fn` per entry point of the header, with as many
    # arguments as the C prototype has
    text = _header_text()
    c_args = {}
    for name, args in re.findall(r"\b(fhip_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        args = " ".join(args.split())
        c_args[name] = 0 if args in ("", "void") else args.count(",") + 1
    rust = open(os.path.join(ROOT, "crates", "ferric-hip", "src", "ffi.rs")).read()
    r_args = {}
    for name, args in re.findall(r"pub fn (fhip_[a-z0-9_]+)\(([^)]*)\)", rust):
        r_args[name] = 0 if not args.strip() else args.count(",") + 1
    assert sorted(r_args) == _declared()
    assert r_args == c_args


def test_size_tables_need_no_device():
    # crates/ferric-gguf/src/lib.rs:471-494 and crates/ferric-tensor/src/dtype.rs:873-889
    from ferric_amd import QMatrix, type_size
    assert QMatrix.block_bytes(8) == (32, 34) and QMatrix.block_bytes(12) == (256, 144) and QMatrix.block_bytes(14) == (256, 210)
    assert [QMatrix.block_bytes(t) for t in (2, 3, 6, 7, 13)] == [(32, 18), (32, 20), (32, 22), (32, 24), (256, 176)]
    assert QMatrix.block_bytes(10) is None and QMatrix.block_bytes(0) is None
    assert type_size(8, 4096 * 4096) == 17825792 and type_size(12, 5120 * 5120) == 14745600 and type_size(14, 5120 * 17408) == 73113600
    assert type_size(12, 300) == 144
    assert type_size(0, 5120) == 20480 and type_size(1, 5120) == 10240 and type_size(30, 5120) == 10240   # F32, F16, BF16
    assert type_size(13, 5120 * 5120) == 18022400 and type_size(2, 64) == 36 and type_size(7, 33) == 24
    with pytest.raises(ValueError, match="unsupported ggml type 10"):
        type_size(10, 256)


def test_compute_refuses_to_run_uninitialised():
    # without fhip_init (no GPU here) every device entry point reports an error instead of falling back
    from ferric_amd import _lib
    lib = _lib.load()
    if _lib._inited:
        pytest.skip("device already initialised in this process")
    p = ctypes.c_void_p()
    assert lib.fhip_malloc(ctypes.byref(p), 16) == _lib.ERR_ARG
    assert b"fhip_init" in lib.fhip_last_error()
    n = ctypes.c_size_t()
    assert lib.fhip_deq_raw(None, 0, 0, 8, None, ctypes.byref(n)) == _lib.ERR_ARG


def test_product_does_not_import_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "ferric_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.lower() or f == "synth.py" and "oracle" not in src, (dirpath, f)
