"""Writes tests/golden/mxfp4_ggml.json: the MXFP4 known-answer data the reference's own tests hold, captured there
from ggml (crates/ferric-gguf/src/lib.rs:1099-1170): GG_E x 16 codes -> GG_GRID (f32 bit patterns), and REAL_RAW (the
first 8 blocks of a real tensor) -> REAL_GGML. Reads the reference's source as text; run once where the checkout is
present:  python tests/golden/make_mxfp4_golden.py [/root/reference]"""
import json
import os
import re
import sys


def array(text, name):
    m = re.search(r"const %s: \[[^\]]+\] = \[(.*?)\];" % name, text, flags=re.S)
    body = re.sub(r"//[^\n]*", "", m.group(1))
    return [int(t, 0) for t in re.findall(r"0x[0-9a-fA-F]+|\b\d+\b", body)]


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    text = open(os.path.join(root, "crates/ferric-gguf/src/lib.rs"), encoding="utf-8").read()
    out = {k: array(text, n) for k, n in (("e", "GG_E"), ("grid_bits", "GG_GRID"), ("real_raw", "REAL_RAW"), ("real_bits", "REAL_GGML"))}
    assert [len(out[k]) for k in ("e", "grid_bits", "real_raw", "real_bits")] == [10, 160, 136, 256]
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "mxfp4_ggml.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))


if __name__ == "__main__":
    main()
