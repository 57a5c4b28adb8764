"""Builds libferric_hip.so (gfx950 only) in-tree with hipcc.

    python -m ferric_amd.build

Every translation unit is compiled for gfx950 with packed-FP32 instruction selection switched
off; dequant.hip and kvquant.hip additionally with -ffp-contract=off, because their outputs
must match the reference's separately-rounded f32 arithmetic bit for bit.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libferric_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

COMMON = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
UNITS = {
    "api.hip": [],
    "dequant.hip": ["-ffp-contract=off"],
    "kvquant.hip": ["-ffp-contract=off"],       # the reference multiplies, then adds: no fused multiply-add
    "gemv.hip": ["-DFHIP_GEMV_PLANES=2"],
    "gemv.hip@p3": ["-DFHIP_GEMV_PLANES=3"],   # the same source again: the 24-bit-activation copy of the streaming mat-vec
    "gemv_quad.hip": ["-DFHIP_GEMV_PLANES=2"],
    "gemv_quad.hip@p3": ["-DFHIP_GEMV_PLANES=3"],
    "gemv_generic.hip": [],
    "gemm_mfma.hip": [],
    "gemm_f16x2.hip": [],
    "moe.hip": [],
    "probe.hip": [],
    "decode_ops.hip": [],
    "prefill_attn.hip": [],
    "gguf.hip": [],
}


def _compile(name, flags, objdir, verbose):
    src = os.path.join(CSRC, name.split("@")[0])
    obj = os.path.join(objdir, name.replace("@", "_") + ".o")
    cmd = [HIPCC] + COMMON + flags + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the device-only feature flag; that warning is noise.
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {name}:\n{out}")
    if verbose and out.strip():
        print(out)
    return obj


def build(verbose=False):
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=6) as ex:
        objs = list(ex.map(lambda kv: _compile(kv[0], kv[1], objdir, verbose), UNITS.items()))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    return OUT


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
