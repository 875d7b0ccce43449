"""Compile libforge_hip.so for gfx950 with hipcc (in-tree; no GPU needed to build)."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
BUILD = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libforge_hip.so")

SOURCES = ["format.hip", "elementwise.hip", "gemv.hip", "gemv_f32.hip", "gemv_kquant.hip", "kquant_prefill.hip", "gemm.hip", "attn_decode.hip", "attn_prefill.hip",
           "attn_exact.hip", "decode_persistent.hip", "api.hip", "model.hip", "gguf.cpp", "sampling.cpp"]

# -packed-fp32-ops off: keep hipcc from forming packed FP32 instructions.
# -ffp-contract=off: the CPU path never fuses a*b+c; kernels say fmaf() where a fused op is meant.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-Wno-pass-failed", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-I", INCLUDE, "-I", CSRC]


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    return "hipcc"


def _compile(src):
    obj = os.path.join(BUILD, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless, filter it
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=True):
    os.makedirs(BUILD, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build()
