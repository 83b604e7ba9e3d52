"""Builds libllmq_fp8.so (the C-ABI library with the gfx950 kernels) with hipcc, in-tree.

    python -m llmq_amd.build          # rebuild everything
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "build")
LIB = os.path.join(HERE, "lib", "libllmq_fp8.so")

SOURCES = ["runtime.hip", "absmax.hip", "quantize.hip", "transpose.hip", "gemm_e4m3.hip", "bias.hip", "swiglu.hip", "rmsnorm.hip", "rope.hip", "adamw.hip", "calibrate.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC",
    "-ffp-contract=off",                       # the epilogue and the quantize multiply are defined op by op
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-enable-post-misched=0",       # keep the hand-specified interleave of the GEMM K loop
    "-Wall", "-Wextra", "-Wno-unused-parameter", "-Wno-unknown-warning-option",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def _compile(src):
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, out


def build(verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        results = list(ex.map(_compile, SOURCES))
    for obj, out in results:
        if verbose and out.strip():
            print(out)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + [o for o, _ in results]
    subprocess.check_call(cmd)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
