"""Builds the gfx950 libraries with hipcc, in-tree.

    python -m llmq_amd.build          # rebuild everything

lib/libllmq_fp8.so          the product: the C ABI of include/llmq_fp8.h and nothing else (hidden visibility)
lib/libllmq_fp8_testaid.so  for tests and bench.py only: the GEMM file compiled with LLMQ_TEST_HOOKS (the parity
                            tests force every kernel instantiation through llmq_debug_set_gemm_variant) plus the
                            measurement aids of calibrate.hip (plain copy kernel, register-only MFMA loop)
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
TESTAID_LIB = os.path.join(HERE, "lib", "libllmq_fp8_testaid.so")

SOURCES = ["runtime.hip", "absmax.hip", "quantize.hip", "transpose.hip", "gemm_e4m3.hip", "bias.hip", "swiglu.hip",
           "rmsnorm.hip", "rope.hip", "adamw.hip", "producers_f32.hip"]
# (source, object name, extra flags)
TESTAID_UNITS = [("gemm_e4m3.hip", "gemm_e4m3_hooks.o", ["-DLLMQ_TEST_HOOKS"]), ("calibrate.hip", "calibrate.o", []),
                 ("runtime.hip", "runtime.o", [])]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-fvisibility=hidden",
    "-ffp-contract=off",                       # the epilogue and the quantize multiply are defined op by op
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-enable-post-misched=0",       # keep the hand-specified interleave of the GEMM K loop
    "-Wall", "-Wextra", "-Wno-unused-parameter", "-Wno-unknown-warning-option",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def _compile(unit):
    src, obj_name, extra = unit
    obj = os.path.join(OBJ, obj_name)
    cmd = [HIPCC] + FLAGS + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, out


def _hazard_scan(_unit=None):
    """The GEMM file compiled to assembly text and scanned for the two hazards its inline-asm copies could meet
    (asm_check.py); runs beside the object compiles.  A violation raises and nothing is linked."""
    from llmq_amd import asm_check
    return asm_check.check_source(HIPCC, FLAGS, os.path.join(CSRC, "gemm_e4m3.hip"), os.path.join(OBJ, "gemm_e4m3.hazard_scan.s"))


def _link(lib, objs):
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-Bsymbolic",
                           "-Wl,--version-script=" + os.path.join(CSRC, "exports.map"), "-o", lib] + objs)


def build(verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    units = [(s, s.replace(".hip", ".o"), []) for s in SOURCES]
    extra_units = [u for u in TESTAID_UNITS if u[1] not in {n for _, n, _ in units}]
    with ThreadPoolExecutor(max_workers=8) as ex:
        scan = ex.submit(_hazard_scan)
        results = dict(zip([u[1] for u in units + extra_units], ex.map(_compile, units + extra_units)))
        kernels, copies = scan.result()   # raises on a hazard: nothing is linked
    if verbose:
        print("hazard scan of the four-wave GEMM: %d kernel instances, %d copies, clean" % (kernels, copies))
    for obj, out in results.values():
        if verbose and out.strip():
            print(out)
    _link(LIB, [results[n][0] for _, n, _ in units])
    _link(TESTAID_LIB, [results[n][0] for _, n, _ in TESTAID_UNITS])
    if verbose:
        print("built", LIB)
        print("built", TESTAID_LIB)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
