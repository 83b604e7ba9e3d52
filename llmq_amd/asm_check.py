"""Static check of the generated code of the four-wave GEMM (gemm_e4m3.hip).

The kernel issues its global->LDS copies from inline-asm statements.  The compiler does not know that such a
statement is a memory instruction that reads scalar registers, so its hazard recognizer does not keep the 5 wait
states the hardware needs between a vector instruction writing a scalar register (v_readlane reloading a spilled
scalar, v_readfirstlane, a v_cmp writing a lane mask) and a memory instruction reading it, nor is it asked to keep
the one wait state between a write of M0 and the copy that takes its LDS destination from M0.  The kernel is written
so that neither happens (no scalar of the copy stream is spilled; a matrix instruction or an LDS read sits between
the write of M0 and the copy).  A stale scalar means a wrong address: wrong data or a memory fault.  This module
scans the assembly text for both distances at every copy; the library build runs it and fails on a violation, and
tests/test_asm_hazards.py runs it on its own."""
import os
import re
import subprocess

_VECTOR_SCALAR_WRITERS = ("v_readlane", "v_readfirstlane", "v_cmp")


def instructions(body):
    out = []
    for line in body.split("\n"):
        l = line.split(";")[0].strip()
        if l and not l.startswith(".") and not l.endswith(":"):
            out.append(l)
    return out


def scalar_destinations(ins):
    """Names of the scalar registers the first operand of `ins` denotes: 's7', 's[10:11]' -> s10, s11, 'vcc' (and its
    halves), 'm0'.  The e32 form of v_cmp has no explicit destination and writes vcc."""
    parts = ins.split(None, 1)
    if len(parts) < 2:
        return set()
    mnemonic, first = parts[0], parts[1].split(",")[0].strip()
    m = re.fullmatch(r"s\[(\d+):(\d+)\]", first)
    if m:
        return {"s%d" % r for r in range(int(m.group(1)), int(m.group(2)) + 1)}
    if re.fullmatch(r"s\d+", first) or first == "m0":
        return {first}
    if first in ("vcc", "vcc_lo", "vcc_hi"):
        return {"vcc", "vcc_lo", "vcc_hi"}
    if mnemonic.startswith("v_cmp") and "_e64" not in mnemonic and not first.startswith("s"):
        return {"vcc", "vcc_lo", "vcc_hi"}
    return set()


def copy_scalar_sources(ins):
    m = re.search(r"s\[(\d+):(\d+)\]", ins)
    regs = {"m0"}
    if m:
        regs |= {"s%d" % r for r in range(int(m.group(1)), int(m.group(2)) + 1)}
    if "vcc" in ins:
        regs |= {"vcc", "vcc_lo", "vcc_hi"}
    return regs


def check_text(text, min_kernels=10, min_copies=1000):
    """Raises AssertionError naming the kernel and the instruction pair on a violation; returns (kernels, copies)."""
    kernels = re.findall(r"^(_Z\S*w4_kernel\S*):[^\n]*\n(.*?)\.end_amdhsa_kernel", text, re.S | re.M)
    assert len(kernels) >= min_kernels, "only %d four-wave kernel instances found in the assembly" % len(kernels)
    copies = 0
    for name, body in kernels:
        ins = instructions(body)
        for i, l in enumerate(ins):
            if not l.startswith("global_load_lds"):
                continue
            copies += 1
            regs = copy_scalar_sources(l)
            assert i > 0 and not re.match(r"s_\w+\s+m0,", ins[i - 1]), "%s: M0 written right in front of '%s'" % (name, l)
            wait, j = 0, i - 1
            while j >= 0 and wait < 5:
                p = ins[j]
                if p.startswith("s_nop"):
                    wait += int(p.split()[1]) + 1
                else:
                    if p.startswith(_VECTOR_SCALAR_WRITERS):
                        hit = scalar_destinations(p) & regs
                        assert not hit, "%s: '%s' writes %s only %d wait states before '%s'" % (
                            name, p, sorted(hit), wait, l)
                    wait += 1
                j -= 1
    assert copies >= min_copies, "only %d global->LDS copies found in the assembly" % copies
    return len(kernels), copies


def compile_to_assembly(hipcc, flags, source, out_path, extra=()):
    cmd = [hipcc] + [f for f in flags if not f.startswith("-W")] + list(extra) + ["--cuda-device-only", "-S", source, "-o", out_path]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc -S failed for %s:\n%s" % (source, r.stderr[-4000:]))
    return out_path


def check_source(hipcc, flags, source, out_path, extra=()):
    compile_to_assembly(hipcc, flags, source, out_path, extra)
    with open(out_path) as f:
        text = f.read()
    try:
        return check_text(text)
    finally:
        if os.path.exists(out_path):
            os.remove(out_path)
