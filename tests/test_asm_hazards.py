"""The four-wave GEMM issues its global->LDS copies from inline-asm statements.  The compiler does not know that
such a statement is a memory instruction that reads scalar registers, so its hazard recognizer does not keep the
5 wait states the hardware needs between a vector instruction writing a scalar register (v_readlane reloading a
spilled scalar, v_readfirstlane) and a memory instruction reading it, nor is it asked to keep the one wait state
between a write of M0 and the copy that takes its LDS destination from M0.  The kernel is written so that neither
happens (no scalar of the copy stream is spilled; a matrix instruction or an LDS read sits between the write of
M0 and the copy); this test compiles the file to assembly and checks both distances for every copy (a stale
scalar means a wrong address: wrong data or a memory fault)."""
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def instructions(body):
    out = []
    for line in body.split("\n"):
        l = line.strip()
        if l and not l.startswith(";") and not l.startswith(".") and not l.endswith(":"):
            out.append(l)
    return out


def test_lds_copies_keep_their_distance_from_scalar_writes(tmp_path):
    from llmq_amd import build as B
    asm = tmp_path / "gemm.s"
    cmd = [B.HIPCC] + [f for f in B.FLAGS if not f.startswith("-W")] + [
        "--cuda-device-only", "-S", os.path.join(B.CSRC, "gemm_e4m3.hip"), "-o", str(asm)]
    subprocess.run(cmd, check=True, capture_output=True)
    text = asm.read_text()
    kernels = re.findall(r"^(_Z\S*w4_kernel\S*):[^\n]*\n(.*?)\.end_amdhsa_kernel", text, re.S | re.M)
    assert len(kernels) >= 10
    copies = 0
    for name, body in kernels:
        ins = instructions(body)
        for i, l in enumerate(ins):
            if not l.startswith("global_load_lds"):
                continue
            copies += 1
            m = re.search(r"s\[(\d+):(\d+)\]", l)
            regs = {"s%d" % r for r in range(int(m.group(1)), int(m.group(2)) + 1)} | {"m0"}
            assert not re.match(r"s_\w+ m0,", ins[i - 1]), "%s: M0 written right in front of '%s'" % (name, l)
            wait, j = 0, i - 1
            while j >= 0 and wait < 5:
                p = ins[j]
                if p.startswith("s_nop"):
                    wait += int(p.split()[1]) + 1
                else:
                    if p.startswith(("v_readlane", "v_readfirstlane", "v_cmp")):
                        assert p.split()[1].rstrip(",") not in regs, "%s: '%s' only %d wait states before '%s'" % (
                            name, p, wait, l)
                    wait += 1
                j -= 1
    assert copies >= 1000
