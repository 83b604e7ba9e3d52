"""The hazard scan of the four-wave GEMM's generated code (llmq_amd/asm_check.py), run on its own: the scanner's
parsing on hand-written snippets, and the scan of the product source compiled to assembly (the library build runs
the same scan and refuses to link on a violation)."""
import os

import pytest

from llmq_amd import asm_check


def _kernel(body):
    return "_Z4demow4_kernelv:\n" + body + "\n.end_amdhsa_kernel\n"


def test_scanner_parses_scalar_destinations():
    d = asm_check.scalar_destinations
    assert d("v_readlane_b32 s10, v3, 0") == {"s10"}
    assert d("v_readfirstlane_b32 s7, v1") == {"s7"}
    assert d("v_cmp_lt_u32_e64 s[10:11], v1, v2") == {"s10", "s11"}
    assert "vcc" in d("v_cmp_eq_u32_e32 vcc, v1, v2")
    assert "vcc" in d("v_cmp_eq_u32 v1, v2")
    assert d("v_add_u32 v1, v2, v3") == set()


def test_scanner_flags_each_hazard():
    filler = "\n".join("v_mov_b32 v1, v2" for _ in range(6))
    ok = _kernel("s_add_i32 m0, s3, 16\nv_mov_b32 v1, v2\n" + filler + "\nglobal_load_lds_dwordx4 v5, s[10:11]")
    asm_check.check_text(ok, min_kernels=1, min_copies=1)
    with pytest.raises(AssertionError, match="M0 written right in front"):
        asm_check.check_text(_kernel(filler + "\ns_add_i32 m0, s3, 16\nglobal_load_lds_dwordx4 v5, s[10:11]"), 1, 1)
    with pytest.raises(AssertionError, match="wait states"):
        asm_check.check_text(_kernel(filler + "\nv_readlane_b32 s11, v9, 3\nv_mov_b32 v1, v2\nglobal_load_lds_dwordx4 v5, s[10:11]"), 1, 1)
    with pytest.raises(AssertionError, match="wait states"):   # a lane mask written as a register pair
        asm_check.check_text(_kernel(filler + "\nv_cmp_lt_u32_e64 s[10:11], v1, v2\nv_mov_b32 v1, v2\nglobal_load_lds_dwordx4 v5, s[10:11]"), 1, 1)
    # five wait states (an s_nop counts its argument + 1) are enough
    asm_check.check_text(_kernel(filler + "\nv_readlane_b32 s11, v9, 3\ns_nop 4\nglobal_load_lds_dwordx4 v5, s[10:11]"), 1, 1)


def test_lds_copies_keep_their_distance_from_scalar_writes(tmp_path):
    from llmq_amd import build as B
    kernels, copies = asm_check.check_source(B.HIPCC, B.FLAGS, os.path.join(B.CSRC, "gemm_e4m3.hip"), str(tmp_path / "gemm.s"))
    assert kernels >= 10 and copies >= 1000
