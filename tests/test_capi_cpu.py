"""CPU-side checks of the C-ABI library: it loads, exports every symbol include/llmq_fp8.h declares,
and rejects bad arguments with the documented codes before touching the GPU."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def capi():
    from llmq_amd import capi
    return capi


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "llmq_fp8.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(llmq_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(capi):
    names = declared_symbols()
    assert len(names) >= 11
    for n in names:
        assert hasattr(capi.lib, n), n
    assert sorted(capi.EXPORTS) == names


def test_product_library_exports_exactly_the_header(capi):
    """The dynamic symbol table of libllmq_fp8.so is the set of functions include/llmq_fp8.h declares: no tuning
    knobs, no measurement aids, no C++ internals (those live in the test-aid library, see llmq_amd/build.py)."""
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", capi.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if line.strip())
    assert exported == declared_symbols()
    out = subprocess.run(["nm", "-D", "--defined-only", capi.TESTAID_PATH], capture_output=True, text=True, check=True).stdout
    aid = {line.split()[-1] for line in out.splitlines() if line.strip()}
    assert {"llmq_debug_set_gemm_variant", "llmq_debug_set_gemm_persist", "llmq_debug_copy_u8",
            "llmq_debug_mfma_ceiling"} <= aid


def test_version_and_arch(capi):
    assert capi.target_arch() == "gfx950"
    assert capi.version()


def test_invalid_arguments_are_rejected_without_a_gpu(capi):
    L = capi.lib
    buf = (C.c_char * 4096)()
    p = (C.addressof(buf) + 15) & ~15
    INV = capi.LLMQ_ERR_INVALID_ARGUMENT
    assert L.llmq_abs_max_bf16(None, p, 8, None) == INV
    assert L.llmq_abs_max_bf16(p, p, -8, None) == INV
    assert L.llmq_abs_max_bf16(p, p + 2, 8, None) == INV                     # misaligned input
    assert L.llmq_quantize_e4m3_bf16(p, None, p, None, 8, None) == INV       # null abs-max
    assert L.llmq_quantize_e4m3_bf16(p + 1, None, p, p, 8, None) == INV      # misaligned output
    assert L.llmq_quantize_transpose_e4m3_bf16(p, None, p, p, 12, 16, None) == INV   # rows % 8
    assert L.llmq_quantize_transpose_e4m3_bf16(p, None, p, p, 16, 20, None) == INV   # cols % 8
    assert L.llmq_transpose_u8(p, p, 16, 16, None) == INV                    # in place
    assert L.llmq_transpose_u8(None, p, 16, 16, None) == INV
    assert L.llmq_transpose_u8(p, p, 0, 16, None) == capi.LLMQ_OK            # empty: nothing to do
    # GEMM: rows of the fp8 operands must be 16-byte aligned (src/kernels/matmul.cpp:55-57), i.e. K % 16 == 0;
    # M and N are free
    assert L.llmq_gemm_tn_e4m3_bf16(p, p, p, None, None, None, None, 0, 128, 128, 72, 0, None) == INV
    assert b"multiple of 16" in L.llmq_last_error()
    assert L.llmq_gemm_tn_e4m3_bf16(p, p, p, None, None, None, None, 0, 0, 128, 128, 0, None) == INV
    assert L.llmq_gemm_tn_e4m3_bf16(p, None, p, None, None, None, None, 0, 128, 128, 128, 0, None) == INV
    assert L.llmq_gemm_tn_e4m3_bf16(p, p + 8, p, None, None, None, None, 0, 128, 128, 128, 0, None) == INV
    assert b"aligned" in L.llmq_last_error()
    assert L.llmq_gemm_tn_e4m3_f32(p, p, p, None, 0, None, None, None, 0, 0, 128, 128, 0, None) == INV
    assert L.llmq_gemm_tn_e4m3_bf16(p, p, p, None, None, None, None, 4096, 128, 128, 128, 0, None) == INV
    assert b"workspace" in L.llmq_last_error()
    assert L.llmq_gemm_tn_e4m3_bf16(p, p, p, None, None, None, p + 4, 4096, 128, 128, 128, 0, None) == INV
    # backward_bias: both-or-neither scales, vector-size rule, scratch size (bias.cu:163-168, kernels.cpp:378-380)
    assert L.llmq_backward_bias_bf16(p, p, 0, p, None, p, 1 << 20, 8, 64, None) == INV
    assert L.llmq_backward_bias_bf16(p, p, 0, None, None, p, 1 << 20, 8, 24, None) == INV
    assert L.llmq_backward_bias_bf16(p, p, 0, None, None, p, 4, 8, 64, None) == INV
    assert b"scratch buffer too small" in L.llmq_last_error()
    assert L.llmq_backward_bias_bf16(p, p, 7, None, None, p, 1 << 20, 8, 64, None) == INV
    assert L.llmq_backward_bias_scratch_bytes(8192, 1152, 0) >= 1152 * 4
    # the variant with built-in scratch refuses what its array cannot hold, before any GPU call
    assert L.llmq_backward_bias_bf16_static_scratch(p, p, 0, None, None, 64, 5 << 20, None) == INV
    assert b"built-in scratch" in L.llmq_last_error()
    with pytest.raises(ValueError):
        capi.check(INV)
    with pytest.raises(RuntimeError):
        capi.check(capi.LLMQ_ERR_RUNTIME)


def test_producer_entry_points_reject_bad_arguments_without_a_gpu(capi):
    """Shape rules of the producers (src/kernels/swiglu.cu:306-318, rope.cu:137, adamw.cu:150) are checked before
    anything is launched."""
    L = capi.lib
    buf = (C.c_char * 4096)()
    p = (C.addressof(buf) + 15) & ~15
    INV = capi.LLMQ_ERR_INVALID_ARGUMENT
    f = C.c_float
    assert L.llmq_swiglu_forward_bf16(p, p, None, 1, 4, 12, None) == INV and b"divisible by 8" in L.llmq_last_error()
    assert L.llmq_swiglu_forward_bf16(p, p, None, 1 << 15, 1 << 15, 8, None) == INV and b"too large" in L.llmq_last_error()
    assert L.llmq_swiglu_forward_quant_bf16(p, None, p, None, 1, 4, 16, None) == INV
    assert L.llmq_swiglu_backward_bf16(p, p, p, None, 1, 4, 20, None) == INV
    assert L.llmq_rmsnorm_forward_bf16(p, None, p, p, None, f(1e-6), 1, 4, 12, None) == INV
    assert L.llmq_rmsnorm_forward_bf16(p, None, p, p, None, f(1e-6), 1, 4, 16392, None) == INV and b"16384" in L.llmq_last_error()
    assert L.llmq_fused_residual_rmsnorm_forward_bf16(None, p, p, p, p, p, None, f(1e-6), 4, 16, None) == INV
    assert L.llmq_rmsnorm_backward_bf16(p, p, p, 16, p, p, p, p, p, None, 1, 4, 64, None) == INV and b"scratch" in L.llmq_last_error()
    assert L.llmq_rmsnorm_backward_scratch_bytes(3584) >= 3584 * 4 and L.llmq_rmsnorm_backward_scratch_bytes(0) == 0
    assert L.llmq_rope_forward_bf16(p, p, p, None, 1, 4, 2, 1, 12, None) == INV and b"head_dim" in L.llmq_last_error()
    assert L.llmq_rope_backward_bf16(p, p + 2, p, None, 1, 4, 2, 1, 16, None) == INV
    assert L.llmq_adamw_update_bf16(p, p, p, 0, p, 0, 12, f(1e-3), f(0.9), f(0.99), 1, f(1e-8), f(0.0), p, None, 1, None) == INV
    assert L.llmq_adamw_update_bf16(p, p, p, 0, p, 1, 16, f(1e-3), f(0.9), f(0.99), 1, f(1e-8), f(0.0), p, None, 1, None) == INV
    assert b"moment types" in L.llmq_last_error()
    assert L.llmq_adamw_update_bf16(p, p, p, 0, p, 0, 16, f(1e-3), f(0.9), f(0.99), 1, f(1e-8), f(0.0), None, None, 1, None) == INV


def test_precompute_freqs_cis_on_the_host(capi):
    """The rope table is host code (src/kernels/rope.cu:15-40): cos / sin of t / theta^(2i/dim) in fp16."""
    import numpy as np
    dim, end, theta = 16, 9, 10000.0
    tab = np.zeros((end, dim), dtype=np.float16)
    assert capi.lib.llmq_precompute_freqs_cis_f16(tab.ctypes.data, dim, end, C.c_float(theta)) == capi.LLMQ_OK
    ang = np.arange(end)[:, None] / theta ** (2 * np.arange(dim // 2) / dim)[None, :]
    assert np.allclose(tab[:, 0::2], np.cos(ang), atol=2.0 ** -10) and np.allclose(tab[:, 1::2], np.sin(ang), atol=2.0 ** -10)
    assert capi.lib.llmq_precompute_freqs_cis_f16(tab.ctypes.data, 15, end, C.c_float(theta)) == capi.LLMQ_ERR_INVALID_ARGUMENT


def test_reference_python_ops_register_without_a_gpu():
    """llmq_amd.ops registers the reference's operator names (src/binding/python/kernels.py:118-165) at import."""
    import torch
    from llmq_amd import ops
    for name in ("abs_max", "quantize_with_abs_max", "quantize_and_transpose_with_abs_max", "transpose", "matmul",
                 "backward_bias", "swiglu_forward", "swiglu_forward_quant", "swiglu_backward", "rmsnorm_forward",
                 "fused_residual_rmsnorm_forward", "rmsnorm_backward", "rope_forward", "rope_backward", "adamw_update"):
        assert hasattr(torch.ops.llmq, name)
    assert ops.MODE_NT == 2 and ops.create_cublas_handle() == 0
    with pytest.raises(ValueError):                      # host tensors are rejected before any launch
        ops.abs_max(torch.zeros(1), torch.zeros(8, dtype=torch.bfloat16))


def test_stored_layout_plan_and_stack_of_backward_qmm():
    """Host logic of the C++ glue (tests/cpp/plan_check.cpp): which backward matmuls read their operands where
    they lie (QmmRunState::direct_layout_plan) on layers of the Qwen2.5 sizes, and the stack backward_qmm then needs."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "build", "plan_check")
    assert os.path.exists(exe), "build it with `make -C tests/cpp` (done by __graft_entry__.build())"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    print(r.stdout[-2000:], r.stderr[-1000:])
    assert r.returncode == 0 and "RESULT: PASS" in r.stdout
