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
    # GEMM: the 128-divisibility rule of the reference's custom kernel (gemm_mma.cu:261-263)
    assert L.llmq_gemm_tn_e4m3_bf16(p, p, p, None, None, None, None, 0, 128, 128, 64, 0, None) == INV
    assert b"divisible by 128" in L.llmq_last_error()
    assert L.llmq_gemm_tn_e4m3_bf16(p, p, p, None, None, None, None, 0, 100, 128, 128, 0, None) == INV
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
    with pytest.raises(ValueError):
        capi.check(INV)
    with pytest.raises(RuntimeError):
        capi.check(capi.LLMQ_ERR_RUNTIME)


def test_reference_python_ops_register_without_a_gpu():
    """llmq_amd.ops registers the reference's operator names (src/binding/python/kernels.py:118-165) at import."""
    import torch
    from llmq_amd import ops
    for name in ("abs_max", "quantize_with_abs_max", "quantize_and_transpose_with_abs_max", "transpose", "matmul",
                 "backward_bias"):
        assert hasattr(torch.ops.llmq, name)
    assert ops.MODE_NT == 2 and ops.create_cublas_handle() == 0
    with pytest.raises(ValueError):                      # host tensors are rejected before any launch
        ops.abs_max(torch.zeros(1), torch.zeros(8, dtype=torch.bfloat16))
