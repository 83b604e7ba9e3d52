"""ctypes binding of the C ABI declared in include/llmq_fp8.h.

Raw device pointers in, status codes turned into exceptions: LLMQ_ERR_INVALID_ARGUMENT -> ValueError
(the reference throws std::invalid_argument), LLMQ_ERR_RUNTIME -> RuntimeError.  There is no CPU
fallback: if the library is not built the import of this module fails.
"""
import ctypes as C
import os

# torch bundles its own HIP runtime (same SONAME as /opt/rocm's, requested under a different file
# name): whichever copy is loaded first must serve the whole process, so torch goes first.
import torch  # noqa: F401

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libllmq_fp8.so")

EXPORTS = [
    "llmq_last_error", "llmq_version", "llmq_target_arch",
    "llmq_abs_max_bf16", "llmq_abs_max_f32",
    "llmq_quantize_e4m3_bf16", "llmq_quantize_e5m2_bf16", "llmq_quantize_transpose_e4m3_bf16", "llmq_quantize_transpose_e4m3_f32",
    "llmq_transpose_u8", "llmq_gemm_tn_e4m3_bf16", "llmq_gemm_e4m3_bf16_mode", "llmq_gemm_e4m3_f32_mode", "llmq_gemm_tn_e4m3_f32", "llmq_gemm_tn_e4m3_e5m2_bf16", "llmq_gemm_tn_e4m3_e5m2_f32",
    "llmq_backward_bias_bf16", "llmq_backward_bias_scratch_bytes", "llmq_backward_bias_bf16_static_scratch", "llmq_quantize_both_bf16", "llmq_quantize_e4m3_f32", "llmq_quantize_e5m2_f32",
    "llmq_swiglu_forward_bf16", "llmq_swiglu_forward_quant_bf16", "llmq_swiglu_backward_bf16",
    "llmq_rmsnorm_forward_bf16", "llmq_fused_residual_rmsnorm_forward_bf16",
    "llmq_rmsnorm_backward_bf16", "llmq_rmsnorm_backward_scratch_bytes",
    "llmq_rope_forward_bf16", "llmq_rope_backward_bf16", "llmq_precompute_freqs_cis_f16",
    "llmq_adamw_update_bf16", "llmq_adamw_update_bf16_fp8m",
    "llmq_swiglu_forward_f32", "llmq_swiglu_backward_f32", "llmq_rope_forward_f32", "llmq_rope_backward_f32",
    "llmq_precompute_freqs_cis_f32", "llmq_rmsnorm_forward_f32", "llmq_fused_residual_rmsnorm_forward_f32",
    "llmq_rmsnorm_backward_f32", "llmq_adamw_update_f32",
]

if not os.path.exists(LIB_PATH):
    raise ImportError("%s is missing: build it with `python -m llmq_amd.build` (hipcc, gfx950)" % LIB_PATH)

lib = C.CDLL(LIB_PATH)

_vp, _i64, _int = C.c_void_p, C.c_int64, C.c_int
lib.llmq_last_error.restype = C.c_char_p
lib.llmq_version.restype = C.c_char_p
lib.llmq_target_arch.restype = C.c_char_p
lib.llmq_abs_max_bf16.argtypes = [_vp, _vp, _i64, _vp]
lib.llmq_abs_max_f32.argtypes = [_vp, _vp, _i64, _vp]
lib.llmq_quantize_e4m3_bf16.argtypes = [_vp, _vp, _vp, _vp, _i64, _vp]
lib.llmq_quantize_e5m2_bf16.argtypes = [_vp, _vp, _vp, _vp, _i64, _vp]
lib.llmq_quantize_transpose_e4m3_bf16.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _vp]
lib.llmq_quantize_transpose_e4m3_f32.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _vp]
lib.llmq_quantize_e4m3_f32.argtypes = [_vp, _vp, _vp, _vp, _i64, _vp]
lib.llmq_quantize_e5m2_f32.argtypes = [_vp, _vp, _vp, _vp, _i64, _vp]
lib.llmq_quantize_both_bf16.argtypes = [_vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp]
lib.llmq_transpose_u8.argtypes = [_vp, _vp, _int, _int, _vp]
lib.llmq_gemm_tn_e4m3_bf16.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, C.c_size_t, _int, _int, _int, _int, _vp]
lib.llmq_gemm_e4m3_bf16_mode.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, C.c_size_t, _int, _int, _int, _int, _int, _int, _vp]
lib.llmq_gemm_e4m3_f32_mode.argtypes = [_vp, _vp, _vp, _vp, _int, _vp, _vp, _vp, C.c_size_t, _int, _int, _int, _int, _int, _int, _vp]
lib.llmq_gemm_tn_e4m3_f32.argtypes = [_vp, _vp, _vp, _vp, _int, _vp, _vp, _vp, C.c_size_t, _int, _int, _int, _int, _vp]
lib.llmq_gemm_tn_e4m3_e5m2_bf16.argtypes = lib.llmq_gemm_tn_e4m3_bf16.argtypes
lib.llmq_gemm_tn_e4m3_e5m2_f32.argtypes = lib.llmq_gemm_tn_e4m3_f32.argtypes
lib.llmq_backward_bias_bf16.argtypes = [_vp, _vp, _int, _vp, _vp, _vp, C.c_size_t, _int, _int, _vp]
lib.llmq_backward_bias_scratch_bytes.argtypes = [_int, _int, _int]
lib.llmq_backward_bias_bf16_static_scratch.argtypes = [_vp, _vp, _int, _vp, _vp, _int, _int, _vp]
lib.llmq_swiglu_forward_bf16.argtypes = [_vp, _vp, _vp, _int, _int, _int, _vp]
lib.llmq_swiglu_forward_quant_bf16.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _vp]
lib.llmq_swiglu_backward_bf16.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _vp]
lib.llmq_rmsnorm_forward_bf16.argtypes = [_vp, _vp, _vp, _vp, _vp, C.c_float, _int, _int, _int, _vp]
lib.llmq_fused_residual_rmsnorm_forward_bf16.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, C.c_float, _int, _int, _vp]
lib.llmq_rmsnorm_backward_bf16.argtypes = [_vp, _vp, _vp, C.c_size_t, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp]
lib.llmq_rmsnorm_backward_scratch_bytes.argtypes = [_int]
lib.llmq_rope_forward_bf16.argtypes = [_vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _vp]
lib.llmq_rope_backward_bf16.argtypes = lib.llmq_rope_forward_bf16.argtypes
lib.llmq_precompute_freqs_cis_f16.argtypes = [_vp, _int, _int, C.c_float]
lib.llmq_adamw_update_bf16_fp8m.argtypes = [_vp, _vp, _vp, _vp, _vp, _i64, C.c_float, C.c_float, C.c_float, _int, C.c_float,
                                            C.c_float, _vp, _vp, C.c_uint, _vp]
lib.llmq_adamw_update_bf16.argtypes = [_vp, _vp, _vp, _int, _vp, _int, _i64, C.c_float, C.c_float, C.c_float, _int, C.c_float,
                                       C.c_float, _vp, _vp, C.c_uint, _vp]
# the fp32 overloads of the producers take the arguments of their bf16 namesakes
for _name in ("swiglu_forward", "swiglu_backward", "rope_forward", "rope_backward", "rmsnorm_forward",
              "fused_residual_rmsnorm_forward", "rmsnorm_backward"):
    getattr(lib, "llmq_%s_f32" % _name).argtypes = getattr(lib, "llmq_%s_bf16" % _name).argtypes
lib.llmq_precompute_freqs_cis_f32.argtypes = lib.llmq_precompute_freqs_cis_f16.argtypes
lib.llmq_adamw_update_f32.argtypes = [_vp, _vp, _vp, _vp, _i64, C.c_float, C.c_float, C.c_float, _int, C.c_float, C.c_float, _vp,
                                      _vp, C.c_uint, _vp]
for _name in EXPORTS[3:]:
    getattr(lib, _name).restype = _int
lib.llmq_backward_bias_scratch_bytes.restype = _i64
lib.llmq_rmsnorm_backward_scratch_bytes.restype = _i64

LLMQ_OK, LLMQ_ERR_INVALID_ARGUMENT, LLMQ_ERR_RUNTIME = 0, 1, 2

TESTAID_PATH = os.path.join(_HERE, "lib", "libllmq_fp8_testaid.so")
_testaid = None


def testaid():
    """The test-aid library (tests and bench.py only; never needed by a user of the path): the matmul
    entry points from a build of the GEMM file whose kernel selection can be forced
    (llmq_debug_set_gemm_variant / llmq_debug_set_gemm_persist / llmq_debug_set_gemm_fuse), and the measurement aids llmq_debug_copy_u8 and llmq_debug_stream_u8
    (plain copy, read-only and write-only kernels) and llmq_debug_mfma_ceiling (register-only matrix-instruction loop)."""
    global _testaid
    if _testaid is None:
        if not os.path.exists(TESTAID_PATH):
            raise ImportError("%s is missing: build it with `python -m llmq_amd.build`" % TESTAID_PATH)
        t = C.CDLL(TESTAID_PATH)
        t.llmq_last_error.restype = C.c_char_p
        for name in ("llmq_gemm_tn_e4m3_bf16", "llmq_gemm_tn_e4m3_f32", "llmq_gemm_tn_e4m3_e5m2_bf16",
                     "llmq_gemm_tn_e4m3_e5m2_f32", "llmq_gemm_e4m3_bf16_mode", "llmq_gemm_e4m3_f32_mode"):
            getattr(t, name).argtypes = getattr(lib, name).argtypes
            getattr(t, name).restype = _int
        t.llmq_debug_set_gemm_variant.argtypes = [_int, _int]
        t.llmq_debug_set_gemm_variant.restype = None
        t.llmq_debug_set_gemm_persist.argtypes = [_int]
        t.llmq_debug_set_gemm_persist.restype = None
        t.llmq_debug_set_gemm_fuse.argtypes = [_int]
        t.llmq_debug_set_gemm_fuse.restype = None
        t.llmq_debug_copy_u8.argtypes = [_vp, _vp, _i64, _vp]
        t.llmq_debug_copy_u8.restype = _int
        t.llmq_debug_stream_u8.argtypes = [_vp, _vp, _i64, _int, _vp]
        t.llmq_debug_stream_u8.restype = _int
        t.llmq_debug_mfma_ceiling.argtypes = [_vp, _int, _int, _int, _vp]
        t.llmq_debug_mfma_ceiling.restype = _int
        _testaid = t
    return _testaid


def check(code, from_lib=None):
    if code == LLMQ_OK:
        return
    msg = (from_lib or lib).llmq_last_error().decode("utf-8", "replace")
    if code == LLMQ_ERR_INVALID_ARGUMENT:
        raise ValueError(msg)
    raise RuntimeError(msg)


def version():
    return lib.llmq_version().decode()


def target_arch():
    return lib.llmq_target_arch().decode()
