"""Helpers shared by the GPU parity tests: host<->device moves of raw bit patterns and the GEMM
tolerance of the path (stated once, here)."""
import contextlib
import os

import numpy as np
import torch


@contextlib.contextmanager
def gemm_library(lib):
    """Runs llmq_amd.kernels on `lib` instead of the product library for the duration of the block (None: no change).
    The parity tests pass the test-aid build of the GEMM entry points (capi.testaid()), whose kernel selection can be
    forced; the product wrapper itself has no such switch."""
    from llmq_amd import capi
    if lib is None:
        yield
        return
    saved = capi.lib
    capi.lib = lib
    try:
        yield
    finally:
        capi.lib = saved


def dev_bf16(bits):
    """uint16 bf16 patterns (numpy) -> bf16 device tensor with the same bits."""
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16).cuda()


def dev_u8(codes):
    return torch.from_numpy(np.ascontiguousarray(codes, dtype=np.uint8)).cuda()


def host_bits(t):
    """device tensor -> numpy array of raw patterns (uint16 for bf16, uint8 for fp8/uint8, fp32 as is)."""
    t = t.detach().cpu()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        return t.view(torch.uint8).numpy()
    return t.numpy()


def dev_scalar(v):
    return torch.tensor([v], dtype=torch.float32, device="cuda")


# GEMM tolerance versus the exact (fp64) product of the same e4m3 operands times the fp32 factor sa*sb:
#   bf16 output:  |err| <= 2^-8 * |ref| + 2^-11 * (sa*sb) * sum_k |a_k b_k|     and rel-Frobenius <= 2.5e-3
#   fp32 output:  |err| <= 2^-11 * (sa*sb) * sum_k |a_k b_k|                    and rel-Frobenius <= 1e-4
# 2^-8 is half a bf16 ulp of the result.  The second term is the accumulation error of the gfx950 FP8
# matrix instruction itself, measured with one-hot probes on the device: inside each group of 8
# consecutive K positions the products are aligned to the group's largest product and truncated
# (towards zero) 14 bits below its leading bit, so a group loses less than 7 * 2^-14 of its largest
# term; summed over groups that is below 7 * 2^-14 * sum|a b| < 2^-11 * sum|a b|.  (Across groups and
# into the fp32 accumulator the window is 27 bits, negligible next to it.)  Integer-valued operands
# with |product| < 2^14 are unaffected, which is why the known-answer tests are bit exact.
# tests/test_gpu_mfma_model.py pins that behaviour with the same probes.  The Frobenius limits are at most twice
# what was measured: fp32 output 4.8e-5 on uniformly random codes (the worst magnitudes; 1.5e-5 on quantized
# Gaussian data), bf16 output 1.7e-3 (the output rounding itself, 2^-9 / sqrt(3) = 1.1e-3 for a flat mantissa).
ACC_TERM = 2.0 ** -11


def gemm_check(got_f32, exact, sumabs, scale, out_is_bf16, extra=None):
    """got_f32: decoded device result; exact/sumabs: oracle fp64 arrays of the same shape; extra: fp64
    array added after scaling (bias + old c).  Returns (max_abs_err, rel_frobenius); asserts the bounds."""
    ref = exact * float(scale)
    if extra is not None:
        ref = ref + extra
    err = np.abs(got_f32.astype(np.float64) - ref)
    mag = np.abs(float(scale)) * sumabs + (np.abs(extra) if extra is not None else 0.0)
    if out_is_bf16:
        bound = 2.0 ** -8 * np.abs(ref) + ACC_TERM * mag + 1e-38
        fro_lim = 2.5e-3
    else:
        bound = ACC_TERM * mag + 1e-38
        fro_lim = 1e-4
    worst = float((err / bound).max())
    assert worst <= 1.0, "GEMM element error exceeds the stated bound by x%.3f" % worst
    fro = float(np.sqrt((err ** 2).sum()) / max(np.sqrt((ref ** 2).sum()), 1e-300))
    assert fro <= fro_lim, "relative Frobenius error %.3e > %.1e" % (fro, fro_lim)
    return float(err.max()), fro


def report_gemm_error(config, name, N, M, K, max_abs, fro, sampled):
    """Appends one line per checked GEMM to the file named by LLMQ_GEMM_ERROR_REPORT (unset: nothing is
    written): the per-shape max-abs / relative-Frobenius figures of BASELINE.json's configurations."""
    path = os.environ.get("LLMQ_GEMM_ERROR_REPORT")
    if path:
        with open(path, "a") as f:
            f.write("%-8s %-28s c[%5d x %5d] K=%5d  max_abs %.3e  rel_frobenius %.3e  (%s)\n" % (
                config, name, N, M, K, max_abs, fro, sampled))
