"""The reference's Python-visible contract for the path (src/binding/python/kernels.py:118-165): the same
operator names and signatures, called through torch.ops.llmq.* and through the module functions, on the
constructions of the reference's scripts/test_kernels.py (abs-max :40-65, quantize :641-652, 1168-1185,
matmul :937-1040 restricted to what FP8 supports, backward_bias :834-890)."""
import numpy as np
import pytest
import torch

from gpu_util import gemm_check

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def P():
    from llmq_amd import ops
    return ops


def test_ops_are_registered_with_reference_names(P):
    for name in ("abs_max", "quantize_with_abs_max", "quantize_and_transpose_with_abs_max", "transpose", "matmul",
                 "backward_bias"):
        assert hasattr(torch.ops.llmq, name)


def test_abs_max_and_quantize_through_ops(P, O):
    torch.manual_seed(0)
    x = torch.randn(1000 * 64, device="cuda", dtype=torch.bfloat16) * 3
    scale = torch.zeros(1, device="cuda")
    torch.ops.llmq.abs_max(scale, x)
    assert scale.item() == x.float().abs().max().item()                      # exact, as test_kernels.py:56-65
    q = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device="cuda")
    dq = torch.zeros(1, device="cuda")
    P.quantize_with_abs_max(q, dq, x, scale)
    assert dq.item() == pytest.approx(scale.item() / 448.0, rel=1e-6)        # test_kernels.py:223-241
    back = q.float() * dq
    assert torch.allclose(back, x.float(), rtol=0.1, atol=0.1 * scale.item() / 448 * 8)   # loose dequant check :641-652
    x2 = x.view(1000, 64)
    qt = torch.empty((64, 1000), dtype=torch.float8_e4m3fn, device="cuda")
    P.quantize_and_transpose_with_abs_max(qt, dq, x2, scale)
    assert torch.equal(qt.view(torch.uint8), q.view(1000, 64).view(torch.uint8).T)
    t2 = torch.empty((1000, 64), dtype=torch.float8_e4m3fn, device="cuda")
    P.transpose(t2, qt)
    assert torch.equal(t2.view(torch.uint8), q.view(1000, 64).view(torch.uint8))


def test_matmul_torch_convention(P, O):
    """c[M,N] = (a[M,K] @ b[N,K]^T) * scale_a * scale_b + bias[N] (+ c), mode NT."""
    M, N, Kd = 384, 256, 512
    rng = np.random.default_rng(4)
    a = rng.integers(0, 0x7E, (M, Kd)).astype(np.uint8)
    b = (rng.integers(0, 0x7E, (N, Kd)).astype(np.uint8) | 0x80)
    ad = torch.from_numpy(a).cuda().view(torch.float8_e4m3fn)
    bd = torch.from_numpy(b).cuda().view(torch.float8_e4m3fn)
    sa, sb = torch.tensor([0.03], device="cuda"), torch.tensor([0.5], device="cuda")
    bias = torch.randn(N, device="cuda", dtype=torch.bfloat16)
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    handle = P.create_cublas_handle()
    c = torch.randn(M, N, device="cuda", dtype=torch.bfloat16)
    old = c.clone()
    P.matmul(c, ad, bd, bias, sa, sb, handle, ws, P.MODE_NT, True)
    P.destroy_cublas_handle(handle)
    exact, sumabs = O.gemm_exact(b, a)            # oracle convention: rows of the first operand index the columns of c
    scale = np.float32(np.float32(0.03) * np.float32(0.5))
    extra = bias.float().cpu().numpy().astype(np.float64)[None, :] + old.float().cpu().numpy().astype(np.float64)
    gemm_check(c.float().cpu().numpy(), exact, sumabs, scale, True, extra=extra)
    with pytest.raises(ValueError):
        P.matmul(c, ad, bd, None, None, None, 0, ws, P.MODE_NN, False)       # mode NN wants b as [K, N]: shapes do not match
    with pytest.raises(ValueError):
        P.matmul(c, ad, bd[:, :256].contiguous(), None, None, None, 0, ws, P.MODE_NT, False)


def test_matmul_mode_tt_reads_the_first_operand_in_k_major_storage(P, O):
    """Mode TT in the torch sense: c[M,N] = a[K,M]^T @ b[N,K]^T.  The same codes handed over as a[M,K] in mode NT
    give the same result to the tolerance, and both are checked against the exact product."""
    M, N, Kd = 512, 256, 768
    rng = np.random.default_rng(14)
    a = rng.integers(0, 0x7E, (M, Kd)).astype(np.uint8) | (rng.integers(0, 2, (M, Kd)).astype(np.uint8) << 7)
    b = rng.integers(0, 0x7E, (N, Kd)).astype(np.uint8)
    ad = torch.from_numpy(a).cuda().view(torch.float8_e4m3fn)
    at = torch.from_numpy(np.ascontiguousarray(a.T)).cuda().view(torch.float8_e4m3fn)      # [K, M]
    bd = torch.from_numpy(b).cuda().view(torch.float8_e4m3fn)
    sa, sb = torch.tensor([0.25], device="cuda"), torch.tensor([0.125], device="cuda")
    bias = torch.randn(N, device="cuda", dtype=torch.bfloat16)
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    c = torch.full((M, N), float("nan"), device="cuda", dtype=torch.bfloat16)
    P.matmul(c, at, bd, bias, sa, sb, 0, ws, P.MODE_TT, False)
    exact, sumabs = O.gemm_exact(b, a)
    extra = bias.float().cpu().numpy().astype(np.float64)[None, :]
    gemm_check(c.float().cpu().numpy(), exact, sumabs, np.float32(0.25 * 0.125), True, extra=extra)
    c32 = torch.full((M, N), float("nan"), device="cuda")                      # fp32 output in the same mode, accumulating
    c32.copy_(extra_old := torch.randn((M, N), device="cuda"))
    P.matmul(c32, at, bd, bias, sa, sb, 0, ws, P.MODE_TT, True)
    gemm_check(c32.cpu().numpy(), exact, sumabs, np.float32(0.25 * 0.125), False,
               extra=extra + extra_old.cpu().numpy().astype(np.float64))
    with pytest.raises(ValueError):                                            # a is [K, M]: handing over [M, K] mismatches c
        P.matmul(c, ad, bd, None, None, None, 0, ws, P.MODE_TT, False)


@pytest.mark.parametrize("mode", ["NN", "TN"])
def test_matmul_modes_with_b_in_k_major_storage(P, O, mode):
    """Torch-sense modes NN (c = a @ b, b stored [K, N]) and TN (c = a^T @ b, a stored [K, M] as well): the kernel layer's
    modes NN and NT after the operand swap of the binding (src/binding/kernel_binding.cpp:403-431)."""
    M, N, Kd = 512, 256, 768
    rng = np.random.default_rng(15)
    a = rng.integers(0, 0x7E, (M, Kd)).astype(np.uint8) | (rng.integers(0, 2, (M, Kd)).astype(np.uint8) << 7)
    b = rng.integers(0, 0x7E, (N, Kd)).astype(np.uint8)
    dev = lambda x: torch.from_numpy(np.ascontiguousarray(x)).cuda().view(torch.float8_e4m3fn)
    ad = dev(a) if mode == "NN" else dev(a.T)            # [M, K] or [K, M]
    bd = dev(b.T)                                        # [K, N]
    sa, sb = torch.tensor([0.25], device="cuda"), torch.tensor([0.125], device="cuda")
    bias = torch.randn(N, device="cuda", dtype=torch.bfloat16)
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    c = torch.full((M, N), float("nan"), device="cuda", dtype=torch.bfloat16)
    P.matmul(c, ad, bd, bias, sa, sb, 0, ws, P.MODE_NN if mode == "NN" else P.MODE_TN, False)
    exact, sumabs = O.gemm_exact(b, a)
    extra = bias.float().cpu().numpy().astype(np.float64)[None, :]
    gemm_check(c.float().cpu().numpy(), exact, sumabs, np.float32(0.25 * 0.125), True, extra=extra)
    old = c.clone()                                      # the same modes accumulating into c
    P.matmul(c, ad, bd, None, sa, sb, 0, ws, P.MODE_NN if mode == "NN" else P.MODE_TN, True)
    gemm_check(c.float().cpu().numpy(), exact, sumabs, np.float32(0.25 * 0.125), True, extra=old.float().cpu().numpy().astype(np.float64))


def test_backward_bias_through_ops(P):
    torch.manual_seed(0)
    B, T, OC = 8, 16, 512                                                    # test_kernels.py:837-853
    dout = torch.randn((B, T, OC), device="cuda", dtype=torch.bfloat16)
    initial = torch.randn((OC,), device="cuda", dtype=torch.bfloat16)
    dbias = initial.clone()
    buf = torch.empty(P.get_bias_backward_scratch_size(torch.bfloat16, OC) // 4, device="cuda", dtype=torch.float32)
    torch.ops.llmq.backward_bias(dbias, dout, None, None, buf)
    ref = (initial.float() + dout.float().sum(dim=(0, 1))).to(torch.bfloat16)
    assert torch.allclose(dbias.float(), ref.float(), rtol=1e-2, atol=1e-2)
