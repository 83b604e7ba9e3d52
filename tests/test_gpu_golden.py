"""The HIP library (through the C ABI, llmq_amd.kernels) against the committed fixtures of tests/golden/ alone:
no oracle in the loop.  fp8 codes, scales and the integer GEMM case bit for bit; the random GEMM case within
the GEMM tolerance of tests/gpu_util.py; the producers within bf16 rounding of the float64 formula values."""
import os

import numpy as np
import pytest
import torch

from gpu_util import dev_bf16, dev_scalar, dev_u8, gemm_check, host_bits

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ALL_BF16 = np.arange(65536, dtype=np.uint32).astype(np.uint16)
F8 = {"e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from llmq_amd import kernels
    return kernels


def bf16_value(bits):
    return (np.asarray(bits).astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def assert_within(bits, exact, rel, slack=0.0):
    err = np.abs(bf16_value(bits) - exact)
    bound = rel * np.abs(exact) + slack
    assert np.all(err <= bound), float((err - bound).max())


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_quantize_all_bf16_patterns(K, fmt):
    g = load("fp8_encode.npz")
    x = dev_bf16(ALL_BF16)
    for i, absmax in enumerate(g["absmax"]):
        out = torch.zeros(65536, dtype=F8[fmt], device="cuda")
        scale = torch.full((1,), -1.0, dtype=torch.float32, device="cuda")
        K.quantize_with_abs_max(out, scale, x, dev_scalar(float(absmax)))
        got = host_bits(out)
        bad = np.nonzero(got != g[fmt][i])[0]
        assert bad.size == 0, [(hex(int(ALL_BF16[j])), hex(int(got[j])), hex(int(g[fmt][i][j]))) for j in bad[:8]]
        assert scale.cpu().numpy().view(np.uint32)[0] == g["recip_bits"][i]
    # the transposing quantizer and the single-read "plain + transposed" one write the same codes
    absmax = float(g["absmax"][1])
    want = g["e4m3"][1].reshape(256, 256)
    if fmt == "e4m3":
        out_t = torch.zeros((256, 256), dtype=F8[fmt], device="cuda")
        K.quantize_and_transpose_with_abs_max(out_t, None, x.view(256, 256), dev_scalar(absmax))
        assert np.array_equal(host_bits(out_t), want.T)
        o, ot = torch.zeros((256, 256), dtype=F8[fmt], device="cuda"), torch.zeros((256, 256), dtype=F8[fmt], device="cuda")
        K.quantize_with_abs_max_and_transpose(o, ot, None, x.view(256, 256), dev_scalar(absmax))
        assert np.array_equal(host_bits(o), want) and np.array_equal(host_bits(ot), want.T)
        t = torch.zeros((256, 256), dtype=torch.uint8, device="cuda")
        K.transpose(t, dev_u8(want))
        assert np.array_equal(t.cpu().numpy(), want.T)


def test_gemm_integer_known_answer(K):
    g = load("gemm_kat.npz")
    a, b = g["int_a"], g["int_b"]
    (M, Kd), N = a.shape, b.shape[0]
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    qa, qb = dev_u8(a).view(torch.float8_e4m3fn), dev_u8(b).view(torch.float8_e4m3fn)
    bias = dev_bf16(g["int_bias_bf16"])
    sa, sb = dev_scalar(float(g["int_sa"])), dev_scalar(float(g["int_sb"]))
    c16 = torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
    K.matmul(c16, qa, qb, bias, sa, sb, M, N, Kd, workspace=ws)
    assert np.array_equal(host_bits(c16), g["int_c_bf16"])
    c32 = torch.full((N, M), float("nan"), dtype=torch.float32, device="cuda")
    K.matmul(c32, qa, qb, bias, sa, sb, M, N, Kd, workspace=ws)
    assert np.array_equal(c32.cpu().numpy().view(np.uint32), g["int_c_f32"].view(np.uint32))
    # accumulate: c <- c + result, on the halved known answer's complement (all values stay exact)
    c_acc = torch.from_numpy(-g["int_c_f32"]).cuda()
    K.matmul(c_acc, qa, qb, bias, sa, sb, M, N, Kd, accumulate=True, workspace=ws)
    assert torch.count_nonzero(c_acc).item() == 0


def test_gemm_random_codes(K):
    g = load("gemm_kat.npz")
    a, b = g["rnd_a"], g["rnd_b"]
    (M, Kd), N = a.shape, b.shape[0]
    qa, qb = dev_u8(a).view(torch.float8_e4m3fn), dev_u8(b).view(torch.float8_e4m3fn)
    sa, sb = np.float32(g["rnd_sa"]), np.float32(g["rnd_sb"])
    scale = np.float32(sa * sb)
    for dt in (torch.bfloat16, torch.float32):
        c = torch.full((N, M), float("nan"), dtype=dt, device="cuda")
        K.matmul(c, qa, qb, None, dev_scalar(float(sa)), dev_scalar(float(sb)), M, N, Kd)
        gemm_check(c.float().cpu().numpy(), g["rnd_exact"], g["rnd_sumabs"], scale, dt == torch.bfloat16)


def test_swiglu(K):
    g = load("producers.npz")
    inp, dout = g["swiglu_inp"], g["swiglu_dout"]
    BT, D = dout.shape
    x = dev_bf16(inp).view(1, BT, 2 * D)
    out = torch.empty((1, BT, D), dtype=torch.bfloat16, device="cuda")
    am = torch.full((1,), 9.0, device="cuda")
    K.swiglu_forward(out, x, am)
    # fp32 evaluation with the hardware's exp2 / reciprocal approximations: 2^-20 relative on top of the rounding
    assert_within(host_bits(out).reshape(BT, D), g["swiglu_out"], 2.0 ** -8 + 2.0 ** -20)
    assert am.item() == out.float().abs().max().item()
    dinp = torch.empty((1, BT, 2 * D), dtype=torch.bfloat16, device="cuda")
    K.swiglu_backward(dinp, dev_bf16(dout).view(1, BT, D), x, None)
    assert_within(host_bits(dinp).reshape(BT, 2 * D), g["swiglu_dinp"], 2.0 ** -8 + 2.0 ** -19,
                  slack=2.0 ** -20 * np.abs(np.tile(bf16_value(dout), 2)))


def test_rmsnorm_forward(K):
    g = load("producers.npz")
    eps = float(g["rms_eps"])
    N, C = g["rms_inp1"].shape
    i1, i2, w = dev_bf16(g["rms_inp1"]).view(1, N, C), dev_bf16(g["rms_inp2"]).view(1, N, C), dev_bf16(g["rms_weight"])
    out = torch.empty((1, N, C), dtype=torch.bfloat16, device="cuda")
    rms = torch.empty((1, N), dtype=torch.float32, device="cuda")
    K.rmsnorm_forward(out, rms, i1, w, None, eps)
    # two bf16 roundings (the normalised value, then the product with the weight: src/kernels/rmsnorm.cu:68-71)
    two = 2.0 ** -7 * 1.01 + 4e-6
    assert np.allclose(rms.cpu().numpy().reshape(N), g["rms_rstd"], rtol=2e-6)
    assert_within(host_bits(out).reshape(N, C), g["rms_out"], two)
    res = torch.empty((1, N, C), dtype=torch.bfloat16, device="cuda")
    K.fused_residual_rmsnorm_forward(res, out, rms, i1, i2, w, None, eps)
    assert np.array_equal(host_bits(res).reshape(N, C), g["rms_residual"])
    assert np.allclose(rms.cpu().numpy().reshape(N), g["rms_fused_rstd"], rtol=2e-6)
    assert_within(host_bits(out).reshape(N, C), g["rms_fused_out"], two)


def test_rope(K):
    g = load("producers.npz")
    B, T, Nq, Nkv, HD = (int(v) for v in g["rope_dims"])
    N = Nq + 2 * Nkv
    # the library's host table equals the fixture's (cos, sin) table up to an fp16 ulp of the C library's cosf / sinf
    tab = K.precompute_freqs_cis(HD, T, float(g["rope_theta"]))
    fix = torch.from_numpy(g["rope_table_f16"].view(np.int16)).view(torch.float16)
    assert torch.all((tab.float() - fix.float()).abs() <= 2.0 ** -10)
    x = dev_bf16(g["rope_qkv"]).view(B, T, N * HD)
    mag = np.abs(bf16_value(g["rope_qkv"]))
    mag = np.concatenate([mag[..., :HD // 2] + mag[..., HD // 2:]] * 2, axis=-1)     # |re| + |im| bounds both products
    for fn, key in ((K.rope_forward, "rope_forward"), (K.rope_backward, "rope_backward")):
        out = torch.empty_like(x)
        fn(out, x, fix.cuda(), None, Nq, Nkv)
        got = host_bits(out).reshape(B, T, N, HD)
        assert_within(got, g[key], 2.0 ** -8, slack=2.0 ** -22 * mag)
        assert np.array_equal(got[:, :, Nq + Nkv:], g["rope_qkv"][:, :, Nq + Nkv:])
