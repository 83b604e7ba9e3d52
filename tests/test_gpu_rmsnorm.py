"""GPU parity tests of the RMSNorm forward producers (through the C ABI, llmq_amd.kernels).

Bars:
  * residual = bf16(inp1 + inp2): bit exact against the oracle (one fp32 add, one rounding).
  * 1/rms: within 2^-18 relative of the oracle's (double-precision sum, correctly rounded); the kernel sums
    the squares in fp32.  The reference's own value is not bit-specified (launch-dependent summation
    order, approximate rsqrt) and its tests accept rtol 1e-2 (scripts/test_kernels.py:12-15,129-131).
  * normed: at most two bf16 ulp from the oracle and bit-identical for at least 99.5 % of the elements
    (a last-bit difference in 1/rms flips the intermediate bf16 rounding of a value that sits next to a
    tie); bit exact against the oracle's rounding chain evaluated with the GPU's own 1/rms.
  * bit exact: the abs-max epilogue against abs_max() of the tensor the kernel wrote; repeated launches.
"""
import numpy as np
import pytest
import torch

from gpu_util import dev_bf16, host_bits

pytestmark = pytest.mark.gpu

# (B, T, C): the reference's cases (scripts/test_kernels.py:116,574), the model widths of the bench
# configurations, the widest supported row, and row counts that do not fill the last workgroup
SHAPES = [(2, 3, 16), (1, 2, 64), (8, 256, 1024), (2, 5, 64), (1, 3, 256), (4, 8, 128), (8, 16, 512),
          (1, 37, 3584), (1, 9, 896), (1, 5, 8192), (1, 3, 16384), (1, 1, 8), (3, 7, 24)]


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from llmq_amd import kernels
    return kernels


def make_inputs(O, N, C, seed):
    x1 = O.fill_normal_bf16(N * C, seed, 0, 0.0, 1.5).reshape(N, C)
    x2 = O.fill_normal_bf16(N * C, seed, 1, 0.0, 0.7).reshape(N, C)
    w = O.fill_normal_bf16(C, seed, 2, 1.0, 0.3)
    return x1, x2, w


def chain_with_given_rrms(O, res_bits, w_bits, rrms):
    """The reference's rounding chain (src/kernels/rmsnorm.cu:68-71) with a given fp32 1/rms per row."""
    n = O.bf16_to_f32(O.f32_to_bf16((rrms[:, None] * O.bf16_to_f32(res_bits)).astype(np.float32)))
    return O.f32_to_bf16((n * O.bf16_to_f32(w_bits)[None, :]).astype(np.float32))


def check_normed(O, got, want, exact, res_bits, w_bits, got_rrms, want_rrms):
    assert np.all(np.abs(got_rrms.astype(np.float64) - want_rrms) <= np.abs(want_rrms) * 2.0 ** -18)
    g, wv = O.bf16_to_f32(got).astype(np.float64), O.bf16_to_f32(want).astype(np.float64)
    assert np.all(np.abs(g - wv) <= np.abs(exact) * 2.0 ** -6 + 1e-38)
    assert np.mean(got != want) <= 5e-3
    assert np.array_equal(got, chain_with_given_rrms(O, res_bits, w_bits, got_rrms))


@pytest.mark.parametrize("btc", SHAPES)
def test_rmsnorm_forward_matches_oracle(K, O, btc):
    B, T, C = btc
    N, eps = B * T, 1e-6
    x1, _, w = make_inputs(O, N, C, 600 + C)
    want, want_rrms, exact, _ = O.rmsnorm_forward(x1, w, eps)
    out = torch.full((B, T, C), float("nan"), dtype=torch.bfloat16, device="cuda")
    rms = torch.full((B, T), -1.0, dtype=torch.float32, device="cuda")
    am = torch.full((1,), 55.0, dtype=torch.float32, device="cuda")
    K.rmsnorm_forward(out, rms, dev_bf16(x1).reshape(B, T, C), dev_bf16(w), am, eps)
    got = host_bits(out).reshape(N, C)
    check_normed(O, got, want, exact, x1, w, rms.cpu().numpy().reshape(N), want_rrms)
    ref_am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.abs_max(ref_am, out)
    assert am.cpu().numpy().view(np.uint32)[0] == ref_am.cpu().numpy().view(np.uint32)[0]
    # without abs-max and without the rms output: same tensor
    out2 = torch.empty_like(out)
    K.rmsnorm_forward(out2, None, dev_bf16(x1).reshape(B, T, C), dev_bf16(w), None, eps)
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))


@pytest.mark.parametrize("btc", SHAPES)
def test_fused_residual_rmsnorm_forward_matches_oracle(K, O, btc):
    B, T, C = btc
    N, eps = B * T, 1e-5
    x1, x2, w = make_inputs(O, N, C, 700 + C)
    want, want_rrms, exact, want_res = O.rmsnorm_forward(x1, w, eps, x2)
    res = torch.full((B, T, C), float("nan"), dtype=torch.bfloat16, device="cuda")
    normed = torch.full((B, T, C), float("nan"), dtype=torch.bfloat16, device="cuda")
    rrms = torch.full((B, T), -1.0, dtype=torch.float32, device="cuda")
    am = torch.full((1,), 55.0, dtype=torch.float32, device="cuda")
    a, b = dev_bf16(x1).reshape(B, T, C), dev_bf16(x2).reshape(B, T, C)
    K.fused_residual_rmsnorm_forward(res, normed, rrms, a, b, dev_bf16(w), am, eps)
    assert np.array_equal(host_bits(res).reshape(N, C), want_res)
    check_normed(O, host_bits(normed).reshape(N, C), want, exact, want_res, w, rrms.cpu().numpy().reshape(N), want_rrms)
    ref_am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.abs_max(ref_am, normed)
    assert am.cpu().numpy().view(np.uint32)[0] == ref_am.cpu().numpy().view(np.uint32)[0]
    # in place on the first input (the residual stream updated where it lives), and repeatable
    normed2, rrms2 = torch.empty_like(normed), torch.empty_like(rrms)
    a2 = a.clone()
    K.fused_residual_rmsnorm_forward(a2, normed2, rrms2, a2, b, dev_bf16(w), None, eps)
    assert torch.equal(a2.view(torch.int16), res.view(torch.int16))
    assert torch.equal(normed2.view(torch.int16), normed.view(torch.int16)) and torch.equal(rrms2, rrms)


def test_rmsnorm_reference_test_tolerances(K, O):
    """The reference's own check (scripts/test_kernels.py:116-131): randn inputs and weights, torch float
    reference with a single rounding, rtol 1e-2 / atol 5e-3."""
    B, T, C, eps = 8, 256, 1024, 1e-6
    g = torch.Generator(device="cuda").manual_seed(0)
    inp = torch.randn((B, T, C), device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16)
    weight = torch.randn((C,), device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16)
    out, rms = torch.empty_like(inp), torch.empty((B, T), device="cuda", dtype=torch.float32)
    K.rmsnorm_forward(out, rms, inp, weight, None, eps)
    var = (inp.float() ** 2).mean(dim=-1, keepdim=True)
    r_rms = 1.0 / torch.sqrt(var + eps)
    ref = (inp.float() * r_rms * weight.float()).to(torch.bfloat16)
    assert torch.allclose(rms, r_rms.squeeze(-1), rtol=1e-2, atol=5e-3)
    assert torch.allclose(out.float(), ref.float(), rtol=1e-2, atol=5e-3)


def test_rmsnorm_argument_errors(K):
    x = torch.zeros((1, 4, 12), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="divisible by 8"):
        K.rmsnorm_forward(torch.empty_like(x), None, x, torch.zeros(12, dtype=torch.bfloat16, device="cuda"), None, 1e-6)
    x = torch.zeros((1, 2, 16392), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="16384"):
        K.rmsnorm_forward(torch.empty_like(x), None, x, torch.zeros(16392, dtype=torch.bfloat16, device="cuda"), None, 1e-6)
    x = torch.zeros((1, 4, 16), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        K.rmsnorm_forward(torch.empty_like(x), None, x, torch.zeros(8, dtype=torch.bfloat16, device="cuda"), None, 1e-6)
    # empty: the abs-max slot is still reset
    am = torch.full((1,), 5.0, dtype=torch.float32, device="cuda")
    e = torch.zeros((0, 4, 16), dtype=torch.bfloat16, device="cuda")
    K.rmsnorm_forward(torch.empty_like(e), None, e, torch.zeros(16, dtype=torch.bfloat16, device="cuda"), am, 1e-6)
    assert am.item() == 0.0


def test_rmsnorm_full_size_properties(K, O):
    """Configuration-4 token count and width (8192 x 3584): sampled rows against the oracle, abs-max invariant
    on the whole tensor, and the chain into quantize_with_abs_max as the model runs it."""
    B, T, C, eps = 8, 1024, 3584, 1e-6
    g = torch.Generator(device="cuda").manual_seed(9)
    a = torch.randn((B, T, C), device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16)
    b = (0.3 * torch.randn((B, T, C), device="cuda", dtype=torch.float32, generator=g)).to(torch.bfloat16)
    w = (1.0 + 0.2 * torch.randn((C,), device="cuda", dtype=torch.float32, generator=g)).to(torch.bfloat16)
    res, normed = torch.empty_like(a), torch.empty_like(a)
    rrms = torch.empty((B, T), dtype=torch.float32, device="cuda")
    stats = torch.zeros(2, dtype=torch.float32, device="cuda")
    K.fused_residual_rmsnorm_forward(res, normed, rrms, a, b, w, stats[0:1], eps)
    ref_am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.abs_max(ref_am, normed)
    assert stats[0].item() == ref_am.item() and ref_am.item() > 0
    rows = torch.tensor([0, 3, 4098, 8191], device="cuda")
    want, want_rrms, exact, want_res = O.rmsnorm_forward(host_bits(a.reshape(-1, C)[rows]), host_bits(w), eps,
                                                         host_bits(b.reshape(-1, C)[rows]))
    assert np.array_equal(host_bits(res.reshape(-1, C)[rows]), want_res)
    check_normed(O, host_bits(normed.reshape(-1, C)[rows]), want, exact, want_res, host_bits(w),
                 rrms.reshape(-1)[rows].cpu().numpy(), want_rrms)
    q = torch.empty((B * T, C), dtype=torch.float8_e4m3fn, device="cuda")
    K.quantize_with_abs_max(q, stats[1:2], normed, stats[0:1])
    codes, dq = O.quantize_e4m3(host_bits(normed.reshape(-1, C)[rows]), stats[0].item())
    assert np.array_equal(host_bits(q[rows]), codes) and np.float32(dq) == stats[1].item()


# ---------------------------------------------------------------------------------------- backward
# Bars for rmsnorm_backward against the oracle (double evaluation, one rounding):
#   dinp:    |err| <= one bf16 ulp of the value + 2^-18 of the sum of the magnitudes of its terms (the scale of
#            the fp32 evaluation error where the terms cancel);
#   dweight: the same with the sum over all rows of |inp * rstd * dout| as the magnitude;
#   bit exact: abs-max against abs_max(dinp); repeated launches (fixed summation order).
# The reference's own tolerances (rtol 1e-2 / atol 5e-3, scripts/test_kernels.py:153-157) are asserted on its
# construction as well.
BWD_SHAPES = [(2, 3, 16), (1, 4, 64), (4, 8, 256), (1, 37, 3584), (1, 9, 896), (1, 5, 8192), (2, 600, 128), (1, 1, 8)]


def run_backward(K, dres, dw0, dout, x, w, rstd, B, T, C, with_absmax=True, in_place=False):
    d_dres = dev_bf16(dres).reshape(B, T, C)
    dinp = d_dres if in_place else torch.full((B, T, C), float("nan"), dtype=torch.bfloat16, device="cuda")
    dweight = dev_bf16(dw0).clone()
    scratch = torch.full((K.get_rmsnorm_backward_scratch_size(C),), float("nan"), dtype=torch.float32, device="cuda")
    am = torch.full((1,), 9.0, dtype=torch.float32, device="cuda") if with_absmax else None
    K.rmsnorm_backward(dinp, dweight, scratch, d_dres, dev_bf16(dout).reshape(B, T, C), dev_bf16(x).reshape(B, T, C),
                       dev_bf16(w), torch.from_numpy(rstd).cuda().reshape(B, T), am)
    return dinp, dweight, am


@pytest.mark.parametrize("btc", BWD_SHAPES)
def test_rmsnorm_backward_matches_oracle(K, O, btc):
    B, T, C = btc
    N = B * T
    x, _, w = make_inputs(O, N, C, 800 + C)
    dout = O.fill_normal_bf16(N * C, 800 + C, 3, 0.0, 0.8).reshape(N, C)
    dres = O.fill_normal_bf16(N * C, 800 + C, 4, 0.0, 0.5).reshape(N, C)
    dw0 = O.fill_normal_bf16(C, 800 + C, 5, 0.0, 2.0)
    _, rstd, _, _ = O.rmsnorm_forward(x, w, 1e-6)
    want = O.rmsnorm_backward(dres, dw0, dout, x, w, rstd)
    dinp, dweight, am = run_backward(K, dres, dw0, dout, x, w, rstd, B, T, C)
    got = O.bf16_to_f32(host_bits(dinp)).reshape(N, C).astype(np.float64)
    tol = np.abs(want["exact_dinp"]) * 2.0 ** -7 + want["mag_dinp"] * 2.0 ** -18 + 1e-38
    assert np.all(np.abs(got - O.bf16_to_f32(want["dinp"])) <= tol)
    gw = O.bf16_to_f32(host_bits(dweight)).astype(np.float64)
    tolw = np.abs(want["exact_dw"]) * 2.0 ** -7 + want["mag_dw"] * 2.0 ** -18 + 1e-38
    assert np.all(np.abs(gw - O.bf16_to_f32(want["dweight"])) <= tolw)
    ref_am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.abs_max(ref_am, dinp)
    assert am.cpu().numpy().view(np.uint32)[0] == ref_am.cpu().numpy().view(np.uint32)[0]
    # in place on dresidual, without the abs-max: the same bits, twice
    dinp2, dweight2, _ = run_backward(K, dres, dw0, dout, x, w, rstd, B, T, C, with_absmax=False, in_place=True)
    assert torch.equal(dinp.view(torch.int16), dinp2.view(torch.int16))
    assert torch.equal(dweight.view(torch.int16), dweight2.view(torch.int16))


def test_rmsnorm_backward_reference_test_construction(K, O):
    """scripts/test_kernels.py:136-190: randn tensors, zero and non-zero dresidual, torch float reference."""
    B, T, C, eps = 4, 8, 256, 1e-6
    g = torch.Generator(device="cuda").manual_seed(1)
    rn = lambda *s: torch.randn(s, device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16)
    inp, weight, dout, dres = rn(B, T, C), rn(C), rn(B, T, C), rn(B, T, C)
    r = 1.0 / torch.sqrt((inp.float() ** 2).mean(dim=-1, keepdim=True) + eps)
    normed, dy_w = inp.float() * r, dout.float() * weight.float()
    ref_dinp = r * (dy_w - normed * (dy_w * normed).sum(dim=-1, keepdim=True) / C)
    ref_dw = (dout.float() * inp.float() * r).sum(dim=(0, 1))
    scratch = torch.zeros(K.get_rmsnorm_backward_scratch_size(C), device="cuda", dtype=torch.float32)
    for start in (torch.zeros_like(dres), dres):
        dinp, dweight = torch.empty_like(inp), torch.zeros(C, device="cuda", dtype=torch.bfloat16)
        K.rmsnorm_backward(dinp, dweight, scratch, start, dout, inp, weight, r.squeeze(-1).contiguous(), None)
        assert torch.allclose(dinp.float(), (start.float() + ref_dinp).to(torch.bfloat16).float(), rtol=1e-2, atol=5e-3)
        assert torch.allclose(dweight.float(), ref_dw.to(torch.bfloat16).float(), rtol=1e-2, atol=5e-3)


def test_rmsnorm_backward_argument_errors(K):
    B, T, C = 1, 4, 64
    z = lambda *s: torch.zeros(s, dtype=torch.bfloat16, device="cuda")
    rstd = torch.ones((B, T), dtype=torch.float32, device="cuda")
    small = torch.zeros(8, dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError, match="scratch"):
        K.rmsnorm_backward(z(B, T, C), z(C), small, z(B, T, C), z(B, T, C), z(B, T, C), z(C), rstd, None)
    scratch = torch.zeros(K.get_rmsnorm_backward_scratch_size(8200), dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError, match="8192"):
        K.rmsnorm_backward(z(B, T, 8200), z(8200), scratch, z(B, T, 8200), z(B, T, 8200), z(B, T, 8200), z(8200), rstd, None)
    with pytest.raises(ValueError):
        K.rmsnorm_backward(z(B, T, C), z(C), scratch, z(B, T, C), z(B, T, C), z(B, T, C), z(C // 2), rstd, None)


def test_rmsnorm_backward_full_size_properties(K, O):
    """Configuration-4 size (8192 x 3584): sampled rows of dinp and all of dweight against the oracle run on a
    row subset is not possible for dweight (it sums every row), so dweight is checked against a float64 torch
    reduction on the device; abs-max invariant on the whole tensor."""
    B, T, C, eps = 8, 1024, 3584, 1e-6
    g = torch.Generator(device="cuda").manual_seed(3)
    rn = lambda s, std: (std * torch.randn(s, device="cuda", dtype=torch.float32, generator=g)).to(torch.bfloat16)
    inp, dout, dres = rn((B, T, C), 1.0), rn((B, T, C), 0.01), rn((B, T, C), 0.01)
    w = (1.0 + 0.2 * torch.randn((C,), device="cuda", dtype=torch.float32, generator=g)).to(torch.bfloat16)
    out, rstd = torch.empty_like(inp), torch.empty((B, T), dtype=torch.float32, device="cuda")
    K.rmsnorm_forward(out, rstd, inp, w, None, eps)
    dinp, dweight = torch.empty_like(inp), torch.zeros(C, dtype=torch.bfloat16, device="cuda")
    scratch = torch.empty(K.get_rmsnorm_backward_scratch_size(C), dtype=torch.float32, device="cuda")
    am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.rmsnorm_backward(dinp, dweight, scratch, dres, dout, inp, w, rstd, am)
    ref_am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.abs_max(ref_am, dinp)
    assert am.item() == ref_am.item() and am.item() > 0
    rows = torch.tensor([0, 5, 4099, 8191], device="cuda")
    sub = lambda t: host_bits(t.reshape(-1, C)[rows])
    want = O.rmsnorm_backward(sub(dres), np.zeros(C, np.uint16), sub(dout), sub(inp), host_bits(w),
                              rstd.reshape(-1)[rows].cpu().numpy())
    got = O.bf16_to_f32(sub(dinp)).astype(np.float64)
    tol = np.abs(want["exact_dinp"]) * 2.0 ** -7 + want["mag_dinp"] * 2.0 ** -18 + 1e-38
    assert np.all(np.abs(got - O.bf16_to_f32(want["dinp"])) <= tol)
    terms = inp.double().reshape(-1, C) * rstd.double().reshape(-1, 1) * dout.double().reshape(-1, C)
    exact_dw, mag_dw = terms.sum(dim=0).cpu().numpy(), terms.abs().sum(dim=0).cpu().numpy()
    gw = dweight.float().cpu().numpy().astype(np.float64)
    assert np.all(np.abs(gw - exact_dw) <= np.abs(exact_dw) * 2.0 ** -7 + mag_dw * 2.0 ** -18)
