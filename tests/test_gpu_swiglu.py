"""GPU parity tests of the SwiGLU producers (through the C ABI, llmq_amd.kernels).

Bars:
  * bf16 values against the CPU oracle (correctly rounded double evaluation): at most ONE bf16 ulp
    (2^-7 relative) plus, for the gate gradient, 2^-20 of its factors' magnitude where the bracket
    1 + gate * (1 - s) cancels.  The reference's device code is not bit-specified (CUDA expf, approximate
    reciprocal) and its own tests accept 3e-2 / 5e-3 absolute error on U(-1, 1) inputs
    (src/testing/test-swiglu.cu:202,207,238,243), which is asserted as well.
  * bit exact: the abs-max epilogue against abs_max() of the tensor the kernel wrote; swiglu_forward_quant
    against swiglu_forward + quantize_with_abs_max (bytes and scale, src/testing/test-swiglu.cu:243-315).
"""
import numpy as np
import pytest
import torch

from gpu_util import dev_bf16, dev_scalar, host_bits

pytestmark = pytest.mark.gpu

# (B, T, C): the reference's own cases (scripts/test_kernels.py:210,224,244) and ragged ones whose size is
# not a multiple of a workgroup's share
SHAPES = [(1, 16, 128), (8, 8, 16), (5, 32, 32), (32, 32, 1024), (2, 8, 64), (4, 16, 128), (1, 8, 256), (4, 16, 64),
          (3, 5, 24), (1, 1, 8), (7, 13, 40)]


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from llmq_amd import kernels
    return kernels


def inputs(O, B, T, C, seed, spread=2.0):
    inp = O.fill_normal_bf16(B * T * 2 * C, seed, 0, 0.0, spread).reshape(B * T, 2 * C)
    dout = O.fill_normal_bf16(B * T * C, seed, 1, 0.0, 1.0).reshape(B * T, C)
    return inp, dout


def within_one_ulp(O, got_bits, want_bits, exact, slack=None):
    got, want = O.bf16_to_f32(got_bits).astype(np.float64), O.bf16_to_f32(want_bits).astype(np.float64)
    tol = np.abs(exact) * 2.0 ** -7 + 1e-38
    if slack is not None:
        tol = tol + slack
    bad = np.abs(got - want) > tol
    assert not bad.any(), "first mismatch: got %r want %r exact %r" % (got[bad][0], want[bad][0], exact[bad][0])


def run_forward(K, inp, B, T, C, with_absmax):
    out = torch.full((B, T, C), float("nan"), dtype=torch.bfloat16, device="cuda")
    am = torch.full((1,), 123.0, dtype=torch.float32, device="cuda") if with_absmax else None
    K.swiglu_forward(out, dev_bf16(inp).reshape(B, T, 2 * C), am)
    return out, am


@pytest.mark.parametrize("btc", SHAPES)
def test_swiglu_forward_matches_oracle(K, O, btc):
    B, T, C = btc
    inp, _ = inputs(O, B, T, C, 300 + C)
    want, exact = O.swiglu_forward(inp)
    out, am = run_forward(K, inp, B, T, C, True)
    got = host_bits(out).reshape(B * T, C)
    within_one_ulp(O, got, want, exact)
    # the abs-max epilogue is the abs-max of what was written, bit for bit, and the variant without it
    # writes the same tensor
    ref_am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.abs_max(ref_am, out)
    assert am.cpu().numpy().view(np.uint32)[0] == ref_am.cpu().numpy().view(np.uint32)[0]
    assert am.item() == np.abs(O.bf16_to_f32(got)).max()
    out2, _ = run_forward(K, inp, B, T, C, False)
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))


def test_swiglu_reference_test_construction(K, O):
    """Inputs uniform in (-1, 1) as in src/testing/test-swiglu.cu:166-207: the reference's margins
    (3e-2 per value, 5e-3 on the abs-max) hold with a wide gap."""
    B, T, C = 4, 64, 256
    rng = np.random.default_rng(1337)
    inp = O.f32_to_bf16(rng.uniform(-1, 1, (B * T, 2 * C)).astype(np.float32))
    dout = O.f32_to_bf16(rng.uniform(-0.5, 0.5, (B * T, C)).astype(np.float32))
    _, exact = O.swiglu_forward(inp)
    out, am = run_forward(K, inp, B, T, C, True)
    got = O.bf16_to_f32(host_bits(out)).reshape(B * T, C)
    assert np.abs(got - exact).max() < 3e-2 and abs(am.item() - np.abs(exact).max()) < 5e-3
    dinp = torch.empty((B, T, 2 * C), dtype=torch.bfloat16, device="cuda")
    am2 = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.swiglu_backward(dinp, dev_bf16(dout).reshape(B, T, C), dev_bf16(inp).reshape(B, T, 2 * C), am2)
    _, dexact = O.swiglu_backward(dout, inp)
    gotd = O.bf16_to_f32(host_bits(dinp)).reshape(B * T, 2 * C)
    assert np.abs(gotd - dexact).max() < 3e-2 and abs(am2.item() - np.abs(dexact).max()) < 5e-3


@pytest.mark.parametrize("btc", SHAPES)
def test_swiglu_forward_quant_is_forward_plus_quantize(K, O, btc):
    B, T, C = btc
    inp, _ = inputs(O, B, T, C, 400 + C)
    x = dev_bf16(inp).reshape(B, T, 2 * C)
    out, am = run_forward(K, inp, B, T, C, True)
    two_step = torch.empty((B, T, C), dtype=torch.float8_e4m3fn, device="cuda")
    scale_a = torch.full((1,), -1.0, dtype=torch.float32, device="cuda")
    K.quantize_with_abs_max(two_step, scale_a, out, am)
    direct = torch.full((B, T, C), 0x55, dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
    scale_b = torch.full((1,), -1.0, dtype=torch.float32, device="cuda")
    K.swiglu_forward_quant(direct, scale_b, x, am)
    assert torch.equal(two_step.view(torch.uint8), direct.view(torch.uint8))
    assert scale_a.cpu().numpy().view(np.uint32)[0] == scale_b.cpu().numpy().view(np.uint32)[0]
    # and against the oracle's quantizer applied to the tensor the GPU wrote
    q, dq = O.quantize_e4m3(host_bits(out).reshape(-1), am.item())
    assert np.array_equal(host_bits(direct).reshape(-1), q) and np.float32(dq) == scale_b.item()
    # no scale pointer: same bytes
    direct2 = torch.empty_like(direct)
    K.swiglu_forward_quant(direct2, None, x, am)
    assert torch.equal(direct.view(torch.uint8), direct2.view(torch.uint8))


@pytest.mark.parametrize("btc", SHAPES)
def test_swiglu_backward_matches_oracle(K, O, btc):
    B, T, C = btc
    inp, dout = inputs(O, B, T, C, 500 + C)
    want, exact = O.swiglu_backward(dout, inp)
    dinp = torch.full((B, T, 2 * C), float("nan"), dtype=torch.bfloat16, device="cuda")
    am = torch.full((1,), 77.0, dtype=torch.float32, device="cuda")
    K.swiglu_backward(dinp, dev_bf16(dout).reshape(B, T, C), dev_bf16(inp).reshape(B, T, 2 * C), am)
    got = host_bits(dinp).reshape(B * T, 2 * C)
    up = np.abs(O.bf16_to_f32(inp[:, :C]).astype(np.float64))
    gate = np.abs(O.bf16_to_f32(inp[:, C:]).astype(np.float64))
    d = np.abs(O.bf16_to_f32(dout).astype(np.float64))
    slack = np.concatenate([np.zeros_like(up), d * up * (1.0 + gate) * 2.0 ** -20], axis=1)
    within_one_ulp(O, got, want, exact, slack)
    ref_am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.abs_max(ref_am, dinp)
    assert am.cpu().numpy().view(np.uint32)[0] == ref_am.cpu().numpy().view(np.uint32)[0]
    dinp2 = torch.empty_like(dinp)
    K.swiglu_backward(dinp2, dev_bf16(dout).reshape(B, T, C), dev_bf16(inp).reshape(B, T, 2 * C), None)
    assert torch.equal(dinp.view(torch.int16), dinp2.view(torch.int16))


def test_swiglu_special_values(K, O):
    """gate = 0 -> 0; huge gate -> up * gate; very negative gate -> 0; NaN inputs give NaN outputs that the
    abs-max skips; Inf propagates into the abs-max."""
    C = 8
    f = lambda v: O.f32_to_bf16(np.asarray(v, dtype=np.float32))
    up = f([1.5, -2.0, 3.0, 0.5, 1.0, -1.0, 7.0, 0.25])
    rows = [np.concatenate([up, f([g] * C)]) for g in (0.0, 64.0, -200.0)]
    rows.append(np.concatenate([f([np.nan, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0]), f([1.0, np.nan, 2.0, 2.0, 2.0, 2.0, 2.0, 2.0])]))
    inp = np.stack(rows)
    out, am = run_forward(K, inp, 1, 4, C, True)
    got = O.bf16_to_f32(host_bits(out)).reshape(4, C)
    u = O.bf16_to_f32(up)
    assert np.array_equal(got[0], 0.0 * u) and np.array_equal(got[1], u * 64.0) and np.array_equal(np.abs(got[2]), 0.0 * np.abs(u))
    assert np.isnan(got[3, :2]).all() and np.isfinite(got[3, 2:]).all()
    assert am.item() == 7.0 * 64.0
    inf_row = np.concatenate([f([np.inf] + [1.0] * 7), f([3.0] * C)]).reshape(1, 2 * C)
    _, am2 = run_forward(K, inf_row, 1, 1, C, True)
    assert am2.item() == np.inf


def test_swiglu_argument_errors(K):
    x = torch.zeros((2, 4, 24), dtype=torch.bfloat16, device="cuda")      # C = 12: not a multiple of 8
    out = torch.zeros((2, 4, 12), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="divisible by 8"):
        K.swiglu_forward(out, x, None)
    with pytest.raises(ValueError, match="divisible by 8"):
        K.swiglu_backward(torch.zeros_like(x), out, x, None)
    with pytest.raises(ValueError):
        K.swiglu_forward(torch.zeros((2, 4, 16), dtype=torch.bfloat16, device="cuda"), x, None)   # shape mismatch
    with pytest.raises(ValueError, match="abs_max"):
        K.swiglu_forward_quant(torch.zeros((2, 4, 16), dtype=torch.uint8, device="cuda"), None,
                               torch.zeros((2, 4, 32), dtype=torch.bfloat16, device="cuda"), None)
    # empty tensors are fine and still reset / write the scalars
    am = torch.full((1,), 5.0, dtype=torch.float32, device="cuda")
    K.swiglu_forward(torch.zeros((0, 4, 16), dtype=torch.bfloat16, device="cuda"),
                     torch.zeros((0, 4, 32), dtype=torch.bfloat16, device="cuda"), am)
    assert am.item() == 0.0


def test_swiglu_full_size_properties(K, O):
    """Configuration-4 activation size (8192 tokens x 18944): sampled values against the oracle, the abs-max
    and the quantizing invariants on the whole tensor."""
    B, T, C = 8, 1024, 18944
    g = torch.Generator(device="cuda").manual_seed(5)
    x = (torch.randn((B, T, 2 * C), device="cuda", dtype=torch.float32, generator=g) * 1.5).to(torch.bfloat16)
    out = torch.empty((B, T, C), dtype=torch.bfloat16, device="cuda")
    am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.swiglu_forward(out, x, am)
    ref_am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.abs_max(ref_am, out)
    assert am.item() == ref_am.item() and am.item() > 0
    rows = torch.tensor([0, 1, 4097, 8191], device="cuda")
    sub_in = host_bits(x.reshape(B * T, 2 * C)[rows])
    want, exact = O.swiglu_forward(sub_in)
    within_one_ulp(O, host_bits(out.reshape(B * T, C)[rows]), want, exact)
    q2 = torch.empty((B, T, C), dtype=torch.float8_e4m3fn, device="cuda")
    K.quantize_with_abs_max(q2, None, out, am)
    q1 = torch.empty((B, T, C), dtype=torch.float8_e4m3fn, device="cuda")
    K.swiglu_forward_quant(q1, None, x, am)
    assert torch.equal(q1.view(torch.uint8), q2.view(torch.uint8))
    dout = torch.randn((B, T, C), device="cuda", dtype=torch.bfloat16, generator=g)
    dinp = torch.empty_like(x)
    K.swiglu_backward(dinp, dout, x, am)
    K.abs_max(ref_am, dinp)
    assert am.item() == ref_am.item()
    wantd, exactd = O.swiglu_backward(host_bits(dout.reshape(B * T, C)[rows]), sub_in)
    upv = np.abs(O.bf16_to_f32(sub_in[:, :C]).astype(np.float64))
    gv = np.abs(O.bf16_to_f32(sub_in[:, C:]).astype(np.float64))
    dv = np.abs(O.bf16_to_f32(host_bits(dout.reshape(B * T, C)[rows])).astype(np.float64))
    slack = np.concatenate([np.zeros_like(upv), dv * upv * (1.0 + gv) * 2.0 ** -20], axis=1)
    within_one_ulp(O, host_bits(dinp.reshape(B * T, 2 * C)[rows]), wantd, exactd, slack)
