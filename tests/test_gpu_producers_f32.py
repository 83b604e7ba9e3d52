"""GPU parity tests of the fp32 overloads of the producers (SwiGLU, rotary embedding, RMSNorm forward / backward),
through the C ABI (llmq_amd.kernels dispatches on the tensors' dtype).

Bars (ulp = 2^-23 relative, the spacing of fp32):
  * values against the CPU oracle's double evaluation: a few ulp of the result plus, where terms cancel, 2^-21 of
    the terms' magnitudes.  The reference's device code is not bit-specified (CUDA expf, approximate reciprocal and
    rsqrt, launch-dependent summation order); its own tests accept 1e-6 / 1e-5 absolute on U(-1, 1) inputs for
    SwiGLU (src/testing/test-swiglu.cu:117,147) and 1e-5 for rope (src/testing/test-rope.cu), asserted as well.
  * bit exact: the abs-max epilogue against abs_max() of the tensor the kernel wrote (and against numpy); the variant
    without abs-max writes the same tensor; repeated launches; the fused residual (one fp32 add).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
ULP = 2.0 ** -23


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from llmq_amd import kernels
    return kernels


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def normal_f32(O, n, seed, stream, mean=0.0, std=1.0):
    """fp32 values that are not bf16-representable: a bf16 draw plus a smaller second one."""
    a = O.bf16_to_f32(O.fill_normal_bf16(n, seed, stream, mean, std)).astype(np.float32)
    b = O.bf16_to_f32(O.fill_normal_bf16(n, seed, stream + 100, 0.0, std * 2.0 ** -9)).astype(np.float32)
    return (a + b).astype(np.float32)


def slot(value=123.0):
    return torch.full((1,), value, dtype=torch.float32, device="cuda")


def absmax_is_exact(K, am, tensor):
    ref = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.abs_max(ref, tensor)
    assert host(am).view(np.uint32)[0] == host(ref).view(np.uint32)[0]
    assert am.item() == np.abs(host(tensor)).max()


SWIGLU_SHAPES = [(1, 16, 128), (8, 8, 16), (5, 32, 32), (32, 32, 1024), (3, 5, 12), (1, 1, 4), (7, 13, 20), (2, 64, 3584)]


@pytest.mark.parametrize("btc", SWIGLU_SHAPES)
def test_swiglu_f32_matches_oracle(K, O, btc):
    B, T, C = btc
    inp = normal_f32(O, B * T * 2 * C, 900 + C, 0, 0.0, 2.0).reshape(B * T, 2 * C)
    dout = normal_f32(O, B * T * C, 900 + C, 1).reshape(B * T, C)
    _, exact = O.swiglu_forward(inp)
    x = dev(inp).reshape(B, T, 2 * C)
    out = torch.full((B, T, C), float("nan"), dtype=torch.float32, device="cuda")
    am = slot()
    K.swiglu_forward(out, x, am)
    got = host(out).reshape(B * T, C).astype(np.float64)
    assert np.all(np.abs(got - exact) <= np.abs(exact) * 4 * ULP + 1e-37)
    absmax_is_exact(K, am, out)
    out2 = torch.empty_like(out)
    K.swiglu_forward(out2, x, None)
    assert torch.equal(out.view(torch.int32), out2.view(torch.int32))

    _, dexact = O.swiglu_backward(dout, inp)
    dinp = torch.full((B, T, 2 * C), float("nan"), dtype=torch.float32, device="cuda")
    am2 = slot(77.0)
    K.swiglu_backward(dinp, dev(dout).reshape(B, T, C), x, am2)
    gotd = host(dinp).reshape(B * T, 2 * C).astype(np.float64)
    up, gate, d = np.abs(inp[:, :C].astype(np.float64)), np.abs(inp[:, C:].astype(np.float64)), np.abs(dout.astype(np.float64))
    # the bracket 1 + gate (1 - s) of the gate gradient cancels for negative gates
    slack = np.concatenate([np.zeros_like(up), d * up * (1.0 + gate) * 4 * ULP], axis=1)
    assert np.all(np.abs(gotd - dexact) <= np.abs(dexact) * 6 * ULP + slack + 1e-37)
    absmax_is_exact(K, am2, dinp)
    dinp2 = torch.empty_like(dinp)
    K.swiglu_backward(dinp2, dev(dout).reshape(B, T, C), x, None)
    assert torch.equal(dinp.view(torch.int32), dinp2.view(torch.int32))


def test_swiglu_f32_reference_test_construction(K, O):
    """src/testing/test-swiglu.cu:83-156: U(-1, 1) inputs, U(-0.5, 0.5) gradients; margins 1e-6 (forward, abs-max) and
    1e-5 (backward)."""
    B, T, C = 4, 64, 256
    rng = np.random.default_rng(1337)
    inp = rng.uniform(-1, 1, (B * T, 2 * C)).astype(np.float32)
    dout = rng.uniform(-0.5, 0.5, (B * T, C)).astype(np.float32)
    _, exact = O.swiglu_forward(inp)
    _, dexact = O.swiglu_backward(dout, inp)
    out = torch.empty((B, T, C), dtype=torch.float32, device="cuda")
    dinp = torch.empty((B, T, 2 * C), dtype=torch.float32, device="cuda")
    am, am2 = slot(), slot()
    K.swiglu_forward(out, dev(inp).reshape(B, T, 2 * C), am)
    K.swiglu_backward(dinp, dev(dout).reshape(B, T, C), dev(inp).reshape(B, T, 2 * C), am2)
    assert np.abs(host(out).reshape(B * T, C) - exact).max() < 1e-6 and abs(am.item() - np.abs(exact).max()) < 1e-6
    assert np.abs(host(dinp).reshape(B * T, 2 * C) - dexact).max() < 1e-5 and abs(am2.item() - np.abs(dexact).max()) < 1e-6


def test_swiglu_f32_special_values_and_errors(K, O):
    """gate = 0 -> 0; huge gate -> up * gate; gate below -88.7 (exp overflows fp32, as the reference's expf does) ->
    (signed) zero, not NaN; gate = -80 still accurate; NaNs are skipped by the abs-max; C must be a multiple of 4 and
    dtypes must agree."""
    C = 4
    up = np.array([1.5, -2.0, 3.0, 0.5], dtype=np.float32)
    rows = [np.concatenate([up, np.full(C, g, dtype=np.float32)]) for g in (0.0, 64.0, -200.0, -80.0)]
    rows.append(np.array([np.nan, 1.0, 1.0, 1.0, 1.0, np.nan, 2.0, 2.0], dtype=np.float32))
    inp = np.stack(rows)
    out = torch.empty((1, 5, C), dtype=torch.float32, device="cuda")
    am = slot()
    K.swiglu_forward(out, dev(inp).reshape(1, 5, 2 * C), am)
    got = host(out).reshape(5, C)
    assert np.array_equal(got[0], 0.0 * up) and np.array_equal(got[1], up * np.float32(64.0))
    assert np.array_equal(np.abs(got[2]), np.zeros(C, dtype=np.float32))
    _, exact = O.swiglu_forward(inp[3:4])
    assert np.all(np.abs(got[3] - exact[0]) <= np.abs(exact[0]) * 4 * ULP)
    assert np.isnan(got[4, :2]).all() and np.isfinite(got[4, 2:]).all()
    assert am.item() == np.nanmax(np.abs(got))
    with pytest.raises(ValueError):
        K.swiglu_forward(torch.empty((1, 1, 6), dtype=torch.float32, device="cuda"),
                         torch.empty((1, 1, 12), dtype=torch.float32, device="cuda"), None)
    with pytest.raises(ValueError, match="dtype"):
        K.swiglu_forward(torch.empty((1, 1, 8), dtype=torch.bfloat16, device="cuda"),
                         torch.empty((1, 1, 16), dtype=torch.float32, device="cuda"), None)


# (B, T, Nq, Nkv, HD): the reference's own (src/testing/test-rope.cu), grouped-query shapes, head sizes 8 .. 128
ROPE_SHAPES = [(2, 16, 4, 4, 64), (1, 5, 3, 2, 16), (2, 7, 14, 2, 64), (1, 33, 28, 4, 128), (3, 4, 2, 1, 8), (1, 1, 1, 1, 24)]


@pytest.mark.parametrize("shape", ROPE_SHAPES)
def test_rope_f32_matches_oracle(K, O, shape):
    B, T, Nq, Nkv, HD = shape
    N = Nq + 2 * Nkv
    x = normal_f32(O, B * T * N * HD, 950 + HD, 0).reshape(B * T, N, HD)
    tab = K.precompute_freqs_cis(HD, T, 10000.0, dtype=torch.float32)
    tab_np = tab.numpy()
    # the host table: numpy float64 cos / sin of the fp32 angle, within the rounding of powf and of the angle
    i = np.arange(HD // 2)
    inv = (np.float32(1.0) / np.power(np.float32(10000.0), (2 * i).astype(np.float32) / np.float32(HD))).astype(np.float32)
    ang = (np.arange(T, dtype=np.float32)[:, None] * inv[None, :]).astype(np.float32).astype(np.float64)
    assert np.allclose(tab_np[:, 0::2], np.cos(ang), rtol=0, atol=1e-5) and np.allclose(tab_np[:, 1::2], np.sin(ang), rtol=0, atol=1e-5)
    for backward in (False, True):
        want, exact, mag = O.rope(x, tab_np, T, Nq, Nkv, backward=backward)
        xin = dev(x).reshape(B, T, N * HD)
        out = torch.full((B, T, N * HD), float("nan"), dtype=torch.float32, device="cuda")
        am = slot()
        fn = K.rope_backward if backward else K.rope_forward
        fn(out, xin, tab.cuda(), am, Nq, Nkv)
        got = host(out).reshape(B * T, N, HD)
        assert np.all(np.abs(got.astype(np.float64) - exact) <= mag * 2 * ULP + 1e-37)
        assert np.array_equal(got[:, Nq + Nkv:].view(np.uint32), x[:, Nq + Nkv:].view(np.uint32))   # value heads: copied
        absmax_is_exact(K, am, out)
        # in place, without abs-max: the same tensor
        buf = xin.clone()
        fn(buf, buf, tab.cuda(), None, Nq, Nkv)
        assert torch.equal(buf.view(torch.int32), out.view(torch.int32))
        assert np.abs(got - want).max() <= 1e-5 * max(1.0, np.abs(want).max())


RMS_SHAPES = [(2, 3, 16), (1, 2, 64), (8, 64, 1024), (2, 5, 60), (1, 3, 256), (4, 8, 128), (1, 37, 3584), (1, 9, 896),
              (1, 5, 8192), (1, 4, 5120), (1, 1, 4), (3, 7, 24), (1, 300, 2048)]


def rms_inputs(O, N, C, seed):
    x1 = normal_f32(O, N * C, seed, 0, 0.0, 1.5).reshape(N, C)
    x2 = normal_f32(O, N * C, seed, 1, 0.0, 0.7).reshape(N, C)
    w = normal_f32(O, C, seed, 2, 1.0, 0.3)
    return x1, x2, w


@pytest.mark.parametrize("btc", RMS_SHAPES)
@pytest.mark.parametrize("fused", [False, True])
def test_rmsnorm_forward_f32_matches_oracle(K, O, btc, fused):
    B, T, C = btc
    N, eps = B * T, 1e-6
    x1, x2, w = rms_inputs(O, N, C, 600 + C)
    want, want_rrms, exact, res = O.rmsnorm_forward(x1, w, eps, x2 if fused else None)
    out = torch.full((B, T, C), float("nan"), dtype=torch.float32, device="cuda")
    rr = torch.full((B, T), float("nan"), dtype=torch.float32, device="cuda")
    am = slot()
    if fused:
        resid = torch.full((B, T, C), float("nan"), dtype=torch.float32, device="cuda")
        K.fused_residual_rmsnorm_forward(resid, out, rr, dev(x1).reshape(B, T, C), dev(x2).reshape(B, T, C), dev(w), am, eps)
        assert np.array_equal(host(resid).reshape(N, C).view(np.uint32), res.view(np.uint32))      # one fp32 add
        base = res
    else:
        K.rmsnorm_forward(out, rr, dev(x1).reshape(B, T, C), dev(w), am, eps)
        base = x1
    got, got_rr = host(out).reshape(N, C), host(rr).reshape(N)
    assert np.all(np.abs(got_rr.astype(np.float64) - want_rrms) <= np.abs(want_rrms) * 2.0 ** -18)
    assert np.all(np.abs(got.astype(np.float64) - exact) <= np.abs(exact) * 2.0 ** -17 + 1e-37)
    # the rounding chain itself, with the GPU's own 1/rms: fl(fl(s x) w), bit for bit
    chain = ((got_rr[:, None] * base).astype(np.float32) * w[None, :]).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), chain.view(np.uint32))
    absmax_is_exact(K, am, out)
    out2 = torch.empty_like(out)
    if fused:
        K.fused_residual_rmsnorm_forward(resid, out2, rr, dev(x1).reshape(B, T, C), dev(x2).reshape(B, T, C), dev(w), None, eps)
    else:
        K.rmsnorm_forward(out2, None, dev(x1).reshape(B, T, C), dev(w), None, eps)
    assert torch.equal(out.view(torch.int32), out2.view(torch.int32))


@pytest.mark.parametrize("btc", RMS_SHAPES)
def test_rmsnorm_backward_f32_matches_oracle(K, O, btc):
    B, T, C = btc
    N = B * T
    x, _, w = rms_inputs(O, N, C, 700 + C)
    d = normal_f32(O, N * C, 700 + C, 3, 0.0, 0.8).reshape(N, C)
    dres = normal_f32(O, N * C, 700 + C, 4, 0.0, 0.5).reshape(N, C)
    dw0 = normal_f32(O, C, 700 + C, 5, 0.0, 2.0)
    rstd = (1.0 / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1) + 1e-6)).astype(np.float32)
    want = O.rmsnorm_backward(dres, dw0, d, x, w, rstd)
    scratch = torch.empty(K.get_rmsnorm_backward_scratch_size(C), dtype=torch.float32, device="cuda")
    t3 = lambda a: dev(a).reshape(B, T, C)
    first = None
    for rep in range(3):
        dinp = torch.full((B, T, C), float("nan"), dtype=torch.float32, device="cuda")
        dweight = dev(dw0)
        am = slot()
        K.rmsnorm_backward(dinp, dweight, scratch, t3(dres), t3(d), t3(x), dev(w), dev(rstd).reshape(B, T), am)
        got, gw = host(dinp).reshape(N, C).astype(np.float64), host(dweight).astype(np.float64)
        if first is None:
            first = (got.copy(), gw.copy())
            assert np.all(np.abs(got - want["exact_dinp"]) <= np.abs(want["exact_dinp"]) * 2 * ULP + want["mag_dinp"] * 2.0 ** -18 + 1e-37)
            assert np.all(np.abs(gw - want["exact_dw"]) <= np.abs(want["exact_dw"]) * 2 * ULP + want["mag_dw"] * 2.0 ** -18 + 1e-37)
            absmax_is_exact(K, am, dinp)
        else:
            assert np.array_equal(got, first[0]) and np.array_equal(gw, first[1])      # fixed summation order
    # in place on dresidual, no abs-max: same dinp
    buf = t3(dres).clone()
    dweight = dev(dw0)
    K.rmsnorm_backward(buf, dweight, scratch, buf, t3(d), t3(x), dev(w), dev(rstd).reshape(B, T), None)
    assert np.array_equal(host(buf).reshape(N, C).astype(np.float64), first[0])


def test_rmsnorm_f32_argument_errors(K):
    f = lambda *s: torch.zeros(s, dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError, match="divisible by 4"):
        K.rmsnorm_forward(f(1, 1, 6), None, f(1, 1, 6), f(6), None, 1e-6)
    with pytest.raises(ValueError, match="8192"):
        K.rmsnorm_forward(f(1, 1, 8196), None, f(1, 1, 8196), f(8196), None, 1e-6)
    with pytest.raises(ValueError, match="dtype"):
        K.rmsnorm_forward(f(1, 1, 8), None, f(1, 1, 8), torch.zeros(8, dtype=torch.bfloat16, device="cuda"), None, 1e-6)
    with pytest.raises(ValueError, match="scratch"):
        K.rmsnorm_backward(f(1, 4, 64), f(64), torch.zeros(8, dtype=torch.float32, device="cuda"), f(1, 4, 64), f(1, 4, 64),
                           f(1, 4, 64), f(64), f(1, 4), None)
