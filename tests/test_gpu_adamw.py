"""GPU parity tests of the AdamW update with stochastic rounding (through the C ABI, llmq_amd.kernels).

Bar: BIT EXACT against the CPU oracle for the parameters, both moments and the abs-max: the hash is integer
arithmetic and every floating-point operation of the update is a correctly rounded IEEE operation on both
sides.  Plus the reference's own check (scripts/test_kernels.py:695-727, rtol 1e-2 / atol 5e-3 against the
torch formulas) and its abs-max convention (merged into the slot, not reset)."""
import numpy as np
import pytest
import torch

from gpu_util import dev_bf16, host_bits

pytestmark = pytest.mark.gpu
MOMENTS = [(torch.float32, torch.float32), (torch.bfloat16, torch.float32), (torch.bfloat16, torch.bfloat16)]


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from llmq_amd import kernels
    return kernels


def make(O, n, seed, m_dt, v_dt):
    rng = np.random.default_rng(seed)
    f = lambda a: O.f32_to_bf16(a.astype(np.float32))
    params, grads = f(rng.standard_normal(n) * 0.05), f(rng.standard_normal(n) * 2e-3)
    m0 = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    v0 = (rng.random(n) * 1e-5 + 1e-8).astype(np.float32)
    m = f(m0) if m_dt == torch.bfloat16 else m0
    v = f(v0) if v_dt == torch.bfloat16 else v0
    return params, grads, m, v


def to_dev(a):
    return dev_bf16(a) if a.dtype == np.uint16 else torch.from_numpy(a).cuda()


@pytest.mark.parametrize("m_dt,v_dt", MOMENTS)
@pytest.mark.parametrize("n", [8, 1024, 8192 + 8, 1 << 20])
def test_adamw_bit_exact(K, O, m_dt, v_dt, n):
    params, grads, m, v = make(O, n, 5 + n % 7, m_dt, v_dt)
    hp = dict(lr=3e-4, beta1=0.9, beta2=0.95, t=7, eps=1e-8, wd=0.1, gs=0.625, seed=0xC0FFEE + n)
    want_p, want_m, want_v, want_am = O.adamw_update(params, grads, m, v, hp["lr"], hp["beta1"], hp["beta2"], hp["t"],
                                                     hp["eps"], hp["wd"], hp["gs"], hp["seed"])
    dp, dg, dm, dv = to_dev(params), to_dev(grads), to_dev(m), to_dev(v)
    gs = torch.tensor([hp["gs"]], dtype=torch.float32, device="cuda")
    am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.adamw_update(dp, dg, dm, dv, hp["lr"], hp["beta1"], hp["beta2"], hp["t"], hp["eps"], hp["wd"], gs, None, am, hp["seed"])
    assert np.array_equal(host_bits(dp), want_p)
    got_m = host_bits(dm) if m_dt == torch.bfloat16 else dm.cpu().numpy().view(np.uint32)
    got_v = host_bits(dv) if v_dt == torch.bfloat16 else dv.cpu().numpy().view(np.uint32)
    assert np.array_equal(got_m, want_m if m_dt == torch.bfloat16 else want_m.view(np.uint32))
    assert np.array_equal(got_v, want_v if v_dt == torch.bfloat16 else want_v.view(np.uint32))
    assert am.cpu().numpy().view(np.uint32)[0] == np.float32(want_am).view(np.uint32)
    # without abs-max: the same tensors
    dp2, dm2, dv2 = to_dev(params), to_dev(m), to_dev(v)
    K.adamw_update(dp2, dg, dm2, dv2, hp["lr"], hp["beta1"], hp["beta2"], hp["t"], hp["eps"], hp["wd"], gs, None, None, hp["seed"])
    assert torch.equal(dp2.view(torch.int16), dp.view(torch.int16))
    # a different seed changes roundings but never moves a value by more than one bf16 step
    dp3, dm3, dv3 = to_dev(params), to_dev(m), to_dev(v)
    K.adamw_update(dp3, dg, dm3, dv3, hp["lr"], hp["beta1"], hp["beta2"], hp["t"], hp["eps"], hp["wd"], gs, None, None, hp["seed"] + 1)
    diff = (dp3.view(torch.int16).int() - dp.view(torch.int16).int()).abs()
    assert int(diff.max()) <= 1 and (n < 1024 or int((diff != 0).sum()) > 0)


def test_adamw_abs_max_is_merged_not_reset(K, O):
    """The slot keeps a larger value it already holds (src/kernels/adamw.cu has no reset: one slot can cover
    several calls) and equals abs_max() of the new parameters when it starts from zero."""
    n = 4096
    params, grads, m, v = make(O, n, 3, torch.float32, torch.float32)
    gs = torch.ones(1, dtype=torch.float32, device="cuda")
    for start in (0.0, 1e6):
        dp, dm, dv = to_dev(params), to_dev(m), to_dev(v)
        am = torch.full((1,), start, dtype=torch.float32, device="cuda")
        K.adamw_update(dp, to_dev(grads), dm, dv, 1e-3, 0.9, 0.999, 1, 1e-8, 0.0, gs, None, am, 1)
        ref = torch.zeros(1, dtype=torch.float32, device="cuda")
        K.abs_max(ref, dp)
        assert am.item() == max(start, ref.item())


@pytest.mark.parametrize("m_dt,v_dt", MOMENTS)
def test_adamw_reference_test_construction(K, m_dt, v_dt):
    N = 65536
    g = torch.Generator(device="cuda").manual_seed(0)
    r = lambda: torch.randn((N,), device="cuda", dtype=torch.float32, generator=g)
    params, grads = r().to(torch.bfloat16), r().to(torch.bfloat16)
    m = (r() * 0.1).to(m_dt)
    v = (torch.rand((N,), device="cuda", generator=g) * 0.01 + 1e-8).to(v_dt)
    g_scale = torch.rand((1,), device="cuda", generator=g) * 0.5 + 0.5
    lr, beta1, beta2, t, eps, wd = 1e-3, 0.9, 0.999, 1, 1e-8, 0.1
    gf = grads.float() * g_scale
    m_new = beta1 * m.float() + (1 - beta1) * gf
    v_new = beta2 * v.float() + (1 - beta2) * gf ** 2
    p_new = params.float() * (1 - lr * wd) - lr * (m_new / (1 - beta1 ** t)) / ((v_new / (1 - beta2 ** t)).sqrt() + eps)
    K.adamw_update(params, grads, m, v, lr, beta1, beta2, t, eps, wd, g_scale)
    assert torch.allclose(params.float(), p_new, rtol=1e-2, atol=5e-3)
    tol = lambda dt: (1e-2, 5e-3) if dt == torch.bfloat16 else (5e-4, 5e-5)
    assert torch.allclose(m.float(), m_new, rtol=tol(m_dt)[0], atol=tol(m_dt)[1])
    assert torch.allclose(v.float(), v_new, rtol=tol(v_dt)[0], atol=tol(v_dt)[1])


def test_adamw_argument_errors(K):
    z = lambda n, dt=torch.bfloat16: torch.zeros(n, dtype=dt, device="cuda")
    gs = torch.ones(1, dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError, match="divisible by 8"):
        K.adamw_update(z(12), z(12), z(12), z(12), 1e-3, 0.9, 0.99, 1, 1e-8, 0.0, gs)
    with pytest.raises(ValueError, match="moment types"):
        K.adamw_update(z(16), z(16), z(16, torch.float32), z(16), 1e-3, 0.9, 0.99, 1, 1e-8, 0.0, gs)
    with pytest.raises(ValueError, match="shape mismatch"):
        K.adamw_update(z(16), z(8), z(16), z(16), 1e-3, 0.9, 0.99, 1, 1e-8, 0.0, gs)


# ------------------------------------------------------------------ e4m3 first moment with block scales
def make_fp8m(O, n, seed):
    rng = np.random.default_rng(seed)
    f = lambda a: O.f32_to_bf16(a.astype(np.float32))
    params, grads = f(rng.standard_normal(n) * 0.05), f(rng.standard_normal(n) * 2e-3)
    v = f(rng.random(n) * 1e-5 + 1e-8)
    m = rng.integers(0, 256, n).astype(np.uint8)
    m[(m & 0x7F) == 0x7F] ^= 1
    nb = (n + 127) // 128
    scales = (10.0 ** rng.uniform(-6, -2, nb)).astype(np.float32)
    if nb > 2:                      # a block that stays exactly zero (scale 1 path) and one with a tiny moment
        m[128:256] = 0
        grads[128:256] = 0
        scales[2] = 1e-30
    return params, grads, m, scales, v


@pytest.mark.parametrize("n", [8, 128, 1000, 8192 + 72, 1 << 20])
def test_adamw_fp8_first_moment_bit_exact(K, O, n):
    """adamw_update with an e4m3 first moment and one scale per 128 elements (src/kernels/kernels.h:237-239,
    adamw.cu:22-66): parameters, codes, scales, second moment and abs-max bit exact against the oracle, including
    a last block shorter than 128, an all-zero block and a vanishing one."""
    params, grads, m, scales, v = make_fp8m(O, n, 11 + n % 5)
    hp = dict(lr=3e-4, beta1=0.9, beta2=0.95, t=5, eps=1e-8, wd=0.1, gs=0.625, seed=0xBEEF + n)
    wp, wm, ws, wv, wam = O.adamw_update_fp8m(params, grads, m, scales, v, hp["lr"], hp["beta1"], hp["beta2"], hp["t"],
                                              hp["eps"], hp["wd"], hp["gs"], hp["seed"])
    dp, dg, dv = dev_bf16(params), dev_bf16(grads), dev_bf16(v)
    dm, ds = torch.from_numpy(m).cuda(), torch.from_numpy(scales).cuda()
    gs = torch.tensor([hp["gs"]], dtype=torch.float32, device="cuda")
    am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.adamw_update(dp, dg, dm, dv, hp["lr"], hp["beta1"], hp["beta2"], hp["t"], hp["eps"], hp["wd"], gs, ds, am, hp["seed"])
    assert np.array_equal(host_bits(dp), wp) and np.array_equal(host_bits(dv), wv)
    assert np.array_equal(ds.cpu().numpy().view(np.uint32), ws.view(np.uint32))
    assert np.array_equal(dm.cpu().numpy(), wm)
    assert am.cpu().numpy().view(np.uint32)[0] == np.float32(wam).view(np.uint32)
    # the stored moment dequantizes to within one e4m3 step (2^-3 relative) of the exact new moment
    if n >= 1024:
        dec = O.e4m3_table()
        got = dec[wm].astype(np.float64) * np.repeat(ws, 128)[:n]
        m_old = dec[m].astype(np.float64) * np.repeat(scales, 128)[:n]
        g = O.bf16_to_f32(grads).astype(np.float64) * hp["gs"]
        exact = hp["beta1"] * m_old + (1 - hp["beta1"]) * g
        blk = np.repeat(ws.astype(np.float64) * 448, 128)[:n]              # block abs-max
        assert np.all(np.abs(got - exact) <= 0.126 * np.abs(exact) + blk * 2.0 ** -9 + 1e-30)


def test_adamw_golden_known_answers(K):
    """The library against the numpy / exact-rational vectors of tests/golden/adamw_kat.npz: pins the hash bits,
    rotations, thresholds and block scales with no oracle in the loop."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "adamw_kat.npz"), allow_pickle=False)
    lr, b1, b2, t, eps, wd, gsv, seed = (float(x) for x in g["step_hyper"])
    gs = torch.tensor([gsv], dtype=torch.float32, device="cuda")
    dp, dg, dm, dv = dev_bf16(g["step_p"]), dev_bf16(g["step_g"]), dev_bf16(g["bf16_m"]), dev_bf16(g["step_v"])
    K.adamw_update(dp, dg, dm, dv, lr, b1, b2, int(t), eps, wd, gs, None, None, int(seed))
    assert np.array_equal(host_bits(dp), g["bf16_p_out"]) and np.array_equal(host_bits(dm), g["bf16_m_out"])
    assert np.array_equal(host_bits(dv), g["bf16_v_out"])
    dp, dg, dv = dev_bf16(g["step_p"]), dev_bf16(g["fp8_g"]), dev_bf16(g["step_v"])
    dm, ds = torch.from_numpy(g["fp8_m"]).cuda(), torch.from_numpy(g["fp8_scales"]).cuda()
    K.adamw_update(dp, dg, dm, dv, lr, b1, b2, int(t), eps, wd, gs, ds, None, int(seed))
    assert np.array_equal(host_bits(dp), g["fp8_p_out"]) and np.array_equal(host_bits(dv), g["fp8_v_out"])
    assert np.array_equal(ds.cpu().numpy().view(np.uint32), g["fp8_scales_out"].view(np.uint32))
    assert np.array_equal(dm.cpu().numpy(), g["fp8_m_out"])


@pytest.mark.parametrize("n", [4, 1020, 8192 + 4, 1 << 20])
def test_adamw_fp32_parameters_bit_exact(K, O, n):
    """The all-fp32 overload (src/kernels/kernels.h:221-223): nothing is rounded stochastically, every operation is a
    correctly rounded fp32 one -> parameters, moments and abs-max equal the oracle's bit for bit, whatever the seed;
    the abs-max is merged into the slot; the reference's own check (rtol 1e-2 / atol 5e-3 against the float64
    formulas, scripts/test_kernels.py:695-727) holds as well."""
    rng = np.random.default_rng(n)
    params, grads = (rng.standard_normal(n) * 0.05).astype(np.float32), (rng.standard_normal(n) * 2e-3).astype(np.float32)
    m, v = (rng.standard_normal(n) * 1e-3).astype(np.float32), (rng.random(n) * 1e-5 + 1e-8).astype(np.float32)
    lr, b1, b2, t, eps, wd, gsv = 3e-4, 0.9, 0.95, 7, 1e-8, 0.1, 0.625
    want_p, want_m, want_v, want_am = O.adamw_update(params, grads, m, v, lr, b1, b2, t, eps, wd, gsv, 0)
    gs = torch.tensor([gsv], dtype=torch.float32, device="cuda")
    for seed in (0, 12345):
        dp, dg, dm, dv = (torch.from_numpy(a.copy()).cuda() for a in (params, grads, m, v))
        am = torch.zeros(1, dtype=torch.float32, device="cuda")
        K.adamw_update(dp, dg, dm, dv, lr, b1, b2, t, eps, wd, gs, None, am, seed)
        for got, want in ((dp, want_p), (dm, want_m), (dv, want_v)):
            assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
        assert am.cpu().numpy().view(np.uint32)[0] == np.float32(want_am).view(np.uint32)
    big = torch.full((1,), 1e6, dtype=torch.float32, device="cuda")
    dp, dg, dm, dv = (torch.from_numpy(a.copy()).cuda() for a in (params, grads, m, v))
    K.adamw_update(dp, dg, dm, dv, lr, b1, b2, t, eps, wd, gs, None, big, 0)
    assert big.item() == 1e6                                                      # merged, not reset
    g64, p64 = grads.astype(np.float64) * gsv, params.astype(np.float64)
    m_new = b1 * m.astype(np.float64) + (1 - b1) * g64
    v_new = b2 * v.astype(np.float64) + (1 - b2) * g64 ** 2
    p_new = p64 * (1 - lr * wd) - lr * (m_new / (1 - b1 ** t)) / (np.sqrt(v_new / (1 - b2 ** t)) + eps)
    assert np.allclose(want_p, p_new, rtol=1e-2, atol=5e-3) and np.allclose(want_p, p_new, rtol=1e-5, atol=1e-9)
    with pytest.raises(ValueError, match="divisible by 4"):
        f = lambda: torch.zeros(6, dtype=torch.float32, device="cuda")
        K.adamw_update(f(), f(), f(), f(), lr, b1, b2, t, eps, wd, gs, None, None, 0)
