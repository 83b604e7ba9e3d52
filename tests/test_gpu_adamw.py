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
