"""The CPU oracle against the committed fixtures of tests/golden/ (written by tests/golden/make_golden.py
from the formats' and formulas' definitions, with numpy alone and by other methods than the oracle's).
The same fixtures are what tests/test_gpu_golden.py holds the HIP library to."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ALL_BF16 = np.arange(65536, dtype=np.uint32).astype(np.uint16)


def load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def bf16_value(bits):
    return (np.asarray(bits).astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def within_bf16_rounding(bits, exact, slack):
    """|value(bits) - exact| <= half a bf16 ulp of the exact value (at most 2^-8 relative) + slack (the fp32
    evaluation error of the producer, given by the caller as an absolute array or number)."""
    err = np.abs(bf16_value(bits) - exact)
    return bool(np.all(err <= 2.0 ** -8 * np.abs(exact) + slack))


def test_fixture_files_are_present():
    for f in ("fp8_encode.npz", "gemm_kat.npz", "producers.npz", "adamw_kat.npz", "make_golden.py"):
        assert os.path.exists(os.path.join(GOLDEN, f)), f


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_quantize_all_bf16_patterns(O, fmt):
    g = load("fp8_encode.npz")
    for i, absmax in enumerate(g["absmax"]):
        s, d = O.quant_scale(float(absmax))
        assert np.float32(s).view(np.uint32) == g["scale_bits"][i] and np.float32(d).view(np.uint32) == g["recip_bits"][i]
        got, recip = O.quantize_e4m3(ALL_BF16, float(absmax), fmt=fmt)
        assert np.array_equal(got, g[fmt][i]), (fmt, float(absmax), np.nonzero(got != g[fmt][i])[0][:8])
        assert np.float32(recip).view(np.uint32) == g["recip_bits"][i]
        got_mt, _ = O.quantize_e4m3(ALL_BF16, float(absmax), fmt=fmt, mt=True) if fmt == "e4m3" else (got, None)
        assert np.array_equal(got_mt, g[fmt][i])


def test_gemm_integer_known_answer(O):
    g = load("gemm_kat.npz")
    sa, sb = float(g["int_sa"]), float(g["int_sb"])
    for mt in (False, True):
        c16 = O.gemm_tn(g["int_a"], g["int_b"], sa, sb, bias=g["int_bias_bf16"], mt=mt)
        assert np.array_equal(c16, g["int_c_bf16"])
        c32 = O.gemm_tn(g["int_a"], g["int_b"], sa, sb, bias=g["int_bias_bf16"], out_f32=True, mt=mt)
        assert np.array_equal(c32.view(np.uint32), g["int_c_f32"].view(np.uint32))


def test_gemm_random_codes(O):
    g = load("gemm_kat.npz")
    ex, sumabs = O.gemm_exact(g["rnd_a"], g["rnd_b"])
    assert np.array_equal(ex, g["rnd_exact"]) and np.array_equal(sumabs, g["rnd_sumabs"])
    sa, sb = np.float32(g["rnd_sa"]), np.float32(g["rnd_sb"])
    ref = g["rnd_exact"] * float(np.float32(sa * sb))
    c32 = O.gemm_tn(g["rnd_a"], g["rnd_b"], float(sa), float(sb), out_f32=True)
    assert np.all(np.abs(c32 - ref) <= 2.0 ** -22 * float(sa * sb) * g["rnd_sumabs"] + 2.0 ** -23 * np.abs(ref))
    c16 = O.gemm_tn(g["rnd_a"], g["rnd_b"], float(sa), float(sb))
    assert within_bf16_rounding(c16, ref, 2.0 ** -20 * float(sa * sb) * g["rnd_sumabs"])


def test_swiglu(O):
    g = load("producers.npz")
    out, exact = O.swiglu_forward(g["swiglu_inp"])
    assert np.allclose(exact, g["swiglu_out"], rtol=1e-12, atol=1e-300)
    assert within_bf16_rounding(out, g["swiglu_out"], 0.0)
    dinp, exact_d = O.swiglu_backward(g["swiglu_dout"], g["swiglu_inp"])
    assert np.allclose(exact_d, g["swiglu_dinp"], rtol=1e-12, atol=1e-300)
    assert within_bf16_rounding(dinp, g["swiglu_dinp"], 0.0)


def test_rmsnorm_forward(O):
    g = load("producers.npz")
    eps = float(g["rms_eps"])
    normed, rrms, _, _ = O.rmsnorm_forward(g["rms_inp1"], g["rms_weight"], eps)
    assert np.allclose(rrms, g["rms_rstd"], rtol=2e-6)
    # the reference rounds s * x to bf16 before the multiplication with the weight (src/kernels/rmsnorm.cu:68-71):
    # two roundings, hence a second half ulp
    two = lambda exact: (2.0 ** -8 * 1.01 + 4e-6) * np.abs(exact)
    assert within_bf16_rounding(normed, g["rms_out"], two(g["rms_out"]))
    normed, rrms, _, res = O.rmsnorm_forward(g["rms_inp1"], g["rms_weight"], eps, inp2=g["rms_inp2"])
    assert np.array_equal(res, g["rms_residual"])
    assert np.allclose(rrms, g["rms_fused_rstd"], rtol=2e-6)
    assert within_bf16_rounding(normed, g["rms_fused_out"], two(g["rms_fused_out"]))


def test_rope(O):
    g = load("producers.npz")
    B, T, Nq, Nkv, HD = (int(v) for v in g["rope_dims"])
    qkv = g["rope_qkv"].reshape(B * T, Nq + 2 * Nkv, HD)
    for backward, key in ((False, "rope_forward"), (True, "rope_backward")):
        out, _, mag = O.rope(qkv, g["rope_table_f16"], T, Nq, Nkv, backward=backward)
        want = g[key].reshape(out.shape)
        assert within_bf16_rounding(out, want, 2.0 ** -22 * mag)
        assert np.array_equal(out[:, Nq + Nkv:], qkv[:, Nq + Nkv:])      # value heads: copied bit for bit


def test_adamw_hash_and_stochastic_rounding_known_answers(O):
    """SquirrelNoise5 and the stochastic roundings against vectors written with Python integers
    (src/kernels/squirrel_noise.cuh:15-75)."""
    g = load("adamw_kat.npz")
    L = O.lib()
    for pos, seed, want in zip(g["hash_position"], g["hash_seed"], g["hash_value"]):
        assert L.orc_squirrel_noise_5(int(pos), int(seed)) == int(want)
    vals = g["sr_pattern"].view(np.float32)
    for x, r, w16, w8 in zip(vals, g["sr_random"], g["sr_bf16"], g["sr_e4m3"]):
        assert L.orc_stochastic_round_bf16(float(x), int(r)) == int(w16), (x, r)
        assert L.orc_stochastic_round_e4m3(float(x), int(r)) == int(w8), (x, r)


def test_adamw_whole_step_known_answers(O):
    """One AdamW step on 384 parameters, bf16 / bf16 moments and e4m3 first moment with block scales, against the
    exact-rational evaluation of tests/golden/make_golden.py (src/kernels/adamw.cu:22-113)."""
    g = load("adamw_kat.npz")
    lr, b1, b2, t, eps, wd, gs, seed = g["step_hyper"]
    p, m, v, _ = O.adamw_update(g["step_p"], g["step_g"], g["bf16_m"], g["step_v"], lr, b1, b2, int(t), eps, wd, gs, int(seed))
    assert np.array_equal(p, g["bf16_p_out"]) and np.array_equal(m, g["bf16_m_out"]) and np.array_equal(v, g["bf16_v_out"])
    p, mc, ms, v, _ = O.adamw_update_fp8m(g["step_p"], g["fp8_g"], g["fp8_m"], g["fp8_scales"], g["step_v"], lr, b1, b2, int(t),
                                          eps, wd, gs, int(seed))
    assert np.array_equal(p, g["fp8_p_out"]) and np.array_equal(v, g["fp8_v_out"])
    assert np.array_equal(ms.view(np.uint32), g["fp8_scales_out"].view(np.uint32))
    assert np.array_equal(mc, g["fp8_m_out"])
