"""Pins the CPU oracle against evidence that does not come from the oracle itself: the OCP e4m3
format definition (nearest-code search), torch's CPU float8 casts, numpy float32/int64/float64
arithmetic, and the constructions the reference's own tests use (src/testing/test-gemm.cpp:54-85,
scripts/test_kernels.py:40-65,641-652,1168-1185 in the reference tree)."""
import numpy as np
import pytest
import torch

ALL_BF16 = np.arange(65536, dtype=np.uint32).astype(np.uint16)


# ------------------------------------------------------------------ independent e4m3 definitions
def e4m3_value_of_code(c):
    """OCP FP8 E4M3 ("fn") value of a 7-bit magnitude code, from the format definition."""
    e, m = c >> 3, c & 7
    if e == 0:
        return m * 2.0 ** -9
    return (8 + m) * 2.0 ** (e - 10)


def e4m3_encode_search(y):
    """Nearest-of-127-finite-codes search in float64 with ties to the even code, saturating."""
    y = np.asarray(y, dtype=np.float32)
    vals = np.array([e4m3_value_of_code(c) for c in range(0x7F)], dtype=np.float64)  # 0 .. 448
    a = np.abs(y.astype(np.float64))
    hi = np.searchsorted(vals, a, side="left")            # first code with value >= a
    hi = np.clip(hi, 0, 0x7E)
    lo = np.clip(hi - 1, 0, 0x7E)
    dlo, dhi = np.abs(a - vals[lo]), np.abs(vals[hi] - a)
    code = np.where(dlo < dhi, lo, np.where(dhi < dlo, hi, np.where(lo % 2 == 0, lo, hi)))
    code = np.where(a >= 448.0, 0x7E, code)                # saturate-to-finite (Inf included)
    sign = (y.view(np.uint32) >> 31).astype(np.uint8) << 7
    out = (code.astype(np.uint8) | sign).astype(np.uint8)
    out[np.isnan(y)] = 0x7F                                # canonical NaN, sign dropped
    return out


def oracle_encode(O, y):
    y = np.ascontiguousarray(y, dtype=np.float32)
    L = O.lib()
    return np.array([L.orc_e4m3_encode(float(v)) if not np.isnan(v) else L.orc_e4m3_encode(float("nan"))
                     for v in y], dtype=np.uint8)


def encode_via_quantize(O, bits, absmax):
    """Vectorised route into the oracle's encoder: quantize bf16 patterns with a given abs-max."""
    q, _ = O.quantize_e4m3(bits, absmax)
    return q


# ------------------------------------------------------------------------------------ bf16 helpers
def test_bf16_roundtrip_matches_torch(O):
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-30, 30, 20000),
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf], np.float32)])
    ours = O.f32_to_bf16(x)
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours, ref)
    L = O.lib()
    for v in x[:2000]:
        assert L.orc_f32_to_bf16(float(v)) == int(torch.tensor(float(v)).to(torch.bfloat16).view(torch.int16)) & 0xFFFF
    assert np.array_equal(O.bf16_to_f32(ours), torch.from_numpy(ours.view(np.int16)).view(torch.bfloat16).float().numpy())


# ---------------------------------------------------------------------------------------- abs-max
def test_abs_max_matches_numpy(O):
    # shapes of scripts/test_kernels.py:56-65 plus larger ones
    for shape, seed in [((16, 64), 0), ((4, 128, 32), 1), ((1000, 8), 2), ((1 << 18,), 3)]:
        x = O.fill_normal_bf16(int(np.prod(shape)), seed, 7, 0.0, 3.0)
        assert O.abs_max_bf16(x) == np.abs(O.bf16_to_f32(x)).max()
        assert O.lib().mt_abs_max_bf16(x.ctypes.data_as(__import__("ctypes").POINTER(__import__("ctypes").c_uint16)), x.size) \
            == O.abs_max_bf16(x)


def test_abs_max_special_values(O):
    nan, snan, ninf, nzero = 0x7FC0, 0x7F81, 0xFF80, 0x8000
    assert O.abs_max_bf16(np.array([nan, snan, 0xFFC1], np.uint16)) == 0.0          # all NaN -> 0
    assert O.abs_max_bf16(np.array([nzero] * 8, np.uint16)) == 0.0
    assert np.signbit(np.float32(O.abs_max_bf16(np.array([nzero] * 8, np.uint16)))) == False  # noqa: E712
    assert O.abs_max_bf16(np.array([0x3F80, nan, 0xC000, snan], np.uint16)) == 2.0  # NaN skipped
    assert O.abs_max_bf16(np.array([0x3F80, ninf, nan], np.uint16)) == np.inf       # |-Inf| wins
    assert O.abs_max_bf16(np.array([0x0001, 0x8003], np.uint16)) == O.bf16_to_f32(np.array([3], np.uint16))[0]  # denormals kept
    assert O.abs_max_bf16(np.zeros(0, np.uint16)) == 0.0


# ------------------------------------------------------------------------------------ e4m3 encode
def test_e4m3_decode_matches_definition_and_torch(O):
    tab = O.e4m3_table()
    for c in range(0x7F):
        assert tab[c] == np.float32(e4m3_value_of_code(c))
        assert tab[c | 0x80] == -np.float32(e4m3_value_of_code(c))
    assert np.isnan(tab[0x7F]) and np.isnan(tab[0xFF])
    t = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.nan_to_num(t, nan=12345.0), np.nan_to_num(tab, nan=12345.0))
    assert np.array_equal(np.signbit(t), np.signbit(tab))


def test_e4m3_encode_boundaries_closed_form(O):
    L = O.lib()
    enc = L.orc_e4m3_encode
    assert enc(0.0) == 0x00 and enc(-0.0) == 0x80
    assert enc(2.0 ** -10) == 0x00 and enc(-(2.0 ** -10)) == 0x80            # tie to even (zero)
    assert enc(float(np.nextafter(np.float32(2.0 ** -10), np.float32(1)))) == 0x01
    assert enc(2.0 ** -9) == 0x01 and enc(3 * 2.0 ** -10) == 0x02            # tie 1.5 ulp -> even (2)
    assert enc(7.5 * 2.0 ** -9) == 0x08                                      # tie rounds up into the normals
    assert enc(2.0 ** -6) == 0x08
    assert enc(448.0) == 0x7E and enc(464.0) == 0x7E and enc(-464.0) == 0xFE
    assert enc(float(np.nextafter(np.float32(464), np.float32(1e9)))) == 0x7E  # saturates
    assert enc(1e30) == 0x7E and enc(float("inf")) == 0x7E and enc(float("-inf")) == 0xFE
    assert enc(float("nan")) == 0x7F
    assert enc(float(np.uint32(0xFFC00000).view(np.float32))) == 0x7F        # -NaN: sign dropped
    assert enc(1.0) == 0x38 and enc(-1.0) == 0xB8 and enc(1.0625) == 0x38 and enc(1.1875) == 0x3A
    assert enc(1e-45) == 0x00 and enc(-1e-45) == 0x80                        # fp32 denormal underflows


@pytest.mark.parametrize("absmax", [448.0, 1.0, 5.15625, 0.072265625, 3.0e-5, 1e4, 0.0, 447.0, 1.7e38])
def test_e4m3_encode_exhaustive_bf16_vs_search_and_torch(O, absmax):
    """All 65536 bf16 inputs through scale*x, against the nearest-code search and torch's cast."""
    s, d = O.quant_scale(absmax)
    s32 = np.float32(s)
    assert s32 == np.float32(448.0) / max(np.float32(absmax), np.float32(1e-10))
    assert np.float32(d) == np.float32(1.0) / s32
    with np.errstate(over="ignore", invalid="ignore"):
        y = (s32 * O.bf16_to_f32(ALL_BF16)).astype(np.float32)
    got = encode_via_quantize(O, ALL_BF16, absmax)
    want = e4m3_encode_search(y)
    assert np.array_equal(got, want)
    # third opinion: torch's float8_e4m3fn cast (which does not saturate, hence the clamp)
    finite = ~np.isnan(y)
    t = torch.from_numpy(y[finite]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(got[finite], t)
    assert np.all(got[~finite] == 0x7F)
    # the multithreaded port agrees bit for bit
    got_mt, d_mt = O.quantize_e4m3(ALL_BF16, absmax, mt=True)
    assert np.array_equal(got_mt, got) and d_mt == np.float32(d)


def test_e4m3_encode_fp32_grid_vs_search(O):
    """Dense fp32 probes around every rounding boundary (midpoints between codes, +-1 ulp)."""
    vals = np.array([e4m3_value_of_code(c) for c in range(0x7F)], dtype=np.float64)
    mids = ((vals[1:] + vals[:-1]) / 2).astype(np.float32)
    pts = np.concatenate([mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9)),
                          vals.astype(np.float32), np.array([464, 465, 480, 1e9, 2.0 ** -10, 2.0 ** -11], np.float32)])
    pts = np.concatenate([pts, -pts])
    rng = np.random.default_rng(5)
    rnd = (rng.standard_normal(20000) * 10.0 ** rng.uniform(-4, 3, 20000)).astype(np.float32)
    pts = np.concatenate([pts, rnd])
    assert np.array_equal(oracle_encode(O, pts), e4m3_encode_search(pts))


def test_quantize_reference_style_checks(O):
    # scripts/test_kernels.py:641-652: scale ~= absmax/448, dequantised values within 10 %
    for n, seed in [(1024, 0), (8192, 1)]:
        x = O.fill_normal_bf16(n, seed, 3)
        am = O.abs_max_bf16(x)
        q, d = O.quantize_e4m3(x, am)
        assert d == pytest.approx(am / 448.0, rel=1e-6)
        deq = O.e4m3_decode(q) * d
        xf = O.bf16_to_f32(x)
        big = np.abs(xf) > am * 2.0 ** -6 / 448 * 8
        assert np.allclose(deq[big], xf[big], rtol=0.1)


def test_zero_tensor_quantize(O):
    x = np.array([0x0000, 0x8000] * 8, np.uint16)
    q, d = O.quantize_e4m3(x, 0.0)
    assert list(q[:2]) == [0x00, 0x80]
    s, _ = O.quant_scale(0.0)
    assert np.float32(s) == np.float32(448.0) / np.float32(1e-10)


# -------------------------------------------------------------------------- transpose / q+transpose
@pytest.mark.parametrize("shape", [(32, 32), (128, 256), (512, 1024), (8, 40), (72, 8)])
def test_transpose_and_quantize_transpose(O, shape):
    rows, cols = shape
    x = O.fill_normal_bf16(rows * cols, 11, rows, 0.0, 2.0).reshape(rows, cols)
    am = O.abs_max_bf16(x)
    q, d = O.quantize_e4m3(x, am)
    assert np.array_equal(O.transpose_u8(q), q.T)
    assert np.array_equal(O.transpose_u8(q, mt=True), q.T)
    qt, dt = O.quantize_transpose_e4m3(x, am)
    assert np.array_equal(qt, q.T) and dt == d
    qt2, _ = O.quantize_transpose_e4m3(x, am, mt=True)
    assert np.array_equal(qt2, q.T)


# ------------------------------------------------------------------------------------------- GEMM
@pytest.mark.parametrize("mnk,scale", [((128, 128, 128), 4.0 / 128), ((128, 96, 768), 4.0 / 768)])
def test_gemm_integer_known_answer(O, mnk, scale):
    """The construction of src/testing/test-gemm.cpp: integers in [-15,15] are exact in e4m3, every
    partial sum stays below 2^24, so the product is an exact integer matrix: numpy int64 is the truth."""
    M, N, K = mnk
    a, av = O.fill_int_e4m3(M * K, 12345, 0)
    b, bv = O.fill_int_e4m3(N * K, 12345, 1)
    a, av, b, bv = a.reshape(M, K), av.reshape(M, K), b.reshape(N, K), bv.reshape(N, K)
    assert np.array_equal(O.e4m3_decode(a), av.astype(np.float32))
    truth = bv.astype(np.int64) @ av.astype(np.int64).T          # [N, M]
    ex, sabs = O.gemm_exact(a, b)
    assert np.array_equal(ex, truth.astype(np.float64))
    assert np.array_equal(sabs, (np.abs(bv).astype(np.int64) @ np.abs(av).astype(np.int64).T).astype(np.float64))
    s = np.float32(np.sqrt(np.float32(scale)))
    ss = np.float32(s * s)
    c = O.gemm_tn(a, b, sa=float(s), sb=float(s), out_f32=True)
    assert np.array_equal(c, truth.astype(np.float32) * ss)
    cb = O.gemm_tn(a, b, sa=float(s), sb=float(s))
    assert np.array_equal(cb, O.f32_to_bf16(truth.astype(np.float32) * ss))
    # bias and accumulate (fp32 adds, single rounding)
    _, biasv = O.fill_int_e4m3(M, 12345, 2)
    _, oldv = O.fill_int_e4m3(N * M, 12345, 3)
    bias = O.f32_to_bf16(biasv.astype(np.float32))
    old = O.f32_to_bf16(oldv.astype(np.float32)).reshape(N, M)
    want = ((truth.astype(np.float32) * ss) + biasv.astype(np.float32)[None, :]) + oldv.reshape(N, M).astype(np.float32)
    got = O.gemm_tn(a, b, sa=float(s), sb=float(s), bias=bias, c_old=old)
    assert np.array_equal(got, O.f32_to_bf16(want))
    # the reference's own acceptance test (test-gemm.cpp:114-148): rel 1e-2 against the fp32 product
    exp = truth.astype(np.float32) * s * s
    assert np.all(np.abs(O.bf16_to_f32(cb) - exp) <= np.maximum(1e-2 * np.maximum(np.abs(exp), np.abs(O.bf16_to_f32(cb))), 1e-4))
    # multithreaded port: exact here too (integer sums are order independent)
    if M % 64 == 0 and N % 4 == 0:
        assert np.array_equal(O.gemm_tn(a, b, sa=float(s), sb=float(s), mt=True), cb)
        assert np.array_equal(O.gemm_tn(a, b, sa=float(s), sb=float(s), bias=bias, c_old=old, mt=True), got)


# ------------------------------------------------------------------ e5m2 (gradient dtype), same evidence
def e5m2_value_of_code(c):
    """IEEE-like binary8 E5M2 value of a 7-bit magnitude code below the Inf/NaN block (c < 0x7C)."""
    e, m = c >> 2, c & 3
    if e == 0:
        return m * 2.0 ** -16
    return (4 + m) * 2.0 ** (e - 17)


def e5m2_encode_search(y):
    y = np.asarray(y, dtype=np.float32)
    vals = np.array([e5m2_value_of_code(c) for c in range(0x7C)], dtype=np.float64)   # 0 .. 57344
    a = np.abs(y.astype(np.float64))
    hi = np.clip(np.searchsorted(vals, a, side="left"), 0, 0x7B)
    lo = np.clip(hi - 1, 0, 0x7B)
    dlo, dhi = np.abs(a - vals[lo]), np.abs(vals[hi] - a)
    code = np.where(dlo < dhi, lo, np.where(dhi < dlo, hi, np.where(lo % 2 == 0, lo, hi)))
    code = np.where(a >= 57344.0, 0x7B, code)
    sign = (y.view(np.uint32) >> 31).astype(np.uint8) << 7
    out = (code.astype(np.uint8) | sign).astype(np.uint8)
    out[np.isnan(y)] = 0x7F
    return out


def test_e5m2_decode_matches_definition_and_torch(O):
    tab = O.e5m2_table()
    for c in range(0x7C):
        assert tab[c] == np.float32(e5m2_value_of_code(c)) and tab[c | 0x80] == -np.float32(e5m2_value_of_code(c))
    assert np.isinf(tab[0x7C]) and np.isinf(tab[0xFC]) and np.all(np.isnan(tab[[0x7D, 0x7E, 0x7F, 0xFD, 0xFE, 0xFF]]))
    t = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(torch.float8_e5m2).float().numpy()
    assert np.array_equal(np.nan_to_num(t, nan=12345.0), np.nan_to_num(tab, nan=12345.0))


@pytest.mark.parametrize("absmax", [448.0, 1.0, 5.15625, 3.0e-5, 1e4, 0.0, 2.0 ** -7])
def test_e5m2_encode_exhaustive_bf16_vs_search_and_torch(O, absmax):
    """All 65536 bf16 inputs through the reference's 448-based scale (quant.cu:79 serves both fp8 output
    types) into e5m2, against the nearest-code search and torch's float8_e5m2 cast."""
    s, _ = O.quant_scale(absmax)
    with np.errstate(over="ignore", invalid="ignore"):
        y = (np.float32(s) * O.bf16_to_f32(ALL_BF16)).astype(np.float32)
    got, _ = O.quantize_e4m3(ALL_BF16, absmax, fmt="e5m2")
    assert np.array_equal(got, e5m2_encode_search(y))
    finite = ~np.isnan(y)
    t = torch.from_numpy(y[finite]).clamp(-57344.0, 57344.0).to(torch.float8_e5m2).view(torch.uint8).numpy()
    assert np.array_equal(got[finite], t)
    assert np.all(got[~finite] == 0x7F)


def test_e5m2_encode_boundaries_closed_form(O):
    enc = O.lib().orc_e5m2_encode
    assert enc(0.0) == 0x00 and enc(-0.0) == 0x80 and enc(1.0) == 0x3C and enc(-1.0) == 0xBC
    assert enc(2.0 ** -17) == 0x00 and enc(float(np.nextafter(np.float32(2.0 ** -17), np.float32(1)))) == 0x01
    assert enc(1.125) == 0x3C and enc(1.375) == 0x3E                          # ties to even
    assert enc(57344.0) == 0x7B and enc(61439.0) == 0x7B and enc(61440.0) == 0x7B and enc(1e30) == 0x7B
    assert enc(float("inf")) == 0x7B and enc(float("-inf")) == 0xFB and enc(float("nan")) == 0x7F


def test_gemm_e5m2_b_operand_vs_float64_matmul(O):
    """a e4m3, b e5m2 (src/kernels/kernels.h:92-94): every product is exact in fp64 (4 x 3 significand
    bits), so the oracle must equal numpy's float64 matmul of the decoded operands."""
    rng = np.random.default_rng(8)
    M, N, K = 64, 40, 384
    a = rng.integers(0, 256, (M, K)).astype(np.uint8)
    b = rng.integers(0, 256, (N, K)).astype(np.uint8)
    a[(a & 0x7F) == 0x7F] = 0x7E
    b[(b & 0x7C) == 0x7C] = 0x70                                                 # no Inf / NaN codes
    ex, sabs = O.gemm_exact(a, b, b_e5m2=True)
    ad = O.e4m3_decode(a).astype(np.float64)
    bd = O.e5m2_table()[b].astype(np.float64)
    ref, refabs = bd @ ad.T, np.abs(bd) @ np.abs(ad).T
    assert np.allclose(ex, ref, rtol=0, atol=1e-9 * refabs) and np.allclose(sabs, refabs, rtol=1e-12)
    idx_n = rng.integers(0, N, 64).astype(np.int32)
    idx_m = rng.integers(0, M, 64).astype(np.int32)
    exs, _ = O.gemm_exact_sampled(a, b, idx_n, idx_m, b_e5m2=True)
    assert np.array_equal(exs, ex[idx_n, idx_m])
    # small integers are exact in both formats -> int64 known answer through the full epilogue
    ai = rng.integers(-4, 5, (M, K))
    bi = rng.integers(-4, 5, (N, K))
    lib = O.lib()
    a8 = np.array([lib.orc_e4m3_encode(float(v)) for v in ai.ravel()], dtype=np.uint8).reshape(M, K)
    b8 = np.array([lib.orc_e5m2_encode(float(v)) for v in bi.ravel()], dtype=np.uint8).reshape(N, K)
    want = (bi.astype(np.int64) @ ai.astype(np.int64).T).astype(np.float32) * np.float32(0.25)
    for mt in (False, True):
        got = O.gemm_tn(a8, b8, sa=0.5, sb=0.5, out_f32=True, mt=mt, b_e5m2=True)
        assert np.array_equal(got, want)


def test_gemm_random_codes_vs_float64_matmul(O):
    rng = np.random.default_rng(3)
    M, N, K = 64, 48, 512
    a = rng.integers(0, 256, (M, K)).astype(np.uint8)
    b = rng.integers(0, 256, (N, K)).astype(np.uint8)
    a[(a & 0x7F) == 0x7F] = 0x7E
    b[(b & 0x7F) == 0x7F] = 0x7E
    ex, sabs = O.gemm_exact(a, b)
    ad, bd = O.e4m3_decode(a).astype(np.float64), O.e4m3_decode(b).astype(np.float64)
    ref = bd @ ad.T
    assert np.allclose(ex, ref, rtol=0, atol=1e-9 * np.abs(bd) @ np.abs(ad).T)
    assert np.allclose(sabs, np.abs(bd) @ np.abs(ad).T, rtol=1e-12)
    idx_n = rng.integers(0, N, 100).astype(np.int32)
    idx_m = rng.integers(0, M, 100).astype(np.int32)
    exs, sabss = O.gemm_exact_sampled(a, b, idx_n, idx_m)
    assert np.array_equal(exs, ex[idx_n, idx_m]) and np.array_equal(sabss, sabs[idx_n, idx_m])
    # rows subset
    ex2, _ = O.gemm_exact(a, b, rows=(8, 16))
    assert np.array_equal(ex2[8:16], ex[8:16]) and not ex2[:8].any()
    # transposed-operand identity: swapping a and b transposes the result
    ex_t, _ = O.gemm_exact(b, a)
    assert np.array_equal(ex_t, ex.T)
    # mt port stays within fp32 accumulation error of the exact result
    cm = O.gemm_tn(a, b, sa=0.5, sb=0.25, out_f32=True, mt=True)
    assert np.all(np.abs(cm - ex * 0.125) <= 2.0 ** -18 * 0.125 * sabs + 1e-30)


# ------------------------------------------------------------------------------------- generators
def test_generators_are_deterministic_and_sane(O):
    x1 = O.fill_normal_bf16(1 << 16, 4, 9, 0.0, 0.02)
    x2 = O.fill_normal_bf16(1 << 16, 4, 9, 0.0, 0.02)
    assert np.array_equal(x1, x2)
    assert not np.array_equal(x1, O.fill_normal_bf16(1 << 16, 4, 10, 0.0, 0.02))
    xf = O.bf16_to_f32(x1)
    assert abs(xf.mean()) < 5e-4 and abs(xf.std() - 0.02) < 5e-4
    # prefix property of a counter-based stream
    assert np.array_equal(O.fill_normal_bf16(100, 4, 9, 0.0, 0.02), x1[:100])
    t = O.bf16_to_f32(O.fill_student_t3_bf16(1 << 16, 5, 1))
    assert np.isfinite(t).all() and np.abs(t).max() > 8.0 and abs(np.median(t)) < 0.02


# ----------------------------------------------------------------------------------- backward_bias
@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "bf16"])
def test_backward_bias_vs_numpy(O, fmt):
    """Column sums against numpy float64 / int64 (the constructions of scripts/test_kernels.py:834-890
    in the reference: plain sum, with scales, accumulating into an existing dbias)."""
    rng = np.random.default_rng(12)
    BT, OC = 80, 64
    if fmt == "bf16":
        vals = rng.standard_normal((BT, OC)).astype(np.float32)
        dout = O.f32_to_bf16(vals)
        dec = O.bf16_to_f32(dout).astype(np.float64)
    else:
        dout = rng.integers(0, 256, (BT, OC)).astype(np.uint8)
        if fmt == "e4m3":
            dout[(dout & 0x7F) == 0x7F] = 0x7E
            dec = O.e4m3_table()[dout].astype(np.float64)
        else:
            dout[(dout & 0x7C) == 0x7C] = 0x70
            dec = O.e5m2_table()[dout].astype(np.float64)
    zero = np.zeros(OC, dtype=np.uint16)
    got, cs, ca = O.backward_bias(zero, dout, fmt)
    assert np.allclose(cs, dec.sum(0), rtol=1e-12, atol=1e-12) and np.allclose(ca, np.abs(dec).sum(0), rtol=1e-12)
    assert np.array_equal(got, O.f32_to_bf16(dec.sum(0).astype(np.float32)))
    # scales and accumulation: dbias_new = bf16(old + 0.5 * sum), evaluated in fp32
    old = O.f32_to_bf16(rng.standard_normal(OC).astype(np.float32))
    got2, _, _ = O.backward_bias(old, dout, fmt, sa=0.25, sb=2.0)
    want2 = O.f32_to_bf16((dec.sum(0).astype(np.float32) * np.float32(0.5) + O.bf16_to_f32(old)).astype(np.float32))
    assert np.array_equal(got2, want2)
    # integer-valued gradients: exact known answer
    ints = rng.integers(-3, 4, (BT, OC))
    if fmt == "bf16":
        di = O.f32_to_bf16(ints.astype(np.float32))
    else:
        enc = O.lib().orc_e4m3_encode if fmt == "e4m3" else O.lib().orc_e5m2_encode
        lut = {v: enc(float(v)) for v in range(-3, 4)}
        di = np.vectorize(lut.get)(ints).astype(np.uint8)
    got3, _, _ = O.backward_bias(zero, di, fmt)
    assert np.array_equal(O.bf16_to_f32(got3), ints.sum(0).astype(np.float32))


def test_quantize_fp32_input_vs_search(O):
    """fp32-input overloads (src/kernels/kernels.h:251-252): scale*x in fp32, then the same encoders; checked against
    the nearest-code searches on a wide random sample plus the special values."""
    rng = np.random.default_rng(21)
    x = (rng.standard_normal(50000) * 10.0 ** rng.uniform(-6, 2, 50000)).astype(np.float32)
    x[:6] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1e-30]
    am = float(np.abs(x[np.isfinite(x)]).max())
    s, d = O.quant_scale(am)
    with np.errstate(over="ignore", invalid="ignore"):
        y = (np.float32(s) * x).astype(np.float32)
    q4, d4 = O.quantize_f32(x, am, "e4m3")
    q5, d5 = O.quantize_f32(x, am, "e5m2")
    assert np.array_equal(q4, e4m3_encode_search(y)) and np.array_equal(q5, e5m2_encode_search(y))
    assert d4 == np.float32(d) and d5 == np.float32(d)


# ------------------------------------------------------------------------------------------ swiglu
def _swiglu_inputs(O, BT, C, seed, spread=2.0):
    inp = O.fill_normal_bf16(BT * 2 * C, seed, 0, 0.0, spread).reshape(BT, 2 * C)
    dout = O.fill_normal_bf16(BT * C, seed, 1, 0.0, 1.0).reshape(BT, C)
    return inp, dout


def test_swiglu_forward_vs_torch_silu_and_expit(O):
    """The construction of the reference's scripts/test_kernels.py:197-199 (silu(second half) * first half)
    in float64 on torch's CPU kernels, and scipy's expit: the oracle's double values must agree to
    double precision and its bf16 bits must be the rounding of those values."""
    from scipy.special import expit
    BT, C = 37, 48
    inp, _ = _swiglu_inputs(O, BT, C, 101)
    bits, exact = O.swiglu_forward(inp)
    x = torch.from_numpy(O.bf16_to_f32(inp).astype(np.float64))
    a, b = torch.tensor_split(x, 2, dim=-1)
    ref = (torch.nn.functional.silu(b) * a).numpy()
    assert np.allclose(exact, ref, rtol=1e-13, atol=1e-300)
    up, gate = O.bf16_to_f32(inp[:, :C]).astype(np.float64), O.bf16_to_f32(inp[:, C:]).astype(np.float64)
    assert np.allclose(exact, up * gate * expit(gate), rtol=1e-13, atol=1e-300)
    # rounding: bits are the nearest bf16 of the double value (ties are measure-zero here)
    want = O.f32_to_bf16(ref.astype(np.float32))
    assert np.array_equal(bits, want)


def test_swiglu_forward_closed_forms(O):
    """gate = 0 gives 0; large gate gives up * gate; very negative gate gives (signed) zero;
    silu(g) - silu(-g) = g."""
    C = 8
    f = lambda v: O.f32_to_bf16(np.asarray(v, dtype=np.float32))
    up = f([1.5, -2.0, 3.0, 0.5, 1.0, -1.0, 7.0, 0.25])
    for gate_val, expect in ((0.0, lambda u: 0.0 * u), (64.0, lambda u: u * 64.0), (-200.0, lambda u: 0.0 * u)):
        inp = np.concatenate([up, f([gate_val] * C)]).reshape(1, 2 * C)
        bits, _ = O.swiglu_forward(inp)
        assert np.array_equal(O.bf16_to_f32(bits)[0], expect(O.bf16_to_f32(up)).astype(np.float32))
    g = f(np.linspace(-6, 6, C))
    ones = f([1.0] * C)
    _, pos = O.swiglu_forward(np.concatenate([ones, g]).reshape(1, 2 * C))
    neg_g = f(-O.bf16_to_f32(g))
    _, neg = O.swiglu_forward(np.concatenate([ones, neg_g]).reshape(1, 2 * C))
    assert np.allclose(pos - neg, O.bf16_to_f32(g).astype(np.float64), rtol=1e-12, atol=1e-12)


def test_swiglu_backward_vs_torch_autograd_and_differences(O):
    """Gradient against torch autograd in float64 (scripts/test_kernels.py:202-207 in the reference) and
    against central differences of the forward formula; the halves of dinp are [dup | dgate]."""
    BT, C = 9, 24
    inp, dout = _swiglu_inputs(O, BT, C, 202)
    bits, exact = O.swiglu_backward(dout, inp)
    x = torch.from_numpy(O.bf16_to_f32(inp).astype(np.float64)).requires_grad_(True)
    a, b = torch.tensor_split(x, 2, dim=-1)
    (torch.nn.functional.silu(b) * a).backward(torch.from_numpy(O.bf16_to_f32(dout).astype(np.float64)))
    ref = x.grad.numpy()
    assert np.allclose(exact, ref, rtol=1e-12, atol=1e-14)
    assert np.array_equal(bits, O.f32_to_bf16(ref.astype(np.float32)))
    xv = O.bf16_to_f32(inp).astype(np.float64)
    fwd = lambda v: v[:, :C] * v[:, C:] / (1.0 + np.exp(-v[:, C:]))
    h = 1e-6
    d = O.bf16_to_f32(dout).astype(np.float64)
    for half in (0, 1):
        step = np.zeros_like(xv)
        step[:, half * C:(half + 1) * C] = h
        num = (fwd(xv + step) - fwd(xv - step)) / (2 * h) * d
        assert np.allclose(exact[:, half * C:(half + 1) * C], num, rtol=1e-6, atol=1e-8)


# ----------------------------------------------------------------------------------------- rmsnorm
def test_rmsnorm_forward_vs_torch(O):
    """Construction of the reference's scripts/test_kernels.py:88-93 and :583-586 in float64 on torch's CPU
    kernels: 1/rms and the unrounded product agree to double precision; the bf16 bits are torch's bf16
    rounding of s*x followed by torch's bf16 multiply with the weight (the reference's order of roundings,
    src/kernels/rmsnorm.cu:68-71); the residual is torch's bf16 rounding of the fp32 sum."""
    N, Cc, eps = 13, 96, 1e-6
    x1 = O.fill_normal_bf16(N * Cc, 31, 0, 0.0, 1.5).reshape(N, Cc)
    x2 = O.fill_normal_bf16(N * Cc, 31, 1, 0.0, 0.7).reshape(N, Cc)
    w = O.fill_normal_bf16(Cc, 31, 2, 1.0, 0.3)
    as_t = lambda bits: torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16)
    for fused in (False, True):
        normed, rrms, exact, res = O.rmsnorm_forward(x1, w, eps, x2 if fused else None)
        r = as_t(x1)
        if fused:
            r = (as_t(x1).float() + as_t(x2).float()).to(torch.bfloat16)
            assert np.array_equal(res, r.view(torch.int16).numpy().view(np.uint16))
        rd = r.double()
        r_rms = 1.0 / torch.sqrt((rd ** 2).mean(dim=-1, keepdim=True) + float(np.float32(eps)))
        assert np.allclose(exact, (rd * r_rms * as_t(w).double()).numpy(), rtol=1e-13, atol=0)
        assert np.array_equal(rrms, r_rms.squeeze(-1).float().numpy())
        n_b = (r.float() * torch.from_numpy(rrms).unsqueeze(-1)).to(torch.bfloat16)
        want = (n_b * as_t(w)).view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(normed, want)


def test_rmsnorm_forward_closed_forms(O):
    """A constant row v gives s = 1/sqrt(v^2 + eps) and out = bf16(bf16(s v) w); scaling the input by a
    power of two leaves the output unchanged when eps is 0."""
    Cc = 64
    f = lambda v: O.f32_to_bf16(np.asarray(v, dtype=np.float32))
    w = f(np.linspace(0.5, 2.0, Cc))
    row = f([3.0] * Cc).reshape(1, Cc)
    normed, rrms, _, _ = O.rmsnorm_forward(row, w, 0.25)
    s = np.float32(1.0 / np.sqrt(9.0 + 0.25))
    assert rrms[0] == s
    nb = O.bf16_to_f32(f([s * np.float32(3.0)]))[0]
    assert np.array_equal(normed[0], f(nb * O.bf16_to_f32(w)))
    x = O.fill_normal_bf16(4 * Cc, 77, 0).reshape(4, Cc)
    a, ra, _, _ = O.rmsnorm_forward(x, w, 0.0)
    b, rb, _, _ = O.rmsnorm_forward(f(O.bf16_to_f32(x) * 8.0), w, 0.0)
    assert np.array_equal(a, b) and np.array_equal(ra, rb * np.float32(8.0))


def test_rmsnorm_backward_vs_torch_autograd(O):
    """The gradient of out = x * rsqrt(mean(x^2) + eps) * w by torch autograd in float64 (eps = 0 so that the
    stored 1/rms determines the forward exactly), plus the reference's explicit formulas
    (scripts/test_kernels.py:96-113), with accumulation into a non-zero dresidual and dweight."""
    N, Cc = 11, 40
    x = O.fill_normal_bf16(N * Cc, 41, 0, 0.0, 1.3).reshape(N, Cc)
    d = O.fill_normal_bf16(N * Cc, 41, 1, 0.0, 0.8).reshape(N, Cc)
    w = O.fill_normal_bf16(Cc, 41, 2, 1.0, 0.4)
    dres = O.fill_normal_bf16(N * Cc, 41, 3, 0.0, 0.5).reshape(N, Cc)
    dw0 = O.fill_normal_bf16(Cc, 41, 4, 0.0, 2.0)
    t64 = lambda bits: torch.from_numpy(O.bf16_to_f32(bits).astype(np.float64))
    xt = t64(x).requires_grad_(True)
    wt = t64(w).requires_grad_(True)
    r = torch.rsqrt((xt ** 2).mean(dim=-1, keepdim=True))
    (xt * r * wt).backward(t64(d))
    rstd = r.detach().squeeze(-1).numpy()
    # the oracle takes rstd as fp32 (what the forward stored): feed the double value's rounding and allow for it
    res = O.rmsnorm_backward(dres, dw0, d, x, w, rstd.astype(np.float32))
    assert np.allclose(res["exact_dinp"], t64(dres).numpy() + xt.grad.numpy(), rtol=2e-6, atol=1e-7)
    assert np.allclose(res["exact_dw"], t64(dw0).numpy() + wt.grad.numpy(), rtol=2e-6, atol=1e-6)
    # explicit formulas with the same fp32 rstd: agreement to double precision
    rr = torch.from_numpy(rstd.astype(np.float32).astype(np.float64)).unsqueeze(-1)
    xd, dd, wd = t64(x), t64(d), t64(w)
    normed = xd * rr
    dy_w = dd * wd
    dinp = rr * (dy_w - normed * (dy_w * normed).sum(dim=-1, keepdim=True) / Cc)
    assert np.allclose(res["exact_dinp"], (t64(dres) + dinp).numpy(), rtol=1e-12, atol=1e-14)
    assert np.allclose(res["exact_dw"], (t64(dw0) + (dd * xd * rr).sum(dim=0)).numpy(), rtol=1e-12, atol=1e-14)
    assert np.array_equal(res["dinp"], O.f32_to_bf16((t64(dres) + dinp).numpy().astype(np.float32)))
    assert np.array_equal(res["dweight"], O.f32_to_bf16((t64(dw0) + (dd * xd * rr).sum(dim=0)).numpy().astype(np.float32)))


# -------------------------------------------------------------------------------------------- rope
def _rope_table(T, HD, theta=10000.0):
    i = np.arange(HD // 2, dtype=np.float64)
    ang = np.arange(T, dtype=np.float64)[:, None] / theta ** (2 * i / HD)[None, :]
    tab = np.empty((T, HD), dtype=np.float16)
    tab[:, 0::2], tab[:, 1::2] = np.cos(ang), np.sin(ang)
    return tab


def test_rope_vs_complex_multiplication(O):
    """Rotation = multiplication of (real + i imag) by (cos + i sin) in numpy complex128 with numpy's own
    fp16 decoding of the table; value heads untouched; norm preserved up to cos^2 + sin^2 of the rounded
    table; the backward undoes the forward up to that factor."""
    B, T, Nq, Nkv, HD = 2, 5, 3, 2, 16
    N, half = Nq + 2 * Nkv, HD // 2
    x = O.fill_normal_bf16(B * T * N * HD, 51, 0).reshape(B * T, N, HD)
    tab = _rope_table(T, HD)
    out, exact, _ = O.rope(x, tab.view(np.uint16), T, Nq, Nkv)
    xf = O.bf16_to_f32(x).astype(np.float64)
    z = xf[..., :half] + 1j * xf[..., half:]
    rot = (tab[:, 0::2].astype(np.float64) + 1j * tab[:, 1::2].astype(np.float64))
    rot_bt = np.tile(rot, (B, 1))[:, None, :]                      # t = bt % T
    want = z * rot_bt
    qk = slice(0, Nq + Nkv)
    assert np.allclose(exact[:, qk, :half], want[:, qk].real, rtol=1e-14, atol=1e-300)
    assert np.allclose(exact[:, qk, half:], want[:, qk].imag, rtol=1e-14, atol=1e-300)
    assert np.array_equal(out[:, Nq + Nkv:], x[:, Nq + Nkv:]) and np.array_equal(exact[:, Nq + Nkv:], xf[:, Nq + Nkv:])
    assert np.array_equal(out[:, qk], O.f32_to_bf16(np.concatenate([want[:, qk].real, want[:, qk].imag], -1).astype(np.float32)))
    gain = np.abs(rot_bt) ** 2
    n_in, n_out = np.abs(z[:, qk]) ** 2, exact[:, qk, :half] ** 2 + exact[:, qk, half:] ** 2
    assert np.allclose(n_out, n_in * gain, rtol=1e-12)
    # backward of the exact forward values = x * (cos^2 + sin^2)
    fwd_bits = O.f32_to_bf16(exact.astype(np.float32))
    _, back, _ = O.rope(fwd_bits, tab.view(np.uint16), T, Nq, Nkv, backward=True)
    zf = O.bf16_to_f32(fwd_bits).astype(np.float64)
    zz = (zf[..., :half] + 1j * zf[..., half:]) * np.conj(rot_bt)
    assert np.allclose(back[:, qk, :half], zz[:, qk].real, rtol=1e-14, atol=1e-300)
    assert np.allclose(back[:, qk, half:], zz[:, qk].imag, rtol=1e-14, atol=1e-300)


def test_adamw_fp32_parameters_vs_torch_formulas(O):
    """The all-fp32 overload: the reference's test formulas (scripts/test_kernels.py:695-727) in float64; every output is
    an fp32 evaluation of them (no stochastic rounding), so it agrees to a few fp32 ulp of the terms, and the abs-max is
    that of the new parameters."""
    n = 4096
    rng = np.random.default_rng(3)
    params, grads = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    m0 = (rng.standard_normal(n) * 0.1).astype(np.float32)
    v0 = (rng.random(n) * 0.01 + 1e-8).astype(np.float32)
    lr, b1, b2, t, eps, wd, gs = 1e-3, 0.9, 0.999, 3, 1e-8, 0.1, 0.75
    p1, m1, v1, am = O.adamw_update(params, grads, m0, v0, lr, b1, b2, t, eps, wd, gs, 42)
    f = lambda x: np.float64(np.float32(x))
    g, p, m, v = grads.astype(np.float64) * f(gs), params.astype(np.float64), m0.astype(np.float64), v0.astype(np.float64)
    m_new = f(b1) * m + (1 - f(b1)) * g
    v_new = f(b2) * v + (1 - f(b2)) * g ** 2
    c1, c2 = np.float64(np.float32(1.0) / (np.float32(1.0) - np.float32(b1) ** np.float32(t))), np.float64(np.float32(1.0) / (np.float32(1.0) - np.float32(b2) ** np.float32(t)))
    quot = (m_new * c1) / (np.sqrt(v_new * c2) + f(eps))
    p_new = p - f(lr) * (quot + f(wd) * p)
    assert p1.dtype == np.float32 and m1.dtype == np.float32 and v1.dtype == np.float32
    assert np.all(np.abs(m1 - m_new) <= 2.0 ** -22 * (np.abs(m) + np.abs(g)))
    assert np.all(np.abs(v1 - v_new) <= 2.0 ** -22 * (np.abs(v) + g ** 2))
    assert np.all(np.abs(p1 - p_new) <= 2.0 ** -22 * (np.abs(p) + f(lr) * np.abs(quot)) + f(lr) * np.abs(quot) * 2.0 ** -20)
    assert am == np.abs(p1).max()
    # the seed plays no role
    p2, _, _, _ = O.adamw_update(params, grads, m0, v0, lr, b1, b2, t, eps, wd, gs, 7)
    assert np.array_equal(p1, p2)


# ----------------------------------------------------------------------------- fp32 producer variants
def test_fp32_producer_oracles_reduce_to_the_pinned_bf16_ones_and_match_torch(O):
    """The fp32 variants share the formula code of the bf16 ones (pinned above): on bf16-representable inputs their
    double values must be identical and their outputs the fp32 rounding of those; on general fp32 inputs SwiGLU and
    RMSNorm agree with torch float64 (silu, autograd, mean / rsqrt) and rope with complex multiplication."""
    BT, Cc = 7, 24
    inp_b = O.fill_normal_bf16(BT * 2 * Cc, 61, 0, 0.0, 2.0).reshape(BT, 2 * Cc)
    dout_b = O.fill_normal_bf16(BT * Cc, 61, 1).reshape(BT, Cc)
    inp_f, dout_f = O.bf16_to_f32(inp_b), O.bf16_to_f32(dout_b)
    for fn_args_b, fn_args_f in (((O.swiglu_forward, (inp_b,)), (O.swiglu_forward, (inp_f,))),
                                 ((O.swiglu_backward, (dout_b, inp_b)), (O.swiglu_backward, (dout_f, inp_f)))):
        _, ex_b = fn_args_b[0](*fn_args_b[1])
        out_f, ex_f = fn_args_f[0](*fn_args_f[1])
        assert out_f.dtype == np.float32 and np.array_equal(ex_b, ex_f) and np.array_equal(out_f, ex_f.astype(np.float32))
    # general fp32 inputs against torch float64
    rng = np.random.default_rng(5)
    x = rng.normal(0, 2, (BT, 2 * Cc)).astype(np.float32)
    d = rng.normal(0, 1, (BT, Cc)).astype(np.float32)
    xt = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    a, b = torch.tensor_split(xt, 2, dim=-1)
    y = torch.nn.functional.silu(b) * a
    y.backward(torch.from_numpy(d.astype(np.float64)))
    out, ex = O.swiglu_forward(x)
    assert np.allclose(ex, y.detach().numpy(), rtol=1e-13, atol=1e-300) and np.array_equal(out, y.detach().numpy().astype(np.float32))
    dinp, dex = O.swiglu_backward(d, x)
    assert np.allclose(dex, xt.grad.numpy(), rtol=1e-12, atol=1e-14) and np.array_equal(dinp, xt.grad.numpy().astype(np.float32))

    # rmsnorm forward: fp32 chain fl(fl(s x) w), residual one fp32 add
    N, eps = 5, 1e-6
    x1, x2 = rng.normal(0, 1.5, (N, Cc)).astype(np.float32), rng.normal(0, 0.7, (N, Cc)).astype(np.float32)
    w = rng.normal(1, 0.3, Cc).astype(np.float32)
    for fused in (False, True):
        normed, rrms, exact, res = O.rmsnorm_forward(x1, w, eps, x2 if fused else None)
        r = (x1 + x2).astype(np.float32) if fused else x1
        if fused:
            assert np.array_equal(res, r)
        rd = torch.from_numpy(r.astype(np.float64))
        r_rms = 1.0 / torch.sqrt((rd ** 2).mean(dim=-1, keepdim=True) + float(np.float32(eps)))
        assert np.allclose(exact, (rd * r_rms * torch.from_numpy(w.astype(np.float64))).numpy(), rtol=1e-13, atol=0)
        assert np.array_equal(rrms, r_rms.squeeze(-1).float().numpy())
        assert np.array_equal(normed, ((rrms[:, None] * r).astype(np.float32) * w[None, :]).astype(np.float32))
    # rmsnorm backward: the explicit formulas of the reference's test in float64 with the same fp32 rstd
    dres, dw0 = rng.normal(0, 0.5, (N, Cc)).astype(np.float32), rng.normal(0, 2, Cc).astype(np.float32)
    dd = rng.normal(0, 0.8, (N, Cc)).astype(np.float32)
    rstd = (1.0 / np.sqrt((x1.astype(np.float64) ** 2).mean(axis=1))).astype(np.float32)
    got = O.rmsnorm_backward(dres, dw0, dd, x1, w, rstd)
    t64 = lambda v: torch.from_numpy(v.astype(np.float64))
    rr = t64(rstd).unsqueeze(-1)
    normed_t = t64(x1) * rr
    dy_w = t64(dd) * t64(w)
    dinp_t = rr * (dy_w - normed_t * (dy_w * normed_t).sum(dim=-1, keepdim=True) / Cc)
    assert np.allclose(got["exact_dinp"], (t64(dres) + dinp_t).numpy(), rtol=1e-12, atol=1e-14)
    assert np.allclose(got["exact_dw"], (t64(dw0) + (t64(dd) * t64(x1) * rr).sum(dim=0)).numpy(), rtol=1e-12, atol=1e-14)
    assert np.array_equal(got["dinp"], got["exact_dinp"].astype(np.float32)) and np.array_equal(got["dweight"], got["exact_dw"].astype(np.float32))

    # rope: complex multiplication with an fp32 table; value heads copied
    B, T, Nq, Nkv, HD = 2, 5, 3, 2, 16
    Nh, half = Nq + 2 * Nkv, HD // 2
    xr = rng.normal(0, 1, (B * T, Nh, HD)).astype(np.float32)
    tab = _rope_table(T, HD).astype(np.float32) + np.float32(1e-4) * rng.normal(0, 1, (T, HD)).astype(np.float32)
    for backward in (False, True):
        out, exact, _ = O.rope(xr, tab, T, Nq, Nkv, backward=backward)
        z = xr[..., :half].astype(np.float64) + 1j * xr[..., half:].astype(np.float64)
        rot = tab[:, 0::2].astype(np.float64) + 1j * tab[:, 1::2].astype(np.float64)
        rot_bt = np.tile(np.conj(rot) if backward else rot, (B, 1))[:, None, :]
        want = z * rot_bt
        qk = slice(0, Nq + Nkv)
        assert np.allclose(exact[:, qk, :half], want[:, qk].real, rtol=1e-14, atol=1e-300)
        assert np.allclose(exact[:, qk, half:], want[:, qk].imag, rtol=1e-14, atol=1e-300)
        assert np.array_equal(out[:, Nq + Nkv:], xr[:, Nq + Nkv:]) and out.dtype == np.float32
        assert np.array_equal(out[:, qk], np.concatenate([want[:, qk].real, want[:, qk].imag], -1).astype(np.float32))


# ------------------------------------------------------------------------------------------- adamw
def test_squirrel_noise_properties(O):
    """No known-answer vectors exist in the reference tree; what the construction guarantees is checked: for a
    fixed seed the hash is a bijection of the position (no collisions), its bits are balanced, and different
    seeds give unrelated streams."""
    L = O.lib()
    n = 1 << 20
    vals = np.fromiter((L.orc_squirrel_noise_5(i, 1234) for i in range(0, n, 1)), dtype=np.uint32, count=n)
    assert np.unique(vals).size == n
    bits = np.unpackbits(vals[: 1 << 16].view(np.uint8))
    assert abs(bits.mean() - 0.5) < 0.004
    other = np.fromiter((L.orc_squirrel_noise_5(i, 1235) for i in range(1 << 16)), dtype=np.uint32, count=1 << 16)
    assert np.mean(other == vals[: 1 << 16]) < 1e-3
    low = vals[: 1 << 18] & 0xFFFF                   # the 16-bit thresholds: uniform
    hist = np.bincount(low >> 8, minlength=256)
    assert hist.min() > 0.85 * (1 << 18) / 256 and hist.max() < 1.15 * (1 << 18) / 256


def test_stochastic_rounding_properties(O):
    """Values exactly representable in bf16 are unchanged; any other value goes to one of its two bf16
    neighbours (away from zero iff its low 16 bits exceed the threshold); the mean over the hash's thresholds
    is the value itself (the reference's own unbiasedness test, scripts/test_kernels.py:812-828)."""
    L = O.lib()
    for x in (1.0, -2.5, 0.0, 3.0e5, -7.0e-9):
        xb = np.asarray(O.bf16_to_f32(O.f32_to_bf16(np.array([x], np.float32)))).reshape(-1)[0]
        for rnd in (0, 0x1234, 0xFFFF, 0xFFFFFFFF):
            assert O.bf16_to_f32(np.array([L.orc_stochastic_round_bf16(float(xb), rnd)], np.uint16))[0] == xb
    x = np.float32(1.0 + 2.0 ** -9 + 2.0 ** -13)           # between 1 and 1 + 2^-7
    lo, hi = np.float32(1.0), np.float32(1.0 + 2.0 ** -7)
    low_bits = int(np.float32(x).view(np.uint32)) & 0xFFFF
    outs = []
    for i in range(1 << 16):
        rnd = L.orc_squirrel_noise_5(i, 99)
        r = O.bf16_to_f32(np.array([L.orc_stochastic_round_bf16(float(x), rnd)], np.uint16))[0]
        assert r == (hi if low_bits > (rnd & 0xFFFF) else lo)
        outs.append(r)
    assert abs(np.mean(outs, dtype=np.float64) - float(x)) < 2.0 ** -7 * 0.01
    neg = [O.bf16_to_f32(np.array([L.orc_stochastic_round_bf16(float(-x), L.orc_squirrel_noise_5(i, 7))], np.uint16))[0] for i in range(4096)]
    assert set(neg) == {-lo, -hi}


@pytest.mark.parametrize("moments", ["f32f32", "bf16f32", "bf16bf16"])
def test_adamw_vs_torch_formulas(O, moments):
    """The reference's test construction (scripts/test_kernels.py:695-727) in float64."""
    n = 4096
    rng = np.random.default_rng(0)
    f = lambda a: O.f32_to_bf16(a.astype(np.float32))
    params, grads = f(rng.standard_normal(n)), f(rng.standard_normal(n))
    m0 = (rng.standard_normal(n) * 0.1).astype(np.float32)
    v0 = (rng.random(n) * 0.01 + 1e-8).astype(np.float32)
    m_in = f(m0) if moments.startswith("bf16") else m0
    v_in = f(v0) if moments.endswith("bf16") else v0
    lr, b1, b2, t, eps, wd, gs = 1e-3, 0.9, 0.999, 1, 1e-8, 0.1, 0.75
    p1, m1, v1, am = O.adamw_update(params, grads, m_in, v_in, lr, b1, b2, t, eps, wd, gs, 42)
    dec = lambda a: O.bf16_to_f32(a).astype(np.float64) if a.dtype == np.uint16 else a.astype(np.float64)
    g, p, m, v = dec(grads) * np.float64(np.float32(gs)), dec(params), dec(m_in), dec(v_in)
    b1d, b2d = np.float64(np.float32(b1)), np.float64(np.float32(b2))
    m_new = b1d * m + (1 - b1d) * g
    v_new = b2d * v + (1 - b2d) * g ** 2
    p_new = p * (1 - np.float64(np.float32(lr)) * np.float64(np.float32(wd))) - np.float64(np.float32(lr)) * (m_new / (1 - b1d ** t)) / (
        np.sqrt(v_new / (1 - b2d ** t)) + np.float64(np.float32(eps)))
    ulp = lambda x: np.maximum(np.abs(x), 1e-30) * 2.0 ** -7
    assert np.all(np.abs(dec(p1) - p_new) <= ulp(p_new))                      # one of the two bf16 neighbours
    if m1.dtype == np.uint16:
        assert np.all(np.abs(dec(m1) - m_new) <= ulp(m_new) + 2.0 ** -22 * (np.abs(m) + np.abs(g)))
    else:
        assert np.all(np.abs(m1 - m_new) <= 2.0 ** -22 * (np.abs(m) + np.abs(g)))     # fp32 evaluation of the lerp
    if v1.dtype == np.uint16:
        assert np.all(np.abs(dec(v1) - v_new) <= ulp(v_new))
    else:
        assert np.all(np.abs(v1 - v_new) <= 2.0 ** -22 * (np.abs(v) + g ** 2))
    assert am == np.abs(O.bf16_to_f32(p1)).max()
    # stochastic rounding is unbiased: the mean error of the parameters is far below half an ulp
    assert abs(np.mean((dec(p1) - p_new) / ulp(p_new))) < 0.05
