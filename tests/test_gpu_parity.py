"""GPU parity tests: every call goes through the C ABI (llmq_amd.capi via llmq_amd.kernels) and is
compared with the CPU oracle on identical inputs.  abs-max, scales and fp8 bytes must be bit exact;
GEMM results must meet the tolerance stated in tests/gpu_util.py."""
import numpy as np
import pytest
import torch

from gpu_util import dev_bf16, dev_scalar, dev_u8, gemm_check, gemm_library, host_bits, report_gemm_error

pytestmark = pytest.mark.gpu

ALL_BF16 = np.arange(65536, dtype=np.uint32).astype(np.uint16)


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from llmq_amd import kernels
    return kernels


def gpu_abs_max(K, bits):
    out = torch.full((1,), 123.0, dtype=torch.float32, device="cuda")   # stale value must be overwritten
    K.abs_max(out, dev_bf16(bits))
    return out.cpu().numpy()[0]


def gpu_quantize(K, bits, absmax, fmt=torch.float8_e4m3fn, with_scale=True):
    x = dev_bf16(bits)
    out = torch.empty(x.shape, dtype=fmt, device="cuda")
    scale = torch.full((1,), -1.0, dtype=torch.float32, device="cuda") if with_scale else None
    K.quantize_with_abs_max(out, scale, x, dev_scalar(absmax))
    return host_bits(out), (scale.cpu().numpy()[0] if with_scale else None)


# ------------------------------------------------------------------------------------------ abs-max
@pytest.mark.parametrize("n", [8, 64, 1000, 1024, 16 * 64, 4 * 128 * 32, 1 << 20, (1 << 20) + 8, 3 * 1000 * 1000 + 5, 7])
def test_abs_max_bit_exact(K, O, n):
    x = O.fill_normal_bf16(n, 100 + n % 97, 1, 0.0, 2.5)
    assert gpu_abs_max(K, x).view(np.uint32) == np.float32(O.abs_max_bf16(x)).view(np.uint32)


def test_abs_max_special_values(K, O):
    cases = [
        np.array([0x7FC0, 0x7F81, 0xFFC1, 0xFFFF] * 2, np.uint16),                 # all NaN -> 0
        np.array([0x8000] * 16, np.uint16),                                         # -0 -> +0
        np.array([0x3F80, 0x7FC0, 0xC000, 0x7F81, 0, 0, 0, 0], np.uint16),          # NaN skipped -> 2
        np.array([0x3F80, 0xFF80, 0x7FC0, 0, 0, 0, 0, 0], np.uint16),               # -Inf wins
        np.array([0x0001, 0x8003, 0, 0, 0, 0, 0, 0], np.uint16),                    # denormals kept
        np.array([0x7F7F, 0xFF7F] + [0] * 6, np.uint16),                            # max finite
        np.zeros(0, np.uint16),                                                     # empty -> 0
    ]
    for c in cases:
        got, want = gpu_abs_max(K, c), np.float32(O.abs_max_bf16(c))
        assert got.view(np.uint32) == want.view(np.uint32), (c, got, want)
    # maximum hidden at every position of a block-sized tensor's tail
    base = O.fill_normal_bf16(1 << 16, 5, 5)
    for pos in [0, 1, 7, 8, 65535, 65528, 4099]:
        x = base.copy()
        x[pos] = 0xC2C8  # -100
        assert gpu_abs_max(K, x) == 100.0


def test_abs_max_f32(K):
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(1000003, device="cuda", generator=g) * 7
    x[12345] = float("nan")
    out = torch.zeros(1, device="cuda")
    K.abs_max(out, x)
    assert out.item() == torch.nan_to_num(x, nan=0.0).abs().max().item()


def test_abs_max_single_launch_arrival_area_is_reusable(K):
    """abs_max is one launch: the workgroups meet in an arrival area of the device code that the last of them
    leaves ready for the next call.  A run of calls of different sizes into ONE result slot (one area: many
    workgroups, few, one, many again) must each give the exact maximum, whatever the slot and the area held before."""
    g = torch.Generator(device="cuda").manual_seed(21)
    out = torch.full((1,), float("nan"), device="cuda")
    big = torch.randn(40 * 1000 * 1000 + 24, device="cuda", generator=g).to(torch.bfloat16)
    for rep in range(3):
        for n in (big.numel(), 3 * 1000 * 1000 + 5, 65536, 64, 65537, 9 * 65536, big.numel() - 8):
            x = big[:n] * float(1 + rep)
            K.abs_max(out, x)
            assert out.item() == x.float().abs().max().item(), (rep, n)
    # the maximum hidden in every workgroup's chunk in turn (a chunk is 16384 elements)
    x = torch.zeros(40 * 16384 + 8, dtype=torch.bfloat16, device="cuda")
    for blk in range(41):
        x.zero_()
        x[min(blk * 16384 + 4321, x.numel() - 1)] = -3.0
        K.abs_max(out, x)
        assert out.item() == 3.0, blk


def test_abs_max_beyond_the_workgroup_cap(K):
    """A tensor of more than 1 GiB: every workgroup of the capped grid walks many chunks, 64-bit element offsets."""
    n = 8192 * 65536 + 3 * 65536 + 40
    x = torch.zeros(n, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(1, device="cuda")
    for pos, v in ((5, 1.5), (8192 * 65536 + 77, -2.5), (n - 1, 7.0)):
        x[pos] = v
        K.abs_max(out, x)
        assert out.item() == abs(v)
    del x


def test_abs_max_neighbouring_slots_on_two_streams(K):
    """Result slots 4 bytes apart (the [abs_max, ...] tables of the reference's run state) map to different arrival
    areas, so their calls may overlap in time: two streams, no ordering between them, 40 rounds."""
    g = torch.Generator(device="cuda").manual_seed(22)
    xs = [torch.randn(6 * 1000 * 1000, device="cuda", generator=g).to(torch.bfloat16) * s for s in (1.0, 3.0)]
    want = [x.float().abs().max().item() for x in xs]
    table = torch.zeros(2, device="cuda")
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    for rnd in range(40):
        for i, st in enumerate(streams):
            K.abs_max(table[i:i + 1], xs[i], stream=st.cuda_stream)
    torch.cuda.synchronize()
    assert table.tolist() == want


# ----------------------------------------------------------------------------------------- quantize
@pytest.mark.parametrize("absmax", [448.0, 1.0, 5.15625, 0.072265625, 3.0e-5, 1e4, 0.0, 447.0, 1.7e38, float("inf")])
def test_quantize_exhaustive_all_bf16_inputs(K, O, absmax):
    got, scale = gpu_quantize(K, ALL_BF16, absmax)
    want, d = O.quantize_e4m3(ALL_BF16, absmax)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(hex(int(ALL_BF16[i])), hex(int(got[i])), hex(int(want[i]))) for i in bad[:10]]
    assert np.float32(scale).view(np.uint32) == np.float32(d).view(np.uint32)


@pytest.mark.parametrize("absmax", [448.0, 57344.0, 1.0, 3.0e-5, 0.0])
def test_quantize_e5m2_exhaustive(K, O, absmax):
    got, scale = gpu_quantize(K, ALL_BF16, absmax, fmt=torch.float8_e5m2)
    want, d = O.quantize_e4m3(ALL_BF16, absmax, fmt="e5m2")
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(hex(int(ALL_BF16[i])), hex(int(got[i])), hex(int(want[i]))) for i in bad[:10]]
    assert np.float32(scale).view(np.uint32) == np.float32(d).view(np.uint32)


@pytest.mark.parametrize("n", [8, 1024, 8192, 8200, 1 << 20, 4096 * 896, 13])
def test_quantize_random_tensors(K, O, n):
    x = O.fill_normal_bf16(n, 7, n % 11)
    am = O.abs_max_bf16(x)
    got, scale = gpu_quantize(K, x, am)
    want, d = O.quantize_e4m3(x, am, mt=True)
    assert np.array_equal(got, want) and np.float32(scale) == d
    got2, none = gpu_quantize(K, x, am, with_scale=False)      # null scale pointer
    assert np.array_equal(got2, want) and none is None


def test_quantize_stale_absmax_saturates(K, O):
    x = O.fill_normal_bf16(1 << 16, 9, 9, 0.0, 10.0)
    got, _ = gpu_quantize(K, x, 1.0)              # abs-max far too small: values clamp at +-448
    want, _ = O.quantize_e4m3(x, 1.0)
    assert np.array_equal(got, want) and (got == 0x7E).any() and (got == 0xFE).any()


# ------------------------------------------------------------------------- quantize + transpose, transpose
QT_SHAPES = [(32, 32), (128, 256), (512, 1024), (8, 8), (8, 72), (72, 8), (264, 136), (256, 64), (1000, 24),
             (4096, 896), (520, 1160), (2048, 4864)]


@pytest.mark.parametrize("shape", QT_SHAPES)
def test_quantize_transpose_bit_exact(K, O, shape):
    rows, cols = shape
    x = O.fill_normal_bf16(rows * cols, 21, rows + cols).reshape(rows, cols)
    am = O.abs_max_bf16(x)
    want, d = O.quantize_e4m3(x, am, mt=True)
    xd = dev_bf16(x)
    out = torch.empty((cols, rows), dtype=torch.float8_e4m3fn, device="cuda")
    scale = torch.zeros(1, device="cuda")
    K.quantize_and_transpose_with_abs_max(out, scale, xd, dev_scalar(am))
    assert np.array_equal(host_bits(out), want.T)
    assert scale.item() == d
    out2 = torch.empty((cols, rows), dtype=torch.float8_e4m3fn, device="cuda")
    K.quantize_and_transpose_with_abs_max(out2, None, xd, dev_scalar(am))   # null scale as at llama_model.cpp:328
    assert np.array_equal(host_bits(out2), want.T)


@pytest.mark.parametrize("shape", QT_SHAPES)
def test_quantize_transpose_fp32_input_bit_exact(K, O, shape):
    """fp32-input overload (src/kernels/kernels.h:261): the bytes of the fp32 quantizer, transposed; NaN, +-Inf,
    signed zeros and denormals included."""
    rows, cols = shape
    rng = np.random.default_rng(rows * 3 + cols)
    x = (rng.standard_normal((rows, cols)) * 10.0 ** rng.uniform(-6, 2, (rows, cols))).astype(np.float32)
    flat = x.reshape(-1)
    flat[:6] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1e-40]
    am = float(np.abs(flat[np.isfinite(flat)]).max())
    want, d = O.quantize_f32(x, am)
    out = torch.empty((cols, rows), dtype=torch.float8_e4m3fn, device="cuda")
    scale = torch.zeros(1, device="cuda")
    K.quantize_and_transpose_with_abs_max(out, scale, torch.from_numpy(x).cuda(), dev_scalar(am))
    assert np.array_equal(host_bits(out), want.T)
    assert scale.item() == d


@pytest.mark.parametrize("fmt", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("shape", QT_SHAPES)
def test_quantize_plain_and_transposed_in_one_read(K, O, shape, fmt):
    """The fused kernel must give exactly the bytes of quantize_with_abs_max followed by transpose (the
    two-route byte identity idea of src/testing/test-swiglu.cu:243-315), for both fp8 formats."""
    rows, cols = shape
    x = O.fill_student_t3_bf16(rows * cols, 9, rows + cols, 0.5).reshape(rows, cols)
    x[0, 0] = 0x7FC0                                   # a NaN
    x[rows - 1, cols - 1] = 0xFF80                     # -Inf
    am = O.abs_max_bf16(x[np.isfinite(O.bf16_to_f32(x))])
    e5 = fmt == torch.float8_e5m2
    want, d = O.quantize_e4m3(x, am, mt=not e5, fmt="e5m2" if e5 else "e4m3")
    xd = dev_bf16(x)
    out = torch.zeros((rows, cols), dtype=fmt, device="cuda")
    out_t = torch.zeros((cols, rows), dtype=fmt, device="cuda")
    sc = torch.zeros(1, device="cuda")
    K.quantize_with_abs_max_and_transpose(out, out_t, sc, xd, dev_scalar(am))
    assert np.array_equal(host_bits(out), want.reshape(rows, cols))
    assert np.array_equal(host_bits(out_t), want.reshape(rows, cols).T)
    assert sc.cpu().numpy()[0] == d


@pytest.mark.parametrize("shape", QT_SHAPES + [(1, 1), (3, 5), (17, 33), (100, 7), (64, 65), (4864, 896), (16, 4096)])
def test_transpose_bit_exact(K, shape):
    rows, cols = shape
    rng = np.random.default_rng(rows * 131 + cols)
    src = rng.integers(0, 256, (rows, cols)).astype(np.uint8)
    d = torch.empty((cols, rows), dtype=torch.uint8, device="cuda")
    K.transpose(d, dev_u8(src))
    assert np.array_equal(d.cpu().numpy(), src.T)


@pytest.mark.parametrize("fmt", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("n", [0, 1, 3, 4, 1000, 4099, 1 << 20])
def test_quantize_fp32_input_bit_exact(K, O, fmt, n):
    """fp32-input overloads of quantize_with_abs_max (src/kernels/kernels.h:251-252), incl. ragged tails."""
    rng = np.random.default_rng(n + 5)
    x = (rng.standard_normal(n) * 10.0 ** rng.uniform(-6, 2, n)).astype(np.float32)
    if n >= 1000:
        x[:6] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1e-30]
    fin = x[np.isfinite(x)]
    am = float(np.abs(fin).max()) if fin.size else 0.0
    want, d = O.quantize_f32(x, am, "e5m2" if fmt == torch.float8_e5m2 else "e4m3")
    out = torch.zeros(n, dtype=fmt, device="cuda")
    sc = torch.zeros(1, device="cuda")
    K.quantize_with_abs_max(out, sc, torch.from_numpy(x).cuda(), dev_scalar(am))
    assert np.array_equal(host_bits(out), want) and sc.cpu().numpy()[0] == d


# --------------------------------------------------------------------------------------------- GEMM
_FORCED = {"lib": None}


def set_variant(v):
    """v = (tile, splits[, persistent]): tile 0 = automatic, 1 = 256 x 256 (8 waves), 2 = 128 x 128, 3 = 256 x 256
    (4 waves, 16x16x128 matrix instruction), 4 / 5 = its 224- / 192-wide tiles; splits 0 = automatic; persistent
    -1 = automatic, 0 = one workgroup per tile, 1 = persistent tile walk.  The product library has no such
    switch: a forced variant runs on the test-aid build of the same GEMM source (capi.testaid()), the automatic
    choice (0, 0) on the product library."""
    from llmq_amd import capi
    forced = tuple(v) not in ((0, 0), (0, 0, -1))
    if forced or _FORCED["lib"] is not None:
        t = capi.testaid()
        t.llmq_debug_set_gemm_variant(v[0], v[1])
        t.llmq_debug_set_gemm_persist(v[2] if len(v) > 2 else -1)
    _FORCED["lib"] = capi.testaid() if forced else None


def mm(K, *args, **kw):
    """K.matmul on whichever library set_variant selected."""
    with gemm_library(_FORCED["lib"]):
        return K.matmul(*args, **kw)


# (tile selector, K splits[, persistent walk]); for the four-wave kernel (tile 3) the second number cuts the
# tiles of each XCD's last round into that many K segments
VARIANTS = [(0, 0), (1, 0, 0), (1, 1, 1), (2, 0), (1, 2), (2, 2), (2, 3), (3, 1), (3, 2), (3, 4)]
_WORKSPACE = {}


def workspace():
    if "ws" not in _WORKSPACE:
        _WORKSPACE["ws"] = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    return _WORKSPACE["ws"]


def skip_unsupported(variant, M, N, Kd):
    if variant[0] in (1, 3) and (M % 256 or N % 256):
        pytest.skip("the 256 x 256 tile needs multiples of 256")
    if variant[0] == 3 and Kd % 256 and (Kd < 384 or variant[1] > 1):
        pytest.skip("the four-wave kernel takes an odd number of K-steps from 3 up, and cuts only even ones into segments")
    if variant[0] == 3 and variant[1] > 1:
        # mirrors the launch plan: 32 workgroups per XCD, segments of whole pairs of K-steps, none empty,
        # and one 256 KiB partial tile per segment in the 32 MiB workspace
        S, pairs, tiles = variant[1], Kd // 256, (M // 256) * (N // 256)
        xq, xr = divmod(tiles, 8)
        rem_max = max((xq + 1) % 32 if xr else 0, xq % 32)
        seg = -(-pairs // S)
        if rem_max == 0 or rem_max * S > 32 or 8 * rem_max * S > 128 or (S - 1) * seg >= pairs:
            pytest.skip("the last round cannot be cut this way")
        return
    if variant[1] > Kd // 128:
        pytest.skip("more splits than K-steps")
    if len(variant) > 2 and variant[2] == 1 and Kd < 256:
        pytest.skip("the persistent walk needs two K-steps")


def run_gemm(K, a, b, M, N, Kd, sa, sb, bias_bits=None, old=None, out_f32=False):
    dt = torch.float32 if out_f32 else torch.bfloat16
    if old is not None:
        c = (torch.from_numpy(old).cuda() if out_f32 else dev_bf16(old)).reshape(N, M).clone()
    else:
        c = torch.full((N, M), float("nan"), dtype=dt, device="cuda")
    bias = dev_bf16(bias_bits) if bias_bits is not None else None
    mm(K, c, dev_u8(a), dev_u8(b), bias, dev_scalar(sa) if sa is not None else None,
             dev_scalar(sb) if sb is not None else None, M, N, Kd, accumulate=old is not None, workspace=workspace())
    torch.cuda.synchronize()
    return c


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("mnk", [(128, 128, 128), (256, 256, 256), (512, 768, 384), (256, 512, 1024), (768, 512, 512)])
def test_gemm_integer_known_answer_exact(K, O, variant, mnk):
    """Construction of src/testing/test-gemm.cpp:54-85: integer operands, exact fp32 sums -> the bf16
    output must equal the oracle bit for bit (set / bias / accumulate)."""
    M, N, Kd = mnk
    skip_unsupported(variant, M, N, Kd)
    a, _ = O.fill_int_e4m3(M * Kd, 12345, 0)
    b, _ = O.fill_int_e4m3(N * Kd, 12345, 1)
    a, b = a.reshape(M, Kd), b.reshape(N, Kd)
    s = float(np.sqrt(np.float32(4.0 / Kd)))
    _, biasv = O.fill_int_e4m3(M, 12345, 2)
    _, oldv = O.fill_int_e4m3(N * M, 12345, 3)
    bias = O.f32_to_bf16(biasv.astype(np.float32))
    old = O.f32_to_bf16(oldv.astype(np.float32)).reshape(N, M)
    set_variant(variant)
    try:
        for use_bias, use_old in [(False, False), (True, False), (False, True), (True, True)]:
            want = O.gemm_tn(a, b, sa=s, sb=s, bias=bias if use_bias else None, c_old=old if use_old else None, mt=True)
            got = run_gemm(K, a, b, M, N, Kd, s, s, bias if use_bias else None, old if use_old else None)
            assert np.array_equal(host_bits(got), want), (use_bias, use_old)
        want32 = O.gemm_tn(a, b, sa=s, sb=s, out_f32=True, mt=True)
        got32 = run_gemm(K, a, b, M, N, Kd, s, s, out_f32=True)
        assert np.array_equal(got32.cpu().numpy(), want32)
    finally:
        set_variant((0, 0))


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("out_f32", [False, True])
def test_gemm_random_codes_within_tolerance(K, O, variant, out_f32):
    M, N, Kd = (512, 256, 896) if variant[0] != 3 else (512, 256, 1024)
    skip_unsupported(variant, M, N, Kd)
    rng = np.random.default_rng(17)
    a = rng.integers(0, 256, (M, Kd)).astype(np.uint8)
    b = rng.integers(0, 256, (N, Kd)).astype(np.uint8)
    a[(a & 0x7F) == 0x7F] ^= 1      # no NaN codes
    b[(b & 0x7F) == 0x7F] ^= 1
    sa, sb = 0.37, 1.0 / 448
    exact, sumabs = O.gemm_exact(a, b)
    scale = np.float32(np.float32(sa) * np.float32(sb))
    set_variant(variant)
    try:
        got = run_gemm(K, a, b, M, N, Kd, sa, sb, out_f32=out_f32)
        g32 = got.float().cpu().numpy()
        gemm_check(g32, exact, sumabs, scale, not out_f32)
        # no scales at all (null pointers)
        got1 = run_gemm(K, a, b, M, N, Kd, None, None, out_f32=True)
        gemm_check(got1.cpu().numpy(), exact, sumabs, 1.0, False)
        # bias + accumulate on top
        bias = O.fill_normal_bf16(M, 3, 3, 0.0, 50.0)
        old = O.bf16_to_f32(O.fill_normal_bf16(N * M, 3, 4, 0.0, 100.0)).reshape(N, M)
        oldp = old if out_f32 else O.f32_to_bf16(old)
        got2 = run_gemm(K, a, b, M, N, Kd, sa, sb, bias, oldp, out_f32=out_f32)
        extra = O.bf16_to_f32(bias).astype(np.float64)[None, :] + old.astype(np.float64)
        gemm_check(got2.float().cpu().numpy(), exact, sumabs, scale, not out_f32, extra=extra)
    finally:
        set_variant((0, 0))


@pytest.mark.parametrize("forced", [True, False])
@pytest.mark.parametrize("mnk", [(224, 256, 256), (448, 512, 512), (3584, 8192, 256), (3584, 8192, 512), (1792, 8448, 768),
                                 (7168, 4352, 256), (192, 256, 256), (576, 512, 512), (1536, 16384, 256), (1536, 8448, 768),
                                 (4608, 4352, 512)])
def test_gemm_narrow_tile(K, O, mnk, forced):
    """The four-wave kernel with 256 x 224 and 256 x 192 tiles (tile selectors 4 and 5, and whatever the automatic
    choice takes for these shapes): less than one round of tiles, exactly two rounds, uneven persistent walks;
    integer operands -> bit exact against the oracle, with and without bias; random codes within the GEMM
    tolerance; accumulation and fp32 output are refused by the forced selector and served by the other kernels
    automatically."""
    M, N, Kd = mnk
    selector = 4 if M % 224 == 0 else 5
    a, _ = O.fill_int_e4m3(M * Kd, 777, 0)
    b, _ = O.fill_int_e4m3(N * Kd, 777, 1)
    a, b = a.reshape(M, Kd), b.reshape(N, Kd)
    s = float(np.sqrt(np.float32(4.0 / Kd)))
    mt = M % 64 == 0          # the threaded oracle works on 64-column blocks
    set_variant((selector, 0) if forced else (0, 0))
    try:
        want = O.gemm_tn(a, b, sa=s, sb=s, mt=mt)
        got = run_gemm(K, a, b, M, N, Kd, s, s)
        assert np.array_equal(host_bits(got), want)
        got = run_gemm(K, a, b, M, N, Kd, None, None)
        assert np.array_equal(host_bits(got), O.gemm_tn(a, b, mt=mt))
        if M * N <= 3584 * 8192 and Kd <= 512:
            rng = np.random.default_rng(M + Kd)
            ar = rng.integers(0, 256, (M, Kd)).astype(np.uint8)
            br = rng.integers(0, 256, (N, Kd)).astype(np.uint8)
            ar[(ar & 0x7F) == 0x7F] ^= 1
            br[(br & 0x7F) == 0x7F] ^= 1
            rows = (0, N) if N <= 512 else (N - 300, N)
            exact, sumabs = O.gemm_exact(ar, br, rows=rows)
            g32 = run_gemm(K, ar, br, M, N, Kd, 0.37, 1.0 / 448).float().cpu().numpy()
            scale = np.float32(np.float32(0.37) * np.float32(1.0 / 448))
            gemm_check(g32[rows[0]:rows[1]], exact[rows[0]:rows[1]], sumabs[rows[0]:rows[1]], scale, True)
        _, biasv = O.fill_int_e4m3(M, 777, 2)
        bias = O.f32_to_bf16(biasv.astype(np.float32))
        got = run_gemm(K, a, b, M, N, Kd, s, s, bias)
        assert np.array_equal(host_bits(got), O.gemm_tn(a, b, sa=s, sb=s, bias=bias, mt=mt))
        _, oldv = O.fill_int_e4m3(N * M, 777, 3)
        old = O.f32_to_bf16(oldv.astype(np.float32)).reshape(N, M)
        if forced:
            with pytest.raises(ValueError, match="narrow tile|off the lattice"):
                run_gemm(K, a, b, M, N, Kd, s, s, None, old)
            with pytest.raises(ValueError, match="narrow tile|off the lattice"):
                run_gemm(K, a, b, M, N, Kd, s, s, out_f32=True)
        else:   # accumulation and fp32 output: the other tiled kernels, or the general-shape kernel when M % 128 != 0
            got = run_gemm(K, a, b, M, N, Kd, s, s, bias, old)
            assert np.array_equal(host_bits(got), O.gemm_tn(a, b, sa=s, sb=s, bias=bias, c_old=old, mt=mt))
            got32 = run_gemm(K, a, b, M, N, Kd, s, s, out_f32=True)
            assert np.array_equal(got32.cpu().numpy(), O.gemm_tn(a, b, sa=s, sb=s, out_f32=True, mt=mt))
    finally:
        set_variant((0, 0))


def _dispatch_sweep_cases():
    """Deterministic pseudo-random shapes for the automatic kernel choice: M from multiples of 128, 192, 224 and
    256, N from multiples of 128 and 256, K from multiples of 128 and 256, tile counts from a handful to a few
    rounds of the chip, every epilogue flavour (an M off the 128 lattice with accumulation or fp32 output, or with
    an N off the 256 lattice, ends on the general-shape kernel in whole or for its last rows)."""
    rng = np.random.default_rng(2024)
    cases = []
    for idx in range(48):
        unit_m = [128, 192, 224, 256][idx % 4]
        M = int(unit_m * rng.integers(1, [24, 16, 16, 14][idx % 4]))
        N = int([128, 256][idx % 2] * rng.integers(1, [40, 24][idx % 2]))
        Kd = int([128, 256][(idx // 2) % 2] * rng.integers(1, 9))
        if M % 64:                                 # outside the threaded oracle's 64-column blocks: keep it small
            N, Kd = min(N, 1024), min(Kd, 512)
        cases.append((M, N, Kd, idx % 3 == 1, idx % 5 == 2, idx % 7 == 3, idx % 4 != 3))
    return cases


@pytest.mark.parametrize("case", _dispatch_sweep_cases())
def test_gemm_automatic_choice_sweep(K, O, case):
    """Whatever kernel, tile width and K split the dispatcher picks: integer operands -> bit exact against the
    oracle (bf16 and fp32 output, bias, accumulation, with and without a workspace)."""
    M, N, Kd, use_bias, use_old, out_f32, with_ws = case
    a, _ = O.fill_int_e4m3(M * Kd, 31 + M, 0)
    b, _ = O.fill_int_e4m3(N * Kd, 31 + N, 1)
    a, b = a.reshape(M, Kd), b.reshape(N, Kd)
    s = float(np.sqrt(np.float32(4.0 / Kd)))
    _, biasv = O.fill_int_e4m3(M, 31, 2)
    _, oldv = O.fill_int_e4m3(N * M, 31, 3)
    bias = O.f32_to_bf16(biasv.astype(np.float32)) if use_bias else None
    oldf = oldv.astype(np.float32).reshape(N, M)
    old = (oldf if out_f32 else O.f32_to_bf16(oldf).reshape(N, M)) if use_old else None
    want = O.gemm_tn(a, b, sa=s, sb=s, bias=bias, c_old=old, out_f32=out_f32, mt=M % 64 == 0)
    dt = torch.float32 if out_f32 else torch.bfloat16
    if old is not None:
        c = (torch.from_numpy(old).cuda() if out_f32 else dev_bf16(old)).reshape(N, M).clone()
    else:
        c = torch.full((N, M), float("nan"), dtype=dt, device="cuda")
    mm(K, c, dev_u8(a), dev_u8(b), dev_bf16(bias) if use_bias else None, dev_scalar(s), dev_scalar(s), M, N, Kd,
             accumulate=use_old, workspace=workspace() if with_ws else None)
    got = c.cpu().numpy() if out_f32 else host_bits(c)
    assert np.array_equal(got, want), case


@pytest.mark.parametrize("variant", [(1, 1, 1), (3, 1), (3, 2), (3, 3), (3, 4)])
@pytest.mark.parametrize("mnk", [(4352, 4352, 384), (4608, 4096, 256), (8192, 4864, 512), (4352, 4352, 1024),
                                 (4352, 4096, 1024), (4352, 4352, 1536)])
def test_gemm_persistent_tile_walk(K, O, mnk, variant):
    """More tiles than compute units: workgroups walk several tiles each and the operand stream crosses
    tile boundaries (odd and even numbers of K-steps flip the LDS stage parity differently); the (3, S)
    variants cut the tiles left over after the full rounds into S segments of K (XCDs with 5 and 4, or
    2 such tiles; segments of equal and unequal length).  Integer
    operands -> bit-exact against the oracle, with bias and accumulation, bf16 and fp32 outputs."""
    M, N, Kd = mnk
    skip_unsupported(variant, M, N, Kd)
    a, _ = O.fill_int_e4m3(M * Kd, 4242, 0)
    b, _ = O.fill_int_e4m3(N * Kd, 4242, 1)
    a, b = a.reshape(M, Kd), b.reshape(N, Kd)
    s = float(np.sqrt(np.float32(4.0 / Kd)))
    _, biasv = O.fill_int_e4m3(M, 4242, 2)
    _, oldv = O.fill_int_e4m3(N * M, 4242, 3)
    bias = O.f32_to_bf16(biasv.astype(np.float32))
    old = O.f32_to_bf16(oldv.astype(np.float32)).reshape(N, M)
    set_variant(variant)
    try:
        want = O.gemm_tn(a, b, sa=s, sb=s, mt=True)
        got = run_gemm(K, a, b, M, N, Kd, s, s)
        assert np.array_equal(host_bits(got), want)
        want = O.gemm_tn(a, b, sa=s, sb=s, bias=bias, c_old=old, mt=True)
        got = run_gemm(K, a, b, M, N, Kd, s, s, bias, old)
        assert np.array_equal(host_bits(got), want)
        want32 = O.gemm_tn(a, b, sa=s, sb=s, out_f32=True, mt=True)
        got32 = run_gemm(K, a, b, M, N, Kd, s, s, out_f32=True)
        assert np.array_equal(got32.cpu().numpy(), want32)
    finally:
        set_variant((0, 0))


@pytest.mark.parametrize("variant,mnk", [((3, 1), (4096, 8192, 2048)), ((0, 0), (18944, 3584, 8192))])
def test_gemm_four_wave_large_repeatable(K, O, variant, mnk):
    """The four-wave kernel issues its matrix instructions from asm statements (the compiler does not see
    them as such), so beyond the exact small cases: a chip-filling shape with random codes, repeated, must
    give bit-identical results every time and agree with the exact product on sampled outputs.  The
    second case is a weight-gradient shape on which the automatic plan cuts the last round's one or two
    tiles per XCD into K segments summed by a separate kernel."""
    M, N, Kd = mnk
    rng = np.random.default_rng(33)
    a = rng.integers(0, 0x7E, (M, Kd)).astype(np.uint8) | (rng.integers(0, 2, (M, Kd)).astype(np.uint8) << 7)
    b = rng.integers(0, 0x7E, (N, Kd)).astype(np.uint8) | (rng.integers(0, 2, (N, Kd)).astype(np.uint8) << 7)
    ad, bd = dev_u8(a), dev_u8(b)
    sa = dev_scalar(2.0 ** -6)
    set_variant(variant)
    try:
        first = None
        for rep in range(8):
            c = torch.full((N, M), float("nan"), dtype=torch.float32, device="cuda")
            mm(K, c, ad, bd, None, sa, None, M, N, Kd, workspace=workspace())
            torch.cuda.synchronize()
            if first is None:
                first = c
            else:
                assert torch.equal(first.view(torch.int32), c.view(torch.int32)), "run %d differs" % rep
    finally:
        set_variant((0, 0))
    idx_n = rng.integers(0, N, 40000).astype(np.int32)
    idx_m = rng.integers(0, M, 40000).astype(np.int32)
    ex, sabs = O.gemm_exact_sampled(a, b, idx_n, idx_m)
    gemm_check(first.cpu().numpy()[idx_n, idx_m], ex, sabs, np.float32(2.0 ** -6), False)


@pytest.mark.parametrize("mnk", [(128, 128, 4096), (256, 384, 2048), (896, 896, 8192)])
def test_gemm_automatic_split_k(K, O, mnk):
    """Few-tile shapes with a workspace take the split-K path on their own; integer operands keep
    every partial sum exact, so the result must still equal the oracle bit for bit, and repeated
    calls must agree (fixed summation order)."""
    M, N, Kd = mnk
    a, _ = O.fill_int_e4m3(M * Kd, 777, 0)
    b, _ = O.fill_int_e4m3(N * Kd, 777, 1)
    a, b = a.reshape(M, Kd), b.reshape(N, Kd)
    s = float(np.sqrt(np.float32(4.0 / Kd)))
    _, biasv = O.fill_int_e4m3(M, 777, 2)
    bias = O.f32_to_bf16(biasv.astype(np.float32))
    want = O.gemm_tn(a, b, sa=s, sb=s, bias=bias, mt=True)
    got = run_gemm(K, a, b, M, N, Kd, s, s, bias)
    assert np.array_equal(host_bits(got), want)
    rng = np.random.default_rng(5)
    ar = rng.integers(0, 0x7E, (M, Kd)).astype(np.uint8)
    br = rng.integers(0, 0x7E, (N, Kd)).astype(np.uint8) | 0x80
    c1 = run_gemm(K, ar, br, M, N, Kd, 0.01, 0.02, out_f32=True)
    c2 = run_gemm(K, ar, br, M, N, Kd, 0.01, 0.02, out_f32=True)
    assert torch.equal(c1, c2)
    exact, sumabs = O.gemm_exact(ar, br)
    gemm_check(c1.cpu().numpy(), exact, sumabs, np.float32(np.float32(0.01) * np.float32(0.02)), False)


@pytest.mark.parametrize("variant", [(0, 0), (1, 1, 1), (2, 2), (3, 1), (4, 0), (5, 0)])
def test_gemm_e5m2_b_operand(K, O, variant):
    """a e4m3, b e5m2 (src/kernels/kernels.h:92-94): small integers are exact in both formats ->
    bit-exact against the oracle; random codes within the stated tolerance of the exact product.  Selectors 4
    and 5 are the narrow tiles (bf16 output only: their fp32 check runs on the automatic choice)."""
    M, N, Kd = {4: (448, 768, 768), 5: (576, 768, 768)}.get(variant[0], (512, 768, 768))
    rng = np.random.default_rng(91)
    ai, bi = rng.integers(-4, 5, (M, Kd)), rng.integers(-4, 5, (N, Kd))
    enc4 = {v: O.lib().orc_e4m3_encode(float(v)) for v in range(-4, 5)}
    enc5 = {v: O.lib().orc_e5m2_encode(float(v)) for v in range(-4, 5)}
    a = np.vectorize(enc4.get)(ai).astype(np.uint8)
    b = np.vectorize(enc5.get)(bi).astype(np.uint8)
    s = float(np.sqrt(np.float32(4.0 / Kd)))
    _, biasv = O.fill_int_e4m3(M, 91, 2)
    bias = O.f32_to_bf16(biasv.astype(np.float32))
    set_variant(variant)
    try:
        want = O.gemm_tn(a, b, sa=s, sb=s, bias=bias, mt=True, b_e5m2=True)
        c = torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
        mm(K, c, dev_u8(a), dev_u8(b).view(torch.float8_e5m2), dev_bf16(bias), dev_scalar(s), dev_scalar(s), M, N, Kd,
                 workspace=workspace())
        assert np.array_equal(host_bits(c), want)
        # same integers: the e5m2 result must equal the int64 product, i.e. differ from reading b as e4m3
        ar = rng.integers(0, 256, (M, Kd)).astype(np.uint8)
        br = rng.integers(0, 256, (N, Kd)).astype(np.uint8)
        ar[(ar & 0x7F) == 0x7F] ^= 1
        br[(br & 0x7C) == 0x7C] ^= 0x40                      # no Inf / NaN codes
        br &= 0xBF                                           # magnitudes below 2: products stay modest
        exact, sumabs = O.gemm_exact(ar, br, b_e5m2=True)
        if variant[0] in (4, 5):
            c16 = torch.empty((N, M), dtype=torch.bfloat16, device="cuda")
            mm(K, c16, dev_u8(ar), dev_u8(br), None, dev_scalar(0.25), None, M, N, Kd, workspace=workspace(), b_e5m2=True)
            gemm_check(c16.float().cpu().numpy(), exact, sumabs, 0.25, True)
        else:
            c32 = torch.empty((N, M), dtype=torch.float32, device="cuda")
            mm(K, c32, dev_u8(ar), dev_u8(br), None, dev_scalar(0.25), None, M, N, Kd, workspace=workspace(), b_e5m2=True)
            gemm_check(c32.cpu().numpy(), exact, sumabs, 0.25, False)
    finally:
        set_variant((0, 0))


def test_gemm_matches_swapped_operand_transpose(K, O):
    """c(a,b)^T == c(b,a): a size-independent identity that catches row/column mix-ups."""
    M, N, Kd = 384, 640, 256
    rng = np.random.default_rng(2)
    a = rng.integers(0, 0x7E, (M, Kd)).astype(np.uint8) | (rng.integers(0, 2, (M, Kd)).astype(np.uint8) << 7)
    b = rng.integers(0, 0x7E, (N, Kd)).astype(np.uint8) | (rng.integers(0, 2, (N, Kd)).astype(np.uint8) << 7)
    c1 = run_gemm(K, a, b, M, N, Kd, 0.01, 0.5, out_f32=True)
    c2 = run_gemm(K, b, a, N, M, Kd, 0.5, 0.01, out_f32=True)
    assert torch.allclose(c1, c2.T, rtol=1e-5, atol=1e-4)


GENERAL_SHAPES = [(144, 272, 400), (1152, 8192, 896), (896, 2048, 896), (1024, 512, 896), (512, 256, 384),
                  (256, 1000, 512), (3584, 300, 256), (8, 8, 16), (1, 1, 16), (130, 70, 48), (200, 264, 1024), (448, 520, 640),
                  (2112, 2064, 656), (2112, 4104, 528), (1000, 4104, 400), (2056, 2049, 400), (2296, 2303, 496),
                  (4104, 1025, 640)]


RAGGED_SHAPES = [(264, 300, 384), (1000, 1000, 400), (1000, 520, 1040), (512, 776, 3600), (1000, 8192, 3584), (2056, 4100, 1552),
                 (4360, 4100, 656), (3584, 8200, 3600), (1032, 72, 48), (136, 5000, 112)]


@pytest.mark.parametrize("mnk", RAGGED_SHAPES)
def test_gemm_off_lattice_kernels_agree(K, O, mnk):
    """Shapes off the tile lattice have three kernels: the ragged instances of the four-wave kernel (moved-back 256 x 256
    tiles, masked last K-step) and of the 128 x 128 tiles (clamped rows, zero chunks beyond K), and the 64 x 64 kernel.
    The dispatch picks by estimated time; here each is forced in turn (test-aid build) on integer operands and all must
    give the same bits for bf16 and fp32 output, with bias and with accumulation -- and the first shape's bits are the
    oracle's.  (test_gemm_general_shapes compares the automatic choice with the oracle on further shapes.)"""
    M, N, Kd = mnk
    a, _ = O.fill_int_e4m3(M * Kd, 77, 0)
    b, _ = O.fill_int_e4m3(N * Kd, 77, 1)
    a, b = a.reshape(M, Kd), b.reshape(N, Kd)
    s = float(np.sqrt(np.float32(4.0 / Kd)))
    _, biasv = O.fill_int_e4m3(M, 77, 2)
    _, oldv = O.fill_int_e4m3(N * M, 77, 3)
    bias = O.f32_to_bf16(biasv.astype(np.float32))
    old = O.f32_to_bf16(oldv.astype(np.float32)).reshape(N, M)
    old32 = oldv.astype(np.float32).reshape(N, M)
    four_wave = M >= 256 and N >= 256 and Kd >= 384
    results = {}
    try:
        for tile in (6, 2) + ((3,) if four_wave else ()):
            set_variant((tile, 0))
            results[tile] = [host_bits(run_gemm(K, a, b, M, N, Kd, s, s)),
                             host_bits(run_gemm(K, a, b, M, N, Kd, s, s, bias)),
                             host_bits(run_gemm(K, a, b, M, N, Kd, s, s, bias, old)),
                             run_gemm(K, a, b, M, N, Kd, s, s, out_f32=True).cpu().numpy(),
                             run_gemm(K, a, b, M, N, Kd, None, None, bias, old32, out_f32=True).cpu().numpy()]
    finally:
        set_variant((0, 0))
    for tile in results:
        for i, (x, y) in enumerate(zip(results[6], results[tile])):
            assert np.array_equal(x, y), (tile, i)
    if mnk == RAGGED_SHAPES[0]:
        assert np.array_equal(results[6][2], O.gemm_tn(a, b, sa=s, sb=s, bias=bias, c_old=old))
    if four_wave:
        set_variant((3, 0))
        try:
            with pytest.raises(ValueError):   # two K-steps: fewer than the ragged four-wave instances walk
                run_gemm(K, a[:, :256].copy(), b[:, :256].copy(), M, N, 256, s, s)
        finally:
            set_variant((0, 0))


@pytest.mark.parametrize("mnk", GENERAL_SHAPES)
def test_gemm_general_shapes(K, O, mnk):
    """The reference's default backend serves every FP8 shape with 16-byte aligned rows
    (src/kernels/matmul.cpp:55-57, 160-184).  Here: M, K off the 128 lattice or N below 128 -> the general-shape
    kernel; a ragged N on top of regular M, K -> tiled kernels for the rows before the last N % 128, general-shape
    kernel for those; K an odd multiple of 128 -> the four-wave kernel's odd-K instances ((1152, 8192, 896) and
    (896, 2048, 896) on its 192- and 224-wide tiles, (1024, 512, 896) on the full tile); the last six shapes (64 and
    more 256 x 256 tiles; M 8 or 248 past a tile boundary, N 1 or 255 past one, so that moved-back tiles overlap their
    neighbours by almost a whole tile or by one row; K tails of 16 and 112 bytes and none; even and odd K-step counts)
    -> the four-wave kernel's ragged instances.  Integer operands -> bit
    exact against the oracle for bf16 / fp32 output with bias and accumulation; random codes within the tolerance."""
    M, N, Kd = mnk
    a, _ = O.fill_int_e4m3(M * Kd, 2024, 0)
    b, _ = O.fill_int_e4m3(N * Kd, 2024, 1)
    a, b = a.reshape(M, Kd), b.reshape(N, Kd)
    s = float(np.sqrt(np.float32(4.0 / Kd)))
    _, biasv = O.fill_int_e4m3(M, 2024, 2)
    _, oldv = O.fill_int_e4m3(N * M, 2024, 3)
    bias = O.f32_to_bf16(biasv.astype(np.float32))
    old = O.f32_to_bf16(oldv.astype(np.float32)).reshape(N, M)
    mt = M % 64 == 0
    for use_bias, use_old in [(False, False), (True, False), (True, True)]:
        want = O.gemm_tn(a, b, sa=s, sb=s, bias=bias if use_bias else None, c_old=old if use_old else None, mt=mt)
        got = run_gemm(K, a, b, M, N, Kd, s, s, bias if use_bias else None, old if use_old else None)
        assert np.array_equal(host_bits(got), want), (use_bias, use_old)
    got32 = run_gemm(K, a, b, M, N, Kd, s, s, out_f32=True)
    assert np.array_equal(got32.cpu().numpy(), O.gemm_tn(a, b, sa=s, sb=s, out_f32=True, mt=mt))
    got32 = run_gemm(K, a, b, M, N, Kd, None, None, bias, oldv.astype(np.float32), out_f32=True)
    want32 = O.gemm_tn(a, b, bias=bias, c_old=oldv.astype(np.float32).reshape(N, M), out_f32=True, mt=mt)
    assert np.array_equal(got32.cpu().numpy(), want32)
    if M * N <= 1 << 21:
        rng = np.random.default_rng(M + N + Kd)
        ar = rng.integers(0, 256, (M, Kd)).astype(np.uint8)
        br = rng.integers(0, 256, (N, Kd)).astype(np.uint8)
        ar[(ar & 0x7F) == 0x7F] ^= 1
        br[(br & 0x7F) == 0x7F] ^= 1
        exact, sumabs = O.gemm_exact(ar, br)
        g16 = run_gemm(K, ar, br, M, N, Kd, 0.37, 1.0 / 448).float().cpu().numpy()
        gemm_check(g16, exact, sumabs, np.float32(np.float32(0.37) * np.float32(1.0 / 448)), True)
        # e5m2 second operand on the same shapes
        br5 = br.copy()
        br5[(br5 & 0x7C) == 0x7C] ^= 0x40
        br5 &= 0xBF
        exact5, sumabs5 = O.gemm_exact(ar, br5, b_e5m2=True)
        c5 = torch.empty((N, M), dtype=torch.float32, device="cuda")
        mm(K, c5, dev_u8(ar), dev_u8(br5), None, dev_scalar(0.25), None, M, N, Kd, workspace=workspace(), b_e5m2=True)
        gemm_check(c5.cpu().numpy(), exact5, sumabs5, 0.25, False)


def _swept_shapes():
    """Seeded shapes around the edges of the dispatch's lattice: M on or just off multiples of 128 / 192 / 224 / 256, N
    with every kind of remainder, K any multiple of 16 (one K-step, odd and even step counts, not a multiple of 128)."""
    rng = np.random.default_rng(20260)
    shapes = []
    for _ in range(28):
        base_m = int(rng.choice([128, 192, 224, 256, 384, 448, 512, 640, 768]))
        M = max(1, base_m + int(rng.choice([0, 0, 0, 0, -8, 8, -1, 1, 16])))
        N = int(rng.choice([1, 17, 64, 127, 128, 129, 200, 255, 256, 257, 300, 384, 511, 512, 520, 640, 777]))
        Kd = 16 * int(rng.choice([1, 2, 5, 8, 9, 16, 17, 24, 32, 40, 48, 56, 64]))
        shapes.append((M, N, Kd))
    return shapes


@pytest.mark.parametrize("mnk", _swept_shapes())
def test_gemm_swept_shapes_exact_and_inside_their_rows(K, O, mnk):
    """Integer operands -> bit exact against the oracle, for whatever mix of tiled and general-shape launches the
    dispatch picks; the output sits between guard rows that must come back untouched (a kernel that wrote past its
    part of c, e.g. the tiled part into the remainder rows' neighbours, would show here)."""
    M, N, Kd = mnk
    a, _ = O.fill_int_e4m3(M * Kd, 909, 0)
    b, _ = O.fill_int_e4m3(N * Kd, 909, 1)
    a, b = a.reshape(M, Kd), b.reshape(N, Kd)
    s = float(np.sqrt(np.float32(4.0 / Kd)))
    _, biasv = O.fill_int_e4m3(M, 909, 2)
    bias = O.f32_to_bf16(biasv.astype(np.float32))
    pad = 8                                              # 8 rows of M bf16 / fp32 values: the interior stays 16-byte aligned
    for out_f32, use_bias in ((False, False), (False, True), (True, True)):
        dt = torch.float32 if out_f32 else torch.bfloat16
        guard = -7.0 if out_f32 else -1.5
        big = torch.full((N + 2 * pad, M), guard, dtype=dt, device="cuda")
        c = big[pad:pad + N]
        assert c.data_ptr() % 16 == 0                  # only the base of c has to be aligned; an odd M gives unaligned rows
        mm(K, c, dev_u8(a), dev_u8(b), dev_bf16(bias) if use_bias else None, dev_scalar(s), dev_scalar(s), M, N, Kd,
           workspace=workspace())
        torch.cuda.synchronize()
        want = O.gemm_tn(a, b, sa=s, sb=s, bias=bias if use_bias else None, out_f32=out_f32, mt=False)
        got = c.cpu().numpy() if out_f32 else host_bits(c)
        assert np.array_equal(got, want), (out_f32, use_bias)
        assert bool((big[:pad] == guard).all()) and bool((big[pad + N:] == guard).all()), "guard rows were written"


@pytest.mark.parametrize("mode", ["TT", "NN", "NT"])
@pytest.mark.parametrize("mnk", [(256, 256, 256), (512, 768, 512), (448, 512, 768), (1024, 2048, 1024), (2304, 512, 2816),
                                 (3584, 4096, 512), (576, 768, 512), (1536, 16384, 256)])
def test_gemm_operands_in_k_major_layout(K, O, mnk, mode):
    """Modes TT / NN / NT of the reference's matmul signature (src/kernels/kernels.h:22, matmul.cpp:66-67): b stored
    [K, N] and / or a stored [K, M] row-major, read through transposing LDS reads instead of a materialised transpose
    (what backward_qmm does with the output gradient, the weight and the activation,
    src/models/llama_model.cpp:309-339).  Integer operands -> bit exact against the oracle, with bias and (mode TT)
    accumulation; random codes (e5m2 included) within the tolerance of the exact product, bit-identical to mode TN on
    the transposed copies when that runs on the same kernel family (same sums in the same order), and the same bits on
    every one of 8 repeated launches."""
    M, N, Kd = mnk
    a_km, b_km = mode[0] == "N", mode[1] == "T"
    if a_km and b_km and M % 256:
        pytest.skip("two K-major operands are served on 256-wide tiles only")
    if not a_km and M % 256 and M % 224:
        pytest.skip("mode TT has 256- and 224-wide tiles")
    if mnk == (1536, 16384, 256) and mode != "NN":
        pytest.skip("this shape is here for mode NN's automatic choice of 192-wide tiles")
    lay_a = (lambda x: np.ascontiguousarray(x.T)) if a_km else (lambda x: x)      # [K, M]: what the caller holds
    lay_b = (lambda x: np.ascontiguousarray(x.T)) if b_km else (lambda x: x)      # [K, N]
    a, _ = O.fill_int_e4m3(M * Kd, 606, 0)
    b, _ = O.fill_int_e4m3(N * Kd, 606, 1)
    a, b = a.reshape(M, Kd), b.reshape(N, Kd)
    s = float(np.sqrt(np.float32(4.0 / Kd)))
    _, biasv = O.fill_int_e4m3(M, 606, 2)
    _, oldv = O.fill_int_e4m3(N * M, 606, 3)
    bias = O.f32_to_bf16(biasv.astype(np.float32))
    old = O.f32_to_bf16(oldv.astype(np.float32)).reshape(N, M)
    mt = M % 64 == 0
    cases = [(False, False), (True, False)] + ([(True, True)] if M % 256 == 0 else [])
    for use_bias, use_old in cases:
        want = O.gemm_tn(a, b, sa=s, sb=s, bias=bias if use_bias else None, c_old=old if use_old else None, mt=mt)
        c = dev_bf16(old).reshape(N, M).clone() if use_old else torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
        K.matmul(c, dev_u8(lay_a(a)), dev_u8(lay_b(b)), dev_bf16(bias) if use_bias else None, dev_scalar(s), dev_scalar(s), M, N, Kd,
                 accumulate=use_old, a_kmajor=a_km, b_kmajor=b_km)
        assert np.array_equal(host_bits(c), want), (use_bias, use_old)
    rng = np.random.default_rng(M + Kd)
    for e5m2 in (False, True):
        ar = rng.integers(0, 256, (M, Kd)).astype(np.uint8)
        br = rng.integers(0, 256, (N, Kd)).astype(np.uint8)
        ar[(ar & 0x7F) == 0x7F] ^= 1
        if e5m2:
            br[(br & 0x7C) == 0x7C] ^= 0x40
            br &= 0xBF
        else:
            br[(br & 0x7F) == 0x7F] ^= 1
        da, db = dev_u8(lay_a(ar)), dev_u8(lay_b(br))
        c_tn = torch.empty((N, M), dtype=torch.bfloat16, device="cuda")
        c_km = torch.empty((N, M), dtype=torch.bfloat16, device="cuda")
        K.matmul(c_km, da, db, None, dev_scalar(0.37), dev_scalar(1.0 / 448), M, N, Kd, b_e5m2=e5m2, a_kmajor=a_km, b_kmajor=b_km)
        exact, sumabs = O.gemm_exact(ar, br, b_e5m2=e5m2)
        gemm_check(c_km.float().cpu().numpy(), exact, sumabs, np.float32(np.float32(0.37) * np.float32(1.0 / 448)), True)
        # mode TN on the same kernel family: the same sums in the same order (without a cut of the last round the sums
        # do not depend on the tile width)
        set_variant(((4, 0) if M % 224 == 0 else (5, 0)) if M % 256 else (3, 1))
        try:
            mm(K, c_tn, dev_u8(ar), dev_u8(br), None, dev_scalar(0.37), dev_scalar(1.0 / 448), M, N, Kd, b_e5m2=e5m2)
        finally:
            set_variant((0, 0))
        assert torch.equal(c_tn.view(torch.int16), c_km.view(torch.int16)), e5m2
        for _ in range(8):                                  # repeated launches: the same bits every time
            again = torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
            K.matmul(again, da, db, None, dev_scalar(0.37), dev_scalar(1.0 / 448), M, N, Kd, b_e5m2=e5m2, a_kmajor=a_km,
                     b_kmajor=b_km)
            assert torch.equal(again.view(torch.int16), c_km.view(torch.int16)), e5m2


@pytest.mark.parametrize("mode", ["TT", "NN", "NT"])
@pytest.mark.parametrize("mnk", [(256, 256, 256), (512, 768, 512), (1024, 2048, 1024), (4352, 4352, 1024), (4608, 4096, 512)])
def test_gemm_k_major_fp32_output_and_accumulation(K, O, mnk, mode):
    """The K-major modes with fp32 output and with accumulation into c (the reference's matmul takes every mode with
    either, src/kernels/matmul.cpp:66-92: fp32 weight gradients, gradient-accumulation micro-steps).  With a K-major
    first operand these go through the fp32-staged epilogue.  Integer operands -> bit exact against the oracle (bias,
    old values, both output types, with and without a workspace, i.e. with the last round cut where the plan cuts it);
    random codes -> bit-identical to mode TN on the transposed copies under the same plan, launch after launch."""
    M, N, Kd = mnk
    a_km, b_km = mode[0] == "N", mode[1] == "T"
    lay_a = (lambda x: np.ascontiguousarray(x.T)) if a_km else (lambda x: x)
    lay_b = (lambda x: np.ascontiguousarray(x.T)) if b_km else (lambda x: x)
    a, _ = O.fill_int_e4m3(M * Kd, 919, 0)
    b, _ = O.fill_int_e4m3(N * Kd, 919, 1)
    a, b = a.reshape(M, Kd), b.reshape(N, Kd)
    s = float(np.sqrt(np.float32(4.0 / Kd)))
    _, biasv = O.fill_int_e4m3(M, 919, 2)
    _, oldv = O.fill_int_e4m3(N * M, 919, 3)
    bias = O.f32_to_bf16(biasv.astype(np.float32))
    oldf = oldv.astype(np.float32).reshape(N, M)
    for out_f32, use_bias, use_old, with_ws in [(True, False, False, False), (True, True, True, True), (True, False, True, False),
                                                (False, True, True, False), (False, False, True, True)]:
        old = (oldf if out_f32 else O.f32_to_bf16(oldf).reshape(N, M)) if use_old else None
        want = O.gemm_tn(a, b, sa=s, sb=s, bias=bias if use_bias else None, c_old=old, out_f32=out_f32, mt=True)
        dt = torch.float32 if out_f32 else torch.bfloat16
        if use_old:
            c = (torch.from_numpy(old).cuda() if out_f32 else dev_bf16(old)).reshape(N, M).clone()
        else:
            c = torch.full((N, M), float("nan"), dtype=dt, device="cuda")
        K.matmul(c, dev_u8(lay_a(a)), dev_u8(lay_b(b)), dev_bf16(bias) if use_bias else None, dev_scalar(s), dev_scalar(s), M, N, Kd,
                 accumulate=use_old, a_kmajor=a_km, b_kmajor=b_km, workspace=workspace() if with_ws else None)
        got = c.cpu().numpy() if out_f32 else host_bits(c)
        assert np.array_equal(got, want), (out_f32, use_bias, use_old, with_ws)
    rng = np.random.default_rng(M + N)
    ar = rng.integers(0, 256, (M, Kd)).astype(np.uint8)
    br = rng.integers(0, 256, (N, Kd)).astype(np.uint8)
    ar[(ar & 0x7F) == 0x7F] ^= 1
    br[(br & 0x7F) == 0x7F] ^= 1
    start = torch.from_numpy(rng.standard_normal((N, M)).astype(np.float32)).cuda()
    set_variant((3, 0))                       # mode TN on the four-wave kernel: the same sums in the same order
    try:
        c_tn = start.clone()
        mm(K, c_tn, dev_u8(ar), dev_u8(br), None, dev_scalar(0.37), dev_scalar(1.0 / 448), M, N, Kd, accumulate=True, workspace=workspace())
        for _ in range(3):
            c_km = start.clone()
            mm(K, c_km, dev_u8(lay_a(ar)), dev_u8(lay_b(br)), None, dev_scalar(0.37), dev_scalar(1.0 / 448), M, N, Kd, accumulate=True,
               a_kmajor=a_km, b_kmajor=b_km, workspace=workspace())
            assert torch.equal(c_tn.view(torch.int32), c_km.view(torch.int32))
    finally:
        set_variant((0, 0))


@pytest.mark.parametrize("mode", ["TT", "NN", "NT"])
@pytest.mark.parametrize("cut", [0, 2, 4])
@pytest.mark.parametrize("mnk", [(4352, 4352, 1024), (4608, 4096, 512), (4352, 4096, 1536), (8192, 4864, 512)])
def test_gemm_k_major_last_round_cut(K, O, mnk, mode, cut):
    """K-major operands with a workspace: the tiles left over after the full rounds are cut into K segments (a
    second launch of the same operand mode writing raw fp32 tiles, summed in a fixed order by the reduction kernel),
    as in mode TN.  cut = 2, 4: forced; 0: whatever the plan decides with the workspace given.  Integer operands ->
    bit exact against the oracle, with bias and accumulation; random codes bit-identical to mode TN under
    the same plan, and on repeated launches."""
    M, N, Kd = mnk
    variant = (3, cut)          # mode TN on the four-wave kernel as well: the same sums in the same order
    skip_unsupported(variant, M, N, Kd)
    a_km, b_km = mode[0] == "N", mode[1] == "T"
    lay_a = (lambda x: np.ascontiguousarray(x.T)) if a_km else (lambda x: x)
    lay_b = (lambda x: np.ascontiguousarray(x.T)) if b_km else (lambda x: x)
    a, _ = O.fill_int_e4m3(M * Kd, 818, 0)
    b, _ = O.fill_int_e4m3(N * Kd, 818, 1)
    a, b = a.reshape(M, Kd), b.reshape(N, Kd)
    s = float(np.sqrt(np.float32(4.0 / Kd)))
    _, biasv = O.fill_int_e4m3(M, 818, 2)
    _, oldv = O.fill_int_e4m3(N * M, 818, 3)
    bias = O.f32_to_bf16(biasv.astype(np.float32))
    old = O.f32_to_bf16(oldv.astype(np.float32)).reshape(N, M)
    rng = np.random.default_rng(M + N + Kd)
    ar = rng.integers(0, 256, (M, Kd)).astype(np.uint8)
    br = rng.integers(0, 256, (N, Kd)).astype(np.uint8)
    ar[(ar & 0x7F) == 0x7F] ^= 1
    br[(br & 0x7F) == 0x7F] ^= 1
    set_variant(variant)
    try:
        for use_bias, use_old in [(False, False), (True, False), (True, True)]:
            want = O.gemm_tn(a, b, sa=s, sb=s, bias=bias if use_bias else None, c_old=old if use_old else None, mt=True)
            c = dev_bf16(old).reshape(N, M).clone() if use_old else torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
            mm(K, c, dev_u8(lay_a(a)), dev_u8(lay_b(b)), dev_bf16(bias) if use_bias else None, dev_scalar(s), dev_scalar(s), M, N, Kd,
               accumulate=use_old, a_kmajor=a_km, b_kmajor=b_km, workspace=workspace())
            assert np.array_equal(host_bits(c), want), (use_bias, use_old)
        c_tn = torch.empty((N, M), dtype=torch.bfloat16, device="cuda")
        mm(K, c_tn, dev_u8(ar), dev_u8(br), None, dev_scalar(0.37), dev_scalar(1.0 / 448), M, N, Kd, workspace=workspace())
        da, db = dev_u8(lay_a(ar)), dev_u8(lay_b(br))
        for _ in range(4):
            c_km = torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
            mm(K, c_km, da, db, None, dev_scalar(0.37), dev_scalar(1.0 / 448), M, N, Kd, a_kmajor=a_km, b_kmajor=b_km,
               workspace=workspace())
            assert torch.equal(c_tn.view(torch.int16), c_km.view(torch.int16))
    finally:
        set_variant((0, 0))


@pytest.mark.parametrize("mode", ["TT", "NN", "NT"])
def test_gemm_k_major_automatic_cut_on_a_weight_gradient_shape(K, mode):
    """18944 x 3584 x 8192 (the down projection's weight gradient of the headline layer): with a workspace the plan
    cuts the one or two last-round tiles per XCD into K segments in every operand mode; the K-major modes must give
    the bits of mode TN on the transposed copies (same plan, same sums in the same order), launch after launch."""
    M, N, Kd = 18944, 3584, 8192
    g = torch.Generator(device="cuda").manual_seed(5)
    a = torch.randint(0, 0x7E, (M, Kd), dtype=torch.uint8, device="cuda", generator=g) | (torch.randint(0, 2, (M, Kd), dtype=torch.uint8, device="cuda", generator=g) << 7)
    b = torch.randint(0, 0x7E, (N, Kd), dtype=torch.uint8, device="cuda", generator=g) | (torch.randint(0, 2, (N, Kd), dtype=torch.uint8, device="cuda", generator=g) << 7)
    a_km, b_km = mode[0] == "N", mode[1] == "T"
    da = a.t().contiguous() if a_km else a
    db = b.t().contiguous() if b_km else b
    sa = dev_scalar(2.0 ** -6)
    c_tn = torch.empty((N, M), dtype=torch.bfloat16, device="cuda")
    K.matmul(c_tn, a, b, None, sa, None, M, N, Kd, workspace=workspace())
    c_whole = torch.empty((N, M), dtype=torch.bfloat16, device="cuda")
    K.matmul(c_whole, da, db, None, sa, None, M, N, Kd, a_kmajor=a_km, b_kmajor=b_km)
    for _ in range(4):
        c_km = torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
        K.matmul(c_km, da, db, None, sa, None, M, N, Kd, a_kmajor=a_km, b_kmajor=b_km, workspace=workspace())
        assert torch.equal(c_tn.view(torch.int16), c_km.view(torch.int16))
    # the cut changes the order of the sums in the cut tiles only: a few outputs differ from the uncut launch by an ulp
    differing = (c_whole.view(torch.int16) != c_tn.view(torch.int16)).float().mean().item()
    assert 0 < differing < 0.02, differing


FUSED_EPILOGUE_SHAPES = [(256, 256, 256), (256, 256, 384), (512, 768, 896), (4352, 4352, 512), (4352, 4096, 1024), (4608, 4096, 256),
                         (8192, 4608, 1536), (4352, 4352, 640), (9728, 8192, 896), (18944, 3584, 8192)]


@pytest.mark.parametrize("mnk", FUSED_EPILOGUE_SHAPES)
def test_gemm_epilogue_under_matrix_instructions_matches_epilogue_after_the_loop(K, O, mnk):
    """The four-wave kernel writes full-width bf16 tiles (no bias, no accumulation) out under matrix instructions: rows
    0..3 under the tile's last K-step, rows 4..7 under the next tile's first K-step, the last tile's on their own.  Same
    arithmetic in the same order as the epilogue after the K loop, so the two instances must agree bit for bit: one tile
    and many per workgroup, two K-steps per tile (the last step follows the first directly), odd K-step counts, a cut
    last round; repeated launches; and integer-valued operands against the exact product."""
    from llmq_amd import capi
    M, N, Kd = mnk
    t = capi.testaid()
    g = torch.Generator(device="cuda").manual_seed(M + N + Kd)
    a = torch.randint(0, 0x7E, (M, Kd), dtype=torch.uint8, device="cuda", generator=g) | (torch.randint(0, 2, (M, Kd), dtype=torch.uint8, device="cuda", generator=g) << 7)
    b = torch.randint(0, 0x7E, (N, Kd), dtype=torch.uint8, device="cuda", generator=g) | (torch.randint(0, 2, (N, Kd), dtype=torch.uint8, device="cuda", generator=g) << 7)
    sa = dev_scalar(2.0 ** -7 * 1.37)
    try:
        with gemm_library(t):
            t.llmq_debug_set_gemm_fuse(0)
            c0 = torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
            K.matmul(c0, a, b, None, sa, None, M, N, Kd, workspace=workspace())
            t.llmq_debug_set_gemm_fuse(1)
            for _ in range(3):
                c1 = torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
                K.matmul(c1, a, b, None, sa, None, M, N, Kd, workspace=workspace())
                assert torch.equal(c0.view(torch.int16), c1.view(torch.int16))
            if M * N * Kd <= 4352 * 4352 * 1024:
                ai, _ = O.fill_int_e4m3(M * Kd, 7 + M, 0)
                bi, _ = O.fill_int_e4m3(N * Kd, 7 + N, 1)
                ai, bi = ai.reshape(M, Kd), bi.reshape(N, Kd)
                s = float(np.sqrt(np.float32(4.0 / Kd)))
                want = O.gemm_tn(ai, bi, sa=s, sb=s, mt=True)
                c2 = torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
                K.matmul(c2, dev_u8(ai), dev_u8(bi), None, dev_scalar(s), dev_scalar(s), M, N, Kd, workspace=workspace())
                assert np.array_equal(host_bits(c2), want)
    finally:
        t.llmq_debug_set_gemm_fuse(-1)


def test_product_library_cuts_the_last_round_into_k_segments(K):
    """The K-segment instance of the four-wave kernel, reached on the product library through the automatic plan (no
    forced variant): 18944 x 3584 x 8192 leaves one or two tiles per XCD for the last round, and with a workspace the
    plan cuts them.  Proof that the segment launch ran: it is the only kernel that writes the workspace, so the
    workspace (filled with a pattern no partial sum has) must afterwards hold 12 S partial tiles of 256 KiB (XCDs 0-3
    have two last-round tiles, XCDs 4-7 one; S segments each), S >= 2, in the places the plan reserves per XCD.
    Integer-valued operands: every sum is exact in fp32 in any order, so the cut result must equal the uncut one and
    the int64 product bit for bit."""
    M, N, Kd = 18944, 3584, 8192
    g = torch.Generator(device="cuda").manual_seed(77)
    ints = torch.tensor([0x00, 0x38, 0x40, 0x44, 0x48, 0xB8, 0xC0, 0xC4], dtype=torch.uint8, device="cuda")   # 0, 1, 2, 3, 4, -1, -2, -3
    vals = torch.tensor([0, 1, 2, 3, 4, -1, -2, -3], dtype=torch.float64)
    ia = torch.randint(0, 8, (M, Kd), device="cuda", generator=g)
    ib = torch.randint(0, 8, (N, Kd), device="cuda", generator=g)
    a, b = ints[ia], ints[ib]
    ws = torch.full((32 << 20,), 0xFF, dtype=torch.uint8, device="cuda")
    c_cut = torch.full((N, M), float("nan"), dtype=torch.float32, device="cuda")
    K.matmul(c_cut, a, b, None, None, None, M, N, Kd, workspace=ws)
    c_whole = torch.full((N, M), float("nan"), dtype=torch.float32, device="cuda")
    K.matmul(c_whole, a, b, None, None, None, M, N, Kd)
    torch.cuda.synchronize()
    touched = (ws.view(128, 256 * 1024) != 0xFF).any(dim=1).cpu().numpy()
    n_touched = int(touched.sum())
    assert n_touched >= 24 and n_touched % 12 == 0, n_touched        # 12 tiles x S segments, S >= 2
    S = n_touched // 12
    expect = np.zeros(128, dtype=bool)
    for xcd in range(8):
        rem = 2 if xcd < 4 else 1
        expect[xcd * 2 * S: xcd * 2 * S + rem * S] = True            # part_per_xcd = rem_max * S = 2 S
    assert np.array_equal(touched, expect), (S, np.flatnonzero(touched))
    assert torch.equal(c_cut, c_whole)
    # the last-round tiles and a sample of the others against the int64 product
    rows = np.r_[0:8, 1700:1708, N - 256:N - 248, N - 8:N]
    want = (vals[ib[rows].cpu()] @ vals[ia.cpu()].T).numpy()
    assert np.array_equal(c_cut[rows].cpu().numpy().astype(np.float64), want)


@pytest.mark.parametrize("mode", ["TT", "NN"])
def test_gemm_k_major_operand_near_the_size_limit(K, mode):
    """A K-major operand of 1.88 GB (the lane offsets of its copies are 32-bit and walk the whole operand; 2 GiB is the
    documented limit): the result must equal mode TN on the transposed copy bit for bit, including the tiles whose
    operand bytes lie at the far end."""
    big, small, Kd = 57344, 256, 32768
    M, N = (small, big) if mode == "TT" else (big, small)
    g = torch.Generator(device="cuda").manual_seed(11)
    codes = lambda r, c: torch.randint(0, 0x7E, (r, c), dtype=torch.uint8, device="cuda", generator=g)
    a, b = codes(M, Kd), codes(N, Kd)
    sa = dev_scalar(2.0 ** -9)
    c_tn = torch.empty((N, M), dtype=torch.bfloat16, device="cuda")
    K.matmul(c_tn, a, b, None, sa, None, M, N, Kd)
    if mode == "TT":
        b_km = b.t().contiguous()
        del b
        c_km = torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
        K.matmul(c_km, a, b_km, None, sa, None, M, N, Kd, b_kmajor=True)
    else:
        a_km = a.t().contiguous()
        del a
        c_km = torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
        K.matmul(c_km, a_km, b, None, sa, None, M, N, Kd, a_kmajor=True)
    assert torch.equal(c_tn.view(torch.int16), c_km.view(torch.int16))
    assert bool(torch.isfinite(c_km.float()).all()) and float(c_km.float().abs().max()) > 0


def test_gemm_k_major_operand_rejects_what_it_cannot_serve(K):
    a = torch.zeros((256, 384), dtype=torch.uint8, device="cuda")
    b = torch.zeros((384, 256), dtype=torch.uint8, device="cuda")
    c = torch.zeros((256, 256), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="mode TT"):
        K.matmul(c, a, b, None, None, None, 256, 256, 384, b_kmajor=True)      # K % 256 != 0
    with pytest.raises(ValueError, match="mode NN"):
        K.matmul(torch.zeros((256, 224), device="cuda"), torch.zeros((256, 224), dtype=torch.uint8, device="cuda"),
                 torch.zeros((256, 256), dtype=torch.uint8, device="cuda"), None, None, None, 224, 256, 256, a_kmajor=True)   # needs M % 256 == 0
    with pytest.raises(ValueError, match="mode TT"):
        K.matmul(torch.zeros((256, 224), device="cuda"), torch.zeros((224, 256), dtype=torch.uint8, device="cuda"),
                 torch.zeros((256, 256), dtype=torch.uint8, device="cuda"), None, None, None, 224, 256, 256, b_kmajor=True)   # 224-wide tiles: bf16 only
    # a bias that is too short would be read out of bounds by the epilogue: refused by the wrapper in every operand mode
    short_bias = torch.zeros(128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="bias must have M elements"):
        K.matmul(c, torch.zeros((256, 256), dtype=torch.uint8, device="cuda"), torch.zeros((256, 256), dtype=torch.uint8, device="cuda"),
                 short_bias, None, None, 256, 256, 256, b_kmajor=True)
    # a K-major operand of 2 GiB or more is refused before anything is launched (32-bit lane offsets walk it);
    # called through the C ABI with the sizes alone, no such tensor is allocated
    from llmq_amd import capi
    rc = capi.lib.llmq_gemm_e4m3_bf16_mode(c.data_ptr(), a.data_ptr(), b.data_ptr(), None, None, None, None, 0,
                                           256, 65536, 32768, 0, 0, 0, None)
    assert rc == capi.LLMQ_ERR_INVALID_ARGUMENT and b"2 GiB" in capi.lib.llmq_last_error()


def test_gemm_rejects_unaligned_k(K):
    a = torch.zeros((128, 72), dtype=torch.uint8, device="cuda")
    c = torch.zeros((128, 128), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="multiple of 16"):
        mm(K, c, a, a, None, None, None, 128, 128, 72)


# ------------------------------------------------------------------------------------ backward_bias
BIAS_SHAPES = [(10, 64), (3, 256), (32, 128), (128, 512), (8192, 1152), (8192, 4608), (5000, 16), (16384, 2560)]


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "bf16"])
@pytest.mark.parametrize("shape", BIAS_SHAPES)
def test_backward_bias(K, O, fmt, shape):
    """dbias += sa*sb * column sums of the (quantized) gradient, reference src/kernels/bias.cu:151-195 and
    its tests scripts/test_kernels.py:834-890 (plain, scaled, accumulating).  Integer-valued gradients
    make every fp32 partial sum exact -> bit-exact against the oracle; random gradients are checked
    against the exact column sums within fp32 accumulation + bf16 rounding error."""
    BT, OC = shape
    rng = np.random.default_rng(BT * 7 + OC)
    tdt = {"e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2, "bf16": torch.bfloat16}[fmt]
    buf = torch.empty(K.get_bias_backward_scratch_size(tdt, OC, BT) // 4 + 4, dtype=torch.float32, device="cuda")

    def dev(x):
        return dev_bf16(x) if fmt == "bf16" else dev_u8(x).view(tdt)

    ints = rng.integers(-3, 4, (BT, OC))
    if fmt == "bf16":
        di = O.f32_to_bf16(ints.astype(np.float32))
    else:
        enc = O.lib().orc_e4m3_encode if fmt == "e4m3" else O.lib().orc_e5m2_encode
        lut = np.array([enc(float(v)) for v in range(-3, 4)], dtype=np.uint8)
        di = lut[ints + 3]
    old = O.f32_to_bf16(rng.integers(-8, 9, OC).astype(np.float32))
    for sa, sb, use_old in [(None, None, False), (0.25, 2.0, False), (0.5, 4.0, True)]:
        start = old if use_old else np.zeros(OC, dtype=np.uint16)
        want, _, _ = O.backward_bias(start, di, fmt, sa, sb)
        dbias = dev_bf16(start).clone()
        buf.fill_(float("nan"))                       # the scratch never needs clearing
        K.backward_bias(dbias, dev(di), dev_scalar(sa) if sa is not None else None,
                        dev_scalar(sb) if sb is not None else None, buf)
        assert np.array_equal(host_bits(dbias), want), (sa, sb, use_old)
    # random values
    if fmt == "bf16":
        dr = O.fill_normal_bf16(BT * OC, 77, BT + OC, 0.0, 1.0).reshape(BT, OC)
    else:
        dr = rng.integers(0, 256, (BT, OC)).astype(np.uint8)
        dr[(dr & 0x7C) == 0x7C] ^= 0x40
    startf = rng.standard_normal(OC).astype(np.float32)
    start = O.f32_to_bf16(startf)
    _, cs, ca = O.backward_bias(start, dr, fmt, 0.125, 0.5)
    dbias = dev_bf16(start).clone()
    K.backward_bias(dbias, dev(dr), dev_scalar(0.125), dev_scalar(0.5), buf)
    got = O.bf16_to_f32(host_bits(dbias)).astype(np.float64)
    ref = cs * 0.0625 + O.bf16_to_f32(start).astype(np.float64)
    bound = 2.0 ** -8 * np.abs(ref) + 2.0 ** -18 * 0.0625 * ca + 1e-30
    assert np.all(np.abs(got - ref) <= bound), float(np.max(np.abs(got - ref) / bound))


def test_backward_bias_rejects_bad_arguments(K):
    g = torch.zeros((8, 64), dtype=torch.float8_e4m3fn, device="cuda")
    d = torch.zeros(64, dtype=torch.bfloat16, device="cuda")
    s = torch.ones(1, device="cuda")
    buf = torch.empty(K.get_bias_backward_scratch_size(torch.float8_e4m3fn, 64, 8) // 4, dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError):
        K.backward_bias(d, g, s, None, buf)                                   # one scale only (bias.cu:163-165)
    with pytest.raises(ValueError):
        K.backward_bias(d, g, None, None, buf[:1])                            # scratch too small (kernels.cpp:378-380)
    g2 = torch.zeros((8, 24), dtype=torch.float8_e4m3fn, device="cuda")
    with pytest.raises(ValueError):
        K.backward_bias(d[:24].contiguous(), g2, None, None, buf)             # OC % vector size (bias.cu:167-168)


# ----------------------------------------------------------------------- configuration 1, end to end
def test_config1_forward_pipeline(K, O):
    """X[4096x896]~N(0,1), W[4864x896]~N(0,0.02), seed 0: abs-max, quantize both, Y = X W^T (bf16)."""
    BT, C, OC = 4096, 896, 4864
    x = O.fill_normal_bf16(BT * C, 0, 1, 0.0, 1.0).reshape(BT, C)
    w = O.fill_normal_bf16(OC * C, 0, 2, 0.0, 0.02).reshape(OC, C)
    xd, wd = dev_bf16(x), dev_bf16(w)
    stats = torch.zeros(4, device="cuda")          # [x absmax, x scale, w absmax, w scale]
    xq = torch.empty((BT, C), dtype=torch.float8_e4m3fn, device="cuda")
    wq = torch.empty((OC, C), dtype=torch.float8_e4m3fn, device="cuda")
    y = torch.empty((BT, OC), dtype=torch.bfloat16, device="cuda")
    K.abs_max(stats[0:1], xd)
    K.abs_max(stats[2:3], wd)
    K.quantize_with_abs_max(xq, stats[1:2], xd, stats[0:1])
    K.quantize_with_abs_max(wq, stats[3:4], wd, stats[2:3])
    mm(K, y, wq, xq, None, stats[3:4], stats[1:2], OC, BT, C)       # forward_qmm call, llama_model.cpp:44
    torch.cuda.synchronize()
    st = stats.cpu().numpy()
    ax, aw = O.abs_max_bf16(x), O.abs_max_bf16(w)
    xq_o, dx = O.quantize_e4m3(x, ax, mt=True)
    wq_o, dw = O.quantize_e4m3(w, aw, mt=True)
    assert st[0] == np.float32(ax) and st[2] == np.float32(aw) and st[1] == dx and st[3] == dw
    assert np.array_equal(host_bits(xq), xq_o) and np.array_equal(host_bits(wq), wq_o)
    rng = np.random.default_rng(0)
    idx_n = np.concatenate([rng.integers(0, BT, 60000), np.full(OC, 4095), np.arange(BT)]).astype(np.int32)
    idx_m = np.concatenate([rng.integers(0, OC, 60000), np.arange(OC), np.full(BT, 4863)]).astype(np.int32)
    ex, sabs = O.gemm_exact_sampled(wq_o, xq_o, idx_n, idx_m)
    got = y.float().cpu().numpy()[idx_n, idx_m]
    scale = np.float32(dw * dx)
    max_abs, fro = gemm_check(got, ex, sabs, scale, True)
    report_gemm_error("config1", "forward y", BT, OC, C, max_abs, fro, "%d sampled outputs incl. boundary rows/columns" % idx_n.size)
    # Every one of the 4096 x 4864 outputs: the exact product as a float64 matrix product of the decoded codes (every
    # e4m3 product and every partial sum of 896 of them fits 53 bits, so the library routine returns the exact sums
    # in any order), tied to the oracle's exact sums on the sampled coordinates above.
    xf, wf = O.e4m3_decode(xq_o).astype(np.float64), O.e4m3_decode(wq_o).astype(np.float64)
    ex_all, sabs_all = xf @ wf.T, np.abs(xf) @ np.abs(wf).T
    assert np.array_equal(ex_all[idx_n, idx_m], ex) and np.array_equal(sabs_all[idx_n, idx_m], sabs)
    max_abs_all, fro_all = gemm_check(y.float().cpu().numpy(), ex_all, sabs_all, scale, True)
    report_gemm_error("config1", "forward y (all outputs)", BT, OC, C, max_abs_all, fro_all, "all %d outputs" % (BT * OC))
    del xf, wf, ex_all, sabs_all
    # closeness to the unquantised product, as a sanity check of the whole path (fp8 noise ~ 3-4 %)
    ref = (O.bf16_to_f32(x)[idx_n[:2000]].astype(np.float64) * O.bf16_to_f32(w)[idx_m[:2000]].astype(np.float64)).sum(1)
    rel = np.linalg.norm(got[:2000] - ref) / np.linalg.norm(ref)
    assert rel < 0.08, rel
