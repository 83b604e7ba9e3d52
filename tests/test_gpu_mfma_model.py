"""Pins the accumulation behaviour of the gfx950 FP8 matrix instructions that the stated GEMM tolerance
(tests/gpu_util.py: 2^-11 * sum|a b| per element) is derived from.

One-hot probes through the library's own GEMM: a dot product holds one large product P = 2^16 at position k0 and
one small product p = +-2^(16-d) at position k1, everything else is zero, no scales, fp32 output.  The exact sum
P + p is representable in fp32 for d <= 23, so any deviation is the instruction's doing.  Asserted model:

  * K positions form aligned groups of 8.  Inside a group the products are aligned to the group's largest and
    truncated 14 bits below its leading bit: p survives exactly for d <= 13 and vanishes for d >= 14.
  * Across groups (and K-steps) the sums are kept to full fp32 precision: p survives for d <= 23.

Consequence used by the tolerance: a group loses less than 7 * 2^-14 of its largest |product|, a dot product
less than 7 * 2^-14 * sum|a b| < 2^-11 * sum|a b|.  The last test drives a dot product to that worst case and
checks both that the loss is real (the 2^-20 bound of an ideal fp32 accumulation would fail) and that it stays
inside the stated bound.  Every kernel family (both matrix instructions) is probed, forced through the test-aid
build of the GEMM source; the automatic choice runs on the product library."""
import numpy as np
import pytest
import torch

from gpu_util import ACC_TERM, gemm_library

pytestmark = pytest.mark.gpu

KD = 256
# (tile selector, splits, persistent): automatic, 128 x 128 tiles and 256 x 256 tiles of the 8-wave kernel
# (v_mfma_f32_32x32x64_f8f6f4), the four-wave kernel (v_mfma_f32_16x16x128_f8f6f4)
VARIANTS = [(0, 0), (2, 0), (1, 0, 0), (3, 1)]


def code(v):
    """e4m3 code of a value that the format holds exactly."""
    t = torch.tensor([v], dtype=torch.float32).to(torch.float8_e4m3fn)
    assert float(t.float()) == v, v
    return int(t.view(torch.uint8))


def gemm_f32(variant, a, b):
    from llmq_amd import capi, kernels as K
    lib = None
    if variant != (0, 0):
        lib = capi.testaid()
        lib.llmq_debug_set_gemm_variant(variant[0], variant[1])
        lib.llmq_debug_set_gemm_persist(variant[2] if len(variant) > 2 else -1)
    try:
        M, N = a.shape[0], b.shape[0]
        c = torch.full((N, M), float("nan"), dtype=torch.float32, device="cuda")
        with gemm_library(lib):
            K.matmul(c, torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), None, None, None, M, N, a.shape[1])
        torch.cuda.synchronize()
        return c.cpu().numpy().astype(np.float64)
    finally:
        if lib is not None:
            lib.llmq_debug_set_gemm_variant(0, 0)
            lib.llmq_debug_set_gemm_persist(-1)


def probe(variant, k0, k1s, sign):
    """Returns {(k1, d): c - P} for P = 2^16 at k0 and p = sign * 2^(16-d) at k1, d = 0 .. 34.
    a row m carries 2^8 at k0 and sign * 2^(m-9) everywhere else; b row n carries 2^8 at k0 and 2^e at k1s[n]:
    c[n, m] = 2^16 + sign * 2^(m - 9 + e)."""
    out = {}
    for e in range(-9, 9):
        a = np.zeros((256, KD), np.uint8)
        b = np.zeros((256, KD), np.uint8)
        for m in range(18):
            a[m, :] = code(sign * 2.0 ** (m - 9))
            a[m, k0] = code(256.0)
        for n, k1 in enumerate(k1s):
            b[n, k0] = code(256.0)
            b[n, k1] = code(2.0 ** e)
        c = gemm_f32(variant, a, b)
        for m in range(18):
            d = 16 - (m - 9 + e)
            for n, k1 in enumerate(k1s):
                out.setdefault((k1, d), set()).add(c[n, m] - 65536.0)
    return out


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("k0", [0, 5, 130])
def test_products_are_truncated_14_bits_below_the_largest_of_their_group_of_8(variant, k0):
    g0 = k0 - k0 % 8
    same = [k for k in range(g0, g0 + 8) if k != k0]
    other = [g0 + 8, g0 + 15, (g0 + 64) % KD, (g0 + 127) % KD, (g0 + 128) % KD, (g0 - 1) % KD]
    for sign in (1.0, -1.0):
        got = probe(variant, k0, same + other, sign)
        for k1 in same:
            for d in range(0, 35):
                want = {sign * 2.0 ** (16 - d)} if d <= 13 else {0.0}
                assert got[(k1, d)] == want, "same group: k0=%d k1=%d d=%d sign=%+d: %r" % (k0, k1, d, sign, got[(k1, d)])
        for k1 in other:
            for d in range(0, 24):
                assert got[(k1, d)] == {sign * 2.0 ** (16 - d)}, "other group: k0=%d k1=%d d=%d: %r" % (k0, k1, d, got[(k1, d)])
            for d in range(26, 35):      # far below half an fp32 ulp of P: at most one ulp of P is lost
                assert all(abs(x) <= 2.0 ** -7 for x in got[(k1, d)]), (k1, d, got[(k1, d)])


@pytest.mark.parametrize("variant", VARIANTS)
def test_worst_case_group_loss_is_real_and_inside_the_stated_bound(variant):
    """Every group of 8: one product 2^16 and seven products 2^2 (d = 14), all positive: the exact sum is
    K/8 * (2^16 + 7 * 4), the instruction returns K/8 * 2^16.  The loss, 7 * 2^-14 of the large products, exceeds
    what an ideal fp32 accumulation could lose (2^-20 * sum|a b| was the first proposal for the tolerance) and
    lies inside ACC_TERM * sum|a b|."""
    a = np.full((256, KD), code(2.0), np.uint8)
    b = np.full((256, KD), code(2.0), np.uint8)
    a[:, ::8] = code(256.0)
    b[:, ::8] = code(256.0)
    c = gemm_f32(variant, a, b)
    groups = KD // 8
    exact = groups * (65536.0 + 7 * 4.0)
    sumabs = exact
    assert np.all(c == groups * 65536.0), "the d = 14 products were expected to vanish: %r" % np.unique(c)[:4]
    loss = exact - c[0, 0]
    assert loss > 2.0 ** -20 * sumabs          # an ideal fp32 accumulation would not lose this much
    assert loss <= 7 * 2.0 ** -14 * sumabs < ACC_TERM * sumabs
