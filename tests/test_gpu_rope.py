"""GPU parity tests of the rotary-embedding kernels (through the C ABI, llmq_amd.kernels).

Bars: values against the CPU oracle (double evaluation, one rounding): one bf16 ulp plus 2^-22 of the summed
magnitudes of the two products (fp32 evaluation where they cancel); value heads bit exact (copied); the abs-max
epilogue bit exact against abs_max() of the written tensor; in-place == out-of-place; the reference's own
tolerance (rtol 1e-2 / atol 5e-3, scripts/test_kernels.py:385-411) on its torch construction."""
import numpy as np
import pytest
import torch

from gpu_util import dev_bf16, host_bits

pytestmark = pytest.mark.gpu

# (B, T, Nq, Nkv, HD): the reference's cases and the head shapes of the Qwen2.5 0.5B / 7B configurations
SHAPES = [(1, 8, 2, 1, 8), (2, 4, 1, 2, 16), (2, 16, 4, 2, 32), (4, 32, 8, 4, 64), (1, 40, 14, 2, 64), (1, 24, 28, 4, 128),
          (3, 7, 2, 2, 24)]


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from llmq_amd import kernels
    return kernels


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("backward", [False, True])
def test_rope_matches_oracle(K, O, shape, backward):
    B, T, Nq, Nkv, HD = shape
    N = Nq + 2 * Nkv
    x = O.fill_normal_bf16(B * T * N * HD, 900 + HD, 0).reshape(B * T, N, HD)
    tab = K.precompute_freqs_cis(HD, T, 1_000_000.0)
    want, exact, mag = O.rope(x, tab.view(torch.int16).numpy().view(np.uint16), T, Nq, Nkv, backward=backward)
    fn = K.rope_backward if backward else K.rope_forward
    xin = dev_bf16(x).reshape(B, T, N * HD)
    out = torch.full((B, T, N * HD), float("nan"), dtype=torch.bfloat16, device="cuda")
    am = torch.full((1,), 3.0, dtype=torch.float32, device="cuda")
    fn(out, xin, tab.cuda(), am, Nq, Nkv)
    got = host_bits(out).reshape(B * T, N, HD)
    g, w = O.bf16_to_f32(got).astype(np.float64), O.bf16_to_f32(want).astype(np.float64)
    assert np.all(np.abs(g - w) <= np.abs(exact) * 2.0 ** -7 + mag * 2.0 ** -22 + 1e-38)
    assert np.array_equal(got[:, Nq + Nkv:], x[:, Nq + Nkv:])
    ref_am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.abs_max(ref_am, out)
    assert am.cpu().numpy().view(np.uint32)[0] == ref_am.cpu().numpy().view(np.uint32)[0]
    # in place, without abs-max: same tensor (value heads are not even read)
    y = xin.clone()
    fn(y, y, tab.cuda(), None, Nq, Nkv)
    assert torch.equal(y.view(torch.int16), out.view(torch.int16))
    # in place with abs-max: the value heads still count
    y2, am2 = xin.clone(), torch.zeros(1, dtype=torch.float32, device="cuda")
    fn(y2, y2, tab.cuda(), am2, Nq, Nkv)
    assert torch.equal(y2.view(torch.int16), out.view(torch.int16)) and am2.item() == am.item()


def test_rope_reference_test_construction(K):
    """scripts/test_kernels.py:361-411: torch float reference, randn inputs, theta 1e6."""
    B, T, Nq, Nkv, HD = 4, 32, 8, 4, 64
    N = Nq + 2 * Nkv
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn((B, T, N * HD), device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16)
    freqs = K.precompute_freqs_cis(HD, T, 1_000_000.0).cuda()

    def rope_python(x4, backward):
        half = HD // 2
        cos, sin = freqs[:, 0::2].float()[None, :, None, :], freqs[:, 1::2].float()[None, :, None, :]
        if backward:
            sin = -sin
        rot = lambda h: torch.cat([h[..., :half].float() * cos - h[..., half:].float() * sin,
                                   h[..., :half].float() * sin + h[..., half:].float() * cos], dim=-1).to(x4.dtype)
        return torch.cat([rot(x4[:, :, :Nq]), rot(x4[:, :, Nq:Nq + Nkv]), x4[:, :, Nq + Nkv:]], dim=2)

    for backward, fn in ((False, K.rope_forward), (True, K.rope_backward)):
        out = torch.empty_like(x)
        fn(out, x, freqs, None, Nq, Nkv)
        ref = rope_python(x.view(B, T, N, HD), backward).view(B, T, N * HD)
        assert torch.allclose(out.float(), ref.float(), rtol=1e-2, atol=5e-3)


def test_precompute_freqs_cis_table(K):
    """The host table against numpy float64 cos / sin: within one fp16 ulp plus the angle's fp32 rounding."""
    HD, T, theta = 128, 2048, 1_000_000.0
    tab = K.precompute_freqs_cis(HD, T, theta).numpy().astype(np.float64)
    i = np.arange(HD // 2, dtype=np.float64)
    ang = np.arange(T, dtype=np.float64)[:, None] / theta ** (2 * i / HD)[None, :]
    tol = 2.0 ** -10 + ang * 2.0 ** -22          # fp16 rounding of values in [-1, 1]; fp32 angle error
    assert np.all(np.abs(tab[:, 0::2] - np.cos(ang)) <= tol) and np.all(np.abs(tab[:, 1::2] - np.sin(ang)) <= tol)
    assert np.array_equal(tab[0, 0::2], np.ones(HD // 2)) and np.array_equal(tab[0, 1::2], np.zeros(HD // 2))


def test_rope_argument_errors(K):
    x = torch.zeros((1, 4, 3 * 12), dtype=torch.bfloat16, device="cuda")
    tab = torch.zeros((4, 12), dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError, match="divisible by 8"):
        K.rope_forward(x, x, tab, None, 1, 1)
    tab = torch.zeros((4, 16), dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        K.rope_forward(x, x, tab, None, 1, 1)            # C != (Nq + 2 Nkv) * HD


def test_rope_full_size_properties(K, O):
    """Qwen2.5-7B attention shape at 8192 tokens (28 query and 4 key/value heads of 128): forward then backward
    returns the input up to rounding; abs-max invariant; sampled tokens against the oracle."""
    B, T, Nq, Nkv, HD = 8, 1024, 28, 4, 128
    N = Nq + 2 * Nkv
    g = torch.Generator(device="cuda").manual_seed(4)
    x = torch.randn((B, T, N * HD), device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16)
    tab = K.precompute_freqs_cis(HD, T, 1_000_000.0)
    freqs = tab.cuda()
    y, am = torch.empty_like(x), torch.zeros(1, dtype=torch.float32, device="cuda")
    K.rope_forward(y, x, freqs, am, Nq, Nkv)
    ref_am = torch.zeros(1, dtype=torch.float32, device="cuda")
    K.abs_max(ref_am, y)
    assert am.item() == ref_am.item() and am.item() > 0
    back = torch.empty_like(x)
    K.rope_backward(back, y, freqs, None, Nq, Nkv)
    assert torch.allclose(back.float(), x.float(), rtol=2.0 ** -6, atol=2.0 ** -6)
    sel = torch.tensor([0, 1023, 1024, 8191], device="cuda")
    sub = host_bits(x.view(B * T, N, HD)[sel])
    # tokens 0, 1023, 1024, 8191 sit at positions t = 0, 1023, 0, 1023: feed the oracle a table of those rows
    rows = tab.view(torch.int16).numpy().view(np.uint16)[[0, 1023, 0, 1023]]
    want, exact, mag = O.rope(sub, rows, 4, Nq, Nkv)
    got = O.bf16_to_f32(host_bits(y.view(B * T, N, HD)[sel])).astype(np.float64)
    assert np.all(np.abs(got - O.bf16_to_f32(want)) <= np.abs(exact) * 2.0 ** -7 + mag * 2.0 ** -22 + 1e-38)
