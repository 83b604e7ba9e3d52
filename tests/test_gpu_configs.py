"""GPU parity at the shapes of BASELINE.json's configurations 2-5: the call sequences of the
reference's forward_qmm / backward_qmm (src/models/llama_model.cpp:25-47, 309-339) replayed through
the C ABI, every intermediate compared with the CPU oracle: abs-max, scales and fp8 bytes bit exact,
GEMM outputs within the stated tolerance on a deterministic sample of output coordinates plus whole
boundary rows/columns.  Inputs are seeded: small tensors come from the oracle's counter-based
generator, large ones from a seeded torch generator on the device (same bytes feed both sides)."""
import os

import numpy as np
import pytest
import torch

from gpu_util import dev_bf16, gemm_check, host_bits, report_gemm_error

pytestmark = pytest.mark.gpu
F8 = torch.float8_e4m3fn


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available()
    from llmq_amd import kernels
    return kernels


def randn_bf16(shape, std, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, device="cuda", generator=g) * std).to(torch.bfloat16)


def student_t3_bf16(shape, seed, outlier_channels=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    z = torch.randn(shape, device="cuda", generator=g)
    chi = sum(torch.randn(shape, device="cuda", generator=g) ** 2 for _ in range(3)) / 3.0
    x = z / chi.sqrt()
    if outlier_channels:
        cg = torch.Generator().manual_seed(seed)
        ch = torch.randperm(shape[1], generator=cg)[:outlier_channels].cuda()
        x[:, ch] *= 100.0
    return x.to(torch.bfloat16)


class QT:
    """Value + quantized copy + [abs_max, scale] stats, the reference's QuantizableTensor
    (src/models/llama_run_state.h:19-24, src/utilities/tensor.h:123-131)."""

    def __init__(self, value):
        self.value = value
        self.quant = torch.empty(value.shape, dtype=F8, device="cuda")
        self.stats = torch.zeros(2, device="cuda")

    @property
    def abs_max(self):
        return self.stats[0:1]

    @property
    def scale(self):
        return self.stats[1:2]


_WS = {}


def workspace():
    """Matmul workspace sized like the reference's (src/training/model.cpp:69)."""
    if "ws" not in _WS:
        _WS["ws"] = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
    return _WS["ws"]


def forward_qmm(K, out, inp, weight_q, weight_scale, BT, C, OC):
    K.quantize_with_abs_max(inp.quant, inp.scale, inp.value, inp.abs_max)
    K.matmul(out, weight_q, inp.quant, None, weight_scale, inp.scale, OC, BT, C, workspace=workspace())


def backward_qmm(K, dinp, dweight, dout, inp, weight_q, weight_scale, BT, C, OC, reuse_inp, accumulate=False):
    K.quantize_with_abs_max(dout.quant, dout.scale, dout.value, dout.abs_max)
    weight_tp = torch.empty((C, OC), dtype=F8, device="cuda")
    K.transpose(weight_tp, weight_q)
    K.matmul(dinp, weight_tp, dout.quant, None, weight_scale, dout.scale, C, BT, OC, workspace=workspace())
    act_tp = torch.empty((C, BT), dtype=F8, device="cuda")
    grad_tp = torch.empty((OC, BT), dtype=F8, device="cuda")
    if reuse_inp:
        K.transpose(act_tp, inp.quant)
    else:
        K.quantize_and_transpose_with_abs_max(act_tp, None, inp.value, inp.abs_max)
    K.transpose(grad_tp, dout.quant)
    K.matmul(dweight, act_tp, grad_tp, None, inp.scale, dout.scale, C, OC, BT, accumulate=accumulate,
             workspace=workspace())
    return weight_tp, act_tp, grad_tp


def check_quant(O, qt, name):
    """abs-max, scale and bytes of a QT against the oracle; returns (codes, dequant scale)."""
    bits = host_bits(qt.value)
    am = O.abs_max_bf16(bits)
    st = qt.stats.cpu().numpy()
    assert st[0].view(np.uint32) == np.float32(am).view(np.uint32), name + ": abs-max"
    codes, d = O.quantize_e4m3(bits, am, mt=True)
    assert st[1].view(np.uint32) == np.float32(d).view(np.uint32), name + ": scale"
    got = host_bits(qt.quant)
    assert np.array_equal(got, codes), name + ": quantized bytes"
    return codes, d


def sample_idx(N, M, seed, count=30000):
    rng = np.random.default_rng(seed)
    n = np.concatenate([rng.integers(0, N, count), np.full(min(M, 4096), N - 1), np.arange(min(N, 4096)), [0]])
    m = np.concatenate([rng.integers(0, M, count), np.arange(min(M, 4096)), np.full(min(N, 4096), M - 1), [0]])
    return n.astype(np.int32), m.astype(np.int32)


def check_gemm(O, c, a_codes, b_codes, sa, sb, seed, name, c_old=None):
    """c[N,M] against exact(b . a^T) * sa*sb on sampled coordinates."""
    N, M = c.shape
    idx_n, idx_m = sample_idx(N, M, seed)
    ex, sabs = O.gemm_exact_sampled(a_codes, b_codes, idx_n, idx_m)
    got = c.float().cpu().numpy()[idx_n, idx_m]
    extra = c_old[idx_n, idx_m].astype(np.float64) if c_old is not None else None
    scale = np.float32(np.float32(sa) * np.float32(sb))
    mx, fro = gemm_check(got, ex, sabs, scale, c.dtype == torch.bfloat16, extra=extra)
    print("%-28s [%5d x %5d] max-abs err %.3e  rel-Frobenius %.3e" % (name, N, M, mx, fro))
    cfg = os.environ.get("PYTEST_CURRENT_TEST", "").split("::")[-1].split(" ")[0]
    report_gemm_error(cfg, name, N, M, a_codes.shape[1], mx, fro, "%d sampled outputs incl. boundary rows/columns" % idx_n.size)
    return mx, fro


def run_linear_fwd_bwd(K, O, BT, C, OC, x, w, dy, seed, backward=True, reuse_inp=False, dw_dtype=torch.bfloat16):
    inp, wq, dout = QT(x), QT(w), QT(dy) if dy is not None else None
    K.abs_max(inp.abs_max, inp.value)
    K.abs_max(wq.abs_max, wq.value)
    K.quantize_with_abs_max(wq.quant, wq.scale, wq.value, wq.abs_max)     # llama_weights.cpp:207-223
    y = torch.empty((BT, OC), dtype=torch.bfloat16, device="cuda")
    forward_qmm(K, y, inp, wq.quant, wq.scale, BT, C, OC)
    torch.cuda.synchronize()
    xc, dx_s = check_quant(O, inp, "x")
    wc, dw_s = check_quant(O, wq, "w")
    check_gemm(O, y, wc, xc, dw_s, dx_s, seed, "forward y")
    if not backward:
        return
    K.abs_max(dout.abs_max, dout.value)
    dinp = torch.empty((BT, C), dtype=torch.bfloat16, device="cuda")
    dweight = torch.empty((OC, C), dtype=dw_dtype, device="cuda")
    w_tp, a_tp, g_tp = backward_qmm(K, dinp, dweight, dout, inp, wq.quant, wq.scale, BT, C, OC, reuse_inp)
    torch.cuda.synchronize()
    gc, dg_s = check_quant(O, dout, "dy")
    assert np.array_equal(host_bits(w_tp), wc.T), "weight transpose"
    assert np.array_equal(host_bits(a_tp), xc.T), "activation (quantize+)transpose"
    assert np.array_equal(host_bits(g_tp), gc.T), "gradient transpose"
    check_gemm(O, dinp, np.ascontiguousarray(wc.T), gc, dw_s, dg_s, seed + 1, "dgrad dx")
    check_gemm(O, dweight, np.ascontiguousarray(xc.T), np.ascontiguousarray(gc.T), dx_s, dg_s, seed + 2, "wgrad dw")
    # The same gradients with operands read where they lie, wherever the K-major modes serve the shape: dgrad with the
    # weight [OC, C] as the K-major first operand (mode NN), wgrad with activation [BT, C] and gradient [BT, OC] both in
    # place (mode NT) ...
    if OC % 256 == 0 and BT % 256 == 0 and C % 256 == 0:
        dx_nn = torch.full((BT, C), float("nan"), dtype=torch.bfloat16, device="cuda")
        K.matmul(dx_nn, wq.quant, dout.quant, None, wq.scale, dout.scale, C, BT, OC, a_kmajor=True)
        dw_nt = torch.full((OC, C), float("nan"), dtype=torch.bfloat16, device="cuda")
        K.matmul(dw_nt, inp.quant, dout.quant, None, inp.scale, dout.scale, C, OC, BT, a_kmajor=True, b_kmajor=True)
        torch.cuda.synchronize()
        check_gemm(O, dx_nn, np.ascontiguousarray(wc.T), gc, dw_s, dg_s, seed + 1, "dgrad dx, mode NN")
        check_gemm(O, dw_nt, np.ascontiguousarray(xc.T), np.ascontiguousarray(gc.T), dx_s, dg_s, seed + 2, "wgrad dw, mode NT")
        del dx_nn, dw_nt
    # ... and with the quantized output gradient alone read in place (matmul mode TT: dout.quant [BT, OC] as the
    # K-major second operand)
    if OC % 256 == 0 and BT % 256 == 0 and (C % 256 == 0 or C % 224 == 0):
        dw_tt = torch.full((OC, C), float("nan"), dtype=torch.bfloat16, device="cuda")
        K.matmul(dw_tt, a_tp, dout.quant, None, inp.scale, dout.scale, C, OC, BT, b_kmajor=True)
        torch.cuda.synchronize()
        check_gemm(O, dw_tt, np.ascontiguousarray(xc.T), np.ascontiguousarray(gc.T), dx_s, dg_s, seed + 2, "wgrad dw, mode TT")
        if C % 256 == 0:
            old_tt = dw_tt.float().cpu().numpy()
            K.matmul(dw_tt, a_tp, dout.quant, None, inp.scale, dout.scale, C, OC, BT, accumulate=True, b_kmajor=True)
            torch.cuda.synchronize()
            check_gemm(O, dw_tt, np.ascontiguousarray(xc.T), np.ascontiguousarray(gc.T), dx_s, dg_s, seed + 2,
                       "wgrad dw +=, mode TT", c_old=old_tt)
        del dw_tt
    # accumulate into an existing gradient (second micro-step of gradient accumulation)
    old = dweight.float().cpu().numpy()
    K.matmul(dweight, a_tp, g_tp, None, inp.scale, dout.scale, C, OC, BT, accumulate=True,
             workspace=workspace())
    torch.cuda.synchronize()
    check_gemm(O, dweight, np.ascontiguousarray(xc.T), np.ascontiguousarray(gc.T), dx_s, dg_s, seed + 2, "wgrad dw +=", c_old=old)


QWEN05 = [("qkv", 896, 1152), ("o_proj", 896, 896), ("gate_up", 896, 9728), ("down", 4864, 896)]


@pytest.mark.parametrize("name,C,OC", QWEN05)
def test_config2_qwen05b_block_forward(K, O, name, C, OC):
    BT = 8192
    x = dev_bf16(O.fill_normal_bf16(BT * C, 2, 10 + C % 7).reshape(BT, C))
    w = dev_bf16(O.fill_normal_bf16(OC * C, 2, 20 + OC % 7, 0.0, 0.02).reshape(OC, C))
    run_linear_fwd_bwd(K, O, BT, C, OC, x, w, None, seed=200 + OC, backward=False)


@pytest.mark.parametrize("name,C,OC", QWEN05)
@pytest.mark.parametrize("reuse_inp", [False, True])
def test_config3_qwen05b_block_backward(K, O, name, C, OC, reuse_inp):
    BT = 8192
    x = dev_bf16(O.fill_normal_bf16(BT * C, 3, 10 + C % 7).reshape(BT, C))
    w = dev_bf16(O.fill_normal_bf16(OC * C, 3, 20 + OC % 7, 0.0, 0.02).reshape(OC, C))
    dy = dev_bf16(O.fill_normal_bf16(BT * OC, 3, 30 + OC % 7, 0.0, 1e-3).reshape(BT, OC))
    run_linear_fwd_bwd(K, O, BT, C, OC, x, w, dy, seed=300 + OC, reuse_inp=reuse_inp, dw_dtype=torch.float32)


@pytest.mark.parametrize("name,C,OC", [("gate_up", 3584, 37888), ("down", 18944, 3584)])
def test_config4_qwen7b_mlp(K, O, name, C, OC):
    BT = 8192
    x = randn_bf16((BT, C), 1.0, 41)
    w = randn_bf16((OC, C), 0.015, 42)
    dy = randn_bf16((BT, OC), 1e-4, 43)
    run_linear_fwd_bwd(K, O, BT, C, OC, x, w, dy, seed=400 + OC % 100)


@pytest.mark.parametrize("name,C,OC", [("gate_up", 1536, 17920), ("down", 8960, 1536)])
def test_config5_outlier_stress(K, O, name, C, OC):
    """Student-t(3) activations with 8 hidden channels x100: the abs-max is set by the outliers, so
    most values land in the subnormal / underflow range of e4m3 while the outliers sit at +-448."""
    BT = 16384
    x = student_t3_bf16((BT, C), 51, outlier_channels=8)
    w = randn_bf16((OC, C), 0.02, 52)
    dy = student_t3_bf16((BT, OC), 53) * 1e-3
    inp = QT(x)
    K.abs_max(inp.abs_max, inp.value)
    K.quantize_with_abs_max(inp.quant, inp.scale, inp.value, inp.abs_max)
    torch.cuda.synchronize()
    codes, _ = check_quant(O, inp, "x outliers")
    mag = codes & 0x7F
    assert (mag == 0x7E).any(), "the abs-max element must saturate to +-448"
    zero_frac, sub_frac = (mag == 0).mean(), ((mag > 0) & (mag < 8)).mean()
    print("outlier stress: underflow-to-zero fraction %.4f, subnormal fraction %.4f" % (zero_frac, sub_frac))
    assert zero_frac > 1e-3, "expected a visible underflow-to-zero fraction"
    assert sub_frac > 0.05, "expected many subnormal codes"
    run_linear_fwd_bwd(K, O, BT, C, OC, x, w, dy.to(torch.bfloat16), seed=500 + OC % 100)


def test_hip_graph_replay_matches_eager(K, O):
    """The whole call sequence of one linear layer (abs-max, quantize, forward, backward with split-K
    wgrad) recorded into a HIP graph, as the reference records a transformer block
    (src/models/llama_model.cpp:49-71): every replay, with new inputs and eager work in between, must
    reproduce the eager result bit for bit."""
    BT, C, OC = 2048, 896, 1152
    x = torch.empty((BT, C), dtype=torch.bfloat16, device="cuda")
    w = torch.empty((OC, C), dtype=torch.bfloat16, device="cuda")
    dy = torch.empty((BT, OC), dtype=torch.bfloat16, device="cuda")
    inp, wq, dout = QT(x), QT(w), QT(dy)
    y = torch.empty((BT, OC), dtype=torch.bfloat16, device="cuda")
    dinp = torch.empty((BT, C), dtype=torch.bfloat16, device="cuda")
    dweight = torch.empty((OC, C), dtype=torch.float32, device="cuda")
    workspace()                                    # allocate outside the capture

    def fill(seed):
        x.copy_(dev_bf16(O.fill_normal_bf16(BT * C, seed, 1).reshape(BT, C)))
        w.copy_(dev_bf16(O.fill_normal_bf16(OC * C, seed, 2, 0.0, 0.02).reshape(OC, C)))
        dy.copy_(dev_bf16(O.fill_normal_bf16(BT * OC, seed, 3, 0.0, 1e-3).reshape(BT, OC)))

    def sequence():
        K.abs_max(inp.abs_max, inp.value)
        K.abs_max(wq.abs_max, wq.value)
        K.abs_max(dout.abs_max, dout.value)
        K.quantize_with_abs_max(wq.quant, wq.scale, wq.value, wq.abs_max)
        forward_qmm(K, y, inp, wq.quant, wq.scale, BT, C, OC)
        backward_qmm(K, dinp, dweight, dout, inp, wq.quant, wq.scale, BT, C, OC, reuse_inp=False)

    def snapshot():
        torch.cuda.synchronize()
        return [t.clone() for t in (inp.stats, wq.stats, dout.stats, inp.quant.view(torch.uint8), y, dinp, dweight)]

    fill(50)
    sequence()                                     # warm-up (also creates the transposed temporaries' pool)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        sequence()
        with torch.cuda.graph(graph, stream=side):
            sequence()
    torch.cuda.current_stream().wait_stream(side)
    for seed in (51, 52, 53):
        fill(seed)
        sequence()
        want = snapshot()
        for t in (y, dinp, dweight):
            t.fill_(float("nan"))
        inp.stats.zero_()
        graph.replay()
        got = snapshot()
        for a, b in zip(want, got):
            assert torch.equal(a.view(torch.uint8) if a.dtype != torch.uint8 else a,
                               b.view(torch.uint8) if b.dtype != torch.uint8 else b), "replay for seed %d differs" % seed


@pytest.mark.parametrize("wgrad", ["NT", "TT"])
def test_hip_graph_replay_of_the_stored_layout_backward(K, O, wgrad):
    """The backward of a layer with its matmuls in the K-major operand modes (dgrad NN on the weight as stored,
    weight gradient NT on activation and gradient as stored, or TT on the gradient as stored), recorded into a HIP
    graph: every replay, with new inputs and eager work in between, must reproduce the eager result bit for bit, and
    the eager result must equal the transposing route's."""
    BT, C, OC = 1024, 768, 512
    x = torch.empty((BT, C), dtype=torch.bfloat16, device="cuda")
    w = torch.empty((OC, C), dtype=torch.bfloat16, device="cuda")
    dy = torch.empty((BT, OC), dtype=torch.bfloat16, device="cuda")
    inp, wq, dout = QT(x), QT(w), QT(dy)
    dinp = torch.empty((BT, C), dtype=torch.bfloat16, device="cuda")
    dweight = torch.empty((OC, C), dtype=torch.bfloat16, device="cuda")
    act_tp = torch.empty((C, BT), dtype=F8, device="cuda")
    ref_dinp, ref_dweight = torch.empty_like(dinp), torch.empty_like(dweight)
    workspace()

    def fill(seed):
        x.copy_(dev_bf16(O.fill_normal_bf16(BT * C, seed, 1).reshape(BT, C)))
        w.copy_(dev_bf16(O.fill_normal_bf16(OC * C, seed, 2, 0.0, 0.02).reshape(OC, C)))
        dy.copy_(dev_bf16(O.fill_normal_bf16(BT * OC, seed, 3, 0.0, 1e-3).reshape(BT, OC)))

    def sequence():
        for qt in (inp, wq, dout):
            K.abs_max(qt.abs_max, qt.value)
            K.quantize_with_abs_max(qt.quant, qt.scale, qt.value, qt.abs_max)
        K.matmul(dinp, wq.quant, dout.quant, None, wq.scale, dout.scale, C, BT, OC, a_kmajor=True)
        if wgrad == "NT":
            K.matmul(dweight, inp.quant, dout.quant, None, inp.scale, dout.scale, C, OC, BT, a_kmajor=True, b_kmajor=True)
        else:
            K.quantize_and_transpose_with_abs_max(act_tp, None, inp.value, inp.abs_max)
            K.matmul(dweight, act_tp, dout.quant, None, inp.scale, dout.scale, C, OC, BT, b_kmajor=True)

    fill(60)
    sequence()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        sequence()
        with torch.cuda.graph(graph, stream=side):
            sequence()
    torch.cuda.current_stream().wait_stream(side)
    for seed in (61, 62, 63):
        fill(seed)
        sequence()
        torch.cuda.synchronize()
        want = [dinp.clone(), dweight.clone()]
        backward_qmm(K, ref_dinp, ref_dweight, dout, inp, wq.quant, wq.scale, BT, C, OC, reuse_inp=False)
        torch.cuda.synchronize()
        # 768 x 512 outputs: both routes run whole 256-tiles of the four-wave kernel over the same K order
        assert torch.equal(ref_dinp.view(torch.int16), dinp.view(torch.int16)), "dgrad differs from the transposing route"
        assert torch.equal(ref_dweight.view(torch.int16), dweight.view(torch.int16)), "wgrad differs from the transposing route"
        dinp.fill_(float("nan"))
        dweight.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(want[0].view(torch.int16), dinp.view(torch.int16)), "replay for seed %d differs" % seed
        assert torch.equal(want[1].view(torch.int16), dweight.view(torch.int16)), "replay for seed %d differs" % seed


def test_backward_with_e5m2_gradients(K, O):
    """The e5m2 gradient dtype (`--gradient-dtype=e5m2` in the reference): dY is quantized to e5m2 with the
    same 448-based scale (src/kernels/quant.cu:79, 130-132), transposed as bytes, and multiplied as the b
    operand of e4m3 x e5m2 matmuls (src/kernels/kernels.h:92-94); the bias gradient reads the same bytes
    (src/kernels/bias.cu:193-195)."""
    BT, C, OC = 4096, 896, 1152
    F5 = torch.float8_e5m2
    x = dev_bf16(O.fill_normal_bf16(BT * C, 6, 1).reshape(BT, C))
    w = dev_bf16(O.fill_normal_bf16(OC * C, 6, 2, 0.0, 0.02).reshape(OC, C))
    dy = dev_bf16(O.fill_normal_bf16(BT * OC, 6, 3, 0.0, 1e-3).reshape(BT, OC))
    inp, wq, dout = QT(x), QT(w), QT(dy)
    dout.quant = torch.empty(dy.shape, dtype=F5, device="cuda")
    for t in (inp, wq, dout):
        K.abs_max(t.abs_max, t.value)
    K.quantize_with_abs_max(wq.quant, wq.scale, wq.value, wq.abs_max)
    K.quantize_with_abs_max(inp.quant, inp.scale, inp.value, inp.abs_max)
    # backward_qmm with an e5m2 gradient
    K.quantize_with_abs_max(dout.quant, dout.scale, dout.value, dout.abs_max)
    w_tp = torch.empty((C, OC), dtype=F8, device="cuda")
    K.transpose(w_tp, wq.quant)
    dinp = torch.empty((BT, C), dtype=torch.bfloat16, device="cuda")
    K.matmul(dinp, w_tp, dout.quant, None, wq.scale, dout.scale, C, BT, OC, workspace=workspace())
    a_tp = torch.empty((C, BT), dtype=F8, device="cuda")
    g_tp = torch.empty((OC, BT), dtype=F5, device="cuda")
    K.quantize_and_transpose_with_abs_max(a_tp, None, inp.value, inp.abs_max)
    K.transpose(g_tp, dout.quant)
    dweight = torch.empty((OC, C), dtype=torch.bfloat16, device="cuda")
    K.matmul(dweight, a_tp, g_tp, None, inp.scale, dout.scale, C, OC, BT, workspace=workspace())
    dbias = torch.zeros(OC, dtype=torch.bfloat16, device="cuda")
    buf = torch.empty(K.get_bias_backward_scratch_size(F5, OC, BT) // 4, dtype=torch.float32, device="cuda")
    K.backward_bias(dbias, dout.quant, inp.scale, dout.scale, buf)
    torch.cuda.synchronize()

    gbits = host_bits(dy)
    ag = O.abs_max_bf16(gbits)
    gc, dg_s = O.quantize_e4m3(gbits, ag, mt=False, fmt="e5m2")
    assert np.array_equal(host_bits(dout.quant), gc) and dout.stats.cpu().numpy()[1] == dg_s
    assert np.array_equal(host_bits(g_tp), gc.T)
    xc, dx_s = check_quant(O, inp, "x")
    wc, dw_s = check_quant(O, wq, "w")
    for name, c, a_codes, b_codes, sa in (("dgrad e5m2", dinp, np.ascontiguousarray(wc.T), gc, dw_s),
                                          ("wgrad e5m2", dweight, np.ascontiguousarray(xc.T), np.ascontiguousarray(gc.T), dx_s)):
        N, M = c.shape
        idx_n, idx_m = sample_idx(N, M, 61)
        ex, sabs = O.gemm_exact_sampled(a_codes, b_codes, idx_n, idx_m, b_e5m2=True)
        got = c.float().cpu().numpy()[idx_n, idx_m]
        mx, fro = gemm_check(got, ex, sabs, np.float32(np.float32(sa) * np.float32(dg_s)), True)
        print("%-12s max-abs err %.3e  rel-Frobenius %.3e" % (name, mx, fro))
    want, cs, ca = O.backward_bias(np.zeros(OC, dtype=np.uint16), gc, "e5m2", float(dx_s), float(dg_s))
    got = O.bf16_to_f32(host_bits(dbias)).astype(np.float64)
    ref = cs * float(np.float32(dx_s) * np.float32(dg_s))
    assert np.all(np.abs(got - ref) <= 2.0 ** -8 * np.abs(ref) + 2.0 ** -18 * float(dx_s * dg_s) * ca + 1e-30)
