"""The MLP half of a transformer block as the reference runs it (src/models/llama_model.cpp:209-220 forward,
:613-660 backward), composed from the library's entry points with the abs-max of every GEMM input coming
from its producer's epilogue -- no standalone abs-max pass on activations or gradients:

    res, ln   = fused_residual_rmsnorm_forward(residual, att_out, ln_w)      -> abs-max(ln)
    y_up      = forward_qmm(ln, W_up)                                         (quantize + e4m3 GEMM)
    h         = swiglu_forward(y_up)                                          -> abs-max(h)
    y_down    = forward_qmm(h, W_down)
    backward:   backward_qmm(dy) -> dh, dW_down;  swiglu_backward -> abs-max(dy_up);  backward_qmm -> dln, dW_up;
                rmsnorm_backward(dresidual = dy, dout = dln) -> abs-max(dres), dln_w

Checks: (1) the abs-max each producer wrote equals abs_max() of its tensor bit for bit, so every quantized
tensor equals what the standalone sequence gives; (2) the block's outputs and gradients against the same
block in float64 on torch's CPU autograd without any quantization: relative Frobenius error within 6-9 %
(forward, growing along the chain) and 6-12 % (gradients), the level that per-tensor e4m3 quantization of
Gaussian data leaves (about 4.5 % per quantized GEMM)."""
import pytest
import torch

pytestmark = pytest.mark.gpu
F8 = torch.float8_e4m3fn
BF = torch.bfloat16


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available()
    from llmq_amd import kernels
    return kernels


class QT:
    def __init__(self, shape):
        self.value = torch.empty(shape, dtype=BF, device="cuda")
        self.quant = torch.empty(shape, dtype=F8, device="cuda")
        self.stats = torch.zeros(2, device="cuda")

    abs_max = property(lambda s: s.stats[0:1])
    scale = property(lambda s: s.stats[1:2])


def rel_fro(got, ref):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return float((got - ref).norm() / ref.norm())


def test_mlp_block_forward_backward(K):
    BT, C, D, eps = 1024, 512, 1024, 1e-6
    g = torch.Generator(device="cuda").manual_seed(11)
    rn = lambda shape, std: (std * torch.randn(shape, device="cuda", generator=g)).to(BF)
    residual, att_out = rn((1, BT, C), 1.0), rn((1, BT, C), 0.5)
    ln_w = (1.0 + 0.1 * torch.randn(C, device="cuda", generator=g)).to(BF)
    w_up, w_down = rn((2 * D, C), C ** -0.5), rn((C, D), D ** -0.5)
    dy = rn((1, BT, C), 1.0)
    ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")

    def weight(w):
        q, st = torch.empty(w.shape, dtype=F8, device="cuda"), torch.zeros(2, device="cuda")
        K.abs_max(st[0:1], w)
        K.quantize_with_abs_max(q, st[1:2], w, st[0:1])
        return q, st

    wq_up, st_up = weight(w_up)
    wq_down, st_down = weight(w_down)

    # ---- forward
    res = torch.empty((1, BT, C), dtype=BF, device="cuda")
    ln, rstd = QT((1, BT, C)), torch.empty((1, BT), device="cuda")
    K.fused_residual_rmsnorm_forward(res, ln.value, rstd, residual, att_out, ln_w, ln.abs_max, eps)
    K.quantize_with_abs_max(ln.quant, ln.scale, ln.value, ln.abs_max)
    y_up = torch.empty((BT, 2 * D), dtype=BF, device="cuda")
    K.matmul(y_up, wq_up, ln.quant.view(BT, C), None, st_up[1:2], ln.scale, 2 * D, BT, C, workspace=ws)
    h = QT((1, BT, D))
    K.swiglu_forward(h.value, y_up.view(1, BT, 2 * D), h.abs_max)
    K.quantize_with_abs_max(h.quant, h.scale, h.value, h.abs_max)
    y_down = torch.empty((BT, C), dtype=BF, device="cuda")
    K.matmul(y_down, wq_down, h.quant.view(BT, D), None, st_down[1:2], h.scale, C, BT, D, workspace=ws)
    # the recompute path writes the same codes without the bf16 tensor
    h_q2 = torch.empty((1, BT, D), dtype=F8, device="cuda")
    K.swiglu_forward_quant(h_q2, None, y_up.view(1, BT, 2 * D), h.abs_max)
    assert torch.equal(h_q2.view(torch.uint8), h.quant.view(torch.uint8))

    # ---- backward
    def backward_qmm(dinp, dweight, dout_q, dout_scale, inp, wq, st_w, BT_, C_, OC_):
        w_t = torch.empty((C_, OC_), dtype=F8, device="cuda")
        K.transpose(w_t, wq)
        K.matmul(dinp, w_t, dout_q, None, st_w[1:2], dout_scale, C_, BT_, OC_, workspace=ws)
        a_t, g_t = torch.empty((C_, BT_), dtype=F8, device="cuda"), torch.empty((OC_, BT_), dtype=F8, device="cuda")
        K.transpose(a_t, inp.quant.view(BT_, C_))
        K.transpose(g_t, dout_q)
        K.matmul(dweight, a_t, g_t, None, inp.scale, dout_scale, C_, OC_, BT_, workspace=ws)

    dyq = QT((1, BT, C))
    dyq.value.copy_(dy)
    K.abs_max(dyq.abs_max, dyq.value)        # the block's incoming gradient: its producer is outside this test
    K.quantize_with_abs_max(dyq.quant, dyq.scale, dyq.value, dyq.abs_max)
    dh = torch.empty((BT, D), dtype=BF, device="cuda")
    dw_down = torch.empty((C, D), dtype=torch.float32, device="cuda")
    backward_qmm(dh, dw_down, dyq.quant.view(BT, C), dyq.scale, h, wq_down, st_down, BT, D, C)
    dy_up = QT((1, BT, 2 * D))
    K.swiglu_backward(dy_up.value, dh.view(1, BT, D), y_up.view(1, BT, 2 * D), dy_up.abs_max)
    K.quantize_with_abs_max(dy_up.quant, dy_up.scale, dy_up.value, dy_up.abs_max)
    dln = torch.empty((BT, C), dtype=BF, device="cuda")
    dw_up = torch.empty((2 * D, C), dtype=torch.float32, device="cuda")
    backward_qmm(dln, dw_up, dy_up.quant.view(BT, 2 * D), dy_up.scale, ln, wq_up, st_up, BT, C, 2 * D)
    dres = QT((1, BT, C))
    dln_w = torch.zeros(C, dtype=BF, device="cuda")
    scratch = torch.empty(K.get_rmsnorm_backward_scratch_size(C), dtype=torch.float32, device="cuda")
    K.rmsnorm_backward(dres.value, dln_w, scratch, dy, dln.view(1, BT, C), res, ln_w, rstd, dres.abs_max)

    # (1) producer abs-max == standalone abs-max, bit for bit
    ref = torch.zeros(1, device="cuda")
    for name, qt in (("ln", ln), ("h", h), ("dy_up", dy_up), ("dres", dres)):
        K.abs_max(ref, qt.value)
        assert qt.abs_max.view(torch.int32).item() == ref.view(torch.int32).item(), name

    # (2) the same block in float64 without quantization
    to64 = lambda t: t.detach().double().cpu()
    r0, a0 = to64(residual).requires_grad_(True), to64(att_out)
    lw, wu, wd = to64(ln_w).requires_grad_(True), to64(w_up).requires_grad_(True), to64(w_down).requires_grad_(True)
    r1 = r0 + a0
    n = r1 * torch.rsqrt((r1 ** 2).mean(dim=-1, keepdim=True) + eps) * lw
    yu = n @ wu.t()
    up, gate = yu[..., :D], yu[..., D:]
    hh = up * gate * torch.sigmoid(gate)
    yd = hh @ wd.t()
    out = r1 + yd                              # the residual stream after the block
    out.backward(to64(dy))
    errs = {"y_up": rel_fro(y_up.view(1, BT, 2 * D), yu), "h": rel_fro(h.value, hh), "y_down": rel_fro(y_down.view(1, BT, C), yd),
            "dw_down": rel_fro(dw_down, wd.grad), "dw_up": rel_fro(dw_up, wu.grad),
            "dres": rel_fro(dres.value, r0.grad),   # d(out)/d(residual) = dy + rmsnorm backward of the MLP path
            "dln_w": rel_fro(dln_w, lw.grad)}
    print({k: round(v, 4) for k, v in errs.items()})
    limits = {"y_up": 0.06, "h": 0.08, "y_down": 0.09, "dw_down": 0.10, "dw_up": 0.12, "dres": 0.06, "dln_w": 0.12}
    for k, v in errs.items():
        assert v < limits[k], (k, v)
