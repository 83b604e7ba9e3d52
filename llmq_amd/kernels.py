"""Host-side mirror of the reference's per-kernel Python entry points for the FP8 path
(reference: src/binding/python/kernels.py:121-165, src/binding/kernel_binding.cpp:393-509), on torch
tensors that live on the MI355X.  torch is used only for device memory and streams; every call goes
through the C ABI (llmq_amd.capi) into the hand-written gfx950 kernels.

Names, argument order and in-place "out first" convention are the reference's:
    abs_max(scale, x, stream=0)
    quantize_with_abs_max(out, scale, x, abs_max, stream=0)
    quantize_and_transpose_with_abs_max(out, scale, x, abs_max, stream=0)
    transpose(dst, src, stream=0)
    matmul(c, a, b, bias, scale_a, scale_b, M, N, K, accumulate=False, stream=0)   [kernels.h convention]
    backward_bias(dbias, dout, scale_a, scale_b, dbias_buffer, stream=0)
    get_bias_backward_scratch_size(dtype, OC, BT=...)
    swiglu_forward(out, inp, abs_max, stream=0)
    swiglu_forward_quant(out, scale, inp, abs_max, stream=0)
    swiglu_backward(dinp, dout, inp, abs_max, stream=0)
    rmsnorm_forward(out, rms, inp, weight, abs_max, epsilon, stream=0)
    fused_residual_rmsnorm_forward(residual, normed, rrms, inp1, inp2, weight, abs_max, epsilon, stream=0)
    rmsnorm_backward(dinp, dweight, scratch, dresidual, dout, inp, weight, rstd, abs_max, stream=0)
    get_rmsnorm_backward_scratch_size(C)
    rope_forward(out, inp, freqs_cis, abs_max, Nq, Nkv, stream=0);  rope_backward(dinp, dout, freqs_cis, abs_max, Nq, Nkv, stream=0)
    precompute_freqs_cis(dim, end, theta)
    adamw_update(params, grads, m, v, learning_rate, beta1, beta2, t, eps, weight_decay, grad_scale, m_scales=None,
                 abs_max=None, seed=0, stream=0)
`stream` is a raw hipStream_t handle (0 = torch's current stream).
"""
import torch

from . import capi

_FP8 = (torch.float8_e4m3fn, torch.float8_e5m2, torch.uint8)


def _stream(stream):
    return stream if stream else torch.cuda.current_stream().cuda_stream


def _dev(t, name, dtypes=None, optional=False):
    if t is None:
        if optional:
            return None
        raise ValueError("%s must not be None" % name)
    if not t.is_cuda:
        raise ValueError("%s must be a device tensor" % name)
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    if dtypes is not None and t.dtype not in dtypes:
        raise ValueError("%s: unsupported dtype %s" % (name, t.dtype))
    return t.data_ptr()


def abs_max(scale, x, stream=0):
    """scale[0] = max |x| (fp32).  x: bf16 or fp32 device tensor."""
    out = _dev(scale, "scale", (torch.float32,))
    ptr = _dev(x, "x", (torch.bfloat16, torch.float32))
    f = capi.lib.llmq_abs_max_bf16 if x.dtype == torch.bfloat16 else capi.lib.llmq_abs_max_f32
    capi.check(f(out, ptr, x.numel(), _stream(stream)))


def quantize_with_abs_max(out, scale, x, abs_max, stream=0):
    """out = fp8(448/abs_max * x); scale[0] = abs_max/448 (as 1/(448/abs_max)).  scale may be None."""
    o = _dev(out, "out", _FP8)
    s = _dev(scale, "scale", (torch.float32,), optional=True)
    i = _dev(x, "x", (torch.bfloat16, torch.float32))
    a = _dev(abs_max, "abs_max", (torch.float32,))
    if out.numel() != x.numel():
        raise ValueError("out and x must have the same number of elements")
    e5 = out.dtype == torch.float8_e5m2
    if x.dtype == torch.float32:
        f = capi.lib.llmq_quantize_e5m2_f32 if e5 else capi.lib.llmq_quantize_e4m3_f32
    else:
        f = capi.lib.llmq_quantize_e5m2_bf16 if e5 else capi.lib.llmq_quantize_e4m3_bf16
    capi.check(f(o, s, i, a, x.numel(), _stream(stream)))


def quantize_and_transpose_with_abs_max(out, scale, x, abs_max, stream=0):
    """x: [rows, cols] bf16 or fp32 -> out: [cols, rows] e4m3."""
    if x.dim() != 2 or out.dim() != 2 or out.shape[0] != x.shape[1] or out.shape[1] != x.shape[0]:
        raise ValueError("x must be [rows, cols] and out [cols, rows]")
    o = _dev(out, "out", (torch.float8_e4m3fn, torch.uint8))
    s = _dev(scale, "scale", (torch.float32,), optional=True)
    i = _dev(x, "x", (torch.bfloat16, torch.float32))
    a = _dev(abs_max, "abs_max", (torch.float32,))
    fn = capi.lib.llmq_quantize_transpose_e4m3_f32 if x.dtype == torch.float32 else capi.lib.llmq_quantize_transpose_e4m3_bf16
    capi.check(fn(o, s, i, a, x.shape[0], x.shape[1], _stream(stream)))


def quantize_with_abs_max_and_transpose(out, out_t, scale, x, abs_max, stream=0):
    """One read of x [rows, cols] (bf16) gives out [rows, cols] and out_t [cols, rows] in the fp8 dtype of
    `out` -- the bytes of quantize_with_abs_max followed by transpose.  No counterpart in the reference."""
    if x.dim() != 2 or out.shape != x.shape or out_t.dim() != 2 or out_t.shape[0] != x.shape[1] or out_t.shape[1] != x.shape[0]:
        raise ValueError("x and out must be [rows, cols], out_t [cols, rows]")
    if out.dtype != out_t.dtype:
        raise ValueError("out and out_t must have the same dtype")
    o = _dev(out, "out", _FP8)
    ot = _dev(out_t, "out_t", _FP8)
    s = _dev(scale, "scale", (torch.float32,), optional=True)
    i = _dev(x, "x", (torch.bfloat16,))
    a = _dev(abs_max, "abs_max", (torch.float32,))
    fmt = 1 if out.dtype == torch.float8_e5m2 else 0
    capi.check(capi.lib.llmq_quantize_both_bf16(o, ot, s, i, a, x.shape[0], x.shape[1], fmt, _stream(stream)))


def transpose(dst, src, stream=0):
    """src: [rows, cols] fp8 codes -> dst: [cols, rows]."""
    if src.dim() != 2 or dst.dim() != 2 or dst.shape[0] != src.shape[1] or dst.shape[1] != src.shape[0]:
        raise ValueError("src must be [rows, cols] and dst [cols, rows]")
    if dst.dtype != src.dtype:
        raise ValueError("dst and src must have the same dtype")
    d = _dev(dst, "dst", _FP8)
    s = _dev(src, "src", _FP8)
    capi.check(capi.lib.llmq_transpose_u8(d, s, src.shape[0], src.shape[1], _stream(stream)))


def matmul(c, a, b, bias, scale_a, scale_b, M, N, K, accumulate=False, stream=0, workspace=None, b_e5m2=False,
           b_kmajor=False, a_kmajor=False):
    """TN matmul in the convention of the reference's kernels.h: row-major a[M,K], b[N,K] (e4m3) give
    row-major c[N,M] = (b @ a.T) * scale_a * scale_b (+ bias[M]) (+ c).  c: bf16 or fp32.
    workspace: optional device byte tensor (the reference passes a 32 MiB one); it enables the
    split-K path for outputs with too few tiles to fill the chip and the cut of a last, partial round of tiles into
    K segments (all operand modes).  b may hold e5m2 codes (the gradient
    dtype option): a float8_e5m2 tensor, or uint8 with b_e5m2=True."""
    L = capi.lib
    pws, ws_bytes = None, 0
    if workspace is not None:
        pws = _dev(workspace, "workspace", (torch.uint8, torch.int8, torch.float32))
        ws_bytes = workspace.numel() * workspace.element_size()
    if b_kmajor or a_kmajor:
        # the reference's modes TT (b stored [K, N] row-major, e.g. the output gradient dY[BT, OC] as the second operand
        # of the weight gradient without its transposed copy), NN (a stored [K, M], e.g. the weight W[OC, C] as the
        # first operand of the dgrad) and NT (both); whole 256-tiles only
        pa = _dev(a, "a", (torch.float8_e4m3fn, torch.uint8))
        pb = _dev(b, "b", (torch.float8_e4m3fn, torch.float8_e5m2, torch.uint8))
        pc = _dev(c, "c", (torch.bfloat16, torch.float32))
        if a.numel() != M * K or b.numel() != N * K or c.numel() != N * M:
            raise ValueError("operand sizes do not match M, N, K")
        if bias is not None and bias.numel() != M:
            raise ValueError("bias must have M elements")
        sa = _dev(scale_a, "scale_a", (torch.float32,), optional=True)
        sb = _dev(scale_b, "scale_b", (torch.float32,), optional=True)
        mode = (2 if b_kmajor else 3) if a_kmajor else 0      # EMMTranspose: TT = 0, TN = 1, NT = 2, NN = 3
        fmt = int(bool(b_e5m2) or b.dtype == torch.float8_e5m2)
        if c.dtype == torch.bfloat16:
            pbias = _dev(bias, "bias", (torch.bfloat16,), optional=True)
            capi.check(L.llmq_gemm_e4m3_bf16_mode(pc, pa, pb, pbias, sa, sb, pws, ws_bytes, M, N, K, mode, fmt, int(accumulate),
                                                  _stream(stream)), L)
        else:
            pbias = _dev(bias, "bias", (torch.bfloat16, torch.float32), optional=True)
            is_bf16 = int(bias is not None and bias.dtype == torch.bfloat16)
            capi.check(L.llmq_gemm_e4m3_f32_mode(pc, pa, pb, pbias, is_bf16, sa, sb, pws, ws_bytes, M, N, K, mode, fmt,
                                                 int(accumulate), _stream(stream)), L)
        return
    pa = _dev(a, "a", (torch.float8_e4m3fn, torch.uint8))   # e5m2 is supported for b only (kernels.h:92-94)
    pb = _dev(b, "b", (torch.float8_e4m3fn, torch.float8_e5m2, torch.uint8))
    b_e5m2 = bool(b_e5m2) or b.dtype == torch.float8_e5m2
    pc = _dev(c, "c", (torch.bfloat16, torch.float32))
    if a.numel() != M * K or b.numel() != N * K or c.numel() != N * M:
        raise ValueError("operand sizes do not match M, N, K")
    sa = _dev(scale_a, "scale_a", (torch.float32,), optional=True)
    sb = _dev(scale_b, "scale_b", (torch.float32,), optional=True)
    if c.dtype == torch.bfloat16:
        pbias = _dev(bias, "bias", (torch.bfloat16,), optional=True)
        if bias is not None and bias.numel() != M:
            raise ValueError("bias must have M elements")
        fn = L.llmq_gemm_tn_e4m3_e5m2_bf16 if b_e5m2 else L.llmq_gemm_tn_e4m3_bf16
        capi.check(fn(pc, pa, pb, pbias, sa, sb, pws, ws_bytes, M, N, K, int(accumulate), _stream(stream)), L)
    else:
        pbias = _dev(bias, "bias", (torch.bfloat16, torch.float32), optional=True)
        if bias is not None and bias.numel() != M:
            raise ValueError("bias must have M elements")
        is_bf16 = int(bias is not None and bias.dtype == torch.bfloat16)
        fn = L.llmq_gemm_tn_e4m3_e5m2_f32 if b_e5m2 else L.llmq_gemm_tn_e4m3_f32
        capi.check(fn(pc, pa, pb, pbias, is_bf16, sa, sb, pws, ws_bytes, M, N, K, int(accumulate), _stream(stream)), L)


_BIAS_FMT = {torch.float8_e4m3fn: 0, torch.float8_e5m2: 1, torch.bfloat16: 2}


def get_bias_backward_scratch_size(dtype, OC, BT=1 << 20):
    """Bytes of scratch backward_bias needs for gradients of `dtype` with OC columns (reference:
    get_bias_backward_scratch_size, src/kernels/bias.cu:142-148).  The reference sizes it from OC alone;
    here the number of row bands also depends on the row count, so the default assumes a large one
    (the value for a given B*T is never larger than for a larger B*T)."""
    return int(capi.lib.llmq_backward_bias_scratch_bytes(int(BT), int(OC), _BIAS_FMT[dtype]))


def backward_bias(dbias, dout, scale_a, scale_b, dbias_buffer, stream=0):
    """dbias[OC] (bf16) += scale_a * scale_b * dout.sum over all leading dims.  dout: [..., OC] in
    float8_e4m3fn, float8_e5m2 or bfloat16; scales both None or both fp32 device scalars
    (reference: src/kernels/bias.cu:151-195, src/binding/kernel_binding.cpp:445-459)."""
    if dout.dtype not in _BIAS_FMT:
        raise ValueError("dout: unsupported dtype %s" % dout.dtype)
    pd = _dev(dbias, "dbias", (torch.bfloat16,))
    po = _dev(dout, "dout")
    OC = dout.shape[-1]
    if dbias.numel() != OC:
        raise ValueError("dbias must have OC elements")
    BT = dout.numel() // OC if OC else 0
    sa = _dev(scale_a, "scale_a", (torch.float32,), optional=True)
    sb = _dev(scale_b, "scale_b", (torch.float32,), optional=True)
    pbuf = _dev(dbias_buffer, "dbias_buffer", (torch.float32,))
    capi.check(capi.lib.llmq_backward_bias_bf16(pd, po, _BIAS_FMT[dout.dtype], sa, sb, pbuf, dbias_buffer.numel() * 4,
                                                BT, OC, _stream(stream)))


_PRODUCER_DTYPES = (torch.bfloat16, torch.float32)


def _producer_entry(name, t):
    """The C entry point of producer `name` for tensors of t's dtype (bf16, or the fp32 overload) and that dtype as
    the one every tensor of the call must have."""
    if t.dtype not in _PRODUCER_DTYPES:
        raise ValueError("%s: tensors must be bfloat16 or float32 (got %s)" % (name, t.dtype))
    return getattr(capi.lib, "llmq_%s_%s" % (name, "f32" if t.dtype == torch.float32 else "bf16")), (t.dtype,)


def _swiglu_dims(inp, other, name):
    """inp: [B, T, 2C]; other: [B, T, C] (reference: src/binding/kernel_binding.cpp:289-322)."""
    if inp.dim() != 3 or other.dim() != 3:
        raise ValueError("inp and %s must have 3 dimensions" % name)
    if inp.shape[2] % 2 or inp.shape[0] != other.shape[0] or inp.shape[1] != other.shape[1] or inp.shape[2] != 2 * other.shape[2]:
        raise ValueError("inp must be [B, T, 2C] and %s [B, T, C]" % name)
    return int(inp.shape[0]), int(inp.shape[1]), int(other.shape[2])


def swiglu_forward(out, inp, abs_max, stream=0):
    """out[B,T,C] = up * gate * sigmoid(gate) for inp[B,T,2C] = [up | gate] (bf16, or fp32 throughout); abs_max (fp32
    device scalar or None) receives max |out|."""
    B, T, Cc = _swiglu_dims(inp, out, "out")
    fn, dt = _producer_entry("swiglu_forward", inp)
    o = _dev(out, "out", dt)
    i = _dev(inp, "inp", dt)
    a = _dev(abs_max, "abs_max", (torch.float32,), optional=True)
    capi.check(fn(o, i, a, B, T, Cc, _stream(stream)))


def swiglu_forward_quant(out, scale, inp, abs_max, stream=0):
    """e4m3 codes of swiglu_forward(inp) for a known abs_max, the bytes of swiglu_forward followed by
    quantize_with_abs_max; scale[0] = abs_max / 448."""
    B, T, Cc = _swiglu_dims(inp, out, "out")
    o = _dev(out, "out", (torch.float8_e4m3fn, torch.uint8))
    s = _dev(scale, "scale", (torch.float32,), optional=True)
    i = _dev(inp, "inp", (torch.bfloat16,))
    a = _dev(abs_max, "abs_max", (torch.float32,))
    capi.check(capi.lib.llmq_swiglu_forward_quant_bf16(o, s, i, a, B, T, Cc, _stream(stream)))


def swiglu_backward(dinp, dout, inp, abs_max, stream=0):
    """dinp[B,T,2C] = [dup | dgate] from dout[B,T,C] and the forward input; abs_max receives max |dinp|."""
    B, T, Cc = _swiglu_dims(inp, dout, "dout")
    if dinp.shape != inp.shape:
        raise ValueError("dinp must have the shape of inp")
    fn, dt = _producer_entry("swiglu_backward", inp)
    d = _dev(dinp, "dinp", dt)
    g = _dev(dout, "dout", dt)
    i = _dev(inp, "inp", dt)
    a = _dev(abs_max, "abs_max", (torch.float32,), optional=True)
    capi.check(fn(d, g, i, a, B, T, Cc, _stream(stream)))


def rmsnorm_forward(out, rms, inp, weight, abs_max, epsilon, stream=0):
    """out[B,T,C] = bf16(bf16(inp / rms(inp)) * weight), rms[B,T] = 1/sqrt(mean(inp^2) + epsilon); abs_max (fp32
    device scalar or None) receives max |out| (reference: src/binding/kernel_binding.cpp:130-143).  fp32 tensors
    throughout take the fp32 overload (no intermediate rounding)."""
    if inp.dim() != 3 or out.shape != inp.shape or weight.dim() != 1 or weight.shape[0] != inp.shape[2]:
        raise ValueError("inp and out must be [B, T, C] and weight [C]")
    if rms is not None and (rms.dim() != 2 or rms.shape[0] != inp.shape[0] or rms.shape[1] != inp.shape[1]):
        raise ValueError("rms must be [B, T]")
    fn, dt = _producer_entry("rmsnorm_forward", inp)
    o = _dev(out, "out", dt)
    r = _dev(rms, "rms", (torch.float32,), optional=True)
    i = _dev(inp, "inp", dt)
    w = _dev(weight, "weight", dt)
    a = _dev(abs_max, "abs_max", (torch.float32,), optional=True)
    B, T, Cc = (int(v) for v in inp.shape)
    capi.check(fn(o, r, i, w, a, float(epsilon), B, T, Cc, _stream(stream)))


def fused_residual_rmsnorm_forward(residual, normed, rrms, inp1, inp2, weight, abs_max, epsilon, stream=0):
    """residual = bf16(inp1 + inp2); normed, rrms = rmsnorm(residual) as above
    (reference: src/binding/kernel_binding.cpp:172-190)."""
    if inp1.dim() != 3 or any(t.shape != inp1.shape for t in (inp2, residual, normed)) or weight.dim() != 1 \
            or weight.shape[0] != inp1.shape[2]:
        raise ValueError("inp1, inp2, residual and normed must be [B, T, C] and weight [C]")
    if rrms.dim() != 2 or rrms.shape[0] != inp1.shape[0] or rrms.shape[1] != inp1.shape[1]:
        raise ValueError("rrms must be [B, T]")
    fn, dt = _producer_entry("fused_residual_rmsnorm_forward", inp1)
    ptrs = [_dev(t, n, dt) for t, n in ((residual, "residual"), (normed, "normed"))]
    r = _dev(rrms, "rrms", (torch.float32,))
    ins = [_dev(t, n, dt) for t, n in ((inp1, "inp1"), (inp2, "inp2"), (weight, "weight"))]
    a = _dev(abs_max, "abs_max", (torch.float32,), optional=True)
    N, Cc = int(inp1.shape[0] * inp1.shape[1]), int(inp1.shape[2])
    capi.check(fn(ptrs[0], ptrs[1], r, ins[0], ins[1], ins[2], a, float(epsilon), N, Cc, _stream(stream)))


def get_rmsnorm_backward_scratch_size(C):
    """Number of fp32 elements of the scratch tensor rmsnorm_backward needs for rows of C elements (the reference's
    binding sizes it in fp32 elements too: scripts/test_kernels.py:149)."""
    return int(capi.lib.llmq_rmsnorm_backward_scratch_bytes(int(C))) // 4


def rmsnorm_backward(dinp, dweight, scratch, dresidual, dout, inp, weight, rstd, abs_max, stream=0):
    """dinp = dresidual + d(rmsnorm)/d(inp) . dout; dweight += d/d(weight); abs_max receives max |dinp|
    (reference: src/binding/kernel_binding.cpp:145-169).  scratch: fp32 device tensor of
    get_rmsnorm_backward_scratch_size(C) elements."""
    if inp.dim() != 3 or any(t.shape != inp.shape for t in (dinp, dresidual, dout)) or weight.dim() != 1 \
            or weight.shape[0] != inp.shape[2] or dweight.shape != weight.shape:
        raise ValueError("dinp, dresidual, dout and inp must be [B, T, C], weight and dweight [C]")
    if rstd.dim() != 2 or rstd.shape[0] != inp.shape[0] or rstd.shape[1] != inp.shape[1]:
        raise ValueError("rstd must be [B, T]")
    fn, bf = _producer_entry("rmsnorm_backward", inp)
    p = [_dev(t, n, bf) for t, n in ((dinp, "dinp"), (dweight, "dweight"))]
    sc = _dev(scratch, "scratch")
    q = [_dev(t, n, bf) for t, n in ((dresidual, "dresidual"), (dout, "dout"), (inp, "inp"), (weight, "weight"))]
    r = _dev(rstd, "rstd", (torch.float32,))
    a = _dev(abs_max, "abs_max", (torch.float32,), optional=True)
    B, T, Cc = (int(v) for v in inp.shape)
    capi.check(fn(p[0], p[1], sc, scratch.numel() * scratch.element_size(), q[0], q[1], q[2], q[3], r, a, B, T, Cc,
                  _stream(stream)))


def _rope(name, out, inp, freqs_cis, abs_max, Nq, Nkv, stream):
    """Tensors [B, T, (Nq + 2 Nkv) * HD] bf16 with freqs_cis [T, HD] fp16, or fp32 with an fp32 table (reference:
    src/binding/kernel_binding.cpp:193-223)."""
    if inp.dim() != 3 or out.shape != inp.shape or freqs_cis.dim() != 2 or freqs_cis.shape[0] < inp.shape[1]:
        raise ValueError("inp and out must be [B, T, C] and freqs_cis [>= T, HD]")
    HD = int(freqs_cis.shape[1])
    if HD == 0 or inp.shape[2] != (Nq + 2 * Nkv) * HD:
        raise ValueError("C must equal (Nq + 2 Nkv) * head_dim")
    fn, dt = _producer_entry(name, inp)
    o = _dev(out, "out", dt)
    i = _dev(inp, "inp", dt)
    f = _dev(freqs_cis, "freqs_cis", (torch.float32 if inp.dtype == torch.float32 else torch.float16,))
    a = _dev(abs_max, "abs_max", (torch.float32,), optional=True)
    capi.check(fn(o, i, f, a, int(inp.shape[0]), int(inp.shape[1]), int(Nq), int(Nkv), HD, _stream(stream)))


def rope_forward(out, inp, freqs_cis, abs_max, Nq, Nkv, stream=0):
    """Rotary embedding of the query and key heads of the fused QKV tensor (out may be inp); abs_max receives max |out|."""
    _rope("rope_forward", out, inp, freqs_cis, abs_max, Nq, Nkv, stream)


def rope_backward(dinp, dout, freqs_cis, abs_max, Nq, Nkv, stream=0):
    """Gradient of rope_forward: the rotation by the negative angle."""
    _rope("rope_backward", dinp, dout, freqs_cis, abs_max, Nq, Nkv, stream)


def precompute_freqs_cis(dim, end, theta, dtype=torch.float16):
    """Host tensor [end, dim] of (cos, sin) pairs, fp16 (for bf16 tensors) or fp32 (reference: precompute_freqs_cis,
    src/kernels/rope.cu:15-40)."""
    if dtype not in (torch.float16, torch.float32):
        raise ValueError("precompute_freqs_cis: the table is float16 or float32")
    tab = torch.empty((end, dim), dtype=dtype)
    fn = capi.lib.llmq_precompute_freqs_cis_f32 if dtype == torch.float32 else capi.lib.llmq_precompute_freqs_cis_f16
    capi.check(fn(tab.data_ptr(), int(dim), int(end), float(theta)))
    return tab


def adamw_update(params, grads, m, v, learning_rate, beta1, beta2, t, eps, weight_decay, grad_scale, m_scales=None,
                 abs_max=None, seed=0, stream=0):
    """In-place AdamW step on bf16 params with stochastic rounding (reference:
    src/binding/kernel_binding.cpp:536-551).  Moments: fp32 / fp32, bf16 / fp32, bf16 / bf16, or an e4m3 first
    moment (float8_e4m3fn or uint8 codes) with m_scales, one fp32 scale per 128 elements, and a bf16 second moment; or
    fp32 params, grads and moments (no stochastic rounding).  grad_scale: fp32 device scalar.  abs_max, if given, is merged with max |new params| (not reset)."""
    if m_scales is not None or m.dtype in (torch.float8_e4m3fn, torch.uint8):
        n = params.numel()
        if m_scales is None or any(x.numel() != n for x in (grads, m, v)) or m_scales.numel() < (n + 127) // 128:
            raise ValueError("adamw_update: the e4m3 first moment needs m_scales with one entry per 128 elements")
        capi.check(capi.lib.llmq_adamw_update_bf16_fp8m(
            _dev(params, "params", (torch.bfloat16,)), _dev(grads, "grads", (torch.bfloat16,)),
            _dev(m, "m", (torch.float8_e4m3fn, torch.uint8)), _dev(m_scales, "m_scales", (torch.float32,)),
            _dev(v, "v", (torch.bfloat16,)), n, float(learning_rate), float(beta1), float(beta2), int(t), float(eps),
            float(weight_decay), _dev(grad_scale, "grad_scale", (torch.float32,)),
            _dev(abs_max, "abs_max", (torch.float32,), optional=True), int(seed) & 0xFFFFFFFF, _stream(stream)))
        return
    n = params.numel()
    if any(x.numel() != n for x in (grads, m, v)):
        raise ValueError("adamw_update: shape mismatch")
    if params.dtype == torch.float32:       # the all-fp32 overload: nothing to round stochastically, seed unused
        f32 = (torch.float32,)
        capi.check(capi.lib.llmq_adamw_update_f32(
            _dev(params, "params", f32), _dev(grads, "grads", f32), _dev(m, "m", f32), _dev(v, "v", f32), n, float(learning_rate),
            float(beta1), float(beta2), int(t), float(eps), float(weight_decay), _dev(grad_scale, "grad_scale", f32),
            _dev(abs_max, "abs_max", f32, optional=True), int(seed) & 0xFFFFFFFF, _stream(stream)))
        return
    p = _dev(params, "params", (torch.bfloat16,))
    g = _dev(grads, "grads", (torch.bfloat16,))
    pm = _dev(m, "m", (torch.float32, torch.bfloat16))
    pv = _dev(v, "v", (torch.float32, torch.bfloat16))
    gs = _dev(grad_scale, "grad_scale", (torch.float32,))
    a = _dev(abs_max, "abs_max", (torch.float32,), optional=True)
    capi.check(capi.lib.llmq_adamw_update_bf16(p, g, pm, int(m.dtype == torch.bfloat16), pv, int(v.dtype == torch.bfloat16), n,
                                               float(learning_rate), float(beta1), float(beta2), int(t), float(eps),
                                               float(weight_decay), gs, a, int(seed) & 0xFFFFFFFF, _stream(stream)))
