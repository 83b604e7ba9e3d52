"""Writes the golden fixtures of this directory.  Run once: python tests/golden/make_golden.py

Everything here is computed from the published definitions with numpy alone (no call into oracle/ or
into the HIP library), by a different method than the implementations under test use, so that the
fixtures are independent evidence for both:

fp8_encode.npz   all 65536 bf16 bit patterns quantized with five abs-max values, to e4m3 and to e5m2.
                 Method: y = fp32(scale * x) with numpy's IEEE fp32 arithmetic, scale = 448 / max(absmax, 1e-10)
                 (src/kernels/quant.cu:79-82); then a search for the nearest representable code value in
                 float64 (exact: y and every code value are fp32 numbers), ties to the even code, saturation
                 to the largest finite code, NaN -> 0x7F.  The code values come from the formats' definition
                 (OCP 8-bit floating point: E4M3 bias 7 without infinities, E5M2 bias 15).  While writing, the
                 finite inputs are cross-checked against torch's CPU float8 casts.
gemm_kat.npz     two GEMM cases in the library's convention c[N, M] = b[N, K] . a[M, K]^T * sa * sb + bias[M]
                 (src/kernels/matmul.cpp:59-142):
                 "int":  integer-valued operands in [-15, 15] (the construction of src/testing/test-gemm.cpp:54-85),
                         power-of-two scales and integer bias, so every fp32 partial sum is exact in any order and
                         the bf16 / fp32 outputs are known bit for bit; computed with int64 arithmetic.
                 "rnd":  random non-NaN codes and arbitrary scales; the exact sum of products and the sum of their
                         magnitudes in float64 (every product of two e4m3 values is exact in float64 and so is a
                         sum of 256 of them), to be met within the stated GEMM tolerance.
producers.npz    small inputs and float64 results of swiglu (src/kernels/swiglu.cu:20-36), rmsnorm
                 (src/kernels/rmsnorm.cu:22-83) and the rotary embedding (src/kernels/rope.cu:42-100), straight
                 from their formulas; implementations computing in fp32 and rounding to bf16 meet them within
                 bf16 rounding.
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def bf16_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_rne(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def code_values(exp_bits, man_bits, bias, top_code):
    """Magnitudes of the 7-bit codes 0 .. top_code of a binary8 format (float64, exact)."""
    vals = []
    for c in range(top_code + 1):
        e, m = c >> man_bits, c & ((1 << man_bits) - 1)
        if e == 0:
            vals.append(m * 2.0 ** (1 - bias - man_bits))
        else:
            vals.append(((1 << man_bits) + m) * 2.0 ** (e - bias - man_bits))
    return np.array(vals, dtype=np.float64)


E4M3 = code_values(4, 3, 7, 0x7E)    # 0 .. 448
E5M2 = code_values(5, 2, 15, 0x7B)   # 0 .. 57344


def encode_nearest(y, vals):
    y = np.ascontiguousarray(y, dtype=np.float32)
    top = len(vals) - 1
    a = np.abs(y.astype(np.float64))
    a = np.where(np.isnan(a), 0.0, a)
    hi = np.clip(np.searchsorted(vals, a, side="left"), 0, top)
    lo = np.clip(hi - 1, 0, top)
    dlo, dhi = np.abs(a - vals[lo]), np.abs(vals[hi] - a)
    code = np.where(dlo < dhi, lo, np.where(dhi < dlo, hi, np.where(lo % 2 == 0, lo, hi)))
    code = np.where(a >= vals[top], top, code)
    out = (code.astype(np.uint8) | ((y.view(np.uint32) >> 31).astype(np.uint8) << 7)).astype(np.uint8)
    out[np.isnan(y)] = 0x7F
    return out


def make_fp8_encode():
    import torch
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = bf16_to_f32(bits)
    absmax = np.array([1.0, 5.15625, 0.072265625, 3.0e-5, 1.0e4], dtype=np.float32)
    scale = (np.float32(448.0) / np.maximum(absmax, np.float32(1e-10))).astype(np.float32)
    recip = (np.float32(1.0) / scale).astype(np.float32)
    e4 = np.empty((absmax.size, 65536), np.uint8)
    e5 = np.empty((absmax.size, 65536), np.uint8)
    for i, s in enumerate(scale):
        with np.errstate(over="ignore", invalid="ignore"):
            y = (s * x).astype(np.float32)
        e4[i], e5[i] = encode_nearest(y, E4M3), encode_nearest(y, E5M2)
        fin = ~np.isnan(y)
        t = torch.from_numpy(y[fin])
        assert np.array_equal(e4[i][fin], t.clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy())
        assert np.array_equal(e5[i][fin], t.clamp(-57344.0, 57344.0).to(torch.float8_e5m2).view(torch.uint8).numpy())
    np.savez_compressed(os.path.join(HERE, "fp8_encode.npz"), absmax=absmax, scale_bits=scale.view(np.uint32),
                        recip_bits=recip.view(np.uint32), e4m3=e4, e5m2=e5)


def decode_table(vals):
    tab = np.full(256, np.nan)
    tab[:len(vals)] = vals
    tab[128:128 + len(vals)] = -vals
    return tab


def make_gemm_kat():
    rng = np.random.default_rng(20240607)
    tab = decode_table(E4M3)
    code_of_int = {int(v): c for c, v in enumerate(E4M3) if v == int(v) and v <= 15}
    out = {}
    # integer case
    M, N, K = 256, 128, 256
    ai = rng.integers(-15, 16, size=(M, K))
    bi = rng.integers(-15, 16, size=(N, K))
    to_code = np.vectorize(lambda v: code_of_int[abs(int(v))] | (0x80 if v < 0 else 0), otypes=[np.uint8])
    a, b = to_code(ai), to_code(bi)
    bias_i = rng.integers(-64, 65, size=M)
    sa, sb = np.float32(0.5), np.float32(0.0625)
    acc = bi.astype(np.int64) @ ai.astype(np.int64).T                     # [N, M], |acc| <= 225 * 256 < 2^16
    c = acc.astype(np.float64) * float(sa) * float(sb) + bias_i[None, :]  # multiples of 2^-5 below 2^11: exact in fp32
    c32 = c.astype(np.float32)
    assert np.array_equal(c32.astype(np.float64), c)
    out.update(int_a=a, int_b=b, int_sa=sa, int_sb=sb, int_bias_bf16=f32_to_bf16_rne(bias_i.astype(np.float32)),
               int_c_f32=c32, int_c_bf16=f32_to_bf16_rne(c32))
    # random codes
    M, N, K = 128, 128, 256
    a = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    b = rng.integers(0, 256, size=(N, K)).astype(np.uint8)
    a[(a & 0x7F) == 0x7F] = 0x3A
    b[(b & 0x7F) == 0x7F] = 0xB1
    av, bv = tab[a], tab[b]
    exact = bv @ av.T                                                      # products exact; |sum| < 2^26 with 2^-18 grain
    # float64 matmul may reorder, but every partial sum is a multiple of 2^-18 below 2^27: exact in 53 bits
    sumabs = np.abs(bv) @ np.abs(av).T
    out.update(rnd_a=a, rnd_b=b, rnd_sa=np.float32(0.0123), rnd_sb=np.float32(3.7e-3), rnd_exact=exact, rnd_sumabs=sumabs)
    np.savez_compressed(os.path.join(HERE, "gemm_kat.npz"), **out)


def make_producers():
    rng = np.random.default_rng(77)
    out = {}
    # swiglu: inp [BT, 2D] = (up | gate); out = up * gate * sigmoid(gate)
    BT, D = 24, 64
    inp = f32_to_bf16_rne((rng.standard_normal((BT, 2 * D)) * 2.0).astype(np.float32))
    dout = f32_to_bf16_rne(rng.standard_normal((BT, D)).astype(np.float32))
    x = bf16_to_f32(inp).astype(np.float64)
    up, gate = x[:, :D], x[:, D:]
    sig = 1.0 / (1.0 + np.exp(-gate))
    g = bf16_to_f32(dout).astype(np.float64)
    out.update(swiglu_inp=inp, swiglu_dout=dout, swiglu_out=up * gate * sig,
               swiglu_dinp=np.concatenate([g * gate * sig, g * up * sig * (1.0 + gate * (1.0 - sig))], axis=1))
    # rmsnorm: out = x * rsqrt(mean(x^2) + eps) * w, optionally x = inp1 + inp2 rounded to bf16 first
    BT, C, eps = 16, 128, 1e-5
    i1 = f32_to_bf16_rne(rng.standard_normal((BT, C)).astype(np.float32))
    i2 = f32_to_bf16_rne((0.5 * rng.standard_normal((BT, C))).astype(np.float32))
    w = f32_to_bf16_rne((1.0 + 0.1 * rng.standard_normal(C)).astype(np.float32))
    x = bf16_to_f32(i1).astype(np.float64)
    rstd = 1.0 / np.sqrt((x * x).mean(axis=1) + eps)
    res_bits = f32_to_bf16_rne(bf16_to_f32(i1) + bf16_to_f32(i2))
    xr = bf16_to_f32(res_bits).astype(np.float64)
    rstd_r = 1.0 / np.sqrt((xr * xr).mean(axis=1) + eps)
    wv = bf16_to_f32(w).astype(np.float64)
    out.update(rms_inp1=i1, rms_inp2=i2, rms_weight=w, rms_eps=np.float32(eps), rms_out=x * rstd[:, None] * wv,
               rms_rstd=rstd, rms_residual=res_bits, rms_fused_out=xr * rstd_r[:, None] * wv, rms_fused_rstd=rstd_r)
    # rope: [B, T, Nq + 2 Nkv, HD]; (real, imag) = (x[d], x[d + HD/2]) rotated by the angle t * theta^(-2d/HD)
    # with the (cos, sin) factors rounded to fp16 as the reference's table holds them (src/kernels/rope.cu:15-31)
    B, T, Nq, Nkv, HD, theta = 2, 12, 4, 2, 32, 10000.0
    N = Nq + 2 * Nkv
    qkv = f32_to_bf16_rne(rng.standard_normal((B, T, N, HD)).astype(np.float32))
    inv = (1.0 / np.power(np.float32(theta), (2 * np.arange(HD // 2)).astype(np.float32) / np.float32(HD))).astype(np.float32)
    ang = (np.arange(T, dtype=np.float32)[:, None] * inv[None, :]).astype(np.float32)
    table = np.stack([np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16)], axis=-1).reshape(T, HD)
    cs, sn = table[:, 0::2].astype(np.float64), table[:, 1::2].astype(np.float64)
    x = bf16_to_f32(qkv).astype(np.float64)
    re, im = x[..., :HD // 2], x[..., HD // 2:]
    c4, s4 = cs[None, :, None, :], sn[None, :, None, :]
    fwd = np.concatenate([re * c4 - im * s4, re * s4 + im * c4], axis=-1)
    bwd = np.concatenate([re * c4 + im * s4, -re * s4 + im * c4], axis=-1)
    fwd[:, :, Nq + Nkv:], bwd[:, :, Nq + Nkv:] = x[:, :, Nq + Nkv:], x[:, :, Nq + Nkv:]   # value heads pass through
    out.update(rope_qkv=qkv, rope_table_f16=table.view(np.uint16), rope_dims=np.array([B, T, Nq, Nkv, HD]),
               rope_theta=np.float32(theta), rope_forward=fwd, rope_backward=bwd)
    np.savez_compressed(os.path.join(HERE, "producers.npz"), **out)


if __name__ == "__main__":
    make_fp8_encode()
    make_gemm_kat()
    make_producers()
    for f in ("fp8_encode.npz", "gemm_kat.npz", "producers.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
