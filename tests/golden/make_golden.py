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
adamw_kat.npz    known answers for the optimizer's integer hash and stochastic rounding, and two whole AdamW steps
                 (bf16 / bf16 moments; e4m3 first moment with 128-element block scales):
                 "hash":  SquirrelNoise5 (src/kernels/squirrel_noise.cuh:15-36) for a list of (position, seed), with
                          Python integers reduced mod 2^32 after every step;
                 "sr":    stochastic rounding of fp32 patterns to bf16 and to e4m3 (squirrel_noise.cuh:47-75) for a
                          list of (pattern, random): the threshold comparison on Python integers, the final
                          conversion by the nearest-code search used for fp8_encode.npz (bf16: integer RNE);
                 "step":  src/kernels/adamw.cu:22-113 on 384 parameters: every fp32 operation through float64 with one
                          final rounding (innocuous for +, *, /, sqrt, Figueroa), the three fused multiply-adds in exact
                          rational arithmetic rounded once to fp32; the parameter line is evaluated in its contracted
                          form fma(-lr, fma(wd, p, q), p), which the reference leaves to its compiler.
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



# ---------------------------------------------------------------------------------------- AdamW known answers
M32 = 0xFFFFFFFF


def squirrel_noise_5(position, seed):
    b = position & M32
    b = (b * 0xd2a80a3f) & M32
    b = (b + seed) & M32
    b ^= b >> 9
    b = (b + 0xa884f197) & M32
    b ^= b >> 11
    b = (b * 0x6C736F4B) & M32
    b ^= b >> 13
    b = (b + 0xB79F3ABB) & M32
    b ^= b >> 15
    b = (b * 0x1b56c4f5) & M32
    b ^= b >> 17
    return b


def rotl(x, k):
    k %= 32
    return ((x << k) | (x >> (32 - k))) & M32 if k else x


def f32(x):
    return float(np.float32(x))


def bits_of(x):
    return int(np.float32(x).view(np.uint32))


def float_of(bits):
    return float(np.uint32(bits).view(np.float32))


def bf16_rne_bits(pattern):
    """fp32 pattern -> bf16 pattern, round to nearest even (finite values)."""
    return ((pattern + 0x7FFF + ((pattern >> 16) & 1)) >> 16) & 0xFFFF


def sr_bf16(x, random):
    b = bits_of(x)
    b = (b | 0xFFFF) if (b & 0xFFFF) > (random & 0xFFFF) else (b & ~0xFFFF & M32)
    return bf16_rne_bits(b)


def e4m3_nearest(y):
    return int(encode_nearest(np.array([y], dtype=np.float32), E4M3)[0])


def sr_e4m3(x, random):
    x = f32(x)
    if abs(x) > 448.0 or abs(x) < 0.015625:
        return e4m3_nearest(x)
    b = bits_of(x)
    b = (b | 0xFFFFF) if (b & 0xFFFFF) > (random & 0xFFFFF) else (b & ~0xFFFFF & M32)
    return e4m3_nearest(float_of(b))


def round_fraction_to_f32(q):
    """Exact rational -> nearest fp32 (ties to even), normal range."""
    from fractions import Fraction
    if q == 0:
        return 0.0
    sign = -1 if q < 0 else 1
    q = abs(q)
    e = q.numerator.bit_length() - q.denominator.bit_length()
    if Fraction(2) ** e > q:
        e -= 1
    assert Fraction(2) ** e <= q < Fraction(2) ** (e + 1) and -126 <= e <= 127
    scaled = q / Fraction(2) ** (e - 23)          # in [2^23, 2^24)
    n, rem = divmod(scaled.numerator, scaled.denominator)
    twice = 2 * rem
    if twice > scaled.denominator or (twice == scaled.denominator and n & 1):
        n += 1
    return sign * float(Fraction(n) * Fraction(2) ** (e - 23))


def fma32(a, b, c):
    from fractions import Fraction
    return round_fraction_to_f32(Fraction(f32(a)) * Fraction(f32(b)) + Fraction(f32(c)))


def adamw_step(p_bits, g_bits, m_in, v_bits, fp8m, m_scales, lr, beta1, beta2, t, eps, wd, gs, seed):
    """One AdamW step on Python numbers.  m_in: bf16 patterns, or e4m3 codes when fp8m."""
    dec4 = decode_table(E4M3)
    lr, beta1, beta2, eps, wd, gs = (f32(x) for x in (lr, beta1, beta2, eps, wd, gs))
    c1 = f32(1.0 / f32(1.0 - f32(np.float32(beta1) ** np.float32(t))))
    c2 = f32(1.0 / f32(1.0 - f32(np.float32(beta2) ** np.float32(t))))
    n = len(p_bits)
    p_out, v_out, m_new = [], [], []
    for i in range(n):
        p_old = float_of(int(p_bits[i]) << 16)
        v_old = float_of(int(v_bits[i]) << 16)
        if fp8m:
            m_old = f32(float(dec4[int(m_in[i])]) * f32(m_scales[i // 128]))
        else:
            m_old = float_of(int(m_in[i]) << 16)
        grad = f32(gs * float_of(int(g_bits[i]) << 16))
        mn = fma32(beta1, m_old, fma32(-beta1, grad, grad))
        g2 = f32(grad * grad)
        vn = fma32(beta2, v_old, fma32(-beta2, g2, g2))
        random = squirrel_noise_5(i, seed)
        m_hat, v_hat = f32(mn * c1), f32(vn * c2)
        den = f32(f32(np.sqrt(np.float64(v_hat))) + eps)
        quot = f32(m_hat / den)
        pn = fma32(-lr, fma32(wd, p_old, quot), p_old)
        p_out.append(sr_bf16(pn, random))
        v_out.append(sr_bf16(vn, rotl(random, 20)))
        m_new.append(mn)
    if not fp8m:
        m_out = [sr_bf16(m_new[i], rotl(squirrel_noise_5(i - i % 8, 51245), 7 * (i % 8))) for i in range(n)]
        return p_out, m_out, None, v_out
    m_out, scales = [], []
    for b0 in range(0, n, 128):
        blk = m_new[b0:b0 + 128]
        amax = max(abs(x) for x in blk)
        factor, scale = 1.0, 1.0
        if amax > f32(1e-10):
            factor = f32(448.0 / amax)
            scale = f32(1.0 / factor)
        scales.append(scale)
        for k, x in enumerate(blk):
            i = b0 + k
            m_out.append(sr_e4m3(f32(x * factor), rotl(squirrel_noise_5(i - i % 8, 51245), 7 * (i % 8))))
    return p_out, m_out, scales, v_out


def make_adamw_kat():
    rng = np.random.default_rng(20250)
    out = {}
    pos = np.concatenate([[0, 1, 2, 7, 8, 255, 256, 0x7FFFFFFF, 0x80000000, 0xFFFFFFFF],
                          rng.integers(0, 1 << 32, 54)]).astype(np.uint32)
    seeds = np.concatenate([[0, 1, 51245, 0xFFFFFFFF], rng.integers(0, 1 << 32, 60)]).astype(np.uint32)
    out["hash_position"], out["hash_seed"] = pos, seeds
    out["hash_value"] = np.array([squirrel_noise_5(int(a), int(b)) for a, b in zip(pos, seeds)], dtype=np.uint32)
    # stochastic rounding: patterns near thresholds and random ones
    vals = np.concatenate([rng.standard_normal(200) * 10.0 ** rng.uniform(-4, 3, 200),
                           [0.0, -0.0, 448.0, 449.0, -500.0, 0.015625, 0.0156, -0.0157, 1.0, 1.0625, 447.9, 3e-5]]).astype(np.float32)
    rnd = rng.integers(0, 1 << 32, vals.size).astype(np.uint32)
    rnd[:8] = [0, 0xFFFF, 0xFFFFF, 0xFFFFFFFF, 0x8000, 0x80000, 1, 0xFFFE]
    out["sr_pattern"], out["sr_random"] = vals.view(np.uint32), rnd
    out["sr_bf16"] = np.array([sr_bf16(float(v), int(r)) for v, r in zip(vals, rnd)], dtype=np.uint16)
    out["sr_e4m3"] = np.array([sr_e4m3(float(v), int(r)) for v, r in zip(vals, rnd)], dtype=np.uint8)
    # whole steps
    n = 384
    p = f32_to_bf16_rne((rng.standard_normal(n) * 0.05).astype(np.float32))
    g = f32_to_bf16_rne((rng.standard_normal(n) * 1e-2).astype(np.float32))
    v = f32_to_bf16_rne((rng.uniform(0, 1, n) ** 4 * 1e-4).astype(np.float32))
    hyper = dict(lr=3e-3, beta1=0.9, beta2=0.95, t=3, eps=1e-8, wd=0.1, gs=0.5, seed=1234567)
    out["step_hyper"] = np.array([hyper[k] for k in ("lr", "beta1", "beta2", "t", "eps", "wd", "gs", "seed")], dtype=np.float64)
    out["step_p"], out["step_g"], out["step_v"] = p, g, v
    m16 = f32_to_bf16_rne((rng.standard_normal(n) * 5e-3).astype(np.float32))
    po, mo, _, vo = adamw_step(p, g, m16, v, False, None, **hyper)
    out["bf16_m"], out["bf16_p_out"], out["bf16_m_out"], out["bf16_v_out"] = m16, np.array(po, np.uint16), np.array(mo, np.uint16), np.array(vo, np.uint16)
    m8 = rng.integers(0, 256, n).astype(np.uint8)
    m8[(m8 & 0x7F) == 0x7F] ^= 1
    m8[256:384] = 0                                   # a block whose new moment comes from the gradient alone
    g8 = g.copy()
    g8[256:320] = 0                                   # half of it exactly zero
    ms = np.array([2.5e-5, 1.0 / 448, 1.0], dtype=np.float32)
    po, mo, so, vo = adamw_step(p, g8, m8, v, True, ms, **hyper)
    out["fp8_g"], out["fp8_m"], out["fp8_scales"] = g8, m8, ms
    out["fp8_p_out"], out["fp8_m_out"], out["fp8_v_out"] = np.array(po, np.uint16), np.array(mo, np.uint8), np.array(vo, np.uint16)
    out["fp8_scales_out"] = np.array(so, dtype=np.float32)
    np.savez_compressed(os.path.join(HERE, "adamw_kat.npz"), **out)

if __name__ == "__main__":
    make_fp8_encode()
    make_gemm_kat()
    make_producers()
    make_adamw_kat()
    for f in ("fp8_encode.npz", "gemm_kat.npz", "producers.npz", "adamw_kat.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
