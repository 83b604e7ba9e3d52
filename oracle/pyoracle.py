"""ctypes loader for the CPU oracle (oracle/llmq_oracle.c + oracle/llmq_cpu_mt.c).

Test infrastructure only.  Arrays are numpy: bf16 tensors travel as uint16 bit patterns, e4m3/e5m2
tensors as uint8 codes.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libllmq_oracle.so")
_lib = None


def build(force=False):
    """Compile the oracle with gcc (a second or two)."""
    sources = [os.path.join(_HERE, f) for f in ("llmq_oracle.c", "llmq_cpu_mt.c", "Makefile")]
    stale = not os.path.exists(_LIB_PATH) or any(os.path.getmtime(f) > os.path.getmtime(_LIB_PATH) for f in sources)
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []), stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _p(arr, ctype):
    return arr.ctypes.data_as(C.POINTER(ctype))


def lib():
    global _lib
    if _lib is not None:
        return _lib
    build()
    L = C.CDLL(_LIB_PATH)
    u8p, u16p, f32p, f64p, i32p = (C.POINTER(t) for t in (C.c_uint8, C.c_uint16, C.c_float, C.c_double, C.c_int32))
    L.orc_bf16_to_f32.restype = C.c_float
    L.orc_bf16_to_f32.argtypes = [C.c_uint16]
    L.orc_f32_to_bf16.restype = C.c_uint16
    L.orc_f32_to_bf16.argtypes = [C.c_float]
    L.orc_abs_max_bf16.restype = C.c_float
    L.orc_abs_max_bf16.argtypes = [u16p, C.c_int64]
    L.orc_abs_max_f32.restype = C.c_float
    L.orc_abs_max_f32.argtypes = [f32p, C.c_int64]
    L.orc_e4m3_encode.restype = C.c_uint8
    L.orc_e4m3_encode.argtypes = [C.c_float]
    L.orc_e4m3_decode.restype = C.c_float
    L.orc_e4m3_decode.argtypes = [C.c_uint8]
    L.orc_e5m2_encode.restype = C.c_uint8
    L.orc_e5m2_encode.argtypes = [C.c_float]
    L.orc_e5m2_decode.restype = C.c_float
    L.orc_e5m2_decode.argtypes = [C.c_uint8]
    L.orc_quant_scale.restype = None
    L.orc_quant_scale.argtypes = [C.c_float, f32p, f32p]
    for name in ("orc_quantize_e4m3_bf16", "orc_quantize_e5m2_bf16", "mt_quantize_e4m3_bf16"):
        f = getattr(L, name)
        f.restype = None
        f.argtypes = [u8p, f32p, u16p, C.c_float, C.c_int64]
    for name in ("orc_quantize_transpose_e4m3_bf16", "mt_quantize_transpose_e4m3_bf16"):
        f = getattr(L, name)
        f.restype = None
        f.argtypes = [u8p, f32p, u16p, C.c_float, C.c_int, C.c_int]
    for name in ("orc_transpose_u8", "mt_transpose_u8"):
        f = getattr(L, name)
        f.restype = None
        f.argtypes = [u8p, u8p, C.c_int, C.c_int]
    L.orc_gemm_tn_e4m3_exact.restype = None
    L.orc_gemm_tn_e4m3_exact.argtypes = [f64p, f64p, u8p, u8p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    L.orc_gemm_tn_e4m3_exact_sampled.restype = None
    L.orc_gemm_tn_e4m3_exact_sampled.argtypes = [f64p, f64p, u8p, u8p, C.c_int, C.c_int, C.c_int, i32p, i32p, C.c_int64]
    L.orc_gemm_epilogue_f32.restype = C.c_float
    L.orc_gemm_epilogue_f32.argtypes = [C.c_double, C.c_float, f32p, f32p]
    L.orc_gemm_tn_e4m3.restype = None
    L.orc_gemm_tn_e4m3.argtypes = [C.c_void_p, C.c_int, u8p, u8p, u16p, f32p, f32p, f32p,
                                   C.c_int, C.c_int, C.c_int, C.c_int]
    L.orc_fill_normal_bf16.restype = None
    L.orc_fill_normal_bf16.argtypes = [u16p, C.c_int64, C.c_uint64, C.c_uint64, C.c_float, C.c_float]
    L.orc_fill_student_t3_bf16.restype = None
    L.orc_fill_student_t3_bf16.argtypes = [u16p, C.c_int64, C.c_uint64, C.c_uint64, C.c_float]
    L.orc_fill_int_e4m3.restype = None
    L.orc_fill_int_e4m3.argtypes = [u8p, i32p, C.c_int64, C.c_uint64, C.c_uint64, C.c_int, C.c_int]
    L.mt_num_threads.restype = C.c_int
    L.mt_set_num_threads.argtypes = [C.c_int]
    L.mt_abs_max_bf16.restype = C.c_float
    L.mt_abs_max_bf16.argtypes = [u16p, C.c_int64]
    L.mt_gemm_tn_e4m3.restype = C.c_int
    L.mt_gemm_tn_e4m3.argtypes = [C.c_void_p, C.c_int, u8p, u8p, u16p, f32p, f32p,
                                  C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    L.orc_gemm_tn_fp8_exact.restype = None
    L.orc_gemm_tn_fp8_exact.argtypes = [f64p, f64p, u8p, u8p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    L.orc_gemm_tn_fp8_exact_sampled.restype = None
    L.orc_gemm_tn_fp8_exact_sampled.argtypes = [f64p, f64p, u8p, u8p, C.c_int, C.c_int, C.c_int, C.c_int, i32p, i32p,
                                                C.c_int64]
    L.orc_gemm_tn_fp8.restype = None
    L.orc_gemm_tn_fp8.argtypes = [C.c_void_p, C.c_int, u8p, u8p, C.c_int, u16p, f32p, f32p, f32p,
                                  C.c_int, C.c_int, C.c_int, C.c_int]
    L.mt_gemm_tn_fp8.restype = C.c_int
    L.mt_gemm_tn_fp8.argtypes = [C.c_void_p, C.c_int, u8p, u8p, C.c_int, u16p, f32p, f32p,
                                 C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    L.orc_quantize_fp8_f32.restype = None
    L.orc_quantize_fp8_f32.argtypes = [u8p, f32p, f32p, C.c_float, C.c_int64, C.c_int]
    L.orc_backward_bias_bf16.restype = None
    L.orc_backward_bias_bf16.argtypes = [u16p, C.c_void_p, C.c_int, f32p, f32p, C.c_int64, C.c_int, f64p, f64p]
    L.orc_swiglu_forward_bf16.restype = None
    L.orc_swiglu_forward_bf16.argtypes = [u16p, f64p, u16p, C.c_int64, C.c_int]
    L.orc_swiglu_backward_bf16.restype = None
    L.orc_swiglu_backward_bf16.argtypes = [u16p, f64p, u16p, u16p, C.c_int64, C.c_int]
    L.orc_rmsnorm_forward_bf16.restype = None
    L.orc_rmsnorm_forward_bf16.argtypes = [u16p, u16p, f32p, f64p, u16p, u16p, u16p, C.c_float, C.c_int64, C.c_int]
    L.orc_rmsnorm_backward_bf16.restype = None
    L.orc_rmsnorm_backward_bf16.argtypes = [u16p, u16p, f64p, f64p, f64p, f64p, u16p, u16p, u16p, u16p, f32p, C.c_int64, C.c_int]
    L.orc_rope_bf16.restype = None
    L.orc_rope_bf16.argtypes = [u16p, f64p, f64p, u16p, u16p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    L.orc_swiglu_forward_f32.restype = None
    L.orc_swiglu_forward_f32.argtypes = [f32p, f64p, f32p, C.c_int64, C.c_int]
    L.orc_swiglu_backward_f32.restype = None
    L.orc_swiglu_backward_f32.argtypes = [f32p, f64p, f32p, f32p, C.c_int64, C.c_int]
    L.orc_rmsnorm_forward_f32.restype = None
    L.orc_rmsnorm_forward_f32.argtypes = [f32p, f32p, f32p, f64p, f32p, f32p, f32p, C.c_float, C.c_int64, C.c_int]
    L.orc_rmsnorm_backward_f32.restype = None
    L.orc_rmsnorm_backward_f32.argtypes = [f32p, f32p, f64p, f64p, f64p, f64p, f32p, f32p, f32p, f32p, f32p, C.c_int64, C.c_int]
    L.orc_rope_f32.restype = None
    L.orc_rope_f32.argtypes = [f32p, f64p, f64p, f32p, f32p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    L.orc_squirrel_noise_5.restype = C.c_uint32
    L.orc_squirrel_noise_5.argtypes = [C.c_uint32, C.c_uint32]
    L.orc_stochastic_round_bf16.restype = C.c_uint16
    L.orc_stochastic_round_bf16.argtypes = [C.c_float, C.c_uint32]
    L.orc_adamw_update_bf16.restype = C.c_float
    L.orc_adamw_update_bf16.argtypes = [u16p, u16p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_float,
                                        C.c_float, C.c_int, C.c_float, C.c_float, C.c_float, C.c_uint32]
    L.orc_adamw_update_f32.restype = C.c_float
    L.orc_adamw_update_f32.argtypes = [f32p, f32p, f32p, f32p, C.c_int64, C.c_float, C.c_float, C.c_float, C.c_int, C.c_float,
                                       C.c_float, C.c_float]
    L.orc_adamw_update_bf16_fp8m.restype = C.c_float
    L.orc_adamw_update_bf16_fp8m.argtypes = [u16p, u16p, C.POINTER(C.c_uint8), C.POINTER(C.c_float), u16p, C.c_int64, C.c_float,
                                             C.c_float, C.c_float, C.c_int, C.c_float, C.c_float, C.c_float, C.c_uint32]
    L.orc_stochastic_round_e4m3.restype = C.c_uint8
    L.orc_stochastic_round_e4m3.argtypes = [C.c_float, C.c_uint32]
    L.orc_stochastic_round_bf16.restype = C.c_uint16
    L.orc_stochastic_round_bf16.argtypes = [C.c_float, C.c_uint32]
    L.orc_squirrel_noise_5.restype = C.c_uint32
    L.orc_squirrel_noise_5.argtypes = [C.c_uint32, C.c_uint32]
    _lib = L
    return L


# ---------------------------------------------------------------------------------- numpy helpers
def bf16_to_f32(bits):
    """uint16 bf16 patterns -> float32 (exact)."""
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(x):
    """float32 -> uint16 bf16 patterns, round to nearest even (finite inputs)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = u + (0x7FFF + ((u >> 16) & 1)).astype(np.uint32)
    out = (r >> 16).astype(np.uint16)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    if nan.any():
        out[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return out


_E4M3_TABLE = None


def e4m3_table():
    """float32[256] decode table of every e4m3 code (0x7F/0xFF are NaN)."""
    global _E4M3_TABLE
    if _E4M3_TABLE is None:
        L = lib()
        _E4M3_TABLE = np.array([L.orc_e4m3_decode(i) for i in range(256)], dtype=np.float32)
    return _E4M3_TABLE


def e5m2_table():
    """float32[256]: value of every e5m2 code (NaN / Inf codes included)."""
    L = lib()
    return np.array([L.orc_e5m2_decode(i) for i in range(256)], dtype=np.float32)


def e4m3_decode(codes):
    return e4m3_table()[np.asarray(codes, dtype=np.uint8)]


def abs_max_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    return float(lib().orc_abs_max_bf16(_p(x, C.c_uint16), x.size))


def quant_scale(absmax):
    s, d = C.c_float(), C.c_float()
    lib().orc_quant_scale(C.c_float(absmax), C.byref(s), C.byref(d))
    return s.value, d.value


def quantize_e4m3(x, absmax, mt=False, fmt="e4m3"):
    """Returns (codes uint8 like x, dequant scale float32)."""
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.uint8)
    d = C.c_float()
    name = ("mt_" if mt else "orc_") + "quantize_%s_bf16" % fmt
    getattr(lib(), name)(_p(out, C.c_uint8), C.byref(d), _p(x, C.c_uint16), C.c_float(absmax), x.size)
    return out, np.float32(d.value)


def quantize_transpose_e4m3(x, absmax, mt=False):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    rows, cols = x.shape
    out = np.empty((cols, rows), dtype=np.uint8)
    d = C.c_float()
    f = lib().mt_quantize_transpose_e4m3_bf16 if mt else lib().orc_quantize_transpose_e4m3_bf16
    f(_p(out, C.c_uint8), C.byref(d), _p(x, C.c_uint16), C.c_float(absmax), rows, cols)
    return out, np.float32(d.value)


def transpose_u8(x, mt=False):
    x = np.ascontiguousarray(x, dtype=np.uint8)
    rows, cols = x.shape
    out = np.empty((cols, rows), dtype=np.uint8)
    f = lib().mt_transpose_u8 if mt else lib().orc_transpose_u8
    f(_p(out, C.c_uint8), _p(x, C.c_uint8), rows, cols)
    return out


def gemm_exact(a, b, rows=None, b_e5m2=False):
    """a[M,K] e4m3 codes, b[N,K] e4m3 (or e5m2) codes -> (exact float64 [N,M], sum|terms| float64 [N,M]);
    rows=(n0,n1) restricts the computed rows (others are left zero)."""
    a = np.ascontiguousarray(a, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.uint8)
    M, K = a.shape
    N, K2 = b.shape
    assert K == K2
    n0, n1 = rows if rows is not None else (0, N)
    ex = np.zeros((N, M), dtype=np.float64)
    sa = np.zeros((N, M), dtype=np.float64)
    lib().orc_gemm_tn_fp8_exact(_p(ex, C.c_double), _p(sa, C.c_double), _p(a, C.c_uint8), _p(b, C.c_uint8),
                                int(b_e5m2), M, N, K, n0, n1)
    return ex, sa


def gemm_exact_sampled(a, b, idx_n, idx_m, b_e5m2=False):
    a = np.ascontiguousarray(a, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.uint8)
    M, K = a.shape
    N, _ = b.shape
    idx_n = np.ascontiguousarray(idx_n, dtype=np.int32)
    idx_m = np.ascontiguousarray(idx_m, dtype=np.int32)
    ex = np.zeros(idx_n.size, dtype=np.float64)
    sa = np.zeros(idx_n.size, dtype=np.float64)
    lib().orc_gemm_tn_fp8_exact_sampled(_p(ex, C.c_double), _p(sa, C.c_double), _p(a, C.c_uint8),
                                        _p(b, C.c_uint8), int(b_e5m2), M, N, K, _p(idx_n, C.c_int32),
                                        _p(idx_m, C.c_int32), idx_n.size)
    return ex, sa


def gemm_tn(a, b, sa=None, sb=None, bias=None, c_old=None, out_f32=False, mt=False, b_e5m2=False):
    """Full GEMM + epilogue.  bias: uint16 bf16 [M] or None.  c_old: previous c (accumulate) or None.
    Returns uint16 bf16 [N,M] or float32 [N,M]."""
    a = np.ascontiguousarray(a, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.uint8)
    M, K = a.shape
    N, _ = b.shape
    dt = np.float32 if out_f32 else np.uint16
    c = np.array(c_old, dtype=dt, copy=True).reshape(N, M) if c_old is not None else np.zeros((N, M), dtype=dt)
    keep_a = C.c_float(sa) if sa is not None else None
    keep_b = C.c_float(sb) if sb is not None else None
    fsa = C.pointer(keep_a) if keep_a is not None else None
    fsb = C.pointer(keep_b) if keep_b is not None else None
    bp = None
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.uint16)
        bp = _p(bias, C.c_uint16)
    if mt:
        rc = lib().mt_gemm_tn_fp8(c.ctypes.data, int(out_f32), _p(a, C.c_uint8), _p(b, C.c_uint8), int(b_e5m2), bp,
                                  fsa, fsb, M, N, K, int(c_old is not None), 0, N)
        assert rc == 0
    else:
        lib().orc_gemm_tn_fp8(c.ctypes.data, int(out_f32), _p(a, C.c_uint8), _p(b, C.c_uint8), int(b_e5m2), bp, None,
                              fsa, fsb, M, N, K, int(c_old is not None))
    return c


def fill_normal_bf16(n, seed, stream, mean=0.0, std=1.0):
    out = np.empty(int(n), dtype=np.uint16)
    lib().orc_fill_normal_bf16(_p(out, C.c_uint16), out.size, seed, stream, C.c_float(mean), C.c_float(std))
    return out


def fill_student_t3_bf16(n, seed, stream, scale=1.0):
    out = np.empty(int(n), dtype=np.uint16)
    lib().orc_fill_student_t3_bf16(_p(out, C.c_uint16), out.size, seed, stream, C.c_float(scale))
    return out


def fill_int_e4m3(n, seed, stream, lo=-15, hi=15):
    out = np.empty(int(n), dtype=np.uint8)
    vals = np.empty(int(n), dtype=np.int32)
    lib().orc_fill_int_e4m3(_p(out, C.c_uint8), _p(vals, C.c_int32), out.size, seed, stream, lo, hi)
    return out, vals


def backward_bias(dbias, dout, fmt, sa=None, sb=None):
    """dbias: uint16 bf16 [OC] (old value); dout: [BT, OC] uint8 codes (fmt "e4m3" / "e5m2") or uint16
    bf16 (fmt "bf16").  Returns (new dbias uint16 [OC], exact column sums float64, sum |values| float64)."""
    code = {"e4m3": 0, "e5m2": 1, "bf16": 2}[fmt]
    dout = np.ascontiguousarray(dout, dtype=np.uint16 if code == 2 else np.uint8)
    BT, OC = dout.shape
    out = np.array(dbias, dtype=np.uint16, copy=True)
    cs, ca = np.zeros(OC, dtype=np.float64), np.zeros(OC, dtype=np.float64)
    ka = C.c_float(sa) if sa is not None else None
    kb = C.c_float(sb) if sb is not None else None
    lib().orc_backward_bias_bf16(_p(out, C.c_uint16), dout.ctypes.data, code, C.pointer(ka) if ka is not None else None,
                                 C.pointer(kb) if kb is not None else None, BT, OC, _p(cs, C.c_double), _p(ca, C.c_double))
    return out, cs, ca


def quantize_f32(x, absmax, fmt="e4m3"):
    """x: float32 array -> (fp8 codes uint8, dequant scale float32), fp32-input overloads of quantize_with_abs_max."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint8)
    sc = np.zeros(1, dtype=np.float32)
    lib().orc_quantize_fp8_f32(_p(out, C.c_uint8), _p(sc, C.c_float), _p(x, C.c_float), C.c_float(absmax), x.size,
                               1 if fmt == "e5m2" else 0)
    return out, sc[0]


def _elem(arr):
    """(numpy dtype, ctypes element type, suffix of the oracle function) of a producer tensor: bf16 bits or fp32."""
    if np.asarray(arr).dtype == np.float32:
        return np.float32, C.c_float, "f32"
    return np.uint16, C.c_uint16, "bf16"


def swiglu_forward(inp):
    """inp: uint16 bf16 bits or float32 [BT, 2C] (rows [up | gate]) -> (out of the same type [BT, C], exact float64)."""
    dt, ct, sfx = _elem(inp)
    inp = np.ascontiguousarray(inp, dtype=dt)
    BT, C2 = inp.shape
    out = np.empty((BT, C2 // 2), dtype=dt)
    exact = np.empty((BT, C2 // 2), dtype=np.float64)
    getattr(lib(), "orc_swiglu_forward_" + sfx)(_p(out, ct), _p(exact, C.c_double), _p(inp, ct), BT, C2 // 2)
    return out, exact


def swiglu_backward(dout, inp):
    """dout: [BT, C], inp: [BT, 2C] (bf16 bits or float32) -> (dinp of the same type [BT, 2C] = [dup | dgate], exact)."""
    dt, ct, sfx = _elem(inp)
    inp = np.ascontiguousarray(inp, dtype=dt)
    dout = np.ascontiguousarray(dout, dtype=dt)
    BT, C2 = inp.shape
    dinp = np.empty((BT, C2), dtype=dt)
    exact = np.empty((BT, C2), dtype=np.float64)
    getattr(lib(), "orc_swiglu_backward_" + sfx)(_p(dinp, ct), _p(exact, C.c_double), _p(dout, ct), _p(inp, ct), BT, C2 // 2)
    return dinp, exact


def rmsnorm_forward(inp1, weight, eps, inp2=None):
    """inp1 (and inp2): bf16 bits or float32 [N, C]; weight: [C] of the same type.  Returns (normed [N, C], rrms
    float32 [N], exact float64 [N, C], residual [N, C] or None)."""
    dt, ct, sfx = _elem(inp1)
    inp1 = np.ascontiguousarray(inp1, dtype=dt)
    weight = np.ascontiguousarray(weight, dtype=dt)
    N, Cc = inp1.shape
    normed = np.empty((N, Cc), dtype=dt)
    rrms = np.empty(N, dtype=np.float32)
    exact = np.empty((N, Cc), dtype=np.float64)
    res = None
    p2 = None
    if inp2 is not None:
        inp2 = np.ascontiguousarray(inp2, dtype=dt)
        res = np.empty((N, Cc), dtype=dt)
        p2 = _p(inp2, ct)
    getattr(lib(), "orc_rmsnorm_forward_" + sfx)(_p(res, ct) if res is not None else None, _p(normed, ct),
                                                 _p(rrms, C.c_float), _p(exact, C.c_double), _p(inp1, ct), p2,
                                                 _p(weight, ct), C.c_float(eps), N, Cc)
    return normed, rrms, exact, res


def rmsnorm_backward(dresidual, dweight, dout, inp, weight, rstd):
    """bf16 bits or float32: dresidual, dout, inp [N, C]; dweight (old value), weight [C]; rstd float32 [N].
    Returns dict(dinp, dweight (same type), exact_dinp, mag_dinp, exact_dw, mag_dw (float64))."""
    dt, ct, sfx = _elem(inp)
    inp = np.ascontiguousarray(inp, dtype=dt)
    N, Cc = inp.shape
    dres = np.ascontiguousarray(dresidual, dtype=dt)
    dout = np.ascontiguousarray(dout, dtype=dt)
    weight = np.ascontiguousarray(weight, dtype=dt)
    rstd = np.ascontiguousarray(rstd, dtype=np.float32)
    dinp = np.empty((N, Cc), dtype=dt)
    dw = np.array(dweight, dtype=dt, copy=True)
    ed, md = np.empty((N, Cc)), np.empty((N, Cc))
    ew, mw = np.empty(Cc), np.empty(Cc)
    getattr(lib(), "orc_rmsnorm_backward_" + sfx)(_p(dinp, ct), _p(dw, ct), _p(ed, C.c_double), _p(md, C.c_double),
                                                  _p(ew, C.c_double), _p(mw, C.c_double), _p(dres, ct), _p(dout, ct),
                                                  _p(inp, ct), _p(weight, ct), _p(rstd, C.c_float), N, Cc)
    return dict(dinp=dinp, dweight=dw, exact_dinp=ed, mag_dinp=md, exact_dw=ew, mag_dw=mw)


def rope(inp, freqs, T, Nq, Nkv, backward=False):
    """inp: bf16 bits with an fp16-bits table, or float32 with a float32 table; inp [BT, Nq + 2 Nkv, HD], table [T, HD]
    of (cos, sin) pairs.  Returns (out of inp's type, exact float64, magnitude float64), all shaped like inp."""
    dt, ct, sfx = _elem(inp)
    inp = np.ascontiguousarray(inp, dtype=dt)
    freqs = np.ascontiguousarray(freqs, dtype=dt)
    BT, N, HD = inp.shape
    out = np.empty_like(inp)
    exact, mag = np.empty(inp.shape), np.empty(inp.shape)
    getattr(lib(), "orc_rope_" + sfx)(_p(out, ct), _p(exact, C.c_double), _p(mag, C.c_double), _p(inp, ct), _p(freqs, ct),
                                      BT, T, Nq, Nkv, HD, 1 if backward else 0)
    return out, exact, mag


def adamw_update(params, grads, m, v, lr, beta1, beta2, t, eps, wd, grad_scale, seed):
    """params, grads: bf16 bits; m, v: float32 arrays (fp32 moments) or uint16 bf16 bits -- or everything float32 (the
    all-fp32 overload).  Returns new (params, m, v, abs-max of the new params); inputs are not modified."""
    if np.asarray(params).dtype == np.float32:      # the all-fp32 overload: no stochastic rounding, seed unused
        p, g = np.array(params, dtype=np.float32, copy=True), np.ascontiguousarray(grads, dtype=np.float32)
        mm, vv = np.array(m, dtype=np.float32, copy=True), np.array(v, dtype=np.float32, copy=True)
        am = lib().orc_adamw_update_f32(_p(p, C.c_float), _p(g, C.c_float), _p(mm, C.c_float), _p(vv, C.c_float), p.size, lr, beta1,
                                        beta2, t, eps, wd, grad_scale)
        return p, mm, vv, np.float32(am)
    p = np.array(params, dtype=np.uint16, copy=True)
    g = np.ascontiguousarray(grads, dtype=np.uint16)
    mm, vv = np.array(m, copy=True), np.array(v, copy=True)
    md, vd = int(mm.dtype == np.uint16), int(vv.dtype == np.uint16)
    am = lib().orc_adamw_update_bf16(_p(p, C.c_uint16), _p(g, C.c_uint16), mm.ctypes.data, md, vv.ctypes.data, vd, p.size,
                                     lr, beta1, beta2, t, eps, wd, grad_scale, seed)
    return p, mm, vv, np.float32(am)


def adamw_update_fp8m(params, grads, m_codes, m_scales, v, lr, beta1, beta2, t, eps, wd, grad_scale, seed):
    """AdamW with e4m3 first moment + one fp32 scale per 128 elements, bf16 second moment.  params, grads, v: bf16
    bits; m_codes: uint8; m_scales: float32 [ceil(n / 128)].  Returns new (params, m_codes, m_scales, v, abs-max of
    the new params); inputs are not modified."""
    p = np.array(params, dtype=np.uint16, copy=True)
    g = np.ascontiguousarray(grads, dtype=np.uint16)
    mc = np.array(m_codes, dtype=np.uint8, copy=True)
    ms = np.array(m_scales, dtype=np.float32, copy=True)
    vv = np.array(v, dtype=np.uint16, copy=True)
    am = lib().orc_adamw_update_bf16_fp8m(_p(p, C.c_uint16), _p(g, C.c_uint16), _p(mc, C.c_uint8), _p(ms, C.c_float),
                                          _p(vv, C.c_uint16), p.size, lr, beta1, beta2, t, eps, wd, grad_scale, seed)
    return p, mc, ms, vv, np.float32(am)
