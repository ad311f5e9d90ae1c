"""ctypes binding of the CPU oracle (``liboracle.so``) -- TEST INFRASTRUCTURE ONLY.

Only the test-suite, the smoke check and the benchmark's labelled CPU-baseline leg
import this module; the shipped library never does. Every function takes and
returns numpy arrays in the ONNX layouts of the operators.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force: bool = False) -> str:
    """Compile liboracle.so with gcc (a few seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True)
    return _LIB_PATH


class ConvGeom(C.Structure):
    _fields_ = [(n, C.c_int64) for n in (
        "n", "c_in", "h", "w", "c_out", "kh", "kw", "stride_h", "stride_w", "dil_h", "dil_w",
        "pad_top", "pad_left", "pad_bottom", "pad_right", "group")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.oracle_threads.restype = C.c_int
        _lib.oracle_f32_to_f16.restype = C.c_uint16
        _lib.oracle_f32_to_f16.argtypes = [C.c_float]
        _lib.oracle_f16_to_f32.restype = C.c_float
        _lib.oracle_f16_to_f32.argtypes = [C.c_uint16]
        _lib.oracle_conv_out_dim.restype = C.c_int64
        _lib.oracle_conv_out_dim.argtypes = [C.c_int64] * 6
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


def threads() -> int:
    return lib().oracle_threads()


def set_threads(n: int) -> None:
    lib().oracle_set_threads(C.c_int(n))


def matmul_nbits(A, B, scales, zp, K, N, block_size):
    """A [M,K] float32 or float16; returns Y [M,N] in A's dtype."""
    A = np.ascontiguousarray(A)
    M = A.size // K if K else 0
    B = _c(B, np.uint8)
    zp = _c(zp, np.uint8)
    i64 = C.c_int64
    if A.dtype == np.float16:
        s = _c(scales, np.float16)
        Y = np.empty((M, N), np.float16)
        lib().oracle_matmul_nbits_f16(_p(A.view(np.uint16)), _p(B), _p(s.view(np.uint16)), _p(zp),
                                      _p(Y.view(np.uint16)), i64(M), i64(K), i64(N), i64(block_size))
    else:
        A = _c(A, np.float32)
        s = _c(scales, np.float32)
        Y = np.empty((M, N), np.float32)
        lib().oracle_matmul_nbits_f32(_p(A), _p(B), _p(s), _p(zp), _p(Y), i64(M), i64(K), i64(N),
                                      i64(block_size))
    return Y


def dynamic_quantize_linear(x):
    x = _c(x, np.float32)
    y = np.empty(x.shape, np.uint8)
    scale = C.c_float()
    zp = C.c_uint8()
    lib().oracle_dynamic_quantize_linear(_p(x), C.c_int64(x.size), _p(y), C.byref(scale), C.byref(zp))
    return y, np.float32(scale.value), int(zp.value)


def erf_approx(x):
    """The reference's erf (shaders/elementwise.rs:71-80: Abramowitz-Stegun 7.1.26), every step in float32."""
    f = np.float32
    x = np.asarray(x, f)
    a = np.abs(x)
    with np.errstate(over="ignore", invalid="ignore"):   # a * a overflows to inf for huge |x|: exp(-inf) = 0, erf = +-1
        t = (f(1.0) / (f(1.0) + f(0.3275911) * a)).astype(f)
        poly = t * (f(0.254829592) + t * (f(-0.284496736) + t * (f(1.421413741) + t * (f(-1.453152027) + t * f(1.061405429)))))
        return (np.sign(x).astype(f) * (f(1.0) - poly.astype(f) * np.exp(-a * a).astype(f))).astype(f)


def decomposed_gelu(x, divisor=np.float32(np.sqrt(2.0)), offset=1.0, factor=0.5, factor_first=False):
    """Div -> Erf -> Add -> Mul -> Mul, each rounding to float32 (shaders/elementwise.rs:82-118):
    (x * (erf(x / divisor) + offset)) * factor, or x * ((erf + offset) * factor) with factor_first."""
    f = np.float32
    x = np.asarray(x, f)
    e = (erf_approx((x / f(divisor)).astype(f)) + f(offset)).astype(f)
    with np.errstate(over="ignore", invalid="ignore"):
        if factor_first:
            return (x * (e * f(factor)).astype(f)).astype(f)
        return ((x * e).astype(f) * f(factor)).astype(f)


def _signed(a):
    return 1 if a.dtype == np.int8 else 0


def matmul_integer(A, B, a_zp=0, b_zp=0):
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    assert A.dtype in (np.uint8, np.int8) and B.dtype in (np.uint8, np.int8)
    K, N = B.shape
    M = A.size // K if K else 0
    Y = np.empty((M, N), np.int32)
    lib().oracle_matmul_integer(_p(A), _signed(A), _p(B), _signed(B), C.c_int32(int(a_zp)),
                                C.c_int32(int(b_zp)), _p(Y), C.c_int64(M), C.c_int64(K), C.c_int64(N))
    return Y


def rescale(acc, scale, bias=None, product=None, relu=False):
    acc = _c(acc, np.int32)
    M, N = acc.shape
    scale = _c(np.atleast_1d(scale), np.float32)
    bias = None if bias is None else _c(np.atleast_1d(bias), np.float32)
    product = None if product is None else _c(np.atleast_1d(product), np.float32)
    step = lambda a: 0 if a is None or a.size == 1 else 1
    out = np.empty((M, N), np.float32)
    lib().oracle_rescale(_p(acc), _p(scale), step(scale), _p(product), step(product), _p(bias),
                         step(bias), int(bool(relu)), _p(out), C.c_int64(M), C.c_int64(N))
    return out


def requantize_ratio(x_scale, w_scale, y_scale):
    w = _c(np.atleast_1d(w_scale), np.float32)
    r = np.empty(w.shape, np.float32)
    lib().oracle_requantize_ratio(C.c_float(x_scale), _p(w), C.c_int64(w.size), C.c_float(y_scale), _p(r))
    return r


def requantize(acc, bias, ratio, inner, y_zp, out_signed):
    acc = _c(acc, np.int32)
    ratio = _c(np.atleast_1d(ratio), np.float32)
    bias = None if bias is None else _c(bias, np.int32)
    out = np.empty(acc.shape, np.int8 if out_signed else np.uint8)
    lib().oracle_requantize(_p(acc), _p(bias), _p(ratio), C.c_int64(acc.size), C.c_int64(inner),
                            C.c_int64(ratio.size), C.c_int32(int(y_zp)), int(bool(out_signed)), _p(out))
    return out


def conv_geom(x_shape, w_shape, strides=(1, 1), dilations=(1, 1), pads=(0, 0, 0, 0), group=1):
    """pads = (top, left, bottom, right), the ONNX order for 2-D."""
    n, c_in, h, w = x_shape
    c_out, _, kh, kw = w_shape
    return ConvGeom(n, c_in, h, w, c_out, kh, kw, strides[0], strides[1], dilations[0], dilations[1],
                    pads[0], pads[1], pads[2], pads[3], group)


def conv_out_shape(g: ConvGeom):
    ho = lib().oracle_conv_out_dim(g.h, g.pad_top, g.pad_bottom, g.kh, g.stride_h, g.dil_h)
    wo = lib().oracle_conv_out_dim(g.w, g.pad_left, g.pad_right, g.kw, g.stride_w, g.dil_w)
    return (g.n, g.c_out, ho, wo)


def same_pads(size, kernel, stride, dilation, upper=True):
    b, e = C.c_int64(), C.c_int64()
    lib().oracle_same_pads(C.c_int64(size), C.c_int64(kernel), C.c_int64(stride), C.c_int64(dilation),
                           int(upper), C.byref(b), C.byref(e))
    return b.value, e.value


def conv_integer(X, W, x_zp, w_zp, g: ConvGeom):
    X = np.ascontiguousarray(X)
    W = np.ascontiguousarray(W)
    Y = np.empty(conv_out_shape(g), np.int32)
    lib().oracle_conv_integer(_p(X), _signed(X), _p(W), _signed(W), C.c_int32(int(x_zp)),
                              C.c_int32(int(w_zp)), C.byref(g), _p(Y))
    return Y


def qlinear_conv(X, x_scale, x_zp, W, w_scale, w_zp, y_scale, y_zp, bias, g: ConvGeom, y_signed=False):
    X = np.ascontiguousarray(X)
    W = np.ascontiguousarray(W)
    ws = _c(np.atleast_1d(w_scale), np.float32)
    bias = None if bias is None else _c(bias, np.int32)
    Y = np.empty(conv_out_shape(g), np.int8 if y_signed else np.uint8)
    lib().oracle_qlinear_conv(_p(X), _signed(X), C.c_float(x_scale), C.c_int32(int(x_zp)), _p(W),
                              _signed(W), _p(ws), C.c_int64(ws.size), C.c_int32(int(w_zp)),
                              C.c_float(y_scale), C.c_int32(int(y_zp)), int(bool(y_signed)), _p(bias),
                              C.byref(g), _p(Y))
    return Y


def qlinear_matmul(A, a_scale, a_zp, B, b_scale, b_zp, y_scale, y_zp, y_signed=False):
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    K, N = B.shape
    M = A.size // K
    bs = _c(np.atleast_1d(b_scale), np.float32)
    Y = np.empty((M, N), np.int8 if y_signed else np.uint8)
    lib().oracle_qlinear_matmul(_p(A), _signed(A), C.c_float(a_scale), C.c_int32(int(a_zp)), _p(B),
                                _signed(B), _p(bs), C.c_int64(bs.size), C.c_int32(int(b_zp)),
                                C.c_float(y_scale), C.c_int32(int(y_zp)), int(bool(y_signed)), _p(Y),
                                C.c_int64(M), C.c_int64(K), C.c_int64(N))
    return Y
