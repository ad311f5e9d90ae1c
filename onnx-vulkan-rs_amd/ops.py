"""Operator entry points over the C ABI.

Two levels: ``*_device`` functions take device pointers / ``Buffer`` objects and only
enqueue (what a benchmark or a captured graph calls); the plain functions take and return
numpy arrays in the ONNX layouts (what the parity tests call) and flush before returning.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from .runtime import Buffer, Context, ConvGeom, F16, F32, I8, U8, _ptr, hipc_dtype

_vp = C.c_void_p


# ------------------------------------------------------------------ MatMulNBits

class NBitsWeight:
    """A prepacked MatMulNBits weight (``hipc_nbits_weight``)."""

    def __init__(self, ctx: Context, B, scales, zp, K: int, N: int, block_size: int):
        """B / scales / zp: numpy arrays in the ONNX layout (zp may be None)."""
        self.ctx, self.K, self.N, self.block_size = ctx, K, N, block_size
        B = np.ascontiguousarray(B, np.uint8)
        scales = np.ascontiguousarray(scales)
        dB, dS = ctx.upload(B), ctx.upload(scales)
        dZ = None if zp is None else ctx.upload(np.ascontiguousarray(zp, np.uint8))
        h = _vp()
        ctx._check(ctx.lib.hipc_prepack_matmul_nbits(
            ctx.handle, dB.ptr, B.size, dS.ptr, hipc_dtype(scales.dtype), scales.size,
            _ptr(dZ), 0 if zp is None else zp.size, K, N, block_size, C.byref(h)))
        ctx.flush()
        for b in (dB, dS, dZ):
            if b is not None:
                b.free()
        self.handle = h

    @property
    def nbytes(self) -> int:
        return self.ctx.lib.hipc_nbits_weight_bytes(self.handle)

    def destroy(self):
        if self.handle:
            self.ctx.lib.hipc_nbits_weight_destroy(self.ctx.handle, self.handle)
            self.handle = None


def matmul_nbits_device(ctx, A, a_dtype, B, b_len, scales, scale_dtype, scales_len, zp, zp_len, Y, M, K, N,
                        block_size, accuracy_level=0):
    ctx._check(ctx.lib.hipc_matmul_nbits(ctx.handle, _ptr(A), a_dtype, _ptr(B), b_len, _ptr(scales), scale_dtype,
                                         scales_len, _ptr(zp), zp_len, _ptr(Y), M, K, N, block_size, accuracy_level))


def matmul_nbits_packed_device(ctx, A, a_dtype, weight: NBitsWeight, Y, M, accuracy_level=0):
    ctx._check(ctx.lib.hipc_matmul_nbits_packed(ctx.handle, _ptr(A), a_dtype, weight.handle, _ptr(Y), M,
                                                accuracy_level))


def matmul_nbits(ctx: Context, A, B, scales, zp, K, N, block_size, accuracy_level=0, weight: NBitsWeight = None):
    """``MatMulNBits`` on numpy operands. With ``weight`` the prepacked path runs."""
    A = np.ascontiguousarray(A)
    M = A.size // K if K else 0
    dA = ctx.upload(A)
    dY = ctx.alloc(max(M * N * A.dtype.itemsize, 4))
    if weight is not None:
        matmul_nbits_packed_device(ctx, dA, hipc_dtype(A.dtype), weight, dY, M, accuracy_level)
        tmp = []
    else:
        B = np.ascontiguousarray(B, np.uint8)
        scales = np.ascontiguousarray(scales)
        dB, dS = ctx.upload(B), ctx.upload(scales)
        dZ = None if zp is None else ctx.upload(np.ascontiguousarray(zp, np.uint8))
        matmul_nbits_device(ctx, dA, hipc_dtype(A.dtype), dB, B.size, dS, hipc_dtype(scales.dtype), scales.size,
                            dZ, 0 if zp is None else zp.size, dY, M, K, N, block_size, accuracy_level)
        tmp = [dB, dS, dZ]
    Y = ctx.download(dY, A.dtype, (M, N))
    for b in [dA, dY] + tmp:
        if b is not None:
            b.free()
    return Y.reshape(A.shape[:-1] + (N,)) if A.ndim >= 1 else Y


# -------------------------------------------------------- DynamicQuantizeLinear

def dynamic_quantize_linear_device(ctx, X, n, Y, scale_out, zp_out, range_slot=None, range_ready=False):
    ctx._check(ctx.lib.hipc_dynamic_quantize_linear(ctx.handle, _ptr(X), n, _ptr(Y), _ptr(scale_out), _ptr(zp_out),
                                                    _ptr(range_slot), int(range_ready)))


def dynamic_quantize_linear(ctx: Context, x):
    """Returns (y uint8 like x, scale float32, zero_point int)."""
    x = np.ascontiguousarray(x, np.float32)
    dX = ctx.upload(x)
    dY = ctx.alloc(max(x.size, 4))
    dP = ctx.alloc(8)
    dynamic_quantize_linear_device(ctx, dX if x.size else None, x.size, dY if x.size else None, dP, dP.at(4))
    y = ctx.download(dY, np.uint8, x.shape)
    scale = ctx.download(dP, np.float32, (1,))[0]
    zp = int(ctx.download(dP, np.uint8, (1,), offset=4)[0])
    for b in (dX, dY, dP):
        b.free()
    return y, scale, zp


def dynamic_quantize_linear_static(ctx: Context, x):
    """The same through the entry point that allocates nothing (``hipc_dynamic_quantize_linear_static``)."""
    x = np.ascontiguousarray(x, np.float32)
    dX = ctx.upload(x)
    dY = ctx.alloc(max(x.size, 4))
    dP = ctx.alloc(8)
    ctx._check(ctx.lib.hipc_dynamic_quantize_linear_static(ctx.handle, dX.ptr if x.size else None, x.size,
                                                           dY.ptr if x.size else None, dP.ptr, dP.ptr + 4))
    y = ctx.download(dY, np.uint8, x.shape)
    scale = ctx.download(dP, np.float32, (1,))[0]
    zp = int(ctx.download(dP, np.uint8, (1,), offset=4)[0])
    for b in (dX, dY, dP):
        b.free()
    return y, scale, zp


SQRT2_F32 = float(np.float32(np.sqrt(2.0)))


def decomposed_gelu(ctx: Context, x, divisor=SQRT2_F32, offset=1.0, factor=0.5, factor_first=False):
    """The exact GELU as Div, Erf, Add, Mul, Mul in one kernel (``DecomposedGelu``)."""
    x = np.ascontiguousarray(x, np.float32)
    dX, dY = ctx.upload(x), ctx.alloc(max(x.nbytes, 4))
    ctx._check(ctx.lib.hipc_decomposed_gelu(ctx.handle, dX.ptr, x.size, divisor, offset, factor, int(factor_first), dY.ptr))
    y = ctx.download(dY, np.float32, x.shape)
    dX.free(), dY.free()
    return y


def dynamic_quantize_linear_gelu(ctx: Context, x, divisor=SQRT2_F32, offset=1.0, factor=0.5, factor_first=False):
    """DynamicQuantizeLinear(DecomposedGelu(x)) in two passes over x (``DecomposedGeluQuantize``)."""
    x = np.ascontiguousarray(x, np.float32)
    dX = ctx.upload(x)
    dY = ctx.alloc(max(x.size, 4))
    dP = ctx.alloc(8)
    ctx._check(ctx.lib.hipc_dynamic_quantize_linear_gelu(ctx.handle, dX.ptr if x.size else None, x.size, divisor, offset, factor,
                                                         int(factor_first), dY.ptr if x.size else None, dP.ptr, dP.ptr + 4, None))
    y = ctx.download(dY, np.uint8, x.shape)
    scale = ctx.download(dP, np.float32, (1,))[0]
    zp = int(ctx.download(dP, np.uint8, (1,), offset=4)[0])
    for b in (dX, dY, dP):
        b.free()
    return y, scale, zp


# ------------------------------------------------------------------ MatMulInteger

class Int8Weight:
    """A prepacked MatMulInteger / QLinearMatMul B (``hipc_int8_weight``)."""

    def __init__(self, ctx: Context, B):
        B = np.ascontiguousarray(B)
        assert B.dtype in (np.uint8, np.int8) and B.ndim == 2
        self.ctx, self.K, self.N, self.dtype = ctx, B.shape[0], B.shape[1], B.dtype
        dB = ctx.upload(B)
        h = _vp()
        ctx._check(ctx.lib.hipc_prepack_int8_b(ctx.handle, dB.ptr, hipc_dtype(B.dtype), self.K, self.N, C.byref(h)))
        ctx.flush()
        dB.free()
        self.handle = h

    def destroy(self):
        if self.handle:
            self.ctx.lib.hipc_int8_weight_destroy(self.ctx.handle, self.handle)
            self.handle = None


def matmul_integer_device(ctx, A, a_dtype, weight: Int8Weight, a_zp, b_zp, Y, M):
    ctx._check(ctx.lib.hipc_matmul_integer(ctx.handle, _ptr(A), a_dtype, weight.handle, _ptr(a_zp), _ptr(b_zp),
                                           _ptr(Y), M))


def matmul_integer_scale_bias_device(ctx, A, a_dtype, weight, a_zp, b_zp, scale, scale_step, product, product_step,
                                     bias, bias_step, relu, range_slot, Y, M):
    ctx._check(ctx.lib.hipc_matmul_integer_scale_bias(
        ctx.handle, _ptr(A), a_dtype, weight.handle, _ptr(a_zp), _ptr(b_zp), _ptr(scale), scale_step, _ptr(product),
        product_step, _ptr(bias), bias_step, int(bool(relu)), _ptr(range_slot), _ptr(Y), M))


def _zp_buffer(ctx, value, dtype):
    return None if value is None else ctx.upload(np.array([value]).astype(dtype))


def matmul_integer(ctx: Context, A, B, a_zp=None, b_zp=None, weight: Int8Weight = None, raw: bool = False):
    """``MatMulInteger`` -> int32 [.., M, N]. ``raw`` packs B inside the call."""
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    K, N = B.shape
    M = A.size // K if K else 0
    dA = ctx.upload(A)
    dY = ctx.alloc(max(M * N * 4, 4))
    dza, dzb = _zp_buffer(ctx, a_zp, A.dtype), _zp_buffer(ctx, b_zp, B.dtype)
    own = None
    tmp = [dA, dY, dza, dzb]
    if raw:
        dB = ctx.upload(B)
        tmp.append(dB)
        ctx._check(ctx.lib.hipc_matmul_integer_raw(ctx.handle, dA.ptr, hipc_dtype(A.dtype), dB.ptr, hipc_dtype(B.dtype),
                                                   _ptr(dza), _ptr(dzb), dY.ptr, M, K, N))
    else:
        if weight is None:
            weight = own = Int8Weight(ctx, B)
        matmul_integer_device(ctx, dA, hipc_dtype(A.dtype), weight, dza, dzb, dY, M)
    Y = ctx.download(dY, np.int32, (M, N))
    for b in tmp:
        if b is not None:
            b.free()
    if own:
        own.destroy()
    return Y.reshape(A.shape[:-1] + (N,))


def matmul_integer_scale_bias(ctx: Context, A, B, a_zp, b_zp, scale, bias=None, product=None, relu=False,
                              fold_range=False, weight: Int8Weight = None):
    """The fused dequantising linear layer; returns float32 [M, N] (and the folded range bits)."""
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    K, N = B.shape
    M = A.size // K
    own = None
    if weight is None:
        weight = own = Int8Weight(ctx, B)
    dA = ctx.upload(A)
    dY = ctx.alloc(max(M * N * 4, 4))
    dza, dzb = _zp_buffer(ctx, a_zp, A.dtype), _zp_buffer(ctx, b_zp, B.dtype)

    def vec(v):
        if v is None:
            return None, 0
        a = np.ascontiguousarray(np.atleast_1d(v), np.float32)
        return ctx.upload(a), (0 if a.size == 1 else 1)

    (ds, ss), (dp, ps), (db, bs) = vec(scale), vec(product), vec(bias)
    dr = None
    if fold_range:
        dr = ctx.alloc(8)
        ctx.fill(dr, 0, 8, 0)
    matmul_integer_scale_bias_device(ctx, dA, hipc_dtype(A.dtype), weight, dza, dzb, ds, ss, dp, ps, db, bs, relu, dr,
                                     dY, M)
    Y = ctx.download(dY, np.float32, (M, N))
    rng = ctx.download(dr, np.uint32, (2,)) if dr else None
    for b in (dA, dY, dza, dzb, ds, dp, db, dr):
        if b is not None:
            b.free()
    if own:
        own.destroy()
    return (Y, rng) if fold_range else Y


def requantize(ctx: Context, acc, bias, ratio, inner, y_zp, out_signed=False):
    acc = np.ascontiguousarray(acc, np.int32)
    ratio = np.ascontiguousarray(np.atleast_1d(ratio), np.float32)
    dA, dR = ctx.upload(acc), ctx.upload(ratio)
    dB = None if bias is None else ctx.upload(np.ascontiguousarray(bias, np.int32))
    dO = ctx.alloc(max(acc.size, 4))
    ctx._check(ctx.lib.hipc_requantize(ctx.handle, dA.ptr, _ptr(dB), dR.ptr, acc.size, inner, ratio.size, int(y_zp),
                                       I8 if out_signed else U8, dO.ptr))
    out = ctx.download(dO, np.int8 if out_signed else np.uint8, acc.shape)
    for b in (dA, dR, dB, dO):
        if b is not None:
            b.free()
    return out


def qlinear_matmul_device(ctx, A, a_dtype, a_scale, a_zp, weight: Int8Weight, b_scale, b_zp, y_scale, y_zp, y_dtype, Y, M):
    bs = np.ascontiguousarray(np.atleast_1d(b_scale), np.float32)
    ctx._check(ctx.lib.hipc_qlinear_matmul(
        ctx.handle, _ptr(A), a_dtype, float(a_scale), int(a_zp), weight.handle, bs.ctypes.data_as(C.POINTER(C.c_float)),
        bs.size, int(b_zp), float(y_scale), int(y_zp), y_dtype, _ptr(Y), M))


def qlinear_matmul(ctx: Context, A, a_scale, a_zp, B, b_scale, b_zp, y_scale, y_zp, y_signed=False,
                   weight: Int8Weight = None):
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    K, N = B.shape
    M = A.size // K
    own = None
    if weight is None:
        weight = own = Int8Weight(ctx, B)
    bs = np.ascontiguousarray(np.atleast_1d(b_scale), np.float32)
    dA = ctx.upload(A)
    dY = ctx.alloc(max(M * N, 4))
    ctx._check(ctx.lib.hipc_qlinear_matmul(
        ctx.handle, dA.ptr, hipc_dtype(A.dtype), float(a_scale), int(a_zp), weight.handle,
        bs.ctypes.data_as(C.POINTER(C.c_float)), bs.size, int(b_zp), float(y_scale), int(y_zp),
        I8 if y_signed else U8, dY.ptr, M))
    Y = ctx.download(dY, np.int8 if y_signed else np.uint8, (M, N))
    dA.free(), dY.free()
    if own:
        own.destroy()
    return Y


# ------------------------------------------------------ ConvInteger / QLinearConv

class ConvWeight:
    """A prepacked convolution weight (``hipc_conv_weight``)."""

    def __init__(self, ctx: Context, W, geom: ConvGeom):
        W = np.ascontiguousarray(W)
        assert W.dtype in (np.uint8, np.int8) and W.ndim == 4
        self.ctx, self.dtype = ctx, W.dtype
        dW = ctx.upload(W)
        h = _vp()
        ctx._check(ctx.lib.hipc_prepack_conv_w(ctx.handle, dW.ptr, hipc_dtype(W.dtype), C.byref(geom), C.byref(h)))
        ctx.flush()
        dW.free()
        self.handle = h

    def destroy(self):
        if self.handle:
            self.ctx.lib.hipc_conv_weight_destroy(self.ctx.handle, self.handle)
            self.handle = None


def conv_out_shape(ctx_or_lib, geom: ConvGeom):
    lib = ctx_or_lib.lib if isinstance(ctx_or_lib, Context) else ctx_or_lib
    ho, wo = C.c_int64(), C.c_int64()
    rc = lib.hipc_conv_out_shape(C.byref(geom), C.byref(ho), C.byref(wo))
    if rc != 0:
        raise ValueError("the kernel window does not fit the padded input")
    return (geom.n, geom.c_out, ho.value, wo.value)


def conv_integer(ctx: Context, X, W, x_zp, w_zp, geom: ConvGeom, weight: ConvWeight = None):
    X = np.ascontiguousarray(X)
    W = np.ascontiguousarray(W)
    own = None
    if weight is None:
        weight = own = ConvWeight(ctx, W, geom)
    shape = conv_out_shape(ctx, geom)
    dX = ctx.upload(X)
    dY = ctx.alloc(max(int(np.prod(shape)) * 4, 4))
    dzx, dzw = _zp_buffer(ctx, x_zp, X.dtype), _zp_buffer(ctx, w_zp, W.dtype)
    ctx._check(ctx.lib.hipc_conv_integer(ctx.handle, dX.ptr, hipc_dtype(X.dtype), weight.handle, _ptr(dzx), _ptr(dzw),
                                         C.byref(geom), dY.ptr))
    Y = ctx.download(dY, np.int32, shape)
    for b in (dX, dY, dzx, dzw):
        if b is not None:
            b.free()
    if own:
        own.destroy()
    return Y


def qlinear_conv_device(ctx, X, x_dtype, x_scale, x_zp, weight: ConvWeight, w_scale: np.ndarray, w_zp, y_scale, y_zp,
                        y_dtype, bias, geom: ConvGeom, Y):
    ws = np.ascontiguousarray(np.atleast_1d(w_scale), np.float32)
    ctx._check(ctx.lib.hipc_qlinear_conv(
        ctx.handle, _ptr(X), x_dtype, float(x_scale), int(x_zp), weight.handle,
        ws.ctypes.data_as(C.POINTER(C.c_float)), ws.size, int(w_zp), float(y_scale), int(y_zp), y_dtype, _ptr(bias),
        C.byref(geom), _ptr(Y)))


def qlinear_conv(ctx: Context, X, x_scale, x_zp, W, w_scale, w_zp, y_scale, y_zp, bias, geom: ConvGeom,
                 y_signed=False, weight: ConvWeight = None):
    X = np.ascontiguousarray(X)
    W = np.ascontiguousarray(W)
    own = None
    if weight is None:
        weight = own = ConvWeight(ctx, W, geom)
    shape = conv_out_shape(ctx, geom)
    dX = ctx.upload(X)
    dY = ctx.alloc(max(int(np.prod(shape)), 4))
    dB = None if bias is None else ctx.upload(np.ascontiguousarray(bias, np.int32))
    qlinear_conv_device(ctx, dX, hipc_dtype(X.dtype), x_scale, x_zp, weight, w_scale, w_zp, y_scale, y_zp,
                        I8 if y_signed else U8, dB, geom, dY)
    Y = ctx.download(dY, np.int8 if y_signed else np.uint8, shape)
    for b in (dX, dY, dB):
        if b is not None:
            b.free()
    if own:
        own.destroy()
    return Y
