"""ONNX initializers in front of the prepack calls: a model file's weights as the arrays the operators take.

The reading itself (storage forms of a TensorProto, weights kept in a file beside the model) is the
library's host code (``hipc_initializer_read``, ``hipc_model_initializers``; the reference's
``crates/onnx-vulkan-frontend/src/convert.rs:51-113, 247-384``); this module only carries bytes across
and checks the operand shapes of MatMulNBits (``crates/onnx-vulkan-core/src/interp.rs:6455-6472``).
Nothing here needs a GPU.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from .runtime import HipComputeError, InitializerInfo, load_library

# TensorProto.DataType -> numpy (the dtypes the quantized operators and their neighbours use)
NUMPY_OF = {1: np.float32, 2: np.uint8, 3: np.int8, 4: np.uint16, 5: np.int16, 6: np.int32, 7: np.int64, 9: np.bool_,
            10: np.float16, 11: np.float64, 12: np.uint32, 13: np.uint64}


def _check(lib, rc):
    if rc != 0:
        raise HipComputeError(rc, lib.hipc_host_error().decode())


def read_initializer(tensor: bytes, base_dir: str | None = None):
    """A serialized TensorProto -> ``(name, data_type, shape, payload bytes)`` (little-endian, row-major)."""
    lib = load_library()
    info = InitializerInfo()
    base = None if base_dir is None else str(base_dir).encode()
    _check(lib, lib.hipc_initializer_read(tensor, len(tensor), base, C.byref(info), None, 0))
    buf = C.create_string_buffer(max(info.bytes, 1))
    _check(lib, lib.hipc_initializer_read(tensor, len(tensor), base, C.byref(info), buf, info.bytes))
    return info.name.decode(), info.data_type, tuple(info.dims[i] for i in range(info.n_dims)), buf.raw[:info.bytes]


def as_array(data_type: int, shape, payload: bytes) -> np.ndarray:
    """The payload as a numpy array of the declared shape (bfloat16 and other dtypes numpy lacks: raised)."""
    if data_type not in NUMPY_OF:
        raise HipComputeError(2, f"dtype {data_type} has no numpy counterpart")
    a = np.frombuffer(payload, dtype=np.dtype(NUMPY_OF[data_type]).newbyteorder("<"))
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    if a.size != n:
        raise HipComputeError(1, f"{a.size} elements for shape {tuple(shape)}")
    return a.reshape(shape)


def model_initializers(model: bytes, base_dir: str | None = None) -> dict:
    """Every initializer of a serialized ModelProto: ``name -> (data_type, shape, payload bytes)``. An
    unnamed initializer is refused, as in the reference (convert.rs:66-69)."""
    lib = load_library()
    count = C.c_int64()
    _check(lib, lib.hipc_model_initializers(model, len(model), None, None, 0, C.byref(count)))
    n = count.value
    offsets, sizes = (C.c_size_t * max(n, 1))(), (C.c_size_t * max(n, 1))()
    _check(lib, lib.hipc_model_initializers(model, len(model), offsets, sizes, n, C.byref(count)))
    out = {}
    for i in range(n):
        name, dt, shape, payload = read_initializer(model[offsets[i]:offsets[i] + sizes[i]], base_dir)
        if not name:
            raise HipComputeError(1, "unnamed initializer")
        out[name] = (dt, shape, payload)
    return out


def matmul_nbits_operands(inits: dict, b: str, scales: str, zero_points: str | None, K: int, N: int, block_size: int):
    """The three constant inputs of a MatMulNBits node, taken from ``model_initializers`` by name and
    checked against K, N and block_size the way the operator does: B ``[N, n_blocks, block_size/2]`` u8,
    scales ``N * n_blocks`` f32 or f16, zero points ``N * ceil(n_blocks / 2)`` u8 (or absent).
    Returns ``(B, scales, zp)`` as the arrays ``ops.NBitsWeight`` takes."""
    nb = -(-K // block_size)
    short = HipComputeError(1, f"MatMulNBits: packed weight is short for K={K} N={N} block_size={block_size}")
    dt, _, payload = inits[b]
    if dt != 2:
        raise HipComputeError(1, f"MatMulNBits: expected u8 weight, got dtype {dt} for '{b}'")
    if len(payload) < N * nb * (block_size // 2):     # longer buffers are accepted, as in the reference (`>=`)
        raise short
    B = np.frombuffer(payload, np.uint8)[:N * nb * (block_size // 2)].reshape(N, nb, block_size // 2)
    dt, _, payload = inits[scales]
    if dt not in (1, 10):                              # the reference takes f32 only; f16 scales are this library's extension
        raise HipComputeError(2, f"MatMulNBits: scales '{scales}' of dtype {dt}")
    S = np.frombuffer(payload, dtype=np.dtype(NUMPY_OF[dt]).newbyteorder("<"))
    if S.size < N * nb:
        raise short
    S = S[:N * nb]
    Z = None
    if zero_points:
        dt, _, payload = inits[zero_points]
        if dt != 2:
            raise HipComputeError(2, f"MatMulNBits: zero points '{zero_points}' of dtype {dt} (unpacked zero points are refused)")
        if len(payload) < N * ((nb + 1) // 2):
            raise short
        Z = np.frombuffer(payload, np.uint8)[:N * ((nb + 1) // 2)].reshape(N, (nb + 1) // 2)
    return B, S, Z
