"""The reference's node-level view of the hot operators, over the C ABI.

``NodeIr`` and ``execute`` mirror crates/onnx-vulkan-core's ``NodeIr`` / ``interp::execute`` for
the operators on the quantized matrix-product path only, so a parity test can be written the
way the reference writes its own (one hand-built node, tensors by name). Attribute names,
input order and refusals follow the reference:

* input order of the QLinear operators: x, x_scale, x_zp, w, w_scale, w_zp, y_scale, y_zp[, B]
  (interp.rs:4796-4837);
* ``unsupported_quantization`` is the load-time refusal envelope of interp.rs:781-847;
* ``MatMulNBits`` refuses g_idx / bias inputs and bits != 4 (interp.rs:447-464).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np

from . import ops
from .runtime import Context, ConvGeom

HOT_OPS = ("MatMulNBits", "DynamicQuantizeLinear", "MatMulInteger", "MatMulIntegerScaleBias", "QLinearMatMul",
           "QLinearConv", "ConvInteger", "DecomposedGelu", "DecomposedGeluQuantize")


class Unsupported(Exception):
    """A form of an operator the path refuses (the reference's ``Error::Unsupported``)."""


@dataclass
class NodeIr:
    op: str
    inputs: List[str]
    outputs: List[str]
    attrs: Dict[str, object] = field(default_factory=dict)
    domain: str = ""
    name: str = ""


def _present(node: NodeIr, i: int) -> bool:
    return i < len(node.inputs) and node.inputs[i] != ""


def is_implemented_node(node: NodeIr) -> bool:
    if node.op not in HOT_OPS:
        return False
    if node.op == "MatMulNBits":
        # g_idx (input 4) and bias (input 5) are refused, bits must be 4 (interp.rs:447-464)
        if _present(node, 4) or _present(node, 5):
            return False
        if int(node.attrs.get("bits", 4)) != 4:
            return False
        # "block_size must be a multiple of 8 so a packed u32 never straddles two blocks"; K and N positive
        bs = int(node.attrs.get("block_size", 0))
        if bs <= 0 or bs % 8 != 0 or int(node.attrs.get("K", 0)) <= 0 or int(node.attrs.get("N", 0)) <= 0:
            return False
    return True


def unsupported_quantization(node: NodeIr, initializers: Dict[str, np.ndarray]) -> Optional[str]:
    """Why a QLinear node is refused, or None (interp.rs:781-847)."""
    def constant(i):
        return initializers.get(node.inputs[i]) if _present(node, i) else None

    def refuse(slot, why):
        return f"{node.op}: {slot} {why}"

    pairs = {"QLinearConv": [(1, 2, "x"), (6, 7, "y")], "QLinearMatMul": [(1, 2, "a"), (6, 7, "y")]}.get(node.op)
    if pairs is None:
        return None
    for scale_i, zero_i, slot in pairs:
        scale, zero = constant(scale_i), constant(zero_i)
        if scale is None or zero is None:
            return refuse(slot, "scale or zero point is not a constant")
        if scale.dtype != np.float32:
            return refuse(slot, "scale is not float32")
        if max(scale.size, 1) != 1 or max(zero.size, 1) != 1:
            return refuse(slot, "scale or zero point is not per-tensor")
    slot = "w" if node.op == "QLinearConv" else "b"
    scale, zero = constant(4), constant(5)
    if scale is None or zero is None:
        return refuse(slot, "scale or zero point is not a constant")
    if scale.dtype != np.float32:
        return refuse(slot, "scale is not float32")
    if max(scale.size, 1) != max(zero.size, 1):
        return refuse(slot, "scale and zero point have different lengths")
    if zero.size > 1 and np.any(zero.view(np.uint8) != 0):
        return refuse(slot, "per-channel zero point is not zero (asymmetric weights)")
    if node.op == "QLinearConv":
        bias = constant(8)
        if bias is not None and bias.dtype != np.int32:
            return refuse("B", "bias is not int32")
    return None


def conv_geometry(node: NodeIr, x_shape, w_shape) -> ConvGeom:
    """``conv_geometry`` (interp.rs:3439-3536): 1-D is lifted to 2-D with H = 1; auto_pad is resolved."""
    rank = len(x_shape) - 2
    if rank not in (1, 2):
        raise Unsupported(f"{node.op}: only 1-D and 2-D convolutions are supported")
    lift = (lambda v, fill: [fill] + list(v)) if rank == 1 else (lambda v, fill: list(v))
    xs = list(x_shape[:2]) + lift(x_shape[2:], 1)
    ws = list(w_shape[:2]) + lift(w_shape[2:], 1)
    strides = lift(node.attrs.get("strides", [1] * rank), 1)
    dil = lift(node.attrs.get("dilations", [1] * rank), 1)
    group = int(node.attrs.get("group", 1))
    auto_pad = node.attrs.get("auto_pad", "NOTSET")
    if auto_pad in ("SAME_UPPER", "SAME_LOWER"):
        import ctypes as C
        from .runtime import load_library
        lib = load_library()
        begins, ends = [], []
        for ax in range(2):
            b, e = C.c_int64(), C.c_int64()
            lib.hipc_same_pads(xs[2 + ax], ws[2 + ax], strides[ax], dil[ax], int(auto_pad == "SAME_UPPER"),
                               C.byref(b), C.byref(e))
            begins.append(b.value)
            ends.append(e.value)
        pads = begins + ends
    elif auto_pad == "VALID":
        pads = [0, 0, 0, 0]
    else:
        p = list(node.attrs.get("pads", [0] * (2 * rank)))
        pads = [0, p[0], 0, p[1]] if rank == 1 else p
    return ConvGeom.make(xs, ws, strides, dil, pads, group)


def _scalar(env, name, default=0):
    return default if name is None else int(np.asarray(env[name]).reshape(-1)[0])


def execute(ctx: Context, nodes: List[NodeIr], env: Dict[str, np.ndarray]) -> None:
    """Run hot-path nodes in order; tensors are numpy arrays in ``env`` by name."""
    for node in nodes:
        if not is_implemented_node(node):
            raise Unsupported(f"{node.domain}::{node.op} is not an operator of this path, or a refused form")
        why = unsupported_quantization(node, env)
        if why:
            raise Unsupported(why)
        inp = lambda i: env[node.inputs[i]] if _present(node, i) else None  # noqa: E731
        if node.op == "MatMulNBits":
            K, N, bs = int(node.attrs["K"]), int(node.attrs["N"]), int(node.attrs["block_size"])
            a = inp(0)
            y = ops.matmul_nbits(ctx, a, inp(1), inp(2), inp(3), K, N, bs, int(node.attrs.get("accuracy_level", 0)))
            env[node.outputs[0]] = y.reshape(a.shape[:-1] + (N,))
        elif node.op == "DynamicQuantizeLinear":
            y, s, z = ops.dynamic_quantize_linear(ctx, inp(0))
            env[node.outputs[0]], env[node.outputs[1]], env[node.outputs[2]] = y, np.float32(s), np.uint8(z)
        elif node.op in ("DecomposedGelu", "DecomposedGeluQuantize"):
            # the rewrite's nodes (rewrite.rs:660-735): inputs x and the graph's three scalar constants
            # (what it divides by, adds, multiplies by), attribute factor_first
            c = [float(np.asarray(env[name], np.float32).reshape(-1)[0]) for name in node.inputs[1:4]]
            k = dict(divisor=c[0], offset=c[1], factor=c[2], factor_first=bool(node.attrs.get("factor_first", 0)))
            if node.op == "DecomposedGelu":
                env[node.outputs[0]] = ops.decomposed_gelu(ctx, inp(0), **k)
            else:
                y, s, z = ops.dynamic_quantize_linear_gelu(ctx, inp(0), **k)
                env[node.outputs[0]], env[node.outputs[1]], env[node.outputs[2]] = y, np.float32(s), np.uint8(z)
        elif node.op == "MatMulInteger":
            a, b = inp(0), inp(1)
            if a.ndim < 2 or b.ndim != 2:
                raise ValueError(f"MatMulInteger: A rank {a.ndim} / B rank {b.ndim}")
            if a.shape[-1] != b.shape[0]:
                raise ValueError(f"MatMulInteger: K mismatch (A {a.shape[-1]}, B {b.shape[0]})")
            za = _scalar(env, node.inputs[2]) if _present(node, 2) else None
            zb = _scalar(env, node.inputs[3]) if _present(node, 3) else None
            env[node.outputs[0]] = ops.matmul_integer(ctx, a, b, za, zb)
        elif node.op == "MatMulIntegerScaleBias":
            # inputs: a, w, a_zp, w_zp, scale, bias[, product]  (rewrite.rs:475-519)
            a, b = inp(0), inp(1)
            y = ops.matmul_integer_scale_bias(ctx, a, b, _scalar(env, node.inputs[2]), _scalar(env, node.inputs[3]),
                                              inp(4), inp(5), inp(6), relu=bool(node.attrs.get("relu", 0)))
            env[node.outputs[0]] = y.reshape(a.shape[:-1] + (b.shape[1],))
        elif node.op == "QLinearMatMul":
            a, b = inp(0), inp(3)
            y_signed = np.asarray(inp(7)).dtype == np.int8
            y = ops.qlinear_matmul(ctx, a, float(np.asarray(inp(1)).reshape(-1)[0]), _scalar(env, node.inputs[2]), b,
                                   np.asarray(inp(4), np.float32).reshape(-1),
                                   int(np.asarray(inp(5)).reshape(-1)[0]), float(np.asarray(inp(6)).reshape(-1)[0]),
                                   _scalar(env, node.inputs[7]), y_signed)
            env[node.outputs[0]] = y.reshape(a.shape[:-1] + (b.shape[1],))
        elif node.op in ("QLinearConv", "ConvInteger"):
            x = inp(0)
            w = inp(3) if node.op == "QLinearConv" else inp(1)
            geom = conv_geometry(node, x.shape, w.shape)
            x4 = x.reshape(geom.n, geom.c_in, geom.h, geom.w)
            w4 = w.reshape(geom.c_out, geom.c_in // geom.group, geom.kh, geom.kw)
            if node.op == "ConvInteger":
                zx = _scalar(env, node.inputs[2]) if _present(node, 2) else None
                zw = _scalar(env, node.inputs[3]) if _present(node, 3) else None
                y = ops.conv_integer(ctx, x4, w4, zx, zw, geom)
            else:
                y_signed = np.asarray(inp(7)).dtype == np.int8
                y = ops.qlinear_conv(ctx, x4, float(np.asarray(inp(1)).reshape(-1)[0]), _scalar(env, node.inputs[2]),
                                     w4, np.asarray(inp(4), np.float32).reshape(-1),
                                     int(np.asarray(inp(5)).reshape(-1)[0]), float(np.asarray(inp(6)).reshape(-1)[0]),
                                     _scalar(env, node.inputs[7]), inp(8), geom, y_signed)
            if x.ndim == 3:
                y = y.reshape(y.shape[0], y.shape[1], y.shape[3])
            env[node.outputs[0]] = y
