"""Writes tests/golden/qlinear_golden.json: the literal operands of the reference's QLinear tests
(crates/onnx-vulkan-core/tests/qlinear.rs:106-275) with their expected outputs.

The expected outputs are evaluated here with Python integers for the accumulators and the
exact-rational requantisation of tests/refcases.py -- neither the oracle nor the library is
involved, so the fixture pins both. Run from the repository root:
    python tests/golden/make_qlinear_golden.py
"""
import json
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
from refcases import requantize_exact  # noqa: E402


def conv2x2(x, xw, w, c_out, x_zp, bias, x_scale, w_scales, y_scale, y_zp):
    """2x2 window, stride 1, no padding over a xw-wide square input, one input channel."""
    ho = xw - 1
    out = []
    for c in range(c_out):
        for oh in range(ho):
            for ow in range(ho):
                acc = bias[c] if bias else 0
                for r in range(2):
                    for s in range(2):
                        acc += (x[(oh + r) * xw + ow + s] - x_zp) * w[c * 4 + r * 2 + s]
                ws = w_scales[c] if len(w_scales) > 1 else w_scales[0]
                out.append(requantize_exact(acc, x_scale, ws, y_scale, y_zp, False))
    return out


cases = []
x = [130, 120, 140, 128, 200, 60, 10, 250, 128]
w = [1, -2, 3, 4, -5, 6, -7, 8]
cases.append(dict(
    name="a_convolution_accumulates_in_int32_and_requantizes_once", op="QLinearConv",
    x=x, x_shape=[1, 1, 3, 3], x_scale=0.02, x_zp=128, w=w, w_shape=[2, 1, 2, 2], w_scale=[0.01, 0.03],
    w_zp=[0, 0], y_scale=0.05, y_zp=10, bias=[7, -13],
    want=conv2x2(x, 3, w, 2, 128, [7, -13], 0.02, [0.01, 0.03], 0.05, 10)))
cases.append(dict(
    name="a_per_tensor_weight_scale_keeps_the_per_channel_bias", op="QLinearConv",
    x=x, x_shape=[1, 1, 3, 3], x_scale=0.02, x_zp=128, w=w, w_shape=[2, 1, 2, 2], w_scale=[0.01],
    w_zp=[0], y_scale=0.05, y_zp=10, bias=[7, -400],
    want=conv2x2(x, 3, w, 2, 128, [7, -400], 0.02, [0.01], 0.05, 10)))
x2, w2 = [200, 10, 50, 128], [2, -3, 4, 5]
cases.append(dict(
    name="a_convolution_without_bias_is_the_same_computation", op="QLinearConv",
    x=x2, x_shape=[1, 1, 2, 2], x_scale=0.03, x_zp=100, w=w2, w_shape=[1, 1, 2, 2], w_scale=[0.02],
    w_zp=[0], y_scale=0.1, y_zp=20, bias=None,
    want=conv2x2(x2, 2, w2, 1, 100, None, 0.03, [0.02], 0.1, 20)))
a, b = [130, 120, 140, 128], [1, -2, 3, 4, -5, 6, 7, -8]
want = []
for col in range(2):
    acc = sum((a[k] - 128) * b[k * 2 + col] for k in range(4))
    want.append(requantize_exact(acc, 0.02, [0.01, 0.03][col], 0.05, 10, False))
cases.append(dict(
    name="a_matmul_scales_per_column", op="QLinearMatMul",
    a=a, a_shape=[1, 4], a_scale=0.02, a_zp=128, b=b, b_shape=[4, 2], b_scale=[0.01, 0.03], b_zp=[0, 0],
    y_scale=0.05, y_zp=10, want=want))

path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "qlinear_golden.json")
with open(path, "w") as f:
    json.dump(cases, f, indent=1)
print("wrote", path, [c["want"] for c in cases])
