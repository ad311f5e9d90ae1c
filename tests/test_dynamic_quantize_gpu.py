"""DynamicQuantizeLinear on the GPU: bit-exact scale, exact zero point, zero differing codes --
the assertions of crates/onnx-vulkan-core/tests/dynamic_quantize.rs:63-75."""
import numpy as np
import pytest

import refcases as rc

pytestmark = pytest.mark.gpu


def check(ctx, pkg, oracle, x):
    node = pkg.graph.NodeIr("DynamicQuantizeLinear", ["x"], ["y", "y_scale", "y_zp"], name="dql")
    env = {"x": x}
    pkg.graph.execute(ctx, [node], env)
    wy, ws, wz = oracle.dynamic_quantize_linear(x)
    assert np.float32(env["y_scale"]).tobytes() == np.float32(ws).tobytes(), "scale"
    assert int(env["y_zp"]) == wz, "zero point"
    wrong = int(np.count_nonzero(env["y"] != wy))
    assert wrong == 0, f"{wrong} of {x.size} values quantized differently"
    assert env["y"].shape == x.shape


@pytest.mark.parametrize("r", [0.6, 1.0, 0.5, 2.0, 3.7])
def test_a_symmetric_range_rounds_the_zero_point_tie_to_even(ctx, pkg, oracle, r):
    check(ctx, pkg, oracle, rc.dql_symmetric(r))


def test_quantized_values_follow_the_correctly_rounded_quotient(ctx, pkg, oracle):
    check(ctx, pkg, oracle, rc.dql_xorshift())


def test_ffn_activation_shape(ctx, pkg, oracle):
    check(ctx, pkg, oracle, pkg.synth.normal_f32(1000 * 1024, 2).reshape(1000, 1024))
    check(ctx, pkg, oracle, pkg.synth.normal_f32(1000 * 4096, 3).reshape(1000, 4096) * np.float32(37.5))


@pytest.mark.parametrize("n", [1, 2, 3, 5, 255, 256, 257, 1023, 4099])
def test_ragged_lengths(ctx, pkg, oracle, n):
    check(ctx, pkg, oracle, pkg.synth.normal_f32(n, 40 + n))


def test_one_sided_constant_and_empty_inputs(ctx, pkg, oracle):
    check(ctx, pkg, oracle, np.abs(pkg.synth.normal_f32(3000, 4)) + np.float32(2))      # min stays 0
    check(ctx, pkg, oracle, -np.abs(pkg.synth.normal_f32(3000, 5)) - np.float32(2))     # max stays 0
    check(ctx, pkg, oracle, np.zeros(100, np.float32))                                  # scale becomes 1
    check(ctx, pkg, oracle, np.full(100, -0.0, np.float32))
    y, s, z = pkg.ops.dynamic_quantize_linear(ctx, np.zeros(0, np.float32))             # interp.rs:1949-1966
    assert y.size == 0 and s == 1.0 and z == 0


def test_unaligned_device_pointers(ctx, pkg, oracle):
    x = pkg.synth.normal_f32(1001, 6)
    dX = ctx.alloc(4 * 1002)
    dY = ctx.alloc(1008)
    dP = ctx.alloc(8)
    ctx.upload(x, dX, offset=4)                                  # 4-byte, not 16-byte aligned
    pkg.ops.dynamic_quantize_linear_device(ctx, dX.at(4), x.size, dY.at(1), dP, dP.at(4))
    y = ctx.download(dY, np.uint8, (1001,), offset=1)
    wy, ws, wz = oracle.dynamic_quantize_linear(x)
    assert np.array_equal(y, wy)
    assert ctx.download(dP, np.float32, (1,))[0].tobytes() == np.float32(ws).tobytes()
    assert ctx.download(dP, np.uint8, (1,), offset=4)[0] == wz


def test_a_range_folded_by_a_producer_skips_the_min_max_pass(ctx, pkg, oracle):
    x = pkg.synth.normal_f32(5000, 7)
    rng = np.array([np.float32(-x.min()).view(np.uint32), np.float32(x.max()).view(np.uint32)], np.uint32)
    dX, dR = ctx.upload(x), ctx.upload(rng)
    dY, dP = ctx.alloc(5000), ctx.alloc(8)
    pkg.ops.dynamic_quantize_linear_device(ctx, dX, x.size, dY, dP, dP.at(4), range_slot=dR, range_ready=True)
    wy, ws, wz = oracle.dynamic_quantize_linear(x)
    assert np.array_equal(ctx.download(dY, np.uint8, (5000,)), wy)
    assert ctx.download(dP, np.float32, (1,))[0].tobytes() == np.float32(ws).tobytes()
