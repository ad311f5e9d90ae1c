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


# ---- DecomposedGelu and its fused quantizer (crates/onnx-vulkan-core/tests/decomposed_gelu.rs)

def _gelu_inputs():
    """Every 4096th float32 bit pattern -- both signs, subnormals, infinities -- without the NaNs,
    plus a dense sweep of the range where erf is neither 0 nor +-1 (decomposed_gelu.rs:134-141)."""
    bits = (np.arange(1 << 20, dtype=np.uint64) << 12).astype(np.uint32)
    x = bits.view(np.float32)
    x = x[~np.isnan(x)]
    dense = 1 << 19
    sweep = ((np.arange(dense, dtype=np.float32) / np.float32(dense) * np.float32(2.0) - np.float32(1.0)) * np.float32(8.0))
    return np.concatenate([x, sweep]).astype(np.float32)


@pytest.mark.parametrize("factor_first", [False, True])
def test_decomposed_gelu_follows_the_five_steps(ctx, pkg, oracle, factor_first):
    """Against the float32 restatement of Div, Erf, Add, Mul, Mul: the polynomial and every product
    round alike on both sides; exp is the one library call, so a few units in the last place of
    1 - poly * exp(-a^2) are allowed where that difference is not absorbed: |d| <= 1e-6 + 4e-6 |ref|."""
    x = _gelu_inputs()
    x = x[np.isfinite(x)]
    got = pkg.ops.decomposed_gelu(ctx, x, factor_first=factor_first)
    want = oracle.decomposed_gelu(x, factor_first=factor_first)
    with np.errstate(invalid="ignore", over="ignore"):
        ok = np.abs(got - want) <= 1e-6 + 4e-6 * np.abs(want)
    ok |= (got == want) | (np.isnan(got) & np.isnan(want))
    assert ok.all(), (x[~ok][:5], got[~ok][:5], want[~ok][:5])
    # the values a model meets: gelu(0) = 0, large x is the identity, large -x is -0
    probe = pkg.ops.decomposed_gelu(ctx, np.array([0.0, 9.0, -9.0, 1.0], np.float32), factor_first=factor_first)
    assert probe[0] == 0.0 and probe[1] == 9.0 and probe[2] == 0.0 and abs(probe[3] - 0.8413447) < 1e-6


@pytest.mark.parametrize("factor_first", [False, True])
def test_fused_gelu_quantization_equals_gelu_then_quantize_byte_for_byte(ctx, pkg, oracle, factor_first):
    """The reference's own check (decomposed_gelu.rs:202-245): the fused node against the kernels it
    replaces on the same device -- codes, scale and zero point identical -- and the device's GELU
    values through the CPU oracle's DynamicQuantizeLinear give the same bytes again."""
    x = (pkg.synth.normal_f32(300_003, 61) * np.float32(2.5)).astype(np.float32)   # ragged tail: not a multiple of 4
    y, scale, zp = pkg.ops.dynamic_quantize_linear_gelu(ctx, x, factor_first=factor_first)
    g = pkg.ops.decomposed_gelu(ctx, x, factor_first=factor_first)
    y2, scale2, zp2 = pkg.ops.dynamic_quantize_linear(ctx, g)
    assert np.float32(scale).tobytes() == np.float32(scale2).tobytes() and zp == zp2
    assert np.array_equal(y, y2)
    wy, ws, wz = oracle.dynamic_quantize_linear(g)
    assert np.float32(scale).tobytes() == np.float32(ws).tobytes() and zp == wz and np.array_equal(y, wy)


def test_gelu_nodes_as_the_rewrite_emits_them(ctx, pkg):
    """DecomposedGelu / DecomposedGeluQuantize carry x and the graph's three scalars as inputs and
    factor_first as an attribute (rewrite.rs:660-735)."""
    x = pkg.synth.normal_f32(1000, 62)
    env = {"x": x, "sqrt2": np.float32(np.sqrt(2.0)), "one": np.float32(1.0), "half": np.float32(0.5)}
    nodes = [pkg.graph.NodeIr("DecomposedGelu", ["x", "sqrt2", "one", "half"], ["y"], attrs={"factor_first": 1}),
             pkg.graph.NodeIr("DecomposedGeluQuantize", ["x", "sqrt2", "one", "half"], ["q", "scale", "zp"], attrs={"factor_first": 1})]
    pkg.graph.execute(ctx, nodes, env)
    assert np.array_equal(env["y"], pkg.ops.decomposed_gelu(ctx, x, factor_first=True))
    q, s, z = pkg.ops.dynamic_quantize_linear(ctx, env["y"])
    assert np.array_equal(env["q"], q) and np.float32(env["scale"]) == s and int(env["zp"]) == z


def test_fused_gelu_quantization_of_nothing_and_bad_constants(ctx, pkg):
    y, scale, zp = pkg.ops.dynamic_quantize_linear_gelu(ctx, np.zeros(0, np.float32))
    assert y.size == 0 and scale == 1.0 and zp == 0
    with pytest.raises(pkg.HipComputeError):
        pkg.ops.decomposed_gelu(ctx, np.ones(4, np.float32), divisor=0.0)
