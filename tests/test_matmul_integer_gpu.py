"""MatMulInteger, its fused dequantising epilogue and QLinearMatMul on the GPU: integers exact,
floats bit for bit (the epilogue rounds twice, like the unfused Cast, Mul, Add)."""
import json
import os

import numpy as np
import pytest

import refcases as rc

pytestmark = pytest.mark.gpu


def test_reference_variants_cases(ctx, pkg, oracle):
    """crates/onnx-vulkan-core/tests/matmul_integer_variants.rs:113-137, 174-196, 255-282."""
    a = rc.pseudo_plus1(7 * 12, 11).reshape(7, 12)
    b = rc.pseudo_plus1(12 * 5, 29).reshape(12, 5)
    assert np.array_equal(pkg.ops.matmul_integer(ctx, a, b, 37, 211), rc.matmul_integer_bigint(a, b, 37, 211))
    for (m, k, n) in [(20, 64, 18), (150, 96, 90)]:
        a = rc.pseudo_plus1(m * k, 3).reshape(m, k)
        b = rc.pseudo_plus1(k * n, 41).reshape(k, n)
        assert np.array_equal(pkg.ops.matmul_integer(ctx, a, b, 37, 211), oracle.matmul_integer(a, b, 37, 211))
        bi = b.view(np.int8)
        assert np.array_equal(pkg.ops.matmul_integer(ctx, a, bi, 37, -73), oracle.matmul_integer(a, bi, 37, -73))


def test_as_a_node_with_leading_dimensions(ctx, pkg, oracle):
    a = rc.pseudo_plus1(2 * 50 * 64, 1).reshape(2, 50, 64)
    w = rc.pseudo_plus1(64 * 200, 2).view(np.int8).reshape(64, 200)
    node = pkg.graph.NodeIr("MatMulInteger", ["a", "w", "a_zp", "w_zp"], ["acc"])
    env = {"a": a, "w": w, "a_zp": np.array(131, np.uint8), "w_zp": np.array(-7, np.int8)}
    pkg.graph.execute(ctx, [node], env)
    assert env["acc"].shape == (2, 50, 200) and env["acc"].dtype == np.int32
    assert np.array_equal(env["acc"].reshape(100, 200), oracle.matmul_integer(a.reshape(100, 64), w, 131, -7))
    with pytest.raises(ValueError):
        pkg.graph.execute(ctx, [node], dict(env, w=w[:60]))


@pytest.mark.parametrize("a_dt,b_dt", [(np.uint8, np.int8), (np.uint8, np.uint8), (np.int8, np.int8), (np.int8, np.uint8)])
@pytest.mark.parametrize("shape", [(1, 4, 1), (3, 2, 5), (33, 49, 130), (130, 100, 257), (7, 1000, 3), (256, 128, 128)],
                         ids=lambda s: "M%d_K%d_N%d" % s)
def test_any_k_any_sign(ctx, pkg, oracle, shape, a_dt, b_dt):
    """K not a multiple of 4 or 16, tiles with ragged edges, all four sign combinations
    (tests/matmul_integer_any_k.rs:141-150)."""
    m, k, n = shape
    a = rc.pseudo_plus1(m * k, 5).view(a_dt).reshape(m, k)
    b = rc.pseudo_plus1(k * n, 6).view(b_dt).reshape(k, n)
    za = -9 if a_dt == np.int8 else 200
    zb = 17 if b_dt == np.int8 else 3
    want = oracle.matmul_integer(a, b, za, zb)
    assert np.array_equal(pkg.ops.matmul_integer(ctx, a, b, za, zb), want)
    assert np.array_equal(pkg.ops.matmul_integer(ctx, a, b, za, zb, raw=True), want)
    assert np.array_equal(pkg.ops.matmul_integer(ctx, a, b, None, None), oracle.matmul_integer(a, b, 0, 0))


@pytest.mark.parametrize("shape", [(1000, 1024, 4096), (1000, 4096, 1024)], ids=lambda s: "M%d_K%d_N%d" % s)
def test_ffn_pair_shapes(ctx, pkg, oracle, shape):
    """The dynamic int8 FFN pair: DynamicQuantizeLinear output times symmetric int8 weights."""
    m, k, n = shape
    x = pkg.synth.normal_f32(m * k, 21).reshape(m, k)
    a, a_scale, a_zp = pkg.ops.dynamic_quantize_linear(ctx, x)
    w = pkg.synth.int8_weight(k, n, 22)
    want = oracle.matmul_integer(a, w, a_zp, 0)
    weight = pkg.ops.Int8Weight(ctx, w)
    got = pkg.ops.matmul_integer(ctx, a, w, a_zp, 0, weight=weight)
    assert np.array_equal(got, want)
    # "then fp32 rescale": scale = a_scale * w_scale formed by the fused node, bias per column
    w_scale = np.float32(0.01)
    bias = pkg.synth.uniform_f32(n, 23, -0.5, 0.5)
    got = pkg.ops.matmul_integer_scale_bias(ctx, a, w, a_zp, 0, a_scale, bias, product=w_scale, weight=weight)
    ref = oracle.rescale(want, a_scale, bias, product=w_scale)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    weight.destroy()


@pytest.mark.parametrize("a_dt,b_dt", [(np.uint8, np.int8), (np.int8, np.uint8)])
def test_large_products_take_the_256x256_tiles(ctx, pkg, oracle, a_dt, b_dt):
    """Enough 256x256 tiles to fill the chip switches to the large tile of the kernel that keeps B out of
    LDS: ragged edges in both directions, an odd number of k stages, both zero points non-zero, then the
    same product through the float epilogue."""
    m, k, n = 3601, 384, 3585
    a = rc.pseudo_plus1(m * k, 31).view(a_dt).reshape(m, k)
    b = rc.pseudo_plus1(k * n, 32).view(b_dt).reshape(k, n)
    za = -9 if a_dt == np.int8 else 200
    zb = 17 if b_dt == np.int8 else 3
    want = oracle.matmul_integer(a, b, za, zb)
    weight = pkg.ops.Int8Weight(ctx, b)
    assert np.array_equal(pkg.ops.matmul_integer(ctx, a, b, za, zb, weight=weight), want)
    scale = np.float32(0.003)
    bias = pkg.synth.uniform_f32(n, 33, -0.5, 0.5)
    got = pkg.ops.matmul_integer_scale_bias(ctx, a, b, za, zb, scale, bias, weight=weight)
    assert np.array_equal(got.view(np.uint32), oracle.rescale(want, scale, bias).view(np.uint32))
    weight.destroy()


@pytest.mark.parametrize("a_dt,b_dt", [(np.uint8, np.int8), (np.uint8, np.uint8), (np.int8, np.int8), (np.int8, np.uint8)])
@pytest.mark.parametrize("shape", [(130, 640, 257), (70, 1536, 64), (1, 512, 1), (333, 4096, 200)], ids=lambda s: "M%d_K%d_N%d" % s)
def test_few_tiles_and_long_k_take_the_k_split_kernel(ctx, pkg, oracle, shape, a_dt, b_dt):
    """Up to two 64x64 tiles per CU with k a multiple of 128 and at least 512: the workgroup's
    wavefronts split k, A alone passes through LDS, B comes fragment by fragment from the
    fragment-major prepacked weight. Stage counts that are not a multiple of the four in flight
    (5, 12, 4, 32), ragged edges, zero points on both sides or none, and the float epilogue."""
    m, k, n = shape
    a = rc.pseudo_plus1(m * k, 51).view(a_dt).reshape(m, k)
    b = rc.pseudo_plus1(k * n, 52).view(b_dt).reshape(k, n)
    za = -9 if a_dt == np.int8 else 200
    zb = 17 if b_dt == np.int8 else 3
    want = oracle.matmul_integer(a, b, za, zb)
    weight = pkg.ops.Int8Weight(ctx, b)
    assert np.array_equal(pkg.ops.matmul_integer(ctx, a, b, za, zb, weight=weight), want)
    assert np.array_equal(pkg.ops.matmul_integer(ctx, a, b, None, None, weight=weight), oracle.matmul_integer(a, b, 0, 0))
    scale = np.float32(0.002)
    bias = pkg.synth.uniform_f32(n, 53, -0.5, 0.5)
    got = pkg.ops.matmul_integer_scale_bias(ctx, a, b, za, zb, scale, bias, weight=weight)
    assert np.array_equal(got.view(np.uint32), oracle.rescale(want, scale, bias).view(np.uint32))
    weight.destroy()


LAYERS = [  # tests/matmul_integer_epilogue.rs:352-420: (a_shape, N, weight int8?, relu, per-column scale)
    ((2, 50, 64), 200, False, False, False), ((700, 96), 330, True, False, False),
    ((1100, 64), 1040, False, True, False), ((1, 128, 32), 48, True, False, True),
    ((5, 70), 9, True, True, True),      # K % 4 != 0, fewer than 16 rows and columns
]


@pytest.mark.parametrize("layer", LAYERS, ids=lambda l: "x".join(map(str, l[0])) + "_N%d" % l[1])
def test_fused_epilogue_equals_cast_mul_add_bit_for_bit(ctx, pkg, oracle, layer):
    a_shape, n, w_signed, relu, per_col = layer
    k = a_shape[-1]
    m = int(np.prod(a_shape[:-1]))
    a = rc.pseudo_plus1(m * k, 1).reshape(m, k)
    w = rc.pseudo_plus1(k * n, 2).view(np.int8 if w_signed else np.uint8).reshape(k, n)
    a_zp, w_zp = 131, (-7 if w_signed else 121)
    a_scale = np.float32(0.0123)
    w_scale = pkg.synth.uniform_f32(n, 4, 1e-3, 5e-3) if per_col else np.float32(3.1e-3)
    bias = pkg.synth.uniform_f32(n, 3, -0.5, 0.5)
    acc = oracle.matmul_integer(a, w, a_zp, w_zp)
    ref = oracle.rescale(acc, a_scale, bias, product=w_scale, relu=relu)
    got, folded = pkg.ops.matmul_integer_scale_bias(ctx, a, w, a_zp, w_zp, a_scale, bias, product=w_scale, relu=relu,
                                                    fold_range=True)
    differing = int(np.count_nonzero(got.view(np.uint32) != ref.view(np.uint32)))
    assert differing == 0, f"{differing} of {got.size} elements differ"
    if relu:
        assert np.count_nonzero(got == 0) > got.size // 8
    # the folded range is the one a min/max pass over the result finds
    assert folded[0] == np.float32(-min(ref.min(), 0)).view(np.uint32) & 0x7FFFFFFF
    assert folded[1] == np.float32(max(ref.max(), 0)).view(np.uint32)
    # without a bias and with a scalar scale only
    got = pkg.ops.matmul_integer_scale_bias(ctx, a, w, a_zp, w_zp, a_scale)
    assert np.array_equal(got.view(np.uint32), oracle.rescale(acc, a_scale).view(np.uint32))


def test_a_folded_range_feeds_the_next_quantisation(ctx, pkg, oracle):
    """MatMulIntegerScaleBias(range) -> DynamicQuantizeLinear(range_ready) must give the bytes,
    scale and zero point of a DynamicQuantizeLinear with its own pass (matmul_integer_epilogue.rs:1-12)."""
    m, k, n = 300, 128, 260
    a = rc.pseudo_plus1(m * k, 9).reshape(m, k)
    w = rc.pseudo_plus1(k * n, 10).view(np.int8).reshape(k, n)
    weight = pkg.ops.Int8Weight(ctx, w)
    dA, dza = ctx.upload(a), ctx.upload(np.array([128], np.uint8))
    dS = ctx.upload(np.array([0.004], np.float32))
    dY, dR, dQ, dP = ctx.alloc(m * n * 4), ctx.alloc(8), ctx.alloc(m * n), ctx.alloc(8)
    ctx.fill(dR, 0, 8, 0)
    pkg.ops.matmul_integer_scale_bias_device(ctx, dA, pkg.U8, weight, dza, None, dS, 0, None, 0, None, 0, False, dR, dY, m)
    pkg.ops.dynamic_quantize_linear_device(ctx, dY, m * n, dQ, dP, dP.at(4), range_slot=dR, range_ready=True)
    y = oracle.rescale(oracle.matmul_integer(a, w, 128, 0), np.float32(0.004))
    wq, ws, wz = oracle.dynamic_quantize_linear(y)
    assert np.array_equal(ctx.download(dQ, np.uint8, (m, n)), wq)
    assert ctx.download(dP, np.float32, (1,))[0].tobytes() == np.float32(ws).tobytes()
    assert ctx.download(dP, np.uint8, (1,), offset=4)[0] == wz
    weight.destroy()


def _golden():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "qlinear_golden.json")
    with open(path) as f:
        return [c for c in json.load(f) if c["op"] == "QLinearMatMul"]


@pytest.mark.parametrize("case", _golden(), ids=lambda c: c["name"])
def test_qlinear_matmul_golden_literals(ctx, pkg, case):
    node = pkg.graph.NodeIr("QLinearMatMul", ["a", "a_scale", "a_zp", "b", "b_scale", "b_zp", "y_scale", "y_zp"], ["out"])
    env = {"a": np.array(case["a"], np.uint8).reshape(case["a_shape"]), "a_scale": np.float32(case["a_scale"]),
           "a_zp": np.array(case["a_zp"], np.uint8), "b": np.array(case["b"], np.int8).reshape(case["b_shape"]),
           "b_scale": np.array(case["b_scale"], np.float32), "b_zp": np.array(case["b_zp"], np.int8),
           "y_scale": np.float32(case["y_scale"]), "y_zp": np.array(case["y_zp"], np.uint8)}
    pkg.graph.execute(ctx, [node], env)
    assert env["out"].reshape(-1).tolist() == case["want"]


@pytest.mark.parametrize("per_col", [False, True])
@pytest.mark.parametrize("y_signed", [False, True])
def test_qlinear_matmul_seeded(ctx, pkg, oracle, per_col, y_signed):
    m, k, n = 77, 200, 150
    a = rc.pseudo_plus1(m * k, 12).reshape(m, k)
    b = rc.pseudo_plus1(k * n, 13).view(np.int8).reshape(k, n)
    b_scale = pkg.synth.uniform_f32(n, 14, 0.001, 0.02) if per_col else np.float32(0.01)
    b_zp = 0 if per_col else 5
    y_zp = -3 if y_signed else 120
    got = pkg.ops.qlinear_matmul(ctx, a, 0.02, 128, b, b_scale, b_zp, 0.9, y_zp, y_signed)
    want = oracle.qlinear_matmul(a, 0.02, 128, b, b_scale, b_zp, 0.9, y_zp, y_signed)
    assert np.max(np.abs(got.astype(int) - want.astype(int))) <= 1     # the stated +-1 LSB ...
    assert np.array_equal(got, want)                                   # ... and in fact identical
    assert 0.2 < np.mean((got != got.max()) & (got != got.min())), "the case must not saturate everywhere"


def test_qlinear_matmul_refuses_asymmetric_per_column_weights(ctx, pkg):
    a = np.zeros((4, 16), np.uint8)
    b = np.zeros((16, 8), np.int8)
    with pytest.raises(pkg.HipComputeError) as e:
        pkg.ops.qlinear_matmul(ctx, a, 0.02, 128, b, np.full(8, 0.01, np.float32), 3, 0.05, 10)
    assert e.value.code == 2 and "per-channel zero point" in e.value.message
    with pytest.raises(pkg.HipComputeError) as e:
        pkg.ops.qlinear_matmul(ctx, a, 0.02, 128, b, np.full(5, 0.01, np.float32), 0, 0.05, 10)
    assert e.value.code == 1


def test_requantize_alone(ctx, pkg, oracle):
    acc = pkg.synth.uniform_ints(3 * 7 * 11, 15, -90000, 90000).astype(np.int32).reshape(3, 7, 11)
    ratio = pkg.synth.uniform_f32(7, 16, 0.0005, 0.003)
    bias = pkg.synth.uniform_ints(7, 17, -5000, 5000).astype(np.int32)
    for signed, zp in [(False, 100), (True, -20)]:
        got = pkg.ops.requantize(ctx, acc, bias, ratio, 11, zp, signed)
        assert np.array_equal(got, oracle.requantize(acc, bias, ratio, 11, zp, signed))
    got = pkg.ops.requantize(ctx, acc.reshape(-1)[:229], None, ratio[:1], 1, 7, False)   # ragged tail, scalar ratio
    assert np.array_equal(got, oracle.requantize(acc.reshape(-1)[:229], None, ratio[:1], 1, 7, False))


SIGNS = [(np.uint8, np.int8), (np.uint8, np.uint8), (np.int8, np.int8), (np.int8, np.uint8)]


def _mm_three_epilogues(ctx, pkg, oracle, m, k, n, a_dt, b_dt, seed):
    """int32, rescaled float and requantised byte outputs of one product against the oracle."""
    a = rc.pseudo_plus1(m * k, seed).view(a_dt).reshape(m, k)
    b = rc.pseudo_plus1(k * n, seed + 1).view(b_dt).reshape(k, n)
    za = -9 if a_dt == np.int8 else 200
    zb = 17 if b_dt == np.int8 else 3
    want = oracle.matmul_integer(a, b, za, zb)
    weight = pkg.ops.Int8Weight(ctx, b)
    assert np.array_equal(pkg.ops.matmul_integer(ctx, a, b, za, zb, weight=weight), want)
    scale = np.float32(0.003)
    bias = pkg.synth.uniform_f32(n, seed + 2, -0.5, 0.5)
    got = pkg.ops.matmul_integer_scale_bias(ctx, a, b, za, zb, scale, bias, relu=True, weight=weight)
    assert np.array_equal(got.view(np.uint32), oracle.rescale(want, scale, bias, relu=True).view(np.uint32))
    ys = float(0.02 * 0.01 * 74 * 73 * np.sqrt(k) / 100.0)
    got = pkg.ops.qlinear_matmul(ctx, a, 0.02, za, b, np.float32(0.01), zb, ys, 7, True, weight=weight)
    assert np.array_equal(got, oracle.qlinear_matmul(a, 0.02, za, b, np.float32(0.01), zb, ys, 7, True))
    weight.destroy()


@pytest.mark.parametrize("a_dt,b_dt", SIGNS)
@pytest.mark.parametrize("shape", [(2048, 384, 4096), (2017, 200, 4001), (3000, 256, 3000)], ids=lambda s: "M%d_K%d_N%d" % s)
def test_many_tiles_take_the_128x128_kernel(ctx, pkg, oracle, shape, a_dt, b_dt):
    """192 or more 128x128 tiles but fewer than 192 of 256x256: with whole 128-byte k stages the 128x128
    tile of the kernel that keeps B out of LDS (three stages, then an even count), with k = 200 and
    ragged rows and columns the LDS-staged 128x128 kernel in its unaligned form; every sign
    combination, both zero points non-zero, all three epilogues."""
    m, k, n = shape
    _mm_three_epilogues(ctx, pkg, oracle, m, k, n, a_dt, b_dt, seed=61)


ROUTES = [  # (options, M, K, N): every alternative route of the integer product once, forced in process
    ({"HIPC_GEMM_TILE": 128, "HIPC_GEMM_BIG": 0, "HIPC_GEMM_SMALL": 0}, 300, 640, 260),
    ({"HIPC_GEMM_TILE": 64, "HIPC_GEMM_BIG": 0, "HIPC_GEMM_SMALL": 0}, 1000, 1024, 520),
    ({"HIPC_GEMM_BIG": 1}, 700, 384, 520),                  # B out of LDS, 256x256 tiles: ragged, three stages
    ({"HIPC_GEMM_BIG": 2}, 333, 128, 390),                  # ... 128x128 tiles: ragged, a single stage
    ({"HIPC_GEMM_BIG": 2}, 1000, 1024, 4096),               # ... the first product of the dynamic int8 FFN
    ({"HIPC_GEMM_SMALL": 1, "HIPC_GEMM_BIG": 0}, 2100, 256, 1030),
    ({"HIPC_GEMM_SMALL": 0, "HIPC_GEMM_BIG": 0}, 1000, 1024, 1024),
]


@pytest.mark.parametrize("options,m,k,n", ROUTES, ids=lambda v: str(v).replace(" ", "") if isinstance(v, dict) else str(v))
def test_every_route_of_the_integer_product_can_be_forced(ctx, pkg, oracle, options, m, k, n):
    with ctx.options(**options):
        _mm_three_epilogues(ctx, pkg, oracle, m, k, n, np.uint8, np.int8, seed=71)
        _mm_three_epilogues(ctx, pkg, oracle, m, k, n, np.int8, np.uint8, seed=73)
