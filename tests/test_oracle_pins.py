"""Pins of the CPU oracle (no GPU): every oracle function is checked against something that is
not its own formula -- known answers, the reference's closed-form test inputs evaluated by an
independent route, committed golden literals, or an invariant the mathematics fixes.
"""
import json
import os

import numpy as np
import pytest

import refcases as rc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ------------------------------------------------------------------ binary16

def test_f16_conversions_match_numpy(oracle):
    lib = oracle.lib()
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * np.float32(100.0),
        rng.standard_normal(2000).astype(np.float32) * np.float32(1e-6),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 6e-8, 2.98e-8, 2.99e-8, 6.1e-5, 1.0009765625,
                  1.00048828125, 1.00146484375, np.inf, -np.inf], np.float32)])
    for v in vals:
        got = lib.oracle_f32_to_f16(float(v))
        want = int(np.float32(v).astype(np.float16).view(np.uint16))
        assert got == want, (v, got, want)
    for h in list(range(0, 0x7C01, 37)) + [0x8000, 0x8001, 0xFBFF, 0x0001, 0x03FF, 0x0400]:
        got = np.float32(lib.oracle_f16_to_f32(h))
        want = np.array([h], np.uint16).view(np.float16).astype(np.float32)[0]
        assert got.tobytes() == want.tobytes(), hex(h)


# --------------------------------------------------------------- MatMulNBits

def _packed(pkg, nib, zp, bs):
    return pkg.synth.pack_nibbles(nib, bs), pkg.synth.pack_zero_points(zp)


def test_nbits_one_hot_weights_pin_the_nibble_and_block_order(oracle, pkg):
    """A single non-zero (q - zp) at (n, k) must give Y[n] = a[k] * scale(n, k/bs): a swapped
    nibble, a transposed block index or a wrong zero-point nibble moves or changes it."""
    K, N, bs = 100, 7, 16  # 7 blocks: odd, so zero-point rows are 4 bytes with a dangling nibble
    nb = -(-K // bs)
    rng = np.random.default_rng(3)
    a = rng.standard_normal((1, K)).astype(np.float32)
    for (n, k) in [(0, 0), (0, 1), (3, 16), (3, 17), (6, 99), (2, 31), (5, 64), (4, 95)]:
        zp = rng.integers(0, 16, (N, nb)).astype(np.uint8)
        nib = zp[:, np.arange(K) // bs].copy()          # every weight dequantises to exactly 0
        nib[n, k] = (nib[n, k] + 5) % 16                # ... except one: q - zp = +5 or -11
        scale = rng.uniform(0.5, 2.0, (N, nb)).astype(np.float32)
        B, Z = _packed(pkg, nib, zp, bs)
        y = oracle.matmul_nbits(a, B, scale.reshape(-1), Z, K, N, bs)
        want = np.zeros((1, N), np.float32)
        d = np.float32(int(nib[n, k]) - int(zp[n, k // bs]))
        want[0, n] = a[0, k] * (d * scale[n, k // bs])
        assert np.array_equal(y, want), (n, k)


def test_nbits_all_ones_is_the_row_sum(oracle, pkg):
    K, N, bs = 96, 5, 32
    a = (np.arange(K, dtype=np.float32) - 40).reshape(1, K)
    nib = np.full((N, K), 9, np.uint8)
    B = pkg.synth.pack_nibbles(nib, bs)
    scales = np.ones(N * 3, np.float32)
    y = oracle.matmul_nbits(a, B, scales, None, K, N, bs)   # zp omitted => 8 => every weight is 1
    assert np.array_equal(y, np.full((1, N), a.sum(), np.float32))


def test_nbits_missing_zero_points_mean_eight(oracle, pkg):
    a, nib, zp, scale = rc.matmul_nbits_case(3, 200, 19, 32)
    B = pkg.synth.pack_nibbles(nib, 32)
    eight = pkg.synth.pack_zero_points(np.full_like(zp, 8))
    y0 = oracle.matmul_nbits(a, B, scale.reshape(-1), None, 200, 19, 32)
    y8 = oracle.matmul_nbits(a, B, scale.reshape(-1), eight, 200, 19, 32)
    assert np.array_equal(y0, y8)


@pytest.mark.parametrize("case", rc.MATMUL_NBITS_CASES, ids=lambda c: "M%d_K%d_N%d_bs%d" % c)
def test_nbits_reference_cases_against_the_float64_product(oracle, pkg, case):
    m, k, n, bs = case
    a, nib, zp, scale = rc.matmul_nbits_case(m, k, n, bs)
    B, Z = _packed(pkg, nib, zp, bs)
    y = oracle.matmul_nbits(a, B, scale.reshape(-1), Z, k, n, bs)
    want = rc.matmul_nbits_f64(a, nib, zp, scale, bs)
    # the reference's own bound (tests/matmul_nbits.rs:159-163)
    assert np.all(np.abs(y - want) <= 1e-4 * np.maximum(np.abs(want), 1.0))


def test_nbits_padding_of_a_partial_block_is_ignored(oracle, pkg):
    """K = 100 with 32-wide blocks: the 28 padding nibbles of the last block must not count."""
    a, nib, zp, scale = rc.matmul_nbits_case(2, 100, 17, 32)
    B, Z = _packed(pkg, nib, zp, 32)
    y = oracle.matmul_nbits(a, B, scale.reshape(-1), Z, 100, 17, 32)
    B2 = B.copy()
    B2[:, 3, 2:] = 0xFF  # k = 100..127 live in bytes 2.. of block 3
    assert np.array_equal(y, oracle.matmul_nbits(a, B2, scale.reshape(-1), Z, 100, 17, 32))


def test_nbits_f16_is_the_f32_computation_rounded_once(oracle, pkg):
    a, nib, zp, scale = rc.matmul_nbits_case(4, 256, 24, 128)
    B, Z = _packed(pkg, nib, zp, 128)
    a16, s16 = a.astype(np.float16), scale.astype(np.float16)
    y16 = oracle.matmul_nbits(a16, B, s16.reshape(-1), Z, 256, 24, 128)
    y32 = oracle.matmul_nbits(a16.astype(np.float32), B, s16.astype(np.float32).reshape(-1), Z, 256, 24, 128)
    assert y16.dtype == np.float16 and np.array_equal(y16, y32.astype(np.float16))


# ----------------------------------------------------- DynamicQuantizeLinear

@pytest.mark.parametrize("r,want_zp", [(0.6, 128), (1.0, 127), (0.5, 127), (2.0, 127), (3.7, 127)])
def test_dql_symmetric_range_zero_point_sits_on_the_tie(oracle, r, want_zp):
    """-min/scale is 127.5 up to rounding (tests/dynamic_quantize.rs:1-7, 78-88): for r = 0.6 the
    correctly rounded quotient is exactly 127.5 and ties to the even 128, for the other ranges
    it is the float just below and gives 127 -- a quotient one ULP off flips either."""
    x = rc.dql_symmetric(r)
    y, scale, zp = oracle.dynamic_quantize_linear(x)
    want_scale = np.float32(np.float64(np.float32(x.max() - x.min())) / 255.0)
    assert np.float32(scale).tobytes() == want_scale.tobytes()
    # f64 quotient of two f32, cast once: the correctly rounded f32 quotient
    q = np.float32(np.float64(-x.min()) / np.float64(want_scale))
    assert zp == int(np.rint(q)) == want_zp
    assert y[0] == 0 and y[-1] == min(255, int(np.rint(q)) + want_zp) and np.all(np.diff(y.astype(int)) >= 0)


def test_dql_integer_ramp_is_the_identity(oracle):
    x = np.arange(256, dtype=np.float32)
    y, scale, zp = oracle.dynamic_quantize_linear(x)
    assert scale == 1.0 and zp == 0 and np.array_equal(y, np.arange(256, dtype=np.uint8))
    y, scale, zp = oracle.dynamic_quantize_linear(x - 100)
    assert scale == 1.0 and zp == 100 and np.array_equal(y, np.arange(256, dtype=np.uint8))


def test_dql_range_always_contains_zero_and_constants(oracle):
    y, scale, zp = oracle.dynamic_quantize_linear(np.full(9, 5.1, np.float32))
    assert zp == 0 and np.float32(scale).tobytes() == np.float32(np.float64(np.float32(5.1)) / 255).tobytes()
    assert np.all(y == 255)
    y, scale, zp = oracle.dynamic_quantize_linear(np.zeros(5, np.float32))
    assert scale == 1.0 and zp == 0 and np.all(y == 0)
    y, scale, zp = oracle.dynamic_quantize_linear(np.zeros(0, np.float32))   # interp.rs:1949-1966
    assert y.size == 0 and scale == 1.0 and zp == 0


def test_dql_division_agrees_with_the_reference_double_single_reciprocal(oracle):
    """The reference replaces d/255 by fma(d, hi, d*lo) with the constants of
    shaders/dynamic_quantize.rs:183 and proves it equal to the rounded quotient on xorshift values
    (:255-285). The oracle's plain division must land on the same floats."""
    hi, lo = np.float32(3.921568859e-3), np.float32(-2.319175824e-10)
    assert hi == np.float32(1.0 / 255.0) and lo == np.float32(1.0 / 255.0 - np.float64(hi))
    mask = (1 << 64) - 1
    s = 0x2545F4914F6CDD1D
    for _ in range(3000):
        s ^= (s << 13) & mask
        s ^= s >> 7
        s ^= (s << 17) & mask
        d = np.float32(np.float32(s >> 40) / np.float32(512.0))
        if d == 0:
            continue
        _, scale, _ = oracle.dynamic_quantize_linear(np.array([0.0, d], np.float32))
        # fma in exact arithmetic: d*hi + fl(d*lo), rounded once
        fma = np.float32(np.float64(d) * np.float64(hi) + np.float64(np.float32(d * lo)))
        assert np.float32(scale).tobytes() == fma.tobytes(), d


def test_dql_codes_follow_the_rounded_quotient(oracle):
    x = rc.dql_xorshift(1 << 14)
    y, scale, zp = oracle.dynamic_quantize_linear(x)
    q = np.float64(x) / np.float64(scale)          # f64 quotient of two f32: rounds like the exact one
    want = np.clip(np.rint(q.astype(np.float32)) + zp, 0, 255).astype(np.uint8)
    assert np.array_equal(y, want)


# ------------------------------------------------------------- MatMulInteger

def test_matmul_integer_reference_cases_against_big_integers(oracle):
    # tests/matmul_integer_variants.rs:113-137: M7 K12 N5, both zero points non-zero
    a = rc.pseudo_plus1(7 * 12, 11).reshape(7, 12)
    b = rc.pseudo_plus1(12 * 5, 29).reshape(12, 5)
    assert np.array_equal(oracle.matmul_integer(a, b, 37, 211), rc.matmul_integer_bigint(a, b, 37, 211))
    # :255-282: int8 B reinterpreted from the same bytes, negative zero point
    a = rc.pseudo_plus1(20 * 64, 3).reshape(20, 64)
    b = rc.pseudo_plus1(64 * 18, 41).view(np.int8).reshape(64, 18)
    assert np.array_equal(oracle.matmul_integer(a, b, 37, -73), rc.matmul_integer_bigint(a, b, 37, -73))
    # signed A as well
    a8 = a.view(np.int8)
    assert np.array_equal(oracle.matmul_integer(a8, b, -5, 9), rc.matmul_integer_bigint(a8, b, -5, 9))


def test_matmul_integer_extremes(oracle):
    """255 * 255 * K with zero points 0: a dropped sign or a narrow accumulator shows at once."""
    K = 300
    a = np.full((2, K), 255, np.uint8)
    b = np.full((K, 3), 255, np.uint8)
    assert np.all(oracle.matmul_integer(a, b, 0, 0) == 255 * 255 * K)
    bi = np.full((K, 3), -128, np.int8)
    assert np.all(oracle.matmul_integer(a, bi, 0, 127) == 255 * (-255) * K)


def test_rescale_rounds_twice(oracle):
    rng = np.random.default_rng(5)
    acc = rng.integers(-2 ** 22, 2 ** 22, (6, 40)).astype(np.int32)
    scale = rng.uniform(1e-4, 1e-2, 40).astype(np.float32)
    bias = rng.uniform(-1, 1, 40).astype(np.float32)
    got = oracle.rescale(acc, scale, bias)
    # acc < 2^24 is exact in f32; the product of two f32 is exact in f64; one cast rounds it
    prod = (acc.astype(np.float64) * scale.astype(np.float64)).astype(np.float32)
    want = (prod.astype(np.float64) + bias.astype(np.float64)).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    fused = (acc.astype(np.float64) * scale.astype(np.float64) + bias.astype(np.float64)).astype(np.float32)
    assert np.any(fused.view(np.uint32) != want.view(np.uint32)), "the case must tell an fma from two roundings"
    relu = oracle.rescale(acc, scale, bias, relu=True)
    assert np.array_equal(relu, np.maximum(want, 0)) and not np.signbit(relu).any()
    # the product of scales is formed first, with its own rounding
    p = np.float32(0.0123)
    got = oracle.rescale(acc, p, bias, product=scale)
    s2 = (np.float64(p) * scale.astype(np.float64)).astype(np.float32)
    want = ((acc.astype(np.float64) * s2.astype(np.float64)).astype(np.float32).astype(np.float64)
            + bias.astype(np.float64)).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


# ------------------------------------------- Requantize / QLinear literals

def test_requantize_against_exact_rationals(oracle):
    rng = np.random.default_rng(7)
    acc = rng.integers(-60000, 60000, 400).astype(np.int32)
    for (xs, ws, ys, zp, signed) in [(0.02, 0.01, 0.05, 10, False), (0.03, 0.02, 0.1, -3, True),
                                     (0.5, 0.5, 0.25, 128, False)]:   # the last lands on exact .5 ties
        ratio = oracle.requantize_ratio(xs, [ws], ys)
        got = oracle.requantize(acc, None, ratio, 1, zp, signed)
        want = [rc.requantize_exact(int(a), xs, ws, ys, zp, signed) for a in acc]
        assert np.array_equal(got.astype(int), np.array(want))


def test_requantize_channel_index_and_bias(oracle):
    # conv layout: c = (i / inner) % axis_len, bias added before the scaling
    acc = np.arange(2 * 3 * 4, dtype=np.int32).reshape(2, 3, 4) * 100
    ratio = np.array([0.01, 0.02, 0.04], np.float32)
    bias = np.array([1000, -500, 0], np.int32)
    got = oracle.requantize(acc, bias, ratio, 4, 3, False)
    for n in range(2):
        for c in range(3):
            for i in range(4):
                v = int(acc[n, c, i]) + int(bias[c])
                want = min(255, max(0, int(np.rint(np.float32(v) * ratio[c])) + 3))
                assert got[n, c, i] == want


def _golden():
    with open(os.path.join(GOLDEN, "qlinear_golden.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _golden(), ids=lambda c: c["name"])
def test_qlinear_golden_literals(oracle, case):
    if case["op"] == "QLinearConv":
        X = np.array(case["x"], np.uint8).reshape(case["x_shape"])
        W = np.array(case["w"], np.int8).reshape(case["w_shape"])
        g = oracle.conv_geom(X.shape, W.shape)
        bias = None if case["bias"] is None else np.array(case["bias"], np.int32)
        got = oracle.qlinear_conv(X, case["x_scale"], case["x_zp"], W, np.array(case["w_scale"], np.float32),
                                  case["w_zp"][0], case["y_scale"], case["y_zp"], bias, g)
    else:
        A = np.array(case["a"], np.uint8).reshape(case["a_shape"])
        B = np.array(case["b"], np.int8).reshape(case["b_shape"])
        got = oracle.qlinear_matmul(A, case["a_scale"], case["a_zp"], B, np.array(case["b_scale"], np.float32),
                                    case["b_zp"][0], case["y_scale"], case["y_zp"])
    assert got.reshape(-1).tolist() == case["want"]


# --------------------------------------------------------------- ConvInteger

@pytest.mark.parametrize("case", rc.CONV_CASES, ids=lambda c: "c%d_o%d_%dx%d_s%d_d%d" % (
    c["c_in"], c["c_out"], c["h"], c["w"], c["stride"], c["dilation"]))
def test_conv_integer_reference_cases_against_the_dense_route(oracle, case):
    X, W, x_zp, w_zp = rc.conv_case_operands(case)
    s, d = case["stride"], case["dilation"]
    g = oracle.conv_geom(X.shape, W.shape, (s, s), (d, d), case["pads"])
    got = oracle.conv_integer(X, W, x_zp, w_zp, g)
    want = rc.conv_integer_dense(X, W, x_zp, w_zp, (s, s), (d, d), case["pads"])
    assert got.shape == want.shape and np.array_equal(got, want)


def test_conv_integer_groups_and_1d(oracle):
    rng = np.random.default_rng(9)
    X = rng.integers(0, 256, (2, 8, 1, 50)).astype(np.uint8)
    W = rng.integers(-128, 128, (12, 2, 1, 7)).astype(np.int8)   # group 4
    g = oracle.conv_geom(X.shape, W.shape, (1, 2), (1, 3), (0, 9, 0, 9), group=4)
    got = oracle.conv_integer(X, W, 128, 0, g)
    want = rc.conv_integer_dense(X, W, 128, 0, (1, 2), (1, 3), (0, 9, 0, 9), group=4)
    assert np.array_equal(got, want)


def test_conv_geometry_known_answers(oracle):
    lib = oracle.lib()
    assert lib.oracle_conv_out_dim(4096, 3, 3, 7, 1, 1) == 4096
    assert lib.oracle_conv_out_dim(4096, 15, 15, 7, 1, 5) == 4096
    assert lib.oracle_conv_out_dim(224, 3, 3, 7, 2, 1) == 112       # resnet stem
    assert lib.oracle_conv_out_dim(5, 0, 0, 7, 1, 1) == 0
    assert oracle.same_pads(4096, 7, 1, 5) == (15, 15)
    assert oracle.same_pads(224, 7, 2, 1, upper=True) == (2, 3)      # odd total: the extra goes last
    assert oracle.same_pads(224, 7, 2, 1, upper=False) == (3, 2)
    assert oracle.same_pads(10, 1, 1, 1) == (0, 0)


# ------------------------------------------------------------- DecomposedGelu

def test_decomposed_gelu_is_the_exact_gelu_to_the_polynomial_s_error(oracle):
    """erf_approx is Abramowitz-Stegun 7.1.26 (|error| <= 1.5e-7); with divisor sqrt(2), offset 1 and
    factor 0.5 the five steps are x * Phi(x). Against math.erf in float64, both product orders; and
    the two orders differ from each other only by rounding."""
    import math
    x = np.linspace(-6.0, 6.0, 4001).astype(np.float32)
    erf64 = np.array([math.erf(float(v)) for v in x])
    assert np.max(np.abs(oracle.erf_approx(x).astype(np.float64) - erf64)) < 6e-7   # 1.5e-7 of the formula + float32 steps
    assert oracle.erf_approx(np.float32(0.0)) == 0.0 and oracle.erf_approx(np.float32(-7.0)) == -1.0
    want = x.astype(np.float64) * 0.5 * (1.0 + np.array([math.erf(float(v) / math.sqrt(2.0)) for v in x]))
    for ff in (False, True):
        got = oracle.decomposed_gelu(x, factor_first=ff).astype(np.float64)
        assert np.max(np.abs(got - want)) < 3e-6, ff
    a, b = oracle.decomposed_gelu(x), oracle.decomposed_gelu(x, factor_first=True)
    assert np.max(np.abs(a - b)) <= 5e-7
    # other constants: offset and factor enter as written (a plain erf: divisor 1, offset 0, factor 1 gives x * erf(x))
    assert np.allclose(oracle.decomposed_gelu(x, 1.0, 0.0, 1.0), x * oracle.erf_approx(x), rtol=0, atol=0)


# ------------------------------------------------------------- decoder glue

def test_decoder_glue_against_float64_closed_forms(oracle):
    from oracle import decoder as od
    rng = np.random.default_rng(11)
    x = rng.standard_normal(96).astype(np.float32) * 3
    w = rng.standard_normal(96).astype(np.float32)
    want = x.astype(np.float64) / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-6) * w
    assert np.allclose(od.rmsnorm(x, w, 1e-6), want, rtol=2e-6, atol=1e-6)
    assert np.allclose(od.rmsnorm(np.full(8, 2.0, np.float32), np.ones(8, np.float32), 0.0), 1.0)   # known answer
    # rotary: position 0 is the identity, a rotation keeps the norm of every (j, j + half) pair, and
    # rotating by p then by q (same frequencies) equals rotating by p + q
    v = rng.standard_normal(64).astype(np.float32)
    assert np.array_equal(od.rope_half(v, 0, 10000.0), v)
    r = od.rope_half(v, 7, 10000.0)
    assert np.allclose(r[:32] ** 2 + r[32:] ** 2, v[:32] ** 2 + v[32:] ** 2, rtol=1e-5)
    assert np.allclose(od.rope_half(r, 5, 10000.0), od.rope_half(v, 12, 10000.0), atol=2e-5)
    assert np.allclose(od.rope_half(np.concatenate([np.ones(1), np.zeros(1)]).astype(np.float32), 1, 10000.0),
                       [np.cos(1.0), np.sin(1.0)], atol=1e-6)                                       # pair (0, half)
    g = od.gelu_tanh(np.array([-3.0, -1.0, 0.0, 0.5, 2.0], np.float32))
    t = np.array([-3.0, -1.0, 0.0, 0.5, 2.0])
    assert np.allclose(g, 0.5 * t * (1 + np.tanh(np.sqrt(2 / np.pi) * (t + 0.044715 * t ** 3))), atol=1e-6)


def test_attention_window_is_the_reference_mask(oracle):
    """The oracle slices the visible keys; the reference writes -3.4028235e38 into the masked scores
    of the whole row (`t > pq`, and with a window `pq - t >= window`, shaders/attention.rs:249-254)
    and takes a softmax over all of it. Same result, in float64, for windows around every boundary."""
    from oracle import decoder as od
    rng = np.random.default_rng(5)
    hd, rows = 16, 40
    K = rng.standard_normal((rows, hd)).astype(np.float16)
    V = rng.standard_normal((rows, hd)).astype(np.float16)
    q = rng.standard_normal(hd).astype(np.float32)
    for pq in (0, 1, 7, 31):
        for window in (-1, 0, 1, 2, 7, 8, 9, 32, 100):
            t = np.arange(rows)
            masked = t > pq
            if window > 0:                       # the operator's attribute defaults to -1: no window
                masked |= (pq - t) >= window
            scores = np.where(masked, -3.4028235e38, 0.25 * (K.astype(np.float64) @ q.astype(np.float64)))
            p = np.exp(scores - scores.max())
            want = (p / p.sum()) @ V.astype(np.float64)
            assert int((~masked).sum()) == (min(window, pq + 1) if window > 0 else pq + 1)
            got = od.attend(q, K, V, pq, window, 0.25)
            assert np.allclose(got, want, rtol=2e-5, atol=2e-6), (pq, window)


def test_gather_block_quantized_is_a_row_of_the_dequantised_table(oracle, pkg):
    from oracle import decoder as od
    a, nib, zp, scale = rc.matmul_nbits_case(1, 100, 9, 32)
    table = (pkg.synth.pack_nibbles(nib, 32), scale.reshape(-1), pkg.synth.pack_zero_points(zp))
    for row in (0, 4, 8):
        blk = np.arange(100) // 32
        want = (nib[row].astype(np.float32) - zp[row][blk]) * scale[row][blk]
        assert np.array_equal(od.gather_block_quantized(table, row, 100, 32), want)


# ---------------------------------------------------------------- the decode step as a whole

def _dense_f64(lin, K, bs):
    """(B, scales, zp) in the MatMulNBits layout -> float64 [N, K], written out from the format's
    definition (low nibble first, zero-point nibble b & 1 of byte b / 2) without the oracle."""
    B, scales, zp = lin
    N, nb = B.shape[0], B.shape[1]
    q = np.empty((N, nb * bs), np.float64)
    flat = B.reshape(N, -1)
    q[:, 0::2], q[:, 1::2] = flat & 15, flat >> 4
    z = np.empty((N, 2 * zp.shape[1]), np.float64)
    z[:, 0::2], z[:, 1::2] = zp & 15, zp >> 4
    w = (q.reshape(N, nb, bs) - z[:, :nb, None]) * scales.reshape(N, nb, 1).astype(np.float64)
    return w.reshape(N, nb * bs)[:, :K]


def _step_f64(w, caches, token, pos, windows, thetas):
    """One decode step in float64 from the layer formula of the C header (rmsnorm -> qkv -> per-head
    norm + rotary -> f16 cache -> attention -> o -> post-norm residual -> pre-norm -> gated GELU ->
    down -> post-norm residual; final norm -> lm_head). No call into oracle.decoder."""
    from oracle import decoder as od
    c = w.cfg
    hd, nq, nkv, H, F, bs = c["head_dim"], c["n_q_heads"], c["n_kv_heads"], c["hidden"], c["ffn"], c["block_size"]

    def rms(x, g):
        return x / np.sqrt(np.mean(x * x) + c["rms_eps"]) * g.astype(np.float64)

    def rope(x, theta):
        half = hd // 2
        ang = pos * theta ** (-2.0 * np.arange(half) / hd)
        cs, sn = np.cos(ang), np.sin(ang)
        return np.concatenate([x[:half] * cs - x[half:] * sn, x[half:] * cs + x[:half] * sn])

    scale = c["attn_scale"] if c["attn_scale"] > 0 else 1.0 / np.sqrt(hd)
    x = _dense_f64(w.embedding, H, bs)[token] * c["embed_scale"]
    for li in range(c["n_layers"]):
        n = lambda which: w.norms[(li, which)]
        qkv = _dense_f64(w.linears[(li, od.QKV)], H, bs) @ rms(x, n(od.NORM_INPUT))
        q = qkv[: nq * hd].reshape(nq, hd)
        k = qkv[nq * hd: (nq + nkv) * hd].reshape(nkv, hd)
        v = qkv[(nq + nkv) * hd:].reshape(nkv, hd)
        K, V = caches[li]
        for h in range(nkv):
            K[h, pos] = rope(rms(k[h], n(od.NORM_K)), thetas[li]).astype(np.float16)
            V[h, pos] = v[h].astype(np.float16)
        first = max(0, pos + 1 - windows[li]) if windows[li] > 0 else 0
        a = np.empty((nq, hd))
        for h in range(nq):
            qh = rope(rms(q[h], n(od.NORM_Q)), thetas[li])
            kv = h // (nq // nkv)
            s = K[kv, first: pos + 1].astype(np.float64) @ qh * scale
            p = np.exp(s - s.max())
            a[h] = (p / p.sum()) @ V[kv, first: pos + 1].astype(np.float64)
        x = x + rms(_dense_f64(w.linears[(li, od.O)], nq * hd, bs) @ a.reshape(-1), n(od.NORM_POST_ATTN))
        gu = _dense_f64(w.linears[(li, od.GATE_UP)], H, bs) @ rms(x, n(od.NORM_PRE_FFN))
        g, u = gu[:F], gu[F:]
        hcur = 0.5 * g * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (g + 0.044715 * g ** 3))) * u
        x = x + rms(_dense_f64(w.linears[(li, od.DOWN)], F, bs) @ hcur, n(od.NORM_POST_FFN))
    return _dense_f64(w.linears[(0, od.LM_HEAD)], H, bs) @ rms(x, w.norms[(0, od.NORM_FINAL)])


_TINY = dict(n_layers=2, hidden=64, ffn=96, n_q_heads=4, n_kv_heads=2, head_dim=32, vocab=80, block_size=32,
             rms_eps=1e-6, rope_theta=10000.0, attn_scale=0.0, embed_scale=8.0)


def test_decoder_step_composition_against_a_float64_route(oracle, pkg):
    """The wiring of Decoder.step (where the four norms sit, the order of the residual adds, the
    embedding scale, the gate | up split, the window bound, the per-layer rotary base) against a
    float64 evaluation with dense matrices, over several positions so that the cache and the
    window are exercised. A misplaced norm or a swapped gate / up moves the logits by O(1)."""
    from oracle import decoder as od
    w = pkg.decoder.build_weights(_TINY, seed=21)
    max_seq = 12
    ref = od.Decoder(w, max_seq)
    ref.set_layer_attention(1, 3, 500.0)
    windows, thetas = [0, 3], [_TINY["rope_theta"], 500.0]
    caches = [(np.zeros((2, max_seq, 32), np.float16), np.zeros((2, max_seq, 32), np.float16)) for _ in range(2)]
    token = 7
    for pos in range(8):
        got, nxt = ref.step(token, pos)
        want = _step_f64(w, caches, token, pos, windows, thetas)
        assert got.dtype == np.float32 and got.shape == (80,)
        assert np.all(np.abs(got - want) <= 1e-3 + 1e-3 * np.abs(want)), (pos, float(np.abs(got - want).max()))
        assert np.ptp(want) > 0.5, "the case must not be degenerate"
        assert nxt == int(np.argmax(got))
        token = nxt


def test_decoder_step_with_silent_branches_is_the_unembedded_embedding(oracle, pkg):
    """With the output and down projections at zero (all scales 0) both residual branches add
    rmsnorm(0) = 0, so the logits are lm_head(rmsnorm(embed_scale * embedding row, w_final)):
    a closed form that involves none of the per-layer code."""
    from oracle import decoder as od
    w = pkg.decoder.build_weights(_TINY, seed=22)
    for li in range(2):
        for which in (od.O, od.DOWN):
            B, scales, zp = w.linears[(li, which)]
            w.linears[(li, which)] = (B, np.zeros_like(scales), zp)
    ref = od.Decoder(w, 4)
    for token in (0, 5, 79):
        got, _ = ref.step(token, 1)
        x = _dense_f64(w.embedding, 64, 32)[token] * _TINY["embed_scale"]
        xn = x / np.sqrt(np.mean(x * x) + 1e-6) * w.norms[(0, od.NORM_FINAL)]
        want = _dense_f64(w.linears[(0, od.LM_HEAD)], 64, 32) @ xn
        assert np.all(np.abs(got - want) <= 1e-4 + 1e-4 * np.abs(want)), token


def test_decoder_state_rule(oracle):
    """advance_state: smallest index among equal maxima, index 0 when nothing compares, and a step
    at a full cache changes nothing and is reported."""
    from oracle.decoder import advance_state
    logits = np.array([0.5, 3.0, -1.0, 3.0, 2.0], np.float32)
    assert advance_state(9, 4, logits, 8) == (1, 5, False)
    assert advance_state(9, 7, logits, 8) == (1, 8, False)          # the last row of the cache is usable
    assert advance_state(9, 8, logits, 8) == (9, 8, True)           # full: nothing moves
    assert advance_state(9, 2, np.full(5, np.nan, np.float32), 8) == (0, 3, False)
    assert advance_state(9, 2, np.array([np.nan, -np.inf, 1.0], np.float32), 8) == (2, 3, False)
    assert advance_state(9, 2, np.full(4, -np.inf, np.float32), 8)[0] == 0
