"""ConvInteger and QLinearConv on the GPU: int32 accumulators exact, requantised bytes within
one LSB of the oracle (and in practice identical)."""
import json
import os

import numpy as np
import pytest

import refcases as rc

pytestmark = pytest.mark.gpu


def _golden():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "qlinear_golden.json")
    with open(path) as f:
        return [c for c in json.load(f) if c["op"] == "QLinearConv"]


@pytest.mark.parametrize("case", _golden(), ids=lambda c: c["name"])
def test_qlinear_conv_golden_literals(ctx, pkg, case):
    """The literal nodes of crates/onnx-vulkan-core/tests/qlinear.rs:106-236."""
    names = ["x", "x_scale", "x_zp", "w", "w_scale", "w_zp", "y_scale", "y_zp"]
    env = {"x": np.array(case["x"], np.uint8).reshape(case["x_shape"]), "x_scale": np.float32(case["x_scale"]),
           "x_zp": np.array(case["x_zp"], np.uint8), "w": np.array(case["w"], np.int8).reshape(case["w_shape"]),
           "w_scale": np.array(case["w_scale"], np.float32), "w_zp": np.array(case["w_zp"], np.int8),
           "y_scale": np.float32(case["y_scale"]), "y_zp": np.array(case["y_zp"], np.uint8)}
    if case["bias"] is not None:
        names.append("B")
        env["B"] = np.array(case["bias"], np.int32)
    node = pkg.graph.NodeIr("QLinearConv", names, ["out"], {"kernel_shape": [2, 2]})
    pkg.graph.execute(ctx, [node], env)
    assert env["out"].dtype == np.uint8 and env["out"].reshape(-1).tolist() == case["want"]


@pytest.mark.parametrize("case", rc.CONV_CASES, ids=lambda c: "c%d_o%d_%dx%d_s%d_d%d" % (
    c["c_in"], c["c_out"], c["h"], c["w"], c["stride"], c["dilation"]))
def test_conv_integer_reference_cases(ctx, pkg, oracle, case):
    """crates/onnx-vulkan-core/tests/conv_integer_im2col.rs:185-247, as ConvInteger nodes."""
    X, W, x_zp, w_zp = rc.conv_case_operands(case)
    s, d = case["stride"], case["dilation"]
    t, l, b, r = case["pads"]
    node = pkg.graph.NodeIr("ConvInteger", ["x", "w", "x_zp", "w_zp"], ["y"],
                            {"strides": [s, s], "dilations": [d, d], "pads": [t, l, b, r]})
    env = {"x": X, "w": W, "x_zp": np.array(x_zp, X.dtype), "w_zp": np.array(w_zp, W.dtype)}
    pkg.graph.execute(ctx, [node], env)
    want = rc.conv_integer_dense(X, W, x_zp, w_zp, (s, s), (d, d), case["pads"])
    assert env["y"].shape == want.shape and np.array_equal(env["y"], want)


def _qconv_case(pkg, c_in, c_out, t, kw, dil, seed, n=1, h=1, kh=1, group=1, stride=1):
    X = pkg.synth.uniform_ints(n * c_in * h * t, seed, 0, 255).astype(np.uint8).reshape(n, c_in, h, t)
    W = pkg.synth.uniform_ints(c_out * (c_in // group) * kh * kw, seed + 1, -127, 127).astype(np.int8).reshape(
        c_out, c_in // group, kh, kw)
    w_scale = pkg.synth.uniform_f32(c_out, seed + 2, 0.001, 0.02)
    bias = pkg.synth.uniform_ints(c_out, seed + 3, -4096, 4096).astype(np.int32)
    pad_w = dil * (kw - 1) // 2
    pad_h = (kh - 1) // 2
    kwargs = dict(strides=(stride, stride), dilations=(1, dil), pads=(pad_h, pad_w, pad_h, pad_w), group=group)
    return X, W, w_scale, bias, kwargs


def _y_scale(x_scale, w_scale, k):
    # chosen so the outputs span the byte range instead of saturating
    return float(x_scale * np.mean(w_scale) * 74 * 73 * np.sqrt(k) / 100.0)


@pytest.mark.parametrize("dil", [1, 3, 5])
def test_vocoder_resblock_shape(ctx, pkg, oracle, dil):
    """192 -> 192 channels, kernel 7, T = 4096, 'same' padding, dilation 1 / 3 / 5."""
    X, W, w_scale, bias, kw = _qconv_case(pkg, 192, 192, 4096, 7, dil, seed=50 + dil)
    geom, og = pkg.ConvGeom.make(X.shape, W.shape, **kw), oracle.conv_geom(X.shape, W.shape, **kw)
    acc = pkg.ops.conv_integer(ctx, X, W, 128, 0, geom)
    assert np.array_equal(acc, oracle.conv_integer(X, W, 128, 0, og))                       # bit-exact accumulators
    ys = _y_scale(0.02, w_scale, 192 * 7)
    got = pkg.ops.qlinear_conv(ctx, X, 0.02, 128, W, w_scale, 0, ys, 128, bias, geom)
    want = oracle.qlinear_conv(X, 0.02, 128, W, w_scale, 0, ys, 128, bias, og)
    assert got.shape == (1, 192, 1, 4096)
    assert np.max(np.abs(got.astype(int) - want.astype(int))) <= 1
    assert np.array_equal(got, want)
    assert np.count_nonzero((got > 0) & (got < 255)) > 0.6 * got.size   # the case must not saturate away


def test_replays_from_a_graph_once_its_ratios_are_resident(ctx, pkg, oracle):
    """The requantisation ratios are uploaded by the first call with given scales and kept with the
    weight: the same call is then captured, and each replay requantises a new input correctly. A
    call whose scales differ would have to upload inside the capture and is refused."""
    X, W, w_scale, bias, kw = _qconv_case(pkg, 64, 64, 512, 7, 3, seed=77)
    geom, og = pkg.ConvGeom.make(X.shape, W.shape, **kw), oracle.conv_geom(X.shape, W.shape, **kw)
    ys = _y_scale(0.02, w_scale, 64 * 7)
    weight = pkg.ops.ConvWeight(ctx, W, geom)
    dX, dY, dB = ctx.upload(X), ctx.alloc(X.size), ctx.upload(bias.astype(np.int32))
    run = lambda s: pkg.ops.qlinear_conv_device(ctx, dX, pkg.U8, 0.02, 128, weight, w_scale, 0, s, 128, pkg.U8, dB, geom, dY)
    run(ys)
    ctx.flush()
    ctx.capture_begin()
    run(ys)
    with pytest.raises(pkg.HipComputeError) as e:
        run(2 * ys)
    assert e.value.code == 2
    graph = ctx.capture_end()
    for seed in (78, 79):
        X2 = pkg.synth.uniform_ints(X.size, seed, 0, 255).astype(np.uint8).reshape(X.shape)
        ctx.upload(X2, dX)
        ctx.graph_launch(graph)
        got = ctx.download(dY, np.uint8, X.shape)
        assert np.array_equal(got, oracle.qlinear_conv(X2, 0.02, 128, W, w_scale, 0, ys, 128, bias, og))
    ctx.graph_destroy(graph)
    weight.destroy()
    for b in (dX, dY, dB):
        b.free()


def test_wide_decoder_variant(ctx, pkg, oracle):
    """512 -> 512 channels, kernel 7, stride 1, T = 4096: the size the benchmark times."""
    X, W, w_scale, bias, kw = _qconv_case(pkg, 512, 512, 4096, 7, 1, seed=60)
    geom, og = pkg.ConvGeom.make(X.shape, W.shape, **kw), oracle.conv_geom(X.shape, W.shape, **kw)
    ys = _y_scale(0.02, w_scale, 512 * 7)
    got = pkg.ops.qlinear_conv(ctx, X, 0.02, 128, W, w_scale, 0, ys, 128, bias, geom)
    assert np.array_equal(got, oracle.qlinear_conv(X, 0.02, 128, W, w_scale, 0, ys, 128, bias, og))


@pytest.mark.parametrize("cfg", [
    dict(c_in=16, c_out=8, t=37, kw=3, dil=1, n=3, h=9, kh=3),               # batch > 1, 2-D, ragged tiles
    dict(c_in=48, c_out=130, t=70, kw=5, dil=2, n=2, h=4, kh=3, stride=2),   # strided, more than one row tile
    dict(c_in=24, c_out=24, t=50, kw=7, dil=3, group=24),                    # depthwise: direct kernel
    dict(c_in=8, c_out=12, t=50, kw=7, dil=1, group=4),                      # grouped
    dict(c_in=3, c_out=10, t=64, kw=3, dil=1, h=8, kh=3),                    # channels not a multiple of 16
], ids=lambda c: "c%d_o%d_g%d" % (c["c_in"], c["c_out"], c.get("group", 1)))
@pytest.mark.parametrize("signs", [(np.uint8, np.int8), (np.int8, np.uint8)], ids=["u8xi8", "i8xu8"])
def test_geometries_and_signs(ctx, pkg, oracle, cfg, signs):
    X, W, w_scale, bias, kw = _qconv_case(pkg, seed=70, **cfg)
    X, W = X.view(signs[0]), W.view(signs[1])
    geom, og = pkg.ConvGeom.make(X.shape, W.shape, **kw), oracle.conv_geom(X.shape, W.shape, **kw)
    x_zp = 100 if signs[0] == np.uint8 else -20
    w_zp = 0 if signs[1] == np.int8 else 131
    acc = pkg.ops.conv_integer(ctx, X, W, x_zp, w_zp, geom)
    want = rc.conv_integer_dense(X, W, x_zp, w_zp, kw["strides"], kw["dilations"], kw["pads"], kw["group"])
    assert np.array_equal(acc, want)
    # per-tensor weight scale so an asymmetric weight zero point is allowed; int8 output
    got = pkg.ops.qlinear_conv(ctx, X, 0.03, x_zp, W, np.float32(0.004), w_zp, 0.7, -5, bias, geom, y_signed=True)
    assert np.array_equal(got, oracle.qlinear_conv(X, 0.03, x_zp, W, np.float32(0.004), w_zp, 0.7, -5, bias, og, True))
    got = pkg.ops.qlinear_conv(ctx, X, 0.03, x_zp, W, np.float32(0.004), w_zp, 0.7, 99, None, geom)
    assert np.array_equal(got, oracle.qlinear_conv(X, 0.03, x_zp, W, np.float32(0.004), w_zp, 0.7, 99, None, og))


ROWS = [  # 1-D convolutions whose input slab stays in LDS: (c_in, c_out, t, kw, dilation, stride, pads l/r, batch)
    (112, 70, 200, 5, 2, 2, (3, 6), 2),     # an odd number of 16-channel chunks, strided, lopsided pads, ragged tiles
    (32, 64, 260, 17, 1, 3, (0, 5), 1),     # four taps per product step; no left pad
    (208, 96, 128, 3, 7, 1, (7, 7), 3),     # a tap straddles product steps (208 = 128 + 80)
    (512, 64, 64, 7, 20, 1, (60, 60), 1),   # the slab would not fit: the general route
]


@pytest.mark.parametrize("signs", [(np.uint8, np.int8), (np.int8, np.uint8)], ids=["u8xi8", "i8xu8"])
@pytest.mark.parametrize("c_in,c_out,t,kw,dil,stride,pads,n", ROWS, ids=lambda v: str(v).replace(" ", ""))
def test_row_convolutions_straight_from_nchw(ctx, pkg, oracle, c_in, c_out, t, kw, dil, stride, pads, n, signs):
    """One filter axis, k >= 512: the kernel that keeps a tile's input positions in LDS and reads the
    NCHW activation itself -- against the dense definition (tests/conv_integer_im2col.rs:58-89)
    and the oracle's requantisation."""
    X, W, w_scale, bias, kwargs = _qconv_case(pkg, c_in, c_out, t, kw, dil, seed=90 + c_in, n=n, stride=stride)
    kwargs["pads"] = (0, pads[0], 0, pads[1])
    kwargs["strides"] = (1, stride)
    X, W = X.view(signs[0]), W.view(signs[1])
    geom, og = pkg.ConvGeom.make(X.shape, W.shape, **kwargs), oracle.conv_geom(X.shape, W.shape, **kwargs)
    x_zp = 100 if signs[0] == np.uint8 else -20
    w_zp = 0 if signs[1] == np.int8 else 131
    acc = pkg.ops.conv_integer(ctx, X, W, x_zp, w_zp, geom)
    want = rc.conv_integer_dense(X, W, x_zp, w_zp, kwargs["strides"], kwargs["dilations"], kwargs["pads"], 1)
    assert acc.shape == want.shape and np.array_equal(acc, want)
    got = pkg.ops.qlinear_conv(ctx, X, 0.03, x_zp, W, np.float32(0.004), w_zp, 2.5, -5, bias, geom, y_signed=True)
    assert np.array_equal(got, oracle.qlinear_conv(X, 0.03, x_zp, W, np.float32(0.004), w_zp, 2.5, -5, bias, og, True))


def test_one_dimensional_node_with_auto_pad(ctx, pkg, oracle):
    X, W, w_scale, bias, _ = _qconv_case(pkg, 32, 32, 300, 7, 3, seed=80)
    node = pkg.graph.NodeIr("QLinearConv", ["x", "x_scale", "x_zp", "w", "w_scale", "w_zp", "y_scale", "y_zp", "B"],
                            ["y"], {"auto_pad": "SAME_UPPER", "dilations": [3]})
    env = {"x": X.reshape(1, 32, 300), "x_scale": np.float32(0.02), "x_zp": np.array(128, np.uint8),
           "w": W.reshape(32, 32, 7), "w_scale": w_scale, "w_zp": np.zeros(32, np.int8),
           "y_scale": np.float32(0.4), "y_zp": np.array(128, np.uint8), "B": bias}
    pkg.graph.execute(ctx, [node], env)
    og = oracle.conv_geom(X.shape, W.shape, dilations=(1, 3), pads=(0, 9, 0, 9))
    want = oracle.qlinear_conv(X, 0.02, 128, W, w_scale, 0, 0.4, 128, bias, og)
    assert env["y"].shape == (1, 32, 300) and np.array_equal(env["y"].reshape(want.shape), want)


def test_refusals(ctx, pkg):
    X = np.zeros((1, 16, 1, 32), np.uint8)
    W = np.zeros((8, 16, 1, 3), np.int8)
    geom = pkg.ConvGeom.make(X.shape, W.shape, pads=(0, 1, 0, 1))
    with pytest.raises(pkg.HipComputeError) as e:   # asymmetric per-channel weights (interp.rs:830-835)
        pkg.ops.qlinear_conv(ctx, X, 0.02, 128, W, np.full(8, 0.01, np.float32), 3, 0.05, 10, None, geom)
    assert e.value.code == 2 and "per-channel zero point" in e.value.message
    with pytest.raises(pkg.HipComputeError) as e:   # y_scale == 0 (interp.rs:4692)
        pkg.ops.qlinear_conv(ctx, X, 0.02, 128, W, np.full(8, 0.01, np.float32), 0, 0.0, 10, None, geom)
    assert e.value.code == 1
    bad = pkg.ConvGeom.make((1, 16, 1, 2), W.shape)     # the window does not fit
    with pytest.raises(ValueError):
        pkg.ops.conv_integer(ctx, X[..., :2], W, 0, 0, bad)


@pytest.mark.parametrize("signs", [(np.uint8, np.int8), (np.int8, np.uint8)], ids=["u8xi8", "i8xu8"])
def test_many_tiles_in_two_dimensions_take_the_128x128_kernel(ctx, pkg, oracle, signs):
    """A 3x3 convolution over a 192 x 200 image: 2 x 300 tiles of 128x128, the LDS-staged
    128x128 kernel in its gathering form (NHWC copy, padding taps read the zero point)."""
    X, W, w_scale, bias, kw = _qconv_case(pkg, 32, 200, 200, 3, 1, seed=140, h=192, kh=3)
    X, W = X.view(signs[0]), W.view(signs[1])
    geom, og = pkg.ConvGeom.make(X.shape, W.shape, **kw), oracle.conv_geom(X.shape, W.shape, **kw)
    x_zp = 100 if signs[0] == np.uint8 else -20
    w_zp = 0 if signs[1] == np.int8 else 131
    acc = pkg.ops.conv_integer(ctx, X, W, x_zp, w_zp, geom)
    assert np.array_equal(acc, oracle.conv_integer(X, W, x_zp, w_zp, og))
    got = pkg.ops.qlinear_conv(ctx, X, 0.03, x_zp, W, np.float32(0.004), w_zp, 0.7, -5, bias, geom, y_signed=True)
    assert np.array_equal(got, oracle.qlinear_conv(X, 0.03, x_zp, W, np.float32(0.004), w_zp, 0.7, -5, bias, og, True))


CONV_ROUTES = [  # every alternative route of a convolution along one axis, forced in process
    {"HIPC_CONV_ROW": 0},                                               # NHWC copy + the k-split gathering kernel
    {"HIPC_CONV_ROW": 0, "HIPC_GEMM_SMALL": 0, "HIPC_GEMM_TILE": 64},   # ... + LDS-staged 64x64 tiles
    {"HIPC_CONV_ROW": 0, "HIPC_GEMM_SMALL": 0, "HIPC_GEMM_TILE": 128},  # ... + LDS-staged 128x128 tiles
]


@pytest.mark.parametrize("options", CONV_ROUTES, ids=lambda o: ",".join("%s=%d" % kv for kv in o.items()))
def test_every_route_of_a_row_convolution_can_be_forced(ctx, pkg, oracle, options):
    X, W, w_scale, bias, kw = _qconv_case(pkg, 96, 80, 700, 7, 3, seed=150, n=2)
    geom, og = pkg.ConvGeom.make(X.shape, W.shape, **kw), oracle.conv_geom(X.shape, W.shape, **kw)
    ys = _y_scale(0.02, w_scale, 96 * 7)
    want_acc = oracle.conv_integer(X, W, 128, 0, og)
    want = oracle.qlinear_conv(X, 0.02, 128, W, w_scale, 0, ys, 128, bias, og)
    with ctx.options(**options):
        assert np.array_equal(pkg.ops.conv_integer(ctx, X, W, 128, 0, geom), want_acc)
        assert np.array_equal(pkg.ops.qlinear_conv(ctx, X, 0.02, 128, W, w_scale, 0, ys, 128, bias, geom), want)


def test_a_recorded_graph_survives_scratch_growth_and_new_scales(ctx, pkg, oracle):
    """A captured QLinearConv on the route that transposes into scratch, then a larger one run
    eagerly (the scratch block must grow) with other scales on the same weight (new ratios), a flush,
    and the replay: the graph still owns the block and the ratios it was recorded with."""
    with ctx.options(HIPC_CONV_ROW=0):
        X, W, w_scale, bias, kw = _qconv_case(pkg, 64, 64, 512, 7, 3, seed=160)
        geom, og = pkg.ConvGeom.make(X.shape, W.shape, **kw), oracle.conv_geom(X.shape, W.shape, **kw)
        ys = _y_scale(0.02, w_scale, 64 * 7)
        weight = pkg.ops.ConvWeight(ctx, W, geom)
        dX, dY, dB = ctx.upload(X), ctx.alloc(X.size), ctx.upload(bias.astype(np.int32))
        run = lambda s: pkg.ops.qlinear_conv_device(ctx, dX, pkg.U8, 0.02, 128, weight, w_scale, 0, s, 128, pkg.U8, dB, geom, dY)
        run(ys)
        ctx.flush()
        ctx.capture_begin()
        run(ys)
        graph = ctx.capture_end()
        # eager work that retires both blocks the graph names
        Xb, Wb, wsb, bb, kwb = _qconv_case(pkg, 64, 64, 70000, 7, 3, seed=161, n=4)   # 18 MB to transpose: the scratch grows
        gb, ogb = pkg.ConvGeom.make(Xb.shape, Wb.shape, **kwb), oracle.conv_geom(Xb.shape, Wb.shape, **kwb)
        big = pkg.ops.qlinear_conv(ctx, Xb, 0.02, 128, Wb, wsb, 0, ys, 128, bb, gb)
        assert np.array_equal(big[:, :, :, :300], oracle.qlinear_conv(Xb[:, :, :, :320], 0.02, 128, Wb, wsb, 0, ys, 128, bb,
                                                                    oracle.conv_geom(Xb[:, :, :, :320].shape, Wb.shape, **kwb))[:, :, :, :300])
        run(3 * ys)                        # new ratios on the recorded weight
        ctx.flush()
        filler = [ctx.alloc(1 << 20) for _ in range(8)]   # whatever was freed is handed out again
        for b in filler:
            ctx.fill(b, 0, 1 << 20, 0xFFFFFFFF)
        ctx.flush()
        ctx.graph_launch(graph)
        got = ctx.download(dY, np.uint8, X.shape)
        assert np.array_equal(got, oracle.qlinear_conv(X, 0.02, 128, W, w_scale, 0, ys, 128, bias, og))
        ctx.graph_destroy(graph)
        weight.destroy()
        for b in [dX, dY, dB] + filler:
            b.free()
        ctx.flush()
