"""The runtime half of the boundary: buffers, ordering, capture / replay, timing, errors."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_upload_copy_fill_download(ctx):
    a = np.arange(1000, dtype=np.int32)
    d = ctx.upload(a)
    e = ctx.alloc(4000)
    ctx.fill(e, 0, 4000, 0xDEADBEEF)
    ctx.copy(e, 400, d, 0, 2000)
    out = ctx.download(e, np.uint32, (1000,))
    assert np.all(out[:100] == 0xDEADBEEF) and np.array_equal(out[100:600], a[:500].astype(np.uint32))
    assert np.all(out[600:] == 0xDEADBEEF)
    d.free(), e.free()
    ctx.flush()


def test_capture_replays_equal_eager_every_time(ctx, pkg, oracle):
    """A captured MatMulNBits decode step + DynamicQuantizeLinear, replayed several times with
    eager work and synchronisations in between; every replay must equal the eager result."""
    k, n, bs = 1152, 1024, 32
    B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=31)
    w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
    dA, dY = ctx.alloc(4 * k), ctx.alloc(4 * n)
    dQ, dP = ctx.alloc(n), ctx.alloc(8)

    def step():
        pkg.ops.matmul_nbits_packed_device(ctx, dA, pkg.F32, w, dY, 1)
        pkg.ops.dynamic_quantize_linear_device(ctx, dY, n, dQ, dP, dP.at(4))

    a0 = pkg.synth.normal_f32(k, 32).reshape(1, k)
    ctx.upload(a0, dA)
    step()                                  # warm: scratch is sized before the capture
    ctx.flush()
    ctx.capture_begin()
    step()
    graph = ctx.capture_end()
    for i in range(4):
        a = pkg.synth.normal_f32(k, 40 + i).reshape(1, k)
        ctx.upload(a, dA)
        ctx.fill(dY, 0, 4 * n, 0)           # eager work between replays
        ctx.flush()
        ctx.graph_launch(graph)
        y = ctx.download(dY, np.float32, (1, n))
        want = oracle.matmul_nbits(a, B, scales, zp, k, n, bs)
        assert np.all(np.abs(y - want) <= 1e-3 + 1e-4 * np.abs(want)), i
        q, s, z = oracle.dynamic_quantize_linear(y)
        assert np.array_equal(ctx.download(dQ, np.uint8, (1, n)), q)
        assert ctx.download(dP, np.float32, (1,))[0].tobytes() == np.float32(s).tobytes()
        step()                              # the same step, eagerly
        assert np.array_equal(ctx.download(dY, np.float32, (1, n)), y)
    ns = ctx.measure_graph(graph, 5, 20)
    assert ns.shape == (5,) and np.all(ns > 0) and np.all(ns < 1e9)
    ctx.graph_destroy(graph)
    w.destroy()


def test_errors_carry_a_message_and_leave_the_context_usable(ctx, pkg):
    with pytest.raises(pkg.HipComputeError) as e:
        ctx.fill(ctx.alloc(16), 0, 6, 0)
    assert e.value.code == 1 and "multiples of 4" in e.value.message
    with pytest.raises(pkg.HipComputeError):
        ctx.capture_end()
    scratch = ctx.alloc(64)
    ctx.capture_begin()
    with pytest.raises(pkg.HipComputeError) as e:
        ctx.alloc(64)
    assert e.value.code == 2
    ctx.fill(scratch, 0, 64, 1)
    ctx.graph_destroy(ctx.capture_end())
    d = ctx.upload(np.arange(4, dtype=np.int32))
    assert np.array_equal(ctx.download(d, np.int32, (4,)), np.arange(4))


def test_a_second_context_on_a_caller_stream(ctx, pkg, oracle):
    """Adopting a stream the caller owns keeps the library's work on that stream. The stream comes
    from the HIP runtime the library itself is linked against (a second HIP runtime in the process,
    such as the one a PyTorch wheel bundles, does not see the device once this one holds it)."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    stream = C.c_void_p()
    assert hip.hipStreamCreateWithFlags(C.byref(stream), 1) == 0      # hipStreamNonBlocking
    with pkg.Context(0, stream=stream.value) as c2:
        assert c2.stream == stream.value
        x = pkg.synth.normal_f32(4096, 50)
        y, sc, z = pkg.ops.dynamic_quantize_linear(c2, x)
        wy, ws, wz = oracle.dynamic_quantize_linear(x)
        assert np.array_equal(y, wy) and z == wz
    assert hip.hipStreamDestroy(stream) == 0


def test_freed_blocks_are_handed_out_again_by_size_class(ctx):
    """hipc_alloc serves a request from the blocks earlier frees of its size class left behind
    (crates/vk-compute/src/buffer.rs:303-341): after a flush the same address comes back and no
    device allocation happens."""
    ctx.flush()
    a = ctx.alloc(3000)                    # class 4096
    first = a.ptr
    a.free()
    b = ctx.alloc(3500)                    # before the flush the block is still in use: another one
    assert b.ptr != first
    ctx.flush()
    hits0, misses0, _ = ctx.pool_stats()
    c = ctx.alloc(4096)
    assert c.ptr == first
    hits1, misses1, waiting = ctx.pool_stats()
    assert (hits1, misses1) == (hits0 + 1, misses0)
    big = ctx.alloc((5 << 20) + 1)         # whole MiB above 1 MiB: class 6 MiB
    p = big.ptr
    big.free()
    ctx.flush()
    again = ctx.alloc(6 << 20)
    assert again.ptr == p
    for x in (b, c, again):
        x.free()
    ctx.flush()


def test_uploads_only_record(ctx):
    """hipc_upload stages the bytes and returns: the source may be overwritten at once, uploads
    larger than the staging ring arrive whole, and order with other stream work is call order."""
    n = 50 << 20                            # three times the ring
    src = np.arange(n // 4, dtype=np.uint32)
    d = ctx.alloc(n)
    ctx.fill(d, 0, n, 0)
    ctx.upload(src, d)
    src[:] = 0                              # the call has copied what it needs
    ctx.fill(d, 4 * 1000, 4 * 10, 7)        # later stream work lands on top
    out = ctx.download(d, np.uint32, (n // 4,))
    want = np.arange(n // 4, dtype=np.uint32)
    want[1000:1010] = 7
    assert np.array_equal(out, want)
    small = [ctx.upload(np.full(5, i, np.int32)) for i in range(300)]   # many small uploads share slots
    for i in (0, 150, 299):
        assert np.array_equal(ctx.download(small[i], np.int32, (5,)), np.full(5, i, np.int32))
    for b in small + [d]:
        b.free()
    ctx.flush()


def test_unknown_options_are_refused(ctx, pkg):
    with pytest.raises(pkg.HipComputeError) as e:
        ctx.set_option("HIPC_NO_SUCH_THING", 1)
    assert e.value.code == 1
    ctx.set_option("HIPC_GEMM_TILE", 128)
    ctx.set_option("HIPC_GEMM_TILE", -1)


def test_scalars_of_a_recorded_graph_can_be_patched(ctx, pkg, oracle):
    """The reference patches push-constant words of a recorded step between replays
    (crates/onnx-vulkan-core/src/plan.rs:52-68). Here: a graph of QLinearMatMul, QLinearConv and the fused
    rescale is recorded once and replayed with other zero points / the relu attribute, every replay against
    the oracle; a scalar the recorded call does not carry is refused."""
    ops, rt = pkg.ops, pkg.runtime
    rng = np.random.default_rng(5)
    m, k, n = 70, 256, 96
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(0, 256, (k, n), dtype=np.uint8)
    w = ops.Int8Weight(ctx, b)
    dA, dY = ctx.upload(a), ctx.alloc(m * n)
    ys = 0.9
    qmm = lambda a_zp, b_zp, y_zp: ops.qlinear_matmul_device(ctx, dA, pkg.U8, 0.02, a_zp, w, np.float32(0.01), b_zp, ys, y_zp, pkg.U8, dY, m)  # noqa: E731
    # conv: 1-D, grouped (the direct kernel) and dense (the slab kernel)
    X = rng.integers(0, 256, (1, 32, 1, 64), dtype=np.uint8)
    W = rng.integers(-127, 128, (32, 32, 1, 3), dtype=np.int8)
    geom = pkg.ConvGeom.make(X.shape, W.shape, pads=(0, 1, 0, 1))
    og = oracle.conv_geom(X.shape, W.shape, pads=(0, 1, 0, 1))
    cw = ops.ConvWeight(ctx, W, geom)
    dX, dC = ctx.upload(X), ctx.alloc(X.size)
    wsc = np.full(32, 0.01, np.float32)
    qconv = lambda x_zp, y_zp: ops.qlinear_conv_device(ctx, dX, pkg.U8, 0.02, x_zp, cw, wsc, 0, 0.3, y_zp, pkg.U8, None, geom, dC)  # noqa: E731
    # fused rescale
    dS = ctx.upload(np.array([0.003], np.float32))
    dZ = ctx.upload(np.array([131, 0, 0, 0], np.uint8))
    dF = ctx.alloc(m * n * 4)
    resc = lambda relu: ops.matmul_integer_scale_bias_device(ctx, dA, pkg.U8, w, dZ, None, dS, 0, None, 0, None, 0, relu, None, dF, m)  # noqa: E731
    qmm(128, 121, 7), qconv(128, 10), resc(False)      # once eagerly: ratios uploaded, scratch sized
    ctx.flush()
    ctx.capture_begin()
    qmm(128, 121, 7), qconv(128, 10), resc(False)
    g = ctx.capture_end()
    assert ctx.graph_op_count(g) == 3

    def check(a_zp, b_zp, y_zp, x_zp, cy_zp, relu):
        ctx.graph_launch(g)
        got = ctx.download(dY, np.uint8, (m, n))
        assert np.array_equal(got, oracle.qlinear_matmul(a, 0.02, a_zp, b, np.float32(0.01), b_zp, ys, y_zp, False))
        gotc = ctx.download(dC, np.uint8, X.shape)
        assert np.array_equal(gotc, oracle.qlinear_conv(X, 0.02, x_zp, W, wsc, 0, 0.3, cy_zp, None, og))
        acc = oracle.matmul_integer(a, b, 131, 0)
        want = oracle.rescale(acc, np.float32(0.003), None)
        gotf = ctx.download(dF, np.float32, (m, n))
        assert np.array_equal(gotf.view(np.uint32), (np.maximum(want, 0) if relu else want).view(np.uint32))

    check(128, 121, 7, 128, 10, False)
    ctx.graph_set_scalar(g, 0, rt.SCALAR_A_ZERO_POINT, 90)
    ctx.graph_set_scalar(g, 0, rt.SCALAR_B_ZERO_POINT, 3)
    ctx.graph_set_scalar(g, 0, rt.SCALAR_Y_ZERO_POINT, 200)
    ctx.graph_set_scalar(g, 1, rt.SCALAR_A_ZERO_POINT, 77)
    ctx.graph_set_scalar(g, 1, rt.SCALAR_Y_ZERO_POINT, 130)
    ctx.graph_set_scalar(g, 2, rt.SCALAR_RELU, 1)
    check(90, 3, 200, 77, 130, True)
    check(90, 3, 200, 77, 130, True)                   # a patch holds for every later replay
    with pytest.raises(pkg.HipComputeError) as e:      # the int8 weight's zero point was known to be zero when the conv was recorded
        ctx.graph_set_scalar(g, 1, rt.SCALAR_B_ZERO_POINT, 5)
    assert e.value.code == 2
    with pytest.raises(pkg.HipComputeError) as e:
        ctx.graph_set_scalar(g, 2, rt.SCALAR_Y_ZERO_POINT, 5)
    assert e.value.code == 2
    with pytest.raises(pkg.HipComputeError) as e:
        ctx.graph_set_scalar(g, 3, rt.SCALAR_RELU, 1)
    assert e.value.code == 1
    ctx.graph_destroy(g)
    w.destroy(), cw.destroy()
    for buf in (dA, dY, dX, dC, dS, dZ, dF):
        buf.free()
