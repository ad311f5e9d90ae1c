"""The DynamicQuantizeLinear entry point that allocates nothing (its range partials live in a static
array of the library's device image) against the ordinary entry point: bit for bit, on two calls in
a row, the second with a smaller input than the first."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_static_scratch_variant_equals_the_ordinary_entry_point(ctx, pkg, oracle):
    for n, seed in ((1000 * 1024 + 3, 501), (4099, 502)):          # 250 range partials, then 2
        x = (pkg.synth.normal_f32(n, seed) * np.float32(1.0 + seed % 7)).astype(np.float32)
        want = pkg.ops.dynamic_quantize_linear(ctx, x)
        got = pkg.ops.dynamic_quantize_linear_static(ctx, x)
        assert np.array_equal(got[0], want[0])
        assert np.float32(got[1]).tobytes() == np.float32(want[1]).tobytes() and got[2] == want[2]
        ref = oracle.dynamic_quantize_linear(x)
        assert np.array_equal(got[0], ref[0]) and np.float32(got[1]).tobytes() == np.float32(ref[1]).tobytes() and got[2] == ref[2]


def test_static_scratch_variant_limits_and_empty_input(ctx, pkg):
    import ctypes as C
    d = ctx.alloc(64)
    rc = ctx.lib.hipc_dynamic_quantize_linear_static(ctx.handle, d.ptr, (1 << 30) + 1, d.ptr, d.ptr, d.ptr + 4)
    assert rc == 1 and b"exceed the limit" in ctx.lib.hipc_last_error(ctx.handle)
    y, scale, zp = pkg.ops.dynamic_quantize_linear_static(ctx, np.zeros(0, np.float32))
    assert y.size == 0 and scale == 1.0 and zp == 0
    d.free()


def test_static_scratch_variant_allocates_nothing(ctx, pkg, oracle):
    """Recorded into a graph before it ever ran eagerly at this size (allocation and scratch growth are
    refused while a capture is open, so a hidden allocation would fail here), replayed twice on fresh
    input, every replay against the oracle; the allocation pool sees no request across the calls."""
    n = 300 * 1024 + 5
    dX, dY, dP = ctx.alloc(4 * n), ctx.alloc(n), ctx.alloc(8)
    before = ctx.pool_stats()
    ctx.capture_begin()
    ctx._check(ctx.lib.hipc_dynamic_quantize_linear_static(ctx.handle, dX.ptr, n, dY.ptr, dP.ptr, dP.ptr + 4))
    g = ctx.capture_end()
    for seed, gain in ((511, 0.5), (512, 3.0)):
        x = (pkg.synth.normal_f32(n, seed) * np.float32(gain)).astype(np.float32)
        ctx.upload(x, dX)
        ctx.graph_launch(g)
        y = ctx.download(dY, np.uint8, (n,))
        scale = ctx.download(dP, np.float32, (1,))[0]
        zp = int(ctx.download(dP, np.uint8, (1,), offset=4)[0])
        ref = oracle.dynamic_quantize_linear(x)
        assert np.array_equal(y, ref[0]) and np.float32(scale).tobytes() == np.float32(ref[1]).tobytes() and zp == ref[2]
    hits, misses, _ = ctx.pool_stats()
    assert (hits, misses) == before[:2]
    ctx.graph_destroy(g)
    for b in (dX, dY, dP):
        b.free()
