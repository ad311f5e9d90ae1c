"""MatMulNBits on the GPU against the oracle, through the C ABI.

Tolerance (the one the task states for this operator): |got - ref| <= atol + rtol * |ref| with
atol = 1e-3 and rtol = 1e-4 for f32 tensors, rtol = 1e-3 for f16 tensors.
"""
import numpy as np
import pytest

import refcases as rc

pytestmark = pytest.mark.gpu

ATOL, RTOL32, RTOL16 = 1e-3, 1e-4, 1e-3


def close(got, ref, rtol):
    got, ref = got.astype(np.float64), ref.astype(np.float64)
    return np.all(np.abs(got - ref) <= ATOL + rtol * np.abs(ref))


def worst(got, ref):
    return float(np.max(np.abs(got.astype(np.float64) - ref.astype(np.float64))))


@pytest.mark.parametrize("case", rc.MATMUL_NBITS_CASES, ids=lambda c: "M%d_K%d_N%d_bs%d" % c)
def test_reference_cases_as_nodes(ctx, pkg, oracle, case):
    """The seven cases of crates/onnx-vulkan-core/tests/matmul_nbits.rs, built as the reference
    builds them: one com.microsoft::MatMulNBits node, tensors by name."""
    m, k, n, bs = case
    a, nib, zp, scale = rc.matmul_nbits_case(m, k, n, bs)
    B, Z = pkg.synth.pack_nibbles(nib, bs), pkg.synth.pack_zero_points(zp)
    node = pkg.graph.NodeIr("MatMulNBits", ["a", "quant", "scales", "zp"], ["out"],
                            {"K": k, "N": n, "bits": 4, "block_size": bs}, domain="com.microsoft", name="mmnb")
    assert pkg.graph.is_implemented_node(node)
    env = {"a": a, "quant": B, "scales": scale.reshape(-1), "zp": Z}
    pkg.graph.execute(ctx, [node], env)
    want = oracle.matmul_nbits(a, B, scale.reshape(-1), Z, k, n, bs)
    got = env["out"]
    assert got.shape == (m, n) and got.dtype == np.float32
    assert close(got, want, RTOL32), worst(got, want)
    # and the reference's own bound against the mathematics
    f64 = rc.matmul_nbits_f64(a, nib, zp, scale, bs)
    assert np.all(np.abs(got - f64) <= 1e-4 * np.maximum(np.abs(f64), 1.0))


@pytest.mark.parametrize("case", [c for c in rc.MATMUL_NBITS_CASES if c[3] >= 32], ids=lambda c: "M%d_K%d_N%d_bs%d" % c)
def test_reference_cases_on_the_prepacked_path(ctx, pkg, oracle, case):
    m, k, n, bs = case
    a, nib, zp, scale = rc.matmul_nbits_case(m, k, n, bs)
    B, Z = pkg.synth.pack_nibbles(nib, bs), pkg.synth.pack_zero_points(zp)
    w = pkg.ops.NBitsWeight(ctx, B, scale.reshape(-1), Z, k, n, bs)
    got = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
    w.destroy()
    want = oracle.matmul_nbits(a, B, scale.reshape(-1), Z, k, n, bs)
    assert close(got, want, RTOL32), worst(got, want)


SHAPES = [  # (M, K, N, block_size, with_zp)
    (1, 1152, 6912, 32, True),    # gemma3 up / gate projection
    (1, 6912, 1152, 32, True),    # down projection
    (1, 1152, 1024, 32, True), (1, 1024, 1152, 32, True), (1, 1152, 256, 32, True),
    (2, 2048, 2560, 128, False),  # qwen-style block 128 without zero points
    (4, 300, 100, 64, True),      # partial last block, N not a multiple of 16
    (5, 4096, 48, 256, True),
    (8, 1152, 512, 32, True), (9, 512, 80, 32, False), (16, 640, 96, 32, True),
    (17, 256, 64, 32, True),      # more than one group of 16 rows
    (3, 7000, 40, 32, True),      # K large enough to split across workgroups
    (8, 6912, 1152, 32, True),
]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "M%d_K%d_N%d_bs%d_zp%d" % s)
def test_seeded_shapes_both_paths(ctx, pkg, oracle, shape):
    m, k, n, bs, with_zp = shape
    B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=100 + n, with_zp=with_zp)
    a = pkg.synth.normal_f32(m * k, 7).reshape(m, k)
    want = oracle.matmul_nbits(a, B, scales, zp, k, n, bs)
    got = pkg.ops.matmul_nbits(ctx, a, B, scales, zp, k, n, bs)
    assert close(got, want, RTOL32), ("direct", worst(got, want))
    w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
    got = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
    w.destroy()
    assert close(got, want, RTOL32), ("gemv", worst(got, want))


@pytest.mark.parametrize("k,n,bs", [(208, 50, 16), (200, 33, 8), (240, 50, 24), (1000, 64, 40), (330, 17, 48)],
                         ids=lambda v: str(v))
def test_small_and_odd_block_sizes(ctx, pkg, oracle, k, n, bs):
    """The reference accepts every block_size that is a positive multiple of 8 (interp.rs:447-464); those
    below 32 or not a power of two run on the kernel that reads the ONNX layout. 13 blocks of 16: odd,
    zero-point rows off word boundaries; 8, 24, 40, 48: blocks that are no power of two, partial last block.
    A handle for such a weight keeps the tensors as they are (the caller's copies may go) and gives the
    same bits; one row, a few and more than 32 (no tiled kernel for them)."""
    B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=3)
    w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
    for m in (1, 3, 40):
        a = pkg.synth.normal_f32(m * k, 8 + m).reshape(m, k)
        got = pkg.ops.matmul_nbits(ctx, a, B, scales, zp, k, n, bs)
        assert close(got, oracle.matmul_nbits(a, B, scales, zp, k, n, bs), RTOL32)
        by_handle = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
        assert np.array_equal(by_handle, got)
    a16 = pkg.synth.normal_f32(5 * k, 9).reshape(5, k).astype(np.float16)
    B16, s16, _ = pkg.synth.nbits_weight(n, k, bs, seed=4, with_zp=False, scale_dtype=np.float16)
    w16 = pkg.ops.NBitsWeight(ctx, B16, s16, None, k, n, bs)
    got = pkg.ops.matmul_nbits(ctx, a16, None, None, None, k, n, bs, weight=w16)
    assert got.dtype == np.float16 and close(got, oracle.matmul_nbits(a16, B16, s16, None, k, n, bs), RTOL16)
    assert w.nbytes == B.size + 4 * scales.size + zp.size
    w.destroy(), w16.destroy()


@pytest.mark.parametrize("shape", [(1, 2048, 2560, 128), (6, 1024, 300, 32), (40, 512, 128, 128)],
                         ids=lambda s: "M%d_K%d_N%d_bs%d" % s)
def test_f16_tensors(ctx, pkg, oracle, shape):
    m, k, n, bs = shape
    B, scales, _ = pkg.synth.nbits_weight(n, k, bs, seed=5, with_zp=False, scale_dtype=np.float16)
    a = pkg.synth.normal_f32(m * k, 9).reshape(m, k).astype(np.float16)
    want = oracle.matmul_nbits(a, B, scales, None, k, n, bs)
    got = pkg.ops.matmul_nbits(ctx, a, B, scales, None, k, n, bs)
    assert got.dtype == np.float16 and close(got, want, RTOL16), ("direct", worst(got, want))
    w = pkg.ops.NBitsWeight(ctx, B, scales, None, k, n, bs)
    got = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
    w.destroy()
    assert got.dtype == np.float16 and close(got, want, RTOL16), ("gemv", worst(got, want))


PREFILL = [  # (M, K, N, block_size, zero points): ragged tiles, partial last stage, every scale grouping
    (100, 1000, 200, 32, True), (130, 384, 131, 64, True), (257, 640, 96, 128, True), (64, 256, 1024, 256, False),
    (17, 72, 16, 32, True),
]


@pytest.mark.parametrize("shape", PREFILL, ids=lambda s: "M%d_K%d_N%d_bs%d_zp%d" % s)
def test_f16_rows_beyond_sixteen_run_the_tiled_kernel(ctx, pkg, oracle, shape):
    """A and the scales share one element type in MatMulNBits, so the scales are f16 here too."""
    m, k, n, bs, with_zp = shape
    B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=41, with_zp=with_zp, scale_dtype=np.float16)
    a = pkg.synth.normal_f32(m * k, 42).reshape(m, k).astype(np.float16)
    want = oracle.matmul_nbits(a, B, scales, zp, k, n, bs)
    w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
    got = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
    w.destroy()
    assert got.dtype == np.float16 and close(got, want, RTOL16), worst(got, want)


WIDE_ROUTES = [  # the 128-row tiles, forced on shapes that would take 64x64: each kernel, alone and with k split over workgroups
    {"HIPC_PREFILL_TILE": 192}, {"HIPC_PREFILL_TILE": 192, "HIPC_PREFILL_SPLIT": 2}, {"HIPC_PREFILL_TILE": 128},
    {"HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_SPLIT": 2},
    {"HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_DIRECT": 0}, {"HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_DIRECT": 0, "HIPC_PREFILL_SPLIT": 3},
    {"HIPC_PREFILL_TILE": 64}, {"HIPC_PREFILL_TILE": 64, "HIPC_PREFILL_DIRECT": 0},
    # two groups of four wavefronts per workgroup, each with half of k (a group without a trip of its own among them)
    {"HIPC_PREFILL_TILE": 192, "HIPC_PREFILL_GROUPS": 2}, {"HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_GROUPS": 2},
    {"HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_GROUPS": 2, "HIPC_PREFILL_SPLIT": 2}, {"HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_GROUPS": 1},
    {"HIPC_PREFILL_TILE": 64, "HIPC_PREFILL_GROUPS": 2}, {"HIPC_PREFILL_TILE": 64, "HIPC_PREFILL_GROUPS": 1},
]


@pytest.mark.parametrize("options", WIDE_ROUTES, ids=lambda v: str(v).replace(" ", ""))
@pytest.mark.parametrize("shape", PREFILL + [(300, 1152, 392, 32, True), (129, 512, 260, 64, False)], ids=lambda s: "M%d_K%d_N%d_bs%d_zp%d" % s)
def test_both_wide_tile_kernels_on_ragged_shapes(ctx, pkg, oracle, shape, options):
    """The kernel that dequantises the weight in the registers of the wavefront that multiplies it (its k order
    inside a stage differs from memory order, for both operands alike) and the one that passes it through LDS:
    ragged rows and columns, a partial last stage, an odd stage count, every scale grouping, zero points."""
    m, k, n, bs, with_zp = shape
    B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=47, with_zp=with_zp, scale_dtype=np.float16)
    a = pkg.synth.normal_f32(m * k, 48).reshape(m, k).astype(np.float16)
    want = oracle.matmul_nbits(a, B, scales, zp, k, n, bs)
    w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
    with ctx.options(**options):
        got = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
    w.destroy()
    assert got.dtype == np.float16 and close(got, want, RTOL16), worst(got, want)


@pytest.mark.parametrize("options", [{"HIPC_PREFILL_TILE": 192}, {"HIPC_PREFILL_TILE": 128}, {"HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_GROUPS": 2}, {"HIPC_PREFILL_TILE": 64},
                                     {"HIPC_PREFILL_TILE": 64, "HIPC_PREFILL_DIRECT": 0}], ids=lambda v: str(v).replace(" ", ""))
@pytest.mark.parametrize("bs,dtype", [(32, np.float16), (128, np.float16), (64, np.float32)], ids=lambda v: str(getattr(v, "__name__", v)))
def test_block_scales_of_zero_and_of_very_different_size(ctx, pkg, oracle, bs, dtype, options):
    """The kernels that keep the weight out of LDS hold their accumulators in units of the open block's scale and
    rescale them when the next block opens: blocks whose scale is 0 (a block of zeros), 1000 times larger or 10000
    times smaller than their neighbours must come out as from the running total the other kernels keep (the
    64x64 tiles are in the list as that control), first block and last block included."""
    m, k, n = 96, 1024, 200
    B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=49, with_zp=True, scale_dtype=dtype)
    sc = scales.reshape(n, -1).copy()
    sc[:, ::3] = 0
    sc[:, 1::7] *= dtype(1000)
    sc[:, 2::5] *= dtype(1e-4)
    sc[5] = 0                      # a column of zeros
    sc[6, :-1] = 0                 # only the last block counts
    sc[7, 1:] = 0                  # only the first
    scales = sc.reshape(scales.shape)
    a = pkg.synth.normal_f32(m * k, 50).reshape(m, k).astype(dtype)
    w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
    with ctx.options(**options):
        got = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
    w.destroy()
    assert np.all(got[:, 5] == 0)
    # Scales seven orders of magnitude apart make sums that cancel: against the float64 product, with the f32
    # accumulation's share stated in units of the row's largest result (the oracle itself is 4e-4 of it away; a
    # rescaled accumulator rounds once more per block than a running total does)
    nib, z = _unpack(B, zp, k, n, bs)
    f64 = rc.matmul_nbits_f64(a, nib, z, scales.reshape(n, -1), bs)
    big = np.abs(f64).max(axis=1, keepdims=True)
    err = np.abs(got.astype(np.float64) - f64)
    if dtype is np.float16:
        assert np.all(err <= 1e-3 + 1e-3 * np.abs(f64) + 1e-6 * big), float((err - 1e-3 * np.abs(f64)).max())
    else:   # f32 rows travel as two f16 rows (22 bits): as in the test of that route
        assert np.all(err <= 2e-5 * big + 1e-3), float((err / big).max())


@pytest.mark.parametrize("shape", [(100, 1000, 200, 32, True), (257, 640, 96, 128, False)], ids=lambda s: "M%d_K%d_N%d_bs%d_zp%d" % s)
def test_many_rows_on_the_onnx_layout_take_the_tiled_kernels(ctx, pkg, oracle, shape):
    """hipc_matmul_nbits (the reference's own calling convention: the ONNX tensors on every call) with more rows
    than the decode kernels take writes the tiled form into scratch memory and runs the kernels of the prepacked
    path: the same bits as a handle gives, f16 and f32 rows, twice in a row with different weights (the scratch
    block is reused)."""
    m, k, n, bs, with_zp = shape
    for seed, dtype in ((61, np.float32), (62, np.float16), (63, np.float32)):   # (scales in the activations' type, as the operator has them)
        B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=seed, with_zp=with_zp, scale_dtype=dtype)
        rows = pkg.synth.normal_f32(m * k, seed + 10).reshape(m, k).astype(dtype)
        w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
        got = pkg.ops.matmul_nbits(ctx, rows, B, scales, zp, k, n, bs)
        by_handle = pkg.ops.matmul_nbits(ctx, rows, None, None, None, k, n, bs, weight=w)
        w.destroy()
        assert got.dtype == dtype and np.array_equal(got, by_handle)
        want = oracle.matmul_nbits(rows, B, scales, zp, k, n, bs)
        assert close(got, want, RTOL32 if dtype == np.float32 else RTOL16), worst(got, want)


F32_PREFILL = [  # (M, K, N, block_size, zero points)
    (100, 1000, 200, 32, True), (130, 384, 131, 64, True), (257, 640, 96, 128, False), (33, 72, 16, 32, True),
    (512, 2048, 2560, 128, False),
]


F32_ROUTES = [  # the default; the two terms of a row as the two row blocks of a wavefront (128 x 128 and 128 x 192 tiles, two k
    # groups per workgroup, k split over workgroups, a forced 64-row tile that such rows cannot take); the kernel
    # with both operands in LDS, whose 2 M result rows a last launch adds up
    {}, {"HIPC_PREFILL_TILE": 128}, {"HIPC_PREFILL_TILE": 192}, {"HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_GROUPS": 2},
    {"HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_SPLIT": 2}, {"HIPC_PREFILL_TILE": 192, "HIPC_PREFILL_GROUPS": 2, "HIPC_PREFILL_SPLIT": 2},
    {"HIPC_PREFILL_TILE": 64}, {"HIPC_PREFILL_DIRECT": 0}, {"HIPC_PREFILL_DIRECT": 0, "HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_SPLIT": 2},
]


@pytest.mark.parametrize("options", F32_ROUTES, ids=lambda v: str(v).replace(" ", ""))
@pytest.mark.parametrize("shape", F32_PREFILL, ids=lambda s: "M%d_K%d_N%d_bs%d_zp%d" % s)
def test_f32_rows_beyond_thirty_two_run_the_tiled_kernel(ctx, pkg, oracle, shape, options):
    """More than 32 rows of f32 activations (the reference's own element type, interp.rs:6455-6472) go through
    the tiled matrix-core kernel as two f16 rows each, scaled per row by a power of two: against the oracle at
    the operator's f32 tolerance, against the float64 product at 2e-5 of the row's largest output, and equal
    in quality to the decode kernel's route (the same rows, 16 at a time)."""
    m, k, n, bs, with_zp = shape
    B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=45, with_zp=with_zp)
    a = pkg.synth.normal_f32(m * k, 46).reshape(m, k)
    a[0] *= np.float32(3.0e7)      # a row far beyond the f16 range, one far below it, one of zeros
    a[1] *= np.float32(1.0e-9)
    a[2] = 0
    want = oracle.matmul_nbits(a, B, scales, zp, k, n, bs)
    w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
    with ctx.options(**options):
        got = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
    by_rows = np.concatenate([pkg.ops.matmul_nbits(ctx, a[i:i + 16], None, None, None, k, n, bs, weight=w) for i in range(0, m, 16)])
    w.destroy()
    assert got.dtype == np.float32 and got.shape == (m, n)
    # rows 0 and 1 are out of the absolute tolerance's scale: compare them relative to their own size
    scale = np.maximum(np.abs(want).max(axis=1, keepdims=True), 1e-30)
    assert np.all(np.abs(got - want) <= (1e-3 + 1e-4 * np.abs(want)) * np.maximum(scale / np.abs(want[3:]).max(), 1e-30) + 1e-4 * scale), worst(got, want)
    nib, z = _unpack(B, zp if zp is not None else np.full((n, (-(-k // bs) + 1) // 2), 0x88, np.uint8), k, n, bs)
    f64 = rc.matmul_nbits_f64(a, nib, z, scales.reshape(n, -1), bs)
    big = np.abs(f64).max(axis=1, keepdims=True)
    assert np.all(np.abs(got - f64) <= 2e-5 * np.maximum(big, 1e-300)), float(np.max(np.abs(got - f64) / np.maximum(big, 1e-300)))
    assert np.all(np.abs(got - f64) <= np.abs(by_rows - f64).max(axis=1, keepdims=True) * 1.5 + 2e-6 * big)
    assert np.all(got[2] == 0)


@pytest.mark.parametrize("options", [{}, {"HIPC_PREFILL_TILE": 64}, {"HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_GROUPS": 2}, {"HIPC_PREFILL_TILE": 192},
                                     {"HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_SPLIT": 2}, {"HIPC_PREFILL_DIRECT": 0}], ids=lambda v: str(v).replace(" ", ""))
@pytest.mark.parametrize("level", [2, 3, 4])
@pytest.mark.parametrize("shape", F32_PREFILL, ids=lambda s: "M%d_K%d_N%d_bs%d_zp%d" % s)
def test_f32_rows_at_a_level_that_allows_f16_activations(ctx, pkg, oracle, shape, level, options):
    """accuracy_level 2, 3 and 4 allow the activations to be reduced to f16, bf16 or int8 (the reference never reads
    the attribute and computes in f32). More than 32 rows of f32 then travel as ONE f16 row each: the row times the
    power of two that puts its largest value into [2^14, 2^15), rounded to f16 (11 bits of every value, whatever the
    row's size). The result is the operator on exactly those rounded rows, at the f32 tolerance -- and so within
    what each of the three levels permits."""
    m, k, n, bs, with_zp = shape
    B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=45, with_zp=with_zp)
    a = pkg.synth.normal_f32(m * k, 46).reshape(m, k)
    a[0] *= np.float32(3.0e7)
    a[1] *= np.float32(1.0e-9)
    a[2] = 0
    mx = np.abs(a).max(axis=1, keepdims=True)
    e = np.where(mx > 0, np.floor(np.log2(np.maximum(mx, np.float32(1e-30)))) - 14, 0).astype(np.int32)
    rounded = np.ldexp(np.ldexp(a, -e).astype(np.float16).astype(np.float32), e).astype(np.float32)
    assert np.all(np.abs(rounded - a) <= 2.0 ** -11 * mx)
    want = oracle.matmul_nbits(rounded, B, scales, zp, k, n, bs)
    w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
    with ctx.options(**options):
        got = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, accuracy_level=level, weight=w)
    w.destroy()
    assert got.dtype == np.float32 and got.shape == (m, n)
    scale = np.maximum(np.abs(want).max(axis=1, keepdims=True), 1e-30)
    assert np.all(np.abs(got - want) <= (1e-3 + 1e-4 * np.abs(want)) * np.maximum(scale / np.abs(want[3:]).max(), 1e-30) + 1e-4 * scale), worst(got, want)
    assert np.all(got[2] == 0)


@pytest.mark.parametrize("options", [{}, {"HIPC_PREFILL_TILE": 128, "HIPC_PREFILL_SPLIT": 2}, {"HIPC_PREFILL_TILE": 192}, {"HIPC_PREFILL_DIRECT": 0}],
                         ids=lambda v: str(v).replace(" ", ""))
@pytest.mark.parametrize("shape", F32_PREFILL, ids=lambda s: "M%d_K%d_N%d_bs%d_zp%d" % s)
def test_f32_rows_with_f32_pinned(ctx, pkg, oracle, shape, options):
    """accuracy_level 1 pins f32: more than 32 rows travel as THREE f16 rows each (every bit of the row's values
    beside its power of two) through the tiled kernel, and a launch adds the three results. Against the oracle at
    the operator's tolerance; against the float64 product no worse than the default's two terms, and within what f32
    accumulation leaves."""
    m, k, n, bs, with_zp = shape
    B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=45, with_zp=with_zp)
    a = pkg.synth.normal_f32(m * k, 46).reshape(m, k)
    a[0] *= np.float32(3.0e7)
    a[1] *= np.float32(1.0e-9)
    a[2] = 0
    want = oracle.matmul_nbits(a, B, scales, zp, k, n, bs)
    w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
    with ctx.options(**options):
        got = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, accuracy_level=1, weight=w)
        two = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
    w.destroy()
    scale = np.maximum(np.abs(want).max(axis=1, keepdims=True), 1e-30)
    assert np.all(np.abs(got - want) <= (1e-3 + 1e-4 * np.abs(want)) * np.maximum(scale / np.abs(want[3:]).max(), 1e-30) + 1e-4 * scale), worst(got, want)
    nib, z = _unpack(B, zp if zp is not None else np.full((n, (-(-k // bs) + 1) // 2), 0x88, np.uint8), k, n, bs)
    f64 = rc.matmul_nbits_f64(a, nib, z, scales.reshape(n, -1), bs)
    big = np.maximum(np.abs(f64).max(axis=1, keepdims=True), 1e-300)
    e3, e2 = np.abs(got - f64) / big, np.abs(two - f64) / big
    assert e3.max() <= 2e-5, float(e3.max())
    assert e3.max() <= e2.max() * 1.05 + 1e-7, (float(e3.max()), float(e2.max()))
    assert np.all(got[2] == 0)


@pytest.mark.parametrize("kn", [(2048, 11008), (11008, 2048), (2048, 2560)], ids=lambda s: "K%d_N%d" % s)
def test_prefill_configuration_full_size(ctx, pkg, oracle, kn):
    """512 rows of f16 activations against block-128 symmetric weights with f16 scales (no zero
    points: 8 is implied), the three linears of the prefill configuration at full size."""
    k, n = kn
    m, bs = 512, 128
    B, scales, _ = pkg.synth.fast_nbits_weight(n, k, bs, seed=43, with_zp=False, scale_dtype=np.float16)
    a = pkg.synth.normal_f32(m * k, 44).reshape(m, k).astype(np.float16)
    want = oracle.matmul_nbits(a, B, scales, None, k, n, bs)
    w = pkg.ops.NBitsWeight(ctx, B, scales, None, k, n, bs)
    got = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
    # linearity in A, a size-independent property: f(2a) == 2 f(a) exactly (a power of two scales every product, every
    # partial sum and the rounding to a normal f16 alike)
    got2 = pkg.ops.matmul_nbits(ctx, (2 * a).astype(np.float16), None, None, None, k, n, bs, weight=w)
    w.destroy()
    assert close(got, want, RTOL16), worst(got, want)
    normal = np.abs(got.astype(np.float32)) >= 2.0 ** -13   # (a subnormal f16 result has no spare bit to double into)
    assert np.array_equal(got2.astype(np.float32)[normal], 2 * got.astype(np.float32)[normal]) and normal.mean() > 0.99


def test_unembedding_width_full_size(ctx, pkg, oracle):
    """lm_head of the decoder configuration: K = 1152, N = 262144, every column checked."""
    k, n, bs = 1152, 262144, 32
    B, scales, zp = pkg.synth.fast_nbits_weight(n, k, bs, seed=17)
    a = pkg.synth.normal_f32(k, 18).reshape(1, k)
    want = oracle.matmul_nbits(a, B, scales, zp, k, n, bs)
    w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
    got = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
    assert close(got, want, RTOL32), worst(got, want)
    # linearity in A, a size-independent property: f(2a) == 2 f(a) exactly (power-of-two scaling)
    got2 = pkg.ops.matmul_nbits(ctx, 2 * a, None, None, None, k, n, bs, weight=w)
    assert np.array_equal(got2, 2 * got)
    w.destroy()


def test_refusals_and_short_buffers(ctx, pkg):
    k, n, bs = 128, 16, 32
    B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=1)
    a = np.zeros((1, k), np.float32)
    with pytest.raises(pkg.HipComputeError) as e:   # the operator defines levels 0..4
        pkg.ops.matmul_nbits(ctx, a, B, scales, zp, k, n, bs, accuracy_level=5)
    assert e.value.code == 2
    with pytest.raises(pkg.HipComputeError) as e:   # the weight is short for N (interp.rs:6465-6472)
        pkg.ops.matmul_nbits(ctx, a, B[: n - 1], scales, zp, k, n, bs)
    assert e.value.code == 1 and "short" in e.value.message
    with pytest.raises(pkg.HipComputeError) as e:   # not a multiple of 8: a packed word would straddle two blocks
        pkg.ops.matmul_nbits(ctx, a, B, scales, zp, k, n, 20)
    assert e.value.code == 1
    y = pkg.ops.matmul_nbits(ctx, np.zeros((0, k), np.float32), B, scales, zp, k, n, bs)   # no rows: a no-op
    assert y.shape == (0, n)


def _unpack(B, zp, k, n, bs):
    nb = -(-k // bs)
    flat = B.reshape(n, -1)
    nib = np.empty((n, nb * bs), np.uint8)
    nib[:, 0::2], nib[:, 1::2] = flat & 15, flat >> 4
    z = np.empty((n, 2 * zp.shape[1]), np.uint8)
    z[:, 0::2], z[:, 1::2] = zp & 15, zp >> 4
    return nib[:, :k], z[:, :nb]


@pytest.mark.parametrize("shape", [(1, 1152, 6912), (1, 6912, 1152), (8, 1152, 512), (1, 1152, 32768 + 48)], ids=lambda s: "M%d_K%d_N%d" % s)
def test_accuracy_levels(ctx, pkg, oracle, shape):
    """accuracy_level 0 (unset), 2, 3 and 4 (a lower bound: the reference computes every level in f32) let
    an f32 activation enter the matrix cores as two bf16 terms; 1 pins f32 and sends all 24 bits (three terms). The last shape has more than 2048 column tiles, so
    its one row takes the wide streaming kernel (the unembedding's route) and level 1 that kernel's
    three-term instance. Every level meets the operator's tolerance
    against the oracle; level 1 is held to a tighter bound against the float64 product -- 2e-5 of
    the row's largest output, what the f32 accumulation of the +128-biased block dots leaves --
    and must not be worse than the default."""
    m, k, n = shape
    bs = 32
    B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=300 + n)
    a = pkg.synth.normal_f32(m * k, 301).reshape(m, k)
    want = oracle.matmul_nbits(a, B, scales, zp, k, n, bs)
    nib, z = _unpack(B, zp, k, n, bs)
    f64 = rc.matmul_nbits_f64(a, nib, z, scales.reshape(n, -1), bs)
    w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
    err = {}
    for level in (0, 1, 2, 3, 4):
        got = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, accuracy_level=level, weight=w)
        assert close(got, want, RTOL32), (level, worst(got, want))
        err[level] = float(np.max(np.abs(got - f64)))
    w.destroy()
    assert err[1] <= 2e-5 * float(np.max(np.abs(f64))), err
    assert err[1] <= err[0] * 1.05 + 1e-7, err
    assert err[2] == err[0] and err[3] == err[0] and err[4] == err[0], err     # the same kernel instance as the default


@pytest.mark.parametrize("shape", [(1, 1152, 6912, 32, True), (1, 6912, 1152, 32, True), (1, 2048, 2560, 128, False),
                                   (1, 300, 100, 64, True), (1, 1024, 48, 32, True)], ids=lambda s: "M%d_K%d_N%d_bs%d_zp%d" % s)
def test_one_row_on_the_streaming_kernel(ctx, pkg, oracle, shape):
    """One f32 row takes the kernel built for latency by default; with the HIPC_GEMV_LEAN option at 0 the
    same product runs on the streaming kernel: both against the oracle, and against each other."""
    m, k, n, bs, with_zp = shape
    B, scales, zp = pkg.synth.nbits_weight(n, k, bs, seed=400 + n, with_zp=with_zp)
    a = pkg.synth.normal_f32(m * k, 401).reshape(m, k)
    want = oracle.matmul_nbits(a, B, scales, zp, k, n, bs)
    w = pkg.ops.NBitsWeight(ctx, B, scales, zp, k, n, bs)
    lean = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
    with ctx.options(HIPC_GEMV_LEAN=0):
        streaming = pkg.ops.matmul_nbits(ctx, a, None, None, None, k, n, bs, weight=w)
    w.destroy()
    assert close(lean, want, RTOL32), ("lean", worst(lean, want))
    assert close(streaming, want, RTOL32), ("streaming", worst(streaming, want))
    assert close(lean, streaming, RTOL32)
