"""Host-side logic that needs no GPU: the library loads and exports every declared symbol, the
refusal envelope of the QLinear operators, geometry, packers and the seeded generators."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "hipcompute.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hipc_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg.load_library()
    declared = _declared_symbols()
    assert len(declared) >= 30
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/hipcompute.h but not exported"
    from onnx_vulkan_rs_amd.runtime import SIGNATURES
    assert sorted(SIGNATURES) == declared, "the ctypes table and the header disagree"
    assert lib.hipc_version().startswith(b"hipcompute")


def test_geometry_helpers_need_no_device(pkg, oracle):
    lib = pkg.load_library()
    g = pkg.ConvGeom.make((1, 192, 1, 4096), (192, 192, 1, 7), dilations=(1, 5), pads=(0, 15, 0, 15))
    assert pkg.ops.conv_out_shape(lib, g) == (1, 192, 1, 4096)
    g = pkg.ConvGeom.make((1, 3, 5, 5), (8, 3, 7, 7))
    with pytest.raises(ValueError):
        pkg.ops.conv_out_shape(lib, g)
    for args in [(4096, 7, 1, 5), (224, 7, 2, 1), (15, 3, 2, 2), (10, 1, 1, 1)]:
        for upper in (True, False):
            b, e = C.c_int64(), C.c_int64()
            lib.hipc_same_pads(*args, int(upper), C.byref(b), C.byref(e))
            assert (b.value, e.value) == oracle.same_pads(*args, upper=upper)


def _qconv(pkg, n_inputs=9):
    names = ["x", "x_scale", "x_zp", "w", "w_scale", "w_zp", "y_scale", "y_zp", "bias"][:n_inputs]
    return pkg.graph.NodeIr("QLinearConv", names, ["out"])


def _qconv_params(ch=8):
    return {"x_scale": np.zeros((), np.float32), "x_zp": np.array(0, np.uint8), "w_scale": np.zeros(ch, np.float32),
            "w_zp": np.zeros(ch, np.int8), "y_scale": np.zeros((), np.float32), "y_zp": np.array(7, np.uint8),
            "bias": np.zeros(ch, np.int32)}


def test_refusal_envelope_of_the_qlinear_operators(pkg):
    """The cases of crates/onnx-vulkan-core/tests/qlinear_coverage.rs:76-176."""
    g = pkg.graph
    full, no_bias = _qconv(pkg), _qconv(pkg, 8)
    assert g.is_implemented_node(full) and g.unsupported_quantization(full, _qconv_params()) is None
    assert g.is_implemented_node(no_bias) and g.unsupported_quantization(no_bias, _qconv_params()) is None
    p = _qconv_params()
    p["w_zp"] = np.array([0, 0, 3, 0, 0, 0, 0, 0], np.int8)
    assert "per-channel zero point" in g.unsupported_quantization(full, p)
    p = _qconv_params()
    p["w_scale"], p["w_zp"] = np.zeros((), np.float32), np.array(9, np.int8)
    assert g.unsupported_quantization(full, p) is None
    p = _qconv_params()
    p["y_scale"] = np.zeros(4, np.float32)
    assert "per-tensor" in g.unsupported_quantization(full, p)
    p = _qconv_params()
    del p["x_scale"]
    assert "not a constant" in g.unsupported_quantization(full, p)
    p = _qconv_params()
    p["bias"] = np.zeros(8, np.float32)
    assert "int32" in g.unsupported_quantization(full, p)
    mm = g.NodeIr("QLinearMatMul", ["a", "a_scale", "a_zp", "b", "b_scale", "b_zp", "y_scale", "y_zp"], ["out"])
    base = {"a_scale": np.zeros((), np.float32), "a_zp": np.array(128, np.uint8), "y_scale": np.zeros((), np.float32),
            "y_zp": np.array(64, np.uint8)}
    assert g.unsupported_quantization(mm, dict(base, b_scale=np.zeros((), np.float32), b_zp=np.array(0, np.int8))) is None
    assert g.unsupported_quantization(mm, dict(base, b_scale=np.zeros(16, np.float32), b_zp=np.zeros(16, np.int8))) is None


def test_matmul_nbits_node_forms(pkg):
    g = pkg.graph
    node = g.NodeIr("MatMulNBits", ["a", "q", "s", "zp"], ["y"], {"K": 64, "N": 8, "bits": 4, "block_size": 32},
                    domain="com.microsoft")
    assert g.is_implemented_node(node)
    assert g.is_implemented_node(g.NodeIr("MatMulNBits", ["a", "q", "s"], ["y"], dict(node.attrs)))  # zp omitted
    assert not g.is_implemented_node(g.NodeIr("MatMulNBits", ["a", "q", "s", "zp", "g_idx"], ["y"], dict(node.attrs)))
    assert not g.is_implemented_node(g.NodeIr("MatMulNBits", ["a", "q", "s", "zp", "", "bias"], ["y"], dict(node.attrs)))
    assert not g.is_implemented_node(g.NodeIr("MatMulNBits", ["a", "q", "s"], ["y"], dict(node.attrs, bits=8)))
    for bs, ok in ((8, True), (24, True), (40, True), (20, False), (0, False)):   # any positive multiple of 8
        assert g.is_implemented_node(g.NodeIr("MatMulNBits", ["a", "q", "s", "zp"], ["y"], dict(node.attrs, block_size=bs))) == ok
    assert not g.is_implemented_node(g.NodeIr("Softmax", ["a"], ["y"]))


def test_conv_geometry_lifts_1d_and_resolves_auto_pad(pkg):
    g = pkg.graph
    node = g.NodeIr("QLinearConv", [], [], {"dilations": [3], "pads": [9, 9]})
    geom = g.conv_geometry(node, (1, 192, 4096), (192, 192, 7))
    assert (geom.h, geom.w, geom.kh, geom.kw, geom.dil_h, geom.dil_w) == (1, 4096, 1, 7, 1, 3)
    assert (geom.pad_top, geom.pad_left, geom.pad_bottom, geom.pad_right) == (0, 9, 0, 9)
    node = g.NodeIr("ConvInteger", [], [], {"auto_pad": "SAME_UPPER", "strides": [2, 2]})
    geom = g.conv_geometry(node, (1, 3, 224, 224), (64, 3, 7, 7))
    assert (geom.pad_top, geom.pad_left, geom.pad_bottom, geom.pad_right) == (2, 2, 3, 3)


def test_packers_round_trip(pkg):
    rng = np.random.default_rng(0)
    q = rng.integers(0, 16, (5, 100)).astype(np.uint8)
    B = pkg.synth.pack_nibbles(q, 32)
    assert B.shape == (5, 4, 16)
    flat = B.reshape(5, -1)
    assert np.array_equal(flat[:, :50] & 15, q[:, 0::2]) and np.array_equal(flat[:, :50] >> 4, q[:, 1::2])
    z = rng.integers(0, 16, (5, 7)).astype(np.uint8)
    Z = pkg.synth.pack_zero_points(z)
    assert Z.shape == (5, 4) and np.array_equal(Z[:, :3] >> 4, z[:, 1::2]) and np.array_equal(Z & 15, z[:, 0::2])


def test_lcg_matches_the_scalar_recurrence(pkg):
    s = 12345
    got = pkg.synth.lcg_states(3 + (1 << 20), s)     # crosses a chunk boundary
    for i in list(range(5)):
        s = (s * 6364136223846793005 + 1442695040888963407) % (1 << 64)
        assert int(got[i]) == s
    s = 12345
    for i in range(3 + (1 << 20)):
        s = (s * 6364136223846793005 + 1442695040888963407) & 0xFFFFFFFFFFFFFFFF
    assert int(got[-1]) == s
    v = pkg.synth.uniform_ints(100000, 5, -127, 127)
    assert v.min() == -127 and v.max() == 127 and abs(v.mean()) < 1.0
    n = pkg.synth.normal_f32(200000, 6)
    assert abs(n.mean()) < 0.01 and abs(n.std() - 1) < 0.01


def test_missing_gpu_is_an_error_not_a_fallback(pkg):
    try:
        c = pkg.Context(0)
    except pkg.HipComputeError as e:
        assert e.code == 3
        return
    c.close()
    pytest.skip("a GPU is present")


def test_shared_index_arithmetic_on_the_host(tmp_path):
    """The chunk split of the decode attention and the read-ahead helpers' tile runs are plain index
    arithmetic in headers that host and device code share: tests/host/geometry_checks.cpp compiles
    them for the host alone and checks their invariants (chunks cover the visible context, every tile
    is read ahead once, from inside its array, by a helper of the consumer's XCD class)."""
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = str(tmp_path / "geometry_checks")
    subprocess.run([hipcc, "--cuda-host-only", "-x", "hip", "-std=c++17", "-O1", "-I", os.path.join(root, "onnx-vulkan-rs_amd", "csrc"),
                    os.path.join(root, "tests", "host", "geometry_checks.cpp"), "-o", exe], check=True, capture_output=True)
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout + out.stderr


def test_the_rust_binding_declares_every_entry_point():
    """crates/hip-compute/src/sys.rs cannot be compiled here (no Rust toolchain); at least it must name
    exactly the functions the header declares, with as many parameters each."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    header = re.sub(r"/\*.*?\*/", "", open(os.path.join(root, "include", "hipcompute.h")).read(), flags=re.S)
    rust = re.sub(r"//[^\n]*", "", open(os.path.join(root, "crates", "hip-compute", "src", "sys.rs")).read())
    c_protos = {m.group(1): m.group(2) for m in re.finditer(r"\b(hipc_\w+)\(([^;{]*)\);", header)}
    r_protos = {m.group(1): m.group(2) for m in re.finditer(r"pub fn (hipc_\w+)\(([^;{]*?)\)\s*(?:->[^;]*)?;", rust, flags=re.S)}
    assert sorted(c_protos) == sorted(r_protos)
    for name, args in c_protos.items():
        n_c = 0 if args.strip() in ("", "void") else args.count(",") + 1
        n_r = len([a for a in r_protos[name].split(",") if a.strip()])
        assert n_c == n_r, (name, n_c, n_r)


def test_the_library_carries_the_build_id_of_the_sources_beside_it(pkg):
    """hipc_version() ends in a hash over the sources and headers the library was compiled from, and
    load_library() refuses a library whose id is not the tree's (a stale object once hid a fix)."""
    rt = pkg.runtime
    lib = rt.load_library()
    built = lib.hipc_version().decode().rsplit(" ", 1)[-1]
    assert re.fullmatch(r"[0-9a-f]{16}", built), built
    assert built == rt.source_build_id()


def test_a_stale_library_is_refused(pkg, monkeypatch):
    rt = pkg.runtime
    rt.load_library()
    monkeypatch.setattr(rt, "_lib", None)
    monkeypatch.setattr(rt, "source_build_id", lambda: "0123456789abcdef")
    with pytest.raises(rt.HipComputeError, match="stale"):
        rt.load_library()


def test_kernel_addresses_on_the_cpu_model(tmp_path):
    """tests/host/decoder_model.cpp: the decode step's kernel sources compiled as plain C++ (buffer loads
    replaced by a checker that applies the hardware's range rule, everything else under
    AddressSanitizer) and run thread by thread with the read-ahead helper rows on: whole steps at the
    positions around every chunk boundary for the shapes of the GPU tests and gemma3-1b's, and the
    position-dependent launches of gemma3-1b's shape over the whole cache. (`decoder_model sweep` runs
    every position of every shape; it takes a few minutes and is not part of this suite.)"""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = str(tmp_path / "model")
    build = subprocess.run(["make", "-C", os.path.join(root, "tests", "host"), "-j", "4", "OUT=" + out], capture_output=True, text=True)
    assert build.returncode == 0, build.stdout[-2000:] + build.stderr[-2000:]
    run = subprocess.run([os.path.join(out, "decoder_model"), "quick", "8"], capture_output=True, text=True)
    assert run.returncode == 0 and run.stdout.strip().endswith("ok"), run.stdout[-2000:] + run.stderr[-2000:]
    # the same build holds the int8 operators' model (tests/host/int8_model.cpp): every matrix-product route -- the
    # kernels that step along k in a buffer load's scalar offset among them -- and the convolution routes, on tiny,
    # ragged and aligned shapes and on the benchmark's, with operands of exactly the operator's size
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    run = subprocess.run([os.path.join(out, "int8_model")], capture_output=True, text=True, env=env)
    assert run.returncode == 0 and run.stdout.strip().endswith("ok"), run.stdout[-2000:] + run.stderr[-2000:]
    # and the tiled MatMulNBits kernels' (tests/host/prefill_model.cpp): every instance, scale grouping and k split,
    # f16 and f32 rows, on ragged shapes with operands of exactly the operator's size
    run = subprocess.run([os.path.join(out, "prefill_model")], capture_output=True, text=True, env=env)
    assert run.returncode == 0 and run.stdout.strip().endswith("ok"), run.stdout[-2000:] + run.stderr[-2000:]
