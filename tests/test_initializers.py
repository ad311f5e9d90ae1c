"""ONNX initializers -> raw bytes (the data format in front of the prepack calls), on the CPU.

Golden data: `tests/golden/onnx/{mixed,external}.onnx` and `external.weights` are the data files of the
reference's own frontend tests (crates/onnx-vulkan-frontend/tests/models/, generated there with the `onnx`
package), and the expected bytes below are the literals those tests assert
(crates/onnx-vulkan-frontend/tests/frontend.rs:30-81, 141-168): what `numpy_helper.to_array(t).tobytes()`
says, so the yardstick is the ONNX implementation. The remaining cases build TensorProto messages with a
ten-line wire-format writer and check them against `struct.pack`.
"""
import os
import struct

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "onnx")

# frontend.rs:34-58 (bytes) and :66-80 (dtype, shape)
EXPECTED = {
    "w_raw": (1, (2, 2), [0, 0, 192, 63, 0, 0, 32, 192, 0, 0, 0, 63, 0, 0, 64, 64]),
    "w_typed": (1, (3,), [0, 0, 128, 63, 0, 0, 0, 64, 0, 0, 64, 64]),
    "i64": (7, (2,), [249, 255, 255, 255, 255, 255, 255, 255, 9, 0, 0, 0, 0, 0, 0, 0]),
    "u8": (2, (4,), [0, 1, 254, 255]),
    "i8": (3, (3,), [128, 0, 127]),
    "bool_": (9, (3,), [1, 0, 1]),
    "f16": (10, (2,), [192, 115, 0, 122]),
}


def _read(name):
    with open(os.path.join(GOLDEN, name), "rb") as f:
        return f.read()


def test_every_storage_form_decodes_to_the_bytes_onnx_declares(pkg):
    inits = pkg.initializers.model_initializers(_read("mixed.onnx"))
    assert sorted(inits) == sorted(EXPECTED)
    for name, (dtype, shape, data) in EXPECTED.items():
        got_dtype, got_shape, payload = inits[name]
        assert (got_dtype, got_shape, list(payload)) == (dtype, shape, data), name
    assert pkg.initializers.as_array(*inits["i64"]).tolist() == [-7, 9]
    assert pkg.initializers.as_array(*inits["f16"]).dtype == np.float16


def test_external_weights_give_the_same_initializers(pkg):
    inline = pkg.initializers.model_initializers(_read("mixed.onnx"))
    external = pkg.initializers.model_initializers(_read("external.onnx"), GOLDEN)
    assert external == inline


def test_external_weights_without_a_base_directory_are_refused(pkg):
    with pytest.raises(pkg.HipComputeError) as e:
        pkg.initializers.model_initializers(_read("external.onnx"), None)
    assert "w_raw" in str(e.value)          # the error must say which one (frontend.rs:160-163)


def test_a_file_that_is_not_a_model_is_refused(pkg):
    with pytest.raises(pkg.HipComputeError):
        pkg.initializers.model_initializers(b"this is not an ONNX protobuf")


# ---- a minimal wire-format writer for the cases the fixtures do not hold
def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        out.append((v & 0x7f) | (0x80 if v > 0x7f else 0))
        v >>= 7
        if not v:
            return bytes(out)


def _field(number, wire, payload):
    return _varint(number << 3 | wire) + (_varint(len(payload)) + payload if wire == 2 else payload)


def _tensor(name, dtype, dims, **fields):
    msg = b"".join(_field(1, 0, _varint(d)) for d in dims) + _field(2, 0, _varint(dtype)) + _field(8, 2, name.encode())
    for key, value in fields.items():
        number = {"raw": 9, "floats": 4, "int32s": 5, "int64s": 7, "doubles": 10, "uint64s": 11}[key.removesuffix("_unpacked")]
        if key == "raw":
            msg += _field(9, 2, value)
        elif key.endswith("_unpacked"):                       # one element per key instead of a packed run
            wire = {4: 5, 10: 1}.get(number, 0)
            enc = {5: lambda v: struct.pack("<f", v), 1: lambda v: struct.pack("<d", v), 0: _varint}[wire]
            msg += b"".join(_field(number, wire, enc(v)) for v in value)
        elif number == 4:
            msg += _field(4, 2, struct.pack(f"<{len(value)}f", *value))
        elif number == 10:
            msg += _field(10, 2, struct.pack(f"<{len(value)}d", *value))
        else:
            msg += _field(number, 2, b"".join(_varint(v) for v in value))
    return msg


def _external(name, dtype, dims, **entries):
    msg = _tensor(name, dtype, dims)
    for k, v in entries.items():
        msg += _field(13, 2, _field(1, 2, k.encode()) + _field(2, 2, str(v).encode()))
    return msg + _field(14, 0, _varint(1))


def test_typed_fields_take_the_width_of_the_dtype(pkg):
    rd = pkg.initializers.read_initializer
    assert rd(_tensor("d", 11, [2], doubles=[1.5, -2.0]))[3] == struct.pack("<2d", 1.5, -2.0)
    assert rd(_tensor("d", 11, [2], doubles_unpacked=[1.5, -2.0]))[3] == struct.pack("<2d", 1.5, -2.0)
    assert rd(_tensor("f", 1, [2], floats_unpacked=[0.25, 3.0]))[3] == struct.pack("<2f", 0.25, 3.0)
    assert rd(_tensor("i", 6, [3], int32s=[-1, 2, 1 << 30]))[3] == struct.pack("<3i", -1, 2, 1 << 30)
    assert rd(_tensor("i", 6, [2], int32s_unpacked=[-5, 7]))[3] == struct.pack("<2i", -5, 7)
    assert rd(_tensor("h", 5, [2], int32s=[-2, 300]))[3] == struct.pack("<2h", -2, 300)            # int16
    assert rd(_tensor("b", 16, [1], int32s=[0x3f80]))[3] == b"\x80\x3f"                              # bfloat16 1.0
    assert rd(_tensor("u", 12, [2], uint64s=[7, 0xfffffffe]))[3] == struct.pack("<2I", 7, 0xfffffffe)   # uint32 travels in uint64_data
    assert rd(_tensor("q", 13, [1], uint64s=[(1 << 64) - 2]))[3] == struct.pack("<Q", (1 << 64) - 2)
    name, dtype, shape, payload = rd(_tensor("scalar", 1, [], floats=[6.0]))
    assert (name, dtype, shape, payload) == ("scalar", 1, (), struct.pack("<f", 6.0))              # the Constant of frontend.rs:131-137
    # raw_data wins over the typed fields; an empty tensor is empty
    assert rd(_tensor("r", 2, [2], raw=b"\x01\x02", int32s=[9, 9]))[3] == b"\x01\x02"
    assert rd(_tensor("e", 1, [0]))[3] == b""


def test_unreadable_and_malformed_tensors(pkg):
    rd, Err = pkg.initializers.read_initializer, pkg.HipComputeError
    with pytest.raises(Err) as e:
        rd(_tensor("s", 8, [1]) + _field(6, 2, b"text"))        # STRING: no numeric payload
    assert e.value.code == 2 and "dtype 8" in str(e.value)
    good = _tensor("w", 1, [2], floats=[1.0, 2.0])
    with pytest.raises(Err) as e:
        rd(good[:-3])                                            # cut inside the packed run
    assert e.value.code == 1
    with pytest.raises(Err):
        rd(_tensor("w", 1, [1]) + _field(4, 2, b"\x00\x00\x80"))  # three bytes of float_data
    with pytest.raises(Err):
        rd(b"\xff\xff\xff\xff\xff\xff\xff\xff\xff\xff\xff")        # a varint that never ends


def test_external_slices_and_their_refusals(pkg, tmp_path):
    rd, Err = pkg.initializers.read_initializer, pkg.HipComputeError
    blob = bytes(range(64))
    (tmp_path / "w.bin").write_bytes(blob)
    (tmp_path / "sub").mkdir()
    (tmp_path / "sub" / "w2.bin").write_bytes(blob[::-1])
    base = str(tmp_path)
    assert rd(_external("a", 2, [8], location="w.bin", offset=16, length=8), base)[3] == blob[16:24]
    assert rd(_external("a", 2, [48], location="w.bin", offset=16), base)[3] == blob[16:]        # no length: to the end of the file
    assert rd(_external("a", 2, [64], location="w.bin"), base)[3] == blob
    assert rd(_external("a", 2, [4], location="sub/w2.bin", length=4), base)[3] == blob[::-1][:4]
    for location in ("../w.bin", "/etc/passwd", "sub/../w.bin", "./w.bin", ""):
        with pytest.raises(Err) as e:
            rd(_external("a", 2, [1], location=location, length=1), base)
        assert "not relative" in str(e.value) or "location" in str(e.value), location
    with pytest.raises(Err) as e:
        rd(_external("a", 2, [8], location="w.bin", offset=60, length=8), base)                      # past the end of the file
    assert "60..68" in str(e.value) and "64" in str(e.value)
    with pytest.raises(Err):
        rd(_external("a", 2, [8], location="w.bin", offset="x"), base)
    with pytest.raises(Err):
        rd(_external("a", 2, [8], location="absent.bin"), base)
    with pytest.raises(Err):
        rd(_external("a", 2, [8], offset=0), base)                                                   # no location key


def test_model_walk_refusals(pkg):
    mi, Err = pkg.initializers.model_initializers, pkg.HipComputeError
    graph = _field(5, 2, _tensor("w", 1, [1], floats=[1.0])) + _field(5, 2, _tensor("", 1, [1], floats=[2.0]))
    with pytest.raises(Err) as e:
        mi(_field(7, 2, graph))
    assert "unnamed" in str(e.value)                              # convert.rs:66-69
    with pytest.raises(Err) as e:
        mi(_field(7, 2, _field(15, 2, b"")))                      # a sparse initializer (convert.rs:72-77)
    assert e.value.code == 2
    with pytest.raises(Err) as e:
        mi(_field(1, 0, _varint(8)))                              # ir_version only
    assert "no graph" in str(e.value)
    assert mi(_field(7, 2, b"")) == {}


def test_matmul_nbits_operands_from_a_model(pkg, oracle):
    """A MatMulNBits node's constant inputs, stored three different ways, come out as the arrays the
    prepack call takes -- checked by running the oracle on them against the arrays they were made from."""
    K, N, bs = 96, 24, 32
    B, scales, zp = pkg.synth.nbits_weight(N, K, bs, seed=77)
    graph = (_field(5, 2, _tensor("B", 2, list(B.shape), raw=B.tobytes())) +
             _field(5, 2, _tensor("S", 1, [scales.size], floats=[float(v) for v in scales.ravel()])) +
             _field(5, 2, _tensor("Z", 2, list(zp.shape), int32s=[int(v) for v in zp.ravel()])))
    inits = pkg.initializers.model_initializers(_field(7, 2, graph))
    gB, gS, gZ = pkg.initializers.matmul_nbits_operands(inits, "B", "S", "Z", K, N, bs)
    assert np.array_equal(gB.reshape(B.shape), B) and np.array_equal(gS, scales.ravel()) and np.array_equal(gZ.reshape(zp.shape), zp)
    a = pkg.synth.normal_f32(K, 78).reshape(1, K)
    assert np.array_equal(oracle.matmul_nbits(a, gB, gS, gZ, K, N, bs), oracle.matmul_nbits(a, B, scales, zp, K, N, bs))
    with pytest.raises(pkg.HipComputeError):
        pkg.initializers.matmul_nbits_operands(inits, "B", "S", "Z", K + 32, N, bs)     # short for a larger K
    with pytest.raises(pkg.HipComputeError):
        pkg.initializers.matmul_nbits_operands(inits, "S", "S", "Z", K, N, bs)          # a float weight
