"""ctypes binding of libhipcompute.so: context, device buffers, capture/replay, timing.

Mirrors the method set of the reference's ``VkContext`` (crates/vk-compute/src/lib.rs:16-20):
enqueue-only calls, one explicit ``flush``.
"""
from __future__ import annotations

import contextlib
import ctypes as C
import os

import numpy as np

F32, U8, I8, I32, F16 = 1, 2, 3, 6, 10
SCALAR_A_ZERO_POINT, SCALAR_B_ZERO_POINT, SCALAR_Y_ZERO_POINT, SCALAR_RELU = 1, 2, 3, 4
_NP_TO_HIPC = {np.dtype(np.float32): F32, np.dtype(np.uint8): U8, np.dtype(np.int8): I8,
               np.dtype(np.int32): I32, np.dtype(np.float16): F16}

_HERE = os.path.dirname(os.path.abspath(__file__))


class HipComputeError(RuntimeError):
    """A call into libhipcompute failed; ``code`` is the HIPC_ERR_* status."""

    def __init__(self, code: int, message: str):
        super().__init__(f"hipcompute error {code}: {message}")
        self.code = code
        self.message = message


class ConvGeom(C.Structure):
    """``hipc_conv_geom`` -- the reference's ``ConvGeom`` (interp.rs:3361-3536)."""
    _fields_ = [(n, C.c_int64) for n in (
        "n", "c_in", "h", "w", "c_out", "kh", "kw", "stride_h", "stride_w", "dil_h", "dil_w",
        "pad_top", "pad_left", "pad_bottom", "pad_right", "group")]

    @classmethod
    def make(cls, x_shape, w_shape, strides=(1, 1), dilations=(1, 1), pads=(0, 0, 0, 0), group=1):
        n, c_in, h, w = x_shape
        c_out, _, kh, kw = w_shape
        return cls(n, c_in, h, w, c_out, kh, kw, strides[0], strides[1], dilations[0], dilations[1],
                   pads[0], pads[1], pads[2], pads[3], group)


def library_path() -> str:
    """The library beside this package; HIPC_LIBRARY names another build of the same sources there (the one with phase
    time stamps, libhipcompute_stamps.so, for ``bench.py --only phases``)."""
    return os.path.join(_HERE, os.environ.get("HIPC_LIBRARY", "libhipcompute.so"))


class DecoderConfig(C.Structure):
    """``hipc_decoder_config``."""
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "hidden", "ffn", "n_q_heads", "n_kv_heads", "head_dim", "vocab",
                                         "max_seq", "block_size")] + \
               [(n, C.c_float) for n in ("rms_eps", "rope_theta", "attn_scale", "embed_scale")]


class InitializerInfo(C.Structure):
    """``hipc_initializer_info``."""
    _fields_ = [("data_type", C.c_int32), ("n_dims", C.c_int32), ("dims", C.c_int64 * 8), ("bytes", C.c_size_t),
                ("name", C.c_char * 256)]


_lib = None

# name -> (restype, argtypes); every symbol include/hipcompute.h declares
_vp, _i64, _sz, _int, _f = C.c_void_p, C.c_int64, C.c_size_t, C.c_int, C.c_float
SIGNATURES = {
    "hipc_ctx_create": (_int, [_int, C.POINTER(_vp)]),
    "hipc_ctx_create_on_stream": (_int, [_int, _vp, C.POINTER(_vp)]),
    "hipc_ctx_destroy": (None, [_vp]),
    "hipc_last_error": (C.c_char_p, [_vp]),
    "hipc_version": (C.c_char_p, []),
    "hipc_stream": (_vp, [_vp]),
    "hipc_set_option": (_int, [_vp, C.c_char_p, _int]),
    "hipc_initializer_read": (_int, [_vp, _sz, C.c_char_p, C.POINTER(InitializerInfo), _vp, _sz]),
    "hipc_model_initializers": (_int, [_vp, _sz, C.POINTER(_sz), C.POINTER(_sz), _i64, C.POINTER(_i64)]),
    "hipc_host_error": (C.c_char_p, []),
    "hipc_pool_stats": (_int, [_vp, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz)]),
    "hipc_alloc": (_int, [_vp, _sz, C.POINTER(_vp)]),
    "hipc_free_deferred": (_int, [_vp, _vp]),
    "hipc_upload": (_int, [_vp, _vp, _sz, _vp, _sz]),
    "hipc_download": (_int, [_vp, _vp, _vp, _sz, _sz]),
    "hipc_copy": (_int, [_vp, _vp, _sz, _vp, _sz, _sz]),
    "hipc_fill": (_int, [_vp, _vp, _sz, _sz, C.c_uint32]),
    "hipc_flush": (_int, [_vp]),
    "hipc_capture_begin": (_int, [_vp]),
    "hipc_capture_end": (_int, [_vp, C.POINTER(_vp)]),
    "hipc_graph_launch": (_int, [_vp, _vp]),
    "hipc_graph_destroy": (None, [_vp, _vp]),
    "hipc_measure_graph": (_int, [_vp, _vp, _int, _int, C.POINTER(C.c_double)]),
    "hipc_graph_op_count": (_int, [_vp, _vp, C.POINTER(_int)]),
    "hipc_graph_set_scalar": (_int, [_vp, _vp, _int, _int, C.c_int32]),
    "hipc_probe_int8_mfma": (_int, [_vp, _int, _int, _int, C.POINTER(C.c_double)]),
    "hipc_matmul_nbits": (_int, [_vp, _vp, _int, _vp, _sz, _vp, _int, _sz, _vp, _sz, _vp, _i64, _i64, _i64,
                                 _i64, _int]),
    "hipc_prepack_matmul_nbits": (_int, [_vp, _vp, _sz, _vp, _int, _sz, _vp, _sz, _i64, _i64, _i64,
                                         C.POINTER(_vp)]),
    "hipc_nbits_weight_destroy": (None, [_vp, _vp]),
    "hipc_nbits_weight_bytes": (_sz, [_vp]),
    "hipc_matmul_nbits_packed": (_int, [_vp, _vp, _int, _vp, _vp, _i64, _int]),
    "hipc_dynamic_quantize_linear": (_int, [_vp, _vp, _i64, _vp, _vp, _vp, _vp, _int]),
    "hipc_dynamic_quantize_linear_static": (_int, [_vp, _vp, _i64, _vp, _vp, _vp]),
    "hipc_decomposed_gelu": (_int, [_vp, _vp, _i64, _f, _f, _f, _int, _vp]),
    "hipc_dynamic_quantize_linear_gelu": (_int, [_vp, _vp, _i64, _f, _f, _f, _int, _vp, _vp, _vp, _vp]),
    "hipc_prepack_int8_b": (_int, [_vp, _vp, _int, _i64, _i64, C.POINTER(_vp)]),
    "hipc_int8_weight_destroy": (None, [_vp, _vp]),
    "hipc_matmul_integer": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _vp, _i64]),
    "hipc_matmul_integer_raw": (_int, [_vp, _vp, _int, _vp, _int, _vp, _vp, _vp, _i64, _i64, _i64]),
    "hipc_matmul_integer_scale_bias": (_int, [_vp, _vp, _int, _vp, _vp, _vp, _vp, _int, _vp, _int, _vp, _int,
                                              _int, _vp, _vp, _i64]),
    "hipc_requantize": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, C.c_int32, _int, _vp]),
    "hipc_qlinear_matmul": (_int, [_vp, _vp, _int, _f, C.c_int32, _vp, C.POINTER(_f), _i64, C.c_int32, _f,
                                   C.c_int32, _int, _vp, _i64]),
    "hipc_conv_out_shape": (_int, [C.POINTER(ConvGeom), C.POINTER(_i64), C.POINTER(_i64)]),
    "hipc_same_pads": (None, [_i64, _i64, _i64, _i64, _int, C.POINTER(_i64), C.POINTER(_i64)]),
    "hipc_prepack_conv_w": (_int, [_vp, _vp, _int, C.POINTER(ConvGeom), C.POINTER(_vp)]),
    "hipc_conv_weight_destroy": (None, [_vp, _vp]),
    "hipc_conv_integer": (_int, [_vp, _vp, _int, _vp, _vp, _vp, C.POINTER(ConvGeom), _vp]),
    "hipc_qlinear_conv": (_int, [_vp, _vp, _int, _f, C.c_int32, _vp, C.POINTER(_f), _i64, C.c_int32, _f,
                                 C.c_int32, _int, _vp, C.POINTER(ConvGeom), _vp]),
    "hipc_decoder_create": (_int, [_vp, C.POINTER(DecoderConfig), C.POINTER(_vp)]),
    "hipc_decoder_destroy": (None, [_vp, _vp]),
    "hipc_decoder_set_linear": (_int, [_vp, _vp, _int, _int, _vp, _sz, _vp, _sz, _vp, _sz]),
    "hipc_decoder_set_norm": (_int, [_vp, _vp, _int, _int, _vp]),
    "hipc_decoder_set_embedding": (_int, [_vp, _vp, _vp, _sz, _vp, _sz, _vp, _sz]),
    "hipc_decoder_reset": (_int, [_vp, _vp, C.c_int32, C.c_int32]),
    "hipc_decoder_set_layer_attention": (_int, [_vp, _vp, _int, C.c_int32, _f]),
    "hipc_decoder_kv_cache": (_int, [_vp, _vp, _int, C.POINTER(_vp), C.POINTER(_vp)]),
    "hipc_decoder_step": (_int, [_vp, _vp]),
    "hipc_decoder_read": (_int, [_vp, _vp, C.POINTER(C.c_int32), C.POINTER(C.c_int32), _vp, _vp, C.c_int32]),
}


def source_build_id():
    """The build id of the sources in this tree, as csrc/Makefile computes it: sha256 over the sorted
    ``*.hip`` and ``*.h`` of csrc/, the public header and the Makefile (first 16 hex digits).
    None when the sources are not there (a library deployed on its own)."""
    import glob
    import hashlib
    csrc = os.path.join(_HERE, "csrc")
    names = sorted(os.path.basename(f) for f in glob.glob(os.path.join(csrc, "*.hip")) + glob.glob(os.path.join(csrc, "*.h")))
    files = [os.path.join(csrc, n) for n in names] + [os.path.join(_HERE, "..", "include", "hipcompute.h"),
                                                      os.path.join(csrc, "Makefile")]
    if not names or not all(os.path.exists(f) for f in files):
        return None
    h = hashlib.sha256()
    for f in files:
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def load_library():
    """Load libhipcompute.so and declare its signatures. Raises if it has not been built, or if it
    was built from other sources than the ones beside it (a stale library must not run)."""
    global _lib
    if _lib is None:
        path = library_path()
        if not os.path.exists(path):
            raise HipComputeError(3, f"{path} is missing: build it with __graft_entry__.build() "
                                     f"(make -C onnx-vulkan-rs_amd/csrc); there is no fallback path")
        lib = C.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError here means the header and the library disagree
            fn.restype = res
            fn.argtypes = args
        built, want = lib.hipc_version().decode().rsplit(" ", 1)[-1], source_build_id()
        if want is not None and built != want:
            raise HipComputeError(3, f"{path} is stale: built from sources with id {built}, the tree has {want}; "
                                     f"rebuild it (make -C onnx-vulkan-rs_amd/csrc)")
        _lib = lib
    return _lib


def hipc_dtype(dt) -> int:
    return _NP_TO_HIPC[np.dtype(dt)]


class Buffer:
    """A device allocation (``GpuBuffer``). ``ptr`` is the raw device address."""

    def __init__(self, ctx: "Context", nbytes: int):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        p = _vp()
        ctx._check(ctx.lib.hipc_alloc(ctx.handle, self.nbytes, C.byref(p)))
        self.ptr = p.value

    def at(self, offset: int) -> int:
        return self.ptr + int(offset)

    def free(self):
        if self.ptr:
            self.ctx.lib.hipc_free_deferred(self.ctx.handle, self.ptr)
            self.ptr = None


class Context:
    """One device, one in-order stream (``VkContext``)."""

    def __init__(self, device: int = 0, stream: int | None = None):
        self.lib = load_library()
        h = _vp()
        if stream is None:
            rc = self.lib.hipc_ctx_create(device, C.byref(h))
        else:
            rc = self.lib.hipc_ctx_create_on_stream(device, stream, C.byref(h))
        if rc != 0:
            raise HipComputeError(rc, f"cannot create a context on device {device} (no GPU?)")
        self.handle = h

    def close(self):
        if self.handle:
            self.lib.hipc_ctx_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _check(self, rc: int):
        if rc != 0:
            raise HipComputeError(rc, self.lib.hipc_last_error(self.handle).decode())

    @property
    def stream(self) -> int:
        return self.lib.hipc_stream(self.handle)

    def set_option(self, name: str, value: int):
        """A route / launch-shape override (``hipc_set_option``); a negative value restores the default."""
        self._check(self.lib.hipc_set_option(self.handle, name.encode(), int(value)))

    @contextlib.contextmanager
    def options(self, **values):
        """``with ctx.options(HIPC_GEMM_TILE=128): ...`` -- overrides for the duration of the block."""
        for k, v in values.items():
            self.set_option(k, v)
        try:
            yield self
        finally:
            for k in values:
                self.set_option(k, -1)

    def pool_stats(self):
        """(hits, misses, bytes waiting) of the allocation pool."""
        h, m, b = _sz(), _sz(), _sz()
        self._check(self.lib.hipc_pool_stats(self.handle, C.byref(h), C.byref(m), C.byref(b)))
        return h.value, m.value, b.value

    # ---- buffers
    def alloc(self, nbytes: int) -> Buffer:
        return Buffer(self, nbytes)

    def upload(self, array: np.ndarray, buf: Buffer | None = None, offset: int = 0) -> Buffer:
        a = np.ascontiguousarray(array)
        if buf is None:
            buf = self.alloc(max(a.nbytes, 4))
        self._check(self.lib.hipc_upload(self.handle, buf.ptr, offset, a.ctypes.data, a.nbytes))
        return buf

    def download(self, buf, dtype, shape, offset: int = 0) -> np.ndarray:
        out = np.empty(shape, dtype)
        ptr = buf.ptr if isinstance(buf, Buffer) else buf
        self._check(self.lib.hipc_download(self.handle, out.ctypes.data, ptr, offset, out.nbytes))
        return out

    def copy(self, dst, dst_offset, src, src_offset, nbytes):
        self._check(self.lib.hipc_copy(self.handle, _ptr(dst), dst_offset, _ptr(src), src_offset, nbytes))

    def fill(self, buf, offset, nbytes, word):
        self._check(self.lib.hipc_fill(self.handle, _ptr(buf), offset, nbytes, word))

    def flush(self):
        self._check(self.lib.hipc_flush(self.handle))

    # ---- capture / replay / timing
    def capture_begin(self):
        self._check(self.lib.hipc_capture_begin(self.handle))

    def capture_end(self):
        g = _vp()
        self._check(self.lib.hipc_capture_end(self.handle, C.byref(g)))
        return g

    def graph_launch(self, graph):
        self._check(self.lib.hipc_graph_launch(self.handle, graph))

    def graph_destroy(self, graph):
        self.lib.hipc_graph_destroy(self.handle, graph)

    def graph_op_count(self, graph) -> int:
        """How many calls recorded work while the capture of `graph` was open."""
        n = _int()
        self._check(self.lib.hipc_graph_op_count(self.handle, graph, C.byref(n)))
        return n.value

    def graph_set_scalar(self, graph, op: int, which: int, value: int):
        """Change a scalar of recorded call `op` for the replays that follow (the reference's ``PushPatch``)."""
        self._check(self.lib.hipc_graph_set_scalar(self.handle, graph, op, which, value))

    def probe_int8_mfma(self, random_operands: bool, waves_per_simd: int = 2, iterations: int = 4096) -> float:
        """Sustained int8 matrix-core rate (TOPS) of a register-only MFMA loop."""
        out = C.c_double()
        self._check(self.lib.hipc_probe_int8_mfma(self.handle, int(random_operands), waves_per_simd, iterations, C.byref(out)))
        return out.value

    def measure_graph(self, graph, samples: int, launches_per_sample: int) -> np.ndarray:
        """Nanoseconds per launch for each sample (``measure_dispatch_gpu``)."""
        out = (C.c_double * samples)()
        self._check(self.lib.hipc_measure_graph(self.handle, graph, samples, launches_per_sample, out))
        return np.array(out[:], dtype=np.float64)


def _ptr(b):
    if b is None:
        return None
    return b.ptr if isinstance(b, Buffer) else int(b)
