"""MI355X (gfx950) kernels for the quantized matrix-product operators of onnx-vulkan-rs.

The product is ``libhipcompute.so`` (C ABI in ``include/hipcompute.h``); this package is
the thin ctypes layer the tests and the benchmark drive it through, plus the seeded
input generators of the benchmark configurations. It contains no compute of its own and
no CPU fallback: if the library is missing, importing the runtime raises.

The directory name carries a hyphen, so it is loaded by path and registered under the
module name ``onnx_vulkan_rs_amd`` (see ``__graft_entry__.load_package``).
"""
from .runtime import (  # noqa: F401
    Context,
    Buffer,
    HipComputeError,
    ConvGeom,
    DecoderConfig,
    library_path,
    load_library,
    F32, F16, U8, I8, I32,
)
from . import ops, synth, graph, decoder, initializers, runtime  # noqa: F401
