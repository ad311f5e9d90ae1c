//! `hip-compute`: the quantized matrix-product operators of `onnx-vulkan-core` on an MI355X, behind the
//! same kind of runtime object `vk-compute` gives the interpreter (`VkContext`: buffers, an
//! enqueue-only stream, flush, capture / replay, GPU timing).
//!
//! NOT BUILT where libhipcompute was written (there is no Rust toolchain there). Every method below is a
//! thin, complete call into `sys` (one C entry point each, the header's comments say which reference
//! function it replaces); what the compiler would still have to confirm is syntax and lifetimes, not
//! behaviour.
//!
//! Conventions carried over from the C ABI:
//! * every method only ENQUEUES on the context's one in-order stream; the host blocks in `flush` and
//!   in the download calls only (`stream.rs:11-14, 702` of `vk-compute`);
//! * operands are device buffers (`GpuBuffer`) or regions of them (`BufferSlice`);
//! * a failed call carries the library's message; `Error::kind` tells the interpreter which of its own
//!   error variants to raise (`crates/onnx-vulkan-core/src/error.rs:6-13`).

pub mod sys;

use std::ffi::{CStr, CString};
use std::os::raw::{c_int, c_void};
use std::ptr;

pub use sys::{hipc_conv_geom as ConvGeom, hipc_decoder_config as DecoderConfig};

/// What went wrong, in the interpreter's terms.
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum ErrorKind {
    /// bad shape / short buffer / null pointer -> `Error::InvalidShape`, `Error::InvalidTensor`
    Invalid,
    /// a form of the operator the library refuses -> `Error::Unsupported`
    Unsupported,
    /// a HIP call failed -> `Error::Backend`
    Backend,
}

#[derive(Debug)]
pub struct Error {
    pub kind: ErrorKind,
    pub message: String,
}

impl std::fmt::Display for Error {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "hip-compute ({:?}): {}", self.kind, self.message)
    }
}
impl std::error::Error for Error {}

pub type Result<T> = std::result::Result<T, Error>;

/// ONNX element types the operators take (`TensorProto.DataType` numbers).
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
#[repr(i32)]
pub enum DType {
    F32 = sys::HIPC_F32,
    U8 = sys::HIPC_U8,
    I8 = sys::HIPC_I8,
    I32 = sys::HIPC_I32,
    F16 = sys::HIPC_F16,
}

impl DType {
    pub fn size(self) -> usize {
        match self {
            DType::F32 | DType::I32 => 4,
            DType::F16 => 2,
            DType::U8 | DType::I8 => 1,
        }
    }
    fn raw(self) -> c_int {
        self as c_int
    }
}

/// A device allocation of the context's pool (`vk_compute::GpuBuffer`).
#[derive(Debug)]
pub struct GpuBuffer {
    ptr: *mut c_void,
    pub size: u64,
}

impl GpuBuffer {
    /// the raw device address (for callers that hand it to other HIP code on the same stream)
    pub fn device_ptr(&self) -> *mut c_void {
        self.ptr
    }
    pub fn slice(&self, offset: u64) -> BufferSlice<'_> {
        BufferSlice { buf: self, offset }
    }
    /// Wraps memory the caller owns (ORT's allocator hands the plugin raw `hipMalloc` pointers): never
    /// give such a buffer to `defer_destroy`.
    ///
    /// # Safety
    /// `ptr` must be a device address valid for `size` bytes on the context's device for as long as
    /// anything enqueued with it may run.
    pub unsafe fn from_raw(ptr: *mut c_void, size: u64) -> Self {
        GpuBuffer { ptr, size }
    }
}

/// A region of a buffer that starts at `offset` (`vk_compute::BufferSlice`).
#[derive(Clone, Copy, Debug)]
pub struct BufferSlice<'a> {
    pub buf: &'a GpuBuffer,
    pub offset: u64,
}

impl<'a> BufferSlice<'a> {
    fn ptr(&self) -> *mut c_void {
        // device pointers are plain addresses: offsetting one is integer arithmetic
        (self.buf.ptr as usize + self.offset as usize) as *mut c_void
    }
    fn remaining(&self) -> u64 {
        self.buf.size.saturating_sub(self.offset)
    }
}

impl<'a> From<&'a GpuBuffer> for BufferSlice<'a> {
    fn from(buf: &'a GpuBuffer) -> Self {
        BufferSlice { buf, offset: 0 }
    }
}

fn opt_ptr(s: Option<BufferSlice<'_>>) -> *mut c_void {
    s.map_or(ptr::null_mut(), |s| s.ptr())
}

/// A recorded stream (`Vec<StreamOp>` in `vk-compute`, `capture.rs:29-126`). Buffers and weight handles
/// named while recording must outlive it.
pub struct Graph {
    raw: *mut sys::hipc_graph,
}

/// Which scalar of a recorded call a replay changes (`HIPC_SCALAR_*`).
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
#[repr(i32)]
pub enum Scalar {
    AZeroPoint = 1,
    BZeroPoint = 2,
    YZeroPoint = 3,
    Relu = 4,
}
/// One patch of a replay: recorded call `op` (in call order, from 0), its scalar `which`, the new value.
#[derive(Clone, Copy, Debug)]
pub struct ScalarPatch {
    pub op: usize,
    pub which: Scalar,
    pub value: i32,
}

/// Prepacked MatMulNBits weight (the role `packed_b` plays for MatMulInteger, `interp.rs:2712-2768`).
pub struct NBitsWeight {
    raw: *mut sys::hipc_nbits_weight,
}
/// Prepacked MatMulInteger / QLinearMatMul B.
pub struct Int8Weight {
    raw: *mut sys::hipc_int8_weight,
}
/// Prepacked ConvInteger / QLinearConv W.
pub struct ConvWeight {
    raw: *mut sys::hipc_conv_weight,
}

impl NBitsWeight {
    /// device bytes of the prepacked form (for `KernelCache`'s memory accounting)
    pub fn bytes(&self) -> usize {
        unsafe { sys::hipc_nbits_weight_bytes(self.raw) }
    }
}

/// MatMulNBits operands in the ONNX layout (`shaders/matmul_nbits.rs:1-25`); lengths in elements.
pub struct NBitsOperands<'a> {
    pub b: BufferSlice<'a>,
    pub b_len: usize,
    pub scales: BufferSlice<'a>,
    pub scale_dtype: DType,
    pub scales_len: usize,
    /// `None`: zero point 8 for every block
    pub zero_points: Option<(BufferSlice<'a>, usize)>,
    pub k: i64,
    pub n: i64,
    pub block_size: i64,
}

/// The epilogue of the fused MatMulInteger -> Cast -> Mul -> Add [-> Relu] (`interp.rs:2405-2572`):
/// device f32 operands, each a scalar (step 0) or one value per column (step 1).
pub struct ScaleBias<'a> {
    pub scale: BufferSlice<'a>,
    pub scale_per_column: bool,
    pub product: Option<(BufferSlice<'a>, bool)>,
    pub bias: Option<(BufferSlice<'a>, bool)>,
    pub relu: bool,
    /// 8-byte slot the output's range is folded into (cleared by the caller), for a following
    /// `dynamic_quantize` with `range_ready`
    pub range: Option<BufferSlice<'a>>,
}

/// Per-tensor quantisation of an activation or an output, host constants (`interp.rs:781-847`).
#[derive(Clone, Copy, Debug)]
pub struct QParams {
    pub scale: f32,
    pub zero_point: i32,
}

/// One process-wide runtime object, like `VkContext` (`crates/vk-compute/src/lib.rs:16-20`).
pub struct HipContext {
    raw: *mut sys::hipc_ctx,
}

// The library serialises calls on a context internally (`submit_lock`, stream.rs:77).
unsafe impl Send for HipContext {}
unsafe impl Sync for HipContext {}

impl Drop for HipContext {
    fn drop(&mut self) {
        unsafe { sys::hipc_ctx_destroy(self.raw) }
    }
}

impl HipContext {
    /// `VkContext::new`: one in-order stream at the default priority on `device`.
    pub fn new(device: i32) -> Result<Self> {
        let mut raw = ptr::null_mut();
        let rc = unsafe { sys::hipc_ctx_create(device as c_int, &mut raw) };
        if rc != sys::HIPC_OK || raw.is_null() {
            return Err(Error { kind: kind_of(rc), message: format!("hipc_ctx_create({device}) failed with status {rc}") });
        }
        Ok(HipContext { raw })
    }

    /// Shares a HIP stream the caller owns (ORT's, in the plugin).
    ///
    /// # Safety
    /// `stream` must be a valid `hipStream_t` of `device` that outlives the context.
    pub unsafe fn on_stream(device: i32, stream: *mut c_void) -> Result<Self> {
        let mut raw = ptr::null_mut();
        let rc = unsafe { sys::hipc_ctx_create_on_stream(device as c_int, stream, &mut raw) };
        if rc != sys::HIPC_OK || raw.is_null() {
            return Err(Error { kind: kind_of(rc), message: format!("hipc_ctx_create_on_stream({device}) failed with status {rc}") });
        }
        Ok(HipContext { raw })
    }

    /// the library's version string (checked at load: "hipcompute <major>.<minor> (gfx950)")
    pub fn version() -> String {
        unsafe { CStr::from_ptr(sys::hipc_version()) }.to_string_lossy().into_owned()
    }

    /// the context's `hipStream_t`, for callers that order their own work against it
    pub fn stream(&self) -> *mut c_void {
        unsafe { sys::hipc_stream(self.raw) }
    }

    fn check(&self, rc: c_int) -> Result<()> {
        if rc == sys::HIPC_OK {
            return Ok(());
        }
        let message = unsafe { CStr::from_ptr(sys::hipc_last_error(self.raw)) }.to_string_lossy().into_owned();
        Err(Error { kind: kind_of(rc), message })
    }

    /// Route and launch-shape overrides (the reference keeps the same kind of switch in its tactic
    /// keys, `tuning.rs`): `name` as in the header, `value < 0` returns the choice to the library.
    pub fn set_option(&self, name: &str, value: i32) -> Result<()> {
        let c = CString::new(name).map_err(|_| Error { kind: ErrorKind::Invalid, message: "option name holds a NUL".into() })?;
        self.check(unsafe { sys::hipc_set_option(self.raw, c.as_ptr(), value as c_int) })
    }

    // ------------------------------------------------------------------ buffers

    /// `create_storage_buffer` / `take_scratch_buffer` (buffer.rs:239, 317): served from the pool's size classes.
    pub fn create_storage_buffer(&self, size: u64) -> Result<GpuBuffer> {
        let mut p = ptr::null_mut();
        self.check(unsafe { sys::hipc_alloc(self.raw, size as usize, &mut p) })?;
        Ok(GpuBuffer { ptr: p, size })
    }
    pub fn take_scratch_buffer(&self, size: u64) -> Result<GpuBuffer> {
        self.create_storage_buffer(size)
    }

    /// `defer_destroy` / `recycle_*` (stream.rs:691, buffer.rs:303-341): valid for everything already
    /// enqueued; back to the pool at the next flush.
    pub fn defer_destroy(&self, buffer: GpuBuffer) {
        // the only failure is a pointer the context does not know, which a GpuBuffer of this context cannot be
        let _ = unsafe { sys::hipc_free_deferred(self.raw, buffer.ptr) };
    }
    pub fn recycle_scratch_buffer(&self, buffer: GpuBuffer) {
        self.defer_destroy(buffer)
    }

    /// (pool hits, pool misses, bytes waiting in the pool) -- `stats.rs:302-312`
    pub fn pool_stats(&self) -> Result<(usize, usize, usize)> {
        let (mut hits, mut misses, mut waiting) = (0usize, 0usize, 0usize);
        self.check(unsafe { sys::hipc_pool_stats(self.raw, &mut hits, &mut misses, &mut waiting) })?;
        Ok((hits, misses, waiting))
    }

    /// `stream_upload_at` (stream.rs:321): records only; `data` may be reused when the call returns.
    pub fn stream_upload_at(&self, dst: &GpuBuffer, dst_offset: u64, data: &[u8]) -> Result<()> {
        if dst_offset + data.len() as u64 > dst.size {
            return Err(Error { kind: ErrorKind::Invalid, message: format!("upload out of bounds: {dst_offset}+{} on {}", data.len(), dst.size) });
        }
        if data.is_empty() {
            return Ok(());
        }
        self.check(unsafe { sys::hipc_upload(self.raw, dst.ptr, dst_offset as usize, data.as_ptr() as *const c_void, data.len()) })
    }
    pub fn stream_upload(&self, dst: &GpuBuffer, data: &[u8]) -> Result<()> {
        self.stream_upload_at(dst, 0, data)
    }

    /// `stream_download_into` (stream.rs:918): flushes, then copies into memory the caller owns.
    pub fn stream_download_into(&self, src: &GpuBuffer, src_offset: u64, out: &mut [u8]) -> Result<()> {
        if src_offset + out.len() as u64 > src.size {
            return Err(Error { kind: ErrorKind::Invalid, message: format!("download out of bounds: {src_offset}+{} on {}", out.len(), src.size) });
        }
        if out.is_empty() {
            return self.flush();
        }
        self.check(unsafe { sys::hipc_download(self.raw, out.as_mut_ptr() as *mut c_void, src.ptr, src_offset as usize, out.len()) })
    }
    pub fn stream_download_at(&self, src: &GpuBuffer, src_offset: u64, bytes: usize) -> Result<Vec<u8>> {
        let mut data = vec![0u8; bytes];
        self.stream_download_into(src, src_offset, &mut data)?;
        Ok(data)
    }
    pub fn stream_download(&self, src: &GpuBuffer, bytes: usize) -> Result<Vec<u8>> {
        self.stream_download_at(src, 0, bytes)
    }

    /// `stream_copy_range` (stream.rs:431)
    pub fn stream_copy_range(&self, src: &GpuBuffer, src_offset: u64, dst: &GpuBuffer, dst_offset: u64, bytes: u64) -> Result<()> {
        if bytes == 0 {
            return Ok(());
        }
        if src_offset + bytes > src.size || dst_offset + bytes > dst.size {
            return Err(Error { kind: ErrorKind::Invalid, message: format!("copy out of bounds: {bytes} bytes from {src_offset} of {} to {dst_offset} of {}", src.size, dst.size) });
        }
        self.check(unsafe { sys::hipc_copy(self.raw, dst.ptr, dst_offset as usize, src.ptr, src_offset as usize, bytes as usize) })
    }
    pub fn stream_copy(&self, src: &GpuBuffer, dst: &GpuBuffer, bytes: u64) -> Result<()> {
        self.stream_copy_range(src, 0, dst, 0, bytes)
    }

    /// `stream_fill` (stream.rs:481): offset and length are multiples of 4; a fill kernel, so it may be captured.
    pub fn stream_fill(&self, dst: &GpuBuffer, dst_offset: u64, bytes: u64, value: u32) -> Result<()> {
        if bytes == 0 {
            return Ok(());
        }
        if dst_offset + bytes > dst.size {
            return Err(Error { kind: ErrorKind::Invalid, message: format!("fill out of bounds: {dst_offset}+{bytes} on {}", dst.size) });
        }
        self.check(unsafe { sys::hipc_fill(self.raw, dst.ptr, dst_offset as usize, bytes as usize, value) })
    }

    /// `flush` (stream.rs:702): the only host <-> device synchronisation.
    pub fn flush(&self) -> Result<()> {
        self.check(unsafe { sys::hipc_flush(self.raw) })
    }

    // ------------------------------------------------------- capture and replay

    /// `begin_capture` (stream.rs:537): what is enqueued from here to `end_capture` is recorded, not run.
    pub fn begin_capture(&self) -> Result<()> {
        self.check(unsafe { sys::hipc_capture_begin(self.raw) })
    }
    /// `end_capture` (stream.rs:542)
    pub fn end_capture(&self) -> Result<Graph> {
        let mut raw = ptr::null_mut();
        self.check(unsafe { sys::hipc_capture_end(self.raw, &mut raw) })?;
        Ok(Graph { raw })
    }
    /// `replay` (stream.rs:572) of a graph as recorded: most quantities that change between replays (token,
    /// position, the zero points and ranges of the dynamic operators) are read from device memory by the kernels.
    pub fn replay(&self, graph: &Graph) -> Result<()> {
        self.check(unsafe { sys::hipc_graph_launch(self.raw, graph.raw) })
    }
    /// `replay` with patches (the reference's `PushPatch`, onnx-vulkan-core/src/plan.rs:52-68): the scalars that were
    /// given by value when the graph was recorded -- the zero points of QLinearMatMul / QLinearConv, the relu
    /// attribute of the fused rescale -- are changed in the instantiated graph first, then it is launched.
    pub fn replay_patched(&self, graph: &Graph, patches: &[ScalarPatch]) -> Result<()> {
        for p in patches {
            self.check(unsafe { sys::hipc_graph_set_scalar(self.raw, graph.raw, p.op as c_int, p.which as c_int, p.value) })?;
        }
        self.replay(graph)
    }
    /// how many calls recorded work while the capture of `graph` was open (the `op` of a `ScalarPatch` counts them from 0)
    pub fn graph_op_count(&self, graph: &Graph) -> Result<usize> {
        let mut n: c_int = 0;
        self.check(unsafe { sys::hipc_graph_op_count(self.raw, graph.raw, &mut n) })?;
        Ok(n as usize)
    }
    pub fn destroy_graph(&self, graph: Graph) {
        unsafe { sys::hipc_graph_destroy(self.raw, graph.raw) }
    }
    /// `measure_dispatch_gpu` (pipeline.rs:246): nanoseconds PER LAUNCH for each of `samples` groups of
    /// `launches_per_sample` replays, by device events on the context's stream.
    pub fn measure_graph(&self, graph: &Graph, samples: usize, launches_per_sample: usize) -> Result<Vec<f64>> {
        let mut ns = vec![0f64; samples];
        self.check(unsafe { sys::hipc_measure_graph(self.raw, graph.raw, samples as c_int, launches_per_sample as c_int, ns.as_mut_ptr()) })?;
        Ok(ns)
    }
    /// what the matrix cores sustain on int8 with operands in registers, in tera-operations per second
    pub fn probe_int8_mfma(&self, random_operands: bool, waves_per_simd: i32, iterations: i32) -> Result<f64> {
        let mut tops = 0f64;
        self.check(unsafe { sys::hipc_probe_int8_mfma(self.raw, random_operands as c_int, waves_per_simd as c_int, iterations as c_int, &mut tops) })?;
        Ok(tops)
    }

    // -------------------------------------------------------------- MatMulNBits

    /// `interp::matmul_nbits` (interp.rs:6429-6561) on the ONNX layout: a weight used once (`prepack_matmul_nbits` takes every block size).
    pub fn matmul_nbits(&self, a: BufferSlice<'_>, a_dtype: DType, w: &NBitsOperands<'_>, y: BufferSlice<'_>, m: i64, accuracy_level: i32) -> Result<()> {
        let (zp, zp_len) = w.zero_points.map_or((ptr::null_mut(), 0), |(s, n)| (s.ptr(), n));
        self.check(unsafe {
            sys::hipc_matmul_nbits(
                self.raw, a.ptr(), a_dtype.raw(), w.b.ptr(), w.b_len, w.scales.ptr(), w.scale_dtype.raw(), w.scales_len, zp, zp_len,
                y.ptr(), m, w.k, w.n, w.block_size, accuracy_level as c_int,
            )
        })
    }
    /// Repack a constant weight once; the operands may be released after the next flush.
    pub fn prepack_matmul_nbits(&self, w: &NBitsOperands<'_>) -> Result<NBitsWeight> {
        let (zp, zp_len) = w.zero_points.map_or((ptr::null_mut(), 0), |(s, n)| (s.ptr(), n));
        let mut raw = ptr::null_mut();
        self.check(unsafe {
            sys::hipc_prepack_matmul_nbits(
                self.raw, w.b.ptr(), w.b_len, w.scales.ptr(), w.scale_dtype.raw(), w.scales_len, zp, zp_len, w.k, w.n, w.block_size, &mut raw,
            )
        })?;
        Ok(NBitsWeight { raw })
    }
    /// MatMulNBits on a prepacked weight: decode rows on the GEMV kernels, more than 16 rows of f16 on the
    /// tiled matrix-core kernel. `accuracy_level` as in the operator (0..4, a lower bound: 1 keeps all 24 bits; many f32 rows travel as two f16 terms, three at level 1, one from level 2 on).
    pub fn matmul_nbits_packed(&self, a: BufferSlice<'_>, a_dtype: DType, w: &NBitsWeight, y: BufferSlice<'_>, m: i64, accuracy_level: i32) -> Result<()> {
        self.check(unsafe { sys::hipc_matmul_nbits_packed(self.raw, a.ptr(), a_dtype.raw(), w.raw, y.ptr(), m, accuracy_level as c_int) })
    }
    pub fn destroy_nbits_weight(&self, w: NBitsWeight) {
        unsafe { sys::hipc_nbits_weight_destroy(self.raw, w.raw) }
    }

    // ---------------------------------------------------- DynamicQuantizeLinear

    /// `interp::dynamic_quantize` + `quantize_on_device` (interp.rs:1945-2085): `x` [n] f32 -> `y` [n] u8, one f32
    /// scale and one u8 zero point on the device. `range`: the 8-byte slot of `execution.rs:80-97` (`None`: the
    /// context's own); `range_ready`: a producer already folded the range of `x` into it (`computed_range`).
    pub fn dynamic_quantize(
        &self, x: BufferSlice<'_>, n: i64, y: BufferSlice<'_>, scale: BufferSlice<'_>, zero_point: BufferSlice<'_>,
        range: Option<BufferSlice<'_>>, range_ready: bool,
    ) -> Result<()> {
        if x.remaining() < 4 * n.max(0) as u64 || y.remaining() < n.max(0) as u64 {
            return Err(Error { kind: ErrorKind::Invalid, message: format!("DynamicQuantizeLinear: {n} elements do not fit the operands") });
        }
        self.check(unsafe { sys::hipc_dynamic_quantize_linear(self.raw, x.ptr(), n, y.ptr(), scale.ptr(), zero_point.ptr(), opt_ptr(range), range_ready as c_int) })
    }
    /// The same without any allocation (code under capture, serving loops): n <= 2^30; calls that overlap on one GPU race.
    pub fn dynamic_quantize_static(&self, x: BufferSlice<'_>, n: i64, y: BufferSlice<'_>, scale: BufferSlice<'_>, zero_point: BufferSlice<'_>) -> Result<()> {
        self.check(unsafe { sys::hipc_dynamic_quantize_linear_static(self.raw, x.ptr(), n, y.ptr(), scale.ptr(), zero_point.ptr()) })
    }
    /// `decomposed_gelu` (interp.rs:1188; rewrite.rs:683-698)
    pub fn decomposed_gelu(&self, x: BufferSlice<'_>, n: i64, divisor: f32, offset: f32, factor: f32, factor_first: bool, y: BufferSlice<'_>) -> Result<()> {
        self.check(unsafe { sys::hipc_decomposed_gelu(self.raw, x.ptr(), n, divisor, offset, factor, factor_first as c_int, y.ptr()) })
    }
    /// `decomposed_gelu_quantize` (interp.rs:1976-2030): DynamicQuantizeLinear of the GELU without storing it.
    pub fn decomposed_gelu_quantize(
        &self, x: BufferSlice<'_>, n: i64, divisor: f32, offset: f32, factor: f32, factor_first: bool, y: BufferSlice<'_>,
        scale: BufferSlice<'_>, zero_point: BufferSlice<'_>, range: Option<BufferSlice<'_>>,
    ) -> Result<()> {
        self.check(unsafe {
            sys::hipc_dynamic_quantize_linear_gelu(
                self.raw, x.ptr(), n, divisor, offset, factor, factor_first as c_int, y.ptr(), scale.ptr(), zero_point.ptr(), opt_ptr(range),
            )
        })
    }

    // ------------------------------------------------------------ MatMulInteger

    /// `packed_b` (interp.rs:2712-2768): `b` [K, N] u8 / i8 -> the layout the GEMM reads + per-column sums.
    pub fn prepack_int8_b(&self, b: BufferSlice<'_>, b_dtype: DType, k: i64, n: i64) -> Result<Int8Weight> {
        let mut raw = ptr::null_mut();
        self.check(unsafe { sys::hipc_prepack_int8_b(self.raw, b.ptr(), b_dtype.raw(), k, n, &mut raw) })?;
        Ok(Int8Weight { raw })
    }
    pub fn destroy_int8_weight(&self, w: Int8Weight) {
        unsafe { sys::hipc_int8_weight_destroy(self.raw, w.raw) }
    }
    /// `interp::matmul_integer` (interp.rs:2090-2183): any K; zero points are device bytes (`None`: 0).
    pub fn matmul_integer(
        &self, a: BufferSlice<'_>, a_dtype: DType, b: &Int8Weight, a_zp: Option<BufferSlice<'_>>, b_zp: Option<BufferSlice<'_>>,
        y: BufferSlice<'_>, m: i64,
    ) -> Result<()> {
        self.check(unsafe { sys::hipc_matmul_integer(self.raw, a.ptr(), a_dtype.raw(), b.raw, opt_ptr(a_zp), opt_ptr(b_zp), y.ptr(), m) })
    }
    /// Both operands dynamic: packs `b` [K, N] into scratch on the stream, then the same kernels.
    pub fn matmul_integer_raw(
        &self, a: BufferSlice<'_>, a_dtype: DType, b: BufferSlice<'_>, b_dtype: DType, a_zp: Option<BufferSlice<'_>>,
        b_zp: Option<BufferSlice<'_>>, y: BufferSlice<'_>, m: i64, k: i64, n: i64,
    ) -> Result<()> {
        self.check(unsafe {
            sys::hipc_matmul_integer_raw(self.raw, a.ptr(), a_dtype.raw(), b.ptr(), b_dtype.raw(), opt_ptr(a_zp), opt_ptr(b_zp), y.ptr(), m, k, n)
        })
    }
    /// `matmul_integer_scale_bias` (interp.rs:2405-2572): two roundings, no fused multiply-add.
    pub fn matmul_integer_scale_bias(
        &self, a: BufferSlice<'_>, a_dtype: DType, b: &Int8Weight, a_zp: Option<BufferSlice<'_>>, b_zp: Option<BufferSlice<'_>>,
        e: &ScaleBias<'_>, y: BufferSlice<'_>, m: i64,
    ) -> Result<()> {
        let (product, product_step) = e.product.map_or((ptr::null_mut(), 0), |(s, per_col)| (s.ptr(), per_col as c_int));
        let (bias, bias_step) = e.bias.map_or((ptr::null_mut(), 0), |(s, per_col)| (s.ptr(), per_col as c_int));
        self.check(unsafe {
            sys::hipc_matmul_integer_scale_bias(
                self.raw, a.ptr(), a_dtype.raw(), b.raw, opt_ptr(a_zp), opt_ptr(b_zp), e.scale.ptr(), e.scale_per_column as c_int,
                product, product_step, bias, bias_step, e.relu as c_int, opt_ptr(e.range), y.ptr(), m,
            )
        })
    }

    // ------------------------------------------------ Requantize / QLinearMatMul

    /// `requantize` (interp.rs:4714-4788): `ratio` [axis_len] f32 and `bias` [axis_len] i32 on the device.
    pub fn requantize(
        &self, acc: BufferSlice<'_>, bias: Option<BufferSlice<'_>>, ratio: BufferSlice<'_>, n: i64, inner: i64, axis_len: i64,
        y_zero_point: i32, out_dtype: DType, out: BufferSlice<'_>,
    ) -> Result<()> {
        self.check(unsafe { sys::hipc_requantize(self.raw, acc.ptr(), opt_ptr(bias), ratio.ptr(), n, inner, axis_len, y_zero_point, out_dtype.raw(), out.ptr()) })
    }
    /// `qlinear_matmul` (interp.rs:4845-4875); `b_scale` is a HOST slice of 1 or N values.
    pub fn qlinear_matmul(
        &self, a: BufferSlice<'_>, a_dtype: DType, a_q: QParams, b: &Int8Weight, b_scale: &[f32], b_zero_point: i32, y_q: QParams,
        y_dtype: DType, y: BufferSlice<'_>, m: i64,
    ) -> Result<()> {
        self.check(unsafe {
            sys::hipc_qlinear_matmul(
                self.raw, a.ptr(), a_dtype.raw(), a_q.scale, a_q.zero_point, b.raw, b_scale.as_ptr(), b_scale.len() as i64, b_zero_point,
                y_q.scale, y_q.zero_point, y_dtype.raw(), y.ptr(), m,
            )
        })
    }

    // ------------------------------------------------- ConvInteger / QLinearConv

    /// `hwc_weight` (interp.rs:5719-5748): `w` [c_out, c_in/group, kh, kw] u8 / i8.
    pub fn prepack_conv_w(&self, w: BufferSlice<'_>, w_dtype: DType, g: &ConvGeom) -> Result<ConvWeight> {
        let mut raw = ptr::null_mut();
        self.check(unsafe { sys::hipc_prepack_conv_w(self.raw, w.ptr(), w_dtype.raw(), g, &mut raw) })?;
        Ok(ConvWeight { raw })
    }
    pub fn destroy_conv_weight(&self, w: ConvWeight) {
        unsafe { sys::hipc_conv_weight_destroy(self.raw, w.raw) }
    }
    /// `conv_integer_with` (interp.rs:4421-4651)
    pub fn conv_integer(
        &self, x: BufferSlice<'_>, x_dtype: DType, w: &ConvWeight, x_zp: Option<BufferSlice<'_>>, w_zp: Option<BufferSlice<'_>>,
        g: &ConvGeom, y: BufferSlice<'_>,
    ) -> Result<()> {
        self.check(unsafe { sys::hipc_conv_integer(self.raw, x.ptr(), x_dtype.raw(), w.raw, opt_ptr(x_zp), opt_ptr(w_zp), g, y.ptr()) })
    }
    /// `qlinear_conv` (interp.rs:4796-4837); `w_scale` is a HOST slice of 1 or c_out values, `bias` [c_out] i32 on the device.
    pub fn qlinear_conv(
        &self, x: BufferSlice<'_>, x_dtype: DType, x_q: QParams, w: &ConvWeight, w_scale: &[f32], w_zero_point: i32, y_q: QParams,
        y_dtype: DType, bias: Option<BufferSlice<'_>>, g: &ConvGeom, y: BufferSlice<'_>,
    ) -> Result<()> {
        self.check(unsafe {
            sys::hipc_qlinear_conv(
                self.raw, x.ptr(), x_dtype.raw(), x_q.scale, x_q.zero_point, w.raw, w_scale.as_ptr(), w_scale.len() as i64, w_zero_point,
                y_q.scale, y_q.zero_point, y_dtype.raw(), opt_ptr(bias), g, y.ptr(),
            )
        })
    }

    // ------------------------------------------------------------ decode step

    /// Caches, scratch and the `{token, position}` state of one decoder, all on the device.
    pub fn create_decoder(&self, cfg: &DecoderConfig) -> Result<Decoder<'_>> {
        let mut raw = ptr::null_mut();
        self.check(unsafe { sys::hipc_decoder_create(self.raw, cfg, &mut raw) })?;
        Ok(Decoder { ctx: self, raw, cfg: *cfg })
    }
}

fn kind_of(rc: c_int) -> ErrorKind {
    match rc {
        sys::HIPC_ERR_INVALID => ErrorKind::Invalid,
        sys::HIPC_ERR_UNSUPPORTED => ErrorKind::Unsupported,
        _ => ErrorKind::Backend,
    }
}

/// output extents of a geometry (`ConvGeom::out_dim`, interp.rs:3361-3536); `None` if the window does not fit
pub fn conv_out_shape(g: &ConvGeom) -> Option<(i64, i64)> {
    let (mut h, mut w) = (0i64, 0i64);
    let rc = unsafe { sys::hipc_conv_out_shape(g, &mut h, &mut w) };
    (rc == sys::HIPC_OK).then_some((h, w))
}

/// `same_pads` (interp.rs:3427-3436): (begin, end) padding of one axis for SAME_UPPER / SAME_LOWER
pub fn same_pads(input: i64, kernel: i64, stride: i64, dilation: i64, upper: bool) -> (i64, i64) {
    let (mut b, mut e) = (0i64, 0i64);
    unsafe { sys::hipc_same_pads(input, kernel, stride, dilation, upper as c_int, &mut b, &mut e) };
    (b, e)
}

/// One initializer of a model file: what `tensor_to_initializer` yields (`convert.rs:247-300`).
#[derive(Clone, Debug, PartialEq, Eq)]
pub struct Initializer {
    pub name: String,
    /// `TensorProto.DataType`
    pub dtype: i32,
    pub shape: Vec<i64>,
    /// little-endian, row-major
    pub data: Vec<u8>,
}

fn host_error(rc: c_int) -> Error {
    let message = unsafe { CStr::from_ptr(sys::hipc_host_error()) }.to_string_lossy().into_owned();
    Error { kind: kind_of(rc), message }
}

/// A serialized `TensorProto` -> its payload, whatever the storage form (`raw_data`, typed fields, or a
/// slice of a file beside the model: `base_dir` is the model's directory, `None` refuses external data).
pub fn read_initializer(tensor: &[u8], base_dir: Option<&std::path::Path>) -> Result<Initializer> {
    let base = match base_dir {
        Some(p) => Some(CString::new(p.to_string_lossy().as_bytes()).map_err(|_| Error { kind: ErrorKind::Invalid, message: "model directory holds a NUL".into() })?),
        None => None,
    };
    let base_ptr = base.as_ref().map_or(ptr::null(), |c| c.as_ptr());
    let mut info: sys::hipc_initializer_info = unsafe { std::mem::zeroed() };
    let rc = unsafe { sys::hipc_initializer_read(tensor.as_ptr() as *const c_void, tensor.len(), base_ptr, &mut info, ptr::null_mut(), 0) };
    if rc != sys::HIPC_OK {
        return Err(host_error(rc));
    }
    let mut data = vec![0u8; info.bytes];
    let rc = unsafe { sys::hipc_initializer_read(tensor.as_ptr() as *const c_void, tensor.len(), base_ptr, &mut info, data.as_mut_ptr() as *mut c_void, data.len()) };
    if rc != sys::HIPC_OK {
        return Err(host_error(rc));
    }
    let name = unsafe { CStr::from_ptr(info.name.as_ptr()) }.to_string_lossy().into_owned();
    Ok(Initializer { name, dtype: info.data_type, shape: info.dims[..info.n_dims as usize].to_vec(), data })
}

/// Every initializer of a serialized `ModelProto`, in file order (`model_to_ir`, `convert.rs:51-76`):
/// unnamed initializers and sparse initializers are refused as there.
pub fn model_initializers(model: &[u8], base_dir: Option<&std::path::Path>) -> Result<Vec<Initializer>> {
    let mut count = 0i64;
    let rc = unsafe { sys::hipc_model_initializers(model.as_ptr() as *const c_void, model.len(), ptr::null_mut(), ptr::null_mut(), 0, &mut count) };
    if rc != sys::HIPC_OK {
        return Err(host_error(rc));
    }
    let n = count as usize;
    let (mut offsets, mut sizes) = (vec![0usize; n], vec![0usize; n]);
    let rc = unsafe { sys::hipc_model_initializers(model.as_ptr() as *const c_void, model.len(), offsets.as_mut_ptr(), sizes.as_mut_ptr(), count, &mut count) };
    if rc != sys::HIPC_OK {
        return Err(host_error(rc));
    }
    let mut out = Vec::with_capacity(n);
    for i in 0..n {
        let t = read_initializer(&model[offsets[i]..offsets[i] + sizes[i]], base_dir)?;
        if t.name.is_empty() {
            return Err(Error { kind: ErrorKind::Invalid, message: "unnamed initializer".into() });
        }
        out.push(t);
    }
    Ok(out)
}

/// Which linear of a layer (`q|k|v` and `gate|up` are given concatenated along N).
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
#[repr(i32)]
pub enum Linear {
    Qkv = sys::HIPC_DEC_QKV,
    O = sys::HIPC_DEC_O,
    GateUp = sys::HIPC_DEC_GATE_UP,
    Down = sys::HIPC_DEC_DOWN,
    /// the layer argument is ignored
    LmHead = sys::HIPC_DEC_LM_HEAD,
}

#[derive(Clone, Copy, Debug, PartialEq, Eq)]
#[repr(i32)]
pub enum Norm {
    Input = sys::HIPC_DEC_NORM_INPUT,
    PostAttn = sys::HIPC_DEC_NORM_POST_ATTN,
    PreFfn = sys::HIPC_DEC_NORM_PRE_FFN,
    PostFfn = sys::HIPC_DEC_NORM_POST_FFN,
    Q = sys::HIPC_DEC_NORM_Q,
    K = sys::HIPC_DEC_NORM_K,
    /// the layer argument is ignored
    Final = sys::HIPC_DEC_NORM_FINAL,
}

/// What `Decoder::read` returns.
#[derive(Clone, Debug)]
pub struct DecoderState {
    /// the token the next step consumes
    pub token: i32,
    /// its position (= tokens already in the cache)
    pub position: i32,
    /// a step was enqueued with the cache full: it wrote nothing; `reset` clears the flag
    pub cache_full: bool,
}

/// The decode loop of `crates/onnx-vulkan/src/lib.rs:509-623` with its state on the device: a captured
/// step replays as it is.
pub struct Decoder<'c> {
    ctx: &'c HipContext,
    raw: *mut sys::hipc_decoder,
    cfg: DecoderConfig,
}

impl Drop for Decoder<'_> {
    fn drop(&mut self) {
        unsafe { sys::hipc_decoder_destroy(self.ctx.raw, self.raw) }
    }
}

impl Decoder<'_> {
    pub fn config(&self) -> &DecoderConfig {
        &self.cfg
    }
    /// 4-bit MatMulNBits operands in the ONNX layout with f32 scales; prepacked inside, free to release after the next flush.
    pub fn set_linear(&self, layer: i32, which: Linear, w: &NBitsOperands<'_>) -> Result<()> {
        let (zp, zp_len) = w.zero_points.map_or((ptr::null_mut(), 0), |(s, n)| (s.ptr(), n));
        self.ctx.check(unsafe {
            sys::hipc_decoder_set_linear(self.ctx.raw, self.raw, layer as c_int, which as c_int, w.b.ptr(), w.b_len, w.scales.ptr(), w.scales_len, zp, zp_len)
        })
    }
    /// RMS-norm weights, f32 on the device ([hidden], or [head_dim] for `Norm::Q` / `Norm::K`).
    pub fn set_norm(&self, layer: i32, which: Norm, w: BufferSlice<'_>) -> Result<()> {
        self.ctx.check(unsafe { sys::hipc_decoder_set_norm(self.ctx.raw, self.raw, layer as c_int, which as c_int, w.ptr()) })
    }
    /// the int4 embedding table [vocab, hidden] in the GatherBlockQuantized layout
    pub fn set_embedding(&self, w: &NBitsOperands<'_>) -> Result<()> {
        let (zp, zp_len) = w.zero_points.map_or((ptr::null_mut(), 0), |(s, n)| (s.ptr(), n));
        self.ctx.check(unsafe { sys::hipc_decoder_set_embedding(self.ctx.raw, self.raw, w.b.ptr(), w.b_len, w.scales.ptr(), w.scales_len, zp, zp_len) })
    }
    /// `local_window_size` of GroupQueryAttention (interp.rs:7528) and the layer's rotary base (0: the configuration's).
    pub fn set_layer_attention(&self, layer: i32, window: i32, rope_theta: f32) -> Result<()> {
        self.ctx.check(unsafe { sys::hipc_decoder_set_layer_attention(self.ctx.raw, self.raw, layer as c_int, window, rope_theta) })
    }
    pub fn reset(&self, token: i32, position: i32) -> Result<()> {
        self.ctx.check(unsafe { sys::hipc_decoder_reset(self.ctx.raw, self.raw, token, position) })
    }
    /// Device addresses of one layer's f16 cache: keys [n_kv_heads, max_seq, head_dim]; values TRANSPOSED,
    /// [n_kv_heads, head_dim, v_stride] with `v_stride()` positions per row. A prefill writes position t of
    /// channel c of head h at `v[(h * head_dim + c) * v_stride + t]`.
    pub fn kv_cache(&self, layer: i32) -> Result<(*mut c_void, *mut c_void)> {
        let (mut k, mut v) = (ptr::null_mut(), ptr::null_mut());
        self.ctx.check(unsafe { sys::hipc_decoder_kv_cache(self.ctx.raw, self.raw, layer as c_int, &mut k, &mut v) })?;
        Ok((k, v))
    }
    /// positions per row of the transposed value cache: max_seq rounded up to a multiple of 64
    pub fn v_stride(&self) -> usize {
        (self.cfg.max_seq as usize + 63) / 64 * 64
    }
    /// Enqueue one decode step (capturable).
    pub fn step(&self) -> Result<()> {
        self.ctx.check(unsafe { sys::hipc_decoder_step(self.ctx.raw, self.raw) })
    }
    /// Flush, then read the state; `logits` ([vocab]) and `history` (the tokens chosen at positions
    /// 0..history.len()) are filled when given.
    pub fn read(&self, logits: Option<&mut [f32]>, history: Option<&mut [i32]>) -> Result<DecoderState> {
        if let Some(l) = &logits {
            if l.len() < self.cfg.vocab as usize {
                return Err(Error { kind: ErrorKind::Invalid, message: format!("logits: {} values for a vocabulary of {}", l.len(), self.cfg.vocab) });
            }
        }
        let (mut token, mut position) = (0i32, 0i32);
        let lp = logits.map_or(ptr::null_mut(), |l| l.as_mut_ptr());
        let (hp, hn) = history.map_or((ptr::null_mut(), 0), |h| (h.as_mut_ptr(), h.len() as i32));
        let rc = unsafe { sys::hipc_decoder_read(self.ctx.raw, self.raw, &mut token, &mut position, lp, hp, hn) };
        match rc {
            sys::HIPC_OK => Ok(DecoderState { token, position, cache_full: false }),
            // the outputs are filled; the status only reports the sticky flag
            sys::HIPC_ERR_INVALID if position >= self.cfg.max_seq => Ok(DecoderState { token, position, cache_full: true }),
            _ => self.ctx.check(rc).map(|_| DecoderState { token, position, cache_full: false }),
        }
    }
}

/// The replayed decode loop, written out (what `Decoder::step` of the reference does per token, minus the patching):
///
/// ```ignore
/// let ctx = HipContext::new(0)?;
/// let dec = ctx.create_decoder(&cfg)?;
/// // set_linear / set_norm / set_embedding / set_layer_attention for every layer, then:
/// dec.reset(first_token, prompt_len)?;          // the prefill filled the caches through kv_cache()
/// dec.step()?; ctx.flush()?;                    // warm every launch shape
/// ctx.begin_capture()?; dec.step()?; let g = ctx.end_capture()?;
/// loop {
///     ctx.replay(&g)?;
///     // every n tokens:
///     let st = dec.read(None, Some(&mut history))?;
///     if st.cache_full || is_eos(st.token) { break; }
/// }
/// ```
#[allow(dead_code)]
struct DecodeLoopExample;
