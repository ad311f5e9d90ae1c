/*
 * libhipcompute -- gfx950 (MI355X) kernels for the quantized matrix-product
 * operators, behind a plain C ABI.
 *
 * The library is the HIP sibling of the reference's `vk-compute` runtime plus
 * the host functions of `onnx-vulkan-core` that sit on the quantized matmul
 * path. Every entry point names the reference interface it stands in for
 * (paths relative to the reference tree). Conventions shared by all calls:
 *
 *   - every function returns an int status: 0 ok, HIPC_ERR_* otherwise; the text
 *     of the last failure on a context is `hipc_last_error(ctx)`
 *     (the reference flattens every backend failure to `Error::Backend(String)`,
 *     crates/onnx-vulkan-core/src/error.rs:6-13, interp.rs:892-894);
 *   - tensor arguments are raw DEVICE pointers (a `hipc_alloc` result plus any
 *     byte offset the caller likes -- the reference's `BufferSlice{buf,offset}`,
 *     crates/vk-compute/src/pipeline.rs:12-21) in the ONNX layout of the operator;
 *   - operator calls only ENQUEUE on the context's stream, in call order; the
 *     host blocks only in `hipc_flush` and `hipc_download`
 *     (crates/vk-compute/src/stream.rs:8-28, 370-383, 702). `hipc_upload` copies the
 *     bytes into a pinned staging ring and records the transfer; it waits (for the
 *     ring's oldest slot, not for the stream) only while more than the ring's 16 MiB
 *     are in flight;
 *   - memory the library itself retires while recorded graphs exist (a scratch block
 *     that had to grow, requantisation ratios that changed, a replaced decoder weight)
 *     stays allocated until the context's last graph is destroyed, so replaying an
 *     older graph never touches freed memory and keeps the scales it was recorded with;
 *   - zero points of the integer operators are read ON THE DEVICE, never read
 *     back (crates/onnx-vulkan-core/src/shaders/matmul_integer.rs:55-56);
 *   - a context may be used from any thread; calls are serialised inside
 *     (`submit_lock`, crates/vk-compute/src/stream.rs:77).
 */
#ifndef HIPCOMPUTE_H
#define HIPCOMPUTE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HIPC_OK 0
#define HIPC_ERR_INVALID 1     /* bad shape / short buffer / null pointer  (Error::InvalidShape, ::InvalidTensor) */
#define HIPC_ERR_UNSUPPORTED 2 /* a form of the operator this library refuses (Error::Unsupported) */
#define HIPC_ERR_BACKEND 3     /* a HIP call failed                        (Error::Backend) */

/* element types, numbered as ONNX TensorProto.DataType (crates/onnx-vulkan-core/src/host_ops.rs) */
#define HIPC_F32 1
#define HIPC_U8 2
#define HIPC_I8 3
#define HIPC_I32 6
#define HIPC_F16 10

typedef struct hipc_ctx hipc_ctx;
typedef struct hipc_graph hipc_graph;
typedef struct hipc_nbits_weight hipc_nbits_weight; /* prepacked MatMulNBits weight */
typedef struct hipc_int8_weight hipc_int8_weight;   /* prepacked MatMulInteger / QLinearMatMul B */
typedef struct hipc_conv_weight hipc_conv_weight;   /* prepacked ConvInteger / QLinearConv W */

/* ------------------------------------------------------------------ context */

/* `VkContext::new` (crates/vk-compute/src/lib.rs:16-20; one per process in the
 * plugin, crates/vulkan-ep/src/vk.rs:6-18). Creates one in-order stream at the
 * default priority on `device`. */
int hipc_ctx_create(int device, hipc_ctx **out);
/* Same, but enqueue on a stream the caller owns (a `hipStream_t`, e.g. the one a
 * host framework already uses), so work interleaves with the caller's in order. */
int hipc_ctx_create_on_stream(int device, void *stream, hipc_ctx **out);
void hipc_ctx_destroy(hipc_ctx *ctx);
const char *hipc_last_error(hipc_ctx *ctx);
const char *hipc_version(void);
/* the `hipStream_t` operators are enqueued on */
void *hipc_stream(hipc_ctx *ctx);
/* Route and launch-shape overrides, for experiments and for tests that must reach every kernel
 * (the reference keeps the same kind of switch in its tactic keys, crates/onnx-vulkan-core/src/tuning.rs).
 * `name` is one of HIPC_GEMV_T, HIPC_GEMV_WAVES, HIPC_GEMV_PER_CU, HIPC_GEMM_TILE, HIPC_GEMM_BIG,
 * HIPC_GEMM_SMALL, HIPC_CONV_ROW, HIPC_PREFILL_TILE, HIPC_PREFILL_SPLIT, HIPC_PREFILL_DIRECT, HIPC_PREFILL_GROUPS,
 * HIPC_DEC_FUSED_GLUE, HIPC_DEC_FUSED_ATTN, HIPC_DEC_FUSED_ARGMAX, HIPC_GEMV_LEAN, HIPC_DEC_LEAN, HIPC_DEC_PREFETCH; a context starts from the environment
 * variables of the same names; value < 0 returns the choice to the library. */
int hipc_set_option(hipc_ctx *ctx, const char *name, int value);

/* ------------------------------------------------------------------ buffers */

/* `create_storage_buffer` + `take_scratch_buffer` (crates/vk-compute/src/buffer.rs:239, 303-341).
 * 256-byte aligned. Requests are served by size class (a power of two up to 1 MiB, whole MiB above)
 * from the blocks earlier frees left behind; only a class with no free block allocates. */
int hipc_alloc(hipc_ctx *ctx, size_t bytes, void **dptr);
/* `defer_destroy` + `recycle_*` (crates/vk-compute/src/stream.rs:691, buffer.rs:303-341): the memory
 * stays valid for everything already enqueued; at the next flush it returns to its size class's
 * free list (up to 1 GiB waiting in all), or to the device. */
int hipc_free_deferred(hipc_ctx *ctx, void *dptr);
/* pool counters (the reference's alloc / pool-hit counters, crates/vk-compute/src/stats.rs:302-312);
 * any pointer may be NULL */
int hipc_pool_stats(hipc_ctx *ctx, size_t *hits, size_t *misses, size_t *bytes_waiting);
/* `stream_upload_at` (stream.rs:310-321): records only; `host` may be reused when the call returns. */
int hipc_upload(hipc_ctx *ctx, void *dst, size_t dst_offset, const void *host, size_t bytes);
/* `stream_download` (stream.rs:773-918): flushes, then copies to `host`. */
int hipc_download(hipc_ctx *ctx, void *host, const void *src, size_t src_offset, size_t bytes);
/* `stream_copy_range` (stream.rs:431) */
int hipc_copy(hipc_ctx *ctx, void *dst, size_t dst_offset, const void *src, size_t src_offset, size_t bytes);
/* `stream_fill` (stream.rs:481): `bytes` must be a multiple of 4; done by a fill kernel,
 * so it may be recorded into a captured graph. */
int hipc_fill(hipc_ctx *ctx, void *dst, size_t dst_offset, size_t bytes, uint32_t word);
/* `flush` (stream.rs:702): the only host<->device synchronisation. */
int hipc_flush(hipc_ctx *ctx);

/* ------------------------------------------------------- capture and replay */

/* `begin_capture` / `end_capture` / `replay` (crates/vk-compute/src/capture.rs:29-126,
 * crates/vk-compute/src/stream.rs:537-572): everything enqueued between begin and end is recorded
 * instead of run, and `hipc_graph_launch` re-issues it. Buffers and weight handles the CALLER named
 * while recording must stay alive and keep their addresses until the graph is destroyed (the
 * reference's preconditions, crates/onnx-vulkan-core/src/plan.rs:21-29); the library's own
 * temporaries are kept alive for it (see the conventions above). */
int hipc_capture_begin(hipc_ctx *ctx);
int hipc_capture_end(hipc_ctx *ctx, hipc_graph **out);
int hipc_graph_launch(hipc_ctx *ctx, hipc_graph *graph);
void hipc_graph_destroy(hipc_ctx *ctx, hipc_graph *graph);

/* The reference patches push-constant words of a recorded step between replays (`PushPatch`,
 * crates/onnx-vulkan-core/src/plan.rs:52-68: "a push-constant word that moves with the step"). Here a graph
 * keeps, for every call that recorded work while the capture was open (numbered from 0 in call order,
 * `hipc_graph_op_count` of them), the scalars of that call a replay may change without recording again:
 *   QLinearMatMul, QLinearConv        the three zero points given by value
 *   MatMulIntegerScaleBias            the relu attribute (0 / 1)
 * `hipc_graph_set_scalar` changes one (a kernel-node parameter update of the instantiated graph); the next
 * `hipc_graph_launch` uses it. Everything that decides a launch's grid (M, the conv geometry) and everything
 * the library keeps in device memory (requantisation ratios, weights) is fixed at recording time, as in the
 * reference ("step-invariant grids and sizes", plan.rs:21-29); MatMulNBits, MatMulInteger and
 * DynamicQuantizeLinear read their zero points, scales and ranges from device memory and carry no such scalar
 * (asking for one is HIPC_ERR_UNSUPPORTED). The decoder needs none: token and position live in device memory. */
#define HIPC_SCALAR_A_ZERO_POINT 1
#define HIPC_SCALAR_B_ZERO_POINT 2
#define HIPC_SCALAR_Y_ZERO_POINT 3
#define HIPC_SCALAR_RELU 4
int hipc_graph_op_count(hipc_ctx *ctx, hipc_graph *graph, int *count);
int hipc_graph_set_scalar(hipc_ctx *ctx, hipc_graph *graph, int op, int which, int32_t value);

/* `measure_dispatch_gpu` (crates/vk-compute/src/pipeline.rs:246): time `samples`
 * groups of `launches_per_sample` launches of a recorded graph with device
 * events on the context's stream; writes nanoseconds PER LAUNCH to ns_out[samples]. */
int hipc_measure_graph(hipc_ctx *ctx, hipc_graph *graph, int samples, int launches_per_sample, double *ns_out);

/* Measurement aid with no counterpart in the reference: what the matrix cores of this device
 * sustain on int8 when nothing else happens. Every CU runs `waves_per_simd` (1 or 2) wavefronts
 * per SIMD, each issuing `iterations` x 8 independent v_mfma_i32_32x32x32_i8 on operands that stay
 * in registers (uniformly random bytes when random_operands != 0, constants otherwise: the clock
 * the device holds depends on how many bits toggle). Writes tera-operations per second, measured
 * with device events on the context's stream, to *tops. The int8 GEMM figures are read against
 * this ceiling as well as against the published peak. */
int hipc_probe_int8_mfma(hipc_ctx *ctx, int random_operands, int waves_per_simd, int iterations, double *tops);

/* -------------------------------------------------------------- MatMulNBits */

/*
 * `interp::matmul_nbits` (crates/onnx-vulkan-core/src/interp.rs:6429-6561) on the
 * tensor format of shaders/matmul_nbits.rs:1-25:
 *   A      [M, K]  f32 or f16 (a_dtype)
 *   B      [N, n_blocks, block_size/2] u8, element 2i in the low nibble of byte i
 *   scales [N * n_blocks]  f32 or f16 (scale_dtype)
 *   zp     [N, ceil(n_blocks/2)] u8, packed like B; NULL => 8 for every block
 *   Y      [M, N]  the dtype of A (crates/onnx-vulkan-frontend/src/shape.rs:497-512)
 * bits is fixed at 4; block_size is any positive multiple of 8, the reference's envelope (the
 * operator's own definition asks for a power of two >= 16); g_idx and bias are
 * refused as in the reference (interp.rs:447-464). `accuracy_level` is 0 (unset)
 * or 1..4, a lower bound on the activations' precision that the reference never reads (it
 * computes every level in f32): see hipc_matmul_nbits_packed for what each level gets here.
 * Buffer lengths are in elements and are checked against K, N and block_size
 * as the reference does (interp.rs:6455-6472); M*N == 0 is a no-op.
 * With more rows than the decode kernels take (16 of f16, 32 of f32) and a block_size that has a
 * tiled form, the call first writes that form into the context's scratch memory and then runs the
 * kernels of hipc_matmul_nbits_packed (the same results as a handle gives, bit for bit); a weight
 * that is used again is better prepacked once.
 */
int hipc_matmul_nbits(hipc_ctx *ctx, const void *A, int a_dtype, const void *B, size_t b_len,
                      const void *scales, int scale_dtype, size_t scales_len, const void *zp,
                      size_t zp_len, void *Y, int64_t M, int64_t K, int64_t N, int64_t block_size,
                      int accuracy_level);

/* Repack a constant weight once (the role `packed_b` plays for MatMulInteger,
 * interp.rs:2712-2768; the reference feeds MatMulNBits the ONNX layout directly).
 * The operands are device pointers in the ONNX layout above and may be released
 * after the next flush. A block_size below 32 or not a power of two has no tiled form:
 * its handle holds copies of the tensors as they are and hipc_matmul_nbits_packed runs
 * the kernel of hipc_matmul_nbits on them (the same results, bit for bit). */
int hipc_prepack_matmul_nbits(hipc_ctx *ctx, const void *B, size_t b_len, const void *scales,
                              int scale_dtype, size_t scales_len, const void *zp, size_t zp_len,
                              int64_t K, int64_t N, int64_t block_size, hipc_nbits_weight **out);
void hipc_nbits_weight_destroy(hipc_ctx *ctx, hipc_nbits_weight *w);
/* bytes of device memory the prepacked form occupies */
size_t hipc_nbits_weight_bytes(const hipc_nbits_weight *w);
/* MatMulNBits on a prepacked weight. `accuracy_level` as in the operator, a lower bound on what the
 * activations may be reduced to (the reference never reads it and computes in f32). Up to 32 rows
 * of f32: 0 (unset), 2, 3 and 4 enter the matrix cores as two bf16 terms (16 significant bits, less
 * error than f32 accumulation over K adds), 1 pins f32 and uses three terms (all 24 bits).
 * More than 16 rows of f16, or 32 of f32, run a tiled f16 matrix-core kernel; an f32 row travels
 * as f16 terms of the row times the power of two that puts its largest value into [2^14, 2^15):
 * two terms (22 bits) at level 0, one (11 bits of every value) at levels 2, 3 and 4, which allow
 * f16, bf16 or int8 activations, three (every bit of the row's values) at level 1.
 * The tiled kernel keeps its accumulators in units of the open quantisation block's scale: there a
 * scale of magnitude below 2^-64 counts as 2^-64 (what such a block adds is below
 * 2^-64 x 15 x sum |a|), and a column whose scales are all below it is stored as 0. */
int hipc_matmul_nbits_packed(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_nbits_weight *w,
                             void *Y, int64_t M, int accuracy_level);

/* ---------------------------------------------------- DynamicQuantizeLinear */

/*
 * `interp::dynamic_quantize` + `quantize_on_device` (interp.rs:1945-2085),
 * arithmetic of shaders/dynamic_quantize.rs:106-222:
 *   X [n] f32 -> Y [n] u8, scale (one f32, device), zero point (one u8, device).
 * n == 0 writes scale 1 and zero point 0 (interp.rs:1949-1966).
 * `range` is an 8-byte device slot {bits(-min), bits(max)}; NULL lets the call use
 * the context's own. When `range_ready` != 0 the slot already holds the range of X
 * (a producer folded it, `computed_range`) and the min/max pass is skipped.
 */
int hipc_dynamic_quantize_linear(hipc_ctx *ctx, const void *X, int64_t n, void *Y, void *scale_out,
                                 void *zp_out, void *range, int range_ready);

/*
 * DecomposedGelu: the exact GELU written out as Div -> Erf -> Add -> Mul -> Mul, which the
 * reference fuses at load time (rewrite.rs:683-698, kernel shaders/elementwise.rs:71-118):
 *   e = erf(x / divisor) + offset;  y = (x * e) * factor,  or  x * (e * factor) with factor_first
 * erf is the reference's polynomial (Abramowitz-Stegun 7.1.26); every step rounds on its own.
 * X, Y: n f32 on the device.
 */
int hipc_decomposed_gelu(hipc_ctx *ctx, const void *X, int64_t n, float divisor, float offset, float factor,
                         int factor_first, void *Y);

/*
 * DecomposedGeluQuantize: DynamicQuantizeLinear of DecomposedGelu(x) without ever storing the
 * GELU (rewrite.rs:699-735; shaders/dynamic_quantize.rs:224-247; interp.rs:1976-2030): both passes
 * evaluate the GELU again from X. Byte for byte what hipc_decomposed_gelu followed by
 * hipc_dynamic_quantize_linear gives (the reference's own test, tests/decomposed_gelu.rs).
 * `range` as in hipc_dynamic_quantize_linear (NULL: the context's own).
 */
int hipc_dynamic_quantize_linear_gelu(hipc_ctx *ctx, const void *X, int64_t n, float divisor, float offset, float factor,
                                      int factor_first, void *Y, void *scale_out, void *zp_out, void *range);

/*
 * hipc_dynamic_quantize_linear (range == NULL) for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the
 * reference. The call allocates nothing, on the device or through any library: the per-workgroup
 * range pairs of the first pass live in a 16 KiB array that is part of the library's own device
 * image (one copy per GPU, held until the process ends), whose address on the context's device was
 * looked up when the context was created. Results are bit for bit those of
 * hipc_dynamic_quantize_linear. n is limited to HIPC_DQL_STATIC_MAX_N elements (HIPC_ERR_INVALID
 * beyond). Every call on one GPU shares that GPU's array, whatever the context: calls that may
 * overlap on one GPU (two contexts, two streams) race; calls on one context are ordered by its stream.
 */
#define HIPC_DQL_STATIC_MAX_N ((int64_t)1 << 30)
int hipc_dynamic_quantize_linear_static(hipc_ctx *ctx, const void *X, int64_t n, void *Y, void *scale_out,
                                        void *zp_out);

/* ------------------------------------------------------------ MatMulInteger */

/* `packed_b` + `flipped_const` (interp.rs:2673-2768; shaders/matmul_integer.rs:135-158):
 * B [K, N] u8 / i8 (b_dtype) -> the layout the GEMM reads, plus per-column sums
 * for the zero-point correction. */
int hipc_prepack_int8_b(hipc_ctx *ctx, const void *B, int b_dtype, int64_t K, int64_t N,
                        hipc_int8_weight **out);
void hipc_int8_weight_destroy(hipc_ctx *ctx, hipc_int8_weight *w);

/*
 * `interp::matmul_integer` (interp.rs:2090-2183), definition host_ops.rs:1157-1199:
 *   Y [M, N] i32 = sum_k (A[m,k] - a_zp) * (B[k,n] - b_zp)
 * A [M, K] u8 / i8 (a_dtype); a_zp / b_zp are device pointers to ONE byte of the
 * operand's dtype, or NULL for 0. Any K (the reference needs a second kernel
 * for K % 4 != 0, interp.rs:2193). K <= 33025 so the i32 sum cannot overflow
 * (interp.rs:2216-2218) is NOT required here: sums wrap as the reference's.
 */
int hipc_matmul_integer(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_int8_weight *B,
                        const void *a_zp, const void *b_zp, void *Y, int64_t M);
/* The same with B in the ONNX layout [K, N]; packs into scratch on every call. */
int hipc_matmul_integer_raw(hipc_ctx *ctx, const void *A, int a_dtype, const void *B, int b_dtype,
                            const void *a_zp, const void *b_zp, void *Y, int64_t M, int64_t K, int64_t N);

/*
 * `matmul_integer_scale_bias` (interp.rs:2405-2572; epilogue rounding
 * shaders/glsl/matmul_integer_coop.comp:39-60): the fused
 * MatMulInteger -> Cast -> Mul(scale) -> Add(bias) [-> Relu]:
 *   Y [M, N] f32 = fadd(fmul(float(acc), s[n]), bias[n]),  s[n] = scale[n*scale_step] (* product[n*product_step])
 * two roundings, no fused multiply-add. scale / product / bias are DEVICE f32
 * pointers; *_step is 0 (scalar) or 1 (per column); product and bias may be NULL.
 * With `range` != NULL the output's {bits(-min), bits(max)} are folded into that
 * 8-byte slot (which the caller cleared), ready for a following
 * hipc_dynamic_quantize_linear(range_ready = 1).
 */
int hipc_matmul_integer_scale_bias(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_int8_weight *B,
                                   const void *a_zp, const void *b_zp, const void *scale, int scale_step,
                                   const void *product, int product_step, const void *bias, int bias_step,
                                   int relu, void *range, void *Y, int64_t M);

/* ------------------------------------------------ Requantize / QLinearMatMul */

/*
 * `requantize` (interp.rs:4714-4788; shaders/qlinear.rs:28-63):
 *   c = (i / inner) % axis_len
 *   out[i] = sat(int32(rte(float(acc[i] + bias[c]) * ratio[c])) + y_zp)   as u8 / i8 (out_dtype)
 * ratio [axis_len] f32 and bias [axis_len] i32 (or NULL) are device pointers.
 */
int hipc_requantize(hipc_ctx *ctx, const void *acc, const void *bias, const void *ratio, int64_t n,
                    int64_t inner, int64_t axis_len, int32_t y_zp, int out_dtype, void *out);

/*
 * `qlinear_matmul` (interp.rs:4845-4875) within the envelope of
 * `unsupported_quantization` (interp.rs:781-847): per-tensor activation and
 * output quantisation given as HOST constants; weight scale per tensor or per
 * column (n_b_scale == 1 or N), per-column weights must have zero point 0.
 * ratio[c] = a_scale * b_scale[c] / y_scale in f32, left to right (interp.rs:4693).
 * `b_scale` is a HOST array.
 */
int hipc_qlinear_matmul(hipc_ctx *ctx, const void *A, int a_dtype, float a_scale, int32_t a_zp,
                        const hipc_int8_weight *B, const float *b_scale, int64_t n_b_scale, int32_t b_zp,
                        float y_scale, int32_t y_zp, int y_dtype, void *Y, int64_t M);

/* ------------------------------------------------- ConvInteger / QLinearConv */

/* `ConvGeom` (interp.rs:3361-3536): NCHW, 1-D given as H = 1. */
typedef struct {
    int64_t n, c_in, h, w;
    int64_t c_out, kh, kw;
    int64_t stride_h, stride_w, dil_h, dil_w;
    int64_t pad_top, pad_left, pad_bottom, pad_right;
    int64_t group;
} hipc_conv_geom;

/* output extents of a geometry; HIPC_ERR_INVALID if the window does not fit */
int hipc_conv_out_shape(const hipc_conv_geom *g, int64_t *h_out, int64_t *w_out);
/* `same_pads` (interp.rs:3427-3436): auto_pad SAME_UPPER (upper != 0) / SAME_LOWER for one axis */
void hipc_same_pads(int64_t in, int64_t kernel, int64_t stride, int64_t dilation, int upper,
                    int64_t *pad_begin, int64_t *pad_end);

/* `hwc_weight` (interp.rs:5719-5748): W [c_out, c_in/group, kh, kw] u8 / i8 -> the
 * layout the implicit-GEMM kernel reads (K ordered (kh, kw, c)). */
int hipc_prepack_conv_w(hipc_ctx *ctx, const void *W, int w_dtype, const hipc_conv_geom *g,
                        hipc_conv_weight **out);
void hipc_conv_weight_destroy(hipc_ctx *ctx, hipc_conv_weight *w);

/*
 * `conv_integer_with` (interp.rs:4421-4651), definition tests/conv_integer_im2col.rs:58-89:
 *   Y [n, c_out, h_out, w_out] i32; out-of-bounds taps contribute 0.
 * x_zp / w_zp are device pointers to one byte, or NULL for 0.
 */
int hipc_conv_integer(hipc_ctx *ctx, const void *X, int x_dtype, const hipc_conv_weight *W,
                      const void *x_zp, const void *w_zp, const hipc_conv_geom *g, void *Y);

/*
 * `qlinear_conv` (interp.rs:4796-4837): ConvInteger, then Requantize with
 * ratio[c] = x_scale * w_scale[c] / y_scale; a per-tensor w_scale (n_w_scale == 1)
 * is broadcast to c_out so `bias` [c_out] i32 (device, may be NULL) stays per channel.
 * Scales and zero points are HOST constants; per-channel weights need w_zp == 0
 * (interp.rs:830-835). Y is u8 / i8 (y_dtype).
 */
int hipc_qlinear_conv(hipc_ctx *ctx, const void *X, int x_dtype, float x_scale, int32_t x_zp,
                      const hipc_conv_weight *W, const float *w_scale, int64_t n_w_scale, int32_t w_zp,
                      float y_scale, int32_t y_zp, int y_dtype, const void *bias,
                      const hipc_conv_geom *g, void *Y);

/* ------------------------------------------------------- ONNX initializers */

/*
 * The data format in front of the prepack calls: a weight as the model file holds it. Host code only
 * (no context, no GPU); a failed call leaves its message in `hipc_host_error` (per thread).
 *
 * `tensor_to_initializer` + `read_external` (crates/onnx-vulkan-frontend/src/convert.rs:247-384):
 * `tensor` is a serialized TensorProto. Its payload is, in this order of precedence, the slice
 * [offset, offset + length) of the file `location` beside the model (data_location EXTERNAL; the path
 * must be relative without "." or ".." components, `base_dir` NULL refuses it), `raw_data` as it is,
 * or the typed repeated fields narrowed to the width `data_type` says (ONNX packs every narrow
 * dtype into int32_data). Fills *info; with data != NULL also copies the little-endian payload
 * (HIPC_ERR_INVALID when data_cap < info->bytes). Call once with data == NULL to size the buffer.
 * A dtype with no readable field is HIPC_ERR_UNSUPPORTED, a malformed message HIPC_ERR_INVALID.
 */
#define HIPC_INITIALIZER_MAX_DIMS 8
typedef struct {
    int32_t data_type; /* TensorProto.DataType (the HIPC_* element types use the same numbers) */
    int32_t n_dims;
    int64_t dims[HIPC_INITIALIZER_MAX_DIMS];
    size_t bytes;      /* length of the payload */
    char name[256];
} hipc_initializer_info;
int hipc_initializer_read(const void *tensor, size_t len, const char *base_dir, hipc_initializer_info *info,
                          void *data, size_t data_cap);
/* `model_to_ir`'s walk over graph.initializer (convert.rs:51-76): `model` is a serialized ModelProto;
 * writes the number of initializers to *count and, for the first `cap` of them, where each one's
 * TensorProto lies inside `model` (offsets / sizes may be NULL to count only). A model without a
 * graph is HIPC_ERR_INVALID, one with sparse initializers HIPC_ERR_UNSUPPORTED, as in the reference. */
int hipc_model_initializers(const void *model, size_t len, size_t *offsets, size_t *sizes, int64_t cap,
                            int64_t *count);
/* message of the last failed host-only call (the two above) on the calling thread */
const char *hipc_host_error(void);

/* ------------------------------------------------------------ decode step */

/*
 * The glue around the MatMulNBits GEMV that turns it into a decoder-only decode step
 * (batch 1, greedy), so that its bandwidth can be quoted as tokens per second. It stands in
 * for these reference operators (crates/onnx-vulkan-core/src): SimplifiedLayerNormalization
 * (shaders/normalization.rs:109-181), GroupQueryAttention with half-split rotary embedding and
 * cache append (shaders/attention.rs:128-317), Gelu approximate="tanh" (interp.rs:9020-9027),
 * GatherBlockQuantized (shaders/gather_block_quantized.rs:26-57), ArgMax
 * (shaders/reduction.rs:76-191), and for the replayed decode loop of
 * crates/onnx-vulkan/src/lib.rs:509-623. One layer is
 *   xn = rmsnorm(x, w_input); qkv = xn W_qkv; q, k = rope(rmsnorm_per_head(q|k, w_q|w_k), pos);
 *   cache[pos] = (k, v) as f16; a = softmax(scale q K^T) V over positions 0..pos;
 *   x += rmsnorm(a W_o, w_post_attn); xn = rmsnorm(x, w_pre_ffn);
 *   h = gelu_tanh(xn W_gate) * (xn W_up); x += rmsnorm(h W_down, w_post_ffn)
 * followed by logits = rmsnorm(x, w_final) W_lm_head and token = argmax(logits).
 * The current token and position live in device memory and are advanced by the step itself,
 * so a captured graph of one step replays without patching.
 * Limits kept on the device: the cache holds `max_seq` positions, so at most `max_seq` steps can
 * follow a reset to position 0. A step enqueued (or replayed) with the cache full writes nothing,
 * leaves token and position as they are and raises a sticky flag that `hipc_decoder_read` reports
 * as HIPC_ERR_INVALID until the next `hipc_decoder_reset`. The chosen token is always inside
 * [0, vocab): if no logit compares (all NaN) it is 0, ArgMax's answer for such a row.
 */
typedef struct hipc_decoder hipc_decoder;
typedef struct {
    int32_t n_layers, hidden, ffn, n_q_heads, n_kv_heads, head_dim, vocab, max_seq, block_size;
    float rms_eps, rope_theta;
    float attn_scale;  /* 0 => 1 / sqrt(head_dim) */
    float embed_scale; /* the embedding row is multiplied by this (gemma: sqrt(hidden)) */
} hipc_decoder_config;

/* linears: all MatMulNBits, 4 bit, f32 scales, ONNX layout. q|k|v and gate|up are given
 * concatenated along N (they share their input, so each pair is one GEMV). */
#define HIPC_DEC_QKV 0      /* [hidden -> (n_q + 2 n_kv) * head_dim] */
#define HIPC_DEC_O 1        /* [n_q * head_dim -> hidden] */
#define HIPC_DEC_GATE_UP 2  /* [hidden -> 2 * ffn] */
#define HIPC_DEC_DOWN 3     /* [ffn -> hidden] */
#define HIPC_DEC_LM_HEAD 4  /* [hidden -> vocab]; `layer` is ignored */
/* RMS-norm weights, f32 */
#define HIPC_DEC_NORM_INPUT 0
#define HIPC_DEC_NORM_POST_ATTN 1
#define HIPC_DEC_NORM_PRE_FFN 2
#define HIPC_DEC_NORM_POST_FFN 3
#define HIPC_DEC_NORM_Q 4     /* [head_dim] */
#define HIPC_DEC_NORM_K 5     /* [head_dim] */
#define HIPC_DEC_NORM_FINAL 6 /* `layer` is ignored */

int hipc_decoder_create(hipc_ctx *ctx, const hipc_decoder_config *cfg, hipc_decoder **out);
void hipc_decoder_destroy(hipc_ctx *ctx, hipc_decoder *dec);
/* Operands are device pointers (element counts in *_len); they are prepacked / copied and may be
 * released after the next flush. zp may be NULL (zero point 8). */
int hipc_decoder_set_linear(hipc_ctx *ctx, hipc_decoder *dec, int layer, int which, const void *B, size_t b_len,
                            const void *scales, size_t scales_len, const void *zp, size_t zp_len);
int hipc_decoder_set_norm(hipc_ctx *ctx, hipc_decoder *dec, int layer, int which, const void *w);
/* the int4 embedding table [vocab, hidden] in the GatherBlockQuantized layout */
int hipc_decoder_set_embedding(hipc_ctx *ctx, hipc_decoder *dec, const void *B, size_t b_len, const void *scales,
                               size_t scales_len, const void *zp, size_t zp_len);
/* Attention of one layer: `window` > 0 limits it to the last `window` positions, the step's own
 * included (GroupQueryAttention's local_window_size, interp.rs:7528; the bound is the reference's,
 * shaders/attention.rs:202-214 and :250: key t is masked when pos - t >= window); window <= 0 is
 * the default, the whole context. `rope_theta` > 0 replaces the configuration's base for this layer
 * (gemma3's local layers rotate with another base than its global ones; the reference gets the
 * tables as the operator's cos / sin cache inputs); at most two distinct bases per decoder. */
int hipc_decoder_set_layer_attention(hipc_ctx *ctx, hipc_decoder *dec, int layer, int32_t window, float rope_theta);
/* the token the next step consumes and its position (= tokens already in the cache). When the embedding table and
 * the first layer's input norm are set, the reset also embeds the token: a step expects the embedded row of the
 * state's token (every step leaves the one of the token it picked behind; a step that finds none -- no reset since
 * the embedding, a norm or a layer's rotary base changed -- embeds first). */
int hipc_decoder_reset(hipc_ctx *ctx, hipc_decoder *dec, int32_t token, int32_t pos);
/* Device pointers of one layer's resident f16 cache. Keys: [n_kv_heads, max_seq, head_dim]. Values are
 * kept transposed, [n_kv_heads, head_dim, v_stride] with v_stride = max_seq rounded up to a multiple of
 * 64, so that the positions a channel is summed over are consecutive (a matrix-core operand is then
 * one 16-byte load). A caller that fills the cache itself (a prefill) writes position t of channel c of
 * kv head h at v_cache[(h * head_dim + c) * v_stride + t]. */
int hipc_decoder_kv_cache(hipc_ctx *ctx, hipc_decoder *dec, int layer, void **k_cache, void **v_cache);
/* enqueue one decode step (capturable; record it after a reset or a step has run, so that the recorded launches do
 * not include an embedding launch of their own) */
int hipc_decoder_step(hipc_ctx *ctx, hipc_decoder *dec);
/* flush, then read the state: next token, next position, the last step's logits [vocab] (or NULL),
 * and the tokens chosen at positions 0..n_history-1 (or NULL). Returns HIPC_ERR_INVALID (outputs
 * still filled) when a step was enqueued with the cache full. */
int hipc_decoder_read(hipc_ctx *ctx, hipc_decoder *dec, int32_t *token, int32_t *pos, float *logits,
                      int32_t *history, int32_t n_history);

#ifdef __cplusplus
}
#endif
#endif
