/*
 * CPU oracle for the quantized matrix-product path. TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of what the reference's own tests define as the
 * right answer for MatMulNBits, DynamicQuantizeLinear, MatMulInteger (+ the fused
 * rescale epilogue), Requantize / QLinearMatMul / QLinearConv and ConvInteger.
 * It exists to check the HIP library; nothing in the shipped library links,
 * loads or calls it, and it is never the thing being measured except as the
 * labelled CPU baseline of the benchmark.
 *
 * Paths are relative to the reference tree (crates/onnx-vulkan-core unless
 * stated otherwise).
 *
 * Pin status (what fixes each function besides its own formula):
 *   oracle_matmul_nbits*     one-hot / all-ones known answers, float64 dense
 *                            dequantised product, the reference test's closed
 *                            form inputs incl. partial last block and unaligned
 *                            zero-point rows (tests/matmul_nbits.rs:64-252)
 *   oracle_dynamic_quantize  symmetric ranges must give zero point 128, integer
 *                            ramps must be the identity, the reference's
 *                            double-single 1/255 constants must reproduce the
 *                            division (src/shaders/dynamic_quantize.rs:183,255-285)
 *   oracle_matmul_integer    arbitrary-precision brute force on the reference's
 *                            LCG bytes and zero points (tests/matmul_integer_variants.rs)
 *   oracle_rescale           float64 re-derivation (product exact in f64, one
 *                            rounding to f32, then the add)
 *   oracle_requantize        hand-evaluated literals of tests/qlinear.rs:106-275
 *   oracle_conv_integer      brute force by explicit zero-point padding and a
 *                            dense matrix product (tests/conv_integer_im2col.rs:58-89)
 *   oracle_qlinear_*         composition of the above, literals of tests/qlinear.rs
 *   MatMulNBits without zero points / with fp16 tensors: the reference refuses
 *   these forms (src/interp.rs:447-464); pinned only by the invariant
 *   "zp omitted == zp identically 8" and "fp16 == fp32 oracle on fp16-rounded
 *   inputs, rounded once" -- no reference vector exists for them.
 */
#ifndef HIPC_ORACLE_H
#define HIPC_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* number of OpenMP threads the oracle will use (1 when built without OpenMP) */
int oracle_threads(void);
void oracle_set_threads(int n);

/* IEEE binary16 <-> binary32, round to nearest even */
uint16_t oracle_f32_to_f16(float v);
float oracle_f16_to_f32(uint16_t h);

/*
 * MatMulNBits, 4-bit. Layout and arithmetic: src/shaders/matmul_nbits.rs:1-25,
 * tests/matmul_nbits.rs:18-91.
 *   B      [N, n_blocks, block_size/2] bytes, element 2i in the LOW nibble of byte i
 *   scales [N * n_blocks]
 *   zp     [N, ceil(n_blocks/2)] bytes, block 2j in the low nibble; NULL => 8
 *   Y[m,n] = sum_k A[m,k] * ((nib(n,k) - zp(n,k/bs)) * scale(n,k/bs)),  k < K only
 * The weight is dequantised to f32 first and the sum runs in k order in f32,
 * exactly as the reference test's scalar loop does.
 */
void oracle_matmul_nbits_f32(const float *A, const uint8_t *B, const float *scales,
                             const uint8_t *zp, float *Y, int64_t M, int64_t K, int64_t N,
                             int64_t block_size);

/* fp16 tensors (A, scales, Y as binary16 bit patterns); f32 arithmetic inside,
 * one rounding at the store. */
void oracle_matmul_nbits_f16(const uint16_t *A, const uint8_t *B, const uint16_t *scales,
                             const uint8_t *zp, uint16_t *Y, int64_t M, int64_t K, int64_t N,
                             int64_t block_size);

/*
 * DynamicQuantizeLinear: tests/dynamic_quantize.rs:16-26; empty input rule
 * src/interp.rs:1949-1966 (y empty, scale 1, zero point 0).
 */
void oracle_dynamic_quantize_linear(const float *x, int64_t n, uint8_t *y, float *scale,
                                    uint8_t *zp);

/*
 * MatMulInteger with scalar zero points: src/host_ops.rs:1157-1199.
 *   A [M,K] u8 or i8, B [K,N] u8 or i8, Y [M,N] i32 = sum (A-a_zp)(B-b_zp)
 */
void oracle_matmul_integer(const void *A, int a_signed, const void *B, int b_signed,
                           int32_t a_zp, int32_t b_zp, int32_t *Y, int64_t M, int64_t K,
                           int64_t N);

/*
 * The dequantising epilogue of a dynamically quantised linear layer, as the
 * unfused Cast -> Mul -> Add [-> Relu] chain rounds it
 * (src/shaders/glsl/matmul_integer_coop.comp:39-55, tests/matmul_integer_epilogue.rs):
 *   out[m,n] = fadd(fmul(float(acc[m,n]), scale[n*scale_step]), bias[n*bias_step])
 * two roundings, never one fused multiply-add. scale_step/bias_step are 0
 * (scalar) or 1 (per column); bias may be NULL. If product != NULL the scale
 * is first multiplied by product[n*product_step] (one more f32 rounding), as
 * the fused node forms a_scale * w_scale.
 */
void oracle_rescale(const int32_t *acc, const float *scale, int scale_step, const float *product,
                    int product_step, const float *bias, int bias_step, int relu, float *out,
                    int64_t M, int64_t N);

/*
 * Requantize: src/shaders/qlinear.rs:28-63, src/interp.rs:4682-4705.
 *   c = (i / inner) % axis_len
 *   q = (int32)rte(float(acc[i] + bias[c]) * ratio[c]) + y_zp, saturated to u8 / i8
 * bias may be NULL.
 */
void oracle_requantize(const int32_t *acc, const int32_t *bias, const float *ratio, int64_t n,
                       int64_t inner, int64_t axis_len, int32_t y_zp, int out_signed, void *out);

/* ratio[c] = x_scale * w_scale[c] / y_scale in f32, left to right (src/interp.rs:4693) */
void oracle_requantize_ratio(float x_scale, const float *w_scale, int64_t n_w, float y_scale,
                             float *ratio);

typedef struct {
    int64_t n, c_in, h, w;     /* input  [n, c_in, h, w] */
    int64_t c_out, kh, kw;     /* weight [c_out, c_in/group, kh, kw] */
    int64_t stride_h, stride_w, dil_h, dil_w;
    int64_t pad_top, pad_left, pad_bottom, pad_right;
    int64_t group;
} oracle_conv_geom;

/* output extent: (in + pb + pe - (d*(k-1)+1)) / s + 1   (src/interp.rs:3427-3536) */
int64_t oracle_conv_out_dim(int64_t in, int64_t pad_begin, int64_t pad_end, int64_t kernel,
                            int64_t stride, int64_t dilation);

/* SAME_UPPER / SAME_LOWER pads for one axis (src/interp.rs:3427-3436) */
void oracle_same_pads(int64_t in, int64_t kernel, int64_t stride, int64_t dilation, int upper,
                      int64_t *pad_begin, int64_t *pad_end);

/*
 * ConvInteger, NCHW, scalar zero points: tests/conv_integer_im2col.rs:58-89.
 * Out-of-bounds taps contribute nothing (padding equals the zero point).
 * Y [n, c_out, h_out, w_out] i32.
 */
void oracle_conv_integer(const void *X, int x_signed, const void *W, int w_signed, int32_t x_zp,
                         int32_t w_zp, const oracle_conv_geom *g, int32_t *Y);

/*
 * QLinearConv == ConvInteger + Requantize (src/interp.rs:4796-4837):
 * w_scale has n_w_scale entries (1 or c_out); a per-tensor scale is broadcast
 * so the bias stays per channel. Output dtype u8 / i8 by y_signed.
 */
void oracle_qlinear_conv(const void *X, int x_signed, float x_scale, int32_t x_zp, const void *W,
                         int w_signed, const float *w_scale, int64_t n_w_scale, int32_t w_zp,
                         float y_scale, int32_t y_zp, int y_signed, const int32_t *bias,
                         const oracle_conv_geom *g, void *Y);

/* QLinearMatMul == MatMulInteger + Requantize on the columns (src/interp.rs:4845-4875) */
void oracle_qlinear_matmul(const void *A, int a_signed, float a_scale, int32_t a_zp, const void *B,
                           int b_signed, const float *b_scale, int64_t n_b_scale, int32_t b_zp,
                           float y_scale, int32_t y_zp, int y_signed, void *Y, int64_t M, int64_t K,
                           int64_t N);

#ifdef __cplusplus
}
#endif
#endif
