/*
 * CPU oracle -- TEST INFRASTRUCTURE ONLY, see oracle.h for what each function
 * follows in the reference and what pins it. Build with -ffp-contract=off: the
 * reference's definitions round every f32 operation separately.
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 0;

int oracle_threads(void) {
#ifdef _OPENMP
    return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
    return 1;
#endif
}

void oracle_set_threads(int n) {
    g_threads = n;
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#endif
}

/* ---------------------------------------------------------------- binary16 */

uint16_t oracle_f32_to_f16(float v) {
    uint32_t x;
    memcpy(&x, &v, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mag = x & 0x7fffffffu;
    if (mag >= 0x7f800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | (mag > 0x7f800000u ? 0x0200u : 0));
    }
    if (mag >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (mag < 0x33000001u) { /* below half the smallest subnormal -> 0 */
        return (uint16_t)sign;
    }
    int32_t exp = (int32_t)(mag >> 23) - 127;
    uint32_t man = (mag & 0x007fffffu) | 0x00800000u;
    uint32_t shift;
    uint32_t base;
    if (exp < -14) { /* subnormal result */
        shift = (uint32_t)(13 + (-14 - exp));
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(exp + 15) << 10;
        man &= 0x007fffffu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q += 1; /* carries into the exponent correctly */
    return (uint16_t)(sign | (base + q));
}

float oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            bits = sign | (uint32_t)(127 - 15 - e) << 23 | (man & 0x3ffu) << 13;
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | man << 13;
    } else {
        bits = sign | (exp + 112) << 23 | man << 13;
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* -------------------------------------------------------------- MatMulNBits */

static inline int nibble_at(const uint8_t *row, int64_t i) {
    return (row[i >> 1] >> (4 * (i & 1))) & 15;
}

void oracle_matmul_nbits_f32(const float *A, const uint8_t *B, const float *scales,
                             const uint8_t *zp, float *Y, int64_t M, int64_t K, int64_t N,
                             int64_t block_size) {
    const int64_t n_blocks = (K + block_size - 1) / block_size;
    const int64_t row_bytes = n_blocks * block_size / 2;
    const int64_t zp_row = (n_blocks + 1) / 2;
#pragma omp parallel
    {
        float *w = (float *)malloc((size_t)(K > 0 ? K : 1) * sizeof(float));
#pragma omp for schedule(static)
        for (int64_t n = 0; n < N; n++) {
            const uint8_t *brow = B + n * row_bytes;
            for (int64_t k = 0; k < K; k++) {
                int64_t b = k / block_size;
                int z = zp ? nibble_at(zp + n * zp_row, b) : 8;
                /* block-local index == k - b*bs, and the row is block-contiguous */
                w[k] = ((float)nibble_at(brow, k) - (float)z) * scales[n * n_blocks + b];
            }
            for (int64_t m = 0; m < M; m++) {
                const float *a = A + m * K;
                float acc = 0.0f;
                for (int64_t k = 0; k < K; k++) acc += a[k] * w[k];
                Y[m * N + n] = acc;
            }
        }
        free(w);
    }
}

void oracle_matmul_nbits_f16(const uint16_t *A, const uint8_t *B, const uint16_t *scales,
                             const uint8_t *zp, uint16_t *Y, int64_t M, int64_t K, int64_t N,
                             int64_t block_size) {
    const int64_t n_blocks = (K + block_size - 1) / block_size;
    float *a32 = (float *)malloc((size_t)(M * K > 0 ? M * K : 1) * sizeof(float));
    float *s32 = (float *)malloc((size_t)(N * n_blocks > 0 ? N * n_blocks : 1) * sizeof(float));
    float *y32 = (float *)malloc((size_t)(M * N > 0 ? M * N : 1) * sizeof(float));
    for (int64_t i = 0; i < M * K; i++) a32[i] = oracle_f16_to_f32(A[i]);
    for (int64_t i = 0; i < N * n_blocks; i++) s32[i] = oracle_f16_to_f32(scales[i]);
    oracle_matmul_nbits_f32(a32, B, s32, zp, y32, M, K, N, block_size);
    for (int64_t i = 0; i < M * N; i++) Y[i] = oracle_f32_to_f16(y32[i]);
    free(a32);
    free(s32);
    free(y32);
}

/* ---------------------------------------------------- DynamicQuantizeLinear */

static inline float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

void oracle_dynamic_quantize_linear(const float *x, int64_t n, uint8_t *y, float *scale,
                                    uint8_t *zp) {
    if (n <= 0) {
        *scale = 1.0f;
        *zp = 0;
        return;
    }
    float mn = 0.0f, mx = 0.0f;
    for (int64_t i = 0; i < n; i++) {
        mn = fminf(mn, x[i]);
        mx = fmaxf(mx, x[i]);
    }
    float s = (mx == mn) ? 1.0f : (mx - mn) / 255.0f;
    float z = nearbyintf(clampf(-mn / s, 0.0f, 255.0f)); /* default mode: ties to even */
    *scale = s;
    *zp = (uint8_t)z;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        float q = nearbyintf(x[i] / s) + z;
        y[i] = (uint8_t)clampf(q, 0.0f, 255.0f);
    }
}

/* ------------------------------------------------------------ MatMulInteger */

static inline int32_t byte_value(const void *p, int64_t i, int is_signed) {
    return is_signed ? (int32_t)((const int8_t *)p)[i] : (int32_t)((const uint8_t *)p)[i];
}

void oracle_matmul_integer(const void *A, int a_signed, const void *B, int b_signed,
                           int32_t a_zp, int32_t b_zp, int32_t *Y, int64_t M, int64_t K,
                           int64_t N) {
#pragma omp parallel
    {
        int32_t *arow = (int32_t *)malloc((size_t)(K > 0 ? K : 1) * sizeof(int32_t));
        int64_t *acc = (int64_t *)malloc((size_t)(N > 0 ? N : 1) * sizeof(int64_t));
#pragma omp for schedule(static)
        for (int64_t m = 0; m < M; m++) {
            for (int64_t k = 0; k < K; k++) arow[k] = byte_value(A, m * K + k, a_signed) - a_zp;
            for (int64_t n = 0; n < N; n++) acc[n] = 0;
            for (int64_t k = 0; k < K; k++) {
                const int64_t av = arow[k];
                if (b_signed) {
                    const int8_t *brow = (const int8_t *)B + k * N;
                    for (int64_t n = 0; n < N; n++) acc[n] += av * ((int32_t)brow[n] - b_zp);
                } else {
                    const uint8_t *brow = (const uint8_t *)B + k * N;
                    for (int64_t n = 0; n < N; n++) acc[n] += av * ((int32_t)brow[n] - b_zp);
                }
            }
            /* the sum is the mathematical one; the i32 store wraps like the reference's
             * `as i32` (src/host_ops.rs:1184-1192) */
            for (int64_t n = 0; n < N; n++) Y[m * N + n] = (int32_t)(uint32_t)(uint64_t)acc[n];
        }
        free(arow);
        free(acc);
    }
}

void oracle_rescale(const int32_t *acc, const float *scale, int scale_step, const float *product,
                    int product_step, const float *bias, int bias_step, int relu, float *out,
                    int64_t M, int64_t N) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; m++) {
        for (int64_t n = 0; n < N; n++) {
            volatile float s = scale[n * scale_step];
            if (product) {
                volatile float p = s * product[n * product_step];
                s = p;
            }
            volatile float t = (float)acc[m * N + n] * s; /* first rounding */
            float v = t;
            if (bias) {
                volatile float u = t + bias[n * bias_step]; /* second rounding */
                v = u;
            }
            if (relu && !(v > 0.0f)) v = 0.0f;
            out[m * N + n] = v;
        }
    }
}

/* --------------------------------------------------------------- Requantize */

void oracle_requantize_ratio(float x_scale, const float *w_scale, int64_t n_w, float y_scale,
                             float *ratio) {
    for (int64_t c = 0; c < n_w; c++) {
        volatile float t = x_scale * w_scale[c];
        ratio[c] = t / y_scale;
    }
}

void oracle_requantize(const int32_t *acc, const int32_t *bias, const float *ratio, int64_t n,
                       int64_t inner, int64_t axis_len, int32_t y_zp, int out_signed, void *out) {
    if (inner < 1) inner = 1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        int64_t c = (i / inner) % axis_len;
        int32_t a = acc[i];
        if (bias) a = (int32_t)((uint32_t)a + (uint32_t)bias[c]);
        volatile float t = (float)a * ratio[c];
        float r = nearbyintf(t);
        /* `as i32` saturates in the reference; values here are far inside the range */
        int64_t q = (int64_t)r + (int64_t)y_zp;
        if (out_signed) {
            q = q < -128 ? -128 : (q > 127 ? 127 : q);
            ((int8_t *)out)[i] = (int8_t)q;
        } else {
            q = q < 0 ? 0 : (q > 255 ? 255 : q);
            ((uint8_t *)out)[i] = (uint8_t)q;
        }
    }
}

/* -------------------------------------------------------------- ConvInteger */

int64_t oracle_conv_out_dim(int64_t in, int64_t pad_begin, int64_t pad_end, int64_t kernel,
                            int64_t stride, int64_t dilation) {
    int64_t span = dilation * (kernel - 1) + 1;
    int64_t padded = in + pad_begin + pad_end;
    if (padded < span) return 0;
    return (padded - span) / stride + 1;
}

void oracle_same_pads(int64_t in, int64_t kernel, int64_t stride, int64_t dilation, int upper,
                      int64_t *pad_begin, int64_t *pad_end) {
    int64_t out = (in + stride - 1) / stride;
    int64_t span = dilation * (kernel - 1) + 1;
    int64_t total = (out - 1) * stride + span - in;
    if (total < 0) total = 0;
    int64_t small = total / 2, large = total - small;
    *pad_begin = upper ? small : large;
    *pad_end = upper ? large : small;
}

void oracle_conv_integer(const void *X, int x_signed, const void *W, int w_signed, int32_t x_zp,
                         int32_t w_zp, const oracle_conv_geom *g, int32_t *Y) {
    const int64_t ho = oracle_conv_out_dim(g->h, g->pad_top, g->pad_bottom, g->kh, g->stride_h, g->dil_h);
    const int64_t wo = oracle_conv_out_dim(g->w, g->pad_left, g->pad_right, g->kw, g->stride_w, g->dil_w);
    const int64_t cpg = g->c_in / g->group;   /* input channels per group */
    const int64_t opg = g->c_out / g->group;  /* output channels per group */
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t b = 0; b < g->n; b++) {
        for (int64_t o = 0; o < g->c_out; o++) {
            const int64_t grp = o / opg;
            for (int64_t oh = 0; oh < ho; oh++) {
                for (int64_t ow = 0; ow < wo; ow++) {
                    int64_t acc = 0;
                    for (int64_t c = 0; c < cpg; c++) {
                        const int64_t ci = grp * cpg + c;
                        for (int64_t r = 0; r < g->kh; r++) {
                            const int64_t ih = oh * g->stride_h + r * g->dil_h - g->pad_top;
                            if (ih < 0 || ih >= g->h) continue;
                            for (int64_t s = 0; s < g->kw; s++) {
                                const int64_t iw = ow * g->stride_w + s * g->dil_w - g->pad_left;
                                if (iw < 0 || iw >= g->w) continue;
                                const int64_t xi = ((b * g->c_in + ci) * g->h + ih) * g->w + iw;
                                const int64_t wi = ((o * cpg + c) * g->kh + r) * g->kw + s;
                                acc += (int64_t)(byte_value(X, xi, x_signed) - x_zp) *
                                       (int64_t)(byte_value(W, wi, w_signed) - w_zp);
                            }
                        }
                    }
                    Y[((b * g->c_out + o) * ho + oh) * wo + ow] = (int32_t)(uint32_t)(uint64_t)acc;
                }
            }
        }
    }
}

void oracle_qlinear_conv(const void *X, int x_signed, float x_scale, int32_t x_zp, const void *W,
                         int w_signed, const float *w_scale, int64_t n_w_scale, int32_t w_zp,
                         float y_scale, int32_t y_zp, int y_signed, const int32_t *bias,
                         const oracle_conv_geom *g, void *Y) {
    const int64_t ho = oracle_conv_out_dim(g->h, g->pad_top, g->pad_bottom, g->kh, g->stride_h, g->dil_h);
    const int64_t wo = oracle_conv_out_dim(g->w, g->pad_left, g->pad_right, g->kw, g->stride_w, g->dil_w);
    const int64_t total = g->n * g->c_out * ho * wo;
    int32_t *acc = (int32_t *)malloc((size_t)(total > 0 ? total : 1) * sizeof(int32_t));
    float *ratio = (float *)malloc((size_t)g->c_out * sizeof(float));
    oracle_conv_integer(X, x_signed, W, w_signed, x_zp, w_zp, g, acc);
    if (n_w_scale == 1) {
        float r;
        oracle_requantize_ratio(x_scale, w_scale, 1, y_scale, &r);
        for (int64_t c = 0; c < g->c_out; c++) ratio[c] = r;
    } else {
        oracle_requantize_ratio(x_scale, w_scale, g->c_out, y_scale, ratio);
    }
    oracle_requantize(acc, bias, ratio, total, ho * wo, g->c_out, y_zp, y_signed, Y);
    free(acc);
    free(ratio);
}

void oracle_qlinear_matmul(const void *A, int a_signed, float a_scale, int32_t a_zp, const void *B,
                           int b_signed, const float *b_scale, int64_t n_b_scale, int32_t b_zp,
                           float y_scale, int32_t y_zp, int y_signed, void *Y, int64_t M, int64_t K,
                           int64_t N) {
    int32_t *acc = (int32_t *)malloc((size_t)(M * N > 0 ? M * N : 1) * sizeof(int32_t));
    float *ratio = (float *)malloc((size_t)(n_b_scale > 0 ? n_b_scale : 1) * sizeof(float));
    oracle_matmul_integer(A, a_signed, B, b_signed, a_zp, b_zp, acc, M, K, N);
    oracle_requantize_ratio(a_scale, b_scale, n_b_scale, y_scale, ratio);
    oracle_requantize(acc, NULL, ratio, M * N, 1, n_b_scale, y_zp, y_signed, Y);
    free(acc);
    free(ratio);
}
