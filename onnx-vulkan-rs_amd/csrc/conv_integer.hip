// ConvInteger and QLinearConv (static int8, NCHW) for gfx950.
//
// Reference: crates/onnx-vulkan-core/src/interp.rs:3361-3536 (geometry), :4421-4651
// (conv_integer_with routing), :4796-4837 (qlinear_conv), :5680-5748 (HWC weight and
// activation layout); kernels shaders/conv_integer.rs; definition
// tests/conv_integer_im2col.rs:58-89.
//
// The reference materialises an im2col matrix [P, K] and runs its matmul on it
// (interp.rs:5319-5469). Here nothing of size P*K exists: the activation is
// turned once into NHWC (1x its own size, uint8 shifted to signed on the way),
// and the int8 MFMA contraction gathers its k-contiguous 16-byte operand chunks
// straight from it, with K ordered (kh, kw, c) and the weight prepacked to
// match. Padding taps read the zero point, so they contribute nothing and the
// zero-point algebra of the plain matmul applies unchanged
// (shaders/conv_integer.rs:112-119, 350-371).
// A window along one axis (H = 1, 1 x kw: the vocoder shapes) skips even that
// copy: each workgroup reads the input positions its 64 outputs see straight
// from NCHW, transposes them in registers and keeps them in LDS for the whole
// product (int8_conv_row_kernel).
// Grouped convolutions and channel counts that are not multiples of 16 take a
// direct kernel, one output per thread, as the reference does for grouped ones.
#include <algorithm>

#include "int8_gemm.h"

namespace hipc {

// X [C, HW] bytes -> Xt [HW, C] bytes (per image), xor `flip` on the way. 32x32 tiles.
__global__ void __launch_bounds__(256)
nchw_to_nhwc_kernel(const uint8_t *__restrict__ X, uint8_t *__restrict__ Xt, int C, int HW, uint8_t flip) {
    __shared__ uint8_t tile[32][33];
    const size_t img = (size_t)blockIdx.z * C * HW;
    const int hw0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const int c = c0 + r, hw = hw0 + tx;
        tile[r][tx] = (c < C && hw < HW) ? X[img + (size_t)c * HW + hw] ^ flip : 0;
    }
    __syncthreads();
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const int hw = hw0 + r, c = c0 + tx;
        if (c < C && hw < HW) Xt[img + (size_t)hw * C + c] = tile[tx][r];
    }
}

// The same for C and HW multiples of 4 with 4-byte aligned images, 32 bits at a time: a thread reads
// four positions of four channels (16 lanes x 4 bytes are one 64-byte run of a channel), transposes
// the 4 x 4 bytes in registers, and the words change hands through LDS so that the stores run along
// the channels (16 lanes x 4 bytes of one position). 64 channels x 64 positions per workgroup.
__global__ void __launch_bounds__(256)
nchw_to_nhwc4_kernel(const uint8_t *__restrict__ X, uint8_t *__restrict__ Xt, int C, int HW, uint32_t flip4) {
    __shared__ uint32_t words[64][17];  // [position][channel quad], padded
    const size_t img = (size_t)blockIdx.z * C * HW;
    const int hw0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
    const int hq = threadIdx.x & 15, cq = threadIdx.x >> 4;  // position quad, channel quad
    uint32_t in[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int c = c0 + 4 * cq + i, hw = hw0 + 4 * hq;
        in[i] = (c < C && hw < HW) ? *reinterpret_cast<const uint32_t *>(X + img + (size_t)c * HW + hw) ^ flip4 : 0u;
    }
    // out[j] = bytes j of in[0..3]: the four channels of position 4 hq + j
    const uint32_t lo01 = __builtin_amdgcn_perm(in[1], in[0], 0x05010400u);  // a0 b0 a1 b1
    const uint32_t hi01 = __builtin_amdgcn_perm(in[1], in[0], 0x07030602u);  // a2 b2 a3 b3
    const uint32_t lo23 = __builtin_amdgcn_perm(in[3], in[2], 0x05010400u);  // c0 d0 c1 d1
    const uint32_t hi23 = __builtin_amdgcn_perm(in[3], in[2], 0x07030602u);  // c2 d2 c3 d3
    words[4 * hq + 0][cq] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);  // a0 b0 c0 d0
    words[4 * hq + 1][cq] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);  // a1 b1 c1 d1
    words[4 * hq + 2][cq] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
    words[4 * hq + 3][cq] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
    __syncthreads();
    const int oq = threadIdx.x & 15, op = threadIdx.x >> 4;  // channel quad, position (of 16 per pass)
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int pos = op + 16 * r, hw = hw0 + pos, c = c0 + 4 * oq;
        if (c < C && hw < HW) *reinterpret_cast<uint32_t *>(Xt + img + (size_t)hw * C + c) = words[pos][oq];
    }
}

// W [O, C, kh, kw] -> Wp, O_pad x K_pad bytes in the fragment-major order of qfrag_offset,
// k = (r*kw + s)*C + c, signed domain, zero padded;
// rowsum[o] = sum_k Wp[o][k].
__global__ void __launch_bounds__(256)
pack_conv_w_kernel(const uint8_t *__restrict__ W, uint8_t *__restrict__ Wp, int32_t *__restrict__ rowsum, int O, int C,
                   int kh, int kw, int O_pad, int K_pad, int is_signed, int shift) {
    const int o = blockIdx.x;
    const int K = C * kh * kw;
    int local = 0;
    for (int k = threadIdx.x; k < K_pad; k += 256) {
        uint8_t out = 0;
        if (o < O && k < K) {
            const int tap = k / C, c = k - tap * C;
            const uint8_t v = W[((size_t)o * C + c) * kh * kw + tap];
            const int sv = (is_signed ? (int)(int8_t)v : (int)v) - shift;
            local += sv;
            out = (uint8_t)sv;
        }
        Wp[qfrag_offset(o, k, K_pad)] = out;
    }
    __shared__ int part[256];
    part[threadIdx.x] = local;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) part[threadIdx.x] += part[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) rowsum[o] = part[0];
}

struct DirectConvArgs {
    const uint8_t *X, *W;
    const uint8_t *x_zp, *w_zp;
    int x_signed, w_signed, host_zp, x_zp_value, w_zp_value;
    int n, C, H, Wd, O, kh, kw, sh, sw, dh, dw, pt, pl, group, Ho, Wo;
    void *Y;
    int requant;
    const float *ratio;
    int ratio_step;
    const int32_t *qbias;
    int y_zp, out_signed;
};

__global__ void __launch_bounds__(256) conv_direct_kernel(const DirectConvArgs p) {
    const long total = (long)p.n * p.O * p.Ho * p.Wo;
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int ow = (int)(idx % p.Wo);
    const int oh = (int)((idx / p.Wo) % p.Ho);
    const int o = (int)((idx / ((long)p.Wo * p.Ho)) % p.O);
    const int b = (int)(idx / ((long)p.Wo * p.Ho * p.O));
    const int zx = p.host_zp ? p.x_zp_value : zp_byte(p.x_zp, p.x_signed);
    const int zw = p.host_zp ? p.w_zp_value : zp_byte(p.w_zp, p.w_signed);
    const int cpg = p.C / p.group, opg = p.O / p.group;
    const int grp = o / opg;
    int acc = 0;
    for (int c = 0; c < cpg; c++) {
        const int ci = grp * cpg + c;
        for (int r = 0; r < p.kh; r++) {
            const int ih = oh * p.sh + r * p.dh - p.pt;
            if (ih < 0 || ih >= p.H) continue;
            for (int s = 0; s < p.kw; s++) {
                const int iw = ow * p.sw + s * p.dw - p.pl;
                if (iw < 0 || iw >= p.Wd) continue;
                const uint8_t xv = p.X[(((size_t)b * p.C + ci) * p.H + ih) * p.Wd + iw];
                const uint8_t wv = p.W[(((size_t)o * cpg + c) * p.kh + r) * p.kw + s];
                const int xi = (p.x_signed ? (int)(int8_t)xv : (int)xv) - zx;
                const int wi = (p.w_signed ? (int)(int8_t)wv : (int)wv) - zw;
                acc += xi * wi;
            }
        }
    }
    if (!p.requant) {
        static_cast<int32_t *>(p.Y)[idx] = acc;
    } else {
        if (p.qbias) acc += p.qbias[o];
        int q = (int)rintf(__fmul_rn((float)acc, p.ratio[(size_t)o * p.ratio_step])) + p.y_zp;
        if (p.out_signed)
            static_cast<int8_t *>(p.Y)[idx] = (int8_t)min(max(q, -128), 127);
        else
            static_cast<uint8_t *>(p.Y)[idx] = (uint8_t)min(max(q, 0), 255);
    }
}

}  // namespace hipc

using namespace hipc;

struct hipc_conv_weight {
    hipc_conv_geom geom{};   // the geometry the weight was packed for (c_out, c_in, kh, kw, group)
    int w_dtype = HIPC_I8;
    uint8_t *raw = nullptr;  // ONNX layout copy, for the direct path
    uint8_t *Wp = nullptr;   // [O_pad, K_pad], (kh, kw, c) order; null when the MFMA path does not apply
    int32_t *rowsum = nullptr;
    int O_pad = 0, K_pad = 0;
    mutable hipc::RatioCache ratios;  // QLinearConv's requantisation ratios as last used
};

namespace {

int out_dim(int64_t in, int64_t pb, int64_t pe, int64_t k, int64_t s, int64_t d, int64_t *out) {
    const int64_t span = d * (k - 1) + 1, padded = in + pb + pe;
    if (padded < span) return HIPC_ERR_INVALID;
    *out = (padded - span) / s + 1;
    return HIPC_OK;
}

int check_geom(hipc_ctx *ctx, const hipc_conv_geom *g, int64_t *ho, int64_t *wo) {
    HIPC_REQUIRE(ctx, g, "Conv: null geometry");
    HIPC_REQUIRE(ctx, g->n >= 0 && g->c_in > 0 && g->h > 0 && g->w > 0 && g->c_out > 0 && g->kh > 0 && g->kw > 0,
                 "Conv: non-positive dimension");
    HIPC_REQUIRE(ctx, g->stride_h > 0 && g->stride_w > 0 && g->dil_h > 0 && g->dil_w > 0, "Conv: strides and dilations must be positive");
    HIPC_REQUIRE(ctx, g->pad_top >= 0 && g->pad_left >= 0 && g->pad_bottom >= 0 && g->pad_right >= 0, "Conv: negative padding");
    HIPC_REQUIRE(ctx, g->group > 0 && g->c_in % g->group == 0 && g->c_out % g->group == 0,
                 "Conv: group %ld does not divide the channels (%ld in, %ld out)", (long)g->group, (long)g->c_in, (long)g->c_out);
    HIPC_REQUIRE(ctx,
                 out_dim(g->h, g->pad_top, g->pad_bottom, g->kh, g->stride_h, g->dil_h, ho) == HIPC_OK &&
                     out_dim(g->w, g->pad_left, g->pad_right, g->kw, g->stride_w, g->dil_w, wo) == HIPC_OK,
                 "Conv: the kernel window does not fit the padded input");
    const int64_t big = int64_t(1) << 30;
    HIPC_REQUIRE(ctx, g->n * g->c_out * *ho * *wo < big * 2 && g->n * g->c_in * g->h * g->w < big * 2 && g->c_in * g->kh * g->kw < big,
                 "Conv: tensor too large");
    return HIPC_OK;
}

bool same_weight_shape(const hipc_conv_geom &a, const hipc_conv_geom &b) {
    return a.c_in == b.c_in && a.c_out == b.c_out && a.kh == b.kh && a.kw == b.kw && a.group == b.group;
}

struct ConvEpilogue {
    int requant = 0;
    const float *ratio = nullptr;  // device
    int ratio_step = 0;
    const int32_t *qbias = nullptr;
    int y_zp = 0, out_signed = 0;
};

int run_conv(hipc_ctx *ctx, const void *X, int x_dtype, const hipc_conv_weight *W, const void *x_zp, const void *w_zp,
             int host_zp, int x_zp_value, int w_zp_value, const hipc_conv_geom *g, void *Y, const ConvEpilogue &ep) {
    int64_t ho = 0, wo = 0;
    int rc = check_geom(ctx, g, &ho, &wo);
    if (rc != HIPC_OK) return rc;
    HIPC_REQUIRE(ctx, W, "Conv: null weight");
    HIPC_REQUIRE(ctx, same_weight_shape(*g, W->geom), "Conv: the weight was prepacked for a different shape");
    HIPC_REFUSE(ctx, !is_byte_dtype(x_dtype), "Conv: X must be uint8 or int8, got %d", x_dtype);
    const int64_t total = g->n * g->c_out * ho * wo;
    if (total == 0) return HIPC_OK;
    HIPC_REQUIRE(ctx, X && Y, "Conv: null tensor");

    if (W->Wp) {
        GemmArgs ga{};
        ga.P = W->Wp;
        ga.const_sum = W->rowsum;
        ga.dyn_zp = static_cast<const uint8_t *>(x_zp), ga.const_zp = static_cast<const uint8_t *>(w_zp);
        ga.dyn_shift = x_dtype == HIPC_U8 ? 128 : 0, ga.const_shift = W->w_dtype == HIPC_U8 ? 128 : 0;
        ga.dyn_signed = x_dtype == HIPC_I8, ga.const_signed = W->w_dtype == HIPC_I8;
        ga.host_zp = host_zp, ga.dyn_zp_value = x_zp_value, ga.const_zp_value = w_zp_value;
        ga.I = (int)g->c_out, ga.J = (int)(ho * wo), ga.K = (int)(g->c_in * g->kh * g->kw), ga.K_pad = W->K_pad;
        ga.C = (int)g->c_in, ga.H = (int)g->h, ga.W = (int)g->w, ga.Ho = (int)ho, ga.Wo = (int)wo;
        ga.kh = (int)g->kh, ga.kw = (int)g->kw, ga.sh = (int)g->stride_h, ga.sw = (int)g->stride_w;
        ga.dh = (int)g->dil_h, ga.dw = (int)g->dil_w, ga.pt = (int)g->pad_top, ga.pl = (int)g->pad_left;
        ga.Y = Y;
        ga.ratio = ep.ratio, ga.ratio_step = ep.ratio_step, ga.qbias = ep.qbias, ga.y_zp = ep.y_zp,
        ga.out_signed = ep.out_signed;
        HIPC_REQUIRE(ctx, g->n <= 65535, "Conv: batch %ld too large", (long)g->n);
        // few 64x64 tiles and a long k: the wavefronts of a workgroup split k and the weight stays out of LDS
        // (the gemm_small option, 0 / 1, overrides: tuning, tests)
        const int forced = ctx->tune.gemm_small;
        const int64_t tiles64 = ceil_div(ga.I, 64) * ceil_div(ga.J, 64) * g->n;
        const bool small = forced >= 0 ? forced != 0 : (tiles64 <= 2 * (int64_t)ctx->cu_count && ga.K_pad >= 4 * kBK);
        // the row sums of the activations only matter when the weight's zero point, in the signed domain, is not zero
        const bool zero_known = ga.const_shift == 0 && (host_zp ? w_zp_value == 0 : w_zp == nullptr);

        // A convolution along W alone whose per-tile input slab fits LDS reads the NCHW activation
        // directly: no transposed copy at all, whatever the number of tiles (on 8 x 512 x 4096 inputs,
        // k = 7, it still finishes before the tiled route: 120 against 147 us).
        // The conv_row option set to 0 takes the general route (tuning, tests).
        const bool row_off = ctx->tune.conv_row == 0;
        const int64_t slab_pos = (3 + 63 * g->stride_w + (g->kw - 1) * g->dil_w + 1 + 3) / 4 * 4;
        const size_t slab_bytes = (size_t)(slab_pos * g->c_in);
        if (!row_off && g->h == 1 && g->kh == 1 && ho == 1 && g->pad_top == 0 && g->w % 4 == 0 && aligned(X, 4) &&
            slab_bytes <= 64 * 1024) {
            ga.Q = static_cast<const uint8_t *>(X);
            ga.slab_pos = (int)slab_pos;
            const size_t lds = std::max(kSmallLds, slab_bytes);
            const dim3 grid(gemm_grid(ga, 64), 1, (unsigned)g->n);
            if (ep.requant) {
                if (zero_known) hipLaunchKernelGGL((int8_conv_row_kernel<EPI_REQUANT, false>), grid, 256, lds, ctx->stream, ga);
                else hipLaunchKernelGGL((int8_conv_row_kernel<EPI_REQUANT, true>), grid, 256, lds, ctx->stream, ga);
            } else {
                if (zero_known) hipLaunchKernelGGL((int8_conv_row_kernel<EPI_I32, false>), grid, 256, lds, ctx->stream, ga);
                else hipLaunchKernelGGL((int8_conv_row_kernel<EPI_I32, true>), grid, 256, lds, ctx->stream, ga);
            }
            HIPC_LAUNCHED(ctx);
            gemm_note_scalars(ctx, ga, !zero_known);
            return HIPC_OK;
        }

        // NHWC copy of the activation, shifted to the signed domain
        void *xt = nullptr;
        const size_t x_bytes = (size_t)(g->n * g->c_in * g->h * g->w);
        rc = scratch_get(ctx, 1, x_bytes + 16, &xt);
        if (rc != HIPC_OK) return rc;
        const int HW = (int)(g->h * g->w);
        if (g->c_in % 4 == 0 && HW % 4 == 0 && aligned(X, 4))
            hipLaunchKernelGGL((nchw_to_nhwc4_kernel), dim3((unsigned)ceil_div(HW, 64), (unsigned)ceil_div(g->c_in, 64), (unsigned)g->n), 256, 0, ctx->stream, static_cast<const uint8_t *>(X), static_cast<uint8_t *>(xt), (int)g->c_in, HW,
                                                  x_dtype == HIPC_U8 ? 0x80808080u : 0u);
        else
            hipLaunchKernelGGL((nchw_to_nhwc_kernel), dim3((unsigned)ceil_div(HW, 32), (unsigned)ceil_div(g->c_in, 32), (unsigned)g->n), 256, 0, ctx->stream, static_cast<const uint8_t *>(X), static_cast<uint8_t *>(xt), (int)g->c_in, HW,
                                                 x_dtype == HIPC_U8 ? 0x80 : 0);
        HIPC_LAUNCHED(ctx);
        ga.Q = static_cast<const uint8_t *>(xt);
        if (small) {
            const dim3 grid(gemm_grid(ga, 64), 1, (unsigned)g->n);
            if (ep.requant) {
                if (zero_known) hipLaunchKernelGGL((int8_conv_small_kernel<EPI_REQUANT, false>), grid, 256, kSmallLds, ctx->stream, ga);
                else hipLaunchKernelGGL((int8_conv_small_kernel<EPI_REQUANT, true>), grid, 256, kSmallLds, ctx->stream, ga);
            } else {
                if (zero_known) hipLaunchKernelGGL((int8_conv_small_kernel<EPI_I32, false>), grid, 256, kSmallLds, ctx->stream, ga);
                else hipLaunchKernelGGL((int8_conv_small_kernel<EPI_I32, true>), grid, 256, kSmallLds, ctx->stream, ga);
            }
            HIPC_LAUNCHED(ctx);
            gemm_note_scalars(ctx, ga, !zero_known);
            return HIPC_OK;
        }
        return ep.requant ? gemm_launch<MODE_CONV, EPI_REQUANT, true>(ctx, ga, (unsigned)g->n)
                          : gemm_launch<MODE_CONV, EPI_I32, true>(ctx, ga, (unsigned)g->n);
    }

    DirectConvArgs d{};
    d.X = static_cast<const uint8_t *>(X), d.W = W->raw;
    d.x_zp = static_cast<const uint8_t *>(x_zp), d.w_zp = static_cast<const uint8_t *>(w_zp);
    d.x_signed = x_dtype == HIPC_I8, d.w_signed = W->w_dtype == HIPC_I8;
    d.host_zp = host_zp, d.x_zp_value = x_zp_value, d.w_zp_value = w_zp_value;
    d.n = (int)g->n, d.C = (int)g->c_in, d.H = (int)g->h, d.Wd = (int)g->w, d.O = (int)g->c_out;
    d.kh = (int)g->kh, d.kw = (int)g->kw, d.sh = (int)g->stride_h, d.sw = (int)g->stride_w, d.dh = (int)g->dil_h,
    d.dw = (int)g->dil_w, d.pt = (int)g->pad_top, d.pl = (int)g->pad_left, d.group = (int)g->group;
    d.Ho = (int)ho, d.Wo = (int)wo;
    d.Y = Y;
    d.requant = ep.requant, d.ratio = ep.ratio, d.ratio_step = ep.ratio_step, d.qbias = ep.qbias, d.y_zp = ep.y_zp,
    d.out_signed = ep.out_signed;
    hipLaunchKernelGGL((conv_direct_kernel), dim3((unsigned)ceil_div(total, 256)), 256, 0, ctx->stream, d);
    HIPC_LAUNCHED(ctx);
    if (host_zp) {
        note_scalar(ctx, HIPC_SCALAR_A_ZERO_POINT, offsetof(DirectConvArgs, x_zp_value));
        note_scalar(ctx, HIPC_SCALAR_B_ZERO_POINT, offsetof(DirectConvArgs, w_zp_value));
    }
    if (ep.requant) note_scalar(ctx, HIPC_SCALAR_Y_ZERO_POINT, offsetof(DirectConvArgs, y_zp));
    return HIPC_OK;
}

}  // namespace

extern "C" {

int hipc_conv_out_shape(const hipc_conv_geom *g, int64_t *h_out, int64_t *w_out) {
    if (!g || !h_out || !w_out) return HIPC_ERR_INVALID;
    if (g->kh <= 0 || g->kw <= 0 || g->stride_h <= 0 || g->stride_w <= 0 || g->dil_h <= 0 || g->dil_w <= 0)
        return HIPC_ERR_INVALID;
    if (out_dim(g->h, g->pad_top, g->pad_bottom, g->kh, g->stride_h, g->dil_h, h_out) != HIPC_OK) return HIPC_ERR_INVALID;
    return out_dim(g->w, g->pad_left, g->pad_right, g->kw, g->stride_w, g->dil_w, w_out);
}

void hipc_same_pads(int64_t in, int64_t kernel, int64_t stride, int64_t dilation, int upper, int64_t *pad_begin,
                    int64_t *pad_end) {
    const int64_t out = (in + stride - 1) / stride;
    const int64_t span = dilation * (kernel - 1) + 1;
    int64_t total = (out - 1) * stride + span - in;
    if (total < 0) total = 0;
    const int64_t small = total / 2, large = total - small;
    *pad_begin = upper ? small : large;
    *pad_end = upper ? large : small;
}

int hipc_prepack_conv_w(hipc_ctx *ctx, const void *W, int w_dtype, const hipc_conv_geom *g, hipc_conv_weight **out) {
    if (!out) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        *out = nullptr;
        HIPC_REFUSE(ctx, ctx->capturing, "Conv prepack while a capture is open");
        HIPC_REFUSE(ctx, !is_byte_dtype(w_dtype), "Conv: W must be uint8 or int8, got %d", w_dtype);
        HIPC_REQUIRE(ctx, W && g, "Conv prepack: null argument");
        HIPC_REQUIRE(ctx, g->c_in > 0 && g->c_out > 0 && g->kh > 0 && g->kw > 0 && g->group > 0 && g->c_in % g->group == 0 &&
                              g->c_out % g->group == 0 && g->c_in * g->kh * g->kw < (int64_t(1) << 30),
                     "Conv prepack: bad weight shape");
        hipc_conv_weight *w = new hipc_conv_weight();
        w->geom = *g;
        w->w_dtype = w_dtype;
        const size_t raw_bytes = (size_t)(g->c_out * (g->c_in / g->group) * g->kh * g->kw);
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&w->raw), raw_bytes);
        if (e == hipSuccess)
            e = hipMemcpyAsync(w->raw, W, raw_bytes, hipMemcpyDeviceToDevice, ctx->stream);
        const bool mfma = g->group == 1 && g->c_in % 16 == 0;
        if (e == hipSuccess && mfma) {
            w->O_pad = (int)(ceil_div(g->c_out, kBM) * kBM);
            w->K_pad = (int)(ceil_div(g->c_in * g->kh * g->kw, kBK) * kBK);
            e = hipMalloc(reinterpret_cast<void **>(&w->Wp), (size_t)w->O_pad * w->K_pad);
            if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&w->rowsum), (size_t)w->O_pad * 4);
            if (e == hipSuccess) {
                hipLaunchKernelGGL((pack_conv_w_kernel), dim3((unsigned)w->O_pad), 256, 0, ctx->stream, static_cast<const uint8_t *>(W), w->Wp, w->rowsum, (int)g->c_out, (int)g->c_in, (int)g->kh, (int)g->kw,
                    w->O_pad, w->K_pad, w_dtype == HIPC_I8, w_dtype == HIPC_U8 ? 128 : 0);
                e = hipGetLastError();
            }
        }
        if (e != hipSuccess) {
            if (w->raw) (void)hipFree(w->raw);
            if (w->Wp) (void)hipFree(w->Wp);
            if (w->rowsum) (void)hipFree(w->rowsum);
            delete w;
            return fail(ctx, HIPC_ERR_BACKEND, "Conv prepack: %s", hipGetErrorString(e));
        }
        *out = w;
        return HIPC_OK;
    });
}

void hipc_conv_weight_destroy(hipc_ctx *ctx, hipc_conv_weight *w) {
    if (!w) return;
    entry_void(ctx, [&] {
        if (w->raw) ctx->deferred.push_back(w->raw);
        if (w->Wp) ctx->deferred.push_back(w->Wp);
        if (w->rowsum) ctx->deferred.push_back(w->rowsum);
        ratio_release(ctx, w->ratios);
        delete w;
    });
}

int hipc_conv_integer(hipc_ctx *ctx, const void *X, int x_dtype, const hipc_conv_weight *W, const void *x_zp,
                      const void *w_zp, const hipc_conv_geom *g, void *Y) {
    return entry(ctx, [&]() -> int {
        return run_conv(ctx, X, x_dtype, W, x_zp, w_zp, 0, 0, 0, g, Y, ConvEpilogue{});
    });
}

int hipc_qlinear_conv(hipc_ctx *ctx, const void *X, int x_dtype, float x_scale, int32_t x_zp, const hipc_conv_weight *W,
                      const float *w_scale, int64_t n_w_scale, int32_t w_zp, float y_scale, int32_t y_zp, int y_dtype,
                      const void *bias, const hipc_conv_geom *g, void *Y) {
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, g && w_scale, "QLinearConv: null geometry or scale");
        HIPC_REFUSE(ctx, !is_byte_dtype(y_dtype), "QLinearConv: output must be uint8 or int8, got %d", y_dtype);
        // the accepted envelope of `unsupported_quantization` (interp.rs:781-847)
        HIPC_REQUIRE(ctx, n_w_scale == 1 || n_w_scale == g->c_out, "QLinearConv: %ld weight scales for %ld channels",
                     (long)n_w_scale, (long)g->c_out);
        HIPC_REFUSE(ctx, n_w_scale > 1 && w_zp != 0, "QLinearConv: w per-channel zero point is not zero (asymmetric weights)");
        HIPC_REQUIRE(ctx, y_scale != 0.f, "QLinear: y_scale is zero");
        HIPC_REQUIRE(ctx, W, "QLinearConv: null weight");
        // ratio[c] = x_scale * w_scale[c] / y_scale (interp.rs:4693); a per-tensor scale is
        // broadcast to c_out so the bias stays per channel (interp.rs:4815-4823)
        std::vector<float> ratio((size_t)g->c_out);
        for (int64_t c = 0; c < g->c_out; c++) {
            volatile float t = x_scale * w_scale[n_w_scale == 1 ? 0 : c];
            ratio[(size_t)c] = t / y_scale;
        }
        const float *dratio = nullptr;
        int rc = ratio_resident(ctx, W->ratios, ratio, &dratio);
        if (rc != HIPC_OK) return rc;
        ConvEpilogue ep;
        ep.requant = 1;
        ep.ratio = dratio, ep.ratio_step = 1;
        ep.qbias = static_cast<const int32_t *>(bias);
        ep.y_zp = y_zp, ep.out_signed = y_dtype == HIPC_I8;
        return run_conv(ctx, X, x_dtype, W, nullptr, nullptr, 1, x_zp, w_zp, g, Y, ep);
    });
}

}  // extern "C"
