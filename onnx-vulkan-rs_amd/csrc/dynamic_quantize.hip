// DynamicQuantizeLinear for gfx950.
//
// Reference: crates/onnx-vulkan-core/src/shaders/dynamic_quantize.rs:106-222 (the two
// passes and the range slot), interp.rs:1945-2085 (host side), definition
// tests/dynamic_quantize.rs:16-26.
//
// The range slot is 8 bytes {bits(-min), bits(max)}. The range always contains 0,
// so both values are >= 0 and their bit patterns order like the values: an
// unsigned atomicMax on the words is a float max, independent of the order the
// workgroups arrive in. The reference replaces `/` by a double-single reciprocal
// because Vulkan's OpFDiv may be 2.5 ULP off; here `__fdiv_rn` is the IEEE
// division, so the operator's definition is evaluated as written.
#include "internal.h"

namespace hipc {

// Range partials of hipc_dynamic_quantize_linear_static: {bits(-min), bits(max)} per workgroup of
// the first pass, kParamPartsMax pairs = 16 KiB, part of the library's device image. In host code
// this name is a stand-in, not a device address: dql_static_init asks the runtime where the array
// lives on the context's device, and every launch gets that pointer.
static __device__ __align__(256) __attribute__((used)) uint32_t scratch[2 * kParamPartsMax];

int dql_static_init(hipc_ctx *ctx) {
    void *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) return HIPC_ERR_BACKEND;
    ctx->dql_static = ptr;
    return HIPC_OK;
}

// What the quantizer reads: x itself, or DecomposedGelu(x), the exact GELU written out as
// Div -> Erf -> Add -> Mul -> Mul and fused by the reference (rewrite.rs:683-735). Every step rounds
// on its own, as the five kernels it replaces do (shaders/elementwise.rs:71-118): this file is
// compiled with floating-point contraction off, so the fused quantizer and the plain GELU kernel
// below evaluate bit for bit the same function.
struct GeluParams {
    int on;             // 0: the identity
    float divisor, offset, factor;
    int factor_first;   // x * ((erf + offset) * factor) instead of (x * (erf + offset)) * factor
};

__device__ __forceinline__ float erf_approx(float x) {  // shaders/elementwise.rs:71-80 (Abramowitz-Stegun 7.1.26)
    const float s = x > 0.f ? 1.f : (x < 0.f ? -1.f : 0.f);
    const float a = fabsf(x);
    const float t = 1.f / (1.f + 0.3275911f * a);
    const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
    return s * (1.f - poly * expf(-a * a));
}

__device__ __forceinline__ float gelu_load(float v, const GeluParams &g) {
    if (!g.on) return v;
    const float e = erf_approx(v / g.divisor) + g.offset;
    return g.factor_first ? v * (e * g.factor) : (v * e) * g.factor;
}

__global__ void __launch_bounds__(256)
decomposed_gelu_kernel(const float *__restrict__ x, long n, GeluParams g, float *__restrict__ y) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] = gelu_load(x[i], g);
}

__global__ void dql_clear_range_kernel(uint32_t *range) {
    if (threadIdx.x < 2) range[threadIdx.x] = 0u;
}

__global__ void __launch_bounds__(256)
dql_range_kernel(const float *__restrict__ x, long n, uint32_t *__restrict__ range, int vec_ok, int per_block, GeluParams g) {
    float mn = 0.f, mx = 0.f;
    auto L = [&](float4 v) { return g.on ? make_float4(gelu_load(v.x, g), gelu_load(v.y, g), gelu_load(v.z, g), gelu_load(v.w, g)) : v; };
    const long tid = (long)blockIdx.x * 256 + threadIdx.x;
    const long nthreads = (long)gridDim.x * 256;
    if (vec_ok) {
        const long n4 = n >> 2;
        const float4 *x4 = reinterpret_cast<const float4 *>(x);
        long i = tid;
        for (; i + 3 * nthreads < n4; i += 4 * nthreads) {  // four independent loads in flight
            const float4 a = L(x4[i]), b = L(x4[i + nthreads]), c = L(x4[i + 2 * nthreads]), d = L(x4[i + 3 * nthreads]);
            mn = fminf(mn, fminf(fminf(fminf(a.x, a.y), fminf(a.z, a.w)), fminf(fminf(b.x, b.y), fminf(b.z, b.w))));
            mn = fminf(mn, fminf(fminf(fminf(c.x, c.y), fminf(c.z, c.w)), fminf(fminf(d.x, d.y), fminf(d.z, d.w))));
            mx = fmaxf(mx, fmaxf(fmaxf(fmaxf(a.x, a.y), fmaxf(a.z, a.w)), fmaxf(fmaxf(b.x, b.y), fmaxf(b.z, b.w))));
            mx = fmaxf(mx, fmaxf(fmaxf(fmaxf(c.x, c.y), fmaxf(c.z, c.w)), fmaxf(fmaxf(d.x, d.y), fmaxf(d.z, d.w))));
        }
        for (; i < n4; i += nthreads) {
            const float4 v = L(x4[i]);
            mn = fminf(mn, fminf(fminf(v.x, v.y), fminf(v.z, v.w)));
            mx = fmaxf(mx, fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w)));
        }
        for (long i = (n4 << 2) + tid; i < n; i += nthreads) {
            const float v = gelu_load(x[i], g);
            mn = fminf(mn, v);
            mx = fmaxf(mx, v);
        }
    } else {
        for (long i = tid; i < n; i += nthreads) {
            const float v = gelu_load(x[i], g);
            mn = fminf(mn, v);
            mx = fmaxf(mx, v);
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        mn = fminf(mn, __shfl_xor(mn, off, 64));
        mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    }
    __shared__ float smn[4], smx[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) smn[wave] = mn, smx[wave] = mx;
    __syncthreads();
    if (threadIdx.x == 0) {
        mn = fminf(fminf(smn[0], smn[1]), fminf(smn[2], smn[3]));
        mx = fmaxf(fmaxf(smx[0], smx[1]), fmaxf(smx[2], smx[3]));
        // -0.0 counts as 0: drop the sign bit
        if (per_block) {  // one {bits(-min), bits(max)} pair per workgroup, joined by the quantize pass
            range[2 * blockIdx.x] = __float_as_uint(-mn) & 0x7fffffffu;
            range[2 * blockIdx.x + 1] = __float_as_uint(mx) & 0x7fffffffu;
        } else {
            atomicMax(&range[0], __float_as_uint(-mn) & 0x7fffffffu);
            atomicMax(&range[1], __float_as_uint(mx) & 0x7fffffffu);
        }
    }
}

__device__ __forceinline__ void dql_params(const uint32_t *range, float &scale, float &zp) {
    const float neg_min = __uint_as_float(range[0]);
    const float mx = __uint_as_float(range[1]);
    // max - min with min = -neg_min; max == min only when both are 0
    const float span = __fadd_rn(mx, neg_min);
    scale = span == 0.f ? 1.f : __fdiv_rn(span, 255.f);
    zp = rintf(fminf(fmaxf(__fdiv_rn(neg_min, scale), 0.f), 255.f));
}

__device__ __forceinline__ uint32_t dql_one(float v, float scale, float zp) {
    const float q = __fadd_rn(rintf(__fdiv_rn(v, scale)), zp);
    return (uint32_t)fminf(fmaxf(q, 0.f), 255.f);
}

// four values per thread, packed into one 32-bit store where the output allows it
__global__ void __launch_bounds__(256)
dql_quantize_kernel(const float *__restrict__ x, long n, const uint32_t *__restrict__ range, int nparts,
                    uint8_t *__restrict__ y, float *__restrict__ scale_out, uint8_t *__restrict__ zp_out, int vec_ok,
                    GeluParams g) {
    float scale, zp;
    if (nparts > 0) {
        // range holds nparts pairs: every workgroup joins them itself; the maximum of
        // non-negative floats is the maximum of their bit patterns
        __shared__ uint32_t joined[2];
        __shared__ uint32_t wave_max[4][2];
        uint32_t a = 0, b = 0;
        for (int i = threadIdx.x; i < nparts; i += 256) a = max(a, range[2 * i]), b = max(b, range[2 * i + 1]);
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            a = max(a, (uint32_t)__shfl_xor((int)a, off, 64));
            b = max(b, (uint32_t)__shfl_xor((int)b, off, 64));
        }
        if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6][0] = a, wave_max[threadIdx.x >> 6][1] = b;
        __syncthreads();
        if (threadIdx.x == 0) {
            joined[0] = max(max(wave_max[0][0], wave_max[1][0]), max(wave_max[2][0], wave_max[3][0]));
            joined[1] = max(max(wave_max[0][1], wave_max[1][1]), max(wave_max[2][1], wave_max[3][1]));
        }
        __syncthreads();
        dql_params(joined, scale, zp);
    } else {
        dql_params(range, scale, zp);
    }
    const long i4 = (long)blockIdx.x * 256 + threadIdx.x;
    if (i4 == 0) {
        *scale_out = scale;
        *zp_out = (uint8_t)zp;
    }
    const long base = i4 << 2;
    if (base >= n) return;
    if (vec_ok && base + 4 <= n) {
        float4 v = reinterpret_cast<const float4 *>(x)[i4];
        if (g.on) v = make_float4(gelu_load(v.x, g), gelu_load(v.y, g), gelu_load(v.z, g), gelu_load(v.w, g));
        const uint32_t packed = dql_one(v.x, scale, zp) | dql_one(v.y, scale, zp) << 8 |
                                dql_one(v.z, scale, zp) << 16 | dql_one(v.w, scale, zp) << 24;
        reinterpret_cast<uint32_t *>(y)[i4] = packed;
    } else {
        for (long i = base; i < n && i < base + 4; i++) y[i] = (uint8_t)dql_one(gelu_load(x[i], g), scale, zp);
    }
}

__global__ void dql_empty_kernel(float *scale_out, uint8_t *zp_out) {
    if (threadIdx.x == 0) {
        *scale_out = 1.f;
        *zp_out = 0;
    }
}

}  // namespace hipc

using namespace hipc;

namespace {

// `parts`: where the per-workgroup range pairs of a call without a caller-owned slot go (the
// context's own block, or this device's static array)
int dql_launch(hipc_ctx *ctx, const void *X, int64_t n, void *Y, void *scale_out, void *zp_out, void *range, int range_ready,
               const GeluParams &gelu, uint32_t *parts = nullptr) {
    HIPC_REQUIRE(ctx, n >= 0, "DynamicQuantizeLinear: negative length");
    HIPC_REQUIRE(ctx, scale_out && zp_out, "DynamicQuantizeLinear: null scale or zero-point output");
    HIPC_REQUIRE(ctx, aligned(scale_out, 4), "DynamicQuantizeLinear: scale output must be 4-byte aligned");
    if (n == 0) {  // empty input: y empty, scale 1, zero point 0 (interp.rs:1949-1966)
        hipLaunchKernelGGL((dql_empty_kernel), 1, 64, 0, ctx->stream, static_cast<float *>(scale_out), static_cast<uint8_t *>(zp_out));
        HIPC_LAUNCHED(ctx);
        return HIPC_OK;
    }
    HIPC_REQUIRE(ctx, X && Y, "DynamicQuantizeLinear: null tensor");
    HIPC_REQUIRE(ctx, aligned(X, 4), "DynamicQuantizeLinear: input must be 4-byte aligned");
    uint32_t *slot = static_cast<uint32_t *>(range ? range : static_cast<void *>(static_cast<char *>(ctx->params) + kParamRange));
    HIPC_REQUIRE(ctx, aligned(slot, 4), "DynamicQuantizeLinear: range slot must be 4-byte aligned");
    HIPC_REQUIRE(ctx, !(range_ready && !range), "DynamicQuantizeLinear: range_ready needs a caller-owned range slot");
    const int vec_ok = aligned(X, 16) && aligned(Y, 4);
    const float *x = static_cast<const float *>(X);
    int nparts = 0;
    if (!range_ready && !range) {
        // no slot of the caller's to fill: per-workgroup pairs in the context's block, joined by the
        // second pass -- no clearing launch and no atomics
        slot = parts ? parts : reinterpret_cast<uint32_t *>(static_cast<char *>(ctx->params) + kParamParts);
        nparts = (int)std::min<long>(std::max<long>(ceil_div(n, 256 * 16), 1), kParamPartsMax);
        hipLaunchKernelGGL((dql_range_kernel), (unsigned)nparts, 256, 0, ctx->stream, x, (long)n, slot, vec_ok, 1, gelu);
        HIPC_LAUNCHED(ctx);
    } else if (!range_ready) {
        hipLaunchKernelGGL((dql_clear_range_kernel), 1, 64, 0, ctx->stream, slot);
        HIPC_LAUNCHED(ctx);
        // enough workgroups to pull from every HBM channel, few enough that the atomics are noise
        const long want = ceil_div(n, 256 * 16);
        const unsigned grid = (unsigned)std::min<long>(std::max<long>(want, 1), 8L * ctx->cu_count);
        hipLaunchKernelGGL((dql_range_kernel), grid, 256, 0, ctx->stream, x, (long)n, slot, vec_ok, 0, gelu);
        HIPC_LAUNCHED(ctx);
    }
    const long quads = ceil_div(n, 4);
    HIPC_REQUIRE(ctx, ceil_div(quads, 256) < (int64_t(1) << 31), "DynamicQuantizeLinear: tensor too large");
    hipLaunchKernelGGL((dql_quantize_kernel), (unsigned)ceil_div(quads, 256), 256, 0, ctx->stream, x, (long)n, slot, nparts, static_cast<uint8_t *>(Y), static_cast<float *>(scale_out), static_cast<uint8_t *>(zp_out),
        vec_ok, gelu);
    HIPC_LAUNCHED(ctx);
    return HIPC_OK;
}

int gelu_params(hipc_ctx *ctx, float divisor, float offset, float factor, int factor_first, GeluParams *out) {
    HIPC_REQUIRE(ctx, divisor == divisor && offset == offset && factor == factor && divisor != 0.f, "DecomposedGelu: bad constants");
    *out = GeluParams{1, divisor, offset, factor, factor_first != 0};
    return HIPC_OK;
}

}  // namespace

extern "C" {

int hipc_dynamic_quantize_linear(hipc_ctx *ctx, const void *X, int64_t n, void *Y, void *scale_out, void *zp_out,
                                 void *range, int range_ready) {
    return entry(ctx, [&]() -> int {
        return dql_launch(ctx, X, n, Y, scale_out, zp_out, range, range_ready, GeluParams{0, 1.f, 0.f, 1.f, 0});
    });
}

int hipc_dynamic_quantize_linear_static(hipc_ctx *ctx, const void *X, int64_t n, void *Y, void *scale_out, void *zp_out) {
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, n <= HIPC_DQL_STATIC_MAX_N, "DynamicQuantizeLinear (static): %ld elements exceed the limit of %ld", (long)n,
                     (long)HIPC_DQL_STATIC_MAX_N);
        HIPC_REQUIRE(ctx, ctx->dql_static, "DynamicQuantizeLinear (static): the static array was not found on this device");
        // every pair the second pass reads is written by the first pass of this same call, so
        // what an earlier (larger) call left in the array is never seen and nothing needs clearing
        return dql_launch(ctx, X, n, Y, scale_out, zp_out, nullptr, 0, GeluParams{0, 1.f, 0.f, 1.f, 0},
                          static_cast<uint32_t *>(ctx->dql_static));
    });
}

int hipc_dynamic_quantize_linear_gelu(hipc_ctx *ctx, const void *X, int64_t n, float divisor, float offset, float factor,
                                      int factor_first, void *Y, void *scale_out, void *zp_out, void *range) {
    return entry(ctx, [&]() -> int {
        GeluParams gp;
        if (int rc = gelu_params(ctx, divisor, offset, factor, factor_first, &gp)) return rc;
        return dql_launch(ctx, X, n, Y, scale_out, zp_out, range, 0, gp);
    });
}

int hipc_decomposed_gelu(hipc_ctx *ctx, const void *X, int64_t n, float divisor, float offset, float factor,
                         int factor_first, void *Y) {
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, n >= 0, "DecomposedGelu: negative length");
        GeluParams gp;
        if (int rc = gelu_params(ctx, divisor, offset, factor, factor_first, &gp)) return rc;
        if (n == 0) return HIPC_OK;
        HIPC_REQUIRE(ctx, X && Y && aligned(X, 4) && aligned(Y, 4), "DecomposedGelu: null or unaligned tensor");
        HIPC_REQUIRE(ctx, ceil_div(n, 256) < (int64_t(1) << 31), "DecomposedGelu: tensor too large");
        hipLaunchKernelGGL((decomposed_gelu_kernel), (unsigned)ceil_div(n, 256), 256, 0, ctx->stream, static_cast<const float *>(X), (long)n, gp,
                                                                                    static_cast<float *>(Y));
        HIPC_LAUNCHED(ctx);
        return HIPC_OK;
    });
}

}  // extern "C"
