// Address model of the int8 operators: dynamic_quantize.hip, matmul_integer.hip and conv_integer.hip (with int8_gemm.h
// and int8_gemm_bdirect.h) compiled as host code behind gpu_model.h and driven through the entry points a caller uses.
// Every launch runs thread by thread on the CPU; every buffer load is checked against the allocations the library
// and this driver made (operands of exactly the operator's size, no slack), under the hardware's rule that the
// descriptor's range check sees the per-lane offset only -- the kernels that read B straight from the prepacked
// weight step along k in the SCALAR offset -- and every ordinary load and store is checked by AddressSanitizer.
// Values are not checked here (the matrix cores are stubs): parity is the GPU tests' business.
//
//   int8_model [quick]   DynamicQuantizeLinear (every entry point, aligned and unaligned, sizes around the vector and
//                        workgroup boundaries); every matrix-product route (LDS-staged 64 / 128 tiles, the k-split 64x64 kernel, the two
//                        B-direct kernels) on aligned, ragged and tiny shapes, u8 / i8 operands, zero points by
//                        pointer and by value, the three epilogues; the convolution routes (row-resident, gathered,
//                        tiled, grouped) on the shapes of the GPU tests. `quick` leaves out the largest shapes.
#include <cstdio>
#include <cstring>
#include <vector>

#include "internal.h"

namespace hipc {
alignas(16) thread_local uint8_t lds_raw[160 * 1024];   // the kernels' dynamic LDS (`extern __shared__`)
int scratch_get(hipc_ctx *ctx, int slot, size_t bytes, void **out) {
    Scratch &s = ctx->scratch[slot];
    if (s.bytes < bytes) {
        if (s.ptr) gpu_model::release(s.ptr);
        s.ptr = gpu_model::alloc(bytes);   // exactly what was asked for: stricter than the library's rounding
        s.bytes = bytes;
    }
    *out = s.ptr;
    return HIPC_OK;
}
int ratio_resident(hipc_ctx *, RatioCache &cache, const std::vector<float> &ratio, const float **out) {
    if (cache.dev) gpu_model::release(cache.dev);
    cache.dev = static_cast<float *>(gpu_model::alloc(ratio.size() * sizeof(float)));
    std::memcpy(cache.dev, ratio.data(), ratio.size() * sizeof(float));
    cache.host = ratio;
    *out = cache.dev;
    return HIPC_OK;
}
void ratio_release(hipc_ctx *, RatioCache &cache) {
    if (cache.dev) gpu_model::release(cache.dev);
    cache.dev = nullptr;
}
}  // namespace hipc
extern "C" {
const char *hipGetErrorString(hipError_t) { return "model"; }
hipError_t hipSetDevice(int) { return hipSuccess; }
hipError_t hipEventCreate(hipEvent_t *) { return hipSuccess; }
hipError_t hipEventDestroy(hipEvent_t) { return hipSuccess; }
hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
hipError_t hipEventElapsedTime(float *ms, hipEvent_t, hipEvent_t) { *ms = 1.f; return hipSuccess; }
hipError_t hipStreamGetCaptureInfo_v2(hipStream_t, hipStreamCaptureStatus *status, unsigned long long *, hipGraph_t *, const hipGraphNode_t **, size_t *n) {
    *status = hipStreamCaptureStatusNone, *n = 0;
    return hipSuccess;
}
}

#define MUST(call)                                                                    \
    do {                                                                              \
        const int rc_ = (call);                                                       \
        if (rc_ != HIPC_OK) {                                                         \
            std::printf("FAILED %s:%d: %s -> %d (%s)\n", __FILE__, __LINE__, #call, rc_, ctx.err.c_str()); \
            std::exit(1);                                                             \
        }                                                                             \
    } while (0)

namespace {

hipc_ctx ctx;
std::vector<void *> inputs;
void *input(size_t bytes, int fill = 0) {
    void *p = gpu_model::alloc(bytes);
    std::memset(p, fill, bytes);
    inputs.push_back(p);
    return p;
}
void release_all() {
    for (void *p : ctx.deferred) gpu_model::release(p);
    ctx.deferred.clear();
    for (void *p : inputs) gpu_model::release(p);
    inputs.clear();
}
void report(const char *what) {
    gpu_model::Registry &g = gpu_model::reg();
    std::printf("%-64s %6zu launches %10zu threads %10zu buffer loads (%zu answered with zeros)\n", what, g.launches, g.threads, g.loads, g.loads_clipped);
    std::fflush(stdout);
    g.launches = g.threads = g.loads = g.loads_clipped = 0;
}

struct Route {
    const char *name;
    int tile, big, small_;   // HIPC_GEMM_TILE, HIPC_GEMM_BIG, HIPC_GEMM_SMALL (-1: the library's choice)
};
const Route kRoutes[] = {
    {"library's choice", -1, -1, -1},       {"LDS-staged 64x64", 64, 0, 0},       {"LDS-staged 128x128", 128, 0, 0},
    {"k-split 64x64 (B not in LDS)", -1, 0, 1}, {"B-direct 256x256", -1, 1, 0},   {"B-direct 128x128", -1, 2, 0},
};

// one matrix product through the three epilogues
void products(int64_t M, int64_t K, int64_t N, int a_dtype, int b_dtype, bool zp_by_pointer) {
    void *A = input((size_t)M * K, 3), *B = input((size_t)K * N, 5);
    hipc_int8_weight *w = nullptr;
    MUST(hipc_prepack_int8_b(&ctx, B, b_dtype, K, N, &w));
    void *azp = zp_by_pointer ? input(1, 7) : nullptr, *bzp = zp_by_pointer ? input(1, 2) : nullptr;
    void *Y = input((size_t)M * N * 4);
    for (const Route &r : kRoutes) {
        ctx.tune.gemm_tile = r.tile, ctx.tune.gemm_big = r.big, ctx.tune.gemm_small = r.small_;
        char where[160];
        std::snprintf(where, sizeof where, "%lld x %lld x %lld %s x %s, %s", (long long)M, (long long)K, (long long)N, a_dtype == HIPC_U8 ? "u8" : "i8",
                      b_dtype == HIPC_U8 ? "u8" : "i8", r.name);
        gpu_model::reg().where = where;
        MUST(hipc_matmul_integer(&ctx, A, a_dtype, w, azp, bzp, Y, M));
        void *scale = input((size_t)N * 4), *bias = input((size_t)N * 4), *range = input(8);
        MUST(hipc_matmul_integer_scale_bias(&ctx, A, a_dtype, w, azp, bzp, scale, 1, nullptr, 0, bias, 1, 1, range, Y, M));
        std::vector<float> bs((size_t)N, 0.01f);
        MUST(hipc_qlinear_matmul(&ctx, A, a_dtype, 0.02f, a_dtype == HIPC_U8 ? 128 : 5, w, bs.data(), N, 0, 0.05f, 128, HIPC_U8, Y, M));                       // per-channel scales
        MUST(hipc_qlinear_matmul(&ctx, A, a_dtype, 0.02f, 0, w, bs.data(), 1, b_dtype == HIPC_U8 ? 131 : 3, 0.05f, -3, HIPC_I8, Y, M));   // one scale, a weight zero point
    }
    ctx.tune.gemm_tile = ctx.tune.gemm_big = ctx.tune.gemm_small = -1;
    hipc_int8_weight_destroy(&ctx, w);
    release_all();
}

void conv(int64_t n, int64_t c_in, int64_t h, int64_t w, int64_t c_out, int64_t kh, int64_t kw, int64_t sh, int64_t sw, int64_t dh, int64_t dw,
          int64_t pt, int64_t pl, int64_t pb, int64_t pr, int64_t group, int x_dtype, const char *what) {
    hipc_conv_geom g{n, c_in, h, w, c_out, kh, kw, sh, sw, dh, dw, pt, pl, pb, pr, group};
    int64_t ho = 0, wo = 0;
    MUST(hipc_conv_out_shape(&g, &ho, &wo));
    void *X = input((size_t)(n * c_in * h * w), 9), *W = input((size_t)(c_out * (c_in / group) * kh * kw), 1);
    hipc_conv_weight *cw = nullptr;
    MUST(hipc_prepack_conv_w(&ctx, W, HIPC_I8, &g, &cw));
    void *Y = input((size_t)(n * c_out * ho * wo) * 4), *xzp = input(1, 128), *bias = input((size_t)c_out * 4);
    std::vector<float> ws((size_t)c_out, 0.01f);
    for (int row = -1; row <= 0; row++) {   // the library's choice, then without the row-resident route
        ctx.tune.conv_row = row;
        gpu_model::reg().where = what;
        MUST(hipc_conv_integer(&ctx, X, x_dtype, cw, xzp, nullptr, &g, Y));
        MUST(hipc_qlinear_conv(&ctx, X, x_dtype, 0.02f, 128, cw, ws.data(), c_out, 0, 0.05f, 128, HIPC_U8, bias, &g, Y));
        MUST(hipc_qlinear_conv(&ctx, X, x_dtype, 0.02f, 128, cw, ws.data(), 1, 0, 0.05f, 0, HIPC_I8, nullptr, &g, Y));
    }
    ctx.tune.conv_row = -1;
    hipc_conv_weight_destroy(&ctx, cw);
    release_all();
}

}  // namespace

// DynamicQuantizeLinear on n values: the context's range slot and a caller's, the variant that allocates nothing,
// the fused GELU, the GELU alone -- X with the alignment given (vector loads need 16 bytes, the others take the
// element path), Y and the two parameters of exactly their sizes
void quantize(int64_t n, int misalign) {
    uint8_t *xraw = static_cast<uint8_t *>(input((size_t)n * 4 + 16));
    void *X = xraw + misalign;
    void *Y = input((size_t)(n > 0 ? n : 1)), *scale = input(4), *zp = input(1), *range = input(8), *G = input((size_t)(n > 0 ? n : 1) * 4);
    char where[96];
    std::snprintf(where, sizeof where, "DynamicQuantizeLinear, %lld values, X at +%d", (long long)n, misalign);
    gpu_model::reg().where = where;
    MUST(hipc_dynamic_quantize_linear(&ctx, X, n, Y, scale, zp, nullptr, 0));
    MUST(hipc_dynamic_quantize_linear(&ctx, X, n, Y, scale, zp, range, 0));
    MUST(hipc_dynamic_quantize_linear(&ctx, X, n, Y, scale, zp, range, 1));
    MUST(hipc_dynamic_quantize_linear_static(&ctx, X, n, Y, scale, zp));
    MUST(hipc_dynamic_quantize_linear_gelu(&ctx, X, n, 1.41421356f, 1.f, 0.5f, 0, Y, scale, zp, nullptr));
    MUST(hipc_decomposed_gelu(&ctx, X, n, 1.41421356f, 1.f, 0.5f, 1, G));
    release_all();
}

int main(int argc, char **argv) {
    const bool quick = argc > 1 && std::strcmp(argv[1], "quick") == 0;
    ctx.params = gpu_model::alloc(hipc::kParamBytes);
    ctx.cu_count = 256;
    MUST(hipc::dql_static_init(&ctx));
    for (int64_t n : {0, 1, 3, 4, 5, 255, 256, 257, 1000, 4096, 4099, 65536 + 7, 1000 * 1024})
        for (int misalign : {0, 4}) quantize(n, misalign);
    report("DynamicQuantizeLinear and the decomposed GELU");
    // matrix products: tiny, ragged in every direction, aligned, one tile more than a multiple, both signs
    const int64_t shapes[][3] = {{1, 8, 1}, {5, 7, 3}, {33, 100, 65}, {64, 128, 64}, {129, 257, 130}, {200, 512, 264}, {256, 1024, 512}, {300, 640, 520}};
    for (const auto &s : shapes) {
        products(s[0], s[1], s[2], HIPC_U8, HIPC_I8, true);
        products(s[0], s[1], s[2], HIPC_I8, HIPC_U8, false);
    }
    report("matrix products, six routes x four epilogue calls");
    if (!quick) {
        products(1000, 1024, 4096, HIPC_U8, HIPC_I8, true);   // the benchmark's pair
        products(1000, 4096, 1024, HIPC_U8, HIPC_I8, true);
        report("1000 x 1024 x 4096 and 1000 x 4096 x 1024");
    }
    // convolutions: the benchmark's 1-D shapes (dilations 1 / 3 / 5, same padding), a strided 2-D one, a grouped one
    for (int d : {1, 3, 5}) conv(1, 192, 1, quick ? 300 : 4096, 192, 1, 7, 1, 1, 1, d, 0, 3 * d, 0, 3 * d, 1, HIPC_U8, "192 channels, 1 x 7, dilated");
    conv(2, 24, 19, 23, 40, 3, 3, 2, 2, 1, 1, 1, 1, 1, 1, 1, HIPC_U8, "2-D 3 x 3, stride 2");
    conv(1, 32, 1, 200, 64, 1, 5, 1, 2, 1, 2, 0, 4, 0, 4, 4, HIPC_I8, "grouped, 1 x 5, stride 2, dilation 2");
    conv(1, 20, 9, 11, 33, 2, 4, 1, 1, 2, 1, 1, 0, 0, 3, 1, HIPC_U8, "ragged channels, 2 x 4");
    if (!quick) conv(1, 512, 1, 1024, 512, 1, 7, 1, 1, 1, 1, 0, 3, 0, 3, 1, HIPC_U8, "512 channels, 1 x 7");
    report("convolutions");
    for (hipc::Scratch &s : ctx.scratch)
        if (s.ptr) gpu_model::release(s.ptr);
    gpu_model::release(ctx.params);
    release_all();
    std::printf("ok\n");
    return 0;
}
