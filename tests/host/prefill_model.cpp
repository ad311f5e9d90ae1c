// Address model of the tiled MatMulNBits kernels (many rows of f16 or f32 activations): matmul_nbits_prefill.hip,
// compiled twice as the library does, with matmul_nbits.hip for the prepack and the operator's entry point, as host
// code behind gpu_model.h. Every launch runs thread by thread on the CPU; the operands are allocations of exactly the
// operator's sizes (no slack), and AddressSanitizer checks every load and store of every thread: the clamped rows
// and tiles past the edges of ragged shapes, the stage past the end of an odd stage count, the k split's partials.
// Values are not checked here (the matrix cores are stubs): parity is the GPU tests' business.
//
//   prefill_model   every instance (64x64, 128x128 and 128x192 tiles with the weight read into operand registers,
//                   one or two groups of wavefronts per workgroup; 64x64 and 128x128 with both operands through LDS),
//                   every scale grouping, k split 1 / 2 / 3 ways,
//                   f16 rows and f32 rows, on ragged and aligned shapes; then the operator with few rows, on the ONNX
//                   layout (block sizes 8, 24, 40 among them) and on the decode kernels.
#include <cstdio>
#include <cstring>
#include <vector>

#include "internal.h"

namespace hipc {
alignas(16) thread_local uint8_t lds_raw[160 * 1024];   // the kernels' dynamic LDS (`extern __shared__`)
alignas(16) thread_local uint4 lean_smem[160 * 1024 / 16];
alignas(16) thread_local uint4 smem[160 * 1024 / 16];
thread_local float wgt[40960];
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
}  // namespace hipc
extern "C" {
const char *hipGetErrorString(hipError_t) { return "model"; }
hipError_t hipMemcpy(void *d, const void *s, size_t n, hipMemcpyKind) { std::memcpy(d, s, n); return hipSuccess; }
hipError_t hipSetDevice(int) { return hipSuccess; }
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
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
size_t prefill_launches = 0;

struct Route {
    int tile, direct, split, groups;   // HIPC_PREFILL_TILE, _DIRECT, _SPLIT, _GROUPS (-1: the library's choice)
};
const Route kRoutes[] = {{-1, -1, -1, -1}, {64, -1, -1, -1}, {64, 0, -1, -1},  {128, -1, 0, 1},  {128, -1, 2, 1}, {128, 0, 3, -1}, {128, 0, 0, -1},
                         {192, -1, 0, 1},  {192, -1, 2, 1},  {192, -1, 3, 1},  {128, -1, 0, 2},  {128, -1, 2, 2}, {192, -1, 0, 2},  {192, -1, 3, 2},
                         {64, -1, -1, 2},  {64, -1, -1, 1}};

void product(int64_t M, int64_t K, int64_t N, int64_t bs, bool with_zp, int a_dtype) {
    const int64_t nb = (K + bs - 1) / bs;
    const size_t b_len = (size_t)(N * nb * bs / 2), s_len = (size_t)(N * nb), z_len = (size_t)(N * ((nb + 1) / 2));
    const size_t esz = a_dtype == HIPC_F16 ? 2 : 4;
    std::vector<uint8_t> B(b_len, 0x5a), Z(z_len, 0x88), S(s_len * esz, 0);
    hipc_nbits_weight *w = nullptr;
    MUST(hipc_prepack_matmul_nbits(&ctx, B.data(), b_len, S.data(), a_dtype, s_len, with_zp ? Z.data() : nullptr, with_zp ? z_len : 0, K, N, bs, &w));
    void *A = gpu_model::alloc((size_t)(M * K) * esz), *Y = gpu_model::alloc((size_t)(M * N) * esz);
    std::memset(A, 0, (size_t)(M * K) * esz);
    for (const Route &r : kRoutes) {
        ctx.tune.prefill_tile = r.tile, ctx.tune.prefill_direct = r.direct, ctx.tune.prefill_split = r.split, ctx.tune.prefill_groups = r.groups;
        char where[160];
        std::snprintf(where, sizeof where, "%lld x %lld x %lld block %lld %s, tile %d direct %d split %d groups %d", (long long)M, (long long)K, (long long)N, (long long)bs,
                      a_dtype == HIPC_F16 ? "f16" : "f32", r.tile, r.direct, r.split, r.groups);
        gpu_model::reg().where = where;
        MUST(hipc_matmul_nbits_packed(&ctx, A, a_dtype, w, Y, M, 0));
        // (f32 rows at a level that allows f16 activations: one term per row, the kernel scales the result's rows)
        if (a_dtype == HIPC_F32) MUST(hipc_matmul_nbits_packed(&ctx, A, a_dtype, w, Y, M, 2));
        // (and with f32 pinned: three terms per row, 3 M rows and the launch that adds them)
        if (a_dtype == HIPC_F32) MUST(hipc_matmul_nbits_packed(&ctx, A, a_dtype, w, Y, M, 1));
    }
    ctx.tune.prefill_tile = ctx.tune.prefill_direct = ctx.tune.prefill_split = ctx.tune.prefill_groups = -1;
    // the operator on the ONNX layout with this many rows: the tiled form goes to scratch memory first
    gpu_model::reg().where = "many rows on the ONNX layout";
    MUST(hipc_matmul_nbits(&ctx, A, a_dtype, B.data(), b_len, S.data(), a_dtype, s_len, with_zp ? Z.data() : nullptr, with_zp ? z_len : 0, Y, M, K, N, bs, 0));
    gpu_model::release(A), gpu_model::release(Y);
    hipc_nbits_weight_destroy(&ctx, w);
    for (void *p : ctx.deferred) gpu_model::release(p);
    ctx.deferred.clear();
}

// the operator on the ONNX layout (no prepack: the kernel that takes every block size the reference takes) and, on a
// prepacked weight, the row counts the decode kernels serve
void rows(int64_t M, int64_t K, int64_t N, int64_t bs, bool with_zp, int a_dtype) {
    const int64_t nb = (K + bs - 1) / bs;
    const size_t b_len = (size_t)(N * nb * bs / 2), s_len = (size_t)(N * nb), z_len = (size_t)(N * ((nb + 1) / 2));
    const size_t esz = a_dtype == HIPC_F16 ? 2 : 4;
    void *B = gpu_model::alloc(b_len), *S = gpu_model::alloc(s_len * esz), *Z = gpu_model::alloc(z_len);
    std::memset(B, 0x5a, b_len), std::memset(S, 0, s_len * esz), std::memset(Z, 0x88, z_len);
    void *A = gpu_model::alloc((size_t)(M * K) * esz), *Y = gpu_model::alloc((size_t)(M * N) * esz);
    std::memset(A, 0, (size_t)(M * K) * esz);
    char where[160];
    std::snprintf(where, sizeof where, "%lld x %lld x %lld block %lld %s, ONNX layout / decode kernels", (long long)M, (long long)K, (long long)N, (long long)bs,
                  a_dtype == HIPC_F16 ? "f16" : "f32");
    gpu_model::reg().where = where;
    for (int level : {0, 1})
        MUST(hipc_matmul_nbits(&ctx, A, a_dtype, B, b_len, S, a_dtype, s_len, with_zp ? Z : nullptr, with_zp ? z_len : 0, Y, M, K, N, bs, level));
    {   // (a block size without a tiled form: the handle's own copies of the tensors, exactly as long as they are)
        hipc_nbits_weight *w = nullptr;
        MUST(hipc_prepack_matmul_nbits(&ctx, B, b_len, S, a_dtype, s_len, with_zp ? Z : nullptr, with_zp ? z_len : 0, K, N, bs, &w));
        for (int level : {0, 1}) MUST(hipc_matmul_nbits_packed(&ctx, A, a_dtype, w, Y, M, level));
        for (int lean = 0; lean <= 1 && M == 1; lean++) {
            ctx.tune.gemv_lean = lean;
            MUST(hipc_matmul_nbits_packed(&ctx, A, a_dtype, w, Y, M, 0));
        }
        ctx.tune.gemv_lean = -1;
        hipc_nbits_weight_destroy(&ctx, w);
    }
    for (void *p : {A, Y, B, S, Z}) gpu_model::release(p);
    for (void *p : ctx.deferred) gpu_model::release(p);
    ctx.deferred.clear();
}

}  // namespace

int main() {
    ctx.params = gpu_model::alloc(hipc::kParamBytes);
    ctx.cu_count = 256;
    gpu_model_select = [](const char *name, dim3, unsigned *, unsigned *) {
        if (std::strstr(name, "prefill")) prefill_launches++;
        return true;
    };
    // (M, K, N, block, zero points): ragged in every direction, a partial last stage, an odd stage count, one tile,
    // more tiles than one XCD rectangle holds, every scale grouping
    const int64_t shapes[][5] = {{17, 72, 16, 32, 1},   {100, 1000, 200, 32, 1}, {130, 384, 131, 64, 1}, {257, 640, 96, 128, 1},
                                 {64, 256, 1024, 256, 0}, {129, 512, 392, 64, 0},  {300, 1152, 200, 128, 1}};
    for (const auto &s : shapes) {
        product(s[0], s[1], s[2], s[3], s[4] != 0, HIPC_F16);
        if (s[0] > 32) product(s[0], s[1], s[2], s[3], s[4] != 0, HIPC_F32);
    }
    // few rows: block sizes of the reference's envelope that only the ONNX-layout kernel takes (8, 24, 40), the
    // prepacked ones on the decode kernels; one row, a partial 16-row group, a full one; ragged K and N
    const int64_t few[][5] = {{1, 72, 16, 8, 1},   {3, 120, 50, 24, 1},  {16, 200, 33, 40, 0}, {1, 1000, 200, 32, 1}, {5, 384, 131, 64, 1},
                              {16, 640, 96, 128, 0}, {1, 1152, 1536, 32, 1}, {2, 256, 1024, 256, 1},
                              // the stand-alone launches of a gemma3-1b token (one k tile per wavefront up to sixteen tiles,
                              // four column tiles per workgroup on the widest, four k tiles per wavefront on the longest), a ragged k
                              {1, 1024, 1152, 32, 1}, {1, 1152, 13824, 32, 1}, {1, 6912, 1152, 32, 1}, {1, 1480, 64, 32, 1}};
    for (const auto &s : few)
        for (int dt : {HIPC_F32, HIPC_F16}) rows(s[0], s[1], s[2], s[3], s[4] != 0, dt);
    gpu_model::Registry &g = gpu_model::reg();
    std::printf("%zu launches (%zu of the tiled kernels and their helpers), %zu threads\n", g.launches, prefill_launches, g.threads);
    if (prefill_launches < 300) {
        std::printf("FAILED: the tiled kernels were not reached\n");
        return 1;
    }
    for (hipc::Scratch &s : ctx.scratch)
        if (s.ptr) gpu_model::release(s.ptr);
    gpu_model::release(ctx.params);
    std::printf("ok\n");
    return 0;
}
