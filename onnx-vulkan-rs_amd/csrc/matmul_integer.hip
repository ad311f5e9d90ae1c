// MatMulInteger, its fused dequantising epilogue, Requantize and QLinearMatMul.
//
// Reference: crates/onnx-vulkan-core/src/interp.rs:2090-2183 (matmul_integer),
// :2405-2572 (matmul_integer_scale_bias), :2712-2768 (packed_b), :4682-4788
// (requantize), :4845-4875 (qlinear_matmul); kernels shaders/matmul_integer.rs and
// shaders/glsl/matmul_integer_coop_smem.comp; definition host_ops.rs:1157-1199.
#include <algorithm>

#include "int8_gemm.h"
#include "int8_gemm_bdirect.h"

namespace hipc {

// B [K, N] (N contiguous) -> Bp, N_pad x K_pad bytes in the fragment-major order of qfrag_offset,
// signed domain, zero padded. One thread writes one 32-bit word (4 consecutive k of one column);
// reads are coalesced along n, and so are the writes (16 bytes apart).
__global__ void __launch_bounds__(256)
pack_b_kernel(const uint8_t *__restrict__ B, uint32_t *__restrict__ Bp, int K, int N, int K_pad, int N_pad,
              uint32_t flip) {
    const int n = blockIdx.x * 64 + (threadIdx.x & 63);
    const int kw = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (n >= N_pad || kw >= K_pad / 4) return;
    uint32_t word = 0;
    if (n < N) {
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const int k = kw * 4 + b;
            if (k < K) word |= (uint32_t)(B[(size_t)k * N + n] ^ (flip & 0xff)) << (8 * b);
        }
    }
    Bp[qfrag_offset(n, kw * 4, K_pad) / 4] = word;
}

// per-column sums of the shifted weight, from the packed form: one wavefront per column, 16 bytes
// per lane and step (the padding is zero, so whole rows can be summed)
__global__ void __launch_bounds__(256)
col_sum_kernel(const uint8_t *__restrict__ Bp, int32_t *__restrict__ sums, int K_pad, int N_pad) {
    const int lane = threadIdx.x & 63;
    const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N_pad) return;
    int s = 0;
    for (int c = lane; c < K_pad / 16; c += 64) s += dot_ones(*reinterpret_cast<const uint4 *>(Bp + qfrag_offset(n, c * 16, K_pad)));
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
    if (lane == 0) sums[n] = s;
}

// register-only MFMA loop: 8 independent accumulators per wavefront (128 registers, so two wavefronts fit a SIMD), operands never reloaded
__global__ void __launch_bounds__(256) int8_mfma_probe_kernel(int iterations, uint32_t seed, int random_operands, int *sink) {
    uint32_t x = seed ^ (blockIdx.x * 256u + threadIdx.x) * 2654435761u;
    auto next = [&]() {
        x = x * 1664525u + 1013904223u;
        return random_operands ? (int)(x ^ (x >> 15)) : 0x01010101;
    };
    i32x4 a[2], b[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        if (i < 2) a[i] = i32x4{next(), next(), next(), next()};
        b[i] = i32x4{next(), next(), next(), next()};
    }
    i32x16 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
    for (int it = 0; it < iterations; it++) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) s ^= acc[i][j][r];
    if (s == 0x7fffffff) sink[0] = s;  // keeps the loop alive; practically never true
}

__global__ void __launch_bounds__(256)
requantize_kernel(const int32_t *__restrict__ acc, const int32_t *__restrict__ bias, const float *__restrict__ ratio,
                  long n, long inner, long axis_len, int y_zp, int out_signed, uint8_t *__restrict__ out) {
    const long word = (long)blockIdx.x * 256 + threadIdx.x;
    const long base = word * 4;
    if (base >= n) return;
    uint32_t packed = 0;
    int count = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const long i = base + j;
        if (i >= n) break;
        const long c = (i / inner) % axis_len;
        int a = acc[i];
        if (bias) a += bias[c];
        int q = (int)rintf(__fmul_rn((float)a, ratio[c])) + y_zp;
        q = out_signed ? min(max(q, -128), 127) : min(max(q, 0), 255);
        packed |= ((uint32_t)q & 0xffu) << (8 * j);
        count++;
    }
    if (count == 4 && ((reinterpret_cast<uintptr_t>(out) & 3) == 0)) {
        reinterpret_cast<uint32_t *>(out)[word] = packed;
    } else {
        for (int j = 0; j < count; j++) out[base + j] = (uint8_t)(packed >> (8 * j));
    }
}

}  // namespace hipc

using namespace hipc;

struct hipc_int8_weight {
    int64_t K = 0, N = 0;
    int K_pad = 0, N_pad = 0;
    int b_dtype = HIPC_I8;
    uint8_t *Bp = nullptr;
    int32_t *colsum = nullptr;
    mutable hipc::RatioCache ratios;  // QLinearMatMul's requantisation ratios as last used
};

namespace {

int pack_into(hipc_ctx *ctx, const void *B, int b_dtype, int64_t K, int64_t N, int K_pad, int N_pad, uint8_t *Bp,
              int32_t *colsum) {
    const uint32_t flip = b_dtype == HIPC_U8 ? 0x80808080u : 0u;
    hipLaunchKernelGGL((pack_b_kernel), dim3((unsigned)ceil_div(N_pad, 64), (unsigned)ceil_div(K_pad / 4, 4)), 256, 0, ctx->stream, static_cast<const uint8_t *>(B), reinterpret_cast<uint32_t *>(Bp), (int)K, (int)N, K_pad, N_pad, flip);
    HIPC_LAUNCHED(ctx);
    hipLaunchKernelGGL((col_sum_kernel), dim3((unsigned)ceil_div(N_pad, 4)), 256, 0, ctx->stream, Bp, colsum, K_pad, N_pad);
    HIPC_LAUNCHED(ctx);
    return HIPC_OK;
}

struct MmOperands {
    const void *A;
    int a_dtype;
    const uint8_t *Bp;
    const int32_t *colsum;
    int b_dtype;
    int64_t M, K, N;
    int K_pad;
};

int fill_common(hipc_ctx *ctx, const MmOperands &o, GemmArgs &g) {
    HIPC_REFUSE(ctx, !is_byte_dtype(o.a_dtype), "MatMulInteger: A must be uint8 or int8, got %d", o.a_dtype);
    HIPC_REQUIRE(ctx, o.M >= 0 && o.M < (int64_t(1) << 30), "MatMulInteger: bad M=%ld", (long)o.M);
    g = GemmArgs{};
    g.P = static_cast<const uint8_t *>(o.A);
    g.Q = o.Bp;
    g.const_sum = o.colsum;
    g.dyn_shift = o.a_dtype == HIPC_U8 ? 128 : 0;
    g.const_shift = o.b_dtype == HIPC_U8 ? 128 : 0;
    g.dyn_signed = o.a_dtype == HIPC_I8;
    g.const_signed = o.b_dtype == HIPC_I8;
    g.I = (int)o.M, g.J = (int)o.N, g.K = (int)o.K, g.K_pad = o.K_pad;
    // the fast loader: whole 128-byte k stages, 16-byte aligned rows, 32-bit offsets
    g.p_aligned = (o.K % kBK == 0) && aligned(o.A, 16) && o.M * o.K < (int64_t(1) << 32);
    return HIPC_OK;
}

template <int EPI, bool DYN, int T, int W>
int launch_mm_bdirect_dyn(hipc_ctx *ctx, GemmArgs g) {
    static bool lds_allowed[kMaxDevices] = {};
    if (int rc = allow_dynamic_lds(ctx, int8_gemm_bdirect_kernel<EPI, DYN, T, W>, bd_lds(T), lds_allowed)) return rc;
    const dim3 grid(gemm_grid(g, T), 1, 1);
    hipLaunchKernelGGL((int8_gemm_bdirect_kernel<EPI, DYN, T, W>), grid, 64 * W, bd_lds(T), ctx->stream, g);
    HIPC_LAUNCHED(ctx);
    gemm_note_scalars(ctx, g, DYN);
    return HIPC_OK;
}

// The kernels that keep B out of LDS (int8_gemm_bdirect.h): 256x256 tiles once they fill most of the chip's
// 256 CUs, 128x128 tiles once those do; 0 neither. The gemm_big option overrides (0 never, 1 / 2 the
// 256 / 128 tile whenever A allows; tuning, tests).
int big_tile_choice(hipc_ctx *ctx, const GemmArgs &g) {
    const int forced = ctx->tune.gemm_big;
    if (!g.p_aligned) return 0;
    if (forced >= 0) return forced <= 2 ? forced : 0;
    if (ceil_div(g.I, kBigTile) * ceil_div(g.J, kBigTile) >= 192) return 1;
    if (ceil_div(g.I, kBM) * ceil_div(g.J, kBN) >= 192) return 2;
    return 0;
}

template <int EPI>
int launch_mm_big(hipc_ctx *ctx, const GemmArgs &g, int choice) {
    // the row sums of A only matter when the weight's zero point, shifted to the signed domain, is
    // not zero; the host knows that it is zero when the weight is int8 and carries no zero point
    const bool zero_known = g.const_shift == 0 && (g.host_zp ? g.const_zp_value == 0 : g.const_zp == nullptr);
    if (choice == 1) return zero_known ? launch_mm_bdirect_dyn<EPI, false, 256, 8>(ctx, g) : launch_mm_bdirect_dyn<EPI, true, 256, 8>(ctx, g);
    return zero_known ? launch_mm_bdirect_dyn<EPI, false, 128, 8>(ctx, g) : launch_mm_bdirect_dyn<EPI, true, 128, 8>(ctx, g);
}

// Products of a few 64x64 tiles per CU and a long enough k run on the kernel that keeps B out of LDS
// and splits k over the wavefronts of a workgroup. The gemm_small option (0 / 1) overrides (tuning, tests).
bool wants_small_tiles(hipc_ctx *ctx, const GemmArgs &g) {
    const int forced = ctx->tune.gemm_small;
    if (!g.p_aligned) return false;
    if (forced >= 0) return forced != 0;
    // measured against the LDS-staged 64x64 tiles: ahead up to four tiles per CU from k = 1024 on (14.1
    // against 15.3 us for 1000 x 1024 x 4096), up to two per CU from k = 512 on; behind with k = 256
    const int64_t tiles64 = ceil_div(g.I, 64) * ceil_div(g.J, 64);
    return (tiles64 <= 2 * (int64_t)ctx->cu_count && g.K >= 4 * kBK) || (tiles64 <= 4 * (int64_t)ctx->cu_count && g.K >= 8 * kBK);
}
template <int EPI, bool DYN>
int launch_mm_small_dyn(hipc_ctx *ctx, GemmArgs g) {
    const dim3 grid(gemm_grid(g, 64));
    hipLaunchKernelGGL((int8_gemm_small_kernel<EPI, DYN>), grid, 256, kSmallLds, ctx->stream, g);
    HIPC_LAUNCHED(ctx);
    gemm_note_scalars(ctx, g, DYN);
    return HIPC_OK;
}
template <int EPI>
int launch_mm_small(hipc_ctx *ctx, const GemmArgs &g) {
    const bool zero_known = g.const_shift == 0 && (g.host_zp ? g.const_zp_value == 0 : g.const_zp == nullptr);
    return zero_known ? launch_mm_small_dyn<EPI, false>(ctx, g) : launch_mm_small_dyn<EPI, true>(ctx, g);
}
template <int EPI>
int launch_mm(hipc_ctx *ctx, const GemmArgs &g) {
    if (g.I == 0 || g.J == 0) return HIPC_OK;
    if (const int big = big_tile_choice(ctx, g)) return launch_mm_big<EPI>(ctx, g, big);
    if (wants_small_tiles(ctx, g)) return launch_mm_small<EPI>(ctx, g);
    return g.p_aligned ? gemm_launch<MODE_MM, EPI, true>(ctx, g, 1) : gemm_launch<MODE_MM, EPI, false>(ctx, g, 1);
}

}  // namespace

extern "C" {

int hipc_probe_int8_mfma(hipc_ctx *ctx, int random_operands, int waves_per_simd, int iterations, double *tops) {
    if (!tops) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, (waves_per_simd == 1 || waves_per_simd == 2) && iterations > 0 && iterations <= (1 << 20),
                     "hipc_probe_int8_mfma: waves_per_simd must be 1 or 2, iterations in 1..2^20");
        HIPC_REFUSE(ctx, ctx->capturing, "hipc_probe_int8_mfma while a capture is open");
        hipEvent_t t0, t1;
        HIPC_TRY(ctx, hipEventCreate(&t0));
        HIPC_TRY(ctx, hipEventCreate(&t1));
        int *sink = reinterpret_cast<int *>(static_cast<char *>(ctx->params) + 128);
        const unsigned grid = (unsigned)(ctx->cu_count * waves_per_simd);  // 4 wavefronts per workgroup, one per SIMD
        hipLaunchKernelGGL((int8_mfma_probe_kernel), grid, 256, 0, ctx->stream, 64, 1u, random_operands, sink);  // warm the clocks and the code
        hipError_t e = hipEventRecord(t0, ctx->stream);
        hipLaunchKernelGGL((int8_mfma_probe_kernel), grid, 256, 0, ctx->stream, iterations, 7u, random_operands, sink);
        if (e == hipSuccess) e = hipGetLastError();
        if (e == hipSuccess) e = hipEventRecord(t1, ctx->stream);
        if (e == hipSuccess) e = hipEventSynchronize(t1);
        float ms = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, t0, t1);
        (void)hipEventDestroy(t0);
        (void)hipEventDestroy(t1);
        if (e != hipSuccess) return fail(ctx, HIPC_ERR_BACKEND, "hipc_probe_int8_mfma: %s", hipGetErrorString(e));
        const double ops = 2.0 * 32 * 32 * 32 * 8.0 * iterations * 4.0 * grid;
        *tops = ops / (ms * 1e-3) / 1e12;
        return HIPC_OK;
    });
}

int hipc_prepack_int8_b(hipc_ctx *ctx, const void *B, int b_dtype, int64_t K, int64_t N, hipc_int8_weight **out) {
    if (!out) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        *out = nullptr;
        HIPC_REFUSE(ctx, ctx->capturing, "MatMulInteger prepack while a capture is open");
        HIPC_REFUSE(ctx, !is_byte_dtype(b_dtype), "MatMulInteger: B must be uint8 or int8, got %d", b_dtype);
        HIPC_REQUIRE(ctx, B && K > 0 && N > 0 && K < (int64_t(1) << 30) && N < (int64_t(1) << 30),
                     "MatMulInteger prepack: bad shape K=%ld N=%ld", (long)K, (long)N);
        hipc_int8_weight *w = new hipc_int8_weight();
        w->K = K, w->N = N, w->b_dtype = b_dtype;
        w->K_pad = (int)(ceil_div(K, kBK) * kBK);
        w->N_pad = (int)(ceil_div(N, kBN) * kBN);
        if ((int64_t)w->K_pad * w->N_pad >= (int64_t(1) << 32)) {
            delete w;
            return fail(ctx, HIPC_ERR_UNSUPPORTED, "MatMulInteger prepack: a %ld x %ld weight exceeds the 4 GiB the kernel addresses", (long)K, (long)N);
        }
        hipError_t e = hipMalloc(reinterpret_cast<void **>(&w->Bp), (size_t)w->K_pad * w->N_pad);
        if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&w->colsum), (size_t)w->N_pad * 4);
        if (e != hipSuccess) {
            if (w->Bp) (void)hipFree(w->Bp);
            delete w;
            return fail(ctx, HIPC_ERR_BACKEND, "MatMulInteger prepack: %s", hipGetErrorString(e));
        }
        int rc = pack_into(ctx, B, b_dtype, K, N, w->K_pad, w->N_pad, w->Bp, w->colsum);
        if (rc != HIPC_OK) {
            (void)hipFree(w->Bp);
            (void)hipFree(w->colsum);
            delete w;
            return rc;
        }
        *out = w;
        return HIPC_OK;
    });
}

void hipc_int8_weight_destroy(hipc_ctx *ctx, hipc_int8_weight *w) {
    if (!w) return;
    entry_void(ctx, [&] {
        if (w->Bp) ctx->deferred.push_back(w->Bp);
        if (w->colsum) ctx->deferred.push_back(w->colsum);
        ratio_release(ctx, w->ratios);
        delete w;
    });
}

int hipc_matmul_integer(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_int8_weight *B, const void *a_zp,
                        const void *b_zp, void *Y, int64_t M) {
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, B, "MatMulInteger: null weight");
        GemmArgs ga;
        int rc = fill_common(ctx, MmOperands{A, a_dtype, B->Bp, B->colsum, B->b_dtype, M, B->K, B->N, B->K_pad}, ga);
        if (rc != HIPC_OK) return rc;
        if (M == 0) return HIPC_OK;
        HIPC_REQUIRE(ctx, A && Y, "MatMulInteger: null operand");
        ga.dyn_zp = static_cast<const uint8_t *>(a_zp);
        ga.const_zp = static_cast<const uint8_t *>(b_zp);
        ga.Y = Y;
        return launch_mm<EPI_I32>(ctx, ga);
    });
}

int hipc_matmul_integer_raw(hipc_ctx *ctx, const void *A, int a_dtype, const void *B, int b_dtype, const void *a_zp,
                            const void *b_zp, void *Y, int64_t M, int64_t K, int64_t N) {
    return entry(ctx, [&]() -> int {
        HIPC_REFUSE(ctx, !is_byte_dtype(b_dtype), "MatMulInteger: B must be uint8 or int8, got %d", b_dtype);
        HIPC_REQUIRE(ctx, K > 0 && N >= 0 && K < (int64_t(1) << 30) && N < (int64_t(1) << 30),
                     "MatMulInteger: bad shape K=%ld N=%ld", (long)K, (long)N);
        if (M == 0 || N == 0) return HIPC_OK;
        HIPC_REQUIRE(ctx, A && B && Y, "MatMulInteger: null operand");
        const int K_pad = (int)(ceil_div(K, kBK) * kBK), N_pad = (int)(ceil_div(N, kBN) * kBN);
        HIPC_REFUSE(ctx, (int64_t)K_pad * N_pad >= (int64_t(1) << 32), "MatMulInteger: a %ld x %ld weight exceeds the 4 GiB the kernel addresses", (long)K, (long)N);
        void *scratch = nullptr;
        const size_t bp_bytes = (size_t)K_pad * N_pad;
        int rc = scratch_get(ctx, 1, bp_bytes + (size_t)N_pad * 4, &scratch);
        if (rc != HIPC_OK) return rc;
        uint8_t *Bp = static_cast<uint8_t *>(scratch);
        int32_t *colsum = reinterpret_cast<int32_t *>(Bp + bp_bytes);
        rc = pack_into(ctx, B, b_dtype, K, N, K_pad, N_pad, Bp, colsum);
        if (rc != HIPC_OK) return rc;
        GemmArgs ga;
        rc = fill_common(ctx, MmOperands{A, a_dtype, Bp, colsum, b_dtype, M, K, N, K_pad}, ga);
        if (rc != HIPC_OK) return rc;
        ga.dyn_zp = static_cast<const uint8_t *>(a_zp);
        ga.const_zp = static_cast<const uint8_t *>(b_zp);
        ga.Y = Y;
        return launch_mm<EPI_I32>(ctx, ga);
    });
}

int hipc_matmul_integer_scale_bias(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_int8_weight *B,
                                   const void *a_zp, const void *b_zp, const void *scale, int scale_step,
                                   const void *product, int product_step, const void *bias, int bias_step, int relu,
                                   void *range, void *Y, int64_t M) {
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, B, "MatMulIntegerScaleBias: null weight");
        HIPC_REQUIRE(ctx, scale, "MatMulIntegerScaleBias: null scale");
        HIPC_REQUIRE(ctx, (scale_step | 1) == 1 && (product_step | 1) == 1 && (bias_step | 1) == 1,
                     "MatMulIntegerScaleBias: broadcast steps must be 0 (scalar) or 1 (per column)");
        GemmArgs ga;
        int rc = fill_common(ctx, MmOperands{A, a_dtype, B->Bp, B->colsum, B->b_dtype, M, B->K, B->N, B->K_pad}, ga);
        if (rc != HIPC_OK) return rc;
        if (M == 0) return HIPC_OK;
        HIPC_REQUIRE(ctx, A && Y, "MatMulIntegerScaleBias: null operand");
        ga.dyn_zp = static_cast<const uint8_t *>(a_zp);
        ga.const_zp = static_cast<const uint8_t *>(b_zp);
        ga.Y = Y;
        ga.scale = static_cast<const float *>(scale), ga.scale_step = scale_step;
        ga.product = static_cast<const float *>(product), ga.product_step = product_step;
        ga.bias = static_cast<const float *>(bias), ga.bias_step = bias_step;
        ga.relu = relu;
        ga.range = static_cast<uint32_t *>(range);
        return launch_mm<EPI_SCALE_BIAS>(ctx, ga);
    });
}

int hipc_requantize(hipc_ctx *ctx, const void *acc, const void *bias, const void *ratio, int64_t n, int64_t inner,
                    int64_t axis_len, int32_t y_zp, int out_dtype, void *out) {
    return entry(ctx, [&]() -> int {
        HIPC_REFUSE(ctx, !is_byte_dtype(out_dtype), "Requantize: output must be uint8 or int8, got %d", out_dtype);
        HIPC_REQUIRE(ctx, n >= 0, "Requantize: negative length");
        HIPC_REQUIRE(ctx, axis_len > 0, "Requantize: empty scale");  // interp.rs:4732
        if (n == 0) return HIPC_OK;
        HIPC_REQUIRE(ctx, acc && ratio && out, "Requantize: null operand");
        const long words = ceil_div(n, 4);
        hipLaunchKernelGGL((requantize_kernel), dim3((unsigned)ceil_div(words, 256)), 256, 0, ctx->stream, static_cast<const int32_t *>(acc), static_cast<const int32_t *>(bias), static_cast<const float *>(ratio), (long)n,
            (long)std::max<int64_t>(inner, 1), (long)axis_len, y_zp, out_dtype == HIPC_I8, static_cast<uint8_t *>(out));
        HIPC_LAUNCHED(ctx);
        return HIPC_OK;
    });
}

int hipc_qlinear_matmul(hipc_ctx *ctx, const void *A, int a_dtype, float a_scale, int32_t a_zp,
                        const hipc_int8_weight *B, const float *b_scale, int64_t n_b_scale, int32_t b_zp, float y_scale,
                        int32_t y_zp, int y_dtype, void *Y, int64_t M) {
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, B && b_scale, "QLinearMatMul: null weight or scale");
        HIPC_REFUSE(ctx, !is_byte_dtype(y_dtype), "QLinearMatMul: output must be uint8 or int8, got %d", y_dtype);
        // the accepted envelope of `unsupported_quantization` (interp.rs:781-847, :4862-4866)
        HIPC_REQUIRE(ctx, n_b_scale == 1 || n_b_scale == B->N, "QLinearMatMul: %ld scales for %ld columns", (long)n_b_scale,
                     (long)B->N);
        HIPC_REFUSE(ctx, n_b_scale > 1 && b_zp != 0, "QLinearMatMul: b per-channel zero point is not zero (asymmetric weights)");
        HIPC_REQUIRE(ctx, y_scale != 0.f, "QLinear: y_scale is zero");
        GemmArgs ga;
        int rc = fill_common(ctx, MmOperands{A, a_dtype, B->Bp, B->colsum, B->b_dtype, M, B->K, B->N, B->K_pad}, ga);
        if (rc != HIPC_OK) return rc;
        if (M == 0) return HIPC_OK;
        HIPC_REQUIRE(ctx, A && Y, "QLinearMatMul: null operand");
        // ratio[c] = a_scale * b_scale[c] / y_scale, f32, left to right (interp.rs:4693)
        std::vector<float> ratio((size_t)n_b_scale);
        for (int64_t c = 0; c < n_b_scale; c++) {
            volatile float t = a_scale * b_scale[c];
            ratio[(size_t)c] = t / y_scale;
        }
        const float *dratio = nullptr;
        rc = ratio_resident(ctx, B->ratios, ratio, &dratio);
        if (rc != HIPC_OK) return rc;
        ga.host_zp = 1, ga.dyn_zp_value = a_zp, ga.const_zp_value = b_zp;
        ga.Y = Y;
        ga.ratio = dratio, ga.ratio_step = n_b_scale > 1 ? 1 : 0;
        ga.y_zp = y_zp, ga.out_signed = y_dtype == HIPC_I8;
        return launch_mm<EPI_REQUANT>(ctx, ga);
    });
}

}  // extern "C"
