// MatMulNBits (4-bit, block-quantised along K) for gfx950.
//
// Reference: crates/onnx-vulkan-core/src/shaders/matmul_nbits.rs (tensor format :1-25,
// row kernel :316-374, wide decode kernel :458-516) and interp.rs:6429-6561 (host side).
//
// Two device paths:
//
//   direct   reads the ONNX layout as it is. One wavefront per output column,
//            lanes stride over the row's 32-bit words (8 nibbles), f32 FMA,
//            butterfly reduction. Any M, K, block size >= 16, f32 / f16.
//
//   gemv     decode shapes (M <= 16) on a prepacked weight. The weight streams
//            from HBM once in 1 KiB tiles (16 columns x 128 k) with one 128-bit
//            load per lane; nibbles become bf16 integers 128+q with four
//            and-or operations per word and go straight into
//            v_mfma_f32_16x16x32_bf16 as the B operand. The f32 activations are
//            split once per workgroup into three bf16 terms (hi + mid + lo,
//            24 significant bits) that are the A operands of three chained MFMAs,
//            so products are exact and the sum is f32. The +128 bias and the
//            zero point leave in the per-block epilogue:
//                acc += scale * (dot - (128 + zp) * sum_k a_k).
//            HBM-bound: 16 B of nibbles + 4 B scale + 1 B zero point per 32 weights.
#include <hip/hip_fp16.h>

#include <algorithm>
#include <cstdlib>

#include "internal.h"

namespace hipc {

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

template <typename T>
__device__ __forceinline__ float to_f32(T v);
template <>
__device__ __forceinline__ float to_f32<float>(float v) {
    return v;
}
template <>
__device__ __forceinline__ float to_f32<__half>(__half v) {
    return __half2float(v);
}
template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) {
    return v;
}
template <>
__device__ __forceinline__ __half from_f32<__half>(float v) {
    return __float2half(v);
}

// ------------------------------------------------------------------ direct

template <typename AT, typename ST, int MR>
__global__ void __launch_bounds__(256)
mmnb_direct_kernel(const AT *__restrict__ A, const uint32_t *__restrict__ B, const ST *__restrict__ scales,
                   const uint8_t *__restrict__ zp, AT *__restrict__ Y, int M, int K, int N, int bs_shift,
                   int n_blocks, int row_words, int zp_row) {
    const int lane = threadIdx.x & 63;
    const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int m0 = blockIdx.y * MR;
    if (n >= N) return;  // a whole wavefront leaves; no block-level barrier below
    const uint32_t *brow = B + (size_t)n * row_words;
    float acc[MR];
#pragma unroll
    for (int r = 0; r < MR; r++) acc[r] = 0.f;

    for (int w = lane; w < row_words; w += 64) {
        const int k0 = w * 8;
        if (k0 >= K) break;
        const uint32_t q = brow[w];
        const int b = k0 >> bs_shift;
        const float s = to_f32<ST>(scales[(size_t)n * n_blocks + b]);
        const int z = zp ? (zp[(size_t)n * zp_row + (b >> 1)] >> (4 * (b & 1))) & 15 : 8;
        const float zf = (float)z;
        float wv[8];
#pragma unroll
        for (int i = 0; i < 8; i++) wv[i] = ((float)((q >> (4 * i)) & 15u) - zf) * s;
#pragma unroll
        for (int r = 0; r < MR; r++) {
            const int m = m0 + r;
            if (m < M) {
                const AT *a = A + (size_t)m * K + k0;
#pragma unroll
                for (int i = 0; i < 8; i++)
                    if (k0 + i < K) acc[r] = fmaf(to_f32<AT>(a[i]), wv[i], acc[r]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < MR; r++) {
        float v = acc[r];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
        if (lane == 0 && m0 + r < M) Y[(size_t)(m0 + r) * N + n] = from_f32<AT>(v);
    }
}

// ----------------------------------------------------------------- prepack

// Tile (nt, cg): 16 columns n = 16*nt + (lane & 15), four 32-k chunks c = 4*cg + j.
// Lane l's 128-bit element holds, in word j, the 8 nibbles k = 32*c + 8*(l >> 4) .. +8
// of column n -- exactly the B operand of one 16x16x32 MFMA per word.
// SG scale groups per tile (4 when block_size == 32, 2 for 64, 1 for >= 128).
template <typename ST>
__global__ void __launch_bounds__(256)
mmnb_prepack_kernel(const uint32_t *__restrict__ B, const ST *__restrict__ scales, const uint8_t *__restrict__ zp,
                    uint4 *__restrict__ Wq, float *__restrict__ Sc, uint8_t *__restrict__ Zb, int N, int n_blocks,
                    int row_words, int zp_row, long n_tile_total, int n_cg, int cpb_shift, int SG) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    const long tile = idx >> 6;
    if (tile >= n_tile_total) return;
    const int lane = (int)(idx & 63);
    const int nt = (int)(tile / n_cg), cg = (int)(tile % n_cg);
    const int i16 = lane & 15, w = lane >> 4;
    const int n = nt * 16 + i16;
    uint32_t v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int widx = (cg * 4 + j) * 4 + w;
        v[j] = (n < N && widx < row_words) ? B[(size_t)n * row_words + widx] : 0u;
    }
    Wq[idx] = make_uint4(v[0], v[1], v[2], v[3]);
    if (w == 0) {
        for (int g = 0; g < SG; g++) {
            const int c = cg * 4 + g * (4 / SG);
            const int b = c >> cpb_shift;
            float s = 0.f;
            int z = 8;
            if (n < N && b < n_blocks) {
                s = to_f32<ST>(scales[(size_t)n * n_blocks + b]);
                if (zp) z = (zp[(size_t)n * zp_row + (b >> 1)] >> (4 * (b & 1))) & 15;
            }
            Sc[(tile * 16 + i16) * SG + g] = s;
            Zb[(tile * 16 + i16) * SG + g] = (uint8_t)(128 + z);
        }
    }
}

// -------------------------------------------------------------------- gemv

struct GemvArgs {
    const void *A;
    const uint4 *Wq;
    const float *Sc;
    const uint8_t *Zb;
    void *Y;
    float *Ypart;
    int M, K, N;
    int n_tiles, n_cg;
    int WK, WN;        // wavefronts along k and along n in a workgroup
    int slice_tiles;   // k tiles (128 k) per workgroup slice
    int ksplit;        // number of slices (gridDim.y)
    int a_f16;
};

__device__ __forceinline__ uint32_t bf16_pair(float lo, float hi) {
    return (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xffff0000u);
}

template <int SG>
struct ScaleVec;
template <>
struct ScaleVec<4> {
    float s[4];
    uint32_t z;
    __device__ __forceinline__ void load(const float *sc, const uint8_t *zb, size_t at) {
        const float4 v = *reinterpret_cast<const float4 *>(sc + at * 4);
        s[0] = v.x, s[1] = v.y, s[2] = v.z, s[3] = v.w;
        z = *reinterpret_cast<const uint32_t *>(zb + at * 4);
    }
    __device__ __forceinline__ void clear() { s[0] = s[1] = s[2] = s[3] = 0.f, z = 0; }
};
template <>
struct ScaleVec<2> {
    float s[2];
    uint32_t z;
    __device__ __forceinline__ void load(const float *sc, const uint8_t *zb, size_t at) {
        const float2 v = *reinterpret_cast<const float2 *>(sc + at * 2);
        s[0] = v.x, s[1] = v.y;
        z = *reinterpret_cast<const uint16_t *>(zb + at * 2);
    }
    __device__ __forceinline__ void clear() { s[0] = s[1] = 0.f, z = 0; }
};
template <>
struct ScaleVec<1> {
    float s[1];
    uint32_t z;
    __device__ __forceinline__ void load(const float *sc, const uint8_t *zb, size_t at) {
        s[0] = sc[at];
        z = zb[at];
    }
    __device__ __forceinline__ void clear() { s[0] = 0.f, z = 0; }
};

// T: 16-column tiles per wavefront; NR: accumulator registers in use (rows m = (lane>>4) + 4r,
// r < NR, so M <= 4*NR); SG: scale groups per 128-k tile.
// The workgroup is at most 16 / T wavefronts, which leaves the wide variants their registers.
template <int T, int NR, int SG>
__global__ void __launch_bounds__(1024 / T) mmnb_gemv_kernel(const GemvArgs p) {
    extern __shared__ uint4 smem[];
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int M = p.M;
    const int tile0 = blockIdx.y * p.slice_tiles;
    const int tile1 = min(p.n_cg, tile0 + p.slice_tiles);
    const int nch = (tile1 - tile0) * 4;  // 32-k chunks in this slice

    uint4 *As = smem;                                              // [3][nch][4][M]
    float *asum = reinterpret_cast<float *>(As + (size_t)3 * nch * 4 * M);  // [nch][M]
    float *red = asum + ((nch * M + 3) & ~3);                      // [WN][WK][T][NR][64]

    // ---- split the activations of this k slice into three bf16 terms, in operand order
    {
        const int nitems = M * nch * 4;
        const int kbase = tile0 * 128;
        for (int item = tid; item < nitems; item += nthreads) {
            const int w = item & 3;
            const int c = (item >> 2) % nch;
            const int m = (item >> 2) / nch;
            const int k0 = kbase + c * 32 + w * 8;
            float a[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int k = k0 + i;
                float v = 0.f;
                if (k < p.K) {
                    v = p.a_f16 ? __half2float(static_cast<const __half *>(p.A)[(size_t)m * p.K + k])
                                : static_cast<const float *>(p.A)[(size_t)m * p.K + k];
                }
                a[i] = v;
            }
            float s = ((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7]));
            s += __shfl_xor(s, 1, 64);
            s += __shfl_xor(s, 2, 64);
            float hi[8], mid[8], lo[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                hi[i] = __uint_as_float(__float_as_uint(a[i]) & 0xffff0000u);
                const float r1 = a[i] - hi[i];  // exact
                mid[i] = __uint_as_float(__float_as_uint(r1) & 0xffff0000u);
                lo[i] = r1 - mid[i];            // exact; truncated to bf16 by the pack
            }
            const size_t slot = ((size_t)c * 4 + w) * M + m;
            const size_t term = (size_t)nch * 4 * M;
            // slot order (k0,k4,k1,k5,k2,k6,k3,k7) matches the nibble unpack below
            As[slot] = make_uint4(bf16_pair(hi[0], hi[4]), bf16_pair(hi[1], hi[5]), bf16_pair(hi[2], hi[6]),
                                  bf16_pair(hi[3], hi[7]));
            As[term + slot] = make_uint4(bf16_pair(mid[0], mid[4]), bf16_pair(mid[1], mid[5]),
                                         bf16_pair(mid[2], mid[6]), bf16_pair(mid[3], mid[7]));
            As[2 * term + slot] = make_uint4(bf16_pair(lo[0], lo[4]), bf16_pair(lo[1], lo[5]),
                                             bf16_pair(lo[2], lo[6]), bf16_pair(lo[3], lo[7]));
            if (w == 0) asum[c * M + m] = s;
        }
    }
    __syncthreads();

    const int lane = tid & 63, wave = tid >> 6;
    const int wk = wave % p.WK, wn = wave / p.WK;
    const int i16 = lane & 15, g4 = lane >> 4;
    const int mA = (i16 >> 2) + 4 * (i16 & 3);  // activation row this lane feeds as the A operand
    const bool a_valid = mA < M;
    const int nt0 = (blockIdx.x * p.WN + wn) * T;
    const size_t term = (size_t)nch * 4 * M;

    f32x4 acc[T];
#pragma unroll
    for (int t = 0; t < T; t++) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    if (nt0 < p.n_tiles) {
        for (int tile = tile0 + wk; tile < tile1; tile += p.WK) {
            uint4 wq[T];
            ScaleVec<SG> sv[T];
#pragma unroll
            for (int t = 0; t < T; t++) {
                if (nt0 + t < p.n_tiles) {
                    const size_t tl = (size_t)(nt0 + t) * p.n_cg + tile;
                    wq[t] = p.Wq[tl * 64 + lane];
                    sv[t].load(p.Sc, p.Zb, tl * 16 + i16);
                } else {
                    wq[t] = make_uint4(0, 0, 0, 0);
                    sv[t].clear();
                }
            }
            f32x4 c[T];
            float asg[NR];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int cl = (tile - tile0) * 4 + j;
                uint4 ah = make_uint4(0, 0, 0, 0), am = ah, al = ah;
                if (a_valid) {
                    const size_t slot = ((size_t)cl * 4 + g4) * M + mA;
                    ah = As[slot];
                    am = As[term + slot];
                    al = As[2 * term + slot];
                }
                const bf16x8 a_hi = __builtin_bit_cast(bf16x8, ah);
                const bf16x8 a_mid = __builtin_bit_cast(bf16x8, am);
                const bf16x8 a_lo = __builtin_bit_cast(bf16x8, al);
                constexpr int CPG = 4 / SG;  // chunks per scale group
                const bool first = (j % CPG) == 0, last = (j % CPG) == CPG - 1;
#pragma unroll
                for (int r = 0; r < NR; r++) {
                    const int m = g4 + 4 * r;
                    const float v = (m < M) ? asum[cl * M + m] : 0.f;
                    asg[r] = first ? v : asg[r] + v;
                }
#pragma unroll
                for (int t = 0; t < T; t++) {
                    const uint32_t word = j == 0 ? wq[t].x : j == 1 ? wq[t].y : j == 2 ? wq[t].z : wq[t].w;
                    const uint4 bw = make_uint4((word & 0x000f000fu) | 0x43004300u,
                                                ((word >> 4) & 0x000f000fu) | 0x43004300u,
                                                ((word >> 8) & 0x000f000fu) | 0x43004300u,
                                                ((word >> 12) & 0x000f000fu) | 0x43004300u);
                    const bf16x8 b = __builtin_bit_cast(bf16x8, bw);
                    f32x4 d = first ? f32x4{0.f, 0.f, 0.f, 0.f} : c[t];
                    d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, b, d, 0, 0, 0);
                    d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_mid, b, d, 0, 0, 0);
                    d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, b, d, 0, 0, 0);
                    c[t] = d;
                    if (last) {
                        const int g = j / CPG;
                        const float s = sv[t].s[g];
                        const float zb = (float)((sv[t].z >> (8 * g)) & 0xffu);
#pragma unroll
                        for (int r = 0; r < NR; r++) acc[t][r] = fmaf(s, fmaf(-zb, asg[r], d[r]), acc[t][r]);
                    }
                }
            }
        }
    }

    if (p.WK > 1) {
#pragma unroll
        for (int t = 0; t < T; t++)
#pragma unroll
            for (int r = 0; r < NR; r++) red[((((size_t)wn * p.WK + wk) * T + t) * NR + r) * 64 + lane] = acc[t][r];
        __syncthreads();
        if (wk == 0) {
#pragma unroll
            for (int t = 0; t < T; t++)
#pragma unroll
                for (int r = 0; r < NR; r++) {
                    float v = acc[t][r];
                    for (int k = 1; k < p.WK; k++) v += red[((((size_t)wn * p.WK + k) * T + t) * NR + r) * 64 + lane];
                    acc[t][r] = v;
                }
        }
    }
    if (wk == 0 && nt0 < p.n_tiles) {
#pragma unroll
        for (int t = 0; t < T; t++) {
            const int n = (nt0 + t) * 16 + i16;
#pragma unroll
            for (int r = 0; r < NR; r++) {
                const int m = g4 + 4 * r;
                if (m < M && n < p.N) {
                    if (p.ksplit > 1) {
                        p.Ypart[((size_t)blockIdx.y * M + m) * p.N + n] = acc[t][r];
                    } else if (p.a_f16) {
                        static_cast<__half *>(p.Y)[(size_t)m * p.N + n] = __float2half(acc[t][r]);
                    } else {
                        static_cast<float *>(p.Y)[(size_t)m * p.N + n] = acc[t][r];
                    }
                }
            }
        }
    }
}

__global__ void __launch_bounds__(256)
mmnb_ksplit_reduce_kernel(const float *__restrict__ part, void *__restrict__ Y, long total, int ksplit, int f16) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    float v = part[i];
    for (int s = 1; s < ksplit; s++) v += part[(size_t)s * total + i];
    if (f16)
        static_cast<__half *>(Y)[i] = __float2half(v);
    else
        static_cast<float *>(Y)[i] = v;
}

}  // namespace hipc

using namespace hipc;

struct hipc_nbits_weight {
    int64_t K = 0, N = 0, block_size = 0;
    int n_tiles = 0, n_cg = 0, SG = 0;
    uint4 *Wq = nullptr;
    float *Sc = nullptr;
    uint8_t *Zb = nullptr;
    size_t bytes = 0;
};

namespace {

// Launch-shape overrides for experiments: HIPC_GEMV_T (16-column tiles per
// wavefront: 1, 2 or 4) and HIPC_GEMV_WAVES (wavefronts to aim for).
struct GemvTune {
    int T = 0, waves = 0;
    GemvTune() {
        if (const char *e = getenv("HIPC_GEMV_T")) T = atoi(e);
        if (const char *e = getenv("HIPC_GEMV_WAVES")) waves = atoi(e);
    }
};
const GemvTune g_tune;

int log2i(int64_t v) {
    int s = 0;
    while ((int64_t(1) << s) < v) s++;
    return s;
}

int check_nbits_shape(hipc_ctx *ctx, int64_t M, int64_t K, int64_t N, int64_t block_size, size_t b_len,
                      size_t scales_len, const void *zp, size_t zp_len, int scale_dtype) {
    HIPC_REQUIRE(ctx, M >= 0 && K > 0 && N >= 0, "MatMulNBits: bad dimensions M=%ld K=%ld N=%ld", (long)M, (long)K,
                 (long)N);
    HIPC_REQUIRE(ctx, is_pow2(block_size) && block_size >= 16, "MatMulNBits: block_size %ld is not a power of two >= 16",
                 (long)block_size);
    HIPC_REQUIRE(ctx, K < (int64_t(1) << 30) && N < (int64_t(1) << 30) && M < (int64_t(1) << 30),
                 "MatMulNBits: dimension too large");
    HIPC_REFUSE(ctx, scale_dtype != HIPC_F32 && scale_dtype != HIPC_F16, "MatMulNBits: scales must be f32 or f16, got %d",
                scale_dtype);
    const int64_t n_blocks = ceil_div(K, block_size);
    // the same three length checks as the reference (interp.rs:6465-6472)
    HIPC_REQUIRE(ctx,
                 b_len >= (size_t)(N * n_blocks * block_size / 2) && scales_len >= (size_t)(N * n_blocks) &&
                     (!zp || zp_len >= (size_t)(N * ceil_div(n_blocks, 2))),
                 "MatMulNBits: packed weight is short for K=%ld N=%ld block_size=%ld", (long)K, (long)N,
                 (long)block_size);
    return HIPC_OK;
}

template <typename AT, typename ST>
int launch_direct(hipc_ctx *ctx, const void *A, const void *B, const void *scales, const void *zp, void *Y, int64_t M,
                  int64_t K, int64_t N, int64_t block_size) {
    const int n_blocks = (int)ceil_div(K, block_size);
    const int row_words = (int)(n_blocks * block_size / 8);
    const int zp_row = (n_blocks + 1) / 2;
    const int bs_shift = log2i(block_size);
    const dim3 block(256);
    int64_t m_done = 0;
    while (m_done < M) {  // grid.y is limited to 65535 row groups
        const int64_t rows = std::min<int64_t>(M - m_done, 65535 * 4);
        const AT *a = static_cast<const AT *>(A) + m_done * K;
        AT *y = static_cast<AT *>(Y) + m_done * N;
        if (rows == 1) {
            mmnb_direct_kernel<AT, ST, 1><<<dim3((unsigned)ceil_div(N, 4), 1), block, 0, ctx->stream>>>(
                a, static_cast<const uint32_t *>(B), static_cast<const ST *>(scales), static_cast<const uint8_t *>(zp),
                y, (int)rows, (int)K, (int)N, bs_shift, n_blocks, row_words, zp_row);
        } else {
            mmnb_direct_kernel<AT, ST, 4>
                <<<dim3((unsigned)ceil_div(N, 4), (unsigned)ceil_div(rows, 4)), block, 0, ctx->stream>>>(
                    a, static_cast<const uint32_t *>(B), static_cast<const ST *>(scales),
                    static_cast<const uint8_t *>(zp), y, (int)rows, (int)K, (int)N, bs_shift, n_blocks, row_words,
                    zp_row);
        }
        HIPC_LAUNCHED(ctx);
        m_done += rows;
    }
    return HIPC_OK;
}

template <int T, int NR>
void launch_gemv_sg(const GemvArgs &a, int SG, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
    if (SG == 4)
        mmnb_gemv_kernel<T, NR, 4><<<grid, block, lds, s>>>(a);
    else if (SG == 2)
        mmnb_gemv_kernel<T, NR, 2><<<grid, block, lds, s>>>(a);
    else
        mmnb_gemv_kernel<T, NR, 1><<<grid, block, lds, s>>>(a);
}

template <int T>
void launch_gemv_nr(const GemvArgs &a, int NR, int SG, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
    if (NR == 1)
        launch_gemv_sg<T, 1>(a, SG, grid, block, lds, s);
    else if (NR == 2)
        launch_gemv_sg<T, 2>(a, SG, grid, block, lds, s);
    else
        launch_gemv_sg<T, 4>(a, SG, grid, block, lds, s);
}

// rows [0, M) with M <= 16 of one activation matrix against a prepacked weight
int launch_gemv(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_nbits_weight *w, void *Y, int M) {
    GemvArgs a{};
    a.A = A, a.Wq = w->Wq, a.Sc = w->Sc, a.Zb = w->Zb, a.Y = Y, a.Ypart = nullptr;
    a.M = M, a.K = (int)w->K, a.N = (int)w->N, a.n_tiles = w->n_tiles, a.n_cg = w->n_cg;
    a.a_f16 = a_dtype == HIPC_F16;
    const int NR = M <= 4 ? 1 : (M <= 8 ? 2 : 4);
    const int n_tiles = w->n_tiles, n_cg = w->n_cg;

    // columns per wavefront: wide outputs amortise the activation operands over more tiles
    int T = n_tiles >= 8192 ? 4 : (n_tiles >= 2048 ? 2 : 1);
    if (g_tune.T == 1 || g_tune.T == 2 || g_tune.T == 4) T = g_tune.T;
    const int groups = (int)ceil_div(n_tiles, T);
    // k partition inside a workgroup: enough wavefronts to cover the chip a few times over
    const int want_waves = g_tune.waves > 0 ? g_tune.waves : 8 * ctx->cu_count;
    const int kparts = (int)std::min<int64_t>(n_cg, std::max<int64_t>(1, ceil_div(want_waves, groups)));
    // the activation slice of a workgroup must fit the LDS budget: 196 bytes per row per 32-k chunk;
    // only then is k also split across workgroups (partials + a reduce launch)
    const int lds_budget = 44 * 1024;
    const int max_slice_tiles = std::max(1, lds_budget / (196 * 4 * M));
    int ksplit = (int)ceil_div(n_cg, max_slice_tiles);
    const int slice_tiles = (int)ceil_div(n_cg, ksplit);
    ksplit = (int)ceil_div(n_cg, slice_tiles);
    const int WK = std::max(1, std::min(std::min(16 / T, kparts), slice_tiles));
    const int WN = std::max(1, std::min(4 / WK, groups));
    a.WK = WK, a.WN = WN, a.slice_tiles = slice_tiles, a.ksplit = ksplit;

    const int nch = slice_tiles * 4;
    size_t lds = (size_t)3 * nch * 4 * M * 16 + (size_t)((nch * M + 3) & ~3) * 4;
    if (WK > 1) lds += (size_t)WN * WK * T * NR * 64 * 4;
    HIPC_REQUIRE(ctx, lds <= 64 * 1024, "MatMulNBits gemv: LDS plan of %zu bytes does not fit", lds);

    if (ksplit > 1) {
        void *part = nullptr;
        int rc = scratch_get(ctx, 0, (size_t)ksplit * M * w->N * sizeof(float), &part);
        if (rc != HIPC_OK) return rc;
        a.Ypart = static_cast<float *>(part);
    }
    const dim3 grid((unsigned)ceil_div(groups, WN), (unsigned)ksplit);
    const dim3 block(64 * WK * WN);
    if (T == 4)
        launch_gemv_nr<4>(a, NR, w->SG, grid, block, lds, ctx->stream);
    else if (T == 2)
        launch_gemv_nr<2>(a, NR, w->SG, grid, block, lds, ctx->stream);
    else
        launch_gemv_nr<1>(a, NR, w->SG, grid, block, lds, ctx->stream);
    HIPC_LAUNCHED(ctx);
    if (ksplit > 1) {
        const long total = (long)M * w->N;
        mmnb_ksplit_reduce_kernel<<<dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, ctx->stream>>>(
            a.Ypart, Y, total, ksplit, a.a_f16);
        HIPC_LAUNCHED(ctx);
    }
    return HIPC_OK;
}

}  // namespace

extern "C" {

int hipc_matmul_nbits(hipc_ctx *ctx, const void *A, int a_dtype, const void *B, size_t b_len, const void *scales,
                      int scale_dtype, size_t scales_len, const void *zp, size_t zp_len, void *Y, int64_t M, int64_t K,
                      int64_t N, int64_t block_size, int accuracy_level) {
    if (!ctx) return HIPC_ERR_INVALID;
    Guard g(ctx);
    HIPC_REFUSE(ctx, a_dtype != HIPC_F32 && a_dtype != HIPC_F16, "MatMulNBits: A must be f32 or f16, got %d", a_dtype);
    HIPC_REFUSE(ctx, accuracy_level < 0 || accuracy_level > 3,
                "MatMulNBits: accuracy_level %d asks for quantised activations", accuracy_level);
    int rc = check_nbits_shape(ctx, M, K, N, block_size, b_len, scales_len, zp, zp_len, scale_dtype);
    if (rc != HIPC_OK) return rc;
    if (M == 0 || N == 0) return HIPC_OK;
    HIPC_REQUIRE(ctx, A && B && scales && Y, "MatMulNBits: null operand");
    HIPC_REQUIRE(ctx, aligned(B, 4), "MatMulNBits: packed weight must be 4-byte aligned");
    const bool af16 = a_dtype == HIPC_F16, sf16 = scale_dtype == HIPC_F16;
    if (af16 && sf16) return launch_direct<__half, __half>(ctx, A, B, scales, zp, Y, M, K, N, block_size);
    if (af16) return launch_direct<__half, float>(ctx, A, B, scales, zp, Y, M, K, N, block_size);
    if (sf16) return launch_direct<float, __half>(ctx, A, B, scales, zp, Y, M, K, N, block_size);
    return launch_direct<float, float>(ctx, A, B, scales, zp, Y, M, K, N, block_size);
}

int hipc_prepack_matmul_nbits(hipc_ctx *ctx, const void *B, size_t b_len, const void *scales, int scale_dtype,
                              size_t scales_len, const void *zp, size_t zp_len, int64_t K, int64_t N, int64_t block_size,
                              hipc_nbits_weight **out) {
    if (!ctx || !out) return HIPC_ERR_INVALID;
    Guard g(ctx);
    *out = nullptr;
    HIPC_REFUSE(ctx, ctx->capturing, "MatMulNBits prepack while a capture is open");
    int rc = check_nbits_shape(ctx, 1, K, N, block_size, b_len, scales_len, zp, zp_len, scale_dtype);
    if (rc != HIPC_OK) return rc;
    HIPC_REQUIRE(ctx, N > 0 && B && scales, "MatMulNBits prepack: empty weight");
    HIPC_REQUIRE(ctx, aligned(B, 4), "MatMulNBits: packed weight must be 4-byte aligned");
    HIPC_REFUSE(ctx, block_size < 32, "MatMulNBits prepack: block_size %ld < 32 only runs on the direct path",
                (long)block_size);
    hipc_nbits_weight *w = new hipc_nbits_weight();
    w->K = K, w->N = N, w->block_size = block_size;
    const int n_blocks = (int)ceil_div(K, block_size);
    const int n_chunks = (int)ceil_div(K, 32);
    w->n_tiles = (int)ceil_div(N, 16);
    w->n_cg = (int)ceil_div(n_chunks, 4);
    const int cpb = (int)(block_size / 32);
    w->SG = cpb >= 4 ? 1 : 4 / cpb;
    const size_t tiles = (size_t)w->n_tiles * w->n_cg;
    const size_t wq_bytes = tiles * 1024, sc_bytes = tiles * 16 * w->SG * 4, zb_bytes = tiles * 16 * w->SG;
    auto cleanup = [&]() {
        if (w->Wq) (void)hipFree(w->Wq);
        if (w->Sc) (void)hipFree(w->Sc);
        if (w->Zb) (void)hipFree(w->Zb);
        delete w;
    };
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&w->Wq), wq_bytes);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&w->Sc), sc_bytes);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&w->Zb), (zb_bytes + 3) & ~(size_t)3);
    if (e != hipSuccess) {
        cleanup();
        return fail(ctx, HIPC_ERR_BACKEND, "MatMulNBits prepack: %s", hipGetErrorString(e));
    }
    w->bytes = wq_bytes + sc_bytes + zb_bytes;
    const int row_words = (int)(n_blocks * block_size / 8);
    const int zp_row = (n_blocks + 1) / 2;
    const long threads = (long)tiles * 64;
    const dim3 grid((unsigned)ceil_div(threads, 256)), block(256);
    if (scale_dtype == HIPC_F16)
        mmnb_prepack_kernel<__half><<<grid, block, 0, ctx->stream>>>(
            static_cast<const uint32_t *>(B), static_cast<const __half *>(scales), static_cast<const uint8_t *>(zp),
            w->Wq, w->Sc, w->Zb, (int)N, n_blocks, row_words, zp_row, (long)tiles, w->n_cg, log2i(cpb), w->SG);
    else
        mmnb_prepack_kernel<float><<<grid, block, 0, ctx->stream>>>(
            static_cast<const uint32_t *>(B), static_cast<const float *>(scales), static_cast<const uint8_t *>(zp),
            w->Wq, w->Sc, w->Zb, (int)N, n_blocks, row_words, zp_row, (long)tiles, w->n_cg, log2i(cpb), w->SG);
    e = hipGetLastError();
    if (e != hipSuccess) {
        cleanup();
        return fail(ctx, HIPC_ERR_BACKEND, "MatMulNBits prepack launch: %s", hipGetErrorString(e));
    }
    *out = w;
    return HIPC_OK;
}

void hipc_nbits_weight_destroy(hipc_ctx *ctx, hipc_nbits_weight *w) {
    if (!ctx || !w) return;
    Guard g(ctx);
    // enqueued work may still read the weight: release at the next flush
    if (w->Wq) ctx->deferred.push_back(w->Wq);
    if (w->Sc) ctx->deferred.push_back(w->Sc);
    if (w->Zb) ctx->deferred.push_back(w->Zb);
    delete w;
}

size_t hipc_nbits_weight_bytes(const hipc_nbits_weight *w) { return w ? w->bytes : 0; }

int hipc_matmul_nbits_packed(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_nbits_weight *w, void *Y, int64_t M) {
    if (!ctx) return HIPC_ERR_INVALID;
    Guard g(ctx);
    HIPC_REQUIRE(ctx, w, "MatMulNBits: null weight");
    HIPC_REFUSE(ctx, a_dtype != HIPC_F32 && a_dtype != HIPC_F16, "MatMulNBits: A must be f32 or f16, got %d", a_dtype);
    HIPC_REQUIRE(ctx, M >= 0 && M < (int64_t(1) << 30), "MatMulNBits: bad M=%ld", (long)M);
    if (M == 0) return HIPC_OK;
    HIPC_REQUIRE(ctx, A && Y, "MatMulNBits: null operand");
    const size_t esz = a_dtype == HIPC_F16 ? 2 : 4;
    for (int64_t m0 = 0; m0 < M; m0 += 16) {
        const int rows = (int)std::min<int64_t>(16, M - m0);
        int rc = launch_gemv(ctx, static_cast<const char *>(A) + (size_t)m0 * w->K * esz, a_dtype, w,
                             static_cast<char *>(Y) + (size_t)m0 * w->N * esz, rows);
        if (rc != HIPC_OK) return rc;
    }
    return HIPC_OK;
}

}  // extern "C"
