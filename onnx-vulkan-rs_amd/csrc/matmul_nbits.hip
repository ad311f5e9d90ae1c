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
//            split once per workgroup into bf16 terms that are the A operands of
//            chained MFMAs, so products are exact and the sum is f32: two terms
//            by default (hi + lo, 16 significant bits), three (hi + mid + lo, all
//            24 bits) with accuracy_level 1. The +128 bias and the
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
                   const uint8_t *__restrict__ zp, AT *__restrict__ Y, int M, int K, int N, int bs_shift, int block_size,
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
        // a word's eight values lie in one block (block_size is a multiple of 8); a shift when it is a power of two
        const int b = bs_shift >= 0 ? k0 >> bs_shift : k0 / block_size;
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
// of column n -- exactly the B operand of one 16x16x32 MFMA per word -- in the nibble order
// k0 k2 k4 k6 k1 k3 k5 k7, so that (word >> 4 i) & 0x000f000f is the pair (k_2i, k_2i+1).
// SG scale groups per tile (4 when block_size == 32, 2 for 64, 1 for >= 128).
template <typename ST>
__global__ void __launch_bounds__(256)
mmnb_prepack_kernel(const uint32_t *__restrict__ B, const ST *__restrict__ scales, const uint8_t *__restrict__ zp,
                    uint4 *__restrict__ Wq, float *__restrict__ Sc, uint8_t *__restrict__ Zb, int N, int n_blocks,
                    int row_words, int zp_row, long n_tile_total, int n_cg, int cpb_shift, int SG, int half) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    const long tile = idx >> 6;
    if (tile >= n_tile_total) return;
    const int lane = (int)(idx & 63);
    const int nt = (int)(tile / n_cg), cg = (int)(tile % n_cg);
    const int i16 = lane & 15, w = lane >> 4;
    // half > 0: the weight is two matrices side by side ([gate | up], `half` columns each) and the
    // packed column tiles alternate between them: tile 2 b holds columns 16 b .. of the first, tile
    // 2 b + 1 the same columns of the second, so that one workgroup holds both halves of an output
    int n = nt * 16 + i16;
    if (half > 0) {
        const int c = (nt >> 1) * 16 + i16;
        n = c < half ? c + (nt & 1) * half : N;
    }
    uint32_t v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int widx = (cg * 4 + j) * 4 + w;
        const uint32_t raw = (n < N && widx < row_words) ? B[(size_t)n * row_words + widx] : 0u;
        // nibble order k0 k2 k4 k6 k1 k3 k5 k7: then (word >> 4 i) & 0x000f000f is the pair (k_2i, k_2i+1)
        const uint32_t even = raw & 0x0f0f0f0fu, odd = (raw >> 4) & 0x0f0f0f0fu;
        auto squeeze = [](uint32_t e) { return (e & 0xfu) | ((e >> 4) & 0xf0u) | ((e >> 8) & 0xf00u) | ((e >> 12) & 0xf000u); };
        v[j] = squeeze(even) | (squeeze(odd) << 16);
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
    int a_vec;  // rows of A may be read 8 elements at a time (base 16-byte aligned, K % 8 == 0)
    uint32_t nib_mask, magic;  // 0x000f000f and 0x43004300 (bf16 128.0 in both halves)
    // activation prologues of the decoder (one row of f32): see GemvPrologue
    const float *nx, *ny, *nw_post, *nw_in;
    float *nx_out;
    float eps;
    // attention-merge prologue: nx = partial outputs, ny = (max, sum) pairs
    const int *npos;
    int ngroup, nhd, nwindow;
    int nparts;   // ways the live chunks are divided among threads that share four channels
    int ny_slices; // norm prologue: ny is this many partial rows, K floats apart, that add up to y
    int pro_off;  // byte offset of the prologue's own LDS area
    // argmax epilogue (one f32 row, k not split over workgroups): workgroup b leaves the largest result it stored and
    // its column in am_v[b], am_i[b]; null: no epilogue
    float *am_v;
    int *am_i;
};

template <int SG>
struct ScaleVec;
template <>
struct ScaleVec<4> {
    float s[4];
    uint32_t z;
    __device__ __forceinline__ void load(const float *sc, const uint8_t *zb, uint32_t at, bool stream = false) {
        typedef float nt_f32x4 __attribute__((ext_vector_type(4)));
        const nt_f32x4 *sp = reinterpret_cast<const nt_f32x4 *>(reinterpret_cast<const char *>(sc) + at * 16u);
        const uint32_t *zp = reinterpret_cast<const uint32_t *>(zb + at * 4u);
        const nt_f32x4 v = stream ? __builtin_nontemporal_load(sp) : *sp;  // see load_stage
        s[0] = v.x, s[1] = v.y, s[2] = v.z, s[3] = v.w;
        z = stream ? __builtin_nontemporal_load(zp) : *zp;
    }
};
template <>
struct ScaleVec<2> {
    float s[2];
    uint32_t z;
    __device__ __forceinline__ void load(const float *sc, const uint8_t *zb, uint32_t at) {
        const float2 v = *reinterpret_cast<const float2 *>(reinterpret_cast<const char *>(sc) + at * 8u);
        s[0] = v.x, s[1] = v.y;
        z = *reinterpret_cast<const uint16_t *>(zb + at * 2u);
    }
};
template <>
struct ScaleVec<1> {
    float s[1];
    uint32_t z;
    __device__ __forceinline__ void load(const float *sc, const uint8_t *zb, uint32_t at) {
        s[0] = *reinterpret_cast<const float *>(reinterpret_cast<const char *>(sc) + at * 4u);
        z = zb[at];
    }
};

// One k tile (128 k) of T column tiles, as it arrives from HBM.
template <int T, int SG>
struct GemvStage {
    uint4 wq[T];
    ScaleVec<SG> sv[T];
};

__device__ __forceinline__ uint32_t bf16_rne(float v) {  // bits of the nearest bf16, in the high half
    const uint32_t u = __float_as_uint(v);
    return (u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u;
}

// T:  16-column tiles per wavefront.
// NR: accumulator registers in use (rows m = (lane>>4) + 4r, r < NR, so M <= 4*NR).
// SG: scale groups per 128-k tile.
// MC: M when it is known at compile time (1), else 0 -- with it the LDS offsets of the activation
//     operands become immediates.
// NT: bf16 terms an activation is split into. Three terms carry all 24 bits of an f32; two carry
//     16 (relative error 2^-17 per element after rounding, below what f32 accumulation over K
//     itself loses) and are exact for f16 activations. The block sums that remove the +128 bias
//     are taken over the SAME split values, so the bias cancels exactly either way.
//
// A workgroup is WK x WN wavefronts: WN column groups side by side, each split WK ways along k.
// It walks column groups blockIdx.x*WN, += gridDim.x*WN (a persistent grid when N is large), so
// the activation split is paid once per workgroup, and every wavefront keeps the next tile's
// loads in flight while it multiplies the current one -- across group boundaries too. Those
// loads are unconditional (indices are clamped instead), so the wait counters stay exact, and
// the two stage buffers swap roles by code duplication, not by copies.
// The workgroup is at most 16 / T wavefronts (8 / T with all four accumulator registers in use),
// which leaves the wide variants their registers.
// PRO selects what the one activation row is (decoder glue folded into the prologue, M == 1, f32):
//   0  A as given
//   1  gelu_tanh(A[k]) * A[K + k]                      (gated FFN: A = [gate | up])
//   2  rmsnorm(x', nw_in) with x' = nx + rmsnorm(ny, nw_post) (x' = nx when ny is null); every
//      workgroup forms the two sums of squares over the whole row itself, workgroup (0, 0) also
//      writes x' to nx_out (a different buffer than nx: others may still be reading nx)
//   3  the attention output of the step: sum_s exp(m_s - m) o_s / sum_s exp(m_s - m) l_s over the
//      live context chunks s of each head (flash-decoding merge); every workgroup forms the whole
//      row itself out of L2
template <int T, int NR, int SG, int MC, int NT, int PRO>
__global__ void __launch_bounds__(1024 / T / (NR == 4 ? 2 : 1)) mmnb_gemv_kernel(const GemvArgs p) {
    extern __shared__ uint4 smem[];
    // the arguments every instance uses are read here, in one batch (left to the compiler, each is read next to its first
    // use: a trip to memory of its own in the middle of the kernel, since the scalar cache starts every launch empty)
    HIPC_ARG_NOW(p.A); HIPC_ARG_NOW(p.Wq); HIPC_ARG_NOW(p.Sc); HIPC_ARG_NOW(p.Zb); HIPC_ARG_NOW(p.Y); HIPC_ARG_NOW(p.Ypart);
    HIPC_ARG_NOW(p.M); HIPC_ARG_NOW(p.K); HIPC_ARG_NOW(p.N); HIPC_ARG_NOW(p.n_tiles); HIPC_ARG_NOW(p.n_cg); HIPC_ARG_NOW(p.WK); HIPC_ARG_NOW(p.WN);
    HIPC_ARG_NOW(p.slice_tiles); HIPC_ARG_NOW(p.ksplit); HIPC_ARG_NOW(p.a_f16); HIPC_ARG_NOW(p.a_vec); HIPC_ARG_NOW(p.nib_mask); HIPC_ARG_NOW(p.magic);
    HIPC_ARG_NOW(p.am_v); HIPC_ARG_NOW(p.am_i);
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int M = MC > 0 ? MC : p.M;
    const int tile0 = blockIdx.y * p.slice_tiles;
    const int tile1 = min(p.n_cg, tile0 + p.slice_tiles);
    const int nch = (tile1 - tile0) * 4;  // 32-k chunks in this slice

    // LDS: As [nch][NT terms][4 k-groups][M] 16-byte operands | asum [nch][M] | red
    uint4 *As = smem;
    float *asum = reinterpret_cast<float *>(As + (size_t)nch * (4 * NT) * M);
    float *red = asum + ((nch * M + 3) & ~3);  // [WN][WK][T][NR][64]

    // the wavefront's number is told to the compiler as the scalar it is: the tile cursors derived
    // from it then live in scalar registers and cost the vector unit nothing
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wk = wave % p.WK, wn = wave / p.WK;
    const int i16 = lane & 15, g4 = lane >> 4;
    const int groups = (p.n_tiles + T - 1) / T;
    const int gstride = gridDim.x * p.WN;
    // the nibble mask and the bf16 bias pattern travel as kernel arguments so that they live in
    // registers and each unpack step is one v_and_or_b32 instead of an and and an or with literals
    const uint32_t nib_mask = p.nib_mask;
    uint32_t magic;  // held in a vector register: only one scalar operand fits the constant bus
    HIPC_VGPR_FROM_SGPR(magic, p.magic);

    // 32-bit byte offsets from uniform bases (the prepacked weight is below 4 GiB)
    const char *wq_base = reinterpret_cast<const char *>(p.Wq);
    const uint32_t lane16 = (uint32_t)lane * 16u;
    auto load_stage = [&](int ng, int tile, GemvStage<T, SG> &st) {
#pragma unroll
        for (int t = 0; t < T; t++) {
            const uint32_t nt = (uint32_t)min(ng * T + t, p.n_tiles - 1);
            const uint32_t tl = nt * (uint32_t)p.n_cg + (uint32_t)tile;
            // The wide variant runs where a weight of hundreds of MB is streamed once: its nibbles are
            // read with non-temporal loads (36 against 40 us on the 1152 x 262144 unembedding). The
            // narrow variant keeps ordinary loads: its few tiles per wavefront are re-read (clamped
            // loads past the end, the other k wavefronts' neighbours) and it lost 8 % with them.
            typedef unsigned int nt_u32x4 __attribute__((ext_vector_type(4)));
            const nt_u32x4 *src = reinterpret_cast<const nt_u32x4 *>(wq_base + (tl * 1024u + lane16));
            st.wq[t] = __builtin_bit_cast(uint4, T >= 2 ? __builtin_nontemporal_load(src) : *src);
            if constexpr (SG == 4)
                st.sv[t].load(p.Sc, p.Zb, tl * 16u + (uint32_t)i16, T >= 2);
            else
                st.sv[t].load(p.Sc, p.Zb, tl * 16u + (uint32_t)i16);
        }
    };

    // ---- Prologue. The activations are split into NT bf16 terms, in operand order, into LDS.
    // An "item" is 8 consecutive k of one row. On the fast path (aligned rows) a thread's first
    // item is read with two unconditional 128-bit loads issued BEFORE the first weight tile's
    // loads, so the split only waits for the activations (an L2 hit) while the weights stream in.
    const int nitems = M * nch * 4;
    const int kbase = tile0 * 128;
    auto item_k0 = [&](int item, int &m, int &c, int &w) {
        w = item & 3, c = (item >> 2) % nch, m = (item >> 2) / nch;
        return kbase + c * 32 + w * 8;
    };
    // D stage buffers per wavefront: one tile is multiplied while the next travels. Four buffers
    // (three tiles in flight) measured slower everywhere: 43.8 against 39.7 us on the 1152 x 262144
    // unembedding (T = 2), and 0.3 to 0.5 us more on each of the decoder's projections (T = 1),
    // whose wavefronts have only three or four tiles to fetch in the first place.
    constexpr int D = 2;
    GemvStage<T, SG> st[D];
    int ng = blockIdx.x * p.WN + wn;
    const int first_ng = min(ng, groups - 1), first_tile = min(tile0 + wk, tile1 - 1);
    // every wavefront of the workgroup sees the same number of column groups (and so of barriers);
    // the number of k tiles per group may differ by one between wavefronts, and can be zero
    const int first_group = blockIdx.x * p.WN;
    const int my_groups = first_group < groups ? (groups - first_group + gstride - 1) / gstride : 0;
    const int span = tile1 - tile0;
    const int my_tiles = wk < span ? (span - wk + p.WK - 1) / p.WK : 0;
    // the load cursor runs D - 1 tiles ahead of the one being multiplied: same group, or the first
    // tile of this wavefront's next group, or (past the end) tiles of a group that does not exist,
    // which become loads of one tile that the caches hold
    int l_tile = first_tile, l_ng = ng, l_ti = 0;
    auto load_ahead = [&](GemvStage<T, SG> &dst) {
        const bool group_done = l_ti + 1 >= my_tiles;
        l_tile = group_done ? first_tile : l_tile + p.WK;
        l_ng = group_done ? l_ng + gstride : l_ng;
        l_ti = group_done ? 0 : l_ti + 1;
        // past the end: every wavefront asks for the same tile (0, 0), which the caches hold, instead
        // of fetching another tile of its own that nobody will use
        const bool past = l_ng >= groups;
        load_stage(past ? 0 : l_ng, past ? 0 : l_tile, dst);
    };
    auto load_first = [&]() {
        load_stage(first_ng, first_tile, st[0]);
#pragma unroll
        for (int d = 1; d < D; d++) load_ahead(st[d]);
    };
    float inv1 = 0.f, inv2 = 0.f;
    // PRO 2, whole row in this workgroup and at most one item per thread: the operands of the item
    // are read once, the two sums of squares are taken over the registers, and the item is split
    // from them -- one memory round trip where the general path below makes three.
    const bool row_once = PRO == 2 && tile0 == 0 && tile1 * 128 >= p.K && nitems <= nthreads;
    float av_row[8];
    // PRO 2: element c of y, which may arrive as ny_slices partial rows
    auto y_at = [&](int c) {
        float v = p.ny[c];
        for (int s = 1; s < p.ny_slices; s++) v += p.ny[(size_t)s * p.K + c];
        return v;
    };
    if (PRO == 2) {
        __shared__ float nred[16];
        const int nw = nthreads >> 6;
        auto block_total = [&](float v) {
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
            __syncthreads();
            if ((tid & 63) == 0) nred[tid >> 6] = v;
            __syncthreads();
            float t = 0.f;
            for (int i = 0; i < nw; i++) t += nred[i];
            return t;
        };
        const bool writer = blockIdx.x == 0 && blockIdx.y == 0 && p.nx_out;
        if (row_once) {
            const bool mine = tid * 8 < p.K;  // K % 8 == 0; items past K are padding
            const int k0 = min(tid * 8, p.K - 8);
            auto ld8 = [&](const float *src, float o[8]) {
                const float4 a = reinterpret_cast<const float4 *>(src + k0)[0], b = reinterpret_cast<const float4 *>(src + k0)[1];
                o[0] = a.x, o[1] = a.y, o[2] = a.z, o[3] = a.w, o[4] = b.x, o[5] = b.y, o[6] = b.z, o[7] = b.w;
            };
            float x8[8], y8[8], p8[8], w8[8];
            ld8(p.nx, x8), ld8(p.nw_in, w8);
            if (p.ny) {
                ld8(p.ny, y8), ld8(p.nw_post, p8);
                for (int s = 1; s < p.ny_slices; s++) {   // y arrives as partial rows
                    float t8[8];
                    ld8(p.ny + (size_t)s * p.K, t8);
#pragma unroll
                    for (int i = 0; i < 8; i++) y8[i] += t8[i];
                }
            }
            load_first();  // the first weight tiles travel while the row is normalised
            if (p.ny) {
                float sq = 0.f;
#pragma unroll
                for (int i = 0; i < 8; i++) sq += y8[i] * y8[i];
                inv1 = rsqrtf(block_total(mine ? sq : 0.f) / (float)p.K + p.eps);
#pragma unroll
                for (int i = 0; i < 8; i++) x8[i] += y8[i] * inv1 * p8[i];
            }
            float sq2 = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) sq2 += x8[i] * x8[i];
            inv2 = rsqrtf(block_total(mine ? sq2 : 0.f) / (float)p.K + p.eps);
            if (writer && mine) {
                reinterpret_cast<float4 *>(p.nx_out + k0)[0] = make_float4(x8[0], x8[1], x8[2], x8[3]);
                reinterpret_cast<float4 *>(p.nx_out + k0)[1] = make_float4(x8[4], x8[5], x8[6], x8[7]);
            }
#pragma unroll
            for (int i = 0; i < 8; i++) av_row[i] = x8[i] * inv2 * w8[i];
        } else {
            load_first();
            if (p.ny) {
                float sq = 0.f;
                for (int c = tid; c < p.K; c += nthreads) sq += y_at(c) * y_at(c);
                inv1 = rsqrtf(block_total(sq) / (float)p.K + p.eps);
            }
            float sq2 = 0.f;
            for (int c = tid; c < p.K; c += nthreads) {
                const float xp = p.ny ? p.nx[c] + y_at(c) * inv1 * p.nw_post[c] : p.nx[c];
                sq2 += xp * xp;
                if (writer) p.nx_out[c] = xp;
            }
            inv2 = rsqrtf(block_total(sq2) / (float)p.K + p.eps);
        }
    }
    float *mrow = nullptr;  // PRO 3: [nparts][K] partial sums of the merged row, then inv per head
    float *minv = nullptr;
    if (PRO == 3) {
        const int total = *p.npos + 1;
        const int live = attn_live_chunks(attn_span(total, p.nwindow));
        const int G = p.ngroup, hd = p.nhd, GH = G * hd, n_q = p.K / hd;
        float *wgt = reinterpret_cast<float *>(reinterpret_cast<char *>(smem) + p.pro_off);  // [n_q][kAttnSplits]
        minv = wgt + n_q * kAttnSplits;                                                     // [n_q]
        mrow = minv + ((n_q + 3) & ~3);
        const int nw = nthreads >> 6, ln = tid & 63, wv = tid >> 6;
        static_assert(kAttnSplits <= 64, "one lane per chunk");
        auto stat_at = [&](int h) {
            const int hh = min(h, n_q - 1), kvh = hh / G, g = hh % G;
            return *reinterpret_cast<const float2 *>(p.ny + (((size_t)kvh * kAttnSplits + min(ln, live - 1)) * G + g) * 2);
        };
        float2 ml = stat_at(wv);                 // the statistics are asked for first ...
        load_first();                            // ... the first weight tiles travel meanwhile
        for (int h = wv; h < n_q; h += nw) {
            if (h != wv) ml = stat_at(h);
            const bool on = ln < live;
            float m = on ? ml.x : -3.0e38f;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
            const float e = on ? __expf(ml.x - m) : 0.f;
            float l = on ? ml.y * e : 0.f;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) l += __shfl_xor(l, off, 64);
            if (ln < kAttnSplits) wgt[h * kAttnSplits + ln] = e;
            if (ln == 0) minv[h] = 1.f / l;
        }
        __syncthreads();
        const int groups4 = p.K >> 2;
        for (int u = tid; u < groups4 * p.nparts; u += nthreads) {
            const int c4 = u % groups4, part = u / groups4;
            const int e0 = c4 * 4, h = e0 / hd, kvh = h / G;
            const int s0 = part * live / p.nparts, s1 = (part + 1) * live / p.nparts;
            const float *src = p.nx + (size_t)kvh * kAttnSplits * GH + (e0 - kvh * GH);
            const float *wh = wgt + h * kAttnSplits;
            float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
            for (int s = s0; s < s1; s += 8) {
                float4 f[8];
#pragma unroll
                for (int j = 0; j < 8; j++) f[j] = *reinterpret_cast<const float4 *>(src + (size_t)min(s + j, s1 - 1) * GH);
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const float ws = s + j < s1 ? wh[s + j] : 0.f;
                    o.x += f[j].x * ws, o.y += f[j].y * ws, o.z += f[j].z * ws, o.w += f[j].w * ws;
                }
            }
            *reinterpret_cast<float4 *>(mrow + (size_t)part * p.K + e0) = o;
        }
        __syncthreads();
    }
    auto load_item_vec = [&](int item, float av[8]) {
        int m, c, w;
        const int k0 = min(item_k0(item, m, c, w), p.K - 8);  // padding chunks are zeroed by split_item
        if (PRO == 1) {
            const float4 *g = reinterpret_cast<const float4 *>(static_cast<const float *>(p.A) + k0);
            const float4 *u = reinterpret_cast<const float4 *>(static_cast<const float *>(p.A) + p.K + k0);
            const float4 g0 = g[0], g1 = g[1], u0 = u[0], u1 = u[1];
            const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
            const float uv[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float v = gv[i];
                av[i] = 0.5f * v * (1.f + tanhf(0.79788456080286536f * fmaf(0.044715f, v * v * v, v))) * uv[i];
            }
        } else if (PRO == 2) {
            auto ld8 = [&](const float *src, float o[8]) {
                const float4 a = reinterpret_cast<const float4 *>(src + k0)[0], b = reinterpret_cast<const float4 *>(src + k0)[1];
                o[0] = a.x, o[1] = a.y, o[2] = a.z, o[3] = a.w, o[4] = b.x, o[5] = b.y, o[6] = b.z, o[7] = b.w;
            };
            float x8[8], y8[8], p8[8], w8[8];
            ld8(p.nx, x8), ld8(p.nw_in, w8);
            if (p.ny) {
                ld8(p.ny, y8), ld8(p.nw_post, p8);
                for (int s = 1; s < p.ny_slices; s++) {
                    float t8[8];
                    ld8(p.ny + (size_t)s * p.K, t8);
#pragma unroll
                    for (int i = 0; i < 8; i++) y8[i] += t8[i];
                }
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float xp = p.ny ? x8[i] + y8[i] * inv1 * p8[i] : x8[i];
                av[i] = xp * inv2 * w8[i];
            }
        } else if (PRO == 3) {
            const float inv = minv[k0 / p.nhd];
#pragma unroll
            for (int i = 0; i < 8; i++) av[i] = 0.f;
            for (int part = 0; part < p.nparts; part++) {
                const float4 a = *reinterpret_cast<const float4 *>(mrow + (size_t)part * p.K + k0);
                const float4 b = *reinterpret_cast<const float4 *>(mrow + (size_t)part * p.K + k0 + 4);
                av[0] += a.x, av[1] += a.y, av[2] += a.z, av[3] += a.w, av[4] += b.x, av[5] += b.y, av[6] += b.z, av[7] += b.w;
            }
#pragma unroll
            for (int i = 0; i < 8; i++) av[i] *= inv;
        } else if (p.a_f16) {
            const uint4 raw = *reinterpret_cast<const uint4 *>(static_cast<const __half *>(p.A) + (size_t)m * p.K + k0);
            const __half2 *h = reinterpret_cast<const __half2 *>(&raw);
#pragma unroll
            for (int i = 0; i < 4; i++) av[2 * i] = __low2float(h[i]), av[2 * i + 1] = __high2float(h[i]);
        } else {
            const float4 *src = reinterpret_cast<const float4 *>(static_cast<const float *>(p.A) + (size_t)m * p.K + k0);
            const float4 lo4 = src[0], hi4 = src[1];
            av[0] = lo4.x, av[1] = lo4.y, av[2] = lo4.z, av[3] = lo4.w;
            av[4] = hi4.x, av[5] = hi4.y, av[6] = hi4.z, av[7] = hi4.w;
        }
    };
    auto load_item_scalar = [&](int item, float av[8]) {
        int m, c, w;
        const int k0 = item_k0(item, m, c, w);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int k = min(k0 + i, p.K - 1);
            av[i] = p.a_f16 ? __half2float(static_cast<const __half *>(p.A)[(size_t)m * p.K + k])
                            : static_cast<const float *>(p.A)[(size_t)m * p.K + k];
        }
    };
    // splits one item and writes it (all four lanes of a chunk are active together: items come in fours)
    auto split_item = [&](int item, const float av[8]) {
        int m, c, w;
        const int k0 = item_k0(item, m, c, w);
        uint32_t t0[8], t1[8], t2[8];
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float a = (k0 + i < p.K) ? av[i] : 0.f;
            t0[i] = __float_as_uint(a) & 0xffff0000u;                 // hi: truncated
            const float r1 = a - __uint_as_float(t0[i]);              // exact
            float rep;
            if (NT == 2) {
                t1[i] = bf16_rne(r1);
                t2[i] = 0;
                rep = __uint_as_float(t0[i]) + __uint_as_float(t1[i]);  // exact: 16 significant bits
            } else {
                t1[i] = __float_as_uint(r1) & 0xffff0000u;
                t2[i] = bf16_rne(r1 - __uint_as_float(t1[i]));
                rep = a;  // the three terms carry every bit of a (up to one rounding in the last)
            }
            s += rep;
        }
        s += __shfl_xor(s, 1, 64);
        s += __shfl_xor(s, 2, 64);
        const size_t slot = ((size_t)c * (4 * NT) + w) * M + m;
        // k order, two bf16 per word: the nibble unpack below yields the pairs (k0,k1) (k2,k3) (k4,k5) (k6,k7)
        As[slot] = make_uint4((t0[0] >> 16) | t0[1], (t0[2] >> 16) | t0[3], (t0[4] >> 16) | t0[5], (t0[6] >> 16) | t0[7]);
        As[slot + 4 * M] = make_uint4((t1[0] >> 16) | t1[1], (t1[2] >> 16) | t1[3], (t1[4] >> 16) | t1[5], (t1[6] >> 16) | t1[7]);
        if (NT == 3)
            As[slot + 8 * M] = make_uint4((t2[0] >> 16) | t2[1], (t2[2] >> 16) | t2[3], (t2[4] >> 16) | t2[5], (t2[6] >> 16) | t2[7]);
        if (w == 0) asum[c * M + m] = s;
    };

    if (p.a_vec) {
        float av[8];
        if (row_once) {
#pragma unroll
            for (int i = 0; i < 8; i++) av[i] = av_row[i];
        } else {
            load_item_vec(min(tid, nitems - 1), av);
        }
        if (PRO != 2 && PRO != 3) load_first();
        if (tid < nitems) split_item(tid, av);
        for (int item = tid + nthreads; item < nitems; item += nthreads) {
            load_item_vec(item, av);
            split_item(item, av);
        }
    } else {
        load_first();
        for (int item = tid; item < nitems; item += nthreads) {
            float av[8];
            load_item_scalar(item, av);
            split_item(item, av);
        }
    }
    __syncthreads();

    // The row of the 16x16 tile this lane feeds as the A operand. Lanes whose row is not one of
    // the M activations read row 0 instead: the rows of a matrix product are independent, and the
    // output rows they pollute are never stored.
    const int mA = (i16 >> 2) + 4 * (i16 & 3);
    const uint4 *a_lane = As + g4 * M + (mA < M ? mA : 0);
    const float *s_lane[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) s_lane[r] = asum + (g4 + 4 * r < M ? g4 + 4 * r : 0);

    f32x4 acc[T];
#pragma unroll
    for (int t = 0; t < T; t++) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto compute = [&](const GemvStage<T, SG> &cur, int tile) {
        const uint4 *a_tile = a_lane + (size_t)(tile - tile0) * (16 * NT) * M;
        f32x4 c[T];
        float asg[NR], s_q[T], zb_q[T], as_q[NR];
        f32x4 d_q[T];
        constexpr int CPG = 4 / SG;  // chunks per scale group
#pragma unroll
        for (int j = 0; j < 4; j++) {
            bf16x8 a_op[NT];
#pragma unroll
            for (int e = 0; e < NT; e++) a_op[e] = __builtin_bit_cast(bf16x8, a_tile[(j * (4 * NT) + 4 * e) * M]);
            const bool first = (j % CPG) == 0, last = (j % CPG) == CPG - 1;
#pragma unroll
            for (int r = 0; r < NR; r++) {
                const float v = s_lane[r][((tile - tile0) * 4 + j) * M];
                asg[r] = first ? v : asg[r] + v;
            }
#pragma unroll
            for (int t = 0; t < T; t++) {
                const uint32_t word = j == 0 ? cur.wq[t].x : j == 1 ? cur.wq[t].y : j == 2 ? cur.wq[t].z : cur.wq[t].w;
                const uint4 bw = make_uint4((word & nib_mask) | magic, ((word >> 4) & nib_mask) | magic,
                                            ((word >> 8) & nib_mask) | magic, ((word >> 12) & nib_mask) | magic);
                const bf16x8 b = __builtin_bit_cast(bf16x8, bw);
                f32x4 d = first ? f32x4{0.f, 0.f, 0.f, 0.f} : c[t];
#pragma unroll
                for (int e = 0; e < NT; e++) d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_op[e], b, d, 0, 0, 0);
                c[t] = d;
            }
            // the epilogue of the scale group that ended one chunk ago runs behind this chunk's MFMAs
            if (j > 0 && ((j - 1) % CPG) == CPG - 1) {
#pragma unroll
                for (int t = 0; t < T; t++)
#pragma unroll
                    for (int r = 0; r < NR; r++)
                        acc[t][r] = fmaf(s_q[t], fmaf(-zb_q[t], as_q[r], d_q[t][r]), acc[t][r]);
            }
            if (last) {
                const int g = j / CPG;
#pragma unroll
                for (int t = 0; t < T; t++) {
                    d_q[t] = c[t];
                    s_q[t] = cur.sv[t].s[g];
                    zb_q[t] = (float)((cur.sv[t].z >> (8 * g)) & 0xffu);
                }
#pragma unroll
                for (int r = 0; r < NR; r++) as_q[r] = asg[r];
            }
        }
#pragma unroll
        for (int t = 0; t < T; t++)
#pragma unroll
            for (int r = 0; r < NR; r++) acc[t][r] = fmaf(s_q[t], fmaf(-zb_q[t], as_q[r], d_q[t][r]), acc[t][r]);
    };

    // argmax epilogue: the largest result this lane has stored and its column (smallest column on ties; a NaN never wins)
    float am_best = -3.4e38f;
    int am_col = 0x7fffffff;
    __shared__ float am_sv[16];
    __shared__ int am_si[16];
    auto argmax_out = [&]() {   // the workgroup's candidate: over the lanes, then over the wavefronts
        if (!p.am_v) return;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const float ov = __shfl_xor(am_best, off, 64);
            const int oc = __shfl_xor(am_col, off, 64);
            if (ov > am_best || (ov == am_best && oc < am_col)) am_best = ov, am_col = oc;
        }
        if (lane == 0) am_sv[wave] = am_best, am_si[wave] = am_col;
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < nthreads / 64; w++)
                if (am_sv[w] > am_best || (am_sv[w] == am_best && am_si[w] < am_col)) am_best = am_sv[w], am_col = am_si[w];
            p.am_v[blockIdx.x] = am_best, p.am_i[blockIdx.x] = am_col;
        }
    };

    // one column group is done: reduce over the k wavefronts, store, clear
    auto group_end = [&](bool more_groups) {
        if (p.WK > 1) {
#pragma unroll
            for (int t = 0; t < T; t++)
#pragma unroll
                for (int r = 0; r < NR; r++)
                    red[((((size_t)wn * p.WK + wk) * T + t) * NR + r) * 64 + lane] = acc[t][r];
            __syncthreads();
            if (wk == 0) {
#pragma unroll
                for (int t = 0; t < T; t++)
#pragma unroll
                    for (int r = 0; r < NR; r++) {
                        float v = acc[t][r];
                        for (int k = 1; k < p.WK; k++)
                            v += red[((((size_t)wn * p.WK + k) * T + t) * NR + r) * 64 + lane];
                        acc[t][r] = v;
                    }
            }
            if (more_groups) __syncthreads();  // the buffer is written again next round
        }
        if (wk == 0 && ng < groups) {
#pragma unroll
            for (int t = 0; t < T; t++) {
                const int n = (ng * T + t) * 16 + i16;
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
                            if (p.am_v && (acc[t][r] > am_best || (acc[t][r] == am_best && n < am_col))) am_best = acc[t][r], am_col = n;   // (M is 1 there)
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int t = 0; t < T; t++) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    };

    if (my_tiles == 0) {
        for (int g = 0; g < my_groups; g++) {
            group_end(g + 1 < my_groups);
            ng += gstride;
        }
        argmax_out();
        return;
    }
    int tile = tile0 + wk, ti = 0, gi = 0;
    // The steps come in rounds of D with nothing conditional about their loads, so that every wait
    // is for exactly the tile about to be multiplied. Steps past the last group (the final round is
    // padded) multiply nothing and end no group; what they load is clamped and stays unused.
    auto step = [&](GemvStage<T, SG> &cur) {
        const bool live = ng < groups;
        if (live) compute(cur, tile);
        load_ahead(cur);  // its registers are free again: the tile D ahead
        const bool group_done = live && ti + 1 == my_tiles;
        if (group_done) {
            gi++;
            group_end(gi < my_groups);
        }
        ti = group_done ? 0 : ti + 1;
        tile = group_done ? tile0 + wk : tile + p.WK;
        ng = group_done ? ng + gstride : ng;
    };
    const int rounds = (my_groups * my_tiles + D - 1) / D;
    for (int r = 0; r < rounds; r++) {
#pragma unroll
        for (int d = 0; d < D; d++) step(st[d]);
    }
    argmax_out();
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

namespace {

// Launch-shape overrides (the context's Tuning): gemv_t (16-column tiles per wavefront: 1, 2 or 4),
// gemv_waves (wavefronts to aim for when k is split inside a workgroup) and gemv_per_cu (resident
// wavefronts per CU of the persistent grid).

int log2i(int64_t v) {
    int s = 0;
    while ((int64_t(1) << s) < v) s++;
    return s;
}

int check_nbits_shape(hipc_ctx *ctx, int64_t M, int64_t K, int64_t N, int64_t block_size, size_t b_len,
                      size_t scales_len, const void *zp, size_t zp_len, int scale_dtype) {
    HIPC_REQUIRE(ctx, M >= 0 && K > 0 && N >= 0, "MatMulNBits: bad dimensions M=%ld K=%ld N=%ld", (long)M, (long)K,
                 (long)N);
    // the reference's envelope (interp.rs:447-464): any positive multiple of 8, "so a packed u32 never straddles
    // two blocks"; the operator's own definition asks for a power of two >= 16
    HIPC_REQUIRE(ctx, block_size > 0 && block_size % 8 == 0, "MatMulNBits: block_size %ld is not a positive multiple of 8",
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
    const int bs_shift = is_pow2(block_size) ? log2i(block_size) : -1;
    const dim3 block(256);
    int64_t m_done = 0;
    while (m_done < M) {  // grid.y is limited to 65535 row groups
        const int64_t rows = std::min<int64_t>(M - m_done, 65535 * 4);
        const AT *a = static_cast<const AT *>(A) + m_done * K;
        AT *y = static_cast<AT *>(Y) + m_done * N;
        if (rows == 1) {
            hipLaunchKernelGGL((mmnb_direct_kernel<AT, ST, 1>), dim3((unsigned)ceil_div(N, 4), 1), block, 0, ctx->stream, a, static_cast<const uint32_t *>(B), static_cast<const ST *>(scales), static_cast<const uint8_t *>(zp),
                y, (int)rows, (int)K, (int)N, bs_shift, (int)block_size, n_blocks, row_words, zp_row);
        } else {
            hipLaunchKernelGGL((mmnb_direct_kernel<AT, ST, 4>), dim3((unsigned)ceil_div(N, 4), (unsigned)ceil_div(rows, 4)), block, 0, ctx->stream, a, static_cast<const uint32_t *>(B), static_cast<const ST *>(scales),
                    static_cast<const uint8_t *>(zp), y, (int)rows, (int)K, (int)N, bs_shift, (int)block_size, n_blocks, row_words,
                    zp_row);
        }
        HIPC_LAUNCHED(ctx);
        m_done += rows;
    }
    return HIPC_OK;
}

template <int T, int NR, int MC, int NT, int PRO = 0>
void launch_gemv_sg(const GemvArgs &a, int SG, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
    if (SG == 4)
        hipLaunchKernelGGL((mmnb_gemv_kernel<T, NR, 4, MC, NT, PRO>), grid, block, lds, s, a);
    else if (SG == 2)
        hipLaunchKernelGGL((mmnb_gemv_kernel<T, NR, 2, MC, NT, PRO>), grid, block, lds, s, a);
    else
        hipLaunchKernelGGL((mmnb_gemv_kernel<T, NR, 1, MC, NT, PRO>), grid, block, lds, s, a);
}

template <int T, int NT>
void launch_gemv_nr(const GemvArgs &a, int pro, int NR, int SG, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
    if (a.M == 1 && pro == 1 && NT == 2)
        launch_gemv_sg<T, 1, 1, 2, 1>(a, SG, grid, block, lds, s);
    else if (a.M == 1 && pro == 2 && NT == 2)
        launch_gemv_sg<T, 1, 1, 2, 2>(a, SG, grid, block, lds, s);
    else if (a.M == 1 && pro == 3 && NT == 2)
        launch_gemv_sg<T, 1, 1, 2, 3>(a, SG, grid, block, lds, s);
    else if (a.M == 1)
        launch_gemv_sg<T, 1, 1, NT>(a, SG, grid, block, lds, s);
    else if (NR == 1)
        launch_gemv_sg<T, 1, 0, NT>(a, SG, grid, block, lds, s);
    else if (NR == 2)
        launch_gemv_sg<T, 2, 0, NT>(a, SG, grid, block, lds, s);
    else
        launch_gemv_sg<T, 4, 0, NT>(a, SG, grid, block, lds, s);
}

template <int T>
void launch_gemv_nt(const GemvArgs &a, int pro, int NT, int NR, int SG, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
    if (NT == 3)
        launch_gemv_nr<T, 3>(a, 0, NR, SG, grid, block, lds, s);
    else
        launch_gemv_nr<T, 2>(a, pro, NR, SG, grid, block, lds, s);
}

// rows [0, M) with M <= 16 of one activation matrix against a prepacked weight
int launch_gemv(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_nbits_weight *w, void *Y, int M, int NT,
                const GemvPrologue *pro = nullptr, GemvArgmax *am = nullptr) {
    if (am) am->parts = 0;
    HIPC_REQUIRE(ctx, w->interleave_half == 0, "MatMulNBits gemv: this weight was prepacked with interleaved halves for the decoder");
    // one plain f32 row on a narrow output: the kernel built for latency (gemv_lean.hip); the
    // gemv_lean option set to 0 keeps this kernel (tuning, tests)
    if (M == 1 && a_dtype == HIPC_F32 && !(pro && pro->mode) && aligned(A, 16) && aligned(Y, 4) && w->n_tiles < 2048 &&
        ctx->tune.gemv_lean != 0) {
        LeanPlan pl;
        // several column tiles per workgroup once that still leaves a workgroup for most CUs: the row is then prepared
        // (read, split into terms, written to LDS) by a half or a quarter as many workgroups (1152 -> 13824: 5.4 -> 5.0 us)
        const int WN = w->n_tiles >= 768 ? 4 : w->n_tiles >= 384 ? 2 : 1;
        if (lean_plan(ctx, w, 1, WN, &pl, 16, false)) {
            LeanArgs la{};
            la.A = static_cast<const float *>(A), la.Y = static_cast<float *>(Y);
            return lean_gemv(ctx, w, pl, la, 0, 0, NT);
        }
    }
    GemvArgs a{};
    a.A = A, a.Wq = w->Wq, a.Sc = w->Sc, a.Zb = w->Zb, a.Y = Y, a.Ypart = nullptr;
    a.M = M, a.K = (int)w->K, a.N = (int)w->N, a.n_tiles = w->n_tiles, a.n_cg = w->n_cg;
    a.a_f16 = a_dtype == HIPC_F16;
    a.nib_mask = 0x000f000fu, a.magic = 0x43004300u;
    a.a_vec = aligned(A, 16) && w->K % 8 == 0;
    const int NR = M <= 4 ? 1 : (M <= 8 ? 2 : 4);
    const int n_tiles = w->n_tiles, n_cg = w->n_cg;

    // columns per wavefront: wide outputs amortise the activation operands over more tiles
    int T = n_tiles >= 2048 ? 2 : 1;
    if (ctx->tune.gemv_t == 1 || ctx->tune.gemv_t == 2 || ctx->tune.gemv_t == 4) T = ctx->tune.gemv_t;
    if (NR == 4 && T == 4) T = 2;  // four tiles x four accumulator registers do not fit the register file
    const int groups = (int)ceil_div(n_tiles, T);
    // k partition inside a workgroup: enough wavefronts to cover the chip a few times over
    const int want_waves = ctx->tune.gemv_waves > 0 ? ctx->tune.gemv_waves : 8 * ctx->cu_count;
    const int kparts = (int)std::min<int64_t>(n_cg, std::max<int64_t>(1, ceil_div(want_waves, groups)));
    // the activation slice of a workgroup must fit the LDS budget: NT*64 + 4 bytes per row per 32-k
    // chunk; only then is k also split across workgroups (partials + a reduce launch)
    const int lds_budget = 44 * 1024;
    const int max_slice_tiles = std::max(1, lds_budget / ((NT * 64 + 4) * 4 * M));
    int ksplit = (int)ceil_div(n_cg, max_slice_tiles);
    const int slice_tiles = (int)ceil_div(n_cg, ksplit);
    ksplit = (int)ceil_div(n_cg, slice_tiles);
    const int max_waves = 16 / T / (NR == 4 ? 2 : 1);
    const int WK = std::max(1, std::min(std::min(max_waves, kparts), slice_tiles));
    const int WN = std::max(1, std::min(4 / WK, groups));
    a.WK = WK, a.WN = WN, a.slice_tiles = slice_tiles, a.ksplit = ksplit;

    const int nch = slice_tiles * 4;
    size_t lds = (size_t)nch * (4 * NT) * M * 16 + (size_t)((nch * M + 3) & ~3) * 4;
    if (WK > 1) lds += (size_t)WN * WK * T * NR * 64 * 4;
    HIPC_REQUIRE(ctx, lds <= 64 * 1024, "MatMulNBits gemv: LDS plan of %zu bytes does not fit", lds);

    if (ksplit > 1) {
        void *part = nullptr;
        int rc = scratch_get(ctx, 0, (size_t)ksplit * M * w->N * sizeof(float), &part);
        if (rc != HIPC_OK) return rc;
        a.Ypart = static_cast<float *>(part);
    }
    // persistent over the column groups once there are more workgroups than the chip holds at the
    // occupancy aimed for (16 wavefronts per CU unless overridden)
    const int waves_per_cu = ctx->tune.gemv_per_cu > 0 ? ctx->tune.gemv_per_cu : 16;
    const int resident = std::max(1, ctx->cu_count * std::max(1, waves_per_cu / (WK * WN)) / ksplit);
    const dim3 grid((unsigned)std::min<int64_t>(ceil_div(groups, WN), resident), (unsigned)ksplit);
    const dim3 block(64 * WK * WN);
    int mode = 0;
    if (pro && pro->mode != 0) {
        mode = pro->mode;
        HIPC_REQUIRE(ctx, M == 1 && a_dtype == HIPC_F32 && NT == 2 && a.a_vec, "MatMulNBits gemv: a prologue needs one aligned f32 row");
        if (mode == 2) {
            HIPC_REQUIRE(ctx, pro->x && pro->w_in && (!pro->y || pro->w_post), "MatMulNBits gemv: norm prologue operands missing");
            HIPC_REQUIRE(ctx, aligned(pro->x, 16) && aligned(pro->w_in, 16) && (!pro->y || (aligned(pro->y, 16) && aligned(pro->w_post, 16))),
                         "MatMulNBits gemv: norm prologue operands must be 16-byte aligned");
            a.nx = pro->x, a.ny = pro->y, a.nw_post = pro->w_post, a.nw_in = pro->w_in, a.nx_out = pro->x_out, a.eps = pro->eps;
            a.ny_slices = std::max(1, pro->y_slices);
            a.a_vec = 1;
        }
        if (mode == 3) {
            HIPC_REQUIRE(ctx, pro->part_o && pro->part_ml && pro->pos && pro->group > 0 && pro->head_dim > 0 &&
                                  pro->head_dim % 8 == 0 && w->K % ((int64_t)pro->group * pro->head_dim) == 0,
                         "MatMulNBits gemv: attention prologue operands missing or K not a whole number of head groups");
            HIPC_REQUIRE(ctx, aligned(pro->part_o, 16) && aligned(pro->part_ml, 8), "MatMulNBits gemv: attention partials must be 16-byte aligned");
            HIPC_REQUIRE(ctx, ksplit == 1, "MatMulNBits gemv: the attention prologue needs the whole row in one workgroup");
            a.nx = pro->part_o, a.ny = pro->part_ml, a.npos = pro->pos, a.ngroup = pro->group, a.nhd = pro->head_dim, a.nwindow = pro->window;
            const int groups4 = (int)(w->K / 4), n_q = (int)(w->K / pro->head_dim);
            a.nparts = std::max(1, std::min(4, (int)block.x / groups4));
            a.pro_off = (int)((lds + 15) & ~(size_t)15);
            lds = (size_t)a.pro_off + ((size_t)n_q * kAttnSplits + ((n_q + 3) & ~3) + (size_t)a.nparts * w->K) * 4;
            HIPC_REQUIRE(ctx, lds <= 64 * 1024, "MatMulNBits gemv: LDS plan of %zu bytes does not fit", lds);
            a.a_vec = 1;
        }
    }
    if (am && am->v && am->i && M == 1 && !a.a_f16 && ksplit == 1 && (int)grid.x <= am->capacity) {
        a.am_v = am->v, a.am_i = am->i;
        am->parts = (int)grid.x;
    }
    if (T == 4)
        launch_gemv_nt<4>(a, mode, NT, NR, w->SG, grid, block, lds, ctx->stream);
    else if (T == 2)
        launch_gemv_nt<2>(a, mode, NT, NR, w->SG, grid, block, lds, ctx->stream);
    else
        launch_gemv_nt<1>(a, mode, NT, NR, w->SG, grid, block, lds, ctx->stream);
    HIPC_LAUNCHED(ctx);
    if (ksplit > 1) {
        const long total = (long)M * w->N;
        hipLaunchKernelGGL((mmnb_ksplit_reduce_kernel), dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, ctx->stream, a.Ypart, Y, total, ksplit, a.a_f16);
        HIPC_LAUNCHED(ctx);
    }
    return HIPC_OK;
}

}  // namespace

namespace {
int packed_run(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_nbits_weight *w, void *Y, int64_t M, int accuracy_level);
int tiled_from_onnx_layout(hipc_ctx *ctx, const void *A, int a_dtype, const void *B, const void *scales, int scale_dtype, const void *zp, void *Y,
                           int64_t M, int64_t K, int64_t N, int64_t block_size, int accuracy_level, bool *taken);
}  // namespace

extern "C" {

int hipc_matmul_nbits(hipc_ctx *ctx, const void *A, int a_dtype, const void *B, size_t b_len, const void *scales,
                      int scale_dtype, size_t scales_len, const void *zp, size_t zp_len, void *Y, int64_t M, int64_t K,
                      int64_t N, int64_t block_size, int accuracy_level) {
    return entry(ctx, [&]() -> int {
        HIPC_REFUSE(ctx, a_dtype != HIPC_F32 && a_dtype != HIPC_F16, "MatMulNBits: A must be f32 or f16, got %d", a_dtype);
        // (the attribute is a lower bound on what the activations may be reduced to; the reference never reads it and
        // computes every level in f32. Level 4 allows int8 activations: two bf16 terms are more than it asks for.)
        HIPC_REFUSE(ctx, accuracy_level < 0 || accuracy_level > 4, "MatMulNBits: accuracy_level %d is not one of 0..4", accuracy_level);
        int rc = check_nbits_shape(ctx, M, K, N, block_size, b_len, scales_len, zp, zp_len, scale_dtype);
        if (rc != HIPC_OK) return rc;
        if (M == 0 || N == 0) return HIPC_OK;
        HIPC_REQUIRE(ctx, A && B && scales && Y, "MatMulNBits: null operand");
        HIPC_REQUIRE(ctx, aligned(B, 4), "MatMulNBits: packed weight must be 4-byte aligned");
        const bool af16 = a_dtype == HIPC_F16, sf16 = scale_dtype == HIPC_F16;
        // many rows: the tiled form of the weight written to scratch memory first, then the matrix-core kernels
        // (this kernel reads the whole weight once per four rows)
        bool taken = false;
        rc = tiled_from_onnx_layout(ctx, A, a_dtype, B, scales, scale_dtype, zp, Y, M, K, N, block_size, accuracy_level, &taken);
        if (taken) return rc;
        if (af16 && sf16) return launch_direct<__half, __half>(ctx, A, B, scales, zp, Y, M, K, N, block_size);
        if (af16) return launch_direct<__half, float>(ctx, A, B, scales, zp, Y, M, K, N, block_size);
        if (sf16) return launch_direct<float, __half>(ctx, A, B, scales, zp, Y, M, K, N, block_size);
        return launch_direct<float, float>(ctx, A, B, scales, zp, Y, M, K, N, block_size);
    });
}

int hipc_prepack_matmul_nbits(hipc_ctx *ctx, const void *B, size_t b_len, const void *scales, int scale_dtype,
                              size_t scales_len, const void *zp, size_t zp_len, int64_t K, int64_t N, int64_t block_size,
                              hipc_nbits_weight **out) {
    if (!out) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        return hipc::nbits_prepack(ctx, B, b_len, scales, scale_dtype, scales_len, zp, zp_len, K, N, block_size, out, 0, true);
    });
}

}  // extern "C"

namespace {

// tile counts and scale grouping of the tiled form of a weight (K, N, block_size set; block_size a power of two >= 32), and
// the bytes of its three arrays
void tiled_geometry(hipc_nbits_weight *w, size_t *wq_bytes, size_t *sc_bytes, size_t *zb_bytes) {
    const int n_chunks = (int)ceil_div(w->K, 32);
    w->n_tiles = (int)ceil_div(w->N, 16);
    w->n_cg = (int)ceil_div(n_chunks, 4);
    const int cpb = (int)(w->block_size / 32);
    w->SG = cpb >= 4 ? 1 : 4 / cpb;
    const size_t tiles = (size_t)w->n_tiles * w->n_cg;
    *wq_bytes = tiles * 1024, *sc_bytes = tiles * 16 * w->SG * 4, *zb_bytes = tiles * 16 * w->SG;
}
// the launch that writes the tiled form from the operator's tensors (device pointers)
hipError_t tiled_fill(hipc_ctx *ctx, const hipc_nbits_weight *w, const void *B, const void *scales, int scale_dtype, const void *zp) {
    const int n_blocks = (int)ceil_div(w->K, w->block_size);
    const int cpb = (int)(w->block_size / 32);
    const size_t tiles = (size_t)w->n_tiles * w->n_cg;
    const int row_words = (int)(n_blocks * w->block_size / 8);
    const int zp_row = (n_blocks + 1) / 2;
    const long threads = (long)tiles * 64;
    const dim3 grid((unsigned)ceil_div(threads, 256)), block(256);
    if (scale_dtype == HIPC_F16)
        hipLaunchKernelGGL((mmnb_prepack_kernel<__half>), grid, block, 0, ctx->stream, static_cast<const uint32_t *>(B), static_cast<const __half *>(scales), static_cast<const uint8_t *>(zp),
            w->Wq, w->Sc, w->Zb, (int)w->N, n_blocks, row_words, zp_row, (long)tiles, w->n_cg, log2i(cpb), w->SG, w->interleave_half);
    else
        hipLaunchKernelGGL((mmnb_prepack_kernel<float>), grid, block, 0, ctx->stream, static_cast<const uint32_t *>(B), static_cast<const float *>(scales), static_cast<const uint8_t *>(zp),
            w->Wq, w->Sc, w->Zb, (int)w->N, n_blocks, row_words, zp_row, (long)tiles, w->n_cg, log2i(cpb), w->SG, w->interleave_half);
    return hipGetLastError();
}

}  // namespace

// The same operations for callers inside the library that already hold the context's lock.
int hipc::nbits_prepack(hipc_ctx *ctx, const void *B, size_t b_len, const void *scales, int scale_dtype,
                        size_t scales_len, const void *zp, size_t zp_len, int64_t K, int64_t N, int64_t block_size,
                        hipc_nbits_weight **out, int interleave_half, bool any_block_size) {
    *out = nullptr;
    HIPC_REQUIRE(ctx, interleave_half == 0 || (interleave_half % 16 == 0 && 2 * (int64_t)interleave_half == N),
                 "MatMulNBits prepack: interleaved halves of %d columns do not make up N=%ld in whole tiles", interleave_half, (long)N);
    HIPC_REFUSE(ctx, ctx->capturing, "MatMulNBits prepack while a capture is open");
    int rc = check_nbits_shape(ctx, 1, K, N, block_size, b_len, scales_len, zp, zp_len, scale_dtype);
    if (rc != HIPC_OK) return rc;
    HIPC_REQUIRE(ctx, N > 0 && B && scales, "MatMulNBits prepack: empty weight");
    HIPC_REQUIRE(ctx, aligned(B, 4), "MatMulNBits: packed weight must be 4-byte aligned");
    const bool tiled = block_size >= 32 && is_pow2(block_size);
    HIPC_REFUSE(ctx, !tiled && (!any_block_size || interleave_half != 0),
                "MatMulNBits prepack: block_size %ld (below 32, or not a power of two) has no tiled form", (long)block_size);
    hipc_nbits_weight *w = new hipc_nbits_weight();
    w->K = K, w->N = N, w->block_size = block_size;
    if (!tiled) {
        // the reference's envelope is every positive multiple of 8 (interp.rs:447-464): copies of the tensors as they are
        const size_t esz = scale_dtype == HIPC_F16 ? 2 : 4;
        const size_t sizes[3] = {b_len, scales_len * esz, zp ? zp_len : 0};
        const void *from[3] = {B, scales, zp};
        void **to[3] = {&w->raw_B, &w->raw_scales, &w->raw_zp};
        hipError_t e = hipSuccess;
        for (int i = 0; i < 3 && e == hipSuccess; i++) {
            if (sizes[i] == 0) continue;
            e = hipMalloc(to[i], (sizes[i] + 3) & ~(size_t)3);
            if (e == hipSuccess) e = hipMemcpyAsync(*to[i], from[i], sizes[i], hipMemcpyDeviceToDevice, ctx->stream);
        }
        if (e == hipSuccess) e = hipGetLastError();
        if (e != hipSuccess) {
            for (int i = 0; i < 3; i++)
                if (*to[i]) (void)hipFree(*to[i]);
            delete w;
            return fail(ctx, HIPC_ERR_BACKEND, "MatMulNBits prepack: %s", hipGetErrorString(e));
        }
        w->raw_scale_dtype = scale_dtype;
        w->bytes = sizes[0] + sizes[1] + sizes[2];
        *out = w;
        return HIPC_OK;
    }
    w->interleave_half = interleave_half;
    size_t wq_bytes, sc_bytes, zb_bytes;
    tiled_geometry(w, &wq_bytes, &sc_bytes, &zb_bytes);
    if (wq_bytes >= (size_t(1) << 32)) {
        delete w;
        return fail(ctx, HIPC_ERR_UNSUPPORTED, "MatMulNBits prepack: a %zu-byte weight exceeds the 4 GiB the kernel addresses", wq_bytes);
    }
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
    e = tiled_fill(ctx, w, B, scales, scale_dtype, zp);
    if (e != hipSuccess) {
        cleanup();
        return fail(ctx, HIPC_ERR_BACKEND, "MatMulNBits prepack launch: %s", hipGetErrorString(e));
    }
    *out = w;
    return HIPC_OK;
}

void hipc::nbits_release(hipc_ctx *ctx, hipc_nbits_weight *w) {
    if (!w) return;
    // enqueued work may still read the weight: release at the next flush
    if (w->Wq) ctx->deferred.push_back(w->Wq);
    if (w->Sc) ctx->deferred.push_back(w->Sc);
    if (w->Zb) ctx->deferred.push_back(w->Zb);
    for (void *p : {w->raw_B, w->raw_scales, w->raw_zp})
        if (p) ctx->deferred.push_back(p);
    delete w;
}

int hipc::nbits_gemv(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_nbits_weight *w, void *Y, int M, int terms,
                     const GemvPrologue *pro, GemvArgmax *am) {
    return launch_gemv(ctx, A, a_dtype, w, Y, M, terms, pro, am);
}

int64_t hipc::nbits_cols(const hipc_nbits_weight *w) { return w->N; }
int64_t hipc::nbits_depth(const hipc_nbits_weight *w) { return w->K; }

extern "C" {

void hipc_nbits_weight_destroy(hipc_ctx *ctx, hipc_nbits_weight *w) {
    if (!w) return;
    entry_void(ctx, [&] {
        hipc::nbits_release(ctx, w);
    });
}

size_t hipc_nbits_weight_bytes(const hipc_nbits_weight *w) { return w ? w->bytes : 0; }

int hipc_matmul_nbits_packed(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_nbits_weight *w, void *Y, int64_t M,
                             int accuracy_level) {
    return entry(ctx, [&]() -> int { return packed_run(ctx, A, a_dtype, w, Y, M, accuracy_level); });
}

}  // extern "C"

namespace {

int packed_run(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_nbits_weight *w, void *Y, int64_t M, int accuracy_level) {
    HIPC_REQUIRE(ctx, w, "MatMulNBits: null weight");
    HIPC_REFUSE(ctx, a_dtype != HIPC_F32 && a_dtype != HIPC_F16, "MatMulNBits: A must be f32 or f16, got %d", a_dtype);
    // (the attribute is a lower bound on what the activations may be reduced to; the reference never reads it and
    // computes every level in f32. Level 4 allows int8 activations: two bf16 terms are more than it asks for.)
    HIPC_REFUSE(ctx, accuracy_level < 0 || accuracy_level > 4, "MatMulNBits: accuracy_level %d is not one of 0..4", accuracy_level);
    HIPC_REQUIRE(ctx, M >= 0 && M < (int64_t(1) << 30), "MatMulNBits: bad M=%ld", (long)M);
    if (M == 0) return HIPC_OK;
    HIPC_REQUIRE(ctx, A && Y, "MatMulNBits: null operand");
    if (!w->Wq) {   // a handle in the operator's own layout (block_size below 32 or not a power of two)
        const bool af16 = a_dtype == HIPC_F16, sf16 = w->raw_scale_dtype == HIPC_F16;
        if (af16 && sf16) return launch_direct<__half, __half>(ctx, A, w->raw_B, w->raw_scales, w->raw_zp, Y, M, w->K, w->N, w->block_size);
        if (af16) return launch_direct<__half, float>(ctx, A, w->raw_B, w->raw_scales, w->raw_zp, Y, M, w->K, w->N, w->block_size);
        if (sf16) return launch_direct<float, __half>(ctx, A, w->raw_B, w->raw_scales, w->raw_zp, Y, M, w->K, w->N, w->block_size);
        return launch_direct<float, float>(ctx, A, w->raw_B, w->raw_scales, w->raw_zp, Y, M, w->K, w->N, w->block_size);
    }
    const size_t esz = a_dtype == HIPC_F16 ? 2 : 4;
    // accuracy_level 1 pins f32 activations: all 24 bits go through the matrix cores (3 bf16
    // terms). Unset, or 2 / 3 / 4 (f16 / bf16 / int8 are enough): 2 terms. f16 activations are exact in 2.
    const int NT = (accuracy_level == 1 && a_dtype == HIPC_F32) ? 3 : 2;
    // many rows of f16: the tiled kernel reads the weight once per row tile instead of once per 16 rows
    if (a_dtype == HIPC_F16 && nbits_prefill_takes(A, w, M)) return nbits_prefill(ctx, A, w, Y, M);
    // many rows of f32: two f16 rows each (22 bits) through the same kernel; one (11 bits beside the row's own
    // power of two) where the operator's attribute allows f16, bf16 or int8 activations; three (all 24 bits) at
    // accuracy_level 1, which pins f32
    if (a_dtype == HIPC_F32 && nbits_prefill_f32_takes(A, w, M)) return nbits_prefill_f32(ctx, A, w, Y, M, NT == 3 ? 3 : accuracy_level >= 2 ? 1 : 2);
    for (int64_t m0 = 0; m0 < M; m0 += 16) {
        const int rows = (int)std::min<int64_t>(16, M - m0);
        int rc = launch_gemv(ctx, static_cast<const char *>(A) + (size_t)m0 * w->K * esz, a_dtype, w,
                             static_cast<char *>(Y) + (size_t)m0 * w->N * esz, rows, NT);
        if (rc != HIPC_OK) return rc;
    }
    return HIPC_OK;
}

// hipc_matmul_nbits with more rows than the decode kernels take, on a block size that has a tiled form: the tiled
// arrays are written into scratch memory (they live until the next call of this kind on the stream) and the product
// runs as on a prepacked handle. *taken is false where the shape stays on the kernel that reads the ONNX layout.
int tiled_from_onnx_layout(hipc_ctx *ctx, const void *A, int a_dtype, const void *B, const void *scales, int scale_dtype, const void *zp, void *Y,
                           int64_t M, int64_t K, int64_t N, int64_t block_size, int accuracy_level, bool *taken) {
    *taken = false;
    if (block_size < 32 || !is_pow2(block_size)) return HIPC_OK;
    hipc_nbits_weight w;
    w.K = K, w.N = N, w.block_size = block_size;
    size_t wq_bytes, sc_bytes, zb_bytes;
    tiled_geometry(&w, &wq_bytes, &sc_bytes, &zb_bytes);
    if (wq_bytes >= (size_t(1) << 32)) return HIPC_OK;
    // only where a tiled kernel will take the rows (otherwise sixteen rows at a time on the decode kernel: no gain)
    const bool many = a_dtype == HIPC_F16 ? nbits_prefill_takes(A, &w, M) : nbits_prefill_f32_takes(A, &w, M);
    if (!many) return HIPC_OK;
    *taken = true;
    const size_t wq_r = (wq_bytes + 255) & ~(size_t)255, sc_r = (sc_bytes + 255) & ~(size_t)255;
    void *block = nullptr;
    if (int rc = scratch_get(ctx, 4, wq_r + sc_r + zb_bytes, &block)) return rc;
    w.Wq = static_cast<uint4 *>(block);
    w.Sc = reinterpret_cast<float *>(static_cast<char *>(block) + wq_r);
    w.Zb = reinterpret_cast<uint8_t *>(block) + wq_r + sc_r;
    HIPC_TRY(ctx, tiled_fill(ctx, &w, B, scales, scale_dtype, zp));
    return packed_run(ctx, A, a_dtype, &w, Y, M, accuracy_level);
}

}  // namespace
