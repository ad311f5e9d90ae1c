// MatMulNBits for many rows of f16 activations (prefill): Y[M, N] = A[M, K] x dequant(W)[K, N].
//
// The reference has no tiled path for this shape: its kernels re-read the weight once per row
// (crates/onnx-vulkan-core/src/shaders/matmul_nbits.rs:21-25). Here the weight is read once per
// 64- or 128-row tile of A and the products run on the matrix cores. Two kernels: the one further
// down (mmnb_prefill_direct_kernel), which every shape takes by default, keeps the weight out of LDS;
// the first one passes both operands through LDS and stays behind the prefill_direct option as the
// control the other is tested against:
//
//   * a 256-thread workgroup owns a T x T tile of Y (T = 128, or 64 when that would leave CUs
//     idle), four wavefronts as 2 x 2, each T/2 x T/2 as 32x32 accumulators of
//     v_mfma_f32_32x32x16_f16 (f16 x f16 products are exact in the f32 accumulator);
//   * a k stage is 64 values: 128-byte LDS rows (pitch 144, conflict-free 128-bit reads) for
//     both operands. A goes memory -> registers -> LDS as it is. The weight comes from the
//     prepacked tiles as 32-bit words of eight nibbles and becomes f16 on the way into LDS:
//     the prepacked nibble order makes (word >> 4 i) & 0x000f000f the pair (k_2i, k_2i+1); or-ed with
//     0x6400 that is f16 1024 + q (exact), and the f16 value 1024 + zero_point is subtracted, so LDS
//     holds the exact integers q - zp;
//   * scales stay out of the f16 operands (folding them in would round every weight): the
//     accumulators of one quantisation block are multiplied by the block's scale and added to
//     the running total in f32, once per block (per 32, 64 or 128 k).
//
// Two register sets and two LDS buffers keep two stages in flight, as in the int8 kernel.
#include <hip/hip_fp16.h>

#include <algorithm>
#include <cstdlib>

#include "internal.h"

namespace hipc {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kPK = 64;          // k values per stage
constexpr int kPPitch = 144;     // bytes between LDS rows (128 of data)
constexpr size_t prefill_lds(int tile) { return 4 * (size_t)tile * kPPitch; }

struct PrefillArgs {
    const __half *A;
    const uint4 *Wq;
    const float *Sc;
    const uint8_t *Zb;
    __half *Y;
    int M, K, N;
    int n_tiles, n_cg;
    int xcd_rows, xcd_cols;
    // k split over workgroups (gridDim.y): each takes `split_stages` stages (an even number, so that
    // weight tiles are not cut) and writes f32 partials [split][M][N] that a second launch adds up
    int ksplit, split_stages;
    float *Ypart;
    float *Yf32;   // when set, the result is written here as f32 and Y is not used (rows of f32 activations, see nbits_prefill_f32)
    // Paired rows (set together; only the kernel that keeps the weight out of LDS, 128-row tiles): A holds the two
    // f16 terms of `pair_rows` f32 rows, 32 rows of high terms followed by the 32 rows of their low terms, so that a
    // wavefront's two row blocks are the two terms of the same 32 rows; it adds them and stores row r of the result
    // times 2^exps[r] -- into Yf32, or unscaled into the k split's partials [split][pair_rows][N].
    // exps without pair_rows: A holds one f16 term per f32 row and row r of the f32 result is stored times 2^exps[r]
    // (any of the kernels; the k split's partials stay unscaled).
    const int *exps;
    int pair_rows;
};

// two f16 values as one word, the first in the low half
__device__ __forceinline__ uint32_t two_halves(__half lo, __half hi) {
    return (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
}

// eight nibbles (order k0 k2 k4 k6 k1 k3 k5 k7) -> eight f16 values q - zp in k order, as four words of pairs
__device__ __forceinline__ uint4 dequant8(uint32_t w, uint32_t zb) {
    // 1024 + zp in both halves; zb carries 128 + zp
    const uint32_t zh = 0x6400u + (zb - 128u);
    const f16x2 z2 = __builtin_bit_cast(f16x2, zh | (zh << 16));
    uint32_t out[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        // nibbles i and i + 4 into the two halves, then the exponent of 1024: f16 (1024 + q), exact
        const uint32_t pair = ((w >> (4 * i)) & 0x000f000fu) | 0x64006400u;
        out[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, pair) - z2);
    }
    return make_uint4(out[0], out[1], out[2], out[3]);
}

// the wavefront's accumulators (F x F blocks of 32x32, first row i0, first column j0) to Y, to the f32 result or to
// the k split's partials. Which of the three, and whether the wavefront's square lies inside the matrix, is decided
// once (asked per element, the same questions made 3000 instructions of this and 5 of the kernel's 45 us).
template <int FM, int FN, bool CHECKED, typename OUT>
__device__ __forceinline__ void prefill_store_as(OUT *__restrict__ dst, int M, int N, const f32x16 (&total)[FM][FN], int i0, int j0, int r32, int kg,
                                                 const int *__restrict__ exps = nullptr) {   // exps (f32 results only): row r times 2^exps[r]
#pragma unroll
    for (int i = 0; i < FM; i++) {
        int e[16];
        if constexpr (sizeof(OUT) == 4) {
#pragma unroll
            for (int r = 0; r < 16; r++) e[r] = exps ? exps[min(i0 + i * 32 + kg * 4 + (r >> 2) * 8 + (r & 3), M - 1)] : 0;
        }
#pragma unroll
        for (int j = 0; j < FN; j++) {
            const int gj = j0 + j * 32 + r32;
            OUT *at = dst + (size_t)(i0 + i * 32 + kg * 4) * N + gj;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int rf = (r >> 2) * 8 + (r & 3);   // (+ kg * 4, which is in `at`)
                if (!CHECKED || (i0 + i * 32 + kg * 4 + rf < M && gj < N)) {
                    if constexpr (sizeof(OUT) == 2) at[(size_t)rf * N] = __float2half(total[i][j][r]);
                    else at[(size_t)rf * N] = exps ? ldexpf(total[i][j][r], e[r]) : total[i][j][r];
                }
            }
        }
    }
}
template <int FM, int FN>
__device__ __forceinline__ void prefill_store(const PrefillArgs &p, const f32x16 (&total)[FM][FN], int i0, int j0, int r32, int kg) {
    const bool inside = i0 + FM * 32 <= p.M && j0 + FN * 32 <= p.N;
    float *f32_to = p.ksplit > 1 ? p.Ypart + (size_t)blockIdx.y * p.M * p.N : p.Yf32;
    if (f32_to) {
        const int *exps = p.ksplit > 1 ? nullptr : p.exps;
        if (inside) prefill_store_as<FM, FN, false>(f32_to, p.M, p.N, total, i0, j0, r32, kg, exps);
        else prefill_store_as<FM, FN, true>(f32_to, p.M, p.N, total, i0, j0, r32, kg, exps);
    } else {
        if (inside) prefill_store_as<FM, FN, false>(p.Y, p.M, p.N, total, i0, j0, r32, kg);
        else prefill_store_as<FM, FN, true>(p.Y, p.M, p.N, total, i0, j0, r32, kg);
    }
}

// paired rows: one block of 32 result rows (first row i0 of the result) times 2^exps[row], or unscaled partials
template <int FN, bool CHECKED>
__device__ __forceinline__ void prefill_store_pairs_as(float *__restrict__ dst, const int *__restrict__ exps, int M, int N, const f32x16 (&total)[1][FN], int i0, int j0, int r32, int kg) {
    int e[16];
#pragma unroll
    for (int r = 0; r < 16; r++) e[r] = exps ? exps[min(i0 + kg * 4 + (r >> 2) * 8 + (r & 3), M - 1)] : 0;
#pragma unroll
    for (int j = 0; j < FN; j++) {
        const int gj = j0 + j * 32 + r32;
        float *at = dst + (size_t)(i0 + kg * 4) * N + gj;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int rf = (r >> 2) * 8 + (r & 3);
            if (!CHECKED || (i0 + kg * 4 + rf < M && gj < N)) at[(size_t)rf * N] = ldexpf(total[0][j][r], e[r]);
        }
    }
}
template <int FN>
__device__ __forceinline__ void prefill_store_pairs(const PrefillArgs &p, const f32x16 (&total)[1][FN], int i0, int j0, int r32, int kg) {
    const bool inside = i0 + 32 <= p.pair_rows && j0 + FN * 32 <= p.N;
    float *to = p.ksplit > 1 ? p.Ypart + (size_t)blockIdx.y * p.pair_rows * p.N : p.Yf32;
    const int *exps = p.ksplit > 1 ? nullptr : p.exps;
    if (inside) prefill_store_pairs_as<FN, false>(to, exps, p.pair_rows, p.N, total, i0, j0, r32, kg);
    else prefill_store_pairs_as<FN, true>(to, exps, p.pair_rows, p.N, total, i0, j0, r32, kg);
}

// FULL: K is a multiple of 128, so no stage is partial or missing and nothing needs masking.
template <int SG, int T, bool FULL>
__global__ void __launch_bounds__(256) mmnb_prefill_kernel(const PrefillArgs p) {
    constexpr int kChunks = T / 32;  // 16-byte chunks of the A slab per thread
    constexpr int kPairs = T / 64;   // (weight tile, lane) pairs per thread, two words each
    constexpr int kF = T / 64;       // 32x32 accumulators per wavefront, per direction
    constexpr int kWT = T / 2;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    uint8_t *lds_a = lds_raw;                    // [2][T * kPPitch]
    uint8_t *lds_w = lds_raw + 2 * T * kPPitch;  // [2][T * kPPitch], row = column of W

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int r32 = lane & 31, kg = lane >> 5;

    // one rectangle of the tile grid per XCD (round-robin workgroup ids), as in the int8 kernel
    const int tiles_x = (p.N + T - 1) / T, tiles_y = (p.M + T - 1) / T;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int rows_per = (tiles_y + p.xcd_rows - 1) / p.xcd_rows, cols_per = (tiles_x + p.xcd_cols - 1) / p.xcd_cols;
    const int ty = (xcd / p.xcd_cols) * rows_per + idx / cols_per, tx = (xcd % p.xcd_cols) * cols_per + idx % cols_per;
    if (idx >= rows_per * cols_per || ty >= tiles_y || tx >= tiles_x) return;
    const int i0 = ty * T, j0 = tx * T;

    // A: chunk c = tid + 256 u -> slab row c / 8, 16-byte column c % 8 (8 halves)
    uint32_t a_off[kChunks], a_lds[kChunks];
    int a_k[kChunks];
#pragma unroll
    for (int u = 0; u < kChunks; u++) {
        const int c = tid + 256 * u, row = c >> 3, kc = c & 7;
        a_off[u] = ((uint32_t)min(i0 + row, p.M - 1) * (uint32_t)p.K + kc * 8) * 2;  // rows past M: clamped, never stored
        a_lds[u] = row * kPPitch + kc * 16;
        a_k[u] = kc * 8;
    }
    // W: pair q = tid + 256 u -> weight tile q / 64 of this column range, lane q % 64 of that tile
    uint32_t w_tile[kPairs], w_lds[kPairs], w_sz[kPairs];
#pragma unroll
    for (int u = 0; u < kPairs; u++) {
        const int q = tid + 256 * u, t = q >> 6, l = q & 63;
        const int nt = min(j0 / 16 + t, p.n_tiles - 1);  // tiles past N: clamped, never stored
        w_tile[u] = (uint32_t)nt * (uint32_t)p.n_cg;
        w_lds[u] = (t * 16 + (l & 15)) * kPPitch + (l >> 4) * 16;
        w_sz[u] = (l & 15);
    }
    struct Regs {
        uint4 a[kChunks];
        uint2 w[kPairs];
        uint32_t z[kPairs];  // two (128 + zp) bytes: for word 0 and word 1 of the stage
    };
    const char *a_base = reinterpret_cast<const char *>(p.A);
    auto load_regs = [&](Regs &r, int stage) {
        const int k0 = stage * kPK;
#pragma unroll
        for (int u = 0; u < kChunks; u++) {
            // K is a multiple of 8: a chunk is inside or outside as a whole; one outside is read from the row's last
            // chunk instead (the load is issued whatever the mask says, and past the last row lies the end of A)
            const bool in = FULL || k0 + a_k[u] < p.K;
            const int back = FULL ? 0 : max(0, k0 + a_k[u] - (p.K - 8));
            const uint4 v = HIPC_LOAD_ALWAYS(reinterpret_cast<const uint4 *>(a_base + a_off[u] + ((size_t)k0 - back) * 2));
            r.a[u] = make_uint4(in ? v.x : 0u, in ? v.y : 0u, in ? v.z : 0u, in ? v.w : 0u);
        }
        const int cg = stage >> 1, half = stage & 1;
#pragma unroll
        for (int u = 0; u < kPairs; u++) {
            const uint32_t tile = w_tile[u] + cg;
            const int l = (tid + 256 * u) & 63;
            r.w[u] = *reinterpret_cast<const uint2 *>(reinterpret_cast<const char *>(p.Wq + (size_t)tile * 64 + l) + half * 8);
            const uint8_t *zb = p.Zb + ((size_t)tile * 16 + w_sz[u]) * SG;
            // the scale group of word j (0..3) of a tile: j for SG 4, j / 2 for SG 2, 0 for SG 1
            if (SG == 4) {
                r.z[u] = *reinterpret_cast<const uint16_t *>(zb + half * 2);  // groups 2 half and 2 half + 1
            } else {
                const uint32_t z = zb[SG == 2 ? half : 0];
                r.z[u] = z | (z << 8);
            }
        }
    };
    // a stage past the end reads clamped addresses and stores zeros for A: it adds nothing
    auto store_regs = [&](const Regs &r, int buf, bool live) {
        const uint32_t keep = FULL || live ? 0xffffffffu : 0u;
#pragma unroll
        for (int u = 0; u < kChunks; u++)
            *reinterpret_cast<uint4 *>(lds_a + buf * T * kPPitch + a_lds[u]) =
                make_uint4(r.a[u].x & keep, r.a[u].y & keep, r.a[u].z & keep, r.a[u].w & keep);
#pragma unroll
        for (int u = 0; u < kPairs; u++) {
            uint8_t *dst = lds_w + buf * T * kPPitch + w_lds[u];
            *reinterpret_cast<uint4 *>(dst) = dequant8(r.w[u].x, r.z[u] & 0xffu);        // k = 8 (l >> 4) .. + 8
            *reinterpret_cast<uint4 *>(dst + 64) = dequant8(r.w[u].y, r.z[u] >> 8);     // k + 32
        }
    };

    f32x16 total[kF][kF], raw[kF][kF];
#pragma unroll
    for (int i = 0; i < kF; i++)
#pragma unroll
        for (int j = 0; j < kF; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) total[i][j][r] = 0.f, raw[i][j][r] = 0.f;

    // scales of the lane's columns (one per accumulator column block)
    uint32_t sc_at[kF];
#pragma unroll
    for (int j = 0; j < kF; j++) {
        const int col = wn * kWT + j * 32 + r32;
        const int nt = min((j0 + col) / 16, p.n_tiles - 1);
        sc_at[j] = ((uint32_t)nt * (uint32_t)p.n_cg * 16 + (col & 15)) * SG;
    }
    auto scale_of = [&](int j, int cg, int g) { return p.Sc[sc_at[j] + (uint32_t)cg * 16 * SG + g]; };
    auto fold = [&](const float (&s)[kF]) {
#pragma unroll
        for (int i = 0; i < kF; i++)
#pragma unroll
            for (int j = 0; j < kF; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) total[i][j][r] = fmaf(raw[i][j][r], s[j], total[i][j][r]);
    };

    // One stage = four k steps of 16. `half` is the stage's parity inside its 128-k weight tile;
    // scale groups end after every second step (SG 4), every stage (SG 2) or every odd stage (SG 1).
    // The scales of a stage are requested before the operand loads of the stage after next, so
    // that waiting for them (loads retire in order) never waits for those.
    float s0[kF], s1[kF];
    auto fetch_scales = [&](int stage, int half) {
        const int cg = stage >> 1;
#pragma unroll
        for (int j = 0; j < kF; j++) {
            if (SG == 4) s0[j] = scale_of(j, cg, half * 2), s1[j] = scale_of(j, cg, half * 2 + 1);
            else if (SG == 2) s1[j] = scale_of(j, cg, half);
            else if (half == 1) s1[j] = scale_of(j, cg, 0);
        }
    };
    // the first product of a quantisation block starts from zero instead of from a cleared register
    f32x16 zero;
#pragma unroll
    for (int r = 0; r < 16; r++) zero[r] = 0.f;
    auto compute = [&](int buf, int half) {
        auto opens_block = [&](int step) { return SG == 4 ? (step & 1) == 0 : SG == 2 ? step == 0 : step == 0 && half == 0; };
        const uint8_t *ba = lds_a + buf * T * kPPitch + (wm * kWT + r32) * kPPitch + kg * 16;
        const uint8_t *bw = lds_w + buf * T * kPPitch + (wn * kWT + r32) * kPPitch + kg * 16;
#pragma unroll
        for (int step = 0; step < 4; step++) {
            f16x8 af[kF], wf[kF];
#pragma unroll
            for (int i = 0; i < kF; i++) af[i] = *reinterpret_cast<const f16x8 *>(ba + i * 32 * kPPitch + step * 32);
#pragma unroll
            for (int j = 0; j < kF; j++) wf[j] = *reinterpret_cast<const f16x8 *>(bw + j * 32 * kPPitch + step * 32);
#pragma unroll
            for (int i = 0; i < kF; i++)
#pragma unroll
                for (int j = 0; j < kF; j++)
                    raw[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], wf[j], opens_block(step) ? zero : raw[i][j], 0, 0, 0);
            if (SG == 4 && step == 1) fold(s0);
            if (step == 3 && (SG != 1 || half == 1)) fold(s1);
        }
    };

    const int nk_all = (p.K + kPK - 1) / kPK;
    const int ks0 = blockIdx.y * p.split_stages, nk = min(nk_all, ks0 + p.split_stages);  // this workgroup's stages
    Regs r0, r1;
    load_regs(r0, ks0);
    load_regs(r1, min(ks0 + 1, nk - 1));
    store_regs(r0, 0, true);
    __syncthreads();
    // two stages per trip and no exit in between, so the memory counters stay exact; with an odd
    // stage count the second half of the last trip multiplies a stage whose A is all zeros
    for (int ks = ks0; ks < nk; ks += 2) {
        fetch_scales(ks, 0);
        load_regs(r0, min(ks + 2, nk - 1));
        compute(0, 0);
        store_regs(r1, 1, ks + 1 < nk);
        __syncthreads();
        fetch_scales(min(ks + 1, nk - 1), 1);
        load_regs(r1, min(ks + 3, nk - 1));
        compute(1, 1);
        store_regs(r0, 0, true);
        __syncthreads();
    }

    prefill_store<kF, kF>(p, total, i0 + wm * kWT, j0 + wn * kWT, r32, kg);
}

// ---- the weight never enters LDS --------------------------------------------------------------------------------
// The B operand of v_mfma_f32_32x32x16_f16 is eight k values of one column per lane, and a 32-bit word of the
// prepacked weight is eight k values of one column: tile lane (c, q) of a 128-k weight tile holds, in its word j,
// k = 32 j + 8 q + 0..7 of column c. The wavefront that multiplies a 32-column block reads the words itself (lane
// (r32, kg) takes tile lanes q = 2 kg and 2 kg + 1 of its column: two 16-byte loads per 128 k), turns a word into
// the operand in registers (nine instructions) and uses it for every 32-row block it owns. A k step (j, h) then
// covers k = 32 j + 16 kg + 8 h + 0..7 -- an order of its own, which only has to be the same for both operands: A
// is read from LDS at that offset. LDS carries A alone (half the traffic and half the writes of the kernel above,
// and no conversion ahead of a barrier).

// 1024 + zp and 64 + zp as f16 in both halves of a word (zb carries 128 + zp)
struct ZeroPair {
    f16x2 unit, sixteenth;
};
__device__ __forceinline__ ZeroPair zero_pair(uint32_t zb) {
    const uint32_t zp = zb - 128u, a = 0x6400u + zp, b = 0x5400u + (zp << 4);
    return {__builtin_bit_cast(f16x2, a | (a << 16)), __builtin_bit_cast(f16x2, b | (b << 16))};
}
// eight nibbles (k0 k2 k4 k6 in the low half, k1 k3 k5 k7 in the high half) -> the f16 values q - zp in k order.
// Nibbles 0 and 2 of each half sit where the low mantissa bits are: or-ed with the exponent of 1024 that is
// 1024 + q. Nibbles 1 and 3 sit four bits higher: 1024 + 16 q, and one fused multiply-add by 1/16 makes q - zp
// of it ((1024 + 16 q) / 16 = 64 + q is exact). One shift instead of three.
// (x & mask) | 0x64006400 as one instruction: v_and_or_b32 can take one scalar operand only, so the compiler, which
// keeps both constants in scalar registers, emits two; the exponent pattern is handed over in a vector register
__device__ __forceinline__ uint32_t and_or_1024(uint32_t x, uint32_t mask, uint32_t ones) {
#ifdef HIPC_HOST_MODEL
    return (x & mask) | ones;
#else
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(ones));
    return r;
#endif
}
__device__ __forceinline__ f16x8 dequant_operand(uint32_t w, const ZeroPair &z, uint32_t ones) {
    const f16x2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
    const uint32_t w8 = w >> 8;
    const f16x2 p0 = __builtin_bit_cast(f16x2, and_or_1024(w, 0x000f000fu, ones)) - z.unit;
    const f16x2 p1 = __builtin_bit_cast(f16x2, and_or_1024(w, 0x00f000f0u, ones)) * sixteenth - z.sixteenth;
    const f16x2 p2 = __builtin_bit_cast(f16x2, and_or_1024(w8, 0x000f000fu, ones)) - z.unit;
    const f16x2 p3 = __builtin_bit_cast(f16x2, and_or_1024(w8, 0x00f000f0u, ones)) * sixteenth - z.sixteenth;
    return f16x8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}
__device__ __forceinline__ uint32_t word_of(const uint4 &v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }

// NJ: 32-column blocks per wavefront. 2: a 128x128 tile. 3: a 128x192 tile -- a third less LDS traffic per product,
// and a matrix of 512 x 11008 becomes 232 workgroups for 256 CUs where 128x128 tiles make 344, two of them on every
// third CU.
// MI: 32-row blocks per wavefront. 2 with the tiles above; 1 with NJ 1 is a 64x64 tile for matrices that have too few
// of the large ones (four wavefronts of 32x32: a conversion per product, but many short wavefronts per SIMD).
// KG: groups of four wavefronts per workgroup. With 2 (512 threads) each group takes half of the workgroup's k range
// with LDS buffers of its own, and the two sets of accumulators are added through LDS at the end (128-row tiles: each
// group hands over the 32-row blocks the other one stores; 64-row tiles: the second hands everything to the first).
// For launches that leave wavefront slots of the SIMDs empty: a second wavefront issues while the first waits for
// LDS, a barrier or the matrix core.
template <int SG, int MI, int NJ, int KG, bool FULL>
__global__ void __launch_bounds__(256 * KG, KG > 1 ? 1 : MI * NJ == 1 ? 4 : MI * NJ <= 4 ? 2 : 1) mmnb_prefill_direct_kernel(const PrefillArgs p) {
    static_assert(KG == 1 || KG == 2, "one or two groups");
    constexpr int T = 64 * MI, TN = 64 * NJ, kChunks = T / 32, kF = MI, kWT = 32 * MI, kWN = 32 * NJ;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    const int grp = KG > 1 ? (int)(threadIdx.x >> 8) : 0;
    uint8_t *lds_a = lds_raw + grp * 2 * T * kPPitch;  // [KG][2][T * kPPitch]

    const int tid = threadIdx.x & 255;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int r32 = lane & 31, kg = lane >> 5;

    const int tiles_x = (p.N + TN - 1) / TN, tiles_y = (p.M + T - 1) / T;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int rows_per = (tiles_y + p.xcd_rows - 1) / p.xcd_rows, cols_per = (tiles_x + p.xcd_cols - 1) / p.xcd_cols;
    const int ty = (xcd / p.xcd_cols) * rows_per + idx / cols_per, tx = (xcd % p.xcd_cols) * cols_per + idx % cols_per;
    if (idx >= rows_per * cols_per || ty >= tiles_y || tx >= tiles_x) return;
    const int i0 = ty * T, j0 = tx * TN;

    // A: chunk c = tid + 256 u -> slab row c / 8, 16-byte column c % 8 (8 halves)
    uint32_t a_off[kChunks], a_lds[kChunks];
    int a_k[kChunks];
#pragma unroll
    for (int u = 0; u < kChunks; u++) {
        const int c = tid + 256 * u, row = c >> 3, kc = c & 7;
        a_off[u] = ((uint32_t)min(i0 + row, p.M - 1) * (uint32_t)p.K + kc * 8) * 2;  // rows past M: clamped, never stored
        a_lds[u] = row * kPPitch + kc * 16;
        a_k[u] = kc * 8;
    }
    struct ARegs {
        uint4 a[kChunks];
    };
    const char *a_base = reinterpret_cast<const char *>(p.A);
    auto load_a = [&](ARegs &r, int stage) {
        const int k0 = stage * kPK;
#pragma unroll
        for (int u = 0; u < kChunks; u++) {
            // K is a multiple of 8: a chunk is inside or outside as a whole; one outside is read from the row's last
            // chunk instead (the load is issued whatever the mask says, and past the last row lies the end of A)
            const bool in = FULL || k0 + a_k[u] < p.K;
            const uint32_t back = FULL ? 0u : (uint32_t)max(0, k0 + a_k[u] - (p.K - 8)) * 2u;
            const uint4 v = HIPC_LOAD_ALWAYS(reinterpret_cast<const uint4 *>((a_base + (size_t)k0 * 2) + (a_off[u] - back)));   // (uniform part first: a scalar base and a 32-bit lane offset)
            r.a[u] = make_uint4(in ? v.x : 0u, in ? v.y : 0u, in ? v.z : 0u, in ? v.w : 0u);
        }
    };
    // a stage past the end reads clamped addresses and stores zeros for A: it adds nothing
    auto store_a = [&](const ARegs &r, int buf, bool live) {   // (`live` is the same for the whole workgroup group: a branch, no masks)
        if ((FULL && KG == 1) || live) {
#pragma unroll
            for (int u = 0; u < kChunks; u++) *reinterpret_cast<uint4 *>(lds_a + buf * T * kPPitch + a_lds[u]) = r.a[u];
        } else {
#pragma unroll
            for (int u = 0; u < kChunks; u++) *reinterpret_cast<uint4 *>(lds_a + buf * T * kPPitch + a_lds[u]) = make_uint4(0u, 0u, 0u, 0u);
        }
    };

    // B: column block j of the wavefront = 32 columns = two weight tiles; the lane's column is r32 of the block
    uint32_t b_at[NJ], sc_at[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int nt = min(j0 / 16 + wn * (2 * NJ) + j * 2 + (r32 >> 4), p.n_tiles - 1);  // tiles past N: clamped, never stored
        b_at[j] = (uint32_t)nt * (uint32_t)p.n_cg * 64 + (r32 & 15) + 32 * kg;
        sc_at[j] = ((uint32_t)nt * (uint32_t)p.n_cg * 16 + (r32 & 15)) * SG;
    }
    struct BRegs {
        uint4 w[NJ][2];
        float s[NJ][SG];
        uint32_t z[NJ];  // SG bytes of 128 + zp
    };
    auto load_b = [&](BRegs &b, int cg) {
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const uint4 *src = (p.Wq + (size_t)cg * 64) + b_at[j];
            b.w[j][0] = src[0];
            b.w[j][1] = src[16];
            const float *sc = (p.Sc + (size_t)cg * 16 * SG) + sc_at[j];
            const uint8_t *zb = (p.Zb + (size_t)cg * 16 * SG) + sc_at[j];
            if (SG == 4) {
                const float4 v = *reinterpret_cast<const float4 *>(sc);
                b.s[j][0] = v.x, b.s[j][1 % SG] = v.y, b.s[j][2 % SG] = v.z, b.s[j][3 % SG] = v.w;
                b.z[j] = *reinterpret_cast<const uint32_t *>(zb);
            } else if (SG == 2) {
                const float2 v = *reinterpret_cast<const float2 *>(sc);
                b.s[j][0] = v.x, b.s[j][1 % SG] = v.y;
                b.z[j] = *reinterpret_cast<const uint16_t *>(zb);
            } else {
                b.s[j][0] = sc[0];
                b.z[j] = zb[0];
            }
        }
    };

    // One set of accumulators, kept in units of the scale of the quantisation block that is open: when the next
    // block opens they are multiplied by (scale of the old block) / (scale of the new one), the products of the new
    // block add to them as they are, and the store multiplies by the last scale. That is one multiplication per
    // accumulator and block, like adding scale x (block sum) to a running total, without the second set of
    // registers for the block sum (which is what lets a wavefront own three 32-column blocks). A scale of magnitude
    // below 2^-64 (a block of zeros carries 0) counts as 2^-64: the quotient stays finite, and what such a block
    // adds, at most 2^-64 x 15 x sum |a|, is far below one unit of the last place of any result that has a block
    // with a real scale; a column without one is stored as 0.
    f32x16 acc[kF][NJ];
#pragma unroll
    for (int i = 0; i < kF; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
    float unit[NJ];   // the scale the accumulators of column block j are in
    bool scaled[NJ];  // the lane's column of block j has met a scale of 2^-64 or more
#pragma unroll
    for (int j = 0; j < NJ; j++) unit[j] = 1.f, scaled[j] = false;
    // the scales of a weight tile's groups -> the factors that take the accumulators from each group to the next
    // (worked out when the trip begins, next to the loads, not in front of the products that wait for them)
    auto scales_to_ratios = [&](BRegs &b) {
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int g = 0; g < SG; g++) {
                const bool real = !(fabsf(b.s[j][g]) < 0x1p-64f);
                const float s = real ? b.s[j][g] : 0x1p-64f;
                scaled[j] |= real;
                b.s[j][g] = unit[j] * __builtin_amdgcn_rcpf(s);   // (1 ulp: a relative error of 1e-7 in what was added so far)
                unit[j] = s;
            }
    };
    auto reopen = [&](int j, float ratio) {
#pragma unroll
        for (int i = 0; i < kF; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] *= ratio;
    };

    uint32_t ones = 0x64006400u;   // kept in a vector register (see and_or_1024)
#ifndef HIPC_HOST_MODEL
    asm volatile("" : "+v"(ones));
#endif
    // One stage = 64 k = the k steps (j, h) with j = 2 half + 0 / 1 of the weight tile the stage lies in;
    // a scale group opens at every second step (SG 4), every stage (SG 2) or every even stage (SG 1).
    // the zero points of a stage as f16 pairs (with one scale group per weight tile: of the whole tile, made once per trip)
    struct ZeroPairs {
        ZeroPair at[NJ][SG == 4 ? 2 : 1];
    };
    auto zero_pairs = [&](const BRegs &b, int half) {
        ZeroPairs zp;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            if (SG == 4) {
                zp.at[j][0] = zero_pair((b.z[j] >> (16 * half)) & 0xffu);
                zp.at[j][SG == 4 ? 1 : 0] = zero_pair((b.z[j] >> (16 * half + 8)) & 0xffu);
            } else {
                zp.at[j][0] = zero_pair(SG == 2 ? (b.z[j] >> (8 * half)) & 0xffu : b.z[j]);
            }
        }
        return zp;
    };
    auto compute = [&](const BRegs &b, const ZeroPairs &zp, int buf, int half) {   // (b.s holds ratios by now)
        const uint8_t *ba = lds_a + buf * T * kPPitch + (wm * kWT + r32) * kPPitch + kg * 32;
#pragma unroll
        for (int step = 0; step < 4; step++) {
            const int word = half * 2 + (step >> 1), h = step & 1;
            const bool opens = SG == 4 ? h == 0 : SG == 2 ? step == 0 : step == 0 && half == 0;
            f16x8 af[kF], wf[NJ];
            if (opens) {
                const int g = SG == 4 ? word : SG == 2 ? half : 0;
#pragma unroll
                for (int j = 0; j < NJ; j++) reopen(j, b.s[j][g % SG]);
            }
#pragma unroll
            for (int i = 0; i < kF; i++) af[i] = *reinterpret_cast<const f16x8 *>(ba + i * 32 * kPPitch + (step >> 1) * 64 + h * 16);
#pragma unroll
            for (int j = 0; j < NJ; j++) wf[j] = dequant_operand(word_of(b.w[j][h], word), zp.at[j][SG == 4 ? step >> 1 : 0], ones);
#pragma unroll
            for (int i = 0; i < kF; i++)
#pragma unroll
                for (int j = 0; j < NJ; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], wf[j], acc[i][j], 0, 0, 0);
        }
    };

    const int nk_all = (p.K + kPK - 1) / kPK;
    const int wg_ks0 = blockIdx.y * p.split_stages, wg_nk = min(nk_all, wg_ks0 + p.split_stages);  // this workgroup's stages (wg_ks0 is even)
    // ... and this group's: with two groups the first takes the larger half of the trips; both run as many trips as
    // the first (the barriers are the workgroup's), the second's last one, if it has one less, on zeros
    const int wg_trips = (wg_nk - wg_ks0 + 1) >> 1, my_trips = (wg_trips + KG - 1) / KG;
    const int ks0 = wg_ks0 + grp * 2 * my_trips, nk = KG == 1 ? wg_nk : min(wg_nk, ks0 + 2 * my_trips);
    const int last = min(wg_nk - 1, max(nk - 1, wg_ks0));   // the last stage whose addresses this group may form
    const int cg_last = last >> 1;
    ARegs r0, r1;
    BRegs bc, bn;
    load_b(bc, min(ks0, last) >> 1);
    load_a(r0, min(ks0, last));
    load_a(r1, min(ks0 + 1, last));
    store_a(r0, 0, ks0 < nk);
    __syncthreads();
    // two stages = one weight tile per trip; with an odd stage count the second half of the last trip multiplies
    // a stage whose A is all zeros. (The fences keep the order written here: left alone, the compiler moves the
    // stores -- and with them the wait for the loads they store -- ahead of the products and the next loads behind
    // them, and every half trip then waits out a whole trip to memory.)
    auto trip = [&](BRegs &bcur, BRegs &bnext, int ks) {
        load_b(bnext, min((ks >> 1) + 1, cg_last));
        load_a(r0, min(ks + 2, last));
        scales_to_ratios(bcur);
        ZeroPairs zp = zero_pairs(bcur, 0);
        __builtin_amdgcn_sched_barrier(0);
        compute(bcur, zp, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        store_a(r1, 1, ks + 1 < nk);
        __syncthreads();
        load_a(r1, min(ks + 3, last));
        if (SG != 1) zp = zero_pairs(bcur, 1);
        __builtin_amdgcn_sched_barrier(0);
        compute(bcur, zp, 1, 1);
        __builtin_amdgcn_sched_barrier(0);
        store_a(r0, 0, ks + 2 < nk);
        __syncthreads();
    };
    for (int t = 0; t < my_trips; t += 2) {   // the two register sets of the weight take turns
        trip(bc, bn, ks0 + 2 * t);
        if (t + 1 < my_trips) trip(bn, bc, ks0 + 2 * t + 2);
    }
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
        for (int i = 0; i < kF; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] *= scaled[j] ? unit[j] : 0.f;
    if constexpr (MI == 2) {
        if (p.pair_rows > 0) {
            // paired rows: the wavefront's two row blocks are the two terms of the same 32 rows. Every group adds its
            // own two, the second hands its sums to the first ([16-byte piece][thread] in LDS, as below), which adds
            // them and stores.
            f32x16 pair[1][NJ];
#pragma unroll
            for (int j = 0; j < NJ; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) pair[0][j][r] = acc[0][j][r] + acc[1][j][r];
            if constexpr (KG == 2) {
                float4 *slot = reinterpret_cast<float4 *>(lds_raw);
                if (grp > 0) {
#pragma unroll
                    for (int j = 0; j < NJ; j++)
#pragma unroll
                        for (int q = 0; q < 4; q++)
                            slot[(j * 4 + q) * 256 + tid] = make_float4(pair[0][j][4 * q], pair[0][j][4 * q + 1], pair[0][j][4 * q + 2], pair[0][j][4 * q + 3]);
                }
                __syncthreads();
                if (grp > 0) return;
#pragma unroll
                for (int j = 0; j < NJ; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const float4 o = slot[(j * 4 + q) * 256 + tid];
                        pair[0][j][4 * q] += o.x, pair[0][j][4 * q + 1] += o.y, pair[0][j][4 * q + 2] += o.z, pair[0][j][4 * q + 3] += o.w;
                    }
            }
            prefill_store_pairs<NJ>(p, pair, (i0 + wm * kWT) >> 1, j0 + wn * kWN, r32, kg);
            return;
        }
    }
    if constexpr (KG > 1 && MI == 1) {
        // the later groups hand their accumulators to the first: [group - 1][16-byte piece][thread] in LDS (the A
        // buffers are done with: the last barrier of the loop is behind every read of them), added in group order
        float4 *slot = reinterpret_cast<float4 *>(lds_raw);
        if (grp > 0) {
#pragma unroll
            for (int j = 0; j < NJ; j++)
#pragma unroll
                for (int q = 0; q < 4; q++)
                    slot[((grp - 1) * NJ * 4 + j * 4 + q) * 256 + tid] = make_float4(acc[0][j][4 * q], acc[0][j][4 * q + 1], acc[0][j][4 * q + 2], acc[0][j][4 * q + 3]);
        }
        __syncthreads();
        if (grp > 0) return;
#pragma unroll
        for (int g = 1; g < KG; g++)
#pragma unroll
            for (int j = 0; j < NJ; j++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float4 o = slot[((g - 1) * NJ * 4 + j * 4 + q) * 256 + tid];
                    acc[0][j][4 * q] += o.x, acc[0][j][4 * q + 1] += o.y, acc[0][j][4 * q + 2] += o.z, acc[0][j][4 * q + 3] += o.w;
                }
        prefill_store<kF, NJ>(p, acc, i0 + wm * kWT, j0 + wn * kWN, r32, kg);
    } else if constexpr (KG == 2) {
        // group g keeps row block g and hands the other one over: [group][16-byte piece][thread] in LDS (the A
        // buffers are done with: the last barrier of the loop is behind every read of them)
        float4 *mine = reinterpret_cast<float4 *>(lds_raw) + grp * (NJ * 4 * 256), *theirs = reinterpret_cast<float4 *>(lds_raw) + (grp ^ 1) * (NJ * 4 * 256);
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const f32x16 &v = grp == 0 ? acc[1][j] : acc[0][j];
                mine[(j * 4 + q) * 256 + tid] = make_float4(v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
            }
        __syncthreads();
        f32x16 sum[1][NJ];
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4 o = theirs[(j * 4 + q) * 256 + tid];
                const f32x16 &v = grp == 0 ? acc[0][j] : acc[1][j];
                // (first group's share + second group's share, whichever of them adds)
                sum[0][j][4 * q] = grp == 0 ? v[4 * q] + o.x : o.x + v[4 * q];
                sum[0][j][4 * q + 1] = grp == 0 ? v[4 * q + 1] + o.y : o.y + v[4 * q + 1];
                sum[0][j][4 * q + 2] = grp == 0 ? v[4 * q + 2] + o.z : o.z + v[4 * q + 2];
                sum[0][j][4 * q + 3] = grp == 0 ? v[4 * q + 3] + o.w : o.w + v[4 * q + 3];
            }
        prefill_store<1, NJ>(p, sum, i0 + wm * kWT + grp * 32, j0 + wn * kWN, r32, kg);
    } else {
        prefill_store<kF, NJ>(p, acc, i0 + wm * kWT, j0 + wn * kWN, r32, kg);
    }
}

// Y = f16(sum over splits of the f32 partials), in split order; or the f32 sum itself into Yf32. Four results per
// thread; VEC: the element count is a multiple of four and the rows are aligned for 16-byte loads and one 8- or
// 16-byte store. (static: this file is compiled twice)
template <bool VEC>
static __global__ void __launch_bounds__(256)
mmnb_prefill_reduce_kernel(const float *__restrict__ part, __half *__restrict__ Y, float *__restrict__ Yf32, long total, int ksplit,
                           const int *__restrict__ exps, int N) {   // exps: the f32 result's row r times 2^exps[r] (paired rows; VEC then has N a multiple of four)
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= total) return;
    if (VEC) {
        float4 v = *reinterpret_cast<const float4 *>(part + i);
        for (int s = 1; s < ksplit; s++) {
            const float4 u = *reinterpret_cast<const float4 *>(part + (size_t)s * total + i);
            v.x += u.x, v.y += u.y, v.z += u.z, v.w += u.w;
        }
        if (exps) {
            const int e = exps[i / N];
            v = make_float4(ldexpf(v.x, e), ldexpf(v.y, e), ldexpf(v.z, e), ldexpf(v.w, e));
        }
        if (Yf32) {
            *reinterpret_cast<float4 *>(Yf32 + i) = v;
        } else {
            *reinterpret_cast<uint2 *>(Y + i) = make_uint2(two_halves(__float2half(v.x), __float2half(v.y)), two_halves(__float2half(v.z), __float2half(v.w)));
        }
        return;
    }
    for (long j = i; j < min(i + 4, total); j++) {
        float v = part[j];
        for (int s = 1; s < ksplit; s++) v += part[(size_t)s * total + j];
        if (exps) v = ldexpf(v, exps[j / N]);
        if (Yf32) Yf32[j] = v;
        else Y[j] = __float2half(v);
    }
}

namespace {

// The tile grid cut into one rectangle per XCD, the k split (prefill_split option: 0 never splits k, n > 0 forces n
// ways; unset: chosen by shape) with its partials in scratch memory; returns the launch grid in *grid.
int prefill_plan(hipc_ctx *ctx, PrefillArgs &a, int TM, int TN, bool may_split, dim3 *grid) {
    const int tiles_x = (int)ceil_div(a.N, TN), tiles_y = (int)ceil_div(a.M, TM);
    int best = 8, best_cost = 1 << 30;
    for (int r = 1; r <= 8; r *= 2) {
        const int cost = (int)(ceil_div(tiles_y, r) + ceil_div(tiles_x, 8 / r));
        if (cost < best_cost) best_cost = cost, best = r;
    }
    a.xcd_rows = best, a.xcd_cols = 8 / best;
    const unsigned gx = 8u * (unsigned)(ceil_div(tiles_y, a.xcd_rows) * ceil_div(tiles_x, a.xcd_cols));
    // Too few tiles for the chip: split k over workgroups, as many ways as gives every CU a
    // workgroup, at least 32 stages each (with fewer, the second launch and the partials cost more
    // than the idle CUs: 512 x 2048 x 2560 took 27 us split three ways, 21 us on 64x64 tiles). The
    // partials go through scratch memory.
    const int nk = (int)ceil_div(a.K, kPK);
    int ksplit = 1;
    const int g_prefill_split = ctx->tune.prefill_split;
    if (may_split && g_prefill_split != 0) {
        const int tiles = tiles_x * tiles_y;
        ksplit = g_prefill_split > 0 ? g_prefill_split : std::min(4, ctx->cu_count / std::max(1, tiles));
        ksplit = std::max(1, std::min(ksplit, g_prefill_split > 0 ? nk / 2 : nk / 32));
    }
    a.split_stages = (int)(ceil_div(ceil_div(nk, ksplit), 2) * 2);
    a.ksplit = (int)ceil_div(nk, a.split_stages);
    a.Ypart = nullptr;
    if (a.ksplit > 1) {
        void *part = nullptr;
        if (int rc = scratch_get(ctx, 0, (size_t)a.ksplit * a.M * a.N * sizeof(float), &part)) return rc;
        a.Ypart = static_cast<float *>(part);
    }
    *grid = dim3(gx, (unsigned)a.ksplit);
    return HIPC_OK;
}
// the second launch of a k split
int prefill_join_splits(hipc_ctx *ctx, const PrefillArgs &a) {
    if (a.ksplit > 1) {
        const long total = (long)(a.pair_rows > 0 ? a.pair_rows : a.M) * a.N;
        const bool vec = (a.exps ? a.N % 4 == 0 : total % 4 == 0) && (a.Yf32 ? aligned(a.Yf32, 16) : aligned(a.Y, 8));
        if (vec)
            hipLaunchKernelGGL((mmnb_prefill_reduce_kernel<true>), dim3((unsigned)ceil_div(total, 1024)), dim3(256), 0, ctx->stream, a.Ypart, a.Y, a.Yf32, total, a.ksplit, a.exps, a.N);
        else
            hipLaunchKernelGGL((mmnb_prefill_reduce_kernel<false>), dim3((unsigned)ceil_div(total, 1024)), dim3(256), 0, ctx->stream, a.Ypart, a.Y, a.Yf32, total, a.ksplit, a.exps, a.N);
        HIPC_LAUNCHED(ctx);
    }
    return HIPC_OK;
}

// both operands through LDS
template <int SG, int T>
int prefill_launch_tile(hipc_ctx *ctx, PrefillArgs a) {
    const bool full = a.K % (2 * kPK) == 0;
    static bool lds_allowed[2][kMaxDevices] = {};
    if (int rc = full ? allow_dynamic_lds(ctx, mmnb_prefill_kernel<SG, T, true>, prefill_lds(T), lds_allowed[1])
                      : allow_dynamic_lds(ctx, mmnb_prefill_kernel<SG, T, false>, prefill_lds(T), lds_allowed[0]))
        return rc;
    dim3 grid;
    if (int rc = prefill_plan(ctx, a, T, T, T == 128, &grid)) return rc;
    if (full)
        hipLaunchKernelGGL((mmnb_prefill_kernel<SG, T, true>), grid, dim3(256), prefill_lds(T), ctx->stream, a);
    else
        hipLaunchKernelGGL((mmnb_prefill_kernel<SG, T, false>), grid, dim3(256), prefill_lds(T), ctx->stream, a);
    HIPC_LAUNCHED(ctx);
    return prefill_join_splits(ctx, a);
}

// the weight from memory into the operand registers; A alone in LDS
template <int SG, int MI, int NJ, int KG>
int prefill_launch_direct_groups(hipc_ctx *ctx, const PrefillArgs &a, dim3 grid) {
    const bool full = a.K % (2 * kPK) == 0;
    // one group: at most 36 KB, inside the limit that needs no permission; two: their A buffers, then the hand-over
    constexpr size_t lds = KG == 1 ? prefill_lds(64 * MI) / 2 : std::max(KG * prefill_lds(64 * MI) / 2, (size_t)(MI == 2 ? 2 : KG - 1) * NJ * 4 * 256 * 16);
    if (KG > 1 && lds > 64 * 1024) {
        static bool lds_allowed[2][kMaxDevices] = {};
        if (int rc = full ? allow_dynamic_lds(ctx, mmnb_prefill_direct_kernel<SG, MI, NJ, KG, true>, lds, lds_allowed[1])
                          : allow_dynamic_lds(ctx, mmnb_prefill_direct_kernel<SG, MI, NJ, KG, false>, lds, lds_allowed[0]))
            return rc;
    }
    if (full)
        hipLaunchKernelGGL((mmnb_prefill_direct_kernel<SG, MI, NJ, KG, true>), grid, dim3(256 * KG), lds, ctx->stream, a);
    else
        hipLaunchKernelGGL((mmnb_prefill_direct_kernel<SG, MI, NJ, KG, false>), grid, dim3(256 * KG), lds, ctx->stream, a);
    HIPC_LAUNCHED(ctx);
    return HIPC_OK;
}
template <int SG, int MI, int NJ>
int prefill_launch_direct(hipc_ctx *ctx, PrefillArgs a) {
    dim3 grid;
    if (int rc = prefill_plan(ctx, a, 64 * MI, 64 * NJ, MI == 2, &grid)) return rc;
    if constexpr (MI == 2) {
        // Two k groups per workgroup when the launch leaves the second wavefront slot of the SIMDs empty (no more
        // workgroups than CUs) and every group gets two trips or more; prefill_groups 1 / 2 forces the choice.
        const int trips = (a.split_stages + 1) / 2, forced = ctx->tune.prefill_groups;
        const long wgs = (long)ceil_div(a.M, 64 * MI) * ceil_div(a.N, 64 * NJ) * a.ksplit;
        // (three column blocks and two groups leave no register for more than one scale per weight tile)
        const bool two = (NJ == 2 || SG == 1) && (forced == 1 ? false : forced == 2 ? true : wgs <= ctx->cu_count && trips >= 4);
        if constexpr (NJ == 2 || SG == 1) if (two) {
            if (int rc = prefill_launch_direct_groups<SG, MI, NJ, 2>(ctx, a, grid)) return rc;
            return prefill_join_splits(ctx, a);
        }
    }
    if constexpr (MI == 1) {
        // 64-row tiles: two groups when the launch has too few wavefronts to hide one another's waits (no more than
        // two workgroups per CU) and each group keeps two trips (512 x 2048 x 2560: 15.9 against 16.9 us; four
        // groups, 18.3 us, cost more in prologues than they hide)
        const int trips = (a.split_stages + 1) / 2, forced = ctx->tune.prefill_groups;
        const long wgs = (long)ceil_div(a.M, 64) * ceil_div(a.N, 64 * NJ) * a.ksplit;
        if (forced == 1 ? false : forced == 2 ? true : wgs <= 2 * ctx->cu_count && trips >= 4) {
            if (int rc = prefill_launch_direct_groups<SG, MI, NJ, 2>(ctx, a, grid)) return rc;
            return prefill_join_splits(ctx, a);
        }
    }
    if (int rc = prefill_launch_direct_groups<SG, MI, NJ, 1>(ctx, a, grid)) return rc;
    return prefill_join_splits(ctx, a);
}

}  // namespace

// This file is compiled twice. The 128x128 instances live in an object of their own, built with
// HIPC_PREFILL_WIDE and with the matrix-core accumulators in ordinary vector registers (the block
// scales then multiply them without copies out of the accumulation file: 48.5 -> 44.7 us for
// 512 x 2048 x 11008); the 64x64 instances are faster with the accumulation file (80.6 against
// 87.9 us for 512 x 11008 x 2048), and that is a switch of the whole compilation.
int prefill_launch_wide(hipc_ctx *ctx, const PrefillArgs &a, int SG, int tile);

#ifdef HIPC_PREFILL_WIDE

int prefill_launch_wide(hipc_ctx *ctx, const PrefillArgs &a, int SG, int tile) {
    if (tile == 192) switch (SG) {
            case 4: return prefill_launch_direct<4, 2, 3>(ctx, a);
            case 2: return prefill_launch_direct<2, 2, 3>(ctx, a);
            default: return prefill_launch_direct<1, 2, 3>(ctx, a);
        }
    if (tile == 64) switch (SG) {
            case 4: return prefill_launch_direct<4, 1, 1>(ctx, a);
            case 2: return prefill_launch_direct<2, 1, 1>(ctx, a);
            default: return prefill_launch_direct<1, 1, 1>(ctx, a);
        }
    if (ctx->tune.prefill_direct != 0) switch (SG) {
            case 4: return prefill_launch_direct<4, 2, 2>(ctx, a);
            case 2: return prefill_launch_direct<2, 2, 2>(ctx, a);
            default: return prefill_launch_direct<1, 2, 2>(ctx, a);
        }
    switch (SG) {
        case 4: return prefill_launch_tile<4, 128>(ctx, a);
        case 2: return prefill_launch_tile<2, 128>(ctx, a);
        default: return prefill_launch_tile<1, 128>(ctx, a);
    }
}

#else

namespace {

template <int SG>
int prefill_launch(hipc_ctx *ctx, const PrefillArgs &a) {
    const int forced = ctx->tune.prefill_tile, g_prefill_split = ctx->tune.prefill_split;
    // 128-row tiles when they give every CU a workgroup, directly or (long k) with k split over up
    // to four workgroups per tile; else 64x64
    const int64_t rows128 = ceil_div(a.M, 128), tiles128 = rows128 * ceil_div(a.N, 128), tiles192 = rows128 * ceil_div(a.N, 192);
    const int nk = (int)ceil_div(a.K, kPK);
    const bool by_split = g_prefill_split != 0 && tiles128 * std::min<int64_t>(4, nk / 32) >= 192;
    int tile = tiles128 >= 256 || by_split ? 128 : 64;
    // 128x192 where that shortens the longest queue of a SIMD: rounds of workgroups over the CUs times the wavefront's
    // 32-column blocks (512 x 11008: 344 tiles of 128x128 are two rounds of 2, 232 of 128x192 one round of 3)
    const int64_t cus = std::max(1, ctx->cu_count);
    if (tile == 128 && tiles128 >= 256 && ctx->tune.prefill_direct != 0 && ceil_div(tiles192, cus) * 3 < ceil_div(tiles128, cus) * 2) tile = 192;
    if (forced == 64 || forced == 128 || (forced == 192 && ctx->tune.prefill_direct != 0)) tile = forced;
    if (a.pair_rows > 0 && tile == 64) tile = 128;   // paired rows are the two row blocks of a wavefront: 128-row tiles
    return tile == 64 && ctx->tune.prefill_direct == 0 ? prefill_launch_tile<SG, 64>(ctx, a) : prefill_launch_wide(ctx, a, SG, tile);
}

}  // namespace

bool nbits_prefill_takes(const void *A, const hipc_nbits_weight *w, int64_t M) {
    return M > 16 && w->K % 8 == 0 && aligned(A, 16) && M * w->K < (int64_t(1) << 31);
}

int nbits_prefill(hipc_ctx *ctx, const void *A, const hipc_nbits_weight *w, void *Y, int64_t M) {
    HIPC_REFUSE(ctx, !nbits_prefill_takes(A, w, M), "MatMulNBits prefill: shape or alignment not taken by the tiled kernel");
    PrefillArgs a{};
    a.A = static_cast<const __half *>(A), a.Wq = w->Wq, a.Sc = w->Sc, a.Zb = w->Zb, a.Y = static_cast<__half *>(Y);
    a.M = (int)M, a.K = (int)w->K, a.N = (int)w->N, a.n_tiles = w->n_tiles, a.n_cg = w->n_cg;
    switch (w->SG) {
        case 4: return prefill_launch<4>(ctx, a);
        case 2: return prefill_launch<2>(ctx, a);
        default: return prefill_launch<1>(ctx, a);
    }
}

// Rows of f32 activations for the f16 matrix cores: row m becomes two f16 rows, hi = f16(a 2^-e) and
// lo = f16(a 2^-e - hi) (22 significant bits), with 2^e the row's own power of two that brings its
// largest magnitude into [2^14, 2^15) -- exact, and no value of the row leaves the f16 range. The rows
// are stored as A2[m] = hi, A2[M + m] = lo; one workgroup per row. PAIRED: 32 rows of high terms are followed by the
// 32 rows of their low terms (row m: hi at 64 (m / 32) + m % 32, lo 32 rows on), the grid covers a multiple of 32
// rows and the rows past M are zeros.
template <bool PAIRED, int TERMS = 2>   // TERMS 1: the high terms alone, M rows; 3: a third term (all 24 bits of the row's values), rows 2 M + m
static __global__ void __launch_bounds__(256)
mmnb_prefill_split_rows_kernel(const float *__restrict__ A, int M, int K, __half *__restrict__ A2, int *__restrict__ exps) {
    __shared__ float red[4];
    const int m = blockIdx.x, tid = threadIdx.x;
    const size_t hi_at = PAIRED ? (size_t)(64 * (m >> 5) + (m & 31)) : (size_t)m, lo_at = PAIRED ? hi_at + 32 : (size_t)M + m;
    if (PAIRED && m >= M) {
        uint4 *hi_row = reinterpret_cast<uint4 *>(A2 + hi_at * K), *lo_row = reinterpret_cast<uint4 *>(A2 + lo_at * K);
        for (int c = tid; c < K / 8; c += 256) hi_row[c] = make_uint4(0u, 0u, 0u, 0u), lo_row[c] = make_uint4(0u, 0u, 0u, 0u);
        return;
    }
    const float4 *row = reinterpret_cast<const float4 *>(A + (size_t)m * K);   // (K is a multiple of 8 and A is aligned: see nbits_prefill_f32_takes)
    const int nv = K / 4;
    constexpr int kHeld = 4;   // 16-byte pieces a thread keeps between the two passes: rows up to 4096 values are read once
    float4 held[kHeld];
    float mx = 0.f;
#pragma unroll
    for (int u = 0; u < kHeld; u++) {
        const int c = tid + 256 * u;
        held[u] = c < nv ? row[c] : make_float4(0.f, 0.f, 0.f, 0.f);
        mx = fmaxf(mx, fmaxf(fmaxf(fabsf(held[u].x), fabsf(held[u].y)), fmaxf(fabsf(held[u].z), fabsf(held[u].w))));   // (a NaN does not raise the maximum: it passes through below)
    }
    for (int c = tid + 256 * kHeld; c < nv; c += 256) {
        const float4 v = row[c];
        mx = fmaxf(mx, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    // bits of mx: exponent field - 127 = floor(log2 mx) for a normal number; zero, subnormal or infinite rows are not scaled
    const int ef = (int)((__float_as_uint(mx) >> 23) & 0xffu);
    const int e = (ef == 0 || ef == 255) ? 0 : ef - 127 - 14;
    if (tid == 0) exps[m] = e;
    const float down = __uint_as_float((uint32_t)(127 - e) << 23);   // 2^-e: e is in [-140, 113], 2^-e a normal number
    uint2 *hi_row = reinterpret_cast<uint2 *>(A2 + hi_at * K), *lo_row = reinterpret_cast<uint2 *>(A2 + lo_at * K);
    auto split4 = [&](const float4 &v, int c) {
        const float a[4] = {v.x * down, v.y * down, v.z * down, v.w * down};
        __half hi[4], lo[4], lo2[4];
#pragma unroll
        for (int t = 0; t < 4; t++) {
            hi[t] = __float2half(a[t]);
            const float r = a[t] - __half2float(hi[t]);   // (exact, like the next one)
            lo[t] = __float2half(r);
            lo2[t] = __float2half(r - __half2float(lo[t]));
        }
        hi_row[c] = make_uint2(two_halves(hi[0], hi[1]), two_halves(hi[2], hi[3]));
        if (TERMS >= 2) lo_row[c] = make_uint2(two_halves(lo[0], lo[1]), two_halves(lo[2], lo[3]));
        if (TERMS == 3) lo_row[c + (size_t)M * (K / 4)] = make_uint2(two_halves(lo2[0], lo2[1]), two_halves(lo2[2], lo2[3]));
    };
#pragma unroll
    for (int u = 0; u < kHeld; u++)
        if (tid + 256 * u < nv) split4(held[u], tid + 256 * u);
    for (int c = tid + 256 * kHeld; c < nv; c += 256) split4(row[c], c);
}
// Y[m] = (P[m] + P[M + m]) 2^e[m], or with three terms (P[m] + (P[M + m] + P[2 M + m])) 2^e[m]: the small ones first
template <bool VEC>   // VEC: N is a multiple of four and Y is aligned for 16-byte stores
static __global__ void __launch_bounds__(256)
mmnb_prefill_join_rows_kernel(const float *__restrict__ P, const int *__restrict__ exps, int M, int N, float *__restrict__ Y, int terms) {
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * (VEC ? 4 : 1), plane = (long)M * N;
    if (i >= plane) return;
    const int e = exps[(int)(i / N)];
    if (VEC) {
        const float4 a = *reinterpret_cast<const float4 *>(P + i);
        float4 b = *reinterpret_cast<const float4 *>(P + i + plane);
        if (terms == 3) {
            const float4 c = *reinterpret_cast<const float4 *>(P + i + 2 * plane);
            b = make_float4(b.x + c.x, b.y + c.y, b.z + c.z, b.w + c.w);
        }
        *reinterpret_cast<float4 *>(Y + i) = make_float4(ldexpf(a.x + b.x, e), ldexpf(a.y + b.y, e), ldexpf(a.z + b.z, e), ldexpf(a.w + b.w, e));
    } else {
        const float b = terms == 3 ? P[i + plane] + P[i + 2 * plane] : P[i + plane];
        Y[i] = ldexpf(P[i] + b, e);
    }
}

// Many rows of f32 activations: each row as two f16 rows (22 bits) through the same tiled kernel. Twice the products
// of the f16 case, against one pass over the whole weight per 16 rows on the decode kernel. With the kernel that
// keeps the weight out of LDS the two terms of a row are the two row blocks of one wavefront, which adds them and
// puts the rows' powers of two back itself; the kernel that stages both operands through LDS writes 2 M rows of f32
// results and a last launch adds the pairs.
bool nbits_prefill_f32_takes(const void *A, const hipc_nbits_weight *w, int64_t M) {
    return M > 32 && w->K % 8 == 0 && aligned(A, 16) && (3 * M + 64) * w->K < (int64_t(1) << 31) && 3 * M * w->N < (int64_t(1) << 31);
}

int nbits_prefill_f32(hipc_ctx *ctx, const void *A, const hipc_nbits_weight *w, void *Y, int64_t M, int terms) {
    HIPC_REFUSE(ctx, !nbits_prefill_f32_takes(A, w, M), "MatMulNBits prefill: shape or alignment not taken by the tiled kernel");
    if (terms == 1) {
        // one f16 term per row (11 bits beside the row's own power of two): M rows through the kernel, which scales
        // the rows of its f32 result back itself (after a k split, the reduce launch does)
        const size_t e_bytes = ((size_t)M * sizeof(int) + 255) & ~(size_t)255;
        void *split = nullptr;
        if (int rc = scratch_get(ctx, 2, (size_t)M * w->K * sizeof(__half) + e_bytes, &split)) return rc;
        __half *A1 = reinterpret_cast<__half *>(static_cast<char *>(split) + e_bytes);
        int *exps = static_cast<int *>(split);
        hipLaunchKernelGGL((mmnb_prefill_split_rows_kernel<false, 1>), dim3((unsigned)M), dim3(256), 0, ctx->stream, static_cast<const float *>(A), (int)M, (int)w->K, A1, exps);
        HIPC_LAUNCHED(ctx);
        PrefillArgs a{};
        a.A = A1, a.Wq = w->Wq, a.Sc = w->Sc, a.Zb = w->Zb, a.Y = nullptr, a.Yf32 = static_cast<float *>(Y), a.exps = exps;
        a.M = (int)M, a.K = (int)w->K, a.N = (int)w->N, a.n_tiles = w->n_tiles, a.n_cg = w->n_cg;
        switch (w->SG) {
            case 4: return prefill_launch<4>(ctx, a);
            case 2: return prefill_launch<2>(ctx, a);
            default: return prefill_launch<1>(ctx, a);
        }
    }
    // two terms: the pairs of the kernel that keeps the weight out of LDS; three (f32 pinned: all 24 bits), or the
    // kernel with both operands in LDS: `terms` M rows, and a launch that adds them
    const bool paired = terms == 2 && ctx->tune.prefill_direct != 0;
    const int64_t rows2 = paired ? 64 * ceil_div(M, 32) : terms * M;
    const size_t a2_bytes = (size_t)rows2 * w->K * sizeof(__half), e_bytes = ((size_t)M * sizeof(int) + 255) & ~(size_t)255;
    void *split = nullptr, *sums = nullptr;
    if (int rc = scratch_get(ctx, 2, a2_bytes + e_bytes, &split)) return rc;
    if (!paired)
        if (int rc = scratch_get(ctx, 3, (size_t)terms * M * w->N * sizeof(float), &sums)) return rc;
    __half *A2 = reinterpret_cast<__half *>(static_cast<char *>(split) + e_bytes);
    int *exps = static_cast<int *>(split);
    if (paired)
        hipLaunchKernelGGL((mmnb_prefill_split_rows_kernel<true, 2>), dim3((unsigned)(rows2 / 2)), dim3(256), 0, ctx->stream, static_cast<const float *>(A), (int)M, (int)w->K, A2, exps);
    else if (terms == 3)
        hipLaunchKernelGGL((mmnb_prefill_split_rows_kernel<false, 3>), dim3((unsigned)M), dim3(256), 0, ctx->stream, static_cast<const float *>(A), (int)M, (int)w->K, A2, exps);
    else
        hipLaunchKernelGGL((mmnb_prefill_split_rows_kernel<false, 2>), dim3((unsigned)M), dim3(256), 0, ctx->stream, static_cast<const float *>(A), (int)M, (int)w->K, A2, exps);
    HIPC_LAUNCHED(ctx);
    PrefillArgs a{};
    a.A = A2, a.Wq = w->Wq, a.Sc = w->Sc, a.Zb = w->Zb, a.Y = nullptr, a.Yf32 = static_cast<float *>(paired ? Y : sums);
    a.M = (int)rows2, a.K = (int)w->K, a.N = (int)w->N, a.n_tiles = w->n_tiles, a.n_cg = w->n_cg;
    if (paired) a.exps = exps, a.pair_rows = (int)M;
    int rc;
    switch (w->SG) {
        case 4: rc = prefill_launch<4>(ctx, a); break;
        case 2: rc = prefill_launch<2>(ctx, a); break;
        default: rc = prefill_launch<1>(ctx, a); break;
    }
    if (rc != HIPC_OK || paired) return rc;
    const long total = (long)M * w->N;
    if (w->N % 4 == 0 && aligned(Y, 16))
        hipLaunchKernelGGL((mmnb_prefill_join_rows_kernel<true>), dim3((unsigned)ceil_div(total, 1024)), dim3(256), 0, ctx->stream, static_cast<const float *>(sums), exps, (int)M, (int)w->N, static_cast<float *>(Y), terms);
    else
        hipLaunchKernelGGL((mmnb_prefill_join_rows_kernel<false>), dim3((unsigned)ceil_div(total, 256)), dim3(256), 0, ctx->stream, static_cast<const float *>(sums), exps, (int)M, (int)w->N, static_cast<float *>(Y), terms);
    HIPC_LAUNCHED(ctx);
    return HIPC_OK;
}

#endif  // HIPC_PREFILL_WIDE

}  // namespace hipc
