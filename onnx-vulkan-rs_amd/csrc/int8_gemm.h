// The int8 MFMA contraction shared by MatMulInteger / QLinearMatMul and
// ConvInteger / QLinearConv:
//
//     C[i][j] = sum_k P[i][k] * Q[j][k]          (both operands k-contiguous, signed bytes)
//
// One 256-thread workgroup owns a 128x128 tile of C; its four wavefronts own
// 64x64 each as 2x2 v_mfma_i32_32x32x32_i8 accumulators (this file's LDS-staged kernel; the
// kernels for products with hundreds of tiles keep the constant operand out of LDS: int8_gemm_bdirect.h). Each k stage moves a
// 128x128-byte slab of P and of Q through LDS with 128-bit accesses (row pitch
// 144 bytes, conflict-free for ds_read_b128); two further stages are on their
// way from memory while one is multiplied.
//
// gfx950's int8 MFMA is signed x signed, so uint8 operands are shifted by 128
// (x ^ 0x80), their zero points with them -- the identity the reference uses
// the other way round (crates/onnx-vulkan-core/src/shaders/matmul_integer.rs:11-24) --
// and the zero points leave in the epilogue
// (shaders/glsl/matmul_integer_coop.comp:22-31):
//     sum (p-zp)(q-zq) = sum p*q - zq*sum_k p - zp*sum_k q + K*zp*zq
// The constant operand's sums come from prepacking; the dynamic operand's are
// taken from its MFMA operand registers with v_dot4 only when the other zero
// point is not 0.
#pragma once

#include <cstddef>
#include <cstdlib>

#include "internal.h"

namespace hipc {

typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

constexpr int kBM = 128, kBN = 128, kBK = 128, kPitch = kBK + 16;
constexpr size_t gemm_lds(int tile) { return 4 * (size_t)tile * kPitch + 4 * (tile / 2) * sizeof(int); }

enum { EPI_I32 = 0, EPI_SCALE_BIAS = 1, EPI_REQUANT = 2 };
enum { MODE_MM = 0, MODE_CONV = 1 };

struct GemmArgs {
    // P operand: MODE_MM  -> the activation matrix A [I, K] (u8 / i8, pitch K)
    //            MODE_CONV -> prepacked weight, I_pad x K_pad signed bytes, fragment-major (qfrag_offset)
    const uint8_t *P;
    // Q operand: MODE_MM  -> prepacked B, J_pad x K_pad signed bytes, fragment-major (qfrag_offset)
    //            MODE_CONV -> NHWC activations, already signed
    const uint8_t *Q;
    const int32_t *const_sum;  // sums over k of the prepacked operand (per j in MM, per i in CONV)
    const uint8_t *dyn_zp;     // device zero point of the dynamic operand (may be null)
    const uint8_t *const_zp;   // device zero point of the prepacked operand (may be null)
    int dyn_shift, const_shift;    // 128 when that operand is uint8, else 0
    int dyn_signed, const_signed;  // how to read the zero-point byte
    int host_zp;                   // zero points given by value instead of by pointer
    int dyn_zp_value, const_zp_value;
    int I, J, K, K_pad;
    int p_aligned;  // MODE_MM: rows of A can be read with 128-bit loads
    int xcd_rows, xcd_cols;  // the 8 XCDs as a grid over the tiles (set by gemm_grid)

    // conv geometry (MODE_CONV); Q is [n][H][W][C]
    int C, H, W, Ho, Wo, kh, kw, sh, sw, dh, dw, pt, pl;
    int slab_pos;  // int8_conv_row_kernel: input positions held per tile

    // epilogue
    void *Y;
    const float *scale, *product, *bias;   // EPI_SCALE_BIAS (per j)
    int scale_step, product_step, bias_step, relu;
    uint32_t *range;
    const float *ratio;                    // EPI_REQUANT: per j in MM, per i in CONV
    int ratio_step;
    const int32_t *qbias;                  // EPI_REQUANT int32 bias (per i in CONV)
    int y_zp, out_signed;
};

// Chooses how the 8 XCDs tile the grid of output tiles (fewest operand slabs per XCD) and
// returns the number of workgroups to launch.
inline unsigned gemm_grid(GemmArgs &g, int tile = kBM) {
    const int tiles_x = (g.J + tile - 1) / tile, tiles_y = (g.I + tile - 1) / tile;
    int best_a = 8, best_cost = 1 << 30;
    for (int a = 1; a <= 8; a *= 2) {
        const int b = 8 / a;
        const int cost = (tiles_y + a - 1) / a + (tiles_x + b - 1) / b;
        if (cost < best_cost) best_cost = cost, best_a = a;
    }
    g.xcd_rows = best_a, g.xcd_cols = 8 / best_a;
    const int rows_per = (tiles_y + g.xcd_rows - 1) / g.xcd_rows, cols_per = (tiles_x + g.xcd_cols - 1) / g.xcd_cols;
    return 8u * (unsigned)(rows_per * cols_per);
}

// Where byte (n, k) of the prepacked constant operand of a matrix product lives. The operand is kept
// fragment-major: a fragment is 32 columns n x 32 bytes of k, stored as the matrix core takes it --
// lane (n % 32, h = (k / 16) % 2) holds 16 bytes, lanes in order, 1 KB per fragment -- and the
// fragments of 32 columns follow each other along k. A kernel that stages the operand through LDS
// still reads whole 128-byte lines (eight consecutive columns of one k half), and a kernel that
// feeds the matrix cores straight from memory reads a fragment with one fully coalesced load.
__host__ __device__ __forceinline__ uint32_t qfrag_offset(int n, int k, int K_pad) {
    return ((uint32_t)(n >> 5) * (uint32_t)(K_pad >> 5) + (uint32_t)(k >> 5)) * 1024u +
           ((uint32_t)(((k >> 4) & 1) << 5) + (uint32_t)(n & 31)) * 16u + (uint32_t)(k & 15);
}

__device__ __forceinline__ int zp_byte(const uint8_t *ptr, int is_signed) {
    if (!ptr) return 0;
    const uint8_t v = *ptr;
    return is_signed ? (int)(int8_t)v : (int)v;
}

__device__ __forceinline__ uint4 xor4(uint4 v, uint32_t m) { return make_uint4(v.x ^ m, v.y ^ m, v.z ^ m, v.w ^ m); }

__device__ __forceinline__ int dot_ones(uint4 v) {
    int s = __builtin_amdgcn_sdot4((int)v.x, 0x01010101, 0, false);
    s = __builtin_amdgcn_sdot4((int)v.y, 0x01010101, s, false);
    s = __builtin_amdgcn_sdot4((int)v.z, 0x01010101, s, false);
    return __builtin_amdgcn_sdot4((int)v.w, 0x01010101, s, false);
}

// One finished accumulator (zero points already taken out) on its way to memory: the raw
// int32, the rescaled float (MatMulInteger followed by Mul/Add/Relu, feeding the running
// min/max of the next DynamicQuantizeLinear) or the requantized byte.
template <int MODE, int EPI>
__device__ __forceinline__ void gemm_emit(const GemmArgs &p, int img, int gi, int gj, int v, float &fmn, float &fmx) {
    const size_t at = MODE == MODE_MM ? (size_t)gi * p.J + gj : ((size_t)img * p.I + gi) * p.J + gj;
    // the int32 / float outputs are written once and are several times the operands: non-temporal
    // stores keep them from displacing the operand tiles other workgroups are about to read
    // (1000 x 1024 x 4096: 16.5 -> 14.9 us, 8192^3: 605 -> 585 us)
    if (EPI == EPI_I32) {
        __builtin_nontemporal_store(v, static_cast<int32_t *>(p.Y) + at);
    } else if (EPI == EPI_SCALE_BIAS) {
        float s = p.scale[(size_t)gj * p.scale_step];
        if (p.product) s = __fmul_rn(s, p.product[(size_t)gj * p.product_step]);
        float o = __fmul_rn((float)v, s);
        // the product and the sum round separately, as the unfused Cast, Mul, Add do; the _rn
        // functions are plain operators to the compiler, which may otherwise fuse them
        asm volatile("" : "+v"(o));
        if (p.bias) o = __fadd_rn(o, p.bias[(size_t)gj * p.bias_step]);
        if (p.relu) o = o > 0.f ? o : 0.f;
        __builtin_nontemporal_store(o, static_cast<float *>(p.Y) + at);
        fmn = fminf(fmn, o);
        fmx = fmaxf(fmx, o);
    } else {
        const int c = MODE == MODE_MM ? gj : gi;
        if (p.qbias) v += p.qbias[c];
        const float t = __fmul_rn((float)v, p.ratio[(size_t)c * p.ratio_step]);
        int q = (int)rintf(t) + p.y_zp;
        if (p.out_signed) {
            q = min(max(q, -128), 127);
            static_cast<int8_t *>(p.Y)[at] = (int8_t)q;
        } else {
            q = min(max(q, 0), 255);
            static_cast<uint8_t *>(p.Y)[at] = (uint8_t)q;
        }
    }
}

// The same for a kernel all of whose outputs in a lane share the column: what the column
// contributes is loaded once, ahead of time, and the stores then wait for nothing.
struct EmitColumn {
    float s = 0.f, b = 0.f;  // scale (times product) or requantisation ratio; float bias
    int qb = 0;              // requantisation's int32 bias
};
template <int EPI>
__device__ __forceinline__ EmitColumn gemm_emit_column(const GemmArgs &p, int gj) {
    EmitColumn e;
    if (EPI == EPI_SCALE_BIAS) {
        e.s = p.scale[(size_t)gj * p.scale_step];
        if (p.product) e.s = __fmul_rn(e.s, p.product[(size_t)gj * p.product_step]);
        if (p.bias) e.b = p.bias[(size_t)gj * p.bias_step];
    } else if (EPI == EPI_REQUANT) {
        e.s = p.ratio[(size_t)gj * p.ratio_step];
        if (p.qbias) e.qb = p.qbias[gj];
    }
    return e;
}
template <int EPI>
__device__ __forceinline__ void gemm_emit_mm(const GemmArgs &p, const EmitColumn &e, int gi, int gj, int v, float &fmn, float &fmx) {
    const size_t at = (size_t)gi * p.J + gj;
    if (EPI == EPI_I32) {
        __builtin_nontemporal_store(v, static_cast<int32_t *>(p.Y) + at);
    } else if (EPI == EPI_SCALE_BIAS) {
        float o = __fmul_rn((float)v, e.s);
        asm volatile("" : "+v"(o));  // two roundings, as in gemm_emit
        if (p.bias) o = __fadd_rn(o, e.b);
        if (p.relu) o = o > 0.f ? o : 0.f;
        __builtin_nontemporal_store(o, static_cast<float *>(p.Y) + at);
        fmn = fminf(fmn, o);
        fmx = fmaxf(fmx, o);
    } else {
        const float t = __fmul_rn((float)(v + e.qb), e.s);
        int q = (int)rintf(t) + p.y_zp;
        if (p.out_signed) {
            q = min(max(q, -128), 127);
            static_cast<int8_t *>(p.Y)[at] = (int8_t)q;
        } else {
            q = min(max(q, 0), 255);
            static_cast<uint8_t *>(p.Y)[at] = (uint8_t)q;
        }
    }
}

// folds a wavefront's min/max of the floats it emitted into the range slot
__device__ __forceinline__ void gemm_emit_range(const GemmArgs &p, int lane, float fmn, float fmx) {
    if (!p.range) return;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        fmn = fminf(fmn, __shfl_xor(fmn, off, 64));
        fmx = fmaxf(fmx, __shfl_xor(fmx, off, 64));
    }
    if (lane == 0) {
        atomicMax(&p.range[0], __float_as_uint(-fmn) & 0x7fffffffu);
        atomicMax(&p.range[1], __float_as_uint(fmx) & 0x7fffffffu);
    }
}

// One k stage of both operand slabs as a thread holds it between global memory and LDS.
template <int N>
struct GemmRegs {
    uint4 p[N], q[N];
};

// ALIGNED (MODE_MM only): rows of A start on 16 bytes and K % 128 == 0, so A is read with
// unconditional 128-bit loads at base + 32-bit offset (no branch, which keeps the load counters
// exact and two stages in flight; no per-stage address arithmetic).
// T is the tile edge: 128, or 64 when 128x128 tiles would leave most CUs idle or alone with one
// workgroup (several small workgroups per CU then overlap each other's memory and LDS latency).
template <int MODE, int EPI, bool ALIGNED, int T>
__global__ void __launch_bounds__(256) int8_gemm_kernel(const GemmArgs p) {
    constexpr int kChunks = T / 32;  // 16-byte chunks of a slab per thread
    constexpr int kF = T / 64;       // 32x32 accumulators per wavefront, per direction
    constexpr int kWT = T / 2;       // edge of a wavefront's part of the tile
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    uint8_t *lds_p = lds_raw;                       // [2][T * kPitch]
    uint8_t *lds_q = lds_raw + 2 * T * kPitch;      // [2][T * kPitch]
    int *lds_sum = reinterpret_cast<int *>(lds_raw + 4 * T * kPitch);  // [4][kWT]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int r32 = lane & 31, kg = lane >> 5;
    const int img = blockIdx.z;

    // Tile order: consecutive workgroup ids land on different XCDs (round robin), each with
    // its own L2. The tile grid is cut into xcd_rows x xcd_cols = 8 rectangles, one per XCD, so
    // the operand slabs an XCD pulls through its L2 are as few as the shape allows.
    const int tiles_x = (p.J + T - 1) / T, tiles_y = (p.I + T - 1) / T;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int rows_per = (tiles_y + p.xcd_rows - 1) / p.xcd_rows, cols_per = (tiles_x + p.xcd_cols - 1) / p.xcd_cols;
    const int ty = (xcd / p.xcd_cols) * rows_per + idx / cols_per, tx = (xcd % p.xcd_cols) * cols_per + idx % cols_per;
    if (idx >= rows_per * cols_per || ty >= tiles_y || tx >= tiles_x) return;
    const int i0 = ty * T, j0 = tx * T;

    // zero points in the shifted (signed) domain
    const int zd = (p.host_zp ? p.dyn_zp_value : zp_byte(p.dyn_zp, p.dyn_signed)) - p.dyn_shift;
    const int zc = (p.host_zp ? p.const_zp_value : zp_byte(p.const_zp, p.const_signed)) - p.const_shift;
    const bool need_dyn_sum = zc != 0;
    const uint32_t flip = p.dyn_shift ? 0x80808080u : 0u;
    const uint32_t pad_word = (uint32_t)(zd & 0xff) * 0x01010101u;

    // the four 16-byte chunks of each operand slab this thread moves: slab row and k chunk (of 8)
    int row_[kChunks], kc_[kChunks];
    // the fragment-major constant operand of a matrix product is read with consecutive lanes on
    // consecutive columns (16 bytes apart in memory), its k chunk changing with the chunk index
    int qrow_[kChunks], qkc_[kChunks];
#pragma unroll
    for (int u = 0; u < kChunks; u++) {
        const int c = tid + 256 * u;
        row_[u] = c >> 3;
        kc_[u] = c & 7;
        qrow_[u] = MODE == MODE_MM ? c % T : row_[u];
        qkc_[u] = MODE == MODE_MM ? c / T : kc_[u];
    }
    // (a convolution's constant operand is P, the prepacked weight, and it is read the same way)
    int prow_[kChunks], pkc_[kChunks];
#pragma unroll
    for (int u = 0; u < kChunks; u++) {
        const int c = tid + 256 * u;
        prow_[u] = MODE == MODE_CONV ? c % T : row_[u];
        pkc_[u] = MODE == MODE_CONV ? c / T : kc_[u];
    }
    // MODE_CONV: where this thread's positions sit in the input
    int base_h[kChunks] = {}, base_w[kChunks] = {};
    bool pos_ok[kChunks] = {};
    const uint8_t *q_img = p.Q;
    if (MODE == MODE_CONV) {
        q_img = p.Q + (size_t)img * p.H * p.W * p.C;
#pragma unroll
        for (int u = 0; u < kChunks; u++) {
            const int gj = j0 + row_[u];
            pos_ok[u] = gj < p.J;
            const int oh = gj / p.Wo, ow = gj - oh * p.Wo;
            base_h[u] = oh * p.sh - p.pt;
            base_w[u] = ow * p.sw - p.pl;
        }
    }

    // Byte offsets of this thread's chunks at k = 0, as 32-bit values added to a uniform base
    // that advances with k: the loads then need no per-stage address arithmetic at all.
    uint32_t p_off[kChunks], q_off[kChunks];
#pragma unroll
    for (int u = 0; u < kChunks; u++) {
        const int gi = i0 + prow_[u], gj = j0 + qrow_[u];
        p_off[u] = MODE == MODE_CONV ? qfrag_offset(gi, pkc_[u] * 16, p.K_pad)  // a stage of 128 k is 4 KB further on
                                     : (uint32_t)min(gi, p.I - 1) * (uint32_t)p.K + kc_[u] * 16;
        q_off[u] = MODE == MODE_MM ? qfrag_offset(gj, qkc_[u] * 16, p.K_pad) : 0u;  // a stage of 128 k is 4 KB further on
    }
    auto load_p = [&](int u, int k0) -> uint4 {
        if (MODE == MODE_CONV) {
            return *reinterpret_cast<const uint4 *>(p.P + (size_t)k0 * 32 + p_off[u]);
        } else if (ALIGNED) {
            // K % 128 == 0: every chunk is inside the row. Rows past I are clamped, not zeroed:
            // the rows of a product are independent and those outputs are never stored.
            // (the sign flip of a u8 operand is applied when the chunk is stored to LDS, so the
            // load has no consumer until then)
            return *reinterpret_cast<const uint4 *>(p.P + k0 + p_off[u]);
        } else {
            const int gi = i0 + row_[u], gk = k0 + kc_[u] * 16;
            if (gi >= p.I || gk >= p.K) return make_uint4(0, 0, 0, 0);
            const uint8_t *src = p.P + (size_t)gi * p.K + gk;
            uint32_t w[4] = {0, 0, 0, 0};
            for (int b = 0; b < 16; b++)
                if (gk + b < p.K) w[b >> 2] |= (uint32_t)(src[b] ^ (flip & 0xff)) << (8 * (b & 3));
            return make_uint4(w[0], w[1], w[2], w[3]);
        }
    };
    auto load_q = [&](int u, int k0) -> uint4 {
        const int gk = k0 + kc_[u] * 16;
        if (MODE == MODE_MM) {
            return *reinterpret_cast<const uint4 *>(p.Q + (size_t)k0 * 32 + q_off[u]);
        } else {
            const int gkc = min(gk, p.K - 16);
            const int tap = gkc / p.C, c0 = gkc - tap * p.C;
            const int r = tap / p.kw, s = tap - r * p.kw;
            const int ih = base_h[u] + r * p.dh, iw = base_w[u] + s * p.dw;
            const bool inside = ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
            const int ihc = min(max(ih, 0), p.H - 1), iwc = min(max(iw, 0), p.W - 1);
            const uint4 v = HIPC_LOAD_ALWAYS(reinterpret_cast<const uint4 *>(q_img + ((size_t)ihc * p.W + iwc) * p.C + c0));
            const bool live = pos_ok[u] && gk < p.K;  // beyond the problem: zeros; padding taps: the zero point
            const uint32_t alt = live ? pad_word : 0u;
            const bool take = live && inside;
            return make_uint4(take ? v.x : alt, take ? v.y : alt, take ? v.z : alt, take ? v.w : alt);
        }
    };
    auto load_regs = [&](GemmRegs<kChunks> &r, int stage) {
        const int k0 = stage * kBK;
#pragma unroll
        for (int u = 0; u < kChunks; u++) r.p[u] = load_p(u, k0);
#pragma unroll
        for (int u = 0; u < kChunks; u++) r.q[u] = load_q(u, k0);
    };
    // `live` false (a stage past the end, only met when the stage count is odd) stores zeros,
    // which add nothing to the product or to the operand sums.
    auto store_regs = [&](const GemmRegs<kChunks> &r, int buf, bool live) {
        const uint32_t keep = live ? 0xffffffffu : 0u;
        const uint32_t late_flip = (MODE == MODE_MM && ALIGNED) ? flip : 0u;
#pragma unroll
        for (int u = 0; u < kChunks; u++) {
            *reinterpret_cast<uint4 *>(lds_p + buf * T * kPitch + prow_[u] * kPitch + pkc_[u] * 16) =
                make_uint4((r.p[u].x ^ late_flip) & keep, (r.p[u].y ^ late_flip) & keep, (r.p[u].z ^ late_flip) & keep,
                           (r.p[u].w ^ late_flip) & keep);
            *reinterpret_cast<uint4 *>(lds_q + buf * T * kPitch + qrow_[u] * kPitch + qkc_[u] * 16) =
                make_uint4(r.q[u].x & keep, r.q[u].y & keep, r.q[u].z & keep, r.q[u].w & keep);
        }
    };

    i32x16 acc[kF][kF];
#pragma unroll
    for (int i = 0; i < kF; i++)
#pragma unroll
        for (int j = 0; j < kF; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
    int dsum[kF] = {};

    auto compute = [&](int buf) {
        const uint8_t *bp = lds_p + buf * T * kPitch + (wm * kWT + r32) * kPitch + kg * 16;
        const uint8_t *bq = lds_q + buf * T * kPitch + (wn * kWT + r32) * kPitch + kg * 16;
#pragma unroll
        for (int step = 0; step < kBK / 32; step++) {
            uint4 pf[kF], qf[kF];
#pragma unroll
            for (int i = 0; i < kF; i++) pf[i] = *reinterpret_cast<const uint4 *>(bp + i * 32 * kPitch + step * 32);
#pragma unroll
            for (int j = 0; j < kF; j++) qf[j] = *reinterpret_cast<const uint4 *>(bq + j * 32 * kPitch + step * 32);
            // always taken: a branch here would cost more than the eight dot instructions
#pragma unroll
            for (int f = 0; f < kF; f++) dsum[f] += dot_ones(MODE == MODE_MM ? pf[f] : qf[f]);
#pragma unroll
            for (int i = 0; i < kF; i++)
#pragma unroll
                for (int j = 0; j < kF; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, pf[i]),
                                                                      __builtin_bit_cast(i32x4, qf[j]), acc[i][j], 0, 0, 0);
        }
    };

    // Two register sets and two LDS buffers: while stage s is multiplied out of LDS, stage s+1
    // sits in registers and stage s+2 is in flight. Stage indices past the end are clamped
    // (a redundant, cached load) rather than branched around.
    const int nk = p.K_pad / kBK;
    GemmRegs<kChunks> r0, r1;
    load_regs(r0, 0);
    load_regs(r1, min(1, nk - 1));
    store_regs(r0, 0, true);
    __syncthreads();
    // Two stages per trip and no exit in between, so the memory counters stay exact. With an
    // odd stage count the second half of the last trip multiplies a stage of zeros.
    for (int ks = 0; ks < nk; ks += 2) {
        load_regs(r0, min(ks + 2, nk - 1));
        compute(0);
        store_regs(r1, 1, ks + 1 < nk);
        __syncthreads();
        load_regs(r1, min(ks + 3, nk - 1));
        compute(1);
        store_regs(r0, 0, true);
        __syncthreads();
    }

    // sums of the dynamic operand over k: the two k halves of a row live in lanes l and l+32
    if (need_dyn_sum) {
#pragma unroll
        for (int f = 0; f < kF; f++) dsum[f] += __shfl_xor(dsum[f], 32, 64);
        if (MODE == MODE_MM) {
            if (kg == 0) {
#pragma unroll
                for (int f = 0; f < kF; f++) lds_sum[wave * kWT + f * 32 + r32] = dsum[f];
            }
        }
    }
    __syncthreads();

    const int kzz = p.K * zd * zc;
    float fmn = 0.f, fmx = 0.f;
#pragma unroll
    for (int i = 0; i < kF; i++) {
#pragma unroll
        for (int j = 0; j < kF; j++) {
            const int gj = j0 + wn * kWT + j * 32 + r32;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int rf = (r >> 2) * 8 + kg * 4 + (r & 3);  // row inside the 32x32 fragment
                const int gi = i0 + wm * kWT + i * 32 + rf;
                if (gi >= p.I || gj >= p.J) continue;
                int v = acc[i][j][r];
                const int csum = p.const_sum[MODE == MODE_MM ? gj : gi];
                v = v - zd * csum + kzz;
                if (need_dyn_sum) v -= zc * (MODE == MODE_MM ? lds_sum[wave * kWT + i * 32 + rf] : dsum[j]);
                gemm_emit<MODE, EPI>(p, img, gi, gj, v, fmn, fmx);
            }
        }
    }
    if (EPI == EPI_SCALE_BIAS) gemm_emit_range(p, lane, fmn, fmx);
}

// After a launch whose argument is a GemmArgs: the scalars of it that a replay of a recorded graph may change
// (hipc_graph_set_scalar). Zero points only when they were given by value (the QLinear operators).
// `sums`: the launched instance forms the dynamic operand's sums over k, which a non-zero zero point of the
// constant operand needs (an instance chosen because that zero point was known to be zero cannot take another).
inline void gemm_note_scalars(hipc_ctx *ctx, const GemmArgs &g, bool sums) {
    if (!ctx->capturing) return;
    if (g.host_zp) {
        note_scalar(ctx, HIPC_SCALAR_A_ZERO_POINT, offsetof(GemmArgs, dyn_zp_value));
        if (sums) note_scalar(ctx, HIPC_SCALAR_B_ZERO_POINT, offsetof(GemmArgs, const_zp_value));
    }
    if (g.ratio) note_scalar(ctx, HIPC_SCALAR_Y_ZERO_POINT, offsetof(GemmArgs, y_zp));
    if (g.scale) note_scalar(ctx, HIPC_SCALAR_RELU, offsetof(GemmArgs, relu));
}

// ---- host side: tile choice and launch of the kernel above ---------------------------------
// 64x64 tiles until 128x128 ones would give every CU at least two workgroups;
// the gemm_tile option (64 / 128) overrides (tuning, tests).
inline int gemm_tile(hipc_ctx *ctx, const GemmArgs &g, unsigned batch) {
    const int forced = ctx->tune.gemm_tile;
    if (forced == 64 || forced == 128) return forced;
    const int64_t tiles = ceil_div(g.I, kBM) * ceil_div(g.J, kBN) * (int64_t)batch;
    return tiles >= 512 ? 128 : 64;
}

template <int MODE, int EPI, bool ALIGNED, int T>
int gemm_launch_tile(hipc_ctx *ctx, GemmArgs g, unsigned batch) {
    static bool lds_allowed[kMaxDevices] = {};
    if (int rc = allow_dynamic_lds(ctx, int8_gemm_kernel<MODE, EPI, ALIGNED, T>, gemm_lds(T), lds_allowed)) return rc;
    const dim3 grid(gemm_grid(g, T), 1, batch);
    hipLaunchKernelGGL((int8_gemm_kernel<MODE, EPI, ALIGNED, T>), grid, 256, gemm_lds(T), ctx->stream, g);
    HIPC_LAUNCHED(ctx);
    gemm_note_scalars(ctx, g, true);
    return HIPC_OK;
}

template <int MODE, int EPI, bool ALIGNED>
int gemm_launch(hipc_ctx *ctx, const GemmArgs &g, unsigned batch) {
    return gemm_tile(ctx, g, batch) == 64 ? gemm_launch_tile<MODE, EPI, ALIGNED, 64>(ctx, g, batch)
                                     : gemm_launch_tile<MODE, EPI, ALIGNED, 128>(ctx, g, batch);
}

// ---- the small-problem variant (MODE_MM, aligned A) ---------------------------------------
// A product of a few hundred 64x64 tiles. The LDS-staged kernel above is bound by LDS bandwidth
// there: per 128-k stage a 64x64 tile stores 16 KB and its four 32x32 wavefronts read 32 KB, 384
// clocks of LDS for 128 clocks of products. Here
//   * the four wavefronts of a workgroup split the four 32-k product steps of a stage between them
//     and each owns the whole 64x64 tile (2x2 accumulators), so every byte in LDS is read once;
//   * only A goes through LDS (8 KB stored, 8 KB read per stage); the fragments of the prepacked,
//     fragment-major B come straight from memory into the matrix-core layout, one fully coalesced
//     1 KB load each, four stages ahead;
//   * the four partial tiles are added through LDS at the end, wavefront w finishing fragment w.
// Measured against the LDS-staged 64x64 tiles: 12.8 against 17.3 us for 1000 x 4096 x 1024, 7.8
// against 8.5 us at k = 1024; from about four tiles per CU on, or with very short k, the reduction
// at the end costs more than the loop saves. (The same kernel with 128x128 tiles, wavefronts 2x2
// and no k split was slower than either: 16 products per stage issued back to back keep the
// wavefront from issuing the stage's memory instructions, as in the 128x128 LDS-staged kernel.)
constexpr int kSmallSets = 4;  // register sets of A chunks and of B fragments: stages in flight
// the hand-over of three fragments per wavefront reuses the two A buffers (18 KB of its 48 KB)
constexpr size_t kSmallLds = 4 * 3 * 16 * 64 * sizeof(int) + 4 * 64 * sizeof(int);

template <int EPI, bool DYN>
__global__ void __launch_bounds__(256, 3) int8_gemm_small_kernel(const GemmArgs p) {  // three workgroups per CU (LDS allows no more): 168 registers
    constexpr int T = 64;                       // edge of the workgroup's tile
    constexpr int kCh = T / 32;                 // 16-byte chunks of an A slab per thread
    constexpr int kSteps = 1;                   // product steps of a stage per wavefront
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    uint8_t *lds_a = lds_raw;                                              // [2][T * kPitch]
    int *lds_acc = reinterpret_cast<int *>(lds_raw);                       // after the loop: [owner][source 0..2][16][64]
    int *lds_sum = lds_acc + 4 * 3 * 16 * 64;                              // [4 wavefronts][64 rows]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r32 = lane & 31, kg = lane >> 5;
    auto handed = [&](int owner, int slot, int r) -> int & { return lds_acc[((owner * 3 + slot) * 16 + r) * 64 + lane]; };

    const int tiles_x = (p.J + T - 1) / T, tiles_y = (p.I + T - 1) / T;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int rows_per = (tiles_y + p.xcd_rows - 1) / p.xcd_rows, cols_per = (tiles_x + p.xcd_cols - 1) / p.xcd_cols;
    const int ty = (xcd / p.xcd_cols) * rows_per + idx / cols_per, tx = (xcd % p.xcd_cols) * cols_per + idx % cols_per;
    if (idx >= rows_per * cols_per || ty >= tiles_y || tx >= tiles_x) return;
    const int i0 = ty * T, j0 = tx * T;
    const int nk = p.K / kBK;

    const int zd = (p.host_zp ? p.dyn_zp_value : zp_byte(p.dyn_zp, p.dyn_signed)) - p.dyn_shift;
    const int zc = (p.host_zp ? p.const_zp_value : zp_byte(p.const_zp, p.const_signed)) - p.const_shift;
    const uint32_t flip = p.dyn_shift ? 0x80808080u : 0u;

    // A: chunk c = tid + 256 u of a T-row slab: row c / 8, 16-byte column c % 8 (whole lines per row)
    uint32_t p_off[kCh], l_off[kCh];
#pragma unroll
    for (int u = 0; u < kCh; u++) {
        const int c = tid + 256 * u, row = c >> 3, kc = c & 7;
        p_off[u] = (uint32_t)min(i0 + row, p.I - 1) * (uint32_t)p.K + kc * 16;  // rows past I: clamped, never stored
        l_off[u] = row * kPitch + kc * 16;
    }
    // B: fragments j0 / 32 and j0 / 32 + 1 of this wavefront's product step; a step is 1 KB on, a stage 4 KB.
    // Wavefront w will finish fragment (rows w >> 1, columns w & 1) and numbers its operands and
    // accumulators from that one: acc[di][dj] is fragment ((w >> 1) ^ di, (w & 1) ^ dj), so its own
    // part is acc[0][0] whatever w is and the epilogue is one piece of code.
    const int j_last = (p.J + kBN - 1) / kBN * kBN - 1;  // B is packed in whole 128-column tiles
    uint32_t q_off[2];
#pragma unroll
    for (int f = 0; f < 2; f++)
        q_off[f] = qfrag_offset(min(j0 + (f ^ (wave & 1)) * 32, j_last - 31), wave * 32, p.K_pad) + lane * 16;
    const __amdgpu_buffer_rsrc_t rsrc_p = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(p.P), 0, (int)((uint32_t)p.I * (uint32_t)p.K), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_q = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(p.Q), 0, (int)((uint32_t)(j_last + 1) * (uint32_t)p.K_pad), 0x00020000);

    u32x4 ra[kSmallSets][kCh], rb[kSmallSets][kSteps][2];
    auto load_a = [&](int set, int stage) {
#pragma unroll
        for (int u = 0; u < kCh; u++) ra[set][u] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_p, p_off[u], min(stage, nk - 1) * kBK, 0);
    };
    auto load_b = [&](int set, int stage) {
#pragma unroll
        for (int step = 0; step < kSteps; step++)
#pragma unroll
            for (int f = 0; f < 2; f++)
                rb[set][step][f] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_q, q_off[f] + step * 1024, min(stage, nk - 1) * kBK * 32, 0);
    };
    // a stage past the end is stored as zeros: its products add nothing whatever B holds
    auto store_a = [&](int set, int buf, bool live) {
        const uint32_t keep = live ? 0xffffffffu : 0u;
#pragma unroll
        for (int u = 0; u < kCh; u++)
            *reinterpret_cast<u32x4 *>(lds_a + buf * T * kPitch + l_off[u]) = (ra[set][u] ^ flip) & keep;
    };

    // what this lane's outputs need of their column (fragment (wave >> 1, wave & 1), column r32): asked
    // for now, so that the epilogue does not start with a memory round trip
    const int my_col = min(j0 + (wave & 1) * 32 + r32, p.J - 1);
    const int my_csum = p.const_sum[my_col];
    const EmitColumn my_emit = gemm_emit_column<EPI>(p, my_col);

    i32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
    int dsum[2] = {0, 0};
    const uint32_t frag_a = r32 * kPitch + wave * 32 + kg * 16;
    auto compute = [&](int buf, int set) {
        uint4 av[kSteps][2];
#pragma unroll
        for (int step = 0; step < kSteps; step++)
#pragma unroll
            for (int f = 0; f < 2; f++)
                av[step][f] = *reinterpret_cast<const uint4 *>(lds_a + buf * T * kPitch + frag_a + (f ^ (wave >> 1)) * 32 * kPitch + step * 32);
#pragma unroll
        for (int step = 0; step < kSteps; step++) {
            if (DYN) {
#pragma unroll
                for (int f = 0; f < 2; f++) dsum[f] += dot_ones(av[step][f]);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, av[step][i]),
                                                                      __builtin_bit_cast(i32x4, rb[set][step][j]), acc[i][j], 0, 0, 0);
        }
    };

#pragma unroll
    for (int d = 0; d < kSmallSets; d++) load_a(d, d), load_b(d, d);
    store_a(0, 0, true);
    load_a(0, kSmallSets);
    __syncthreads();
    // Stage s: multiply it out of LDS buffer s & 1 with B set s % 4, refill that B set with stage
    // s + 4, move stage s + 1 from its A set into the other LDS buffer (last read during stage s - 1,
    // before the previous barrier) and refill that A set with stage s + 5. Nothing in the loop is
    // conditional, so the memory counters stay exact.
    for (int s = 0; s < nk; s += kSmallSets) {
#pragma unroll
        for (int d = 0; d < kSmallSets; d++) {
            compute(d & 1, d);
            load_b(d, s + d + kSmallSets);
            store_a((d + 1) % kSmallSets, (d + 1) & 1, s + d + 1 < nk);
            load_a((d + 1) % kSmallSets, s + d + 1 + kSmallSets);
            __syncthreads();
        }
    }

    // row sums of A over this wavefront's product steps: the two k halves of a row live in lanes l and l + 32
    const int ifr = wave >> 1, jf = wave & 1;
    if (DYN) {
#pragma unroll
        for (int f = 0; f < 2; f++) dsum[f] += __shfl_xor(dsum[f], 32, 64);
        if (kg == 0) {
#pragma unroll
            for (int f = 0; f < 2; f++) lds_sum[wave * 64 + (f ^ ifr) * 32 + r32] = dsum[f];
        }
    }
    // the other three fragments are handed over (the A buffers are free: the loop ended with a barrier)
#pragma unroll
    for (int di = 0; di < 2; di++)
#pragma unroll
        for (int dj = 0; dj < 2; dj++) {
            if (di == 0 && dj == 0) continue;
            const int owner = ((ifr ^ di) << 1) | (jf ^ dj);
            const int slot = wave < owner ? wave : wave - 1;  // 0..2 among the three sources
#pragma unroll
            for (int r = 0; r < 16; r++) handed(owner, slot, r) = acc[di][dj][r];
        }
    __syncthreads();

    // The handed-over parts are read four output rows ahead of their use: the LDS latency is paid
    // once, not per output, and the stores still leave spread out (other workgroups of the CU are
    // in their product loops meanwhile).
    const int fixed = p.K * zd * zc - zd * my_csum;
    const int gj = j0 + jf * 32 + r32;
    float fmn = 0.f, fmx = 0.f;
    int part[2][4], rs[2][4];
    auto read_group = [&](int g, int par) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int r = 4 * g + e;
            part[par][e] = handed(wave, 0, r) + handed(wave, 1, r) + handed(wave, 2, r);
            if (DYN) {
                const int at = ifr * 32 + g * 8 + kg * 4 + e;
                rs[par][e] = lds_sum[at] + lds_sum[64 + at] + lds_sum[128 + at] + lds_sum[192 + at];
            }
        }
    };
    read_group(0, 0);
#pragma unroll
    for (int g = 0; g < 4; g++) {
        if (g + 1 < 4) read_group(g + 1, (g + 1) & 1);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int gi = i0 + ifr * 32 + g * 8 + kg * 4 + e;
            int v = acc[0][0][4 * g + e] + part[g & 1][e] + fixed;
            if (DYN) v -= zc * rs[g & 1][e];
            if (gi < p.I && gj < p.J) gemm_emit_mm<EPI>(p, my_emit, gi, gj, v, fmn, fmx);
        }
    }
    if (EPI == EPI_SCALE_BIAS) gemm_emit_range(p, lane, fmn, fmx);
}

// What the k-split convolution kernels below end with. The four wavefronts hold partial products
// of all four 32x32 fragments of the 64x64 tile, positions x channels, with the positions along
// the rows of the matrix-core result: register r of lane l is position (r >> 2) * 8 + (l >> 5) * 4
// + (r & 3), channel l & 31. Wavefront w finishes fragment (positions jf = w & 1, channels
// ifr = w >> 1), and every wavefront numbers its accumulators from that one: acc[dj][di] is
// fragment (jf ^ dj, ifr ^ di), so its own part is acc[0][0] and needs no choosing. The other three
// wavefronts' parts arrive through LDS (lds_acc: [owner][source 0..2][16][64], lds_sum:
// [4 wavefronts][64 positions] activation sums, dsum[f] being those of positions fragment jf ^ f).
// A lane then owns one output channel -- one weight sum, ratio and bias -- and runs of four
// consecutive positions of it, which leave as one 32-bit (bytes) or 128-bit (int32) store.
// Every wavefront must be past its last read of whatever else lived in that LDS before this is called.
struct ConvChannel {
    int csum = 0, qb = 0;
    float ratio = 0.f;
};
template <int EPI>
__device__ __forceinline__ ConvChannel conv_small_channel(const GemmArgs &p, int i0) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ch = i0 + (wave >> 1) * 32 + (lane & 31);
    ConvChannel c;
    c.csum = p.const_sum[ch];  // I_pad rows exist
    const int cc = min(ch, p.I - 1);
    if (EPI == EPI_REQUANT) {
        c.ratio = p.ratio[(size_t)cc * p.ratio_step];
        if (p.qbias) c.qb = p.qbias[cc];
    }
    return c;
}

template <int EPI, bool DYN>
__device__ __forceinline__ void conv_small_finish(const GemmArgs &p, i32x16 (&acc)[2][2], int (&dsum)[2], const ConvChannel &chan,
                                                  int *lds_acc, int *lds_sum, int i0, int j0, int img, int zd, int zc) {
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r32 = lane & 31, kg = lane >> 5;
    auto handed = [&](int owner, int slot, int r) -> int & { return lds_acc[((owner * 3 + slot) * 16 + r) * 64 + lane]; };
    const int jf = wave & 1, ifr = wave >> 1;
    // sums of the activations over this wavefront's product steps, per position: the two k halves live in lanes l and l + 32
    if (DYN) {
#pragma unroll
        for (int f = 0; f < 2; f++) dsum[f] += __shfl_xor(dsum[f], 32, 64);
        if (kg == 0) {
#pragma unroll
            for (int f = 0; f < 2; f++) lds_sum[wave * 64 + (f ^ jf) * 32 + r32] = dsum[f];
        }
    }
#pragma unroll
    for (int dj = 0; dj < 2; dj++)
#pragma unroll
        for (int di = 0; di < 2; di++) {
            if (dj == 0 && di == 0) continue;
            const int owner = ((ifr ^ di) << 1) | (jf ^ dj);
            const int slot = wave < owner ? wave : wave - 1;
#pragma unroll
            for (int r = 0; r < 16; r++) handed(owner, slot, r) = acc[dj][di][r];
        }
    __syncthreads();

    // all of the LDS reads first, so that their latency is paid once and not per output
    int part[3][16], qs[16];
#pragma unroll
    for (int slot = 0; slot < 3; slot++)
#pragma unroll
        for (int r = 0; r < 16; r++) part[slot][r] = handed(wave, slot, r);
    if (DYN) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int at = jf * 32 + (r >> 2) * 8 + kg * 4 + (r & 3);
            qs[r] = lds_sum[at] + lds_sum[64 + at] + lds_sum[128 + at] + lds_sum[192 + at];
        }
    }
    const int ch = i0 + ifr * 32 + r32;
    const int fixed = p.K * zd * zc - zd * chan.csum + (EPI == EPI_REQUANT ? chan.qb : 0);
    const int lo = p.out_signed ? -128 : 0, hi = p.out_signed ? 127 : 255;
    int out[16];
#pragma unroll
    for (int r = 0; r < 16; r++) {
        int v = acc[0][0][r] + part[0][r] + part[1][r] + part[2][r] + fixed;
        if (DYN) v -= zc * qs[r];
        if (EPI == EPI_REQUANT) v = min(max((int)rintf(__fmul_rn((float)v, chan.ratio)) + p.y_zp, lo), hi) & 0xff;
        out[r] = v;
    }
    if (ch >= p.I) return;
    const size_t row = ((size_t)img * p.I + ch) * p.J;
    const bool wide = (p.J & 3) == 0 && (reinterpret_cast<uintptr_t>(p.Y) & (EPI == EPI_REQUANT ? 3 : 15)) == 0;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const int pos = j0 + jf * 32 + g * 8 + kg * 4;   // four consecutive positions: out[4 g ..]
        if (wide && pos + 3 < p.J) {
            if (EPI == EPI_REQUANT) {
                const uint32_t word = (uint32_t)out[4 * g] | (uint32_t)out[4 * g + 1] << 8 | (uint32_t)out[4 * g + 2] << 16 |
                                      (uint32_t)out[4 * g + 3] << 24;
                *reinterpret_cast<uint32_t *>(static_cast<uint8_t *>(p.Y) + row + pos) = word;
            } else {
                // written once and several times the operands: kept from displacing them in the caches
                i32x4 quad = {out[4 * g], out[4 * g + 1], out[4 * g + 2], out[4 * g + 3]};
                __builtin_nontemporal_store(quad, reinterpret_cast<i32x4 *>(static_cast<int32_t *>(p.Y) + row + pos));
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                if (pos + e >= p.J) continue;
                if (EPI == EPI_REQUANT) static_cast<uint8_t *>(p.Y)[row + pos + e] = (uint8_t)out[4 * g + e];
                else static_cast<int32_t *>(p.Y)[row + pos + e] = out[4 * g + e];
            }
        }
    }
}

// The same arrangement for a convolution with few 64x64 tiles (MODE_CONV): the gathered activation
// chunks (the Q operand: 64 output positions x 128 bytes of (kh, kw, c) per stage) go through LDS,
// the fragments of the prepacked, fragment-major weight (the P operand) come straight from memory,
// and the four wavefronts split the product steps of a stage and add up at the end.
template <int EPI, bool DYN>
__global__ void __launch_bounds__(256) int8_conv_small_kernel(const GemmArgs p) {
    constexpr int T = 64;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    uint8_t *lds_q = lds_raw;                                              // [2][T * kPitch]
    int *lds_acc = reinterpret_cast<int *>(lds_raw);                       // after the loop: [owner][source 0..2][16][64]
    int *lds_sum = lds_acc + 4 * 3 * 16 * 64;                              // [4 wavefronts][64 positions]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r32 = lane & 31, kg = lane >> 5;
    const int img = blockIdx.z;

    const int tiles_x = (p.J + T - 1) / T, tiles_y = (p.I + T - 1) / T;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int rows_per = (tiles_y + p.xcd_rows - 1) / p.xcd_rows, cols_per = (tiles_x + p.xcd_cols - 1) / p.xcd_cols;
    const int ty = (xcd / p.xcd_cols) * rows_per + idx / cols_per, tx = (xcd % p.xcd_cols) * cols_per + idx % cols_per;
    if (idx >= rows_per * cols_per || ty >= tiles_y || tx >= tiles_x) return;
    const int i0 = ty * T, j0 = tx * T;
    const int nk = p.K_pad / kBK;

    const int zd = (p.host_zp ? p.dyn_zp_value : zp_byte(p.dyn_zp, p.dyn_signed)) - p.dyn_shift;
    const int zc = (p.host_zp ? p.const_zp_value : zp_byte(p.const_zp, p.const_signed)) - p.const_shift;
    const uint32_t pad_word = (uint32_t)(zd & 0xff) * 0x01010101u;

    // Q: chunk c = tid + 256 u of a 64-position slab: position c / 8, 16-byte k chunk c % 8
    int kc_[2], base_h[2], base_w[2];
    bool pos_ok[2];
    uint32_t l_off[2];
    const uint8_t *q_img = p.Q + (size_t)img * p.H * p.W * p.C;
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const int c = tid + 256 * u, row = c >> 3;
        kc_[u] = c & 7;
        const int gj = j0 + row;
        pos_ok[u] = gj < p.J;
        const int oh = gj / p.Wo, ow = gj - oh * p.Wo;
        base_h[u] = oh * p.sh - p.pt;
        base_w[u] = ow * p.sw - p.pl;
        l_off[u] = row * kPitch + kc_[u] * 16;
    }
    // P: fragments i0 / 32 and i0 / 32 + 1 of this wavefront's product step, the one this wavefront
    // will finish first (see conv_small_finish); a step is 1 KB on, a stage 4 KB
    const uint8_t *p_frag[2];
#pragma unroll
    for (int f = 0; f < 2; f++)
        p_frag[f] = p.P + qfrag_offset(i0 + (f ^ (wave >> 1)) * 32, wave * 32, p.K_pad) + lane * 16;  // I_pad is a multiple of 128

    uint4 rq[kSmallSets][2], rp[kSmallSets][2];
    // Where a chunk's 16 bytes sit in the filter window: (row, column, first channel) of the stage
    // about to be loaded. load_q is called for stages 0, 1, 2, ... in turn, so the triple moves on
    // by one stage (kBK bytes of k) per call with adds and compares only; the divisions are made
    // once, here, and the step's own quotients are the same for every thread.
    const int adv_tap = kBK / p.C, adv_c = kBK - adv_tap * p.C;
    const int adv_r = adv_tap / p.kw, adv_s = adv_tap - adv_r * p.kw;
    int q_k[2], q_r[2], q_s[2], q_c[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
        q_k[u] = kc_[u] * 16;
        const int tap = q_k[u] / p.C;
        q_c[u] = q_k[u] - tap * p.C;
        q_r[u] = tap / p.kw;
        q_s[u] = tap - q_r[u] * p.kw;
    }
    // beyond the problem: zeros; padding taps: the zero point (which contributes nothing).
    // Past K the triple points outside the window; the clamps keep the address inside the image.
    auto load_q = [&](int set) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int ih = base_h[u] + q_r[u] * p.dh, iw = base_w[u] + q_s[u] * p.dw;
            const bool inside = ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
            const int ihc = min(max(ih, 0), p.H - 1), iwc = min(max(iw, 0), p.W - 1);
            const uint4 v = HIPC_LOAD_ALWAYS(reinterpret_cast<const uint4 *>(q_img + ((size_t)ihc * p.W + iwc) * p.C + q_c[u]));
            const bool live = pos_ok[u] && q_k[u] < p.K;
            const uint32_t alt = live ? pad_word : 0u;
            const bool take = live && inside;
            rq[set][u] = make_uint4(take ? v.x : alt, take ? v.y : alt, take ? v.z : alt, take ? v.w : alt);
            q_k[u] += kBK;
            q_c[u] += adv_c;
            const int wrap = q_c[u] >= p.C ? 1 : 0;
            q_c[u] -= wrap ? p.C : 0;
            q_s[u] += adv_s + wrap;
            const int down = q_s[u] >= p.kw ? 1 : 0;
            q_s[u] -= down ? p.kw : 0;
            q_r[u] = min(q_r[u] + adv_r + down, 1 << 20);
        }
    };
    auto load_p = [&](int set, int stage) {
#pragma unroll
        for (int f = 0; f < 2; f++) rp[set][f] = *reinterpret_cast<const uint4 *>(p_frag[f] + (size_t)min(stage, nk - 1) * kBK * 32);
    };
    // a stage past the end is stored as zeros: its products add nothing whatever the weight holds
    auto store_q = [&](int set, int buf, bool live) {
        const uint32_t keep = live ? 0xffffffffu : 0u;
#pragma unroll
        for (int u = 0; u < 2; u++)
            *reinterpret_cast<uint4 *>(lds_q + buf * T * kPitch + l_off[u]) =
                make_uint4(rq[set][u].x & keep, rq[set][u].y & keep, rq[set][u].z & keep, rq[set][u].w & keep);
    };

    i32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
    int dsum[2] = {0, 0};
    const uint32_t frag_q = r32 * kPitch + wave * 32 + kg * 16;
    auto compute = [&](int buf, int set) {
        i32x4 b[2];
#pragma unroll
        for (int f = 0; f < 2; f++) {
            const uint4 v = *reinterpret_cast<const uint4 *>(lds_q + buf * T * kPitch + frag_q + (f ^ (wave & 1)) * 32 * kPitch);
            b[f] = __builtin_bit_cast(i32x4, v);
            if (DYN) dsum[f] += dot_ones(v);
        }
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
                acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[j], __builtin_bit_cast(i32x4, rp[set][i]), acc[j][i], 0, 0, 0);
    };

#pragma unroll
    for (int d = 0; d < kSmallSets; d++) load_q(d), load_p(d, d);
    store_q(0, 0, true);
    load_q(0);
    __syncthreads();
    for (int s = 0; s < nk; s += kSmallSets) {
#pragma unroll
        for (int d = 0; d < kSmallSets; d++) {
            compute(d & 1, d);
            load_p(d, s + d + kSmallSets);
            store_q((d + 1) % kSmallSets, (d + 1) & 1, s + d + 1 < nk);
            load_q((d + 1) % kSmallSets);
            __syncthreads();
        }
    }

    // asked for before the hand-over, so that the epilogue does not start with a memory round trip
    const ConvChannel chan = conv_small_channel<EPI>(p, i0);
    conv_small_finish<EPI, DYN>(p, acc, dsum, chan, lds_acc, lds_sum, i0, j0, img, zd, zc);
}

// A convolution along one axis (H = 1, a 1 x kw window) with few 64x64 tiles, straight from the
// NCHW activation. The 64 output positions of a tile see 63 sw + (kw - 1) dw + 1 input positions
// of every channel: that slab is read once, as 32-bit words along the positions, transposed 4 x 4
// in registers and kept in LDS for the whole product as [16-channel chunk][position][16 bytes].
// A lane's operand chunk of product step k = tap * C + c is then one 16-byte LDS read at position
// (output position) * sw + tap * dw, consecutive lanes reading consecutive 16 bytes; nothing is
// gathered from memory and the k loop has no barrier. The weight fragments come straight from
// memory and the four wavefronts split the product steps, as in the kernel above.
// p.Q is the NCHW activation as the caller gave it (uint8 is shifted to signed on the way in),
// p.slab_pos the positions a slab holds (a multiple of 4). Needs W % 4 == 0 and 4-byte aligned images.
constexpr int kRowBatch = 4;  // steps of the slab loader whose loads are in flight together
template <int EPI, bool DYN>
__global__ void __launch_bounds__(256, 3) int8_conv_row_kernel(const GemmArgs p) {
    constexpr int T = 64;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    uint8_t *slab = lds_raw;                                               // [C / 16][slab_pos][16]
    int *lds_acc = reinterpret_cast<int *>(lds_raw);                       // after the loop: [owner][source 0..2][16][64]
    int *lds_sum = lds_acc + 4 * 3 * 16 * 64;                              // [4 wavefronts][64 positions]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r32 = lane & 31, kg = lane >> 5;
    const int img = blockIdx.z;

    const int tiles_x = (p.J + T - 1) / T, tiles_y = (p.I + T - 1) / T;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int rows_per = (tiles_y + p.xcd_rows - 1) / p.xcd_rows, cols_per = (tiles_x + p.xcd_cols - 1) / p.xcd_cols;
    const int ty = (xcd / p.xcd_cols) * rows_per + idx / cols_per, tx = (xcd % p.xcd_cols) * cols_per + idx % cols_per;
    if (idx >= rows_per * cols_per || ty >= tiles_y || tx >= tiles_x) return;
    const int i0 = ty * T, j0 = tx * T;
    const int nk = p.K_pad / kBK;

    const int zd = (p.host_zp ? p.dyn_zp_value : zp_byte(p.dyn_zp, p.dyn_signed)) - p.dyn_shift;
    const int zc = (p.host_zp ? p.const_zp_value : zp_byte(p.const_zp, p.const_signed)) - p.const_shift;
    const uint32_t pad_word = (uint32_t)(zd & 0xff) * 0x01010101u;
    const uint32_t flip4 = p.dyn_shift ? 0x80808080u : 0u;

    // P: fragments i0 / 32 and i0 / 32 + 1 of this wavefront's product step; a step is 1 KB on, a stage 4 KB
    const uint8_t *p_frag[2];
#pragma unroll
    for (int f = 0; f < 2; f++)
        p_frag[f] = p.P + qfrag_offset(i0 + (f ^ (wave >> 1)) * 32, wave * 32, p.K_pad) + lane * 16;  // I_pad is a multiple of 128
    uint4 rp[kSmallSets][2];
    auto load_p = [&](int set, int stage) {
#pragma unroll
        for (int f = 0; f < 2; f++) rp[set][f] = *reinterpret_cast<const uint4 *>(p_frag[f] + (size_t)min(stage, nk - 1) * kBK * 32);
    };
#pragma unroll
    for (int d = 0; d < kSmallSets; d++) load_p(d, d);
    // the epilogue's per-channel constants travel with the first loads
    const ConvChannel chan = conv_small_channel<EPI>(p, i0);

    // The slab starts at the 4-aligned input position at or below the tile's first one. Its
    // (16-channel chunk, position quad) pairs are numbered chunk * npq + quad and dealt 16 to a
    // wavefront instruction, 64 to a step of the workgroup: lane l takes pair 16 wave + (l >> 2) +
    // 64 step and, of it, channel quad l & 3 -- it reads four positions of four channels and writes
    // four words, each the four channels of one position. A lane's pair moves on by 64 per step:
    // 64 / npq chunks and 64 % npq quads, with adds and compares. Words outside the row hold the
    // zero point (W % 4 == 0: a word is inside or outside as a whole).
    const int SP = p.slab_pos, npq = SP >> 2;
    const int in0 = j0 * p.sw - p.pl;
    const int base = in0 & ~3, lead = in0 - base;
    const int n_chunks = p.C >> 4, n_pairs = n_chunks * npq;
    const uint8_t *x_img = p.Q + (size_t)img * p.C * p.W;
    const int cq4 = (lane & 3) * 4;
    const int adv_chunk = 64 / npq, adv_pq = 64 - adv_chunk * npq;
    int pair = wave * 16 + (lane >> 2);
    int chunk = pair / npq, pq = pair - chunk * npq;
    for (int first = 0; first < n_pairs; first += 64 * kRowBatch) {   // the same count for every lane
        uint32_t in[kRowBatch][4];
        int at[kRowBatch];   // byte offset of the pair's first word in the slab, or -1: nothing to store
#pragma unroll
        for (int u = 0; u < kRowBatch; u++) {
            at[u] = -1;
            if (first + 64 * u >= n_pairs) continue;   // a step with no pair at all asks for nothing
            const int gpos = base + 4 * pq;
            const bool live = pair < n_pairs;
            const bool inside = live && gpos >= 0 && gpos < p.W;
            const uint8_t *src = x_img + (size_t)(min(chunk, n_chunks - 1) * 16 + cq4) * p.W + (inside ? gpos : 0);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t v = *reinterpret_cast<const uint32_t *>(src + (size_t)i * p.W);
                in[u][i] = inside ? v ^ flip4 : pad_word;
            }
            at[u] = live ? (chunk * SP + 4 * pq) * 16 + cq4 : -1;
            pair += 64;
            pq += adv_pq, chunk += adv_chunk;
            if (pq >= npq) pq -= npq, chunk++;
        }
#pragma unroll
        for (int u = 0; u < kRowBatch; u++) {
            if (at[u] < 0) continue;
            const uint32_t lo01 = __builtin_amdgcn_perm(in[u][1], in[u][0], 0x05010400u);  // a0 b0 a1 b1
            const uint32_t hi01 = __builtin_amdgcn_perm(in[u][1], in[u][0], 0x07030602u);  // a2 b2 a3 b3
            const uint32_t lo23 = __builtin_amdgcn_perm(in[u][3], in[u][2], 0x05010400u);  // c0 d0 c1 d1
            const uint32_t hi23 = __builtin_amdgcn_perm(in[u][3], in[u][2], 0x07030602u);  // c2 d2 c3 d3
            uint32_t *dst = reinterpret_cast<uint32_t *>(slab + at[u]);
            dst[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);   // a0 b0 c0 d0: position 4 pq
            dst[4] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
            dst[8] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
            dst[12] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
        }
    }

    // This lane's 16 bytes of product step n (k = 128 n + 32 wave + 16 kg) are channels q_c.. of some
    // tap: in the slab, `off` bytes from its start for the lane's position in fragment 0. Both move
    // on by 128 bytes of k per step with adds and compares (the quotients of the step are the same
    // for every thread): (adv_c / 16) chunks and adv_tap taps on, and one tap on less a whole row
    // of chunks when the channel wraps. Past K the weight is zero and the address is clamped into
    // the slab, so the product adds nothing; the activation sums skip those steps.
    const int adv_tap = kBK / p.C, adv_c = kBK - adv_tap * p.C;
    const int SP16 = SP * 16;
    const int step_off = (adv_c >> 4) * SP16 + adv_tap * p.dw * 16, wrap_off = p.dw * 16 - (p.C >> 4) * SP16;
    const int last_off = (p.C >> 4) * SP16 - 16;
    int q_k = wave * 32 + kg * 16;
    const int tap0 = q_k / p.C;
    int q_c = q_k - tap0 * p.C;
    int off = (q_c >> 4) * SP16 + (lead + r32 * p.sw + tap0 * p.dw) * 16;
    int frag_off[2];   // the wavefront's own positions fragment first (see conv_small_finish)
#pragma unroll
    for (int f = 0; f < 2; f++) frag_off[f] = (f ^ (wave & 1)) * 32 * p.sw * 16;

    i32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
    int dsum[2] = {0, 0};
    // the operand of the next step is read from LDS before this step's products are issued
    uint4 bq[2][2];
    auto read_q = [&](int par) {
#pragma unroll
        for (int f = 0; f < 2; f++) bq[par][f] = *reinterpret_cast<const uint4 *>(slab + min(off + frag_off[f], last_off));
        off += step_off;
        q_c += adv_c;
        const bool wrap = q_c >= p.C;
        q_c -= wrap ? p.C : 0;
        off += wrap ? wrap_off : 0;
    };
    auto compute = [&](int set, int par) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
            if (DYN) dsum[j] += q_k < p.K ? dot_ones(bq[par][j]) : 0;
#pragma unroll
            for (int i = 0; i < 2; i++)
                acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, bq[par][j]), __builtin_bit_cast(i32x4, rp[set][i]),
                                                                  acc[j][i], 0, 0, 0);
        }
        q_k += kBK;
    };

    __syncthreads();
    read_q(0);
    // whole rounds without a branch, so that the weight loads stay counted exactly; then the rest
    int s = 0;
    for (; s + kSmallSets <= nk; s += kSmallSets) {
#pragma unroll
        for (int d = 0; d < kSmallSets; d++) {
            read_q((d + 1) & 1);
            compute(d, d & 1);
            load_p(d, s + d + kSmallSets);
        }
    }
#pragma unroll
    for (int d = 0; d < kSmallSets - 1; d++)
        if (s + d < nk) {
            read_q((d + 1) & 1);
            compute(d, d & 1);
        }
    __syncthreads();   // the hand-over reuses the slab's LDS
    conv_small_finish<EPI, DYN>(p, acc, dsum, chan, lds_acc, lds_sum, i0, j0, img, zd, zc);
}

}  // namespace hipc
