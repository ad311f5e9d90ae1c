// MatMulNBits for ONE activation row (M = 1, f32) on narrow outputs: the decode-step linears.
//
// Reference: crates/onnx-vulkan-core/src/shaders/matmul_nbits.rs:316-374 (the row kernel these
// shapes take there) and interp.rs:6429-6561. Same prepacked weight and the same arithmetic as
// mmnb_gemv_kernel (matmul_nbits.hip): nibbles become bf16 integers 128 + q, the activations are
// split into bf16 terms, products run on v_mfma_f32_16x16x32_bf16 and the bias and zero point
// leave per quantisation block: acc += scale * (dot - (128 + zp) * sum_k a_k).
//
// What differs is that everything here is built for latency, because these launches move a few MB
// and last microseconds: a launch in a replayed graph costs 1.6 us before its first instruction,
// an instruction of a workgroup whose wavefronts share a SIMD costs every one of them its issue
// slot, and every barrier costs the slowest wavefront's arrival. So
//   * nothing is persistent and nothing loops over column groups: a wavefront owns one 16-column
//     tile and at most four 128-k tiles of it, all of whose loads are issued before anything else;
//   * the bf16 terms of an activation sit in DIFFERENT ROWS of the matrix-core A operand (row 0 the
//     high term, row 1 the low one, row 2 the third) instead of in chained products: one MFMA per
//     32-k chunk whatever the number of terms, and the sum of the result rows is the dot product;
//   * the launch shape is given by the host (wavefronts along k, tiles per wavefront, k slices over
//     workgroups), so the kernel divides nothing at run time;
//   * the sum over the wavefronts that split k is taken by all 64 lanes of one wavefront (four
//     partials per lane and two cross-lane steps) instead of one lane after the other;
//   * a long k may be cut into slices over workgroups; each slice writes a partial output row and
//     the consumer adds the rows (the decoder's next kernel reads them anyway);
//   * the decoder's glue is folded in as prologues and epilogues that do no redundant work:
//       PRO 2  rmsnorm(x + rmsnorm(y)) with ONE workgroup-wide reduction (the second sum of
//              squares follows from sums that do not depend on the first norm's factor),
//       PRO 3  the flash-decoding join of the attention partials for the channels of the
//              workgroup's own k slice only,
//       PRO 4  an activation row that the producer already wrote as bf16 terms in operand order:
//              straight from memory into the operand registers, no LDS and no barrier,
//       EPI 1  gelu_tanh(gate) * up, written as such bf16 terms (the weight is prepacked with the
//              gate and up column tiles interleaved, so one workgroup holds both).
#include <hip/hip_fp16.h>

#include <algorithm>

#include "internal.h"
#include "lanes.h"
#include "prefetch.h"

namespace hipc {

typedef __attribute__((ext_vector_type(4))) float lf32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 lbf16x8;

// scales and (128 + zero point) bytes of one 16-column x 128-k tile column: SG groups, by buffer load
// (v_sc / v_zb: the lane's byte offsets inside a tile's scale and zero-point blocks; tl: the tile, scalar)
template <int SG>
struct ScaleVecLean;
template <>
struct ScaleVecLean<4> {
    float s[4];
    uint32_t z;
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t sc, __amdgpu_buffer_rsrc_t zb, uint32_t v_sc, uint32_t v_zb, uint32_t tl) {
        const auto v = __builtin_amdgcn_raw_buffer_load_b128(sc, (int)v_sc, (int)(tl * 256u), 0);
        s[0] = __uint_as_float(v[0]), s[1] = __uint_as_float(v[1]), s[2] = __uint_as_float(v[2]), s[3] = __uint_as_float(v[3]);
        z = __builtin_amdgcn_raw_buffer_load_b32(zb, (int)v_zb, (int)(tl * 64u), 0);
    }
};
template <>
struct ScaleVecLean<2> {
    float s[2];
    uint32_t z;
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t sc, __amdgpu_buffer_rsrc_t zb, uint32_t v_sc, uint32_t v_zb, uint32_t tl) {
        const auto v = __builtin_amdgcn_raw_buffer_load_b64(sc, (int)v_sc, (int)(tl * 128u), 0);
        s[0] = __uint_as_float(v[0]), s[1] = __uint_as_float(v[1]);
        z = __builtin_amdgcn_raw_buffer_load_b16(zb, (int)v_zb, (int)(tl * 32u), 0);
    }
};
template <>
struct ScaleVecLean<1> {
    float s[1];
    uint32_t z;
    __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t sc, __amdgpu_buffer_rsrc_t zb, uint32_t v_sc, uint32_t v_zb, uint32_t tl) {
        s[0] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(sc, (int)v_sc, (int)(tl * 64u), 0));
        z = __builtin_amdgcn_raw_buffer_load_b8(zb, (int)v_zb, (int)(tl * 16u), 0);
    }
};

__device__ __forceinline__ float lean_gelu_tanh(float v) {
    return 0.5f * v * (1.f + tanhf(0.79788456080286536f * fmaf(0.044715f, v * v * v, v)));
}

// ---- buffer loads: a uniform descriptor, a per-lane byte offset computed once and a SCALAR offset per
// load, so that asking for a tile, a partial row or a context chunk costs the vector unit nothing;
// a load whose per-lane offset lies past the end of the descriptor's range returns zeros (no clamping,
// no zero filling); the scalar offset is NOT part of that check and must stay inside the buffer
typedef unsigned int lu32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t lean_rsrc(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint4 lean_ld16(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    return __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0));
}
__device__ __forceinline__ void lean_ld8f(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff, float (&o)[8]) {
    const uint4 a = lean_ld16(r, voff, soff), b = lean_ld16(r, voff + 16u, soff);
    o[0] = __uint_as_float(a.x), o[1] = __uint_as_float(a.y), o[2] = __uint_as_float(a.z), o[3] = __uint_as_float(a.w);
    o[4] = __uint_as_float(b.x), o[5] = __uint_as_float(b.y), o[6] = __uint_as_float(b.z), o[7] = __uint_as_float(b.w);
}

// eight consecutive values -> NT operands of eight bf16 each: the nearest bf16 of the value, of the
// remainder, of the second remainder (every remainder is exact in f32)
typedef __attribute__((ext_vector_type(2))) __bf16 lbf16x2;
typedef __attribute__((ext_vector_type(2))) float lf32x2;
// The sum of the two bf16 halves of every word of NT operands (f32): what a product of the operands with ones
// would give, on the vector unit (one v_dot2c_f32_bf16 per word).
typedef __attribute__((ext_vector_type(2))) __bf16 lbf16pair;
template <int NT>
__device__ __forceinline__ float lean_term_sum(const uint4 (&op)[3]) {
    const lbf16pair ones = __builtin_bit_cast(lbf16pair, 0x3f803f80u);
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int t = 0; t < NT; t++) {
        s0 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(lbf16pair, op[t].x), ones, s0, false);
        s1 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(lbf16pair, op[t].y), ones, s1, false);
        s0 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(lbf16pair, op[t].z), ones, s0, false);
        s1 = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(lbf16pair, op[t].w), ones, s1, false);
    }
    return s0 + s1;
}
template <int NT>
__device__ __forceinline__ void lean_split8(const float (&av)[8], uint4 (&op)[3]) {
    uint32_t w[3][4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        float r0 = av[2 * q], r1 = av[2 * q + 1];
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const uint32_t pk = __builtin_bit_cast(uint32_t, __builtin_convertvector(lf32x2{r0, r1}, lbf16x2));
            w[t][q] = pk;
            if (t + 1 < NT) r0 -= __uint_as_float(pk << 16), r1 -= __uint_as_float(pk & 0xffff0000u);
        }
    }
#pragma unroll
    for (int t = 0; t < NT; t++) op[t] = make_uint4(w[t][0], w[t][1], w[t][2], w[t][3]);
}
// one value -> its NT bf16 terms (16 bits each)
template <int NT>
__device__ __forceinline__ void lean_split1(float v, uint16_t (&t)[3]) {
    float r = v;
#pragma unroll
    for (int e = 0; e < NT; e++) {
        const uint32_t pk = __builtin_bit_cast(uint32_t, __builtin_convertvector(lf32x2{r, 0.f}, lbf16x2));
        t[e] = (uint16_t)pk;
        if (e + 1 < NT) r -= __uint_as_float(pk << 16);
    }
}

// Phase time stamps (only in the library built with `make stamps`, which defines HIPC_PHASE_STAMPS): wavefront w of
// workgroup g of the last launch of an instance leaves the 100 MHz device clock at up to twelve points of the kernel in
// lean_stamps[slot][g][w][phase] (slot = PRO, or 1 for the gated epilogue); LEAN_STAMP_AFTER first waits for the value it
// names. hipc_debug_lean_stamps copies the table out. This is how the kernel's time was found to go into instruction
// issue, argument fetches and the first trip to memory rather than into moving the weights.
#ifdef HIPC_PHASE_STAMPS
__device__ unsigned long long lean_stamps[5 * 1024 * 8 * 12];
#define LEAN_STAMP(ph)                                                                                       \
    do {                                                                                                     \
        const unsigned long long t_ = (unsigned long long)wall_clock64();                                    \
        if ((threadIdx.x & 63) == 0 && st_wg < 1024 && (threadIdx.x >> 6) < 8)                               \
            lean_stamps[((st_slot * 1024 + st_wg) * 8 + (threadIdx.x >> 6)) * 12 + (ph)] = t_;               \
    } while (0)
#define LEAN_STAMP_AFTER(v, ph) do { asm volatile("" ::"v"(v)); LEAN_STAMP(ph); } while (0)
#else
#define LEAN_STAMP(ph)
#define LEAN_STAMP_AFTER(v, ph)
#endif
constexpr int kLeanMaxSlices = 4;   // partial rows a norm prologue adds up at most

// PRO: 0 plain row, 2 norm, 3 attention join, 4 row already split by the producer
// EPI: 0 store (a partial row per k slice), 1 gated GELU of a (gate, up) tile pair -> split row
// KT:  128-k tiles per wavefront (tile i of wavefront wk is k tile kt0 + wk + i WK of the slice)
//
// The vector unit is what these kernels wait for (a wavefront alone on its SIMD issues one vector
// instruction per four clocks, and every instruction of a prologue is on the critical path), so:
// addresses are scalar (buffer loads), nothing is divided at run time, and values are split into
// bf16 terms with the packed conversion. The sums over a quantisation block's activations that take
// the weights' +128 bias out again come from where they are cheapest: a prologue that holds eight
// consecutive values per thread (PRO 0, 2) adds its terms up with eight dot instructions and two
// steps inside a quad and leaves one sum per 32-k chunk in LDS (twelve matrix-core products per
// wavefront less at three tiles: 0.1 us per launch); the others (PRO 3: one value per lane, PRO 4:
// no prologue) multiply the operands with ones on the matrix cores.
template <int SG, int NT, int PRO, int EPI, int KT>
__global__ void __launch_bounds__(PRO == 0 ? 1024 : 512) mmnb_lean_kernel(const LeanArgs p) {
    extern __shared__ uint4 lean_smem[];
    constexpr int CPG = 4 / SG;  // 32-k chunks per scale group
#ifdef HIPC_PHASE_STAMPS
    const int st_slot = PRO + (EPI ? -1 : 0), st_wg = (int)(blockIdx.y * gridDim.x + blockIdx.x);
#endif
    // Every argument this instance uses is read here, in one batch: left to itself the compiler reads an argument
    // next to its first use, and each such group is a round trip of its own to memory (the scalar cache starts
    // every launch empty) in the middle of the kernel -- five of them before the norm prologue's first load.
    HIPC_ARG_NOW(p.Wq); HIPC_ARG_NOW(p.Sc); HIPC_ARG_NOW(p.Zb);
    HIPC_ARG_NOW(p.K); HIPC_ARG_NOW(p.N); HIPC_ARG_NOW(p.n_tiles); HIPC_ARG_NOW(p.n_cg);
    HIPC_ARG_NOW(p.WK); HIPC_ARG_NOW(p.WN); HIPC_ARG_NOW(p.slices); HIPC_ARG_NOW(p.nib_mask); HIPC_ARG_NOW(p.magic);
    if (PRO == 0) { HIPC_ARG_NOW(p.A); }
    if (PRO == 2) {
        HIPC_ARG_NOW(p.x); HIPC_ARG_NOW(p.yparts); HIPC_ARG_NOW(p.w_post); HIPC_ARG_NOW(p.w_in); HIPC_ARG_NOW(p.x_out);
        HIPC_ARG_NOW(p.y_slices); HIPC_ARG_NOW(p.eps);
    }
    if (PRO == 3) {
        HIPC_ARG_NOW(p.part_o); HIPC_ARG_NOW(p.part_ml); HIPC_ARG_NOW(p.pos);
        HIPC_ARG_NOW(p.lg_group); HIPC_ARG_NOW(p.lg_hd); HIPC_ARG_NOW(p.n_kv); HIPC_ARG_NOW(p.window);
    }
    if (PRO == 4) { HIPC_ARG_NOW(p.a_split); }
    if (EPI == 0) { HIPC_ARG_NOW(p.Y); }
    if (EPI == 1) { HIPC_ARG_NOW(p.h_split); }
    LEAN_STAMP(0);
    if (__builtin_expect((int)blockIdx.y >= p.slices, 0)) {   // a helper row: read ahead for the next launch, nothing else
        prefetch_for_next(p.pf, ((int)blockIdx.y - p.slices) * (int)gridDim.x + (int)blockIdx.x, p.pf.rows * (int)gridDim.x,
                          (int)blockIdx.y * (int)gridDim.x + (int)blockIdx.x, p.pf.sink);
        LEAN_STAMP(7);
        return;
    }
    LEAN_STAMP(8);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // PRO 2: the row's operands are asked for before anything else is worked out. They come from the launch
    // before this one, i.e. from memory and not from this XCD's L2, and the instructions between here and their
    // first use (index arithmetic, descriptors, the weight loads) take about as long to arrive as they do.
    // The wavefronts that hold items ask (the others would only spend issue slots); a thread past the end of the
    // row reads zeros and causes no traffic, and so does a partial row that does not exist (an empty descriptor).
    float x8[8], w8[8], wp8[8], part[kLeanMaxSlices][8];
    if (PRO == 2 && wave < ((min(p.WK * KT, p.n_cg) * 16 + 63) >> 6)) {
        const uint32_t row_bytes = (uint32_t)p.K * 4u, voff = (uint32_t)tid * 32u;
        const bool has_y = p.yparts != nullptr;
        const int ys = has_y ? p.y_slices : 0;
        lean_ld8f(lean_rsrc(p.x, row_bytes), voff, 0, x8);
        lean_ld8f(lean_rsrc(p.w_in, row_bytes), voff, 0, w8);
        lean_ld8f(lean_rsrc(has_y ? p.w_post : p.w_in, row_bytes), voff, 0, wp8);
#pragma unroll
        for (int s = 0; s < kLeanMaxSlices; s++) lean_ld8f(lean_rsrc(p.yparts + (size_t)s * p.K, s < ys ? row_bytes : 0u), voff, 0, part[s]);
        __builtin_amdgcn_sched_barrier(0);
    }
    LEAN_STAMP(9);
    // wave = wn * WK + wk without a division: WK is at most 16 and WN at most 4
    int wn = 0, wk = wave;
    while (wk >= p.WK) wk -= p.WK, wn++;
    const int i16 = lane & 15, g4 = lane >> 4;
    const int slice = blockIdx.y;
    const int slice_tiles = p.WK * KT;
    const int kt0 = slice * slice_tiles;                  // first k tile of the workgroup
    const int nch = min(slice_tiles, p.n_cg - kt0) * 4;   // 32-k chunks this workgroup multiplies
    const int nt_raw = blockIdx.x * p.WN + wn;
    const int nt = min(nt_raw, p.n_tiles - 1);

    // ---- every load of this wavefront's weight tiles at once -- but AFTER the prologue's own loads:
    // loads return in the order they were issued, so a prologue that waits for its activations
    // would otherwise wait for the (cold, far larger) weight tiles too. A tile past the end of k (the
    // last wavefronts of a ragged slice) repeats the wavefront's first tile and counts for nothing.
    uint4 wq[KT];
    ScaleVecLean<SG> sv[KT];
    int tile_in_slice[KT];
    float tile_live[KT];   // 1 or 0: multiplies the tile's scales where they are used (zeroing the loaded registers here would wait for the loads)
    const uint32_t tiles_total = (uint32_t)p.n_tiles * (uint32_t)p.n_cg;
    const __amdgpu_buffer_rsrc_t r_wq = lean_rsrc(p.Wq, tiles_total * 1024u);
    const __amdgpu_buffer_rsrc_t r_sc = lean_rsrc(p.Sc, tiles_total * 64u * SG);
    const __amdgpu_buffer_rsrc_t r_zb = lean_rsrc(p.Zb, tiles_total * 16u * SG);
    const uint32_t v_wq = (uint32_t)lane * 16u, v_sc = (uint32_t)i16 * 4u * SG, v_zb = (uint32_t)i16 * SG;
    auto load_weights = [&]() {
#pragma unroll
        for (int i = 0; i < KT; i++) {
            const int kt = kt0 + wk + i * p.WK;
            const bool live = kt < p.n_cg;
            tile_live[i] = live ? 1.f : 0.f;
            tile_in_slice[i] = live ? wk + i * p.WK : min(wk, p.n_cg - 1 - kt0);
            const uint32_t tl = (uint32_t)nt * (uint32_t)p.n_cg + (uint32_t)(kt0 + tile_in_slice[i]);   // scalar
            wq[i] = lean_ld16(r_wq, v_wq, tl * 1024u);
            sv[i].load(r_sc, r_zb, v_sc, v_zb, tl);
        }
    };
    // Marks the point where values asked for in (wave-uniform) branches above are first needed: the
    // compiler may otherwise pull the arithmetic that consumes a load into the branch that issued it,
    // which turns one memory round trip into one per branch.
#define LEAN_NEEDED_HERE(v) HIPC_PIN_VGPR(v)

    uint4 *As = lean_smem;                                                     // [nch][NT][4] operands
    float *red = reinterpret_cast<float *>(As + (size_t)slice_tiles * 4 * NT * 4);   // [WN][16 columns][16 k wavefronts]; before that the norm's partial sums
    // The sums of the split activations over every 32-k chunk, which take the weights' +128 bias and the zero
    // points out again, are left here by the prologue that splits the row (four per tile, read back with one
    // broadcast load). A row that arrives already split (PRO 4) has no prologue, and the attention join (PRO 3)
    // holds one value per lane, whose sums over 32 lanes cost more than they save: those two take the sums from
    // a second product against ones.
    constexpr bool kSumsAhead = PRO == 0 || PRO == 2;
    float *bsum = red + (size_t)p.WN * 256;   // [slice tiles][4 chunks]
    const int nthreads = blockDim.x;
    const int kbase = kt0 * 128;
    const int nitems = nch * 4;   // one item = 8 consecutive k of the row = one operand per term

    // item -> LDS: chunk item / 4, k group item % 4; the terms of a chunk are 64 bytes apart
    auto put_item = [&](int item, const float (&av)[8]) {
        uint4 op[3];
        lean_split8<NT>(av, op);
        uint4 *dst = As + (size_t)(item >> 2) * NT * 4 + (item & 3);
#pragma unroll
        for (int t = 0; t < NT; t++) dst[4 * t] = op[t];
        // the four items of a chunk sit in the four lanes of a quad (the number of items is a multiple of four)
        float cs = lean_term_sum<NT>(op);
        cs += lean_dpp<0xB1>(cs);
        cs += lean_dpp<0x4E>(cs);
        if ((item & 3) == 0) bsum[item >> 2] = cs;
    };

    if (PRO == 0) {
        const __amdgpu_buffer_rsrc_t r_a = lean_rsrc(p.A, (uint32_t)p.K * 4u);   // past K: zeros
        float first[8];
        lean_ld8f(r_a, (uint32_t)(kbase * 4 + tid * 32), 0, first);   // this thread's first item, ahead of the weights
        load_weights();
        if (tid < nitems) put_item(tid, first);
        for (int item = tid + nthreads; item < nitems; item += nthreads) {
            float av[8];
            lean_ld8f(r_a, (uint32_t)(kbase * 4 + item * 32), 0, av);
            put_item(item, av);
        }
        __syncthreads();
    } else if (PRO == 2) {
        // x' = x + rmsnorm(y, w_post) with y = the sum of y_slices partial rows (x' = x without y);
        // row = rmsnorm(x', w_in). The workgroup covers the whole row (one k slice), one item per
        // thread of the first wavefronts; the others only meet the barriers. Four sums that do not
        // depend on each other give both norm factors after ONE reduction:
        //   sum y^2 -> f1;   sum x'^2 = sum x^2 + 2 f1 sum(x y w) + f1^2 sum((y w)^2) -> f2.
        // Every load is issued before the first sum: one memory round trip. Only the partial rows that
        // exist are asked for; items past K read zeros.
        const int pw = (nitems + 63) >> 6;  // wavefronts that hold items
        float yw8[8];
        float4 *red4 = reinterpret_cast<float4 *>(red);
        load_weights();
        if (wave < pw) {
            LEAN_STAMP(1);
#pragma unroll
            for (int s = 0; s < kLeanMaxSlices; s++)
#pragma unroll
                for (int i = 0; i < 8; i++) LEAN_NEEDED_HERE(part[s][i]);
            LEAN_STAMP(2);
            float s_yy = 0.f, s_xx = 0.f, s_xyw = 0.f, s_ywyw = 0.f;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float y = part[0][i];
#pragma unroll
                for (int s = 1; s < kLeanMaxSlices; s++) y += part[s][i];
                yw8[i] = y * wp8[i];
                s_yy = fmaf(y, y, s_yy), s_xx = fmaf(x8[i], x8[i], s_xx);
                s_xyw = fmaf(x8[i], yw8[i], s_xyw), s_ywyw = fmaf(yw8[i], yw8[i], s_ywyw);
            }
            s_yy = lean_row_sum(s_yy), s_xx = lean_row_sum(s_xx), s_xyw = lean_row_sum(s_xyw), s_ywyw = lean_row_sum(s_ywyw);
            if (i16 == 0) red4[wave * 4 + g4] = make_float4(s_yy, s_xx, s_xyw, s_ywyw);
        }
        __syncthreads();
        if (wave < pw) {
            // lane l takes partial l of the pw * 4 row sums (at most 32: two rows of lanes)
            const float4 v = lane < pw * 4 ? red4[lane] : make_float4(0.f, 0.f, 0.f, 0.f);
            const float r_yy = lean_row_sum(v.x), r_xx = lean_row_sum(v.y), r_xyw = lean_row_sum(v.z), r_ywyw = lean_row_sum(v.w);
            const float t_yy = lean_lane(r_yy, 0) + lean_lane(r_yy, 16), t_xx = lean_lane(r_xx, 0) + lean_lane(r_xx, 16);
            const float t_xyw = lean_lane(r_xyw, 0) + lean_lane(r_xyw, 16), t_ywyw = lean_lane(r_ywyw, 0) + lean_lane(r_ywyw, 16);
            const float invK = 1.f / (float)p.K;
            const float f1 = rsqrtf(t_yy * invK + p.eps);
            const float sq2 = fmaf(f1 * f1, t_ywyw, fmaf(2.f * f1, t_xyw, t_xx));
            const float f2 = rsqrtf(fmaxf(sq2, 0.f) * invK + p.eps);
            float av[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                x8[i] = fmaf(yw8[i], f1, x8[i]);
                av[i] = x8[i] * f2 * w8[i];
            }
            if (p.x_out && blockIdx.x == 0 && tid * 8 < p.K) {
                reinterpret_cast<float4 *>(p.x_out + tid * 8)[0] = make_float4(x8[0], x8[1], x8[2], x8[3]);
                reinterpret_cast<float4 *>(p.x_out + tid * 8)[1] = make_float4(x8[4], x8[5], x8[6], x8[7]);
            }
            if (tid < nitems) put_item(tid, av);
        }
        __syncthreads();  // also: `red` is free for the k reduction
        LEAN_STAMP(3);
    } else if (PRO == 3) {
        // The channels of this workgroup's k slice, joined over the live context chunks of their
        // head: sum_s e_s o_s / sum_s e_s l_s with e_s = exp(m_s - max m). A wavefront's 64 channels
        // belong to one head (head_dim is a power of two >= 64, as is the group size: shifts, no
        // division). The first sixteen chunks' values of the lane's channel are asked for before
        // anything is known about the position (the partials are finite wherever they were never
        // written: they were cleared once; a chunk that is not live has weight zero), the others once
        // the number of live chunks is there; the weights are formed on the vector unit (lane s holds
        // chunk s) and read lane by lane as scalars.
        static_assert(kAttnSplits == 64, "one lane per chunk");
        const int G = 1 << p.lg_group, GH = G << p.lg_hd;
        const int slice_ch = nch * 32;
        const uint32_t chunk_bytes = (uint32_t)GH * 4u;
        const __amdgpu_buffer_rsrc_t r_o = lean_rsrc(p.part_o, (uint32_t)p.n_kv * kAttnSplits * chunk_bytes);
        const __amdgpu_buffer_rsrc_t r_ml = lean_rsrc(p.part_ml, (uint32_t)p.n_kv * kAttnSplits * (uint32_t)G * 8u);
        bool weights_asked = false;
        for (int c0 = wave * 64; c0 < slice_ch; c0 += nthreads) {   // wave-uniform
            const int h = (kbase + c0) >> p.lg_hd, kvh = h >> p.lg_group, g = h & (G - 1);
            const uint32_t v_o = (uint32_t)(kbase + c0 + lane - kvh * GH) * 4u;      // the lane's channel inside its kv head's block
            const uint32_t s_o = (uint32_t)kvh * kAttnSplits * chunk_bytes;
            float f[kAttnSplits];
#pragma unroll
            for (int j = 0; j < 16; j++) f[j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r_o, (int)v_o, (int)(s_o + (uint32_t)j * chunk_bytes), 0));
            const uint2 ml_raw = __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(r_ml, (int)((uint32_t)lane * (uint32_t)G * 8u),
                                                                                              (int)(((uint32_t)kvh * kAttnSplits * G + g) * 8u), 0));
            const int total = *p.pos + 1;
            const int live = attn_live_chunks(attn_span(total, p.window));
#pragma unroll
            for (int q = 1; q < 4; q++) {
                if (q * 16 < live) {   // wave-uniform: a quarter of the chunks at a time
#pragma unroll
                    for (int j = 0; j < 16; j++)
                        f[q * 16 + j] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r_o, (int)v_o, (int)(s_o + (uint32_t)(q * 16 + j) * chunk_bytes), 0));
                } else {
#pragma unroll
                    for (int j = 0; j < 16; j++) f[q * 16 + j] = 0.f;
                }
            }
            if (!weights_asked) load_weights(), weights_asked = true;
            LEAN_STAMP(1);
            float mx = __uint_as_float(ml_raw.x), ls = __uint_as_float(ml_raw.y);
            LEAN_NEEDED_HERE(mx);
#pragma unroll
            for (int j = 0; j < kAttnSplits; j++) LEAN_NEEDED_HERE(f[j]);
            LEAN_STAMP(2);
            const bool on = lane < live;
            const float m = lean_wave_max(on ? mx : -3.0e38f);
            const float e = on ? __expf(mx - m) : 0.f;
            const float l = lean_wave_sum(on ? ls * e : 0.f);
            float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
            for (int j = 0; j < kAttnSplits; j += 4) {   // chunks past the last: weight 0
                o0 = fmaf(f[j], lean_lane(e, j), o0);
                o1 = fmaf(f[j + 1], lean_lane(e, j + 1), o1);
                o2 = fmaf(f[j + 2], lean_lane(e, j + 2), o2);
                o3 = fmaf(f[j + 3], lean_lane(e, j + 3), o3);
            }
            const float val = kbase + c0 + lane < p.K ? ((o0 + o1) + (o2 + o3)) / l : 0.f;
            // this lane's value is element (c0 + lane) of the slice: 16-bit stores into operand order
            uint16_t t[3];
            lean_split1<NT>(val, t);
            const int el = c0 + lane;
            uint16_t *dst = reinterpret_cast<uint16_t *>(As + (size_t)(el >> 5) * NT * 4 + ((el >> 3) & 3)) + (el & 7);
#pragma unroll
            for (int q = 0; q < NT; q++) dst[32 * q] = t[q];   // the next term's operands are 4 x 16 bytes on
        }
        if (!weights_asked) load_weights();
        __syncthreads();
        LEAN_STAMP(3);
    } else {
        load_weights();
        LEAN_STAMP(1);
    }

    // ---- products, phase by phase so that nothing waits for its neighbour: every operand first
    // (from LDS, or for PRO 4 straight from the row the producer wrote), then every unpack and
    // matrix-core product (independent accumulators), then the per-block sums. The operand rows of a
    // lane: every group of four rows of the 16-row A operand holds the NT terms (row 4 q + t is term
    // t), so ONE product per chunk multiplies all terms and the result rows 0 .. NT-1 add up to the dot
    // product; where no prologue left the chunks' sums, a second product against ones gives them.
    const int term = min(i16 & 3, NT - 1);
    const uint32_t nib_mask = p.nib_mask;
    uint32_t magic;
    HIPC_VGPR_FROM_SGPR(magic, p.magic);
    // (with three terms and four tiles the sixteen operands read ahead do not fit the 128 registers a
    // wavefront of a 1024-thread workgroup may hold: that instance reads a tile's operands when it multiplies it)
    constexpr bool kOperandsAhead = !(NT == 3 && KT == 4);
    uint4 aop[KT][4];
    float4 bs[KT];
    const uint4 *a_lane = As + term * 4 + g4;
    if (PRO == 4) {
        const __amdgpu_buffer_rsrc_t r_a = lean_rsrc(p.a_split, (uint32_t)p.n_cg * 4u * NT * 64u);
        const uint32_t v_a = (uint32_t)(term * 4 + g4) * 16u;
#pragma unroll
        for (int i = 0; i < KT; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) aop[i][j] = lean_ld16(r_a, v_a, (uint32_t)((kt0 + tile_in_slice[i]) * 4 + j) * (NT * 64u));
    } else if (kOperandsAhead) {
#pragma unroll
        for (int i = 0; i < KT; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) aop[i][j] = a_lane[(size_t)(tile_in_slice[i] * 4 + j) * NT * 4];
        if (kSumsAhead) {
#pragma unroll
            for (int i = 0; i < KT; i++) bs[i] = reinterpret_cast<const float4 *>(bsum)[tile_in_slice[i]];
        }
    }
    LEAN_STAMP_AFTER(aop[KT - 1][3].x, 4);
    const uint32_t one2 = 0x3f803f80u;   // bf16 1.0 twice
    const lbf16x8 ones = __builtin_bit_cast(lbf16x8, make_uint4(one2, one2, one2, one2));
    lf32x4 d[KT][SG], e[KT][SG];
    float acc = 0.f;
    auto multiply_tile = [&](int i) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t word = j == 0 ? wq[i].x : j == 1 ? wq[i].y : j == 2 ? wq[i].z : wq[i].w;
            const uint4 bw = make_uint4((word & nib_mask) | magic, ((word >> 4) & nib_mask) | magic,
                                        ((word >> 8) & nib_mask) | magic, ((word >> 12) & nib_mask) | magic);
            const int g = j / CPG;
            const bool first = (j % CPG) == 0;
            const lbf16x8 a = __builtin_bit_cast(lbf16x8, aop[i][j]);
            d[i][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(lbf16x8, bw), first ? lf32x4{0.f, 0.f, 0.f, 0.f} : d[i][g], 0, 0, 0);
            if (!kSumsAhead) e[i][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, ones, first ? lf32x4{0.f, 0.f, 0.f, 0.f} : e[i][g], 0, 0, 0);
        }
    };
    auto fold_tile = [&](int i) {
#pragma unroll
        for (int g = 0; g < SG; g++) {
            const float dsum = NT == 3 ? (d[i][g][0] + d[i][g][1]) + d[i][g][2] : d[i][g][0] + d[i][g][1];
            float asg;
            if (!kSumsAhead) asg = NT == 3 ? (e[i][g][0] + e[i][g][1]) + e[i][g][2] : e[i][g][0] + e[i][g][1];
            else if (SG == 4) asg = g == 0 ? bs[i].x : g == 1 ? bs[i].y : g == 2 ? bs[i].z : bs[i].w;
            else if (SG == 2) asg = g == 0 ? bs[i].x + bs[i].y : bs[i].z + bs[i].w;
            else asg = (bs[i].x + bs[i].y) + (bs[i].z + bs[i].w);
            const float zb = (float)((sv[i].z >> (8 * g)) & 0xffu);
            acc = fmaf(sv[i].s[g] * tile_live[i], fmaf(-zb, asg, dsum), acc);
        }
    };
    if (kOperandsAhead) {
#pragma unroll
        for (int i = 0; i < KT; i++) multiply_tile(i);
#pragma unroll
        for (int i = 0; i < KT; i++) fold_tile(i);
    } else {
        // one tile after the other, and nothing moved across a tile's end: a tile's operands and its 32
        // result registers are dead before the next tile's are live
#pragma unroll
        for (int i = 0; i < KT; i++) {
            if (PRO != 4) {
#pragma unroll
                for (int j = 0; j < 4; j++) aop[i][j] = a_lane[(size_t)(tile_in_slice[i] * 4 + j) * NT * 4];
                if (kSumsAhead) bs[i] = reinterpret_cast<const float4 *>(bsum)[tile_in_slice[i]];
            }
            multiply_tile(i);
            fold_tile(i);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- the sum over the wavefronts that split k: column n's partials sit side by side, and every
    // lane of the finishing wavefront reads its column's slots and adds the first WK in order
    LEAN_STAMP_AFTER(acc, 5);
    const bool through_lds = p.WK > 1 || EPI == 1;   // the gated epilogue's two tiles meet in LDS even when k is not split
    if (through_lds) {
        if (g4 == 0) red[(wn * 16 + i16) * 16 + wk] = acc;
        __syncthreads();
    }
    LEAN_STAMP(6);
    const bool reducer = wk == 0 && (EPI == 0 || wn == 0);
    if (!reducer) return;
    auto reduce_tile = [&](int tile_wn, float own) {
        if (!through_lds) return own;
        const float4 *col = reinterpret_cast<const float4 *>(red + (tile_wn * 16 + i16) * 16);
        float t = 0.f;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            if (q * 4 < p.WK) {   // wave-uniform
                const float4 v = col[q];
                t += v.x;
                t += q * 4 + 1 < p.WK ? v.y : 0.f;
                t += q * 4 + 2 < p.WK ? v.z : 0.f;
                t += q * 4 + 3 < p.WK ? v.w : 0.f;
            }
        }
        return t;
    };
    if (EPI == 0) {
        const float total = reduce_tile(wn, acc);
        const int n = nt_raw * 16 + i16;
        if (g4 == 0 && nt_raw < p.n_tiles && n < p.N) p.Y[(size_t)slice * p.N + n] = total;
    } else {
        // tiles 2 b and 2 b + 1 of the interleaved weight are gate and up columns 16 b .. 16 b + 15.
        // (the up tile's sums belong to other wavefronts: both tiles are read back from LDS)
        const float gate = reduce_tile(0, 0.f), up = reduce_tile(1, 0.f);
        const int n = blockIdx.x * 16 + i16;   // WN == 2: one (gate, up) pair per workgroup; n indexes the gated row, the next product's k
        const float h = lean_gelu_tanh(gate) * up;
        uint16_t t[3];
        lean_split1<NT>(h, t);
        if (g4 == 0) {
            uint16_t *dst = reinterpret_cast<uint16_t *>(p.h_split + (size_t)(n >> 5) * NT * 4 + ((n >> 3) & 3)) + (n & 7);
#pragma unroll
            for (int q = 0; q < NT; q++) dst[32 * q] = t[q];
        }
    }
    LEAN_STAMP(7);
}

}  // namespace hipc

#ifdef HIPC_PHASE_STAMPS
extern "C" int hipc_debug_lean_stamps(void *dst, size_t bytes) {
    return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(hipc::lean_stamps), bytes, 0, hipMemcpyDeviceToHost);
}
#endif

using namespace hipc;

namespace {

template <int SG, int NT, int PRO, int EPI>
void lean_launch_one(const LeanArgs &a, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
    switch (a.KT) {
        case 1: hipLaunchKernelGGL((mmnb_lean_kernel<SG, NT, PRO, EPI, 1>), grid, block, lds, s, a); break;
        case 2: hipLaunchKernelGGL((mmnb_lean_kernel<SG, NT, PRO, EPI, 2>), grid, block, lds, s, a); break;
        case 3: hipLaunchKernelGGL((mmnb_lean_kernel<SG, NT, PRO, EPI, 3>), grid, block, lds, s, a); break;
        default: hipLaunchKernelGGL((mmnb_lean_kernel<SG, NT, PRO, EPI, 4>), grid, block, lds, s, a); break;
    }
}

template <int SG, int NT>
int lean_launch_pro(hipc_ctx *ctx, const LeanArgs &a, int pro, int epi, dim3 grid, dim3 block, size_t lds) {
    hipStream_t s = ctx->stream;
    if (pro == 0 && epi == 0) lean_launch_one<SG, NT, 0, 0>(a, grid, block, lds, s);
    else if (pro == 2 && epi == 0 && NT == 2) lean_launch_one<SG, 2, 2, 0>(a, grid, block, lds, s);
    else if (pro == 2 && epi == 1 && NT == 2) lean_launch_one<SG, 2, 2, 1>(a, grid, block, lds, s);
    else if (pro == 3 && epi == 0 && NT == 2) lean_launch_one<SG, 2, 3, 0>(a, grid, block, lds, s);
    else if (pro == 4 && epi == 0 && NT == 2) lean_launch_one<SG, 2, 4, 0>(a, grid, block, lds, s);
    else return fail(ctx, HIPC_ERR_INVALID, "MatMulNBits lean gemv: no instance for prologue %d, epilogue %d, %d terms", pro, epi, NT);
    HIPC_LAUNCHED(ctx);
    return HIPC_OK;
}

}  // namespace

bool hipc::lean_plan(hipc_ctx *ctx, const hipc_nbits_weight *w, int slices, int WN, LeanPlan *out, int max_waves, bool short_in_three) {
    if (w->K % 8 != 0 || slices < 1 || WN < 1 || WN > max_waves) return false;
    const int per_slice = (w->n_cg + slices - 1) / slices;   // k tiles a workgroup covers
    // k tiles per wavefront: the fewest that fit the wavefronts a workgroup may have. short_in_three: three when
    // the slice is short (a workgroup of three wavefronts then holds the row and all of them take part in a norm or
    // join prologue; the plain-row prologue is over sooner than two more tiles' products: 1152 -> 1536 as nine
    // wavefronts of one tile each, 4.25 against 4.36 us over a token's stand-alone launches)
    const int max_wk = max_waves / WN;
    int KT = (per_slice + max_wk - 1) / max_wk;
    if (ctx->tune.gemv_t >= 1 && ctx->tune.gemv_t <= 4) KT = std::max(KT, ctx->tune.gemv_t);
    else if (short_in_three && per_slice <= 12 && per_slice >= 3) KT = std::max(KT, 3);
    if (KT > 4) return false;
    LeanPlan pl{};
    pl.KT = KT, pl.WK = (per_slice + KT - 1) / KT, pl.WN = WN, pl.slices = slices;
    *out = pl;
    return true;
}

PrefetchArgs hipc::lean_prefetch_of(const hipc_nbits_weight *w, const LeanPlan &pl, int rows, uint32_t *sink) {
    PrefetchArgs pf;
    pf.kind = 1, pf.rows = rows, pf.sink = sink;
    pf.wq = w->Wq, pf.sc = w->Sc, pf.zb = w->Zb;
    pf.gx = (int)ceil_div(w->n_tiles, pl.WN), pf.gy = pl.slices, pf.WN = pl.WN, pf.slice_tiles = pl.WK * pl.KT;
    pf.n_cg = w->n_cg, pf.n_tiles = w->n_tiles, pf.SG = w->SG;
    return pf;
}

int hipc::lean_gemv(hipc_ctx *ctx, const hipc_nbits_weight *w, const LeanPlan &pl, LeanArgs a, int pro, int epi, int NT) {
    a.Wq = w->Wq, a.Sc = w->Sc, a.Zb = w->Zb;
    a.K = (int)w->K, a.N = (int)w->N, a.n_tiles = w->n_tiles, a.n_cg = w->n_cg;
    a.WK = pl.WK, a.KT = pl.KT, a.WN = pl.WN, a.slices = pl.slices;
    a.nib_mask = 0x000f000fu, a.magic = 0x43004300u;
    HIPC_REQUIRE(ctx, pl.WK >= 1 && pl.WK <= 16 && pl.KT >= 1 && pl.KT <= 4 && pl.WN >= 1 && pl.WK * pl.WN <= 16 &&
                          pl.slices >= 1 && (int64_t)pl.slices * pl.WK * pl.KT >= w->n_cg,
                 "MatMulNBits lean gemv: launch plan %d x %d x %d, %d slices does not cover %d k tiles", pl.WK, pl.KT, pl.WN,
                 pl.slices, w->n_cg);
    HIPC_REQUIRE(ctx, w->K % 8 == 0, "MatMulNBits lean gemv: K must be a multiple of 8");
    HIPC_REQUIRE(ctx, epi == 0 || (pl.WN == 2 && w->n_tiles % 2 == 0 && pl.slices == 1), "MatMulNBits lean gemv: the gated epilogue needs tile pairs and the whole k");
    HIPC_REQUIRE(ctx, pro != 2 || pl.slices == 1, "MatMulNBits lean gemv: the norm prologue needs the whole row in one workgroup");
    const int slice_tiles = pl.WK * pl.KT;
    const int threads = 64 * pl.WK * pl.WN;
    HIPC_REQUIRE(ctx, pro != 2 || slice_tiles * 16 <= threads, "MatMulNBits lean gemv: the norm prologue needs one item per thread");
    HIPC_REQUIRE(ctx, pro != 2 || a.y_slices <= kLeanMaxSlices, "MatMulNBits lean gemv: at most %d partial rows", kLeanMaxSlices);
    HIPC_REQUIRE(ctx, pro == 0 || threads <= 512, "MatMulNBits lean gemv: at most eight wavefronts with a prologue");
    size_t lds = (size_t)slice_tiles * 4 * NT * 4 * 16;
    lds += (size_t)pl.WN * 16 * 16 * 4;   // reduction area [WN][16][16]; the norm's partial sums [16][4][4] fit its first KiB
    lds += (size_t)slice_tiles * 16;          // the chunks' activation sums
    HIPC_REQUIRE(ctx, lds <= 64 * 1024, "MatMulNBits lean gemv: LDS plan of %zu bytes does not fit", lds);
    if (a.pf.kind == 0) a.pf.rows = 0;
    const dim3 grid((unsigned)ceil_div(w->n_tiles, pl.WN), (unsigned)(pl.slices + a.pf.rows));
    const dim3 block((unsigned)threads);
    switch (w->SG) {
        case 4: return NT == 3 ? lean_launch_pro<4, 3>(ctx, a, pro, epi, grid, block, lds) : lean_launch_pro<4, 2>(ctx, a, pro, epi, grid, block, lds);
        case 2: return NT == 3 ? lean_launch_pro<2, 3>(ctx, a, pro, epi, grid, block, lds) : lean_launch_pro<2, 2>(ctx, a, pro, epi, grid, block, lds);
        default: return NT == 3 ? lean_launch_pro<1, 3>(ctx, a, pro, epi, grid, block, lds) : lean_launch_pro<1, 2>(ctx, a, pro, epi, grid, block, lds);
    }
}
