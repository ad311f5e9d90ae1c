// The int8 matrix product for shapes with hundreds of tiles (MatMulInteger / QLinearMatMul, A with
// whole 128-byte k stages and 16-byte aligned rows): the constant operand never touches LDS.
//
// The prepacked B is fragment-major (qfrag_offset): the 16 bytes a lane feeds the matrix core for a
// 32-column x 32-k fragment lie at fragment base + 16 lane, so a wavefront reads a B fragment with ONE
// fully coalesced 1 KB load straight into the operand registers. Each wavefront loads the fragments
// of its own columns per 32-k step, three steps ahead of their use (a ring of four register sets);
// only A goes through LDS (memory -> registers -> LDS, sign flip on the way, pitch 144: conflict-free
// 128-bit reads). The wavefronts that share columns ask for the same B lines; the later requests are
// served by the CU's L1. A tile has eight wavefronts, two per SIMD: a wavefront that waits for
// memory or at the stage's barrier leaves the matrix core to its neighbour.
//
// What this replaced, and what was measured on the way (8192^3, random bytes, one MI355X):
//   * both operands through LDS, 256x256 tile, four wavefronts of 128x128 (one per SIMD): 585-609 us.
//     LDS reads saturate at about 147 bytes per nanosecond and CU (a loop of conflict-free
//     ds_read_b128 on all 256 CUs) and that kernel needed 96 of them, so LDS looked like the bound;
//   * the same tile and wavefronts with B straight from memory (half the LDS traffic): 576-595 us, and
//     with every workgroup reading the SAME tile (all loads cache hits): 569 us -- neither LDS nor
//     the memory system is what it waits for;
//   * eight wavefronts of 128x64 (this kernel): 541-587 us box to box (2.03-1.87 POPS), the fixed cost
//     per call (prologues, 268 MB of int32 output) down from 93 to 47 us, the k loop at 2.04-2.13 POPS
//     in both. Counters: the chip holds 1.66-1.77 GHz under this load (GRBM_GUI_ACTIVE / duration),
//     where 100 % matrix-core occupancy would be 3.5 POPS; SQ_VALU_MFMA_BUSY_CYCLES is 62 % of the
//     SIMD cycles here against 55 % for the LDS-staged kernel.
// The 128x128 tile of the same kernel serves shapes with too few 256x256 tiles to fill the chip:
// 1000 x 1024 x 4096 takes 10.0 us (14.1 on the k-split 64x64 kernel), 4096 x 1024 x 4096 27.5 us
// (51.2), 2048^3 15.2 us (19.8).
#pragma once

#include "int8_gemm.h"

namespace hipc {

constexpr int kBigTile = 256;
constexpr size_t bd_lds(int tile) { return 2 * (size_t)tile * kPitch + tile * sizeof(int); }
constexpr int kBdAhead = 3;   // k steps between a B fragment's load and its use

// T: the tile's edge, 256 or 128 (128 when 256 x 256 tiles would leave most CUs without one).
// W wavefronts, 2 over the rows x W / 2 over the columns: 4 (one per SIMD) or 8 (two per SIMD: a wavefront that
// waits for memory or at the barrier leaves the matrix core to its neighbour).
template <int EPI, bool DYN, int T, int W>
__global__ void __launch_bounds__(64 * W) int8_gemm_bdirect_kernel(const GemmArgs p) {
    constexpr int WN = W / 2;                            // wavefronts over the columns (2 over the rows)
    constexpr int FI = T / 64, FJ = T / (32 * WN);       // 32x32 accumulators per wavefront
    constexpr int kCh = T * (kBK / 16) / (64 * W);       // 16-byte chunks of an A slab per thread
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
    uint8_t *lds_p = lds_raw;                                                  // [2][256 * kPitch]
    int *lds_sum = reinterpret_cast<int *>(lds_raw + 2 * T * kPitch);   // [256]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int r32 = lane & 31, kg = lane >> 5;

    const int tiles_x = (p.J + T - 1) / T, tiles_y = (p.I + T - 1) / T;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int rows_per = (tiles_y + p.xcd_rows - 1) / p.xcd_rows, cols_per = (tiles_x + p.xcd_cols - 1) / p.xcd_cols;
    const int ty = (xcd / p.xcd_cols) * rows_per + idx / cols_per, tx = (xcd % p.xcd_cols) * cols_per + idx % cols_per;
    if (idx >= rows_per * cols_per || ty >= tiles_y || tx >= tiles_x) return;
    const int i0 = ty * T, j0 = tx * T;

    const int zd = (p.host_zp ? p.dyn_zp_value : zp_byte(p.dyn_zp, p.dyn_signed)) - p.dyn_shift;
    const int zc = (p.host_zp ? p.const_zp_value : zp_byte(p.const_zp, p.const_signed)) - p.const_shift;
    const uint32_t flip = p.dyn_shift ? 0x80808080u : 0u;

    // A: chunk c = tid + 256 u of a 256-row slab: row c / 8, 16-byte column c % 8 (whole 128-byte lines per row)
    uint32_t p_off[kCh], l_off[kCh];
#pragma unroll
    for (int u = 0; u < kCh; u++) {
        const int c = tid + 64 * W * u, row = c >> 3, kc = c & 7;
        p_off[u] = (uint32_t)min(i0 + row, p.I - 1) * (uint32_t)p.K + kc * 16;   // rows past I: clamped, never stored
        l_off[u] = row * kPitch + kc * 16;
    }
    // B: fragment j of this wavefront's 128 columns at k step g lies g KB behind the fragment column's start
    const int j_last = (p.J + kBN - 1) / kBN * kBN - 1;   // B is packed in whole 128-column tiles
    uint32_t q_off[FJ];
#pragma unroll
    for (int j = 0; j < FJ; j++) q_off[j] = qfrag_offset(min(j0 + wn * FJ * 32 + j * 32, j_last - 31), 0, p.K_pad) + lane * 16;
    const __amdgpu_buffer_rsrc_t rsrc_p = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(p.P), 0, (int)((uint32_t)p.I * (uint32_t)p.K), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_q = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t *>(p.Q), 0, (int)((uint32_t)(j_last + 1) * (uint32_t)p.K_pad), 0x00020000);
    const int nk = p.K_pad / kBK, nsteps = nk * 4;

    u32x4 ra[kCh];          // the next stage of A between memory and LDS
    u32x4 rb[4][FJ];        // B fragments of four consecutive k steps: a ring
    auto load_a = [&](int stage) {
#pragma unroll
        for (int u = 0; u < kCh; u++) ra[u] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_p, p_off[u], stage * kBK, 0);
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int u = 0; u < kCh; u++) *reinterpret_cast<u32x4 *>(lds_p + buf * T * kPitch + l_off[u]) = ra[u] ^ flip;
    };
    auto load_b = [&](int slot, int g) {   // a step past the end reloads the last one (cached, never multiplied)
        const int gc = min(g, nsteps - 1);
#pragma unroll
        for (int j = 0; j < FJ; j++) rb[slot][j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_q, q_off[j], gc * 1024, 0);
    };

    i32x16 acc[FI][FJ];
#pragma unroll
    for (int i = 0; i < FI; i++)
#pragma unroll
        for (int j = 0; j < FJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
    int dsum[FI] = {};

    uint4 fa[2][FI];   // A fragments of two k steps: the next step's are read while this step's are multiplied
    const uint32_t frag_p = (wm * FI * 32 + r32) * kPitch + kg * 16;
    auto read_a = [&](int set, int buf, int step) {
        const uint8_t *bp = lds_p + buf * T * kPitch + frag_p + step * 32;
#pragma unroll
        for (int i = 0; i < FI; i++) fa[set][i] = *reinterpret_cast<const uint4 *>(bp + i * 32 * kPitch);
    };
    // The products of one k step in a fixed pattern with the memory instructions written next to them (a burst of
    // them would stall the SIMD's only wavefront in the issue queues while the matrix core runs dry):
    // `reads` LDS reads, `loads` buffer loads and `writes` LDS writes are spread over the 16 products.
    auto multiply = [&](int set, int slot, int reads, int loads, int writes) {
#pragma unroll
        for (int i = 0; i < FI; i++)
            if (DYN) dsum[i] += dot_ones(fa[set][i]);
#pragma unroll
        for (int i = 0; i < FI; i++)
#pragma unroll
            for (int j = 0; j < FJ; j++)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, fa[set][i]),
                                                                  __builtin_bit_cast(i32x4, rb[slot][j]), acc[i][j], 0, 0, 0);
        // product g is preceded by its share of each kind: floor(n (g + 1) / products) - floor(n g / products)
        constexpr int MF = FI * FJ;
#pragma unroll
        for (int g = 0; g < MF; g++) {
#pragma unroll
            for (int q = reads * g / MF; q < reads * (g + 1) / MF; q++) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
#pragma unroll
            for (int q = loads * g / MF; q < loads * (g + 1) / MF; q++) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
#pragma unroll
            for (int q = writes * g / MF; q < writes * (g + 1) / MF; q++) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // Stage s is multiplied out of LDS buffer s % 2. The next stage's A is already in registers when a stage
    // begins (asked for during the last step of the stage before), goes to the other buffer during step 2, and
    // the stage's one barrier follows step 2 -- so that the first fragments of the next stage are read from LDS
    // behind the sixteen products of step 3 instead of in front of an idle matrix core.
    load_a(0);
#pragma unroll
    for (int g = 0; g < kBdAhead; g++) load_b(g, g);
    // what a lane's outputs need of their columns (it owns FJ of them) travels with the first loads, so that
    // the epilogue does not begin with a memory round trip
    int csum[FJ];
    EmitColumn ecol[FJ];
#pragma unroll
    for (int j = 0; j < FJ; j++) {
        const int gj = min(j0 + wn * FJ * 32 + j * 32 + r32, p.J - 1);
        csum[j] = p.const_sum[gj];
        ecol[j] = gemm_emit_column<EPI>(p, gj);
    }
    store_a(0);
    load_a(min(1, nk - 1));
    __syncthreads();
    read_a(0, 0, 0);
    for (int ks = 0; ks < nk; ks++) {
        const int cur = ks & 1;
        const int g0 = ks * 4;
        read_a(1, cur, 1);
        load_b(3, g0 + 3);
        multiply(0, 0, FI, FJ, 0);
        read_a(0, cur, 2);
        load_b(0, g0 + 4);
        multiply(1, 1, FI, FJ, 0);
        read_a(1, cur, 3);           // the last read of this buffer
        load_b(1, g0 + 5);
        store_a(cur ^ 1);            // stage ks + 1 (past the end: a copy of the last stage that nobody multiplies)
        multiply(0, 2, FI, FJ, kCh);
        __syncthreads();
        read_a(0, cur ^ 1, 0);
        load_b(2, g0 + 6);
        load_a(min(ks + 2, nk - 1));
        multiply(1, 3, FI, FJ + kCh, 0);
    }

    // row sums of A: the two k halves of a row sit in lanes l and l + 32; the wavefronts of a row group hold the same sums
#pragma unroll
    for (int i = 0; i < FI; i++) dsum[i] += __shfl_xor(dsum[i], 32, 64);
    if (wn == 0 && kg == 0) {
#pragma unroll
        for (int i = 0; i < FI; i++) lds_sum[wm * FI * 32 + i * 32 + r32] = dsum[i];
    }
    __syncthreads();

    const int kzz = p.K * zd * zc;
    float fmn = 0.f, fmx = 0.f;
#pragma unroll
    for (int i = 0; i < FI; i++) {
#pragma unroll
        for (int j = 0; j < FJ; j++) {
            const int gj = j0 + wn * FJ * 32 + j * 32 + r32;
            const int fixed = kzz - zd * csum[j];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int rf = (r >> 2) * 8 + kg * 4 + (r & 3);
                const int gi = i0 + wm * FI * 32 + i * 32 + rf;
                if (gi >= p.I || gj >= p.J) continue;
                int v = acc[i][j][r] + fixed;
                if (DYN) v -= zc * lds_sum[wm * FI * 32 + i * 32 + rf];
                gemm_emit_mm<EPI>(p, ecol[j], gi, gj, v, fmn, fmx);
            }
        }
    }
    if (EPI == EPI_SCALE_BIAS) gemm_emit_range(p, lane, fmn, fmx);
}

}  // namespace hipc
