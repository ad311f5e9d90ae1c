// Helper workgroups that warm the L2 of the right XCD for the NEXT launch of a chain.
//
// Launches of one decode step depend on each other, so a kernel's weights start to stream only when
// its predecessor has finished, and a workgroup then waits 1.3-1.6 us for its first tiles: the time
// HBM takes for the whole launch's few megabytes. Those bytes do not depend on the predecessor's
// results. So the predecessor's grid gets extra rows of workgroups that do nothing but read what the
// next launch will read. Workgroups go to the eight XCDs round robin by linear id -- the same way in
// every launch -- and every XCD has its own L2: a helper with linear id b therefore reads for the
// consumers j with j = b (mod 8), and the consumer's loads hit its own L2 (measured on a 5 MB weight:
// a consumer's wait for 16 KiB falls from 1.6 us to 0.7 us; 1.2 us when the helper sits on another XCD
// and only the memory-side cache holds the lines).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include "internal.h"

namespace hipc {

__device__ __forceinline__ uint32_t pf_fold(uint32_t acc, __amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    const auto v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0);
    return acc ^ v[0] ^ v[3];
}

// every thread of the workgroup asks for its 16-byte pieces of [base, base + bytes): up to ROUNDS
// pieces per thread, all in flight together (pieces past the end: the descriptor answers with zeros,
// without traffic)
template <int ROUNDS>
__device__ __forceinline__ uint32_t pf_span(uint32_t acc, const void *base, uint32_t bytes, int tid, int nthreads) {
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
    uint32_t parts[ROUNDS];
#pragma unroll
    for (int i = 0; i < ROUNDS; i++) parts[i] = pf_fold(0u, r, (uint32_t)(tid + i * nthreads) * 16u, 0u);   // the range check covers the per-lane offset only
#pragma unroll
    for (int i = 0; i < ROUNDS; i++) acc ^= parts[i];
    return acc;
}

// h: this helper's index among the H helpers of the launch; b: its linear workgroup id in the launch
__device__ inline void prefetch_for_next(const PrefetchArgs &pf, int h, int H, int b, uint32_t *sink) {
    int first, step;
    pf_consumers_of(h, H, b, &first, &step);
    const int tid = threadIdx.x, nthreads = blockDim.x;
    uint32_t acc = 0;
    if (pf.kind == 1) {
        // consumer j of a one-row product's grid reads, for each of its WN column tiles, a run of tiles
        // that is contiguous in all three arrays
        const int n_cons = pf.gx * pf.gy;
        for (int j = first; j < n_cons; j += step) {
            for (int wn = 0; wn < pf.WN; wn++) {
                size_t tile0;
                const int cnt = pf_tile_run(pf, j, wn, &tile0);
                if (cnt == 0) break;
                // six rounds of >= 192 threads cover a run of 18 tiles (18 KiB of weights, 4.5 KiB of scales, 1.1 KiB of
                // zero points); of a longer run only that much is read ahead
                acc = pf_span<6>(acc, pf.wq + tile0 * 64, (uint32_t)cnt * 1024u, tid, nthreads);
                acc = pf_span<2>(acc, pf.sc + tile0 * 16 * pf.SG, (uint32_t)cnt * 64u * pf.SG, tid, nthreads);
                acc = pf_span<1>(acc, pf.zb + tile0 * 16 * pf.SG, (uint32_t)cnt * 16u * pf.SG, tid, nthreads);
            }
        }
    } else if (pf.kind == 2) {
        // consumer (split, kvh) of the attention launch reads the key rows and value columns of its chunk's
        // first pass (the later passes of a long context follow behind the first)
        const int pos = *pf.pos, total = pos + 1;
        const int base = attn_base(total, pf.window);
        const int chunk = attn_chunk(total - base);
        const int n_cons = kAttnSplits * pf.n_kv;
        for (int j = first; j < n_cons; j += step) {
            const int split = j & (kAttnSplits - 1), kvh = j / kAttnSplits;
            const int t0 = base + split * chunk;
            if (pos >= pf.max_seq || t0 >= total) continue;
            const int rows = min(kAttnPass, total - t0);
            const __half *k = static_cast<const __half *>(pf.k) + ((size_t)kvh * pf.max_seq + t0) * pf.hd;
            acc = pf_span<6>(acc, k, (uint32_t)(rows * pf.hd) * 2u, tid, nthreads);
            // 64 bytes (32 positions) of each channel's row: four 16-byte pieces per channel
            const __half *v = static_cast<const __half *>(pf.v) + (size_t)kvh * pf.hd * pf.v_stride + t0;
            const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(v), 0, (int)((uint32_t)pf.hd * (uint32_t)pf.v_stride * 2u), 0x00020000);
            for (int i = tid; i < pf.hd * 4; i += nthreads) acc = pf_fold(acc, r, ((uint32_t)(i >> 2) * (uint32_t)pf.v_stride) * 2u + (uint32_t)(i & 3) * 16u, 0);
        }
    }
    if (acc == 0x9e3779b9u && sink) *sink = acc;   // keeps the loads alive; practically never true
}

}  // namespace hipc
