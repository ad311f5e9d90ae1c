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

// One 32-bit word of each 128-byte line is enough to bring the line into L2. `pf_touch` asks for the
// lines tid, tid + nthreads, ... of [base, base + bytes), ROUNDS of them per thread, and returns without
// waiting: the words land in `out`. The descriptor covers exactly the span and the whole offset is the
// lane's, so a line past the end is answered with zero and costs no traffic (the hardware's range check
// sees the per-lane offset only: nothing here uses the scalar offset).
template <int ROUNDS>
__device__ __forceinline__ void pf_touch(uint32_t (&out)[ROUNDS], const void *base, uint32_t bytes, int tid, int nthreads) {
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
#pragma unroll
    for (int i = 0; i < ROUNDS; i++) out[i] = __builtin_amdgcn_raw_buffer_load_b32(r, (int)((uint32_t)(tid + i * nthreads) * 128u), 0, 0);
}

// h: this helper's index among the H helpers of the launch; b: its linear workgroup id in the launch.
// A helper walks its consumers one after the other, but never waits for what it has just asked for: the
// words of one consumer are folded into the checksum while the next consumer's are in flight, so the
// helper lasts one memory latency plus the transfer, not one latency per consumer.
__device__ inline void prefetch_for_next(const PrefetchArgs &pf, int h, int H, int b, uint32_t *sink) {
    int first, step;
    pf_consumers_of(h, H, b, &first, &step);
    const int tid = threadIdx.x, nthreads = blockDim.x;
    uint32_t acc = 0;
    if (pf.kind == 1 && pf.gate_chunks > 0 && attn_live_chunks(attn_span(*pf.pos + 1, pf.gate_window)) < pf.gate_chunks) return;
    if (pf.kind == 1) {
        // consumer j of a one-row product's grid reads, for each of its WN column tiles, a run of tiles that is
        // contiguous in all three arrays: 8 lines of weights, SG / 2 of scales and SG / 8 of zero points per tile.
        // Three rounds of >= 192 threads cover the weights of a run of 72 tiles, one round its scales and zero points.
        const int n_cons = pf.gx * pf.gy;
        uint32_t prev[5] = {0u, 0u, 0u, 0u, 0u};
        for (int j = first; j < n_cons; j += step) {
            for (int wn = 0; wn < pf.WN; wn++) {
                size_t tile0;
                const int cnt = pf_tile_run(pf, j, wn, &tile0);
                if (cnt == 0) break;
                uint32_t wq[3], sc[1], zb[1];
                pf_touch<3>(wq, pf.wq + tile0 * 64, (uint32_t)cnt * 1024u, tid, nthreads);
                pf_touch<1>(sc, pf.sc + tile0 * 16 * pf.SG, (uint32_t)cnt * 64u * pf.SG, tid, nthreads);
                pf_touch<1>(zb, pf.zb + tile0 * 16 * pf.SG, (uint32_t)cnt * 16u * pf.SG, tid, nthreads);
                acc ^= (prev[0] ^ prev[1]) ^ (prev[2] ^ prev[3]) ^ prev[4];   // the run before this one
                prev[0] = wq[0], prev[1] = wq[1], prev[2] = wq[2], prev[3] = sc[0], prev[4] = zb[0];
            }
        }
        acc ^= (prev[0] ^ prev[1]) ^ (prev[2] ^ prev[3]) ^ prev[4];
    } else if (pf.kind == 2) {
        // consumer (split, kvh) of the attention launch reads the key rows and value columns of its chunk's
        // first pass (the later passes of a long context follow behind the first): the key rows are one span
        // (a line per thread: 32 rows of at most 256 halfs are 128 lines); of the values, 64 bytes (32 positions)
        // of each channel's row, i.e. one word per channel, rows v_stride halfs apart.
        const int pos = *pf.pos, total = pos + 1;
        const int base = attn_base(total, pf.window);
        const int chunk = attn_chunk(total - base);
        const int n_cons = kAttnSplits * pf.n_kv;
        uint32_t prev[4] = {0u, 0u, 0u, 0u};
        for (int j = first; j < n_cons; j += step) {
            const int split = j & (kAttnSplits - 1), kvh = j / kAttnSplits;
            const int t0 = base + split * chunk;
            if (pos >= pf.max_seq || t0 >= total) continue;
            const int rows = min(kAttnPass, total - t0);
            const __half *k = static_cast<const __half *>(pf.k) + ((size_t)kvh * pf.max_seq + t0) * pf.hd;
            uint32_t kw[2], vw[2];
            pf_touch<2>(kw, k, (uint32_t)(rows * pf.hd) * 2u, tid, nthreads);
            // the descriptor starts at the chunk's first position of channel 0 and ends with the LAST channel's 64 bytes
            const __half *v = static_cast<const __half *>(pf.v) + (size_t)kvh * pf.hd * pf.v_stride + t0;
            const uint32_t v_bytes = ((uint32_t)(pf.hd - 1) * (uint32_t)pf.v_stride + (uint32_t)kAttnPass) * 2u;
            const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(v), 0, (int)v_bytes, 0x00020000);
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const uint32_t ch = (uint32_t)(tid + i * nthreads);   // a channel past the last: past the descriptor, zero
                vw[i] = __builtin_amdgcn_raw_buffer_load_b32(r, (int)(min(ch, 65535u) * (uint32_t)pf.v_stride * 2u), 0, 0);
            }
            acc ^= (prev[0] ^ prev[1]) ^ (prev[2] ^ prev[3]);
            prev[0] = kw[0], prev[1] = kw[1], prev[2] = vw[0], prev[3] = vw[1];
        }
        acc ^= (prev[0] ^ prev[1]) ^ (prev[2] ^ prev[3]);
    }
    if (acc == 0x9e3779b9u && sink) *sink = acc;   // keeps the loads alive; practically never true
}

}  // namespace hipc
