// A decoder-only decode step (batch 1) around the int4 MatMulNBits GEMV: the glue a
// gemma3-1b-shaped model needs so that the GEMV's bandwidth becomes a tokens-per-second figure.
//
// Reference operators this stands in for (crates/onnx-vulkan-core/src):
//   SimplifiedLayerNormalization  shaders/normalization.rs:109-181  y = x * rsqrt(mean(x^2) + eps) * w
//   GroupQueryAttention           shaders/attention.rs:128-317      half-split rotary, cache append,
//                                                                   scale * q.k^T, causal softmax, p.V
//   Gelu (approximate = "tanh")   interp.rs:9020-9027               0.5 v (1 + tanh(0.797884 (v + 0.044715 v^3)))
//   GatherBlockQuantized          shaders/gather_block_quantized.rs:26-57
//   ArgMax                        shaders/reduction.rs:76-191
//   the replayed decode loop      crates/onnx-vulkan/src/lib.rs:509-623, core/src/plan.rs
//
// The reference replays a recorded command list and patches the scalars that move with the
// token (plan.rs:52-61). Here nothing needs patching: the position and the current token live in
// device memory, every kernel reads them there, and the last kernel of a step advances them, so
// a captured graph of one step replays unchanged. The KV cache is resident and laid out for
// max_seq (the reference's rule, attention.rs:22-35), in f16.
#include <hip/hip_fp16.h>

#include <cstdlib>
#include <type_traits>
#include <utility>
#include <vector>

#include "internal.h"

namespace hipc {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

struct DecState {      // device-resident loop state
    int32_t token;     // the token the next step consumes
    int32_t pos;       // its position = number of tokens already in the cache
    int32_t overflow;  // sticky: a step was asked for with the cache full (pos == max_seq); that step did nothing
};

__device__ __forceinline__ float block_sum(float v, float *red) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    __syncthreads();  // red may still be read from a previous call
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float s = 0.f;
    for (int w = 0; w < nw; w++) s += red[w];
    return s;
}

// x = embed_scale * dequant(table[token]); xn = rmsnorm(x, w). One workgroup. It also leaves the
// step's rotary table behind: rope[j] = cos(pos * theta^(-2j/hd)), rope[hd/2 + j] = the sine, which
// every layer's attention reads instead of evaluating the functions again; a second table for the
// layers that rotate with another base follows at rope[hd...] when theta2 > 0.
__global__ void __launch_bounds__(256)
dec_embed_kernel(const DecState *st, const uint8_t *__restrict__ q, const float *__restrict__ scales,
                 const uint8_t *__restrict__ zp, int hidden, int bs, int n_blocks, float embed_scale,
                 const float *__restrict__ w, float eps, float *__restrict__ x, float *__restrict__ xn, int hd, float theta,
                 float theta2, float *__restrict__ rope) {
    __shared__ float red[4];
    for (int j = threadIdx.x; j < hd / 2; j += 256) {
        const float ang = (float)st->pos * powf(theta, -2.f * (float)j / (float)hd);
        rope[j] = cosf(ang), rope[hd / 2 + j] = sinf(ang);
        if (theta2 > 0.f) {
            const float ang2 = (float)st->pos * powf(theta2, -2.f * (float)j / (float)hd);
            rope[hd + j] = cosf(ang2), rope[hd + hd / 2 + j] = sinf(ang2);
        }
    }
    const size_t row = (size_t)st->token;
    const size_t row_bytes = (size_t)n_blocks * bs / 2, zp_row = (n_blocks + 1) / 2;
    float sq = 0.f;
    for (int c = threadIdx.x; c < hidden; c += 256) {
        const int b = c / bs;
        const int nib = (q[row * row_bytes + c / 2] >> (4 * (c & 1))) & 15;
        const int z = zp ? (zp[row * zp_row + b / 2] >> (4 * (b & 1))) & 15 : 8;
        const float v = ((float)nib - (float)z) * scales[row * n_blocks + b] * embed_scale;
        x[c] = v;
        sq += v * v;
    }
    const float inv = rsqrtf(block_sum(sq, red) / (float)hidden + eps);
    for (int c = threadIdx.x; c < hidden; c += 256) xn[c] = x[c] * inv * w[c];
}

// x += rmsnorm(y, w_post); xn = rmsnorm(x, w_next). One workgroup of 256; every operand is read once,
// up front (hidden <= 256 * kNormPer), so the kernel costs one memory round trip and two reductions.
constexpr int kNormPer = 8;
// y may arrive as y_slices partial rows (the k slices of the product that made it), hidden apart.
__global__ void __launch_bounds__(256)
dec_norm_residual_kernel(const float *__restrict__ y, int y_slices, const float *__restrict__ w_post, const float *__restrict__ w_next,
                         int hidden, float eps, const float *__restrict__ x_in, float *__restrict__ x, float *__restrict__ xn) {
    __shared__ float red[4];
    float yv[kNormPer], xv[kNormPer], wp[kNormPer], wn[kNormPer];
#pragma unroll
    for (int e = 0; e < kNormPer; e++) {
        const int c = threadIdx.x + e * 256;
        const bool ok = c < hidden;
        yv[e] = ok ? y[c] : 0.f, xv[e] = ok ? x_in[c] : 0.f, wp[e] = ok ? w_post[c] : 0.f, wn[e] = ok ? w_next[c] : 0.f;
        for (int s = 1; s < y_slices; s++) yv[e] += ok ? y[(size_t)s * hidden + c] : 0.f;
    }
    float sq = 0.f;
#pragma unroll
    for (int e = 0; e < kNormPer; e++) sq += yv[e] * yv[e];
    const float inv = rsqrtf(block_sum(sq, red) / (float)hidden + eps);
    float sq2 = 0.f;
#pragma unroll
    for (int e = 0; e < kNormPer; e++) {
        xv[e] = xv[e] + yv[e] * inv * wp[e];
        sq2 += xv[e] * xv[e];
    }
    const float inv2 = rsqrtf(block_sum(sq2, red) / (float)hidden + eps);
#pragma unroll
    for (int e = 0; e < kNormPer; e++) {
        const int c = threadIdx.x + e * 256;
        if (c < hidden) x[c] = xv[e], xn[c] = xv[e] * inv2 * wn[e];
    }
}

// One workgroup per head of the fused qkv vector: q heads and k heads get a per-head RMS norm and
// the half-split rotary embedding at `pos`; k and v go to the f16 cache row `pos`; q stays f32.
__global__ void __launch_bounds__(256)
dec_qkv_kernel(const DecState *st, const float *__restrict__ qkv, const float *__restrict__ q_norm,
               const float *__restrict__ k_norm, int n_q, int n_kv, int hd, float eps, float theta, int max_seq,
               float *__restrict__ q_out, __half *__restrict__ k_cache, __half *__restrict__ v_cache) {
    __shared__ float red[4];
    __shared__ float buf[512];
    const int head = blockIdx.x;
    const int pos = st->pos;
    if (pos >= max_seq) return;  // the cache is full: the step is a no-op (dec_argmax_final_kernel reports it)
    const float *src = qkv + (size_t)head * hd;
    const bool is_q = head < n_q, is_k = !is_q && head < n_q + n_kv;
    if (!is_q && !is_k) {  // a value head: straight into the cache
        const int kvh = head - n_q - n_kv;
        for (int d = threadIdx.x; d < hd; d += 256)
            v_cache[((size_t)kvh * max_seq + pos) * hd + d] = __float2half(src[d]);
        return;
    }
    const float *w = is_q ? q_norm : k_norm;
    float sq = 0.f;
    for (int d = threadIdx.x; d < hd; d += 256) sq += src[d] * src[d];
    const float inv = rsqrtf(block_sum(sq, red) / (float)hd + eps);
    for (int d = threadIdx.x; d < hd; d += 256) buf[d] = src[d] * inv * w[d];
    __syncthreads();
    const int half = hd / 2;
    for (int d = threadIdx.x; d < hd; d += 256) {
        const int j = d < half ? d : d - half;
        const float ang = (float)pos * powf(theta, -2.f * (float)j / (float)hd);
        const float c = cosf(ang), s = sinf(ang);
        const float v = d < half ? buf[d] * c - buf[d + half] * s : buf[d] * c + buf[d - half] * s;
        if (is_q)
            q_out[(size_t)head * hd + d] = v;
        else
            k_cache[((size_t)(head - n_q) * max_seq + pos) * hd + d] = __float2half(v);
    }
}

// Decode attention, split over the context: workgroup `split` of kv head `kvh` owns kAttnChunk
// positions and serves all G query heads of the group from one read of K and V. Every load of the
// chunk is independent of every other and is issued up front (one 32-byte piece of a key row per
// thread; the chunk's values of one channel per thread), so a workgroup costs about two memory
// round trips. It writes the chunk's running max, sum and unnormalised output;
// dec_attn_merge_kernel joins them.
constexpr int kAttnChunk = 16;
constexpr int kMaxGroup = 8;
__global__ void __launch_bounds__(256)
dec_attn_partial_kernel(const DecState *st, const float *__restrict__ q, const __half *__restrict__ k_cache,
                        const __half *__restrict__ v_cache, int n_q, int n_kv, int hd, int max_seq, float scale, int window,
                        float *__restrict__ part_ml, float *__restrict__ part_o) {
    __shared__ float qs[kMaxGroup * 512];
    __shared__ float sc[kMaxGroup][kAttnChunk];
    const int split = blockIdx.x, kvh = blockIdx.y, nsplit = gridDim.x;
    const int G = n_q / n_kv;
    if (st->pos >= max_seq) return;  // the cache is full: the step is a no-op
    const int total = st->pos + 1;  // the step's own key is already in the cache
    const int t0 = split * kAttnChunk;
    const int tid = threadIdx.x;
    const int cnt = min(kAttnChunk, total - t0);
    float *ml = part_ml + ((size_t)kvh * nsplit + split) * G * 2;
    const int t_first = attn_first(total, window);  // positions before it are outside the layer's window
    if (cnt <= 0 || t0 + cnt <= t_first) {  // nothing here yet, or nothing visible any more: a neutral partial
        if (tid < G) ml[tid * 2] = -3.0e38f, ml[tid * 2 + 1] = 0.f;
        if (cnt > 0)
            for (int i = tid; i < G * hd; i += 256) part_o[((size_t)kvh * nsplit + split) * G * hd + i] = 0.f;
        return;
    }
    // values first: thread d owns channel d (and d + 256) of every row of the chunk
    float vreg[2][kAttnChunk];
#pragma unroll
    for (int c = 0; c < 2; c++) {
        const int d = tid + c * 256;
#pragma unroll
        for (int t = 0; t < kAttnChunk; t++) {
            const int tt = min(t, cnt - 1);
            vreg[c][t] = d < hd ? __half2float(v_cache[((size_t)kvh * max_seq + t0 + tt) * hd + d]) : 0.f;
        }
    }
    // keys: 16 threads per position, 16 channels (32 bytes) each per pass over the head
    const int p = tid >> 4, seg = tid & 15;
    const int pp = min(p, cnt - 1);
    float dot[kMaxGroup];
#pragma unroll
    for (int g = 0; g < kMaxGroup; g++) dot[g] = 0.f;
    for (int i = tid; i < G * hd; i += 256) qs[i] = q[(size_t)kvh * G * hd + i];
    __syncthreads();
    for (int c0 = seg * 16; c0 < hd; c0 += 256) {
        const uint4 *kr = reinterpret_cast<const uint4 *>(k_cache + ((size_t)kvh * max_seq + t0 + pp) * hd + c0);
        const uint4 ka = kr[0], kb = kr[1];
        const __half2 *h2a = reinterpret_cast<const __half2 *>(&ka), *h2b = reinterpret_cast<const __half2 *>(&kb);
        float kf[16];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            kf[2 * e] = __low2float(h2a[e]), kf[2 * e + 1] = __high2float(h2a[e]);
            kf[8 + 2 * e] = __low2float(h2b[e]), kf[8 + 2 * e + 1] = __high2float(h2b[e]);
        }
#pragma unroll
        for (int g = 0; g < kMaxGroup; g++) {
            if (g < G) {
#pragma unroll
                for (int e = 0; e < 16; e++) dot[g] += qs[g * hd + c0 + e] * kf[e];
            }
        }
    }
#pragma unroll
    for (int g = 0; g < kMaxGroup; g++) {
        if (g < G) {
            float v = dot[g];
            v += __shfl_xor(v, 1, 64);
            v += __shfl_xor(v, 2, 64);
            v += __shfl_xor(v, 4, 64);
            v += __shfl_xor(v, 8, 64);
            if (seg == 0) sc[g][p] = v * scale;
        }
    }
    __syncthreads();
    // softmax pieces: thread g handles head g (the chunk is 16 values)
    if (tid < G) {
        const int lo = max(0, t_first - t0);  // first visible position of the chunk
        float m = -3.0e38f;
        for (int t = lo; t < cnt; t++) m = fmaxf(m, sc[tid][t]);
        float l = 0.f;
        for (int t = 0; t < kAttnChunk; t++) {
            const float pv = t >= lo && t < cnt ? __expf(sc[tid][t] - m) : 0.f;
            sc[tid][t] = pv;
            l += pv;
        }
        ml[tid * 2] = m, ml[tid * 2 + 1] = l;
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < 2; c++) {
        const int d = tid + c * 256;
        if (d < hd) {
            for (int g = 0; g < G; g++) {
                float o = 0.f;
#pragma unroll
                for (int t = 0; t < kAttnChunk; t++) o += sc[g][t] * vreg[c][t];
                part_o[(((size_t)kvh * nsplit + split) * G + g) * hd + d] = o;
            }
        }
    }
}

// one workgroup per query head: the weights exp(m_s - m) of the live chunks are formed once,
// then every thread sums its channel over the chunks
__global__ void __launch_bounds__(256)
dec_attn_merge_kernel(const DecState *st, const float *__restrict__ part_ml, const float *__restrict__ part_o, int n_q,
                      int n_kv, int hd, int nsplit, int even_chunks, int window, float *__restrict__ out) {
    extern __shared__ float wgt[];  // [nsplit]
    __shared__ float red[4];
    const int head = blockIdx.x;
    const int G = n_q / n_kv, kvh = head / G, g = head % G;
    // chunks holding at least one position: kAttnChunk each, or the context dealt evenly to kAttnSplits
    const int total = st->pos + 1;
    const int live = even_chunks ? attn_live_chunks(total - attn_first(total, window)) : min(nsplit, (st->pos + kAttnChunk) / kAttnChunk);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float m = -3.0e38f;
    for (int s = tid; s < live; s += 256) m = fmaxf(m, part_ml[(((size_t)kvh * nsplit + s) * G + g) * 2]);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if (lane == 0) red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float l = 0.f;
    for (int s = tid; s < live; s += 256) {
        const float *p = part_ml + (((size_t)kvh * nsplit + s) * G + g) * 2;
        const float e = __expf(p[0] - m);
        wgt[s] = e;
        l += p[1] * e;
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) l += __shfl_xor(l, off, 64);
    if (lane == 0) red[wave] = l;
    __syncthreads();
    l = (red[0] + red[1]) + (red[2] + red[3]);
    const float inv = 1.f / l;
    for (int d = tid; d < hd; d += 256) {
        float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
        int s = 0;
        for (; s + 4 <= live; s += 4) {
            const float *base = part_o + (((size_t)kvh * nsplit + s) * G + g) * hd + d;
            const size_t step = (size_t)G * hd;
            o0 += base[0] * wgt[s];
            o1 += base[step] * wgt[s + 1];
            o2 += base[2 * step] * wgt[s + 2];
            o3 += base[3 * step] * wgt[s + 3];
        }
        for (; s < live; s++) o0 += part_o[(((size_t)kvh * nsplit + s) * G + g) * hd + d] * wgt[s];
        out[(size_t)head * hd + d] = ((o0 + o1) + (o2 + o3)) * inv;
    }
}

// ---- the context chunks of one decode step's attention in one launch (head_dim 64 / 128 / 256) ----
// Workgroup (split, kvh) owns attn_chunk(span) consecutive visible positions of kv head kvh, walks them
// kAttnPass at a time (kAttnShortPass when that is the whole chunk) and serves all G query heads of the group. It
//   1. asks for the fused qkv vector's pieces it needs and for the K and V rows of its first pass
//      (16-byte pieces, every load of a pass independent of every other),
//   2. prepares the step's own q, k, v: per-head RMS norm and half-split rotary embedding for q
//      and k (every workgroup does this redundantly: 1.3 k values), k and v rounded to f16 as the
//      cache holds them; the workgroup whose chunk holds position `pos` writes them into the cache,
//      and every use of that position takes the LDS copy,
//   3. per pass: scores, running max / sum (rescaling what it has), unnormalised output, and
//   4. writes the chunk's (max, sum) pairs and unnormalised output: the flash-decoding partial.
// The partials of the live chunks are joined by the consumer (the output projection's prologue,
// or dec_attn_merge_kernel). HD and G are template parameters so that the body is straight-line
// code: with them as run-time values it was several times as long, and a workgroup that runs its
// code once pays for every instruction-cache line it touches.
template <int HD, int G>
__global__ void __launch_bounds__(256)
dec_attn_chunks_kernel(const DecState *st, const float *__restrict__ qkv, const float *__restrict__ q_norm,
                       const float *__restrict__ k_norm, int n_q, int n_kv, float eps, const float *__restrict__ rope,
                       int max_seq, float scale, int window, __half *__restrict__ k_cache, __half *__restrict__ v_cache,
                       float *__restrict__ part_ml, float *__restrict__ part_o) {
    constexpr int GH = G * HD, NK = HD / 64, HALF = HD / 2;
    constexpr int VT = HD / 8;                 // threads per value row (8 channels each)
    constexpr int VPP = 256 / VT;              // value rows in flight per pass of the workgroup
    constexpr int ROWS = (G + 1 + 3) / 4;      // q heads and the k head, dealt to four wavefronts
    static_assert(kAttnPass == 64 && kAttnShortPass == 32, "at most one lane per position of a pass");
    __shared__ __attribute__((aligned(16))) float qs[GH];      // query heads, normed and rotated
    __shared__ __attribute__((aligned(16))) float kn[HD];      // the step's key, as the cache will hold it
    __shared__ __attribute__((aligned(16))) float vn[HD];      // the step's value
    __shared__ __attribute__((aligned(16))) float sc[G * kAttnPass];
    __shared__ __attribute__((aligned(16))) float ored[4 * GH];
    __shared__ float mrun[G], lrun[G], fac[G];

    const int split = blockIdx.x, kvh = blockIdx.y;
    const int pos = st->pos, total = pos + 1;
    if (pos >= max_seq) return;  // the cache is full: the step is a no-op
    const int t_first = attn_first(total, window);  // a local layer sees the last `window` positions only
    const int chunk = attn_chunk(total - t_first);
    const int t_begin = t_first + split * chunk;
    if (t_begin >= total) return;  // no position of this chunk exists yet
    const int t_end = min(total, t_begin + chunk);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // 1. the step's own rows first (they come out of L2 and are needed first): rows 0..G-1 are the
    //    query heads, row G the key head; wavefront w prepares rows w, w + 4, ...; lane l holds
    //    elements l + 64 i of a row
    float px[ROWS][NK], pw[ROWS][NK], pc[NK], psn[NK];
#pragma unroll
    for (int i = 0; i < NK; i++) {
        const int j = (lane + 64 * i) % HALF;
        pc[i] = rope[j], psn[i] = rope[HALF + j];
    }
#pragma unroll
    for (int rr = 0; rr < ROWS; rr++) {
        const int row = min(wave + 4 * rr, G);
        const float *src = row < G ? qkv + (size_t)(kvh * G + row) * HD : qkv + (size_t)(n_q + kvh) * HD;
        const float *w = row < G ? q_norm : k_norm;
#pragma unroll
        for (int i = 0; i < NK; i++) px[rr][i] = src[lane + 64 * i], pw[rr][i] = w[lane + 64 * i];
    }
    const float pv_own = qkv[(size_t)(n_q + n_kv + kvh) * HD + min(tid, HD - 1)];
    //    K: thread (kp, seg) reads the 16-byte piece `seg` of every 128-byte run of rows kp and
    //    kp + 32 (a row is read in whole cache lines); V: thread (pg, cb) reads 8 channels of rows
    //    pg, pg + VPP, ...  Rows past the end repeat the last one (their weights are zero).
    // Everything from here on is written once for a pass of P positions and instantiated for the
    // two pass lengths; a launch runs one of them (chunks of 32 positions are walked 32 at a time:
    // half the score and value work per workgroup, on twice as many CUs).
    auto walk = [&](auto pass_length) {
    constexpr int P = decltype(pass_length)::value;
    constexpr int KP = P / 32;                 // passes of 32 positions over the keys (8 threads per position)
    constexpr int VI = P / VPP;                // value rows per thread
    static_assert(VI >= 1, "a pass holds at least one value row per thread");
    const int kp = tid >> 3, seg = tid & 7;
    const int pg = tid / VT, cb = tid % VT;
    const __half *k_head = k_cache + (size_t)kvh * max_seq * HD + seg * 8;
    const __half *v_head = v_cache + (size_t)kvh * max_seq * HD + cb * 8;
    uint4 kreg[KP][NK], vreg[VI];
    auto load_k = [&](int t0) {
#pragma unroll
        for (int ps = 0; ps < KP; ps++) {
            const __half *krow = k_head + (size_t)min(t0 + kp + 32 * ps, t_end - 1) * HD;
#pragma unroll
            for (int u = 0; u < NK; u++) kreg[ps][u] = *reinterpret_cast<const uint4 *>(krow + u * 64);
        }
    };
    auto load_v = [&](int t0) {
#pragma unroll
        for (int i = 0; i < VI; i++)
            vreg[i] = *reinterpret_cast<const uint4 *>(v_head + (size_t)min(t0 + pg + VPP * i, t_end - 1) * HD);
    };
    load_k(t_begin);
    load_v(t_begin);

    // 2. per-head RMS norm and half-split rotary embedding (pairs d, d + HD/2), one wavefront per
    //    row and no workgroup barrier: with HD = 128 or 256 both members of a pair sit in one lane
    //    (elements i and i + NK/2), with HD = 64 in lanes l and l + 32
#pragma unroll
    for (int rr = 0; rr < ROWS; rr++) {
        const int row = wave + 4 * rr;
        if (row <= G) {
            float sq = 0.f;
#pragma unroll
            for (int i = 0; i < NK; i++) sq += px[rr][i] * px[rr][i];
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) sq += __shfl_xor(sq, off, 64);
            const float inv = rsqrtf(sq / (float)HD + eps);
            float x[NK], r[NK];
#pragma unroll
            for (int i = 0; i < NK; i++) x[i] = px[rr][i] * inv * pw[rr][i];
            if (NK == 1) {
                const float other = __shfl_xor(x[0], 32, 64);
                r[0] = lane < 32 ? x[0] * pc[0] - other * psn[0] : x[0] * pc[0] + other * psn[0];
            } else {
                constexpr int HK = NK / 2 > 0 ? NK / 2 : 1;
#pragma unroll
                for (int i = 0; i < HK; i++) {
                    r[i] = x[i] * pc[i] - x[(i + HK) % NK] * psn[i];
                    r[(i + HK) % NK] = x[(i + HK) % NK] * pc[i] + x[i] * psn[i];
                }
            }
            float *dst = row < G ? qs + row * HD : kn;
#pragma unroll
            for (int i = 0; i < NK; i++) dst[lane + 64 * i] = row < G ? r[i] : __half2float(__float2half(r[i]));
        }
    }
    if (tid < HD) vn[tid] = __half2float(__float2half(pv_own));
    if (tid < G) mrun[tid] = -3.0e38f, lrun[tid] = 0.f;
    __syncthreads();
    if (pos >= t_begin && tid < HD) {  // pos = total - 1 lies in the last live chunk
        k_cache[((size_t)kvh * max_seq + pos) * HD + tid] = __float2half(kn[tid]);
        v_cache[((size_t)kvh * max_seq + pos) * HD + tid] = __float2half(vn[tid]);
    }

    float o[G][8];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int e = 0; e < 8; e++) o[g][e] = 0.f;

    for (int t0 = t_begin; t0 < t_end; t0 += P) {
        const int cnt = min(P, t_end - t0);
        const bool more = t0 + P < t_end;
        // 3a. scores. The row of `pos` as loaded is not the step's key: it counts as zero here and
        //     the thread that owns it takes the key from LDS below.
        //     A thread's two positions (kp and kp + 32) share every q value it reads from LDS.
        float dot[KP][G];
#pragma unroll
        for (int ps = 0; ps < KP; ps++)
#pragma unroll
            for (int g = 0; g < G; g++) dot[ps][g] = 0.f;
#pragma unroll
        for (int u = 0; u < NK; u++) {
            float kf[KP][8];
#pragma unroll
            for (int ps = 0; ps < KP; ps++) {
                const bool stale = min(t0 + kp + 32 * ps, t_end - 1) == pos;
                const uint4 raw = stale ? make_uint4(0, 0, 0, 0) : kreg[ps][u];
                const __half2 *h2 = reinterpret_cast<const __half2 *>(&raw);
#pragma unroll
                for (int e = 0; e < 4; e++) kf[ps][2 * e] = __low2float(h2[e]), kf[ps][2 * e + 1] = __high2float(h2[e]);
            }
            const int c0 = u * 64 + seg * 8;
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float4 qa = *reinterpret_cast<const float4 *>(qs + g * HD + c0);
                const float4 qb = *reinterpret_cast<const float4 *>(qs + g * HD + c0 + 4);
#pragma unroll
                for (int ps = 0; ps < KP; ps++)
                    dot[ps][g] += (qa.x * kf[ps][0] + qa.y * kf[ps][1]) + (qa.z * kf[ps][2] + qa.w * kf[ps][3]) +
                                  (qb.x * kf[ps][4] + qb.y * kf[ps][5]) + (qb.z * kf[ps][6] + qb.w * kf[ps][7]);
            }
        }
#pragma unroll
        for (int ps = 0; ps < KP; ps++) {
            const int tp = kp + 32 * ps;
            if (t0 + tp == pos) {
#pragma unroll 1
                for (int u = 0; u < NK; u++) {
                    const int c0 = u * 64 + seg * 8;
                    const float4 ka = *reinterpret_cast<const float4 *>(kn + c0), kb = *reinterpret_cast<const float4 *>(kn + c0 + 4);
#pragma unroll
                    for (int g = 0; g < G; g++) {
                        const float4 qa = *reinterpret_cast<const float4 *>(qs + g * HD + c0);
                        const float4 qb = *reinterpret_cast<const float4 *>(qs + g * HD + c0 + 4);
                        dot[ps][g] += (qa.x * ka.x + qa.y * ka.y) + (qa.z * ka.z + qa.w * ka.w) +
                                      (qb.x * kb.x + qb.y * kb.y) + (qb.z * kb.z + qb.w * kb.w);
                    }
                }
            }
#pragma unroll
            for (int g = 0; g < G; g++) {
                float v = dot[ps][g];
                v += __shfl_xor(v, 1, 64);
                v += __shfl_xor(v, 2, 64);
                v += __shfl_xor(v, 4, 64);
                if (seg == 0) sc[g * P + tp] = v * scale;
            }
        }
        if (more) load_k(t0 + P);
        __syncthreads();
        // 3b. one wavefront per head: the pass's max and sum join the running pair
        for (int g = wave; g < G; g += 4) {
            const float x = lane < cnt ? sc[g * P + lane] : -3.0e38f;
            const float m_old = mrun[g], l_old = lrun[g];
            float m = x;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
            m = fmaxf(m, m_old);
            const float pv = lane < cnt ? __expf(x - m) : 0.f;
            float l = pv;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) l += __shfl_xor(l, off, 64);
            const float f = __expf(m_old - m);
            if (lane < P) sc[g * P + lane] = pv;
            if (lane == 0) mrun[g] = m, lrun[g] = l_old * f + l, fac[g] = f;
        }
        __syncthreads();
        // 3c. unnormalised output: 8 channels x G heads per thread over its rows
        {
            float fg[G];
#pragma unroll
            for (int g = 0; g < G; g++) fg[g] = fac[g];
#pragma unroll
            for (int g = 0; g < G; g++)
#pragma unroll
                for (int e = 0; e < 8; e++) o[g][e] *= fg[g];
#pragma unroll
            for (int i = 0; i < VI; i++) {
                const int tp = pg + VPP * i;
                const bool stale = min(t0 + tp, t_end - 1) == pos;
                const uint4 raw = stale ? make_uint4(0, 0, 0, 0) : vreg[i];
                const __half2 *h2 = reinterpret_cast<const __half2 *>(&raw);
                float vf[8];
#pragma unroll
                for (int e = 0; e < 4; e++) vf[2 * e] = __low2float(h2[e]), vf[2 * e + 1] = __high2float(h2[e]);
#pragma unroll
                for (int g = 0; g < G; g++) {
                    const float w = sc[g * P + tp];  // zero past the end of the pass
#pragma unroll
                    for (int e = 0; e < 8; e++) o[g][e] += w * vf[e];
                }
            }
            const int own = pos - t0;  // the step's own position, if this pass holds it
            if (own >= 0 && own < P && (own % VPP) == pg) {
                const float4 va = *reinterpret_cast<const float4 *>(vn + cb * 8), vb = *reinterpret_cast<const float4 *>(vn + cb * 8 + 4);
#pragma unroll
                for (int g = 0; g < G; g++) {
                    const float w = sc[g * P + own];
                    o[g][0] += w * va.x, o[g][1] += w * va.y, o[g][2] += w * va.z, o[g][3] += w * va.w;
                    o[g][4] += w * vb.x, o[g][5] += w * vb.y, o[g][6] += w * vb.z, o[g][7] += w * vb.w;
                }
            }
        }
        if (more) load_v(t0 + P);
        // the next pass rewrites sc only after the barrier that follows its scores' LDS reads of qs;
        // its writes to sc must not overtake this pass's reads of sc
        __syncthreads();
    }
    // 4. lanes VT apart hold the same channels of neighbouring rows; then the four wavefronts
#pragma unroll
    for (int g = 0; g < G; g++) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
#pragma unroll
            for (int off = VT; off < 64; off <<= 1) o[g][e] += __shfl_xor(o[g][e], off, 64);
        }
        if (lane < VT) {
            float4 *dst = reinterpret_cast<float4 *>(ored + (wave * G + g) * HD + cb * 8);
            dst[0] = make_float4(o[g][0], o[g][1], o[g][2], o[g][3]);
            dst[1] = make_float4(o[g][4], o[g][5], o[g][6], o[g][7]);
        }
    }
    __syncthreads();
    float *po = part_o + ((size_t)kvh * kAttnSplits + split) * GH;
    for (int idx = tid; idx < GH; idx += 256)
        po[idx] = (ored[idx] + ored[GH + idx]) + (ored[2 * GH + idx] + ored[3 * GH + idx]);
    float *ml = part_ml + ((size_t)kvh * kAttnSplits + split) * G * 2;
    if (tid < G) ml[tid * 2] = mrun[tid], ml[tid * 2 + 1] = lrun[tid];
    };
    if (chunk == kAttnShortPass) walk(std::integral_constant<int, kAttnShortPass>{});
    else walk(std::integral_constant<int, kAttnPass>{});
}


// h[i] = gelu_tanh(gu[i]) * gu[ffn + i]
__global__ void __launch_bounds__(256) dec_gelu_mul_kernel(const float *__restrict__ gu, int ffn, float *__restrict__ h) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= ffn) return;
    const float v = gu[i];
    const float g = 0.5f * v * (1.f + tanhf(0.79788456080286536f * fmaf(0.044715f, v * v * v, v)));
    h[i] = g * gu[ffn + i];
}

// argmax, smallest index on ties: per-workgroup candidates, then one workgroup picks and advances the state
__global__ void __launch_bounds__(256)
dec_argmax_partial_kernel(const float *__restrict__ logits, int n, float *__restrict__ pv, int *__restrict__ pi) {
    __shared__ float sv[4];
    __shared__ int si[4];
    float best = -3.4e38f;
    int bi = 0x7fffffff;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
        const float v = logits[i];
        if (v > best || (v == best && i < bi)) best = v, bi = i;
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (ov > best || (ov == best && oi < bi)) best = ov, bi = oi;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) sv[wave] = best, si[wave] = bi;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; w++)
            if (sv[w] > best || (sv[w] == best && si[w] < bi)) best = sv[w], bi = si[w];
        pv[blockIdx.x] = best, pi[blockIdx.x] = bi;
    }
}

// The state only ever holds a token inside the vocabulary and a position inside the cache: a
// candidate outside [0, vocab) (every logit NaN: no comparison succeeds) becomes token 0, and a step
// taken with the cache full (pos == max_seq) changes nothing and raises the sticky overflow flag.
__global__ void __launch_bounds__(64)
dec_argmax_final_kernel(const float *__restrict__ pv, const int *__restrict__ pi, int nparts, DecState *st,
                        int32_t *__restrict__ history, int max_hist, int vocab) {
    float best = -3.4e38f;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < nparts; i += 64) {
        if (pv[i] > best || (pv[i] == best && pi[i] < bi)) best = pv[i], bi = pi[i];
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (ov > best || (ov == best && oi < bi)) best = ov, bi = oi;
    }
    if (threadIdx.x == 0) {
        const int pos = st->pos;
        if (pos >= max_hist) {
            st->overflow = 1;
        } else {
            if (bi < 0 || bi >= vocab) bi = 0;
            history[pos] = bi;
            st->token = bi;
            st->pos = pos + 1;
        }
    }
}

__global__ void dec_set_state_kernel(DecState *st, int token, int pos) {
    if (threadIdx.x == 0) st->token = token, st->pos = pos, st->overflow = 0;
}

}  // namespace hipc

using namespace hipc;

struct DecLayer {
    hipc_nbits_weight *qkv = nullptr, *o = nullptr, *gate_up = nullptr, *down = nullptr;
    float *norm[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};  // input, post_attn, pre_ffn, post_ffn, q, k
    __half *k_cache = nullptr, *v_cache = nullptr;
    int window = 0;      // > 0: attention sees the last `window` positions only
    int rope_table = 0;  // 0: the configuration's rotary base, 1: the decoder's second base
};

struct hipc_decoder {
    hipc_decoder_config cfg{};
    std::vector<DecLayer> layers;
    hipc_nbits_weight *lm_head = nullptr;
    float *final_norm = nullptr;
    uint8_t *emb_q = nullptr, *emb_zp = nullptr;
    float *emb_scales = nullptr;
    DecState *state = nullptr;
    int32_t *history = nullptr;
    float *x = nullptr, *xn = nullptr, *qkv = nullptr, *q = nullptr, *attn = nullptr, *y = nullptr, *gu = nullptr,
          *h = nullptr, *logits = nullptr, *part_ml = nullptr, *part_o = nullptr, *am_v = nullptr;
    int *am_i = nullptr;
    float *rope = nullptr;      // 2 x [head_dim]: cosines then sines of the current position, per rotary base
    float theta2 = 0.f;         // the second rotary base (0: none in use)
    float *x2 = nullptr;        // second buffer of the residual stream
    bool fused_glue = false;    // norms, residual adds and the gated GELU run inside the GEMV prologues
    // The default path: every per-layer product on the one-row kernel built for latency, the gated
    // GELU in the gate|up product's epilogue (its weight prepacked with interleaved halves), the
    // output and down projections cut into k slices whose partial rows the next kernel adds up.
    bool lean = false;
    int o_slices = 1, down_slices = 1;
    float *yo = nullptr, *yd = nullptr;      // [o_slices][hidden], [down_slices][hidden] partial rows
    uint4 *h_split = nullptr;                // the gated row in operand order (see LeanArgs)
    int nsplit = 0;
    bool one_launch_attn = false;  // head_dim and group size have an instance of dec_attn_chunks_kernel
    std::vector<void *> owned;
};

namespace {

constexpr int kArgmaxParts = 256;

template <typename T>
int dev_alloc(hipc_ctx *ctx, hipc_decoder *d, T **p, size_t count) {
    HIPC_TRY(ctx, hipMalloc(reinterpret_cast<void **>(p), std::max<size_t>(count * sizeof(T), 16)));
    d->owned.push_back(*p);
    return HIPC_OK;
}

template <int HD, int G>
void attn_chunks_launch(hipc_ctx *ctx, hipc_decoder *d, DecLayer &l, float scale) {
    const hipc_decoder_config &c = d->cfg;
    dec_attn_chunks_kernel<HD, G><<<dim3(kAttnSplits, c.n_kv_heads), 256, 0, ctx->stream>>>(
        d->state, d->qkv, l.norm[HIPC_DEC_NORM_Q], l.norm[HIPC_DEC_NORM_K], c.n_q_heads, c.n_kv_heads, c.rms_eps,
        d->rope + (size_t)l.rope_table * c.head_dim, c.max_seq, scale, l.window, l.k_cache, l.v_cache, d->part_ml, d->part_o);
}

template <int HD>
void attn_chunks_launch_g(hipc_ctx *ctx, hipc_decoder *d, DecLayer &l, float scale, int G) {
    switch (G) {
        case 1: attn_chunks_launch<HD, 1>(ctx, d, l, scale); break;
        case 2: attn_chunks_launch<HD, 2>(ctx, d, l, scale); break;
        case 4: attn_chunks_launch<HD, 4>(ctx, d, l, scale); break;
        default: attn_chunks_launch<HD, 8>(ctx, d, l, scale); break;
    }
}

int launch_attn_chunks(hipc_ctx *ctx, hipc_decoder *d, DecLayer &l, float scale) {
    const int G = d->cfg.n_q_heads / d->cfg.n_kv_heads;
    switch (d->cfg.head_dim) {
        case 64: attn_chunks_launch_g<64>(ctx, d, l, scale, G); break;
        case 128: attn_chunks_launch_g<128>(ctx, d, l, scale, G); break;
        default: attn_chunks_launch_g<256>(ctx, d, l, scale, G); break;
    }
    HIPC_LAUNCHED(ctx);
    return HIPC_OK;
}

bool complete(const hipc_decoder *d) {
    if (!d->lm_head || !d->final_norm || !d->emb_q) return false;
    for (const DecLayer &l : d->layers) {
        if (!l.qkv || !l.o || !l.gate_up || !l.down) return false;
        for (float *n : l.norm)
            if (!n) return false;
    }
    return true;
}

}  // namespace

extern "C" {

int hipc_decoder_create(hipc_ctx *ctx, const hipc_decoder_config *cfg, hipc_decoder **out) {
    if (!cfg || !out) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        *out = nullptr;
        HIPC_REFUSE(ctx, ctx->capturing, "decoder create while a capture is open");
        const hipc_decoder_config &c = *cfg;
        HIPC_REQUIRE(ctx, c.n_layers > 0 && c.hidden > 0 && c.ffn > 0 && c.n_q_heads > 0 && c.n_kv_heads > 0 && c.head_dim > 0 &&
                              c.vocab > 0 && c.max_seq > 0, "decoder: non-positive dimension");
        HIPC_REQUIRE(ctx, c.n_q_heads % c.n_kv_heads == 0 && c.n_q_heads / c.n_kv_heads <= kMaxGroup,
                     "decoder: %d query heads over %d kv heads (at most %d per group)", c.n_q_heads, c.n_kv_heads, kMaxGroup);
        HIPC_REQUIRE(ctx, c.head_dim % 64 == 0 && c.head_dim <= 512, "decoder: head_dim %d must be a multiple of 64, at most 512", c.head_dim);
        HIPC_REQUIRE(ctx, is_pow2(c.block_size) && c.block_size >= 32, "decoder: block_size %d", c.block_size);
        HIPC_REQUIRE(ctx, c.hidden <= 256 * kNormPer, "decoder: hidden %d exceeds %d", c.hidden, 256 * kNormPer);
        HIPC_REQUIRE(ctx, c.max_seq <= 8192 * kAttnChunk, "decoder: max_seq %d exceeds %d", c.max_seq, 8192 * kAttnChunk);
        hipc_decoder *d = new hipc_decoder();
        d->cfg = c;
        d->layers.resize(c.n_layers);
        d->nsplit = (int)ceil_div(c.max_seq, kAttnChunk);
        const size_t kv = (size_t)c.n_kv_heads * c.max_seq * c.head_dim;
        const int G = c.n_q_heads / c.n_kv_heads;
        int rc = HIPC_OK;
        auto A = [&](auto **p, size_t n) { if (rc == HIPC_OK) rc = dev_alloc(ctx, d, p, n); };
        for (DecLayer &l : d->layers) {
            A(&l.k_cache, kv);
            A(&l.v_cache, kv);
        }
        A(&d->state, 1), A(&d->history, (size_t)c.max_seq);
        A(&d->x, c.hidden), A(&d->xn, c.hidden), A(&d->qkv, (size_t)(c.n_q_heads + 2 * c.n_kv_heads) * c.head_dim);
        A(&d->q, (size_t)c.n_q_heads * c.head_dim), A(&d->attn, (size_t)c.n_q_heads * c.head_dim), A(&d->y, c.hidden);
        A(&d->gu, (size_t)2 * c.ffn), A(&d->h, c.ffn), A(&d->logits, c.vocab);
        const size_t parts = (size_t)c.n_kv_heads * std::max(d->nsplit, kAttnSplits) * G;
        A(&d->part_ml, parts * 2), A(&d->part_o, parts * c.head_dim);
        A(&d->am_v, kArgmaxParts), A(&d->am_i, kArgmaxParts);
        A(&d->rope, (size_t)2 * c.head_dim), A(&d->x2, c.hidden);
        // options read when the decoder is created: dec_fused_glue = 0 keeps the separate norm / GELU
        // kernels, dec_fused_attn = 0 the three-kernel attention (tests of those paths)
        d->fused_glue = c.hidden % 8 == 0 && c.ffn % 8 == 0 && ctx->tune.dec_fused_glue != 0;
        d->one_launch_attn = (c.head_dim == 64 || c.head_dim == 128 || c.head_dim == 256) && (G == 1 || G == 2 || G == 4 || G == 8) &&
                             ctx->tune.dec_fused_attn != 0;
        // the lean path (the dec_lean option set to 0 keeps the streaming kernel and its prologues)
        {
            const int n_cg_h = (int)ceil_div(c.hidden, 128), n_cg_o = (int)ceil_div((int64_t)c.n_q_heads * c.head_dim, 128);
            const int n_cg_f = (int)ceil_div(c.ffn, 128);
            d->lean = d->fused_glue && d->one_launch_attn && ctx->tune.dec_lean != 0 && c.ffn % 16 == 0 && n_cg_h <= 32 &&
                      c.hidden % 8 == 0;
            // output projection: a k slice is one head (or one 128-k tile when heads are shorter), at most 8 slices
            int o_tiles = std::max(1, c.head_dim / 128);
            while (ceil_div(n_cg_o, o_tiles) > 8 && o_tiles < 4) o_tiles *= 2;
            d->o_slices = (int)ceil_div(n_cg_o, o_tiles);
            if (d->o_slices > 8 || o_tiles > 4) d->lean = false;
            // down projection: 18 k tiles per slice (six wavefronts of three tiles), at most 8 slices
            d->down_slices = (int)std::max<int64_t>(1, ceil_div(n_cg_f, 18));
            if (d->down_slices > 8) d->lean = false;
            if (d->lean) {
                A(&d->yo, (size_t)d->o_slices * c.hidden), A(&d->yd, (size_t)d->down_slices * c.hidden);
                const size_t chunks = (size_t)n_cg_f * 4;
                A(&d->h_split, chunks * 2 * 4);
                // the join in the output projection's prologue reads a chunk's partials before it knows whether
                // the chunk is live (and weighs them with zero if not): they must be finite from the start
                if (rc == HIPC_OK &&
                    (hipMemsetAsync(d->h_split, 0, chunks * 2 * 4 * 16, ctx->stream) != hipSuccess ||
                     hipMemsetAsync(d->part_o, 0, parts * c.head_dim * 4, ctx->stream) != hipSuccess ||
                     hipMemsetAsync(d->part_ml, 0, parts * 2 * 4, ctx->stream) != hipSuccess))
                    rc = fail(ctx, HIPC_ERR_BACKEND, "decoder: cannot clear the gated row and the attention partials");
            }
        }
        if (rc == HIPC_OK) {
            for (DecLayer &l : d->layers) {  // an unwritten cache row must not hold NaN bit patterns
                if (hipMemsetAsync(l.k_cache, 0, kv * 2, ctx->stream) != hipSuccess || hipMemsetAsync(l.v_cache, 0, kv * 2, ctx->stream) != hipSuccess)
                    rc = fail(ctx, HIPC_ERR_BACKEND, "decoder: cannot clear the KV cache");
            }
            dec_set_state_kernel<<<1, 64, 0, ctx->stream>>>(d->state, 0, 0);
        }
        if (rc != HIPC_OK) {
            for (void *p : d->owned) (void)hipFree(p);
            delete d;
            return rc;
        }
        *out = d;
        return HIPC_OK;
    });
}

void hipc_decoder_destroy(hipc_ctx *ctx, hipc_decoder *d) {
    if (!d) return;
    entry_void(ctx, [&] {
        for (DecLayer &l : d->layers) {
            nbits_release(ctx, l.qkv), nbits_release(ctx, l.o), nbits_release(ctx, l.gate_up), nbits_release(ctx, l.down);
        }
        nbits_release(ctx, d->lm_head);
        for (void *p : d->owned) ctx->deferred.push_back(p);
        delete d;
    });
}

int hipc_decoder_set_linear(hipc_ctx *ctx, hipc_decoder *d, int layer, int which, const void *B, size_t b_len,
                            const void *scales, size_t scales_len, const void *zp, size_t zp_len) {
    if (!d) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        const hipc_decoder_config &c = d->cfg;
        const int64_t qd = (int64_t)c.n_q_heads * c.head_dim, kvd = (int64_t)c.n_kv_heads * c.head_dim;
        int64_t K = 0, N = 0;
        hipc_nbits_weight **slot = nullptr;
        if (which == HIPC_DEC_LM_HEAD) {
            K = c.hidden, N = c.vocab, slot = &d->lm_head;
        } else {
            HIPC_REQUIRE(ctx, layer >= 0 && layer < c.n_layers, "decoder: layer %d out of range", layer);
            DecLayer &l = d->layers[layer];
            switch (which) {
                case HIPC_DEC_QKV: K = c.hidden, N = qd + 2 * kvd, slot = &l.qkv; break;
                case HIPC_DEC_O: K = qd, N = c.hidden, slot = &l.o; break;
                case HIPC_DEC_GATE_UP: K = c.hidden, N = 2 * (int64_t)c.ffn, slot = &l.gate_up; break;
                case HIPC_DEC_DOWN: K = c.ffn, N = c.hidden, slot = &l.down; break;
                default: return fail(ctx, HIPC_ERR_INVALID, "decoder: unknown linear %d", which);
            }
        }
        if (*slot) {  // a recorded step may still name the old weight: it is retired, not freed
            retire(ctx, (*slot)->Wq), retire(ctx, (*slot)->Sc), retire(ctx, (*slot)->Zb);
            delete *slot;
            *slot = nullptr;
        }
        const int half = (d->lean && which == HIPC_DEC_GATE_UP) ? c.ffn : 0;
        return nbits_prepack(ctx, B, b_len, scales, HIPC_F32, scales_len, zp, zp_len, K, N, c.block_size, slot, half);
    });
}

int hipc_decoder_set_norm(hipc_ctx *ctx, hipc_decoder *d, int layer, int which, const void *w) {
    if (!d || !w) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        const hipc_decoder_config &c = d->cfg;
        float **slot = nullptr;
        size_t n = c.hidden;
        if (which == HIPC_DEC_NORM_FINAL) {
            slot = &d->final_norm;
        } else {
            HIPC_REQUIRE(ctx, layer >= 0 && layer < c.n_layers, "decoder: layer %d out of range", layer);
            HIPC_REQUIRE(ctx, which >= 0 && which < 6, "decoder: unknown norm %d", which);
            slot = &d->layers[layer].norm[which];
            if (which == HIPC_DEC_NORM_Q || which == HIPC_DEC_NORM_K) n = c.head_dim;
        }
        if (!*slot) {
            int rc = dev_alloc(ctx, d, slot, n);
            if (rc != HIPC_OK) return rc;
        }
        HIPC_TRY(ctx, hipMemcpyAsync(*slot, w, n * 4, hipMemcpyDeviceToDevice, ctx->stream));
        return HIPC_OK;
    });
}

int hipc_decoder_set_embedding(hipc_ctx *ctx, hipc_decoder *d, const void *B, size_t b_len, const void *scales,
                               size_t scales_len, const void *zp, size_t zp_len) {
    if (!d || !B || !scales) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        const hipc_decoder_config &c = d->cfg;
        const size_t nb = (size_t)ceil_div(c.hidden, c.block_size);
        const size_t qb = (size_t)c.vocab * nb * c.block_size / 2, sb = (size_t)c.vocab * nb, zb = (size_t)c.vocab * ((nb + 1) / 2);
        HIPC_REQUIRE(ctx, b_len >= qb && scales_len >= sb && (!zp || zp_len >= zb), "decoder: embedding table is short");
        if (!d->emb_q) {
            int rc = dev_alloc(ctx, d, &d->emb_q, qb);
            if (rc == HIPC_OK) rc = dev_alloc(ctx, d, &d->emb_scales, sb);
            if (rc == HIPC_OK && zp) rc = dev_alloc(ctx, d, &d->emb_zp, zb);
            if (rc != HIPC_OK) return rc;
        }
        HIPC_TRY(ctx, hipMemcpyAsync(d->emb_q, B, qb, hipMemcpyDeviceToDevice, ctx->stream));
        HIPC_TRY(ctx, hipMemcpyAsync(d->emb_scales, scales, sb * 4, hipMemcpyDeviceToDevice, ctx->stream));
        if (zp) HIPC_TRY(ctx, hipMemcpyAsync(d->emb_zp, zp, zb, hipMemcpyDeviceToDevice, ctx->stream));
        return HIPC_OK;
    });
}

int hipc_decoder_set_layer_attention(hipc_ctx *ctx, hipc_decoder *d, int layer, int32_t window, float rope_theta) {
    if (!d) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        HIPC_REFUSE(ctx, ctx->capturing, "decoder: layer attention changed while a capture is open");
        HIPC_REQUIRE(ctx, layer >= 0 && layer < d->cfg.n_layers, "decoder: layer %d out of range", layer);
        HIPC_REQUIRE(ctx, !(rope_theta < 0.f) && rope_theta == rope_theta, "decoder: bad rotary base");
        DecLayer &l = d->layers[layer];
        int table = 0;
        if (rope_theta > 0.f && rope_theta != d->cfg.rope_theta) {
            HIPC_REQUIRE(ctx, d->theta2 == 0.f || d->theta2 == rope_theta,
                         "decoder: a third rotary base (%g beside %g and %g)", rope_theta, d->cfg.rope_theta, d->theta2);
            d->theta2 = rope_theta;
            table = 1;
        }
        l.window = window > 0 ? window : 0;
        l.rope_table = table;
        return HIPC_OK;
    });
}

int hipc_decoder_reset(hipc_ctx *ctx, hipc_decoder *d, int32_t token, int32_t pos) {
    if (!d) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, token >= 0 && token < d->cfg.vocab && pos >= 0 && pos < d->cfg.max_seq, "decoder: bad token %d or position %d", token, pos);
        dec_set_state_kernel<<<1, 64, 0, ctx->stream>>>(d->state, token, pos);
        HIPC_LAUNCHED(ctx);
        return HIPC_OK;
    });
}

int hipc_decoder_kv_cache(hipc_ctx *ctx, hipc_decoder *d, int layer, void **k_cache, void **v_cache) {
    if (!d || !k_cache || !v_cache) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, layer >= 0 && layer < d->cfg.n_layers, "decoder: layer %d out of range", layer);
        *k_cache = d->layers[layer].k_cache, *v_cache = d->layers[layer].v_cache;
        return HIPC_OK;
    });
}

int hipc_decoder_step(hipc_ctx *ctx, hipc_decoder *d) {
    if (!d) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, complete(d), "decoder: not every weight has been set");
        const hipc_decoder_config &c = d->cfg;
        hipStream_t s = ctx->stream;
        const int nb = (int)ceil_div(c.hidden, c.block_size);
        const int heads = c.n_q_heads + 2 * c.n_kv_heads;
        const float scale = c.attn_scale > 0.f ? c.attn_scale : 1.f / sqrtf((float)c.head_dim);
        const int terms = 2;
        int rc;
        dec_embed_kernel<<<1, 256, 0, s>>>(d->state, d->emb_q, d->emb_scales, d->emb_zp, c.hidden, c.block_size, nb, c.embed_scale,
                                           d->layers[0].norm[HIPC_DEC_NORM_INPUT], c.rms_eps, d->x, d->xn, c.head_dim, c.rope_theta,
                                           d->theta2, d->rope);
        HIPC_LAUNCHED(ctx);
        // The residual stream alternates between two buffers: a GEMV whose prologue folds the previous
        // branch into the stream reads one and (its first workgroup) writes the other.
        float *xc = d->x, *xo = d->x2;
        for (int li = 0; li < c.n_layers && d->lean; li++) {
            DecLayer &l = d->layers[li];
            LeanPlan pl;
            // qkv: row = rmsnorm(x', w_input), x' = x + rmsnorm(sum of the down projection's partial rows, w_post_ffn of the layer before)
            {
                LeanArgs a{};
                a.x = xc, a.w_in = l.norm[HIPC_DEC_NORM_INPUT], a.x_out = xo, a.eps = c.rms_eps;
                if (li > 0) a.yparts = d->yd, a.y_slices = d->down_slices, a.w_post = d->layers[li - 1].norm[HIPC_DEC_NORM_POST_FFN];
                a.Y = d->qkv;
                HIPC_REQUIRE(ctx, lean_plan(ctx, l.qkv, 1, 1, &pl), "decoder: no launch plan for the qkv projection");
                if ((rc = lean_gemv(ctx, l.qkv, pl, a, 2, 0, terms)) != HIPC_OK) return rc;
                std::swap(xc, xo);
            }
            if ((rc = launch_attn_chunks(ctx, d, l, scale)) != HIPC_OK) return rc;
            // output projection: a k slice per head, joined from the attention partials; partial rows out
            {
                LeanArgs a{};
                a.part_o = d->part_o, a.part_ml = d->part_ml, a.pos = &d->state->pos;
                a.lg_group = __builtin_ctz((unsigned)(c.n_q_heads / c.n_kv_heads)), a.lg_hd = __builtin_ctz((unsigned)c.head_dim);   // powers of two where the one-launch attention runs
                a.n_kv = c.n_kv_heads, a.window = l.window;
                a.Y = d->yo;
                const int per_slice = (int)ceil_div(l.o->n_cg, d->o_slices);
                pl = LeanPlan{1, per_slice, 4, d->o_slices};   // four wavefronts, each all k tiles of the slice: no sum over wavefronts
                if ((rc = lean_gemv(ctx, l.o, pl, a, 3, 0, terms)) != HIPC_OK) return rc;
            }
            // gate | up: row = rmsnorm(x'', w_pre_ffn), x'' = x' + rmsnorm(sum of the output projection's partial rows, w_post_attn);
            // epilogue gelu_tanh(gate) * up in operand order
            {
                LeanArgs a{};
                a.x = xc, a.w_in = l.norm[HIPC_DEC_NORM_PRE_FFN], a.x_out = xo, a.eps = c.rms_eps;
                a.yparts = d->yo, a.y_slices = d->o_slices, a.w_post = l.norm[HIPC_DEC_NORM_POST_ATTN];
                a.h_split = d->h_split;
                HIPC_REQUIRE(ctx, lean_plan(ctx, l.gate_up, 1, 2, &pl), "decoder: no launch plan for the gate | up projection");
                if ((rc = lean_gemv(ctx, l.gate_up, pl, a, 2, 1, terms)) != HIPC_OK) return rc;
                std::swap(xc, xo);
            }
            // down: the gated row straight into the operand registers; partial rows out
            {
                LeanArgs a{};
                a.a_split = d->h_split;
                a.Y = d->yd;
                HIPC_REQUIRE(ctx, lean_plan(ctx, l.down, d->down_slices, 1, &pl, 8),
                             "decoder: no launch plan for the down projection");
                if ((rc = lean_gemv(ctx, l.down, pl, a, 4, 0, terms)) != HIPC_OK) return rc;
            }
        }
        for (int li = 0; li < c.n_layers && !d->lean; li++) {
            DecLayer &l = d->layers[li];
            if (d->fused_glue && li > 0) {
                GemvPrologue pro;
                pro.mode = 2, pro.x = xc, pro.y = d->y, pro.w_post = d->layers[li - 1].norm[HIPC_DEC_NORM_POST_FFN];
                pro.w_in = l.norm[HIPC_DEC_NORM_INPUT], pro.x_out = xo, pro.eps = c.rms_eps;
                if ((rc = nbits_gemv(ctx, xc, HIPC_F32, l.qkv, d->qkv, 1, terms, &pro)) != HIPC_OK) return rc;
                std::swap(xc, xo);
            } else {
                if ((rc = nbits_gemv(ctx, d->xn, HIPC_F32, l.qkv, d->qkv, 1, terms)) != HIPC_OK) return rc;
            }
            if (d->one_launch_attn) {
                if ((rc = launch_attn_chunks(ctx, d, l, scale)) != HIPC_OK) return rc;
                if (d->fused_glue) {  // the output projection joins the chunks' partials in its prologue
                    GemvPrologue merge;
                    merge.mode = 3, merge.part_o = d->part_o, merge.part_ml = d->part_ml, merge.pos = &d->state->pos;
                    merge.group = c.n_q_heads / c.n_kv_heads, merge.head_dim = c.head_dim, merge.window = l.window;
                    if ((rc = nbits_gemv(ctx, d->attn, HIPC_F32, l.o, d->y, 1, terms, &merge)) != HIPC_OK) return rc;
                } else {
                    dec_attn_merge_kernel<<<c.n_q_heads, 256, (size_t)kAttnSplits * sizeof(float), s>>>(
                        d->state, d->part_ml, d->part_o, c.n_q_heads, c.n_kv_heads, c.head_dim, kAttnSplits, 1, l.window, d->attn);
                    HIPC_LAUNCHED(ctx);
                    if ((rc = nbits_gemv(ctx, d->attn, HIPC_F32, l.o, d->y, 1, terms)) != HIPC_OK) return rc;
                }
            } else {
                dec_qkv_kernel<<<heads, 256, 0, s>>>(d->state, d->qkv, l.norm[HIPC_DEC_NORM_Q], l.norm[HIPC_DEC_NORM_K], c.n_q_heads,
                                                     c.n_kv_heads, c.head_dim, c.rms_eps, l.rope_table ? d->theta2 : c.rope_theta, c.max_seq, d->q,
                                                     l.k_cache, l.v_cache);
                HIPC_LAUNCHED(ctx);
                dec_attn_partial_kernel<<<dim3(d->nsplit, c.n_kv_heads), 256, 0, s>>>(d->state, d->q, l.k_cache, l.v_cache, c.n_q_heads, c.n_kv_heads,
                                                                                     c.head_dim, c.max_seq, scale, l.window, d->part_ml, d->part_o);
                HIPC_LAUNCHED(ctx);
                dec_attn_merge_kernel<<<c.n_q_heads, 256, (size_t)d->nsplit * sizeof(float), s>>>(d->state, d->part_ml, d->part_o, c.n_q_heads, c.n_kv_heads,
                                                                                                 c.head_dim, d->nsplit, 0, l.window, d->attn);
                HIPC_LAUNCHED(ctx);
                if ((rc = nbits_gemv(ctx, d->attn, HIPC_F32, l.o, d->y, 1, terms)) != HIPC_OK) return rc;
            }
            if (d->fused_glue) {
                GemvPrologue pro;
                pro.mode = 2, pro.x = xc, pro.y = d->y, pro.w_post = l.norm[HIPC_DEC_NORM_POST_ATTN];
                pro.w_in = l.norm[HIPC_DEC_NORM_PRE_FFN], pro.x_out = xo, pro.eps = c.rms_eps;
                if ((rc = nbits_gemv(ctx, xc, HIPC_F32, l.gate_up, d->gu, 1, terms, &pro)) != HIPC_OK) return rc;
                std::swap(xc, xo);
                GemvPrologue gelu;
                gelu.mode = 1;
                if ((rc = nbits_gemv(ctx, d->gu, HIPC_F32, l.down, d->y, 1, terms, &gelu)) != HIPC_OK) return rc;
            } else {
                dec_norm_residual_kernel<<<1, 256, 0, s>>>(d->y, 1, l.norm[HIPC_DEC_NORM_POST_ATTN], l.norm[HIPC_DEC_NORM_PRE_FFN], c.hidden, c.rms_eps, d->x, d->x, d->xn);
                HIPC_LAUNCHED(ctx);
                if ((rc = nbits_gemv(ctx, d->xn, HIPC_F32, l.gate_up, d->gu, 1, terms)) != HIPC_OK) return rc;
                dec_gelu_mul_kernel<<<(unsigned)ceil_div(c.ffn, 256), 256, 0, s>>>(d->gu, c.ffn, d->h);
                HIPC_LAUNCHED(ctx);
                if ((rc = nbits_gemv(ctx, d->h, HIPC_F32, l.down, d->y, 1, terms)) != HIPC_OK) return rc;
                const float *next = li + 1 < c.n_layers ? d->layers[li + 1].norm[HIPC_DEC_NORM_INPUT] : d->final_norm;
                dec_norm_residual_kernel<<<1, 256, 0, s>>>(d->y, 1, l.norm[HIPC_DEC_NORM_POST_FFN], next, c.hidden, c.rms_eps, d->x, d->x, d->xn);
                HIPC_LAUNCHED(ctx);
            }
        }
        if (d->fused_glue) {
            // the unembedding streams ~200 MB: its workgroups start on the weights at once and the
            // final norm stays a launch of its own
            dec_norm_residual_kernel<<<1, 256, 0, s>>>(d->lean ? d->yd : d->y, d->lean ? d->down_slices : 1,
                                                       d->layers[c.n_layers - 1].norm[HIPC_DEC_NORM_POST_FFN], d->final_norm, c.hidden,
                                                       c.rms_eps, xc, xc, d->xn);
            HIPC_LAUNCHED(ctx);
        }
        if ((rc = nbits_gemv(ctx, d->xn, HIPC_F32, d->lm_head, d->logits, 1, terms)) != HIPC_OK) return rc;
        dec_argmax_partial_kernel<<<kArgmaxParts, 256, 0, s>>>(d->logits, c.vocab, d->am_v, d->am_i);
        HIPC_LAUNCHED(ctx);
        dec_argmax_final_kernel<<<1, 64, 0, s>>>(d->am_v, d->am_i, kArgmaxParts, d->state, d->history, c.max_seq, c.vocab);
        HIPC_LAUNCHED(ctx);
        return HIPC_OK;
    });
}

int hipc_decoder_read(hipc_ctx *ctx, hipc_decoder *d, int32_t *token, int32_t *pos, float *logits, int32_t *history, int32_t n_history) {
    if (!d) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        HIPC_REFUSE(ctx, ctx->capturing, "decoder read while a capture is open");
        HIPC_TRY(ctx, hipStreamSynchronize(ctx->stream));
        DecState st{};
        HIPC_TRY(ctx, hipMemcpy(&st, d->state, sizeof st, hipMemcpyDeviceToHost));
        if (token) *token = st.token;
        if (pos) *pos = st.pos;
        if (logits) HIPC_TRY(ctx, hipMemcpy(logits, d->logits, (size_t)d->cfg.vocab * 4, hipMemcpyDeviceToHost));
        if (history && n_history > 0)
            HIPC_TRY(ctx, hipMemcpy(history, d->history, (size_t)std::min<int32_t>(n_history, d->cfg.max_seq) * 4, hipMemcpyDeviceToHost));
        HIPC_REQUIRE(ctx, !st.overflow, "decoder: a step was enqueued with the cache full (%d positions); it did nothing", d->cfg.max_seq);
        return HIPC_OK;
    });
}

}  // extern "C"
