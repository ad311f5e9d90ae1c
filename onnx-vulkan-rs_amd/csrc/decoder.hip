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
#include "lanes.h"
#include "prefetch.h"

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

// x = embed_scale * dequant(table[token]); xn = rmsnorm(x, w). One workgroup of 256. It also leaves the
// step's rotary table behind: rope[j] = cos(pos * theta^(-2j/hd)), rope[hd/2 + j] = the sine, which
// every layer's attention reads instead of evaluating the functions again; a second table for the
// layers that rotate with another base follows at rope[hd...] when theta2 > 0. The table is the work of
// the upper two wavefronts (powers and range reductions: hundreds of instructions), the row of the lower two.
struct EmbedArgs {
    const uint8_t *q;
    const float *scales;
    const uint8_t *zp;
    const float *w;   // the first layer's input norm
    float *x, *xn, *rope;
    int hidden, bs, n_blocks, hd;
    float embed_scale, eps, theta, theta2;
};
// the rotary table of position `pos`: the work of threads 128 .. 255
__device__ __forceinline__ void dec_rope_table(const EmbedArgs &e, int pos) {
    if (threadIdx.x >= 128) {
        for (int j = threadIdx.x - 128; j < e.hd / 2; j += 128) {
            const float ang = (float)pos * powf(e.theta, -2.f * (float)j / (float)e.hd);
            e.rope[j] = cosf(ang), e.rope[e.hd / 2 + j] = sinf(ang);
            if (e.theta2 > 0.f) {
                const float ang2 = (float)pos * powf(e.theta2, -2.f * (float)j / (float)e.hd);
                e.rope[e.hd + j] = cosf(ang2), e.rope[e.hd + e.hd / 2 + j] = sinf(ang2);
            }
        }
    }
}
// ROPE: the table is worked out here, between asking for the row and using it (else the caller has done it)
template <bool ROPE>
__device__ __forceinline__ void dec_embed_token(const EmbedArgs &e, int token, int pos, float *red) {
    const size_t row = (size_t)token;
    const size_t row_bytes = (size_t)e.n_blocks * e.bs / 2, zp_row = (e.n_blocks + 1) / 2;
    // The row comes from a table far larger than any cache: every load of it is a trip to memory, so all of them are
    // asked for at once -- a thread takes eight consecutive elements (one word of nibbles, one scale, one zero-point
    // byte) of up to two places of the row -- and the rotary table is worked out while they are on their way.
    constexpr int kPlaces = 2;
    const bool wide = e.hidden % 8 == 0 && e.bs % 8 == 0 && e.hidden <= 256 * 8 * kPlaces;
    uint32_t word[kPlaces];
    float sc[kPlaces], v[kPlaces][8];
    float4 w_lo[kPlaces], w_hi[kPlaces];
    int zq[kPlaces];
    if (wide) {
#pragma unroll
        for (int u = 0; u < kPlaces; u++) {
            const int k0 = min(((int)threadIdx.x + 256 * u) * 8, e.hidden - 8), b = k0 / e.bs;
            word[u] = *reinterpret_cast<const uint32_t *>(e.q + row * row_bytes + k0 / 2);
            sc[u] = e.scales[row * e.n_blocks + b];
            zq[u] = e.zp ? (e.zp[row * zp_row + b / 2] >> (4 * (b & 1))) & 15 : 8;
            w_lo[u] = *reinterpret_cast<const float4 *>(e.w + k0), w_hi[u] = *reinterpret_cast<const float4 *>(e.w + k0 + 4);
        }
    }
    if (ROPE) dec_rope_table(e, pos);
    float sq = 0.f;
    if (wide) {
#pragma unroll
        for (int u = 0; u < kPlaces; u++) {
            const int k0 = ((int)threadIdx.x + 256 * u) * 8;
            if (k0 < e.hidden) {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    v[u][i] = ((float)((word[u] >> (4 * i)) & 15u) - (float)zq[u]) * sc[u] * e.embed_scale;
                    sq += v[u][i] * v[u][i];
                }
                reinterpret_cast<float4 *>(e.x + k0)[0] = make_float4(v[u][0], v[u][1], v[u][2], v[u][3]);
                reinterpret_cast<float4 *>(e.x + k0)[1] = make_float4(v[u][4], v[u][5], v[u][6], v[u][7]);
            }
        }
    } else {
        for (int c = threadIdx.x; c < e.hidden; c += 256) {
            const int b = c / e.bs;
            const int nib = (e.q[row * row_bytes + c / 2] >> (4 * (c & 1))) & 15;
            const int z = e.zp ? (e.zp[row * zp_row + b / 2] >> (4 * (b & 1))) & 15 : 8;
            const float val = ((float)nib - (float)z) * e.scales[row * e.n_blocks + b] * e.embed_scale;
            e.x[c] = val;
            sq += val * val;
        }
    }
    const float inv = rsqrtf(block_sum(sq, red) / (float)e.hidden + e.eps);
    if (wide) {
#pragma unroll
        for (int u = 0; u < kPlaces; u++) {
            const int k0 = ((int)threadIdx.x + 256 * u) * 8;
            if (k0 < e.hidden) {
                reinterpret_cast<float4 *>(e.xn + k0)[0] = make_float4(v[u][0] * inv * w_lo[u].x, v[u][1] * inv * w_lo[u].y, v[u][2] * inv * w_lo[u].z, v[u][3] * inv * w_lo[u].w);
                reinterpret_cast<float4 *>(e.xn + k0)[1] = make_float4(v[u][4] * inv * w_hi[u].x, v[u][5] * inv * w_hi[u].y, v[u][6] * inv * w_hi[u].z, v[u][7] * inv * w_hi[u].w);
            }
        }
    } else {
        for (int c = threadIdx.x; c < e.hidden; c += 256) e.xn[c] = e.x[c] * inv * e.w[c];   // (x[c] is this thread's own store)
    }
}
__global__ void __launch_bounds__(256) dec_embed_kernel(const DecState *st, const EmbedArgs e) {
    __shared__ float red[4];
    dec_embed_token<true>(e, st->token, st->pos, red);
}

// x += rmsnorm(y, w_post); xn = rmsnorm(x, w_next). One workgroup of 256; every operand is read once,
// up front (hidden <= 256 * kNormPer), so the kernel costs one memory round trip and two reductions.
constexpr int kNormPer = 8;
// y may arrive as y_slices partial rows (the k slices of the product that made it), hidden apart.
__global__ void __launch_bounds__(256)
dec_norm_residual_kernel(const float *__restrict__ y, int y_slices, const float *__restrict__ w_post, const float *__restrict__ w_next,
                         int hidden, float eps, const float *__restrict__ x_in, float *__restrict__ x, float *__restrict__ xn) {
    __shared__ float red[4];
    HIPC_ARG_NOW(y); HIPC_ARG_NOW(y_slices); HIPC_ARG_NOW(w_post); HIPC_ARG_NOW(w_next); HIPC_ARG_NOW(hidden); HIPC_ARG_NOW(eps);
    HIPC_ARG_NOW(x_in); HIPC_ARG_NOW(x); HIPC_ARG_NOW(xn);
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
// the half-split rotary embedding at `pos`; k goes to the f16 cache row `pos`, v to column `pos` of the transposed value cache; q stays f32.
__global__ void __launch_bounds__(256)
dec_qkv_kernel(const DecState *st, const float *__restrict__ qkv, const float *__restrict__ q_norm,
               const float *__restrict__ k_norm, int n_q, int n_kv, int hd, float eps, float theta, int max_seq, int v_stride,
               float *__restrict__ q_out, __half *__restrict__ k_cache, __half *__restrict__ v_cache) {
    __shared__ float red[4];
    __shared__ float buf[512];
    const int head = blockIdx.x;
    const int pos = st->pos;
    if (pos >= max_seq) return;  // the cache is full: the step is a no-op (dec_pick_embed_kernel reports it)
    const float *src = qkv + (size_t)head * hd;
    const bool is_q = head < n_q, is_k = !is_q && head < n_q + n_kv;
    if (!is_q && !is_k) {  // a value head: straight into the cache
        const int kvh = head - n_q - n_kv;
        for (int d = threadIdx.x; d < hd; d += 256)
            v_cache[((size_t)kvh * hd + d) * v_stride + pos] = __float2half(src[d]);
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
                        const __half *__restrict__ v_cache, int n_q, int n_kv, int hd, int max_seq, int v_stride, float scale, int window,
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
    // values first: thread d owns channel d (and d + 256): the chunk's 16 positions are 32 consecutive
    // bytes of the transposed cache (positions past the end have weight zero below)
    float vreg[2][kAttnChunk];
    static_assert(kAttnChunk == 16, "two 16-byte loads per channel");
#pragma unroll
    for (int c = 0; c < 2; c++) {
        const int d = min(tid + c * 256, hd - 1);
        const uint4 *src = reinterpret_cast<const uint4 *>(v_cache + ((size_t)kvh * hd + d) * v_stride + t0);
        const uint4 va = src[0], vb = src[1];
        const __half2 *ha = reinterpret_cast<const __half2 *>(&va), *hb = reinterpret_cast<const __half2 *>(&vb);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            vreg[c][2 * e] = __low2float(ha[e]), vreg[c][2 * e + 1] = __high2float(ha[e]);
            vreg[c][8 + 2 * e] = __low2float(hb[e]), vreg[c][8 + 2 * e + 1] = __high2float(hb[e]);
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
    const int live = even_chunks ? attn_live_chunks(attn_span(total, window)) : min(nsplit, (st->pos + kAttnChunk) / kAttnChunk);
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
// Workgroup (split, kvh) owns attn_chunk(span) consecutive positions of kv head kvh, walks them
// kAttnPass = 32 at a time and serves all G query heads of the group. What bounds the kernel is the
// rate at which one CU takes K and V in (64 bytes a clock), so a chunk is as short as the join of the
// partials allows: 32 positions while the span is at most 2048. Both products run on the matrix
// cores, 16x16x32 f16:
//   scores   S[row, t] = sum_d q[row, d] K[t, d]: wavefront (pb, dh) multiplies positions 16 pb .. + 16
//            by half dh of the channels; the B operand of position t is 16 bytes of the row-major key
//            cache as they lie; the A operand's rows 2 g and 2 g + 1 are head g's query as two f16
//            terms (hi = f16(q), lo = f16(q - hi): 22 bits), so that a lane's result registers (rows
//            4 j .. 4 j + 3) add up to two heads' scores. The halves meet in LDS (one barrier);
//   softmax  every wavefront forms the pass's weights for all 32 positions (the same arithmetic in
//            each: nothing to exchange, and all hold the same running max and sum);
//   outputs  O[row, c] = sum_t p[row, t] V[t, c]: wavefront w multiplies all 32 positions by its
//            quarter of the channels; the B operand of channel c is 16 bytes (8 positions) of the
//            TRANSPOSED value cache [kv head][channel][position]; the A operand's rows are the heads'
//            weights as two f16 terms, turned from the scores' layout (lane = position) into the
//            operand's (lane = row) through the wavefront's own LDS rows.
// A wavefront's outputs are complete for its channels, so there is nothing to join at the end. The
// step's own position never comes from the cache: the workgroup that owns it (the last live one)
// writes the cache rows and adds q.k_new / v_new to its running triple. A workgroup writes (max, sum)
// per head and the unnormalised output: the flash-decoding partial that the consumer joins over the
// live chunks (the output projection's prologue, or dec_attn_merge_kernel).
// Nothing branches on the position before the end: a workgroup without positions runs on with empty
// descriptors and skips the stores. (An early exit would let the compiler sink the first loads
// below the wait for the position.) HD and G are template parameters: straight-line code.
typedef _Float16 dh16x8 __attribute__((ext_vector_type(8)));
typedef float df32x4 __attribute__((ext_vector_type(4)));

// phase time stamps of the attention launch (library built with `make stamps` only; see gemv_lean.hip):
// attn_stamps[split][wavefront][phase] of kv head 0, read out by hipc_debug_attn_stamps
#ifdef HIPC_PHASE_STAMPS
__device__ unsigned long long attn_stamps[64 * 4 * 12];
#define ATTN_STAMP(ph)                                                                                          \
    do {                                                                                                        \
        const unsigned long long t_ = (unsigned long long)wall_clock64();                                       \
        if ((threadIdx.x & 63) == 0 && blockIdx.y == 0) attn_stamps[(blockIdx.x * 4 + (threadIdx.x >> 6)) * 12 + (ph)] = t_; \
    } while (0)
#define ATTN_STAMP_AFTER(v, ph) do { asm volatile("" ::"v"(v)); ATTN_STAMP(ph); } while (0)
#else
#define ATTN_STAMP(ph)
#define ATTN_STAMP_AFTER(v, ph)
#endif
template <int HD, int G>
__global__ void __launch_bounds__(256)
dec_attn_chunks_kernel(const DecState *st, const float *__restrict__ qkv, const float *__restrict__ q_norm,
                       const float *__restrict__ k_norm, int n_q, int n_kv, float eps, const float *__restrict__ rope,
                       int max_seq, int v_stride, float scale, int window, __half *__restrict__ k_cache, __half *__restrict__ v_cache,
                       float *__restrict__ part_ml, float *__restrict__ part_o, const PrefetchArgs pf) {
    constexpr int GH = G * HD, NK = HD / 64, HALF = HD / 2;
    constexpr int KS = HD / 64;                // 32-channel steps of a wavefront's half of the score product
    constexpr int NB = HD / 64;                // 16-channel blocks of a wavefront's quarter of the output product
    constexpr int R = 2 * G;                   // operand rows in use: two terms per head
    constexpr int ROWS = (G + 1 + 3) / 4;      // q heads and the k head, dealt to four wavefronts
    constexpr int QS = HD + 8;                 // halfs per operand row of q (16 bytes of padding: rows start in different banks)
    constexpr int PS = kAttnPass + 8;          // halfs per operand row of p
    constexpr int HL = (G + 1) / 2;            // rows of 16 lanes that hold scores (two heads each)
    constexpr float NEG = -3.0e38f;
    static_assert(kAttnPass == 32, "two blocks of 16 positions; the output product's k");
    __shared__ __attribute__((aligned(16))) __half qa[R * QS];       // query heads, normed, rotated, scaled: rows 2 g + term
    __shared__ __attribute__((aligned(16))) float4 sp[4][64];          // per wavefront: its half of the scores, as the lanes hold them
    __shared__ __attribute__((aligned(16))) __half pa[4][16 * PS];    // per wavefront: the pass's weights, rows as in qa
    __shared__ __attribute__((aligned(16))) float kn[HD];             // the step's key, as the cache will hold it
    __shared__ __attribute__((aligned(16))) float vn[HD];             // the step's value
    __shared__ float sown[2 * HL];                                      // the step's own scores

    // every argument is read here, in one batch (left to the compiler, each is read next to its first use: a trip to
    // memory of its own in the middle of the kernel, since the scalar cache starts every launch empty)
    HIPC_ARG_NOW(st); HIPC_ARG_NOW(qkv); HIPC_ARG_NOW(q_norm); HIPC_ARG_NOW(k_norm); HIPC_ARG_NOW(n_q); HIPC_ARG_NOW(n_kv);
    HIPC_ARG_NOW(eps); HIPC_ARG_NOW(rope); HIPC_ARG_NOW(max_seq); HIPC_ARG_NOW(v_stride); HIPC_ARG_NOW(scale); HIPC_ARG_NOW(window);
    HIPC_ARG_NOW(k_cache); HIPC_ARG_NOW(v_cache); HIPC_ARG_NOW(part_ml); HIPC_ARG_NOW(part_o);
    if (__builtin_expect((int)blockIdx.y >= n_kv, 0)) {   // a helper row: read ahead for the next launch, nothing else
        prefetch_for_next(pf, ((int)blockIdx.y - n_kv) * (int)gridDim.x + (int)blockIdx.x, pf.rows * (int)gridDim.x,
                          (int)blockIdx.y * (int)gridDim.x + (int)blockIdx.x, pf.sink);
        return;
    }
    ATTN_STAMP(0);
    const int split = blockIdx.x, kvh = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int pb = wave & 1, dh = wave >> 1;
    const int i16 = lane & 15, g4 = lane >> 4;
    const int pos = st->pos;

    // 1. the step's own rows (they come out of L2 and are needed first): rows 0..G-1 are the query
    //    heads, row G the key head; wavefront w prepares rows w, w + 4, ...; lane l holds elements
    //    l + 64 i of a row
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

    const int total = pos + 1;
    const int t_first = attn_first(total, window);  // a local layer sees the last `window` positions only
    const int base = t_first & ~15;
    const int chunk = attn_chunk(total - base);
    const int t_begin = base + split * chunk;
    const bool dead = pos >= max_seq || t_begin >= total;   // the cache is full (the step is a no-op), or no position of this chunk exists yet
    const int t_end = min(total, t_begin + chunk);
    const bool is_last = !dead && t_end == total;           // this workgroup owns the step's own position
    const int hist_end = min(t_end, pos);                   // positions below come from the cache

    //    K: step u of lane (position i16 of block pb, quarter g4) reads channels 32 u + 8 g4 .. + 8 of
    //    half dh: the four quarters of a position ask for 64 consecutive bytes in one instruction;
    //    V: lane (channel i16 of a block, quarter g4) reads positions 8 g4 .. + 8 of the pass. Rows past the end of the cache are
    //    padding; positions that do not count are masked below.
    const __amdgpu_buffer_rsrc_t r_k = __builtin_amdgcn_make_buffer_rsrc(
        k_cache, 0, dead ? 0 : (int)(((uint32_t)n_kv * (uint32_t)max_seq + 64u) * HD * 2u), 0x00020000);
    const __amdgpu_buffer_rsrc_t r_v = __builtin_amdgcn_make_buffer_rsrc(
        v_cache, 0, dead ? 0 : (int)((uint32_t)n_kv * HD * (uint32_t)v_stride * 2u), 0x00020000);
    const uint32_t v_k = (uint32_t)((pb * 16 + i16) * HD + dh * HALF + g4 * 8) * 2u;
    const uint32_t v_v = ((uint32_t)(wave * (HD / 4) + i16) * (uint32_t)v_stride + (uint32_t)(g4 * 8)) * 2u;
    uint4 kreg[KS], vreg[NB];
    auto load_k = [&](int t0) {
        const uint32_t s_k = ((uint32_t)kvh * (uint32_t)max_seq + (uint32_t)t0) * HD * 2u;
#pragma unroll
        for (int u = 0; u < KS; u++) kreg[u] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(r_k, (int)(v_k + u * 64u), (int)s_k, 0));
    };
    auto load_v = [&](int t0) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const uint32_t s_v = (((uint32_t)kvh * HD + b * 16u) * (uint32_t)v_stride + (uint32_t)t0) * 2u;
            vreg[b] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(r_v, (int)v_v, (int)s_v, 0));
        }
    };
    ATTN_STAMP(1);
    load_k(t_begin);
    load_v(t_begin);
    ATTN_STAMP(2);

    // 2. per-head RMS norm and half-split rotary embedding (pairs d, d + HD/2), one wavefront per
    //    row and no workgroup barrier: with HD = 128 or 256 both members of a pair sit in one lane
    //    (elements i and i + NK/2), with HD = 64 in lanes l and l + 32. Query rows are scaled and
    //    kept (for the step's own score); only the workgroup that owns the position prepares k.
    float rq[ROWS][NK];
#pragma unroll
    for (int rr = 0; rr < ROWS; rr++) {
        const int row = wave + 4 * rr;
        if (row < G || (row == G && is_last)) {
            float sq = 0.f;
#pragma unroll
            for (int i = 0; i < NK; i++) sq += px[rr][i] * px[rr][i];
            sq = lean_wave_sum(sq);
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
            if (row < G) {
#pragma unroll
                for (int i = 0; i < NK; i++) {
                    const float v = r[i] * scale;
                    const __half hi = __float2half(v);
                    rq[rr][i] = v;
                    qa[(2 * row) * QS + lane + 64 * i] = hi;
                    qa[(2 * row + 1) * QS + lane + 64 * i] = __float2half(v - __half2float(hi));
                }
            } else {
#pragma unroll
                for (int i = 0; i < NK; i++) kn[lane + 64 * i] = __half2float(__float2half(r[i]));
            }
        }
    }
    if (is_last && tid < HD) vn[tid] = __half2float(__float2half(pv_own));
    ATTN_STAMP(3);
    __syncthreads();
    ATTN_STAMP(4);
    if (is_last) {
        if (tid < HD) {
            k_cache[((size_t)kvh * max_seq + pos) * HD + tid] = __float2half(kn[tid]);
            v_cache[((size_t)kvh * HD + tid) * v_stride + pos] = __float2half(vn[tid]);
        }
#pragma unroll
        for (int rr = 0; rr < ROWS; rr++) {
            const int row = wave + 4 * rr;
            if (row < G) {
                float dot = 0.f;
#pragma unroll
                for (int i = 0; i < NK; i++) dot = fmaf(rq[rr][i], kn[lane + 64 * i], dot);
                dot = lean_wave_sum(dot);
                if (lane == 0) sown[row] = dot;
            }
        }
    }

    // 3. the query operand: row i16 (rows past the last in use: zeros), channels in the key loads' order
    dh16x8 aq[KS];
#pragma unroll
    for (int u = 0; u < KS; u++) {
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (i16 < R) raw = *reinterpret_cast<const uint4 *>(qa + i16 * QS + dh * HALF + u * 32 + g4 * 8);
        aq[u] = __builtin_bit_cast(dh16x8, raw);
    }

    float m_run0 = NEG, m_run1 = NEG, l_run0 = 0.f, l_run1 = 0.f;   // heads 2 g4 and 2 g4 + 1; the same in every lane of a row of 16 and in every wavefront
    df32x4 o[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) o[b] = df32x4{0.f, 0.f, 0.f, 0.f};

    ATTN_STAMP_AFTER(aq[KS - 1], 5);
    for (int t0 = t_begin; t0 < t_end; t0 += kAttnPass) {   // (a workgroup without positions: not once)
        const bool more = t0 + kAttnPass < t_end;
        // 3a. this wavefront's half of the scores of its 16 positions, all heads
        df32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < KS; u++) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(aq[u], __builtin_bit_cast(dh16x8, kreg[u]), acc, 0, 0, 0);
        sp[wave][lane] = make_float4(acc[0], acc[1], acc[2], acc[3]);
        if (t0 == t_begin) ATTN_STAMP_AFTER(acc[0], 6);
        if (more) load_k(t0 + kAttnPass);
        __syncthreads();
        // 3b. all 32 positions' scores (block b: wavefronts b and b + 2), the pass's max and sum
        float s0[2], s1[2], p0[2], p1[2];
        bool valid[2];
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const float4 lo = sp[b][lane], hi = sp[b + 2][lane];
            const int t = t0 + b * 16 + i16;
            valid[b] = t >= t_first && t < hist_end;
            s0[b] = valid[b] ? (lo.x + hi.x) + (lo.y + hi.y) : NEG;
            s1[b] = valid[b] ? (lo.z + hi.z) + (lo.w + hi.w) : NEG;
        }
        const float m0 = fmaxf(m_run0, lean_row_max(fmaxf(s0[0], s0[1]))), m1 = fmaxf(m_run1, lean_row_max(fmaxf(s1[0], s1[1])));
        const float f0 = __expf(m_run0 - m0), f1 = __expf(m_run1 - m1);
#pragma unroll
        for (int b = 0; b < 2; b++) p0[b] = valid[b] ? __expf(s0[b] - m0) : 0.f, p1[b] = valid[b] ? __expf(s1[b] - m1) : 0.f;
        l_run0 = fmaf(l_run0, f0, lean_row_sum(p0[0] + p0[1])), l_run1 = fmaf(l_run1, f1, lean_row_sum(p1[0] + p1[1]));
        m_run0 = m0, m_run1 = m1;
        //     weights as two f16 terms into the wavefront's LDS rows 4 g4 .. 4 g4 + 3, column = position
        if (g4 < HL) {
#pragma unroll
            for (int b = 0; b < 2; b++) {
                const __half h0 = __float2half(p0[b]), h1 = __float2half(p1[b]);
                __half *dst = pa[wave] + (4 * g4) * PS + b * 16 + i16;
                dst[0] = h0, dst[PS] = __float2half(p0[b] - __half2float(h0));
                dst[2 * PS] = h1, dst[3 * PS] = __float2half(p1[b] - __half2float(h1));
            }
        }
        // the rows are this wavefront's own: its LDS operations complete in order, the compiler only must not reorder them
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        uint4 praw = make_uint4(0, 0, 0, 0);
        if (i16 < R) praw = *reinterpret_cast<const uint4 *>(pa[wave] + i16 * PS + g4 * 8);
        const dh16x8 ap = __builtin_bit_cast(dh16x8, praw);
        if (t0 == t_begin) ATTN_STAMP_AFTER(praw.x, 7);
        // 3c. unnormalised outputs of this wavefront's channels: a lane's result registers are rows
        //     4 g4 .. + 3, the heads whose factors it holds
#pragma unroll
        for (int b = 0; b < NB; b++) {
            o[b][0] *= f0, o[b][1] *= f0, o[b][2] *= f1, o[b][3] *= f1;
            o[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ap, __builtin_bit_cast(dh16x8, vreg[b]), o[b], 0, 0, 0);
        }
        if (t0 == t_begin) ATTN_STAMP_AFTER(o[NB - 1][0], 8);
        if (more) {
            load_v(t0 + kAttnPass);
            __syncthreads();   // the next pass's scores must not overtake this pass's reads of sp
        }
    }
    ATTN_STAMP_AFTER(o[0][0], 9);

    // 4. the step's own position joins in the workgroup that owns it; then the partial goes out
    float e0 = 1.f, e1 = 1.f, eo0 = 0.f, eo1 = 0.f;
    if (is_last) {
        const float so0 = sown[min(2 * g4, 2 * HL - 1)], so1 = sown[min(2 * g4 + 1, 2 * HL - 1)];
        const float M0 = fmaxf(m_run0, so0), M1 = fmaxf(m_run1, so1);
        e0 = __expf(m_run0 - M0), e1 = __expf(m_run1 - M1), eo0 = __expf(so0 - M0), eo1 = __expf(so1 - M1);
        m_run0 = M0, m_run1 = M1;
        l_run0 = fmaf(l_run0, e0, eo0), l_run1 = fmaf(l_run1, e1, eo1);
    }
    if (dead) return;
    float *po = part_o + ((size_t)kvh * kAttnSplits + split) * GH;
    float *ml = part_ml + ((size_t)kvh * kAttnSplits + split) * G * 2;
    if (g4 < HL) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
            const int ch = wave * (HD / 4) + b * 16 + i16;
            const float own = is_last ? vn[ch] : 0.f;
            po[(2 * g4) * HD + ch] = fmaf(o[b][0] + o[b][1], e0, eo0 * own);
            if (2 * g4 + 1 < G) po[(2 * g4 + 1) * HD + ch] = fmaf(o[b][2] + o[b][3], e1, eo1 * own);
        }
        if (wave == 0 && i16 == 0) {
            ml[4 * g4] = m_run0, ml[4 * g4 + 1] = l_run0;
            if (2 * g4 + 1 < G) ml[4 * g4 + 2] = m_run1, ml[4 * g4 + 3] = l_run1;
        }
    }
    ATTN_STAMP(10);
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
constexpr int kArgmaxParts = 256;   // workgroups of the separate scan over the logits
constexpr int kArgmaxCap = 1024;    // candidates the token pick takes: the scan's, or one per workgroup of an lm_head launch that leaves them
__global__ void __launch_bounds__(256)
dec_argmax_partial_kernel(const float *__restrict__ logits, int n, float *__restrict__ pv, int *__restrict__ pi) {
    __shared__ float sv[4];
    __shared__ int si[4];
    float best = -3.4e38f;
    int bi = 0x7fffffff;
    auto take = [&](float v, int i) {
        if (v > best || (v == best && i < bi)) best = v, bi = i;
    };
    // four logits per load (the logits buffer is the library's own allocation: 16-byte aligned); with a vocabulary of
    // 2^18 that is one load per thread, in flight together with every other thread's
    const int n4 = n >> 2;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n4; i += gridDim.x * 256) {
        const float4 v = reinterpret_cast<const float4 *>(logits)[i];
        take(v.x, 4 * i), take(v.y, 4 * i + 1), take(v.z, 4 * i + 2), take(v.w, 4 * i + 3);
    }
    for (int i = 4 * n4 + blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) take(logits[i], i);
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
// The same launch then embeds the chosen token for the next step (x, xn and the rotary table of the new
// position): a step begins with its q|k|v product, not with a launch of its own for the embedding.
__global__ void __launch_bounds__(256)
dec_pick_embed_kernel(const float *__restrict__ pv, const int *__restrict__ pi, int nparts, DecState *st,
                      int32_t *__restrict__ history, int max_hist, int vocab, const EmbedArgs e) {
    __shared__ float red[4];
    __shared__ int next[2];
    // the upper two wavefronts work out the next position's rotary table (it follows from the position alone) while
    // the first picks the token
    const int pos_now = st->pos, token_now = st->token;   // (both read here, once: asked for again after the pick they would be a trip to memory on its critical path)
    dec_rope_table(e, pos_now >= max_hist ? pos_now : pos_now + 1);
    if (threadIdx.x < 64) {
        float best = -3.4e38f;
        int bi = 0x7fffffff;
        // up to kArgmaxCap candidates: a lane's sixteen are asked for together, then compared
        float cv[kArgmaxCap / 64];
        int ci[kArgmaxCap / 64];
#pragma unroll
        for (int u = 0; u < kArgmaxCap / 64; u++) {
            const int i = min((int)threadIdx.x + 64 * u, nparts - 1);
            cv[u] = pv[i], ci[u] = pi[i];
        }
#pragma unroll
        for (int u = 0; u < kArgmaxCap / 64; u++)
            if ((int)threadIdx.x + 64 * u < nparts && (cv[u] > best || (cv[u] == best && ci[u] < bi))) best = cv[u], bi = ci[u];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const float ov = __shfl_xor(best, off, 64);
            const int oi = __shfl_xor(bi, off, 64);
            if (ov > best || (ov == best && oi < bi)) best = ov, bi = oi;
        }
        if (threadIdx.x == 0) {
            const int pos = pos_now;
            int token = token_now, new_pos = pos;
            if (pos >= max_hist) {
                st->overflow = 1;
            } else {
                if (bi < 0 || bi >= vocab) bi = 0;
                history[pos] = bi;
                st->token = token = bi;
                st->pos = new_pos = pos + 1;
            }
            next[0] = token, next[1] = new_pos;
        }
    }
    __syncthreads();
    dec_embed_token<false>(e, next[0], next[1], red);
}

__global__ void dec_set_state_kernel(DecState *st, int token, int pos) {
    if (threadIdx.x == 0) st->token = token, st->pos = pos, st->overflow = 0;
}

}  // namespace hipc

using namespace hipc;

#ifdef HIPC_PHASE_STAMPS
extern "C" int hipc_debug_attn_stamps(void *dst, size_t bytes) {
    return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(hipc::attn_stamps), bytes, 0, hipMemcpyDeviceToHost);
}
#endif

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
    uint32_t *pf_sink = nullptr;   // where a helper workgroup would write (it never does: keeps its loads alive)
    // x, xn and the rotary table hold the state's token and position (left by the reset or by the step before);
    // anything that changes what they are made of clears it, and a step that finds it cleared embeds first
    bool x_ready = false;
    bool one_launch_attn = false;  // head_dim and group size have an instance of dec_attn_chunks_kernel
    std::vector<void *> owned;
};

namespace {


template <typename T>
int dev_alloc(hipc_ctx *ctx, hipc_decoder *d, T **p, size_t count) {
    HIPC_TRY(ctx, hipMalloc(reinterpret_cast<void **>(p), std::max<size_t>(count * sizeof(T), 16)));
    d->owned.push_back(*p);
    return HIPC_OK;
}

template <int HD, int G>
void attn_chunks_launch(hipc_ctx *ctx, hipc_decoder *d, DecLayer &l, float scale, const PrefetchArgs &pf) {
    const hipc_decoder_config &c = d->cfg;
    hipLaunchKernelGGL((dec_attn_chunks_kernel<HD, G>), dim3(kAttnSplits, c.n_kv_heads + (pf.kind ? pf.rows : 0)), 256, 0, ctx->stream, d->state, d->qkv, l.norm[HIPC_DEC_NORM_Q], l.norm[HIPC_DEC_NORM_K], c.n_q_heads, c.n_kv_heads, c.rms_eps,
        d->rope + (size_t)l.rope_table * c.head_dim, c.max_seq, attn_v_stride(c.max_seq), scale, l.window, l.k_cache, l.v_cache,
        d->part_ml, d->part_o, pf);
}

template <int HD>
void attn_chunks_launch_g(hipc_ctx *ctx, hipc_decoder *d, DecLayer &l, float scale, int G, const PrefetchArgs &pf) {
    switch (G) {
        case 1: attn_chunks_launch<HD, 1>(ctx, d, l, scale, pf); break;
        case 2: attn_chunks_launch<HD, 2>(ctx, d, l, scale, pf); break;
        case 4: attn_chunks_launch<HD, 4>(ctx, d, l, scale, pf); break;
        default: attn_chunks_launch<HD, 8>(ctx, d, l, scale, pf); break;
    }
}

// pf: what the launch's helper rows read ahead for the launch after it (kind 0: no helper rows)
int launch_attn_chunks(hipc_ctx *ctx, hipc_decoder *d, DecLayer &l, float scale, const PrefetchArgs &pf = PrefetchArgs()) {
    const int G = d->cfg.n_q_heads / d->cfg.n_kv_heads;
    switch (d->cfg.head_dim) {
        case 64: attn_chunks_launch_g<64>(ctx, d, l, scale, G, pf); break;
        case 128: attn_chunks_launch_g<128>(ctx, d, l, scale, G, pf); break;
        default: attn_chunks_launch_g<256>(ctx, d, l, scale, G, pf); break;
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
        // keys [kv head][position][channel] with a pass of padding rows behind the last head (the one-launch
        // attention reads whole passes); values transposed, [kv head][channel][position], rows of v_stride
        const size_t k_halfs = ((size_t)c.n_kv_heads * c.max_seq + 64) * c.head_dim;
        // (+ a pass: a chunk that starts less than a pass before the end of a row reads on into the next row,
        // the last row's into this padding; those positions are masked)
        const size_t v_halfs = (size_t)c.n_kv_heads * c.head_dim * attn_v_stride(c.max_seq) + 2 * kAttnPass;
        const int G = c.n_q_heads / c.n_kv_heads;
        int rc = HIPC_OK;
        auto A = [&](auto **p, size_t n) { if (rc == HIPC_OK) rc = dev_alloc(ctx, d, p, n); };
        for (DecLayer &l : d->layers) {
            A(&l.k_cache, k_halfs);
            A(&l.v_cache, v_halfs);
        }
        A(&d->state, 1), A(&d->history, (size_t)c.max_seq);
        A(&d->x, c.hidden), A(&d->xn, c.hidden), A(&d->qkv, (size_t)(c.n_q_heads + 2 * c.n_kv_heads) * c.head_dim);
        A(&d->q, (size_t)c.n_q_heads * c.head_dim), A(&d->attn, (size_t)c.n_q_heads * c.head_dim), A(&d->y, c.hidden);
        A(&d->gu, (size_t)2 * c.ffn), A(&d->h, c.ffn), A(&d->logits, c.vocab);
        const size_t parts = (size_t)c.n_kv_heads * std::max(d->nsplit, kAttnSplits) * G;
        A(&d->part_ml, parts * 2), A(&d->part_o, parts * c.head_dim);
        A(&d->am_v, kArgmaxCap), A(&d->am_i, kArgmaxCap);
        A(&d->pf_sink, 4);
        A(&d->rope, (size_t)2 * c.head_dim), A(&d->x2, c.hidden);
        // options read when the decoder is created: dec_fused_glue = 0 keeps the separate norm / GELU
        // kernels, dec_fused_attn = 0 the three-kernel attention (tests of those paths)
        d->fused_glue = c.hidden % 8 == 0 && c.ffn % 8 == 0 && ctx->tune.dec_fused_glue != 0;
        d->one_launch_attn = (c.head_dim == 64 || c.head_dim == 128 || c.head_dim == 256) && (G == 1 || G == 2 || G == 4 || G == 8) &&
                             k_halfs * 2 < (1ull << 32) && v_halfs * 2 < (1ull << 32) &&   // 32-bit buffer offsets
                             ctx->tune.dec_fused_attn != 0;
        // the lean path (the dec_lean option set to 0 keeps the streaming kernel and its prologues)
        {
            const int n_cg_h = (int)ceil_div(c.hidden, 128), n_cg_o = (int)ceil_div((int64_t)c.n_q_heads * c.head_dim, 128);
            const int n_cg_f = (int)ceil_div(c.ffn, 128);
            d->lean = d->fused_glue && d->one_launch_attn && ctx->tune.dec_lean != 0 && c.ffn % 16 == 0 && n_cg_h <= 32 &&
                      c.hidden % 8 == 0;
            // output projection: a k slice is one head (or one 128-k tile when heads are shorter), at most 4 slices
            // (the consumer's norm prologue adds up at most four partial rows: every row is code it has to fetch)
            int o_tiles = std::max(1, c.head_dim / 128);
            while (ceil_div(n_cg_o, o_tiles) > 4 && o_tiles < 4) o_tiles *= 2;
            d->o_slices = (int)ceil_div(n_cg_o, o_tiles);
            if (d->o_slices > 4 || o_tiles > 4) d->lean = false;
            // down projection: 18 k tiles per slice (six wavefronts of three tiles); a longer row in four slices of
            // up to 32 tiles (eight wavefronts of four)
            d->down_slices = (int)std::max<int64_t>(1, ceil_div(n_cg_f, 18));
            if (d->down_slices > 4) d->down_slices = 4;
            if (ceil_div(n_cg_f, d->down_slices) > 32) d->lean = false;
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
                if (hipMemsetAsync(l.k_cache, 0, k_halfs * 2, ctx->stream) != hipSuccess ||
                    hipMemsetAsync(l.v_cache, 0, v_halfs * 2, ctx->stream) != hipSuccess)
                    rc = fail(ctx, HIPC_ERR_BACKEND, "decoder: cannot clear the KV cache");
            }
            hipLaunchKernelGGL((dec_set_state_kernel), 1, 64, 0, ctx->stream, d->state, 0, 0);
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
        d->x_ready = false;
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
        d->x_ready = false;
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
        d->x_ready = false;   // the rotary table may need its second half
        return HIPC_OK;
    });
}

namespace {

bool can_embed(const hipc_decoder *d) { return d->emb_q && d->emb_scales && d->layers[0].norm[HIPC_DEC_NORM_INPUT]; }

EmbedArgs embed_args(const hipc_decoder *d) {
    const hipc_decoder_config &c = d->cfg;
    EmbedArgs e{};
    e.q = d->emb_q, e.scales = d->emb_scales, e.zp = d->emb_zp, e.w = d->layers[0].norm[HIPC_DEC_NORM_INPUT];
    e.x = d->x, e.xn = d->xn, e.rope = d->rope;
    e.hidden = c.hidden, e.bs = c.block_size, e.n_blocks = (int)ceil_div(c.hidden, c.block_size), e.hd = c.head_dim;
    e.embed_scale = c.embed_scale, e.eps = c.rms_eps, e.theta = c.rope_theta, e.theta2 = d->theta2;
    return e;
}

}  // namespace

int hipc_decoder_reset(hipc_ctx *ctx, hipc_decoder *d, int32_t token, int32_t pos) {
    if (!d) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, token >= 0 && token < d->cfg.vocab && pos >= 0 && pos < d->cfg.max_seq, "decoder: bad token %d or position %d", token, pos);
        hipLaunchKernelGGL((dec_set_state_kernel), 1, 64, 0, ctx->stream, d->state, token, pos);
        HIPC_LAUNCHED(ctx);
        // the step expects the token embedded (x, xn, the position's rotary table): every step leaves that behind for
        // the next one, the reset does it for the first
        d->x_ready = false;
        if (can_embed(d)) {
            hipLaunchKernelGGL((dec_embed_kernel), 1, 256, 0, ctx->stream, d->state, embed_args(d));
            HIPC_LAUNCHED(ctx);
            d->x_ready = !ctx->capturing;   // a recorded launch has not run yet
        }
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
        const int heads = c.n_q_heads + 2 * c.n_kv_heads;
        const float scale = c.attn_scale > 0.f ? c.attn_scale : 1.f / sqrtf((float)c.head_dim);
        const int terms = 2;
        int rc;
        if (!d->x_ready) {   // nothing has embedded the state's token yet (no reset since the weights changed)
            hipLaunchKernelGGL((dec_embed_kernel), 1, 256, 0, s, d->state, embed_args(d));
            HIPC_LAUNCHED(ctx);
        }
        // The residual stream alternates between two buffers: a GEMV whose prologue folds the previous
        // branch into the stream reads one and (its first workgroup) writes the other.
        float *xc = d->x, *xo = d->x2;
        // Launches of a layer may carry helper rows of workgroups that read ahead what the NEXT launch will read
        // (its weights, or the attention's cache rows) into the L2 of the XCD that will ask for it (prefetch.h).
        // The dec_prefetch option is a set of bits, one per producer: 1 q|k|v reads the attention's cache rows,
        // 2 the attention reads o's weights, 4 o reads gate|up's, 8 gate|up reads down's, 16 down reads the next
        // layer's q|k|v; 0 switches the helpers off. The default is 1 + 2 + 8: measured per producer on the
        // gemma3-1b shape at context 2048, those three save 0.2-0.6 us per launch, the o launch (72 workgroups of
        // its own) is lengthened by helpers that read gate|up's 10 MB, and the q|k|v launch hides its weights'
        // arrival behind its norm prologue anyway.
        const int ahead_mask = !kReadAheadVerified ? 0 : ctx->tune.dec_prefetch < 0 ? 9 : ctx->tune.dec_prefetch;
        // helper rows of a producer whose grid is gx wide: about one helper workgroup per consumer workgroup (a helper
        // that serves several consumers lasts longer than the launch it rides on), at least 192 and at most 512 in all
        auto rows_for = [](int64_t gx, int64_t consumers) {
            const int64_t want = std::min<int64_t>(512, std::max<int64_t>(192, consumers));
            return (int)std::max<int64_t>(1, std::min<int64_t>(32, (want + gx - 1) / gx));
        };
        for (int li = 0; li < c.n_layers && d->lean; li++) {
            DecLayer &l = d->layers[li];
            LeanPlan pl_qkv, pl_o, pl_gu, pl_down, pl_next;
            HIPC_REQUIRE(ctx, lean_plan(ctx, l.qkv, 1, 1, &pl_qkv, 8), "decoder: no launch plan for the qkv projection");
            pl_o = LeanPlan{1, (int)ceil_div(l.o->n_cg, d->o_slices), 4, d->o_slices};   // four wavefronts, each all k tiles of the slice: no sum over wavefronts
            HIPC_REQUIRE(ctx, lean_plan(ctx, l.gate_up, 1, 2, &pl_gu, 8), "decoder: no launch plan for the gate | up projection");
            HIPC_REQUIRE(ctx, lean_plan(ctx, l.down, d->down_slices, 1, &pl_down, 8), "decoder: no launch plan for the down projection");
            auto gx_of = [](const hipc_nbits_weight *w, const LeanPlan &p) { return ceil_div(w->n_tiles, p.WN); };
            // qkv: row = rmsnorm(x', w_input), x' = x + rmsnorm(sum of the down projection's partial rows, w_post_ffn of the layer before)
            {
                LeanArgs a{};
                a.x = xc, a.w_in = l.norm[HIPC_DEC_NORM_INPUT], a.x_out = xo, a.eps = c.rms_eps;
                if (li > 0) a.yparts = d->yd, a.y_slices = d->down_slices, a.w_post = d->layers[li - 1].norm[HIPC_DEC_NORM_POST_FFN];
                a.Y = d->qkv;
                if (ahead_mask & 1) {   // the attention's cache rows
                    PrefetchArgs &pf = a.pf;
                    pf.kind = 2, pf.rows = rows_for(gx_of(l.qkv, pl_qkv), (int64_t)kAttnSplits * c.n_kv_heads), pf.sink = d->pf_sink;
                    pf.pos = &d->state->pos, pf.k = l.k_cache, pf.v = l.v_cache, pf.window = l.window, pf.max_seq = c.max_seq;
                    pf.v_stride = attn_v_stride(c.max_seq), pf.hd = c.head_dim, pf.n_kv = c.n_kv_heads;
                }
                if ((rc = lean_gemv(ctx, l.qkv, pl_qkv, a, 2, 0, terms)) != HIPC_OK) return rc;
                std::swap(xc, xo);
            }
            {
                PrefetchArgs pf;
                if (ahead_mask & 2) {
                    pf = lean_prefetch_of(l.o, pl_o, rows_for(kAttnSplits, gx_of(l.o, pl_o) * pl_o.slices), d->pf_sink);
                    // only while the attention itself is long: behind a short one (a local layer's window, the first
                    // positions of a context) the helpers would be what the launch waits for
                    pf.pos = &d->state->pos, pf.gate_window = l.window, pf.gate_chunks = kAttnSplits / 2;
                }
                if ((rc = launch_attn_chunks(ctx, d, l, scale, pf)) != HIPC_OK) return rc;
            }
            // output projection: a k slice per head, joined from the attention partials; partial rows out
            {
                LeanArgs a{};
                a.part_o = d->part_o, a.part_ml = d->part_ml, a.pos = &d->state->pos;
                a.lg_group = __builtin_ctz((unsigned)(c.n_q_heads / c.n_kv_heads)), a.lg_hd = __builtin_ctz((unsigned)c.head_dim);   // powers of two where the one-launch attention runs
                a.n_kv = c.n_kv_heads, a.window = l.window;
                a.Y = d->yo;
                if (ahead_mask & 4) a.pf = lean_prefetch_of(l.gate_up, pl_gu, rows_for(gx_of(l.o, pl_o), gx_of(l.gate_up, pl_gu) * pl_gu.slices), d->pf_sink);
                if ((rc = lean_gemv(ctx, l.o, pl_o, a, 3, 0, terms)) != HIPC_OK) return rc;
            }
            // gate | up: row = rmsnorm(x'', w_pre_ffn), x'' = x' + rmsnorm(sum of the output projection's partial rows, w_post_attn);
            // epilogue gelu_tanh(gate) * up in operand order
            {
                LeanArgs a{};
                a.x = xc, a.w_in = l.norm[HIPC_DEC_NORM_PRE_FFN], a.x_out = xo, a.eps = c.rms_eps;
                a.yparts = d->yo, a.y_slices = d->o_slices, a.w_post = l.norm[HIPC_DEC_NORM_POST_ATTN];
                a.h_split = d->h_split;
                if (ahead_mask & 8) a.pf = lean_prefetch_of(l.down, pl_down, rows_for(gx_of(l.gate_up, pl_gu), gx_of(l.down, pl_down) * pl_down.slices), d->pf_sink);
                if ((rc = lean_gemv(ctx, l.gate_up, pl_gu, a, 2, 1, terms)) != HIPC_OK) return rc;
                std::swap(xc, xo);
            }
            // down: the gated row straight into the operand registers; partial rows out
            {
                LeanArgs a{};
                a.a_split = d->h_split;
                a.Y = d->yd;
                if ((ahead_mask & 16) && li + 1 < c.n_layers && lean_plan(ctx, d->layers[li + 1].qkv, 1, 1, &pl_next, 8))
                    a.pf = lean_prefetch_of(d->layers[li + 1].qkv, pl_next, rows_for(gx_of(l.down, pl_down), gx_of(d->layers[li + 1].qkv, pl_next)), d->pf_sink);
                if ((rc = lean_gemv(ctx, l.down, pl_down, a, 4, 0, terms)) != HIPC_OK) return rc;
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
                    hipLaunchKernelGGL((dec_attn_merge_kernel), c.n_q_heads, 256, (size_t)kAttnSplits * sizeof(float), s, d->state, d->part_ml, d->part_o, c.n_q_heads, c.n_kv_heads, c.head_dim, kAttnSplits, 1, l.window, d->attn);
                    HIPC_LAUNCHED(ctx);
                    if ((rc = nbits_gemv(ctx, d->attn, HIPC_F32, l.o, d->y, 1, terms)) != HIPC_OK) return rc;
                }
            } else {
                hipLaunchKernelGGL((dec_qkv_kernel), heads, 256, 0, s, d->state, d->qkv, l.norm[HIPC_DEC_NORM_Q], l.norm[HIPC_DEC_NORM_K], c.n_q_heads,
                                                     c.n_kv_heads, c.head_dim, c.rms_eps, l.rope_table ? d->theta2 : c.rope_theta, c.max_seq,
                                                     attn_v_stride(c.max_seq), d->q, l.k_cache, l.v_cache);
                HIPC_LAUNCHED(ctx);
                hipLaunchKernelGGL((dec_attn_partial_kernel), dim3(d->nsplit, c.n_kv_heads), 256, 0, s, d->state, d->q, l.k_cache, l.v_cache, c.n_q_heads, c.n_kv_heads,
                                                                                     c.head_dim, c.max_seq, attn_v_stride(c.max_seq), scale, l.window, d->part_ml, d->part_o);
                HIPC_LAUNCHED(ctx);
                hipLaunchKernelGGL((dec_attn_merge_kernel), c.n_q_heads, 256, (size_t)d->nsplit * sizeof(float), s, d->state, d->part_ml, d->part_o, c.n_q_heads, c.n_kv_heads,
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
                hipLaunchKernelGGL((dec_norm_residual_kernel), 1, 256, 0, s, d->y, 1, l.norm[HIPC_DEC_NORM_POST_ATTN], l.norm[HIPC_DEC_NORM_PRE_FFN], c.hidden, c.rms_eps, d->x, d->x, d->xn);
                HIPC_LAUNCHED(ctx);
                if ((rc = nbits_gemv(ctx, d->xn, HIPC_F32, l.gate_up, d->gu, 1, terms)) != HIPC_OK) return rc;
                hipLaunchKernelGGL((dec_gelu_mul_kernel), (unsigned)ceil_div(c.ffn, 256), 256, 0, s, d->gu, c.ffn, d->h);
                HIPC_LAUNCHED(ctx);
                if ((rc = nbits_gemv(ctx, d->h, HIPC_F32, l.down, d->y, 1, terms)) != HIPC_OK) return rc;
                const float *next = li + 1 < c.n_layers ? d->layers[li + 1].norm[HIPC_DEC_NORM_INPUT] : d->final_norm;
                hipLaunchKernelGGL((dec_norm_residual_kernel), 1, 256, 0, s, d->y, 1, l.norm[HIPC_DEC_NORM_POST_FFN], next, c.hidden, c.rms_eps, d->x, d->x, d->xn);
                HIPC_LAUNCHED(ctx);
            }
        }
        GemvArgmax am;
        am.v = d->am_v, am.i = d->am_i, am.capacity = ctx->tune.dec_fused_argmax == 0 ? 0 : kArgmaxCap;
        if (d->fused_glue) {
            // the unembedding's prologue adds the last branch to the stream and applies the final norm (every workgroup
            // for itself, while its first weight tiles are on their way)
            GemvPrologue pro;
            pro.mode = 2, pro.x = xc, pro.y = d->lean ? d->yd : d->y, pro.y_slices = d->lean ? d->down_slices : 1;
            pro.w_post = d->layers[c.n_layers - 1].norm[HIPC_DEC_NORM_POST_FFN], pro.w_in = d->final_norm, pro.eps = c.rms_eps;
            if ((rc = nbits_gemv(ctx, xc, HIPC_F32, d->lm_head, d->logits, 1, terms, &pro, &am)) != HIPC_OK) return rc;
        } else {
            if ((rc = nbits_gemv(ctx, d->xn, HIPC_F32, d->lm_head, d->logits, 1, terms, nullptr, &am)) != HIPC_OK) return rc;
        }
        // the unembedding's workgroups leave their candidates themselves when its launch can carry that (the kernel
        // for wide outputs); else a launch of its own scans the logits
        int parts = am.parts;
        if (parts == 0) {
            parts = kArgmaxParts;
            hipLaunchKernelGGL((dec_argmax_partial_kernel), kArgmaxParts, 256, 0, s, d->logits, c.vocab, d->am_v, d->am_i);
            HIPC_LAUNCHED(ctx);
        }
        hipLaunchKernelGGL((dec_pick_embed_kernel), 1, 256, 0, s, d->am_v, d->am_i, parts, d->state, d->history, c.max_seq, c.vocab, embed_args(d));
        HIPC_LAUNCHED(ctx);
        if (!ctx->capturing) d->x_ready = true;
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
