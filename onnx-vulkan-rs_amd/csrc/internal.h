// Shared internals of libhipcompute: the context object, status plumbing and
// launch helpers. Nothing here is part of the C ABI.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <exception>
#include <map>
#include <mutex>
#include <new>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/hipcompute.h"

// The inline assembly the kernels use sits behind macros, so that a host build of the kernel sources
// (the address model under tests/host, which runs every thread of a launch on the CPU with checked
// loads) can compile them: HIPC_HOST_MODEL is defined there and nowhere else.
#ifndef HIPC_HOST_MODEL
#define HIPC_PIN_VGPR(v) asm volatile("" : "+v"(v))                                              // the value is needed here, in a vector register
#define HIPC_VGPR_FROM_SGPR(dst, src) asm volatile("v_mov_b32 %0, %1" : "=v"(dst) : "s"(src))   // a uniform value kept in a vector register
#define HIPC_ARG_NOW(v) asm volatile("" ::"s"(v))                                                // the kernel argument is read here
// A load whose value may go unused on some paths (it is masked afterwards): on the GPU it is issued whatever the mask
// says, so the model must perform it too -- a plain load there may be moved under the condition and never be checked.
#define HIPC_LOAD_ALWAYS(ptr) (*(ptr))
#else
#define HIPC_LOAD_ALWAYS(ptr) gpu_model_load_always(ptr)
#define HIPC_ARG_NOW(v) ((void)0)
#define HIPC_PIN_VGPR(v) ((void)0)
#define HIPC_VGPR_FROM_SGPR(dst, src) ((dst) = (src))
#endif

namespace hipc {

constexpr int kScratchSlots = 5;

// grow-only device scratch reused by operators that need a temporary (packed
// B of a raw call, the i32 accumulator of a QLinear op). One in-order stream
// makes sequential reuse safe: the next user starts after the previous one ended.
struct Scratch {
    void *ptr = nullptr;
    size_t bytes = 0;
};

// Route and launch-shape overrides (experiments, and tests that must reach every kernel that
// ships). -1 leaves the choice to the library. A context starts from the environment variables of
// the same names (HIPC_GEMV_T ...) and hipc_set_option changes one afterwards.
struct Tuning {
    int gemv_t = -1;          // HIPC_GEMV_T         16-column tiles per GEMV wavefront: 1, 2 or 4
    int gemv_waves = -1;      // HIPC_GEMV_WAVES     wavefronts the GEMV aims for when it splits k inside a workgroup
    int gemv_per_cu = -1;     // HIPC_GEMV_PER_CU    resident GEMV wavefronts per CU of the persistent grid
    int gemm_tile = -1;       // HIPC_GEMM_TILE      LDS-staged int8 tiles: 64 or 128
    int gemm_big = -1;        // HIPC_GEMM_BIG       the int8 kernels that keep B out of LDS: 0 never, 1 / 2 the 256x256 / 128x128 tile whenever A allows
    int gemm_small = -1;      // HIPC_GEMM_SMALL     the k-split 64x64 kernels: 0 never, 1 whenever A allows
    int conv_row = -1;        // HIPC_CONV_ROW       0: convolutions along one axis take the general route
    int prefill_tile = -1;    // HIPC_PREFILL_TILE   64, 128 or 192 (columns; 192 has 128 rows)
    int prefill_split = -1;   // HIPC_PREFILL_SPLIT  0 never splits k, n forces n ways
    int prefill_groups = -1;  // HIPC_PREFILL_GROUPS 1 / 2: groups of four wavefronts per workgroup of the prefill tiles (2: each takes half of k)
    int prefill_direct = -1;  // HIPC_PREFILL_DIRECT 0: 128-row tiles keep the kernel that passes the weight through LDS (and are never 192 wide)
    int dec_fused_glue = -1;  // HIPC_DEC_FUSED_GLUE 0 keeps the separate norm / GELU kernels (read when a decoder is created)
    int dec_fused_argmax = -1; // HIPC_DEC_FUSED_ARGMAX 0: a launch of its own scans the logits for the token pick
    int dec_fused_attn = -1;  // HIPC_DEC_FUSED_ATTN 0 keeps the three-kernel attention (read when a decoder is created)
    int gemv_lean = -1;       // HIPC_GEMV_LEAN      0: one-row products keep the streaming GEMV kernel
    int dec_lean = -1;        // HIPC_DEC_LEAN       0: the decoder keeps the streaming GEMV and its prologues (read when a decoder is created)
    int dec_prefetch = -1;    // HIPC_DEC_PREFETCH   bits: which launches of a layer carry helper rows that read ahead for the next launch (0 none, 31 all; see hipc_decoder_step)
};

// The read-ahead helper rows (prefetch.h) once read past the end of a weight and faulted the GPU (a buffer
// load's scalar offset is outside the hardware's range check). While this constant is false the route is
// unreachable: hipc_set_option refuses HIPC_DEC_PREFETCH > 0, the environment variable is not read, the
// decoder ignores the field. It is true since the helper's byte addresses pass the host-side model of
// tests/host (decoder_model.cpp: the kernel sources run thread by thread on the CPU, every load of every
// helper thread inside its allocation, at every position of the cache).
constexpr bool kReadAheadVerified = true;

// Pinned staging ring of hipc_upload: the bytes are copied into a slot and travel from there, so the
// call returns without waiting for the stream. A slot is reused once the copies that read it are done.
constexpr int kStageSlots = 4;
constexpr size_t kStageSlotBytes = size_t(4) << 20;
struct StageRing {
    char *base = nullptr;               // kStageSlots * kStageSlotBytes of pinned host memory (allocated on first use)
    hipEvent_t done[kStageSlots] = {};  // recorded when the ring leaves a slot
    bool pending[kStageSlots] = {};
    int slot = 0;
    size_t used = 0;                    // bytes of the current slot handed out
};

// What a recorded operator call left in the graph: the scalars of it that a replay may change
// (hipc_graph_set_scalar), each a 32-bit word inside the first argument of one kernel node.
struct ScalarPatch {
    int which;              // HIPC_SCALAR_*
    hipGraphNode_t node;
    size_t offset;          // byte offset of the word inside the kernel's argument struct
};
struct RecordedOp {
    std::vector<ScalarPatch> patches;
};

}  // namespace hipc

struct hipc_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool owns_stream = false;
    bool capturing = false;
    std::mutex mu;
    std::string err;
    std::vector<void *> deferred;        // released at the next flush
    // Blocks the library itself retired (a scratch slot that grew, requantisation ratios that changed, a
    // replaced decoder weight) while recorded graphs exist: a graph may hold their addresses, so they stay
    // allocated until the last graph of the context is destroyed.
    std::vector<void *> retained;
    int live_graphs = 0;
    hipc::Scratch scratch[hipc::kScratchSlots];
    void *params = nullptr;              // small device block: range slot, scalars, range partials
    void *dql_static = nullptr;          // this device's address of the static range-partials array (see dynamic_quantize.hip)
    int cu_count = 256;
    std::vector<hipc::RecordedOp> cap_ops;     // while a capture is open: the calls that recorded work so far
    std::vector<hipc::ScalarPatch> cap_patches;   // ... the patchable scalars the current call has noted
    hipc::Tuning tune;
    hipc::StageRing stage;
    // hipc_alloc's blocks by size class (the reference's pooled scratch buffers,
    // crates/vk-compute/src/buffer.rs:303-341): a freed block waits in `pool` for the next request of its class
    std::unordered_map<void *, size_t> alloc_class;      // live hipc_alloc blocks -> class bytes
    std::map<size_t, std::vector<void *>> pool;          // class bytes -> free blocks
    size_t pool_bytes = 0;                               // bytes waiting in `pool`
    size_t pool_hits = 0, pool_misses = 0;
};

struct hipc_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<hipc::RecordedOp> ops;   // the entry-point calls that recorded work, in call order
};

// A MatMulNBits weight repacked for the matrix cores: 1 KiB tiles of 16 columns x 128 k. Lane l
// of tile (nt, cg) = Wq[(nt * n_cg + cg) * 64 + l] holds, in word j, the eight nibbles
// k = 128 cg + 32 j + 8 (l >> 4) .. + 8 of column 16 nt + (l & 15), in the order k0 k2 k4 k6 k1 k3 k5 k7. Sc / Zb hold SG scales
// and (128 + zero point) bytes per tile column, SG = 4, 2, 1 for block sizes 32, 64, >= 128.
struct hipc_nbits_weight {
    int64_t K = 0, N = 0, block_size = 0;
    int n_tiles = 0, n_cg = 0, SG = 0;
    int interleave_half = 0;  // > 0: column tiles alternate between the two halves of N (see mmnb_prepack_kernel)
    uint4 *Wq = nullptr;
    float *Sc = nullptr;
    uint8_t *Zb = nullptr;
    size_t bytes = 0;
    // A block_size below 32 or not a power of two has no tiled form (a 32-k product step would straddle scale
    // groups): the handle then keeps device copies of the operator's own tensors (Wq is null) and the product
    // runs on the kernel that reads that layout. Only hipc_matmul_nbits_packed takes such a handle.
    void *raw_B = nullptr, *raw_scales = nullptr, *raw_zp = nullptr;
    int raw_scale_dtype = 0;
};

namespace hipc {

inline int fail(hipc_ctx *ctx, int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (ctx) ctx->err = buf;
    return code;
}

// RAII: serialise the call and make the context's device current.
struct Guard {
    std::unique_lock<std::mutex> lock;
    explicit Guard(hipc_ctx *ctx) : lock(ctx->mu) { (void)hipSetDevice(ctx->device); }
};

// The body of an entry point: takes the context's lock, makes its device current and keeps C++
// exceptions (a failed host allocation, a length error) from crossing the C ABI -- they become
// HIPC_ERR_BACKEND with a message, under the same lock.
// The kernel node a launch on the capturing stream has just added (null when nothing is being captured).
inline hipGraphNode_t last_captured_node(hipc_ctx *ctx) {
    if (!ctx->capturing) return nullptr;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    const hipGraphNode_t *deps = nullptr;
    size_t n = 0;
    if (hipStreamGetCaptureInfo_v2(ctx->stream, &status, nullptr, nullptr, &deps, &n) != hipSuccess || status != hipStreamCaptureStatusActive || n == 0)
        return nullptr;
    return deps[n - 1];
}
// called right after the launch whose argument struct holds the scalar: the word at `offset` of that struct may be
// changed in the instantiated graph later (hipc_graph_set_scalar)
inline void note_scalar(hipc_ctx *ctx, int which, size_t offset) {
    if (hipGraphNode_t node = last_captured_node(ctx)) ctx->cap_patches.push_back(ScalarPatch{which, node, offset});
}

template <typename F>
int entry(hipc_ctx *ctx, F &&body) noexcept {
    if (!ctx) return HIPC_ERR_INVALID;
    try {
        Guard g(ctx);
        try {
            if (!ctx->capturing) return body();
            // while a capture is open every call that records work becomes an entry of the graph's operator list
            const hipGraphNode_t before = last_captured_node(ctx);
            ctx->cap_patches.clear();
            const int rc = body();
            if (ctx->capturing && rc == HIPC_OK && last_captured_node(ctx) != before) {
                ctx->cap_ops.emplace_back();
                ctx->cap_ops.back().patches.swap(ctx->cap_patches);
            }
            return rc;
        } catch (const std::bad_alloc &) {
            return fail(ctx, HIPC_ERR_BACKEND, "out of host memory");
        } catch (const std::exception &e) {
            return fail(ctx, HIPC_ERR_BACKEND, "internal error: %s", e.what());
        } catch (...) {
            return fail(ctx, HIPC_ERR_BACKEND, "internal error");
        }
    } catch (...) {
        return HIPC_ERR_BACKEND;
    }
}
template <typename F>
void entry_void(hipc_ctx *ctx, F &&body) noexcept {
    if (!ctx) return;
    try {
        Guard g(ctx);
        body();
    } catch (...) {
    }
}

// A block of the library's own that later work no longer uses: freed at the next flush, or, while
// recorded graphs exist (they may hold its address), when the last of them is destroyed.
inline void retire(hipc_ctx *ctx, void *p) {
    if (!p) return;
    if (ctx->live_graphs > 0) ctx->retained.push_back(p);
    else ctx->deferred.push_back(p);
}

#define HIPC_TRY(ctx, expr)                                                                      \
    do {                                                                                         \
        hipError_t e_ = (expr);                                                                  \
        if (e_ != hipSuccess)                                                                    \
            return hipc::fail((ctx), HIPC_ERR_BACKEND, "%s: %s (%s:%d)", #expr,                  \
                              hipGetErrorString(e_), __FILE__, __LINE__);                        \
    } while (0)

#define HIPC_REQUIRE(ctx, cond, ...)                                                             \
    do {                                                                                         \
        if (!(cond)) return hipc::fail((ctx), HIPC_ERR_INVALID, __VA_ARGS__);                    \
    } while (0)

#define HIPC_REFUSE(ctx, cond, ...)                                                              \
    do {                                                                                         \
        if (cond) return hipc::fail((ctx), HIPC_ERR_UNSUPPORTED, __VA_ARGS__);                   \
    } while (0)

// status of the launch just made (configuration errors surface here, not at the next sync)
#define HIPC_LAUNCHED(ctx) HIPC_TRY((ctx), hipGetLastError())

// Requantisation ratios of a QLinear operator, kept with the weight handle. They are formed on the
// host from the operator's scale attributes; as long as those do not change between calls the
// device copy is reused, so a call neither uploads nor synchronises and can be captured.
struct RatioCache {
    float *dev = nullptr;
    std::vector<float> host;
};
// *out = device pointer holding `ratio` (uploading it first when it differs from the cached copy;
// that upload is refused while a capture is open)
int ratio_resident(hipc_ctx *ctx, RatioCache &cache, const std::vector<float> &ratio, const float **out);
void ratio_release(hipc_ctx *ctx, RatioCache &cache);

// Kernels that use more than the default 64 KiB of dynamic LDS must say so once per device. `done` is
// the launcher's own flag array (one per kernel instantiation); a race between two contexts merely
// sets the attribute twice.
constexpr int kMaxDevices = 64;
template <typename K>
int allow_dynamic_lds(hipc_ctx *ctx, K kernel, size_t bytes, bool (&done)[kMaxDevices]) {
    const int d = ctx->device >= 0 && ctx->device < kMaxDevices ? ctx->device : 0;
    if (done[d] && ctx->device == d) return HIPC_OK;
    HIPC_TRY(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    done[d] = true;
    return HIPC_OK;
}

// Returns ctx->scratch[slot] grown to at least `bytes`. Growth allocates, so it is
// refused while a capture is open.
int scratch_get(hipc_ctx *ctx, int slot, size_t bytes, void **out);
// host bytes -> device through the context's pinned staging ring; records only (see StageRing)
int stage_upload(hipc_ctx *ctx, void *dst, const void *host, size_t bytes);
// looks up this device's address of the static range-partials array of the DynamicQuantizeLinear
// variant that allocates nothing, and keeps it in ctx->dql_static (dynamic_quantize.hip)
int dql_static_init(hipc_ctx *ctx);

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
inline bool is_byte_dtype(int dt) { return dt == HIPC_U8 || dt == HIPC_I8; }
inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// MatMulNBits pieces other operators of the library build on (the caller holds the lock)
int nbits_prepack(hipc_ctx *ctx, const void *B, size_t b_len, const void *scales, int scale_dtype, size_t scales_len,
                  const void *zp, size_t zp_len, int64_t K, int64_t N, int64_t block_size, hipc_nbits_weight **out,
                  int interleave_half = 0, bool any_block_size = false);   // any_block_size: may return a handle in the operator's layout
void nbits_release(hipc_ctx *ctx, hipc_nbits_weight *w);
// rows [0, M), M <= 16, of A against a prepacked weight; `terms` = bf16 terms per activation (2 or 3)
// What the single activation row of a decode GEMV is computed from (mode 0 / null: A as given):
//   mode 1  A = [gate | up] (2K floats): the row is gelu_tanh(gate) * up
//   mode 2  the row is rmsnorm(x', w_in), x' = x + rmsnorm(y, w_post) (x' = x when y is null);
//           x' is also written to x_out (not x itself) when x_out is set. A is ignored.
//   mode 3  the row is the attention output of the step, joined from the flash-decoding partials
//           of its kAttnSplits context chunks: part_o [kv head][split][group * head_dim]
//           unnormalised outputs, part_ml [kv head][split][group] (max, sum) pairs; the number of
//           live chunks follows from *pos and the layer's window (see attn_live_chunks). A is ignored.
struct GemvPrologue {
    int mode = 0;
    const float *x = nullptr, *y = nullptr, *w_post = nullptr, *w_in = nullptr;
    int y_slices = 1;   // y is the sum of this many partial rows, K floats apart
    float *x_out = nullptr;
    float eps = 0.f;
    const float *part_o = nullptr, *part_ml = nullptr;
    const int *pos = nullptr;
    int group = 0, head_dim = 0, window = 0;
};
// Decode attention splits the visible context of a kv head over kAttnSplits workgroups. The split
// starts at attn_base: the first visible position rounded down to 16 (16 positions are then 32 bytes,
// aligned, in the transposed value cache; positions before the first visible one are masked). Each
// workgroup takes attn_chunk(span) consecutive positions of the span from there to the end,
// kAttnPass at a time: one pass while span <= kAttnPass * kAttnSplits = 2048 positions. The first
// attn_live_chunks(span) splits hold at least one position and only those write a partial.
constexpr int kAttnPass = 32;
constexpr int kAttnSplits = 64;
// first visible position of a step that sees `total` positions through a window (<= 0: no window)
__host__ __device__ inline int attn_first(int total, int window) { return window > 0 && total > window ? total - window : 0; }
__host__ __device__ inline int attn_base(int total, int window) { return attn_first(total, window) & ~15; }
__host__ __device__ inline int attn_span(int total, int window) { return total - attn_base(total, window); }
__host__ __device__ inline int attn_chunk(int span) {
    return kAttnPass * ((span + kAttnPass * kAttnSplits - 1) / (kAttnPass * kAttnSplits));
}
__host__ __device__ inline int attn_live_chunks(int span) {
    if (span <= kAttnPass * kAttnSplits) return (span + kAttnPass - 1) / kAttnPass;   // no run-time division on the common path
    const int c = attn_chunk(span);
    return (span + c - 1) / c;
}
// the transposed value cache's row length: max_seq rounded up to 64
__host__ __device__ inline int attn_v_stride(int max_seq) { return (max_seq + 63) / 64 * 64; }
// Optional epilogue of nbits_gemv for one f32 row: every workgroup of the wide kernel also leaves the largest of the
// results it stored and its column (smallest column on ties; NaN never wins) in v[workgroup], i[workgroup]. `parts`
// comes back as the number of workgroups that wrote a candidate, or 0 when the launch could not carry the epilogue
// (another kernel took the product, k was split over workgroups, more workgroups than `capacity`): the caller then
// scans Y itself.
struct GemvArgmax {
    float *v = nullptr;
    int *i = nullptr;
    int capacity = 0;
    int parts = 0;
};
int nbits_gemv(hipc_ctx *ctx, const void *A, int a_dtype, const hipc_nbits_weight *w, void *Y, int M, int terms,
               const GemvPrologue *pro = nullptr, GemvArgmax *am = nullptr);

// ---- the latency-built kernel for one f32 row (gemv_lean.hip) -------------------------------------
// A row "in operand order": per 32-k chunk c, NT terms x 4 k groups of 8 bf16 (16 bytes each), term
// major -- split[(c * NT + term) * 4 + group] -- so that a lane's matrix-core A operand is one
// 16-byte load. (The sums over a quantisation block's activations, which take the +128 bias of the
// weights out again, are formed by the consumer on the matrix cores: a product against ones.)
// What the helper rows of a launch read ahead for the launch that follows it (prefetch.h).
struct PrefetchArgs {
    int kind = 0;          // 0 nothing; 1 the weight tiles of a one-row product; 2 the cache rows of an attention launch
    int rows = 0;          // helper rows appended to the producer's grid (gridDim.x workgroups each)
    uint32_t *sink = nullptr;
    // kind 1: the consumer's weight and launch shape
    const uint4 *wq = nullptr;
    const float *sc = nullptr;
    const uint8_t *zb = nullptr;
    int gx = 0, gy = 0, WN = 0, slice_tiles = 0, n_cg = 0, n_tiles = 0, SG = 0;
    // kind 1 behind an attention launch: the helpers read only when the step's context is at least gate_chunks
    // chunks long (attn_live_chunks; a short attention launch would be lengthened by them); pos as for kind 2
    int gate_chunks = 0, gate_window = 0;
    // kind 2: the attention launch's cache
    const int *pos = nullptr;
    const void *k = nullptr, *v = nullptr;
    int window = 0, max_seq = 0, v_stride = 0, hd = 0, n_kv = 0;
};
// The tiles consumer j (= y * gx + x of the consumer's grid) reads for its column tile wn: a run of
// `count` consecutive tiles from `*tile0` in all three weight arrays (0: nothing).
__host__ __device__ inline int pf_tile_run(const PrefetchArgs &pf, int j, int wn, size_t *tile0) {
    int x = j, y = 0;
    while (x >= pf.gx) x -= pf.gx, y++;
    const int kt0 = y * pf.slice_tiles;
    const int cnt = pf.slice_tiles < pf.n_cg - kt0 ? pf.slice_tiles : pf.n_cg - kt0;
    const int nt = x * pf.WN + wn;
    if (y >= pf.gy || nt >= pf.n_tiles || cnt <= 0) return 0;
    *tile0 = (size_t)nt * pf.n_cg + kt0;
    return cnt;
}
// Helper h of H (linear workgroup id b in its launch) serves the consumers j = first, first + step, ...:
// those of its own XCD class (j = b mod 8), dealt round robin to the helpers of that class.
__host__ __device__ inline void pf_consumers_of(int h, int H, int b, int *first, int *step) {
    *first = (b & 7) + 8 * (h >> 3);
    *step = 8 * ((H + 7) >> 3);
}
// The first 120 bytes -- two lines of the scalar cache -- hold everything a workgroup of the product itself reads, and
// the kernel reads them in one batch at its entry: the scalar cache starts every launch empty, every line is a trip to
// memory of its own, and an argument read where it is first used puts that trip into the middle of the kernel. The
// operands of the prologues share their bytes (a launch has one prologue); the read-ahead description behind them is read
// by the helper rows only.
struct LeanArgs {
    const uint4 *Wq;
    const float *Sc;
    const uint8_t *Zb;
    union {
        float *Y;        // EPI 0: [slices][N] partial rows (the row itself when slices == 1)
        uint4 *h_split;  // EPI 1: gelu_tanh(gate) * up of the interleaved (gate, up) tile pairs, in operand order
    };
    int K, N, n_tiles, n_cg;
    int WK, KT, WN, slices;      // wavefronts along k, k tiles per wavefront (<= 4), column tiles per workgroup, k slices (gridDim.y)
    uint32_t nib_mask, magic;    // 0x000f000f and 0x43004300 (bf16 128.0 in both halves)
    union {
        // PRO 2: row = rmsnorm(x', w_in), x' = x + rmsnorm(sum of y_slices rows of yparts, w_post) (x' = x when yparts is null);
        //        workgroup (0, 0) also writes x' to x_out
        struct {
            const float *x, *yparts, *w_post, *w_in;
            float *x_out;
            int y_slices;
            float eps;
        };
        // PRO 3: the attention output joined from the flash-decoding partials (see GemvPrologue mode 3)
        struct {
            const float *part_o, *part_ml;
            const int *pos;
            int lg_group, lg_hd, n_kv, window;   // log2 of the query heads per kv head and of head_dim (both powers of two), kv heads
        };
        const float *A;          // PRO 0: the row
        const uint4 *a_split;    // PRO 4: the row in operand order
    };
    PrefetchArgs pf;             // helper rows behind the `slices` rows of the grid
};
static_assert(offsetof(LeanArgs, pf) == 120, "the arguments of the product fill two 64-byte lines");
struct LeanPlan {
    int WK, KT, WN, slices;
};
// false when the shape does not fit the kernel (k tiles per wavefront would exceed 4)
bool lean_plan(hipc_ctx *ctx, const hipc_nbits_weight *w, int slices, int WN, LeanPlan *out, int max_waves = 16, bool short_in_three = true);
// `a` carries the prologue / epilogue operands; weight and launch-shape fields are filled in here
int lean_gemv(hipc_ctx *ctx, const hipc_nbits_weight *w, const LeanPlan &pl, LeanArgs a, int pro, int epi, int NT);
// the prefetch description of a one-row product launched with plan `pl` (for the launch before it)
PrefetchArgs lean_prefetch_of(const hipc_nbits_weight *w, const LeanPlan &pl, int rows, uint32_t *sink);

int64_t nbits_cols(const hipc_nbits_weight *w);
int64_t nbits_depth(const hipc_nbits_weight *w);
// f16 activations, any M: tiled matrix-core kernel that dequantises the weight on its way to LDS.
// Returns HIPC_ERR_UNSUPPORTED (and launches nothing) for shapes it does not take.
bool nbits_prefill_takes(const void *A, const hipc_nbits_weight *w, int64_t M);
int nbits_prefill(hipc_ctx *ctx, const void *A, const hipc_nbits_weight *w, void *Y, int64_t M);
// f32 activations, more than 32 rows: the same kernel on two f16 rows per row (see matmul_nbits_prefill.hip)
bool nbits_prefill_f32_takes(const void *A, const hipc_nbits_weight *w, int64_t M);
int nbits_prefill_f32(hipc_ctx *ctx, const void *A, const hipc_nbits_weight *w, void *Y, int64_t M, int terms);   // f16 terms per f32 row: 2 (22 bits), 1 (11) or 3 (all 24)

// offsets inside ctx->params
constexpr size_t kParamRange = 0;   // 8 B  {bits(-min), bits(max)}
constexpr size_t kParamParts = 256; // 16 KiB: per-workgroup {bits(-min), bits(max)} pairs of DynamicQuantizeLinear
constexpr int kParamPartsMax = 2048;
constexpr size_t kParamBytes = 256 + 8 * kParamPartsMax;

}  // namespace hipc
