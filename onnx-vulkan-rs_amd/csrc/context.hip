// Context, buffers, capture/replay and timing: the part of the library that
// stands where the reference's `vk-compute` runtime does
// (crates/vk-compute/src/{buffer,stream,pipeline}.rs). One in-order HIP stream
// gives the reference's "every command waits for everything before it"
// semantics (stream.rs:11-14) by construction; a HIP graph is its capture/replay.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <iterator>

#include "internal.h"

namespace hipc {

__global__ void fill_words(uint32_t *dst, size_t words, uint32_t value) {
    size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < words; i += stride) dst[i] = value;
}

int scratch_get(hipc_ctx *ctx, int slot, size_t bytes, void **out) {
    Scratch &s = ctx->scratch[slot];
    if (s.bytes < bytes) {
        if (ctx->capturing)
            return fail(ctx, HIPC_ERR_UNSUPPORTED,
                        "scratch slot %d must grow to %zu bytes while a capture is open: run the "
                        "operator once before capturing",
                        slot, bytes);
        retire(ctx, s.ptr);  // earlier launches, or a recorded graph, may still use the old block
        s.ptr = nullptr;
        s.bytes = 0;
        size_t want = (bytes + 0xfffff) & ~(size_t)0xfffff;
        HIPC_TRY(ctx, hipMalloc(&s.ptr, want));
        s.bytes = want;
    }
    *out = s.ptr;
    return HIPC_OK;
}

namespace {

constexpr size_t kPoolCap = size_t(1) << 30;  // bytes of freed hipc_alloc blocks kept for reuse

// the size class of a request: a power of two up to 1 MiB, a whole number of MiB above
size_t alloc_class_of(size_t bytes) {
    if (bytes <= 256) return 256;
    if (bytes > (size_t(1) << 20)) return (bytes + 0xfffff) & ~(size_t)0xfffff;
    size_t c = 256;
    while (c < bytes) c <<= 1;
    return c;
}

// nothing enqueued uses `p` any more: back to the pool if hipc_alloc made it, else freed
void release_block(hipc_ctx *ctx, void *p) {
    auto it = ctx->alloc_class.find(p);
    if (it == ctx->alloc_class.end()) {
        (void)hipFree(p);
        return;
    }
    const size_t cls = it->second;
    ctx->alloc_class.erase(it);
    if (cls > kPoolCap) {
        (void)hipFree(p);
        return;
    }
    // over the cap: the largest waiting blocks go back to the device first
    while (ctx->pool_bytes + cls > kPoolCap && !ctx->pool.empty()) {
        auto big = std::prev(ctx->pool.end());
        if (big->second.empty()) {
            ctx->pool.erase(big);
            continue;
        }
        (void)hipFree(big->second.back());
        big->second.pop_back();
        ctx->pool_bytes -= big->first;
    }
    ctx->pool[cls].push_back(p);
    ctx->pool_bytes += cls;
}

int release_deferred(hipc_ctx *ctx) {
    for (void *p : ctx->deferred) release_block(ctx, p);
    ctx->deferred.clear();
    // the stream is idle: every staging slot is free again
    for (bool &b : ctx->stage.pending) b = false;
    ctx->stage.used = 0;
    return HIPC_OK;
}

int env_int(const char *name) {
    const char *e = getenv(name);
    return e && *e ? atoi(e) : -1;
}

struct OptionName {
    const char *name;
    int Tuning::*field;
};
const OptionName kOptions[] = {
    {"HIPC_GEMV_T", &Tuning::gemv_t},
    {"HIPC_GEMV_WAVES", &Tuning::gemv_waves},
    {"HIPC_GEMV_PER_CU", &Tuning::gemv_per_cu},
    {"HIPC_GEMM_TILE", &Tuning::gemm_tile},
    {"HIPC_GEMM_BIG", &Tuning::gemm_big},
    {"HIPC_GEMM_SMALL", &Tuning::gemm_small},
    {"HIPC_CONV_ROW", &Tuning::conv_row},
    {"HIPC_PREFILL_TILE", &Tuning::prefill_tile},
    {"HIPC_PREFILL_SPLIT", &Tuning::prefill_split},
    {"HIPC_PREFILL_DIRECT", &Tuning::prefill_direct},
    {"HIPC_PREFILL_GROUPS", &Tuning::prefill_groups},
    {"HIPC_DEC_FUSED_GLUE", &Tuning::dec_fused_glue},
    {"HIPC_DEC_FUSED_ATTN", &Tuning::dec_fused_attn},
    {"HIPC_DEC_FUSED_ARGMAX", &Tuning::dec_fused_argmax},
    {"HIPC_GEMV_LEAN", &Tuning::gemv_lean},
    {"HIPC_DEC_LEAN", &Tuning::dec_lean},
    {"HIPC_DEC_PREFETCH", &Tuning::dec_prefetch},
};

int create(int device, void *stream, bool adopt, hipc_ctx **out) {
    if (!out) return HIPC_ERR_INVALID;
    *out = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count) return HIPC_ERR_BACKEND;
    if (hipSetDevice(device) != hipSuccess) return HIPC_ERR_BACKEND;
    hipc_ctx *ctx = new (std::nothrow) hipc_ctx();
    if (!ctx) return HIPC_ERR_BACKEND;
    ctx->device = device;
    if (adopt) {
        ctx->stream = static_cast<hipStream_t>(stream);
    } else {
        if (hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking) != hipSuccess) {
            delete ctx;
            return HIPC_ERR_BACKEND;
        }
        ctx->owns_stream = true;
    }
    for (const OptionName &o : kOptions) ctx->tune.*(o.field) = env_int(o.name);
    if (!kReadAheadVerified) ctx->tune.dec_prefetch = -1;   // not reachable from the environment either
    if (hipMalloc(&ctx->params, kParamBytes) != hipSuccess ||
        hipMemsetAsync(ctx->params, 0, kParamBytes, ctx->stream) != hipSuccess ||
        dql_static_init(ctx) != HIPC_OK) {
        if (ctx->params) (void)hipFree(ctx->params);
        if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return HIPC_ERR_BACKEND;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0)
        ctx->cu_count = prop.multiProcessorCount;
    *out = ctx;
    return HIPC_OK;
}

// The current slot is full (or the caller wants its bytes on their way): an event marks the end of
// the copies that read it, and the ring moves on to the next slot once that slot's own copies are done.
int stage_next_slot(hipc_ctx *ctx) {
    StageRing &r = ctx->stage;
    HIPC_TRY(ctx, hipEventRecord(r.done[r.slot], ctx->stream));
    r.pending[r.slot] = true;
    r.slot = (r.slot + 1) % kStageSlots;
    r.used = 0;
    if (r.pending[r.slot]) {
        HIPC_TRY(ctx, hipEventSynchronize(r.done[r.slot]));
        r.pending[r.slot] = false;
    }
    return HIPC_OK;
}

}  // namespace

// host bytes -> device, through the pinned ring: `host` is free again on return and the host has not
// waited for the stream (only, when more than the ring holds is in flight, for the ring's oldest slot)
int stage_upload(hipc_ctx *ctx, void *dst, const void *host, size_t bytes) {
    StageRing &r = ctx->stage;
    if (!r.base) {
        HIPC_TRY(ctx, hipHostMalloc(reinterpret_cast<void **>(&r.base), kStageSlots * kStageSlotBytes, hipHostMallocDefault));
        for (hipEvent_t &e : r.done) HIPC_TRY(ctx, hipEventCreateWithFlags(&e, hipEventDisableTiming));
    }
    const char *src = static_cast<const char *>(host);
    char *to = static_cast<char *>(dst);
    while (bytes > 0) {
        if (r.used >= kStageSlotBytes)
            if (int rc = stage_next_slot(ctx)) return rc;
        const size_t n = std::min(bytes, kStageSlotBytes - r.used);
        char *pinned = r.base + (size_t)r.slot * kStageSlotBytes + r.used;
        memcpy(pinned, src, n);
        HIPC_TRY(ctx, hipMemcpyAsync(to, pinned, n, hipMemcpyHostToDevice, ctx->stream));
        r.used += (n + 63) & ~(size_t)63;
        src += n, to += n, bytes -= n;
    }
    return HIPC_OK;
}

int ratio_resident(hipc_ctx *ctx, RatioCache &cache, const std::vector<float> &ratio, const float **out) {
    if (cache.dev && cache.host.size() == ratio.size() &&
        memcmp(cache.host.data(), ratio.data(), ratio.size() * sizeof(float)) == 0) {
        *out = cache.dev;
        return HIPC_OK;
    }
    HIPC_REFUSE(ctx, ctx->capturing, "QLinear: the requantisation ratios changed and would have to be uploaded inside a capture; run the operator once before capturing");
    // A new block every time the ratios change: earlier launches, and graphs recorded with the old
    // scales, keep reading the old one (it is retired, not rewritten).
    retire(ctx, cache.dev);
    cache.dev = nullptr;
    cache.host.clear();
    HIPC_TRY(ctx, hipMalloc(reinterpret_cast<void **>(&cache.dev), std::max<size_t>(ratio.size() * sizeof(float), 16)));
    if (int rc = stage_upload(ctx, cache.dev, ratio.data(), ratio.size() * sizeof(float))) return rc;
    cache.host = ratio;
    *out = cache.dev;
    return HIPC_OK;
}

void ratio_release(hipc_ctx *ctx, RatioCache &cache) {
    if (cache.dev) ctx->deferred.push_back(cache.dev);
    cache.dev = nullptr;
    cache.host.clear();
}

}  // namespace hipc

using namespace hipc;

extern "C" {

#ifndef HIPC_BUILD_ID
#define HIPC_BUILD_ID "unknown"
#endif
// "... build <id>": the id is a hash over the sources and headers the library was compiled from (csrc/Makefile)
const char *hipc_version(void) { return "hipcompute 0.3 (gfx950) build " HIPC_BUILD_ID; }

int hipc_ctx_create(int device, hipc_ctx **out) {
    try {
        return create(device, nullptr, false, out);
    } catch (...) {
        return HIPC_ERR_BACKEND;
    }
}

int hipc_ctx_create_on_stream(int device, void *stream, hipc_ctx **out) {
    try {
        return create(device, stream, true, out);
    } catch (...) {
        return HIPC_ERR_BACKEND;
    }
}

void hipc_ctx_destroy(hipc_ctx *ctx) {
    if (!ctx) return;
    entry_void(ctx, [&] {
        (void)hipStreamSynchronize(ctx->stream);
        release_deferred(ctx);
        for (void *p : ctx->retained) (void)hipFree(p);
        for (auto &cls : ctx->pool)
            for (void *p : cls.second) (void)hipFree(p);
        for (Scratch &s : ctx->scratch)
            if (s.ptr) (void)hipFree(s.ptr);
        if (ctx->params) (void)hipFree(ctx->params);
        if (ctx->stage.base) {
            (void)hipHostFree(ctx->stage.base);
            for (hipEvent_t e : ctx->stage.done)
                if (e) (void)hipEventDestroy(e);
        }
        if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
    });
    delete ctx;
}

// The text is copied under the context's lock into storage of the calling thread, so another
// thread failing on the same context meanwhile cannot pull the string from under the reader.
const char *hipc_last_error(hipc_ctx *ctx) {
    if (!ctx) return "null context";
    static thread_local char text[512];
    text[0] = 0;
    entry_void(ctx, [&] { snprintf(text, sizeof text, "%s", ctx->err.c_str()); });
    return text;
}

void *hipc_stream(hipc_ctx *ctx) { return ctx ? static_cast<void *>(ctx->stream) : nullptr; }

int hipc_set_option(hipc_ctx *ctx, const char *name, int value) {
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, name, "hipc_set_option: null name");
        for (const OptionName &o : kOptions)
            if (strcmp(o.name, name) == 0) {
                HIPC_REFUSE(ctx, !kReadAheadVerified && o.field == &Tuning::dec_prefetch && value > 0,
                            "HIPC_DEC_PREFETCH: the read-ahead route is switched off in this build");
                ctx->tune.*(o.field) = value < 0 ? -1 : value;   // (0 is a value of its own: HIPC_DEC_PREFETCH = 0 switches the helpers off)
                return HIPC_OK;
            }
        return fail(ctx, HIPC_ERR_INVALID, "hipc_set_option: unknown option %s", name);
    });
}

int hipc_alloc(hipc_ctx *ctx, size_t bytes, void **dptr) {
    if (!dptr) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        HIPC_REFUSE(ctx, ctx->capturing, "hipc_alloc while a capture is open");
        *dptr = nullptr;
        const size_t cls = alloc_class_of(bytes);
        void *p = nullptr;
        auto it = ctx->pool.find(cls);
        if (it != ctx->pool.end() && !it->second.empty()) {
            p = it->second.back();
            it->second.pop_back();
            ctx->pool_bytes -= cls;
            ctx->pool_hits++;
        } else {
            hipError_t e = hipMalloc(&p, cls);
            if (e != hipSuccess && ctx->pool_bytes > 0) {  // out of device memory: give back what the pool holds and retry
                (void)hipGetLastError();
                for (auto &c : ctx->pool) {
                    for (void *q : c.second) (void)hipFree(q);
                    c.second.clear();
                }
                ctx->pool_bytes = 0;
                e = hipMalloc(&p, cls);
            }
            if (e != hipSuccess) return fail(ctx, HIPC_ERR_BACKEND, "hipc_alloc(%zu): %s", bytes, hipGetErrorString(e));
            ctx->pool_misses++;
        }
        ctx->alloc_class[p] = cls;
        *dptr = p;
        return HIPC_OK;
    });
}

int hipc_free_deferred(hipc_ctx *ctx, void *dptr) {
    return entry(ctx, [&]() -> int {
        if (dptr) ctx->deferred.push_back(dptr);
        return HIPC_OK;
    });
}

int hipc_pool_stats(hipc_ctx *ctx, size_t *hits, size_t *misses, size_t *bytes_waiting) {
    return entry(ctx, [&]() -> int {
        if (hits) *hits = ctx->pool_hits;
        if (misses) *misses = ctx->pool_misses;
        if (bytes_waiting) *bytes_waiting = ctx->pool_bytes;
        return HIPC_OK;
    });
}

int hipc_upload(hipc_ctx *ctx, void *dst, size_t dst_offset, const void *host, size_t bytes) {
    return entry(ctx, [&]() -> int {
        HIPC_REFUSE(ctx, ctx->capturing, "hipc_upload while a capture is open: a replay would re-read the host pointer");
        if (bytes == 0) return HIPC_OK;
        HIPC_REQUIRE(ctx, dst && host, "hipc_upload: null pointer");
        return stage_upload(ctx, static_cast<char *>(dst) + dst_offset, host, bytes);
    });
}

int hipc_download(hipc_ctx *ctx, void *host, const void *src, size_t src_offset, size_t bytes) {
    return entry(ctx, [&]() -> int {
        HIPC_REFUSE(ctx, ctx->capturing, "hipc_download while a capture is open");
        HIPC_TRY(ctx, hipStreamSynchronize(ctx->stream));
        release_deferred(ctx);
        if (bytes == 0) return HIPC_OK;
        HIPC_REQUIRE(ctx, host && src, "hipc_download: null pointer");
        HIPC_TRY(ctx, hipMemcpy(host, static_cast<const char *>(src) + src_offset, bytes, hipMemcpyDeviceToHost));
        return HIPC_OK;
    });
}

int hipc_copy(hipc_ctx *ctx, void *dst, size_t dst_offset, const void *src, size_t src_offset, size_t bytes) {
    return entry(ctx, [&]() -> int {
        if (bytes == 0) return HIPC_OK;
        HIPC_REQUIRE(ctx, dst && src, "hipc_copy: null pointer");
        HIPC_TRY(ctx, hipMemcpyAsync(static_cast<char *>(dst) + dst_offset, static_cast<const char *>(src) + src_offset,
                                     bytes, hipMemcpyDeviceToDevice, ctx->stream));
        return HIPC_OK;
    });
}

int hipc_fill(hipc_ctx *ctx, void *dst, size_t dst_offset, size_t bytes, uint32_t word) {
    return entry(ctx, [&]() -> int {
        if (bytes == 0) return HIPC_OK;
        HIPC_REQUIRE(ctx, dst, "hipc_fill: null pointer");
        HIPC_REQUIRE(ctx, bytes % 4 == 0 && dst_offset % 4 == 0, "hipc_fill: offset and length must be multiples of 4");
        const size_t words = bytes / 4;
        const int block = 256;
        size_t grid = (words + block - 1) / block;
        if (grid > 4096) grid = 4096;
        fill_words<<<dim3((unsigned)grid), dim3(block), 0, ctx->stream>>>(
            reinterpret_cast<uint32_t *>(static_cast<char *>(dst) + dst_offset), words, word);
        HIPC_LAUNCHED(ctx);
        return HIPC_OK;
    });
}

int hipc_flush(hipc_ctx *ctx) {
    return entry(ctx, [&]() -> int {
        HIPC_REFUSE(ctx, ctx->capturing, "hipc_flush while a capture is open");
        HIPC_TRY(ctx, hipStreamSynchronize(ctx->stream));
        release_deferred(ctx);
        return HIPC_OK;
    });
}

int hipc_capture_begin(hipc_ctx *ctx) {
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, !ctx->capturing, "hipc_capture_begin: a capture is already open");
        HIPC_TRY(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
        ctx->capturing = true;
        ctx->cap_ops.clear();
        return HIPC_OK;
    });
}

int hipc_capture_end(hipc_ctx *ctx, hipc_graph **out) {
    if (!out) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, ctx->capturing, "hipc_capture_end: no capture is open");
        *out = nullptr;
        hipGraph_t graph = nullptr;
        ctx->capturing = false;
        HIPC_TRY(ctx, hipStreamEndCapture(ctx->stream, &graph));
        hipGraphExec_t exec = nullptr;
        hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
        if (e != hipSuccess) {
            (void)hipGraphDestroy(graph);
            return fail(ctx, HIPC_ERR_BACKEND, "hipGraphInstantiate: %s", hipGetErrorString(e));
        }
        hipc_graph *gr = new hipc_graph();
        gr->graph = graph;
        gr->exec = exec;
        gr->ops.swap(ctx->cap_ops);
        ctx->live_graphs++;
        *out = gr;
        return HIPC_OK;
    });
}

int hipc_graph_launch(hipc_ctx *ctx, hipc_graph *graph) {
    if (!graph) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, !ctx->capturing, "hipc_graph_launch while a capture is open");
        HIPC_TRY(ctx, hipGraphLaunch(graph->exec, ctx->stream));
        return HIPC_OK;
    });
}

void hipc_graph_destroy(hipc_ctx *ctx, hipc_graph *graph) {
    if (!graph) return;
    entry_void(ctx, [&] {
        (void)hipStreamSynchronize(ctx->stream);
        if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
        if (graph->graph) (void)hipGraphDestroy(graph->graph);
        delete graph;
        // the last graph is gone: nothing can name the blocks retired while graphs existed
        if (--ctx->live_graphs <= 0) {
            ctx->live_graphs = 0;
            for (void *p : ctx->retained) ctx->deferred.push_back(p);
            ctx->retained.clear();
        }
    });
}

int hipc_graph_op_count(hipc_ctx *ctx, hipc_graph *graph, int *count) {
    if (!graph || !count) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        *count = (int)graph->ops.size();
        return HIPC_OK;
    });
}

int hipc_graph_set_scalar(hipc_ctx *ctx, hipc_graph *graph, int op, int which, int32_t value) {
    if (!graph) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, !ctx->capturing, "hipc_graph_set_scalar while a capture is open");
        HIPC_REQUIRE(ctx, op >= 0 && op < (int)graph->ops.size(), "hipc_graph_set_scalar: the graph recorded %zu operator calls, not %d", graph->ops.size(), op + 1);
        int changed = 0;
        for (const ScalarPatch &sp : graph->ops[(size_t)op].patches) {
            if (sp.which != which) continue;
            hipKernelNodeParams params{};
            HIPC_TRY(ctx, hipGraphKernelNodeGetParams(sp.node, &params));
            HIPC_REQUIRE(ctx, params.kernelParams && params.kernelParams[0], "hipc_graph_set_scalar: the kernel node carries no arguments");
            memcpy(static_cast<char *>(params.kernelParams[0]) + sp.offset, &value, sizeof value);
            HIPC_TRY(ctx, hipGraphKernelNodeSetParams(sp.node, &params));           // the graph itself, for later instantiations
            HIPC_TRY(ctx, hipGraphExecKernelNodeSetParams(graph->exec, sp.node, &params));
            changed++;
        }
        HIPC_REFUSE(ctx, changed == 0, "hipc_graph_set_scalar: operator call %d of the graph has no scalar %d that a replay can change", op, which);
        return HIPC_OK;
    });
}

int hipc_measure_graph(hipc_ctx *ctx, hipc_graph *graph, int samples, int launches_per_sample, double *ns_out) {
    if (!graph || !ns_out) return HIPC_ERR_INVALID;
    return entry(ctx, [&]() -> int {
        HIPC_REQUIRE(ctx, samples > 0 && launches_per_sample > 0, "hipc_measure_graph: counts must be positive");
        HIPC_REQUIRE(ctx, !ctx->capturing, "hipc_measure_graph while a capture is open");
        hipEvent_t t0, t1;
        HIPC_TRY(ctx, hipEventCreate(&t0));
        HIPC_TRY(ctx, hipEventCreate(&t1));
        int rc = HIPC_OK;
        for (int s = 0; s < samples && rc == HIPC_OK; s++) {
            hipError_t e = hipEventRecord(t0, ctx->stream);
            for (int i = 0; i < launches_per_sample && e == hipSuccess; i++) e = hipGraphLaunch(graph->exec, ctx->stream);
            if (e == hipSuccess) e = hipEventRecord(t1, ctx->stream);
            if (e == hipSuccess) e = hipEventSynchronize(t1);
            float ms = 0.f;
            if (e == hipSuccess) e = hipEventElapsedTime(&ms, t0, t1);
            if (e != hipSuccess) {
                rc = fail(ctx, HIPC_ERR_BACKEND, "hipc_measure_graph: %s", hipGetErrorString(e));
                break;
            }
            ns_out[s] = (double)ms * 1e6 / launches_per_sample;
        }
        (void)hipEventDestroy(t0);
        (void)hipEventDestroy(t1);
        return rc;
    });
}

}  // extern "C"
