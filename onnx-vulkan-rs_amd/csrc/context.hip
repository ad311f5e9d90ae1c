// Context, buffers, capture/replay and timing: the part of the library that
// stands where the reference's `vk-compute` runtime does
// (crates/vk-compute/src/{buffer,stream,pipeline}.rs). One in-order HIP stream
// gives the reference's "every command waits for everything before it"
// semantics (stream.rs:11-14) by construction; a HIP graph is its capture/replay.
#include <algorithm>
#include <cstring>

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
        if (s.ptr) ctx->deferred.push_back(s.ptr);
        s.ptr = nullptr;
        s.bytes = 0;
        size_t want = (bytes + 0xfffff) & ~(size_t)0xfffff;
        HIPC_TRY(ctx, hipMalloc(&s.ptr, want));
        s.bytes = want;
    }
    *out = s.ptr;
    return HIPC_OK;
}

static int release_deferred(hipc_ctx *ctx) {
    for (void *p : ctx->deferred) (void)hipFree(p);
    ctx->deferred.clear();
    return HIPC_OK;
}

static int create(int device, void *stream, bool adopt, hipc_ctx **out) {
    if (!out) return HIPC_ERR_INVALID;
    *out = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count) return HIPC_ERR_BACKEND;
    if (hipSetDevice(device) != hipSuccess) return HIPC_ERR_BACKEND;
    hipc_ctx *ctx = new hipc_ctx();
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
    if (hipMalloc(&ctx->params, kParamBytes) != hipSuccess ||
        hipMemsetAsync(ctx->params, 0, kParamBytes, ctx->stream) != hipSuccess) {
        delete ctx;
        return HIPC_ERR_BACKEND;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0)
        ctx->cu_count = prop.multiProcessorCount;
    *out = ctx;
    return HIPC_OK;
}

int ratio_resident(hipc_ctx *ctx, RatioCache &cache, const std::vector<float> &ratio, const float **out) {
    if (cache.dev && cache.host.size() == ratio.size() &&
        memcmp(cache.host.data(), ratio.data(), ratio.size() * sizeof(float)) == 0) {
        *out = cache.dev;
        return HIPC_OK;
    }
    HIPC_REFUSE(ctx, ctx->capturing, "QLinear: the requantisation ratios changed and would have to be uploaded inside a capture; run the operator once before capturing");
    if (cache.host.size() != ratio.size() || !cache.dev) {
        // earlier launches may still read the old buffer: it goes with the next flush
        if (cache.dev) ctx->deferred.push_back(cache.dev);
        cache.dev = nullptr;
        HIPC_TRY(ctx, hipMalloc(reinterpret_cast<void **>(&cache.dev), std::max<size_t>(ratio.size() * sizeof(float), 16)));
    } else {
        HIPC_TRY(ctx, hipStreamSynchronize(ctx->stream));  // nobody reads the buffer while it is rewritten
    }
    HIPC_TRY(ctx, hipMemcpyAsync(cache.dev, ratio.data(), ratio.size() * sizeof(float), hipMemcpyHostToDevice, ctx->stream));
    HIPC_TRY(ctx, hipStreamSynchronize(ctx->stream));
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

const char *hipc_version(void) { return "hipcompute 0.1 (gfx950)"; }

int hipc_ctx_create(int device, hipc_ctx **out) { return create(device, nullptr, false, out); }

int hipc_ctx_create_on_stream(int device, void *stream, hipc_ctx **out) {
    return create(device, stream, true, out);
}

void hipc_ctx_destroy(hipc_ctx *ctx) {
    if (!ctx) return;
    {
        Guard g(ctx);
        (void)hipStreamSynchronize(ctx->stream);
        release_deferred(ctx);
        for (Scratch &s : ctx->scratch)
            if (s.ptr) (void)hipFree(s.ptr);
        if (ctx->params) (void)hipFree(ctx->params);
        if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
    }
    delete ctx;
}

const char *hipc_last_error(hipc_ctx *ctx) { return ctx ? ctx->err.c_str() : "null context"; }

void *hipc_stream(hipc_ctx *ctx) { return ctx ? static_cast<void *>(ctx->stream) : nullptr; }

int hipc_alloc(hipc_ctx *ctx, size_t bytes, void **dptr) {
    if (!ctx || !dptr) return HIPC_ERR_INVALID;
    Guard g(ctx);
    HIPC_REFUSE(ctx, ctx->capturing, "hipc_alloc while a capture is open");
    *dptr = nullptr;
    HIPC_TRY(ctx, hipMalloc(dptr, bytes ? bytes : 4));
    return HIPC_OK;
}

int hipc_free_deferred(hipc_ctx *ctx, void *dptr) {
    if (!ctx) return HIPC_ERR_INVALID;
    Guard g(ctx);
    if (dptr) ctx->deferred.push_back(dptr);
    return HIPC_OK;
}

int hipc_upload(hipc_ctx *ctx, void *dst, size_t dst_offset, const void *host, size_t bytes) {
    if (!ctx) return HIPC_ERR_INVALID;
    Guard g(ctx);
    HIPC_REFUSE(ctx, ctx->capturing, "hipc_upload while a capture is open: a replay would re-read the host pointer");
    if (bytes == 0) return HIPC_OK;
    HIPC_REQUIRE(ctx, dst && host, "hipc_upload: null pointer");
    // pageable source: the runtime stages the bytes before returning, so `host` is free again
    HIPC_TRY(ctx, hipMemcpyAsync(static_cast<char *>(dst) + dst_offset, host, bytes, hipMemcpyHostToDevice,
                                 ctx->stream));
    HIPC_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return HIPC_OK;
}

int hipc_download(hipc_ctx *ctx, void *host, const void *src, size_t src_offset, size_t bytes) {
    if (!ctx) return HIPC_ERR_INVALID;
    Guard g(ctx);
    HIPC_REFUSE(ctx, ctx->capturing, "hipc_download while a capture is open");
    HIPC_TRY(ctx, hipStreamSynchronize(ctx->stream));
    release_deferred(ctx);
    if (bytes == 0) return HIPC_OK;
    HIPC_REQUIRE(ctx, host && src, "hipc_download: null pointer");
    HIPC_TRY(ctx, hipMemcpy(host, static_cast<const char *>(src) + src_offset, bytes, hipMemcpyDeviceToHost));
    return HIPC_OK;
}

int hipc_copy(hipc_ctx *ctx, void *dst, size_t dst_offset, const void *src, size_t src_offset, size_t bytes) {
    if (!ctx) return HIPC_ERR_INVALID;
    Guard g(ctx);
    if (bytes == 0) return HIPC_OK;
    HIPC_REQUIRE(ctx, dst && src, "hipc_copy: null pointer");
    HIPC_TRY(ctx, hipMemcpyAsync(static_cast<char *>(dst) + dst_offset, static_cast<const char *>(src) + src_offset,
                                 bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return HIPC_OK;
}

int hipc_fill(hipc_ctx *ctx, void *dst, size_t dst_offset, size_t bytes, uint32_t word) {
    if (!ctx) return HIPC_ERR_INVALID;
    Guard g(ctx);
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
}

int hipc_flush(hipc_ctx *ctx) {
    if (!ctx) return HIPC_ERR_INVALID;
    Guard g(ctx);
    HIPC_REFUSE(ctx, ctx->capturing, "hipc_flush while a capture is open");
    HIPC_TRY(ctx, hipStreamSynchronize(ctx->stream));
    release_deferred(ctx);
    return HIPC_OK;
}

int hipc_capture_begin(hipc_ctx *ctx) {
    if (!ctx) return HIPC_ERR_INVALID;
    Guard g(ctx);
    HIPC_REQUIRE(ctx, !ctx->capturing, "hipc_capture_begin: a capture is already open");
    HIPC_TRY(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    return HIPC_OK;
}

int hipc_capture_end(hipc_ctx *ctx, hipc_graph **out) {
    if (!ctx || !out) return HIPC_ERR_INVALID;
    Guard g(ctx);
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
    *out = gr;
    return HIPC_OK;
}

int hipc_graph_launch(hipc_ctx *ctx, hipc_graph *graph) {
    if (!ctx || !graph) return HIPC_ERR_INVALID;
    Guard g(ctx);
    HIPC_REQUIRE(ctx, !ctx->capturing, "hipc_graph_launch while a capture is open");
    HIPC_TRY(ctx, hipGraphLaunch(graph->exec, ctx->stream));
    return HIPC_OK;
}

void hipc_graph_destroy(hipc_ctx *ctx, hipc_graph *graph) {
    if (!ctx || !graph) return;
    Guard g(ctx);
    (void)hipStreamSynchronize(ctx->stream);
    if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph) (void)hipGraphDestroy(graph->graph);
    delete graph;
}

int hipc_measure_graph(hipc_ctx *ctx, hipc_graph *graph, int samples, int launches_per_sample, double *ns_out) {
    if (!ctx || !graph || !ns_out) return HIPC_ERR_INVALID;
    Guard g(ctx);
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
}

}  // extern "C"
