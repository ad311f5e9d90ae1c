// Address model of the decode step: the library's own sources (matmul_nbits.hip, gemv_lean.hip,
// decoder.hip, with prefetch.h and lanes.h) compiled as host code behind gpu_model.h, driven through
// the same entry points a caller uses. Every launch of a step runs thread by thread on the CPU; every
// buffer load is checked against the allocations the library itself made (hipc_decoder_create,
// nbits_prepack: their sizes, byte for byte), under the hardware's rule that the descriptor's range
// check sees the per-lane offset only; every ordinary load and store is checked by AddressSanitizer.
// The read-ahead helper rows are on (kReadAheadVerified is true in this build): what this program
// verifies is exactly what that constant stands for.
//
//   decoder_model full           whole steps at positions around every boundary of the chunking (0, 16, 32, 64, 512,
//                                2048, the windows, the end of the cache), windows 0 / 70 / 512 / 4200, every shape
//                                below: the shapes of the GPU tests and gemma3-1b's (two layers of it, whole vocabulary)
//   decoder_model sweep [threads] the launches whose addresses depend on the position (the q|k|v launch's helper rows,
//                                which read the cache ahead; the attention launch; the output projection's join) at
//                                EVERY position of the cache, the same windows and shapes
//   decoder_model quick [threads] what the test suite runs: the full steps on a shorter list of positions, and the
//                                sweep of gemma3-1b's shape at every position below 96, every 29th beyond and the
//                                last 40, windows 0 and 512
#include <cstdio>
#include <mutex>
#include <thread>
#include <vector>

#include "internal.h"

// ---- what the three sources leave undefined ---------------------------------------------------
namespace hipc {
alignas(16) thread_local uint4 lean_smem[160 * 1024 / 16];   // the kernels' dynamic LDS (`extern __shared__`)
alignas(16) thread_local uint4 smem[160 * 1024 / 16];
thread_local float wgt[40960];
int scratch_get(hipc_ctx *ctx, int slot, size_t bytes, void **out) {
    Scratch &s = ctx->scratch[slot];
    if (s.bytes < bytes) {
        if (s.ptr) gpu_model::release(s.ptr);
        s.ptr = gpu_model::alloc(bytes);   // exactly what was asked for: stricter than the library's rounding
        s.bytes = bytes;
    }
    *out = s.ptr;
    return HIPC_OK;
}
bool nbits_prefill_takes(const void *, const hipc_nbits_weight *, int64_t) { return false; }
int nbits_prefill(hipc_ctx *, const void *, const hipc_nbits_weight *, void *, int64_t) { return HIPC_ERR_UNSUPPORTED; }
bool nbits_prefill_f32_takes(const void *, const hipc_nbits_weight *, int64_t) { return false; }
int nbits_prefill_f32(hipc_ctx *, const void *, const hipc_nbits_weight *, void *, int64_t, int) { return HIPC_ERR_UNSUPPORTED; }
}  // namespace hipc
extern "C" {
const char *hipGetErrorString(hipError_t) { return "model"; }
hipError_t hipMemcpy(void *d, const void *s, size_t n, hipMemcpyKind) { std::memcpy(d, s, n); return hipSuccess; }
hipError_t hipSetDevice(int) { return hipSuccess; }
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
hipError_t hipStreamGetCaptureInfo_v2(hipStream_t, hipStreamCaptureStatus *status, unsigned long long *, hipGraph_t *, const hipGraphNode_t **, size_t *n) {
    *status = hipStreamCaptureStatusNone, *n = 0;
    return hipSuccess;
}
}

#define MUST(call)                                                                    \
    do {                                                                              \
        const int rc_ = (call);                                                       \
        if (rc_ != HIPC_OK) {                                                         \
            std::printf("FAILED %s:%d: %s -> %d (%s)\n", __FILE__, __LINE__, #call, rc_, ctx.err.c_str()); \
            std::exit(1);                                                             \
        }                                                                             \
    } while (0)

namespace {

struct Shape {
    const char *name;
    int layers, hidden, ffn, nq, nkv, hd, vocab, max_seq;
};

// which launches of a step run, and which rows of their grids (set per run; read by gpu_model_launch)
struct Select {
    bool on = false;
    int index = 0;                       // launches seen since the step began
    std::function<bool(int, unsigned *, unsigned *)> rows;   // launch index -> run? and its blockIdx.y range
};
thread_local Select g_select;

struct Model {
    hipc_ctx ctx;
    hipc_decoder *dec = nullptr;
    hipc_decoder_config cfg{};
    std::vector<void *> inputs;

    void *input(size_t bytes) {
        void *p = gpu_model::alloc(bytes);
        inputs.push_back(p);
        return p;
    }
    void build(const Shape &s) {
        ctx.tune.dec_prefetch = 31;   // the helper rows are what is being verified
        cfg.n_layers = s.layers, cfg.hidden = s.hidden, cfg.ffn = s.ffn, cfg.n_q_heads = s.nq, cfg.n_kv_heads = s.nkv;
        cfg.head_dim = s.hd, cfg.vocab = s.vocab, cfg.max_seq = s.max_seq, cfg.block_size = 32;
        cfg.rms_eps = 1e-6f, cfg.rope_theta = 10000.f, cfg.attn_scale = 0.f, cfg.embed_scale = 1.f;
        MUST(hipc_decoder_create(&ctx, &cfg, &dec));
        const int64_t qd = (int64_t)s.nq * s.hd, kvd = (int64_t)s.nkv * s.hd;
        auto linear = [&](int layer, int which, int64_t K, int64_t N) {
            const int64_t nb = (K + 31) / 32;
            const size_t b_len = (size_t)N * nb * 16, s_len = (size_t)N * nb, z_len = (size_t)N * ((nb + 1) / 2);
            void *B = input(b_len), *S = input(s_len * 4), *Z = input(z_len);
            MUST(hipc_decoder_set_linear(&ctx, dec, layer, which, B, b_len, S, s_len, Z, z_len));
        };
        for (int li = 0; li < s.layers; li++) {
            linear(li, HIPC_DEC_QKV, s.hidden, qd + 2 * kvd);
            linear(li, HIPC_DEC_O, qd, s.hidden);
            linear(li, HIPC_DEC_GATE_UP, s.hidden, 2 * (int64_t)s.ffn);
            linear(li, HIPC_DEC_DOWN, s.ffn, s.hidden);
            for (int n = 0; n < 6; n++) {
                void *w = input((size_t)std::max(s.hidden, s.hd) * 4);
                MUST(hipc_decoder_set_norm(&ctx, dec, li, n, w));
            }
        }
        linear(0, HIPC_DEC_LM_HEAD, s.hidden, s.vocab);
        MUST(hipc_decoder_set_norm(&ctx, dec, 0, HIPC_DEC_NORM_FINAL, input((size_t)s.hidden * 4)));
        const int64_t nb = (s.hidden + 31) / 32;
        const size_t qb = (size_t)s.vocab * nb * 16, sb = (size_t)s.vocab * nb, zb = (size_t)s.vocab * ((nb + 1) / 2);
        MUST(hipc_decoder_set_embedding(&ctx, dec, input(qb), qb, input(sb * 4), sb, input(zb), zb));
    }
    void step_at(int pos, int token) {
        g_select.index = 0;
        const bool was = g_select.on;
        g_select.on = false;
        MUST(hipc_decoder_reset(&ctx, dec, token, pos));
        g_select.on = was;
        g_select.index = 0;
        MUST(hipc_decoder_step(&ctx, dec));
    }
    void windows(int w) {
        for (int li = 0; li < cfg.n_layers; li++) MUST(hipc_decoder_set_layer_attention(&ctx, dec, li, li == 0 ? w : 0, li == 0 && w ? 1.0e6f : 0.f));
    }
    void destroy() {
        hipc_decoder_destroy(&ctx, dec);
        for (void *p : ctx.deferred) gpu_model::release(p);
        ctx.deferred.clear();
        for (void *p : inputs) gpu_model::release(p);
        inputs.clear();
        for (hipc::Scratch &s : ctx.scratch)
            if (s.ptr) gpu_model::release(s.ptr), s.ptr = nullptr, s.bytes = 0;
    }
};

const Shape kGemma = {"gemma3-1b (two layers)", 2, 1152, 6912, 4, 1, 256, 262144, 2112};
const Shape kSmall[] = {
    {"small hd 64, 4 q / 2 kv", 2, 128, 256, 4, 2, 64, 512, 80},
    {"small hd 256, 4 q / 1 kv", 2, 128, 256, 4, 1, 256, 512, 2054},
    {"small hd 128, 8 q / 1 kv", 2, 128, 256, 8, 1, 128, 512, 4298},
    {"small hd 64, 2 q / 2 kv", 2, 128, 256, 2, 2, 64, 512, 2308},
    {"small hd 128, 4 q / 2 kv", 2, 128, 256, 4, 2, 128, 512, 517},
    {"small hd 192 (three-kernel attention)", 2, 128, 256, 2, 1, 192, 512, 108},
};

// counters of all host threads (a thread adds its registry's when it is done)
std::mutex g_totals_mu;
size_t g_launches = 0, g_threads = 0, g_loads = 0, g_clipped = 0;
void add_totals() {
    gpu_model::Registry &g = gpu_model::reg();
    std::lock_guard<std::mutex> lock(g_totals_mu);
    g_launches += g.launches, g_threads += g.threads, g_loads += g.loads, g_clipped += g.loads_clipped;
    g.launches = g.threads = g.loads = g.loads_clipped = 0;
}
void report(const char *what) {
    add_totals();
    std::printf("%-44s %7zu launches %11zu threads %11zu buffer loads (%zu answered with zeros)\n", what, g_launches, g_threads, g_loads, g_clipped);
    std::fflush(stdout);
    g_launches = g_threads = g_loads = g_clipped = 0;
}

bool g_quick = false;
std::vector<int> windows_of(const Shape &s) {
    if (g_quick) return {0, 512};
    std::vector<int> w = {0, 70, 512, 4200};
    w.erase(std::remove_if(w.begin(), w.end(), [&](int v) { return v >= s.max_seq; }), w.end());
    return w;
}

void full(const Shape &s) {
    Model m;
    gpu_model::reg().where = s.name;
    m.build(s);
    const int last = s.max_seq - 1;
    const std::vector<int> all = {0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 69, 70, 71, 511, 512, 513, 527, 528, 1023, 2039, 2040, 2047, 2048, 2049, 4199, 4200, 4201, last - 1, last};
    const std::vector<int> few = {0, 1, 31, 32, 33, 512, 513, 2048, last};
    for (int w : windows_of(s)) {
        m.windows(w);
        for (int pos : g_quick ? few : all)
            if (pos >= 0 && pos <= last) m.step_at(pos, (pos * 7 + 3) % s.vocab);
    }
    // a step with the cache full changes nothing and reads nothing out of range
    m.step_at(last, s.vocab - 1);
    {
        hipc_ctx &ctx = m.ctx;
        MUST(hipc_decoder_step(&ctx, m.dec));
        int32_t token = 0, pos = 0;
        const int rc = hipc_decoder_read(&ctx, m.dec, &token, &pos, nullptr, nullptr, 0);
        if (rc == HIPC_OK || pos != s.max_seq) {
            std::printf("FAILED: a step past the end of the cache was not reported (rc %d, position %d)\n", rc, pos);
            std::exit(1);
        }
    }
    m.destroy();
    report(s.name);
}

// The launches whose addresses depend on the position, at every position. In the lean path a layer's
// launches are, from index 1 + 5 layer on: q|k|v (its helper rows read the cache ahead: rows >= 1),
// attention (rows < kv heads: its own; the helper rows behind them read the next launch's weights and
// do not depend on the position), output projection (rows < 8 cover its k slices), gate|up, down.
void sweep(const Shape &s, int threads) {
    // the output projection's own rows: its k slices, as hipc_decoder_create cuts them (one head per slice, at most 8)
    const int n_cg_o = (s.nq * s.hd + 127) / 128;
    int o_tiles = std::max(1, s.hd / 128);
    while ((n_cg_o + o_tiles - 1) / o_tiles > 4 && o_tiles < 4) o_tiles *= 2;
    const unsigned o_slices = (unsigned)((n_cg_o + o_tiles - 1) / o_tiles);
    for (int w : windows_of(s)) {
        std::vector<std::thread> pool;
        for (int t = 0; t < threads; t++) {
            pool.emplace_back([&, t] {
                gpu_model::reg().where = s.name;
                Model m;
                m.build(s);
                m.windows(w);
                g_select.on = true;
                g_select.rows = [&](int index, unsigned *y0, unsigned *y1) {
                    if (index == 1) { *y0 = 1, *y1 = ~0u; return true; }
                    if (index == 2) { *y0 = 0, *y1 = (unsigned)s.nkv; return true; }
                    if (index == 3) { *y0 = 0, *y1 = o_slices; return true; }
                    return false;
                };
                for (int pos = t; pos < s.max_seq; pos += threads)
                    if (!g_quick || pos < 96 || pos % 29 == 0 || pos >= s.max_seq - 40) m.step_at(pos, 1);
                g_select.on = false;
                m.destroy();
                add_totals();
            });
        }
        for (std::thread &th : pool) th.join();
    }
    report(s.name);
}

}  // namespace

int main(int argc, char **argv) {
    const std::string mode = argc > 1 ? argv[1] : "full";
    const int threads = argc > 2 ? std::atoi(argv[2]) : 1;
    gpu_model_select = [](const char *, dim3, unsigned *y0, unsigned *y1) {
        if (!g_select.on) return true;
        return g_select.rows(g_select.index++, y0, y1);
    };
    if (mode == "full") {
        for (const Shape &s : kSmall) full(s);
        full(kGemma);
    } else if (mode == "quick") {
        g_quick = true;
        for (const Shape &s : kSmall) full(s);
        Shape g = kGemma;
        full(g);
        g.vocab = 4096;   // the unembedding is not part of the swept launches
        sweep(g, threads);
    } else if (mode == "sweep") {
        for (const Shape &s : kSmall)
            if (s.hd != 192) sweep(s, threads);   // (no one-launch attention for that head_dim: nothing of it depends on the position this way)
        Shape g = kGemma;
        g.vocab = 4096;   // the unembedding is not part of the swept launches
        sweep(g, threads);
    } else {
        std::printf("usage: decoder_model full | sweep [threads] | quick [threads]\n");
        return 2;
    }
    std::printf("ok\n");
    return 0;
}
