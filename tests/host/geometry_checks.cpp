// Host-side checks of the index arithmetic that host and device code share (compiled for the host
// only, run without a GPU): the split of a decode step's context into chunks, and which weight tiles
// the read-ahead helper workgroups of a launch ask for.
#include <cstdio>
#include <cstdlib>
#include <set>
#include <vector>

#include "internal.h"

using namespace hipc;

#define CHECK(cond, ...)                                     \
    do {                                                     \
        if (!(cond)) {                                       \
            std::printf("FAILED %s:%d: ", __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);                        \
            std::printf("\n");                               \
            std::exit(1);                                    \
        }                                                    \
    } while (0)

static void attention_chunks() {
    const int windows[] = {0, 1, 15, 16, 17, 70, 100, 512, 2048, 4200};
    for (int window : windows) {
        for (int total = 1; total <= 20000; total += (total < 5000 ? 1 : 37)) {
            const int first = attn_first(total, window), base = attn_base(total, window), span = attn_span(total, window);
            CHECK(first >= 0 && first < total, "first %d of %d", first, total);
            CHECK(window <= 0 || total - first <= window, "window %d: %d visible", window, total - first);
            CHECK(window <= 0 || total <= window || total - first == window, "window %d at %d: %d visible", window, total, total - first);
            CHECK(base % 16 == 0 && base <= first && first - base < 16, "base %d of first %d", base, first);
            CHECK(span == total - base, "span");
            const int chunk = attn_chunk(span), live = attn_live_chunks(span);
            CHECK(chunk >= kAttnPass && chunk % kAttnPass == 0, "chunk %d", chunk);
            CHECK(live >= 1 && live <= kAttnSplits, "live %d (span %d, chunk %d)", live, span, chunk);
            // the live chunks cover [base, total), the last one holds the step's own position, the next would be empty
            CHECK(base + (live - 1) * chunk < total && base + live * chunk >= total, "cover: base %d live %d chunk %d total %d", base, live, chunk, total);
            // a chunk starts on a multiple of 16 (32 bytes of the transposed value cache)
            CHECK((base + chunk) % 16 == 0, "alignment");
        }
    }
    CHECK(attn_v_stride(1) == 64 && attn_v_stride(64) == 64 && attn_v_stride(65) == 128, "v stride");
}

// every tile of the consumer is read ahead by exactly one helper, from inside the arrays, and by a
// helper whose linear id is congruent to the consumer's modulo 8 (same XCD, same L2)
static void read_ahead(int n_tiles, int n_cg, int WN, int slice_tiles, int gy, int producer_gx, int producer_main_rows, int rows) {
    PrefetchArgs pf;
    pf.kind = 1, pf.rows = rows;
    pf.gx = (n_tiles + WN - 1) / WN, pf.gy = gy, pf.WN = WN, pf.slice_tiles = slice_tiles, pf.n_cg = n_cg, pf.n_tiles = n_tiles, pf.SG = 4;
    CHECK((long long)gy * slice_tiles >= n_cg, "plan does not cover k");
    const int H = rows * producer_gx;
    const size_t total_tiles = (size_t)n_tiles * n_cg;
    std::vector<int> seen(total_tiles, 0);
    for (int h = 0; h < H; h++) {
        const int b = producer_main_rows * producer_gx + h;   // the helper rows follow the main rows of the producer's grid
        int first, step;
        pf_consumers_of(h, H, b, &first, &step);
        CHECK(step > 0, "step");
        for (int j = first; j < pf.gx * pf.gy; j += step) {
            CHECK((j & 7) == (b & 7), "consumer %d on another XCD than helper %d", j, b);
            for (int wn = 0; wn < WN; wn++) {
                size_t tile0 = 0;
                const int cnt = pf_tile_run(pf, j, wn, &tile0);
                if (cnt == 0) break;
                CHECK(tile0 + cnt <= total_tiles, "run [%zu, +%d) past %zu tiles", tile0, cnt, total_tiles);
                for (int t = 0; t < cnt; t++) seen[tile0 + t]++;
            }
        }
    }
    // with at least eight helpers per class every consumer has a helper; tiles are never read twice
    size_t covered = 0;
    for (size_t t = 0; t < total_tiles; t++) {
        CHECK(seen[t] <= 1, "tile %zu read ahead %d times", t, seen[t]);
        covered += seen[t];
    }
    if (H % 8 == 0 && H >= 8) CHECK(covered == total_tiles, "%zu of %zu tiles read ahead (H = %d)", covered, total_tiles, H);
}

int main() {
    attention_chunks();
    // the decoder's launches at the 1152 / 6912 shape: consumer o (read ahead by the attention launch,
    // 64 x (1 + 3) workgroups), gate | up (by o: 18 x (4 + 8)), down (by gate | up: 432 x (1 + 1)), qkv (by down: 72 x (3 + 3))
    read_ahead(72, 8, 4, 2, 4, 64, 1, 3);
    read_ahead(864, 9, 2, 9, 1, 18, 4, 8);
    read_ahead(72, 54, 1, 18, 3, 432, 1, 1);
    read_ahead(96, 9, 1, 9, 1, 72, 3, 3);
    // ragged shapes: a last slice that is shorter, a column tile count that WN does not divide, helpers not a multiple of 8
    read_ahead(10, 7, 4, 3, 3, 20, 1, 2);
    read_ahead(33, 5, 2, 5, 1, 9, 2, 3);
    std::printf("ok\n");
    return 0;
}
