// Host-side bounds check of the attention kernels' index arithmetic (csrc/attn_window.h): for caches of 192, 520 and
// 32,768 cells, every window position from well below 0 to well past the end, every row count and every block of the
// first pass (whole splits, and the half splits of a window of few queries), walk the chunks as the kernel's loop does and check that each K row and V block it would fetch lies inside
// the cache, that every query's context does, and that the fit predicate is exact. No GPU: an out-of-range position is
// never run on one.
#include <cstdio>
#include <cstdlib>

#include "attn_window.h"

using namespace fnx;

static long checked = 0;
static void require(bool ok, const char* what, int max_ctx, int pos0, int T, int s, int c0) {
    ++checked;
    if (ok) return;
    std::printf("FAILED %s: max_ctx %d pos0 %d T %d split %d chunk %d\n", what, max_ctx, pos0, T, s, c0);
    std::exit(1);
}

int main() {
    const int caps[] = {8, 192, 520, 32768};
    for (int max_ctx : caps) {
        const int nsplit = attn_splits(max_ctx), vblocks = (max_ctx + AT_VB - 1) / AT_VB;
        const int step = max_ctx > 1024 ? 97 : 1;
        for (int pos0 = -40; pos0 <= max_ctx + 40; pos0 += (pos0 > 64 && pos0 < max_ctx - 64 ? step : 1))
            for (int T = 1; T <= 16; ++T) {
                const AttWindow w = att_window(pos0, T, max_ctx);
                const bool fits = pos0 >= 0 && pos0 + T <= max_ctx;
                require(att_window_fits(pos0, T, max_ctx) == fits, "fit predicate", max_ctx, pos0, T, -1, -1);
                require(w.pos0 >= 0 && w.pos0 < max_ctx && w.ctx_max >= 1 && w.ctx_max <= max_ctx, "window", max_ctx, pos0, T, -1, -1);
                if (fits) require(w.pos0 == pos0 && w.ctx_max == pos0 + T, "a window that fits is left alone", max_ctx, pos0, T, -1, -1);
                for (int qt = 0; qt < T; ++qt) {
                    const int c = att_ctx_q(w, qt);
                    require(c >= 1 && c <= w.ctx_max, "query context", max_ctx, pos0, T, -1, qt);
                    if (fits) require(c == pos0 + qt + 1, "query context of a window that fits", max_ctx, pos0, T, -1, qt);
                }
                for (int halves = 0; halves < 2; ++halves) {
                    const int live = att_live_parts(w, nsplit, halves != 0);
                    require(live >= 1 && live <= att_part_slots(nsplit), "live parts", max_ctx, pos0, T, -1, -1);
                    int covered = 0, seen = 0;
                    for (int s = 0; s < nsplit; ++s)
                        for (int z = 0; z < (halves ? 2 : 1); ++z) {
                            const int p0 = att_part_begin(s, z, halves != 0), p1 = att_part_end(w, s, z, halves != 0);
                            const int idx = att_part_index(s, z, halves != 0);
                            require(idx == seen && idx < att_part_stride(nsplit, halves != 0) && att_part_stride(nsplit, halves != 0) <= att_part_slots(nsplit),
                                    "parts are numbered in position order, inside a query's stride", max_ctx, pos0, T, s, z);
                            ++seen;
                            if (p0 >= p1) {
                                require(idx >= live, "an empty part is not a live one", max_ctx, pos0, T, s, z);
                                continue;
                            }
                            require(idx < live, "a part with data is a live one", max_ctx, pos0, T, s, z);
                            require(p0 == covered, "the parts follow one another", max_ctx, pos0, T, s, z);
                            covered = p1;
                            auto fetch = [&](int c0) {
                                for (int r = 0; r < AT_CH; ++r) {
                                    const int row = att_fetch_row(w, c0, r);
                                    require(row >= 0 && row < max_ctx, "K row", max_ctx, pos0, T, s, c0);
                                }
                                for (int b = 0; b < AT_CH / AT_VB; ++b) {
                                    const int blk = att_fetch_vblock(w, c0, b);
                                    require(blk >= 0 && blk < vblocks, "V block", max_ctx, pos0, T, s, c0);
                                }
                            };
                            // the kernel's order: the first chunk, the second if the part has one, then two ahead each trip
                            fetch(p0);
                            if (p0 + AT_CH < p1) fetch(p0 + AT_CH);
                            for (int c0 = p0; c0 < p1; c0 += AT_CH)
                                if (c0 + 2 * AT_CH < p1) fetch(c0 + 2 * AT_CH);
                        }
                    require(covered == w.ctx_max, "the parts cover the window's context", max_ctx, pos0, T, -1, halves);
                }
            }
    }
    std::printf("ok %ld\n", checked);
    return 0;
}
