// Host-side check of the one-launch verify window's work split (csrc/moe_window_plan.h): for every grid size, row count,
// expert width, pick count and expert count the window accepts, walk the blocks as the kernel does and check that every
// router row, every gate|up item and every unit of the down matrices is taken exactly once, that a wave never holds more
// units than its registers allow, and that each hand-over's count equals the number of blocks that arrive on it. No GPU:
// a count that no block brings up would be a wait that only its time limit ends.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "moe_window_plan.h"

using namespace fnx;

static long checked = 0;
static void require(bool ok, const char* what, int nb, int Tl, int ff, int topk, int nexp, int shared) {
    ++checked;
    if (ok) return;
    std::printf("FAILED %s: blocks %d rows %d ff %d topk %d nexp %d shared %d\n", what, nb, Tl, ff, topk, nexp, shared);
    std::exit(1);
}

int main() {
    const int grids[] = {256, 304, 320, 512}, widths[] = {256, 512, 1024}, experts[] = {1, 8, 60, 64, 100, 512, 1000, 1024};
    for (int nb : grids)
        for (int Tl = 1; Tl <= 16 && WN_WAVES * Tl <= nb; ++Tl)
            for (int ff : widths)
                for (int topk = 1; topk <= 16; ++topk)
                    for (int nexp : experts)
                        for (int shared = 0; shared < 2; ++shared) {
#define REQ(c, what) require(c, what, nb, Tl, ff, topk, nexp, shared)
                            const WinPlan p = win_plan(nb, Tl, nexp, topk, shared != 0, ff);
                            REQ(p.G >= WN_WAVES && (p.G & (p.G - 1)) == 0 && p.G * Tl <= nb, "blocks a row");
                            REQ(p.nk == topk + shared && p.k0 == 1 - shared && p.per_row == (ff / 32) * p.nk, "items a row");
                            // gate|up items: block g's run, as the kernel takes it
                            std::vector<int> item(p.per_row, 0);
                            int with_items = 0;
                            for (int g = 0; g < p.G; ++g) {
                                const int I0 = g * p.ipb, I1 = I0 + p.ipb < p.per_row ? I0 + p.ipb : p.per_row;
                                if (I1 > I0) ++with_items;
                                for (int I = I0; I < I1; ++I) {
                                    const int j = I / p.nk, k = p.k0 + I - j * p.nk;
                                    REQ(j >= 0 && j < ff / 32 && k >= p.k0 && k <= topk, "an item's block of 32 and matrix");
                                    // the sixteen waves' units of the item: gate rows 32 j + 2 w, + 1 and the same up rows, inside the 2 ff rows
                                    REQ(32 * j + 2 * (WN_WAVES - 1) + 1 < ff, "an item's units");
                                    ++item[I];
                                }
                            }
                            for (int v : item) REQ(v == 1, "every item once");
                            REQ(with_items == p.nbi && p.nbi >= 1 && p.nbi <= p.G, "the h hand-over's count");
                            // router rows
                            std::vector<int> row(nexp, 0);
                            for (int g = 0; g < p.G; ++g) {
                                const int r0 = g * p.rpb, r1 = r0 + p.rpb < nexp ? r0 + p.rpb : nexp;
                                for (int w = 0; w < WN_WAVES; ++w)
                                    for (int r = r0 + w; r < r1; r += WN_WAVES) ++row[r];
                            }
                            for (int v : row) REQ(v == 1, "every router row once");
                            // units of a down matrix
                            std::vector<int> unit(ff, 0);
                            REQ(p.R >= 1 && p.R <= win_rmax(ff / 32) && p.dwaves >= 1 && p.dwaves <= WN_WAVES && p.dwaves * p.R == p.upb, "units a wave");
                            for (int g = 0; g < p.G; ++g)
                                for (int w = 0; w < p.dwaves; ++w)
                                    for (int r = 0; r < p.R; ++r) {
                                        const int u = g * p.upb + w * p.R + r;
                                        REQ(u >= 0 && u < ff, "a unit inside the matrix");
                                        ++unit[u];
                                    }
                            for (int v : unit) REQ(v == 1, "every unit once");
#undef REQ
                        }
    std::printf("ok %ld\n", checked);
    return 0;
}
