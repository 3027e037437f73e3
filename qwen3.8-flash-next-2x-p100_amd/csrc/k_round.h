// A greedy decode round that the host only enqueues (session.cpp:530-679 drives the same steps from the host and waits
// for each; the reference captures its windows in graphs, engine_common.cu:993-1021, but accepts on the host):
//   verify the window -> accept -> commit -> draft from the rows kept -> prompt lookup -> the next window.
// What one step leaves for the next lives in device words (fnx_round.state), so a round's launches take no argument that
// changes from round to round: rounds can be enqueued back to back, or captured once in a graph and replayed.
//
// A window always has FNX_MAXT rows; state[FNX_RS_ROWS] says how many of them count. The others hold token 0: they
// append their K and V like any row (their cache cells are overwritten by the next window, as a rejected draft's are)
// but ask no queries and are not routed, so they pull no expert's weights, and acceptance never reaches them.
#pragma once

#include "../../include/fnx_mi355x.h"

namespace fnx {

// after the verify (session.cpp:565-573, 616-640): n = 1 + the drafts that equal the row before's pick; the picks of the
// rows kept join the context; the positions move on by n. One wave.
// A round whose next window would not fit the caches (max_ctx) or the context buffer raises FNX_RS_STOP and changes
// nothing; every later round then finds the same state and repeats the same work. So does the first round of a badly
// placed session (a position below zero, or a window that does not fit to begin with: the verify before this computed
// over the cells that exist and is not kept).
__global__ void k_round_commit(const int* __restrict__ rows, const int* __restrict__ best, int* __restrict__ state, int* __restrict__ ctx,
                               int ctx_cap, int max_ctx, int* __restrict__ log, int log_cap) {
    const int i = threadIdx.x;
    const int R = min(max(state[FNX_RS_ROWS], 1), FNX_MAXT), n_ctx = state[FNX_RS_NCTX], pos = state[FNX_RS_POS], rounds = state[FNX_RS_ROUNDS];
    const int stop = state[FNX_RS_STOP];
    const bool ok = i + 1 < R && rows[i + 1] == best[i];
    const int n = 1 + (int) __builtin_ctzll(~__ballot(ok));
    const int pick = i < n ? best[i] : 0;
    if (stop || pos < 0 || pos + n + FNX_MAXT > max_ctx || n_ctx + n + FNX_MAXT > ctx_cap) {
        if (i == 0) state[FNX_RS_STOP] = 1;
        return;
    }
    if (i < n) ctx[n_ctx + i] = pick;
    if (i == 0) {
        state[FNX_RS_NCTX] = n_ctx + n;
        state[FNX_RS_POS] = pos + n;
        state[FNX_RS_POS_PREV] = pos;
        state[FNX_RS_ACCEPTED] = n;
        state[FNX_RS_ROUNDS] = rounds + 1;
        if (log && rounds < log_cap) {
            log[2 * rounds] = R - 1;
            log[2 * rounds + 1] = n;
        }
    }
}

// the MTP chain (session.cpp:666-678) starts when the lookup found nothing: its first draft is the draft layer's pick for
// the last row kept, its source that row of the draft layer's output. The steps' positions are written in any case (a
// step that does not count still appends its row to the draft layer's cache, in cells that the next round's pass over the
// rows kept writes again before anything reads them). One block.
__global__ void k_chain_begin(int* __restrict__ state, int* __restrict__ scratch, const int* __restrict__ draft_best,
                              const float* __restrict__ hidden, int n, float* __restrict__ chain_src, int K) {
    const int kept = min(max(state[FNX_RS_ACCEPTED], 1), FNX_MAXT), pos = state[FNX_RS_POS];
    const bool run = !state[FNX_RS_STOP] && scratch[0] <= 0;
    __syncthreads();   // every thread has read the words that thread 0 is about to write
    if (threadIdx.x < FNX_MAXT) state[FNX_RS_CHAIN_POS + threadIdx.x] = pos + threadIdx.x;
    if (threadIdx.x == 0) {
        state[FNX_RS_CHAIN] = run ? 1 : 0;
        if (run) scratch[1] = draft_best[kept - 1];
    }
    if (run)
        for (int i = threadIdx.x; i < n; i += blockDim.x) chain_src[i] = hidden[(size_t) (kept - 1) * n + i];
}
// after step j (1 .. K - 1) of the chain: its pick is draft j + 1; the last step hands the K drafts to the next window
__global__ void k_chain_keep(const int* __restrict__ state, int* __restrict__ scratch, const int* __restrict__ best, int j, int K) {
    if (threadIdx.x != 0 || !state[FNX_RS_CHAIN]) return;
    scratch[1 + j] = best[0];
    if (j == K - 1) scratch[0] = K;
}

// the next window (session.cpp:530-560): the last token of the context, then the lookup's drafts, or else the draft
// layer's pick for the last row kept; without speculation the token alone. One wave.
__global__ void k_round_window(const int* __restrict__ ctx, int* __restrict__ state, const int* __restrict__ drafts,
                               const int* __restrict__ n_drafts, const int* __restrict__ draft_best, int speculate, int* __restrict__ rows) {
    const int i = threadIdx.x;
    if (state[FNX_RS_STOP]) return;
    const int n_ctx = state[FNX_RS_NCTX], n = min(max(state[FNX_RS_ACCEPTED], 1), FNX_MAXT);
    int R = 1, tok = 0;
    if (speculate) {
        const int nd = min(max(*n_drafts, 0), FNX_MAXT - 1);
        if (nd > 0) {
            R = 1 + nd;
            if (i >= 1 && i <= nd) tok = drafts[i - 1];
        } else {
            R = 2;
            if (i == 1) tok = draft_best[n - 1];
        }
    }
    if (i == 0) tok = ctx[n_ctx - 1];
    if (i < FNX_MAXT) rows[i] = tok;
    if (i == 0) state[FNX_RS_ROWS] = R;
}

}  // namespace fnx
