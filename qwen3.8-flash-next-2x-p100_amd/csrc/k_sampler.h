// The sampler's candidates (kernels.hpp:434-447 top_tokens / penalize_row, topk.cuh): per row of the head's logits the
// row's logit_bias and penalties applied in place (repeat multiplies a non-positive logit and divides a positive one,
// then frequency x count and presence once), then its 64 highest, ordered by logit (descending) and token id (ascending)
// on ties, however many tie. err bit 16: a logit was NaN or inf before the penalties.
//
// The reference ranks a row in one block (radix passes over the whole row). Here a row is cut into slices of 2,560
// logits, one block each, so a window's rows fill the chip: a block keeps its slice's 64 best, a second launch keeps the
// 64 best of a row's slices and sorts them. "The 64 best" is always the same selection by a wave over the values its
// lanes hold: the threshold key found bit by bit (counting with ballots: no memory traffic), ties at the threshold taken by
// lowest id the same way; every (key, id) pair is distinct, so the result does not depend on how the row was cut.
#pragma once

#include "fnx_device.h"

namespace fnx {

constexpr int SM_N = 64;                                                    // candidates a row (kernels.hpp:440 TOPK_N)
constexpr int SM_THREADS = 256, SM_V = 10, SM_SLICE = SM_THREADS * SM_V;   // a block's slice: 2,560 logits
constexpr int SM_PEN_CAP = 4096;                                            // penalized tokens a row, at most (engine.hpp:73 PEN_CAP)
constexpr int SM_MAXS = 128;                                                // slices a row, at most (327,680 logits)
constexpr int SM_MERGE_THREADS = 1024, SM_MERGE_V = SM_MAXS * SM_N / SM_MERGE_THREADS;   // 8 candidates a lane
// the slices' candidates between the two launches: one top_tokens in flight per device
__device__ unsigned long long g_topk_cand[FNX_MAXT * SM_MAXS * SM_N];

// order-preserving key of a float's bits: a larger float, a larger key (topk.cuh:13-16)
__device__ __forceinline__ unsigned tk_key(float v) {
    const unsigned u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// a small count summed over the wave's lanes with DPP adds; every lane gets the total. (Counting with a ballot a value
// costs a trip from the vector to the scalar unit each, one after another through the one condition register.)
__device__ __forceinline__ int wave_total(int v) {
#define FNX_DPP_ADDI(ctrl, rmask) v += __builtin_amdgcn_update_dpp(0, v, ctrl, rmask, 0xF, false)
    FNX_DPP_ADDI(0xB1, 0xF);    // quad_perm [1,0,3,2]
    FNX_DPP_ADDI(0x4E, 0xF);    // quad_perm [2,3,0,1]
    FNX_DPP_ADDI(0x141, 0xF);   // row_half_mirror
    FNX_DPP_ADDI(0x140, 0xF);   // row_mirror
    FNX_DPP_ADDI(0x142, 0xA);   // row_bcast15 into rows 1 and 3
    FNX_DPP_ADDI(0x143, 0xC);   // row_bcast31 into rows 2 and 3
#undef FNX_DPP_ADDI
    return __builtin_amdgcn_readlane(v, 63);
}

// The 64 greatest of a wave's 64 V (key, idf) pairs, as a mask of each lane's slots. Real pairs are distinct and have
// idf != 0 (idf = 0xffffffff - id); empty slots are (0, 0), lose to every real pair and are only "selected" by being
// left over when fewer than 64 pairs are real. Greater key first, then greater idf (= the lower id).
template <int V>
__device__ __forceinline__ unsigned wave_select64(const unsigned (&key)[V], const unsigned (&idf)[V]) {
    // 64 real pairs or fewer (a short tail slice, a wave past the row's end): all of them
    int mine = 0;
    unsigned all = 0;
#pragma unroll
    for (int v = 0; v < V; ++v) {
        mine += idf[v] != 0u;
        all |= (idf[v] != 0u ? 1u : 0u) << v;
    }
    if (wave_total(mine) <= SM_N) return all;
    const auto count_ge = [&](unsigned th) {
        int c = 0;
#pragma unroll
        for (int v = 0; v < V; ++v) c += key[v] >= th;
        return wave_total(c);
    };
    // the greatest k with at least 64 keys >= k, bit by bit; a threshold with exactly 64 at or above it ends the search
    unsigned k = 0;
    for (unsigned bit = 0x80000000u; bit; bit >>= 1) {
        const int c = count_ge(k | bit);
        if (c >= SM_N) k |= bit;
        if (c == SM_N) {
            unsigned sel = 0;
#pragma unroll
            for (int v = 0; v < V; ++v) sel |= (key[v] >= k ? 1u : 0u) << v;
            return sel;
        }
    }
    // more than 64 keys >= k, fewer than 64 above it: the rest come from the pairs at k, the greatest idf first
    int above = 0, at = 0;
#pragma unroll
    for (int v = 0; v < V; ++v) {
        above += key[v] > k;
        at += key[v] == k;
    }
    above = wave_total(above);
    at = wave_total(at);
    const int want = SM_N - above;
    unsigned f = 0;   // all of them: every idf >= 0
    if (at > want) {
        // the greatest f with at least `want` pairs (k, idf >= f): idfs are distinct, so exactly `want` at the end
        for (unsigned bit = 0x80000000u; bit; bit >>= 1) {
            int c = 0;
#pragma unroll
            for (int v = 0; v < V; ++v) c += key[v] == k && idf[v] >= (f | bit);
            c = wave_total(c);
            if (c >= want) f |= bit;
            if (c == want) break;
        }
    }
    unsigned sel = 0;
#pragma unroll
    for (int v = 0; v < V; ++v) sel |= (key[v] > k || (key[v] == k && idf[v] >= f) ? 1u : 0u) << v;
    return sel;
}
// the selected pairs, packed (key << 32 | idf), to out[0 .. 64) in (slot, lane) order
template <int V>
__device__ __forceinline__ void wave_emit64(const unsigned (&key)[V], const unsigned (&idf)[V], unsigned sel, unsigned long long* out) {
    const int lane = threadIdx.x & 63;
    int base = 0;
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const bool on = (sel >> v) & 1u;
        const unsigned long long b = __ballot(on);
        if (on) out[base + __popcll(b & ((1ull << lane) - 1ull))] = (unsigned long long) key[v] << 32 | idf[v];
        base += __popcll(b);
    }
    if (base + lane < SM_N) out[base + lane] = 0ull;   // fewer than 64 real pairs: the rest are empty
}

struct TopArgs {
    float* logits;
    int n, v0, nslice;
    const int *pen_tok, *pen_cnt, *pen_n;
    int pen_stride;
    const float* pen_par;
    const int* bias_tok;
    const float* bias_val;
    const int *bias_off, *bias_n;
    unsigned* err;
};
// launch 1: block (slice, row)
__global__ void __launch_bounds__(SM_THREADS) k_top_slices(const TopArgs a) {
    __shared__ float vals[SM_SLICE];
    __shared__ unsigned long long cand[SM_THREADS / 64][SM_N];
    const int row = blockIdx.y, s = blockIdx.x, tid = threadIdx.x, wave = uniform(tid >> 6);
    const int i0 = s * SM_SLICE, len = min(SM_SLICE, a.n - i0);
    float* L = a.logits + (size_t) row * a.n + i0;
    bool bad = false;
#pragma unroll
    for (int v = 0; v < SM_V; ++v) {
        const int i = v * SM_THREADS + tid;
        const float x = i < len ? L[i] : 0.f;
        bad = bad || !isfinite(x);
        vals[i] = x;
    }
    if (__any(bad) && (tid & 63) == 0) atomicOr(a.err, 16u);
    __syncthreads();
    // the row's logit_bias on this slice's tokens (each token once in a list), before its penalties (topk.cuh:31-37)
    const int nb = a.bias_n ? min(max(a.bias_n[row], 0), SM_PEN_CAP) : 0, np = a.pen_n ? min(max(a.pen_n[row], 0), a.pen_stride) : 0;
    for (int i = tid; i < nb; i += SM_THREADS) {
        const int at = a.bias_off[row] + i, tok = a.bias_tok[at] - a.v0 - i0;
        if (tok >= 0 && tok < len) vals[tok] += a.bias_val[at];
    }
    __syncthreads();
    if (np) {
        const float repeat = a.pen_par[row * 3], freq = a.pen_par[row * 3 + 1], present = a.pen_par[row * 3 + 2];
        for (int i = tid; i < np; i += SM_THREADS) {
            const int tok = a.pen_tok[row * a.pen_stride + i] - a.v0 - i0, cnt = a.pen_cnt[row * a.pen_stride + i];
            if (tok < 0 || tok >= len || cnt <= 0) continue;
            float l = vals[tok];
            l = l <= 0.f ? l * repeat : l / repeat;
            vals[tok] = l - (float) cnt * freq - present;
        }
    }
    __syncthreads();
    // the changed logits go back to the row (the operator changes it in place)
    for (int i = tid; i < nb; i += SM_THREADS) {
        const int tok = a.bias_tok[a.bias_off[row] + i] - a.v0 - i0;
        if (tok >= 0 && tok < len) L[tok] = vals[tok];
    }
    for (int i = tid; i < np; i += SM_THREADS) {
        const int tok = a.pen_tok[row * a.pen_stride + i] - a.v0 - i0;
        if (tok >= 0 && tok < len) L[tok] = vals[tok];
    }
    unsigned key[SM_V], idf[SM_V];
#pragma unroll
    for (int v = 0; v < SM_V; ++v) {
        const int i = v * SM_THREADS + tid;
        key[v] = i < len ? tk_key(vals[i]) : 0u;
        idf[v] = i < len ? 0xffffffffu - (unsigned) (i0 + i) : 0u;
    }
    wave_emit64<SM_V>(key, idf, wave_select64<SM_V>(key, idf), cand[wave]);
    __syncthreads();
    if (wave != 0) return;
    constexpr int W = SM_THREADS / 64;
    unsigned k2[W], f2[W];
#pragma unroll
    for (int j = 0; j < W; ++j) {
        const unsigned long long c = cand[j][tid];
        k2[j] = (unsigned) (c >> 32);
        f2[j] = (unsigned) c;
    }
    wave_emit64<W>(k2, f2, wave_select64<W>(k2, f2), g_topk_cand + ((size_t) row * a.nslice + s) * SM_N);
}
// launch 2: a block per row: the 64 best of its slices' candidates, sorted
__global__ void __launch_bounds__(SM_MERGE_THREADS) k_top_merge(const float* __restrict__ logits, int n, int v0, int nslice, float* __restrict__ out_v,
                                                               int* __restrict__ out_i) {
    __shared__ unsigned long long cand[SM_MERGE_THREADS / 64][SM_N];
    const int row = blockIdx.x, tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63;
    const unsigned long long* C = g_topk_cand + (size_t) row * nslice * SM_N;
    const int total = nslice * SM_N;
    {
        unsigned key[SM_MERGE_V], idf[SM_MERGE_V];
#pragma unroll
        for (int v = 0; v < SM_MERGE_V; ++v) {
            const int i = v * SM_MERGE_THREADS + tid;
            const unsigned long long c = i < total ? C[i] : 0ull;
            key[v] = (unsigned) (c >> 32);
            idf[v] = (unsigned) c;
        }
        wave_emit64<SM_MERGE_V>(key, idf, wave_select64<SM_MERGE_V>(key, idf), cand[wave]);
    }
    __syncthreads();
    if (wave != 0) return;
    constexpr int W = SM_MERGE_THREADS / 64;
    __shared__ unsigned long long best[SM_N];
    {
        unsigned key[W], idf[W];
#pragma unroll
        for (int j = 0; j < W; ++j) {
            const unsigned long long c = cand[j][lane];
            key[j] = (unsigned) (c >> 32);
            idf[j] = (unsigned) c;
        }
        wave_emit64<W>(key, idf, wave_select64<W>(key, idf), best);
    }
    // one pair a lane, sorted descending across the lanes (a bitonic network of exchanges between lanes)
    unsigned long long c = best[lane];
#pragma unroll
    for (int size = 2; size <= 64; size <<= 1)
#pragma unroll
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            const unsigned lo = (unsigned) __shfl_xor((int) (unsigned) c, stride, 64), hi = (unsigned) __shfl_xor((int) (unsigned) (c >> 32), stride, 64);
            const unsigned long long o = (unsigned long long) hi << 32 | lo;
            const bool upper = lane & stride, desc = (lane & size) == 0;   // the lower lane of a pair keeps the greater where the run descends
            const bool take_max = desc != upper;
            c = take_max ? (c > o ? c : o) : (c < o ? c : o);
        }
    const int j = (int) (0xffffffffu - (unsigned) c);
    out_i[row * SM_N + lane] = v0 + j;
    out_v[row * SM_N + lane] = logits[(size_t) row * n + j];
}

// penalize_row (kernels.hpp:434-436): pen = {k, k indexes into the row, their k counts}, par = {repeat, freq, present}
__global__ void k_penalize_row(float* __restrict__ L, int n, const int* __restrict__ pen, const float* __restrict__ par) {
    const int k = min(max(pen[0], 0), SM_PEN_CAP);   // a count past the cap is not a list: never walk off the buffer on its word
    const float repeat = par[0], freq = par[1], present = par[2];
    for (int i = threadIdx.x; i < k; i += blockDim.x) {
        const int j = pen[1 + i], cnt = pen[1 + k + i];
        if (j < 0 || j >= n || cnt <= 0) continue;
        float l = L[j];
        l = l <= 0.f ? l * repeat : l / repeat;
        L[j] = l - (float) cnt * freq - present;
    }
}

}  // namespace fnx
