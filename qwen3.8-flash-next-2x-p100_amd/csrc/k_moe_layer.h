// The MoE half of a verify window (the work of Engine::ffn_half, engine.cu:1569-1757 of the reference, on one GPU) in
// three launches: [router logits | q8_1 rows of x] -> [top-k, jobs and plan, gate|up of the routed and the shared expert,
// SwiGLU to q8_1] -> [down of the routed and the shared expert with the combine's chains].
//
// Arithmetic is the operators': the router sums in the fixed 64-lane order, top-k by (value, lower index), the q8_1
// rounding, the IQ3_S sub-block terms, the combine's fmaf chain. Only the order in which a row's 64 (or 16) lane
// sums are added differs from the one-operator-per-launch path.
//
// (A single persistent kernel with grid barriers between these phases was measured and dropped: on MI355X a barrier
// of 512 blocks costs ~8.5 us in device-scope atomics alone and ~31 us with the release/acquire cache maintenance the
// exchange of results between XCDs needs, against ~4 us for a kernel boundary.)
#pragma once

#include "k_iq3s_packed.h"

namespace fnx {

constexpr int FL_THREADS = 512, FL_WAVES = FL_THREADS / 64;
constexpr int FL_MAXP = FNX_MAXT * 10;    // routed pairs of a window (T * topk), at most
constexpr int FL_MAXJ = FL_MAXP + 1;      // their jobs, and the shared expert's
constexpr int FL_N = 2048;                // hidden size these kernels are built for (gate|up rows of 64 sub-blocks)

// wave-wide max / min with DPP moves; every lane gets the result
__device__ __forceinline__ float wave_max(float v) {
#define FNX_DPP_MAX(ctrl, rmask) v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), ctrl, rmask, 0xF, false)))
    FNX_DPP_MAX(0xB1, 0xF);
    FNX_DPP_MAX(0x4E, 0xF);
    FNX_DPP_MAX(0x141, 0xF);
    FNX_DPP_MAX(0x140, 0xF);
    FNX_DPP_MAX(0x142, 0xA);
    FNX_DPP_MAX(0x143, 0xC);
#undef FNX_DPP_MAX
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
// Ranking by unsigned keys: key(v) rises with v (kernels.cu:1045-1083 uses the same key for its argmax), -0 counts as +0 as
// in a float comparison, a NaN gets key 0 and so is never taken; a value can be picked if its key is above -inf's.
__device__ __forceinline__ unsigned rank_key(float v) {
    const unsigned u = __float_as_uint(v + 0.0f);
    return v != v ? 0u : (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float rank_key_inv(unsigned k) { return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k); }
constexpr unsigned RANK_KEY_NEG_INF = 0x007FFFFFu;
// every lane: the greatest key of its row of 16 lanes (one instruction a step; the s_nop cover the wait states between a
// vector write and a DPP read of the same register, which the compiler cannot see inside the asm)
__device__ __forceinline__ unsigned row_umax(unsigned v) {
    asm volatile(
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(v));
    return v;
}
__device__ __forceinline__ unsigned wave_umax(unsigned v) {   // the wave's greatest key, in a scalar register
    const int r = (int) row_umax(v);
    const unsigned a = (unsigned) __builtin_amdgcn_readlane(r, 0), b = (unsigned) __builtin_amdgcn_readlane(r, 16);
    const unsigned c = (unsigned) __builtin_amdgcn_readlane(r, 32), d = (unsigned) __builtin_amdgcn_readlane(r, 48);
    return max(max(a, b), max(c, d));
}
__device__ __forceinline__ int wave_min(int v) {
#define FNX_DPP_MIN(ctrl, rmask) v = min(v, __builtin_amdgcn_update_dpp(v, v, ctrl, rmask, 0xF, false))
    FNX_DPP_MIN(0xB1, 0xF);
    FNX_DPP_MIN(0x4E, 0xF);
    FNX_DPP_MIN(0x141, 0xF);
    FNX_DPP_MIN(0x140, 0xF);
    FNX_DPP_MIN(0x142, 0xA);
    FNX_DPP_MIN(0x143, 0xC);
#undef FNX_DPP_MIN
    return __builtin_amdgcn_readlane(v, 63);
}

// one token's top-k: the lanes hold its logits (lane l: experts l, l + 64, ...). Picks into ex[0..topk), topi, topw.
// moe.cuh:382-411: greater value first, the lower index on a tie; w_k = exp(l_k - l_0) / sum in pick order.
// publish: also write topi and topw (else only ex)
template <int NE>
__device__ __forceinline__ void wave_topk(const float* __restrict__ row, int nexp, int topk, int lane, int* __restrict__ ex,
                                          int* __restrict__ topi, float* __restrict__ topw, bool publish = true) {
    float v[NE];
#pragma unroll
    for (int i = 0; i < NE; ++i) {
        const int e = lane + 64 * i;
        v[i] = e < nexp ? row[e] : -INFINITY;
    }
    float top0 = 0.f, z = 0.f, wk = 0.f;
    unsigned taken = 0;   // bit i: this lane's entry i has been picked
    for (int k = 0; k < topk; ++k) {
        // the lane's greatest value still to be picked (a picked one becomes -inf) and the lowest of its indexes that hold
        // it, as a tree of maxima and a mask of equalities rather than a chain over the NE values. A NaN is never the
        // maximum and never equal; a lane with nothing left (-inf) offers index nexp.
        float bv = v[0];
#pragma unroll
        for (int i = 1; i + 1 < NE; i += 2) bv = fmaxf(bv, fmaxf(v[i], v[i + 1]));
        bv = fmaxf(bv, v[NE - 1]);
        unsigned eq = 0;
#pragma unroll
        for (int i = 0; i < NE; ++i) eq |= (v[i] == bv ? 1u : 0u) << i;
        const int bi = bv > -INFINITY && eq ? lane + 64 * (int) __builtin_ctz(eq) : nexp;
        const float m = wave_max(bv);
        // the lowest index among the lanes that hold the maximum: nearly always one lane, found by a ballot
        const unsigned long long holders = __ballot(bv == m);
        int mi;
        if (__popcll(holders) == 1) mi = __builtin_amdgcn_readlane(bi, (int) __builtin_ctzll(holders));
        else mi = wave_min(bv == m ? bi : 0x7fffffff);
        bool found = mi < nexp;
        if (!found) {   // nothing above -inf is left (masked or NaN logits): the lowest index not yet picked, at weight 0
            unsigned left = 0;
#pragma unroll
            for (int i = 0; i < NE; ++i) left |= (lane + 64 * i < nexp && !((taken >> i) & 1u) ? 1u : 0u) << i;
            mi = wave_min(left ? lane + 64 * (int) __builtin_ctz(left) : 0x7fffffff);
        }
        const bool mine = mi < nexp && (mi & 63) == lane;
#pragma unroll
        for (int i = 0; i < NE; ++i)
            if (mine && (mi >> 6) == i) v[i] = -INFINITY;
        if (mine) taken |= 1u << (mi >> 6);
        if (k == 0) top0 = m;
        const float ek = found ? expf(m - top0) : 0.f;
        z += ek;
        if (lane == k) {
            wk = ek;
            const int pick = mi < nexp ? mi : nexp - 1;   // more picks than experts: refused by the host, kept inside the tables here
            ex[k] = pick;
            if (publish) topi[k] = pick;
        }
    }
    if (publish && lane < topk) topw[lane] = z > 0.f ? wk / z : 0.f;
}

// ---------------------------------------------------------------- the job lists of a window's picks
// The reference's window hands its caller the jobs as lists (kernels.hpp:18-23, 277-282); this window's own launches do
// not read them (they walk a row's picks directly), so a spare block of the last launch writes them, off the critical
// path. They follow from all rows' picks without any serial loop: a token picks an expert at most once, so a pair's
// slot in its job is the number of earlier tokens in the expert's token mask, and a job's number is the rank of its first
// pair among the first pairs (the order k_router_route's last block gives them, moe.cuh:324-330).
struct RouteArgs {
    int nexp, topk, T;
    const float* logits;
    int* topi;
    float* topw;
    fnx_job* jobs_gu;
    fnx_job* jobs_dn;
    int* njobs;   // [0] the job count
    const int* live;   // may be null; else a device word: only the window's first *live rows are routed (the others get no
                       // pairs, and the shared expert's job stops before them), while the lists keep the indexes T gives them
};
template <int NT>
struct RouteLds {
    unsigned mask[1024];      // per expert: the window rows that picked it
    int first[1024];          // per expert: its first pair
    int jobof[1024];
    int wcnt[NT / 64];
};
// All NT threads of a block. Tl: the rows that count.
template <int NT>
__device__ __forceinline__ void write_job_lists(RouteLds<NT>& L, const RouteArgs& a, int Tl) {
    static_assert(FL_MAXP <= NT, "a thread per pair");
    const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63;
    const int T = a.T, topk = a.topk, P = T * topk, Pl = Tl * topk;
    // the picks were written by other blocks of this launch: read at the device's level, past this XCD's L2
    const int e_mine = tid < Pl ? __hip_atomic_load(&a.topi[tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
    for (int e = tid; e < a.nexp; e += NT) {
        L.mask[e] = 0u;
        L.first[e] = P;
    }
    __syncthreads();
    if (tid < Pl) {
        atomicOr(&L.mask[e_mine], 1u << (tid / topk));
        atomicMin(&L.first[e_mine], tid);
    }
    __syncthreads();
    // job numbers: the rank of an expert's first pair among all first pairs (ballots over the pairs in order)
    const bool isfirst = tid < Pl && L.first[e_mine] == tid;
    const unsigned long long b = __ballot(isfirst);
    if (lane == 0) L.wcnt[wave] = __popcll(b);
    __syncthreads();
    int before = 0, nj = 0;
    for (int w = 0; w < NT / 64; ++w) {
        before += w < wave ? L.wcnt[w] : 0;
        nj += L.wcnt[w];
    }
    if (isfirst) {
        const int j = before + __popcll(b & ((1ull << lane) - 1ull)), cnt = __popc(L.mask[e_mine]);
        L.jobof[e_mine] = j;
        a.jobs_gu[j].w = a.jobs_dn[j].w = e_mine;
        a.jobs_gu[j].n = a.jobs_dn[j].n = cnt;
    }
    if (tid == 0) a.njobs[0] = nj;
    __syncthreads();
    // a pair's slot in its job: the earlier rows in its expert's mask (pairs of a job ascend with the row)
    if (tid < Pl) {
        const int j = L.jobof[e_mine], row = tid / topk, slot = __popc(L.mask[e_mine] & ((1u << row) - 1u));
        a.jobs_gu[j].y[slot] = row;
        a.jobs_gu[j].out[slot] = tid;
        a.jobs_dn[j].y[slot] = tid;
        a.jobs_dn[j].out[slot] = tid;
    }
    if (tid < max(Tl, 1)) {   // the shared expert's job, at index P of the lists (kernels.hpp:277-282)
        a.jobs_gu[P].y[tid] = tid;
        a.jobs_gu[P].out[tid] = P + tid;
        a.jobs_dn[P].y[tid] = P + tid;
        a.jobs_dn[P].out[tid] = P + tid;
        if (tid == 0) {
            a.jobs_gu[P].w = a.jobs_dn[P].w = 0;
            a.jobs_gu[P].n = a.jobs_dn[P].n = Tl;
        }
    }
}

// ---------------------------------------------------------------- launch 1: router logits | q8_1 rows of x
// Blocks [0, rblocks): a wave per router row with the row in registers; the window's x comes through LDS in two halves
// of 1024 columns, the second half's loads in flight while the first is used: about one memory round trip in all.
// Sums in the fixed order of k_gemv_rows (and of the CPU oracle): lane l takes float4 chunks l, l + 64, ... in order,
// fmaf over x, y, z, w; then the xor-butterfly. Blocks after them: 16 q8_1 blocks of x each.
struct RouterArgs {
    int nexp, T;
    const float* x;
    const void* router;
    int router_bf16;
    float* logits;
    uint8_t* xq;
    const int* live;   // may be null; else a device word: with no row routed the launch leaves at once
};
constexpr int RQ_ROWS = 4;   // router rows per block: two waves per row, each with half of the window's rows
__global__ void __launch_bounds__(FL_THREADS) k_router_quant(const RouterArgs a) {
    __shared__ float4 xt[FNX_MAXT][4][64];   // [token][chunk][lane]: half of x
    if (a.live && uniform(*a.live) <= 0) return;
    const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63;
    const int T = a.T, n = FL_N, LS = a.nexp + 1;
    const int rblocks = (LS + RQ_ROWS - 1) / RQ_ROWS, b = blockIdx.x;
    if (b >= rblocks) {
        const int qb = (b - rblocks) * 2 * FL_WAVES + wave * 2 + (lane >> 5);
        if (qb < T * 64) {
            const int t = qb >> 6, blk = qb & 63;
            const float xi = a.x[(size_t) t * n + blk * 32 + (lane & 31)];
            q8_1_store(xi, a.xq + (size_t) qb * FNX_Q8_1_BLOCK, lane & 31);
        }
        return;
    }
    const int row = b * RQ_ROWS + (wave >> 1), tb = (wave & 1) * (FNX_MAXT / 2);   // this wave: tokens tb .. tb + 7
    const bool live = row < LS;
    float4 w[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        if (!live) w[c] = make_float4(0.f, 0.f, 0.f, 0.f);
        else if (a.router_bf16) {
            const uint2 u = reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(a.router) + (size_t) row * n)[c * 64 + lane];
            w[c] = make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                               __uint_as_float(u.y & 0xffff0000u));
        } else w[c] = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(a.router) + (size_t) row * n)[c * 64 + lane];
    }
    auto load_half = [&](int h, float4(&xr)[8]) {   // item i = tid + 512 k of [token][chunk][lane]
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int i = tid + k * FL_THREADS, t = i >> 8, c = (i >> 6) & 3, l = i & 63;
            xr[k] = t < T ? reinterpret_cast<const float4*>(a.x + (size_t) t * n)[(4 * h + c) * 64 + l] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    float acc[FNX_MAXT / 2];
#pragma unroll
    for (int t = 0; t < FNX_MAXT / 2; ++t) acc[t] = 0.f;
    float4 xr[8];
    load_half(0, xr);
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int i = tid + k * FL_THREADS;
            xt[i >> 8][(i >> 6) & 3][i & 63] = xr[k];
        }
        __syncthreads();
        if (h == 0) load_half(1, xr);
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int t = 0; t < FNX_MAXT / 2; ++t)
                if (tb + t < T) {
                    const float4 bx = xt[tb + t][c][lane];
                    const float4 wc = w[4 * h + c];
                    float s = acc[t];
                    s = fmaf(wc.x, bx.x, s);
                    s = fmaf(wc.y, bx.y, s);
                    s = fmaf(wc.z, bx.z, s);
                    s = fmaf(wc.w, bx.w, s);
                    acc[t] = s;
                }
        __syncthreads();
    }
    // The wave's eight sums over the 64 lanes at once: at the butterfly's levels 32, 16 and 8 a lane keeps the half of
    // its values whose index bit equals its lane bit and adds its partner's copy of them (the pairwise adds group_sum<64>
    // makes for each value, so the same bits), then levels 4, 2, 1 on the one value left: 10 exchanges instead of 48.
    // Lanes 8 j .. 8 j + 7 end with token tb + j's sum.
    static_assert(FNX_MAXT / 2 == 8, "eight sums a wave");
    float v4[4], v2[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) v4[i] = swap32_add(acc[i], acc[i + 4]);
#pragma unroll
    for (int i = 0; i < 2; ++i) v2[i] = swap16_add(v4[i], v4[i + 2]);
    const bool up = lane & 8;
    float v = (up ? v2[1] : v2[0]) + __shfl_xor(up ? v2[0] : v2[1], 8, WAVE);
    v += __shfl_xor(v, 4, WAVE);
    v += __shfl_xor(v, 2, WAVE);
    v += __shfl_xor(v, 1, WAVE);
    const int t = tb + (lane >> 3);
    if (live && (lane & 7) == 0 && t < T) a.logits[(size_t) t * LS + row] = v;
}

// ---------------------------------------------------------------- launch 2: top-k, gate|up, h in q8_1 form
// An item = (pair, block of 32 h values): the 32 gate rows and the 32 up rows that one q8_1 block of
// h = silu(gate) * up needs (k_moe_h, moe.cuh:597-608), 64 units of the pair's expert. A thread block of 16 waves takes
// one item a sweep, four units a wave: gate rows 2 i, 2 i + 1 and up rows 2 i, 2 i + 1, whose four sums give two h values.
// The items are numbered (row, block of 32, pick) and dealt to the blocks of the grid in runs: with a full window of 16
// rows and 256 blocks a thread block has one row's one block of 32 for the shared expert and then all the row's picks
// (the shared expert's matrix is known before the picks are: its loads are in flight while the row is ranked). So
// it needs the picks of one row only (two when a run crosses rows): it ranks that row itself, a wave a row, while its
// codebook loads are in flight - no launch of its own for the top-k (a kernel boundary on the window's critical path),
// no list of jobs, no plan - and its lanes keep their activations for the whole launch. An expert that several rows
// picked is decoded once per row (the later reads come from the caches); in exchange every sweep of every block is the
// same work, and at any time the grid reads one expert a row, each as one front moving through the matrix, which HBM
// serves better than a range of its own per wave (25 against 29 us for a plain read of a window's gate|up bytes).
// The sixteen waves' values of an item meet in LDS without a barrier: a wave writes its two values and its flag and goes
// on; two sweeps later the wave whose turn it is makes the q8_1 block of that sweep and writes it out (by then the
// others have long arrived; it waits if not).
// hq rows as the down launch reads them: per pair and block of 32: 8 words of int8 values, the scale as a float, 3 unused.
constexpr int GH_THREADS = 1024, GH_WAVES = GH_THREADS / 64, HQ_WORDS = 12, GH_SLOTS = 4, GH_LAG = 2;
constexpr int FL_MAXK = 16;   // picks a row that the window's launches take
struct GateUpArgs {
    int ff;                   // expert width: the matrices have 2 ff rows (gate rows, then up rows) of FL_N columns
    const uint8_t* w;         // routed experts: expert e at w + e * stride, or ep[e]
    size_t stride;
    const uint8_t* const* ep;
    const uint8_t* w_shared;
    const uint8_t* xq;        // the window's q8_1 rows
    uint32_t* hq;             // [pair][ff / 32][HQ_WORDS]
    RouteArgs route;          // logits in; picks and weights out (the block that has a row's first item writes them)
};
struct GhLds {
    uint32_t tab[SGRID_WORDS];
    uint32_t wp[2][FL_MAXK + 1][2];   // the matrices of the block's (at most two) rows: the shared expert's, then the picks'
    float hg[GH_SLOTS][32], hu[GH_SLOTS][32];   // [slot][row of the block of 32]: the gate sums, the up sums
    int flag[GH_SLOTS][GH_WAVES];     // sweep + 1 of the values a wave last wrote into the slot
    int made[GH_SLOTS];               // sweeps whose block has been made from the slot: a writer of sweep s waits for made >= s - GH_SLOTS + 1
    uint2 cand[2][16][FL_MAXK];       // the rows' candidates: per slice of 64 experts its greatest (value, expert) in order
    int sliced[2 * 16];               // set once a slice's candidates are written
    int ready[2];                     // how many of a row's picks' matrices are known
};
struct GhItem {   // (row, block of 32, matrix: 0 the shared expert's, k pick k - 1's) of an item number, kept by stepping
    int t, j, k;
};
__global__ void __launch_bounds__(GH_THREADS) k_moe_gate_up_h(const GateUpArgs a) {
    __shared__ GhLds S;
    const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63;
    // The codebook's 512 unsigned entries, the launch's first load (the barrier below waits for nothing else). Every thread
    // of the grid wants them as the launch starts: read from one place, those 2 KiB - sixteen cache lines - kept the blocks
    // waiting for 2 to 3 us. The table in memory holds all sixteen signed forms, 2 KiB apart, and a signed form negated
    // again is the unsigned one: the half-blocks read different forms.
    const int form = (2 * (int) blockIdx.x + (tid >> 9)) & 15;
    const uint32_t tab0 = signed_entry(g_sgrid.v[(form << 9) + (tid & 511)], form);
    // k0: a row's first matrix - 0, the shared expert, or 1 when that one is not this launch's (w_shared null: run elsewhere)
    const int T = a.route.T, topk = a.route.topk, nexp = a.route.nexp, P = T * topk, qpp = a.ff >> 5, k0 = a.w_shared ? 0 : 1;
    const int nk = topk + 1 - k0, per_row = qpp * nk;
    const int Tl = a.route.live ? uniform(max(0, min(*a.route.live, T))) : T;
    // Quotients of small numbers (below 2^14, the divisor a few hundred at most) by a multiplication: with the divisor's
    // reciprocal rounded once and the dividend moved half a step up, the product misses the exact quotient by less than
    // the distance to the next integer. (Every wave of every block works these out: as integer divisions they were half
    // of what a wave executes before the barrier.)
    const float r_nb = 1.0f / (float) gridDim.x, r_row = 1.0f / (float) per_row, r_k1 = 1.0f / (float) nk;
    auto quot = [](int x, float r) { return (int) (((float) x + 0.5f) * r); };
    // this block's run of items
    const int total = Tl * per_row, nb = gridDim.x, ipb = quot(total + nb - 1, r_nb);
    const int I0 = (int) blockIdx.x * ipb, I1 = min(total, I0 + ipb), nsweep = I1 - I0;
    if (nsweep <= 0) return;
    const int t0 = quot(I0, r_row), t1 = quot(I1 - 1, r_row);   // ipb <= per_row (the launcher sees to it): two rows at most
    const int nr = t1 - t0 + 1, ns = (nexp + 63) >> 6;           // rows of the run, slices of 64 experts a row
    // this wave's first slice of logits: asked for now, ranked once the codebook is in LDS
    float v0 = -INFINITY;
    if (wave < nr * ns) {
        const int r = wave / ns, e = 64 * (wave - r * ns) + lane;
        if (e < nexp) v0 = a.route.logits[(size_t) (t0 + r) * (nexp + 1) + e];
    }
    auto load_x = [&](int t, int (&xs)[8], float& dx) {   // the lane's sub-block of row t's activations: 36 bytes in three loads
        typedef unsigned u4a __attribute__((ext_vector_type(4), aligned(4)));
        const uint8_t* yb = a.xq + ((size_t) t * 64 + lane) * FNX_Q8_1_BLOCK;
        const uint32_t head = *reinterpret_cast<const uint32_t*>(yb);
        const u4a lo = *reinterpret_cast<const u4a*>(yb + 4), hi = *reinterpret_cast<const u4a*>(yb + 20);
        dx = half_bits_to_float(head & 0xFFFFu);
        xs[0] = (int) lo.x, xs[1] = (int) lo.y, xs[2] = (int) lo.z, xs[3] = (int) lo.w;
        xs[4] = (int) hi.x, xs[5] = (int) hi.y, xs[6] = (int) hi.z, xs[7] = (int) hi.w;
    };
    int xs[8], tx = t0;
    float dx;
    load_x(t0, xs, dx);
    const PackedVOffs o = packed_voffs(lane);
    // byte offsets of the wave's gate units and up units from its item's first gate unit
    const int uo_g = wave * 2 * UNIT_BYTES, uo_u = uo_g + a.ff * UNIT_BYTES;
    auto item_of = [&](int I) {
        GhItem m;
        m.t = quot(I, r_row);
        const int r = I - m.t * per_row;
        m.j = quot(r, r_k1);
        m.k = k0 + r - m.j * nk;
        return m;
    };
    auto step = [&](GhItem& m) {
        if (++m.k > topk) {
            m.k = k0;
            if (++m.j == qpp) {
                m.j = 0;
                ++m.t;
            }
        }
    };
    PackedSub A[4];
    auto issue_from = [&](const uint8_t* e, int j) {   // e: wave-uniform
        const __amdgpu_buffer_rsrc_t mtx = matrix_rsrc(e);
        const int ub = j * 32 * UNIT_BYTES;
        A[0] = load_packed_buf(mtx, ub + uo_g, o);
        A[1] = load_packed_buf(mtx, ub + uo_g + UNIT_BYTES, o);
        A[2] = load_packed_buf(mtx, ub + uo_u, o);
        A[3] = load_packed_buf(mtx, ub + uo_u + UNIT_BYTES, o);
    };
    GhItem ma = item_of(I0);
    const bool early = ma.k == 0;   // the run starts with a shared expert's item: no pick needed to ask for it
    if (tid < GH_SLOTS * GH_WAVES) (&S.flag[0][0])[tid] = 0;
    if (tid < GH_SLOTS) S.made[tid] = 0;
    if (tid < 32) S.sliced[tid] = 0;
    if (tid < 2) S.ready[tid] = 0;
    // the codebook: two threads a code, eight signed forms each
#pragma unroll
    for (int i = 0; i < 8; ++i) S.tab[tid + i * GH_THREADS] = signed_entry(tab0, (tid >> 9) + 2 * i);
    __syncthreads();
    if (early) issue_from(a.w_shared, ma.j);   // (asked for ahead of the barrier, these twenty loads a wave held the waves up on their way to it)
    // The rows' picks (moe.cuh:382-411: greater value first, the lower index on a tie; w_k = exp(l_k - l_0) / sum in pick
    // order), without another barrier. Every wave lists the topk greatest of a slice of 64 experts, in order (a wave-wide
    // maximum a round); a wave a row then merges the slices' lists by their heads while the other waves decode the shared
    // expert's item, and says when the row's matrices are known. (One wave ranking a whole row, eight values a lane, took
    // 4.5 us, with every other wave of the block waiting for it.)
    if (wave < nr * ns) __builtin_amdgcn_s_setprio(2);
    for (int task = wave; task < nr * ns; task += GH_WAVES) {
        const int r = task / ns, sl = task - r * ns;
        float v = v0;
        if (task != wave) {
            const int e = 64 * sl + lane;
            v = e < nexp ? a.route.logits[(size_t) (t0 + r) * (nexp + 1) + e] : -INFINITY;
        }
        unsigned key = rank_key(v);
        for (int k = 0; k < topk; ++k) {
            const unsigned m = wave_umax(key);
            const unsigned long long hold = m > RANK_KEY_NEG_INF ? __ballot(key == m) : 0ull;
            const int l = hold ? (int) __builtin_ctzll(hold) : 64;   // the lowest lane that holds the maximum is the lowest expert
            key = lane == l ? 0u : key;
            if (lane == 0) S.cand[r][sl][k] = make_uint2(hold ? m : 0u, (uint32_t) (hold ? 64 * sl + l : nexp));
        }
        if (lane == 0) __hip_atomic_store(&S.sliced[task], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    __builtin_amdgcn_s_setprio(0);
    if (wave < nr) {   // the merge; the row's first item's block writes the picks and their weights out
        const int t = t0 + wave;
        const bool publish = t * per_row >= I0;
        __builtin_amdgcn_s_setprio(3);   // the other waves of the block will soon wait for this one
        while (true) {
            const int f = lane < ns ? __hip_atomic_load(&S.sliced[wave * ns + lane], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) : 1;
            if (__ballot(f == 0) == 0ull) break;
            __builtin_amdgcn_s_sleep(1);
        }
        // All of the row's candidates in registers, entry p of list j in lane (16 j + p) mod 64 of register (16 j + p) / 64
        // (the LDS is busy with the other waves' codebook reads: a read a round of a list's next entry took longer than the
        // rest of the round). Lane j < ns keeps list j's head and its position; the list whose head is picked gets its next
        // entry by a read of that lane.
        static_assert(FL_MAXK == 16, "sixteen entries a list, four lists a register");
        int ck[4], ce[4];
        {
            const uint2* flat = &S.cand[wave][0][0];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint2 c = flat[q * 64 + lane];
                ck[q] = (int) c.x;
                ce[q] = (int) c.y;
            }
        }
        unsigned hk = lane < ns ? S.cand[wave][min(lane, ns - 1)][0].x : 0u;
        int he = S.cand[wave][min(lane, ns - 1)][0].y, hp = 0;
        unsigned mk = 0u;
        int ei = 0x7fffffff;
        unsigned long long low_taken = 0ull;   // which of experts 0 .. 63 are picked: what a row with fewer than topk finite logits falls back on
        for (int k = 0; k < topk; ++k) {
            unsigned m = (unsigned) __builtin_amdgcn_readlane((int) row_umax(hk), 0);
            const unsigned long long hold = m > RANK_KEY_NEG_INF ? __ballot(hk == m) & 0xFFFFull : 0ull;
            const int l = hold ? (int) __builtin_ctzll(hold) : 64;   // the lowest lane that holds the maximum has the lowest expert
            int idx;
            unsigned nk = 0u;
            int ne = nexp, np = 0;
            if (hold) {
                idx = __builtin_amdgcn_readlane(he, l);
                np = __builtin_amdgcn_readlane(hp, l) + 1;
                if (np < topk) {   // list l's next entry
                    const int f = 16 * l + np, fl = f & 63, fq = f >> 6;
                    const int k0 = __builtin_amdgcn_readlane(ck[0], fl), k1 = __builtin_amdgcn_readlane(ck[1], fl);
                    const int k2 = __builtin_amdgcn_readlane(ck[2], fl), k3 = __builtin_amdgcn_readlane(ck[3], fl);
                    const int e0 = __builtin_amdgcn_readlane(ce[0], fl), e1 = __builtin_amdgcn_readlane(ce[1], fl);
                    const int e2 = __builtin_amdgcn_readlane(ce[2], fl), e3 = __builtin_amdgcn_readlane(ce[3], fl);
                    nk = (unsigned) (fq == 0 ? k0 : fq == 1 ? k1 : fq == 2 ? k2 : k3);
                    ne = fq == 0 ? e0 : fq == 1 ? e1 : fq == 2 ? e2 : e3;
                }
            } else {   // nothing finite is left: the lowest expert not picked yet, with weight exp(-inf) = 0
                m = RANK_KEY_NEG_INF;
                idx = (int) __builtin_ctzll(~low_taken);
            }
            if (idx < 64) low_taken |= 1ull << idx;
            if (lane == l) {
                hk = nk;
                he = ne;
                hp = np;
            }
            if (lane == k) {
                mk = m;
                ei = idx;
            }
            {   // the pick's matrix is handed out at once: the sweeps need not wait for the whole ranking
                const uint8_t* e = a.ep ? a.ep[idx] : a.w + (size_t) idx * a.stride;
                if (lane == 0) {
                    S.wp[wave][1 + k][0] = (uint32_t) (uintptr_t) e;
                    S.wp[wave][1 + k][1] = (uint32_t) ((uint64_t) (uintptr_t) e >> 32);
                    __hip_atomic_store(&S.ready[wave], k + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            }
        }
        const float top0 = rank_key_inv((unsigned) __builtin_amdgcn_readlane((int) mk, 0));
        const float ek = expf(rank_key_inv(mk) - top0);
        float z = 0.f;
        for (int k = 0; k < topk; ++k) z += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ek), k));
        if (publish && lane < topk) {
            a.route.topi[t * topk + lane] = ei;
            a.route.topw[t * topk + lane] = ek / z;
        }
        __builtin_amdgcn_s_setprio(0);
    }
    // an item's loads, once its matrix is known: matrix 0 is the shared expert's, matrix k pick k - 1's, known as soon as
    // the merge has found it. (Walking the picks by ascending expert instead, so that rows which share an expert reach it
    // together and the later read hits the L2 of their common XCD, cut the fabric's traffic by 5% - 127 against 134 MB -
    // and gained nothing: it needs the whole ranking before the first pick's sweep.)
    auto issue = [&](const GhItem& m) {
        const uint8_t* e = a.w_shared;
        if (m.k > 0) {
            const int r = m.t - t0;
            while (uniform(__hip_atomic_load(&S.ready[r], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP)) < m.k) __builtin_amdgcn_s_sleep(1);
            const uint2 p = *reinterpret_cast<const uint2*>(S.wp[r][m.k]);
            e = (const uint8_t*) (uintptr_t) ((uint64_t) (uint32_t) uniform((int) p.x) | (uint64_t) (uint32_t) uniform((int) p.y) << 32);
        }
        issue_from(e, m.j);
    };
    const int sc_shift = 4 * (lane & 1);
    // the q8_1 block of sweep q, by the first half of the wave (k_moe_h, moe.cuh:597-608)
    auto make_block = [&](int q) {
        const int slot = q & (GH_SLOTS - 1);
        while (true) {   // all sixteen waves' values of sweep q must be there
            const int f = lane < GH_WAVES ? __hip_atomic_load(&S.flag[slot][lane], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) : q + 1;
            if (__ballot(f < q + 1) == 0ull) break;
            __builtin_amdgcn_s_sleep(2);
        }
        const GhItem m = item_of(I0 + q);
        const int pair = m.k > 0 ? m.t * topk + m.k - 1 : P + m.t;
        if (lane < 32) {
            const float h = silu_f(S.hg[slot][lane]) * S.hu[slot][lane];
            const float amax = group_max<32>(fabsf(h));
            const float d = amax / 127.0f;
            const uint32_t qv = amax == 0.0f ? 0u : (uint32_t) (uint8_t) (int8_t) roundf(h / d);
            uint32_t word = qv | (uint32_t) __shfl_down((int) qv, 1, WAVE) << 8;
            word |= (uint32_t) __shfl_down((int) word, 2, WAVE) << 16;
            uint32_t* dst = a.hq + ((size_t) pair * qpp + m.j) * HQ_WORDS;
            if ((lane & 3) == 0) dst[lane >> 2] = word;
            if (lane == 0) dst[8] = __float_as_uint(half_bits_to_float(float_to_half_bits(d)));
        }
        if (lane == 0) __hip_atomic_store(&S.made[slot], q + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    // where a lane's sum goes after reduce4_units: the 16-lane rows hold gate 2 i, up 2 i, gate 2 i + 1, up 2 i + 1
    float* const zdst0 = (lane & 16 ? &S.hu[0][0] : &S.hg[0][0]) + 2 * wave + (lane >> 5);
    auto decode = [&](const GhItem& m, int sw) {
        if (m.t != tx) {   // the run has crossed into its second row
            tx = m.t;
            load_x(tx, xs, dx);
        }
        const int slot = sw & (GH_SLOTS - 1);
        // the slot's last block (of sweep sw - GH_SLOTS) must have been made: nearly always long ago (asked here, used below)
        int made = sw >= GH_SLOTS ? __hip_atomic_load(&S.made[slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) : 0;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            int w4[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) w4[j] = *reinterpret_cast<const int*>(reinterpret_cast<const uint8_t*>(S.tab) + packed_addr(A[r].idx, j));
            const int sc = 1 + 2 * (int) ((A[r].sc >> sc_shift) & 0xFu);
            const float dw = half_bits_to_float(A[r].d);
            int sum = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) sum = __builtin_amdgcn_sdot4(w4[j], xs[j], sum, false);
            // one sub-block's term as the reference forms it: (d_w * d_x) * (float) (sumi * (1 + 2 s))
            v[r] = (dw * dx) * (float) __mul24(sum, sc);
        }
        // units: gate 2 i, gate 2 i + 1, up 2 i, up 2 i + 1
        const float z = reduce4_units(v[0], v[1], v[2], v[3]);
        if (sw >= GH_SLOTS)
            while (uniform(made) < sw - GH_SLOTS + 1) {
                __builtin_amdgcn_s_sleep(1);
                made = __hip_atomic_load(&S.made[slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        if ((lane & 15) == 0) zdst0[slot * 32] = z;
        if (lane == 0) __hip_atomic_store(&S.flag[slot][wave], sw + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    // Every wave of the block makes the same sweeps: each slot sees all sixteen arrive. An item's loads are asked for when
    // the item before it has been decoded: with sixteen waves a CU that keeps about 56 KB a CU in flight, which is what HBM
    // serves best (an item ahead - twice as much in flight - was measured slower, 35.1 against 33.8 us).
    if (!early) issue(ma);
    for (int sw = 0; sw < nsweep; ++sw) {
        decode(ma, sw);
        if (sw + 1 < nsweep) {
            step(ma);
            issue(ma);
        }
        const int q = sw - GH_LAG;   // the sweep whose block is due; wave q mod 16 makes it
        if (q >= 0 && (q & (GH_WAVES - 1)) == wave) make_block(q);
    }
    for (int q = max(nsweep - GH_LAG, 0); q < nsweep; ++q)   // the last sweeps' blocks
        if ((q & (GH_WAVES - 1)) == wave) make_block(q);
}

// ---------------------------------------------------------------- launch 3: down and the combine
// out[t][r] = sum_k topw[t][k] (down_{e(t,k)}[r] . h[t,k]) + sigmoid(gate logit) (down_shared[r] . h[shared, t]): the
// work of k_moe_down (moe.cuh:613-658) and of the combine (kernels.cu:412-419) with one wave making a row's whole chain.
// A block = one window row and 8 x 4 consecutive units of the output; its waves walk the row's picks in order, the shared
// expert last, four units of that expert's matrix a trip, so at any time the grid reads a few experts' matrices front to
// back. The chain is the combine's: s = fmaf(w_k, part_k, s) over the picks in order, then s + sigmoid * shared; part_k is
// a unit row's sum over its lanes. An expert that several rows picked is read once per row (from the caches after the
// first). The q8_1 rows of h of the row's pairs come from the gate|up launch; a block copies its row's into LDS.
// (With the rows made here from f32 gate|up outputs - SwiGLU, the 32-value maxima, the rounding, for eleven pairs a
// block - this launch took 24 us instead of 18: that work stood between the launch's start and its first decode.)
struct DownArgs {
    int rows, ff, topk, T, nexp;
    const uint8_t* w;          // routed experts: expert e at w + e * stride, or ep[e]
    size_t stride;
    const uint8_t* const* ep;
    const uint8_t* w_shared;
    const uint32_t* hq;        // the pairs' h rows in q8_1 form, [pair][ff / 32][HQ_WORDS], as the gate|up launch leaves them
    const int* topi;
    const float* topw;
    const float* logits;       // [T][nexp + 1]: the shared expert's gate logit is a row's last
    float* out;                // [T][rows]
    const int* live;           // may be null; else a device word: rows from *live on are left alone
    RouteArgs route;           // the job lists that the grid's last block writes
    const float* sh_part;      // may be null; else [T][rows]: the shared expert's down rows, computed elsewhere (w_shared is then not read)
};
template <int SBR>
__global__ void __launch_bounds__(FL_THREADS) k_moe_down_combine(const DownArgs a) {
    constexpr int RW = 64 / SBR, R = 4;   // rows a unit, units a trip
    __shared__ uint32_t tab[SGRID_WORDS];
    __shared__ __align__(16) uint32_t hq[FL_MAXK + 1][SBR][HQ_WORDS];
    const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63, kb = lane % SBR, g = lane / SBR;
    const int nug = a.rows / (RW * R * FL_WAVES);   // blocks a window row
    const int t = blockIdx.x / nug, ug = blockIdx.x % nug;
    const int Tl = a.live ? uniform(max(0, min(*a.live, a.T))) : a.T;
    if (blockIdx.x == gridDim.x - 1) {   // the spare block: the job lists for the caller
        write_job_lists<FL_THREADS>(*reinterpret_cast<RouteLds<FL_THREADS>*>(tab), a.route, Tl);
        return;
    }
    if (t >= Tl) return;
    // the codebook's unsigned entries, the launch's first load; the blocks read different signed forms of the table in
    // memory and negate them back, so that not every wave of the grid asks the same sixteen cache lines at once
    const int form = (int) blockIdx.x & 15;
    const uint32_t tab0 = signed_entry(g_sgrid.v[(form << 9) + tid], form);
    const int topk = a.topk, P = a.T * topk;
    // the row's h rows: asked for next (they depend on nothing the block computes), a pick's words side by side
    constexpr int HQ_PER = SBR * HQ_WORDS, HQ_VPT = ((FL_MAXK + 1) * HQ_PER + FL_THREADS - 1) / FL_THREADS;
    uint32_t hw[HQ_VPT];
#pragma unroll
    for (int j = 0; j < HQ_VPT; ++j) {
        const int i = tid + j * FL_THREADS, k = i / HQ_PER;
        hw[j] = k <= topk ? a.hq[(size_t) (k < topk ? t * topk + k : P + t) * HQ_PER + (i - k * HQ_PER)] : 0u;
    }
    // lane k: pick k's matrix and weight; lane topk: the shared expert's and its gate
    const bool ext = a.sh_part != nullptr;   // the shared expert's rows come from memory: the trips are the picks only
    const int first = ext ? 1 : 0;
    const uint8_t* myw = a.w_shared;
    float myg = 0.f;
    if (lane < topk) {
        const int e = a.topi[t * topk + lane];
        myw = a.ep ? a.ep[e] : a.w + (size_t) e * a.stride;
        myg = a.topw[t * topk + lane];
    } else if (lane == topk) myg = sigmoid_f(a.logits[(size_t) t * (a.nexp + 1) + a.nexp]);
    const uint32_t myw_lo = (uint32_t) (uintptr_t) myw, myw_hi = (uint32_t) ((uint64_t) (uintptr_t) myw >> 32);
    const int u0 = (ug * FL_WAVES + wave) * R;   // this wave's units of every matrix
    const PackedVOffs o = packed_voffs(lane);
    auto issue = [&](PackedSub(&buf)[R], int k) {
        const uint64_t p = (uint64_t) (uint32_t) __builtin_amdgcn_readlane((int) myw_lo, k) | (uint64_t) (uint32_t) __builtin_amdgcn_readlane((int) myw_hi, k) << 32;
        const __amdgpu_buffer_rsrc_t mtx = matrix_rsrc((const uint8_t*) (uintptr_t) p);
#pragma unroll
        for (int r = 0; r < R; ++r) buf[r] = load_packed_buf(mtx, (u0 + r) * UNIT_BYTES, o);
    };
    // Trip 0 is the shared expert's (its matrix is known without the picks: its loads go out with the launch's first),
    // trips 1 .. topk the picks in order; the shared expert's sums wait in registers for the chain's last step.
    auto pick_of = [&](int trip) { return trip == 0 ? topk : trip - 1; };   // the index of a trip's expert in hq and in the lanes
    PackedSub A[R], B[R], C[R];
    float shp[R];
#pragma unroll
    for (int r = 0; r < R; ++r) shp[r] = 0.f;
    if (!ext) {
        const __amdgpu_buffer_rsrc_t mtx = matrix_rsrc(a.w_shared);
#pragma unroll
        for (int r = 0; r < R; ++r) A[r] = load_packed_buf(mtx, (u0 + r) * UNIT_BYTES, o);
    } else if (kb == SBR - 1) {   // the lanes that store a row's result hold its shared part
        const float* sp = a.sh_part + (size_t) t * a.rows + (size_t) u0 * RW + g;
#pragma unroll
        for (int r = 0; r < R; ++r) shp[r] = sp[r * RW];
    }
#pragma unroll
    for (int i = 0; i < SGRID_WORDS / FL_THREADS; ++i) tab[tid + i * FL_THREADS] = signed_entry(tab0, i);
#pragma unroll
    for (int j = 0; j < HQ_VPT; ++j) {
        const int i = tid + j * FL_THREADS;
        if (i < (topk + 1) * HQ_PER) (&hq[0][0][0])[i] = hw[j];
    }
    if (ext) issue(A, pick_of(1));   // topk >= 1
    if (first + 1 <= topk) issue(B, pick_of(first + 1));
    __syncthreads();
    const int sc_shift = 4 * (lane & 1);
    float acc[R], zs[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = zs[r] = 0.f;
    auto decode = [&](const PackedSub(&buf)[R], int trip) {
        const int k = pick_of(trip);
        const uint32_t* hb = hq[k][kb];
        const uint4 lo = *reinterpret_cast<const uint4*>(hb), hi = *reinterpret_cast<const uint4*>(hb + 4);
        const int xs[8] = {(int) lo.x, (int) lo.y, (int) lo.z, (int) lo.w, (int) hi.x, (int) hi.y, (int) hi.z, (int) hi.w};
        const float dx = __uint_as_float(hb[8]);
        const float gk = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, myg), k));
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int w4[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) w4[j] = *reinterpret_cast<const int*>(reinterpret_cast<const uint8_t*>(tab) + packed_addr(buf[r].idx, j));
            const int sc = 1 + 2 * (int) ((buf[r].sc >> sc_shift) & 0xFu);
            const float dw = half_bits_to_float(buf[r].d);
            int sum = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) sum = __builtin_amdgcn_sdot4(w4[j], xs[j], sum, false);
            const float z = dpp_group_sum<SBR>((dw * dx) * (float) __mul24(sum, sc));
            if (trip == 0) zs[r] = gk * z;
            else acc[r] = fmaf(gk, z, acc[r]);
        }
    };
    // two trips' loads are in flight while a third is decoded: with eight waves a CU that is about 56 KB a CU
    for (int trip = first; trip <= topk; trip += 3) {
        if (trip + 2 <= topk) issue(C, pick_of(trip + 2));
        decode(A, trip);
        if (trip + 1 > topk) break;
        if (trip + 3 <= topk) issue(A, pick_of(trip + 3));
        decode(B, trip + 1);
        if (trip + 2 > topk) break;
        if (trip + 4 <= topk) issue(B, pick_of(trip + 4));
        decode(C, trip + 2);
    }
    if (ext) {
        const float gs = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, myg), topk));
#pragma unroll
        for (int r = 0; r < R; ++r) zs[r] = gs * shp[r];
    }
    float res[R];
#pragma unroll
    for (int r = 0; r < R; ++r) res[r] = acc[r] + zs[r];   // the combine's last step: s + sigmoid * shared
    if (kb == SBR - 1) {
        float* orow = a.out + (size_t) t * a.rows + (size_t) u0 * RW + g;
#pragma unroll
        for (int r = 0; r < R; ++r) orow[r * RW] = res[r];
    }
}

}  // namespace fnx
