// The MoE half of a verify window (the work of Engine::ffn_half, engine.cu:1569-1757 of the reference, on one GPU) in
// five launches: [router logits | q8_1 rows of x] -> [top-k] -> [jobs and plan, gate|up, routed and shared] ->
// [SwiGLU to q8_1 on the fly + down, routed and shared] -> [combine].
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

// what the routing block hands to every other block: the jobs in compact form and the list of passes.
// A pass = (job, first token, 1 or 2 tokens) over all the job's units; the passes' units are what the waves split
// evenly, so a job of many rows (the shared expert's has the whole window) weighs as many times as it is walked.
struct LayerPlan {
    int nj, npass;
    int job_w[FL_MAXJ];                       // expert, or -1 for the shared expert
    uint8_t job_n[FL_MAXJ + 3];
    uint8_t job_pairs[FL_MAXJ][FNX_MAXT];     // output rows (pairs t * topk + k, or P + t), ascending
    uint8_t pair_tok[FL_MAXP + FNX_MAXT];     // the window row of a pair
    uint8_t pass_job[FL_MAXP + FNX_MAXT];
    uint8_t pass_t0[FL_MAXP + FNX_MAXT];
};
// one MoE in flight per device (as g_moe_hq)
__device__ LayerPlan g_layer_plan;

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
template <int NE>
__device__ __forceinline__ void wave_topk(const float* __restrict__ row, int nexp, int topk, int lane, int* __restrict__ ex,
                                          int* __restrict__ topi, float* __restrict__ topw) {
    float v[NE];
#pragma unroll
    for (int i = 0; i < NE; ++i) {
        const int e = lane + 64 * i;
        v[i] = e < nexp ? row[e] : -INFINITY;
    }
    float top0 = 0.f, z = 0.f, wk = 0.f;
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
        const bool mine = mi < nexp && (mi & 63) == lane;
#pragma unroll
        for (int i = 0; i < NE; ++i)
            if (mine && (mi >> 6) == i) v[i] = -INFINITY;
        if (k == 0) top0 = m;
        const float ek = expf(m - top0);
        z += ek;
        if (lane == k) {
            wk = ek;
            const int pick = mi < nexp ? mi : nexp - 1;   // fewer than topk finite logits: stay inside the tables
            ex[k] = pick;
            topi[k] = pick;
        }
    }
    if (lane < topk) topw[lane] = wk / z;
}

// ---------------------------------------------------------------- launch 2: top-k; the plan, made by its readers
// k_route_topk: a wave per row of the window ranks the row's logits. The job lists and the plan follow from all rows'
// picks without any serial loop: a token picks an expert at most once, so a pair's slot in its job is the number of
// earlier tokens in the expert's token mask, and a job's number is the rank of its first pair among the first pairs
// (the order k_router_route's last block gives them, moe.cuh:324-330). Every block of the gate|up launch makes the plan
// for itself in LDS from the 160 picks (build_plan), while its codebook loads are in flight; its block 0 also writes the
// plan and the job lists to memory, for the down launch and for the caller. That is quicker than a last-block phase in
// the top-k launch, which costs an atomic and two more memory round trips on the window's critical path.
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
constexpr int RT_THREADS = 64;
__global__ void __launch_bounds__(RT_THREADS) k_route_topk(const RouteArgs a) {
    __shared__ int ex[FL_MAXP];
    const int lane = threadIdx.x, LS = a.nexp + 1, t = blockIdx.x, topk = a.topk;
    const int Tl = a.live ? uniform(max(0, min(*a.live, a.T))) : a.T;
    if (t >= Tl) return;
    if (a.nexp <= 512) wave_topk<8>(a.logits + (size_t) t * LS, a.nexp, topk, lane, ex, a.topi + t * topk, a.topw + t * topk);
    else wave_topk<16>(a.logits + (size_t) t * LS, a.nexp, topk, lane, ex, a.topi + t * topk, a.topw + t * topk);
}

template <int NT>
struct RouteLds {
    LayerPlan plan;
    int ex[FL_MAXP];
    unsigned mask[1024];      // per expert: the window rows that picked it
    int first[1024];          // per expert: its first pair
    int jobof[1024];
    int pass0[FL_MAXJ + 3];   // per job: its first pass
    int wcnt[NT / 64];
};
// All NT threads of a block; ends with a barrier. publish: also write the lists and the plan to memory.
template <int NT>
__device__ __forceinline__ void build_plan(RouteLds<NT>& L, const RouteArgs& a, bool publish) {
    static_assert(FL_MAXP <= NT && FL_MAXJ <= NT, "a thread per pair, a thread per job");
    const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63;
    const int T = a.T, topk = a.topk, P = T * topk;
    const int Tl = a.live ? uniform(max(0, min(*a.live, T))) : T, Pl = Tl * topk;
    LayerPlan& pl = L.plan;
    const int e_mine = tid < Pl ? a.topi[tid] : 0;   // asked for before the tables are cleared
    for (int e = tid; e < a.nexp; e += NT) {
        L.mask[e] = 0u;
        L.first[e] = P;
    }
    __syncthreads();
    if (tid < Pl) {
        L.ex[tid] = e_mine;
        atomicOr(&L.mask[e_mine], 1u << (tid / topk));
        atomicMin(&L.first[e_mine], tid);
        pl.pair_tok[tid] = (uint8_t) (tid / topk);
    }
    if (tid < Tl) pl.pair_tok[P + tid] = (uint8_t) tid;
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
    nj = uniform(nj);
    if (isfirst) {
        const int j = before + __popcll(b & ((1ull << lane) - 1ull)), cnt = __popc(L.mask[e_mine]);
        L.jobof[e_mine] = j;
        pl.job_w[j] = e_mine;
        pl.job_n[j] = (uint8_t) cnt;
        if (publish) {
            a.jobs_gu[j].w = a.jobs_dn[j].w = e_mine;
            a.jobs_gu[j].n = a.jobs_dn[j].n = cnt;
        }
    }
    if (tid == 0) {
        pl.nj = nj;
        pl.job_w[nj] = -1;   // the shared expert's job: every row of the window, pairs P + t
        pl.job_n[nj] = (uint8_t) Tl;
        if (publish) a.njobs[0] = nj;
    }
    __syncthreads();
    // a pair's slot in its job: the earlier rows in its expert's mask (pairs of a job ascend with the row)
    if (tid < Pl) {
        const int j = L.jobof[e_mine], row = tid / topk, slot = __popc(L.mask[e_mine] & ((1u << row) - 1u));
        pl.job_pairs[j][slot] = (uint8_t) tid;
        if (publish) {
            a.jobs_gu[j].y[slot] = row;
            a.jobs_gu[j].out[slot] = tid;
            a.jobs_dn[j].y[slot] = tid;
            a.jobs_dn[j].out[slot] = tid;
        }
    }
    if (tid < max(Tl, 1)) {   // the shared expert's job, at index P of the lists the API returns (kernels.hpp:277-282)
        pl.job_pairs[nj][tid] = (uint8_t) (P + tid);
        if (publish) {
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
    // passes: job j's rows two at a time; job j's first pass = the passes of the jobs before it: a scan over the jobs
    // (wave by wave with the waves' totals in LDS; a thread per job)
    {
        const int cj = tid <= nj ? (pl.job_n[tid] + 1) >> 1 : 0;
        int inc = cj;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int up = __shfl_up(inc, o, 64);
            if (lane >= o) inc += up;
        }
        if (lane == 63) L.wcnt[wave] = inc;   // (the job count's readers of wcnt are behind a barrier)
        __syncthreads();
        int bef = 0;
        for (int w = 0; w < wave; ++w) bef += L.wcnt[w];
        if (tid <= nj) {
            const int p0 = bef + inc - cj, n = pl.job_n[tid];
            for (int t0 = 0, k = 0; t0 < n; t0 += 2, ++k) {
                pl.pass_job[p0 + k] = (uint8_t) tid;
                pl.pass_t0[p0 + k] = (uint8_t) t0;
            }
        }
        if (tid == nj) pl.npass = bef + inc;
    }
    __syncthreads();
    if (publish)
        for (int i = tid; i < (int) (sizeof(LayerPlan) / 4); i += NT) reinterpret_cast<int*>(&g_layer_plan)[i] = reinterpret_cast<const int*>(&pl)[i];
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

// ---------------------------------------------------------------- launches 3 and 4: the passes of the plan
struct PassArgs {
    int rows;                 // rows of every matrix
    const uint8_t* w;         // routed experts: expert e at w + e * stride, or ep[e]
    size_t stride;
    const uint8_t* const* ep;
    const uint8_t* w_shared;
    const uint8_t* xq;        // gate|up: the window's q8_1 rows
    const float* gu;          // down: the gate|up outputs [pair][2 ff]
    int ff;
    float* out;               // [pair][rows]
    RouteArgs route;          // gate|up: what the plan is made from
};
struct PassSeg {   // a stretch of one pass's units
    int ul, ue, ji, t0, nt;
    const uint8_t* we;
};
// Unit numbers are 32-bit and a pass's units a power of two: 64-bit divisions (a few hundred instructions each, five of
// them a wave) held the first weight loads up by one to two microseconds. The host keeps units * waves below 2^32.
// (A division by the number of waves is forty instructions, twice a wave, on every wave of a SIMD at the same moment:
// with a power of two - 2 x 256 CUs x 8 waves - it is a shift.)
__device__ __forceinline__ uint32_t share_begin(uint32_t total, uint32_t gw, uint32_t nw) {
    const uint32_t p = total * gw;
    return (nw & (nw - 1)) == 0 ? p >> (31 - __clz(nw)) : p / nw;
}
__device__ __forceinline__ PassSeg pass_seg(const LayerPlan& pl, const PassArgs& a, uint32_t uu, uint32_t u1, int upj_log2) {
    PassSeg s;
    const int pi = (int) (uu >> upj_log2), upj = 1 << upj_log2;
    s.ul = (int) (uu & (uint32_t) (upj - 1));
    s.ue = (int) min((uint32_t) upj, s.ul + (u1 - uu));
    s.ji = uniform((int) pl.pass_job[pi]);
    s.t0 = uniform((int) pl.pass_t0[pi]);
    const int w = uniform(pl.job_w[s.ji]);
    s.nt = uniform((int) pl.job_n[s.ji]) - s.t0;
    s.we = w < 0 ? a.w_shared : a.ep ? uniform_ptr(a.ep[w]) : a.w + (size_t) w * a.stride;
    return s;
}

// gate|up: rows of 2048 columns; activations: the window's q8_1 rows. The waves of the grid split the passes' units
// evenly and walk them in order.
__global__ void __launch_bounds__(FL_THREADS) k_moe_gate_up_passes(const PassArgs a) {
    constexpr int SBR = 64;
    __shared__ uint32_t tab[SGRID_WORDS];
    __shared__ RouteLds<FL_THREADS> L;
    LayerPlan& pl = L.plan;
    const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63;
    // the codebook's load goes out first (a thread's unsigned entry; its sixteen signed forms are made and stored to
    // LDS once the first weights have been asked for, so that the latencies overlap: sixteen loads a thread and 16 MB
    // from the caches over the grid if the whole table were read)
    static_assert(FL_THREADS == 512, "a thread per 9-bit code: its sixteen signed entries are made from the first");
    const uint32_t tab0 = g_sgrid.v[tid];
    build_plan<FL_THREADS>(L, a.route, blockIdx.x == 0);
    const int upj = uniform(31 - __clz(a.rows));   // log2 of a pass's units
    const uint32_t total = (uint32_t) pl.npass << upj;
    const uint32_t gw = blockIdx.x * FL_WAVES + wave, nw = gridDim.x * FL_WAVES;
    uint32_t u = share_begin(total, gw, nw);
    const uint32_t u1 = share_begin(total, gw + 1, nw);
    PackedSub cur[4];
    PassSeg s{};
    if (u < u1) {
        s = pass_seg(pl, a, u, u1, upj);
        packed_first(s.we, s.ul, s.ue, cur);
    }
#pragma unroll
    for (int i = 0; i < SGRID_WORDS / FL_THREADS; ++i) tab[tid + i * FL_THREADS] = signed_entry(tab0, i);
    __syncthreads();
    while (u < u1) {
        const uint8_t* pairs = pl.job_pairs[s.ji] + s.t0;
        auto prep_for = [&](auto nt_tag) {
            constexpr int NT = decltype(nt_tag)::value;
            const uint8_t* pair_tok = pl.pair_tok;
            return [=](int(&xs)[NT][8], float(&dx)[NT], float*(&orow)[NT]) {
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const int pair = uniform((int) pairs[t]), tok = uniform((int) pair_tok[pair]);
                    const uint8_t* yb = a.xq + ((size_t) tok * SBR + lane) * FNX_Q8_1_BLOCK;
                    dx[t] = half_bits_to_float(*reinterpret_cast<const unsigned short*>(yb));
#pragma unroll
                    for (int j = 0; j < 8; ++j) xs[t][j] = reinterpret_cast<const int*>(yb + 4)[j];
                    orow[t] = a.out + (size_t) pair * a.rows;
                }
            };
        };
        if (s.nt >= 2) packed_units<SBR, 2>(tab, s.we, s.ul, s.ue, cur, prep_for(std::integral_constant<int, 2>{}));
        else packed_units<SBR, 1>(tab, s.we, s.ul, s.ue, cur, prep_for(std::integral_constant<int, 1>{}));
        u += s.ue - s.ul;
        if (u < u1) {
            s = pass_seg(pl, a, u, u1, upj);
            packed_first(s.we, s.ul, s.ue, cur);
        }
    }
}

// down: rows of 32 SBR columns, split over the waves like gate|up. A wave makes the q8_1 form of h = silu(gate) * up
// for its pass's pairs itself (k_moe_down without PRE, moe.cuh:630-641): the 64 / SBR lanes that share a sub-block
// column split its 32 values. (Making h once per block in LDS for the block's 8 waves was measured slower: 30 us
// against 25 us, the block-wide barriers cost more than the repeated SwiGLU.)
template <int SBR>
__global__ void __launch_bounds__(FL_THREADS) k_moe_down_passes(const PassArgs a) {
    constexpr int RW = 64 / SBR;   // rows per unit
    __shared__ uint32_t tab[SGRID_WORDS];
    __shared__ LayerPlan pl;
    // h = silu(gate) * up of the block's pairs in q8_1 form (k_moe_h, moe.cuh:597-608): per pair and 32-value block the
    // 32 int8 values, then the block's scale as a float. A block's eight waves walk consecutive units, fewer than a pass
    // has, so they are in two passes at most: four pairs, made once by the whole block ahead of the barrier that the
    // codebook needs anyway (every wave making its own pairs' rows read the gate|up outputs 21 times over a pass).
    __shared__ __align__(16) uint32_t hq[4][SBR][12];   // 8 words of values, the scale, 3 unused (16-byte rows)
    const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63;
    static_assert(FL_THREADS == 512, "a thread per 9-bit code: its sixteen signed entries are made from the first");
    const uint32_t tab0 = g_sgrid.v[tid];
    for (int i = tid; i < (int) (sizeof(LayerPlan) / 4); i += FL_THREADS) reinterpret_cast<int*>(&pl)[i] = reinterpret_cast<const int*>(&g_layer_plan)[i];
    __syncthreads();
    const int upj = uniform(31 - __clz(a.rows / RW)), ff = a.ff;   // log2 of a pass's units
    const uint32_t total = (uint32_t) pl.npass << upj;
    const uint32_t gw = blockIdx.x * FL_WAVES + wave, nw = gridDim.x * FL_WAVES;
    uint32_t u = share_begin(total, gw, nw);
    const uint32_t u1 = share_begin(total, gw + 1, nw);
    PackedSub cur[4];
    PassSeg s{};
    if (u < u1) {
        s = pass_seg(pl, a, u, u1, upj);
        packed_first(s.we, s.ul, s.ue, cur);
    }
    const int pass0 = (int) (share_begin(total, blockIdx.x * FL_WAVES, nw) >> upj);   // the block's first pass
    {
        constexpr int VPT = (SBR * 32 + FL_THREADS - 1) / FL_THREADS;   // values a thread and pair
        float gv[4][VPT], uv[4][VPT];
        bool on[4];
#pragma unroll
        for (int slot = 0; slot < 4; ++slot) {   // all the loads first: one trip to the cache for the four pairs
            const int pi = pass0 + (slot >> 1), t = slot & 1;
            const int pc = max(min(pi, pl.npass - 1), 0);
            on[slot] = pi < pl.npass && pl.pass_t0[pc] + t < pl.job_n[pl.pass_job[pc]];
            if (on[slot]) {   // the same for every thread of the block
                const int ji = pl.pass_job[pi], pair = pl.job_pairs[ji][pl.pass_t0[pi] + t];
                const float* gp = a.gu + (size_t) pair * 2 * ff;
#pragma unroll
                for (int k = 0; k < VPT; ++k) {
                    const int i = tid + k * FL_THREADS;
                    gv[slot][k] = i < ff ? gp[i] : 0.f;
                    uv[slot][k] = i < ff ? gp[ff + i] : 0.f;
                }
            }
        }
#pragma unroll
        for (int slot = 0; slot < 4; ++slot)
            if (on[slot])
#pragma unroll
                for (int k = 0; k < VPT; ++k) {
                    const int i = tid + k * FL_THREADS;
                    if (i < ff) {   // whole 32-lane groups
                        const float h = silu_f(gv[slot][k]) * uv[slot][k];
                        const float amax = group_max<32>(fabsf(h));
                        const float d = amax / 127.0f;
                        const int q = amax == 0.0f ? 0 : (int) (int8_t) roundf(h / d);
                        reinterpret_cast<int8_t*>(&hq[slot][i >> 5][0])[i & 31] = (int8_t) q;
                        if ((i & 31) == 0) hq[slot][i >> 5][8] = __float_as_uint(half_bits_to_float(float_to_half_bits(d)));
                    }
                }
    }
#pragma unroll
    for (int i = 0; i < SGRID_WORDS / FL_THREADS; ++i) tab[tid + i * FL_THREADS] = signed_entry(tab0, i);
    __syncthreads();
    const int kb = lane % SBR;
    while (u < u1) {
        const int slot0 = 2 * ((int) (u >> upj) - pass0);   // 0 or 2
        auto prep_for = [&](auto nt_tag) {
            constexpr int NT = decltype(nt_tag)::value;
            return [=](int(&xs)[NT][8], float(&dx)[NT], float*(&orow)[NT]) {
                const uint8_t* pairs = pl.job_pairs[s.ji] + s.t0;
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const uint32_t* hb = hq[slot0 + t][kb];
                    const uint4 lo = *reinterpret_cast<const uint4*>(hb), hi = *reinterpret_cast<const uint4*>(hb + 4);
                    xs[t][0] = (int) lo.x, xs[t][1] = (int) lo.y, xs[t][2] = (int) lo.z, xs[t][3] = (int) lo.w;
                    xs[t][4] = (int) hi.x, xs[t][5] = (int) hi.y, xs[t][6] = (int) hi.z, xs[t][7] = (int) hi.w;
                    dx[t] = __uint_as_float(hb[8]);
                    orow[t] = a.out + (size_t) uniform((int) pairs[t]) * a.rows;
                }
            };
        };
        if (s.nt >= 2) packed_units<SBR, 2>(tab, s.we, s.ul, s.ue, cur, prep_for(std::integral_constant<int, 2>{}));
        else packed_units<SBR, 1>(tab, s.we, s.ul, s.ue, cur, prep_for(std::integral_constant<int, 1>{}));
        u += s.ue - s.ul;
        if (u < u1) {
            s = pass_seg(pl, a, u, u1, upj);
            packed_first(s.we, s.ul, s.ue, cur);
        }
    }
}

}  // namespace fnx
