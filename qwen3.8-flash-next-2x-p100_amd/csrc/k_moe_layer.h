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
            if (publish) topi[k] = pick;
        }
    }
    if (publish && lane < topk) topw[lane] = wk / z;
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
    const int e_mine = tid < Pl ? a.topi[tid] : 0;
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
// rows and 256 blocks a thread block has one row's one block of 32 for all the row's picks, the shared expert last. So
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
    uint32_t wp[2][FL_MAXK + 1][2];   // the matrices of the block's (at most two) rows' picks, the shared expert's last
    float hb[GH_SLOTS][32];           // [slot][h value of the block]
    int flag[GH_SLOTS][GH_WAVES];     // sweep + 1 of the values a wave last wrote into the slot
    int made[GH_SLOTS];               // sweeps whose block has been made from the slot: a writer of sweep s waits for made >= s - GH_SLOTS + 1
    int ex[2][FL_MAXK];
};
struct GhItem {   // (row, block of 32, pick) of an item number, kept by stepping
    int t, j, k;
};
__global__ void __launch_bounds__(GH_THREADS) k_moe_gate_up_h(const GateUpArgs a) {
    __shared__ GhLds S;
    const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63;
    const int T = a.route.T, topk = a.route.topk, P = T * topk, qpp = a.ff >> 5, per_row = qpp * (topk + 1);
    const int Tl = a.route.live ? uniform(max(0, min(*a.route.live, T))) : T;
    // this block's run of items
    const int total = Tl * per_row, nb = gridDim.x, ipb = (total + nb - 1) / nb;
    const int I0 = (int) blockIdx.x * ipb, I1 = min(total, I0 + ipb), nsweep = I1 - I0;
    if (nsweep <= 0) return;
    const uint32_t tab0 = g_sgrid.v[tid & 511];
    const int t0 = I0 / per_row, t1 = (I1 - 1) / per_row;   // ipb <= per_row (the launcher sees to it): two rows at most
    auto load_x = [&](int t, int (&xs)[8], float& dx) {   // the lane's sub-block of row t's activations
        const uint32_t* yb = reinterpret_cast<const uint32_t*>(a.xq + ((size_t) t * 64 + lane) * FNX_Q8_1_BLOCK);
        dx = half_bits_to_float(yb[0] & 0xFFFFu);
#pragma unroll
        for (int j = 0; j < 8; ++j) xs[j] = (int) yb[j + 1];
    };
    int xs[8], tx = t0;
    float dx;
    load_x(t0, xs, dx);
    if (wave < 2 && t0 + wave <= t1) {   // the rows' picks (moe.cuh:382-411), a wave a row; the row's first item's block writes them out
        const int t = t0 + wave;
        const bool publish = t * per_row >= I0;
        const float* row = a.route.logits + (size_t) t * (a.route.nexp + 1);
        if (a.route.nexp <= 512) wave_topk<8>(row, a.route.nexp, topk, lane, S.ex[wave], a.route.topi + t * topk, a.route.topw + t * topk, publish);
        else wave_topk<16>(row, a.route.nexp, topk, lane, S.ex[wave], a.route.topi + t * topk, a.route.topw + t * topk, publish);
        if (lane <= topk) {   // LDS writes of this wave, read back in order
            const uint8_t* e = a.w_shared;
            if (lane < topk) {
                const int ei = S.ex[wave][lane];
                e = a.ep ? a.ep[ei] : a.w + (size_t) ei * a.stride;
            }
            S.wp[wave][lane][0] = (uint32_t) (uintptr_t) e;
            S.wp[wave][lane][1] = (uint32_t) ((uint64_t) (uintptr_t) e >> 32);
        }
    }
    if (tid < GH_SLOTS * GH_WAVES) (&S.flag[0][0])[tid] = 0;
    if (tid < GH_SLOTS) S.made[tid] = 0;
    // the codebook: two threads a code, eight signed forms each
#pragma unroll
    for (int i = 0; i < 8; ++i) S.tab[tid + i * GH_THREADS] = signed_entry(tab0, (tid >> 9) + 2 * i);
    __syncthreads();
    const PackedOffs o = packed_offs(lane);
    const int sc_shift = 4 * (lane & 1);
    // byte offsets of the wave's gate units and up units from its item's first gate unit
    const uint32_t uo_g = (uint32_t) (wave * 2) * UNIT_BYTES, uo_u = uo_g + (uint32_t) a.ff * UNIT_BYTES;
    auto item_of = [&](int I) {
        GhItem m;
        m.t = I / per_row;
        const int r = I - m.t * per_row;
        m.j = r / (topk + 1);
        m.k = r - m.j * (topk + 1);
        return m;
    };
    auto step = [&](GhItem& m) {
        if (++m.k > topk) {
            m.k = 0;
            if (++m.j == qpp) {
                m.j = 0;
                ++m.t;
            }
        }
    };
    auto issue = [&](PackedSub(&u)[4], const GhItem& m) {
        const uint2 p = *reinterpret_cast<const uint2*>(S.wp[m.t - t0][m.k]);
        const uint64_t e = (uint64_t) (uint32_t) uniform((int) p.x) | (uint64_t) (uint32_t) uniform((int) p.y) << 32;
        const uint8_t* we = (const uint8_t*) (uintptr_t) e + (size_t) (m.j * 32) * UNIT_BYTES;
        u[0] = load_packed(as_global(we + uo_g), o);
        u[1] = load_packed(as_global(we + uo_g + UNIT_BYTES), o);
        u[2] = load_packed(as_global(we + uo_u), o);
        u[3] = load_packed(as_global(we + uo_u + UNIT_BYTES), o);
    };
    // the q8_1 block of sweep q, by the first half of the wave
    auto make_block = [&](int q) {
        const int slot = q & (GH_SLOTS - 1);
        while (true) {   // all sixteen waves' values of sweep q must be there
            const int f = lane < GH_WAVES ? __hip_atomic_load(&S.flag[slot][lane], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) : q + 1;
            if (__ballot(f < q + 1) == 0ull) break;
            __builtin_amdgcn_s_sleep(2);
        }
        const GhItem m = item_of(I0 + q);
        const int pair = m.k < topk ? m.t * topk + m.k : P + m.t;
        if (lane < 32) {
            const float h = S.hb[slot][lane];
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
    auto decode = [&](const PackedSub(&u)[4], const GhItem& m, int sw) {
        if (m.t != tx) {   // the run has crossed into its second row
            tx = m.t;
            load_x(tx, xs, dx);
        }
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            int w4[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) w4[j] = *reinterpret_cast<const int*>(reinterpret_cast<const uint8_t*>(S.tab) + packed_addr(u[r].idx, j));
            const int sc = 1 + 2 * (int) ((u[r].sc >> sc_shift) & 0xFu);
            const float dw = half_bits_to_float(u[r].d);
            int sum = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) sum = __builtin_amdgcn_sdot4(w4[j], xs[j], sum, false);
            // one sub-block's term as the reference forms it: (d_w * d_x) * (float) (sumi * (1 + 2 s))
            v[r] = (dw * dx) * (float) __mul24(sum, sc);
        }
        // units: gate 2 i, gate 2 i + 1, up 2 i, up 2 i + 1 -> the 16-lane rows hold gate 2 i, up 2 i, gate 2 i + 1, up 2 i + 1
        const float z = reduce4_units(v[0], v[1], v[2], v[3]);
        const int zi = __builtin_bit_cast(int, z);
        const float g0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(zi, 0)), u0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(zi, 16));
        const float g1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(zi, 32)), u1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(zi, 48));
        const float h = silu_f(lane & 1 ? g1 : g0) * (lane & 1 ? u1 : u0);   // lane 0: h of row 2 i, lane 1: of row 2 i + 1
        const int slot = sw & (GH_SLOTS - 1);
        // the slot's last block (of sweep sw - GH_SLOTS) must have been made: nearly always long ago
        if (sw >= GH_SLOTS)
            while (uniform(__hip_atomic_load(&S.made[slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP)) < sw - GH_SLOTS + 1) __builtin_amdgcn_s_sleep(1);
        if (lane < 2) S.hb[slot][2 * wave + lane] = h;
        if (lane == 0) __hip_atomic_store(&S.flag[slot][wave], sw + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
        const int q = sw - GH_LAG;   // the sweep whose block is due; wave q mod 16 makes it
        if (q >= 0 && (q & (GH_WAVES - 1)) == wave) make_block(q);
    };
    // every wave of the block makes the same sweeps: each slot sees all sixteen arrive
    PackedSub cur[4], nxt[4];
    GhItem mc = item_of(I0), mn = mc;
    issue(cur, mc);
    for (int sw = 0; sw < nsweep; ++sw) {
        if (sw + 1 < nsweep) step(mn);
        issue(nxt, mn);   // past the end: the last item again (a read of what the caches hold)
        decode(cur, mc, sw);
#pragma unroll
        for (int r = 0; r < 4; ++r) cur[r] = nxt[r];
        mc = mn;
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
    const int topk = a.topk, P = a.T * topk;
    const uint32_t tab0 = g_sgrid.v[tid];
    // the row's h rows: asked for first (they depend on nothing the block computes), a pick's words side by side
    constexpr int HQ_PER = SBR * HQ_WORDS, HQ_VPT = ((FL_MAXK + 1) * HQ_PER + FL_THREADS - 1) / FL_THREADS;
    uint32_t hw[HQ_VPT];
#pragma unroll
    for (int j = 0; j < HQ_VPT; ++j) {
        const int i = tid + j * FL_THREADS, k = i / HQ_PER;
        hw[j] = k <= topk ? a.hq[(size_t) (k < topk ? t * topk + k : P + t) * HQ_PER + (i - k * HQ_PER)] : 0u;
    }
    // lane k: pick k's matrix and weight; lane topk: the shared expert's and its gate
    const uint8_t* myw = a.w_shared;
    float myg = 0.f;
    if (lane < topk) {
        const int e = a.topi[t * topk + lane];
        myw = a.ep ? a.ep[e] : a.w + (size_t) e * a.stride;
        myg = a.topw[t * topk + lane];
    } else if (lane == topk) myg = sigmoid_f(a.logits[(size_t) t * (a.nexp + 1) + a.nexp]);
    const uint32_t myw_lo = (uint32_t) (uintptr_t) myw, myw_hi = (uint32_t) ((uint64_t) (uintptr_t) myw >> 32);
    const int u0 = (ug * FL_WAVES + wave) * R;   // this wave's units of every matrix
    const PackedOffs o = packed_offs(lane);
    auto issue = [&](PackedSub(&buf)[R], int k) {
        const uint64_t p = (uint64_t) (uint32_t) __builtin_amdgcn_readlane((int) myw_lo, k) | (uint64_t) (uint32_t) __builtin_amdgcn_readlane((int) myw_hi, k) << 32;
        const uint8_t* we = (const uint8_t*) (uintptr_t) p + (size_t) u0 * UNIT_BYTES;
#pragma unroll
        for (int r = 0; r < R; ++r) buf[r] = load_packed(as_global(we + r * UNIT_BYTES), o);
    };
    PackedSub A[R], B[R], C[R];
    issue(A, 0);
    issue(B, 1);   // topk >= 1: the shared expert is trip topk
#pragma unroll
    for (int j = 0; j < HQ_VPT; ++j) {
        const int i = tid + j * FL_THREADS;
        if (i < (topk + 1) * HQ_PER) (&hq[0][0][0])[i] = hw[j];
    }
#pragma unroll
    for (int i = 0; i < SGRID_WORDS / FL_THREADS; ++i) tab[tid + i * FL_THREADS] = signed_entry(tab0, i);
    __syncthreads();
    const int sc_shift = 4 * (lane & 1);
    float acc[R], res[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = res[r] = 0.f;
    auto decode = [&](const PackedSub(&buf)[R], int k) {
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
            if (k < topk) acc[r] = fmaf(gk, z, acc[r]);
            else res[r] = acc[r] + gk * z;
        }
    };
    for (int k = 0; k <= topk; k += 3) {
        if (k + 2 <= topk) issue(C, k + 2);
        decode(A, k);
        if (k + 1 > topk) break;
        if (k + 3 <= topk) issue(A, k + 3);
        decode(B, k + 1);
        if (k + 2 > topk) break;
        if (k + 4 <= topk) issue(B, k + 4);
        decode(C, k + 2);
    }
    if (kb == SBR - 1) {
        float* orow = a.out + (size_t) t * a.rows + (size_t) u0 * RW + g;
#pragma unroll
        for (int r = 0; r < R; ++r) orow[r * RW] = res[r];
    }
}

}  // namespace fnx
