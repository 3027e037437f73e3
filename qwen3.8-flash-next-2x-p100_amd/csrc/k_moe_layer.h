// What the verify window's MoE half (k_moe_window.h) shares with the prompt path's routing (k_prefill.h): wave-wide
// maxima by DPP, the rank keys of the top-k, one token's top-k by a single wave, and the job lists of a window's picks.
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
        const float ek = found ? fnx_expf(m - top0) : 0.f;
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

// a pair's h rows as the window keeps them between its gate|up sweeps and its down trips: per pair and block of 32 values 8
// words of int8 values, the scale as a float, 3 unused
constexpr int HQ_WORDS = 12;
constexpr int FL_MAXK = 16;   // picks a row that the window takes

}  // namespace fnx
