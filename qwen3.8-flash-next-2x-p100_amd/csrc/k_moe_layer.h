// The MoE half of a verify window as ONE persistent kernel (the work of Engine::ffn_half, engine.cu:1569-1757 of the
// reference, on one GPU): router logits and q8_1 rows -> top-k and jobs -> routed + shared gate|up -> SwiGLU to q8_1
// -> routed + shared down -> combine. The grid is sized to be resident at once (two blocks of 8 waves per CU) and its
// phases meet at grid barriers, so the window pays one launch instead of nine and none of the ~4 us fixed cost each
// small kernel has on this GPU.
//
// Arithmetic is the operators': the router sums in the fixed 64-lane order, top-k by (value, lower index), the q8_1
// rounding, the IQ3_S sub-block terms, the combine's fmaf chain. Only the order in which a row's 64 (or 16) lane
// sums are added differs from the one-operator-per-launch path.
#pragma once

#include "k_iq3s_packed.h"

namespace fnx {

constexpr int FL_THREADS = 512, FL_WAVES = FL_THREADS / 64;
constexpr int FL_MAXP = FNX_MAXT * 10;    // routed pairs of a window (T * topk), at most
constexpr int FL_MAXJ = FL_MAXP + 1;      // their jobs, and the shared expert's
constexpr int FL_N = 2048;                // hidden size this kernel is built for (gate|up rows of 64 sub-blocks)
constexpr unsigned FL_SPIN_LIMIT = 1u << 22;
constexpr unsigned FL_ERR_BARRIER = 4u;   // error-word bit: a grid barrier timed out (engine_impl.hpp:211-218)

struct LayerArgs {
    int ff, nexp, topk, T;
    const float* x;
    const void* router;
    int router_bf16;
    const uint8_t* gu;
    size_t gu_stride;
    const uint8_t* const* gu_ep;
    const uint8_t* dn;
    size_t dn_stride;
    const uint8_t* const* dn_ep;
    const uint8_t* sh_gu;
    const uint8_t* sh_dn;
    uint8_t* xq;
    float* logits;
    int* topi;
    float* topw;
    fnx_job* jobs_gu;
    fnx_job* jobs_dn;
    int* njobs;
    float* gu_out;
    float* part;
    float* out;
    unsigned* sync;   // [0] barrier arrivals, [1] exits, [2] error word; all zero at launch, left at zero
};

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

struct LayerLds {
    // phase 1 (router blocks): [tab | a] together hold half of the window's x (float4 [16][4][64] = 64 KiB)
    uint32_t tab[SGRID_WORDS];
    __attribute__((aligned(16))) uint8_t a[FNX_MAXT * 64 * FNX_Q8_1_BLOCK];   // from phase 3 on: the window's q8_1 rows
    LayerPlan plan;
    int ex[FL_MAXP];
    int jobof[1024];
    int last;
    uint8_t isfirst[FL_MAXP];
};

// Phase stamps of the last launch, taken by block 0 (the counterpart of the reference's FNX_RR_TIMES stamps inside its
// router launch, moe.cuh:247-255): wall_clock64() ticks at [start, logits/q8 done, routed and plan in LDS, gate|up done,
// after barrier, down done, after barrier, end].
__device__ unsigned long long g_layer_stamps[8];
__device__ __forceinline__ void layer_stamp(int i) {
    if (blockIdx.x == 0 && threadIdx.x == 0) g_layer_stamps[i] = wall_clock64();
}

// every block of the grid arrives; nobody leaves before all have. Bounded: after FL_SPIN_LIMIT polls the block goes on
// and the error word says so (the results are then wrong, but every wave still reaches the end of the kernel).
__device__ __forceinline__ void spin_until(unsigned* word, unsigned target, unsigned* err) {
    unsigned spins = 0;
    while (__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
        __builtin_amdgcn_s_sleep(1);
        if (++spins > FL_SPIN_LIMIT) {
            atomicOr(err, FL_ERR_BARRIER);
            break;
        }
    }
}
__device__ __forceinline__ void grid_sync(unsigned* sync, unsigned nblocks, unsigned& epoch) {
    __syncthreads();
    if (threadIdx.x == 0) {
        ++epoch;
        __threadfence();
        atomicAdd(&sync[0], 1u);
        spin_until(&sync[0], epoch * nblocks, &sync[2]);
        __threadfence();
    }
    __syncthreads();
}

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
    unsigned taken = 0;
    float top0 = 0.f, z = 0.f, wk = 0.f;
    for (int k = 0; k < topk; ++k) {
        float bv = -INFINITY;
        int bi = nexp;
#pragma unroll
        for (int i = 0; i < NE; ++i)
            if (!((taken >> i) & 1u) && v[i] > bv) {   // ascending i: a lane's lower index wins its own ties
                bv = v[i];
                bi = lane + 64 * i;
            }
        const float m = wave_max(bv);
        const int mi = wave_min(bv == m ? bi : 0x7fffffff);   // the lowest index among the lanes that hold the maximum
        if (mi < nexp && (mi & 63) == lane) taken |= 1u << (mi >> 6);
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

// routing by one block: top-k per row of the window, the job lists the operator API returns, the plan for the grid
__device__ __forceinline__ void route_block(const LayerArgs& a, LayerLds& L) {
    const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63;
    const int T = a.T, P = T * a.topk, LS = a.nexp + 1;
    LayerPlan& pl = L.plan;
    for (int t = wave; t < T; t += FL_WAVES) {
        if (a.nexp <= 512) wave_topk<8>(a.logits + (size_t) t * LS, a.nexp, a.topk, lane, L.ex + t * a.topk, a.topi + t * a.topk, a.topw + t * a.topk);
        else wave_topk<16>(a.logits + (size_t) t * LS, a.nexp, a.topk, lane, L.ex + t * a.topk, a.topi + t * a.topk, a.topw + t * a.topk);
    }
    __syncthreads();
    // jobs: one per distinct expert, numbered by first pick, a job's pairs ascending (kernels.cu:381-398)
    const int p = tid;
    int slot = 0, e = -1;
    if (p < P) {
        e = L.ex[p];
        for (int q = 0; q < p; ++q) slot += L.ex[q] == e;
        L.isfirst[p] = slot == 0;
        pl.pair_tok[p] = (uint8_t) (p / a.topk);
    }
    if (p < T) pl.pair_tok[P + p] = (uint8_t) p;
    __syncthreads();
    if (p < P && slot == 0) {
        int j = 0, cnt = 0;
        for (int q = 0; q < P; ++q) {
            j += q < p && L.isfirst[q];
            cnt += L.ex[q] == e;
        }
        L.jobof[e] = j;
        pl.job_w[j] = e;
        pl.job_n[j] = (uint8_t) cnt;
        a.jobs_gu[j].w = a.jobs_dn[j].w = e;
        a.jobs_gu[j].n = a.jobs_dn[j].n = cnt;
    }
    if (p == P) {
        int nj = 0;
        for (int q = 0; q < P; ++q) nj += L.isfirst[q];
        pl.nj = nj;
        pl.job_w[nj] = -1;   // the shared expert's job: every row of the window, pairs P + t
        pl.job_n[nj] = (uint8_t) T;
        a.njobs[0] = nj;
    }
    __syncthreads();
    if (p < P) {
        const int j = L.jobof[e];
        pl.job_pairs[j][slot] = (uint8_t) p;
        a.jobs_gu[j].y[slot] = p / a.topk;
        a.jobs_gu[j].out[slot] = p;
        a.jobs_dn[j].y[slot] = p;
        a.jobs_dn[j].out[slot] = p;
    }
    if (p < T) {   // the shared expert's job, at index P of the lists the API returns (kernels.hpp:277-282)
        pl.job_pairs[pl.nj][p] = (uint8_t) (P + p);
        a.jobs_gu[P].y[p] = p;
        a.jobs_gu[P].out[p] = P + p;
        a.jobs_dn[P].y[p] = P + p;
        a.jobs_dn[P].out[p] = P + p;
        if (p == 0) {
            a.jobs_gu[P].w = a.jobs_dn[P].w = 0;
            a.jobs_gu[P].n = a.jobs_dn[P].n = T;
        }
    }
    // passes: job j's rows two at a time
    if (p == 0) {
        int np = 0;
        for (int j = 0; j <= pl.nj; ++j)
            for (int t0 = 0; t0 < pl.job_n[j]; t0 += 2) {
                pl.pass_job[np] = (uint8_t) j;
                pl.pass_t0[np] = (uint8_t) t0;
                ++np;
            }
        pl.npass = np;
    }
    __syncthreads();
    for (int i = tid; i < (int) (sizeof(LayerPlan) / 4); i += FL_THREADS) reinterpret_cast<int*>(&g_layer_plan)[i] = reinterpret_cast<const int*>(&pl)[i];
}

// SBR_D: sub-blocks per row of the down matrices (ff / 32): 8, 16 or 32
template <int SBR_D>
__global__ void __launch_bounds__(FL_THREADS, 4) k_moe_layer(const LayerArgs a) {   // 4 waves per SIMD: two blocks per CU
    __shared__ LayerLds L;
    const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63;
    const unsigned nblocks = gridDim.x;
    unsigned epoch = 0;
    const int T = a.T, n = FL_N, ff = a.ff, P = T * a.topk, LS = a.nexp + 1;
    layer_stamp(0);

    // ------------------------------------------------------------ phase 1: router logits | q8_1 rows of x
    {
        const int rblocks = (LS + FL_WAVES - 1) / FL_WAVES, qblocks = (T * 64 + 2 * FL_WAVES - 1) / (2 * FL_WAVES);
        for (int b = blockIdx.x; b < rblocks + qblocks; b += nblocks) {
            if (b < rblocks) {
                // A wave per router row with the row in registers; the window's x comes through LDS in two halves of
                // 1024 columns, the second half's loads in flight while the first is used: about one memory round trip
                // in all. Sums in the fixed order of k_gemv_rows (and of the CPU oracle): lane l takes float4 chunks
                // l, l + 64, ... in order, fmaf over x, y, z, w; then the xor-butterfly.
                float4(*xt)[4][64] = reinterpret_cast<float4(*)[4][64]>(L.tab);   // [token][chunk][lane], over tab and a
                static_assert(sizeof(float4) * FNX_MAXT * 4 * 64 <= sizeof(L.tab) + sizeof(L.a), "half of x fits the stage");
                const int row = b * FL_WAVES + wave;
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
                // thread -> 8 float4 of a half: token q / 32 ... : item i = tid + k * 512 over [token][chunk][lane]
                auto load_half = [&](int h, float4(&xr)[8]) {
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        const int i = tid + k * FL_THREADS, t = i >> 8, c = (i >> 6) & 3, l = i & 63;
                        xr[k] = t < T ? reinterpret_cast<const float4*>(a.x + (size_t) t * n)[(4 * h + c) * 64 + l] : make_float4(0.f, 0.f, 0.f, 0.f);
                    }
                };
                float acc[FNX_MAXT];
#pragma unroll
                for (int t = 0; t < FNX_MAXT; ++t) acc[t] = 0.f;
                float4 xr[8];
                load_half(0, xr);
                __syncthreads();   // a previous pass of this loop may still be reading the stage
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
                        for (int t = 0; t < FNX_MAXT; ++t)
                            if (t < T) {
                                const float4 bx = xt[t][c][lane];
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
#pragma unroll
                for (int t = 0; t < FNX_MAXT; ++t)
                    if (t < T) {
                        const float v = group_sum<64>(acc[t]);
                        if (live && lane == 0) a.logits[(size_t) t * LS + row] = v;
                    }
            } else {
                const int qb = (b - rblocks) * 2 * FL_WAVES + wave * 2 + (lane >> 5);
                if (qb < T * 64) {
                    const int t = qb >> 6, blk = qb & 63;
                    const float xi = a.x[(size_t) t * n + blk * 32 + (lane & 31)];
                    q8_1_store(xi, a.xq + (size_t) qb * FNX_Q8_1_BLOCK, lane & 31);
                }
            }
        }
    }
    layer_stamp(1);

    // ------------------------------------------------------------ the block that arrives last routes for everybody;
    // the others wait for its word, having filled their codebook meanwhile
    __syncthreads();
    if (tid == 0) {
        __threadfence();
        L.last = atomicAdd(&a.sync[0], 1u) == nblocks - 1;
        if (L.last) __threadfence();
        ++epoch;
    }
    for (int i = tid; i < SGRID_WORDS; i += FL_THREADS) L.tab[i] = g_sgrid.v[i];
    __syncthreads();
    if (L.last) {
        route_block(a, L);
        __syncthreads();
        if (tid == 0) {
            __threadfence();
            __hip_atomic_store(&a.sync[3], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    } else {
        if (tid == 0) {
            spin_until(&a.sync[3], 1u, &a.sync[2]);
            __threadfence();
        }
        __syncthreads();
        for (int i = tid; i < (int) (sizeof(LayerPlan) / 4); i += FL_THREADS) reinterpret_cast<int*>(&L.plan)[i] = reinterpret_cast<const int*>(&g_layer_plan)[i];
    }
    for (int i = tid; i < T * 64 * FNX_Q8_1_BLOCK / 4; i += FL_THREADS) reinterpret_cast<int*>(L.a)[i] = reinterpret_cast<const int*>(a.xq)[i];
    __syncthreads();
    layer_stamp(2);
    const LayerPlan& pl = L.plan;
    const int npass = pl.npass;
    const long gw = (long) blockIdx.x * FL_WAVES + wave, nw = (long) nblocks * FL_WAVES;

    // ------------------------------------------------------------ phase 3: gate|up, routed and shared
    {
        const int upj = 2 * ff;   // a unit is a row of 2048 columns
        const long total = (long) npass * upj;
        long u = total * gw / nw;
        const long u1 = total * (gw + 1) / nw;
        while (u < u1) {
            const int pi = (int) (u / upj), ul = (int) (u % upj);
            const int ue = (int) min((long) upj, ul + (u1 - u));
            const int ji = uniform((int) pl.pass_job[pi]), t0 = uniform((int) pl.pass_t0[pi]);
            const int w = uniform(pl.job_w[ji]), nt = uniform((int) pl.job_n[ji]) - t0;
            const uint8_t* we = w < 0 ? a.sh_gu : a.gu_ep ? uniform_ptr(a.gu_ep[w]) : a.gu + (size_t) w * a.gu_stride;
            const uint8_t* pairs = pl.job_pairs[ji] + t0;
            const uint8_t* pair_tok = pl.pair_tok;
            const uint8_t* xq = L.a;
            auto prep_for = [&](auto nt_tag) {
                constexpr int NT = decltype(nt_tag)::value;
                return [=](int(&xs)[NT][8], float(&dx)[NT], float*(&orow)[NT]) {
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        const int pair = uniform((int) pairs[t]), tok = uniform((int) pair_tok[pair]);
                        const uint8_t* yb = xq + (tok * 64 + lane) * FNX_Q8_1_BLOCK;
                        dx[t] = half_bits_to_float(*reinterpret_cast<const unsigned short*>(yb));
#pragma unroll
                        for (int j = 0; j < 8; ++j) xs[t][j] = reinterpret_cast<const int*>(yb + 4)[j];
                        orow[t] = a.gu_out + (size_t) pair * 2 * ff;
                    }
                };
            };
            if (nt >= 2) packed_units<64, 2>(L.tab, we, ul, ue, prep_for(std::integral_constant<int, 2>{}));
            else packed_units<64, 1>(L.tab, we, ul, ue, prep_for(std::integral_constant<int, 1>{}));
            u += ue - ul;
        }
    }
    layer_stamp(3);
    grid_sync(a.sync, nblocks, epoch);
    layer_stamp(4);

    // ------------------------------------------------------------ phase 5: down, routed and shared. A wave makes the
    // q8_1 form of h = silu(gate) * up for its pass's pairs itself (k_moe_down without PRE, moe.cuh:630-641): the
    // 64 / SBR_D lanes that share a sub-block column split its 32 values.
    {
        constexpr int RW = 64 / SBR_D, VPL = 32 / RW;   // rows per unit; h values a lane makes
        const int upj = n / RW;
        const long total = (long) npass * upj;
        long u = total * gw / nw;
        const long u1 = total * (gw + 1) / nw;
        const int g = lane / SBR_D, kb = lane % SBR_D;
        while (u < u1) {
            const int pi = (int) (u / upj), ul = (int) (u % upj);
            const int ue = (int) min((long) upj, ul + (u1 - u));
            const int ji = uniform((int) pl.pass_job[pi]), t0 = uniform((int) pl.pass_t0[pi]);
            const int w = uniform(pl.job_w[ji]), nt = uniform((int) pl.job_n[ji]) - t0;
            const uint8_t* we = w < 0 ? a.sh_dn : a.dn_ep ? uniform_ptr(a.dn_ep[w]) : a.dn + (size_t) w * a.dn_stride;
            const uint8_t* pairs = pl.job_pairs[ji] + t0;
            auto prep_for = [&](auto nt_tag) {
                constexpr int NT = decltype(nt_tag)::value;
                return [=](int(&xs)[NT][8], float(&dx)[NT], float*(&orow)[NT]) {
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        const int pair = uniform((int) pairs[t]);
                        const float* gp = a.gu_out + (size_t) pair * 2 * ff + kb * 32 + g * VPL;
                        float h[VPL];
                        float amax = 0.f;
#pragma unroll
                        for (int j = 0; j < VPL; j += 4) {
                            const float4 gv = *reinterpret_cast<const float4*>(gp + j), uv = *reinterpret_cast<const float4*>(gp + ff + j);
                            h[j] = silu_f(gv.x) * uv.x;
                            h[j + 1] = silu_f(gv.y) * uv.y;
                            h[j + 2] = silu_f(gv.z) * uv.z;
                            h[j + 3] = silu_f(gv.w) * uv.w;
                        }
#pragma unroll
                        for (int j = 0; j < VPL; ++j) amax = fmaxf(amax, fabsf(h[j]));
#pragma unroll
                        for (int o = SBR_D; o < 64; o <<= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
                        const float d = amax / 127.0f;
                        int pk[VPL / 4];
#pragma unroll
                        for (int j = 0; j < VPL; j += 4) {
                            uint32_t v = 0;
#pragma unroll
                            for (int k = 0; k < 4; ++k) {
                                const int q = amax == 0.0f ? 0 : (int) (int8_t) roundf(h[j + k] / d);
                                v |= ((uint32_t) q & 0xFFu) << (8 * k);
                            }
                            pk[j / 4] = (int) v;
                        }
#pragma unroll
                        for (int gg = 0; gg < RW; ++gg)
#pragma unroll
                            for (int k = 0; k < VPL / 4; ++k) xs[t][gg * (VPL / 4) + k] = __shfl(pk[k], kb + SBR_D * gg, 64);
                        dx[t] = half_bits_to_float(float_to_half_bits(d));
                        orow[t] = a.part + (size_t) pair * n;
                    }
                };
            };
            if (nt >= 2) packed_units<SBR_D, 2>(L.tab, we, ul, ue, prep_for(std::integral_constant<int, 2>{}));
            else packed_units<SBR_D, 1>(L.tab, we, ul, ue, prep_for(std::integral_constant<int, 1>{}));
            u += ue - ul;
        }
    }
    layer_stamp(5);
    grid_sync(a.sync, nblocks, epoch);
    layer_stamp(6);

    // ------------------------------------------------------------ phase 6: combine (kernels.cu:412-419)
    for (long i = (long) blockIdx.x * FL_THREADS + tid; i < (long) T * n; i += (long) nblocks * FL_THREADS) {
        const int t = (int) (i / n), c = (int) (i % n);
        float s = 0.f;
        for (int k = 0; k < a.topk; ++k) s = fmaf(a.topw[t * a.topk + k], a.part[((size_t) t * a.topk + k) * n + c], s);
        a.out[i] = s + sigmoid_f(a.logits[(size_t) t * LS + a.nexp]) * a.part[((size_t) P + t) * n + c];
    }
    layer_stamp(7);

    // the last block out leaves the barrier words at zero for the next launch
    __syncthreads();
    if (tid == 0) {
        if (atomicAdd(&a.sync[1], 1u) == nblocks - 1) {
            a.sync[0] = 0u;
            a.sync[1] = 0u;
            a.sync[3] = 0u;
            __threadfence();
        }
    }
}

}  // namespace fnx
