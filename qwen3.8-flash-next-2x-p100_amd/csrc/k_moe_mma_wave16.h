// The routed experts' down projection on the matrix cores over tile16 matrices of 512 columns, a wave a tile of 16 rows.
//
// A block that takes one (job, 256 rows) task at a time, its activations staged per step, meets at two barriers a stage:
// with rows of 512 columns a task is a single stage, the eight waves of such a block meet four times per 32 rows each, and
// at two waves a SIMD little covers the codebook lookups' latency. Here the whole activation tile of a job - up to 64 tokens x 512
// columns of f16, 64 KiB - is put in LDS once (by loads that write LDS directly, a token's row per wave instruction), and
// after that a wave needs nothing from the others: it takes tiles of 16 rows, a lane decodes its four sub-blocks of its
// row from one contiguous load of the tile16 layout, and the sixteen waves of a block (four a SIMD) meet only where the
// block goes from one job to the next. The blocks split the (job, sixteen tiles) units of all jobs by cost - a tile's
// decode and its job's token tiles of multiplications - into contiguous runs.
// part[job.out[t]][row] = W[job.w][row] . h16[job.y[t]] as kernels.hpp:330 (moe_down_mma) defines it, with the weights as
// f16 (d (1 + 2 s) g, the f32 value rounded once, as k_moe_mma rounds it) and a row's sub-blocks accumulated super-step by
// super-step (S, then the four steps, then a step's four operands).
#pragma once

#include "k_prefill.h"

namespace fnx {

constexpr int W16_THREADS = 1024, W16_WAVES = 16, W16_COLS = 512;
constexpr int W16_XROW = 2 * W16_COLS + 16;   // bytes of a token's f16 row in LDS (260 words: the 16 tokens of a 16-byte operand read fall on 64 different banks)
constexpr int W16_DEC = 3, W16_MUL = 1;   // an item's cost: W16_DEC for its decode and W16_MUL a token tile of its job (measured: 2.7 us a round of
                                          // sixteen tiles with one token tile, 4.7 us with four)
constexpr int W16_HELD = 2048;  // jobs of a list whose token counts and matrices are read into LDS at once, ahead of the split
struct Wave16Lds {
    uint2 tab[SGRID_WORDS];
    __attribute__((aligned(16))) uint8_t xt[MB_TOK64 * W16_XROW];
    int first_job, first_tile, last_job, last_tile;   // the block's run: from (first_job, first_tile) up to but not including (last_job, last_tile)
    uint8_t jn[2][W16_HELD];                          // the token counts of the two lists' jobs, as far as they fit
    int jw[W16_HELD];                                 // the first list's matrices
};

// A tile's super-step: the lane's four sub-blocks of its row (fields f) as f16 operands, against the nt token tiles of
// the activation tile in LDS (xlane: token r's row at this lane group's sub-blocks), added to acc
__device__ __forceinline__ void w16_super_step(const uint2* tab, const uint8_t* xlane, const SuperFields& f, int nt, v4f (&acc)[MB_TP]) {
    // the token tiles two at a time against the sub-block's operands
    auto pair = [&](const v8h (&A)[4], int p, auto t0_tag, auto cnt_tag) {
        constexpr int T0 = decltype(t0_tag)::value, CNT = decltype(cnt_tag)::value;
#pragma unroll
        for (int h = 0; h < 2; ++h) {   // two of the four operands at a time: the registers of a block of 1024 threads
            v4u B[2][2];
#pragma unroll
            for (int tt = 0; tt < CNT; ++tt)
#pragma unroll
                for (int i = 0; i < 2; ++i) B[tt][i] = *reinterpret_cast<const v4u*>(xlane + (T0 + tt) * 16 * W16_XROW + 64 * p + 32 * h + 16 * i);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int tt = 0; tt < CNT; ++tt)
                    acc[T0 + tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[2 * h + i], __builtin_bit_cast(v8h, B[tt][i]), acc[T0 + tt], 0, 0, 0);
        }
    };
    auto step = [&](auto p_c) {
        constexpr int p = decltype(p_c)::value;
        const SubFields s = super_sub<p>(f);
        const _Float16 sc = (_Float16) (int) (1 + 2 * s.sc), d = __builtin_bit_cast(_Float16, (unsigned short) s.d);
        const v2h s2 = {sc, sc}, d2 = {d, d};
        v8h A[4];   // the lane's sub-block (row r, 4 grp + p) as 32 f16 weights
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const uint2 en = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint8_t*>(tab) + sub_entry<true>(s, k));
            const v2h lo = (as_v2h(en.x) * s2) * d2, hi = (as_v2h(en.y) * s2) * d2;
            A[k >> 1][4 * (k & 1) + 0] = lo.x;
            A[k >> 1][4 * (k & 1) + 1] = lo.y;
            A[k >> 1][4 * (k & 1) + 2] = hi.x;
            A[k >> 1][4 * (k & 1) + 3] = hi.y;
        }
        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        using I2 = std::integral_constant<int, 2>;
        if (nt >= 2) pair(A, p, I0{}, I2{});
        else pair(A, p, I0{}, I1{});
        if (nt == 3) pair(A, p, I2{}, I1{});
        else if (nt == 4) pair(A, p, I2{}, I2{});
    };
    step(std::integral_constant<int, 0>{});
    step(std::integral_constant<int, 1>{});
    step(std::integral_constant<int, 2>{});
    step(std::integral_constant<int, 3>{});
}

__global__ void __launch_bounds__(W16_THREADS) k_moe_mma_wave16(const MmaArgs a) {
    // the block's place in the plan: blocks with neighbouring places run on one XCD (workgroups go to the eight XCDs in turn), so
    // the units of one expert, which the plan deals to neighbouring places, find the expert's weights in that XCD's L2
    const unsigned vb = gridDim.x % 8 == 0 ? (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8 : blockIdx.x;
    __shared__ Wave16Lds L;
    const int tid = threadIdx.x, lane = tid & 63, wave = uniform(tid >> 6), r = lane & 15, grp = lane >> 4;
    // every job's token count and matrix, a thread a job, both lists at once (entries past a list's count are read too - the
    // arrays hold cap jobs - and not used): one round of loads instead of dependent ones wherever a job's turn comes
    // (asked for ahead of the codebook's entries, made meanwhile)
    int hn[2] = {0, 0}, hn2 = 0, hw[2] = {0, 0};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int j = tid + i * W16_THREADS;
        if (j < min(a.cap, W16_HELD)) hn[i] = a.jobs[j].n, hw[i] = a.jobs[j].w;
    }
    if (a.jobs2 && tid < min(a.cap2, W16_HELD)) hn2 = a.jobs2[tid].n;
    const int nj_raw = *a.njobs, nj2_raw = a.jobs2 ? *a.njobs2 : 0;
    {
        const uint32_t tab0 = g_sgrid.v[tid & 511];   // a thread's code: its sixteen signed entries are made here
#pragma unroll
        for (int i = tid; i < SGRID_WORDS; i += W16_THREADS) {
            const uint32_t g = signed_entry(tab0, i >> 9);
            v2h lo, hi;
            lo.x = (_Float16) (int) (int8_t) (g & 0xFFu);
            lo.y = (_Float16) (int) (int8_t) ((g >> 8) & 0xFFu);
            hi.x = (_Float16) (int) (int8_t) ((g >> 16) & 0xFFu);
            hi.y = (_Float16) (int) (int8_t) (g >> 24);
            L.tab[i] = make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
        }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int j = tid + i * W16_THREADS;
        if (j < min(a.cap, W16_HELD)) L.jn[0][j] = (uint8_t) max(0, min(FNX_PF_JOB, hn[i])), L.jw[j] = hw[i];
    }
    if (a.jobs2) {
        if (tid < min(a.cap2, W16_HELD)) L.jn[1][tid] = (uint8_t) max(0, min(FNX_PF_JOB, hn2));
        for (int j = tid + W16_THREADS; j < min(a.cap2, W16_HELD); j += W16_THREADS) L.jn[1][j] = (uint8_t) max(0, min(FNX_PF_JOB, a.jobs2[j].n));
    }
    const int nj = min(a.cap, uniform(nj_raw)), nj2 = a.jobs2 ? min(a.cap2, uniform(nj2_raw)) : 0, njall = nj + nj2;
    const int gpj = a.nrows >> 4;   // items a job
    // a unit: a tile for every wave of the block - or, where that would leave blocks without work, a single tile
    const int ut = (long) njall * ((gpj + W16_WAVES - 1) / W16_WAVES) >= 2l * gridDim.x ? W16_WAVES : 1, upj = (gpj + ut - 1) / ut;
    auto job_at = [&](int j) { return j < nj ? a.jobs + j : a.jobs2 + (j - nj); };
    auto n_of = [&](int j) {   // job j's tokens, 0 .. FNX_PF_JOB
        const int l = j < nj ? 0 : 1, k = j < nj ? j : j - nj;
        return k < W16_HELD ? (int) L.jn[l][k] : max(0, min(FNX_PF_JOB, job_at(j)->n));
    };
    __syncthreads();
    // The block's run of items, in units (a run that ended inside a round of the block's waves would leave most of them
    // waiting for the few). A unit of job j costs w_j = W16_DEC + W16_MUL * (token tiles of j), a job upj * w_j;
    // unit (j, u) begins at (the cost of the jobs before j) + u * w_j, and block b takes the units that begin in
    // [total * b / blocks, total * (b + 1) / blocks). One wave finds the run: a lane adds up a stretch of jobs, the
    // stretches' sums are added up over the lanes, and the lanes whose stretch holds an end of the run walk it.
    if (wave == 0) {
        auto weight_of = [&](int j) {
            const int n = n_of(j);
            return n >= 1 ? (uint32_t) (W16_DEC + W16_MUL * ((n + 15) >> 4)) : 0u;
        };
        const int per = (njall + 63) >> 6, j0 = min(njall, lane * per), j1 = min(njall, j0 + per);
        unsigned long long sum = 0;
        for (int j = j0; j < j1; ++j) sum += (unsigned long long) weight_of(j) * (uint32_t) upj;
        unsigned long long incl = sum;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const unsigned long long up = __shfl_up(incl, o);
            if (lane >= o) incl += up;
        }
        const unsigned long long total = __shfl(incl, 63);
        unsigned long long c0, c1;   // (64-bit quotients take a few hundred instructions)
        if (total <= 0xFFFFFFFFull / gridDim.x) c0 = (uint32_t) total * vb / gridDim.x, c1 = (uint32_t) total * (vb + 1) / gridDim.x;
        else c0 = total * vb / gridDim.x, c1 = total * (vb + 1) / gridDim.x;
        if (lane == 0) {   // ends that lie past every job's items
            L.first_job = L.last_job = njall;
            L.first_tile = L.last_tile = 0;
        }
        // the first unit that begins at or after a point inside a job (past its last unit: the next job's first, as a tile past gpj)
        auto find = [&](unsigned long long c, int& job, int& tile) {
            unsigned long long at = incl - sum;   // where this lane's stretch begins
            if (!(at <= c && c < at + sum)) return;
            for (int j = j0; j < j1; ++j) {
                const uint32_t w = weight_of(j);
                const unsigned long long cj = (unsigned long long) w * (uint32_t) upj;
                if (c < at + cj) {
                    job = j;
                    tile = ut * (int) ((uint32_t) (c - at + w - 1) / w);
                    return;
                }
                at += cj;
            }
        };
        find(c0, L.first_job, L.first_tile);
        find(c1, L.last_job, L.last_tile);
    }
    __syncthreads();   // the codebook and the run
    const int jA = uniform(L.first_job), tA = uniform(L.first_tile), jB = uniform(L.last_job), tB = uniform(L.last_tile);
    const uint32_t xt_at = (uint32_t) (size_t) (__attribute__((address_space(3))) uint8_t*) L.xt;
    const uint8_t* xlane = L.xt + r * W16_XROW + 256 * grp;   // token r of a tile, this lane group's four sub-blocks of a super-step
    int yahead[MB_TP] = {0, 0, 0, 0}, ahead = -1;
    for (int j = jA; j <= jB && j < njall; ++j) {
        const int g0 = j == jA ? tA : 0, g1 = j == jB ? min(tB, gpj) : gpj;
        const fnx_bigjob* jb = job_at(j);
        const int n = uniform(n_of(j));
        if (n < 1 || g0 >= g1) continue;   // the same for the whole block
        const int nt = (n + 15) >> 4, e = j >= nj ? 0 : uniform(j < W16_HELD ? L.jw[j] : jb->w);
        const uint8_t* we = j >= nj ? a.w2 : a.ep ? uniform_ptr((const uint8_t*) a.ep[e]) : a.w + (size_t) e * a.stride;
        // the wave's tokens' rows, tokens wave, wave + 16, .. (past the job's last: that one again): asked for while the job
        // before was multiplied, if that was the list's job before this one
        int y[MB_TP];
#pragma unroll
        for (int i = 0; i < MB_TP; ++i) y[i] = ahead == j ? yahead[i] : uniform(jb->y[min(wave + 16 * i, n - 1)]);
        __syncthreads();   // the job before has been read
#pragma unroll
        for (int i = 0; i < MB_TP; ++i)   // a token's row a wave instruction, 16 bytes a lane
            if (i < nt) lds_load16(a.x + (size_t) y[i] * a.ldx, 16u * lane, xt_at + (wave + 16 * i) * W16_XROW);
        if (j + 1 <= jB && j + 1 < njall) {
            const int nn = uniform(n_of(j + 1));
            const fnx_bigjob* jn = job_at(j + 1);
#pragma unroll
            for (int i = 0; i < MB_TP; ++i) yahead[i] = uniform(jn->y[max(0, min(wave + 16 * i, nn - 1))]);
            ahead = j + 1;
        }
        int orow[MB_TP];
#pragma unroll
        for (int tt = 0; tt < MB_TP; ++tt) orow[tt] = tt * 16 + r < n ? jb->out[tt * 16 + r] : -1;
        int g = g0 + wave;
        SuperFields f = tile16_load(we, 16 * min(g, g1 - 1) + r, 0, 1);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        for (; g < g1; g += W16_WAVES) {
            // The oldest wave of a SIMD goes first, so a block's waves drift apart and the first ones wait at the job's end
            // for the last: every wave takes every priority in turn, a tile each
            switch (((wave >> 2) + ((g - g0) >> 4)) & 3) {
                case 0: __builtin_amdgcn_s_setprio(0); break;
                case 1: __builtin_amdgcn_s_setprio(1); break;
                case 2: __builtin_amdgcn_s_setprio(2); break;
                default: __builtin_amdgcn_s_setprio(3); break;
            }
            const SuperFields nf = tile16_load(we, 16 * (g + W16_WAVES < g1 ? g + W16_WAVES : g) + r, 0, 1);
            v4f acc[MB_TP];
#pragma unroll
            for (int tt = 0; tt < MB_TP; ++tt) acc[tt] = v4f{0.f, 0.f, 0.f, 0.f};
            w16_super_step(L.tab, xlane, f, nt, acc);
            // lane: token r of each tile, rows 4 grp .. 4 grp + 3 of the tile
#pragma unroll
            for (int tt = 0; tt < MB_TP; ++tt)
                if (orow[tt] >= 0)
                    *reinterpret_cast<float4*>(a.out + (size_t) orow[tt] * a.nrows + 16 * g + 4 * grp) = make_float4(acc[tt].x, acc[tt].y, acc[tt].z, acc[tt].w);
            f = nf;
        }
    }
}

// ---------------------------------------------------------------- the same form for stacked gate|up matrices (rows of 512 S columns)
// A job's activations are S tiles of 64 tokens x 512 columns here, and LDS holds one: a block takes units of (job, sixteen
// gate tiles and the sixteen up tiles that go with them), a wave one such pair, and walks the S super-steps with the
// pair's accumulators in registers - activation tile S in (two barriers), the gate tile's super-step, the up tile's -
// and leaves h = silu(gate) * up as f16 (k_swiglu_h16's values). Such a unit is eight rounds of the down kernel's kind:
// too coarse for runs by cost, and two of even the lightest on one block made the launch half as long again as its mean
// block. So the jobs are ranked by token tiles, the units of those with two token tiles and more dealt heaviest first,
// to and fro over the blocks, and the jobs of up to 16 tokens cut finer - eight pairs a unit, a wave a single tile, all S
// tiles of the 16 tokens in LDS at once, the up tiles' sums handed to the gate tiles' waves through LDS - and spread so
// that every block comes near the mean load. The weights of the next tile's super-step are asked for a tile ahead. Every
// tile is accumulated in one order (S, then the four steps, then a step's four operands) whatever a job's size or the
// unit it falls in: a row's h does not depend on what else is in the chunk.
constexpr int W16_SORTJ = 1024, W16_GU_HELD = 1024, W16_PLAN = 4;   // (W16_PLAN: blocks a lane of the planning wave looks after)
struct Wave16GuLds {
    uint2 tab[SGRID_WORDS];
    __attribute__((aligned(16))) uint8_t xt[MB_TOK64 * W16_XROW];
    __attribute__((aligned(16))) uint8_t xs[8 * 64 * 16];      // the up tiles' sums of a light unit on their way to the gate tiles' waves
    uint8_t jn[2][W16_GU_HELD];
    int jw[W16_GU_HELD];
    unsigned short jorder[W16_SORTJ];   // the jobs, most token tiles first (the lower index first among equals)
    int p_total[MB_TP + 1], p_sumk, p_s0, p_k;   // the jobs by token tiles; the plan where one wave made it: this block's share of the light units
};
__global__ void __launch_bounds__(W16_THREADS) k_moe_mma_wave16_gu(const MmaArgs a) {
    // the block's place in the plan: blocks with neighbouring places run on one XCD (workgroups go to the eight XCDs in turn), so
    // the units of one expert, which the plan deals to neighbouring places, find the expert's weights in that XCD's L2
    const unsigned vb = gridDim.x % 8 == 0 ? (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8 : blockIdx.x;
    __shared__ Wave16GuLds L;
    const int tid = threadIdx.x, lane = tid & 63, wave = uniform(tid >> 6), r = lane & 15, grp = lane >> 4;
    int hn[2] = {0, 0}, hn2 = 0, hw[2] = {0, 0};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int j = tid + i * W16_THREADS;
        if (j < min(a.cap, W16_GU_HELD)) hn[i] = a.jobs[j].n, hw[i] = a.jobs[j].w;
    }
    if (a.jobs2 && tid < min(a.cap2, W16_GU_HELD)) hn2 = a.jobs2[tid].n;
    const int nj_raw = *a.njobs, nj2_raw = a.jobs2 ? *a.njobs2 : 0;
    {
        const uint32_t tab0 = g_sgrid.v[tid & 511];
#pragma unroll
        for (int i = tid; i < SGRID_WORDS; i += W16_THREADS) {
            const uint32_t g = signed_entry(tab0, i >> 9);
            v2h lo, hi;
            lo.x = (_Float16) (int) (int8_t) (g & 0xFFu);
            lo.y = (_Float16) (int) (int8_t) ((g >> 8) & 0xFFu);
            hi.x = (_Float16) (int) (int8_t) ((g >> 16) & 0xFFu);
            hi.y = (_Float16) (int) (int8_t) (g >> 24);
            L.tab[i] = make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
        }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int j = tid + i * W16_THREADS;
        if (j < min(a.cap, W16_GU_HELD)) L.jn[0][j] = (uint8_t) max(0, min(FNX_PF_JOB, hn[i])), L.jw[j] = hw[i];
    }
    if (a.jobs2) {
        if (tid < min(a.cap2, W16_GU_HELD)) L.jn[1][tid] = (uint8_t) max(0, min(FNX_PF_JOB, hn2));
        for (int j = tid + W16_THREADS; j < min(a.cap2, W16_GU_HELD); j += W16_THREADS) L.jn[1][j] = (uint8_t) max(0, min(FNX_PF_JOB, a.jobs2[j].n));
    }
    const int nj = min(a.cap, uniform(nj_raw)), nj2 = a.jobs2 ? min(a.cap2, uniform(nj2_raw)) : 0, njall = nj + nj2;
    const int ffh = a.ffh, nsuper = a.ncols >> 9, ppj = ffh >> 4;                      // pairs of tiles a job
    const int upj = (ppj + W16_WAVES - 1) / W16_WAVES, upj_s = (ppj + 7) / 8;   // units a job: of sixteen pairs, of eight
    auto job_at = [&](int j) { return j < nj ? a.jobs + j : a.jobs2 + (j - nj); };
    auto n_of = [&](int j) {
        const int l = j < nj ? 0 : 1, k = j < nj ? j : j - nj;
        return k < W16_GU_HELD ? (int) L.jn[l][k] : max(0, min(FNX_PF_JOB, job_at(j)->n));
    };
    __syncthreads();
    const bool sorted = njall <= W16_SORTJ;
    if (sorted && wave == 0) {   // a counting sort by one wave, 64 jobs a trip: class totals, then every job's place
        int total[MB_TP + 1];
#pragma unroll
        for (int c = 0; c <= MB_TP; ++c) total[c] = 0;
        for (int j0 = 0; j0 < njall; j0 += 64) {
            const int kj = j0 + lane < njall ? (n_of(j0 + lane) + 15) >> 4 : -1;
#pragma unroll
            for (int c = 0; c <= MB_TP; ++c) total[c] += __popcll(__ballot(kj == c));
        }
        int base[MB_TP + 1];   // where a class starts: the classes in descending order
        base[MB_TP] = 0;
#pragma unroll
        for (int c = MB_TP - 1; c >= 0; --c) base[c] = base[c + 1] + total[c + 1];
        for (int j0 = 0; j0 < njall; j0 += 64) {
            const int kj = j0 + lane < njall ? (n_of(j0 + lane) + 15) >> 4 : -1;
#pragma unroll
            for (int c = 0; c <= MB_TP; ++c) {
                const unsigned long long m = __ballot(kj == c);
                if (kj == c) L.jorder[base[c] + __popcll(m & ((1ull << lane) - 1ull))] = (unsigned short) (j0 + lane);
                base[c] += __popcll(m);
            }
        }
        // The plan. Jobs of two token tiles and more go as units of sixteen pairs (a wave a pair), dealt heaviest first, to
        // and fro over the blocks. Jobs of up to 16 tokens (where a row's S <= 4 activation tiles of 16 tokens fit LDS
        // together) go as units of eight pairs, a wave a single tile, and fill the blocks up to the mean load: block b
        // takes k_b = (mean - its heavy units' cost) / (a light unit's cost) of them, rounded, in the order of the blocks
        // from the last one down (the lightest first); what the rounding leaves over goes one a block in that order.
        const int G = gridDim.x, ome = G - 1 - (int) vb;
        const bool split = nsuper <= 4;
        const int nbj = total[4] + total[3] + total[2] + (split ? 0 : total[1]), nb = nbj * upj, ns = split ? total[1] * upj_s : 0;
        // costs as measured for S = 4 (us: 20 + 5.5 a token tile the heavy unit, 13.5 the light one), in halves of a us
        if (lane == 0) {
#pragma unroll
            for (int c = 0; c <= MB_TP; ++c) L.p_total[c] = total[c];
        }
        const int cs = 27 * nsuper;
        if (nb > G) {   // (heavy units on one block or none: the same plan in closed form, below, by every wave)
        auto big_cost = [&](int u) {
            const int jo = u / upj, nt_ = jo < total[4] ? 4 : jo < total[4] + total[3] ? 3 : jo < total[4] + total[3] + total[2] ? 2 : 1;
            return (40 + 11 * nt_) * nsuper;
        };
        auto load_of = [&](int bb) {   // block bb's heavy units
            int l = 0;
            for (int k = 0; k * G < nb; ++k) {
                const int u = k * G + ((k & 1) ? G - 1 - bb : bb);
                if (u < nb) l += big_cost(u);
            }
            return l;
        };
        // a lane looks after W16_PLAN blocks (a grid of up to 64 W16_PLAN), in the order from the last block down
        const int o0 = lane * W16_PLAN;
        int ld[W16_PLAN], mine_sum = 0;
#pragma unroll
        for (int i = 0; i < W16_PLAN; ++i) {
            ld[i] = o0 + i < G ? load_of(G - 1 - (o0 + i)) : 0;
            mine_sum += ld[i];
        }
#pragma unroll
        for (int sh = 32; sh >= 1; sh >>= 1) mine_sum += __shfl_xor(mine_sum, sh);
        const int mean = (int) (((long) mine_sum + (long) ns * cs + G - 1) / G);
        int kk[W16_PLAN], kl = 0;
#pragma unroll
        for (int i = 0; i < W16_PLAN; ++i) {
            kk[i] = o0 + i < G ? max(0, (mean - ld[i] + cs / 2) / cs) : 0;
            kl += kk[i];
        }
        int incl = kl;
#pragma unroll
        for (int sh = 1; sh < 64; sh <<= 1) {
            const int up = __shfl_up(incl, sh);
            if (lane >= sh) incl += up;
        }
        const int sumk = __shfl(incl, 63);
        if (o0 <= ome && ome < o0 + W16_PLAN) {
            int s0 = incl - kl;
#pragma unroll
            for (int i = 0; i < W16_PLAN; ++i) {
                if (o0 + i < ome) s0 += kk[i];
                if (o0 + i == ome) L.p_k = kk[i];
            }
            L.p_s0 = s0;
        }
        if (lane == 0) L.p_sumk = sumk;
        }
    }
    __syncthreads();   // the codebook, the order and the plan
    const uint32_t xt_at = (uint32_t) (size_t) (__attribute__((address_space(3))) uint8_t*) L.xt;
    const uint8_t* xlane = L.xt + r * W16_XROW + 256 * grp;
    const int G = gridDim.x;
    int tot[MB_TP + 1] = {0, 0, 0, 0, 0};
    if (sorted) {
#pragma unroll
        for (int c = 0; c <= MB_TP; ++c) tot[c] = uniform(L.p_total[c]);
    }
    const bool split = nsuper <= 4;
    const int nbj = sorted ? tot[4] + tot[3] + tot[2] + (split ? 0 : tot[1]) : njall, nb = nbj * upj, ns = sorted && split ? tot[1] * upj_s : 0;
    int sumk, s0, kme;
    if (nb <= G) {
        // every heavy unit on a block of its own, block b's of the class its place in the order says: the blocks of a class
        // take the same number of light units, and the blocks after b (they come first) are counted class by class
        const int cs = 27 * nsuper, b1 = (int) vb + 1;
        const int hi4 = tot[4] * upj, hi3 = hi4 + tot[3] * upj, hi2 = hi3 + tot[2] * upj;   // where the classes end (class 1: nb)
        const int c4 = 84 * nsuper, c3 = 73 * nsuper, c2 = 62 * nsuper, c1 = 51 * nsuper;      // (40 + 11 token tiles) S
        const int mean = (hi4 * c4 + (hi3 - hi4) * c3 + (hi2 - hi3) * c2 + (nb - hi2) * c1 + ns * cs + G - 1) / G;
        auto k_for = [&](int load) { return max(0, (mean - load + cs / 2) / cs); };
        const int k4 = k_for(c4), k3 = k_for(c3), k2 = k_for(c2), k1 = k_for(c1), k0 = k_for(0);
        auto after = [&](int lo, int hi) { return max(0, hi - max(lo, b1)); };   // blocks of [lo, hi) past this one
        s0 = after(nb, G) * k0 + after(hi2, nb) * k1 + after(hi3, hi2) * k2 + after(hi4, hi3) * k3 + after(0, hi4) * k4;
        kme = b1 > nb ? k0 : b1 > hi2 ? k1 : b1 > hi3 ? k2 : b1 > hi4 ? k3 : k4;
        sumk = (G - nb) * k0 + (nb - hi2) * k1 + (hi2 - hi3) * k2 + (hi3 - hi4) * k3 + hi4 * k4;
    } else {
        sumk = sorted ? uniform(L.p_sumk) : 0, s0 = sorted ? uniform(L.p_s0) : 0, kme = sorted ? uniform(L.p_k) : 0;
    }
    // The oldest wave of a SIMD goes first and the block's waves drift apart between two barriers: every wave takes each
    // priority in turn, a super-step each
    auto turn = [&](int S) {
        switch (((wave >> 2) + S) & 3) {
            case 0: __builtin_amdgcn_s_setprio(0); break;
            case 1: __builtin_amdgcn_s_setprio(1); break;
            case 2: __builtin_amdgcn_s_setprio(2); break;
            default: __builtin_amdgcn_s_setprio(3); break;
        }
    };
    auto matrix_of = [&](int j, const fnx_bigjob* jb) {
        const int e = j >= nj ? 0 : uniform(j < W16_GU_HELD ? L.jw[j] : jb->w);
        return j >= nj ? a.w2 : a.ep ? uniform_ptr((const uint8_t*) a.ep[e]) : a.w + (size_t) e * a.stride;
    };
    // ---- the heavy units: sixteen pairs of tiles, a pair a wave
    for (int round = 0; round * G < nb; ++round) {
        const int u = round * G + ((round & 1) ? G - 1 - (int) vb : (int) vb);
        if (u >= nb) continue;   // the same for the whole block
        const int jo = u / upj, q = u - jo * upj, j = sorted ? (int) uniform(L.jorder[jo]) : jo;
        const fnx_bigjob* jb = job_at(j);
        const int n = uniform(n_of(j));
        if (n < 1) continue;
        const int nt = (n + 15) >> 4;
        const uint8_t* we = matrix_of(j, jb);
        const int pr = q * W16_WAVES + wave;   // the wave's pair: gate rows 16 pr .., up rows ffh + 16 pr ..
        const bool mine = pr < ppj;
        const int grow = 16 * min(pr, ppj - 1) + r;
        int y[MB_TP];   // the wave's tokens' rows: tokens wave, wave + 16, .. (past the job's last: that one again)
#pragma unroll
        for (int i = 0; i < MB_TP; ++i) y[i] = uniform(jb->y[min(wave + 16 * i, n - 1)]);
        int orow[MB_TP];
#pragma unroll
        for (int tt = 0; tt < MB_TP; ++tt) orow[tt] = mine && tt * 16 + r < n ? jb->out[tt * 16 + r] : -1;
        v4f accg[MB_TP], accu[MB_TP];
#pragma unroll
        for (int tt = 0; tt < MB_TP; ++tt) accg[tt] = accu[tt] = v4f{0.f, 0.f, 0.f, 0.f};
        SuperFields f = tile16_load(we, grow, 0, nsuper);
        for (int S = 0; S < nsuper; ++S) {
            __syncthreads();   // the tile before has been read
#pragma unroll
            for (int i = 0; i < MB_TP; ++i)   // a token's 512 columns a wave instruction, 16 bytes a lane
                if (i < nt) lds_load16(a.x + (size_t) y[i] * a.ldx + 512 * S, 16u * lane, xt_at + (wave + 16 * i) * W16_XROW);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            turn(S);
            const SuperFields fu = tile16_load(we, ffh + grow, S, nsuper);
            if (mine) w16_super_step(L.tab, xlane, f, nt, accg);
            f = tile16_load(we, grow, min(S + 1, nsuper - 1), nsuper);
            if (mine) w16_super_step(L.tab, xlane, fu, nt, accu);
        }
        // lane: token r of each tile, rows 4 grp .. 4 grp + 3 of the pair's tiles
#pragma unroll
        for (int tt = 0; tt < MB_TP; ++tt)
            if (orow[tt] >= 0) {
                const v4f gt = accg[tt], up = accu[tt];
                uint2 hv;
                hv.x = (uint32_t) float_to_half_bits(silu_f(gt.x) * up.x) | (uint32_t) float_to_half_bits(silu_f(gt.y) * up.y) << 16;
                hv.y = (uint32_t) float_to_half_bits(silu_f(gt.z) * up.z) | (uint32_t) float_to_half_bits(silu_f(gt.w) * up.w) << 16;
                *reinterpret_cast<uint2*>(a.h16 + (size_t) orow[tt] * ffh + 16 * pr + 4 * grp) = hv;
            }
    }
    if (!sorted) return;
    // ---- the light units: eight pairs of tiles, waves 0 .. 7 the gate tiles, 8 .. 15 the up tiles; the job's up to 16 tokens'
    // S tiles all in LDS ([S][token]), so the waves do not meet until the up tiles' sums go over to the gate tiles' waves
    const int ome = G - 1 - (int) vb;
    float4* ex = reinterpret_cast<float4*>(L.xs);
    for (int t = 0;; ++t) {
        const int idx = t < kme ? s0 + t : sumk + (t - kme) * G + ome;
        if (t < kme ? idx >= min(ns, sumk) : idx >= ns) {
            if (t < kme) {   // (this block's share was cut short: on to what is left over, if anything)
                t = kme - 1;
                continue;
            }
            break;
        }
        const int jo = idx / upj_s, q = idx - jo * upj_s, j = (int) uniform(L.jorder[nbj + jo]);
        const fnx_bigjob* jb = job_at(j);
        const int n = uniform(n_of(j));   // 1 .. 16
        const uint8_t* we = matrix_of(j, jb);
        const int pr = q * 8 + (wave & 7), up_wave = wave >> 3;
        const bool mine = pr < ppj;
        const int row = up_wave * ffh + 16 * min(pr, ppj - 1) + r;
        const int y = uniform(jb->y[min(wave, n - 1)]);
        const int orow = mine && !up_wave && r < n ? jb->out[r] : -1;
        SuperFields f = tile16_load(we, row, 0, nsuper);
        __syncthreads();   // the unit before has been read, its sums handed over
        for (int S = 0; S < nsuper; ++S) lds_load16(a.x + (size_t) y * a.ldx + 512 * S, 16u * lane, xt_at + (16 * S + wave) * W16_XROW);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        v4f acc[MB_TP];
#pragma unroll
        for (int tt = 0; tt < MB_TP; ++tt) acc[tt] = v4f{0.f, 0.f, 0.f, 0.f};
        for (int S = 0; S < nsuper; ++S) {
            turn(S);
            const SuperFields nf = tile16_load(we, row, min(S + 1, nsuper - 1), nsuper);
            if (mine) w16_super_step(L.tab, xlane + S * 16 * W16_XROW, f, 1, acc);
            f = nf;
        }
        if (up_wave) ex[(wave & 7) * 64 + lane] = make_float4(acc[0].x, acc[0].y, acc[0].z, acc[0].w);
        __syncthreads();
        if (orow >= 0) {
            const float4 up = ex[wave * 64 + lane];
            const v4f gt = acc[0];
            uint2 hv;
            hv.x = (uint32_t) float_to_half_bits(silu_f(gt.x) * up.x) | (uint32_t) float_to_half_bits(silu_f(gt.y) * up.y) << 16;
            hv.y = (uint32_t) float_to_half_bits(silu_f(gt.z) * up.z) | (uint32_t) float_to_half_bits(silu_f(gt.w) * up.w) << 16;
            *reinterpret_cast<uint2*>(a.h16 + (size_t) orow * ffh + 16 * pr + 4 * grp) = hv;
        }
    }
}

}  // namespace fnx
