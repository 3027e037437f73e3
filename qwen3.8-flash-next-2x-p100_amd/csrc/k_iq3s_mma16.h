// Jobs of many rows over tile16 matrices, on the matrix cores, with no decoded weight in LDS.
//
// k_iq3s_jobs_mma (unit64: a lane = a sub-block of one row) has to turn its decoded rows by way of LDS before the matrix
// cores can take 16 rows of a sub-block at once, and the 16 waves' partial sums meet there too: the LDS is its limit.
// The prompt path's layout gives lane (r, g) of a wave four consecutive sub-blocks of row r of a tile of 16 rows - at
// step p sub-block 4 g + p of the tile's 16. v_mfma_i32_16x16x32_i8 wants a sub-block of 16 rows as lane (r, G): row r,
// bytes 8 G .. 8 G + 7. What the four lane groups hold after a step's decode - four sub-blocks, 32 bytes a lane - is
// that, for all four sub-blocks, up to a 4 x 4 transpose of 8-byte pairs between lane group and register pair: eight
// permlane swaps. Then one MFMA a sub-block gives the 16 x 16 integer sums, which take their scales and are added; no
// decoded weight ever reaches LDS. What is left for the LDS: the codebook lookups, the job's int8 activations (staged
// once a job, four 8-byte reads a lane and step), and the sixteen rows' scales of a sub-block, which go from the
// decoding lanes (row r) to the accumulator's (rows 4 G .. 4 G + 3) through a few words of the wave's own. A wave takes
// whole tiles of 16 rows and all the columns: no sums to add between waves, no barrier but those around a job's staging.
// out[job.out[j]][r] = W[job.w][r] . y[job.y[j]] as kernels.hpp:49 and moe.cuh:613-658 define it, a term as in
// k_iq3s_jobs_mma: d_w (1 + 2 s) d_x sumi; a row's sub-blocks are added in the order the steps give them
// (16 S + p + 4 j for S, then p, then j ascending), whatever the job's rows are.
#pragma once

#include "k_prefill.h"

namespace fnx {

constexpr int J16_THREADS = 1024, J16_WAVES = 16, J16_MAXCOLS = 2048;
constexpr int J16_XLD = J16_MAXCOLS + 32;   // bytes of a token's int8 row in LDS: a wave's 8-byte reads of a sub-block then take the two passes their 512 bytes need
typedef int j16_v4i __attribute__((ext_vector_type(4)));
// x's lanes 32 .. 63 <-> y's lanes 0 .. 31; x's 16-lane rows 1, 3 <-> y's rows 0, 2 (as instructions: see swap32_add)
__device__ __forceinline__ void swap32(uint32_t& x, uint32_t& y) { asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(x), "+v"(y)); }
__device__ __forceinline__ void swap16(uint32_t& x, uint32_t& y) { asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(x), "+v"(y)); }
// The signed codebook twice, entry i's two copies side by side (words 2 i and 2 i + 1): even lanes read the even words,
// odd lanes the odd ones, so the 64 random lookups of a wave instruction are two sets of 32 over 32 banks each.
struct J16Lds {
    uint32_t tab[2 * SGRID_WORDS];
    __attribute__((aligned(16))) uint8_t xq[FNX_MAXT * J16_XLD];
    __attribute__((aligned(16))) float dx[(J16_MAXCOLS / 128) * FNX_MAXT * 4];   // [super-step][step p][token][lane group g]: the activations' block scales
    __attribute__((aligned(16))) float sw[J16_WAVES][4][16];                     // [wave][lane group][row]: a step's weight scales d (1 + 2 s)
};

// tiles [g0, g1) of 16 rows of matrix `we` (ncols columns) against the job's tokens, staged in L: the whole block
__device__ __forceinline__ void j16_segment(J16Lds& L, const uint8_t* __restrict__ we, int g0, int g1, int ncols, const int* __restrict__ outs, int n,
                                            float* __restrict__ out, int out_stride) {
    const int lane = threadIdx.x & 63, wave = uniform((int) (threadIdx.x >> 6));
    const int r = lane & 15, grp = lane >> 4;   // decoding: row r of the tile, lane group grp; accumulating: token r, rows 4 grp .. 4 grp + 3
    const int nsuper = ncols / 512;
    float* orow = out + (size_t) (r < n ? outs[r] : 0) * out_stride + 4 * grp;
    const uint8_t* xrow = L.xq + r * J16_XLD + 8 * grp;   // bytes 8 grp .. of sub-block 16 S + 4 j + p of token r lie 512 S + 128 j + 32 p further
    float* myw = &L.sw[wave][grp][r];
    const uint32_t copy_at = 4u * (lane & 1);
    if (g0 + wave >= g1) return;
    // the fields of the super-step at hand; a tile's last super-step leaves the next tile's first ones here
    SuperFields f = tile16_load(we, 16 * (g0 + wave) + r, 0, nsuper);
    for (int g = g0 + wave; g < g1; g += J16_WAVES) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        for (int S = 0; S < nsuper; ++S) {
            // the next super-step's fields (past the tile's last: the next tile of this wave, or this one again)
            const int gn = S + 1 < nsuper ? g : (g + J16_WAVES < g1 ? g + J16_WAVES : g);
            const SuperFields nf = tile16_load(we, 16 * gn + r, S + 1 < nsuper ? S + 1 : 0, nsuper);
            auto step = [&](auto p_c) {
                constexpr int p = decltype(p_c)::value;
                const SubFields s = super_sub<p>(f);
                const v4u idx = {s.q0, s.q1, s.q2, s.q3};
                uint32_t w8[8];   // this lane's sub-block (row r, 16 S + 4 grp + p): 32 int8
#pragma unroll
                for (int j = 0; j < 8; ++j) w8[j] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint8_t*>(L.tab) + 2 * packed_addr(idx, j) + copy_at);
                *myw = half_bits_to_float(s.d) * (float) (int) (1u + 2u * s.sc);
                long b[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) b[j] = *reinterpret_cast<const long*>(xrow + 512 * S + 128 * j + 32 * p);
                const float4 dxv = *reinterpret_cast<const float4*>(&L.dx[((S * 4 + p) * FNX_MAXT + r) * 4]);
                const float dxs[4] = {dxv.x, dxv.y, dxv.z, dxv.w};
                // pair P_k = bytes 8 k .. 8 k + 7 of the lane's sub-block; afterwards pair j holds bytes 8 grp .. of lane group j's
                swap32(w8[0], w8[4]);
                swap32(w8[1], w8[5]);
                swap32(w8[2], w8[6]);
                swap32(w8[3], w8[7]);
                swap16(w8[0], w8[2]);
                swap16(w8[1], w8[3]);
                swap16(w8[4], w8[6]);
                swap16(w8[5], w8[7]);
#pragma unroll
                for (int j = 0; j < 4; ++j) {   // lane group j's sub-block, 16 S + 4 j + p
                    const long a = (long) ((unsigned long) w8[2 * j] | (unsigned long) w8[2 * j + 1] << 32);
                    const j16_v4i d = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b[j], j16_v4i{0, 0, 0, 0}, 0, 0, 0);
                    const float4 fw = *reinterpret_cast<const float4*>(&L.sw[wave][j][4 * grp]);
                    acc[0] = fmaf(fw.x * dxs[j], (float) d[0], acc[0]);
                    acc[1] = fmaf(fw.y * dxs[j], (float) d[1], acc[1]);
                    acc[2] = fmaf(fw.z * dxs[j], (float) d[2], acc[2]);
                    acc[3] = fmaf(fw.w * dxs[j], (float) d[3], acc[3]);
                }
            };
            step(std::integral_constant<int, 0>{});
            step(std::integral_constant<int, 1>{});
            step(std::integral_constant<int, 2>{});
            step(std::integral_constant<int, 3>{});
            f = nf;
        }
        if (r < n) {
            float* op = orow + 16 * g;
            op[0] = acc[0], op[1] = acc[1], op[2] = acc[2], op[3] = acc[3];
        }
    }
}

// tile16 matrices of up to 2048 columns (a multiple of 512), rows in 16s. The blocks split the (job, tile of 16 rows) items
// of all jobs evenly and walk them in order; a job's activations are staged when the block comes to it.
// MODE 0: jobs of up to FNX_MAXT rows (kernels.hpp:18-23) over q8_1 rows. MODE 1: the prompt path's jobs of up to
// FNX_PF_JOB rows (kernels.hpp:324, moe_gate_up_big): a job's rows in tiles of sixteen, each (job, token tile) a unit that
// is staged and walked like a job of MODE 0; the units are counted first (a prefix sum over the jobs' tile counts in LDS)
// so that the blocks split live units only. MODE 2 (kernels.hpp:325, moe_down_big): the same with the unit's activations
// made on the way from the rows [gate | up] of 2 ncols floats: h = silu(gate) * up quantised as k_swiglu_q8_1 does it.
constexpr int J16_MAXJOBS = 4096;   // big jobs a launch (their tile counts' prefix sums live in LDS)
template <int MODE>
__global__ void __launch_bounds__(J16_THREADS) k_iq3s_jobs_mma16(const RowsArgs a) {
    __shared__ J16Lds L;
    __shared__ uint32_t before[MODE ? J16_MAXJOBS + 1 : 1];   // units of the jobs before job j
    for (int g = threadIdx.x; g < 512; g += J16_THREADS) {   // a code's sixteen signed entries from its unsigned one
        const uint32_t g0 = g_sgrid.v[g];
#pragma unroll
        for (int sg = 0; sg < 16; ++sg) L.tab[2 * (sg * 512 + g)] = L.tab[2 * (sg * 512 + g) + 1] = signed_entry(g0, sg);
    }
    const int nj = min(a.njobs ? min(uniform(*a.njobs), a.njobs_max) : a.njobs_max, MODE ? J16_MAXJOBS : a.njobs_max);
    const uint32_t gpj = (uint32_t) a.nrows / 16;   // items per unit
    uint32_t units = (uint32_t) nj;
    if constexpr (MODE != 0) {
        // token tiles a job, then their running sum: a wave's lanes take consecutive runs of jobs
        for (int j = threadIdx.x; j < nj; j += J16_THREADS) before[j + 1] = (uint32_t) (min(max(a.big[j].n, 0), FNX_PF_JOB) + 15) / 16;
        if (threadIdx.x == 0) before[0] = 0;
        __syncthreads();
        if (threadIdx.x < 64) {
            const int per = (nj + 63) / 64, j0 = min(nj, (int) threadIdx.x * per), j1 = min(nj, j0 + per);
            uint32_t mine = 0;
            for (int j = j0; j < j1; ++j) mine += before[j + 1];
            uint32_t incl = mine;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const uint32_t v = __shfl_up(incl, o, 64);
                if ((int) threadIdx.x >= o) incl += v;
            }
            uint32_t run = incl - mine;
            for (int j = j0; j < j1; ++j) {
                run += before[j + 1];
                before[j + 1] = run;
            }
        }
        __syncthreads();
        units = before[nj];
    }
    const unsigned long long total = (unsigned long long) units * gpj;
    uint32_t i = (uint32_t) (total * blockIdx.x / gridDim.x);
    const uint32_t i1 = (uint32_t) (total * (blockIdx.x + 1) / gridDim.x);
    const uint8_t* y = a.y ? a.y : g_moe_hq;
    const int nsb = a.ncols / 32;
    while (i < i1) {
        const uint32_t ui = i / gpj;
        const int g0 = (int) (i - ui * gpj), g1 = (int) min(gpj, g0 + (i1 - i));
        int n, w;
        const int *ys, *outs;
        if constexpr (MODE == 0) {
            const fnx_job* jb = a.jobs + ui;
            n = uniform(min(jb->n, FNX_MAXT)), w = uniform(jb->w);
            ys = jb->y, outs = jb->out;
        } else {
            int lo = 0, hi = nj - 1;   // the job whose units hold ui: before[j] <= ui < before[j + 1]
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if (before[mid + 1] <= ui) lo = mid + 1;
                else hi = mid;
            }
            const fnx_bigjob* jb = a.big + uniform(lo);
            const int q = (int) (ui - before[lo]);
            n = uniform(min(min(max(jb->n, 0), FNX_PF_JOB) - 16 * q, FNX_MAXT)), w = uniform(jb->w);
            ys = jb->y + 16 * q, outs = jb->out + 16 * q;
        }
        const uint8_t* we = a.ep ? uniform_ptr(a.ep[w]) : a.wbase + (size_t) w * a.w_stride;
        __syncthreads();   // the unit before has been read (and the codebook written)
        for (int q = threadIdx.x; q < FNX_MAXT * nsb; q += J16_THREADS) {   // (token, sub-block): its 32 int8 and its scale
            const int t = q / nsb, sb = q - t * nsb;
            uint32_t v[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
            float d = 0.f;
            if (t < n) {
                if constexpr (MODE == 2) {
                    const float* gp = a.gu + (size_t) ys[t] * (2 * a.ncols) + 32 * sb;
                    float4 gv[8], uv[8];
#pragma unroll
                    for (int k = 0; k < 8; ++k) gv[k] = reinterpret_cast<const float4*>(gp)[k], uv[k] = reinterpret_cast<const float4*>(gp + a.ncols)[k];
                    float h[32], amax = 0.f;
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        h[4 * k] = silu_f(gv[k].x) * uv[k].x, h[4 * k + 1] = silu_f(gv[k].y) * uv[k].y;
                        h[4 * k + 2] = silu_f(gv[k].z) * uv[k].z, h[4 * k + 3] = silu_f(gv[k].w) * uv[k].w;
                    }
#pragma unroll
                    for (int k = 0; k < 32; ++k) amax = fmaxf(amax, fabsf(h[k]));
                    const float dq = amax / 127.0f;   // q8_1_store's arithmetic (kernels.cu:131-145)
                    d = half_bits_to_float(float_to_half_bits(dq));
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        uint32_t word = 0;
#pragma unroll
                        for (int b = 0; b < 4; ++b) {
                            const int8_t qv = amax == 0.0f ? (int8_t) 0 : (int8_t) roundf(h[4 * k + b] / dq);
                            word |= (uint32_t) (uint8_t) qv << (8 * b);
                        }
                        v[k] = word;
                    }
                } else {
                    const uint8_t* yb = y + ((size_t) ys[t] * nsb + sb) * FNX_Q8_1_BLOCK;
                    d = half_bits_to_float(*reinterpret_cast<const unsigned short*>(yb));
#pragma unroll
                    for (int k = 0; k < 8; ++k) v[k] = *reinterpret_cast<const uint32_t*>(yb + 4 + 4 * k);
                }
            }
            uint32_t* dst = reinterpret_cast<uint32_t*>(L.xq + t * J16_XLD + 32 * sb);
#pragma unroll
            for (int k = 0; k < 8; ++k) dst[k] = v[k];
            L.dx[(((sb >> 4) * 4 + (sb & 3)) * FNX_MAXT + t) * 4 + ((sb >> 2) & 3)] = d;
        }
        __syncthreads();
        if (n >= 1) j16_segment(L, we, g0, g1, a.ncols, outs, n, a.out, a.out_stride);
        i += (uint32_t) (g1 - g0);
    }
}

}  // namespace fnx
