// Jobs of many rows over tile16 matrices, on the matrix cores, with no decoded weight in LDS.
//
// k_iq3s_jobs_mma (unit64: a lane = a sub-block of one row) has to turn its decoded rows by way of LDS before the matrix
// cores can take 16 rows of a sub-block at once, and the 16 waves' partial sums meet there too: the LDS is its limit.
// The prompt path's layout gives lane (r, g) of a wave four consecutive sub-blocks of row r of a tile of 16 rows - at
// step p sub-block 4 g + p of the tile's 16 - which is the A operand of v_mfma_i32_16x16x64_i8 as it is decoded: row r,
// lane group g, 16 bytes, two instructions a sub-block. The four lane groups then hold four different sub-blocks, whose
// integer sums must not meet before they have taken their scales; so a step multiplies four times, each time with the
// activations of three lane groups zeroed (the matrix core is idle most of the time anyway). What is left for the LDS:
// the codebook lookups, the job's int8 activations (staged once a job, 32 bytes a lane and step), and the sixteen rows'
// scales of a sub-block, which go from the decoding lanes (row r) to the accumulator's (rows 4 G .. 4 G + 3) through a
// few words of the wave's own. A wave takes whole tiles of 16 rows and all the columns: no sums to add between waves,
// no barrier but those around a job's staging.
// out[job.out[j]][r] = W[job.w][r] . y[job.y[j]] as kernels.hpp:49 and moe.cuh:613-658 define it, a term as in
// k_iq3s_jobs_mma: d_w (1 + 2 s) d_x sumi; a row's sub-blocks are added in the order the steps and lane groups give them
// (16 S + p + 4 g for S, then p, then g ascending), whatever the job's rows are.
#pragma once

#include "k_prefill.h"

namespace fnx {

constexpr int J16_THREADS = 1024, J16_WAVES = 16, J16_MAXCOLS = 2048;
constexpr int J16_XLD = J16_MAXCOLS + 16;   // bytes of a token's int8 row in LDS: 16 lanes' 16-byte reads of one sub-block then fall on all 64 banks
typedef int j16_v4i __attribute__((ext_vector_type(4)));
struct J16Lds {
    uint32_t tab[SGRID_WORDS];
    __attribute__((aligned(16))) uint8_t xq[FNX_MAXT * J16_XLD];
    __attribute__((aligned(16))) float dx[(J16_MAXCOLS / 128) * FNX_MAXT * 4];   // [super-step][step p][token][lane group g]: the activations' block scales
    __attribute__((aligned(16))) float sw[J16_WAVES][4][16];                     // [wave][lane group][row]: a step's weight scales d (1 + 2 s)
};

// tiles [g0, g1) of 16 rows of matrix `we` (ncols columns) against the job's tokens, staged in L: the whole block
__device__ __forceinline__ void j16_segment(J16Lds& L, const uint8_t* __restrict__ we, int g0, int g1, int ncols, const fnx_job* __restrict__ jb, int n,
                                            float* __restrict__ out, int out_stride) {
    const int lane = threadIdx.x & 63, wave = uniform((int) (threadIdx.x >> 6));
    const int r = lane & 15, grp = lane >> 4;   // decoding: row r of the tile, lane group grp; accumulating: token r, rows 4 grp .. 4 grp + 3
    const int nsuper = ncols / 512;
    const uint32_t keep[4] = {grp == 0 ? ~0u : 0u, grp == 1 ? ~0u : 0u, grp == 2 ? ~0u : 0u, grp == 3 ? ~0u : 0u};
    float* orow = out + (size_t) (r < n ? jb->out[r] : 0) * out_stride + 4 * grp;
    const uint8_t* xrow = L.xq + r * J16_XLD + 128 * grp;   // sub-block 16 S + 4 grp + p of token r lies 512 S + 32 p further
    float* myw = &L.sw[wave][grp][r];
    for (int g = g0 + wave; g < g1; g += J16_WAVES) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        SuperFields f = tile16_load(we, 16 * g + r, 0, nsuper);
        for (int S = 0; S < nsuper; ++S) {
            // the next super-step's fields (past the tile's last: the next tile of this wave, or this one again)
            const int gn = S + 1 < nsuper ? g : (g + J16_WAVES < g1 ? g + J16_WAVES : g);
            const SuperFields nf = tile16_load(we, 16 * gn + r, S + 1 < nsuper ? S + 1 : 0, nsuper);
            auto step = [&](auto p_c) {
                constexpr int p = decltype(p_c)::value;
                const SubFields s = super_sub<p>(f);
                const v4u idx = {s.q0, s.q1, s.q2, s.q3};
                v4u lo, hi;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    lo[j] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint8_t*>(L.tab) + packed_addr(idx, j));
                    hi[j] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint8_t*>(L.tab) + packed_addr(idx, 4 + j));
                }
                *myw = half_bits_to_float(s.d) * (float) (int) (1u + 2u * s.sc);
                const v4u b0 = *reinterpret_cast<const v4u*>(xrow + 512 * S + 32 * p), b1 = *reinterpret_cast<const v4u*>(xrow + 512 * S + 32 * p + 16);
                const float4 dxv = *reinterpret_cast<const float4*>(&L.dx[((S * 4 + p) * FNX_MAXT + r) * 4]);
                const float dxs[4] = {dxv.x, dxv.y, dxv.z, dxv.w};
#pragma unroll
                for (int gs = 0; gs < 4; ++gs) {   // lane group gs's sub-block: the other groups' activations zeroed
                    const v4u m0 = {b0.x & keep[gs], b0.y & keep[gs], b0.z & keep[gs], b0.w & keep[gs]};
                    const v4u m1 = {b1.x & keep[gs], b1.y & keep[gs], b1.z & keep[gs], b1.w & keep[gs]};
                    j16_v4i d = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(j16_v4i, lo), __builtin_bit_cast(j16_v4i, m0), j16_v4i{0, 0, 0, 0}, 0, 0, 0);
                    d = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(j16_v4i, hi), __builtin_bit_cast(j16_v4i, m1), d, 0, 0, 0);
                    const float4 fw = *reinterpret_cast<const float4*>(&L.sw[wave][gs][4 * grp]);
                    acc[0] = fmaf(fw.x * dxs[gs], (float) d[0], acc[0]);
                    acc[1] = fmaf(fw.y * dxs[gs], (float) d[1], acc[1]);
                    acc[2] = fmaf(fw.z * dxs[gs], (float) d[2], acc[2]);
                    acc[3] = fmaf(fw.w * dxs[gs], (float) d[3], acc[3]);
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
__global__ void __launch_bounds__(J16_THREADS) k_iq3s_jobs_mma16(const RowsArgs a) {
    __shared__ J16Lds L;
    for (int g = threadIdx.x; g < 512; g += J16_THREADS) {   // a code's sixteen signed entries from its unsigned one
        const uint32_t g0 = g_sgrid.v[g];
#pragma unroll
        for (int sg = 0; sg < 16; ++sg) L.tab[sg * 512 + g] = signed_entry(g0, sg);
    }
    const int nj = a.njobs ? min(uniform(*a.njobs), a.njobs_max) : a.njobs_max;
    const uint32_t gpj = (uint32_t) a.nrows / 16;   // items per job
    const unsigned long long total = (unsigned long long) nj * gpj;
    uint32_t i = (uint32_t) (total * blockIdx.x / gridDim.x);
    const uint32_t i1 = (uint32_t) (total * (blockIdx.x + 1) / gridDim.x);
    const uint8_t* y = a.y ? a.y : g_moe_hq;
    const int nsb = a.ncols / 32;
    while (i < i1) {
        const uint32_t ji = i / gpj;
        const int g0 = (int) (i - ji * gpj), g1 = (int) min(gpj, g0 + (i1 - i));
        const fnx_job* jb = a.jobs + ji;
        const int n = uniform(min(jb->n, FNX_MAXT)), w = uniform(jb->w);
        const uint8_t* we = a.ep ? uniform_ptr(a.ep[w]) : a.wbase + (size_t) w * a.w_stride;
        __syncthreads();   // the job before has been read (and the codebook written)
        for (int q = threadIdx.x; q < FNX_MAXT * nsb; q += J16_THREADS) {   // (token, sub-block): its 32 int8 and its scale
            const int t = q / nsb, sb = q - t * nsb;
            uint32_t v[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
            float d = 0.f;
            if (t < n) {
                const uint8_t* yb = y + ((size_t) jb->y[t] * nsb + sb) * FNX_Q8_1_BLOCK;
                d = half_bits_to_float(*reinterpret_cast<const unsigned short*>(yb));
#pragma unroll
                for (int k = 0; k < 8; ++k) v[k] = *reinterpret_cast<const uint32_t*>(yb + 4 + 4 * k);
            }
            uint32_t* dst = reinterpret_cast<uint32_t*>(L.xq + t * J16_XLD + 32 * sb);
#pragma unroll
            for (int k = 0; k < 8; ++k) dst[k] = v[k];
            L.dx[(((sb >> 4) * 4 + (sb & 3)) * FNX_MAXT + t) * 4 + ((sb >> 2) & 3)] = d;
        }
        __syncthreads();
        if (n >= 1) j16_segment(L, we, g0, g1, a.ncols, jb, n, a.out, a.out_stride);
        i += (uint32_t) (g1 - g0);
    }
}

}  // namespace fnx
