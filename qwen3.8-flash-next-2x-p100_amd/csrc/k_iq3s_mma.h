// Jobs of many rows over unit64 matrices of 2048 columns (a unit = one weight row), on the matrix cores.
//
// The vector-ALU job kernel dots a decoded sub-block with one or two tokens; with sixteen tokens a job that is eight
// decodes of every weight, or sixteen dot products a decode. Here a block of 16 waves takes 16 weight rows at a time:
//   1. wave w decodes row 16 g + w as the mat-vec kernels do (lane = sub-block, 8 codebook lookups: 32 int8 weights a lane)
//      and stores them, the sub-block's integer scale and the row's d in LDS;
//   2. wave w then owns sub-blocks 4 w .. 4 w + 3 of all 16 rows: v_mfma_i32_16x16x32_i8 takes the 16 rows x 32 columns
//      of one sub-block as A (8 bytes a lane from LDS) and the job's up to 16 tokens' int8 activations of that sub-block
//      as B (in registers for the whole job), and leaves every lane four exact integer dot products; each takes its
//      scales (the reference's term (d_w * d_x) * (float) (sumi * (1 + 2 s)), moe.cuh's vec_dot, as d_w (1 + 2 s) * d_x * sumi) and
//      is added to the lane's four sums;
//   3. the waves' sums (each over 128 columns) meet in LDS and one wave adds them in wave order and stores the 16 x 16 tile.
// A weight is decoded once per job whatever the job's rows. Jobs of one row keep the vector-ALU path (its waves
// share a block's run of units). (kernels.hpp:49, moe.cuh:613-658 give the semantics: out[job.out[j]][r] =
// W[job.w][r] . y[job.y[j]].)
#pragma once

#include "k_iq3s_packed.h"

namespace fnx {

constexpr int JM_THREADS = 1024, JM_WAVES = 16, JM_ROWS = 16;
constexpr int JM_ROWLD = 2048 + 32;   // bytes of a decoded row in LDS: 64 sub-blocks x 32 int8, padded so that rows m and m + 1 start 8 banks apart
constexpr int JM_SLD = 20;            // floats of a sub-block's scale record: its 16 rows + 4 (records 16-byte aligned, 20 words apart)
constexpr int JM_MIN = 2;             // rows from which a job goes to the matrix cores (two tokens a pass on the vector ALU does not fit 128 registers with four units in flight)
constexpr int JM_AHEAD = 3;           // units a wave has in flight beyond the one it decodes
typedef int jm_v4i __attribute__((ext_vector_type(4)));

constexpr int JM_NI = 2;   // groups of 16 rows between two barriers: each wave decodes JM_NI rows, then multiplies its sub-blocks of JM_NI tiles
struct JmLds {
    uint32_t tab[SGRID_WORDS];
    __attribute__((aligned(16))) uint8_t tile[JM_NI][JM_ROWS * JM_ROWLD];
    __attribute__((aligned(16))) float sw[JM_NI][64][JM_SLD];   // [sub-block][row]: d (1 + 2 s), exact in f32 (11 + 5 bits): a lane's four rows are one 16-byte read
    __attribute__((aligned(16))) float red[JM_NI][JM_WAVES][64][4];
};

// rows [16 g0, 16 g1) of matrix `we` against the job's tokens: the whole block
__device__ __forceinline__ void jm_segment(JmLds& L, const uint8_t* __restrict__ we, int g0, int g1, const fnx_job* __restrict__ jb, int n,
                                           const uint8_t* __restrict__ y, float* __restrict__ out, int out_stride) {
    const int lane = threadIdx.x & 63, wave = uniform((int) (threadIdx.x >> 6));
    const int col = lane & 15, kg = lane >> 4;   // as B column / accumulator column: token col; as A row: weight row col of the 16
    // the job's activations of this wave's four sub-blocks: token col's bytes 8 kg .. 8 kg + 7 and its block scale
    long xb[4];
    float dx[4];
    {
        const bool on = col < n;
        const uint8_t* yr = y + (size_t) (on ? jb->y[col] : jb->y[0]) * 64 * FNX_Q8_1_BLOCK;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const uint8_t* yb = yr + (size_t) (4 * wave + s) * FNX_Q8_1_BLOCK;
            const uint32_t lo = *reinterpret_cast<const uint32_t*>(yb + 4 + 8 * kg), hi = *reinterpret_cast<const uint32_t*>(yb + 8 + 8 * kg);
            xb[s] = on ? (long) ((unsigned long) lo | (unsigned long) hi << 32) : 0l;
            dx[s] = on ? half_bits_to_float(*reinterpret_cast<const unsigned short*>(yb)) : 0.f;
        }
    }
    float* orow = out + (size_t) (col < n ? jb->out[col] : 0) * out_stride + 4 * kg;   // token col's row of the output, this lane's four rows of a tile
    const PackedVOffs o = packed_voffs(lane);
    const __amdgpu_buffer_rsrc_t mtx = matrix_rsrc(we);
    const int sc_shift = 4 * (lane & 1);
    auto load = [&](int g) { return load_packed_buf(mtx, (JM_ROWS * min(g, g1 - 1) + wave) * UNIT_BYTES, o); };   // past the end: the last group again
    constexpr int RING = JM_AHEAD + 1;
    static_assert(RING % JM_NI == 0, "a round takes whole slots of the ring");
    PackedSub ring[RING];
#pragma unroll
    for (int i = 0; i < RING; ++i) ring[i] = load(g0 + i);
    for (int gb = g0; gb < g1; gb += RING)
#pragma unroll
    for (int rb = 0; rb < RING; rb += JM_NI) {   // the ring's slots in turn: no register moves
        const int g = gb + rb;   // this round: groups g .. g + JM_NI - 1 (those below g1)
        if (g >= g1) break;
        // 1. this wave's row of each group: 32 int8 weights a lane
#pragma unroll
        for (int i = 0; i < JM_NI; ++i) {
            const PackedSub cur = ring[rb + i];
            ring[rb + i] = load(g + i + RING);
            v4u lo, hi;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                lo[j] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint8_t*>(L.tab) + packed_addr(cur.idx, j));
                hi[j] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint8_t*>(L.tab) + packed_addr(cur.idx, 4 + j));
            }
            uint8_t* dst = L.tile[i] + wave * JM_ROWLD + lane * 32;
            *reinterpret_cast<v4u*>(dst) = lo;
            *reinterpret_cast<v4u*>(dst + 16) = hi;
            L.sw[i][lane][wave] = half_bits_to_float(cur.d) * (float) (int) (1u + 2u * ((cur.sc >> sc_shift) & 0xFu));
        }
        __syncthreads();   // the rows are in LDS
        // 2. this wave's four sub-blocks of each group's 16 rows against the tokens
#pragma unroll
        for (int i = 0; i < JM_NI; ++i) {
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int sb = 4 * wave + s;
                const long a = *reinterpret_cast<const long*>(L.tile[i] + col * JM_ROWLD + sb * 32 + 8 * kg);
                const float4 f = *reinterpret_cast<const float4*>(&L.sw[i][sb][4 * kg]);
                const jm_v4i d = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, xb[s], jm_v4i{0, 0, 0, 0}, 0, 0, 0);
                // a term is d_w (1 + 2 s) d_x sumi: the reference's (d_w d_x) (float) (sumi (1 + 2 s)) with the factors taken in another order
                acc[0] = fmaf(f.x * dx[s], (float) d[0], acc[0]);
                acc[1] = fmaf(f.y * dx[s], (float) d[1], acc[1]);
                acc[2] = fmaf(f.z * dx[s], (float) d[2], acc[2]);
                acc[3] = fmaf(f.w * dx[s], (float) d[3], acc[3]);
            }
            *reinterpret_cast<float4*>(L.red[i][wave][lane]) = make_float4(acc[0], acc[1], acc[2], acc[3]);
        }
        __syncthreads();   // the waves' sums are in LDS (and the tiles have been read: the next decode may overwrite them)
        // 3. a wave a group (they take turns) adds the sixteen in wave order and stores the tile
#pragma unroll
        for (int i = 0; i < JM_NI; ++i)
            if (g + i < g1 && wave == ((g + i - g0) & (JM_WAVES - 1)) && col < n) {
                float4 z = *reinterpret_cast<const float4*>(L.red[i][0][lane]);
#pragma unroll
                for (int w = 1; w < JM_WAVES; ++w) {
                    const float4 p = *reinterpret_cast<const float4*>(L.red[i][w][lane]);
                    z.x += p.x, z.y += p.y, z.z += p.z, z.w += p.w;
                }
                float* op = orow + JM_ROWS * (g + i);
                op[0] = z.x, op[1] = z.y, op[2] = z.z, op[3] = z.w;
            }
    }
}

// units [u0, u1) of matrix `we` for a job of one row: the block's waves share them, each a contiguous run
__device__ __forceinline__ void jm_narrow(const uint32_t* tab, const uint8_t* we, int u0, int u1, const fnx_job* jb, const uint8_t* y,
                                          float* out, int out_stride) {
    const int wave = uniform((int) (threadIdx.x >> 6)), per = (u1 - u0 + JM_WAVES - 1) / JM_WAVES;
    const int ua = u0 + wave * per, ub = min(u1, ua + per);
    if (ua >= ub) return;
    PackedSub cur[4];
    packed_first(we, ua, ub, cur);
    packed_units<64, 1>(tab, we, ua, ub, cur, JobPrep<64, 1>{jb, 0, y, out, out_stride});
}

// rows of 2048 columns, a multiple of 16 of them; unit64. The blocks split the (job, 16 rows) items of all jobs evenly and
// walk them in order, so a block streams a contiguous range of memory and changes job a few times at most.
__global__ void __launch_bounds__(JM_THREADS) k_iq3s_jobs_mma(const RowsArgs a) {
    __shared__ JmLds L;
    for (int g = threadIdx.x; g < 512; g += JM_THREADS) {   // a code's sixteen signed entries from its unsigned one
        const uint32_t g0 = g_sgrid.v[g];
#pragma unroll
        for (int sg = 0; sg < 16; ++sg) L.tab[sg * 512 + g] = signed_entry(g0, sg);
    }
    const int nj = a.njobs ? min(uniform(*a.njobs), a.njobs_max) : a.njobs_max;
    __syncthreads();
    const uint32_t gpj = (uint32_t) a.nrows / JM_ROWS;   // items per job
    const unsigned long long total = (unsigned long long) nj * gpj;
    uint32_t i = (uint32_t) (total * blockIdx.x / gridDim.x);
    const uint32_t i1 = (uint32_t) (total * (blockIdx.x + 1) / gridDim.x);
    const uint8_t* y = a.y ? a.y : g_moe_hq;
    while (i < i1) {
        const uint32_t ji = i / gpj;
        const int g0 = (int) (i - ji * gpj), g1 = (int) min(gpj, g0 + (i1 - i));
        const fnx_job* jb = a.jobs + ji;
        const int n = uniform(min(jb->n, FNX_MAXT)), w = uniform(jb->w);
        const uint8_t* we = a.ep ? uniform_ptr(a.ep[w]) : a.wbase + (size_t) w * a.w_stride;
        if (n >= JM_MIN) jm_segment(L, we, g0, g1, jb, n, y, a.out, a.out_stride);
        else if (n >= 1) jm_narrow(L.tab, we, JM_ROWS * g0, JM_ROWS * g1, jb, y, a.out, a.out_stride);
        i += (uint32_t) (g1 - g0);
    }
}

}  // namespace fnx
