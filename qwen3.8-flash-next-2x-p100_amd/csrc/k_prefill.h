// The prompt path's MoE: routing into jobs of up to FNX_PF_JOB rows per expert, and the routed experts on the matrix
// cores with f16 weights and activations and fp32 accumulation (the numerics of the reference's moe_mma.cuh:1-11).
//
// Matrix-core kernel, CDNA4 form. A wave owns 16 (or 32) weight rows of one job and walks K; v_mfma_f32_16x16x32_f16
// wants from lane l the operand row l % 16 and eight consecutive k "slots" of group l / 16. Which k a slot means is
// free as long as both operands agree, so group g is given the sub-blocks sb = 4 q + g: a lane then decodes one whole
// IQ3_S sub-block (32 weights, exactly what a lane of the mat-vec kernels decodes) straight into the A operands of four
// MFMAs, and the B operand of MFMA i is the 16 contiguous bytes x[token][32 sb + 8 i ..]. The dequantised weights
// never pass through LDS; LDS holds only the signed codebook as f16 (8192 entries of 4 halves, 64 KiB).
// A weight becomes f16 as (grid * (1 + 2 s)) * d: the first product is an integer below 2048, exact in f16, so the
// second rounds once - the same value as the reference's f32 product rounded to f16 (moe_mma_iq.cuh:136-149).
#pragma once

#include "k_moe_layer.h"

namespace fnx {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------- routing (prefill.cu:288-377)
// a wave per row: top-k of its logits, the weights. The blocks past the rows' (cvt_n > 0) turn cvt_n floats at cvt_x into
// f16 at cvt_y: the activations' copy for the matrix cores, which waits for nothing, rides along instead of a launch.
constexpr int PF_TOPK_WAVES = 4;
__global__ void __launch_bounds__(PF_TOPK_WAVES * 64) k_pf_topk(const float* __restrict__ logits, int ls, int C, int nexp, int topk,
                                                               int* __restrict__ topi, float* __restrict__ topw, const float* __restrict__ cvt_x,
                                                               size_t cvt_n, uint16_t* __restrict__ cvt_y) {
    __shared__ int ex[PF_TOPK_WAVES][64];
    const int row_blocks = (C + PF_TOPK_WAVES - 1) / PF_TOPK_WAVES;
    if ((int) blockIdx.x >= row_blocks) {   // four values a thread and step
        const size_t nb = gridDim.x - row_blocks, stride = nb * blockDim.x * 4;
        for (size_t i = ((size_t) (blockIdx.x - row_blocks) * blockDim.x + threadIdx.x) * 4; i < cvt_n; i += stride) {
            if (i + 3 < cvt_n && ((uintptr_t) cvt_x & 15) == 0 && ((uintptr_t) cvt_y & 7) == 0) {
                const float4 v = *reinterpret_cast<const float4*>(cvt_x + i);
                uint2 h;
                h.x = (uint32_t) float_to_half_bits(v.x) | (uint32_t) float_to_half_bits(v.y) << 16;
                h.y = (uint32_t) float_to_half_bits(v.z) | (uint32_t) float_to_half_bits(v.w) << 16;
                *reinterpret_cast<uint2*>(cvt_y + i) = h;
            } else {
                for (size_t j = i; j < i + 4 && j < cvt_n; ++j) cvt_y[j] = float_to_half_bits(cvt_x[j]);
            }
        }
        return;
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, t = blockIdx.x * PF_TOPK_WAVES + wave;
    if (t >= C) return;
    if (nexp <= 512) wave_topk<8>(logits + (size_t) t * ls, nexp, topk, lane, ex[wave], topi + (size_t) t * topk, topw + (size_t) t * topk);
    else wave_topk<16>(logits + (size_t) t * ls, nexp, topk, lane, ex[wave], topi + (size_t) t * topk, topw + (size_t) t * topk);
}
// a block per expert: its pairs in ascending order into the slots of its jobs (a pair always lands in the same job and
// slot, prefill.cu:340-343). A thread looks at PF_ROUNDS pairs a pass (p = p0 + 256 r + tid), all loaded together; the
// slots come from the waves' ballot counts, one barrier a pass. Blocks past the experts write the shared expert's
// jobs (every row: gate|up reads row t, writes row P + t; down reads and writes row P + t) and their count.
// Where its jobs start an expert's block works out for itself - every expert's pair count (the picks are a few KB, which each
// block reads anyway), ceil(count / FNX_PF_JOB) jobs each, the jobs of the experts before it - instead of waiting for a
// launch of one block that does it for all; it leaves its expert's count and first job (cnt, jbase), the last expert's
// block the job count.
constexpr int PF_FILL_THREADS = 256, PF_ROUNDS = 8, PF_MAXE = 1024;   // (PF_MAXE: the most experts)
__global__ void __launch_bounds__(PF_FILL_THREADS) k_pf_fill(const int* __restrict__ topi, int P, int topk, int nexp, int* __restrict__ cnt,
                                                            int* __restrict__ jbase, int* __restrict__ njobs, fnx_bigjob* __restrict__ gu,
                                                            fnx_bigjob* __restrict__ dn, int cap, int C, fnx_bigjob* __restrict__ sh_gu,
                                                            fnx_bigjob* __restrict__ sh_dn, int* __restrict__ nsh) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if ((int) blockIdx.x >= nexp) {
        if (!sh_gu) return;
        const int t = ((int) blockIdx.x - nexp) * PF_FILL_THREADS + tid;
        if (t == 0) *nsh = (C + FNX_PF_JOB - 1) / FNX_PF_JOB;
        if (t >= C) return;
        const int j = t / FNX_PF_JOB, k = t % FNX_PF_JOB;
        sh_gu[j].y[k] = t;
        sh_gu[j].out[k] = P + t;
        sh_dn[j].y[k] = P + t;
        sh_dn[j].out[k] = P + t;
        if (k == 0) {
            sh_gu[j].w = sh_dn[j].w = 0;
            sh_gu[j].n = sh_dn[j].n = min(FNX_PF_JOB, C - j * FNX_PF_JOB);
        }
        return;
    }
    const int e = blockIdx.x;
    constexpr int NW = PF_FILL_THREADS / 64;
    __shared__ int hist[PF_MAXE], wjobs[NW];
    __shared__ int wsum[PF_ROUNDS][NW];
    for (int i = tid; i < nexp; i += PF_FILL_THREADS) hist[i] = 0;
    __syncthreads();
    for (int p = tid; p < P; p += PF_FILL_THREADS) atomicAdd(&hist[topi[p]], 1);
    __syncthreads();
    int before_me = 0;   // jobs of the experts before this one
    for (int i = tid; i < e; i += PF_FILL_THREADS) before_me += (hist[i] + FNX_PF_JOB - 1) / FNX_PF_JOB;
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) before_me += __shfl_xor(before_me, o, 64);
    if (lane == 0) wjobs[wave] = before_me;
    __syncthreads();
    int jb = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) jb += wjobs[w];
    const int ce = hist[e];
    if (tid == 0) {
        cnt[e] = ce;
        jbase[e] = jb;
        if (e == nexp - 1) njobs[0] = jb + (ce + FNX_PF_JOB - 1) / FNX_PF_JOB;
    }
    if (ce == 0) return;
    int base = 0;
    for (int p0 = 0; p0 < P; p0 += PF_FILL_THREADS * PF_ROUNDS) {
        int pick[PF_ROUNDS];
#pragma unroll
        for (int r = 0; r < PF_ROUNDS; ++r) {
            const int p = p0 + r * PF_FILL_THREADS + tid;
            pick[r] = p < P ? topi[p] : -1;
        }
        unsigned long long m[PF_ROUNDS];
#pragma unroll
        for (int r = 0; r < PF_ROUNDS; ++r) {
            m[r] = __ballot(pick[r] == e);
            if (lane == 0) wsum[r][wave] = __popcll(m[r]);
        }
        __syncthreads();
        int before = base;   // pairs of this expert before round r's wave `wave`
#pragma unroll
        for (int r = 0; r < PF_ROUNDS; ++r) {
            int mine_before = before;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                mine_before += w < wave ? wsum[r][w] : 0;
                before += wsum[r][w];
            }
            if (pick[r] == e) {
                const int p = p0 + r * PF_FILL_THREADS + tid;
                const int s = mine_before + __popcll(m[r] & ((1ull << lane) - 1ull)), j = jb + s / FNX_PF_JOB, k = s % FNX_PF_JOB;
                if (j < cap) {
                    gu[j].y[k] = p / topk;
                    gu[j].out[k] = p;
                    dn[j].y[k] = p;
                    dn[j].out[k] = p;
                    if (k == 0) {
                        gu[j].w = dn[j].w = e;
                        gu[j].n = dn[j].n = min(FNX_PF_JOB, ce - (s / FNX_PF_JOB) * FNX_PF_JOB);
                    }
                }
            }
        }
        base = before;
        __syncthreads();
    }
}

// ---------------------------------------------------------------- element-wise
__global__ void k_f32_f16(const float* __restrict__ x, size_t n, uint16_t* __restrict__ y) {
    for (size_t i = blockIdx.x * (size_t) blockDim.x + threadIdx.x; i < n; i += (size_t) gridDim.x * blockDim.x) y[i] = float_to_half_bits(x[i]);
}
// moe_mma.cuh:500-507
__global__ void k_swiglu_h16(const float* __restrict__ gu, int ffs, size_t total, uint16_t* __restrict__ h) {
    for (size_t e = blockIdx.x * (size_t) blockDim.x + threadIdx.x; e < total; e += (size_t) gridDim.x * blockDim.x) {
        const size_t r = e / ffs, i = e % ffs;
        const float g = gu[r * 2 * ffs + i];
        h[e] = float_to_half_bits(silu_f(g) * gu[r * 2 * ffs + ffs + i]);
    }
}

// ---------------------------------------------------------------- router logits of a chunk
// The same sums for many activation rows (the prompt path's router logits): a wave takes GR_ROWS weight rows x a group
// of FNX_MAXT activation rows, lane l the float4 chunks l, l + 64, ... of all of them, so every activation chunk it
// loads (coalesced, straight from the caches: no LDS, no barriers) feeds GR_ROWS chains. Order per sum as above.
constexpr int GM_WAVES = 8, GR_ROWS = 4, GM_BATCH = 8;
static_assert(GR_ROWS * FNX_MAXT == 64, "64 sums a wave, one per lane in the end");
// one wave: weight rows row0 .. row0 + GR_ROWS - 1 against the activation rows FNX_MAXT tgroup ..
template <bool BF>
__device__ __forceinline__ void gemv_rows_many_wave(const void* __restrict__ Wv, const float* __restrict__ x, float* __restrict__ y, int rows, int n,
                                                    int T, int row0, int tgroup, int lane) {
    x += (size_t) tgroup * FNX_MAXT * n;
    y += (size_t) tgroup * FNX_MAXT * rows;
    T = min(FNX_MAXT, T - tgroup * FNX_MAXT);
    if (row0 >= rows || T <= 0) return;
    float acc[GR_ROWS][FNX_MAXT];
#pragma unroll
    for (int r = 0; r < GR_ROWS; ++r)
#pragma unroll
        for (int t = 0; t < FNX_MAXT; ++t) acc[r][t] = 0.f;
    const float4* xr[FNX_MAXT];
#pragma unroll
    for (int t = 0; t < FNX_MAXT; ++t) xr[t] = reinterpret_cast<const float4*>(x + (size_t) min(t, T - 1) * n) + lane;
    for (int c0 = 0; c0 < n / 4; c0 += 64) {
        float4 w[GR_ROWS];
#pragma unroll
        for (int r = 0; r < GR_ROWS; ++r) {
            const size_t row = (size_t) min(row0 + r, rows - 1);
            if constexpr (BF) {
                const uint2 u = reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(Wv) + row * n)[c0 + lane];
                w[r] = make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                                   __uint_as_float(u.y & 0xffff0000u));
            } else {
                w[r] = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(Wv) + row * n)[c0 + lane];
            }
        }
        // GM_BATCH activation chunks in flight at a time (left to itself the compiler loads them one by one, each a cache
        // round trip before its 16 fmaf)
#pragma unroll
        for (int t0 = 0; t0 < FNX_MAXT; t0 += GM_BATCH) {
            float4 b[GM_BATCH];
#pragma unroll
            for (int t = 0; t < GM_BATCH; ++t) b[t] = xr[t0 + t][c0];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < GM_BATCH; ++t)
#pragma unroll
                for (int r = 0; r < GR_ROWS; ++r) {
                    float a = acc[r][t0 + t];
                    a = fmaf(w[r].x, b[t].x, a);
                    a = fmaf(w[r].y, b[t].y, a);
                    a = fmaf(w[r].z, b[t].z, a);
                    a = fmaf(w[r].w, b[t].w, a);
                    acc[r][t0 + t] = a;
                }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // The 64 sums (value j = 16 r + t) over the 64 lanes, all at once: at the butterfly's level for lane bit b a lane
    // keeps the half of its values whose index has bit b equal to its own and adds its partner's copy of them - the
    // same pairwise adds, level by level, as group_sum<64> makes for each value, in 63 exchanges instead of 384.
    // Lane l ends with value l.
    float v32[32], v16[16], v8[8];
#pragma unroll
    for (int i = 0; i < 32; ++i) v32[i] = swap32_add(acc[i >> 4][i & 15], acc[2 + (i >> 4)][i & 15]);
#pragma unroll
    for (int i = 0; i < 16; ++i) v16[i] = swap16_add(v32[i], v32[i + 16]);
    auto fold = [&](const float lo, const float hi, int o) {
        const bool up = lane & o;
        return (up ? hi : lo) + __shfl_xor(up ? lo : hi, o, WAVE);
    };
#pragma unroll
    for (int i = 0; i < 8; ++i) v8[i] = fold(v16[i], v16[i + 8], 8);
    const float a0 = fold(v8[0], v8[4], 4), a1 = fold(v8[1], v8[5], 4), a2 = fold(v8[2], v8[6], 4), a3 = fold(v8[3], v8[7], 4);
    const float b0 = fold(a0, a2, 2), b1 = fold(a1, a3, 2);
    const float v = fold(b0, b1, 1);
    const int r = lane >> 4, t = lane & 15;
    if (t < T && row0 + r < rows) y[(size_t) t * rows + row0 + r] = v;
}
template <bool BF>
__global__ void __launch_bounds__(GM_WAVES * 64) k_gemv_rows_many(const void* __restrict__ Wv, const float* __restrict__ x, float* __restrict__ y,
                                                                 int rows, int n, int T, int row_begin) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    gemv_rows_many_wave<BF>(Wv, x, y, rows, n, T, row_begin + (blockIdx.x * GM_WAVES + wave) * GR_ROWS, blockIdx.y, lane);
}

// ---------------------------------------------------------------- the same sums on the matrix cores
// v_mfma_f32_32x32x1_2b_f32 is D = fma(a, b, D) element by element with one rounding - the fmaf of the chains above
// (checked bit for bit on this GPU, products in the denormal range included). A chain of them over the chunks
// l, l + 64, ... therefore leaves lane l's partial sum of 32 activation rows x 32 weight rows at once; the instruction's
// two blocks take l and l + 32, the pair that the butterfly adds first. A block owns such a tile of 32 x 32 sums. Wave
// w of its RM_WAVES multiplying waves walks the lanes l = w mod 4 in eight phases - l = 8 a + 4 h + w and l + 32, (h; a)
// in the order (0; 0, 2, 1, 3), (1; 0, 2, 1, 3) - so that the butterfly's levels 16, 8 and 4 are adds of whole
// accumulator tiles as the phases end (done while the next phase multiplies into a second accumulator); levels 2 and 1
// add the four waves' tiles through LDS. The operands (f32 weights only) come through LDS: a stage is 64 rows (32 of x,
// 32 of W) x 512 bytes - four chunks of the four lanes l and of l + 32 - sent there by global_load_lds_dwordx4 from two
// waves of their own (an instruction issued between MFMAs holds its wave up for about 40 cycles), two stages ahead, into
// one of three buffers; an instruction carries two rows, and row r's piece p lies at place p ^ (r % 16) (within its
// half of 16), so that the 16 rows an operand read touches fall on 16 different bank groups. The waves read a stage's
// operands right after the meeting that says it has landed and multiply the stage before it meanwhile.
// The weight rows past the last full 32 (the router's 513th) are left to the first loading wave, idle half of the
// time: an item is one such row against four rows of x, its loads go out in pieces after the first stages' and are
// back, the loads completing in order, where a stage asked for after them is waited for.
typedef float v32f __attribute__((ext_vector_type(32)));
typedef float v16f __attribute__((ext_vector_type(16)));
constexpr int RM_TILE = 32, RM_WAVES = 4, RM_LOADERS = 2, RM_THREADS = (RM_WAVES + RM_LOADERS) * 64, RM_ROWB = 512, RM_STAGE = 2 * RM_TILE * RM_ROWB, RM_BUFS = 3;
constexpr int RM_PIECE = 10 * 1024, RM_PIECES = 4;   // an item's loads of two steps (a weight row's and four x rows' chunks), pieces in LDS at a time
constexpr int RM_ITEM_AT = 4;                        // the stage after whose loads an item's first piece goes out
__global__ void __launch_bounds__(RM_THREADS) k_gemv_rows_mfma(const float* __restrict__ W, const float* __restrict__ x, float* __restrict__ y,
                                                              int rows, int n, int T, int ntt, int net, int tile_blocks, int along) {
    __shared__ __align__(16) uint8_t lds[RM_BUFS * RM_STAGE + RM_PIECES * RM_PIECE];
    const int wave = uniform((int) (threadIdx.x >> 6)), lane = threadIdx.x & 63;
    // Which tile: block ids go round the eight XCDs, each with an L2 of its own, so an XCD's blocks are given one patch of
    // 4 x 8 tiles after another (1 MB of x and 2 MB of W for rows of 2048: its L2 holds them, every block re-reads both
    // eight times over the phases). The grid covers whole patches; a block whose tile lies outside leaves.
    const int lin = ((int) blockIdx.x % 8) * (tile_blocks / 8) + (int) blockIdx.x / 8, patches_e = (net + 7) / 8;
    const int tt = 4 * ((lin / 32) / patches_e) + (lin % 32) / 8, et = 8 * ((lin / 32) % patches_e) + lin % 8;
    if (tt >= ntt || et >= net) return;
    const int t0 = tt * RM_TILE, e0 = et * RM_TILE;
    const int nh = n / 1024, S = 8 * nh;   // stages: phase-major, a row's quarters of 1024 values within a phase (nh is even)
    const uint32_t lds_at = (uint32_t) (size_t) (__attribute__((address_space(3))) uint8_t*) lds;
    // All waves meet where a stage must have landed. A loader's loads complete in order: it waits until only the newest
    // stage's (and an item's pieces after them) may be on their way; the others wait for their own LDS reads. (A plain barrier instruction: __syncthreads() would wait for every load.)
    auto meet = [&](int in_flight) {
        __builtin_amdgcn_sched_barrier(0);
        if (in_flight == 36) __builtin_amdgcn_s_waitcnt(0x8074);        // vmcnt(36) lgkmcnt(0)
        else if (in_flight == 26) __builtin_amdgcn_s_waitcnt(0x407A);   // vmcnt(26) lgkmcnt(0)
        else if (in_flight == 16) __builtin_amdgcn_s_waitcnt(0x4070);   // vmcnt(16) lgkmcnt(0)
        else __builtin_amdgcn_s_waitcnt(0x0070);                        // vmcnt(0) lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    if (wave >= RM_WAVES) {   // a loader: the first takes the stages' rows of x, the second those of W
        const int lw = wave - RM_WAVES;
        uint32_t off[16];   // instruction j: rows 2 j and 2 j + 1 of this loader's half of the stage, this lane's piece
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int row = 2 * j + (lane >> 5), q = lane & 31, p = (q & 16) | ((q & 15) ^ (row & 15));
            const int r = lw == 0 ? min(t0 + row, T - 1) : e0 + row;
            off[j] = (uint32_t) r * (uint32_t) n * 4u + 1024u * (p >> 3) + 512u * ((p >> 2) & 1) + 16u * (p & 3);
        }
        const uint8_t* src = reinterpret_cast<const uint8_t*>(lw == 0 ? x : W);
        int ph = 0, hf = 0;   // the next stage to fetch
        auto fetch = [&](int buf) {
            const int q = ph & 3, l0 = 8 * (((q & 1) << 1) | (q >> 1)) + 4 * (ph >> 2);
            const uint8_t* from = src + 16 * l0 + 4096 * hf;
#pragma unroll
            for (int j = 0; j < 16; ++j) lds_load16(from, off[j], lds_at + buf * RM_STAGE + lw * (RM_TILE * RM_ROWB) + j * 1024);
            if (++hf == nh) hf = 0, ++ph;
        };
        // This loader's item of the rows past the tiles: weight row irow against the rows it0 .. it0 + 3 of x, lane l the
        // chunks l, l + 64, ... A piece - two steps' chunks, ten instructions - goes out after each of the first stages'
        // loads, into LDS like them (so that every load in flight is one that the meetings count), and is added up three
        // meetings later: the stage waited for there was asked for after it.
        // (Block (tt, et) takes the row et / 8 past the tiles against the et % 8-th four of its own 32 rows of x: rows that its
        // XCD's L2 holds anyway.)
        const int steps = n / 256, pieces = steps / 2;
        const bool has_item = lw == 0 && along && et < 8 * (rows - net * RM_TILE);
        const int irow = has_item ? net * RM_TILE + et / 8 : 0, it0 = has_item ? t0 + 4 * (et % 8) : 0;
        const uint8_t* irows[5] = {reinterpret_cast<const uint8_t*>(W + (size_t) irow * n), nullptr, nullptr, nullptr, nullptr};
#pragma unroll
        for (int t = 0; t < 4; ++t) irows[1 + t] = reinterpret_cast<const uint8_t*>(x + (size_t) min(it0 + t, T - 1) * n);
        const uint8_t* ilds = lds + RM_BUFS * RM_STAGE;
        float iacc[4] = {0.f, 0.f, 0.f, 0.f};
        fetch(0);
        fetch(1);   // (S >= 16)
        int buf = 2;
        for (int k = 0; k <= S; ++k) {   // (the others meet once more than there are stages: they read one ahead)
            const int kp = k - RM_ITEM_AT;   // the piece that goes out in this round
            const int younger = (has_item && kp >= 2 && kp - 2 < pieces ? 10 : 0) + (has_item && kp >= 1 && kp - 1 < pieces ? 10 : 0);
            meet(k + 1 >= S ? 0 : 16 + younger);
            if (k + 2 < S) fetch(buf);
            buf = buf == RM_BUFS - 1 ? 0 : buf + 1;
            if (has_item && kp >= 0 && kp < pieces) {
                const uint32_t at = lds_at + RM_BUFS * RM_STAGE + (kp & (RM_PIECES - 1)) * RM_PIECE;
#pragma unroll
                for (int s = 0; s < 2; ++s)
#pragma unroll
                    for (int r = 0; r < 5; ++r) lds_load16(irows[r] + (2 * kp + s) * 1024, 16u * lane, at + (5 * s + r) * 1024);
            }
            if (has_item && kp >= 3 && kp - 3 < pieces) {
                const uint8_t* p = ilds + ((kp - 3) & (RM_PIECES - 1)) * RM_PIECE + 16 * lane;
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const float4 w = *reinterpret_cast<const float4*>(p + 5 * s * 1024);
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const float4 bv = *reinterpret_cast<const float4*>(p + (5 * s + 1 + t) * 1024);
                        float a = iacc[t];
                        a = fmaf(w.x, bv.x, a);
                        a = fmaf(w.y, bv.y, a);
                        a = fmaf(w.z, bv.z, a);
                        a = fmaf(w.w, bv.w, a);
                        iacc[t] = a;
                    }
                }
            }
        }
        meet(0);   // the tiles' meeting below
        if (has_item) {   // the butterfly over the item's four sums (when nobody waits for this wave any more): levels 32 and 16
                          // for all four at once, a 16-lane row then holds one sum's values for levels 8 .. 1
            float v = swap16_add(swap32_add(iacc[0], iacc[1]), swap32_add(iacc[2], iacc[3]));   // rows: sums 0, 2, 1, 3
#pragma unroll
            for (int o = 8; o; o >>= 1) v += __shfl_xor(v, o, WAVE);
            const int row = lane >> 4, ti = it0 + (((row & 1) << 1) | (row >> 1));
            if ((lane & 15) == 0 && ti < T) y[(size_t) ti * rows + irow] = v;
        }
        return;
    }
    const int i = lane & 31, b = lane >> 5;
    // this lane's operands of a stage: row i of x and row i of W, chunks 0 .. 3 of lane l (block b: l + 32)
    const uint8_t* r0 = lds + i * RM_ROWB + 16 * ((4 * b + wave) ^ (i & 15));       // chunks 0 and 2 (256 bytes on)
    const uint8_t* r1 = lds + i * RM_ROWB + 16 * ((8 + 4 * b + wave) ^ (i & 15));   // chunks 1 and 3
    float4 A[2][4], B[2][4];
    int buf = 0;   // the buffer whose operands are read next
    auto next_stage = [&](float4 (&a)[4], float4 (&bb)[4]) {
        meet(0);
        const int o = buf * RM_STAGE;   // (past the last stage: a buffer's old contents, not used)
        a[0] = *reinterpret_cast<const float4*>(r0 + o);
        a[1] = *reinterpret_cast<const float4*>(r1 + o);
        a[2] = *reinterpret_cast<const float4*>(r0 + o + 256);
        a[3] = *reinterpret_cast<const float4*>(r1 + o + 256);
        bb[0] = *reinterpret_cast<const float4*>(r0 + o + RM_TILE * RM_ROWB);
        bb[1] = *reinterpret_cast<const float4*>(r1 + o + RM_TILE * RM_ROWB);
        bb[2] = *reinterpret_cast<const float4*>(r0 + o + RM_TILE * RM_ROWB + 256);
        bb[3] = *reinterpret_cast<const float4*>(r1 + o + RM_TILE * RM_ROWB + 256);
        buf = buf == RM_BUFS - 1 ? 0 : buf + 1;
        __builtin_amdgcn_sched_barrier(0);
    };
    v32f acc[2];
    float held[16], u0[16], sum[16];   // (plain arrays: no need for runs of 16 registers)
    // The fold of a phase, whose accumulator is cf: the butterfly's levels 32 (the instruction's two blocks; the sums
    // take the place of the first block), 16, 8 and 4, in three pieces that go between the next phase's first MFMAs on
    // the vector unit. The phases of a = 0 and a = 1 (kind 0) leave held; that of a = 2 (odd) adds level 16 with a = 0
    // into u0; that of a = 3 adds level 16 with a = 1 and level 8 into sum, and at the very end (last) level 4. Which of
    // the latter two it is, is a select on a scalar, not a branch: the stretch of MFMAs stays one block of code.
    auto fold_a = [&](v32f& cf) {
#pragma unroll
        for (int v = 0; v < 16; ++v) cf[v] = cf[v] + cf[16 + v];
    };
    auto fold_b = [&](bool first_of_pair, bool odd, v32f& cf) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            if (first_of_pair) {
                held[v] = cf[v];
            } else {
                cf[v] = held[v] + cf[v];
                u0[v] = odd ? cf[v] : u0[v];
            }
        }
    };
    auto fold_c = [&](bool first_of_pair, bool odd, bool last, const v32f& cf) {
        if (first_of_pair) return;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            if (last) sum[v] = sum[v] + (u0[v] + cf[v]);
            else sum[v] = odd ? sum[v] : u0[v] + cf[v];
        }
    };
    // a stage's 16 steps into accumulator c (first: the phase's first stage, which starts from zero, with the fold of the
    // phase before, unless it is a later stage)
    auto multiply = [&](const float4 (&a)[4], const float4 (&bb)[4], v32f& c, auto first_c, bool first_of_pair, bool odd, v32f& cf) {
        constexpr bool first = decltype(first_c)::value;
        if constexpr (first) asm volatile("" : "+v"(cf));   // (keeps the fold's adds on this side of the meeting)
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
            if (first && cc == 0) {
                v32f z;
#pragma unroll
                for (int v = 0; v < 32; ++v) z[v] = 0.f;
                c = __builtin_amdgcn_mfma_f32_32x32x1f32(a[cc].x, bb[cc].x, z, 0, 0, 0);
            } else {
                c = __builtin_amdgcn_mfma_f32_32x32x1f32(a[cc].x, bb[cc].x, c, 0, 0, 0);
            }
            if constexpr (first) {
                if (cc < 3) {
                    __builtin_amdgcn_sched_barrier(0);
                    if (cc == 0) fold_a(cf);
                    else if (cc == 1) fold_b(first_of_pair, odd, cf);
                    else fold_c(first_of_pair, odd, false, cf);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            c = __builtin_amdgcn_mfma_f32_32x32x1f32(a[cc].y, bb[cc].y, c, 0, 0, 0);
            c = __builtin_amdgcn_mfma_f32_32x32x1f32(a[cc].z, bb[cc].z, c, 0, 0, 0);
            c = __builtin_amdgcn_mfma_f32_32x32x1f32(a[cc].w, bb[cc].w, c, 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    using std::integral_constant;
    constexpr integral_constant<bool, true> yes{};
    constexpr integral_constant<bool, false> no{};
    // a phase into accumulator c, the phase before's fold (accumulator cf) along with its first stage
    auto phase = [&](v32f& c, bool first_of_pair, bool odd, v32f& cf) {
        next_stage(A[1], B[1]);
        multiply(A[0], B[0], c, yes, first_of_pair, odd, cf);
        next_stage(A[0], B[0]);
        multiply(A[1], B[1], c, no, false, false, c);
        for (int h2 = 2; h2 < nh; h2 += 2) {
            next_stage(A[1], B[1]);
            multiply(A[0], B[0], c, no, false, false, c);
            next_stage(A[0], B[0]);
            multiply(A[1], B[1], c, no, false, false, c);
        }
    };
#pragma unroll
    for (int v = 0; v < 32; ++v) acc[1][v] = 0.f;
#pragma unroll
    for (int v = 0; v < 16; ++v) held[v] = u0[v] = sum[v] = 0.f;
    next_stage(A[0], B[0]);
    // pairs of phases: (a = 0, a = 2), (a = 1, a = 3), and again for h = 1. The first of a pair folds the second of the pair
    // before (the very first: nothing, and what that leaves is overwritten), the second the first.
#pragma unroll 1
    for (int pp = 0; pp < 4; ++pp) {
        phase(acc[0], false, (pp & 1) != 0, acc[1]);
        phase(acc[1], true, false, acc[0]);
    }
    fold_a(acc[1]);
    fold_b(false, false, acc[1]);
    fold_c(false, false, true, acc[1]);
    // levels 2 and 1 over the waves' tiles, in the buffer that the stage before the last left (all have read it; the
    // last one's successor may still be being read, for nothing, by another wave)
    float* red = reinterpret_cast<float*>(lds + ((S - 2) % RM_BUFS) * RM_STAGE);
#pragma unroll
    for (int v = 0; v < 16; ++v) red[(wave * 16 + v) * 64 + lane] = sum[v];
    meet(0);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int v = 4 * wave + q;
        const float s = (red[v * 64 + lane] + red[(32 + v) * 64 + lane]) + (red[(16 + v) * 64 + lane] + red[(48 + v) * 64 + lane]);
        const int tk = t0 + 8 * (v >> 2) + 4 * b + (v & 3);
        if (tk < T) y[(size_t) tk * rows + e0 + i] = s;
    }
}

// ---------------------------------------------------------------- the routed experts on the matrix cores
struct MmaArgs {
    const uint8_t* w;       // the experts' matrices: expert e at w + e * stride, or ep[e]
    size_t stride;
    const void* const* ep;
    int nrows, ncols;
    const fnx_bigjob* jobs;
    const int* njobs;
    int cap;
    const uint16_t* x;      // f16 activation rows of ldx values
    int ldx;
    float* out;             // rows of nrows
    // a second job list over one more matrix (the shared expert's, whatever its jobs' w says), in the same launch: alone
    // its few jobs fill a quarter of the chip (the wave forms)
    const uint8_t* w2 = nullptr;
    const fnx_bigjob* jobs2 = nullptr;
    const int* njobs2 = nullptr;
    int cap2 = 0;
    // wave form, stacked gate|up matrices (nrows = 2 ffh, ffh in 16s): a wave's two tiles are 16 gate rows and the
    // 16 up rows that go with them, and what is written is h = silu(gate) * up as f16 rows of ffh (k_swiglu_h16's values)
    // instead of the products themselves
    uint16_t* h16 = nullptr;
    int ffh = 0;
};
constexpr int MM_THREADS = 512, MM_WAVES = MM_THREADS / 64, MM_TT = FNX_PF_JOB / 16;

struct SubFields {   // one sub-block as loaded: four words of codes, the scale nibble, d's bits
    uint32_t q0, q1, q2, q3, sc, d;
};
// loads through address-space-1 pointers: global_load, which (unlike flat_load) does not tie up the LDS counter that
// the codebook reads wait on
template <bool PACKED>
__device__ __forceinline__ SubFields sub_load(const uint8_t* __restrict__ we, int row, int sb, int ks) {
    typedef __attribute__((address_space(1))) const v2u g64;
    typedef __attribute__((address_space(1))) const uint32_t g32;
    typedef __attribute__((address_space(1))) const unsigned short g16;
    SubFields r;
    if constexpr (PACKED) {
        const uint32_t L = (uint32_t) row * ks + sb, l = L & 63u;
        const gbytes u = as_global(we + (size_t) (L >> 6) * UNIT_BYTES);
        const v2u a = *(g64*) (u + 8 * l);
        r.q0 = a.x;
        r.q1 = a.y;
        r.q2 = *(g32*) (u + UNIT_B_AT + 4 * l);
        r.q3 = u[UNIT_C_AT + l];
        r.sc = u[UNIT_SCALES_AT + (l >> 1)] >> (4 * (l & 1));
        r.d = *(g16*) (u + UNIT_D_AT + 2 * (l >> 3));
    } else {
        const int ib = sb & 7;
        const gbytes b = as_global(we + ((size_t) row * (ks >> 3) + (sb >> 3)) * 110);
        const g16* q = (g16*) (b + 2 + 8 * ib);
        r.q0 = q[0] | (uint32_t) q[1] << 16;
        r.q1 = q[2] | (uint32_t) q[3] << 16;
        const g16* sg = (g16*) (b + 74 + 4 * ib);
        r.q2 = sg[0] | (uint32_t) sg[1] << 16;
        r.q3 = b[66 + ib];
        r.sc = b[106 + (ib >> 1)] >> (4 * (ib & 1));
        r.d = *(g16*) b;
    }
    return r;
}
// LDS byte offset of group j's entry in the f16 codebook (entries of 8 bytes)
template <bool PACKED>
__device__ __forceinline__ uint32_t sub_entry(const SubFields& f, int j) {
    if constexpr (PACKED) {
        const uint32_t q[4] = {f.q0, f.q1, f.q2, f.q3};
        const int bit = 13 * j, w = bit >> 5, s = bit & 31;
        uint32_t v;
        if (s + 13 <= 32) v = s >= 3 ? q[w] >> (s - 3) : q[w] << (3 - s);
        else v = __builtin_amdgcn_alignbit(q[w + 1], q[w], s - 3);
        return v & 0xFFF8u;
    } else {
        const uint32_t code = ((j < 4 ? f.q0 >> (8 * j) : f.q1 >> (8 * (j - 4))) & 0xFFu) | (((f.q3 >> j) & 1u) << 8);
        return (((f.q2 >> (4 * j)) & 0xFu) << 12) | (code << 3);
    }
}
__device__ __forceinline__ v2h as_v2h(uint32_t u) { return __builtin_bit_cast(v2h, u); }

// A task = (job, RG * 16 weight rows, MM_TP token tiles of 16): uniform pieces, so a static split over the waves
// balances; consecutive waves take the same job's next rows and share its activation rows in the caches.
// Order of a k-step's loads matters because loads return in order: first this step's activation operands (from L2,
// consumed after the decode), then the weights of two steps ahead (from HBM) - a wait for the former never waits for
// the latter.
constexpr int MM_TP = 2;
template <bool PACKED, int RG>
__global__ void __launch_bounds__(MM_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) k_moe_mma(const MmaArgs a) {
    typedef __attribute__((address_space(1))) const v4u gx4;
    __shared__ uint2 tab[SGRID_WORDS];
    const uint32_t tab0 = g_sgrid.v[threadIdx.x];   // (512 threads: a thread's code, its sixteen signed entries made here)
#pragma unroll
    for (int i = threadIdx.x; i < SGRID_WORDS; i += MM_THREADS) {
        const uint32_t g = signed_entry(tab0, i >> 9);
        v2h lo, hi;
        lo.x = (_Float16) (int) (int8_t) (g & 0xFFu);
        lo.y = (_Float16) (int) (int8_t) ((g >> 8) & 0xFFu);
        hi.x = (_Float16) (int) (int8_t) ((g >> 16) & 0xFFu);
        hi.y = (_Float16) (int) (int8_t) (g >> 24);
        tab[i] = make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int nj = min(a.cap, uniform(*a.njobs));
    const int ks = a.ncols >> 5, groups = a.nrows / (16 * RG), steps = ks >> 2;
    constexpr int HALVES = MM_TT / MM_TP;
    const int nwaves = gridDim.x * MM_WAVES, per_job = groups * HALVES;
    for (int task = uniform(blockIdx.x * MM_WAVES + (threadIdx.x >> 6)); task < nj * per_job; task += nwaves) {
        const int ji = task / per_job, rem = task - ji * per_job, t0 = (rem / groups) * MM_TP, row0 = (rem % groups) * 16 * RG;
        const fnx_bigjob* jb = a.jobs + ji;
        const int n = min(FNX_PF_JOB, uniform(jb->n)), e = uniform(jb->w), nt = (n + 15) >> 4;
        if (t0 >= nt) continue;
        const int ntile = min(MM_TP, nt - t0);
        const uint8_t* we = a.ep ? (const uint8_t*) a.ep[e] : a.w + (size_t) e * a.stride;
        const uint16_t* xr[MM_TP];
#pragma unroll
        for (int tt = 0; tt < MM_TP; ++tt) xr[tt] = a.x + (size_t) jb->y[min((t0 + tt) * 16 + r, n - 1)] * a.ldx + 32 * g;
        v4f acc[RG][MM_TP];
#pragma unroll
        for (int q = 0; q < RG; ++q)
#pragma unroll
            for (int tt = 0; tt < MM_TP; ++tt) acc[q][tt] = v4f{0.f, 0.f, 0.f, 0.f};
        SubFields w0[RG], w1[RG];
#pragma unroll
        for (int q = 0; q < RG; ++q) w0[q] = sub_load<PACKED>(we, row0 + 16 * q + r, g, ks);
        // one k-step: cur holds its weights' fields; nxt receives the next step's (no register copies between steps: a
        // copy of a loaded register would wait for the load)
        auto step = [&](SubFields (&cur)[RG], SubFields (&nxt)[RG], int st) {
            v4u B[MM_TP][4];
#pragma unroll
            for (int tt = 0; tt < MM_TP; ++tt)
                if (tt < ntile) {
                    const gx4* xp = (gx4*) (uintptr_t) (xr[tt] + 128 * st);
#pragma unroll
                    for (int i = 0; i < 4; ++i) B[tt][i] = xp[i];
                }
            const int sbn = 4 * min(st + 1, steps - 1) + g;   // past the end: the last step's again
#pragma unroll
            for (int q = 0; q < RG; ++q) nxt[q] = sub_load<PACKED>(we, row0 + 16 * q + r, sbn, ks);
            // this lane's sub-block of each row group as 32 f16 weights: the A operands of four MFMAs
            v8h A[RG][4];
#pragma unroll
            for (int q = 0; q < RG; ++q) {
                const _Float16 sc = (_Float16) (int) (1 + 2 * (cur[q].sc & 0xFu)), d = __builtin_bit_cast(_Float16, (unsigned short) cur[q].d);
                const v2h s2 = {sc, sc}, d2 = {d, d};
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint2 en = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint8_t*>(tab) + sub_entry<PACKED>(cur[q], j));
                    const v2h lo = (as_v2h(en.x) * s2) * d2, hi = (as_v2h(en.y) * s2) * d2;
                    A[q][j >> 1][4 * (j & 1) + 0] = lo.x;
                    A[q][j >> 1][4 * (j & 1) + 1] = lo.y;
                    A[q][j >> 1][4 * (j & 1) + 2] = hi.x;
                    A[q][j >> 1][4 * (j & 1) + 3] = hi.y;
                }
            }
#pragma unroll
            for (int tt = 0; tt < MM_TP; ++tt)
                if (tt < ntile) {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
#pragma unroll
                        for (int q = 0; q < RG; ++q)
                            acc[q][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[q][i], __builtin_bit_cast(v8h, B[tt][i]), acc[q][tt], 0, 0, 0);
                }
        };
        for (int st = 0; st < steps; st += 2) {   // steps = ncols / 128, even for whole 256-column blocks
            step(w0, w1, st);
            step(w1, w0, st + 1);
        }
        // lane: token r of each tile, weight rows 4 g .. 4 g + 3 of each group
#pragma unroll
        for (int tt = 0; tt < MM_TP; ++tt) {
            const int tok = (t0 + tt) * 16 + r;
            if (tt < ntile && tok < n) {
                float* o = a.out + (size_t) jb->out[tok] * a.nrows + row0 + 4 * g;
#pragma unroll
                for (int q = 0; q < RG; ++q) *reinterpret_cast<float4*>(o + 16 * q) = make_float4(acc[q][tt].x, acc[q][tt].y, acc[q][tt].z, acc[q][tt].w);
            }
        }
    }
}

// ---------------------------------------------------------------- a lane's four consecutive sub-blocks of a row
// What limits the wave-a-task kernel above on MI355X is the vector-memory front end: every wave gathers its weights 32
// bytes per row at a time, so each cache line is fetched four times. A lane that owns four consecutive sub-blocks of its
// row per super-step of 512 columns (sub-block 16 S + 4 g + p at step p) loads whole 32/16/4/2-byte runs of the planes,
// 6 loads per row and super-step, each line of a plane touched once: the loads of the tile16 re-laying below and of the
// wave forms (k_moe_mma_wave16.h), which read the same fields from the tile16 layout.
struct SuperFields {   // a lane's four sub-blocks of one row as loaded
    v4u a0, a1, b;
    uint32_t c, sc, d;
};
__device__ __forceinline__ SuperFields super_load(const uint8_t* __restrict__ we, int row, int sb0, int ks) {
    typedef __attribute__((address_space(1))) const v4u g128;
    typedef __attribute__((address_space(1))) const uint32_t g32;
    typedef __attribute__((address_space(1))) const unsigned short g16;
    const uint32_t L = (uint32_t) row * ks + sb0, l = L & 63u;   // l: a multiple of 4
    const gbytes u = as_global(we + (size_t) (L >> 6) * UNIT_BYTES);
    SuperFields r;
    r.a0 = *(g128*) (u + 8 * l);
    r.a1 = *(g128*) (u + 8 * l + 16);
    r.b = *(g128*) (u + UNIT_B_AT + 4 * l);
    r.c = *(g32*) (u + UNIT_C_AT + l);
    r.sc = *(g16*) (u + UNIT_SCALES_AT + (l >> 1));
    r.d = *(g16*) (u + UNIT_D_AT + 2 * (l >> 3));
    return r;
}
template <int P>
__device__ __forceinline__ SubFields super_sub(const SuperFields& f) {
    SubFields s;
    s.q0 = P < 2 ? f.a0[2 * (P & 1)] : f.a1[2 * (P & 1)];
    s.q1 = P < 2 ? f.a0[2 * (P & 1) + 1] : f.a1[2 * (P & 1) + 1];
    s.q2 = f.b[P];
    s.q3 = (f.c >> (8 * P)) & 0xFFu;
    s.sc = (f.sc >> (4 * P)) & 0xFu;
    s.d = f.d;
    return s;
}
// The same fields from the prompt path's own layout ("tile16", FNX_T_IQ3S_TILE16): a matrix as tiles of 16 rows x 512
// columns, tile (row / 16, column / 512) at ((row / 16) * (ncols / 512) + column / 512) * TILE16_BYTES, and in a tile the
// 64 lanes' shares side by side, plane by plane: lane (row % 16) + 16 g holds sub-blocks 4 g .. 4 g + 3 of the tile's 16 -
// A 32 bytes a lane, B 16, C 4, the scale nibbles 2, d 2. Every load of a wave is then one contiguous run (2 KiB, 1 KiB,
// 256, 128, 128 bytes) and a wave's super-steps follow each other in memory, where the unit64 planes give the matrix
// cores' lanes - sixteen different rows - a cache line each. 3,584 bytes per 8,192 weights (unit64: 3,520; d is held by
// both lanes of a super-block).
constexpr int TILE16_BYTES = 3584, TILE16_B_AT = 2048, TILE16_C_AT = 3072, TILE16_SC_AT = 3328, TILE16_D_AT = 3456;
__device__ __forceinline__ SuperFields tile16_load(const uint8_t* __restrict__ we, int row, int S, int nsuper) {   // row: the lane's row
    typedef __attribute__((address_space(1))) const v4u g128;
    typedef __attribute__((address_space(1))) const uint32_t g32;
    typedef __attribute__((address_space(1))) const unsigned short g16;
    const int lane = (row & 15) | (int) (threadIdx.x & 48u);
    const gbytes u = as_global(we + ((size_t) (row >> 4) * nsuper + S) * TILE16_BYTES);
    SuperFields r;
    r.a0 = *(g128*) (u + 32 * lane);
    r.a1 = *(g128*) (u + 32 * lane + 16);
    r.b = *(g128*) (u + TILE16_B_AT + 16 * lane);
    r.c = *(g32*) (u + TILE16_C_AT + 4 * lane);
    r.sc = *(g16*) (u + TILE16_SC_AT + 2 * lane);
    r.d = *(g16*) (u + TILE16_D_AT + 2 * lane);
    return r;
}
// unit64 -> tile16 (once, at load; out of place): a wave a tile, every lane reads its four sub-blocks of its row
__global__ void __launch_bounds__(256) k_iq3s_tile16(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int nrows, int ncols, long tiles) {
    const long t = (long) blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= tiles) return;
    const int lane = threadIdx.x & 63, nsuper = ncols >> 9, ks = ncols >> 5;
    const long per = (long) (nrows >> 4) * nsuper;   // tiles a matrix
    const long m = t / per, tl = t - m * per;
    const int R = (int) (tl / nsuper), S = (int) (tl - (long) R * nsuper);
    const uint8_t* we = src + (size_t) m * ((size_t) nrows * ks / 64 * UNIT_BYTES);
    const SuperFields f = super_load(we, 16 * R + (lane & 15), 16 * S + 4 * (lane >> 4), ks);
    uint8_t* u = dst + (size_t) t * TILE16_BYTES;
    *reinterpret_cast<v4u*>(u + 32 * lane) = f.a0;
    *reinterpret_cast<v4u*>(u + 32 * lane + 16) = f.a1;
    *reinterpret_cast<v4u*>(u + TILE16_B_AT + 16 * lane) = f.b;
    *reinterpret_cast<uint32_t*>(u + TILE16_C_AT + 4 * lane) = f.c;
    *reinterpret_cast<unsigned short*>(u + TILE16_SC_AT + 2 * lane) = (unsigned short) f.sc;
    *reinterpret_cast<unsigned short*>(u + TILE16_D_AT + 2 * lane) = (unsigned short) f.d;
}
// tokens of a job's tile that the wave forms (k_moe_mma_wave16.h) multiply at a time: four tiles of 16
constexpr int MB_TP = 4, MB_TOK64 = 16 * MB_TP;

}  // namespace fnx
