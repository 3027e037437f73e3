// MI355X (gfx950) kernels and C ABI of the speculative-decode verify path: q8_1 activation quantisation, f32/bf16
// router mat-vec, top-k routing and job lists, IQ3_S x q8_1 expert mat-vec (gate|up, down, generic jobs), SwiGLU,
// combine, argmax, prompt-lookup drafting and greedy acceptance. Each entry point names the reference operator it
// replaces in include/fnx_mi355x.h.
//
// There is no CPU path in this library: every compute entry point launches HIP kernels and reports a HIP error
// through its status when no device can run them.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <type_traits>
#include <vector>

#include "../../include/fnx_mi355x.h"
#include "fnx_device.h"
#include "host_gguf.h"

namespace fnx {

// ================================================================ error plumbing
static thread_local std::string t_err;
static int fail(const std::string& m) {
    t_err = m;
    return 1;
}
static int launch_status(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(std::string(what) + ": " + hipGetErrorString(e));
    return 0;
}
static int env_int(const char* name, int dflt, int lo, int hi) {
    const char* s = std::getenv(name);
    if (!s || !*s) return dflt;
    char* end = nullptr;
    const long v = std::strtol(s, &end, 10);
    if (*end || v < lo || v > hi) {
        std::fprintf(stderr, "fnx: %s=%s ignored (want %d..%d)\n", name, s, lo, hi);
        return dflt;
    }
    return (int) v;
}

// ================================================================ device globals
__device__ const SignedGrid g_sgrid{};
// h = silu(gate) * up of every pair of the window as q8_1 rows, made once for moe_down (one MoE in flight per device,
// as the reference's g_moe_hq, moe.cuh:592-594)
constexpr int HQ_ROWS = FNX_MAXT * 10 + FNX_MAXT, HQ_MAX_FF = 1024;
__device__ uint8_t g_moe_hq[HQ_ROWS * (HQ_MAX_FF / 32) * FNX_Q8_1_BLOCK];

// ================================================================ q8_1 quantisation (kernels.cu:131-145)
// one 32-lane half-wave per block of 32 values
__device__ __forceinline__ void q8_1_store(float xi, uint8_t* blk, int lane32) {
    const float amax = group_max<32>(fabsf(xi)), sum = group_sum<32>(xi);
    const float d = amax / 127.0f;
    const int8_t qv = amax == 0.0f ? (int8_t) 0 : (int8_t) roundf(xi / d);
    reinterpret_cast<int8_t*>(blk + 4)[lane32] = qv;
    if (lane32 == 0) {
        reinterpret_cast<unsigned short*>(blk)[0] = float_to_half_bits(d);
        reinterpret_cast<unsigned short*>(blk)[1] = float_to_half_bits(sum);
    }
}
__global__ void __launch_bounds__(256) k_quantize_q8_1(const float* __restrict__ x, uint8_t* __restrict__ q, int n) {
    const int row = blockIdx.y, b = blockIdx.x * 8 + (threadIdx.x >> 5), lane = threadIdx.x & 31;
    if (b >= n / 32) return;
    const float xi = x[(size_t) row * n + b * 32 + lane];
    q8_1_store(xi, q + ((size_t) row * (n / 32) + b) * FNX_Q8_1_BLOCK, lane);
}
// h = silu(g) * u -> q8_1 (kernels.cu:400-410, moe.cuh:597-608). q null: the library's own pair buffer
__global__ void __launch_bounds__(256) k_swiglu_q8_1(const float* __restrict__ g, const float* __restrict__ u, size_t row_stride,
                                                    uint8_t* __restrict__ q, int n) {
    const int row = blockIdx.y, b = blockIdx.x * 8 + (threadIdx.x >> 5), lane = threadIdx.x & 31;
    if (b >= n / 32) return;
    const size_t i = (size_t) row * row_stride + b * 32 + lane;
    const float xi = silu_f(g[i]) * u[i];
    uint8_t* dst = q ? q : g_moe_hq;
    q8_1_store(xi, dst + ((size_t) row * (n / 32) + b) * FNX_Q8_1_BLOCK, lane);
}

// ================================================================ f32 / bf16 mat-vec (router; kernels.cu:239-287)
// A wave per weight row, the window's rows of x staged 256 columns at a time in LDS. Summation order (shared with
// the CPU oracle, so routing picks are bit-exact): lane l takes float4 chunks l, l + 64, ... in order, fmaf over
// x, y, z, w; then the xor-butterfly 32..1.
constexpr int GV_WAVES = 8;
template <bool BF>
__global__ void __launch_bounds__(GV_WAVES * 64) k_gemv_rows(const void* __restrict__ Wv, const float* __restrict__ x, float* __restrict__ y,
                                                            int rows, int n, int T) {
    __shared__ float4 xs[FNX_MAXT][64];
    // blockIdx.y: a group of FNX_MAXT activation rows (each (row, token) sum stands alone, so the grouping is free)
    x += (size_t) blockIdx.y * FNX_MAXT * n;
    y += (size_t) blockIdx.y * FNX_MAXT * rows;
    T = min(FNX_MAXT, T - (int) blockIdx.y * FNX_MAXT);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int row = blockIdx.x * GV_WAVES + wave;
    const bool live = row < rows;
    float acc[FNX_MAXT];
#pragma unroll
    for (int t = 0; t < FNX_MAXT; ++t) acc[t] = 0.f;
    for (int c0 = 0; c0 < n / 4; c0 += 64) {
        __syncthreads();
        for (int q = threadIdx.x; q < T * 64; q += GV_WAVES * 64) {
            const int t = q >> 6, l = q & 63;
            xs[t][l] = reinterpret_cast<const float4*>(x + (size_t) t * n)[c0 + l];
        }
        __syncthreads();
        if (live) {
            float4 w;
            if constexpr (BF) {
                const uint2 u = reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(Wv) + (size_t) row * n)[c0 + lane];
                w = make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                                __uint_as_float(u.y & 0xffff0000u));
            } else {
                w = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(Wv) + (size_t) row * n)[c0 + lane];
            }
#pragma unroll
            for (int t = 0; t < FNX_MAXT; ++t)
                if (t < T) {
                    const float4 b = xs[t][lane];
                    float a = acc[t];
                    a = fmaf(w.x, b.x, a);
                    a = fmaf(w.y, b.y, a);
                    a = fmaf(w.z, b.z, a);
                    a = fmaf(w.w, b.w, a);
                    acc[t] = a;
                }
        }
    }
    if (!live) return;
#pragma unroll
    for (int t = 0; t < FNX_MAXT; ++t)
        if (t < T) {
            const float v = group_sum<64>(acc[t]);
            if (lane == 0) y[(size_t) t * rows + row] = v;
        }
}

// ================================================================ top-k and jobs (moe.cuh:382-462, kernels.cu:381-398)
// One block; wave t ranks token t's logits: topk rounds of a wave arg-max, greater value first, lower index on a tie.
// Weights exp(l_k - l_0) / sum in pick order. Jobs: one per distinct expert, numbered by first pick, a job's pairs in
// ascending order (the order k_jobs gives).
constexpr int TK_MAXE = 1024, TK_THREADS = 1024;
__global__ void __launch_bounds__(TK_THREADS) k_topk_jobs(const float* __restrict__ logits, int stride, int T, int nexp, int topk,
                                                         int* __restrict__ topi, float* __restrict__ topw, fnx_job* __restrict__ gu,
                                                         fnx_job* __restrict__ dn, int* __restrict__ njobs, int both_counts,
                                                         int shared_job) {
    __shared__ int ex[FNX_MAXT * 64];
    __shared__ int jobof[TK_MAXE];
    __shared__ unsigned char isfirst[FNX_MAXT * 64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, P = T * topk;
    if (wave < T) {
        const int t = wave;
        float v[TK_MAXE / 64];
#pragma unroll
        for (int i = 0; i < TK_MAXE / 64; ++i) {
            const int e = lane + 64 * i;
            v[i] = e < nexp ? logits[(size_t) t * stride + e] : -INFINITY;
        }
        unsigned taken = 0;
        float top0 = 0.f, z = 0.f, wk = 0.f;
        for (int k = 0; k < topk; ++k) {
            float bv = -INFINITY;
            int bi = nexp;
#pragma unroll
            for (int i = 0; i < TK_MAXE / 64; ++i)
                if (!((taken >> i) & 1u) && v[i] > bv) {
                    bv = v[i];
                    bi = lane + 64 * i;
                }
#pragma unroll
            for (int o = 32; o; o >>= 1) {
                const float ov = __shfl_xor(bv, o, 64);
                const int oi = __shfl_xor(bi, o, 64);
                if (ov > bv || (ov == bv && oi < bi)) {
                    bv = ov;
                    bi = oi;
                }
            }
            const bool found = bi < nexp;
            if (!found) {   // nothing above -inf is left (masked or NaN logits): the lowest index not yet picked, at weight 0
                bi = 0x7fffffff;
#pragma unroll
                for (int i = TK_MAXE / 64 - 1; i >= 0; --i)
                    if (lane + 64 * i < nexp && !((taken >> i) & 1u)) bi = lane + 64 * i;
#pragma unroll
                for (int o = 32; o; o >>= 1) bi = min(bi, __shfl_xor(bi, o, 64));
            }
            if (bi < nexp && (bi & 63) == lane) taken |= 1u << (bi >> 6);
            if (k == 0) top0 = bv;
            const float ek = found ? fnx_expf(bv - top0) : 0.f;
            z += ek;
            if (lane == k) {
                wk = ek;
                const int pick = bi < nexp ? bi : nexp - 1;   // more picks than experts: refused by the host, kept inside the tables here
                topi[t * topk + k] = pick;
                ex[t * topk + k] = pick;
            }
        }
        if (lane < topk) topw[t * topk + lane] = z > 0.f ? wk / z : 0.f;
    }
    __syncthreads();
    if (!gu) return;
    const int p = threadIdx.x;
    int slot = 0, e = -1;
    if (p < P) {
        e = ex[p];
        for (int q = 0; q < p; ++q) slot += ex[q] == e;
        isfirst[p] = slot == 0;
    }
    __syncthreads();
    if (p < P && slot == 0) {
        int j = 0, cnt = 0;
        for (int q = 0; q < p; ++q) j += isfirst[q];
        for (int q = 0; q < P; ++q) cnt += ex[q] == e;
        jobof[e] = j;
        gu[j].w = dn[j].w = e;
        gu[j].n = dn[j].n = cnt;
    }
    __syncthreads();
    if (p < P) {
        const int j = jobof[e];
        gu[j].y[slot] = p / topk;
        gu[j].out[slot] = p;
        dn[j].y[slot] = p;
        dn[j].out[slot] = p;
    }
    if (p == P) {
        int nj = 0;
        for (int q = 0; q < P; ++q) nj += isfirst[q];
        njobs[0] = nj;
        if (both_counts) njobs[1] = nj;
    }
    // the shared expert's job at index P: every row of the window, outputs at rows P + t (kernels.hpp:277-282)
    if (shared_job && p < T) {
        gu[P].y[p] = p;
        gu[P].out[p] = P + p;
        dn[P].y[p] = P + p;
        dn[P].out[p] = P + p;
        if (p == 0) {
            gu[P].w = dn[P].w = 0;
            gu[P].n = dn[P].n = T;
        }
    }
}

// ================================================================ IQ3_S x q8_1 jobs: the expert mat-vec
// (k_mmvq kernels.cu:192-229, k_moe_gu moe.cuh:572-585, k_moe_down moe.cuh:613-658, vec_dot iq3s_x.cuh:4-41)
//
// Work is cut in units of 64 sub-blocks of 32 weights = 880 contiguous bytes: one row of 2048 columns, 4 rows of
// 512, 8 rows of 256. Lane l of a wave owns sub-block l of the unit: it reads its 8 code bytes, its sign dword, its
// high-bit byte and scale nibble straight from the raw ggml block, builds eight 13-bit indexes (sign nibble | high
// bit | code) into the signed codebook in LDS and feeds each looked-up dword to v_dot4_i32_i8 against the token's
// int8 activations, which stay in registers for the whole job (a lane's sub-block column never changes).
// The waves of the grid split the units of all jobs evenly and walk them in order: consecutive rows, one expert
// after the other, so every wave streams contiguous memory.
struct RowsArgs {
    const uint8_t* wbase;
    size_t w_stride;
    const uint8_t* const* ep;
    size_t row_bytes;
    int nrows, ncols;
    const fnx_job* jobs;
    const int* njobs;
    int njobs_max;
    const uint8_t* y;   // q8_1 rows; null: the library's pair buffer
    float* out;
    int out_stride;
    // the prompt path's jobs of up to FNX_PF_JOB rows (k_iq3s_jobs_mma16<1 | 2>), instead of `jobs`; gu: their activations are
    // made on the way from rows [gate | up] of 2 ncols floats (h = silu(gate) * up as q8_1), instead of read from y
    const fnx_bigjob* big = nullptr;
    const float* gu = nullptr;
};

struct RawSub {   // one lane's share of a unit as read from memory; nothing is combined until it is used
    uint32_t q0, q1, sg, qh, sc, d;   // codes 0..3, 4..7, sign nibbles, high bits, scales byte, d bits
};
struct LaneOffs {   // byte offsets of a lane's fields inside a unit
    uint32_t d, qs, qh, sg, sc;
};
__device__ __forceinline__ RawSub load_sub(gbytes unit, const LaneOffs& o) {   // unit: wave-uniform; o: per lane
    typedef __attribute__((address_space(1), aligned(2))) const uint32_t gu32;
    typedef __attribute__((address_space(1), aligned(2))) const unsigned short gu16;
    // the empty asm keeps each 32-bit offset's zero-extension next to its load, where instruction selection can fold
    // it into the SGPR-base addressing form (hoisted out of the loop it becomes a 64-bit add per load)
    uint32_t od = o.d, oq = o.qs, os = o.sg, oh = o.qh, oc = o.sc;
    asm volatile("" : "+v"(od), "+v"(oq), "+v"(os), "+v"(oh), "+v"(oc));
    RawSub r;
    r.d = *(gu16*) (unit + od);
    r.q0 = *(gu32*) (unit + oq);
    r.q1 = *(gu32*) (unit + oq + 4);
    r.sg = *(gu32*) (unit + os);
    r.qh = unit[oh];
    r.sc = unit[oc];
    return r;
}

// byte address into the signed codebook of group j of a sub-block: (sign nibble << 9 | high bit << 8 | code) * 4.
// Five VALU ops: byte select with shift (SDWA), two shifts, two and-or; the empty asm keeps the two and-or apart.
__device__ __forceinline__ uint32_t code_addr(const RawSub& r, int j) {
    uint32_t a = (((j < 4 ? r.q0 : r.q1) >> (8 * (j & 3))) & 0xFFu) << 2;
    const uint32_t sg = 4 * j <= 11 ? r.sg << (11 - 4 * j) : r.sg >> (4 * j - 11);
    a = (sg & 0x7800u) | a;
    asm volatile("" : "+v"(a));
    const uint32_t qh = r.qh << (10 - j);
    return (qh & 0x400u) | a;
}

// sum over groups of `width` lanes with DPP moves (no LDS traffic). The lane with the highest index of each group
// ends with the group's sum (for width <= 16 every lane does).
template <int width>
__device__ __forceinline__ float dpp_group_sum(float v) {
#define FNX_DPP_ADD(ctrl, rmask)                                                                                          \
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, rmask, 0xF, false))
    if constexpr (width >= 2) FNX_DPP_ADD(0xB1, 0xF);    // quad_perm [1,0,3,2]
    if constexpr (width >= 4) FNX_DPP_ADD(0x4E, 0xF);    // quad_perm [2,3,0,1]
    if constexpr (width >= 8) FNX_DPP_ADD(0x141, 0xF);   // row_half_mirror
    if constexpr (width >= 16) FNX_DPP_ADD(0x140, 0xF);  // row_mirror
    if constexpr (width >= 32) FNX_DPP_ADD(0x142, 0xA);  // row_bcast15 into rows 1 and 3
    if constexpr (width >= 64) FNX_DPP_ADD(0x143, 0xC);  // row_bcast31 into rows 2 and 3
#undef FNX_DPP_ADD
    return v;
}

// SBR: sub-blocks per weight row (ncols / 32), a power of two <= 64. NT: tokens of the job held in registers.
// R: units in flight per wave: the loads of the next R units are issued before the current R are decoded.
template <int SBR, int NT, int R>
__device__ __forceinline__ void job_units(const uint32_t* __restrict__ tab, const uint8_t* __restrict__ we, size_t row_bytes, int ua,
                                          int ub, const fnx_job* __restrict__ jb, int t0, const uint8_t* __restrict__ y,
                                          float* __restrict__ out, int out_stride) {
    constexpr int RW = 64 / SBR;   // rows per unit
    const int lane = threadIdx.x & 63, g = lane / SBR, kb = lane % SBR, sb = kb >> 3, ib = kb & 7;
    int xs[NT][8];
    float dx[NT];
    float* orow[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const uint8_t* yb = y + ((size_t) uniform(jb->y[t0 + t]) * SBR + kb) * FNX_Q8_1_BLOCK;
        dx[t] = half_bits_to_float(*reinterpret_cast<const unsigned short*>(yb));
#pragma unroll
        for (int j = 0; j < 8; ++j) xs[t][j] = reinterpret_cast<const int*>(yb + 4)[j];
        orow[t] = out + (size_t) uniform(jb->out[t0 + t]) * out_stride + g;
    }
    LaneOffs o;
    o.d = (uint32_t) (g * row_bytes) + sb * FNX_IQ3S_BLOCK;
    o.qs = o.d + 2 + 8 * ib;
    o.qh = o.d + 66 + ib;
    o.sg = o.d + 74 + 4 * ib;
    o.sc = o.d + 106 + (ib >> 1);
    const size_t step = (size_t) RW * row_bytes;
    const int last = ub - 1;
    // a unit's address as a scalar pair, the lane's field offsets as 32-bit registers: global_load with an SGPR base
    auto unit_at = [&](int ui) { return as_global(uniform_ptr(we + (size_t) min(ui, last) * step)); };
    const int sc_shift = 4 * (ib & 1);
    RawSub cur[R];
#pragma unroll
    for (int r = 0; r < R; ++r) cur[r] = load_sub(unit_at(ua + r), o);
    for (int u = ua; u < ub; u += R) {
        RawSub nxt[R];
#pragma unroll
        for (int r = 0; r < R; ++r) nxt[r] = load_sub(unit_at(u + R + r), o);   // past the end: the last unit again
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int w4[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) w4[j] = *reinterpret_cast<const int*>(reinterpret_cast<const uint8_t*>(tab) + code_addr(cur[r], j));
            const int sc = 1 + 2 * (int) ((cur[r].sc >> sc_shift) & 0xFu);
            const float dw = half_bits_to_float(cur[r].d);
            const bool store = kb == SBR - 1 && u + r < ub;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                int sum = 0;
#pragma unroll
                for (int j = 0; j < 8; ++j) sum = __builtin_amdgcn_sdot4(w4[j], xs[t][j], sum, false);
                // one sub-block's term exactly as the reference forms it: (d_w * d_x) * (float) (sumi * (1 + 2 s))
                const float v = butterfly_sum<SBR>((dw * dx[t]) * (float) __mul24(sum, sc));
                if (store) orow[t][(size_t) (u + r) * RW] = v;
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) cur[r] = nxt[r];
    }
}

// WIDE: jobs of many rows go up to sixteen tokens at a time in the unit64 layout (four with raw blocks, fewer units in
// flight to stay within the registers); the narrow
// variant takes one or two tokens a pass, which is what a verify window's routed jobs have (1.15 rows on average)
template <int SBR, bool WIDE>
__device__ __forceinline__ void job_range(const uint32_t* tab, const uint8_t* we, const RowsArgs& a, int ua, int ub, const fnx_job* jb,
                                          const uint8_t* y) {
    const int n = uniform(jb->n);
    for (int t0 = 0; t0 < n;) {
        const int nt = n - t0;
        if (WIDE && nt >= 4) {
            job_units<SBR, 4, 2>(tab, we, a.row_bytes, ua, ub, jb, t0, y, a.out, a.out_stride);
            t0 += 4;
        } else if (WIDE && nt == 3) {
            job_units<SBR, 3, 2>(tab, we, a.row_bytes, ua, ub, jb, t0, y, a.out, a.out_stride);
            t0 += 3;
        } else if (nt >= 2) {
            job_units<SBR, 2, 4>(tab, we, a.row_bytes, ua, ub, jb, t0, y, a.out, a.out_stride);
            t0 += 2;
        } else {
            job_units<SBR, 1, 4>(tab, we, a.row_bytes, ua, ub, jb, t0, y, a.out, a.out_stride);
            t0 += 1;
        }
    }
}

}  // namespace fnx
#include "k_iq3s_packed.h"
namespace fnx {

// requires nrows % (64 / SBR) == 0 (checked by the launcher): every unit is whole. PACKED: the unit64 layout.
// The waves of the grid split the units of all jobs evenly and walk them in order (consecutive rows, one expert after
// the other), so a wave streams one contiguous range of memory and changes job at most once or twice.
template <int SBR, bool WIDE, bool PACKED>
__global__ void __launch_bounds__(512) k_iq3s_jobs(const RowsArgs a) {
    __shared__ uint32_t tab[SGRID_WORDS];
    for (int g = threadIdx.x; g < 512; g += blockDim.x) {   // a code's sixteen signed entries from its unsigned one
        const uint32_t g0 = g_sgrid.v[g];
#pragma unroll
        for (int sg = 0; sg < 16; ++sg) tab[sg * 512 + g] = signed_entry(g0, sg);
    }
    constexpr int RW = 64 / SBR;
    const int nj = a.njobs ? min(uniform(*a.njobs), a.njobs_max) : a.njobs_max;
    __syncthreads();
    // unit numbers fit 32 bits (the launcher checks); the shares' products need 64 only for very large launches
    // (a 64-bit division is a few hundred instructions, and every wave of the grid makes them as it starts)
    const uint32_t upj = a.nrows / RW;   // units per job
    const uint32_t total = (uint32_t) nj * upj;
    const uint32_t wpb = blockDim.x >> 6;
    const uint32_t gw = blockIdx.x * wpb + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), nw = gridDim.x * wpb;
    uint32_t u, u1;
    if ((unsigned long long) total * nw >> 32 == 0) {
        u = total * gw / nw;
        u1 = total * (gw + 1) / nw;
    } else {
        u = (uint32_t) ((unsigned long long) total * gw / nw);
        u1 = (uint32_t) ((unsigned long long) total * (gw + 1) / nw);
    }
    const uint8_t* y = a.y ? a.y : g_moe_hq;
    while (u < u1) {
        const uint32_t ji = u / upj;
        const int ul = (int) (u - ji * upj);
        const int ue = (int) min(upj, ul + (u1 - u));
        const fnx_job* jb = a.jobs + ji;
        const int w = uniform(jb->w);
        const uint8_t* we = a.ep ? uniform_ptr(a.ep[w]) : a.wbase + (size_t) w * a.w_stride;
        if constexpr (PACKED) packed_range<SBR, WIDE>(tab, we, ul, ue, jb, y, a.out, a.out_stride);
        else job_range<SBR, WIDE>(tab, we, a, ul, ue, jb, y);
        u += ue - ul;
    }
}

}  // namespace fnx
#include "k_iq3s_mma.h"
#include "k_moe_layer.h"
#include "k_moe_window.h"
#include "k_prefill.h"
#include "k_iq3s_mma16.h"
#include "k_moe_mma_wave16.h"
#include "k_decoder.h"
#include "k_round.h"
#include "k_sampler.h"
#include "k_qtypes.h"
#include "k_stream.h"
namespace fnx {

// any other row length (a multiple of 256): a wave per (row, job), sub-blocks dealt round-robin to the lanes, the
// codebook read from global memory. Not a tuned path.
__global__ void __launch_bounds__(256) k_iq3s_jobs_any(const RowsArgs a) {
    const int ji = blockIdx.y;
    if (ji >= (a.njobs ? min(*a.njobs, a.njobs_max) : a.njobs_max)) return;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= a.nrows) return;
    const fnx_job* jb = a.jobs + ji;
    const uint8_t* we = (a.ep ? a.ep[jb->w] : a.wbase + (size_t) jb->w * a.w_stride) + (size_t) row * a.row_bytes;
    const uint8_t* y = a.y ? a.y : g_moe_hq;
    const int sbr = a.ncols / 32;
    for (int t = 0; t < jb->n; ++t) {
        float acc = 0.f;
        for (int kb = lane; kb < sbr; kb += 64) {
            const int ib = kb & 7;
            LaneOffs o;
            o.d = (uint32_t) (kb >> 3) * FNX_IQ3S_BLOCK;
            o.qs = o.d + 2 + 8 * ib;
            o.qh = o.d + 66 + ib;
            o.sg = o.d + 74 + 4 * ib;
            o.sc = o.d + 106 + (ib >> 1);
            const RawSub r = load_sub(as_global(we), o);
            const uint8_t* yb = y + ((size_t) jb->y[t] * sbr + kb) * FNX_Q8_1_BLOCK;
            int sum = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                sum = __builtin_amdgcn_sdot4((int) g_sgrid.v[code_addr(r, j) >> 2], reinterpret_cast<const int*>(yb + 4)[j], sum, false);
            }
            const int sc = 1 + 2 * (int) ((r.sc >> (4 * (ib & 1))) & 0xFu);
            acc += (half_bits_to_float(r.d) * half_bits_to_float(*reinterpret_cast<const unsigned short*>(yb))) * (float) (sum * sc);
        }
        acc = group_sum<64>(acc);
        if (lane == 0) a.out[(size_t) jb->out[t] * a.out_stride + row] = acc;
    }
}

// ================================================================ combine (kernels.cu:412-419)
__global__ void __launch_bounds__(256) k_combine(const float* __restrict__ part, const float* __restrict__ topw, const float* __restrict__ sh,
                                                const float* __restrict__ sh_logit, int sh_logit_stride, float* __restrict__ out, int n,
                                                int topk) {
    const int t = blockIdx.y, i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    // the chain in pick order, eight partial sums in flight at a time (one load per trip of the loop otherwise)
    const float shv = sh[(size_t) t * n + i], sg = sigmoid_f(sh_logit[(size_t) t * sh_logit_stride]);
    float s = 0.f;
    int k0 = 0;
    for (; k0 + 8 <= topk; k0 += 8) {
        float pv[8], wk[8];
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            wk[kk] = topw[t * topk + k0 + kk];
            pv[kk] = part[((size_t) t * topk + k0 + kk) * n + i];
        }
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) s = fmaf(wk[kk], pv[kk], s);
    }
    if (k0 < topk) {   // the last few together too
        float pv[8], wk[8];
#pragma unroll
        for (int kk = 0; kk < 8; ++kk)
            if (k0 + kk < topk) {
                wk[kk] = topw[t * topk + k0 + kk];
                pv[kk] = part[((size_t) t * topk + k0 + kk) * n + i];
            }
#pragma unroll
        for (int kk = 0; kk < 8; ++kk)
            if (k0 + kk < topk) s = fmaf(wk[kk], pv[kk], s);
    }
    out[(size_t) t * n + i] = s + sg * shv;
}

// ================================================================ argmax (kernels.cu:1045-1083)
__device__ __forceinline__ unsigned fkey(float v) {
    const unsigned u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float fkey_inv(unsigned k) { return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k); }
constexpr int AM_THREADS = 1024, AM_PER_BLOCK = 16384;
// keys[t] = max over the row of (fkey(value) << 32 | ~index): the greatest value, the lower index on a tie. A block
// folds its 16,384 values to one key (four independent 16-byte loads a thread, wave butterflies, LDS) and issues one
// atomic: atomics on one address serialise, and a row's address would otherwise take one per wave. The row's last block
// to arrive (a count beside the keys, keys[FNX_MAXT + t]) decodes the key into (value, index + v0) and leaves both words
// at zero for the next argmax.
__global__ void __launch_bounds__(AM_THREADS) k_argmax(const float* __restrict__ logits, int rows, unsigned long long* __restrict__ keys,
                                                      unsigned* __restrict__ err, int v0, float* __restrict__ bv, int* __restrict__ bi,
                                                      const int* __restrict__ live) {
    __shared__ unsigned long long wbest[AM_THREADS / 64];
    __shared__ int wbad;
    // live (may be null): a device word; rows from *live on do not count: they are not scanned and their picks stay what they were
    if (live && (int) blockIdx.y >= max(1, *live)) return;
    const int t = blockIdx.y, i0 = blockIdx.x * AM_PER_BLOCK, i1 = min(rows, i0 + AM_PER_BLOCK), tid = threadIdx.x;
    const float* r = logits + (size_t) t * rows;
    if (tid == 0) wbad = 0;
    unsigned long long best = 0;
    bool bad = false;
    auto take = [&](float v, int i) {
        bad = bad || !isfinite(v);
        const unsigned long long k = (unsigned long long) fkey(v) << 32 | (unsigned) ~i;
        best = k > best ? k : best;
    };
    if ((((uintptr_t) r) & 15) == 0 && (i0 & 3) == 0) {
        float4 v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = i0 + 4 * (tid + AM_THREADS * j);
            v[j] = i + 3 < i1 ? *reinterpret_cast<const float4*>(r + i) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = i0 + 4 * (tid + AM_THREADS * j);
            if (i + 3 < i1) {
                take(v[j].x, i);
                take(v[j].y, i + 1);
                take(v[j].z, i + 2);
                take(v[j].w, i + 3);
            } else {
                for (int k = i; k < i1; ++k) take(r[k], k);
            }
        }
    } else {
        for (int i = i0 + tid; i < i1; i += AM_THREADS) take(r[i], i);
    }
#pragma unroll
    for (int o = 32; o; o >>= 1) {
        const unsigned long long ok = __shfl_xor(best, o, 64);
        best = ok > best ? ok : best;
    }
    __syncthreads();
    if (bad) wbad = 1;
    if ((tid & 63) == 0) wbest[tid >> 6] = best;
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < AM_THREADS / 64; ++w) best = wbest[w] > best ? wbest[w] : best;
        if (wbad) atomicOr(err, FNX_ERR_NONFINITE);
        // the maximum has been taken at the device's level (its old value is back) before this block counts as arrived
        const unsigned long long old = __hip_atomic_fetch_max(&keys[t], best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long mine = old > best ? old : best;
        asm volatile("" ::"v"(mine));
        const unsigned long long arrived = __hip_atomic_fetch_add(&keys[FNX_MAXT + t], 1ull, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        if (arrived == gridDim.x - 1) {
            const unsigned long long k = __hip_atomic_load(&keys[t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            bv[t] = fkey_inv((unsigned) (k >> 32));
            bi[t] = (int) ~(unsigned) k + v0;
            __hip_atomic_store(&keys[t], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&keys[FNX_MAXT + t], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// ================================================================ prompt lookup and acceptance on the device
// (session.cpp:428-447, 573). One block: every thread tests its share of start positions for the key, the block keeps
// the greatest matching start, the first wave measures the backward match and copies the drafts (a lane per token).
// Nothing here waits for one load after another: a thread's loads of a round are issued together (four start positions
// a step - the 4 + 3 tokens they need are two 16-byte loads - and LK_STEPS steps a round), and the match and the copy are
// a ballot each.
constexpr int LK_THREADS = 1024, LK_STEPS = 10, LOOKUP_MIN = 3, IMAGE_TOK = 1 << 30;   // 40,960 start positions a round
// n_ctx_p (may be null): the context's length is that device word instead of n_ctx; d1_at (may be null): d1 is
// d1p[*d1_at - 1] instead of d1p[0] (the pick of the last row kept). rs, rs_rows (may be null; only with n_ctx_p and d1_at
// the round's own words): a decode round's state and window - the round's next window (k_round_window's rows and count,
// k_round.h) is made here as well, from the drafts this launch finds: a launch less a round.
__global__ void __launch_bounds__(LK_THREADS) k_lookup(const int* __restrict__ ctx, int n_ctx, int key_n, int lk, const int* __restrict__ d1p,
                                                      int* __restrict__ out, int* __restrict__ n_out, int* __restrict__ match,
                                                      const int* __restrict__ n_ctx_p, const int* __restrict__ d1_at,
                                                      int* __restrict__ rs = nullptr, int* __restrict__ rs_rows = nullptr) {
    __shared__ int best;
    if (threadIdx.x == 0) best = -1;
    if (n_ctx_p) n_ctx = *n_ctx_p;
    const int d1 = d1p[d1_at ? min(max(*d1_at, 1), FNX_MAXT) - 1 : 0];   // asked for now, used at the end
    // (what the next window needs beside the drafts, asked for now as well)
    const int rs_stop = rs ? rs[FNX_RS_STOP] : 1, last_tok = rs && n_ctx > 0 ? ctx[n_ctx - 1] : 0;
    __syncthreads();
    const int n0 = n_ctx - key_n;
    if (lk > 0 && n0 > 0) {
        int key[4];
        for (int j = 0; j < key_n; ++j) key[j] = ctx[n0 + j];
        int mine = -1;
        // start positions below vec_end are tested four at a time from whole 16-byte loads; the few after them one by one
        const bool aligned = (((uintptr_t) ctx) & 15) == 0;
        const int vec_end = aligned && n_ctx >= 8 ? ((n_ctx - 8) / 4) * 4 + 4 : 0;
        for (int base = 0; base < vec_end; base += 4 * LK_THREADS * LK_STEPS) {
            int4 a[LK_STEPS], b[LK_STEPS];
#pragma unroll
            for (int k = 0; k < LK_STEPS; ++k) {
                const int s4 = min(base + 4 * ((int) threadIdx.x + LK_THREADS * k), vec_end - 4);   // past the end: the last step again
                a[k] = *reinterpret_cast<const int4*>(ctx + s4);
                b[k] = *reinterpret_cast<const int4*>(ctx + s4 + 4);
            }
#pragma unroll
            for (int k = 0; k < LK_STEPS; ++k) {
                const int s4 = base + 4 * ((int) threadIdx.x + LK_THREADS * k);
                const int w[8] = {a[k].x, a[k].y, a[k].z, a[k].w, b[k].x, b[k].y, b[k].z, b[k].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    bool eq = s4 < vec_end && s4 + i < n0;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (j < key_n) eq = eq && w[i + j] == key[j];
                    if (eq) mine = s4 + i;   // ascending: the last one kept is this thread's greatest
                }
            }
        }
        for (int s = vec_end + threadIdx.x; s < n0; s += LK_THREADS) {
            bool eq = true;
            for (int j = 0; j < key_n; ++j) eq = eq && ctx[s + j] == key[j];
            if (eq) mine = s;   // ascending s: the last one kept is this thread's greatest
        }
#pragma unroll
        for (int o = 32; o; o >>= 1) mine = max(mine, __shfl_xor(mine, o, 64));
        if ((threadIdx.x & 63) == 0 && mine >= 0) atomicMax(&best, mine);
    }
    __syncthreads();
    if (threadIdx.x >= 64) return;
    const int lane = threadIdx.x;
    int nr = 0, m_at = -1, dtok = 0;   // (dtok: this lane's draft)
    const int s = best;
    if (s >= 0 && s + key_n < n_ctx) {
        // one trip to memory for everything the rest needs: the tokens before the match and before the key (lane j: the
        // j-th back), and the up to lk tokens after the match (lane i: the i-th)
        const int back = min(lk - key_n, s);
        const int before_s = lane < back ? ctx[s - 1 - lane] : 0, before_k = lane < back ? ctx[n0 - 1 - lane] : 1;
        const int tok = lane < lk && s + key_n + lane < n_ctx ? ctx[s + key_n + lane] : 0;
        const int first = __builtin_amdgcn_readfirstlane(tok);   // ctx[s + key_n]
        if (d1 >= 0 && first != d1) goto done;
        // m = key_n + the tokens before the match that also agree (at most lk - key_n of them, and not before the context's start)
        const unsigned long long miss = ~__ballot(before_s == before_k);   // lanes >= back are misses: the count stops there at the latest
        const int m = key_n + (int) __builtin_ctzll(miss | (1ull << 63));
        const int k = min(lk, max(LOOKUP_MIN, m)), end = min(n_ctx, s + key_n + k), want = end - (s + key_n);
        // the drafts: a lane per token; an image cell is never a draft, nor anything after it
        const unsigned long long stop = __ballot(lane < want && tok >= IMAGE_TOK);
        nr = stop ? min(want, (int) __builtin_ctzll(stop)) : want;
        if (lane < nr) out[lane] = dtok = tok;
        m_at = s;
    }
done:
    if (lane == 0) {
        *n_out = nr;
        if (match) *match = m_at;
    }
    if (rs && !rs_stop) {   // session.cpp:530-560: the context's last token, then the drafts, or else the draft layer's pick
        const int nd = min(nr, FNX_MAXT - 1), before = __shfl_up(dtok, 1, 64);   // lane i: draft i - 1
        int tok = 0;
        if (lane == 0) tok = last_tok;
        else if (nd > 0) tok = lane <= nd ? before : 0;
        else if (lane == 1) tok = d1;
        if (lane < FNX_MAXT) rs_rows[lane] = tok;
        if (lane == 0) rs[FNX_RS_ROWS] = nd > 0 ? 1 + nd : 2;
    }
}
__global__ void k_accept(const int* __restrict__ rows, const int* __restrict__ o, int R, int* __restrict__ n_accept) {
    const int i = threadIdx.x;   // one wave; lane i tests draft i + 1 against row i's pick
    const bool ok = i + 1 < R && rows[i + 1] == o[i];
    const unsigned long long b = __ballot(ok);
    if (i == 0) n_accept[0] = 1 + __builtin_ctzll(~b);
}

// ================================================================ launchers
static int cu_count() {
    static int cus[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (!cus[dev]) {
        int n = 0;
        cus[dev] = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0 ? n : 256;
    }
    return cus[dev];
}
// The library's own device buffers that one call's kernels write and then read (the pair buffer of q8_1 rows behind
// moe_down and the operator-by-operator window, the sampler's candidate lists): one per device, as the reference's
// (moe.cuh:592-594), so calls that use one must not overlap. Calls on different streams are put in order here: a call
// waits for the event the call before it recorded, and records its own when its launches are enqueued. A stream under
// graph capture is left alone (waiting for an event from outside would end the capture): a captured graph that holds such
// calls must not be replayed beside other users of the buffer.
struct BufferOrder {
    std::mutex m;
    hipEvent_t ev[64] = {};
    hipStream_t last[64] = {};
    bool used[64] = {};
    static bool capturing(hipStream_t s) {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        return hipStreamIsCapturing(s, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone;
    }
    void enter(hipStream_t s) {
        int dev = -1;
        if (capturing(s) || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return;
        std::lock_guard<std::mutex> g(m);
        if (used[dev] && last[dev] != s) (void) hipStreamWaitEvent(s, ev[dev], 0);
    }
    void leave(hipStream_t s) {
        int dev = -1;
        if (capturing(s) || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return;
        std::lock_guard<std::mutex> g(m);
        if (!ev[dev] && hipEventCreateWithFlags(&ev[dev], hipEventDisableTiming) != hipSuccess) return;
        if (hipEventRecord(ev[dev], s) == hipSuccess) {
            used[dev] = true;
            last[dev] = s;
        }
    }
};
static BufferOrder g_pair_order, g_cand_order;
// The one-launch window's blocks wait for each other, which needs all of them resident: a grid of one block a CU, alone
// on the chip. Two windows enqueued on two streams could be dispatched block by block beside each other, each holding
// CUs the other waits for, until both give up their waits. So a window on another stream than the window before it first
// waits for everything enqueued on that stream so far (an event recorded there now); windows on one stream, the usual
// case, pay nothing. A stream under graph capture is left alone, as in BufferOrder.
struct WindowOrder {
    std::mutex m;
    hipEvent_t ev[64] = {};
    hipStream_t last[64] = {};
    bool used[64] = {};
    void enter(hipStream_t s) {
        int dev = -1;
        if (BufferOrder::capturing(s) || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return;
        std::lock_guard<std::mutex> g(m);
        if (used[dev] && last[dev] != s) {
            if (!ev[dev] && hipEventCreateWithFlags(&ev[dev], hipEventDisableTiming) != hipSuccess) ev[dev] = nullptr;
            if (ev[dev] && hipEventRecord(ev[dev], last[dev]) == hipSuccess) (void) hipStreamWaitEvent(s, ev[dev], 0);
            else (void) hipGetLastError();   // (the stream before may be gone: then nothing of it is left to wait for)
        }
        used[dev] = true;
        last[dev] = s;
    }
};
static WindowOrder g_window_order;
struct BufferScope {   // enter now, leave when the call returns
    BufferOrder& o;
    hipStream_t s;
    BufferScope(BufferOrder& o_, void* st) : o(o_), s((hipStream_t) st) { o.enter(s); }
    ~BufferScope() { o.leave(s); }
};

// wide: the jobs are expected to hold many rows each (a dense matrix over the whole window) rather than one or two
static int rows_launch(const fnx_dw* W, size_t w_stride, const fnx_job* jobs, const int* njobs, int njobs_max, const void* y, float* out,
                       int out_stride, void* st, const char* who, bool wide = false) {
    if (!W || !jobs || !out) return fail(std::string(who) + ": null argument");
    if (W->type == QT_Q4_0 || W->type == QT_Q5_1 || W->type == QT_Q8_0 || W->type == QT_IQ4_NL || W->type == QT_IQ4_XS || W->type == QT_Q4_K || W->type == QT_Q5_K) {
        // the other types of kernels.cu:2454-2471 that the reference's own host code can decode (k_qtypes.h)
        gguf::BlockShape bs{};
        gguf::block_shape(W->type, bs);
        if (W->n_in <= 0 || W->n_in % bs.values || W->n_out <= 0) return fail(std::string(who) + ": shape does not fit the type's blocks");
        if (W->row_bytes != (size_t) (W->n_in / bs.values) * (size_t) bs.bytes) return fail(std::string(who) + ": row_bytes does not match n_in");
        if (njobs_max <= 0) return fail(std::string(who) + ": njobs_max must be positive");
        if (!W->p && !W->ep) return fail(std::string(who) + ": no weights");
        const QtArgs q{(const uint8_t*) W->p, w_stride, (const uint8_t* const*) W->ep, W->row_bytes, W->n_out, W->n_in, jobs, njobs, njobs_max,
                       (const uint8_t*) y, out, out_stride};
        const dim3 grid((W->n_out + 3) / 4, njobs_max);
        hipStream_t s = (hipStream_t) st;
        switch (W->type) {
            case QT_Q4_0: k_qt_jobs<QT_Q4_0><<<grid, 256, 0, s>>>(q); break;
            case QT_Q5_1: k_qt_jobs<QT_Q5_1><<<grid, 256, 0, s>>>(q); break;
            case QT_Q8_0: k_qt_jobs<QT_Q8_0><<<grid, 256, 0, s>>>(q); break;
            case QT_IQ4_NL: k_qt_jobs<QT_IQ4_NL><<<grid, 256, 0, s>>>(q); break;
            case QT_IQ4_XS: k_qt_jobs<QT_IQ4_XS><<<grid, 256, 0, s>>>(q); break;
            case QT_Q4_K: k_qt_jobs<QT_Q4_K><<<grid, 256, 0, s>>>(q); break;
            default: k_qt_jobs<QT_Q5_K><<<grid, 256, 0, s>>>(q); break;
        }
        return launch_status(who);
    }
    if (W->type == FNX_T_IQ3S_TILE16) {   // the prompt path's layout: jobs of many rows, decoded straight into matrix-core operands (k_iq3s_mma16.h)
        if (W->n_in <= 0 || W->n_in % 512 || W->n_in > J16_MAXCOLS || W->n_out <= 0 || W->n_out % 16)
            return fail(std::string(who) + ": the tile16 layout takes rows in 16s and 512, 1024, 1536 or 2048 columns here");
        if (W->row_bytes != (size_t) (W->n_in / 256) * FNX_IQ3S_BLOCK) return fail(std::string(who) + ": row_bytes does not match n_in");
        if (njobs_max <= 0) return fail(std::string(who) + ": njobs_max must be positive");
        if (!W->p && !W->ep) return fail(std::string(who) + ": no weights");
        const RowsArgs a{(const uint8_t*) W->p, w_stride, (const uint8_t* const*) W->ep, W->row_bytes, W->n_out, W->n_in,
                         jobs, njobs, njobs_max, (const uint8_t*) y, out, out_stride};
        const long items = (long) njobs_max * (W->n_out / 16);
        k_iq3s_jobs_mma16<0><<<(int) std::max(1L, std::min((long) cu_count(), items)), J16_THREADS, 0, (hipStream_t) st>>>(a);
        return launch_status(who);
    }
    if (W->type != FNX_T_IQ3_S && W->type != FNX_T_IQ3S_UNIT64)
        return fail(std::string(who) + ": expert type " + std::to_string(W->type) +
                    " not handled (IQ3_S, and Q4_0, Q5_1, Q8_0, IQ4_NL, IQ4_XS, Q4_K, Q5_K through the plain path)");
    if (W->n_in <= 0 || W->n_in % 256 || W->n_out <= 0) return fail(std::string(who) + ": shape does not fit IQ3_S super-blocks");
    if (W->row_bytes != (size_t) (W->n_in / 256) * FNX_IQ3S_BLOCK) return fail(std::string(who) + ": row_bytes does not match n_in");
    if (njobs_max <= 0) return fail(std::string(who) + ": njobs_max must be positive");
    if (!W->p && !W->ep) return fail(std::string(who) + ": no weights");
    RowsArgs a{(const uint8_t*) W->p, w_stride, (const uint8_t* const*) W->ep, W->row_bytes, W->n_out, W->n_in,
               jobs, njobs, njobs_max, (const uint8_t*) y, out, out_stride};
    hipStream_t s = (hipStream_t) st;
    // two blocks of 8 waves per CU by default: every block copies the 32 KiB codebook into LDS once
    static const int blocks = env_int("FNX_ROWS_BLOCKS", 0, 0, 65536), threads = env_int("FNX_ROWS_THREADS", 512, 64, 512) / 64 * 64;
    // no more waves than groups of four units: a wave with an empty range only fills the LDS
    const long units = (long) njobs_max * ((W->n_out * (long) (W->n_in / 32) + 63) / 64);
    if (units >= (1L << 31)) return fail(std::string(who) + ": more than 2^31 units of 64 sub-blocks in one launch");
    const long want = (units / 4 + threads / 64 - 1) / (threads / 64);
    const int grid = (int) std::max(1L, std::min((long) (blocks ? blocks : 2 * cu_count()), want));
    const int sbr = W->n_in / 32;
    const bool whole_units = sbr <= 64 && 64 % sbr == 0 && W->n_out % (64 / sbr) == 0;
    const bool packed = W->type == FNX_T_IQ3S_UNIT64;
    if (packed && !whole_units) return fail(std::string(who) + ": the unit64 layout needs rows of 256, 512, 1024 or 2048 columns in whole units");
    if (packed && (w_stride % UNIT_BYTES)) return fail(std::string(who) + ": the unit64 layout needs expert strides in whole units");
#define FNX_ROWS(SBR_, WIDE_, PACKED_) k_iq3s_jobs<SBR_, WIDE_, PACKED_><<<grid, threads, 0, s>>>(a)
#define FNX_ROWS_SBR(WIDE_, PACKED_)                                                                     \
    do {                                                                                                 \
        if (sbr == 64) FNX_ROWS(64, WIDE_, PACKED_);                                                     \
        else if (sbr == 32) FNX_ROWS(32, WIDE_, PACKED_);                                                \
        else if (sbr == 16) FNX_ROWS(16, WIDE_, PACKED_);                                                \
        else FNX_ROWS(8, WIDE_, PACKED_);                                                                \
    } while (0)
    // rows of 2048 columns in whole groups of 16: jobs of two rows and more go to the matrix cores, decoded once (k_iq3s_mma.h)
    static const int jobs_mma = env_int("FNX_JOBS_MMA", 1, 0, 1);
    if (packed && jobs_mma && sbr == 64 && W->n_out % JM_ROWS == 0) {
        const long items = (long) njobs_max * (W->n_out / JM_ROWS);
        k_iq3s_jobs_mma<<<(int) std::max(1L, std::min((long) (blocks ? blocks : cu_count()), items)), JM_THREADS, 0, s>>>(a);
    } else if (!whole_units) k_iq3s_jobs_any<<<dim3((W->n_out + 3) / 4, njobs_max), 256, 0, s>>>(a);
    else if (packed && wide) FNX_ROWS_SBR(true, true);
    else if (packed) FNX_ROWS_SBR(false, true);
    else if (wide) FNX_ROWS_SBR(true, false);
    else FNX_ROWS_SBR(false, false);
#undef FNX_ROWS_SBR
#undef FNX_ROWS
    return launch_status(who);
}

// the shapes and layouts the one-launch window takes (k_moe_window.h)
// the shared expert as dense split Q8_0 (engine.cu:1600-1604) instead of sh_gu / sh_down
static bool shared_is_q8(const fnx_moe_layer* L) { return L->sh_gu_q8.q && L->sh_down_q8.q; }
static bool layer_fused_ok(const fnx_moe_layer* L, int T) {
    static const int on = env_int("FNX_LAYER_FUSED", 1, 0, 1);
    const auto packed = [](const fnx_dw& w) { return w.type == FNX_T_IQ3S_UNIT64; };
    const bool shared_ok = shared_is_q8(L) || (packed(L->sh_gu) && packed(L->sh_down) && L->sh_gu.p && L->sh_down.p);
    return on && L->n == FL_N && (L->ff == 256 || L->ff == 512 || L->ff == 1024) && L->nexp <= 1024 && L->topk <= FL_MAXK &&
           T * L->topk <= FL_MAXP && packed(L->gu) && packed(L->down) && shared_ok && L->gu_stride % UNIT_BYTES == 0 &&
           L->down_stride % UNIT_BYTES == 0 && cu_count() >= WN_WAVES * T;   // sixteen blocks a row at least (moe_window_plan.h)
}
// timing of the window (fnx_layer_profile): events recorded on the launch stream around the window's launch (and around the
// dense launches of a split-Q8_0 shared expert before it); the counterpart of the reference's FNX_PROF stamps in its window
// graph (engine.cu:1382-1530)
static bool g_prof_on = false;
static hipEvent_t g_prof_ev[3] = {};
static void prof_mark(int i, hipStream_t s) {
    if (g_prof_on) (void) hipEventRecord(g_prof_ev[i], s);
}
// the window's MoE half as one launch (k_moe_window.h): router logits, top-k, gate|up -> h as q8_1 rows (in ws->gu), down with
// the combine's chains -> out
// live (may be null): a device word, the rows of the window that count; the others are not routed and their rows of out are left alone
// What a decoder does with the window's rows next, handed to the window's launch (k_moe_window.h: the row's last block):
// x[t] += out[t], then the q8_1 rows of rms_norm(x[t]) * w, the rows after the add copied to xcopy if wanted
// pre_w: the pass before the window too (x[t] += pre_o[t], the norm with pre_w): the window's input is then x itself
struct WinNext {
    float* x = nullptr;
    const float* w = nullptr;
    void* xq = nullptr;
    float* xcopy = nullptr;
    float eps = 0.f;
    const float* pre_o = nullptr;
    const float* pre_w = nullptr;
};
static int layer_fused(const fnx_moe_layer* L, const float* x, int T, float* out, const fnx_moe_ws* ws, void* st, const int* live = nullptr,
                       const WinNext* next = nullptr) {
    hipStream_t s = (hipStream_t) st;
    const int n = L->n, ff = L->ff;
    g_window_order.enter(s);
    prof_mark(0, s);
    // a split-Q8_0 shared expert runs as the reference runs it, three dense launches on the q8_1 rows of x
    // (q8s_gemv -> swiglu_stacked_q8_1 -> q8s_gemv); its f32 rows, q8_1 rows of h and down rows take the workspace's
    // part buffer, which the window does not use otherwise; the window's down phase adds its gated rows
    const bool q8sh = shared_is_q8(L);
    float* sh_part = nullptr;
    if (q8sh) {
        float* sgu = ws->part;                                                              // [T][2 ff]
        uint8_t* shq = reinterpret_cast<uint8_t*>(sgu + (size_t) T * 2 * ff);                // [T][ff / 32] q8_1 blocks
        sh_part = sgu + (size_t) T * 2 * ff + ((size_t) T * (ff / 32) * FNX_Q8_1_BLOCK + 255) / 256 * 64;   // [T][n], 256-byte aligned after shq
        if (fnx_quantize_q8_1(x, ws->xq, n, T, st)) return 1;
        if (fnx_q8s_gemv(&L->sh_gu_q8, ws->xq, sgu, 2 * ff, T, st)) return 1;
        if (fnx_swiglu_stacked_q8_1(sgu, shq, ff, T, st)) return 1;
        if (fnx_q8s_gemv(&L->sh_down_q8, shq, sh_part, n, T, st)) return 1;
    }
    prof_mark(1, s);
    // a wait for another block gives up after this many ticks of the 100 MHz wall clock (FNX_WINDOW_WAIT_TICKS: for tests of the error path)
    static const long long wait_ticks = env_int("FNX_WINDOW_WAIT_TICKS", 20000000, 0, 2000000000);
    WindowArgs wa{ff, L->nexp, L->topk, T, n, x, L->router, L->router_bf16,
                        (const uint8_t*) L->gu.p, L->gu_stride, (const uint8_t* const*) L->gu.ep, q8sh ? nullptr : (const uint8_t*) L->sh_gu.p,
                        (const uint8_t*) L->down.p, L->down_stride, (const uint8_t* const*) L->down.ep, q8sh ? nullptr : (const uint8_t*) L->sh_down.p,
                        sh_part, ws->logits, ws->topi, ws->topw, (uint8_t*) ws->xq, (uint32_t*) ws->gu, out, ws->sync, live,
                        ws->jobs_gu, ws->jobs_dn, ws->njobs, wait_ticks};
    if (next && next->x) {
        wa.next_x = next->x;
        wa.next_w = next->w;
        wa.next_xq = (uint8_t*) next->xq;
        wa.next_xcopy = next->xcopy;
        wa.next_eps = next->eps;
        wa.pre_o = next->pre_o;
        wa.pre_w = next->pre_w;
    }
    // one block a CU; a row's blocks are a power of two of at least sixteen (moe_window_plan.h)
    const int nb = cu_count();
    const auto launch = [&](auto sbr, auto dec) {
        constexpr int SBR = decltype(sbr)::value;
        constexpr bool DEC = decltype(dec)::value;
        if (wa.router_bf16) k_moe_window<SBR, DEC, true><<<nb, WN_THREADS, 0, s>>>(wa);
        else k_moe_window<SBR, DEC, false><<<nb, WN_THREADS, 0, s>>>(wa);
    };
    const auto launch_dec = [&](auto sbr) {
        if (wa.next_x) launch(sbr, std::true_type{});
        else launch(sbr, std::false_type{});
    };
    if (ff == 256) launch_dec(std::integral_constant<int, 8>{});
    else if (ff == 512) launch_dec(std::integral_constant<int, 16>{});
    else launch_dec(std::integral_constant<int, 32>{});
    prof_mark(2, s);
    return launch_status("moe_verify_layer");
}

}  // namespace fnx

using namespace fnx;

// ================================================================ C ABI
extern "C" {

const char* fnx_last_error(void) { return t_err.c_str(); }
const char* fnx_version(void) { return "fnx-mi355x gfx950 verify path 0.1"; }

int fnx_iq3s_repack(const void* src, void* dst, size_t n_weights, void* st) {
    if (!src || !dst) return fail("iq3s_repack: null argument");
    if (n_weights == 0 || n_weights % 2048) return fail("iq3s_repack: whole units of 2048 weights");
    const long units = (long) (n_weights / 2048);
    k_iq3s_repack<<<(unsigned) ((units + 3) / 4), 256, 0, (hipStream_t) st>>>((const uint8_t*) src, (uint8_t*) dst, units);
    return launch_status("iq3s_repack");
}
int fnx_iq3s_tile16(const void* src, void* dst, int nrows, int ncols, int nmat, void* st) {
    if (!src || !dst || src == dst) return fail("iq3s_tile16: two distinct buffers");
    if (nrows < 16 || nrows % 16 || ncols < 512 || ncols % 512 || nmat < 1) return fail("iq3s_tile16: matrices of rows in 16s and columns in 512s");
    const long tiles = (long) nmat * (nrows / 16) * (ncols / 512);
    if ((tiles + 3) / 4 > 0x7fffffffL) return fail("iq3s_tile16: too many tiles for one launch");
    k_iq3s_tile16<<<(unsigned) ((tiles + 3) / 4), 256, 0, (hipStream_t) st>>>((const uint8_t*) src, (uint8_t*) dst, nrows, ncols, tiles);
    return launch_status("iq3s_tile16");
}
size_t fnx_iq3s_tile16_bytes(int nrows, int ncols, int nmat) {
    if (nrows < 16 || nrows % 16 || ncols < 512 || ncols % 512 || nmat < 1) return 0;
    return (size_t) nmat * (nrows / 16) * (ncols / 512) * TILE16_BYTES;
}
int fnx_quantize_q8_1(const float* x, void* q, int n, int rows, void* st) {
    if (!x || !q) return fail("quantize_q8_1: null argument");
    if (n <= 0 || n % 32 || rows <= 0) return fail("quantize_q8_1: rows of whole 32-value blocks");
    k_quantize_q8_1<<<dim3((n / 32 + 7) / 8, rows), 256, 0, (hipStream_t) st>>>(x, (uint8_t*) q, n);
    return launch_status("quantize_q8_1");
}

int fnx_mmvq(const fnx_dw* W, size_t w_stride, const fnx_job* jobs, const int* njobs, int njobs_max, const void* y, float* out,
             int out_stride, void* st) {
    if (!y) return fail("mmvq: null activations");
    return rows_launch(W, w_stride, jobs, njobs, njobs_max, y, out, out_stride, st, "mmvq", njobs_max <= 8);
}

static int gemv_any(const void* W, bool bf, const float* x, float* y, int rows, int n, int T, void* st, const char* who) {
    if (!W || !x || !y) return fail(std::string(who) + ": null argument");
    if (rows <= 0 || n <= 0 || n % 256) return fail(std::string(who) + ": n must be a positive multiple of 256");
    if (T < 1 || T > 65535 * FNX_MAXT) return fail(std::string(who) + ": T out of range");
    hipStream_t s = (hipStream_t) st;
    if (!bf && T >= 2 * RM_TILE && rows >= RM_TILE && n % 2048 == 0 && (uint64_t) T * n * 4 < (1ull << 32) && (uint64_t) rows * n * 4 < (1ull << 32) &&
        (((uintptr_t) W | (uintptr_t) x) & 15) == 0) {
        // a chunk's worth of rows against f32 weights: tiles of 32 x 32 sums on the matrix cores. The weight rows past the
        // last full 32 ride with the tiles' blocks, an item a block (a row x four rows of x); if there are more items
        // than blocks in a row of tiles, those rows go to the kernel below.
        const int ntt = (T + RM_TILE - 1) / RM_TILE, net = rows / RM_TILE, left = rows - net * RM_TILE;
        const int tile_blocks = ((ntt + 3) / 4) * ((net + 7) / 8) * 32;
        const bool along = 8 * left <= net;   // a row and four rows of x a block, within the block's own rows of x
        k_gemv_rows_mfma<<<tile_blocks, RM_THREADS, 0, s>>>((const float*) W, x, y, rows, n, T, ntt, net, tile_blocks, along ? 1 : 0);
        if (left == 0 || along) return launch_status(who);
        const dim3 gm((left + GM_WAVES * GR_ROWS - 1) / (GM_WAVES * GR_ROWS), (T + FNX_MAXT - 1) / FNX_MAXT);
        k_gemv_rows_many<false><<<gm, GM_WAVES * 64, 0, s>>>(W, x, y, rows, n, T, net * RM_TILE);
        return launch_status(who);
    }
    if (T > FNX_MAXT) {   // many rows of x: GR_ROWS weight rows a wave
        const dim3 gm((rows + GM_WAVES * GR_ROWS - 1) / (GM_WAVES * GR_ROWS), (T + FNX_MAXT - 1) / FNX_MAXT);
        if (bf) k_gemv_rows_many<true><<<gm, GM_WAVES * 64, 0, s>>>(W, x, y, rows, n, T, 0);
        else k_gemv_rows_many<false><<<gm, GM_WAVES * 64, 0, s>>>(W, x, y, rows, n, T, 0);
        return launch_status(who);
    }
    const dim3 grid((rows + GV_WAVES - 1) / GV_WAVES, (T + FNX_MAXT - 1) / FNX_MAXT);
    if (bf) k_gemv_rows<true><<<grid, GV_WAVES * 64, 0, s>>>(W, x, y, rows, n, T);
    else k_gemv_rows<false><<<grid, GV_WAVES * 64, 0, s>>>(W, x, y, rows, n, T);
    return launch_status(who);
}
int fnx_gemv_f32(const float* W, const float* x, float* y, int rows, int n, int T, void* st) {
    return gemv_any(W, false, x, y, rows, n, T, st, "gemv_f32");
}
int fnx_gemv_bf16(const uint16_t* W, const float* x, float* y, int rows, int n, int T, void* st) {
    return gemv_any(W, true, x, y, rows, n, T, st, "gemv_bf16");
}

static int topk_check(int T, int nexp, int topk, const char* who) {
    if (T < 1 || T > FNX_MAXT) return fail(std::string(who) + ": T out of range");
    if (nexp < 1 || nexp > TK_MAXE) return fail(std::string(who) + ": 1..1024 experts");
    if (topk < 1 || topk > 64 || topk > nexp) return fail(std::string(who) + ": topk out of range");
    if (T * topk > TK_THREADS - 1) return fail(std::string(who) + ": too many pairs");
    return 0;
}
int fnx_route(const float* logits, int logits_stride, int T, int nexp, int topk, int* topi, float* topw, fnx_job* jobs_gu, fnx_job* jobs_dn,
              int* njobs, void* st) {
    if (!logits || !topi || !topw || !jobs_gu || !jobs_dn || !njobs) return fail("route: null argument");
    if (topk_check(T, nexp, topk, "route")) return 1;
    if (logits_stride < nexp) return fail("route: logits_stride smaller than nexp");
    k_topk_jobs<<<1, TK_THREADS, 0, (hipStream_t) st>>>(logits, logits_stride, T, nexp, topk, topi, topw, jobs_gu, jobs_dn, njobs, 1, 0);
    return launch_status("route");
}
int fnx_router_route(const void* W, int w_bf16, const float* x, float* logits, int T, int n, int nexp, int topk, int* topi, float* topw,
                     fnx_job* jobs_gu, fnx_job* jobs_dn, int* njobs, void* st) {
    if (!W || !x || !logits || !topi || !topw || !jobs_gu || !jobs_dn || !njobs) return fail("router_route: null argument");
    if (topk_check(T, nexp, topk, "router_route")) return 1;
    if (gemv_any(W, w_bf16 != 0, x, logits, nexp + 1, n, T, st, "router_route")) return 1;
    k_topk_jobs<<<1, TK_THREADS, 0, (hipStream_t) st>>>(logits, nexp + 1, T, nexp, topk, topi, topw, jobs_gu, jobs_dn, njobs, 0, 0);
    return launch_status("router_route");
}

int fnx_swiglu_q8_1(const float* g, const float* u, void* q, int n, int rows, void* st) {
    if (!g || !u || !q) return fail("swiglu_q8_1: null argument");
    if (n <= 0 || n % 32 || rows <= 0) return fail("swiglu_q8_1: rows of whole 32-value blocks");
    k_swiglu_q8_1<<<dim3((n / 32 + 7) / 8, rows), 256, 0, (hipStream_t) st>>>(g, u, (size_t) n, (uint8_t*) q, n);
    return launch_status("swiglu_q8_1");
}
int fnx_swiglu_stacked_q8_1(const float* gu, void* hq, int ffs, int T, void* st) {
    if (!gu || !hq) return fail("swiglu_stacked_q8_1: null argument");
    if (ffs <= 0 || ffs % 32 || T <= 0) return fail("swiglu_stacked_q8_1: rows of whole 32-value blocks");
    k_swiglu_q8_1<<<dim3((ffs / 32 + 7) / 8, T), 256, 0, (hipStream_t) st>>>(gu, gu + ffs, (size_t) 2 * ffs, (uint8_t*) hq, ffs);
    return launch_status("swiglu_stacked_q8_1");
}

int fnx_moe_gate_up(const fnx_dw* A, size_t sa, const fnx_job* jobs, const int* njobs, int njobs_max, const void* xq, float* gu, int topk,
                    void* st) {
    if (!xq) return fail("moe_gate_up: null activations");
    if (A && (A->n_out & 1)) return fail("moe_gate_up: rows are [gate | up], an even count");
    if (topk < 1 || njobs_max % topk) return fail("moe_gate_up: njobs_max is the window's pairs, a multiple of topk");
    // the window's rows: njobs_max / topk of them (kernels.cu:2449, T = njobs_max / TOPK); xq holds that many
    return rows_launch(A, sa, jobs, njobs, njobs_max, xq, gu, A ? A->n_out : 0, st, "moe_gate_up");
}
int fnx_moe_down(const fnx_dw* A, size_t sa, const fnx_job* jobs, const int* njobs, int njobs_max, const float* gu, float* part, void* st) {
    if (!A || !gu) return fail("moe_down: null argument");
    const int ffs = A->n_in;
    if (ffs <= 0 || ffs % 32 || ffs > HQ_MAX_FF) return fail("moe_down: expert width does not fit the pair buffer");
    if (njobs_max < 1 || njobs_max > HQ_ROWS) return fail("moe_down: more pairs than the pair buffer holds");
    // every pair's h once (moe.cuh:597-608), then the rows against it
    BufferScope pair_buffer(g_pair_order, st);
    k_swiglu_q8_1<<<dim3((ffs / 32 + 7) / 8, njobs_max), 256, 0, (hipStream_t) st>>>(gu, gu + ffs, (size_t) 2 * ffs, nullptr, ffs);
    if (launch_status("moe_down")) return 1;
    return rows_launch(A, sa, jobs, njobs, njobs_max, nullptr, part, A->n_out, st, "moe_down");
}
// the prompt path's jobs over q8_1 activations (kernels.hpp:324-325): tile16 matrices, a job's rows sixteen at a time on the
// int8 matrix cores (k_iq3s_mma16.h)
static int big_launch(const fnx_dw* W, size_t w_stride, const fnx_bigjob* jobs, const int* njobs, int njobs_cap, const void* xq, const float* gu,
                      float* out, const char* who) {
    if (!W || !jobs || !njobs || !out || (!xq && !gu)) return fail(std::string(who) + ": null argument");
    if (W->type != FNX_T_IQ3S_TILE16) return fail(std::string(who) + ": jobs of up to FNX_PF_JOB rows take tile16 matrices (fnx_iq3s_tile16)");
    if (W->n_in <= 0 || W->n_in % 512 || W->n_in > J16_MAXCOLS || W->n_out <= 0 || W->n_out % 16)
        return fail(std::string(who) + ": the tile16 layout takes rows in 16s and 512, 1024, 1536 or 2048 columns here");
    if (W->row_bytes != (size_t) (W->n_in / 256) * FNX_IQ3S_BLOCK) return fail(std::string(who) + ": row_bytes does not match n_in");
    if (njobs_cap < 1 || njobs_cap > J16_MAXJOBS) return fail(std::string(who) + ": 1 .. 4096 jobs a launch");
    if (!W->p && !W->ep) return fail(std::string(who) + ": no weights");
    if (gu && ((uintptr_t) gu & 15)) return fail(std::string(who) + ": 16-byte aligned rows");
    return 0;
}
int fnx_moe_gate_up_big(const fnx_dw* A, size_t sa, const fnx_bigjob* jobs, const int* njobs, int njobs_cap, const void* xq, float* gu, void* st) {
    if (big_launch(A, sa, jobs, njobs, njobs_cap, xq, nullptr, gu, "moe_gate_up_big")) return 1;
    RowsArgs a{(const uint8_t*) A->p, sa, (const uint8_t* const*) A->ep, A->row_bytes, A->n_out, A->n_in, nullptr, njobs, njobs_cap,
               (const uint8_t*) xq, gu, A->n_out};
    a.big = jobs;
    const long items = (long) njobs_cap * (FNX_PF_JOB / FNX_MAXT) * (A->n_out / 16);
    k_iq3s_jobs_mma16<1><<<(int) std::max(1L, std::min((long) cu_count(), items)), J16_THREADS, 0, (hipStream_t) st>>>(a);
    return launch_status("moe_gate_up_big");
}
int fnx_moe_down_big(const fnx_dw* A, size_t sa, const fnx_bigjob* jobs, const int* njobs, int njobs_cap, const float* gu, float* part, void* st) {
    if (big_launch(A, sa, jobs, njobs, njobs_cap, nullptr, gu, part, "moe_down_big")) return 1;
    RowsArgs a{(const uint8_t*) A->p, sa, (const uint8_t* const*) A->ep, A->row_bytes, A->n_out, A->n_in, nullptr, njobs, njobs_cap,
               nullptr, part, A->n_out};
    a.big = jobs;
    a.gu = gu;
    const long items = (long) njobs_cap * (FNX_PF_JOB / FNX_MAXT) * (A->n_out / 16);
    k_iq3s_jobs_mma16<2><<<(int) std::max(1L, std::min((long) cu_count(), items)), J16_THREADS, 0, (hipStream_t) st>>>(a);
    return launch_status("moe_down_big");
}
int fnx_moe_combine(const float* part, const float* topw, const float* sh, const float* sh_logit, int sh_logit_stride, float* out, int T, int n,
                    int topk, void* st) {
    if (!part || !topw || !sh || !sh_logit || !out) return fail("moe_combine: null argument");
    if (T < 1 || n < 1 || topk < 1) return fail("moe_combine: bad shape");
    k_combine<<<dim3((n + 255) / 256, T), 256, 0, (hipStream_t) st>>>(part, topw, sh, sh_logit, sh_logit_stride, out, n, topk);
    return launch_status("moe_combine");
}

static int argmax_launch(const float* logits, int rows, int T, int v0, float* best_v, int* best_i, unsigned long long* keys, unsigned* err, void* st,
                         const int* live) {
    if (!logits || !best_v || !best_i || !keys || !err) return fail("argmax: null argument");
    if (rows < 1 || T < 1 || T > FNX_MAXT) return fail("argmax: bad shape");
    k_argmax<<<dim3((rows + AM_PER_BLOCK - 1) / AM_PER_BLOCK, T), AM_THREADS, 0, (hipStream_t) st>>>(logits, rows, keys, err, v0, best_v, best_i, live);
    return launch_status("argmax");
}
int fnx_argmax(const float* logits, int rows, int T, int v0, float* best_v, int* best_i, unsigned long long* keys, unsigned* err, void* st) {
    return argmax_launch(logits, rows, T, v0, best_v, best_i, keys, err, st, nullptr);
}

int fnx_lookup_drafts(const int* ctx, int n_ctx, int key_n, int lk, int d1, int* out, int* match) {
    if (match) *match = -1;
    if (!ctx || !out || n_ctx < 0 || lk < 0 || key_n < 1 || key_n > 4) {
        fail("lookup_drafts: bad argument");
        return -1;
    }
    if (lk == 0 || n_ctx <= key_n) return 0;
    const int n0 = n_ctx - key_n;
    int nr = 0;
    for (int s = n0; s-- > 0;) {
        if (std::memcmp(ctx + s, ctx + n0, (size_t) key_n * sizeof(int)) != 0) continue;
        // only the latest earlier place is examined (session.cpp:442)
        if (s + key_n < n_ctx && (d1 < 0 || ctx[s + key_n] == d1)) {
            int m = key_n;
            while (m < lk && (m - key_n) < s && ctx[s - 1 - (m - key_n)] == ctx[n0 - 1 - (m - key_n)]) ++m;
            const int k = std::min(lk, std::max(LOOKUP_MIN, m)), end = std::min(n_ctx, s + key_n + k);
            for (int i = s + key_n; i < end && ctx[i] < IMAGE_TOK; ++i) out[nr++] = ctx[i];
            if (match) *match = s;
        }
        break;
    }
    return nr;
}
int fnx_lookup_drafts_dev(const int* ctx, int n_ctx, int key_n, int lk, const int* d1, int* out, int* n_out, int* match, void* st) {
    if (!ctx || !d1 || !out || !n_out) return fail("lookup_drafts_dev: null argument");
    if (n_ctx < 0 || lk < 0 || lk > 64 || key_n < 1 || key_n > 4) return fail("lookup_drafts_dev: bad argument (keys of 1..4 tokens, up to 64 drafts)");
    k_lookup<<<1, LK_THREADS, 0, (hipStream_t) st>>>(ctx, n_ctx, key_n, lk, d1, out, n_out, match, nullptr, nullptr);
    return launch_status("lookup_drafts_dev");
}

int fnx_accept_greedy(const int* rows, const int* o, int R) {
    if (!rows || !o || R < 1) {
        fail("accept_greedy: bad argument");
        return -1;
    }
    int n = 1;
    while (n < R && rows[n] == o[n - 1]) ++n;
    return n;
}
int fnx_accept_greedy_dev(const int* rows, const int* o, int R, int* n_accept, void* st) {
    if (!rows || !o || !n_accept) return fail("accept_greedy_dev: null argument");
    if (R < 1 || R > 64) return fail("accept_greedy_dev: 1..64 rows");
    k_accept<<<1, 64, 0, (hipStream_t) st>>>(rows, o, R, n_accept);
    return launch_status("accept_greedy_dev");
}

int fnx_layer_profile(int on) {
    if (on && !g_prof_ev[0])
        for (hipEvent_t& e : g_prof_ev)
            if (hipEventCreate(&e) != hipSuccess) return fail("layer_profile: hipEventCreate failed");
    g_prof_on = on != 0;
    return 0;
}
int fnx_layer_profile_read(float* ms2) {
    if (!ms2) return fail("layer_profile_read: null argument");
    if (!g_prof_ev[0]) return fail("layer_profile_read: profiling was never switched on");
    if (hipEventSynchronize(g_prof_ev[2]) != hipSuccess) return fail("layer_profile_read: no window was recorded");
    for (int i = 0; i < 2; ++i)
        if (hipEventElapsedTime(&ms2[i], g_prof_ev[i], g_prof_ev[i + 1]) != hipSuccess) return fail("layer_profile_read: no window was recorded");
    return 0;
}

// the layer's matrices against n / ff; the shared expert in whichever form it comes
static bool moe_shapes_ok(const fnx_moe_layer* L) {
    const int n = L->n, ff = L->ff;
    if (L->gu.n_in != n || L->gu.n_out != 2 * ff || L->down.n_in != ff || L->down.n_out != n) return false;
    if (shared_is_q8(L))
        return L->sh_gu_q8.d && L->sh_down_q8.d && L->sh_gu_q8.n_in == n && L->sh_gu_q8.n_out == 2 * ff && L->sh_down_q8.n_in == ff &&
               L->sh_down_q8.n_out == n;
    return L->sh_gu.n_in == n && L->sh_gu.n_out == 2 * ff && L->sh_down.n_in == ff && L->sh_down.n_out == n;
}
// next (may be null): see WinNext; *next_done says whether the window's launch took it over (the one-launch window does)
static int moe_layer_checked(const fnx_moe_layer* L, const float* x, int T, float* out, const fnx_moe_ws* ws, void* st, const int* live = nullptr,
                             const WinNext* next = nullptr, bool* next_done = nullptr) {
    if (next_done) *next_done = false;
    if (!L || !x || !ws) return fail("moe_verify_layer: null argument");
    if (!ws->xq || !ws->logits || !ws->topi || !ws->topw || !ws->jobs_gu || !ws->jobs_dn || !ws->njobs || !ws->gu || !ws->part || !ws->sync)
        return fail("moe_verify_layer: incomplete workspace");
    if ((uintptr_t) ws->sync & 7) return fail("moe_verify_layer: the sync words are 8-byte aligned");
    if (topk_check(T, L->nexp, L->topk, "moe_verify_layer")) return 1;
    const int P = T * L->topk, n = L->n, ff = L->ff;
    if (P + T > HQ_ROWS) return fail("moe_verify_layer: more pairs than the pair buffer holds");
    if (!moe_shapes_ok(L)) return fail("moe_verify_layer: weight shapes do not match n / ff");
    if (!out) return fail("moe_verify_layer: null argument");
    if (live && !layer_fused_ok(L, T)) return fail("moe_verify_layer: a device-side row count needs the one-launch window");
    if (layer_fused_ok(L, T)) {
        if (next_done) *next_done = next && next->x;
        return layer_fused(L, x, T, out, ws, st, live, next);
    }
    // operator by operator the pairs' q8_1 rows of h go through the library's pair buffer, rows of ff / 32 blocks
    if (ff <= 0 || ff % 32 || ff > HQ_MAX_FF) return fail("moe_verify_layer: expert width does not fit the pair buffer");
    hipStream_t s = (hipStream_t) st;
    BufferScope pair_buffer(g_pair_order, st);   // operator by operator the pairs' q8_1 rows go through the library's buffer
    if (fnx_quantize_q8_1(x, ws->xq, n, T, st)) return 1;
    if (gemv_any(L->router, L->router_bf16 != 0, x, ws->logits, L->nexp + 1, n, T, st, "moe_verify_layer router")) return 1;
    k_topk_jobs<<<1, TK_THREADS, 0, s>>>(ws->logits, L->nexp + 1, T, L->nexp, L->topk, ws->topi, ws->topw, ws->jobs_gu, ws->jobs_dn, ws->njobs,
                                         0, 1);
    if (launch_status("moe_verify_layer topk")) return 1;
    if (rows_launch(&L->gu, L->gu_stride, ws->jobs_gu, ws->njobs, P, ws->xq, ws->gu, 2 * ff, st, "moe_verify_layer gate|up")) return 1;
    const bool q8sh = shared_is_q8(L);   // engine.cu:1600-1604: the rows P + t of gu, of the q8_1 rows of h and of part
    if (q8sh) {
        if (fnx_q8s_gemv(&L->sh_gu_q8, ws->xq, ws->gu + (size_t) P * 2 * ff, 2 * ff, T, st)) return 1;
    } else if (rows_launch(&L->sh_gu, 0, ws->jobs_gu + P, nullptr, 1, ws->xq, ws->gu, 2 * ff, st, "moe_verify_layer shared gate|up", true)) return 1;
    k_swiglu_q8_1<<<dim3((ff / 32 + 7) / 8, P + T), 256, 0, s>>>(ws->gu, ws->gu + ff, (size_t) 2 * ff, nullptr, ff);
    if (launch_status("moe_verify_layer swiglu")) return 1;
    if (rows_launch(&L->down, L->down_stride, ws->jobs_dn, ws->njobs, P, nullptr, ws->part, n, st, "moe_verify_layer down")) return 1;
    if (q8sh) {
        const uint8_t* hq_dev = nullptr;   // the device's pair buffer of q8_1 rows (k_swiglu_q8_1 wrote it): the shared rows start at pair P
        if (hipGetSymbolAddress((void**) &hq_dev, HIP_SYMBOL(g_moe_hq)) != hipSuccess) return fail("moe_verify_layer: no pair buffer");
        if (fnx_q8s_gemv(&L->sh_down_q8, hq_dev + (size_t) P * (ff / 32) * FNX_Q8_1_BLOCK, ws->part + (size_t) P * n, n, T, st)) return 1;
    } else if (rows_launch(&L->sh_down, 0, ws->jobs_dn + P, nullptr, 1, nullptr, ws->part, n, st, "moe_verify_layer shared down", true)) return 1;
    return fnx_moe_combine(ws->part, ws->topw, ws->part + (size_t) P * n, ws->logits + L->nexp, L->nexp + 1, out, T, n, L->topk, st);
}
int fnx_moe_verify_layer(const fnx_moe_layer* L, const float* x, int T, float* out, const fnx_moe_ws* ws, void* st) {
    if (!out) return fail("moe_verify_layer: null argument");
    return moe_layer_checked(L, x, T, out, ws, st);
}

// ---------------------------------------------------------------- the window on a workspace of the library's own
// fnx_moe_verify_layer with its scratch (the q8_1 rows of x, the logits, the picks and weights, the job lists, the q8_1
// rows of h) in a file-scope device array instead of a caller's fnx_moe_ws, for callers that cannot allocate. The array's
// name is only a host-side handle: its device address is asked for once per device (hipGetSymbolAddress) and kept.
constexpr size_t NA_XQ = (size_t) FNX_MAXT * (FL_N / 32) * FNX_Q8_1_BLOCK;            // 36,864
constexpr size_t NA_LOGITS = (size_t) FNX_MAXT * (1024 + 1) * sizeof(float);           // 65,600
constexpr size_t NA_TOP = (size_t) FL_MAXP * sizeof(int);                              // 640 (topi), 640 (topw)
constexpr size_t NA_JOBS = (size_t) (FL_MAXP + 1) * sizeof(fnx_job);                   // 21,896 each
constexpr size_t NA_HQ = (size_t) (FL_MAXP + FNX_MAXT) * (1024 / 32) * HQ_WORDS * 4;   // 270,336
constexpr size_t na_up(size_t v) { return (v + 255) / 256 * 256; }
constexpr size_t NA_OFF_LOGITS = na_up(NA_XQ), NA_OFF_TOPI = NA_OFF_LOGITS + na_up(NA_LOGITS), NA_OFF_TOPW = NA_OFF_TOPI + na_up(NA_TOP),
                 NA_OFF_JGU = NA_OFF_TOPW + na_up(NA_TOP), NA_OFF_JDN = NA_OFF_JGU + na_up(NA_JOBS), NA_OFF_NJOBS = NA_OFF_JDN + na_up(NA_JOBS),
                 NA_OFF_SYNC = NA_OFF_NJOBS + 256, NA_OFF_HQ = NA_OFF_SYNC + na_up(FNX_MOE_SYNC_WORDS * 4), NA_BYTES = NA_OFF_HQ + na_up(NA_HQ);
static_assert(NA_BYTES <= FNX_MOE_STATIC_WS_BYTES, "the header states the array's size");
static __device__ __align__(256) unsigned char scratch[FNX_MOE_STATIC_WS_BYTES];
static unsigned char* g_scratch_ptr[64] = {};   // per device: the array's address there
static std::mutex g_scratch_mutex;
// the array's address on the current device: asked once per device, with that device current; threads that arrive together
// take turns (a failed query is asked again)
static unsigned char* static_ws(const char* who) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        fail(std::string(who) + ": no current device");
        return nullptr;
    }
    std::lock_guard<std::mutex> g(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        unsigned char* p = nullptr;
        const hipError_t e = hipGetSymbolAddress((void**) &p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            fail(std::string(who) + ": hipGetSymbolAddress: " + hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}
int fnx_moe_static_status(unsigned* err, void* st) {
    if (!err) return fail("moe_static_status: null argument");
    unsigned char* w = static_ws("moe_static_status");
    if (!w) return 1;
    if (hipStreamSynchronize((hipStream_t) st) != hipSuccess) return fail("moe_static_status: the stream failed");
    if (hipMemcpy(err, w + NA_OFF_SYNC, sizeof(unsigned), hipMemcpyDeviceToHost) != hipSuccess) return fail("moe_static_status: copy failed");
    if (*err && hipMemset(w + NA_OFF_SYNC, 0, FNX_MOE_SYNC_WORDS * sizeof(unsigned)) != hipSuccess) return fail("moe_static_status: reset failed");
    return 0;
}
int fnx_moe_verify_layer_static(const fnx_moe_layer* L, const float* x, int T, float* out, void* st) {
    if (!L || !x || !out) return fail("moe_verify_layer_static: null argument");
    if (T < 1 || T > FNX_MAXT) return fail("moe_verify_layer_static: T out of range");
    if (!layer_fused_ok(L, T))
        return fail("moe_verify_layer_static: only the one-launch window runs on the library's own workspace (unit64 experts, hidden 2048, "
                    "ff 256 / 512 / 1024, up to 1024 experts, up to 16 picks a row, up to 160 pairs a window)");
    unsigned char* w = static_ws("moe_verify_layer_static");
    if (!w) return 1;
    // the sync words start at zero with the device image and every window leaves them zero; nothing else has to: every
    // launch writes what it reads, and the job count is stored, not added to
    const fnx_moe_ws ws{w, (float*) (w + NA_OFF_LOGITS), (int*) (w + NA_OFF_TOPI), (float*) (w + NA_OFF_TOPW), (fnx_job*) (w + NA_OFF_JGU),
                        (fnx_job*) (w + NA_OFF_JDN), (int*) (w + NA_OFF_NJOBS), (float*) (w + NA_OFF_HQ), nullptr, (unsigned*) (w + NA_OFF_SYNC)};
    const int P = T * L->topk;
    if (shared_is_q8(L)) return fail("moe_verify_layer_static: a split-Q8_0 shared expert needs a caller's workspace (fnx_moe_verify_layer)");
    if (!moe_shapes_ok(L)) return fail("moe_verify_layer_static: weight shapes do not match n / ff");
    if (topk_check(T, L->nexp, L->topk, "moe_verify_layer_static")) return 1;
    (void) P;
    return layer_fused(L, x, T, out, &ws, st);
}

#ifdef FNX_WIN_TS
int fnx_debug_win_ts(unsigned long long* host, size_t words) {   // timing build only
    return hipMemcpyFromSymbol(host, HIP_SYMBOL(g_win_ts), words * 8) == hipSuccess ? 0 : fail("debug_win_ts");
}
#endif
// ---------------------------------------------------------------- streaming calibration (k_stream.h)
int fnx_stream_read(const void* p, size_t bytes, int variant, int blocks, int threads, void* sink, void* st) {
    if (!p || !sink) return fail("stream_read: null argument");
    if (threads < 64 || threads > 1024 || threads % 64) return fail("stream_read: 64..1024 threads in whole waves");
    if (blocks < 1 || blocks > 65535) return fail("stream_read: 1..65535 blocks");
    if (((uintptr_t) p & 15u) || bytes < 1024) return fail("stream_read: a 16-byte aligned buffer of at least 1 KiB");
    hipStream_t s = (hipStream_t) st;
    const uint8_t* b = (const uint8_t*) p;
    uint32_t* k = (uint32_t*) sink;
    const size_t c16 = bytes / 1024, c8 = bytes / 512;
    switch (variant) {
        case 0: k_stream_read<16, 4, false, true><<<blocks, threads, 0, s>>>(b, c16, k); break;
        case 1: k_stream_read<16, 8, false, true><<<blocks, threads, 0, s>>>(b, c16, k); break;
        case 2: k_stream_read<16, 4, false, false><<<blocks, threads, 0, s>>>(b, c16, k); break;
        case 3: k_stream_read<16, 8, false, false><<<blocks, threads, 0, s>>>(b, c16, k); break;
        case 4: k_stream_read<8, 8, false, true><<<blocks, threads, 0, s>>>(b, c8, k); break;
        case 5: k_stream_read<16, 8, true, true><<<blocks, threads, 0, s>>>(b, c16, k); break;
        case 6: k_stream_read_units<0, false><<<blocks, threads, 0, s>>>(b, bytes / UNIT_BYTES, k); break;
        case 7: k_stream_read<16, 16, false, true><<<blocks, threads, 0, s>>>(b, c16, k); break;
        case 8: k_stream_read<16, 2, false, true><<<blocks, threads, 0, s>>>(b, c16, k); break;
        case 9: k_stream_read_units<1, false><<<blocks, threads, 0, s>>>(b, bytes / UNIT_BYTES, k); break;
        case 10: k_stream_read_units<2, false><<<blocks, threads, 0, s>>>(b, bytes / UNIT_BYTES, k); break;
        case 11: k_stream_read_units<0, true><<<blocks, threads, 0, s>>>(b, bytes / UNIT_BYTES, k); break;
        case 12: k_stream_read_units<1, true><<<blocks, threads, 0, s>>>(b, bytes / UNIT_BYTES, k); break;
        case 13: k_stream_read_units<2, true><<<blocks, threads, 0, s>>>(b, bytes / UNIT_BYTES, k); break;
        case 14: k_stream_read_quads<false><<<blocks, threads, 0, s>>>(b, bytes / QUAD_BYTES, k); break;
        case 15: k_stream_read_quads<true><<<blocks, threads, 0, s>>>(b, bytes / QUAD_BYTES, k); break;
        default:
            // 1000 s + K: segments of 256 s units (s = 4: a gate|up matrix, 2: a down matrix), K trips a wave and segment
            if (variant >= 1000 && variant < 9000 && variant % 1000 >= 1 && variant % 1000 <= 64 && (256 * (variant / 1000) / 4) % (variant % 1000) == 0) {
                k_stream_read_segments<<<blocks, threads, 0, s>>>(b, bytes / UNIT_BYTES, 256u * (variant / 1000), (uint32_t) (variant % 1000), k);
                break;
            }
            return fail("stream_read: variants 0..15, or 1000 s + K");
    }
    return launch_status("stream_read");
}

// ---------------------------------------------------------------- the prompt path
// sh_gu, sh_dn, nsh (null or all set): the shared expert's jobs over every row and their count, from the same launch;
// cvt_x, cvt_n, cvt_y (cvt_n > 0): floats to turn into f16 on the way (the first launch carries them)
static int pf_route(const float* logits, int logits_stride, int C, int nexp, int topk, int* topi, float* topw, int* cnt, int* jbase,
                    fnx_bigjob* jobs_gu, fnx_bigjob* jobs_dn, int njobs_cap, int* njobs, fnx_bigjob* sh_gu, fnx_bigjob* sh_dn, int* nsh, void* st,
                    const float* cvt_x = nullptr, size_t cvt_n = 0, uint16_t* cvt_y = nullptr) {
    if (!logits || !topi || !topw || !cnt || !jbase || !jobs_gu || !jobs_dn || !njobs) return fail("pf_route: null argument");
    static_assert(TK_MAXE <= PF_MAXE, "k_pf_fill counts every expert's pairs in LDS");
    if (C < 1 || nexp < 1 || nexp > TK_MAXE || topk < 1 || topk > 64 || topk > nexp) return fail("pf_route: bad shape");
    if (logits_stride < nexp) return fail("pf_route: logits_stride smaller than nexp");
    if ((long) C * topk > (1l << 30)) return fail("pf_route: too many pairs");
    if (njobs_cap < 1) return fail("pf_route: no room for jobs");
    hipStream_t s = (hipStream_t) st;
    const int P = C * topk;
    const int cvt_blocks = cvt_n ? (int) std::min<size_t>((cvt_n + 4095) / 4096, 2048) : 0;   // 16 values a thread or more
    k_pf_topk<<<(C + PF_TOPK_WAVES - 1) / PF_TOPK_WAVES + cvt_blocks, PF_TOPK_WAVES * 64, 0, s>>>(logits, logits_stride, C, nexp, topk, topi, topw,
                                                                                                  cvt_x, cvt_n, cvt_y);
    const int shb = sh_gu ? (C + PF_FILL_THREADS - 1) / PF_FILL_THREADS : 0;
    k_pf_fill<<<nexp + shb, PF_FILL_THREADS, 0, s>>>(topi, P, topk, nexp, cnt, jbase, njobs, jobs_gu, jobs_dn, njobs_cap, C, sh_gu, sh_dn, nsh);
    return launch_status("pf_route");
}
int fnx_pf_route(const float* logits, int logits_stride, int C, int nexp, int topk, int* topi, float* topw, int* cnt, int* jbase,
                 fnx_bigjob* jobs_gu, fnx_bigjob* jobs_dn, int njobs_cap, int* njobs, void* st) {
    return pf_route(logits, logits_stride, C, nexp, topk, topi, topw, cnt, jbase, jobs_gu, jobs_dn, njobs_cap, njobs, nullptr, nullptr, nullptr, st);
}
int fnx_f32_f16(const float* x, size_t n, uint16_t* out, void* st) {
    if (!x || !out) return fail("f32_f16: null argument");
    if (n == 0) return 0;
    k_f32_f16<<<(unsigned) std::min<size_t>((n + 255) / 256, 8192), 256, 0, (hipStream_t) st>>>(x, n, out);
    return launch_status("f32_f16");
}
int fnx_swiglu_h16(const float* gu, int ffs, int P, uint16_t* h16, void* st) {
    if (!gu || !h16) return fail("swiglu_h16: null argument");
    if (ffs < 1 || P < 1) return fail("swiglu_h16: bad shape");
    const size_t total = (size_t) P * ffs;
    k_swiglu_h16<<<(unsigned) std::min<size_t>((total + 255) / 256, 8192), 256, 0, (hipStream_t) st>>>(gu, ffs, total, h16);
    return launch_status("swiglu_h16");
}
// A2 (may be null): one more matrix of the same shape and layout with a job list of its own (jobs2, njobs2, cap2), run in
// the same launch by the wave forms (tile16), else right after
static int mma_launch(const fnx_dw* A, size_t sa, const fnx_bigjob* jobs, const int* njobs, int njobs_cap, const uint16_t* x, float* out,
                      void* st, const char* who, const fnx_dw* A2 = nullptr, const fnx_bigjob* jobs2 = nullptr, const int* njobs2 = nullptr,
                      int cap2 = 0, uint16_t* h16 = nullptr, bool* h16_done = nullptr) {
    if (!A || !jobs || !njobs || !x || (!out && !h16)) return fail(std::string(who) + ": null argument");
    if (!A->p && !A->ep) return fail(std::string(who) + ": no weights");
    if (A->type != FNX_T_IQ3_S && A->type != FNX_T_IQ3S_UNIT64 && A->type != FNX_T_IQ3S_TILE16) return fail(std::string(who) + ": IQ3_S weights only");
    if (A->type == FNX_T_IQ3S_TILE16 && (A->n_in % 512 || A->n_out % 16)) return fail(std::string(who) + ": the tile16 layout takes rows in 16s and columns in 512s");
    if (A->n_in < 256 || A->n_in % 256 || A->n_out < 32 || A->n_out % 32) return fail(std::string(who) + ": columns in 256s, rows in 32s");
    if (A->type == FNX_T_IQ3S_UNIT64 && ((size_t) A->n_out * A->n_in) % 2048) return fail(std::string(who) + ": whole units of 2048 weights");
    if (njobs_cap < 1) return fail(std::string(who) + ": no jobs");
    MmaArgs a{(const uint8_t*) A->p, sa, A->ep, A->n_out, A->n_in, jobs, njobs, njobs_cap, x, A->n_in, out};
    const bool tile16 = A->type == FNX_T_IQ3S_TILE16;
    // the wave forms (tile16) take the second list - the shared expert's matrix - in the same launch
    const bool merged = A2 && tile16 && A2->p && A2->type == A->type && A2->n_in == A->n_in && A2->n_out == A->n_out;
    if (A2 && !merged) {   // two launches
        if (h16_done) *h16_done = false;
        if (!out) return fail(std::string(who) + ": h alone is left by the wave form only (both matrices tile16)");
        if (mma_launch(A, sa, jobs, njobs, njobs_cap, x, out, st, who)) return 1;
        return mma_launch(A2, 0, jobs2, njobs2, cap2, x, out, st, who);
    }
    if (merged) {
        if (!jobs2 || !njobs2 || cap2 < 1) return fail(std::string(who) + ": null argument");
        a.w2 = (const uint8_t*) A2->p;
        a.jobs2 = jobs2;
        a.njobs2 = njobs2;
        a.cap2 = cap2;
    }
    const long caps = (long) njobs_cap + (merged ? cap2 : 0);
    if (h16_done) *h16_done = false;
    if (tile16 && h16 && A->n_out % 32 == 0) {
        // wave form for stacked gate|up matrices, which leaves h = silu(gate) * up itself: a wave a (gate tile, up tile) pair over
        // the row's super-steps, one block a CU
        a.h16 = h16;
        a.ffh = A->n_out / 2;
        if (h16_done) *h16_done = true;
        const long upj = (a.ffh / 16 + 7) / 8;   // the finer of its two kinds of units
        const int grid = (int) std::max(1l, std::min<long>(std::min(cu_count(), 64 * W16_PLAN), caps * upj));
        k_moe_mma_wave16_gu<<<grid, W16_THREADS, 0, (hipStream_t) st>>>(a);
        return launch_status(who);
    }
    if (!out) return fail(std::string(who) + ": h alone is left by the wave form only (tile16 gate|up, 2 ff rows in 32s)");
    if (tile16 && A->n_in == W16_COLS) {
        // wave form: rows of 512 columns (the down projection), a job's whole activation tile in LDS, one block a CU
        const int grid = (int) std::max(1l, std::min<long>((long) cu_count(), caps * (A->n_out / 16)));
        k_moe_mma_wave16<<<grid, W16_THREADS, 0, (hipStream_t) st>>>(a);
        return launch_status(who);
    }
    if (tile16) return fail(std::string(who) + ": tile16 matrices are the prompt path's two: stacked gate|up leaving h, and rows of 512 columns");
    // raw blocks and unit64: a wave a task of 32 rows x 32 tokens
    static const int per_cu = env_int("FNX_MMA_BLOCKS_PER_CU", 2, 1, 8);
    const long tasks = (long) njobs_cap * (A->n_out / 32) * (MM_TT / MM_TP);
    const int grid = (int) std::max(1l, std::min<long>((long) per_cu * cu_count(), (tasks + MM_WAVES - 1) / MM_WAVES));
    if (A->type == FNX_T_IQ3S_UNIT64) k_moe_mma<true, 2><<<grid, MM_THREADS, 0, (hipStream_t) st>>>(a);
    else k_moe_mma<false, 2><<<grid, MM_THREADS, 0, (hipStream_t) st>>>(a);
    return launch_status(who);
}
int fnx_moe_gate_up_mma(const fnx_dw* A, size_t sa, const fnx_bigjob* jobs, const int* njobs, int njobs_cap, const uint16_t* xh, float* gu,
                        void* st) {
    return mma_launch(A, sa, jobs, njobs, njobs_cap, xh, gu, st, "moe_gate_up_mma");
}
int fnx_moe_gate_up_h16_mma(const fnx_dw* A, size_t sa, const fnx_bigjob* jobs, const int* njobs, int njobs_cap, const uint16_t* xh,
                            uint16_t* h16, void* st) {
    if (!h16) return fail("moe_gate_up_h16_mma: null argument");
    return mma_launch(A, sa, jobs, njobs, njobs_cap, xh, nullptr, st, "moe_gate_up_h16_mma", nullptr, nullptr, nullptr, 0, h16);
}
int fnx_moe_down_mma(const fnx_dw* A, size_t sa, const fnx_bigjob* jobs, const int* njobs, int njobs_cap, const uint16_t* h16, float* part,
                     void* st) {
    return mma_launch(A, sa, jobs, njobs, njobs_cap, h16, part, st, "moe_down_mma");
}
int fnx_moe_prefill_layer(const fnx_moe_layer* L, const float* x, int C, float* out, const fnx_pf_ws* ws, void* st) {
    if (!L || !x || !out || !ws) return fail("moe_prefill_layer: null argument");
    if (!ws->logits || !ws->topi || !ws->topw || !ws->cnt || !ws->jbase || !ws->jobs_gu || !ws->jobs_dn || !ws->njobs || !ws->xh || !ws->gu ||
        !ws->h16 || !ws->part)
        return fail("moe_prefill_layer: incomplete workspace");
    const int n = L->n, ff = L->ff, nexp = L->nexp, topk = L->topk;
    if (C < 1 || C > 65535) return fail("moe_prefill_layer: 1..65535 rows a chunk (the combine takes a grid row per chunk row)");
    if (L->gu.n_in != n || L->gu.n_out != 2 * ff || L->down.n_in != ff || L->down.n_out != n || L->sh_gu.n_in != n ||
        L->sh_gu.n_out != 2 * ff || L->sh_down.n_in != ff || L->sh_down.n_out != n)
        return fail("moe_prefill_layer: weight shapes do not match n / ff");
    const int P = C * topk, J = P / FNX_PF_JOB + nexp, S = (C + FNX_PF_JOB - 1) / FNX_PF_JOB;
    // the router logits; the routed experts' jobs, the shared expert's and x as f16 from the same launches
    if (gemv_any(L->router, L->router_bf16 != 0, x, ws->logits, nexp + 1, n, C, st, "moe_prefill_layer router")) return 1;
    if (pf_route(ws->logits, nexp + 1, C, nexp, topk, ws->topi, ws->topw, ws->cnt, ws->jbase, ws->jobs_gu, ws->jobs_dn, J, ws->njobs, ws->jobs_gu + J,
                 ws->jobs_dn + J, ws->njobs + 1, st, x, (size_t) C * n, ws->xh))
        return 1;
    // the routed experts' jobs and the shared expert's in one launch each way
    bool h16_done = false;
    if (mma_launch(&L->gu, L->gu_stride, ws->jobs_gu, ws->njobs, J, ws->xh, ws->gu, st, "moe_prefill_layer gate|up", &L->sh_gu, ws->jobs_gu + J,
                   ws->njobs + 1, S, ws->h16, &h16_done))
        return 1;
    if (!h16_done && fnx_swiglu_h16(ws->gu, ff, P + C, ws->h16, st)) return 1;
    if (mma_launch(&L->down, L->down_stride, ws->jobs_dn, ws->njobs, J, ws->h16, ws->part, st, "moe_prefill_layer down", &L->sh_down, ws->jobs_dn + J,
                   ws->njobs + 1, S))
        return 1;
    return fnx_moe_combine(ws->part, ws->topw, ws->part + (size_t) P * n, ws->logits + nexp, nexp + 1, out, C, n, topk, st);
}

// ---------------------------------------------------------------- around the MoE half: norms, dense projections, attention
int fnx_rms_norm_rows(const float* x, const float* w, float* y, int rows, int n, float eps, void* st) {
    if (!x || !w || !y) return fail("rms_norm_rows: null argument");
    if (rows < 1 || n < 1) return fail("rms_norm_rows: bad shape");
    k_rms_norm_rows<<<rows, 256, 0, (hipStream_t) st>>>(x, w, y, n, eps);
    return launch_status("rms_norm_rows");
}
int fnx_add_norm_q8(float* x, const float* add, const float* w, float* xn, void* xq, int rows, int n, float eps, void* st) {
    if (!x || !w) return fail("add_norm_q8: null argument");
    if (rows < 1 || n < 32 || n % 32 || n > 256 * NQ_MAXJ) return fail("add_norm_q8: rows of 32 .. 4096 values in whole 32-value blocks");
    k_add_norm_q8<false><<<rows, 256, 0, (hipStream_t) st>>>(x, add, CombineArgs{}, w, xn, (uint8_t*) xq, n, eps);
    return launch_status("add_norm_q8");
}
int fnx_combine_add_norm_q8(const float* part, const float* topw, const float* sh, const float* sh_logit, int sh_logit_stride, int topk, float* x,
                            const float* w, float* xn, void* xq, int rows, int n, float eps, void* st) {
    if (!part || !topw || !sh || !sh_logit || !x || !w) return fail("combine_add_norm_q8: null argument");
    if (rows < 1 || n < 32 || n % 32 || n > 256 * NQ_MAXJ || topk < 1) return fail("combine_add_norm_q8: rows of 32 .. 4096 values in whole 32-value blocks");
    k_add_norm_q8<true><<<rows, 1024, 0, (hipStream_t) st>>>(x, nullptr, CombineArgs{part, topw, sh, sh_logit, sh_logit_stride, topk, nullptr, nullptr, nullptr, 0},
                                                             w, xn, (uint8_t*) xq, n, eps);
    return launch_status("combine_add_norm_q8");
}
int fnx_add_rows(const float* a, const float* b, float* y, size_t n, void* st) {
    if (!a || !b || !y) return fail("add_rows: null argument");
    if (n == 0) return 0;
    k_add_rows<<<(unsigned) std::min<size_t>((n + 255) / 256, 4096), 256, 0, (hipStream_t) st>>>(a, b, y, n);
    return launch_status("add_rows");
}
int fnx_embed_rows(const uint16_t* emb, const int* tokens, int T, int vocab, int n, float* y, void* st) {
    if (!emb || !tokens || !y) return fail("embed_rows: null argument");
    if (T < 1 || vocab < 1 || n < 1) return fail("embed_rows: bad shape");
    k_embed_rows<<<T, 256, 0, (hipStream_t) st>>>(emb, tokens, vocab, n, y);
    return launch_status("embed_rows");
}
// (the forms of the kernel for a launch with a device-side row count: defined at the end of this file)
static bool q8s_live_lds(int bytes);
static void q8s_live_launch(bool tiled, int grid, size_t lds, hipStream_t st, const Q8sArgs& a);
// yq2 (may be null): two matrices, the second one over rows of its own - as long as every block has one tile, which is then of
// one matrix (else refused: the caller launches twice)
// live (may be null): a device word, the rows that count; the others are not read and their products are zeros
static int q8s_launch(const fnx_q8s* const* W, float* const* out, const int* out_stride, int n, const void* yq, int T, void* st, const char* who,
                      const int* gate = nullptr, const void* yq2 = nullptr, const int* live = nullptr) {
    if (!W || !out || !out_stride || !yq || n < 1 || n > 3) return fail(std::string(who) + ": null argument");
    Q8sArgs a{};
    long tiles = 0;
    for (int s = 0; s < n; ++s) {
        if (!W[s] || !W[s]->q || !W[s]->d || !out[s]) return fail(std::string(who) + ": null argument");
        if (W[s]->n_out < 1 || W[s]->n_in < 256 || W[s]->n_in % 256) return fail(std::string(who) + ": columns in 256s");
        if (W[s]->n_in != W[0]->n_in) return fail(std::string(who) + ": the matrices share the activations: the same columns");
        if (((uintptr_t) W[s]->q & 15) || ((uintptr_t) W[s]->d & 3)) return fail(std::string(who) + ": 16-byte aligned rows");
        if (s + 1 < n && W[s]->n_out % 16) return fail(std::string(who) + ": all but the last matrix in whole 16-row tiles");
        if ((W[s]->tiled != 0) != (W[0]->tiled != 0)) return fail(std::string(who) + ": the matrices of one launch share a layout");
        if (out_stride[s] < W[s]->n_out) return fail(std::string(who) + ": out_stride smaller than the rows");
        a.seg[s] = Q8sSeg{W[s]->q, W[s]->d, out[s], W[s]->n_out, out_stride[s]};
        tiles += (W[s]->n_out + 15) / 16;
    }
    if (T < 1 || T > FNX_MAXT) return fail(std::string(who) + ": T out of range");
    a.nseg = n;
    a.cols = W[0]->n_in;
    a.T = T;
    a.yq = (const uint8_t*) yq;
    const size_t lds = (size_t) FNX_MAXT * (a.cols + Q8S_XPAD) + (size_t) FNX_MAXT * (a.cols / 32 + 2) * 4 + (Q8S_WAVES - 1) * 64 * 16;
    if (lds > 150 * 1024) return fail(std::string(who) + ": the window's activations do not fit LDS");
    static bool attr_set[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64 && !attr_set[dev]) {
        if (hipFuncSetAttribute((const void*) k_q8s_gemv<1>, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024) != hipSuccess ||
            hipFuncSetAttribute((const void*) k_q8s_gemv<1, true>, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024) != hipSuccess ||
            !q8s_live_lds(150 * 1024))
            return fail(std::string(who) + ": cannot raise the dynamic LDS limit");
        attr_set[dev] = true;
    }
    static const int per_cu = env_int("FNX_Q8S_BLOCKS_PER_CU", 4, 1, 16);   // what the LDS of a 2048-column matrix lets a CU hold
    const int grid = (int) std::max(1l, std::min<long>((long) per_cu * cu_count(), tiles));
    a.gate = gate;
    a.live = live;
    if (yq2) {
        if (n != 2 || grid < tiles) return fail(std::string(who) + ": two sets of rows want two matrices and a block a tile");
        a.yq2 = (const uint8_t*) yq2;
    }
    if (live) q8s_live_launch(W[0]->tiled != 0, grid, lds, (hipStream_t) st, a);
    else if (W[0]->tiled) k_q8s_gemv<1, true><<<grid, Q8S_WAVES * 64, lds, (hipStream_t) st>>>(a);
    else k_q8s_gemv<1><<<grid, Q8S_WAVES * 64, lds, (hipStream_t) st>>>(a);
    return launch_status(who);
}
size_t fnx_q8s_tile_bytes(int rows, int cols) { return rows < 1 || cols < 64 || cols % 64 ? 0 : (size_t) ((rows + 15) / 16) * 16 * (size_t) cols; }
int fnx_q8s_tile(const int8_t* src, int8_t* dst, int rows, int cols, void* st) {
    if (!src || !dst || src == dst) return fail("q8s_tile: two buffers");
    if (rows < 1 || cols < 256 || cols % 256) return fail("q8s_tile: columns in 256s");
    if (((uintptr_t) src & 15) || ((uintptr_t) dst & 15)) return fail("q8s_tile: 16-byte aligned buffers");
    const size_t pieces = fnx_q8s_tile_bytes(rows, cols) / 16;
    k_q8s_tile<<<(unsigned) std::min<size_t>((pieces + 255) / 256, 65536), 256, 0, (hipStream_t) st>>>(src, dst, rows, cols);
    return launch_status("q8s_tile");
}
int fnx_q8s_gemv(const fnx_q8s* W, const void* yq, float* out, int out_stride, int T, void* st) {
    return q8s_launch(&W, &out, &out_stride, 1, yq, T, st, "q8s_gemv");
}
int fnx_q8s_gemv_segs(const fnx_q8s* const* W, float* const* out, const int* out_stride, int n, const void* yq, int T, void* st) {
    return q8s_launch(W, out, out_stride, n, yq, T, st, "q8s_gemv_segs");
}
}  // extern "C"
static int attn_prep_append(float* qg, float* k, const float* v, const float* q_norm, const float* k_norm, uint16_t* kc, uint16_t* vc, int nq,
                            int nkv, int T, const int* pos0, int max_ctx, float eps, const fnx_rope* rope, void* st, const int* gate) {
    if (!qg || !k || !v || !q_norm || !k_norm || !kc || !vc || !pos0 || !rope) return fail("attn_prep_append: null argument");
    if (nq < 1 || nkv < 1 || nq % nkv || T < 1 || T > FNX_MAXT || max_ctx < AT_VB || max_ctx % AT_VB) return fail("attn_prep_append: bad shape (the cache holds a multiple of 8 positions)");
    RopeDev r;
    for (int pair = 0; pair < AT_NROT / 2; ++pair) {   // rope.hpp:33-39
        const float fe = powf(rope->base, -2.0f * (float) pair / (float) AT_NROT);
        float f = fe;
        if (rope->scaled) {
            const float y = ((float) pair - rope->c_low) / fmaxf(0.001f, rope->c_high - rope->c_low);
            const float ramp = 1.0f - fminf(1.0f, fmaxf(0.0f, y));
            f = fe * (ramp + (1.0f - ramp) * rope->inv_scale);
        }
        r.freq[pair] = f;
    }
    r.mscale = rope->mscale;
    k_attn_prep_append<<<dim3(nq + 2 * nkv, T), AT_HD, 0, (hipStream_t) st>>>(qg, k, v, q_norm, k_norm, kc, vc, nq, nkv, pos0, max_ctx, eps, r, gate);
    return launch_status("attn_prep_append");
}
extern "C" {
int fnx_attn_prep_append(float* qg, float* k, const float* v, const float* q_norm, const float* k_norm, uint16_t* kc, uint16_t* vc, int nq,
                         int nkv, int T, const int* pos0, int max_ctx, float eps, const fnx_rope* rope, void* st) {
    return attn_prep_append(qg, k, v, q_norm, k_norm, kc, vc, nq, nkv, T, pos0, max_ctx, eps, rope, st, nullptr);
}
// splits for a context of up to max_ctx positions
size_t fnx_attn_scratch_floats(int nq, int T, int max_ctx) { return (size_t) T * nq * att_part_slots(attn_splits(max_ctx)) * (AT_HD + 2); }
static int q8s_one(const fnx_q8s* W, const void* yq, float* out, int out_stride, int T, void* st, const int* gate, const int* live = nullptr) {
    return q8s_launch(&W, &out, &out_stride, 1, yq, T, st, "q8s_gemv", gate, nullptr, live);
}
static int attn_launch(const float* qg, const uint16_t* kc, const uint16_t* vc, float* out, uint8_t* outq, int nq, int nkv, const int* pos0, int T,
                       int max_ctx, float* scratch, void* st, const int* gate = nullptr, const int* live = nullptr, unsigned* err = nullptr) {
    if (!qg || !kc || !vc || (!out && !outq) || !pos0 || !scratch) return fail("attn: null argument");
    if (nq < 1 || nkv < 1 || nq % nkv || nq / nkv > AT_MAXQ || T < 1 || T > FNX_MAXT) return fail("attn: bad shape");
    // the V cache lies in blocks of AT_VB positions and the kernel fetches whole blocks: a capacity that ends inside a block would be read past its end
    if (max_ctx < AT_VB || max_ctx % AT_VB) return fail("attn: the cache holds a multiple of 8 positions");
    if (attn_splits(max_ctx) > AT_MAXSPLIT) return fail("attn: the cache is larger than the split table");
    if (((unsigned long long) max_ctx + 3) * nkv * (AT_HD * 2) >= (1ull << 32)) return fail("attn: a cache of 4 GiB or more (the kernel's byte offsets are 32 bits)");
    // the grid covers the cache's capacity (the position is on the device): splits past the context write empty parts
    // (two layers of blocks always: for a window whose queries fit one, the second takes the splits' second halves)
    const int nsplit = attn_splits(max_ctx), waves = (T * (nq / nkv) + 15) / 16;
    float* acc = scratch;
    AttPart* mz = reinterpret_cast<AttPart*>(scratch + (size_t) T * nq * att_part_slots(nsplit) * AT_HD);
    k_attn_part<<<dim3(nsplit, nkv, std::max(2, (waves + AT_WAVES - 1) / AT_WAVES)), AT_THREADS, 0, (hipStream_t) st>>>(qg, kc, vc, acc, mz, nq, nkv, T,
                                                                                                                       nsplit, pos0, max_ctx, gate, live);
    k_attn_combine<<<dim3(nq, T), AT_HD, 0, (hipStream_t) st>>>(qg, acc, mz, out, outq, nq, nkv, nsplit, T, pos0, max_ctx, err, gate, live);
    return launch_status("attn");
}
int fnx_attn(const float* qg, const uint16_t* kc, const uint16_t* vc, float* out, int nq, int nkv, const int* pos0, int T, int max_ctx,
             float* scratch, void* st) {
    if (!out) return fail("attn: null argument");
    return attn_launch(qg, kc, vc, out, nullptr, nq, nkv, pos0, T, max_ctx, scratch, st);
}
static int dec_ws_check(const fnx_dec_ws* ws, const char* who) {
    if (!ws->x || !ws->xn || !ws->qg || !ws->k || !ws->v || !ws->att || !ws->o || !ws->attn_scratch || !ws->xq || !ws->hidden || !ws->logits ||
        !ws->best_v || !ws->best_i || !ws->keys || !ws->err)
        return fail(std::string(who) + ": incomplete workspace");
    return 0;
}
// What is still to be added to x when a layer (or the head) starts: rows (may be null) - the attention half's or the MoE
// half's output - of which only the first *live (live not null) were written.
struct DecPending {
    const float* rows;
    const int* tokens;   // not null: x itself is still to come - the embedding rows of these tokens (nothing else pending then)
    const int* live;
    // set by a layer whose window already made the pass that would come next: the add, the norm with these weights, the
    // q8_1 rows in ws->xq and the copy (if any) - the pass is then skipped by whoever asks for exactly that
    const float* done_w = nullptr;
    const float* done_xcopy = nullptr;
};
// xcopy (may be null): the rows after the add go there too
static int dec_add_norm_q8(const fnx_decoder* D, const DecPending& pend, const float* w, int T, const fnx_dec_ws* ws, void* st, float* xcopy = nullptr,
                           const int* gate = nullptr) {
    if (pend.done_w && pend.done_w == w && (!xcopy || pend.done_xcopy == xcopy)) return 0;   // the window before made this pass
    CombineArgs c{};
    c.live = pend.live;
    c.xcopy = xcopy;
    c.gate = gate;
    if (pend.tokens) {
        c.emb = D->emb;
        c.tokens = pend.tokens;
        c.vocab = D->vocab;
    }
    if (D->n < 32 || D->n % 32 || D->n > 256 * NQ_MAXJ) return fail("decoder: rows of 32 .. 4096 values in whole 32-value blocks");
    // (after a window that made another pass than this one, x already holds the add)
    k_add_norm_q8<false><<<T, 256, 0, (hipStream_t) st>>>(ws->x, pend.done_w ? nullptr : pend.rows, c, w, nullptr, (uint8_t*) ws->xq, D->n, D->eps);
    return launch_status("decoder add_norm_q8");
}
// x (ws->x) through one layer, in place; the layer's own MoE output is left pending for whatever comes next
// live (may be null): a device word, how many of the T rows count; the others still append their K and V (their cache
// cells are overwritten by the next window) but ask no queries and are not routed, so they pull no expert's weights
// gate (may be null): a device word; at zero the layer's dense products and its attention's scan leave at once
// next_w (may be null): the weights of the norm that follows this layer (the next layer's, or the head's), next_xcopy where
// the rows after the add are wanted as well: the window's launch then makes that pass itself
static int dec_layer(const fnx_decoder* D, const fnx_dec_layer* L, int T, const int* pos0, const fnx_dec_ws* ws, DecPending& pend, void* st,
                     const int* live = nullptr, const int* gate = nullptr, const float* next_w = nullptr, float* next_xcopy = nullptr) {
    const int n = D->n, nq = D->nq, nkv = D->nkv;
    if (dec_add_norm_q8(D, pend, L->attn_norm, T, ws, st, nullptr, gate)) return 1;
    {   // q, k and v in one launch (engine.cu:1547-1552)
        const fnx_q8s* w3[3] = {&L->wq, &L->wk, &L->wv};
        float* const o3[3] = {ws->qg, ws->k, ws->v};
        const int s3[3] = {nq * 2 * AT_HD, nkv * AT_HD, nkv * AT_HD};
        if (q8s_launch(w3, o3, s3, 3, ws->xq, T, st, "q8s_gemv_segs", gate, nullptr, live)) return 1;
    }
    if (attn_prep_append(ws->qg, ws->k, ws->v, L->q_norm, L->k_norm, L->kc, L->vc, nq, nkv, T, pos0, D->max_ctx, D->eps, &D->rope, st, gate)) return 1;
    // the attention's rows leave its last kernel in q8_1 form, ready for the output projection
    if (attn_launch(ws->qg, L->kc, L->vc, nullptr, (uint8_t*) ws->xq, nq, nkv, pos0, T, D->max_ctx, ws->attn_scratch, st, gate, live, (unsigned*) ws->err))
        return 1;
    if (q8s_one(&L->wo, ws->xq, ws->o, n, T, st, gate, live)) return 1;
    if (live && !layer_fused_ok(&L->moe, T)) return fail("decoder: a device-side row count needs the one-launch window (unit64 experts, hidden 2048)");
    if (next_w && layer_fused_ok(&L->moe, T) && !shared_is_q8(&L->moe)) {
        // The one-launch window takes the passes either side of it: every block makes its row's x + o and the norm for itself,
        // the row's last block adds the window's rows and makes the next norm's q8_1 rows (k_moe_window.h). Its rows go to
        // ws->xn, which nothing else needs then (ws->o holds the attention half's rows until the last block has read them)
        const WinNext next{ws->x, next_w, ws->xq, next_xcopy, D->eps, ws->o, L->ffn_norm};
        bool done = false;
        if (moe_layer_checked(&L->moe, ws->x, T, ws->xn, &ws->moe, st, live, &next, &done)) return 1;
        if (!done) return fail("decoder: the window did not take the passes around it");
        pend = DecPending{nullptr, nullptr, live};
        pend.done_w = next_w;
        pend.done_xcopy = next_xcopy;
        return 0;
    }
    {   // x += o; xn = norm(x) (fnx_add_norm_q8)
        CombineArgs c{};
        c.gate = gate;
        k_add_norm_q8<false><<<T, 256, 0, (hipStream_t) st>>>(ws->x, ws->o, c, L->ffn_norm, ws->xn, nullptr, n, D->eps);
        if (launch_status("decoder add_norm")) return 1;
    }
    // the MoE half's rows (those that count) are added by the next pass over x
    pend = DecPending{ws->o, nullptr, live};
    return moe_layer_checked(&L->moe, ws->xn, T, ws->o, &ws->moe, st, live);
}
static int dec_shape_check(const fnx_decoder* D, int T, const char* who) {
    if (D->n < 256 || D->n % 256 || D->n > 4096 || D->nq < 1 || D->nkv < 1 || D->nq % D->nkv || D->nq / D->nkv > AT_MAXQ || D->vocab < 1 ||
        D->max_ctx < AT_VB || D->max_ctx % AT_VB)
        return fail(std::string(who) + ": bad model shape");
    if (T < 1 || T > FNX_MAXT) return fail(std::string(who) + ": T out of range");
    return 0;
}
// x += pending; hidden = x; the output norm, the head, argmax
// nv head rows for the tokens from v0; pen (may be null): the last row's penalty list, applied before the picks (engine.cu:2130-2131)
static int dec_head(const fnx_decoder* D, const float* norm, const fnx_q8s* head, int T, const fnx_dec_ws* ws, const DecPending& pend, void* st,
                    const int* gate = nullptr, int nv = 0, int v0 = 0, const int* pen = nullptr, const float* pen_par = nullptr,
                    const int* live = nullptr) {
    if (nv == 0) nv = D->vocab;
    if (dec_add_norm_q8(D, pend, norm, T, ws, st, ws->hidden, gate)) return 1;   // hidden = x, written by the same pass
    if (q8s_one(head, ws->xq, ws->logits, nv, T, st, gate, live)) return 1;
    if (pen && fnx_penalize_row(ws->logits + (size_t) (T - 1) * nv, nv, pen, pen_par, st)) return 1;
    return argmax_launch(ws->logits, nv, T, v0, ws->best_v, ws->best_i, ws->keys, ws->err, st, live);
}
static int decoder_verify(const fnx_decoder* D, const int* tokens, int T, const int* pos0, const fnx_dec_ws* ws, void* st, const int* live) {
    if (!D || !tokens || !pos0 || !ws || !D->layers || !D->out_norm || !D->emb) return fail("decoder_verify: null argument");
    if (dec_shape_check(D, T, "decoder_verify") || dec_ws_check(ws, "decoder_verify")) return 1;
    DecPending pend{nullptr, tokens, nullptr};   // the window's input rows are read by the first pass over them
    for (int l = 0; l < D->nlayers; ++l) {
        const bool last = l + 1 == D->nlayers;
        if (dec_layer(D, &D->layers[l], T, pos0, ws, pend, st, live, nullptr, last ? D->out_norm : D->layers[l + 1].attn_norm, last ? ws->hidden : nullptr))
            return 1;
    }
    return dec_head(D, D->out_norm, &D->head, T, ws, pend, st, nullptr, 0, 0, nullptr, nullptr, live);
}
int fnx_decoder_verify(const fnx_decoder* D, const int* tokens, int T, const int* pos0, const fnx_dec_ws* ws, void* st) {
    return decoder_verify(D, tokens, T, pos0, ws, st, nullptr);
}
int fnx_decoder_layer(const fnx_decoder* D, const fnx_dec_layer* L, const float* x, int T, const int* pos0, const fnx_dec_ws* ws, void* st) {
    if (!D || !L || !x || !pos0 || !ws) return fail("decoder_layer: null argument");
    if (dec_shape_check(D, T, "decoder_layer") || dec_ws_check(ws, "decoder_layer")) return 1;
    if (hipMemcpyAsync(ws->x, x, (size_t) T * D->n * sizeof(float), hipMemcpyDeviceToDevice, (hipStream_t) st) != hipSuccess)
        return fail("decoder_layer: copy of the rows failed");
    DecPending pend{nullptr, nullptr, nullptr};   // nothing is still to be added to the rows
    return dec_layer(D, L, T, pos0, ws, pend, st);
}
static int mtp_draft(const fnx_decoder* D, const fnx_mtp* M, const float* src, const int* tokens, int T, const int* pos0, const fnx_dec_ws* ws,
                     void* st, const int* live, const int* gate = nullptr) {
    if (!D || !M || !src || !tokens || !pos0 || !ws || !M->norm_emb || !M->norm_hid || !M->out_norm || !D->emb) return fail("mtp_draft: null argument");
    if (dec_shape_check(D, T, "mtp_draft") || dec_ws_check(ws, "mtp_draft")) return 1;
    const bool whole = M->dv0 == 0 && M->dv1 == 0;
    if (!whole && (M->dv0 < 0 || M->dv1 <= M->dv0 || M->dv1 > D->vocab)) return fail("mtp_draft: the head's tokens [dv0, dv1) must lie in the vocabulary");
    const int nv = whole ? D->vocab : M->dv1 - M->dv0;
    if (M->head.n_out != nv) return fail("mtp_draft: the head has one row a token of [dv0, dv1)");
    if (M->pen && !M->pen_par) return fail("mtp_draft: a penalty list without its parameters");
    const int n = D->n;
    // R = fc_hid(rms(src)) + fc_emb(rms(emb)): the sum is taken by the layer's first pass over the rows
    if (D->nq * AT_HD >= 2 * n) {
        // both inputs' passes in one launch (fnx_add_norm_q8's, twice): src is only read, nothing is added; the tokens' embedding
        // rows are normed and quantised by the pass that reads them from the table (rms(emb[tokens])). Their q8_1 rows go to
        // the second half of the workspace's q8_1 rows, which hold max(n, nq * 256) values a row.
        uint8_t* xq2 = (uint8_t*) ws->xq + (size_t) FNX_MAXT * (n / 32) * FNX_Q8_1_BLOCK;
        CombineArgs c{};
        c.gate = gate;
        c.tokens = tokens;
        c.vocab = D->vocab;
        c.rows1 = T, c.rows2 = T;
        c.x2 = ws->xn, c.w2 = M->norm_emb, c.xq2 = xq2, c.emb2 = D->emb;
        k_add_norm_q8<false><<<2 * T, 256, 0, (hipStream_t) st>>>(const_cast<float*>(src), nullptr, c, M->norm_hid, nullptr, (uint8_t*) ws->xq, n, D->eps);
        if (launch_status("mtp_draft")) return 1;
        // and the two projections one: a block a tile of one of the two matrices, over that matrix's rows
        const long fc_tiles = (M->fc_hid.n_out + 15) / 16 + (M->fc_emb.n_out + 15) / 16;
        static const int per_cu = env_int("FNX_Q8S_BLOCKS_PER_CU", 4, 1, 16);
        if (fc_tiles <= (long) per_cu * cu_count() && M->fc_hid.n_out % 16 == 0 && M->fc_hid.n_in == M->fc_emb.n_in &&
            (M->fc_hid.tiled != 0) == (M->fc_emb.tiled != 0)) {
            const fnx_q8s* W2[2] = {&M->fc_hid, &M->fc_emb};
            float* out2[2] = {ws->x, ws->o};
            const int stride2[2] = {n, n};
            if (q8s_launch(W2, out2, stride2, 2, ws->xq, T, st, "q8s_gemv", gate, xq2, live)) return 1;
        } else {
            if (q8s_one(&M->fc_hid, ws->xq, ws->x, n, T, st, gate, live)) return 1;
            if (q8s_one(&M->fc_emb, xq2, ws->o, n, T, st, gate, live)) return 1;
        }
    } else {
        {   // nothing to add: src is only read (fnx_add_norm_q8)
            CombineArgs c{};
            c.gate = gate;
            k_add_norm_q8<false><<<T, 256, 0, (hipStream_t) st>>>(const_cast<float*>(src), nullptr, c, M->norm_hid, nullptr, (uint8_t*) ws->xq, n, D->eps);
            if (launch_status("mtp_draft")) return 1;
        }
        if (q8s_one(&M->fc_hid, ws->xq, ws->x, n, T, st, gate, live)) return 1;
        {   // the tokens' embedding rows (rms(emb[tokens]))
            CombineArgs c{};
            c.emb = D->emb;
            c.tokens = tokens;
            c.vocab = D->vocab;
            c.gate = gate;
            k_add_norm_q8<false><<<T, 256, 0, (hipStream_t) st>>>(ws->xn, nullptr, c, M->norm_emb, nullptr, (uint8_t*) ws->xq, n, D->eps);
            if (launch_status("mtp_draft")) return 1;
        }
        if (q8s_one(&M->fc_emb, ws->xq, ws->o, n, T, st, gate, live)) return 1;
    }
    DecPending pend{ws->o, nullptr, nullptr};
    if (dec_layer(D, &M->layer, T, pos0, ws, pend, st, live, gate, M->out_norm, ws->hidden)) return 1;
    return dec_head(D, M->out_norm, &M->head, T, ws, pend, st, gate, nv, M->dv0, M->pen, M->pen_par, live);
}
int fnx_mtp_draft(const fnx_decoder* D, const fnx_mtp* M, const float* src, const int* tokens, int T, const int* pos0, const fnx_dec_ws* ws,
                  void* st) {
    return mtp_draft(D, M, src, tokens, T, pos0, ws, st, nullptr);
}
int fnx_decode_round(const fnx_decoder* D, const fnx_mtp* M, const fnx_round* R, const fnx_dec_ws* ws, void* st) {
    if (!D || !R || !ws || !R->state || !R->rows || !R->ctx || !R->scratch) return fail("decode_round: null argument");
    if (R->speculate && !M) return fail("decode_round: speculation needs the draft layer");
    if (R->ctx_cap < 2 * FNX_MAXT || R->log_cap < 0 || (R->log_cap > 0 && !R->log)) return fail("decode_round: bad buffer sizes");
    if (R->speculate && (R->key_n < 1 || R->key_n > 4 || R->lk < 0 || R->lk > FNX_MAXT - 1))
        return fail("decode_round: keys of 1..4 tokens, up to 15 drafts");
    const int K = R->speculate ? std::max(R->chain, 1) : 1;
    if (K > FNX_MAXT - 1) return fail("decode_round: a chain of up to 15 drafts");
    if (K > 1 && !R->chain_src) return fail("decode_round: the chain needs its source row's buffer");
    hipStream_t s = (hipStream_t) st;
    int* S = R->state;
    if (decoder_verify(D, R->rows, FNX_MAXT, S + FNX_RS_POS, ws, st, S + FNX_RS_ROWS)) return 1;
    k_round_commit<<<1, 64, 0, s>>>(R->rows, ws->best_i, S, R->ctx, R->ctx_cap, D->max_ctx, R->log_cap ? R->log : nullptr, R->log_cap);
    if (R->speculate) {
        // the rows kept and their picks are where the verify left them; the draft layer overwrites both only at its end
        if (mtp_draft(D, M, ws->hidden, ws->best_i, FNX_MAXT, S + FNX_RS_POS_PREV, ws, st, S + FNX_RS_ACCEPTED)) return 1;
        // (with a single draft a round the lookup's launch makes the next window too)
        k_lookup<<<1, LK_THREADS, 0, s>>>(R->ctx, 0, R->key_n, R->lk, ws->best_i, R->scratch + 1, R->scratch, nullptr, S + FNX_RS_NCTX,
                                          S + FNX_RS_ACCEPTED, K == 1 ? S : nullptr, K == 1 ? R->rows : nullptr);
        if (K > 1) {
            // the chain (session.cpp:666-678): step j reads the draft before it at the position after it, from the draft
            // layer's own row; one row, which counts (is routed, runs the big kernels) only while state[CHAIN] is set
            const int* on = S + FNX_RS_CHAIN;
            k_chain_begin<<<1, 256, 0, s>>>(S, R->scratch, ws->best_i, ws->hidden, D->n, R->chain_src, K);
            for (int j = 1; j < K; ++j) {
                if (mtp_draft(D, M, j == 1 ? R->chain_src : ws->hidden, R->scratch + j, 1, S + FNX_RS_CHAIN_POS + (j - 1), ws, st, on, on)) return 1;
                k_chain_keep<<<1, 64, 0, s>>>(S, R->scratch, ws->best_i, j, K);
            }
        }
    }
    if (!R->speculate || K > 1) k_round_window<<<1, 64, 0, s>>>(R->ctx, S, R->scratch + 1, R->scratch, ws->best_i, R->speculate, R->rows);
    return launch_status("decode_round");
}

// ---------------------------------------------------------------- the sampler: candidates on the device, the draw on the host
int fnx_top_tokens(float* logits, int n, int T, int v0, const int* pen_tok, const int* pen_cnt, const int* pen_n, int pen_stride,
                   const float* pen_par, const int* bias_tok, const float* bias_val, const int* bias_off, const int* bias_n, float* out_v,
                   int* out_i, unsigned* err, void* st) {
    if (!logits || !out_v || !out_i || !err) return fail("top_tokens: null argument");
    if (n < SM_N) return fail("top_tokens: a vocabulary slice smaller than the candidates");
    if (T < 1 || T > FNX_MAXT) return fail("top_tokens: T out of range");
    if (n > SM_MAXS * SM_SLICE) return fail("top_tokens: rows of up to 327,680 logits");
    if ((pen_n && (!pen_tok || !pen_cnt || !pen_par || pen_stride < 0)) || (bias_n && (!bias_tok || !bias_val || !bias_off)))
        return fail("top_tokens: a list's count without the list");
    const int nslice = (n + SM_SLICE - 1) / SM_SLICE;
    hipStream_t s = (hipStream_t) st;
    BufferScope candidates(g_cand_order, st);
    k_top_slices<<<dim3(nslice, T), SM_THREADS, 0, s>>>(
        TopArgs{logits, n, v0, nslice, pen_tok, pen_cnt, pen_n, pen_stride, pen_par, bias_tok, bias_val, bias_off, bias_n, err});
    k_top_merge<<<T, SM_MERGE_THREADS, 0, s>>>(logits, n, v0, nslice, out_v, out_i);
    return launch_status("top_tokens");
}
int fnx_penalize_row(float* row, int n, const int* pen, const float* par, void* st) {
    if (!row || !pen || !par || n < 1) return fail("penalize_row: bad argument");
    k_penalize_row<<<1, 256, 0, (hipStream_t) st>>>(row, n, pen, par);
    return launch_status("penalize_row");
}
}  // extern "C"
namespace {
struct HostDist {
    std::vector<int> ids;
    std::vector<double> p;
    double of(int id) const {
        for (size_t i = 0; i < ids.size(); ++i)
            if (ids[i] == id) return p[i];
        return 0.0;
    }
};
// session.cpp:41-75: top_k, then top_p over the untempered softmax of those, then min_p as a logit threshold, then the
// temperature's softmax over what is left; all in double on the f32 candidates
HostDist host_dist(const float* v, const int* id, int ncand, const fnx_sampling& s) {
    const int k = (s.top_k <= 0 || s.top_k > ncand) ? ncand : s.top_k;
    int keep = k;
    const double top = v[0];
    if (s.top_p < 1.f) {
        double z = 0.0, run = 0.0;
        for (int i = 0; i < k; ++i) z += std::exp((double) v[i] - top);
        for (int i = 0; i < k; ++i) {
            run += std::exp((double) v[i] - top) / z;
            if (run >= (double) s.top_p) {
                keep = i + 1;
                break;
            }
        }
    }
    if (s.min_p > 0.f) {
        const float floor_v = v[0] + std::log(s.min_p);
        int i = 1;
        while (i < keep && !(v[i] < floor_v)) ++i;
        keep = std::min(keep, i);
    }
    HostDist d;
    const double inv_t = 1.0 / s.temperature, shift = v[0] * inv_t;
    double z = 0.0;
    for (int i = 0; i < keep; ++i) {
        d.ids.push_back(id[i]);
        d.p.push_back(std::exp(v[i] * inv_t - shift));
        z += d.p.back();
    }
    for (double& x : d.p) x /= z;
    return d;
}
int host_draw(const HostDist& d, double u) {   // session.cpp:77-84
    double run = 0.0;
    for (size_t i = 0; i < d.ids.size(); ++i) {
        run += d.p[i];
        if (u < run) return d.ids[i];
    }
    return d.ids.back();
}
bool sampling_ok(const fnx_sampling* s, int ncand) {
    return s && ncand >= 1 && std::isfinite(s->temperature) && s->temperature > 0.f && s->top_p > 0.f && s->top_p <= 1.f && s->min_p >= 0.f &&
           s->min_p <= 1.f && s->top_k >= 0;
}
}  // namespace
extern "C" {
int fnx_make_dist(const float* cand_v, const int* cand_i, int ncand, const fnx_sampling* s, int* ids, double* p) {
    if (!cand_v || !cand_i || !ids || !p || !sampling_ok(s, ncand)) {
        fail("make_dist: bad argument (temperature > 0, top_p in (0, 1], min_p in [0, 1], top_k >= 0)");
        return -1;
    }
    const HostDist d = host_dist(cand_v, cand_i, ncand, *s);
    std::copy(d.ids.begin(), d.ids.end(), ids);
    std::copy(d.p.begin(), d.p.end(), p);
    return (int) d.ids.size();
}
int fnx_draw(const int* ids, const double* p, int n, double u) {
    if (!ids || !p || n < 1) {
        fail("draw: bad argument");
        return -1;
    }
    HostDist d;
    d.ids.assign(ids, ids + n);
    d.p.assign(p, p + n);
    return host_draw(d, u);
}
int fnx_accept_sampled(const float* cand_v, const int* cand_i, int ncand, int T, const int* rows, const fnx_sampling* s, const int* q_ids,
                       const double* q_p, const int* q_n, int q_stride, const double* u, int nu, int* o, int* used_u) {
    if (!cand_v || !cand_i || !rows || !u || !o || T < 1 || T > FNX_MAXT || !sampling_ok(s, ncand) || (q_n && (!q_ids || !q_p || q_stride < 1))) {
        fail("accept_sampled: bad argument");
        return -1;
    }
    int n = 0, at = 0;
    const auto next_u = [&]() { return at < nu ? u[at++] : (++at, 0.0); };
    for (; n < T; ++n) {
        HostDist d = host_dist(cand_v + (size_t) n * ncand, cand_i + (size_t) n * ncand, ncand, *s);
        if (n + 1 < T) {
            const int draft = rows[n + 1];
            HostDist q;   // empty: a fixed draft, all of q on it
            if (q_n && q_n[n] > 0) {
                q.ids.assign(q_ids + (size_t) n * q_stride, q_ids + (size_t) n * q_stride + q_n[n]);
                q.p.assign(q_p + (size_t) n * q_stride, q_p + (size_t) n * q_stride + q_n[n]);
            }
            const bool fixed = q.ids.empty();
            // the draft stands with probability min(1, p / q)
            if (next_u() * (fixed ? 1.0 : q.of(draft)) < d.of(draft)) {
                o[n] = draft;
                continue;
            }
            // else the row's token comes from max(0, p - q), normalized; p <= q everywhere means p == q up to rounding: from p
            const HostDist whole = d;
            double rest = 0.0;
            for (size_t i = 0; i < d.ids.size(); ++i) {
                const double qi = fixed ? (d.ids[i] == draft ? 1.0 : 0.0) : q.of(d.ids[i]);
                d.p[i] = std::max(0.0, d.p[i] - qi);
                rest += d.p[i];
            }
            if (rest > 1e-12)
                for (double& x : d.p) x /= rest;
            else
                d = whole;
        }
        o[n] = host_draw(d, next_u());
        ++n;
        break;
    }
    if (used_u) *used_u = at;
    if (at > nu) {
        fail("accept_sampled: more uniforms were needed than given");
        return -1;
    }
    return n;
}

// ---------------------------------------------------------------- GGUF ingestion (host_gguf.h)
fnx_gguf* fnx_gguf_open(const char* first_shard) {
    if (!first_shard) {
        fail("gguf_open: null argument");
        return nullptr;
    }
    try {
        return new fnx_gguf(first_shard);
    } catch (const std::exception& e) {
        fail(e.what());
        return nullptr;
    }
}
void fnx_gguf_close(fnx_gguf* g) { delete g; }
int fnx_gguf_shards(const fnx_gguf* g) { return g ? (int) g->maps.size() : 0; }
int fnx_gguf_count(const fnx_gguf* g) { return g ? (int) g->order.size() : 0; }
int fnx_gguf_at(const fnx_gguf* g, int i, fnx_gguf_tensor* t) {
    if (!g || !t || i < 0 || i >= (int) g->order.size()) return fail("gguf_at: bad argument");
    gguf::describe(*g->order[(size_t) i], t);
    return 0;
}
int fnx_gguf_find(const fnx_gguf* g, const char* name, fnx_gguf_tensor* t) {
    if (!g || !name || !t) return fail("gguf_find: null argument");
    const auto it = g->tensors.find(name);
    if (it == g->tensors.end()) return fail(std::string("gguf: no tensor ") + name);
    gguf::describe(it->second, t);
    return 0;
}
size_t fnx_gguf_row_bytes(const fnx_gguf_tensor* t) {
    gguf::BlockShape bs;
    if (!t || !gguf::block_shape(t->type, bs)) return 0;
    return (size_t) (t->ne[0] / bs.values) * (size_t) bs.bytes;
}
int fnx_gguf_key_type(const fnx_gguf* g, const char* key) {
    if (!g || !key) return -1;
    const auto it = g->keys.find(key);
    return it == g->keys.end() ? -1 : it->second;
}
int fnx_gguf_int(const fnx_gguf* g, const char* key, int64_t* v) {
    if (!g || !key || !v) return fail("gguf_int: null argument");
    const auto it = g->ints.find(key);
    if (it == g->ints.end()) return fail(std::string("gguf: no integer key ") + key);
    *v = it->second;
    return 0;
}
int fnx_gguf_num(const fnx_gguf* g, const char* key, double* v) {
    if (!g || !key || !v) return fail("gguf_num: null argument");
    const auto ii = g->ints.find(key);
    const auto fi = g->floats.find(key);
    if (ii != g->ints.end()) *v = (double) ii->second;
    else if (fi != g->floats.end()) *v = fi->second;
    else return fail(std::string("gguf: no number key ") + key);
    return 0;
}
const char* fnx_gguf_str(const fnx_gguf* g, const char* key) {
    if (!g || !key) return nullptr;
    const auto it = g->strings.find(key);
    return it == g->strings.end() ? nullptr : it->second.c_str();
}
int fnx_gguf_expert_rows2(const fnx_gguf_tensor* gate, const fnx_gguf_tensor* up, int r0, int r1, void* dst, size_t dst_bytes, fnx_dw* w,
                          size_t* stride, size_t* bytes) {
    if (!gate || !up) return fail("gguf_expert_rows2: null argument");
    try {
        const size_t n = gguf::expert_rows2(*gate, *up, r0, r1, (uint8_t*) dst, dst_bytes, w, stride);
        if (bytes) *bytes = n;
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}
int fnx_gguf_expert_cols(const fnx_gguf_tensor* down, int c0, int c1, void* dst, size_t dst_bytes, fnx_dw* w, size_t* stride, size_t* bytes) {
    if (!down) return fail("gguf_expert_cols: null argument");
    try {
        const size_t n = gguf::expert_cols(*down, c0, c1, (uint8_t*) dst, dst_bytes, w, stride);
        if (bytes) *bytes = n;
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}
namespace {
struct MoeTensors {
    fnx_gguf_tensor gi, gs, ge, ue, de, gsh, ush, dsh;
};
MoeTensors moe_tensors(const fnx_gguf* g, int layer) {
    const std::string b = "blk." + std::to_string(layer) + ".";
    const auto get = [&](const char* s) {
        const auto it = g->tensors.find(b + s);
        if (it == g->tensors.end()) throw std::runtime_error("gguf: no tensor " + b + s);
        fnx_gguf_tensor t;
        gguf::describe(it->second, &t);
        return t;
    };
    MoeTensors m{get("ffn_gate_inp.weight"), get("ffn_gate_inp_shexp.weight"), get("ffn_gate_exps.weight"), get("ffn_up_exps.weight"),
                 get("ffn_down_exps.weight"), get("ffn_gate_shexp.weight"), get("ffn_up_shexp.weight"), get("ffn_down_shexp.weight")};
    for (const fnx_gguf_tensor* t : {&m.ge, &m.ue, &m.de, &m.gsh, &m.ush, &m.dsh})
        if (t->type != gguf::T_IQ3_S && t->type != QT_Q4_0 && t->type != QT_Q5_1 && t->type != QT_Q8_0 && t->type != QT_IQ4_NL && t->type != QT_IQ4_XS && t->type != QT_Q4_K && t->type != QT_Q5_K)
            throw std::runtime_error(gguf::nm(*t) + ": ggml type " + std::to_string(t->type) +
                                     ", this path reads experts in IQ3_S (and Q4_0, Q5_1, Q8_0, IQ4_NL, IQ4_XS, Q4_K, Q5_K through its plain operators)");
    if (m.gi.ne[0] != m.ge.ne[0] || m.gi.ne[1] != m.ge.ne[2] || m.gs.ne[1] != 1 || m.de.ne[1] != m.ge.ne[0] || m.de.ne[0] != m.ge.ne[1] ||
        m.de.ne[2] != m.ge.ne[2] || m.gsh.ne[0] != m.ge.ne[0] || m.dsh.ne[1] != m.ge.ne[0] || m.dsh.ne[0] != m.gsh.ne[1] || m.gsh.ne[2] != 1 ||
        m.dsh.ne[2] != 1)
        throw std::runtime_error("gguf: the MoE tensors of " + b + " do not fit one another");
    return m;
}
void moe_sizes(const MoeTensors& m, int ff0, int ff1, fnx_moe_bufs* z) {
    z->router_bytes = (size_t) (m.gi.ne[1] + 1) * (size_t) m.gi.ne[0] * 4;
    z->gu_bytes = gguf::expert_rows2(m.ge, m.ue, ff0, ff1, nullptr, 0, nullptr, nullptr);
    z->down_bytes = gguf::expert_cols(m.de, ff0, ff1, nullptr, 0, nullptr, nullptr);
    z->sh_gu_bytes = gguf::expert_rows2(m.gsh, m.ush, ff0, ff1, nullptr, 0, nullptr, nullptr);
    z->sh_down_bytes = gguf::expert_cols(m.dsh, ff0, ff1, nullptr, 0, nullptr, nullptr);
}
}  // namespace
int fnx_gguf_moe_layer_bytes(const fnx_gguf* g, int layer, int ff0, int ff1, fnx_moe_bufs* sizes) {
    if (!g || !sizes) return fail("gguf_moe_layer_bytes: null argument");
    try {
        moe_sizes(moe_tensors(g, layer), ff0, ff1, sizes);
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}
int fnx_gguf_load_moe_layer(const fnx_gguf* g, int layer, int ff0, int ff1, int topk, const fnx_moe_bufs* dev, fnx_moe_layer* L, void* st) {
    if (!g || !dev || !L || !dev->router || !dev->gu || !dev->down || !dev->sh_gu || !dev->sh_down) return fail("gguf_load_moe_layer: null argument");
    try {
        const MoeTensors m = moe_tensors(g, layer);
        fnx_moe_bufs need{};
        moe_sizes(m, ff0, ff1, &need);
        if (dev->router_bytes < need.router_bytes || dev->gu_bytes < need.gu_bytes || dev->down_bytes < need.down_bytes ||
            dev->sh_gu_bytes < need.sh_gu_bytes || dev->sh_down_bytes < need.sh_down_bytes)
            return fail("gguf_load_moe_layer: a device buffer is smaller than fnx_gguf_moe_layer_bytes says");
        if (topk <= 0) {
            const char* arch = fnx_gguf_str(g, "general.architecture");
            int64_t v = 0;
            if (!arch || fnx_gguf_int(g, (std::string(arch) + ".expert_used_count").c_str(), &v)) return fail("gguf_load_moe_layer: no <architecture>.expert_used_count key and no topk given");
            topk = (int) v;
        }
        std::memset(L, 0, sizeof *L);
        L->n = (int) m.ge.ne[0];
        L->ff = ff1 - ff0;
        L->nexp = (int) m.ge.ne[2];
        L->topk = topk;
        std::vector<uint8_t> host(std::max({need.router_bytes, need.gu_bytes, need.down_bytes, need.sh_gu_bytes, need.sh_down_bytes}));
        const auto upload = [&](void* d, size_t n, const char* what) {
            if (hipMemcpy(d, host.data(), n, hipMemcpyHostToDevice) != hipSuccess) throw std::runtime_error(std::string("gguf_load_moe_layer: upload of ") + what + " failed");
        };
        // IQ3_S: raw ggml blocks -> the unit64 layout, in place; other types stay as the file has them. A Q8_0 shared
        // expert (the reference's own form, engine.cu:1600-1604) becomes the split layout of fnx_q8s in its buffers, the
        // same number of bytes: the int8 values of all rows, then the rows' f16 scales.
        const bool routed_iq3s = m.ge.type == gguf::T_IQ3_S && m.de.type == gguf::T_IQ3_S;
        const bool shared_iq3s = m.gsh.type == gguf::T_IQ3_S && m.dsh.type == gguf::T_IQ3_S;
        const bool shared_q8 = m.gsh.type == QT_Q8_0 && m.dsh.type == QT_Q8_0;
        const bool fast = routed_iq3s && (shared_iq3s || shared_q8);   // the one-launch window takes these
        const auto relay = [&](fnx_dw& w, void* d, size_t n) {
            w.p = d;
            if (!fast) return;   // operator by operator raw blocks do as well
            if (fnx_iq3s_repack(d, d, n / FNX_IQ3S_BLOCK * 256, st)) throw std::runtime_error(fnx_last_error());
            w.type = FNX_T_IQ3S_UNIT64;
        };
        std::vector<uint8_t> split;
        const auto split_q8 = [&](fnx_dw& w, fnx_q8s& q, void* d, size_t n) {   // host holds the rows as raw Q8_0 blocks (34 bytes per 32 values)
            const size_t nblk = n / 34, nval = nblk * 32;
            split.resize(n);
            for (size_t b = 0; b < nblk; ++b) {
                std::memcpy(split.data() + 32 * b, host.data() + 34 * b + 2, 32);
                std::memcpy(split.data() + nval + 2 * b, host.data() + 34 * b, 2);
            }
            if (hipMemcpy(d, split.data(), n, hipMemcpyHostToDevice) != hipSuccess) throw std::runtime_error("gguf_load_moe_layer: upload of the shared expert failed");
            q.q = reinterpret_cast<const int8_t*>(d);
            q.d = reinterpret_cast<const uint16_t*>(reinterpret_cast<const uint8_t*>(d) + nval);
            q.n_out = w.n_out;
            q.n_in = w.n_in;
            q.tiled = 0;
            w.p = nullptr;   // the raw form is not kept
        };
        gguf::router_rows(m.gi, m.gs, reinterpret_cast<float*>(host.data()));
        upload(dev->router, need.router_bytes, "the router");
        L->router = dev->router;
        L->router_bf16 = 0;
        gguf::expert_rows2(m.ge, m.ue, ff0, ff1, host.data(), host.size(), &L->gu, &L->gu_stride);
        upload(dev->gu, need.gu_bytes, "gate|up");
        relay(L->gu, dev->gu, need.gu_bytes);
        gguf::expert_cols(m.de, ff0, ff1, host.data(), host.size(), &L->down, &L->down_stride);
        upload(dev->down, need.down_bytes, "down");
        relay(L->down, dev->down, need.down_bytes);
        size_t unused;
        gguf::expert_rows2(m.gsh, m.ush, ff0, ff1, host.data(), host.size(), &L->sh_gu, &unused);
        if (fast && shared_q8) split_q8(L->sh_gu, L->sh_gu_q8, dev->sh_gu, need.sh_gu_bytes);
        else {
            upload(dev->sh_gu, need.sh_gu_bytes, "the shared gate|up");
            if (shared_iq3s) relay(L->sh_gu, dev->sh_gu, need.sh_gu_bytes);
            else L->sh_gu.p = dev->sh_gu;
        }
        gguf::expert_cols(m.dsh, ff0, ff1, host.data(), host.size(), &L->sh_down, &unused);
        if (fast && shared_q8) split_q8(L->sh_down, L->sh_down_q8, dev->sh_down, need.sh_down_bytes);
        else {
            upload(dev->sh_down, need.sh_down_bytes, "the shared down");
            if (shared_iq3s) relay(L->sh_down, dev->sh_down, need.sh_down_bytes);
            else L->sh_down.p = dev->sh_down;
        }
        return 0;
    } catch (const std::exception& e) {
        return fail(e.what());
    }
}

}  // extern "C"

// The dense mat-vec's forms for a launch with a device-side row count (k_q8s_gemv<.., LIVE = true>), asked for here, after
// everything else, so that the kernels before them lie in the code object where they lay without them.
static bool q8s_live_lds(int bytes) {
    return hipFuncSetAttribute((const void*) fnx::k_q8s_gemv<1, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess &&
           hipFuncSetAttribute((const void*) fnx::k_q8s_gemv<1, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess;
}
static void q8s_live_launch(bool tiled, int grid, size_t lds, hipStream_t st, const fnx::Q8sArgs& a) {
    if (tiled) fnx::k_q8s_gemv<1, true, true><<<grid, fnx::Q8S_WAVES * 64, lds, st>>>(a);
    else fnx::k_q8s_gemv<1, false, true><<<grid, fnx::Q8S_WAVES * 64, lds, st>>>(a);
}
