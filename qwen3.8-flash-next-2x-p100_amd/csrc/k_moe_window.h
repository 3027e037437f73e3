// The MoE half of a verify window (the work of Engine::ffn_half, engine.cu:1569-1757 of the reference, on one GPU) as ONE
// launch: router logits -> top-k -> gate|up of the shared and the routed experts -> SwiGLU to q8_1 -> down with the
// combine's chains. The reference runs these as operators of their own inside a captured graph; on this GPU every
// kernel boundary costs the start and the drain of a launch that streams ~100 MB (a fifth of its time), and the
// dependencies between the phases are local to a window row: a row's router logits are needed by that row's blocks only,
// and a row's h (8 KB) is made and used by the same sixteen blocks. So a block belongs to one row for the whole launch
// and the row's blocks hand over through two arrival counters in the workspace - never the whole grid.
//
//   phase R   block (t, g) computes row t's logits of its slice of the router (slice g is read by the blocks g of all
//             rows, which share an XCD and its L2: the router leaves HBM once) and the q8_1 blocks of x[t] (kept in LDS),
//             then arrives on the row's first counter; the shared expert's gate|up item, which needs no pick, runs
//             while the row's logits gather.
//   phase G   every block ranks its row itself (slices of 64 experts a wave, one wave merges) and sweeps its gate|up
//             items - (32 values of h) x (matrix), sixteen waves x four units (gate rows 2 i, 2 i + 1 and their up rows) a
//             sweep, the next item's loads asked for before the current one is decoded; a sweep's sums meet in LDS behind
//             flags and leave as a q8_1 block two sweeps later; the block arrives on the row's second counter.
//   phase D   the block's units of the down matrices: the first trips' weights are asked for before the wait for the row's
//             h; then the trips with the combine's fmaf chain in pick order (kernels.cu:412-419).
//
// What crosses blocks (logits, picks, h) is written and read with agent-scope accesses that go past the XCDs' own L2s;
// no fence that writes back or invalidates a cache is needed. Every wait is bounded: a wait on another block by a
// wall-clock budget, a wait inside the block by a trip count; a wait that gives up sets FNX_ERR_BARRIER in the
// workspace's sync word 0 and the block leaves (the reference bounds its device waits the same way, kernels.cu:884, 899,
// bit 4 of engine_impl.hpp:211-218). A block waits only for blocks of its own row, which lie next to it in the grid: with
// blocks dispatched in order a row's blocks are resident together, or become so as earlier rows finish.
//
// Arithmetic is the operators': the router sums in the fixed 64-lane order, top-k by (value, lower index), the q8_1
// rounding, the IQ3_S sub-block terms, the combine's fmaf chain.
#pragma once

#include <type_traits>

#include "k_moe_layer.h"
#include "moe_window_plan.h"

namespace fnx {

constexpr int WN_THREADS = WN_WAVES * 64;
constexpr int WN_SLOTS = 4, WN_LAG = 2;
constexpr unsigned WN_LDS_SPINS = 1u << 22;   // trips of a wait inside the block before it gives up (tenths of a second)
// the workspace's sync words (zero before the first window; every window leaves them zero)
constexpr int WS_ERR = 0, WS_ROUTED = 1, WS_FIN = 2, WS_ROW0 = 32, WS_ROW_STRIDE = 32;   // a row's words: 0 logits arrivals, 1 h arrivals, 2 blocks done
// A window of few rows has many blocks a row, and their arrivals on one word are taken one after another (some 40 ns
// each: 128 of them were most of such a window's hand-overs). The sixteen rows' cache lines are dealt to the rows that
// count - win_lines(Tl) lines a row, row t's first at line t * win_lines(Tl) - and block g arrives on line g mod lines;
// a wait adds the lines' words up. (The blocks-done word stays on the row's first line: nothing waits for it.)
__host__ __device__ constexpr int win_lines(int Tl) { return Tl <= 1 ? 16 : Tl <= 2 ? 8 : Tl <= 4 ? 4 : Tl <= 8 ? 2 : 1; }
// After the rows' lines: the rows' router logits as the blocks hand them to one another, a 64-bit word an expert - the logit's
// bits and a mark above them - so that a word that has been written says so itself: a block takes its row's logits as soon
// as their words are there, without an arrival count in between (a count costs its own trip to memory, and the wait for the
// stores before it). Zero (not written) before a window and again after it: the row's last block clears them.
constexpr int WS_LX0 = WS_ROW0 + FNX_MAXT * WS_ROW_STRIDE, WS_LX_STRIDE = 1032;   // (64-bit words a row: up to 1,024 experts)
constexpr unsigned long long WS_LX_MARK = 1ull << 32;
static_assert(WS_LX0 % 2 == 0 && WS_LX0 + 2 * FNX_MAXT * WS_LX_STRIDE <= FNX_MOE_SYNC_WORDS, "the header states the sync area's size");

struct WindowArgs {
    int ff, nexp, topk, T, rows;
    const float* x;           // [T][FL_N]
    const void* router;       // [nexp + 1][FL_N]
    int router_bf16;
    const uint8_t* gu;        // routed gate|up: expert e at gu + e * gu_stride, or gu_ep[e]
    size_t gu_stride;
    const uint8_t* const* gu_ep;
    const uint8_t* gu_shared; // null: the shared expert runs elsewhere (its down rows come in sh_part)
    const uint8_t* dn;
    size_t dn_stride;
    const uint8_t* const* dn_ep;
    const uint8_t* dn_shared;
    const float* sh_part;     // [T][rows] when gu_shared is null
    float* logits;            // [T][nexp + 1]
    int* topi;                // [T][topk]
    float* topw;
    uint8_t* xq;              // [T][FL_N / 32] q8_1 blocks (an output for the caller; the blocks keep their own copy in LDS)
    uint32_t* hq;             // [pair][ff / 32][HQ_WORDS]
    float* out;               // [T][rows]
    unsigned* sync;           // FNX_MOE_SYNC_WORDS words
    const int* live;          // may be null; else a device word: rows from *live on are left alone
    fnx_job* jobs_gu;
    fnx_job* jobs_dn;
    int* njobs;
    long long wait_ticks;     // budget of a wait for another block, in ticks of the 100 MHz wall clock
    // What follows the window in a decoder, done here by the row's last block instead of by a launch of its own
    // (fnx_add_norm_q8's pass: the residual add, the next RMS norm, its q8_1 rows). next_x null: not wanted.
    float* next_x = nullptr;            // [T][rows]: x[t] += out[t] for the rows that count
    const float* next_w = nullptr;      // [rows]: the next norm's weights
    uint8_t* next_xq = nullptr;         // [T][rows / 32] q8_1 blocks of rms_norm(x[t]) * next_w
    float* next_xcopy = nullptr;        // may be null: the rows after the add go there as well
    float next_eps = 0.f;
    // What comes before the window in a decoder, done by every block for its own row instead of by a launch (fnx_add_norm_q8's
    // pass without the q8_1 rows): with pre_w set, x is not the normed row but the row before the attention's rows are
    // added: the window's input is rms_norm(x[t] + pre_o[t]) * pre_w (eps = next_eps), and what the row's last block adds
    // the window's rows to is x[t] + pre_o[t]. Only together with next_x = x.
    const float* pre_o = nullptr;       // [T][rows]
    const float* pre_w = nullptr;       // [rows]
};

template <int SBR>
struct WinLds {
    uint32_t tab[SGRID_WORDS];
    uint32_t wp[FL_MAXK + 1][2];       // the picks' gate|up matrices at 1 + k, when they come from a table of pointers
    uint32_t dp[FL_MAXK + 1][2];       // down matrices, the same way
    float hgu[WN_SLOTS][64];           // a sweep's sums: the 32 gate rows', then the 32 up rows'
    int flag[WN_SLOTS][WN_WAVES];
    int made[WN_SLOTS];
    uint2 cand[16][FL_MAXK];
    int sliced[16];
    int ready;                         // picks whose matrices are known
    int pe[FL_MAXK];                   // the picks
    unsigned pk[FL_MAXK];              // their keys
    float pw[FL_MAXK];                 // their weights
    float gate;                        // sigmoid of the shared expert's gate logit
    int harrive;                       // waves of the block that have finished their sweeps
    int hready;                        // 1: the row's h rows are complete; -1: the wait gave up
    int abort;                         // a wait inside the block gave up
    int last;                          // this block is the last of its row to finish
    int fin;                           // the row's ticket among the rows that have finished
    int lists;                         // 1: every row has been ranked, the job lists can be written; -1: the wait gave up
    uint32_t xq[FL_N / 32][FNX_Q8_1_BLOCK / 4];          // the row's q8_1 blocks
    float4 xf[FL_N / 4];                                 // the row of x
    __attribute__((aligned(16))) uint32_t hq[FL_MAXK + 1][SBR][HQ_WORDS];   // the row's pairs' h rows (phase D)
    float zx[FL_MAXK + 1][WN_WAVES / 2][64 / SBR];   // a block of few units: a trip's sums of a unit's rows, from the wave that made them
};

// A wait of one wave for the sum of a word over `lines` consecutive rows' lines. False: the budget ran out (the error bit is set).
__device__ __forceinline__ bool win_wait_lines(const unsigned* p, int lines, unsigned want, long long ticks, unsigned* err) {
    const long long t0 = (long long) wall_clock64();
    const int lane = threadIdx.x & 63;
    while (true) {
        unsigned v = lane < lines ? __hip_atomic_load(p + lane * WS_ROW_STRIDE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
#pragma unroll
        for (int o = 8; o >= 1; o >>= 1) v += (unsigned) __shfl_xor((int) v, o, 64);   // (lines <= 16)
        if (uniform((int) v) >= (int) want) return true;
        if ((long long) wall_clock64() - t0 > ticks) {
            if (lane == 0) atomicOr(err, FNX_ERR_BARRIER);
            return false;
        }
        __builtin_amdgcn_s_sleep(4);
    }
}
// A wait of one wave for a word of another block's. False: the budget ran out (the error bit is set).
__device__ __forceinline__ bool win_wait_word(const unsigned* p, unsigned want, long long ticks, unsigned* err) {
    const long long t0 = (long long) wall_clock64();
    while (true) {
        const unsigned v = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (uniform((int) v) >= (int) want) return true;
        if ((long long) wall_clock64() - t0 > ticks) {
            if ((threadIdx.x & 63) == 0) atomicOr(err, FNX_ERR_BARRIER);
            return false;
        }
        __builtin_amdgcn_s_sleep(4);
    }
}
#ifdef FNX_WIN_TS
// timing build only: wall-clock stamps of every wave at the phases' ends
constexpr int WIN_NTS = 32;
__device__ unsigned long long g_win_ts[1024 * WN_WAVES * WIN_NTS];
#define WIN_TS(i)                                                                                                 \
    do {                                                                                                          \
        if ((threadIdx.x & 63) == 0) g_win_ts[((size_t) blockIdx.x * WN_WAVES + (threadIdx.x >> 6)) * WIN_NTS + (i)] = wall_clock64(); \
    } while (0)
#else
#define WIN_TS(i)
#endif
// The block's barrier as the plain instruction, with the wait for this wave's LDS accesses written out: __syncthreads()
// also waits for every global load in flight, and the down phase meets with its first trips' weights on their way.
__device__ __forceinline__ void win_meet() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
// all of this wave's memory writes have been taken at the device's level before anything after this line
__device__ __forceinline__ void win_stores_done() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Row t of the pass that follows a window in a decoder - k_add_norm_q8<false>'s values in its orders: v = x (+ out, read at
// the device's level: other blocks wrote it), the sum of squares as 256 threads' fmaf chains over columns tid, tid + 256, ...,
// a 64-lane sum a wave, (s0 + s1 + s2 + s3), the row times rsqrtf and the weights, q8_1 blocks a half-wave each. Called by
// all threads of the block (the first 256 work); sh: four floats of LDS.
__device__ __forceinline__ void win_next_row(const WindowArgs& a, int t, bool add, float* sh) {
    constexpr int MAXJ = FL_N / 256;
    const int tid = threadIdx.x, n = a.rows;
    float v[MAXJ], wv[MAXJ];
    float s = 0.f;
    if (tid < 256) {
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) {
            const int i = tid + 256 * j;
            v[j] = a.next_x[(size_t) t * n + i];
            wv[j] = a.next_w[i];
        }
        if (a.pre_o) {   // (the pass before the window, which its blocks made for themselves only: the same add)
            float pv[MAXJ];
#pragma unroll
            for (int j = 0; j < MAXJ; ++j) pv[j] = a.pre_o[(size_t) t * n + tid + 256 * j];
#pragma unroll
            for (int j = 0; j < MAXJ; ++j) v[j] += pv[j];
        }
        if (add) {
            float av[MAXJ];
#pragma unroll
            for (int j = 0; j < MAXJ; ++j)
                av[j] = __uint_as_float(__hip_atomic_load(reinterpret_cast<const unsigned*>(a.out) + (size_t) t * n + tid + 256 * j, __ATOMIC_RELAXED,
                                                          __HIP_MEMORY_SCOPE_AGENT));
#pragma unroll
            for (int j = 0; j < MAXJ; ++j) v[j] += av[j];
        }
        if (add || a.pre_o) {
#pragma unroll
            for (int j = 0; j < MAXJ; ++j) a.next_x[(size_t) t * n + tid + 256 * j] = v[j];
        }
        if (a.next_xcopy) {
#pragma unroll
            for (int j = 0; j < MAXJ; ++j) a.next_xcopy[(size_t) t * n + tid + 256 * j] = v[j];
        }
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) s = fmaf(v[j], v[j], s);
        s = group_sum<64>(s);
        if ((tid & 63) == 0) sh[tid >> 6] = s;
    }
    __syncthreads();
    if (tid < 256) {
        const float r = rsqrtf((sh[0] + sh[1] + sh[2] + sh[3]) / (float) n + a.next_eps);
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) {
            const int i = tid + 256 * j;
            q8_1_store(v[j] * r * wv[j], a.next_xq + ((size_t) t * (n / 32) + i / 32) * FNX_Q8_1_BLOCK, tid & 31);
        }
    }
    __syncthreads();   // sh may be written again
}

// DEC: the launch of a decoder's layer, which may also take the passes either side of the window (next_x, pre_w); without it
// those arguments are not looked at and their code is not there
// RBF: the router's rows are bf16 (a.router_bf16). A template argument, and a row past the block's slice is loaded all the same
// (the slice's last, its sum thrown away): the number of loads behind the block's row of x is then the same on every path,
// the compiler knows it, and the block's first meeting does not wait for the router's rows as well.
template <int SBR, bool DEC = false, bool RBF = false>
__global__ void __launch_bounds__(WN_THREADS) k_moe_window(const WindowArgs a) {
    __shared__ WinLds<SBR> S;
    constexpr int RW = 64 / SBR, RMAX = SBR / 8, NB = RMAX == 4 ? 2 : 3, DEPTH = RMAX == 4 ? 1 : 2;   // rows a unit; units a wave and trip at most; trips' buffers
    const int tid = threadIdx.x, wave = uniform(tid >> 6), lane = tid & 63;
    // the codebook's 512 unsigned entries: the launch's first load; the blocks read different signed forms of the table in
    // memory (2 KiB apart) and negate them back, so that not every wave of the grid asks the same sixteen cache lines at once
    const int form = (2 * (int) blockIdx.x + (tid >> 9)) & 15;
    const uint32_t tab0 = signed_entry(g_sgrid.v[(form << 9) + (tid & 511)], form);
    const int T = a.T, topk = a.topk, nexp = a.nexp, LS = nexp + 1, P = T * topk;
    const int Tl = a.live ? uniform(max(0, min(*a.live, T))) : T;
    if (Tl <= 0) return;
    const WinPlan pl = win_plan((int) gridDim.x, Tl, nexp, topk, a.gu_shared != nullptr, a.ff);
    const int t = (int) blockIdx.x / pl.G, g = (int) blockIdx.x - t * pl.G;
    if (t >= Tl) return;
    WIN_TS(0);
    const int k0 = pl.k0, nk = pl.nk, qpp = pl.qpp;
    unsigned* const srow = a.sync + WS_ROW0 + t * win_lines(Tl) * WS_ROW_STRIDE;   // the row's first line
    // the line this block arrives on (worked out where it is wanted: one value fewer to keep through the launch)
    auto arrival_line = [&] { return srow + (g & (win_lines(Tl) - 1)) * WS_ROW_STRIDE; };
    unsigned* const serr = a.sync + WS_ERR;
    unsigned long long* const lx = reinterpret_cast<unsigned long long*>(a.sync + WS_LX0) + (size_t) t * WS_LX_STRIDE;   // the row's logits on their way
    const float* xrow = a.x + (size_t) t * FL_N;

    // ---------------------------------------------------------------- phase R: loads
    // the row of x as the router's sums take it (lane l: float4 chunks l, l + 64, ...), and the values this wave quantises
    // (blocks 4 wave .. 4 wave + 3 of the row's 64, a half-wave a block)
    // (a row of x is 512 float4: half the block's threads bring one each into LDS for all sixteen waves; every wave loading
    // the row itself was 128 KB through the CU's vector cache on top of the router's rows)
    float4 xmine = make_float4(0.f, 0.f, 0.f, 0.f);
    if (tid < FL_N / 4) xmine = reinterpret_cast<const float4*>(xrow)[tid];
    float xv[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) xv[r] = xrow[(4 * wave + 2 * r + (lane >> 5)) * 32 + (lane & 31)];
    // With pre_w the row is still to be made: (x + o) * rsqrt(mean square + eps) * w, k_add_norm_q8's values in its orders - the
    // sum of squares as 256 threads' fmaf chains over columns tid, tid + 256, ..., a 64-lane sum a wave, (s0 + s1 + s2 + s3).
    // Every block of the row makes it for itself; its loads go out here, before the router's rows, which stay in flight
    // while the sum is made
    const bool pre = DEC && a.pre_w != nullptr;
    const float* orow = pre ? a.pre_o + (size_t) t * FL_N : xrow;
    const float* wrow = pre ? a.pre_w : xrow;
    float4 om = make_float4(0.f, 0.f, 0.f, 0.f), wm = om;
    float ov[2] = {0.f, 0.f}, wv2[2] = {0.f, 0.f}, sq[FL_N / 256], so[FL_N / 256];
    if (pre) {
        if (tid < FL_N / 4) om = reinterpret_cast<const float4*>(orow)[tid], wm = reinterpret_cast<const float4*>(wrow)[tid];
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int i = (4 * wave + 2 * r + (lane >> 5)) * 32 + (lane & 31);
            ov[r] = orow[i], wv2[r] = wrow[i];
        }
        if (tid < 256) {
#pragma unroll
            for (int j = 0; j < FL_N / 256; ++j) sq[j] = xrow[tid + 256 * j], so[j] = orow[tid + 256 * j];
        }
    }
    // this wave's router rows: rows r0 + wave, r0 + wave + 16, ... of the block's slice, two at a time
    const int r0 = g * pl.rpb, r1 = min(nexp, r0 + pl.rpb);
    auto load_router_row = [&](int row, float4(&w)[8]) {
        row = min(row, max(r1, 1) - 1);
        if constexpr (RBF) {
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const uint2 u = reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(a.router) + (size_t) row * FL_N)[c * 64 + lane];
                w[c] = make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                                   __uint_as_float(u.y & 0xffff0000u));
            }
        } else {
#pragma unroll
            for (int c = 0; c < 8; ++c) w[c] = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(a.router) + (size_t) row * FL_N)[c * 64 + lane];
        }
    };
    // the fixed order of k_gemv_rows (and of the CPU oracle): chunks in order, fmaf over x, y, z, w, then the xor butterfly
    auto router_dot = [&](const float4(&w)[8], const float4(&x)[8]) {
        float s = 0.f;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            s = fmaf(w[c].x, x[c].x, s);
            s = fmaf(w[c].y, x[c].y, s);
            s = fmaf(w[c].z, x[c].z, s);
            s = fmaf(w[c].w, x[c].w, s);
        }
        return group_sum<64>(s);
    };
    float4 wa[8], wb[8];
    load_router_row(r0 + wave, wa);
    load_router_row(r0 + wave + WN_WAVES, wb);
    if (pre) {
        if (tid < 256) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < FL_N / 256; ++j) {
                const float v = sq[j] + so[j];
                s = fmaf(v, v, s);
            }
            s = group_sum<64>(s);
            if (lane == 0) S.hgu[0][wave] = s;
        }
        win_meet();
        const float rn = rsqrtf((S.hgu[0][0] + S.hgu[0][1] + S.hgu[0][2] + S.hgu[0][3]) / (float) FL_N + a.next_eps);
        xmine = make_float4((xmine.x + om.x) * rn * wm.x, (xmine.y + om.y) * rn * wm.y, (xmine.z + om.z) * rn * wm.z, (xmine.w + om.w) * rn * wm.w);
#pragma unroll
        for (int r = 0; r < 2; ++r) xv[r] = (xv[r] + ov[r]) * rn * wv2[r];
        win_meet();   // S.hgu is free again
    }

    // ---------------------------------------------------------------- LDS: flags, the codebook, the row's q8_1 blocks
    if (tid < WN_SLOTS * WN_WAVES) (&S.flag[0][0])[tid] = 0;
    if (tid < WN_SLOTS) S.made[tid] = 0;
    if (tid < 16) S.sliced[tid] = 0;
    if (tid == 0) {
        S.ready = 0;
        S.harrive = 0;
        S.hready = 0;
        S.abort = 0;
        S.last = 0;
        S.fin = -1;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) S.tab[tid + i * WN_THREADS] = signed_entry(tab0, (tid >> 9) + 2 * i);
    if (tid < FL_N / 4) S.xf[tid] = xmine;
#pragma unroll
    for (int r = 0; r < 2; ++r) {   // kernels.cu:131-145 (quantize_q8_1), a half-wave a block
        const int b = 4 * wave + 2 * r + (lane >> 5), l32 = lane & 31;
        const float xi = xv[r];
        const float amax = group_max<32>(fabsf(xi)), sum = group_sum<32>(xi);
        const float d = amax / 127.0f;
        const int8_t qv = amax == 0.0f ? (int8_t) 0 : (int8_t) roundf(xi / d);
        reinterpret_cast<int8_t*>(&S.xq[b][1])[l32] = qv;
        if (l32 == 0) S.xq[b][0] = (uint32_t) float_to_half_bits(d) | (uint32_t) float_to_half_bits(sum) << 16;
    }
    // the block meets with the router's rows still on their way: they were asked for last, after what the lines above wait for
    win_meet();
    WIN_TS(1);
    if (g == 0 && tid < (FL_N / 32) * (FNX_Q8_1_BLOCK / 4))   // the caller's copy of the row's q8_1 blocks
        reinterpret_cast<uint32_t*>(a.xq + (size_t) t * (FL_N / 32) * FNX_Q8_1_BLOCK)[tid] = (&S.xq[0][0])[tid];

    // ---------------------------------------------------------------- phase R: the sums, the arrival
    float4 xr[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) xr[c] = S.xf[c * 64 + lane];
    {
        int row = r0 + wave;
        while (true) {
            const float va = router_dot(wa, xr), vb = router_dot(wb, xr);
            if (lane == 0) {   // to the caller's array, and marked to the row's other blocks
                if (row < r1) {
                    a.logits[(size_t) t * LS + row] = va;
                    __hip_atomic_store(&lx[row], WS_LX_MARK | __float_as_uint(va), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                if (row + WN_WAVES < r1) {
                    a.logits[(size_t) t * LS + row + WN_WAVES] = vb;
                    __hip_atomic_store(&lx[row + WN_WAVES], WS_LX_MARK | __float_as_uint(vb), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            row += 2 * WN_WAVES;
            if (row >= r1) break;
            load_router_row(row, wa);
            load_router_row(row + WN_WAVES, wb);
        }
        WIN_TS(2);
    }

    // ---------------------------------------------------------------- phase G
    // the lane's sub-block of the row's activations
    int xs[8];
    float dx;
    {
        const uint32_t* xb = S.xq[lane];
        dx = half_bits_to_float(xb[0] & 0xFFFFu);
#pragma unroll
        for (int j = 0; j < 8; ++j) xs[j] = (int) xb[1 + j];
    }
    const int I0 = g * pl.ipb, I1 = min(pl.per_row, I0 + pl.ipb), nsweep = max(I1 - I0, 0);   // this block's items of its row
    const PackedVOffs o = packed_voffs(lane);
    const int uo_g = wave * 2 * UNIT_BYTES, uo_u = uo_g + a.ff * UNIT_BYTES;   // the wave's gate units and up units from an item's first gate unit
    struct Item {
        int j, k;   // block of 32 h values, matrix (0: the shared expert's, k: pick k - 1's)
    };
    auto item_of = [&](int I) {
        Item m;
        m.j = uniform(I / nk);
        m.k = k0 + I - m.j * nk;
        return m;
    };
    auto step = [&](Item& m) {
        if (++m.k > topk) {
            m.k = k0;
            ++m.j;
        }
    };
    PackedSub A[4];
    auto issue_from = [&](const uint8_t* e, int j) {   // e: wave-uniform
        const __amdgpu_buffer_rsrc_t mtx = matrix_rsrc(e);
        const int ub = uniform(j) * 32 * UNIT_BYTES;
        A[0] = load_packed_buf(mtx, ub + uo_g, o);
        A[1] = load_packed_buf(mtx, ub + uo_g + UNIT_BYTES, o);
        A[2] = load_packed_buf(mtx, ub + uo_u, o);
        A[3] = load_packed_buf(mtx, ub + uo_u + UNIT_BYTES, o);
    };
    // a wait on a word of this block's LDS; false: gave up (or another wave did)
    auto lds_wait = [&](auto cond) {
        for (unsigned n = 0; !cond(); ++n) {
            // (every condition here is wave-uniform and says so: a loop left on a per-lane condition would make the compiler treat
            // the item counters that live across it as per-lane values, and every load that takes one as a loop over the lanes)
            if (n >= WN_LDS_SPINS || uniform(__hip_atomic_load(&S.abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP))) {
                if (lane == 0) {
                    __hip_atomic_store(&S.abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    atomicOr(serr, FNX_ERR_BARRIER);
                }
                return false;
            }
            __builtin_amdgcn_s_sleep(1);
        }
        return true;
    };
    Item ma = item_of(I0);
    const bool early = nsweep > 0 && ma.k == 0;   // the run starts with a shared expert's item: no pick needed to ask for it
    if (early) issue_from(a.gu_shared, ma.j);
    const int sc_shift = 4 * (lane & 1);
    // where a lane's sum goes after reduce4_units: the 16-lane rows hold gate 2 i, up 2 i, gate 2 i + 1, up 2 i + 1
    const int zidx = (lane & 16 ? 32 : 0) + 2 * wave + (lane >> 5);
    auto decode = [&](int sw) {
        const int slot = sw & (WN_SLOTS - 1);
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            int w4[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) w4[j] = *reinterpret_cast<const int*>(reinterpret_cast<const uint8_t*>(S.tab) + packed_addr(A[r].idx, j));
            const int sc = 1 + 2 * (int) ((A[r].sc >> sc_shift) & 0xFu);
            const float dw = half_bits_to_float(A[r].d);
            int sum = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) sum = __builtin_amdgcn_sdot4(w4[j], xs[j], sum, false);
            // one sub-block's term as the reference forms it: (d_w * d_x) * (float) (sumi * (1 + 2 s))
            v[r] = (dw * dx) * (float) __mul24(sum, sc);
        }
        const float z = reduce4_units(v[0], v[1], v[2], v[3]);   // units: gate 2 i, gate 2 i + 1, up 2 i, up 2 i + 1
        // the slot's last block (of sweep sw - WN_SLOTS) must have been made: nearly always long ago
        if (sw >= WN_SLOTS &&
            !lds_wait([&] { return uniform(__hip_atomic_load(&S.made[slot], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP)) >= sw - WN_SLOTS + 1; }))
            return false;
        if ((lane & 15) == 0) S.hgu[slot][zidx] = z;
        if (lane == 0) __hip_atomic_store(&S.flag[slot][wave], sw + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
        return true;
    };
    // the q8_1 block of sweep q, by the first half of the wave whose turn it is (k_moe_h, moe.cuh:597-608)
    auto make_block = [&](int q) {
        const int slot = q & (WN_SLOTS - 1);
        if (!lds_wait([&] {   // all sixteen waves' values of sweep q must be there
                const int f = lane < WN_WAVES ? __hip_atomic_load(&S.flag[slot][lane], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) : q + 1;
                return __ballot(f < q + 1) == 0ull;
            }))
            return false;
        const Item m = item_of(I0 + q);
        const int pair = m.k > 0 ? t * topk + m.k - 1 : P + t;
        if (lane < 32) {
            const float h = silu_f(S.hgu[slot][lane]) * S.hgu[slot][32 + lane];
            const float amax = group_max<32>(fabsf(h));
            const float d = amax / 127.0f;
            const uint32_t qv = amax == 0.0f ? 0u : (uint32_t) (uint8_t) (int8_t) roundf(h / d);
            uint32_t word = qv | (uint32_t) __shfl_down((int) qv, 1, WAVE) << 8;
            word |= (uint32_t) __shfl_down((int) word, 2, WAVE) << 16;
            uint32_t* dst = a.hq + ((size_t) pair * qpp + m.j) * HQ_WORDS;
            if ((lane & 3) == 0) __hip_atomic_store(&dst[lane >> 2], word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (lane == 0) __hip_atomic_store(&dst[8], __float_as_uint(half_bits_to_float(float_to_half_bits(d))), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (lane == 0) __hip_atomic_store(&S.made[slot], q + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
        return true;
    };
    int sw = 0;
    if (early) {   // the shared expert's item while the row's logits gather
        if (!decode(0)) return;
        sw = 1;
    }
    WIN_TS(13);
    // The row's picks (moe.cuh:382-411: greater value first, the lower index on a tie; w_k = exp(l_k - l_0) / sum in pick
    // order). Every wave with a slice lists the topk greatest of its 64 experts in order; wave 0 merges the slices' lists by
    // their heads and hands each pick's matrix out as soon as it is known.
    const int ns = (nexp + 63) >> 6;   // slices of 64 experts
    for (int sl = wave; sl < ns; sl += WN_WAVES) {
        const int e = 64 * sl + lane;
        // the slice's logits, as soon as the row's blocks have written them all: every word says so itself
        unsigned long long lw;
        {
            const long long t0 = (long long) wall_clock64();
            while (true) {
                lw = e < nexp ? __hip_atomic_load(&lx[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : WS_LX_MARK | __float_as_uint(-INFINITY);
                if (__ballot(lw == 0ull) == 0ull) break;
                if ((long long) wall_clock64() - t0 > a.wait_ticks || uniform(__hip_atomic_load(&S.abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP))) {
                    if (lane == 0) {
                        __hip_atomic_store(&S.abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        atomicOr(serr, FNX_ERR_BARRIER);
                    }
                    return;
                }
                __builtin_amdgcn_s_sleep(2);
            }
        }
        WIN_TS(3);
        const float v = __uint_as_float((unsigned) lw);
        unsigned key = rank_key(v);
        for (int k = 0; k < topk; ++k) {
            const unsigned m = wave_umax(key);
            const unsigned long long hold = m > RANK_KEY_NEG_INF ? __ballot(key == m) : 0ull;
            const int l = hold ? (int) __builtin_ctzll(hold) : 64;   // the lowest lane that holds the maximum is the lowest expert
            key = lane == l ? 0u : key;
            if (lane == 0) S.cand[sl][k] = make_uint2(hold ? m : 0u, (uint32_t) (hold ? 64 * sl + l : nexp));
        }
        if (lane == 0) __hip_atomic_store(&S.sliced[sl], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    WIN_TS(4);
    if (wave == 0) {   // the merge
        if (!lds_wait([&] {
                const int f = lane < ns ? __hip_atomic_load(&S.sliced[lane], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) : 1;
                return __ballot(f == 0) == 0ull;
            }))
            return;
        // All of the row's candidates in registers, entry p of list j in lane (16 j + p) mod 64 of register (16 j + p) / 64: a
        // pick is the greatest key of them all, and among equal keys the first in that order - the lists follow the experts'
        // order and each list its own, so that is the lowest expert. (Entries past a list's topk, and lists past the last
        // slice, count as nothing.) The merging wave goes first on its SIMD: the block's sweeps wait for its picks.
        static_assert(FL_MAXK == 16, "sixteen entries a list, four lists a register");
        WIN_TS(14);
        __builtin_amdgcn_s_setprio(3);
        // (once for rows of up to 512 experts - two registers of candidates - and once for more: the merging wave's instructions
        // are the block's critical path here)
        auto merge = [&](auto NRC) {
            constexpr int NR = decltype(NRC)::value;
            unsigned ck[NR];
            int ce[NR];
            {
                const uint2* flat = &S.cand[0][0];
#pragma unroll
                for (int q = 0; q < NR; ++q) {
                    const uint2 c = flat[q * 64 + lane];
                    const bool there = 4 * q + (lane >> 4) < ns && (lane & 15) < topk;
                    ck[q] = there ? c.x : 0u;
                    ce[q] = (int) c.y;
                }
            }
            unsigned long long low_taken = 0ull;   // which of experts 0 .. 63 are picked: what a row with fewer than topk finite logits falls back on
            for (int k = 0; k < topk; ++k) {
                unsigned mx = ck[0];
#pragma unroll
                for (int q = 1; q < NR; ++q) mx = max(mx, ck[q]);
                unsigned m = wave_umax(mx);
                int idx;
                if (m > RANK_KEY_NEG_INF) {
                    unsigned long long b[NR];
#pragma unroll
                    for (int q = 0; q < NR; ++q) b[q] = __ballot(ck[q] == m);
                    int q0 = NR - 1;
                    unsigned long long bb = b[NR - 1];
#pragma unroll
                    for (int q = NR - 2; q >= 0; --q)
                        if (b[q]) q0 = q, bb = b[q];
                    const int l = (int) __builtin_ctzll(bb);
                    idx = __builtin_amdgcn_readlane(ce[NR - 1], l);
#pragma unroll
                    for (int q = NR - 2; q >= 0; --q) {
                        const int e = __builtin_amdgcn_readlane(ce[q], l);
                        if (q0 == q) idx = e;
                    }
#pragma unroll
                    for (int r = 0; r < NR; ++r) ck[r] = r == q0 && lane == l ? 0u : ck[r];
                } else {   // nothing finite is left: the lowest expert not picked yet, with weight exp(-inf) = 0
                    m = RANK_KEY_NEG_INF;
                    idx = (int) __builtin_ctzll(~low_taken);
                }
                if (idx < 64) low_taken |= 1ull << idx;
                // The pick is handed out at once: the sweeps need not wait for the whole ranking. Matrices that lie a stride apart
                // are found by the waves that want them; a table of pointers is looked up here, for both matrices (a sweep or trip
                // that looked its pointer up in memory would wait for the lookup, and with it for every load of weights in flight).
                if (a.gu_ep) {
                    const uint8_t* e = a.gu_ep[idx];
                    if (lane == 0) {
                        S.wp[1 + k][0] = (uint32_t) (uintptr_t) e;
                        S.wp[1 + k][1] = (uint32_t) ((uint64_t) (uintptr_t) e >> 32);
                    }
                }
                if (a.dn_ep) {
                    const uint8_t* ed = a.dn_ep[idx];
                    if (lane == 0) {
                        S.dp[1 + k][0] = (uint32_t) (uintptr_t) ed;
                        S.dp[1 + k][1] = (uint32_t) ((uint64_t) (uintptr_t) ed >> 32);
                    }
                }
                if (lane == 0) {
                    S.pe[k] = idx;
                    S.pk[k] = m;
                    __hip_atomic_store(&S.ready, k + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            }
        };
        if (ns <= 8) merge(std::integral_constant<int, 2>{});
        else merge(std::integral_constant<int, 4>{});
        __builtin_amdgcn_s_setprio(0);
        WIN_TS(15);
        WIN_TS(5);
    }
    // an item's loads, once its matrix is known: matrix 0 is the shared expert's, matrix k pick k - 1's
    auto issue = [&](const Item& m) {
        const uint8_t* e = a.gu_shared;
        const int mk_ = uniform(m.k);
        if (mk_ > 0) {
            if (!lds_wait([&] { return uniform(__hip_atomic_load(&S.ready, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP)) >= mk_; })) return false;
            if (a.gu_ep) {
                const uint2 p = *reinterpret_cast<const uint2*>(S.wp[mk_]);
                e = (const uint8_t*) (uintptr_t) ((uint64_t) (uint32_t) uniform((int) p.x) | (uint64_t) (uint32_t) uniform((int) p.y) << 32);
            } else {
                e = a.gu + (size_t) uniform(S.pe[mk_ - 1]) * a.gu_stride;
            }
        }
        issue_from(e, m.j);
        return true;
    };
    // Every wave of the block makes the same sweeps: each slot sees all sixteen arrive. An item's loads are asked for when
    // the item before it has been decoded; two sweeps later the wave whose turn it is makes the sweep's q8_1 block.
    if (nsweep > 0) {
        if (early) {
            if (nsweep > 1) {
                step(ma);
                if (!issue(ma)) return;
            }
        } else if (!issue(ma)) return;
        for (; sw < nsweep; ++sw) {
            // the oldest wave of a SIMD issues first, so a block's waves drift apart sweep by sweep: every wave takes each of
            // the four priorities in turn
            switch ((wave >> 2) + sw & 3) {
                case 0: __builtin_amdgcn_s_setprio(0); break;
                case 1: __builtin_amdgcn_s_setprio(1); break;
                case 2: __builtin_amdgcn_s_setprio(2); break;
                default: __builtin_amdgcn_s_setprio(3); break;
            }
            if (!decode(sw)) return;
            WIN_TS(16 + (sw & 15));
            if (sw + 1 < nsweep) {
                step(ma);
                if (!issue(ma)) return;
            }
            const int q = sw - WN_LAG;   // the sweep whose block is due; wave q mod 16 makes it
            if (q >= 0 && (q & (WN_WAVES - 1)) == wave)
                if (!make_block(q)) return;
        }
        for (int q = max(nsweep - WN_LAG, 0); q < nsweep; ++q)   // the last sweeps' blocks
            if ((q & (WN_WAVES - 1)) == wave)
                if (!make_block(q)) return;
    }

    __builtin_amdgcn_s_setprio(0);
    WIN_TS(6);
    // ---------------------------------------------------------------- phase D
    const bool ext = a.sh_part != nullptr;   // the shared expert's rows come from memory: the trips are the picks only
    const int first = ext ? 1 : 0;
    // A block of few units (a window of few rows, whose rows have many blocks) would leave most waves standing by while one
    // wave a unit makes the row's trips one after the other: there the trips are dealt out as well - wave w takes unit
    // w % dwaves and, of the row's trips, every TG-th from trip w / dwaves on; the sums meet in LDS and the units' first
    // waves run the combine's chain over them in the picks' order (the same operations on the same values).
    // (Only where a wave has one unit: the other forms of the phase are compiled without it.)
    const int R = pl.R;
    const int kb = lane % SBR, gl = lane / SBR;
    // trip 0 is the shared expert's, trips 1 .. topk the picks in order
    auto down_matrix = [&](int trip) -> const uint8_t* {
        if (trip == 0) return a.dn_shared;
        if (!a.dn_ep) return a.dn + (size_t) uniform(S.pe[trip - 1]) * a.dn_stride;
        const uint2 p = *reinterpret_cast<const uint2*>(S.dp[trip]);
        return (const uint8_t*) (uintptr_t) ((uint64_t) (uint32_t) uniform((int) p.x) | (uint64_t) (uint32_t) uniform((int) p.y) << 32);
    };
    // The rest of the phase once for every number of units a wave can have (RC::value == R): with the count a constant, every
    // load of a trip is issued on every path, the compiler knows how many loads lie behind the one it waits for, and a decode
    // waits for its own trip's weights only - not, as with loads under "if (r < R)", for everything in flight.
    auto down_phase = [&](auto RC) -> bool {
    constexpr int RR = decltype(RC)::value;
    int TG = 1;
    if constexpr (RR == 1) TG = pl.dwaves <= WN_WAVES / 2 && WN_WAVES % pl.dwaves == 0 ? WN_WAVES / pl.dwaves : 1;
    const bool dwave = TG > 1 || wave < pl.dwaves;
    const int tgrp = TG > 1 ? wave / pl.dwaves : 0, uw = TG > 1 ? wave - tgrp * pl.dwaves : wave;
    const int u0 = g * pl.upb + uw * RR;   // this wave's units of every matrix
    auto trip_of = [&](int i) { return first + tgrp + i * TG; };   // the wave's i-th trip
    PackedSub B[NB][RR];
    auto issue_trip = [&](PackedSub(&buf)[RR], int trip) {
        const __amdgpu_buffer_rsrc_t mtx = matrix_rsrc(down_matrix(trip));
#pragma unroll
        for (int r = 0; r < RR; ++r) buf[r] = load_packed_buf(mtx, (u0 + r) * UNIT_BYTES, o);
    };
    // The picks are known (this block ranked its row), so the first trips' weights are asked for before the wait for h.
    // (The hand-over of the last pick's matrix has been seen by every wave that swept; a block without items waits here.)
    if (!lds_wait([&] { return uniform(__hip_atomic_load(&S.ready, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP)) >= topk; })) return false;
    if (nsweep > 0) {   // this wave's h blocks are out: arrive
        win_stores_done();
        int old = 0;
        if (lane == 0) old = atomicAdd(&S.harrive, 1);
        if (uniform(old) == WN_WAVES - 1)
            if (lane == 0) __hip_atomic_fetch_add(&arrival_line()[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    WIN_TS(7);
    if (wave == 2) {   // the picks' weights from their keys (the merging wave has the block waiting for it: it leaves this to a
                       // wave that waits for the row's h here); the row's first block writes the picks and their weights out
        const unsigned mk = lane < topk ? S.pk[lane] : 0u;
        const int ei = lane < topk ? S.pe[lane] : 0x7fffffff;
        const float top0 = rank_key_inv((unsigned) __builtin_amdgcn_readlane((int) mk, 0));
        const float ek = mk > RANK_KEY_NEG_INF ? fnx_expf(rank_key_inv(mk) - top0) : 0.f;   // a pick without a finite logit weighs nothing
        float z = 0.f;
        for (int k = 0; k < topk; ++k) z += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ek), k));
        const float wk = z > 0.f ? ek / z : 0.f;
        if (lane < topk) S.pw[lane] = wk;
        if (g == 0) {
            if (lane < topk) {
                __hip_atomic_store(&a.topi[t * topk + lane], ei, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&a.topw[t * topk + lane], wk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            win_stores_done();
            if (lane == 0) __hip_atomic_fetch_add(&a.sync[WS_ROUTED], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (wave == 1) {   // the shared expert's gate: the router's last row against the row of x, in the router's order
        float4 wg[8];
        int l2 = lane;
        asm volatile("" : "+v"(l2));   // the addresses are worked out here, not kept in registers since phase R
#pragma unroll
        for (int c = 0; c < 8; ++c) xr[c] = S.xf[c * 64 + l2];
        if constexpr (RBF) {
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const uint2 u = reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(a.router) + (size_t) nexp * FL_N)[c * 64 + l2];
                wg[c] = make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                                    __uint_as_float(u.y & 0xffff0000u));
            }
        } else {
#pragma unroll
            for (int c = 0; c < 8; ++c) wg[c] = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(a.router) + (size_t) nexp * FL_N)[c * 64 + l2];
        }
        const float v = router_dot(wg, xr);
        if (lane == 0) {
            S.gate = sigmoid_f(v);
            if (g == 0) a.logits[(size_t) t * LS + nexp] = v;
        }
    }
    // The row's h rows: wave 0 waits for the row's blocks that make them. A wave's loads return in order, so it asks for its
    // own first trips' weights only afterwards: the count it waits for is then not queued behind them. The other waves'
    // first trips are on their way while the row's last blocks finish their sweeps.
    auto first_trips = [&] {
#pragma unroll
        for (int i = 0; i < NB; ++i)
            if (trip_of(i) <= topk) issue_trip(B[i], trip_of(i));
    };
    if (dwave && wave != 0) first_trips();
    if (wave == 0) {
        const bool ok = win_wait_lines(&srow[1], win_lines(Tl), (unsigned) pl.nbi, a.wait_ticks, serr);
        if (lane == 0) __hip_atomic_store(&S.hready, ok ? 1 : -1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (dwave) first_trips();
    }
    if (!lds_wait([&] { return uniform(__hip_atomic_load(&S.hready, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP)) != 0; })) return false;
    if (uniform(__hip_atomic_load(&S.hready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) < 0) return false;
    WIN_TS(8);
    {   // the row's pairs' h rows into LDS, a pick's words side by side; the shared expert's are index topk
        constexpr int HQ_PER = SBR * HQ_WORDS, HQ_VPT = ((FL_MAXK + 1) * HQ_PER + WN_THREADS - 1) / WN_THREADS;
        uint32_t hw[HQ_VPT];
#pragma unroll
        for (int q = 0; q < HQ_VPT; ++q) {
            const int i = tid + q * WN_THREADS, k = i / HQ_PER;
            const bool has = k < topk || (k == topk && !ext);
            hw[q] = has ? __hip_atomic_load(&a.hq[(size_t) (k < topk ? t * topk + k : P + t) * HQ_PER + (i - k * HQ_PER)], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
        }
#pragma unroll
        for (int q = 0; q < HQ_VPT; ++q) {
            const int i = tid + q * WN_THREADS;
            if (i < (topk + 1) * HQ_PER) (&S.hq[0][0][0])[i] = hw[q];
        }
    }
    win_meet();
    WIN_TS(9);
    if (dwave) {
        auto pick_of = [&](int trip) { return trip == 0 ? topk : trip - 1; };   // the index of a trip's expert in S.hq
        float acc[RR], zs[RR];
#pragma unroll
        for (int r = 0; r < RR; ++r) acc[r] = zs[r] = 0.f;
        const float gate = S.gate;
        // a trip's sums of this wave's units' rows (every lane of a row's group holds the row's)
        auto trip_rows = [&](const PackedSub(&buf)[RR], int trip, auto after_h, auto sink) {
            const int k = pick_of(trip);
            const uint32_t* hb = S.hq[k][kb];
            const uint4 lo = *reinterpret_cast<const uint4*>(hb), hi = *reinterpret_cast<const uint4*>(hb + 4);
            const int hx[8] = {(int) lo.x, (int) lo.y, (int) lo.z, (int) lo.w, (int) hi.x, (int) hi.y, (int) hi.z, (int) hi.w};
            const float dh = __uint_as_float(hb[8]);
            after_h();
#pragma unroll
            for (int r = 0; r < RR; ++r) {
                int w4[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) w4[j] = *reinterpret_cast<const int*>(reinterpret_cast<const uint8_t*>(S.tab) + packed_addr(buf[r].idx, j));
                const int sc = 1 + 2 * (int) ((buf[r].sc >> sc_shift) & 0xFu);
                const float dw = half_bits_to_float(buf[r].d);
                int sum = 0;
#pragma unroll
                for (int j = 0; j < 8; ++j) sum = __builtin_amdgcn_sdot4(w4[j], hx[j], sum, false);
                sink(r, butterfly_sum<SBR>((dw * dh) * (float) __mul24(sum, sc)));
            }
        };
        auto decode_trip = [&](const PackedSub(&buf)[RR], int trip) {
            switch ((wave >> 2) + trip & 3) {   // every wave takes each of the four priorities in turn (see the sweeps)
                case 0: __builtin_amdgcn_s_setprio(0); break;
                case 1: __builtin_amdgcn_s_setprio(1); break;
                case 2: __builtin_amdgcn_s_setprio(2); break;
                default: __builtin_amdgcn_s_setprio(3); break;
            }
            float gk;
            trip_rows(
                buf, trip, [&] { gk = trip == 0 ? gate : S.pw[trip - 1]; },
                [&](int r, float z) {
                    if (trip == 0) zs[r] = gk * z;
                    else acc[r] = fmaf(gk, z, acc[r]);
                });
        };
        if constexpr (RR == 1) {
            if (TG > 1) {   // (the same for the whole block)
                constexpr int MAXI = (FL_MAXK + 2) / 2;   // trips a wave at most (TG >= 2)
#pragma unroll
                for (int i = 0; i < MAXI; ++i) {
                    const int trip = trip_of(i);
                    if (trip <= topk) {
                        trip_rows(
                            B[i % NB], trip, [] {},
                            [&](int, float z) {
                                if (kb == SBR - 1) S.zx[trip][uw][gl] = z;
                            });
                        if (trip_of(i + NB) <= topk) issue_trip(B[i % NB], trip_of(i + NB));
                    }
                }
                win_meet();
                if (tgrp == 0 && kb == SBR - 1) {
                    float s = 0.f, shared = 0.f;
                    for (int trip = first; trip <= topk; ++trip) {
                        const float zt = S.zx[trip][uw][gl], gk = trip == 0 ? gate : S.pw[trip - 1];
                        if (trip == 0) shared = gk * zt;
                        else s = fmaf(gk, zt, s);
                    }
                    if (ext) shared = gate * a.sh_part[(size_t) t * a.rows + (size_t) u0 * RW + gl];
                    __hip_atomic_store(reinterpret_cast<unsigned*>(a.out + (size_t) t * a.rows + (size_t) u0 * RW + gl), __float_as_uint(s + shared), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                }
                return true;
            }
        }
        // A trip's loads go to the buffer that held trip nx - NB, decoded before this one. The rounds in which every trip exists
        // and so does the one it asks for come first, without a condition on a load (see above); the last trips follow with them.
        int trip = first;
        if (topk + 1 - first >= NB + DEPTH) {
#pragma unroll
            for (int i = 0; i < NB; ++i) {   // the first round: its own buffers came before the wait for h
                decode_trip(B[i], first + i);
                if (i + DEPTH >= NB) issue_trip(B[(i + DEPTH) % NB], first + i + DEPTH);
            }
            for (trip = first + NB; trip + NB - 1 + DEPTH <= topk; trip += NB) {
#pragma unroll
                for (int i = 0; i < NB; ++i) {
                    decode_trip(B[i], trip + i);
                    issue_trip(B[(i + DEPTH) % NB], trip + i + DEPTH);
                }
            }
        }
        for (; trip <= topk; trip += NB) {
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const int tr = trip + i;
                if (tr > topk) break;
                decode_trip(B[i], tr);
                const int nx = tr + DEPTH;
                if (nx >= first + NB && nx <= topk) issue_trip(B[(i + DEPTH) % NB], nx);
            }
        }
        __builtin_amdgcn_s_setprio(0);
        if (kb == SBR - 1) {   // the combine's last step: s + sigmoid * shared
            float* orow = a.out + (size_t) t * a.rows + (size_t) u0 * RW + gl;
#pragma unroll
            for (int r = 0; r < RR; ++r) {
                    const float shared = ext ? gate * a.sh_part[(size_t) t * a.rows + (size_t) (u0 + r) * RW + gl] : zs[r];
                    // (at the device's level: the row's last block may read the row back below, from another XCD)
                    __hip_atomic_store(reinterpret_cast<unsigned*>(orow + r * RW), __float_as_uint(acc[r] + shared), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
        }
    }
    return true;
    };
    {
        bool ok;
        if (R == RMAX) ok = down_phase(std::integral_constant<int, RMAX>{});
        else if (RMAX > 2 && R == 2) ok = down_phase(std::integral_constant<int, (RMAX > 2 ? 2 : 1)>{});
        else ok = down_phase(std::integral_constant<int, 1>{});
        if (!ok) return;
    }
    win_stores_done();
    // rows past the ones that count get no window's rows added, but whatever follows still reads their normed rows: block g of
    // row 0 makes row Tl + g's (nothing else in this launch touches those rows; G >= 16 >= T - Tl)
    if (DEC && a.next_x && t == 0 && Tl + g < T) win_next_row(a, Tl + g, false, reinterpret_cast<float*>(&S.hgu[0][0]));

    WIN_TS(10);
    // ---------------------------------------------------------------- the end of the block, of the row, of the window
    // The last block of a row to get here puts the row's counters back; it takes the row's ticket among the finished
    // rows: the first row to finish writes the job lists the operator API promises the caller (kernels.hpp:18-23, 277-282;
    // nothing in this launch reads them), the last one puts the window's counters back.
    __syncthreads();
    if (tid == 0) {
        const unsigned done = __hip_atomic_fetch_add(&srow[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (done == (unsigned) pl.G - 1) {
            for (int l = 0; l < win_lines(Tl); ++l) __hip_atomic_store(&srow[l * WS_ROW_STRIDE + 1], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&srow[2], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            S.fin = (int) __hip_atomic_fetch_add(&a.sync[WS_FIN], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            S.last = 1;
        }
    }
    __syncthreads();
    WIN_TS(11);
    if (!S.last) return;
    // the row is complete (every block of it waited for its stores before it counted itself done); its logits' words, which
    // every block of the row has long read, go back to "not written"
    // (by the block's upper half: the lower one's first waves make the row's pass below, whose loads would wait behind these stores)
    for (int i = tid - WN_THREADS / 2; i >= 0 && i < nexp; i += WN_THREADS / 2) __hip_atomic_store(&lx[i], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (DEC && a.next_x) win_next_row(a, t, true, reinterpret_cast<float*>(&S.hgu[0][0]));
    const int fin = S.fin;
    // (A decoder's layer has no caller for the job lists - nothing reads them - and a window of few rows would end with them:
    // there the count of ranked rows is put back by the last row to finish, by when every row has counted itself.)
    if (DEC && a.next_x) {
        if (fin == Tl - 1 && tid == 0) {
            __hip_atomic_store(&a.sync[WS_ROUTED], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&a.sync[WS_FIN], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        WIN_TS(12);
        return;
    }
    if (fin == 0) {   // every row has been ranked long ago; the count says so
        if (wave == 0) {
            const bool ok = win_wait_word(&a.sync[WS_ROUTED], (unsigned) Tl, a.wait_ticks, serr);
            if (lane == 0) {
                S.lists = ok ? 1 : -1;
                if (ok) __hip_atomic_store(&a.sync[WS_ROUTED], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        __syncthreads();
        if (S.lists == 1) {
            const RouteArgs route{nexp, topk, T, a.logits, a.topi, a.topw, a.jobs_gu, a.jobs_dn, a.njobs, a.live};
            write_job_lists<WN_THREADS>(*reinterpret_cast<RouteLds<WN_THREADS>*>(S.tab), route, Tl);
        }
    }
    if (fin == Tl - 1 && tid == 0) __hip_atomic_store(&a.sync[WS_FIN], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    WIN_TS(12);
}

}  // namespace fnx
