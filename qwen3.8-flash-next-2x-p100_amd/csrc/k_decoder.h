// The pieces a whole verify step needs around the MoE half: RMS norm, the dense Q8_0 (split layout) mat-vec of the
// projections and the output head, the attention's prepare/append and split-K decode kernels, embedding rows.
#pragma once

#include "attn_window.h"

#include "fnx_device.h"

namespace fnx {

constexpr int AT_HD = 256, AT_NROT = 64;   // head width and rotated dims (model.hpp:41 of the reference)
typedef unsigned at_v4u_t __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------- RMS norm (kernels.cu:2818-2826)
// y[r] = x[r] / sqrt(mean(x[r]^2) + eps) * w, a block per row
__global__ void __launch_bounds__(256) k_rms_norm_rows(const float* __restrict__ x, const float* __restrict__ w, float* __restrict__ y, int n,
                                                      float eps) {
    __shared__ float sh[4];
    const float* xr = x + (size_t) blockIdx.x * n;
    float s = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) s = fmaf(xr[i], xr[i], s);
    s = group_sum<64>(s);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = s;
    __syncthreads();
    const float r = rsqrtf((sh[0] + sh[1] + sh[2] + sh[3]) / (float) n + eps);
    for (int i = threadIdx.x; i < n; i += 256) y[(size_t) blockIdx.x * n + i] = xr[i] * r * w[i];
}
// x[r] += add[r] (add may be null); xn[r] = rms_norm(x[r]) * w; xq[r] = q8_1(xn[r]) (either may be null): the residual add,
// the norm and the quantisation that follow one another between a layer's halves, in one pass over the row. The sums
// run in k_rms_norm_rows' and k_quantize_q8_1's orders, so the results are theirs bit for bit.
// With c.part set, what is added is the MoE half's combine (k_combine's chain, kernels.cu:412-419) of the partial sums,
// made here instead of being written out and read back by a launch of its own.
constexpr int NQ_MAXJ = 16;   // rows of up to 4096 values
struct CombineArgs {
    const float* part;   // null: no combine
    const float* topw;
    const float* sh;
    const float* sh_logit;
    int sh_logit_stride, topk;
    float* xcopy;        // may be null: the rows after the add go there as well (the hidden rows the draft layer starts from)
    const uint16_t* emb;  // may be null: the rows do not come from x but are rows tokens[r] of this f16 table (and go to x)
    const int* tokens;
    int vocab;
    const int* live;      // may be null; else a device word: rows from *live on were not routed and get no combine added
    const int* gate;      // may be null; else a device word: at zero the launch leaves at once (a chain step that does not count)
    // A second pass in the same launch (the narrow form; rows2 > 0): blocks from rows1 on are rows 0 .. rows2 - 1 of a pass over
    // x2 with the weights w2, into xq2, their rows from the table if emb2 is set (the draft layer's two inputs, each with a
    // norm of its own, are one launch this way)
    int rows1, rows2;
    float* x2;
    const float* w2;
    uint8_t* xq2;
    const uint16_t* emb2;
};
// WIDE (the combine's form): 1024 threads make the row after the add - a thread the columns p, p + 1024, ..., with all
// of an expert batch's partial sums in flight (256 threads with 8 columns each took 13 us a call, against 7 us without
// the combine) - and hand it over in LDS to the first 256, which go on as in the narrow form: the same values and orders.
template <bool WIDE>
__global__ void __launch_bounds__(WIDE ? 1024 : 256) k_add_norm_q8(float* __restrict__ x, const float* __restrict__ add, const CombineArgs c,
                                                                  const float* __restrict__ w, float* __restrict__ xn, uint8_t* __restrict__ xq, int n,
                                                                  float eps) {
    __shared__ float sh[4];
    __shared__ float vrow[WIDE ? 256 * NQ_MAXJ : 1];
    if (c.gate && uniform(*c.gate) == 0) return;
    size_t row = blockIdx.x;
    const uint16_t* emb = c.emb;
    if (!WIDE && c.rows2 > 0 && (int) blockIdx.x >= c.rows1) {   // the launch's second pass
        row = blockIdx.x - c.rows1;
        x = c.x2, w = c.w2, xq = c.xq2, emb = c.emb2;
        xn = nullptr, add = nullptr;
    }
    float v[NQ_MAXJ];
    float s = 0.f;
    if constexpr (WIDE) {
        // the combine's chains (k_combine's order: the picks ascending), NQ_KB experts' partial sums of this thread's
        // columns in flight at a time (one by one, each load would be a trip to the cache of its own)
        constexpr int NQ_KB = 5, NQ_WJ = NQ_MAXJ / 4;
        float m[NQ_WJ];
#pragma unroll
        for (int j = 0; j < NQ_WJ; ++j) m[j] = 0.f;
        const bool routed = !c.live || (int) row < *c.live;
        const int topk = routed ? c.topk : 0;
        for (int k0 = 0; k0 < topk; k0 += NQ_KB) {
            float pv[NQ_KB][NQ_WJ], wk[NQ_KB];
#pragma unroll
            for (int kk = 0; kk < NQ_KB; ++kk) {
                const int k = min(k0 + kk, topk - 1);
                wk[kk] = c.topw[row * c.topk + k];
#pragma unroll
                for (int j = 0; j < NQ_WJ; ++j) {
                    const int i = threadIdx.x + 1024 * j;
                    pv[kk][j] = i < n ? c.part[(row * c.topk + k) * n + i] : 0.f;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kk = 0; kk < NQ_KB; ++kk)
                if (k0 + kk < topk) {
#pragma unroll
                    for (int j = 0; j < NQ_WJ; ++j) m[j] = fmaf(wk[kk], pv[kk][j], m[j]);
                }
        }
        const float sg = sigmoid_f(c.sh_logit[row * c.sh_logit_stride]);
        float xv[NQ_WJ], shv[NQ_WJ];
#pragma unroll
        for (int j = 0; j < NQ_WJ; ++j) {
            const int i = threadIdx.x + 1024 * j;
            xv[j] = i < n ? x[row * n + i] : 0.f;
            shv[j] = i < n ? c.sh[row * n + i] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < NQ_WJ; ++j) {
            const int i = threadIdx.x + 1024 * j;
            const float r = routed ? xv[j] + (m[j] + sg * shv[j]) : xv[j];
            vrow[i] = i < n ? r : 0.f;
            if (i < n) {
                x[row * n + i] = r;
                if (c.xcopy) c.xcopy[row * n + i] = r;
            }
        }
        __syncthreads();
        if (threadIdx.x >= 256) return;
#pragma unroll
        for (int j = 0; j < NQ_MAXJ; ++j) v[j] = vrow[threadIdx.x + 256 * j];
    } else {
        // all loads first: a store to x between them would keep the next load waiting for it
        float av[NQ_MAXJ];
        const size_t erow = emb ? (size_t) min(max(c.tokens[row], 0), c.vocab - 1) : 0;   // k_embed_rows' clamp
#pragma unroll
        for (int j = 0; j < NQ_MAXJ; ++j) {
            const int i = threadIdx.x + 256 * j;
            if (emb) v[j] = i < n ? half_bits_to_float(emb[erow * n + i]) : 0.f;
            else v[j] = i < n ? x[row * n + i] : 0.f;
            av[j] = add && i < n ? add[row * n + i] : 0.f;
        }
        if (add && (!c.live || (int) row < *c.live)) {
#pragma unroll
            for (int j = 0; j < NQ_MAXJ; ++j) v[j] += av[j];
        }
    }
    float wv[NQ_MAXJ];   // the norm's weights too, before any store
#pragma unroll
    for (int j = 0; j < NQ_MAXJ; ++j) {
        const int i = threadIdx.x + 256 * j;
        wv[j] = i < n ? w[i] : 0.f;
    }
    if (!WIDE && (add || emb)) {
#pragma unroll
        for (int j = 0; j < NQ_MAXJ; ++j) {
            const int i = threadIdx.x + 256 * j;
            if (i < n) x[row * n + i] = v[j];
        }
    }
    if (!WIDE && c.xcopy) {
#pragma unroll
        for (int j = 0; j < NQ_MAXJ; ++j) {
            const int i = threadIdx.x + 256 * j;
            if (i < n) c.xcopy[row * n + i] = v[j];
        }
    }
#pragma unroll
    for (int j = 0; j < NQ_MAXJ; ++j) s = fmaf(v[j], v[j], s);   // columns past n hold zeros
    s = group_sum<64>(s);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = s;
    __syncthreads();
    const float r = rsqrtf((sh[0] + sh[1] + sh[2] + sh[3]) / (float) n + eps);
#pragma unroll
    for (int j = 0; j < NQ_MAXJ; ++j) {
        const int i = threadIdx.x + 256 * j;
        if (i < n) {   // n is a multiple of 32: the 32 threads of a q8_1 block are live together
            const float y = v[j] * r * wv[j];
            if (xn) xn[row * n + i] = y;
            if (xq) q8_1_store(y, xq + (row * (n / 32) + i / 32) * FNX_Q8_1_BLOCK, threadIdx.x & 31);
        }
    }
}
__global__ void k_add_rows(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ y, size_t n) {
    for (size_t i = blockIdx.x * (size_t) blockDim.x + threadIdx.x; i < n; i += (size_t) gridDim.x * blockDim.x) y[i] = a[i] + b[i];
}
// rows of an f16 table as f32
__global__ void k_embed_rows(const uint16_t* __restrict__ emb, const int* __restrict__ tokens, int vocab, int n, float* __restrict__ y) {
    const int t = blockIdx.x, tok = min(max(tokens[t], 0), vocab - 1);
    for (int i = threadIdx.x; i < n; i += blockDim.x) y[(size_t) t * n + i] = half_bits_to_float(emb[(size_t) tok * n + i]);
}

// ---------------------------------------------------------------- dense Q8_0, split layout (dense.cuh:79-214)
// int8 values [rows][cols], f16 scales [rows][cols / 32]; activations q8_1 (up to 16 rows). The result is defined as
//   out[t][r] = (s0 + s1) + (s2 + s3),  s_q = fold over the 32-column blocks b of the q-th quarter of the columns, in
//               ascending order, of acc = fmaf(d_w[r][b] * d_x[t][b], (float) dot_b, acc)
// (dot_b the exact integer dot product of the block): the reference's term (dense.cuh:196-200) in one fixed order, which
// the CPU oracle follows bit for bit.
// On the matrix cores: a block owns 16 weight rows, each of its four waves a quarter of the columns (so that a matrix
// of a few hundred rows still fills the chip and a wave's chain of dependent loads is short). v_mfma_i32_16x16x32_i8
// wants 8 bytes of k from each of 4 lane groups. A lane loads 16 contiguous bytes of its row per 64 columns (group g:
// bytes 16 g ..), so groups 0-1 hold block 2 j and groups 2-3 block 2 j + 1; each block's dot product is two MFMAs (the
// lanes' low and high 8 bytes) whose B operand is zero in the other block's groups. The 16 x 16 integer sums then take
// their scales in 12 VALU ops, against 44 for the same block on the vector ALU, and no cross-lane reduction is left.
constexpr int Q8S_WAVES = 4, Q8S_XPAD = 16, Q8S_BATCH = 4;   // double steps (64 columns) loaded at once
// The tile-major layout of the int8 values (made once at load, k_q8s_tile): the matrix in tiles of 16 rows (the last one
// padded with zero rows), a tile its 64-column steps one after another, a step 1 KiB: lane (r, g) of the wave that takes it
// - row r of the tile, columns 16 g .. 16 g + 15 of the step - finds its 16 bytes at 16 (r + 16 g). The scales stay
// [rows][cols / 32].
constexpr int Q8S_TILE_STEP = 1024;
__global__ void __launch_bounds__(256) k_q8s_tile(const int8_t* __restrict__ src, int8_t* __restrict__ dst, int rows, int cols) {
    // a thread a 16-byte piece: piece p of the output, in output order
    const size_t pieces = (size_t) ((rows + 15) / 16) * 16 * (cols / 16);
    for (size_t p = (size_t) blockIdx.x * blockDim.x + threadIdx.x; p < pieces; p += (size_t) gridDim.x * blockDim.x) {
        const size_t step = p / 64;   // (tile, 64-column step)
        const int l = (int) (p - step * 64), r = l & 15, g = l >> 4;
        const size_t tile = step / (cols / 64), j = step - tile * (cols / 64);
        const size_t row = tile * 16 + r;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (row < (size_t) rows) v = *reinterpret_cast<const uint4*>(src + row * cols + 64 * j + 16 * g);
        *reinterpret_cast<uint4*>(dst + p * 16) = v;
    }
}
struct Q8sSeg {
    const int8_t* q;
    const uint16_t* d;
    float* out;
    int rows, out_stride;
};
struct Q8sArgs {
    Q8sSeg seg[3];       // up to three matrices over the same activations, their 16-row tiles one after another
    int nseg, cols, T;
    const uint8_t* yq;   // q8_1 rows
    const int* gate;     // may be null; else a device word: at zero the launch leaves at once (a chain step that does not count)
    const uint8_t* yq2;  // may be null; else the second matrix's rows are these (two matrices, a block a tile: the host sees to that)
    const int* live;     // may be null; else a device word: rows from *live on do not count - they are not read and their products are zeros
};
typedef int q8s_v4i __attribute__((ext_vector_type(4)));
// DEPTH: the (tile, batch) items whose loads are in flight ahead of the one being worked on. (With 3 - all of a tile's
// batches on their way before the activations are staged - a matrix of a few thousand rows was not faster: its launch is
// the block's start, the staging of the activations and the first pass through the code, not the weights' round trips.)
// TILED: the int8 values in the tile-major layout of k_q8s_tile below (every matrix of the launch): a wave's load is then
// 1 KiB in a row - eight whole cache lines instead of half a line of each of sixteen rows - and takes the streaming policy
// (read once). 4.7 against 4.1 TB/s for the output head; with the policy alone, over rows, 3.9.
// LIVE: a.live is set (a launch of its own: the word is then read on every path, through the scalar unit, and waiting for it
// does not wait for the weights on their way).
template <int DEPTH, bool TILED = false, bool LIVE = false>
__global__ void __launch_bounds__(Q8S_WAVES * 64) k_q8s_gemv(const Q8sArgs a) {
    typedef __attribute__((address_space(1))) const at_v4u_t g128;
    extern __shared__ __align__(16) uint8_t q8s_lds[];   // [16][cols + pad] int8, [16][nb + 2] f32 scales, [3][64][4] partial sums
    if (a.gate && uniform(*a.gate) == 0) return;
    const int nb = a.cols >> 5, T = a.T, xld = a.cols + Q8S_XPAD, dld = nb + 2;
    int8_t* xs = reinterpret_cast<int8_t*>(q8s_lds);
    float* xd = reinterpret_cast<float*>(q8s_lds + (size_t) FNX_MAXT * xld);
    float* part = xd + FNX_MAXT * dld;
    const int lane = threadIdx.x & 63, wave = uniform(threadIdx.x >> 6), r16 = lane & 15, g = lane >> 4;
    const int t0 = (a.seg[0].rows + 15) / 16, t1 = t0 + (a.nseg > 1 ? (a.seg[1].rows + 15) / 16 : 0),
              tiles = t1 + (a.nseg > 2 ? (a.seg[2].rows + 15) / 16 : 0);
    const int nq4 = a.cols >> 8;   // double steps per wave: a quarter of cols / 64
    const bool lo_groups = g < 2;
    const int j0 = wave * nq4;     // this wave's first double step
    struct Tile {
        gbytes wrow, drow[4];
        float* out;
        int rows, row0;
    };
    auto tile_of = [&](int tile) {
        const int si = tile < t0 ? 0 : tile < t1 ? 1 : 2;
        const int8_t* sq = si == 0 ? a.seg[0].q : si == 1 ? a.seg[1].q : a.seg[2].q;
        const uint16_t* sd = si == 0 ? a.seg[0].d : si == 1 ? a.seg[1].d : a.seg[2].d;
        float* sout = si == 0 ? a.seg[0].out : si == 1 ? a.seg[1].out : a.seg[2].out;
        const int sstride = si == 0 ? a.seg[0].out_stride : si == 1 ? a.seg[1].out_stride : a.seg[2].out_stride;
        Tile c;
        c.rows = si == 0 ? a.seg[0].rows : si == 1 ? a.seg[1].rows : a.seg[2].rows;
        c.row0 = (tile - (si == 0 ? 0 : si == 1 ? t0 : t1)) * 16;
        if constexpr (TILED) c.wrow = as_global(reinterpret_cast<const uint8_t*>(sq) + (size_t) c.row0 * a.cols + 16 * lane + Q8S_TILE_STEP * j0);
        else c.wrow = as_global(reinterpret_cast<const uint8_t*>(sq) + (size_t) min(c.row0 + r16, c.rows - 1) * a.cols + 16 * g + 64 * j0);
        // the scales of the accumulator's rows 4 g .. 4 g + 3, from this wave's first block on
#pragma unroll
        for (int r = 0; r < 4; ++r)
            c.drow[r] = as_global(reinterpret_cast<const uint8_t*>(sd + (size_t) min(c.row0 + 4 * g + r, c.rows - 1) * nb + 2 * j0));
        c.out = sout + (size_t) r16 * sstride + c.row0 + 4 * g;   // accumulator lane (g, token r16): rows row0 + 4 g + r
        return c;
    };
    struct Batch {
        at_v4u_t w[Q8S_BATCH];
        at_v4u_t dd[4];   // per accumulator row: the scale pairs of the batch's double steps
    };
    static_assert(Q8S_BATCH == 4, "a row's scales of one batch are one 16-byte load");
    auto load = [&](const Tile& c, int jb, Batch& o) {   // nq4 is 1, 2 or a multiple of 4 (cols a multiple of 256)
        const int nstep = min(Q8S_BATCH, nq4 - jb);
#pragma unroll
        for (int u = 0; u < Q8S_BATCH; ++u) {
            if constexpr (TILED) o.w[u] = __builtin_nontemporal_load((g128*) (c.wrow + Q8S_TILE_STEP * (jb + min(u, nstep - 1))));
            else o.w[u] = *(g128*) (c.wrow + 64 * (jb + min(u, nstep - 1)));
        }
        if (nq4 >= Q8S_BATCH) {
#pragma unroll
            for (int r = 0; r < 4; ++r) o.dd[r] = *(g128*) (c.drow[r] + 4 * jb);
        } else {
#pragma unroll
            for (int u = 0; u < Q8S_BATCH; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r) o.dd[r][u] = *(const __attribute__((address_space(1))) uint32_t*) (c.drow[r] + 4 * min(u, nstep - 1));
        }
    };
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    auto compute = [&](int jb, const Batch& in) {
        const int nstep = min(Q8S_BATCH, nq4 - jb);
#pragma unroll
        for (int u = 0; u < Q8S_BATCH; ++u)
            if (u < nstep) {
                const int j = j0 + jb + u;
                const at_v4u_t x = *reinterpret_cast<const at_v4u_t*>(xs + (size_t) r16 * xld + 64 * j + 16 * g);
                const float2 dx = *reinterpret_cast<const float2*>(xd + r16 * dld + 2 * j);
                const long wl = (long) in.w[u].x | (long) in.w[u].y << 32, wh = (long) in.w[u].z | (long) in.w[u].w << 32;
                const long xl = (long) x.x | (long) x.y << 32, xh = (long) x.z | (long) x.w << 32;
                const long xl0 = lo_groups ? xl : 0, xh0 = lo_groups ? xh : 0, xl1 = lo_groups ? 0 : xl, xh1 = lo_groups ? 0 : xh;
                q8s_v4i s0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(wl, xl0, q8s_v4i{0, 0, 0, 0}, 0, 0, 0);
                s0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(wh, xh0, s0, 0, 0, 0);
                q8s_v4i s1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(wl, xl1, q8s_v4i{0, 0, 0, 0}, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(wh, xh1, s1, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    acc[r] = fmaf(half_bits_to_float(in.dd[r][u] & 0xFFFFu) * dx.x, (float) s0[r], acc[r]);
                    acc[r] = fmaf(half_bits_to_float(in.dd[r][u] >> 16) * dx.y, (float) s1[r], acc[r]);
                }
            }
    };
    auto finish = [&](const Tile& c) {   // the four quarters through LDS: (s0 + s1) + (s2 + s3)
        __syncthreads();   // the previous tile's sums have been read
        if (wave) *reinterpret_cast<float4*>(part + ((wave - 1) * 64 + lane) * 4) = make_float4(acc[0], acc[1], acc[2], acc[3]);
        __syncthreads();
        if (wave == 0 && r16 < T) {   // the first quarter's sums never leave its wave (and the block fits a CU four times)
            const float4 p0 = make_float4(acc[0], acc[1], acc[2], acc[3]), p1 = *reinterpret_cast<const float4*>(part + lane * 4),
                         p2 = *reinterpret_cast<const float4*>(part + (64 + lane) * 4), p3 = *reinterpret_cast<const float4*>(part + (128 + lane) * 4);
            const float v[4] = {(p0.x + p1.x) + (p2.x + p3.x), (p0.y + p1.y) + (p2.y + p3.y), (p0.z + p1.z) + (p2.z + p3.z),
                                (p0.w + p1.w) + (p2.w + p3.w)};
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (c.row0 + 4 * g + r < c.rows) c.out[r] = v[r];
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] = 0.f;
    };
    // The (tile, batch) items of this block in one sequence: the loads of the items ahead - the next tiles' first ones
    // too - are in flight while the current one is worked on and while a tile's quarters are summed.
    if ((int) blockIdx.x >= tiles) return;   // the same for every thread of the block
    struct Cursor {
        int tile, jb;
        bool valid;
        Tile t;
    };
    auto advance = [&](Cursor& c) {
        c.jb += Q8S_BATCH;
        if (c.jb >= nq4) {
            c.jb = 0;
            c.tile += gridDim.x;
            c.valid = c.tile < tiles;
            if (c.valid) c.t = tile_of(c.tile);
        }
    };
    Cursor lc{(int) blockIdx.x, 0, true, tile_of(blockIdx.x)}, cc = lc;   // the loads' place and the arithmetic's
    Batch ring[DEPTH + 1];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
        if (lc.valid) {
            load(lc.t, lc.jb, ring[d]);
            advance(lc);
        }
    // the window's q8_1 rows into LDS (the first weights are on their way meanwhile). The copy takes 3 us (6-7 us in a
    // launch of 1,024 blocks, beside their weight loads) whatever the width of its loads - nine 16-byte loads for four
    // blocks of a row were no faster than 4-byte ones - and wherever in the rows a block starts.
    int Tl = T;   // (a window of a decode round: most of its sixteen rows do not count)
    if constexpr (LIVE) Tl = max(1, min(*a.live, T));
    for (int i = threadIdx.x; i < FNX_MAXT * nb; i += blockDim.x) {
        const int t = i / nb, b = i - t * nb;
        uint32_t* dst = reinterpret_cast<uint32_t*>(xs + (size_t) t * xld + 32 * b);
        if (t < Tl) {
            const uint8_t* blk = (a.yq2 && (int) blockIdx.x >= t0 ? a.yq2 : a.yq) + (size_t) i * 36;
            xd[t * dld + b] = half_bits_to_float(load_u16(blk));
            const uint32_t* src = reinterpret_cast<const uint32_t*>(blk + 4);
#pragma unroll
            for (int k = 0; k < 8; ++k) dst[k] = src[k];
        } else {   // rows past the window: zeros, so their lanes' products stay finite
            xd[t * dld + b] = 0.f;
#pragma unroll
            for (int k = 0; k < 8; ++k) dst[k] = 0u;
        }
    }
    __syncthreads();
    while (cc.valid) {
#pragma unroll
        for (int slot = 0; slot <= DEPTH; ++slot) {
            if (!cc.valid) break;
            if (lc.valid) {
                load(lc.t, lc.jb, ring[(slot + DEPTH) % (DEPTH + 1)]);
                advance(lc);
            }
            compute(cc.jb, ring[slot]);
            if (cc.jb + Q8S_BATCH >= nq4) finish(cc.t);
            advance(cc);
        }
    }
}

// ---------------------------------------------------------------- attention: prepare and append (kernels.cu:513-537, 1878-1910)
// the 32 pairs' unit frequencies (rope.hpp:33-39) come from the host: an angle reaches 3e4 radians at long contexts, where
// one ulp of the frequency moves sin and cos by 1e-3, so the powf must be one and the same everywhere
struct RopeDev {
    float freq[AT_NROT / 2];
    float mscale;
};
__device__ __forceinline__ size_t vcache_at(int pos, int nkv, int kvh, int d) {   // the V cache's element index
    return (((size_t) (pos / AT_VB) * nkv + kvh) * AT_HD + d) * AT_VB + (pos % AT_VB);
}
// block (head h, row t), AT_HD threads: q heads normed and rotated in place; k heads normed, rotated and appended; v heads
// appended. The K cache is [position][kv head][AT_HD] f16; the V cache keeps eight positions of a dimension together,
// [position / 8][kv head][AT_HD][position % 8]: 16 bytes, the matrix-core attention's V operand of one lane.
__global__ void __launch_bounds__(AT_HD) k_attn_prep_append(float* __restrict__ qg, float* __restrict__ k, const float* __restrict__ v,
                                                           const float* __restrict__ qn, const float* __restrict__ kn,
                                                           uint16_t* __restrict__ kc, uint16_t* __restrict__ vc, int nq, int nkv,
                                                           const int* __restrict__ pos0p, int max_ctx, float eps, RopeDev rope,
                                                           const int* __restrict__ gate) {
    __shared__ float sh[AT_HD / 64];
    __shared__ float xs[AT_HD];
    if (gate && uniform(*gate) == 0) return;   // a chain step that does not count appends nothing
    const int t = blockIdx.y, h = blockIdx.x, i = threadIdx.x, p = *pos0p + t;
    const bool is_q = h < nq, is_k = !is_q && h < nq + nkv;
    const int kh = h - nq - (is_k ? 0 : nkv);
    float x;
    if (is_q || is_k) {
        float* row = is_q ? qg + ((size_t) t * nq + h) * 2 * AT_HD : k + ((size_t) t * nkv + kh) * AT_HD;
        const float* w = is_q ? qn : kn;
        const float val = row[i];
        const float s = group_sum<64>(val * val);
        if ((i & 63) == 0) sh[i >> 6] = s;
        __syncthreads();
        const float ms = (sh[0] + sh[1] + sh[2] + sh[3]) / (float) AT_HD;
        xs[i] = val * rsqrtf(ms + eps) * w[i];
        __syncthreads();
        x = xs[i];
        if (i < AT_NROT) {
            const int pair = i & (AT_NROT / 2 - 1);
            const float theta = (float) p * rope.freq[pair];
            float sn, cs;
            sincosf(theta, &sn, &cs);
            sn *= rope.mscale;
            cs *= rope.mscale;
            const float x0 = xs[pair], x1 = xs[pair + AT_NROT / 2];
            x = i < AT_NROT / 2 ? x0 * cs - x1 * sn : x0 * sn + x1 * cs;
        }
        row[i] = x;
        if (is_q) return;
    } else {
        x = v[((size_t) t * nkv + kh) * AT_HD + i];
    }
    if (p < 0 || p >= max_ctx) return;
    if (is_k) kc[((size_t) p * nkv + kh) * AT_HD + i] = float_to_half_bits(x);
    else vc[vcache_at(p, nkv, kh, i)] = float_to_half_bits(x);
}

// ---------------------------------------------------------------- attention: split-K decode on the matrix cores
// (kernels.cu:541-643, 786-803 give the arithmetic: scores q.k / 16 over positions [0, pos0 + t], online softmax in
// splits, the splits merged by their maxima, the result times sigmoid(gate).)
//
// A window's rows times a kv head's q heads are up to 128 query vectors against the same K/V rows: a dense contraction,
// so it runs on v_mfma_f32_16x16x32_f16. A block takes (split of AT_SPLIT positions, kv head, half of the query tiles);
// a wave takes 16 queries (query = row * heads-per-kv + head). Per chunk of 32 positions:
//   S^T = K Q^T  : A = K rows (two tiles of 16 positions; row i of tile t is position 8 (i / 4) + 4 t + i % 4 of the chunk;
//                  a lane holds the 64 dims of lane group l / 16, 16 bytes a step), B = Q^T (held in registers for the
//                  whole split, scaled by 1/16, as two f16 terms hi + lo);
//                  the accumulator leaves lane (group pg, query q) with rows 4 pg .. 4 pg + 3 of both tiles, which with
//                  that order of the rows are positions 8 pg .. 8 pg + 7: the softmax of query q needs only in-lane work
//                  and two cross-group shuffles;
//   O^T += V^T P^T: those eight positions are exactly lane group pg's contraction slots, so P goes from the accumulator
//                  registers straight into the B operand, and V^T's A operand is one 16-byte read because the V cache
//                  keeps eight positions of a dimension together ([position / 8][kv head][dim][position % 8]).
// The probabilities never pass through LDS; K and V chunks do, once per block, loaded straight into it two chunks ahead.
// Each (query, split) leaves its maximum, sum and 256 accumulators; k_attn_combine merges.
constexpr int AT_MAXQ = 8;   // AT_SPLIT, AT_CH: attn_window.h
struct AttPart {
    float m, z;
};
typedef _Float16 at_v8h __attribute__((ext_vector_type(8)));
typedef _Float16 at_v4h __attribute__((ext_vector_type(4)));
typedef float at_v4f __attribute__((ext_vector_type(4)));
typedef unsigned at_v4u __attribute__((ext_vector_type(4)));
typedef unsigned at_v2u __attribute__((ext_vector_type(2)));


// maximum / sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (a query's four lane groups), left in all four: two row
// swaps each instead of two trips through the LDS crossbar. (Inline asm, with the wait states the swap needs after a
// vector write, as for the other uses of these swaps.)
__device__ __forceinline__ float groups4_max(float v) {
    float x = v, y = v;
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(x), "+v"(y));
    x = y = fmaxf(x, y);
    asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(x), "+v"(y));
    return fmaxf(x, y);
}
__device__ __forceinline__ float groups4_sum(float v) {
    float x = v, y = v;
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(x), "+v"(y));
    x = y = x + y;
    asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(x), "+v"(y));
    return x + y;
}
constexpr int AT_WAVES = 4;   // q tiles (of 16 queries) per block, blockIdx.z picks which
constexpr int AT_THREADS = (AT_WAVES + 1) * 64;   // and one wave more that only brings the K and V chunks in
__global__ void __launch_bounds__(AT_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) k_attn_part(const float* __restrict__ qg, const uint16_t* __restrict__ kc,
                                                            const uint16_t* __restrict__ vc, float* __restrict__ acc_out,
                                                            AttPart* __restrict__ mz_out, int nq, int nkv, int T, int nsplit,
                                                            const int* __restrict__ pos0p, int max_ctx, const int* __restrict__ gate,
                                                            const int* __restrict__ live) {
    // the launch's device words, asked for together (one after the other, each would be a trip to memory of its own)
    const int gate_v = gate ? *gate : 1, live_v = live ? *live : T, pos0_v = *pos0p;
    if (uniform(gate_v) == 0) return;   // a chain step that does not count: its parts stay what they were, nothing reads the result
    // live (may be null): a device word, the rows of the window that count; the others' queries are left out (nothing reads
    // their results), the positions past the last row that counts with them
    const int s = blockIdx.x, kvh = blockIdx.y, lane = threadIdx.x & 63;
    const bool loader = uniform((int) (threadIdx.x >> 6)) == AT_WAVES;   // the block's last wave: no queries, all the loads
    const int qpk = nq / nkv;
    T = uniform(max(1, min(live_v, T)));
    const int nquery = T * qpk;
    // a window of few queries: the grid's second layer of blocks takes the second halves of the splits (attn_window.h)
    const bool halves = att_halves(nquery);
    const int wave = (halves ? 0 : blockIdx.z * AT_WAVES) + (threadIdx.x >> 6);
    // this lane's query row, 64 of its dims: loaded before anything that waits for the window's position (a lane past the
    // window's queries reads the last query's row; its operands become zeros below)
    float4 qa[8], qb[8];
    if (!loader) {
        const int qc = min(wave * 16 + (lane & 15), T * qpk - 1);
        const float* qr = qg + ((size_t) (qc / qpk) * nq + kvh * qpk + qc % qpk) * 2 * AT_HD + 64 * (lane >> 4);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            qa[ks] = *reinterpret_cast<const float4*>(qr + 8 * ks);
            qb[ks] = *reinterpret_cast<const float4*>(qr + 8 * ks + 4);
        }
    }
    const AttWindow win = att_window(uniform(pos0_v), T, max_ctx);   // no index below leaves the cache, whatever the device word holds
    if (!halves && (int) blockIdx.z * AT_WAVES * 16 >= nquery) return;   // none of the block's queries count
    const bool wave_on = uniform(wave * 16 < nquery) && !loader;   // a wave without queries only meets the others
    const int ql = lane & 15, pg = lane >> 4;
    const int qi = wave * 16 + ql;                      // this lane's query (as B column / accumulator column)
    const bool qlive = qi < nquery && !loader;
    const int qt = qlive ? qi / qpk : 0, qh = kvh * qpk + (qlive ? qi % qpk : 0);
    const int ctx_q = qlive ? att_ctx_q(win, qt) : 0;   // positions [0, ctx_q) are this query's
    const int ctx_max = win.ctx_max;                    // the window's last row sees this many
    const int p0 = att_part_begin(s, blockIdx.z, halves), p1 = att_part_end(win, s, blockIdx.z, halves);
    const int vis = uniform(wave_on ? min(att_ctx_q(win, (wave * 16) / qpk), p1) : 0);   // the wave's first query is its earliest row's
    const size_t slot = ((size_t) qt * nq + qh) * att_part_stride(nsplit, halves) + att_part_index(s, blockIdx.z, halves);
    if (p0 >= p1) {   // a part past the context: empty
        if (qlive && pg == 0) mz_out[slot] = AttPart{-INFINITY, 0.f};
        return;
    }
    // A chunk's K rows (32 x 512 bytes) and V blocks (8 x 2048 bytes) go from the caches straight into LDS
    // (global_load_lds_dwordx4: a wave instruction lays its 64 lanes' 16-byte pieces down one after the other, 1 KiB from
    // a wave-uniform address), two chunks ahead of the one being multiplied, into one of three stages; no registers and
    // no stores of the block's own in between. 32 instructions a chunk, all issued by a wave of their own: the memory
    // pipe takes an instruction every 16 cycles or so, and a wave that multiplies would stand still for a sixth of a
    // chunk's time while its share is taken.
    //   K: an instruction carries two rows. The LDS takes the rows' pieces in lane order, so the bank spread that padding
    //      a row would give comes from which piece a lane loads: the second row of a pair holds piece c at place c ^ 2, and
    //      a pair starts 1040 bytes after the one before (the 16 rows that an operand read touches then start at 16
    //      different multiples of 16 bytes modulo 256).
    //   V: an instruction carries a quarter of a block (64 dims x eight positions), the layout the operands are read in.
    // (byte offsets in 32 bits: the host refuses caches of 4 GiB and more)
    constexpr int AT_STAGES = 3, AT_KPAIR = 2 * AT_HD * 2 + 16, AT_KSTAGE = (AT_CH / 2) * AT_KPAIR, AT_VBLK = AT_HD * AT_VB * 2, AT_VSTAGE = (AT_CH / AT_VB) * AT_VBLK;
    __shared__ __align__(16) uint8_t lk[AT_STAGES * AT_KSTAGE];
    __shared__ __align__(16) uint8_t lv[AT_STAGES * AT_VSTAGE];
    const uint32_t lk_at = (uint32_t) (size_t) (__attribute__((address_space(3))) uint8_t*) lk, lv_at = (uint32_t) (size_t) (__attribute__((address_space(3))) uint8_t*) lv;
    const uint32_t krowb = (uint32_t) nkv * (AT_HD * 2), vblkb = (uint32_t) nkv * AT_VBLK;   // bytes between two rows of K, two blocks of V
    const int kh = lane >> 5;          // which row of a pair this lane loads, and
    const uint32_t kpiece = 16u * ((uint32_t) (lane & 31) ^ (2u * kh));   // which piece of it
    // chunk c0 into a stage: the loader wave's 32 instructions
    auto fetch = [&](int c0, int stage) {
        const bool inside = uniform(c0 + AT_CH <= ctx_max);   // a chunk inside the window's rows: no clamping
#pragma unroll
        for (int j = 0; j < AT_CH / 2; ++j) {   // K: rows c0 + 2 j, c0 + 2 j + 1
            const int row = inside ? c0 + 2 * j + kh : att_fetch_row(win, c0, 2 * j + kh);
            lds_load16(kc, (uint32_t) row * krowb + (uint32_t) kvh * (AT_HD * 2) + kpiece, lk_at + stage * AT_KSTAGE + j * AT_KPAIR);
        }
#pragma unroll
        for (int i = 0; i < 4 * (AT_CH / AT_VB); ++i) {   // V: quarter qq of block b of the chunk
            const int b = i >> 2, qq = i & 3;
            const int blk = inside ? c0 / AT_VB + b : att_fetch_vblock(win, c0, b);
            lds_load16(vc, (uint32_t) blk * vblkb + (uint32_t) kvh * AT_VBLK + 1024u * qq + 16u * lane, lv_at + stage * AT_VSTAGE + b * AT_VBLK + qq * 1024);
        }
    };
    // The block meets where a chunk's pieces must all have landed. The loader's loads complete in order, so it waits until
    // only the newest chunk's 32 may be on their way (or none); the others wait for their LDS reads and writes; then all
    // for one another. (A plain barrier instruction: __syncthreads() would also wait for the loads that are meant to stay
    // in flight.)
    auto meet = [&](bool newest_in_flight) {
        __builtin_amdgcn_sched_barrier(0);
        if (newest_in_flight) __builtin_amdgcn_s_waitcnt(0x8070);   // vmcnt(32) lgkmcnt(0)
        else __builtin_amdgcn_s_waitcnt(0x0070);                    // vmcnt(0) lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    // The loader: two chunks ahead of the others, meeting them at every barrier of theirs (one when the first chunk has
    // landed, one at the end of every chunk, and one more in a chunk that reaches past the window's rows, whose V slots the
    // others then zero).
    if (loader) {
        fetch(p0, 0);
        if (p0 + AT_CH < p1) fetch(p0 + AT_CH, 1);
        meet(p0 + AT_CH < p1);
        int stage = 0;
        for (int c0 = p0; c0 < p1; c0 += AT_CH, stage = stage == AT_STAGES - 1 ? 0 : stage + 1) {
            if (uniform(c0 + AT_CH > ctx_max)) meet(false);
            const bool more2 = uniform(c0 + 2 * AT_CH < p1);
            if (more2) fetch(c0 + 2 * AT_CH, stage == 0 ? 2 : stage - 1);   // into the stage that the chunk before this one left
            meet(more2);
        }
        return;
    }
    // Q^T operands: step ks holds dims 64 pg + 8 ks .. + 7 of query ql, times 1/16 (exact), as two f16 terms hi + lo:
    // the cache is f16 already, so with q (and below the probabilities) split this way the products carry fp32's
    // precision, as the reference's f32 arithmetic on the f16 cache does. (Converted while the first chunk is on its way.)
    at_v8h Q[8], Ql[8];
    {
        const float sc = qlive ? 0.0625f : 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const float4 a = qa[ks], b = qb[ks];
            const float v[8] = {a.x * sc, a.y * sc, a.z * sc, a.w * sc, b.x * sc, b.y * sc, b.z * sc, b.w * sc};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const _Float16 hi = (_Float16) v[j];
                Q[ks][j] = hi;
                Ql[ks][j] = (_Float16) (v[j] - (float) hi);
            }
        }
    }
    at_v4f O[16];
#pragma unroll
    for (int dt = 0; dt < 16; ++dt) O[dt] = at_v4f{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, z = 0.f;
    meet(false);
    // lane (ql, pg) as row ql of a tile of K: position 8 (ql / 4) + ql % 4 of the chunk (tile 1: four further, two pairs);
    // an odd row is the second of its pair, where piece c lies at c ^ 2: steps 0, 1, 4, 5 and steps 2, 3, 6, 7 from two bases
    const int krow = 8 * (ql >> 2) + (ql & 3), kswz = 32 * (krow & 1);
    const uint8_t* kev = lk + (krow >> 1) * AT_KPAIR + (krow & 1) * (AT_HD * 2) + 128 * pg + kswz;
    const uint8_t* kod = kev - 2 * kswz;
    const uint8_t* vlane = lv + pg * AT_VBLK + 16 * ql;   // dim ql of block pg: the operand of dim tile dt lies 256 dt further
    int stage = 0;
    for (int c0 = p0; c0 < p1; c0 += AT_CH, stage = stage == AT_STAGES - 1 ? 0 : stage + 1) {
        // Positions past the window's rows were never written: whatever their cells hold must not reach the P V products (a
        // zero probability does not stop a NaN). In a chunk that reaches past the rows - the last one of a context, no
        // other - their slots of the V stage are zeroed here, thread by dimension (a block clamped to the window's last
        // repeats that block: all of its slots are past the rows).
        if (uniform(c0 + AT_CH > ctx_max)) {
            for (int p = max(ctx_max - c0, 0); p < AT_CH; ++p)   // (threads 0 .. 255: the loader is not here)
                *reinterpret_cast<volatile uint16_t*>(lv + stage * AT_VSTAGE + (p / AT_VB) * AT_VBLK + threadIdx.x * (AT_VB * 2) + 2 * (p % AT_VB)) = 0;
            meet(false);   // (nothing is in flight in a context's last chunk)
        }
        // The K operands are read a group (two steps of both tiles: four 16-byte reads) ahead of the products that use them,
        // the first group before the block's own stores and loads below: after the barrier the four waves ask the LDS for
        // the same rows at the same time, and a read that is only issued when it is needed waits for all four.
        const uint8_t* k0a = kev + stage * AT_KSTAGE;   // tile 0, steps 0, 1, 4, 5; tile 1 lies two pairs further
        const uint8_t* k0b = kod + stage * AT_KSTAGE;   // steps 2, 3, 6, 7
        at_v4u kq[2][4];
        auto kread = [&](int g, at_v4u (&o)[4]) {   // steps 2 g and 2 g + 1 of both tiles
            const uint8_t* k0 = (g & 1) ? k0b : k0a;
            o[0] = *reinterpret_cast<const at_v4u*>(k0 + 32 * g);
            o[1] = *reinterpret_cast<const at_v4u*>(k0 + 2 * AT_KPAIR + 32 * g);
            o[2] = *reinterpret_cast<const at_v4u*>(k0 + 32 * g + 16);
            o[3] = *reinterpret_cast<const at_v4u*>(k0 + 2 * AT_KPAIR + 32 * g + 16);
        };
        if (wave_on) kread(0, kq[0]);
        __builtin_amdgcn_sched_barrier(0);
        if (wave_on) {
        // the two tiles' hi and lo terms in chains of their own, interleaved: a chain's next MFMA is four issues away, so
        // none waits for the one before it
        at_v4f S[2];
        {
            at_v4f a0 = at_v4f{0.f, 0.f, 0.f, 0.f}, a0l = a0, a1 = a0, a1l = a0;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                if (g < 3) kread(g + 1, kq[(g + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int ks = 2 * g + j;
                    const at_v8h kk0 = __builtin_bit_cast(at_v8h, kq[g & 1][2 * j]), kk1 = __builtin_bit_cast(at_v8h, kq[g & 1][2 * j + 1]);
                    a0l = __builtin_amdgcn_mfma_f32_16x16x32_f16(kk0, Ql[ks], a0l, 0, 0, 0);
                    a1l = __builtin_amdgcn_mfma_f32_16x16x32_f16(kk1, Ql[ks], a1l, 0, 0, 0);
                    a0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kk0, Q[ks], a0, 0, 0, 0);
                    a1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(kk1, Q[ks], a1, 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            S[0] = a0 + a0l;
            S[1] = a1 + a1l;
        }
        const uint8_t* vb = vlane + stage * AT_VSTAGE;
        // four dim tiles at a time: the lo products of all four, then the hi ones (a chain's next MFMA four issues away);
        // the next four tiles' V reads are issued before this group's arithmetic
        at_v4u ra[2][4];
        auto vread = [&](int d0, at_v4u (&o)[4]) {
#pragma unroll
            for (int u = 0; u < 4; ++u) o[u] = *reinterpret_cast<const at_v4u*>(vb + 256 * (d0 + u));
        };
        vread(0, ra[0]);   // (on its way during the softmax below)
        __builtin_amdgcn_sched_barrier(0);
        // this lane: query ql, positions c0 + 8 pg + r (tile 0) and c0 + 8 pg + 4 + r (tile 1). A chunk that every query of
        // the wave sees whole (all but the last ones of a context) needs no masks: its maximum is finite
        float pw[8], ps = 0.f, mn, sc;
        if (uniform(c0 + AT_CH <= vis)) {
            const float mx = groups4_max(fmaxf(fmaxf(fmaxf(S[0][0], S[0][1]), fmaxf(S[0][2], S[0][3])), fmaxf(fmaxf(S[1][0], S[1][1]), fmaxf(S[1][2], S[1][3]))));
            mn = fmaxf(m, mx);
            sc = __expf(m - mn);   // m = -inf before the first chunk: 0
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                pw[r] = __expf(S[r >> 2][r & 3] - mn);
                ps += pw[r];
            }
        } else {
            float sv[8];
            float mx = -INFINITY;
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const int pos = c0 + 8 * pg + r;
                sv[r] = pos < ctx_q && pos < p1 ? S[r >> 2][r & 3] : -INFINITY;
                mx = fmaxf(mx, sv[r]);
            }
            mx = groups4_max(mx);
            mn = fmaxf(m, mx);
            sc = m == -INFINITY ? 0.f : __expf(m - mn);
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                pw[r] = sv[r] == -INFINITY ? 0.f : __expf(sv[r] - mn);
                ps += pw[r];
            }
        }
        ps = groups4_sum(ps);
        z = z * sc + ps;
        m = mn;
        at_v8h P, Pl;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const _Float16 hi = (_Float16) pw[r];
            P[r] = hi;
            Pl[r] = (_Float16) (pw[r] - (float) hi);
        }
        // V^T operands: positions c0 + 8 pg .. + 7 (block pg of the chunk), dim 16 dt + ql (slots past the window's rows
        // hold zeros: see the loop's top)
        if (__any(sc != 1.0f)) {   // the running maximum moved (rare once the first chunks are behind)
#pragma unroll
            for (int dt = 0; dt < 16; ++dt) {
                O[dt].x *= sc;
                O[dt].y *= sc;
                O[dt].z *= sc;
                O[dt].w *= sc;
            }
        }
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
            if (gq < 3) vread(4 * (gq + 1), ra[(gq + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
            at_v8h a[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) a[u] = __builtin_bit_cast(at_v8h, ra[gq & 1][u]);
#pragma unroll
            for (int u = 0; u < 4; ++u) O[4 * gq + u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u], Pl, O[4 * gq + u], 0, 0, 0);
#pragma unroll
            for (int u = 0; u < 4; ++u) O[4 * gq + u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u], P, O[4 * gq + u], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        }
        meet(false);   // the next chunk's pieces have landed, and this chunk's stage is free for the chunk after it
    }
    if (!qlive) return;
    // accumulator lane (dim group pg, query ql): dims 16 dt + 4 pg + r
#pragma unroll
    for (int dt = 0; dt < 16; ++dt)
        *reinterpret_cast<float4*>(acc_out + slot * AT_HD + 16 * dt + 4 * pg) = make_float4(O[dt].x, O[dt].y, O[dt].z, O[dt].w);
    if (pg == 0) mz_out[slot] = AttPart{m, z};
}
// a block per (head, row): the splits' weights exp(m_s - max) first (LDS), then every thread sums its dimension over the
// splits that hold data, several loads in flight. out (f32) and outq (q8_1 rows) may each be null.
constexpr int AT_MAXSPLIT = 2048;   // splits of the largest cache; a query has twice as many parts at most
__global__ void __launch_bounds__(AT_HD) k_attn_combine(const float* __restrict__ qg, const float* __restrict__ acc_in,
                                                       const AttPart* __restrict__ mz_in, float* __restrict__ out, uint8_t* __restrict__ outq,
                                                       int nq, int nkv, int nsplit, int T, const int* __restrict__ pos0p, int max_ctx,
                                                       unsigned* __restrict__ err, const int* __restrict__ gate, const int* __restrict__ live) {
    __shared__ float wsp[2 * AT_MAXSPLIT];
    __shared__ float red[AT_HD / 64];
    const int gate_v = gate ? *gate : 1, live_v = live ? *live : T, pos0_v = uniform(*pos0p);   // (asked for together)
    if (uniform(gate_v) == 0) return;
    // a window that leaves the cache: reported (err may be null), and computed over the cells that exist
    if (err && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0 && !att_window_fits(pos0_v, T, max_ctx)) atomicOr(err, FNX_ERR_WINDOW);
    T = uniform(max(1, min(live_v, T)));
    const int h = blockIdx.x, t = blockIdx.y, i = threadIdx.x;
    if (t >= T) {   // a row that does not count: zeros (its queries were left out; what follows it stays finite)
        if (out) out[((size_t) t * nq + h) * AT_HD + i] = 0.f;
        if (outq) q8_1_store(0.f, outq + (((size_t) t * nq + h) * (AT_HD / 32) + i / 32) * FNX_Q8_1_BLOCK, i & 31);
        return;
    }
    const bool halves = att_halves(T * (nq / nkv));
    const size_t base = ((size_t) t * nq + h) * att_part_stride(nsplit, halves);
    // the parts the window's context reaches: they were written (whole splits, or their halves for a window of few queries)
    const int nlive = att_live_parts(att_window(pos0_v, T, max_ctx), nsplit, halves);
    float mx = -INFINITY;
    for (int s = i; s < nlive; s += AT_HD) mx = fmaxf(mx, mz_in[base + s].m);
    mx = group_max<64>(mx);
    if ((i & 63) == 0) red[i >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float zp = 0.f;
    for (int s = i; s < nlive; s += AT_HD) {
        const AttPart p = mz_in[base + s];
        const float w = p.m == -INFINITY ? 0.f : expf(p.m - mx);
        wsp[s] = w;
        zp = fmaf(w, p.z, zp);
    }
    zp = group_sum<64>(zp);
    if ((i & 63) == 0) red[i >> 6] = zp;
    __syncthreads();
    const float z = (red[0] + red[1]) + (red[2] + red[3]);
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    const float* ap = acc_in + base * AT_HD + i;
    int s = 0;
    // A window of few rows has few blocks here, each with twice the parts: its time is the round trips of a thread's loads one
    // batch after the other, so thirty-two are asked for at once (the chains take them in the same order; with a block a
    // (head, row) of a full window, whose parts' 17 MB are the time, that was slower than four).
    if (T * nq <= 128) {
        for (; s + 32 <= nlive; s += 32) {
            float v[32];
#pragma unroll
            for (int j = 0; j < 32; ++j) v[j] = ap[(size_t) (s + j) * AT_HD];
#pragma unroll
            for (int j = 0; j < 32; j += 4) {
                a0 = fmaf(wsp[s + j], v[j], a0);
                a1 = fmaf(wsp[s + j + 1], v[j + 1], a1);
                a2 = fmaf(wsp[s + j + 2], v[j + 2], a2);
                a3 = fmaf(wsp[s + j + 3], v[j + 3], a3);
            }
        }
    }
#pragma unroll 4
    for (; s + 4 <= nlive; s += 4) {
        a0 = fmaf(wsp[s], ap[(size_t) s * AT_HD], a0);
        a1 = fmaf(wsp[s + 1], ap[(size_t) (s + 1) * AT_HD], a1);
        a2 = fmaf(wsp[s + 2], ap[(size_t) (s + 2) * AT_HD], a2);
        a3 = fmaf(wsp[s + 3], ap[(size_t) (s + 3) * AT_HD], a3);
    }
    for (; s < nlive; ++s) a0 = fmaf(wsp[s], ap[(size_t) s * AT_HD], a0);
    const float acc = (a0 + a1) + (a2 + a3);
    const float v = acc / z * sigmoid_f(qg[((size_t) t * nq + h) * 2 * AT_HD + AT_HD + i]);
    if (out) out[((size_t) t * nq + h) * AT_HD + i] = v;
    // the row's q8_1 form (the input of the output projection): a head is eight blocks of 32 dims, a half-wave each
    if (outq) q8_1_store(v, outq + (((size_t) t * nq + h) * (AT_HD / 32) + i / 32) * FNX_Q8_1_BLOCK, i & 31);
}

}  // namespace fnx
