// The pieces a whole verify step needs around the MoE half: RMS norm, the dense Q8_0 (split layout) mat-vec of the
// projections and the output head, the attention's prepare/append and split-K decode kernels, embedding rows.
#pragma once

#include "fnx_device.h"

namespace fnx {

constexpr int AT_HD = 256, AT_NROT = 64;   // head width and rotated dims (model.hpp:41 of the reference)

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
__global__ void k_add_rows(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ y, size_t n) {
    for (size_t i = blockIdx.x * (size_t) blockDim.x + threadIdx.x; i < n; i += (size_t) gridDim.x * blockDim.x) y[i] = a[i] + b[i];
}
// rows of an f16 table as f32
__global__ void k_embed_rows(const uint16_t* __restrict__ emb, const int* __restrict__ tokens, int vocab, int n, float* __restrict__ y) {
    const int t = blockIdx.x, tok = min(max(tokens[t], 0), vocab - 1);
    for (int i = threadIdx.x; i < n; i += blockDim.x) y[(size_t) t * n + i] = half_bits_to_float(emb[(size_t) tok * n + i]);
}

// ---------------------------------------------------------------- dense Q8_0, split layout (dense.cuh:79-214)
// int8 values [rows][cols], f16 scales [rows][cols / 32]; activations q8_1. A wave takes Q8S_R rows at a time; lane l takes
// the 16-column pieces l, l + 64, ... of each row (one 16-byte load), acc = fmaf(d_w * d_x, (float) dot, acc) in that
// order, then the xor-butterfly: this order is part of the result's definition (the CPU oracle follows it).
constexpr int Q8S_R = 4, Q8S_WAVES = 4;
struct Q8sArgs {
    const int8_t* q;
    const uint16_t* d;
    int rows, cols;
    const uint8_t* yq;   // q8_1 rows
    float* out;
    int out_stride, T;
};
__global__ void __launch_bounds__(Q8S_WAVES * 64) k_q8s_gemv(const Q8sArgs a) {
    extern __shared__ __align__(16) uint8_t q8s_lds[];   // [T][cols] int8, then [T][cols / 32] f32 scales
    const int nb = a.cols >> 5, T = a.T;
    int8_t* xs = reinterpret_cast<int8_t*>(q8s_lds);
    float* xd = reinterpret_cast<float*>(q8s_lds + (size_t) T * a.cols);
    for (int i = threadIdx.x; i < T * nb; i += blockDim.x) {
        const uint8_t* blk = a.yq + (size_t) i * 36;   // row t = i / nb, block i % nb: rows are contiguous
        xd[i] = half_bits_to_float(load_u16(blk));
        const uint32_t* src = reinterpret_cast<const uint32_t*>(blk + 4);
        uint32_t* dst = reinterpret_cast<uint32_t*>(xs + (size_t) i * 32);
#pragma unroll
        for (int k = 0; k < 8; ++k) dst[k] = src[k];
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int groups = (a.rows + Q8S_R - 1) / Q8S_R;
    for (int grp = blockIdx.x * Q8S_WAVES + wave; grp < groups; grp += gridDim.x * Q8S_WAVES) {
        const int row0 = grp * Q8S_R;
        float acc[Q8S_R][FNX_MAXT];
#pragma unroll
        for (int r = 0; r < Q8S_R; ++r)
#pragma unroll
            for (int t = 0; t < FNX_MAXT; ++t) acc[r][t] = 0.f;
        for (int c = lane * 16; c < a.cols; c += 1024) {
            int4 w[Q8S_R];
            float dw[Q8S_R];
#pragma unroll
            for (int r = 0; r < Q8S_R; ++r) {
                const int row = min(row0 + r, a.rows - 1);
                w[r] = *reinterpret_cast<const int4*>(a.q + (size_t) row * a.cols + c);
                dw[r] = half_bits_to_float(a.d[(size_t) row * nb + (c >> 5)]);
            }
#pragma unroll
            for (int t = 0; t < FNX_MAXT; ++t)
                if (t < T) {
                    const int4 x = *reinterpret_cast<const int4*>(xs + (size_t) t * a.cols + c);
                    const float da = xd[t * nb + (c >> 5)];
#pragma unroll
                    for (int r = 0; r < Q8S_R; ++r) {
                        int s = __builtin_amdgcn_sdot4(w[r].x, x.x, 0, false);
                        s = __builtin_amdgcn_sdot4(w[r].y, x.y, s, false);
                        s = __builtin_amdgcn_sdot4(w[r].z, x.z, s, false);
                        s = __builtin_amdgcn_sdot4(w[r].w, x.w, s, false);
                        acc[r][t] = fmaf(dw[r] * da, (float) s, acc[r][t]);
                    }
                }
        }
#pragma unroll
        for (int r = 0; r < Q8S_R; ++r)
#pragma unroll
            for (int t = 0; t < FNX_MAXT; ++t)
                if (t < T) {
                    const float v = group_sum<64>(acc[r][t]);
                    if (lane == 0 && row0 + r < a.rows) a.out[(size_t) t * a.out_stride + row0 + r] = v;
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
// block (head h, row t), AT_HD threads: q heads normed and rotated in place; k heads normed, rotated and appended; v heads
// appended. The cache is [position][kv head][AT_HD] f16.
__global__ void __launch_bounds__(AT_HD) k_attn_prep_append(float* __restrict__ qg, float* __restrict__ k, const float* __restrict__ v,
                                                           const float* __restrict__ qn, const float* __restrict__ kn,
                                                           uint16_t* __restrict__ kc, uint16_t* __restrict__ vc, int nq, int nkv,
                                                           const int* __restrict__ pos0p, int max_ctx, float eps, RopeDev rope) {
    __shared__ float sh[AT_HD / 64];
    __shared__ float xs[AT_HD];
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
    (is_k ? kc : vc)[((size_t) p * nkv + kh) * AT_HD + i] = float_to_half_bits(x);
}

// ---------------------------------------------------------------- attention: split-K decode (kernels.cu:541-643, 786-803)
// block (split s, row t, kv head): positions [s * len, (s + 1) * len) of [0, pos0 + t] in chunks of 32, for the q heads
// of that kv head, online softmax; each head's running max, sum and AT_HD accumulators go to scratch, the combine
// weighs the splits, divides and applies sigmoid(gate).
constexpr int AT_SPLITS = 16, AT_CH = 32, AT_MAXQ = 8;   // q heads per kv head held by a block
struct AttPart {
    float m, z;
};
__global__ void __launch_bounds__(AT_HD) k_attn_part(const float* __restrict__ qg, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
                                                    float* __restrict__ acc_out, AttPart* __restrict__ mz_out, int nq, int nkv,
                                                    const int* __restrict__ pos0p) {
    const int s = blockIdx.x, t = blockIdx.y, kvh = blockIdx.z, i = threadIdx.x;
    const int qpk = nq / nkv, h0 = kvh * qpk, ctx = *pos0p + t + 1;
    const int len = ((ctx + AT_SPLITS - 1) / AT_SPLITS + AT_CH - 1) / AT_CH * AT_CH;
    const int p0 = s * len, p1 = min(ctx, p0 + len);
    __shared__ float q[AT_MAXQ][AT_HD];
    __shared__ float kk[AT_CH][AT_HD + 1];
    __shared__ float e[AT_MAXQ][AT_CH];
    __shared__ float scale[AT_MAXQ];
    for (int k = i; k < qpk * AT_HD; k += AT_HD) q[k / AT_HD][k % AT_HD] = qg[((size_t) t * nq + h0 + k / AT_HD) * 2 * AT_HD + k % AT_HD];
    // thread (head hh, position pp) of a chunk's scores; thread i also owns dimension i of the accumulators
    const int hh = i >> 5, pp = i & 31;
    float m = -INFINITY, z = 0.f;
    float acc[AT_MAXQ];
#pragma unroll
    for (int k = 0; k < AT_MAXQ; ++k) acc[k] = 0.f;
    __syncthreads();
    for (int c0 = p0; c0 < p1; c0 += AT_CH) {
        const int np = min(AT_CH, p1 - c0);
        float vr[AT_CH];
#pragma unroll
        for (int j = 0; j < AT_CH; ++j) {
            const size_t r = ((size_t) (c0 + min(j, np - 1)) * nkv + kvh) * AT_HD + i;
            kk[j][i] = j < np ? half_bits_to_float(kc[r]) : 0.f;
            vr[j] = j < np ? half_bits_to_float(vc[r]) : 0.f;
        }
        __syncthreads();
        if (hh < qpk) {
            float sacc = 0.f;
#pragma unroll 8
            for (int d = 0; d < AT_HD; ++d) sacc = fmaf(q[hh][d], kk[pp][d], sacc);
            const float sv = pp < np ? sacc * rsqrtf((float) AT_HD) : -INFINITY;
            const float mn = fmaxf(m, group_max<32>(sv));
            const float w = sv == -INFINITY ? 0.f : expf(sv - mn);
            const float sc = m == -INFINITY ? 0.f : expf(m - mn);
            z = z * sc + group_sum<32>(w);
            m = mn;
            e[hh][pp] = w;
            if (pp == 0) scale[hh] = sc;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < AT_MAXQ; ++k)
            if (k < qpk) {
                float av = acc[k] * scale[k];
#pragma unroll
                for (int j = 0; j < AT_CH; ++j) av = fmaf(e[k][j], vr[j], av);
                acc[k] = av;
            }
        __syncthreads();
    }
#pragma unroll
    for (int k = 0; k < AT_MAXQ; ++k)
        if (k < qpk) acc_out[(((size_t) t * nq + h0 + k) * AT_SPLITS + s) * AT_HD + i] = acc[k];
    if (hh < qpk && pp == 0) mz_out[((size_t) t * nq + h0 + hh) * AT_SPLITS + s] = AttPart{m, z};
}
__global__ void __launch_bounds__(AT_HD) k_attn_combine(const float* __restrict__ qg, const float* __restrict__ acc_in,
                                                       const AttPart* __restrict__ mz_in, float* __restrict__ out, int nq) {
    const int h = blockIdx.x, t = blockIdx.y, i = threadIdx.x;
    const size_t base = ((size_t) t * nq + h) * AT_SPLITS;
    float mx = -INFINITY;
#pragma unroll
    for (int s = 0; s < AT_SPLITS; ++s) mx = fmaxf(mx, mz_in[base + s].m);
    float z = 0.f, acc = 0.f;
#pragma unroll
    for (int s = 0; s < AT_SPLITS; ++s) {
        const AttPart p = mz_in[base + s];
        if (p.m == -INFINITY) continue;
        const float w = expf(p.m - mx);
        z = fmaf(w, p.z, z);
        acc = fmaf(w, acc_in[(base + s) * AT_HD + i], acc);
    }
    out[((size_t) t * nq + h) * AT_HD + i] = acc / z * sigmoid_f(qg[((size_t) t * nq + h) * 2 * AT_HD + AT_HD + i]);
}

}  // namespace fnx
