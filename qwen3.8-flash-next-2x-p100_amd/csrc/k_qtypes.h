// The other expert types the reference's operators take at the boundary (kernels.cu:2454-2471 moe_mm): rows of Q4_0, Q8_0,
// Q5_1, IQ4_NL (32-value blocks) and Q4_K, Q5_K, IQ4_XS (256-value super-blocks of eight 32-value sub-blocks) against q8_1 activation
// rows, through the same job lists. Block layouts as tensor_convert.hpp:152-265 decodes them; a sub-block's term of the
// dot is ggml's vec_dot_<type>_q8_1 per 32 values (the integers through sdot4, the q8_1 sum field for Q4_0's offset and
// the activations' sum for the K-quants' minimum).
//
// Not a tuned path (the benchmark's model keeps its experts in IQ3_S): a wave per (row, job), sub-blocks dealt round-robin
// to the lanes, lane sums added by the xor butterfly.
#pragma once

#include "fnx_device.h"

namespace fnx {

constexpr uint32_t QT_Q4_0 = 2, QT_Q5_1 = 7, QT_Q8_0 = 8, QT_Q4_K = 12, QT_Q5_K = 13, QT_IQ4_NL = 20, QT_IQ4_XS = 23;
// kvalues_iq4nl (tensor_convert.hpp): {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113}, four to a word.
// Four 4-bit indexes (one a byte) -> their four table bytes: a byte permute over each half of the table (selector bytes
// 0..3 take from the second operand, 4..7 from the first), the index's top bit choosing between the halves.
__device__ __forceinline__ uint32_t iq4_values4(uint32_t idx4) {
    constexpr uint32_t t0 = 0xBFAD9881u, t1 = 0xF6EADDCFu, t2 = 0x26190D01u, t3 = 0x71594535u;
    const uint32_t sel = idx4 & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel), hi = __builtin_amdgcn_perm(t3, t2, sel);
    const uint32_t upper = ((idx4 >> 3) & 0x01010101u) * 0xFFu;   // 0xFF in the bytes whose index is 8..15
    return (hi & upper) | (lo & ~upper);
}

struct QtSub {
    int w4[8];       // the sub-block's 32 integers, four to a word
    float d, dmin;   // the block's scales
    int sc, m;       // K-quants: the sub-block's 6-bit scale and minimum
};
// ggml's get_scale_min_k4 (tensor_convert.hpp scale_min_k4)
__device__ __forceinline__ void qt_scale_min(int j, const uint8_t* q, int& sc, int& m) {
    if (j < 4) {
        sc = q[j] & 63;
        m = q[j + 4] & 63;
    } else {
        sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4);
        m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}
template <uint32_t TYPE>
__device__ __forceinline__ QtSub qt_decode(const uint8_t* row, int kb) {
    QtSub o;
    o.dmin = 0.f;
    o.sc = 1;
    o.m = 0;
    if constexpr (TYPE == QT_Q8_0) {
        const uint8_t* p = row + (size_t) kb * 34;
        o.d = half_bits_to_float((unsigned short) load_u16(p));
#pragma unroll
        for (int j = 0; j < 8; ++j) o.w4[j] = (int) load_u32_a2(p + 2 + 4 * j);
    } else if constexpr (TYPE == QT_Q5_1) {   // ggml block_q5_1 {half d; half m; u32 qh; u8 qs[16]}: value = d * q + m
        const uint8_t* p = row + (size_t) kb * 24;
        o.d = half_bits_to_float((unsigned short) load_u16(p));
        o.dmin = half_bits_to_float((unsigned short) load_u16(p + 2));   // m: added
        const uint32_t qh = load_u32_a2(p + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {   // value j: nibble | bit j of qh << 4; value 16 + j: high nibble | bit 16 + j << 4
            const uint32_t v = load_u32_a2(p + 8 + 4 * i);
            uint32_t lo = v & 0x0F0F0F0Fu, hi = (v >> 4) & 0x0F0F0F0Fu;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                lo |= ((qh >> (4 * i + b)) & 1u) << (8 * b + 4);
                hi |= ((qh >> (16 + 4 * i + b)) & 1u) << (8 * b + 4);
            }
            o.w4[i] = (int) lo;
            o.w4[4 + i] = (int) hi;
        }
    } else if constexpr (TYPE == QT_Q4_0) {
        const uint8_t* p = row + (size_t) kb * 18;
        o.d = half_bits_to_float((unsigned short) load_u16(p));
#pragma unroll
        for (int i = 0; i < 4; ++i) {   // low nibbles: values 0..15; high nibbles: 16..31
            const uint32_t v = load_u32_a2(p + 2 + 4 * i);
            o.w4[i] = (int) (v & 0x0F0F0F0Fu);
            o.w4[4 + i] = (int) ((v >> 4) & 0x0F0F0F0Fu);
        }
    } else if constexpr (TYPE == QT_IQ4_NL || TYPE == QT_IQ4_XS) {
        const uint8_t* qs;
        if constexpr (TYPE == QT_IQ4_NL) {
            const uint8_t* p = row + (size_t) kb * 18;
            o.d = half_bits_to_float((unsigned short) load_u16(p));
            qs = p + 2;
        } else {   // {half d; u16 scales_h; u8 scales_l[4]; u8 qs[128]}: sub-block ib's 6-bit scale - 32
            const int ib = kb & 7;
            const uint8_t* p = row + (size_t) (kb >> 3) * 136;
            o.d = half_bits_to_float((unsigned short) load_u16(p));
            const uint32_t sh = load_u16(p + 2);
            o.sc = (int) (((p[4 + ib / 2] >> (4 * (ib % 2))) & 0xFu) | (((sh >> (2 * ib)) & 3u) << 4)) - 32;
            qs = p + 8 + 16 * ib;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t v = load_u32_a2(qs + 4 * i);
            o.w4[i] = (int) iq4_values4(v & 0x0F0F0F0Fu);
            o.w4[4 + i] = (int) iq4_values4((v >> 4) & 0x0F0F0F0Fu);
        }
    } else {
        constexpr bool FIVE = TYPE == QT_Q5_K;
        const int sb = kb & 7;
        const uint8_t* p = row + (size_t) (kb >> 3) * (FIVE ? 176 : 144);
        o.d = half_bits_to_float((unsigned short) load_u16(p));
        o.dmin = half_bits_to_float((unsigned short) load_u16(p + 2));
        qt_scale_min(sb, p + 4, o.sc, o.m);
        const uint8_t *qh = p + 16, *ql = p + (FIVE ? 48 : 16) + 32 * (sb >> 1);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t v = load_u32_a2(ql + 4 * i);
            uint32_t w = (sb & 1) ? (v >> 4) & 0x0F0F0F0Fu : v & 0x0F0F0F0Fu;
            if constexpr (FIVE) w |= ((load_u32_a2(qh + 4 * i) >> sb) & 0x01010101u) << 4;
            o.w4[i] = (int) w;
        }
    }
    return o;
}
// the sub-block's term against one q8_1 block {half d; half sum; int8 qs[32]}
template <uint32_t TYPE>
__device__ __forceinline__ float qt_term(const QtSub& s, const uint8_t* yb) {
    const float dx = half_bits_to_float((unsigned short) load_u16(yb));
    int dot = 0, qsum = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int x = reinterpret_cast<const int*>(yb + 4)[j];
        dot = __builtin_amdgcn_sdot4(s.w4[j], x, dot, false);
        if constexpr (TYPE == QT_Q4_K || TYPE == QT_Q5_K) qsum = __builtin_amdgcn_sdot4(0x01010101, x, qsum, false);
    }
    if constexpr (TYPE == QT_Q4_0) return s.d * ((float) dot * dx - 8.0f * half_bits_to_float((unsigned short) load_u16(yb + 2)));
    else if constexpr (TYPE == QT_Q5_1) return (float) dot * (s.d * dx) + s.dmin * half_bits_to_float((unsigned short) load_u16(yb + 2));
    else if constexpr (TYPE == QT_Q4_K || TYPE == QT_Q5_K) return s.d * (dx * (float) (dot * s.sc)) - s.dmin * (dx * (float) (qsum * s.m));
    else if constexpr (TYPE == QT_IQ4_XS) return (s.d * dx) * (float) (dot * s.sc);
    else return (s.d * dx) * (float) dot;
}

struct QtArgs {
    const uint8_t* wbase;
    size_t w_stride;
    const uint8_t* const* ep;
    size_t row_bytes;
    int nrows, ncols;
    const fnx_job* jobs;
    const int* njobs;
    int njobs_max;
    const uint8_t* y;
    float* out;
    int out_stride;
};
template <uint32_t TYPE>
__global__ void __launch_bounds__(256) k_qt_jobs(const QtArgs a) {
    const int ji = blockIdx.y;
    if (ji >= (a.njobs ? min(*a.njobs, a.njobs_max) : a.njobs_max)) return;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= a.nrows) return;
    const fnx_job* jb = a.jobs + ji;
    const uint8_t* we = (a.ep ? a.ep[jb->w] : a.wbase + (size_t) jb->w * a.w_stride) + (size_t) row * a.row_bytes;
    const int sbr = a.ncols / 32, n = min(max(jb->n, 0), FNX_MAXT);
    const uint8_t* y = a.y ? a.y : g_moe_hq;   // moe_down: the pairs' q8_1 rows in the library's buffer
    for (int t = 0; t < n; ++t) {
        float acc = 0.f;
        for (int kb = lane; kb < sbr; kb += 64) {
            const QtSub s = qt_decode<TYPE>(we, kb);
            acc += qt_term<TYPE>(s, y + ((size_t) jb->y[t] * sbr + kb) * FNX_Q8_1_BLOCK);
        }
        acc = group_sum<64>(acc);
        if (lane == 0) a.out[(size_t) jb->out[t] * a.out_stride + row] = acc;
    }
}

}  // namespace fnx
