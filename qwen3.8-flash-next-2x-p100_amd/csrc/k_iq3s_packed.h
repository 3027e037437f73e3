// IQ3_S expert mat-vec on the unit-packed layout: the verify window's hot kernels.
//
// Layout ("unit64", type id FNX_T_IQ3S_UNIT64): the tensor's sub-blocks of 32 weights, in memory order, are taken 64
// at a time; each such unit still occupies 64/8 x 110 = 880 bytes:
// Sub-block l's eight 13-bit codebook indexes (index = sign nibble << 9 | high bit << 8 | code byte: the signed
// codebook's index) form a 104-bit little-endian string, stored in three planes so that every load of a wave is
// aligned and contiguous over its 64 lanes:
//     bytes [  0, 512): plane A: bits  0..63 of sub-block l at byte 8 l
//     bytes [512, 768): plane B: bits 64..95 at byte 512 + 4 l
//     bytes [768, 832): plane C: bits 96..103 at byte 768 + l
//     bytes [832, 864): the 64 scale nibbles, sub-block l in nibble l & 1 of byte 832 + l / 2
//     bytes [864, 880): the unit's eight super-block scales d (f16)
// Same bits as ggml's block_iq3_s (tensor_convert.hpp:295-301 of the reference), re-laid once at load the way the
// reference re-lays its dense matrices (model.hpp:78-82). A lane turns a group of 4 weights into a dot-product operand
// with two ALU ops and one LDS read. (Measured on MI355X: 13-byte chunks per lane read with unaligned 16-byte loads
// stream at 3.4 TB/s, these planes at 4.6 TB/s, against 5.0 TB/s for a plain aligned read of the same bytes.)
#pragma once

#include "fnx_device.h"

namespace fnx {

constexpr int UNIT_BYTES = 880, UNIT_B_AT = 512, UNIT_C_AT = 768, UNIT_SCALES_AT = 832, UNIT_D_AT = 864;

typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));

struct PackedSub {   // one lane's share of a unit as loaded
    v4u idx;         // the 104 bits of indexes: planes A (x, y), B (z), C (w)
    uint32_t sc, d;  // the scales byte, the d bits
};
struct PackedOffs {
    uint32_t a, b, c, sc, d;
};
__device__ __forceinline__ PackedOffs packed_offs(int lane) {
    PackedOffs o;
    o.a = 8 * lane;
    o.b = UNIT_B_AT + 4 * lane;
    o.c = UNIT_C_AT + lane;
    o.sc = UNIT_SCALES_AT + (lane >> 1);
    o.d = UNIT_D_AT + 2 * (lane >> 3);
    return o;
}
__device__ __forceinline__ PackedSub load_packed(gbytes unit, const PackedOffs& o) {   // unit: wave-uniform
    typedef __attribute__((address_space(1))) const v2u g64;
    typedef __attribute__((address_space(1))) const uint32_t g32;
    typedef __attribute__((address_space(1))) const unsigned short gu16;
    uint32_t oa = o.a, ob = o.b, oc = o.c, os = o.sc, od = o.d;
    asm volatile("" : "+v"(oa), "+v"(ob), "+v"(oc), "+v"(os), "+v"(od));   // keeps the zero-extensions next to the loads (SGPR-base addressing)
    PackedSub r;
    const v2u a = *(g64*) (unit + oa);
    r.idx.x = a.x;
    r.idx.y = a.y;
    r.idx.z = *(g32*) (unit + ob);
    r.idx.w = unit[oc];
    r.sc = unit[os];
    r.d = *(gu16*) (unit + od);
    return r;
}
// The same loads through a buffer descriptor: base = a matrix (wave-uniform), a scalar byte offset for the unit, the
// lane's five offsets as they are - no vector arithmetic per load, and the planes' positions ride in the instructions.
struct PackedVOffs {
    int a, b, c, sc, d;
};
__device__ __forceinline__ PackedVOffs packed_voffs(int lane) {
    return PackedVOffs{8 * lane, 4 * lane, lane, lane >> 1, 2 * (lane >> 3)};
}
__device__ __forceinline__ __amdgpu_buffer_rsrc_t matrix_rsrc(const uint8_t* base) {   // base: wave-uniform
    return __builtin_amdgcn_make_buffer_rsrc((void*) base, 0, -1, 0x00020000);
}
__device__ __forceinline__ PackedSub load_packed_buf(__amdgpu_buffer_rsrc_t m, int unit_byte, const PackedVOffs& o) {   // unit_byte: wave-uniform
    PackedSub r;
    const v2u a = __builtin_amdgcn_raw_buffer_load_b64(m, o.a, unit_byte, 0);
    r.idx.x = a.x;
    r.idx.y = a.y;
    r.idx.z = __builtin_amdgcn_raw_buffer_load_b32(m, o.b + UNIT_B_AT, unit_byte, 0);
    r.idx.w = __builtin_amdgcn_raw_buffer_load_b8(m, o.c + UNIT_C_AT, unit_byte, 0);
    r.sc = __builtin_amdgcn_raw_buffer_load_b8(m, o.sc + UNIT_SCALES_AT, unit_byte, 0);
    r.d = __builtin_amdgcn_raw_buffer_load_b16(m, o.d + UNIT_D_AT, unit_byte, 0);
    return r;
}
// LDS byte address of group j's entry in the signed codebook: field j << 2
__device__ __forceinline__ uint32_t packed_addr(const v4u& q, int j) {
    const int bit = 13 * j, w = bit >> 5, s = bit & 31;
    uint32_t v;
    if (s + 13 <= 32) v = s >= 2 ? q[w] >> (s - 2) : q[w] << (2 - s);
    else v = __builtin_amdgcn_alignbit(q[w + 1], q[w], s - 2);   // the field straddles two words (s >= 20 there)
    return v & 0x7FFCu;
}

// four per-lane partial sums (one per unit, a unit a row of 64 sub-blocks) -> each unit's total over the 64 lanes, in
// butterfly_sum<64>'s order (l ^ 32, l ^ 16, then 8, 4, 2, 1) with the first two steps of the four units done together. On
// return every lane of 16-lane row 0 holds a's total, row 1 c's, row 2 b's, row 3 d's.
__device__ __forceinline__ float reduce4_units(float a, float b, float c, float d) {
    const float p = swap32_add(a, b), q = swap32_add(c, d);
    return butterfly_sum<16>(swap16_add(p, q));   // rows: a, c, b, d
}
// which of the four units a lane's 16-lane row holds after reduce4_units
__device__ __forceinline__ int reduce4_unit_of_row(int row) { return ((row & 1) << 1) | (row >> 1); }

// SBR: sub-blocks per weight row (ncols / 32): 64, 32, 16 or 8. NT: tokens of the job kept in registers.
// Units go four at a time; the loads of the next four are issued before the current four are decoded.
// prep(xs, dx, orow): fills the NT tokens' int8 activations of this lane's sub-block column (8 dwords each), their
// scales and their output rows; it runs after the first weight loads are issued, so its own latency hides behind them.
// issues the loads of units ua .. ua + 3 of an expert's matrix (past ub - 1: the last unit again)
__device__ __forceinline__ void packed_first(const uint8_t* __restrict__ we, int ua, int ub, PackedSub (&cur)[4]) {
    const PackedOffs o = packed_offs(threadIdx.x & 63);
#pragma unroll
    for (int r = 0; r < 4; ++r) cur[r] = load_packed(as_global(uniform_ptr(we + (size_t) min(ua + r, ub - 1) * UNIT_BYTES)), o);
}
// cur: the first four units, loads already issued by packed_first (so the caller can put other latencies behind them)
template <int SBR, int NT, class Prep>
__device__ __forceinline__ void packed_units(const uint32_t* __restrict__ tab, const uint8_t* __restrict__ we, int ua, int ub,
                                             PackedSub (&cur)[4], Prep prep) {
    constexpr int R = 4, RW = 64 / SBR;   // units in flight, rows per unit
    const int lane = threadIdx.x & 63, g = lane / SBR, kb = lane % SBR;
    const PackedOffs o = packed_offs(lane);
    const int sc_shift = 4 * (lane & 1), last = ub - 1;
    auto unit_at = [&](int ui) { return as_global(uniform_ptr(we + (size_t) min(ui, last) * UNIT_BYTES)); };
    int xs[NT][8];
    float dx[NT];
    float* orow[NT];
    prep(xs, dx, orow);
    for (int u = ua; u < ub; u += R) {
        PackedSub nxt[R];
#pragma unroll
        for (int r = 0; r < R; ++r) nxt[r] = load_packed(unit_at(u + R + r), o);   // past the end: the last unit again
        float v[R][NT];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int w4[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) w4[j] = *reinterpret_cast<const int*>(reinterpret_cast<const uint8_t*>(tab) + packed_addr(cur[r].idx, j));
            const int sc = 1 + 2 * (int) ((cur[r].sc >> sc_shift) & 0xFu);
            const float dw = half_bits_to_float(cur[r].d);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                int sum = 0;
#pragma unroll
                for (int j = 0; j < 8; ++j) sum = __builtin_amdgcn_sdot4(w4[j], xs[t][j], sum, false);
                // one sub-block's term as the reference forms it: (d_w * d_x) * (float) (sumi * (1 + 2 s))
                v[r][t] = (dw * dx[t]) * (float) __mul24(sum, sc);
            }
        }
        if constexpr (SBR == 64) {
            // a unit is one row: the four units' sums in one transposed reduction, one store for the four rows
            const int row4 = lane >> 4, ur = reduce4_unit_of_row(row4);
            const bool store = (lane & 15) == 0 && u + ur < ub;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const float z = reduce4_units(v[0][t], v[1][t], v[2][t], v[3][t]);
                if (store) orow[t][u + ur] = z;
            }
        } else {
            // a unit holds 64 / SBR rows, one per group of SBR lanes
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const float z = butterfly_sum<SBR>(v[r][t]);
                    if (kb == SBR - 1 && u + r < ub) orow[t][(size_t) (u + r) * RW + g] = z;
                }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) cur[r] = nxt[r];
    }
}

// tokens from a job list and q8_1 rows in memory (the operator entry points)
template <int SBR, int NT>
struct JobPrep {
    const fnx_job* jb;
    int t0;
    const uint8_t* y;
    float* out;
    int out_stride;
    __device__ __forceinline__ void operator()(int (&xs)[NT][8], float (&dx)[NT], float* (&orow)[NT]) const {
        const int kb = (threadIdx.x & 63) % SBR;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const uint8_t* yb = y + ((size_t) uniform(jb->y[t0 + t]) * SBR + kb) * FNX_Q8_1_BLOCK;
            dx[t] = half_bits_to_float(*reinterpret_cast<const unsigned short*>(yb));
#pragma unroll
            for (int j = 0; j < 8; ++j) xs[t][j] = reinterpret_cast<const int*>(yb + 4)[j];
            orow[t] = out + (size_t) uniform(jb->out[t0 + t]) * out_stride;
        }
    }
};

template <int SBR, bool WIDE>
__device__ __forceinline__ void packed_range(const uint32_t* tab, const uint8_t* we, int ua, int ub, const fnx_job* jb, const uint8_t* y,
                                             float* out, int out_stride) {
    const int n = uniform(jb->n);
    PackedSub cur[4];
    for (int t0 = 0; t0 < n;) {
        const int nt = n - t0;
        packed_first(we, ua, ub, cur);
        if (WIDE && nt >= 16) {
            packed_units<SBR, 16>(tab, we, ua, ub, cur, JobPrep<SBR, 16>{jb, t0, y, out, out_stride});
            t0 += 16;
        } else if (WIDE && nt >= 8) {
            packed_units<SBR, 8>(tab, we, ua, ub, cur, JobPrep<SBR, 8>{jb, t0, y, out, out_stride});
            t0 += 8;
        } else if (WIDE && nt >= 4) {
            packed_units<SBR, 4>(tab, we, ua, ub, cur, JobPrep<SBR, 4>{jb, t0, y, out, out_stride});
            t0 += 4;
        } else if (WIDE && nt == 3) {
            packed_units<SBR, 3>(tab, we, ua, ub, cur, JobPrep<SBR, 3>{jb, t0, y, out, out_stride});
            t0 += 3;
        } else if (nt >= 2) {
            packed_units<SBR, 2>(tab, we, ua, ub, cur, JobPrep<SBR, 2>{jb, t0, y, out, out_stride});
            t0 += 2;
        } else {
            packed_units<SBR, 1>(tab, we, ua, ub, cur, JobPrep<SBR, 1>{jb, t0, y, out, out_stride});
            t0 += 1;
        }
    }
}

// ---------------------------------------------------------------- raw ggml blocks -> unit64 (once, at load)
// One wave per unit. Every lane reads its sub-block's raw fields first, the wave then writes the unit, so src and dst
// may be the same buffer.
__global__ void __launch_bounds__(256) k_iq3s_repack(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, long units) {
    __shared__ uint32_t stage[4][UNIT_BYTES / 4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, sb = lane >> 3, ib = lane & 7;
    const long u = (long) blockIdx.x * 4 + wave;
    const bool live = u < units;
    uint32_t q0 = 0, q1 = 0, sg = 0, qh = 0, sc = 0, d = 0;
    if (live) {
        const uint8_t* blk = src + u * UNIT_BYTES + sb * FNX_IQ3S_BLOCK;
        d = load_u16(blk);
        q0 = load_u32_a2(blk + 2 + 8 * ib);
        q1 = load_u32_a2(blk + 6 + 8 * ib);
        sg = load_u32_a2(blk + 74 + 4 * ib);
        qh = blk[66 + ib];
        sc = blk[106 + (ib >> 1)];
    }
    uint8_t* st = reinterpret_cast<uint8_t*>(stage[wave]);
    // 8 fields of 13 bits -> 13 bytes
    unsigned long long lo = 0, hi = 0;   // bits 0..63, 64..103
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const unsigned long long f = (((j < 4 ? q0 : q1) >> (8 * (j & 3))) & 0xFFu) | (((qh >> j) & 1u) << 8) | (((sg >> (4 * j)) & 0xFu) << 9);
        const int bit = 13 * j;
        if (bit < 64) lo |= f << bit;
        if (bit + 13 > 64) hi |= bit >= 64 ? f << (bit - 64) : f >> (64 - bit);
    }
    reinterpret_cast<unsigned long long*>(st)[lane] = lo;                       // plane A
    reinterpret_cast<uint32_t*>(st + UNIT_B_AT)[lane] = (uint32_t) hi;          // plane B
    st[UNIT_C_AT + lane] = (uint8_t) (hi >> 32);                                // plane C
    // scales: sub-block l's nibble to nibble l & 1 of byte l / 2 (raw: nibble ib & 1 of byte ib / 2 of its super-block: the same order)
    if ((ib & 1) == 0) st[UNIT_SCALES_AT + (lane >> 1)] = (uint8_t) sc;
    if (ib == 0) reinterpret_cast<unsigned short*>(st + UNIT_D_AT)[sb] = (unsigned short) d;
    __syncthreads();
    if (live)
        for (int i = lane; i < UNIT_BYTES / 4; i += 64) reinterpret_cast<uint32_t*>(dst + u * UNIT_BYTES)[i] = stage[wave][i];
}

}  // namespace fnx
