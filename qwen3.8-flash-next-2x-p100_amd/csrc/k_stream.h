// Read-only streaming calibration: what this GPU's HBM gives a kernel that only reads, with the load shapes of the
// expert mat-vec kernels (the unit64 planes, four units in flight a wave) and with plain 8- and 16-byte loads at several
// depths. The verify window's pass launches are judged against these rates. No counterpart in the reference.
#pragma once

#include "k_iq3s_packed.h"

namespace fnx {

typedef __attribute__((address_space(1))) const v4u g128;
typedef __attribute__((address_space(1))) const v2u g64v;

// the share of `total` items that wave gw of nw takes when the items are split evenly in order
__device__ __forceinline__ size_t stream_share(size_t total, uint32_t gw, uint32_t nw) { return (size_t) ((unsigned __int128) total * gw / nw); }

// VB: bytes a lane and load (8 or 16). DEPTH: loads a lane has in flight. NT: nontemporal loads. RANGE: a wave reads one
// contiguous range (as the job kernels do); else chunk c goes to wave c mod the grid's waves.
template <int VB, int DEPTH, bool NT, bool RANGE>
__global__ void __launch_bounds__(1024) k_stream_read(const uint8_t* __restrict__ p, size_t chunks, uint32_t* __restrict__ sink) {
    const uint32_t lane = threadIdx.x & 63, wpb = blockDim.x >> 6;
    const uint32_t gw = blockIdx.x * wpb + (uint32_t) uniform((int) (threadIdx.x >> 6)), nw = gridDim.x * wpb;
    size_t c, c1, step;
    if (RANGE) {
        c = stream_share(chunks, gw, nw);
        c1 = stream_share(chunks, gw + 1, nw);
        step = 1;
    } else {
        c = gw;
        c1 = chunks;
        step = nw;
    }
    const uint32_t off = lane * VB;
    auto load = [&](size_t ci) {
        gbytes base = as_global(uniform_ptr(p + ci * (size_t) (64 * VB)));
        uint32_t o = off;
        asm volatile("" : "+v"(o));
        v4u r;
        if constexpr (VB == 16) {
            r = NT ? __builtin_nontemporal_load((g128*) (base + o)) : *(g128*) (base + o);
        } else {
            const v2u h = NT ? __builtin_nontemporal_load((g64v*) (base + o)) : *(g64v*) (base + o);
            r = v4u{h.x, h.y, 0u, 0u};
        }
        return r;
    };
    uint32_t acc = 0;
    v4u cur[DEPTH];
#pragma unroll
    for (int i = 0; i < DEPTH; ++i) cur[i] = c + i * step < c1 ? load(c + i * step) : v4u{0u, 0u, 0u, 0u};
    for (; c < c1; c += DEPTH * step) {
        v4u nxt[DEPTH];
#pragma unroll
        for (int i = 0; i < DEPTH; ++i) {
            const size_t ci = c + (DEPTH + i) * step;
            nxt[i] = ci < c1 ? load(ci) : v4u{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int i = 0; i < DEPTH; ++i) acc ^= cur[i].x ^ cur[i].y ^ cur[i].z ^ cur[i].w;
#pragma unroll
        for (int i = 0; i < DEPTH; ++i) cur[i] = nxt[i];
    }
    if (acc == 0x9E3779B9u) sink[0] = acc;   // keeps the loads alive; practically never taken
}

// the unit64 planes as the expert kernels ask for them: five loads a unit and lane, four units (a group) in flight.
// SPLIT 0: every wave one contiguous range of units; 1: group g goes to wave g mod the grid's waves; 2: every block one
// contiguous range, its waves taking the range's groups in turn. NT: nontemporal loads.
template <bool NT>
__device__ __forceinline__ PackedSub stream_load_packed(gbytes unit, const PackedOffs& o) {
    if constexpr (!NT) return load_packed(unit, o);
    typedef __attribute__((address_space(1))) const v2u g64;
    typedef __attribute__((address_space(1))) const uint32_t g32;
    typedef __attribute__((address_space(1))) const unsigned short gu16;
    uint32_t oa = o.a, ob = o.b, oc = o.c, os = o.sc, od = o.d;
    asm volatile("" : "+v"(oa), "+v"(ob), "+v"(oc), "+v"(os), "+v"(od));
    PackedSub r;
    const v2u a = __builtin_nontemporal_load((g64*) (unit + oa));
    r.idx.x = a.x;
    r.idx.y = a.y;
    r.idx.z = __builtin_nontemporal_load((g32*) (unit + ob));
    r.idx.w = __builtin_nontemporal_load(unit + oc);
    r.sc = __builtin_nontemporal_load(unit + os);
    r.d = __builtin_nontemporal_load((gu16*) (unit + od));
    return r;
}
template <int SPLIT, bool NT>
__global__ void __launch_bounds__(1024) k_stream_read_units(const uint8_t* __restrict__ p, size_t units, uint32_t* __restrict__ sink) {
    const uint32_t wpb = blockDim.x >> 6, wave = (uint32_t) uniform((int) (threadIdx.x >> 6));
    const uint32_t gw = blockIdx.x * wpb + wave, nw = gridDim.x * wpb;
    const size_t groups = (units + 3) / 4;
    size_t g, g1, step;   // this wave's groups: g, g + step, ... below g1
    if (SPLIT == 0) {
        g = stream_share(groups, gw, nw);
        g1 = stream_share(groups, gw + 1, nw);
        step = 1;
    } else if (SPLIT == 1) {
        g = gw;
        g1 = groups;
        step = nw;
    } else {
        g = stream_share(groups, blockIdx.x, gridDim.x) + wave;
        g1 = stream_share(groups, blockIdx.x + 1, gridDim.x);
        step = wpb;
    }
    const PackedOffs o = packed_offs(threadIdx.x & 63);
    auto unit_at = [&](size_t ui) { return as_global(uniform_ptr(p + (ui < units ? ui : units - 1) * UNIT_BYTES)); };
    uint32_t acc = 0;
    if (g >= g1) return;
    PackedSub cur[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) cur[r] = stream_load_packed<NT>(unit_at(4 * g + r), o);
    for (; g < g1; g += step) {
        PackedSub nxt[4];
        const size_t gn = g + step < g1 ? g + step : g;   // past the end: the last group again
#pragma unroll
        for (int r = 0; r < 4; ++r) nxt[r] = stream_load_packed<NT>(unit_at(4 * gn + r), o);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc ^= cur[r].idx.x ^ cur[r].idx.y ^ cur[r].idx.z ^ cur[r].idx.w ^ cur[r].sc ^ cur[r].d;
#pragma unroll
        for (int r = 0; r < 4; ++r) cur[r] = nxt[r];
    }
    if (acc == 0x9E3779B9u) sink[0] = acc;
}

// Four units a lane-interleaved record of 3,520 bytes (the planes of four units side by side a lane): six loads a lane of
// 16, 16, 16, 4, 4 and 8 bytes instead of the twenty of four unit64 units. Record q goes to wave q mod the grid's waves,
// one record in flight while one is summed. NT: nontemporal loads.
constexpr int QUAD_BYTES = 4 * UNIT_BYTES, QUAD_B_AT = 2048, QUAD_C_AT = 3072, QUAD_SC_AT = 3328, QUAD_D_AT = 3456;
struct QuadRaw {
    v4u a0, a1, b;
    uint32_t c, sc;
    v2u d;
};
template <bool NT>
__device__ __forceinline__ QuadRaw stream_load_quad(gbytes q, uint32_t lane) {
    uint32_t oa = 32 * lane, ob = QUAD_B_AT + 16 * lane, oc = QUAD_C_AT + 4 * lane, os = QUAD_SC_AT + 4 * (lane >> 1), od = QUAD_D_AT + 8 * (lane >> 3);
    asm volatile("" : "+v"(oa), "+v"(ob), "+v"(oc), "+v"(os), "+v"(od));
    typedef __attribute__((address_space(1))) const uint32_t g32;
    QuadRaw r;
    if constexpr (NT) {
        r.a0 = __builtin_nontemporal_load((g128*) (q + oa));
        r.a1 = __builtin_nontemporal_load((g128*) (q + oa + 16));
        r.b = __builtin_nontemporal_load((g128*) (q + ob));
        r.c = __builtin_nontemporal_load((g32*) (q + oc));
        r.sc = __builtin_nontemporal_load((g32*) (q + os));
        r.d = __builtin_nontemporal_load((g64v*) (q + od));
    } else {
        r.a0 = *(g128*) (q + oa);
        r.a1 = *(g128*) (q + oa + 16);
        r.b = *(g128*) (q + ob);
        r.c = *(g32*) (q + oc);
        r.sc = *(g32*) (q + os);
        r.d = *(g64v*) (q + od);
    }
    return r;
}
template <bool NT>
__global__ void __launch_bounds__(1024) k_stream_read_quads(const uint8_t* __restrict__ p, size_t quads, uint32_t* __restrict__ sink) {
    const uint32_t wpb = blockDim.x >> 6, wave = (uint32_t) uniform((int) (threadIdx.x >> 6)), lane = threadIdx.x & 63;
    const uint32_t gw = blockIdx.x * wpb + wave, nw = gridDim.x * wpb;
    if (gw >= quads) return;
    auto quad_at = [&](size_t qi) { return as_global(uniform_ptr(p + (qi < quads ? qi : quads - 1) * QUAD_BYTES)); };
    uint32_t acc = 0;
    QuadRaw cur = stream_load_quad<NT>(quad_at(gw), lane);
    for (size_t q = gw; q < quads; q += nw) {
        const QuadRaw nxt = stream_load_quad<NT>(quad_at(q + nw < quads ? q + nw : q), lane);
        acc ^= cur.a0.x ^ cur.a0.y ^ cur.a0.z ^ cur.a0.w ^ cur.a1.x ^ cur.a1.y ^ cur.a1.z ^ cur.a1.w ^ cur.b.x ^ cur.b.y ^ cur.b.z ^ cur.b.w ^ cur.c ^ cur.sc ^
               cur.d.x ^ cur.d.y;
        cur = nxt;
    }
    if (acc == 0x9E3779B9u) sink[0] = acc;
}

// the window kernels' case: segments of `seg_units` units (an expert's matrix) scattered over the buffer, walked in a
// fixed shuffled order; wave gw keeps to a segment for K trips of one group, so the grid reads waves * K * 4 / seg_units
// segments at a time, each as one front that moves through the segment
__global__ void __launch_bounds__(1024) k_stream_read_segments(const uint8_t* __restrict__ p, size_t units, uint32_t seg_units, uint32_t K,
                                                              uint32_t* __restrict__ sink) {
    const uint32_t wpb = blockDim.x >> 6, wave = (uint32_t) uniform((int) (threadIdx.x >> 6));
    const uint32_t gw = blockIdx.x * wpb + wave, nw = gridDim.x * wpb;
    const uint32_t nseg = (uint32_t) (units / seg_units), gps = seg_units / 4;   // groups a segment
    const uint32_t wps = gps / K;                                                // waves a segment
    const uint32_t conc = nw / wps;                                              // segments read at a time
    if (conc == 0 || gw >= conc * wps) return;
    const uint32_t q = gw / wps, j = gw % wps;
    const PackedOffs o = packed_offs(threadIdx.x & 63);
    auto seg_base = [&](uint32_t si) { return (size_t) ((si * 7919u) % nseg) * seg_units; };   // 7919 is prime: a permutation unless nseg is its multiple
    uint32_t acc = 0;
    const uint32_t trips = ((nseg + conc - 1) / conc) * K;
    auto unit_at = [&](uint32_t trip, int r) {
        uint32_t si = (trip / K) * conc + q;
        if (si >= nseg) si = q < nseg ? q : 0;   // past the end: an earlier segment again (the loop below skips the sum)
        return as_global(uniform_ptr(p + (seg_base(si) + 4 * (j + (trip % K) * wps) + r) * UNIT_BYTES));
    };
    PackedSub cur[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) cur[r] = load_packed(unit_at(0, r), o);
    for (uint32_t trip = 0; trip < trips; ++trip) {
        PackedSub nxt[4];
        const uint32_t tn = trip + 1 < trips ? trip + 1 : trip;
#pragma unroll
        for (int r = 0; r < 4; ++r) nxt[r] = load_packed(unit_at(tn, r), o);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc ^= cur[r].idx.x ^ cur[r].idx.y ^ cur[r].idx.z ^ cur[r].idx.w ^ cur[r].sc ^ cur[r].d;
#pragma unroll
        for (int r = 0; r < 4; ++r) cur[r] = nxt[r];
    }
    if (acc == 0x9E3779B9u) sink[0] = acc;
}

}  // namespace fnx
