// Device-side helpers shared by the gfx950 kernels: wave64 reductions, half conversion, the signed IQ3_S lookup table.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fnx_expf.h"
#include "iq3s_grid.h"

namespace fnx {

constexpr int WAVE = 64;

// ---- the signed codebook: entry (sign nibble << 9 | 9-bit code) = the group's four weights as signed bytes.
// A lane turns 4 weights into one v_dot4_i32_i8 operand with a single LDS read: 8192 entries, 32 KiB.
struct SignedGrid {
    uint32_t v[8192];
    constexpr SignedGrid() : v() {
        for (int s = 0; s < 16; ++s)
            for (int g = 0; g < 512; ++g) {
                const uint32_t m = fnx_iq3s_grid_host[g];
                uint32_t r = 0;
                for (int j = 0; j < 4; ++j) {
                    int b = (int) ((m >> (8 * j)) & 255u);
                    if ((s >> j) & 1) b = -b;
                    r |= ((uint32_t) b & 255u) << (8 * j);
                }
                v[s * 512 + g] = r;
            }
    }
};
constexpr int SGRID_WORDS = 8192;
// entry (s, g) from entry (0, g): the bytes whose bit of s is set, negated. No byte of the codebook is zero, so
// (b ^ 0xFF) + 1 = 256 - b never carries into the next byte and the four bytes go in one xor and one add.
constexpr bool grid_bytes_nonzero() {
    for (int g = 0; g < 512; ++g)
        for (int j = 0; j < 4; ++j)
            if (((fnx_iq3s_grid_host[g] >> (8 * j)) & 255u) == 0) return false;
    return true;
}
static_assert(grid_bytes_nonzero(), "signed_entry() counts on it");
__device__ __forceinline__ uint32_t signed_entry(uint32_t g0, int s) {
    const uint32_t m = ((s & 1) ? 0xFFu : 0u) | ((s & 2) ? 0xFF00u : 0u) | ((s & 4) ? 0xFF0000u : 0u) | ((s & 8) ? 0xFF000000u : 0u);
    return (g0 ^ m) + (m & 0x01010101u);
}

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
    return __half2float(__ushort_as_half((unsigned short) h));
}
__device__ __forceinline__ unsigned short float_to_half_bits(float f) { return __half_as_ushort(__float2half_rn(f)); }

// xor-butterfly over `width` lanes (a power of two <= 64): every lane of a group ends with the group's sum.
// The order of the adds is part of the results' definition for the f32 mat-vec (the CPU oracle follows it).
template <int width>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int o = width / 2; o; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
template <int width>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
    for (int o = width / 2; o; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}

// kernels.cu:67-68 (sigm, silu_) over this library's exp (include/fnx_expf.h: fixed operation by operation, the CPU oracle
// includes the same lines), so that the q8_1 codes of h and the combine's gate come out bit for bit on both sides
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + fnx_expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + fnx_expf(-x)); }

// Sums over a weight row's lanes in the reference's order: lane l holds the terms of sub-block l of the row (for rows of 64
// sub-blocks: l and l + 32 are the two super-blocks a lane of the reference's 32 takes, kernels.cu:209-228, moe.cuh:664-670),
// and the lanes' sums meet in an xor butterfly width / 2, ..., 2, 1. Every add is of two partners' values, so it commutes:
// every lane of a group ends with the same bits, and they are the CPU oracle's.
// (The swaps are written as inline asm: with this toolchain the two results of the __builtin_amdgcn_permlane*_swap builtins
// were folded into one register when both fed the same add. The s_nop covers the VALU-write -> swap-read wait states.)
__device__ __forceinline__ float swap32_add(float x, float y) {   // lanes 0..31: x[l] + x[l + 32]; lanes 32..63: y[l - 32] + y[l]
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(x), "+v"(y));
    return x + y;
}
__device__ __forceinline__ float swap16_add(float x, float y) {   // 16-lane rows 0, 2: x's rows 0 + 1, 2 + 3; rows 1, 3: y's
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(x), "+v"(y));
    return x + y;
}
template <int width>
__device__ __forceinline__ float butterfly_sum(float v) {
#define FNX_DPP_ADD(ctrl) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, false))
    if constexpr (width >= 64) v = swap32_add(v, v);   // l ^ 32
    if constexpr (width >= 32) v = swap16_add(v, v);   // l ^ 16
    if constexpr (width >= 16) FNX_DPP_ADD(0x128);     // row_ror:8 = l ^ 8
    if constexpr (width >= 16) {
        FNX_DPP_ADD(0x124);   // row_ror:4: after the step before lanes l and l ^ 8 hold the same value, so lane (l + 4) mod 16 holds lane l ^ 4's
    } else if constexpr (width >= 8) {   // l ^ 4 without that symmetry: lanes 0-3 and 8-11 of a row look four up, the others four down
        int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x104, 0xF, 0x5, false);    // row_shl:4 into banks 0 and 2
        t = __builtin_amdgcn_update_dpp(t, __builtin_bit_cast(int, v), 0x114, 0xF, 0xA, false);        // row_shr:4 into banks 1 and 3
        v += __builtin_bit_cast(float, t);
    }
    if constexpr (width >= 4) FNX_DPP_ADD(0x4E);   // quad_perm [2,3,0,1] = l ^ 2
    if constexpr (width >= 2) FNX_DPP_ADD(0xB1);   // quad_perm [1,0,3,2] = l ^ 1
#undef FNX_DPP_ADD
    return v;
}

// A value every lane of the wave holds alike, moved to a scalar register: what is computed from it (addresses, loop
// bounds) then runs on the scalar unit. Loads from memory the kernel may also write are vector loads even at a uniform
// address, so job fields and table entries pass through here.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ const uint8_t* uniform_ptr(const uint8_t* p) {
    const uint64_t u = (uint64_t) (uintptr_t) p;
    const uint32_t lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) u);
    const uint32_t hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (u >> 32));
    return (const uint8_t*) (uintptr_t) ((uint64_t) hi << 32 | lo);
}

// global-memory byte pointer (address space 1): loads through it are global_load, never flat_load
typedef const __attribute__((address_space(1))) uint8_t* gbytes;
__device__ __forceinline__ gbytes as_global(const uint8_t* p) { return (gbytes) (uintptr_t) p; }

// little-endian loads from addresses that are only 2-byte aligned (IQ3_S blocks are 110 bytes)
__device__ __forceinline__ uint32_t load_u32_a2(const uint8_t* p) {
    uint32_t v;
    __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 4);
    return v;
}
__device__ __forceinline__ uint32_t load_u16(const uint8_t* p) {
    unsigned short v;
    __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 2);
    return v;
}

// 64 lanes x 16 bytes from base + each lane's byte offset straight into LDS, laid down in lane order from lds_at on (a
// wave-uniform LDS address, through M0). Written as an instruction so that the compiler, which cannot tell one LDS buffer
// of such loads from another, does not wait for every one of them before each LDS read: the kernel counts them itself
// (vmcnt) where it needs their data.
__device__ __forceinline__ void lds_load16(const void* base, uint32_t lane_offset, uint32_t lds_at) {
    // M0 is put back before the statement ends: the compiler keeps values of its own there (it does not accept M0 in a
    // clobber list); the load has taken its LDS address by then
    uint32_t m0_kept;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3\n\ts_mov_b32 m0, %0"
                 : "=&s"(m0_kept)
                 : "s"(lds_at), "v"(lane_offset), "s"(base)
                 : "memory");
}

}  // namespace fnx
