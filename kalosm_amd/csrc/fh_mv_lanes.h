// Lane-level helpers shared by the single-row MFMA matvec kernels (Q4_K, Q6_K).
#pragma once
#include "fh_internal.h"

// Cross-lane moves inside a row of 16 lanes as DPP modifiers (one VALU op, no LDS round trip).
#define DPP_XOR1 0xB1        // quad_perm [1,0,3,2]
#define DPP_XOR2 0x4E        // quad_perm [2,3,0,1]
#define DPP_HALF_MIRROR 0x141 // lane i <- lane 7-i within each group of 8
#define DPP_ROW_MIRROR 0x140  // lane i <- lane 15-i within each row of 16
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xF, 0xF, true));
}

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, CTRL, 0xF, 0xF, true);
}
// sum over the four rows of 16 lanes of a wavefront (lane i of every row gets it): two register swaps, no LDS
__device__ __forceinline__ float rows_sum(float a) {
    const uint32_t u = __float_as_uint(a);
    auto s16 = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = __uint_as_float(s16[0]) + __uint_as_float(s16[1]);
    const uint32_t w = __float_as_uint(a);
    auto s32 = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return __uint_as_float(s32[0]) + __uint_as_float(s32[1]);
}
// LDS addresses as 32-bit integers, so that a per-lane choice between two of them is one v_cndmask on a constant
// lane mask held in scalar registers.
__device__ __forceinline__ uint32_t lds_addr(const void *p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
}
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 lds_read16(uint32_t a) {
    const u32x4 v = *(__attribute__((address_space(3))) const u32x4 *)(uintptr_t)a;
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint32_t sel_lanes(uint64_t mask, uint32_t yes, uint32_t no) {
    uint32_t r;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(r) : "v"(no), "v"(yes), "s"(mask));
    return r;
}

