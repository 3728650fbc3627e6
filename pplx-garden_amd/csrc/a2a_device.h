// Device helpers shared by the dispatch kernels: DPP group reductions, lane
// broadcasts and the fp8 e4m3 block quantiser.
#pragma once

#include "a2a_internal.h"

namespace a2a {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// A barrier for data that wavefronts of a workgroup hand to each other through LDS: it waits for this
// wavefront's LDS operations only.  Loads from memory that were asked for earlier stay in flight across
// it (in front of its own barrier the compiler may wait for every outstanding access to memory).
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(
        __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// Maximum over the aligned group of 8 lanes this lane belongs to.
__device__ __forceinline__ float group8_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_move<0x141>(v));  // row_half_mirror
    return v;
}

// Sum over the aligned group of 8 lanes this lane belongs to (every lane gets it).
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_move_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}

__device__ __forceinline__ uint32_t group8_sum(uint32_t v) {
    v += dpp_move_u32<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_move_u32<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_move_u32<0x141>(v);  // row_half_mirror
    return v;
}

__device__ __forceinline__ uint64_t read_lane64(uint64_t v, uint32_t lane) {
    const uint32_t lo = __builtin_amdgcn_readlane((int)(uint32_t)v, (int)lane);
    const uint32_t hi = __builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), (int)lane);
    return ((uint64_t)hi << 32) | lo;
}

// fp8 e4m3 quantisation of 16 floats that share one scale group with 7 other
// lanes.  Returns the packed codes; *scale_out is the group's scale.
__device__ __forceinline__ u32x4 quantize16(const u32x4 a, const u32x4 b, float *scale_out) {
    float f[16];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f[2 * j] = __uint_as_float(a[j] << 16);
        f[2 * j + 1] = __uint_as_float(a[j] & 0xFFFF0000u);
        f[8 + 2 * j] = __uint_as_float(b[j] << 16);
        f[8 + 2 * j + 1] = __uint_as_float(b[j] & 0xFFFF0000u);
    }
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fabsf(f[j]));
    amax = fmaxf(group8_max(amax), 1e-4f);
    const float inv = 448.0f / amax;   // correctly rounded division
    *scale_out = amax / 448.0f;
    u32x4 q;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[i] = __builtin_amdgcn_fmed3f(f[4 * j + i] * inv, -448.0f, 448.0f);
        }
        int w = 0;
        w = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], w, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], w, true);
        q[j] = (uint32_t)w;
    }
    return q;
}

}  // namespace a2a
