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

// Maximum over the aligned group of 8 lanes this lane belongs to, of unsigned words.
__device__ __forceinline__ uint32_t group8_max_u32(uint32_t v) {
    uint32_t o = dpp_move_u32<0xB1>(v);   // quad_perm [1,0,3,2]
    v = o > v ? o : v;
    o = dpp_move_u32<0x4E>(v);            // quad_perm [2,3,0,1]
    v = o > v ? o : v;
    o = dpp_move_u32<0x141>(v);           // row_half_mirror
    return o > v ? o : v;
}

typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));

// Larger of the two bf16 magnitudes in each half of a word (bit patterns with the sign cleared, compared
// as integers: for magnitudes that is the order of the values, with infinity above every finite value
// and every NaN above infinity).
__device__ __forceinline__ uint32_t pair_max_magnitude(uint32_t m, uint32_t packed) {
    const uint32_t a = packed & 0x7FFF7FFFu;
    const u16x2 r = __builtin_elementwise_max(__builtin_bit_cast(u16x2, m), __builtin_bit_cast(u16x2, a));
    return __builtin_bit_cast(uint32_t, r);
}

constexpr uint32_t kF32Inf = 0x7F800000u;
constexpr uint32_t kF32QuietNan = 0x7FC00000u;
constexpr uint32_t kAmaxFloorBits = 0x38D1B717u;   // 1e-4f

// fp8 e4m3 quantisation of 16 bf16 values that share one scale group with 7 other
// lanes.  Returns the packed codes; *scale_out is the group's scale.
//
// The group's largest magnitude is taken on the bit patterns, so that a NaN or an
// infinity among the 128 values is seen (a floating-point maximum drops NaNs).  A
// group with a non-finite value comes out as float arithmetic on it would, with one
// spelling of NaN: a NaN makes the scale NaN (0x7FC00000) and every code of the
// group the NaN code 0x7F; an infinity (and no NaN) makes the scale +infinity, the
// code of an infinite value 0x7F and the code of a finite value a zero with its sign.
// The rare case: a group that holds a NaN or an infinity (`top` = bits of its largest magnitude).
// Spelled out from the raw bf16 pairs, whatever the conversion instruction makes of NaN; kept out
// of line so that the ordinary path keeps its registers and its schedule.
__device__ __forceinline__ u32x4 quantize16_nonfinite(const u32x4 a, const u32x4 b, uint32_t top) {
    const bool has_nan = top > kF32Inf;
    u32x4 q;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        // elements 4j .. 4j+3 of the piece are the halves of two words: a[0], a[1] | a[2], a[3] | b[0], b[1] | b[2], b[3]
        const uint32_t w0 = j < 2 ? a[2 * j] : b[2 * j - 4];
        const uint32_t w1 = j < 2 ? a[2 * j + 1] : b[2 * j - 3];
        const uint32_t half[4] = {w0 & 0xFFFFu, w0 >> 16, w1 & 0xFFFFu, w1 >> 16};
        uint32_t w = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t code = has_nan || (half[i] & 0x7FFFu) == 0x7F80u ? 0x7Fu : half[i] >> 8 & 0x80u;
            w |= code << (8 * i);
        }
        q[j] = w;
    }
    return q;
}

__device__ __forceinline__ u32x4 quantize16(const u32x4 a, const u32x4 b, float *scale_out) {
    uint32_t mag = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        mag = pair_max_magnitude(mag, a[j]);
        mag = pair_max_magnitude(mag, b[j]);
    }
    const uint32_t lo = mag << 16, hi = mag & 0xFFFF0000u;
    const uint32_t top = group8_max_u32(lo > hi ? lo : hi);   // float bits of the group's largest magnitude
    if (__builtin_expect(top >= kF32Inf, 0)) {
        *scale_out = __uint_as_float(top > kF32Inf ? kF32QuietNan : kF32Inf);
        return quantize16_nonfinite(a, b, top);
    }
    float f[16];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f[2 * j] = __uint_as_float(a[j] << 16);
        f[2 * j + 1] = __uint_as_float(a[j] & 0xFFFF0000u);
        f[8 + 2 * j] = __uint_as_float(b[j] << 16);
        f[8 + 2 * j + 1] = __uint_as_float(b[j] & 0xFFFF0000u);
    }
    const float amax = __uint_as_float(top > kAmaxFloorBits ? top : kAmaxFloorBits);
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
