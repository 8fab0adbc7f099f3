// Device-side helpers shared by the qproj kernels (gfx950, wave64).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qproj {

// fp16 bits -> fp32, exact for every finite half including subnormals (v_cvt_f32_f16).
__device__ __forceinline__ float h2f(uint32_t h) {
    return __half2float(__ushort_as_half((unsigned short)(h & 0xffffu)));
}

// fp32 -> fp16 bits, round to nearest even (v_cvt_f16_f32).
__device__ __forceinline__ uint16_t f2h(float f) { return __half_as_ushort(__float2half_rn(f)); }

// 4-way signed int8 dot product with int32 accumulate (v_dot4_i32_i8).
__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// Sum over the 64 lanes of a wave; every lane must be active.  Four DPP steps give each row of
// 16 lanes its row sum, the four row sums are then read through SGPRs.  All lanes get the total.
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_move<0x141>(v);  // row_half_mirror
    v += dpp_move<0x140>(v);  // row_mirror
    const int b = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
    return (r0 + r1) + (r2 + r3);
}

// Sums of FOUR per-lane values at once, "transposed": after the call, lane 12 + i of every row of
// 16 lanes holds the 64-lane sum of v[i].  The first two steps fold pairs of values into
// alternating lanes, so the whole thing costs about as much as one and a half plain reductions.
__device__ __forceinline__ float wave_sum4(const float (&v)[4], int lane) {
    const bool odd = lane & 1, hi2 = lane & 2;
    // lanes xor 1: even lanes collect v0 / v2, odd lanes collect v1 / v3
    const float s01 = (odd ? v[1] : v[0]) + dpp_move<0xB1>(odd ? v[0] : v[1]);
    const float s23 = (odd ? v[3] : v[2]) + dpp_move<0xB1>(odd ? v[2] : v[3]);
    // lanes xor 2: lane & 3 == i now collects v[i] over its quad
    float t = (hi2 ? s23 : s01) + dpp_move<0x4E>(hi2 ? s01 : s23);
    t += dpp_move<0x114>(t);  // row_shr:4
    t += dpp_move<0x118>(t);  // row_shr:8  -> lanes 12..15 of each row hold the row's sums
    t += __shfl_xor(t, 16);
    t += __shfl_xor(t, 32);
    return t;
}

// The 6-bit (scale, min) pairs of a Q4_K super-block, unpacked four at a time from the 12-byte
// field (three dwords s0, s1, s2).  Byte j of `sc_lo`/`mn_lo` is sub-block j (0..3); byte j of
// `sc_hi`/`mn_hi` is sub-block 4+j.
struct ScalesK4 {
    uint32_t sc_lo, mn_lo, sc_hi, mn_hi;
};

__device__ __forceinline__ ScalesK4 unpack_scales_k4(uint32_t s0, uint32_t s1, uint32_t s2) {
    ScalesK4 r;
    r.sc_lo = s0 & 0x3f3f3f3fu;
    r.mn_lo = s1 & 0x3f3f3f3fu;
    r.sc_hi = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
    r.mn_hi = ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u);
    return r;
}

// scale / min of sub-block j (0..7)
__device__ __forceinline__ uint32_t scale_k4(const ScalesK4 &s, int j) {
    const uint32_t w = j < 4 ? s.sc_lo : s.sc_hi;
    return (w >> (8 * (j & 3))) & 0xffu;
}
__device__ __forceinline__ uint32_t min_k4(const ScalesK4 &s, int j) {
    const uint32_t w = j < 4 ? s.mn_lo : s.mn_hi;
    return (w >> (8 * (j & 3))) & 0xffu;
}

// ggml nearest_int: round half to even through the 2^23 + 2^22 addend.
__device__ __forceinline__ int nearest_int(float f) {
    const float v = __fadd_rn(f, 12582912.f);
    return (__float_as_int(v) & 0x007fffff) - 0x00400000;
}

}  // namespace qproj
