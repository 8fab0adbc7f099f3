// Wave-level activation quantizers shared by the stand-alone quantize kernels and by the
// projection kernels that quantize their activation row in the prologue.  A wave handles 256
// consecutive floats: lane l owns elements 4l..4l+3.  Bit-identical to ggml's scalar routines.
#pragma once

#include "qproj_device.h"

namespace qproj {

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) |
           ((uint32_t)(d & 0xff) << 24);
}

template <int CTRL>
__device__ __forceinline__ int dpp_move_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}

// max over the 64 lanes (all active), result in every lane
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));
    v = fmaxf(v, dpp_move<0x4E>(v));
    v = fmaxf(v, dpp_move<0x141>(v));
    v = fmaxf(v, dpp_move<0x140>(v));
    const int b = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// quantize_row_q8_K on one super-block.  Returns the lane's 4 packed int8; `bsum` is the sum of
// the 16-element group the lane belongs to (same value on its 4 lanes); `d` is the block scale.
__device__ __forceinline__ uint32_t wave_quantize_q8k(const float4 v, int lane, int &bsum, float &d) {
    const float e[4] = {v.x, v.y, v.z, v.w};
    const float a[4] = {fabsf(v.x), fabsf(v.y), fabsf(v.z), fabsf(v.w)};
    const float amax = wave_max(fmaxf(fmaxf(a[0], a[1]), fmaxf(a[2], a[3])));
    // ggml keeps the FIRST element whose magnitude is the largest: lowest lane that holds it,
    // lowest element inside that lane
    float cand = e[3];
    if (a[2] == amax) cand = e[2];
    if (a[1] == amax) cand = e[1];
    if (a[0] == amax) cand = e[0];
    const bool has = (a[0] == amax) | (a[1] == amax) | (a[2] == amax) | (a[3] == amax);
    const unsigned long long mask = __ballot(has);
    const int first = mask ? (int)__ffsll((long long)mask) - 1 : 0;
    const float mx = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cand), first));
    (void)lane;
    uint32_t packed = 0;
    int s = 0;
    d = 0.f;
    if (amax != 0.f) {
        const float iscale = -127.f / mx;
        int q[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = nearest_int(__fmul_rn(iscale, e[i]));
            q[i] = r < 127 ? r : 127;
            s += q[i];
        }
        packed = pack4(q[0], q[1], q[2], q[3]);
        d = 1.f / iscale;
    }
    s += dpp_move_i<0xB1>(s);
    s += dpp_move_i<0x4E>(s);
    bsum = s;
    return packed;
}

// quantize_row_q8_0_ref arithmetic on the 32-block the lane belongs to (8 lanes per block):
// d = amax/127, q = roundf(x * (1/d)).  `isum` is the block's integer sum, `d` the fp32 scale
// before any fp16 rounding.
__device__ __forceinline__ uint32_t wave_quantize_q8_32(const float4 v, int &isum, float &d) {
    const float e[4] = {v.x, v.y, v.z, v.w};
    float amax = fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3])));
    amax = fmaxf(amax, dpp_move<0xB1>(amax));
    amax = fmaxf(amax, dpp_move<0x4E>(amax));
    amax = fmaxf(amax, dpp_move<0x141>(amax));  // row_half_mirror: the other quad of the 8 lanes
    d = amax / 127.f;
    const float id = d != 0.f ? 1.0f / d : 0.0f;
    int q[4];
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        q[i] = (int)roundf(__fmul_rn(e[i], id));
        s += q[i];
    }
    s += dpp_move_i<0xB1>(s);
    s += dpp_move_i<0x4E>(s);
    s += dpp_move_i<0x141>(s);
    isum = s;
    return pack4(q[0], q[1], q[2], q[3]);
}

}  // namespace qproj
