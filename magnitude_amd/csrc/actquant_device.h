// Wave-level activation quantizers shared by the stand-alone quantize kernels and by the
// projection kernels that quantize their activation row in the prologue.  A wave handles 256
// consecutive floats: lane l owns elements 4l..4l+3.  Bit-identical to ggml's scalar routines.
#pragma once

#include "qproj_device.h"
#include "qproj_internal.h"

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


// One wave quantizes 256 consecutive floats (lane l holds elements 4l..4l+3 in `v`) as ggml's block_q8_K and
// writes super-block `sb` of the planes qs, d, bsums (the min-term plane is made afterwards, row by row:
// minterm_rows_kernel)
__device__ __forceinline__ void wave_store_q8k(const float4 &v, int lane, int64_t sb, int8_t *__restrict__ qs,
                                               float *__restrict__ d, int16_t *__restrict__ bsums) {
    int bsum;
    float dd;
    const uint32_t packed = wave_quantize_q8k(v, lane, bsum, dd);
    reinterpret_cast<uint32_t *>(qs + sb * 256)[lane] = packed;
    if ((lane & 3) == 0) bsums[sb * 16 + (lane >> 2)] = (int16_t)bsum;
    if (lane == 0) d[sb] = dd;
}

// The per-32 formats: lane l's four floats belong to block (e0 >> 5) of the flattened input, e0 = the lane's
// first element.  FP16_SCALE: ggml Q8_0 blocks (scale rounded through fp16); otherwise fp32 scale and the integer
// sum of the block.  Every lane of the wave must call this (shuffles inside); `live` = the lane's elements exist.
template <bool FP16_SCALE>
__device__ __forceinline__ void wave_store_q8_32(const float4 &v, int lane, int64_t e0, bool live,
                                                 int8_t *__restrict__ qs, float *__restrict__ d,
                                                 int32_t *__restrict__ isum) {
    int s;
    float dd;
    const uint32_t packed = wave_quantize_q8_32(v, s, dd);
    if (!live) return;
    *reinterpret_cast<uint32_t *>(qs + e0) = packed;
    if ((lane & 7) == 0) {
        const int64_t b = e0 >> 5;
        d[b] = FP16_SCALE ? h2f(f2h(dd)) : dd;
        if (!FP16_SCALE) isum[b] = s;
    }
}

// The largest power of two not above v (v > 0 and normal), 1 for v = 0 or a subnormal.
__device__ __forceinline__ float pow2_floor(float v) {
    const uint32_t e = __float_as_uint(v) & 0x7f800000u;
    return e ? __uint_as_float(e) : 1.0f;
}

// ---- quantizer and min-term operand in one launch: a 16-wave workgroup owns an activation row.
// The waves quantize the row's super-blocks as above and also leave the row's scales (`ld`: nb, or 8 nb for the
// per-32 format) and sums of 32 codes (`ls`: [nb][8]) in LDS; row_minterm_finish then finds the row's normaliser
// and writes the min-term plane with the arithmetic of minterm_rows_kernel (the same bits as that launch).
constexpr int kRowWaves = 16, kRowThreads = 64 * kRowWaves;
__host__ __device__ constexpr size_t row_minterm_lds_bytes(bool per32, int nb) { return (size_t)nb * (per32 ? 16 : 9) * 4; }
constexpr size_t kRowLdsMax = 48 * 1024;   // rows beyond it (K > 196608 in the per-32 format) take the min-term launch

__device__ __forceinline__ void wave_store_q8k_row(const float4 &v, int lane, int64_t g, int sb, int8_t *__restrict__ qs,
                                                   float *__restrict__ d, int16_t *__restrict__ bsums, float *ld, int *ls) {
    int bsum;
    float dd;
    const uint32_t packed = wave_quantize_q8k(v, lane, bsum, dd);
    reinterpret_cast<uint32_t *>(qs + g * 256)[lane] = packed;
    if ((lane & 3) == 0) bsums[g * 16 + (lane >> 2)] = (int16_t)bsum;
    const int pair = bsum + __shfl_down(bsum, 4);   // two neighbouring groups of 16
    if ((lane & 7) == 0) ls[sb * 8 + (lane >> 3)] = pair;
    if (lane == 0) {
        d[g] = dd;
        ld[sb] = dd;
    }
}

__device__ __forceinline__ void wave_store_q8x32_row(const float4 &v, int lane, int64_t g, int sb, int8_t *__restrict__ qs,
                                                     float *__restrict__ d, int32_t *__restrict__ isum, float *ld, int *ls) {
    int sum;
    float dd;
    const uint32_t packed = wave_quantize_q8_32(v, sum, dd);
    reinterpret_cast<uint32_t *>(qs + g * 256)[lane] = packed;
    if ((lane & 7) == 0) {
        d[g * 8 + (lane >> 3)] = dd;
        isum[g * 8 + (lane >> 3)] = sum;
        ld[sb * 8 + (lane >> 3)] = dd;
        ls[sb * 8 + (lane >> 3)] = sum;
    }
}

// called by all kRowThreads threads of the workgroup after their stores into ld / ls; `wmax`: kRowWaves floats of LDS
template <bool PER32>
__device__ __forceinline__ void row_minterm_finish(const float *ld, const int *ls, int nb, int64_t m,
                                                   uint16_t *__restrict__ msum, float *__restrict__ rs, float *wmax) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nd = PER32 ? nb * 8 : nb;
    __syncthreads();
    float dmax = 0.f;
    for (int i = tid; i < nd; i += kRowThreads) dmax = fmaxf(dmax, fabsf(ld[i]));   // a Q8_K scale carries a sign
    dmax = wave_max(dmax);
    if (lane == 0) wmax[wave] = dmax;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kRowWaves; ++w) dmax = fmaxf(dmax, wmax[w]);
    const float r = pow2_floor(dmax), inv = 1.0f / r;   // exact: a power of two
    if (tid == 0) rs[m] = r;
    for (int sb = tid; sb < nb; sb += kRowThreads) {
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const float dd = PER32 ? ld[sb * 8 + t] : ld[sb];
            const float v = (dd * inv) * (float)ls[sb * 8 + t] * kMinPrescale;
            const _Float16 h = (_Float16)v, l = (_Float16)(v - (float)h);
            const uint32_t hb = __builtin_bit_cast(uint16_t, h), lb = __builtin_bit_cast(uint16_t, l);
            if (t & 1) {
                hi[t >> 1] |= hb << 16;
                lo[t >> 1] |= lb << 16;
            } else {
                hi[t >> 1] = hb;
                lo[t >> 1] = lb;
            }
        }
        uint4 *dst = reinterpret_cast<uint4 *>(msum + (m * nb + sb) * 16);
        dst[0] = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        dst[1] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    }
}

// Sum of squares of a row spread over a workgroup of 16 waves in ggml's precision (float products summed in
// double).  The order is fixed - lane's own pieces, butterfly over the wave, waves 0..15 - so that every
// kernel that normalises a row gets the same bits.  `partial` is 16 doubles of LDS; contains a barrier.
__device__ __forceinline__ double sum4_sq(const float4 &v) {
    return (double)(v.x * v.x) + (double)(v.y * v.y) + (double)(v.z * v.z) + (double)(v.w * v.w);
}
__device__ __forceinline__ double workgroup_sum16(double s, double *partial) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) s += __shfl_xor(s, d);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = s;
    __syncthreads();
    double total = 0.0;
#pragma unroll
    for (int w = 0; w < 16; ++w) total += partial[w];
    return total;
}

}  // namespace qproj
