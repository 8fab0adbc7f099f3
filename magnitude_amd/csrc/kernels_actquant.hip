// Activation quantizers (ggml from_float of the vec_dot_type, and the per-32 prefill format).
//
// One wave handles 256 consecutive floats of one row: lane l owns elements 4l..4l+3, so loads
// and stores are one 16-byte / 4-byte access per lane.  Results are bit-identical to the scalar
// ggml routines: the same fp32 operations in the same order per element, and the max search
// keeps ggml's "first element with the strictly largest magnitude" rule.
#include "qproj_device.h"
#include "qproj_internal.h"

namespace qproj {

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) |
           ((uint32_t)(d & 0xff) << 24);
}

// quantize_row_q8_K: per 256, iscale = -127/max (max = signed value of the largest magnitude),
// q = min(127, nearest_int(iscale*x)), bsums over 16, d = 1/iscale.
__global__ __launch_bounds__(256) void quant_q8k_kernel(const float *__restrict__ x, int64_t n_super,
                                                        int8_t *__restrict__ qs, float *__restrict__ d,
                                                        int16_t *__restrict__ bsums) {
    const int64_t sb = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (sb >= n_super) return;  // whole wave leaves together
    const float4 v = reinterpret_cast<const float4 *>(x + sb * 256)[lane];
    const float e[4] = {v.x, v.y, v.z, v.w};
    float amax = 0.f, mx = 0.f;
    int idx = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float ax = fabsf(e[i]);
        if (ax > amax) {
            amax = ax;
            mx = e[i];
            idx = 4 * lane + i;
        }
    }
    if (amax == 0.f) idx = 4 * lane;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float oa = __shfl_xor(amax, off);
        const float om = __shfl_xor(mx, off);
        const int oi = __shfl_xor(idx, off);
        if (oa > amax || (oa == amax && oi < idx)) {
            amax = oa;
            mx = om;
            idx = oi;
        }
    }
    uint32_t packed = 0;
    int s = 0;
    float dd = 0.f;
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
        dd = 1.f / iscale;
    }
    reinterpret_cast<uint32_t *>(qs + sb * 256)[lane] = packed;
    s += __shfl_xor(s, 1);
    s += __shfl_xor(s, 2);
    if ((lane & 3) == 0) bsums[sb * 16 + (lane >> 2)] = (int16_t)s;
    if (lane == 0) d[sb] = dd;
}

// quantize_row_q8_0_ref (FP16_SCALE) and the per-32 prefill format (fp32 scale + integer sum):
// per 32, d = amax/127, id = d ? 1/d : 0, q = roundf(x*id).
template <bool FP16_SCALE>
__global__ __launch_bounds__(256) void quant_q8_32_kernel(const float *__restrict__ x, int64_t n_chunks256,
                                                          int64_t n_elems, int8_t *__restrict__ qs,
                                                          float *__restrict__ d, int32_t *__restrict__ isum) {
    const int64_t ch = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (ch >= n_chunks256) return;
    const int64_t e0 = ch * 256 + 4 * lane;
    const bool live = e0 < n_elems;  // rows are multiples of 32, so a lane is all in or all out
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live) v = *reinterpret_cast<const float4 *>(x + e0);
    const float e[4] = {v.x, v.y, v.z, v.w};
    float amax = fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3])));
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    amax = fmaxf(amax, __shfl_xor(amax, 2));
    amax = fmaxf(amax, __shfl_xor(amax, 4));
    const float dd = amax / 127.f;
    const float id = dd != 0.f ? 1.0f / dd : 0.0f;
    int q[4];
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        q[i] = (int)roundf(__fmul_rn(e[i], id));
        s += q[i];
    }
    s += __shfl_xor(s, 1);
    s += __shfl_xor(s, 2);
    s += __shfl_xor(s, 4);
    if (!live) return;
    *reinterpret_cast<uint32_t *>(qs + e0) = pack4(q[0], q[1], q[2], q[3]);
    if ((lane & 7) == 0) {
        const int64_t b = e0 >> 5;
        d[b] = FP16_SCALE ? h2f(f2h(dd)) : dd;
        if (!FP16_SCALE) isum[b] = s;
    }
}

hipError_t launch_quantize_act(int kind, const float *x, int64_t M, int64_t K, int8_t *qs, float *d,
                               int16_t *bsums, int32_t *isum, hipStream_t s) {
    const int64_t n = M * K;
    if (n == 0) return hipSuccess;
    const int64_t chunks = (n + 255) / 256;
    const dim3 grid((unsigned)((chunks + 3) / 4)), block(256);
    if (kind == kActKindQ8_K) {
        hipLaunchKernelGGL(quant_q8k_kernel, grid, block, 0, s, x, n / 256, qs, d, bsums);
    } else if (kind == kActKindQ8_0) {
        hipLaunchKernelGGL(quant_q8_32_kernel<true>, grid, block, 0, s, x, chunks, n, qs, d, isum);
    } else if (kind == kActKindQ8X32) {
        hipLaunchKernelGGL(quant_q8_32_kernel<false>, grid, block, 0, s, x, chunks, n, qs, d, isum);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace qproj
