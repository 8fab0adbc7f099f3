// RMS normalisation with the norm weights, alone or fused with the activation quantizer.
//
// llama.cpp puts GGML_OP_RMS_NORM and GGML_OP_MUL (by the norm weights) in front of every attention and
// feed-forward block, and MUL_MAT then converts the result to the weights' vec_dot type: three passes over
// the activations.  Here one workgroup owns a row: its waves keep the row in registers (256 floats per wave
// and piece), the sum of squares is taken in double like ggml's ggml_float accumulator, and the normalised
// row is either stored (rms_norm) or quantized straight out of the registers into the activation planes
// the projection kernels read (rms_norm_quantize) - it never goes to memory as fp32.
//
//   sum = sum_k (double)(x[k]*x[k]);  scale = 1/sqrtf((float)(sum/K) + eps);  y[k] = (x[k]*scale)*gamma[k]
//
// Both roundings of y (scale, then weight) are kept so that the result equals the two ggml nodes run one
// after the other; only the order in which the double-precision sum is formed differs from a sequential loop.
#include "actquant_device.h"
#include "qproj_internal.h"

namespace qproj {

namespace {

constexpr int kNormWaves = 16, kNormThreads = 64 * kNormWaves;
constexpr int kHeld = 4;   // 256-float pieces a wave keeps in registers: rows up to 16384 floats are read once

// MODE 0: store fp32.  MODE 1: Q8_K planes.  MODE 2: ggml Q8_0 blocks.  MODE 3: per-32 prefill format.
// MT (modes 1 and 3): also the row normaliser and the min-term plane of the tiled Q4_K kernels, from scales and
// sums left in dynamic LDS (row_minterm_lds_bytes), so that no second launch goes over the row.
template <int MODE, bool MT>
__global__ __launch_bounds__(kNormThreads) void rms_norm_kernel(const float *__restrict__ x, const float *__restrict__ gamma,
                                                                float eps, int64_t K, float *__restrict__ y,
                                                                int8_t *__restrict__ qs, float *__restrict__ d,
                                                                int16_t *__restrict__ bsums, int32_t *__restrict__ isum,
                                                                uint16_t *__restrict__ msum, float *__restrict__ rs) {
    static_assert(kNormThreads == kRowThreads, "the row helpers assume this workgroup");
    extern __shared__ __align__(16) float row_lds[];
    __shared__ double partial[kNormWaves];
    __shared__ float wmax[kNormWaves];
    const int nb = (int)(K / 256);
    float *ld = row_lds;
    int *ls = reinterpret_cast<int *>(row_lds + (MODE == 3 ? nb * 8 : nb));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row = blockIdx.x;
    const float *xr = x + row * K;
    const int n_pieces = (int)((K + 255) / 256);   // K is a multiple of 32; the last piece may be short
    float4 held[kHeld];
    double s = 0.0;
#pragma unroll
    for (int i = 0; i < kHeld; ++i) {
        const int64_t e0 = (int64_t)(wave + kNormWaves * i) * 256 + 4 * lane;
        held[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (e0 < K) held[i] = *reinterpret_cast<const float4 *>(xr + e0);
        s += sum4_sq(held[i]);
    }
    for (int p = wave + kNormWaves * kHeld; p < n_pieces; p += kNormWaves) {   // rows longer than 16384
        const int64_t e0 = (int64_t)p * 256 + 4 * lane;
        if (e0 < K) {
            const float4 v = *reinterpret_cast<const float4 *>(xr + e0);
            s += sum4_sq(v);
        }
    }
    const double total = workgroup_sum16(s, partial);
    const float mean = (float)(total / (double)K);
    const float scale = 1.0f / sqrtf(mean + eps);

    for (int p = wave, i = 0; p < n_pieces; p += kNormWaves, ++i) {
        const int64_t e0 = (int64_t)p * 256 + 4 * lane;
        const bool live = e0 < K;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i < kHeld) {
            v = held[0];
#pragma unroll
            for (int q = 1; q < kHeld; ++q)
                if (i == q) v = held[q];
        } else if (live) {
            v = *reinterpret_cast<const float4 *>(xr + e0);
        }
        v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
        if (gamma && live) {
            const float4 g = *reinterpret_cast<const float4 *>(gamma + e0);
            v.x *= g.x; v.y *= g.y; v.z *= g.z; v.w *= g.w;
        }
        if (MODE == 0) {
            if (live) *reinterpret_cast<float4 *>(y + row * K + e0) = v;
        } else if (MODE == 1) {   // K is a multiple of 256 here: every piece is whole
            if constexpr (MT) wave_store_q8k_row(v, lane, row * nb + p, p, qs, d, bsums, ld, ls);
            else wave_store_q8k(v, lane, row * nb + p, qs, d, bsums);
        } else if (MODE == 3 && MT) {
            wave_store_q8x32_row(v, lane, row * nb + p, p, qs, d, isum, ld, ls);
        } else {
            // the planes are indexed by the flattened element: row * K is a multiple of 32
            wave_store_q8_32<MODE == 2>(v, lane, row * K + e0, live, qs, d, isum);
        }
    }
    if constexpr (MT) row_minterm_finish<MODE == 3>(ld, ls, nb, row, msum, rs, wmax);
}

}  // namespace

// y (fp32) when kind < 0, otherwise the activation planes of `kind` (msum / rs null: no min-term plane wanted)
hipError_t launch_rms_norm(int kind, const float *x, const float *gamma, float eps, int64_t M, int64_t K, float *y,
                           int8_t *qs, float *d, int16_t *bsums, uint16_t *msum, int32_t *isum, float *rs, hipStream_t s) {
    if (M == 0) return hipSuccess;
    if (K <= 0 || K % 32 != 0) return hipErrorInvalidValue;
    if ((kind == kActKindQ8_K || kind == kActKindQ8X32) && K % 256 != 0) return hipErrorInvalidValue;
    if (kind >= 0 && kind != kActKindQ8_K && kind != kActKindQ8_0 && kind != kActKindQ8X32) return hipErrorInvalidValue;
    if (dry_run()) {
        plan_note("rms_norm_kernel: %lld x %lld -> %s%s, grid %lld x %d", (long long)M, (long long)K,
                  kind < 0 ? "fp32 rows" : kind == kActKindQ8_K ? "Q8_K" : kind == kActKindQ8_0 ? "Q8_0 blocks" : "per-32 int8",
                  msum && rs ? " + min-term plane" : "", (long long)M, kNormThreads);
        return hipSuccess;
    }
    const dim3 grid((unsigned)M), block(kNormThreads);
    const bool mt = msum && rs && (kind == kActKindQ8_K || kind == kActKindQ8X32) &&
                    row_minterm_lds_bytes(kind == kActKindQ8X32, (int)(K / 256)) <= kRowLdsMax;
    if (kind < 0) hipLaunchKernelGGL((rms_norm_kernel<0, false>), grid, block, 0, s, x, gamma, eps, K, y, qs, d, bsums, isum, msum, rs);
    else if (kind == kActKindQ8_0) hipLaunchKernelGGL((rms_norm_kernel<2, false>), grid, block, 0, s, x, gamma, eps, K, y, qs, d, bsums, isum, msum, rs);
    else if (kind == kActKindQ8_K && mt)
        hipLaunchKernelGGL((rms_norm_kernel<1, true>), grid, block, row_minterm_lds_bytes(false, (int)(K / 256)), s, x, gamma, eps, K, y, qs, d, bsums, isum, msum, rs);
    else if (kind == kActKindQ8_K) hipLaunchKernelGGL((rms_norm_kernel<1, false>), grid, block, 0, s, x, gamma, eps, K, y, qs, d, bsums, isum, msum, rs);
    else if (mt)
        hipLaunchKernelGGL((rms_norm_kernel<3, true>), grid, block, row_minterm_lds_bytes(true, (int)(K / 256)), s, x, gamma, eps, K, y, qs, d, bsums, isum, msum, rs);
    else hipLaunchKernelGGL((rms_norm_kernel<3, false>), grid, block, 0, s, x, gamma, eps, K, y, qs, d, bsums, isum, msum, rs);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || kind < 0 || kind == kActKindQ8_0 || !msum || mt) return e;
    return launch_minterm_rows(kind, d, bsums, isum, M, K, msum, rs, s);
}

}  // namespace qproj
