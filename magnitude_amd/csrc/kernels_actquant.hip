// Activation quantizers (ggml from_float of the vec_dot_type, and the per-32 prefill format).
// One wave handles 256 consecutive floats of the flattened [M][K] input, so loads and stores
// are one 16-byte / 4-byte access per lane.
#include "actquant_device.h"
#include "qproj_internal.h"

namespace qproj {

// Every quantizer below takes an optional second input `u` of the same shape: the rows quantized are then
// silu(x) * u, the swiglu that joins the gate and up projections of a feed-forward block (the expression of
// swiglu_kernel, so the planes are the ones that kernel followed by the plain quantizer would write), and the
// intermediate rows never go to memory as fp32.
__device__ __forceinline__ float silu_mul(float x, float u) { return (x / (1.0f + expf(-x))) * u; }
__device__ __forceinline__ float4 load_rows4(const float *__restrict__ x, const float *__restrict__ u, int64_t e0) {
    float4 v = *reinterpret_cast<const float4 *>(x + e0);
    if (u) {   // uniform over the launch
        const float4 w = *reinterpret_cast<const float4 *>(u + e0);
        v.x = silu_mul(v.x, w.x); v.y = silu_mul(v.y, w.y); v.z = silu_mul(v.z, w.z); v.w = silu_mul(v.w, w.w);
    }
    return v;
}

// the launch's threads clear the job's rows between them, four floats a store
__device__ __forceinline__ void zero_rows(const ZeroJob &z) {
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, nthr = (int64_t)gridDim.x * blockDim.x;
    for (int i = 0; i < z.count; ++i)
        for (int64_t e = tid * 4; e < z.n[i]; e += nthr * 4)
            *reinterpret_cast<float4 *>(z.p[i] + e) = make_float4(0.f, 0.f, 0.f, 0.f);
}

__global__ __launch_bounds__(256) void quant_q8k_kernel(const float *__restrict__ x, const float *__restrict__ u, int64_t n_super,
                                                        int8_t *__restrict__ qs, float *__restrict__ d,
                                                        int16_t *__restrict__ bsums, const ZeroJob zero) {
    zero_rows(zero);
    const int64_t sb = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (sb >= n_super) return;  // whole wave leaves together
    const float4 v = load_rows4(x, u, sb * 256 + 4 * lane);
    wave_store_q8k(v, lane, sb, qs, d, bsums);
}

// FP16_SCALE: ggml Q8_0 blocks (scale rounded through fp16).  Otherwise the prefill format:
// fp32 scale plus the integer sum of the block.
template <bool FP16_SCALE>
__global__ __launch_bounds__(256) void quant_q8_32_kernel(const float *__restrict__ x, const float *__restrict__ u, int64_t n_chunks256,
                                                          int64_t n_elems, int8_t *__restrict__ qs,
                                                          float *__restrict__ d, int32_t *__restrict__ isum,
                                                          const ZeroJob zero) {
    zero_rows(zero);
    const int64_t ch = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (ch >= n_chunks256) return;
    const int64_t e0 = ch * 256 + 4 * lane;
    const bool live = e0 < n_elems;  // rows are multiples of 32, so a block is all in or all out
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live) v = load_rows4(x, u, e0);
    wave_store_q8_32<FP16_SCALE>(v, lane, e0, live, qs, d, isum);
}

// The min-term operand of the tiled Q4_K kernels, one wave per activation row, after the row's blocks are quantized.
// For every 32-wide sub-block the kernels want d * (sum of its 32 codes) as an fp16 high / low pair (22 bits).  fp16
// has a narrow range, so the values are normalised by the row: rs[m] = the largest power of two not above the
// row's largest block scale, and the pair holds (d / rs[m]) * sum / 16 -- at most 2 * 4064 / 16 whatever the size of
// the activations; a block far below the row's largest loses bits only where they no longer matter to the row.
// The kernels scale the activation scales by 1 / rs[m] and the result by 16 * rs[m], both exact.
// Per super-block: eight high parts, then eight low parts (the order the fp16 matrix instruction is fed).
// PER32: scales and sums per 32-block (d [K/32], isum [K/32]); otherwise per 256 (d [K/256], bsums [K/16]).
template <bool PER32>
__global__ __launch_bounds__(256) void minterm_rows_kernel(const float *__restrict__ d, const int16_t *__restrict__ bsums,
                                                           const int32_t *__restrict__ isum, int64_t M, int nb,
                                                           uint16_t *__restrict__ msum, float *__restrict__ rs) {
    const int64_t m = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (m >= M) return;   // whole wave leaves together
    const int nd = PER32 ? nb * 8 : nb;   // scales of the row
    const float *dr = d + m * nd;
    float dmax = 0.f;
    for (int i = lane; i < nd; i += 64) dmax = fmaxf(dmax, fabsf(dr[i]));   // a Q8_K scale carries a sign
    dmax = wave_max(dmax);
    const float r = pow2_floor(dmax), inv = 1.0f / r;   // exact: a power of two
    if (lane == 0) rs[m] = r;
    for (int sb = lane; sb < nb; sb += 64) {
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            float dd;
            int sum;
            if (PER32) {
                dd = dr[sb * 8 + t];
                sum = isum[(m * nb + sb) * 8 + t];
            } else {
                dd = dr[sb];
                const int16_t *b = bsums + (m * nb + sb) * 16 + 2 * t;
                sum = (int)b[0] + (int)b[1];
            }
            const float v = (dd * inv) * (float)sum * kMinPrescale;
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

// Quantizer and min-term operand in one launch: one 16-wave workgroup per activation row; a wave quantizes
// super-blocks wave, wave + 16, ... of the row.  Dynamic LDS: row_minterm_lds_bytes(PER32, nb).
template <bool PER32>
__global__ __launch_bounds__(kRowThreads) void quant_rows_minterm_kernel(const float *__restrict__ x, const float *__restrict__ u, int nb,
                                                                         int8_t *__restrict__ qs, float *__restrict__ d,
                                                                         int16_t *__restrict__ bsums,
                                                                         int32_t *__restrict__ isum,
                                                                         uint16_t *__restrict__ msum, float *__restrict__ rs,
                                                                         const ZeroJob zero) {
    zero_rows(zero);
    extern __shared__ __align__(16) float row_lds[];
    __shared__ float wmax[kRowWaves];
    float *ld = row_lds;
    int *ls = reinterpret_cast<int *>(row_lds + (PER32 ? nb * 8 : nb));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t m = blockIdx.x;
    for (int sb = wave; sb < nb; sb += kRowWaves) {
        const int64_t g = m * nb + sb;
        const float4 v = load_rows4(x, u, g * 256 + 4 * lane);
        if constexpr (PER32) wave_store_q8x32_row(v, lane, g, sb, qs, d, isum, ld, ls);
        else wave_store_q8k_row(v, lane, g, sb, qs, d, bsums, ld, ls);
    }
    row_minterm_finish<PER32>(ld, ls, nb, m, msum, rs, wmax);
}

hipError_t launch_minterm_rows(int kind, const float *d, const int16_t *bsums, const int32_t *isum, int64_t M, int64_t K,
                               uint16_t *msum, float *rs, hipStream_t s) {
    if (M == 0) return hipSuccess;
    if (K % 256 != 0 || !msum || !rs || (kind != kActKindQ8_K && kind != kActKindQ8X32)) return hipErrorInvalidValue;
    if (dry_run()) {
        plan_note("minterm_rows_kernel: min-term plane of %lld rows, grid %lld x 256", (long long)M, (long long)((M + 3) / 4));
        return hipSuccess;
    }
    const dim3 grid((unsigned)((M + 3) / 4)), block(256);
    if (kind == kActKindQ8_K)
        hipLaunchKernelGGL(minterm_rows_kernel<false>, grid, block, 0, s, d, bsums, isum, M, (int)(K / 256), msum, rs);
    else
        hipLaunchKernelGGL(minterm_rows_kernel<true>, grid, block, 0, s, d, bsums, isum, M, (int)(K / 256), msum, rs);
    return hipGetLastError();
}

// msum / rs null: the min-term plane is not wanted (the decode, small-batch and expert-grouped kernels take the block
// sums themselves)
hipError_t launch_quantize_act(int kind, const float *x, int64_t M, int64_t K, int8_t *qs, float *d,
                               int16_t *bsums, uint16_t *msum, int32_t *isum, float *rs, hipStream_t s, const float *u,
                               const ZeroJob *zero) {
    const int64_t n = M * K;
    if (n == 0) return hipSuccess;
    if (kind != kActKindQ8_K && kind != kActKindQ8_0 && kind != kActKindQ8X32) return hipErrorInvalidValue;
    ZeroJob zj{};
    if (zero) {
        zj = *zero;
        for (int i = 0; i < zj.count; ++i)
            if (zj.n[i] % 4 != 0 || (reinterpret_cast<uintptr_t>(zj.p[i]) & 15) != 0) return hipErrorInvalidValue;
    }
    if (dry_run()) {
        plan_note("quantizer: %lld x %lld -> %s%s%s%s", (long long)M, (long long)K,
                  kind == kActKindQ8_K ? "Q8_K" : kind == kActKindQ8_0 ? "Q8_0 blocks" : "per-32 int8",
                  msum && rs ? " + min-term plane" : "", u ? ", rows = silu(x) * u" : "",
                  zj.count ? ", clears the output rows of a projection that adds its two K parts" : "");
        return hipSuccess;
    }
    // with the min-term plane wanted: one launch, a workgroup per row (measured against the quantizer followed by
    // the min-term launch: 4.6 against 7.1 us at 128 x 4096, 9.3 against 10.6 at 512 x 14336; many short rows are
    // the exception, 22.8 against 18.8 us at 4096 x 4096, where a workgroup has one chunk a wave and two barriers)
    static const int rows_max_short = tuning_int("QPROJ_ROW_QUANT_MAX_M", 1024);
    if (msum && rs && kind != kActKindQ8_0 && K % 256 == 0 && row_minterm_lds_bytes(kind == kActKindQ8X32, (int)(K / 256)) <= kRowLdsMax &&
        (K / 256 >= 32 || M <= rows_max_short)) {
        const int nb = (int)(K / 256);
        const dim3 rgrid((unsigned)M), rblock(kRowThreads);
        if (kind == kActKindQ8_K)
            hipLaunchKernelGGL(quant_rows_minterm_kernel<false>, rgrid, rblock, row_minterm_lds_bytes(false, nb), s, x, u, nb, qs, d, bsums, isum, msum, rs, zj);
        else
            hipLaunchKernelGGL(quant_rows_minterm_kernel<true>, rgrid, rblock, row_minterm_lds_bytes(true, nb), s, x, u, nb, qs, d, bsums, isum, msum, rs, zj);
        return hipGetLastError();
    }
    const int64_t chunks = (n + 255) / 256;
    const dim3 grid((unsigned)((chunks + 3) / 4)), block(256);
    if (kind == kActKindQ8_K) {
        hipLaunchKernelGGL(quant_q8k_kernel, grid, block, 0, s, x, u, n / 256, qs, d, bsums, zj);
    } else if (kind == kActKindQ8_0) {
        hipLaunchKernelGGL(quant_q8_32_kernel<true>, grid, block, 0, s, x, u, chunks, n, qs, d, isum, zj);
    } else {
        hipLaunchKernelGGL(quant_q8_32_kernel<false>, grid, block, 0, s, x, u, chunks, n, qs, d, isum, zj);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || kind == kActKindQ8_0 || !msum) return e;
    return launch_minterm_rows(kind, d, bsums, isum, M, K, msum, rs, s);
}

}  // namespace qproj
