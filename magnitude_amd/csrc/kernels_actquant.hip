// Activation quantizers (ggml from_float of the vec_dot_type, and the per-32 prefill format).
// One wave handles 256 consecutive floats of the flattened [M][K] input, so loads and stores
// are one 16-byte / 4-byte access per lane.
#include "actquant_device.h"
#include "qproj_internal.h"

namespace qproj {

__global__ __launch_bounds__(256) void quant_q8k_kernel(const float *__restrict__ x, int64_t n_super,
                                                        int8_t *__restrict__ qs, float *__restrict__ d,
                                                        int16_t *__restrict__ bsums, uint16_t *__restrict__ msum) {
    const int64_t sb = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (sb >= n_super) return;  // whole wave leaves together
    const float4 v = reinterpret_cast<const float4 *>(x + sb * 256)[lane];
    wave_store_q8k(v, lane, sb, qs, d, bsums, msum);
}

// FP16_SCALE: ggml Q8_0 blocks (scale rounded through fp16).  Otherwise the prefill format:
// fp32 scale plus the integer sum of the block.
template <bool FP16_SCALE>
__global__ __launch_bounds__(256) void quant_q8_32_kernel(const float *__restrict__ x, int64_t n_chunks256,
                                                          int64_t n_elems, int8_t *__restrict__ qs,
                                                          float *__restrict__ d, int32_t *__restrict__ isum,
                                                          uint16_t *__restrict__ msum) {
    const int64_t ch = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (ch >= n_chunks256) return;
    const int64_t e0 = ch * 256 + 4 * lane;
    const bool live = e0 < n_elems;  // rows are multiples of 32, so a block is all in or all out
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live) v = *reinterpret_cast<const float4 *>(x + e0);
    wave_store_q8_32<FP16_SCALE>(v, lane, e0, ch, live, qs, d, isum, msum);
}

hipError_t launch_quantize_act(int kind, const float *x, int64_t M, int64_t K, int8_t *qs, float *d,
                               int16_t *bsums, uint16_t *msum, int32_t *isum, hipStream_t s) {
    const int64_t n = M * K;
    if (n == 0) return hipSuccess;
    if (dry_run()) return kind == kActKindQ8_K || kind == kActKindQ8_0 || kind == kActKindQ8X32 ? hipSuccess : hipErrorInvalidValue;
    const int64_t chunks = (n + 255) / 256;
    const dim3 grid((unsigned)((chunks + 3) / 4)), block(256);
    if (kind == kActKindQ8_K) {
        hipLaunchKernelGGL(quant_q8k_kernel, grid, block, 0, s, x, n / 256, qs, d, bsums, msum);
    } else if (kind == kActKindQ8_0) {
        hipLaunchKernelGGL(quant_q8_32_kernel<true>, grid, block, 0, s, x, chunks, n, qs, d, isum, msum);
    } else if (kind == kActKindQ8X32) {
        hipLaunchKernelGGL(quant_q8_32_kernel<false>, grid, block, 0, s, x, chunks, n, qs, d, isum, msum);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace qproj
