// Dequantization (ggml to_float) and the upload-time plane split for Q8_0 / Q6_K.
//
// Bit-exactness: every product and difference is a single IEEE fp32 operation in the order
// ggml's dequantize_row_* performs them -- (d*sc)*q - (dmin*m) for Q4_K, (d*sc)*q for Q6_K,
// q*d for Q8_0 -- written with __fmul_rn/__fsub_rn so the compiler cannot contract them to FMA.
#include "qproj_device.h"
#include "qproj_internal.h"

namespace qproj {

// one 256-thread block per super-block; thread t produces weight t
__global__ __launch_bounds__(256) void dequant_q4k_kernel(const uint8_t *__restrict__ blocks,
                                                          float *__restrict__ out, int64_t n_blocks) {
    const int64_t b = blockIdx.x;
    if (b >= n_blocks) return;
    const uint8_t *blk = blocks + b * 144;
    const uint32_t *hdr = reinterpret_cast<const uint32_t *>(blk);
    const int t = threadIdx.x;
    const int c = t >> 6;        // 64-weight chunk
    const int hi = (t >> 5) & 1; // high nibbles are the second 32 of the chunk
    const int l = t & 31;
    const int j = 2 * c + hi;    // sub-block
    const ScalesK4 s = unpack_scales_k4(hdr[1], hdr[2], hdr[3]);
    const float d = h2f(hdr[0]);
    const float dmin = h2f(hdr[0] >> 16);
    const float dj = __fmul_rn(d, (float)scale_k4(s, j));
    const float mj = __fmul_rn(dmin, (float)min_k4(s, j));
    const uint32_t byte = blk[16 + 32 * c + l];
    const uint32_t q = hi ? (byte >> 4) : (byte & 0xFu);
    out[b * 256 + t] = __fsub_rn(__fmul_rn(dj, (float)q), mj);
}

__global__ __launch_bounds__(256) void dequant_q6k_kernel(const uint8_t *__restrict__ ql,
                                                          const uint8_t *__restrict__ qh,
                                                          const int8_t *__restrict__ sc,
                                                          const uint16_t *__restrict__ dh,
                                                          float *__restrict__ out, int64_t n_blocks) {
    const int64_t b = blockIdx.x;
    if (b >= n_blocks) return;
    const int t = threadIdx.x;
    const int half = t >> 7;      // 128-weight half
    const int g = (t >> 5) & 3;   // 32-weight group inside the half
    const int l = t & 31;
    const uint32_t lo_byte = ql[b * 128 + 64 * half + 32 * (g & 1) + l];
    const uint32_t lo = (g & 2) ? (lo_byte >> 4) : (lo_byte & 0xFu);
    const uint32_t hb = (qh[b * 64 + 32 * half + l] >> (2 * g)) & 3u;
    const int q = (int)(lo | (hb << 4)) - 32;
    const int s = sc[b * 16 + 8 * half + 2 * g + (l >> 4)];
    const float d = h2f(dh[b]);
    out[b * 256 + t] = __fmul_rn(__fmul_rn(d, (float)s), (float)q);
}

__global__ __launch_bounds__(256) void dequant_q80_kernel(const int8_t *__restrict__ qs,
                                                          const uint16_t *__restrict__ dh,
                                                          float *__restrict__ out, int64_t n_elems) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n_elems) return;
    out[i] = __fmul_rn((float)qs[i], h2f(dh[i >> 5]));
}

hipError_t launch_dequantize(const WeightView &w, float *out, hipStream_t s) {
    const int64_t rows = w.N * w.E;
    const int64_t n_blocks = rows * w.nb;
    if (n_blocks == 0) return hipSuccess;
    if (n_blocks > 0x7fffffff) return hipErrorInvalidValue;
    switch (w.type) {
    case kTypeQ4_K:
        hipLaunchKernelGGL(dequant_q4k_kernel, dim3((unsigned)n_blocks), dim3(256), 0, s, w.q4k, out, n_blocks);
        break;
    case kTypeQ6_K:
        hipLaunchKernelGGL(dequant_q6k_kernel, dim3((unsigned)n_blocks), dim3(256), 0, s, w.q6_ql, w.q6_qh,
                           w.q6_sc, w.q6_d, out, n_blocks);
        break;
    case kTypeQ8_0: {
        const int64_t n = rows * w.K;
        hipLaunchKernelGGL(dequant_q80_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, w.q8_qs,
                           w.q8_d, out, n);
        break;
    }
    default:
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// Plane split.  GGUF blocks are read as 16-bit words (the only alignment GGUF guarantees for
// these two formats) and scattered to the planes; `to_gguf` runs the same mapping backwards.

template <bool TO_GGUF>
__global__ __launch_bounds__(256) void repack_q80_kernel(uint16_t *__restrict__ gguf, uint16_t *__restrict__ qs,
                                                         uint16_t *__restrict__ d, int64_t n_blocks) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // halfword index in GGUF
    if (i >= n_blocks * 17) return;
    const int64_t b = i / 17;
    const int j = (int)(i - b * 17);
    uint16_t *p = (j == 0) ? (d + b) : (qs + b * 16 + (j - 1));
    if (TO_GGUF)
        gguf[i] = *p;
    else
        *p = gguf[i];
}

template <bool TO_GGUF>
__global__ __launch_bounds__(256) void repack_q6k_kernel(uint16_t *__restrict__ gguf, uint16_t *__restrict__ ql,
                                                         uint16_t *__restrict__ qh, uint16_t *__restrict__ sc,
                                                         uint16_t *__restrict__ d, int64_t n_blocks) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n_blocks * 105) return;
    const int64_t b = i / 105;
    const int j = (int)(i - b * 105);
    uint16_t *p;
    if (j < 64)
        p = ql + b * 64 + j;
    else if (j < 96)
        p = qh + b * 32 + (j - 64);
    else if (j < 104)
        p = sc + b * 8 + (j - 96);
    else
        p = d + b;
    if (TO_GGUF)
        gguf[i] = *p;
    else
        *p = gguf[i];
}

template <bool TO_GGUF>
static hipError_t repack(int type, uint16_t *gguf, const WeightView &w, int64_t n_blocks, hipStream_t s) {
    if (n_blocks == 0) return hipSuccess;
    if (type == kTypeQ8_0) {
        const int64_t n = n_blocks * 17;
        hipLaunchKernelGGL(repack_q80_kernel<TO_GGUF>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, gguf,
                           (uint16_t *)w.q8_qs, (uint16_t *)w.q8_d, n_blocks);
    } else if (type == kTypeQ6_K) {
        const int64_t n = n_blocks * 105;
        hipLaunchKernelGGL(repack_q6k_kernel<TO_GGUF>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, gguf,
                           (uint16_t *)w.q6_ql, (uint16_t *)w.q6_qh, (uint16_t *)w.q6_sc, (uint16_t *)w.q6_d,
                           n_blocks);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_repack_to_planes(int type, const uint8_t *gguf, uint8_t *, const WeightView &w,
                                   int64_t n_blocks, hipStream_t s) {
    return repack<false>(type, (uint16_t *)gguf, w, n_blocks, s);
}

hipError_t launch_repack_to_gguf(int type, const WeightView &w, uint8_t *gguf, int64_t n_blocks, hipStream_t s) {
    return repack<true>(type, (uint16_t *)gguf, w, n_blocks, s);
}

}  // namespace qproj
