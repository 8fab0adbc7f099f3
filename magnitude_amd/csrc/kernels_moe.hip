// Expert grouping for MUL_MAT_ID and the weighted combine of the MoE feed-forward.
#include "qproj_device.h"
#include "qproj_internal.h"

namespace qproj {

// Counting sort of (token, slot) pairs by expert id, one workgroup.  offsets[e]..offsets[e+1]
// indexes the pairs of expert e inside order[].  Ids outside [0, n_expert) raise *error_flag and
// their pairs are left out (their outputs are not written).  Pairs of one expert keep ascending
// pair order so repeated runs produce the same launch geometry.
__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t *__restrict__ ids, int n_pairs, int n_expert,
                                                         int32_t *__restrict__ order, int32_t *__restrict__ offsets,
                                                         int32_t *__restrict__ error_flag) {
    extern __shared__ int32_t cnt[];  // [n_expert + 1]
    const int tid = threadIdx.x;
    for (int e = tid; e <= n_expert; e += blockDim.x) cnt[e] = 0;
    __syncthreads();
    for (int p = tid; p < n_pairs; p += blockDim.x) {
        const int e = ids[p];
        if (e < 0 || e >= n_expert) {
            atomicOr(error_flag, 1);
        } else {
            atomicAdd(&cnt[e], 1);
        }
    }
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int e = 0; e < n_expert; ++e) {
            const int c = cnt[e];
            offsets[e] = run;
            cnt[e] = run;
            run += c;
        }
        offsets[n_expert] = run;
    }
    __syncthreads();
    // stable placement: thread e walks the pairs in order for its experts (n_pairs is small
    // next to the projections that follow)
    for (int e = tid; e < n_expert; e += blockDim.x) {
        const int begin = offsets[e], end = offsets[e + 1];
        if (begin == end) continue;
        int w = begin;
        for (int p = 0; p < n_pairs && w < end; ++p)
            if (ids[p] == e) order[w++] = p;
    }
}

hipError_t launch_moe_group(const int32_t *ids, int64_t n_pairs, int64_t n_expert, int32_t *order,
                            int32_t *offsets, int32_t *error_flag, hipStream_t s) {
    if (n_expert > 8192 || n_pairs > 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), (size_t)(n_expert + 1) * sizeof(int32_t), s, ids,
                       (int)n_pairs, (int)n_expert, order, offsets, error_flag);
    return hipGetLastError();
}

// y[b][c] = e[b][0][c]*w[b][0] + e[b][1][c]*w[b][1] + ... in slot order, each product rounded
// before it is added (llama.cpp multiplies by the routing weights, then adds the expert views
// one after the other).
__global__ __launch_bounds__(256) void moe_combine_kernel(const float *__restrict__ e, const float *__restrict__ w,
                                                          int64_t B, int n_used, int64_t N, float *__restrict__ y) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= B * N) return;
    const int64_t b = i / N, c = i - b * N;
    float s = __fmul_rn(e[(b * n_used) * N + c], w[b * n_used]);
    for (int j = 1; j < n_used; ++j) s = __fadd_rn(s, __fmul_rn(e[(b * n_used + j) * N + c], w[b * n_used + j]));
    y[i] = s;
}

hipError_t launch_moe_combine(const float *e, const float *weights, int64_t B, int64_t n_used, int64_t N,
                              float *y, hipStream_t s) {
    const int64_t n = B * N;
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, e, weights, B,
                       (int)n_used, N, y);
    return hipGetLastError();
}

}  // namespace qproj
