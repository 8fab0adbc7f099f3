// Expert grouping for MUL_MAT_ID and the weighted combine of the MoE feed-forward.
#include "qproj_device.h"
#include "qproj_internal.h"

namespace qproj {

// Counting sort of (token, slot) pairs by expert id, one workgroup.  offsets[e]..offsets[e+1]
// indexes the pairs of expert e inside order[]; active[0..active[n_expert]) lists the experts that
// have pairs, ascending.  Ids outside [0, n_expert) raise *error_flag and
// their pairs are left out (their outputs are not written).  Pairs of one expert keep ascending
// pair order so repeated runs produce the same launch geometry: the pair list is cut into S
// segments, (expert, segment) tasks count their matches, a prefix over segments gives every task
// its first slot, and a second scan places the pairs.
constexpr int kGroupThreads = 1024;
constexpr int kGroupLdsIds = 8192;   // pair ids staged in LDS up to this many, read from global beyond

__global__ __launch_bounds__(kGroupThreads) void moe_group_kernel(const int32_t *__restrict__ ids, int n_pairs,
                                                                  int n_expert, int S, int32_t *__restrict__ order,
                                                                  int32_t *__restrict__ offsets,
                                                                  int32_t *__restrict__ active,
                                                                  int32_t *__restrict__ error_flag) {
    extern __shared__ int32_t lds[];
    int32_t *segcnt = lds;                     // [n_expert * S], then turned into first slots
    int32_t *first = lds + n_expert * S;       // [n_expert + 1]
    int32_t *wsum = first + n_expert + 1;      // [32] wave totals of the two scans
    int32_t *sid = wsum + 32;                  // [min(n_pairs, kGroupLdsIds)]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool staged = n_pairs <= kGroupLdsIds;
    bool bad = false;
    for (int p = tid; p < n_pairs; p += kGroupThreads) {
        const int e = ids[p];
        bad |= e < 0 || e >= n_expert;
        if (staged) sid[p] = e;
    }
    if (bad) atomicOr(error_flag, 1);
    __syncthreads();
    const int32_t *src = staged ? sid : ids;
    const int seg_len = (n_pairs + S - 1) / S;
    const int n_tasks = n_expert * S;
    // pass 1: matches of (expert, segment); eight independent reads in flight per step
    for (int t = tid; t < n_tasks; t += kGroupThreads) {
        const int e = t / S, sg = t - e * S;
        const int lo = min(sg * seg_len, n_pairs), hi = min(lo + seg_len, n_pairs);
        int c = 0;
        for (int p = lo; p < hi; p += 8) {
            int v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = src[min(p + u, hi - 1)];
#pragma unroll
            for (int u = 0; u < 8; ++u) c += (p + u < hi) & (v[u] == e);
        }
        segcnt[t] = c;
    }
    __syncthreads();
    // segment counts -> running starts inside the expert; thread t owns experts [t * per, t * per + per)
    const int per = (n_expert + kGroupThreads - 1) / kGroupThreads;
    int tot[8], local = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int e = tid * per + i;
        tot[i] = 0;
        if (i < per && e < n_expert) {
            int run = 0;
            for (int sg = 0; sg < S; ++sg) {
                const int c = segcnt[e * S + sg];
                segcnt[e * S + sg] = run;
                run += c;
            }
            tot[i] = run;
        }
        local += tot[i];
    }
    // exclusive scans over the workgroup (shuffles inside a wave, wave totals through LDS) of the pair
    // counts (-> offsets) and of the non-empty flags (-> compact list of the experts that have work)
    int local_f = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) local_f += tot[i] > 0;
    int incl = local, incl_f = local_f;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d), up_f = __shfl_up(incl_f, d);
        if (lane >= d) {
            incl += up;
            incl_f += up_f;
        }
    }
    if (lane == 63) {
        wsum[wave] = incl;
        wsum[16 + wave] = incl_f;
    }
    __syncthreads();
    int before = incl - local, before_f = incl_f - local_f;
    for (int w = 0; w < wave; ++w) {
        before += wsum[w];
        before_f += wsum[16 + w];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int e = tid * per + i;
        if (i < per && e < n_expert) {
            first[e] = before;
            offsets[e] = before;
            before += tot[i];
            if (tot[i] > 0) active[before_f++] = e;
        }
    }
    if (tid == kGroupThreads - 1) {
        offsets[n_expert] = before;
        active[n_expert] = before_f;   // how many experts have pairs
    }
    __syncthreads();
    // pass 2: placement, ascending pair order inside every expert
    for (int t = tid; t < n_tasks; t += kGroupThreads) {
        const int e = t / S, sg = t - e * S;
        const int lo = min(sg * seg_len, n_pairs), hi = min(lo + seg_len, n_pairs);
        int w = first[e] + segcnt[t];
        for (int p = lo; p < hi; p += 8) {
            int v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = src[min(p + u, hi - 1)];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (p + u < hi && v[u] == e) order[w++] = p + u;
        }
    }
}

hipError_t launch_moe_group(const int32_t *ids, int64_t n_pairs, int64_t n_expert, int32_t *order,
                            int32_t *offsets, int32_t *active, int32_t *error_flag, hipStream_t s) {
    if (n_expert > 8192 || n_pairs > 0x7fffffff) return hipErrorInvalidValue;
    int S = (int)(kGroupThreads / n_expert);
    if (S < 1) S = 1;
    if (S > n_pairs) S = (int)(n_pairs > 0 ? n_pairs : 1);
    const size_t lds = ((size_t)n_expert * S + n_expert + 1 + 32 + (n_pairs <= kGroupLdsIds ? n_pairs : 0)) * sizeof(int32_t);
    static size_t allowed = 48 * 1024;
    if (lds > allowed) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(moe_group_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        allowed = lds;
    }
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(kGroupThreads), lds, s, ids, (int)n_pairs, (int)n_expert, S,
                       order, offsets, active, error_flag);
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
