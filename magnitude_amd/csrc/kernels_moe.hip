// Expert grouping for MUL_MAT_ID and the weighted combine of the MoE feed-forward.
#include "actquant_device.h"
#include "qproj_device.h"
#include "qproj_internal.h"

namespace qproj {

// Counting sort of (token, slot) pairs by expert id, one workgroup.  offsets[e]..offsets[e+1]
// indexes the pairs of expert e inside order[]; active[0..active[n_expert]) lists the experts that
// have pairs (those with more than pass_rows pairs first, ascending within both parts).  Ids outside [0, n_expert) raise *error_flag and
// their pairs are left out (their outputs are not written).  Pairs of one expert keep ascending
// pair order so repeated runs produce the same launch geometry.  Each of the 16 waves takes every
// 16th expert and sweeps the pair list 64 ids at a time (consecutive lanes on consecutive ids):
// a ballot of the matches gives the count in the first sweep and, with the number of matching
// lanes below one's own, the slot in the second.  (A version that read the ids from LDS inside the
// sweeps was a chain of dependent loads: 19 us for 512 pairs and 128 experts.)
constexpr int kGroupThreads = 1024;
constexpr int kGroupLdsIds = 8192;   // pair ids staged in LDS up to this many, read from global beyond

// cnt[e] = pairs of expert e on entry; on exit cnt[e] = offsets[e] = its first slot, active[] lists the
// experts that have pairs.  All threads of the workgroup call it; the caller synchronizes afterwards.
__device__ __forceinline__ void group_scan(int n_expert, int32_t *cnt, int32_t *wsum, int32_t *__restrict__ offsets,
                                           int32_t *__restrict__ active, int pass_rows) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // exclusive scans over the workgroup (shuffles inside a wave, wave totals through LDS) of the pair
    // counts (-> offsets) and of the non-empty flags (-> compact list of the experts that have work);
    // thread t owns experts [t * per, t * per + per)
    const int per = (n_expert + kGroupThreads - 1) / kGroupThreads;
    int tot[8], local = 0, local_f = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int e = tid * per + i;
        tot[i] = i < per && e < n_expert ? cnt[e] : 0;
        local += tot[i];
        local_f += tot[i] > 0;
    }
    // The experts with more pairs than one pass of the grouped kernels stages (two passes over their weights) go
    // to the front of the list, everything else stays in ascending order: the grouped kernels hand their
    // workgroups out in list order, and a two-pass expert then starts with the grid instead of stretching its
    // tail.  A third scan, over the "heavy" flags, gives the positions.  (The whole list ordered by pair count
    // evened the launches out as well but cost the ordinary case 3 us: neighbouring workgroups no longer read
    // neighbouring experts.)
    int local_h = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) local_h += pass_rows > 0 && tot[i] > pass_rows;
    int incl = local, incl_f = local_f, incl_h = local_h;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d), up_f = __shfl_up(incl_f, d), up_h = __shfl_up(incl_h, d);
        if (lane >= d) {
            incl += up;
            incl_f += up_f;
            incl_h += up_h;
        }
    }
    if (lane == 63) {
        wsum[wave] = incl;
        wsum[16 + wave] = incl_f;
        wsum[32 + wave] = incl_h;
    }
    __syncthreads();
    int before = incl - local, before_f = incl_f - local_f, before_h = incl_h - local_h, n_heavy = 0;
    for (int w = 0; w < kGroupThreads / 64; ++w) {
        if (w < wave) {
            before += wsum[w];
            before_f += wsum[16 + w];
            before_h += wsum[32 + w];
        }
        n_heavy += wsum[32 + w];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int e = tid * per + i;
        if (i < per && e < n_expert) {
            cnt[e] = before;   // from here on: the expert's first slot
            offsets[e] = before;
            before += tot[i];
            if (tot[i] > 0) {
                const bool heavy = pass_rows > 0 && tot[i] > pass_rows;
                const int pos = heavy ? before_h : n_heavy + (before_f - before_h);
                active[pos] = e;
                reinterpret_cast<int4 *>(active + active_slots_offset(n_expert))[pos] = make_int4(e, before - tot[i], tot[i], 0);
                ++before_f;
                before_h += heavy;
            }
        }
    }
    if (tid == kGroupThreads - 1) {
        offsets[n_expert] = before;
        active[n_expert] = before_f;   // how many experts have pairs
    }
}

template <bool STAGED>
__device__ __forceinline__ void group_sweeps(const int32_t *__restrict__ ids, const int32_t *sid, int n_pairs, int n_expert,
                                             int32_t *cnt, int32_t *wsum, int32_t *__restrict__ order,
                                             int32_t *__restrict__ offsets, int32_t *__restrict__ active, int pass_rows) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int kWaves = kGroupThreads / 64;
    auto id_at = [&](int p) { return p < n_pairs ? (STAGED ? sid[p] : ids[p]) : -1; };
    // A lane keeps the ids of its positions in registers, kHeld at a time (1024 pairs per wave and block),
    // and runs through its experts on them: the sweeps are ballots on registers, not a chain of loads.
    constexpr int kHeld = 16;
    // sweep 1: pairs per expert (cnt starts at zero)
    for (int base = 0; base < n_pairs; base += 64 * kHeld) {
        int v[kHeld];
#pragma unroll
        for (int u = 0; u < kHeld; ++u) v[u] = id_at(base + 64 * u + lane);
        for (int e = wave; e < n_expert; e += kWaves) {
            int c = 0;
#pragma unroll
            for (int u = 0; u < kHeld; ++u) c += __popcll(__ballot(v[u] == e));
            if (lane == 0) cnt[e] += c;   // every expert belongs to one wave
        }
    }
    __syncthreads();
    group_scan(n_expert, cnt, wsum, offsets, active, pass_rows);
    __syncthreads();
    // sweep 2: placement, ascending pair order inside every expert (cnt[e] = the expert's next free slot)
    for (int base = 0; base < n_pairs; base += 64 * kHeld) {
        int v[kHeld];
#pragma unroll
        for (int u = 0; u < kHeld; ++u) v[u] = id_at(base + 64 * u + lane);
        for (int e = wave; e < n_expert; e += kWaves) {
            int w = cnt[e];
#pragma unroll
            for (int u = 0; u < kHeld; ++u) {
                const bool mine = v[u] == e;
                const unsigned long long m = __ballot(mine);
                if (mine)
                    order[w + __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0))] =
                        base + 64 * u + lane;
                w += __popcll(m);
            }
            if (lane == 0) cnt[e] = w;
        }
    }
}

// The sweeps above cost n_expert x n_pairs / 1024 steps.  Up to 8192 pairs (and while the table below fits
// LDS) the work is made proportional to n_pairs instead: a wave takes 64 consecutive pairs, and 64 rounds of
// "broadcast lane j's id, ballot who has the same" give every lane its rank among the equal ids of the block
// and the size of its group; the first lane of a group files that size under blk[block][expert].  A prefix
// over the blocks per expert, the scan over the experts, and every pair knows its slot:
// first[expert] + blk[block][expert] + rank.
constexpr int kBlocksPerWave = 8;   // 16 waves x 8 blocks x 64 = 8192 pairs

__global__ __launch_bounds__(kGroupThreads) void moe_group_kernel(const int32_t *__restrict__ ids, int n_pairs,
                                                                  int n_expert, int32_t *__restrict__ order,
                                                                  int32_t *__restrict__ offsets,
                                                                  int32_t *__restrict__ active,
                                                                  int32_t *__restrict__ error_flag, int by_block,
                                                                  int pass_rows, const RowQuantJob job) {
    // Workgroups past the first have nothing to do with the grouping: they quantize the activation rows the
    // grouped projection is going to read (one 256-wide chunk a wave, ggml's quantize_row_q8_K as in the
    // standalone quantizer), so that the two passes, which depend only on the call's inputs, share a launch.
    if (blockIdx.x > 0) {
        const int64_t sb = (int64_t)(blockIdx.x - 1) * (kGroupThreads / 64) + (threadIdx.x >> 6);
        if (sb < job.n_super) {   // whole wave decides together
            const int lane = threadIdx.x & 63;
            const float4 v = reinterpret_cast<const float4 *>(job.x + sb * 256)[lane];
            wave_store_q8k(v, lane, sb, job.qs, job.d, job.bsums);
        }
        return;
    }
    extern __shared__ int32_t lds[];
    int32_t *cnt = lds;                 // [n_expert] pairs of the expert, then its first slot
    int32_t *wsum = cnt + n_expert;     // [48] wave totals of the three scans
    int32_t *tab = wsum + 48;           // by_block: blk[n_blocks][n_expert]; else the staged ids
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (!by_block) {
        const bool staged = n_pairs <= kGroupLdsIds;
        bool bad = false;
        for (int p = tid; p < n_pairs; p += kGroupThreads) {
            const int e = ids[p];
            bad |= e < 0 || e >= n_expert;
            if (staged) tab[p] = e;
        }
        for (int e = tid; e < n_expert; e += kGroupThreads) cnt[e] = 0;
        if (bad) atomicOr(error_flag, 1);
        __syncthreads();
        if (staged) group_sweeps<true>(ids, tab, n_pairs, n_expert, cnt, wsum, order, offsets, active, pass_rows);
        else group_sweeps<false>(ids, tab, n_pairs, n_expert, cnt, wsum, order, offsets, active, pass_rows);
        return;
    }
    const int n_blocks = (n_pairs + 63) / 64;
    const int id_bits = n_expert > 1 ? 32 - __builtin_clz((unsigned)(n_expert - 1)) : 0;
    int vid[kBlocksPerWave], rank[kBlocksPerWave];
    bool bad = false;
#pragma unroll
    for (int i = 0; i < kBlocksPerWave; ++i) {   // the loads first: they travel while the table is cleared
        const int p = 64 * (wave + 16 * i) + lane;
        vid[i] = p < n_pairs ? ids[p] : -1;
        bad |= p < n_pairs && (vid[i] < 0 || vid[i] >= n_expert);
        if (vid[i] >= n_expert) vid[i] = -1;
    }
    for (int t = tid; t < n_blocks * n_expert; t += kGroupThreads) tab[t] = 0;
    if (bad) atomicOr(error_flag, 1);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kBlocksPerWave; ++i) {
        const int blk = wave + 16 * i;
        if (blk < n_blocks) {   // wave-uniform
            const int v = vid[i];
            // the lanes of the block that hold the same expert: one ballot per bit of the id (and one for "names an
            // expert at all") instead of one per lane
            unsigned long long m = ~0ull;
            {
                const unsigned long long b = __ballot(v >= 0);
                m &= v >= 0 ? b : ~b;
            }
            for (int bit = 0; bit < id_bits; ++bit) {
                const bool set = (v >> bit) & 1;
                const unsigned long long b = __ballot(set);
                m &= set ? b : ~b;
            }
            const int r = __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0));
            const int size = __popcll(m);
            rank[i] = r;
            if (r == 0 && v >= 0) tab[blk * n_expert + v] = size;
        }
    }
    __syncthreads();
    // per expert: group sizes of the blocks -> first slot of the block's group inside the expert; total
    for (int e = tid; e < n_expert; e += kGroupThreads) {
        int run = 0;
        for (int b = 0; b < n_blocks; ++b) {
            const int c = tab[b * n_expert + e];
            tab[b * n_expert + e] = run;
            run += c;
        }
        cnt[e] = run;
    }
    __syncthreads();
    group_scan(n_expert, cnt, wsum, offsets, active, pass_rows);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kBlocksPerWave; ++i) {
        const int blk = wave + 16 * i, v = vid[i];
        if (blk < n_blocks && v >= 0) order[cnt[v] + tab[blk * n_expert + v] + rank[i]] = 64 * blk + lane;
    }
}

hipError_t launch_moe_group(const int32_t *ids, int64_t n_pairs, int64_t n_expert, int32_t *order,
                            int32_t *offsets, int32_t *active, int32_t *error_flag, const RowQuantJob *quantize,
                            hipStream_t s) {
    if (n_expert > 8192 || n_pairs > 0x7fffffff) return hipErrorInvalidValue;
    const size_t table = (size_t)((n_pairs + 63) / 64) * (size_t)n_expert;
    const bool by_block = n_pairs <= 64 * 16 * kBlocksPerWave && table <= 24 * 1024;   // at most 96 KB of LDS
    const size_t lds = ((size_t)n_expert + 48 + (by_block ? table : n_pairs <= kGroupLdsIds ? (size_t)n_pairs : 0)) * sizeof(int32_t);
    if (dry_run()) {
        plan_note("moe_group_kernel: %lld pairs over %lld experts (%s)%s", (long long)n_pairs, (long long)n_expert,
                  by_block ? "ballot per bit of the id, prefix over 64-pair blocks" : "ballot sweeps per expert",
                  quantize ? ", spare workgroups quantize the token rows" : "");
        return hipSuccess;
    }
    static size_t allowed = 48 * 1024;
    if (lds > allowed) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(moe_group_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        allowed = lds;
    }
    RowQuantJob job{};
    if (quantize) job = *quantize;
    const int64_t extra = (job.n_super + kGroupThreads / 64 - 1) / (kGroupThreads / 64);
    if (extra >= 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL(moe_group_kernel, dim3((unsigned)(1 + extra)), dim3(kGroupThreads), lds, s, ids, (int)n_pairs,
                       (int)n_expert, order, offsets, active, error_flag, by_block ? 1 : 0,
                       n_pairs <= 4 * n_expert ? 8 : 16 /* rows a pass of the grouped matrix-core kernel stages */, job);
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

// h = silu(g) * u with ggml's expression for silu, x / (1 + expf(-x))
__global__ __launch_bounds__(256) void swiglu_kernel(const float *__restrict__ g, const float *__restrict__ u, size_t n,
                                                     float *__restrict__ h) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        const float x = g[i];
        h[i] = (x / (1.0f + expf(-x))) * u[i];
    }
}

hipError_t launch_swiglu(const float *g, const float *u, size_t n, float *h, hipStream_t s) {
    if (n == 0) return hipSuccess;
    if (dry_run()) {
        plan_note("swiglu_kernel: %zu elements", n);
        return hipSuccess;
    }
    hipLaunchKernelGGL(swiglu_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, g, u, n, h);
    return hipGetLastError();
}

hipError_t launch_moe_combine(const float *e, const float *weights, int64_t B, int64_t n_used, int64_t N,
                              float *y, hipStream_t s) {
    const int64_t n = B * N;
    if (n == 0) return hipSuccess;
    if (dry_run()) {
        plan_note("moe_combine_kernel: %lld tokens x %lld, %lld experts a token in slot order", (long long)B, (long long)N, (long long)n_used);
        return hipSuccess;
    }
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, e, weights, B,
                       (int)n_used, N, y);
    return hipGetLastError();
}

}  // namespace qproj
