// Decode-regime projection (1..4 activation rows): a persistent, software-pipelined GEMV.
//
// One 1024-thread workgroup per CU.  The workgroup quantizes the activation rows (or copies
// rows quantized earlier) into LDS once; when a single K-chunk covers the whole row every lane
// then keeps its slice of the activations in registers for the rest of the kernel.  Each of
// the 16 waves walks its own run of consecutive weight rows, R at a time, with two register
// buffers filled and drained alternately, so the loads of step i+1 are outstanding while step i
// is computed.  Row addresses are a wave-uniform base plus 32-bit offsets, so the scalar unit
// does a handful of operations per step and the vector unit only the dot products.
#include "actquant_device.h"
#include "gemv_frags.h"
#include <stdio.h>

namespace qproj {

namespace {

constexpr int kDecodeThreads = 1024;
constexpr int kDecodeWaves = kDecodeThreads / 64;

// activations into LDS: FUSE quantizes fp32 rows here; otherwise planes quantized earlier are copied
// 256-wide pieces of an activation row that a wave fetches ahead of its first weights: four a row for one or two
// rows (K up to 16384 is covered; pieces fetched inside the quantizing loop instead come one after the other, a trip to
// L2 each: the down projection at two rows, 3.5 pieces a row and wave, 20.2 -> 17.5 us with one-row steps, then
// this), one a row for four rows (which take this kernel for K <= 4096 only)
__host__ __device__ constexpr int prefetched_pieces(int mt) { return mt <= 2 ? 4 : 1; }

template <int QT, int MT, bool FUSE>
__device__ __forceinline__ void stage_activations(uint8_t *smem, const GemvArgs &args, int64_t K, int kpad,
                                                  const float4 *first = nullptr) {
    constexpr int BLK = Geo<QT>::kBlk;
    int8_t *sq = reinterpret_cast<int8_t *>(smem);
    float *sd = reinterpret_cast<float *>(smem + MT * kpad);
    int16_t *sb = reinterpret_cast<int16_t *>(smem + MT * kpad + MT * (kpad / BLK) * 4);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int m = 0; m < MT; ++m) {
        const bool have = m < args.M;
        if (FUSE) {
            const float *x = args.x + (int64_t)m * K;
            const int n_chunks = (int)((K + 255) / 256);
            for (int ch = wave; ch < n_chunks; ch += kDecodeWaves) {
                const int e0 = ch * 256 + 4 * lane;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                constexpr int kPer = prefetched_pieces(MT);   // pieces per row the caller fetched
                if (first && ch < wave + kDecodeWaves * kPer)
                    v = first[m * kPer + (ch - wave) / kDecodeWaves];
                else if (have && e0 < K) v = *reinterpret_cast<const float4 *>(x + e0);
                if (is_q8_0<QT>) {
                    int s;
                    float dd;
                    const uint32_t packed = wave_quantize_q8_32(v, s, dd);
                    if (e0 < K) {
                        *reinterpret_cast<uint32_t *>(sq + m * kpad + e0) = packed;
                        if ((lane & 7) == 0) sd[m * (kpad / 32) + (e0 >> 5)] = h2f(f2h(dd));
                    }
                } else {
                    int bsum;
                    float dd;
                    const uint32_t packed = wave_quantize_q8k(v, lane, bsum, dd);
                    *reinterpret_cast<uint32_t *>(sq + m * kpad + e0) = packed;
                    if ((lane & 3) == 0) sb[m * (kpad / 16) + ch * 16 + (lane >> 2)] = (int16_t)bsum;
                    if (lane == 0) sd[m * (kpad / 256) + ch] = dd;
                }
            }
        } else {
            const ActView &a = args.a;
            for (int i = tid; i < K / 16; i += kDecodeThreads) {
                uint4 v = make_uint4(0, 0, 0, 0);
                if (have) v = *reinterpret_cast<const uint4 *>(a.qs + (int64_t)m * K + i * 16);
                *reinterpret_cast<uint4 *>(sq + m * kpad + i * 16) = v;
            }
            for (int i = tid; i < K / BLK; i += kDecodeThreads)
                sd[m * (kpad / BLK) + i] = have ? a.d[(int64_t)m * (K / BLK) + i] : 0.f;
            if (!is_q8_0<QT>)
                for (int i = tid; i < K / 16; i += kDecodeThreads)
                    sb[m * (kpad / 16) + i] = have ? a.bsums[(int64_t)m * (K / 16) + i] : (int16_t)0;
        }
    }
}

template <int QT, int R>
__device__ __forceinline__ void issue(Raw<QT> (&raw)[R], const RowPtr<QT> &rp, int g, int c, int last_row, int nb, int lane) {
    constexpr int BPC = Geo<QT>::kChunk / Geo<QT>::kBlk;
    // Lanes past the end of a row (last, partial chunk) and rows past the end of the run load the
    // last valid block / row instead: always in bounds, never used.
    int blk = c * BPC + lane / Geo<QT>::kLanesPerBlk;
    if (blk >= nb) blk = nb - 1;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int rel = g * R + r;
        if (rel > last_row) rel = last_row;
        raw[r].load(rp, (uint32_t)blk, lane, (uint32_t)rel);
    }
}

// gate / up pairing: step g is row g of both tensors
template <int QT>
__device__ __forceinline__ void issue_pair(Raw<QT> (&raw)[2], const RowPtr<QT> &rp_gate, const RowPtr<QT> &rp_up, int g, int c,
                                           int last_row, int nb, int lane) {
    constexpr int BPC = Geo<QT>::kChunk / Geo<QT>::kBlk;
    int blk = c * BPC + lane / Geo<QT>::kLanesPerBlk;
    if (blk >= nb) blk = nb - 1;
    const int rel = g > last_row ? last_row : g;
    raw[0].load(rp_gate, (uint32_t)blk, lane, (uint32_t)rel);
    raw[1].load(rp_up, (uint32_t)blk, lane, (uint32_t)rel);
}

// XREG: the lane's activation slices live in `xr` (one chunk covers K); otherwise they are read
// from the LDS image for chunk c.  PAIR (R = 2): the two rows of a step are row g of the gate and of the up
// tensor, and what is stored is silu(gate) * up.
template <int QT, int MT, int R, bool XREG, bool PAIR = false>
__device__ __forceinline__ void consume(const Raw<QT> (&raw)[R], float (&acc)[MT][R], const Dot<QT> (&xr)[MT], const XTile &xt,
                                        int g, int c, int nch, int nb, int n_rows, int64_t row_begin, int64_t N,
                                        float *y, int M, int lane) {
    constexpr int CH = Geo<QT>::kChunk;
    if (lane_block<QT>((int64_t)c * CH, lane) < nb) {
        Frag<QT> f[R];
#pragma unroll
        for (int r = 0; r < R; ++r) f[r].unpack(raw[r], lane);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (XREG) {
#pragma unroll
                for (int r = 0; r < R; ++r) acc[m][r] += xr[m].dot(f[r]);
            } else {
                Dot<QT> dx;
                dx.load_x(xt, m, c * CH, lane);
#pragma unroll
                for (int r = 0; r < R; ++r) acc[m][r] += dx.dot(f[r]);
            }
        }
    }
    if (c + 1 == nch) {  // row group finished: reduce over the wave, store, start over
        constexpr int V = MT * R;
#pragma unroll
        for (int v0 = 0; v0 < V; v0 += 4) {
            float q[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) q[i] = (v0 + i < V) ? acc[(v0 + i) / R][(v0 + i) % R] : 0.f;
            const float t = wave_sum4(q, lane);
            const int i = lane - 12;  // lanes 12..15 hold the four sums
            if constexpr (PAIR) {
                const float up = __shfl_down(t, 1);   // sums 2m (gate) and 2m+1 (up) sit in neighbouring lanes
                if (i >= 0 && i < 4 && v0 + i < V && ((v0 + i) & 1) == 0) {
                    const int m = (v0 + i) / 2;
                    if (m < M && g < n_rows) y[(int64_t)m * N + row_begin + g] = (t / (1.0f + expf(-t))) * up;
                }
            } else if (i >= 0 && i < 4 && v0 + i < V) {
                const int m = (v0 + i) / R, r = (v0 + i) % R;
                if (m < M && g * R + r < n_rows) y[(int64_t)m * N + row_begin + g * R + r] = t;
            }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) acc[m][r] = 0.f;
    }
}

template <int QT, int MT, int R, bool XREG, bool FUSE, bool PAIR = false>
__global__ __launch_bounds__(kDecodeThreads) void gemv_decode_kernel(const GemvArgs args, int kpad) {
    static_assert(!PAIR || R == 2, "the gate/up pairing walks two rows a step");
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int CH = Geo<QT>::kChunk;
    constexpr int BLK = Geo<QT>::kBlk;
    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    const int gw = blockIdx.x * kDecodeWaves + wave;  // global wave index
    const int64_t K = args.t[0].w.K;
    const int nb = (int)args.t[0].w.nb;
    const int nch = XREG ? 1 : kpad / CH;

    // this wave's target and run of rows (selected once; everything below is wave-uniform)
    WeightView w = args.t[0].w;
    float *y = args.t[0].y;
    int wave_first = 0, rpp = args.t[0].rows_per_pair;
#pragma unroll
    for (int i = 1; i < kMaxTargets; ++i) {
        if (!PAIR && i < args.n_targets && gw >= args.t[i].first_block) {
            w = args.t[i].w;
            y = args.t[i].y;
            wave_first = args.t[i].first_block;
            rpp = args.t[i].rows_per_pair;
        }
    }
    const int64_t N = w.N;
    // Rows are dealt to pairs of neighbouring waves: rpp consecutive rows a pair, the even wave taking the larger
    // part.  A target with 1.5 rows per wave then keeps every wave busy (2 + 1) where whole rows per wave would
    // leave a third of the workgroups without work, and with two rows a step the even wave's part is rounded up
    // to an even count so that no step fetches its last row twice (7 + 7 becomes 8 + 6).
    const int wl = gw - wave_first;
    int part_even = (rpp + 1) >> 1;
    if (!PAIR && R == 2) part_even = (part_even + 1) & ~1;
    if (part_even > rpp) part_even = rpp;
    const int64_t row_begin = (int64_t)(wl >> 1) * rpp + ((wl & 1) ? part_even : 0);
    const int own = (wl & 1) ? rpp - part_even : part_even;
    int n_rows = 0;  // rows this wave owns
    if (row_begin < N) n_rows = (int)((N - row_begin) < own ? (N - row_begin) : own);
    n_rows = uniform(n_rows);
    const int n_groups = PAIR ? n_rows : (n_rows + R - 1) / R;
    const int n_iter = n_groups * nch;
    const int last_row = n_rows > 0 ? n_rows - 1 : 0;
    RowPtr<QT> rp, rp_up;
    rp.set(w, row_begin < N ? row_begin : 0);
    rp_up.set(PAIR ? args.t[1].w : w, row_begin < N ? row_begin : 0);
    auto issue_rows = [&](Raw<QT> (&raw)[R], int g, int c) {
        if constexpr (PAIR) issue_pair<QT>(raw, rp, rp_up, g, c, last_row, nb, lane);
        else issue<QT, R>(raw, rp, g, c, last_row, nb, lane);
    };

    // The wave's piece of the activation row is requested BEFORE the first weights: loads return in order, and
    // behind a step of weights coming from HBM the quantizing prologue would wait two microseconds for sixteen
    // bytes that sit in L2 (phase clocks: staging 3000-4400 cycles of a workgroup's 25000).
    float4 x_first[MT * prefetched_pieces(MT)];
    if (FUSE) {
        constexpr int kPer = prefetched_pieces(MT);
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int i = 0; i < kPer; ++i) {
                const int e0 = (wave + kDecodeWaves * i) * 256 + 4 * lane;
                x_first[m * kPer + i] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (m < args.M && e0 < K) x_first[m * kPer + i] = *reinterpret_cast<const float4 *>(args.x + (int64_t)m * K + e0);
            }
    }
    // RMS norm fused in front of the quantizer (the launcher only asks for it when the prefetched pieces are the
    // whole row): weights of the norm fetched with the row, sum of squares over the workgroup in the order of
    // the standalone kernel, then the pieces are replaced by (x * scale) * gamma.
    float4 g_first[prefetched_pieces(MT)];
    if (FUSE && args.norm) {
#pragma unroll
        for (int i = 0; i < prefetched_pieces(MT); ++i) {
            const int e0 = (wave + kDecodeWaves * i) * 256 + 4 * lane;
            g_first[i] = make_float4(1.f, 1.f, 1.f, 1.f);
            if (args.norm_gamma && e0 < K) g_first[i] = *reinterpret_cast<const float4 *>(args.norm_gamma + e0);
        }
    }
    Raw<QT> buf_a[R], buf_b[R];
    issue_rows(buf_a, 0, 0);  // in flight while the activations are staged
    if (FUSE && args.norm) {
        __shared__ double norm_partial[kDecodeWaves];
        constexpr int kPer = prefetched_pieces(MT);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            double sq = 0.0;
#pragma unroll
            for (int i = 0; i < kPer; ++i) sq += sum4_sq(x_first[m * kPer + i]);
            if (m > 0) __syncthreads();   // the partial sums of the previous row have been read
            const double total = workgroup_sum16(sq, norm_partial);
            const float mean = (float)(total / (double)K);
            const float scale = 1.0f / sqrtf(mean + args.norm_eps);
#pragma unroll
            for (int i = 0; i < kPer; ++i) {
                float4 &v = x_first[m * kPer + i];
                v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
                if (args.norm_gamma) {
                    v.x *= g_first[i].x; v.y *= g_first[i].y; v.z *= g_first[i].z; v.w *= g_first[i].w;
                }
            }
        }
    }

    stage_activations<QT, MT, FUSE>(smem, args, K, kpad, FUSE ? x_first : nullptr);
    __syncthreads();

    XTile xt;
    xt.qs = reinterpret_cast<const int8_t *>(smem);
    xt.d = reinterpret_cast<const float *>(smem + MT * kpad);
    xt.bs = reinterpret_cast<const int16_t *>(smem + MT * kpad + MT * (kpad / BLK) * 4);
    xt.kt = kpad;
    Dot<QT> xr[MT];
    if (XREG) {
#pragma unroll
        for (int m = 0; m < MT; ++m) xr[m].load_x(xt, m, 0, lane);
    }

    float acc[MT][R];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[m][r] = 0.f;

    // (g, c) = (row group, chunk) cursors; the issue cursor runs one step ahead of the consume
    // cursor and stops on the last step, whose cache lines were just fetched, so every issue is
    // unconditional and no wait ever has to cover a maybe-issued load.
    if constexpr (XREG && (MT == 1 || (MT == 2 && QT == kTypeQ4_K && FUSE && !PAIR))) {  // one chunk per row, one or two activation rows: the step index is the row group
        // No load is issued twice (a repeated load of the last step, cheap as it looks, costs 0.4 us of the
        // gate+up launch at one activation row and 0.8 us at two): the loop runs while two more steps follow,
        // the last one or two steps are peeled, and every block still knows exactly which loads are outstanding.
        // (Two rows of the wider formats, of the gate/up pairing and of rows quantized earlier keep the plain loop
        // below: peeled they run out of registers.)
        int g = 0;
        for (; g + 2 < n_groups; g += 2) {
            issue_rows(buf_b, g + 1, 0);
            __builtin_amdgcn_sched_barrier(0);
            consume<QT, MT, R, XREG, PAIR>(buf_a, acc, xr, xt, g, 0, 1, nb, n_rows, row_begin, N, y, args.M, lane);
            issue_rows(buf_a, g + 2, 0);
            __builtin_amdgcn_sched_barrier(0);
            consume<QT, MT, R, XREG, PAIR>(buf_b, acc, xr, xt, g + 1, 0, 1, nb, n_rows, row_begin, N, y, args.M, lane);
        }
        if (g + 1 < n_groups) {
            issue_rows(buf_b, g + 1, 0);
            __builtin_amdgcn_sched_barrier(0);
            consume<QT, MT, R, XREG, PAIR>(buf_a, acc, xr, xt, g, 0, 1, nb, n_rows, row_begin, N, y, args.M, lane);
            consume<QT, MT, R, XREG, PAIR>(buf_b, acc, xr, xt, g + 1, 0, 1, nb, n_rows, row_begin, N, y, args.M, lane);
        } else if (g < n_groups) {
            consume<QT, MT, R, XREG, PAIR>(buf_a, acc, xr, xt, g, 0, 1, nb, n_rows, row_begin, N, y, args.M, lane);
        }
        return;
    }
    if (XREG) {  // one chunk per row: the step index is the row group
        for (int g = 0; g < n_groups; g += 2) {
            issue_rows(buf_b, g + 1 < n_groups ? g + 1 : n_groups - 1, 0);
            __builtin_amdgcn_sched_barrier(0);
            consume<QT, MT, R, XREG, PAIR>(buf_a, acc, xr, xt, g, 0, 1, nb, n_rows, row_begin, N, y, args.M, lane);
            issue_rows(buf_a, g + 2 < n_groups ? g + 2 : n_groups - 1, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (g + 1 < n_groups) consume<QT, MT, R, XREG, PAIR>(buf_b, acc, xr, xt, g + 1, 0, 1, nb, n_rows, row_begin, N, y, args.M, lane);
        }
        return;
    }
    int ig = 0, ic = 0, cg = 0, cc = 0, issued = 0;
    auto advance = [&](int &g, int &c) {
        c += 1;
        if (c == nch) {
            c = 0;
            g += 1;
        }
    };
    for (int it = 0; it < n_iter; it += 2) {
        if (issued + 1 < n_iter) { advance(ig, ic); ++issued; }
        issue_rows(buf_b, uniform(ig), uniform(ic));
        __builtin_amdgcn_sched_barrier(0);  // keep the loads ahead of the arithmetic that follows
        consume<QT, MT, R, XREG, PAIR>(buf_a, acc, xr, xt, uniform(cg), uniform(cc), nch, nb, n_rows, row_begin, N, y, args.M, lane);
        advance(cg, cc);
        if (issued + 1 < n_iter) { advance(ig, ic); ++issued; }
        issue_rows(buf_a, uniform(ig), uniform(ic));
        __builtin_amdgcn_sched_barrier(0);
        if (it + 1 < n_iter) {
            consume<QT, MT, R, XREG, PAIR>(buf_b, acc, xr, xt, uniform(cg), uniform(cc), nch, nb, n_rows, row_begin, N, y, args.M, lane);
            advance(cg, cc);
        }
    }
}


template <int QT, int MT, int R, bool XREG, bool FUSE, bool PAIR = false>
hipError_t launch_decode(const GemvArgs &args, hipStream_t s) {
    constexpr int CH = Geo<QT>::kChunk;
    constexpr int BLK = Geo<QT>::kBlk;
    GemvArgs a = args;
    if (PAIR) {   // gate and up are walked together: the waves are dealt over the rows of one of them
        if (a.n_targets != 2 || a.t[0].w.N != a.t[1].w.N || a.t[0].w.K != a.t[1].w.K) return hipErrorInvalidValue;
        a.n_targets = 1;
    }
    int64_t rows_total = 0;
    for (int i = 0; i < a.n_targets; ++i) rows_total += a.t[i].w.N;
    if (rows_total == 0) return hipSuccess;
    // one workgroup per CU, fewer when there are not enough rows to give every wave one
    static const int wgs_per_cu = tuning_int("QPROJ_DECODE_WGS_PER_CU", 1);
    int64_t grid = (int64_t)cu_count() * wgs_per_cu;
    const int64_t need = (rows_total + kDecodeWaves - 1) / kDecodeWaves;  // at least one row per wave
    if (grid > need) grid = need;
    const int n_waves = (int)grid * kDecodeWaves;
    // waves are dealt to the targets in proportion to their rows; a wave never straddles targets
    int given = 0;
    for (int i = 0; i < a.n_targets; ++i) {
        const int left_after = a.n_targets - 1 - i;  // every later target gets at least one wave
        int share = (int)((a.t[i].w.N * n_waves + rows_total - 1) / rows_total);
        if (share < 1) share = 1;
        if (i == a.n_targets - 1 || given + share > n_waves - left_after) share = n_waves - left_after - given;
        if (share < 1) return hipErrorInvalidValue;
        a.t[i].first_block = given;
        const int rpp = (int)((2 * a.t[i].w.N + share - 1) / share);  // rows per pair of waves
        a.t[i].rows_per_pair = rpp;
        if ((int64_t)rpp * (int64_t)a.t[i].w.nb * 256 >= ((int64_t)1 << 31)) return hipErrorInvalidValue;  // 32-bit row offsets
        given += share;
    }
    const int64_t K = a.t[0].w.K;
    const int kpad = (int)((K + CH - 1) / CH * CH);
    const size_t smem = (size_t)MT * kpad + (size_t)MT * (kpad / BLK) * 4 + (!is_q8_0<QT> ? (size_t)MT * (kpad / 16) * 2 : 0);
    if (PAIR) a.n_targets = 2;
    if (dry_run()) {
        char rows[96] = "";
        for (int i = 0, o = 0; i < (PAIR ? 1 : a.n_targets) && o < 80; ++i)
            o += snprintf(rows + o, sizeof rows - o, "%s%lld rows/%d a wave pair", i ? ", " : "", (long long)a.t[i].w.N, a.t[i].rows_per_pair);
        plan_note("gemv_decode_kernel<%s, %d activation rows, %d weight rows a step, activations in %s, %s%s>: grid %lld x %d, %s, LDS %zu B",
                  plan_type_name(QT), MT, R, XREG ? "registers" : "LDS", FUSE ? "quantizer in the prologue" : "rows quantized earlier",
                  PAIR ? ", gate/up paired + swiglu" : "", (long long)grid, kDecodeThreads, rows, smem);
        return hipSuccess;
    }
    auto kern = &gemv_decode_kernel<QT, MT, R, XREG, FUSE, PAIR>;
    if (smem > 48 * 1024) {
        static size_t allowed = 0;
        if (smem > allowed) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
            if (e != hipSuccess) return e;
            allowed = smem;
        }
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kDecodeThreads), smem, s, a, kpad);
    return hipGetLastError();
}

template <int QT, bool FUSE>
hipError_t launch_decode_mt(const GemvArgs &args, int mt, hipStream_t s) {
    // the wide Q8_0 geometry keeps its 20 activation registers a row only for one row and plain projections (two
    // rows, or the gate/up pairing, would spill); otherwise it reads them from the LDS image like a longer K
    const bool one_chunk = args.t[0].w.K <= Geo<QT>::kChunk && !(QT == kTypeQ8_0Wide && (mt > 1 || args.swiglu_pair));
    if (args.swiglu_pair) {
        if (mt == 1) return one_chunk ? launch_decode<QT, 1, 2, true, FUSE, true>(args, s) : launch_decode<QT, 1, 2, false, FUSE, true>(args, s);
        if (mt == 2) return one_chunk ? launch_decode<QT, 2, 2, true, FUSE, true>(args, s) : launch_decode<QT, 2, 2, false, FUSE, true>(args, s);
        return hipErrorInvalidValue;
    }
    // two rows per step only when every wave has at least two rows to walk (with 1.5 rows per wave, split
    // 2 + 1 over a pair of waves, two-row steps measured slower: q/k/v 7.4 against 6.4 us; with one row a wave
    // a two-row step fetches that row twice)
    int64_t rows_total = 0;
    for (int i = 0; i < args.n_targets; ++i) rows_total += args.t[i].w.N;
    static const int two_rows_env = tuning_int("QPROJ_DECODE_TWO_ROWS", -1);
    const bool pairs = two_rows_env >= 0 ? two_rows_env != 0 : rows_total >= (int64_t)2 * cu_count() * kDecodeWaves;
    switch (mt) {
    case 1: {
        if (one_chunk) return pairs ? launch_decode<QT, 1, 2, true, FUSE>(args, s) : launch_decode<QT, 1, 1, true, FUSE>(args, s);
        // (rows of several chunks in the wider formats: one row a step -- 8192 x 8192 Q8_0 19.2 -> 16.9 us, Q6_K 15.6 -> 14.3)
        const bool two = pairs && (QT == kTypeQ4_K || two_rows_env > 0);
        return two ? launch_decode<QT, 1, 2, false, FUSE>(args, s) : launch_decode<QT, 1, 1, false, FUSE>(args, s);
    }
    case 2: {
        // (two rows of the wider formats walk one weight row a step whatever the row count: their two-row steps
        // run out of registers -- Q6_K 4096 -> 14336 17.5 -> 13.9 us, Q8_0 8192 x 8192 20.1 -> 17.6)
        const bool two = pairs && (QT == kTypeQ4_K || two_rows_env > 0);
        if (one_chunk) return two ? launch_decode<QT, 2, 2, true, FUSE>(args, s) : launch_decode<QT, 2, 1, true, FUSE>(args, s);
        return two ? launch_decode<QT, 2, 2, false, FUSE>(args, s) : launch_decode<QT, 2, 1, false, FUSE>(args, s);
    }
    case 4:
        if constexpr (QT == kTypeQ4_K)
            if (one_chunk) return launch_decode<QT, 4, 1, true, FUSE>(args, s);
        return launch_decode<QT, 4, 1, false, FUSE>(args, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

int cu_count() {
    static int n = [] {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
        return v;
    }();
    return n;
}

bool decode_kernel_norm_fits(int mt, int64_t K) {
    return mt >= 1 && mt <= 4 && K <= (int64_t)256 * kDecodeWaves * prefetched_pieces(mt);
}

// the largest K whose activation rows fit the LDS image (mt rows)
bool decode_kernel_fits(int type, int mt, int64_t K) {
    const int ch = 4096;
    const int blk = type == kTypeQ8_0 ? 32 : 256;
    const int64_t kpad = (K + ch - 1) / ch * ch;
    const int64_t smem = mt * kpad + mt * (kpad / blk) * 4 + (type != kTypeQ8_0 ? mt * (kpad / 16) * 2 : 0);
    return mt <= 4 && smem <= 96 * 1024;
}

hipError_t launch_gemv_decode(const GemvArgs &args, int mt, bool fuse_quantize, hipStream_t s) {
    switch (args.t[0].w.type) {
    case kTypeQ4_K: return fuse_quantize ? launch_decode_mt<kTypeQ4_K, true>(args, mt, s) : launch_decode_mt<kTypeQ4_K, false>(args, mt, s);
    case kTypeQ6_K: return fuse_quantize ? launch_decode_mt<kTypeQ6_K, true>(args, mt, s) : launch_decode_mt<kTypeQ6_K, false>(args, mt, s);
    case kTypeQ8_0: return fuse_quantize ? launch_decode_mt<kTypeQ8_0Wide, true>(args, mt, s) : launch_decode_mt<kTypeQ8_0Wide, false>(args, mt, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace qproj
