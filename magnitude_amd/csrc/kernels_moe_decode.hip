// MUL_MAT_ID for decode-sized batches (a few tokens; at most about one (token, expert) pair an expert) on the
// vector ALU: no grouping pass, no matrix cores, no separate quantizer or combine launch.
//
// Every pair has its own expert matrix and, for the down projection, its own activation row, so the launch is
// a set of independent short GEMVs: a workgroup of 16 waves serves a run of weight rows for a GROUP of pairs
// (one pair; the n_used pairs of one token when their results are combined here; or, with more pairs than the
// compute units have workgroups for, a few consecutive pairs that read the same activation row).  It quantizes the
// group's activation rows into LDS with the arithmetic of the standalone quantizer, and its waves then walk
// (row step, pair) units.  Expert rows are short (K = 768 .. 4096), so a step covers S = 64 / (4 K/256) whole
// rows at once: lane = (row slot, super-block, quarter of the super-block), the row slots' partial dot products
// are summed over their own lanes only.  (Longer rows, LONGK: one row a unit, walked 4096 weights a step.)  Consecutive rows of a matrix are consecutive in memory, so a step's
// loads cover one contiguous stretch.  With gate and up given, a step walks the same rows of both and stores
// silu(gate . x) * (up . x); with routing weights given, the workgroup adds its pairs' results in slot order,
// each product rounded first, which is what the separate combine pass does.
#include <algorithm>

#include "actquant_device.h"
#include "gemv_frags.h"

namespace qproj {

namespace {

constexpr int kThreads = 1024, kWaves = kThreads / 64;
constexpr int kMaxGroup = 16;

struct MoeDecodeArgs {
    WeightView w0, w1;       // w1: the up tensor when gate / up are paired
    const float *x;          // fp32 activation rows [.][K]
    int x_div;               // the activation row of pair p is p / x_div
    const int32_t *ids;      // expert of pair p
    int n_pairs, n_expert;
    int32_t *error_flag;
    float *y;                // [n_pairs][N]; with routing weights [n_pairs / group][N]
    const float *cw;         // routing weights [n_pairs], or null
    int group;               // pairs a workgroup serves
    int x_shared;            // the pairs of a group all read ONE activation row (group divides x_div): staged once
    int wgs_per_group;       // workgroups that share the rows of a group
    int rows_per_wg;         // a multiple of the rows a step covers
};

// sum of v over the `lpr` lanes of each row slot (lpr a multiple of 4); valid in the slot's first lane
__device__ __forceinline__ float slot_sum(float v, int vlane, int lpr) {
    v += dpp_move<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
#pragma unroll
    for (int o = 32; o >= 4; o >>= 1) {
        if (o < lpr) {   // wave-uniform
            const float t = __shfl_down(v, o);
            if (vlane + o < lpr) v += t;
        }
    }
    return v;
}

// R: row steps a unit covers (two where a wave has several units of short rows: fewer, larger requests)
// LONGK: rows of more than 4096 weights -- a unit is one row, walked in steps of 16 super-blocks
template <int QT, bool SWIGLU, bool COMBINE, int R, bool LONGK = false>
__global__ __launch_bounds__(kThreads) void moe_decode_kernel(const MoeDecodeArgs g) {
    static_assert(!SWIGLU || R == 1, "gate / up already load two tensors a unit");
    static_assert(!LONGK || R == 1, "long rows are walked one at a time");
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int NT = SWIGLU ? 2 : R;   // register sets a unit loads
    const int tid = threadIdx.x, lane = tid & 63, wave = uniform(tid >> 6);
    const int K = (int)g.w0.K, nb = (int)g.w0.nb, N = (int)g.w0.N;
    const int lpr = LONGK ? 64 : 4 * nb, S = 64 / lpr;
    const int nch = LONGK ? (nb + 15) / 16 : 1;   // steps a unit
    const bool live = lane < S * lpr;
    const int slot = live ? lane / lpr : 0;
    const int vlane = live ? lane - slot * lpr : 0;   // idle lanes repeat a valid address and add nothing
    const int grp = (int)blockIdx.x / g.wgs_per_group, j = (int)blockIdx.x - grp * g.wgs_per_group;
    const int p0 = grp * g.group, G = g.group;
    const int GS = g.x_shared ? 1 : G;   // activation rows staged
    const int r0 = j * g.rows_per_wg;
    const int r1 = min(N, r0 + g.rows_per_wg);
    const int steps = r1 > r0 ? (r1 - r0 + S * R - 1) / (S * R) : 0;   // units a pair has here
    const int units = G * steps;
    const int n_u = (units > wave ? (units - wave + kWaves - 1) / kWaves : 0) * nch;   // this wave's units (wave, wave + 16, ..) x their steps

    // LDS: the group's quantized activation rows, then the results to combine
    int8_t *sq = reinterpret_cast<int8_t *>(smem);
    const int d_bytes = (GS * nb * 4 + 15) & ~15;   // the block sums behind it are read eight bytes at a time
    float *sd = reinterpret_cast<float *>(smem + GS * K);
    int16_t *sb = reinterpret_cast<int16_t *>(smem + GS * K + d_bytes);
    float *res = reinterpret_cast<float *>(smem + GS * K + d_bytes + GS * (K / 16) * 2);
    float *cwl = res + G * g.rows_per_wg;
    XTile xt;
    xt.qs = sq;
    xt.d = sd;
    xt.bs = sb;
    xt.kt = K;

    // the wave's first piece of the activation rows is requested ahead of its first weights (loads return in order)
    const int n_chunks = GS * nb;
    constexpr int kAhead = 2;
    float4 x_first[kAhead];
#pragma unroll
    for (int a = 0; a < kAhead; ++a) {
        const int c = wave + kWaves * a;
        x_first[a] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c < n_chunks) {
            const int s = c / nb, ch = c - s * nb;
            x_first[a] = *reinterpret_cast<const float4 *>(g.x + (int64_t)((p0 + s) / g.x_div) * K + ch * 256 + 4 * lane);
        }
    }
    float cw_mine = 0.f;   // routing weights go through LDS: the adding threads would otherwise wait for them at the very end
    if (COMBINE && tid < G) cw_mine = g.cw[p0 + tid];
    if (j == 0 && tid < G) {   // one workgroup of the group reports ids that name no expert
        const int e = g.ids[p0 + tid];
        if (e < 0 || e >= g.n_expert) atomicOr(g.error_flag, 1);
    }

    // unit u = (row step st, pair s of the group), pairs running fastest: with 1, 2, 4, 8 or 16 pairs a group a wave
    // (units wave, wave + 16, ..) stays with ONE pair, whose expert it reads once (a scalar load) and whose
    // activation slices it keeps in registers; otherwise both are fetched again whenever the pair changes
    struct Unit {
        int s, row;
    };
    auto unit_of = [&](int i) {
        Unit u;
        const int idx = wave + kWaves * (LONGK ? i / nch : i);
        const int st = idx / G;
        u.s = idx - st * G;
        u.row = r0 + st * S * R;
        return u;
    };
    auto expert_of = [&](int s_) {   // -1: the pair names no expert and is left out
        const int e = uniform(g.ids[p0 + s_]);
        return e >= 0 && e < g.n_expert ? e : -1;
    };
    int issue_s = -1, issue_e = -1;
    auto issue = [&](Raw<QT> (&raw)[NT], int i) {
        const Unit u = unit_of(i);
        if (u.s != issue_s) {
            issue_s = u.s;
            issue_e = expert_of(u.s);
        }
        const int64_t first = (int64_t)(issue_e < 0 ? 0 : issue_e) * N + u.row;   // (a pair left out loads somewhere valid)
        RowPtr<QT> rp;
        rp.set(g.w0, first);
        if constexpr (LONGK) {   // lanes past the end of the row repeat its last block
            const uint32_t blk = (uint32_t)min((i % nch) * 16 + (lane >> 2), nb - 1);
            raw[0].load(rp, blk, lane, 0);
            if constexpr (SWIGLU) {
                RowPtr<QT> ru;
                ru.set(g.w1, first);
                raw[NT - 1].load(ru, blk, lane, 0);
            }
        } else if constexpr (SWIGLU) {
            const uint32_t rel = (uint32_t)min(slot, r1 - 1 - u.row);
            raw[0].load(rp, (uint32_t)(vlane >> 2), vlane, rel);
            RowPtr<QT> ru;
            ru.set(g.w1, first);
            raw[NT - 1].load(ru, (uint32_t)(vlane >> 2), vlane, rel);
        } else {
#pragma unroll
            for (int r = 0; r < R; ++r)   // rows past the end of the range repeat its last row
                raw[r].load(rp, (uint32_t)(vlane >> 2), vlane, (uint32_t)min(r * S + slot, r1 - 1 - u.row));
        }
    };
    int cur_s = -1;
    bool cur_ok = false;
    Dot<QT> dx;
    float part[NT];   // LONGK: the row's sum so far
#pragma unroll
    for (int t = 0; t < NT; ++t) part[t] = 0.f;
    auto consume = [&](const Raw<QT> (&raw)[NT], int i) {
        const Unit u = unit_of(i);
        if (u.s != cur_s) {
            cur_s = u.s;
            cur_ok = expert_of(u.s) >= 0;
            if constexpr (!LONGK) dx.load_x(xt, g.x_shared ? 0 : u.s, 0, vlane);
        }
        float acc[NT];
        if constexpr (LONGK) {
            const int c = i % nch, left = nb - c * 16;          // super-blocks left in the row from this step on
            const bool there = (lane >> 2) < left;
            dx.load_x(xt, g.x_shared ? 0 : u.s, c * 4096, there ? lane : (lane & 3));   // (lanes past the end read the step's first block)
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                Frag<QT> f;
                f.unpack(raw[t], lane);
                part[t] += there ? dx.dot(f) : 0.f;
            }
            if (c + 1 < nch) return;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                acc[t] = slot_sum(part[t], lane, 64);
                part[t] = 0.f;
            }
        } else {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                Frag<QT> f;
                f.unpack(raw[t], vlane);
                acc[t] = slot_sum(live ? dx.dot(f) : 0.f, vlane, lpr);
            }
        }
#pragma unroll
        for (int t = 0; t < (SWIGLU ? 1 : R); ++t) {
            const int row = u.row + t * S + slot;
            if (live && vlane == 0 && row < r1) {
                float r = acc[t];
                if constexpr (SWIGLU) r = (r / (1.0f + expf(-r))) * acc[NT - 1];
                if constexpr (COMBINE) res[u.s * g.rows_per_wg + (row - r0)] = cur_ok ? r : 0.f;
                else if (cur_ok) g.y[(int64_t)(p0 + u.s) * N + row] = r;
            }
        }
    };

    Raw<QT> buf_a[NT], buf_b[NT];
    if (n_u > 0) issue(buf_a, 0);   // in flight while the activations are quantized

    if (COMBINE && tid < G) cwl[tid] = cw_mine;
    auto x_piece = [&](int c) {
        const int s = c / nb, ch = c - s * nb;
        return *reinterpret_cast<const float4 *>(g.x + (int64_t)((p0 + s) / g.x_div) * K + ch * 256 + 4 * lane);
    };
    float4 x_next = x_first[kAhead - 1];   // pieces beyond the first two are requested one round ahead
    for (int c = wave, a = 0; c < n_chunks; c += kWaves, ++a) {
        const int s = c / nb, ch = c - s * nb;
        const float4 v = a == 0 ? x_first[0] : x_next;
        if (a >= 1 && c + kWaves < n_chunks) x_next = x_piece(c + kWaves);
        int bsum;
        float dd;
        const uint32_t packed = wave_quantize_q8k(v, lane, bsum, dd);
        *reinterpret_cast<uint32_t *>(sq + s * K + ch * 256 + 4 * lane) = packed;
        if ((lane & 3) == 0) sb[s * (K / 16) + ch * 16 + (lane >> 2)] = (int16_t)bsum;
        if (lane == 0) sd[s * nb + ch] = dd;
    }
    __syncthreads();

    // two register buffers, the next unit's loads outstanding while this one is multiplied; no load is issued twice
    int i = 0;
    for (; i + 2 < n_u; i += 2) {
        issue(buf_b, i + 1);
        __builtin_amdgcn_sched_barrier(0);
        consume(buf_a, i);
        issue(buf_a, i + 2);
        __builtin_amdgcn_sched_barrier(0);
        consume(buf_b, i + 1);
    }
    if (i + 1 < n_u) {
        issue(buf_b, i + 1);
        __builtin_amdgcn_sched_barrier(0);
        consume(buf_a, i);
        consume(buf_b, i + 1);
    } else if (i < n_u) {
        consume(buf_a, i);
    }

    if constexpr (COMBINE) {
        __syncthreads();
        for (int i = tid; i < r1 - r0; i += kThreads) {
            float s = __fmul_rn(res[i], cwl[0]);
            for (int q = 1; q < G; ++q) s = __fadd_rn(s, __fmul_rn(res[q * g.rows_per_wg + i], cwl[q]));
            g.y[(int64_t)grp * N + r0 + i] = s;
        }
    }
}

template <int QT, bool SWIGLU, bool COMBINE, int R = 1, bool LONGK = false>
hipError_t launch_typed(const MoeDecodeArgs &g, unsigned grid, size_t lds, hipStream_t s) {
    auto kern = &moe_decode_kernel<QT, SWIGLU, COMBINE, R, LONGK>;
    static size_t allowed = 48 * 1024;
    if (lds > allowed) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        allowed = lds;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), lds, s, g);
    return hipGetLastError();
}

}  // namespace

namespace {
constexpr size_t kLdsBudget = 158 * 1024;
// LDS of the group's quantized rows: codes, scales (padded to 16 bytes), block sums
size_t staged_bytes(int64_t K, int64_t group) {
    return (size_t)group * K + (((size_t)group * (K / 256) * 4 + 15) & ~(size_t)15) + (size_t)group * (K / 16) * 2;
}
}  // namespace

// Every condition on the SHAPE that launch_moe_decode refuses a call for (the dispatch asks this before it picks the
// route, the launcher asserts the same predicate: one rule, so a shape the launcher would turn down never reaches it
// and takes the grouped route instead).  With it the launcher's LDS never exceeds the budget: the staged rows leave
// room for 64 result rows a pair, and the results a workgroup keeps are cut to what is left.
bool moe_decode_fits(int type, int64_t K, int64_t N, int64_t n_pairs, int64_t group, int64_t n_expert) {
    return (type == kTypeQ4_K || type == kTypeQ6_K) && K % 256 == 0 && K >= 256 && K <= (1 << 20) && n_pairs >= 1 &&
           n_pairs <= (1 << 20) && group >= 1 && group <= kMaxGroup && n_pairs % group == 0 && N >= 1 && N <= (1 << 24) &&
           n_expert >= 1 && staged_bytes(K, group) + (size_t)group * 4 * 64 + 64 <= kLdsBudget;
}

// args: t[0] (and t[1] = up when swiglu) expert stacks, x fp32 rows, x_div, ids, n_pairs, error_flag as for the
// pair mode of the grouped kernel; n_expert experts a stack.  combine_weights null: t[0].y is [n_pairs][N].
// Otherwise the pairs of a token (n_used of them, consecutive) are added with their routing weights and
// t[0].y is [n_pairs / n_used][N].
hipError_t launch_moe_decode(const GemvArgs &args, int n_expert, bool swiglu, const float *combine_weights, int n_used,
                             hipStream_t s) {
    const WeightView &w = args.t[0].w;
    if (args.n_pairs < 1 || args.x_div < 1 || w.nb < 1) return hipErrorInvalidValue;
    const int nb = (int)w.nb;
    const bool long_k = nb > 16;
    const int S = long_k ? 1 : 64 / (4 * nb);
    const int64_t steps_total = (w.N + S - 1) / S;
    // The launch is latency-bound (all loads of the call are in flight at once): the rows are spread over all
    // compute units, a unit or two a wave, at least half the waves of a workgroup busy.  The registers of a 16-wave
    // workgroup leave room for one a compute unit, so the grid stays within one round.
    const auto steps_for = [&](int group) {
        const int64_t max_wgs = std::max<int64_t>(1, (int64_t)cu_count() / (args.n_pairs / group));
        return std::max<int64_t>((steps_total + max_wgs - 1) / max_wgs, std::max<int64_t>(1, kWaves / 2 / group));
    };
    const auto grid_for = [&](int group) {
        const int64_t per = steps_for(group) * S;
        return (int64_t)(args.n_pairs / group) * ((w.N + per - 1) / per);
    };
    // Pairs a workgroup serves.  Combined results: the pairs of a token.  Otherwise one - unless that leaves compute
    // units without a workgroup (more pairs than half the units: 160 pairs were 160 workgroups): then 2, 4, 8 or 16
    // pairs that read the same activation row (consecutive pairs of a token), staged once, share a set of workgroups,
    // whichever count fills the round best.
    int group = combine_weights ? n_used : 1;
    static const bool no_share = tuning_int("QPROJ_MOE_DECODE_NO_SHARED_ROW", 0) != 0;
    if (!combine_weights && !no_share && grid_for(1) * 8 < (int64_t)cu_count() * 7) {
        int64_t best = grid_for(1);
        for (int c = 2; c <= kMaxGroup; c *= 2) {
            if (args.n_pairs % c != 0 || args.x_div % c != 0) continue;
            const int64_t gr = grid_for(c);
            if (gr <= cu_count() && gr > best) {
                best = gr;
                group = c;
            }
        }
    }
    const bool x_shared = !combine_weights && group > 1;
    if (!moe_decode_fits(w.type, w.K, w.N, args.n_pairs, x_shared ? 1 : group, n_expert) || args.n_pairs % group != 0 || !args.x ||
        !args.ids || !args.error_flag || (swiglu && combine_weights))
        return hipErrorInvalidValue;
    if (swiglu && (args.n_targets != 2 || args.t[1].w.type != w.type || args.t[1].w.K != w.K || args.t[1].w.N != w.N))
        return hipErrorInvalidValue;
    MoeDecodeArgs g{};
    g.w0 = w;
    g.w1 = swiglu ? args.t[1].w : w;
    g.x = args.x;
    g.x_div = args.x_div;
    g.ids = args.ids;
    g.n_pairs = args.n_pairs;
    g.n_expert = n_expert;
    g.error_flag = args.error_flag;
    g.y = args.t[0].y;
    g.cw = combine_weights;
    g.group = group;
    g.x_shared = x_shared ? 1 : 0;
    const int n_groups = args.n_pairs / group;
    int64_t steps_per_wg = steps_for(group);
    // the results a workgroup combines wait in LDS: 48 KB of them at most, less beside long staged rows (more
    // workgroups a group beyond that)
    const size_t staged = staged_bytes(w.K, x_shared ? 1 : group);
    if (combine_weights) {
        const size_t room = std::min<size_t>(48 * 1024, kLdsBudget - staged - 64);
        steps_per_wg = std::min<int64_t>(steps_per_wg, std::max<int64_t>(1, (int64_t)(room / 4 / group / S)));
    }
    g.rows_per_wg = (int)(steps_per_wg * S);
    g.wgs_per_group = (int)((w.N + g.rows_per_wg - 1) / g.rows_per_wg);
    const size_t lds = staged + (combine_weights ? (size_t)group * (g.rows_per_wg + 1) * 4 : 0);
    if (lds > 160 * 1024) return hipErrorInvalidValue;   // (cannot happen for a shape moe_decode_fits accepts; kept as a guard)
    if (dry_run()) {
        plan_note("moe_decode_kernel<%s%s%s>: an expert read per pair, %d pairs, %d pairs share a workgroup set%s, %d workgroups, LDS %zu B",
                  plan_type_name(w.type), swiglu ? ", gate/up + swiglu" : "", combine_weights ? ", weighted sum over a token's experts" : "",
                  args.n_pairs, group, x_shared ? " (one staged token row)" : "", n_groups * g.wgs_per_group, lds);
        return hipSuccess;
    }
    const unsigned grid = (unsigned)(n_groups * g.wgs_per_group);
    // two row steps a unit where a wave would otherwise walk four or more units of rows that fill under 4 KB a step
    static const int two_env = tuning_int("QPROJ_MOE_DECODE_TWO_STEPS", -1);
    const bool two = !long_k && (two_env >= 0 ? two_env != 0 : (!swiglu && group * steps_per_wg >= 4 * kWaves));
    if (long_k) {
        if (w.type == kTypeQ4_K) {
            if (swiglu) return launch_typed<kTypeQ4_K, true, false, 1, true>(g, grid, lds, s);
            return combine_weights ? launch_typed<kTypeQ4_K, false, true, 1, true>(g, grid, lds, s) : launch_typed<kTypeQ4_K, false, false, 1, true>(g, grid, lds, s);
        }
        if (swiglu) return launch_typed<kTypeQ6_K, true, false, 1, true>(g, grid, lds, s);
        return combine_weights ? launch_typed<kTypeQ6_K, false, true, 1, true>(g, grid, lds, s) : launch_typed<kTypeQ6_K, false, false, 1, true>(g, grid, lds, s);
    }
    if (w.type == kTypeQ4_K) {
        if (swiglu) return launch_typed<kTypeQ4_K, true, false>(g, grid, lds, s);
        if (two) return combine_weights ? launch_typed<kTypeQ4_K, false, true, 2>(g, grid, lds, s) : launch_typed<kTypeQ4_K, false, false, 2>(g, grid, lds, s);
        return combine_weights ? launch_typed<kTypeQ4_K, false, true>(g, grid, lds, s) : launch_typed<kTypeQ4_K, false, false>(g, grid, lds, s);
    }
    if (swiglu) return launch_typed<kTypeQ6_K, true, false>(g, grid, lds, s);
    if (two) return combine_weights ? launch_typed<kTypeQ6_K, false, true, 2>(g, grid, lds, s) : launch_typed<kTypeQ6_K, false, false, 2>(g, grid, lds, s);
    return combine_weights ? launch_typed<kTypeQ6_K, false, true>(g, grid, lds, s) : launch_typed<kTypeQ6_K, false, false>(g, grid, lds, s);
}

}  // namespace qproj
