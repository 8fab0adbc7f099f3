// Memory-bound projection kernels for 1..16 activation rows (decode and speculative verify),
// dense (MUL_MAT) and expert-grouped (MUL_MAT_ID), over quantized activations.
//
// Shape of the work: a workgroup is 4 waves; each wave owns R weight rows and walks K in
// chunks.  In one chunk every lane owns 32 weights (16 for Q8_0) of one super-block, fetched
// with one or two vector loads per row, so a wave streams 8 super-blocks (1152 B of Q4_K) per
// row per step, fully coalesced.  Activations are int8 (ggml's Q8_K / Q8_0 vec_dot_type)
// staged once per workgroup in LDS and shared by the R rows; all multiplies are v_dot4_i32_i8.
// Integer partial sums are exact; each lane keeps an fp32 partial per (activation row, weight
// row) and one DPP wave reduction per output finishes the dot product.
#include "gemv_frags.h"

namespace qproj {

namespace {

// K-tile staged in LDS per activation row count: MT * kTile bytes of int8 (<= 32 KiB).
// Never smaller than one chunk of the weight type (4096 for the K-quants).
__host__ __device__ constexpr int tile_k(int qt, int mt) {
    const int base = mt <= 1 ? 16384 : (mt == 2 ? 8192 : (mt == 4 ? 4096 : 2048));
    const int chunk = qt == kTypeQ8_0 ? 1024 : 4096;
    return base > chunk ? base : chunk;
}

struct TargetSel {
    WeightView w;
    float *y;
    int bx;
};

__device__ __forceinline__ TargetSel select_target(const GemvArgs &a) {
    TargetSel s;
    s.w = a.t[0].w;
    s.y = a.t[0].y;
    int first = 0;
#pragma unroll
    for (int i = 1; i < kMaxTargets; ++i) {
        if (i < a.n_targets && (int)blockIdx.x >= a.t[i].first_block) {
            s.w = a.t[i].w;
            s.y = a.t[i].y;
            first = a.t[i].first_block;
        }
    }
    s.bx = (int)blockIdx.x - first;
    return s;
}

template <int QT, int MT>
__device__ __forceinline__ void stage_tile(uint8_t *smem, const ActView &a, const int64_t *arow, int kt0,
                                           int kt_len, int kt_pad) {
    constexpr int KT = tile_k(QT, MT);
    constexpr int BLK = Geo<QT>::kBlk;
    int8_t *sq = reinterpret_cast<int8_t *>(smem);
    float *sd = reinterpret_cast<float *>(smem + MT * KT);
    int16_t *sb = reinterpret_cast<int16_t *>(smem + MT * KT + MT * (KT / BLK) * 4);
    const int tid = threadIdx.x;
    for (int m = 0; m < MT; ++m) {
        const int64_t r = arow[m];
        for (int i = tid; i < kt_pad / 16; i += 256) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (r >= 0 && i * 16 < kt_len) v = *reinterpret_cast<const uint4 *>(a.qs + r * a.K + kt0 + i * 16);
            *reinterpret_cast<uint4 *>(sq + m * KT + i * 16) = v;
        }
        for (int i = tid; i < kt_pad / BLK; i += 256) {
            float v = 0.f;
            if (r >= 0 && i * BLK < kt_len) v = a.d[r * (a.K / BLK) + kt0 / BLK + i];
            sd[m * (KT / BLK) + i] = v;
        }
        if (QT != kTypeQ8_0) {
            for (int i = tid; i < kt_pad / 16; i += 256) {
                int16_t v = 0;
                if (r >= 0 && i * 16 < kt_len) v = a.bsums[r * (a.K / 16) + kt0 / 16 + i];
                sb[m * (KT / 16) + i] = v;
            }
        }
    }
}

constexpr size_t gemv_smem_bytes(int qt, int mt) {
    const int kt = tile_k(qt, mt);
    const int blk = qt == kTypeQ8_0 ? 32 : 256;
    return (size_t)mt * kt + (size_t)mt * (kt / blk) * 4 + (qt != kTypeQ8_0 ? (size_t)mt * (kt / 16) * 2 : 0);
}

// QT weight type; MT activation rows per pass; R weight rows per wave; GROUPED: blockIdx.y is an
// expert and the activation rows are that expert's (token, slot) pairs; SWIGLU: targets 0 and 1
// are gate and up of the same expert and the output is silu(gate.x) * (up.x).
template <int QT, int MT, int R, bool GROUPED, bool SWIGLU>
__global__ __launch_bounds__(256) void gemv_q8act_kernel(const GemvArgs args) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int KT = tile_k(QT, MT);
    constexpr int CH = Geo<QT>::kChunk;
    constexpr int BLK = Geo<QT>::kBlk;
    constexpr int NT = SWIGLU ? 2 : 1;

    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    TargetSel T;
    if (SWIGLU) {
        T.w = args.t[0].w;
        T.y = args.t[0].y;
        T.bx = blockIdx.x;
    } else {
        T = select_target(args);
    }
    const int64_t N = T.w.N, K = T.w.K, nb = T.w.nb;
    const int64_t row0 = ((int64_t)T.bx * 4 + wave) * R;
    const int64_t e_base = GROUPED ? (int64_t)blockIdx.y * N : 0;

    int p_begin = 0, p_end = args.M;
    if (GROUPED) {
        p_begin = args.offsets[blockIdx.y];
        p_end = args.offsets[blockIdx.y + 1];
    }

    XTile xt;
    xt.qs = reinterpret_cast<const int8_t *>(smem);
    xt.d = reinterpret_cast<const float *>(smem + MT * KT);
    xt.bs = reinterpret_cast<const int16_t *>(smem + MT * KT + MT * (KT / BLK) * 4);
    xt.kt = KT;

    for (int pb = p_begin; pb < p_end; pb += MT) {
        int64_t arow[MT], yrow[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (pb + m < p_end) {
                const int64_t p = GROUPED ? (int64_t)args.order[pb + m] : (int64_t)(pb + m);
                arow[m] = GROUPED ? p / args.x_div : p;
                yrow[m] = p;
            } else {
                arow[m] = -1;
                yrow[m] = -1;
            }
        }
        float acc[NT][MT][R];
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int r = 0; r < R; ++r) acc[t][m][r] = 0.f;

        for (int64_t kt0 = 0; kt0 < K; kt0 += KT) {
            const int kt_len = (int)((K - kt0) < KT ? (K - kt0) : KT);
            const int kt_pad = (kt_len + CH - 1) / CH * CH;
            __syncthreads();
            stage_tile<QT, MT>(smem, args.a, arow, (int)kt0, kt_len, kt_pad);
            __syncthreads();
            for (int c0 = 0; c0 < kt_len; c0 += CH) {
                // block index of this lane inside the row
                const int64_t blk = lane_block<QT>(kt0 + c0, lane);
                if (blk < nb) {
                    Frag<QT> f[NT][R];
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
#pragma unroll
                        for (int r = 0; r < R; ++r) {
                            int64_t row = row0 + r;
                            if (row >= N) row = N - 1;
                            RowPtr<QT> rp;
                            rp.set(t == 0 ? T.w : args.t[1].w, e_base + row);
                            Raw<QT> raw;
                            raw.load(rp, (uint32_t)blk, lane);
                            f[t][r].unpack(raw, lane);
                        }
                    }
#pragma unroll
                    for (int m = 0; m < MT; ++m) {
                        Dot<QT> dx;
                        dx.load_x(xt, m, c0, lane);
#pragma unroll
                        for (int t = 0; t < NT; ++t)
#pragma unroll
                            for (int r = 0; r < R; ++r) acc[t][m][r] += dx.dot(f[t][r]);
                    }
                }
            }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float v = wave_sum(acc[0][m][r]);
                if (SWIGLU) {
                    const float u = wave_sum(acc[NT - 1][m][r]);
                    v = (v / (1.0f + expf(-v))) * u;
                }
                if (lane == 0 && yrow[m] >= 0 && row0 + r < N) T.y[yrow[m] * N + row0 + r] = v;
            }
        }
    }
}

template <int QT, int MT, int R, bool GROUPED, bool SWIGLU>
hipError_t launch_one(const GemvArgs &args, int n_experts_grid, hipStream_t s) {
    int total_blocks = 0;
    GemvArgs a = args;
    const int n_t = SWIGLU ? 1 : a.n_targets;
    for (int i = 0; i < n_t; ++i) {
        a.t[i].first_block = total_blocks;
        total_blocks += (int)((a.t[i].w.N + 4 * R - 1) / (4 * R));
    }
    if (total_blocks == 0) return hipSuccess;
    if (dry_run()) {
        plan_note("gemv_q8act_kernel<%s, %d rows, %d weight rows a wave%s%s>: grid %d x %d", plan_type_name(QT), MT, R, GROUPED ? ", expert-grouped" : "",
                  SWIGLU ? ", swiglu" : "", total_blocks, GROUPED ? n_experts_grid : 1);
        return hipSuccess;
    }
    const dim3 grid((unsigned)total_blocks, (unsigned)(GROUPED ? n_experts_grid : 1));
    constexpr size_t smem = gemv_smem_bytes(QT, MT);
    if (smem > 48 * 1024) {  // above the default dynamic-LDS allowance: opt in once per kernel
        static hipError_t attr = hipFuncSetAttribute(
            reinterpret_cast<const void *>(&gemv_q8act_kernel<QT, MT, R, GROUPED, SWIGLU>),
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (attr != hipSuccess) return attr;
    }
    hipLaunchKernelGGL((gemv_q8act_kernel<QT, MT, R, GROUPED, SWIGLU>), grid, dim3(256), smem, s, a);
    return hipGetLastError();
}

template <int QT, bool GROUPED, bool SWIGLU>
hipError_t launch_by_mt(const GemvArgs &args, int mt, int n_experts_grid, hipStream_t s) {
    switch (mt) {
    case 1: return launch_one<QT, 1, SWIGLU ? 2 : 4, GROUPED, SWIGLU>(args, n_experts_grid, s);
    case 2: return launch_one<QT, 2, 2, GROUPED, SWIGLU>(args, n_experts_grid, s);
    case 4: return launch_one<QT, 4, 2, GROUPED, SWIGLU>(args, n_experts_grid, s);
    case 8: return launch_one<QT, 8, SWIGLU ? 1 : 2, GROUPED, SWIGLU>(args, n_experts_grid, s);
    case 16: return launch_one<QT, 16, 1, GROUPED, SWIGLU>(args, n_experts_grid, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

hipError_t launch_gemv_q8act(const GemvArgs &args, int mt, int n_experts_grid, hipStream_t s) {
    const bool grouped = args.order != nullptr;
    switch (args.t[0].w.type) {
    case kTypeQ4_K:
        return grouped ? launch_by_mt<kTypeQ4_K, true, false>(args, mt, n_experts_grid, s)
                       : launch_by_mt<kTypeQ4_K, false, false>(args, mt, 1, s);
    case kTypeQ6_K:
        return grouped ? launch_by_mt<kTypeQ6_K, true, false>(args, mt, n_experts_grid, s)
                       : launch_by_mt<kTypeQ6_K, false, false>(args, mt, 1, s);
    case kTypeQ8_0:
        return grouped ? launch_by_mt<kTypeQ8_0, true, false>(args, mt, n_experts_grid, s)
                       : launch_by_mt<kTypeQ8_0, false, false>(args, mt, 1, s);
    default:
        return hipErrorInvalidValue;
    }
}

// gate and up of the same experts in one pass, SwiGLU in the epilogue: h[pair][n]
hipError_t launch_moe_swiglu_gemv(const GemvArgs &args, int mt, int n_experts_grid, hipStream_t s) {
    switch (args.t[0].w.type) {
    case kTypeQ4_K: return launch_by_mt<kTypeQ4_K, true, true>(args, mt, n_experts_grid, s);
    case kTypeQ6_K: return launch_by_mt<kTypeQ6_K, true, true>(args, mt, n_experts_grid, s);
    case kTypeQ8_0: return launch_by_mt<kTypeQ8_0, true, true>(args, mt, n_experts_grid, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace qproj
