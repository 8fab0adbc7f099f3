// Projection over fp32 activations (no activation rounding): y = dequant(W) . x with fp32
// accumulation.  Same lane geometry as the int8-activation kernels; the weights are expanded
// in registers (v_cvt_f32_ubyte) and the scale / min are applied once per lane per sub-block:
//   sum (d*sc*q - dmin*m) x = (d*sc) * sum q x - (dmin*m) * sum x.
// Dense only, 1..4 activation rows per pass.
#include "qproj_device.h"
#include "qproj_internal.h"

namespace qproj {

namespace {

__host__ __device__ constexpr int tile_kf(int mt) { return mt <= 2 ? 4096 : 2048; }

__device__ __forceinline__ float ub(uint32_t w, int j) { return (float)((w >> (8 * j)) & 0xffu); }
__device__ __forceinline__ float sb8(uint32_t w, int j) { return (float)(int)(int8_t)(w >> (8 * j)); }
// c + sum of the four unsigned bytes of w times the four floats of x
__device__ __forceinline__ float dot4f(uint32_t w, const float4 &x, float c) {
    return fmaf(ub(w, 3), x.w, fmaf(ub(w, 2), x.z, fmaf(ub(w, 1), x.y, fmaf(ub(w, 0), x.x, c))));
}

template <int QT> struct FragF;

template <> struct FragF<kTypeQ4_K> {
    uint32_t lo[4], hi[4];
    float d0, d1, mn0, mn1;
    static constexpr int kChunk = 2048;
    __device__ __forceinline__ void load(const WeightView &w, int64_t row, int64_t sb, int lane) {
        const int sub = lane & 7, c = sub >> 1, h = sub & 1;
        const uint8_t *blk = w.q4k + (row * w.nb + sb) * 144;
        const uint4 hd = *reinterpret_cast<const uint4 *>(blk);
        const uint4 q = *reinterpret_cast<const uint4 *>(blk + 16 + 32 * c + 16 * h);
        const uint32_t qq[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            lo[i] = qq[i] & 0x0f0f0f0fu;
            hi[i] = (qq[i] >> 4) & 0x0f0f0f0fu;
        }
        const ScalesK4 s = unpack_scales_k4(hd.y, hd.z, hd.w);
        const float d = h2f(hd.x), dmin = h2f(hd.x >> 16);
        d0 = d * (float)scale_k4(s, 2 * c);
        d1 = d * (float)scale_k4(s, 2 * c + 1);
        mn0 = dmin * (float)min_k4(s, 2 * c);
        mn1 = dmin * (float)min_k4(s, 2 * c + 1);
    }
    // x: tile pointer of this activation row; c0: chunk offset inside the tile
    __device__ __forceinline__ float dot(const float *x, int c0, int lane) const {
        const int sbl = lane >> 3, sub = lane & 7, c = sub >> 1, h = sub & 1;
        const float *xl = x + c0 + sbl * 256 + 64 * c + 16 * h;
        const float *xh = xl + 32;
        float ql = 0.f, sl = 0.f, qh = 0.f, sh = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 a = *reinterpret_cast<const float4 *>(xl + 4 * i);
            const float4 b = *reinterpret_cast<const float4 *>(xh + 4 * i);
            ql = dot4f(lo[i], a, ql);
            sl += (a.x + a.y) + (a.z + a.w);
            qh = dot4f(hi[i], b, qh);
            sh += (b.x + b.y) + (b.z + b.w);
        }
        return fmaf(d0, ql, -(mn0 * sl)) + fmaf(d1, qh, -(mn1 * sh));
    }
};

template <> struct FragF<kTypeQ6_K> {
    uint32_t q[4][2];
    float ds[4];
    static constexpr int kChunk = 2048;
    __device__ __forceinline__ void load(const WeightView &w, int64_t row, int64_t sb, int lane) {
        const int i = lane & 7, h = i >> 2, l0 = 8 * (i & 3);
        const int64_t b = row * w.nb + sb;
        const uint2 A = *reinterpret_cast<const uint2 *>(w.q6_ql + b * 128 + 64 * h + l0);
        const uint2 B = *reinterpret_cast<const uint2 *>(w.q6_ql + b * 128 + 64 * h + 32 + l0);
        const uint2 H = *reinterpret_cast<const uint2 *>(w.q6_qh + b * 64 + 32 * h + l0);
        const uint2 S = *reinterpret_cast<const uint2 *>(w.q6_sc + b * 16 + 8 * h);
        const uint32_t a[2] = {A.x, A.y}, bb[2] = {B.x, B.y}, hh[2] = {H.x, H.y};
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            q[0][t] = (a[t] & 0x0f0f0f0fu) | ((hh[t] << 4) & 0x30303030u);
            q[1][t] = (bb[t] & 0x0f0f0f0fu) | ((hh[t] << 2) & 0x30303030u);
            q[2][t] = ((a[t] >> 4) & 0x0f0f0f0fu) | (hh[t] & 0x30303030u);
            q[3][t] = ((bb[t] >> 4) & 0x0f0f0f0fu) | ((hh[t] >> 2) & 0x30303030u);
        }
        const int e = l0 >> 4;
        const uint64_t s64 = (uint64_t)S.x | ((uint64_t)S.y << 32);
        const float d = h2f(w.q6_d[b]);
#pragma unroll
        for (int g = 0; g < 4; ++g) ds[g] = d * (float)(int)(int8_t)(s64 >> (8 * (2 * g + e)));
    }
    __device__ __forceinline__ float dot(const float *x, int c0, int lane) const {
        const int sbl = lane >> 3, i = lane & 7, h = i >> 2, l0 = 8 * (i & 3);
        const float *xb = x + c0 + sbl * 256 + 128 * h + l0;
        float r = 0.f;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float4 a = *reinterpret_cast<const float4 *>(xb + 32 * g);
            const float4 b = *reinterpret_cast<const float4 *>(xb + 32 * g + 4);
            const float sq = dot4f(q[g][1], b, dot4f(q[g][0], a, 0.f));
            const float sx = ((a.x + a.y) + (a.z + a.w)) + ((b.x + b.y) + (b.z + b.w));
            r = fmaf(ds[g], fmaf(-32.f, sx, sq), r);
        }
        return r;
    }
};

template <> struct FragF<kTypeQ8_0> {
    uint32_t q[4];
    float d;
    static constexpr int kChunk = 1024;
    __device__ __forceinline__ void load(const WeightView &w, int64_t row, int64_t blk, int lane) {
        const uint4 v = *reinterpret_cast<const uint4 *>(w.q8_qs + row * w.K + blk * 32 + 16 * (lane & 1));
        q[0] = v.x; q[1] = v.y; q[2] = v.z; q[3] = v.w;
        d = h2f(w.q8_d[row * w.nb + blk]);
    }
    __device__ __forceinline__ float dot(const float *x, int c0, int lane) const {
        const float *xb = x + c0 + 16 * lane;
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 a = *reinterpret_cast<const float4 *>(xb + 4 * i);
            s = fmaf(sb8(q[i], 3), a.w, fmaf(sb8(q[i], 2), a.z, fmaf(sb8(q[i], 1), a.y, fmaf(sb8(q[i], 0), a.x, s))));
        }
        return d * s;
    }
};

template <int QT, int MT, int R>
__global__ __launch_bounds__(256) void gemv_f32_kernel(const GemvArgs args) {
    extern __shared__ __align__(16) uint8_t smem[];
    float *sx = reinterpret_cast<float *>(smem);
    constexpr int KT = tile_kf(MT);
    constexpr int CH = FragF<QT>::kChunk;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    WeightView w = args.t[0].w;
    float *y = args.t[0].y;
    int first = 0;
#pragma unroll
    for (int i = 1; i < kMaxTargets; ++i) {
        if (i < args.n_targets && (int)blockIdx.x >= args.t[i].first_block) {
            w = args.t[i].w;
            y = args.t[i].y;
            first = args.t[i].first_block;
        }
    }
    const int64_t N = w.N, K = w.K, nb = w.nb;
    const int64_t row0 = ((int64_t)((int)blockIdx.x - first) * 4 + wave) * R;

    float acc[MT][R];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[m][r] = 0.f;

    for (int64_t kt0 = 0; kt0 < K; kt0 += KT) {
        const int kt_len = (int)((K - kt0) < KT ? (K - kt0) : KT);
        const int kt_pad = (kt_len + CH - 1) / CH * CH;
        __syncthreads();
        for (int m = 0; m < MT; ++m) {
            for (int i = threadIdx.x; i < kt_pad / 4; i += 256) {
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (m < args.M && i * 4 < kt_len) v = *reinterpret_cast<const float4 *>(args.x + (int64_t)m * K + kt0 + i * 4);
                *reinterpret_cast<float4 *>(sx + m * KT + i * 4) = v;
            }
        }
        __syncthreads();
        for (int c0 = 0; c0 < kt_len; c0 += CH) {
            const int64_t blk = (QT == kTypeQ8_0) ? (kt0 + c0) / 32 + (lane >> 1) : (kt0 + c0) / 256 + (lane >> 3);
            if (blk < nb) {
                FragF<QT> f[R];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    int64_t row = row0 + r;
                    if (row >= N) row = N - 1;
                    f[r].load(w, row, blk, lane);
                }
#pragma unroll
                for (int m = 0; m < MT; ++m)
#pragma unroll
                    for (int r = 0; r < R; ++r) acc[m][r] += f[r].dot(sx + m * KT, c0, lane);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float v = wave_sum(acc[m][r]);
            if (lane == 0 && m < args.M && row0 + r < N) y[(int64_t)m * N + row0 + r] = v;
        }
    }
}

template <int QT, int MT, int R>
hipError_t launch_f32(const GemvArgs &args, hipStream_t s) {
    GemvArgs a = args;
    int total = 0;
    for (int i = 0; i < a.n_targets; ++i) {
        a.t[i].first_block = total;
        total += (int)((a.t[i].w.N + 4 * R - 1) / (4 * R));
    }
    if (total == 0) return hipSuccess;
    if (dry_run()) {
        plan_note("gemv_f32_kernel<%s, %d rows>: fp32 activations x dequantized weights, grid %d x 256", plan_type_name(QT), MT, total);
        return hipSuccess;
    }
    hipLaunchKernelGGL((gemv_f32_kernel<QT, MT, R>), dim3((unsigned)total), dim3(256), (size_t)MT * tile_kf(MT) * 4, s, a);
    return hipGetLastError();
}

template <int QT>
hipError_t launch_f32_mt(const GemvArgs &args, int mt, hipStream_t s) {
    switch (mt) {
    case 1: return launch_f32<QT, 1, 2>(args, s);
    case 2: return launch_f32<QT, 2, 2>(args, s);
    case 4: return launch_f32<QT, 4, 1>(args, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace

hipError_t launch_gemv_f32(const GemvArgs &args, int mt, int, hipStream_t s) {
    switch (args.t[0].w.type) {
    case kTypeQ4_K: return launch_f32_mt<kTypeQ4_K>(args, mt, s);
    case kTypeQ6_K: return launch_f32_mt<kTypeQ6_K>(args, mt, s);
    case kTypeQ8_0: return launch_f32_mt<kTypeQ8_0>(args, mt, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace qproj
