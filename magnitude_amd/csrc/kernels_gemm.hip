// Prefill projection: Q4_K weights x per-32 int8 activations on the int8 matrix cores.
//
//   y[m][n] = sum_blk (d_n*sc_{n,blk}) * da_{m,blk} * I_{m,n,blk} - (dmin_n*mn_{n,blk}) * (da_{m,blk}*isum_{m,blk})
//   I_{m,n,blk} = sum over the 32 weights of the sub-block of q * a      (exact, int32)
//
// A workgroup owns a 128 (tokens) x 128 (weight rows) tile and walks K in steps of 128 (four
// sub-blocks).  Per step the 4-bit weights are expanded to int8 into LDS together with the
// activation tile; each of the 4 waves owns a 64x64 sub-tile = 2x2 v_mfma_i32_32x32x32_i8
// products per sub-block.  An int32 accumulator is only meaningful inside one sub-block
// (both operands change scale every 32), so every product is folded into the fp32 accumulators
// right away: acc += float(I) * (da * ws) - asum * wm.
#include "qproj_device.h"
#include "qproj_internal.h"

namespace qproj {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, BK = 128;
constexpr int LDT = BK + 16;  // LDS row stride in bytes, padded against bank conflicts

struct GemmSmem {
    int8_t a[BM * LDT];      // activations  [m][k]
    int8_t b[BN * LDT];      // weights      [n][k], nibbles expanded
    float a_d[4][BM];        // da           [sub-block][m]
    float a_s[4][BM];        // da * isum
    float w_s[4][BN];        // d * sc       [sub-block][n]
    float w_m[4][BN];        // dmin * mn
};

__global__ __launch_bounds__(256) void gemm_q4k_q8x32_kernel(const WeightView w, const ActView a, int64_t M,
                                                             float *__restrict__ y) {
    __shared__ GemmSmem sm;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t n0 = (int64_t)blockIdx.x * BN, m0 = (int64_t)blockIdx.y * BM;
    const int64_t N = w.N, K = w.K;
    const int64_t kb32 = K / 32;

    float acc[2][2][16];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    for (int64_t k0 = 0; k0 < K; k0 += BK) {
        __syncthreads();
        // ---- activations: 128 rows x 128 B
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = tid + 256 * i;
            const int row = idx >> 3, seg = idx & 7;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (m0 + row < M) v = *reinterpret_cast<const uint4 *>(a.qs + (m0 + row) * K + k0 + 16 * seg);
            *reinterpret_cast<uint4 *>(sm.a + row * LDT + 16 * seg) = v;
        }
        // ---- weights: 128 rows x half a super-block (two 64-weight chunks = 64 packed bytes)
        {
            const int row = tid >> 1, ch = tid & 1;
            int64_t n = n0 + row;
            if (n >= N) n = N - 1;
            const int64_t sb = k0 >> 8;
            const int c = (int)((k0 & 255) >> 6) + ch;  // chunk inside the super-block
            const uint8_t *blk = w.q4k + (n * w.nb + sb) * 144;
            const uint4 p0 = *reinterpret_cast<const uint4 *>(blk + 16 + 32 * c);
            const uint4 p1 = *reinterpret_cast<const uint4 *>(blk + 16 + 32 * c + 16);
            const uint32_t pk[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
            uint32_t *dst = reinterpret_cast<uint32_t *>(sm.b + row * LDT + 64 * ch);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                dst[i] = pk[i] & 0x0f0f0f0fu;             // sub-block 2c
                dst[8 + i] = (pk[i] >> 4) & 0x0f0f0f0fu;  // sub-block 2c+1
            }
        }
        // ---- scales
        if (tid < 128) {
            int64_t n = n0 + tid;
            if (n >= N) n = N - 1;
            const uint4 hd = *reinterpret_cast<const uint4 *>(w.q4k + (n * w.nb + (k0 >> 8)) * 144);
            const ScalesK4 s = unpack_scales_k4(hd.y, hd.z, hd.w);
            const float d = h2f(hd.x), dmin = h2f(hd.x >> 16);
            const int j0 = (int)((k0 & 255) >> 5);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                sm.w_s[j][tid] = d * (float)scale_k4(s, j0 + j);
                sm.w_m[j][tid] = dmin * (float)min_k4(s, j0 + j);
            }
        } else {
            const int row = tid - 128;
            float4 dv = make_float4(0.f, 0.f, 0.f, 0.f);
            int4 sv = make_int4(0, 0, 0, 0);
            if (m0 + row < M) {
                dv = *reinterpret_cast<const float4 *>(a.d + (m0 + row) * kb32 + (k0 >> 5));
                sv = *reinterpret_cast<const int4 *>(a.isum + (m0 + row) * kb32 + (k0 >> 5));
            }
            sm.a_d[0][row] = dv.x; sm.a_d[1][row] = dv.y; sm.a_d[2][row] = dv.z; sm.a_d[3][row] = dv.w;
            sm.a_s[0][row] = dv.x * (float)sv.x; sm.a_s[1][row] = dv.y * (float)sv.y;
            sm.a_s[2][row] = dv.z * (float)sv.z; sm.a_s[3][row] = dv.w * (float)sv.w;
        }
        __syncthreads();

        // ---- four sub-blocks
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            v4i af[2], bf[2];
            float ws[2], wmn[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                af[i] = *reinterpret_cast<const v4i *>(sm.a + (wm * 64 + i * 32 + (lane & 31)) * LDT + kb * 32 + 16 * (lane >> 5));
                bf[i] = *reinterpret_cast<const v4i *>(sm.b + (wn * 64 + i * 32 + (lane & 31)) * LDT + kb * 32 + 16 * (lane >> 5));
                ws[i] = sm.w_s[kb][wn * 64 + i * 32 + (lane & 31)];
                wmn[i] = sm.w_m[kb][wn * 64 + i * 32 + (lane & 31)];
            }
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                float ad[16], as[16];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int r = wm * 64 + i * 32 + 8 * g + 4 * (lane >> 5);
                    const float4 d4 = *reinterpret_cast<const float4 *>(&sm.a_d[kb][r]);
                    const float4 s4 = *reinterpret_cast<const float4 *>(&sm.a_s[kb][r]);
                    ad[4 * g + 0] = d4.x; ad[4 * g + 1] = d4.y; ad[4 * g + 2] = d4.z; ad[4 * g + 3] = d4.w;
                    as[4 * g + 0] = s4.x; as[4 * g + 1] = s4.y; as[4 * g + 2] = s4.z; as[4 * g + 3] = s4.w;
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    v16i z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    const v16i I = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], z, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        acc[i][j][v] = fmaf((float)I[v], ad[v] * ws[j], acc[i][j][v]);
                        acc[i][j][v] = fmaf(-as[v], wmn[j], acc[i][j][v]);
                    }
                }
            }
        }
    }

    // ---- store: accumulator register v of lane l is row 8*(v/4) + 4*(l/32) + v%4, column l%32
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int64_t n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int64_t m = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (m < M && n < N) y[m * N + n] = acc[i][j][v];
            }
        }
    }
}

}  // namespace

hipError_t launch_gemm_q8x32(const WeightView &w, const ActView &a, int64_t M, float *y, hipStream_t s) {
    if (w.type != kTypeQ4_K || w.K % BK != 0) return hipErrorInvalidValue;
    const dim3 grid((unsigned)((w.N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
    hipLaunchKernelGGL(gemm_q4k_q8x32_kernel, grid, dim3(256), 0, s, w, a, M, y);
    return hipGetLastError();
}

}  // namespace qproj
