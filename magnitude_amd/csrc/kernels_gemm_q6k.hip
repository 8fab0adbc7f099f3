// Prefill-sized batches for Q6_K weights x ggml Q8_K activations on the int8 matrix cores.
//
//   y[m][n] = sum_sb d_n * dx_m * sum_{s<16} sc_{n,s} * sum_{k in s} (q_k - 32) * a_k
//
// A Q6_K sub-block is 16 weights with a signed 8-bit scale: sc*q does not fit an int8 operand in
// any two-way split, so each sub-block gets one v_mfma_i32_32x32x16_i8 on the raw 6-bit codes
// (0..63) and the vector ALU multiplies the 16 results of a lane by the lane's scale into an
// int32 sum that lives for the whole super-block (one mad per output and sub-block).  The -32 of
// every code is taken out exactly with the activation block sums the quantizer already wrote:
// sum_s sc_s * bsum_s is a K=16 product per super-block, run as two more matrix instructions with
// the 12-bit sums split into a signed high byte and a 6-bit low byte (bsum = 64*hi + lo).  The
// vector ALU touches floating point once per 256 weights.
//
// Layout of the work is that of the Q4_K kernel for the same activations: 64 tokens x 32*NW weight
// rows per workgroup, each wave 64 tokens x 32 rows (one weight operand feeds both token tiles);
// each wave fetches the ql/qh/scale planes of its 32 rows with consecutive lanes on consecutive
// 16-byte pieces and parks them in wave-private LDS strips, from which every lane picks the eight
// bytes of its own row it needs per sub-block; LDS otherwise holds one super-block of
// activations, double-buffered, so there is one workgroup barrier per 256 weights.
#include "qproj_device.h"
#include "qproj_internal.h"
#include "gemm_tiles.h"

namespace qproj {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int LA = 256 + 16;   // activation row stride in LDS (bytes)
constexpr int SQL = 128 + 8;   // strip row strides: conflict-free for 8-byte reads by consecutive rows
constexpr int SQH = 64 + 8;

template <int NW, int JT>   // NW waves of 32 weight rows each, JT token tiles of 32
struct Q6Smem {
    // activations of one super-block, per token: the first eight bytes of the 16 sub-blocks, then
    // the second eight bytes of the 16 sub-blocks (a lane's operands of two neighbouring
    // sub-blocks are then one 16-byte read)
    int8_t a[2][32 * JT * LA];
    int16_t bs[2][32 * JT * 16];   // activation block sums per 16
    float dx[2][32 * JT];
    uint8_t ql[NW][32 * SQL];
    uint8_t qh[NW][32 * SQH];
    int8_t sc[NW][32 * 16];
};

__device__ __forceinline__ long as_i64(uint32_t lo, uint32_t hi) { return (long)(((uint64_t)hi << 32) | lo); }

template <int NW, int JT>
__global__ __launch_bounds__(64 * NW, 2) void gemm_q6k_q8k_kernel(const WeightView w, const ActView a, int64_t M,
                                                                 float *__restrict__ y, float *__restrict__ part) {
    constexpr int NT = 64 * NW, TN = 32 * NW, TM = 32 * JT;
    constexpr int PA = TM * 16 / NT;   // 16-byte activation pieces a thread moves per super-block
    static_assert(PA >= 1 && TM * 2 <= NT, "tile does not fit the staging scheme");
    extern __shared__ __align__(16) uint8_t smem_raw[];
    Q6Smem<NW, JT> &sm = *reinterpret_cast<Q6Smem<NW, JT> *>(smem_raw);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t N = w.N, K = w.K, nb = w.nb;
    int tile_n, tile_m;
    tile_of_workgroup((int)((N + TN - 1) / TN), (int)((M + TM - 1) / TM), tile_n, tile_m);
    const int64_t n0 = (int64_t)tile_n * TN, m0 = (int64_t)tile_m * TM;
    const int l32 = lane & 31, lh = lane >> 5;

    v16f acc[JT];
#pragma unroll
    for (int j = 0; j < JT; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

    // ---- global -> register -> LDS plumbing: wave-uniform bases plus 32-bit lane offsets; rows past
    // the edge of the matrix repeat the last valid row (their results are never stored)
    const int64_t wave_row0 = n0 + wave * 32 < N ? n0 + wave * 32 : N - 1;
    const int wrow_cap = (int)(N - 1 - wave_row0 < 31 ? N - 1 - wave_row0 : 31);
    const uint8_t *qlbase = w.q6_ql + wave_row0 * nb * 128;
    const uint8_t *qhbase = w.q6_qh + wave_row0 * nb * 64;
    const uint8_t *scbase = reinterpret_cast<const uint8_t *>(w.q6_sc) + wave_row0 * nb * 16;
    const uint16_t *dbase = w.q6_d + wave_row0 * nb;
    uint32_t qloff[4], qhoff[2];
    int qlpark[4], qhpark[2];
#pragma unroll
    for (int c = 0; c < 4; ++c) {   // 256 pieces of ql: row p / 8, part p % 8
        const int p = lane + 64 * c, r = (p >> 3) < wrow_cap ? (p >> 3) : wrow_cap;
        qloff[c] = (uint32_t)(r * (int)nb * 128 + 16 * (p & 7));
        qlpark[c] = (p >> 3) * SQL + 16 * (p & 7);
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {   // 128 pieces of qh: row p / 4, part p % 4
        const int p = lane + 64 * c, r = (p >> 2) < wrow_cap ? (p >> 2) : wrow_cap;
        qhoff[c] = (uint32_t)(r * (int)nb * 64 + 16 * (p & 3));
        qhpark[c] = (p >> 2) * SQH + 16 * (p & 3);
    }
    const int myrow = l32 < wrow_cap ? l32 : wrow_cap;
    const uint32_t scoff = (uint32_t)(myrow * (int)nb * 16);   // 32 pieces of scales: row l%32 (both halves store)
    const uint32_t doff = (uint32_t)(myrow * (int)nb);
    // activations: piece id = tid + NT*p -> token id / 16, sub-block id % 16
    const int mrow_cap = (int)(M - 1 - m0 < TM - 1 ? M - 1 - m0 : TM - 1);
    const int8_t *abase = a.qs + m0 * K;
    uint32_t aoffg[PA];
    int aoffl[PA];
#pragma unroll
    for (int p = 0; p < PA; ++p) {
        const int id = tid + NT * p, row = id >> 4, seg = id & 15;
        aoffg[p] = (uint32_t)((row < mrow_cap ? row : mrow_cap) * (int)K + 16 * seg);
        aoffl[p] = row * LA + 8 * seg;
    }
    // block sums: TM tokens x 32 bytes, thread t (mod 2*TM) moves 16 bytes; scale: thread t (mod TM)
    const uint8_t *bsbase = reinterpret_cast<const uint8_t *>(a.bsums) + m0 * nb * 32;
    const int bsrow = (tid & (2 * TM - 1)) >> 1;
    const uint32_t bsoffg = (uint32_t)((bsrow < mrow_cap ? bsrow : mrow_cap) * (int)nb * 32 + 16 * (tid & 1));
    const float *dxbase = a.d + m0 * nb;
    const uint32_t dxoffg = (uint32_t)(((tid & (TM - 1)) < mrow_cap ? (tid & (TM - 1)) : mrow_cap) * (int)nb);

    v4i sql[4], sqh[2], ssc, areg[PA], bsreg;
    float dxreg;
    uint32_t dcur = 0, dnext = 0;   // fp16 d of the lane's row: current super-block, next
    auto load_next = [&](int64_t sb) {   // activations first: they are wanted at the end of this trip already
#pragma unroll
        for (int p = 0; p < PA; ++p) areg[p] = *reinterpret_cast<const v4i *>(abase + sb * 256 + aoffg[p]);
        bsreg = *reinterpret_cast<const v4i *>(bsbase + sb * 32 + bsoffg);
        dxreg = dxbase[sb + dxoffg];
#pragma unroll
        for (int c = 0; c < 4; ++c) sql[c] = *reinterpret_cast<const v4i *>(qlbase + sb * 128 + qloff[c]);
#pragma unroll
        for (int c = 0; c < 2; ++c) sqh[c] = *reinterpret_cast<const v4i *>(qhbase + sb * 64 + qhoff[c]);
        ssc = *reinterpret_cast<const v4i *>(scbase + sb * 16 + scoff);
        dnext = dbase[sb + doff];
    };
    uint8_t *pql = sm.ql[wave], *pqh = sm.qh[wave];
    int8_t *psc = sm.sc[wave];
    auto store_next = [&](int buf) {
#pragma unroll
        for (int p = 0; p < PA; ++p) {
            *reinterpret_cast<v2i *>(sm.a[buf] + aoffl[p]) = areg[p].xy;
            *reinterpret_cast<v2i *>(sm.a[buf] + aoffl[p] + 128) = areg[p].zw;
        }
        // threads beyond the first 2*TM / TM repeat a store of the same value: no branch, no load sunk into one
        *reinterpret_cast<v4i *>(reinterpret_cast<uint8_t *>(sm.bs[buf]) + 16 * (tid & (2 * TM - 1))) = bsreg;
        sm.dx[buf][tid & (TM - 1)] = dxreg;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            *reinterpret_cast<v2i *>(pql + qlpark[c]) = sql[c].xy;
            *reinterpret_cast<v2i *>(pql + qlpark[c] + 8) = sql[c].zw;
        }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            *reinterpret_cast<v2i *>(pqh + qhpark[c]) = sqh[c].xy;
            *reinterpret_cast<v2i *>(pqh + qhpark[c] + 8) = sqh[c].zw;
        }
        *reinterpret_cast<v4i *>(psc + l32 * 16) = ssc;
        dcur = dnext;
    };

    const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    auto superblock = [&](int buf, uint32_t dbits) {
        const v4i scv = *reinterpret_cast<const v4i *>(psc + l32 * 16);   // the 16 scales of the lane's row
        const int8_t *ap = sm.a[buf] + l32 * LA + 128 * lh;
        v16i isum[JT];
        // ---- -32 * sum_s sc_s * bsum_s: block sums as 64*hi + lo against the scales of k-half l/32
        {
            const long bsc = lh ? as_i64((uint32_t)scv[2], (uint32_t)scv[3]) : as_i64((uint32_t)scv[0], (uint32_t)scv[1]);
#pragma unroll
            for (int j = 0; j < JT; ++j) {
                const v4i b = *reinterpret_cast<const v4i *>(reinterpret_cast<const uint8_t *>(sm.bs[buf]) +
                                                           (j * 32 + l32) * 32 + 16 * lh);
                uint32_t lo[4], hi[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    lo[c] = (uint32_t)b[c] & 0x003f003fu;
                    hi[c] = ((uint32_t)b[c] >> 6) & 0x00ff00ffu;   // bits 6..13 of each half: the low byte of (sum >> 6)
                }
                // bytes 0 and 2 of two dwords -> four bytes (v_perm_b32: selectors 0..3 second operand, 4..7 first)
                const long alo = as_i64(__builtin_amdgcn_perm(lo[1], lo[0], 0x06040200u), __builtin_amdgcn_perm(lo[3], lo[2], 0x06040200u));
                const long ahi = as_i64(__builtin_amdgcn_perm(hi[1], hi[0], 0x06040200u), __builtin_amdgcn_perm(hi[3], hi[2], 0x06040200u));
                const v16i tl = __builtin_amdgcn_mfma_i32_32x32x16_i8(alo, bsc, zi, 0, 0, 0);
                const v16i th = __builtin_amdgcn_mfma_i32_32x32x16_i8(ahi, bsc, zi, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 16; ++v) isum[j][v] = __mul24(th[v], -2048) + __mul24(tl[v], -32);
            }
        }
        // ---- the 16 sub-blocks: j = 8f + 2k + p holds weights 128f + 32k + 16p + (0..15)
#pragma unroll
        for (int f = 0; f < 2; ++f) {
            uint32_t wl[2][4], wh[2][4];
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                // bytes shared by the four sub-blocks k = 0..3 of (f, p): the lane's eight of each
                const v2i qa = *reinterpret_cast<const v2i *>(pql + l32 * SQL + 64 * f + 16 * p + 8 * lh);
                const v2i qb = *reinterpret_cast<const v2i *>(pql + l32 * SQL + 64 * f + 32 + 16 * p + 8 * lh);
                const v2i qh = *reinterpret_cast<const v2i *>(pqh + l32 * SQH + 32 * f + 16 * p + 8 * lh);
                const uint32_t ax = (uint32_t)qa.x, ay = (uint32_t)qa.y, bx = (uint32_t)qb.x, by = (uint32_t)qb.y;
                const uint32_t hx = (uint32_t)qh.x, hy = (uint32_t)qh.y;
                wl[p][0] = (ax & 0x0f0f0f0fu) | ((hx << 4) & 0x30303030u);
                wh[p][0] = (ay & 0x0f0f0f0fu) | ((hy << 4) & 0x30303030u);
                wl[p][1] = (bx & 0x0f0f0f0fu) | ((hx << 2) & 0x30303030u);
                wh[p][1] = (by & 0x0f0f0f0fu) | ((hy << 2) & 0x30303030u);
                wl[p][2] = ((ax >> 4) & 0x0f0f0f0fu) | (hx & 0x30303030u);
                wh[p][2] = ((ay >> 4) & 0x0f0f0f0fu) | (hy & 0x30303030u);
                wl[p][3] = ((bx >> 4) & 0x0f0f0f0fu) | ((hx >> 2) & 0x30303030u);
                wh[p][3] = ((by >> 4) & 0x0f0f0f0fu) | ((hy >> 2) & 0x30303030u);
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int sb0 = 8 * f + 2 * k;   // sub-blocks sb0 (p = 0) and sb0 + 1 (p = 1) lie side by side in the tile
                int s0 = (int)(int8_t)((uint32_t)scv[sb0 >> 2] >> (8 * (sb0 & 3)));
                int s1 = (int)(int8_t)((uint32_t)scv[(sb0 + 1) >> 2] >> (8 * ((sb0 + 1) & 3)));
                // The scales are made opaque registers on purpose: left to itself the compiler reads the byte
                // straight out of the packed word with a sub-dword operand select, which only exists for the
                // two-operand multiply, and then needs separate additions (1.5 instructions per product
                // instead of one multiply-add).
                asm volatile("" : "+v"(s0), "+v"(s1));
#pragma unroll
                for (int j = 0; j < JT; ++j) {
                    const v4i av = *reinterpret_cast<const v4i *>(ap + j * 32 * LA + 8 * sb0);
                    const v16i i0 = __builtin_amdgcn_mfma_i32_32x32x16_i8(as_i64((uint32_t)av[0], (uint32_t)av[1]),
                                                                          as_i64(wl[0][k], wh[0][k]), zi, 0, 0, 0);
                    const v16i i1 = __builtin_amdgcn_mfma_i32_32x32x16_i8(as_i64((uint32_t)av[2], (uint32_t)av[3]),
                                                                          as_i64(wl[1][k], wh[1][k]), zi, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        int t = __mul24(i0[v], s0) + isum[j][v];
                        asm("" : "+v"(t));   // keeps the multiply-adds apart (see above: otherwise mul, mul, add3)
                        t = __mul24(i1[v], s1) + t;
                        asm("" : "+v"(t));
                        isum[j][v] = t;
                    }
                }
            }
        }
        const float dn = h2f(dbits);
        const float *dxs = sm.dx[buf];
#pragma unroll
        for (int j = 0; j < JT; ++j) {
            float dxv[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 d4 = *reinterpret_cast<const float4 *>(dxs + j * 32 + 8 * i + 4 * lh);
                dxv[4 * i] = d4.x; dxv[4 * i + 1] = d4.y; dxv[4 * i + 2] = d4.z; dxv[4 * i + 3] = d4.w;
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][v] = fmaf((float)isum[j][v], dxv[v] * dn, acc[j][v]);
        }
    };

    // a grid with gridDim.y > 1 cuts K: this workgroup does the super-blocks [sb_begin, sb_end) and writes a
    // partial tile; the partial tiles are added in order afterwards
    const int64_t sb_begin = nb * blockIdx.y / gridDim.y, sb_end = nb * (blockIdx.y + 1) / gridDim.y;
    load_next(sb_begin);
    store_next((int)(sb_begin & 1));
    __syncthreads();
    for (int64_t sb = sb_begin; sb < sb_end; ++sb) {
        const int buf = (int)(sb & 1);
        const uint32_t dbits = dcur;
        // past the end the last super-block is fetched again: unconditional loads keep the wait counters exact
        load_next(sb + 1 < sb_end ? sb + 1 : sb_end - 1);
        __builtin_amdgcn_sched_barrier(0);   // the loads stay ahead of the arithmetic they overlap with
        superblock(buf, dbits);
        __builtin_amdgcn_sched_barrier(0);   // the strips are read above and overwritten below
        store_next(buf ^ 1);
        __syncthreads();
    }

    // ---- store: accumulator register v of lane l is row 8*(v/4) + 4*(l/32) + v%4, column l%32
    const int64_t n = n0 + wave * 32 + l32;
    float *out = gridDim.y > 1 ? part + (size_t)blockIdx.y * M * N : y;
#pragma unroll
    for (int j = 0; j < JT; ++j) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int64_t m = m0 + j * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
            if (m < M && n < N) out[m * N + n] = acc[j][v];
        }
    }
}

}  // namespace

namespace {
template <int NW, int JT>
hipError_t launch_q6k(const WeightView &w, const ActView &a, int64_t M, float *y, float *scratch, int n_split, hipStream_t s) {
    if (dry_run()) return hipSuccess;
    using Smem = Q6Smem<NW, JT>;
    const auto kern = &gemm_q6k_q8k_kernel<NW, JT>;
    static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(Smem));
    if (attr != hipSuccess) return attr;
    const dim3 grid((unsigned)(((w.N + 32 * NW - 1) / (32 * NW)) * ((M + 32 * JT - 1) / (32 * JT))), (unsigned)n_split);
    hipLaunchKernelGGL(kern, grid, dim3(64 * NW), sizeof(Smem), s, w, a, M, y, scratch);
    if (n_split > 1) return launch_sum_parts(scratch, n_split, (size_t)M * w.N, y, s);
    return hipGetLastError();
}
}  // namespace

// ggml-format activations (Q8_K planes in `a`), Q6_K weights, any M
hipError_t launch_gemm_q6k_q8k(const WeightView &w, const ActView &a, int64_t M, float *y, const Scratch &scratch, hipStream_t s) {
    if (w.type != kTypeQ6_K || a.kind != kActKindQ8_K || !a.bsums || M <= 0) return hipErrorInvalidValue;
    if (w.K > (1 << 24)) return hipErrorInvalidValue;   // 32-bit lane offsets: 64 token rows of K bytes, 32 weight rows of K/2
    // 64 tokens x 128 weight rows per workgroup, two workgroups per compute unit.  A grid of such tiles that
    // would leave compute units idle is filled by cutting K into stretches (partial tiles added afterwards);
    // where K is too short for that, 32-token tiles double the number of workgroups instead.
    const int n_split = scratch.p ? q8k_tile_splits(w.K, M, w.N) : 1;
    if (n_split > 1 && (size_t)n_split * M * w.N * 4 > scratch.bytes) return hipErrorInvalidValue;   // partial tiles would not fit
    if (n_split > 1 || ((w.N + 127) / 128) * ((M + 63) / 64) >= 384) return launch_q6k<4, 2>(w, a, M, y, scratch.p, n_split, s);
    return launch_q6k<4, 1>(w, a, M, y, nullptr, 1, s);
}

}  // namespace qproj
