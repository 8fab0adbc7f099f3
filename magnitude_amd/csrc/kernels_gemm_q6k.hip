// Prefill-sized batches for Q6_K weights x ggml Q8_K activations on the int8 matrix cores.
//
//   y[m][n] = sum_sb d_n * dx_m * sum_{s<16} sc_{n,s} * sum_{k in s} (q_k - 32) * a_k
//
// A Q6_K sub-block is 16 weights with a signed 8-bit scale.  The scale does not split into parts that stay
// int8 after the multiply, but the PRODUCT does: w = sc * (q - 32) lies in [-4096, 4064], and
//     w = 256 * hi + lo,   lo = the low byte of w read as a signed byte, in [-128, 127],   hi = (w + 128) >> 8, in [-16, 16]
// are two int8 operands.  Each lane converts the 128 weights of its half super-block once into both operands
// (packed 16-bit multiply-add: w + 128 = sc * q + (128 - 32 * sc); the high bytes of that are hi, its low bytes
// with bit 7 flipped are lo) and both chains then stay inside the matrix cores for the whole super-block:
// eight v_mfma_i32_32x32x32_i8 per chain and 32 x 32 tile, (I_hi << 8) + I_lo is the exact integer sum that
// ggml's vec_dot forms, and the vector ALU touches the outputs once per 256 weights.  Because both chains run
// over the whole super-block the order of its 256 products is free: step t of lane (row l%32, half f = l/32) is
// sub-block 8f + t, sixteen consecutive weights, against the sixteen activations at the same place.  No block
// sums are needed: the -32 is inside the operand.
//
// Layout of the work: 32*JT tokens x 32*NW weight rows per workgroup, each wave 32 rows x all tokens of the tile
// (a converted operand feeds every token tile in turn).  Each wave fetches the ql / qh / scale planes of its 32
// rows with consecutive lanes on consecutive 16-byte pieces and parks them in wave-private LDS strips (row
// strides of 144 and 80 bytes: conflict-free for 16-byte reads by consecutive rows); LDS otherwise holds one
// super-block of activations, double-buffered: one workgroup barrier per 256 weights.
#include <type_traits>

#include "qproj_device.h"
#include "qproj_internal.h"
#include "gemm_tiles.h"
#include "lds_direct.h"

namespace qproj {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int LA = 256 + 16;   // activation row stride in LDS (bytes)
constexpr int SQL = 128 + 16;  // strip row strides
constexpr int SQH = 64 + 16;

template <int NW, int JT>   // NW waves of 32 weight rows each, JT token tiles of 32
struct Q6Smem {
    int8_t a[2][32 * JT * LA];   // activations of one super-block [token][256 (+16)]
    float dx[2][32 * JT];        // activation scale of the super-block
    uint8_t ql[NW][32 * SQL];
    uint8_t qh[NW][32 * SQH];
    int8_t sc[NW][32 * 16];
};

// two 16-bit lanes: x * s + c, each lane modulo 2^16
__device__ __forceinline__ uint32_t pk_mad_u16(uint32_t x, uint32_t s, uint32_t c) {
    uint32_t r;
    asm("v_pk_mad_u16 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(s), "v"(c));
    return r;
}

// The 16 + 16 weights that one 16-byte piece of ql (group gl of the half, bytes 16e .. 16e+15) holds in its low and
// high nibbles, with the matching piece of qh, into both int8 operands.  Step t of a lane is sub-block 8f + t of its
// half f = group g = t/2 (ql byte 32*(g%2) + l, nibble g/2, qh bits 2g and 2g+1), bytes l = 16*(t%2) .. +15; `scq`
// holds the eight scales of the half.
__device__ __forceinline__ void convert_pieces(const v4i &lq, const v4i &hq, const v2i &scq, int gl, int e, v4i (&cl)[8], v4i (&ch)[8]) {
#pragma unroll
    for (int nib = 0; nib < 2; ++nib) {
        const int g = gl + 2 * nib, t = 2 * g + e;
        const int s = (int)(int8_t)((uint32_t)scq[t >> 2] >> (8 * (t & 3)));
        const uint32_t s16 = __builtin_amdgcn_perm((uint32_t)s, (uint32_t)s, 0x01000100u);
        const int cc = 128 - 32 * s;
        const uint32_t c16 = __builtin_amdgcn_perm((uint32_t)cc, (uint32_t)cc, 0x01000100u);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t lw = (uint32_t)lq[c], hw = (uint32_t)hq[c];
            const uint32_t x = nib ? (lw >> 4) & 0x0f0f0f0fu : lw & 0x0f0f0f0fu;
            const uint32_t hs = g == 0 ? hw << 4 : g == 1 ? hw << 2 : g == 2 ? hw : hw >> 2;
            const uint32_t q = (hs & 0x30303030u) | x;                          // four codes 0..63
            // codes 0, 2 and 1, 3 in 16-bit lanes: byte permutes over zeros (a mask for the first pair made the compiler
            // build the four codes twice, once for each pair)
            const uint32_t e0 = __builtin_amdgcn_perm(0u, q, 0x0c020c00u), e1 = __builtin_amdgcn_perm(0u, q, 0x0c030c01u);
            const uint32_t w0 = pk_mad_u16(e0, s16, c16), w1 = pk_mad_u16(e1, s16, c16);   // sc * (q - 32) + 128
            // low bytes (bit 7 flipped: minus 128 modulo 256) and high bytes, back in the order of the codes
            cl[t][c] = (int)(__builtin_amdgcn_perm(w1, w0, 0x06020400u) ^ 0x80808080u);
            ch[t][c] = (int)__builtin_amdgcn_perm(w1, w0, 0x07030501u);
        }
    }
}

template <int NW, int JT>
__global__ __launch_bounds__(64 * NW, 2) void gemm_q6k_q8k_kernel(const WeightView w, const ActView a, int64_t M,
                                                                              float *__restrict__ y, float *__restrict__ part) {
    constexpr int NT = 64 * NW, TN = 32 * NW, TM = 32 * JT;
    constexpr int PA = TM * 16 / NT;   // 16-byte activation pieces a thread moves per super-block
    static_assert(PA >= 1 && TM <= NT, "tile does not fit the staging scheme");
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
    // activations: piece id = tid + NT*p -> token id / 16, 16-byte segment id % 16
    const int mrow_cap = (int)(M - 1 - m0 < TM - 1 ? M - 1 - m0 : TM - 1);
    const int8_t *abase = a.qs + m0 * K;
    uint32_t aoffg[PA];
    int aoffl[PA];
#pragma unroll
    for (int p = 0; p < PA; ++p) {
        const int id = tid + NT * p, row = id >> 4, seg = id & 15;
        aoffg[p] = (uint32_t)((row < mrow_cap ? row : mrow_cap) * (int)K + 16 * seg);
        aoffl[p] = row * LA + 16 * seg;
    }
    const float *dxbase = a.d + m0 * nb;
    const uint32_t dxoffg = (uint32_t)(((tid & (TM - 1)) < mrow_cap ? (tid & (TM - 1)) : mrow_cap) * (int)nb);

    v4i sql[4], sqh[2], ssc, areg[PA];
    float dxreg;
    uint32_t dcur = 0, dnext = 0;   // fp16 d of the lane's row: current super-block, next
    auto load_next = [&](int64_t sb) {   // activations first: they are wanted at the end of this trip already
#pragma unroll
        for (int p = 0; p < PA; ++p) areg[p] = *reinterpret_cast<const v4i *>(abase + sb * 256 + aoffg[p]);
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
        for (int p = 0; p < PA; ++p) *reinterpret_cast<v4i *>(sm.a[buf] + aoffl[p]) = areg[p];
        // threads beyond the first TM repeat a store of the same value: no branch, no load sunk into one
        sm.dx[buf][tid & (TM - 1)] = dxreg;
#pragma unroll
        for (int c = 0; c < 4; ++c) *reinterpret_cast<v4i *>(pql + qlpark[c]) = sql[c];
#pragma unroll
        for (int c = 0; c < 2; ++c) *reinterpret_cast<v4i *>(pqh + qhpark[c]) = sqh[c];
        *reinterpret_cast<v4i *>(psc + l32 * 16) = ssc;
        dcur = dnext;
    };

    const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    auto superblock = [&](int buf, uint32_t dbits) {
        const v2i scq = *reinterpret_cast<const v2i *>(psc + l32 * 16 + 8 * lh);   // the eight scales of the half
        v4i cl[8], ch[8];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const v4i hq = *reinterpret_cast<const v4i *>(pqh + l32 * SQH + 32 * lh + 16 * e);
#pragma unroll
            for (int gl = 0; gl < 2; ++gl) {
                const v4i lq = *reinterpret_cast<const v4i *>(pql + l32 * SQL + 64 * lh + 32 * gl + 16 * e);
                convert_pieces(lq, hq, scq, gl, e, cl, ch);
            }
        }
        const float dn = h2f(dbits);
        const int8_t *ap = sm.a[buf] + l32 * LA + 128 * lh;
        const float *dxs = sm.dx[buf];
#pragma unroll
        for (int j = 0; j < JT; ++j) {
            v16i ilo = zi, ihi = zi;
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const v4i af = *reinterpret_cast<const v4i *>(ap + j * 32 * LA + 16 * t);
                ilo = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, cl[t], ilo, 0, 0, 0);
                ihi = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, ch[t], ihi, 0, 0, 0);
            }
            float dxv[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 d4 = *reinterpret_cast<const float4 *>(dxs + j * 32 + 8 * i + 4 * lh);
                dxv[4 * i] = d4.x; dxv[4 * i + 1] = d4.y; dxv[4 * i + 2] = d4.z; dxv[4 * i + 3] = d4.w;
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][v] = fmaf((float)((ihi[v] << 8) + ilo[v]), dxv[v] * dn, acc[j][v]);
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


// ------------------------------------------------------------------------------------------------
// The same product for large grids: 128 tokens x 256 weight rows per workgroup (eight waves, one workgroup per
// compute unit), so a wave converts its weights once per 128 tokens.  Nothing is staged through registers:
// activations, activation scales and the raw planes of the wave's 32 rows go from global memory straight into LDS
// (16 bytes a lane, a wave writes a contiguous kilobyte per request).  Such a load cannot pad LDS rows, so the
// 16-byte segments of a row are XOR-swizzled by the row index instead -- the loading lane simply asks global memory
// for the segment that belongs in its slot: activations [token][16 slots], slot s holds segment s ^ (token % 16);
// ql [row][8 slots], slot s holds piece s ^ (row % 8); qh [row][4 slots], slot s holds piece s ^ ((row / 2) % 4);
// the 16 scales of a row lie as they are.
struct Q6WideSmem {
    int8_t a[2][128 * 256];
    float dx[2][128];
    uint8_t ql[8][32 * 128];
    uint8_t qh[8][32 * 64];
    int8_t sc[8][64 * 16];   // 32 rows; the upper half takes the duplicate pieces of lanes 32..63
};

__global__ __launch_bounds__(512, 1) void gemm_q6k_q8k_wide_kernel(const WeightView w, const ActView a, int64_t M,
                                                                 float *__restrict__ y, float *__restrict__ part) {
    constexpr int NW = 8, TM = 128, TN = 256, JT = 4, PA = 4;
    extern __shared__ __align__(16) uint8_t smem_raw[];
    Q6WideSmem &sm = *reinterpret_cast<Q6WideSmem *>(smem_raw);
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

    // ---- global -> LDS requests: wave-uniform bases plus 32-bit lane offsets; rows past the edge of the matrix
    // repeat its last valid row (computed, never stored)
    const int64_t wave_row0 = n0 + wave * 32 < N ? n0 + wave * 32 : N - 1;
    const int wrow_cap = (int)(N - 1 - wave_row0 < 31 ? N - 1 - wave_row0 : 31);
    const uint8_t *qlbase = scalar_pointer(w.q6_ql + wave_row0 * nb * 128);
    const uint8_t *qhbase = scalar_pointer(w.q6_qh + wave_row0 * nb * 64);
    const uint8_t *scbase = scalar_pointer(reinterpret_cast<const uint8_t *>(w.q6_sc) + wave_row0 * nb * 16);
    const global_ptr<uint16_t> dbase = scalar_global(w.q6_d + wave_row0 * nb);
    uint32_t qloff[4], qhoff[2];
#pragma unroll
    for (int c = 0; c < 4; ++c) {   // slot p = lane + 64*c of the wave's 256: row p / 8, slot p % 8
        const int p = lane + 64 * c, row = p >> 3, r = row < wrow_cap ? row : wrow_cap;
        qloff[c] = (uint32_t)(r * (int)nb * 128 + 16 * ((p & 7) ^ (row & 7)));
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {   // slot p of 128: row p / 4, slot p % 4
        const int p = lane + 64 * c, row = p >> 2, r = row < wrow_cap ? row : wrow_cap;
        qhoff[c] = (uint32_t)(r * (int)nb * 64 + 16 * ((p & 3) ^ ((row >> 1) & 3)));
    }
    const int myrow = l32 < wrow_cap ? l32 : wrow_cap;
    const uint32_t scoff = (uint32_t)(myrow * (int)nb * 16);
    const uint32_t doff = (uint32_t)(myrow * (int)nb);
    const int mrow_cap = (int)(M - 1 - m0 < TM - 1 ? M - 1 - m0 : TM - 1);
    const int8_t *abase = scalar_pointer(a.qs + m0 * K);
    uint32_t aoffg[PA];   // chunk wave + NW*p = tokens 4*chunk .. +3; lane -> token lane/16, slot lane%16
#pragma unroll
    for (int p = 0; p < PA; ++p) {
        const int row = 4 * (wave + NW * p) + (lane >> 4), seg = (lane & 15) ^ (row & 15);
        aoffg[p] = (uint32_t)((row < mrow_cap ? row : mrow_cap) * (int)K + 16 * seg);
    }
    const global_ptr<float> dxbase = scalar_global(a.d + m0 * nb);
    const int dxtok = tid & 127;
    const uint32_t dxoffg = (uint32_t)((dxtok < mrow_cap ? dxtok : mrow_cap) * (int)nb);
    uint8_t *pql = sm.ql[wave], *pqh = sm.qh[wave];
    int8_t *psc = sm.sc[wave];

    auto request_strip = [&](uint32_t sb) {
#pragma unroll
        for (int c = 0; c < 4; ++c) global_to_lds16(qlbase + (qloff[c] + sb * 128u), pql + 1024 * c);
#pragma unroll
        for (int c = 0; c < 2; ++c) global_to_lds16(qhbase + (qhoff[c] + sb * 64u), pqh + 1024 * c);
        global_to_lds16(scbase + (scoff + sb * 16u), psc);
    };
    auto request_act = [&](uint32_t sb, int buf, int p) {
        global_to_lds16(abase + (aoffg[p] + sb * 256u), sm.a[buf] + (wave + NW * p) * 1024);
    };
    // the lane's reads: ql piece q8 = 4f + 2gl + e of row l%32 sits in slot q8 ^ (l%8); qh piece 2f + e in slot
    // (2f + e) ^ ((l%32 / 2) % 4); activation segment 8f + t of token l%32 (+32j) in slot (8f + t) ^ (l%16)
    const int qlrow = l32 * 128, qhrow = l32 * 64;
    const int qlx = l32 & 7, qhx = (l32 >> 1) & 3;
    const int aoffl = l32 * 256 + 16 * ((8 * lh) ^ (l32 & 15));
    const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    // a grid with gridDim.y > 1 cuts K: this workgroup does the super-blocks [sb_begin, sb_end) and writes a
    // partial tile; the partial tiles are added in order afterwards
    const int64_t sb_begin = nb * blockIdx.y / gridDim.y, sb_end = nb * (blockIdx.y + 1) / gridDim.y;
    // ---- prologue: requests of the first super-block
    request_strip((uint32_t)sb_begin);
#pragma unroll
    for (int p = 0; p < PA; ++p) request_act((uint32_t)sb_begin, 0, p);
    sm.dx[0][dxtok] = dxbase[dxoffg + (uint32_t)sb_begin];
    uint32_t dcur = dbase[doff + (uint32_t)sb_begin];
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // The two waves that share a SIMD (w and w + 4) run a super-block in opposite orders, as in the Q4_K kernel of
    // this shape: EARLY waves (0..3) convert the weights of a super-block at its start, LATE waves (4..7) convert
    // the weights of the NEXT super-block at the end of the current one, after their last tile - so one of the two
    // has matrix work while the other has vector work, instead of both wanting the same pipe at the same time.
    v4i cl[8], ch[8];
    auto convert_strip = [&]() {   // the lane's 128 weights into both int8 operands, out of the strip
        const v2i scq = *reinterpret_cast<const v2i *>(psc + l32 * 16 + 8 * lh);
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const v4i hq = *reinterpret_cast<const v4i *>(pqh + qhrow + 16 * ((2 * lh + e) ^ qhx));
#pragma unroll
            for (int gl = 0; gl < 2; ++gl) {
                const v4i lq = *reinterpret_cast<const v4i *>(pql + qlrow + 16 * ((4 * lh + 2 * gl + e) ^ qlx));
                convert_pieces(lq, hq, scq, gl, e, cl, ch);
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the strip has been read: it may be overwritten
    };
    auto run = [&](auto late_tag) {
        constexpr bool LATE = decltype(late_tag)::value;
        if (LATE) convert_strip();   // weights of the first super-block, with nothing to overlap
        for (int64_t sb = sb_begin; sb < sb_end; ++sb) {
            const int buf = (int)((sb - sb_begin) & 1);
            const uint32_t sb_next = (uint32_t)(sb + 1 < sb_end ? sb + 1 : sb_end - 1);   // past the end: requested again, never used
            if (!LATE) convert_strip();
            const float dn = h2f(dcur);
            const uint32_t dnext = dbase[doff + sb_next];
            const float dxreg = dxbase[dxoffg + sb_next];
            __builtin_amdgcn_sched_barrier(0);
            request_strip(sb_next);   // its previous content was read above (early waves) or at the end of the last trip (late waves)
            __builtin_amdgcn_sched_barrier(0);
            const int8_t *ab = sm.a[buf];
            const float *dxs = sm.dx[buf];
            // the tiles as a two-stage pipeline: while tile j is multiplied (two chains of eight matrix instructions into one
            // of two accumulator pairs), the finished sums of tile j - 1 are flushed from the other pair - independent work
            // the scheduler can put between the matrix instructions
            v16i ilo[2], ihi[2];
#pragma unroll
            for (int j = 0; j <= JT; ++j) {
                if (j < JT) {
                    ilo[j & 1] = zi;
                    ihi[j & 1] = zi;
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        const v4i af = *reinterpret_cast<const v4i *>(ab + j * 32 * 256 + (aoffl ^ (16 * t)));
                        ilo[j & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, cl[t], ilo[j & 1], 0, 0, 0);
                        ihi[j & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, ch[t], ihi[j & 1], 0, 0, 0);
                    }
                }
                if (j == 1) {   // the next super-block's activations, once the strip requests are under way
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int p = 0; p < PA; ++p) request_act(sb_next, buf ^ 1, p);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (j > 0) {
                    const int jf = j - 1;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float4 d4 = *reinterpret_cast<const float4 *>(dxs + jf * 32 + 8 * i + 4 * lh);
                        const float dxv[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int v = 4 * i + r;
                            acc[jf][v] = fmaf((float)((ihi[jf & 1][v] << 8) + ilo[jf & 1][v]), dxv[r] * dn, acc[jf][v]);
                        }
                    }
                }
                if (j > 0 && j < JT) {   // one matrix instruction, its share of the operand reads, four of the flush instructions
#pragma unroll
                    for (int g = 0; g < 16; ++g) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
                    }
                }
            }
            if (LATE) {
                // the next super-block's strip was requested at the top of this trip; of the requests made since then
                // (PA activation chunks) none needs to have landed
                static_assert(PA == 4, "the wait below counts the activation requests");
                __builtin_amdgcn_sched_barrier(0);
                asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
                convert_strip();
            }
            sm.dx[buf ^ 1][dxtok] = dxreg;   // every thread stores (a repeated value past 128): no branch
            dcur = dnext;
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __syncthreads();
        }
    };
    if (wave < 4) run(std::false_type{});
    else run(std::true_type{});

    // ---- store: accumulator register v of lane l is row 8*(v/4) + 4*(l/32) + v%4, column l%32 (the lane's coordinates
    // are worked out again from the thread index, made opaque, so that no address arithmetic is carried through the loop)
    int tid_s = tid, pid_s = (int)blockIdx.x;
    asm volatile("" : "+v"(tid_s));
    asm volatile("" : "+s"(pid_s));
    int tile_n_s, tile_m_s;
    tile_of_workgroup((int)((N + TN - 1) / TN), (int)((M + TM - 1) / TM), pid_s, tile_n_s, tile_m_s);
    const int64_t n0_s = (int64_t)tile_n_s * TN, m0_s = (int64_t)tile_m_s * TM;
    const int l32_s = tid_s & 31, lh_s = (tid_s >> 5) & 1, wave_s = tid_s >> 6;
    const int64_t n = n0_s + wave_s * 32 + l32_s;
    float *out = gridDim.y > 1 ? part + (size_t)blockIdx.y * M * N : y;
#pragma unroll
    for (int j = 0; j < JT; ++j) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int64_t m = m0_s + j * 32 + 8 * (v >> 2) + 4 * lh_s + (v & 3);
            if (m < M && n < N) out[m * N + n] = acc[j][v];
        }
    }
}
}  // namespace

namespace {
template <int NW, int JT>
hipError_t launch_q6k(const WeightView &w, const ActView &a, int64_t M, float *y, float *scratch, int n_split, hipStream_t s) {
    if (dry_run()) {
        if (n_split > 1) plan_note_cut();
        plan_note("gemm_q6k_q8k_kernel<%d waves, %d token tiles>: tile %d tokens x %d rows, %lld tiles x %d K stretches%s", NW, JT, 32 * JT, 32 * NW,
                  (long long)(((w.N + 32 * NW - 1) / (32 * NW)) * ((M + 32 * JT - 1) / (32 * JT))), n_split, n_split > 1 ? " + sum_parts_kernel" : "");
        return hipSuccess;
    }
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

// Which kernel and how many stretches of K.  The 128-token kernel (256 weight rows a workgroup, one workgroup per
// compute unit) wants about 192 workgroups or more: a grid of 48..191 such tiles is multiplied by cutting K into the
// stretches wide_tile_splits picks (64 tiles of K = 14336: four; 80 tiles of K = 13824: three, 240 workgroups in one
// round, where four made 320).  Smaller grids take 64-token tiles (128 rows, two
// workgroups per compute unit) with the stretches of q8k_tile_splits, or 32-token tiles where K is too short for that.
namespace {
struct Q6Plan {
    bool wide;
    int n_split;
};
// Stretches of K for the 64-token tiles (128 rows, two workgroups a compute unit = 512 places).  This kernel's
// workgroups are slow next to the pass that adds the partial tiles, so under 192 tiles it takes as many stretches as
// fill the places once, eight at most, four super-blocks a stretch at least.  14336 -> 4096, per call, us, stretches of
// the common rule -> these: 128 tokens (64 tiles) 4 -> 8: 49.0 -> 46.7; 160 / 192 tokens (96 tiles) 3 -> 5: 79.7 / 79.4 ->
// 60.4 / 59.4; 256 tokens (128 tiles) 3 -> 4: 81.4 -> 72.4.
int q6k_tile_splits(int64_t K, int64_t M, int64_t N) {
    static const int forced = tuning_int("QPROJ_Q8K_SPLITS", 0);
    const int64_t tiles = ((N + 127) / 128) * ((M + 63) / 64);
    if (forced > 0 || tiles >= 192 || (M * N) % 4 != 0) return q8k_tile_splits(K, M, N, false);
    int n = (int)std::min<int64_t>(8, std::max<int64_t>(1, 512 / tiles));
    while (n > 1 && K / 256 < 4 * n) --n;
    return n;
}

Q6Plan q6k_plan(int64_t K, int64_t M, int64_t N, bool have_scratch) {
    const int64_t wide_tiles = ((N + 255) / 256) * ((M + 127) / 128);
    // (from 160 tiles: 4096 -> 14336 at 320 / 384 tokens, 168 tiles, 98.5 / 98.0 -> 87.2 / 85.3 us; from 112 on it loses,
    // 8192 x 8192 at 448 tokens 101 -> 147)
    static const int wide_min = tuning_int("QPROJ_Q6K_WIDE_MIN_TILES", 160);
    if (wide_tiles >= wide_min) return {true, 1};
    if (have_scratch && (M * N) % 4 == 0 && wide_tiles >= 48) {
        const int n = wide_tile_splits(wide_tiles, K / 256, M, N, cu_count(), 5.0);
        if (n > 1) return {true, n};
    }
    return {false, have_scratch ? q6k_tile_splits(K, M, N) : 1};
}
}  // namespace

size_t q6k_tile_scratch_bytes(int64_t K, int64_t M, int64_t N) {
    const Q6Plan p = q6k_plan(K, M, N, true);
    return p.n_split > 1 ? (size_t)p.n_split * M * N * 4 : 0;
}

// ggml-format activations (Q8_K planes in `a`), Q6_K weights, any M
hipError_t launch_gemm_q6k_q8k(const WeightView &w, const ActView &a, int64_t M, float *y, const Scratch &scratch, hipStream_t s) {
    if (w.type != kTypeQ6_K || a.kind != kActKindQ8_K || M <= 0) return hipErrorInvalidValue;
    if (w.K > (1 << 24)) return hipErrorInvalidValue;   // 32-bit lane offsets: 128 token rows of K bytes, 32 weight rows of K/2
    const Q6Plan p = q6k_plan(w.K, M, w.N, scratch.p != nullptr);
    if (p.n_split > 1 && (size_t)p.n_split * M * w.N * 4 > scratch.bytes) return hipErrorInvalidValue;   // partial tiles would not fit
    if (p.wide) {
        if (dry_run()) {
            if (p.n_split > 1) plan_note_cut();
            plan_note("gemm_q6k_q8k_wide_kernel: tile 128 tokens x 256 rows, %lld tiles x %d K stretches%s, partial tiles %zu B",
                      (long long)(((w.N + 255) / 256) * ((M + 127) / 128)), p.n_split, p.n_split > 1 ? " + sum_parts_kernel" : "",
                      p.n_split > 1 ? (size_t)p.n_split * M * w.N * 4 : (size_t)0);
            return hipSuccess;
        }
        static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q6k_q8k_wide_kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(Q6WideSmem));
        if (attr != hipSuccess) return attr;
        const int64_t wide_tiles = ((w.N + 255) / 256) * ((M + 127) / 128);
        hipLaunchKernelGGL(gemm_q6k_q8k_wide_kernel, dim3((unsigned)wide_tiles, (unsigned)p.n_split), dim3(512), sizeof(Q6WideSmem),
                           s, w, a, M, y, scratch.p);
        if (p.n_split > 1) return launch_sum_parts(scratch.p, p.n_split, (size_t)M * w.N, y, s);
        return hipGetLastError();
    }
    // 64-token tiles from 192 tiles on (32-token tiles below, twice the workgroups): 4096 -> 14336 at 160 / 192 tokens,
    // 336 tiles, 74.2 / 76.8 -> 66.1 / 64.3 us; 4096 x 4096 at 384 tokens 49.4 -> 42.9 (the threshold was 384)
    static const int tile64_min = tuning_int("QPROJ_Q6K_TILE64_MIN", 192);
    if (p.n_split > 1 || ((w.N + 127) / 128) * ((M + 63) / 64) >= tile64_min) return launch_q6k<4, 2>(w, a, M, y, scratch.p, p.n_split, s);
    return launch_q6k<4, 1>(w, a, M, y, nullptr, 1, s);
}

}  // namespace qproj
