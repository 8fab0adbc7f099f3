// Small-batch projection (2..16 activation rows, the speculative-verify regime) on the int8 matrix
// cores: the weights are streamed from HBM once and every row of activations is applied to them.
//
// One v_mfma_i32_32x32x32_i8 (Q4_K, Q8_0) or v_mfma_i32_32x32x16_i8 (Q6_K) multiplies the int8
// activations of up to 32 tokens (A operand) with one sub-block of 32 weight rows (B operand), so
// that lane l ends up with the integer dots of weight row l%32 against 8 (or 16) tokens.  A
// sub-block's integer scale is applied with one v_mad_i32_i24 per output, the super-block's fp32
// scales once per 256 weights.  The terms that ggml takes from the activation block sums (the
// Q4_K mins, the -32 offset of Q6_K) are two more products each: block sums split into a signed
// high and a 6-bit low byte against the 6-bit mins / 8-bit scales.
//
// Data movement.  The B operand wants lane l to hold bytes of weight row l%32, i.e. 32 rows that
// lie K/256 blocks apart in memory; loading it that way touches every cache line from five
// instructions and thrashes the vector L1.  Instead a wave copies the 32 rows' current
// super-block with fully coalesced 16-byte loads (consecutive lanes = consecutive 16-byte pieces
// of a row's block), two super-blocks ahead of the arithmetic, parks the registers in a
// wave-private LDS region and reads the region back in operand order.  The quantized
// activations of the workgroup's K range are staged in LDS once.
//
// Work split.  A workgroup is 4 waves = rw row groups (32 rows each) x kw K-parts; the K-parts
// of a row group are summed through LDS in a fixed order.  When one workgroup cannot hold the
// whole K range (LDS) or there would be too few workgroups, K is also cut into chunks whose
// results go to a scratch buffer that a second small kernel sums in chunk order, so results do
// not depend on scheduling.  Exactly two chunks, with output rows that the quantizer launch in
// front has cleared, add their results to the output themselves (float add at the memory side,
// nothing returned): two addends on zero give the same sum in either order, so this does not
// depend on scheduling either, and the summing launch goes.  (The memory-side adder may flush a
// sum below the smallest normal float to zero.)
#include <stdlib.h>

#include <algorithm>

#include "qproj_device.h"
#include "qproj_internal.h"
#include "actquant_device.h"

namespace qproj {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));


struct MfmaTarget {
    WeightView w;
    float *y;
    float *part;       // [n_chunks][M][N] when n_chunks > 1
    int first_wg;
    int n_rowsets;
};

struct MfmaArgs {
    int n_targets;
    MfmaTarget t[kMaxTargets];
    ActView a;
    const float *x;        // non-null: fp32 activation rows [rows][K], quantized by every workgroup in its prologue
    int M, n_chunks, chunk_sb, kw, rw, n_wgs;
    int rpg;               // weight rows a row group (32 fill the matrix instruction; dense launches may take fewer, below)
    int add_out;           // dense mode, two chunks, output rows cleared before the launch: both chunks add to y
    int64_t part_plane;    // expert-grouped mode with K in chunks: floats of one chunk's results, [n_pairs][N], in t[0].part
    // expert-grouped mode (MUL_MAT_ID): activation rows of expert e are the pairs order[offsets[e]..offsets[e+1])
    const int32_t *order;
    const int32_t *offsets;
    const int32_t *active;  // experts that have pairs; active[n_expert] = how many
    int n_expert;
    int x_div;             // activation row of pair p is p / x_div
    int wgs_per_expert;
    int rg_loop;           // row groups a wave works through one after the other (the staged rows are reused)
    // pair mode (ids non-null): workgroup set s serves pair s alone with expert ids[s]; no order / offsets / active
    const int32_t *ids;
    int n_pairs;
    int32_t *error_flag;
};

template <int QT>
struct Cfg;
template <>
struct Cfg<kTypeQ4_K> {
    static constexpr int kAux = 16;      // per (token, super-block): 8 high + 8 low bytes of the 32-wide block sums
    static constexpr int kDx = 1;        // activation scales per super-block
    static constexpr int kRegion = 32 * 144;
};
template <>
struct Cfg<kTypeQ6_K> {
    static constexpr int kAux = 32;      // 16 high + 16 low bytes of the 16-wide block sums
    static constexpr int kDx = 1;
    static constexpr int kQl = 0, kQh = 32 * 144, kSc = kQh + 32 * 80, kD = kSc + 32 * 16;
    static constexpr int kRegion = kD + 32 * 4;
};
template <>
struct Cfg<kTypeQ8_0> {
    static constexpr int kAux = 0;
    static constexpr int kDx = 8;        // Q8_0 activations carry a scale per 32
    static constexpr int kD = 32 * 272;
    static constexpr int kRegion = kD + 32 * 16;
};

struct Layout {
    int lda, off_dx, off_aux, off_map, off_w, total;
};
template <int QT, int MT, int W>
__host__ __device__ inline Layout layout(int chunk_sb) {
    Layout l;
    l.lda = chunk_sb * 256 + 16;
    l.off_dx = MT * l.lda;
    l.off_aux = l.off_dx + chunk_sb * Cfg<QT>::kDx * MT * 4;
    l.off_map = l.off_aux + chunk_sb * MT * Cfg<QT>::kAux;   // MT ints: which pair each staged row is
    l.off_w = l.off_map + MT * 4;
    l.total = l.off_w + W * Cfg<QT>::kRegion;   // a region doubles as the wave's partial tile at the end
    return l;
}

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ v4i as_v4i(const uint4 &u) { return v4i{(int)u.x, (int)u.y, (int)u.z, (int)u.w}; }
__device__ __forceinline__ long as_i64(uint32_t lo, uint32_t hi) { return (long)(((uint64_t)hi << 32) | lo); }
__device__ __forceinline__ int sbyte(uint32_t w, int i) { return (int)(int8_t)(w >> (8 * i)); }

// ------------------------------------------------------------------------------------------------
// Coalesced copy of one super-block of 32 consecutive rows: global -> registers -> wave's LDS region.
// `row0 + r` is clamped to N - 1 so that a ragged last row group reads valid memory.
template <int QT>
struct Stager;

template <>
struct Stager<kTypeQ4_K> {
    v4i r[5];                 // first member: no padding in front of the 16-byte registers
    const uint8_t *base[2];   // wave-uniform: block 0 of the first row, per tensor (gate / up)
    uint32_t off[5], lds[5];
    // 288 pieces of 16 bytes: piece p = lane + 64k is bytes 16j.. of row p / 9, j = p % 9
    // (lanes 32..63 repeat piece 287 in their fifth slot, so every load and store is unpredicated)
    __device__ __forceinline__ void rebase(int t, const WeightView &w, int64_t row) {
        base[t] = w.q4k + (size_t)row * (size_t)w.nb * 144;
    }
    __device__ __forceinline__ void init(const WeightView &w, int last, int lane) {
        const uint32_t row_bytes = (uint32_t)w.nb * 144u;
#pragma unroll
        for (int k = 0; k < 5; ++k) {
            int p = lane + 64 * k;
            if (p > 287) p = 287;
            const int r = p / 9, j = p - 9 * r;
            off[k] = (uint32_t)min(r, last) * row_bytes + 16u * j;
            lds[k] = (uint32_t)p * 16u;
        }
    }
    __device__ __forceinline__ void issue(int t, int sb) {
        const uint8_t *b = (t ? base[1] : base[0]) + (size_t)sb * 144;
#pragma unroll
        for (int k = 0; k < 5; ++k) r[k] = *reinterpret_cast<const v4i *>(b + off[k]);
    }
    __device__ __forceinline__ void park(uint8_t *region, int) const {
#pragma unroll
        for (int k = 0; k < 5; ++k) *reinterpret_cast<v4i *>(region + lds[k]) = r[k];
    }
};

template <>
struct Stager<kTypeQ6_K> {
    // ql: 8 pieces a row (4 per lane), qh: 4 pieces a row (2 per lane), scales: 1 piece a row, d: 2 bytes a row
    v4i l[4], h[2], s;        // first members: no padding in front of the 16-byte registers
    const uint8_t *bl[2], *bh[2], *bs[2], *bd[2];
    uint32_t off_l[4], off_h[2], off_s, off_d, lds_l[4], lds_h[2];
    uint32_t d;
    __device__ __forceinline__ void rebase(int t, const WeightView &w, int64_t row) {
        const size_t rb = (size_t)row * (size_t)w.nb;
        bl[t] = w.q6_ql + rb * 128;
        bh[t] = w.q6_qh + rb * 64;
        bs[t] = reinterpret_cast<const uint8_t *>(w.q6_sc) + rb * 16;
        bd[t] = reinterpret_cast<const uint8_t *>(w.q6_d) + rb * 2;
    }
    __device__ __forceinline__ void init(const WeightView &w, int last, int lane) {
        const uint32_t nb = (uint32_t)w.nb;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int p = lane + 64 * k, r = p >> 3, j = p & 7;
            off_l[k] = (uint32_t)min(r, last) * nb * 128u + 16u * j;
            lds_l[k] = Cfg<kTypeQ6_K>::kQl + r * 144 + 16 * j;
        }
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const int p = lane + 64 * k, r = p >> 2, j = p & 3;
            off_h[k] = (uint32_t)min(r, last) * nb * 64u + 16u * j;
            lds_h[k] = Cfg<kTypeQ6_K>::kQh + r * 80 + 16 * j;
        }
        const uint32_t r = (uint32_t)min(lane & 31, last);
        off_s = r * nb * 16u;
        off_d = r * nb * 2u;
    }
    __device__ __forceinline__ void issue(int t, int sb) {
        const uint8_t *pl = (t ? bl[1] : bl[0]) + (size_t)sb * 128, *ph = (t ? bh[1] : bh[0]) + (size_t)sb * 64;
        const uint8_t *ps = (t ? bs[1] : bs[0]) + (size_t)sb * 16, *pd = (t ? bd[1] : bd[0]) + (size_t)sb * 2;
#pragma unroll
        for (int k = 0; k < 4; ++k) l[k] = *reinterpret_cast<const v4i *>(pl + off_l[k]);
#pragma unroll
        for (int k = 0; k < 2; ++k) h[k] = *reinterpret_cast<const v4i *>(ph + off_h[k]);
        s = *reinterpret_cast<const v4i *>(ps + off_s);
        d = *reinterpret_cast<const uint16_t *>(pd + off_d);
    }
    __device__ __forceinline__ void park(uint8_t *region, int lane) const {
#pragma unroll
        for (int k = 0; k < 4; ++k) *reinterpret_cast<v4i *>(region + lds_l[k]) = l[k];
#pragma unroll
        for (int k = 0; k < 2; ++k) *reinterpret_cast<v4i *>(region + lds_h[k]) = h[k];
        // both lane halves hold the same row's scales and d: identical stores
        *reinterpret_cast<v4i *>(region + Cfg<kTypeQ6_K>::kSc + (lane & 31) * 16) = s;
        *reinterpret_cast<uint32_t *>(region + Cfg<kTypeQ6_K>::kD + (lane & 31) * 4) = d;
    }
};

template <>
struct Stager<kTypeQ8_0> {
    // one "super-block" = 256 weights = 8 blocks: 16 pieces of quants and one piece of 8 fp16 scales a row
    v4i q[8], d;              // first members: no padding in front of the 16-byte registers
    const uint8_t *bq[2], *bd[2];
    uint32_t off_q[8], off_d, lds_q[8];
    __device__ __forceinline__ void rebase(int t, const WeightView &w, int64_t row) {
        bq[t] = reinterpret_cast<const uint8_t *>(w.q8_qs) + (size_t)row * (size_t)w.K;
        bd[t] = reinterpret_cast<const uint8_t *>(w.q8_d) + (size_t)row * (size_t)(w.K / 32) * 2;
    }
    __device__ __forceinline__ void init(const WeightView &w, int last, int lane) {
        const uint32_t K = (uint32_t)w.K;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int p = lane + 64 * k, r = p >> 4, j = p & 15;
            off_q[k] = (uint32_t)min(r, last) * K + 16u * j;
            lds_q[k] = r * 272 + 16 * j;
        }
        off_d = (uint32_t)min(lane & 31, last) * (K / 32) * 2u;
    }
    __device__ __forceinline__ void issue(int t, int sb) {
        const uint8_t *pq = (t ? bq[1] : bq[0]) + (size_t)sb * 256, *pd = (t ? bd[1] : bd[0]) + (size_t)sb * 16;
#pragma unroll
        for (int k = 0; k < 8; ++k) q[k] = *reinterpret_cast<const v4i *>(pq + off_q[k]);
        d = *reinterpret_cast<const v4i *>(pd + off_d);
    }
    __device__ __forceinline__ void park(uint8_t *region, int lane) const {
#pragma unroll
        for (int k = 0; k < 8; ++k) *reinterpret_cast<v4i *>(region + lds_q[k]) = q[k];
        *reinterpret_cast<v4i *>(region + Cfg<kTypeQ8_0>::kD + (lane & 31) * 16) = d;
    }
};

// ------------------------------------------------------------------------------------------------
// One super-block of 32 rows against the staged activations: out[4*i + j] += contribution to token
// 8*i + 4*h + j of weight row lane % 32.  `region` is the wave's parked copy, `ks` the super-block's
// index inside the staged K range.
template <int QT, int NI>
__device__ __forceinline__ void compute(const uint8_t *region, const uint8_t *smem, const Layout &L, int ks, int lane,
                                        float (&out)[4 * NI]) {
    constexpr int MT = 8 * NI, NV = 4 * NI;
    const int h = lane >> 5, n = lane & 31, mrow = lane & (MT - 1);
    const v16i z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const uint8_t *arow = smem + mrow * L.lda + ks * 256;
    const float *dxs = reinterpret_cast<const float *>(smem + L.off_dx);

    if constexpr (QT == kTypeQ4_K) {
        const uint8_t *wrow = region + n * 144;
        const uint4 hdr = *reinterpret_cast<const uint4 *>(wrow);
        uint4 qv[4];
        v4i av[8];
#pragma unroll
        for (int g = 0; g < 4; ++g) qv[g] = *reinterpret_cast<const uint4 *>(wrow + 16 + g * 32 + h * 16);
#pragma unroll
        for (int j = 0; j < 8; ++j) av[j] = *reinterpret_cast<const v4i *>(arow + j * 32 + h * 16);
        const uint4 bs = *reinterpret_cast<const uint4 *>(smem + L.off_aux + (ks * MT + mrow) * 16);
        float4 dxq[NI];
#pragma unroll
        for (int i = 0; i < NI; ++i) dxq[i] = *reinterpret_cast<const float4 *>(dxs + ks * MT + 8 * i + 4 * h);
        __builtin_amdgcn_sched_barrier(0);
        const ScalesK4 sk = unpack_scales_k4(hdr.y, hdr.z, hdr.w);
        const float d = h2f(hdr.x), dmin = h2f(hdr.x >> 16);
        int isum[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) isum[v] = 0;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const uint4 q = qv[g];
            const v4i lo = {(int)(q.x & 0x0f0f0f0fu), (int)(q.y & 0x0f0f0f0fu), (int)(q.z & 0x0f0f0f0fu),
                            (int)(q.w & 0x0f0f0f0fu)};
            const v4i hi = {(int)((q.x >> 4) & 0x0f0f0f0fu), (int)((q.y >> 4) & 0x0f0f0f0fu),
                            (int)((q.z >> 4) & 0x0f0f0f0fu), (int)((q.w >> 4) & 0x0f0f0f0fu)};
            const v16i I0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[2 * g], lo, z, 0, 0, 0);
            const v16i I1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[2 * g + 1], hi, z, 0, 0, 0);
            const int s0 = (int)scale_k4(sk, 2 * g), s1 = (int)scale_k4(sk, 2 * g + 1);
#pragma unroll
            for (int v = 0; v < NV; ++v) isum[v] = __mul24(I1[v], s1) + (__mul24(I0[v], s0) + isum[v]);
        }
        const v4i ahi = h ? v4i{0, 0, 0, 0} : v4i{(int)bs.x, (int)bs.y, 0, 0};
        const v4i alo = h ? v4i{0, 0, 0, 0} : v4i{(int)bs.z, (int)bs.w, 0, 0};
        const v4i bmn = h ? v4i{0, 0, 0, 0} : v4i{(int)sk.mn_lo, (int)sk.mn_hi, 0, 0};
        const v16i Mh = __builtin_amdgcn_mfma_i32_32x32x32_i8(ahi, bmn, z, 0, 0, 0);
        const v16i Ml = __builtin_amdgcn_mfma_i32_32x32x32_i8(alo, bmn, z, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const float dxv[4] = {dxq[i].x, dxq[i].y, dxq[i].z, dxq[i].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int v = 4 * i + j;
                const int msum = (Mh[v] << 6) + Ml[v];
                out[v] = fmaf(dxv[j], d * (float)isum[v] - dmin * (float)msum, out[v]);
            }
        }
    } else if constexpr (QT == kTypeQ6_K) {
        using C = Cfg<kTypeQ6_K>;
        int isum[NV];
        const uint4 sc = *reinterpret_cast<const uint4 *>(region + C::kSc + n * 16);
        const uint32_t scw[4] = {sc.x, sc.y, sc.z, sc.w};
        {   // -32 * sum_j sc_j * bsum_j first (block sums split as 64*hi + lo against the 16 scales): the integer sum
            // starts from it, and the two results are gone before the sixteen products below need their registers
            const uint8_t *aux = smem + L.off_aux + (ks * MT + mrow) * 32;
            const uint2 bhi = *reinterpret_cast<const uint2 *>(aux + 8 * h);
            const uint2 blo = *reinterpret_cast<const uint2 *>(aux + 16 + 8 * h);
            const long bsc = h ? as_i64(sc.z, sc.w) : as_i64(sc.x, sc.y);
            const v16i Ch = __builtin_amdgcn_mfma_i32_32x32x16_i8(as_i64(bhi.x, bhi.y), bsc, z, 0, 0, 0);
            const v16i Cl = __builtin_amdgcn_mfma_i32_32x32x16_i8(as_i64(blo.x, blo.y), bsc, z, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < NV; ++v) isum[v] = -32 * ((Ch[v] << 6) + Cl[v]);
        }
#pragma unroll
        for (int f = 0; f < 2; ++f)
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                // bytes shared by the four sub-blocks k = 0..3: weights 128f + 32k + 16p + 8h + e
                const uint2 qa = *reinterpret_cast<const uint2 *>(region + C::kQl + n * 144 + 64 * f + 16 * p + 8 * h);
                const uint2 qb = *reinterpret_cast<const uint2 *>(region + C::kQl + n * 144 + 64 * f + 32 + 16 * p + 8 * h);
                const uint2 qh = *reinterpret_cast<const uint2 *>(region + C::kQh + n * 80 + 32 * f + 16 * p + 8 * h);
                uint32_t wl[4], wh[4];
                wl[0] = (qa.x & 0x0f0f0f0fu) | ((qh.x << 4) & 0x30303030u);
                wh[0] = (qa.y & 0x0f0f0f0fu) | ((qh.y << 4) & 0x30303030u);
                wl[1] = (qb.x & 0x0f0f0f0fu) | ((qh.x << 2) & 0x30303030u);
                wh[1] = (qb.y & 0x0f0f0f0fu) | ((qh.y << 2) & 0x30303030u);
                wl[2] = ((qa.x >> 4) & 0x0f0f0f0fu) | (qh.x & 0x30303030u);
                wh[2] = ((qa.y >> 4) & 0x0f0f0f0fu) | (qh.y & 0x30303030u);
                wl[3] = ((qb.x >> 4) & 0x0f0f0f0fu) | ((qh.x >> 2) & 0x30303030u);
                wh[3] = ((qb.y >> 4) & 0x0f0f0f0fu) | ((qh.y >> 2) & 0x30303030u);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint2 av = *reinterpret_cast<const uint2 *>(arow + 128 * f + 32 * k + 16 * p + 8 * h);
                    const v16i I = __builtin_amdgcn_mfma_i32_32x32x16_i8(as_i64(av.x, av.y), as_i64(wl[k], wh[k]), z, 0, 0, 0);
                    const int j = 8 * f + 2 * k + p;  // sub-block index
                    const int s = sbyte(scw[j >> 2], j & 3);
#pragma unroll
                    for (int v = 0; v < NV; ++v) isum[v] = __mul24(I[v], s) + isum[v];
                }
                __builtin_amdgcn_sched_barrier(0);   // keeps the four groups' operand loads from piling up in registers
            }
        const float d = h2f(*reinterpret_cast<const uint32_t *>(region + C::kD + n * 4));
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const float4 dx = *reinterpret_cast<const float4 *>(dxs + ks * MT + 8 * i + 4 * h);
            const float dxv[4] = {dx.x, dx.y, dx.z, dx.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int v = 4 * i + j;
                out[v] = fmaf(dxv[j] * d, (float)isum[v], out[v]);
            }
        }
    } else {
        using C = Cfg<kTypeQ8_0>;
        const uint4 dq = *reinterpret_cast<const uint4 *>(region + C::kD + n * 16);
        const uint32_t dw[4] = {dq.x, dq.y, dq.z, dq.w};
#pragma unroll
        for (int blk = 0; blk < 8; ++blk) {
            const v4i av = *reinterpret_cast<const v4i *>(arow + blk * 32 + h * 16);
            const uint4 q = *reinterpret_cast<const uint4 *>(region + n * 272 + blk * 32 + h * 16);
            const v16i I = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, as_v4i(q), z, 0, 0, 0);
            const float wd = h2f(dw[blk >> 1] >> (16 * (blk & 1)));
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const float4 dx = *reinterpret_cast<const float4 *>(dxs + (ks * 8 + blk) * MT + 8 * i + 4 * h);
                const float dxv[4] = {dx.x, dx.y, dx.z, dx.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) out[4 * i + j] = fmaf((float)I[4 * i + j], wd * dxv[j], out[4 * i + j]);
            }
        }
    }
}

// splits a block sum into a signed high byte and a 6-bit low byte: s = 64*hi + lo
__device__ __forceinline__ void split_sum(int s, uint32_t &hi, uint32_t &lo, int pos) {
    hi |= (uint32_t)((s >> 6) & 0xff) << (8 * pos);
    lo |= (uint32_t)(s & 63) << (8 * pos);
}

// Copies the quantized activations of super-blocks [c0, c0 + nsb) into LDS: staged row m (< n_rows) comes from
// activation row src_row(m).
template <int QT, int MT, int kThreads, bool MAPPED>
__device__ __forceinline__ void stage_activations(const MfmaArgs &g, uint8_t *smem, const Layout &L, int c0, int nsb,
                                                  int n_rows, int m0) {
    const int tid = threadIdx.x;
    const int nb = (int)(g.a.K >> 8);
    const int row16 = nsb * 16;
    const int *map = reinterpret_cast<const int *>(smem + L.off_map);
    auto src_row = [&](int m) -> size_t { return MAPPED ? (size_t)(map[m] / g.x_div) : (size_t)(m0 + m); };
    const int total = n_rows * row16;
    for (int base = 0; base < total; base += 4 * kThreads) {
        uint4 v[4];
        int dst[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {   // four independent loads in flight per thread
            const int idx = min(base + u * kThreads + tid, total - 1);
            const int m = idx / row16, j = idx - m * row16;
            v[u] = *reinterpret_cast<const uint4 *>(g.a.qs + src_row(m) * g.a.K + (size_t)c0 * 256 + j * 16);
            dst[u] = m * L.lda + j * 16;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) *reinterpret_cast<uint4 *>(smem + dst[u]) = v[u];
    }
    float *dxs = reinterpret_cast<float *>(smem + L.off_dx);
    constexpr int ND = Cfg<QT>::kDx;
    const int nd = nsb * ND;  // scales per row in this range
    for (int idx = tid; idx < n_rows * nd; idx += kThreads) {
        const int m = idx / nd, j = idx - m * nd;
        dxs[j * MT + m] = g.a.d[src_row(m) * (nb * ND) + c0 * ND + j];
    }
    if constexpr (QT != kTypeQ8_0) {
        for (int idx = tid; idx < n_rows * nsb; idx += kThreads) {
            const int m = idx / nsb, sb = idx - m * nsb;
            const uint4 *src = reinterpret_cast<const uint4 *>(g.a.bsums + (src_row(m) * nb + c0 + sb) * 16);
            const uint4 b0 = src[0], b1 = src[1];
            const uint32_t w[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
            uint8_t *dst = smem + L.off_aux + (sb * MT + m) * Cfg<QT>::kAux;
            if constexpr (QT == kTypeQ4_K) {
                uint32_t hi[2] = {0, 0}, lo[2] = {0, 0};
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int s = (int)(int16_t)(w[j] & 0xffff) + (int)(int16_t)(w[j] >> 16);
                    split_sum(s, hi[j >> 2], lo[j >> 2], j & 3);
                }
                *reinterpret_cast<uint4 *>(dst) = make_uint4(hi[0], hi[1], lo[0], lo[1]);
            } else {
                uint32_t hi[4] = {0, 0, 0, 0}, lo[4] = {0, 0, 0, 0};
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int s = (int)(int16_t)((w[j >> 1] >> (16 * (j & 1))) & 0xffff);
                    split_sum(s, hi[j >> 2], lo[j >> 2], j & 3);
                }
                *reinterpret_cast<uint4 *>(dst) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
                *reinterpret_cast<uint4 *>(dst + 16) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
            }
        }
    }
}

// The same staging in two halves for the expert-grouped launches, whose few rows (a handful of pairs an expert) are
// one request or two a thread: `request` asks for everything -- codes, scales, block sums -- and `store` files it in
// LDS.  In between the workgroup asks for its first weights.  Loads return in order: requested behind the weights
// (as the one-piece version above is), these few kilobytes that sit in L2 came back only after the weights' trip to
// HBM, one dependent round after the other -- 4.6 us of a workgroup's 12.5 (down projection, 64 tokens, phase clocks).
template <int QT, int MT, int kThreads>
struct StagedRows {
    static constexpr int kPieces = 4;
    uint4 v[kPieces], b0, b1;
    int dst[kPieces];
    float dval;
    static __device__ __forceinline__ bool fits(int n_rows, int nsb) {
        return QT != kTypeQ8_0 && MT <= 16 /* (those instances have no registers to spare) */ && n_rows * nsb * 16 <= kPieces * kThreads &&
               n_rows * nsb * Cfg<QT>::kDx <= kThreads;
    }
    __device__ __forceinline__ void request(const MfmaArgs &g, const uint8_t *smem, const Layout &L, int c0, int nsb, int n_rows) {
        const int tid = threadIdx.x, nb = (int)(g.a.K >> 8), row16 = nsb * 16, total = n_rows * row16;
        const int *map = reinterpret_cast<const int *>(smem + L.off_map);
        auto src_row = [&](int m) -> size_t { return (size_t)(map[m] / g.x_div); };
#pragma unroll
        for (int u = 0; u < kPieces; ++u) {
            const int idx = min(u * kThreads + tid, total - 1);
            const int m = idx / row16, j = idx - m * row16;
            v[u] = *reinterpret_cast<const uint4 *>(g.a.qs + src_row(m) * g.a.K + (size_t)c0 * 256 + j * 16);
            dst[u] = m * L.lda + j * 16;
        }
        constexpr int ND = Cfg<QT>::kDx;
        const int nd = nsb * ND;
        dval = 0.f;
        if (tid < n_rows * nd) {
            const int m = tid / nd, j = tid - m * nd;
            dval = g.a.d[src_row(m) * (nb * ND) + c0 * ND + j];
        }
        b0 = b1 = make_uint4(0, 0, 0, 0);
        if (QT != kTypeQ8_0 && tid < n_rows * nsb) {
            const int m = tid / nsb, sb = tid - m * nsb;
            const uint4 *src = reinterpret_cast<const uint4 *>(g.a.bsums + (src_row(m) * nb + c0 + sb) * 16);
            b0 = src[0];
            b1 = src[1];
        }
    }
    __device__ __forceinline__ void store(uint8_t *smem, const Layout &L, int nsb, int n_rows) const {
        const int tid = threadIdx.x;
#pragma unroll
        for (int u = 0; u < kPieces; ++u) *reinterpret_cast<uint4 *>(smem + dst[u]) = v[u];
        constexpr int ND = Cfg<QT>::kDx;
        const int nd = nsb * ND;
        if (tid < n_rows * nd) {
            const int m = tid / nd, j = tid - m * nd;
            reinterpret_cast<float *>(smem + L.off_dx)[j * MT + m] = dval;
        }
        if constexpr (QT != kTypeQ8_0) {
            if (tid < n_rows * nsb) {
                const int m = tid / nsb, sb = tid - m * nsb;
                const uint32_t w[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
                uint8_t *dstb = smem + L.off_aux + (sb * MT + m) * Cfg<QT>::kAux;
                if constexpr (QT == kTypeQ4_K) {
                    uint32_t hi[2] = {0, 0}, lo[2] = {0, 0};
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int s = (int)(int16_t)(w[j] & 0xffff) + (int)(int16_t)(w[j] >> 16);
                        split_sum(s, hi[j >> 2], lo[j >> 2], j & 3);
                    }
                    *reinterpret_cast<uint4 *>(dstb) = make_uint4(hi[0], hi[1], lo[0], lo[1]);
                } else {
                    uint32_t hi[4] = {0, 0, 0, 0}, lo[4] = {0, 0, 0, 0};
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        const int s = (int)(int16_t)((w[j >> 1] >> (16 * (j & 1))) & 0xffff);
                        split_sum(s, hi[j >> 2], lo[j >> 2], j & 3);
                    }
                    *reinterpret_cast<uint4 *>(dstb) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
                    *reinterpret_cast<uint4 *>(dstb + 16) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
                }
            }
        }
    }
};

// The same LDS image made from fp32 rows: each wave quantizes whole 256-element chunks (ggml's
// quantize_row_q8_K, or eight quantize_row_q8_0 blocks for Q8_0 weights) exactly as the standalone
// quantizer kernels do, so both routes stage identical bytes.  Two chunks are in flight per wave.
template <int QT, int MT, int kThreads, bool MAPPED>
__device__ __forceinline__ void stage_quantize(const MfmaArgs &g, uint8_t *smem, const Layout &L, int c0, int nsb,
                                               int n_rows, int m0) {
    constexpr int NWAVES = kThreads / 64;
    const int lane = threadIdx.x & 63, wave = uniform(threadIdx.x >> 6);
    const int *map = reinterpret_cast<const int *>(smem + L.off_map);
    auto src_row = [&](int m) -> size_t { return MAPPED ? (size_t)(map[m] / g.x_div) : (size_t)(m0 + m); };
    float *dxs = reinterpret_cast<float *>(smem + L.off_dx);
    const int total = n_rows * nsb;
    for (int base = 0; base < total; base += 2 * NWAVES) {
        float4 v[2];
        int mm[2], ss[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int idx = min(base + u * NWAVES + wave, total - 1);
            mm[u] = idx / nsb;
            ss[u] = idx - mm[u] * nsb;
            v[u] = *reinterpret_cast<const float4 *>(g.x + src_row(mm[u]) * (size_t)g.a.K + (size_t)(c0 + ss[u]) * 256 + 4 * lane);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            if (base + u * NWAVES + wave >= total) continue;   // wave-uniform
            const int m = mm[u], sb = ss[u];
            uint32_t *dst = reinterpret_cast<uint32_t *>(smem + m * L.lda + sb * 256 + 4 * lane);
            if constexpr (QT == kTypeQ8_0) {
                int s;
                float dd;
                *dst = wave_quantize_q8_32(v[u], s, dd);
                if ((lane & 7) == 0) dxs[(sb * 8 + (lane >> 3)) * MT + m] = h2f(f2h(dd));
            } else {
                int bsum;
                float dd;
                *dst = wave_quantize_q8k(v[u], lane, bsum, dd);
                if (lane == 0) dxs[sb * MT + m] = dd;
                uint8_t *aux = smem + L.off_aux + (sb * MT + m) * Cfg<QT>::kAux;
                if constexpr (QT == kTypeQ4_K) {   // sums of 32: bytes 0..7 high parts, 8..15 low parts
                    const int s32 = bsum + __shfl_xor(bsum, 4);
                    if ((lane & 7) == 0) {
                        aux[lane >> 3] = (uint8_t)((s32 >> 6) & 0xff);
                        aux[8 + (lane >> 3)] = (uint8_t)(s32 & 63);
                    }
                } else {                           // sums of 16: bytes 0..15 high parts, 16..31 low parts
                    if ((lane & 3) == 0) {
                        aux[lane >> 2] = (uint8_t)((bsum >> 6) & 0xff);
                        aux[16 + (lane >> 2)] = (uint8_t)(bsum & 63);
                    }
                }
            }
        }
    }
}

constexpr int kDense = 0, kGrouped = 1, kGroupedSwiglu = 2;

// MODE kDense: y[m][n] for the M rows of `a`.  kGrouped: the workgroup's expert e multiplies its
// own pairs, y[pair][n].  kGroupedSwiglu: tensors 0 and 1 are gate and up of the same expert and
// y[pair][n] = silu(gate . x) * (up . x).
// FLAT (expert-grouped launches with K in one part, kw = 1): the wave's row groups as one stream of items.
template <int QT, int NI, int W, int MODE, bool FLAT = false>
__global__ __launch_bounds__(W * 64) void gemv_mfma_kernel(const MfmaArgs g) {
    static_assert(!FLAT || MODE != kDense, "the flat item stream is for the expert-grouped modes");
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int MT = 8 * NI, NV = 4 * NI;
    constexpr bool GROUPED = MODE != kDense, SWIGLU = MODE == kGroupedSwiglu;
    constexpr int NT = SWIGLU ? 2 : 1;   // tensors streamed by one wave
    const Layout L = layout<QT, MT, W>(g.chunk_sb);
    const int lane = threadIdx.x & 63, wave = uniform(threadIdx.x >> 6);
    const int h = lane >> 5, nl = lane & 31;

    // workgroup -> (tensor or expert, K chunk, set of rw row groups)
    WeightView w = g.t[0].w;
    float *y = g.t[0].y, *part = g.t[0].part;
    int c = 0, rs, expert = 0, pair0 = 0, n_rows = g.M;
    if constexpr (GROUPED) {
        const int slotc = (int)blockIdx.x / g.wgs_per_expert;   // the grid covers min(E, pairs) experts x K chunks
        rs = (int)blockIdx.x - slotc * g.wgs_per_expert;
        const int slot = slotc / g.n_chunks;
        c = slotc - slot * g.n_chunks;
        if (g.ids) {   // a workgroup set per pair
            if (slot >= g.n_pairs) return;
            expert = g.ids[slot];
            if (expert < 0 || expert >= g.n_expert) {   // the pair is left out, as the grouping pass would
                if (rs == 0 && threadIdx.x == 0) atomicOr(g.error_flag, 1);
                return;
            }
            pair0 = slot;
            n_rows = 1;
        } else {
            if (slot >= g.active[g.n_expert]) return;
            const int4 rec = reinterpret_cast<const int4 *>(g.active + active_slots_offset(g.n_expert))[slot];
            expert = rec.x;   // (one load: the list position's expert, first pair slot and pair count)
            pair0 = rec.y;
            n_rows = rec.z;
            if (n_rows <= 0) return;
        }
    } else {
        int ti = 0;
#pragma unroll
        for (int i = 1; i < kMaxTargets; ++i)
            if (i < g.n_targets && (int)blockIdx.x >= g.t[i].first_wg) ti = i;
        int first = g.t[0].first_wg, nrs = g.t[0].n_rowsets;
#pragma unroll
        for (int i = 1; i < kMaxTargets; ++i)
            if (ti == i) {
                w = g.t[i].w;
                y = g.t[i].y;
                part = g.t[i].part;
                first = g.t[i].first_wg;
                nrs = g.t[i].n_rowsets;
            }
        const int local = (int)blockIdx.x - first;
        c = local / nrs;
        rs = local - c * nrs;
    }
    const int N = (int)w.N;
    const int nb = (int)(g.a.K >> 8);
    const int c0 = c * g.chunk_sb, nsb = min(g.chunk_sb, nb - c0);
    if constexpr (GROUPED)   // K in chunks: the chunk's results go to its plane of the scratch, a pass adds the planes
        if (g.n_chunks > 1) y = part + (size_t)c * g.part_plane;

    // wave -> (row group, K part)
    const int rgl = wave / g.kw, kp = wave - rgl * g.kw;
    const int part_sb = (nsb + g.kw - 1) / g.kw;
    const int s0 = min(kp * part_sb, nsb), s1 = min(s0 + part_sb, nsb);  // range inside the staged chunk
    int row0 = 0, steps = 0, items = 0, last_sb = c0;
    bool rows_ok = false;
    Stager<QT> sa, sb_;
    // the wave's rg-th row group: rows, how much of K, where its blocks start
    auto set_rowgroup = [&](int rg) {
        row0 = ((rs * (GROUPED ? g.rg_loop : 1) + rg) * g.rw + rgl) * (GROUPED ? 32 : g.rpg);
        rows_ok = row0 < N;
        steps = rows_ok ? s1 - s0 : 0;
        items = NT * steps;                       // (tensor, super-block) pairs this wave streams
        last_sb = c0 + (steps > 0 ? s1 - 1 : 0);  // loads past the range repeat its last super-block
        const int64_t row = (int64_t)expert * N + (rows_ok ? row0 : 0);
        sa.rebase(0, w, row);
        sa.rebase(1, SWIGLU ? g.t[1].w : w, row);
        const int last_row = rows_ok ? min((GROUPED ? 32 : g.rpg) - 1, N - 1 - row0) : 0;   // rows past it repeat it
        sa.init(w, last_row, lane);
        sb_.rebase(0, w, row);
        sb_.rebase(1, SWIGLU ? g.t[1].w : w, row);
        sb_.init(w, last_row, lane);
    };
    // item i -> tensor i / steps, super-block c0 + s0 + i % steps (clamped: harmless repeats past the end)
    auto issue = [&](Stager<QT> &st, int i) {
        const int t = SWIGLU && steps > 0 && i >= steps ? 1 : 0;
        st.issue(t, min(c0 + s0 + i - t * steps, last_sb));
    };
    uint8_t *region = smem + L.off_w + wave * Cfg<QT>::kRegion;
    int *map = reinterpret_cast<int *>(smem + L.off_map);

    // Expert-grouped launches with K in one part: the wave's row groups are ONE stream of (row group, tensor,
    // super-block) items, so the loads of the next row group are in flight while the last items of this one are
    // worked on (with short K a row group is three items: restarting the pipeline for each one left the memory
    // system idle for a round trip per row group).
    if constexpr (FLAT) {
        {
            const int per = NT * nsb;   // items of a row group
            int n_rg = 0;               // the wave's row groups that exist (a prefix)
            for (int rg = 0; rg < g.rg_loop; ++rg) n_rg += ((rs * g.rg_loop + rg) * g.rw + rgl) * 32 < N ? 1 : 0;
            const int total = n_rg * per;
            auto row_of = [&](int rg) { return ((rs * g.rg_loop + rg) * g.rw + rgl) * 32; };
            auto setup = [&](Stager<QT> &st, int rg) {
                const int r0 = row_of(rg);
                const int64_t row = (int64_t)expert * N + r0;
                st.rebase(0, w, row);
                st.rebase(1, SWIGLU ? g.t[1].w : w, row);
                st.init(w, min(31, N - 1 - r0), lane);
            };
            int rg_a = -1, rg_b = -1;   // the row group each stager's addresses stand at
            auto issue_at = [&](Stager<QT> &st, int &st_rg, int rg, int i) {
                if (rg >= n_rg) {   // past the end: the last item again, harmless
                    rg = n_rg - 1;
                    i = per - 1;
                }
                if (rg != st_rg) {
                    setup(st, rg);
                    st_rg = rg;
                }
                const int t = SWIGLU && i >= nsb ? 1 : 0;
                st.issue(t, c0 + i - t * nsb);
            };
            for (int m0 = 0; m0 < n_rows; m0 += MT) {
                const int m_cnt = min(MT, n_rows - m0);
                // cursors of the two stagers (items 0, 2, 4, .. and 1, 3, 5, ..) and of the consumer; a wave whose row
                // groups all lie past the end of the matrix (total = 0) only takes part in the staging and the barriers
                int arg = 0, ai = 0, brg = 0, bi = 1, crg = 0, ci = 0;
                while (bi >= per) { bi -= per; ++brg; }
                // rows quantized earlier, few enough for one request round: asked for AHEAD of the first weights
                const bool rows_first = !g.x && StagedRows<QT, MT, W * 64>::fits(m_cnt, nsb);
                if (!rows_first && total > 0) {
                    issue_at(sa, rg_a, arg, ai);
                    issue_at(sb_, rg_b, brg, bi);
                }
                if (m0 > 0) __syncthreads();   // the previous pass is done with the staged rows and the regions
                if ((int)threadIdx.x < MT)
                    map[threadIdx.x] = (int)threadIdx.x >= m_cnt ? 0
                                       : g.ids      ? pair0 + m0 + (int)threadIdx.x
                                                    : g.order[pair0 + m0 + (int)threadIdx.x];
                __syncthreads();
                if (rows_first) {
                    StagedRows<QT, MT, W * 64> rows;
                    rows.request(g, smem, L, c0, nsb, m_cnt);
                    if (total > 0) {
                        issue_at(sa, rg_a, arg, ai);
                        issue_at(sb_, rg_b, brg, bi);
                    }
                    rows.store(smem, L, nsb, m_cnt);
                } else if (g.x) {
                    stage_quantize<QT, MT, W * 64, GROUPED>(g, smem, L, c0, nsb, m_cnt, m0);
                } else {
                    stage_activations<QT, MT, W * 64, GROUPED>(g, smem, L, c0, nsb, m_cnt, m0);
                }
                __syncthreads();

                float out[NT][NV];
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int v = 0; v < NV; ++v) out[t][v] = 0.f;
                auto consume = [&]() {
                    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                    if (SWIGLU && ci >= nsb)
                        compute<QT, NI>(region, smem, L, ci - nsb, lane, out[NT - 1]);
                    else
                        compute<QT, NI>(region, smem, L, ci, lane, out[0]);
                    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                    if (++ci == per) {   // the row group is complete: store it, start the next one
                        const int n = row_of(crg) + nl;
#pragma unroll
                        for (int v = 0; v < NV; ++v) {
                            const int m = 8 * (v >> 2) + 4 * h + (v & 3);
                            float r = out[0][v];
                            if constexpr (SWIGLU) r = (r / (1.0f + expf(-r))) * out[NT - 1][v];
                            if (m < m_cnt && n < N) y[(size_t)map[m] * N + n] = r;
                        }
#pragma unroll
                        for (int t = 0; t < NT; ++t)
#pragma unroll
                            for (int v = 0; v < NV; ++v) out[t][v] = 0.f;
                        ci = 0;
                        ++crg;
                    }
                };
                auto advance2 = [&](int &rg, int &i) {
                    i += 2;
                    while (i >= per) { i -= per; ++rg; }
                };
                int j = 0;
                for (; j + 1 < total; j += 2) {
                    sa.park(region, lane);
                    advance2(arg, ai);
                    issue_at(sa, rg_a, arg, ai);
                    consume();
                    sb_.park(region, lane);
                    advance2(brg, bi);
                    issue_at(sb_, rg_b, brg, bi);
                    consume();
                }
                if (j < total) {
                    sa.park(region, lane);
                    consume();
                }
            }
            return;
        }
    }

    // dense launches stage all (<= MT) rows at once; an expert with more than MT pairs takes several passes
    if constexpr (!FLAT)
    for (int m0 = 0; m0 < (GROUPED ? n_rows : 1); m0 += MT)
    for (int rg = 0; rg < (GROUPED ? g.rg_loop : 1); ++rg) {   // the rows staged for this pass serve all of the wave's row groups
        const int m_cnt = min(MT, n_rows - m0);
        set_rowgroup(rg);
        issue(sa, 0);
        issue(sb_, 1);
        if (rg == 0) {
            if constexpr (GROUPED) {
                if (m0 > 0) __syncthreads();   // the previous pass is done with the staged rows and the regions
                if ((int)threadIdx.x < MT)
                    map[threadIdx.x] = (int)threadIdx.x >= m_cnt ? 0
                                       : g.ids      ? pair0 + m0 + (int)threadIdx.x
                                                    : g.order[pair0 + m0 + (int)threadIdx.x];
                __syncthreads();
            }
            if (g.x)
                stage_quantize<QT, MT, W * 64, GROUPED>(g, smem, L, c0, nsb, m_cnt, m0);
            else
                stage_activations<QT, MT, W * 64, GROUPED>(g, smem, L, c0, nsb, m_cnt, m0);
            __syncthreads();
        } else if (g.kw > 1) {
            __syncthreads();   // the partial tiles the previous row group left in the regions have been summed
        }

        float out[NT][NV];
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int v = 0; v < NV; ++v) out[t][v] = 0.f;
        auto consume = [&](int i) {
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            if (SWIGLU && i >= steps)
                compute<QT, NI>(region, smem, L, s0 + i - steps, lane, out[NT - 1]);
            else
                compute<QT, NI>(region, smem, L, s0 + i, lane, out[0]);
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        };
        int i = 0;
        for (; i + 1 < items; i += 2) {
            sa.park(region, lane);
            issue(sa, i + 2);
            consume(i);
            sb_.park(region, lane);
            issue(sb_, i + 3);
            consume(i + 1);
        }
        if (i < items) {
            sa.park(region, lane);
            consume(i);
        }

        // sum the K parts of a row group in a fixed order (through the waves' regions), then store
        if (g.kw > 1) {
            float *mine = reinterpret_cast<float *>(region);
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int v = 0; v < NV; ++v)
                    mine[t * (MT * 32) + (8 * (v >> 2) + 4 * h + (v & 3)) * 32 + nl] = out[t][v];
            __syncthreads();
            if (kp == 0) {
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int v = 0; v < NV; ++v) {
                        const uint8_t *src = region + (t * (MT * 32) + (8 * (v >> 2) + 4 * h + (v & 3)) * 32 + nl) * 4;
                        float acc = *reinterpret_cast<const float *>(src);
                        for (int q = 1; q < g.kw; ++q) acc += *reinterpret_cast<const float *>(src + q * Cfg<QT>::kRegion);
                        out[t][v] = acc;
                    }
            }
        }
        if (kp == 0 && rows_ok) {
            const bool add = !GROUPED && g.add_out;
            float *dst = GROUPED || g.n_chunks == 1 || add ? y : part + (size_t)c * g.M * N;
            const int n = row0 + nl;
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const int m = 8 * (v >> 2) + 4 * h + (v & 3);
                float r = out[0][v];
                if constexpr (SWIGLU) r = (r / (1.0f + expf(-r))) * out[NT - 1][v];
                if (m < m_cnt && n < N && (GROUPED || nl < g.rpg)) {
                    float *o = dst + (size_t)(GROUPED ? map[m] : m0 + m) * N + n;
                    // two addends on zero: the sum does not depend on which chunk arrives first
                    if (add) unsafeAtomicAdd(o, r);
                    else *o = r;
                }
            }
        }
    }
}

// y[i] = sum over chunks of part[c][i], chunk order fixed
__global__ __launch_bounds__(256) void sum_chunks_kernel(const MfmaArgs g) {
    for (int ti = 0; ti < g.n_targets; ++ti) {
        const size_t n = (size_t)g.M * g.t[ti].w.N;
        for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
            float s = g.t[ti].part[i];
            for (int c = 1; c < g.n_chunks; ++c) s += g.t[ti].part[(size_t)c * n + i];
            g.t[ti].y[i] = s;
        }
    }
}

template <int QT, int NI, int W, int MODE, bool FLAT = false>
hipError_t launch_one(const MfmaArgs &g, hipStream_t s) {
    // (the 16-row instances of the larger formats would spill registers in the flat form: they keep the loop per row group)
    if constexpr (MODE != kDense && !FLAT && (QT == kTypeQ4_K || NI == 1)) {
        static const bool no_flat = tuning_int("QPROJ_MOE_NO_FLAT", 0) != 0;
        if (g.kw == 1 && !no_flat) return launch_one<QT, NI, W, MODE, true>(g, s);
    }
    // K parts of a row group are summed through the waves' regions: a wave's partial tile must fit its region
    if (g.kw > 1 && (MODE == kGroupedSwiglu ? 2 : 1) * (8 * NI) * 32 * 4 > Cfg<QT>::kRegion) return hipErrorInvalidValue;
    if (dry_run()) {
        if (g.n_chunks > 1 && !g.add_out) plan_note_cut();
        plan_note("gemv_mfma_kernel<%s, %d staged rows, %d waves, %s%s>: %d workgroups, K in %d chunk(s) of %d super-blocks x %d parts a row group of %d rows%s",
                  plan_type_name(QT), 8 * NI, W, MODE == kDense ? "dense" : MODE == kGroupedSwiglu ? "expert-grouped + swiglu" : "expert-grouped",
                  FLAT ? ", one item stream a wave" : "", g.n_wgs, g.n_chunks, g.chunk_sb, g.kw, MODE == kDense ? g.rpg : 32,
                  g.n_chunks == 1 ? "" : g.add_out ? ", the two chunks add themselves to cleared rows"
                                   : MODE == kDense ? " + sum_chunks_kernel" : " + sum_parts_kernel");
        return hipSuccess;
    }
    const Layout L = layout<QT, 8 * NI, W>(g.chunk_sb);
    auto kern = gemv_mfma_kernel<QT, NI, W, MODE, FLAT>;
    static int allowed = 0;
    if (L.total > allowed) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, L.total);
        if (e != hipSuccess) return e;
        allowed = L.total;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)g.n_wgs), dim3(W * 64), (size_t)L.total, s, g);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || g.n_chunks == 1 || g.add_out || MODE != kDense) return e;
    size_t n_out = 0;
    for (int i = 0; i < g.n_targets; ++i) n_out = std::max(n_out, (size_t)g.M * (size_t)g.t[i].w.N);
    const unsigned blocks = (unsigned)std::min<size_t>(256, (n_out + 255) / 256);
    hipLaunchKernelGGL(sum_chunks_kernel, dim3(blocks), dim3(256), 0, s, g);
    return hipGetLastError();
}

int waves_per_wg(int type) {
    static const int w = [] {
        const int v = tuning_int("QPROJ_MFMA_WAVES", 8);
        return v == 4 || v == 16 ? v : 8;
    }();
    return w == 16 && type != kTypeQ4_K ? 8 : w;   // 16 regions of the larger formats do not fit LDS
}

// The split of K: how many chunks (workgroups along K) and K parts (waves along K inside a workgroup).
struct Split {
    int n_chunks, chunk_sb, kw;
};
constexpr int kMaxSb16 = 16;   // super-blocks of 16 staged rows that fit LDS beside the wave regions (~66 KB)
// `dense`: the launch is one workgroup a compute unit (eight waves of ~200 registers), so the K parts are chosen
// with the chunks that LDS forces counted in, and a grid of a round and a bit is traded for one round of longer
// workgroups.  (Before, 16 rows of K = 14336 got 8 K parts x 4 chunks = 512 workgroups, two rounds: the Q6_K down
// projection 36.3 -> 26.9 us with 4 K parts, 256 workgroups; Q4_K 14336 -> 4096 28.0 -> 20.2, 8192 x 8192 28.7 ->
// 21.8; 13824 -> 5120 at 8 rows 37.7 -> 27.5 with 4 K parts x 3 chunks = 240 workgroups instead of 8 x 2 = 320.)
Split plan(int64_t K, int64_t M, int64_t total_rg, int W, int min_wgs = 200, bool dense = false, int cus = 256) {
    const int nb = (int)(K / 256);
    const int max_sb = M <= 8 ? 2 * kMaxSb16 : M <= 16 ? kMaxSb16 : kMaxSb16 / 2;
    int nc = (nb + max_sb - 1) / max_sb;
    const int nc_forced = dense ? nc : 1;
    Split p;
    p.kw = 1;
    while (p.kw < W && p.kw * 2 <= nb && total_rg * p.kw / W * nc_forced < min_wgs) p.kw *= 2;
    auto wgs_of = [&](int kw) { return (total_rg + W / kw - 1) / (W / kw); };
    if (dense && p.kw > 1 && wgs_of(p.kw) * nc > cus && wgs_of(p.kw / 2) * nc <= cus) p.kw /= 2;
    const int64_t wgs1 = wgs_of(p.kw);
    // few workgroups: more chunks - in a dense launch (one workgroup a compute unit) as many as still make ONE round
    // (96 row-group sets of K = 8192 got three chunks, 288 workgroups, a round and an eighth: Q4_K 8192 -> 3072 at
    // 4 / 8 rows 20.6 / 20.8 us against 15.8 at 16 rows, whose two chunks are 192)
    if (wgs1 * nc < 128)
        nc = std::max(nc, (int)std::min<int64_t>(std::max(1, nb / p.kw), dense ? std::max<int64_t>(1, cus / wgs1) : (255 + wgs1) / wgs1));
    else if (dense && nc > 1 && wgs1 * nc * 10 < cus * 7)   // the sum over chunks is paid for anyway: fill the round
        nc = std::max(nc, (int)std::min<int64_t>(std::max(1, nb / p.kw), cus / wgs1));
    p.chunk_sb = (nb + nc - 1) / nc;
    p.n_chunks = (nb + p.chunk_sb - 1) / p.chunk_sb;
    return p;
}

template <int QT, int NI, int MODE>
hipError_t launch_w(const MfmaArgs &g, int W, hipStream_t s) {
    if (W == 4) return launch_one<QT, NI, 4, MODE>(g, s);
    if constexpr (QT == kTypeQ4_K)
        if (W == 16) return launch_one<QT, NI, 16, MODE>(g, s);
    return launch_one<QT, NI, 8, MODE>(g, s);
}

// ni: activation rows a pass in eights -- 1, 2, or (dense launches of eight waves only) 4: all 32 token rows of the
// matrix instruction carry a row of their own, at the same number of matrix instructions
template <int MODE>
hipError_t launch_typed(const MfmaArgs &g, int type, int ni, int W, hipStream_t s) {
    if (ni == 4) {
        if constexpr (MODE == kDense) {
            if (W != 8) return hipErrorInvalidValue;
            if (type == kTypeQ4_K) return launch_one<kTypeQ4_K, 4, 8, kDense>(g, s);
            if (type == kTypeQ6_K) return launch_one<kTypeQ6_K, 4, 8, kDense>(g, s);
            return launch_one<kTypeQ8_0, 4, 8, kDense>(g, s);
        } else {
            // expert-grouped: Q4_K experts with K of at most eight super-blocks (the staged rows of 32 pairs)
            if (W != 8 || type != kTypeQ4_K) return hipErrorInvalidValue;
            return launch_one<kTypeQ4_K, 4, 8, MODE>(g, s);
        }
    }
    const bool small = ni == 1;
    if (type == kTypeQ4_K) return small ? launch_w<kTypeQ4_K, 1, MODE>(g, W, s) : launch_w<kTypeQ4_K, 2, MODE>(g, W, s);
    if (type == kTypeQ6_K) return small ? launch_w<kTypeQ6_K, 1, MODE>(g, W, s) : launch_w<kTypeQ6_K, 2, MODE>(g, W, s);
    return small ? launch_w<kTypeQ8_0, 1, MODE>(g, W, s) : launch_w<kTypeQ8_0, 2, MODE>(g, W, s);
}

// waves a workgroup of a dense launch: the 32-row instances exist for eight waves only
int dense_waves(int type, int64_t M) { return M > 16 ? 8 : waves_per_wg(type); }

}  // namespace

bool mfma_gemv_fits(int type, int64_t M, int64_t K) {
    (void)type;
    return M >= 1 && M <= 32 && K % 256 == 0;
}

bool mfma_grouped_fits(int type, int64_t K) {
    (void)type;
    return K % 256 == 0 && K / 256 <= kMaxSb16;
}

// Expert-grouped launches of rows longer than the staged rows of a pass allow (K / 256 > 32 with 8 rows a pass, > 16
// with 16): K goes in chunks, one set of workgroups a chunk, each chunk's results to its own plane [n_pairs][N] of
// the scratch, added up in chunk order by a pass afterwards.  Not for the gate / up launch with its SwiGLU epilogue.
int mfma_grouped_chunks(int64_t K, int64_t n_pairs, int64_t E) {
    const int nb = (int)(K / 256);
    const int max_sb = n_pairs <= 4 * E ? 2 * kMaxSb16 : kMaxSb16;
    return (nb + max_sb - 1) / max_sb;
}
bool mfma_grouped_chunked_fits(int type, int64_t K, int64_t N, int64_t n_pairs) {
    (void)type;
    return K % 256 == 0 && K / 256 > kMaxSb16 && (n_pairs * N) % 4 == 0;
}
size_t mfma_grouped_scratch_bytes(int64_t K, int64_t N, int64_t n_pairs, int64_t E) {
    const int nc = mfma_grouped_chunks(K, n_pairs, E);
    return nc > 1 ? (size_t)nc * (size_t)n_pairs * (size_t)N * 4 : 0;
}

size_t mfma_gemv_scratch_bytes(int type, int64_t K, int64_t M, int64_t sum_n, int64_t total_rg) {
    const Split p = plan(K, M, total_rg, dense_waves(type, M), 200, true, cu_count());
    return p.n_chunks > 1 ? (size_t)p.n_chunks * (size_t)M * (size_t)sum_n * 4 : 0;
}

bool mfma_gemv_two_chunks(int type, int64_t K, int64_t M, int64_t total_rg) {
    static const bool off = tuning_int("QPROJ_NO_CHUNK_ADD", 0) != 0;
    return !off && plan(K, M, total_rg, dense_waves(type, M), 200, true, cu_count()).n_chunks == 2;
}

hipError_t launch_gemv_mfma(const GemvArgs &args, const Scratch &scratch, hipStream_t s) {
    MfmaArgs g{};
    g.n_targets = args.n_targets;
    g.a = args.a;
    g.x = args.x;
    g.M = args.M;
    g.x_div = 1;
    int64_t total_rg = 0;
    for (int i = 0; i < args.n_targets; ++i) total_rg += (args.t[i].w.N + 31) / 32;
    if (args.M < 1 || args.M > 32) return hipErrorInvalidValue;
    const int W = dense_waves(args.t[0].w.type, args.M);
    const Split p = plan(args.a.K, args.M, total_rg, W, 200, true, cu_count());
    g.n_chunks = p.n_chunks;
    g.chunk_sb = p.chunk_sb;
    g.kw = p.kw;
    g.rw = W / p.kw;
    g.rg_loop = 1;
    g.add_out = args.y_zeroed && mfma_gemv_two_chunks(args.t[0].w.type, args.a.K, args.M, total_rg);
    // Rows a row group.  The kernel streams weights and the matrix cores idle, so a grid that leaves compute units
    // without a workgroup is evened out with row groups of fewer than the instruction's 32 rows (the spare columns
    // repeat the group's last row and are not stored): the fewest rows, 24 at least, whose grid is still one round.
    // Gate + up of 14336 rows each are 896 groups of 32 = 224 workgroups, and 1024 groups of 28 = 256.
    const auto wgs_with = [&](int rpg) {
        int64_t n = 0;
        for (int i = 0; i < args.n_targets; ++i) n += ((args.t[i].w.N + rpg - 1) / rpg + g.rw - 1) / g.rw;
        return n * g.n_chunks;
    };
    g.rpg = 32;
    static const bool even_out = tuning_int("QPROJ_MFMA_NO_SHORT_GROUPS", 0) == 0;
    if (even_out && wgs_with(32) < cu_count())
        for (int r = 31; r >= 24 && wgs_with(r) <= cu_count(); --r) g.rpg = r;
    int wg = 0;
    size_t part_off = 0;
    for (int i = 0; i < args.n_targets; ++i) {
        g.t[i].w = args.t[i].w;
        g.t[i].y = args.t[i].y;
        g.t[i].part = scratch.p ? scratch.p + part_off : nullptr;
        part_off += (size_t)g.n_chunks * args.M * args.t[i].w.N;
        const int n_rg = (int)((args.t[i].w.N + g.rpg - 1) / g.rpg);
        g.t[i].n_rowsets = (n_rg + g.rw - 1) / g.rw;
        g.t[i].first_wg = wg;
        wg += g.t[i].n_rowsets * g.n_chunks;
    }
    g.n_wgs = wg;
    // the per-chunk results of all targets lie one behind the other in the scratch: refuse what would not fit
    if (g.n_chunks > 1 && !g.add_out && (!scratch.p || part_off * sizeof(float) > scratch.bytes)) return hipErrorInvalidValue;
    return launch_typed<kDense>(g, args.t[0].w.type, args.M <= 8 ? 1 : args.M <= 16 ? 2 : 4, W, s);
}

// Expert-grouped form: args.order / args.offsets list each expert's pairs; `swiglu` takes tensors 0 and 1
// as gate and up.  n_pairs only steers the launch shape (how many experts can be busy at once).
hipError_t launch_gemv_mfma_grouped(const GemvArgs &args, int64_t n_pairs, bool swiglu, hipStream_t s, const Scratch &scratch) {
    MfmaArgs g{};
    g.n_targets = swiglu ? 2 : 1;
    g.a = args.a;
    g.x = args.x;
    g.M = 0;
    g.order = args.order;
    g.offsets = args.offsets;
    g.active = args.active;
    g.x_div = args.x_div;
    const WeightView &w = args.t[0].w;
    const int type = w.type;
    // Q4_K experts: four waves a workgroup, two workgroups a compute unit - the prologue of one (expert lookup,
    // row map, staged rows: a chain of dependent loads) hides behind the other's weight stream.  Measured on the
    // 128-expert FFN against eight waves: 23.2 -> 21.1 us at one token, 121.9 -> 115.5 us at 64.
    static const int moe_waves = tuning_int("QPROJ_MOE_WAVES", 4);
    const int64_t rg_e = (w.N + 31) / 32;
    const bool small = n_pairs <= 4 * w.E;   // few pairs an expert: 8 staged rows a pass are enough
    // more than 16 pairs an expert (prompt-sized batches): 32 staged rows a pass halve the passes over an expert's
    // weights (Q4_K experts whose K fits LDS beside 32 rows; eight waves, one workgroup a compute unit)
    static const bool no_wide_pass = tuning_int("QPROJ_MOE_NO_32_ROW_PASS", 0) != 0;
    bool wide_pass = !no_wide_pass && !args.ids && type == kTypeQ4_K && w.K / 256 <= kMaxSb16 / 2 && n_pairs > 16 * w.E;
    // (only with K in one part a wave: the partial tiles of K parts, 32 rows x 32 x two tensors, would not fit a wave's region)
    if (wide_pass && plan(w.K, 32, std::min<int64_t>(w.E, n_pairs) * rg_e, 8).kw != 1) wide_pass = false;
    const int W = wide_pass ? 8 : type == kTypeQ4_K && (moe_waves == 4 || moe_waves == 8) ? moe_waves : waves_per_wg(type);
    Split p = plan(w.K, small ? 8 : wide_pass ? 32 : 16, std::min<int64_t>(w.E, n_pairs) * rg_e, W);
    const int nb = (int)(w.K / 256);
    // K stays inside one workgroup unless the staged rows of a pass do not fit: then the chunks LDS forces, no more
    const int nc = wide_pass ? 1 : mfma_grouped_chunks(w.K, n_pairs, w.E);
    if (nc > 1) {
        if (swiglu || args.ids || !scratch.p || (size_t)nc * (size_t)n_pairs * (size_t)w.N * 4 > scratch.bytes ||
            (n_pairs * w.N) % 4 != 0)
            return hipErrorInvalidValue;
        p.chunk_sb = (nb + nc - 1) / nc;
        p.n_chunks = (nb + p.chunk_sb - 1) / p.chunk_sb;
        while (p.kw > 1 && p.kw * 2 > p.chunk_sb) p.kw /= 2;   // K parts of a chunk, not of the row
    } else {
        p.n_chunks = 1;
        p.chunk_sb = nb;
    }
    g.n_chunks = p.n_chunks;
    g.chunk_sb = p.chunk_sb;
    g.part_plane = n_pairs * w.N;
    g.kw = p.kw;
    g.rw = W / p.kw;
    for (int i = 0; i < g.n_targets; ++i) {
        g.t[i].w = args.t[i].w;
        g.t[i].y = args.t[i].y;
        g.t[i].part = g.n_chunks > 1 ? scratch.p : nullptr;
    }
    // Short K makes a row group a few steps of work against a prologue (row map, staged rows, barriers) of
    // several microseconds.  A wave can take two row groups in a row (one stream of items) and pay the prologue
    // once; measured on the 128-expert FFN (K = 768 down, K = 2048 gate / up): worth it for grids beyond three
    // workgroups per compute unit (down at 8 and 64 tokens: 62.3 -> 58.8 and 115.5 -> 111.3 us), harmful for small
    // grids (one token: 21.1 -> 22.9 us; gate / up at 64 tokens, 744 workgroups: 111.3 -> 128 us).  Four in a row
    // lost everywhere at first; with the shorter prologue they pay for the down projection where an expert has more
    // than four pairs (16 staged rows a pass), Q4_K experts: 118.0 -> 111.4 us a call at 96 tokens, 121.8 -> 117.3 at
    // 128, 169.0 -> 159.8 at 256 (Q6_K down experts, which keep the loop per row group there: 180.5 -> 184.9, so two).
    static const int forced_all = tuning_int("QPROJ_MOE_RG_LOOP", 0), forced_down = tuning_int("QPROJ_MOE_RG_LOOP_DOWN", 0);
    const int forced_loop = !swiglu && forced_down > 0 ? forced_down : forced_all;
    {
        const int64_t wgs1 = (args.ids ? n_pairs : std::min<int64_t>(w.E, n_pairs)) * ((rg_e + g.rw - 1) / g.rw);
        const int64_t cus = 256;
        int loop = forced_loop > 0 ? forced_loop : wgs1 > 3 * cus ? (!small && !swiglu && type == kTypeQ4_K ? 4 : 2) : 1;
        loop = (int)std::min<int64_t>(loop, std::max<int64_t>(1, rg_e / g.rw));
        while (loop > 1 && rg_e % ((int64_t)g.rw * loop) != 0) --loop;   // no half-empty last workgroup
        g.rg_loop = std::min(loop, 8);
    }
    g.wgs_per_expert = (int)((rg_e + (int64_t)g.rw * g.rg_loop - 1) / ((int64_t)g.rw * g.rg_loop));
    g.n_expert = (int)w.E;
    g.ids = args.ids;
    g.n_pairs = args.n_pairs;
    g.error_flag = args.error_flag;
    g.n_wgs = (int)((args.ids ? n_pairs : std::min<int64_t>(w.E, n_pairs)) * g.n_chunks * g.wgs_per_expert);
    const int ni = small ? 1 : wide_pass ? 4 : 2;
    if (swiglu) return launch_typed<kGroupedSwiglu>(g, type, ni, W, s);
    hipError_t e = launch_typed<kGrouped>(g, type, ni, W, s);
    if (e != hipSuccess || g.n_chunks == 1 || dry_run()) return e;
    return launch_sum_parts(scratch.p, g.n_chunks, (size_t)n_pairs * (size_t)w.N, args.t[0].y, s);
}

}  // namespace qproj
