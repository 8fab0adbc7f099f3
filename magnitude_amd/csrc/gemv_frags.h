// Per-lane pieces of the int8-activation projection kernels, one set per weight type:
//   Raw<QT>  : the registers one lane loads of one weight row for one chunk of K (nothing
//              decoded, so it can sit in flight across a loop iteration as a prefetch);
//   Frag<QT> : the same data decoded into int8 lanes, integer sub-scales and the fp32 scale;
//   Dot<QT>  : the lane's slice of one quantized activation row and the partial dot product.
//
// Chunk geometry (weights of one row covered by one wave per step):
//   Q4_K : 4096 weights = 16 super-blocks; lane = (super-block, 64-chunk c): 32 bytes of qs =
//          32 low nibbles (sub-block 2c) + 32 high nibbles (sub-block 2c+1), plus the 16-byte
//          block header (read by the 4 lanes of the super-block, one request);
//   Q6_K : 4096 weights = 16 super-blocks; lane = (super-block, 128-half h, 16-run e): 16 bytes
//          of each of the two ql runs and of qh = four 16-weight groups, each with one scale
//          and one Q8_K bsum;
//   Q8_0 : 1024 weights = 32 blocks; lane = half a block (16 int8).
#pragma once

#include "qproj_device.h"
#include "qproj_internal.h"

namespace qproj {

template <int QT> struct Geo;
template <> struct Geo<kTypeQ4_K> {
    static constexpr int kChunk = 4096, kBlk = 256, kLanesPerBlk = 4;
};
template <> struct Geo<kTypeQ6_K> {
    static constexpr int kChunk = 4096, kBlk = 256, kLanesPerBlk = 4;
};
template <> struct Geo<kTypeQ8_0> {
    static constexpr int kChunk = 1024, kBlk = 32, kLanesPerBlk = 2;
};
// Q8_0 for the decode kernel: a step covers 4096 weights as four 1024-wide parts, lane l holding half a block
// (16 weights) of each -- blocks l/2, 32 + l/2, 64 + l/2, 96 + l/2 of the chunk -- so that a row of K = 4096
// is one step of five loads a lane instead of four dependent steps.  Same planes, same arithmetic per block.
constexpr int kTypeQ8_0Wide = 1008;
template <> struct Geo<kTypeQ8_0Wide> {
    static constexpr int kChunk = 4096, kBlk = 32, kLanesPerBlk = 2;
};
template <int QT> constexpr bool is_q8_0 = QT == kTypeQ8_0 || QT == kTypeQ8_0Wide;

// block (super-block) index inside the row that `lane` works on in the chunk starting at k0
template <int QT>
__device__ __forceinline__ int64_t lane_block(int64_t k0, int lane) {
    return k0 / Geo<QT>::kBlk + lane / Geo<QT>::kLanesPerBlk;
}

// Wave-uniform values are kept in SGPRs explicitly: the compiler cannot prove that
// threadIdx.x / 64 is uniform, and without this every row address becomes 64-bit VALU math.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int64_t uniform64(int64_t v) {
    const int lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const int hi = __builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)(uint32_t)hi << 32) | (uint32_t)lo);
}

// Start of one weight row in each plane (wave-uniform pointers).
template <int QT> struct RowPtr;
template <> struct RowPtr<kTypeQ4_K> {
    const uint8_t *p;
    uint32_t nb;  // blocks per row: row r of the walk starts r * nb blocks further on
    __device__ __forceinline__ void set(const WeightView &w, int64_t row) {
        p = w.q4k + row * w.nb * 144;
        nb = (uint32_t)w.nb;
    }
    __device__ __forceinline__ const void *dummy() const { return p; }
};
template <> struct RowPtr<kTypeQ6_K> {
    const uint8_t *ql, *qh;
    const int8_t *sc;
    const uint16_t *d;
    uint32_t nb;
    __device__ __forceinline__ void set(const WeightView &w, int64_t row) {
        const int64_t b = row * w.nb;
        nb = (uint32_t)w.nb;
        ql = w.q6_ql + b * 128;
        qh = w.q6_qh + b * 64;
        sc = w.q6_sc + b * 16;
        d = w.q6_d + b;
    }
    __device__ __forceinline__ const void *dummy() const { return ql; }
};
template <> struct RowPtr<kTypeQ8_0> {
    const int8_t *qs;
    const uint16_t *d;
    uint32_t nb;
    __device__ __forceinline__ void set(const WeightView &w, int64_t row) {
        nb = (uint32_t)w.nb;
        qs = w.q8_qs + row * w.K;
        d = w.q8_d + row * w.nb;
    }
    __device__ __forceinline__ const void *dummy() const { return qs; }
};
template <> struct RowPtr<kTypeQ8_0Wide> : RowPtr<kTypeQ8_0> {};

// ------------------------------------------------------------------------------------------
template <int QT> struct Raw;
template <int QT> struct Frag;

template <> struct Raw<kTypeQ4_K> {
    uint32_t hd[4], q[8];
    // blk: block index inside the row (already clamped to the row), 32-bit
    // rel: row relative to rp (wave-uniform)
    __device__ __forceinline__ void load(const RowPtr<kTypeQ4_K> &rp, uint32_t blk, int lane, uint32_t rel = 0) {
        const uint32_t off = (rel * rp.nb + blk) * 144u;
        const uint32_t qoff = off + 16u + 32u * (uint32_t)(lane & 3);
        const uint4 h = *reinterpret_cast<const uint4 *>(rp.p + off);
        const uint4 v0 = *reinterpret_cast<const uint4 *>(rp.p + qoff);
        const uint4 v1 = *reinterpret_cast<const uint4 *>(rp.p + (qoff + 16u));
        hd[0] = h.x; hd[1] = h.y; hd[2] = h.z; hd[3] = h.w;
        q[0] = v0.x; q[1] = v0.y; q[2] = v0.z; q[3] = v0.w;
        q[4] = v1.x; q[5] = v1.y; q[6] = v1.z; q[7] = v1.w;
    }
    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int i = 0; i < 4; ++i) hd[i] = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = 0;
    }
};

template <> struct Frag<kTypeQ4_K> {
    uint32_t lo[8], hi[8];  // 32 low-nibble weights (sub-block 2c) and 32 high-nibble (2c+1)
    int sc0, sc1, m0, m1;
    float d, dmin;
    __device__ __forceinline__ void unpack(const Raw<kTypeQ4_K> &r, int lane) {
        const int c = lane & 3;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            lo[i] = r.q[i] & 0x0f0f0f0fu;
            hi[i] = (r.q[i] >> 4) & 0x0f0f0f0fu;
        }
        // (scale, min) of sub-blocks 2c and 2c+1: bytes 2(c&1), 2(c&1)+1 of the low or high word
        const ScalesK4 s = unpack_scales_k4(r.hd[1], r.hd[2], r.hd[3]);
        const uint32_t sw = c < 2 ? s.sc_lo : s.sc_hi;
        const uint32_t mw = c < 2 ? s.mn_lo : s.mn_hi;
        const int sh = 16 * (c & 1);
        sc0 = (int)((sw >> sh) & 0xffu);
        sc1 = (int)((sw >> (sh + 8)) & 0xffu);
        m0 = (int)((mw >> sh) & 0xffu);
        m1 = (int)((mw >> (sh + 8)) & 0xffu);
        d = h2f(r.hd[0]);
        dmin = h2f(r.hd[0] >> 16);
    }
};

template <> struct Raw<kTypeQ6_K> {
    uint4 a, b, h;  // ql run, ql run + 32, qh run
    uint2 s;        // the 8 scales of the lane's 128-half
    uint32_t d;
    __device__ __forceinline__ void load(const RowPtr<kTypeQ6_K> &rp, uint32_t blk_, int lane, uint32_t rel = 0) {
        const uint32_t i = lane & 3, hf = i >> 1, e = i & 1;
        const uint32_t blk = rel * rp.nb + blk_;
        a = *reinterpret_cast<const uint4 *>(rp.ql + (blk * 128u + 64u * hf + 16u * e));
        b = *reinterpret_cast<const uint4 *>(rp.ql + (blk * 128u + 64u * hf + 32u + 16u * e));
        h = *reinterpret_cast<const uint4 *>(rp.qh + (blk * 64u + 32u * hf + 16u * e));
        s = *reinterpret_cast<const uint2 *>(rp.sc + (blk * 16u + 8u * hf));
        d = rp.d[blk];
    }
    __device__ __forceinline__ void zero() { a = make_uint4(0, 0, 0, 0); b = a; h = a; s = make_uint2(0, 0); d = 0; }
};

template <> struct Frag<kTypeQ6_K> {
    uint32_t q[4][4];  // group g = weights 32g + 16e .. +16 of the 128-half, values 0..63
    int sc[4];
    float d;
    __device__ __forceinline__ void unpack(const Raw<kTypeQ6_K> &r, int lane) {
        const int e = lane & 1;
        const uint32_t a[4] = {r.a.x, r.a.y, r.a.z, r.a.w}, b[4] = {r.b.x, r.b.y, r.b.z, r.b.w},
                       h[4] = {r.h.x, r.h.y, r.h.z, r.h.w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            q[0][t] = (a[t] & 0x0f0f0f0fu) | ((h[t] << 4) & 0x30303030u);
            q[1][t] = (b[t] & 0x0f0f0f0fu) | ((h[t] << 2) & 0x30303030u);
            q[2][t] = ((a[t] >> 4) & 0x0f0f0f0fu) | (h[t] & 0x30303030u);
            q[3][t] = ((b[t] >> 4) & 0x0f0f0f0fu) | ((h[t] >> 2) & 0x30303030u);
        }
        const uint64_t s64 = (uint64_t)r.s.x | ((uint64_t)r.s.y << 32);
#pragma unroll
        for (int g = 0; g < 4; ++g) sc[g] = (int)(int8_t)(s64 >> (8 * (2 * g + e)));
        d = h2f(r.d);
    }
};

template <> struct Raw<kTypeQ8_0> {
    uint4 q;
    uint32_t d;
    __device__ __forceinline__ void load(const RowPtr<kTypeQ8_0> &rp, uint32_t blk_, int lane, uint32_t rel = 0) {
        const uint32_t blk = rel * rp.nb + blk_;
        q = *reinterpret_cast<const uint4 *>(rp.qs + (blk * 32u + 16u * (uint32_t)(lane & 1)));
        d = rp.d[blk];
    }
    __device__ __forceinline__ void zero() { q = make_uint4(0, 0, 0, 0); d = 0; }
};

template <> struct Frag<kTypeQ8_0> {
    uint32_t q[4];  // 16 int8 weights: half of a 32-block
    float d;
    __device__ __forceinline__ void unpack(const Raw<kTypeQ8_0> &r, int) {
        q[0] = r.q.x; q[1] = r.q.y; q[2] = r.q.z; q[3] = r.q.w;
        d = h2f(r.d);
    }
};

template <> struct Raw<kTypeQ8_0Wide> {
    uint4 q[4];
    uint32_t d[4];
    uint32_t live;   // bit j: part j's block lies inside the row (a short last chunk)
    __device__ __forceinline__ void load(const RowPtr<kTypeQ8_0Wide> &rp, uint32_t blk_, int lane, uint32_t rel = 0) {
        live = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t b = blk_ + 32u * j;
            if (b < rp.nb) live |= 1u << j;
            else b = rp.nb - 1;   // in bounds, never used
            const uint32_t blk = rel * rp.nb + b;
            q[j] = *reinterpret_cast<const uint4 *>(rp.qs + (blk * 32u + 16u * (uint32_t)(lane & 1)));
            d[j] = rp.d[blk];
        }
    }
    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int j = 0; j < 4; ++j) { q[j] = make_uint4(0, 0, 0, 0); d[j] = 0; }
        live = 0;
    }
};

template <> struct Frag<kTypeQ8_0Wide> {
    uint32_t q[16];
    float d[4];
    uint32_t live;
    __device__ __forceinline__ void unpack(const Raw<kTypeQ8_0Wide> &r, int) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            q[4 * j] = r.q[j].x; q[4 * j + 1] = r.q[j].y; q[4 * j + 2] = r.q[j].z; q[4 * j + 3] = r.q[j].w;
            d[j] = h2f(r.d[j]);
        }
        live = r.live;
    }
};

// ------------------------------------------------------------------------------------------
// LDS image of staged quantized activations: MT rows, `kt` bytes of K each.
struct XTile {
    const int8_t *qs;   // [MT][kt]
    const float *d;     // [MT][kt / blk]
    const int16_t *bs;  // [MT][kt / 16]  (Q8_K activations)
    int kt;
};

template <int QT> struct Dot;

template <> struct Dot<kTypeQ4_K> {
    uint32_t xl[8], xh[8];
    int bl, bh;  // sums of the 32 activations under sub-block 2c / 2c+1
    float xd;
    // c0: offset of the chunk inside the tile
    __device__ __forceinline__ void load_x(const XTile &x, int m, int c0, int lane) {
        const int sbl = lane >> 2, c = lane & 3;
        const int xo = c0 + sbl * 256 + 64 * c;
        const uint4 *p = reinterpret_cast<const uint4 *>(x.qs + m * x.kt + xo);
        const uint4 a0 = p[0], a1 = p[1], b0 = p[2], b1 = p[3];
        xl[0] = a0.x; xl[1] = a0.y; xl[2] = a0.z; xl[3] = a0.w;
        xl[4] = a1.x; xl[5] = a1.y; xl[6] = a1.z; xl[7] = a1.w;
        xh[0] = b0.x; xh[1] = b0.y; xh[2] = b0.z; xh[3] = b0.w;
        xh[4] = b1.x; xh[5] = b1.y; xh[6] = b1.z; xh[7] = b1.w;
        const int2 *bp = reinterpret_cast<const int2 *>(x.bs + m * (x.kt / 16) + (c0 + sbl * 256) / 16 + 4 * c);
        const int2 b = *bp;  // four int16 sums of 16
        bl = (int)(int16_t)(b.x & 0xffff) + (b.x >> 16);
        bh = (int)(int16_t)(b.y & 0xffff) + (b.y >> 16);
        xd = x.d[m * (x.kt / 256) + c0 / 256 + sbl];
    }
    __device__ __forceinline__ float dot(const Frag<kTypeQ4_K> &f) const {
        int sl = 0, sh = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            sl = dot4(f.lo[i], xl[i], sl);
            sh = dot4(f.hi[i], xh[i], sh);
        }
        // every factor fits 24 bits (6-bit scales and mins, sums of 32 products of a nibble and an int8):
        // the full-rate 24-bit multiply instead of the quarter-rate 32-bit one
        const int isum = __mul24(f.sc0, sl) + __mul24(f.sc1, sh);
        const int msum = __mul24(f.m0, bl) + __mul24(f.m1, bh);
        return fmaf(f.d * xd, (float)isum, -((f.dmin * xd) * (float)msum));
    }
};

template <> struct Dot<kTypeQ6_K> {
    uint32_t xg[4][4];
    int bs[4];
    float xd;
    __device__ __forceinline__ void load_x(const XTile &x, int m, int c0, int lane) {
        const int sbl = lane >> 2, i = lane & 3, hf = i >> 1, e = i & 1;
        const int xo = c0 + sbl * 256 + 128 * hf + 16 * e;
        const int bi = m * (x.kt / 16) + (c0 + sbl * 256) / 16 + 8 * hf + e;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const uint4 v = *reinterpret_cast<const uint4 *>(x.qs + m * x.kt + xo + 32 * g);
            xg[g][0] = v.x; xg[g][1] = v.y; xg[g][2] = v.z; xg[g][3] = v.w;
            bs[g] = x.bs[bi + 2 * g];
        }
        xd = x.d[m * (x.kt / 256) + c0 / 256 + sbl];
    }
    __device__ __forceinline__ float dot(const Frag<kTypeQ6_K> &f) const {
        int isum = 0;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            int s = 0;
#pragma unroll
            for (int t = 0; t < 4; ++t) s = dot4(f.q[g][t], xg[g][t], s);
            isum += __mul24(f.sc[g], s - 32 * bs[g]);  // weights are stored +32; both factors fit 24 bits
        }
        return (f.d * xd) * (float)isum;
    }
};

template <> struct Dot<kTypeQ8_0> {
    uint32_t xq[4];
    float xd;
    __device__ __forceinline__ void load_x(const XTile &x, int m, int c0, int lane) {
        const int xo = c0 + 16 * lane;
        const uint4 a = *reinterpret_cast<const uint4 *>(x.qs + m * x.kt + xo);
        xq[0] = a.x; xq[1] = a.y; xq[2] = a.z; xq[3] = a.w;
        xd = x.d[m * (x.kt / 32) + (c0 >> 5) + (lane >> 1)];
    }
    __device__ __forceinline__ float dot(const Frag<kTypeQ8_0> &f) const {
        int s = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) s = dot4(f.q[i], xq[i], s);
        return (float)s * (f.d * xd);
    }
};

template <> struct Dot<kTypeQ8_0Wide> {
    uint32_t xq[16];
    float xd[4];
    __device__ __forceinline__ void load_x(const XTile &x, int m, int c0, int lane) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int xo = c0 + 1024 * j + 16 * lane;
            const uint4 a = *reinterpret_cast<const uint4 *>(x.qs + m * x.kt + xo);
            xq[4 * j] = a.x; xq[4 * j + 1] = a.y; xq[4 * j + 2] = a.z; xq[4 * j + 3] = a.w;
            xd[j] = x.d[m * (x.kt / 32) + (c0 >> 5) + 32 * j + (lane >> 1)];
        }
    }
    // the parts are added in the order of K, as four steps of the narrow geometry would add them; a part past
    // the end of the row is left out by selection (its activation bytes were never staged)
    __device__ __forceinline__ float dot(const Frag<kTypeQ8_0Wide> &f) const {
        float t = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int s = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) s = dot4(f.q[4 * j + i], xq[4 * j + i], s);
            const float term = (float)s * (f.d[j] * xd[j]);
            t = j == 0 ? term : t + (((f.live >> j) & 1u) ? term : 0.f);
        }
        return t;
    }
};

}  // namespace qproj
