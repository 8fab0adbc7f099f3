// Prefill projection: Q4_K weights x per-32 int8 activations on the int8 matrix cores.
//
//   y[m][n] = sum_blk (d_n*sc_{n,blk}) * da_{m,blk} * I_{m,n,blk}  -  sum_blk (dmin_n*mn_{n,blk}) * (da_{m,blk}*isum_{m,blk})
//   I_{m,n,blk} = sum over the 32 weights of the sub-block of q * a      (exact, int32)
//
// A workgroup owns a 128 (tokens) x 128 (weight rows) tile; each of its 8 waves a 32x64
// sub-tile = two v_mfma_i32_32x32x32_i8 products per 32-wide sub-block.  Both operands change
// scale every 32 K-elements, so an int32 accumulator is meaningful for ONE product only: each
// product is folded into the fp32 accumulators right away (cvt, scale product, fma per output).
// That fp32 work, not the matrix cores, bounds this kernel, so everything else is kept off the
// vector ALU:
//   - the min term is a separate small GEMM over K/32 (activation block sums x mins) done on the
//     fp16 matrix cores before the main loop, with both operands split into fp16 high and low
//     parts (the mins are 17-bit products, split exactly; the sums keep 22 bits);
//   - the weight-side scales d*sc of a lane's own output column are unpacked from the block
//     header by that lane and held in registers for the 8 sub-blocks of a super-block;
//   - LDS holds only the two int8 operand tiles and the transposed activation scales, double
//     buffered over K-steps of 128 so that the global loads of step s+1 overlap step s.
#include <cstdlib>
#include <type_traits>
#include "qproj_device.h"
#include "qproj_internal.h"
#include "gemm_tiles.h"
#include "lds_direct.h"

namespace qproj {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int BM = 128, BN = 128, BK = 128;
constexpr int LDT = BK + 16;  // LDS row stride in bytes, padded against bank conflicts

struct GemmStage {
    int8_t a[BM * LDT];  // activations  [m][k]
    int8_t b[BN * LDT];  // weights      [n][k], nibbles expanded
    float a_d[4][BM];    // da           [sub-block][m]
};

struct GemmSmem {
    GemmStage st[2];
    float w_s[8][BN];  // d*sc of the 8 sub-blocks of the current super-block [n]
};

// registers one thread carries from global memory to LDS for one K-step
struct StageRegs {
    uint4 act[2];
    uint4 wq, wq2;   // wq2: Q8_0 only (its rows are 128 bytes per K-step, Q4_K's 64)
    float4 ad;  // threads 0..127: activation scales; threads 128..255: block header of a weight row
};

__device__ __forceinline__ void split_h(float v, _Float16 &hi, _Float16 &lo) {
    hi = (_Float16)v;
    lo = (_Float16)(v - (float)hi);
}

constexpr int kGemmThreads = 512;

// QT = Q4_K: per-32 int8 activations with fp32 scales and block sums (the prefill format).
// QT = Q8_0: ggml's Q8_0 activation blocks against Q8_0 weights: the same product without nibbles,
// without a min term, and with a weight scale per 32 instead of d*sc per sub-block.
// blockIdx.y selects one of gridDim.y equal stretches of K (whole super-blocks for Q4_K); with more than one
// the tile goes to part[blockIdx.y][M][N] and sum_parts_kernel adds the stretches up in order.
template <int QT>
__global__ __launch_bounds__(kGemmThreads, 4) void gemm_per32_kernel(const WeightView w, const ActView a, int64_t M,
                                                                   float *__restrict__ y, float *__restrict__ part) {
    constexpr bool kQ4 = QT == kTypeQ4_K;
    extern __shared__ __align__(16) uint8_t smem_raw[];
    GemmSmem &sm = *reinterpret_cast<GemmSmem *>(smem_raw);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;  // 4 x 2 waves
    const int64_t N = w.N, K = w.K;
    int tile_n, tile_m;
    tile_of_workgroup((int)((N + BN - 1) / BN), (int)((M + BM - 1) / BM), tile_n, tile_m);
    const int64_t n0 = (int64_t)tile_n * BN, m0 = (int64_t)tile_m * BM;
    const int64_t kb32 = K / 32;
    const int l32 = lane & 31, lh = lane >> 5;
    // this workgroup's stretch of K, in units of 256 (Q4_K super-blocks; two K-steps)
    const int64_t n_units = (K + 255) / 256, per = (n_units + gridDim.y - 1) / gridDim.y;
    const int64_t u_begin = min((int64_t)blockIdx.y * per, n_units), u_end = min(u_begin + per, n_units);
    if (gridDim.y > 1) y = part + (size_t)blockIdx.y * M * N;

    v16f acc[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

    // ---------------------------------------------------------------- min term on the fp16 cores
    // acc = -(1/prescale) * sum_kb A[m][kb] * B[n][kb] is built as +sum with negated B and scaled later.
    // The activation side (d * block sum, as fp16 high and low parts) comes ready from the quantizer.  The
    // weight side (-dmin * min of every sub-block, split the same way) is worked out once per workgroup,
    // 16 super-blocks at a time, into the LDS the main loop will use afterwards: two planes
    // [super-block][row][8 x fp16], so that every wave only reads operands and issues matrix instructions.
    if constexpr (kQ4) {
        constexpr int SBC = 16;                                   // super-blocks per pass (2 x 16 x 128 x 16 B = 64 KB)
        static_assert(2 * SBC * BN * 16 <= (int)sizeof(GemmSmem), "the min-term planes must fit the main loop's LDS");
        uint8_t *plane_hi = smem_raw, *plane_lo = smem_raw + SBC * BN * 16;
        const int64_t mrow = m0 + wm * 32 + l32 < M ? m0 + wm * 32 + l32 : M - 1;   // rows past M are never stored
        for (int64_t c0 = u_begin; c0 < u_end; c0 += SBC) {
            const int nsbc = (int)(u_end - c0 < SBC ? u_end - c0 : SBC);
            if (c0 > u_begin) __syncthreads();   // the previous pass has been read
            for (int base = 0; base < BN * nsbc; base += 4 * kGemmThreads) {
                v4i hd[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {   // four headers in flight per thread
                    const int item = min(base + u * kGemmThreads + tid, BN * nsbc - 1);
                    int64_t n = n0 + (item & (BN - 1));
                    if (n >= N) n = N - 1;
                    hd[u] = *reinterpret_cast<const v4i *>(w.q4k + (n * w.nb + c0 + (item >> 7)) * 144);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int item = base + u * kGemmThreads + tid;
                    if (item >= BN * nsbc) continue;
                    const ScalesK4 sc = unpack_scales_k4((uint32_t)hd[u][1], (uint32_t)hd[u][2], (uint32_t)hd[u][3]);
                    const float dmin = h2f((uint32_t)hd[u][0] >> 16);
                    v8h bh, bl;
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        _Float16 h, l;
                        split_h(-(dmin * (float)min_k4(sc, t)), h, l);
                        bh[t] = h;
                        bl[t] = l;
                    }
                    *reinterpret_cast<v8h *>(plane_hi + item * 16) = bh;   // item = super-block * 128 + row
                    *reinterpret_cast<v8h *>(plane_lo + item * 16) = bl;
                }
            }
            __syncthreads();
            const int n_steps = (nsbc + 1) / 2;   // 16 sub-blocks = two super-blocks per product
            v8h ah, al, ah_n, al_n;
            auto load_a = [&](v8h &h, v8h &l, int s) {
                int sbl = 2 * s + lh;
                if (sbl >= nsbc) sbl = nsbc - 1;   // past the end: any finite operand, the weight side is zero there
                const v8h *mp = reinterpret_cast<const v8h *>(a.msum + (mrow * w.nb + c0 + sbl) * 16);
                h = mp[0];
                l = mp[1];
            };
            load_a(ah, al, 0);
            for (int s = 0; s < n_steps; ++s) {
                load_a(ah_n, al_n, s + 1 < n_steps ? s + 1 : s);   // in flight during this step
                const int sbl = 2 * s + lh;
                const bool live = sbl < nsbc;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int o = ((live ? sbl : 0) * BN + wn * 64 + j * 32 + l32) * 16;
                    v8h bh = *reinterpret_cast<const v8h *>(plane_hi + o);
                    v8h bl = *reinterpret_cast<const v8h *>(plane_lo + o);
                    if (!live) {
#pragma unroll
                        for (int t = 0; t < 8; ++t) bh[t] = bl[t] = (_Float16)0.f;
                    }
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh, acc[j], 0, 0, 0);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bl, acc[j], 0, 0, 0);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, bh, acc[j], 0, 0, 0);
                }
                ah = ah_n;
                al = al_n;
            }
        }
        // the operand was normalised by the row (rs[m], a power of two) and pre-scaled by 1/16: both undone exactly
        __syncthreads();   // the planes have been read
        float *rs_tile = reinterpret_cast<float *>(smem_raw);   // the tile's 128 row normalisers, times 16
        if (tid < BM) rs_tile[tid] = a.rs[m0 + tid < M ? m0 + tid : M - 1] * (1.0f / kMinPrescale);
        __syncthreads();
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float4 f = *reinterpret_cast<const float4 *>(rs_tile + wm * 32 + 8 * g + 4 * lh);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                acc[j][4 * g] *= f.x; acc[j][4 * g + 1] *= f.y; acc[j][4 * g + 2] *= f.z; acc[j][4 * g + 3] *= f.w;
            }
        }
        __syncthreads();   // the main loop may overwrite the tile
    }

    // ---------------------------------------------------------------- main loop, int8 cores
    // Addresses: a scalar base per operand plus a 32-bit lane offset that never changes; the K position is added
    // to the scalar side.  (64-bit pointers per lane cost the registers this kernel does not have.)  Rows past the
    // end of a tile read the last valid row: their results are never stored.
    const int mrow_cap = (int)(M - 1 - m0 < BM - 1 ? M - 1 - m0 : BM - 1);
    const int nrow_cap = (int)(N - 1 - n0 < BN - 1 ? N - 1 - n0 : BN - 1);
    const global_ptr<int8_t> abase_s = scalar_global(a.qs + m0 * K);
    const global_ptr<float> adbase_s = scalar_global(a.d + m0 * kb32);
    uint32_t aoffg[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int idx = tid + kGemmThreads * i, row = idx >> 3, seg = idx & 7;
        aoffg[i] = (uint32_t)(row < mrow_cap ? row : mrow_cap) * (uint32_t)K + 16u * seg;
    }
    const uint32_t wrow = (uint32_t)((tid >> 2) < nrow_cap ? (tid >> 2) : nrow_cap);
    const uint32_t hrow = (uint32_t)(tid - BM < 0 ? 0 : (tid - BM < nrow_cap ? tid - BM : nrow_cap));
    const uint32_t adoffg = (uint32_t)(tid < mrow_cap ? tid : mrow_cap) * (uint32_t)kb32;
    global_ptr<uint8_t> wbase_s = nullptr;
    global_ptr<int8_t> w8base_s = nullptr;
    global_ptr<uint16_t> w8d_s = nullptr;
    uint32_t woffg, hoffg;
    if constexpr (kQ4) {
        wbase_s = scalar_global(w.q4k + n0 * w.nb * 144);
        woffg = wrow * (uint32_t)w.nb * 144u + 16u + 16u * (tid & 3);
        hoffg = hrow * (uint32_t)w.nb * 144u;
    } else {
        w8base_s = scalar_global(w.q8_qs + n0 * K);
        w8d_s = scalar_global(w.q8_d + n0 * w.nb);
        woffg = wrow * (uint32_t)K + 32u * (tid & 3);
        hoffg = hrow * (uint32_t)w.nb;
    }
    auto load_stage = [&](StageRegs &r, int64_t k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i)   // activations: 128 rows x 128 B
            r.act[i] = load_global<uint4>(abase_s + k0, aoffg[i]);
        if constexpr (kQ4) {  // weights: 128 rows x 64 packed bytes (two 64-weight chunks of the super-block)
            const int c2 = (int)((k0 & 255) >> 5);  // 32-byte chunk pair index * 2
            r.wq = load_global<uint4>(wbase_s + ((k0 >> 8) * 144 + 16 * c2), woffg);
        } else {              // weights: 128 rows x 128 int8
            r.wq = load_global<uint4>(w8base_s + k0, woffg);
            r.wq2 = load_global<uint4>(w8base_s + k0 + 16, woffg);
        }
        r.ad = make_float4(0.f, 0.f, 0.f, 0.f);
        if (tid < BM) {
            r.ad = load_global<float4>(adbase_s + (k0 >> 5), 4u * adoffg);
        } else if (tid < BM + BN && (!kQ4 || (k0 & 255) == 0)) {
            if constexpr (kQ4) {   // a new super-block starts: its header
                r.ad = load_global<float4>(wbase_s + (k0 >> 8) * 144, hoffg);
            } else {               // the four fp16 scales of this K-step
                const uint2 d4 = load_global<uint2>(w8d_s + (k0 >> 5), 2u * hoffg);
                r.ad.x = __uint_as_float(d4.x);
                r.ad.y = __uint_as_float(d4.y);
            }
        }
    };
    auto store_stage = [&](const StageRegs &r, GemmStage &st, int64_t k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = tid + kGemmThreads * i;
            const int row = idx >> 3, seg = idx & 7;
            *reinterpret_cast<uint4 *>(st.a + row * LDT + 16 * seg) = r.act[i];
        }
        if constexpr (!kQ4) {
            const int row = tid >> 2, part = tid & 3;
            *reinterpret_cast<uint4 *>(st.b + row * LDT + 32 * part) = r.wq;
            *reinterpret_cast<uint4 *>(st.b + row * LDT + 32 * part + 16) = r.wq2;
        } else {
            // 16 packed bytes = bytes 16*(part&1).. of chunk (part>>1): low nibbles -> sub-block 2c, high -> 2c+1
            const int row = tid >> 2, part = tid & 3, ch = part >> 1, half = part & 1;
            int8_t *base = st.b + row * LDT + 64 * ch + 16 * half;
            *reinterpret_cast<uint4 *>(base) = make_uint4(r.wq.x & 0x0f0f0f0fu, r.wq.y & 0x0f0f0f0fu, r.wq.z & 0x0f0f0f0fu, r.wq.w & 0x0f0f0f0fu);
            *reinterpret_cast<uint4 *>(base + 32) = make_uint4((r.wq.x >> 4) & 0x0f0f0f0fu, (r.wq.y >> 4) & 0x0f0f0f0fu,
                                                               (r.wq.z >> 4) & 0x0f0f0f0fu, (r.wq.w >> 4) & 0x0f0f0f0fu);
        }
        if (tid < BM) {
            st.a_d[0][tid] = r.ad.x;
            st.a_d[1][tid] = r.ad.y;
            st.a_d[2][tid] = r.ad.z;
            st.a_d[3][tid] = r.ad.w;
        } else if (tid < BM + BN && (!kQ4 || (k0 & 255) == 0)) {
            if constexpr (kQ4) {
                const uint32_t h0 = __float_as_uint(r.ad.x);
                const ScalesK4 sc = unpack_scales_k4(__float_as_uint(r.ad.y), __float_as_uint(r.ad.z), __float_as_uint(r.ad.w));
                const float d = h2f(h0);
                float *dst = &sm.w_s[0][tid - BM];
#pragma unroll
                for (int t = 0; t < 8; ++t) dst[t * BN] = d * (float)scale_k4(sc, t);
            } else {   // scale slots 0..3 and 4..7 alternate with the K-steps, like the operand stages
                const uint32_t lo = __float_as_uint(r.ad.x), hi = __float_as_uint(r.ad.y);
                float *dst = &sm.w_s[(int)((k0 / BK) & 1) * 4][tid - BM];
                dst[0] = h2f(lo & 0xffffu);
                dst[BN] = h2f(lo >> 16);
                dst[2 * BN] = h2f(hi & 0xffffu);
                dst[3 * BN] = h2f(hi >> 16);
            }
        }
    };

    const int64_t ks_begin = u_begin * 2, n_ksteps = min(u_end * 2, K / BK);
    StageRegs regs;
    if (ks_begin < n_ksteps) {
        load_stage(regs, ks_begin * BK);
        store_stage(regs, sm.st[ks_begin & 1], ks_begin * BK);
    }
    __syncthreads();

    for (int64_t ks = ks_begin; ks < n_ksteps; ++ks) {
        const int64_t k0 = ks * BK;
        const GemmStage &st = sm.st[ks & 1];
        if (ks + 1 < n_ksteps) load_stage(regs, k0 + BK);  // in flight during the arithmetic below
        const float *wsp = &sm.w_s[kQ4 ? (int)((k0 & 255) >> 5) : (int)(ks & 1) * 4][wn * 64 + l32];
#pragma unroll 1
        for (int kb = 0; kb < 4; ++kb) {
            const v4i af = *reinterpret_cast<const v4i *>(st.a + (wm * 32 + l32) * LDT + kb * 32 + 16 * lh);
            v4i bf[2];
#pragma unroll
            for (int j = 0; j < 2; ++j)
                bf[j] = *reinterpret_cast<const v4i *>(st.b + (wn * 64 + j * 32 + l32) * LDT + kb * 32 + 16 * lh);
            const float w0 = wsp[kb * BN], w1 = wsp[kb * BN + 32];
            float ad[16];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 d4 = *reinterpret_cast<const float4 *>(&st.a_d[kb][wm * 32 + 8 * g + 4 * lh]);
                ad[4 * g + 0] = d4.x; ad[4 * g + 1] = d4.y; ad[4 * g + 2] = d4.z; ad[4 * g + 3] = d4.w;
            }
            const v16i z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const v16i I0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bf[0], z, 0, 0, 0);
            const v16i I1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bf[1], z, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[0][v] = fmaf((float)I0[v], ad[v] * w0, acc[0][v]);
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[1][v] = fmaf((float)I1[v], ad[v] * w1, acc[1][v]);
        }
        // the next step starts a new super-block: its scales replace the ones other waves may still read
        if (kQ4 && ((k0 + BK) & 255) == 0) __syncthreads();
        if (ks + 1 < n_ksteps) store_stage(regs, sm.st[(ks + 1) & 1], k0 + BK);
        __syncthreads();
    }

    // ---- store: accumulator register v of lane l is row 8*(v/4) + 4*(l/32) + v%4, column l%32
    // (the lane's coordinates are worked out again from the thread index, made opaque so that nothing of the
    // address arithmetic is carried through the main loop in registers the loop needs)
    int tid_s = tid;
    asm volatile("" : "+v"(tid_s));
    const int l32_s = tid_s & 31, lh_s = (tid_s >> 5) & 1, wm_s = tid_s >> 7, wn_s = (tid_s >> 6) & 1;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int64_t n = n0 + wn_s * 64 + j * 32 + l32_s;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int64_t m = m0 + wm_s * 32 + 8 * (v >> 2) + 4 * lh_s + (v & 3);
            if (m < M && n < N) y[m * N + n] = acc[j][v];
        }
    }
}

// ------------------------------------------------------------------------------------------------
// ggml activation format (Q8_K: one scale per 256) x Q4_K on the int8 matrix cores.
//
// With a single activation scale per super-block the integer sums of its eight sub-blocks may be
// added before anything turns into floating point; only the 6-bit sub-block scale sc stands in the
// way, and sc*q (up to 945) does not fit an int8 operand.  Written in base 8, sc = 8*sc_hi + sc_lo,
// both products sc_lo*q and sc_hi*q stay below 106: two int8 weight operands and two accumulation
// chains over the whole super-block run entirely inside the matrix cores,
//     I_lo = sum_k (sc_lo*q) * a,   I_hi = sum_k (sc_hi*q) * a,   sum_k sc*q*a = 8*I_hi + I_lo,
// so the vector ALU only works once per 256 weights (shift-add, int->float, one fma with dx*d).
// Twice the matrix instructions of the per-32 kernel, a third of its vector instructions.
typedef unsigned short v2us __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_mul_u16(uint32_t x, uint32_t s2) {
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(v2us, x) * __builtin_bit_cast(v2us, s2));
}

// The weights never become an LDS tile: they are converted in registers.  Inside a super-block
// the order of the 256 products is free (both chains run over all of it), so a lane may feed the matrix
// instruction with whichever 16 weights it likes as long as the activation operand carries the
// matching 16: lane (row l%32, half l/32) takes the 64 contiguous nibble bytes [64*half, 64*half+64)
// of its own weight row = sub-blocks 4*half .. 4*half+3, expands and scales them in registers, and
// reads the activations of exactly those sub-blocks from LDS.  Each of the NW waves owns 32 weight
// rows of the tile and all of its 64 tokens.
//
// Memory side: a lane-per-row load touches 64 cache lines per instruction and the vector memory
// pipeline, not the arithmetic, becomes the limit.  So every wave fetches its 32 raw 144-byte blocks
// with consecutive lanes on consecutive 16-byte pieces (288 pieces, five loads), parks them in a
// wave-private LDS strip exactly as they lie in memory (a row stride of 144 bytes is conflict-free
// for 16-byte reads) and picks its row's header and nibbles out of the strip.  The min term rides
// along: the activation quantizer has already written d*(sub-block sum)/16 as fp16 pairs, the tile
// of those is staged with the activations, and two fp16 matrix instructions per super-block and
// token tile (operand [high | low] against [-dmin*min high | same], then [high | low] against
// [-dmin*min low | 0]) add it to the accumulators, which therefore run in units of 1/16 until the
// final store.  One workgroup barrier per 256 weights.
constexpr int DLA = 256 + 16;   // LDS row stride of the activation tile in bytes

template <int NW>
struct DirectSmem {
    int8_t a[2][64 * DLA];           // activations of one super-block [token][256 + pad]
    uint16_t ms[2][64 * 16];         // min-term operand [token][8 high | 8 low] (fp16 bits)
    float dx[2][64];                 // activation scale of the super-block
    uint8_t park[NW][32 * 144];      // per wave: the raw blocks of its 32 weight rows
};

struct DirectB {     // one super-block of the lane's weight row
    v4i hdr;         // d, dmin, 12 bytes of 6-bit scales and mins
    v4i q[4];        // 64 nibble bytes: q[2*gg + half] = bytes 16*half.. of the 32-byte group 2*(l/32) + gg
};

__device__ __forceinline__ uint32_t byte_to_u16x2(uint32_t word, int i) {
    // byte i of word -> both 16-bit halves (v_perm_b32: selector 0x0c yields a zero byte)
    return __builtin_amdgcn_perm(0u, word, 0x0c000c00u | (uint32_t)(i << 16) | (uint32_t)i);
}

// Up to three matrices that multiply the same activation rows (q/k/v, gate/up) ride in one launch: a matrix of
// 1024 rows against 512 tokens is 64 tiles, an eighth of the workgroups the chip holds, and took as long alone
// as the 4096-row one beside it.  Each matrix owns a run of workgroups that starts at a multiple of 8.
struct DirectTargets {
    int n;
    WeightView w[3];
    float *y[3];
    int first_wg[3];
};

template <int NW>
__global__ __launch_bounds__(64 * NW, 2) void gemm_q4k_q8k_direct_kernel(const DirectTargets tg, const ActView a, int64_t M,
                                                                        float *__restrict__ part) {
    constexpr int NT = 64 * NW, TN = 32 * NW;
    constexpr int PA = 1024 / NT;   // 16-byte activation pieces a thread moves per super-block
    extern __shared__ __align__(16) uint8_t smem_raw[];
    DirectSmem<NW> &sm = *reinterpret_cast<DirectSmem<NW> *>(smem_raw);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    WeightView w = tg.w[0];
    float *__restrict__ y = tg.y[0];
    int first_wg = 0;
#pragma unroll
    for (int i = 1; i < 3; ++i)
        if (i < tg.n && (int)blockIdx.x >= tg.first_wg[i]) {
            w = tg.w[i];
            y = tg.y[i];
            first_wg = tg.first_wg[i];
        }
    const int64_t N = w.N, K = w.K, nb = w.nb;
    int tile_n, tile_m;
    {
        const int tiles_n = (int)((N + TN - 1) / TN), tiles_m = (int)((M + 63) / 64), pid = (int)blockIdx.x - first_wg;
        if (pid >= tiles_n * tiles_m) return;   // padding between two matrices: the whole workgroup leaves
        tile_of_workgroup(tiles_n, tiles_m, pid, tile_n, tile_m);
    }
    const int64_t n0 = (int64_t)tile_n * TN, m0 = (int64_t)tile_m * 64;
    const int l32 = lane & 31, lh = lane >> 5;

    v16f acc[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

    // ---- global -> register -> LDS plumbing.  Every address is a wave-uniform base plus a 32-bit
    // lane offset; rows past the edge of the matrix repeat the last valid row (never stored).
    // weights: piece p = lane + 64*c of the wave's 288 -> row p / 9, 16-byte part p % 9
    const int64_t wave_row0 = n0 + wave * 32 < N ? n0 + wave * 32 : N - 1;
    const int wrow_cap = (int)(N - 1 - wave_row0 < 31 ? N - 1 - wave_row0 : 31);
    const uint8_t *wbase = w.q4k + wave_row0 * nb * 144;
    uint32_t woff[5];
    int wpark[5];
#pragma unroll
    for (int c = 0; c < 5; ++c) {
        const int p = lane + 64 * c < 287 ? lane + 64 * c : 287;
        const int r = p / 9 < wrow_cap ? p / 9 : wrow_cap;
        woff[c] = (uint32_t)(r * (int)nb * 144 + 16 * (p % 9));
        wpark[c] = 16 * p;
    }
    // activations: piece id = tid + NT*p -> token id / 16, 16-byte segment id % 16
    const int mrow_cap = (int)(M - 1 - m0 < 63 ? M - 1 - m0 : 63);
    const int8_t *abase = a.qs + m0 * K;
    uint32_t aoffg[PA];
    int aoffl[PA];
#pragma unroll
    for (int p = 0; p < PA; ++p) {
        const int id = tid + NT * p, row = id >> 4, seg = id & 15;
        aoffg[p] = (uint32_t)((row < mrow_cap ? row : mrow_cap) * (int)K + 16 * seg);
        aoffl[p] = row * DLA + 16 * seg;
    }
    // min-term operand: 64 tokens x 32 bytes, thread t (mod 128) moves 16 bytes; scale: thread t (mod 64)
    const uint8_t *msbase = reinterpret_cast<const uint8_t *>(a.msum) + m0 * nb * 32;
    const int msrow = (tid & 127) >> 1;
    const uint32_t msoffg = (uint32_t)((msrow < mrow_cap ? msrow : mrow_cap) * (int)nb * 32 + 16 * (tid & 1));
    const float *dxbase = a.d + m0 * nb;
    const uint32_t dxoffg = (uint32_t)(((tid & 63) < mrow_cap ? (tid & 63) : mrow_cap) * (int)nb);
    // the min-term operand is normalised by the row (rs[m], a power of two): the accumulators run in units of
    // 1 / (16 * rs[m]) until the store, so the activation scales are divided by rs[m] as they are staged (exact)
    const float rs_mine = a.rs[m0 + ((tid & 63) < mrow_cap ? (tid & 63) : mrow_cap)];
    const float inv_rs = 1.0f / rs_mine;

    v4i stg[5], areg[PA], msreg;
    float dxreg;
    auto load_next = [&](int64_t sb) {   // activations first: they are wanted at the end of this trip already
#pragma unroll
        for (int p = 0; p < PA; ++p) areg[p] = *reinterpret_cast<const v4i *>(abase + sb * 256 + aoffg[p]);
        msreg = *reinterpret_cast<const v4i *>(msbase + sb * 32 + msoffg);
        dxreg = dxbase[sb + dxoffg];
#pragma unroll
        for (int c = 0; c < 5; ++c) stg[c] = *reinterpret_cast<const v4i *>(wbase + sb * 144 + woff[c]);
    };
    uint8_t *park = sm.park[wave];
    auto store_next = [&](int buf) {
#pragma unroll
        for (int p = 0; p < PA; ++p) *reinterpret_cast<v4i *>(sm.a[buf] + aoffl[p]) = areg[p];
        // threads beyond the first 128 / 64 repeat a store of the same value: no branch, no load sunk into one
        *reinterpret_cast<v4i *>(reinterpret_cast<uint8_t *>(sm.ms[buf]) + 16 * (tid & 127)) = msreg;
        sm.dx[buf][tid & 63] = dxreg * inv_rs;   // (here, not at the load: nothing waits for the load before it must)
#pragma unroll
        for (int c = 0; c < 5; ++c) *reinterpret_cast<v4i *>(park + wpark[c]) = stg[c];
    };

    const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    auto superblock = [&](const DirectB &b, int buf) {
        const ScalesK4 sc = unpack_scales_k4((uint32_t)b.hdr[1], (uint32_t)b.hdr[2], (uint32_t)b.hdr[3]);
        // ---- min term: -dmin*min of the 8 sub-blocks as fp16 high and low parts
        {
            const float ndmin = -h2f((uint32_t)b.hdr[0] >> 16);
            v8h bh, bl;
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                _Float16 h, l;
                split_h(ndmin * (float)min_k4(sc, t), h, l);
                bh[t] = h;
                bl[t] = lh ? (_Float16)0.f : l;
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const v8h am = *reinterpret_cast<const v8h *>(reinterpret_cast<const uint8_t *>(sm.ms[buf]) +
                                                             (j * 32 + l32) * 32 + 16 * lh);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(am, bh, acc[j], 0, 0, 0);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(am, bl, acc[j], 0, 0, 0);
            }
        }
        // ---- the lane's four sub-block scales, split in base 8 and spread over both 16-bit halves
        const uint32_t scw = lh ? sc.sc_hi : sc.sc_lo;
        const uint32_t lo_w = scw & 0x07070707u, hi_w = (scw >> 3) & 0x07070707u;
        const int8_t *ap = sm.a[buf] + l32 * DLA + 128 * lh;
        v16i ilo[2], ihi[2];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const int gg = t >> 2, nib = (t >> 1) & 1, half = t & 1, i = 2 * gg + nib;
            const uint32_t sl = byte_to_u16x2(lo_w, i), sh = byte_to_u16x2(hi_w, i);
            const v4i raw = b.q[2 * gg + half];
            v4i bl, bh;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t x = nib ? ((uint32_t)raw[c] >> 4) & 0x0f0f0f0fu : (uint32_t)raw[c] & 0x0f0f0f0fu;
                bl[c] = (int)pk_mul_u16(x, sl);
                bh[c] = (int)pk_mul_u16(x, sh);
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const v4i af = *reinterpret_cast<const v4i *>(ap + j * 32 * DLA + 32 * i + 16 * half);
                ilo[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bl, t == 0 ? zi : ilo[j], 0, 0, 0);
                ihi[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bh, t == 0 ? zi : ihi[j], 0, 0, 0);
            }
        }
        const float dn = h2f((uint32_t)b.hdr[0] & 0xffffu) * kMinPrescale;   // exact: a power of two
        const float *dxs = sm.dx[buf];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            float dxv[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 d4 = *reinterpret_cast<const float4 *>(dxs + j * 32 + 8 * i + 4 * lh);
                dxv[4 * i] = d4.x; dxv[4 * i + 1] = d4.y; dxv[4 * i + 2] = d4.z; dxv[4 * i + 3] = d4.w;
            }
#pragma unroll
            for (int v = 0; v < 16; ++v)
                acc[j][v] = fmaf((float)((ihi[j][v] << 3) + ilo[j][v]), dxv[v] * dn, acc[j][v]);
        }
    };

    // a grid with gridDim.y > 1 cuts K: this workgroup does the super-blocks [sb_begin, sb_end) and writes a
    // partial tile that sum_parts_kernel adds to the others in order
    const int64_t sb_begin = nb * blockIdx.y / gridDim.y, sb_end = nb * (blockIdx.y + 1) / gridDim.y;
    load_next(sb_begin);
    store_next((int)(sb_begin & 1));
    __syncthreads();
    for (int64_t sb = sb_begin; sb < sb_end; ++sb) {
        const int buf = (int)(sb & 1);
        DirectB b;   // out of the strip: header of row l%32, then the lane's 64 nibble bytes
        b.hdr = *reinterpret_cast<const v4i *>(park + l32 * 144);
#pragma unroll
        for (int i = 0; i < 4; ++i) b.q[i] = *reinterpret_cast<const v4i *>(park + l32 * 144 + 16 + 64 * lh + 16 * i);
        // past the end the last super-block is fetched again: unconditional loads keep the wait counters exact
        load_next(sb + 1 < sb_end ? sb + 1 : sb_end - 1);
        __builtin_amdgcn_sched_barrier(0);   // the loads stay ahead of the arithmetic they overlap with
        superblock(b, buf);
        store_next(buf ^ 1);
        __syncthreads();
    }

    // ---- store: accumulator register v of lane l is row 8*(v/4) + 4*(l/32) + v%4, column l%32
    const int64_t n = n0 + wave * 32 + l32;
    // the rows' factors (normaliser / 16) go through the idle scale buffer: four rows per read, no load per store
    sm.dx[0][tid & 63] = rs_mine * (1.0f / kMinPrescale);
    __syncthreads();
    // two stretches and no scratch: the output rows were cleared before the launch and both stretches add their
    // tile to them (0 + a + b is a + b in either order, so the result does not depend on which arrives first)
    const bool add = gridDim.y > 1 && part == nullptr;
    float *out = gridDim.y > 1 && !add ? part + (size_t)blockIdx.y * M * N : y;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float4 f4 = *reinterpret_cast<const float4 *>(&sm.dx[0][j * 32 + 8 * g + 4 * lh]);
            const float f[4] = {f4.x, f4.y, f4.z, f4.w};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t m = m0 + j * 32 + 8 * g + 4 * lh + r;
                if (m < M && n < N) {
                    if (add) unsafeAtomicAdd(out + m * N + n, acc[j][4 * g + r] * f[r]);
                    else out[m * N + n] = acc[j][4 * g + r] * f[r];
                }
            }
        }
    }
}


// ------------------------------------------------------------------------------------------------
// The same product for large batches: every wave keeps its 32 weight rows but works on 128 tokens.
//
// The kernel above spends four vector instructions per matrix instruction on expanding and scaling
// weights, because a converted weight fragment feeds only two token tiles.  Here a wave converts the
// whole super-block of its 32 rows once into 64 registers (both chains, all eight steps) and then
// walks four token tiles with them, so the conversion is paid once per 128 tokens.  Eight waves =
// 256 weight rows x 128 tokens per workgroup, one workgroup per compute unit.
//
// Nothing passes through staging registers: activations, the min-term tile, the activation scales
// and the raw weight blocks go from global memory straight into LDS (global_load_lds, 16 bytes a
// lane, a wave writes one contiguous kilobyte per instruction).  Because such a load cannot pad LDS
// rows, the activation tile is stored [token][256] with the 16-byte segments of a row XOR-swizzled
// by the token index: slot s of token r holds segment s ^ (r & 15), which the loading lane simply
// requests from global memory, and 16 consecutive tokens reading "their" segment g hit 16 different
// slots.
template <int NW>
struct WideSmem {
    int8_t a[2][128 * 256];          // activations of one super-block [token][16 swizzled segments]
    uint16_t ms[2][128 * 16];        // min-term operand [token][8 high | 8 low] (fp16 bits)
    float dx[2][128];                // activation scale of the super-block
    uint8_t park[NW][5 * 1024];      // per wave: raw blocks of its 32 weight rows (4608 bytes used)
};

template <int NW>
__global__ __launch_bounds__(64 * NW, 1) void gemm_q4k_q8k_wide_kernel(const WeightView w, const ActView a, int64_t M,
                                                                      float *__restrict__ y, float *__restrict__ part) {
    static_assert(NW == 8, "the loading roles below are laid out for eight waves");
    constexpr int TM = 128, TN = 32 * NW, JT = TM / 32;
    constexpr int PA = (TM * 16) / (64 * NW);   // 1-KB activation chunks (4 tokens) a wave requests per super-block
    extern __shared__ __align__(16) uint8_t smem_raw[];
    WideSmem<NW> &sm = *reinterpret_cast<WideSmem<NW> *>(smem_raw);
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

    // ---- global -> LDS requests: wave-uniform bases plus 32-bit lane offsets; rows past the edge of
    // a matrix repeat its last valid row (computed, never stored)
    const int64_t wave_row0 = n0 + wave * 32 < N ? n0 + wave * 32 : N - 1;
    const int wrow_cap = (int)(N - 1 - wave_row0 < 31 ? N - 1 - wave_row0 : 31);
    const uint8_t *wbase = w.q4k + wave_row0 * nb * 144;
    uint32_t woff[5];   // piece p = lane + 64*c of the wave's 288 -> row p / 9, 16-byte part p % 9
#pragma unroll
    for (int c = 0; c < 5; ++c) {
        const int p = lane + 64 * c < 287 ? lane + 64 * c : 287;
        const int r = p / 9 < wrow_cap ? p / 9 : wrow_cap;
        woff[c] = (uint32_t)(r * (int)nb * 144 + 16 * (p % 9));
    }
    const int mrow_cap = (int)(M - 1 - m0 < TM - 1 ? M - 1 - m0 : TM - 1);
    const int8_t *abase = a.qs + m0 * K;
    uint32_t aoffg[PA];   // chunk wave + NW*p = tokens 4*chunk .. +3; lane -> token lane/16, slot lane%16
#pragma unroll
    for (int p = 0; p < PA; ++p) {
        const int row = 4 * (wave + NW * p) + (lane >> 4), seg = (lane & 15) ^ (row & 15);
        aoffg[p] = (uint32_t)((row < mrow_cap ? row : mrow_cap) * (int)K + 16 * seg);
    }
    // waves 0..3: min-term tile (2 pieces a token); waves 4, 5: activation scales (one float a token)
    const uint8_t *msbase = reinterpret_cast<const uint8_t *>(a.msum) + m0 * nb * 32;
    const int mstok = (wave & 3) * 32 + (lane >> 1), dxtok = tid & 127;
    const uint32_t msoffg = (uint32_t)((mstok < mrow_cap ? mstok : mrow_cap) * (int)nb * 32 + 16 * (lane & 1));
    const float *dxbase = a.d + m0 * nb;
    const uint32_t dxoffg = (uint32_t)((dxtok < mrow_cap ? dxtok : mrow_cap) * (int)nb);
    // the min-term operand is normalised by the row (rs[m], a power of two): the accumulators run in units of
    // 1 / (16 * rs[m]) until the store, so the activation scales are divided by rs[m] as they are staged (exact)
    const float rs_mine = a.rs[m0 + (dxtok < mrow_cap ? dxtok : mrow_cap)];
    const float inv_rs = 1.0f / rs_mine;
    uint8_t *park = sm.park[wave];

    // Addresses are a scalar base that never moves plus a 32-bit lane offset to which the super-block's
    // displacement is added on the spot: one vector register per request stays live, not a 64-bit pointer.
    const uint8_t *wbase_s = scalar_pointer(wbase);
    const int8_t *abase_s = scalar_pointer(abase);
    const uint8_t *msbase_s = scalar_pointer(msbase);
    const global_ptr<float> dxbase_s = scalar_global(dxbase);
    auto request_strip = [&](uint32_t sb, int c) {
        global_to_lds16(wbase_s + (woff[c] + sb * 144u), park + 1024 * c);
    };
    auto request_act = [&](uint32_t sb, int buf, int p) {
        global_to_lds16(abase_s + (aoffg[p] + sb * 256u), sm.a[buf] + (wave + NW * p) * 1024);
    };
    auto request_ms = [&](uint32_t sb, int buf) {
        if (wave < 4) global_to_lds16(msbase_s + (msoffg + sb * 32u), reinterpret_cast<uint8_t *>(sm.ms[buf]) + wave * 1024);
    };

    // the lane's eight activation reads of a token tile: segment t + 8*(l/32) of token l%32 (+32*j) sits in
    // slot (t + 8*(l/32)) ^ (l%16) = t ^ z with z = 8*(l/32) ^ (l%16), i.e. at byte (256*(l%32) + 16*z) ^ 16*t
    const int aoffl = l32 * 256 + 16 * ((8 * lh) ^ (l32 & 15));
    const v16i zi = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    // both scaled int8 copies of the lane's 128 weights (step t = sub-block 4*(l/32) + t/2, half t%2) and the header
    v4i hdr, cl[8], ch[8];
    uint32_t lo_w, hi_w;   // base-8 digits of the lane's four sub-block scales
    auto read_header = [&]() {
        hdr = *reinterpret_cast<const v4i *>(park + l32 * 144);
        const ScalesK4 sc = unpack_scales_k4((uint32_t)hdr[1], (uint32_t)hdr[2], (uint32_t)hdr[3]);
        const uint32_t scw = lh ? sc.sc_hi : sc.sc_lo;
        lo_w = scw & 0x07070707u;
        hi_w = (scw >> 3) & 0x07070707u;
    };
    auto strip_piece = [&](int t) {   // nibble bytes of step t: 16-byte piece 2*(t/4) + t%2 of the lane's 64
        return *reinterpret_cast<const v4i *>(park + l32 * 144 + 16 + 64 * lh + 16 * (2 * (t >> 2) + (t & 1)));
    };
    auto convert = [&](int t, const v4i &raw) {
        const int i = t >> 1, nib = i & 1;
        const uint32_t sl = byte_to_u16x2(lo_w, i), sh = byte_to_u16x2(hi_w, i);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t x = nib ? ((uint32_t)raw[c] >> 4) & 0x0f0f0f0fu : (uint32_t)raw[c] & 0x0f0f0f0fu;
            cl[t][c] = (int)pk_mul_u16(x, sl);
            ch[t][c] = (int)pk_mul_u16(x, sh);
        }
    };

    // a grid with gridDim.y > 1 cuts K: this workgroup does the super-blocks [sb_begin, sb_end) and writes a
    // partial tile that sum_parts_kernel adds to the others in order
    const int64_t sb_begin = nb * blockIdx.y / gridDim.y, sb_end = nb * (blockIdx.y + 1) / gridDim.y;
    // ---- prologue: requests of the first super-block
#pragma unroll
    for (int c = 0; c < 5; ++c) request_strip((uint32_t)sb_begin, c);
#pragma unroll
    for (int p = 0; p < PA; ++p) request_act((uint32_t)sb_begin, 0, p);
    request_ms((uint32_t)sb_begin, 0);
    sm.dx[0][tid & 127] = dxbase_s[dxoffg + (uint32_t)sb_begin] * inv_rs;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // The two waves that share a SIMD (w and w+4) must not want the same pipe at the same time: the older one
    // wins every arbitration and the younger one only gets what is left.  So they run the same super-block in
    // opposite orders.  EARLY waves (0..3) convert the weights of a super-block at its start (vector work first,
    // the conversion of step t+1 sits between the matrix instructions of step t of the first tile); LATE waves
    // (4..7) convert the weights of the NEXT super-block at the end of the current one, after their last tile,
    // so that they start every super-block with matrix work while their partner converts.
    //
    // Inside a super-block the order is pinned step by step (the scheduling barriers let nothing cross): four
    // activation fragments are always in flight, a fragment register is refilled as soon as its two matrix
    // instructions are issued, the activation scales of a tile arrive during its last four steps, the next
    // tile's first fragments during the flush.  The requests for the next super-block are issued one per step
    // in the tiles without conversion work: all waves asking at once right after the barrier only queue up in
    // the memory pipeline.
    auto run = [&](auto late_tag) {
        constexpr bool LATE = decltype(late_tag)::value;
        if (LATE) {   // weights of the first super-block, with nothing to overlap
            read_header();
#pragma unroll
            for (int t = 0; t < 8; ++t) convert(t, strip_piece(t));
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the strip is about to be overwritten
        }
        for (int64_t sb = sb_begin; sb < sb_end; ++sb) {
            const int buf = (int)((sb - sb_begin) & 1);
            const uint32_t sb_next = (uint32_t)(sb + 1 < sb_end ? sb + 1 : sb_end - 1);   // past the end: requested again, never used
            v4i raw[4];
            if (!LATE) {   // out of the strip: header of row l%32, then the lane's 64 nibble bytes
                read_header();
#pragma unroll
                for (int i = 0; i < 4; ++i) raw[i] = *reinterpret_cast<const v4i *>(park + l32 * 144 + 16 + 64 * lh + 16 * i);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the strip is about to be overwritten
            }
            const float dxreg = dxbase_s[dxoffg + sb_next];
            __builtin_amdgcn_sched_barrier(0);
            const int8_t *ab = sm.a[buf];
            const uint8_t *msb = reinterpret_cast<const uint8_t *>(sm.ms[buf]);
            const float *dxs = sm.dx[buf];
            auto fragment = [&](int j, int t) {
                return *reinterpret_cast<const v4i *>(ab + j * 32 * 256 + (aoffl ^ (16 * t)));
            };
            v4i ring[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) ring[t] = fragment(0, t);
            // ---- min term: -dmin*min of the 8 sub-blocks as fp16 high and low parts
            const float dn = h2f((uint32_t)hdr[0] & 0xffffu) * kMinPrescale;   // exact: a power of two
            {
                const ScalesK4 sc = unpack_scales_k4((uint32_t)hdr[1], (uint32_t)hdr[2], (uint32_t)hdr[3]);
                const float ndmin = -h2f((uint32_t)hdr[0] >> 16);
                v8h mh, ml;
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    _Float16 h, l;
                    split_h(ndmin * (float)min_k4(sc, t), h, l);
                    mh[t] = h;
                    ml[t] = lh ? (_Float16)0.f : l;
                }
#pragma unroll
                for (int j = 0; j < JT; ++j) {
                    const v8h am = *reinterpret_cast<const v8h *>(msb + (j * 32 + l32) * 32 + 16 * lh);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(am, mh, acc[j], 0, 0, 0);
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(am, ml, acc[j], 0, 0, 0);
                }
            }
            if (!LATE) convert(0, raw[0]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < JT; ++j) {
                v16i ilo, ihi;
                v4i dq[4];
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    ilo = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[t & 3], cl[t], t == 0 ? zi : ilo, 0, 0, 0);
                    ihi = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[t & 3], ch[t], t == 0 ? zi : ihi, 0, 0, 0);
                    if (t < 4) ring[t & 3] = fragment(j, t + 4);
                    else dq[t - 4] = *reinterpret_cast<const v4i *>(dxs + j * 32 + 8 * (t - 4) + 4 * lh);
                    if (!LATE && j == 0 && t < 7) convert(t + 1, raw[2 * ((t + 1) >> 2) + ((t + 1) & 1)]);
                    // requests for the next super-block, one per step: the strip first (its previous content was
                    // read at the top of this trip by the early waves, at the end of the last one by the late waves)
                    if (j == (LATE ? 0 : 1) && t < 5) request_strip(sb_next, t);
                    if (j == (LATE ? 1 : 2) && (t & 1)) request_act(sb_next, buf ^ 1, t >> 1);
                    if (j == (LATE ? 1 : 2) && t == 0) request_ms(sb_next, buf ^ 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (j + 1 < JT) {
#pragma unroll
                    for (int t = 0; t < 4; ++t) ring[t] = fragment(j + 1, t);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    acc[j][v] = fmaf((float)((ihi[v] << 3) + ilo[v]), __int_as_float(dq[v >> 2][v & 3]) * dn, acc[j][v]);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (LATE) {
                // the next super-block's raw weights were requested at the top of this trip; of the requests
                // made since then (four activation chunks; these waves load no min-term piece) none needs
                // to have landed
                asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
                read_header();
#pragma unroll
                for (int t = 0; t < 8; ++t) convert(t, strip_piece(t));
            }
            sm.dx[buf ^ 1][tid & 127] = dxreg * inv_rs;   // every thread stores (a repeated value past 128): no branch
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __syncthreads();
        }
    };
    if (wave < 4) run(std::false_type{});
    else run(std::true_type{});

    // ---- store: accumulator register v of lane l is row 8*(v/4) + 4*(l/32) + v%4, column l%32
    const int64_t n = n0 + wave * 32 + l32;
    // the rows' factors (normaliser / 16) go through the idle scale buffer: four rows per read, no load per store
    sm.dx[0][tid & 127] = rs_mine * (1.0f / kMinPrescale);
    __syncthreads();
    // two stretches and no scratch: the output rows were cleared before the launch and both stretches add their
    // tile to them (0 + a + b is a + b in either order, so the result does not depend on which arrives first)
    const bool add = gridDim.y > 1 && part == nullptr;
    float *out = gridDim.y > 1 && !add ? part + (size_t)blockIdx.y * M * N : y;
#pragma unroll
    for (int j = 0; j < JT; ++j) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float4 f4 = *reinterpret_cast<const float4 *>(&sm.dx[0][j * 32 + 8 * g + 4 * lh]);
            const float f[4] = {f4.x, f4.y, f4.z, f4.w};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t m = m0 + j * 32 + 8 * g + 4 * lh + r;
                if (m < M && n < N) {
                    if (add) unsafeAtomicAdd(out + m * N + n, acc[j][4 * g + r] * f[r]);
                    else out[m * N + n] = acc[j][4 * g + r] * f[r];
                }
            }
        }
    }
}

}  // namespace

namespace {
// y[i] = part[0][i] + part[1][i] + ... in that order
__global__ __launch_bounds__(256) void sum_parts_kernel(const float *__restrict__ part, int n_split, size_t n4,
                                                        float *__restrict__ y) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    float4 s = reinterpret_cast<const float4 *>(part)[i];
    for (int c = 1; c < n_split; ++c) {
        const float4 v = reinterpret_cast<const float4 *>(part)[(size_t)c * n4 + i];
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    reinterpret_cast<float4 *>(y)[i] = s;
}

template <int QT>
hipError_t launch_per32(const WeightView &w, const ActView &a, int64_t M, float *y, const Scratch &sc, hipStream_t s) {
    if (w.K > (1 << 24)) return hipErrorInvalidValue;   // 32-bit lane offsets: 128 rows of K bytes
    const int n_split = sc.p ? per32_splits(w.K, M, w.N) : 1;
    if (n_split > 1 && (size_t)n_split * M * w.N * 4 > sc.bytes) return hipErrorInvalidValue;   // partial tiles would not fit
    if (dry_run()) {
        if (n_split > 1) plan_note_cut();
        plan_note("gemm_per32_kernel<%s>: tile 128 tokens x 128 rows, %lld tiles x %d K stretches%s", plan_type_name(QT),
                  (long long)(((w.N + BN - 1) / BN) * ((M + BM - 1) / BM)), n_split, n_split > 1 ? " + sum_parts_kernel" : "");
        return hipSuccess;
    }
    const auto kern = &gemm_per32_kernel<QT>;
    static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(GemmSmem));
    if (attr != hipSuccess) return attr;
    const dim3 grid((unsigned)(((w.N + BN - 1) / BN) * ((M + BM - 1) / BM)), (unsigned)n_split);
    hipLaunchKernelGGL(kern, grid, dim3(kGemmThreads), sizeof(GemmSmem), s, w, a, M, y, sc.p);
    if (n_split > 1) {
        const size_t n4 = (size_t)M * w.N / 4;
        hipLaunchKernelGGL(sum_parts_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s, sc.p, n_split, n4, y);
    }
    return hipGetLastError();
}
}  // namespace

hipError_t launch_sum_parts(const float *part, int n_split, size_t n, float *y, hipStream_t s) {
    if (dry_run()) {
        plan_note("sum_parts_kernel: adds %d partial results of %zu outputs in order", n_split, n);
        return hipSuccess;
    }
    const size_t n4 = n / 4;   // callers only split when n is a multiple of 4
    hipLaunchKernelGGL(sum_parts_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s, part, n_split, n4, y);
    return hipGetLastError();
}

// K stretches for the kernels that take ggml-format activations (64-token x 128-row tiles, two workgroups per
// compute unit = 512 places): below 384 tiles K is cut in 2, below 192 in 3, below 96 in 4, below 64 in 8, never under twelve super-blocks a
// stretch (K = 4096 cut in two measured slower than whole: the pass that adds the partial tiles costs more
// than the fuller grid gains).
int q8k_tile_splits(int64_t K, int64_t M, int64_t N, bool add_ok) {
    static const int forced = tuning_int("QPROJ_Q8K_SPLITS", 0);
    static const bool no_add = tuning_int("QPROJ_NO_TILE_ADD", 0) != 0;
    const int64_t tiles = ((N + 127) / 128) * ((M + 63) / 64);
    // Two stretches that add themselves to cleared output rows cost no pass over partial tiles: from 96 tiles on that
    // beats three stretches with the pass, and K = 4096 (eight super-blocks a stretch) is worth cutting while the whole-K
    // tiles would not give every compute unit a workgroup.  Per call, us: 4096 x 4096 at 192 / 256 tokens 32.7 / 34.2 ->
    // 26.5 / 28.8 (at 512 tokens, 256 tiles, the cut loses: 39.9 -> 42.8, so it stays whole); 4096 -> 14336 at 64 tokens
    // 32.0 -> 27.7; 14336 -> 4096 at 192 / 256 tokens 65.3 / 67.6 -> 59.9 / 63.2.
    if (add_ok && !no_add && forced <= 0 && (M * N) % 4 == 0 && tiles >= 96 && tiles < 384 && K / 256 >= 16 &&
        (K / 256 >= 24 || tiles < 256))
        return 2;
    // (under 64 tiles - a down projection of 4096 rows at up to 64 tokens is 32 - eight stretches: 14336 -> 4096 at
    // 33 / 64 tokens, four -> eight stretches, Q6_K 42.0 / 43.5 -> 29.7 / 31.1 us, Q4_K 35.6 / 37.4 -> 27.9 / 29.7; ten to
    // fourteen were slower again, the pass over the partial tiles grows; 64 tiles keep four: seven 47.2 -> 46.1 for Q6_K
    // and 40.5 -> 42.8 for Q4_K)
    int n = forced > 0 ? forced : tiles >= 384 ? 1 : tiles >= 192 ? 2 : tiles >= 96 ? 3 : tiles >= 64 ? 4 : 8;
    if ((M * N) % 4 != 0) n = 1;
    // a stretch is at least 12 super-blocks (the pass that adds the partial tiles has to be earned), 4 where the
    // grid is under a fifth of the workgroups the chip holds and a workgroup's K loop is pure latency
    const int min_sb = tiles >= 192 ? 12 : 4;
    while (n > 1 && K / 256 < min_sb * n) --n;
    return n;
}
size_t q8k_tile_scratch_bytes(int64_t K, int64_t M, int64_t N) {
    const int n = q8k_tile_splits(K, M, N, false);
    return n > 1 ? (size_t)n * M * N * 4 : 0;
}

// A grid of fewer than 192 tiles leaves the 256 compute units mostly idle and a workgroup's K loop is
// latency-bound: K is then cut into stretches done by different workgroups, as many as fill one round (32 tiles of
// K = 14336, Q8_0 at 64 - 128 tokens: 8 stretches instead of 3).
int per32_splits(int64_t K, int64_t M, int64_t N) {
    static const int forced = tuning_int("QPROJ_PER32_SPLITS", 0);
    const int64_t tiles = ((N + BN - 1) / BN) * ((M + BM - 1) / BM);
    // as many stretches as fill one round of workgroups (one a compute unit), eight at most
    int n = forced > 0 ? forced : tiles >= 192 ? 1 : (int)std::min<int64_t>(8, std::max<int64_t>(1, cu_count() / tiles));
    if ((M * N) % 4 != 0) n = 1;
    while (n > 1 && K / 256 < 4 * n) --n;   // at least four super-blocks a stretch
    return n;
}
size_t per32_scratch_bytes(int64_t K, int64_t M, int64_t N) {
    const int n = per32_splits(K, M, N);
    return n > 1 ? (size_t)n * M * N * 4 : 0;
}

hipError_t launch_gemm_q8x32(const WeightView &w, const ActView &a, int64_t M, float *y, const Scratch &scratch, hipStream_t s) {
    if (w.type != kTypeQ4_K || w.K % 256 != 0 || M <= 0 || !a.msum || !a.rs) return hipErrorInvalidValue;
    return launch_per32<kTypeQ4_K>(w, a, M, y, scratch, s);
}

// Q8_0 weights x ggml Q8_0 activation blocks (planes in `a`), K a multiple of 128
hipError_t launch_gemm_q8_0(const WeightView &w, const ActView &a, int64_t M, float *y, const Scratch &scratch, hipStream_t s) {
    if (w.type != kTypeQ8_0 || a.kind != kActKindQ8_0 || w.K % BK != 0 || M <= 0) return hipErrorInvalidValue;
    return launch_per32<kTypeQ8_0>(w, a, M, y, scratch, s);
}

// Which Q4_K kernel and how many stretches of K (one rule for the launcher and for the scratch sizing).  The
// 128-token kernel (256 weight rows a workgroup, one workgroup per compute unit) wants about 192 workgroups or more:
// a grid of 48..191 such tiles is multiplied by cutting K into the stretches wide_tile_splits picks (64 tiles of
// K = 14336: four; of K = 11008: three, 192 workgroups, where the halving rule before left half the chip idle).
// Everything else takes 64-token tiles with the stretches of q8k_tile_splits.
namespace {
struct Q4Plan {
    bool wide;
    int n_split;
};
// add_ok: the output rows hold zeros when the launch starts (Scratch::zeroed)
Q4Plan q4k_plan(int64_t K, int64_t M, int64_t N, bool have_scratch, bool add_ok = false) {
    static const int wide_env = tuning_int("QPROJ_Q8K_WIDE", -1);
    const int64_t wide_tiles = ((N + 255) / 256) * ((M + 127) / 128);
    if (wide_env >= 0 ? wide_env != 0 : wide_tiles >= 192) return {true, 1};
    if (wide_env < 0 && have_scratch && (M * N) % 4 == 0 && wide_tiles >= 48) {
        const int n = wide_tile_splits(wide_tiles, K / 256, M, N, cu_count(), 4.5);
        if (n > 1) return {true, n};
    }
    return {false, have_scratch || add_ok ? q8k_tile_splits(K, M, N, add_ok) : 1};
}
}  // namespace


size_t q4k_tile_scratch_bytes(int64_t K, int64_t M, int64_t N) {
    const Q4Plan p = q4k_plan(K, M, N, true);
    return p.n_split > 1 ? (size_t)p.n_split * M * N * 4 : 0;
}

// ggml-format activations (Q8_K planes in `a`, including the min-term plane), Q4_K weights, any M
hipError_t launch_gemm_q8k(const WeightView &w, const ActView &a, int64_t M, float *y, const Scratch &scratch, hipStream_t s) {
    if (w.type != kTypeQ4_K || a.kind != kActKindQ8_K || !a.msum || !a.rs || M <= 0) return hipErrorInvalidValue;
    if (w.K > (1 << 24)) return hipErrorInvalidValue;   // 32-bit lane offsets: 128 token rows of K bytes, 32 weight rows of K*144/256
    const bool zeroed = (scratch.zeroed & 1u) != 0;
    Q4Plan p = q4k_plan(w.K, M, w.N, scratch.p != nullptr, zeroed);
    const bool add = zeroed && p.n_split == 2;   // both stretches add to the cleared rows: no partial tiles
    if (zeroed && !add) p = q4k_plan(w.K, M, w.N, scratch.p != nullptr);
    if (p.n_split > 1 && !add && (size_t)p.n_split * M * w.N * 4 > scratch.bytes) return hipErrorInvalidValue;   // partial tiles would not fit
    if (dry_run()) {
        if (p.n_split > 1 && !add) plan_note_cut();
        const long long tiles = p.wide ? (long long)(((w.N + 255) / 256) * ((M + 127) / 128)) : (long long)(((w.N + 127) / 128) * ((M + 63) / 64));
        plan_note("%s: tile %s, %lld tiles x %d K stretches%s, partial tiles %zu B", p.wide ? "gemm_q4k_q8k_wide_kernel" : "gemm_q4k_q8k_direct_kernel",
                  p.wide ? "128 tokens x 256 rows" : "64 tokens x 128 rows", tiles, p.n_split,
                  p.n_split == 1 ? "" : add ? ", the two stretches add themselves to cleared rows" : " + sum_parts_kernel",
                  p.n_split > 1 && !add ? (size_t)p.n_split * M * w.N * 4 : (size_t)0);
        return hipSuccess;
    }
    float *const part = add ? nullptr : scratch.p;
    if (p.wide) {   // 128 tokens x 256 weight rows per workgroup, one workgroup per compute unit
        using Smem = WideSmem<8>;
        const auto kern = &gemm_q4k_q8k_wide_kernel<8>;
        static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(Smem));
        if (attr != hipSuccess) return attr;
        const int64_t wide_tiles = ((w.N + 255) / 256) * ((M + 127) / 128);
        hipLaunchKernelGGL(kern, dim3((unsigned)wide_tiles, (unsigned)p.n_split), dim3(512), sizeof(Smem), s, w, a, M, y, part);
        if (p.n_split > 1 && !add) return launch_sum_parts(scratch.p, p.n_split, (size_t)M * w.N, y, s);
        return hipGetLastError();
    }
    constexpr int NW = 4;   // 64 tokens x 128 weight rows per workgroup, two workgroups per compute unit
    using Smem = DirectSmem<NW>;
    static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4k_q8k_direct_kernel<NW>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(Smem));
    if (attr != hipSuccess) return attr;
    const dim3 grid((unsigned)(((w.N + 32 * NW - 1) / (32 * NW)) * ((M + 63) / 64)), (unsigned)p.n_split);
    DirectTargets tg{};
    tg.n = 1;
    tg.w[0] = w;
    tg.y[0] = y;
    hipLaunchKernelGGL(gemm_q4k_q8k_direct_kernel<NW>, grid, dim3(64 * NW), sizeof(Smem), s, tg, a, M, part);
    if (p.n_split > 1 && !add) return launch_sum_parts(scratch.p, p.n_split, (size_t)M * w.N, y, s);
    return hipGetLastError();
}

namespace {
// Which of n matrices over the same activation rows share ONE launch of the 64-token kernel: those that would take it
// with K in one stretch (or are small enough to be better off together than cut).  The others (128-token tiles, K cut
// into stretches) get launches of their own.  Fills joined[], returns how many (0 or >= 2).
int q4k_joined_set(int n, const WeightView *w, int64_t M, bool have_scratch, bool planes_ok, int (&joined)[3]) {
    static const int wide_env = tuning_int("QPROJ_Q8K_WIDE", -1);
    static const bool off = tuning_int("QPROJ_Q8K_NO_MULTI", 0) != 0;
    const bool can = !off && n >= 2 && n <= 3 && wide_env < 0 && planes_ok && M > 0;
    int n_joined = 0;
    for (int i = 0; i < n; ++i) {
        const Q4Plan p = q4k_plan(w[i].K, M, w[i].N, have_scratch);
        const bool fits = can && w[i].type == kTypeQ4_K && w[i].K == w[0].K && w[i].K <= (1 << 24) && !p.wide &&
                          (p.n_split == 1 || ((w[i].N + 127) / 128) * ((M + 63) / 64) < 96);   // small ones are better off together than cut
        if (fits) joined[n_joined++] = i;
    }
    return n_joined < 2 ? 0 : n_joined;
}
}  // namespace

// bit i: matrix i of a launch_gemm_q8k_multi call gets a launch of its own that cuts K in two stretches which add
// themselves, if its output rows are cleared beforehand
uint32_t q4k_multi_adds(int n, const WeightView *w, int64_t M, bool have_scratch) {
    int joined[3];
    const int n_joined = n <= 3 ? q4k_joined_set(n, w, M, have_scratch, true, joined) : 0;
    uint32_t mask = 0;
    for (int i = 0; i < n; ++i) {
        bool in = false;
        for (int j = 0; j < n_joined; ++j) in = in || joined[j] == i;
        if (!in && w[i].type == kTypeQ4_K && q4k_plan(w[i].K, M, w[i].N, have_scratch, true).n_split == 2) mask |= 1u << i;
    }
    return mask;
}

// The same for n matrices over the same activation rows.  One launch where every matrix would take the
// 64-token kernel with K in one stretch; otherwise one launch a matrix, as above.
hipError_t launch_gemm_q8k_multi(int n, const WeightView *w, const ActView &a, int64_t M, float *const *y,
                                 const Scratch &scratch, hipStream_t s) {
    constexpr int NW = 4;
    int joined[3];
    int n_joined = n <= 3 ? q4k_joined_set(n, w, M, scratch.p != nullptr, a.kind == kActKindQ8_K && a.msum && a.rs, joined) : 0;
    for (int i = 0; i < n; ++i) {
        bool in = false;
        for (int j = 0; j < n_joined; ++j) in = in || joined[j] == i;
        if (in) continue;
        hipError_t e = launch_gemm_q8k(w[i], a, M, y[i], scratch.for_target(i), s);
        if (e != hipSuccess) return e;
    }
    if (n_joined == 0) return hipSuccess;
    if (dry_run()) {
        long long wgs = 0;
        for (int j = 0; j < n_joined; ++j) {
            wgs += (long long)(((w[joined[j]].N + 32 * NW - 1) / (32 * NW)) * ((M + 63) / 64));
            wgs = (wgs + 7) / 8 * 8;
        }
        plan_note("gemm_q4k_q8k_direct_kernel: %d matrices in one launch, tile 64 tokens x 128 rows, %lld workgroups, K whole", n_joined, wgs);
        return hipSuccess;
    }
    using Smem = DirectSmem<NW>;
    static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q4k_q8k_direct_kernel<NW>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(Smem));
    if (attr != hipSuccess) return attr;
    DirectTargets tg{};
    tg.n = n_joined;
    int64_t wg = 0;
    for (int j = 0; j < n_joined; ++j) {
        const int i = joined[j];
        tg.w[j] = w[i];
        tg.y[j] = y[i];
        tg.first_wg[j] = (int)wg;
        wg += ((w[i].N + 32 * NW - 1) / (32 * NW)) * ((M + 63) / 64);
        wg = (wg + 7) / 8 * 8;   // the next matrix starts on XCD 0 again
    }
    if (wg >= 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL(gemm_q4k_q8k_direct_kernel<NW>, dim3((unsigned)wg), dim3(64 * NW), sizeof(Smem), s, tg, a, M,
                       static_cast<float *>(nullptr));
    return hipGetLastError();
}

}  // namespace qproj
