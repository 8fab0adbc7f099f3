/*
 * CPU oracle for the quantized projection path -- see qproj_oracle.h for scope,
 * provenance and pin status.  TEST INFRASTRUCTURE ONLY.
 *
 * Upstream functions restated here live in llama.cpp @ 0b1bad14 (absent from
 * /root/reference; pinned by /root/reference/inference/native-pin.toml:11-14):
 *   ggml/src/ggml-common.h      block_q8_0, block_q4_K, block_q6_K, block_q8_K
 *   ggml/src/ggml-quants.c      quantize_row_q8_0_ref, dequantize_row_*, nearest_int, get_scale_min_k4
 *   ggml/src/ggml-cpu/quants.c  ggml_vec_dot_*_generic, quantize_row_q8_K
 *   ggml/src/ggml-cpu/ggml-cpu.c ggml_compute_forward_mul_mat{,_id}
 *   src/llama-graph.cpp         build_moe_ffn
 *
 * Build with -ffp-contract=off: "d*q - m" must stay a multiply followed by a
 * subtract so that bit-exact dequantization has one meaning.
 */
#include "qproj_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#if defined(__F16C__) || defined(__AVX2__)
#include <immintrin.h>
#endif

/* ---------------------------------------------------------------- sizes */

size_t orc_sizeof_block(int type) {
    switch (type) {
    case ORC_TYPE_Q8_0: return sizeof(orc_block_q8_0);
    case ORC_TYPE_Q4_K: return sizeof(orc_block_q4_K);
    case ORC_TYPE_Q6_K: return sizeof(orc_block_q6_K);
    default: return 0;
    }
}

int orc_block_elems(int type) {
    switch (type) {
    case ORC_TYPE_Q8_0: return ORC_QK8_0;
    case ORC_TYPE_Q4_K:
    case ORC_TYPE_Q6_K: return ORC_QK_K;
    default: return 0;
    }
}

size_t orc_row_bytes(int type, int64_t k) {
    int be = orc_block_elems(type);
    if (be == 0 || k % be != 0) return 0;
    return (size_t)(k / be) * orc_sizeof_block(type);
}

_Static_assert(sizeof(orc_block_q8_0) == 34, "block_q8_0 is 34 bytes");
_Static_assert(sizeof(orc_block_q4_K) == 144, "block_q4_K is 144 bytes");
_Static_assert(sizeof(orc_block_q6_K) == 210, "block_q6_K is 210 bytes");
_Static_assert(sizeof(orc_block_q8_K) == 292, "block_q8_K is 292 bytes");

/* ---------------------------------------------------------------- fp16 */

/* IEEE binary16 -> binary32, exact, subnormals included (ggml GGML_FP16_TO_FP32). */
float orc_fp16_to_fp32(orc_half h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while ((man & 0x400u) == 0);
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* binary32 -> binary16, round to nearest even (ggml GGML_FP32_TO_FP16). */
orc_half orc_fp32_to_fp16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        return (orc_half)(sign | 0x7c00u | ((ax > 0x7f800000u) ? (0x200u | ((ax >> 13) & 0x3ffu)) : 0));
    }
    int32_t e = (int32_t)(ax >> 23) - 127 + 15;
    uint32_t man = ax & 0x7fffffu;
    if (e >= 31) return (orc_half)(sign | 0x7c00u); /* overflow -> inf */
    if (e <= 0) {
        if (e < -10) return (orc_half)sign; /* underflow -> 0 */
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1u))) half++;
        return (orc_half)(sign | half);
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) half++; /* may carry into exponent: correct */
    return (orc_half)(sign | half);
}

float orc_fp16_to_fp32_f16c(orc_half h) {
#if defined(__F16C__)
    return _cvtsh_ss(h);
#else
    return orc_fp16_to_fp32(h);
#endif
}

orc_half orc_fp32_to_fp16_f16c(float f) {
#if defined(__F16C__)
    return (orc_half)_cvtss_sh(f, 0);
#else
    return orc_fp32_to_fp16(f);
#endif
}

/* ---------------------------------------------------------------- 6-bit scales */

/* ggml-quants.c get_scale_min_k4: sub-block j of a Q4_K super-block keeps a
 * 6-bit scale and a 6-bit min inside 12 bytes. */
void orc_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0x0f) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* inverse of the above, as written by quantize_row_q4_K_ref */
void orc_pack_scale_min_k4(const uint8_t sc[8], const uint8_t mn[8], uint8_t out[12]) {
    memset(out, 0, 12);
    for (int j = 0; j < 8; ++j) {
        uint8_t ls = sc[j] & 63, lm = mn[j] & 63;
        if (j < 4) {
            out[j] |= ls;
            out[j + 4] |= lm;
        } else {
            out[j + 4] = (uint8_t)((ls & 0x0f) | ((lm & 0x0f) << 4));
            out[j - 4] |= (uint8_t)((ls >> 4) << 6);
            out[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
}

/* ---------------------------------------------------------------- dequantize */

/* ggml-quants.c dequantize_row_q8_0: y = q * d */
void orc_dequantize_row_q8_0(const orc_block_q8_0 *x, float *y, int64_t k) {
    const int64_t nb = k / ORC_QK8_0;
    for (int64_t i = 0; i < nb; ++i) {
        const float d = orc_fp16_to_fp32(x[i].d);
        for (int j = 0; j < ORC_QK8_0; ++j) y[i * ORC_QK8_0 + j] = x[i].qs[j] * d;
    }
}

/* ggml-quants.c dequantize_row_q4_K: y = (d*sc)*q - (dmin*m), multiply then subtract */
void orc_dequantize_row_q4_K(const orc_block_q4_K *x, float *y, int64_t k) {
    const int64_t nb = k / ORC_QK_K;
    for (int64_t i = 0; i < nb; ++i) {
        const uint8_t *q = x[i].qs;
        const float d = orc_fp16_to_fp32(x[i].d);
        const float min = orc_fp16_to_fp32(x[i].dmin);
        int is = 0;
        for (int j = 0; j < ORC_QK_K; j += 64) {
            uint8_t sc, m;
            orc_get_scale_min_k4(is + 0, x[i].scales, &sc, &m);
            const float d1 = d * sc;
            const float m1 = min * m;
            orc_get_scale_min_k4(is + 1, x[i].scales, &sc, &m);
            const float d2 = d * sc;
            const float m2 = min * m;
            for (int l = 0; l < 32; ++l) *y++ = d1 * (q[l] & 0xF) - m1;
            for (int l = 0; l < 32; ++l) *y++ = d2 * (q[l] >> 4) - m2;
            q += 32;
            is += 2;
        }
    }
}

/* ggml-quants.c dequantize_row_q6_K: y = (d*sc)*(q-32) */
void orc_dequantize_row_q6_K(const orc_block_q6_K *x, float *y, int64_t k) {
    const int64_t nb = k / ORC_QK_K;
    for (int64_t i = 0; i < nb; ++i) {
        const float d = orc_fp16_to_fp32(x[i].d);
        const uint8_t *ql = x[i].ql;
        const uint8_t *qh = x[i].qh;
        const int8_t *sc = x[i].scales;
        for (int n = 0; n < ORC_QK_K; n += 128) {
            for (int l = 0; l < 32; ++l) {
                const int is = l / 16;
                const int8_t q1 = (int8_t)((ql[l + 0] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                const int8_t q2 = (int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                const int8_t q3 = (int8_t)((ql[l + 0] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                const int8_t q4 = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                y[l + 0] = d * sc[is + 0] * q1;
                y[l + 32] = d * sc[is + 2] * q2;
                y[l + 64] = d * sc[is + 4] * q3;
                y[l + 96] = d * sc[is + 6] * q4;
            }
            y += 128;
            ql += 64;
            qh += 32;
            sc += 8;
        }
    }
}

void orc_dequantize_row(int type, const void *blocks, float *y, int64_t k) {
    switch (type) {
    case ORC_TYPE_Q8_0: orc_dequantize_row_q8_0((const orc_block_q8_0 *)blocks, y, k); break;
    case ORC_TYPE_Q4_K: orc_dequantize_row_q4_K((const orc_block_q4_K *)blocks, y, k); break;
    case ORC_TYPE_Q6_K: orc_dequantize_row_q6_K((const orc_block_q6_K *)blocks, y, k); break;
    default: break;
    }
}

/* ---------------------------------------------------------------- quantize */

/* ggml-quants.c nearest_int: round half to even through the 2^23+2^22 trick */
static inline int nearest_int(float fval) {
    float val = fval + 12582912.f;
    int i;
    memcpy(&i, &val, sizeof(int));
    return (i & 0x007fffff) - 0x00400000;
}

#define ORC_MAX(a, b) ((a) > (b) ? (a) : (b))
#define ORC_MIN(a, b) ((a) < (b) ? (a) : (b))
#define ORC_GROUP_MAX_EPS 1e-15f

/* ggml-quants.c quantize_row_q8_0_ref: d = amax/127, q = roundf(x * (1/d)) */
void orc_quantize_row_q8_0(const float *x, orc_block_q8_0 *y, int64_t k) {
    const int64_t nb = k / ORC_QK8_0;
    for (int64_t i = 0; i < nb; ++i) {
        float amax = 0.0f;
        for (int j = 0; j < ORC_QK8_0; ++j) {
            const float v = fabsf(x[i * ORC_QK8_0 + j]);
            amax = ORC_MAX(amax, v);
        }
        const float d = amax / ((1 << 7) - 1);
        const float id = d ? 1.0f / d : 0.0f;
        y[i].d = orc_fp32_to_fp16(d);
        for (int j = 0; j < ORC_QK8_0; ++j) {
            const float x0 = x[i * ORC_QK8_0 + j] * id;
            y[i].qs[j] = (int8_t)roundf(x0);
        }
    }
}

/* per-32 activation block of the prefill path: like q8_0 but the scale stays
 * fp32 and the integer sum of the quants is kept for the Q4_K min term. */
void orc_quantize_row_q8x32(const float *x, orc_block_q8x32 *y, int64_t k) {
    const int64_t nb = k / 32;
    for (int64_t i = 0; i < nb; ++i) {
        float amax = 0.0f;
        for (int j = 0; j < 32; ++j) {
            const float v = fabsf(x[i * 32 + j]);
            amax = ORC_MAX(amax, v);
        }
        const float d = amax / 127.0f;
        const float id = d ? 1.0f / d : 0.0f;
        int32_t s = 0;
        for (int j = 0; j < 32; ++j) {
            const int q = (int)roundf(x[i * 32 + j] * id);
            y[i].qs[j] = (int8_t)q;
            s += q;
        }
        y[i].d = d;
        y[i].isum = s;
    }
}

/* ggml-cpu/quants.c quantize_row_q8_K (== quantize_row_q8_K_ref) */
void orc_quantize_row_q8_K(const float *x, orc_block_q8_K *y, int64_t k) {
    const int64_t nb = k / ORC_QK_K;
    for (int64_t i = 0; i < nb; ++i) {
        float max = 0, amax = 0;
        for (int j = 0; j < ORC_QK_K; ++j) {
            const float ax = fabsf(x[j]);
            if (ax > amax) {
                amax = ax;
                max = x[j];
            }
        }
        if (!amax) {
            memset(&y[i], 0, sizeof(y[i]));
            x += ORC_QK_K;
            continue;
        }
        const float iscale = -127.f / max;
        for (int j = 0; j < ORC_QK_K; ++j) {
            const int v = nearest_int(iscale * x[j]);
            y[i].qs[j] = (int8_t)ORC_MIN(127, v);
        }
        for (int j = 0; j < ORC_QK_K / 16; ++j) {
            int sum = 0;
            for (int ii = 0; ii < 16; ++ii) sum += y[i].qs[j * 16 + ii];
            y[i].bsums[j] = (int16_t)sum;
        }
        y[i].d = 1 / iscale;
        x += ORC_QK_K;
    }
}

/* Weight-side quantizer of the oracle: Q8_0 only (the one the benchmark configuration defines completely).
 * Q4_K / Q6_K weight blocks are INPUTS of this path -- models arrive quantized -- and the tests make them with the
 * format-valid encoders of tests/kquant_encoders.c, which are not part of the oracle. */
int orc_quantize_rows(int type, const float *x, void *blocks, int64_t k, int64_t nrows, int nthreads) {
    if (type != ORC_TYPE_Q8_0 || k % ORC_QK8_0 != 0) return -1;
    const size_t rb = orc_row_bytes(type, k);
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t r = 0; r < nrows; ++r)
        orc_quantize_row_q8_0(x + r * k, (orc_block_q8_0 *)((char *)blocks + (size_t)r * rb), k);
    return 0;
}

/* ---------------------------------------------------------------- dot products */

/* ggml-cpu/quants.c ggml_vec_dot_q8_0_q8_0_generic */
float orc_vec_dot_q8_0_q8_0(int64_t k, const orc_block_q8_0 *w, const orc_block_q8_0 *a) {
    const int64_t nb = k / ORC_QK8_0;
    float sumf = 0;
    for (int64_t ib = 0; ib < nb; ++ib) {
        int sumi = 0;
        for (int j = 0; j < ORC_QK8_0; ++j) sumi += w[ib].qs[j] * a[ib].qs[j];
        sumf += sumi * (orc_fp16_to_fp32(w[ib].d) * orc_fp16_to_fp32(a[ib].d));
    }
    return sumf;
}

/* ggml-cpu/quants.c ggml_vec_dot_q4_K_q8_K_generic.  Eight interleaved int32
 * lanes (element index mod 8) carry scale*(q4*q8); each lane is scaled by
 * d*y.d per super-block into its own fp32 sum; the min term is one fp32
 * accumulator; the lanes are added to it at the end. */
float orc_vec_dot_q4_K_q8_K(int64_t k, const orc_block_q4_K *w, const orc_block_q8_K *a) {
    const int64_t nb = k / ORC_QK_K;
    float lane_sum[8] = {0};
    float sumf = 0;
    for (int64_t i = 0; i < nb; ++i) {
        int8_t q[ORC_QK_K];
        const uint8_t *q4 = w[i].qs;
        for (int c = 0; c < 4; ++c) {
            for (int l = 0; l < 32; ++l) q[64 * c + l] = (int8_t)(q4[32 * c + l] & 0xF);
            for (int l = 0; l < 32; ++l) q[64 * c + 32 + l] = (int8_t)(q4[32 * c + l] >> 4);
        }
        uint8_t sc[8], mn[8];
        for (int j = 0; j < 8; ++j) orc_get_scale_min_k4(j, w[i].scales, &sc[j], &mn[j]);
        int sumi = 0;
        for (int j = 0; j < 16; ++j) sumi += a[i].bsums[j] * mn[j / 2];
        int32_t lane[8] = {0};
        for (int j = 0; j < 8; ++j) {
            const int32_t scale = sc[j];
            for (int l = 0; l < 32; ++l) {
                const int16_t p = (int16_t)(a[i].qs[32 * j + l] * q[32 * j + l]);
                lane[l & 7] += scale * p;
            }
        }
        const float d = orc_fp16_to_fp32(w[i].d) * a[i].d;
        for (int l = 0; l < 8; ++l) lane_sum[l] += d * lane[l];
        const float dmin = orc_fp16_to_fp32(w[i].dmin) * a[i].d;
        sumf -= dmin * sumi;
    }
    for (int l = 0; l < 8; ++l) sumf += lane_sum[l];
    return sumf;
}

/* ggml-cpu/quants.c ggml_vec_dot_q6_K_q8_K_generic */
float orc_vec_dot_q6_K_q8_K(int64_t k, const orc_block_q6_K *w, const orc_block_q8_K *a) {
    const int64_t nb = k / ORC_QK_K;
    float lane_sum[8] = {0};
    for (int64_t i = 0; i < nb; ++i) {
        int8_t q[ORC_QK_K];
        const uint8_t *ql = w[i].ql;
        const uint8_t *qh = w[i].qh;
        for (int n = 0; n < ORC_QK_K; n += 128) {
            for (int l = 0; l < 32; ++l) {
                q[n + l + 0] = (int8_t)((ql[l + 0] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                q[n + l + 32] = (int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                q[n + l + 64] = (int8_t)((ql[l + 0] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                q[n + l + 96] = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
            }
            ql += 64;
            qh += 32;
        }
        int32_t lane[8] = {0};
        for (int j = 0; j < 16; ++j) {
            const int32_t scale = w[i].scales[j];
            for (int l = 0; l < 16; ++l) {
                const int16_t p = (int16_t)(a[i].qs[16 * j + l] * q[16 * j + l]);
                lane[l & 7] += scale * p;
            }
        }
        const float d = orc_fp16_to_fp32(w[i].d) * a[i].d;
        for (int l = 0; l < 8; ++l) lane_sum[l] += d * lane[l];
    }
    float sumf = 0;
    for (int l = 0; l < 8; ++l) sumf += lane_sum[l];
    return sumf;
}

/* Prefill-path dot: activations in per-32 int8 blocks with an fp32 scale.
 * Integer partial sums per 32 (per 16 for Q6_K) are exact; the fp32 order is
 * sequential over K.  This format is the benchmark's own prescription (ggml's
 * GPU backends use the same idea with an fp16 scale), not a ggml CPU routine. */
float orc_vec_dot_q8x32(int type, int64_t k, const void *wv, const orc_block_q8x32 *a) {
    float acc = 0;
    if (type == ORC_TYPE_Q8_0) {
        const orc_block_q8_0 *w = (const orc_block_q8_0 *)wv;
        for (int64_t b = 0; b < k / 32; ++b) {
            int32_t s = 0;
            for (int l = 0; l < 32; ++l) s += w[b].qs[l] * a[b].qs[l];
            acc += (orc_fp16_to_fp32(w[b].d) * a[b].d) * (float)s;
        }
    } else if (type == ORC_TYPE_Q4_K) {
        const orc_block_q4_K *w = (const orc_block_q4_K *)wv;
        for (int64_t i = 0; i < k / ORC_QK_K; ++i) {
            const float d = orc_fp16_to_fp32(w[i].d);
            const float dmin = orc_fp16_to_fp32(w[i].dmin);
            for (int j = 0; j < 8; ++j) {
                uint8_t sc, m;
                orc_get_scale_min_k4(j, w[i].scales, &sc, &m);
                const orc_block_q8x32 *ab = &a[i * 8 + j];
                const uint8_t *q4 = w[i].qs + 32 * (j / 2);
                int32_t s = 0;
                for (int l = 0; l < 32; ++l) {
                    const int q = (j & 1) ? (q4[l] >> 4) : (q4[l] & 0xF);
                    s += q * ab->qs[l];
                }
                acc += ((d * sc) * ab->d) * (float)s - ((dmin * m) * ab->d) * (float)ab->isum;
            }
        }
    } else if (type == ORC_TYPE_Q6_K) {
        const orc_block_q6_K *w = (const orc_block_q6_K *)wv;
        for (int64_t i = 0; i < k / ORC_QK_K; ++i) {
            int8_t q[ORC_QK_K];
            const uint8_t *ql = w[i].ql;
            const uint8_t *qh = w[i].qh;
            for (int n = 0; n < ORC_QK_K; n += 128) {
                for (int l = 0; l < 32; ++l) {
                    q[n + l + 0] = (int8_t)((ql[l + 0] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                    q[n + l + 32] = (int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                    q[n + l + 64] = (int8_t)((ql[l + 0] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                    q[n + l + 96] = (int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                }
                ql += 64;
                qh += 32;
            }
            const float d = orc_fp16_to_fp32(w[i].d);
            for (int j = 0; j < 16; ++j) {
                const orc_block_q8x32 *ab = &a[i * 8 + j / 2];
                int32_t s = 0;
                for (int l = 0; l < 16; ++l) s += q[16 * j + l] * ab->qs[16 * (j & 1) + l];
                acc += ((d * w[i].scales[j]) * ab->d) * (float)s;
            }
        }
    }
    return acc;
}

/* ---------------------------------------------------------------- mul_mat */

static size_t act_row_bytes(int type, int act, int64_t K) {
    if (act == ORC_ACT_Q8X32) return (size_t)(K / 32) * sizeof(orc_block_q8x32);
    if (type == ORC_TYPE_Q8_0) return (size_t)(K / 32) * sizeof(orc_block_q8_0);
    return (size_t)(K / ORC_QK_K) * sizeof(orc_block_q8_K);
}

static void quantize_act_row(int type, int act, const float *x, void *out, int64_t K) {
    if (act == ORC_ACT_Q8X32)
        orc_quantize_row_q8x32(x, (orc_block_q8x32 *)out, K);
    else if (type == ORC_TYPE_Q8_0)
        orc_quantize_row_q8_0(x, (orc_block_q8_0 *)out, K);
    else
        orc_quantize_row_q8_K(x, (orc_block_q8_K *)out, K);
}

static float dot_quantized(int type, int act, int64_t K, const void *wrow, const void *arow) {
    if (act == ORC_ACT_Q8X32) return orc_vec_dot_q8x32(type, K, wrow, (const orc_block_q8x32 *)arow);
    switch (type) {
    case ORC_TYPE_Q8_0:
        return orc_vec_dot_q8_0_q8_0(K, (const orc_block_q8_0 *)wrow, (const orc_block_q8_0 *)arow);
    case ORC_TYPE_Q4_K:
        return orc_vec_dot_q4_K_q8_K(K, (const orc_block_q4_K *)wrow, (const orc_block_q8_K *)arow);
    default:
        return orc_vec_dot_q6_K_q8_K(K, (const orc_block_q6_K *)wrow, (const orc_block_q8_K *)arow);
    }
}

int orc_mul_mat_f64(int type, const void *w, int64_t K, int64_t N, const float *x, int64_t M,
                    double *y, int nthreads) {
    const size_t rb = orc_row_bytes(type, K);
    if (rb == 0) return -1;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel num_threads(nthreads)
    {
        float *row = (float *)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(static)
        for (int64_t n = 0; n < N; ++n) {
            orc_dequantize_row(type, (const char *)w + (size_t)n * rb, row, K);
            for (int64_t m = 0; m < M; ++m) {
                const float *xr = x + m * K;
                double s = 0;
                for (int64_t kk = 0; kk < K; ++kk) s += (double)row[kk] * (double)xr[kk];
                y[m * N + n] = s;
            }
        }
        free(row);
    }
    return 0;
}

/* ggml-cpu.c ggml_compute_forward_mul_mat: src1 rows are converted once to the
 * weight type's vec_dot_type, then every (row of W, row of x) pair is one vec_dot. */
int orc_mul_mat(int type, const void *w, int64_t K, int64_t N, const float *x, int64_t M, float *y,
                int act, int nthreads) {
    const size_t rb = orc_row_bytes(type, K);
    if (rb == 0) return -1;
    if (nthreads < 1) nthreads = 1;
    if (act == ORC_ACT_F64) {
        double *yd = (double *)malloc((size_t)M * N * sizeof(double));
        if (!yd) return -2;
        orc_mul_mat_f64(type, w, K, N, x, M, yd, nthreads);
        for (int64_t i = 0; i < M * N; ++i) y[i] = (float)yd[i];
        free(yd);
        return 0;
    }
    const size_t ab = act_row_bytes(type, act, K);
    char *aq = (char *)malloc(ab * (size_t)M);
    if (!aq) return -2;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t m = 0; m < M; ++m) quantize_act_row(type, act, x + m * K, aq + (size_t)m * ab, K);
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const void *wrow = (const char *)w + (size_t)n * rb;
        for (int64_t m = 0; m < M; ++m)
            y[m * N + n] = dot_quantized(type, act, K, wrow, aq + (size_t)m * ab);
    }
    free(aq);
    return 0;
}

/* ggml-cpu.c ggml_compute_forward_mul_mat_id: for token b and slot j the row
 * b[b, j % nb1, :] is multiplied by expert ids[b, j]; dst is [B, n_used, N]. */
int orc_mul_mat_id(int type, const void *as, int64_t K, int64_t N, int64_t E, const float *b,
                   int64_t nb1, const int32_t *ids, int64_t n_used, int64_t B, float *y, int act,
                   int nthreads) {
    const size_t rb = orc_row_bytes(type, K);
    if (rb == 0 || (nb1 != 1 && nb1 != n_used)) return -1;
    for (int64_t i = 0; i < B * n_used; ++i)
        if (ids[i] < 0 || ids[i] >= E) return -3;
    const size_t expert_bytes = rb * (size_t)N;
    for (int64_t t = 0; t < B; ++t) {
        for (int64_t j = 0; j < n_used; ++j) {
            const void *we = (const char *)as + (size_t)ids[t * n_used + j] * expert_bytes;
            const float *xr = b + (t * nb1 + (j % nb1)) * K;
            int rc = orc_mul_mat(type, we, K, N, xr, 1, y + (t * n_used + j) * N, act, nthreads);
            if (rc) return rc;
        }
    }
    return 0;
}

/* llama-graph.cpp build_moe_ffn (SiLU-gated, weights applied after down):
 *   up = mul_mat_id(up_exps, x); gate = mul_mat_id(gate_exps, x);
 *   h = silu(gate) * up; e = mul_mat_id(down_exps, h); e *= w; y = e[0] + e[1] + ... */
int orc_moe_ffn(int type_gate_up, int type_down, const void *gate, const void *up, const void *down,
                int64_t d_model, int64_t d_ff, int64_t E, const float *x, const int32_t *ids,
                const float *weights, int64_t n_used, int64_t B, float *y, int act, int nthreads) {
    const size_t n_slot = (size_t)B * n_used;
    float *g = (float *)malloc(n_slot * d_ff * sizeof(float));
    float *u = (float *)malloc(n_slot * d_ff * sizeof(float));
    float *e = (float *)malloc(n_slot * d_model * sizeof(float));
    int rc = -2;
    if (g && u && e) {
        rc = orc_mul_mat_id(type_gate_up, up, d_model, d_ff, E, x, 1, ids, n_used, B, u, act, nthreads);
        if (!rc)
            rc = orc_mul_mat_id(type_gate_up, gate, d_model, d_ff, E, x, 1, ids, n_used, B, g, act,
                                nthreads);
        if (!rc) {
            for (size_t i = 0; i < n_slot * (size_t)d_ff; ++i) {
                const float gv = g[i];
                g[i] = (gv / (1.0f + expf(-gv))) * u[i];
            }
            rc = orc_mul_mat_id(type_down, down, d_ff, d_model, E, g, n_used, ids, n_used, B, e, act,
                                nthreads);
        }
        if (!rc) {
            for (int64_t t = 0; t < B; ++t) {
                for (int64_t c = 0; c < d_model; ++c) {
                    float s = e[(t * n_used + 0) * d_model + c] * weights[t * n_used + 0];
                    for (int64_t j = 1; j < n_used; ++j)
                        s += e[(t * n_used + j) * d_model + c] * weights[t * n_used + j];
                    y[t * d_model + c] = s;
                }
            }
        }
    }
    free(g);
    free(u);
    free(e);
    return rc;
}

/* ---------------------------------------------------------------- timing */

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ---------------------------------------------------------------- AVX2 dot products (CPU baseline timing)
 *
 * ggml's CPU backend does not run the generic C loops above on x86: its ggml-cpu/arch/x86/quants.c holds AVX2
 * forms of the same dot products (unsigned x signed byte products with maddubs, 16-bit pair sums with madd, one
 * float multiply-add per block).  These follow that shape so that the CPU baseline timed beside the GPU is the
 * kind of code the reference's CPU path runs, not scalar C.  Same integers as the generic functions, another
 * order of the float additions; tests hold them to the generic ones within 1e-5.  Never used as the parity
 * reference. */
#if defined(__AVX2__)
static inline float hsum8(__m256 v) {
    __m128 r = _mm_add_ps(_mm256_castps256_ps128(v), _mm256_extractf128_ps(v, 1));
    r = _mm_add_ps(r, _mm_movehl_ps(r, r));
    r = _mm_add_ss(r, _mm_movehdup_ps(r));
    return _mm_cvtss_f32(r);
}

float orc_vec_dot_q8_0_q8_0_avx2(int64_t k, const orc_block_q8_0 *w, const orc_block_q8_0 *a) {
    const int64_t nb = k / ORC_QK8_0;
    __m256 acc = _mm256_setzero_ps();
    const __m256i ones = _mm256_set1_epi16(1);
    for (int64_t ib = 0; ib < nb; ++ib) {
        const __m256 d = _mm256_set1_ps(orc_fp16_to_fp32_f16c(w[ib].d) * orc_fp16_to_fp32_f16c(a[ib].d));
        const __m256i qw = _mm256_loadu_si256((const __m256i *)w[ib].qs);
        const __m256i qa = _mm256_loadu_si256((const __m256i *)a[ib].qs);
        /* |w| * sign(w)(a): unsigned x signed bytes */
        const __m256i p16 = _mm256_maddubs_epi16(_mm256_sign_epi8(qw, qw), _mm256_sign_epi8(qa, qw));
        const __m256i p32 = _mm256_madd_epi16(p16, ones);
        acc = _mm256_fmadd_ps(d, _mm256_cvtepi32_ps(p32), acc);
    }
    return hsum8(acc);
}

float orc_vec_dot_q4_K_q8_K_avx2(int64_t k, const orc_block_q4_K *w, const orc_block_q8_K *a) {
    const int64_t nb = k / ORC_QK_K;
    const __m256i m4 = _mm256_set1_epi8(0xF);
    __m256 acc = _mm256_setzero_ps();
    float acc_m = 0.f;
    for (int64_t i = 0; i < nb; ++i) {
        const float d = a[i].d * orc_fp16_to_fp32_f16c(w[i].d);
        const float dmin = a[i].d * orc_fp16_to_fp32_f16c(w[i].dmin);
        uint8_t sc[8], mn[8];
        for (int j = 0; j < 8; ++j) orc_get_scale_min_k4(j, w[i].scales, &sc[j], &mn[j]);
        int summ = 0;
        for (int j = 0; j < 8; ++j) summ += mn[j] * (a[i].bsums[2 * j] + a[i].bsums[2 * j + 1]);
        acc_m += dmin * (float)summ;
        const uint8_t *q4 = w[i].qs;
        const int8_t *q8 = a[i].qs;
        __m256i sumi = _mm256_setzero_si256();
        for (int j = 0; j < ORC_QK_K / 64; ++j) {
            const __m256i s_l = _mm256_set1_epi16(sc[2 * j]), s_h = _mm256_set1_epi16(sc[2 * j + 1]);
            const __m256i q4b = _mm256_loadu_si256((const __m256i *)q4);
            q4 += 32;
            const __m256i q4l = _mm256_and_si256(q4b, m4);
            const __m256i q4h = _mm256_and_si256(_mm256_srli_epi16(q4b, 4), m4);
            const __m256i q8l = _mm256_loadu_si256((const __m256i *)q8);
            q8 += 32;
            const __m256i q8h = _mm256_loadu_si256((const __m256i *)q8);
            q8 += 32;
            const __m256i p16l = _mm256_madd_epi16(s_l, _mm256_maddubs_epi16(q4l, q8l));
            const __m256i p16h = _mm256_madd_epi16(s_h, _mm256_maddubs_epi16(q4h, q8h));
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(p16l, p16h));
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    return hsum8(acc) - acc_m;
}

float orc_vec_dot_q6_K_q8_K_avx2(int64_t k, const orc_block_q6_K *w, const orc_block_q8_K *a) {
    const int64_t nb = k / ORC_QK_K;
    const __m256i m4 = _mm256_set1_epi8(0xF), m2 = _mm256_set1_epi8(3), m32s = _mm256_set1_epi8(32);
    __m256 acc = _mm256_setzero_ps();
    for (int64_t i = 0; i < nb; ++i) {
        const float d = a[i].d * orc_fp16_to_fp32_f16c(w[i].d);
        const uint8_t *q4 = w[i].ql, *qh = w[i].qh;
        const int8_t *q8 = a[i].qs;
        __m256i sumi = _mm256_setzero_si256();
        for (int j = 0; j < ORC_QK_K / 128; ++j) {
            const __m256i q4b1 = _mm256_loadu_si256((const __m256i *)q4);
            const __m256i q4b2 = _mm256_loadu_si256((const __m256i *)(q4 + 32));
            q4 += 64;
            const __m256i q4bh = _mm256_loadu_si256((const __m256i *)qh);
            qh += 32;
            const __m256i h0 = _mm256_slli_epi16(_mm256_and_si256(q4bh, m2), 4);
            const __m256i h1 = _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(q4bh, 2), m2), 4);
            const __m256i h2 = _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(q4bh, 4), m2), 4);
            const __m256i h3 = _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(q4bh, 6), m2), 4);
            const __m256i q0 = _mm256_or_si256(_mm256_and_si256(q4b1, m4), h0);
            const __m256i q1 = _mm256_or_si256(_mm256_and_si256(q4b2, m4), h1);
            const __m256i q2 = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(q4b1, 4), m4), h2);
            const __m256i q3 = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(q4b2, 4), m4), h3);
            const __m256i qs[4] = {q0, q1, q2, q3};
            for (int g = 0; g < 4; ++g) {
                const __m256i q8v = _mm256_loadu_si256((const __m256i *)q8);
                q8 += 32;
                /* (q - 32) * a = q * a - 32 * a, both as unsigned x signed byte products */
                __m256i p16 = _mm256_sub_epi16(_mm256_maddubs_epi16(qs[g], q8v), _mm256_maddubs_epi16(m32s, q8v));
                /* two sub-blocks of 16 in the 32 bytes: scale is[0] for the low lane, is[1] for the high lane */
                const int is = 8 * j + 2 * g;
                const __m256i sc = _mm256_set_m128i(_mm_set1_epi16(w[i].scales[is + 1]), _mm_set1_epi16(w[i].scales[is]));
                sumi = _mm256_add_epi32(sumi, _mm256_madd_epi16(sc, p16));
            }
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    return hsum8(acc);
}

static float dot_quantized_avx2(int type, int64_t K, const void *wrow, const void *arow) {
    switch (type) {
    case ORC_TYPE_Q8_0:
        return orc_vec_dot_q8_0_q8_0_avx2(K, (const orc_block_q8_0 *)wrow, (const orc_block_q8_0 *)arow);
    case ORC_TYPE_Q4_K:
        return orc_vec_dot_q4_K_q8_K_avx2(K, (const orc_block_q4_K *)wrow, (const orc_block_q8_K *)arow);
    default:
        return orc_vec_dot_q6_K_q8_K_avx2(K, (const orc_block_q6_K *)wrow, (const orc_block_q8_K *)arow);
    }
}
#endif

int orc_has_avx2(void) {
#if defined(__AVX2__)
    return 1;
#else
    return 0;
#endif
}

/* orc_mul_mat in the ggml activation mode with the AVX2 dot products (timing and its cross-check only) */
int orc_mul_mat_avx2(int type, const void *w, int64_t K, int64_t N, const float *x, int64_t M, float *y, int nthreads) {
#if defined(__AVX2__)
    const size_t rb = orc_row_bytes(type, K);
    if (rb == 0) return -1;
    if (nthreads < 1) nthreads = 1;
    const size_t ab = act_row_bytes(type, ORC_ACT_GGML, K);
    char *aq = (char *)malloc(ab * (size_t)M);
    if (!aq) return -2;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t m = 0; m < M; ++m) quantize_act_row(type, ORC_ACT_GGML, x + m * K, aq + (size_t)m * ab, K);
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        const void *wrow = (const char *)w + (size_t)n * rb;
        for (int64_t m = 0; m < M; ++m) y[m * N + n] = dot_quantized_avx2(type, K, wrow, aq + (size_t)m * ab);
    }
    free(aq);
    return 0;
#else
    (void)type; (void)w; (void)K; (void)N; (void)x; (void)M; (void)y; (void)nthreads;
    return -3;
#endif
}

double orc_time_mul_mat_avx2(int type, const void *w, int64_t K, int64_t N, const float *x, int64_t M, float *y,
                             int nthreads, int reps) {
    struct timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (int r = 0; r < reps; ++r)
        if (orc_mul_mat_avx2(type, w, K, N, x, M, y, nthreads) != 0) return -1.0;
    clock_gettime(CLOCK_MONOTONIC, &t1);
    return (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
}

double orc_time_mul_mat(int type, const void *w, int64_t K, int64_t N, const float *x, int64_t M,
                        float *y, int act, int nthreads, int reps) {
    struct timespec t0, t1;
    clock_gettime(CLOCK_MONOTONIC, &t0);
    for (int r = 0; r < reps; ++r) orc_mul_mat(type, w, K, N, x, M, y, act, nthreads);
    clock_gettime(CLOCK_MONOTONIC, &t1);
    return (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec);
}

/* ggml-cpu ops.cpp ggml_compute_forward_rms_norm_f32: the squares are formed in float and summed in
 * ggml_float (double), the mean goes back to float before eps is added, the row is scaled in place
 * (ggml_vec_scale_f32), and the multiplication by the norm weights is a separate GGML_OP_MUL node,
 * i.e. a second rounding. */
void orc_rms_norm(const float *x, const float *gamma, float eps, int64_t M, int64_t K, float *y) {
    for (int64_t m = 0; m < M; ++m) {
        const float *xr = x + m * K;
        float *yr = y + m * K;
        double sum = 0.0;
        for (int64_t k = 0; k < K; ++k) sum += (double)(xr[k] * xr[k]);
        const float mean = (float)(sum / (double)K);
        const float scale = 1.0f / sqrtf(mean + eps);
        for (int64_t k = 0; k < K; ++k) {
            const float v = xr[k] * scale;
            yr[k] = gamma ? v * gamma[k] : v;
        }
    }
}
