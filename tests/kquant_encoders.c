/*
 * Format-valid Q4_K / Q6_K weight encoders for the tests (TEST INPUT GENERATORS, not an oracle).
 *
 * The projection path never quantizes weights: models arrive as GGUF blocks, and both sides of every parity test
 * consume the same blocks.  These encoders only have to produce valid, reasonably accurate blocks from float
 * matrices so that the tests run on realistic scale / min / code distributions.  They follow the shape of
 * llama.cpp's offline quantizer (a weighted error search per sub-block, 6-bit scales relative to the largest of
 * the super-block, re-quantization with the rounded scales) as recalled, and claim no bit-level agreement with
 * it; nothing pins them to it and no parity claim depends on them.  What the tests do check of them: every block
 * decodes (through the oracle's pinned dequantizer) to within a quality bound of the input, and zero input gives
 * zero blocks.
 */
#include <immintrin.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define QK_K 256
#define ENC_MAX(a, b) ((a) > (b) ? (a) : (b))
#define ENC_MIN(a, b) ((a) < (b) ? (a) : (b))
#define GROUP_MAX_EPS 1e-15f

#pragma pack(push, 1)
typedef struct { uint16_t d, dmin; uint8_t scales[12]; uint8_t qs[128]; } enc_block_q4_K;
typedef struct { uint8_t ql[128]; uint8_t qh[64]; int8_t scales[16]; uint16_t d; } enc_block_q6_K;
#pragma pack(pop)
_Static_assert(sizeof(enc_block_q4_K) == 144, "Q4_K block");
_Static_assert(sizeof(enc_block_q6_K) == 210, "Q6_K block");

static inline uint16_t to_fp16(float f) { return (uint16_t)_cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT); }
static inline float from_fp16(uint16_t h) { return _cvtsh_ss(h); }

/* round half to even through the 2^23 + 2^22 addend */
static inline int nearest_int(float fval) {
    float val = fval + 12582912.f;
    int i;
    memcpy(&i, &val, sizeof(int));
    return (i & 0x007fffff) - 0x00400000;
}

/* six-bit (scale, min) pairs of the eight sub-blocks into the 12-byte field of a Q4_K block */
static void pack_scale_min(const uint8_t sc[8], const uint8_t mn[8], uint8_t out[12]) {
    memset(out, 0, 12);
    for (int j = 0; j < 8; ++j) {
        if (j < 4) {
            out[j] |= sc[j] & 63;
            out[j + 4] |= mn[j] & 63;
        } else {
            out[j + 4] = (uint8_t)((sc[j] & 0xF) | ((mn[j] & 0xF) << 4));
            out[j - 4] |= (uint8_t)((sc[j] >> 4) << 6);
            out[j] |= (uint8_t)((mn[j] >> 4) << 6);
        }
    }
}

static void unpack_scale_min(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* weighted affine fit (scale, min <= 0) of n values onto 0..nmax, refined over nstep+1 candidate inverse scales
 * (the shape of llama.cpp's make_qkx2_quants) */
static float fit_affine_qkx2(int n, int nmax, const float *x, const float *w, uint8_t *L,
                             float *the_min, uint8_t *Laux, float rmin, float rdelta, int nstep) {
    float lo = x[0], hi = x[0];
    float sum_w = w[0];
    float sum_x = sum_w * x[0];
    for (int i = 1; i < n; ++i) {
        if (x[i] < lo) lo = x[i];
        if (x[i] > hi) hi = x[i];
        sum_w += w[i];
        sum_x += w[i] * x[i];
    }
    if (lo > 0) lo = 0;
    if (hi == lo) {
        for (int i = 0; i < n; ++i) L[i] = 0;
        *the_min = -lo;
        return 0.f;
    }
    float iscale = nmax / (hi - lo);
    float scale = 1 / iscale;
    float best = 0;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * (x[i] - lo));
        L[i] = (uint8_t)ENC_MAX(0, ENC_MIN(nmax, l));
        float diff = scale * L[i] + lo - x[i];
        best += w[i] * (diff * diff);
    }
    for (int is = 0; is <= nstep; ++is) {
        iscale = (rmin + rdelta * is + nmax) / (hi - lo);
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * (x[i] - lo));
            l = ENC_MAX(0, ENC_MIN(nmax, l));
            Laux[i] = (uint8_t)l;
            sum_l += w[i] * l;
            sum_l2 += w[i] * l * l;
            sum_xl += w[i] * l * x[i];
        }
        const float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0) {
                this_min = 0;
                this_scale = sum_xl / sum_l2;
            }
            float err = 0;
            for (int i = 0; i < n; ++i) {
                float diff = this_scale * Laux[i] + this_min - x[i];
                err += w[i] * (diff * diff);
            }
            if (err < best) {
                for (int i = 0; i < n; ++i) L[i] = Laux[i];
                best = err;
                scale = this_scale;
                lo = this_min;
            }
        }
    }
    *the_min = -lo;
    return scale;
}

/* Q4_K: eight sub-blocks of 32, six-bit scales and mins relative to the largest of the super-block */
static void encode_row_q4_K(const float *x, enc_block_q4_K *y, int64_t k) {
    const int64_t nb = k / QK_K;
    uint8_t L[QK_K], Laux[32];
    float weights[32], mins[8], scales[8];
    for (int64_t i = 0; i < nb; ++i) {
        float max_scale = 0, max_min = 0;
        for (int j = 0; j < 8; ++j) {
            float sum_x2 = 0;
            for (int l = 0; l < 32; ++l) sum_x2 += x[32 * j + l] * x[32 * j + l];
            const float av_x = sqrtf(sum_x2 / 32);
            for (int l = 0; l < 32; ++l) weights[l] = av_x + fabsf(x[32 * j + l]);
            scales[j] = fit_affine_qkx2(32, 15, x + 32 * j, weights, L + 32 * j, &mins[j], Laux, -1.f,
                                        0.1f, 20);
            if (scales[j] > max_scale) max_scale = scales[j];
            if (mins[j] > max_min) max_min = mins[j];
        }
        const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
        const float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
        uint8_t ls8[8], lm8[8];
        for (int j = 0; j < 8; ++j) {
            int ls = nearest_int(inv_scale * scales[j]);
            int lm = nearest_int(inv_min * mins[j]);
            ls8[j] = (uint8_t)ENC_MIN(63, ls);
            lm8[j] = (uint8_t)ENC_MIN(63, lm);
        }
        pack_scale_min(ls8, lm8, y[i].scales);
        y[i].d = to_fp16(max_scale / 63.f);
        y[i].dmin = to_fp16(max_min / 63.f);
        for (int j = 0; j < 8; ++j) {
            uint8_t sc, m;
            unpack_scale_min(j, y[i].scales, &sc, &m);
            const float d = from_fp16(y[i].d) * sc;
            if (!d) continue;
            const float dm = from_fp16(y[i].dmin) * m;
            for (int ii = 0; ii < 32; ++ii) {
                int l = nearest_int((x[32 * j + ii] + dm) / d);
                l = ENC_MAX(0, ENC_MIN(15, l));
                L[32 * j + ii] = (uint8_t)l;
            }
        }
        uint8_t *q = y[i].qs;
        for (int j = 0; j < QK_K; j += 64) {
            for (int l = 0; l < 32; ++l) q[l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
            q += 32;
        }
        x += QK_K;
    }
}

/* symmetric fit of n values onto -nmax..nmax-1 weighted by x^2 (the shape of llama.cpp's make_qx_quants) */
static float fit_symmetric_qx(int n, int nmax, const float *x, int8_t *L) {
    float max = 0, amax = 0;
    for (int i = 0; i < n; ++i) {
        float ax = fabsf(x[i]);
        if (ax > amax) {
            amax = ax;
            max = x[i];
        }
    }
    if (amax < GROUP_MAX_EPS) {
        for (int i = 0; i < n; ++i) L[i] = 0;
        return 0.f;
    }
    float iscale = -nmax / max;
    float sumlx = 0, suml2 = 0;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * x[i]);
        l = ENC_MAX(-nmax, ENC_MIN(nmax - 1, l));
        L[i] = (int8_t)(l + nmax);
        float w = x[i] * x[i];
        sumlx += w * x[i] * l;
        suml2 += w * l * l;
    }
    float scale = suml2 ? sumlx / suml2 : 0.0f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; ++is) {
        if (is == 0) continue;
        iscale = -(nmax + 0.1f * is) / max;
        sumlx = suml2 = 0;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * x[i]);
            l = ENC_MAX(-nmax, ENC_MIN(nmax - 1, l));
            float w = x[i] * x[i];
            sumlx += w * x[i] * l;
            suml2 += w * l * l;
        }
        if (suml2 > 0 && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; ++i) {
                int l = nearest_int(iscale * x[i]);
                L[i] = (int8_t)(nmax + ENC_MAX(-nmax, ENC_MIN(nmax - 1, l)));
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

/* Q6_K: sixteen sub-blocks of 16, signed 8-bit scales relative to the largest of the super-block */
static void encode_row_q6_K(const float *x, enc_block_q6_K *y, int64_t k) {
    const int64_t nb = k / QK_K;
    int8_t L[QK_K];
    float scales[16];
    for (int64_t i = 0; i < nb; ++i) {
        float max_scale = 0, max_abs_scale = 0;
        for (int ib = 0; ib < 16; ++ib) {
            const float scale = fit_symmetric_qx(16, 32, x + 16 * ib, L + 16 * ib);
            scales[ib] = scale;
            const float a = fabsf(scale);
            if (a > max_abs_scale) {
                max_abs_scale = a;
                max_scale = scale;
            }
        }
        if (max_abs_scale < GROUP_MAX_EPS) {
            memset(&y[i], 0, sizeof(y[i]));
            x += QK_K;
            continue;
        }
        const float iscale = -128.f / max_scale;
        y[i].d = to_fp16(1 / iscale);
        for (int ib = 0; ib < 16; ++ib)
            y[i].scales[ib] = (int8_t)ENC_MIN(127, nearest_int(iscale * scales[ib]));
        for (int j = 0; j < 16; ++j) {
            const float d = from_fp16(y[i].d) * y[i].scales[j];
            if (!d) continue;
            for (int ii = 0; ii < 16; ++ii) {
                int l = nearest_int(x[16 * j + ii] / d);
                l = ENC_MAX(-32, ENC_MIN(31, l));
                L[16 * j + ii] = (int8_t)(l + 32);
            }
        }
        uint8_t *ql = y[i].ql;
        uint8_t *qh = y[i].qh;
        for (int j = 0; j < QK_K; j += 128) {
            for (int l = 0; l < 32; ++l) {
                const uint8_t q1 = L[j + l + 0] & 0xF;
                const uint8_t q2 = L[j + l + 32] & 0xF;
                const uint8_t q3 = L[j + l + 64] & 0xF;
                const uint8_t q4 = L[j + l + 96] & 0xF;
                ql[l + 0] = (uint8_t)(q1 | (q3 << 4));
                ql[l + 32] = (uint8_t)(q2 | (q4 << 4));
                qh[l] = (uint8_t)((L[j + l] >> 4) | ((L[j + l + 32] >> 4) << 2) |
                                  ((L[j + l + 64] >> 4) << 4) | ((L[j + l + 96] >> 4) << 6));
            }
            ql += 64;
            qh += 32;
        }
        x += QK_K;
    }
}

/* float [nrows][k] -> blocks of `type` (12: Q4_K, 14: Q6_K); returns 0, or -1 for another type or a ragged k */
int enc_quantize_rows(int type, const float *x, void *blocks, int64_t k, int64_t nrows, int nthreads) {
    if ((type != 12 && type != 14) || k % QK_K != 0) return -1;
    const size_t rb = (size_t)(k / QK_K) * (type == 12 ? sizeof(enc_block_q4_K) : sizeof(enc_block_q6_K));
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t r = 0; r < nrows; ++r) {
        void *row = (char *)blocks + (size_t)r * rb;
        if (type == 12) encode_row_q4_K(x + r * k, (enc_block_q4_K *)row, k);
        else encode_row_q6_K(x + r * k, (enc_block_q6_K *)row, k);
    }
    return 0;
}
