/*
 * CPU oracle for the quantized projection path (TEST INFRASTRUCTURE ONLY).
 *
 * This library is the checker, never the product: only tests/, the smoke check
 * and the cpu_baseline leg of the benchmark may load it.  The shipped library
 * (libqproj.so) neither links nor calls anything in this directory.
 *
 * What it restates: the arithmetic Magnitude's engine reaches through
 * `context.decode(batch)` (/root/reference/inference/crates/icn-engine/src/lib.rs:2264)
 * -> llama_decode -> ggml CPU backend MUL_MAT / MUL_MAT_ID on Q8_0 / Q4_K / Q6_K
 * weights.  That arithmetic lives in the third-party dependency llama.cpp,
 * pinned at 0b1bad14ff204627636aeb1de22ddcd5acb859d4
 * (/root/reference/inference/native-pin.toml:11-14), whose sources are NOT
 * vendored in the reference checkout.  Every function below therefore restates
 * the published ggml algorithm (file and function names given per function)
 * rather than following a file under /root/reference.
 *
 * Pin status (what independent evidence holds each function in place):
 *   fp16 conversions ............ pinned: exhaustive 65536-value check against
 *                                 numpy float16 and the x86 F16C instructions.
 *   block layouts ............... pinned: sizeof 34/144/210/292, GGUF spec.
 *   get_scale_min_k4 ............ pinned: exhaustive pack/unpack round trip.
 *   dequantize_row_{q8_0,q4_K,q6_K} pinned: closed forms on hand-built blocks
 *                                 and an independent numpy restatement.
 *   quantize_row_q8_0 ........... pinned: fully specified by the benchmark
 *                                 config (d = amax/127 as fp16, q = round(w/d));
 *                                 roundf's half-away-from-zero ties and the zero
 *                                 block by hand-computed vectors.
 *   vec_dot_* integer partials .. pinned: brute force in int64/fp64 from the
 *                                 dequantized values; one-hot and linearity.
 *   quantize_row_q8_K ........... pinned to the published algorithm by hand-computed
 *                                 vectors that a plausible variant fails: half-to-even
 *                                 ties of nearest_int (roundf differs), the -127
 *                                 constant (-128 differs), "first element of the
 *                                 strictly largest magnitude" (last-wins differs),
 *                                 d = 1/iscale bit for bit (-max/127 differs), the
 *                                 clamp at 127, 16-wide block sums.  No reference-held
 *                                 vector exists for it (llama.cpp is not vendored).
 *   Q4_K / Q6_K weight quantizers  NOT PART OF THE ORACLE: weight blocks are inputs of
 *                                 the path.  The tests make them with the format-valid
 *                                 encoders of tests/kquant_encoders.c.
 *   fp32 association in vec_dot . follows ggml's generic C code; ggml's own
 *                                 SIMD paths associate differently, so GPU
 *                                 comparisons use a tolerance, integers exact.
 *   rms_norm (+ weight multiply) . PARITY UNPINNED against ggml (the double-precision
 *                                 sum of float squares and the two roundings of
 *                                 x*scale*weight are recalled from ggml-cpu's
 *                                 ggml_compute_forward_rms_norm_f32 and ggml_mul;
 *                                 no reference-held vector exists); pinned by what
 *                                 the mathematics fixes: closed forms on constant
 *                                 and one-hot rows, scale invariance, fp64 brute force.
 */
#ifndef QPROJ_ORACLE_H
#define QPROJ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_QK8_0 32
#define ORC_QK_K 256
#define ORC_K_SCALE_SIZE 12

/* ggml type ids (ggml.h enum ggml_type) */
#define ORC_TYPE_Q8_0 8
#define ORC_TYPE_Q4_K 12
#define ORC_TYPE_Q6_K 14

/* activation handling of a mul_mat */
#define ORC_ACT_GGML 0  /* quantize x to the weight's vec_dot_type, integer dots (ggml CPU) */
#define ORC_ACT_F64 1   /* dequantize W, exact fp64 dot with fp32 x (ground truth)         */
#define ORC_ACT_Q8X32 2 /* x per-32 int8 + fp32 scale, integer dots (prefill config)      */

typedef uint16_t orc_half;

#pragma pack(push, 1)
typedef struct { orc_half d; int8_t qs[32]; } orc_block_q8_0;                                   /* 34 B  */
typedef struct { orc_half d; orc_half dmin; uint8_t scales[12]; uint8_t qs[128]; } orc_block_q4_K; /* 144 B */
typedef struct { uint8_t ql[128]; uint8_t qh[64]; int8_t scales[16]; orc_half d; } orc_block_q6_K;  /* 210 B */
typedef struct { float d; int8_t qs[256]; int16_t bsums[16]; } orc_block_q8_K;                   /* 292 B */
/* per-32 activation block of the prefill path: fp32 scale, integer sum, 32 int8 */
typedef struct { float d; int32_t isum; int8_t qs[32]; } orc_block_q8x32;                        /* 40 B  */
#pragma pack(pop)

size_t orc_sizeof_block(int type);   /* 34 / 144 / 210, 0 if unknown  */
int orc_block_elems(int type);       /* 32 / 256 / 256                */
size_t orc_row_bytes(int type, int64_t k);

float orc_fp16_to_fp32(orc_half h);
orc_half orc_fp32_to_fp16(float f);
float orc_fp16_to_fp32_f16c(orc_half h); /* hardware cross-check */
orc_half orc_fp32_to_fp16_f16c(float f);

void orc_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m);
void orc_pack_scale_min_k4(const uint8_t sc[8], const uint8_t mn[8], uint8_t out[12]);

void orc_dequantize_row(int type, const void *blocks, float *y, int64_t k);
void orc_dequantize_row_q8_0(const orc_block_q8_0 *x, float *y, int64_t k);
void orc_dequantize_row_q4_K(const orc_block_q4_K *x, float *y, int64_t k);
void orc_dequantize_row_q6_K(const orc_block_q6_K *x, float *y, int64_t k);

/* Q8_0 only (returns -1 otherwise): Q4_K / Q6_K weight blocks are inputs of the path, not made by the oracle */
int orc_quantize_rows(int type, const float *x, void *blocks, int64_t k, int64_t nrows, int nthreads);
void orc_quantize_row_q8_0(const float *x, orc_block_q8_0 *y, int64_t k);
void orc_quantize_row_q8_K(const float *x, orc_block_q8_K *y, int64_t k);
void orc_quantize_row_q8x32(const float *x, orc_block_q8x32 *y, int64_t k);

float orc_vec_dot_q8_0_q8_0(int64_t k, const orc_block_q8_0 *w, const orc_block_q8_0 *a);
float orc_vec_dot_q4_K_q8_K(int64_t k, const orc_block_q4_K *w, const orc_block_q8_K *a);
float orc_vec_dot_q6_K_q8_K(int64_t k, const orc_block_q6_K *w, const orc_block_q8_K *a);
float orc_vec_dot_q8x32(int type, int64_t k, const void *w, const orc_block_q8x32 *a);

/* AVX2 forms of the three dot products in the shape of ggml's x86 path (CPU-baseline timing only; same integers,
 * another order of the float additions) and the mul_mat / timer built on them; orc_has_avx2() tells whether the
 * library was built with them (orc_mul_mat_avx2 returns -3 otherwise). */
int orc_has_avx2(void);
int orc_mul_mat_avx2(int type, const void *w, int64_t K, int64_t N, const float *x, int64_t M, float *y, int nthreads);
double orc_time_mul_mat_avx2(int type, const void *w, int64_t K, int64_t N, const float *x, int64_t M, float *y,
                             int nthreads, int reps);

/* y[m*N + n] = sum_k W[n,k] * x[m*K + k];  W = N rows of K quantized weights. */
int orc_mul_mat(int type, const void *w, int64_t K, int64_t N, const float *x, int64_t M,
                float *y, int act, int nthreads);
/* same, fp64 result (act is ORC_ACT_F64 semantics) */
int orc_mul_mat_f64(int type, const void *w, int64_t K, int64_t N, const float *x, int64_t M,
                    double *y, int nthreads);

/* ggml MUL_MAT_ID: as = E matrices of N x K; b = [B, nb1, K] with nb1 in {1, n_used};
 * ids = [B, n_used]; y = [B, n_used, N]. */
int orc_mul_mat_id(int type, const void *as, int64_t K, int64_t N, int64_t E, const float *b,
                   int64_t nb1, const int32_t *ids, int64_t n_used, int64_t B, float *y, int act,
                   int nthreads);

/* MoE FFN of llama.cpp build_moe_ffn: y[b] = sum_j w[b,j] * down_e( silu(gate_e x_b) * up_e x_b ) */
int orc_moe_ffn(int type_gate_up, int type_down, const void *gate, const void *up, const void *down,
                int64_t d_model, int64_t d_ff, int64_t E, const float *x, const int32_t *ids,
                const float *weights, int64_t n_used, int64_t B, float *y, int act, int nthreads);

/* timing helper for the CPU baseline: seconds for `reps` calls of orc_mul_mat */
double orc_time_mul_mat(int type, const void *w, int64_t K, int64_t N, const float *x, int64_t M,
                        float *y, int act, int nthreads, int reps);
int orc_max_threads(void);

/* GGML_OP_RMS_NORM followed by GGML_OP_MUL with the norm weights (llama.cpp build_norm, LLM_NORM_RMS):
 * per row  sum = sum_k (double)(x[k]*x[k]);  scale = 1/sqrtf((float)(sum/K) + eps);
 *          y[k] = (x[k]*scale) * gamma[k]      (gamma may be NULL: plain RMS_NORM) */
void orc_rms_norm(const float *x, const float *gamma, float eps, int64_t M, int64_t K, float *y);

#ifdef __cplusplus
}
#endif
#endif
