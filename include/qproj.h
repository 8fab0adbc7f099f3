/*
 * qproj -- MI355X (gfx950) quantized projection operators behind a plain C ABI.
 *
 * The operators keep the semantics of the two ggml graph ops that Magnitude's
 * engine reaches for every linear layer through its single native call
 *   context.decode(batch)      /root/reference/inference/crates/icn-engine/src/lib.rs:2264
 * (-> llama_decode -> ggml backend graph_compute):
 *   GGML_OP_MUL_MAT    (src0 = W[K,N] quantized, src1 = x[K,M] f32) -> dst[N,M] f32
 *   GGML_OP_MUL_MAT_ID (as = W[K,N,E], b = x[K,n_used|1,B], ids[n_used,B] i32) -> dst[N,n_used,B]
 * over GGML_TYPE_Q8_0 / Q4_K / Q6_K weights.  A ggml backend module is what the
 * reference loads for this work
 *   load_backends_from_path(<installation>/backends)
 *                              /root/reference/inference/crates/icn-server/src/main.rs:5290
 * and each entry point below names the backend-interface member it stands in for.
 *
 * Conventions
 *   - every function returns a qproj_status (0 = ok); nothing aborts or throws across the
 *     boundary, so a host can run its decode-failure recovery
 *     (/root/reference/inference/crates/icn-engine/src/lib.rs:1597-1617);
 *   - weight bytes are handed over on the HOST in GGUF block layout, verbatim, and the
 *     library owns their device copy (ggml buffer set_tensor);
 *   - activations, ids and outputs are DEVICE pointers owned by the caller (ggml tensors
 *     living in backend buffers); all work is enqueued on the context's HIP stream.  Outputs
 *     are ordinary device memory (hipMalloc; not host-coherent or managed allocations): some
 *     launches add their partial results to them with the memory side's float adder (two addends
 *     onto rows cleared beforehand: the sum does not depend on their order; sums below the
 *     smallest normal float are flushed to zero by that adder).  Where that route is taken the
 *     launch that quantizes the activation rows also clears the output rows, so it writes y
 *     before the projection does: outputs must not overlap the activations of the same call.
 *     (The library looks for an overlap where it matters and then takes the route that stores
 *     its results instead; callers should not rely on aliasing all the same.)  The add route
 *     needs 16-byte aligned outputs and is skipped for others;
 *   - a context is used by one thread at a time (the reference serialises native calls on one
 *     executor thread: /root/reference/design/inference/engine.md:49-50).
 *   - row-major, ggml element order: x is [M][K], y is [M][N], W is N rows of K weights.
 */
#ifndef QPROJ_H
#define QPROJ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct qproj_ctx qproj_ctx;
typedef struct qproj_weight qproj_weight;

/* values are ggml's enum ggml_type ids, so a GGUF tensor-info type passes through unchanged
 * (the reference reads them at /root/reference/inference/crates/icn-models/src/gguf.rs:240-279) */
enum qproj_type { QPROJ_TYPE_Q8_0 = 8, QPROJ_TYPE_Q4_K = 12, QPROJ_TYPE_Q6_K = 14 };

enum qproj_status {
    QPROJ_OK = 0,
    QPROJ_ERR_INVALID_ARG = 1, /* null pointer, bad shape, unsupported type                 */
    QPROJ_ERR_HIP = 2,         /* a HIP runtime call failed; see qproj_last_error           */
    QPROJ_ERR_OOM = 3,         /* device allocation failed                                   */
    QPROJ_ERR_UNSUPPORTED = 4, /* valid request this build has no kernel for                */
    QPROJ_ERR_NO_DEVICE = 5    /* no gfx950 device visible                                   */
};

/* How a mul_mat treats its f32 activations.
 *   GGML  : rows are quantized to the weight type's ggml vec_dot_type first (Q8_0 blocks for Q8_0
 *           weights, Q8_K super-blocks for Q4_K/Q6_K) and the dot products are integer, exactly as
 *           ggml's CPU backend computes MUL_MAT.  This is the drop-in mode.
 *   F32   : fp32 activations times dequantized weights, fp32 accumulation (no activation rounding).
 *   Q8X32 : rows are quantized to per-32 int8 blocks with an fp32 scale; int8 MFMA for large M.
 */
enum qproj_act { QPROJ_ACT_GGML = 0, QPROJ_ACT_F32 = 1, QPROJ_ACT_Q8X32 = 2 };

/* ggml_backend_reg / ggml_backend_dev: number of usable gfx950 devices. */
int qproj_device_count(int *count);

/* ggml_backend_dev_init.  `stream` is a hipStream_t to enqueue on, or NULL for a stream the
 * context creates (default priority) and owns. */
int qproj_ctx_create(int device, void *stream, qproj_ctx **out);
int qproj_ctx_destroy(qproj_ctx *ctx);
/* ggml_backend_synchronize */
int qproj_sync(qproj_ctx *ctx);
/* text of the most recent failure on this context ("" if none); never NULL */
const char *qproj_last_error(const qproj_ctx *ctx);
/* the stream work is enqueued on (hipStream_t) */
void *qproj_stream(const qproj_ctx *ctx);

/* bytes of one row of K weights in GGUF layout; 0 if K is not a multiple of the block */
size_t qproj_row_bytes(int type, int64_t K);

/* ggml_backend_buffer set_tensor for a quantized weight: copies n_expert * N rows of K weights
 * (GGUF layout, expert-major) to the device.  Q8_0 and Q6_K blocks are re-laid out into
 * same-size aligned planes on the way; qproj_download returns the original bytes. */
int qproj_upload(qproj_ctx *ctx, int type, int64_t K, int64_t N, int64_t n_expert,
                 const void *gguf_bytes, qproj_weight **out);
/* same, source already on the device (GGUF layout) */
int qproj_upload_from_device(qproj_ctx *ctx, int type, int64_t K, int64_t N, int64_t n_expert,
                             const void *gguf_bytes_dev, qproj_weight **out);
/* ggml_backend_buffer get_tensor: GGUF-layout bytes back to the host */
int qproj_download(qproj_ctx *ctx, const qproj_weight *w, void *gguf_bytes_out);
int qproj_weight_free(qproj_ctx *ctx, qproj_weight *w);
int qproj_weight_info(const qproj_weight *w, int *type, int64_t *K, int64_t *N, int64_t *n_expert,
                      size_t *gguf_bytes);

/* ggml to_float (dequantize_row_*): out_dev = f32 [n_expert*N][K], bit-exact with ggml's
 * dequantize_row_q8_0 / q4_K / q6_K. */
int qproj_dequantize(qproj_ctx *ctx, const qproj_weight *w, float *out_dev);

/* ggml from_float of the activation side (quantize_row_q8_0 / quantize_row_q8_K) or the per-32
 * prefill format, for M rows of K floats.  `kind` = QPROJ_ACT_GGML with `wtype` selecting Q8_0 vs
 * Q8_K, or QPROJ_ACT_Q8X32.  Output planes in `out_dev` (size from qproj_act_bytes):
 *   Q8_0  : int8 qs[M][K] | f32 d[M][K/32]   (d already rounded through fp16)
 *   Q8_K  : int8 qs[M][K] | f32 d[M][K/256] | int16 bsums[M][K/16] | f16 msum[M][K/256][16] | f32 rs[M]
 *           (rs[m]: the largest power of two not above the row's largest |d|, 1 for an all-zero row;
 *           msum: (d / rs[m]) * (sum of the 32 codes of a sub-block) / 16 as an fp16 pair, the 8 high parts of a
 *           super-block, then the 8 low parts: the operand of the tiled kernels' min term, normalised by the row so
 *           that it keeps its 22 bits whatever the size of the activations)
 *   Q8X32 : int8 qs[M][K] | f32 d[M][K/32]  | int32 isum[M][K/32] | f16 msum[M][K/256][16] | f32 rs[M] (as above,
 *           with the per-32 scales and sums)
 * each plane starting at a 256-byte aligned offset, in that order.  K must be a multiple of 32 for Q8_0 and of
 * 256 for Q8_K and Q8X32 (both carry one msum record per 256 weights of a row); qproj_act_bytes returns 0 and
 * qproj_quantize_activations QPROJ_ERR_INVALID_ARG otherwise.  Activations may have any finite size; the weight
 * side of the same term is carried as fp16 pairs of dmin * min, which wants dmin * 63 < 65504 (GGUF files are
 * orders of magnitude inside that). */
size_t qproj_act_bytes(int kind, int wtype, int64_t M, int64_t K);
int qproj_quantize_activations(qproj_ctx *ctx, int kind, int wtype, const float *x_dev, int64_t M,
                               int64_t K, void *out_dev);

/* The two graph nodes llama.cpp puts in front of every attention and feed-forward block (build_norm with
 * LLM_NORM_RMS: GGML_OP_RMS_NORM, then GGML_OP_MUL by the norm weights), reached like everything else here
 * through context.decode (/root/reference/inference/crates/icn-engine/src/lib.rs:2264):
 *   y[m][k] = (x[m][k] * (1 / sqrtf(mean_k(x[m]^2) + eps))) * gamma[k],   mean taken in double.
 * gamma_dev may be null (the norm alone).  K a multiple of 32. */
int qproj_rms_norm(qproj_ctx *ctx, const float *x_dev, const float *gamma_dev, float eps, int64_t M, int64_t K,
                   float *y_dev);

/* qproj_rms_norm followed by qproj_quantize_activations in one launch: the normalised rows go straight from
 * registers into the activation planes (same bytes as the two calls one after the other) and feed
 * qproj_mul_mat_quantized.  The per-32 format needs K % 256 == 0 here. */
int qproj_rms_norm_quantize(qproj_ctx *ctx, int kind, int wtype, const float *x_dev, const float *gamma_dev,
                            float eps, int64_t M, int64_t K, void *out_dev);

/* qproj_rms_norm (gamma_dev may be null) followed by qproj_mul_mat_multi on the normalised rows, the sequence
 * norm -> q/k/v and norm -> gate/up of every transformer block.  One launch where the decode kernel serves
 * (its prologue normalises and quantizes the row: M <= 2 with K <= 16384 / M), otherwise the fused
 * norm + quantizer launch followed by the projection.  Same results as the separate calls. */
int qproj_rms_norm_mul_mat(qproj_ctx *ctx, int n, const qproj_weight *const *w, const float *x_dev,
                           const float *gamma_dev, float eps, int64_t M, float *const *y_dev, int act);

/* The front half of llama.cpp's dense feed-forward (build_ffn with LLM_FFN_SILU, LLM_FFN_PAR: the two MUL_MATs
 * and the swiglu that joins them):  h_dev[M][N] = silu(gate . x) * (up . x),  silu(v) = v / (1 + expf(-v)).
 * gate and up are dense tensors of one shape and type.  One launch for M <= 2 (the decode kernel walks row r
 * of both tensors in the same wave), otherwise qproj_mul_mat_multi into scratch and an elementwise pass.
 * The second form puts qproj_rms_norm (gamma_dev may be null) in front: norm -> gate/up -> swiglu. */
int qproj_ffn_gate_up(qproj_ctx *ctx, const qproj_weight *gate, const qproj_weight *up, const float *x_dev,
                      int64_t M, float *h_dev, int act);
int qproj_rms_norm_ffn_gate_up(qproj_ctx *ctx, const qproj_weight *gate, const qproj_weight *up,
                               const float *x_dev, const float *gamma_dev, float eps, int64_t M, float *h_dev,
                               int act);

/* The whole dense feed-forward of llama.cpp's build_ffn (LLM_FFN_SILU, LLM_FFN_PAR), optionally behind the block's
 * RMS norm (use_norm != 0; gamma_dev may be null):
 *     y_dev[M][N] = down . ( silu(gate . x') * (up . x') ),   x' = rms_norm(x) * gamma or x.
 * gate and up are [K -> d_ff], down is [d_ff -> N].  Bit-identical to qproj_(rms_norm_)ffn_gate_up followed by
 * qproj_mul_mat: two launches for M <= 2; for batches the swiglu is formed inside the quantizer of the down projection
 * (gate and up go to scratch of the context, the intermediate rows are never written as fp32).
 * What is promised end to end in the ggml activation mode: each half agrees with ggml's arithmetic to the last bits
 * of fp32 (the integer dot products are exact, only the order of the fp32 additions differs: 5e-5 relative at most
 * in the tests), and so does the whole - EXCEPT where a code of the re-quantized intermediate sits on a rounding tie.
 * The down projection quantizes h to int8 as ggml does; a value of h that lies within an fp32 rounding of the middle
 * between two codes may round the other way than on the CPU, and one code moves every output of that row by
 * 1/127 of the largest |h| of its 256-wide block times a weight.  Measured over thousands of random cases: none at
 * d_ff = 14336; at d_ff = 256..768 about one case in 500, up to 2e-3 relative in 1 % of its outputs.  That is a
 * property of quantizing twice, the same between any two correct implementations of ggml's arithmetic. */
int qproj_ffn(qproj_ctx *ctx, const qproj_weight *gate, const qproj_weight *up, const qproj_weight *down,
              const float *x_dev, const float *gamma_dev, float eps, int use_norm, int64_t M, float *y_dev, int act);

/* GGML_OP_MUL_MAT: y_dev[M][N] = x_dev[M][K] . W^T.  Picks the decode (M=1), small-batch
 * (M<=16) or prefill kernel from M.  W must have n_expert == 1. */
int qproj_mul_mat(qproj_ctx *ctx, const qproj_weight *w, const float *x_dev, int64_t M, float *y_dev,
                  int act);

/* Several MUL_MATs that share one activation (q/k/v, gate/up) in one launch: y_dev[i] is
 * [M][N_i].  Same results as n separate qproj_mul_mat calls. */
int qproj_mul_mat_multi(qproj_ctx *ctx, int n, const qproj_weight *const *w, const float *x_dev,
                        int64_t M, float *const *y_dev, int act);

/* qproj_mul_mat_multi for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (ggml's backends allocate their
 * compute buffers up front through the graph allocator); it exists for those callers.  Same arguments, same
 * kernels and bit-identical results, but the call's scratch -- the quantized activation planes and the partial
 * results of a K cut into stretches or chunks -- lives in one fixed buffer of QPROJ_NOALLOC_SCRATCH_BYTES inside
 * the library (one copy per GPU, held until the process ends) instead of the context's growable workspace, and the
 * call issues no hipMalloc / hipFree.  A call that needs more answers QPROJ_ERR_INVALID_ARG and launches nothing
 * (qproj_workspace_bytes tells the need beforehand; M <= 2 needs none; the 8B-class shapes fit up to M = 512).
 * The buffer keeps the last call's contents (every byte a kernel reads was written earlier in the same call), so
 * two calls that overlap in time on one GPU would overwrite each other's scratch.  One context cannot do that (its
 * calls are ordered on its stream); a second context could, unseen by either, so the buffer of a GPU belongs to the
 * first context that calls this entry point on it until that context is destroyed, and calls from any other context
 * are refused with QPROJ_ERR_UNSUPPORTED.  A call recorded into a HIP graph must not be replayed while other work of
 * the same context that uses the buffer is in flight on another stream. */
#define QPROJ_NOALLOC_SCRATCH_BYTES (64u << 20)
int qproj_mul_mat_multi_noalloc(qproj_ctx *ctx, int n, const qproj_weight *const *w, const float *x_dev,
                                int64_t M, float *const *y_dev, int act);

/* Scratch bytes qproj_mul_mat_multi reserves for n tensors of `type` with rows N[0..n) sharing K, M activation
 * rows and activation mode `act` (0 for the decode regime, which needs none).  Needs no device: it walks the
 * library's own dispatch for that shape without launching, and checks on the way that every kernel launcher it
 * picks accepts what it is handed out of a buffer of exactly that size (each launcher works out its own demand and
 * refuses less), that the reservation refuses a buffer one byte smaller, and that no launcher which cuts K goes
 * ahead when it is handed no scratch at all; *status (may be null) is QPROJ_OK then.  The figure is an upper bound:
 * matrices that ride in one launch with K whole leave the part reserved for their partial tiles unused. */
size_t qproj_workspace_bytes(int type, int64_t K, int n, const int64_t *N, int64_t M, int act, int *status);

/* The second half of a MUL_MAT on its own: `act_dev` holds M rows already quantized by
 * qproj_quantize_activations(kind, type of w[0], ...).  ggml converts src1 once per MUL_MAT; a
 * caller that feeds one activation to several weights (q/k/v) converts once and calls this. */
int qproj_mul_mat_quantized(qproj_ctx *ctx, int n, const qproj_weight *const *w, const void *act_dev,
                            int kind, int64_t M, float *const *y_dev);

/* GGML_OP_MUL_MAT_ID: ids_dev = int32 [B][n_used]; x_dev = f32 [B][nb1][K] with nb1 in
 * {1, n_used}; y_dev = f32 [B][n_used][N].  Expert ids outside [0, n_expert) are an error
 * reported by the next qproj_sync (the ids live on the device). */
int qproj_mul_mat_id(qproj_ctx *ctx, const qproj_weight *w_exps, const float *x_dev, int64_t nb1,
                     const int32_t *ids_dev, int64_t n_used, int64_t B, float *y_dev, int act);

/* The MoE feed-forward of llama.cpp's build_moe_ffn, fused:
 *   y[b] = sum_j weights[b][j] * down_e( silu(gate_e x_b) * (up_e x_b) ),  e = ids[b][j]
 * x_dev f32 [B][d_model]; ids_dev int32 [B][n_used]; weights_dev f32 [B][n_used];
 * y_dev f32 [B][d_model].  gate/up are [d_model -> d_ff], down is [d_ff -> d_model].
 * The same end-to-end promise as qproj_ffn: gate/up products, swiglu and the weighted sum follow ggml's arithmetic
 * (halves within 5e-5 relative of it), the whole within 1e-3 except where a re-quantized code of the intermediate sits
 * on a rounding tie (see qproj_ffn). */
int qproj_moe_ffn(qproj_ctx *ctx, const qproj_weight *gate_exps, const qproj_weight *up_exps,
                  const qproj_weight *down_exps, const float *x_dev, const int32_t *ids_dev,
                  const float *weights_dev, int64_t n_used, int64_t B, float *y_dev, int act);

/* Backend eligibility probe: what the reference's server asks of a GPU runtime before it offers the
 * backend pack that needs it (/root/reference/inference/crates/icn-server/src/cuda_driver.rs:343-401
 * inspect(): initialise, driver version, device count, one architecture string and one hardware label per
 * device; /root/reference/inference/crates/icn-server/src/backend_eligibility.rs:17-31 maps the outcome to
 * the contract's usable / absent / failed states,
 * /root/reference/inference/crates/icn-contracts/src/bootstrap_protocol.rs:22-39).
 *   usable : at least one gfx950 device; architectures / hardware_labels list every device that reported
 *            an architecture, in ordinal order, each entry NUL-terminated;
 *   absent : the runtime reports no device, or none of the devices is a gfx950 (this library carries
 *            gfx950 code objects only);
 *   failed : the runtime is there and a probe call failed.
 * diagnostic is a single line of at most 240 characters, as the reference bounds its own.
 * Never fails across the boundary: the return value is QPROJ_OK unless out is null. */
enum qproj_eligibility_state { QPROJ_ELIGIBILITY_USABLE = 0, QPROJ_ELIGIBILITY_ABSENT = 1, QPROJ_ELIGIBILITY_FAILED = 2 };
#define QPROJ_PROBE_MAX_DEVICES 16
typedef struct qproj_eligibility {
    int state;                                           /* enum qproj_eligibility_state          */
    int driver_api;                                      /* hipDriverGetVersion                   */
    int runtime_api;                                     /* hipRuntimeGetVersion                  */
    int n_devices;                                       /* entries filled below                  */
    char architectures[QPROJ_PROBE_MAX_DEVICES][32];     /* "gfx950"                              */
    char hardware_labels[QPROJ_PROBE_MAX_DEVICES][256];  /* device name, trimmed                  */
    char runtime_library[1024];                          /* path the HIP runtime was loaded from  */
    char diagnostic[244];                                /* absent / failed: why                  */
} qproj_eligibility;
int qproj_probe_eligibility(qproj_eligibility *out);

/* The routing table of the dispatch (no counterpart in the reference: ggml keeps its kernel selection inside each
 * backend's supports_op / graph_compute; here it can be read and pinned by a test).  Writes into buf, one line a
 * launch, the kernels that qproj_mul_mat_multi (with_norm = 0) or qproj_rms_norm_mul_mat (with_norm = 1) would launch
 * for n matrices of `type` with K columns and N[i] rows against M activation rows in mode `act` - kernel, template
 * instance, tile, grid, cuts of K - and a last line "scratch: <bytes> bytes".  The lines are written by the launchers
 * themselves during a dry run of the code that serves the call; no device is touched.  Returns QPROJ_OK, the status
 * the call would be refused with, or QPROJ_ERR_INVALID_ARG when buf is too small (the text is then cut). */
int qproj_plan_mul_mat(int type, int64_t K, int n, const int64_t *N, int64_t M, int act, int with_norm, char *buf, size_t buf_bytes);
/* The same for qproj_moe_ffn: gate/up experts [n_expert][d_ff][d_model] of gate_type, down experts of down_type,
 * B tokens with n_used experts each. */
int qproj_plan_moe_ffn(int gate_type, int down_type, int64_t d_model, int64_t d_ff, int64_t n_expert, int64_t n_used,
                       int64_t B, char *buf, size_t buf_bytes);

/* library build tag: "qproj-<version>-gfx950" */
const char *qproj_version(void);

#ifdef __cplusplus
}
#endif
#endif
