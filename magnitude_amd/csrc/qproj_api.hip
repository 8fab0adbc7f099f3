// C ABI of the qproj library: contexts, weight upload, operator dispatch.
#include "../../include/qproj.h"

#include <dlfcn.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <mutex>
#include <new>
#include <string>

#include "qproj_internal.h"

using namespace qproj;

namespace qproj {
namespace {
thread_local bool g_dry_run = false;
thread_local size_t g_scratch_shave = 0;    // dry runs only: bytes withheld from what the launchers are told they have
thread_local int g_plan_cuts = 0;           // dry runs only: launches noted that cut K into parts kept in scratch
thread_local std::string *g_plan = nullptr;   // where plan_note writes; null: nobody is listening
}
bool dry_run() { return g_dry_run; }
size_t scratch_shave() { return g_dry_run ? g_scratch_shave : 0; }
void set_dry_run(bool on) { g_dry_run = on; }

void plan_note_cut() { ++g_plan_cuts; }

void plan_note(const char *fmt, ...) {
    if (!g_plan) return;
    char line[384];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(line, sizeof line, fmt, ap);
    va_end(ap);
    g_plan->append(line);
    g_plan->push_back('\n');
}
const char *plan_type_name(int type) {
    return type == kTypeQ4_K ? "Q4_K" : type == kTypeQ6_K ? "Q6_K" : type == kTypeQ8_0 || type == 1008 ? "Q8_0" : "?";
}

int tuning_int(const char *name, int dflt) {
#ifdef QPROJ_TUNING
    const char *e = getenv(name);
    return e && *e ? atoi(e) : dflt;
#else
    (void)name;
    return dflt;
#endif
}
}  // namespace qproj

// Scratch of the allocation-free entry point (qproj_mul_mat_multi_noalloc): quantized activation planes and the
// partial results of a K cut into stretches or chunks.  One copy per GPU the library runs on, held until the
// process ends; its device address is looked up once per device in qproj_ctx_create (the name below is a host-side
// stand-in, never a device address).
static __device__ __align__(256) unsigned char scratch[QPROJ_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_noalloc_mu;                    // guards the two tables below
uint8_t *g_noalloc_ptr[kMaxDevices] = {};   // device address of `scratch` on each device, null until looked up
// The context that uses a device's fixed scratch: the first one to call the allocation-free entry point on the device,
// until it is destroyed.  Two contexts launch on two streams, and their calls would overwrite each other's activation
// planes and partial tiles in the one buffer with no error anywhere; a second context is refused instead.
qproj_ctx *g_noalloc_owner[kMaxDevices] = {};
}  // namespace

struct qproj_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool own_stream = false;
    std::string err;
    uint8_t *ws = nullptr;      // scratch: quantized activations, MoE lists and intermediates
    size_t ws_bytes = 0;
    uint8_t *ws2 = nullptr;     // second scratch: gate and up outputs of the unfused FFN front end
    size_t ws2_bytes = 0;
    int32_t *flag_dev = nullptr;  // raised by kernels that meet bad device-side input
};

struct qproj_weight {
    int type = 0;
    int64_t K = 0, N = 0, E = 0;
    size_t gguf_bytes = 0;
    uint8_t *dev = nullptr;
    size_t dev_bytes = 0;
    WeightView view{};
};

namespace {

constexpr size_t kAlign = 256;
inline size_t align_up(size_t v) { return (v + kAlign - 1) / kAlign * kAlign; }

int fail(qproj_ctx *ctx, int status, const char *what, hipError_t e = hipSuccess) {
    if (ctx) {
        char buf[512];
        if (e != hipSuccess)
            snprintf(buf, sizeof buf, "%s: %s", what, hipGetErrorString(e));
        else
            snprintf(buf, sizeof buf, "%s", what);
        ctx->err = buf;
    }
    return status;
}

#define QP_HIP(ctx, call)                                                         \
    do {                                                                          \
        hipError_t e_ = (call);                                                   \
        if (e_ != hipSuccess) {                                                   \
            (void)hipGetLastError();                                              \
            return fail(ctx, e_ == hipErrorOutOfMemory ? QPROJ_ERR_OOM : QPROJ_ERR_HIP, #call, e_); \
        }                                                                         \
    } while (0)

bool type_ok(int t) { return t == kTypeQ8_0 || t == kTypeQ4_K || t == kTypeQ6_K; }
int block_elems(int t) { return t == kTypeQ8_0 ? 32 : 256; }
size_t block_bytes(int t) { return t == kTypeQ8_0 ? 34 : (t == kTypeQ4_K ? 144 : 210); }

int ensure_ws(qproj_ctx *ctx, size_t bytes) {
    if (bytes <= ctx->ws_bytes) return QPROJ_OK;
    if (ctx->ws) {
        QP_HIP(ctx, hipStreamSynchronize(ctx->stream));
        QP_HIP(ctx, hipFree(ctx->ws));
        ctx->ws = nullptr;
        ctx->ws_bytes = 0;
    }
    const size_t want = align_up(bytes + bytes / 4);
    QP_HIP(ctx, hipMalloc((void **)&ctx->ws, want));
    ctx->ws_bytes = want;
    return QPROJ_OK;
}

// Where an operator call keeps its scratch: the context's growable buffer (reserve may allocate), or a fixed
// buffer that is never grown (the allocation-free entry point).
struct Workspace {
    uint8_t *base;
    size_t cap;
    bool fixed;
    size_t reserved = 0;   // what the call asked for (the largest request)
};

int reserve(qproj_ctx *ctx, Workspace &ws, size_t bytes) {
    ws.reserved = std::max(ws.reserved, bytes);
    if (dry_run() && !ws.fixed) {   // sizes only: any non-null base will do, nothing is dereferenced
        ws.base = reinterpret_cast<uint8_t *>(uintptr_t(256));
        ws.cap = bytes;
        if (ctx) ctx->ws_bytes = std::max(ctx->ws_bytes, bytes);   // (a stand-in context: what the call would have asked for)
        return QPROJ_OK;
    }
    if (ws.fixed) {
        if (bytes > ws.cap) {
            char buf[160];
            snprintf(buf, sizeof buf, "this call needs %zu bytes of scratch, the fixed buffer holds %zu", bytes, ws.cap);
            return fail(ctx, QPROJ_ERR_INVALID_ARG, buf);
        }
        return QPROJ_OK;
    }
    int rc = ensure_ws(ctx, bytes);
    if (rc) return rc;
    ws.base = ctx->ws;
    ws.cap = ctx->ws_bytes;
    return QPROJ_OK;
}

int ensure_ws2(qproj_ctx *ctx, size_t bytes) {
    if (bytes <= ctx->ws2_bytes) return QPROJ_OK;
    if (ctx->ws2) {
        QP_HIP(ctx, hipStreamSynchronize(ctx->stream));
        QP_HIP(ctx, hipFree(ctx->ws2));
        ctx->ws2 = nullptr;
        ctx->ws2_bytes = 0;
    }
    const size_t want = align_up(bytes + bytes / 4);
    QP_HIP(ctx, hipMalloc((void **)&ctx->ws2, want));
    ctx->ws2_bytes = want;
    return QPROJ_OK;
}

// planes of a quantized-activation buffer, in the order the header documents
struct ActPlanes {
    size_t off_qs = 0, off_d = 0, off_aux = 0, off_msum = 0, off_rs = 0, total = 0;
    int kind = 0;
};

int act_kind_for(int act, int wtype) {
    if (act == kActQ8X32) return kActKindQ8X32;
    return wtype == kTypeQ8_0 ? kActKindQ8_0 : kActKindQ8_K;
}

ActPlanes act_planes(int kind, int64_t M, int64_t K) {
    ActPlanes p;
    p.kind = kind;
    p.off_qs = 0;
    p.off_d = align_up((size_t)(M * K));
    const int64_t dblk = kind == kActKindQ8_K ? 256 : 32;
    p.off_aux = p.off_d + align_up((size_t)(M * (K / dblk)) * 4);
    size_t aux = 0;
    if (kind == kActKindQ8_K) aux = (size_t)(M * (K / 16)) * 2;
    if (kind == kActKindQ8X32) aux = (size_t)(M * (K / 32)) * 4;
    p.off_msum = p.off_aux + align_up(aux);
    const bool minterm = kind == kActKindQ8_K || kind == kActKindQ8X32;
    p.off_rs = p.off_msum + (minterm ? align_up((size_t)(M * (K / 256)) * 32) : 0);
    p.total = p.off_rs + (minterm ? align_up((size_t)M * 4) : 0);
    return p;
}

ActView act_view(const ActPlanes &p, uint8_t *base, int64_t K) {
    ActView a{};
    a.kind = p.kind;
    a.K = K;
    a.qs = reinterpret_cast<const int8_t *>(base + p.off_qs);
    a.d = reinterpret_cast<const float *>(base + p.off_d);
    a.bsums = p.kind == kActKindQ8_K ? reinterpret_cast<const int16_t *>(base + p.off_aux) : nullptr;
    a.msum = p.kind == kActKindQ8_K || p.kind == kActKindQ8X32 ? reinterpret_cast<const uint16_t *>(base + p.off_msum) : nullptr;
    a.isum = p.kind == kActKindQ8X32 ? reinterpret_cast<const int32_t *>(base + p.off_aux) : nullptr;
    a.rs = a.msum ? reinterpret_cast<const float *>(base + p.off_rs) : nullptr;
    return a;
}

// the same work as run_quantize (Q8_K planes only), described for the grouping launch to carry
RowQuantJob quantize_job(const ActPlanes &p, uint8_t *base, const float *x, int64_t M, int64_t K) {
    RowQuantJob j{};
    j.x = x;
    j.n_super = M * K / 256;
    j.qs = reinterpret_cast<int8_t *>(base + p.off_qs);
    j.d = reinterpret_cast<float *>(base + p.off_d);
    j.bsums = reinterpret_cast<int16_t *>(base + p.off_aux);
    return j;
}

// minterm: also the min-term plane and the row normalisers that only the tiled Q4_K kernels read (a second, small launch)
hipError_t run_quantize(qproj_ctx *ctx, const ActPlanes &p, uint8_t *base, const float *x, int64_t M, int64_t K,
                        bool minterm = true, const float *swiglu_u = nullptr, const ZeroJob *zero = nullptr) {
    const bool mt = minterm && (p.kind == kActKindQ8_K || p.kind == kActKindQ8X32);
    return launch_quantize_act(p.kind, x, M, K, reinterpret_cast<int8_t *>(base + p.off_qs),
                               reinterpret_cast<float *>(base + p.off_d),
                               reinterpret_cast<int16_t *>(base + p.off_aux),
                               mt ? reinterpret_cast<uint16_t *>(base + p.off_msum) : nullptr,
                               reinterpret_cast<int32_t *>(base + p.off_aux),
                               mt ? reinterpret_cast<float *>(base + p.off_rs) : nullptr, ctx->stream, swiglu_u, zero);
}

ActView act_rows(const ActView &a, int64_t m0) {
    ActView r = a;
    const int64_t dblk = a.kind == kActKindQ8_K ? 256 : 32;
    r.qs = a.qs + m0 * a.K;
    r.d = a.d + m0 * (a.K / dblk);
    if (a.bsums) r.bsums = a.bsums + m0 * (a.K / 16);
    if (a.msum) r.msum = a.msum + m0 * (a.K / 16);
    if (a.rs) r.rs = a.rs + m0;
    if (a.isum) r.isum = a.isum + m0 * (a.K / 32);
    return r;
}

int pow2_ceil(int64_t m) {
    int p = 1;
    while (p < m) p <<= 1;
    return p;
}

int make_view(qproj_weight *w) {
    WeightView &v = w->view;
    v = WeightView{};
    v.type = w->type;
    v.K = w->K;
    v.N = w->N;
    v.E = w->E;
    v.nb = w->K / block_elems(w->type);
    const int64_t rows = w->N * w->E;
    const size_t nblk = (size_t)(rows * v.nb);
    uint8_t *b = w->dev;
    if (w->type == kTypeQ4_K) {
        v.q4k = b;
        w->dev_bytes = nblk * 144;
    } else if (w->type == kTypeQ8_0) {
        v.q8_qs = reinterpret_cast<const int8_t *>(b);
        const size_t o = align_up(nblk * 32);
        v.q8_d = reinterpret_cast<const uint16_t *>(b + o);
        w->dev_bytes = o + nblk * 2;
    } else {
        v.q6_ql = b;
        size_t o = align_up(nblk * 128);
        v.q6_qh = b + o;
        o += align_up(nblk * 64);
        v.q6_sc = reinterpret_cast<const int8_t *>(b + o);
        o += align_up(nblk * 16);
        v.q6_d = reinterpret_cast<const uint16_t *>(b + o);
        w->dev_bytes = o + nblk * 2;
    }
    return QPROJ_OK;
}

size_t planes_bytes(int type, size_t nblk) {
    if (type == kTypeQ4_K) return nblk * 144;
    if (type == kTypeQ8_0) return align_up(nblk * 32) + nblk * 2;
    return align_up(nblk * 128) + align_up(nblk * 64) + align_up(nblk * 16) + nblk * 2;
}

int upload_common(qproj_ctx *ctx, int type, int64_t K, int64_t N, int64_t n_expert, const void *src,
                  bool src_on_device, qproj_weight **out) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    if (!out || !src) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_upload: null argument");
    *out = nullptr;
    if (!type_ok(type)) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_upload: unsupported weight type");
    if (K <= 0 || N <= 0 || n_expert <= 0 || K % block_elems(type) != 0)
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_upload: K must be a positive multiple of the block size");
    if (K > (int64_t)1 << 24 || N * n_expert > (int64_t)1 << 31)
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_upload: shape too large");
    QP_HIP(ctx, hipSetDevice(ctx->device));
    qproj_weight *w = new (std::nothrow) qproj_weight();
    if (!w) return fail(ctx, QPROJ_ERR_OOM, "qproj_upload: host allocation failed");
    w->type = type;
    w->K = K;
    w->N = N;
    w->E = n_expert;
    const size_t nblk = (size_t)(N * n_expert) * (size_t)(K / block_elems(type));
    w->gguf_bytes = nblk * block_bytes(type);
    const size_t dev_bytes = planes_bytes(type, nblk);
    hipError_t e = hipMalloc((void **)&w->dev, dev_bytes);
    if (e != hipSuccess) {
        delete w;
        (void)hipGetLastError();
        return fail(ctx, QPROJ_ERR_OOM, "qproj_upload: hipMalloc", e);
    }
    make_view(w);
    int rc = QPROJ_OK;
    if (type == kTypeQ4_K) {
        e = hipMemcpyAsync(w->dev, src, w->gguf_bytes, src_on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice,
                           ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) rc = fail(ctx, QPROJ_ERR_HIP, "qproj_upload: copy", e);
    } else {
        uint8_t *staging = nullptr;
        const uint8_t *gg = static_cast<const uint8_t *>(src);
        if (!src_on_device) {
            e = hipMalloc((void **)&staging, w->gguf_bytes);
            if (e == hipSuccess) e = hipMemcpyAsync(staging, src, w->gguf_bytes, hipMemcpyHostToDevice, ctx->stream);
            gg = staging;
        }
        if (e == hipSuccess) e = launch_repack_to_planes(type, gg, w->dev, w->view, (int64_t)nblk, ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (staging) (void)hipFree(staging);
        if (e != hipSuccess) rc = fail(ctx, e == hipErrorOutOfMemory ? QPROJ_ERR_OOM : QPROJ_ERR_HIP, "qproj_upload: repack", e);
    }
    if (rc != QPROJ_OK) {
        (void)hipGetLastError();
        (void)hipFree(w->dev);
        delete w;
        return rc;
    }
    *out = w;
    return QPROJ_OK;
}

// dense mul_mat over quantized activations already sitting in `a` (M rows)
bool use_decode_kernel(int type, int64_t M, int64_t K) {
    static const bool off = tuning_int("QPROJ_NO_DECODE_KERNEL", 0) != 0;
    return !off && M <= 4 && decode_kernel_fits(type, pow2_ceil(M), K);
}

bool use_mfma_grouped(int type, int64_t K) {
    static const bool off = tuning_int("QPROJ_NO_MFMA_GEMV", 0) != 0;
    return !off && mfma_grouped_fits(type, K);
}

bool use_mfma_kernel(int type, int64_t M, int64_t K) {
    static const bool off = tuning_int("QPROJ_NO_MFMA_GEMV", 0) != 0;
    // Three and four rows stay on the decode kernel (one launch, quantizer in its prologue; Q4_K holds the four
    // activation rows in registers) for K <= 4096 and for Q8_0 of any K.  Measured at 3 - 4 rows, this kernel ->
    // decode kernel, us: Q4_K 4096x4096 10.8 -> 8.4, gate+up 22.0 -> 20.2; Q6_K 4096 -> 1024 13.1 -> 8.4, 4096 -> 14336
    // 21.2 -> 18.5; Q8_0 4096x4096 13.5 -> 8.7, 4096 -> 14336 21.7 -> 17.4, 8192x8192 25.2 -> 22.6.  Longer rows of
    // the K-quants lose there: Q4_K 14336 -> 4096 17.8 -> 21.9, 8192x8192 16.8 -> 19.1; Q6_K 14336 -> 4096 23.6 -> 24.8.
    static const int forced = tuning_int("QPROJ_MFMA_MIN_M", 0);
    const int min_m = forced > 0 ? forced : ((K <= 4096 || type == kTypeQ8_0) && decode_kernel_fits(type, 4, K)) ? 5 : 3;
    return !off && M >= min_m && mfma_gemv_fits(type, std::min<int64_t>(M, 16), K);
}

// scratch bytes run_dense_q8act needs for M rows against these tensors
size_t per32_scratch_max(int n, const qproj_weight *const *w, int64_t M) {   // the targets run one after the other
    size_t need = 0;
    for (int i = 0; i < n; ++i) need = std::max(need, per32_scratch_bytes(w[i]->K, M, w[i]->N));
    return need;
}

// Rows a pass of the small-batch kernel takes: 16, or 32 once there are more than 16 (the matrix instruction has 32
// token rows either way; more staged rows mean shorter K chunks).  Measured, 16-row passes or tiles -> 32-row
// passes, us: Q4_K 4096 -> 14336 at 17 / 32 rows 27.0 / 27.8 (tiled) -> 20.8 / 22.0, 4096 x 4096 17.4 / 18.1 -> 15.8 / 16.3,
// 14336 -> 4096 34.7 / 34.4 -> 25.4 / 26.0; Q8_0 4096 x 4096 26.1 / 30.2 -> 17.8 / 19.4, at 63 rows 55.8 -> 32.5; Q6_K
// 14336 -> 4096 at 17 / 31 rows 44.0 / 48.1 -> 32.6 / 33.0, at 32 rows 39.9 (tiled) -> 34.0, 4096 x 4096 25.6 / 28.5 -> 17.7 / 18.1.
int64_t small_batch_pass(int type, int64_t M) {
    static const int rows = tuning_int("QPROJ_MFMA_PASS_ROWS", 32) > 16 ? 32 : 16;
    (void)type;
    return M > 16 ? rows : 16;
}

// Which batches take the tiled matrix-core products (weights reused across a tile of tokens, K cut into stretches
// where the grid would leave the chip idle) instead of passes of the 16-row small-batch kernel.  ONE predicate for
// the dispatch and for the scratch sizing: the partial tiles of a K cut into stretches go to scratch that only this
// rule provides.  From the row counts below (Q8_0 with K a multiple of 128).
int tiled_min_m(int type) {
    static const int q4 = std::max(3, tuning_int("QPROJ_TILED_MIN_M_Q4K", 33));
    static const int q6 = std::max(3, tuning_int("QPROJ_TILED_MIN_M_Q6K", 33));
    // (Q8_0 took two 32-row passes up to 63 rows: 8192 -> 3072 at 33 / 63 rows 36.8 / 44.6 us against 27.5 / 27.8 tiled,
    // 14336 -> 4096 49.6 / 60.9 against 40.4 / 41.1; at 17..32 rows the one pass stays ahead, 23.6 - 25.8 against 27.2 - 27.7)
    static const int q8 = std::max(3, tuning_int("QPROJ_TILED_MIN_M_Q8_0", 33));
    return type == kTypeQ4_K ? q4 : type == kTypeQ6_K ? q6 : q8;
}
bool takes_tiled(const qproj_weight *t, int64_t M) {
    // (Q6_K rows beyond 16384 weights: a 32-row pass of the small-batch kernel would stage K in more than eight chunks
    // and add as many partial results - 28672 -> 8192 at 17 / 32 rows: 85.5 / 89.5 us in a pass, 72.9 / 77.7 tiled)
    const bool long_q6 = t->type == kTypeQ6_K && t->K > 16384 && M > 16;
    if (M < tiled_min_m(t->type) && !long_q6) return false;
    return t->type != kTypeQ8_0 || t->K % 128 == 0;
}

size_t dense_scratch_bytes(int n, const qproj_weight *const *w, int64_t M) {
    if (takes_tiled(w[0], M)) {
        if (w[0]->type == kTypeQ8_0) return per32_scratch_max(n, w, M);
        size_t need = 0;
        for (int i = 0; i < n; ++i)
            need = std::max(need, w[0]->type == kTypeQ6_K ? q6k_tile_scratch_bytes(w[i]->K, M, w[i]->N)
                                                          : q4k_tile_scratch_bytes(w[i]->K, M, w[i]->N));
        return need;
    }
    if (!use_mfma_kernel(w[0]->type, M, w[0]->K)) return 0;
    int64_t sum_n = 0, rgs = 0;
    for (int i = 0; i < n; ++i) {
        sum_n += w[i]->N;
        rgs += (w[i]->N + 31) / 32;
    }
    const int64_t pass = small_batch_pass(w[0]->type, M);
    size_t need = mfma_gemv_scratch_bytes(w[0]->type, w[0]->K, std::min<int64_t>(M, pass), sum_n, rgs);
    if (M > pass && M % pass) need = std::max(need, mfma_gemv_scratch_bytes(w[0]->type, w[0]->K, M % pass, sum_n, rgs));
    return need;
}

// true when mul_mat of M fp32 rows goes to the small-batch kernel with the quantizer fused into its
// prologue.  Off unless asked for: every one of the ~200 workgroups repeats the quantization of all M
// rows, which costs more than the separate quantizer launch saves (gate+up, M = 4 / 8 / 16: 22.1 /
// 26.9 / 38.5 us fused against 20.5 / 20.8 / 22.7 us).
bool dense_fuses_quantizer(const qproj_weight *w, int64_t M) {
    static const bool on = tuning_int("QPROJ_FUSED_QUANT_DENSE", 0) != 0;
    return on && M <= 16 && use_mfma_kernel(w->type, M, w->K);
}

// The quantizer launch in front of the small-batch kernel clears the output rows where a pass of that kernel cuts K
// in two chunks: the chunks then add themselves to the output and the launch that summed them goes (8B down
// projection, 14336 -> 4096 Q6_K, at 4 and 8 rows).  Fills `z` and answers true when that is the case.
// true when [a, a + na) and [b, b + nb) (floats) share an address
bool overlaps(const float *a, int64_t na, const float *b, int64_t nb) {
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), a1 = a0 + (uintptr_t)na * 4, b0 = reinterpret_cast<uintptr_t>(b), b1 = b0 + (uintptr_t)nb * 4;
    return a0 < b1 && b0 < a1;
}

// (x: the rows the quantizer launch reads, M x K floats.  Output rows that overlap them cannot be cleared by that launch -
// some workgroups would zero what others have yet to read - so such a call keeps the route that stores.)
bool dense_clears_rows(int n, const qproj_weight *const *w, int64_t M, float *const *y, const float *x, ZeroJob &z) {
    if (takes_tiled(w[0], M) || !use_mfma_kernel(w[0]->type, M, w[0]->K)) return false;
    int64_t rgs = 0;
    for (int i = 0; i < n; ++i) rgs += (w[i]->N + 31) / 32;
    const int64_t pass = small_batch_pass(w[0]->type, M);
    bool any = mfma_gemv_two_chunks(w[0]->type, w[0]->K, std::min<int64_t>(M, pass), rgs);
    if (M > pass && M % pass) any = any || mfma_gemv_two_chunks(w[0]->type, w[0]->K, M % pass, rgs);
    if (!any) return false;
    z.count = n;
    for (int i = 0; i < n; ++i) {
        z.p[i] = y[i];
        z.n[i] = M * w[i]->N;
        if (z.n[i] % 4 != 0 || (reinterpret_cast<uintptr_t>(y[i]) & 15) != 0) return false;
        if (overlaps(y[i], z.n[i], x, M * w[0]->K)) return false;
    }
    return true;
}

// The same for the tiled Q4_K kernels: the matrices of the call whose launch cuts K in exactly two stretches get their
// output rows cleared by the quantizer launch, and the stretches add themselves (no partial tiles, no adding pass).
// Returns the mask of those matrices and fills `z` with their rows.
uint32_t tiled_clears_rows(int n, const qproj_weight *const *w, int64_t M, float *const *y, const float *x, bool have_scratch, ZeroJob &z) {
    WeightView views[kMaxTargets];
    for (int i = 0; i < n; ++i) views[i] = w[i]->view;
    uint32_t mask = q4k_multi_adds(n, views, M, have_scratch);
    z.count = 0;
    for (int i = 0; i < n; ++i) {
        if (!((mask >> i) & 1u)) continue;
        const int64_t cnt = M * w[i]->N;
        if (cnt % 4 != 0 || (reinterpret_cast<uintptr_t>(y[i]) & 15) != 0 || overlaps(y[i], cnt, x, M * w[0]->K)) {
            mask &= ~(1u << i);
            continue;
        }
        z.p[z.count] = y[i];
        z.n[z.count] = cnt;
        ++z.count;
    }
    return mask;
}

// x_f32: non-null when `a` carries no planes and the kernel quantizes these rows itself (small batches only);
// y_zeroed: the output rows were cleared by the quantizer launch (dense_clears_rows)
int run_dense_q8act(qproj_ctx *ctx, int n, const qproj_weight *const *w, const ActView &a, int64_t M,
                    float *const *y, const Scratch &sc, const float *x_f32 = nullptr, bool y_zeroed = false) {
    // Beyond the rows one pass of the small-batch kernel takes: the tiled product, weights reused across a tile of
    // tokens, K cut into stretches where the grid would leave the chip idle.  (Measured, 8B shapes, 33 rows: Q6_K
    // 14336 -> 4096 50.9 us in two passes of the small-batch kernel against 41 us tiled, Q4_K 4096 -> 14336 42 against 29.)
    const auto tiled = [&](const qproj_weight *t) { return takes_tiled(t, M); };
    if (tiled(w[0])) {
        if (w[0]->type == kTypeQ4_K && n >= 2 && n <= 3) {   // q/k/v, gate/up: one launch where the tiles allow it
            WeightView views[3];
            for (int i = 0; i < n; ++i) views[i] = w[i]->view;
            QP_HIP(ctx, launch_gemm_q8k_multi(n, views, a, M, y, sc, ctx->stream));
            return QPROJ_OK;
        }
        for (int i = 0; i < n; ++i) {
            const int t = w[0]->type;
            QP_HIP(ctx, t == kTypeQ4_K   ? launch_gemm_q8k(w[i]->view, a, M, y[i], sc.for_target(i), ctx->stream)
                        : t == kTypeQ6_K ? launch_gemm_q6k_q8k(w[i]->view, a, M, y[i], sc, ctx->stream)
                                         : launch_gemm_q8_0(w[i]->view, a, M, y[i], sc, ctx->stream));
        }
        return QPROJ_OK;
    }
    if (use_mfma_kernel(w[0]->type, M, w[0]->K)) {
        const int64_t pass = small_batch_pass(w[0]->type, M);
        for (int64_t m0 = 0; m0 < M; m0 += pass) {
            const int64_t mc = std::min<int64_t>(pass, M - m0);
            GemvArgs g{};
            g.n_targets = n;
            for (int i = 0; i < n; ++i) {
                g.t[i].w = w[i]->view;
                g.t[i].y = y[i] + m0 * w[i]->N;
            }
            g.a = x_f32 ? a : act_rows(a, m0);
            g.x = x_f32;   // (only with M <= 16: a single pass)
            g.M = (int)mc;
            g.x_div = 1;
            g.y_zeroed = y_zeroed;
            QP_HIP(ctx, launch_gemv_mfma(g, sc, ctx->stream));
        }
        return QPROJ_OK;
    }
    if (use_decode_kernel(w[0]->type, M, w[0]->K)) {
        GemvArgs g{};
        g.n_targets = n;
        for (int i = 0; i < n; ++i) {
            g.t[i].w = w[i]->view;
            g.t[i].y = y[i];
        }
        g.a = a;
        g.M = (int)M;
        g.x_div = 1;
        QP_HIP(ctx, launch_gemv_decode(g, pow2_ceil(M), false, ctx->stream));
        return QPROJ_OK;
    }
    for (int64_t m0 = 0; m0 < M; m0 += 16) {
        const int64_t mc = std::min<int64_t>(16, M - m0);
        GemvArgs g{};
        g.n_targets = n;
        for (int i = 0; i < n; ++i) {
            g.t[i].w = w[i]->view;
            g.t[i].y = y[i] + m0 * w[i]->N;
        }
        g.a = act_rows(a, m0);
        g.M = (int)mc;
        g.x_div = 1;
        QP_HIP(ctx, launch_gemv_q8act(g, pow2_ceil(mc), 1, ctx->stream));
    }
    return QPROJ_OK;
}

// the grouped matrix-core kernel quantizes its own activation rows when an expert has few of them
// (every workgroup of the expert repeats that work): two launches less per MoE layer, 40.5 -> 33.7 us
// at one token, 73 -> 68 us at eight, no difference any more at four pairs an expert
bool grouped_fuses_quantizer(int type, int64_t K, int64_t n_pairs, int64_t E) {
    static const bool on = tuning_int("QPROJ_NO_FUSED_QUANT", 0) == 0;
    return on && use_mfma_grouped(type, K) && n_pairs <= 2 * E;
}

// a handful of pairs (one or two decode tokens): no grouping pass, a set of workgroups per pair; an expert
// that does come twice is simply read twice
bool grouped_pair_mode(int type, int64_t K, int64_t n_pairs, int64_t E) {
    static const bool on = tuning_int("QPROJ_NO_PAIR_MODE", 0) == 0;
    return on && grouped_fuses_quantizer(type, K, n_pairs, E) && n_pairs <= 16;
}

// A few decode tokens: the vector-ALU kernel that reads an expert once per PAIR and needs no grouping, quantizer
// or combine launch.  Measured against the grouped route (128 experts, top-8, 2048 x 768, per call): 20.8 -> 15.0 us
// at one token, 24.9 -> 18.8 at two, 41.0 -> 23.2 at four, 57.6 -> 36.2 at eight, 74.1 -> 58.9 at sixteen, 86.0 -> 73.7 at
// twenty, 91.2 -> 84.2 at twenty-four, worse from 28 tokens on (97.6 against 92.8 us; 32: 101 against 95): with more pairs
// than experts the repeated reads of an expert come to outweigh the launches saved.  So: as many pairs as experts
// whatever the expert's size, half as many again while an expert matrix is small (two million weights at most), 256 pairs at most.
// (Up to 16 pairs take it whatever the expert count while an expert matrix is small: launches weigh more than bytes
// there.  Large experts do not: 8 experts of 4096 x 14336, 16 pairs: 214 us grouped, 220 us this way.)
bool moe_decode_route(int type, int64_t K, int64_t N, int64_t n_pairs, int64_t group, int64_t E) {
    static const bool on = tuning_int("QPROJ_NO_MOE_DECODE", 0) == 0;
    // (one workgroup set a pair fills the chip at 256 pairs; 256 experts, top-8, 2048 x 512: 28 / 32 tokens 95.2 / 97.4 us
    // grouped, 77.2 / 79.1 this way; 40 tokens, 320 pairs, 103.6 against 109.8)
    static const int max_pairs = tuning_int("QPROJ_MOE_DECODE_MAX_PAIRS", 256);
    static const int per_4_experts = tuning_int("QPROJ_MOE_DECODE_PAIRS_PER_4_EXPERTS", 4);
    const bool small_expert = K * N <= ((int64_t)2 << 20);
    const bool few = n_pairs <= 16 && small_expert;
    const int64_t per4 = per_4_experts + (small_expert ? per_4_experts / 2 : 0);
    return on && (few || (n_pairs <= max_pairs && 4 * n_pairs <= per4 * E)) && moe_decode_fits(type, K, N, n_pairs, group, E);
}

// Expert rows too long for the staged rows of the grouped matrix-core kernel (K > 4096): from `min_mt` pairs an expert
// on (the rows a pass of the plain grouped kernel would take) that kernel walks K in chunks and a pass adds the chunks'
// results; below, the plain grouped kernel on the vector ALU.  8 experts, top-2, 4096 x 14336 (the down projection is
// the long one), per call, plain kernel -> chunks: 219 -> 189 us at 8 tokens, 270 -> 184 at 16, 409 -> 254 at 32,
// 1231 -> 352 at 64.
int grouped_mt(int64_t n_pairs, int64_t E);
bool grouped_long_rows(const qproj_weight *w, int64_t n_pairs) {
    static const int min_mt = tuning_int("QPROJ_GROUPED_LONG_MIN_MT", 2);
    return min_mt > 0 && !use_mfma_grouped(w->type, w->K) && grouped_mt(n_pairs, w->E) >= min_mt &&
           mfma_grouped_chunked_fits(w->type, w->K, w->N, n_pairs);
}

int grouped_mt(int64_t n_pairs, int64_t E) {
    if (n_pairs * 4 <= E) return 1;
    if (n_pairs <= E) return 2;
    if (n_pairs <= 4 * E) return 4;
    if (n_pairs <= 8 * E) return 8;
    return 16;
}

}  // namespace

extern "C" {

const char *qproj_version(void) { return "qproj-0.1-gfx950"; }

int qproj_probe_eligibility(qproj_eligibility *out) {
    if (!out) return QPROJ_ERR_INVALID_ARG;
    memset(out, 0, sizeof(*out));
    auto say = [&](int state, const char *what, hipError_t e) {
        out->state = state;
        char line[512];
        if (e != hipSuccess) snprintf(line, sizeof(line), "%s: %s", what, hipGetErrorString(e));
        else snprintf(line, sizeof(line), "%s", what);
        size_t n = 0;
        for (const char *c = line; *c && n < 240; ++c) out->diagnostic[n++] = (*c == '\r' || *c == '\n') ? ' ' : *c;
        out->diagnostic[n] = 0;
        (void)hipGetLastError();
        return QPROJ_OK;
    };
    Dl_info info;
    if (dladdr(reinterpret_cast<const void *>(&hipInit), &info) != 0 && info.dli_fname)
        snprintf(out->runtime_library, sizeof(out->runtime_library), "%s", info.dli_fname);
    hipError_t e = hipInit(0);
    if (e == hipErrorNoDevice) return say(QPROJ_ELIGIBILITY_ABSENT, "no HIP device is available", hipSuccess);
    if (e != hipSuccess) return say(QPROJ_ELIGIBILITY_FAILED, "HIP initialisation failed", e);
    const hipError_t ev = hipDriverGetVersion(&out->driver_api);
    (void)hipRuntimeGetVersion(&out->runtime_api);
    int count = 0;
    const hipError_t ec = hipGetDeviceCount(&count);
    if (ec == hipErrorNoDevice || (ec == hipSuccess && count <= 0))
        return say(QPROJ_ELIGIBILITY_ABSENT, "no HIP device is available", hipSuccess);
    if (ev != hipSuccess || ec != hipSuccess || out->driver_api <= 0)
        return say(QPROJ_ELIGIBILITY_FAILED, "HIP probe failed (driver version / device count)", ev != hipSuccess ? ev : ec);
    bool native = false;
    for (int i = 0; i < count && out->n_devices < QPROJ_PROBE_MAX_DEVICES; ++i) {
        hipDeviceProp_t p;
        if (hipGetDeviceProperties(&p, i) != hipSuccess || p.gcnArchName[0] == 0) continue;
        char *arch = out->architectures[out->n_devices];
        size_t n = 0;   // "gfx950:sramecc+:xnack-" -> "gfx950"
        while (p.gcnArchName[n] && p.gcnArchName[n] != ':' && n < 31) { arch[n] = p.gcnArchName[n]; ++n; }
        arch[n] = 0;
        native = native || strcmp(arch, "gfx950") == 0;
        const char *b = p.name;
        while (*b == ' ') ++b;
        size_t len = strlen(b);
        while (len > 0 && b[len - 1] == ' ') --len;
        if (len > 255) len = 255;
        memcpy(out->hardware_labels[out->n_devices], b, len);
        out->n_devices++;
    }
    (void)hipGetLastError();
    if (out->n_devices == 0) return say(QPROJ_ELIGIBILITY_FAILED, "HIP devices did not report an architecture", hipSuccess);
    if (!native) return say(QPROJ_ELIGIBILITY_ABSENT, "no gfx950 device is available", hipSuccess);
    out->state = QPROJ_ELIGIBILITY_USABLE;
    return QPROJ_OK;
}

int qproj_device_count(int *count) {
    if (!count) return QPROJ_ERR_INVALID_ARG;
    *count = 0;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return QPROJ_ERR_NO_DEVICE;
    }
    int ok = 0;
    for (int i = 0; i < n; ++i) {
        hipDeviceProp_t p;
        if (hipGetDeviceProperties(&p, i) == hipSuccess && strncmp(p.gcnArchName, "gfx950", 6) == 0) ok++;
    }
    *count = ok;
    return ok > 0 ? QPROJ_OK : QPROJ_ERR_NO_DEVICE;
}

int qproj_ctx_create(int device, void *stream, qproj_ctx **out) {
    if (!out) return QPROJ_ERR_INVALID_ARG;
    *out = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return QPROJ_ERR_NO_DEVICE;
    }
    if (device < 0 || device >= n) return QPROJ_ERR_INVALID_ARG;
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, device) != hipSuccess) return QPROJ_ERR_HIP;
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0) return QPROJ_ERR_NO_DEVICE;  // kernels exist for gfx950 only
    qproj_ctx *ctx = new (std::nothrow) qproj_ctx();
    if (!ctx) return QPROJ_ERR_OOM;
    ctx->device = device;
    if (hipSetDevice(device) != hipSuccess) {
        delete ctx;
        return QPROJ_ERR_HIP;
    }
    if (stream) {
        ctx->stream = static_cast<hipStream_t>(stream);
    } else {
        if (hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking) != hipSuccess) {
            delete ctx;
            return QPROJ_ERR_HIP;
        }
        ctx->own_stream = true;
    }
    // the fixed scratch of the allocation-free entry point: each device holds its own copy at its own address
    if (device < kMaxDevices) {
        std::lock_guard<std::mutex> lock(g_noalloc_mu);
        if (!g_noalloc_ptr[device]) {
            void *ptr = nullptr;
            if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
                (void)hipGetLastError();
                if (ctx->own_stream) (void)hipStreamDestroy(ctx->stream);
                delete ctx;
                return QPROJ_ERR_HIP;
            }
            g_noalloc_ptr[device] = static_cast<uint8_t *>(ptr);
        }
    }
    if (hipMalloc((void **)&ctx->flag_dev, 256) != hipSuccess ||
        hipMemsetAsync(ctx->flag_dev, 0, 256, ctx->stream) != hipSuccess ||
        hipStreamSynchronize(ctx->stream) != hipSuccess) {
        if (ctx->own_stream) (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return QPROJ_ERR_HIP;
    }
    *out = ctx;
    return QPROJ_OK;
}

int qproj_ctx_destroy(qproj_ctx *ctx) {
    if (!ctx) return QPROJ_OK;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->device >= 0 && ctx->device < kMaxDevices) {   // the device's fixed scratch is free for another context again
        std::lock_guard<std::mutex> lock(g_noalloc_mu);
        if (g_noalloc_owner[ctx->device] == ctx) g_noalloc_owner[ctx->device] = nullptr;
    }
    if (ctx->ws) (void)hipFree(ctx->ws);
    if (ctx->ws2) (void)hipFree(ctx->ws2);
    if (ctx->flag_dev) (void)hipFree(ctx->flag_dev);
    if (ctx->own_stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return QPROJ_OK;
}

int qproj_sync(qproj_ctx *ctx) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    QP_HIP(ctx, hipSetDevice(ctx->device));
    int32_t flag = 0;
    QP_HIP(ctx, hipMemcpyAsync(&flag, ctx->flag_dev, sizeof flag, hipMemcpyDeviceToHost, ctx->stream));
    QP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (flag) {
        QP_HIP(ctx, hipMemsetAsync(ctx->flag_dev, 0, sizeof flag, ctx->stream));
        QP_HIP(ctx, hipStreamSynchronize(ctx->stream));
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "expert id outside [0, n_expert) in a MUL_MAT_ID batch");
    }
    return QPROJ_OK;
}

const char *qproj_last_error(const qproj_ctx *ctx) { return ctx ? ctx->err.c_str() : "null context"; }

void *qproj_stream(const qproj_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

size_t qproj_row_bytes(int type, int64_t K) {
    if (!type_ok(type) || K <= 0 || K % block_elems(type) != 0) return 0;
    return (size_t)(K / block_elems(type)) * block_bytes(type);
}

int qproj_upload(qproj_ctx *ctx, int type, int64_t K, int64_t N, int64_t n_expert, const void *gguf_bytes,
                 qproj_weight **out) {
    return upload_common(ctx, type, K, N, n_expert, gguf_bytes, false, out);
}

int qproj_upload_from_device(qproj_ctx *ctx, int type, int64_t K, int64_t N, int64_t n_expert,
                             const void *gguf_bytes_dev, qproj_weight **out) {
    return upload_common(ctx, type, K, N, n_expert, gguf_bytes_dev, true, out);
}

int qproj_download(qproj_ctx *ctx, const qproj_weight *w, void *out) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    if (!w || !out) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_download: null argument");
    QP_HIP(ctx, hipSetDevice(ctx->device));
    if (w->type == kTypeQ4_K) {
        QP_HIP(ctx, hipMemcpyAsync(out, w->dev, w->gguf_bytes, hipMemcpyDeviceToHost, ctx->stream));
        QP_HIP(ctx, hipStreamSynchronize(ctx->stream));
        return QPROJ_OK;
    }
    uint8_t *staging = nullptr;
    QP_HIP(ctx, hipMalloc((void **)&staging, w->gguf_bytes));
    const int64_t nblk = w->N * w->E * w->view.nb;
    hipError_t e = launch_repack_to_gguf(w->type, w->view, staging, nblk, ctx->stream);
    if (e == hipSuccess) e = hipMemcpyAsync(out, staging, w->gguf_bytes, hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    (void)hipFree(staging);
    if (e != hipSuccess) return fail(ctx, QPROJ_ERR_HIP, "qproj_download", e);
    return QPROJ_OK;
}

int qproj_weight_free(qproj_ctx *ctx, qproj_weight *w) {
    if (!w) return QPROJ_OK;
    if (ctx) {
        (void)hipSetDevice(ctx->device);
        (void)hipStreamSynchronize(ctx->stream);
    }
    if (w->dev) (void)hipFree(w->dev);
    delete w;
    return QPROJ_OK;
}

int qproj_weight_info(const qproj_weight *w, int *type, int64_t *K, int64_t *N, int64_t *n_expert,
                      size_t *gguf_bytes) {
    if (!w) return QPROJ_ERR_INVALID_ARG;
    if (type) *type = w->type;
    if (K) *K = w->K;
    if (N) *N = w->N;
    if (n_expert) *n_expert = w->E;
    if (gguf_bytes) *gguf_bytes = w->gguf_bytes;
    return QPROJ_OK;
}

int qproj_dequantize(qproj_ctx *ctx, const qproj_weight *w, float *out_dev) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    if (!w || !out_dev) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_dequantize: null argument");
    QP_HIP(ctx, hipSetDevice(ctx->device));
    QP_HIP(ctx, launch_dequantize(w->view, out_dev, ctx->stream));
    return QPROJ_OK;
}

size_t qproj_act_bytes(int kind, int wtype, int64_t M, int64_t K) {
    if (M <= 0 || K <= 0) return 0;
    if (kind != kActGGML && kind != kActQ8X32) return 0;
    const int k = act_kind_for(kind, wtype);
    // The per-32 format carries one min-term record (msum) per 256 weights of a row, like Q8_K, and its quantizer
    // walks 256 floats at a time: K must be a whole number of super-blocks for both.
    if (K % (k == kActKindQ8_0 ? 32 : 256) != 0) return 0;
    return act_planes(k, M, K).total;
}

int qproj_quantize_activations(qproj_ctx *ctx, int kind, int wtype, const float *x_dev, int64_t M, int64_t K,
                               void *out_dev) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    if (!x_dev || !out_dev) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_quantize_activations: null argument");
    if (qproj_act_bytes(kind, wtype, M, K) == 0)
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_quantize_activations: bad kind or shape");
    QP_HIP(ctx, hipSetDevice(ctx->device));
    const ActPlanes p = act_planes(act_kind_for(kind, wtype), M, K);
    QP_HIP(ctx, run_quantize(ctx, p, static_cast<uint8_t *>(out_dev), x_dev, M, K));
    return QPROJ_OK;
}

int qproj_rms_norm(qproj_ctx *ctx, const float *x_dev, const float *gamma_dev, float eps, int64_t M, int64_t K,
                   float *y_dev) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    if (!x_dev || !y_dev) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_rms_norm: null argument");
    if (M < 0 || K <= 0 || K % 32 != 0) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_rms_norm: K must be a positive multiple of 32");
    QP_HIP(ctx, hipSetDevice(ctx->device));
    QP_HIP(ctx, launch_rms_norm(-1, x_dev, gamma_dev, eps, M, K, y_dev, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, ctx->stream));
    return QPROJ_OK;
}

int qproj_rms_norm_quantize(qproj_ctx *ctx, int kind, int wtype, const float *x_dev, const float *gamma_dev, float eps,
                            int64_t M, int64_t K, void *out_dev) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    if (!x_dev || !out_dev) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_rms_norm_quantize: null argument");
    if (qproj_act_bytes(kind, wtype, M, K) == 0)
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_rms_norm_quantize: bad kind or shape");
    const int k = act_kind_for(kind, wtype);
    if (k == kActKindQ8X32 && K % 256 != 0)
        return fail(ctx, QPROJ_ERR_UNSUPPORTED, "qproj_rms_norm_quantize: the per-32 format needs K % 256 == 0 here");
    QP_HIP(ctx, hipSetDevice(ctx->device));
    const ActPlanes p = act_planes(k, M, K);
    uint8_t *base = static_cast<uint8_t *>(out_dev);
    const bool mt = k == kActKindQ8_K || k == kActKindQ8X32;
    QP_HIP(ctx, launch_rms_norm(k, x_dev, gamma_dev, eps, M, K, nullptr, reinterpret_cast<int8_t *>(base + p.off_qs),
                                reinterpret_cast<float *>(base + p.off_d), reinterpret_cast<int16_t *>(base + p.off_aux),
                                mt ? reinterpret_cast<uint16_t *>(base + p.off_msum) : nullptr,
                                reinterpret_cast<int32_t *>(base + p.off_aux),
                                mt ? reinterpret_cast<float *>(base + p.off_rs) : nullptr, ctx->stream));
    return QPROJ_OK;
}

namespace {
struct NormSpec {   // RMS norm (+ weights) applied to the rows before they are used
    const float *gamma;
    float eps;
};
}  // namespace

// Can the down projection of a feed-forward block take its rows as silu(gate) * up through the quantizer?  Only the
// routes that quantize in a launch of their own (not the decode kernel, whose prologue reads fp32 rows, nor the
// small-batch variant that quantizes inside the projection, nor fp32 activations).
static bool swiglu_quantizer_serves(const qproj_weight *w, int64_t M, int act) {
    if (act != kActGGML && act != kActQ8X32) return false;
    if (act == kActQ8X32) return w->type == kTypeQ4_K && w->K % 256 == 0;
    if (!use_mfma_kernel(w->type, M, w->K) && use_decode_kernel(w->type, M, w->K)) return false;
    return !dense_fuses_quantizer(w, M);
}

// swiglu_u non-null (callers: the quantized routes beyond the decode regime only): the rows multiplied are
// silu(x_dev) * swiglu_u, formed inside the quantizer
static int mul_mat_multi_impl(qproj_ctx *ctx, int n, const qproj_weight *const *w, const float *x_dev, int64_t M,
                              float *const *y_dev, int act, const NormSpec *norm, Workspace &wsp,
                              const float *swiglu_u = nullptr) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    if (n <= 0 || n > kMaxTargets || !w || !y_dev || !x_dev)
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_mul_mat: null argument or more than 4 tensors");
    if (M < 0) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_mul_mat: negative M");
    for (int i = 0; i < n; ++i) {
        if (!w[i] || !y_dev[i]) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_mul_mat: null tensor");
        if (w[i]->E != 1) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_mul_mat: expert tensors need qproj_mul_mat_id");
        if (w[i]->K != w[0]->K || w[i]->type != w[0]->type)
            return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_mul_mat_multi: tensors must share K and type");
    }
    if (M == 0) return QPROJ_OK;
    if (!dry_run()) QP_HIP(ctx, hipSetDevice(ctx->device));
    const int64_t K = w[0]->K;
    if (swiglu_u && (norm || !swiglu_quantizer_serves(w[0], M, act)))
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj: the fused swiglu needs a quantized route beyond the decode regime");
    if (act == kActGGML && !use_mfma_kernel(w[0]->type, M, K) && use_decode_kernel(w[0]->type, M, K) &&
        (!norm || decode_kernel_norm_fits(pow2_ceil(M), K))) {
        // decode regime: the kernel (normalises and) quantizes the activation rows itself, no scratch needed
        GemvArgs g{};
        g.n_targets = n;
        for (int i = 0; i < n; ++i) {
            g.t[i].w = w[i]->view;
            g.t[i].y = y_dev[i];
        }
        g.x = x_dev;
        g.norm = norm != nullptr;
        g.norm_gamma = norm ? norm->gamma : nullptr;
        g.norm_eps = norm ? norm->eps : 0.f;
        g.M = (int)M;
        g.x_div = 1;
        QP_HIP(ctx, launch_gemv_decode(g, pow2_ceil(M), true, ctx->stream));
        return QPROJ_OK;
    }
    if (act == kActGGML || act == kActQ8X32) {
        if (act == kActQ8X32 && w[0]->type != kTypeQ4_K)
            return fail(ctx, QPROJ_ERR_UNSUPPORTED, "qproj_mul_mat: the per-32 int8 path is built for Q4_K weights");
        if (act == kActGGML && !norm && !swiglu_u && dense_fuses_quantizer(w[0], M)) {
            const size_t extra = dense_scratch_bytes(n, w, M);
            int rc = reserve(ctx, wsp, extra);
            if (rc) return rc;
            ActView a{};
            a.kind = act_kind_for(act, w[0]->type);
            a.K = K;
            return run_dense_q8act(ctx, n, w, a, M, y_dev, Scratch{reinterpret_cast<float *>(wsp.base), extra - std::min(extra, scratch_shave())}, x_dev);
        }
        const ActPlanes p = act_planes(act_kind_for(act, w[0]->type), M, K);
        const size_t extra = act == kActGGML ? dense_scratch_bytes(n, w, M) : per32_scratch_max(n, w, M);
        int rc = reserve(ctx, wsp, p.total + extra);
        if (rc) return rc;
        uint8_t *ws = wsp.base;
        // the min-term plane (a second small launch, one wave a row) only where a tiled Q4_K kernel will read it
        const bool minterm = act == kActQ8X32 || (w[0]->type == kTypeQ4_K && takes_tiled(w[0], M));
        ZeroJob zero{};
        bool y_zeroed = false;
        uint32_t tile_adds = 0;   // tiled Q4_K: the matrices whose two K stretches add themselves to cleared rows
        if (norm) {   // norm, weights and quantizer in one launch
            if (p.kind == kActKindQ8X32 && K % 256 != 0)
                return fail(ctx, QPROJ_ERR_UNSUPPORTED, "qproj_rms_norm_mul_mat: the per-32 format needs K % 256 == 0");
            QP_HIP(ctx, launch_rms_norm(p.kind, x_dev, norm->gamma, norm->eps, M, K, nullptr,
                                        reinterpret_cast<int8_t *>(ws + p.off_qs), reinterpret_cast<float *>(ws + p.off_d),
                                        reinterpret_cast<int16_t *>(ws + p.off_aux),
                                        minterm ? reinterpret_cast<uint16_t *>(ws + p.off_msum) : nullptr,
                                        reinterpret_cast<int32_t *>(ws + p.off_aux),
                                        minterm ? reinterpret_cast<float *>(ws + p.off_rs) : nullptr, ctx->stream));
        } else {
            y_zeroed = act == kActGGML && !minterm && dense_clears_rows(n, w, M, y_dev, x_dev, zero);
            if (act == kActGGML && w[0]->type == kTypeQ4_K && takes_tiled(w[0], M))
                tile_adds = tiled_clears_rows(n, w, M, y_dev, x_dev, extra > 0, zero);
            QP_HIP(ctx, run_quantize(ctx, p, ws, x_dev, M, K, minterm, swiglu_u, y_zeroed || tile_adds ? &zero : nullptr));
        }
        const ActView a = act_view(p, ws, K);
        // the partial results lie behind the activation planes; `extra` is all a launcher may use of it
        const Scratch sc{extra ? reinterpret_cast<float *>(ws + p.total) : nullptr, extra - std::min(extra, scratch_shave()), tile_adds};
        if (act == kActGGML) return run_dense_q8act(ctx, n, w, a, M, y_dev, sc, nullptr, y_zeroed);
        for (int i = 0; i < n; ++i) QP_HIP(ctx, launch_gemm_q8x32(w[i]->view, a, M, y_dev[i], sc, ctx->stream));
        return QPROJ_OK;
    }
    if (act == kActF32) {
        if (norm) {   // normalised rows to the workspace, then the fp32 kernel reads them
            int rc = reserve(ctx, wsp, (size_t)M * K * 4);
            if (rc) return rc;
            QP_HIP(ctx, launch_rms_norm(-1, x_dev, norm->gamma, norm->eps, M, K, reinterpret_cast<float *>(wsp.base), nullptr,
                                        nullptr, nullptr, nullptr, nullptr, nullptr, ctx->stream));
            x_dev = reinterpret_cast<const float *>(wsp.base);
        }
        for (int64_t m0 = 0; m0 < M; m0 += 4) {
            const int64_t mc = std::min<int64_t>(4, M - m0);
            GemvArgs g{};
            g.n_targets = n;
            for (int i = 0; i < n; ++i) {
                g.t[i].w = w[i]->view;
                g.t[i].y = y_dev[i] + m0 * w[i]->N;
            }
            g.x = x_dev + m0 * K;
            g.M = (int)mc;
            g.x_div = 1;
            QP_HIP(ctx, launch_gemv_f32(g, pow2_ceil(mc), 1, ctx->stream));
        }
        return QPROJ_OK;
    }
    return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_mul_mat: unknown activation mode");
}

static Workspace ctx_workspace(qproj_ctx *ctx) { return Workspace{ctx ? ctx->ws : nullptr, ctx ? ctx->ws_bytes : 0, false}; }

int qproj_mul_mat_multi(qproj_ctx *ctx, int n, const qproj_weight *const *w, const float *x_dev, int64_t M,
                        float *const *y_dev, int act) {
    Workspace wsp = ctx_workspace(ctx);
    return mul_mat_multi_impl(ctx, n, w, x_dev, M, y_dev, act, nullptr, wsp);
}

int qproj_mul_mat_multi_noalloc(qproj_ctx *ctx, int n, const qproj_weight *const *w, const float *x_dev, int64_t M,
                                float *const *y_dev, int act) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    uint8_t *fixed = nullptr;
    if (ctx->device >= 0 && ctx->device < kMaxDevices) {
        std::lock_guard<std::mutex> lock(g_noalloc_mu);
        fixed = g_noalloc_ptr[ctx->device];
        if (fixed) {
            if (!g_noalloc_owner[ctx->device]) g_noalloc_owner[ctx->device] = ctx;
            if (g_noalloc_owner[ctx->device] != ctx)
                return fail(ctx, QPROJ_ERR_UNSUPPORTED,
                            "qproj_mul_mat_multi_noalloc: the fixed scratch of this GPU is in use by another context "
                            "(calls from two contexts would overwrite each other's scratch)");
        }
    }
    if (!fixed)
        return fail(ctx, QPROJ_ERR_UNSUPPORTED, "qproj_mul_mat_multi_noalloc: the fixed scratch was not set up for this device");
    Workspace wsp{fixed, (size_t)QPROJ_NOALLOC_SCRATCH_BYTES, true};
    return mul_mat_multi_impl(ctx, n, w, x_dev, M, y_dev, act, nullptr, wsp);
}

size_t qproj_workspace_bytes(int type, int64_t K, int n, const int64_t *N, int64_t M, int act, int *status) {
    // Walks the dispatch of qproj_mul_mat_multi for this shape without touching a device: the same code that serves
    // a call sizes its scratch, hands it to the launchers it picks, and every launcher checks its own demand against
    // what it was given.  *status is QPROJ_OK when all of them were satisfied.
    if (status) *status = QPROJ_ERR_INVALID_ARG;
    if (!type_ok(type) || n <= 0 || n > kMaxTargets || !N || M < 0 || K <= 0 || K % block_elems(type) != 0) return 0;
    qproj_ctx ctx;
    qproj_weight ws[kMaxTargets];
    const qproj_weight *wp[kMaxTargets];
    float *yp[kMaxTargets];
    for (int i = 0; i < n; ++i) {
        if (N[i] <= 0) return 0;
        ws[i].type = type;
        ws[i].K = K;
        ws[i].N = N[i];
        ws[i].E = 1;
        ws[i].dev = reinterpret_cast<uint8_t *>(uintptr_t(256));
        make_view(&ws[i]);
        wp[i] = &ws[i];
        yp[i] = reinterpret_cast<float *>((uintptr_t(1) << 40) + (uintptr_t(i) << 36));   // stand-ins, apart from x and from each other
    }
    const float *fake_x = reinterpret_cast<const float *>(uintptr_t(256));
    set_dry_run(true);
    Workspace sized{nullptr, 0, false};
    int rc = mul_mat_multi_impl(&ctx, n, wp, fake_x, M, yp, act, nullptr, sized);
    const size_t total = sized.reserved;
    if (rc == QPROJ_OK) {   // against a fixed buffer of exactly that size every launcher must be satisfied ...
        Workspace exact{reinterpret_cast<uint8_t *>(uintptr_t(256)), total, true};
        rc = mul_mat_multi_impl(&ctx, n, wp, fake_x, M, yp, act, nullptr, exact);
    }
    if (rc == QPROJ_OK && total > 0) {   // ... one byte less must be refused by the reservation ...
        Workspace less{reinterpret_cast<uint8_t *>(uintptr_t(256)), total - 1, true};
        if (mul_mat_multi_impl(&ctx, n, wp, fake_x, M, yp, act, nullptr, less) == QPROJ_OK) rc = QPROJ_ERR_HIP;
    }
    if (rc == QPROJ_OK && act == kActGGML && dense_scratch_bytes(n, wp, M) > 0) {
        // ... and the launchers' own capacity checks are exercised too: the reservation succeeds, but every launcher is
        // told it has NO scratch beyond the activation planes (and no cleared output rows to add into).  A launcher
        // that cuts K must then refuse; the only calls that may still pass are those whose launchers need none (the
        // reservation is an upper bound: matrices that ride in one launch with K whole use none of it).
        Workspace exact{reinterpret_cast<uint8_t *>(uintptr_t(256)), total, true};
        float *odd[kMaxTargets];   // misaligned outputs: no route that adds into cleared rows instead of using scratch
        for (int i = 0; i < n; ++i) odd[i] = reinterpret_cast<float *>(uintptr_t(260));
        g_plan_cuts = 0;
        g_scratch_shave = ~(size_t)0;
        const int starved = mul_mat_multi_impl(&ctx, n, wp, fake_x, M, odd, act, nullptr, exact);
        g_scratch_shave = 0;
        if (starved == QPROJ_OK && g_plan_cuts > 0) rc = QPROJ_ERR_HIP;   // a K cut went through without scratch
    }
    set_dry_run(false);
    if (status) *status = rc;
    return rc == QPROJ_OK ? total : 0;
}

// The routing table: the launches a call of this shape makes, one line each, written by the launchers themselves
// during a dry run of the dispatch code that serves the call (nothing touches a device).
namespace {
int finish_plan(const std::string &text, int rc, size_t scratch, char *buf, size_t buf_bytes) {
    std::string out = text;
    char tail[96];
    snprintf(tail, sizeof tail, "scratch: %zu bytes\n", scratch);
    out += tail;
    if (rc != QPROJ_OK) out += "(the call is refused with status " + std::to_string(rc) + ")\n";
    if (!buf || buf_bytes == 0) return QPROJ_ERR_INVALID_ARG;
    const size_t n = std::min(out.size(), buf_bytes - 1);
    memcpy(buf, out.data(), n);
    buf[n] = 0;
    return out.size() < buf_bytes ? rc : QPROJ_ERR_INVALID_ARG;
}
void fake_weight(qproj_weight &w, int type, int64_t K, int64_t N, int64_t E) {
    w.type = type;
    w.K = K;
    w.N = N;
    w.E = E;
    w.dev = reinterpret_cast<uint8_t *>(uintptr_t(256));
    make_view(&w);
}
}  // namespace

int qproj_plan_mul_mat(int type, int64_t K, int n, const int64_t *N, int64_t M, int act, int with_norm, char *buf, size_t buf_bytes) {
    if (!type_ok(type) || n <= 0 || n > kMaxTargets || !N || M < 0 || K <= 0 || K % block_elems(type) != 0) return QPROJ_ERR_INVALID_ARG;
    qproj_ctx ctx;
    qproj_weight ws[kMaxTargets];
    const qproj_weight *wp[kMaxTargets];
    float *yp[kMaxTargets];
    for (int i = 0; i < n; ++i) {
        if (N[i] <= 0) return QPROJ_ERR_INVALID_ARG;
        fake_weight(ws[i], type, K, N[i], 1);
        wp[i] = &ws[i];
        yp[i] = reinterpret_cast<float *>((uintptr_t(1) << 40) + (uintptr_t(i) << 36));   // stand-ins, apart from x and from each other
    }
    const float *fake_x = reinterpret_cast<const float *>(uintptr_t(256));
    const NormSpec norm{fake_x, 1e-5f};
    std::string text;
    set_dry_run(true);
    g_plan = &text;
    Workspace sized{nullptr, 0, false};
    const int rc = mul_mat_multi_impl(&ctx, n, wp, fake_x, M, yp, act, with_norm ? &norm : nullptr, sized);
    g_plan = nullptr;
    set_dry_run(false);
    return finish_plan(text, rc, sized.reserved, buf, buf_bytes);
}

int qproj_plan_moe_ffn(int gate_type, int down_type, int64_t d_model, int64_t d_ff, int64_t n_expert, int64_t n_used, int64_t B,
                       char *buf, size_t buf_bytes) {
    if (!type_ok(gate_type) || !type_ok(down_type) || d_model <= 0 || d_ff <= 0 || n_expert <= 0 || n_used <= 0 || B < 0 ||
        d_model % block_elems(gate_type) != 0 || d_ff % block_elems(down_type) != 0)
        return QPROJ_ERR_INVALID_ARG;
    qproj_ctx ctx;
    qproj_weight gate, up, down;
    fake_weight(gate, gate_type, d_model, d_ff, n_expert);
    fake_weight(up, gate_type, d_model, d_ff, n_expert);
    fake_weight(down, down_type, d_ff, d_model, n_expert);
    const float *fx = reinterpret_cast<const float *>(uintptr_t(256));
    std::string text;
    set_dry_run(true);
    g_plan = &text;
    ctx.ws_bytes = 0;
    ctx.flag_dev = reinterpret_cast<int32_t *>(uintptr_t(256));   // never dereferenced in a dry run
    const int rc = qproj_moe_ffn(&ctx, &gate, &up, &down, fx, reinterpret_cast<const int32_t *>(uintptr_t(256)), fx, n_used, B,
                                 reinterpret_cast<float *>(uintptr_t(256)), kActGGML);
    g_plan = nullptr;
    set_dry_run(false);
    const size_t scratch_bytes = ctx.ws_bytes;
    ctx.ws_bytes = 0;
    ctx.flag_dev = nullptr;
    return finish_plan(text, rc, scratch_bytes, buf, buf_bytes);
}

int qproj_rms_norm_mul_mat(qproj_ctx *ctx, int n, const qproj_weight *const *w, const float *x_dev, const float *gamma_dev,
                           float eps, int64_t M, float *const *y_dev, int act) {
    const NormSpec norm{gamma_dev, eps};
    Workspace wsp = ctx_workspace(ctx);
    return mul_mat_multi_impl(ctx, n, w, x_dev, M, y_dev, act, &norm, wsp);
}

// silu(gate . x) * (up . x), optionally behind an RMS norm: one launch where the decode kernel serves
static int ffn_gate_up_impl(qproj_ctx *ctx, const qproj_weight *gate, const qproj_weight *up, const float *x_dev,
                            int64_t M, float *h_dev, int act, const NormSpec *norm) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    if (!gate || !up || !x_dev || !h_dev) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_ffn_gate_up: null argument");
    if (gate->E != 1 || up->E != 1 || gate->K != up->K || gate->N != up->N || gate->type != up->type)
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_ffn_gate_up: gate and up must be dense tensors of one shape and type");
    if (M < 0) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_ffn_gate_up: negative M");
    if (M == 0) return QPROJ_OK;
    QP_HIP(ctx, hipSetDevice(ctx->device));
    const int64_t K = gate->K, N = gate->N;
    if (act == kActGGML && M <= 2 && !use_mfma_kernel(gate->type, M, K) && use_decode_kernel(gate->type, M, K) &&
        (!norm || decode_kernel_norm_fits(pow2_ceil(M), K))) {
        GemvArgs g{};
        g.n_targets = 2;
        g.t[0].w = gate->view;
        g.t[1].w = up->view;
        g.t[0].y = h_dev;
        g.t[1].y = h_dev;
        g.swiglu_pair = true;
        g.x = x_dev;
        g.norm = norm != nullptr;
        g.norm_gamma = norm ? norm->gamma : nullptr;
        g.norm_eps = norm ? norm->eps : 0.f;
        g.M = (int)M;
        g.x_div = 1;
        QP_HIP(ctx, launch_gemv_decode(g, pow2_ceil(M), true, ctx->stream));
        return QPROJ_OK;
    }
    // larger batches: the two projections into scratch, then the elementwise product
    int rc = ensure_ws2(ctx, (size_t)2 * M * N * 4);
    if (rc) return rc;
    float *gu[2] = {reinterpret_cast<float *>(ctx->ws2), reinterpret_cast<float *>(ctx->ws2) + (size_t)M * N};
    const qproj_weight *ws[2] = {gate, up};
    Workspace wsp = ctx_workspace(ctx);
    rc = mul_mat_multi_impl(ctx, 2, ws, x_dev, M, gu, act, norm, wsp);
    if (rc) return rc;
    QP_HIP(ctx, launch_swiglu(gu[0], gu[1], (size_t)M * N, h_dev, ctx->stream));
    return QPROJ_OK;
}

int qproj_ffn_gate_up(qproj_ctx *ctx, const qproj_weight *gate, const qproj_weight *up, const float *x_dev, int64_t M,
                      float *h_dev, int act) {
    return ffn_gate_up_impl(ctx, gate, up, x_dev, M, h_dev, act, nullptr);
}

int qproj_rms_norm_ffn_gate_up(qproj_ctx *ctx, const qproj_weight *gate, const qproj_weight *up, const float *x_dev,
                               const float *gamma_dev, float eps, int64_t M, float *h_dev, int act) {
    const NormSpec norm{gamma_dev, eps};
    return ffn_gate_up_impl(ctx, gate, up, x_dev, M, h_dev, act, &norm);
}

int qproj_ffn(qproj_ctx *ctx, const qproj_weight *gate, const qproj_weight *up, const qproj_weight *down, const float *x_dev,
              const float *gamma_dev, float eps, int use_norm, int64_t M, float *y_dev, int act) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    if (!gate || !up || !down || !x_dev || !y_dev) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_ffn: null argument");
    if (gate->E != 1 || up->E != 1 || down->E != 1 || gate->K != up->K || gate->N != up->N || gate->type != up->type ||
        down->K != gate->N)
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_ffn: gate/up/down shapes do not agree");
    if (M < 0) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_ffn: negative M");
    if (M == 0) return QPROJ_OK;
    QP_HIP(ctx, hipSetDevice(ctx->device));
    const int64_t d_ff = gate->N;
    const NormSpec norm{gamma_dev, eps};
    // the scratch row(s) h between the halves, kept apart from the workspace the projections themselves use
    int rc = ensure_ws2(ctx, (size_t)3 * M * d_ff * 4);
    if (rc) return rc;
    float *h = reinterpret_cast<float *>(ctx->ws2) + (size_t)2 * M * d_ff;
    const bool gate_up_decode = act == kActGGML && M <= 2 && !use_mfma_kernel(gate->type, M, gate->K) &&
                                use_decode_kernel(gate->type, M, gate->K);
    if (!gate_up_decode && swiglu_quantizer_serves(down, M, act)) {
        // batches: gate and up into scratch, then the down projection's quantizer forms silu(gate) * up itself -
        // the intermediate rows are never written as fp32 (the planes are bit for bit those of the separate calls)
        float *gu[2] = {reinterpret_cast<float *>(ctx->ws2), reinterpret_cast<float *>(ctx->ws2) + (size_t)M * d_ff};
        const qproj_weight *ws[2] = {gate, up};
        Workspace wsp = ctx_workspace(ctx);
        rc = mul_mat_multi_impl(ctx, 2, ws, x_dev, M, gu, act, use_norm ? &norm : nullptr, wsp);
        if (rc) return rc;
        const qproj_weight *wd[1] = {down};
        float *yd[1] = {y_dev};
        Workspace wsp2 = ctx_workspace(ctx);
        return mul_mat_multi_impl(ctx, 1, wd, gu[0], M, yd, act, nullptr, wsp2, gu[1]);
    }
    rc = ffn_gate_up_impl(ctx, gate, up, x_dev, M, h, act, use_norm ? &norm : nullptr);
    if (rc) return rc;
    return qproj_mul_mat(ctx, down, h, M, y_dev, act);
}

int qproj_mul_mat_quantized(qproj_ctx *ctx, int n, const qproj_weight *const *w, const void *act_dev, int kind,
                            int64_t M, float *const *y_dev) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    if (n <= 0 || n > kMaxTargets || !w || !y_dev || !act_dev)
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_mul_mat_quantized: null argument or more than 4 tensors");
    if (kind != kActGGML && kind != kActQ8X32)
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_mul_mat_quantized: kind must name a quantized format");
    for (int i = 0; i < n; ++i) {
        if (!w[i] || !y_dev[i] || w[i]->E != 1 || w[i]->K != w[0]->K || w[i]->type != w[0]->type)
            return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_mul_mat_quantized: tensors must be dense and share K and type");
    }
    if (M <= 0) return M == 0 ? QPROJ_OK : fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_mul_mat_quantized: negative M");
    if (kind == kActQ8X32 && w[0]->type != kTypeQ4_K)
        return fail(ctx, QPROJ_ERR_UNSUPPORTED, "qproj_mul_mat_quantized: the per-32 int8 path is built for Q4_K weights");
    QP_HIP(ctx, hipSetDevice(ctx->device));
    const int64_t K = w[0]->K;
    const ActPlanes p = act_planes(act_kind_for(kind, w[0]->type), M, K);
    const ActView a = act_view(p, static_cast<uint8_t *>(const_cast<void *>(act_dev)), K);
    const size_t extra = kind == kActGGML ? dense_scratch_bytes(n, w, M) : per32_scratch_max(n, w, M);
    int rc = ensure_ws(ctx, extra);
    if (rc) return rc;
    const Scratch sc{extra ? reinterpret_cast<float *>(ctx->ws) : nullptr, extra};
    if (kind == kActGGML) return run_dense_q8act(ctx, n, w, a, M, y_dev, sc);
    for (int i = 0; i < n; ++i) QP_HIP(ctx, launch_gemm_q8x32(w[i]->view, a, M, y_dev[i], sc, ctx->stream));
    return QPROJ_OK;
}

int qproj_mul_mat(qproj_ctx *ctx, const qproj_weight *w, const float *x_dev, int64_t M, float *y_dev, int act) {
    const qproj_weight *ws[1] = {w};
    float *ys[1] = {y_dev};
    return qproj_mul_mat_multi(ctx, 1, ws, x_dev, M, ys, act);
}

int qproj_mul_mat_id(qproj_ctx *ctx, const qproj_weight *w, const float *x_dev, int64_t nb1,
                     const int32_t *ids_dev, int64_t n_used, int64_t B, float *y_dev, int act) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    if (!w || !x_dev || !ids_dev || !y_dev) return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_mul_mat_id: null argument");
    if (n_used <= 0 || B < 0 || (nb1 != 1 && nb1 != n_used))
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_mul_mat_id: nb1 must be 1 or n_used");
    if (act != kActGGML) return fail(ctx, QPROJ_ERR_UNSUPPORTED, "qproj_mul_mat_id: only the ggml activation mode");
    if (B == 0) return QPROJ_OK;
    if (!dry_run()) QP_HIP(ctx, hipSetDevice(ctx->device));
    const int64_t K = w->K, n_pairs = B * n_used, rows = B * nb1;
    if (moe_decode_route(w->type, K, w->N, n_pairs, 1, w->E)) {
        GemvArgs g{};
        g.n_targets = 1;
        g.t[0].w = w->view;
        g.t[0].y = y_dev;
        g.x = x_dev;
        g.x_div = nb1 == 1 ? (int)n_used : 1;
        g.ids = ids_dev;
        g.n_pairs = (int)n_pairs;
        g.error_flag = ctx->flag_dev;
        QP_HIP(ctx, launch_moe_decode(g, (int)w->E, false, nullptr, 0, ctx->stream));
        return QPROJ_OK;
    }
    const ActPlanes p = act_planes(act_kind_for(act, w->type), rows, K);
    const size_t off_order = p.total;
    const size_t off_offsets = off_order + align_up((size_t)n_pairs * 4);
    const size_t off_active = off_offsets + align_up((size_t)(w->E + 1) * 4);
    const size_t off_parts = off_active + align_up(active_list_bytes(w->E));
    const bool long_rows = grouped_long_rows(w, n_pairs);
    const size_t parts_bytes = long_rows ? mfma_grouped_scratch_bytes(K, w->N, n_pairs, w->E) : 0;
    const size_t total = off_parts + align_up(parts_bytes);
    Workspace wsp = ctx_workspace(ctx);
    int rc = reserve(ctx, wsp, total);
    if (rc) return rc;
    // few pairs an expert: the grouped kernel quantizes the rows it needs in its prologue
    const bool fuse = grouped_fuses_quantizer(w->type, K, n_pairs, w->E);
    int32_t *order = reinterpret_cast<int32_t *>(wsp.base + off_order);
    int32_t *offsets = reinterpret_cast<int32_t *>(wsp.base + off_offsets);
    int32_t *active = reinterpret_cast<int32_t *>(wsp.base + off_active);
    const bool pair_mode = grouped_pair_mode(w->type, K, n_pairs, w->E);
    // the quantizer and the grouping pass read only the call's inputs: one launch carries both
    const bool joined = !fuse && !pair_mode && p.kind == kActKindQ8_K;
    const RowQuantJob job = quantize_job(p, wsp.base, x_dev, rows, K);
    if (!fuse && !joined) QP_HIP(ctx, run_quantize(ctx, p, wsp.base, x_dev, rows, K, false));
    if (!pair_mode)
        QP_HIP(ctx, launch_moe_group(ids_dev, n_pairs, w->E, order, offsets, active, ctx->flag_dev,
                                     joined ? &job : nullptr, ctx->stream));
    GemvArgs g{};
    g.n_targets = 1;
    g.t[0].w = w->view;
    g.t[0].y = y_dev;
    if (pair_mode) {
        g.ids = ids_dev;
        g.n_pairs = (int)n_pairs;
        g.error_flag = ctx->flag_dev;
    }
    g.a = act_view(p, wsp.base, K);
    g.x = fuse ? x_dev : nullptr;
    g.order = order;
    g.offsets = offsets;
    g.active = active;
    g.x_div = nb1 == 1 ? (int)n_used : 1;
    if (use_mfma_grouped(w->type, K))
        QP_HIP(ctx, launch_gemv_mfma_grouped(g, n_pairs, false, ctx->stream));
    else if (long_rows)
        QP_HIP(ctx, launch_gemv_mfma_grouped(g, n_pairs, false, ctx->stream,
                                             Scratch{reinterpret_cast<float *>(wsp.base + off_parts), parts_bytes}));
    else
        QP_HIP(ctx, launch_gemv_q8act(g, grouped_mt(n_pairs, w->E), (int)w->E, ctx->stream));
    return QPROJ_OK;
}

int qproj_moe_ffn(qproj_ctx *ctx, const qproj_weight *gate, const qproj_weight *up, const qproj_weight *down,
                  const float *x_dev, const int32_t *ids_dev, const float *weights_dev, int64_t n_used, int64_t B,
                  float *y_dev, int act) {
    if (!ctx) return QPROJ_ERR_INVALID_ARG;
    if (!gate || !up || !down || !x_dev || !ids_dev || !weights_dev || !y_dev)
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_moe_ffn: null argument");
    if (act != kActGGML) return fail(ctx, QPROJ_ERR_UNSUPPORTED, "qproj_moe_ffn: only the ggml activation mode");
    const int64_t d_model = gate->K, d_ff = gate->N, E = gate->E;
    if (up->K != d_model || up->N != d_ff || up->E != E || up->type != gate->type || down->K != d_ff ||
        down->N != d_model || down->E != E || n_used <= 0 || B < 0)
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_moe_ffn: gate/up/down shapes do not agree");
    if (d_ff % block_elems(down->type) != 0 || (down->type != kTypeQ8_0 && d_ff % 256 != 0))
        return fail(ctx, QPROJ_ERR_INVALID_ARG, "qproj_moe_ffn: d_ff must be a multiple of the block size");
    if (B == 0) return QPROJ_OK;
    if (!dry_run()) QP_HIP(ctx, hipSetDevice(ctx->device));
    const int64_t n_pairs = B * n_used;
    const ActPlanes px = act_planes(act_kind_for(act, gate->type), B, d_model);
    const ActPlanes ph = act_planes(act_kind_for(act, down->type), n_pairs, d_ff);
    size_t off = px.total;
    const size_t off_order = off;
    off += align_up((size_t)n_pairs * 4);
    const size_t off_offsets = off;
    off += align_up((size_t)(E + 1) * 4);
    const size_t off_active = off;
    off += align_up(active_list_bytes(E));
    const size_t off_h = off;
    off += align_up((size_t)(n_pairs * d_ff) * 4);
    const size_t off_hq = off;
    off += ph.total;
    const size_t off_e = off;
    off += align_up((size_t)(n_pairs * d_model) * 4);
    // rows too long for one pass of the grouped matrix-core kernel go in K chunks (grouped_long_rows); gate and up then
    // take a launch each (the SwiGLU epilogue needs whole sums) and the swiglu is formed by the quantizer behind them
    const bool long_down = grouped_long_rows(down, n_pairs), long_gate = grouped_long_rows(gate, n_pairs);
    const size_t parts_bytes = std::max(long_down ? mfma_grouped_scratch_bytes(d_ff, d_model, n_pairs, E) : 0,
                                        long_gate ? mfma_grouped_scratch_bytes(d_model, d_ff, n_pairs, E) : 0);
    const size_t off_parts = off;
    off += align_up(parts_bytes);
    const size_t off_h2 = off;
    if (long_gate) off += align_up((size_t)(n_pairs * d_ff) * 4);
    Workspace wsp = ctx_workspace(ctx);
    int rc = reserve(ctx, wsp, off);
    if (rc) return rc;
    uint8_t *ws = wsp.base;
    int32_t *order = reinterpret_cast<int32_t *>(ws + off_order);
    int32_t *offsets = reinterpret_cast<int32_t *>(ws + off_offsets);
    int32_t *active = reinterpret_cast<int32_t *>(ws + off_active);
    float *h = reinterpret_cast<float *>(ws + off_h);
    float *e = reinterpret_cast<float *>(ws + off_e);
    const int mt = grouped_mt(n_pairs, E);

    if (moe_decode_route(gate->type, d_model, d_ff, n_pairs, 1, E) && moe_decode_route(down->type, d_ff, d_model, n_pairs, n_used, E)) {
        GemvArgs g{};
        g.n_targets = 2;
        g.t[0].w = gate->view;
        g.t[0].y = h;
        g.t[1].w = up->view;
        g.t[1].y = h;
        g.x = x_dev;
        g.x_div = (int)n_used;
        g.ids = ids_dev;
        g.n_pairs = (int)n_pairs;
        g.error_flag = ctx->flag_dev;
        QP_HIP(ctx, launch_moe_decode(g, (int)E, true, nullptr, 0, ctx->stream));
        GemvArgs gd{};
        gd.n_targets = 1;
        gd.t[0].w = down->view;
        gd.t[0].y = y_dev;
        gd.x = h;
        gd.x_div = 1;
        gd.ids = ids_dev;
        gd.n_pairs = (int)n_pairs;
        gd.error_flag = ctx->flag_dev;
        QP_HIP(ctx, launch_moe_decode(gd, (int)E, false, weights_dev, (int)n_used, ctx->stream));
        return QPROJ_OK;
    }

    const bool fuse_x = grouped_fuses_quantizer(gate->type, d_model, n_pairs, E);
    const bool fuse_h = grouped_fuses_quantizer(down->type, d_ff, n_pairs, E);
    const bool pair_mode = grouped_pair_mode(gate->type, d_model, n_pairs, E) &&
                           grouped_pair_mode(down->type, d_ff, n_pairs, E);
    // the quantizer of x and the grouping pass read only the call's inputs: one launch carries both
    const bool joined = !fuse_x && !pair_mode && px.kind == kActKindQ8_K;
    const RowQuantJob job = quantize_job(px, ws, x_dev, B, d_model);
    if (!fuse_x && !joined) QP_HIP(ctx, run_quantize(ctx, px, ws, x_dev, B, d_model, false));
    if (!pair_mode)
        QP_HIP(ctx, launch_moe_group(ids_dev, n_pairs, E, order, offsets, active, ctx->flag_dev,
                                     joined ? &job : nullptr, ctx->stream));
    GemvArgs g{};
    if (pair_mode) {
        g.ids = ids_dev;
        g.n_pairs = (int)n_pairs;
        g.error_flag = ctx->flag_dev;
    }
    g.n_targets = 2;
    g.t[0].w = gate->view;
    g.t[0].y = h;
    g.t[1].w = up->view;
    g.t[1].y = h;
    g.a = act_view(px, ws, d_model);
    g.x = fuse_x ? x_dev : nullptr;
    g.order = order;
    g.offsets = offsets;
    g.active = active;
    g.x_div = (int)n_used;
    const float *swiglu_u = nullptr;   // non-null: h holds the gate products, this the up products
    if (use_mfma_grouped(gate->type, d_model)) {
        QP_HIP(ctx, launch_gemv_mfma_grouped(g, n_pairs, true, ctx->stream));
    } else if (long_gate) {
        float *h2 = reinterpret_cast<float *>(ws + off_h2);
        const Scratch parts{reinterpret_cast<float *>(ws + off_parts), parts_bytes};
        GemvArgs gu = g;
        g.n_targets = 1;
        gu.n_targets = 1;
        gu.t[0].w = up->view;
        gu.t[0].y = h2;
        QP_HIP(ctx, launch_gemv_mfma_grouped(g, n_pairs, false, ctx->stream, parts));
        QP_HIP(ctx, launch_gemv_mfma_grouped(gu, n_pairs, false, ctx->stream, parts));
        swiglu_u = h2;
        if (fuse_h) {   // the down launch quantizes fp32 rows itself: they must be the swiglu by then
            QP_HIP(ctx, launch_swiglu(h, h2, (size_t)(n_pairs * d_ff), h, ctx->stream));
            swiglu_u = nullptr;
        }
    } else {
        QP_HIP(ctx, launch_moe_swiglu_gemv(g, mt, (int)E, ctx->stream));
    }
    if (!fuse_h) QP_HIP(ctx, run_quantize(ctx, ph, ws + off_hq, h, n_pairs, d_ff, false, swiglu_u));
    GemvArgs gd{};
    if (pair_mode) {
        gd.ids = ids_dev;
        gd.n_pairs = (int)n_pairs;
        gd.error_flag = ctx->flag_dev;
    }
    gd.n_targets = 1;
    gd.t[0].w = down->view;
    gd.t[0].y = e;
    gd.a = act_view(ph, ws + off_hq, d_ff);
    gd.x = fuse_h ? h : nullptr;
    gd.order = order;
    gd.offsets = offsets;
    gd.active = active;
    gd.x_div = 1;
    if (use_mfma_grouped(down->type, d_ff))
        QP_HIP(ctx, launch_gemv_mfma_grouped(gd, n_pairs, false, ctx->stream));
    else if (long_down)
        QP_HIP(ctx, launch_gemv_mfma_grouped(gd, n_pairs, false, ctx->stream,
                                             Scratch{reinterpret_cast<float *>(ws + off_parts), parts_bytes}));
    else
        QP_HIP(ctx, launch_gemv_q8act(gd, mt, (int)E, ctx->stream));
    QP_HIP(ctx, launch_moe_combine(e, weights_dev, B, n_used, d_model, y_dev, ctx->stream));
    return QPROJ_OK;
}

}  // extern "C"
