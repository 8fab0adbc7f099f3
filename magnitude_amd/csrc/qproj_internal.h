// Host/device shared declarations of the qproj library (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace qproj {

constexpr int kTypeQ8_0 = 8;
constexpr int kTypeQ4_K = 12;
constexpr int kTypeQ6_K = 14;

constexpr int kActGGML = 0;
constexpr int kActF32 = 1;
constexpr int kActQ8X32 = 2;

constexpr int kWave = 64;

// Device-side view of an uploaded weight.  Q4_K keeps the GGUF block layout (144-byte
// blocks are 16-byte aligned as they are).  Q8_0 and Q6_K blocks (34 and 210 bytes) are only
// 2-byte aligned in GGUF, so upload splits every field into its own contiguous plane, same
// total bytes, which makes every vector load naturally aligned and coalesced.
struct WeightView {
    int type;
    int64_t K, N, E;       // N rows per expert, E experts; rows are indexed e*N + n
    int64_t nb;            // blocks per row (K/32 for Q8_0, K/256 otherwise)
    const uint8_t *q4k;    // Q4_K: [rows][nb][144]
    const int8_t *q8_qs;   // Q8_0: [rows][K]
    const uint16_t *q8_d;  // Q8_0: [rows][nb] fp16
    const uint8_t *q6_ql;  // Q6_K: [rows][nb][128]
    const uint8_t *q6_qh;  // Q6_K: [rows][nb][64]
    const int8_t *q6_sc;   // Q6_K: [rows][nb][16]
    const uint16_t *q6_d;  // Q6_K: [rows][nb] fp16
};

// Quantized activations, plane per field (row stride in elements is K, K/blk, ...).
struct ActView {
    int kind;              // 0: Q8_0 blocks, 1: Q8_K super-blocks, 2: Q8X32
    int64_t K;
    const int8_t *qs;      // [rows][K]
    const float *d;        // [rows][K/32] (Q8_0, Q8X32) or [rows][K/256] (Q8_K)
    const int16_t *bsums;  // Q8_K: [rows][K/16]
    const uint16_t *msum;  // Q8_K, Q8X32: [rows][K/256][16] fp16: (d / rs[row]) * (sum of 32 codes) * kMinPrescale for the 8
                           //       sub-blocks, high parts, then the 8 low parts (v - high); prefill min term
    const int32_t *isum;   // Q8X32: [rows][K/32]
    const float *rs;       // Q8_K, Q8X32: [rows] the power of two the row's msum entries are normalised by
};
constexpr float kMinPrescale = 0.0625f;  // (d / rs) * sum / 16 <= 2 * 4064 / 16: well inside fp16 whatever the activations
constexpr int kActKindQ8_0 = 0;
constexpr int kActKindQ8_K = 1;
constexpr int kActKindQ8X32 = 2;

// One (weight, output) pair of a multi-tensor launch.
struct GemvTarget {
    WeightView w;
    float *y;              // [rows][N]
    int first_block;       // first blockIdx.x (tiled kernels) or first wave (decode kernel) of the target
    int rows_per_pair;     // decode kernel: consecutive rows each pair of neighbouring waves of the target walks
};
constexpr int kMaxTargets = 4;

struct GemvArgs {
    int n_targets;
    GemvTarget t[kMaxTargets];
    ActView a;
    const float *x;        // f32 activations (F32 mode) [rows][K]
    const float *norm_gamma;   // decode kernel with its quantizer fused: RMS-normalise the rows first and
    float norm_eps;            // multiply by these weights (null: rows are used as they are)
    bool norm;
    bool swiglu_pair;          // decode kernel: targets 0 and 1 are gate and up of one FFN (same K and N); a wave
                               // walks row r of both and stores silu(gate_r . x) * (up_r . x) to t[0].y
    int M;                 // activation rows in this launch (dense mode), <= MT
    bool y_zeroed;         // small-batch kernel, dense mode: the output rows hold zeros when the launch starts (the
                           // quantizer launch in front of it cleared them), so two K chunks may add themselves
    // expert-grouped mode (MUL_MAT_ID); null order = dense
    const int32_t *order;   // pair indices sorted by expert
    const int32_t *offsets; // [E+1] ranges into order
    const int32_t *active;  // [E+1] experts that have pairs, ascending; [E] = how many; behind it (active_slots_offset)
                            // one {expert, first pair slot, pairs, 0} record a list position
    int x_div;              // activation row of pair p is p / x_div
    // pair mode of the grouped matrix-core kernel (a handful of pairs, no grouping pass): a set of
    // workgroups per pair p multiplies row p / x_div by expert ids[p]; ids outside [0, E) raise *error_flag
    const int32_t *ids;
    int n_pairs;
    int32_t *error_flag;
};

// Scratch memory handed to a launcher: where the partial results of a K cut into stretches (tiled kernels) or
// chunks (small-batch kernel) go before a second small kernel adds them.  A launcher works out what its own split
// needs from the variables that pick the split, and answers hipErrorInvalidValue instead of launching when that
// is more than `bytes`.  {nullptr, 0}: K is never cut (the tiled kernels) / the launch is refused if it must be.
struct Scratch {
    float *p;
    size_t bytes;
    uint32_t zeroed = 0;     // bit i: the output rows of the launcher's i-th tensor were cleared by the launch in front
                             // (ZeroJob): a K cut in exactly two may add its two partial results straight to them and
                             // needs neither scratch nor the adding pass
    Scratch for_target(int i) const { return Scratch{p, bytes, (zeroed >> i) & 1u}; }
};

// Dry run: every launcher does its argument and capacity checks and returns without touching the device.  The
// host-side tests walk the dispatch of whole operator calls with it (no GPU needed) to show that the scratch the
// library reserves covers what the launchers it picks ask for.  Thread-local, off by default.
bool dry_run();
void set_dry_run(bool on);
size_t scratch_shave();   // dry runs: bytes withheld from the scratch the launchers are told they have (capacity-check tests)

// Plan recorder: while one is installed on the calling thread (qproj_plan does that around a dry run of the
// dispatch), every launcher writes down the launch it would make - kernel, tile, grid, cuts of K, scratch - as one
// line.  The lines ARE the routing table: they come from the very code that serves a call.
void plan_note(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
const char *plan_type_name(int type);
void plan_note_cut();     // a launcher in a dry run: this launch keeps partial results of a cut K in scratch

// Into how many stretches K is cut for a grid of `tiles` 128-token tiles (one workgroup a compute unit) that would
// not fill the chip by itself: the cut that minimises rounds x (stretch + fixed cost) + the pass that adds the
// partial tiles (M x N x 4 bytes a stretch written and read again), never under twelve super-blocks a stretch.
// `us_per_sb`: what one super-block step of a full round takes (4.5 us for the Q4_K tile, 5 for Q6_K).
inline int wide_tile_splits(int64_t tiles, int64_t nsb, int64_t M, int64_t N, int cus, double us_per_sb) {
    int best = 1;
    double best_cost = 1e300;
    for (int n = 1; n <= 8 && (n == 1 || nsb / n >= 12); ++n) {
        const int64_t per = (nsb + n - 1) / n, rounds = (tiles * n + cus - 1) / cus;
        double cost = (double)rounds * ((double)per * us_per_sb + 8.0);
        if (n > 1) cost += (double)n * (double)M * (double)N * 2.7e-6 + 5.0;
        if (cost < best_cost) {
            best_cost = cost;
            best = n;
        }
    }
    return best;
}

// The busy-expert list of the grouping pass: n_expert + 1 ints (the list, then its length), then from a 16-byte boundary
// one int4 {expert, its first slot in order[], its pairs, 0} per list position, so that a workgroup of the grouped
// kernels learns all three from ONE load instead of a chain of two.
__host__ __device__ inline int64_t active_slots_offset(int64_t n_expert) { return (n_expert + 1 + 3) & ~(int64_t)3; }   // in ints
inline size_t active_list_bytes(int64_t n_expert) { return (size_t)(active_slots_offset(n_expert) + 4 * n_expert) * 4; }

// Compute units of the current device (256 when no device can be asked, e.g. in a dry run on a host without one).
int cu_count();

// Tuning knobs read from the environment exist only in builds made with -DQPROJ_TUNING (kernel-selection sweeps in
// the lab); in the shipped library this returns `dflt` and no environment variable can change a numerics path.
int tuning_int(const char *name, int dflt);

// ---- launchers (each returns the hipError_t of the launch) ----
hipError_t launch_dequantize(const WeightView &w, float *out, hipStream_t s);
hipError_t launch_repack_to_planes(int type, const uint8_t *gguf, uint8_t *planes_base, const WeightView &w,
                                   int64_t n_blocks, hipStream_t s);
hipError_t launch_repack_to_gguf(int type, const WeightView &w, uint8_t *gguf, int64_t n_blocks, hipStream_t s);
// RMS_NORM + MUL by the norm weights (gamma may be null); kind < 0: fp32 rows to y, otherwise the planes of `kind`
// (msum and rs may be null together: the min-term plane of the tiled Q4_K kernels is then not made)
hipError_t launch_rms_norm(int kind, const float *x, const float *gamma, float eps, int64_t M, int64_t K, float *y,
                           int8_t *qs, float *d, int16_t *bsums, uint16_t *msum, int32_t *isum, float *rs, hipStream_t s);
// Output rows that a quantizer launch clears on the side (n[i] floats at p[i], n[i] % 4 == 0, 16-byte aligned): the
// projection launched behind it may then add partial results into them instead of storing them.
struct ZeroJob {
    int count;
    float *p[kMaxTargets];
    int64_t n[kMaxTargets];
};
// u non-null: the rows quantized are silu(x) * u (the swiglu between gate / up and the down projection);
// zero: see ZeroJob (carried by the first launch of the quantizer)
hipError_t launch_quantize_act(int kind, const float *x, int64_t M, int64_t K, int8_t *qs, float *d,
                               int16_t *bsums, uint16_t *msum, int32_t *isum, float *rs, hipStream_t s,
                               const float *u = nullptr, const ZeroJob *zero = nullptr);
// the min-term plane and the row normalisers from planes already quantized (one wave per row)
hipError_t launch_minterm_rows(int kind, const float *d, const int16_t *bsums, const int32_t *isum, int64_t M, int64_t K,
                               uint16_t *msum, float *rs, hipStream_t s);
hipError_t launch_gemv_q8act(const GemvArgs &args, int mt, int n_experts_grid, hipStream_t s);
// persistent decode kernel (mt <= 4 rows); fuse_quantize: args.x holds fp32 rows, else args.a
bool decode_kernel_fits(int type, int mt, int64_t K);
bool decode_kernel_norm_fits(int mt, int64_t K);   // the fused RMS norm needs the whole row in the prologue's registers
hipError_t launch_gemv_decode(const GemvArgs &args, int mt, bool fuse_quantize, hipStream_t s);
// int8 matrix-core kernel for 1..16 activation rows (K % 256 == 0); `scratch` holds the per-K-chunk
// results when K > 4096 (mfma_gemv_scratch_bytes, 0 if none is needed)
bool mfma_gemv_fits(int type, int64_t M, int64_t K);
size_t mfma_gemv_scratch_bytes(int type, int64_t K, int64_t M, int64_t sum_n, int64_t total_row_groups);
// true when the launch cuts K in exactly two chunks: with the output rows cleared beforehand (GemvArgs::y_zeroed) the
// two partial results add themselves to the output (0 + a + b is a + b in either order) and the summing launch goes
bool mfma_gemv_two_chunks(int type, int64_t K, int64_t M, int64_t total_row_groups);
hipError_t launch_gemv_mfma(const GemvArgs &args, const Scratch &scratch, hipStream_t s);
// expert-grouped form (args.order / args.offsets); K / 256 must not exceed 16 (mfma_grouped_fits)
bool mfma_grouped_fits(int type, int64_t K);
// longer rows, not for the SwiGLU launch: K in chunks whose results go to `scratch` (mfma_grouped_scratch_bytes) and are
// added by a pass afterwards; n_pairs * N must be a multiple of 4
bool mfma_grouped_chunked_fits(int type, int64_t K, int64_t N, int64_t n_pairs);
size_t mfma_grouped_scratch_bytes(int64_t K, int64_t N, int64_t n_pairs, int64_t E);
hipError_t launch_gemv_mfma_grouped(const GemvArgs &args, int64_t n_pairs, bool swiglu, hipStream_t s,
                                    const Scratch &scratch = Scratch{nullptr, 0});
hipError_t launch_gemv_f32(const GemvArgs &args, int mt, int n_experts_grid, hipStream_t s);
// h[i] = silu(g[i]) * u[i], the expression of ggml's swiglu on floats
hipError_t launch_swiglu(const float *g, const float *u, size_t n, float *h, hipStream_t s);
// Q8_K quantization of n_super 256-wide chunks of x, carried by the spare workgroups of the grouping launch
struct RowQuantJob {
    const float *x;
    int64_t n_super;
    int8_t *qs;
    float *d;
    int16_t *bsums;
};
hipError_t launch_moe_group(const int32_t *ids, int64_t n_pairs, int64_t n_expert, int32_t *order,
                            int32_t *offsets, int32_t *active, int32_t *error_flag, const RowQuantJob *quantize,
                            hipStream_t s);
hipError_t launch_moe_swiglu_gemv(const GemvArgs &gate_up, int mt, int n_experts_grid, hipStream_t s);
// One or two decode tokens (at most 16 pairs) through expert stacks of Q4_K / Q6_K rows of K <= 4096 on the vector
// ALU: args as for the pair mode of the grouped kernel (t[0], and t[1] = up when `swiglu`; x fp32 rows, x_div, ids,
// n_pairs, error_flag).  combine_weights null: t[0].y is [n_pairs][N]; otherwise the n_used consecutive pairs of a
// token are added with their routing weights in slot order and t[0].y is [n_pairs / n_used][N].
bool moe_decode_fits(int type, int64_t K, int64_t N, int64_t n_pairs, int64_t group, int64_t n_expert);
hipError_t launch_moe_decode(const GemvArgs &args, int n_expert, bool swiglu, const float *combine_weights, int n_used,
                             hipStream_t s);
hipError_t launch_moe_combine(const float *e, const float *weights, int64_t B, int64_t n_used, int64_t N,
                              float *y, hipStream_t s);
// `scratch`: per32_scratch_bytes(K, M, N) bytes (null: K is never split)
int per32_splits(int64_t K, int64_t M, int64_t N);
size_t per32_scratch_bytes(int64_t K, int64_t M, int64_t N);
hipError_t launch_gemm_q8x32(const WeightView &w, const ActView &a, int64_t M, float *y, const Scratch &scratch, hipStream_t s);
// Q4_K weights x ggml Q8_K activations (`a`), large M
// `scratch`: q8k_tile_scratch_bytes(K, M, N) bytes (null: K is never split)
int q8k_tile_splits(int64_t K, int64_t M, int64_t N, bool add_ok);
size_t q8k_tile_scratch_bytes(int64_t K, int64_t M, int64_t N);
hipError_t launch_sum_parts(const float *part, int n_split, size_t n, float *y, hipStream_t s);
size_t q4k_tile_scratch_bytes(int64_t K, int64_t M, int64_t N);   // what launch_gemm_q8k asks of its scratch
// bit i: with cleared output rows, matrix i of a tiled Q4_K call cuts K in two stretches that add themselves (Scratch::zeroed)
uint32_t q4k_multi_adds(int n, const WeightView *w, int64_t M, bool have_scratch);
hipError_t launch_gemm_q8k(const WeightView &w, const ActView &a, int64_t M, float *y, const Scratch &scratch, hipStream_t s);
hipError_t launch_gemm_q8k_multi(int n, const WeightView *w, const ActView &a, int64_t M, float *const *y,
                                 const Scratch &scratch, hipStream_t s);
hipError_t launch_gemm_q8_0(const WeightView &w, const ActView &a, int64_t M, float *y, const Scratch &scratch, hipStream_t s);
size_t q6k_tile_scratch_bytes(int64_t K, int64_t M, int64_t N);   // what launch_gemm_q6k_q8k asks of its scratch
hipError_t launch_gemm_q6k_q8k(const WeightView &w, const ActView &a, int64_t M, float *y, const Scratch &scratch, hipStream_t s);

}  // namespace qproj
