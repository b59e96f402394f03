// kernels.h — shared declarations between the HIP kernels and the C-ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace larql {

enum GemvKind : int32_t {
    KIND_Q4K = 0, KIND_Q8_0 = 1, KIND_MXFP4 = 2, KIND_Q4_0 = 3, KIND_BF16 = 4, KIND_F16 = 5, KIND_F32 = 6,
    KIND_Q4K_MFMA = 7,   // internal: Q4_K rows short enough for the matrix-core kernel (see gemv_effective_kind)
    KIND_MXFP4_MFMA = 8, // internal: likewise for MXFP4
    KIND_BF16_MFMA = 9,  // internal: bf16 rows against 2..8 activations at once (batch field of the job)
    KIND_Q4K_BATCH = 10, // internal: Q4_K rows against 2..4 activations at once
    KIND_Q8_0_MFMA = 11, // internal: ggml Q8_0 rows short enough for the matrix-core kernel
    KIND_Q6K = 12,       // Q6_K, 210-byte super-blocks (K-slice kernel)
    KIND_Q4K_Q8K = 13,   // Q4_K weights against a Q8_K activation (integer dots on the matrix cores); x = the Q8_K device layout
    KIND_Q6K_Q8K = 14,   // Q6_K weights against a Q8_K activation (K-slice kernel, v_dot4)
    KIND_Q6K_MFMA = 15   // internal: Q6_K rows short enough for the matrix-core kernel
};

constexpr int kGemvMaxThreads = 512;
constexpr int kInlineJobs = 8;  // jobs that travel in the kernel arguments (no table upload)

// One matvec of a launch.  The caller fills kind/w/aux/x/out/rows/k; the rest
// is geometry derived by gemv_job_geometry for the launch's block size.
struct GemvJob {
    const uint8_t *w;    // packed weights, [rows] rows of row_bytes
    const uint8_t *aux;  // MXFP4: e8m0 scales [rows, k/32]; Q4_0: f32 activation scales
    const float *x;      // activation (Q4_0: the int8 code stream)
    float *out;
    uint64_t rows, k;
    uint64_t row_bytes;
    uint32_t cpr;         // chunks (threads) per row
    uint32_t rpp;         // rows per pass
    uint32_t n_pass;      // ceil(rows / rpp)
    uint32_t pass_begin;  // first pass of this job in the launch's pass list
    int32_t kind;
    int32_t pad;
    // Optional run-time selection (MoE): when `sel` is set, the job reads expert id e = *sel and
    // uses w + e*w_sel_stride, aux + e*aux_sel_stride (one bank of equally shaped matrices).
    const uint32_t *sel;
    uint64_t w_sel_stride, aux_sel_stride;
    // Optional batch (bf16 / Q4_K gates, MXFP4 experts shared by up to four tokens): `batch` activations x + t*x_stride
    // against the same weights, results to out + t*out_stride (strides in floats).  0 or 1 = a plain matvec.
    // See gemv_batch_capacity.  The MXFP4 matrix-core kernel's tokens sit anywhere: token 1 at x + x_stride (which may
    // wrap, i.e. be negative), tokens 2 and 3 at x + x_off[0], x + x_off[1]; results likewise with out_stride, out_off.
    uint32_t batch, pad2;
    uint64_t x_stride, out_stride;
    int64_t x_off[2], out_off[2];
    // Optional gated activation (MoE down projection, MXFP4 matrix-core kernel only): when `x_glu` is set the
    // activation is ClampedGlu(g = x[i], u = x_glu[i]) computed while the activations are prepared; x_glu == x means
    // that g and u are interleaved in x (g = x[2i], u = x[2i+1]: the result of a fused gate_up matrix walked in place).
    const float *x_glu;
    float glu_limit, glu_alpha;
    // Optional cost model of the job in the launch's pass list (MXFP4 matrix-core kernel): the job's n_pass is
    // su + tiles * cpt (a start-up allowance, then cpt units per 16-row tile); cpt == 0 means cpr units per tile, no allowance.
    uint32_t cpt, su;
    // Optional selection inside the kernel (MXFP4 matrix-core kernel, one token): when `route_logits` is set the job
    // takes the expert of rank `route_rank` of Router::select over those logits (route_n experts <= 64, route_k <= 8,
    // policy as router_select_launch) where it would read *sel, and the workgroup that opens the job also writes the
    // token's selection to route_experts / route_weights if they are set.
    const float *route_logits;
    uint32_t *route_experts;
    float *route_weights;
    uint32_t route_n, route_k, route_rank;
    int32_t route_policy;
    // Optional bias (MoE expert biases; MXFP4 kernels only): out[r] = dot + bias[r * bias_step].  With a run-time
    // selection the bias row of expert e starts e * bias_sel_stride floats further on.
    const float *bias;
    uint64_t bias_sel_stride;
    uint32_t bias_step;
    // Experts in the bank: a selected id >= sel_count contributes nothing (the job writes zeros, no bias; in a folded
    // job that expert's share is dropped) and no byte of the bank is read through it.  0 = unchecked.
    uint32_t sel_count;
    // Optional fold over experts (MXFP4 matrix-core kernel, MoE down projection of one token): when `combine_w` is set
    // the job's `batch` activations (x, x + x_stride, x + x_off[..]) belong to `batch` <= 4 DIFFERENT experts
    // sel[0..batch) of the bank, and the single result row is sum_q combine_w[q] * (W_{sel[q]} . act_q + bias_{sel[q]}):
    // activation q is scaled by its weight before it meets the matrix, so the sum forms in the accumulators.
    const float *combine_w;
    // Optional router bias [route_n], added to route_logits before the selection (it changes which experts win).
    const float *route_bias;
    // Optional (matrix-core Q4_K kernels only): bytes from one weight row to the next when the job covers a column
    // range of a wider matrix — w points at the range's first super-block of row 0.  0 = rows are packed (row_bytes).
    uint64_t row_stride;
};
static_assert(sizeof(GemvJob) % 16 == 0, "the descriptor is a whole number of 16-byte words (moe_plan_kernel stores it that way)");

struct GemvLaunch {
    const GemvJob *table;  // device table, or null to use `inl`
    GemvJob inl[kInlineJobs];
    uint64_t total_passes;
    uint32_t n_jobs;
    uint32_t pad;
    // Optional: the job count and pass total live in device memory ({n_jobs, total_passes}, written by a kernel
    // earlier on the stream) and override the two fields above.  MXFP4 matrix-core kernel only.
    const uint32_t *dyn;
    // Optional: the first job of every workgroup's share ([grid] indices in device memory), so that a workgroup need not
    // search the jobs' pass ranges for it.
    const uint32_t *wg_first;
};

bool gemv_job_geometry(GemvJob &j, uint32_t threads);
// Second pass of the share-out's cost model over the jobs of one launch, once the grid is known (the matrix-core Q4_K
// kernels: a share's set-up is spread over its tiles).  True when costs (n_pass) changed: pass_begin is the caller's to redo.
bool gemv_refine_costs(GemvJob *jobs, size_t n, uint32_t grid);
uint32_t gemv_pick_threads(const GemvJob *jobs, size_t n);
size_t gemv_lds_bytes(const GemvJob *jobs, size_t n, uint32_t threads);
int gemv_effective_kind(const GemvJob &j);
uint32_t gemv_batch_capacity(int kind, uint64_t k);  // activations one job may carry (1: no batched kernel for this shape)
uint32_t gemv_launch_param(const GemvJob *jobs, size_t n);  // goes into GemvLaunch::pad
uint32_t gemv_wgs_per_cu(int kind, uint32_t threads, size_t lds, uint32_t dflt);
hipError_t gemv_launch(hipStream_t stream, int kind, const GemvLaunch &L, uint32_t threads, uint32_t grid, size_t lds);
hipError_t copy_launch(hipStream_t stream, const void *src, void *dst, size_t bytes, uint32_t grid);
hipError_t read_launch(hipStream_t stream, const void *src, uint32_t *sink, size_t bytes, uint32_t grid);

// top-K by |score| (or by value) over rows of a [batch, n] score matrix
constexpr uint32_t kTopkMaxK = 16384;  // winners the selection kernel orders per row (above 64: a bitonic sort in LDS, 8 bytes per winner)
hipError_t topk_launch(hipStream_t stream, const float *scores, uint32_t batch, uint32_t n, uint32_t k,
                       bool by_abs, uint32_t *idx_out, float *val_out, uint32_t *count_out, int *nan_flag,
                       void *workspace, size_t workspace_bytes);
size_t topk_workspace_bytes(uint32_t batch, uint32_t n, uint32_t k);

// encoders and the synthetic data generator
hipError_t quantize_q4_k_launch(hipStream_t s, const float *src, size_t n, uint8_t *dst);
hipError_t quantize_q6_k_launch(hipStream_t s, const float *src, size_t n, uint8_t *dst);
hipError_t quantize_q8_0_launch(hipStream_t s, const float *src, size_t n, uint8_t *dst);
hipError_t quantize_mxfp4_launch(hipStream_t s, const float *src, size_t rows, size_t k, uint8_t *packed,
                                 uint8_t *scales, const uint8_t *log2_up_table);
hipError_t f32_to_bf16_launch(hipStream_t s, const float *src, size_t n, uint16_t *dst);
hipError_t quantize_q4_0_launch(hipStream_t s, const float *src, size_t n, uint8_t *dst);
// Q8_K activation of n elements in its device layout: [n int8 codes | n/256 f32 scales | n/32 i16 sub-block sums]
inline size_t q8k_bytes(size_t n) { return n + (n / 256) * 4 + (n / 32) * 2; }
hipError_t quantize_x_to_q8k_launch(hipStream_t s, const float *src, size_t n, uint8_t *dst);
hipError_t quantize_to_q8_launch(hipStream_t s, const float *src, size_t n, int8_t *q8, float *scales);
hipError_t fill_normal_launch(hipStream_t s, float *dst, size_t n, uint64_t seed, float sigma);

// batched-prefill Q4_K GEMM (f16 MFMA over the integer weights, fp32 accumulate)
// integer-weight formulation: activations prepared once (per-token scale, f16 terms, sub-block sums)
hipError_t q4k_gemm_prep_launch(hipStream_t s, const void *x, int x_is_bf16, uint32_t hidden, uint32_t seq, uint16_t *xh, uint16_t *xl,
                                uint16_t *sx, float *tok_scale, int *any_lo, const uint8_t *w, uint32_t rows, int *rexp);
hipError_t q4k_gemm_f16_launch(hipStream_t s, const uint8_t *w, const uint16_t *xh, const uint16_t *sx, const int *rexp, const float *tok_scale,
                               float *out, uint32_t rows, uint32_t hidden, uint32_t seq, int with_mins, int accumulate, uint32_t splits,
                               float *partial);
uint32_t q4k_gemm_splits(uint32_t rows, uint32_t hidden, uint32_t seq, uint32_t cu_count);  // partial: [splits][seq][rows] floats

// One token through a bank of MXFP4 experts, a launch per projection stage (moe1_launch): a small argument block
// instead of a job table, so a workgroup's first loads leave as soon as the kernel starts.
constexpr uint32_t kMoe1MaxK = 4;  // selected experts per token
struct Moe1Args {
    // The token's selection.  With `logits` set every wavefront selects for itself (Router::select over n_experts <= 64
    // logits, policy as router_select_launch) and workgroup 0 writes experts / weights; without, both are read.
    const float *logits, *router_bias;
    uint32_t *experts;
    float *weights;
    uint32_t n_experts, k;
    int32_t policy;
    uint32_t n_mats;        // matrices per expert in this stage: 2 = gate and up apart, 1 = fused gate_up / down
    // Expert 0's matrices; expert e's start e * stride bytes further on.  An expert id >= n_experts contributes nothing.
    const uint8_t *w[2], *aux[2];
    uint64_t w_stride, aux_stride;
    const float *bias[2];   // optional; expert e's row e * bias_stride floats further on, element r at r * bias_step
    uint64_t bias_stride;
    uint32_t bias_step;
    uint32_t rows, kdim;    // of every matrix
    // Activations: gate/up stage: the token (`x`, the same for every expert).  Down stage: slot q's gate/up results at
    // x + q * x_slot_stride and x_glu + q * x_slot_stride (x_glu == x: interleaved g0 u0 g1 u1 ...), gated on the way in.
    const float *x, *x_glu;
    uint64_t x_slot_stride;
    float glu_limit, glu_alpha;
    // Results: gate/up stage: matrix m of slot q to out[m] + q * out_slot_stride; down stage: out[0], the weighted sum.
    float *out[2];
    uint64_t out_slot_stride;
    uint32_t cw, nw, stages;  // 128-element steps per wavefront, working wavefronts, ring slots per wavefront (3 or 5)
    uint32_t terms_kpad;      // elements per (term, slot) row of `terms`
    uint32_t tile_rows;       // result rows per tile, 1..16 (0: 16); even where `terms` is written
    uint32_t pad;
    // Optional hand-over between the stages (fused interleaved gate_up only): the gate/up stage writes the gated
    // activation of slot q, element i, as its three bf16 terms terms[(t * k + q) * terms_kpad + i] instead of
    // the raw results; the down stage reads its operands from there (and glu_limit / glu_alpha belong to the gate/up
    // stage then).
    uint16_t *terms;
};
bool moe1_geometry(Moe1Args &A, uint32_t *threads, size_t *lds);  // fills cw / nw / stages; false: not served
hipError_t moe1_launch(hipStream_t s, const Moe1Args &A, bool down, uint32_t grid, uint32_t threads, size_t lds);

// MoE helpers
constexpr uint32_t kRouterMaxExperts = 256;      // the selection kernel and the planner (four logits per lane)
constexpr uint32_t kRouterInLaunchExperts = 64;  // a matvec launch that selects for itself (one logit per lane)
hipError_t router_select_launch(hipStream_t s, const float *logits, const float *bias, uint32_t tokens, uint32_t n_experts, uint32_t k,
                                int policy, uint32_t *experts, float *weights);
// (logits != nullptr: the kernel selects the experts itself first — at most kRouterMaxExperts, top-kRouterMaxK — and writes experts / weights)
hipError_t moe_plan_launch(hipStream_t s, const float *logits, const float *router_bias, int policy, float *weights, uint32_t *experts,
                           uint32_t slots, uint32_t k, uint32_t n_experts, const GemvJob &tg,
                           const GemvJob &tu, const GemvJob &td, uint64_t gu_w_stride, uint64_t gu_s_stride, uint64_t dn_w_stride,
                           uint64_t dn_s_stride, uint32_t hidden, uint32_t inter, bool fused, uint32_t group, uint32_t g_grid, uint32_t d_grid,
                           GemvJob *gu_table, uint32_t *gu_hdr, GemvJob *dn_table, uint32_t *dn_hdr, uint32_t *gu_first, uint32_t *dn_first);
hipError_t clamped_glu_interleaved_launch(hipStream_t s, const float *gu, float *h, size_t n, float limit, float alpha);
hipError_t clamped_glu_launch(hipStream_t s, const float *g, const float *u, float *h, size_t n, float limit, float alpha);
hipError_t expert_scale_launch(hipStream_t s, float *weights, const uint32_t *experts, const float *scale, uint32_t n, uint32_t n_scale);
// the k-quant expert path: rows -> Q8_K activations of their own (zero-padded to `cols`), the gated activation of every
// slot -> Q8_K, and the weighted sum with the experts' down bias (rule: 0 ClampedGlu, 1 Gated(gelu_tanh), 2 Gated(silu))
hipError_t quantize_rows_to_q8k_launch(hipStream_t s, const float *src, size_t src_stride, uint32_t src_cols, uint32_t cols, uint32_t rows,
                                       uint8_t *dst, size_t dst_stride);
hipError_t moe_kq_act_q8k_launch(hipStream_t s, const float *g, const float *u, uint32_t inter, uint32_t inter_padded, uint32_t slots,
                                 const uint32_t *experts, uint32_t n_experts, const float *gub, int rule, float limit, float alpha, uint8_t *dst,
                                 size_t dst_stride);
hipError_t moe_kq_route_quant_launch(hipStream_t s, const float *logits, const float *bias, uint32_t tokens, uint32_t n_experts, uint32_t k, int policy,
                                     const float *scale, uint32_t *experts, float *weights, const float *src, size_t src_stride, uint32_t src_cols,
                                     uint32_t cols, uint8_t *dst, size_t dst_stride);
hipError_t pad_rows_f32_launch(hipStream_t s, const float *src, size_t src_stride, uint32_t src_cols, uint32_t cols, uint32_t rows, float *dst);
hipError_t moe_act_f32_launch(hipStream_t s, const float *g, const float *u, uint32_t inter, uint32_t slots, const uint32_t *experts, uint32_t n_experts,
                              const float *gub, int rule, float limit, float alpha, float *act, size_t act_stride);
hipError_t weighted_sum_bias_launch(hipStream_t s, const float *d, const float *weights, const uint32_t *experts, uint32_t n_experts,
                                    const float *bias, float *out, uint32_t tokens, uint32_t k, uint32_t hidden);
hipError_t weighted_sum_launch(hipStream_t s, const float *d, const float *weights, const uint32_t *experts, uint32_t n_experts, float *out,
                               uint32_t tokens, uint32_t k, uint32_t hidden);

}  // namespace larql
