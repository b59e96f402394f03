/*
 * larql_hip.h — C ABI of the MI355X (gfx950) backend for LARQL's quantised
 * decode path.
 *
 * This is the boundary a `larql-compute` backend crate binds over FFI: each
 * entry point serves one method of the reference's `ComputeBackend` trait
 * family (or one free function on the same path) and cites it.  Paths are
 * relative to the reference checkout, under crates/.
 *
 * Conventions
 *   - Plain C: pointers, sizes, no C++ or framework types.
 *   - Return value: LARQL_OK (the reference's `Some`), LARQL_UNSUPPORTED or
 *     LARQL_REFUSED_SHAPE (both map to the reference's `None`: the caller falls
 *     back; the output is left untouched), or a negative LARQL_E_* device error
 *     (also `None`; `larql_hip_last_error` gives the text).
 *   - "Host tier" entry points take host slices, exactly like the trait: the
 *     weight slice is served from a device-resident copy when it lies inside a
 *     region registered with larql_hip_register_weight_region, and is uploaded
 *     for the call otherwise.  Activations and outputs are copied per call.
 *   - "Device tier" entry points (larql_hip_dev_*) take device pointers that
 *     are already resident in HBM and enqueue on the context's stream without
 *     synchronising; weight pointers must be 16-byte aligned.
 *   - A context is bound to one GPU and one stream.  Calls on one context are
 *     serialised by an internal lock (the trait requires Send + Sync).
 */
#ifndef LARQL_HIP_H
#define LARQL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct larql_hip_ctx larql_hip_ctx;

enum {
    LARQL_OK = 0,
    LARQL_UNSUPPORTED = 1,   /* backend has no kernel for the request -> None */
    LARQL_REFUSED_SHAPE = 2, /* operands inconsistent (KernelShapeError)  -> None */
    LARQL_E_DEVICE = -1,     /* HIP runtime error */
    LARQL_E_NO_DEVICE = -2,  /* no usable GPU (BackendSelectError::NoDevice) */
    LARQL_E_ARG = -3,        /* null pointer / bad handle */
    LARQL_E_NAN = -4         /* NaN score in a top-K (the reference panics) */
};

/* QuantFormat — larql-compute/src/pipeline/quant_format/mod.rs:19-62 (same order). */
enum {
    LARQL_FMT_Q4_0 = 0, LARQL_FMT_Q4_K = 1, LARQL_FMT_Q4_KF = 2, LARQL_FMT_Q5_K = 3,
    LARQL_FMT_Q6_K = 4, LARQL_FMT_Q8_0 = 5, LARQL_FMT_BF16 = 6, LARQL_FMT_F16 = 7,
    LARQL_FMT_F32 = 8, LARQL_FMT_I2S = 9, LARQL_FMT_MXFP4 = 10,
    /* ggml's 34-byte Q8_0 block (f16 scale inside the block).  Not the trait's
     * QuantFormat::Q8_0, which is int8 codes + external f32 scales
     * (larql-compute/src/cpu/kquant_gemv.rs:1-12). */
    LARQL_FMT_GGML_Q8_0 = 100,
    /* Q4_K weights against a Q8_K activation (the integer-dot decode path,
     * larql-compute/src/cpu/ops/q4k_q8k_dot): in a device-tier job `x` is the
     * activation in the layout larql_hip_dev_quantize_x_to_q8k writes. */
    LARQL_FMT_Q4_K_Q8K = 101,
    /* Q6_K weights against the same activation layout (cpu/ops/q4k_q8k_dot/q6k.rs). */
    LARQL_FMT_Q6_K_Q8K = 102
};

/* Capability — larql-compute/src/backend/capability.rs:22-102 (the ones this
 * backend answers true for; every other value answers false). */
enum { LARQL_CAP_F32_GEMV = 0, LARQL_CAP_F16_GEMV = 1, LARQL_CAP_QUANT_MATVEC = 2 };

/* ---- lifecycle / metadata ------------------------------------------------ */

/* Constructor a binary registers in its backend registry
 * (larql-cli/src/backend_select.rs:26-41; backend/factory.rs:174-192).
 * LARQL_E_NO_DEVICE when the device does not exist or is not gfx950. */
int  larql_hip_create(larql_hip_ctx **out, int device);
void larql_hip_destroy(larql_hip_ctx *ctx);
/* ComputeBackend::name / device_info — backend/mod.rs:51-57. */
const char *larql_hip_name(const larql_hip_ctx *ctx);
const char *larql_hip_device_info(const larql_hip_ctx *ctx);
/* QuantMatVec::supports_quant — backend/quant_matvec.rs:367-370. */
int  larql_hip_supports_quant(const larql_hip_ctx *ctx, int format);
/* ComputeBackend::supports — backend/mod.rs:59-67. */
int  larql_hip_supports(const larql_hip_ctx *ctx, int capability);
const char *larql_hip_last_error(const larql_hip_ctx *ctx);

/* ComputeBackend::register_weight_region / seal_weight_regions —
 * backend/mod.rs:68-89.  The region must never move and must outlive the
 * context; registering the same base twice is a no-op.  The bytes are
 * uploaded once and later host-tier calls whose weight slice lies inside the
 * region use the resident copy. */
int  larql_hip_register_weight_region(larql_hip_ctx *ctx, const uint8_t *region, size_t len);
int  larql_hip_seal_weight_regions(larql_hip_ctx *ctx);
int  larql_hip_clear_weight_regions(larql_hip_ctx *ctx);

/* MatMul::submission_clock — backend/matmul.rs:34-42,216-218.  One host-tier
 * call is one submission; gpu_nanos is device-event time of its kernels. */
typedef struct {
    uint64_t submissions;
    uint64_t commit_to_done_nanos;
    uint64_t gpu_nanos;
} larql_hip_submission_clock;
int  larql_hip_get_submission_clock(larql_hip_ctx *ctx, larql_hip_submission_clock *out);

/* ---- host tier: quantised matvec (QuantMatVec) ---------------------------- */

/* QuantMatVec::q4k_matvec — backend/quant_matvec.rs:252-260; CPU semantics
 * cpu/mod.rs:95-114 + q4_common/matvec_f32.rs:37-106: out_len == num_rows,
 * x_len == hidden, hidden % 256 == 0, w_len >= rows*(hidden/256)*144, else
 * REFUSED_SHAPE; zero dims write zeros. */
int larql_hip_q4k_matvec(larql_hip_ctx *ctx, const uint8_t *q4k, size_t q4k_len,
                         const float *x, size_t x_len, size_t num_rows, size_t hidden,
                         float *out, size_t out_len);

/* QuantMatVec::q6k_matvec — backend/quant_matvec.rs:335-345; CPU semantics
 * cpu/mod.rs:133-141 + cpu/ops/q6k_matvec.rs:45-91 (210-byte super-blocks in ggml's
 * planar layout, larql-models/src/quant/ggml/q6_k.rs:19-40).  x_len == hidden,
 * hidden % 256 == 0, w_len >= rows*(hidden/256)*210, else REFUSED_SHAPE (the CPU
 * path indexes out of range there); zero dims write zeros. */
int larql_hip_q6k_matvec(larql_hip_ctx *ctx, const uint8_t *q6k, size_t q6k_len,
                         const float *x, size_t x_len, size_t num_rows, size_t hidden, float *out);
/* quantize_x_to_q8k — larql-compute/src/cpu/ops/q4k_q8k_dot/q8k_activation.rs:84-109
 * (Q8KActivation { qs, d, sums }): n % 256 == 0, qs[n], d[n/256], sums[n/32].
 * Bit-exact with the reference. */
int larql_hip_quantize_x_to_q8k(larql_hip_ctx *ctx, const float *x, size_t n, int8_t *qs, float *d, int16_t *sums);
/* q4k_q8k_matvec_into / q4k_q8k_matvec_parallel with format "Q4_K" —
 * cpu/ops/q4k_q8k_dot/dispatch.rs:15-148; value and bits of q4k_q8k_matvec_scalar
 * (q4k_scalar.rs:15-84), which every SIMD kernel of the reference equals bit for
 * bit and so does this one.  Shape rule KernelShapeError::check
 * (cpu/ops/kernel_shape.rs:47-75): out_len == rows, qs_len == cols, cols % 256 == 0,
 * q4k_len >= rows*(cols/256)*144, else REFUSED_SHAPE with `out` untouched; zero
 * dims write zeros.  Rows of more than 10240 elements (the down projections of the larger models) are served as
 * column ranges whose partial sums are added in range order: the integer sums are the same, the f32 accumulation
 * meets in another order than the scalar kernel's single chain (about 1e-7 relative instead of bit-exact). */
int larql_hip_q4k_q8k_matvec(larql_hip_ctx *ctx, const uint8_t *q4k, size_t q4k_len, const int8_t *qs, size_t qs_len,
                             const float *d, const int16_t *sums, size_t num_rows, size_t cols, float *out, size_t out_len);
/* q4k_q8k_gate_up_into — cpu/ops/q4k_q8k_dot/gate_up.rs:30-57 (shape checks :68-87):
 * gate and up rows against one Q8_K activation in one launch; each output is
 * bit-identical to larql_hip_q4k_q8k_matvec on its matrix (the reference holds its
 * fused kernels to the scalar one bit for bit).  Both shape rules are checked
 * before anything is written. */
int larql_hip_q4k_q8k_gate_up(larql_hip_ctx *ctx, const uint8_t *gate_w, size_t gate_len, const uint8_t *up_w, size_t up_len,
                              const int8_t *qs, size_t qs_len, const float *d, const int16_t *sums, size_t num_rows,
                              size_t cols, float *gate_out, float *up_out, size_t out_len);
/* q4k_q8k_gemm_into — cpu/ops/q4k_q8k_dot/gemm.rs:42-112: out[s*rows + r] = W[r,:] . X[s,:]
 * for `seq` activation rows quantised to Q8_K (`qs` seq*cols codes, `d` seq*cols/256,
 * `sums` seq*cols/32, row after row); every activation row bit-identical to the
 * row-at-a-time matvec (gemm.rs:141-170).  One launch, one job per activation row.
 * The reference asserts out_len == seq*rows, cols % 256 == 0 and the slab length;
 * here those are REFUSED_SHAPE. */
int larql_hip_q4k_q8k_gemm(larql_hip_ctx *ctx, const uint8_t *q4k, size_t q4k_len, const int8_t *qs, const float *d,
                           const int16_t *sums, size_t seq, size_t num_rows, size_t cols, float *out, size_t out_len);
/* q6k_q8k_matvec_into / q4k_q8k_matvec_parallel with format "Q6_K" —
 * cpu/ops/q4k_q8k_dot/q6k.rs:15-92, dispatch.rs:100-148: per super-block
 * acc += d_w*d_y*(f32)(sum over the 16 groups of scale_g * dot(q6 - 32, q8)), in
 * super-block order; bit-exact with q6k_q8k_matvec_scalar (the reference's NEON
 * kernel is checked against it to 1e-3).  The activation's `sums` are not used by
 * this format.  Shape rule as above with 210-byte blocks. */
int larql_hip_q6k_q8k_matvec(larql_hip_ctx *ctx, const uint8_t *q6k, size_t q6k_len, const int8_t *qs, size_t qs_len,
                             const float *d, size_t num_rows, size_t cols, float *out, size_t out_len);
/* QuantMatVec::q4k_dual_matvec — quant_matvec.rs:287-296; q4_common/dual.rs:22-167. */
int larql_hip_q4k_dual_matvec(larql_hip_ctx *ctx, const uint8_t *q4k_a, size_t a_len,
                              const uint8_t *q4k_b, size_t b_len,
                              const float *x, size_t x_len, size_t num_rows, size_t hidden,
                              float *out_a, float *out_b, size_t out_len);
/* QuantMatVec::q4k_matmul — quant_matvec.rs:324-333; q4_common/matmul.rs:20-139.
 * out is [seq_len, num_rows] row-major; out_len / x_len must be seq*rows / seq*hidden
 * (else REFUSED_SHAPE).  A zero dimension or a bad shape zero-fills out, as the CPU
 * does (matmul.rs:89-98): hidden == 0 leaves seq*rows zeros. */
int larql_hip_q4k_matmul(larql_hip_ctx *ctx, const uint8_t *q4k, size_t q4k_len,
                         const float *x, size_t x_len, size_t num_rows, size_t hidden,
                         size_t seq_len, float *out, size_t out_len);
/* QuantMatVec::q4k_matvec_topk — quant_matvec.rs:268-277: up to top_k
 * (row, score) pairs by value descending, non-finite scores skipped
 * (lm_head/knn.rs:315-386).  idx_out/score_out hold top_k entries (all copied back);
 * *n_out receives how many of them are hits.  top_k up to 16384. */
int larql_hip_q4k_matvec_topk(larql_hip_ctx *ctx, const uint8_t *q4k, size_t q4k_len,
                              const float *x, size_t x_len, size_t num_rows, size_t hidden,
                              size_t top_k, uint32_t *idx_out, float *score_out, size_t *n_out);
/* QuantMatVec::q4_matvec — quant_matvec.rs:162-171; the CPU path is the C
 * kernel csrc/q4_dot.c:176-207 behind cpu/ops/q4_matvec.rs:24-86.  Q4_0
 * weights (18-byte blocks) x a Q8 activation (int8 + one f32 scale per 32).
 * Bad lengths are REFUSED_SHAPE (the CPU asserts). */
int larql_hip_q4_matvec(larql_hip_ctx *ctx, const uint8_t *q4, size_t q4_len,
                        const int8_t *q8_x, size_t q8_len, const float *q8_scales, size_t n_scales,
                        size_t num_rows, size_t hidden, float *out);
/* q8_0_gemv (ggml 34-byte blocks) — cpu/kquant_gemv.rs:67-109, reached via
 * KQuant::gemv (larql-vindex/src/format/vindex3/represent/kquant.rs:285-298):
 * k > 0, k % 32 == 0, x_len == k and blocks_len == n*(k/32)*34 exactly. */
int larql_hip_q8_0_gemv(larql_hip_ctx *ctx, const uint8_t *blocks, size_t blocks_len,
                        const float *x, size_t x_len, size_t n, size_t k, float *out);
/* lm_head KNN over a ggml Q8_0 head — larql-vindex/src/index/storage/lm_head/knn.rs:126-185 with top_k_sorted
 * (:315-386): larql_hip_q8_0_gemv followed by the top_k (<= 16384) largest scores by value, descending, non-finite
 * scores skipped; the vocabulary's scores stay on the device (1 MB per token for a 262144-row head).  Shape rule of
 * larql_hip_q8_0_gemv.  idx_out/score_out hold top_k entries; *n_out receives how many of them are hits. */
int larql_hip_q8_0_gemv_topk(larql_hip_ctx *ctx, const uint8_t *blocks, size_t blocks_len, const float *x, size_t x_len,
                             size_t n, size_t k, size_t top_k, uint32_t *idx_out, float *score_out, size_t *n_out);
/* QuantMatVec::quant_matvec — quant_matvec.rs:50-98: format dispatch.
 * Q4_K/Q4_KF -> q4k_matvec, Q6_K -> q6k_matvec, Q4_0 -> quantize_to_q8 + q4_matvec,
 * everything else UNSUPPORTED (as the trait default answers None). */
int larql_hip_quant_matvec(larql_hip_ctx *ctx, int format, const uint8_t *weights, size_t w_len,
                           const float *x, size_t x_len, size_t num_rows, size_t hidden, float *out);

/* QuantMatVec::quant_matvec_q8_input — quant_matvec.rs:100-151: the activation arrives as Q8 (int8 codes + one f32
 * scale per 32).  Q4_0 -> q4_matvec; Q4_K / Q4_KF / Q6_K -> dequantise_q8 (quant_matvec.rs:24-39) + the f32 path;
 * the trait's own Q8_0 layout (q8_matvec: None on the CPU backend too), Q5_K, I2S, MXFP4 and the float formats
 * UNSUPPORTED. */
int larql_hip_quant_matvec_q8_input(larql_hip_ctx *ctx, int format, const uint8_t *weights, size_t w_len, const int8_t *q8_x,
                                    size_t q8_len, const float *q8_scales, size_t n_scales, size_t num_rows, size_t hidden,
                                    float *out);

/* ---- host tier: dense / MXFP4 gemv (MatMul) -------------------------------- */

/* MatMul::f32_gemv_force / f16_gemv_force / bf16_gemv_force —
 * backend/matmul.rs:66-170.  w is [n, k] row-major; w_len in bytes must be
 * n*k*sizeof(elem), x_len >= k.  The non-force variants apply the peer's flop
 * threshold (larql-compute-metal/src/trait_impl/matmul.rs:33-88) and answer
 * UNSUPPORTED below it so the caller keeps its BLAS path. */
int larql_hip_f32_gemv(larql_hip_ctx *ctx, const float *w, size_t w_len, const float *x, size_t x_len,
                       size_t n, size_t k, float *out, int force);
int larql_hip_f16_gemv(larql_hip_ctx *ctx, const uint8_t *w_f16, size_t w_len, const float *x, size_t x_len,
                       size_t n, size_t k, float *out, int force);
int larql_hip_bf16_gemv(larql_hip_ctx *ctx, const uint8_t *w_bf16, size_t w_len, const float *x, size_t x_len,
                        size_t n, size_t k, float *out, int force);
/* MatMul::bf16_gemv_multi / f16_gemv_multi — backend/matmul.rs:151-194: several [n_i, k_i] matrices against one
 * x as ONE submission (groups of up to 8 matrices per launch); every k_i must equal x_len and w_len[i] >= n_i*k_i*2,
 * any bad matrix refuses the whole batch before anything is written, n_mats == 0 is OK (Some(vec![])); results are
 * in argument order and bit-identical to the sequential *_gemv_force calls. */
int larql_hip_bf16_gemv_multi(larql_hip_ctx *ctx, size_t n_mats, const uint8_t *const *w_bf16, const size_t *w_len,
                              const size_t *n, const size_t *k, const float *x, size_t x_len, float *const *out);
int larql_hip_f16_gemv_multi(larql_hip_ctx *ctx, size_t n_mats, const uint8_t *const *w_f16, const size_t *w_len,
                             const size_t *n, const size_t *k, const float *x, size_t x_len, float *const *out);
/* MatMul::mxfp4_gemv — backend/matmul.rs:220-235: k % 32 == 0, x_len >= k,
 * packed_len >= n*(k/32)*16, scales_len >= n*(k/32). */
int larql_hip_mxfp4_gemv(larql_hip_ctx *ctx, const uint8_t *packed, size_t packed_len,
                         const uint8_t *scales, size_t scales_len,
                         const float *x, size_t x_len, size_t n, size_t k, float *out);
/* MatMul::mxfp4_gemv_multi — backend/matmul.rs:237-251: several matrices, one
 * x, one submission; any bad matrix refuses the whole batch; n_mats == 0 is OK.
 * Results are bit-identical to the single calls. */
int larql_hip_mxfp4_gemv_multi(larql_hip_ctx *ctx, size_t n_mats,
                               const uint8_t *const *packed, const size_t *packed_len,
                               const uint8_t *const *scales, const size_t *scales_len,
                               const size_t *n, const size_t *k,
                               const float *x, size_t x_len, float *const *out);

/* ---- host tier: gate-KNN (larql-vindex) ------------------------------------- */

/* VectorIndex::gate_knn / gate_walk / gate_knn_batch —
 * larql-vindex/src/index/compute/gate_knn/dispatch.rs:22-121,256-304 with
 * top_k_by_abs (gate_knn/mod.rs:50-108): score `batch` residuals [batch,hidden]
 * against the gate matrix [n_features, hidden] stored as `format`
 * (F32, F16, BF16, Q4_K or Q4_0), keep the min(top_k, n_features) largest
 * |score| per position, sorted by |score| descending (ties: lower index
 * first).  idx_out/score_out are [batch, top_k] (all of it is written; entries
 * past a position's count are unspecified); n_out is [batch] and receives the
 * number of hits of each position.  top_k up to 16384 (top_k_by_abs takes any K; WalkFfn's
 * default is every feature, larql-inference/src/vindex/walk_ffn/mod.rs:186-190);
 * above that LARQL_UNSUPPORTED.  LARQL_E_NAN on a NaN score. */
int larql_hip_gate_knn(larql_hip_ctx *ctx, int format, const uint8_t *gate, size_t gate_len,
                       const float *x, size_t batch, size_t n_features, size_t hidden, size_t top_k,
                       uint32_t *idx_out, float *score_out, size_t *n_out);
/* gate_scores_batch_backend — gate_knn/scores_batch.rs:30-57: the full score
 * matrix [batch, n_features]. */
int larql_hip_gate_scores(larql_hip_ctx *ctx, int format, const uint8_t *gate, size_t gate_len,
                          const float *x, size_t batch, size_t n_features, size_t hidden, float *scores_out);

/* ---- device tier ------------------------------------------------------------ */
/* Memory and ordering helpers for callers that keep operands in HBM. */
int larql_hip_malloc(larql_hip_ctx *ctx, void **dptr, size_t bytes);
int larql_hip_free(larql_hip_ctx *ctx, void *dptr);
int larql_hip_memcpy_h2d(larql_hip_ctx *ctx, void *dst, const void *src, size_t bytes);
int larql_hip_memcpy_d2h(larql_hip_ctx *ctx, void *dst, const void *src, size_t bytes);
int larql_hip_memset(larql_hip_ctx *ctx, void *dst, int value, size_t bytes);
int larql_hip_synchronize(larql_hip_ctx *ctx);
/* Device-event timing on the context's stream (the stream the kernels run on). */
int larql_hip_event_create(larql_hip_ctx *ctx, void **event);
int larql_hip_event_record(larql_hip_ctx *ctx, void *event);
int larql_hip_event_elapsed_ms(larql_hip_ctx *ctx, void *start, void *stop, float *ms);
int larql_hip_event_destroy(larql_hip_ctx *ctx, void *event);

/* Plain streaming kernels: copy `bytes` from src to dst with 16-byte loads
 * and stores, or (dst == NULL) only read src.  No counterpart in the
 * reference: they are the yardstick for achievable HBM bandwidth and for
 * scaling profiler byte counters. */
int larql_hip_dev_copy(larql_hip_ctx *ctx, void *dst, const void *src, size_t bytes);

/* One matvec on resident operands: out[rows] = W[rows,k] . x[k].
 * format: Q4_K, GGML_Q8_0, MXFP4 (aux = e8m0 scale stream), BF16, F16, F32,
 * Q4_0 (x is then the f32 activation, quantised to Q8 on the device as
 * QuantMatVec::quant_matvec does for Q4_0).  Same arithmetic as the host
 * tier. */
int larql_hip_dev_matvec(larql_hip_ctx *ctx, int format, const void *w, const void *aux,
                         const float *x, size_t rows, size_t k, float *out);

/* Several matvecs in ONE launch ("one submission", as MatMul::*_gemv_multi
 * and Metal's decode command buffer do, backend/matmul.rs:151-194): each job
 * has its own format, operands and shape.  Jobs must be independent of one
 * another (no job reads another job's out). */
typedef struct {
    int32_t format;
    int32_t reserved;
    const void *w;
    const void *aux;     /* MXFP4 scale stream, else NULL */
    const float *x;
    float *out;
    uint64_t rows;
    uint64_t k;
} larql_hip_matvec_job;
int larql_hip_dev_matvec_batch(larql_hip_ctx *ctx, const larql_hip_matvec_job *jobs, size_t n_jobs);

/* A recorded submission: the jobs' geometry and device job tables are
 * prepared once, and every run enqueues the same launches (one per format
 * present) on the context's stream without synchronising — what the Metal
 * peer's decode command buffer is to its per-call matvecs
 * (larql-compute-metal backend/decode.rs:338).  Operand pointers are captured
 * by value; the buffers may be rewritten between runs. */
typedef struct larql_hip_plan larql_hip_plan;
int  larql_hip_plan_create(larql_hip_ctx *ctx, const larql_hip_matvec_job *jobs, size_t n_jobs, larql_hip_plan **out);
int  larql_hip_plan_run(larql_hip_ctx *ctx, larql_hip_plan *plan);
int  larql_hip_plan_launch_count(const larql_hip_plan *plan);
void larql_hip_plan_destroy(larql_hip_ctx *ctx, larql_hip_plan *plan);

/* Plans that depend on one another, in order, as one replayable submission: what a token's stages are to the decode
 * loop (q,k,v | o | gate,up | down per layer, each reading what the stage before wrote).  The peers submit a token's
 * matvecs as one command buffer (DecodeBackend::decode_token, larql-compute/src/backend/decode.rs:219-); here the
 * plans' launches are recorded once into a HIP graph — a plan's launches run in order, a plan after the one before
 * it — and a run replays it on the context's stream without synchronising: the per-launch submission cost is paid
 * by the graph, not by the caller.  Creating the sequence runs the plans once.  The plans must outlive it. */
typedef struct larql_hip_sequence larql_hip_sequence;
int  larql_hip_sequence_create(larql_hip_ctx *ctx, larql_hip_plan *const *plans, size_t n_plans, larql_hip_sequence **out);
int  larql_hip_sequence_run(larql_hip_ctx *ctx, larql_hip_sequence *seq);
int  larql_hip_sequence_launch_count(const larql_hip_sequence *seq);
void larql_hip_sequence_destroy(larql_hip_ctx *ctx, larql_hip_sequence *seq);

/* Scores + top-K by |score| on resident operands (see larql_hip_gate_knn).
 * scores_scratch: [batch, n_features] f32 device buffer (also the full score
 * matrix on return); idx_out/score_out: [batch, top_k] device buffers, of which
 * the first count_out[b] entries of row b are written (min(top_k, n_features), fewer
 * when scores are NaN); count_out (device, [batch]) may be NULL.  A NaN score does not
 * stop the call — it only enqueues — but raises a flag: see larql_hip_dev_take_nan_flag. */
int larql_hip_dev_gate_knn(larql_hip_ctx *ctx, int format, const void *gate,
                           const float *x, size_t batch, size_t n_features, size_t hidden,
                           size_t top_k, float *scores_scratch, uint32_t *idx_out, float *score_out, uint32_t *count_out);
/* Waits for the context's stream, reports whether any device-tier gate-KNN / gate walk since the flag was last taken
 * met a NaN score (the host tier answers LARQL_E_NAN there, the reference panics: gate_knn/mod.rs:84) and clears the
 * flag.  The calls themselves only raise it: take it after the calls whose scores matter. */
int larql_hip_dev_take_nan_flag(larql_hip_ctx *ctx, int *flag_out);

/* larql_hip_dev_gate_knn for callers that cannot allocate (tight serving loops, harnesses that forbid hipMalloc).
 * It has no counterpart in the reference.  (It launches on the context's own stream like every other entry point:
 * it is not a call to make under a caller's graph capture.)  Same results as
 * larql_hip_dev_gate_knn, bit for bit, but the score matrix, the hit counts and the quantised activation of
 * Q4_0 gates live in a fixed array in device memory that the library holds on every GPU it runs on until the
 * process ends (larql_hip_static_scratch_bytes(), about 0.7 MiB); the call itself performs no hipMalloc /
 * hipFree, no host allocation and no table upload.  Limits (beyond them: LARQL_REFUSED_SHAPE with a message):
 * batch <= LARQL_HIP_STATIC_MAX_BATCH, batch * n_features <= LARQL_HIP_STATIC_MAX_SCORES, and for Q4_0 gates
 * hidden <= LARQL_HIP_STATIC_MAX_HIDDEN.  count_out (may be NULL): hits per position.  All calls on one GPU
 * share that GPU's array, which keeps the previous call's contents: calls that overlap on one GPU (two
 * contexts, or two streams) race; calls through one context are serialised. */
#define LARQL_HIP_STATIC_MAX_BATCH 8
#define LARQL_HIP_STATIC_MAX_SCORES 131072
#define LARQL_HIP_STATIC_MAX_HIDDEN 16384
size_t larql_hip_static_scratch_bytes(void);
/* How often calls on this context have taken device memory, gone through a staging buffer or uploaded a job table so
 * far (host-side bookkeeping, no GPU work): the number a caller checks before and after a call that must allocate
 * nothing.  No counterpart in the reference. */
int larql_hip_debug_alloc_events(larql_hip_ctx *ctx, uint64_t *out);
int larql_hip_dev_gate_knn_static(larql_hip_ctx *ctx, int format, const void *gate, const float *x, size_t batch,
                                  size_t n_features, size_t hidden, size_t top_k, uint32_t *idx_out, float *score_out,
                                  uint32_t *count_out);

/* Gate-KNN over `n_layers` layers in ONE submission — the shape of LQL WALK / DESCRIBE, where
 * every layer of the index is scored for one query (PatchedVindex::walk,
 * larql-vindex/src/patch/overlay.rs:557-562 over VectorIndex::gate_knn): one matvec launch for all
 * layers' scores and one top-K launch for all (layer, position) rows.  gates[l] is layer l's
 * [n_features, hidden] matrix; x is [batch, hidden] (x_layer_stride == 0: the same residuals
 * for every layer) or [n_layers, batch, hidden] (x_layer_stride == batch*hidden).
 * scores_scratch: [n_layers, batch, n_features]; idx_out/score_out: [n_layers, batch, top_k];
 * count_out (may be NULL): hits per row. */
int larql_hip_dev_gate_walk(larql_hip_ctx *ctx, int format, const void *const *gates, size_t n_layers, const float *x,
                            size_t x_layer_stride, size_t batch, size_t n_features, size_t hidden, size_t top_k,
                            float *scores_scratch, uint32_t *idx_out, float *score_out, uint32_t *count_out);

/* Batched-prefill GEMM on resident operands: out[seq, rows] = X[seq, hidden] . W[rows, hidden]^T,
 * W in Q4_K, X held as bf16 (the top 16 bits of each f32).  Same contraction as
 * QuantMatVec::q4k_matmul (backend/quant_matvec.rs:324-333), on f16 MFMA with fp32 accumulate: the
 * activations are exact in f16 after a per-token power-of-two scale, a weight enters as
 * f16(d 2^E sc6) * (q - 8) (E per row), the sub-blocks' offsets through the sums of the activations.
 * ~3e-4 relative L2 from the CPU value (the f16 roundings of the sub-block scales and weights);
 * larql_hip_q4k_matmul keeps exact integer sums instead (~3e-7).  hidden % 256 == 0; w and x_bf16
 * 16-byte aligned. */
int larql_hip_dev_q4k_gemm(larql_hip_ctx *ctx, const uint8_t *w, const uint16_t *x_bf16, size_t rows, size_t hidden,
                           size_t seq, float *out);
/* The same GEMM for a matrix whose rows' exponents E were computed once (they depend on the weights alone:
 * max(|d|, |dmin|/16) 2^E in [0.5, 1) over the row's super-blocks): larql_hip_dev_q4k_row_exponents fills
 * row_exp[rows] (int32, device memory), larql_hip_dev_q4k_gemm_prepared takes them and skips the pass over the
 * matrix's block headers that larql_hip_dev_q4k_gemm makes on every call.  Results are bit-identical to
 * larql_hip_dev_q4k_gemm.  (No counterpart in the reference: its q4k_matmul dequantises on the fly, matmul.rs:20-139;
 * this is the load-time half of the device-tier call.) */
int larql_hip_dev_q4k_row_exponents(larql_hip_ctx *ctx, const uint8_t *w, size_t rows, size_t hidden, int32_t *row_exp);
int larql_hip_dev_q4k_gemm_prepared(larql_hip_ctx *ctx, const uint8_t *w, const int32_t *row_exp, const uint16_t *x_bf16,
                                    size_t rows, size_t hidden, size_t seq, float *out);

/* ---- device tier: MoE expert block (MXFP4) --------------------------------------
 * router::select — larql-compute/src/ffn/expert_weight/router.rs:33-70: top-k
 * of `n_experts` logits per token (ties: first index), weights softmaxed over
 * the selected logits (policy 1, NormalisedOverSelected: GPT-OSS) or over all
 * experts (policy 0, SoftmaxThenSelect).  experts/weights are [tokens, k].
 * n_experts <= 256, k <= 8 (a launch of the expert block selects for itself up to 64
 * experts; a wider bank — 128 in the larger GPT-OSS and Gemma 4 checkpoints — goes through the
 * selection kernel first). */
int larql_hip_dev_router_select(larql_hip_ctx *ctx, const float *logits, size_t tokens, size_t n_experts, size_t k,
                                int policy, uint32_t *experts, float *weights);
/* One bank of MXFP4 experts: gate/up are [n_experts, inter, hidden] and down is
 * [n_experts, hidden, inter], each as packed nibbles + e8m0 scales (the layout
 * of MatMul::mxfp4_gemv, backend/matmul.rs:220-235, expert after expert). */
typedef struct {
    const uint8_t *gate_packed, *gate_scales, *up_packed, *up_scales, *down_packed, *down_scales;
    size_t n_experts, hidden, inter;
    float limit, alpha; /* MoeGateRule::ClampedGlu — pipeline/moe.rs:88-92 (GPT-OSS: 7, 1.702) */
    /* MoeFusedRowLayout — pipeline/moe.rs:294-332.  0 = the gate and up projections are given
     * apart (ContiguousHalves: up_* = gate_* + inter rows of the same region).  1 = Interleaved,
     * what a GPT-OSS checkpoint ships: gate_packed / gate_scales hold each expert's fused
     * [2*inter, hidden/32] rows with gate = rows 0, 2, 4, ... and up = rows 1, 3, 5, ...
     * (FusedHalf::fused_row, larql-models/src/quant/mxfp4.rs:179-191); up_* are not read.
     * The fused rows are walked in place, one pass over 2*inter rows per (token, expert). */
    int gate_up_interleaved;
    /* Biases of MoeLayerWeights — pipeline/moe.rs:505-516, read by ExpertMlp::{gate_bias, up_bias, add_down_bias}
     * (pipeline/moe.rs:150-176); each may be NULL (none).  router_bias [n_experts] is added to the router logits
     * before the selection (larql_hip_dev_moe_mxfp4_routed only).  gate_up_bias [n_experts, 2*inter] is the fused
     * row as the checkpoint ships it — gate bias j at 2j, up bias j at 2j+1 — whatever the weight layout.
     * down_bias [n_experts, hidden].  The block computes sum_s w_s * (down_e(ClampedGlu(gate_e.x + bg, up_e.x + bu)) + bd). */
    const float *router_bias, *gate_up_bias, *down_bias;
} larql_hip_mxfp4_experts;
/* The expert block of cpu_moe_forward (cpu/ops/moe/forward.rs:201-270) for
 * MXFP4 banks, which the CPU tier refuses (forward.rs:69-75): per token and
 * selected expert, gate/up matvec (+ bias) -> ClampedGlu -> down matvec (+ bias), then the
 * weighted sum in selection order.  `experts` stays on the device (the kernels
 * index the bank with it), so routing needs no host round trip; an expert id >= n_experts is skipped,
 * as the reference skips it (forward.rs:203-208).  One token with k <= 4: two launches — the down
 * projection folds the k experts and the weighted sum into one pass over the output rows (the shape of
 * the Metal peer's mxfp4g_down_combine4, larql-compute-metal/src/shaders/mxfp4_grouped_experts/kernels.rs:482-541).
 * workspace: larql_hip_moe_mxfp4_workspace_bytes(...) of device memory; workspace, x and the packed streams
 * 16-byte aligned (else LARQL_REFUSED_SHAPE). */
size_t larql_hip_moe_mxfp4_workspace_bytes(size_t tokens, size_t k, size_t hidden, size_t inter);
int larql_hip_dev_moe_mxfp4(larql_hip_ctx *ctx, const larql_hip_mxfp4_experts *bank, const float *x, size_t tokens, size_t k,
                            const uint32_t *experts, const float *weights, float *out, void *workspace, size_t workspace_bytes);
/* Router::select (ffn/expert_weight/router.rs:33-70) and the expert block above as one call: the same results as
 * larql_hip_dev_router_select followed by larql_hip_dev_moe_mxfp4, experts / weights [tokens, min(k, n_experts)]
 * written as the former writes them.  For one token the selection runs inside the first matvec launch (one launch
 * fewer: a decode step's expert block is bound by its launches, not by its bytes).  Limits as the two calls. */
int larql_hip_dev_moe_mxfp4_routed(larql_hip_ctx *ctx, const larql_hip_mxfp4_experts *bank, const float *x, size_t tokens, size_t k,
                                   const float *router_logits, int policy, uint32_t *experts, float *weights, float *out,
                                   void *workspace, size_t workspace_bytes);

/* ---- MoE layer: per-expert slices, split scale streams and the router, as MoeLayerWeights brings them ------------
 * MoeLayerWeights — larql-compute/src/pipeline/moe.rs:469-541 — hands a layer's experts over as PER-EXPERT byte slices
 * (experts_gate_up[e], experts_down[e]: mmap ranges layers/{L}/{e}/..., anywhere in memory) with the dequantisation
 * scales either inside the payload (MoeExpertScales::Inline) or as per-expert e8m0 streams index-aligned with them
 * (MoeExpertScales::Paired, moe.rs:214-238), the fused gate+up rows Interleaved or as ContiguousHalves
 * (MoeFusedRowLayout, moe.rs:294-332), and the router's own tensors.  larql_hip_moe_layer_create makes such a layer
 * resident: every slice is uploaded where the expert kernels want it (expert after expert in one region; the halves of
 * a ContiguousHalves MXFP4 bank interleaved row by row on the way up), so the caller gathers nothing.  Served: expert_data_format MXFP4 with Paired scales
 * (what a native GPT-OSS bank is; the CPU tier refuses it, cpu/ops/moe/forward.rs:69-75) and MoeGateRule::ClampedGlu;
 * MXFP4 with Inline scales is LARQL_REFUSED_SHAPE (the format keeps its exponents apart: there is nothing to read them
 * from).  Also served: expert_data_format Q4_K or Q6_K with Inline scales and ContiguousHalves rows — the per-layer
 * k-quant files of Gemma 4 26B-A4B, what cpu_moe_forward's integer path reads (cpu/ops/moe/forward.rs:160-330,
 * expert/q4k.rs:232-351): experts_gate_up[e] is [2*inter, cols] rows, gate half first, cols the stored row width (>= hidden,
 * a multiple of 256, derived from the slice length as stored_gate_up_cols does, moe.rs:659-690); experts_down[e] is
 * [hidden, ceil(inter/256)*256]; the scale tables are NULL; any LARQL_MOE_GATE_* rule.  The expert input is quantised to
 * Q8_K once per token, the gated activation once per expert, and every matvec is the integer Q4_K x Q8_K (Q6_K x Q8_K)
 * kernel, as on the CPU.  A BF16 (the legacy monolith), F16 or F32 bank takes cpu_moe_forward's f32 arm (forward.rs:246-290):
 * f32 activations, the dense matvec kernels, experts_down[e] [hidden, inter] unpadded; its rows are multiples of 16
 * elements, at most 8192 (stored wider than hidden: the expert input goes in zero-padded, as on the CPU).  An Interleaved k-quant or float bank is LARQL_REFUSED_SHAPE (the CPU tier
 * asserts the same, forward.rs:69-75); k-quant rows longer than 10240 elements and other formats LARQL_UNSUPPORTED.
 * num_experts <= 256, top_k <= 8. */
enum { LARQL_MOE_SCALES_INLINE = 0, LARQL_MOE_SCALES_PAIRED = 1 };
/* MoeGateRule (moe.rs:16-118): ClampedGlu{limit, alpha}, Gated(gelu_tanh), Gated(silu), SituGlu{beta, linear_beta}
 * (glu_limit = beta, glu_alpha = linear_beta, 0 for None), ClampedGated{limit, gelu_tanh | silu} (glu_limit = limit). */
enum { LARQL_MOE_GATE_CLAMPED_GLU = 0, LARQL_MOE_GATE_GELU_TANH = 1, LARQL_MOE_GATE_SILU = 2, LARQL_MOE_GATE_SITU_GLU = 3,
       LARQL_MOE_GATE_CLAMPED_GELU_TANH = 4, LARQL_MOE_GATE_CLAMPED_SILU = 5 };
enum { LARQL_MOE_ROWS_CONTIGUOUS_HALVES = 0, LARQL_MOE_ROWS_INTERLEAVED = 1 };
typedef struct {
    size_t num_experts, top_k, hidden, intermediate_size;
    int expert_data_format;                      /* LARQL_FMT_* of the per-expert slices */
    int fused_row_layout;                        /* LARQL_MOE_ROWS_* */
    int expert_scales;                           /* LARQL_MOE_SCALES_* */
    const uint8_t *const *experts_gate_up;       /* [num_experts]: expert e's fused [2*inter, hidden/32, 16] nibble bytes */
    const size_t *experts_gate_up_len;
    const uint8_t *const *experts_down;          /* [num_experts]: expert e's [hidden, inter/32, 16] nibble bytes */
    const size_t *experts_down_len;
    const uint8_t *const *scales_gate_up;        /* Paired: [num_experts] e8m0 streams [2*inter, hidden/32]; else NULL */
    const size_t *scales_gate_up_len;
    const uint8_t *const *scales_down;           /* Paired: [num_experts] e8m0 streams [hidden, inter/32]; else NULL */
    const size_t *scales_down_len;
    const float *router_proj;                    /* [num_experts, hidden] */
    const float *router_bias;                    /* [num_experts], or NULL (the reference: an empty slice) */
    const float *experts_gate_up_bias;           /* [num_experts, 2*inter] as the checkpoint ships it (interleaved), or NULL */
    const float *experts_down_bias;              /* [num_experts, hidden], or NULL */
    const float *router_per_expert_scale;        /* [num_experts], or NULL */
    int renormalized_softmax;                    /* MoeTopKWeightPolicy::RenormalizedSoftmax (else the softmax's own values) */
    int per_expert_scale;                        /* MoeExpertScalePolicy::PerExpert */
    float glu_limit, glu_alpha;                  /* MoeGateRule::ClampedGlu (GPT-OSS: 7, 1.702) */
    int gate_rule;                               /* LARQL_MOE_GATE_* (0 = ClampedGlu with the two parameters above) */
} larql_hip_moe_layer_weights;
typedef struct larql_hip_moe_layer larql_hip_moe_layer;
int  larql_hip_moe_layer_create(larql_hip_ctx *ctx, const larql_hip_moe_layer_weights *weights, larql_hip_moe_layer **out);
void larql_hip_moe_layer_destroy(larql_hip_ctx *ctx, larql_hip_moe_layer *layer);
/* moe_route_from_router_input (cpu/ops/moe/mod.rs:149-186: router_proj . router_in + router_bias, softmax, top_k,
 * renormalise, per-expert scale) followed by the expert block (cpu/ops/moe/forward.rs:201-270) on host slices:
 * router_in and x are [tokens, hidden] (the router's and the experts' input: the reference derives both from the
 * residual under MoeRoutingPolicy, and they may be the same slice), out is [tokens, hidden].  experts_out /
 * weights_out ([tokens, min(top_k, num_experts)], may be NULL) receive the route.  One submission.  A k-quant or float
 * bank takes up to 65535 (token, expert) slots per call (more: LARQL_UNSUPPORTED — split the tokens over calls). */
int  larql_hip_moe_layer_forward(larql_hip_ctx *ctx, larql_hip_moe_layer *layer, const float *router_in, const float *x,
                                 size_t tokens, float *out, uint32_t *experts_out, float *weights_out);
/* The same on resident operands; only enqueues.  The router's projection runs on the device (a [num_experts, hidden]
 * f32 gemv per token), the selection inside the first expert launch for one token: residual -> output without a host
 * round trip.  experts / weights: device buffers [tokens, min(top_k, num_experts)]; router_in, x and out 16-byte
 * aligned with hidden % 4 == 0 (else LARQL_REFUSED_SHAPE). */
int  larql_hip_dev_moe_layer_forward(larql_hip_ctx *ctx, larql_hip_moe_layer *layer, const float *router_in, const float *x,
                                     size_t tokens, float *out, uint32_t *experts, float *weights);

/* ---- device tier: encoders (bit-exact with the reference's host encoders) --- */
/* quantize_q4_k — larql-compute/src/cpu/ops/q4_common/quantize.rs:89-189. */
int larql_hip_dev_quantize_q4_k(larql_hip_ctx *ctx, const float *src, size_t n, uint8_t *dst);
/* quantize_q6_k — larql-compute/src/cpu/ops/q4_common/quantize.rs:198-276 (210-byte super-blocks, ggml's planar layout). */
int larql_hip_dev_quantize_q6_k(larql_hip_ctx *ctx, const float *src, size_t n, uint8_t *dst);
/* quantize_q8_0 — larql-models/src/quant/ggml/quantize.rs:50-77. */
int larql_hip_dev_quantize_q8_0(larql_hip_ctx *ctx, const float *src, size_t n, uint8_t *dst);
/* quantize_mxfp4 — larql-vindex/src/format/vindex3/opplan/exec/weights/load.rs:410-476. */
int larql_hip_dev_quantize_mxfp4(larql_hip_ctx *ctx, const float *src, size_t rows, size_t k,
                                 uint8_t *packed, uint8_t *scales);
/* f32_to_bf16 (truncation) — larql-models/src/quant/half.rs:107-109. */
int larql_hip_dev_f32_to_bf16(larql_hip_ctx *ctx, const float *src, size_t n, uint16_t *dst);
/* quantize_q4_0 / quantize_to_q8 — q4_common/quantize.rs:6-69. */
int larql_hip_dev_quantize_q4_0(larql_hip_ctx *ctx, const float *src, size_t n, uint8_t *dst);
int larql_hip_dev_quantize_to_q8(larql_hip_ctx *ctx, const float *src, size_t n, int8_t *q8, float *scales);
/* quantize_x_to_q8k on the device (q8k_activation.rs:84-109).  `q8k` receives the
 * activation in one buffer of larql_hip_q8k_bytes(n) bytes: n int8 codes, then
 * n/256 f32 scales, then n/32 i16 sub-block sums; that buffer is the `x` of a
 * LARQL_FMT_Q4_K_Q8K job.  Both pointers 16-byte aligned. */
size_t larql_hip_q8k_bytes(size_t n);
int larql_hip_dev_quantize_x_to_q8k(larql_hip_ctx *ctx, const float *x, size_t n, void *q8k);
/* Synthetic N(0, sigma) data for benchmarks: element i of stream `seed` is a
 * fixed function of (seed, i) (sum of twelve 21-bit uniforms from a
 * splitmix64 counter stream: exact integer arithmetic, so host and device
 * agree bit for bit).  No counterpart in the reference, which prescribes no
 * generator. */
int larql_hip_dev_fill_normal(larql_hip_ctx *ctx, float *dst, size_t n, uint64_t seed, float sigma);

#ifdef __cplusplus
}
#endif
#endif
