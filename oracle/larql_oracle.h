/*
 * larql_oracle.h — CPU restatement of the LARQL reference algorithms on the
 * quantised decode path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing here is shipped or measured as the
 * product: only the test-suite, the smoke check and the benchmark's
 * cpu_baseline leg may load this library, and only as the checker.
 *
 * Every function cites the reference file:line (paths relative to the
 * reference checkout) whose arithmetic, operation order and refusal rules it
 * restates.  Build with -ffp-contract=off: the reference is Rust, which never
 * contracts a*b+c into an FMA.
 *
 * Return convention for functions returning int: 0 = Ok / Some,
 * 1 = refused (the reference returns None / Err), and the output is then left
 * untouched unless the comment says otherwise.
 */
#ifndef LARQL_ORACLE_H
#define LARQL_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- half / bf16 conversions ---------------------------------------- */
float    lq_f16_to_f32(uint16_t bits);
uint16_t lq_f32_to_f16_trunc(float v);   /* q4_common/f16.rs:10-41 */
uint16_t lq_f32_to_f16_nearest(float v); /* quant/half.rs:70-104 */
uint16_t lq_f32_to_f16_flush(float v);   /* quantize.rs:41-58 (inline in quantize_q4_0) */
uint16_t lq_f32_to_bf16(float v);        /* quant/half.rs:107-109 */
float    lq_bf16_to_f32(uint16_t bits);  /* quant/half.rs:38-40 */
void     lq_f32_to_bf16_slice(const float *src, size_t n, uint16_t *dst);

/* ---- Q4_K ------------------------------------------------------------ */
int  lq_quantize_q4_k(const float *data, size_t n, uint8_t *out);
int  lq_dequantize_q4_k(const uint8_t *data, size_t data_len, size_t n, float *out);
int  lq_q4k_matvec_into(float *out, size_t out_len, const float *x, size_t x_len,
                        const uint8_t *w, size_t w_len, size_t rows, size_t cols);
int  lq_q4k_matvec_scalar(float *out, const float *x, const uint8_t *w,
                          size_t rows, size_t hidden);
int  lq_q4k_dual_matvec_into(float *out_a, float *out_b, size_t out_len,
                             const float *x, size_t x_len,
                             const uint8_t *w_a, size_t wa_len,
                             const uint8_t *w_b, size_t wb_len,
                             size_t rows, size_t cols);
void lq_q4k_matmul_into(float *out, const float *x, const uint8_t *w, size_t w_len,
                        size_t rows, size_t hidden, size_t seq);

/* ---- Q8_0 (ggml, 34-byte blocks) ------------------------------------- */
/* Q6_K: 210-byte super-blocks (ggml planar layout) */
int  lq_quantize_q6_k(const float *data, size_t n, uint8_t *out);              /* q4_common/quantize.rs:197-276 */
void lq_q6k_subblock_vals(const uint8_t *block, size_t j, int8_t *out16);     /* larql-models/src/quant/ggml/q6_k.rs:19-40 */
int  lq_dequantize_q6_k(const uint8_t *data, size_t data_len, size_t n, float *out); /* q6_k.rs:173-195 */
int  lq_quantize_x_to_q8k(const float *x, size_t n, int8_t *qs, float *d, int16_t *sums); /* cpu/ops/q4k_q8k_dot/q8k_activation.rs:84-109 */
int  lq_q4k_q8k_matvec(float *out, size_t out_len, const int8_t *qs, size_t qs_len, const float *d, const int16_t *sums,
                       const uint8_t *w, size_t w_len, size_t rows, size_t cols); /* cpu/ops/q4k_q8k_dot/q4k_scalar.rs:15-84 */
int  lq_q6k_q8k_matvec(float *out, size_t out_len, const int8_t *qs, size_t qs_len, const float *d,
                       const uint8_t *w, size_t w_len, size_t rows, size_t cols); /* cpu/ops/q4k_q8k_dot/q6k.rs:38-92 */
int  lq_q6k_matvec(const uint8_t *w, size_t w_len, const float *x, size_t rows, size_t hidden, float *out); /* cpu/ops/q6k_matvec.rs:45-91 */

int  lq_quantize_q8_0(const float *data, size_t n, uint8_t *out);
int  lq_dequantize_q8_0(const uint8_t *data, size_t data_len, size_t n, float *out);
int  lq_q8_0_gemv(const uint8_t *blocks, size_t blocks_len, const float *x, size_t x_len,
                  size_t n, size_t k, float *out);

/* ---- Q4_0 x Q8 (gate_knn_q4 path) ------------------------------------ */
void lq_quantize_to_q8(const float *x, size_t n, int8_t *q8, float *scales);
int  lq_quantize_q4_0(const float *data, size_t n, uint8_t *out);
void lq_q4_0_matvec(const uint8_t *q4, const int8_t *q8_x, const float *q8_scales,
                    float *scores, size_t num_rows, size_t hidden);
void lq_dequantise_q8(const int8_t *q8_x, size_t n, const float *scales, float *out);

/* ---- MXFP4 ------------------------------------------------------------ */
float   lq_e8m0_to_f32(uint8_t byte);
float   lq_mxfp4_table(unsigned code);
uint8_t lq_nearest_mxfp4_code(float v);
int     lq_quantize_mxfp4(const float *values, size_t rows, size_t k,
                          uint8_t *packed, uint8_t *scales);
int     lq_dequantize_mxfp4_expert(const uint8_t *blocks, size_t blocks_len,
                                   const uint8_t *scales, size_t scales_len,
                                   size_t out_features, size_t groups, float *out);
int     lq_mxfp4_gemv(const uint8_t *packed, size_t packed_len,
                      const uint8_t *scales, size_t scales_len,
                      const float *x, size_t x_len, size_t n, size_t k, float *out);
int     lq_mxfp4_gemv_dequant(const uint8_t *packed, const uint8_t *scales,
                              const float *x, size_t n, size_t k, float *out);

/* ---- dense gemv variants (gate scores) -------------------------------- */
void lq_bf16_gemv(const uint16_t *w, const float *x, size_t n, size_t k, float *out);
void lq_f16_gemv(const uint16_t *w, const float *x, size_t n, size_t k, float *out);
void lq_f32_gemv(const float *w, const float *x, size_t n, size_t k, float *out);

/* ---- top-K ------------------------------------------------------------- */
/* Returns the number of hits written (<= top_k), or -1 on a NaN score
 * (the reference panics). */
long lq_top_k_by_abs(const float *scores, size_t n, size_t top_k,
                     uint64_t *idx_out, float *val_out);
long lq_top_k_sorted(const float *scores, size_t n, size_t top_k,
                     uint32_t *idx_out, float *val_out);
/* gate_knn_batch's union: scores is [n_features, seq] row-major. */
long lq_gate_knn_batch_union(const float *scores_2d, size_t n_features, size_t seq,
                             size_t top_k, uint64_t *idx_out, size_t idx_cap);

/* ---- MoE routing / combine -------------------------------------------- */
#define LQ_ROUTE_SOFTMAX_THEN_SELECT 0
#define LQ_ROUTE_NORMALISED_OVER_SELECTED 1
size_t lq_router_select(const float *logits, size_t n, size_t k, int policy,
                        uint64_t *experts, float *weights);
size_t lq_moe_top_k(const float *v, size_t n, size_t k, uint64_t *idx, float *val);
void   lq_softmax(float *v, size_t n);
void   lq_moe_router_logits(const float *router_in, const float *router_proj, const float *router_bias, size_t n_experts,
                            size_t hidden, float *logits);
size_t lq_moe_route_from_router_input(const float *router_in, size_t hidden, const float *router_proj, const float *router_bias,
                                      size_t n_experts, size_t top_k, int renormalize, const float *per_expert_scale,
                                      size_t n_scale, uint64_t *experts, float *weights);
float  lq_clamped_glu(float g, float u, float limit, float alpha);
/* ExpertWeightFfn::moe_block (ffn/expert_weight/mod.rs:100-262) on a GPT-OSS-shaped f32 layer; pinned on EXPECTED[48]
 * of larql-compute/tests/test_moe_reference_parity.rs.  router_b / gate_up_bias / down_bias may be NULL. */
int lq_moe_block_f32(const float *x, size_t tokens, size_t hidden, size_t inter, size_t n_experts, size_t top_k, int policy,
                     const float *router_w, const float *router_b, const float *fused, const float *down,
                     const float *gate_up_bias, const float *down_bias, float limit, float alpha, float *out);
/* the same composition over an MXFP4 bank, routing given */
int lq_moe_block_mxfp4(const float *x, size_t tokens, size_t hidden, size_t inter, size_t n_experts, size_t top_k,
                       const uint64_t *experts, const float *weights, const uint8_t *gate_packed, const uint8_t *gate_scales,
                       const uint8_t *up_packed, const uint8_t *up_scales, const uint8_t *down_packed, const uint8_t *down_scales,
                       int interleaved, const float *gate_up_bias, const float *down_bias, float limit, float alpha, float *out);

/* math::silu / gelu_tanh (cpu/ops/moe/math.rs:54-65) and MoeGateRule::combine (pipeline/moe.rs:73-118) */
#define LQ_GATE_CLAMPED_GLU 0
#define LQ_GATE_GELU_TANH 1
#define LQ_GATE_SILU 2
#define LQ_GATE_SITU_GLU 3          /* limit = beta, alpha = linear_beta (0: none) */
#define LQ_GATE_CLAMPED_GELU_TANH 4  /* ClampedGated{limit, gelu_tanh} */
#define LQ_GATE_CLAMPED_SILU 5       /* ClampedGated{limit, silu} */
float lq_silu(float x);
float lq_gelu_tanh(float x);
float lq_moe_combine(int rule, float g, float u, float limit, float alpha);
/* cpu_moe_forward's integer expert path over a Q4_K (format 4) or Q6_K (format 6) bank of per-expert slices, routing
 * given (cpu/ops/moe/forward.rs:160-330, expert/q4k.rs:232-351).  gate_up[e]: [2*inter, cols] rows, gate half first;
 * down[e]: [hidden, ceil(inter/256)*256]; cols >= hidden is the stored (block-padded) row width.  Formats 16 (BF16),
 * 17 (F16) and 32 (F32) take cpu_moe_forward's f32 arm instead (forward.rs:246-290): f32 activations, down [hidden, inter]. */
int lq_moe_block_kq(const float *x, size_t tokens, size_t hidden, size_t cols, size_t inter, size_t n_experts, size_t top_k,
                    const uint64_t *experts, const float *weights, const uint8_t *const *gate_up, const uint8_t *const *down,
                    int format, const float *gate_up_bias, const float *down_bias, int rule, float limit, float alpha, float *out);

/* ---- multi-threaded drivers for the CPU baseline ----------------------- */
/* Row-chunk parallel versions (32-row chunks, as the reference schedules
 * them); per-row arithmetic is identical to the serial functions. */
int lq_q4k_matvec_into_mt(float *out, const float *x, const uint8_t *w, size_t w_len,
                          size_t rows, size_t cols, int threads);
int lq_bf16_gemv_mt(const uint16_t *w, const float *x, size_t n, size_t k, float *out, int threads);
int lq_mxfp4_gemv_mt(const uint8_t *packed, const uint8_t *scales, const float *x, size_t n, size_t k, float *out, int threads);
int lq_q4k_matmul_into_mt(float *out, const float *x, const uint8_t *w, size_t w_len, size_t rows, size_t hidden, size_t seq, int threads);
int lq_q8_0_gemv_mt(const uint8_t *blocks, size_t blocks_len, const float *x,
                    size_t n, size_t k, float *out, int threads);

#ifdef __cplusplus
}
#endif
#endif
