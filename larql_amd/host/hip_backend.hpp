// hip_backend.hpp — C++ host-side mirror of the reference's backend traits for
// the quantised decode path, over the C ABI of include/larql_hip.h.
//
// The reference's host code is Rust (`impl QuantMatVec for ...`); no Rust
// toolchain exists in this environment, so the thin host layer a backend crate
// would contain is written here in C++ with the same method names, argument
// meaning and refusal convention: `std::nullopt` is the trait's `None`
// ("cannot serve this request — fall back"), never a wrong vector.
// Signatures follow larql-compute/src/backend/{quant_matvec.rs,matmul.rs,mod.rs}.
#pragma once
#include <algorithm>
#include <cstdint>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/larql_hip.h"

namespace larql {

enum class QuantFormat : int {  // pipeline/quant_format/mod.rs:19-62
    Q4_0 = LARQL_FMT_Q4_0, Q4_K = LARQL_FMT_Q4_K, Q4_KF = LARQL_FMT_Q4_KF, Q5_K = LARQL_FMT_Q5_K, Q6_K = LARQL_FMT_Q6_K,
    Q8_0 = LARQL_FMT_Q8_0, BF16 = LARQL_FMT_BF16, F16 = LARQL_FMT_F16, F32 = LARQL_FMT_F32, I2S = LARQL_FMT_I2S,
    MXFP4 = LARQL_FMT_MXFP4
};

template <class T> struct Slice {  // a borrowed `&[T]`
    const T *ptr = nullptr;
    size_t len = 0;
    Slice() = default;
    Slice(const T *p, size_t n) : ptr(p), len(n) {}
    Slice(const std::vector<T> &v) : ptr(v.data()), len(v.size()) {}
};

struct SubmissionClock { uint64_t submissions, commit_to_done_nanos, gpu_nanos; };  // backend/matmul.rs:34-42

enum class Capability : int {  // backend/capability.rs:22-102 (the ones this backend answers true for)
    F32Gemv = LARQL_CAP_F32_GEMV, F16Gemv = LARQL_CAP_F16_GEMV, QuantMatVec = LARQL_CAP_QUANT_MATVEC
};

// `&[(&[u8], usize, usize)]` of bf16_gemv_multi / f16_gemv_multi and `&[(&[u8], &[u8], usize, usize)]` of
// mxfp4_gemv_multi (backend/matmul.rs:151-194, 237-251)
struct DenseMatrix { Slice<uint8_t> w; size_t n = 0, k = 0; };
struct Mxfp4Matrix { Slice<uint8_t> packed, scales; size_t n = 0, k = 0; };

// MoeLayerWeights (pipeline/moe.rs:469-541), the fields this path reads.  Borrowed, like the original.
enum class MoeFusedRowLayout { ContiguousHalves = LARQL_MOE_ROWS_CONTIGUOUS_HALVES, Interleaved = LARQL_MOE_ROWS_INTERLEAVED };
struct MoeExpertScales {  // Inline | Paired { gate_up, down } (moe.rs:214-238)
    bool paired = false;
    std::vector<Slice<uint8_t>> gate_up, down;
};
struct MoeGateRule {  // moe.rs:16-118; `Other` stands for a rule without a kernel here (Gated(ReLU))
    enum Kind {
        ClampedGlu = LARQL_MOE_GATE_CLAMPED_GLU, GatedGeluTanh = LARQL_MOE_GATE_GELU_TANH, GatedSilu = LARQL_MOE_GATE_SILU,
        SituGlu = LARQL_MOE_GATE_SITU_GLU, ClampedGatedGeluTanh = LARQL_MOE_GATE_CLAMPED_GELU_TANH, ClampedGatedSilu = LARQL_MOE_GATE_CLAMPED_SILU,
        Other = -1
    };
    Kind kind = ClampedGlu;
    // ClampedGlu { limit, alpha }; SituGlu { beta = limit, linear_beta = alpha (0: None) }; ClampedGated { limit }
    float limit = 7.0f, alpha = 1.702f;
};
struct MoeLayerWeights {
    std::vector<Slice<uint8_t>> experts_gate_up, experts_down;
    MoeExpertScales expert_scales;
    MoeFusedRowLayout fused_row_layout = MoeFusedRowLayout::Interleaved;
    QuantFormat expert_data_format = QuantFormat::MXFP4;
    Slice<float> router_proj, router_bias, experts_gate_up_bias, experts_down_bias, router_per_expert_scale;
    bool renormalized_softmax = true;  // MoeTopKWeightPolicy::RenormalizedSoftmax
    bool per_expert_scale = false;     // MoeExpertScalePolicy::PerExpert
    size_t num_experts = 0, top_k = 0, intermediate_size = 0;
    MoeGateRule gate_rule;
};

class HipBackend;

// One MoE layer resident on the device (HipBackend::moe_layer); destroyed with the object.
class HipMoeLayer {
  public:
    HipMoeLayer(HipMoeLayer &&o) noexcept : ctx_(o.ctx_), layer_(o.layer_), hidden_(o.hidden_), top_k_(o.top_k_) { o.layer_ = nullptr; }
    HipMoeLayer(const HipMoeLayer &) = delete;
    HipMoeLayer &operator=(const HipMoeLayer &) = delete;
    ~HipMoeLayer() { if (layer_) larql_hip_moe_layer_destroy(ctx_, layer_); }
    struct Output { std::vector<float> out; std::vector<uint32_t> experts; std::vector<float> weights; };
    // moe_route_from_router_input + the expert block (cpu/ops/moe/mod.rs:149-186, forward.rs:201-270) for `tokens`
    // rows; router_in and x are [tokens, hidden].
    std::optional<Output> forward(Slice<float> router_in, Slice<float> x, size_t tokens) {
        if (hidden_ != 0 && tokens > (size_t)-1 / hidden_) return std::nullopt;
        const size_t n = tokens * hidden_;
        if (router_in.len != n || x.len != n) return std::nullopt;
        Output o{std::vector<float>(n), std::vector<uint32_t>(tokens * top_k_), std::vector<float>(tokens * top_k_)};
        if (larql_hip_moe_layer_forward(ctx_, layer_, router_in.ptr, x.ptr, tokens, o.out.data(), o.experts.data(), o.weights.data()) !=
            LARQL_OK)
            return std::nullopt;
        return o;
    }
    size_t top_k() const { return top_k_; }

  private:
    friend class HipBackend;
    HipMoeLayer(larql_hip_ctx *c, larql_hip_moe_layer *l, size_t hidden, size_t top_k) : ctx_(c), layer_(l), hidden_(hidden), top_k_(top_k) {}
    larql_hip_ctx *ctx_;
    larql_hip_moe_layer *layer_;
    size_t hidden_, top_k_;
};

class HipBackend {
  public:
    // BackendSelectError::NoDevice (backend/factory.rs:164-173): a named GPU request never falls back to the CPU.
    explicit HipBackend(int device = 0) {
        if (larql_hip_create(&ctx_, device) != LARQL_OK) throw std::runtime_error("HipBackend: no usable gfx950 device");
    }
    ~HipBackend() { larql_hip_destroy(ctx_); }
    HipBackend(const HipBackend &) = delete;
    HipBackend &operator=(const HipBackend &) = delete;

    // ComputeBackend (backend/mod.rs:49-92)
    std::string name() const { return larql_hip_name(ctx_); }
    std::string device_info() const { return larql_hip_device_info(ctx_); }
    bool supports_quant(QuantFormat f) const { return larql_hip_supports_quant(ctx_, (int)f) != 0; }
    bool supports(Capability c) const { return larql_hip_supports(ctx_, (int)c) != 0; }
    void register_weight_region(Slice<uint8_t> region) { larql_hip_register_weight_region(ctx_, region.ptr, region.len); }
    void seal_weight_regions() { larql_hip_seal_weight_regions(ctx_); }
    void clear_weight_regions() { larql_hip_clear_weight_regions(ctx_); }
    std::optional<SubmissionClock> submission_clock() {
        larql_hip_submission_clock c;
        if (larql_hip_get_submission_clock(ctx_, &c) != LARQL_OK) return std::nullopt;
        return SubmissionClock{c.submissions, c.commit_to_done_nanos, c.gpu_nanos};
    }
    std::string last_error() const { return larql_hip_last_error(ctx_); }

    // QuantMatVec (backend/quant_matvec.rs)
    std::optional<std::vector<float>> q4k_matvec(Slice<uint8_t> q4k, Slice<float> x, size_t num_rows, size_t hidden) {
        std::vector<float> out(num_rows);
        return some(larql_hip_q4k_matvec(ctx_, q4k.ptr, q4k.len, x.ptr, x.len, num_rows, hidden, out.data(), out.size()), out);
    }
    std::optional<std::vector<float>> q6k_matvec(Slice<uint8_t> q6k, Slice<float> x, size_t num_rows, size_t hidden) {
        std::vector<float> out(num_rows);
        return some(larql_hip_q6k_matvec(ctx_, q6k.ptr, q6k.len, x.ptr, x.len, num_rows, hidden, out.data()), out);
    }
    // Q8_K-activation integer path (cpu/ops/q4k_q8k_dot): Q8KActivation { qs, d, sums }
    struct Q8KActivation { std::vector<int8_t> qs; std::vector<float> d; std::vector<int16_t> sums; };
    std::optional<Q8KActivation> quantize_x_to_q8k(Slice<float> x) {
        Q8KActivation a{std::vector<int8_t>(x.len), std::vector<float>(x.len / 256), std::vector<int16_t>(x.len / 32)};
        if (larql_hip_quantize_x_to_q8k(ctx_, x.ptr, x.len, a.qs.data(), a.d.data(), a.sums.data()) != LARQL_OK) return std::nullopt;
        return a;
    }
    std::optional<std::vector<float>> q4k_q8k_matvec(Slice<uint8_t> q4k, const Q8KActivation &a, size_t num_rows, size_t cols) {
        std::vector<float> out(num_rows);
        return some(larql_hip_q4k_q8k_matvec(ctx_, q4k.ptr, q4k.len, a.qs.data(), a.qs.size(), a.d.data(), a.sums.data(), num_rows, cols,
                                             out.data(), out.size()), out);
    }
    std::optional<std::pair<std::vector<float>, std::vector<float>>> q4k_q8k_gate_up(Slice<uint8_t> gate_w, Slice<uint8_t> up_w,
                                                                                       const Q8KActivation &a, size_t num_rows,
                                                                                       size_t cols) {
        std::vector<float> g(num_rows), u(num_rows);
        if (larql_hip_q4k_q8k_gate_up(ctx_, gate_w.ptr, gate_w.len, up_w.ptr, up_w.len, a.qs.data(), a.qs.size(), a.d.data(), a.sums.data(),
                                      num_rows, cols, g.data(), u.data(), num_rows) != LARQL_OK)
            return std::nullopt;
        return std::make_pair(std::move(g), std::move(u));
    }
    // q4k_q8k_gemm_into: [seq, rows] from `seq` quantised activation rows
    std::optional<std::vector<float>> q4k_q8k_gemm(Slice<uint8_t> q4k, const std::vector<Q8KActivation> &acts, size_t num_rows, size_t cols) {
        std::vector<int8_t> qs; std::vector<float> d; std::vector<int16_t> sums;
        for (const Q8KActivation &a : acts) {
            if (a.qs.size() != cols || a.d.size() != cols / 256 || a.sums.size() != cols / 32) return std::nullopt;
            qs.insert(qs.end(), a.qs.begin(), a.qs.end()); d.insert(d.end(), a.d.begin(), a.d.end()); sums.insert(sums.end(), a.sums.begin(), a.sums.end());
        }
        std::vector<float> out(acts.size() * num_rows);
        return some(larql_hip_q4k_q8k_gemm(ctx_, q4k.ptr, q4k.len, qs.data(), d.data(), sums.data(), acts.size(), num_rows, cols, out.data(), out.size()), out);
    }
    std::optional<std::vector<float>> q6k_q8k_matvec(Slice<uint8_t> q6k, const Q8KActivation &a, size_t num_rows, size_t cols) {
        std::vector<float> out(num_rows);
        return some(larql_hip_q6k_q8k_matvec(ctx_, q6k.ptr, q6k.len, a.qs.data(), a.qs.size(), a.d.data(), num_rows, cols, out.data(),
                                             out.size()), out);
    }
    std::optional<std::pair<std::vector<float>, std::vector<float>>> q4k_dual_matvec(Slice<uint8_t> a, Slice<uint8_t> b,
                                                                                       Slice<float> x, size_t num_rows,
                                                                                       size_t hidden) {
        std::vector<float> oa(num_rows), ob(num_rows);
        if (larql_hip_q4k_dual_matvec(ctx_, a.ptr, a.len, b.ptr, b.len, x.ptr, x.len, num_rows, hidden, oa.data(), ob.data(),
                                      num_rows) != LARQL_OK)
            return std::nullopt;
        return std::make_pair(std::move(oa), std::move(ob));
    }
    std::optional<std::vector<float>> q4k_matmul(Slice<uint8_t> q4k, Slice<float> x, size_t num_rows, size_t hidden,
                                                 size_t seq_len) {
        std::vector<float> out(seq_len * num_rows);
        return some(larql_hip_q4k_matmul(ctx_, q4k.ptr, q4k.len, x.ptr, x.len, num_rows, hidden, seq_len, out.data(), out.size()),
                    out);
    }
    std::optional<std::vector<std::pair<uint32_t, float>>> q4k_matvec_topk(Slice<uint8_t> q4k, Slice<float> x, size_t num_rows,
                                                                           size_t hidden, size_t top_k) {
        const auto kk = clamp_top_k(top_k, num_rows);
        if (!kk) return std::nullopt;
        top_k = *kk;
        std::vector<uint32_t> idx(top_k ? top_k : 1);
        std::vector<float> val(top_k ? top_k : 1);
        size_t n = 0;
        if (larql_hip_q4k_matvec_topk(ctx_, q4k.ptr, q4k.len, x.ptr, x.len, num_rows, hidden, top_k, idx.data(), val.data(), &n) !=
            LARQL_OK)
            return std::nullopt;
        std::vector<std::pair<uint32_t, float>> hits;
        for (size_t i = 0; i < n; i++) hits.emplace_back(idx[i], val[i]);
        return hits;
    }
    std::optional<std::vector<float>> q4_matvec(Slice<uint8_t> q4, Slice<int8_t> q8_x, Slice<float> q8_scales, size_t num_rows,
                                                size_t hidden) {
        std::vector<float> out(num_rows);
        return some(larql_hip_q4_matvec(ctx_, q4.ptr, q4.len, q8_x.ptr, q8_x.len, q8_scales.ptr, q8_scales.len, num_rows, hidden,
                                        out.data()), out);
    }
    std::optional<std::vector<float>> quant_matvec(QuantFormat f, Slice<uint8_t> w, Slice<float> x, size_t num_rows, size_t hidden) {
        std::vector<float> out(num_rows);
        return some(larql_hip_quant_matvec(ctx_, (int)f, w.ptr, w.len, x.ptr, x.len, num_rows, hidden, out.data()), out);
    }
    // quant_matvec_q8_input (quant_matvec.rs:100-128): the activation arrives as Q8 codes + per-32 scales
    std::optional<std::vector<float>> quant_matvec_q8_input(QuantFormat f, Slice<uint8_t> w, Slice<int8_t> q8_x, Slice<float> q8_scales,
                                                            size_t num_rows, size_t hidden) {
        std::vector<float> out(num_rows);
        return some(larql_hip_quant_matvec_q8_input(ctx_, (int)f, w.ptr, w.len, q8_x.ptr, q8_x.len, q8_scales.ptr, q8_scales.len, num_rows,
                                                    hidden, out.data()), out);
    }
    // free function q8_0_gemv (cpu/kquant_gemv.rs:67-90)
    std::optional<std::vector<float>> q8_0_gemv(Slice<uint8_t> blocks, Slice<float> x, size_t n, size_t k) {
        std::vector<float> out(n);
        return some(larql_hip_q8_0_gemv(ctx_, blocks.ptr, blocks.len, x.ptr, x.len, n, k, out.data()), out);
    }
    // the lm_head's scores stay on the device, only the top-K by value comes back (lm_head/knn.rs:144-175, top_k_sorted)
    std::optional<std::vector<std::pair<uint32_t, float>>> q8_0_gemv_topk(Slice<uint8_t> blocks, Slice<float> x, size_t n, size_t k,
                                                                          size_t top_k) {
        const auto kk = clamp_top_k(top_k, n);
        if (!kk) return std::nullopt;
        top_k = *kk;
        std::vector<uint32_t> idx(top_k ? top_k : 1);
        std::vector<float> val(top_k ? top_k : 1);
        size_t got = 0;
        if (larql_hip_q8_0_gemv_topk(ctx_, blocks.ptr, blocks.len, x.ptr, x.len, n, k, top_k, idx.data(), val.data(), &got) != LARQL_OK)
            return std::nullopt;
        std::vector<std::pair<uint32_t, float>> hits;
        for (size_t i = 0; i < got; i++) hits.emplace_back(idx[i], val[i]);
        return hits;
    }

    // MatMul (backend/matmul.rs)
    std::optional<std::vector<float>> f32_gemv(Slice<float> w, Slice<float> x, size_t n, size_t k, bool force = false) {
        std::vector<float> out(n);
        return some(larql_hip_f32_gemv(ctx_, w.ptr, w.len * 4, x.ptr, x.len, n, k, out.data(), force), out);
    }
    std::optional<std::vector<float>> f32_gemv_force(Slice<float> w, Slice<float> x, size_t n, size_t k) { return f32_gemv(w, x, n, k, true); }
    // (the unforced calls answer None below the size where a launch pays off, as the peers' do: matmul.rs:96-149)
    std::optional<std::vector<float>> f16_gemv(Slice<uint8_t> w, Slice<float> x, size_t n, size_t k) { return dense_half(false, w, x, n, k, 0); }
    std::optional<std::vector<float>> f16_gemv_force(Slice<uint8_t> w, Slice<float> x, size_t n, size_t k) { return dense_half(false, w, x, n, k, 1); }
    std::optional<std::vector<float>> bf16_gemv(Slice<uint8_t> w, Slice<float> x, size_t n, size_t k) { return dense_half(true, w, x, n, k, 0); }
    std::optional<std::vector<float>> bf16_gemv_force(Slice<uint8_t> w, Slice<float> x, size_t n, size_t k) { return dense_half(true, w, x, n, k, 1); }
    // several matrices against one x as one submission (matmul.rs:151-194)
    std::optional<std::vector<std::vector<float>>> bf16_gemv_multi(const std::vector<DenseMatrix> &weights, Slice<float> x) {
        return dense_multi(true, weights, x);
    }
    std::optional<std::vector<std::vector<float>>> f16_gemv_multi(const std::vector<DenseMatrix> &weights, Slice<float> x) {
        return dense_multi(false, weights, x);
    }
    std::optional<std::vector<float>> mxfp4_gemv(Slice<uint8_t> packed, Slice<uint8_t> scales, Slice<float> x, size_t n, size_t k) {
        std::vector<float> out(n);
        return some(larql_hip_mxfp4_gemv(ctx_, packed.ptr, packed.len, scales.ptr, scales.len, x.ptr, x.len, n, k, out.data()), out);
    }

    // mxfp4_gemv_multi (matmul.rs:237-251): one submission for all matrices
    std::optional<std::vector<std::vector<float>>> mxfp4_gemv_multi(const std::vector<Mxfp4Matrix> &weights, Slice<float> x) {
        const size_t m = weights.size();
        std::vector<const uint8_t *> p(m), sc(m);
        std::vector<size_t> pl(m), sl(m), n(m), k(m);
        std::vector<std::vector<float>> outs(m);
        std::vector<float *> op(m);
        for (size_t i = 0; i < m; i++) {
            p[i] = weights[i].packed.ptr; pl[i] = weights[i].packed.len; sc[i] = weights[i].scales.ptr; sl[i] = weights[i].scales.len;
            n[i] = weights[i].n; k[i] = weights[i].k;
            outs[i].resize(n[i]); op[i] = outs[i].data();
        }
        if (larql_hip_mxfp4_gemv_multi(ctx_, m, p.data(), pl.data(), sc.data(), sl.data(), n.data(), k.data(), x.ptr, x.len, op.data()) != LARQL_OK)
            return std::nullopt;
        return outs;
    }

    // A MoE layer made resident from MoeLayerWeights: the per-expert slices and their paired exponent streams go up
    // expert by expert, wherever they lie.  Served: an MXFP4 bank with Paired scales under ClampedGlu, and a Q4_K / Q6_K
    // bank with Inline scales and ContiguousHalves rows under ClampedGlu or Gated (cpu_moe_forward's integer path); a
    // BF16 / F16 / F32 bank likewise (its f32 arm).
    // nullopt where this backend has no kernel for the layer (other formats or rules, more than 256 experts, top-k
    // above 8): the caller keeps cpu_moe_forward.
    std::optional<HipMoeLayer> moe_layer(const MoeLayerWeights &moe, size_t hidden) {
        const size_t n = moe.num_experts;
        if (moe.gate_rule.kind == MoeGateRule::Other) return std::nullopt;
        if (moe.experts_gate_up.size() != n || moe.experts_down.size() != n) return std::nullopt;
        if (hidden != 0 && n > (size_t)-1 / hidden) return std::nullopt;
        if (moe.router_proj.len != n * hidden) return std::nullopt;
        const MoeExpertScales &es = moe.expert_scales;
        if (es.paired && (es.gate_up.size() != n || es.down.size() != n)) return std::nullopt;
        const auto ptrs = [](const std::vector<Slice<uint8_t>> &v) { std::vector<const uint8_t *> r; for (const auto &q : v) r.push_back(q.ptr); return r; };
        const auto lens = [](const std::vector<Slice<uint8_t>> &v) { std::vector<size_t> r; for (const auto &q : v) r.push_back(q.len); return r; };
        const auto gp = ptrs(moe.experts_gate_up), dp = ptrs(moe.experts_down), sgp = ptrs(es.gate_up), sdp = ptrs(es.down);
        const auto gl = lens(moe.experts_gate_up), dl = lens(moe.experts_down), sgl = lens(es.gate_up), sdl = lens(es.down);
        const auto opt = [](Slice<float> f) { return f.len ? f.ptr : nullptr; };  // (an empty slice is "none" in the reference)
        larql_hip_moe_layer_weights w = {};
        w.num_experts = n; w.top_k = moe.top_k; w.hidden = hidden; w.intermediate_size = moe.intermediate_size;
        w.expert_data_format = (int)moe.expert_data_format;
        w.fused_row_layout = (int)moe.fused_row_layout;
        w.expert_scales = es.paired ? LARQL_MOE_SCALES_PAIRED : LARQL_MOE_SCALES_INLINE;
        w.experts_gate_up = gp.data(); w.experts_gate_up_len = gl.data();
        w.experts_down = dp.data(); w.experts_down_len = dl.data();
        w.scales_gate_up = es.paired ? sgp.data() : nullptr; w.scales_gate_up_len = es.paired ? sgl.data() : nullptr;
        w.scales_down = es.paired ? sdp.data() : nullptr; w.scales_down_len = es.paired ? sdl.data() : nullptr;
        w.router_proj = moe.router_proj.ptr; w.router_bias = opt(moe.router_bias);
        w.experts_gate_up_bias = opt(moe.experts_gate_up_bias); w.experts_down_bias = opt(moe.experts_down_bias);
        w.router_per_expert_scale = opt(moe.router_per_expert_scale);
        w.renormalized_softmax = moe.renormalized_softmax ? 1 : 0;
        w.per_expert_scale = moe.per_expert_scale ? 1 : 0;
        w.glu_limit = moe.gate_rule.limit; w.glu_alpha = moe.gate_rule.alpha; w.gate_rule = (int)moe.gate_rule.kind;
        larql_hip_moe_layer *layer = nullptr;
        if (larql_hip_moe_layer_create(ctx_, &w, &layer) != LARQL_OK || !layer) return std::nullopt;
        return HipMoeLayer(ctx_, layer, hidden, std::min(moe.top_k, n));
    }

    // VectorIndex::gate_knn (larql-vindex/src/index/compute/gate_knn/dispatch.rs:22-52)
    std::optional<std::vector<std::pair<size_t, float>>> gate_knn(QuantFormat f, Slice<uint8_t> gate, Slice<float> residual,
                                                                  size_t n_features, size_t hidden, size_t top_k) {
        const auto kk = clamp_top_k(top_k, n_features);
        if (!kk) return std::nullopt;
        top_k = *kk;
        std::vector<uint32_t> idx(top_k ? top_k : 1);
        std::vector<float> val(top_k ? top_k : 1);
        size_t n = 0;
        if (larql_hip_gate_knn(ctx_, (int)f, gate.ptr, gate.len, residual.ptr, 1, n_features, hidden, top_k, idx.data(), val.data(),
                               &n) != LARQL_OK)
            return std::nullopt;
        std::vector<std::pair<size_t, float>> hits;
        for (size_t i = 0; i < n; i++) hits.emplace_back(idx[i], val[i]);
        return hits;
    }

    // gate_knn per position of a batch: x is [batch, hidden]; one hit list per position, |score| descending
    std::optional<std::vector<std::vector<std::pair<size_t, float>>>> gate_knn_positions(QuantFormat f, Slice<uint8_t> gate, Slice<float> x,
                                                                                        size_t batch, size_t n_features, size_t hidden,
                                                                                        size_t top_k) {
        if (hidden != 0 && batch > (size_t)-1 / hidden) return std::nullopt;
        if (x.len != batch * hidden) return std::nullopt;
        const auto kk = clamp_top_k(top_k, n_features);
        if (!kk) return std::nullopt;
        top_k = *kk;
        if (top_k != 0 && batch > (size_t)-1 / top_k) return std::nullopt;
        std::vector<uint32_t> idx(batch * top_k + 1);
        std::vector<float> val(batch * top_k + 1);
        std::vector<size_t> got(batch + 1);
        if (larql_hip_gate_knn(ctx_, (int)f, gate.ptr, gate.len, x.ptr, batch, n_features, hidden, top_k, idx.data(), val.data(), got.data()) !=
            LARQL_OK)
            return std::nullopt;
        std::vector<std::vector<std::pair<size_t, float>>> hits(batch);
        for (size_t b = 0; b < batch; b++)
            for (size_t i = 0; i < std::min(got[b], top_k); i++) hits[b].emplace_back(idx[b * top_k + i], val[b * top_k + i]);
        return hits;
    }
    // VectorIndex::gate_knn_batch (dispatch.rs:256-304): the sorted, de-duplicated union of every position's top-K indices
    std::optional<std::vector<size_t>> gate_knn_batch(QuantFormat f, Slice<uint8_t> gate, Slice<float> x, size_t batch, size_t n_features,
                                                      size_t hidden, size_t top_k) {
        const auto per = gate_knn_positions(f, gate, x, batch, n_features, hidden, top_k);
        if (!per) return std::nullopt;
        std::vector<size_t> all;
        for (const auto &hits : *per)
            for (const auto &h : hits) all.push_back(h.first);
        std::sort(all.begin(), all.end());
        all.erase(std::unique(all.begin(), all.end()), all.end());
        return all;
    }
    // gate_scores_batch_backend (gate_knn/scores_batch.rs:30-57): the full [batch, n_features] score matrix, row-major
    std::optional<std::vector<float>> gate_scores_batch(QuantFormat f, Slice<uint8_t> gate, Slice<float> x, size_t batch, size_t n_features,
                                                        size_t hidden) {
        if (hidden != 0 && batch > (size_t)-1 / hidden) return std::nullopt;
        if (x.len != batch * hidden || (n_features != 0 && batch > (size_t)-1 / n_features)) return std::nullopt;
        std::vector<float> out(batch * n_features);
        return some(larql_hip_gate_scores(ctx_, (int)f, gate.ptr, gate.len, x.ptr, batch, n_features, hidden, out.data()), out);
    }

    larql_hip_ctx *raw() { return ctx_; }

  private:
    static std::optional<std::vector<float>> some(int rc, std::vector<float> &out) {
        if (rc != LARQL_OK) return std::nullopt;
        return std::move(out);
    }
    // A caller may pass a very large K to mean "all": K is clamped to the number of candidates before any buffer is
    // sized from it; a K beyond what the library orders per row (16384) answers nullopt, not an allocation failure.
    static std::optional<size_t> clamp_top_k(size_t top_k, size_t candidates) {
        const size_t k = std::min(top_k, candidates);
        if (k > 16384) return std::nullopt;
        return k;
    }
    std::optional<std::vector<float>> dense_half(bool bf16, Slice<uint8_t> w, Slice<float> x, size_t n, size_t k, int force) {
        if (x.len != k) return std::nullopt;  // the peers answer None unless x is exactly one row long
        std::vector<float> out(n);
        const int rc = bf16 ? larql_hip_bf16_gemv(ctx_, w.ptr, w.len, x.ptr, x.len, n, k, out.data(), force)
                            : larql_hip_f16_gemv(ctx_, w.ptr, w.len, x.ptr, x.len, n, k, out.data(), force);
        return some(rc, out);
    }
    std::optional<std::vector<std::vector<float>>> dense_multi(bool bf16, const std::vector<DenseMatrix> &weights, Slice<float> x) {
        const size_t m = weights.size();
        std::vector<const uint8_t *> w(m);
        std::vector<size_t> wl(m), n(m), k(m);
        std::vector<std::vector<float>> outs(m);
        std::vector<float *> op(m);
        for (size_t i = 0; i < m; i++) {
            w[i] = weights[i].w.ptr; wl[i] = weights[i].w.len; n[i] = weights[i].n; k[i] = weights[i].k;
            outs[i].resize(n[i]); op[i] = outs[i].data();
        }
        const int rc = bf16 ? larql_hip_bf16_gemv_multi(ctx_, m, w.data(), wl.data(), n.data(), k.data(), x.ptr, x.len, op.data())
                            : larql_hip_f16_gemv_multi(ctx_, m, w.data(), wl.data(), n.data(), k.data(), x.ptr, x.len, op.data());
        if (rc != LARQL_OK) return std::nullopt;
        return outs;
    }
    larql_hip_ctx *ctx_ = nullptr;
};

}  // namespace larql
