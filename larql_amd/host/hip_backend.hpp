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
    void register_weight_region(Slice<uint8_t> region) { larql_hip_register_weight_region(ctx_, region.ptr, region.len); }
    void seal_weight_regions() { larql_hip_seal_weight_regions(ctx_); }
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
    // free function q8_0_gemv (cpu/kquant_gemv.rs:67-90)
    std::optional<std::vector<float>> q8_0_gemv(Slice<uint8_t> blocks, Slice<float> x, size_t n, size_t k) {
        std::vector<float> out(n);
        return some(larql_hip_q8_0_gemv(ctx_, blocks.ptr, blocks.len, x.ptr, x.len, n, k, out.data()), out);
    }

    // MatMul (backend/matmul.rs)
    std::optional<std::vector<float>> f32_gemv(Slice<float> w, Slice<float> x, size_t n, size_t k, bool force = false) {
        std::vector<float> out(n);
        return some(larql_hip_f32_gemv(ctx_, w.ptr, w.len * 4, x.ptr, x.len, n, k, out.data(), force), out);
    }
    std::optional<std::vector<float>> f16_gemv_force(Slice<uint8_t> w, Slice<float> x, size_t n, size_t k) {
        std::vector<float> out(n);
        return some(larql_hip_f16_gemv(ctx_, w.ptr, w.len, x.ptr, x.len, n, k, out.data(), 1), out);
    }
    std::optional<std::vector<float>> bf16_gemv_force(Slice<uint8_t> w, Slice<float> x, size_t n, size_t k) {
        std::vector<float> out(n);
        return some(larql_hip_bf16_gemv(ctx_, w.ptr, w.len, x.ptr, x.len, n, k, out.data(), 1), out);
    }
    std::optional<std::vector<float>> mxfp4_gemv(Slice<uint8_t> packed, Slice<uint8_t> scales, Slice<float> x, size_t n, size_t k) {
        std::vector<float> out(n);
        return some(larql_hip_mxfp4_gemv(ctx_, packed.ptr, packed.len, scales.ptr, scales.len, x.ptr, x.len, n, k, out.data()), out);
    }

    // VectorIndex::gate_knn (larql-vindex/src/index/compute/gate_knn/dispatch.rs:22-52)
    std::optional<std::vector<std::pair<size_t, float>>> gate_knn(QuantFormat f, Slice<uint8_t> gate, Slice<float> residual,
                                                                  size_t n_features, size_t hidden, size_t top_k) {
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

    larql_hip_ctx *raw() { return ctx_; }

  private:
    static std::optional<std::vector<float>> some(int rc, std::vector<float> &out) {
        if (rc != LARQL_OK) return std::nullopt;
        return std::move(out);
    }
    larql_hip_ctx *ctx_ = nullptr;
};

}  // namespace larql
