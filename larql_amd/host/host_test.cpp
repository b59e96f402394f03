// host_test.cpp — exercises the C++ HipBackend mirror the way the reference's own
// backend tests read: closed-form Q4_K blocks, refusals as nullopt, the
// trait-default None for formats this entry does not serve.  Exits non-zero on
// the first failed check; prints "host_test ok" otherwise.  Needs a GPU.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#include "hip_backend.hpp"

#define CHECK(cond)                                                          \
    do {                                                                     \
        if (!(cond)) { std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); return 1; } \
    } while (0)

// One Q4_K super-block with d=1, dmin=0.5, scale j = j+1, min j = j, low nibble 3, high nibble 5.
static void make_block(uint8_t *blk) {
    std::memset(blk, 0, 144);
    blk[0] = 0x00; blk[1] = 0x3C; blk[2] = 0x00; blk[3] = 0x38;
    uint8_t sc[8], mn[8];
    for (int j = 0; j < 8; j++) { sc[j] = (uint8_t)(j + 1); mn[j] = (uint8_t)j; }
    for (int j = 0; j < 4; j++) {
        blk[4 + j] = (uint8_t)((sc[j] & 63) | (((sc[j + 4] >> 4) & 3) << 6));
        blk[8 + j] = (uint8_t)((mn[j] & 63) | (((mn[j + 4] >> 4) & 3) << 6));
        blk[12 + j] = (uint8_t)((sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4));
    }
    for (int i = 16; i < 144; i++) blk[i] = (uint8_t)(3 | (5 << 4));
}

int main() {
    larql::HipBackend be;
    std::printf("%s | %s\n", be.name().c_str(), be.device_info().c_str());
    CHECK(be.supports_quant(larql::QuantFormat::Q4_K) && be.supports_quant(larql::QuantFormat::MXFP4));
    CHECK(be.supports_quant(larql::QuantFormat::Q6_K) && !be.supports_quant(larql::QuantFormat::Q5_K));
    {
        // one Q6_K super-block: every code 32 + 5 (low nibble 5, high bits 2), scale 3, d = 0.5 -> weight 7.5; x = 1 -> 1920
        std::vector<uint8_t> b6(210, 0);
        for (int i = 0; i < 128; i++) b6[i] = 0x55;
        for (int i = 128; i < 192; i++) b6[i] = 0xAA;
        for (int i = 192; i < 208; i++) b6[i] = 3;
        b6[208] = 0x00; b6[209] = 0x38;  // f16 0.5
        std::vector<float> x6(256, 1.0f);
        auto o6 = be.q6k_matvec({b6.data(), b6.size()}, {x6.data(), x6.size()}, 1, 256);
        CHECK(o6 && std::fabs((*o6)[0] - 1920.0f) < 1e-2f);
        CHECK(!be.q6k_matvec({b6.data(), b6.size() - 1}, {x6.data(), x6.size()}, 1, 256));
    }

    const size_t rows = 70, hidden = 512;
    std::vector<uint8_t> w(rows * 2 * 144);
    for (size_t b = 0; b < rows * 2; b++) make_block(&w[b * 144]);
    std::vector<float> x(hidden, 1.0f);
    // per super-block: sum_s 32*(sc_s*q - 0.5*mn_s), q = 3 (even s) or 5 (odd s)
    double per_sb = 0;
    for (int s = 0; s < 8; s++) per_sb += 32.0 * ((s + 1) * (s % 2 == 0 ? 3 : 5) - 0.5 * s);
    auto out = be.q4k_matvec(w, x, rows, hidden);
    CHECK(out.has_value() && out->size() == rows);
    for (float v : *out) CHECK(std::fabs(v - 2 * per_sb) < 1e-3);

    {
        // Q8_K-activation path on the same matrix: x = 1 quantises to d = 1/127, every code 127, every sub-block sum 32*127;
        // the integer sums are exact, so the output is 2 * ((d_w*d_y)*sum1 - (dmin_w*d_y)*sum2) up to the two f32 roundings
        auto a = be.quantize_x_to_q8k({x.data(), x.size()});
        CHECK(a && a->qs.size() == hidden && a->d.size() == 2 && a->sums.size() == 16);
        for (int8_t q : a->qs) CHECK(q == 127);
        CHECK(a->d[0] == 1.0f / 127.0f && a->sums[5] == 32 * 127);
        auto o8 = be.q4k_q8k_matvec(w, *a, rows, hidden);
        CHECK(o8.has_value() && o8->size() == rows);
        for (float v : *o8) CHECK(std::fabs(v - 2 * per_sb) < 2e-3 * per_sb);
        a->qs.pop_back();
        CHECK(!be.q4k_q8k_matvec(w, *a, rows, hidden));  // activation of the wrong length: refused
    }

    // refusals: None, never a wrong vector (backend/quant_matvec.rs:378-427, kernel_shape.rs)
    std::vector<float> x_short(hidden - 1, 1.0f);
    CHECK(!be.q4k_matvec(w, x_short, rows, hidden).has_value());
    CHECK(!be.q4k_matvec(larql::Slice<uint8_t>(w.data(), w.size() - 1), x, rows, hidden).has_value());
    CHECK(!be.q4k_matvec(w, x, rows, 500).has_value());
    auto zero = be.q4k_matvec(larql::Slice<uint8_t>(), larql::Slice<float>(), 4, 0);
    CHECK(zero.has_value() && zero->size() == 4 && (*zero)[0] == 0.0f);

    // dual == two singles, bit for bit
    auto dual = be.q4k_dual_matvec(w, w, x, rows, hidden);
    CHECK(dual.has_value() && dual->first == *out && dual->second == *out);
    // matmul rows == stacked matvec
    std::vector<float> X(3 * hidden, 1.0f);
    auto mm = be.q4k_matmul(w, X, rows, hidden, 3);
    CHECK(mm.has_value() && mm->size() == 3 * rows && std::fabs((*mm)[2 * rows + 5] - (*out)[5]) < 1e-4);

    // quant_matvec routes Q4_K, refuses the formats whose scales ride elsewhere
    CHECK(be.quant_matvec(larql::QuantFormat::Q4_K, w, x, rows, hidden).has_value());
    CHECK(!be.quant_matvec(larql::QuantFormat::Q8_0, w, x, rows, hidden).has_value());
    CHECK(!be.quant_matvec(larql::QuantFormat::MXFP4, w, x, rows, hidden).has_value());

    // MXFP4 KATs (larql-models/src/quant/mxfp4.rs:312-380): 0x22 -> 1.0 each, scale 128 -> 2x, scale 0 -> 0
    std::vector<uint8_t> packed(2 * 16, 0x22), scales = {127, 128};
    std::vector<float> x32(32, 1.0f);
    auto m = be.mxfp4_gemv(packed, scales, x32, 2, 32);
    CHECK(m.has_value() && (*m)[0] == 32.0f && (*m)[1] == 64.0f);
    scales = {0, 127};
    m = be.mxfp4_gemv(packed, scales, x32, 2, 32);
    CHECK(m.has_value() && (*m)[0] == 0.0f && (*m)[1] == 32.0f);
    CHECK(!be.mxfp4_gemv(packed, scales, x32, 2, 33).has_value());

    // gate-KNN closed form (gate_knn/mod.rs:231-243) through one-hot f32 gates
    std::vector<float> gate(4 * 256, 0.0f), res(256, 0.0f);
    for (int i = 0; i < 4; i++) gate[i * 256 + i] = 1.0f;
    res[0] = 0.1f; res[1] = -0.9f; res[2] = 0.5f; res[3] = 0.3f;
    auto hits = be.gate_knn(larql::QuantFormat::F32, larql::Slice<uint8_t>((const uint8_t *)gate.data(), gate.size() * 4), res, 4, 256, 2);
    CHECK(hits.has_value() && hits->size() == 2 && (*hits)[0].first == 1 && (*hits)[1].first == 2);
    CHECK(std::fabs((*hits)[0].second + 0.9f) < 1e-6);

    // the batch forms: one hit list per position, the union gate_knn_batch returns, the full score matrix
    {
        std::vector<float> res2(2 * 256, 0.0f);
        for (int i = 0; i < 4; i++) res2[i] = res[i];
        res2[256 + 0] = 0.7f; res2[256 + 3] = -0.2f;
        const larql::Slice<uint8_t> g8((const uint8_t *)gate.data(), gate.size() * 4);
        auto per = be.gate_knn_positions(larql::QuantFormat::F32, g8, res2, 2, 4, 256, 2);
        CHECK(per && per->size() == 2 && (*per)[0].size() == 2 && (*per)[1].size() == 2);
        CHECK((*per)[0][0].first == 1 && (*per)[0][1].first == 2 && (*per)[1][0].first == 0 && (*per)[1][1].first == 3);
        auto uni = be.gate_knn_batch(larql::QuantFormat::F32, g8, res2, 2, 4, 256, 2);
        CHECK(uni && *uni == (std::vector<size_t>{0, 1, 2, 3}));
        auto sc = be.gate_scores_batch(larql::QuantFormat::F32, g8, res2, 2, 4, 256);
        CHECK(sc && sc->size() == 8 && std::fabs((*sc)[1] + 0.9f) < 1e-6 && std::fabs((*sc)[4] - 0.7f) < 1e-6 && (*sc)[5] == 0.0f);
        CHECK(!be.gate_knn_positions(larql::QuantFormat::F32, g8, res2, 3, 4, 256, 2));          // x is not [3, 256]
        auto all = be.gate_knn(larql::QuantFormat::F32, g8, res, 4, 256, (size_t)1 << 40);          // "every feature"
        CHECK(all && all->size() == 4);
    }

    // Q8-input forms (quant_matvec.rs:100-151): codes 2 x scale 0.5 = the activation 1.0 -> the f32 call's bits
    {
        std::vector<int8_t> q8(hidden, 2);
        std::vector<float> q8s(hidden / 32, 0.5f);
        auto o = be.quant_matvec_q8_input(larql::QuantFormat::Q4_K, w, q8, q8s, rows, hidden);
        CHECK(o && *o == *out);
        CHECK(!be.quant_matvec_q8_input(larql::QuantFormat::MXFP4, w, q8, q8s, rows, hidden));
        // Q4_0: d = 0.5, every nibble 10 -> weight 1.0; activation 3 x 0.25 -> 0.75; 64 of them -> 48
        std::vector<uint8_t> q40(3 * 2 * 18);
        for (size_t b = 0; b < 6; b++) { q40[b * 18] = 0x00; q40[b * 18 + 1] = 0x38; std::memset(&q40[b * 18 + 2], 0xAA, 16); }
        std::vector<int8_t> q8b(64, 3);
        std::vector<float> q8bs(2, 0.25f);
        auto o4 = be.q4_matvec(q40, q8b, q8bs, 3, 64);
        CHECK(o4 && o4->size() == 3 && (*o4)[0] == 48.0f && (*o4)[2] == 48.0f);
        auto o4b = be.quant_matvec_q8_input(larql::QuantFormat::Q4_0, q40, q8b, q8bs, 3, 64);
        CHECK(o4b && *o4b == *o4);
    }

    // ggml Q8_0 head: row r has d = 1 and every code r + 1; x = 1 over k = 64 -> 64 (r + 1); top-2 by value = rows 4, 3
    {
        const size_t n = 5, k = 64;
        std::vector<uint8_t> q8w(n * 2 * 34);
        for (size_t r = 0; r < n; r++)
            for (size_t b = 0; b < 2; b++) {
                uint8_t *blk = &q8w[(r * 2 + b) * 34];
                blk[0] = 0x00; blk[1] = 0x3C;
                std::memset(blk + 2, (int)(r + 1), 32);
            }
        std::vector<float> ones(k, 1.0f);
        auto o = be.q8_0_gemv(q8w, ones, n, k);
        CHECK(o && o->size() == n);
        for (size_t r = 0; r < n; r++) CHECK((*o)[r] == 64.0f * (float)(r + 1));
        auto top = be.q8_0_gemv_topk(q8w, ones, n, k, 2);
        CHECK(top && top->size() == 2 && (*top)[0].first == 4 && (*top)[0].second == 320.0f && (*top)[1].first == 3);
        auto every = be.q8_0_gemv_topk(q8w, ones, n, k, 1000);   // K beyond the rows: all of them, in order
        CHECK(every && every->size() == n && (*every)[4].first == 0);
        CHECK(!be.q8_0_gemv(q8w, ones, n, 48));
    }

    // dense gemv: bf16 / f16 rows of 2^r against x = 1 (exact), the multi forms equal to the single calls, a bad
    // matrix refusing the whole batch, the unforced call leaving a tiny matrix to the caller's BLAS
    {
        const size_t n = 4, k = 64;
        const uint16_t bf[4] = {0x3F00, 0x3F80, 0x4000, 0x4080}, hf[4] = {0x3800, 0x3C00, 0x4000, 0x4400};  // 0.5, 1, 2, 4
        std::vector<uint8_t> wb(n * k * 2), wh(n * k * 2);
        for (size_t r = 0; r < n; r++)
            for (size_t c = 0; c < k; c++) { std::memcpy(&wb[(r * k + c) * 2], &bf[r], 2); std::memcpy(&wh[(r * k + c) * 2], &hf[r], 2); }
        std::vector<float> ones(k, 1.0f);
        auto ob = be.bf16_gemv_force(wb, ones, n, k), oh = be.f16_gemv_force(wh, ones, n, k);
        CHECK(ob && oh && (*ob)[0] == 32.0f && (*ob)[3] == 256.0f && *oh == *ob);
        CHECK(!be.bf16_gemv(wb, ones, n, k) && !be.f16_gemv(wh, ones, n, k));       // below the flop threshold
        CHECK(be.supports(larql::Capability::F16Gemv) && be.supports(larql::Capability::QuantMatVec));
        std::vector<larql::DenseMatrix> three = {{wb, n, k}, {larql::Slice<uint8_t>(wb.data(), 2 * k * 2), 2, k}, {wb, n, k}};
        auto mb = be.bf16_gemv_multi(three, ones);
        CHECK(mb && mb->size() == 3 && (*mb)[0] == *ob && (*mb)[2] == *ob && (*mb)[1].size() == 2 && (*mb)[1][1] == 64.0f);
        auto mh = be.f16_gemv_multi({{wh, n, k}}, ones);
        CHECK(mh && mh->size() == 1 && (*mh)[0] == *oh);
        three[1].k = 32;
        CHECK(!be.bf16_gemv_multi(three, ones));
        auto none = be.bf16_gemv_multi({}, ones);
        CHECK(none && none->empty());
        std::vector<float> wf(n * k);
        for (size_t r = 0; r < n; r++) for (size_t c = 0; c < k; c++) wf[r * k + c] = (float)(r + 1);
        auto of = be.f32_gemv_force(wf, ones, n, k);
        CHECK(of && (*of)[2] == 192.0f && !be.f32_gemv(wf, ones, n, k));
    }

    // mxfp4_gemv_multi == the single calls
    {
        std::vector<uint8_t> p2(2 * 16, 0x22), s2 = {127, 128}, s3 = {126, 127};
        auto mm2 = be.mxfp4_gemv_multi({{p2, s2, 2, 32}, {p2, s3, 2, 32}}, x32);
        CHECK(mm2 && mm2->size() == 2 && (*mm2)[0][0] == 32.0f && (*mm2)[0][1] == 64.0f && (*mm2)[1][0] == 16.0f && (*mm2)[1][1] == 32.0f);
        CHECK(!be.mxfp4_gemv_multi({{p2, s2, 2, 32}, {p2, s3, 2, 33}}, x32));
    }

    // A MoE layer from per-expert slices (MoeLayerWeights, pipeline/moe.rs:469-541), closed form: expert 0 is all ones
    // (code 2, exponent 127), expert 1 all zeros; x = 1/128 makes every gate and up row dot 1.0, ClampedGlu gives
    // (1 + 1) * sigmoid(1.702), the down rows sum 128 of those; the router's rows +1 / -1 pick expert 0 with weight 1.
    {
        const size_t H = 128, I = 128, G = H / 32;
        std::vector<uint8_t> gu1(2 * I * G * 16, 0x22), gu0(2 * I * G * 16, 0x00), dn1(H * (I / 32) * 16, 0x22), dn0(H * (I / 32) * 16, 0x00);
        std::vector<uint8_t> sgu(2 * I * G, 127), sdn(H * (I / 32), 127);
        std::vector<float> rp(2 * H);
        for (size_t c = 0; c < H; c++) { rp[c] = 1.0f; rp[H + c] = -1.0f; }
        larql::MoeLayerWeights m;
        m.experts_gate_up = {gu1, gu0}; m.experts_down = {dn1, dn0};
        m.expert_scales.paired = true; m.expert_scales.gate_up = {sgu, sgu}; m.expert_scales.down = {sdn, sdn};
        m.router_proj = rp; m.num_experts = 2; m.top_k = 1; m.intermediate_size = I;
        auto layer = be.moe_layer(m, H);
        CHECK(layer.has_value());
        std::vector<float> xm(2 * H, 1.0f / 128.0f);
        for (size_t c = 0; c < H; c++) xm[H + c] = -1.0f / 128.0f;   // the second token's logits are -1 / +1: expert 1, all zeros
        auto r1 = layer->forward(xm, xm, 2);
        CHECK(r1 && r1->experts.size() == 2 && r1->experts[0] == 0 && r1->experts[1] == 1 && r1->weights[0] == 1.0f && r1->weights[1] == 1.0f);
        const double want = 128.0 * 2.0 / (1.0 + std::exp(-1.702));
        for (size_t c = 0; c < H; c++) { CHECK(std::fabs(r1->out[c] - want) < 1e-4 * want); CHECK(r1->out[H + c] == 0.0f); }
        CHECK(!layer->forward(xm, larql::Slice<float>(xm.data(), H), 2));                 // x is not [2, H]
        m.expert_scales.paired = false;                                                    // Inline scales on an MXFP4 bank: refused
        CHECK(!be.moe_layer(m, H));
        m.expert_scales.paired = true; m.gate_rule.kind = larql::MoeGateRule::GatedSilu;      // an MXFP4 bank under another gate rule: no kernel
        CHECK(!be.moe_layer(m, H));
    }

    // The same from a Q4_K bank (Inline scales, ContiguousHalves rows): cpu_moe_forward's integer path in closed form.
    // Every weight is 0.5 * 1 * 2 = 1.0; x = 127 / 2^14 quantises exactly (d = 2^-14, codes 127), so gate = up =
    // 256 x = 1.984375 in every row, the SiLU-gated activation is one constant (exact as Q8_K too), and a down row sums
    // 256 of them.
    {
        const size_t H = 256, I = 256;
        uint8_t blk[144];
        std::memset(blk, 0, 144);
        blk[0] = 0x00; blk[1] = 0x38;                                  // d = 0.5, dmin = 0
        for (int j = 0; j < 4; j++) { blk[4 + j] = 1; blk[12 + j] = 1; }  // every 6-bit scale 1, every min 0
        std::memset(blk + 16, 0x22, 128);
        std::vector<uint8_t> gu(2 * I * 144), dn(H * 144);
        for (size_t r = 0; r < 2 * I; r++) std::memcpy(&gu[r * 144], blk, 144);
        for (size_t r = 0; r < H; r++) std::memcpy(&dn[r * 144], blk, 144);
        std::vector<float> rp(H, 0.0f);
        larql::MoeLayerWeights m;
        m.experts_gate_up = {gu}; m.experts_down = {dn};
        m.fused_row_layout = larql::MoeFusedRowLayout::ContiguousHalves;
        m.expert_data_format = larql::QuantFormat::Q4_K;
        m.gate_rule.kind = larql::MoeGateRule::GatedSilu;
        m.router_proj = rp; m.num_experts = 1; m.top_k = 1; m.intermediate_size = I;
        auto layer = be.moe_layer(m, H);
        CHECK(layer.has_value());
        std::vector<float> xm(H, 127.0f / 16384.0f);
        auto r1 = layer->forward(xm, xm, 1);
        const double g = 256.0 * 127.0 / 16384.0, want = 256.0 * (g / (1.0 + std::exp(-g))) * g;
        CHECK(r1 && r1->experts[0] == 0 && r1->weights[0] == 1.0f);
        for (size_t c = 0; c < H; c++) CHECK(std::fabs(r1->out[c] - want) < 1e-5 * want);
        m.fused_row_layout = larql::MoeFusedRowLayout::Interleaved;   // the CPU tier refuses an interleaved k-quant bank; so does this one
        CHECK(!be.moe_layer(m, H));
    }

    auto clock = be.submission_clock();
    CHECK(clock.has_value() && clock->submissions > 0);
    std::printf("host_test ok\n");
    return 0;
}
