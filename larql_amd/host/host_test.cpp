// host_test.cpp — exercises the C++ HipBackend mirror the way the reference's own
// backend tests read: closed-form Q4_K blocks, refusals as nullopt, the
// trait-default None for formats this entry does not serve.  Exits non-zero on
// the first failed check; prints "host_test ok" otherwise.  Needs a GPU.
#include <cmath>
#include <cstdio>
#include <cstring>

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

    auto clock = be.submission_clock();
    CHECK(clock.has_value() && clock->submissions > 0);
    std::printf("host_test ok\n");
    return 0;
}
