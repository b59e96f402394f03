/*
 * larql_oracle.c — CPU restatement of the LARQL reference algorithms on the
 * quantised decode path (see larql_oracle.h).
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP path and the CPU baseline
 * of the benchmark.  Never linked into, or called from, the product library.
 *
 * Paths in the citations are relative to the reference checkout, under
 * crates/.  The reference is Rust: f32 arithmetic is never contracted to FMA,
 * `f32::round` rounds half away from zero (roundf), `as u8`/`as i8`/`as i32`
 * casts saturate and map NaN to 0, and `Iterator::sum` adds left to right.
 * Compile with -ffp-contract=off.
 *
 * How each function is pinned is stated at the function.  "restatement +
 * KATs" means no reference-held vector exists for it; the test-suite then
 * holds it to closed-form cases and to an independent numpy restatement.
 */
#include "larql_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ bits */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* Rust `x as u8` / `as i8` / `as i32` for an f32 that was already clamped:
 * saturating, NaN -> 0. */
static inline int32_t sat_i32(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}
static inline uint8_t sat_u8(float v) {
    if (v != v) return 0;
    if (v <= 0.0f) return 0;
    if (v >= 255.0f) return 255;
    return (uint8_t)v;
}
static inline int8_t sat_i8(float v) {
    if (v != v) return 0;
    if (v <= -128.0f) return -128;
    if (v >= 127.0f) return 127;
    return (int8_t)v;
}
/* f32::clamp(lo, hi): NaN stays NaN. */
static inline float clampf(float v, float lo, float hi) {
    if (v < lo) return lo;
    if (v > hi) return hi;
    return v;
}

/* ------------------------------------------------------------ half/bf16 */

/* larql-models/src/quant/half.rs:14-35 and, bit-identically,
 * larql-compute/src/cpu/ops/q4_common/f16.rs:60-102.
 * Pinned: all 65 536 inputs against numpy float16 (IEEE) in the tests, plus
 * the reference's pinned subnormals (q4_common/tests/f16_subnormal_*.rs). */
float lq_f16_to_f32(uint16_t bits) {
    uint32_t sign = ((uint32_t)(bits >> 15)) << 31;
    uint32_t exp = (bits >> 10) & 0x1F;
    uint32_t mant = bits & 0x3FF;
    if (exp == 0) {
        if (mant == 0) return u2f(sign);
        uint32_t e = 1, m = mant;
        while ((m & 0x400) == 0) { m <<= 1; e += 1; }
        return u2f(sign | ((114 - e) << 23) | ((m & 0x3FF) << 13));
    }
    if (exp == 31) return u2f(sign | (0xFFu << 23) | (mant << 13));
    return u2f(sign | ((exp + 127 - 15) << 23) | (mant << 13));
}

/* larql-compute/src/cpu/ops/q4_common/f16.rs:10-41 — truncating, keeps
 * subnormals; the Q4_K encoder's header conversion.
 * Pinned: restatement + KATs (normals truncate, subnormals shift with the
 * implicit one, below 2^-24 gives signed zero). */
uint16_t lq_f32_to_f16_trunc(float val) {
    uint32_t bits = f2u(val);
    uint32_t sign = (bits >> 16) & 0x8000;
    int32_t exp = (int32_t)((bits >> 23) & 0xFF);
    uint32_t mant = bits & 0x7FFFFF;
    if (exp == 0) return (uint16_t)sign;
    if (exp == 255) return (uint16_t)(sign | 0x7C00 | (mant >> 13));
    int32_t new_exp = exp - 127 + 15;
    if (new_exp >= 31) return (uint16_t)(sign | 0x7C00);
    if (new_exp <= 0) {
        int32_t shift = 1 - new_exp;
        if (13 + (uint32_t)shift >= 24) return (uint16_t)sign;
        uint32_t sub_mant = (mant | 0x800000) >> (13 + (uint32_t)shift);
        return (uint16_t)(sign | sub_mant);
    }
    return (uint16_t)(sign | ((uint32_t)new_exp << 10) | (mant >> 13));
}

/* larql-models/src/quant/half.rs:70-104 — IEEE round-to-nearest-even with
 * subnormals; the Q8_0 encoder's scale conversion.
 * Pinned: the reference's table (half.rs:160-200) and numpy float16 on a
 * sweep of bit patterns. */
uint16_t lq_f32_to_f16_nearest(float value) {
    uint32_t bits = f2u(value);
    uint16_t sign = (uint16_t)((bits >> 16) & 0x8000);
    int32_t exp = (int32_t)((bits >> 23) & 0xFF);
    uint32_t mant = bits & 0x007FFFFF;
    if (exp == 255) return (uint16_t)(sign | (mant == 0 ? 0x7C00 : 0x7E00));
    int32_t exp16 = exp - 127 + 15;
    if (exp16 >= 31) return (uint16_t)(sign | 0x7C00);
    uint32_t significand, shift;
    if (exp16 >= 1) { significand = mant; shift = 13; }
    else if (exp == 0 || exp16 < -10) return sign;
    else { significand = mant | 0x00800000; shift = (uint32_t)(14 - exp16); }
    uint32_t magnitude = significand >> shift;
    uint32_t remainder = significand & ((1u << shift) - 1);
    uint32_t half = 1u << (shift - 1);
    if (remainder > half || (remainder == half && (magnitude & 1) == 1)) magnitude += 1;
    if (exp16 >= 1) magnitude += ((uint32_t)exp16) << 10;
    return (uint16_t)(sign | (uint16_t)magnitude);
}

/* The inline conversion inside quantize_q4_0,
 * larql-compute/src/cpu/ops/q4_common/quantize.rs:41-58 — truncating, and
 * everything below the f16 normal range becomes signed zero. */
uint16_t lq_f32_to_f16_flush(float v) {
    uint32_t bits = f2u(v);
    uint32_t sign = (bits >> 16) & 0x8000;
    int32_t exp = (int32_t)((bits >> 23) & 0xFF);
    uint32_t mant = bits & 0x7FFFFF;
    if (exp == 0) return (uint16_t)sign;
    if (exp == 255) return (uint16_t)(sign | 0x7C00 | (mant >> 13));
    int32_t new_exp = exp - 127 + 15;
    if (new_exp >= 31) return (uint16_t)(sign | 0x7C00);
    if (new_exp <= 0) return (uint16_t)sign;
    return (uint16_t)(sign | ((uint32_t)new_exp << 10) | (mant >> 13));
}

/* larql-models/src/quant/half.rs:107-109 (truncate) and :38-40. */
uint16_t lq_f32_to_bf16(float v) { return (uint16_t)(f2u(v) >> 16); }
float lq_bf16_to_f32(uint16_t bits) { return u2f(((uint32_t)bits) << 16); }
void lq_f32_to_bf16_slice(const float *src, size_t n, uint16_t *dst) {
    for (size_t i = 0; i < n; i++) dst[i] = lq_f32_to_bf16(src[i]);
}

/* ------------------------------------------------------------------ Q4_K */

/* get_scale_min_k4 unpack as every Q4_K reader in the reference writes it,
 * e.g. q4_common/matvec_f32.rs:124-131. */
static inline void q4k_unpack_scales(const uint8_t *p, uint8_t scales[8], uint8_t mins[8]) {
    for (int j = 0; j < 4; j++) {
        scales[j] = p[j] & 0x3F;
        mins[j] = p[j + 4] & 0x3F;
        scales[j + 4] = (uint8_t)((p[j + 8] & 0x0F) | ((p[j] >> 6) << 4));
        mins[j + 4] = (uint8_t)((p[j + 8] >> 4) | ((p[j + 4] >> 6) << 4));
    }
}

/* larql-compute/src/cpu/ops/q4_common/quantize.rs:89-189.
 * Note the nibble encode uses the un-rounded f32 d/dmin, not the f16 values
 * written to the header (:170-186).
 * Pinned: restatement + KATs (zero block, constant blocks, two-level block)
 * + byte-for-byte agreement with an independent numpy restatement + the
 * round-trip bound of larql-compute/tests/test_q4k_parity.rs:48-65.
 * No reference-held Q4_K encoder bytes exist. */
int lq_quantize_q4_k(const float *data, size_t n, uint8_t *out) {
    if (n % 256 != 0) return 1; /* the reference asserts */
    size_t n_sb = n / 256;
    for (size_t sb = 0; sb < n_sb; sb++) {
        const float *block = data + sb * 256;
        uint8_t *o = out + sb * 144;
        float sub_mins[8], sub_maxs[8];
        for (int j = 0; j < 8; j++) {
            const float *sub = block + j * 32;
            float mn = INFINITY, mx = -INFINITY;
            for (int l = 0; l < 32; l++) { mn = fminf(mn, sub[l]); mx = fmaxf(mx, sub[l]); }
            sub_mins[j] = fminf(mn, 0.0f);
            sub_maxs[j] = fmaxf(mx, 0.0f);
        }
        float global_max_range = 0.0f;
        for (int j = 0; j < 8; j++) global_max_range = fmaxf(global_max_range, sub_maxs[j] - sub_mins[j]);
        float global_min = INFINITY;
        for (int j = 0; j < 8; j++) global_min = fminf(global_min, sub_mins[j]);

        float d = global_max_range > 0.0f ? global_max_range / (15.0f * 63.0f) : 0.0f;
        float dmin = global_min < 0.0f ? -global_min / 63.0f : 0.0f;

        uint16_t dh = lq_f32_to_f16_trunc(d), mh = lq_f32_to_f16_trunc(dmin);
        o[0] = (uint8_t)(dh & 0xFF); o[1] = (uint8_t)(dh >> 8);
        o[2] = (uint8_t)(mh & 0xFF); o[3] = (uint8_t)(mh >> 8);

        uint8_t q_scales[8], q_mins[8];
        for (int j = 0; j < 8; j++) {
            float range = sub_maxs[j] - sub_mins[j];
            q_scales[j] = d > 0.0f ? sat_u8(clampf(roundf(range / (15.0f * d)), 0.0f, 63.0f)) : 0;
            q_mins[j] = dmin > 0.0f ? sat_u8(clampf(roundf(-sub_mins[j] / dmin), 0.0f, 63.0f)) : 0;
        }
        uint8_t *packed = o + 4;
        for (int j = 0; j < 4; j++) {
            packed[j] = (uint8_t)((q_scales[j] & 0x3F) | (((q_scales[j + 4] >> 4) & 0x03) << 6));
            packed[j + 4] = (uint8_t)((q_mins[j] & 0x3F) | (((q_mins[j + 4] >> 4) & 0x03) << 6));
            packed[j + 8] = (uint8_t)((q_scales[j + 4] & 0x0F) | ((q_mins[j + 4] & 0x0F) << 4));
        }
        uint8_t *qs = o + 16;
        for (int g = 0; g < 4; g++) {
            int sb_lo = 2 * g, sb_hi = 2 * g + 1;
            float sc_lo = d * (float)q_scales[sb_lo];
            float sc_hi = d * (float)q_scales[sb_hi];
            float mn_lo = dmin * (float)q_mins[sb_lo];
            float mn_hi = dmin * (float)q_mins[sb_hi];
            float inv_lo = sc_lo > 0.0f ? 1.0f / sc_lo : 0.0f;
            float inv_hi = sc_hi > 0.0f ? 1.0f / sc_hi : 0.0f;
            const float *lo_sub = block + sb_lo * 32;
            const float *hi_sub = block + sb_hi * 32;
            for (int l = 0; l < 32; l++) {
                uint8_t lo = sat_u8(clampf(roundf((lo_sub[l] + mn_lo) * inv_lo), 0.0f, 15.0f));
                uint8_t hi = sat_u8(clampf(roundf((hi_sub[l] + mn_hi) * inv_hi), 0.0f, 15.0f));
                qs[g * 32 + l] = (uint8_t)(lo | (hi << 4));
            }
        }
    }
    return 0;
}

/* larql-compute/src/cpu/ops/q4_common/dequant.rs:9-53, the same values as
 * larql-models/src/quant/ggml/q4_k.rs:286-338.  Refusal = empty Vec.
 * Pinned: bit-exact against the reference-held llama.cpp golden
 * (larql-vindex/src/format/vindex3/represent/fixtures/ggml_kquant_golden.json,
 * case q4_K). */
int lq_dequantize_q4_k(const uint8_t *data, size_t data_len, size_t n, float *out) {
    if (n % 256 != 0) return 1;
    size_t n_blocks = n / 256;
    if (data_len < n_blocks * 144) return 1;
    for (size_t sb = 0; sb < n_blocks; sb++) {
        const uint8_t *block = data + sb * 144;
        float d = lq_f16_to_f32((uint16_t)(block[0] | (block[1] << 8)));
        float dmin = lq_f16_to_f32((uint16_t)(block[2] | (block[3] << 8)));
        uint8_t scales[8], mins[8];
        q4k_unpack_scales(block + 4, scales, mins);
        const uint8_t *quants = block + 16;
        size_t sb_base = sb * 256;
        for (int g = 0; g < 4; g++) {
            int sb_lo = 2 * g, sb_hi = 2 * g + 1;
            float sc_lo = d * (float)scales[sb_lo], sc_hi = d * (float)scales[sb_hi];
            float mn_lo = dmin * (float)mins[sb_lo], mn_hi = dmin * (float)mins[sb_hi];
            const uint8_t *chunk = quants + g * 32;
            for (int l = 0; l < 32; l++) {
                uint8_t byte = chunk[l];
                out[sb_base + sb_lo * 32 + l] = sc_lo * (float)(byte & 0x0F) - mn_lo;
                out[sb_base + sb_hi * 32 + l] = sc_hi * (float)((byte >> 4) & 0x0F) - mn_hi;
            }
        }
    }
    return 0;
}

/* KernelShapeError::check, larql-compute/src/cpu/ops/kernel_shape.rs:46-75. */
static int kernel_shape_ok(size_t out_len, size_t rows, size_t x_len, size_t cols,
                           size_t weight_bytes, size_t block_elems, size_t block_bytes) {
    size_t needed = (cols / block_elems) * block_bytes * rows;
    return out_len == rows && x_len == cols && cols % block_elems == 0 && weight_bytes >= needed;
}

/* q4_dual_dot_32, scalar arm: q4_common/dual.rs:178-199. */
static inline void q4_dual_dot_32(const uint8_t *chunk, const float *x_lo, const float *x_hi,
                                  float *dot_lo_out, float *dot_hi_out) {
    float dot_lo = 0.0f, dot_hi = 0.0f;
    for (int l = 0; l < 32; l++) {
        uint8_t byte = chunk[l];
        float q_lo = (float)(byte & 0x0F);
        float q_hi = (float)((byte >> 4) & 0x0F);
        dot_lo += q_lo * x_lo[l];
        dot_hi += q_hi * x_hi[l];
    }
    *dot_lo_out = dot_lo; *dot_hi_out = dot_hi;
}

/* process_q4k_superblock: q4_common/matvec_f32.rs:116-155. */
static inline float process_q4k_superblock(const uint8_t *w, const float *x, const float *sum_x,
                                           size_t row_base, size_t sb) {
    const uint8_t *block = w + row_base + sb * 144;
    float d = lq_f16_to_f32((uint16_t)(block[0] | (block[1] << 8)));
    float dmin = lq_f16_to_f32((uint16_t)(block[2] | (block[3] << 8)));
    uint8_t scales[8], mins[8];
    q4k_unpack_scales(block + 4, scales, mins);
    const uint8_t *quants = block + 16;
    size_t x_sb_base = sb * 256;
    float acc = 0.0f;
    for (int g = 0; g < 4; g++) {
        int sb_lo = 2 * g, sb_hi = 2 * g + 1;
        float sc_lo = d * (float)scales[sb_lo], sc_hi = d * (float)scales[sb_hi];
        float mn_lo = dmin * (float)mins[sb_lo], mn_hi = dmin * (float)mins[sb_hi];
        float sumy_lo = sum_x[sb * 8 + sb_lo], sumy_hi = sum_x[sb * 8 + sb_hi];
        float dot_lo, dot_hi;
        q4_dual_dot_32(quants + g * 32, x + x_sb_base + sb_lo * 32, x + x_sb_base + sb_hi * 32,
                       &dot_lo, &dot_hi);
        acc += sc_lo * dot_lo - mn_lo * sumy_lo;
        acc += sc_hi * dot_hi - mn_hi * sumy_hi;
    }
    return acc;
}

static float *q4k_sum_x(const float *x, size_t n_blocks) {
    /* q4_common/matvec_f32.rs:63-74 */
    size_t n_sub = n_blocks * 8;
    float *sum_x = (float *)malloc((n_sub ? n_sub : 1) * sizeof(float));
    for (size_t sub = 0; sub < n_sub; sub++) {
        float s = 0.0f;
        for (int l = 0; l < 32; l++) s += x[sub * 32 + l];
        sum_x[sub] = s;
    }
    return sum_x;
}

static void q4k_rows(float *out, const float *x, const uint8_t *w, const float *sum_x,
                     size_t r0, size_t r1, size_t n_blocks) {
    size_t row_bytes = n_blocks * 144;
    for (size_t r = r0; r < r1; r++) {
        float acc = 0.0f;
        for (size_t sb = 0; sb < n_blocks; sb++)
            acc += process_q4k_superblock(w, x, sum_x, r * row_bytes, sb);
        out[r] = acc;
    }
}

/* CpuBackend::q4k_matvec -> q4k_matvec_into:
 * larql-compute/src/cpu/mod.rs:95-114, q4_common/matvec_f32.rs:37-106.
 * Row chunking only decides which thread runs a row, so the serial loop is
 * the same arithmetic.
 * Pinned: equals sum(dequantize(bytes) * x) to rounding on the golden q4_K
 * bytes and on seeded bytes (the reference's own oracle,
 * q4_common/tests/quantize_q4_0_tests.rs:69-149), f64 brute force on small
 * shapes, and the refusal table of quantize_q4_0_tests.rs:351-389.  The
 * last-ulp accumulation order is restatement only. */
int lq_q4k_matvec_into(float *out, size_t out_len, const float *x, size_t x_len,
                       const uint8_t *w, size_t w_len, size_t rows, size_t cols) {
    if (!kernel_shape_ok(out_len, rows, x_len, cols, w_len, 256, 144)) return 1;
    if (rows == 0 || cols == 0) { for (size_t i = 0; i < out_len; i++) out[i] = 0.0f; return 0; }
    size_t n_blocks = cols / 256;
    float *sum_x = q4k_sum_x(x, n_blocks);
    q4k_rows(out, x, w, sum_x, 0, rows, n_blocks);
    free(sum_x);
    return 0;
}

/* q4k_matvec::dispatch (scalar cross-backend reference):
 * larql-compute/src/cpu/ops/q4k_matvec.rs:72-117 — association
 * (sc*q - mn)*x per element.  Uses the powi-based f16 decode of that file
 * (:22-50), which agrees with lq_f16_to_f32 on every finite input. */
int lq_q4k_matvec_scalar(float *out, const float *x, const uint8_t *w, size_t rows, size_t hidden) {
    size_t superblocks = hidden / 256, bytes_per_row = superblocks * 144;
    for (size_t row = 0; row < rows; row++) {
        float acc = 0.0f;
        for (size_t sb = 0; sb < superblocks; sb++) {
            const uint8_t *block = w + row * bytes_per_row + sb * 144;
            float d = lq_f16_to_f32((uint16_t)(block[0] | (block[1] << 8)));
            float dmin = lq_f16_to_f32((uint16_t)(block[2] | (block[3] << 8)));
            uint8_t scales[8], mins[8];
            q4k_unpack_scales(block + 4, scales, mins);
            const uint8_t *qs = block + 16;
            size_t x_base = sb * 256;
            for (int g = 0; g < 4; g++) {
                int sb_lo = 2 * g, sb_hi = 2 * g + 1;
                float sc_lo = d * (float)scales[sb_lo], sc_hi = d * (float)scales[sb_hi];
                float mn_lo = dmin * (float)mins[sb_lo], mn_hi = dmin * (float)mins[sb_hi];
                for (int l = 0; l < 32; l++) {
                    uint8_t byte = qs[g * 32 + l];
                    float lo = (float)(byte & 0x0F), hi = (float)((byte >> 4) & 0x0F);
                    acc += (sc_lo * lo - mn_lo) * x[x_base + sb_lo * 32 + l];
                    acc += (sc_hi * hi - mn_hi) * x[x_base + sb_hi * 32 + l];
                }
            }
        }
        out[row] = acc;
    }
    return 0;
}

/* q4k_dual_matvec_into: q4_common/dual.rs:22-167 — per-row operation order
 * is that of two q4k_matvec_into calls (the reference's own test,
 * q4_common/neon_tests.rs:75-117). */
int lq_q4k_dual_matvec_into(float *out_a, float *out_b, size_t out_len,
                            const float *x, size_t x_len,
                            const uint8_t *w_a, size_t wa_len,
                            const uint8_t *w_b, size_t wb_len,
                            size_t rows, size_t cols) {
    if (!kernel_shape_ok(out_len, rows, x_len, cols, wa_len, 256, 144)) return 1;
    if (!kernel_shape_ok(out_len, rows, x_len, cols, wb_len, 256, 144)) return 1;
    if (rows == 0 || cols == 0) {
        for (size_t i = 0; i < out_len; i++) { out_a[i] = 0.0f; out_b[i] = 0.0f; }
        return 0;
    }
    size_t n_blocks = cols / 256;
    float *sum_x = q4k_sum_x(x, n_blocks);
    q4k_rows(out_a, x, w_a, sum_x, 0, rows, n_blocks);
    q4k_rows(out_b, x, w_b, sum_x, 0, rows, n_blocks);
    free(sum_x);
    return 0;
}

/* decode_q4k_superblock_into: q4_common/matvec_f32.rs:166-199. */
static void decode_q4k_superblock_into(const uint8_t *w, size_t row_base, size_t sb, float *wf) {
    const uint8_t *block = w + row_base + sb * 144;
    float d = lq_f16_to_f32((uint16_t)(block[0] | (block[1] << 8)));
    float dmin = lq_f16_to_f32((uint16_t)(block[2] | (block[3] << 8)));
    uint8_t scales[8], mins[8];
    q4k_unpack_scales(block + 4, scales, mins);
    const uint8_t *quants = block + 16;
    for (int g = 0; g < 4; g++) {
        int sb_lo = 2 * g, sb_hi = 2 * g + 1;
        float sc_lo = d * (float)scales[sb_lo], sc_hi = d * (float)scales[sb_hi];
        float mn_lo = dmin * (float)mins[sb_lo], mn_hi = dmin * (float)mins[sb_hi];
        const uint8_t *chunk = quants + g * 32;
        for (int i = 0; i < 32; i++) {
            wf[sb_lo * 32 + i] = sc_lo * (float)(chunk[i] & 0x0F) - mn_lo;
            wf[sb_hi * 32 + i] = sc_hi * (float)(chunk[i] >> 4) - mn_hi;
        }
    }
}

/* dot_256_f32_scalar: q4_common/matvec_f32.rs:250-258. */
static float dot_256_f32_scalar(const float *wf, const float *xs) {
    float acc[8] = {0};
    for (int c = 0; c < 32; c++)
        for (int l = 0; l < 8; l++) acc[l] += wf[c * 8 + l] * xs[c * 8 + l];
    float s = 0.0f;
    for (int l = 0; l < 8; l++) s += acc[l];
    return s;
}

/* q4k_matmul_into / kquant_matmul_into: q4_common/matmul.rs:20-139.
 * out is [seq, rows]; shape errors zero the output (:89-98).
 * Pinned: rows equal stacked matvec to 1e-4 and dequant-then-matmul to 5e-3
 * (the reference's tests, quantize_q4_0_tests.rs:155-238). */
void lq_q4k_matmul_into(float *out, const float *x, const uint8_t *w, size_t w_len,
                        size_t rows, size_t hidden, size_t seq) {
    size_t out_len = seq * rows;
    if (rows == 0 || seq == 0 || hidden == 0 || hidden % 256 != 0) {
        for (size_t i = 0; i < out_len; i++) out[i] = 0.0f;
        return;
    }
    size_t n_blocks = hidden / 256, row_bytes = n_blocks * 144;
    if (w_len < rows * row_bytes) {
        for (size_t i = 0; i < out_len; i++) out[i] = 0.0f;
        return;
    }
    float *tmp = (float *)calloc(rows * seq, sizeof(float));
    float wf[256];
    for (size_t r = 0; r < rows; r++) {
        float *out_row = tmp + r * seq;
        for (size_t sb = 0; sb < n_blocks; sb++) {
            decode_q4k_superblock_into(w, r * row_bytes, sb, wf);
            size_t x_off = sb * 256;
            for (size_t s = 0; s < seq; s++) out_row[s] += dot_256_f32_scalar(wf, x + s * hidden + x_off);
        }
    }
    for (size_t r = 0; r < rows; r++)
        for (size_t s = 0; s < seq; s++) out[s * rows + r] = tmp[r * seq + s];
    free(tmp);
}

/* ------------------------------------------------------------------ Q8_0 */

/* ------------------------------------------------------------------------------------------------
 * Q6_K.  Block of 256 values = 210 bytes: ql[128] low nibbles, qh[64] high bit pairs, 16 int8
 * sub-block scales, f16 d.  Value = d * scale[j] * q, q = (lo4 | hi2 << 4) - 32.
 * ---------------------------------------------------------------------------------------------- */

/* quantize_q6_k — larql-compute/src/cpu/ops/q4_common/quantize.rs:197-276 */
int lq_quantize_q6_k(const float *data, size_t n, uint8_t *out) {
    if (n % 256 != 0) return 1;
    size_t nsb = n / 256;
    for (size_t sb = 0; sb < nsb; sb++) {
        const float *block = data + sb * 256;
        uint8_t *o = out + sb * 210;
        float amax = 0.0f;
        for (int i = 0; i < 256; i++) { float a = fabsf(block[i]); amax = fmaxf(amax, a); }
        float d = amax / (31.0f * 127.0f);
        int8_t sub_scales[16];
        for (int j = 0; j < 16; j++) {
            float sub_max = 0.0f;
            for (int i = 0; i < 16; i++) sub_max = fmaxf(sub_max, fabsf(block[j * 16 + i]));
            float sc = d > 0.0f ? sub_max / (31.0f * d) : 0.0f;
            float r = roundf(sc);
            if (r < -128.0f) r = -128.0f;
            if (r > 127.0f) r = 127.0f;
            sub_scales[j] = (int8_t)r;
        }
        uint8_t q6[256];
        for (int j = 0; j < 16; j++) {
            float sc = d * (float)sub_scales[j];
            float inv_sc = fabsf(sc) > 1e-10f ? 1.0f / sc : 0.0f;
            for (int i = 0; i < 16; i++) {
                float r = roundf(block[j * 16 + i] * inv_sc);
                if (r < -32.0f) r = -32.0f;
                if (r > 31.0f) r = 31.0f;
                q6[j * 16 + i] = (uint8_t)((int)r + 32);
            }
        }
        for (int half = 0; half < 2; half++) {
            int e = half * 128;
            for (int l = 0; l < 32; l++) {
                uint8_t q1 = q6[e + l], q2 = q6[e + l + 32], q3 = q6[e + l + 64], q4 = q6[e + l + 96];
                o[half * 64 + l] = (uint8_t)((q1 & 0x0F) | ((q3 & 0x0F) << 4));
                o[half * 64 + l + 32] = (uint8_t)((q2 & 0x0F) | ((q4 & 0x0F) << 4));
                o[128 + half * 32 + l] = (uint8_t)(((q1 >> 4) & 3) | (((q2 >> 4) & 3) << 2) | (((q3 >> 4) & 3) << 4) | (((q4 >> 4) & 3) << 6));
            }
        }
        for (int j = 0; j < 16; j++) o[192 + j] = (uint8_t)sub_scales[j];
        uint16_t db = lq_f32_to_f16_trunc(d);
        o[208] = (uint8_t)(db & 0xFF);
        o[209] = (uint8_t)(db >> 8);
    }
    return 0;
}

/* q6k_subblock_vals — larql-models/src/quant/ggml/q6_k.rs:19-40 */
void lq_q6k_subblock_vals(const uint8_t *block, size_t j, int8_t *out16) {
    const uint8_t *ql = block, *qh = block + 128;
    size_t half = j / 8, g = j % 8, plane = g / 2, lbase = (g % 2) * 16;
    size_t ql_off = half * 64 + (plane & 1) * 32 + lbase, qh_off = half * 32 + lbase;
    unsigned shift = (unsigned)plane * 2;
    for (int i = 0; i < 16; i++) {
        int lo4 = plane < 2 ? (ql[ql_off + i] & 0x0F) : (ql[ql_off + i] >> 4);
        int hi2 = (qh[qh_off + i] >> shift) & 0x03;
        out16[i] = (int8_t)((lo4 | (hi2 << 4)) - 32);
    }
}

/* dequantize_q6_k — q6_k.rs:173-195 */
int lq_dequantize_q6_k(const uint8_t *data, size_t data_len, size_t n, float *out) {
    if (n % 256 != 0) return 1;
    size_t nsb = n / 256;
    if (data_len < nsb * 210) return 1;
    for (size_t sb = 0; sb < nsb; sb++) {
        const uint8_t *block = data + sb * 210;
        float d = lq_f16_to_f32((uint16_t)(block[208] | (block[209] << 8)));
        for (size_t j = 0; j < 16; j++) {
            float sc = d * (float)(int8_t)block[192 + j];
            int8_t vals[16];
            lq_q6k_subblock_vals(block, j, vals);
            for (int i = 0; i < 16; i++) out[sb * 256 + j * 16 + i] = sc * (float)vals[i];
        }
    }
    return 0;
}

/* q6k_matvec::dispatch — larql-compute/src/cpu/ops/q6k_matvec.rs:45-91 (per sub-block: sub = sum v*x; acc += sc*sub) */
int lq_q6k_matvec(const uint8_t *w, size_t w_len, const float *x, size_t rows, size_t hidden, float *out) {
    size_t nsb = hidden / 256, bpr = nsb * 210;
    if (hidden % 256 != 0 || w_len < rows * bpr) return 1;
    for (size_t row = 0; row < rows; row++) {
        float acc = 0.0f;
        for (size_t sb = 0; sb < nsb; sb++) {
            const uint8_t *block = w + row * bpr + sb * 210;
            float d = lq_f16_to_f32((uint16_t)(block[208] | (block[209] << 8)));
            for (size_t j = 0; j < 16; j++) {
                float sc = d * (float)(int8_t)block[192 + j];
                int8_t vals[16];
                lq_q6k_subblock_vals(block, j, vals);
                float sub = 0.0f;
                for (int i = 0; i < 16; i++) sub += (float)vals[i] * x[sb * 256 + j * 16 + i];
                acc += sc * sub;
            }
        }
        out[row] = acc;
    }
    return 0;
}

/* quantize_x_to_q8k — larql-compute/src/cpu/ops/q4k_q8k_dot/q8k_activation.rs:84-109 (and its in-place twin :44-77):
 * per 256-element super-block d = amax/127 (0 for an all-zero block), codes round(x * (1/d)) clamped to +-127
 * (f32::round: half away from zero), sums[8] = the i32 sum of each 32-code sub-block stored as i16.
 * Pinned by the reference's own properties (tests/q8k_quantize_and_matvec.rs:18-50: reconstruction within one
 * step on its ramp input, sums equal the literal sums, zero input clean), closed forms and the numpy restatement;
 * no reference-held vector exists: parity unpinned. */
int lq_quantize_x_to_q8k(const float *x, size_t n, int8_t *qs, float *d, int16_t *sums) {
    if (n % 256 != 0) return 1;
    for (size_t sb = 0; sb < n / 256; sb++) {
        const float *block = x + sb * 256;
        float amax = 0.0f;
        for (int i = 0; i < 256; i++) { float a = fabsf(block[i]); amax = a > amax ? a : amax; }  /* f32::max: a NaN operand is ignored */
        float scale = amax > 0.0f ? amax / 127.0f : 0.0f;
        float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
        d[sb] = scale;
        for (int s = 0; s < 8; s++) {
            int32_t acc = 0;
            for (int j = 0; j < 32; j++) {
                float v = roundf(block[s * 32 + j] * inv);
                v = v < -127.0f ? -127.0f : (v > 127.0f ? 127.0f : v);
                int8_t q = (int8_t)v;  /* `as i8` saturates and maps NaN to 0; after the clamp only NaN differs: (int8_t)NaN is undefined in C */
                if (v != v) q = 0;
                qs[sb * 256 + s * 32 + j] = q;
                acc += q;
            }
            sums[sb * 8 + s] = (int16_t)acc;
        }
    }
    return 0;
}

/* q4k_q8k_matvec_scalar — larql-compute/src/cpu/ops/q4k_q8k_dot/q4k_scalar.rs:15-84, the reference every SIMD
 * kernel of the module is held to bit for bit (NEON, AVX2, the hand assembly; dispatch.rs:15-51):
 * per super-block sum1 = sum_sub sc*dot(q4, q8), sum2 = sum_sub mn*bsum in i32, then
 * acc += d_w*d_y*(f32)sum1 - dmin_w*d_y*(f32)sum2 (left to right, no fused multiply-add), super-blocks in order.
 * Shape rule: KernelShapeError::check (cpu/ops/kernel_shape.rs:47-75): out_len == rows, qs_len == cols,
 * cols % 256 == 0, w_len >= rows*(cols/256)*144; rows == 0 or cols == 0 fill `out` with zeros. */
int lq_q4k_q8k_matvec(float *out, size_t out_len, const int8_t *qs, size_t qs_len, const float *d, const int16_t *sums,
                      const uint8_t *w, size_t w_len, size_t rows, size_t cols) {
    size_t nb = cols / 256, row_bytes = nb * 144;
    if (out_len != rows || qs_len != cols || cols % 256 != 0 || w_len < rows * row_bytes) return 1;
    if (rows == 0 || cols == 0) { for (size_t r = 0; r < out_len; r++) out[r] = 0.0f; return 0; }
    for (size_t r = 0; r < rows; r++) {
        float acc = 0.0f;
        for (size_t sb = 0; sb < nb; sb++) {
            const uint8_t *block = w + r * row_bytes + sb * 144;
            float d_w = lq_f16_to_f32((uint16_t)(block[0] | (block[1] << 8)));
            float dmin_w = lq_f16_to_f32((uint16_t)(block[2] | (block[3] << 8)));
            uint8_t scales[8], mins[8];
            q4k_unpack_scales(block + 4, scales, mins);
            const uint8_t *quants = block + 16;
            const int8_t *y = qs + sb * 256;
            const int16_t *bs = sums + sb * 8;
            float d_y = d[sb];
            int32_t sum1 = 0, sum2 = 0;
            for (int g = 0; g < 4; g++) {
                int32_t dot_lo = 0, dot_hi = 0;
                for (int l = 0; l < 32; l++) {
                    uint8_t byte = quants[g * 32 + l];
                    dot_lo += (int32_t)(byte & 0x0F) * y[(2 * g) * 32 + l];
                    dot_hi += (int32_t)(byte >> 4) * y[(2 * g + 1) * 32 + l];
                }
                sum1 += (int32_t)scales[2 * g] * dot_lo + (int32_t)scales[2 * g + 1] * dot_hi;
                sum2 += (int32_t)mins[2 * g] * bs[2 * g] + (int32_t)mins[2 * g + 1] * bs[2 * g + 1];
            }
            float t1 = d_w * d_y; t1 = t1 * (float)sum1;
            float t2 = dmin_w * d_y; t2 = t2 * (float)sum2;
            acc += t1 - t2;
        }
        out[r] = acc;
    }
    return 0;
}

/* q6k_q8k_matvec_scalar — larql-compute/src/cpu/ops/q4k_q8k_dot/q6k.rs:38-92 (the reference its NEON kernel equals bit
 * for bit): per super-block sum1 = sum over the 16 groups of scale_g * dot(q6 - 32, q8) in i32, acc += d_w*d_y*(f32)sum1,
 * super-blocks in order.  Shape rule: KernelShapeError::check with 210-byte blocks; `out` is zero-filled first.
 * Pinned by the reference's own test inputs and bound (tests/fused_and_q6k_paths.rs:87-110: within 1.2e-1 of the f32
 * Q6_K path, which is itself pinned on the golden Q6_K bytes), a block worked by hand with distinct scales per group,
 * linearity in d_y, and an independently written numpy restatement, bit for bit. */
int lq_q6k_q8k_matvec(float *out, size_t out_len, const int8_t *qs, size_t qs_len, const float *d,
                      const uint8_t *w, size_t w_len, size_t rows, size_t cols) {
    size_t nb = cols / 256, row_bytes = nb * 210;
    if (out_len != rows || qs_len != cols || cols % 256 != 0 || w_len < rows * row_bytes) return 1;
    for (size_t r = 0; r < out_len; r++) out[r] = 0.0f;
    if (rows == 0 || cols == 0) return 0;
    for (size_t r = 0; r < rows; r++) {
        float acc = 0.0f;
        for (size_t sb = 0; sb < nb; sb++) {
            const uint8_t *block = w + r * row_bytes + sb * 210;
            float d_w = lq_f16_to_f32((uint16_t)(block[208] | (block[209] << 8)));
            float d_y = d[sb];
            int32_t sum1 = 0;
            for (size_t g = 0; g < 16; g++) {
                int8_t vals[16];
                lq_q6k_subblock_vals(block, g, vals);
                int32_t dot = 0;
                for (int k = 0; k < 16; k++) dot += (int32_t)vals[k] * qs[sb * 256 + g * 16 + k];
                sum1 += (int32_t)(int8_t)block[192 + g] * dot;
            }
            float t = d_w * d_y;
            acc += t * (float)sum1;
        }
        out[r] = acc;
    }
    return 0;
}

/* larql-models/src/quant/ggml/quantize.rs:50-77.  Codes use the reciprocal
 * of the un-rounded f32 scale.
 * Pinned: byte-for-byte against the reference-held ggml golden blocks
 * (larql-models/src/quant/ggml/tests/q8_0_ggml_golden.rs). */
int lq_quantize_q8_0(const float *data, size_t n, uint8_t *out) {
    if (n % 32 != 0) return 1;
    size_t n_blocks = n / 32;
    for (size_t i = 0; i < n_blocks; i++) {
        const float *block = data + i * 32;
        float amax = 0.0f;
        for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(block[j]));
        float scale = amax / 127.0f;
        float inv_scale = scale > 0.0f ? 1.0f / scale : 0.0f;
        uint16_t sh = lq_f32_to_f16_nearest(scale);
        uint8_t *o = out + i * 34;
        o[0] = (uint8_t)(sh & 0xFF); o[1] = (uint8_t)(sh >> 8);
        for (int j = 0; j < 32; j++)
            o[2 + j] = (uint8_t)sat_i8(clampf(roundf(block[j] * inv_scale), -128.0f, 127.0f));
    }
    return 0;
}

/* larql-models/src/quant/ggml/legacy.rs:68-83.
 * Pinned: bit-exact against ggml_kquant_golden.json case q8_0. */
int lq_dequantize_q8_0(const uint8_t *data, size_t data_len, size_t n, float *out) {
    if (n % 32 != 0) return 1;
    size_t n_blocks = n / 32;
    if (data_len < n_blocks * 34) return 1;
    for (size_t i = 0; i < n_blocks; i++) {
        const uint8_t *block = data + i * 34;
        float scale = lq_f16_to_f32((uint16_t)(block[0] | (block[1] << 8)));
        for (int j = 0; j < 32; j++) out[i * 32 + j] = (float)(int8_t)block[2 + j] * scale;
    }
    return 0;
}

static float q8_0_row_dot(const uint8_t *blocks, const float *x, size_t row, size_t per_row) {
    /* larql-compute/src/cpu/kquant_gemv.rs:92-109 */
    float acc = 0.0f;
    for (size_t b = 0; b < per_row; b++) {
        const uint8_t *base = blocks + (row * per_row + b) * 34;
        float d = lq_f16_to_f32((uint16_t)(base[0] | (base[1] << 8)));
        const float *xs = x + b * 32;
        for (int j = 0; j < 32; j++) acc += ((float)(int8_t)base[2 + j] * d) * xs[j];
    }
    return acc;
}

/* q8_0_gemv: larql-compute/src/cpu/kquant_gemv.rs:67-90.  Exact length.
 * Pinned: bit-for-bit equal to dequantize-then-multiply in element order
 * (the reference's own assert_eq!, kquant_gemv_tests.rs:92-105), on the
 * golden q8_0 bytes and on seeded bytes; refusals of :133-151. */
int lq_q8_0_gemv(const uint8_t *blocks, size_t blocks_len, const float *x, size_t x_len,
                 size_t n, size_t k, float *out) {
    if (k == 0 || k % 32 != 0 || x_len != k) return 1;
    size_t per_row = k / 32;
    if (blocks_len != n * per_row * 34) return 1;
    for (size_t r = 0; r < n; r++) out[r] = q8_0_row_dot(blocks, x, r, per_row);
    return 0;
}

/* ------------------------------------------------------------ Q4_0 x Q8 */

/* quantize_to_q8: q4_common/quantize.rs:6-22. */
void lq_quantize_to_q8(const float *x, size_t n, int8_t *q8, float *scales) {
    size_t n_blocks = n / 32;
    for (size_t i = 0; i < n; i++) q8[i] = 0;
    for (size_t b = 0; b < n_blocks; b++) {
        const float *block = x + b * 32;
        float amax = 0.0f;
        for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(block[j]));
        float scale = amax / 127.0f;
        scales[b] = scale;
        float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
        for (int j = 0; j < 32; j++)
            q8[b * 32 + j] = sat_i8(clampf(roundf(block[j] * inv), -128.0f, 127.0f));
    }
}

/* quantize_q4_0: q4_common/quantize.rs:28-69 (planar nibbles). */
int lq_quantize_q4_0(const float *data, size_t n, uint8_t *out) {
    if (n % 32 != 0) return 1;
    size_t n_blocks = n / 32;
    for (size_t i = 0; i < n_blocks; i++) {
        const float *block = data + i * 32;
        float amax = 0.0f;
        for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(block[j]));
        float scale = amax / 7.0f;
        float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
        uint16_t h = lq_f32_to_f16_flush(scale);
        uint8_t *o = out + i * 18;
        o[0] = (uint8_t)(h & 0xFF); o[1] = (uint8_t)(h >> 8);
        for (int j = 0; j < 16; j++) {
            int32_t lo = sat_i32(roundf(block[j] * inv)) + 8;
            int32_t hi = sat_i32(roundf(block[j + 16] * inv)) + 8;
            lo = lo < 0 ? 0 : (lo > 15 ? 15 : lo);
            hi = hi < 0 ? 0 : (hi > 15 ? 15 : hi);
            o[2 + j] = (uint8_t)(lo | (hi << 4));
        }
    }
    return 0;
}

/* q4_0_matvec_c, scalar arm: larql-compute/csrc/q4_dot.c:176-207.
 * Pinned: bit-for-bit against that C file compiled from the reference tree
 * (oracle/_ref/libq4dot_ref.so) wherever it builds. */
void lq_q4_0_matvec(const uint8_t *q4, const int8_t *q8_x, const float *q8_scales,
                    float *scores, size_t num_rows, size_t hidden) {
    size_t blocks_per_row = hidden / 32, bytes_per_row = blocks_per_row * 18;
    for (size_t row = 0; row < num_rows; row++) {
        float acc = 0.0f;
        const uint8_t *row_data = q4 + row * bytes_per_row;
        for (size_t b = 0; b < blocks_per_row; b++) {
            const uint8_t *block = row_data + b * 18;
            float combined = lq_f16_to_f32((uint16_t)(block[0] | (block[1] << 8))) * q8_scales[b];
            const int8_t *q8p = q8_x + b * 32;
            for (int j = 0; j < 16; j++) {
                uint8_t byte = block[2 + j];
                int lo_v = (byte & 0x0F) - 8, hi_v = ((byte >> 4) & 0x0F) - 8;
                acc += (float)lo_v * (float)q8p[j] * combined;
                acc += (float)hi_v * (float)q8p[j + 16] * combined;
            }
        }
        scores[row] = acc;
    }
}

/* dequantise_q8: larql-compute/src/backend/quant_matvec.rs:24-40. */
void lq_dequantise_q8(const int8_t *q8_x, size_t n, const float *scales, float *out) {
    size_t n_blocks = n / 32;
    for (size_t b = 0; b < n_blocks; b++)
        for (int j = 0; j < 32; j++) out[b * 32 + j] = (float)q8_x[b * 32 + j] * scales[b];
    for (size_t i = n_blocks * 32; i < n; i++) out[i] = (float)q8_x[i];
}

/* ----------------------------------------------------------------- MXFP4 */

static const float MXFP4_TABLE[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                      -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
float lq_mxfp4_table(unsigned code) { return MXFP4_TABLE[code & 15]; }

/* larql-models/src/quant/mxfp4.rs:26-35.  Pinned: KATs of mxfp4.rs:276-297. */
float lq_e8m0_to_f32(uint8_t byte) {
    if (byte == 0) return 0.0f;
    if (byte == 255) return NAN;
    return u2f(((uint32_t)byte) << 23);
}

/* larql-vindex/src/format/vindex3/opplan/exec/weights/quantize.rs:71-88. */
uint8_t lq_nearest_mxfp4_code(float v) {
    uint8_t sign = (f2u(v) >> 31) ? 8 : 0;
    float mag = fminf(fabsf(v), 6.0f);
    uint8_t best = 0;
    float best_err = INFINITY;
    for (unsigned code = 0; code < 8; code++) {
        float err = fabsf(mag - MXFP4_TABLE[code]);
        if (err < best_err || (err == best_err && code % 2 == 0)) { best = (uint8_t)code; best_err = err; }
    }
    return best == 0 ? 0 : (uint8_t)(sign | best);
}

/* quantize_mxfp4: .../opplan/exec/weights/load.rs:410-476.  The shared
 * exponent is floor(log2f(max|x|)) - 2 computed in f32 with libm, as Rust's
 * f32::log2 does.
 * Pinned: restatement + KATs (powers of two, ties, saturation, all-zero
 * group) + round trip through the decoder; no reference-held bytes. */
int lq_quantize_mxfp4(const float *values, size_t rows, size_t k, uint8_t *packed, uint8_t *scales) {
    if (k % 32 != 0) return 1;
    size_t groups = k / 32;
    for (size_t r = 0; r < rows; r++) {
        for (size_t g = 0; g < groups; g++) {
            const float *group = values + r * k + g * 32;
            float max_abs = 0.0f;
            for (int i = 0; i < 32; i++) max_abs = fmaxf(max_abs, fabsf(group[i]));
            uint8_t scale_byte;
            if (max_abs == 0.0f) scale_byte = 0;
            else {
                int32_t exponent = sat_i32(floorf(log2f(max_abs))) - 2;
                int32_t e = exponent + 127;
                e = e < 1 ? 1 : (e > 254 ? 254 : e);
                scale_byte = (uint8_t)e;
            }
            scales[r * groups + g] = scale_byte;
            float scale = lq_e8m0_to_f32(scale_byte);
            float inv = scale == 0.0f ? 0.0f : 1.0f / scale;
            uint8_t *bytes = packed + (r * groups + g) * 16;
            for (int b = 0; b < 16; b++) {
                uint8_t lo = lq_nearest_mxfp4_code(group[2 * b] * inv);
                uint8_t hi = lq_nearest_mxfp4_code(group[2 * b + 1] * inv);
                bytes[b] = (uint8_t)(lo | (hi << 4));
            }
        }
    }
    return 0;
}

/* dequantize_expert: larql-models/src/quant/mxfp4.rs:42-95.
 * Pinned: KATs of mxfp4.rs:312-380. */
int lq_dequantize_mxfp4_expert(const uint8_t *blocks, size_t blocks_len,
                               const uint8_t *scales, size_t scales_len,
                               size_t out_features, size_t groups, float *out) {
    if (blocks_len < out_features * groups * 16) return 1;
    if (scales_len < out_features * groups) return 1;
    size_t in_features = groups * 32;
    for (size_t row = 0; row < out_features; row++)
        for (size_t g = 0; g < groups; g++) {
            float scale = lq_e8m0_to_f32(scales[row * groups + g]);
            const uint8_t *blk = blocks + (row * groups + g) * 16;
            for (int b = 0; b < 16; b++) {
                size_t o = row * in_features + g * 32 + (size_t)b * 2;
                out[o] = MXFP4_TABLE[blk[b] & 0x0F] * scale;
                out[o + 1] = MXFP4_TABLE[(blk[b] >> 4) & 0x0F] * scale;
            }
        }
    return 0;
}

/* The CPU stand-in of MatMul::mxfp4_gemv: LoopDevice::mxfp4_gemv / mxfp4_loop,
 * larql-vindex/src/format/vindex3/opplan/exec/tests/device.rs:87-127, with
 * the validation of larql-compute/src/backend/matmul.rs:226-235 as the Metal
 * peer applies it. */
int lq_mxfp4_gemv(const uint8_t *packed, size_t packed_len, const uint8_t *scales, size_t scales_len,
                  const float *x, size_t x_len, size_t n, size_t k, float *out) {
    if (k % 32 != 0 || x_len < k) return 1;
    if (packed_len < n * (k / 32) * 16 || scales_len < n * (k / 32)) return 1;
    size_t groups = k / 32;
    for (size_t row = 0; row < n; row++) {
        float acc = 0.0f;
        for (size_t g = 0; g < groups; g++) {
            float scale = lq_e8m0_to_f32(scales[row * groups + g]);
            const uint8_t *bytes = packed + (row * groups + g) * 16;
            for (int b = 0; b < 16; b++) {
                size_t e0 = g * 32 + 2 * (size_t)b;
                acc += MXFP4_TABLE[bytes[b] & 0x0F] * scale * x[e0];
                acc += MXFP4_TABLE[bytes[b] >> 4] * scale * x[e0 + 1];
            }
        }
        out[row] = acc;
    }
    return 0;
}

/* dequantize_expert + row dot: the reference the Metal peer's tests use,
 * larql-compute-metal/src/trait_impl/mxfp4.rs:201-206. */
int lq_mxfp4_gemv_dequant(const uint8_t *packed, const uint8_t *scales, const float *x,
                          size_t n, size_t k, float *out) {
    size_t groups = k / 32;
    float *w = (float *)malloc(n * k * sizeof(float));
    lq_dequantize_mxfp4_expert(packed, n * groups * 16, scales, n * groups, n, groups, w);
    for (size_t r = 0; r < n; r++) {
        float acc = 0.0f;
        for (size_t c = 0; c < k; c++) acc += w[r * k + c] * x[c];
        out[r] = acc;
    }
    free(w);
    return 0;
}

/* ----------------------------------------------------------- dense gemv */

/* bf16_dot_portable per row:
 * larql-vindex/src/format/vindex3/opplan/exec/cpu/kernels.rs:718-723. */
void lq_bf16_gemv(const uint16_t *w, const float *x, size_t n, size_t k, float *out) {
    for (size_t r = 0; r < n; r++) {
        float acc = 0.0f;
        for (size_t c = 0; c < k; c++) acc += lq_bf16_to_f32(w[r * k + c]) * x[c];
        out[r] = acc;
    }
}
/* f16 gates are widened then multiplied (gate_store.rs:353-444 decode cache). */
void lq_f16_gemv(const uint16_t *w, const float *x, size_t n, size_t k, float *out) {
    for (size_t r = 0; r < n; r++) {
        float acc = 0.0f;
        for (size_t c = 0; c < k; c++) acc += lq_f16_to_f32(w[r * k + c]) * x[c];
        out[r] = acc;
    }
}
/* gemv: larql-vindex/src/index/storage/gate_store.rs:119-143.  The reference
 * calls cblas_sgemv of whatever OpenBLAS the host has (ndarray 0.16.1 /
 * openblas-src 0.10.15, system library, unpinned): its summation order is not
 * fixed, so this sequential row dot is parity "within fp32 reordering". */
void lq_f32_gemv(const float *w, const float *x, size_t n, size_t k, float *out) {
    for (size_t r = 0; r < n; r++) {
        float acc = 0.0f;
        for (size_t c = 0; c < k; c++) acc += w[r * k + c] * x[c];
        out[r] = acc;
    }
}

/* ---------------------------------------------------------------- top-K */

/* top_k_by_abs: larql-vindex/src/index/compute/gate_knn/mod.rs:50-108.
 * The min-heap is Rust's std BinaryHeap (push = sift_up, pop = swap the last
 * element to the root, sift_down_to_bottom, sift_up), restated so that the
 * eviction among equal |values| follows the same heap order.  The final
 * sort_unstable leaves the order of equal |values| unspecified; a stable
 * sort over the heap's vector order is used here.
 * Pinned: the closed-form cases of gate_knn/mod.rs:231-287 and brute-force
 * full sort on tie-free data; tie eviction is restatement only. */
typedef struct { uint64_t idx; float val; } abs_score;

/* heap order: a <= b  <=>  not (|a| < |b|)   (Ord reversed on |val|) */
static inline int heap_le(const abs_score *a, const abs_score *b) {
    return !(fabsf(a->val) < fabsf(b->val));
}
static size_t heap_sift_up(abs_score *d, size_t start, size_t pos) {
    abs_score elt = d[pos];
    while (pos > start) {
        size_t parent = (pos - 1) / 2;
        if (heap_le(&elt, &d[parent])) break;
        d[pos] = d[parent];
        pos = parent;
    }
    d[pos] = elt;
    return pos;
}
static void heap_sift_down_to_bottom(abs_score *d, size_t len, size_t pos) {
    size_t end = len, start = pos;
    abs_score elt = d[pos];
    size_t child = 2 * pos + 1;
    size_t lim = end >= 2 ? end - 2 : 0;
    while (child <= lim && end >= 2) {
        child += heap_le(&d[child], &d[child + 1]) ? 1 : 0;
        d[pos] = d[child];
        pos = child;
        child = 2 * pos + 1;
    }
    if (child == end - 1) { d[pos] = d[child]; pos = child; }
    d[pos] = elt;
    heap_sift_up(d, start, pos);
}

long lq_top_k_by_abs(const float *scores, size_t n, size_t top_k, uint64_t *idx_out, float *val_out) {
    if (top_k == 0) return 0;
    for (size_t i = 0; i < n; i++) if (scores[i] != scores[i]) return -1; /* partial_cmp().unwrap() panics */
    size_t cap = top_k < n ? top_k : n;
    abs_score *heap = (abs_score *)malloc((cap ? cap : 1) * sizeof(abs_score));
    size_t len = 0;
    for (size_t i = 0; i < n; i++) {
        float v = scores[i];
        if (len < top_k) {
            heap[len].idx = i; heap[len].val = v; len++;
            heap_sift_up(heap, 0, len - 1);
        } else if (fabsf(v) > fabsf(heap[0].val)) {
            /* pop */
            abs_score item = heap[len - 1];
            len--;
            if (len > 0) {
                abs_score t = heap[0]; heap[0] = item; item = t;
                heap_sift_down_to_bottom(heap, len, 0);
            }
            /* push */
            heap[len].idx = i; heap[len].val = v; len++;
            heap_sift_up(heap, 0, len - 1);
        }
    }
    /* stable insertion sort, |val| descending */
    for (size_t i = 1; i < len; i++) {
        abs_score e = heap[i];
        size_t j = i;
        while (j > 0 && fabsf(heap[j - 1].val) < fabsf(e.val)) { heap[j] = heap[j - 1]; j--; }
        heap[j] = e;
    }
    for (size_t i = 0; i < len; i++) { idx_out[i] = heap[i].idx; val_out[i] = heap[i].val; }
    free(heap);
    return (long)len;
}

/* top_k_sorted: larql-vindex/src/index/storage/lm_head/knn.rs:315-386 —
 * by value descending, non-finite scores skipped. */
typedef struct { float s; uint32_t i; } val_score;
static void vs_sift_down(val_score *h, size_t n, size_t i) {
    for (;;) {
        size_t smallest = i, l = 2 * i + 1, r = 2 * i + 2;
        if (l < n && h[l].s < h[smallest].s) smallest = l;
        if (r < n && h[r].s < h[smallest].s) smallest = r;
        if (smallest == i) break;
        val_score t = h[i]; h[i] = h[smallest]; h[smallest] = t;
        i = smallest;
    }
}
long lq_top_k_sorted(const float *scores, size_t n, size_t top_k, uint32_t *idx_out, float *val_out) {
    if (n == 0 || top_k == 0) return 0;
    size_t k = top_k < n ? top_k : n;
    if (k == 1) {
        uint32_t best_i = 0; float best_v = -INFINITY;
        for (size_t i = 0; i < n; i++) if (isfinite(scores[i]) && scores[i] > best_v) { best_v = scores[i]; best_i = (uint32_t)i; }
        if (best_v == -INFINITY) return 0;
        idx_out[0] = best_i; val_out[0] = best_v;
        return 1;
    }
    val_score *heap = (val_score *)malloc((k + 1) * sizeof(val_score));
    size_t len = 0;
    for (size_t i = 0; i < n; i++) {
        float s = scores[i];
        if (!isfinite(s)) continue;
        if (len < k) {
            heap[len].s = s; heap[len].i = (uint32_t)i; len++;
            if (len == k) for (size_t j = k / 2; j-- > 0;) vs_sift_down(heap, len, j);
        } else if (s > heap[0].s) {
            heap[0].s = s; heap[0].i = (uint32_t)i;
            vs_sift_down(heap, len, 0);
        }
    }
    /* (the reference re-heapifies a short heap here; the sort below makes it moot) */
    for (size_t i = 1; i < len; i++) {
        val_score e = heap[i];
        size_t j = i;
        while (j > 0 && heap[j - 1].s < e.s) { heap[j] = heap[j - 1]; j--; }
        heap[j] = e;
    }
    for (size_t i = 0; i < len; i++) { idx_out[i] = heap[i].i; val_out[i] = heap[i].s; }
    free(heap);
    return (long)len;
}

static int cmp_u64(const void *a, const void *b) {
    uint64_t x = *(const uint64_t *)a, y = *(const uint64_t *)b;
    return x < y ? -1 : (x > y ? 1 : 0);
}

/* gate_knn_batch: larql-vindex/src/index/compute/gate_knn/dispatch.rs:256-304
 * — per-position top_k_by_abs over column s of scores_2d [n_features, seq],
 * then the sorted, de-duplicated union of the indices. */
long lq_gate_knn_batch_union(const float *scores_2d, size_t n_features, size_t seq, size_t top_k,
                             uint64_t *idx_out, size_t idx_cap) {
    if (seq == 0) return 0;
    size_t k = top_k < n_features ? top_k : n_features;
    if (k == 0) return 0;
    float *col = (float *)malloc(n_features * sizeof(float));
    uint64_t *all = (uint64_t *)malloc(seq * k * sizeof(uint64_t));
    float *vals = (float *)malloc(k * sizeof(float));
    size_t total = 0;
    for (size_t s = 0; s < seq; s++) {
        for (size_t f = 0; f < n_features; f++) col[f] = scores_2d[f * seq + s];
        long got = lq_top_k_by_abs(col, n_features, k, all + total, vals);
        if (got < 0) { free(col); free(all); free(vals); return -1; }
        total += (size_t)got;
    }
    qsort(all, total, sizeof(uint64_t), cmp_u64);
    size_t m = 0;
    for (size_t i = 0; i < total; i++) if (i == 0 || all[i] != all[i - 1]) { if (m < idx_cap) idx_out[m] = all[i]; m++; }
    free(col); free(all); free(vals);
    return (long)m;
}

/* ---------------------------------------------------------- MoE routing */

/* router::select: larql-compute/src/ffn/expert_weight/router.rs:33-70.
 * Stable sort by logit descending (first index wins ties), softmax with the
 * global max shift over all experts or over the selected ones.
 * Pinned: KATs of router.rs:79-200 (sums to 1, matches a full softmax, ties
 * go to the first index). */
size_t lq_router_select(const float *logits, size_t n, size_t k, int policy,
                        uint64_t *experts, float *weights) {
    if (k > n) k = n;
    if (k == 0) return 0;
    uint64_t *ri = (uint64_t *)malloc(n * sizeof(uint64_t));
    float *rv = (float *)malloc(n * sizeof(float));
    for (size_t i = 0; i < n; i++) { ri[i] = i; rv[i] = logits[i]; }
    for (size_t i = 1; i < n; i++) { /* stable, descending */
        uint64_t ei = ri[i]; float ev = rv[i];
        size_t j = i;
        while (j > 0 && ev > rv[j - 1]) { ri[j] = ri[j - 1]; rv[j] = rv[j - 1]; j--; }
        ri[j] = ei; rv[j] = ev;
    }
    float dmax = -INFINITY;
    for (size_t i = 0; i < n; i++) dmax = fmaxf(dmax, logits[i]);
    float denom = 0.0f;
    if (policy == LQ_ROUTE_SOFTMAX_THEN_SELECT) for (size_t i = 0; i < n; i++) denom += expf(logits[i] - dmax);
    else for (size_t i = 0; i < k; i++) denom += expf(rv[i] - dmax);
    for (size_t i = 0; i < k; i++) {
        experts[i] = ri[i];
        weights[i] = denom > 0.0f ? expf(rv[i] - dmax) / denom : 0.0f;
    }
    free(ri); free(rv);
    return k;
}

/* math::top_k: larql-compute/src/cpu/ops/moe/math.rs:152-164 — value
 * descending, index ascending. */
size_t lq_moe_top_k(const float *v, size_t n, size_t k, uint64_t *idx, float *val) {
    if (k > n) k = n;
    uint64_t *ri = (uint64_t *)malloc((n ? n : 1) * sizeof(uint64_t));
    for (size_t i = 0; i < n; i++) ri[i] = i;
    for (size_t i = 1; i < n; i++) {
        uint64_t e = ri[i];
        size_t j = i;
        while (j > 0 && (v[e] > v[ri[j - 1]])) { ri[j] = ri[j - 1]; j--; }
        ri[j] = e;
    }
    for (size_t i = 0; i < k; i++) { idx[i] = ri[i]; val[i] = v[ri[i]]; }
    free(ri);
    return k;
}

/* math::softmax: moe/math.rs:130-142. */
void lq_softmax(float *v, size_t n) {
    float max = -INFINITY;
    for (size_t i = 0; i < n; i++) max = fmaxf(max, v[i]);
    float sum = 0.0f;
    for (size_t i = 0; i < n; i++) { v[i] = expf(v[i] - max); sum += v[i]; }
    if (sum > 0.0f) for (size_t i = 0; i < n; i++) v[i] /= sum;
}

/* moe_router_logits: larql-compute/src/cpu/ops/moe/mod.rs:127-147 — logits[e] = router_in . router_proj[e] + bias[e]
 * (the bias joins before softmax / selection).  The reference's matmul_vec goes through BLAS, whose summation order
 * is not fixed; a sequential f32 dot stands in for it. */
void lq_moe_router_logits(const float *router_in, const float *router_proj, const float *router_bias, size_t n_experts,
                          size_t hidden, float *logits) {
    for (size_t e = 0; e < n_experts; e++) {
        float acc = 0.0f;
        for (size_t c = 0; c < hidden; c++) acc += router_in[c] * router_proj[e * hidden + c];
        logits[e] = router_bias ? acc + router_bias[e] : acc;
    }
}

/* moe_route_from_router_input: cpu/ops/moe/mod.rs:149-186 — the served tier's route: softmax over ALL logits, top_k
 * of the probabilities (value descending, index ascending), divided by their sum under
 * MoeTopKWeightPolicy::RenormalizedSoftmax (only when the sum is positive), then multiplied by
 * router_per_expert_scale[expert] under MoeExpertScalePolicy::PerExpert (per_expert_scale != NULL here). */
size_t lq_moe_route_from_router_input(const float *router_in, size_t hidden, const float *router_proj, const float *router_bias,
                                      size_t n_experts, size_t top_k, int renormalize, const float *per_expert_scale,
                                      size_t n_scale, uint64_t *experts, float *weights) {
    float *logits = (float *)malloc((n_experts ? n_experts : 1) * sizeof(float));
    lq_moe_router_logits(router_in, router_proj, router_bias, n_experts, hidden, logits);
    lq_softmax(logits, n_experts);
    size_t k = lq_moe_top_k(logits, n_experts, top_k, experts, weights);
    if (renormalize) {
        float sum = 0.0f;
        for (size_t i = 0; i < k; i++) sum += weights[i];
        if (sum > 0.0f) for (size_t i = 0; i < k; i++) weights[i] /= sum;
    }
    if (per_expert_scale && n_scale)
        for (size_t i = 0; i < k; i++)
            if (experts[i] < n_scale) weights[i] *= per_expert_scale[experts[i]];
    free(logits);
    return k;
}

/* MoeGateRule::ClampedGlu: larql-compute/src/pipeline/moe.rs:88-92. */
float lq_clamped_glu(float g, float u, float limit, float alpha) {
    g = fminf(g, limit);
    u = clampf(u, -limit, limit);
    float sig = 1.0f / (1.0f + expf(-(g * alpha)));
    return (u + 1.0f) * (g * sig);
}

/* ------------------------------------------------------ MoE expert block */

/* One weight row against x.  f32 banks: `w` is [rows, k] f32 (dot_proj =
 * x . w^T, larql-compute/src/forward/ops.rs:43-48; the reference's BLAS sums
 * in an order it does not fix, a sequential f32 dot stands in for it).
 * MXFP4 banks: the row loop of lq_mxfp4_gemv above. */
typedef struct {
    int mxfp4;
    const float *w_f32;
    const uint8_t *packed, *scales;
} moe_matrix;

static float moe_row_dot(const moe_matrix *m, size_t row, size_t k, const float *x) {
    float acc = 0.0f;
    if (!m->mxfp4) {
        const float *w = m->w_f32 + row * k;
        for (size_t c = 0; c < k; c++) acc += w[c] * x[c];
        return acc;
    }
    size_t groups = k / 32;
    for (size_t g = 0; g < groups; g++) {
        float scale = lq_e8m0_to_f32(m->scales[row * groups + g]);
        const uint8_t *bytes = m->packed + (row * groups + g) * 16;
        for (int b = 0; b < 16; b++) {
            size_t e0 = g * 32 + 2 * (size_t)b;
            acc += MXFP4_TABLE[bytes[b] & 0x0F] * scale * x[e0];
            acc += MXFP4_TABLE[bytes[b] >> 4] * scale * x[e0 + 1];
        }
    }
    return acc;
}

/* The expert block for one token, given its routing — the composition both
 * tiers of the reference share:
 *   ExpertWeightFfn::run_expert_observed + moe_block's weighted accumulation,
 *     larql-compute/src/ffn/expert_weight/mod.rs:150-262 (f32 experts);
 *   cpu_moe_forward's add_expert, cpu/ops/moe/forward.rs:201-270, and the Metal
 *     combine h + sum_s w_s*(dot_s + bias_s),
 *     larql-compute-metal/src/shaders/mxfp4_grouped_experts/kernels.rs:482-541.
 * act[j] = rule.combine(gate.x + gate_bias[j], up.x + up_bias[j]); the fused bias
 * row is interleaved (gate bias j at 2j, up bias j at 2j+1: ExpertMlp::gate_bias /
 * up_bias, pipeline/moe.rs:150-166, FusedHalf::fused_row) whatever the weight
 * layout; contribution = down.act + down_bias; out += w * contribution in
 * selection order.  An expert id outside the bank is skipped (forward.rs:203-208).
 * gate/up/down describe expert 0; expert e lies e*stride further on.
 * `interleaved`: gate row j is fused row 2j and up row j is fused row 2j+1 of
 * the gate matrix ([2*inter, hidden] per expert); `up` is not read. */
static void moe_token(const float *x, size_t hidden, size_t inter, size_t n_experts, size_t top_k, const uint64_t *experts,
                      const float *weights, const moe_matrix *gate, const moe_matrix *up, const moe_matrix *down,
                      int interleaved, const float *gate_up_bias, const float *down_bias, float limit, float alpha,
                      float *act, float *out) {
    for (size_t c = 0; c < hidden; c++) out[c] = 0.0f;
    for (size_t s = 0; s < top_k; s++) {
        size_t e = (size_t)experts[s];
        float w = weights[s];
        if (e >= n_experts) continue;
        size_t gu_rows = interleaved ? 2 * inter : inter;
        moe_matrix g = *gate, u = interleaved ? *gate : *up, d = *down;
        if (g.mxfp4) {
            g.packed += e * gu_rows * (hidden / 32) * 16; g.scales += e * gu_rows * (hidden / 32);
            u.packed += e * gu_rows * (hidden / 32) * 16; u.scales += e * gu_rows * (hidden / 32);
            d.packed += e * hidden * (inter / 32) * 16; d.scales += e * hidden * (inter / 32);
        } else {
            g.w_f32 += e * gu_rows * hidden; u.w_f32 += e * gu_rows * hidden; d.w_f32 += e * hidden * inter;
        }
        for (size_t j = 0; j < inter; j++) {
            size_t gr = interleaved ? 2 * j : j, ur = interleaved ? 2 * j + 1 : j;
            float gv = moe_row_dot(&g, gr, hidden, x), uv = moe_row_dot(&u, ur, hidden, x);
            if (gate_up_bias) { gv += gate_up_bias[e * 2 * inter + 2 * j]; uv += gate_up_bias[e * 2 * inter + 2 * j + 1]; }
            act[j] = lq_clamped_glu(gv, uv, limit, alpha);
        }
        for (size_t c = 0; c < hidden; c++) {
            float v = moe_row_dot(&d, c, inter, act);
            if (down_bias) v += down_bias[e * hidden + c];
            out[c] += w * v;
        }
    }
}

/* ExpertWeightFfn::moe_block for a GPT-OSS-shaped f32 layer —
 * larql-compute/src/ffn/expert_weight/mod.rs:100-262: router logits = x . W_r^T
 * + b_r, router::select per token, then the block above.  `fused` is
 * [n_experts, 2*inter, hidden] as a checkpoint ships it (gate = even rows,
 * up = odd rows: deinterleave_fused_half, larql-models/src/quant/mxfp4.rs:218-231).
 * The reference groups tokens per expert and so adds a token's contributions in
 * expert-index order; here they are added in selection order, as the served tier
 * does (forward.rs) — the two differ by fp32 reordering only.
 * Pinned: EXPECTED[48] of larql-compute/tests/test_moe_reference_parity.rs:72-85
 * (values of an independent transcription of the GPT-OSS reference model). */
int lq_moe_block_f32(const float *x, size_t tokens, size_t hidden, size_t inter, size_t n_experts, size_t top_k, int policy,
                     const float *router_w, const float *router_b, const float *fused, const float *down,
                     const float *gate_up_bias, const float *down_bias, float limit, float alpha, float *out) {
    if (n_experts == 0 || top_k == 0) { for (size_t i = 0; i < tokens * hidden; i++) out[i] = 0.0f; return 0; }
    float *logits = (float *)malloc(n_experts * sizeof(float));
    float *act = (float *)malloc((inter ? inter : 1) * sizeof(float));
    uint64_t *ex = (uint64_t *)malloc(top_k * sizeof(uint64_t));
    float *wt = (float *)malloc(top_k * sizeof(float));
    moe_matrix g = {0, fused, NULL, NULL}, d = {0, down, NULL, NULL};
    for (size_t t = 0; t < tokens; t++) {
        const float *xt = x + t * hidden;
        for (size_t e = 0; e < n_experts; e++) {
            float acc = 0.0f;
            for (size_t c = 0; c < hidden; c++) acc += xt[c] * router_w[e * hidden + c];
            logits[e] = router_b ? acc + router_b[e] : acc;
        }
        size_t k = lq_router_select(logits, n_experts, top_k, policy, ex, wt);
        moe_token(xt, hidden, inter, n_experts, k, ex, wt, &g, &g, &d, 1, gate_up_bias, down_bias, limit, alpha, act,
                  out + t * hidden);
    }
    free(logits); free(act); free(ex); free(wt);
    return 0;
}

/* The same block over an MXFP4 bank with the routing given (experts / weights
 * [tokens, top_k], as router::select returns them): the CPU tier refuses MXFP4
 * banks (forward.rs:69-75), the Metal peer serves them with this composition. */
int lq_moe_block_mxfp4(const float *x, size_t tokens, size_t hidden, size_t inter, size_t n_experts, size_t top_k,
                       const uint64_t *experts, const float *weights, const uint8_t *gate_packed, const uint8_t *gate_scales,
                       const uint8_t *up_packed, const uint8_t *up_scales, const uint8_t *down_packed, const uint8_t *down_scales,
                       int interleaved, const float *gate_up_bias, const float *down_bias, float limit, float alpha, float *out) {
    if (hidden % 32 != 0 || inter % 32 != 0) return 1;
    float *act = (float *)malloc((inter ? inter : 1) * sizeof(float));
    moe_matrix g = {1, NULL, gate_packed, gate_scales}, u = {1, NULL, up_packed, up_scales}, d = {1, NULL, down_packed, down_scales};
    for (size_t t = 0; t < tokens; t++)
        moe_token(x + t * hidden, hidden, inter, n_experts, top_k, experts + t * top_k, weights + t * top_k, &g, &u, &d, interleaved,
                  gate_up_bias, down_bias, limit, alpha, act, out + t * hidden);
    free(act);
    return 0;
}

/* math::silu / math::gelu_tanh — larql-compute/src/cpu/ops/moe/math.rs:54-65. */
float lq_silu(float x) { return x / (1.0f + expf(-x)); }
float lq_gelu_tanh(float x) {
    const float c = 0.7978846f;
    return 0.5f * x * (1.0f + tanhf(c * (x + 0.044715f * x * x * x)));
}
/* MoeGateRule::combine — larql-compute/src/pipeline/moe.rs:73-118, the rules a k-quant bank is served under:
 * 0 ClampedGlu{limit, alpha}, 1 Gated(gelu_tanh), 2 Gated(silu), 3 SituGlu{beta, linear_beta}, 4 / 5 ClampedGated{limit,
 * gelu_tanh / silu}.  Inputs already carry their biases. */
float lq_moe_combine(int rule, float g, float u, float limit, float alpha) {
    if (rule == LQ_GATE_GELU_TANH) return lq_gelu_tanh(g) * u;
    if (rule == LQ_GATE_SILU) return lq_silu(g) * u;
    if (rule == LQ_GATE_SITU_GLU) {  /* SituGlu{beta = limit, linear_beta = alpha, 0 for None}: moe.rs:100-107 */
        const float situ_a = limit * tanhf(g / limit) * (1.0f / (1.0f + expf(-g)));
        if (alpha != 0.0f) u = alpha * tanhf(u / alpha);
        return situ_a * u;
    }
    if (rule == LQ_GATE_CLAMPED_GELU_TANH || rule == LQ_GATE_CLAMPED_SILU) {  /* ClampedGated{limit, activation}: moe.rs:108-117 */
        g = fminf(g, limit);
        u = clampf(u, -limit, limit);
        return (rule == LQ_GATE_CLAMPED_GELU_TANH ? lq_gelu_tanh(g) : lq_silu(g)) * u;
    }
    return lq_clamped_glu(g, u, limit, alpha);
}

/* cpu_moe_forward's f32 arm (cpu/ops/moe/forward.rs:246-290) over a float bank — format 16 = BF16 (the legacy monolith),
 * 17 = F16, 32 = F32: the slab is dequantised to f32 and met by matmul_vec (BLAS sgemv there; a sequential f32 dot here,
 * as in lq_moe_block_f32), gate and up the two halves of [2*inter, cols], down [hidden, inter] unpadded (a float format has
 * no block to pad to: MoeWeightLayout::down_cols, pipeline/moe.rs:184-200); biases, rule and weighting as below. */
static void float_gemv(int format, const uint8_t *w, const float *x, size_t n, size_t k, float *out) {
    if (format == 16) lq_bf16_gemv((const uint16_t *)w, x, n, k, out);
    else if (format == 17) lq_f16_gemv((const uint16_t *)w, x, n, k, out);
    else lq_f32_gemv((const float *)w, x, n, k, out);
}
static int moe_block_float(const float *x, size_t tokens, size_t hidden, size_t cols, size_t inter, size_t n_experts, size_t top_k,
                           const uint64_t *experts, const float *weights, const uint8_t *const *gate_up, const uint8_t *const *down,
                           int format, const float *gate_up_bias, const float *down_bias, int rule, float limit, float alpha, float *out) {
    if (cols < hidden) return 1;
    const size_t el = format == 32 ? 4 : 2;
    float *xp = (float *)calloc(cols ? cols : 1, sizeof(float));
    float *g = (float *)malloc((inter ? inter : 1) * sizeof(float)), *u = (float *)malloc((inter ? inter : 1) * sizeof(float));
    float *act = (float *)malloc((inter ? inter : 1) * sizeof(float)), *h2 = (float *)malloc((hidden ? hidden : 1) * sizeof(float));
    for (size_t t = 0; t < tokens; t++) {
        float *o = out + t * hidden;
        for (size_t i = 0; i < hidden; i++) { o[i] = 0.0f; xp[i] = x[t * hidden + i]; }
        if (inter == 0) continue;
        for (size_t s = 0; s < top_k; s++) {
            const uint64_t e = experts[t * top_k + s];
            const float w = weights[t * top_k + s];
            if (e >= n_experts) continue;
            float_gemv(format, gate_up[e], xp, inter, cols, g);
            float_gemv(format, gate_up[e] + inter * cols * el, xp, inter, cols, u);
            for (size_t j = 0; j < inter; j++) {
                const float gb = gate_up_bias ? gate_up_bias[e * 2 * inter + 2 * j] : 0.0f;
                const float ub = gate_up_bias ? gate_up_bias[e * 2 * inter + 2 * j + 1] : 0.0f;
                act[j] = lq_moe_combine(rule, g[j] + gb, u[j] + ub, limit, alpha);
            }
            float_gemv(format, down[e], act, hidden, inter, h2);
            for (size_t i = 0; i < hidden; i++) {
                const float v = down_bias ? h2[i] + down_bias[e * hidden + i] : h2[i];
                o[i] += w * v;
            }
        }
    }
    free(xp); free(g); free(u); free(act); free(h2);
    return 0;
}

/* cpu_moe_forward's integer expert path with the routing given — larql-compute/src/cpu/ops/moe/forward.rs:160-330 and
 * run_single_expert_kq_q8k_into, cpu/ops/moe/expert/q4k.rs:232-351.  Per token the expert input is zero-padded to the
 * gate/up matrices' stored row width `cols` (forward.rs:176-184) and quantised to Q8_K once for all its experts; per
 * selected expert, in selection order: gate and up are the first and second half of its [2*inter, cols] slab
 * (ContiguousHalves, the only layout this tier serves: forward.rs:69-75), g and u get their biases from the fused row
 * (gate at 2j, up at 2j+1: ExpertMlp::gate_bias / up_bias, pipeline/moe.rs:150-170), the pair is combined under
 * `rule`, the activation is zero-padded to inter_padded = ceil(inter/256)*256 and quantised to Q8_K, the down matvec
 * over [hidden, inter_padded] gets the expert's down bias, and out += w * that (forward.rs:220-228).  An expert id
 * outside the bank is skipped (forward.rs:203-208).  format: 4 = Q4_K, 6 = Q6_K (one format for the whole bank). */
int lq_moe_block_kq(const float *x, size_t tokens, size_t hidden, size_t cols, size_t inter, size_t n_experts, size_t top_k,
                    const uint64_t *experts, const float *weights, const uint8_t *const *gate_up, const uint8_t *const *down,
                    int format, const float *gate_up_bias, const float *down_bias, int rule, float limit, float alpha, float *out) {
    if (format == 16 || format == 17 || format == 32)
        return moe_block_float(x, tokens, hidden, cols, inter, n_experts, top_k, experts, weights, gate_up, down, format, gate_up_bias, down_bias,
                               rule, limit, alpha, out);
    if ((format != 4 && format != 6) || cols % 256 != 0 || cols < hidden) return 1;
    const size_t blk = format == 6 ? 210 : 144;
    const size_t inter_padded = (inter + 255) / 256 * 256;
    const size_t half = inter * (cols / 256) * blk, down_bytes = hidden * (inter_padded / 256) * blk;
    float *xp = (float *)calloc(cols ? cols : 1, sizeof(float));
    int8_t *xq = (int8_t *)malloc(cols ? cols : 1);
    float *xd = (float *)malloc((cols / 256 + 1) * sizeof(float));
    int16_t *xs = (int16_t *)malloc((cols / 32 + 1) * sizeof(int16_t));
    float *g = (float *)malloc((inter ? inter : 1) * sizeof(float)), *u = (float *)malloc((inter ? inter : 1) * sizeof(float));
    float *act = (float *)calloc(inter_padded ? inter_padded : 1, sizeof(float));
    int8_t *aq = (int8_t *)malloc(inter_padded ? inter_padded : 1);
    float *ad = (float *)malloc((inter_padded / 256 + 1) * sizeof(float));
    int16_t *as = (int16_t *)malloc((inter_padded / 32 + 1) * sizeof(int16_t));
    float *h2 = (float *)malloc((hidden ? hidden : 1) * sizeof(float));
    int rc = 0;
    for (size_t t = 0; t < tokens && !rc; t++) {
        float *o = out + t * hidden;
        for (size_t i = 0; i < hidden; i++) { o[i] = 0.0f; xp[i] = x[t * hidden + i]; }
        if (inter == 0 || cols == 0) continue;
        rc |= lq_quantize_x_to_q8k(xp, cols, xq, xd, xs);
        for (size_t s = 0; s < top_k && !rc; s++) {
            const uint64_t e = experts[t * top_k + s];
            const float w = weights[t * top_k + s];
            if (e >= n_experts) continue;
            if (format == 6) {
                rc |= lq_q6k_q8k_matvec(g, inter, xq, cols, xd, gate_up[e], half, inter, cols);
                rc |= lq_q6k_q8k_matvec(u, inter, xq, cols, xd, gate_up[e] + half, half, inter, cols);
            } else {
                rc |= lq_q4k_q8k_matvec(g, inter, xq, cols, xd, xs, gate_up[e], half, inter, cols);
                rc |= lq_q4k_q8k_matvec(u, inter, xq, cols, xd, xs, gate_up[e] + half, half, inter, cols);
            }
            for (size_t j = 0; j < inter; j++) {
                const float gb = gate_up_bias ? gate_up_bias[e * 2 * inter + 2 * j] : 0.0f;
                const float ub = gate_up_bias ? gate_up_bias[e * 2 * inter + 2 * j + 1] : 0.0f;
                act[j] = lq_moe_combine(rule, g[j] + gb, u[j] + ub, limit, alpha);
            }
            rc |= lq_quantize_x_to_q8k(act, inter_padded, aq, ad, as);
            if (format == 6) rc |= lq_q6k_q8k_matvec(h2, hidden, aq, inter_padded, ad, down[e], down_bytes, hidden, inter_padded);
            else rc |= lq_q4k_q8k_matvec(h2, hidden, aq, inter_padded, ad, as, down[e], down_bytes, hidden, inter_padded);
            for (size_t i = 0; i < hidden; i++) {
                const float v = down_bias ? h2[i] + down_bias[e * hidden + i] : h2[i];
                o[i] += w * v;
            }
        }
    }
    free(xp); free(xq); free(xd); free(xs); free(g); free(u); free(act); free(aq); free(ad); free(as); free(h2);
    return rc;
}

/* ------------------------------------------- multi-threaded CPU baseline */

typedef struct {
    int kind; /* 0 q4k matvec, 1 q8_0 gemv, 2 mxfp4 gemv, 3 q4k matmul, 4 bf16 gemv */
    float *out; const float *x; const uint8_t *w; const float *sum_x;
    size_t rows, blocks_per_row; int tid, nthreads;
    const uint8_t *aux; size_t seq; float *tmp; /* mxfp4 scales; matmul positions and its [rows, seq] scratch */
} mt_job;

static void *mt_worker(void *p) {
    mt_job *j = (mt_job *)p;
    size_t n_chunks = (j->rows + 31) / 32; /* CHUNK_ROWS = 32 in the reference's row-parallel kernels */
    for (size_t c = (size_t)j->tid; c < n_chunks; c += (size_t)j->nthreads) {
        size_t r0 = c * 32, r1 = r0 + 32 < j->rows ? r0 + 32 : j->rows;
        if (j->kind == 0) q4k_rows(j->out, j->x, j->w, j->sum_x, r0, r1, j->blocks_per_row);
        else if (j->kind == 1) for (size_t r = r0; r < r1; r++) j->out[r] = q8_0_row_dot(j->w, j->x, r, j->blocks_per_row);
        else if (j->kind == 2) {
            moe_matrix m = {1, NULL, j->w, j->aux};
            for (size_t r = r0; r < r1; r++) j->out[r] = moe_row_dot(&m, r, j->blocks_per_row * 32, j->x);
        } else if (j->kind == 4) {
            size_t k = j->blocks_per_row;
            lq_bf16_gemv((const uint16_t *)j->w + r0 * k, j->x, r1 - r0, k, j->out + r0);
        } else { /* the row loop of lq_q4k_matmul_into for rows r0..r1 */
            float wf[256];
            size_t n_blocks = j->blocks_per_row, row_bytes = n_blocks * 144, hidden = n_blocks * 256;
            for (size_t r = r0; r < r1; r++) {
                float *out_row = j->tmp + r * j->seq;
                for (size_t sb = 0; sb < n_blocks; sb++) {
                    decode_q4k_superblock_into(j->w, r * row_bytes, sb, wf);
                    for (size_t s = 0; s < j->seq; s++) out_row[s] += dot_256_f32_scalar(wf, j->x + s * hidden + sb * 256);
                }
            }
        }
    }
    return NULL;
}

static void mt_run(mt_job proto, int threads) {
    if (threads < 1) threads = 1;
    if (threads > 256) threads = 256;
    pthread_t th[256]; mt_job jobs[256];
    for (int t = 0; t < threads; t++) { jobs[t] = proto; jobs[t].tid = t; jobs[t].nthreads = threads; }
    for (int t = 1; t < threads; t++) pthread_create(&th[t], NULL, mt_worker, &jobs[t]);
    mt_worker(&jobs[0]);
    for (int t = 1; t < threads; t++) pthread_join(th[t], NULL);
}

/* lq_mxfp4_gemv with its rows shared out in chunks of 32 (timing baseline; same bits per row) */
int lq_mxfp4_gemv_mt(const uint8_t *packed, const uint8_t *scales, const float *x, size_t n, size_t k, float *out, int threads) {
    if (k % 32 != 0) return 1;
    mt_job j = {2, out, x, packed, NULL, n, k / 32, 0, 1, scales, 0, NULL};
    mt_run(j, threads);
    return 0;
}

/* lq_bf16_gemv with its rows shared out in chunks of 32 (timing baseline; same bits per row) */
int lq_bf16_gemv_mt(const uint16_t *w, const float *x, size_t n, size_t k, float *out, int threads) {
    mt_job j = {4, out, x, (const uint8_t *)w, NULL, n, k, 0, 1, NULL, 0, NULL};
    mt_run(j, threads);
    return 0;
}

/* lq_q4k_matmul_into with its rows shared out in chunks of 32, as kquant_matmul_into schedules them
 * (q4_common/matmul.rs:100-139); same bits. */
int lq_q4k_matmul_into_mt(float *out, const float *x, const uint8_t *w, size_t w_len, size_t rows, size_t hidden, size_t seq, int threads) {
    if (rows == 0 || seq == 0 || hidden == 0 || hidden % 256 != 0 || w_len < rows * (hidden / 256) * 144) return 1;
    float *tmp = (float *)calloc(rows * seq, sizeof(float));
    mt_job j = {3, NULL, x, w, NULL, rows, hidden / 256, 0, 1, NULL, seq, tmp};
    mt_run(j, threads);
    for (size_t r = 0; r < rows; r++)
        for (size_t s = 0; s < seq; s++) out[s * rows + r] = tmp[r * seq + s];
    free(tmp);
    return 0;
}

int lq_q4k_matvec_into_mt(float *out, const float *x, const uint8_t *w, size_t w_len,
                          size_t rows, size_t cols, int threads) {
    if (!kernel_shape_ok(rows, rows, cols, cols, w_len, 256, 144)) return 1;
    if (rows == 0 || cols == 0) { for (size_t i = 0; i < rows; i++) out[i] = 0.0f; return 0; }
    size_t n_blocks = cols / 256;
    float *sum_x = q4k_sum_x(x, n_blocks);
    mt_job j = {0, out, x, w, sum_x, rows, n_blocks, 0, 1, NULL, 0, NULL};
    mt_run(j, threads);
    free(sum_x);
    return 0;
}

int lq_q8_0_gemv_mt(const uint8_t *blocks, size_t blocks_len, const float *x,
                    size_t n, size_t k, float *out, int threads) {
    if (k == 0 || k % 32 != 0) return 1;
    size_t per_row = k / 32;
    if (blocks_len != n * per_row * 34) return 1;
    mt_job j = {1, out, x, blocks, NULL, n, per_row, 0, 1, NULL, 0, NULL};
    mt_run(j, threads);
    return 0;
}
