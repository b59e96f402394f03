// quantize.hip — the reference's block encoders as gfx950 kernels, bit-exact
// with the host encoders they restate, plus the synthetic data generator.
//
// Bit-exactness rests on IEEE f32 add/mul/div (HIP's default correctly rounded
// divide), no FMA contraction in this file, f32 denormals preserved, and
// roundf (half away from zero) == Rust's f32::round.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

#pragma clang fp contract(off)

namespace larql {

__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }
// Rust `as u8` after a clamp: NaN -> 0
__device__ __forceinline__ uint32_t sat_u8(float v) { return v != v ? 0u : (uint32_t)v; }
__device__ __forceinline__ int sat_i8(float v) { return v != v ? 0 : (int)v; }

// larql-compute/src/cpu/ops/q4_common/f16.rs:10-41 (truncate, keep subnormals)
__device__ __forceinline__ uint32_t f32_to_f16_trunc(float val) {
    const uint32_t bits = f2u(val);
    const uint32_t sign = (bits >> 16) & 0x8000u;
    const int exp = (int)((bits >> 23) & 0xFF);
    const uint32_t mant = bits & 0x7FFFFFu;
    if (exp == 0) return sign;
    if (exp == 255) return sign | 0x7C00u | (mant >> 13);
    const int new_exp = exp - 127 + 15;
    if (new_exp >= 31) return sign | 0x7C00u;
    if (new_exp <= 0) {
        const uint32_t sh = 13u + (uint32_t)(1 - new_exp);
        if (sh >= 24u) return sign;
        return sign | ((mant | 0x800000u) >> sh);
    }
    return sign | ((uint32_t)new_exp << 10) | (mant >> 13);
}

// larql-models/src/quant/half.rs:70-104 (IEEE round-to-nearest-even, subnormals kept)
__device__ __forceinline__ uint32_t f32_to_f16_nearest(float value) {
    const uint32_t bits = f2u(value);
    const uint32_t sign = (bits >> 16) & 0x8000u;
    const int exp = (int)((bits >> 23) & 0xFF);
    const uint32_t mant = bits & 0x007FFFFFu;
    if (exp == 255) return sign | (mant == 0 ? 0x7C00u : 0x7E00u);
    const int exp16 = exp - 127 + 15;
    if (exp16 >= 31) return sign | 0x7C00u;
    uint32_t significand, shift;
    if (exp16 >= 1) { significand = mant; shift = 13; }
    else if (exp == 0 || exp16 < -10) return sign;
    else { significand = mant | 0x00800000u; shift = (uint32_t)(14 - exp16); }
    uint32_t magnitude = significand >> shift;
    const uint32_t remainder = significand & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1u);
    if (remainder > half || (remainder == half && (magnitude & 1u))) magnitude += 1;
    if (exp16 >= 1) magnitude += ((uint32_t)exp16) << 10;
    return sign | (magnitude & 0xFFFFu);
}

// the inline conversion of quantize_q4_0 (q4_common/quantize.rs:41-58)
__device__ __forceinline__ uint32_t f32_to_f16_flush(float v) {
    const uint32_t bits = f2u(v);
    const uint32_t sign = (bits >> 16) & 0x8000u;
    const int exp = (int)((bits >> 23) & 0xFF);
    const uint32_t mant = bits & 0x7FFFFFu;
    if (exp == 0) return sign;
    if (exp == 255) return sign | 0x7C00u | (mant >> 13);
    const int new_exp = exp - 127 + 15;
    if (new_exp >= 31) return sign | 0x7C00u;
    if (new_exp <= 0) return sign;
    return sign | ((uint32_t)new_exp << 10) | (mant >> 13);
}

// ---------------------------------------------------------------------------
// quantize_q4_k — larql-compute/src/cpu/ops/q4_common/quantize.rs:89-189.
// One wavefront per 256-element super-block; lane l owns elements 4l..4l+3
// (all inside sub-block l/8).  min/max folds are order-independent, so the
// wave reductions give the host's numbers exactly.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float wave_min_span(float v, int span) {
    for (int o = 1; o < span; o <<= 1) v = fminf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_max_span(float v, int span) {
    for (int o = 1; o < span; o <<= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

__global__ void __launch_bounds__(256) quantize_q4_k_kernel(const float *__restrict__ src, size_t n_sb,
                                                            uint8_t *__restrict__ dst) {
    const uint32_t lane = threadIdx.x & 63u;
    const size_t sb = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (sb >= n_sb) return;
    const float4 v = reinterpret_cast<const float4 *>(src + sb * 256)[lane];
    const float e[4] = {v.x, v.y, v.z, v.w};
    const uint32_t sub = lane >> 3;  // 8 lanes per 32-element sub-block
    float mn = fminf(fminf(e[0], e[1]), fminf(e[2], e[3]));
    float mx = fmaxf(fmaxf(e[0], e[1]), fmaxf(e[2], e[3]));
    mn = fminf(wave_min_span(mn, 8), 0.0f);
    mx = fmaxf(wave_max_span(mx, 8), 0.0f);
    const float range = mx - mn;
    // across the 8 sub-blocks (lanes differing in bits 3..5)
    float gmr = range, gmin = mn;
    for (int o = 8; o < 64; o <<= 1) {
        gmr = fmaxf(gmr, __shfl_xor(gmr, o, 64));
        gmin = fminf(gmin, __shfl_xor(gmin, o, 64));
    }
    gmr = fmaxf(gmr, 0.0f);
    const float d = gmr > 0.0f ? gmr / (15.0f * 63.0f) : 0.0f;
    const float dmin = gmin < 0.0f ? -gmin / 63.0f : 0.0f;
    const uint32_t q_scale = d > 0.0f ? sat_u8(clampf(roundf(range / (15.0f * d)), 0.0f, 63.0f)) : 0u;
    const uint32_t q_min = dmin > 0.0f ? sat_u8(clampf(roundf(-mn / dmin), 0.0f, 63.0f)) : 0u;
    const float sc = d * (float)q_scale;
    const float mnv = dmin * (float)q_min;
    const float inv = sc > 0.0f ? 1.0f / sc : 0.0f;
    uint32_t enc = 0;  // 4 codes, one per byte
#pragma unroll
    for (int i = 0; i < 4; i++) enc |= sat_u8(clampf(roundf((e[i] + mnv) * inv), 0.0f, 15.0f)) << (8 * i);
    uint8_t *o = dst + sb * 144;
    // nibble bytes: group g = sub/2 pairs sub-block 2g (low) with 2g+1 (high); lane holds
    // elements 4*(lane&7).. of its sub-block -> bytes g*32 + 4*(lane&7) ..+3
    const uint32_t partner = (uint32_t)__shfl_xor((int)enc, 8, 64);  // same position, other sub-block of the pair
    if ((sub & 1u) == 0) {
        const uint32_t packed = enc | (partner << 4);
        reinterpret_cast<uint32_t *>(o + 16 + (sub >> 1) * 32)[lane & 7u] = packed;
    }
    // header: lanes 0..7*8 hold the per-sub-block scale/min; gather them to lane 0
    uint32_t qs[8], qm[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        qs[j] = (uint32_t)__shfl((int)q_scale, j * 8, 64);
        qm[j] = (uint32_t)__shfl((int)q_min, j * 8, 64);
    }
    if (lane == 0) {
        uint32_t w0 = f32_to_f16_trunc(d) | (f32_to_f16_trunc(dmin) << 16);
        uint32_t w1 = 0, w2 = 0, w3 = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            w1 |= ((qs[j] & 0x3Fu) | (((qs[j + 4] >> 4) & 3u) << 6)) << (8 * j);
            w2 |= ((qm[j] & 0x3Fu) | (((qm[j + 4] >> 4) & 3u) << 6)) << (8 * j);
            w3 |= ((qs[j + 4] & 0x0Fu) | ((qm[j + 4] & 0x0Fu) << 4)) << (8 * j);
        }
        uint4 h = {w0, w1, w2, w3};
        *reinterpret_cast<uint4 *>(o) = h;
    }
}

// ---------------------------------------------------------------------------
// quantize_q6_k — larql-compute/src/cpu/ops/q4_common/quantize.rs:198-276.
// One wavefront per 256-element super-block; lane l owns elements 4l..4l+3, all
// inside the 16-element sub-block l/4.  d = amax / (31*127); sub-block scale =
// round(sub_max / (31 d)) as i8; code = round(v * (1 / (d * scale))) clamped to
// -32..31, biased by 32.  The 256 six-bit codes pass through LDS into ggml's
// planar layout: ql[64h + p] = code[128h + p] & 15 | (code[128h + p + 64] & 15) << 4,
// qh[32h + l] = the top two bits of codes 128h + l + {0, 32, 64, 96}; then the 16
// scales and the truncated f16 d (210 bytes, 2-byte aligned).
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) quantize_q6_k_kernel(const float *__restrict__ src, size_t n_sb, uint8_t *__restrict__ dst) {
    __shared__ uint8_t codes[4][256];
    const uint32_t lane = threadIdx.x & 63u, wv = threadIdx.x >> 6;
    const size_t sb = (size_t)blockIdx.x * 4 + wv;
    if (sb >= n_sb) return;  // (whole wavefronts leave together: no workgroup barrier below)
    const float4 v = reinterpret_cast<const float4 *>(src + sb * 256)[lane];
    const float e[4] = {v.x, v.y, v.z, v.w};
    float sub_max = fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3])));
    sub_max = wave_max_span(sub_max, 4);
    float amax = sub_max;
    for (int o = 4; o < 64; o <<= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
    const float d = amax / (31.0f * 127.0f);
    const float scf = d > 0.0f ? sub_max / (31.0f * d) : 0.0f;
    const int sub_scale = sat_i8(clampf(roundf(scf), -128.0f, 127.0f));
    const float sc = d * (float)sub_scale;
    const float inv = fabsf(sc) > 1e-10f ? 1.0f / sc : 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) codes[wv][4 * lane + i] = (uint8_t)(sat_i8(clampf(roundf(e[i] * inv), -32.0f, 31.0f)) + 32);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const uint8_t *c = codes[wv];
    uint8_t *o = dst + sb * 210;
    {   // ql bytes 2*lane, 2*lane + 1
        const uint32_t i0 = 2 * lane, h = i0 >> 6, p = i0 & 63u;
        const uint32_t b0 = (c[128 * h + p] & 15u) | ((c[128 * h + p + 64] & 15u) << 4);
        const uint32_t b1 = (c[128 * h + p + 1] & 15u) | ((c[128 * h + p + 65] & 15u) << 4);
        *reinterpret_cast<uint16_t *>(o + i0) = (uint16_t)(b0 | (b1 << 8));
    }
    {   // qh byte `lane`
        const uint32_t h = lane >> 5, l = lane & 31u, b = 128 * h + l;
        o[128 + lane] = (uint8_t)(((c[b] >> 4) & 3u) | (((c[b + 32] >> 4) & 3u) << 2) | (((c[b + 64] >> 4) & 3u) << 4) | (((c[b + 96] >> 4) & 3u) << 6));
    }
    const int scale_of = __shfl(sub_scale, (int)((lane & 15u) * 4), 64);  // sub-block j lives in lanes 4j..4j+3
    if (lane < 16) o[192 + lane] = (uint8_t)scale_of;
    if (lane == 0) *reinterpret_cast<uint16_t *>(o + 208) = (uint16_t)f32_to_f16_trunc(d);
}

// ---------------------------------------------------------------------------
// quantize_q8_0 — larql-models/src/quant/ggml/quantize.rs:50-77; and the two
// Q4_0-path encoders, q4_common/quantize.rs:6-69.  One thread per 32-element
// block (the fold over |v| is order-independent).
// ---------------------------------------------------------------------------

__global__ void quantize_q8_0_kernel(const float *__restrict__ src, size_t n_blocks, uint8_t *__restrict__ dst) {
    const size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= n_blocks) return;
    const float4 *p = reinterpret_cast<const float4 *>(src + b * 32);
    float e[32];
#pragma unroll
    for (int i = 0; i < 8; i++) { float4 v = p[i]; e[4 * i] = v.x; e[4 * i + 1] = v.y; e[4 * i + 2] = v.z; e[4 * i + 3] = v.w; }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(e[i]));
    const float scale = amax / 127.0f;
    const float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
    uint16_t *o = reinterpret_cast<uint16_t *>(dst + b * 34);
    o[0] = (uint16_t)f32_to_f16_nearest(scale);
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const uint32_t q0 = (uint32_t)sat_i8(clampf(roundf(e[2 * i] * inv), -128.0f, 127.0f)) & 0xFFu;
        const uint32_t q1 = (uint32_t)sat_i8(clampf(roundf(e[2 * i + 1] * inv), -128.0f, 127.0f)) & 0xFFu;
        o[1 + i] = (uint16_t)(q0 | (q1 << 8));
    }
}

__global__ void quantize_to_q8_kernel(const float *__restrict__ src, size_t n_blocks, int8_t *__restrict__ q8,
                                      float *__restrict__ scales) {
    const size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= n_blocks) return;
    float amax = 0.0f;
    for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(src[b * 32 + i]));
    const float scale = amax / 127.0f;
    scales[b] = scale;
    const float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
    for (int i = 0; i < 32; i++) q8[b * 32 + i] = (int8_t)sat_i8(clampf(roundf(src[b * 32 + i] * inv), -128.0f, 127.0f));
}

// quantize_x_to_q8k — larql-compute/src/cpu/ops/q4k_q8k_dot/q8k_activation.rs:84-109: per 256-element super-block
// d = amax/127, codes round(x * (1/d)) clamped to +-127, and the sum of every 32 codes.  One wavefront per
// super-block, four elements per lane; the eight lanes of a sub-block add their codes by shuffles (integers: any
// order).  Output is the device layout of a Q8_K activation of n elements: [n codes | n/256 f32 scales | n/32 i16 sums].
__global__ void __launch_bounds__(256) quantize_x_to_q8k_kernel(const float *__restrict__ src, size_t n_blocks, uint8_t *__restrict__ dst) {
    const size_t sb = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (sb >= n_blocks) return;
    const uint32_t lane = threadIdx.x & 63u;
    const float4 v = reinterpret_cast<const float4 *>(src + sb * 256)[lane];
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));  // fmaxf ignores a NaN operand, as f32::max does
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    const float scale = amax > 0.0f ? amax / 127.0f : 0.0f;
    const float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
    const int q0 = sat_i8(clampf(roundf(v.x * inv), -127.0f, 127.0f)), q1 = sat_i8(clampf(roundf(v.y * inv), -127.0f, 127.0f));
    const int q2 = sat_i8(clampf(roundf(v.z * inv), -127.0f, 127.0f)), q3 = sat_i8(clampf(roundf(v.w * inv), -127.0f, 127.0f));
    int sum = q0 + q1 + q2 + q3;
    sum += __shfl_xor(sum, 1);
    sum += __shfl_xor(sum, 2);
    sum += __shfl_xor(sum, 4);
    const size_t n = n_blocks * 256;
    reinterpret_cast<uint32_t *>(dst)[sb * 64 + lane] =
        ((uint32_t)q0 & 0xFFu) | (((uint32_t)q1 & 0xFFu) << 8) | (((uint32_t)q2 & 0xFFu) << 16) | (((uint32_t)q3 & 0xFFu) << 24);
    if (lane == 0) reinterpret_cast<float *>(dst + n)[sb] = scale;
    if ((lane & 7u) == 0) reinterpret_cast<int16_t *>(dst + n + n_blocks * 4)[sb * 8 + (lane >> 3)] = (int16_t)sum;
}

__device__ __forceinline__ int sat_i32(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return 2147483647;
    if (v <= -2147483648.0f) return (int)0x80000000;
    return (int)v;
}

__global__ void quantize_q4_0_kernel(const float *__restrict__ src, size_t n_blocks, uint8_t *__restrict__ dst) {
    const size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= n_blocks) return;
    const float *blk = src + b * 32;
    float amax = 0.0f;
    for (int i = 0; i < 32; i++) amax = fmaxf(amax, fabsf(blk[i]));
    const float scale = amax / 7.0f;
    const float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
    uint8_t *o = dst + b * 18;
    const uint32_t h = f32_to_f16_flush(scale);
    o[0] = (uint8_t)(h & 0xFF); o[1] = (uint8_t)(h >> 8);
    for (int j = 0; j < 16; j++) {
        int lo = sat_i32(roundf(blk[j] * inv)) + 8, hi = sat_i32(roundf(blk[j + 16] * inv)) + 8;
        lo = lo < 0 ? 0 : (lo > 15 ? 15 : lo);
        hi = hi < 0 ? 0 : (hi > 15 ? 15 : hi);
        o[2 + j] = (uint8_t)(lo | (hi << 4));
    }
}

// ---------------------------------------------------------------------------
// quantize_mxfp4 — larql-vindex/src/format/vindex3/opplan/exec/weights/
// load.rs:410-476 with nearest_mxfp4_code (weights/quantize.rs:71-88).
// The reference takes floor(log2f(max|x|)) in f32, which is the f32 exponent
// except for the few largest mantissas of a binade, where the host's log2f
// rounds up to the next integer.  `log2_up[E]` (filled on the host by calling
// the host's own log2f) says for how many of the top mantissas of biased
// exponent E that happens, so the kernel reproduces the host's libm exactly.
// One thread per 32-element group.
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint32_t nearest_mxfp4_code(float v) {
    const float T[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    const uint32_t sign = (f2u(v) >> 31) ? 8u : 0u;
    const float mag = fminf(fabsf(v), 6.0f);
    uint32_t best = 0;
    float best_err = __builtin_inff();
#pragma unroll
    for (uint32_t code = 0; code < 8; code++) {
        const float err = fabsf(mag - T[code]);
        if (err < best_err || (err == best_err && (code & 1u) == 0)) { best = code; best_err = err; }
    }
    return best == 0 ? 0u : (sign | best);
}

__global__ void quantize_mxfp4_kernel(const float *__restrict__ src, size_t n_groups, uint8_t *__restrict__ packed,
                                      uint8_t *__restrict__ scales, const uint8_t *__restrict__ log2_up) {
    const size_t g = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= n_groups) return;
    const float4 *p = reinterpret_cast<const float4 *>(src + g * 32);
    float e[32];
#pragma unroll
    for (int i = 0; i < 8; i++) { float4 v = p[i]; e[4 * i] = v.x; e[4 * i + 1] = v.y; e[4 * i + 2] = v.z; e[4 * i + 3] = v.w; }
    float max_abs = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) max_abs = fmaxf(max_abs, fabsf(e[i]));
    uint32_t scale_byte = 0;
    if (max_abs != 0.0f) {
        const uint32_t bits = f2u(max_abs);
        const uint32_t E = bits >> 23, mant = bits & 0x7FFFFFu;
        int fl;  // floor(log2f(max_abs)) as the host computes it
        if (E == 255) fl = 1 << 20;             // inf/NaN: saturates the clamp below either way
        else if (E == 0) fl = -140;             // f32 subnormal: far below the clamp
        else fl = (int)E - 127 + ((0x800000u - mant) <= (uint32_t)log2_up[E] ? 1 : 0);
        int eb = fl - 2 + 127;
        eb = eb < 1 ? 1 : (eb > 254 ? 254 : eb);
        scale_byte = (uint32_t)eb;
    }
    scales[g] = (uint8_t)scale_byte;
    const float scale = scale_byte == 0 ? 0.0f : u2f(scale_byte << 23);
    const float inv = scale == 0.0f ? 0.0f : 1.0f / scale;
    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
    for (int b = 0; b < 16; b++) {
        const uint32_t lo = nearest_mxfp4_code(e[2 * b] * inv), hi = nearest_mxfp4_code(e[2 * b + 1] * inv);
        w[b >> 2] |= (lo | (hi << 4)) << (8 * (b & 3));
    }
    uint4 o = {w[0], w[1], w[2], w[3]};
    reinterpret_cast<uint4 *>(packed)[g] = o;
}

__global__ void f32_to_bf16_kernel(const float *__restrict__ src, size_t n, uint16_t *__restrict__ dst) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = (uint16_t)(f2u(src[i]) >> 16);  // truncation, larql-models/src/quant/half.rs:107-109
}

// ---------------------------------------------------------------------------
// Synthetic N(0, sigma): element i of stream `seed` = sigma * (S - C) / 2^21,
// S = sum of twelve 21-bit fields of four splitmix64 outputs at counters
// 4i..4i+3, C = 6*(2^21-1).  Integer arithmetic up to one exact int->float
// conversion and one multiply: host and device agree bit for bit.
// ---------------------------------------------------------------------------
__host__ __device__ inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__global__ void fill_normal_kernel(float *__restrict__ dst, size_t n, uint64_t seed, float sigma) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int32_t sum = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint64_t r = splitmix64(seed * 0xD1B54A32D192ED03ull + (uint64_t)(4 * i + j));
        sum += (int32_t)(r & 0x1FFFFF) + (int32_t)((r >> 21) & 0x1FFFFF) + (int32_t)((r >> 42) & 0x1FFFFF);
    }
    const float z = (float)(sum - 6 * 0x1FFFFF) * (1.0f / 2097152.0f);
    dst[i] = z * sigma;
}

// ---------------------------------------------------------------------------
static inline dim3 blocks_for(size_t n, uint32_t t) { return dim3((uint32_t)((n + t - 1) / t)); }

hipError_t quantize_q4_k_launch(hipStream_t s, const float *src, size_t n, uint8_t *dst) {
    const size_t n_sb = n / 256;
    if (n_sb == 0) return hipSuccess;
    hipLaunchKernelGGL(quantize_q4_k_kernel, blocks_for(n_sb, 4), dim3(256), 0, s, src, n_sb, dst);
    return hipGetLastError();
}
hipError_t quantize_q6_k_launch(hipStream_t s, const float *src, size_t n, uint8_t *dst) {
    const size_t n_sb = n / 256;
    if (n_sb == 0) return hipSuccess;
    hipLaunchKernelGGL(quantize_q6_k_kernel, blocks_for(n_sb, 4), dim3(256), 0, s, src, n_sb, dst);
    return hipGetLastError();
}
hipError_t quantize_q8_0_launch(hipStream_t s, const float *src, size_t n, uint8_t *dst) {
    const size_t nb = n / 32;
    if (nb == 0) return hipSuccess;
    hipLaunchKernelGGL(quantize_q8_0_kernel, blocks_for(nb, 256), dim3(256), 0, s, src, nb, dst);
    return hipGetLastError();
}
hipError_t quantize_x_to_q8k_launch(hipStream_t s, const float *src, size_t n, uint8_t *dst) {
    const size_t nb = n / 256;
    if (nb == 0) return hipSuccess;
    hipLaunchKernelGGL(quantize_x_to_q8k_kernel, blocks_for(nb, 4), dim3(256), 0, s, src, nb, dst);
    return hipGetLastError();
}
hipError_t quantize_mxfp4_launch(hipStream_t s, const float *src, size_t rows, size_t k, uint8_t *packed, uint8_t *scales,
                                 const uint8_t *log2_up) {
    const size_t ng = rows * (k / 32);
    if (ng == 0) return hipSuccess;
    hipLaunchKernelGGL(quantize_mxfp4_kernel, blocks_for(ng, 256), dim3(256), 0, s, src, ng, packed, scales, log2_up);
    return hipGetLastError();
}
hipError_t f32_to_bf16_launch(hipStream_t s, const float *src, size_t n, uint16_t *dst) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(f32_to_bf16_kernel, blocks_for(n, 256), dim3(256), 0, s, src, n, dst);
    return hipGetLastError();
}
hipError_t quantize_q4_0_launch(hipStream_t s, const float *src, size_t n, uint8_t *dst) {
    const size_t nb = n / 32;
    if (nb == 0) return hipSuccess;
    hipLaunchKernelGGL(quantize_q4_0_kernel, blocks_for(nb, 256), dim3(256), 0, s, src, nb, dst);
    return hipGetLastError();
}
hipError_t quantize_to_q8_launch(hipStream_t s, const float *src, size_t n, int8_t *q8, float *scales) {
    const size_t nb = n / 32;
    if (nb == 0) return hipSuccess;
    hipLaunchKernelGGL(quantize_to_q8_kernel, blocks_for(nb, 256), dim3(256), 0, s, src, nb, q8, scales);
    return hipGetLastError();
}
hipError_t fill_normal_launch(hipStream_t s, float *dst, size_t n, uint64_t seed, float sigma) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(fill_normal_kernel, blocks_for(n, 256), dim3(256), 0, s, dst, n, seed, sigma);
    return hipGetLastError();
}

}  // namespace larql
