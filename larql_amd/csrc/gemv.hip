// gemv.hip — batch-1 matvec engine for gfx950 (MI355X): Q4_K, ggml Q8_0,
// MXFP4, Q4_0 x Q8, bf16, f16, f32 weights against an f32 activation.
//
// One kernel serves every format and any number of independent matvecs
// ("jobs") per launch.  The work of a launch is a flat list of PASSES: in one
// pass the T threads of a workgroup cover `rpp` consecutive rows of a job,
// thread t owning a fixed K-slice ("chunk") c = t % cpr of row t / cpr.
// Because a thread's chunk never changes within a job, its slice of the
// activation lives in registers for the whole job and the main loop touches
// nothing but the weight stream: coalesced 128-bit loads of consecutive
// packed blocks, decode in registers, FMA.  Workgroups take contiguous,
// equally sized ranges of the pass list (passes have near-equal byte size by
// construction), so a launch is a single balanced sweep over HBM.
//
// Reduction: a thread's partial dot goes to LDS (`part[row_in_tile][chunk]`),
// and once per tile each row is summed in chunk order by a 16-lane group —
// a fixed tree, so results are deterministic and independent of the grid.
//
// The arithmetic restates, per format, the reference CPU kernels cited at each
// routine; only the summation order differs (fp32 accumulate throughout).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "kernels.h"

namespace larql {

// Pointers that arrive inside a job record are generic; telling the compiler
// they are global memory turns flat_load into global_load.
#define GLOBAL_AS __attribute__((address_space(1)))
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef const GLOBAL_AS uint8_t *g_u8p;
typedef const GLOBAL_AS uint32_t *g_u32p;
typedef const GLOBAL_AS u32x4 *g_u4p;
typedef const GLOBAL_AS f32x4 *g_f4p;
typedef const GLOBAL_AS float *g_f32p;
typedef GLOBAL_AS float *g_f32wp;

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ __forceinline__ float half_bits_to_float(uint32_t lo16) {
    // hardware f16 -> f32 conversion; f16 subnormals are preserved (the f16
    // denormal mode is on for HIP kernels), which the Q4_K scales rely on.
    return (float)__builtin_bit_cast(_Float16, (uint16_t)lo16);
}

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);
    return v + __builtin_bit_cast(float, moved);
}

// ---------------------------------------------------------------------------
// Q4_K: one thread = one 32-byte nibble group (sub-blocks 2g and 2g+1 of
// super-block sb, 64 consecutive activations).  Value per row, as
// q4k_matvec_into computes it (larql-compute/src/cpu/ops/q4_common/
// matvec_f32.rs:116-155):  sum over sub-blocks of (d*sc)*dot(q,x) - (dmin*mn)*sum(x).
//
// Nibbles reach the FMA without an integer->float conversion: a nibble left in
// bits 0-3 (or 4-7) of a 16-bit lane IS the f16 subnormal q*2^-24 (q*2^-20),
// and v_fma_mix_f32 widens f16 operands exactly, so fma(f16(q'), x, acc)
// accumulates the dot scaled by an exact power of two that is folded back into
// the sub-block scale.
// ---------------------------------------------------------------------------
struct Q4KSlice {
    float x[64];
    float sum_lo, sum_hi;
};

__device__ __forceinline__ void q4k_load_x(Q4KSlice &s, const float *x, uint32_t c) {
    g_f4p xp = (g_f4p)(x + (size_t)(c >> 2) * 256 + (c & 3) * 64);
    float sl = 0.f, sh = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        f32x4 v = xp[i];
        s.x[4 * i + 0] = v.x; s.x[4 * i + 1] = v.y; s.x[4 * i + 2] = v.z; s.x[4 * i + 3] = v.w;
        float q = (v.x + v.y) + (v.z + v.w);
        if (i < 8) sl += q; else sh += q;
    }
    s.sum_lo = sl; s.sum_hi = sh;
}

__device__ __forceinline__ float q4k_group_dot(const u32x4 hdr, const u32x4 q0, const u32x4 q1,
                                               const Q4KSlice &s, uint32_t g) {
    float alo0 = 0.f, alo1 = 0.f, ahi0 = 0.f, ahi1 = 0.f;
    const uint32_t qd[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t v = qd[i], u = v >> 8;
        const half2_t l02 = as_half2(v & 0x000F000Fu);  // low nibbles of bytes 0,2  (q * 2^-24)
        const half2_t h02 = as_half2(v & 0x00F000F0u);  // high nibbles of bytes 0,2 (q * 2^-20)
        const half2_t l13 = as_half2(u & 0x000F000Fu);  // bytes 1,3
        const half2_t h13 = as_half2(u & 0x00F000F0u);
        alo0 = __builtin_fmaf((float)l02.x, s.x[4 * i + 0], alo0);
        alo1 = __builtin_fmaf((float)l13.x, s.x[4 * i + 1], alo1);
        alo0 = __builtin_fmaf((float)l02.y, s.x[4 * i + 2], alo0);
        alo1 = __builtin_fmaf((float)l13.y, s.x[4 * i + 3], alo1);
        ahi0 = __builtin_fmaf((float)h02.x, s.x[32 + 4 * i + 0], ahi0);
        ahi1 = __builtin_fmaf((float)h13.x, s.x[32 + 4 * i + 1], ahi1);
        ahi0 = __builtin_fmaf((float)h02.y, s.x[32 + 4 * i + 2], ahi0);
        ahi1 = __builtin_fmaf((float)h13.y, s.x[32 + 4 * i + 3], ahi1);
    }
    // header: d, dmin (f16) and the 6-bit scales/mins of sub-blocks 2g, 2g+1
    // (get_scale_min_k4 as in matvec_f32.rs:124-131), two bytes at a time.
    const float d = half_bits_to_float(hdr.x & 0xFFFFu);
    const float dmin = half_bits_to_float(hdr.x >> 16);
    const uint32_t sh = (g & 1u) * 16u;
    const uint32_t a = (hdr.y >> sh) & 0xFFFFu, b = (hdr.z >> sh) & 0xFFFFu, c = (hdr.w >> sh) & 0xFFFFu;
    const uint32_t sc_hi2 = (c & 0x0F0Fu) | ((a >> 2) & 0x3030u), mn_hi2 = ((c >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u);
    const uint32_t sc2 = g < 2 ? (a & 0x3F3Fu) : sc_hi2, mn2 = g < 2 ? (b & 0x3F3Fu) : mn_hi2;
    const float sc_lo = d * (float)(sc2 & 0xFFu), sc_hi = d * (float)(sc2 >> 8);
    const float mn_lo = dmin * (float)(mn2 & 0xFFu), mn_hi = dmin * (float)(mn2 >> 8);
    const float dot_lo = (alo0 + alo1) * 16777216.0f;  // * 2^24 (exact)
    const float dot_hi = (ahi0 + ahi1) * 1048576.0f;   // * 2^20 (exact)
    float r = sc_lo * dot_lo - mn_lo * s.sum_lo;
    r += sc_hi * dot_hi - mn_hi * s.sum_hi;
    return r;
}

// ---------------------------------------------------------------------------
// ggml Q8_0: one thread = one 34-byte block (f16 d + 32 int8 codes), 32
// activations.  q8_0_gemv / row_dot (larql-compute/src/cpu/kquant_gemv.rs:
// 67-109) accumulates ((q as f32)*d)*x; here the weight w = q*d is formed
// exactly the same way (q*d is exact in f32) and only the order of the adds
// differs.  Blocks are 2-byte aligned: the thread reads the 9 aligned dwords
// that cover its block and realigns by 16 bits when the block index is even.
// ---------------------------------------------------------------------------
struct X32Slice { float x[32]; };

__device__ __forceinline__ void load_x32(X32Slice &s, const float *x, uint32_t c) {
    g_f4p xp = (g_f4p)(x + (size_t)c * 32);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        f32x4 v = xp[i];
        s.x[4 * i + 0] = v.x; s.x[4 * i + 1] = v.y; s.x[4 * i + 2] = v.z; s.x[4 * i + 3] = v.w;
    }
}

struct Q8Raw { uint32_t d[9]; };

__device__ __forceinline__ Q8Raw q8_0_load(const uint8_t *row, uint32_t c) {
    // block c starts at 34c; the aligned window starts at 34c (c even) or 34c-2 (c odd)
    g_u32p p = (g_u32p)(row + (size_t)c * 34 - ((c & 1u) * 2u));
    Q8Raw r;
#pragma unroll
    for (int i = 0; i < 9; i++) r.d[i] = p[i];
    return r;
}

__device__ __forceinline__ float q8_0_block_dot(const Q8Raw &r, const X32Slice &s, uint32_t c) {
    const bool odd = (c & 1u) != 0;
    // even: [d | q0 q1][q2..q5]...[q30 q31 | next]   odd: [prev | d][q0..q3]...[q28..q31]
    const float d = half_bits_to_float(odd ? (r.d[0] >> 16) : (r.d[0] & 0xFFFFu));
    float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t v = odd ? r.d[i + 1] : __builtin_amdgcn_alignbit(r.d[i + 1], r.d[i], 16);
        const float w0 = (float)(int)(int8_t)(v & 0xFF) * d;
        const float w1 = (float)(int)(int8_t)((v >> 8) & 0xFF) * d;
        const float w2 = (float)(int)(int8_t)((v >> 16) & 0xFF) * d;
        const float w3 = (float)((int)v >> 24) * d;
        acc0 = __builtin_fmaf(w0, s.x[4 * i + 0], acc0);
        acc1 = __builtin_fmaf(w1, s.x[4 * i + 1], acc1);
        acc0 = __builtin_fmaf(w2, s.x[4 * i + 2], acc0);
        acc1 = __builtin_fmaf(w3, s.x[4 * i + 3], acc1);
    }
    return acc0 + acc1;
}

// ---------------------------------------------------------------------------
// MXFP4: one thread = one 32-element group: 16 packed bytes (element 2b in the
// low nibble of byte b) + one e8m0 scale byte.  Value as mxfp4_loop computes it
// (larql-vindex/src/format/vindex3/opplan/exec/tests/device.rs:109-127):
// sum (T[nib]*s)*x.  The scale is a power of two, so s * sum(T[nib]*x) is the
// same number; e8m0 0 -> 0.0 and 255 -> NaN (larql-models/src/quant/
// mxfp4.rs:26-35) then fall out of the one f32 multiply.  Nibbles are decoded
// by the gfx950 fp4 conversion (two e2m1 values per instruction).
// ---------------------------------------------------------------------------
__device__ __forceinline__ float e8m0_to_float(uint32_t b) {
    return b == 0 ? 0.0f : (b == 255 ? __builtin_nanf("") : __builtin_bit_cast(float, b << 23));
}

__device__ __forceinline__ float mxfp4_group_dot(const u32x4 q, uint32_t scale_byte, const X32Slice &s) {
    const uint32_t qd[4] = {q.x, q.y, q.z, q.w};
    float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float2_t p0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(qd[i], 1.0f, 0);
        const float2_t p1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(qd[i], 1.0f, 1);
        const float2_t p2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(qd[i], 1.0f, 2);
        const float2_t p3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(qd[i], 1.0f, 3);
        acc0 = __builtin_fmaf(p0.x, s.x[8 * i + 0], acc0);
        acc1 = __builtin_fmaf(p0.y, s.x[8 * i + 1], acc1);
        acc0 = __builtin_fmaf(p1.x, s.x[8 * i + 2], acc0);
        acc1 = __builtin_fmaf(p1.y, s.x[8 * i + 3], acc1);
        acc0 = __builtin_fmaf(p2.x, s.x[8 * i + 4], acc0);
        acc1 = __builtin_fmaf(p2.y, s.x[8 * i + 5], acc1);
        acc0 = __builtin_fmaf(p3.x, s.x[8 * i + 6], acc0);
        acc1 = __builtin_fmaf(p3.y, s.x[8 * i + 7], acc1);
    }
    return e8m0_to_float(scale_byte) * (acc0 + acc1);
}

// ---------------------------------------------------------------------------
// Q4_0 x Q8: one thread = one 18-byte block (f16 d + 16 planar nibble bytes:
// byte j = element j | element j+16 << 4) against 32 int8 activation codes and
// their f32 block scale.  q4_0_matvec_c (larql-compute/csrc/q4_dot.c:176-207)
// sums (lo-8)*q8*(d*s) per element in f32; the integer products are summed
// exactly here (|sum| < 2^15) and scaled once, which differs from the CPU only
// by f32 rounding of the partial sums.
// ---------------------------------------------------------------------------
struct Q8ActSlice { uint32_t q[8]; float scale; int code_sum; };

__device__ __forceinline__ void load_q8act(Q8ActSlice &s, const int8_t *q8, const float *scales, uint32_t c) {
    g_u4p p = (g_u4p)(q8 + (size_t)c * 32);
    u32x4 a = p[0], b = p[1];
    s.q[0] = a.x; s.q[1] = a.y; s.q[2] = a.z; s.q[3] = a.w;
    s.q[4] = b.x; s.q[5] = b.y; s.q[6] = b.z; s.q[7] = b.w;
    s.scale = ((g_f32p)scales)[c];
    int cs = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) cs = __builtin_amdgcn_sdot4(0x01010101, (int)s.q[i], cs, false);
    s.code_sum = cs;
}

struct Q40Raw { uint32_t d[5]; };

__device__ __forceinline__ Q40Raw q4_0_load(const uint8_t *row, uint32_t c) {
    // block c at 18c: 4-byte aligned when c is even, else window starts at 18c-2
    g_u32p p = (g_u32p)(row + (size_t)c * 18 - ((c & 1u) * 2u));
    Q40Raw r;
#pragma unroll
    for (int i = 0; i < 5; i++) r.d[i] = p[i];
    return r;
}

__device__ __forceinline__ float q4_0_block_dot(const Q40Raw &r, const Q8ActSlice &s, uint32_t c) {
    const bool odd = (c & 1u) != 0;
    const float d = half_bits_to_float(odd ? (r.d[0] >> 16) : (r.d[0] & 0xFFFFu));
    int isum = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t v = odd ? r.d[i + 1] : __builtin_amdgcn_alignbit(r.d[i + 1], r.d[i], 16);
        // bytes 4i..4i+3: low nibbles are elements 4i..4i+3, high nibbles 16+4i..
        const uint32_t lo = v & 0x0F0F0F0Fu, hi = (v >> 4) & 0x0F0F0F0Fu;
        const uint32_t xl = s.q[i], xh = s.q[4 + i];
        isum = __builtin_amdgcn_sdot4((int)lo, (int)xl, isum, false);  // nibbles 0..15 are valid signed bytes
        isum = __builtin_amdgcn_sdot4((int)hi, (int)xh, isum, false);
    }
    isum -= 8 * s.code_sum;  // sum (n-8)*x = sum n*x - 8*sum x
    return (float)isum * (d * s.scale);
}

// ---------------------------------------------------------------------------
// Dense rows (gate vectors): one thread = 16 activations.
//   bf16: f32 = bits << 16 (larql-models/src/quant/half.rs:38-40), dot as
//         bf16_dot_portable (larql-vindex/.../opplan/exec/cpu/kernels.rs:718-723)
//   f16 : widened by the hardware conversion (IEEE, subnormals kept)
//   f32 : gemv of larql-vindex/src/index/storage/gate_store.rs:119-143
// ---------------------------------------------------------------------------
struct X16Slice { float x[16]; };

__device__ __forceinline__ void load_x16(X16Slice &s, const float *x, uint32_t c) {
    g_f4p xp = (g_f4p)(x + (size_t)c * 16);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f32x4 v = xp[i];
        s.x[4 * i + 0] = v.x; s.x[4 * i + 1] = v.y; s.x[4 * i + 2] = v.z; s.x[4 * i + 3] = v.w;
    }
}

__device__ __forceinline__ float bf16x16_dot(const u32x4 a, const u32x4 b, const X16Slice &s) {
    const uint32_t d[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        acc0 = __builtin_fmaf(__builtin_bit_cast(float, d[i] << 16), s.x[2 * i], acc0);
        acc1 = __builtin_fmaf(__builtin_bit_cast(float, d[i] & 0xFFFF0000u), s.x[2 * i + 1], acc1);
    }
    return acc0 + acc1;
}

__device__ __forceinline__ float f16x16_dot(const u32x4 a, const u32x4 b, const X16Slice &s) {
    const uint32_t d[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const half2_t h = as_half2(d[i]);
        acc0 = __builtin_fmaf((float)h.x, s.x[2 * i], acc0);
        acc1 = __builtin_fmaf((float)h.y, s.x[2 * i + 1], acc1);
    }
    return acc0 + acc1;
}

__device__ __forceinline__ float f32x16_dot(const f32x4 *__restrict__ w, const X16Slice &s) {
    float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const f32x4 v = w[i];
        acc0 = __builtin_fmaf(v.x, s.x[4 * i + 0], acc0);
        acc1 = __builtin_fmaf(v.y, s.x[4 * i + 1], acc1);
        acc0 = __builtin_fmaf(v.z, s.x[4 * i + 2], acc0);
        acc1 = __builtin_fmaf(v.w, s.x[4 * i + 3], acc1);
    }
    return acc0 + acc1;
}

// ---------------------------------------------------------------------------
// Tile epilogue: part[row_in_tile * npart + p] -> out[row].  Sixteen lanes
// per row, each summing parts p = lane, lane+16, ... in order, then a 4-step
// DPP reduction inside the 16-lane row.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void tile_epilogue(const float *part, uint32_t npart, uint32_t tile_rows,
                                              float *out, uint32_t row_base) {
    const uint32_t lane16 = threadIdx.x & 15u;
    for (uint32_t r = threadIdx.x >> 4; r < tile_rows; r += blockDim.x >> 4) {
        float v = 0.f;
        for (uint32_t p = lane16; p < npart; p += 16) v += part[r * npart + p];
        v = dpp_add<0x118>(v);  // row_shr:8
        v = dpp_add<0x114>(v);  // row_shr:4
        v = dpp_add<0x112>(v);  // row_shr:2
        v = dpp_add<0x111>(v);  // row_shr:1
        if (lane16 == 15u) ((g_f32wp)out)[row_base + r] = v;
    }
}

// ---------------------------------------------------------------------------
// Per-format pass loops.  `p0..p1` are passes of ONE job; a pass covers rows
// [p*rpp, p*rpp+rpp).  U passes are in flight per thread.
// ---------------------------------------------------------------------------
constexpr int kTilePasses = 16;  // LDS: kTilePasses * rpp rows * npart floats per tile

template <int U>
__device__ __forceinline__ void run_q4k(const GemvJob &j, uint32_t p0, uint32_t p1, float *part) {
    const uint32_t t = threadIdx.x, cpr = j.cpr, rpp = j.rpp;
    const bool active = t < cpr * rpp;
    const uint32_t c = active ? t % cpr : 0, rl = active ? t / cpr : 0;
    const uint32_t sb = c >> 2, g = c & 3, nsb = cpr >> 2;
    Q4KSlice xs;
    q4k_load_x(xs, j.x, c);
    const uint8_t *wbase = j.w + (size_t)sb * 144;
    const size_t row_bytes = j.row_bytes;
    for (uint32_t tp = p0; tp < p1; tp += kTilePasses) {
        const uint32_t tp_end = min(p1, tp + kTilePasses);
        const uint32_t row_base = tp * rpp;
        const uint32_t tile_rows = min((uint32_t)j.rows, tp_end * rpp) - row_base;
        if (active) {
            for (uint32_t lr = rl; lr < tile_rows; lr += rpp * U) {
                u32x4 hdr[U], q0[U], q1[U];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = min(lr + u * rpp, tile_rows - 1) + row_base;
                    g_u4p blk = (g_u4p)(wbase + (size_t)r * row_bytes);
                    hdr[u] = blk[0];
                    q0[u] = blk[1 + 2 * g];
                    q1[u] = blk[2 + 2 * g];
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    float v = q4k_group_dot(hdr[u], q0[u], q1[u], xs, g);
                    v = dpp_add<0xB1>(v);  // quad_perm [1,0,3,2]
                    v = dpp_add<0x4E>(v);  // quad_perm [2,3,0,1]
                    const uint32_t r = lr + u * rpp;
                    if (g == 0 && r < tile_rows) part[r * nsb + sb] = v;
                }
            }
        }
        __syncthreads();
        tile_epilogue(part, nsb, tile_rows, j.out, row_base);
        __syncthreads();
    }
}

template <int U>
__device__ __forceinline__ void run_q8_0(const GemvJob &j, uint32_t p0, uint32_t p1, float *part) {
    const uint32_t t = threadIdx.x, cpr = j.cpr, rpp = j.rpp;
    const bool active = t < cpr * rpp;
    const uint32_t c = active ? t % cpr : 0, rl = active ? t / cpr : 0;
    X32Slice xs;
    load_x32(xs, j.x, c);
    const size_t row_bytes = j.row_bytes;
    for (uint32_t tp = p0; tp < p1; tp += kTilePasses) {
        const uint32_t tp_end = min(p1, tp + kTilePasses);
        const uint32_t row_base = tp * rpp;
        const uint32_t tile_rows = min((uint32_t)j.rows, tp_end * rpp) - row_base;
        if (active) {
            for (uint32_t lr = rl; lr < tile_rows; lr += rpp * U) {
                Q8Raw raw[U];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = min(lr + u * rpp, tile_rows - 1) + row_base;
                    raw[u] = q8_0_load(j.w + (size_t)r * row_bytes, c);
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = lr + u * rpp;
                    const float v = q8_0_block_dot(raw[u], xs, c);
                    if (r < tile_rows) part[r * cpr + c] = v;
                }
            }
        }
        __syncthreads();
        tile_epilogue(part, cpr, tile_rows, j.out, row_base);
        __syncthreads();
    }
}

template <int U>
__device__ __forceinline__ void run_mxfp4(const GemvJob &j, uint32_t p0, uint32_t p1, float *part) {
    const uint32_t t = threadIdx.x, cpr = j.cpr, rpp = j.rpp;
    const bool active = t < cpr * rpp;
    const uint32_t c = active ? t % cpr : 0, rl = active ? t / cpr : 0;
    X32Slice xs;
    load_x32(xs, j.x, c);
    const size_t row_bytes = j.row_bytes;  // packed bytes per row = cpr*16; scale bytes per row = cpr
    for (uint32_t tp = p0; tp < p1; tp += kTilePasses) {
        const uint32_t tp_end = min(p1, tp + kTilePasses);
        const uint32_t row_base = tp * rpp;
        const uint32_t tile_rows = min((uint32_t)j.rows, tp_end * rpp) - row_base;
        if (active) {
            for (uint32_t lr = rl; lr < tile_rows; lr += rpp * U) {
                u32x4 q[U];
                uint32_t sc[U];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = min(lr + u * rpp, tile_rows - 1) + row_base;
                    q[u] = ((g_u4p)(j.w + (size_t)r * row_bytes))[c];
                    sc[u] = ((g_u8p)j.aux)[(size_t)r * cpr + c];
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = lr + u * rpp;
                    const float v = mxfp4_group_dot(q[u], sc[u], xs);
                    if (r < tile_rows) part[r * cpr + c] = v;
                }
            }
        }
        __syncthreads();
        tile_epilogue(part, cpr, tile_rows, j.out, row_base);
        __syncthreads();
    }
}

template <int U>
__device__ __forceinline__ void run_q4_0(const GemvJob &j, uint32_t p0, uint32_t p1, float *part) {
    const uint32_t t = threadIdx.x, cpr = j.cpr, rpp = j.rpp;
    const bool active = t < cpr * rpp;
    const uint32_t c = active ? t % cpr : 0, rl = active ? t / cpr : 0;
    Q8ActSlice xs;
    // for Q4_0 the job's x is the int8 code stream and aux the f32 block scales
    load_q8act(xs, reinterpret_cast<const int8_t *>(j.x), reinterpret_cast<const float *>(j.aux), c);
    const size_t row_bytes = j.row_bytes;
    for (uint32_t tp = p0; tp < p1; tp += kTilePasses) {
        const uint32_t tp_end = min(p1, tp + kTilePasses);
        const uint32_t row_base = tp * rpp;
        const uint32_t tile_rows = min((uint32_t)j.rows, tp_end * rpp) - row_base;
        if (active) {
            for (uint32_t lr = rl; lr < tile_rows; lr += rpp * U) {
                Q40Raw raw[U];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = min(lr + u * rpp, tile_rows - 1) + row_base;
                    raw[u] = q4_0_load(j.w + (size_t)r * row_bytes, c);
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = lr + u * rpp;
                    const float v = q4_0_block_dot(raw[u], xs, c);
                    if (r < tile_rows) part[r * cpr + c] = v;
                }
            }
        }
        __syncthreads();
        tile_epilogue(part, cpr, tile_rows, j.out, row_base);
        __syncthreads();
    }
}

template <int U, int ELEM>  // ELEM: 0 bf16, 1 f16, 2 f32
__device__ __forceinline__ void run_dense(const GemvJob &j, uint32_t p0, uint32_t p1, float *part) {
    const uint32_t t = threadIdx.x, cpr = j.cpr, rpp = j.rpp;
    const bool active = t < cpr * rpp;
    const uint32_t c = active ? t % cpr : 0, rl = active ? t / cpr : 0;
    X16Slice xs;
    load_x16(xs, j.x, c);
    const size_t row_bytes = j.row_bytes;
    constexpr int VECS = ELEM == 2 ? 4 : 2;  // 16-byte vectors per 16 elements
    for (uint32_t tp = p0; tp < p1; tp += kTilePasses) {
        const uint32_t tp_end = min(p1, tp + kTilePasses);
        const uint32_t row_base = tp * rpp;
        const uint32_t tile_rows = min((uint32_t)j.rows, tp_end * rpp) - row_base;
        if (active) {
            for (uint32_t lr = rl; lr < tile_rows; lr += rpp * U) {
                u32x4 v[U][VECS];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = min(lr + u * rpp, tile_rows - 1) + row_base;
                    g_u4p p = (g_u4p)(j.w + (size_t)r * row_bytes) + (size_t)c * VECS;
#pragma unroll
                    for (int k = 0; k < VECS; k++) v[u][k] = p[k];
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = lr + u * rpp;
                    float d;
                    if (ELEM == 0) d = bf16x16_dot(v[u][0], v[u][1], xs);
                    else if (ELEM == 1) d = f16x16_dot(v[u][0], v[u][1], xs);
                    else d = f32x16_dot(reinterpret_cast<const f32x4 *>(&v[u][0]), xs);
                    if (r < tile_rows) part[r * cpr + c] = d;
                }
            }
        }
        __syncthreads();
        tile_epilogue(part, cpr, tile_rows, j.out, row_base);
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------
// The kernels, one per format so each gets its own register budget: workgroup
// b sweeps passes [P*b/G, P*(b+1)/G) of the launch's pass list, job by job.
// ---------------------------------------------------------------------------
template <int KIND, int U>
__device__ __forceinline__ void gemv_body(const GemvLaunch &L, float *part) {
    const GemvJob *jobs = L.table ? L.table : L.inl;
    const uint64_t P = L.total_passes;
    uint32_t p = (uint32_t)(P * blockIdx.x / gridDim.x);
    const uint32_t p_end = (uint32_t)(P * (blockIdx.x + 1) / gridDim.x);
    // first job whose pass range ends after p
    uint32_t lo = 0, hi = L.n_jobs;
    while (lo + 1 < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (jobs[mid].pass_begin <= p) lo = mid; else hi = mid;
    }
    uint32_t ji = lo;
    while (p < p_end) {
        GemvJob j = jobs[ji];
        if (j.sel) {  // run-time expert selection: one bank of equally shaped matrices
            const uint32_t e = __builtin_amdgcn_readfirstlane(*(const GLOBAL_AS uint32_t *)j.sel);
            j.w += (size_t)e * j.w_sel_stride;
            j.aux += (size_t)e * j.aux_sel_stride;
        }
        const uint32_t jp_end = j.pass_begin + j.n_pass;
        const uint32_t seg_end = min(p_end, jp_end);
        const uint32_t a = p - j.pass_begin, b = seg_end - j.pass_begin;
        if (KIND == KIND_Q4K) run_q4k<U>(j, a, b, part);
        else if (KIND == KIND_Q8_0) run_q8_0<U>(j, a, b, part);
        else if (KIND == KIND_MXFP4) run_mxfp4<U>(j, a, b, part);
        else if (KIND == KIND_Q4_0) run_q4_0<U>(j, a, b, part);
        else if (KIND == KIND_BF16) run_dense<U, 0>(j, a, b, part);
        else if (KIND == KIND_F16) run_dense<U, 1>(j, a, b, part);
        else run_dense<U, 2>(j, a, b, part);
        p = seg_end;
        ji++;
    }
}

#define LARQL_GEMV_KERNEL(NAME, KIND, U, WAVES)                                                                 \
    __global__ void __launch_bounds__(kGemvMaxThreads) __attribute__((amdgpu_waves_per_eu(WAVES))) NAME(GemvLaunch L) { \
        extern __shared__ float part[];                                                                         \
        gemv_body<KIND, U>(L, part);                                                                            \
    }
LARQL_GEMV_KERNEL(gemv_q4k_u2_kernel, KIND_Q4K, 2, 4)
LARQL_GEMV_KERNEL(gemv_q4k_u4_kernel, KIND_Q4K, 4, 3)
LARQL_GEMV_KERNEL(gemv_q8_0_u2_kernel, KIND_Q8_0, 2, 4)
LARQL_GEMV_KERNEL(gemv_q8_0_u4_kernel, KIND_Q8_0, 4, 3)
LARQL_GEMV_KERNEL(gemv_mxfp4_u2_kernel, KIND_MXFP4, 2, 4)
LARQL_GEMV_KERNEL(gemv_mxfp4_u4_kernel, KIND_MXFP4, 4, 4)
LARQL_GEMV_KERNEL(gemv_q4_0_kernel, KIND_Q4_0, 4, 4)
LARQL_GEMV_KERNEL(gemv_bf16_kernel, KIND_BF16, 4, 4)
LARQL_GEMV_KERNEL(gemv_f16_kernel, KIND_F16, 4, 4)
LARQL_GEMV_KERNEL(gemv_f32_kernel, KIND_F32, 2, 4)


// ---------------------------------------------------------------------------
// Host side: geometry and launch.
// ---------------------------------------------------------------------------
// experiment knobs (environment): passes in flight per thread, forced block size
static int g_unroll = getenv("LARQL_HIP_UNROLL") ? atoi(getenv("LARQL_HIP_UNROLL")) : 0;  // 0: per-format default
static int g_threads = getenv("LARQL_HIP_THREADS") ? atoi(getenv("LARQL_HIP_THREADS")) : 0;
static uint32_t chunk_elems(int kind) {
    switch (kind) {
        case KIND_Q4K: return 64;
        case KIND_Q8_0: case KIND_MXFP4: case KIND_Q4_0: return 32;
        default: return 16;
    }
}

bool gemv_job_geometry(GemvJob &j, uint32_t threads) {
    const uint32_t ce = chunk_elems(j.kind);
    if (j.k == 0 || j.k % ce != 0) return false;
    const uint64_t cpr = j.k / ce;
    if (cpr > threads) return false;
    j.cpr = (uint32_t)cpr;
    j.rpp = threads / j.cpr;
    switch (j.kind) {
        case KIND_Q4K: j.row_bytes = (j.k / 256) * 144; break;
        case KIND_Q8_0: j.row_bytes = (j.k / 32) * 34; break;
        case KIND_MXFP4: j.row_bytes = (j.k / 32) * 16; break;
        case KIND_Q4_0: j.row_bytes = (j.k / 32) * 18; break;
        case KIND_BF16: case KIND_F16: j.row_bytes = j.k * 2; break;
        case KIND_F32: j.row_bytes = j.k * 4; break;
        default: return false;
    }
    const uint64_t n_pass = (j.rows + j.rpp - 1) / j.rpp;
    if (n_pass > 0x7FFFFFFFull) return false;
    j.n_pass = (uint32_t)n_pass;
    return true;
}

uint32_t gemv_pick_threads(const GemvJob *jobs, size_t n) {
    // Prefer the block size that wastes the fewest lanes over the jobs'
    // chunk counts (weighted by bytes); ties go to the smaller block.
    static const uint32_t cand_all[] = {256, 320, 384, 448, 512};
    const uint32_t forced[] = {(uint32_t)g_threads};
    const uint32_t *cand = g_threads ? forced : cand_all;
    const size_t n_cand = g_threads ? 1 : 5;
    double best = -1.0;
    uint32_t pick = 0;
    for (size_t ci = 0; ci < n_cand; ci++) {
        const uint32_t T = cand[ci];
        double used = 0.0, total = 0.0;
        bool ok = true;
        for (size_t i = 0; i < n; i++) {
            const uint64_t cpr = jobs[i].k / chunk_elems(jobs[i].kind);
            if (cpr == 0 || cpr > T) { ok = false; break; }
            const double wgt = (double)jobs[i].rows * (double)jobs[i].k;
            used += wgt * (double)((T / cpr) * cpr) / (double)T;
            total += wgt;
        }
        if (!ok) continue;
        const double eff = total > 0 ? used / total : 1.0;
        if (eff > best + 1e-9) { best = eff; pick = T; }
    }
    return pick;
}

size_t gemv_lds_bytes(const GemvJob *jobs, size_t n) {
    size_t m = 0;
    for (size_t i = 0; i < n; i++) {
        const size_t npart = jobs[i].kind == KIND_Q4K ? jobs[i].cpr / 4 : jobs[i].cpr;
        const size_t b = (size_t)kTilePasses * jobs[i].rpp * npart * sizeof(float);
        if (b > m) m = b;
    }
    return m;
}

hipError_t gemv_launch(hipStream_t stream, int kind, const GemvLaunch &L, uint32_t threads, uint32_t grid, size_t lds) {
    switch (kind) {
        case KIND_Q4K:
            if (g_unroll != 4) hipLaunchKernelGGL(gemv_q4k_u2_kernel, dim3(grid), dim3(threads), lds, stream, L);
            else hipLaunchKernelGGL(gemv_q4k_u4_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        case KIND_Q8_0:
            if (g_unroll == 2) hipLaunchKernelGGL(gemv_q8_0_u2_kernel, dim3(grid), dim3(threads), lds, stream, L);
            else hipLaunchKernelGGL(gemv_q8_0_u4_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        case KIND_MXFP4:
            if (g_unroll == 2) hipLaunchKernelGGL(gemv_mxfp4_u2_kernel, dim3(grid), dim3(threads), lds, stream, L);
            else hipLaunchKernelGGL(gemv_mxfp4_u4_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        case KIND_Q4_0: hipLaunchKernelGGL(gemv_q4_0_kernel, dim3(grid), dim3(threads), lds, stream, L); break;
        case KIND_BF16: hipLaunchKernelGGL(gemv_bf16_kernel, dim3(grid), dim3(threads), lds, stream, L); break;
        case KIND_F16: hipLaunchKernelGGL(gemv_f16_kernel, dim3(grid), dim3(threads), lds, stream, L); break;
        case KIND_F32: hipLaunchKernelGGL(gemv_f32_kernel, dim3(grid), dim3(threads), lds, stream, L); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// Plain streaming copy (one 16-byte load and store per thread per step): the
// yardstick for achievable HBM bandwidth and for scaling profiler counters.
__global__ void __launch_bounds__(256) copy_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, size_t n_vec) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += stride) dst[i] = src[i];
}
__global__ void __launch_bounds__(256) read_kernel(const u32x4 *__restrict__ src, uint32_t *__restrict__ sink, size_t n_vec) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    uint32_t acc = 0;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += stride) {
        const u32x4 v = src[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9E3779B9u) sink[0] = acc;  // keeps the loads alive; practically never true
}
hipError_t copy_launch(hipStream_t stream, const void *src, void *dst, size_t bytes, uint32_t grid) {
    if (dst) hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(256), 0, stream, (const u32x4 *)src, (u32x4 *)dst, bytes / 16);
    return hipGetLastError();
}
hipError_t read_launch(hipStream_t stream, const void *src, uint32_t *sink, size_t bytes, uint32_t grid) {
    hipLaunchKernelGGL(read_kernel, dim3(grid), dim3(256), 0, stream, (const u32x4 *)src, sink, bytes / 16);
    return hipGetLastError();
}

}  // namespace larql
