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
#include <cstddef>

#include <atomic>
#include <stdint.h>
#include <stdlib.h>

#include <algorithm>

#include "kernels.h"
#include "router.h"

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

// max of a non-negative value over the wavefront, the same in every lane: four steps inside the rows of 16 lanes
// and two row broadcasts (data-parallel primitives, a few cycles each; cross-lane shuffles go through LDS hardware
// and cost a round trip each), then lane 63 holds the result
__device__ __forceinline__ float wave_max_nonneg(float v) {
    int m = __builtin_bit_cast(int, v);  // (non-negative floats order like their bit patterns)
    m = max(m, __builtin_amdgcn_update_dpp(0, m, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    m = max(m, __builtin_amdgcn_update_dpp(0, m, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    m = max(m, __builtin_amdgcn_update_dpp(0, m, 0x141, 0xF, 0xF, true));  // row_half_mirror
    m = max(m, __builtin_amdgcn_update_dpp(0, m, 0x140, 0xF, 0xF, true));  // row_mirror
    m = max(m, __builtin_amdgcn_update_dpp(0, m, 0x142, 0xA, 0xF, false)); // row_bcast:15 into rows 1 and 3
    m = max(m, __builtin_amdgcn_update_dpp(0, m, 0x143, 0xC, 0xF, false)); // row_bcast:31 into rows 2 and 3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(m, 63));
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

struct Q8Raw { uint32_t d[9]; bool odd; };

// `blk` is the block's index in the whole matrix (row * blocks_per_row + c): with an odd number of blocks per row the
// rows themselves alternate between 4-byte and 2-byte alignment, so the parity is the matrix-wide one.
__device__ __forceinline__ Q8Raw q8_0_load(const uint8_t *base, uint64_t blk) {
    // block `blk` starts at 34*blk; the aligned window starts there (even) or 2 bytes earlier (odd)
    Q8Raw r;
    r.odd = (blk & 1u) != 0;
    const uint8_t *b = base + blk * 34 - (r.odd ? 2u : 0u);
    g_u32p p = (g_u32p)b;
#pragma unroll
    for (int i = 0; i < 8; i++) r.d[i] = p[i];
    // an even block's last two codes are half a dword: a 16-bit read, so the last block of a buffer is not overrun
    r.d[8] = r.odd ? p[8] : (uint32_t)*(const GLOBAL_AS uint16_t *)(b + 32);
    return r;
}

__device__ __forceinline__ float q8_0_block_dot(const Q8Raw &r, const X32Slice &s) {
    const bool odd = r.odd;
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
// Q6_K (K-slice kernel): one thread = one 32-byte row of ql of one 128-element half of a 210-byte
// super-block, i.e. 64 weights: the low nibbles are plane r (elements r*32 .. r*32+31 of the half), the
// high nibbles plane r+2; qh of the half carries their two top bits at shifts 2r and 2r+4
// (q6k_subblock_vals, larql-models/src/quant/ggml/q6_k.rs:19-40).  Value per row as q6k_matvec
// (larql-compute/src/cpu/ops/q6k_matvec.rs:45-91): sum over 16-element sub-blocks of (d*scale) * sum (q-32)*x,
// with the -32 taken out through the sub-block sums of x.  Blocks are only 2-byte aligned: every field is read as
// the aligned dwords that cover it and shifted into place (v_alignbit).
// ---------------------------------------------------------------------------
struct Q6KSlice {
    float x[64];     // plane r (32), then plane r+2 (32)
    float sum[4];    // sums of x over the four 16-element sub-blocks, in that order
};

__device__ __forceinline__ void q6k_load_x(Q6KSlice &s, const float *x, uint32_t c) {
    const uint32_t sb = c >> 2, h = (c >> 1) & 1u, r = c & 1u;
    g_f4p lo = (g_f4p)(x + (size_t)sb * 256 + h * 128 + r * 32);
    g_f4p hi = (g_f4p)(x + (size_t)sb * 256 + h * 128 + (r + 2) * 32);
    float sm[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const f32x4 a = lo[i], b = hi[i];
        s.x[4 * i + 0] = a.x; s.x[4 * i + 1] = a.y; s.x[4 * i + 2] = a.z; s.x[4 * i + 3] = a.w;
        s.x[32 + 4 * i + 0] = b.x; s.x[32 + 4 * i + 1] = b.y; s.x[32 + 4 * i + 2] = b.z; s.x[32 + 4 * i + 3] = b.w;
        sm[i >> 2] += (a.x + a.y) + (a.z + a.w);
        sm[2 + (i >> 2)] += (b.x + b.y) + (b.z + b.w);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) s.sum[i] = sm[i];
}

struct Q6KRaw { uint32_t ql[9], qh[9], sc[2], d; };

// 32 bytes starting at the 2-byte-aligned address p, as the 9 aligned dwords that cover them
__device__ __forceinline__ void load9(uint32_t (&dst)[9], const uint8_t *p) {
    g_u32p a = (g_u32p)((uintptr_t)p & ~(uintptr_t)3);
#pragma unroll
    for (int i = 0; i < 9; i++) dst[i] = a[i];
}

__device__ __forceinline__ Q6KRaw q6k_load(const uint8_t *row, uint32_t c) {
    const uint32_t sb = c >> 2, h = (c >> 1) & 1u, r = c & 1u;
    const uint8_t *blk = row + (size_t)sb * 210;
    Q6KRaw raw;
    load9(raw.ql, blk + h * 64 + r * 32);
    load9(raw.qh, blk + 128 + h * 32);
    g_u32p sp = (g_u32p)((uintptr_t)(blk + 192 + h * 8 + 2 * r) & ~(uintptr_t)3);  // scales 2r, 2r+1 and 2r+4, 2r+5 of the half
    raw.sc[0] = sp[0]; raw.sc[1] = sp[1];  // the six bytes needed start at most 2 bytes into this window
    raw.d = *(const GLOBAL_AS uint16_t *)(blk + 208);
    return raw;
}

__device__ __forceinline__ float q6k_chunk_dot(const Q6KRaw &raw, const Q6KSlice &s, const uint8_t *row, uint32_t c) {
    const uint32_t sb = c >> 2, r = c & 1u;
    // all fields of a block share the block's misalignment (0 or 2 bytes): block offset sb*210 on a 4-byte aligned row
    const uint32_t mis = (uint32_t)(((uintptr_t)row + (size_t)sb * 210) & 2u), sh = mis * 8;
    const float d = half_bits_to_float(raw.d);
    // scale bytes: 8 bytes from (block + 192 + h*8 + 2r): parity of (mis + 2r)
    const uint32_t ssh = ((mis + 2 * r) & 2u) * 8;
    const uint32_t s01 = __builtin_amdgcn_alignbit(raw.sc[1], raw.sc[0], ssh), s45 = raw.sc[1] >> ssh;
    const float sc0 = (float)(int)(int8_t)(s01 & 0xFF), sc1 = (float)(int)(int8_t)((s01 >> 8) & 0xFF);
    const float sc2 = (float)(int)(int8_t)(s45 & 0xFF), sc3 = (float)(int)(int8_t)((s45 >> 8) & 0xFF);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    const uint32_t hs = 2 * r;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t ql = __builtin_amdgcn_alignbit(raw.ql[i + 1], raw.ql[i], sh);
        const uint32_t qh = __builtin_amdgcn_alignbit(raw.qh[i + 1], raw.qh[i], sh);
        const uint32_t a = (ql & 0x0F0F0F0Fu) | (((qh >> hs) & 0x03030303u) << 4);              // plane r, elements 4i..4i+3
        const uint32_t b = ((ql >> 4) & 0x0F0F0F0Fu) | (((qh >> (hs + 4)) & 0x03030303u) << 4);  // plane r+2
        float &al = acc[i >> 2], &bh = acc[2 + (i >> 2)];
        al = __builtin_fmaf((float)(a & 0xFFu), s.x[4 * i + 0], al);
        al = __builtin_fmaf((float)((a >> 8) & 0xFFu), s.x[4 * i + 1], al);
        al = __builtin_fmaf((float)((a >> 16) & 0xFFu), s.x[4 * i + 2], al);
        al = __builtin_fmaf((float)(a >> 24), s.x[4 * i + 3], al);
        bh = __builtin_fmaf((float)(b & 0xFFu), s.x[32 + 4 * i + 0], bh);
        bh = __builtin_fmaf((float)((b >> 8) & 0xFFu), s.x[32 + 4 * i + 1], bh);
        bh = __builtin_fmaf((float)((b >> 16) & 0xFFu), s.x[32 + 4 * i + 2], bh);
        bh = __builtin_fmaf((float)(b >> 24), s.x[32 + 4 * i + 3], bh);
    }
    float v = sc0 * (acc[0] - 32.0f * s.sum[0]);
    v += sc1 * (acc[1] - 32.0f * s.sum[1]);
    v += sc2 * (acc[2] - 32.0f * s.sum[2]);
    v += sc3 * (acc[3] - 32.0f * s.sum[3]);
    return d * v;
}

// Q6_K against a Q8_K activation (q6k_q8k_matvec_scalar, larql-compute/src/cpu/ops/q4k_q8k_dot/q6k.rs:38-92): the same
// 64-weight chunk per thread, but the activation is int8: the 6-bit codes (0..63) meet the codes of x in v_dot4_i32_i8,
// the -32 goes through the sums of x's codes per 16-element group, and the four chunks of a super-block (four
// neighbouring lanes) add their integer sums so that one of them can evaluate d_w*d_y*(f32)sum1 as the reference does.
struct Q6KQ8Slice {
    uint32_t y[16];  // codes of plane r (8 dwords), then plane r+2
    int ysum[4];     // sums of the codes over the four 16-element groups, in that order
    float dy;
};

__device__ __forceinline__ void q6k_q8k_load_x(Q6KQ8Slice &s, const uint8_t *q8k, uint32_t k, uint32_t c) {
    const uint32_t sb = c >> 2, h = (c >> 1) & 1u, r = c & 1u;
    g_u4p lo = (g_u4p)(q8k + (size_t)sb * 256 + h * 128 + r * 32);
    g_u4p hi = (g_u4p)(q8k + (size_t)sb * 256 + h * 128 + (r + 2) * 32);
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const u32x4 a = lo[i], b = hi[i];
        s.y[4 * i + 0] = a.x; s.y[4 * i + 1] = a.y; s.y[4 * i + 2] = a.z; s.y[4 * i + 3] = a.w;
        s.y[8 + 4 * i + 0] = b.x; s.y[8 + 4 * i + 1] = b.y; s.y[8 + 4 * i + 2] = b.z; s.y[8 + 4 * i + 3] = b.w;
    }
#pragma unroll
    for (int g = 0; g < 4; g++) {
        int sm = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) sm = __builtin_amdgcn_sdot4(0x01010101, (int)s.y[4 * g + i], sm, false);
        s.ysum[g] = sm;
    }
    s.dy = *(const GLOBAL_AS float *)(q8k + k + (size_t)sb * 4);
}

// this chunk's integer share of its super-block's sum1
__device__ __forceinline__ int q6k_q8k_chunk(const Q6KRaw &raw, const Q6KQ8Slice &s, const uint8_t *row, uint32_t c) {
    const uint32_t sb = c >> 2, r = c & 1u;
    const uint32_t mis = (uint32_t)(((uintptr_t)row + (size_t)sb * 210) & 2u), sh = mis * 8;
    const uint32_t ssh = ((mis + 2 * r) & 2u) * 8;
    const uint32_t s01 = __builtin_amdgcn_alignbit(raw.sc[1], raw.sc[0], ssh), s45 = raw.sc[1] >> ssh;
    const int sc0 = (int)(int8_t)(s01 & 0xFF), sc1 = (int)(int8_t)((s01 >> 8) & 0xFF);
    const int sc2 = (int)(int8_t)(s45 & 0xFF), sc3 = (int)(int8_t)((s45 >> 8) & 0xFF);
    int acc[4] = {0, 0, 0, 0};
    const uint32_t hs = 2 * r;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t ql = __builtin_amdgcn_alignbit(raw.ql[i + 1], raw.ql[i], sh);
        const uint32_t qh = __builtin_amdgcn_alignbit(raw.qh[i + 1], raw.qh[i], sh);
        const uint32_t a = (ql & 0x0F0F0F0Fu) | (((qh >> hs) & 0x03030303u) << 4);              // plane r, elements 4i..4i+3
        const uint32_t b = ((ql >> 4) & 0x0F0F0F0Fu) | (((qh >> (hs + 4)) & 0x03030303u) << 4);  // plane r+2
        acc[i >> 2] = __builtin_amdgcn_sdot4((int)a, (int)s.y[i], acc[i >> 2], false);          // codes <= 63: positive as int8
        acc[2 + (i >> 2)] = __builtin_amdgcn_sdot4((int)b, (int)s.y[8 + i], acc[2 + (i >> 2)], false);
    }
    // |sum (q-32)*y| <= 16*32*127 over a group: the products with the int8 scales fit 24-bit multiplies
    return __mul24(sc0, acc[0] - 32 * s.ysum[0]) + __mul24(sc1, acc[1] - 32 * s.ysum[1]) +
           __mul24(sc2, acc[2] - 32 * s.ysum[2]) + __mul24(sc3, acc[3] - 32 * s.ysum[3]);
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

struct Q40Raw { uint32_t d[5]; bool odd; };

// `blk` is the block's index in the whole matrix, as for q8_0_load.
__device__ __forceinline__ Q40Raw q4_0_load(const uint8_t *base, uint64_t blk) {
    // block `blk` at 18*blk: 4-byte aligned when even, else the window starts 2 bytes earlier
    Q40Raw r;
    r.odd = (blk & 1u) != 0;
    const uint8_t *b = base + blk * 18 - (r.odd ? 2u : 0u);
    g_u32p p = (g_u32p)b;
#pragma unroll
    for (int i = 0; i < 4; i++) r.d[i] = p[i];
    r.d[4] = r.odd ? p[4] : (uint32_t)*(const GLOBAL_AS uint16_t *)(b + 16);
    return r;
}

__device__ __forceinline__ float q4_0_block_dot(const Q40Raw &r, const Q8ActSlice &s) {
    const bool odd = r.odd;
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
                                              float *out, uint32_t row_base, const float *bias = nullptr, uint32_t bias_step = 1) {
    const uint32_t lane16 = threadIdx.x & 15u;
    for (uint32_t r = threadIdx.x >> 4; r < tile_rows; r += blockDim.x >> 4) {
        float v = 0.f;
        for (uint32_t p = lane16; p < npart; p += 16) v += part[r * npart + p];
        v = dpp_add<0x118>(v);  // row_shr:8
        v = dpp_add<0x114>(v);  // row_shr:4
        v = dpp_add<0x112>(v);  // row_shr:2
        v = dpp_add<0x111>(v);  // row_shr:1
        if (lane16 == 15u) {
            if (bias) v += ((const GLOBAL_AS float *)bias)[(size_t)(row_base + r) * bias_step];
            ((g_f32wp)out)[row_base + r] = v;
        }
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

// ---------------------------------------------------------------------------
// Q4_K on the matrix cores (rows of up to 48 super-blocks).
//
// A wavefront owns one super-block column c of a job and walks down the rows
// 16 at a time.  Its 16 x 144 bytes of a tile stream global -> LDS directly
// (global_load_lds, 16 bytes per lane, no VGPRs) into a private ring kQ4kStages
// deep, so the bytes in flight are bounded by LDS, not by registers or
// occupancy, and no wavefront ever waits for another one's loads.
//
// The dot products run on v_mfma_i32_16x16x64_i8, exactly, with the roles
// swapped: the 16 "B" columns are the 16 weight rows of the tile and the "A"
// rows carry the activation.  Per 256-wide column, x is scaled by a power of
// two to 28-bit integers n = rint(x * 2^(27-e)) (2^e > max|x|) and n is split
// into four balanced base-128 digits (int8 "limbs"); A row 4g + 2cl + i holds
// limb i (first operand set) or limb 2+i (second set) of sub-block 2g+cl in
// the k-slots that the sub-block's nibbles occupy in B, zero elsewhere.  Lane
// (row j = lane%16, kq = lane/16) supplies, per 32-byte group, the low nibbles
// of its bytes 8kq..8kq+7 in k-slots 0-7 and the high nibbles in slots 8-15
// (three mask/shift instructions per 8 weights) and, after two MFMAs per group,
// holds for weight row j and group g = kq the eight exact integer sums
// nibbles.limb — it is the very lane that decodes that group's two scales and
// mins from the header.  The limb sums are recombined in f32 (the only
// rounding besides the final scale), so the result differs from an f32 FMA
// chain over exact products only by the 2^-28 relative quantum of x.
// Value per row as q4k_matvec_into (larql-compute/src/cpu/ops/q4_common/
// matvec_f32.rs:116-155): sum over sub-blocks of (d*sc)*dot(q,x) - (dmin*mn)*sum(x).
//
// Rows longer than the workgroup has wavefronts are covered in up to 4 column
// passes per tile (wave w owns columns w, w+nw, ...), summed in registers.
// Row partials meet in LDS every kQ4kBatchTiles tiles: part[row][wave*4 + g],
// folded in a fixed order that depends only on the row length.
// ---------------------------------------------------------------------------
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void *lds_vp;
typedef const GLOBAL_AS void *g_vp;
union Q4kOp { i32x4 v; uint32_t u[4]; };  // one MFMA operand: 16 int8 k-slots of a lane

constexpr int kQ4kStages = 4;      // wave-tiles in flight per wavefront (ring slots of 2304 B)
constexpr int kQ4kBatchTiles = 4;  // 16-row tiles between two folds of the row partials
constexpr int kQ4kMaxColPasses = 4;
constexpr int kQ4kMaxWaves = 10;  // with the ring, the partials and 4 prepared columns per wavefront this fills the 160 KB of LDS
constexpr uint32_t kQ4kTileBytes = 16 * 144;
constexpr uint32_t kQ4kColBytes = 1024 + 64;  // a column's activation limbs for 64 lanes, then {k, -, -, -, sums of 8 sub-blocks}

// s_waitcnt vmcnt(n), n < 64, leaving the other counters alone (gfx9 encoding)
#define LARQL_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

struct Q4kCol {
    uint32_t xq[4];        // this lane's 8 activations as int8 limbs: {limb i: 2 dwords, limb 2+i: 2 dwords}, i = lane & 1
    float k;               // 2^(e-27): integer dot -> value
    float sum_lo, sum_hi;  // sum of x over sub-blocks 2kq and 2kq+1
};

// A column's activations as loaded
struct Q4kRaw { f32x4 v, a, b; };

__device__ __forceinline__ Q4kRaw q4k_mfma_load_col(const float *x, uint32_t c, uint32_t lane) {
    // A-operand row j = 4g + 2cl + i feeds sub-block m = j/2 = 2g+cl: elements 8kq..8kq+7 of it
    const uint32_t j = lane & 15u, kq = lane >> 4, m = j >> 1;
    g_f4p xc = (g_f4p)(x + (size_t)c * 256);
    g_f4p xs = (g_f4p)(x + (size_t)c * 256 + m * 32 + 8 * kq);
    Q4kRaw r;
    r.v = xc[lane];  // 4 consecutive activations per lane: column max and per-sub-block sums (8 lanes each)
    r.a = xs[0];
    r.b = xs[1];
    return r;
}

__device__ __forceinline__ Q4kCol q4k_mfma_finish_col(const Q4kRaw &r, uint32_t lane) {
    const uint32_t j = lane & 15u, kq = lane >> 4;
    float mx = wave_max_nonneg(fmaxf(fmaxf(fabsf(r.v.x), fabsf(r.v.y)), fmaxf(fabsf(r.v.z), fabsf(r.v.w))));
    float sm = (r.v.x + r.v.y) + (r.v.z + r.v.w);
    // sum over the 8 lanes of a sub-block: the exchange pattern of a butterfly (partners 1, 2, 4 lanes away), by DPP
    sm = dpp_add<0xB1>(sm);   // quad_perm [1,0,3,2]
    sm = dpp_add<0x4E>(sm);   // quad_perm [2,3,0,1]
    sm = dpp_add<0x141>(sm);  // row_half_mirror: the other quad of the eight
    Q4kCol col;
    {   // sub-block m's sum sits in lanes 8m .. 8m+7; this lane wants sub-blocks 2kq and 2kq+1
        float sb[8];
#pragma unroll
        for (int m = 0; m < 8; m++) sb[m] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sm), 8 * m));
        col.sum_lo = kq == 0 ? sb[0] : (kq == 1 ? sb[2] : (kq == 2 ? sb[4] : sb[6]));
        col.sum_hi = kq == 0 ? sb[1] : (kq == 1 ? sb[3] : (kq == 2 ? sb[5] : sb[7]));
    }
    int ex = 0;
    if (mx > 0.f && mx < __builtin_inff()) (void)frexpf(mx, &ex);  // mx = f * 2^ex, f in [0.5, 1)
    ex = max(-90, min(120, ex));
    const float to_int = ldexpf(1.f, 27 - ex);  // |x| * to_int < 2^27
    col.k = ldexpf(1.f, ex - 27);
    const float e[8] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w};
    const uint32_t i = j & 1u;
    uint32_t la[8], lb[8];  // limbs i and 2+i of the 8 elements, as unsigned bytes
#pragma unroll
    for (int t = 0; t < 8; t++) {
        // n = l0*128^3 + l1*128^2 + l2*128 + l3 with l1..l3 in [-64, 63], l0 in [-64, 64]
        const int n = (int)__builtin_rintf(e[t] * to_int);
        const int l3 = ((n + 64) & 127) - 64, n1 = (n - l3) >> 7;
        const int l2 = ((n1 + 64) & 127) - 64, n2 = (n1 - l2) >> 7;
        const int l1 = ((n2 + 64) & 127) - 64, l0 = (n2 - l1) >> 7;
        la[t] = (uint32_t)(i ? l1 : l0) & 0xFFu;
        lb[t] = (uint32_t)(i ? l3 : l2) & 0xFFu;
    }
    col.xq[0] = la[0] | (la[1] << 8) | (la[2] << 16) | (la[3] << 24);
    col.xq[1] = la[4] | (la[5] << 8) | (la[6] << 16) | (la[7] << 24);
    col.xq[2] = lb[0] | (lb[1] << 8) | (lb[2] << 16) | (lb[3] << 24);
    col.xq[3] = lb[4] | (lb[5] << 8) | (lb[6] << 16) | (lb[7] << 24);
    return col;
}

// xm[2g] / xm[2g+1]: A operands (limbs 0,1 / limbs 2,3) of the MFMAs of group g.  A lane is non-zero only in
// its own group (j/4) and only in the k-slots of its sub-block's nibbles: 0-7 (low, cl = 0) or 8-15 (high).
__device__ __forceinline__ void q4k_mfma_operands(Q4kOp (&xm)[8], const Q4kCol &col, uint32_t j) {
    const uint32_t my_g = j >> 2, cl = (j >> 1) & 1u;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const bool lo = my_g == (uint32_t)g && cl == 0, hi = my_g == (uint32_t)g && cl == 1;
        xm[2 * g].u[0] = lo ? col.xq[0] : 0u; xm[2 * g].u[1] = lo ? col.xq[1] : 0u;
        xm[2 * g].u[2] = hi ? col.xq[0] : 0u; xm[2 * g].u[3] = hi ? col.xq[1] : 0u;
        xm[2 * g + 1].u[0] = lo ? col.xq[2] : 0u; xm[2 * g + 1].u[1] = lo ? col.xq[3] : 0u;
        xm[2 * g + 1].u[2] = hi ? col.xq[2] : 0u; xm[2 * g + 1].u[3] = hi ? col.xq[3] : 0u;
    }
}

// one wave-tile from its LDS slot: 16 rows x one super-block against the column's activations
__device__ __forceinline__ float q4k_mfma_tile(const uint8_t *slot, const Q4kOp (&xm)[8], const Q4kCol &col, uint32_t j, uint32_t kq) {
    const uint8_t *sp = slot + j * 144;
    const u32x4 hdr = *reinterpret_cast<const u32x4 *>(sp);
    u32x2 q[4];
#pragma unroll
    for (int g = 0; g < 4; g++) q[g] = *reinterpret_cast<const u32x2 *>(sp + 16 + 32 * g + 8 * kq);
    i32x4 Da = {0, 0, 0, 0}, Db = {0, 0, 0, 0};
#pragma unroll
    for (int g = 0; g < 4; g++) {
        Q4kOp b;
        b.u[0] = q[g].x & 0x0F0F0F0Fu; b.u[1] = q[g].y & 0x0F0F0F0Fu;
        b.u[2] = (q[g].x >> 4) & 0x0F0F0F0Fu; b.u[3] = (q[g].y >> 4) & 0x0F0F0F0Fu;
        Da = __builtin_amdgcn_mfma_i32_16x16x64_i8(xm[2 * g].v, b.v, Da, 0, 0, 0);
        Db = __builtin_amdgcn_mfma_i32_16x16x64_i8(xm[2 * g + 1].v, b.v, Db, 0, 0, 0);
    }
    // this lane's group is g = kq.  Da = [lo.l0, lo.l1, hi.l0, hi.l1], Db = [lo.l2, lo.l3, hi.l2, hi.l3]
    float dot_lo = __builtin_fmaf((float)Da[0], 128.f, (float)Da[1]);
    float dot_hi = __builtin_fmaf((float)Da[2], 128.f, (float)Da[3]);
    dot_lo = __builtin_fmaf(dot_lo, 128.f, (float)Db[0]);
    dot_hi = __builtin_fmaf(dot_hi, 128.f, (float)Db[2]);
    dot_lo = __builtin_fmaf(dot_lo, 128.f, (float)Db[1]) * col.k;
    dot_hi = __builtin_fmaf(dot_hi, 128.f, (float)Db[3]) * col.k;
    // header fields as get_scale_min_k4 (matvec_f32.rs:124-131), two bytes at a time
    const float d = half_bits_to_float(hdr.x & 0xFFFFu), dmin = half_bits_to_float(hdr.x >> 16);
    const uint32_t sh = (kq & 1u) * 16u;
    const uint32_t a = (hdr.y >> sh) & 0xFFFFu, b = (hdr.z >> sh) & 0xFFFFu, c = (hdr.w >> sh) & 0xFFFFu;
    const uint32_t sc_hi2 = (c & 0x0F0Fu) | ((a >> 2) & 0x3030u), mn_hi2 = ((c >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u);
    const uint32_t sc2 = kq < 2 ? (a & 0x3F3Fu) : sc_hi2, mn2 = kq < 2 ? (b & 0x3F3Fu) : mn_hi2;
    const float sc_lo = d * (float)(sc2 & 0xFFu), sc_hi = d * (float)(sc2 >> 8);
    const float mn_lo = dmin * (float)(mn2 & 0xFFu), mn_hi = dmin * (float)(mn2 >> 8);
    float r = sc_lo * dot_lo - mn_lo * col.sum_lo;
    r += sc_hi * dot_hi - mn_hi * col.sum_hi;
    return r;
}

// tiles [tile_a, tile_b) of one job; `parity` flips per batch (double-buffered partials)
__device__ __forceinline__ void run_q4k_mfma(const GemvJob &j, uint32_t tile_a, uint32_t tile_b, uint8_t *lds, uint32_t &parity) {
    constexpr int NS = kQ4kStages, R = kQ4kBatchTiles;
    const uint32_t lane = threadIdx.x & 63u, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nw_launch = blockDim.x >> 6;
    const uint32_t jr = lane & 15u, kq = lane >> 4;
    const uint32_t nwj = j.rpp, cpr = j.cpr, PW = nwj * 4;
    const uint32_t rows = (uint32_t)j.rows, row_bytes = (uint32_t)j.row_bytes;
    uint8_t *ring = lds + wv * (NS * kQ4kTileBytes);
    float *part = reinterpret_cast<float *>(lds + nw_launch * (NS * kQ4kTileBytes));
    const uint32_t np = wv < nwj ? (cpr - wv + nwj - 1) / nwj : 0;  // columns wv, wv+nwj, ... of this wavefront

    // lane's three pieces of a wave-tile, in 16-byte units u = row*9 + piece (the last 256 B go dword by dword)
    const uint32_t u0 = lane, u1 = 64 + lane, u2 = 128 + (lane >> 2);
    const uint32_t r0 = u0 / 9, r1 = u1 / 9, r2 = u2 / 9;
    const uint32_t w0 = (u0 - r0 * 9) * 16, w1 = (u1 - r1 * 9) * 16, w2 = (u2 - r2 * 9) * 16 + (lane & 3u) * 4;
    const uint32_t o0 = r0 * row_bytes + w0, o1 = r1 * row_bytes + w1, o2 = r2 * row_bytes + w2;
    const uint8_t *wcol = j.w + (size_t)wv * 144;
    const uint32_t nt = tile_b - tile_a;

    // issue cursor: wave-tiles in the order they are consumed (batch, column pass, tile of the batch)
    uint32_t it_tb = 0, it_p = 0, it_tl = 0, n_issue = 0;
    auto issue = [&]() {
        // past the end the last wave-tile is read again: every wavefront keeps the same number of loads in flight
        const uint32_t tl = min(tile_a + it_tb + it_tl, tile_b - 1);
        // wave-uniform 64-bit base + per-lane 32-bit offset; only a ragged last tile recomputes the offsets
        const uint32_t rb = tl * 16;
        const uint8_t *gp = wcol + (size_t)it_p * nwj * 144 + (size_t)rb * row_bytes;
        uint32_t a0 = o0, a1 = o1, a2 = o2;
        if (rb + 16 > rows) {
            const uint32_t lim = rows - 1 - rb;
            a0 = min(r0, lim) * row_bytes + w0;
            a1 = min(r1, lim) * row_bytes + w1;
            a2 = min(r2, lim) * row_bytes + w2;
        }
        const uint8_t *g0 = gp + a0, *g1 = gp + a1, *g2 = gp + a2;
        uint8_t *lp = ring + (n_issue % NS) * kQ4kTileBytes;
        __builtin_amdgcn_global_load_lds((g_vp)g0, (lds_vp)lp, 16, 0, 0);
        __builtin_amdgcn_global_load_lds((g_vp)g1, (lds_vp)(lp + 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((g_vp)g2, (lds_vp)(lp + 2048), 4, 0, 0);
        n_issue++;
        if (it_tb < nt) {
            const uint32_t nb = min((uint32_t)R, nt - it_tb);
            if (++it_tl == nb) {
                it_tl = 0;
                if (++it_p == np) { it_p = 0; it_tb += R; }
            }
        }
    };
    // the activations of all this wavefront's columns are requested first and together (one memory round
    // trip, ahead of the weight tiles in the in-order return queue), then prepared while the tiles fly
    Q4kRaw raw[kQ4kMaxColPasses];
#pragma unroll
    for (int p = 0; p < kQ4kMaxColPasses; p++)
        if ((uint32_t)p < np) raw[p] = q4k_mfma_load_col(j.x, wv + nwj * p, lane);
    if (np >= 1)
        for (int s = 0; s < NS - 1; s++) issue();

    // Column state: in registers when the wavefront has one column; with several it is prepared once per
    // job into this wavefront's own LDS area (1 KB of operands + 64 B of scales and sums per column) and
    // fetched at every column change.
    uint8_t *cols = lds + nw_launch * (NS * kQ4kTileBytes) + 2 * R * 16 * nw_launch * 4 * sizeof(float) +
                    wv * (kQ4kMaxColPasses * kQ4kColBytes);
    Q4kCol col;
    Q4kOp xm[8];
    auto fetch_col = [&](uint32_t p) {
        const uint8_t *cp = cols + p * kQ4kColBytes;
        const u32x4 xq = *reinterpret_cast<const u32x4 *>(cp + lane * 16);
        const float2_t sm = *reinterpret_cast<const float2_t *>(cp + 1024 + 16 + kq * 8);
        col.xq[0] = xq.x; col.xq[1] = xq.y; col.xq[2] = xq.z; col.xq[3] = xq.w;
        col.k = *reinterpret_cast<const float *>(cp + 1024);
        col.sum_lo = sm.x; col.sum_hi = sm.y;
        q4k_mfma_operands(xm, col, jr);
    };
    if (np == 1) {
        col = q4k_mfma_finish_col(raw[0], lane);
        q4k_mfma_operands(xm, col, jr);
    } else if (np > 1) {
#pragma unroll
        for (int p = 0; p < kQ4kMaxColPasses; p++) {
            if ((uint32_t)p < np) {
                const Q4kCol c = q4k_mfma_finish_col(raw[p], lane);
                uint8_t *cp = cols + p * kQ4kColBytes;
                *reinterpret_cast<u32x4 *>(cp + lane * 16) = (u32x4){c.xq[0], c.xq[1], c.xq[2], c.xq[3]};
                if (lane == 0) *reinterpret_cast<float *>(cp + 1024) = c.k;
                if (jr == 0) *reinterpret_cast<float2_t *>(cp + 1024 + 16 + kq * 8) = (float2_t){c.sum_lo, c.sum_hi};
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // own writes, own reads: program order is enough
    }

    uint32_t n_use = 0;
    for (uint32_t tb = 0; tb < nt; tb += R) {
        float *pb = part + parity * (R * 16 * nw_launch * 4);
        const uint32_t nb = min((uint32_t)R, nt - tb);
        if (np >= 1) {
            float racc[R];
#pragma unroll
            for (int tl = 0; tl < R; tl++) racc[tl] = 0.f;
#pragma unroll 1
            for (uint32_t p = 0; p < np; p++) {
                if (np > 1) fetch_col(p);
#pragma unroll
                for (int tl = 0; tl < R; tl++) {
                    if ((uint32_t)tl < nb) {
                        issue();
                        LARQL_WAIT_VMCNT(3 * (NS - 1));  // at most NS-1 younger wave-tiles still in flight: the oldest has landed
                        asm volatile("" ::: "memory");
                        racc[tl] += q4k_mfma_tile(ring + (n_use % NS) * kQ4kTileBytes, xm, col, jr, kq);
                        n_use++;
                    }
                }
            }
#pragma unroll
            for (int tl = 0; tl < R; tl++)
                if ((uint32_t)tl < nb) pb[(tl * 16 + jr) * PW + wv * 4 + kq] = racc[tl];
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // fold: 4 lanes per row, lane q sums the group-q partial of every wavefront in order
        const uint32_t row_base = (tile_a + tb) * 16;
        for (uint32_t rr = threadIdx.x >> 2; rr < nb * 16; rr += blockDim.x >> 2) {
            const uint32_t qd = threadIdx.x & 3u;
            float s = 0.f;
            for (uint32_t k = 0; k < nwj; k++) s += pb[rr * PW + k * 4 + qd];
            s = dpp_add<0xB1>(s);  // quad_perm [1,0,3,2]
            s = dpp_add<0x4E>(s);  // quad_perm [2,3,0,1]
            if (qd == 0 && row_base + rr < rows) ((g_f32wp)j.out)[row_base + rr] = s;
        }
        parity ^= 1u;
    }
}

// ---------------------------------------------------------------------------
// Q6_K on the matrix cores: the scheme of the Q4_K kernel above for 210-byte super-blocks (q6k_matvec::dispatch,
// larql-compute/src/cpu/ops/q6k_matvec.rs:45-91: per 16-element group sub = sum (q - 32) * x; acc += (d * sc) * sub).
//
// A wave-tile is 16 rows x one super-block, copied global -> LDS as 13 sixteen-byte pieces per row (ql, qh, scales)
// plus the block's last 16 bytes again for d.  The blocks are only 2-byte aligned in memory: the copies take any alignment (at
// ~12 % of the bandwidth that aligned ones reach) and land on a 208-byte pitch, so that every LDS read is an aligned
// ds_read_b128.  (Copying the 14 aligned pieces that contain a block instead moves the misalignment to the LDS side,
// where it costs more: a misaligned ds_read_b128 is correct but slow, five aligned dwords and a byte rotation per
// field add instructions to a kernel that is within reach of the vector issue limit; both were measured slower.)
// One v_mfma_i32_16x16x64_i8 covers 64 weights = four scale
// groups: lane (row j, kq) supplies in its 16 k-slots the 16 six-bit codes of group 4m + kq of weight row j (its 16
// ql bytes serve MFMAs 2h (low nibbles) and 2h+1 (high nibbles) of half h, its 16 qh bytes give both their top bits:
// four instructions per four codes), and A row 4g + i carries limb i of the activations of group 4m + g in that
// group's k-slots, zero elsewhere.  After the MFMA lane (j, rq) holds the four exact limb sums of group 4m + rq of
// row j — the group whose int8 scale it applies.  The -32 goes through the group's sum of x.  Four MFMAs per tile,
// none accumulates into another.  The activations of a column (256 elements) are turned into limbs by all 64 lanes,
// four elements each, and go through LDS (limb planes) into the operand layout; the operands of all the wavefront's
// columns (up to 4) stay in registers and tiles are walked column-innermost.
// ---------------------------------------------------------------------------
constexpr int kQ6kStages = 3;
constexpr int kQ6kBatchTiles = 4;
constexpr int kQ6kMaxColPasses = 4;
constexpr int kQ6kMaxWaves = 10;
constexpr uint32_t kQ6kPitch = 208;                          // ql 128, qh 64, scales 16
constexpr uint32_t kQ6kTileBytes = 16 * kQ6kPitch + 256;     // + a 16-byte slot per row whose last two bytes are d

struct Q6kCol {
    Q4kOp xm[4];     // A operand of MFMA m: limb (row % 4) of group 4m + kq in this lane's k-slots if row / 4 == kq, else zero
    float sumx[4];   // -32 * the sum of x over group 4m + kq
    float k;         // 2^(e-27)
};

// turns the lane's four activations (elements 4*lane .. 4*lane+3 of the column) into limbs and group sums at `cp`
__device__ __forceinline__ void q6k_mfma_prepare_col(const f32x4 v, uint32_t lane, uint8_t *cp) {
    const float mx = wave_max_nonneg(fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    int ex = 0;
    if (mx > 0.f && mx < __builtin_inff()) (void)frexpf(mx, &ex);  // mx = f * 2^ex, f in [0.5, 1)
    ex = max(-90, min(120, ex));
    const float to_int = ldexpf(1.f, 27 - ex);  // |x| * to_int < 2^27
    const float e[4] = {v.x, v.y, v.z, v.w};
    uint32_t pl[4] = {0, 0, 0, 0};
#pragma unroll
    for (int t = 0; t < 4; t++) {
        // n = l0*128^3 + l1*128^2 + l2*128 + l3 with l1..l3 in [-64, 63], l0 in [-64, 64]
        const int n = (int)__builtin_rintf(e[t] * to_int);
        const int l3 = ((n + 64) & 127) - 64, n1 = (n - l3) >> 7;
        const int l2 = ((n1 + 64) & 127) - 64, n2 = (n1 - l2) >> 7;
        const int l1 = ((n2 + 64) & 127) - 64, l0 = (n2 - l1) >> 7;
        pl[0] |= ((uint32_t)l0 & 0xFFu) << (8 * t); pl[1] |= ((uint32_t)l1 & 0xFFu) << (8 * t);
        pl[2] |= ((uint32_t)l2 & 0xFFu) << (8 * t); pl[3] |= ((uint32_t)l3 & 0xFFu) << (8 * t);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) *reinterpret_cast<uint32_t *>(cp + i * 256 + 4 * lane) = pl[i];
    float sm = (v.x + v.y) + (v.z + v.w);
    sm = dpp_add<0xB1>(sm);  // quad_perm [1,0,3,2]
    sm = dpp_add<0x4E>(sm);  // quad_perm [2,3,0,1]: the 16 elements of group lane / 4
    const uint32_t g = lane >> 2;
    if ((lane & 3u) == 0) *reinterpret_cast<float *>(cp + 1024 + 4 * ((g & 3u) * 4 + (g >> 2))) = sm;  // [g % 4][g / 4]
    if (lane == 0) *reinterpret_cast<float *>(cp + 1024 + 64) = ldexpf(1.f, ex - 27);
}

__device__ __forceinline__ void q6k_mfma_fetch_col(Q6kCol &col, const uint8_t *cp, uint32_t jr, uint32_t kq) {
    const bool mine = (jr >> 2) == kq;
    const uint8_t *lp = cp + (jr & 3u) * 256 + 16 * kq;
#pragma unroll
    for (int m = 0; m < 4; m++) {
        const u32x4 t = *reinterpret_cast<const u32x4 *>(lp + 64 * m);  // group 4m + kq
        col.xm[m].u[0] = mine ? t.x : 0u; col.xm[m].u[1] = mine ? t.y : 0u;
        col.xm[m].u[2] = mine ? t.z : 0u; col.xm[m].u[3] = mine ? t.w : 0u;
    }
    const f32x4 sm = *reinterpret_cast<const f32x4 *>(cp + 1024 + 16 * kq);
    col.sumx[0] = -32.f * sm.x; col.sumx[1] = -32.f * sm.y; col.sumx[2] = -32.f * sm.z; col.sumx[3] = -32.f * sm.w;
    col.k = *reinterpret_cast<const float *>(cp + 1024 + 64);
}

// one wave-tile from its LDS slot: 16 rows x one super-block against the column's activations
__device__ __forceinline__ float q6k_mfma_tile(const uint8_t *slot, const Q6kCol &col, uint32_t j, uint32_t kq) {
    const uint8_t *sp = slot + j * kQ6kPitch;
    u32x4 ql[2], qh[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        ql[h] = *reinterpret_cast<const u32x4 *>(sp + 64 * h + 16 * kq);
        qh[h] = *reinterpret_cast<const u32x4 *>(sp + 128 + 32 * h + 16 * (kq & 1u));
    }
    const u32x4 scs = *reinterpret_cast<const u32x4 *>(sp + 192);
    const float d = half_bits_to_float(*reinterpret_cast<const uint32_t *>(slot + 16 * kQ6kPitch + 16 * j + 12) >> 16);
    // top bits: MFMA 2h wants bits s0, s0+1 of the qh bytes in bits 4-5 (a left shift by 4 - s0), MFMA 2h+1 bits
    // s0+4, s0+5 (a right shift by s0); what crosses a byte boundary falls outside the mask
    const uint32_t s0 = 2u * (kq >> 1), sl = 4u - s0;
    const i32x4 zero = {0, 0, 0, 0};
    float acc = 0.f;
#pragma unroll
    for (int m = 0; m < 4; m++) {
        const int h = m >> 1;
        Q4kOp b;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (m & 1) b.u[i] = ((qh[h][i] >> s0) & 0x30303030u) | ((ql[h][i] >> 4) & 0x0F0F0F0Fu);
            else b.u[i] = ((qh[h][i] << sl) & 0x30303030u) | (ql[h][i] & 0x0F0F0F0Fu);
        }
        const i32x4 D = __builtin_amdgcn_mfma_i32_16x16x64_i8(col.xm[m].v, b.v, zero, 0, 0, 0);
        // this lane's group is 4m + kq: D = its four limb sums; pairs of limbs meet as integers (exact, below 2^24)
        const float hi = (float)(D[0] * 128 + D[1]), lo = (float)(D[2] * 128 + D[3]);
        const float dot = __builtin_fmaf(hi, 16384.f, lo);
        const float sc = (float)(int)(int8_t)(scs[m] >> (8u * kq));
        acc = __builtin_fmaf(sc, __builtin_fmaf(dot, col.k, col.sumx[m]), acc);  // (sumx holds -32 * the group's sum of x)
    }
    return d * acc;
}

// tiles [tile_a, tile_b) of one job, columns innermost (the workgroup reads whole rows); `parity` flips per batch
// (double-buffered partials)
__device__ __forceinline__ void run_q6k_mfma(const GemvJob &j, uint32_t tile_a, uint32_t tile_b, uint8_t *lds, uint32_t &parity) {
    constexpr int NS = kQ6kStages, R = kQ6kBatchTiles;
    const uint32_t lane = threadIdx.x & 63u, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nw_launch = blockDim.x >> 6;
    const uint32_t jr = lane & 15u, kq = lane >> 4;
    const uint32_t nwj = j.rpp, cpr = j.cpr, PW = nwj * 4;
    const uint32_t rows = (uint32_t)j.rows, row_bytes = (uint32_t)j.row_bytes;
    uint8_t *ring = lds + wv * (NS * kQ6kTileBytes);
    float *part = reinterpret_cast<float *>(lds + nw_launch * (NS * kQ6kTileBytes));
    const uint32_t np = wv < nwj ? (cpr - wv + nwj - 1) / nwj : 0;  // columns wv, wv+nwj, ... of this wavefront

    // lane's pieces of a wave-tile: 16-byte piece u = 13 * row + piece (u < 208); lanes 16..31 of the fourth copy bring
    // the last 16 bytes of the block of row lane - 16 (bytes 194..209: d is the end of it)
    uint32_t pr[4], po[4], o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t u = min(64u * i + lane, 207u);
        pr[i] = u / 13;
        po[i] = (u - pr[i] * 13) * 16;
        if (i == 3 && lane >= 16) { pr[i] = lane & 15u; po[i] = 194; }
        o[i] = pr[i] * row_bytes + po[i];
    }
    const uint8_t *wcol = j.w + (size_t)wv * 210;
    const uint32_t nt = tile_b - tile_a;

    // issue cursor: wave-tiles in the order they are consumed (batch, column pass, tile of the batch)
    uint32_t it_tb = 0, it_p = 0, it_tl = 0, n_issue = 0;
    auto issue = [&]() {
        // past the end the last wave-tile is read again: every wavefront keeps the same number of loads in flight
        const uint32_t tl = min(tile_a + it_tb + it_tl, tile_b - 1);
        const uint32_t rb = tl * 16, lim = min(15u, rows - 1 - rb);  // (rows of a ragged last tile are clamped)
        const uint8_t *gp = wcol + (size_t)it_p * nwj * 210 + (size_t)rb * row_bytes;
        uint8_t *lp = ring + (n_issue % NS) * kQ6kTileBytes;
        // wave-uniform 64-bit base + per-lane 32-bit offset; only a ragged last tile recomputes the offsets
        uint32_t a0 = o[0], a1 = o[1], a2 = o[2], a3 = o[3];
        if (rb + 16 > rows) {
            a0 = min(pr[0], lim) * row_bytes + po[0]; a1 = min(pr[1], lim) * row_bytes + po[1];
            a2 = min(pr[2], lim) * row_bytes + po[2]; a3 = min(pr[3], lim) * row_bytes + po[3];
        }
        __builtin_amdgcn_global_load_lds((g_vp)(gp + a0), (lds_vp)lp, 16, 0, 0);
        __builtin_amdgcn_global_load_lds((g_vp)(gp + a1), (lds_vp)(lp + 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((g_vp)(gp + a2), (lds_vp)(lp + 2048), 16, 0, 0);
        if (lane < 32) __builtin_amdgcn_global_load_lds((g_vp)(gp + a3), (lds_vp)(lp + 3072), 16, 0, 0);
        n_issue++;
        if (it_tb + it_tl < nt && ++it_p == np) { it_p = 0; it_tl++; }  // (it_tb stays 0: tiles in order, columns innermost)
    };
    // the activations of all this wavefront's columns are requested first and together, then prepared while the tiles fly
    f32x4 raw[kQ6kMaxColPasses];
#pragma unroll
    for (int p = 0; p < kQ6kMaxColPasses; p++)
        if ((uint32_t)p < np) raw[p] = ((g_f4p)(j.x + (size_t)(wv + nwj * p) * 256))[lane];
    if (np >= 1)
        for (int s = 0; s < NS - 1; s++) issue();
    // every column's operands stay in registers for the job; a column passes through the ring's last slot, still
    // free at this point, on its way into the operand layout
    Q6kCol col[kQ6kMaxColPasses];
    uint8_t *scratch = ring + (NS - 1) * kQ6kTileBytes;
#pragma unroll
    for (int p = 0; p < kQ6kMaxColPasses; p++) {
        if ((uint32_t)p < np) {
            q6k_mfma_prepare_col(raw[p], lane, scratch);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // own writes, own reads: program order is enough
            q6k_mfma_fetch_col(col[p], scratch, jr, kq);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // (read before the next column overwrites it)
        }
    }

    uint32_t n_use = 0;
    for (uint32_t tb = 0; tb < nt; tb += R) {
        float *pb = part + parity * (R * 16 * nw_launch * 4);
        const uint32_t nb = min((uint32_t)R, nt - tb);
        if (np >= 1) {
            float racc[R];
#pragma unroll
            for (int tl = 0; tl < R; tl++) {
                racc[tl] = 0.f;
                if ((uint32_t)tl < nb) {
#pragma unroll
                    for (int p = 0; p < kQ6kMaxColPasses; p++) {
                        if ((uint32_t)p < np) {
                            issue();
                            LARQL_WAIT_VMCNT(4 * (NS - 1));  // at most NS-1 younger wave-tiles still in flight: the oldest has landed
                            asm volatile("" ::: "memory");
                            racc[tl] += q6k_mfma_tile(ring + (n_use % NS) * kQ6kTileBytes, col[p], jr, kq);
                            n_use++;
                        }
                    }
                }
            }
#pragma unroll
            for (int tl = 0; tl < R; tl++)
                if ((uint32_t)tl < nb) pb[(tl * 16 + jr) * PW + wv * 4 + kq] = racc[tl];
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // fold: 4 lanes per row, lane q sums the group-q partial of every wavefront in order
        const uint32_t row_base = (tile_a + tb) * 16;
        for (uint32_t rr = threadIdx.x >> 2; rr < nb * 16; rr += blockDim.x >> 2) {
            const uint32_t qd = threadIdx.x & 3u;
            float s = 0.f;
            for (uint32_t k = 0; k < nwj; k++) s += pb[rr * PW + k * 4 + qd];
            s = dpp_add<0xB1>(s);  // quad_perm [1,0,3,2]
            s = dpp_add<0x4E>(s);  // quad_perm [2,3,0,1]
            if (qd == 0 && row_base + rr < rows) ((g_f32wp)j.out)[row_base + rr] = s;
        }
        parity ^= 1u;
    }
}

// ---------------------------------------------------------------------------
// Q4_K weights against a Q8_K activation (q4k_q8k_matvec_scalar, larql-compute/src/cpu/ops/q4k_q8k_dot/
// q4k_scalar.rs:15-84): the activation is already int8, so one operand set replaces the four digit sets of the
// f32 kernel.  A row m of the "A" operand is sub-block m (rows 8..15 are zero): its 32 codes sit in the k-slots
// where "B" carries that sub-block's nibbles (slots 16kq+0..7 = low nibbles = sub-block 2g, 16kq+8..15 = high =
// sub-block 2g+1), so after four MFMAs lane (row j, kq < 2) holds the eight exact integer dots of weight row j,
// four per lane.  sum1 = sum sc*dot and sum2 = sum mn*bsum are formed in integers, the two halves meet by one
// cross-lane add, and the reference's float expression d_w*d_y*sum1 - dmin_w*d_y*sum2 is evaluated once per
// (row, super-block) without contraction.  Every column keeps its own partial and a row is summed by one lane
// in super-block order: the result equals the reference's bit for bit.
// All columns of a wavefront (up to 4) keep their operands in registers; tiles are walked column-innermost, so
// the workgroup reads whole rows.
// ---------------------------------------------------------------------------
struct Q8kCol {
    Q4kOp xm[4];      // operand of group g: this lane's 8 codes in the low or high k-slots if its row is sub-block 2g or 2g+1
    uint32_t bs[2];   // the four i16 sub-block sums of this lane's half (4kq..4kq+3), packed
    float dy;
};

__device__ __forceinline__ Q8kCol q8k_load_col(const uint8_t *q8k, uint32_t k, uint32_t c, uint32_t lane) {
    const uint32_t r = lane & 15u, kq = lane >> 4;
    const GLOBAL_AS uint8_t *base = (const GLOBAL_AS uint8_t *)q8k;
    const u32x2 codes = *(const GLOBAL_AS u32x2 *)(base + (size_t)c * 256 + (r & 7u) * 32 + kq * 8);
    const u32x2 sums = *(const GLOBAL_AS u32x2 *)(base + k + (k / 256) * 4 + (size_t)c * 16 + (kq & 1u) * 8);
    Q8kCol col;
    col.dy = *(const GLOBAL_AS float *)(base + k + (size_t)c * 4);
    col.bs[0] = sums.x; col.bs[1] = sums.y;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const bool lo = r == (uint32_t)(2 * g), hi = r == (uint32_t)(2 * g + 1);
        col.xm[g].u[0] = lo ? codes.x : 0u; col.xm[g].u[1] = lo ? codes.y : 0u;
        col.xm[g].u[2] = hi ? codes.x : 0u; col.xm[g].u[3] = hi ? codes.y : 0u;
    }
    return col;
}

// one wave-tile: 16 rows x one super-block; returns this (row, super-block)'s term in lanes kq == 0
__device__ __forceinline__ float q4k_q8k_tile(const uint8_t *slot, const Q8kCol &col, uint32_t j, uint32_t kq) {
#pragma clang fp contract(off)
    const uint8_t *sp = slot + j * 144;
    const u32x4 hdr = *reinterpret_cast<const u32x4 *>(sp);
    u32x2 q[4];
#pragma unroll
    for (int g = 0; g < 4; g++) q[g] = *reinterpret_cast<const u32x2 *>(sp + 16 + 32 * g + 8 * kq);
    i32x4 D = {0, 0, 0, 0};
#pragma unroll
    for (int g = 0; g < 4; g++) {
        Q4kOp b;
        b.u[0] = q[g].x & 0x0F0F0F0Fu; b.u[1] = q[g].y & 0x0F0F0F0Fu;
        b.u[2] = (q[g].x >> 4) & 0x0F0F0F0Fu; b.u[3] = (q[g].y >> 4) & 0x0F0F0F0Fu;
        D = __builtin_amdgcn_mfma_i32_16x16x64_i8(col.xm[g].v, b.v, D, 0, 0, 0);
    }
    // D[i] = dot of sub-block 4kq + i (lanes kq >= 2 hold the zero rows: they compute with kq & 1 and are ignored)
    const bool upper = (kq & 1u) != 0;
    const uint32_t sc4 = upper ? ((hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u)) : (hdr.y & 0x3F3F3F3Fu);
    const uint32_t mn4 = upper ? (((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u)) : (hdr.z & 0x3F3F3F3Fu);
    // |dot| <= 32*15*127 and |bsum| <= 32*127: the products fit 24-bit multiplies
    int s1 = __mul24((int)(sc4 & 0xFFu), D[0]) + __mul24((int)((sc4 >> 8) & 0xFFu), D[1]) +
             __mul24((int)((sc4 >> 16) & 0xFFu), D[2]) + __mul24((int)(sc4 >> 24), D[3]);
    const int b0 = (int)(int16_t)(col.bs[0] & 0xFFFFu), b1 = (int)col.bs[0] >> 16;
    const int b2 = (int)(int16_t)(col.bs[1] & 0xFFFFu), b3 = (int)col.bs[1] >> 16;
    int s2 = __mul24((int)(mn4 & 0xFFu), b0) + __mul24((int)((mn4 >> 8) & 0xFFu), b1) +
             __mul24((int)((mn4 >> 16) & 0xFFu), b2) + __mul24((int)(mn4 >> 24), b3);
    s1 += __shfl_xor(s1, 16);  // sub-blocks 0..3 + 4..7
    s2 += __shfl_xor(s2, 16);
    const float d_w = half_bits_to_float(hdr.x & 0xFFFFu), dmin_w = half_bits_to_float(hdr.x >> 16);
    float t1 = d_w * col.dy;
    t1 = t1 * (float)s1;
    float t2 = dmin_w * col.dy;
    t2 = t2 * (float)s2;
    return t1 - t2;
}

// tiles [tile_a, tile_b) of one job; `parity` flips per batch (double-buffered partials)
__device__ __forceinline__ void run_q4k_q8k(const GemvJob &j, uint32_t tile_a, uint32_t tile_b, uint8_t *lds, uint32_t &parity) {
    constexpr int NS = kQ4kStages, R = kQ4kBatchTiles, NP = kQ4kMaxColPasses;
    const uint32_t lane = threadIdx.x & 63u, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nw_launch = blockDim.x >> 6;
    const uint32_t jr = lane & 15u, kq = lane >> 4;
    const uint32_t nwj = j.rpp, cpr = j.cpr, PW = cpr;  // one partial per (row, super-block)
    const uint32_t rows = (uint32_t)j.rows, row_bytes = (uint32_t)j.row_bytes;
    uint8_t *ring = lds + wv * (NS * kQ4kTileBytes);
    float *part = reinterpret_cast<float *>(lds + nw_launch * (NS * kQ4kTileBytes));
    const uint32_t np = wv < nwj ? (cpr - wv + nwj - 1) / nwj : 0;  // columns wv, wv+nwj, ... of this wavefront

    const uint32_t u0 = lane, u1 = 64 + lane, u2 = 128 + (lane >> 2);
    const uint32_t r0 = u0 / 9, r1 = u1 / 9, r2 = u2 / 9;
    const uint32_t w0 = (u0 - r0 * 9) * 16, w1 = (u1 - r1 * 9) * 16, w2 = (u2 - r2 * 9) * 16 + (lane & 3u) * 4;
    const uint32_t o0 = r0 * row_bytes + w0, o1 = r1 * row_bytes + w1, o2 = r2 * row_bytes + w2;
    const uint8_t *wcol = j.w + (size_t)wv * 144;
    const uint32_t nt = tile_b - tile_a;

    // issue cursor: wave-tiles in the order they are consumed (tile, then column pass)
    uint32_t it_tile = tile_a, it_p = 0, n_issue = 0;
    auto issue = [&]() {
        const uint32_t rb = min(it_tile, tile_b - 1) * 16;  // past the end: the last tile again (uniform load counts)
        const uint8_t *gp = wcol + (size_t)it_p * nwj * 144 + (size_t)rb * row_bytes;
        uint32_t a0 = o0, a1 = o1, a2 = o2;
        if (rb + 16 > rows) {
            const uint32_t lim = rows - 1 - rb;
            a0 = min(r0, lim) * row_bytes + w0;
            a1 = min(r1, lim) * row_bytes + w1;
            a2 = min(r2, lim) * row_bytes + w2;
        }
        uint8_t *lp = ring + (n_issue % NS) * kQ4kTileBytes;
        __builtin_amdgcn_global_load_lds((g_vp)(gp + a0), (lds_vp)lp, 16, 0, 0);
        __builtin_amdgcn_global_load_lds((g_vp)(gp + a1), (lds_vp)(lp + 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((g_vp)(gp + a2), (lds_vp)(lp + 2048), 4, 0, 0);
        n_issue++;
        if (it_tile < tile_b && ++it_p == np) { it_p = 0; it_tile++; }
    };
    // the activation columns are requested first (ahead of the weight tiles in the in-order return queue)
    Q8kCol col[NP];
#pragma unroll
    for (int p = 0; p < NP; p++)
        col[p] = q8k_load_col((const uint8_t *)j.x, (uint32_t)j.k, min(wv + nwj * (uint32_t)p, cpr - 1), lane);
    if (np >= 1)
        for (int s = 0; s < NS - 1; s++) issue();

    uint32_t n_use = 0;
    for (uint32_t tb = 0; tb < nt; tb += R) {
        float *pb = part + parity * (R * 16 * PW);
        const uint32_t nb = min((uint32_t)R, nt - tb);
        if (np >= 1) {
            for (uint32_t tl = 0; tl < nb; tl++) {
#pragma unroll
                for (int p = 0; p < NP; p++) {
                    if ((uint32_t)p < np) {
                        issue();
                        LARQL_WAIT_VMCNT(3 * (NS - 1));  // at most NS-1 younger wave-tiles still in flight: the oldest has landed
                        asm volatile("" ::: "memory");
                        const float term = q4k_q8k_tile(ring + (n_use % NS) * kQ4kTileBytes, col[p], jr, kq);
                        n_use++;
                        if (kq == 0) pb[(tl * 16 + jr) * PW + wv + nwj * p] = term;
                    }
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // a lane per row: acc += term, super-blocks in order (q4k_scalar.rs:39,79)
        const uint32_t row_base = (tile_a + tb) * 16;
        for (uint32_t rr = threadIdx.x; rr < nb * 16; rr += blockDim.x) {
            float acc = 0.f;
            for (uint32_t c = 0; c < cpr; c++) acc += pb[rr * PW + c];
            if (row_base + rr < rows) ((g_f32wp)j.out)[row_base + rr] = acc;
        }
        parity ^= 1u;
    }
}

// ---------------------------------------------------------------------------
// MXFP4 on the matrix cores (rows of up to 40 x 128 elements).
//
// v_mfma_f32_16x16x32_bf16 with the roles swapped as in the Q4_K kernel: the 16 "B" columns are 16 weight rows, the
// "A" rows carry the activations.  Lane (column j = lane%16, kg = lane/16) owns one MXFP4 block of weight row j per
// 128-element step — 16 packed bytes (low nibble first) and one e8m0 scale byte, exactly as mxfp4.rs lays it out
// (larql-models/src/quant/mxfp4.rs:42-95) — and turns it into four B operands of eight bf16 each with
// v_cvt_scalef32_pk_bf16_fp4 (two e2m1 codes times the block's power of two per instruction; every product of an e2m1
// value and a power of two is a bf16 number, so the conversion is exact).  The weights go global -> LDS -> registers
// as stored: a wavefront owns a K-range of `cw` 128-element steps of the tile's rows and streams its (16 rows x cw
// steps) tiles through a private LDS ring: a 16-byte global_load_lds per lane and step for the nibbles and one 4-byte
// copy per tile for the scale bytes of all its steps (a dword per row and step, at whatever alignment the row has;
// rows need at least 4 blocks).
//
// The activations ride in bf16 as well: x = hi + mid + lo, each term the next 8 significant bits of x (exact, so the
// three terms reproduce the f32 value), and A row 4t + i holds term i of token t (row 4t + 3 is zero): up to four
// tokens share one read of the weights.  MFMA m of a step takes from lane (row, kg) the elements 32kg + 8m .. + 7 of
// the step on both sides (dword m of the lane's block), so neither operand is shuffled.  After the wavefront's steps
// lane (j, rq) holds the three term sums of token rq for weight row j and adds them up.  Products are exact in f32
// (8 x 8 significant bits) and accumulate in f32.
// e8m0 0 means 0.0 in the reference and 255 NaN: the scale handed to the conversion is (byte << 23) as an f32, i.e.
// 2^(byte-127) for 1..254 and 0.0 for 0, and a NaN for 255.
// ---------------------------------------------------------------------------
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
union BfOp { bf16x8_t v; uint32_t u[4]; };
constexpr int kMx4Stages = 3;
constexpr int kMx4BatchTiles = 4;
constexpr int kMx4FoldTiles = 4;   // row tiles per batch of a job folded over experts
constexpr int kMx4MaxSteps = 5;    // 128-element steps per wavefront
constexpr int kMx4MaxWaves = 8;    // (512 threads: a 256-register budget per lane)
constexpr uint32_t kMx4StepBytes = 1024;      // per step of a wave-tile: 64 lanes x 16 B of nibbles
constexpr uint32_t kMx4ScaleBytes = 320;      // per wave-tile: the scale bytes of all its steps, a dword slot per (row, step)
constexpr uint32_t kMx4TermBytes = 768;       // per step: three planes of 128 bf16 terms (the operand scratch)

// A operands of a wavefront's K-range: [step][MFMA of the step]
struct Mx4Ops { BfOp a[kMx4MaxSteps][4]; };

// The two activations of lane `lane` in step `step`, for every token of the job (the gate and up values of a gated
// job): loaded apart from their conversion so that all steps' loads fly together (a load's first use waits for
// everything in flight, the weight tiles included, so loads issued one step at a time cost a round trip each).
constexpr int kMx4MaxTokens = 4;    // tokens that share one job's weights: four A rows each
// (As loaded: `a` and `b` are the two 8-byte reads of a lane — plain: a = x0 x1 (b repeats it); gate and up apart: a = g0 g1,
// b = u0 u1; interleaved g0 u0 g1 u1: a = g0 u0, b = g1 u1 — taken apart when the operands are made, so that no move of
// loaded data sits between the loads: the compiler waits for a load where its result is first touched.)
struct Mx4In { float2_t a[kMx4MaxTokens], b[kMx4MaxTokens]; bool inside; };

// The weight matrices a job reads (wave-uniform): one, or — a job folded over experts (GemvJob::combine_w) — one per
// activation, each with its expert's bias row and combine weight; `ok` is false for an expert id outside the bank.
struct Mx4Sel {
    const uint8_t *w[kMx4MaxTokens], *aux[kMx4MaxTokens];
    const float *bias[kMx4MaxTokens];
    float cw[kMx4MaxTokens];
    bool ok[kMx4MaxTokens];
};

__device__ __forceinline__ uint32_t mx4_tokens(const GemvJob &j) { return j.batch > 1 ? min(j.batch, (uint32_t)kMx4MaxTokens) : 1u; }
__device__ __forceinline__ int64_t mx4_x_off(const GemvJob &j, int q) { return q == 0 ? 0 : q == 1 ? (int64_t)j.x_stride : q == 2 ? j.x_off[0] : j.x_off[1]; }
__device__ __forceinline__ int64_t mx4_out_off(const GemvJob &j, uint32_t q) { return q == 0 ? 0 : q == 1 ? (int64_t)j.out_stride : q == 2 ? j.out_off[0] : j.out_off[1]; }

__device__ __forceinline__ Mx4In mx4_load_step(const GemvJob &j, uint32_t step, uint32_t lane) {
    const uint32_t k = (uint32_t)j.k, i0 = step * 128 + 2 * lane;
    const uint32_t ntok = mx4_tokens(j);
    Mx4In in;
    in.inside = i0 + 2 <= k;  // k is even: a pair is inside or outside
    const uint32_t ic = in.inside ? i0 : 0u;  // (a pair past the row end reads the row's first pair and is zeroed later)
    const bool il = j.x_glu == j.x;
    const float *xg = j.x_glu ? j.x_glu : j.x;
#pragma unroll
    for (int q = 0; q < kMx4MaxTokens; q++) {
        if ((uint32_t)q < ntok) {
            const int64_t off = mx4_x_off(j, q);
            const float *pa = il ? j.x + off + 2 * (size_t)ic : j.x + off + ic;
            const float *pb = il ? j.x + off + 2 * (size_t)ic + 2 : xg + off + ic;
            in.a[q] = *(const GLOBAL_AS float2_t *)pa;
            in.b[q] = *(const GLOBAL_AS float2_t *)pb;
        }
    }
    return in;
}

// The activation pair of token Q as the job means it: v = the values (gate values of a gated job), u = the up values
__device__ __forceinline__ void mx4_pair(const GemvJob &j, const Mx4In &in, int q, float2_t &v, float2_t &u) {
    const bool il = j.x_glu == j.x;
    v.x = in.a[q].x; v.y = il ? in.b[q].x : in.a[q].y;
    u.x = il ? in.a[q].y : in.b[q].x; u.y = in.b[q].y;
    if (!in.inside) { v = (float2_t){0.f, 0.f}; u = (float2_t){0.f, 0.f}; }
}

// MoeGateRule::ClampedGlu (larql-compute/src/pipeline/moe.rs:88-92): g = min(g, L); u = clamp(u, -L, L);
// (u + 1) * (g * sigmoid(alpha * g))
__device__ __forceinline__ float clamped_glu(float g, float u, float L, float al) {
    const float gc = fminf(g, L);
    const float uc = u < -L ? -L : (u > L ? L : u);
    return (uc + 1.0f) * (gc * (1.0f / (1.0f + expf(-(gc * al)))));
}

// The three bf16 terms of two activations, packed pairwise (a in the low half): x = t0 + t1 + t2 exactly.  An infinite
// or NaN activation stays in the first term alone (its residual would be a NaN of its own making).
__device__ __forceinline__ void mx4_terms(float a, float b, uint32_t (&t)[3]) {
    const uint32_t ab = __builtin_bit_cast(uint32_t, a), bb = __builtin_bit_cast(uint32_t, b);
    uint32_t a0 = ab & 0xFFFF0000u, b0 = bb & 0xFFFF0000u;
    float ra = a - __builtin_bit_cast(float, a0), rb = b - __builtin_bit_cast(float, b0);  // exact
    if ((ab & 0x7F800000u) == 0x7F800000u) { ra = 0.f; a0 = (ab & 0x007FFFFFu) ? (a0 | 0x00400000u) : a0; }
    if ((bb & 0x7F800000u) == 0x7F800000u) { rb = 0.f; b0 = (bb & 0x007FFFFFu) ? (b0 | 0x00400000u) : b0; }
    const uint32_t a1 = __builtin_bit_cast(uint32_t, ra) & 0xFFFF0000u, b1 = __builtin_bit_cast(uint32_t, rb) & 0xFFFF0000u;
    ra -= __builtin_bit_cast(float, a1);
    rb -= __builtin_bit_cast(float, b1);
    const uint32_t a2 = __builtin_bit_cast(uint32_t, ra) & 0xFFFF0000u, b2 = __builtin_bit_cast(uint32_t, rb) & 0xFFFF0000u;
    t[0] = (a0 >> 16) | b0;
    t[1] = (a1 >> 16) | b1;
    t[2] = (a2 >> 16) | b2;
}

// One token's operands of all `cw` steps of a wavefront: every lane splits its two activations of a step into terms
// and the wavefront transposes them through `scratch` (768 bytes per step: term plane i at i*256, element e at 2e)
// into the operand layout, so the LDS round trip is paid once per token.  The token's terms become A rows
// 4*trow .. 4*trow+2 of `ops` (the other rows are left as they are); `wq` scales the activation (a folded job's
// routing weight) when `scaled` is set.
template <int Q>
__device__ __forceinline__ void mx4_setup_token(const GemvJob &j, bool scaled, float wq, const Mx4In (&in)[kMx4MaxSteps],
                                                Mx4Ops &ops, uint32_t trow, uint32_t cw, uint32_t lane, uint8_t *scratch) {
    const uint32_t i = lane & 15u, kg = lane >> 4;
#pragma unroll
    for (int s = 0; s < kMx4MaxSteps; s++) {
        if ((uint32_t)s >= cw) continue;
        float2_t v, u;
        mx4_pair(j, in[s], Q, v, u);
        if (j.x_glu) {  // (activations past the row end are zeros: they stay zero)
            v.x = clamped_glu(v.x, u.x, j.glu_limit, j.glu_alpha);
            v.y = clamped_glu(v.y, u.y, j.glu_limit, j.glu_alpha);
        }
        if (scaled) { v.x *= wq; v.y *= wq; }  // the expert's routing weight rides in its activation
        uint32_t t[3];
        mx4_terms(v.x, v.y, t);
        uint32_t *sp = reinterpret_cast<uint32_t *>(scratch + s * kMx4TermBytes) + lane;
        sp[0] = t[0]; sp[64] = t[1]; sp[128] = t[2];
    }
    asm volatile("" ::: "memory");  // same wavefront: LDS executes its writes before the reads that follow
    if ((i >> 2) == trow && (i & 3u) < 3u) {
#pragma unroll
        for (int s = 0; s < kMx4MaxSteps; s++) {
            if ((uint32_t)s >= cw) continue;
            const uint8_t *rp = scratch + s * kMx4TermBytes + (i & 3u) * 256 + kg * 64;  // elements 32kg .. 32kg+31 of term i%4
#pragma unroll
            for (int m = 0; m < 4; m++) {
                const u32x4 op = *reinterpret_cast<const u32x4 *>(rp + 16 * m);
                ops.a[s][m].u[0] = op.x; ops.a[s][m].u[1] = op.y; ops.a[s][m].u[2] = op.z; ops.a[s][m].u[3] = op.w;
            }
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the scratch is reused by the next token
}

__device__ __forceinline__ void mx4_clear_ops(Mx4Ops &ops) {
#pragma unroll
    for (int s = 0; s < kMx4MaxSteps; s++)
#pragma unroll
        for (int m = 0; m < 4; m++) ops.a[s][m].u[0] = ops.a[s][m].u[1] = ops.a[s][m].u[2] = ops.a[s][m].u[3] = 0u;
}

// The operands of every token of a job: token q's terms are A rows 4q .. 4q+2, so its sums come out in D rows of
// their own (lanes with rq = q).
__device__ __forceinline__ void mx4_setup_ops(const GemvJob &j, const Mx4In (&in)[kMx4MaxSteps], Mx4Ops &ops, uint32_t cw,
                                              uint32_t lane, uint8_t *scratch) {
    const uint32_t ntok = mx4_tokens(j);
    mx4_clear_ops(ops);
    mx4_setup_token<0>(j, false, 1.0f, in, ops, 0, cw, lane, scratch);
    if (ntok > 1) mx4_setup_token<1>(j, false, 1.0f, in, ops, 1, cw, lane, scratch);
    if (ntok > 2) mx4_setup_token<2>(j, false, 1.0f, in, ops, 2, cw, lane, scratch);
    if (ntok > 3) mx4_setup_token<3>(j, false, 1.0f, in, ops, 3, cw, lane, scratch);
}

// One step of a wave-tile from its LDS slot: the lane's block (16 bytes of nibbles, scale byte `sc`) against the four
// operands of the step.  `live` is false for a block past the row end or of an expert outside the bank.
__device__ __forceinline__ f32x4 mx4_step_mfma(const BfOp (&a)[4], const u32x4 q, uint32_t sc, bool live, f32x4 D) {
    float scale = __builtin_bit_cast(float, sc << 23);                       // 2^(sc-127); 0 -> 0.0 as the reference reads it
    scale = sc == 255u ? __builtin_bit_cast(float, 0x7FC00000u) : scale;     // 255 -> NaN
    scale = live ? scale : 0.0f;
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int m = 0; m < 4; m++) {
        BfOp b;
        b.u[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[m], scale, 0));
        b.u[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[m], scale, 1));
        b.u[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[m], scale, 2));
        b.u[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[m], scale, 3));
        D = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[m].v, b.v, D, 0, 0, 0);
    }
    return D;
}

// loads of the younger wave-tiles that may still be in flight: CW nibble copies and one scale copy each (two with five steps)
#define LARQL_MX4_WAIT_CASE(CW) case CW: LARQL_WAIT_VMCNT((CW + 1 + (CW > 4)) * (kMx4Stages - 1)); break;

// tiles [tile_a, tile_b) of one job
__device__ __forceinline__ void run_mxfp4_mfma(const GemvJob &j, const Mx4Sel &sel, uint32_t tile_a, uint32_t tile_b, uint8_t *lds,
                                               uint32_t slot_bytes, uint32_t &parity, bool fresh) {
    constexpr int NS = kMx4Stages, R = kMx4BatchTiles;
    const uint32_t lane = threadIdx.x & 63u, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nw_launch = blockDim.x >> 6;
    const uint32_t jr = lane & 15u, kg = lane >> 4;
    // up to four tokens share the weights: token q rides in A rows 4q .. 4q+2, its sums leave in D rows 4q .. 4q+2 (lanes rq = q)
    const uint32_t ntok = mx4_tokens(j);
    const uint32_t hw_sh = ntok == 1 ? 0u : (ntok == 2 ? 1u : 2u), hw = 1u << hw_sh;  // partial sums per weight row and wavefront
    const uint32_t nwj = j.rpp, steps = j.cpr, cw = (uint32_t)j.pad, PW = nwj * hw;
    const uint32_t rows = (uint32_t)j.rows, k = (uint32_t)j.k, nb = k / 32, row_bytes = (uint32_t)j.row_bytes;
    uint8_t *ring = lds + wv * (NS * slot_bytes);
    float *part = reinterpret_cast<float *>(lds + nw_launch * (NS * slot_bytes));
    const uint32_t step0 = wv * cw;
    const bool working = wv < nwj && step0 < steps;

    uint32_t blk[kMx4MaxSteps];   // this lane's block of each step, clamped into the row
    bool valid[kMx4MaxSteps];
#pragma unroll
    for (int s = 0; s < kMx4MaxSteps; s++) {
        const uint32_t b = (step0 + s) * 4 + kg;
        valid[s] = working && (uint32_t)s < cw && b < nb;
        blk[s] = min(b, nb - 1);
    }

    // scale bytes: lane (jr, c) copies the dword that holds blocks 4(step0+c) .. +3 of row jr, moved back to end with the
    // row where the row has fewer; lane (jr, kg) then finds the byte of its block of step s in slot 16s + jr
    const uint32_t sc_dw = min((step0 + kg) * 4, nb - 4);
    const uint32_t sc_dw4 = min((step0 + 4) * 4, nb - 4);
    uint32_t sc_at[kMx4MaxSteps];
#pragma unroll
    for (int s = 0; s < kMx4MaxSteps; s++) sc_at[s] = (16u * s + jr) * 4 + (blk[s] - min((step0 + s) * 4, nb - 4));
    const uint32_t wro_full = jr * row_bytes, sro_full = jr * nb;
    const uint32_t nt = tile_b - tile_a;
    uint32_t it_tile = tile_a, n_issue = 0;
    auto issue = [&]() {
        const uint32_t tl = min(it_tile, tile_b - 1);  // past the end: the last tile again (uniform load counts)
        // wave-uniform 64-bit bases + per-lane 32-bit offsets (the lane's row within the tile, clamped into the matrix)
        const uint32_t rb = tl * 16;
        const uint8_t *wbase = sel.w[0] + (size_t)rb * row_bytes;
        const uint8_t *sbase = sel.aux[0] + (size_t)rb * nb;
        uint32_t wro = wro_full, sro = sro_full;
        if (rb + 16 > rows) {  // ragged last tile only
            const uint32_t rl = min(jr, rows - 1 - rb);
            wro = rl * row_bytes;
            sro = rl * nb;
        }
        uint8_t *lp = ring + (n_issue % NS) * slot_bytes;
#pragma unroll
        for (int s = 0; s < kMx4MaxSteps; s++)
            if ((uint32_t)s < cw) __builtin_amdgcn_global_load_lds((g_vp)(wbase + (wro + blk[s] * 16)), (lds_vp)(lp + s * 1024), 16, 0, 0);
        // the e8m0 bytes of all the wavefront's steps in one copy: lane (row jr, step c = lane/16 < cw) brings the four
        // scale bytes of its row and step as one dword into slot `lane` (the dword is not aligned in general)
        if (lane < 16 * cw) __builtin_amdgcn_global_load_lds((g_vp)(sbase + (sro + sc_dw)), (lds_vp)(lp + cw * 1024), 4, 0, 0);
        if (cw > 4 && lane < 16) __builtin_amdgcn_global_load_lds((g_vp)(sbase + (sro + sc_dw4)), (lds_vp)(lp + cw * 1024 + 256), 4, 0, 0);  // a fifth step's
        n_issue++;
        if (it_tile < tile_b) it_tile++;
    };
    // the activations of all this wavefront's steps are requested first and together, ahead of the weight tiles in
    // the in-order return queue; their terms are prepared while the first tiles are on their way (the ring's last
    // slot is still free and serves as scratch)
    Mx4In xin[kMx4MaxSteps];
#pragma unroll
    for (int s = 0; s < kMx4MaxSteps; s++)
        if (working && (uint32_t)s < cw) xin[s] = mx4_load_step(j, step0 + s, lane);
    if (working)
        for (int s = 0; s < NS - 1; s++) issue();
    Mx4Ops ops;
    if (working) mx4_setup_ops(j, xin, ops, cw, lane, ring + (NS - 1) * slot_bytes);  // (768 bytes per step fit the 1024 of a slot's step)

    // The two partial-sum areas are laid out for this job's own `hw`; the job this workgroup served before may have used
    // another layout, and its last row sums may still be read by a slower wavefront: wait for everybody before writing
    // (`fresh`: the workgroup's first job of the launch has nobody to wait for).
    if (!fresh) __builtin_amdgcn_s_barrier();
    uint32_t n_use = 0;
    for (uint32_t tb = 0; tb < nt; tb += R) {
        float *pb = part + parity * (R * 16 * nw_launch * hw);
        const uint32_t nbt = min((uint32_t)R, nt - tb);
        if (working) {
            for (uint32_t tl = 0; tl < nbt; tl++) {
                issue();
                switch (cw) {  // at most NS-1 younger wave-tiles in flight: the oldest has landed
                    LARQL_MX4_WAIT_CASE(1) LARQL_MX4_WAIT_CASE(2) LARQL_MX4_WAIT_CASE(3) LARQL_MX4_WAIT_CASE(4) LARQL_MX4_WAIT_CASE(5)
                }
                asm volatile("" ::: "memory");
                const uint8_t *slot = ring + (n_use % NS) * slot_bytes;
                f32x4 D = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < kMx4MaxSteps; s++) {
                    if ((uint32_t)s < cw) {
                        const u32x4 q = *reinterpret_cast<const u32x4 *>(slot + s * 1024 + lane * 16);
                        const uint32_t sc = slot[cw * 1024 + sc_at[s]];
                        D = mx4_step_mfma(ops.a[s], q, sc, valid[s], D);  // (blocks past the row end do not exist)
                    }
                }
                n_use++;
                // the three term sums of token kg for weight row jr
                if (kg < hw) pb[(tl * 16 + jr) * PW + wv * hw + kg] = (D[0] + D[1]) + D[2];
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const uint32_t row_base = (tile_a + tb) * 16;
        const uint32_t nwork = min(nwj, (steps + cw - 1) / cw);
        // hw threads per weight row: thread h adds up token h's slot of every wavefront (the same order of additions
        // per token whatever the number of tokens that share the job)
        for (uint32_t rr = threadIdx.x >> hw_sh; rr < nbt * 16; rr += blockDim.x >> hw_sh) {
            const uint32_t h = threadIdx.x & (hw - 1u);
            float s = 0.f;
            for (uint32_t w = 0; w < nwork; w++) s += pb[rr * PW + w * hw + h];
            const uint32_t row = row_base + rr;
            if (h < ntok && row < rows) {
                if (!sel.ok[0]) s = 0.0f;  // an expert outside the bank: no contribution (its stand-in's bytes were read, not used)
                else if (j.bias) s += ((const GLOBAL_AS float *)sel.bias[0])[(size_t)row * j.bias_step];
                ((g_f32wp)(j.out + mx4_out_off(j, h)))[row] = s;
            }
        }
        parity ^= 1u;
    }
}

// A job folded over experts (GemvJob::combine_w): row tiles [tile_a, tile_b) of the result, each the sum over the job's
// `nq` experts of (that expert's 16 weight rows) . (that expert's activation, scaled by its routing weight).  Expert q's
// activation terms are A rows 4q .. 4q+2 of ONE operand set, prepared once per job; expert q's weights meet the whole
// set and accumulate into that expert's own D registers, of which only rows 4q .. 4q+2 (lanes rq = q) mean anything:
// lane (j, rq) ends with expert rq's three term sums for weight row j, and the experts meet in the fold of the row
// partials.  The walk is expert-outermost within a batch of R row tiles.
__device__ __forceinline__ void run_mxfp4_fold(const GemvJob &j, const Mx4Sel &sel, uint32_t tile_a, uint32_t tile_b, uint8_t *lds,
                                               uint32_t slot_bytes, uint32_t &parity) {
    constexpr int NS = kMx4Stages, R = kMx4FoldTiles;
    const uint32_t lane = threadIdx.x & 63u, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nw_launch = blockDim.x >> 6;
    const uint32_t jr = lane & 15u, kg = lane >> 4;
    const uint32_t nq = mx4_tokens(j);
    constexpr uint32_t hw = 4, hw_sh = 2;  // one partial sum per expert, weight row and wavefront
    const uint32_t nwj = j.rpp, steps = j.cpr, cw = (uint32_t)j.pad, PW = nwj * hw;
    const uint32_t rows = (uint32_t)j.rows, k = (uint32_t)j.k, nb = k / 32, row_bytes = (uint32_t)j.row_bytes;
    uint8_t *ring = lds + wv * (NS * slot_bytes);
    float *part = reinterpret_cast<float *>(lds + nw_launch * (NS * slot_bytes));
    const uint32_t step0 = wv * cw;
    const bool working = wv < nwj && step0 < steps;

    uint32_t blk[kMx4MaxSteps];
    bool valid[kMx4MaxSteps];
#pragma unroll
    for (int s = 0; s < kMx4MaxSteps; s++) {
        const uint32_t b = (step0 + s) * 4 + kg;
        valid[s] = working && (uint32_t)s < cw && b < nb;
        blk[s] = min(b, nb - 1);
    }
    const uint32_t sc_dw = min((step0 + kg) * 4, nb - 4);
    const uint32_t sc_dw4 = min((step0 + 4) * 4, nb - 4);
    uint32_t sc_at[kMx4MaxSteps];
#pragma unroll
    for (int s = 0; s < kMx4MaxSteps; s++) sc_at[s] = (16u * s + jr) * 4 + (blk[s] - min((step0 + s) * 4, nb - 4));
    const uint32_t wro_full = jr * row_bytes, sro_full = jr * nb;
    const uint32_t nt = tile_b - tile_a;
    // the order of the virtual tiles: batch of R row tiles, then expert, then row tile of the batch
    uint32_t it_tb = 0, it_q = 0, it_tl = 0, n_issue = 0;
    auto issue = [&]() {
        const uint32_t tl = min(tile_a + it_tb + it_tl, tile_b - 1);  // past the end: the last tile again (uniform load counts)
        const uint32_t rb = tl * 16;
        const uint8_t *wq = it_q == 1 ? sel.w[1] : (it_q == 2 ? sel.w[2] : (it_q == 3 ? sel.w[3] : sel.w[0]));
        const uint8_t *aq = it_q == 1 ? sel.aux[1] : (it_q == 2 ? sel.aux[2] : (it_q == 3 ? sel.aux[3] : sel.aux[0]));
        const uint8_t *wbase = wq + (size_t)rb * row_bytes;
        const uint8_t *sbase = aq + (size_t)rb * nb;
        uint32_t wro = wro_full, sro = sro_full;
        if (rb + 16 > rows) {
            const uint32_t rl = min(jr, rows - 1 - rb);
            wro = rl * row_bytes;
            sro = rl * nb;
        }
        uint8_t *lp = ring + (n_issue % NS) * slot_bytes;
#pragma unroll
        for (int s = 0; s < kMx4MaxSteps; s++)
            if ((uint32_t)s < cw) __builtin_amdgcn_global_load_lds((g_vp)(wbase + (wro + blk[s] * 16)), (lds_vp)(lp + s * 1024), 16, 0, 0);
        if (lane < 16 * cw) __builtin_amdgcn_global_load_lds((g_vp)(sbase + (sro + sc_dw)), (lds_vp)(lp + cw * 1024), 4, 0, 0);
        if (cw > 4 && lane < 16) __builtin_amdgcn_global_load_lds((g_vp)(sbase + (sro + sc_dw4)), (lds_vp)(lp + cw * 1024 + 256), 4, 0, 0);  // a fifth step's
        n_issue++;
        if (it_tb < nt) {  // next virtual tile (stays on the last one once the list is exhausted)
            const uint32_t nbt = min((uint32_t)R, nt - it_tb);
            if (++it_tl >= nbt) {
                it_tl = 0;
                if (++it_q >= nq) { it_q = 0; it_tb += R; }
            }
            if (it_tb >= nt) { it_tb = nt - 1 - ((nt - 1) % R); it_q = nq - 1; it_tl = (nt - 1) % R; }
        }
    };
    Mx4In xin[kMx4MaxSteps];
#pragma unroll
    for (int s = 0; s < kMx4MaxSteps; s++)
        if (working && (uint32_t)s < cw) xin[s] = mx4_load_step(j, step0 + s, lane);
    if (working)
        for (int s = 0; s < NS - 1; s++) issue();

    // every expert's operands, once per job (the ring's last slot is still free and serves as scratch)
    Mx4Ops ops;
    if (working) {
        uint8_t *scratch = ring + (NS - 1) * slot_bytes;
        mx4_clear_ops(ops);
        mx4_setup_token<0>(j, true, sel.cw[0], xin, ops, 0, cw, lane, scratch);
        if (nq > 1) mx4_setup_token<1>(j, true, sel.cw[1], xin, ops, 1, cw, lane, scratch);
        if (nq > 2) mx4_setup_token<2>(j, true, sel.cw[2], xin, ops, 2, cw, lane, scratch);
        if (nq > 3) mx4_setup_token<3>(j, true, sel.cw[3], xin, ops, 3, cw, lane, scratch);
    }
    __builtin_amdgcn_s_barrier();  // (the partial-sum areas follow this job's layout: see run_mxfp4_mfma)
    uint32_t n_use = 0;
    for (uint32_t tb = 0; tb < nt; tb += R) {
        float *pb = part + parity * (R * 16 * nw_launch * hw);
        const uint32_t nbt = min((uint32_t)R, nt - tb);
        if (working) {
            float acc[R];  // this lane's expert (rq = kg) only
#pragma unroll
            for (int t = 0; t < R; t++) acc[t] = 0.f;
#pragma unroll
            for (int q = 0; q < kMx4MaxTokens; q++) {
                if ((uint32_t)q >= nq) break;
#pragma unroll
                for (int tl = 0; tl < R; tl++) {
                    if ((uint32_t)tl >= nbt) break;
                    issue();
                    switch (cw) {
                        LARQL_MX4_WAIT_CASE(1) LARQL_MX4_WAIT_CASE(2) LARQL_MX4_WAIT_CASE(3) LARQL_MX4_WAIT_CASE(4) LARQL_MX4_WAIT_CASE(5)
                    }
                    asm volatile("" ::: "memory");
                    const uint8_t *slot = ring + (n_use % NS) * slot_bytes;
                    f32x4 D = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < kMx4MaxSteps; s++) {
                        if ((uint32_t)s < cw) {
                            const u32x4 qw = *reinterpret_cast<const u32x4 *>(slot + s * 1024 + lane * 16);
                            const uint32_t sc = slot[cw * 1024 + sc_at[s]];
                            // blocks past the row end do not exist; an expert outside the bank has no weights
                            D = mx4_step_mfma(ops.a[s], qw, sc, valid[s] && sel.ok[q], D);
                        }
                    }
                    n_use++;
                    // rows 4q .. 4q+2 of D are expert q's term sums; the other rows met another expert's activation
                    if (kg == (uint32_t)q) acc[tl] = (D[0] + D[1]) + D[2];
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the slot's reads are done before anything reuses it
                }
            }
#pragma unroll
            for (int tl = 0; tl < R; tl++) {
                if ((uint32_t)tl >= nbt) break;
                pb[(tl * 16 + jr) * PW + wv * hw + kg] = kg < nq ? acc[tl] : 0.f;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const uint32_t row_base = (tile_a + tb) * 16;
        const uint32_t nwork = min(nwj, (steps + cw - 1) / cw);
        for (uint32_t rr = threadIdx.x >> hw_sh; rr < nbt * 16; rr += blockDim.x >> hw_sh) {
            const uint32_t h = threadIdx.x & (hw - 1u);
            float s = 0.f;
            for (uint32_t w = 0; w < nwork; w++) s += pb[rr * PW + w * hw + h];
            s = dpp_add<0xB1>(s);  // quad_perm [1,0,3,2]: experts 0+1, 2+3
            s = dpp_add<0x4E>(s);  // quad_perm [2,3,0,1]: all four
            const uint32_t row = row_base + rr;
            if (h == 0 && row < rows) {
                if (j.bias) {  // + sum_q w_q * bias_q[row], in selection order
#pragma unroll
                    for (int q = 0; q < kMx4MaxTokens; q++)
                        if ((uint32_t)q < nq && sel.ok[q]) s += sel.cw[q] * ((const GLOBAL_AS float *)sel.bias[q])[(size_t)row * j.bias_step];
                }
                ((g_f32wp)j.out)[row] = s;
            }
        }
        parity ^= 1u;
    }
}

// ---------------------------------------------------------------------------
// One token through k <= 4 experts of an MXFP4 bank (the decode shape of ExpertWeightFfn::moe_block,
// larql-compute/src/ffn/expert_weight/mod.rs, with the pipeline of larql-compute/src/pipeline/moe.rs:469-541): one launch for the gate / up
// projections of the selected experts, one for the down projections folded over the experts.  The arithmetic is the
// matrix-core scheme above (same operands, same order of additions per row as a one-token job of the general kernel);
// what differs is the way in: the arguments are a small block in the kernel's own argument space, the token's
// activations are requested before anything else, the selection (or the read of it) overlaps them, and a deeper ring
// (up to four wave-tiles in flight per wavefront) covers the memory latency of a launch that lasts only a few
// round trips.
//   gate/up stage: the 16-row tiles of the k x n_mats matrices form one list, shared out evenly over the workgroups.
//                  With a fused interleaved matrix (gate row 2i, up row 2i+1) the fold of the row partials has both
//                  halves of an output side by side: it applies ClampedGlu and writes the activation of the down stage
//                  already split into its three bf16 terms (`terms`: [term][slot < k][kpad] bf16), so the down stage
//                  loads its A operands as stored.
//   down stage:    a workgroup owns row tiles of the result; expert q's activation is A rows 4q .. 4q+2 of one operand
//                  set, each expert's tile meets the whole set and lane (j, rq) keeps expert rq's sums, scaled by the
//                  expert's routing weight; the experts meet in the fold of the row partials, the biases (weighted)
//                  join there.  Without `terms` (gate and up apart) the activations are gated and split here.
// ---------------------------------------------------------------------------
constexpr int kMoe1BatchTiles = 4;
constexpr int moe1_stages(int cw) { return cw <= 3 ? 3 : 3; }  // ring slots per wavefront that fit the LDS beside the partials
constexpr uint32_t moe1_slot_bytes(int cw) { return (uint32_t)cw * kMx4StepBytes + (cw > 4 ? 512u : 256u); }  // steps, then a scale dword per lane (two with five steps)
__device__ const uint32_t kMoe1Zeros[4] = {0u, 0u, 0u, 0u};      // what an operand lane without an activation loads

// CW: 128-element steps per wavefront (the row length decides); NS: ring slots per wavefront
template <bool DOWN, int CW, int NS>
__global__ void __launch_bounds__(kMx4MaxWaves * 64) moe1_kernel(const Moe1Args A) {
    extern __shared__ __attribute__((aligned(16))) uint8_t m1_lds[];
    constexpr int R = DOWN ? kMoe1BatchTiles : 2 * kMoe1BatchTiles;  // row tiles between two folds of the row partials
    constexpr uint32_t cw = CW, slot_bytes = moe1_slot_bytes(CW);
    const uint32_t lane = threadIdx.x & 63u, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nw_launch = blockDim.x >> 6;
    const uint32_t jr = lane & 15u, kg = lane >> 4;
    const uint32_t kdim = A.kdim, nb = kdim / 32, row_bytes = nb * 16, steps = (kdim + 127) / 128, nwj = A.nw;
    const uint32_t rows = A.rows, nq = min(A.k, kMoe1MaxK), TR = A.tile_rows;  // (rows per tile: 16, or fewer to share a short result out evenly)
    uint8_t *ring = m1_lds + wv * (NS * slot_bytes);
    float *part = reinterpret_cast<float *>(m1_lds + nw_launch * (NS * slot_bytes));
    const uint32_t step0 = wv * cw;
    const bool working = wv < nwj && step0 < steps;

    // 0. what the selection needs: the logits, or the selection as stored where an earlier launch made it
    const bool has_logit = A.logits && lane < A.n_experts;
    float logit = has_logit ? ((const GLOBAL_AS float *)A.logits)[lane] : 0.0f;
    if (has_logit && A.router_bias) logit += ((const GLOBAL_AS float *)A.router_bias)[lane];
    const uint32_t ev = (!A.logits && lane < nq) ? ((const GLOBAL_AS uint32_t *)A.experts)[lane] : 0u;
    const float wl = (!A.logits && DOWN && lane < nq) ? ((const GLOBAL_AS float *)A.weights)[lane] : 0.0f;

    // 1. the activations of this wavefront's K-range: nothing they need has to be waited for
    GemvJob jx = {};  // (the fields the activation helpers read)
    jx.k = kdim; jx.x = A.x; jx.x_glu = A.x_glu; jx.glu_limit = A.glu_limit; jx.glu_alpha = A.glu_alpha;
    if (DOWN) { jx.batch = nq; jx.x_stride = A.x_slot_stride; jx.x_off[0] = (int64_t)(2 * A.x_slot_stride); jx.x_off[1] = (int64_t)(3 * A.x_slot_stride); }
    Mx4In xin[kMx4MaxSteps];
    Mx4Ops ops;
    const bool pre = DOWN && A.terms != nullptr;  // the activations arrive as operand terms
    auto load_operands = [&]() {
        // lane (row i = 4q + term, kg): eight consecutive bf16 of term plane `term`, slot q, per MFMA; a lane without an
        // activation (fourth row of a slot, slot >= k, elements past the row end) reads zeros
        const uint32_t tq = jr >> 2, term = jr & 3u;
        const bool mine = working && tq < nq && term < 3u;
        const uint16_t *tp = A.terms + ((size_t)term * nq + tq) * A.terms_kpad;
#pragma unroll
        for (int s = 0; s < CW; s++) {
#pragma unroll
            for (int m = 0; m < 4; m++) {
                const uint32_t el = (step0 + s) * 128 + 32 * kg + 8 * m;  // (kdim % 32 == 0: a group of eight is inside or outside)
                const uint16_t *src = (mine && el < kdim) ? tp + el : reinterpret_cast<const uint16_t *>(kMoe1Zeros);
                const u32x4 t = *(const GLOBAL_AS u32x4 *)src;
                ops.a[s][m].u[0] = t.x; ops.a[s][m].u[1] = t.y; ops.a[s][m].u[2] = t.z; ops.a[s][m].u[3] = t.w;
            }
        }
    };
    if (pre) {
        // (fetched below, behind the first weight tile)
    } else {
#pragma unroll
        for (int s = 0; s < CW; s++)
            if (working) xin[s] = mx4_load_step(jx, step0 + s, lane);
    }

    // 2. the selection
    uint32_t e[kMoe1MaxK];
    float cwt[kMoe1MaxK];
    bool ok[kMoe1MaxK];
    if (A.logits) {
        uint32_t idx[kRouterMaxK];
        float wt[kRouterMaxK];
        const bool writer = A.experts && blockIdx.x == 0 && wv == 0;  // (wave-uniform)
        if (writer || DOWN) router_select_lane<true>(logit, A.n_experts, nq, A.policy, lane, idx, wt);
        else router_select_lane<false>(logit, A.n_experts, nq, A.policy, lane, idx, wt);
#pragma unroll
        for (int q = 0; q < (int)kMoe1MaxK; q++) {
            e[q] = __builtin_amdgcn_readfirstlane(idx[q]);
            cwt[q] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, wt[q])));
        }
        if (writer && lane == 0) {
#pragma unroll
            for (int r = 0; r < (int)kMoe1MaxK; r++)
                if ((uint32_t)r < nq) { A.experts[r] = idx[r]; A.weights[r] = wt[r]; }
        }
    } else {
#pragma unroll
        for (int q = 0; q < (int)kMoe1MaxK; q++) {
            e[q] = (uint32_t)__builtin_amdgcn_readlane((int)ev, q);
            cwt[q] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wl), q));
        }
    }
    // expert q's matrices (wave-uniform 64-bit bases); an id outside the bank contributes nothing and reads nothing of it
    const uint8_t *wq[kMoe1MaxK], *sq[kMoe1MaxK];
#pragma unroll
    for (int q = 0; q < (int)kMoe1MaxK; q++) {
        ok[q] = (uint32_t)q < nq && e[q] < A.n_experts;
        e[q] = ok[q] ? e[q] : 0u;
        cwt[q] = ok[q] ? cwt[q] : 0.0f;
        wq[q] = A.w[0] + (size_t)e[q] * A.w_stride;
        sq[q] = A.aux[0] + (size_t)e[q] * A.aux_stride;
    }
    // (second matrix of a slot: the same expert in the up bank)
    const size_t m1_w = A.n_mats == 2 ? (size_t)(A.w[1] - A.w[0]) : 0, m1_s = A.n_mats == 2 ? (size_t)(A.aux[1] - A.aux[0]) : 0;
    auto expert_of = [&](uint32_t q) { return q == 1 ? e[1] : (q == 2 ? e[2] : (q == 3 ? e[3] : e[0])); };
    auto ok_of = [&](uint32_t q) { return q == 1 ? ok[1] : (q == 2 ? ok[2] : (q == 3 ? ok[3] : ok[0])); };
    auto weight_of = [&](uint32_t q) { return q == 1 ? cwt[1] : (q == 2 ? cwt[2] : (q == 3 ? cwt[3] : cwt[0])); };

    // 3. this workgroup's share.  Gate/up: row tiles [va, vb) of the list (slot, matrix, row tile); down: row tiles of
    // the result, each met by the k experts in turn (expert innermost).
    const uint32_t tpm = (rows + TR - 1) / TR;
    const uint32_t n_units = DOWN ? tpm : nq * A.n_mats * tpm;
    const uint32_t va = n_units * blockIdx.x / gridDim.x, vb = n_units * (blockIdx.x + 1) / gridDim.x;  // (the host keeps the products below 2^32)
    if (va >= vb) return;
    const uint32_t nt = vb - va, n_virtual = DOWN ? nt * nq : nt;

    // per-lane parts of a wave-tile's addresses: the lane's row within the tile and its block of each step
    // (a block past the row end is the row's last block again: its activations are zeros, so it adds nothing)
    uint32_t woff[CW], sc_at[CW];
#pragma unroll
    for (int s = 0; s < CW; s++) {
        const uint32_t b = (step0 + s) * 4 + kg, bc = min(b, nb - 1);
        woff[s] = jr * row_bytes + bc * 16;
        sc_at[s] = (16u * s + jr) * 4 + (bc - min((step0 + s) * 4, nb - 4));
    }
    const uint32_t soff = jr * nb + min((step0 + kg) * 4, nb - 4), soff4 = jr * nb + min((step0 + 4) * 4, nb - 4);
    const uint32_t tile_w = TR * row_bytes, tile_s = TR * nb;

    // issue cursor: (segment = slot * n_mats + matrix, row tile) / (row tile, expert)
    uint32_t it_seg = DOWN ? 0u : va / tpm, it_t = DOWN ? va : va - (va / tpm) * tpm, it_q = 0, it_left = n_virtual, slot_i = 0;
    // the loads of the cursor's wave-tile (every lane takes part: no branch sits between the loads, so what is in flight
    // can be counted; lanes whose step does not exist copy a neighbouring block that nothing reads)
    auto issue_loads = [&]() {
        const uint32_t q = DOWN ? it_q : (A.n_mats == 2 ? it_seg >> 1 : it_seg);
        const uint8_t *wbase = q == 1 ? wq[1] : (q == 2 ? wq[2] : (q == 3 ? wq[3] : wq[0]));
        const uint8_t *sbase = q == 1 ? sq[1] : (q == 2 ? sq[2] : (q == 3 ? sq[3] : sq[0]));
        if (!DOWN && A.n_mats == 2 && (it_seg & 1u)) { wbase += m1_w; sbase += m1_s; }
        wbase += (size_t)it_t * tile_w;
        sbase += (size_t)it_t * tile_s;
        // lanes past the tile's last row (a tile of fewer than 16 rows, a ragged last tile) read that row again
        const uint32_t last = min(TR - 1, rows - 1 - it_t * TR), back = jr > last ? jr - last : 0u;
        const uint32_t bw = back * row_bytes, bs = back * nb;
        uint8_t *lp = ring + slot_i * slot_bytes;
#pragma unroll
        for (int s = 0; s < CW; s++)
            __builtin_amdgcn_global_load_lds((g_vp)(wbase + (woff[s] - bw)), (lds_vp)(lp + s * 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((g_vp)(sbase + (soff - bs)), (lds_vp)(lp + cw * 1024), 4, 0, 0);
        if (CW > 4) __builtin_amdgcn_global_load_lds((g_vp)(sbase + (soff4 - bs)), (lds_vp)(lp + cw * 1024 + 256), 4, 0, 0);
        slot_i = slot_i + 1 == NS ? 0u : slot_i + 1;
    };
    auto advance = [&]() {
        if (DOWN) {
            if (++it_q >= nq) { it_q = 0; it_t++; }
        } else if (++it_t >= tpm) { it_t = 0; it_seg++; }
    };
    auto issue = [&]() {  // the next wave-tile, if there is one (nothing is read twice: the waits below count what is really in flight)
        if (it_left == 0) return;
        issue_loads();
        it_left--;
        advance();
    };
    // the first NS-1 wave-tiles without a branch around their loads (a share of fewer tiles reads its last one again)
    if (working) {
#pragma unroll
        for (int s = 0; s + 1 < NS; s++) {
            issue_loads();
            if (it_left > 1) { it_left--; advance(); } else it_left = 0;
            if (s == 0 && pre) load_operands();  // behind the first tile: they return in order, the tile first
        }
    }
    if (pre) {
        // the operands are in (and the first tile before them) once only the younger tiles' loads are outstanding
        LARQL_WAIT_VMCNT((CW + 1 + (CW > 4)) * (NS - 2));
    }

    // 4. operands, while the first tiles fly (the ring's last slot is still free and serves as scratch)
    if (working && !pre) {
        uint8_t *scratch = ring + (NS - 1) * slot_bytes;
        mx4_clear_ops(ops);
        mx4_setup_token<0>(jx, false, 1.0f, xin, ops, 0, cw, lane, scratch);
        if (DOWN) {
            if (nq > 1) mx4_setup_token<1>(jx, false, 1.0f, xin, ops, 1, cw, lane, scratch);
            if (nq > 2) mx4_setup_token<2>(jx, false, 1.0f, xin, ops, 2, cw, lane, scratch);
            if (nq > 3) mx4_setup_token<3>(jx, false, 1.0f, xin, ops, 3, cw, lane, scratch);
        }
    }

    constexpr uint32_t hw = DOWN ? 4u : 1u;  // partial sums per weight row and wavefront (down: one per expert)
    const uint32_t PW = nwj * hw, nwork = min(nwj, (steps + cw - 1) / cw);
    uint32_t use_i = 0, parity = 0;
    uint32_t f_seg = DOWN ? 0u : va / tpm, f_t = DOWN ? va : va - (va / tpm) * tpm;  // the fold's cursor: first tile of the batch
    uint32_t tl = 0, cq = 0;   // row tile within the batch, expert within the tile
    float acc = 0.f;
    for (uint32_t v = 0; v < n_virtual; v++) {
        float *pb = part + parity * (R * 16 * nw_launch * hw);
        if (working) {
            issue();
            {   // wave-tiles younger than the one about to be used: it has landed when only their loads are outstanding
                constexpr int L = CW + 1 + (CW > 4);  // loads per wave-tile
                const uint32_t younger = min(n_virtual - 1 - v, (uint32_t)(NS - 1));
                if (younger >= 4) LARQL_WAIT_VMCNT(L * (NS - 1 < 4 ? NS - 1 : 4));
                else if (younger == 3) LARQL_WAIT_VMCNT(L * (NS - 1 < 3 ? NS - 1 : 3));
                else if (younger == 2) LARQL_WAIT_VMCNT(L * 2);
                else if (younger == 1) LARQL_WAIT_VMCNT(L * 1);
                else LARQL_WAIT_VMCNT(0);
            }
            asm volatile("" ::: "memory");
            const uint8_t *slot = ring + use_i * slot_bytes;
            f32x4 D = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < CW; s++) {
                const u32x4 qw = *reinterpret_cast<const u32x4 *>(slot + s * 1024 + lane * 16);
                const uint32_t sc = slot[cw * 1024 + sc_at[s]];
                D = mx4_step_mfma(ops.a[s], qw, sc, true, D);  // (an expert outside the bank: its result is dropped in the fold)
            }
            use_i = use_i + 1 == NS ? 0u : use_i + 1;
            const float sum = (D[0] + D[1]) + D[2];  // rows 4rq .. 4rq+2: the term sums of slot rq's activation
            if (DOWN) {
                if (kg == cq) acc = sum * weight_of(cq);
                if (cq + 1 == nq) pb[(tl * 16 + jr) * PW + wv * hw + kg] = ok_of(kg) ? acc : 0.f;
            } else if (kg == 0) {
                pb[(tl * 16 + jr) * PW + wv] = sum;
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the slot's reads are done before anything reuses it
        }
        if (DOWN && ++cq < nq) continue;
        cq = 0;
        if (++tl < (uint32_t)R && v + 1 < n_virtual) continue;
        // a batch of `tl` row tiles is complete: the row partials meet
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (DOWN) {
            // four threads per result row: thread h adds up expert h's slot of every wavefront, then the experts meet
            for (uint32_t rr = threadIdx.x >> 2; rr < tl * 16; rr += blockDim.x >> 2) {
                const uint32_t h = threadIdx.x & 3u;
                float s = 0.f;
                for (uint32_t w = 0; w < nwork; w++) s += pb[rr * PW + w * hw + h];
                s = dpp_add<0xB1>(s);  // quad_perm [1,0,3,2]: experts 0+1, 2+3
                s = dpp_add<0x4E>(s);  // quad_perm [2,3,0,1]: all four
                const uint32_t jt = rr & 15u, row = (f_t + (rr >> 4)) * TR + jt;
                if (h == 0 && jt < TR && row < rows) {
                    if (A.bias[0]) {  // + sum_q w_q * bias_q[row], in selection order
#pragma unroll
                        for (int q = 0; q < (int)kMoe1MaxK; q++)
                            if (ok[q]) s += cwt[q] * ((const GLOBAL_AS float *)A.bias[0])[(size_t)e[q] * A.bias_stride + (size_t)row * A.bias_step];
                    }
                    ((g_f32wp)A.out[0])[row] = s;
                }
            }
            f_t += tl;
        } else {
            for (uint32_t rr = threadIdx.x; rr < tl * 16; rr += blockDim.x) {
                float s = 0.f;
                for (uint32_t w = 0; w < nwork; w++) s += pb[rr * PW + w];
                // the tile of this row: `rr / 16` tiles past the batch's first
                uint32_t seg = f_seg, t = f_t + (rr >> 4);
                while (t >= tpm) { t -= tpm; seg++; }
                const uint32_t q = A.n_mats == 2 ? seg >> 1 : seg, m = A.n_mats == 2 ? (seg & 1u) : 0u;
                const uint32_t jt = rr & 15u, row = t * TR + jt;
                const bool live = jt < TR && row < rows;
                if (live) {
                    const float *bias = m ? A.bias[1] : A.bias[0];
                    if (!ok_of(q)) s = 0.0f;  // an expert outside the bank: no contribution (its stand-in's bytes were read, not used)
                    else if (bias) s += ((const GLOBAL_AS float *)bias)[(size_t)expert_of(q) * A.bias_stride + (size_t)row * A.bias_step];
                }
                if (A.terms) {
                    // rows 2i (gate) and 2i+1 (up) sit in neighbouring lanes (rows and the block size are even)
                    const float other = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, s), 0xB1, 0xF, 0xF, false));  // quad_perm [1,0,3,2]
                    if (live && (row & 1u) == 0 && row + 1 < rows) {  // (an even tile height keeps the pair in one tile)
                        const float hv = ok_of(q) ? clamped_glu(s, other, A.glu_limit, A.glu_alpha) : 0.0f;
                        uint32_t t3[3];
                        mx4_terms(hv, 0.0f, t3);
                        uint16_t *tp = A.terms + (size_t)q * A.terms_kpad + (row >> 1);
                        const size_t plane = (size_t)nq * A.terms_kpad;
                        tp[0] = (uint16_t)t3[0]; tp[plane] = (uint16_t)t3[1]; tp[2 * plane] = (uint16_t)t3[2];
                    }
                } else if (live) {
                    ((g_f32wp)((m ? A.out[1] : A.out[0]) + (size_t)q * A.out_slot_stride))[row] = s;
                }
            }
            f_t += tl;
            while (f_t >= tpm) { f_t -= tpm; f_seg++; }
        }
        tl = 0;
        parity ^= 1u;
    }
    LARQL_WAIT_VMCNT(0);
}

// ---------------------------------------------------------------------------
// bf16 rows against 2..8 activations at once (gate-KNN over several residual positions): the gate
// matrix is read once.  v_mfma_f32_16x16x32_bf16 with the roles swapped as above: the 16 "B" columns are
// 16 weight rows (a lane's operand is 16 contiguous bytes of its row, straight from the LDS ring), the
// "A" rows carry the activations: row 4t + i of set s holds term i of position 4s + t, where
// x = hi + mid + lo is split into three bf16 terms (exact: each term takes the next 8 significant
// bits) and row 4t + 3 is zero.  A wavefront owns 128 elements (4 MFMA steps) of the row per column pass,
// at most 2 passes (K <= 2560), and keeps all its A operands in registers.  Lane (j, rq) ends with the
// three term sums of position 4s + rq for weight row j.  Dot as bf16_dot_portable
// (larql-vindex/.../opplan/exec/cpu/kernels.rs:718-723); only the summation order differs.
// ---------------------------------------------------------------------------
constexpr int kBfStages = 3;
constexpr int kBfBatchTiles = 2;
constexpr int kBfMaxPasses = 2;
constexpr int kBfMaxSets = 2;       // 4 positions each
constexpr int kBfMaxWaves = 10;
constexpr uint32_t kBfTileBytes = 4 * 1024;  // 16 rows x 256 B (four steps of 32 elements)

__device__ __forceinline__ uint32_t bf16_term_bits(float &r) {  // next 8 significant bits of r; r keeps the rest
    const uint32_t b = __builtin_bit_cast(uint32_t, r) & 0xFFFF0000u;
    r -= __builtin_bit_cast(float, b);  // exact
    return b >> 16;
}

// A operand of one step: lane (i = lane%16, kq) holds term i%4 of position pos0 + i/4, elements 8kq..8kq+7
__device__ __forceinline__ BfOp bf16_mfma_operand(const float *x, uint64_t x_stride, uint32_t pos0, uint32_t batch, uint32_t k0,
                                                  uint32_t lane) {
    const uint32_t i = lane & 15u, kq = lane >> 4, pos = pos0 + (i >> 2), term = i & 3u;
    BfOp op;
    op.u[0] = op.u[1] = op.u[2] = op.u[3] = 0u;
    if (pos < batch && term < 3) {
        g_f4p xp = (g_f4p)(x + (size_t)pos * x_stride + k0 + 8 * kq);
        const f32x4 a = xp[0], b = xp[1];
        float e[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        uint32_t h[8];
#pragma unroll
        for (int q = 0; q < 8; q++) {
            uint32_t t0 = bf16_term_bits(e[q]);
            const uint32_t t1 = bf16_term_bits(e[q]), t2 = bf16_term_bits(e[q]);
            h[q] = term == 0 ? t0 : (term == 1 ? t1 : t2);
        }
#pragma unroll
        for (int q = 0; q < 4; q++) op.u[q] = h[2 * q] | (h[2 * q + 1] << 16);
    }
    return op;
}

__device__ __forceinline__ void run_bf16_mfma(const GemvJob &j, uint32_t tile_a, uint32_t tile_b, uint8_t *lds, uint32_t &parity) {
    constexpr int NS = kBfStages, R = kBfBatchTiles;
    const uint32_t lane = threadIdx.x & 63u, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nw_launch = blockDim.x >> 6;
    const uint32_t jr = lane & 15u, kq = lane >> 4;
    const uint32_t nwj = j.rpp, cols = j.cpr, batch = j.batch, nsets = (batch + 3) / 4;
    const uint32_t rows = (uint32_t)j.rows, row_bytes = (uint32_t)j.row_bytes;
    uint8_t *ring = lds + wv * (NS * kBfTileBytes);
    float *part = reinterpret_cast<float *>(lds + nw_launch * (NS * kBfTileBytes));
    const uint32_t np = wv < nwj ? (cols - wv + nwj - 1) / nwj : 0;  // columns wv, wv+nwj of this wavefront
    const uint32_t PW = 8 * nw_launch;                              // partials per row: [position][wavefront]

    // A copy instruction brings whole 128-byte lines: 8 rows x one half of the column's 256 bytes, eight consecutive
    // lanes to a line (instruction i: rows 8 (i % 2) .., half i / 2).  LDS receives a lane's 16 bytes at 16 * lane, so
    // within its line a lane fetches chunk (lane % 8) ^ ((row / 2) % 8): the operand reads below (16 rows, one chunk
    // each) then fall on 16 different bank groups.
    const uint32_t cr8 = lane >> 3, cc8 = lane & 7u;
    uint32_t copy_off[2];
#pragma unroll
    for (int g = 0; g < 2; g++) copy_off[g] = (g * 8 + cr8) * row_bytes + ((cc8 ^ ((g * 4 + (cr8 >> 1)) & 7u)) * 16);
    const uint32_t nt = tile_b - tile_a;
    uint32_t it_tile = tile_a, it_p = 0, n_issue = 0;
    auto issue = [&]() {
        const uint32_t tl = min(it_tile, tile_b - 1);  // past the end: the last wave-tile again (uniform load counts)
        // wave-uniform 64-bit base + per-lane 32-bit offset (the lane's row within the tile, clamped into the matrix)
        const uint32_t rb = tl * 16;
        const uint8_t *gb = j.w + (size_t)rb * row_bytes + (size_t)(wv + nwj * it_p) * 256;
        uint32_t lo[2] = {copy_off[0], copy_off[1]};
        if (rb + 16 > rows) {  // ragged last tile only: rows past the end read the last one
#pragma unroll
            for (int g = 0; g < 2; g++) lo[g] = min(g * 8 + cr8, rows - 1 - rb) * row_bytes + ((cc8 ^ ((g * 4 + (cr8 >> 1)) & 7u)) * 16);
        }
        uint8_t *lp = ring + (n_issue % NS) * kBfTileBytes;
#pragma unroll
        for (int i = 0; i < 4; i++) __builtin_amdgcn_global_load_lds((g_vp)(gb + lo[i & 1] + (i >> 1) * 128), (lds_vp)(lp + i * 1024), 16, 0, 0);
        n_issue++;
        if (it_tile < tile_b && ++it_p == np) { it_p = 0; it_tile++; }
    };
    if (np >= 1)
        for (int s = 0; s < NS - 1; s++) issue();

    // A operands of every (pass, step, set) of this wavefront, prepared while the first tiles are on their way
    BfOp xa[kBfMaxPasses][4][kBfMaxSets];
#pragma unroll
    for (int p = 0; p < kBfMaxPasses; p++)
#pragma unroll
        for (int s = 0; s < 4; s++)
#pragma unroll
            for (int q = 0; q < kBfMaxSets; q++)
                if ((uint32_t)p < np && (uint32_t)q < nsets)
                    xa[p][s][q] = bf16_mfma_operand(j.x, j.x_stride, 4 * q, batch, ((wv + nwj * p) * 4 + s) * 32, lane);

    uint32_t n_use = 0;
    for (uint32_t tb = 0; tb < nt; tb += R) {
        float *pb = part + parity * (R * 16 * PW);
        const uint32_t nbt = min((uint32_t)R, nt - tb);
        if (np >= 1) {
            for (uint32_t tl = 0; tl < nbt; tl++) {
                f32x4 D[kBfMaxSets];
#pragma unroll
                for (int q = 0; q < kBfMaxSets; q++) D[q] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int p = 0; p < kBfMaxPasses; p++) {
                    if ((uint32_t)p < np) {
                        issue();
                        LARQL_WAIT_VMCNT(4 * (NS - 1));  // the oldest wave-tile in flight has landed
                        asm volatile("" ::: "memory");
                        const uint8_t *slot = ring + (n_use % NS) * kBfTileBytes;
#pragma unroll
                        for (int s = 0; s < 4; s++) {
                            BfOp b;
                            // row jr, chunk 4 (s % 2) + kq of half s / 2: instruction jr / 8 + 2 (s / 2), swizzled as it was copied
                            const u32x4 q4 = *reinterpret_cast<const u32x4 *>(slot + ((jr >> 3) + 2 * (s >> 1)) * 1024 +
                                                                              (8 * (jr & 7u) + (((s & 1) * 4 + kq) ^ ((jr >> 1) & 7u))) * 16);
                            b.u[0] = q4.x; b.u[1] = q4.y; b.u[2] = q4.z; b.u[3] = q4.w;
#pragma unroll
                            for (int q = 0; q < kBfMaxSets; q++)
                                if ((uint32_t)q < nsets) D[q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[p][s][q].v, b.v, D[q], 0, 0, 0);
                        }
                        n_use++;
                    }
                }
#pragma unroll
                for (int q = 0; q < kBfMaxSets; q++) {
                    const uint32_t pos = 4 * q + kq;  // lane (jr, kq) holds the terms of position 4q + kq
                    if ((uint32_t)q < nsets && pos < batch) pb[(tl * 16 + jr) * PW + pos * nw_launch + wv] = (D[q][0] + D[q][1]) + D[q][2];
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const uint32_t row_base = (tile_a + tb) * 16, nwork = min(nwj, cols);
        for (uint32_t e = threadIdx.x; e < nbt * 16 * batch; e += blockDim.x) {
            const uint32_t rr = e / batch, pos = e - rr * batch;
            float s = 0.f;
            for (uint32_t w = 0; w < nwork; w++) s += pb[rr * PW + pos * nw_launch + w];
            if (row_base + rr < rows) ((g_f32wp)j.out)[(size_t)pos * j.out_stride + row_base + rr] = s;
        }
        parity ^= 1u;
    }
}

// ---------------------------------------------------------------------------
// Q4_K rows against 2..8 activations at once (gate-KNN over several residual positions, rows of up to 10
// super-blocks): the streaming of the single-activation kernel (a wavefront owns a 256-element column, 16 rows per
// wave-tile, global -> LDS ring), the products on the f16 matrix cores.  A weight is converted once for all
// positions: its nibble is masked in place into the mantissa of an f16 (1024 + q, or 1024 + 16 q for the high
// nibbles) and one packed FMA takes the 1024 away and applies the sub-block's 6-bit scale, so the operand is the
// integer sc6 * q <= 945, exact in f16.  One v_mfma_f32_16x16x32_f16 per sub-block (32 weights of 16 rows): its other
// operand has the activations as rows (position, part), part = the f16 nearest the scaled activation or the f16
// of what that leaves (together 22 bits of the activation; the scale is a power of two per position and column that
// puts the column's largest value below 2^15).  A ninth MFMA multiplies the 6-bit mins by the sub-blocks' activation
// sums, prepared the same way.  The eight products of a (row, position) share one accumulator; the row's f32 d and
// dmin and the column's power of two are applied to the two sums once per tile: d * sum sc6 q x - dmin * sum mn6 Sx,
// the value of q4k_matvec (larql-compute/src/cpu/ops/q4_common/matvec.rs) with the terms in another order.
// Lane (j, kq) supplies row j of the 16 weight rows (k-slots 8 kq .. 8 kq + 7 of every sub-block) and ends with the
// sums of positions 2 kq and 2 kq + 1 of that row.
// ---------------------------------------------------------------------------
constexpr int kQ4kBatchPairs = 4;  // positions per job: 2 * kQ4kBatchPairs
constexpr int kQ4kBatchR = 2;      // 16-row tiles between two folds of the row partials (16 * wavefronts partials per row)
constexpr int kQ4kBatchStages = 4;  // wave-tiles in flight per wavefront
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));

struct Q4kBatchCol {
    u32x4 xa[8];   // activations' operand of sub-block m: row a = (position 2 (a / 4) + (a / 2) % 2, part a % 2)
    uint32_t xs;   // the sums' operand: sub-blocks 2 kq and 2 kq + 1 of this lane's row, scaled by 2^-6 more
    float k[2];    // 2^(e - 15) of positions 2 kq and 2 kq + 1 (the lane's results)
};

// the slots of a lane's eight k in the operand registers: (0, 2), (1, 3), (4, 6), (5, 7) — the order in which the
// weights' nibbles leave their dwords (bytes 0 and 2 by a mask, bytes 1 and 3 after one shift)
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
    const half2_t h = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, h);
}

__device__ __forceinline__ void q4k_batch_setup(Q4kBatchCol &col, const float *x, uint64_t x_stride, uint32_t batch, uint32_t c,
                                                uint32_t lane) {
    const uint32_t a = lane & 15u, kq = lane >> 4;
    const uint32_t pos_a = 2 * (a >> 2) + ((a >> 1) & 1u), part = a & 1u;
    float to_s = 0.f, sx0 = 0.f, sx1 = 0.f;
    col.k[0] = col.k[1] = 0.f;
#pragma unroll
    for (uint32_t pos = 0; pos < 2 * kQ4kBatchPairs; pos++) {
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (pos < batch) v = ((g_f4p)(x + (size_t)pos * x_stride + (size_t)c * 256))[lane];
        float mx = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        float s4 = (v.x + v.y) + (v.z + v.w);  // lanes 8s .. 8s+7 hold sub-block s
#pragma unroll
        for (int o = 1; o < 8; o <<= 1) { s4 += __shfl_xor(s4, o); mx = fmaxf(mx, __shfl_xor(mx, o)); }
#pragma unroll
        for (int o = 8; o < 64; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        int ex = 0;
        if (mx > 0.f && mx < __builtin_inff()) (void)frexpf(mx, &ex);
        ex = max(-90, min(100, ex));
        const float s_a = __shfl(s4, 16 * kq), s_b = __shfl(s4, 16 * kq + 8);
        if (pos == pos_a) { to_s = ldexpf(1.f, 15 - ex); sx0 = s_a; sx1 = s_b; }
        if (pos == 2 * kq) col.k[0] = ldexpf(1.f, ex - 15);
        if (pos == 2 * kq + 1) col.k[1] = ldexpf(1.f, ex - 15);
    }
    const bool live = pos_a < batch;
    {
        const float t0 = sx0 * to_s * 0.015625f, t1 = sx1 * to_s * 0.015625f;
        const float h0 = (float)(_Float16)t0, h1 = (float)(_Float16)t1;
        col.xs = !live ? 0u : part ? pack_f16(t0 - h0, t1 - h1) : pack_f16(h0, h1);
    }
#pragma unroll
    for (int m = 0; m < 8; m++) {
        f32x4 u = {0.f, 0.f, 0.f, 0.f}, w = {0.f, 0.f, 0.f, 0.f};
        if (live) {
            g_f4p xs = (g_f4p)(x + (size_t)pos_a * x_stride + (size_t)c * 256 + m * 32 + 8 * kq);
            u = xs[0]; w = xs[1];
        }
        float e[8] = {u.x, u.y, u.z, u.w, w.x, w.y, w.z, w.w};
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const float t = e[q] * to_s;
            const float h = (float)(_Float16)t;
            e[q] = part ? t - h : h;
        }
        col.xa[m] = (u32x4){pack_f16(e[0], e[2]), pack_f16(e[1], e[3]), pack_f16(e[4], e[6]), pack_f16(e[5], e[7])};
    }
}

// the products of one wave-tile: D rows = (position, part) as dealt in q4k_batch_setup, columns = the 16 weight rows
struct Q4kBatchRaw {  // a lane's bytes of one wave-tile: its row's header and the 8 bytes kq of the four 32-byte chunks
    u32x4 hdr;
    u32x2 q[4];
};
__device__ __forceinline__ void q4k_batch_read(Q4kBatchRaw &r, const uint8_t *sp, uint32_t kq) {
    r.hdr = *reinterpret_cast<const u32x4 *>(sp);
#pragma unroll
    for (int g = 0; g < 4; g++) r.q[g] = *reinterpret_cast<const u32x2 *>(sp + 16 + 32 * g + 8 * kq);
}
__device__ __forceinline__ void q4k_batch_tile(const Q4kBatchRaw &raw_in, uint32_t kq, const Q4kBatchCol &col, uint32_t magic, float (&racc)[2]) {
    const u32x4 hdr = raw_in.hdr;
    const u32x2 (&q)[4] = raw_in.q;
    const float d = half_bits_to_float(hdr.x & 0xFFFFu), dmin64 = half_bits_to_float(hdr.x >> 16) * 64.f;
    // the 6-bit scales and mins of the eight sub-blocks, a byte each (get_scale_min_k4)
    const uint32_t sc_lo = hdr.y & 0x3F3F3F3Fu, mn_lo = hdr.z & 0x3F3F3F3Fu;
    const uint32_t sc_hi = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
    const uint32_t mn_hi = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
    const half2_t m1024 = {(_Float16)-1024.f, (_Float16)-1024.f};
    const half2_t k_lo = {(_Float16)1.f, (_Float16)-1024.f}, k_hi = {(_Float16)0.0625f, (_Float16)-64.f};
    f32x4 D = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int m = 0; m < 8; m++) {
        const int g = m >> 1, h = m & 1;
        // f16(sc6) straight from its byte, then (s, -1024 s) / (s / 16, -64 s) by one packed multiply
        uint32_t sfb;
        const uint32_t scw = m < 4 ? sc_lo : sc_hi;
        if ((m & 3) == 0) asm("v_cvt_f16_u16_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(sfb) : "v"(scw));
        else if ((m & 3) == 1) asm("v_cvt_f16_u16_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1" : "=v"(sfb) : "v"(scw));
        else if ((m & 3) == 2) asm("v_cvt_f16_u16_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(sfb) : "v"(scw));
        else asm("v_cvt_f16_u16_sdwa %0, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3" : "=v"(sfb) : "v"(scw));
        const _Float16 sf = __builtin_bit_cast(half2_t, sfb)[0];
        const half2_t s2 = {sf, sf};
        const half2_t p = s2 * (h ? k_hi : k_lo);
        const half2_t sc2 = {p[0], p[0]}, off2 = {p[1], p[1]};  // (broadcast by the instruction's operand selects)
        const uint32_t mask = h ? 0x00F000F0u : 0x000F000Fu;
        u32x4 bw;
#pragma unroll
        for (int w = 0; w < 2; w++) {
            const uint32_t raw = w ? q[g].y : q[g].x;
            const half2_t m02 = __builtin_bit_cast(half2_t, (raw & mask) | magic);
            const half2_t m13 = __builtin_bit_cast(half2_t, ((raw >> 8) & mask) | magic);
            bw[2 * w] = __builtin_bit_cast(uint32_t, m02 * sc2 + off2);
            bw[2 * w + 1] = __builtin_bit_cast(uint32_t, m13 * sc2 + off2);
        }
        D = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, col.xa[m]), __builtin_bit_cast(f16x8_t, bw), D, 0, 0, 0);
    }
    // the mins of sub-blocks 2 kq and 2 kq + 1 against their activation sums
    const uint32_t msel = (kq & 1u) ? 0x04030402u : 0x04010400u;
    const uint32_t mboth = __builtin_amdgcn_perm(0x64646464u, kq < 2 ? mn_lo : mn_hi, msel);
    const half2_t mn2 = __builtin_bit_cast(half2_t, mboth) + m1024;
    const u32x4 bm = {__builtin_bit_cast(uint32_t, mn2), 0u, 0u, 0u}, am = {col.xs, 0u, 0u, 0u};
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
    const f32x4 Dm = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, am), __builtin_bit_cast(f16x8_t, bm), z, 0, 0, 0);
    racc[0] = col.k[0] * __builtin_fmaf(d, D[0] + D[1], -dmin64 * (Dm[0] + Dm[1]));
    racc[1] = col.k[1] * __builtin_fmaf(d, D[2] + D[3], -dmin64 * (Dm[2] + Dm[3]));
}

__device__ __forceinline__ void run_q4k_batch(const GemvJob &j, uint32_t tile_a, uint32_t tile_b, uint8_t *lds, uint32_t &parity) {
    constexpr int NS = kQ4kBatchStages, R = kQ4kBatchR, NP = kQ4kBatchPairs;
    const uint32_t lane = threadIdx.x & 63u, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nw_launch = blockDim.x >> 6;
    const uint32_t jr = lane & 15u, kq = lane >> 4;
    const uint32_t nwj = j.rpp, batch = j.batch;
    const uint32_t rows = (uint32_t)j.rows, row_bytes = (uint32_t)j.row_bytes;
    uint8_t *ring = lds + wv * (NS * kQ4kTileBytes);
    float *part = reinterpret_cast<float *>(lds + nw_launch * (NS * kQ4kTileBytes));
    const bool working = wv < nwj;
    const uint32_t PW = 2 * NP * nw_launch + 1;  // partials per row: [position][wavefront], an odd stride (the fold reads down the rows)
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));  // (in a register, so that mask-and-or is one instruction)

    const uint32_t u0 = lane, u1 = 64 + lane, u2 = 128 + (lane >> 2);
    const uint32_t r0 = u0 / 9, r1 = u1 / 9, r2 = u2 / 9;
    const uint32_t w0 = (u0 - r0 * 9) * 16, w1 = (u1 - r1 * 9) * 16, w2 = (u2 - r2 * 9) * 16 + (lane & 3u) * 4;
    const uint32_t o0 = r0 * row_bytes + w0, o1 = r1 * row_bytes + w1, o2 = r2 * row_bytes + w2;
    const uint8_t *wcol = j.w + (size_t)wv * 144;
    const uint32_t nt = tile_b - tile_a;
    uint32_t it_tile = tile_a, slot_issue = 0;  // (ring slots by wrapping counters)
    auto issue = [&]() {
        // wave-uniform 64-bit base + per-lane 32-bit offset; only a ragged last tile recomputes the offsets
        const uint32_t rb = min(it_tile, tile_b - 1) * 16;
        const uint8_t *gp = wcol + (size_t)rb * row_bytes;
        uint32_t a0 = o0, a1 = o1, a2 = o2;
        if (rb + 16 > rows) {
            const uint32_t lim = rows - 1 - rb;
            a0 = min(r0, lim) * row_bytes + w0;
            a1 = min(r1, lim) * row_bytes + w1;
            a2 = min(r2, lim) * row_bytes + w2;
        }
        const uint8_t *g0 = gp + a0, *g1 = gp + a1, *g2 = gp + a2;
        uint8_t *lp = ring + slot_issue * kQ4kTileBytes;
        __builtin_amdgcn_global_load_lds((g_vp)g0, (lds_vp)lp, 16, 0, 0);
        __builtin_amdgcn_global_load_lds((g_vp)g1, (lds_vp)(lp + 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((g_vp)g2, (lds_vp)(lp + 2048), 4, 0, 0);
        slot_issue = slot_issue + 1 == (uint32_t)NS ? 0u : slot_issue + 1;
        if (it_tile < tile_b) it_tile++;
    };
    if (working)
        for (int s = 0; s < NS - 1; s++) issue();
    Q4kBatchCol col;
    if (working) q4k_batch_setup(col, j.x, j.x_stride, batch, wv, lane);

    uint32_t slot_use = 0;
    for (uint32_t tb = 0; tb < nt; tb += R) {
        float *pb = part + parity * (R * 16 * PW);
        const uint32_t nbt = min((uint32_t)R, nt - tb);
        if (working) {
            for (uint32_t tl = 0; tl < nbt; tl++) {
                issue();
                LARQL_WAIT_VMCNT(3 * (NS - 1));  // at most NS-1 younger wave-tiles still in flight: the oldest has landed
                asm volatile("" ::: "memory");
                Q4kBatchRaw raw;
                q4k_batch_read(raw, ring + slot_use * kQ4kTileBytes + jr * 144, kq);
                slot_use = slot_use + 1 == (uint32_t)NS ? 0u : slot_use + 1;
                float racc[2];
                q4k_batch_tile(raw, kq, col, magic, racc);
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    const uint32_t pos = 2 * kq + t;
                    if (pos < batch) pb[(tl * 16 + jr) * PW + pos * nw_launch + wv] = racc[t];
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const uint32_t row_base = (tile_a + tb) * 16;
        // a thread per (position, row): consecutive threads write consecutive rows of a position
        // The fold belongs to the wavefronts without a column when the launch has at least two of them (it is
        // launched with two more than its widest job has columns: ten column wavefronts lie 3, 3, 2, 2 on the four
        // SIMDs, the kernel is bound by the instructions of the SIMDs with three, and wavefronts 10 and 11 go to the
        // other two): they add up batch b while the column wavefronts are at batch b + 1 — the partials are double-
        // buffered, and the next barrier comes after both.
        static_assert(R == 1 || R == 2, "rows of a fold: 16 or 32");
        const uint32_t rsh = nbt == 2 ? 5u : 4u;
        const bool spare = nw_launch >= nwj + 2;
        if (spare && working) { parity ^= 1u; continue; }
        const uint32_t f0 = spare ? threadIdx.x - nwj * 64 : threadIdx.x, fstep = spare ? blockDim.x - nwj * 64 : blockDim.x;
        for (uint32_t e = f0; e < (batch << rsh); e += fstep) {
            const uint32_t pos = e >> rsh, rr = e & ((1u << rsh) - 1u);
            float s = 0.f;
            for (uint32_t w = 0; w < nwj; w++) s += pb[rr * PW + pos * nw_launch + w];
            if (row_base + rr < rows) ((g_f32wp)j.out)[(size_t)pos * j.out_stride + row_base + rr] = s;
        }
        parity ^= 1u;
    }
}

// ---------------------------------------------------------------------------
// ggml Q8_0 on the matrix cores (rows of up to 10 x 256 elements): the same streaming as Q4_K — a
// wavefront owns a 256-element column (8 blocks of 34 B = 272 B per row, 16 rows per wave-tile, global ->
// LDS ring) — and the same exact int8 MFMA against four-limb activations.  The weights already are int8:
// lane (row j, kq) feeds the 16 codes of half kq%2 of block 2g + kq/2 of each block pair g (the 34-byte
// blocks leave them 2 bytes off a dword boundary for even blocks: five aligned dwords and v_alignbit).
// A row 4g + 2cl + i carries limb i (or 2+i) of block 2g+cl and is non-zero only in the lanes kq/2 == cl.
// Lane (j, rq) ends with the limb sums of blocks 2rq and 2rq+1 of its row and scales them by the blocks'
// f16 d (q8_0_gemv / row_dot, larql-compute/src/cpu/kquant_gemv.rs:67-109, sums ((q*d)*x); here d*(sum q*x)).
// ---------------------------------------------------------------------------
constexpr int kQ8Stages = 3;
constexpr int kQ8BatchTiles = 4;
constexpr int kQ8MaxWaves = 10;
constexpr int kQ8MaxPasses = 2;  // columns per wavefront (both columns' activations stay in registers): K <= 5120
// wavefronts that work on a row of `cpr` 256-element columns (0: the row is too long for this kernel)
__host__ __device__ inline uint32_t q8_mfma_waves(uint64_t cpr) {
    if (cpr == 0 || cpr > (uint64_t)kQ8MaxWaves * kQ8MaxPasses) return 0;
    return cpr <= (uint64_t)kQ8MaxWaves ? (uint32_t)cpr : (uint32_t)((cpr + 1) / 2);
}
constexpr uint32_t kQ8RowBytes = 8 * 34;             // one column of one row
constexpr uint32_t kQ8TileBytes = 16 * kQ8RowBytes;  // 4352

struct Q8Col {
    uint32_t xa[4], xb[4];  // this lane's 16 activations as limbs i / 2+i (i = lane & 1)
    float k;                // 2^(e-27)
};

__device__ __forceinline__ Q8Col q8_mfma_setup_col(const float *x, uint32_t c, uint32_t lane) {
    const uint32_t j = lane & 15u, kq = lane >> 4;
    g_f4p xc = (g_f4p)(x + (size_t)c * 256);
    const f32x4 v = xc[lane];
    float mx = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    int ex = 0;
    if (mx > 0.f && mx < __builtin_inff()) (void)frexpf(mx, &ex);
    ex = max(-90, min(120, ex));
    const float to_int = ldexpf(1.f, 27 - ex);
    Q8Col col;
    col.k = ldexpf(1.f, ex - 27);
    // A row j = 4g + 2cl + i: block 2g+cl = j/2, elements 16*(kq%2) .. +15 of it
    const uint32_t i = j & 1u;
    g_f4p xs = (g_f4p)(x + (size_t)c * 256 + (j >> 1) * 32 + 16 * (kq & 1u));
    uint32_t la[16], lb[16];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const f32x4 f = xs[q];
        const float e[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
        for (int t = 0; t < 4; t++) {
            // balanced base-128 digits: n + 64*(1 + 128 + 128^2 + 128^3) has the unsigned digits l+64
            const int n = (int)__builtin_rintf(e[t] * to_int) + 0x8102040;
            const int l0 = (n >> 21) - 64, l1 = ((n >> 14) & 127) - 64, l2 = ((n >> 7) & 127) - 64, l3 = (n & 127) - 64;
            la[4 * q + t] = (uint32_t)(i ? l1 : l0) & 0xFFu;
            lb[4 * q + t] = (uint32_t)(i ? l3 : l2) & 0xFFu;
        }
    }
#pragma unroll
    for (int q = 0; q < 4; q++) {
        col.xa[q] = la[4 * q] | (la[4 * q + 1] << 8) | (la[4 * q + 2] << 16) | (la[4 * q + 3] << 24);
        col.xb[q] = lb[4 * q] | (lb[4 * q + 1] << 8) | (lb[4 * q + 2] << 16) | (lb[4 * q + 3] << 24);
    }
    return col;
}

__device__ __forceinline__ void run_q8_0_mfma(const GemvJob &j, uint32_t tile_a, uint32_t tile_b, uint8_t *lds, uint32_t &parity) {
    constexpr int NS = kQ8Stages, R = kQ8BatchTiles, NP = kQ8MaxPasses;
    const uint32_t lane = threadIdx.x & 63u, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t nw_launch = blockDim.x >> 6;
    const uint32_t jr = lane & 15u, kq = lane >> 4;
    const uint32_t nwj = j.rpp, cpr = j.cpr, PW = nwj * 4;
    const uint32_t rows = (uint32_t)j.rows, row_bytes = (uint32_t)j.row_bytes;
    uint8_t *ring = lds + wv * (NS * kQ8TileBytes);
    float *part = reinterpret_cast<float *>(lds + nw_launch * (NS * kQ8TileBytes));
    const uint32_t np = wv < nwj ? (cpr - wv + nwj - 1) / nwj : 0;  // columns wv, wv + nwj of this wavefront
    const bool working = np >= 1;

    // lane's pieces of a wave-tile in 16-byte units u = row*17 + piece: four full loads, then 256 B dword by dword
    uint32_t rw[5], ow[5], off[5];
#pragma unroll
    for (int q = 0; q < 5; q++) {
        const uint32_t u = q < 4 ? 64 * q + lane : 256 + (lane >> 2);
        rw[q] = u / 17;
        ow[q] = (u - rw[q] * 17) * 16 + (q < 4 ? 0 : (lane & 3u) * 4);
        off[q] = rw[q] * row_bytes + ow[q];
    }
    const uint8_t *wcol = j.w + (size_t)wv * kQ8RowBytes;
    const uint32_t nt = tile_b - tile_a;
    // issue cursor: wave-tiles in the order they are consumed (tile, then column pass: the workgroup reads whole rows)
    uint32_t it_tile = tile_a, it_p = 0, n_issue = 0;
    auto issue = [&]() {
        const uint32_t rb = min(it_tile, tile_b - 1) * 16;  // past the end: the last tile again (uniform load counts)
        uint8_t *lp = ring + (n_issue % NS) * kQ8TileBytes;
        // wave-uniform 64-bit base + per-lane 32-bit offset; only a ragged last tile recomputes the offsets
        const uint8_t *gp = wcol + (size_t)it_p * nwj * kQ8RowBytes + (size_t)rb * row_bytes;
        uint32_t a[5];
#pragma unroll
        for (int q = 0; q < 5; q++) a[q] = off[q];
        if (rb + 16 > rows) {
            const uint32_t lim = rows - 1 - rb;
#pragma unroll
            for (int q = 0; q < 5; q++) a[q] = min(rw[q], lim) * row_bytes + ow[q];
        }
#pragma unroll
        for (int q = 0; q < 4; q++)
            __builtin_amdgcn_global_load_lds((g_vp)(gp + a[q]), (lds_vp)(lp + q * 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((g_vp)(gp + a[4]), (lds_vp)(lp + 4096), 4, 0, 0);
        n_issue++;
        if (it_tile < tile_b && ++it_p == np) { it_p = 0; it_tile++; }
    };
    if (working)
        for (int s = 0; s < NS - 1; s++) issue();

    float colk[NP];
    Q4kOp xm[NP][8];
#pragma unroll
    for (int p = 0; p < NP; p++) {
        colk[p] = 0.f;
        if ((uint32_t)p < np) {
            const Q8Col col = q8_mfma_setup_col(j.x, wv + nwj * p, lane);
            colk[p] = col.k;
            const uint32_t my_g = jr >> 2, cl = (jr >> 1) & 1u;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const bool mine = my_g == (uint32_t)g && (kq >> 1) == cl;
#pragma unroll
                for (int q = 0; q < 4; q++) { xm[p][2 * g].u[q] = mine ? col.xa[q] : 0u; xm[p][2 * g + 1].u[q] = mine ? col.xb[q] : 0u; }
            }
        } else {
#pragma unroll
            for (int g = 0; g < 8; g++)
#pragma unroll
                for (int q = 0; q < 4; q++) xm[p][g].u[q] = 0u;
        }
    }
    // this lane's 16 codes of block pair g start at byte (2g + kq/2)*34 + 2 + 16*(kq%2) of its row: the aligned
    // dword below it and the bit offset (0 or 16)
    const uint32_t code_off = (kq >> 1) * 34 + 2 + 16 * (kq & 1u);
    const uint32_t code_dw = code_off & ~3u, code_sh = (code_off & 3u) * 8;

    uint32_t n_use = 0;
    for (uint32_t tb = 0; tb < nt; tb += R) {
        float *pb = part + parity * (R * 16 * nw_launch * 4);
        const uint32_t nbt = min((uint32_t)R, nt - tb);
        if (working) {
            for (uint32_t tl = 0; tl < nbt; tl++) {
                float racc = 0.f;
#pragma unroll
                for (int p = 0; p < NP; p++) {
                    if ((uint32_t)p < np) {
                        issue();
                        LARQL_WAIT_VMCNT(5 * (NS - 1));
                        asm volatile("" ::: "memory");
                        const uint8_t *sp = ring + (n_use % NS) * kQ8TileBytes + jr * kQ8RowBytes;
                        n_use++;
                        i32x4 Da = {0, 0, 0, 0}, Db = {0, 0, 0, 0};
#pragma unroll
                        for (int g = 0; g < 4; g++) {
                            const uint32_t *wp = reinterpret_cast<const uint32_t *>(sp + g * 68 + code_dw);
                            const uint32_t w0 = wp[0], w1 = wp[1], w2 = wp[2], w3 = wp[3], w4 = wp[4];
                            Q4kOp b;
                            b.u[0] = __builtin_amdgcn_alignbit(w1, w0, code_sh); b.u[1] = __builtin_amdgcn_alignbit(w2, w1, code_sh);
                            b.u[2] = __builtin_amdgcn_alignbit(w3, w2, code_sh); b.u[3] = __builtin_amdgcn_alignbit(w4, w3, code_sh);
                            Da = __builtin_amdgcn_mfma_i32_16x16x64_i8(xm[p][2 * g].v, b.v, Da, 0, 0, 0);
                            Db = __builtin_amdgcn_mfma_i32_16x16x64_i8(xm[p][2 * g + 1].v, b.v, Db, 0, 0, 0);
                        }
                        // this lane's pair is g = kq: Da = [b0.l0, b0.l1, b1.l0, b1.l1], Db = [b0.l2, b0.l3, b1.l2, b1.l3]
                        float dot0 = __builtin_fmaf((float)Da[0], 128.f, (float)Da[1]);
                        float dot1 = __builtin_fmaf((float)Da[2], 128.f, (float)Da[3]);
                        dot0 = __builtin_fmaf(dot0, 128.f, (float)Db[0]);
                        dot1 = __builtin_fmaf(dot1, 128.f, (float)Db[2]);
                        dot0 = __builtin_fmaf(dot0, 128.f, (float)Db[1]) * colk[p];
                        dot1 = __builtin_fmaf(dot1, 128.f, (float)Db[3]) * colk[p];
                        const float d0 = half_bits_to_float(*reinterpret_cast<const uint16_t *>(sp + kq * 68));
                        const float d1 = half_bits_to_float(*reinterpret_cast<const uint16_t *>(sp + kq * 68 + 34));
                        racc += d0 * dot0 + d1 * dot1;
                    }
                }
                pb[(tl * 16 + jr) * PW + wv * 4 + kq] = racc;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const uint32_t row_base = (tile_a + tb) * 16;
        for (uint32_t rr = threadIdx.x >> 2; rr < nbt * 16; rr += blockDim.x >> 2) {
            const uint32_t qd = threadIdx.x & 3u;
            float s = 0.f;
            for (uint32_t k = 0; k < nwj; k++) s += pb[rr * PW + k * 4 + qd];
            s = dpp_add<0xB1>(s);
            s = dpp_add<0x4E>(s);
            if (qd == 0 && row_base + rr < rows) ((g_f32wp)j.out)[row_base + rr] = s;
        }
        parity ^= 1u;
    }
}

template <int U>
__device__ __forceinline__ void run_q8_0(const GemvJob &j, uint32_t p0, uint32_t p1, float *part) {
    const uint32_t t = threadIdx.x, cpr = j.cpr, rpp = j.rpp;
    const bool active = t < cpr * rpp;
    const uint32_t c = active ? t % cpr : 0, rl = active ? t / cpr : 0;
    X32Slice xs;
    load_x32(xs, j.x, c);
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
                    raw[u] = q8_0_load(j.w, (uint64_t)r * cpr + c);
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = lr + u * rpp;
                    const float v = q8_0_block_dot(raw[u], xs);
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
__device__ __forceinline__ void run_q6k(const GemvJob &j, uint32_t p0, uint32_t p1, float *part) {
    const uint32_t t = threadIdx.x, cpr = j.cpr, rpp = j.rpp;
    const bool active = t < cpr * rpp;
    const uint32_t c = active ? t % cpr : 0, rl = active ? t / cpr : 0;
    Q6KSlice xs;
    q6k_load_x(xs, j.x, c);
    const size_t row_bytes = j.row_bytes;
    for (uint32_t tp = p0; tp < p1; tp += kTilePasses) {
        const uint32_t tp_end = min(p1, tp + kTilePasses);
        const uint32_t row_base = tp * rpp;
        const uint32_t tile_rows = min((uint32_t)j.rows, tp_end * rpp) - row_base;
        if (active) {
            for (uint32_t lr = rl; lr < tile_rows; lr += rpp * U) {
                Q6KRaw raw[U];
                const uint8_t *rowp[U];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = min(lr + u * rpp, tile_rows - 1) + row_base;
                    rowp[u] = j.w + (size_t)r * row_bytes;
                    raw[u] = q6k_load(rowp[u], c);
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = lr + u * rpp;
                    const float v = q6k_chunk_dot(raw[u], xs, rowp[u], c);
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
__device__ __forceinline__ void run_q6k_q8k(const GemvJob &j, uint32_t p0, uint32_t p1, float *part) {
#pragma clang fp contract(off)
    const uint32_t t = threadIdx.x, cpr = j.cpr, rpp = j.rpp, nsb = cpr >> 2;
    const bool active = t < cpr * rpp;
    const uint32_t c = active ? t % cpr : 0, rl = active ? t / cpr : 0;
    Q6KQ8Slice xs;
    q6k_q8k_load_x(xs, (const uint8_t *)j.x, (uint32_t)j.k, c);
    const size_t row_bytes = j.row_bytes;
    for (uint32_t tp = p0; tp < p1; tp += kTilePasses) {
        const uint32_t tp_end = min(p1, tp + kTilePasses);
        const uint32_t row_base = tp * rpp;
        const uint32_t tile_rows = min((uint32_t)j.rows, tp_end * rpp) - row_base;
        if (active) {
            for (uint32_t lr = rl; lr < tile_rows; lr += rpp * U) {
                Q6KRaw raw[U];
                const uint8_t *rowp[U];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = min(lr + u * rpp, tile_rows - 1) + row_base;
                    rowp[u] = j.w + (size_t)r * row_bytes;
                    raw[u] = q6k_load(rowp[u], c);
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = lr + u * rpp;
                    int s1 = q6k_q8k_chunk(raw[u], xs, rowp[u], c);
                    // the four chunks of a super-block are four neighbouring lanes (cpr % 4 == 0)
                    s1 += __builtin_amdgcn_mov_dpp(s1, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
                    s1 += __builtin_amdgcn_mov_dpp(s1, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
                    float term = half_bits_to_float(raw[u].d) * xs.dy;       // d_w * d_y
                    term = term * (float)s1;
                    if ((c & 3u) == 0 && r < tile_rows) part[r * nsb + (c >> 2)] = term;
                }
            }
        }
        __syncthreads();
        // a lane per row: acc += term, super-blocks in order (q6k.rs:63-89)
        for (uint32_t r = t; r < tile_rows; r += blockDim.x) {
            float acc = 0.f;
            for (uint32_t sb = 0; sb < nsb; sb++) acc += part[r * nsb + sb];
            ((g_f32wp)j.out)[row_base + r] = acc;
        }
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
        tile_epilogue(part, cpr, tile_rows, j.out, row_base, j.bias, j.bias_step);
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
                    raw[u] = q4_0_load(j.w, (uint64_t)r * cpr + c);
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const uint32_t r = lr + u * rpp;
                    const float v = q4_0_block_dot(raw[u], xs);
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

// A job descriptor as wave-uniform values.  The table sits in the kernel-argument block or in device memory that
// nothing writes while the kernel runs (a table built on the device was built by an earlier kernel), so it is read
// through the constant address space: with a wave-uniform address those are scalar loads — a handful of instructions
// and the short scalar path, where a vector load of the same words is repeated by every lane and has to be
// broadcast back word by word — and everything computed from the descriptor stays on the scalar side.
#define CONST_AS __attribute__((address_space(4)))
typedef const CONST_AS GemvJob *job_cp;
__device__ __forceinline__ job_cp job_table(const GemvLaunch &L) { return L.table ? (job_cp)L.table : (job_cp)L.inl; }
__device__ __forceinline__ uint32_t job_pass_begin(job_cp jobs, uint32_t i) {
    return *(const CONST_AS uint32_t *)((const CONST_AS uint8_t *)(jobs + i) + offsetof(GemvJob, pass_begin));
}
// The job that holds pass p, the first of workgroup blockIdx.x: read from the launch's table of first jobs where it has
// one (a single scalar load), else found by bisection over the jobs' pass ranges (a dependent load per step).
__device__ __forceinline__ uint32_t first_job_of_share(const GemvLaunch &L, job_cp jobs, uint32_t n_jobs, uint32_t p) {
    if (L.wg_first) return *((const CONST_AS uint32_t *)L.wg_first + blockIdx.x);
    uint32_t lo = 0, hi = n_jobs;
    while (lo + 1 < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (job_pass_begin(jobs, mid) <= p) lo = mid; else hi = mid;
    }
    return lo;
}
__device__ __forceinline__ GemvJob uniform_job(job_cp src) {
    static_assert(sizeof(GemvJob) % 4 == 0, "descriptor is a whole number of dwords");
    constexpr int N = sizeof(GemvJob) / 4;
    const CONST_AS uint32_t *p = (const CONST_AS uint32_t *)src;
    uint32_t w[N];
#pragma unroll
    for (int i = 0; i < N; i++) w[i] = p[i];
    GemvJob j;
    __builtin_memcpy(&j, w, sizeof(GemvJob));
    return j;
}

// ---------------------------------------------------------------------------
// The kernels, one per format so each gets its own register budget: workgroup
// b sweeps passes [P*b/G, P*(b+1)/G) of the launch's pass list, job by job.
// ---------------------------------------------------------------------------
template <int KIND, int U>
__device__ __forceinline__ void gemv_body(const GemvLaunch &L, float *part) {
    const job_cp jobs = job_table(L);
    const uint64_t P = L.total_passes;
    uint32_t p = (uint32_t)(P * blockIdx.x / gridDim.x);
    const uint32_t p_end = (uint32_t)(P * (blockIdx.x + 1) / gridDim.x);
    const uint32_t lo = first_job_of_share(L, jobs, L.n_jobs, p);
    uint32_t ji = lo;
    while (p < p_end) {
        GemvJob j = uniform_job(jobs + ji);
        bool dead = false;
        if (j.sel) {  // run-time expert selection: one bank of equally shaped matrices
            const uint32_t e = __builtin_amdgcn_readfirstlane(*(const GLOBAL_AS uint32_t *)j.sel);
            dead = j.sel_count != 0 && e >= j.sel_count;  // an id outside the bank: zeros, and no byte of the bank is read
            j.w += (size_t)(dead ? 0u : e) * j.w_sel_stride;
            j.aux += (size_t)(dead ? 0u : e) * j.aux_sel_stride;
            if (j.bias) j.bias += (size_t)(dead ? 0u : e) * j.bias_sel_stride;
        }
        const uint32_t jp_end = j.pass_begin + j.n_pass;
        const uint32_t seg_end = min(p_end, jp_end);
        const uint32_t a = p - j.pass_begin, b = seg_end - j.pass_begin;
        if (dead) {
            const uint64_t r0 = (uint64_t)a * j.rpp, r1 = min(j.rows, (uint64_t)b * j.rpp);
            for (uint64_t r = r0 + threadIdx.x; r < r1; r += blockDim.x) ((g_f32wp)j.out)[r] = 0.0f;
        } else if (KIND == KIND_Q4K) run_q4k<U>(j, a, b, part);
        else if (KIND == KIND_Q8_0) run_q8_0<U>(j, a, b, part);
        else if (KIND == KIND_MXFP4) run_mxfp4<U>(j, a, b, part);
        else if (KIND == KIND_Q6K) run_q6k<U>(j, a, b, part);
        else if (KIND == KIND_Q6K_Q8K) run_q6k_q8k<U>(j, a, b, part);
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
LARQL_GEMV_KERNEL(gemv_q8_0_u4_kernel, KIND_Q8_0, 4, 3)
LARQL_GEMV_KERNEL(gemv_mxfp4_u4_kernel, KIND_MXFP4, 4, 4)
LARQL_GEMV_KERNEL(gemv_q4_0_kernel, KIND_Q4_0, 4, 4)
LARQL_GEMV_KERNEL(gemv_q6k_kernel, KIND_Q6K, 2, 3)
LARQL_GEMV_KERNEL(gemv_q6k_q8k_kernel, KIND_Q6K_Q8K, 2, 4)
LARQL_GEMV_KERNEL(gemv_bf16_kernel, KIND_BF16, 4, 4)
LARQL_GEMV_KERNEL(gemv_f16_kernel, KIND_F16, 4, 4)
LARQL_GEMV_KERNEL(gemv_f32_kernel, KIND_F32, 2, 4)


// Q4_K on the matrix cores: workgroup b sweeps its share of the launch's tile list (a tile = 16 rows of
// a job, weighted by the job's row length so that shares are equal in bytes), job by job.
__global__ void __launch_bounds__(kQ4kMaxWaves * 64) gemv_q4k_mfma_kernel(GemvLaunch L) {
    extern __shared__ __attribute__((aligned(16))) uint8_t q4k_lds[];
    const job_cp jobs = job_table(L);
    const uint64_t P = L.total_passes;
    uint32_t p = (uint32_t)(P * blockIdx.x / gridDim.x);
    const uint32_t p_end = (uint32_t)(P * (blockIdx.x + 1) / gridDim.x);
    const uint32_t lo = first_job_of_share(L, jobs, L.n_jobs, p);
    uint32_t ji = lo, parity = 0;
    while (p < p_end) {
        const GemvJob j = uniform_job(jobs + ji);
        const uint32_t seg_end = min(p_end, j.pass_begin + j.n_pass);
        // a tile belongs to the workgroup whose share contains its first cost unit
        // (the job's cost range opens with its start-up allowance; tile t covers [su + t*cpt, su + (t+1)*cpt))
        const uint32_t a = p - j.pass_begin, b = seg_end - j.pass_begin, cpt = (uint32_t)j.pad, su = j.pad2;
        const uint32_t tile_a = a > su ? (a - su + cpt - 1) / cpt : 0, tile_b = b > su ? (b - su + cpt - 1) / cpt : 0;
        if (tile_a < tile_b) run_q4k_mfma(j, tile_a, tile_b, q4k_lds, parity);
        p = seg_end;
        ji++;
    }
    LARQL_WAIT_VMCNT(0);
}

// Q6_K on the matrix cores: the same sweep and cost model as the Q4_K kernel.
__global__ void __launch_bounds__(kQ6kMaxWaves * 64) gemv_q6k_mfma_kernel(GemvLaunch L) {
    extern __shared__ __attribute__((aligned(16))) uint8_t q6k_lds[];
    const job_cp jobs = job_table(L);
    const uint64_t P = L.total_passes;
    uint32_t p = (uint32_t)(P * blockIdx.x / gridDim.x);
    const uint32_t p_end = (uint32_t)(P * (blockIdx.x + 1) / gridDim.x);
    const uint32_t lo = first_job_of_share(L, jobs, L.n_jobs, p);
    uint32_t ji = lo, parity = 0;
    while (p < p_end) {
        const GemvJob j = uniform_job(jobs + ji);
        const uint32_t seg_end = min(p_end, j.pass_begin + j.n_pass);
        const uint32_t a = p - j.pass_begin, b = seg_end - j.pass_begin, cpt = (uint32_t)j.pad, su = j.pad2;
        const uint32_t tile_a = a > su ? (a - su + cpt - 1) / cpt : 0, tile_b = b > su ? (b - su + cpt - 1) / cpt : 0;
        if (tile_a < tile_b) run_q6k_mfma(j, tile_a, tile_b, q6k_lds, parity);
        p = seg_end;
        ji++;
    }
    LARQL_WAIT_VMCNT(0);
}

// Q4_K x Q8_K: the same sweep and cost model as the Q4_K kernel.
__global__ void __launch_bounds__(kQ4kMaxWaves * 64) gemv_q4k_q8k_kernel(GemvLaunch L) {
    extern __shared__ __attribute__((aligned(16))) uint8_t q8k_lds[];
    const job_cp jobs = job_table(L);
    const uint64_t P = L.total_passes;
    uint32_t p = (uint32_t)(P * blockIdx.x / gridDim.x);
    const uint32_t p_end = (uint32_t)(P * (blockIdx.x + 1) / gridDim.x);
    const uint32_t lo = first_job_of_share(L, jobs, L.n_jobs, p);
    uint32_t ji = lo, parity = 0;
    while (p < p_end) {
        GemvJob j = uniform_job(jobs + ji);
        if (j.sel) {  // run-time expert selection: one bank of equally shaped matrices (an id outside the bank reads matrix 0;
                      // the caller does not use that result)
            uint32_t e = __builtin_amdgcn_readfirstlane(*(const GLOBAL_AS uint32_t *)j.sel);
            e = e < j.sel_count ? e : 0u;
            j.w += (size_t)e * j.w_sel_stride;
        }
        const uint32_t seg_end = min(p_end, j.pass_begin + j.n_pass);
        const uint32_t a = p - j.pass_begin, b = seg_end - j.pass_begin, cpt = (uint32_t)j.pad, su = j.pad2;
        const uint32_t tile_a = a > su ? (a - su + cpt - 1) / cpt : 0, tile_b = b > su ? (b - su + cpt - 1) / cpt : 0;
        if (tile_a < tile_b) run_q4k_q8k(j, tile_a, tile_b, q8k_lds, parity);
        p = seg_end;
        ji++;
    }
    LARQL_WAIT_VMCNT(0);
}

// MXFP4 on the matrix cores: same sweep as the Q4_K kernel (cost unit = one tile x one 128-element step).
__global__ void __launch_bounds__(kMx4MaxWaves * 64) gemv_mxfp4_mfma_kernel(GemvLaunch L) {
    extern __shared__ __attribute__((aligned(16))) uint8_t mx4_lds[];
    const job_cp jobs = job_table(L);
    // (a job list built on the device brings its own count and pass total)
    const uint32_t n_jobs = L.dyn ? (uint32_t)__builtin_amdgcn_readfirstlane(((const GLOBAL_AS uint32_t *)L.dyn)[0]) : L.n_jobs;
    const uint64_t P = L.dyn ? (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane(((const GLOBAL_AS uint32_t *)L.dyn)[1]) : L.total_passes;
    if (P == 0 || n_jobs == 0) return;
    uint32_t p = (uint32_t)(P * blockIdx.x / gridDim.x);
    const uint32_t p_end = (uint32_t)(P * (blockIdx.x + 1) / gridDim.x);
    const uint32_t lo = first_job_of_share(L, jobs, n_jobs, p);
    uint32_t ji = lo, parity = 0;
    bool fresh = true;  // no job of this launch has used the workgroup's LDS yet
    while (p < p_end) {
        GemvJob j = uniform_job(jobs + ji);
        Mx4Sel S;
#pragma unroll
        for (int q = 0; q < kMx4MaxTokens; q++) { S.w[q] = j.w; S.aux[q] = j.aux; S.bias[q] = j.bias; S.cw[q] = 1.0f; S.ok[q] = true; }
        if (j.route_logits) {  // the selection itself, by every wavefront for itself (a load and ~200 instructions)
            uint32_t idx[kRouterMaxK];
            float wt[kRouterMaxK];
            const bool writer = j.route_experts && p == j.pass_begin && threadIdx.x < 64;  // (one workgroup opens the job)
            if (writer) router_select_wave<true>(j.route_logits, j.route_bias, j.route_n, j.route_k, j.route_policy, threadIdx.x & 63u, idx, wt);
            else router_select_wave<false>(j.route_logits, j.route_bias, j.route_n, j.route_k, j.route_policy, threadIdx.x & 63u, idx, wt);
            uint32_t e = idx[0];
#pragma unroll
            for (int r = 1; r < kRouterMaxK; r++) e = j.route_rank == (uint32_t)r ? idx[r] : e;
            e = __builtin_amdgcn_readfirstlane(e);
            S.w[0] = j.w + (size_t)e * j.w_sel_stride;
            S.aux[0] = j.aux + (size_t)e * j.aux_sel_stride;
            if (j.bias) S.bias[0] = j.bias + (size_t)e * j.bias_sel_stride;
            if (writer && threadIdx.x == 0) {
#pragma unroll
                for (int r = 0; r < kRouterMaxK; r++)
                    if ((uint32_t)r < j.route_k) { j.route_experts[r] = idx[r]; j.route_weights[r] = wt[r]; }
            }
        } else if (j.sel) {  // run-time expert selection: one bank of equally shaped matrices (one expert per activation in a folded job)
            const uint32_t n_sel = j.combine_w ? mx4_tokens(j) : 1u;
#pragma unroll
            for (int q = 0; q < kMx4MaxTokens; q++) {
                if ((uint32_t)q >= n_sel) break;
                uint32_t e = __builtin_amdgcn_readfirstlane(((const GLOBAL_AS uint32_t *)j.sel)[q]);
                S.ok[q] = j.sel_count == 0 || e < j.sel_count;  // an id outside the bank contributes nothing and reads nothing of it
                e = S.ok[q] ? e : 0u;
                S.w[q] = j.w + (size_t)e * j.w_sel_stride;
                S.aux[q] = j.aux + (size_t)e * j.aux_sel_stride;
                if (j.bias) S.bias[q] = j.bias + (size_t)e * j.bias_sel_stride;
                if (j.combine_w) {
                    const float wq = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, ((const GLOBAL_AS float *)j.combine_w)[q])));
                    S.cw[q] = S.ok[q] ? wq : 0.0f;
                }
            }
        }
        const uint32_t seg_end = min(p_end, j.pass_begin + j.n_pass);
        // a tile belongs to the workgroup whose share contains its first cost unit (the job's range opens with its
        // start-up allowance, if it has one)
        const uint32_t a = p - j.pass_begin, b = seg_end - j.pass_begin, cpt = j.cpt ? j.cpt : j.cpr, su = j.su;
        const uint32_t tile_a = a > su ? (a - su + cpt - 1) / cpt : 0, tile_b = b > su ? (b - su + cpt - 1) / cpt : 0;
        if (tile_a < tile_b) {
            if (j.combine_w) run_mxfp4_fold(j, S, tile_a, tile_b, mx4_lds, L.pad, parity);
            else run_mxfp4_mfma(j, S, tile_a, tile_b, mx4_lds, L.pad, parity, fresh);
            fresh = false;
        }
        p = seg_end;
        ji++;
    }
    LARQL_WAIT_VMCNT(0);
}

// bf16 rows x several activations: same sweep (cost unit = one tile x one 128-element column)
__global__ void __launch_bounds__(kBfMaxWaves * 64) gemv_bf16_mfma_kernel(GemvLaunch L) {
    extern __shared__ __attribute__((aligned(16))) uint8_t bf_lds[];
    const job_cp jobs = job_table(L);
    const uint64_t P = L.total_passes;
    uint32_t p = (uint32_t)(P * blockIdx.x / gridDim.x);
    const uint32_t p_end = (uint32_t)(P * (blockIdx.x + 1) / gridDim.x);
    const uint32_t lo = first_job_of_share(L, jobs, L.n_jobs, p);
    uint32_t ji = lo, parity = 0;
    while (p < p_end) {
        const GemvJob j = uniform_job(jobs + ji);
        const uint32_t seg_end = min(p_end, j.pass_begin + j.n_pass);
        const uint32_t a = p - j.pass_begin, b = seg_end - j.pass_begin;
        const uint32_t tile_a = (a + j.cpr - 1) / j.cpr, tile_b = (b + j.cpr - 1) / j.cpr;
        if (tile_a < tile_b) run_bf16_mfma(j, tile_a, tile_b, bf_lds, parity);
        p = seg_end;
        ji++;
    }
    LARQL_WAIT_VMCNT(0);
}

// Q4_K rows x several activations: same sweep as the single-activation kernel
__global__ void __launch_bounds__((kQ4kMaxWaves + 2) * 64) gemv_q4k_batch_kernel(GemvLaunch L) {
    extern __shared__ __attribute__((aligned(16))) uint8_t q4kb_lds[];
    const job_cp jobs = job_table(L);
    const uint64_t P = L.total_passes;
    uint32_t p = (uint32_t)(P * blockIdx.x / gridDim.x);
    const uint32_t p_end = (uint32_t)(P * (blockIdx.x + 1) / gridDim.x);
    const uint32_t lo = first_job_of_share(L, jobs, L.n_jobs, p);
    uint32_t ji = lo, parity = 0;
    while (p < p_end) {
        const GemvJob j = uniform_job(jobs + ji);
        const uint32_t seg_end = min(p_end, j.pass_begin + j.n_pass);
        const uint32_t a = p - j.pass_begin, b = seg_end - j.pass_begin;
        const uint32_t tile_a = (a + j.cpr - 1) / j.cpr, tile_b = (b + j.cpr - 1) / j.cpr;
        if (tile_a < tile_b) run_q4k_batch(j, tile_a, tile_b, q4kb_lds, parity);
        p = seg_end;
        ji++;
    }
    LARQL_WAIT_VMCNT(0);
}

// ggml Q8_0 on the matrix cores: same sweep (cost unit = one tile x one 256-element column)
__global__ void __launch_bounds__(kQ8MaxWaves * 64) gemv_q8_0_mfma_kernel(GemvLaunch L) {
    extern __shared__ __attribute__((aligned(16))) uint8_t q8_lds[];
    const job_cp jobs = job_table(L);
    const uint64_t P = L.total_passes;
    uint32_t p = (uint32_t)(P * blockIdx.x / gridDim.x);
    const uint32_t p_end = (uint32_t)(P * (blockIdx.x + 1) / gridDim.x);
    const uint32_t lo = first_job_of_share(L, jobs, L.n_jobs, p);
    uint32_t ji = lo, parity = 0;
    while (p < p_end) {
        const GemvJob j = uniform_job(jobs + ji);
        const uint32_t seg_end = min(p_end, j.pass_begin + j.n_pass);
        const uint32_t a = p - j.pass_begin, b = seg_end - j.pass_begin;
        const uint32_t tile_a = (a + j.cpr - 1) / j.cpr, tile_b = (b + j.cpr - 1) / j.cpr;
        if (tile_a < tile_b) run_q8_0_mfma(j, tile_a, tile_b, q8_lds, parity);
        p = seg_end;
        ji++;
    }
    LARQL_WAIT_VMCNT(0);
}

// ---------------------------------------------------------------------------
// Host side: geometry and launch.
// ---------------------------------------------------------------------------
// experiment knobs (environment): passes in flight per thread, forced block size
static uint32_t chunk_elems(int kind) {
    switch (kind) {
        case KIND_Q4K: case KIND_Q6K: case KIND_Q6K_Q8K: return 64;
        case KIND_Q8_0: case KIND_MXFP4: case KIND_Q4_0: return 32;
        default: return 16;
    }
}

// Q4_K on the matrix cores: wavefronts used for a row of `cpr` super-blocks (a function of the row
// length alone, so a matvec sums in the same order whatever else shares its launch): one wavefront per
// column up to 10, beyond that the count in 6..10 that wastes the fewest column slots over <= 4 passes
// (10 wavefronts x 4 columns of prepared activations is what fits in LDS beside the weight ring).
static uint32_t q4k_mfma_waves(uint64_t cpr) {
    if (cpr <= (uint64_t)kQ4kMaxWaves) return (uint32_t)cpr;
    uint32_t best = 0;
    uint64_t best_slots = ~0ull;
    for (uint32_t nw = 10; nw >= 6; nw--) {
        const uint64_t passes = (cpr + nw - 1) / nw;
        if (passes > (uint64_t)kQ4kMaxColPasses) continue;
        if (passes * nw < best_slots) { best_slots = passes * nw; best = nw; }
    }
    return best;  // 0: row too long for this path
}

static uint32_t q6k_mfma_waves(uint64_t cpr) {  // as q4k_mfma_waves: up to 10 wavefronts, up to 4 columns each
    if (cpr <= (uint64_t)kQ6kMaxWaves) return (uint32_t)cpr;
    uint32_t best = 0;
    uint64_t best_slots = ~0ull;
    for (uint32_t nw = 10; nw >= 6; nw--) {
        const uint64_t passes = (cpr + nw - 1) / nw;
        if (passes > (uint64_t)kQ6kMaxColPasses) continue;
        if (passes * nw < best_slots) { best_slots = passes * nw; best = nw; }
    }
    return best;  // 0: row too long for this path
}




// MXFP4 on the matrix cores: 128-element steps per wavefront (1..4) so that at most 10 wavefronts cover a row
static uint32_t mx4_steps_per_wave(uint64_t steps) {
    for (uint32_t cw = 1; cw <= (uint32_t)kMx4MaxSteps; cw++)
        if ((steps + cw - 1) / cw <= (uint64_t)kMx4MaxWaves) return cw;
    return 0;  // row too long for this path
}


uint32_t gemv_batch_capacity(int kind, uint64_t k) {
    // bf16: 128-element columns, at most 10 wavefronts x 2 passes, two sets of 4 positions
    if (kind == KIND_BF16 && k >= 128 && k % 128 == 0 && k / 128 <= (uint64_t)(kBfMaxWaves * kBfMaxPasses)) return 4 * kBfMaxSets;
    // Q4_K: one wavefront per super-block column, four pairs of positions
    if (kind == KIND_Q4K && k >= 256 && k % 256 == 0 && k / 256 <= (uint64_t)kQ4kMaxWaves) return 2 * kQ4kBatchPairs;
    return 1;
}


int gemv_effective_kind(const GemvJob &j) {
    if (j.kind == KIND_Q8_0 && j.k >= 256 && j.k % 256 == 0 && q8_mfma_waves(j.k / 256) != 0 && j.rows < 0x7FFFFFF0ull)
        return KIND_Q8_0_MFMA;
    if (j.kind == KIND_BF16 && j.batch >= 2) return KIND_BF16_MFMA;
    if (j.kind == KIND_Q4K && j.batch >= 2) return KIND_Q4K_BATCH;
    if (j.kind == KIND_MXFP4 && j.k >= 128 && j.k % 32 == 0 && mx4_steps_per_wave((j.k + 127) / 128) != 0 &&
        j.rows < 0x7FFFFFF0ull)
        return KIND_MXFP4_MFMA;
    if (j.kind == KIND_Q4K && !j.sel && j.k % 256 == 0 && j.k / 256 >= 1 && q4k_mfma_waves(j.k / 256) != 0 &&
        j.rows < 0x7FFFFFF0ull && (j.k / 256) * 144 * j.rows < (1ull << 62))
        return KIND_Q4K_MFMA;
    if (j.kind == KIND_Q6K && !j.sel && j.k % 256 == 0 && j.k / 256 >= 1 && q6k_mfma_waves(j.k / 256) != 0 &&
        j.rows < 0x7FFFFFF0ull && (j.k / 256) * 210 * j.rows < (1ull << 62))
        return KIND_Q6K_MFMA;
    return j.kind;
}

// Cost model of the share-out for the matrix-core Q4_K kernels, in 128ths of the time a ten-column tile takes
// (fitted on time stamps per workgroup and job segment of a mixed 238-job launch: set-up + tiles x cost per job kind):
// a tile of nw columns costs 58 + 7 nw (eight columns: 0.89 of ten), a tile walked in several column passes 19/16 of
// that per pass, and every share of a job — the one that opens it or not — starts with a pipeline refill and the
// activation set-up, worth 4.5 tiles (8.2 with several columns per wavefront).
static void q4k_tile_cost(uint64_t cpr, uint32_t nw, uint64_t *cpt, uint64_t *startup) {
    const uint64_t np = (cpr + nw - 1) / nw;
    const uint64_t one = 58 + 7 * (uint64_t)nw;
    *cpt = np == 1 ? one : (np * one * 19) / 16;
    *startup = np == 1 ? 576 : 1050;
}

// The opening share's set-up is in the job's cost (GemvJob::pad2); the later shares' set-ups ride on the tiles: a
// share of U units holds U / cpt tiles and pays one set-up, so a tile costs cpt (1 + set-up / U), U = the launch's
// units per workgroup.
bool gemv_refine_costs(GemvJob *jobs, size_t n, uint32_t grid) {
    if (n == 0 || grid == 0 || (jobs[0].kind != KIND_Q4K_MFMA && jobs[0].kind != KIND_Q4K_Q8K)) return false;
    uint64_t total = 0;
    for (size_t i = 0; i < n; i++) total += (uint64_t)jobs[i].n_pass;
    const uint64_t U = std::max<uint64_t>(total / grid, 1);
    const auto refined = [&](const GemvJob &j) {  // (a share shorter than its set-up: the tile cost at most doubles)
        const uint64_t cpt = (uint64_t)j.pad, su = j.pad2;
        return cpt + std::min<uint64_t>(cpt, (cpt * su + U / 2) / U);
    };
    for (size_t i = 0; i < n; i++)
        if (jobs[i].pad2 + ((jobs[i].rows + 15) / 16) * refined(jobs[i]) > 0x7FFFFFFFull) return false;  // (nothing changed yet)
    for (size_t i = 0; i < n; i++) {
        GemvJob &j = jobs[i];
        const uint64_t cpt = refined(j);
        j.pad = (int32_t)cpt;
        j.n_pass = (uint32_t)(j.pad2 + ((j.rows + 15) / 16) * cpt);
    }
    return true;
}

bool gemv_job_geometry(GemvJob &j, uint32_t threads) {
    if (j.row_stride && j.kind != KIND_Q4K_MFMA && j.kind != KIND_Q4K_Q8K) return false;  // (column ranges: those two kernels only)
    if (j.kind == KIND_Q8_0_MFMA) {
        const uint64_t cpr = j.k / 256;
        const uint32_t nw = q8_mfma_waves(cpr);
        if (j.k % 256 != 0 || nw == 0 || nw * 64 > threads) return false;
        j.cpr = (uint32_t)cpr;
        j.rpp = nw;  // wavefronts that work on this job
        j.row_bytes = (j.k / 32) * 34;
        const uint64_t tiles = (j.rows + 15) / 16;
        if (tiles * cpr > 0x7FFFFFFFull) return false;
        j.n_pass = (uint32_t)(tiles * cpr);
        return true;
    }
    if (j.kind == KIND_Q4K_BATCH) {
        if (j.batch < 2 || j.batch > gemv_batch_capacity(KIND_Q4K, j.k)) return false;
        const uint64_t cpr = j.k / 256;
        if (cpr * 64 > threads) return false;
        j.cpr = (uint32_t)cpr;
        j.rpp = (uint32_t)cpr;
        j.row_bytes = cpr * 144;
        const uint64_t tiles = (j.rows + 15) / 16;
        if (tiles * cpr > 0x7FFFFFFFull) return false;
        j.n_pass = (uint32_t)(tiles * cpr);
        return true;
    }
    if (j.kind == KIND_BF16_MFMA) {
        if (j.batch < 2 || j.batch > gemv_batch_capacity(KIND_BF16, j.k)) return false;
        const uint64_t cols = j.k / 128;
        const uint32_t nw = (uint32_t)std::min<uint64_t>(cols, kBfMaxWaves);
        if (nw * 64 > threads) return false;
        j.cpr = (uint32_t)cols;  // cost units per tile: one per 128-element column
        j.rpp = nw;
        j.row_bytes = j.k * 2;
        const uint64_t tiles = (j.rows + 15) / 16;
        if (tiles * cols > 0x7FFFFFFFull) return false;
        j.n_pass = (uint32_t)(tiles * cols);
        return true;
    }
    if (j.kind == KIND_MXFP4_MFMA) {
        if (j.k == 0 || j.k % 32 != 0) return false;
        const uint64_t steps = (j.k + 127) / 128;
        const uint32_t cw = mx4_steps_per_wave(steps);
        if (cw == 0) return false;
        const uint32_t nw = (uint32_t)((steps + cw - 1) / cw);
        if (nw * 64 > threads) return false;
        j.cpr = (uint32_t)steps;   // cost units per tile: one per 128-element step
        j.rpp = nw;                // wavefronts that work on this job
        j.pad = (int32_t)cw;       // steps per wavefront
        j.row_bytes = (j.k / 32) * 16;
        const uint64_t tiles = (j.rows + 15) / 16;
        const uint64_t fold = j.combine_w ? std::min<uint64_t>(std::max<uint64_t>(j.batch, 1), kMx4MaxTokens) : 1;  // matrices read per row tile
        if (tiles * steps * fold > 0x7FFFFFFFull) return false;
        j.n_pass = (uint32_t)(tiles * steps * fold);
        j.cpt = fold > 1 ? (uint32_t)(steps * fold) : 0;
        j.su = 0;
        return true;
    }
    if (j.kind == KIND_Q6K_MFMA) {  // geometry and cost model as for the Q4_K matrix-core kernel
        if (j.k == 0 || j.k % 256 != 0) return false;
        const uint64_t cpr = j.k / 256;
        const uint32_t nw = q6k_mfma_waves(cpr);
        if (nw == 0 || nw * 64 > threads) return false;
        j.cpr = (uint32_t)cpr;
        j.rpp = nw;
        j.row_bytes = cpr * 210;
        const uint64_t tiles = (j.rows + 15) / 16;
        const uint64_t np = (cpr + nw - 1) / nw;
        const uint64_t cpt = np == 1 ? 16 : np * 19, startup = np == 1 ? 72 : 180;
        j.pad = (int32_t)cpt;
        j.pad2 = (uint32_t)startup;
        if (startup + tiles * cpt > 0x7FFFFFFFull) return false;
        j.n_pass = (uint32_t)(startup + tiles * cpt);
        return true;
    }
    if (j.kind == KIND_Q4K_MFMA || j.kind == KIND_Q4K_Q8K) {
        if (j.k == 0 || j.k % 256 != 0) return false;
        const uint64_t cpr = j.k / 256;
        const uint32_t nw = q4k_mfma_waves(cpr);
        if (nw == 0 || nw * 64 > threads) return false;
        j.cpr = (uint32_t)cpr;
        j.rpp = nw;  // wavefronts that work on this job
        j.row_bytes = cpr * 144;
        if (j.row_stride) {  // a column range of a wider matrix (the kernels form 16 x row_bytes in 32 bits)
            if (j.row_stride % 144 != 0 || j.row_stride < cpr * 144 || j.row_stride > (1ull << 27)) return false;
            j.row_bytes = j.row_stride;
        }
        const uint64_t tiles = (j.rows + 15) / 16;
        uint64_t cpt, startup;
        q4k_tile_cost(cpr, nw, &cpt, &startup);
        j.pad = (int32_t)cpt;
        j.pad2 = (uint32_t)startup;
        if (startup + tiles * cpt > 0x7FFFFFFFull) return false;
        j.n_pass = (uint32_t)(startup + tiles * cpt);
        return true;
    }
    const uint32_t ce = chunk_elems(j.kind);
    if (j.k == 0 || j.k % ce != 0) return false;
    const uint64_t cpr = j.k / ce;
    if (cpr > threads) return false;
    j.cpr = (uint32_t)cpr;
    j.rpp = threads / j.cpr;
    switch (j.kind) {
        case KIND_Q4K: j.row_bytes = (j.k / 256) * 144; break;
        case KIND_Q8_0: j.row_bytes = (j.k / 32) * 34; break;
        case KIND_Q6K: case KIND_Q6K_Q8K: if (j.k % 256 != 0) return false; j.row_bytes = (j.k / 256) * 210; break;
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
    if (n > 0 && jobs[0].kind == KIND_Q8_0_MFMA) {
        uint32_t nw = 0;
        for (size_t i = 0; i < n; i++) {
            const uint32_t w = q8_mfma_waves(jobs[i].k / 256);
            if (w == 0) return 0;
            nw = std::max(nw, w);
        }
        return nw * 64;
    }
    if (n > 0 && jobs[0].kind == KIND_Q4K_BATCH) {
        uint64_t nw = 0;
        for (size_t i = 0; i < n; i++) nw = std::max<uint64_t>(nw, jobs[i].k / 256);
        return nw <= (uint64_t)kQ4kMaxWaves ? (uint32_t)(nw + 2) * 64 : 0;  // (two wavefronts more: they fold the partial sums)
    }
    if (n > 0 && jobs[0].kind == KIND_BF16_MFMA) {
        uint64_t nw = 0;
        for (size_t i = 0; i < n; i++) nw = std::max<uint64_t>(nw, std::min<uint64_t>(jobs[i].k / 128, kBfMaxWaves));
        return (uint32_t)nw * 64;
    }
    if (n > 0 && jobs[0].kind == KIND_MXFP4_MFMA) {
        uint32_t nw = 0;
        for (size_t i = 0; i < n; i++) {
            const uint64_t steps = (jobs[i].k + 127) / 128;
            const uint32_t cw = mx4_steps_per_wave(steps);
            if (cw == 0) return 0;
            nw = std::max(nw, (uint32_t)((steps + cw - 1) / cw));
        }
        return nw * 64;
    }
    if (n > 0 && jobs[0].kind == KIND_Q6K_MFMA) {
        uint32_t nw = 0;
        for (size_t i = 0; i < n; i++) {
            const uint32_t w = q6k_mfma_waves(jobs[i].k / 256);
            if (w == 0) return 0;
            if (w > nw) nw = w;
        }
        return nw * 64;
    }
    if (n > 0 && (jobs[0].kind == KIND_Q4K_MFMA || jobs[0].kind == KIND_Q4K_Q8K)) {
        uint32_t nw = 0;
        for (size_t i = 0; i < n; i++) {
            const uint32_t w = q4k_mfma_waves(jobs[i].k / 256);
            if (w == 0) return 0;
            if (w > nw) nw = w;
        }
        return nw * 64;
    }
    // Prefer the block size that wastes the fewest lanes over the jobs'
    // chunk counts (weighted by bytes); ties go to the smaller block.
    static const uint32_t cand_all[] = {256, 320, 384, 448, 512};
    const uint32_t *cand = cand_all;
    const size_t n_cand = 5;
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

uint32_t gemv_launch_param(const GemvJob *jobs, size_t n) {
    if (n > 0 && jobs[0].kind == KIND_MXFP4_MFMA) {  // ring slot: room for the longest K-range a wavefront owns
        uint32_t cw = 1;
        for (size_t i = 0; i < n; i++) cw = std::max(cw, mx4_steps_per_wave((jobs[i].k + 127) / 128));
        return cw * kMx4StepBytes + kMx4ScaleBytes;
    }
    if (n > 0 && jobs[0].kind == KIND_Q6K_MFMA) {  // columns per wavefront to keep room for
        uint32_t np = 1;
        for (size_t i = 0; i < n; i++) {
            const uint64_t cpr = jobs[i].k / 256;
            const uint32_t nw = q6k_mfma_waves(cpr);
            if (nw) np = std::max(np, (uint32_t)((cpr + nw - 1) / nw));
        }
        return np;
    }
    return 0;
}

size_t gemv_lds_bytes(const GemvJob *jobs, size_t n, uint32_t threads) {
    if (n > 0 && jobs[0].kind == KIND_Q8_0_MFMA) {
        const size_t nw = threads / 64;
        return nw * kQ8Stages * kQ8TileBytes + 2 * (size_t)kQ8BatchTiles * 16 * nw * 4 * sizeof(float);
    }
    if (n > 0 && jobs[0].kind == KIND_Q4K_BATCH) {
        const size_t nw = threads / 64;
        return nw * kQ4kBatchStages * kQ4kTileBytes + 2 * (size_t)kQ4kBatchR * 16 * (2 * kQ4kBatchPairs * nw + 1) * sizeof(float);
    }
    if (n > 0 && jobs[0].kind == KIND_BF16_MFMA) {
        const size_t nw = threads / 64;
        return nw * kBfStages * kBfTileBytes + 2 * (size_t)kBfBatchTiles * 16 * 8 * nw * sizeof(float);
    }
    if (n > 0 && jobs[0].kind == KIND_MXFP4_MFMA) {
        const size_t nw = threads / 64;
        // ring + two partial-sum areas of up to four sums (tokens, or folded experts) per weight row and wavefront
        return nw * kMx4Stages * gemv_launch_param(jobs, n) + 2 * (size_t)kMx4BatchTiles * 16 * nw * 4 * sizeof(float);
    }
    if (n > 0 && jobs[0].kind == KIND_Q4K_Q8K) {  // rings + one partial per (row, super-block), double-buffered
        const size_t nw = threads / 64;
        uint64_t cpr = 1;
        for (size_t i = 0; i < n; i++) cpr = std::max<uint64_t>(cpr, jobs[i].k / 256);
        return nw * kQ4kStages * kQ4kTileBytes + 2 * (size_t)kQ4kBatchTiles * 16 * cpr * sizeof(float);
    }
    if (n > 0 && jobs[0].kind == KIND_Q6K_MFMA) {
        const size_t nw = threads / 64;
        return nw * kQ6kStages * kQ6kTileBytes + 2 * (size_t)kQ6kBatchTiles * 16 * nw * 4 * sizeof(float);
    }
    if (n > 0 && jobs[0].kind == KIND_Q4K_MFMA) {
        const size_t nw = threads / 64;
        bool multi = false;  // some row needs several column passes: room for the prepared activations
        for (size_t i = 0; i < n; i++) multi = multi || jobs[i].k / 256 > (uint64_t)kQ4kMaxWaves;
        return nw * kQ4kStages * kQ4kTileBytes + 2 * (size_t)kQ4kBatchTiles * 16 * nw * 4 * sizeof(float) +
               (multi ? nw * kQ4kMaxColPasses * kQ4kColBytes : 0);
    }
    size_t m = 0;
    for (size_t i = 0; i < n; i++) {
        const size_t npart = jobs[i].kind == KIND_Q4K ? jobs[i].cpr / 4 : jobs[i].cpr;
        const size_t b = (size_t)kTilePasses * jobs[i].rpp * npart * sizeof(float);
        if (b > m) m = b;
    }
    return m;
}

uint32_t gemv_wgs_per_cu(int kind, uint32_t threads, size_t lds, uint32_t dflt) {
    if (kind != KIND_Q4K_MFMA && kind != KIND_MXFP4_MFMA && kind != KIND_BF16_MFMA && kind != KIND_Q4K_BATCH && kind != KIND_Q8_0_MFMA &&
        kind != KIND_Q4K_Q8K && kind != KIND_Q6K_MFMA)
        return dflt;
    // as many workgroups as LDS (160 KB per CU) allows, up to 12 wavefronts per CU (3 per SIMD at this register count)
    const uint32_t by_lds = (uint32_t)((160 * 1024) / lds), by_waves = 12 / (threads / 64);
    const uint32_t w = by_lds < by_waves ? by_lds : by_waves;
    return w < 1 ? 1 : w;
}

bool moe1_geometry(Moe1Args &A, uint32_t *threads, size_t *lds) {
    if (A.kdim < 128 || A.kdim % 32 != 0 || A.rows == 0 || A.rows >= (1u << 22) || A.k == 0 || A.k > kMoe1MaxK) return false;
    const uint64_t steps = ((uint64_t)A.kdim + 127) / 128;
    const uint32_t cw = mx4_steps_per_wave(steps);
    if (cw == 0) return false;
    const uint32_t nw = (uint32_t)((steps + cw - 1) / cw);
    const size_t slot = moe1_slot_bytes((int)cw);
    const size_t partials = 2 * (size_t)kMoe1BatchTiles * 16 * nw * 4 * sizeof(float);
    A.cw = cw;
    A.nw = nw;
    A.stages = (uint32_t)moe1_stages((int)cw);
    if (A.tile_rows == 0 || A.tile_rows > 16) A.tile_rows = 16;
    *threads = nw * 64;
    *lds = nw * A.stages * slot + partials;
    return *lds <= 160 * 1024;
}

template <bool DOWN, int CW>
static hipError_t moe1_launch_cw(hipStream_t s, const Moe1Args &A, uint32_t grid, uint32_t threads, size_t lds) {
    static std::atomic<bool> attr_set{false};  // dynamic LDS above 64 KB has to be allowed once per kernel
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void *)moe1_kernel<DOWN, CW, moe1_stages(CW)>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    hipLaunchKernelGGL((moe1_kernel<DOWN, CW, moe1_stages(CW)>), dim3(grid), dim3(threads), lds, s, A);
    return hipGetLastError();
}

template <bool DOWN>
static hipError_t moe1_launch_stage(hipStream_t s, const Moe1Args &A, uint32_t grid, uint32_t threads, size_t lds) {
    switch (A.cw) {
        case 1: return moe1_launch_cw<DOWN, 1>(s, A, grid, threads, lds);
        case 2: return moe1_launch_cw<DOWN, 2>(s, A, grid, threads, lds);
        case 3: return moe1_launch_cw<DOWN, 3>(s, A, grid, threads, lds);
        case 4: return moe1_launch_cw<DOWN, 4>(s, A, grid, threads, lds);
        case 5: return moe1_launch_cw<DOWN, 5>(s, A, grid, threads, lds);
        default: return hipErrorInvalidValue;
    }
}

hipError_t moe1_launch(hipStream_t s, const Moe1Args &A, bool down, uint32_t grid, uint32_t threads, size_t lds) {
    return down ? moe1_launch_stage<true>(s, A, grid, threads, lds) : moe1_launch_stage<false>(s, A, grid, threads, lds);
}

hipError_t gemv_launch(hipStream_t stream, int kind, const GemvLaunch &L, uint32_t threads, uint32_t grid, size_t lds) {
    switch (kind) {
        case KIND_Q8_0_MFMA: {
            static std::atomic<bool> attr_set_q8{false};
            if (!attr_set_q8) {
                hipError_t e = hipFuncSetAttribute((const void *)gemv_q8_0_mfma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return e;
                attr_set_q8 = true;
            }
            hipLaunchKernelGGL(gemv_q8_0_mfma_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        }
        case KIND_Q4K_BATCH: {
            static std::atomic<bool> attr_set_qb{false};
            if (!attr_set_qb) {
                hipError_t e = hipFuncSetAttribute((const void *)gemv_q4k_batch_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return e;
                attr_set_qb = true;
            }
            hipLaunchKernelGGL(gemv_q4k_batch_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        }
        case KIND_BF16_MFMA: {
            static std::atomic<bool> attr_set_bf{false};
            if (!attr_set_bf) {
                hipError_t e = hipFuncSetAttribute((const void *)gemv_bf16_mfma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return e;
                attr_set_bf = true;
            }
            hipLaunchKernelGGL(gemv_bf16_mfma_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        }
        case KIND_MXFP4_MFMA: {
            static std::atomic<bool> attr_set_mx4{false};
            if (!attr_set_mx4) {
                hipError_t e = hipFuncSetAttribute((const void *)gemv_mxfp4_mfma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return e;
                attr_set_mx4 = true;
            }
            hipLaunchKernelGGL(gemv_mxfp4_mfma_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        }
        case KIND_Q4K_MFMA: {
            static std::atomic<bool> attr_set{false};  // dynamic LDS above 64 KB has to be allowed once per process
            if (!attr_set) {
                hipError_t e = hipFuncSetAttribute((const void *)gemv_q4k_mfma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return e;
                attr_set = true;
            }
            hipLaunchKernelGGL(gemv_q4k_mfma_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        }
        case KIND_Q6K_MFMA: {
            static std::atomic<bool> attr_set{false};  // dynamic LDS above 64 KB has to be allowed once per process
            if (!attr_set) {
                hipError_t e = hipFuncSetAttribute((const void *)gemv_q6k_mfma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return e;
                attr_set = true;
            }
            hipLaunchKernelGGL(gemv_q6k_mfma_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        }
        case KIND_Q4K_Q8K: {
            static std::atomic<bool> attr_set{false};  // dynamic LDS above 64 KB has to be allowed once per process
            if (!attr_set) {
                hipError_t e = hipFuncSetAttribute((const void *)gemv_q4k_q8k_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess) return e;
                attr_set = true;
            }
            hipLaunchKernelGGL(gemv_q4k_q8k_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        }
        case KIND_Q4K:
            hipLaunchKernelGGL(gemv_q4k_u2_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        case KIND_Q8_0:
            hipLaunchKernelGGL(gemv_q8_0_u4_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        case KIND_MXFP4:
            hipLaunchKernelGGL(gemv_mxfp4_u4_kernel, dim3(grid), dim3(threads), lds, stream, L);
            break;
        case KIND_Q4_0: hipLaunchKernelGGL(gemv_q4_0_kernel, dim3(grid), dim3(threads), lds, stream, L); break;
        case KIND_Q6K: hipLaunchKernelGGL(gemv_q6k_kernel, dim3(grid), dim3(threads), lds, stream, L); break;
        case KIND_Q6K_Q8K: hipLaunchKernelGGL(gemv_q6k_q8k_kernel, dim3(grid), dim3(threads), lds, stream, L); break;
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
