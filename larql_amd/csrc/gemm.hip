// gemm.hip — batched-prefill Q4_K GEMM on the gfx950 matrix cores.
//
//   out[s, r] = sum_k W[r, k] * X[s, k]      W: [rows, hidden] Q4_K,  X: [seq, hidden] bf16 or f32
//
// the contraction q4k_matmul_into computes (larql-compute/src/cpu/ops/q4_common/
// matmul.rs:20-139; `out` is [seq, rows] row-major), on f16 MFMA over the integer
// weights (see the formulation below).
#include <hip/hip_runtime.h>

#include <atomic>
#include <stdint.h>
#include <stdlib.h>

#include "kernels.h"

namespace larql {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------------------
// The formulation: keep the weight integer.
//
//   out[s, r] = sum over super-blocks of  d[r] * (sum_k (sc6*q)[r,k] * x[s,k])  -  dmin[r] * (sum_sub mn6[r,sub] * Sx[s,sub])
//
// sc6*q <= 945 is exact in f16, so the A operand needs no hi/lo split and costs ~1.7 VALU instructions per
// weight (byte gather, mask into an f16 1024+q, one packed FMA against sc6) instead of ~10 for decode + split.
// The activations are prepared once per call (q4k_gemm_prep_kernel): per token a power-of-two scale brings
// max|x| to [2^13, 2^14), x/scale is stored as f16 (exact for bf16 inputs; f32 inputs add a second f16 term
// and a second pass), and Sx, the sum of the represented activations over each 32-element sub-block, is stored
// (divided by 32, to stay inside f16) as an f16 pair (hi, lo).  Per super-block a wavefront accumulates its 64x64 quadrant in D (v_mfma_f32_16x16x32_f16,
// 32 MFMAs per 64-element step), gets sum_sub mn6*Sx from one more MFMA per tile (A slots 2*sub+h = mn6,
// B slots = Sx_h), and folds both into the f32 result with the row's d and dmin.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float half_to_float(uint32_t lo16) { return (float)__builtin_bit_cast(_Float16, (uint16_t)lo16); }

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

// one block per token: scale, f16 terms, sub-block sums.  `x_is_bf16`: 16-bit inputs (exact in one term).
// A thread takes 8 consecutive elements at a time (one or two 16-byte loads); four neighbouring threads hold a
// 32-element sub-block.
__global__ void __launch_bounds__(256) q4k_gemm_prep_kernel(const void *__restrict__ x, int x_is_bf16, uint32_t hidden,
                                                            uint16_t *__restrict__ xh, uint16_t *__restrict__ xl,
                                                            uint16_t *__restrict__ sx, float *__restrict__ tok_scale,
                                                            int *__restrict__ any_lo, int swap12) {
    __shared__ float red[4];
    const uint32_t tok = blockIdx.x, t = threadIdx.x, nvec = hidden >> 3;  // hidden % 256 == 0
    const u32x4 *xb = reinterpret_cast<const u32x4 *>((const uint16_t *)x + (size_t)tok * hidden);
    const f32x4 *xf = reinterpret_cast<const f32x4 *>((const float *)x + (size_t)tok * hidden);
    auto load8 = [&](uint32_t v, float (&o)[8]) {
        if (x_is_bf16) {
            const u32x4 r = xb[v];
            const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                o[2 * i] = __builtin_bit_cast(float, w[i] << 16);
                o[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xFFFF0000u);
            }
        } else {
            const f32x4 a = xf[2 * v], b = xf[2 * v + 1];
            o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
        }
    };
    float mx = 0.f;
    for (uint32_t v = t; v < nvec; v += 256) {
        float o[8];
        load8(v, o);
#pragma unroll
        for (int i = 0; i < 8; i++) mx = fmaxf(mx, fabsf(o[i]));
    }
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if ((t & 63u) == 0) red[t >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    int ex = 0;
    if (mx > 0.f && mx < __builtin_inff()) (void)frexpf(mx, &ex);
    ex = max(-100, min(110, ex));
    const float to_h = ldexpf(1.f, 14 - ex);
    if (t == 0) tok_scale[tok] = ldexpf(1.f, ex - 14);
    int lo_seen = 0;
    u32x4 *oh = reinterpret_cast<u32x4 *>(xh + (size_t)tok * hidden);
    u32x4 *ol = xl ? reinterpret_cast<u32x4 *>(xl + (size_t)tok * hidden) : nullptr;
    for (uint32_t v = t; v < nvec; v += 256) {  // nvec % 32 == 0: the four threads of a sub-block run together
        float o[8];
        load8(v, o);
        uint32_t hw[4] = {0u, 0u, 0u, 0u}, lw[4] = {0u, 0u, 0u, 0u};
        float sm = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float sv = o[i] * to_h;
            const _Float16 h = (_Float16)sv;
            const _Float16 l = (_Float16)(sv - (float)h);
            const uint32_t hb = __builtin_bit_cast(uint16_t, h), lb = __builtin_bit_cast(uint16_t, l);
            // `swap12`: elements 1 and 2 of every four change places (the pipelined GEMM's weight operand comes out of
            // its nibble masks as the pairs (k0, k2), (k1, k3); the MFMA only needs both operands to agree)
            const int pos = swap12 ? ((i & 4) | ((i & 1) << 1) | ((i >> 1) & 1)) : i;
            if (pos & 1) { hw[pos >> 1] |= hb << 16; lw[pos >> 1] |= lb << 16; } else { hw[pos >> 1] |= hb; lw[pos >> 1] |= lb; }
            lo_seen |= (ol && (float)l != 0.f) ? 1 : 0;
            sm += (float)h + (ol ? (float)l : 0.f);  // the activation as the MFMAs will see it
        }
        oh[v] = (u32x4){hw[0], hw[1], hw[2], hw[3]};
        if (ol) ol[v] = (u32x4){lw[0], lw[1], lw[2], lw[3]};
        sm += __shfl_xor(sm, 1);
        sm += __shfl_xor(sm, 2);
        sm *= 0.03125f;  // stored as Sx/32 so that 32 x 2^14 stays inside f16; the min operand carries the 32
        if ((t & 3u) == 0) {
            const _Float16 sh = (_Float16)sm;
            const _Float16 sl = (_Float16)(sm - (float)sh);
            const uint32_t pair = (uint32_t)__builtin_bit_cast(uint16_t, sh) | ((uint32_t)__builtin_bit_cast(uint16_t, sl) << 16);
            reinterpret_cast<uint32_t *>(sx)[(size_t)tok * (hidden / 32) + (v >> 2)] = pair;
        }
    }
    if (lo_seen && any_lo) *any_lo = 1;
}

// adds the partial slabs of a K-split in slab order and applies the token scale
__global__ void __launch_bounds__(256) q4k_gemm_reduce_kernel(const float *__restrict__ partial, uint32_t splits, const float *__restrict__ tok_scale,
                                                              float *__restrict__ out, uint32_t rows, uint32_t seq, int accumulate) {
    const size_t n = (size_t)rows * seq, i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = 0.f;
    for (uint32_t z = 0; z < splits; z++) s += partial[(size_t)z * n + i];
    s *= tok_scale[i / rows];
    out[i] = accumulate ? out[i] + s : s;
}

// ---------------------------------------------------------------------------
// The kernel: software-pipelined; with_mins = 0: the activation term carries no offset part (second pass over the lo terms).
//
// One workgroup of 8 wavefronts per CU owns a 256-row x 128-token tile; a wavefront owns 32 of the rows against
// all 128 tokens.  Everything a step (64 k) needs from global memory was copied global -> LDS (global_load_lds,
// 16 bytes per lane, no registers involved) at least two steps before:
//   * the f16 activations of a step, into a ring of four stages.  Rows are 128 bytes (64 f16) without
//     padding; the 16-byte chunk c of row r is kept at position c ^ (r & 7), chosen on the global side of the
//     copy, so that the eight lanes of an operand read phase hit eight different bank groups;
//   * the raw weight bytes of a step (32 per row), into a ring of five stages (a wavefront copies its own rows);
//   * per super-block the 16-byte headers and the Sx of the tile's tokens; sum mn6*Sx is taken at the
//     super-block's first step, d*D is folded in at its last.
// The f16(sc6*q) operand never exists in memory: lane (l16, kg) of an MFMA holds row l16, k 8kg .. 8kg+7 of a
// 32-wide half, i.e. the low or the high nibbles of 8 raw bytes of that row, so every lane reads the 8 bytes of
// its two rows once per step and converts them, in the MFMAs' shadow, into the operand of the next half.  Only
// the activations cross wavefronts: one barrier per step.  No global load returns into a register, so the
// compiler places no vmcnt waits of its own (it would wait for *all* outstanding loads as soon as register loads
// and LDS copies are in flight together); outstanding copies are counted by hand: at the end of a step only the
// requests of the last two steps may still fly.  For the same reason (an LDS copy in flight makes the compiler
// wait for lgkmcnt(0) at every LDS read) the operand reads of the loop are written as instructions with counted
// waits, P_LA reads ahead of the MFMA group that consumes them.
// ---------------------------------------------------------------------------
constexpr int PM = 256, PN = 128, PTHREADS = 512;
constexpr int P_LA = 4;                                                         // operand reads in flight ahead of the MFMAs
constexpr int P_NB = 4, P_NR = 5;                                               // ring depths: activations, raw weights
constexpr int P_B_STAGE = PN * 128, P_R_STAGE = PM * 32;                        // bytes
constexpr int P_B_OFF = 0, P_R_OFF = P_B_OFF + P_NB * P_B_STAGE, P_H_OFF = P_R_OFF + P_NR * P_R_STAGE,
              P_AM_OFF = P_H_OFF + PM * 32, P_BM_OFF = P_AM_OFF + PM * 32, P_D_OFF = P_BM_OFF + PN * 32,
              P_DMIN_OFF = P_D_OFF + 2 * PM * 4, P_LOOP_BYTES = P_DMIN_OFF + 2 * PM * 4;
constexpr int P_EP_LD = 36, P_EP_BYTES = 8 * PN * P_EP_LD * 4;                  // the results leave through LDS (see the epilogue)
constexpr int P_LDS_BYTES = P_LOOP_BYTES > P_EP_BYTES ? P_LOOP_BYTES : P_EP_BYTES;
static_assert(P_LDS_BYTES <= 160 * 1024, "one workgroup per CU");
typedef __attribute__((address_space(3))) void *p_lds_vp;
typedef const __attribute__((address_space(1))) void *p_g_vp;
#define GEMM_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

__global__ void __launch_bounds__(PTHREADS, 1) q4k_gemm_pipe_kernel(const uint8_t *w, const uint16_t *xh, const uint16_t *sx,
                                                                    const float *__restrict__ tok_scale, float *__restrict__ out,
                                                                    uint32_t rows, uint32_t hidden, uint32_t seq, int with_mins,
                                                                    int accumulate, uint32_t sb_per_split, float *__restrict__ partial) {
    extern __shared__ __attribute__((aligned(16))) uint8_t plds[];
    const uint32_t t = threadIdx.x, lane = t & 63u, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t row0 = blockIdx.x * PM, tok0 = blockIdx.y * PN;
    const uint32_t nsb = hidden >> 8, row_bytes = nsb * 144;
    const uint32_t sb_begin = blockIdx.z * sb_per_split, sb_end = min(nsb, sb_begin + sb_per_split);
    if (sb_begin >= sb_end) return;
    const uint32_t nsteps = (sb_end - sb_begin) * 4;

    // conversion role: thread -> (tile row, 16-byte part of the row's 32 raw bytes = 16 k of a 32-wide half)
    const uint32_t sr = t >> 1, part = t & 1u;
    // copy roles.  Raw weights: thread -> (row t/2, part t&1) of a step, i.e. wavefront w brings rows 32w .. 32w+31.
    const uint8_t *wt = w + (size_t)row0 * row_bytes;                                          // uniform
    const uint32_t r_off = (min(row0 + sr, rows - 1) - row0) * row_bytes + part * 16;
    // headers: a wavefront brings those of its own 32 rows (lanes 32..63 a second copy: the copy is 64 lanes wide)
    const uint32_t h_off = (min(row0 + wave * 32 + (lane & 31u), rows - 1) - row0) * row_bytes;
    // activations: wavefront -> tokens 16w .. 16w+15 (two copies of 8 tokens x 128 bytes), lane -> (token, chunk)
    const uint8_t *xt = (const uint8_t *)xh + (size_t)tok0 * hidden * 2;                       // uniform
    uint32_t b_off[2];
#pragma unroll
    for (int q = 0; q < 2; q++) {
        const uint32_t r = (wave * 2 + q) * 8 + (lane >> 3);
        b_off[q] = (min(tok0 + r, seq - 1) - tok0) * hidden * 2 + (((lane & 7u) ^ (lane >> 3)) * 16);
    }
    // Sx: wavefronts w and w+4 both bring tokens 32*(w&3) .. +31 (two 16-byte halves each)
    const uint8_t *st = (const uint8_t *)sx + (size_t)tok0 * (hidden / 32) * 4;                // uniform
    const uint32_t m_off = (min(tok0 + (wave & 3u) * 32 + (lane >> 1), seq - 1) - tok0) * (hidden / 32) * 4 + (lane & 1u) * 16;

    // compute role: a wavefront owns the 32 rows it converts, against all 128 tokens: the weight operand, the raw
    // bytes, the headers and the per-row constants never cross wavefronts, only the activations (and Sx) do
    const uint32_t wm = wave * 32;
    const uint32_t l16 = lane & 15u, kg = lane >> 4, sw_b = l16 & 7u;

    // (requests past the end are clamped: same number of copies in flight, results unused)
    auto issue_raw = [&](uint32_t s) {
        const uint32_t sc = min(s, nsteps - 1);
        const uint8_t *src = wt + ((size_t)(sb_begin + (sc >> 2)) * 144 + 16 + 32 * (sc & 3u));
        __builtin_amdgcn_global_load_lds((p_g_vp)(src + r_off), (p_lds_vp)(plds + P_R_OFF + (s % P_NR) * P_R_STAGE + wave * 1024), 16, 0, 0);
    };
    auto issue_b = [&](uint32_t s) {
        const uint32_t sc = min(s, nsteps - 1);
        const uint8_t *src = xt + ((size_t)sb_begin * 256 + (size_t)sc * 64) * 2;
        uint8_t *dst = plds + P_B_OFF + (s % P_NB) * P_B_STAGE + wave * 2048;
        __builtin_amdgcn_global_load_lds((p_g_vp)(src + b_off[0]), (p_lds_vp)dst, 16, 0, 0);
        __builtin_amdgcn_global_load_lds((p_g_vp)(src + b_off[1]), (p_lds_vp)(dst + 1024), 16, 0, 0);
    };
    auto issue_sb = [&](uint32_t sb) {  // header and Sx of a super-block
        const uint32_t sbc = min(sb, sb_end - 1);
        __builtin_amdgcn_global_load_lds((p_g_vp)((wt + (size_t)sbc * 144) + h_off), (p_lds_vp)(plds + P_H_OFF + wave * 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((p_g_vp)((st + (size_t)sbc * 32) + m_off), (p_lds_vp)(plds + P_BM_OFF + (wave & 3u) * 1024), 16, 0, 0);
    };
    uint32_t hdr_y[2] = {0, 0}, hdr_w[2] = {0, 0};  // the scale words of this lane's two operand rows, super-block being converted
    auto stage_sb = [&](uint32_t par) {  // a super-block's header: scale words to registers, mn6 / d / dmin to LDS
        const u32x4 hdr = *reinterpret_cast<const u32x4 *>(plds + P_H_OFF + wave * 1024 + (lane >> 1) * 16);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const u32x4 hi = *reinterpret_cast<const u32x4 *>(plds + P_H_OFF + wave * 1024 + (i * 16 + l16) * 16);
            hdr_y[i] = hi.y; hdr_w[i] = hi.w;
        }
        if (with_mins) {
            uint32_t mnw[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {  // this thread's half of the super-block: sub-blocks 4*part .. +3 -> slots 8*part .. +7
                const uint32_t ss = 4 * part + u, shm = 8u * (ss & 3u);
                const uint32_t qb = (hdr.z >> shm) & 0xFFu, qc = (hdr.w >> shm) & 0xFFu;
                const uint32_t mn6 = ss < 4 ? (qb & 63u) : ((qc >> 4) | ((qb >> 6) << 4));
                const uint32_t hb = __builtin_bit_cast(uint16_t, (_Float16)(float)(mn6 * 32u));  // <= 2016: exact; Sx is stored /32
                mnw[u] = hb | (hb << 16);
            }
            *reinterpret_cast<u32x4 *>(plds + P_AM_OFF + sr * 32 + part * 16) = (u32x4){mnw[0], mnw[1], mnw[2], mnw[3]};
        }
        if (part == 0) {
            reinterpret_cast<float *>(plds + P_D_OFF)[par * PM + sr] = half_to_float(hdr.x & 0xFFFFu);
            reinterpret_cast<float *>(plds + P_DMIN_OFF)[par * PM + sr] = half_to_float(hdr.x >> 16);
        }
    };
    // scale of sub-block `sub` (0..7) of the current header as the packed-FMA operands (sc6, -1024*sc6)
    // (odd sub-blocks are the high nibbles: their masked value is 1024 + 16q, so the factor is sc6/16 and the offset -64*sc6)
    auto scale_of = [&](int i, uint32_t sub, _Float16 &sc1, _Float16 &off1) {
        const uint32_t sh = 8u * (sub & 3u);
        const uint32_t pa = (hdr_y[i] >> sh) & 0xFFu, pc = (hdr_w[i] >> sh) & 0xFFu;
        const uint32_t sc6 = sub < 4 ? (pa & 63u) : ((pc & 0x0Fu) | ((pa >> 6) << 4));
        const float f = (float)sc6;
        const _Float16 scf = (_Float16)((sub & 1u) ? f * 0.0625f : f), of = (_Float16)((sub & 1u) ? -64.0f * f : -1024.0f * f);
        sc1 = scf;
        off1 = of;
    };
    // 4 raw bytes (nibble h) -> two dwords of f16(sc6*q), exact (sc6*q <= 945), as the pairs (k0, k2) and (k1, k3):
    // the nibbles of bytes 0 and 2 are masked in place into the mantissas of two f16 (1024 + q, or 1024 + 16q for
    // the high nibbles), those of bytes 1 and 3 after one shift; one packed FMA takes the 1024 away and applies
    // sc6 (sc6/16) with a single rounding.  `magic` is 0x64006400 held in a register so that mask-and-or is one
    // instruction.
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));
    auto convert4 = [&](uint32_t raw, uint32_t h, _Float16 sc1, _Float16 off1, uint32_t &o0, uint32_t &o1) {
        const f16x2 sc2 = {sc1, sc1}, off2 = {off1, off1};  // (broadcast by the instruction's operand selects, not by a pack)
        const uint32_t mask = h ? 0x00F000F0u : 0x000F000Fu;
        const f16x2 m02 = __builtin_bit_cast(f16x2, (raw & mask) | magic);
        const f16x2 m13 = __builtin_bit_cast(f16x2, ((raw >> 8) & mask) | magic);
        o0 = __builtin_bit_cast(uint32_t, m02 * sc2 + off2);
        o1 = __builtin_bit_cast(uint32_t, m13 * sc2 + off2);
    };
    // The weight operand never exists in memory: lane (l16, kg) of an MFMA holds row l16, k 8kg .. 8kg+7 of a
    // 32-wide half, which are the low (first half) or high (second half) nibbles of the row's raw bytes
    // 8kg .. 8kg+7 of the step; the lane reads those 8 bytes of its two rows once per step and converts them
    // into the operand of the next half while the matrix cores work on the current one.
    //
    // The operand reads of the main loop are written as instructions with hand-counted waits: while LDS copies
    // are in flight the compiler's own wait for an LDS read is lgkmcnt(0), i.e. it would drain the reads issued
    // ahead with the one that is needed.  LDS reads return in order, so "all but the last n" is exact.
    const uint32_t lds0 = (uint32_t)(uintptr_t)(p_lds_vp)plds;
    const uint32_t raw_lane = lds0 + P_R_OFF + wave * 1024 + l16 * 32 + kg * 8;
    auto raw_of = [&](uint32_t rs, u32x2 (&rq)[2]) {
        const uint32_t a = raw_lane + (rs % P_NR) * P_R_STAGE;
        asm volatile("ds_read_b64 %0, %1" : "=v"(rq[0]) : "v"(a));
        asm volatile("ds_read_b64 %0, %1 offset:512" : "=v"(rq[1]) : "v"(a));
    };
    const uint32_t b_lane = lds0 + P_B_OFF + l16 * 128;
    uint32_t b_col[2];  // byte position of this lane's chunk in a token's row, for the two halves of a step
#pragma unroll
    for (int kk = 0; kk < 2; kk++) b_col[kk] = (((uint32_t)kk * 4 + kg) ^ sw_b) << 4;

    f32x4 acc[2][8], D[2][8];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int jj = 0; jj < 8; jj++) { acc[i][jj] = (f32x4){0.f, 0.f, 0.f, 0.f}; D[i][jj] = (f32x4){0.f, 0.f, 0.f, 0.f}; }

    // ---- prologue: first super-block's header and Sx, raw steps 0..3, activation steps 0..2; k 0..31 of step 0 converted ----
    issue_sb(sb_begin);
    issue_raw(0); issue_raw(1); issue_raw(2); issue_raw(3);
    issue_b(0); issue_b(1); issue_b(2);
    GEMM_WAIT_VMCNT(0);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    stage_sb(0);
    u32x2 rq[2];       // this lane's raw bytes of the step whose halves are being converted
    uint32_t an[2][4]; // the operand of the coming half, rows l16 and 16 + l16
    raw_of(0, rq);
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(rq[0]), "+v"(rq[1]));
#pragma unroll
    for (int i = 0; i < 2; i++) {
        _Float16 sc2, off2;
        scale_of(i, 0, sc2, off2);
        convert4(rq[i].x, 0, sc2, off2, an[i][0], an[i][1]);
        convert4(rq[i].y, 0, sc2, off2, an[i][2], an[i][3]);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();  // the mn6 / d / dmin that stage_sb wrote are visible
    asm volatile("" ::: "memory");

    uint32_t s = 0;
    for (uint32_t sb = sb_begin; sb < sb_end; sb++) {
        const uint32_t par = (sb - sb_begin) & 1u;
#pragma unroll
        for (int g = 0; g < 4; g++, s++) {
            // ---- requests: raw weights of step s+4, activations of step s+3, (at g = 1) the next super-block's header and Sx ----
            issue_raw(s + 4);
            issue_b(s + 3);
            if (g == 1) issue_sb(sb + 1);  // (after the barrier that ended g = 0: everybody is past this super-block's Sx)
            const uint32_t b_stage = b_lane + (s % P_NB) * P_B_STAGE;
            if (g == 0 && with_mins) {
                // offsets of the super-block: sum_sub mn6 * Sx as one 16-deep MFMA per block (A slots 2*sub+h = 32*mn6,
                // B slots = Sx_h/32: lane (l16, kg) holds slots 4kg .. 4kg+3)
                f16x4 amf[2], bmf[8];
#pragma unroll
                for (int i = 0; i < 2; i++) amf[i] = *reinterpret_cast<const f16x4 *>(plds + P_AM_OFF + (wm + i * 16 + l16) * 32 + kg * 8);
#pragma unroll
                for (int jj = 0; jj < 8; jj++) bmf[jj] = *reinterpret_cast<const f16x4 *>(plds + P_BM_OFF + (jj * 16 + l16) * 32 + kg * 8);
                // (D is free here: the sixteen products go there back to back, then they are folded in)
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int jj = 0; jj < 8; jj++)
                        D[i][jj] = __builtin_amdgcn_mfma_f32_16x16x16f16(amf[i], bmf[jj], (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    const f32x4 mv = *reinterpret_cast<const f32x4 *>(plds + P_DMIN_OFF + (par * PM + wm + i * 16 + kg * 4) * 4);
#pragma unroll
                    for (int jj = 0; jj < 8; jj++)
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[i][jj][e] = __builtin_fmaf(-mv[e], D[i][jj][e], acc[i][jj][e]);
                }
            }
            // ---- the step's sixteen operand reads (two halves x eight token blocks) run P_LA groups ahead of the MFMAs that
            //      use them, across the two halves; the raw bytes of the next step are requested before the first of them ----
            u32x4 bf[16];
            u32x2 rqn[2];
            uint32_t b_addr[2];
#pragma unroll
            for (int kk = 0; kk < 2; kk++) b_addr[kk] = b_stage + b_col[kk];
#define LARQL_RD(G) case G: asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(bf[G]) : "v"(b_addr[(G) >> 3]), "n"(((G) & 7) * 2048)); break;
            auto b_read = [&](int G) {
                switch (G) { LARQL_RD(0) LARQL_RD(1) LARQL_RD(2) LARQL_RD(3) LARQL_RD(4) LARQL_RD(5) LARQL_RD(6) LARQL_RD(7)
                             LARQL_RD(8) LARQL_RD(9) LARQL_RD(10) LARQL_RD(11) LARQL_RD(12) LARQL_RD(13) LARQL_RD(14) LARQL_RD(15) default: break; }
            };
#undef LARQL_RD
            // operand G has arrived when at most the reads issued after it are outstanding (reads return in order; anything
            // else issued in between only makes the wait stricter)
#define LARQL_WT(N) case N: asm volatile("s_waitcnt lgkmcnt(" #N ")" : "+v"(bf[G])); break;
            auto b_wait = [&](int G) {
                switch (min(P_LA, 15 - G)) { LARQL_WT(0) LARQL_WT(1) LARQL_WT(2) LARQL_WT(3) LARQL_WT(4) LARQL_WT(5) LARQL_WT(6) LARQL_WT(7) LARQL_WT(8) default: break; }
            };
#undef LARQL_WT
            asm volatile("" ::: "memory");  // (nothing of the above sinks below the counted reads)
            __builtin_amdgcn_sched_barrier(0);
            raw_of(s + 1, rqn);             // (its copy landed two steps ago: own rows, own copy)
#pragma unroll
            for (int G = 0; G < P_LA; G++) b_read(G);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int h = 0; h < 2; h++) {
                // ---- half h: the matrix cores take k 32h .. 32h+31 of step s; the threads convert, for h = 0, this step's
                //      k 32..63 (high nibbles of raw step s) and, for h = 1, the next step's k 0..31 (low nibbles of s+1).
                //      Both halves of the operand belong to this wavefront alone: no barrier between them ----
                if (h == 1 && g == 3) {
                    stage_sb(par ^ 1u);
                    asm volatile("" ::: "memory");
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (h == 1) { rq[0] = rqn[0]; rq[1] = rqn[1]; }
                const uint32_t nib = 1 - h;                                 // nibble of the half being converted
                const uint32_t nsub = h == 0 ? 2 * g + 1 : 2 * ((g + 1) & 3);
                f16x8 af[2];
#pragma unroll
                for (int i = 0; i < 2; i++) af[i] = __builtin_bit_cast(f16x8, (u32x4){an[i][0], an[i][1], an[i][2], an[i][3]});
                _Float16 sc2[2], off2[2];
                __builtin_amdgcn_sched_barrier(0);
                // eight groups of two MFMAs; six of them carry a piece of the conversion
#pragma unroll
                for (int jj = 0; jj < 8; jj++) {
                    const int G = h * 8 + jj;
                    if (G + P_LA < 16) b_read(G + P_LA);
                    b_wait(G);
                    // (these name what the group before produced: they keep each piece of the conversion between two
                    // groups instead of wherever its first use is; the raw bytes came back before operand 0)
                    if (G == 0) asm volatile("" : "+v"(rqn[0]), "+v"(rqn[1]));
                    if (jj == 1) asm volatile("" : "+v"(sc2[0]), "+v"(off2[0]));
                    if (jj == 2) asm volatile("" : "+v"(sc2[1]), "+v"(off2[1]));
                    if (jj == 3) asm volatile("" : "+v"(an[0][0]), "+v"(an[0][1]));
                    if (jj == 4) asm volatile("" : "+v"(an[0][2]), "+v"(an[0][3]));
                    if (jj == 5) asm volatile("" : "+v"(an[1][0]), "+v"(an[1][1]));
                    if (jj == 6) asm volatile("" : "+v"(an[1][2]), "+v"(an[1][3]));
                    if (jj == 0) scale_of(0, nsub, sc2[0], off2[0]);
                    if (jj == 1) scale_of(1, nsub, sc2[1], off2[1]);
                    if (jj == 2) convert4(rq[0].x, nib, sc2[0], off2[0], an[0][0], an[0][1]);
                    if (jj == 3) convert4(rq[0].y, nib, sc2[0], off2[0], an[0][2], an[0][3]);
                    if (jj == 4) convert4(rq[1].x, nib, sc2[1], off2[1], an[1][0], an[1][1]);
                    if (jj == 5) convert4(rq[1].y, nib, sc2[1], off2[1], an[1][2], an[1][3]);
                    const f16x8 bv = __builtin_bit_cast(f16x8, bf[G]);
#pragma unroll
                    for (int i = 0; i < 2; i++)  // (a super-block's first MFMAs start from zero: D is never cleared)
                        D[i][jj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i], bv, (g == 0 && h == 0) ? (f32x4){0.f, 0.f, 0.f, 0.f} : D[i][jj], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (h == 1 && g == 3) {
                    // ---- end of the super-block: acc += d * D ----
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        const f32x4 dv = *reinterpret_cast<const f32x4 *>(plds + P_D_OFF + (par * PM + wm + i * 16 + kg * 4) * 4);
#pragma unroll
                        for (int jj = 0; jj < 8; jj++) {
#pragma unroll
                            for (int e = 0; e < 4; e++) acc[i][jj][e] = __builtin_fmaf(dv[e], D[i][jj][e], acc[i][jj][e]);
                        }
                    }
                }
                asm volatile("" ::: "memory");
                if (h == 1) {
                    // ---- end of step: only the copies requested in this step and the one before may still fly (3 per
                    //      step, 5 at g = 1); at g = 2 only this step's, so that the header requested at g = 1 is there
                    //      for the conversion that opens the next super-block ----
                    if (g == 0) GEMM_WAIT_VMCNT(6);
                    else if (g == 1) GEMM_WAIT_VMCNT(8);
                    else if (g == 2) GEMM_WAIT_VMCNT(3);
                    else GEMM_WAIT_VMCNT(6);
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    __builtin_amdgcn_s_barrier();  // everybody's activation copies are visible; everybody is done with stage s
                }
                asm volatile("" ::: "memory");
            }
        }
    }
    GEMM_WAIT_VMCNT(0);  // the clamped requests past the end

    // Results leave through LDS so that a store instruction writes whole lines: each wavefront parks its 32-row x
    // 128-token block as [token][row] (token rows padded to 36 floats: the 8 lanes of a write phase hit 8 bank
    // groups) in its own 18 KB, then every lane stores 16 bytes of a 128-byte run of one token.
    __builtin_amdgcn_s_barrier();  // nobody's copies are still landing in what becomes another wavefront's block
    asm volatile("" ::: "memory");
    constexpr uint32_t EP_LD = P_EP_LD;
    float *blk = reinterpret_cast<float *>(plds) + wave * (PN * EP_LD);
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int jj = 0; jj < 8; jj++)
            *reinterpret_cast<f32x4 *>(blk + (jj * 16 + l16) * EP_LD + i * 16 + kg * 4) = acc[i][jj];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // own writes, own reads
    const bool vec_ok = (rows & 3u) == 0 && (((uintptr_t)(partial ? partial : out)) & 15u) == 0;
    const uint32_t rc = (lane & 7u) * 4, r = row0 + wm + rc;
#pragma unroll 4
    for (int it = 0; it < 16; it++) {
        const uint32_t tl = it * 8 + (lane >> 3), tok = tok0 + tl;
        if (tok >= seq) continue;
        f32x4 v = *reinterpret_cast<const f32x4 *>(blk + tl * EP_LD + rc);
        float *o = partial ? partial + ((size_t)blockIdx.z * seq + tok) * rows + r : out + (size_t)tok * rows + r;
        if (!partial) {  // (partial sums stay unscaled; q4k_gemm_reduce_kernel adds the slabs in order and scales)
            const float ts = tok_scale[tok];
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] *= ts;
        }
        if (vec_ok && r + 3 < rows) {
            f32x4 *ov = reinterpret_cast<f32x4 *>(o);
            if (!partial && accumulate) { const f32x4 old = *ov; v += old; }
            *ov = v;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (r + e < rows) o[e] = (!partial && accumulate) ? o[e] + v[e] : v[e];
        }
    }
}

// f32 activations -> bf16 hi (round to nearest even) and the bf16 of the remainder
hipError_t q4k_gemm_prep_launch(hipStream_t s, const void *x, int x_is_bf16, uint32_t hidden, uint32_t seq, uint16_t *xh, uint16_t *xl,
                                uint16_t *sx, float *tok_scale, int *any_lo) {
    if (seq == 0) return hipSuccess;
    hipLaunchKernelGGL(q4k_gemm_prep_kernel, dim3(seq), dim3(256), 0, s, x, x_is_bf16, hidden, xh, xl, sx, tok_scale, any_lo,
                       1);
    return hipGetLastError();
}


// K-ranges per output tile so that a launch fills the CUs (1 = no split)
uint32_t q4k_gemm_splits(uint32_t rows, uint32_t hidden, uint32_t seq, uint32_t cu_count) {
    const uint32_t nsb = hidden / 256;
    uint32_t s = 1;
    // one 256x128 workgroup per CU
    const uint64_t tiles = (uint64_t)((rows + PM - 1) / PM) * ((seq + PN - 1) / PN);
    while (s < 8 && tiles * s * 2 <= (uint64_t)cu_count && nsb / (s * 2) >= 4) s *= 2;
    return s;
}

hipError_t q4k_gemm_f16_launch(hipStream_t s, const uint8_t *w, const uint16_t *xh, const uint16_t *sx, const float *tok_scale, float *out,
                               uint32_t rows, uint32_t hidden, uint32_t seq, int with_mins, int accumulate, uint32_t splits, float *partial) {
    if (rows == 0 || seq == 0) return hipSuccess;
    const uint32_t nsb = hidden / 256;
    const bool split = splits > 1 && partial;
    const uint32_t per = split ? (nsb + splits - 1) / splits : nsb, z = split ? (nsb + per - 1) / per : 1;
    static std::atomic<bool> attr_set{false};  // dynamic LDS above 64 KB has to be allowed once per process
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void *)q4k_gemm_pipe_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    hipLaunchKernelGGL(q4k_gemm_pipe_kernel, dim3((rows + PM - 1) / PM, (seq + PN - 1) / PN, z), dim3(PTHREADS), P_LDS_BYTES, s, w, xh, sx,
                       tok_scale, out, rows, hidden, seq, with_mins, accumulate, per, split ? partial : (float *)nullptr);
    if (split) {
        const size_t n = (size_t)rows * seq;
        hipLaunchKernelGGL(q4k_gemm_reduce_kernel, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, s, partial, z, tok_scale, out, rows, seq, accumulate);
    }
    return hipGetLastError();
}

}  // namespace larql
