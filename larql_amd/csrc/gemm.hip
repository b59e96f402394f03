// gemm.hip — batched-prefill Q4_K GEMM on the gfx950 matrix cores.
//
//   out[s, r] = sum_k W[r, k] * X[s, k]      W: [rows, hidden] Q4_K,  X: [seq, hidden] bf16 or f32
//
// the contraction q4k_matmul_into computes (larql-compute/src/cpu/ops/q4_common/
// matmul.rs:20-139; `out` is [seq, rows] row-major), on f16 MFMA over the integer
// weights (see the formulation below).
#include <hip/hip_runtime.h>

#include <atomic>
#include <type_traits>
#include <stdint.h>
#include <stdlib.h>

#include "kernels.h"

namespace larql {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------------------
// The formulation: keep the weight an integer as long as possible.
//
//   out[s, r] = sum over super-blocks of  d[r] * (sum_k (sc6*q)[r,k] * x[s,k])  -  dmin[r] * (sum_sub mn6[r,sub] * Sx[s,sub])
//
// The activations are prepared once per call (q4k_gemm_prep_kernel): per token a power-of-two scale brings
// max|x| to [2^13, 2^14), x/scale is stored as f16 (exact for bf16 inputs; f32 inputs add a second f16 term
// and a second pass), and Sx, the sum of the represented activations over each 32-element sub-block, is stored
// (divided by 32, to stay inside f16) as an f16 pair (hi, lo).  The weight operand is made in registers from the
// raw nibbles (mask into the mantissa of an f16 1024 + q, one or two packed f16 instructions), never in memory.
// Two kernels share the tile, the copies and the tables:
//   * q4k_gemm_exact_kernel (host tier): the operand is sc6*q <= 945, exact in f16; per super-block a wavefront keeps
//     the integer sums apart (D), gets sum_sub mn6*Sx from one more MFMA per block (A slots 2*sub+h = 32 mn6,
//     B slots = Sx_h/32), and folds both into the f32 result with the row's d and dmin.
//   * q4k_gemm_pair_kernel (device tier): the row's scale rides in the operand, f16(d 2^E sc6) * (q - 8), and the
//     offsets' MFMA adds (8 d sc6 - dmin mn6) 2^E * Sx to the same accumulators; 2^-E and the token's scale are
//     applied once at the end.  3e-4 relative to the CPU value instead of 3e-7, no folds, half the registers.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float half_to_float(uint32_t lo16) { return (float)__builtin_bit_cast(_Float16, (uint16_t)lo16); }

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

// one block per token: scale, f16 terms, sub-block sums.  `x_is_bf16`: 16-bit inputs (exact in one term).
// A thread takes 8 consecutive elements at a time (one or two 16-byte loads); four neighbouring threads hold a
// 32-element sub-block.
__global__ void __launch_bounds__(1024) q4k_gemm_prep_kernel(const void *__restrict__ x, int x_is_bf16, uint32_t hidden,
                                                            uint16_t *__restrict__ xh, uint16_t *__restrict__ xl,
                                                            uint16_t *__restrict__ sx, float *__restrict__ tok_scale,
                                                            int *__restrict__ any_lo, int swap12, uint32_t seq,
                                                            const uint8_t *__restrict__ w, uint32_t rows, int *__restrict__ rexp) {
    __shared__ float red[16];
    const uint32_t t = threadIdx.x, nvec = hidden >> 3;  // hidden % 256 == 0
    if (blockIdx.x >= seq) {
        // the blocks behind the tokens: 16 lanes per weight row, E with max(|d|, |dmin|/16) * 2^E in [0.5, 1) over the row,
        // so that d 2^E sc6 <= 63 and 32 (8 d sc6 + dmin mn6) 2^E <= 48384 stay well inside f16
        const uint32_t row = (blockIdx.x - seq) * (blockDim.x >> 4) + (t >> 4), nsb = hidden >> 8;
        float m = 0.f;
        if (row < rows) {
            const uint8_t *p = w + (size_t)row * nsb * 144;
            for (uint32_t sb0 = t & 15u; sb0 < nsb; sb0 += 64) {  // four independent loads in flight per lane
                uint32_t h[4];
#pragma unroll
                for (int u = 0; u < 4; u++) h[u] = sb0 + 16 * u < nsb ? *reinterpret_cast<const uint32_t *>(p + (size_t)(sb0 + 16 * u) * 144) : 0u;
#pragma unroll
                for (int u = 0; u < 4; u++)
                    m = fmaxf(m, fmaxf(fabsf(half_to_float(h[u] & 0xFFFFu)), 0.0625f * fabsf(half_to_float(h[u] >> 16))));
            }
        }
        for (int o = 8; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
        if (row < rows && (t & 15u) == 0) {
            int e = 0;
            if (m > 0.f && m < __builtin_inff()) (void)frexpf(m, &e);
            rexp[row] = -e;
        }
        return;
    }
    const uint32_t tok = blockIdx.x;
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
    for (uint32_t v = t; v < nvec; v += blockDim.x) {
        float o[8];
        load8(v, o);
#pragma unroll
        for (int i = 0; i < 8; i++) mx = fmaxf(mx, fabsf(o[i]));
    }
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if ((t & 63u) == 0) red[t >> 6] = mx;
    __syncthreads();
    mx = 0.f;
    for (uint32_t wv = 0; wv < (blockDim.x >> 6); wv++) mx = fmaxf(mx, red[wv]);
    int ex = 0;
    if (mx > 0.f && mx < __builtin_inff()) (void)frexpf(mx, &ex);
    ex = max(-100, min(110, ex));
    const float to_h = ldexpf(1.f, 14 - ex);
    if (t == 0) tok_scale[tok] = ldexpf(1.f, ex - 14);
    int lo_seen = 0;
    // the f16 terms are kept as [token][hidden] (a step's 128 bytes of a token are one cache line; a [step][token] order
    // was measured: no faster for the GEMM, slower here) and the sums as [super-block][token][8], so that what a GEMM
    // workgroup copies of them for a super-block is one contiguous run
    u32x4 *oh = reinterpret_cast<u32x4 *>(xh);
    u32x4 *ol = xl ? reinterpret_cast<u32x4 *>(xl) : nullptr;
    for (uint32_t v = t; v < nvec; v += blockDim.x) {  // nvec % 32 == 0: the four threads of a sub-block run together
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
        const size_t at = (size_t)tok * nvec + v;
        oh[at] = (u32x4){hw[0], hw[1], hw[2], hw[3]};
        if (ol) ol[at] = (u32x4){lw[0], lw[1], lw[2], lw[3]};
        sm += __shfl_xor(sm, 1);
        sm += __shfl_xor(sm, 2);
        sm *= 0.03125f;  // stored as Sx/32 so that 32 x 2^14 stays inside f16; the min operand carries the 32
        if ((t & 3u) == 0) {
            const _Float16 sh = (_Float16)sm;
            const _Float16 sl = (_Float16)(sm - (float)sh);
            const uint32_t pair = (uint32_t)__builtin_bit_cast(uint16_t, sh) | ((uint32_t)__builtin_bit_cast(uint16_t, sl) << 16);
            reinterpret_cast<uint32_t *>(sx)[((size_t)(v >> 5) * seq + tok) * 8 + ((v >> 2) & 7u)] = pair;
        }
    }
    if (lo_seen && any_lo) *any_lo = 1;
}

// adds the partial slabs of a K-split in slab order and applies the token scale; VEC elements per thread (4 when
// rows % 4 == 0 and everything is 16-byte aligned: the four are then of one token)
template <int VEC>
__global__ void __launch_bounds__(256) q4k_gemm_reduce_kernel(const float *__restrict__ partial, uint32_t splits, const float *__restrict__ tok_scale,
                                                              float *__restrict__ out, uint32_t rows, uint32_t seq, int accumulate) {
    const size_t n = (size_t)rows * seq, i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if (i >= n) return;
    float s[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) s[e] = 0.f;
    for (uint32_t z = 0; z < splits; z++) {
        if (VEC == 4) {
            const f32x4 v = *reinterpret_cast<const f32x4 *>(partial + (size_t)z * n + i);
#pragma unroll
            for (int e = 0; e < VEC; e++) s[e] += v[e];
        } else {
            s[0] += partial[(size_t)z * n + i];
        }
    }
    const float ts = tok_scale[i / rows];
    if (VEC == 4) {
        f32x4 r = {s[0] * ts, s[VEC > 1 ? 1 : 0] * ts, s[VEC > 2 ? 2 : 0] * ts, s[VEC > 3 ? 3 : 0] * ts};
        f32x4 *o = reinterpret_cast<f32x4 *>(out + i);
        if (accumulate) r += *o;
        *o = r;
    } else {
        out[i] = accumulate ? out[i] + s[0] * ts : s[0] * ts;
    }
}

// ---------------------------------------------------------------------------
// The host tier's kernel: the weight operand is the integer sc6*q, a super-block's sums are kept apart (D) and folded
// into the result with the row's f32 d / dmin, so the only roundings are the f32 accumulations (the trait's callers
// compare a row of the matmul with the CPU matvec at 1e-4 absolute).
// with_mins = 0: the activation term carries no offset part (second pass over the lo terms).
//
// One workgroup of 4 wavefronts per CU owns a 256-row x 128-token tile; a wavefront owns 64 of the rows against
// all 128 tokens (2 x 4 blocks of v_mfma_f32_32x32x16_f16: an operand read from LDS feeds two MFMAs of 32 cycles).
// Everything a step (64 k) needs from global memory was copied global -> LDS (global_load_lds, 16 bytes per lane,
// no registers involved) at least two steps before:
//   * the f16 activations of a step, into a ring of four stages.  Rows are 128 bytes (64 f16) without
//     padding; the 16-byte chunk c of row r is kept at position c ^ ((r >> 1) & 7), chosen on the global side of
//     the copy, so that sixteen neighbouring lanes of an operand read (sixteen rows, one chunk) cover the 64 banks;
//   * the weights a super-block at a time (144 bytes per row, header included: a row's two or three cache lines
//     are asked for once, not once per step), into two stages (a wavefront copies its own rows);
//   * per super-block the Sx of the tile's tokens.
// A wavefront turns the headers of its rows into two small LDS tables once per super-block (one thread per row):
// per sub-block the packed-FMA operands (scale, -1024 * scale) and the offsets' MFMA operand.
// The f16 weight operand never exists in memory: lane (row32, kgrp) of an MFMA holds 8 k of row row32.  The k
// of a step are dealt so that a lane needs 16 consecutive raw bytes of its row: MFMA j of half h takes the
// nibbles h of bytes 16*kgrp + 8j .. +7, i.e. k 32h + 16kgrp + 8j .. +7 (the activations' chunk 4h + 2kgrp + j).
// The lane reads those 16 bytes of its two rows once per step and converts them, in the MFMAs' shadow, into the
// operand of the next half.  Only the activations cross wavefronts: one barrier per step, in the middle of it, so
// that the operand reads of the next step's first MFMAs are already issued when the step ends.  No global load
// returns into a register inside the loop, so the compiler places no vmcnt waits of its own (it would wait for
// *all* outstanding loads as soon as register loads and LDS copies are in flight together); outstanding copies
// are counted by hand: at the barrier only the requests made at the barrier before may still fly.  For the same
// reason (an LDS copy in flight makes the compiler wait for lgkmcnt(0) at every LDS read) the operand reads of
// the loop are written as instructions with counted waits, G_LA reads ahead of the MFMA group that consumes them.
// ---------------------------------------------------------------------------
constexpr int GM = 256, GN = 128, GTHREADS = 256;
constexpr int G_LA = 4;                                                         // operand reads in flight ahead of the MFMAs
constexpr int G_NB = 4, G_NR = 2;                                               // ring depths: activations (steps), weights (super-blocks)
constexpr int G_B_STAGE = GN * 128, G_R_STAGE = GM * 144;                       // bytes
constexpr int G_B_OFF = 0, G_R_OFF = G_B_OFF + G_NB * G_B_STAGE,
              G_BM_OFF = G_R_OFF + G_NR * G_R_STAGE, G_SC_OFF = G_BM_OFF + GN * 32, G_AM_OFF = G_SC_OFF + GM * 32,
              G_D_OFF = G_AM_OFF + GM * 32, G_DMIN_OFF = G_D_OFF + 2 * GM * 4, G_LOOP_BYTES = G_DMIN_OFF + 2 * GM * 4;
constexpr int G_EP_LD = 68, G_EP_BYTES = 4 * GN * G_EP_LD * 4;                  // the results leave through LDS (see the epilogue)
constexpr int G_LDS_BYTES = G_LOOP_BYTES > G_EP_BYTES ? G_LOOP_BYTES : G_EP_BYTES;
static_assert(G_LDS_BYTES <= 160 * 1024, "one workgroup per CU");
static_assert(G_NB == 4 && G_NR == 2, "ring slots are named by the step's position in its super-block and the super-block's parity");
typedef __attribute__((address_space(3))) void *p_lds_vp;
typedef const __attribute__((address_space(1))) void *p_g_vp;
typedef float f32x16 __attribute__((ext_vector_type(16)));
#define GEMM_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

__global__ void __launch_bounds__(GTHREADS, 1) q4k_gemm_exact_kernel(const uint8_t *w, const uint16_t *xh, const uint16_t *sx,
                                                               const float *__restrict__ tok_scale, float *__restrict__ out,
                                                               uint32_t rows, uint32_t hidden, uint32_t seq, int with_mins,
                                                               int accumulate, uint32_t sb_per_split, float *__restrict__ partial) {
    extern __shared__ __attribute__((aligned(16))) uint8_t glds[];
    const uint32_t t = threadIdx.x, lane = t & 63u, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t row0 = blockIdx.x * GM, tok0 = blockIdx.y * GN;
    const uint32_t nsb = hidden >> 8, row_bytes = nsb * 144;
    const uint32_t sb_begin = blockIdx.z * sb_per_split, sb_end = min(nsb, sb_begin + sb_per_split);
    if (sb_begin >= sb_end) return;
    const uint32_t nsteps = (sb_end - sb_begin) * 4;

    // copy roles.  Weights: a super-block of the wavefront's 64 rows (144 bytes each, header included) is nine copies;
    // piece p, lane l brings 16-byte chunk (64p + l) % 9 of row (64p + l) / 9, so that the rows lie in LDS one after the
    // other and a row's two or three cache lines are asked for by neighbouring lanes of one instruction.
    const uint8_t *wt = w + (size_t)row0 * row_bytes;                                          // uniform
    uint32_t r_off[9];
#pragma unroll
    for (int p9 = 0; p9 < 9; p9++) {
        const uint32_t idx = p9 * 64 + lane;
        r_off[p9] = (min(row0 + wave * 64 + idx / 9, rows - 1) - row0) * row_bytes + (idx % 9) * 16;
    }
    // activations ([token][hidden] f16): wavefront -> tokens 32w .. 32w+31 (four copies of 8 tokens x 128 bytes), lane -> (token, chunk)
    const uint8_t *xt = (const uint8_t *)xh;                                                   // uniform
    uint32_t b_off[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const uint32_t r = (wave * 4 + q) * 8 + (lane >> 3);
        b_off[q] = min(tok0 + r, seq - 1) * hidden * 2 + (((lane & 7u) ^ ((r >> 1) & 7u)) * 16);
    }
    // Sx ([super-block][token][8 pairs]): wavefront -> tokens 32w .. 32w+31 (two 16-byte halves each)
    const uint8_t *st = (const uint8_t *)sx;                                                   // uniform
    const uint32_t m_off = min(tok0 + wave * 32 + (lane >> 1), seq - 1) * 32 + (lane & 1u) * 16;

    // compute role: a wavefront owns the 64 rows it converts, against all 128 tokens: the weight operand, the raw
    // bytes, the headers and the per-row tables never cross wavefronts, only the activations (and Sx) do
    const uint32_t wm = wave * 64;
    const uint32_t row32 = lane & 31u, kgrp = lane >> 5;

    // (requests past the end are clamped: same number of copies in flight, results unused)
    auto issue_raw = [&](uint32_t sb, int p9) {  // one of the nine pieces of a super-block
        const uint8_t *src = wt + (size_t)min(sb, sb_end - 1) * 144;
        uint8_t *dst = glds + G_R_OFF + ((sb - sb_begin) & 1u) * G_R_STAGE + wave * 9216;
        __builtin_amdgcn_global_load_lds((p_g_vp)(src + r_off[p9]), (p_lds_vp)(dst + p9 * 1024), 16, 0, 0);
    };
    auto issue_b = [&](uint32_t s, uint32_t slot, int q) {  // one of the four pieces of a step
        const uint32_t sc = min(s, nsteps - 1);
        const uint8_t *src = xt + ((size_t)sb_begin * 4 + sc) * 128;
        uint8_t *dst = glds + G_B_OFF + slot * G_B_STAGE + wave * 4096;
        __builtin_amdgcn_global_load_lds((p_g_vp)(src + b_off[q]), (p_lds_vp)(dst + q * 1024), 16, 0, 0);
    };
    auto issue_sx = [&](uint32_t sb) {  // Sx of a super-block
        const uint32_t sbc = min(sb, sb_end - 1);
        __builtin_amdgcn_global_load_lds((p_g_vp)((st + (size_t)sbc * seq * 32) + m_off), (p_lds_vp)(glds + G_BM_OFF + wave * 1024), 16, 0, 0);
    };
    // a super-block's header -> this row's tables.  Scales: per sub-block the pair (sc6, -1024 sc6) for the packed FMA
    // that turns a masked nibble 1024 + q into sc6*q.  Odd sub-blocks are the high nibbles, whose masked value is
    // 1024 + 16q, so they carry sc6/16.  Offsets: 32 mn6 twice, for the two f16 halves of Sx/32.
    auto stage_sb = [&](uint32_t par) {
        const u32x4 hdr = *reinterpret_cast<const u32x4 *>(glds + G_R_OFF + par * G_R_STAGE + wave * 9216 + lane * 144);
        const float d = half_to_float(hdr.x & 0xFFFFu), dmin = half_to_float(hdr.x >> 16);
        uint32_t mnw[8];
#pragma unroll
        for (int sub = 0; sub < 8; sub++) {
            const uint32_t sh = 8u * (sub & 3u);
            const uint32_t pa = (hdr.y >> sh) & 0xFFu, pb = (hdr.z >> sh) & 0xFFu, pc = (hdr.w >> sh) & 0xFFu;
            const uint32_t sc6 = sub < 4 ? (pa & 63u) : ((pc & 0x0Fu) | ((pa >> 6) << 4));
            const uint32_t mn6 = sub < 4 ? (pb & 63u) : ((pc >> 4) | ((pb >> 6) << 4));
            const float sf = (float)sc6 * ((sub & 1) ? 0.0625f : 1.f);
            const _Float16 s16 = (_Float16)sf, o16 = (_Float16)(-1024.f * sf);
            *reinterpret_cast<uint32_t *>(glds + G_SC_OFF + wave * 2048 + sub * 256 + lane * 4) =
                (uint32_t)__builtin_bit_cast(uint16_t, s16) | ((uint32_t)__builtin_bit_cast(uint16_t, o16) << 16);
            const uint32_t hb = __builtin_bit_cast(uint16_t, (_Float16)(32.f * (float)mn6));
            mnw[sub] = hb | (hb << 16);
        }
        *reinterpret_cast<u32x4 *>(glds + G_AM_OFF + (wm + lane) * 32) = (u32x4){mnw[0], mnw[1], mnw[2], mnw[3]};
        *reinterpret_cast<u32x4 *>(glds + G_AM_OFF + (wm + lane) * 32 + 16) = (u32x4){mnw[4], mnw[5], mnw[6], mnw[7]};
        reinterpret_cast<float *>(glds + G_D_OFF)[par * GM + wm + lane] = d;
        reinterpret_cast<float *>(glds + G_DMIN_OFF)[par * GM + wm + lane] = dmin;
    };
    // 4 raw bytes (nibble h) -> two dwords of f16(sc6*q), exact (sc6*q <= 945), as the pairs (k0, k2) and (k1, k3): the
    // nibbles of bytes 0 and 2 are masked in place into the mantissas of two f16 (1024 + q, or 1024 + 16q for the high
    // nibbles), those of bytes 1 and 3 after one shift; one packed FMA takes the 1024 away and applies sc6.
    // `magic` is 0x64006400 held in a register so that mask-and-or is one instruction; `sp` is a table entry (s, -1024 s).
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));
    auto convert4 = [&](uint32_t raw, uint32_t h, uint32_t sp, uint32_t &o0, uint32_t &o1) {
        const f16x2 p = __builtin_bit_cast(f16x2, sp);
        const f16x2 sc2 = {p[0], p[0]}, off2 = {p[1], p[1]};  // (broadcast by the instruction's operand selects, not by a pack)
        const uint32_t mask = h ? 0x00F000F0u : 0x000F000Fu;
        const f16x2 m02 = __builtin_bit_cast(f16x2, (raw & mask) | magic);
        const f16x2 m13 = __builtin_bit_cast(f16x2, ((raw >> 8) & mask) | magic);
        o0 = __builtin_bit_cast(uint32_t, m02 * sc2 + off2);
        o1 = __builtin_bit_cast(uint32_t, m13 * sc2 + off2);
    };
    // The reads of the main loop are written as instructions with hand-counted waits: while LDS copies are in flight
    // the compiler's own wait for an LDS read is lgkmcnt(0), i.e. it would drain the reads issued ahead with the one
    // that is needed.  LDS reads return in order, so "all but the last n" is exact.
    const uint32_t lds0 = (uint32_t)(uintptr_t)(p_lds_vp)glds;
    const uint32_t raw_lane = lds0 + G_R_OFF + wave * 9216 + row32 * 144 + 16 + kgrp * 16;
    auto raw_of = [&](uint32_t par, uint32_t g4, u32x4 (&rq)[2]) {  // step g4 of the super-block in slot `par`
        const uint32_t a = raw_lane + par * G_R_STAGE + g4 * 32;
        asm volatile("ds_read_b128 %0, %1" : "=v"(rq[0]) : "v"(a));
        asm volatile("ds_read_b128 %0, %1 offset:4608" : "=v"(rq[1]) : "v"(a));
    };
    const uint32_t sc_lane = lds0 + G_SC_OFF + wave * 2048 + row32 * 4;
    auto scales_of = [&](uint32_t sub, uint32_t (&sp)[2]) {  // the table entries of sub-block `sub` for this lane's two rows
        const uint32_t a = sc_lane + sub * 256;
        asm volatile("ds_read_b32 %0, %1" : "=v"(sp[0]) : "v"(a));
        asm volatile("ds_read_b32 %0, %1 offset:128" : "=v"(sp[1]) : "v"(a));
    };
    const uint32_t b_lane = lds0 + G_B_OFF + row32 * 128;
    uint32_t b_col[4];  // byte position of this lane's chunk in a token's row, for the four MFMA depths (h, j) of a step
#pragma unroll
    for (int c = 0; c < 4; c++) b_col[c] = (((uint32_t)(c >> 1) * 4 + 2 * kgrp + (c & 1)) ^ ((row32 >> 1) & 7u)) << 4;

    f32x16 acc[2][4], D[2][4];  // the result; the integer sums of the current super-block
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int jj = 0; jj < 4; jj++)
#pragma unroll
            for (int e = 0; e < 16; e++) {
                acc[i][jj][e] = 0.f;
                D[i][jj][e] = 0.f;
            }

    // ---- prologue: the first super-block's weights and Sx, six pieces of the second's, activation steps 0..2; k 0..31 of step 0 converted ----
    issue_sx(sb_begin);
#pragma unroll
    for (int p9 = 0; p9 < 9; p9++) issue_raw(sb_begin, p9);
#pragma unroll
    for (int p9 = 0; p9 < 6; p9++) issue_raw(sb_begin + 1, p9);
#pragma unroll
    for (int q = 0; q < 4; q++) { issue_b(0, 0, q); issue_b(1, 1, q); issue_b(2, 2, q); }
    GEMM_WAIT_VMCNT(0);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    stage_sb(0);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    u32x4 rq[2];        // this lane's raw bytes of the step whose halves are being converted
    uint32_t an[2][2][4];  // the operand of the coming half: [row block][j][dword]
    uint32_t scn[2];    // table entries for the conversions of the coming half
    u32x4 pf[4];        // the first G_LA operand reads of the coming step
    {
        uint32_t sp0[2];
        raw_of(0, 0, rq);
        scales_of(0, sp0);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(rq[0]), "+v"(rq[1]), "+v"(sp0[0]), "+v"(sp0[1]));
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) {
                convert4(rq[i][2 * j], 0, sp0[i], an[i][j][0], an[i][j][1]);
                convert4(rq[i][2 * j + 1], 0, sp0[i], an[i][j][2], an[i][j][3]);
            }
        scales_of(1, scn);
#pragma unroll
        for (int G = 0; G < G_LA; G++) {
            const uint32_t a = b_lane + b_col[0] + G * 4096;
            asm volatile("ds_read_b128 %0, %1" : "=v"(pf[G]) : "v"(a));
        }
    }

    uint32_t s = 0;
    for (uint32_t sb = sb_begin; sb < sb_end; sb++) {
        const uint32_t par = (sb - sb_begin) & 1u;
#pragma unroll
        for (int g = 0; g < 4; g++, s++) {
            // ---- top of the step: (g = 3) the next super-block's tables, (g = 0) this one's offsets ----
            if (g == 3) {
                stage_sb(par ^ 1u);  // (its weights landed before the barrier of g = 2; the entries still needed of this one are in registers)
                asm volatile("" ::: "memory");
            }
            if (g == 0 && with_mins) {
                // sum_sub mn6 * Sx as one 16-deep MFMA per block (A slots 2*sub+h = the offsets' operand, B slots = Sx_h/32:
                // lane (row32, kgrp) holds slots 8kgrp .. 8kgrp+7)
                f16x8 amf[2], bmf[4];
#pragma unroll
                for (int i = 0; i < 2; i++) amf[i] = *reinterpret_cast<const f16x8 *>(glds + G_AM_OFF + (wm + i * 32 + row32) * 32 + kgrp * 16);
#pragma unroll
                for (int jj = 0; jj < 4; jj++) bmf[jj] = *reinterpret_cast<const f16x8 *>(glds + G_BM_OFF + (jj * 32 + row32) * 32 + kgrp * 16);
                // (D is free here: the products go there, then they are folded in with the rows' dmin)
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int jj = 0; jj < 4; jj++) {
                        f32x16 z;
#pragma unroll
                        for (int e = 0; e < 16; e++) z[e] = 0.f;
                        D[i][jj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(amf[i], bmf[jj], z, 0, 0, 0);
                    }
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const f32x4 mv = *reinterpret_cast<const f32x4 *>(glds + G_DMIN_OFF + (par * GM + wm + i * 32 + q * 8 + kgrp * 4) * 4);
#pragma unroll
                        for (int jj = 0; jj < 4; jj++)
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                acc[i][jj][4 * q + e] = __builtin_fmaf(-mv[e], D[i][jj][4 * q + e], acc[i][jj][4 * q + e]);
                    }
            }
            // ---- the step's sixteen operand reads (four depths x four token blocks) run G_LA groups ahead of the MFMAs that
            //      use them, into the next step at the end; the raw bytes of the next step are requested first ----
            u32x4 bf[16];
            u32x4 rqn[2];
            uint32_t b_addr[4];
#pragma unroll
            for (int c = 0; c < 4; c++) b_addr[c] = b_lane + (uint32_t)g * G_B_STAGE + b_col[c];
            const uint32_t b_next = b_lane + (uint32_t)((g + 1) & 3) * G_B_STAGE + b_col[0];
#define LARQL_RD(G) case G: asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(bf[G]) : "v"(b_addr[(G) >> 2]), "n"(((G) & 3) * 4096)); break;
#define LARQL_RN(G) case 16 + G: asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(pf[G]) : "v"(b_next), "n"((G) * 4096)); break;
            auto b_read = [&](int G) {
                switch (G) { LARQL_RD(4) LARQL_RD(5) LARQL_RD(6) LARQL_RD(7) LARQL_RD(8) LARQL_RD(9) LARQL_RD(10) LARQL_RD(11)
                             LARQL_RD(12) LARQL_RD(13) LARQL_RD(14) LARQL_RD(15) LARQL_RN(0) LARQL_RN(1) LARQL_RN(2) LARQL_RN(3) default: break; }
            };
#undef LARQL_RD
#undef LARQL_RN
            asm volatile("" ::: "memory");  // (nothing of the above sinks below the counted reads)
            __builtin_amdgcn_sched_barrier(0);
            raw_of(g == 3 ? par ^ 1u : par, (uint32_t)((g + 1) & 3), rqn);  // (own rows, own copies, landed before the barrier of the step before)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int h = 0; h < 2; h++) {
                if (h == 1) {
                    // ---- middle of the step: everything requested before the last barrier has landed (after it: the step's 4
                    //      activation copies, plus 3 weight pieces and Sx at g = 0, 3 weight pieces at g = 2 and 3); after this
                    //      barrier everybody's activations of step s+1 are visible and everybody is done with step s-1, whose
                    //      slot the activations of step s+3 take.  The next super-block's weights are complete with the pieces
                    //      of g = 0, two barriers before their first use at the top of g = 3; the slot of the one after is free
                    //      from the top of g = 2.  The requests themselves go out one per MFMA group of the second half (a
                    //      burst of eight here costs the matrix cores 0.1-0.2 us) ----
                    if (g == 1) GEMM_WAIT_VMCNT(8);
                    else if (g == 2) GEMM_WAIT_VMCNT(4);
                    else GEMM_WAIT_VMCNT(7);
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    __builtin_amdgcn_sched_barrier(0);
                }
                // ---- half h: the matrix cores take k 32h .. 32h+31 of step s; the threads convert, for h = 0, this step's
                //      high nibbles and, for h = 1, the next step's low nibbles.  Both halves of the operand belong to this
                //      wavefront alone ----
                if (h == 1) { rq[0] = rqn[0]; rq[1] = rqn[1]; }
                uint32_t scv[2] = {scn[0], scn[1]};
                // table entries for the conversions of the half after this one
                scales_of(h == 0 ? 2u * ((g + 1) & 3) : (g == 3 ? 1u : 2u * (g + 1) + 1u), scn);
                const uint32_t nib = 1 - h;                                 // nibble of the half being converted
                f16x8 af[2][2];
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++) af[i][j] = __builtin_bit_cast(f16x8, (u32x4){an[i][j][0], an[i][j][1], an[i][j][2], an[i][j][3]});
                __builtin_amdgcn_sched_barrier(0);
                // eight groups of two MFMAs; each carries one piece of the conversion
#pragma unroll
                for (int jj = 0; jj < 8; jj++) {
                    const int G = h * 8 + jj;
                    if (h == 1) {  // this group's copy request
                        if (jj < 4) issue_b(s + 3, (uint32_t)((g + 3) & 3), jj);
                        else if (jj < 7) {
                            if (g == 0) issue_raw(sb + 1, 6 + jj - 4);
                            if (g == 2) issue_raw(sb + 2, jj - 4);
                            if (g == 3) issue_raw(sb + 2, 3 + jj - 4);
                        } else if (g == 0) issue_sx(sb + 1);  // (everybody took this super-block's Sx before the barrier)
                    }
                    b_read(G + G_LA);
                    // operand G has arrived when at most the G_LA reads issued after it are outstanding (reads return in order;
                    // anything else issued in between only makes the wait stricter)
                    if (G < 4) asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(pf[G < 4 ? G : 0]));
                    else asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(bf[G]));
                    // (these name what came back before this group's operand: they keep each piece of the conversion between
                    // two groups instead of wherever its first use is)
                    if (jj == 0) asm volatile("" : "+v"(scv[0]), "+v"(scv[1]), "+v"(rq[0]), "+v"(rq[1]));
                    {
                        const int i = jj >> 2, j = (jj >> 1) & 1, dd = jj & 1;
                        if (jj > 0) asm volatile("" : "+v"(an[(jj - 1) >> 2][((jj - 1) >> 1) & 1][2 * ((jj - 1) & 1)]), "+v"(an[(jj - 1) >> 2][((jj - 1) >> 1) & 1][2 * ((jj - 1) & 1) + 1]));
                        convert4(rq[i][2 * j + dd], nib, scv[i], an[i][j][2 * dd], an[i][j][2 * dd + 1]);
                    }
                    const f16x8 bv = __builtin_bit_cast(f16x8, G < 4 ? pf[G < 4 ? G : 0] : bf[G]);
                    const int j = (G >> 2) & 1, tb = G & 3;
#pragma unroll
                    for (int i = 0; i < 2; i++) {  // (a super-block's first MFMAs start from zero: D is never cleared)
                        f32x16 z;
#pragma unroll
                        for (int e = 0; e < 16; e++) z[e] = 0.f;
                        D[i][tb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i][j], bv, (g == 0 && h == 0 && j == 0) ? z : D[i][tb], 0, 0, 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                asm volatile("" ::: "memory");
            }
            if (g == 3) {
                // ---- end of the super-block: acc += d * D ----
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const f32x4 dv = *reinterpret_cast<const f32x4 *>(glds + G_D_OFF + (par * GM + wm + i * 32 + q * 8 + kgrp * 4) * 4);
#pragma unroll
                        for (int jj = 0; jj < 4; jj++)
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                acc[i][jj][4 * q + e] = __builtin_fmaf(dv[e], D[i][jj][4 * q + e], acc[i][jj][4 * q + e]);
                    }
                asm volatile("" ::: "memory");
            }
        }
    }
    // the clamped requests past the end and the operand reads issued for a step that does not exist
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(pf[0]), "+v"(pf[1]), "+v"(pf[2]), "+v"(pf[3]), "+v"(scn[0]), "+v"(scn[1]));
    GEMM_WAIT_VMCNT(0);

    // Results leave through LDS so that a store instruction writes whole lines: each wavefront parks its 64-row x
    // 128-token block as [token][row] (token rows padded to 68 floats: the 8 lanes of a write phase hit 8 bank
    // groups) in its own 34 KB, then every lane stores 16 bytes of a 256-byte run of one token.
    __builtin_amdgcn_s_barrier();  // nobody's copies are still landing in what becomes another wavefront's block
    asm volatile("" ::: "memory");
    constexpr uint32_t EP_LD = G_EP_LD;
    float *blk = reinterpret_cast<float *>(glds) + wave * (GN * EP_LD);
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int jj = 0; jj < 4; jj++)
#pragma unroll
            for (int q = 0; q < 4; q++)  // registers 4q .. 4q+3 of a block: rows 8q + 4kgrp .. +3, token row32
                *reinterpret_cast<f32x4 *>(blk + (jj * 32 + row32) * EP_LD + i * 32 + q * 8 + kgrp * 4) =
                    (f32x4){acc[i][jj][4 * q], acc[i][jj][4 * q + 1], acc[i][jj][4 * q + 2], acc[i][jj][4 * q + 3]};
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // own writes, own reads
    const bool vec_ok = (rows & 3u) == 0 && (((uintptr_t)(partial ? partial : out)) & 15u) == 0;
    const uint32_t rc = (lane & 15u) * 4, r = row0 + wm + rc;
#pragma unroll 4
    for (int it = 0; it < 32; it++) {
        const uint32_t tl = it * 4 + (lane >> 4), tok = tok0 + tl;
        if (tok >= seq) continue;
        f32x4 v = *reinterpret_cast<const f32x4 *>(blk + tl * EP_LD + rc);
        float *o = partial ? partial + ((size_t)blockIdx.z * seq + tok) * rows + r : out + (size_t)tok * rows + r;
        // (partial sums stay without the token's scale; q4k_gemm_reduce_kernel adds the slabs in order and applies it)
        const float ts = partial ? 1.f : tok_scale[tok];
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] *= ts;
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

// ---------------------------------------------------------------------------
// The device tier's kernel: the same tile, copies and tables with 8 wavefronts, two per SIMD.  A wavefront with its
// own instruction stream hides at most ~3 vector instructions per 32x32x16 MFMA (measured: 32, 37, 44, 56 cycles per
// MFMA with 2, 4, 6, 8 vector instructions after it); two wavefronts per SIMD hide ~6 each.  The conversion alone
// is 3.5 per MFMA, so the 64 rows x 128 tokens of a row group are computed by a pair of wavefronts that split every
// step's k: wavefront kh takes the nibbles kh (k 32kh .. 32kh+31 of the step: sub-block 2g + kh) of the same raw bytes
// against the same tokens.  No weight is converted twice and no activation read twice; each wavefront keeps a full
// set of partial sums (128 registers), which the pair adds up through LDS at the end.  The rows' scales ride in the
// operand (the formulation at the top of this file); with a second set of accumulators the exact variant does not
// fit in the 256 registers a wavefront has here and stays with q4k_gemm_exact_kernel.
// The two wavefronts of a SIMD take turns (see the loop): while one issues a step's 16 MFMAs back to back, the other
// prepares its next step; with both doing a bit of everything all the time, a workgroup barrier per step made them
// run one after the other, each at about half the matrix pipe's rate.
// ---------------------------------------------------------------------------
constexpr int QTHREADS = 512;
// one global -> LDS copy of 16 bytes per lane: uniform base + per-lane 32-bit offset on the global side (no 64-bit
// address registers), uniform LDS address (the lanes' 16-byte slots follow one another from there)
__device__ __forceinline__ void copy16_to_lds(const void *base, uint32_t lane_off, uint32_t lds_addr) {
    const uint64_t b = (uint64_t)(uintptr_t)base;  // (uniform by construction: told to the compiler, which otherwise may keep them in vector registers)
    const uint64_t bs = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32)) << 32) | (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(__builtin_amdgcn_readfirstlane((int)lds_addr)), "v"(lane_off), "s"(bs) : "memory");  // (m0 is not the compiler's to allocate; nothing else in these kernels uses it)
}

__global__ void __launch_bounds__(QTHREADS) q4k_gemm_pair_kernel(const uint8_t *w, const uint16_t *xh, const uint16_t *sx, const int *__restrict__ rexp,
                                                                  const float *__restrict__ tok_scale, float *__restrict__ out,
                                                                  uint32_t rows, uint32_t hidden, uint32_t seq, int with_mins,
                                                                  int accumulate, uint32_t sb_per_split, float *__restrict__ partial) {
    extern __shared__ __attribute__((aligned(16))) uint8_t glds[];
    const uint32_t t = threadIdx.x, lane = t & 63u, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t wq = wave & 3u, kh = wave >> 2;  // row group, k half: wavefronts w and w+4 run on one SIMD
    const uint32_t row0 = blockIdx.x * GM, tok0 = blockIdx.y * GN;
    const uint32_t nsb = hidden >> 8, row_bytes = nsb * 144;
    const uint32_t sb_begin = blockIdx.z * sb_per_split, sb_end = min(nsb, sb_begin + sb_per_split);
    if (sb_begin >= sb_end) return;
    const uint32_t nsteps = (sb_end - sb_begin) * 4;
    const uint32_t wm = wq * 64;

    // copy roles.  Weights: a super-block of a row group's 64 rows (144 bytes each, header included) is nine copies; piece p,
    // lane l brings 16-byte chunk (64p + l) % 9 of row (64p + l) / 9, so that the rows lie in LDS one after the other and
    // a row's two or three cache lines are asked for by neighbouring lanes of one instruction.  The nine are shared out
    // 5 : 4 over the pair; the wavefront with 4 brings a quarter of Sx as its fifth copy.
    const uint8_t *wt = w + (size_t)row0 * row_bytes;                                          // uniform
    uint32_t r_off[5];
#pragma unroll
    for (int p = 0; p < 5; p++) {
        const uint32_t idx = min(kh * 5 + p, 8u) * 64 + lane;
        r_off[p] = (min(row0 + wm + idx / 9, rows - 1) - row0) * row_bytes + (idx % 9) * 16;
    }
    const uint32_t own_row = min(row0 + wm + lane, rows - 1);   // the row whose table entries this thread writes
    // activations ([token][hidden] f16): wavefront -> tokens 16w .. 16w+15 (two copies of 8 tokens x 128 bytes)
    const uint8_t *xt = (const uint8_t *)xh;                                                   // uniform
    uint32_t b_off[2];
#pragma unroll
    for (int q = 0; q < 2; q++) {
        const uint32_t r = (wave * 2 + q) * 8 + (lane >> 3);
        b_off[q] = min(tok0 + r, seq - 1) * hidden * 2 + (((lane & 7u) ^ ((r >> 1) & 7u)) * 16);
    }
    // Sx ([super-block][token][8 pairs]): the wavefronts kh = 1 -> tokens 32wq .. 32wq+31 (two 16-byte halves each)
    const uint8_t *st = (const uint8_t *)sx;                                                   // uniform
    const uint32_t m_off = min(tok0 + wq * 32 + (lane >> 1), seq - 1) * 32 + (lane & 1u) * 16;
    const int row_e = rexp[own_row];  // d * 2^row_e <= 1 over the whole row

    const uint32_t row32 = lane & 31u, kgrp = lane >> 5;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(p_lds_vp)glds;

    // (requests past the end are clamped: same number of copies in flight, results unused)
    auto issue_raw = [&](uint32_t sb, int p) {  // piece p (0..4) of this wavefront's share
        const uint8_t *src = wt + (size_t)min(sb, sb_end - 1) * 144;
        copy16_to_lds(src, r_off[p], lds0 + G_R_OFF + ((sb - sb_begin) & 1u) * G_R_STAGE + wq * 9216 + min(kh * 5 + p, 8u) * 1024);
    };
    auto issue_b = [&](uint32_t s, uint32_t slot, int q) {  // one of the two pieces of a step
        const uint32_t sc = min(s, nsteps - 1);
        const uint8_t *src = xt + ((size_t)sb_begin * 4 + sc) * 128;
        copy16_to_lds(src, b_off[q], lds0 + G_B_OFF + slot * G_B_STAGE + wave * 2048 + q * 1024);
    };
    auto issue_sx = [&](uint32_t sb) {  // a quarter of a super-block's Sx
        const uint32_t sbc = min(sb, sb_end - 1);
        copy16_to_lds(st + (size_t)sbc * seq * 32, m_off, lds0 + G_BM_OFF + wq * 1024);
    };
    // a super-block's header -> this row's table entries (one thread per row).  Scales: s = f16(d 2^E sc6) of the
    // sub-blocks 2u + kh, the ones this wavefront converts; the operand is s (q - 8): centred weights, so that the
    // weight term and the offset term are both of the result's size and their f16 roundings are not magnified by a
    // cancellation (with s q and -dmin mn6 Sx the error was 8e-4, so 2.9e-4).  The high nibbles' masked value is
    // 1024 + 16q, so kh = 1 carries s/16.  Offsets' operand of the sub-blocks 4kh .. 4kh+3: 32 (8 d sc6 - dmin mn6) 2^E,
    // twice, for the two f16 halves of Sx/32.
    auto stage_sb = [&](uint32_t par) {
        const u32x4 hdr = *reinterpret_cast<const u32x4 *>(glds + G_R_OFF + par * G_R_STAGE + wq * 9216 + lane * 144);
        const float d = half_to_float(hdr.x & 0xFFFFu), dmin = half_to_float(hdr.x >> 16);
        const float ds = ldexpf(d, row_e), dm = ldexpf(dmin, row_e);
        auto sc6_of = [&](uint32_t sub) {
            const uint32_t sh = 8u * (sub & 3u), pa = (hdr.y >> sh) & 0xFFu, pc = (hdr.w >> sh) & 0xFFu;
            return sub < 4 ? (pa & 63u) : ((pc & 0x0Fu) | ((pa >> 6) << 4));
        };
        auto mn6_of = [&](uint32_t sub) {
            const uint32_t sh = 8u * (sub & 3u), pb = (hdr.z >> sh) & 0xFFu, pc = (hdr.w >> sh) & 0xFFu;
            return sub < 4 ? (pb & 63u) : ((pc >> 4) | ((pb >> 6) << 4));
        };
        uint32_t mnw[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const uint32_t sub = 2 * u + kh;
            const float sf = ds * (float)sc6_of(sub) * (kh ? 0.0625f : 1.f);
            *reinterpret_cast<uint32_t *>(glds + G_SC_OFF + wq * 2048 + sub * 256 + lane * 4) = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)sf);
            const uint32_t ms = 4 * kh + u;
            const uint32_t hb = __builtin_bit_cast(uint16_t, (_Float16)(32.f * (8.f * ds * (float)sc6_of(ms) - dm * (float)mn6_of(ms))));
            mnw[u] = hb | (hb << 16);
        }
        *reinterpret_cast<u32x4 *>(glds + G_AM_OFF + (wm + lane) * 32 + kh * 16) = (u32x4){mnw[0], mnw[1], mnw[2], mnw[3]};
    };
    // 4 raw bytes (nibble kh) -> two dwords of f16(s (q - 8)) as the pairs (k0, k2) and (k1, k3): the nibbles of bytes 0
    // and 2 are masked in place into the mantissas of two f16 (1024 + q, or 1024 + 16q for the high nibbles), those of
    // bytes 1 and 3 after one shift; a packed add takes 1032 (1152) away, which is exact, and a packed multiply applies s:
    // one rounding (-1032 s itself has no f16, so a single FMA cannot do it).  `magic` is 0x64006400 held in a register
    // so that mask-and-or is one instruction.
    uint32_t magic;
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));
    const uint32_t take = kh ? 0xE480E480u : 0xE408E408u;  // -1152 | -1032, twice
    const uint32_t nib_mask = kh ? 0x00F000F0u : 0x000F000Fu;
    auto convert4 = [&](uint32_t raw, uint32_t sp, uint32_t &o0, uint32_t &o1) {
        const f16x2 p = __builtin_bit_cast(f16x2, sp);
        const f16x2 sc2 = {p[0], p[0]}, c2 = __builtin_bit_cast(f16x2, take);
        const f16x2 m02 = __builtin_bit_cast(f16x2, (raw & nib_mask) | magic);
        const f16x2 m13 = __builtin_bit_cast(f16x2, ((raw >> 8) & nib_mask) | magic);
        o0 = __builtin_bit_cast(uint32_t, (m02 + c2) * sc2);
        o1 = __builtin_bit_cast(uint32_t, (m13 + c2) * sc2);
    };
    const uint32_t raw_lane = lds0 + G_R_OFF + wq * 9216 + row32 * 144 + 16 + kgrp * 16;
    auto raw_of = [&](uint32_t par, uint32_t g4, u32x4 (&rq)[2]) {  // step g4 of the super-block in slot `par`
        const uint32_t a = raw_lane + par * G_R_STAGE + g4 * 32;
        asm volatile("ds_read_b128 %0, %1" : "=v"(rq[0]) : "v"(a));
        asm volatile("ds_read_b128 %0, %1 offset:4608" : "=v"(rq[1]) : "v"(a));
    };
    const uint32_t sc_lane = lds0 + G_SC_OFF + wq * 2048 + kh * 256 + row32 * 4;
    auto scales_of = [&](uint32_t g4, uint32_t (&sp)[2]) {  // the entries of sub-block 2 g4 + kh for this lane's two rows
        const uint32_t a = sc_lane + g4 * 512;
        asm volatile("ds_read_b32 %0, %1" : "=v"(sp[0]) : "v"(a));
        asm volatile("ds_read_b32 %0, %1 offset:128" : "=v"(sp[1]) : "v"(a));
    };
    const uint32_t b_lane = lds0 + G_B_OFF + row32 * 128;
    uint32_t b_col[2];  // byte position of this lane's chunk in a token's row, for the two MFMA depths of a step
#pragma unroll
    for (int j = 0; j < 2; j++) b_col[j] = ((kh * 4 + 2 * kgrp + (uint32_t)j) ^ ((row32 >> 1) & 7u)) << 4;

    f32x16 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int jj = 0; jj < 4; jj++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][jj][e] = 0.f;

    uint32_t an[2][2][4];  // the weight operand of the step being prepared / multiplied: [row block][j][dword]
    u32x4 breg[8];         // its activation operands: [j * 4 + token block]

    // ---- X(n): prepare step n (g: its position in super-block sbn): table entries at a super-block's first step, the
    //      activation operands into registers, the weight operand converted, and this wavefront's copy requests:
    //      activations of step n+3 in every X; the next super-block's weights in its X of g = 0 and 1 (the slot's last
    //      reader was X(4 sbn - 1)); Sx of the next super-block in the X of g = 2 (kh = 1).  What is requested in X(n) is
    //      complete when X(n+2) ends, a barrier before the first X that reads it ----
    auto prepare = [&](const int khc, const uint32_t n, const uint32_t sbn, const int g) {
        const uint32_t parn = (sbn - sb_begin) & 1u;
        if (g == 0) {
            stage_sb(parn);
            asm volatile("" ::: "memory");
        }
        uint32_t sp[2];
        u32x4 rq[2];
        scales_of((uint32_t)g, sp);
        raw_of(parn, (uint32_t)g, rq);
        const uint32_t b0 = b_lane + (uint32_t)g * G_B_STAGE + b_col[0], b1 = b_lane + (uint32_t)g * G_B_STAGE + b_col[1];
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(sp[0]), "+v"(sp[1]), "+v"(rq[0]), "+v"(rq[1]));
        // (one activation operand read per piece of the conversion: what LDS returns goes into the register file ahead of the
        // other wavefront's MFMAs when this wavefront is the older of the two, and eight reads in a row hold them up)
#define LARQL_RD(G) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(breg[G]) : "v"((G) < 4 ? b0 : b1), "n"(((G) & 3) * 4096));
#define LARQL_PIECE(G)                                                                                                      \
        LARQL_RD(G)                                                                                                         \
        convert4(rq[(G) >> 2][(G) & 3], sp[(G) >> 2], an[(G) >> 2][((G) >> 1) & 1][2 * ((G) & 1)], an[(G) >> 2][((G) >> 1) & 1][2 * ((G) & 1) + 1]); \
        __builtin_amdgcn_sched_barrier(0);
        LARQL_PIECE(0) LARQL_PIECE(1) LARQL_PIECE(2) LARQL_PIECE(3) LARQL_PIECE(4) LARQL_PIECE(5) LARQL_PIECE(6) LARQL_PIECE(7)
#undef LARQL_PIECE
#undef LARQL_RD
        issue_b(n + 3, (uint32_t)((g + 3) & 3), 0);
        issue_b(n + 3, (uint32_t)((g + 3) & 3), 1);
        if (g == 0) { issue_raw(sbn + 1, 0); issue_raw(sbn + 1, 1); if (!khc) issue_raw(sbn + 1, 2); }
        if (g == 1) { issue_raw(sbn + 1, khc ? 2 : 3); issue_raw(sbn + 1, khc ? 3 : 4); }
        if (g == 2 && khc) issue_sx(sbn + 1);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(breg[0]), "+v"(breg[1]), "+v"(breg[2]), "+v"(breg[3]), "+v"(breg[4]), "+v"(breg[5]), "+v"(breg[6]), "+v"(breg[7]));
        // own requests still in flight: this X's and the one's before
        const int mine[2][4] = {{5, 4, 2, 2}, {4, 4, 3, 2}};
        const int fly = mine[khc][g] + mine[khc][(g + 3) & 3];
        if (fly == 4) GEMM_WAIT_VMCNT(4);
        else if (fly == 5) GEMM_WAIT_VMCNT(5);
        else if (fly == 6) GEMM_WAIT_VMCNT(6);
        else if (fly == 7) GEMM_WAIT_VMCNT(7);
        else if (fly == 8) GEMM_WAIT_VMCNT(8);
        else GEMM_WAIT_VMCNT(9);
        __builtin_amdgcn_s_setprio(3);  // (the multiply phase comes next)
    };
    // ---- M: the sixteen MFMAs of a prepared step, back to back.  At a super-block's second step the wavefront kh = 0
    //      first adds the super-block's offsets, sum_sub (8 d sc6 - dmin mn6) * Sx, one 16-deep MFMA per block (all of
    //      them in one wavefront: a token's sum is then formed in the same order whichever token block it sits in) ----
    auto multiply = [&](const int khc, const int g) {
        if (g == 1 && khc == 0 && with_mins) {
            f16x8 amf[2], bmf[4];
#pragma unroll
            for (int i = 0; i < 2; i++) amf[i] = *reinterpret_cast<const f16x8 *>(glds + G_AM_OFF + (wm + i * 32 + row32) * 32 + kgrp * 16);
#pragma unroll
            for (int jj = 0; jj < 4; jj++) bmf[jj] = *reinterpret_cast<const f16x8 *>(glds + G_BM_OFF + (jj * 32 + row32) * 32 + kgrp * 16);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int jj = 0; jj < 4; jj++) acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(amf[i], bmf[jj], acc[i][jj], 0, 0, 0);
        }
        f16x8 af[2][2];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) af[i][j] = __builtin_bit_cast(f16x8, (u32x4){an[i][j][0], an[i][j][1], an[i][j][2], an[i][j][3]});
#pragma unroll
        for (int G = 0; G < 8; G++)
#pragma unroll
            for (int i = 0; i < 2; i++)
                acc[i][G & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i][G >> 2], __builtin_bit_cast(f16x8, breg[G]), acc[i][G & 3], 0, 0, 0);
        __builtin_amdgcn_s_setprio(0);
    };

    // ---- prologue: the first super-block's weights, the first Sx, activation steps 0..2 ----
    if (kh) issue_sx(sb_begin);
#pragma unroll
    for (int p = 0; p < 5; p++)
        if (p < 4 || !kh) issue_raw(sb_begin, p);
#pragma unroll
    for (int q = 0; q < 2; q++) { issue_b(0, 0, q); issue_b(1, 1, q); issue_b(2, 2, q); }
    GEMM_WAIT_VMCNT(0);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // The two wavefronts of a SIMD take turns: while one multiplies a step, the other prepares its next one.
    //   kh = 0:  X(0) | M(0)   X(1) | M(1)   X(2) | ...
    //   kh = 1:       | X(0)   M(0) | X(1)   M(1) | ...          (| = barrier)
    // (each wavefront runs its own copy of the loop: no merge of the two orders inside it; both pass the same barriers)
    // (nothing moves across a change of phase: not memory accesses, and not the MFMAs either, which the scheduler would
    // otherwise spread over the other phase)
    auto phase_end = [&]() {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::: "memory");
    };
    auto run = [&](auto KH) {
        constexpr int khc = decltype(KH)::value;
        if (khc == 0) prepare(0, 0, sb_begin, 0);
        phase_end();
        uint32_t s = 0;
        for (uint32_t sb = sb_begin; sb < sb_end; sb++) {
#pragma unroll
            for (int g = 0; g < 4; g++, s++) {
                if (khc == 0) multiply(0, g);
                else prepare(1, s, sb, g);
                phase_end();
                if (khc == 0) {
                    if (s + 1 < nsteps) prepare(0, s + 1, g == 3 ? sb + 1 : sb, (g + 1) & 3);
                } else {
                    multiply(1, g);
                }
                phase_end();
            }
        }
    };
    if (!kh) run(std::integral_constant<int, 0>{});
    else run(std::integral_constant<int, 1>{});
    GEMM_WAIT_VMCNT(0);  // the clamped requests past the end

    // The pair adds its partial sums through LDS, where the results also take the shape in which a store instruction
    // writes whole lines: a row group's 64-row x 128-token block as [token][row] (token rows padded to 68 floats: the
    // lanes of a write phase hit different banks) in the pair's own 34 KB; wavefront 1 parks, wavefront 0 adds its own
    // and parks the sum, then every lane of the pair stores 16 bytes of a 256-byte run of one token.
    __builtin_amdgcn_s_barrier();  // nobody's copies are still landing in what becomes somebody's block
    asm volatile("" ::: "memory");
    constexpr uint32_t EP_LD = G_EP_LD;
    float *blk = reinterpret_cast<float *>(glds) + wq * (GN * EP_LD);
    if (kh) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
#pragma unroll
                for (int q = 0; q < 4; q++)  // registers 4q .. 4q+3 of a block: rows 8q + 4kgrp .. +3, token row32
                    *reinterpret_cast<f32x4 *>(blk + (jj * 32 + row32) * EP_LD + i * 32 + q * 8 + kgrp * 4) =
                        (f32x4){acc[i][jj][4 * q], acc[i][jj][4 * q + 1], acc[i][jj][4 * q + 2], acc[i][jj][4 * q + 3]};
    }
    __syncthreads();
    if (!kh) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    f32x4 *at = reinterpret_cast<f32x4 *>(blk + (jj * 32 + row32) * EP_LD + i * 32 + q * 8 + kgrp * 4);
                    const f32x4 other = *at;
                    *at = (f32x4){acc[i][jj][4 * q] + other[0], acc[i][jj][4 * q + 1] + other[1], acc[i][jj][4 * q + 2] + other[2], acc[i][jj][4 * q + 3] + other[3]};
                }
    }
    __syncthreads();
    const bool vec_ok = (rows & 3u) == 0 && (((uintptr_t)(partial ? partial : out)) & 15u) == 0;
    const uint32_t rc = (lane & 15u) * 4, r = row0 + wm + rc;
    float back[4];  // 2^-E of this lane's four rows
#pragma unroll
    for (int e = 0; e < 4; e++) back[e] = ldexpf(1.f, -rexp[min(r + e, rows - 1)]);
#pragma unroll 4
    for (int it = 0; it < 16; it++) {
        const uint32_t tl = (kh * 16 + it) * 4 + (lane >> 4), tok = tok0 + tl;
        if (tok >= seq) continue;
        f32x4 v = *reinterpret_cast<const f32x4 *>(blk + tl * EP_LD + rc);
        float *o = partial ? partial + ((size_t)blockIdx.z * seq + tok) * rows + r : out + (size_t)tok * rows + r;
        // (partial sums stay without the token's scale; q4k_gemm_reduce_kernel adds the slabs in order and applies it)
        const float ts = partial ? 1.f : tok_scale[tok];
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] *= ts * back[e];
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

// activations -> f16 terms, sub-block sums and token scales; with `rexp`, the weight rows' exponents as well
hipError_t q4k_gemm_prep_launch(hipStream_t s, const void *x, int x_is_bf16, uint32_t hidden, uint32_t seq, uint16_t *xh, uint16_t *xl,
                                uint16_t *sx, float *tok_scale, int *any_lo, const uint8_t *w, uint32_t rows, int *rexp) {
    if (seq == 0 && !(rexp && rows)) return hipSuccess;  // (no tokens: only the rows' exponents, if they are asked for)
    // a token per block; wide activations take more threads per token (two passes over the token: 256 threads on 15360
    // elements are 15 dependent rounds of loads)
    const uint32_t threads = hidden >= 8192 ? 1024u : 256u;
    const uint32_t row_blocks = rexp ? (rows + threads / 16 - 1) / (threads / 16) : 0;
    hipLaunchKernelGGL(q4k_gemm_prep_kernel, dim3(seq + row_blocks), dim3(threads), 0, s, x, x_is_bf16, hidden, xh, xl, sx, tok_scale, any_lo,
                       1, seq, w, rows, rexp);
    return hipGetLastError();
}


// K-ranges per output tile so that a launch fills the CUs (1 = no split)
uint32_t q4k_gemm_splits(uint32_t rows, uint32_t hidden, uint32_t seq, uint32_t cu_count) {
    const uint32_t nsb = hidden / 256;
    uint32_t s = 1;
    // one 256x128 workgroup per CU
    const uint64_t tiles = (uint64_t)((rows + GM - 1) / GM) * ((seq + GN - 1) / GN);
    while (s < 8 && tiles * s * 2 <= (uint64_t)cu_count && nsb / (s * 2) >= 4) s *= 2;
    return s;
}

// `rexp` (from q4k_gemm_prep_launch): the rows' scales ride in the f16 weight operand; without it the weight operand is
// the exact integer and the rows' f32 scales are applied per super-block
hipError_t q4k_gemm_f16_launch(hipStream_t s, const uint8_t *w, const uint16_t *xh, const uint16_t *sx, const int *rexp, const float *tok_scale,
                               float *out, uint32_t rows, uint32_t hidden, uint32_t seq, int with_mins, int accumulate, uint32_t splits,
                               float *partial) {
    if (rows == 0 || seq == 0) return hipSuccess;
    const uint32_t nsb = hidden / 256;
    const bool split = splits > 1 && partial;
    const uint32_t per = split ? (nsb + splits - 1) / splits : nsb, z = split ? (nsb + per - 1) / per : 1;
    static std::atomic<bool> attr_set{false};  // dynamic LDS above 64 KB has to be allowed once per process
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void *)q4k_gemm_exact_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e == hipSuccess) e = hipFuncSetAttribute((const void *)q4k_gemm_pair_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const dim3 grid((rows + GM - 1) / GM, (seq + GN - 1) / GN, z);
    float *slab = split ? partial : (float *)nullptr;
    if (rexp)
        hipLaunchKernelGGL(q4k_gemm_pair_kernel, grid, dim3(QTHREADS), G_LDS_BYTES, s, w, xh, sx, rexp, tok_scale, out, rows, hidden, seq,
                           with_mins, accumulate, per, slab);
    else
        hipLaunchKernelGGL(q4k_gemm_exact_kernel, grid, dim3(GTHREADS), G_LDS_BYTES, s, w, xh, sx, tok_scale, out, rows, hidden, seq, with_mins,
                           accumulate, per, slab);
    if (split) {
        const size_t n = (size_t)rows * seq;
        if (rows % 4 == 0 && (((uintptr_t)partial | (uintptr_t)out) & 15u) == 0)
            hipLaunchKernelGGL(q4k_gemm_reduce_kernel<4>, dim3((uint32_t)((n / 4 + 255) / 256)), dim3(256), 0, s, partial, z, tok_scale, out, rows, seq, accumulate);
        else
            hipLaunchKernelGGL(q4k_gemm_reduce_kernel<1>, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, s, partial, z, tok_scale, out, rows, seq, accumulate);
    }
    return hipGetLastError();
}

}  // namespace larql
