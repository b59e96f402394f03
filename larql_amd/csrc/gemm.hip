// gemm.hip — batched-prefill Q4_K GEMM on the gfx950 matrix cores.
//
//   out[s, r] = sum_k W[r, k] * X[s, k]      W: [rows, hidden] Q4_K,  X: [seq, hidden] bf16
//
// the contraction q4k_matmul_into computes (larql-compute/src/cpu/ops/q4_common/
// matmul.rs:20-139; `out` is [seq, rows] row-major).  A workgroup owns a
// 128-row x 128-token tile of `out` and walks K in steps of 64 (one nibble
// group = two 32-element sub-blocks).  Per step it decodes its 128x64 weights
// exactly as decode_q4k_superblock_into does (w = sc*q - mn in f32,
// matvec_f32.rs:166-199), splits each into two bf16 terms hi + lo (so the
// bf16 operand carries 16 significant bits and the product is good to ~2^-17,
// not the 2^-9 of a single bf16 rounding), stages them and the activation tile
// in LDS, and feeds v_mfma_f32_16x16x32_bf16 with fp32 accumulators (two MFMAs
// per tile: hi and lo).  LDS rows are padded to 72 elements so the 16 lanes of
// an operand read hit 16 distinct 16-byte slots.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

namespace larql {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int TM = 128, TN = 128, KS = 64, LDK = 72;  // tile rows, tile tokens, k per step, padded LDS row (bf16 elements)

__device__ __forceinline__ uint32_t bf16_rne_bits(float f) {
    const uint32_t b = __builtin_bit_cast(uint32_t, f);
    return (b + 0x7FFFu + ((b >> 16) & 1u)) >> 16;  // finite inputs only (weights and activations)
}

__device__ __forceinline__ float half_to_float(uint32_t lo16) { return (float)__builtin_bit_cast(_Float16, (uint16_t)lo16); }

__global__ void __launch_bounds__(256) q4k_gemm_kernel(const uint8_t *__restrict__ w, const uint16_t *__restrict__ x,
                                                       float *__restrict__ out, uint32_t rows, uint32_t hidden, uint32_t seq,
                                                       int accumulate) {
    __shared__ __attribute__((aligned(16))) uint16_t a_hi[TM * LDK];
    __shared__ __attribute__((aligned(16))) uint16_t a_lo[TM * LDK];
    __shared__ __attribute__((aligned(16))) uint16_t b_t[TN * LDK];
    const uint32_t t = threadIdx.x, lane = t & 63u, wave = t >> 6;
    const uint32_t row0 = blockIdx.x * TM, tok0 = blockIdx.y * TN;
    const uint32_t nsb = hidden >> 8;
    const size_t row_bytes = (size_t)nsb * 144;

    // staging role: thread -> (tile row / token, half of the 64-wide k step)
    const uint32_t sr = t >> 1, half = t & 1u;
    const uint32_t wrow = min(row0 + sr, rows - 1), xtok = min(tok0 + sr, seq - 1);
    const uint8_t *wp = w + (size_t)wrow * row_bytes;
    const uint16_t *xp = x + (size_t)xtok * hidden + half * 32;

    // compute role: wave -> 64x64 quadrant, lane -> (row / token within a 16-wide tile, k octet)
    const uint32_t wm = (wave >> 1) * 64, wn = (wave & 1u) * 64;
    const uint32_t l16 = lane & 15u, kq = (lane >> 4) * 8;

    f32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

    for (uint32_t ks = 0; ks < hidden; ks += KS) {
        const uint32_t sb = ks >> 8, g = (ks >> 6) & 3u;
        // ---- decode 32 weights of (row sr, sub-block 2g+half) ----
        const u32x4 *blk = reinterpret_cast<const u32x4 *>(wp + (size_t)sb * 144);
        const u32x4 hdr = blk[0], q0 = blk[1 + 2 * g], q1 = blk[2 + 2 * g];
        const float d = half_to_float(hdr.x & 0xFFFFu), dmin = half_to_float(hdr.x >> 16);
        const uint32_t s = 2 * g + half;  // sub-block index 0..7 (get_scale_min_k4)
        const uint32_t sh = 8u * (s & 3u);
        const uint32_t pa = (hdr.y >> sh) & 0xFFu, pb = (hdr.z >> sh) & 0xFFu, pc = (hdr.w >> sh) & 0xFFu;
        const uint32_t sc6 = s < 4 ? (pa & 63u) : ((pc & 0x0Fu) | ((pa >> 6) << 4));
        const uint32_t mn6 = s < 4 ? (pb & 63u) : ((pc >> 4) | ((pb >> 6) << 4));
        const float sc = d * (float)sc6, mn = dmin * (float)mn6;
        const uint32_t qd[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        uint32_t hi_w[16], lo_w[16];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t v = half ? (qd[i] >> 4) : qd[i];
            uint32_t hb[4], lb[4];
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const float wf = sc * (float)((v >> (8 * b)) & 0x0Fu) - mn;
                hb[b] = bf16_rne_bits(wf);
                lb[b] = bf16_rne_bits(wf - __builtin_bit_cast(float, hb[b] << 16));
            }
            hi_w[2 * i] = hb[0] | (hb[1] << 16); hi_w[2 * i + 1] = hb[2] | (hb[3] << 16);
            lo_w[2 * i] = lb[0] | (lb[1] << 16); lo_w[2 * i + 1] = lb[2] | (lb[3] << 16);
        }
        // ---- activation tile: 32 bf16 of token sr ----
        const u32x4 *xv = reinterpret_cast<const u32x4 *>(xp + ks);
        const u32x4 x0 = xv[0], x1 = xv[1], x2 = xv[2], x3 = xv[3];

        __syncthreads();  // previous step's MFMA reads are done
        {
            u32x4 *ah = reinterpret_cast<u32x4 *>(&a_hi[sr * LDK + half * 32]);
            u32x4 *al = reinterpret_cast<u32x4 *>(&a_lo[sr * LDK + half * 32]);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                ah[i] = (u32x4){hi_w[4 * i], hi_w[4 * i + 1], hi_w[4 * i + 2], hi_w[4 * i + 3]};
                al[i] = (u32x4){lo_w[4 * i], lo_w[4 * i + 1], lo_w[4 * i + 2], lo_w[4 * i + 3]};
            }
            u32x4 *bt = reinterpret_cast<u32x4 *>(&b_t[sr * LDK + half * 32]);
            bt[0] = x0; bt[1] = x1; bt[2] = x2; bt[3] = x3;
        }
        __syncthreads();

        // ---- 64x64 quadrant: 2 k-slices x 16 tiles x (hi, lo) ----
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            bf16x8 ah[4], al[4], bb[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t off = (wm + i * 16 + l16) * LDK + kk * 32 + kq;
                ah[i] = *reinterpret_cast<const bf16x8 *>(&a_hi[off]);
                al[i] = *reinterpret_cast<const bf16x8 *>(&a_lo[off]);
                bb[i] = *reinterpret_cast<const bf16x8 *>(&b_t[(wn + i * 16 + l16) * LDK + kk * 32 + kq]);
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[i], bb[j], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al[i], bb[j], acc[i][j], 0, 0, 0);
                }
        }
    }

    // ---- store: lane holds rows 4*(lane/16)..+3 of column (token) lane%16 of each 16x16 tile ----
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t tok = tok0 + wn + j * 16 + l16;
            const uint32_t r = row0 + wm + i * 16 + (lane >> 4) * 4;
            if (tok >= seq) continue;
            float *o = out + (size_t)tok * rows + r;
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (r + e < rows) o[e] = accumulate ? o[e] + acc[i][j][e] : acc[i][j][e];
        }
}

// f32 activations -> bf16 hi (round to nearest even) and the bf16 of the remainder
__global__ void split_bf16_kernel(const float *__restrict__ x, size_t n, uint16_t *__restrict__ hi, uint16_t *__restrict__ lo,
                                  int *__restrict__ any_lo) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = x[i];
    const uint32_t h = bf16_rne_bits(v);
    const uint32_t l = bf16_rne_bits(v - __builtin_bit_cast(float, h << 16));
    hi[i] = (uint16_t)h;
    lo[i] = (uint16_t)l;
    if ((l & 0x7FFFu) != 0) *any_lo = 1;
}

hipError_t q4k_gemm_launch(hipStream_t s, const uint8_t *w, const uint16_t *x_bf16, float *out, uint32_t rows, uint32_t hidden,
                           uint32_t seq, int accumulate) {
    if (rows == 0 || seq == 0) return hipSuccess;
    hipLaunchKernelGGL(q4k_gemm_kernel, dim3((rows + TM - 1) / TM, (seq + TN - 1) / TN), dim3(256), 0, s, w, x_bf16, out, rows, hidden,
                       seq, accumulate);
    return hipGetLastError();
}

hipError_t split_bf16_launch(hipStream_t s, const float *x, size_t n, uint16_t *hi, uint16_t *lo, int *any_lo) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(split_bf16_kernel, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, s, x, n, hi, lo, any_lo);
    return hipGetLastError();
}

}  // namespace larql
