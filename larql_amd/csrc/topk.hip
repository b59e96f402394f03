// topk.hip — top-K selection over rows of a score matrix on gfx950.
//
// Two orderings, both restating the reference's selectors:
//   by |score|  — top_k_by_abs, larql-vindex/src/index/compute/gate_knn/mod.rs:50-108
//                 (NaN is an error there: it panics)
//   by value    — top_k_sorted, larql-vindex/src/index/storage/lm_head/knn.rs:315-386
//                 (non-finite scores are skipped)
// Output is sorted best-first.  Where the reference leaves the order of equal
// keys to its heap and an unstable sort, this kernel fixes it: the lower index
// wins.
//
// Each score becomes a 64-bit key (ordered score bits, then ~index), so one
// unsigned compare decides everything and index recovery needs no side array.
// One workgroup serves one row: every wavefront keeps a sorted top-64 in
// registers (one key per lane), folds 64-score chunks into it with a bitonic
// sort + bitonic merge done by cross-lane shuffles, skipping chunks that cannot
// beat the current 64th key; the wavefronts' lists are then merged by the first
// wavefront through LDS.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

namespace larql {

constexpr int kTopkThreads = 1024;
constexpr int kTopkWaves = kTopkThreads / 64;

__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int mask) {
    uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
    lo = (uint32_t)__shfl_xor((int)lo, mask, 64);
    hi = (uint32_t)__shfl_xor((int)hi, mask, 64);
    return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ uint64_t shfl_u64(uint64_t v, int src) {
    uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
    lo = (uint32_t)__shfl((int)lo, src, 64);
    hi = (uint32_t)__shfl((int)hi, src, 64);
    return ((uint64_t)hi << 32) | lo;
}

// bitonic merge of a bitonic 64-sequence into descending order
__device__ __forceinline__ uint64_t merge_desc(uint64_t key, uint32_t lane) {
#pragma unroll
    for (int j = 32; j > 0; j >>= 1) {
        const uint64_t other = shfl_xor_u64(key, j);
        const bool lower = (lane & j) == 0;
        key = lower ? (key > other ? key : other) : (key < other ? key : other);
    }
    return key;
}

// full bitonic sort of 64 keys, descending by lane
__device__ __forceinline__ uint64_t sort_desc(uint64_t key, uint32_t lane) {
#pragma unroll
    for (int size = 2; size <= 64; size <<= 1) {
        const bool desc_block = (size == 64) || ((lane & size) == 0);
#pragma unroll
        for (int j = size >> 1; j > 0; j >>= 1) {
            const uint64_t other = shfl_xor_u64(key, j);
            const bool lower = (lane & j) == 0;
            const bool take_max = (lower == desc_block);
            key = take_max ? (key > other ? key : other) : (key < other ? key : other);
        }
    }
    return key;
}

// fold a sorted-descending list `in` into the sorted-descending `top`
__device__ __forceinline__ uint64_t fold_sorted(uint64_t top, uint64_t in_desc, uint32_t lane) {
    const uint64_t rev = shfl_u64(in_desc, 63 - (int)lane);
    const uint64_t m = top > rev ? top : rev;  // the 64 largest of the union, bitonic
    return merge_desc(m, lane);
}

template <bool BY_ABS>
__device__ __forceinline__ uint64_t make_key(float s, uint32_t idx, int *nan_flag) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, s);
    uint32_t ord;
    if (BY_ABS) {
        ord = bits & 0x7FFFFFFFu;
        if (ord > 0x7F800000u) { atomicOr(nan_flag, 1); ord = 0; }
        ord += 1;  // keep every real score above the padding key 0
    } else {
        if ((bits & 0x7F800000u) == 0x7F800000u) return 0;  // inf / NaN are skipped
        ord = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    }
    return ((uint64_t)ord << 32) | (uint32_t)(~idx);
}

template <bool BY_ABS>
__global__ void __launch_bounds__(kTopkThreads) topk_kernel(const float *__restrict__ scores, uint32_t n, uint32_t k,
                                                            uint32_t *__restrict__ idx_out, float *__restrict__ val_out,
                                                            uint32_t *__restrict__ count_out, int *nan_flag) {
    __shared__ uint64_t lists[kTopkWaves][64];
    const uint32_t row = blockIdx.x;
    const float *s = scores + (size_t)row * n;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint64_t top = 0;
    // wave w takes chunks w, w+16, ... of 64 consecutive scores
    for (uint32_t base = wave * 64; base < n; base += kTopkThreads) {
        const uint32_t i = base + lane;
        uint64_t key = i < n ? make_key<BY_ABS>(s[i], i, nan_flag) : 0;
        const uint64_t thr = shfl_u64(top, 63);
        if (__ballot(key > thr) == 0) continue;
        key = sort_desc(key, lane);
        top = fold_sorted(top, key, lane);
    }
    lists[wave][lane] = top;
    __syncthreads();
    if (wave == 0) {
        for (int w = 1; w < kTopkWaves; w++) {
            const uint64_t in = lists[w][lane];
            const uint64_t thr = shfl_u64(top, 63);
            if (__ballot(in > thr) == 0) continue;
            top = fold_sorted(top, in, lane);
        }
        const bool valid = top != 0 && lane < k;
        if (valid) {
            const uint32_t idx = ~(uint32_t)top;
            idx_out[(size_t)row * k + lane] = idx;
            val_out[(size_t)row * k + lane] = s[idx];
        }
        const uint64_t mask = __ballot(valid);
        if (lane == 0) count_out[row] = (uint32_t)__popcll(mask);
    }
}

size_t topk_workspace_bytes(uint32_t, uint32_t, uint32_t) { return 0; }

hipError_t topk_launch(hipStream_t stream, const float *scores, uint32_t batch, uint32_t n, uint32_t k, bool by_abs,
                       uint32_t *idx_out, float *val_out, uint32_t *count_out, int *nan_flag, void *, size_t) {
    if (batch == 0) return hipSuccess;
    if (by_abs)
        hipLaunchKernelGGL(topk_kernel<true>, dim3(batch), dim3(kTopkThreads), 0, stream, scores, n, k, idx_out, val_out,
                           count_out, nan_flag);
    else
        hipLaunchKernelGGL(topk_kernel<false>, dim3(batch), dim3(kTopkThreads), 0, stream, scores, n, k, idx_out, val_out,
                           count_out, nan_flag);
    return hipGetLastError();
}

}  // namespace larql
