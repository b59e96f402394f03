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
// One workgroup serves one row, each thread a contiguous run of indices.
// The K-th largest ordered-score value T is found exactly by a 4-pass radix
// select (8 bits per pass, a 256-bin histogram in LDS per pass, one wavefront
// scanning the bins from the top); scores above T are taken, and of the scores
// equal to T the lowest indices fill the remaining places (ranked by a prefix
// count in index order).  The <= 64 winners are gathered in LDS and one
// wavefront orders them best-first with a bitonic sort done by cross-lane
// shuffles.  Cost is a handful of passes over the row, whatever its order.
// Rows of up to 16384 scores (every gate matrix) are read once: a thread keeps
// its up to 16 ordered scores in registers, and a bound with at least 64 scores
// at or above it (the smallest maximum of 64 slices of the row) usually leaves
// a few hundred candidates, which are ranked directly; the radix passes remain
// for rows with more than 1024 candidates and for longer rows (a vocabulary),
// which are streamed.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

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

template <bool BY_ABS>
__device__ __forceinline__ uint64_t make_key(float s, uint32_t idx, int *nan_flag) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, s);
    uint32_t ord;
    if (BY_ABS) {
        ord = bits & 0x7FFFFFFFu;
        if (ord > 0x7F800000u) { if (nan_flag) atomicOr(nan_flag, 1); ord = 0; }
        ord += 1;  // keep every real score above the padding key 0
    } else {
        if ((bits & 0x7F800000u) == 0x7F800000u) return 0;  // inf / NaN are skipped
        ord = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    }
    return ((uint64_t)ord << 32) | (uint32_t)(~idx);
}

constexpr int kTopkCached = 16;  // rounds of 64 scores per wavefront held in registers
constexpr int kTopkCandidates = kTopkThreads;  // candidates of the short way: one per thread

// LARGE (K above 64, up to kTopkMaxK): the selection is the same radix select; the winners are gathered into a
// power-of-two array in dynamic LDS (`cap` keys, zero-padded) and ordered by a bitonic sort of the whole workgroup.
// (80 scalar registers: with the 96 the compiler would take, a second 16-wavefront workgroup was not placed on a CU
// until half of the first one's wavefronts had left — more rows than CUs then ran in two rounds)
template <bool BY_ABS, bool CACHED, bool LARGE>
__global__ void __launch_bounds__(kTopkThreads) __attribute__((amdgpu_num_sgpr(80))) topk_kernel(const float *__restrict__ scores, uint32_t n, uint32_t k,
                                                            uint32_t *__restrict__ idx_out, float *__restrict__ val_out,
                                                            uint32_t *__restrict__ count_out, int *nan_flag, uint32_t cap) {
    static_assert(!(LARGE && CACHED), "the candidate short cut bounds 64 winners only");
    extern __shared__ __attribute__((aligned(16))) uint64_t big[];  // LARGE: cap keys
    __shared__ uint32_t hist[256];
    __shared__ uint32_t wave_ties[kTopkWaves];
    __shared__ uint64_t winners[64];
    __shared__ uint32_t sh_prefix, sh_need, sh_nwin, sh_ncand;
    __shared__ uint32_t group_max[64];
    __shared__ __attribute__((aligned(16))) uint64_t cand[CACHED ? kTopkCandidates + 4 : 1];
    __shared__ uint32_t rank_sh[CACHED ? kTopkCandidates : 1];  // ranks counted in shares (short way)
    const uint32_t row = blockIdx.x, tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const float *s = scores + (size_t)row * n;
    // wavefront w owns the contiguous indices [w0, w1), 64 at a time (lane = index within the 64)
    const uint32_t perw = ((n + kTopkWaves * 64 - 1) / (kTopkWaves * 64)) * 64;
    const uint32_t w0 = min(n, wave * perw), w1 = min(n, w0 + perw);

    // the ordered score of index i (0: nothing there), from the register copy or from memory
    uint32_t cache[CACHED ? kTopkCached : 1];
    if (CACHED) {
        // every load leaves before the first score is looked at (a load inside a condition is waited for where it
        // stands: sixteen round trips instead of one); an index past the wavefront's range reads the row's last score
        float raw[kTopkCached];
#pragma unroll
        for (int it = 0; it < kTopkCached; it++) raw[it] = s[min(w0 + it * 64 + lane, n - 1)];
#pragma unroll
        for (int it = 0; it < kTopkCached; it++) {
            const uint32_t i = w0 + it * 64 + lane;
            cache[it] = i < w1 ? (uint32_t)(make_key<BY_ABS>(raw[it], i, nan_flag) >> 32) : 0u;
        }
    }
    // f(ord, i) for every index of this wavefront, 64 at a time, all lanes taking part in every round
    auto for_each = [&](auto &&f, int *flag) {
        if (CACHED) {
#pragma unroll
            for (int it = 0; it < kTopkCached; it++) f(cache[it], w0 + it * 64 + lane);
        } else {
            for (uint32_t base = w0; base < w1; base += 64) {
                const uint32_t i = base + lane;
                f(i < w1 ? (uint32_t)(make_key<BY_ABS>(s[i], i, flag) >> 32) : 0u, i);
            }
        }
    };

    if (tid < 64) winners[tid] = 0;
    if (LARGE)
        for (uint32_t i = tid; i < cap; i += kTopkThreads) big[i] = 0;
    if (tid == 0) { sh_prefix = 0; sh_need = k; sh_nwin = 0; sh_ncand = 0; }
    if (CACHED) {
        // ---- short way for a row held in registers.  The 64 groups of 16 lanes each own a slice of the row; the
        //      smallest of the 64 group maxima, L, has at least 64 scores at or above it (one per group), so the
        //      winners are among the scores >= L: a few hundred of a typical row.  Those are collected and each one
        //      counts the candidates with a larger key: that count is its place in the output.  A row whose
        //      candidates do not fit (sorted input, a group without valid scores) takes the radix passes below. ----
        uint32_t gmax = 0;
#pragma unroll
        for (int it = 0; it < kTopkCached; it++) gmax = max(gmax, cache[it]);
        // (reductions by DPP row operations: a few cycles each, where a cross-lane shuffle costs an LDS round trip)
        gmax = max(gmax, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)gmax, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
        gmax = max(gmax, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)gmax, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
        gmax = max(gmax, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)gmax, 0x141, 0xF, 0xF, true));  // row_half_mirror
        gmax = max(gmax, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)gmax, 0x140, 0xF, 0xF, true));  // row_mirror
        if ((lane & 15u) == 0) group_max[wave * 4 + (lane >> 4)] = gmax;
        __syncthreads();
        uint32_t L = group_max[lane];
        L = min(L, (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)L, 0xB1, 0xF, 0xF, false));
        L = min(L, (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)L, 0x4E, 0xF, 0xF, false));
        L = min(L, (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)L, 0x141, 0xF, 0xF, false));
        L = min(L, (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)L, 0x140, 0xF, 0xF, false));
        L = min(L, (uint32_t)__builtin_amdgcn_update_dpp((int)L, (int)L, 0x142, 0xA, 0xF, false));     // row_bcast:15 into rows 1 and 3
        L = min(L, (uint32_t)__builtin_amdgcn_update_dpp((int)L, (int)L, 0x143, 0xC, 0xF, false));     // row_bcast:31 into rows 2 and 3
        L = (uint32_t)__builtin_amdgcn_readlane((int)L, 63);
        if (L != 0) {
            // a wavefront reserves room for all its candidates at once, then places them round by round
            uint32_t mine = 0;
#pragma unroll
            for (int it = 0; it < kTopkCached; it++) mine += (uint32_t)__popcll(__ballot(cache[it] >= L));
            uint32_t base = 0;
            if (lane == 0 && mine) base = atomicAdd(&sh_ncand, mine);
            base = (uint32_t)__builtin_amdgcn_readfirstlane((int)base);
#pragma unroll
            for (int it = 0; it < kTopkCached; it++) {
                const bool c = cache[it] >= L;
                const uint64_t m = __ballot(c);
                const uint32_t pos = base + (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
                if (c && pos < (uint32_t)kTopkCandidates) cand[pos] = ((uint64_t)cache[it] << 32) | (uint32_t)(~(w0 + it * 64 + lane));
                base += (uint32_t)__popcll(m);
            }
            __syncthreads();
            const uint32_t nc = sh_ncand;
            if (nc <= (uint32_t)kTopkCandidates) {  // (uniform over the workgroup)
                // (the list is read four keys at a time: zero keys, below every real one, fill it up to a multiple of four)
                if (tid < 4) cand[nc + tid] = 0;
                // A candidate's rank = the candidates above it.  The threads beyond the list take part: with the list
                // rounded up to a power of two, thread t counts for candidate t % that over the t / that -th share of
                // the list, and the shares meet in an LDS counter (half as long for the usual 300-500 candidates).
                uint32_t ncr = 64;
                while (ncr < nc) ncr <<= 1;
                const uint32_t parts = (uint32_t)kTopkThreads / ncr, ci = tid & (ncr - 1u), part = tid / ncr;
                if (parts > 1 && tid < nc) rank_sh[tid] = 0;
                __syncthreads();
                uint64_t key = 0;
                uint32_t rank = 0;
                if (ci < nc) {
                    key = cand[ci];
                    typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
                    const u64x2 *c2 = reinterpret_cast<const u64x2 *>(cand);
                    const uint32_t quads = (nc + 3) / 4, per = (quads + parts - 1) / parts;
                    const uint32_t j0 = part * per, j1 = min(quads, j0 + per);
#pragma unroll 2
                    for (uint32_t j = j0; j < j1; j++) {
                        const u64x2 a = c2[2 * j], b = c2[2 * j + 1];
                        rank += (a.x > key ? 1u : 0u) + (a.y > key ? 1u : 0u) + (b.x > key ? 1u : 0u) + (b.y > key ? 1u : 0u);
                    }
                    if (parts > 1 && rank != 0) atomicAdd(&rank_sh[ci], rank);
                }
                if (parts > 1) {
                    __syncthreads();
                    if (tid < nc) rank = rank_sh[tid];
                }
                if (tid < nc && rank < k) {  // (tid < nc: ci == tid, the key is this thread's candidate)
                    const uint32_t idx = ~(uint32_t)key;
                    idx_out[(size_t)row * k + rank] = idx;
                    val_out[(size_t)row * k + rank] = s[idx];
                }
                if (tid == 0) count_out[row] = min(k, nc);
                return;
            }
        }
        __syncthreads();
    }
    // ---- radix select of the k-th largest ordered score: 8 bits per pass, top byte first ----
    for (int pass = 0; pass < 4; pass++) {
        const int sh = 24 - 8 * pass;
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        const uint32_t prefix = sh_prefix;
        for_each([&](uint32_t ord, uint32_t) {
            // 64-bit shift: the first pass compares nothing (shift by 32)
            if (ord != 0 && ((uint64_t)ord >> (sh + 8)) == ((uint64_t)prefix >> (sh + 8))) atomicAdd(&hist[(ord >> sh) & 255u], 1u);
        }, pass == 0 ? nan_flag : nullptr);
        __syncthreads();
        if (wave == 0) {
            // lane l holds bins 255-4l .. 252-4l (descending); find the bin where the running count reaches `need`
            const uint32_t need = sh_need;
            const uint32_t b0 = 255u - 4u * lane;
            const uint32_t c0 = hist[b0], c1 = hist[b0 - 1], c2 = hist[b0 - 2], c3 = hist[b0 - 3];
            const uint32_t mine = c0 + c1 + c2 + c3;
            uint32_t incl = mine;  // inclusive scan over lanes (bins in descending order)
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const uint32_t t = (uint32_t)__shfl_up((int)incl, o, 64);
                if (lane >= (uint32_t)o) incl += t;
            }
            const uint32_t before = incl - mine;
            const bool here = before < need && incl >= need;
            if (here) {
                uint32_t acc = before, bin = b0, above = before;
                const uint32_t c[4] = {c0, c1, c2, c3};
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    if (acc < need && acc + c[q] >= need) { bin = b0 - q; above = acc; }
                    acc += c[q];
                }
                sh_prefix = prefix | (bin << sh);
                sh_need = need - above;  // still to find inside the chosen bin
            }
            // fewer than `need` valid scores in total: nobody is `here`; prefix stays and everything valid is taken
            const uint32_t total = (uint32_t)__shfl((int)incl, 63, 64);
            if (lane == 0 && total < need) { sh_need = 0xFFFFFFFFu; }
        }
        __syncthreads();
        if (sh_need == 0xFFFFFFFFu) break;
    }
    const bool take_all = sh_need == 0xFFFFFFFFu;
    const uint32_t T = take_all ? 0u : sh_prefix;     // scores with ord > T are in
    const uint32_t r = take_all ? 0xFFFFFFFFu : sh_need;  // this many of the scores with ord == T, lowest indices first
    // ---- rank the ties in index order: per-wavefront counts, then ballots inside the wavefront ----
    uint32_t my_ties = 0;
    if (!take_all)
        for_each([&](uint32_t ord, uint32_t) { my_ties += (uint32_t)__popcll(__ballot(ord != 0 && ord == T)); }, nullptr);
    if (lane == 0) wave_ties[wave] = my_ties;
    __syncthreads();
    uint32_t tie_rank = 0;  // ties at lower indices than this wavefront's current 64
    for (uint32_t w = 0; w < wave; w++) tie_rank += wave_ties[w];
    // ---- gather the winners ----
    for_each([&](uint32_t ord, uint32_t i) {
        const uint64_t key = ((uint64_t)ord << 32) | (uint32_t)(~i);
        bool in = ord != 0 && ord > T;
        if (!take_all) {
            const bool tie = ord != 0 && ord == T;
            const uint64_t m = __ballot(tie);
            const uint32_t before = (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
            if (tie) in = tie_rank + before < r;
            tie_rank += (uint32_t)__popcll(m);
        }
        if (in) {
            const uint32_t pos = atomicAdd(&sh_nwin, 1u);
            if (LARGE) { if (pos < cap) big[pos] = key; }
            else if (pos < 64) winners[pos] = key;
        }
    }, nullptr);
    __syncthreads();
    if (LARGE) {
        // bitonic sort of the cap keys, descending (the padding keys 0 sink to the end): log2(cap)*(log2(cap)+1)/2 rounds of
        // cap/2 compare-exchanges; thread t's pair in a round with distance j is (i, i+j), i = t with a 0 inserted at bit log2(j)
        for (uint32_t size = 2; size <= cap; size <<= 1) {
            for (uint32_t jd = size >> 1; jd > 0; jd >>= 1) {
                for (uint32_t t = tid; t < (cap >> 1); t += kTopkThreads) {
                    const uint32_t lo = 2 * t - (t & (jd - 1)), hi = lo + jd;
                    const bool desc = (lo & size) == 0;
                    const uint64_t a = big[lo], b = big[hi];
                    if ((a < b) == desc) { big[lo] = b; big[hi] = a; }
                }
                __syncthreads();
            }
        }
        const uint32_t nw = min(min(sh_nwin, cap), k);
        for (uint32_t i = tid; i < nw; i += kTopkThreads) {
            const uint32_t idx = ~(uint32_t)big[i];
            idx_out[(size_t)row * k + i] = idx;
            val_out[(size_t)row * k + i] = s[idx];
        }
        if (tid == 0) count_out[row] = nw;
        return;
    }
    if (wave == 0) {
        const uint64_t top = sort_desc(winners[lane], lane);
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
    if (k > kTopkMaxK) return hipErrorInvalidValue;
    if (k > 64 && n > 64) {
        // more than 64 winners: ordered in LDS (room for the next power of two above min(k, n) keys)
        uint32_t cap = 128;
        while (cap < k && cap < n) cap <<= 1;
        const size_t lds = (size_t)cap * sizeof(uint64_t);
        static std::atomic<bool> attr_abs{false}, attr_val{false};
        std::atomic<bool> &flag = by_abs ? attr_abs : attr_val;
        if (!flag) {  // dynamic LDS above 64 KB has to be allowed once per process
            const void *fn = by_abs ? (const void *)topk_kernel<true, false, true> : (const void *)topk_kernel<false, false, true>;
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(kTopkMaxK * sizeof(uint64_t)));
            if (e != hipSuccess) return e;
            flag = true;
        }
        if (by_abs) hipLaunchKernelGGL((topk_kernel<true, false, true>), dim3(batch), dim3(kTopkThreads), lds, stream, scores, n, k, idx_out, val_out, count_out, nan_flag, cap);
        else hipLaunchKernelGGL((topk_kernel<false, false, true>), dim3(batch), dim3(kTopkThreads), lds, stream, scores, n, k, idx_out, val_out, count_out, nan_flag, cap);
        return hipGetLastError();
    }
    const bool cached = n <= (uint32_t)(kTopkWaves * 64 * kTopkCached);
#define LARQL_TOPK(ABS, C) hipLaunchKernelGGL((topk_kernel<ABS, C, false>), dim3(batch), dim3(kTopkThreads), 0, stream, scores, n, k, idx_out, val_out, count_out, nan_flag, 0u)
    if (by_abs) { if (cached) LARQL_TOPK(true, true); else LARQL_TOPK(true, false); }
    else { if (cached) LARQL_TOPK(false, true); else LARQL_TOPK(false, false); }
#undef LARQL_TOPK
    return hipGetLastError();
}

}  // namespace larql
