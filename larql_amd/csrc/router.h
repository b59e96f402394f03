// router.h — Router::select for one token by one wavefront (device code shared by the selection kernel and the
// expert matvec kernel, which can do its own selection).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace larql {

// Reductions over the wavefront by data-parallel primitives (four steps inside the rows of 16 lanes, two row
// broadcasts, then lane 63 holds the result): a few cycles per step, where a cross-lane shuffle costs an LDS round trip.
template <int CTRL, int ROW_MASK, bool BOUND>
__device__ __forceinline__ uint64_t dpp_max_u64(uint64_t v) {  // lanes without a source read 0: the identity here
    const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)v, CTRL, ROW_MASK, 0xF, BOUND);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(v >> 32), CTRL, ROW_MASK, 0xF, BOUND);
    const uint64_t other = ((uint64_t)hi << 32) | lo;
    return other > v ? other : v;
}
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
    v = dpp_max_u64<0xB1, 0xF, true>(v);    // quad_perm [1,0,3,2]
    v = dpp_max_u64<0x4E, 0xF, true>(v);    // quad_perm [2,3,0,1]
    v = dpp_max_u64<0x141, 0xF, true>(v);   // row_half_mirror
    v = dpp_max_u64<0x140, 0xF, true>(v);   // row_mirror
    v = dpp_max_u64<0x142, 0xA, false>(v);  // row_bcast:15 into rows 1 and 3
    v = dpp_max_u64<0x143, 0xC, false>(v);  // row_bcast:31 into rows 2 and 3
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, 63), hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), 63);
    return ((uint64_t)hi << 32) | lo;
}
template <int CTRL, int ROW_MASK, bool BOUND>
__device__ __forceinline__ float dpp_fmax(float v) {  // lanes without a source read -inf
    return fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp((int)0xFF800000u, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, BOUND)));
}
__device__ __forceinline__ float wave_fmax(float v) {
    v = dpp_fmax<0xB1, 0xF, false>(v);
    v = dpp_fmax<0x4E, 0xF, false>(v);
    v = dpp_fmax<0x141, 0xF, false>(v);
    v = dpp_fmax<0x140, 0xF, false>(v);
    v = dpp_fmax<0x142, 0xA, false>(v);
    v = dpp_fmax<0x143, 0xC, false>(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float lane_value(float v, uint32_t lane_uniform) {  // the lane index must be the same in every lane
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), (int)lane_uniform));
}

constexpr int kRouterMaxK = 8;

// router::select — larql-compute/src/ffn/expert_weight/router.rs:33-70 — for one token: lane i holds logit i
// (n_experts <= 64 — router_select_wide below takes up to 256 — and k <= min(8, n_experts)).  Rank by logit descending, first index wins ties (the reference's stable
// sort); weights are exp(l - max_all) / denominator, the denominator summed in f32 over the selected logits in rank
// order (policy 1, NormalisedOverSelected) or over all experts in index order (policy 0, SoftmaxThenSelect).
// Every lane ends with the same sel_idx / sel_w (entries from k on are 0).  WEIGHTS = false leaves sel_w at 0 (a
// caller that only needs to know which experts).
// (router_select_lane: lane i brings its logit, bias already added; lanes from n_experts on bring anything)
template <bool WEIGHTS = true>
__device__ __forceinline__ void router_select_lane(float l, uint32_t n_experts, uint32_t k, int policy, uint32_t lane,
                                                   uint32_t (&sel_idx)[kRouterMaxK], float (&sel_w)[kRouterMaxK]) {
    const bool has = lane < n_experts;
    l = has ? l : 0.0f;
    // orderable key: logit bits made monotone, then ~index so the lower index wins a tie; 0 = absent
    const uint32_t bits = __builtin_bit_cast(uint32_t, l);
    const uint32_t ord = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    uint64_t key = has ? (((uint64_t)ord << 32) | (uint32_t)(~lane)) : 0;
    float ex = 0.0f, denom = 0.0f;
    if (WEIGHTS) {
        const float dmax = wave_fmax(has ? l : -__builtin_inff());
        ex = has ? expf(l - dmax) : 0.0f;
        if (policy == 0)
            for (uint32_t i = 0; i < n_experts; i++) denom += lane_value(ex, i);  // index order, as the iterator sums
    }
    float sel_ex[kRouterMaxK];
#pragma unroll
    for (int r = 0; r < kRouterMaxK; r++) {
        sel_idx[r] = 0; sel_ex[r] = 0.0f;
        if ((uint32_t)r < k) {
            const uint64_t best = wave_max_u64(key);
            const uint32_t idx = ~(uint32_t)best & 63u;  // (k <= n_experts: a key is always left; the mask keeps the lane index in range regardless)
            sel_idx[r] = idx;
            if (WEIGHTS) sel_ex[r] = lane_value(ex, idx);
            if (lane == idx) key = 0;
        }
    }
    if (WEIGHTS && policy != 0) {
#pragma unroll
        for (int r = 0; r < kRouterMaxK; r++)
            if ((uint32_t)r < k) denom += sel_ex[r];  // rank order
    }
#pragma unroll
    for (int r = 0; r < kRouterMaxK; r++) sel_w[r] = (WEIGHTS && (uint32_t)r < k && denom > 0.0f) ? sel_ex[r] / denom : 0.0f;
}

template <bool WEIGHTS = true>
__device__ __forceinline__ void router_select_wave(const float *logits, const float *bias, uint32_t n_experts, uint32_t k, int policy, uint32_t lane,
                                                   uint32_t (&sel_idx)[kRouterMaxK], float (&sel_w)[kRouterMaxK]) {
    // the router bias joins the logit before anything else (MoeLayerWeights::router_bias, larql-compute/src/pipeline/moe.rs:505-508)
    const float l = lane < n_experts ? (bias ? logits[lane] + bias[lane] : logits[lane]) : 0.0f;
    router_select_lane<WEIGHTS>(l, n_experts, k, policy, lane, sel_idx, sel_w);
}

constexpr int kRouterWideSlots = 4;  // logits per lane in router_select_wide

// The same selection over up to 256 experts: lane i holds the logits of experts i, i + 64, i + 128 and i + 192 (the
// banks of 128 experts of the larger GPT-OSS and Gemma 4 checkpoints).  Same order of every f32 sum as above.
template <bool WEIGHTS = true>
__device__ __forceinline__ void router_select_wide(const float *logits, const float *bias, uint32_t n_experts, uint32_t k, int policy, uint32_t lane,
                                                   uint32_t (&sel_idx)[kRouterMaxK], float (&sel_w)[kRouterMaxK]) {
    constexpr int S = kRouterWideSlots;
    float ex[S];
    uint64_t key[S];
    float l[S], lmax = -__builtin_inff();
#pragma unroll
    for (int s = 0; s < S; s++) {
        const uint32_t e = lane + 64u * (uint32_t)s;
        const bool has = e < n_experts;
        l[s] = 0.0f;
        if (has) l[s] = bias ? logits[e] + bias[e] : logits[e];
        const uint32_t bits = __builtin_bit_cast(uint32_t, l[s]);
        const uint32_t ord = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
        key[s] = has ? (((uint64_t)ord << 32) | (uint32_t)(~e)) : 0;
        lmax = has ? fmaxf(lmax, l[s]) : lmax;
    }
    float denom = 0.0f;
    if (WEIGHTS) {
        const float dmax = wave_fmax(lmax);
#pragma unroll
        for (int s = 0; s < S; s++) ex[s] = lane + 64u * (uint32_t)s < n_experts ? expf(l[s] - dmax) : 0.0f;
        if (policy == 0) {
#pragma unroll
            for (int s = 0; s < S; s++)
                for (uint32_t i = 0; i < 64u && 64u * (uint32_t)s + i < n_experts; i++) denom += lane_value(ex[s], i);  // index order
        }
    } else {
#pragma unroll
        for (int s = 0; s < S; s++) ex[s] = 0.0f;
    }
    float sel_ex[kRouterMaxK];
#pragma unroll
    for (int r = 0; r < kRouterMaxK; r++) {
        sel_idx[r] = 0; sel_ex[r] = 0.0f;
        if ((uint32_t)r < k) {
            uint64_t mine = key[0];
#pragma unroll
            for (int s = 1; s < S; s++) mine = key[s] > mine ? key[s] : mine;
            const uint64_t best = wave_max_u64(mine);
            const uint32_t idx = ~(uint32_t)best & (uint32_t)(64 * S - 1);             // (k <= n_experts: a key is always left)
            const uint32_t slot = idx >> 6, owner = idx & 63u;                         // the same in every lane
            sel_idx[r] = idx;
            if (WEIGHTS) {
                float v = ex[0];
#pragma unroll
                for (int s = 1; s < S; s++) v = slot == (uint32_t)s ? ex[s] : v;
                sel_ex[r] = lane_value(v, owner);
            }
#pragma unroll
            for (int s = 0; s < S; s++)
                if (lane == owner && slot == (uint32_t)s) key[s] = 0;
        }
    }
    if (WEIGHTS && policy != 0) {
#pragma unroll
        for (int r = 0; r < kRouterMaxK; r++)
            if ((uint32_t)r < k) denom += sel_ex[r];  // rank order
    }
#pragma unroll
    for (int r = 0; r < kRouterMaxK; r++) sel_w[r] = (WEIGHTS && (uint32_t)r < k && denom > 0.0f) ? sel_ex[r] / denom : 0.0f;
}

// whichever of the two fits the bank (n_experts is the same in every lane)
template <bool WEIGHTS = true>
__device__ __forceinline__ void router_select_any(const float *logits, const float *bias, uint32_t n_experts, uint32_t k, int policy, uint32_t lane,
                                                  uint32_t (&sel_idx)[kRouterMaxK], float (&sel_w)[kRouterMaxK]) {
    if (n_experts <= 64u) router_select_wave<WEIGHTS>(logits, bias, n_experts, k, policy, lane, sel_idx, sel_w);
    else router_select_wide<WEIGHTS>(logits, bias, n_experts, k, policy, lane, sel_idx, sel_w);
}

}  // namespace larql
