// moe.hip — the small kernels around the MXFP4 expert matvecs of a MoE block:
// expert selection, the gate/up combine rule and the weighted sum.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

namespace larql {

// ---------------------------------------------------------------------------
// router::select — larql-compute/src/ffn/expert_weight/router.rs:33-70.
// One wavefront per token, lane i holds logit i (n_experts <= 64).  Rank by
// logit descending, first index wins ties (the reference's stable sort);
// weights are exp(l - max_all) / denominator, the denominator summed in f32
// over the selected logits in rank order (policy 1, NormalisedOverSelected) or
// over all experts in index order (policy 0, SoftmaxThenSelect).
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
    for (int o = 32; o > 0; o >>= 1) {
        uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
        lo = (uint32_t)__shfl_xor((int)lo, o, 64);
        hi = (uint32_t)__shfl_xor((int)hi, o, 64);
        const uint64_t other = ((uint64_t)hi << 32) | lo;
        v = other > v ? other : v;
    }
    return v;
}

__global__ void __launch_bounds__(64) router_select_kernel(const float *__restrict__ logits, uint32_t n_experts, uint32_t k,
                                                           int policy, uint32_t *__restrict__ experts,
                                                           float *__restrict__ weights) {
    const uint32_t t = blockIdx.x, lane = threadIdx.x;
    const bool has = lane < n_experts;
    const float l = has ? logits[(size_t)t * n_experts + lane] : 0.0f;
    // orderable key: logit bits made monotone, then ~index so the lower index wins a tie; 0 = absent
    const uint32_t bits = __builtin_bit_cast(uint32_t, l);
    const uint32_t ord = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    uint64_t key = has ? (((uint64_t)ord << 32) | (uint32_t)(~lane)) : 0;
    float dmax = has ? l : -__builtin_inff();
    for (int o = 32; o > 0; o >>= 1) dmax = fmaxf(dmax, __shfl_xor(dmax, o, 64));
    const float ex = has ? expf(l - dmax) : 0.0f;
    float denom = 0.0f;
    if (policy == 0)
        for (uint32_t i = 0; i < n_experts; i++) denom += __shfl(ex, (int)i, 64);  // index order, as the iterator sums
    uint32_t sel_idx[8];
    float sel_ex[8];
    for (uint32_t r = 0; r < k; r++) {
        const uint64_t best = wave_max_u64(key);
        const uint32_t idx = ~(uint32_t)best;
        sel_idx[r] = idx;
        sel_ex[r] = __shfl(ex, (int)idx, 64);
        if (lane == idx) key = 0;
    }
    if (policy != 0)
        for (uint32_t r = 0; r < k; r++) denom += sel_ex[r];  // rank order
    if (lane == 0)
        for (uint32_t r = 0; r < k; r++) {
            experts[(size_t)t * k + r] = sel_idx[r];
            weights[(size_t)t * k + r] = denom > 0.0f ? sel_ex[r] / denom : 0.0f;
        }
}

// MoeGateRule::ClampedGlu — larql-compute/src/pipeline/moe.rs:88-92:
// g = min(g, L); u = clamp(u, -L, L); (u + 1) * (g * sigmoid(alpha * g)).
__global__ void clamped_glu_kernel(const float *__restrict__ g, const float *__restrict__ u, float *__restrict__ h, size_t n,
                                   float limit, float alpha) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float gv = fminf(g[i], limit);
    float uv = u[i];
    uv = uv < -limit ? -limit : (uv > limit ? limit : uv);
    const float sig = 1.0f / (1.0f + expf(-(gv * alpha)));
    h[i] = (uv + 1.0f) * (gv * sig);
}

// out[t] = sum over the token's k selected experts, in selection order, of w * down-output
// (larql-compute/src/cpu/ops/moe/forward.rs:266-270).
__global__ void weighted_sum_kernel(const float *__restrict__ d, const float *__restrict__ weights, float *__restrict__ out,
                                    uint32_t k, uint32_t hidden) {
    const uint32_t t = blockIdx.y;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= hidden) return;
    float acc = 0.0f;
    for (uint32_t r = 0; r < k; r++) acc += weights[(size_t)t * k + r] * d[((size_t)t * k + r) * hidden + i];
    out[(size_t)t * hidden + i] = acc;
}

hipError_t router_select_launch(hipStream_t s, const float *logits, uint32_t tokens, uint32_t n_experts, uint32_t k, int policy,
                                uint32_t *experts, float *weights) {
    if (tokens == 0) return hipSuccess;
    hipLaunchKernelGGL(router_select_kernel, dim3(tokens), dim3(64), 0, s, logits, n_experts, k, policy, experts, weights);
    return hipGetLastError();
}
hipError_t clamped_glu_launch(hipStream_t s, const float *g, const float *u, float *h, size_t n, float limit, float alpha) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(clamped_glu_kernel, dim3((uint32_t)((n + 255) / 256)), dim3(256), 0, s, g, u, h, n, limit, alpha);
    return hipGetLastError();
}
hipError_t weighted_sum_launch(hipStream_t s, const float *d, const float *weights, float *out, uint32_t tokens, uint32_t k,
                               uint32_t hidden) {
    if (tokens == 0 || hidden == 0) return hipSuccess;
    hipLaunchKernelGGL(weighted_sum_kernel, dim3((hidden + 255) / 256, tokens), dim3(256), 0, s, d, weights, out, k, hidden);
    return hipGetLastError();
}

}  // namespace larql
