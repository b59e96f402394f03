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

// the same on the interleaved result of a fused gate_up matrix: g = gu[2i], u = gu[2i+1]
__global__ void clamped_glu_interleaved_kernel(const float *__restrict__ gu, float *__restrict__ h, size_t n, float limit, float alpha) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float gv = fminf(gu[2 * i], limit);
    float uv = gu[2 * i + 1];
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

// Job lists of an expert block, built on the device from the router's choice (no host round trip): the slots
// (token, rank) that chose the same expert are paired, in slot order, and every pair (or single) becomes one
// gate, one up and one down job whose two activations share the expert's weights (GemvJob::batch = 2; the
// second activation / result sits x_stride / out_stride floats away from the first, in either direction).
// tg / tu / td are the jobs of slot 0 with expert 0 (geometry filled in); tables: [gate jobs | up jobs], [down jobs];
// headers: {job count, pass total}.  One block; a thread per slot, O(slots) work each.
// `fused`: tg walks a fused gate_up matrix of 2*inter interleaved rows (no up jobs; a slot's results and the down
// job's activation are 2*inter floats, gate and up values alternating).
__global__ void __launch_bounds__(256) moe_plan_kernel(const uint32_t *__restrict__ experts, uint32_t slots, uint32_t k, uint32_t n_experts,
                                                       GemvJob tg, GemvJob tu, GemvJob td, uint64_t gu_w_stride, uint64_t gu_s_stride,
                                                       uint64_t dn_w_stride, uint64_t dn_s_stride, uint32_t hidden, uint32_t inter, uint32_t fused,
                                                       GemvJob *__restrict__ gu_table, uint32_t *__restrict__ gu_hdr,
                                                       GemvJob *__restrict__ dn_table, uint32_t *__restrict__ dn_hdr) {
    __shared__ uint32_t first_job[1025];  // first job of expert e; [n_experts] = total
    __shared__ uint32_t first_gcost[1025], first_dcost[1025];  // the same for the jobs' places in the two pass lists
    __shared__ uint32_t cnt[1024];        // slots per expert
    __shared__ uint32_t ex[4096];         // the router's choice, read once
    __shared__ uint32_t partner[4096];    // second slot of a job (or ~0)
    const uint32_t t = threadIdx.x;
    for (uint32_t e = t; e < n_experts; e += blockDim.x) cnt[e] = 0;
    for (uint32_t s = t; s < slots; s += blockDim.x) { ex[s] = experts[s]; partner[s] = 0xFFFFFFFFu; }
    __syncthreads();
    for (uint32_t s = t; s < slots; s += blockDim.x)
        if (ex[s] < n_experts) atomicAdd(&cnt[ex[s]], 1u);
    __syncthreads();
    // Cost of a job in the launches' pass lists, from cycle counts of the kernel: a tile costs the same whether one
    // or two tokens share it (its bytes set the pace), and a job segment starts with the preparation of its
    // activations, worth 4 (one token) or 6 (two) tiles.  Units: steps (a tile = cpr of them).
    const uint32_t g_tiles = ((uint32_t)tg.rows + 15) / 16, d_tiles = ((uint32_t)td.rows + 15) / 16;
    const uint32_t g_c1 = tg.cpr, g_c2 = tg.cpr, d_c1 = td.cpr, d_c2 = td.cpr;
    const uint32_t g_p1 = 4 * g_c1 + g_tiles * g_c1, g_p2 = 6 * g_c1 + g_tiles * g_c2;
    const uint32_t d_p1 = 4 * d_c1 + d_tiles * d_c1, d_p2 = 6 * d_c1 + d_tiles * d_c2;
    for (uint32_t e = t; e <= n_experts; e += blockDim.x) {
        uint32_t f = 0, gc = 0, dc = 0;
        for (uint32_t q = 0; q < e; q++) {
            f += (cnt[q] + 1) / 2;
            gc += (cnt[q] / 2) * g_p2 + (cnt[q] & 1u) * g_p1;
            dc += (cnt[q] / 2) * d_p2 + (cnt[q] & 1u) * d_p1;
        }
        first_job[e] = f; first_gcost[e] = gc; first_dcost[e] = dc;
    }
    __syncthreads();
    const uint32_t n_jobs = first_job[n_experts], g_total = first_gcost[n_experts], d_total = first_dcost[n_experts];
    // a slot's rank among the slots of its expert, in slot order: even ranks open a job, odd ranks join it
    for (uint32_t s = t; s < slots; s += blockDim.x) {
        const uint32_t e = ex[s];
        if (e >= n_experts) continue;
        uint32_t r = 0;
        for (uint32_t q = 0; q < s; q++) r += ex[q] == e ? 1u : 0u;
        if (r & 1u) partner[first_job[e] + r / 2] = s;
    }
    __syncthreads();
    for (uint32_t s1 = t; s1 < slots; s1 += blockDim.x) {
        const uint32_t e = ex[s1];
        if (e >= n_experts) continue;
        uint32_t r = 0;
        for (uint32_t q = 0; q < s1; q++) r += ex[q] == e ? 1u : 0u;
        if (r & 1u) continue;
        const uint32_t jb = first_job[e] + r / 2;
        const bool pair = partner[jb] != 0xFFFFFFFFu;
        const uint32_t s2 = pair ? partner[jb] : s1, nb = pair ? 2u : 1u;
        const uint32_t tok1 = s1 / k, tok2 = s2 / k;
        GemvJob a = tg, b = tu, c = td;
        a.w += (size_t)e * gu_w_stride; a.aux += (size_t)e * gu_s_stride;
        b.w += (size_t)e * gu_w_stride; b.aux += (size_t)e * gu_s_stride;
        c.w += (size_t)e * dn_w_stride; c.aux += (size_t)e * dn_s_stride;
        a.x += (size_t)tok1 * hidden; b.x += (size_t)tok1 * hidden;
        const size_t gs = fused ? 2 * (size_t)inter : (size_t)inter;  // floats of gate/up results per slot and half
        a.out += (size_t)s1 * gs; b.out += (size_t)s1 * gs;
        c.x += (size_t)s1 * gs; c.x_glu += (size_t)s1 * gs; c.out += (size_t)s1 * hidden;
        a.batch = b.batch = c.batch = nb;
        a.x_stride = b.x_stride = (uint64_t)(((int64_t)tok2 - (int64_t)tok1) * (int64_t)hidden);
        a.out_stride = b.out_stride = (uint64_t)(((int64_t)s2 - (int64_t)s1) * (int64_t)gs);
        c.x_stride = (uint64_t)(((int64_t)s2 - (int64_t)s1) * (int64_t)gs);
        c.out_stride = (uint64_t)(((int64_t)s2 - (int64_t)s1) * (int64_t)hidden);
        // (the earlier jobs of this expert are all shared by two tokens)
        a.pass_begin = first_gcost[e] + (r / 2) * g_p2;
        b.pass_begin = g_total + a.pass_begin;
        c.pass_begin = first_dcost[e] + (r / 2) * d_p2;
        a.n_pass = b.n_pass = pair ? g_p2 : g_p1; c.n_pass = pair ? d_p2 : d_p1;
        a.cpt = b.cpt = pair ? g_c2 : g_c1; c.cpt = pair ? d_c2 : d_c1;
        a.su = b.su = (pair ? 6u : 4u) * g_c1; c.su = (pair ? 6u : 4u) * d_c1;
        gu_table[jb] = a; dn_table[jb] = c;
        if (!fused) gu_table[n_jobs + jb] = b;
    }
    if (t == 0) {
        gu_hdr[0] = fused ? n_jobs : 2 * n_jobs; gu_hdr[1] = fused ? g_total : 2 * g_total;
        dn_hdr[0] = n_jobs; dn_hdr[1] = d_total;
    }
}

hipError_t moe_plan_launch(hipStream_t s, const uint32_t *experts, uint32_t slots, uint32_t k, uint32_t n_experts, const GemvJob &tg,
                           const GemvJob &tu, const GemvJob &td, uint64_t gu_w_stride, uint64_t gu_s_stride, uint64_t dn_w_stride,
                           uint64_t dn_s_stride, uint32_t hidden, uint32_t inter, bool fused, GemvJob *gu_table, uint32_t *gu_hdr,
                           GemvJob *dn_table, uint32_t *dn_hdr) {
    if (n_experts > 1024) return hipErrorInvalidValue;
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(256), 0, s, experts, slots, k, n_experts, tg, tu, td, gu_w_stride, gu_s_stride,
                       dn_w_stride, dn_s_stride, hidden, inter, fused ? 1u : 0u, gu_table, gu_hdr, dn_table, dn_hdr);
    return hipGetLastError();
}

hipError_t router_select_launch(hipStream_t s, const float *logits, uint32_t tokens, uint32_t n_experts, uint32_t k, int policy,
                                uint32_t *experts, float *weights) {
    if (tokens == 0) return hipSuccess;
    hipLaunchKernelGGL(router_select_kernel, dim3(tokens), dim3(64), 0, s, logits, n_experts, k, policy, experts, weights);
    return hipGetLastError();
}
hipError_t clamped_glu_interleaved_launch(hipStream_t s, const float *gu, float *h, size_t n, float limit, float alpha) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(clamped_glu_interleaved_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, gu, h, n, limit, alpha);
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
