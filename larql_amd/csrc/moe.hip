// moe.hip — the small kernels around the MXFP4 expert matvecs of a MoE block:
// expert selection, the gate/up combine rule and the weighted sum.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"
#include "router.h"

namespace larql {

static_assert(kRouterMaxExperts == 64u * (uint32_t)kRouterWideSlots, "the wide selection holds kRouterMaxExperts logits");

// router::select for every token: one wavefront per token (router.h).
__global__ void __launch_bounds__(64) router_select_kernel(const float *__restrict__ logits, const float *__restrict__ bias, uint32_t n_experts,
                                                           uint32_t k, int policy, uint32_t *__restrict__ experts,
                                                           float *__restrict__ weights) {
    const uint32_t t = blockIdx.x, lane = threadIdx.x;
    uint32_t sel_idx[kRouterMaxK];
    float sel_w[kRouterMaxK];
    router_select_any(logits + (size_t)t * n_experts, bias, n_experts, k, policy, lane, sel_idx, sel_w);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < kRouterMaxK; r++)
            if ((uint32_t)r < k) {
                experts[(size_t)t * k + r] = sel_idx[r];
                weights[(size_t)t * k + r] = sel_w[r];
            }
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

// weights[i] *= scale[experts[i]] — MoeExpertScalePolicy::PerExpert (larql-compute/src/cpu/ops/moe/mod.rs:168-176);
// a selected id outside the scale table keeps its weight, as the reference leaves it.
__global__ void expert_scale_kernel(float *__restrict__ weights, const uint32_t *__restrict__ experts, const float *__restrict__ scale,
                                    uint32_t n, uint32_t n_scale) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const uint32_t e = experts[i];
    if (e < n_scale) weights[i] *= scale[e];
}

// out[t] = sum over the token's k selected experts, in selection order, of w * down-output
// (larql-compute/src/cpu/ops/moe/forward.rs:266-270).  A slot whose expert id lies outside the bank is skipped
// (forward.rs:203-208): its rows of `d` were never written and are not read.
__global__ void weighted_sum_kernel(const float *__restrict__ d, const float *__restrict__ weights, const uint32_t *__restrict__ experts,
                                    uint32_t n_experts, float *__restrict__ out, uint32_t k, uint32_t hidden) {
    const uint32_t t = blockIdx.y;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= hidden) return;
    float acc = 0.0f;
    for (uint32_t r0 = 0; r0 < k; r0 += 4) {  // four loads in flight, added in selection order
        float w[4], v[4];
#pragma unroll
        for (uint32_t q = 0; q < 4; q++) {
            const bool in = r0 + q < k && experts[(size_t)t * k + r0 + q] < n_experts;
            w[q] = in ? weights[(size_t)t * k + r0 + q] : 0.0f;
            v[q] = in ? d[((size_t)t * k + r0 + q) * hidden + i] : 0.0f;
        }
#pragma unroll
        for (uint32_t q = 0; q < 4; q++)
            if (r0 + q < k && experts[(size_t)t * k + r0 + q] < n_experts) acc += w[q] * v[q];
    }
    out[(size_t)t * hidden + i] = acc;
}

// ---- the k-quant expert path (cpu_moe_forward over Q4_K / Q6_K banks: cpu/ops/moe/forward.rs:160-330) ----------------

// quantize_x_to_q8k (cpu/ops/q4k_q8k_dot/q8k_activation.rs:84-109) of one 256-element super-block that a wavefront
// holds four elements per lane: d = amax / 127, codes round(x * (1/d)) clamped to +-127, NaN -> 0.  `sum` ends, in the
// lanes 8s, as the sum of sub-block s's 32 codes.
__device__ __forceinline__ int q8k_code(float t) {
    float r = roundf(t);
    r = r < -127.0f ? -127.0f : (r > 127.0f ? 127.0f : r);
    return r != r ? 0 : (int)r;
}
__device__ __forceinline__ void q8k_block(const float (&v)[4], uint32_t &codes, float &scale, int &sum) {
    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));  // fmaxf ignores a NaN operand, as f32::max does
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    scale = amax > 0.0f ? amax / 127.0f : 0.0f;
    const float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
    const int q0 = q8k_code(v[0] * inv), q1 = q8k_code(v[1] * inv), q2 = q8k_code(v[2] * inv), q3 = q8k_code(v[3] * inv);
    sum = q0 + q1 + q2 + q3;
    sum += __shfl_xor(sum, 1);
    sum += __shfl_xor(sum, 2);
    sum += __shfl_xor(sum, 4);
    codes = ((uint32_t)q0 & 0xFFu) | (((uint32_t)q1 & 0xFFu) << 8) | (((uint32_t)q2 & 0xFFu) << 16) | (((uint32_t)q3 & 0xFFu) << 24);
}
// the device layout of a Q8_K activation of `cols` elements at `o`: [cols codes | cols/256 f32 scales | cols/32 i16 sums]
__device__ __forceinline__ void q8k_store(uint8_t *o, uint32_t cols, uint32_t sb, uint32_t lane, uint32_t codes, float scale, int sum) {
    const uint32_t nb = cols / 256;
    reinterpret_cast<uint32_t *>(o)[sb * 64 + lane] = codes;
    if (lane == 0) reinterpret_cast<float *>(o + cols)[sb] = scale;
    if ((lane & 7u) == 0) reinterpret_cast<int16_t *>(o + cols + (size_t)nb * 4)[sb * 8 + (lane >> 3)] = (int16_t)sum;
}

// Row `blockIdx.y` of src ([rows, src_cols] floats, src_stride apart), zero-padded to `cols` (a multiple of 256: the
// stored row width of the gate/up matrices, forward.rs:176-184), as a Q8_K activation of its own at dst + row * dst_stride.
// One wavefront per super-block.
__global__ void __launch_bounds__(256) quantize_rows_to_q8k_kernel(const float *__restrict__ src, size_t src_stride, uint32_t src_cols, uint32_t cols,
                                                                  uint8_t *__restrict__ dst, size_t dst_stride) {
    const uint32_t sb = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
    if (sb >= cols / 256) return;
    const float *s = src + (size_t)blockIdx.y * src_stride;
    const uint32_t j = sb * 256 + 4 * lane;
    float v[4];
#pragma unroll
    for (uint32_t i = 0; i < 4; i++) v[i] = j + i < src_cols ? s[j + i] : 0.0f;
    uint32_t codes; float scale; int sum;
    q8k_block(v, codes, scale, sum);
    q8k_store(dst + (size_t)blockIdx.y * dst_stride, cols, sb, lane, codes, scale, sum);
}

// Token `blockIdx.x`'s route and its expert input in one launch (they do not depend on one another): wavefront 0 selects
// as router_select_kernel does and applies MoeExpertScalePolicy::PerExpert where a scale table is given (as
// expert_scale_kernel does); the four wavefronts then quantise the token's row as quantize_rows_to_q8k_kernel does.
__global__ void __launch_bounds__(256) moe_kq_route_quant_kernel(const float *__restrict__ logits, const float *__restrict__ bias, uint32_t n_experts, uint32_t k,
                                                                int policy, const float *__restrict__ scale, uint32_t *__restrict__ experts,
                                                                float *__restrict__ weights, const float *__restrict__ src, size_t src_stride,
                                                                uint32_t src_cols, uint32_t cols, uint8_t *__restrict__ dst, size_t dst_stride) {
    const uint32_t t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    if (wave == 0) {
        uint32_t sel_idx[kRouterMaxK];
        float sel_w[kRouterMaxK];
        router_select_any(logits + (size_t)t * n_experts, bias, n_experts, k, policy, lane, sel_idx, sel_w);
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < kRouterMaxK; r++)
                if ((uint32_t)r < k) {
                    const uint32_t e = sel_idx[r];
                    experts[(size_t)t * k + r] = e;
                    weights[(size_t)t * k + r] = (scale && e < n_experts) ? sel_w[r] * scale[e] : sel_w[r];
                }
        }
    }
    const float *s = src + (size_t)t * src_stride;
    for (uint32_t sb = wave; sb < cols / 256; sb += 4) {
        const uint32_t j = sb * 256 + 4 * lane;
        float v[4];
#pragma unroll
        for (uint32_t i = 0; i < 4; i++) v[i] = j + i < src_cols ? s[j + i] : 0.0f;
        uint32_t codes; float sc; int sum;
        q8k_block(v, codes, sc, sum);
        q8k_store(dst + (size_t)t * dst_stride, cols, sb, lane, codes, sc, sum);
    }
}

// Row `blockIdx.y` of src ([rows, src_cols] floats, src_stride apart) zero-padded to `cols` floats at dst + row * cols:
// the expert input of a float bank whose rows are stored wider than hidden (forward.rs:176-184).
__global__ void __launch_bounds__(256) pad_rows_f32_kernel(const float *__restrict__ src, size_t src_stride, uint32_t src_cols, uint32_t cols,
                                                          float *__restrict__ dst) {
    const uint32_t j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= cols) return;
    dst[(size_t)blockIdx.y * cols + j] = j < src_cols ? src[(size_t)blockIdx.y * src_stride + j] : 0.0f;
}

// math::silu / math::gelu_tanh (cpu/ops/moe/math.rs:54-65) and MoeGateRule::combine (pipeline/moe.rs:73-118)
__device__ __forceinline__ float moe_combine(int rule, float g, float u, float limit, float alpha) {
    if (rule == 1) {
        const float c = 0.7978846f;
        return 0.5f * g * (1.0f + tanhf(c * (g + 0.044715f * g * g * g))) * u;
    }
    if (rule == 2) return g / (1.0f + expf(-g)) * u;
    if (rule == 3) {  // SituGlu { beta = limit, linear_beta = alpha, 0 for None }
        const float situ_a = limit * tanhf(g / limit) * (1.0f / (1.0f + expf(-g)));
        const float uc = alpha != 0.0f ? alpha * tanhf(u / alpha) : u;
        return situ_a * uc;
    }
    const float gv = fminf(g, limit);
    const float uv = u < -limit ? -limit : (u > limit ? limit : u);
    if (rule == 4) return 0.5f * gv * (1.0f + tanhf(0.7978846f * (gv + 0.044715f * gv * gv * gv))) * uv;  // ClampedGated { limit, gelu_tanh }
    if (rule == 5) return gv / (1.0f + expf(-gv)) * uv;                                                    // ClampedGated { limit, silu }
    return (uv + 1.0f) * (gv * (1.0f / (1.0f + expf(-(gv * alpha)))));
}

// Slot `blockIdx.y`'s activation: act[j] = combine(g[j] + gate bias, u[j] + up bias) for j < inter (the fused bias row
// of the slot's expert is interleaved: gate at 2j, up at 2j+1 — ExpertMlp::gate_bias / up_bias, pipeline/moe.rs:150-170),
// zeros up to inter_padded, quantised to a Q8_K activation of inter_padded elements at dst + slot * dst_stride
// (run_single_expert_kq_q8k_into, cpu/ops/moe/expert/q4k.rs:300-325).  A slot whose expert lies outside the bank gets
// no bias; its result is never read.
__global__ void __launch_bounds__(256) moe_kq_act_q8k_kernel(const float *__restrict__ g, const float *__restrict__ u, uint32_t inter, uint32_t inter_padded,
                                                            const uint32_t *__restrict__ experts, uint32_t n_experts, const float *__restrict__ gub,
                                                            int rule, float limit, float alpha, uint8_t *__restrict__ dst, size_t dst_stride) {
    const uint32_t sb = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63u;
    if (sb >= inter_padded / 256) return;
    const uint32_t slot = blockIdx.y;
    const uint32_t e = experts[slot];
    const float *b = (gub && e < n_experts) ? gub + (size_t)e * 2 * inter : nullptr;
    const uint32_t j = sb * 256 + 4 * lane;
    float v[4];
#pragma unroll
    for (uint32_t i = 0; i < 4; i++) {
        v[i] = 0.0f;
        if (j + i < inter) {
            const float gv = g[(size_t)slot * inter + j + i] + (b ? b[2 * (j + i)] : 0.0f);
            const float uv = u[(size_t)slot * inter + j + i] + (b ? b[2 * (j + i) + 1] : 0.0f);
            v[i] = moe_combine(rule, gv, uv, limit, alpha);
        }
    }
    uint32_t codes; float scale; int sum;
    q8k_block(v, codes, scale, sum);
    q8k_store(dst + (size_t)slot * dst_stride, inter_padded, sb, lane, codes, scale, sum);
}

// The same activation kept as f32 (a float bank: cpu_moe_forward's f32 arm, forward.rs:262-267): slot `blockIdx.y`'s row
// of `inter` floats at act + slot * act_stride.
__global__ void __launch_bounds__(256) moe_act_f32_kernel(const float *__restrict__ g, const float *__restrict__ u, uint32_t inter,
                                                         const uint32_t *__restrict__ experts, uint32_t n_experts, const float *__restrict__ gub, int rule,
                                                         float limit, float alpha, float *__restrict__ act, size_t act_stride) {
    const uint32_t j = blockIdx.x * blockDim.x + threadIdx.x, slot = blockIdx.y;
    if (j >= inter) return;
    const uint32_t e = experts[slot];
    const float *b = (gub && e < n_experts) ? gub + (size_t)e * 2 * inter : nullptr;
    const float gv = g[(size_t)slot * inter + j] + (b ? b[2 * j] : 0.0f);
    const float uv = u[(size_t)slot * inter + j] + (b ? b[2 * j + 1] : 0.0f);
    act[(size_t)slot * act_stride + j] = moe_combine(rule, gv, uv, limit, alpha);
}

// out[t] = sum over the token's k slots, in selection order, of w * (down output + the expert's down bias)
// (forward.rs:220-228: add_down_bias, then `*a += w * v`); a slot whose expert lies outside the bank is skipped.
__global__ void weighted_sum_bias_kernel(const float *__restrict__ d, const float *__restrict__ weights, const uint32_t *__restrict__ experts,
                                         uint32_t n_experts, const float *__restrict__ bias, float *__restrict__ out, uint32_t k, uint32_t hidden) {
    const uint32_t t = blockIdx.y;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= hidden) return;
    float acc = 0.0f;
    for (uint32_t r = 0; r < k; r++) {
        const uint32_t e = experts[(size_t)t * k + r];
        if (e >= n_experts) continue;
        float v = d[((size_t)t * k + r) * hidden + i];
        if (bias) v += bias[(size_t)e * hidden + i];
        acc += weights[(size_t)t * k + r] * v;
    }
    out[(size_t)t * hidden + i] = acc;
}

// Job lists of an expert block, built on the device from the router's choice (no host round trip): the slots
// (token, rank) that chose the same expert are grouped by `group` (2 or 4), in slot order, and every group becomes one
// gate, one up and one down job whose activations share the expert's weights (GemvJob::batch = tokens in the group;
// the other activations / results sit x_stride, x_off[] / out_stride, out_off[] floats away from the first).
// tg / tu / td are the jobs of slot 0 with expert 0 (geometry filled in); tables: [gate jobs | up jobs], [down jobs];
// headers: {job count, pass total}.  One block; a thread per slot, O(slots) work each.
// `fused`: tg walks a fused gate_up matrix of 2*inter interleaved rows (no up jobs; a slot's results and the down
// job's activation are 2*inter floats, gate and up values alternating).
// With `logits` the kernel is the router as well (one launch fewer in front of the matvecs): a wavefront per token
// selects as router_select_kernel does and writes `experts` / `weights` before the planning reads the choice.
__global__ void __launch_bounds__(1024) moe_plan_kernel(const float *__restrict__ logits, const float *__restrict__ router_bias, int policy,
                                                       float *__restrict__ weights, uint32_t *__restrict__ experts, uint32_t slots, uint32_t k, uint32_t n_experts,
                                                       GemvJob tg, GemvJob tu, GemvJob td, uint64_t gu_w_stride, uint64_t gu_s_stride,
                                                       uint64_t dn_w_stride, uint64_t dn_s_stride, uint32_t hidden, uint32_t inter, uint32_t fused,
                                                       uint32_t group, uint32_t g_grid, uint32_t d_grid, GemvJob *__restrict__ gu_table,
                                                       uint32_t *__restrict__ gu_hdr, GemvJob *__restrict__ dn_table, uint32_t *__restrict__ dn_hdr,
                                                       uint32_t *__restrict__ gu_first, uint32_t *__restrict__ dn_first) {
    __shared__ uint32_t first_job[1025];  // first job of expert e; [n_experts] = total
    __shared__ uint32_t first_kind_a[1025], first_kind_b[1025];  // the jobs before expert e by kind: {full groups, of 1 slot}, {of 2, of 3}
    __shared__ __attribute__((aligned(16))) uint32_t cnt[1024];  // slots per expert
    __shared__ __attribute__((aligned(16))) uint32_t ex[4096];   // the router's choice, read once
    __shared__ uint32_t first_slot[1025]; // slots of the experts before e
    __shared__ uint16_t rank[4096];       // a slot's rank among the slots of its expert, in slot order
    __shared__ uint16_t by_expert[4096];  // the slots ordered by (expert, rank)
    const uint32_t t = threadIdx.x;
    const uint32_t gsh = group == 4 ? 2u : 1u, gmask = group - 1;  // (group is 2 or 4: no divisions below)
    for (uint32_t e = t; e < ((n_experts + 3u) & ~3u); e += blockDim.x) cnt[e] = 0;
    if (logits) {
        const uint32_t lane = t & 63u, tokens = slots / k;
        for (uint32_t tok = t >> 6; tok < tokens; tok += blockDim.x >> 6) {
            uint32_t sel_idx[kRouterMaxK];
            float sel_w[kRouterMaxK];
            router_select_any(logits + (size_t)tok * n_experts, router_bias, n_experts, k, policy, lane, sel_idx, sel_w);
            if (lane == 0) {
#pragma unroll
                for (int r = 0; r < kRouterMaxK; r++)
                    if ((uint32_t)r < k) {
                        experts[(size_t)tok * k + r] = sel_idx[r];
                        weights[(size_t)tok * k + r] = sel_w[r];
                        ex[tok * k + r] = sel_idx[r];
                    }
            }
        }
        for (uint32_t s2 = slots + t; s2 < ((slots + 3u) & ~3u); s2 += blockDim.x) ex[s2] = 0xFFFFFFFFu;
    } else {
        for (uint32_t s = t; s < ((slots + 3u) & ~3u); s += blockDim.x) ex[s] = s < slots ? experts[s] : 0xFFFFFFFFu;
    }
    __syncthreads();
    if (slots <= 64 && n_experts <= 64) {
        // A block of up to 64 slots and 64 experts is planned by one wavefront without a barrier in between: lane s is
        // slot s (its rank = the earlier lanes with the same expert, one ballot per expert), lane e is expert e (its
        // count from the same ballots, the sums over the experts before it by a scan across the lanes).
        if (t < 64) {
            const uint32_t e = t < slots ? ex[t] : 0xFFFFFFFFu;
            uint32_t r = 0, c = 0;
            for (uint32_t q = 0; q < n_experts; q++) {
                const uint64_t m = __ballot(e == q);
                if (e == q) r = (uint32_t)__popcll(m & ((1ull << t) - 1ull));
                if (t == q) c = (uint32_t)__popcll(m);
            }
            if (t < slots) rank[t] = (uint16_t)r;
            if (t < n_experts) cnt[t] = c;
            // what expert t adds to the sums (lanes from n_experts on add nothing): jobs | slots << 16, and the jobs by kind
            // in one word (full groups, groups of 1, 2, 3 slots: a byte each, at most 64)
            const uint32_t mm = c & gmask;
            uint32_t js = ((c + gmask) >> gsh) | (c << 16);
            uint32_t kk = (c >> gsh) | (mm == 1 ? 0x100u : 0u) | (mm == 2 ? 0x10000u : 0u) | (mm == 3 ? 0x1000000u : 0u);
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {  // inclusive sums over the lanes
                const uint32_t a = (uint32_t)__shfl_up((int)js, o, 64), bq = (uint32_t)__shfl_up((int)kk, o, 64);
                if (t >= (uint32_t)o) { js += a; kk += bq; }
            }
            // entry e = the experts before e: lane e - 1's inclusive sums (entry 0 = nothing, entry n_experts = everything)
            const uint32_t at = t + 1;
            if (at <= n_experts) {
                first_job[at] = js & 0xFFFFu; first_slot[at] = js >> 16;
                first_kind_a[at] = (kk & 0xFFu) | (((kk >> 8) & 0xFFu) << 16);
                first_kind_b[at] = ((kk >> 16) & 0xFFu) | ((kk >> 24) << 16);
            }
            if (t == 0) { first_job[0] = 0; first_slot[0] = 0; first_kind_a[0] = 0; first_kind_b[0] = 0; }
            // (the same wavefront reads what it has just written: LDS executes a wavefront's operations in order)
            if (e < n_experts) by_expert[first_slot[e] + r] = (uint16_t)t;
        }
        __syncthreads();
    } else {
        // ranks: four earlier slots per LDS read, the reads of a round independent of each other
        for (uint32_t s = t; s < slots; s += blockDim.x) {
            const uint32_t e = ex[s];
            uint32_t r = 0;
    #pragma unroll 4
            for (uint32_t q = 0; q < s; q += 4) {
                const uint4 v = *reinterpret_cast<const uint4 *>(&ex[q]);
                r += (v.x == e ? 1u : 0u) + (q + 1 < s && v.y == e ? 1u : 0u) + (q + 2 < s && v.z == e ? 1u : 0u) + (q + 3 < s && v.w == e ? 1u : 0u);
            }
            rank[s] = (uint16_t)r;
            if (e < n_experts) atomicAdd(&cnt[e], 1u);
        }
        __syncthreads();
        // Per expert: the jobs before it, counted by kind (full groups, and groups of 1, 2 or 3 slots), 16 bits a count.
        for (uint32_t e = t; e <= n_experts; e += blockDim.x) {
            uint32_t f = 0, ka = 0, kb = 0, fs = 0;
            auto add = [&](uint32_t c) {
                fs += c;
                f += (c + gmask) >> gsh;
                const uint32_t m = c & gmask;
                ka += (c >> gsh) + (m == 1 ? 0x10000u : 0u);
                kb += (m == 2 ? 1u : 0u) + (m == 3 ? 0x10000u : 0u);
            };
    #pragma unroll 2
            for (uint32_t q = 0; q < e; q += 4) {
                const uint4 v = *reinterpret_cast<const uint4 *>(&cnt[q]);
                add(v.x);
                if (q + 1 < e) add(v.y);
                if (q + 2 < e) add(v.z);
                if (q + 3 < e) add(v.w);
            }
            first_job[e] = f; first_kind_a[e] = ka; first_kind_b[e] = kb; first_slot[e] = fs;
        }
        __syncthreads();
    }
    const uint32_t n_jobs = first_job[n_experts];
    // Cost of a job in a launch's pass list.  A workgroup prepares the activations of every job it takes a share of
    // before the share's first tile: about 3 tiles' time for one token and 2 more for every further one (time
    // stamps of the kernel), whether the share opens the job or not.  A job cut into n shares pays that n times, and
    // n = 1 + tiles / (tiles per workgroup) on average: so a job costs one preparation up front (GemvJob::su) and each
    // of its tiles carries the preparation's part, cpt = 4 * tpw + prep in quarter tiles where a tile's own time is
    // 4 * tpw units (tpw = the launch's tiles per workgroup).  The workgroup that opens a job mid-share also lets its
    // stream of weights run dry in between: 2 tiles more up front.  Launches whose workgroups walk more than 256
    // tiles each leave the parts out (under 4 % of a share).
    struct JobCost {  // of a job with m tokens, in one launch
        uint32_t tiles, unit;  // unit = tpw, or 0 where the parts are left out
        __device__ uint32_t prep(uint32_t m) const { return 12 + 8 * (m - 1); }
        __device__ uint32_t cpt(uint32_t m) const { return unit ? 4 * unit + prep(m) : 4u; }
        __device__ uint32_t su(uint32_t m) const { return (prep(m) + 8) * (unit ? unit : 1u); }
        __device__ uint32_t job(uint32_t m) const { return su(m) + tiles * cpt(m); }
    };
    const auto cost_model = [&](uint32_t tiles, uint32_t grid, uint32_t lists) {
        // (float arithmetic: a rough figure is all the model needs, and a 64-bit division is a hundred instructions)
        const float tpw_f = (float)(lists * n_jobs) * (float)tiles / (float)max(grid, 1u);
        const uint32_t tpw = tpw_f < 1.0f ? 1u : tpw_f > 256.0f ? 0u : (uint32_t)tpw_f;
        return JobCost{tiles, tpw};
    };
    const uint32_t g_tiles = ((uint32_t)tg.rows + 15) / 16, d_tiles = ((uint32_t)td.rows + 15) / 16;
    const JobCost gc = cost_model(g_tiles, g_grid, fused ? 1u : 2u), dc = cost_model(d_tiles, d_grid, 1u);
    const auto jobs_cost = [&](const JobCost &c, uint32_t e) {  // the jobs of the experts before e
        const uint32_t ka = first_kind_a[e], kb = first_kind_b[e];
        return (ka & 0xFFFFu) * c.job(group) + (ka >> 16) * c.job(1) + (kb & 0xFFFFu) * c.job(2) + (kb >> 16) * c.job(3);
    };
    const uint32_t g_total = jobs_cost(gc, n_experts), d_total = jobs_cost(dc, n_experts);
    if (!(slots <= 64 && n_experts <= 64)) {  // (the one-wavefront path has done this)
        for (uint32_t s = t; s < slots; s += blockDim.x) {
            const uint32_t e = ex[s];
            if (e < n_experts) by_expert[first_slot[e] + rank[s]] = (uint16_t)s;
        }
    }
    __syncthreads();
    // Ranks that are multiples of `group` open a job, the `group - 1` that follow join it.  The three descriptors of a
    // job (gate, up, down) are written by three different wavefronts: thread idx serves slot idx % span as kind idx / span.
    const uint32_t span = (slots + 63u) & ~63u;
    for (uint32_t idx = t; idx < 3 * span; idx += blockDim.x) {
        const uint32_t which = idx / span, s1 = idx - which * span;  // (span is a multiple of 64: `which` is the same in a wavefront)
        if (s1 >= slots || (which == 1 && fused)) continue;
        const uint32_t e = ex[s1], r = rank[s1];
        if (e >= n_experts || (r & gmask)) continue;
        const uint32_t jb = first_job[e] + (r >> gsh);
        const uint32_t nb = min(group, cnt[e] - r);
        uint32_t sm[4];
#pragma unroll
        for (uint32_t q = 0; q < 4; q++) sm[q] = q < nb ? by_expert[first_slot[e] + r + q] : s1;
        const uint32_t tok1 = s1 / k;
        const size_t gs = fused ? 2 * (size_t)inter : (size_t)inter;  // floats of gate/up results per slot and half
        const auto tok_off = [&](uint32_t q) { return ((int64_t)(sm[q] / k) - (int64_t)tok1) * (int64_t)hidden; };
        const auto slot_off = [&](uint32_t q, size_t unit) { return ((int64_t)sm[q] - (int64_t)s1) * (int64_t)unit; };
        // a job = the template's words with the fields that differ replaced, kept in registers as plain dwords
        // and stored 16 bytes at a time
        const auto emit = [&](GemvJob *dst, const GemvJob &tm, size_t w_off, size_t aux_off, size_t x_off, size_t out_off, bool x_by_token,
                              size_t out_unit, uint32_t pass_begin, const JobCost &c) {
            static_assert(sizeof(GemvJob) % 16 == 0 && alignof(GemvJob) == 8, "descriptor is a whole number of 16-byte stores");
            constexpr int N = sizeof(GemvJob) / 4;
            const uint32_t *src = reinterpret_cast<const uint32_t *>(&tm);
            uint32_t d[N];
#pragma unroll
            for (int i = 0; i < N; i++) d[i] = src[i];
            const auto put32 = [&](size_t byte_off, uint32_t v) { d[byte_off / 4] = v; };
            const auto put64 = [&](size_t byte_off, uint64_t v) { d[byte_off / 4] = (uint32_t)v; d[byte_off / 4 + 1] = (uint32_t)(v >> 32); };
            put64(offsetof(GemvJob, w), (uint64_t)(tm.w + w_off));
            put64(offsetof(GemvJob, aux), (uint64_t)(tm.aux + aux_off));
            put64(offsetof(GemvJob, x), (uint64_t)(tm.x + x_off));
            put64(offsetof(GemvJob, out), (uint64_t)(tm.out + out_off));
            if (tm.x_glu) put64(offsetof(GemvJob, x_glu), (uint64_t)(tm.x_glu + x_off));
            if (tm.bias) put64(offsetof(GemvJob, bias), (uint64_t)(tm.bias + (size_t)e * tm.bias_sel_stride));  // this expert's bias row
            put32(offsetof(GemvJob, batch), nb);
            put64(offsetof(GemvJob, x_stride), (uint64_t)(x_by_token ? tok_off(1) : slot_off(1, gs)));
            put64(offsetof(GemvJob, out_stride), (uint64_t)slot_off(1, out_unit));
            put64(offsetof(GemvJob, x_off), (uint64_t)(x_by_token ? tok_off(2) : slot_off(2, gs)));
            put64(offsetof(GemvJob, x_off) + 8, (uint64_t)(x_by_token ? tok_off(3) : slot_off(3, gs)));
            put64(offsetof(GemvJob, out_off), (uint64_t)slot_off(2, out_unit));
            put64(offsetof(GemvJob, out_off) + 8, (uint64_t)slot_off(3, out_unit));
            put32(offsetof(GemvJob, pass_begin), pass_begin);
            put32(offsetof(GemvJob, n_pass), c.job(nb));
            put32(offsetof(GemvJob, cpt), c.cpt(nb));
            put32(offsetof(GemvJob, su), c.su(nb));
            uint4 *o = reinterpret_cast<uint4 *>(dst);  // (the tables are 16-byte aligned)
#pragma unroll
            for (int i = 0; i < N / 4; i++) o[i] = make_uint4(d[4 * i], d[4 * i + 1], d[4 * i + 2], d[4 * i + 3]);
        };
        // (the earlier jobs of this expert are all full groups)
        const uint32_t g_begin = jobs_cost(gc, e) + (r >> gsh) * gc.job(group), d_begin = jobs_cost(dc, e) + (r >> gsh) * dc.job(group);
        if (gu_first) {
            // The first job of every workgroup's share (what a workgroup would otherwise find by bisection over the jobs'
            // pass ranges, a dependent load per step): workgroup b starts at pass floor(P b / grid), so this job, whose
            // passes are [begin, begin + cost), is the first of the workgroups from ceil(begin grid / P) up to that of its end.
            const bool dn = which == 2;
            const uint32_t grid = dn ? d_grid : g_grid;
            const uint64_t P = dn ? (uint64_t)d_total : (uint64_t)g_total * (fused ? 1u : 2u);
            const uint64_t begin = dn ? d_begin : (which == 1 ? g_total + g_begin : g_begin), end = begin + (dn ? dc.job(nb) : gc.job(nb));
            const uint32_t b0 = (uint32_t)((begin * grid + P - 1) / P), b1 = min(grid, (uint32_t)((end * grid + P - 1) / P));
            for (uint32_t bb = b0; bb < b1; bb++) (dn ? dn_first : gu_first)[bb] = (which == 1 ? n_jobs : 0u) + jb;
        }
        if (which == 0)
            emit(gu_table + jb, tg, (size_t)e * gu_w_stride, (size_t)e * gu_s_stride, (size_t)tok1 * hidden, (size_t)s1 * gs, true, gs, g_begin, gc);
        else if (which == 1)
            emit(gu_table + n_jobs + jb, tu, (size_t)e * gu_w_stride, (size_t)e * gu_s_stride, (size_t)tok1 * hidden, (size_t)s1 * gs, true, gs,
                 g_total + g_begin, gc);
        else
            emit(dn_table + jb, td, (size_t)e * dn_w_stride, (size_t)e * dn_s_stride, (size_t)s1 * gs, (size_t)s1 * hidden, false, hidden, d_begin, dc);
    }
    if (t == 0) {
        gu_hdr[0] = fused ? n_jobs : 2 * n_jobs; gu_hdr[1] = fused ? g_total : 2 * g_total;
        dn_hdr[0] = n_jobs; dn_hdr[1] = d_total;
    }
}

hipError_t moe_plan_launch(hipStream_t s, const float *logits, const float *router_bias, int policy, float *weights, uint32_t *experts,
                           uint32_t slots, uint32_t k, uint32_t n_experts, const GemvJob &tg,
                           const GemvJob &tu, const GemvJob &td, uint64_t gu_w_stride, uint64_t gu_s_stride, uint64_t dn_w_stride,
                           uint64_t dn_s_stride, uint32_t hidden, uint32_t inter, bool fused, uint32_t group, uint32_t g_grid, uint32_t d_grid, GemvJob *gu_table,
                           uint32_t *gu_hdr, GemvJob *dn_table, uint32_t *dn_hdr, uint32_t *gu_first, uint32_t *dn_first) {
    if (n_experts > 1024 || slots > 4096 || (group != 2 && group != 4)) return hipErrorInvalidValue;
    // (a wavefront per token while selecting: 16 wavefronts when the kernel routes)
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(logits ? 1024 : 256), 0, s, logits, router_bias, policy, weights, experts, slots, k, n_experts, tg, tu, td,
                       gu_w_stride, gu_s_stride,
                       dn_w_stride, dn_s_stride, hidden, inter, fused ? 1u : 0u, group, g_grid, d_grid, gu_table, gu_hdr, dn_table, dn_hdr, gu_first, dn_first);
    return hipGetLastError();
}

hipError_t router_select_launch(hipStream_t s, const float *logits, const float *bias, uint32_t tokens, uint32_t n_experts, uint32_t k,
                                int policy, uint32_t *experts, float *weights) {
    if (tokens == 0) return hipSuccess;
    hipLaunchKernelGGL(router_select_kernel, dim3(tokens), dim3(64), 0, s, logits, bias, n_experts, k, policy, experts, weights);
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
hipError_t expert_scale_launch(hipStream_t s, float *weights, const uint32_t *experts, const float *scale, uint32_t n, uint32_t n_scale) {
    if (n == 0 || n_scale == 0) return hipSuccess;
    hipLaunchKernelGGL(expert_scale_kernel, dim3((n + 255) / 256), dim3(256), 0, s, weights, experts, scale, n, n_scale);
    return hipGetLastError();
}

hipError_t quantize_rows_to_q8k_launch(hipStream_t s, const float *src, size_t src_stride, uint32_t src_cols, uint32_t cols, uint32_t rows,
                                       uint8_t *dst, size_t dst_stride) {
    if (rows == 0 || cols < 256) return hipSuccess;
    hipLaunchKernelGGL(quantize_rows_to_q8k_kernel, dim3((cols / 256 + 3) / 4, rows), dim3(256), 0, s, src, src_stride, src_cols, cols, dst, dst_stride);
    return hipGetLastError();
}
hipError_t moe_kq_act_q8k_launch(hipStream_t s, const float *g, const float *u, uint32_t inter, uint32_t inter_padded, uint32_t slots,
                                 const uint32_t *experts, uint32_t n_experts, const float *gub, int rule, float limit, float alpha, uint8_t *dst,
                                 size_t dst_stride) {
    if (slots == 0 || inter_padded < 256) return hipSuccess;
    hipLaunchKernelGGL(moe_kq_act_q8k_kernel, dim3((inter_padded / 256 + 3) / 4, slots), dim3(256), 0, s, g, u, inter, inter_padded, experts, n_experts,
                       gub, rule, limit, alpha, dst, dst_stride);
    return hipGetLastError();
}
hipError_t moe_kq_route_quant_launch(hipStream_t s, const float *logits, const float *bias, uint32_t tokens, uint32_t n_experts, uint32_t k, int policy,
                                     const float *scale, uint32_t *experts, float *weights, const float *src, size_t src_stride, uint32_t src_cols,
                                     uint32_t cols, uint8_t *dst, size_t dst_stride) {
    if (tokens == 0) return hipSuccess;
    hipLaunchKernelGGL(moe_kq_route_quant_kernel, dim3(tokens), dim3(256), 0, s, logits, bias, n_experts, k, policy, scale, experts, weights, src,
                       src_stride, src_cols, cols, dst, dst_stride);
    return hipGetLastError();
}
hipError_t pad_rows_f32_launch(hipStream_t s, const float *src, size_t src_stride, uint32_t src_cols, uint32_t cols, uint32_t rows, float *dst) {
    if (rows == 0 || cols == 0) return hipSuccess;
    hipLaunchKernelGGL(pad_rows_f32_kernel, dim3((cols + 255) / 256, rows), dim3(256), 0, s, src, src_stride, src_cols, cols, dst);
    return hipGetLastError();
}
hipError_t moe_act_f32_launch(hipStream_t s, const float *g, const float *u, uint32_t inter, uint32_t slots, const uint32_t *experts, uint32_t n_experts,
                              const float *gub, int rule, float limit, float alpha, float *act, size_t act_stride) {
    if (slots == 0 || inter == 0) return hipSuccess;
    hipLaunchKernelGGL(moe_act_f32_kernel, dim3((inter + 255) / 256, slots), dim3(256), 0, s, g, u, inter, experts, n_experts, gub, rule, limit, alpha,
                       act, act_stride);
    return hipGetLastError();
}
hipError_t weighted_sum_bias_launch(hipStream_t s, const float *d, const float *weights, const uint32_t *experts, uint32_t n_experts,
                                    const float *bias, float *out, uint32_t tokens, uint32_t k, uint32_t hidden) {
    if (tokens == 0 || hidden == 0) return hipSuccess;
    hipLaunchKernelGGL(weighted_sum_bias_kernel, dim3((hidden + 255) / 256, tokens), dim3(256), 0, s, d, weights, experts, n_experts, bias, out, k, hidden);
    return hipGetLastError();
}

hipError_t weighted_sum_launch(hipStream_t s, const float *d, const float *weights, const uint32_t *experts, uint32_t n_experts, float *out,
                               uint32_t tokens, uint32_t k, uint32_t hidden) {
    if (tokens == 0 || hidden == 0) return hipSuccess;
    hipLaunchKernelGGL(weighted_sum_kernel, dim3((hidden + 255) / 256, tokens), dim3(256), 0, s, d, weights, experts, n_experts, out, k, hidden);
    return hipGetLastError();
}

}  // namespace larql
