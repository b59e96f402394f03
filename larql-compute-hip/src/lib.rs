//! `HipBackend` — `larql_compute::ComputeBackend` on one AMD MI355X (gfx950).
//!
//! Every method forwards its host slices to one entry point of `liblarql_hip.so` and maps the return code to the
//! trait's `Option`: 0 → `Some`, "unsupported" / "refused shape" / device error → `None`, exactly where the CPU and
//! Metal backends answer `None` (crates/larql-compute/src/backend/quant_matvec.rs:42-371, matmul.rs:44-287).  The
//! library owns the device context, the upload staging, the registered weight regions and its own lock, so `&self`
//! methods are safe from several threads (`ComputeBackend: Send + Sync`, backend/mod.rs:49).
//!
//! The two required dense methods (`matmul`, `matmul_transb`) have no kernel in the library — they are prefill-time
//! f32 BLAS, outside the quantised decode path this backend accelerates — and go to `CpuBackend`, the same answer the
//! Metal backend gives below its flop threshold (larql-compute-metal/src/trait_impl/matmul.rs:13-31).
//! `DecodeBackend` keeps its defaults (`None`: "no fused decode, drive me per matvec"), which is what
//! `larql-inference` does for any backend whose `supports(Capability::DecodeToken)` is false.

mod ffi;

use std::any::Any;
use std::ffi::CStr;
use std::os::raw::c_int;
use std::ptr;

use larql_compute::{
    Activation, Capability, ComputeBackend, CpuBackend, DecodeBackend, MatMul, MoeExpertScalePolicy, MoeExpertScales, MoeFusedRowLayout,
    MoeGateRule, MoeLayerWeights, MoeTopKWeightPolicy, QuantFormat, QuantMatVec, SubmissionClock,
};
use ndarray::{Array2, ArrayView2};

/// One device context.  Dropping it frees the device copies of the registered regions.
pub struct HipBackend {
    ctx: *mut ffi::Ctx,
    name: String,
    cpu: CpuBackend,
}

// The library serialises entry points on the context's own mutex; the raw pointer is only a handle.
unsafe impl Send for HipBackend {}
unsafe impl Sync for HipBackend {}

/// The constructor a binary registers (crates/larql-cli/src/backend_select.rs:26-41).  `None` when device 0 is absent
/// or is not a gfx950 part, so a named `--backend hip` fails loudly instead of running on the CPU.
pub fn hip_backend() -> Option<HipBackend> {
    HipBackend::on_device(0)
}

/// One MoE layer resident on the device (see [`HipBackend::moe_layer`]).
pub struct HipMoeLayer<'a> {
    backend: &'a HipBackend,
    layer: *mut ffi::MoeLayer,
    hidden: usize,
    top_k: usize,
}

unsafe impl Send for HipMoeLayer<'_> {}
unsafe impl Sync for HipMoeLayer<'_> {}

impl HipMoeLayer<'_> {
    /// `moe_route_from_router_input` + the expert block (crates/larql-compute/src/cpu/ops/moe/mod.rs:149-186,
    /// forward.rs:201-270) for `tokens` rows: `router_in` and `x` are `[tokens, hidden]` (the router's and the experts'
    /// input as `MoeRoutingPolicy` derives them from the residual).  Returns the block's output and the route.
    pub fn forward(&self, router_in: &[f32], x: &[f32], tokens: usize) -> Option<(Vec<f32>, Vec<u32>, Vec<f32>)> {
        let n = tokens.checked_mul(self.hidden)?;
        if router_in.len() != n || x.len() != n {
            return None;
        }
        let cells = tokens.checked_mul(self.top_k)?;
        let (mut out, mut experts, mut weights) = (vec![0.0f32; n], vec![0u32; cells], vec![0.0f32; cells]);
        // SAFETY: the buffers have the sizes the library documents: [tokens, hidden] and [tokens, min(top_k, num_experts)].
        let rc = unsafe {
            ffi::larql_hip_moe_layer_forward(self.backend.ctx, self.layer, router_in.as_ptr(), x.as_ptr(), tokens,
                                             out.as_mut_ptr(), experts.as_mut_ptr(), weights.as_mut_ptr())
        };
        some_if_ok(rc, (out, experts, weights))
    }
}

impl HipMoeLayer<'_> {
    /// `cpu_moe_forward(h, moe, norm_offset, eps)` (crates/larql-compute/src/cpu/ops/moe/forward.rs:24-31) for one token,
    /// the router and the expert block on the device: the inputs are derived from the residual and the output is
    /// post-normed under `moe.routing_policy` by the reference's own functions (`moe_expert_input`, `moe_router_input`,
    /// `moe_post_expert_output`, cpu/ops/moe/mod.rs:55-200) — hidden-sized vector work that stays on the host, as it
    /// does in front of the Metal peer's expert dispatch.  `moe` must be the layer this handle was created from.
    pub fn forward_residual(&self, h: &[f32], moe: &MoeLayerWeights<'_>, norm_offset: f32, eps: f32) -> Option<Vec<f32>> {
        use larql_compute::cpu::ops::moe::{moe_expert_input, moe_post_expert_output, moe_router_input};
        if h.len() != self.hidden {
            return None;
        }
        let expert_input = moe_expert_input(h, moe, norm_offset, eps);
        let router_in = moe_router_input(h, &expert_input, moe, norm_offset, eps);
        let (out, _, _) = self.forward(&router_in, &expert_input, 1)?;
        Some(moe_post_expert_output(&out, moe, norm_offset, eps))
    }
}

impl Drop for HipMoeLayer<'_> {
    fn drop(&mut self) {
        // SAFETY: the handle came from larql_hip_moe_layer_create on this context and is dropped once.
        unsafe { ffi::larql_hip_moe_layer_destroy(self.backend.ctx, self.layer) }
    }
}

fn format_code(format: QuantFormat) -> c_int {
    match format {
        QuantFormat::Q4_0 => ffi::FMT_Q4_0,
        QuantFormat::Q4_K => ffi::FMT_Q4_K,
        QuantFormat::Q4_KF => ffi::FMT_Q4_KF,
        QuantFormat::Q5_K => ffi::FMT_Q5_K,
        QuantFormat::Q6_K => ffi::FMT_Q6_K,
        QuantFormat::Q8_0 => ffi::FMT_Q8_0,
        QuantFormat::BF16 => ffi::FMT_BF16,
        QuantFormat::F16 => ffi::FMT_F16,
        QuantFormat::F32 => ffi::FMT_F32,
        QuantFormat::I2S => ffi::FMT_I2S,
        QuantFormat::MXFP4 => ffi::FMT_MXFP4,
    }
}

fn some_if_ok<T>(rc: c_int, value: T) -> Option<T> {
    if rc == ffi::OK {
        Some(value)
    } else {
        None
    }
}

/// The winners the library can order per row (`kTopkMaxK`).
const TOP_K_MAX: usize = 16384;

/// A caller may pass a very large K to mean "all": K is clamped to the number of candidates BEFORE any buffer is sized
/// from it, and a K the library does not serve answers `None` here instead of an allocation failure.
fn clamp_top_k(top_k: usize, candidates: usize) -> Option<usize> {
    let k = top_k.min(candidates);
    if k > TOP_K_MAX {
        None
    } else {
        Some(k)
    }
}

fn pairs(idx: Vec<u32>, score: Vec<f32>, n: usize) -> Vec<(u32, f32)> {
    idx.into_iter().zip(score).take(n).collect()
}

impl HipBackend {
    pub fn on_device(device: i32) -> Option<Self> {
        let mut ctx: *mut ffi::Ctx = ptr::null_mut();
        // SAFETY: `ctx` is a valid out-pointer; the library writes it only on success.
        let rc = unsafe { ffi::larql_hip_create(&mut ctx, device as c_int) };
        if rc != ffi::OK || ctx.is_null() {
            return None;
        }
        // SAFETY: the library returns a NUL-terminated string that lives as long as the context.
        let name = unsafe { CStr::from_ptr(ffi::larql_hip_name(ctx)) }.to_string_lossy().into_owned();
        Some(Self { ctx, name, cpu: CpuBackend })
    }

    /// Text of the last device error on this context ("" when none).
    pub fn last_error(&self) -> String {
        // SAFETY: as in `on_device`.
        unsafe { CStr::from_ptr(ffi::larql_hip_last_error(self.ctx)) }.to_string_lossy().into_owned()
    }

    /// Drops the device copies of every registered region (for a model swap inside one process).
    pub fn clear_weight_regions(&self) {
        // SAFETY: the handle is live for `&self`.
        unsafe { ffi::larql_hip_clear_weight_regions(self.ctx) };
    }

    /// ggml Q8_0 (34-byte blocks) gemv — `KQuant::gemv`'s Q8_0 arm
    /// (crates/larql-vindex/src/format/vindex3/represent/kquant.rs:285-298).
    pub fn q8_0_gemv(&self, blocks: &[u8], x: &[f32], n: usize, k: usize) -> Option<Vec<f32>> {
        let mut out = vec![0.0f32; n];
        // SAFETY: every pointer comes from a live slice and travels with its length; `out` holds `n` floats.
        let rc = unsafe {
            ffi::larql_hip_q8_0_gemv(self.ctx, blocks.as_ptr(), blocks.len(), x.as_ptr(), x.len(), n, k, out.as_mut_ptr())
        };
        some_if_ok(rc, out)
    }

    /// lm_head KNN over a ggml Q8_0 head with the selection on the device
    /// (crates/larql-vindex/src/index/storage/lm_head/knn.rs:126-185, top_k_sorted :315-386).
    pub fn q8_0_gemv_topk(&self, blocks: &[u8], x: &[f32], n: usize, k: usize, top_k: usize) -> Option<Vec<(u32, f32)>> {
        let top_k = clamp_top_k(top_k, n)?;
        let (mut idx, mut score, mut got) = (vec![0u32; top_k], vec![0.0f32; top_k], 0usize);
        // SAFETY: `idx` / `score` hold top_k entries, what the library copies back; `got` says how many are hits.
        let rc = unsafe {
            ffi::larql_hip_q8_0_gemv_topk(self.ctx, blocks.as_ptr(), blocks.len(), x.as_ptr(), x.len(), n, k, top_k,
                                          idx.as_mut_ptr(), score.as_mut_ptr(), &mut got)
        };
        some_if_ok(rc, ()).map(|_| pairs(idx, score, got))
    }

    /// `VectorIndex::gate_knn` / `gate_knn_batch` with `top_k_by_abs` on the device
    /// (crates/larql-vindex/src/index/compute/gate_knn/dispatch.rs:22-121, mod.rs:50-108).  `x` is
    /// `[batch, hidden]`; the result has one hit list per position.
    pub fn gate_knn(&self, format: QuantFormat, gate: &[u8], x: &[f32], batch: usize, n_features: usize, hidden: usize,
                    top_k: usize) -> Option<Vec<Vec<(u32, f32)>>> {
        if Some(x.len()) != batch.checked_mul(hidden) {
            return None;
        }
        let top_k = clamp_top_k(top_k, n_features)?;
        let cells = batch.checked_mul(top_k)?;
        let (mut idx, mut score, mut got) = (vec![0u32; cells], vec![0.0f32; cells], vec![0usize; batch]);
        // SAFETY: the outputs are [batch, top_k] and the counts [batch], as the library documents; `x` was checked above.
        let rc = unsafe {
            ffi::larql_hip_gate_knn(self.ctx, format_code(format), gate.as_ptr(), gate.len(), x.as_ptr(), batch, n_features,
                                    hidden, top_k, idx.as_mut_ptr(), score.as_mut_ptr(), got.as_mut_ptr())
        };
        some_if_ok(rc, ()).map(|_| {
            (0..batch)
                .map(|b| (0..got[b].min(top_k)).map(|i| (idx[b * top_k + i], score[b * top_k + i])).collect())
                .collect()
        })
    }

    /// A MoE layer made resident from `MoeLayerWeights` (crates/larql-compute/src/pipeline/moe.rs:469-541): the
    /// per-expert slices and their paired exponent streams go up expert by expert, wherever their mmap ranges lie.
    /// Served: an MXFP4 bank with `Paired` scales under `ClampedGlu` (a native GPT-OSS bank), and a Q4_K / Q6_K bank with
    /// `Inline` scales and `ContiguousHalves` rows under any `MoeGateRule` (the per-layer k-quant files of Gemma 4
    /// 26B-A4B: `cpu_moe_forward`'s integer path, crates/larql-compute/src/cpu/ops/moe/forward.rs:160-330), and a BF16 /
    /// F16 / F32 bank on that function's f32 arm (forward.rs:246-290).  `None` where
    /// this backend has no kernel for the layer (other formats or rules, more than 256 experts, top-k above 8) — the
    /// caller keeps `cpu_moe_forward`.
    pub fn moe_layer<'a>(&'a self, moe: &MoeLayerWeights<'_>, hidden: usize) -> Option<HipMoeLayer<'a>> {
        // ClampedGlu on any bank, every rule on a k-quant or float bank.  `Activation::ReLU` has no gate/up kernel on the
        // CPU paths either (it panics there: pipeline/enums.rs:79-88); here it is `None`.
        let gelu = |a: Activation| match a {
            Activation::GeluTanh | Activation::GeluExact => Some(true),
            Activation::Silu => Some(false),
            _ => None,
        };
        let (gate_rule, limit, alpha) = match moe.gate_rule {
            MoeGateRule::ClampedGlu { limit, alpha } => (ffi::MOE_GATE_CLAMPED_GLU, limit, alpha),
            MoeGateRule::Gated(a) => (if gelu(a)? { ffi::MOE_GATE_GELU_TANH } else { ffi::MOE_GATE_SILU }, 0.0, 0.0),
            MoeGateRule::SituGlu { beta, linear_beta } => (ffi::MOE_GATE_SITU_GLU, beta, linear_beta.unwrap_or(0.0)),
            MoeGateRule::ClampedGated { limit, activation } => {
                (if gelu(activation)? { ffi::MOE_GATE_CLAMPED_GELU_TANH } else { ffi::MOE_GATE_CLAMPED_SILU }, limit, 0.0)
            }
        };
        let (sg, sd): (Vec<&[u8]>, Vec<&[u8]>) = match &moe.expert_scales {
            MoeExpertScales::Paired { gate_up, down } => (gate_up.clone(), down.clone()),
            MoeExpertScales::Inline => (Vec::new(), Vec::new()),
        };
        let n = moe.num_experts;
        if moe.experts_gate_up.len() != n || moe.experts_down.len() != n || moe.router_proj.len() != n.checked_mul(hidden)? {
            return None;
        }
        if moe.expert_scales.is_paired() && (sg.len() != n || sd.len() != n) {
            return None;
        }
        let ptrs = |v: &[&[u8]]| v.iter().map(|s| s.as_ptr()).collect::<Vec<*const u8>>();
        let lens = |v: &[&[u8]]| v.iter().map(|s| s.len()).collect::<Vec<usize>>();
        let (gp, gl, dp, dl) = (ptrs(&moe.experts_gate_up), lens(&moe.experts_gate_up), ptrs(&moe.experts_down), lens(&moe.experts_down));
        let (sgp, sgl, sdp, sdl) = (ptrs(&sg), lens(&sg), ptrs(&sd), lens(&sd));
        let opt = |s: &[f32]| if s.is_empty() { ptr::null() } else { s.as_ptr() };
        let w = ffi::MoeLayerWeights {
            num_experts: n,
            top_k: moe.top_k,
            hidden,
            intermediate_size: moe.intermediate_size,
            expert_data_format: format_code(moe.expert_data_format),
            fused_row_layout: match moe.fused_row_layout {
                MoeFusedRowLayout::Interleaved => ffi::MOE_ROWS_INTERLEAVED,
                MoeFusedRowLayout::ContiguousHalves => ffi::MOE_ROWS_CONTIGUOUS_HALVES,
            },
            expert_scales: if moe.expert_scales.is_paired() { ffi::MOE_SCALES_PAIRED } else { ffi::MOE_SCALES_INLINE },
            experts_gate_up: gp.as_ptr(),
            experts_gate_up_len: gl.as_ptr(),
            experts_down: dp.as_ptr(),
            experts_down_len: dl.as_ptr(),
            scales_gate_up: if sgp.is_empty() { ptr::null() } else { sgp.as_ptr() },
            scales_gate_up_len: if sgl.is_empty() { ptr::null() } else { sgl.as_ptr() },
            scales_down: if sdp.is_empty() { ptr::null() } else { sdp.as_ptr() },
            scales_down_len: if sdl.is_empty() { ptr::null() } else { sdl.as_ptr() },
            router_proj: moe.router_proj.as_ptr(),
            router_bias: opt(moe.router_bias),
            experts_gate_up_bias: opt(moe.experts_gate_up_bias),
            experts_down_bias: opt(moe.experts_down_bias),
            router_per_expert_scale: opt(moe.router_per_expert_scale),
            renormalized_softmax: (moe.routing_policy.selected_weight == MoeTopKWeightPolicy::RenormalizedSoftmax) as c_int,
            per_expert_scale: (moe.routing_policy.expert_scale == MoeExpertScalePolicy::PerExpert) as c_int,
            glu_limit: limit,
            glu_alpha: alpha,
            gate_rule,
        };
        let mut layer: *mut ffi::MoeLayer = ptr::null_mut();
        // SAFETY: every table holds `n` entries that outlive the call; the library copies the bytes before it returns.
        let rc = unsafe { ffi::larql_hip_moe_layer_create(self.ctx, &w, &mut layer) };
        if rc != ffi::OK || layer.is_null() {
            return None;
        }
        Some(HipMoeLayer { backend: self, layer, hidden, top_k: moe.top_k.min(n) })
    }

    /// `gate_scores_batch_backend` (gate_knn/scores_batch.rs:30-57): the full `[batch, n_features]` score matrix.
    pub fn gate_scores(&self, format: QuantFormat, gate: &[u8], x: &[f32], batch: usize, n_features: usize,
                       hidden: usize) -> Option<Array2<f32>> {
        if x.len() != batch * hidden {
            return None;
        }
        let mut out = vec![0.0f32; batch * n_features];
        // SAFETY: `out` is [batch, n_features].
        let rc = unsafe {
            ffi::larql_hip_gate_scores(self.ctx, format_code(format), gate.as_ptr(), gate.len(), x.as_ptr(), batch,
                                       n_features, hidden, out.as_mut_ptr())
        };
        some_if_ok(rc, ()).and_then(|_| Array2::from_shape_vec((batch, n_features), out).ok())
    }

    fn dense_multi(&self, bf16: bool, weights: &[(&[u8], usize, usize)], x: &[f32]) -> Option<Vec<Vec<f32>>> {
        let w: Vec<*const u8> = weights.iter().map(|t| t.0.as_ptr()).collect();
        let w_len: Vec<usize> = weights.iter().map(|t| t.0.len()).collect();
        let n: Vec<usize> = weights.iter().map(|t| t.1).collect();
        let k: Vec<usize> = weights.iter().map(|t| t.2).collect();
        let mut outs: Vec<Vec<f32>> = n.iter().map(|&rows| vec![0.0f32; rows]).collect();
        let out_ptrs: Vec<*mut f32> = outs.iter_mut().map(|o| o.as_mut_ptr()).collect();
        // SAFETY: the five tables have `weights.len()` entries; each output holds n[i] floats.
        let rc = unsafe {
            if bf16 {
                ffi::larql_hip_bf16_gemv_multi(self.ctx, weights.len(), w.as_ptr(), w_len.as_ptr(), n.as_ptr(), k.as_ptr(),
                                               x.as_ptr(), x.len(), out_ptrs.as_ptr())
            } else {
                ffi::larql_hip_f16_gemv_multi(self.ctx, weights.len(), w.as_ptr(), w_len.as_ptr(), n.as_ptr(), k.as_ptr(),
                                              x.as_ptr(), x.len(), out_ptrs.as_ptr())
            }
        };
        some_if_ok(rc, outs)
    }

    fn dense_half(&self, bf16: bool, w: &[u8], x: &[f32], n: usize, k: usize, force: bool) -> Option<Vec<f32>> {
        // the peers answer None unless x is exactly one row long (larql-compute-metal/src/trait_impl/matmul.rs:53-88)
        if x.len() != k {
            return None;
        }
        let mut out = vec![0.0f32; n];
        // SAFETY: slices with their lengths; `out` holds `n` floats.
        let rc = unsafe {
            if bf16 {
                ffi::larql_hip_bf16_gemv(self.ctx, w.as_ptr(), w.len(), x.as_ptr(), x.len(), n, k, out.as_mut_ptr(), force as c_int)
            } else {
                ffi::larql_hip_f16_gemv(self.ctx, w.as_ptr(), w.len(), x.as_ptr(), x.len(), n, k, out.as_mut_ptr(), force as c_int)
            }
        };
        some_if_ok(rc, out)
    }

    fn dense_f32(&self, w: ArrayView2<f32>, x: &[f32], force: bool) -> Option<Vec<f32>> {
        let (n, k) = (w.shape()[0], w.shape()[1]);
        if x.len() != k {
            return None;
        }
        // a transposed or strided view is copied once into row-major order; the vindex hands contiguous mmaps
        let w = w.as_standard_layout();
        let flat = w.as_slice()?;
        let mut out = vec![0.0f32; n];
        // SAFETY: `flat` is n*k contiguous floats; w_len is in bytes.
        let rc = unsafe {
            ffi::larql_hip_f32_gemv(self.ctx, flat.as_ptr(), flat.len() * 4, x.as_ptr(), x.len(), n, k, out.as_mut_ptr(),
                                    force as c_int)
        };
        some_if_ok(rc, out)
    }
}

impl Drop for HipBackend {
    fn drop(&mut self) {
        // SAFETY: created by larql_hip_create, destroyed once.
        unsafe { ffi::larql_hip_destroy(self.ctx) };
    }
}

impl MatMul for HipBackend {
    fn matmul(&self, a: ArrayView2<f32>, b: ArrayView2<f32>) -> Array2<f32> {
        self.cpu.matmul(a, b)
    }

    fn matmul_transb(&self, a: ArrayView2<f32>, b: ArrayView2<f32>) -> Array2<f32> {
        self.cpu.matmul_transb(a, b)
    }

    // matmul_batch keeps the trait default (a loop over the two methods above).

    fn f32_gemv(&self, w: ArrayView2<f32>, x: &[f32]) -> Option<Vec<f32>> {
        self.dense_f32(w, x, false)
    }

    fn f32_gemv_force(&self, w: ArrayView2<f32>, x: &[f32]) -> Option<Vec<f32>> {
        self.dense_f32(w, x, true)
    }

    fn f16_gemv(&self, w_f16: &[u8], x: &[f32], n: usize, k: usize) -> Option<Vec<f32>> {
        self.dense_half(false, w_f16, x, n, k, false)
    }

    fn f16_gemv_force(&self, w_f16: &[u8], x: &[f32], n: usize, k: usize) -> Option<Vec<f32>> {
        self.dense_half(false, w_f16, x, n, k, true)
    }

    fn bf16_gemv(&self, w_bf16: &[u8], x: &[f32], n: usize, k: usize) -> Option<Vec<f32>> {
        self.dense_half(true, w_bf16, x, n, k, false)
    }

    fn bf16_gemv_force(&self, w_bf16: &[u8], x: &[f32], n: usize, k: usize) -> Option<Vec<f32>> {
        self.dense_half(true, w_bf16, x, n, k, true)
    }

    fn bf16_gemv_multi(&self, weights: &[(&[u8], usize, usize)], x: &[f32]) -> Option<Vec<Vec<f32>>> {
        self.dense_multi(true, weights, x)
    }

    fn f16_gemv_multi(&self, weights: &[(&[u8], usize, usize)], x: &[f32]) -> Option<Vec<Vec<f32>>> {
        self.dense_multi(false, weights, x)
    }

    // f32_gemv_topk1 / f16_gemv_topk1 / f16_gemv_topk keep the trait default (None): the library selects on the device
    // for Q4_K and ggml Q8_0 heads only; a dense head's caller gets the score vector and runs its own top_k_sorted.
    //
    // wire_resident keeps the default no-op on purpose.  It promises nothing about the buffers' lifetime
    // (matmul.rs:196-207), while a registered region is looked up by address on every later call: registering bytes
    // that may be freed and reused would serve stale weights.  Residency here is register_weight_region's job.

    fn submission_clock(&self) -> Option<SubmissionClock> {
        let mut c = ffi::Clock::default();
        // SAFETY: `c` is a valid out-pointer.
        let rc = unsafe { ffi::larql_hip_get_submission_clock(self.ctx, &mut c) };
        some_if_ok(rc, SubmissionClock {
            submissions: c.submissions,
            commit_to_done_nanos: c.commit_to_done_nanos,
            gpu_nanos: c.gpu_nanos,
        })
    }

    fn mxfp4_gemv(&self, packed: &[u8], scales: &[u8], x: &[f32], n: usize, k: usize) -> Option<Vec<f32>> {
        let mut out = vec![0.0f32; n];
        // SAFETY: slices with their lengths; `out` holds `n` floats.
        let rc = unsafe {
            ffi::larql_hip_mxfp4_gemv(self.ctx, packed.as_ptr(), packed.len(), scales.as_ptr(), scales.len(), x.as_ptr(),
                                      x.len(), n, k, out.as_mut_ptr())
        };
        some_if_ok(rc, out)
    }

    fn mxfp4_gemv_multi(&self, weights: &[(&[u8], &[u8], usize, usize)], x: &[f32]) -> Option<Vec<Vec<f32>>> {
        let packed: Vec<*const u8> = weights.iter().map(|t| t.0.as_ptr()).collect();
        let packed_len: Vec<usize> = weights.iter().map(|t| t.0.len()).collect();
        let scales: Vec<*const u8> = weights.iter().map(|t| t.1.as_ptr()).collect();
        let scales_len: Vec<usize> = weights.iter().map(|t| t.1.len()).collect();
        let n: Vec<usize> = weights.iter().map(|t| t.2).collect();
        let k: Vec<usize> = weights.iter().map(|t| t.3).collect();
        let mut outs: Vec<Vec<f32>> = n.iter().map(|&rows| vec![0.0f32; rows]).collect();
        let out_ptrs: Vec<*mut f32> = outs.iter_mut().map(|o| o.as_mut_ptr()).collect();
        // SAFETY: the tables have `weights.len()` entries; each output holds n[i] floats.
        let rc = unsafe {
            ffi::larql_hip_mxfp4_gemv_multi(self.ctx, weights.len(), packed.as_ptr(), packed_len.as_ptr(), scales.as_ptr(),
                                            scales_len.as_ptr(), n.as_ptr(), k.as_ptr(), x.as_ptr(), x.len(),
                                            out_ptrs.as_ptr())
        };
        some_if_ok(rc, outs)
    }

    // nvfp4_gemv / nvfp4_gemv_multi keep the trait default (None): the library has no NVFP4 kernel.
}

impl QuantMatVec for HipBackend {
    fn quant_matvec(&self, format: QuantFormat, weights: &[u8], x: &[f32], num_rows: usize, hidden: usize)
                    -> Option<Vec<f32>> {
        let mut out = vec![0.0f32; num_rows];
        // SAFETY: slices with their lengths; `out` holds `num_rows` floats.  One call, so the Q4_0 arm quantises x on
        // the device instead of on the host as the trait default does (quant_matvec.rs:66-69).
        let rc = unsafe {
            ffi::larql_hip_quant_matvec(self.ctx, format_code(format), weights.as_ptr(), weights.len(), x.as_ptr(), x.len(),
                                        num_rows, hidden, out.as_mut_ptr())
        };
        some_if_ok(rc, out)
    }

    fn quant_matvec_q8_input(&self, format: QuantFormat, weights: &[u8], q8_x: &[i8], q8_scales: &[f32], num_rows: usize,
                             hidden: usize) -> Option<Vec<f32>> {
        let mut out = vec![0.0f32; num_rows];
        // SAFETY: as above.
        let rc = unsafe {
            ffi::larql_hip_quant_matvec_q8_input(self.ctx, format_code(format), weights.as_ptr(), weights.len(), q8_x.as_ptr(),
                                                 q8_x.len(), q8_scales.as_ptr(), q8_scales.len(), num_rows, hidden,
                                                 out.as_mut_ptr())
        };
        some_if_ok(rc, out)
    }

    fn q4_matvec(&self, q4_data: &[u8], q8_x: &[i8], q8_scales: &[f32], num_rows: usize, hidden: usize) -> Option<Vec<f32>> {
        let mut out = vec![0.0f32; num_rows];
        // SAFETY: as above.
        let rc = unsafe {
            ffi::larql_hip_q4_matvec(self.ctx, q4_data.as_ptr(), q4_data.len(), q8_x.as_ptr(), q8_x.len(), q8_scales.as_ptr(),
                                     q8_scales.len(), num_rows, hidden, out.as_mut_ptr())
        };
        some_if_ok(rc, out)
    }

    // q8_matvec, q4_matvec_topk1, q4_matvec_topk, q4_vecmat, q4_matvec_pair_batch, q4k_matvec_stride32 and
    // ternary_matvec keep the trait default (None), as on the CPU backend: the trait's Q8_0 layout, the Q4_0
    // vecmat / pair-batch shapes, the 148-byte stride-32 variant and BitNet have no kernel in the library.

    fn q4k_matvec(&self, q4k_data: &[u8], x: &[f32], num_rows: usize, hidden: usize) -> Option<Vec<f32>> {
        let mut out = vec![0.0f32; num_rows];
        // SAFETY: as above.
        let rc = unsafe {
            ffi::larql_hip_q4k_matvec(self.ctx, q4k_data.as_ptr(), q4k_data.len(), x.as_ptr(), x.len(), num_rows, hidden,
                                      out.as_mut_ptr(), out.len())
        };
        some_if_ok(rc, out)
    }

    fn q4k_matvec_topk(&self, q4k_data: &[u8], x: &[f32], num_rows: usize, hidden: usize, top_k: usize)
                       -> Option<Vec<(u32, f32)>> {
        let top_k = clamp_top_k(top_k, num_rows)?;
        let (mut idx, mut score, mut got) = (vec![0u32; top_k], vec![0.0f32; top_k], 0usize);
        // SAFETY: `idx` / `score` hold top_k entries, what the library copies back; `got` says how many are hits.
        let rc = unsafe {
            ffi::larql_hip_q4k_matvec_topk(self.ctx, q4k_data.as_ptr(), q4k_data.len(), x.as_ptr(), x.len(), num_rows, hidden,
                                           top_k, idx.as_mut_ptr(), score.as_mut_ptr(), &mut got)
        };
        some_if_ok(rc, ()).map(|_| pairs(idx, score, got))
    }

    fn q4k_dual_matvec(&self, q4k_a: &[u8], q4k_b: &[u8], x: &[f32], num_rows: usize, hidden: usize)
                       -> Option<(Vec<f32>, Vec<f32>)> {
        let (mut a, mut b) = (vec![0.0f32; num_rows], vec![0.0f32; num_rows]);
        // SAFETY: as above; both outputs hold `num_rows` floats.
        let rc = unsafe {
            ffi::larql_hip_q4k_dual_matvec(self.ctx, q4k_a.as_ptr(), q4k_a.len(), q4k_b.as_ptr(), q4k_b.len(), x.as_ptr(),
                                           x.len(), num_rows, hidden, a.as_mut_ptr(), b.as_mut_ptr(), num_rows)
        };
        some_if_ok(rc, (a, b))
    }

    fn q4k_matmul(&self, q4k_data: &[u8], x: &[f32], num_rows: usize, hidden: usize, seq_len: usize) -> Option<Vec<f32>> {
        let mut out = vec![0.0f32; seq_len * num_rows];
        // SAFETY: `out` is [seq_len, num_rows].
        let rc = unsafe {
            ffi::larql_hip_q4k_matmul(self.ctx, q4k_data.as_ptr(), q4k_data.len(), x.as_ptr(), x.len(), num_rows, hidden,
                                      seq_len, out.as_mut_ptr(), out.len())
        };
        some_if_ok(rc, out)
    }

    fn q6k_matvec(&self, q6k_data: &[u8], x: &[f32], num_rows: usize, hidden: usize) -> Option<Vec<f32>> {
        let mut out = vec![0.0f32; num_rows];
        // SAFETY: as above.
        let rc = unsafe {
            ffi::larql_hip_q6k_matvec(self.ctx, q6k_data.as_ptr(), q6k_data.len(), x.as_ptr(), x.len(), num_rows, hidden,
                                      out.as_mut_ptr())
        };
        some_if_ok(rc, out)
    }

    fn supports_quant(&self, format: QuantFormat) -> bool {
        // SAFETY: the handle is live for `&self`.
        unsafe { ffi::larql_hip_supports_quant(self.ctx, format_code(format)) != 0 }
    }
}

/// No fused token pipeline: every method keeps its default (`None`), so `larql-inference` drives this backend one
/// matvec at a time, as it does the CPU backend (crates/larql-compute/src/backend/decode.rs:219).
impl DecodeBackend for HipBackend {}

impl ComputeBackend for HipBackend {
    fn name(&self) -> &str {
        &self.name
    }

    fn device_info(&self) -> String {
        // SAFETY: as in `on_device`.
        unsafe { CStr::from_ptr(ffi::larql_hip_device_info(self.ctx)) }.to_string_lossy().into_owned()
    }

    fn supports(&self, cap: Capability) -> bool {
        let code = match cap {
            Capability::F32Gemv => ffi::CAP_F32_GEMV,
            Capability::F16Gemv => ffi::CAP_F16_GEMV,
            Capability::QuantMatVec => ffi::CAP_QUANT_MATVEC,
            _ => return false,
        };
        // SAFETY: the handle is live for `&self`.
        unsafe { ffi::larql_hip_supports(self.ctx, code) != 0 }
    }

    fn register_weight_region(&self, region: &[u8]) {
        // The trait's contract (backend/mod.rs:68-83) is the library's: the region never moves and outlives the
        // backend (the vindex's mmaps do).  A failed upload leaves the region unregistered and later calls stage the
        // weights per call, so the result is the same bytes either way.
        // SAFETY: `region` is a live slice.
        unsafe { ffi::larql_hip_register_weight_region(self.ctx, region.as_ptr(), region.len()) };
    }

    fn seal_weight_regions(&self) {
        // SAFETY: the handle is live for `&self`.
        unsafe { ffi::larql_hip_seal_weight_regions(self.ctx) };
    }

    fn as_any(&self) -> &dyn Any {
        self
    }
}
