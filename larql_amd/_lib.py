"""ctypes binding of liblarql_hip.so (the C ABI of include/larql_hip.h).

The library must have been built in-tree (larql_amd/build.py); there is no
fallback of any kind: a missing library is an ImportError, a missing GPU is a
RuntimeError from HipBackend().
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liblarql_hip.so")

OK, UNSUPPORTED, REFUSED_SHAPE = 0, 1, 2
E_DEVICE, E_NO_DEVICE, E_ARG, E_NAN = -1, -2, -3, -4

FMT_Q4_0, FMT_Q4_K, FMT_Q4_KF, FMT_Q5_K, FMT_Q6_K, FMT_Q8_0 = 0, 1, 2, 3, 4, 5
FMT_BF16, FMT_F16, FMT_F32, FMT_I2S, FMT_MXFP4, FMT_GGML_Q8_0, FMT_Q4_K_Q8K, FMT_Q6_K_Q8K = 6, 7, 8, 9, 10, 100, 101, 102
CAP_F32_GEMV, CAP_F16_GEMV, CAP_QUANT_MATVEC = 0, 1, 2

vp, sz, ci = C.c_void_p, C.c_size_t, C.c_int
u64 = C.c_uint64


class SubmissionClock(C.Structure):
    _fields_ = [("submissions", u64), ("commit_to_done_nanos", u64), ("gpu_nanos", u64)]


class Mxfp4Experts(C.Structure):
    _fields_ = [("gate_packed", vp), ("gate_scales", vp), ("up_packed", vp), ("up_scales", vp), ("down_packed", vp),
                ("down_scales", vp), ("n_experts", sz), ("hidden", sz), ("inter", sz), ("limit", C.c_float),
                ("alpha", C.c_float), ("gate_up_interleaved", C.c_int), ("router_bias", vp), ("gate_up_bias", vp), ("down_bias", vp)]


MOE_SCALES_INLINE, MOE_SCALES_PAIRED = 0, 1
MOE_GATE_CLAMPED_GLU, MOE_GATE_GELU_TANH, MOE_GATE_SILU, MOE_GATE_SITU_GLU, MOE_GATE_CLAMPED_GELU_TANH, MOE_GATE_CLAMPED_SILU = 0, 1, 2, 3, 4, 5
MOE_ROWS_CONTIGUOUS_HALVES, MOE_ROWS_INTERLEAVED = 0, 1


class MoeLayerWeights(C.Structure):
    """larql_hip_moe_layer_weights (MoeLayerWeights, larql-compute/src/pipeline/moe.rs:469-541)."""
    _fields_ = [("num_experts", sz), ("top_k", sz), ("hidden", sz), ("intermediate_size", sz), ("expert_data_format", ci),
                ("fused_row_layout", ci), ("expert_scales", ci), ("experts_gate_up", C.POINTER(vp)), ("experts_gate_up_len", C.POINTER(sz)),
                ("experts_down", C.POINTER(vp)), ("experts_down_len", C.POINTER(sz)), ("scales_gate_up", C.POINTER(vp)),
                ("scales_gate_up_len", C.POINTER(sz)), ("scales_down", C.POINTER(vp)), ("scales_down_len", C.POINTER(sz)),
                ("router_proj", vp), ("router_bias", vp), ("experts_gate_up_bias", vp), ("experts_down_bias", vp),
                ("router_per_expert_scale", vp), ("renormalized_softmax", ci), ("per_expert_scale", ci), ("glu_limit", C.c_float),
                ("glu_alpha", C.c_float), ("gate_rule", ci)]


class MatvecJob(C.Structure):
    _fields_ = [("format", C.c_int32), ("reserved", C.c_int32), ("w", vp), ("aux", vp), ("x", vp),
                ("out", vp), ("rows", u64), ("k", u64)]


# name -> (restype, argtypes): every symbol include/larql_hip.h declares
SIGNATURES = {
    "larql_hip_create": (ci, [C.POINTER(vp), ci]),
    "larql_hip_destroy": (None, [vp]),
    "larql_hip_name": (C.c_char_p, [vp]),
    "larql_hip_device_info": (C.c_char_p, [vp]),
    "larql_hip_supports_quant": (ci, [vp, ci]),
    "larql_hip_supports": (ci, [vp, ci]),
    "larql_hip_last_error": (C.c_char_p, [vp]),
    "larql_hip_register_weight_region": (ci, [vp, vp, sz]),
    "larql_hip_seal_weight_regions": (ci, [vp]),
    "larql_hip_clear_weight_regions": (ci, [vp]),
    "larql_hip_get_submission_clock": (ci, [vp, C.POINTER(SubmissionClock)]),
    "larql_hip_q4k_matvec": (ci, [vp, vp, sz, vp, sz, sz, sz, vp, sz]),
    "larql_hip_q6k_matvec": (ci, [vp, vp, sz, vp, sz, sz, sz, vp]),
    "larql_hip_quantize_x_to_q8k": (ci, [vp, vp, sz, vp, vp, vp]),
    "larql_hip_q4k_q8k_matvec": (ci, [vp, vp, sz, vp, sz, vp, vp, sz, sz, vp, sz]),
    "larql_hip_q6k_q8k_matvec": (ci, [vp, vp, sz, vp, sz, vp, sz, sz, vp, sz]),
    "larql_hip_q4k_q8k_gate_up": (ci, [vp, vp, sz, vp, sz, vp, sz, vp, vp, sz, sz, vp, vp, sz]),
    "larql_hip_q4k_q8k_gemm": (ci, [vp, vp, sz, vp, vp, vp, sz, sz, sz, vp, sz]),
    "larql_hip_q8k_bytes": (sz, [sz]),
    "larql_hip_dev_quantize_x_to_q8k": (ci, [vp, vp, sz, vp]),
    "larql_hip_q4k_dual_matvec": (ci, [vp, vp, sz, vp, sz, vp, sz, sz, sz, vp, vp, sz]),
    "larql_hip_q4k_matmul": (ci, [vp, vp, sz, vp, sz, sz, sz, sz, vp, sz]),
    "larql_hip_q4k_matvec_topk": (ci, [vp, vp, sz, vp, sz, sz, sz, sz, vp, vp, C.POINTER(sz)]),
    "larql_hip_q4_matvec": (ci, [vp, vp, sz, vp, sz, vp, sz, sz, sz, vp]),
    "larql_hip_q8_0_gemv": (ci, [vp, vp, sz, vp, sz, sz, sz, vp]),
    "larql_hip_quant_matvec": (ci, [vp, ci, vp, sz, vp, sz, sz, sz, vp]),
    "larql_hip_quant_matvec_q8_input": (ci, [vp, ci, vp, sz, vp, sz, vp, sz, sz, sz, vp]),
    "larql_hip_q8_0_gemv_topk": (ci, [vp, vp, sz, vp, sz, sz, sz, sz, vp, vp, C.POINTER(sz)]),
    "larql_hip_bf16_gemv_multi": (ci, [vp, sz, C.POINTER(vp), C.POINTER(sz), C.POINTER(sz), C.POINTER(sz), vp, sz, C.POINTER(vp)]),
    "larql_hip_f16_gemv_multi": (ci, [vp, sz, C.POINTER(vp), C.POINTER(sz), C.POINTER(sz), C.POINTER(sz), vp, sz, C.POINTER(vp)]),
    "larql_hip_f32_gemv": (ci, [vp, vp, sz, vp, sz, sz, sz, vp, ci]),
    "larql_hip_f16_gemv": (ci, [vp, vp, sz, vp, sz, sz, sz, vp, ci]),
    "larql_hip_bf16_gemv": (ci, [vp, vp, sz, vp, sz, sz, sz, vp, ci]),
    "larql_hip_mxfp4_gemv": (ci, [vp, vp, sz, vp, sz, vp, sz, sz, sz, vp]),
    "larql_hip_mxfp4_gemv_multi": (ci, [vp, sz, C.POINTER(vp), C.POINTER(sz), C.POINTER(vp), C.POINTER(sz),
                                        C.POINTER(sz), C.POINTER(sz), vp, sz, C.POINTER(vp)]),
    "larql_hip_gate_knn": (ci, [vp, ci, vp, sz, vp, sz, sz, sz, sz, vp, vp, C.POINTER(sz)]),
    "larql_hip_gate_scores": (ci, [vp, ci, vp, sz, vp, sz, sz, sz, vp]),
    "larql_hip_malloc": (ci, [vp, C.POINTER(vp), sz]),
    "larql_hip_free": (ci, [vp, vp]),
    "larql_hip_memcpy_h2d": (ci, [vp, vp, vp, sz]),
    "larql_hip_memcpy_d2h": (ci, [vp, vp, vp, sz]),
    "larql_hip_memset": (ci, [vp, vp, ci, sz]),
    "larql_hip_synchronize": (ci, [vp]),
    "larql_hip_event_create": (ci, [vp, C.POINTER(vp)]),
    "larql_hip_event_record": (ci, [vp, vp]),
    "larql_hip_event_elapsed_ms": (ci, [vp, vp, vp, C.POINTER(C.c_float)]),
    "larql_hip_event_destroy": (ci, [vp, vp]),
    "larql_hip_dev_copy": (ci, [vp, vp, vp, sz]),
    "larql_hip_dev_matvec": (ci, [vp, ci, vp, vp, vp, sz, sz, vp]),
    "larql_hip_dev_matvec_batch": (ci, [vp, C.POINTER(MatvecJob), sz]),
    "larql_hip_plan_create": (ci, [vp, C.POINTER(MatvecJob), sz, C.POINTER(vp)]),
    "larql_hip_plan_run": (ci, [vp, vp]),
    "larql_hip_plan_launch_count": (ci, [vp]),
    "larql_hip_plan_destroy": (None, [vp, vp]),
    "larql_hip_sequence_create": (ci, [vp, C.POINTER(vp), sz, C.POINTER(vp)]),
    "larql_hip_sequence_run": (ci, [vp, vp]),
    "larql_hip_sequence_launch_count": (ci, [vp]),
    "larql_hip_sequence_destroy": (None, [vp, vp]),
    "larql_hip_dev_gate_knn": (ci, [vp, ci, vp, vp, sz, sz, sz, sz, vp, vp, vp, vp]),
    "larql_hip_dev_take_nan_flag": (ci, [vp, C.POINTER(ci)]),
    "larql_hip_static_scratch_bytes": (sz, []),
    "larql_hip_debug_alloc_events": (ci, [vp, C.POINTER(u64)]),
    "larql_hip_dev_gate_knn_static": (ci, [vp, ci, vp, vp, sz, sz, sz, sz, vp, vp, vp]),
    "larql_hip_dev_gate_walk": (ci, [vp, ci, C.POINTER(vp), sz, vp, sz, sz, sz, sz, sz, vp, vp, vp, vp]),
    "larql_hip_dev_q4k_gemm": (ci, [vp, vp, vp, sz, sz, sz, vp]),
    "larql_hip_dev_q4k_row_exponents": (ci, [vp, vp, sz, sz, vp]),
    "larql_hip_dev_q4k_gemm_prepared": (ci, [vp, vp, vp, vp, sz, sz, sz, vp]),
    "larql_hip_dev_router_select": (ci, [vp, vp, sz, sz, sz, ci, vp, vp]),
    "larql_hip_moe_mxfp4_workspace_bytes": (sz, [sz, sz, sz, sz]),
    "larql_hip_dev_moe_mxfp4": (ci, [vp, C.POINTER(Mxfp4Experts), vp, sz, sz, vp, vp, vp, vp, sz]),
    "larql_hip_dev_moe_mxfp4_routed": (ci, [vp, C.POINTER(Mxfp4Experts), vp, sz, sz, vp, ci, vp, vp, vp, vp, sz]),
    "larql_hip_moe_layer_create": (ci, [vp, C.POINTER(MoeLayerWeights), C.POINTER(vp)]),
    "larql_hip_moe_layer_destroy": (None, [vp, vp]),
    "larql_hip_moe_layer_forward": (ci, [vp, vp, vp, vp, sz, vp, vp, vp]),
    "larql_hip_dev_moe_layer_forward": (ci, [vp, vp, vp, vp, sz, vp, vp, vp]),
    "larql_hip_dev_quantize_q4_k": (ci, [vp, vp, sz, vp]),
    "larql_hip_dev_quantize_q6_k": (ci, [vp, vp, sz, vp]),
    "larql_hip_dev_quantize_q8_0": (ci, [vp, vp, sz, vp]),
    "larql_hip_dev_quantize_mxfp4": (ci, [vp, vp, sz, sz, vp, vp]),
    "larql_hip_dev_f32_to_bf16": (ci, [vp, vp, sz, vp]),
    "larql_hip_dev_quantize_q4_0": (ci, [vp, vp, sz, vp]),
    "larql_hip_dev_quantize_to_q8": (ci, [vp, vp, sz, vp, vp]),
    "larql_hip_dev_fill_normal": (ci, [vp, vp, sz, u64, C.c_float]),
}


def load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is not built: run `python larql_amd/build.py` (needs hipcc)")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    return lib


lib = load()
