"""larql_amd — MI355X (gfx950) backend for LARQL's quantised decode path:
hand-written HIP kernels behind the reference's ComputeBackend surface.

`HipBackend` is the host-side mirror of the trait; the C ABI it drives is
declared in include/larql_hip.h and built into larql_amd/liblarql_hip.so.
"""
from ._lib import (CAP_F16_GEMV, CAP_F32_GEMV, CAP_QUANT_MATVEC, FMT_BF16, FMT_F16, FMT_F32, FMT_GGML_Q8_0, FMT_Q4_K_Q8K, FMT_Q6_K_Q8K, FMT_I2S,
                   FMT_MXFP4, FMT_Q4_0, FMT_Q4_K, FMT_Q4_KF, FMT_Q5_K, FMT_Q6_K, FMT_Q8_0)
from ._lib import (MOE_GATE_CLAMPED_GELU_TANH, MOE_GATE_CLAMPED_GLU, MOE_GATE_CLAMPED_SILU, MOE_GATE_GELU_TANH, MOE_GATE_SILU, MOE_GATE_SITU_GLU,
                   MOE_ROWS_CONTIGUOUS_HALVES, MOE_ROWS_INTERLEAVED, MOE_SCALES_INLINE,
                   MOE_SCALES_PAIRED, MoeLayerWeights, Mxfp4Experts)
from .backend import DeviceError, HipBackend, NanScoreError

__all__ = ["HipBackend", "Mxfp4Experts", "MoeLayerWeights", "MOE_ROWS_CONTIGUOUS_HALVES", "MOE_ROWS_INTERLEAVED", "MOE_SCALES_INLINE",
           "MOE_SCALES_PAIRED", "MOE_GATE_CLAMPED_GLU", "MOE_GATE_GELU_TANH", "MOE_GATE_SILU", "MOE_GATE_SITU_GLU", "MOE_GATE_CLAMPED_GELU_TANH", "MOE_GATE_CLAMPED_SILU", "DeviceError", "NanScoreError", "FMT_Q4_0", "FMT_Q4_K", "FMT_Q4_KF", "FMT_Q5_K", "FMT_Q6_K",
           "FMT_Q8_0", "FMT_BF16", "FMT_F16", "FMT_F32", "FMT_I2S", "FMT_MXFP4", "FMT_GGML_Q8_0", "FMT_Q4_K_Q8K", "FMT_Q6_K_Q8K", "CAP_F32_GEMV",
           "CAP_F16_GEMV", "CAP_QUANT_MATVEC"]
