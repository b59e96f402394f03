"""ctypes loader for the CPU checker (oracle/liblarql_oracle.so).

TEST INFRASTRUCTURE ONLY.  Import this from tests/, from the smoke check and
from the benchmark's cpu_baseline leg; the product package never does.

The wrappers take and return numpy arrays and follow the reference's refusal
convention: a refused call returns None.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblarql_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libq4dot_ref.so")


def build(force: bool = False) -> None:
    """Compile the checker (and the reference's C kernel when its tree is present)."""
    if force or not os.path.exists(_LIB_PATH) or os.path.exists("/root/reference"):
        subprocess.run(["make", "-C", _HERE, "-s", "all"], check=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build(force=True)
    return C.CDLL(_LIB_PATH)


_lib = _load()
_tlib = _lib  # the library the *_mt timing baselines run in (see enable_native_timing)


def enable_native_timing() -> str:
    """Build the same C file for the host this runs on (-O3 -march=native, contraction still off: the reference is
    Rust and never fuses a*b+c) and route the multi-threaded timing baselines (*_mt) through it.  The checker
    functions keep the portable -O2 build.  Returns the flags in use; falls back to the portable build if the host
    has no compiler."""
    global _tlib
    import tempfile
    flags = ["-O3", "-march=native", "-fPIC", "-shared", "-std=c11", "-ffp-contract=off", "-fno-fast-math", "-pthread"]
    for d in (os.path.join(_HERE, "_native"), tempfile.mkdtemp(prefix="larql_oracle_")):
        try:
            os.makedirs(d, exist_ok=True)
            out = os.path.join(d, "liblarql_oracle_native.so")
            subprocess.run(["gcc", *flags, "-o", out, os.path.join(_HERE, "larql_oracle.c"), "-lm"], check=True,
                           capture_output=True)
            _tlib = C.CDLL(out)
            return " ".join(["gcc", *flags])
        except (OSError, subprocess.CalledProcessError):
            continue
    _tlib = _lib
    return "portable build (gcc -O2): no compiler on this host"
_u8p = C.POINTER(C.c_uint8)
_i8p = C.POINTER(C.c_int8)
_u16p = C.POINTER(C.c_uint16)
_u32p = C.POINTER(C.c_uint32)
_u64p = C.POINTER(C.c_uint64)
_f32p = C.POINTER(C.c_float)
_sz = C.c_size_t


def _p(a: np.ndarray, t):
    return a.ctypes.data_as(t)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint8)


_lib.lq_f16_to_f32.restype = C.c_float
_lib.lq_f16_to_f32.argtypes = [C.c_uint16]
_lib.lq_bf16_to_f32.restype = C.c_float
_lib.lq_bf16_to_f32.argtypes = [C.c_uint16]
for _n in ("lq_f32_to_f16_trunc", "lq_f32_to_f16_nearest", "lq_f32_to_f16_flush", "lq_f32_to_bf16"):
    getattr(_lib, _n).restype = C.c_uint16
    getattr(_lib, _n).argtypes = [C.c_float]
_lib.lq_e8m0_to_f32.restype = C.c_float
_lib.lq_e8m0_to_f32.argtypes = [C.c_uint8]
_lib.lq_mxfp4_table.restype = C.c_float
_lib.lq_mxfp4_table.argtypes = [C.c_uint]
_lib.lq_nearest_mxfp4_code.restype = C.c_uint8
_lib.lq_nearest_mxfp4_code.argtypes = [C.c_float]
_lib.lq_clamped_glu.restype = C.c_float
_lib.lq_clamped_glu.argtypes = [C.c_float] * 4
for _n in ("lq_silu", "lq_gelu_tanh"):
    getattr(_lib, _n).restype = C.c_float
    getattr(_lib, _n).argtypes = [C.c_float]
_lib.lq_moe_combine.restype = C.c_float
_lib.lq_moe_combine.argtypes = [C.c_int, C.c_float, C.c_float, C.c_float, C.c_float]
_lib.lq_top_k_by_abs.restype = C.c_long
_lib.lq_top_k_sorted.restype = C.c_long
_lib.lq_gate_knn_batch_union.restype = C.c_long
_lib.lq_router_select.restype = _sz
_lib.lq_moe_top_k.restype = _sz


# ---- scalar conversions -------------------------------------------------
def f16_to_f32(bits: int) -> float:
    return _lib.lq_f16_to_f32(bits)


def f32_to_f16_trunc(v: float) -> int:
    return _lib.lq_f32_to_f16_trunc(v)


def f32_to_f16_nearest(v: float) -> int:
    return _lib.lq_f32_to_f16_nearest(v)


def f32_to_f16_flush(v: float) -> int:
    return _lib.lq_f32_to_f16_flush(v)


def f32_to_bf16(a) -> np.ndarray:
    a = _f32(a).ravel()
    out = np.empty(a.size, dtype=np.uint16)
    _lib.lq_f32_to_bf16_slice(_p(a, _f32p), _sz(a.size), _p(out, _u16p))
    return out


def e8m0_to_f32(b: int) -> float:
    return _lib.lq_e8m0_to_f32(b)


def mxfp4_table(code: int) -> float:
    return _lib.lq_mxfp4_table(code)


def nearest_mxfp4_code(v: float) -> int:
    return _lib.lq_nearest_mxfp4_code(v)


def clamped_glu(g: float, u: float, limit: float = 7.0, alpha: float = 1.702) -> float:
    return _lib.lq_clamped_glu(g, u, limit, alpha)


# ---- Q4_K -----------------------------------------------------------------
def quantize_q4_k(data) -> np.ndarray:
    data = _f32(data).ravel()
    out = np.empty(data.size // 256 * 144, dtype=np.uint8)
    if _lib.lq_quantize_q4_k(_p(data, _f32p), _sz(data.size), _p(out, _u8p)):
        raise ValueError("data length must be a multiple of 256")
    return out


def dequantize_q4_k(data, n: int):
    data = _u8(data).ravel()
    out = np.empty(n, dtype=np.float32)
    if _lib.lq_dequantize_q4_k(_p(data, _u8p), _sz(data.size), _sz(n), _p(out, _f32p)):
        return None
    return out


def q4k_matvec(w, x, rows: int, cols: int, out_len: int | None = None):
    w, x = _u8(w).ravel(), _f32(x).ravel()
    out_len = rows if out_len is None else out_len
    out = np.full(out_len, np.nan, dtype=np.float32)
    rc = _lib.lq_q4k_matvec_into(_p(out, _f32p), _sz(out_len), _p(x, _f32p), _sz(x.size),
                                 _p(w, _u8p), _sz(w.size), _sz(rows), _sz(cols))
    return None if rc else out


def q4k_matvec_mt(w, x, rows: int, cols: int, threads: int):
    w, x = _u8(w).ravel(), _f32(x).ravel()
    out = np.empty(rows, dtype=np.float32)
    rc = _tlib.lq_q4k_matvec_into_mt(_p(out, _f32p), _p(x, _f32p), _p(w, _u8p), _sz(w.size),
                                    _sz(rows), _sz(cols), C.c_int(threads))
    return None if rc else out


def q4k_matvec_scalar(w, x, rows: int, hidden: int) -> np.ndarray:
    w, x = _u8(w).ravel(), _f32(x).ravel()
    out = np.empty(rows, dtype=np.float32)
    _lib.lq_q4k_matvec_scalar(_p(out, _f32p), _p(x, _f32p), _p(w, _u8p), _sz(rows), _sz(hidden))
    return out


def q4k_dual_matvec(wa, wb, x, rows: int, cols: int):
    wa, wb, x = _u8(wa).ravel(), _u8(wb).ravel(), _f32(x).ravel()
    oa = np.empty(rows, dtype=np.float32)
    ob = np.empty(rows, dtype=np.float32)
    rc = _lib.lq_q4k_dual_matvec_into(_p(oa, _f32p), _p(ob, _f32p), _sz(rows), _p(x, _f32p), _sz(x.size),
                                      _p(wa, _u8p), _sz(wa.size), _p(wb, _u8p), _sz(wb.size),
                                      _sz(rows), _sz(cols))
    return None if rc else (oa, ob)


def q4k_matmul(w, x, rows: int, hidden: int, seq: int) -> np.ndarray:
    w, x = _u8(w).ravel(), _f32(x).ravel()
    out = np.full(seq * rows, np.nan, dtype=np.float32)
    _lib.lq_q4k_matmul_into(_p(out, _f32p), _p(x, _f32p), _p(w, _u8p), _sz(w.size),
                            _sz(rows), _sz(hidden), _sz(seq))
    return out.reshape(seq, rows) if seq and rows else out


# ---- Q8_0 -----------------------------------------------------------------
def quantize_q6_k(data) -> np.ndarray:
    data = _f32(data).ravel()
    out = np.empty(data.size // 256 * 210, dtype=np.uint8)
    if _lib.lq_quantize_q6_k(_p(data, _f32p), _sz(data.size), _p(out, _u8p)):
        raise ValueError("Q6_K: element count must be multiple of 256")
    return out


def dequantize_q6_k(data, n: int):
    data = _u8(data).ravel()
    out = np.empty(n, dtype=np.float32)
    if _lib.lq_dequantize_q6_k(_p(data, _u8p), _sz(data.size), _sz(n), _p(out, _f32p)):
        return None
    return out


def q6k_matvec(w, x, rows: int, hidden: int):
    w, x = _u8(w).ravel(), _f32(x).ravel()
    out = np.empty(rows, dtype=np.float32)
    if x.size != hidden or _lib.lq_q6k_matvec(_p(w, _u8p), _sz(w.size), _p(x, _f32p), _sz(rows), _sz(hidden), _p(out, _f32p)):
        return None
    return out


def quantize_x_to_q8k(x):
    """Q8_K activation: (qs int8 [n], d f32 [n/256], sums int16 [n/32]); n % 256 == 0."""
    x = _f32(x).ravel()
    if x.size % 256 != 0:
        raise ValueError("Q8_K: element count must be a multiple of 256")
    qs = np.empty(x.size, dtype=np.int8)
    d = np.empty(x.size // 256, dtype=np.float32)
    sums = np.empty(x.size // 32, dtype=np.int16)
    _lib.lq_quantize_x_to_q8k(_p(x, _f32p), _sz(x.size), _p(qs, _i8p), _p(d, _f32p), _p(sums, C.POINTER(C.c_int16)))
    return qs, d, sums


def q4k_q8k_matvec(w, qs, d, sums, rows: int, cols: int):
    """q4k_q8k_matvec_scalar: None where the reference refuses the operands."""
    w = _u8(w).ravel()
    qs = np.ascontiguousarray(qs, dtype=np.int8).ravel()
    d = _f32(d).ravel()
    sums = np.ascontiguousarray(sums, dtype=np.int16).ravel()
    out = np.empty(rows, dtype=np.float32)
    if d.size * 256 != qs.size or sums.size * 32 != qs.size:
        return None
    if _lib.lq_q4k_q8k_matvec(_p(out, _f32p), _sz(rows), _p(qs, _i8p), _sz(qs.size), _p(d, _f32p), _p(sums, C.POINTER(C.c_int16)),
                              _p(w, _u8p), _sz(w.size), _sz(rows), _sz(cols)):
        return None
    return out


def q6k_q8k_matvec(w, qs, d, rows: int, cols: int):
    """q6k_q8k_matvec_scalar: None where the reference refuses the operands."""
    w = _u8(w).ravel()
    qs = np.ascontiguousarray(qs, dtype=np.int8).ravel()
    d = _f32(d).ravel()
    out = np.empty(rows, dtype=np.float32)
    if d.size * 256 != qs.size:
        return None
    if _lib.lq_q6k_q8k_matvec(_p(out, _f32p), _sz(rows), _p(qs, _i8p), _sz(qs.size), _p(d, _f32p), _p(w, _u8p), _sz(w.size), _sz(rows),
                              _sz(cols)):
        return None
    return out


def quantize_q8_0(data) -> np.ndarray:
    data = _f32(data).ravel()
    out = np.empty(data.size // 32 * 34, dtype=np.uint8)
    if _lib.lq_quantize_q8_0(_p(data, _f32p), _sz(data.size), _p(out, _u8p)):
        raise ValueError("Q8_0: element count must be multiple of 32")
    return out


def dequantize_q8_0(data, n: int):
    data = _u8(data).ravel()
    out = np.empty(n, dtype=np.float32)
    if _lib.lq_dequantize_q8_0(_p(data, _u8p), _sz(data.size), _sz(n), _p(out, _f32p)):
        return None
    return out


def q8_0_gemv(blocks, x, n: int, k: int):
    blocks, x = _u8(blocks).ravel(), _f32(x).ravel()
    out = np.empty(n, dtype=np.float32)
    rc = _lib.lq_q8_0_gemv(_p(blocks, _u8p), _sz(blocks.size), _p(x, _f32p), _sz(x.size),
                           _sz(n), _sz(k), _p(out, _f32p))
    return None if rc else out


def q8_0_gemv_mt(blocks, x, n: int, k: int, threads: int):
    blocks, x = _u8(blocks).ravel(), _f32(x).ravel()
    out = np.empty(n, dtype=np.float32)
    rc = _tlib.lq_q8_0_gemv_mt(_p(blocks, _u8p), _sz(blocks.size), _p(x, _f32p),
                              _sz(n), _sz(k), _p(out, _f32p), C.c_int(threads))
    return None if rc else out


# ---- Q4_0 x Q8 --------------------------------------------------------------
def quantize_to_q8(x):
    x = _f32(x).ravel()
    q8 = np.empty(x.size, dtype=np.int8)
    scales = np.empty(x.size // 32, dtype=np.float32)
    _lib.lq_quantize_to_q8(_p(x, _f32p), _sz(x.size), _p(q8, _i8p), _p(scales, _f32p))
    return q8, scales


def quantize_q4_0(data) -> np.ndarray:
    data = _f32(data).ravel()
    out = np.empty(data.size // 32 * 18, dtype=np.uint8)
    if _lib.lq_quantize_q4_0(_p(data, _f32p), _sz(data.size), _p(out, _u8p)):
        raise ValueError("data length must be a multiple of 32")
    return out


def q4_0_matvec(q4, q8_x, q8_scales, rows: int, hidden: int) -> np.ndarray:
    q4 = _u8(q4).ravel()
    q8_x = np.ascontiguousarray(q8_x, dtype=np.int8)
    q8_scales = _f32(q8_scales)
    assert hidden % 32 == 0 and q4.size == rows * (hidden // 32) * 18
    assert q8_x.size == hidden and q8_scales.size == hidden // 32
    out = np.empty(rows, dtype=np.float32)
    _lib.lq_q4_0_matvec(_p(q4, _u8p), _p(q8_x, _i8p), _p(q8_scales, _f32p), _p(out, _f32p),
                        _sz(rows), _sz(hidden))
    return out


def ref_q4_0_matvec(q4, q8_x, q8_scales, rows: int, hidden: int):
    """The reference's own q4_0_matvec_c, compiled from its tree (None if not built)."""
    if not os.path.exists(_REF_PATH):
        return None
    ref = C.CDLL(_REF_PATH)
    q4 = _u8(q4).ravel()
    q8_x = np.ascontiguousarray(q8_x, dtype=np.int8)
    q8_scales = _f32(q8_scales)
    out = np.empty(rows, dtype=np.float32)
    ref.q4_0_matvec_c(_p(q4, _u8p), _p(q8_x, _i8p), _p(q8_scales, _f32p), _p(out, _f32p),
                      _sz(rows), _sz(hidden))
    return out


def dequantise_q8(q8_x, scales) -> np.ndarray:
    q8_x = np.ascontiguousarray(q8_x, dtype=np.int8)
    scales = _f32(scales)
    out = np.empty(q8_x.size, dtype=np.float32)
    _lib.lq_dequantise_q8(_p(q8_x, _i8p), _sz(q8_x.size), _p(scales, _f32p), _p(out, _f32p))
    return out


# ---- MXFP4 ------------------------------------------------------------------
def quantize_mxfp4(values, rows: int, k: int):
    values = _f32(values).ravel()
    assert values.size == rows * k
    packed = np.empty(rows * (k // 32) * 16, dtype=np.uint8)
    scales = np.empty(rows * (k // 32), dtype=np.uint8)
    if _lib.lq_quantize_mxfp4(_p(values, _f32p), _sz(rows), _sz(k), _p(packed, _u8p), _p(scales, _u8p)):
        return None
    return packed, scales


def dequantize_mxfp4_expert(blocks, scales, out_features: int, groups: int):
    blocks, scales = _u8(blocks).ravel(), _u8(scales).ravel()
    out = np.empty(out_features * groups * 32, dtype=np.float32)
    rc = _lib.lq_dequantize_mxfp4_expert(_p(blocks, _u8p), _sz(blocks.size), _p(scales, _u8p),
                                         _sz(scales.size), _sz(out_features), _sz(groups), _p(out, _f32p))
    return None if rc else out


def mxfp4_gemv(packed, scales, x, n: int, k: int):
    packed, scales, x = _u8(packed).ravel(), _u8(scales).ravel(), _f32(x).ravel()
    out = np.empty(n, dtype=np.float32)
    rc = _lib.lq_mxfp4_gemv(_p(packed, _u8p), _sz(packed.size), _p(scales, _u8p), _sz(scales.size),
                            _p(x, _f32p), _sz(x.size), _sz(n), _sz(k), _p(out, _f32p))
    return None if rc else out


def mxfp4_gemv_dequant(packed, scales, x, n: int, k: int) -> np.ndarray:
    packed, scales, x = _u8(packed).ravel(), _u8(scales).ravel(), _f32(x).ravel()
    out = np.empty(n, dtype=np.float32)
    _lib.lq_mxfp4_gemv_dequant(_p(packed, _u8p), _p(scales, _u8p), _p(x, _f32p), _sz(n), _sz(k), _p(out, _f32p))
    return out


# ---- dense gemv -------------------------------------------------------------
def bf16_gemv(w_bits, x, n: int, k: int) -> np.ndarray:
    w = np.ascontiguousarray(w_bits, dtype=np.uint16).ravel()
    x = _f32(x).ravel()
    out = np.empty(n, dtype=np.float32)
    _lib.lq_bf16_gemv(_p(w, _u16p), _p(x, _f32p), _sz(n), _sz(k), _p(out, _f32p))
    return out


def bf16_gemv_mt(w_bits, x, n: int, k: int, threads: int) -> np.ndarray:
    """bf16_gemv with the rows shared out in chunks of 32 over `threads` threads (timing baseline; same bits)."""
    w = np.ascontiguousarray(w_bits, dtype=np.uint16).ravel()
    x = _f32(x).ravel()
    out = np.empty(n, dtype=np.float32)
    _tlib.lq_bf16_gemv_mt(_p(w, _u16p), _p(x, _f32p), _sz(n), _sz(k), _p(out, _f32p), C.c_int(threads))
    return out


def f16_gemv(w_bits, x, n: int, k: int) -> np.ndarray:
    w = np.ascontiguousarray(w_bits, dtype=np.uint16).ravel()
    x = _f32(x).ravel()
    out = np.empty(n, dtype=np.float32)
    _lib.lq_f16_gemv(_p(w, _u16p), _p(x, _f32p), _sz(n), _sz(k), _p(out, _f32p))
    return out


def f32_gemv(w, x, n: int, k: int) -> np.ndarray:
    w, x = _f32(w).ravel(), _f32(x).ravel()
    out = np.empty(n, dtype=np.float32)
    _lib.lq_f32_gemv(_p(w, _f32p), _p(x, _f32p), _sz(n), _sz(k), _p(out, _f32p))
    return out


# ---- top-K ------------------------------------------------------------------
def top_k_by_abs(scores, top_k: int):
    """[(idx, score)] sorted by |score| descending; raises on NaN like the reference panics."""
    scores = _f32(scores).ravel()
    cap = max(1, min(top_k, scores.size))
    idx = np.empty(cap, dtype=np.uint64)
    val = np.empty(cap, dtype=np.float32)
    got = _lib.lq_top_k_by_abs(_p(scores, _f32p), _sz(scores.size), _sz(top_k), _p(idx, _u64p), _p(val, _f32p))
    if got < 0:
        raise ValueError("NaN score")
    return [(int(idx[i]), float(val[i])) for i in range(got)]


def top_k_sorted(scores, top_k: int):
    scores = _f32(scores).ravel()
    cap = max(1, min(top_k, scores.size))
    idx = np.empty(cap, dtype=np.uint32)
    val = np.empty(cap, dtype=np.float32)
    got = _lib.lq_top_k_sorted(_p(scores, _f32p), _sz(scores.size), _sz(top_k), _p(idx, _u32p), _p(val, _f32p))
    return [(int(idx[i]), float(val[i])) for i in range(got)]


def gate_knn_batch_union(scores_2d, top_k: int):
    """scores_2d: [n_features, seq]; returns the sorted de-duplicated union of per-position hits."""
    s = _f32(scores_2d)
    n, seq = s.shape
    cap = max(1, seq * min(top_k, n))
    idx = np.empty(cap, dtype=np.uint64)
    got = _lib.lq_gate_knn_batch_union(_p(s, _f32p), _sz(n), _sz(seq), _sz(top_k), _p(idx, _u64p), _sz(cap))
    if got < 0:
        raise ValueError("NaN score")
    return [int(v) for v in idx[:got]]


# ---- MoE routing ------------------------------------------------------------
SOFTMAX_THEN_SELECT = 0
NORMALISED_OVER_SELECTED = 1


# MoeFusedRowLayout / FusedHalf — larql-compute/src/pipeline/moe.rs:294-332, larql-models/src/quant/mxfp4.rs:168-191
CONTIGUOUS_HALVES, INTERLEAVED = 0, 1
HALF_GATE, HALF_UP = 0, 1


def fused_row_walk(layout: int, half: int, inter: int):
    """MoeFusedRowLayout::row_walk: (first row, row stride) of one half's rows in a fused gate_up region of 2*inter rows."""
    if layout == CONTIGUOUS_HALVES:
        return (0, 1) if half == HALF_GATE else (inter, 1)
    return (2 * 0 + (0 if half == HALF_GATE else 1), 2)  # FusedHalf::fused_row(0), FUSED_HALVES


def deinterleave_fused_half(data, out_features: int, in_features: int, half: int) -> np.ndarray:
    """deinterleave_fused_half (mxfp4.rs:218-231): the rows of one projection out of a fused [out_features, in_features] matrix."""
    m = np.asarray(data).reshape(out_features, in_features)
    first, step = fused_row_walk(INTERLEAVED, half, out_features // 2)
    return m[first::step].reshape(-1).copy()


def router_select(logits, k: int, policy: int = NORMALISED_OVER_SELECTED):
    logits = _f32(logits).ravel()
    cap = max(1, min(k, logits.size))
    e = np.empty(cap, dtype=np.uint64)
    w = np.empty(cap, dtype=np.float32)
    got = _lib.lq_router_select(_p(logits, _f32p), _sz(logits.size), _sz(k), C.c_int(policy), _p(e, _u64p), _p(w, _f32p))
    return [(int(e[i]), float(w[i])) for i in range(got)]


def moe_router_logits(router_in, router_proj, router_bias=None) -> np.ndarray:
    """moe_router_logits (cpu/ops/moe/mod.rs:127-147): router_proj is [n_experts, hidden]."""
    x = _f32(router_in).ravel()
    w = np.ascontiguousarray(router_proj, dtype=np.float32)
    n, hidden = w.shape
    assert hidden == x.size
    b = None if router_bias is None else _f32(router_bias).ravel()
    out = np.empty(n, dtype=np.float32)
    _lib.lq_moe_router_logits(_p(x, _f32p), _p(w, _f32p), _p(b, _f32p) if b is not None else None, _sz(n), _sz(hidden), _p(out, _f32p))
    return out


def moe_route_from_router_input(router_in, router_proj, router_bias, top_k: int, renormalize: bool = True, per_expert_scale=None):
    """moe_route_from_router_input (cpu/ops/moe/mod.rs:149-186): [(expert, weight)] in selection order."""
    x = _f32(router_in).ravel()
    w = np.ascontiguousarray(router_proj, dtype=np.float32)
    n, hidden = w.shape
    b = None if router_bias is None else _f32(router_bias).ravel()
    sc = None if per_expert_scale is None else _f32(per_expert_scale).ravel()
    cap = max(1, min(top_k, n))
    e = np.empty(cap, dtype=np.uint64)
    wt = np.empty(cap, dtype=np.float32)
    _lib.lq_moe_route_from_router_input.restype = C.c_size_t
    got = _lib.lq_moe_route_from_router_input(_p(x, _f32p), _sz(hidden), _p(w, _f32p), _p(b, _f32p) if b is not None else None, _sz(n),
                                              _sz(top_k), C.c_int(1 if renormalize else 0), _p(sc, _f32p) if sc is not None else None,
                                              _sz(0 if sc is None else sc.size), _p(e, _u64p), _p(wt, _f32p))
    return [(int(e[i]), float(wt[i])) for i in range(got)]


def moe_top_k(v, k: int):
    v = _f32(v).ravel()
    cap = max(1, min(k, v.size))
    idx = np.empty(cap, dtype=np.uint64)
    val = np.empty(cap, dtype=np.float32)
    got = _lib.lq_moe_top_k(_p(v, _f32p), _sz(v.size), _sz(k), _p(idx, _u64p), _p(val, _f32p))
    return [int(i) for i in idx[:got]], [float(x) for x in val[:got]]


def softmax(v) -> np.ndarray:
    v = _f32(v).ravel().copy()
    _lib.lq_softmax(_p(v, _f32p), _sz(v.size))
    return v


# ---- MoE expert block -------------------------------------------------------
def _opt_f32(a):
    if a is None:
        return None, None
    a = _f32(a).ravel()
    return a, _p(a, _f32p)


def moe_block_f32(x, router_w, router_b, fused, down, gate_up_bias, down_bias, top_k: int, policy: int = NORMALISED_OVER_SELECTED,
                  limit: float = 7.0, alpha: float = 1.702) -> np.ndarray:
    """ExpertWeightFfn::moe_block (ffn/expert_weight/mod.rs:100-262) on a GPT-OSS-shaped f32 layer.
    x [T, hidden]; router_w [E, hidden]; fused [E, 2*inter, hidden] (gate = even rows, up = odd rows);
    down [E, hidden, inter]; gate_up_bias [E, 2*inter] (interleaved) / down_bias [E, hidden] / router_b [E] or None."""
    x, router_w, fused, down = _f32(x), _f32(router_w), _f32(fused), _f32(down)
    tokens, hidden = x.shape
    n_experts = router_w.shape[0]
    inter = fused.shape[1] // 2
    assert fused.shape == (n_experts, 2 * inter, hidden) and down.shape == (n_experts, hidden, inter)
    rb, rbp = _opt_f32(router_b)
    gb, gbp = _opt_f32(gate_up_bias)
    db, dbp = _opt_f32(down_bias)
    out = np.empty((tokens, hidden), np.float32)
    _lib.lq_moe_block_f32(_p(x, _f32p), _sz(tokens), _sz(hidden), _sz(inter), _sz(n_experts), _sz(top_k), C.c_int(policy),
                          _p(router_w, _f32p), rbp, _p(fused, _f32p), _p(down, _f32p), gbp, dbp, C.c_float(limit), C.c_float(alpha),
                          _p(out, _f32p))
    return out


def moe_block_mxfp4(x, experts, weights, gate, up, down, n_experts: int, hidden: int, inter: int, interleaved: bool = False,
                    gate_up_bias=None, down_bias=None, limit: float = 7.0, alpha: float = 1.702) -> np.ndarray:
    """The expert block over an MXFP4 bank with the routing given.  gate / up / down are (packed, scales) pairs, expert
    after expert; with `interleaved` gate holds each expert's fused [2*inter, hidden/32] rows and `up` is ignored.
    experts / weights: [T, k]."""
    x = _f32(x)
    tokens = x.shape[0]
    ex = np.ascontiguousarray(experts, dtype=np.uint64).reshape(tokens, -1)
    wt = _f32(weights).reshape(tokens, -1)
    k = ex.shape[1]
    gp, gs = _u8(gate[0]), _u8(gate[1])
    up_, us = (gp, gs) if interleaved else (_u8(up[0]), _u8(up[1]))
    dp, ds = _u8(down[0]), _u8(down[1])
    gb, gbp = _opt_f32(gate_up_bias)
    db, dbp = _opt_f32(down_bias)
    out = np.empty((tokens, hidden), np.float32)
    rc = _lib.lq_moe_block_mxfp4(_p(x, _f32p), _sz(tokens), _sz(hidden), _sz(inter), _sz(n_experts), _sz(k), _p(ex, _u64p),
                                 _p(wt, _f32p), _p(gp, _u8p), _p(gs, _u8p), _p(up_, _u8p), _p(us, _u8p), _p(dp, _u8p), _p(ds, _u8p),
                                 C.c_int(1 if interleaved else 0), gbp, dbp, C.c_float(limit), C.c_float(alpha), _p(out, _f32p))
    if rc:
        raise ValueError("hidden and inter must be multiples of 32")
    return out


GATE_CLAMPED_GLU, GATE_GELU_TANH, GATE_SILU, GATE_SITU_GLU, GATE_CLAMPED_GELU_TANH, GATE_CLAMPED_SILU = 0, 1, 2, 3, 4, 5


def silu(x: float) -> float:
    return _lib.lq_silu(x)


def gelu_tanh(x: float) -> float:
    return _lib.lq_gelu_tanh(x)


def moe_combine(rule: int, g: float, u: float, limit: float = 7.0, alpha: float = 1.702) -> float:
    return _lib.lq_moe_combine(rule, g, u, limit, alpha)


def moe_block_kq(x, experts, weights, gate_up, down, hidden: int, cols: int, inter: int, fmt: int = 4, gate_up_bias=None,
                 down_bias=None, rule: int = GATE_GELU_TANH, limit: float = 7.0, alpha: float = 1.702) -> np.ndarray:
    """cpu_moe_forward's integer expert path over per-expert k-quant slices (fmt 4 = Q4_K, 6 = Q6_K), routing given.
    gate_up[e]: bytes of [2*inter, cols] rows (gate half first); down[e]: [hidden, ceil(inter/256)*256] rows.
    fmt 16 / 17 / 32 = a BF16 / F16 / F32 bank on the f32 arm: f32 activations, down [hidden, inter]."""
    x = _f32(x)
    tokens = x.shape[0]
    ex = np.ascontiguousarray(experts, dtype=np.uint64).reshape(tokens, -1)
    wt = _f32(weights).reshape(tokens, -1)
    k = ex.shape[1]
    gu = [_u8(a).ravel() for a in gate_up]
    dn = [_u8(a).ravel() for a in down]
    n_experts = len(gu)
    if fmt in (16, 17, 32):                       # float banks: BF16 / F16 / F32, rows unpadded
        el = 4 if fmt == 32 else 2
        need_gu, need_dn = 2 * inter * cols * el, hidden * inter * el
    else:
        blk = 210 if fmt == 6 else 144
        ip = (inter + 255) // 256 * 256
        need_gu, need_dn = 2 * inter * (cols // 256) * blk, hidden * (ip // 256) * blk
    for a, b in zip(gu, dn):
        if a.size < need_gu or b.size < need_dn:
            raise ValueError("an expert's slices are shorter than the geometry")
    gup = (C.c_void_p * n_experts)(*[a.ctypes.data for a in gu])
    dnp = (C.c_void_p * n_experts)(*[a.ctypes.data for a in dn])
    gb, gbp = _opt_f32(gate_up_bias)
    db, dbp = _opt_f32(down_bias)
    out = np.empty((tokens, hidden), np.float32)
    rc = _lib.lq_moe_block_kq(_p(x, _f32p), _sz(tokens), _sz(hidden), _sz(cols), _sz(inter), _sz(n_experts), _sz(k), _p(ex, _u64p),
                              _p(wt, _f32p), gup, dnp, C.c_int(fmt), gbp, dbp, C.c_int(rule), C.c_float(limit), C.c_float(alpha),
                              _p(out, _f32p))
    if rc:
        raise ValueError("moe_block_kq: bad geometry")
    return out


# ---- multi-threaded timing baselines for the other configurations ------------------------------------------
def mxfp4_gemv_mt(packed, scales, x, n: int, k: int, threads: int):
    p, sc, x = _u8(packed).ravel(), _u8(scales).ravel(), _f32(x).ravel()
    out = np.empty(n, dtype=np.float32)
    rc = _tlib.lq_mxfp4_gemv_mt(_p(p, _u8p), _p(sc, _u8p), _p(x, _f32p), _sz(n), _sz(k), _p(out, _f32p), C.c_int(threads))
    return None if rc else out


def q4k_matmul_mt(w, x, rows: int, hidden: int, seq: int, threads: int):
    w, x = _u8(w).ravel(), _f32(x).ravel()
    out = np.empty((seq, rows), dtype=np.float32)
    rc = _tlib.lq_q4k_matmul_into_mt(_p(out, _f32p), _p(x, _f32p), _p(w, _u8p), _sz(w.size), _sz(rows), _sz(hidden), _sz(seq),
                                     C.c_int(threads))
    return None if rc else out
