"""HipBackend — the host-side mirror of the reference's ComputeBackend trait
family for the quantised decode path, over the C ABI.

Method names, argument meaning and the None-means-"cannot serve, fall back"
convention follow larql-compute/src/backend/{mod,quant_matvec,matmul}.rs; the
gate-KNN methods follow larql-vindex/src/index/compute/gate_knn/dispatch.rs.
Arrays are numpy; weights are uint8 byte streams exactly as the reference
stores them.
"""
from __future__ import annotations

import ctypes as C
from typing import List, Optional, Sequence, Tuple

import numpy as np

from . import _lib as L

lib = L.lib


def _ptr(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _u8(a) -> np.ndarray:
    a = np.asarray(a)
    if a.dtype != np.uint8:
        a = a.view(np.uint8) if a.flags.c_contiguous else np.ascontiguousarray(a).view(np.uint8)
    return np.ascontiguousarray(a).reshape(-1)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32).reshape(-1)


class DeviceError(RuntimeError):
    pass


class NanScoreError(ValueError):
    """A NaN gate score: the reference's top_k_by_abs panics on it."""


class HipBackend:
    """One GPU, one stream.  `HipBackend()` raises if there is no gfx950 device
    (the reference's BackendSelectError::NoDevice: never a silent CPU fallback)."""

    def __init__(self, device: int = 0):
        h = C.c_void_p()
        rc = lib.larql_hip_create(C.byref(h), device)
        if rc != L.OK:
            raise RuntimeError(f"no usable gfx950 device {device} (larql_hip_create -> {rc})")
        self._h = h
        self._regions: list = []  # keeps registered host arrays alive, as the contract demands

    def close(self) -> None:
        if getattr(self, "_h", None):
            lib.larql_hip_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    # -- error mapping ---------------------------------------------------------
    def _some(self, rc: int) -> bool:
        """True for Some, False for None (refusal); raises on device errors."""
        if rc == L.OK:
            return True
        if rc in (L.UNSUPPORTED, L.REFUSED_SHAPE):
            return False
        if rc == L.E_NAN:
            raise NanScoreError(self.last_error())
        raise DeviceError(f"{rc}: {self.last_error()}")

    def last_error(self) -> str:
        return lib.larql_hip_last_error(self._h).decode()

    # -- ComputeBackend metadata -------------------------------------------------
    def name(self) -> str:
        return lib.larql_hip_name(self._h).decode()

    def device_info(self) -> str:
        return lib.larql_hip_device_info(self._h).decode()

    def supports_quant(self, fmt: int) -> bool:
        return bool(lib.larql_hip_supports_quant(self._h, fmt))

    def supports(self, cap: int) -> bool:
        return bool(lib.larql_hip_supports(self._h, cap))

    def register_weight_region(self, region: np.ndarray) -> None:
        region = _u8(region)
        self._regions.append(region)
        self._some(lib.larql_hip_register_weight_region(self._h, _ptr(region), region.size))

    def seal_weight_regions(self) -> None:
        self._some(lib.larql_hip_seal_weight_regions(self._h))

    def clear_weight_regions(self) -> None:
        self._some(lib.larql_hip_clear_weight_regions(self._h))
        self._regions.clear()

    def submission_clock(self) -> dict:
        c = L.SubmissionClock()
        self._some(lib.larql_hip_get_submission_clock(self._h, C.byref(c)))
        return {"submissions": c.submissions, "commit_to_done_nanos": c.commit_to_done_nanos, "gpu_nanos": c.gpu_nanos}

    # -- QuantMatVec ---------------------------------------------------------------
    def q4k_matvec(self, q4k_data, x, num_rows: int, hidden: int, out_len: Optional[int] = None):
        w, x = _u8(q4k_data), _f32(x)
        out = np.empty(num_rows if out_len is None else out_len, np.float32)
        ok = self._some(lib.larql_hip_q4k_matvec(self._h, _ptr(w), w.size, _ptr(x), x.size, num_rows, hidden,
                                                 _ptr(out), out.size))
        return out if ok else None

    def q6k_matvec(self, q6k, x, num_rows: int, hidden: int) -> Optional[np.ndarray]:
        """QuantMatVec::q6k_matvec (backend/quant_matvec.rs:335-345)."""
        w, xv = _u8(q6k), _f32(x)
        out = np.empty(num_rows, np.float32)
        ok = self._some(lib.larql_hip_q6k_matvec(self._h, _ptr(w), w.size, _ptr(xv), xv.size, num_rows, hidden, _ptr(out)))
        return out if ok else None

    def quantize_x_to_q8k(self, x):
        """quantize_x_to_q8k (cpu/ops/q4k_q8k_dot/q8k_activation.rs:84-109) -> (qs int8, d f32, sums int16) or None."""
        xv = _f32(x)
        n = xv.size
        qs, d, sums = np.empty(n, np.int8), np.empty(n // 256, np.float32), np.empty(n // 32, np.int16)
        ok = self._some(lib.larql_hip_quantize_x_to_q8k(self._h, _ptr(xv), n, _ptr(qs), _ptr(d), _ptr(sums)))
        return (qs, d, sums) if ok else None

    def q4k_q8k_matvec(self, q4k, qs, d, sums, num_rows: int, cols: int, out_len: Optional[int] = None) -> Optional[np.ndarray]:
        """q4k_q8k_matvec_into (cpu/ops/q4k_q8k_dot/dispatch.rs:15-51): Q4_K rows against a Q8_K activation."""
        w = _u8(q4k)
        qs = np.ascontiguousarray(qs, dtype=np.int8).reshape(-1)
        d = _f32(d)
        sums = np.ascontiguousarray(sums, dtype=np.int16).reshape(-1)
        if d.size * 256 != qs.size or sums.size * 32 != qs.size:
            return None
        out = np.empty(num_rows if out_len is None else out_len, np.float32)
        ok = self._some(lib.larql_hip_q4k_q8k_matvec(self._h, _ptr(w), w.size, _ptr(qs), qs.size, _ptr(d), _ptr(sums), num_rows, cols,
                                                     _ptr(out), out.size))
        return out if ok else None

    def q4k_q8k_gate_up(self, gate_w, up_w, qs, d, sums, num_rows: int, cols: int):
        """q4k_q8k_gate_up_into (cpu/ops/q4k_q8k_dot/gate_up.rs:30-57) -> (gate_out, up_out) or None."""
        gw, uw = _u8(gate_w), _u8(up_w)
        qs = np.ascontiguousarray(qs, dtype=np.int8).reshape(-1)
        d = _f32(d)
        sums = np.ascontiguousarray(sums, dtype=np.int16).reshape(-1)
        if d.size * 256 != qs.size or sums.size * 32 != qs.size:
            return None
        go, uo = np.empty(num_rows, np.float32), np.empty(num_rows, np.float32)
        ok = self._some(lib.larql_hip_q4k_q8k_gate_up(self._h, _ptr(gw), gw.size, _ptr(uw), uw.size, _ptr(qs), qs.size, _ptr(d), _ptr(sums),
                                                      num_rows, cols, _ptr(go), _ptr(uo), num_rows))
        return (go, uo) if ok else None

    def q4k_q8k_gemm(self, q4k, acts, num_rows: int, cols: int) -> Optional[np.ndarray]:
        """q4k_q8k_gemm_into (cpu/ops/q4k_q8k_dot/gemm.rs:42-112): `acts` is a sequence of (qs, d, sums); -> [seq, rows]."""
        w = _u8(q4k)
        seq = len(acts)
        if any(np.asarray(a[0]).size != cols for a in acts):
            return None
        qs = np.ascontiguousarray(np.concatenate([np.asarray(a[0], np.int8).reshape(-1) for a in acts])) if seq else np.zeros(0, np.int8)
        d = np.ascontiguousarray(np.concatenate([_f32(a[1]) for a in acts])) if seq else np.zeros(0, np.float32)
        sums = np.ascontiguousarray(np.concatenate([np.asarray(a[2], np.int16).reshape(-1) for a in acts])) if seq else np.zeros(0, np.int16)
        out = np.empty(seq * num_rows, np.float32)
        ok = self._some(lib.larql_hip_q4k_q8k_gemm(self._h, _ptr(w), w.size, _ptr(qs), _ptr(d), _ptr(sums), seq, num_rows, cols, _ptr(out), out.size))
        return out.reshape(seq, num_rows) if ok else None

    def q6k_q8k_matvec(self, q6k, qs, d, num_rows: int, cols: int, out_len: Optional[int] = None) -> Optional[np.ndarray]:
        """q6k_q8k_matvec_into (cpu/ops/q4k_q8k_dot/q6k.rs:15-92): Q6_K rows against a Q8_K activation (qs and d; no sums)."""
        w = _u8(q6k)
        qs = np.ascontiguousarray(qs, dtype=np.int8).reshape(-1)
        d = _f32(d)
        if d.size * 256 != qs.size:
            return None
        out = np.empty(num_rows if out_len is None else out_len, np.float32)
        ok = self._some(lib.larql_hip_q6k_q8k_matvec(self._h, _ptr(w), w.size, _ptr(qs), qs.size, _ptr(d), num_rows, cols,
                                                     _ptr(out), out.size))
        return out if ok else None

    def q4k_dual_matvec(self, q4k_a, q4k_b, x, num_rows: int, hidden: int):
        a, b, x = _u8(q4k_a), _u8(q4k_b), _f32(x)
        oa, ob = np.empty(num_rows, np.float32), np.empty(num_rows, np.float32)
        ok = self._some(lib.larql_hip_q4k_dual_matvec(self._h, _ptr(a), a.size, _ptr(b), b.size, _ptr(x), x.size,
                                                      num_rows, hidden, _ptr(oa), _ptr(ob), num_rows))
        return (oa, ob) if ok else None

    def q4k_matmul(self, q4k_data, x, num_rows: int, hidden: int, seq_len: int):
        w, x = _u8(q4k_data), _f32(x)
        out = np.empty(seq_len * num_rows, np.float32)
        ok = self._some(lib.larql_hip_q4k_matmul(self._h, _ptr(w), w.size, _ptr(x), x.size, num_rows, hidden, seq_len,
                                                 _ptr(out), out.size))
        return out if ok else None

    def q4k_matvec_topk(self, q4k_data, x, num_rows: int, hidden: int, top_k: int):
        w, x = _u8(q4k_data), _f32(x)
        idx = np.empty(max(top_k, 1), np.uint32)
        val = np.empty(max(top_k, 1), np.float32)
        n = C.c_size_t(0)
        ok = self._some(lib.larql_hip_q4k_matvec_topk(self._h, _ptr(w), w.size, _ptr(x), x.size, num_rows, hidden, top_k,
                                                      _ptr(idx), _ptr(val), C.byref(n)))
        return [(int(idx[i]), float(val[i])) for i in range(n.value)] if ok else None

    def q4_matvec(self, q4_data, q8_x, q8_scales, num_rows: int, hidden: int):
        w = _u8(q4_data)
        q8 = np.ascontiguousarray(q8_x, dtype=np.int8).reshape(-1)
        sc = _f32(q8_scales)
        out = np.empty(num_rows, np.float32)
        ok = self._some(lib.larql_hip_q4_matvec(self._h, _ptr(w), w.size, _ptr(q8), q8.size, _ptr(sc), sc.size, num_rows,
                                                hidden, _ptr(out)))
        return out if ok else None

    def q8_0_gemv(self, blocks, x, n: int, k: int):
        w, x = _u8(blocks), _f32(x)
        out = np.empty(n, np.float32)
        ok = self._some(lib.larql_hip_q8_0_gemv(self._h, _ptr(w), w.size, _ptr(x), x.size, n, k, _ptr(out)))
        return out if ok else None

    def quant_matvec(self, fmt: int, weights, x, num_rows: int, hidden: int):
        w, x = _u8(weights), _f32(x)
        out = np.empty(num_rows, np.float32)
        ok = self._some(lib.larql_hip_quant_matvec(self._h, fmt, _ptr(w), w.size, _ptr(x), x.size, num_rows, hidden, _ptr(out)))
        return out if ok else None

    def quant_matvec_q8_input(self, fmt: int, weights, q8_x, q8_scales, num_rows: int, hidden: int):
        """QuantMatVec::quant_matvec_q8_input (backend/quant_matvec.rs:100-151)."""
        w = _u8(weights)
        q8 = np.ascontiguousarray(q8_x, dtype=np.int8).reshape(-1)
        sc = _f32(q8_scales)
        out = np.empty(num_rows, np.float32)
        ok = self._some(lib.larql_hip_quant_matvec_q8_input(self._h, fmt, _ptr(w), w.size, _ptr(q8), q8.size, _ptr(sc), sc.size,
                                                            num_rows, hidden, _ptr(out)))
        return out if ok else None

    def q8_0_gemv_topk(self, blocks, x, n: int, k: int, top_k: int):
        """lm_head KNN over a ggml Q8_0 head (lm_head/knn.rs:126-185): [(row, score)] by value descending."""
        w, x = _u8(blocks), _f32(x)
        idx = np.empty(max(top_k, 1), np.uint32)
        val = np.empty(max(top_k, 1), np.float32)
        cnt = C.c_size_t(0)
        ok = self._some(lib.larql_hip_q8_0_gemv_topk(self._h, _ptr(w), w.size, _ptr(x), x.size, n, k, top_k, _ptr(idx), _ptr(val),
                                                     C.byref(cnt)))
        return [(int(idx[i]), float(val[i])) for i in range(cnt.value)] if ok else None

    # -- MatMul ------------------------------------------------------------------------
    def _dense(self, fn, w, x, n, k, force):
        w, x = _u8(w), _f32(x)
        out = np.empty(n, np.float32)
        ok = self._some(fn(self._h, _ptr(w), w.size, _ptr(x), x.size, n, k, _ptr(out), int(force)))
        return out if ok else None

    def f32_gemv(self, w, x):
        w = np.ascontiguousarray(w, dtype=np.float32)
        return self._dense(lib.larql_hip_f32_gemv, w, x, w.shape[0], w.shape[1], False)

    def f32_gemv_force(self, w, x):
        w = np.ascontiguousarray(w, dtype=np.float32)
        return self._dense(lib.larql_hip_f32_gemv, w, x, w.shape[0], w.shape[1], True)

    def f16_gemv(self, w_f16, x, n: int, k: int):
        return self._dense(lib.larql_hip_f16_gemv, w_f16, x, n, k, False)

    def f16_gemv_force(self, w_f16, x, n: int, k: int):
        return self._dense(lib.larql_hip_f16_gemv, w_f16, x, n, k, True)

    def bf16_gemv(self, w_bf16, x, n: int, k: int):
        return self._dense(lib.larql_hip_bf16_gemv, w_bf16, x, n, k, False)

    def bf16_gemv_force(self, w_bf16, x, n: int, k: int):
        return self._dense(lib.larql_hip_bf16_gemv, w_bf16, x, n, k, True)

    def _dense_multi(self, fn, weights: Sequence[Tuple[np.ndarray, int, int]], x):
        m = len(weights)
        x = _f32(x)
        ws = [_u8(w[0]) for w in weights]
        outs = [np.empty(w[1], np.float32) for w in weights]
        VP, SZ = C.c_void_p * max(m, 1), C.c_size_t * max(m, 1)
        rc = fn(self._h, m, VP(*[w.ctypes.data for w in ws]), SZ(*[w.size for w in ws]), SZ(*[w[1] for w in weights]),
                SZ(*[w[2] for w in weights]), _ptr(x), x.size, VP(*[o.ctypes.data for o in outs]))
        return outs if self._some(rc) else None

    def bf16_gemv_multi(self, weights: Sequence[Tuple[np.ndarray, int, int]], x):
        """MatMul::bf16_gemv_multi (backend/matmul.rs:151-170): [(w_bf16, n, k)] against one x, one submission."""
        return self._dense_multi(lib.larql_hip_bf16_gemv_multi, weights, x)

    def f16_gemv_multi(self, weights: Sequence[Tuple[np.ndarray, int, int]], x):
        """MatMul::f16_gemv_multi (backend/matmul.rs:172-194)."""
        return self._dense_multi(lib.larql_hip_f16_gemv_multi, weights, x)

    def mxfp4_gemv(self, packed, scales, x, n: int, k: int):
        p, s, x = _u8(packed), _u8(scales), _f32(x)
        out = np.empty(n, np.float32)
        ok = self._some(lib.larql_hip_mxfp4_gemv(self._h, _ptr(p), p.size, _ptr(s), s.size, _ptr(x), x.size, n, k, _ptr(out)))
        return out if ok else None

    def mxfp4_gemv_multi(self, weights: Sequence[Tuple[np.ndarray, np.ndarray, int, int]], x):
        m = len(weights)
        x = _f32(x)
        ps = [_u8(w[0]) for w in weights]
        ss = [_u8(w[1]) for w in weights]
        outs = [np.empty(w[2], np.float32) for w in weights]
        VP, SZ = C.c_void_p * max(m, 1), C.c_size_t * max(m, 1)
        rc = lib.larql_hip_mxfp4_gemv_multi(
            self._h, m, VP(*[p.ctypes.data for p in ps]), SZ(*[p.size for p in ps]),
            VP(*[s.ctypes.data for s in ss]), SZ(*[s.size for s in ss]),
            SZ(*[w[2] for w in weights]), SZ(*[w[3] for w in weights]), _ptr(x), x.size,
            VP(*[o.ctypes.data for o in outs]))
        return outs if self._some(rc) else None

    # -- gate-KNN (VectorIndex) ------------------------------------------------------------
    def gate_knn_batch_hits(self, fmt: int, gate, x, n_features: int, hidden: int, top_k: int):
        """Per-position hits: list over positions of [(feature, score)] by |score| descending."""
        g = _u8(gate)
        x2 = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, hidden) if hidden else np.zeros((0, 0), np.float32)
        batch = x2.shape[0]
        k = max(top_k, 1)
        idx = np.empty((max(batch, 1), k), np.uint32)
        val = np.empty((max(batch, 1), k), np.float32)
        n_out = (C.c_size_t * max(batch, 1))()
        ok = self._some(lib.larql_hip_gate_knn(self._h, fmt, _ptr(g), g.size, _ptr(x2), batch, n_features, hidden, top_k,
                                               _ptr(idx), _ptr(val), n_out))
        if not ok:
            return None
        return [[(int(idx[b, i]), float(val[b, i])) for i in range(n_out[b])] for b in range(batch)]

    def gate_knn(self, fmt: int, gate, residual, n_features: int, hidden: int, top_k: int):
        """VectorIndex::gate_knn / gate_walk: [(feature, score)] by |score| descending."""
        hits = self.gate_knn_batch_hits(fmt, gate, np.asarray(residual, np.float32).reshape(1, -1), n_features, hidden, top_k)
        return None if hits is None else hits[0]

    def gate_knn_batch(self, fmt: int, gate, x, n_features: int, hidden: int, top_k: int) -> Optional[List[int]]:
        """VectorIndex::gate_knn_batch: sorted, de-duplicated union of the per-position hits."""
        hits = self.gate_knn_batch_hits(fmt, gate, x, n_features, hidden, top_k)
        if hits is None:
            return None
        return sorted({i for pos in hits for (i, _) in pos})

    def gate_scores_batch(self, fmt: int, gate, x, n_features: int, hidden: int):
        g = _u8(gate)
        x2 = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, hidden)
        out = np.empty((x2.shape[0], n_features), np.float32)
        ok = self._some(lib.larql_hip_gate_scores(self._h, fmt, _ptr(g), g.size, _ptr(x2), x2.shape[0], n_features, hidden,
                                                  _ptr(out)))
        return out if ok else None

    # -- device tier -------------------------------------------------------------------------------
    def malloc(self, nbytes: int) -> int:
        p = C.c_void_p()
        self._some(lib.larql_hip_malloc(self._h, C.byref(p), nbytes))
        return p.value

    def free(self, dptr: int) -> None:
        self._some(lib.larql_hip_free(self._h, dptr))

    def h2d(self, dptr: int, a: np.ndarray) -> None:
        a = np.ascontiguousarray(a)
        self._some(lib.larql_hip_memcpy_h2d(self._h, dptr, _ptr(a), a.nbytes))

    def d2h(self, dptr: int, shape, dtype) -> np.ndarray:
        out = np.empty(shape, dtype)
        self._some(lib.larql_hip_memcpy_d2h(self._h, _ptr(out), dptr, out.nbytes))
        return out

    def to_device(self, a: np.ndarray) -> int:
        a = np.ascontiguousarray(a)
        p = self.malloc(max(a.nbytes, 1) + 64)
        if a.nbytes:
            self.h2d(p, a)
        return p

    def synchronize(self) -> None:
        self._some(lib.larql_hip_synchronize(self._h))

    def event(self) -> int:
        e = C.c_void_p()
        self._some(lib.larql_hip_event_create(self._h, C.byref(e)))
        return e.value

    def record(self, ev: int) -> None:
        self._some(lib.larql_hip_event_record(self._h, ev))

    def elapsed_ms(self, a: int, b: int) -> float:
        ms = C.c_float()
        self._some(lib.larql_hip_event_elapsed_ms(self._h, a, b, C.byref(ms)))
        return ms.value

    def dev_copy(self, dst: Optional[int], src: int, nbytes: int) -> bool:
        return self._some(lib.larql_hip_dev_copy(self._h, dst, src, nbytes))

    def dev_matvec(self, fmt: int, w: int, aux: Optional[int], x: int, rows: int, k: int, out: int) -> bool:
        return self._some(lib.larql_hip_dev_matvec(self._h, fmt, w, aux, x, rows, k, out))

    def dev_matvec_batch(self, jobs: Sequence[tuple]) -> bool:
        """jobs: (fmt, w, aux, x, out, rows, k) with device pointers."""
        arr = (L.MatvecJob * max(len(jobs), 1))()
        for i, (fmt, w, aux, x, out, rows, k) in enumerate(jobs):
            arr[i] = L.MatvecJob(fmt, 0, w, aux, x, out, rows, k)
        return self._some(lib.larql_hip_dev_matvec_batch(self._h, arr, len(jobs)))

    def plan_create(self, jobs: Sequence[tuple]) -> Optional[int]:
        """Record a submission of (fmt, w, aux, x, out, rows, k) jobs; returns a plan handle or None."""
        arr = (L.MatvecJob * max(len(jobs), 1))()
        for i, (fmt, w, aux, x, out, rows, k) in enumerate(jobs):
            arr[i] = L.MatvecJob(fmt, 0, w, aux, x, out, rows, k)
        p = C.c_void_p()
        ok = self._some(lib.larql_hip_plan_create(self._h, arr, len(jobs), C.byref(p)))
        return p.value if ok else None

    def plan_run(self, plan: int) -> bool:
        return self._some(lib.larql_hip_plan_run(self._h, plan))

    def plan_launch_count(self, plan: int) -> int:
        return lib.larql_hip_plan_launch_count(plan)

    def plan_destroy(self, plan: int) -> None:
        lib.larql_hip_plan_destroy(self._h, plan)

    def sequence_create(self, plans: Sequence[int]) -> Optional[int]:
        """Plans that depend on one another, in order, as one replayable submission (a HIP graph); None on failure."""
        arr = (C.c_void_p * max(len(plans), 1))(*plans)
        p = C.c_void_p()
        ok = self._some(lib.larql_hip_sequence_create(self._h, arr, len(plans), C.byref(p)))
        return p.value if ok else None

    def sequence_run(self, seq: int) -> bool:
        return self._some(lib.larql_hip_sequence_run(self._h, seq))

    def sequence_launch_count(self, seq: int) -> int:
        return lib.larql_hip_sequence_launch_count(seq)

    def sequence_destroy(self, seq: int) -> None:
        lib.larql_hip_sequence_destroy(self._h, seq)

    def dev_gate_knn(self, fmt: int, gate: int, x: int, batch: int, n: int, hidden: int, top_k: int, scores: int, idx: int,
                     val: int, counts: Optional[int] = None) -> bool:
        return self._some(lib.larql_hip_dev_gate_knn(self._h, fmt, gate, x, batch, n, hidden, top_k, scores, idx, val, counts))

    def dev_take_nan_flag(self) -> bool:
        """True if the last device-tier gate-KNN / gate walk met a NaN score (waits for the stream, clears the flag)."""
        f = C.c_int(0)
        self._some(lib.larql_hip_dev_take_nan_flag(self._h, C.byref(f)))
        return bool(f.value)

    def debug_alloc_events(self) -> int:
        """Allocations, stagings and table uploads made through this context so far (host-side counter)."""
        v = L.u64()
        self._some(lib.larql_hip_debug_alloc_events(self._h, C.byref(v)))
        return v.value

    def static_scratch_bytes(self) -> int:
        return int(lib.larql_hip_static_scratch_bytes())

    def dev_gate_knn_static(self, fmt: int, gate: int, x: int, batch: int, n: int, hidden: int, top_k: int, idx: int,
                            val: int, counts: Optional[int] = None) -> bool:
        """larql_hip_dev_gate_knn without any allocation (scores live in the library's static device array)."""
        return self._some(lib.larql_hip_dev_gate_knn_static(self._h, fmt, gate, x, batch, n, hidden, top_k, idx, val, counts))

    def dev_gate_walk(self, fmt: int, gates: Sequence[int], x: int, x_layer_stride: int, batch: int, n: int, hidden: int,
                      top_k: int, scores: int, idx: int, val: int, count: Optional[int] = None) -> bool:
        arr = (C.c_void_p * max(len(gates), 1))(*gates)
        return self._some(lib.larql_hip_dev_gate_walk(self._h, fmt, arr, len(gates), x, x_layer_stride, batch, n, hidden, top_k,
                                                      scores, idx, val, count))

    def dev_q4k_gemm(self, w: int, x_bf16: int, rows: int, hidden: int, seq: int, out: int) -> bool:
        return self._some(lib.larql_hip_dev_q4k_gemm(self._h, w, x_bf16, rows, hidden, seq, out))

    def dev_q4k_row_exponents(self, w: int, rows: int, hidden: int, row_exp: int) -> bool:
        """The rows' exponents of a resident Q4_K matrix (int32[rows], device memory): once per matrix."""
        return self._some(lib.larql_hip_dev_q4k_row_exponents(self._h, w, rows, hidden, row_exp))

    def dev_q4k_gemm_prepared(self, w: int, row_exp: int, x_bf16: int, rows: int, hidden: int, seq: int, out: int) -> bool:
        """dev_q4k_gemm with the rows' exponents from dev_q4k_row_exponents (bit-identical results)."""
        return self._some(lib.larql_hip_dev_q4k_gemm_prepared(self._h, w, row_exp, x_bf16, rows, hidden, seq, out))

    def dev_router_select(self, logits: int, tokens: int, n_experts: int, k: int, policy: int, experts: int, weights: int) -> bool:
        return self._some(lib.larql_hip_dev_router_select(self._h, logits, tokens, n_experts, k, policy, experts, weights))

    def moe_mxfp4_workspace_bytes(self, tokens: int, k: int, hidden: int, inter: int) -> int:
        return lib.larql_hip_moe_mxfp4_workspace_bytes(tokens, k, hidden, inter)

    def dev_moe_mxfp4(self, bank: "L.Mxfp4Experts", x: int, tokens: int, k: int, experts: int, weights: int, out: int,
                      workspace: int, workspace_bytes: int) -> bool:
        return self._some(lib.larql_hip_dev_moe_mxfp4(self._h, C.byref(bank), x, tokens, k, experts, weights, out, workspace,
                                                      workspace_bytes))

    def dev_moe_mxfp4_routed(self, bank: "L.Mxfp4Experts", x: int, tokens: int, k: int, logits: int, policy: int, experts: int,
                             weights: int, out: int, workspace: int, workspace_bytes: int) -> bool:
        """Router::select and the expert block in one call (one launch fewer for a single token); experts / weights are
        written as dev_router_select writes them."""
        return self._some(lib.larql_hip_dev_moe_mxfp4_routed(self._h, C.byref(bank), x, tokens, k, logits, policy, experts, weights,
                                                             out, workspace, workspace_bytes))

    # -- MoE layer: per-expert slices, split scale streams and the router (MoeLayerWeights) ----------------------
    def moe_layer_create(self, experts_gate_up, experts_down, scales_gate_up, scales_down, router_proj, top_k: int, hidden: int,
                         inter: int, fused_row_layout: int = L.MOE_ROWS_INTERLEAVED, router_bias=None, gate_up_bias=None,
                         down_bias=None, per_expert_scale=None, renormalized: bool = True, expert_scales: int = L.MOE_SCALES_PAIRED,
                         expert_data_format: int = L.FMT_MXFP4, limit: float = 7.0, alpha: float = 1.702,
                         gate_rule: int = L.MOE_GATE_CLAMPED_GLU) -> Optional[int]:
        """experts_gate_up / experts_down / scales_*: one uint8 array per expert (separate allocations, as mmap ranges
        would be); a Q4_K / Q6_K bank has no scale tables (None, MOE_SCALES_INLINE) and ContiguousHalves rows.  Returns a
        layer handle, or None where the backend refuses the layer."""
        n = len(experts_gate_up)
        keep = []  # host arrays have to outlive the call

        def table(arrs):
            if arrs is None:
                return None, None
            a = [np.ascontiguousarray(x, dtype=np.uint8).ravel() for x in arrs]
            keep.append(a)
            ptrs = (vp_t * max(len(a), 1))(*[x.ctypes.data for x in a])
            lens = (C.c_size_t * max(len(a), 1))(*[x.size for x in a])
            keep.append((ptrs, lens))
            return C.cast(ptrs, C.POINTER(vp_t)), C.cast(lens, C.POINTER(C.c_size_t))

        def f32(a):
            if a is None:
                return None
            a = np.ascontiguousarray(a, dtype=np.float32)
            keep.append(a)
            return a.ctypes.data
        vp_t = C.c_void_p
        w = L.MoeLayerWeights()
        w.num_experts, w.top_k, w.hidden, w.intermediate_size = n, top_k, hidden, inter
        w.expert_data_format, w.fused_row_layout, w.expert_scales = expert_data_format, fused_row_layout, expert_scales
        w.experts_gate_up, w.experts_gate_up_len = table(experts_gate_up)
        w.experts_down, w.experts_down_len = table(experts_down)
        sg, sgl = table(scales_gate_up)
        sd, sdl = table(scales_down)
        if sg is not None:
            w.scales_gate_up, w.scales_gate_up_len = sg, sgl
        if sd is not None:
            w.scales_down, w.scales_down_len = sd, sdl
        w.router_proj, w.router_bias = f32(router_proj), f32(router_bias)
        w.experts_gate_up_bias, w.experts_down_bias = f32(gate_up_bias), f32(down_bias)
        w.router_per_expert_scale = f32(per_expert_scale)
        w.renormalized_softmax, w.per_expert_scale = int(renormalized), int(per_expert_scale is not None)
        w.glu_limit, w.glu_alpha, w.gate_rule = limit, alpha, gate_rule
        h = C.c_void_p()
        ok = self._some(lib.larql_hip_moe_layer_create(self._h, C.byref(w), C.byref(h)))
        return h.value if ok else None

    def moe_layer_destroy(self, layer: int) -> None:
        lib.larql_hip_moe_layer_destroy(self._h, layer)

    def moe_layer_forward(self, layer: int, router_in, x, top_k: int):
        """Host tier: (out [tokens, hidden], experts [tokens, k], weights [tokens, k]) or None."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        rin = x if router_in is x else np.ascontiguousarray(router_in, dtype=np.float32)
        tokens = x.shape[0]
        out = np.empty_like(x)
        ex, wt = np.zeros((tokens, top_k), np.uint32), np.zeros((tokens, top_k), np.float32)
        ok = self._some(lib.larql_hip_moe_layer_forward(self._h, layer, rin.ctypes.data, x.ctypes.data, tokens, out.ctypes.data,
                                                        ex.ctypes.data, wt.ctypes.data))
        return (out, ex, wt) if ok else None

    def dev_moe_layer_forward(self, layer: int, router_in: int, x: int, tokens: int, out: int, experts: int, weights: int) -> bool:
        return self._some(lib.larql_hip_dev_moe_layer_forward(self._h, layer, router_in, x, tokens, out, experts, weights))

    def dev_quantize_q4_k(self, src: int, n: int, dst: int) -> bool:
        return self._some(lib.larql_hip_dev_quantize_q4_k(self._h, src, n, dst))

    def dev_quantize_q6_k(self, src: int, n: int, dst: int) -> bool:
        return self._some(lib.larql_hip_dev_quantize_q6_k(self._h, src, n, dst))

    def dev_quantize_q8_0(self, src: int, n: int, dst: int) -> bool:
        return self._some(lib.larql_hip_dev_quantize_q8_0(self._h, src, n, dst))

    def dev_quantize_mxfp4(self, src: int, rows: int, k: int, packed: int, scales: int) -> bool:
        return self._some(lib.larql_hip_dev_quantize_mxfp4(self._h, src, rows, k, packed, scales))

    def dev_f32_to_bf16(self, src: int, n: int, dst: int) -> bool:
        return self._some(lib.larql_hip_dev_f32_to_bf16(self._h, src, n, dst))

    def dev_quantize_q4_0(self, src: int, n: int, dst: int) -> bool:
        return self._some(lib.larql_hip_dev_quantize_q4_0(self._h, src, n, dst))

    def dev_quantize_to_q8(self, src: int, n: int, q8: int, scales: int) -> bool:
        return self._some(lib.larql_hip_dev_quantize_to_q8(self._h, src, n, q8, scales))

    def q8k_bytes(self, n: int) -> int:
        return int(lib.larql_hip_q8k_bytes(n))

    def dev_quantize_x_to_q8k(self, x: int, n: int, q8k: int) -> bool:
        return self._some(lib.larql_hip_dev_quantize_x_to_q8k(self._h, x, n, q8k))

    def dev_fill_normal(self, dst: int, n: int, seed: int, sigma: float) -> bool:
        return self._some(lib.larql_hip_dev_fill_normal(self._h, dst, n, seed, sigma))
