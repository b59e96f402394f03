#!/usr/bin/env python3
"""Benchmark of the quantised decode matvec stack on one MI355X.

Workload (BASELINE.json configs[1]): the full decode-step matvec stack at
Gemma-3-4B shapes, batch 1 — per layer q 2048x2560, k/v 1024x2560, o 2560x2048,
gate/up 10240x2560, down 2560x10240 in Q4_K, 34 distinct layers, then the
lm_head 262144x2560 in ggml Q8_0.  Weights are N(0, 0.02) drawn on the device
from a seeded counter generator and quantised on the device with the
reference's encoders (bit-exact kernels); every matvec has its own N(0, 1)
activation.  One step = one token = all 239 matvecs, submitted as two recorded
launches (238 Q4_K jobs, 1 Q8_0 job); inputs are resident in HBM before the
timed region.

Prints ONE JSON line: whole-job HBM throughput in GB/s over the algorithmic
bytes (weight bytes + 4*K + 4*N per matvec), plus `roofline` for the dominant
kernel (Q4_K matvec, timed with HIP events on the launch stream inside the timed
region) and `cpu_baseline` (the CPU oracle's restatement of the reference
kernels, multi-threaded, on a bounded sample of the same weights).

The headline step submits the 239 matvecs as mutually independent jobs: it is
a streaming-bandwidth figure, not a decode rate.  `decode_in_dependency_order`
(beside `value`; in full under `config.dependency_ordered`)
reports the same weights walked as a token would walk them — per layer the
stages q,k,v | o | gate,up | down, each stage reading the previous stage's
output, 137 dependent launches — with its own ms per token.  `config.other_configs`
carries a short run of BASELINE's other configurations and of the other block
formats of the matvec family (Q6_K, MXFP4), each verified against the oracle in
the same run, `config.host_tier_us_per_call` what a trait-shaped
call on host slices costs end to end.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HIDDEN, LAYERS, VOCAB = 2560, 34, 262144
# (name, rows, k) in trait orientation [num_rows, hidden]
LAYER_MATS = [("q", 2048, 2560), ("k", 1024, 2560), ("v", 1024, 2560), ("o", 2560, 2048),
              ("gate", 10240, 2560), ("up", 10240, 2560), ("down", 2560, 10240)]
HBM_PEAK_GBS = 8000.0
CONFIG_ID = 2  # seeds: 0x5EED0000 + config*256 + tensor_id (mod 2^32 per layer below)


def q4k_bytes(rows, k):
    return rows * (k // 256) * 144


def q8_0_bytes(rows, k):
    return rows * (k // 32) * 34


class Stack:
    """Device-resident weights, activations and outputs of the whole stack."""

    def __init__(self, be, fmt, layers=LAYERS, vocab=VOCAB):
        self.be, self.fmt = be, fmt
        self.q4k_jobs, self.q8_jobs, self.meta = [], [], []
        tmp_elems = max(vocab * HIDDEN, 10240 * 2560)
        tmp = be.malloc(tmp_elems * 4)
        tid = 0
        for layer in range(layers):
            for name, rows, k in LAYER_MATS:
                seed = 0x5EED0000 + CONFIG_ID * 256 + tid
                tid += 1
                w = be.malloc(q4k_bytes(rows, k) + 64)
                assert be.dev_fill_normal(tmp, rows * k, seed, 0.02)
                assert be.dev_quantize_q4_k(tmp, rows * k, w)
                x = be.malloc(k * 4 + 64)
                assert be.dev_fill_normal(x, k, seed ^ 0xA5A50000, 1.0)
                out = be.malloc(rows * 4 + 64)
                self.q4k_jobs.append((fmt.FMT_Q4_K, w, None, x, out, rows, k))
                self.meta.append((f"L{layer}.{name}", "q4k", rows, k))
        seed = 0x5EED0000 + CONFIG_ID * 256 + 0xFFFF
        w = be.malloc(q8_0_bytes(vocab, HIDDEN) + 64)
        assert be.dev_fill_normal(tmp, vocab * HIDDEN, seed, 0.02)
        assert be.dev_quantize_q8_0(tmp, vocab * HIDDEN, w)
        x = be.malloc(HIDDEN * 4 + 64)
        assert be.dev_fill_normal(x, HIDDEN, seed ^ 0xA5A50000, 1.0)
        out = be.malloc(vocab * 4 + 64)
        self.q8_jobs.append((fmt.FMT_GGML_Q8_0, w, None, x, out, vocab, HIDDEN))
        be.synchronize()
        be.free(tmp)
        self.q4k_weight_bytes = sum(q4k_bytes(r, k) for (_, _, _, _, _, r, k) in self.q4k_jobs)
        self.q8_weight_bytes = q8_0_bytes(vocab, HIDDEN)
        self.q4k_algo_bytes = self.q4k_weight_bytes + sum(4 * k + 4 * r for (_, _, _, _, _, r, k) in self.q4k_jobs)
        self.q8_algo_bytes = self.q8_weight_bytes + 4 * HIDDEN + 4 * vocab
        self.plan_q4k = be.plan_create(self.q4k_jobs)
        self.plan_q8 = be.plan_create(self.q8_jobs)
        assert self.plan_q4k and self.plan_q8, be.last_error()

    def step(self):
        self.be.plan_run(self.plan_q4k)
        self.be.plan_run(self.plan_q8)


def _window(rows, idx, n=48):
    """First row of an n-row window of result number idx: the first rows, the last rows, or somewhere inside."""
    return (0, rows - n, ((rows * ((idx * 37) % 97)) // 97) & ~15, (rows // 2 + 8 * idx) % (rows - n))[idx % 4]


def verify_and_cpu_baseline(be, stack, lm_rows=16384, min_seconds=10.0):
    """Check the GPU outputs against the CPU oracle before any time is recorded: every row of layer 0's seven
    matvecs, a 48-row window of EVERY other Q4_K result of the launch (all layers, all seven matrices; windows at the
    first rows, the last rows and inside), and three lm_head windows (first, middle and last rows).  Then time the
    oracle (the reference's CPU algorithm restated, row-chunk threaded as the reference schedules it) on layer 0 +
    the first lm_head rows."""
    O = _oracle()
    threads = cpu_threads()
    sample, worst = [], 0.0

    def rel(got, want):
        return float(np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want))
    for (f, w, _, x, out, rows, k), (name, kind, _, _) in zip(stack.q4k_jobs[:7], stack.meta[:7]):
        wb = be.d2h(w, q4k_bytes(rows, k), np.uint8)
        xv = be.d2h(x, k, np.float32)
        worst = max(worst, rel(be.d2h(out, rows, np.float32), O.q4k_matvec_mt(wb, xv, rows, k, threads)))
        sample.append(("q4k", wb, xv, rows, k))
    windows = 7
    for idx, (f, w, _, x, out, rows, k) in enumerate(stack.q4k_jobs[7:], start=7):
        r0 = _window(rows, idx)
        wb = be.d2h(w + r0 * (k // 256) * 144, q4k_bytes(48, k), np.uint8)
        worst = max(worst, rel(be.d2h(out + 4 * r0, 48, np.float32), O.q4k_matvec(wb, be.d2h(x, k, np.float32), 48, k)))
        windows += 1
    (f, w, _, x, out, rows, k) = stack.q8_jobs[0]
    lm_rows = min(lm_rows, rows)
    xv = be.d2h(x, k, np.float32)
    for r0, n in ((0, lm_rows), (rows // 2 - 1000, 2048), (rows - 2048, 2048)):
        if r0 < 0 or r0 + n > rows or (r0 and r0 < lm_rows):
            continue
        wb = be.d2h(w + r0 * (k // 32) * 34, q8_0_bytes(n, k), np.uint8)
        worst = max(worst, rel(be.d2h(out + 4 * r0, n, np.float32), O.q8_0_gemv_mt(wb, xv, n, k, threads)))
        if r0 == 0:
            sample.append(("q8", wb, xv, n, k))
    if not worst < 1e-3:
        raise SystemExit(f"bench: GPU outputs differ from the CPU oracle (rel-L2 {worst:.3e}); no number recorded")
    stack.verified = f"{windows} of {len(stack.q4k_jobs)} Q4_K results (layer 0 in full, a 48-row window of every other) + 3 lm_head windows"

    sample_bytes = sum(s[1].nbytes for s in sample)

    def one_pass():
        for kind, wb, xv, rows, k in sample:
            (O.q4k_matvec_mt if kind == "q4k" else O.q8_0_gemv_mt)(wb, xv, rows, k, threads)

    one_pass()
    times = []
    t_end = time.perf_counter() + min_seconds
    while time.perf_counter() < t_end or len(times) < 5:
        t0 = time.perf_counter()
        one_pass()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    # one thread, on the two largest matvecs of the sample
    kind, wb1, xv1, rows1, k1 = sample[4]
    med1, n1 = _cpu_time(lambda: O.q4k_matvec_mt(wb1, xv1, rows1, k1, 1), max(1.0, min_seconds / 5))
    return worst, {
        "value": round(sample_bytes / med / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": f"layer 0 (7 Q4_K matvecs) + first {lm_rows} lm_head rows (Q8_0), {sample_bytes / 1e6:.1f} MB, "
                  f"median of {len(times)} passes",
        "build": _NATIVE, "one_thread_GBps": round(wb1.nbytes / med1 / 1e9, 3),
        "one_thread_sample": f"gate 10240x2560 Q4_K, median of {n1}",
        "stack_steps_per_s_extrapolated": round(1.0 / (med * (stack.q4k_weight_bytes + stack.q8_weight_bytes) / sample_bytes), 3),
    }


class Chain:
    """The stack's own weights walked in dependency order: per layer the stages q,k,v | o | gate,up | down, each stage
    reading the previous stage's output (no norms, attention or activations between them: the matvec launches of a
    token and their dependencies, nothing else), then the lm_head on the last layer's output."""

    def __init__(self, be, fmt, stack, graph=True):
        self.be, self.plans, self.jobs = be, [], []
        layers = len(stack.q4k_jobs) // 7
        self.h0 = be.malloc(HIDDEN * 4 + 64)
        assert be.dev_fill_normal(self.h0, HIDDEN, 0x5EED02C0, 1.0)
        h = self.h0
        for l in range(layers):
            w = [j[1] for j in stack.q4k_jobs[7 * l:7 * l + 7]]
            buf = {n: be.malloc(r * 4 + 64) for n, r in (("q", 2048), ("k", 1024), ("v", 1024), ("o", 2560), ("gate", 10240), ("up", 10240), ("down", 2560))}
            stages = [[(fmt.FMT_Q4_K, w[0], None, h, buf["q"], 2048, 2560), (fmt.FMT_Q4_K, w[1], None, h, buf["k"], 1024, 2560),
                       (fmt.FMT_Q4_K, w[2], None, h, buf["v"], 1024, 2560)],
                      [(fmt.FMT_Q4_K, w[3], None, buf["q"], buf["o"], 2560, 2048)],
                      [(fmt.FMT_Q4_K, w[4], None, buf["o"], buf["gate"], 10240, 2560), (fmt.FMT_Q4_K, w[5], None, buf["o"], buf["up"], 10240, 2560)],
                      [(fmt.FMT_Q4_K, w[6], None, buf["gate"], buf["down"], 2560, 10240)]]
            for st in stages:
                p = be.plan_create(st)
                assert p, be.last_error()
                self.plans.append(p)
                self.jobs.extend(st)
            h = buf["down"]
        f, w, _, _, out, rows, k = stack.q8_jobs[0]
        p = be.plan_create([(f, w, None, h, out, rows, k)])
        assert p, be.last_error()
        self.plans.append(p)
        self.lm_head = (w, h, out, rows, k)

        self.seq = None
        if graph:
            self.seq = be.sequence_create(self.plans)   # the same launches recorded once as a HIP graph
            assert self.seq, be.last_error()

    def step(self):
        """One token: the recorded sequence (one submission); without one, a host call per stage."""
        if self.seq is None:
            return self.step_eager()
        self.be.sequence_run(self.seq)

    def step_eager(self):
        """One token, a host call per stage (137 submissions)."""
        for p in self.plans:
            self.be.plan_run(p)

    def verify(self, O):
        """Every stage of the walk against the oracle, each on the activation the GPU itself read (the stage before
        it wrote it): layer 0's chain in full from h0 (h0 -> q -> o -> gate -> down), then a 48-row window of every
        one of the walk's Q4_K results through the last layer, then three windows of the lm_head on the last layer's
        output.  By induction over the stages the whole token is held to the oracle."""
        be = self.be
        threads = cpu_threads()

        def rel(got, want):
            return float(np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want))
        x = be.d2h(self.h0, HIDDEN, np.float32)
        worst = 0.0
        for ji in (0, 3, 4, 6):                                     # q, o, gate, down of layer 0, chained on the CPU
            _, w, _, _, out, rows, k = self.jobs[ji]
            x = O.q4k_matvec_mt(be.d2h(w, q4k_bytes(rows, k), np.uint8), x, rows, k, threads)
            worst = max(worst, rel(be.d2h(out, rows, np.float32), x))
        for idx, (_, w, _, xin, out, rows, k) in enumerate(self.jobs):
            r0 = _window(rows, idx)
            wb = be.d2h(w + r0 * (k // 256) * 144, q4k_bytes(48, k), np.uint8)
            want = O.q4k_matvec(wb, be.d2h(xin, k, np.float32), 48, k)
            worst = max(worst, rel(be.d2h(out + 4 * r0, 48, np.float32), want))
        w, xin, out, rows, k = self.lm_head
        xv = be.d2h(xin, k, np.float32)
        for r0 in (0, rows // 2 - 1000, rows - 2048):
            wb = be.d2h(w + r0 * (k // 32) * 34, q8_0_bytes(2048, k), np.uint8)
            worst = max(worst, rel(be.d2h(out + 4 * r0, 2048, np.float32), O.q8_0_gemv_mt(wb, xv, 2048, k, threads)))
        return worst


PRE_WARM_S = 0.2  # untimed stretch of the same work before each arm: GPU clocks ramp for milliseconds after idling


def _timeit(be, fn, reps, warm=2):
    t = time.perf_counter()
    while time.perf_counter() - t < PRE_WARM_S:
        for _ in range(10):
            fn()
        be.synchronize()
    for _ in range(warm):
        fn()
    be.synchronize()
    e0, e1 = be.event(), be.event()
    be.record(e0)
    for _ in range(reps):
        fn()
    be.record(e1)
    return be.elapsed_ms(e0, e1) / reps


_NATIVE = None


def _oracle():
    """The checker, with its timing baselines (*_mt) built for this host's CPU (-O3 -march=native)."""
    global _NATIVE
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle as O  # the checker / CPU baseline; never the product
    if _NATIVE is None:
        _NATIVE = O.enable_native_timing()
    return O


def _cpu_time(fn, seconds):
    fn()
    times, t_end = [], time.perf_counter() + seconds
    while time.perf_counter() < t_end or len(times) < 3:
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return float(np.median(times)), len(times)


_COLLECT = None  # a list while the default run gathers the other configurations' lines instead of printing them


def _emit(metric, value, unit, ms, steps, warmup, config, roofline, cpu, higher=True, dtype="f32"):
    line = {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": round(ms, 5), "higher_is_better": higher, "scaling": "weak", "vs_baseline": None,
            "dtype": dtype, "data": "synthetic", "config": config, "roofline": roofline, "cpu_baseline": cpu}
    if _COLLECT is not None:
        _COLLECT.append(line)
    else:
        print(json.dumps(line))


def cpu_threads():
    """Worker threads of the CPU baseline: the cores this process may use, capped by the host's configured share
    (OMP_NUM_THREADS where the machine sets one)."""
    n = len(os.sched_getaffinity(0))
    try:
        n = min(n, max(1, int(os.environ.get("OMP_NUM_THREADS", n))))
    except ValueError:
        pass
    return n


def run_c1(be, fmt, args):
    """BASELINE configs[0]: Q4_K 3072x1024 matvec, batch 1 (cold: 256 distinct copies in one launch; hot: one copy)."""
    O = _oracle()
    rows, k, copies = 3072, 1024, 256
    tmp = be.malloc(rows * k * 4)
    x = be.malloc(k * 4 + 64)
    be.dev_fill_normal(x, k, 0x5EED0100 ^ 0xA5A50000, 1.0)
    ws, outs = [], []
    for i in range(copies):
        w = be.malloc(q4k_bytes(rows, k) + 64)
        be.dev_fill_normal(tmp, rows * k, 0x5EED0100 + i, 0.02)
        be.dev_quantize_q4_k(tmp, rows * k, w)
        ws.append(w); outs.append(be.malloc(rows * 4 + 64))
    cold = be.plan_create([(fmt.FMT_Q4_K, w, None, x, o, rows, k) for w, o in zip(ws, outs)])
    hot = be.plan_create([(fmt.FMT_Q4_K, ws[0], None, x, o, rows, k) for o in outs])
    be.plan_run(cold); be.synchronize()
    wb, xv = be.d2h(ws[3], q4k_bytes(rows, k), np.uint8), be.d2h(x, k, np.float32)
    want = O.q4k_matvec(wb, xv, rows, k)
    rel = float(np.linalg.norm(be.d2h(outs[3], rows, np.float32).astype(np.float64) - want) / np.linalg.norm(want))
    assert rel < 1e-3, rel
    algo = q4k_bytes(rows, k) + 4 * k + 4 * rows
    ms_cold = _timeit(be, lambda: be.plan_run(cold), args.steps)
    ms_hot = _timeit(be, lambda: be.plan_run(hot), args.steps)
    ms_one = _timeit(be, lambda: be.dev_matvec(fmt.FMT_Q4_K, ws[5], None, x, rows, k, outs[5]), args.steps)
    threads = cpu_threads()
    med, n = _cpu_time(lambda: O.q4k_matvec_mt(wb, xv, rows, k, threads), args.cpu_seconds)
    gbs = copies * algo / ms_cold / 1e6
    _emit("Q4_K 3072x1024 matvec HBM GB/s (cold, 256 distinct copies per launch)", round(gbs, 1), "GB/s", ms_cold, args.steps,
          2, {"workload": "BASELINE configs[0]: Q4_K matvec 3072x1024, batch 1", "us_per_matvec_cold": round(ms_cold * 1e3 / copies, 3),
              "us_per_matvec_hot": round(ms_hot * 1e3 / copies, 3), "GBps_hot": round(copies * algo / ms_hot / 1e6, 1),
              "us_single_launch_device_resident": round(ms_one * 1e3, 2), "verified_rel_l2_vs_oracle": rel},
          {"kernel": "gemv_q4k", "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
          {"value": round(algo / med / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
           "sample": f"one 3072x1024 matvec, median of {n}", "us_per_matvec": round(med * 1e6, 1)})


def run_c3(be, fmt, args):
    """BASELINE configs[2]: gate-KNN 10240x2560, bf16 and Q4_K gates, top-64 by |score|, 34 layers, batch 1 and 8."""
    O = _oracle()
    n, hidden, k, layers = 10240, 2560, 64, 34
    tmp = be.malloc(n * hidden * 4)
    threads = cpu_threads()
    for variant, f, nbytes in (("bf16", fmt.FMT_BF16, 2 * n * hidden), ("q4k", fmt.FMT_Q4_K, q4k_bytes(n, hidden))):
        gates = []
        for layer in range(layers):
            g = be.malloc(nbytes + 64)
            be.dev_fill_normal(tmp, n * hidden, 0x5EED0300 + layer, 0.02)
            (be.dev_f32_to_bf16 if variant == "bf16" else be.dev_quantize_q4_k)(tmp, n * hidden, g)
            gates.append(g)
        for batch in (1, 8):
            x = be.malloc(batch * hidden * 4 + 64)
            be.dev_fill_normal(x, batch * hidden, 0x5EED03F0 + batch, 1.0)
            scores = be.malloc(layers * batch * n * 4)
            idx, val = be.malloc(layers * batch * k * 4), be.malloc(layers * batch * k * 4)

            def walk():  # all 34 layers in one submission (2 launches)
                be.dev_gate_walk(f, gates, x, 0, batch, n, hidden, k, scores, idx, val)
            walk(); be.synchronize()
            # verify the last layer against the oracle
            gb, xv = be.d2h(gates[-1], nbytes, np.uint8), be.d2h(x, (batch, hidden), np.float32)
            got_i = be.d2h(idx, (layers, batch, k), np.uint32)[-1]
            for b in range(batch):
                sc = (O.bf16_gemv(gb.view(np.uint16), xv[b], n, hidden) if variant == "bf16" else O.q4k_matvec(gb, xv[b], n, hidden))
                want = O.top_k_by_abs(sc, k)
                diff = {int(i) for i in got_i[b]} ^ {i for i, _ in want}
                kth = abs(want[-1][1])
                assert all(abs(abs(float(sc[i])) - kth) <= 1e-5 * max(1.0, kth) for i in diff), (variant, batch, b)
            ms = _timeit(be, walk, max(3, args.steps // 5)) / layers
            algo = nbytes + batch * (4 * hidden + 4 * n + 8 * k)

            def cpu_one():
                for b in range(batch):
                    sc = (O.bf16_gemv_mt(gb.view(np.uint16), xv[b], n, hidden, threads) if variant == "bf16"
                          else O.q4k_matvec_mt(gb, xv[b], n, hidden, threads))
                    O.top_k_by_abs(sc, k)

            def cpu_one_thread():  # one position, one thread
                sc = (O.bf16_gemv_mt(gb.view(np.uint16), xv[0], n, hidden, 1) if variant == "bf16" else O.q4k_matvec_mt(gb, xv[0], n, hidden, 1))
                O.top_k_by_abs(sc, k)
            med, nrep = _cpu_time(cpu_one, args.cpu_seconds / 4)
            med1, _ = _cpu_time(cpu_one_thread, args.cpu_seconds / 8)
            _emit(f"gate-KNN top-64 us/layer ({variant} gate 10240x2560, batch {batch})", round(ms * 1e3, 2), "us/layer", ms * layers,
                  max(3, args.steps // 5), 2,
                  {"workload": f"BASELINE configs[2]: vindex gate-KNN walk, {variant} gate, K=64, 34 layers, batch {batch}",
                   "launches_per_walk": 2, "GBps_weights_once": round(algo / ms / 1e6, 1), "topk_identical_up_to_ties": True},
                  {"kernel": f"gemv_{variant} + topk", "bound": "hbm", "achieved": round(algo / ms / 1e6, 1), "peak": HBM_PEAK_GBS,
                   "unit": "GB/s", "frac": round(algo / ms / 1e6 / HBM_PEAK_GBS, 4), "traffic": None},
                  {"value": round(med * 1e6, 1), "unit": "us/layer", "cores": threads, "kind": "port",
                   "sample": f"one layer, batch {batch}, median of {nrep}", "one_thread_us_per_position": round(med1 * 1e6, 1)}, higher=False)
            for p in (x, scores, idx, val):
                be.free(p)
        for g in gates:
            be.free(g)


def run_c4(be, fmt, args):
    """BASELINE configs[3]: MXFP4 MoE experts, 32 experts x (gate, up, down 2880x2880), top-4, batch 1 and 16."""
    O = _oracle()
    E, H, I, k = 32, 2880, 2880, 4
    per = H * I
    tmp = be.malloc(per * 4)
    bufs = {}
    for name, seed in (("gate", 0x5EED0400), ("up", 0x5EED0440), ("down", 0x5EED0480)):
        p, s = be.malloc(E * per // 2 + 64), be.malloc(E * per // 32 + 64)
        for e in range(E):
            be.dev_fill_normal(tmp, per, seed + e, 0.02)
            be.dev_quantize_mxfp4(tmp, H if name != "down" else H, I if name != "down" else I, p + e * per // 2, s + e * per // 32)
        bufs[name] = (p, s)
    # the same experts as one fused gate_up region each, gate on the even and up on the odd rows (what a GPT-OSS checkpoint ships)
    fp, fs = be.malloc(E * per + 64), be.malloc(E * per // 16 + 64)
    tmp2 = be.malloc(2 * per * 4)
    for e in range(E):
        be.dev_fill_normal(tmp2, 2 * per, 0x5EED04C0 + e, 0.02)
        be.dev_quantize_mxfp4(tmp2, 2 * I, H, fp + e * per, fs + e * per // 16)
    be.free(tmp2)
    banks = {"separate": fmt.Mxfp4Experts(bufs["gate"][0], bufs["gate"][1], bufs["up"][0], bufs["up"][1], bufs["down"][0], bufs["down"][1],
                                          E, H, I, 7.0, 1.702, 0),
             "interleaved": fmt.Mxfp4Experts(fp, fs, None, None, bufs["down"][0], bufs["down"][1], E, H, I, 7.0, 1.702, 1)}
    expert_bytes = 3 * (per // 2 + per // 32)
    for T, layout in ((1, "separate"), (1, "interleaved"), (16, "separate"), (16, "interleaved")):
        bank = banks[layout]
        x, lg = be.malloc(T * H * 4 + 64), be.malloc(T * E * 4 + 64)
        be.dev_fill_normal(x, T * H, 0x5EED04F0 + T, 1.0)
        be.dev_fill_normal(lg, T * E, 0x5EED04E0 + T, 1.0)
        de, dw, out = be.malloc(T * k * 4), be.malloc(T * k * 4), be.malloc(T * H * 4)
        wsb = be.moe_mxfp4_workspace_bytes(T, k, H, I)
        ws = be.malloc(wsb)

        def block():  # Router::select + the expert block (one token: the selection runs inside the first matvec launch)
            be.dev_moe_mxfp4_routed(bank, x, T, k, lg, 1, de, dw, out, ws, wsb)
        block(); be.synchronize()
        experts = be.d2h(de, (T, k), np.uint32)
        distinct = len(set(int(v) for v in experts.reshape(-1)))
        # verify token 0 against the oracle
        xv, lv, wv = be.d2h(x, (T, H), np.float32), be.d2h(lg, (T, E), np.float32), be.d2h(dw, (T, k), np.float32)
        acc = np.zeros(H, np.float32)
        mats = {}
        for (e, w) in O.router_select(lv[0], k):
            for name in ("gate", "up", "down"):
                mats[name] = (be.d2h(bufs[name][0] + e * per // 2, per // 2, np.uint8), be.d2h(bufs[name][1] + e * per // 32, per // 32, np.uint8))
            if layout == "interleaved":
                G = H // 32
                fpe, fse = be.d2h(fp + e * per, per, np.uint8).reshape(2 * I, G * 16), be.d2h(fs + e * per // 16, per // 16, np.uint8).reshape(2 * I, G)
                mats["gate"] = (fpe[0::2].reshape(-1).copy(), fse[0::2].reshape(-1).copy())
                mats["up"] = (fpe[1::2].reshape(-1).copy(), fse[1::2].reshape(-1).copy())
            g = O.mxfp4_gemv(*mats["gate"], xv[0], I, H); u = O.mxfp4_gemv(*mats["up"], xv[0], I, H)
            h = np.array([O.clamped_glu(float(a), float(b)) for a, b in zip(g, u)], np.float32)
            acc = (acc + np.float32(w) * O.mxfp4_gemv(*mats["down"], h, H, I)).astype(np.float32)
        got = be.d2h(out, (T, H), np.float32)[0]
        rel = float(np.linalg.norm(got.astype(np.float64) - acc) / np.linalg.norm(acc))
        assert rel < 1e-3, rel
        ms = _timeit(be, block, args.steps)
        algo = distinct * expert_bytes + T * (8 * H + 4 * E)
        threads = cpu_threads()
        med, nrep = _cpu_time(lambda: O.mxfp4_gemv_mt(*mats["gate"], xv[0], I, H, threads), args.cpu_seconds / 4)
        _emit(f"MXFP4 MoE expert block us (32 experts, top-4, batch {T}, gate/up {layout})", round(ms * 1e3, 2), "us/block", ms, args.steps, 2,
              {"workload": f"BASELINE configs[3]: MXFP4 experts 32 x (gate, up, down 2880x2880), top-4, batch {T}",
               "gate_up_layout": layout, "distinct_experts": distinct, "launches_per_block": 4 if T > 1 else 2, "GBps_over_distinct_expert_bytes": round(algo / ms / 1e6, 1),
               "us_per_expert_matvec": round(ms * 1e3 / (3 * T * k), 2), "verified_rel_l2_vs_oracle": rel},
              {"kernel": "gemv_mxfp4 (gate/up + down launches)", "bound": "hbm", "achieved": round(algo / ms / 1e6, 1), "peak": HBM_PEAK_GBS,
               "unit": "GB/s", "frac": round(algo / ms / 1e6 / HBM_PEAK_GBS, 4), "traffic": None},
              {"value": round(med * 1e6 * 3 * T * k, 1), "unit": "us/block", "cores": threads, "kind": "port",
               "sample": f"one 2880x2880 MXFP4 matvec (dequant-order loop, rows in chunks of 32 over the threads), median of {nrep}, scaled by {3 * T * k} matvecs"}, higher=False)
        for p in (x, lg, de, dw, out, ws):
            be.free(p)
    # The same bank handed over as MoeLayerWeights brings it (per-expert slices + Paired exponent streams + router_proj):
    # residual -> output with the router's projection on the device.
    G = H // 32
    fph, fsh = be.d2h(fp, E * per, np.uint8), be.d2h(fs, E * per // 16, np.uint8)
    dph, dsh = be.d2h(bufs["down"][0], E * per // 2, np.uint8), be.d2h(bufs["down"][1], E * per // 32, np.uint8)
    gu_p, gu_s = [fph[e * per:(e + 1) * per] for e in range(E)], [fsh[e * per // 16:(e + 1) * per // 16] for e in range(E)]
    dn_p, dn_s = [dph[e * per // 2:(e + 1) * per // 2] for e in range(E)], [dsh[e * per // 32:(e + 1) * per // 32] for e in range(E)]
    rng = np.random.default_rng(0x5EED04A0)
    router_w = (rng.standard_normal((E, H)) * 0.05).astype(np.float32)
    layer = be.moe_layer_create(gu_p, dn_p, gu_s, dn_s, router_w, k, H, I, fmt.MOE_ROWS_INTERLEAVED)
    assert layer, be.last_error()
    for T in (1, 16):
        x = be.malloc(T * H * 4 + 64)
        be.dev_fill_normal(x, T * H, 0x5EED04F0 + T, 1.0)
        de, dw, out = be.malloc(T * k * 4), be.malloc(T * k * 4), be.malloc(T * H * 4)

        def layer_fwd():
            be.dev_moe_layer_forward(layer, x, x, T, out, de, dw)
        layer_fwd(); be.synchronize()
        xv = be.d2h(x, (T, H), np.float32)
        experts, wts = be.d2h(de, (T, k), np.uint32), be.d2h(dw, (T, k), np.float32)
        want_route = O.moe_route_from_router_input(xv[0], router_w, None, k)
        assert [int(e) for e in experts[0]] == [e for e, _ in want_route] and np.allclose(wts[0], [w for _, w in want_route], rtol=5e-5)
        want = O.moe_block_mxfp4(xv[:1], experts[:1].astype(np.uint64), wts[:1], (fph, fsh), None, (dph, dsh), E, H, I, interleaved=True)
        got = be.d2h(out, (T, H), np.float32)[:1]
        rel = float(np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want))
        assert rel < 1e-3, rel
        distinct = len(set(int(v) for v in experts.reshape(-1)))
        ms = _timeit(be, layer_fwd, args.steps)
        algo = distinct * expert_bytes + E * H * 4 + T * (8 * H + 4 * E)
        _emit(f"MXFP4 MoE layer us, router projection included (per-expert slices, batch {T})", round(ms * 1e3, 2), "us/block", ms, args.steps, 2,
              {"workload": f"BASELINE configs[3] as MoeLayerWeights hands it over: 32 per-expert slices, router_proj 32x2880 on the device, top-4, batch {T}",
               "distinct_experts": distinct, "launches_per_block": 3 if T == 1 else 5, "verified_rel_l2_vs_oracle": rel},
              {"kernel": "f32 gemv (router) + gemv_mxfp4 (gate/up, down)", "bound": "hbm", "achieved": round(algo / ms / 1e6, 1), "peak": HBM_PEAK_GBS,
               "unit": "GB/s", "frac": round(algo / ms / 1e6 / HBM_PEAK_GBS, 4), "traffic": None}, None, higher=False)
        for p in (x, de, dw, out):
            be.free(p)
    be.moe_layer_destroy(layer)


def run_kq(be, fmt, args):
    """Beside BASELINE configs[3]: the MoE layer over a Q4_K expert bank at Gemma-4-26B-A4B's shapes (128 experts, top-8,
    hidden 2816, intermediate 704 stored 768 wide, GeluTanh) — cpu_moe_forward's integer expert path, residual -> output."""
    O = _oracle()
    E, k, H, I, IP = 128, 8, 2816, 704, 768
    rng = np.random.default_rng(0x5EED0600)
    # (a bank of 128 distinct experts on the device; four distinct weight sets on the host keep the set-up short)
    gus = [O.quantize_q4_k((rng.standard_normal((2 * I, H)) * 0.05).astype(np.float32)) for _ in range(4)]
    dns = [O.quantize_q4_k((rng.standard_normal((H, IP)) * 0.05).astype(np.float32)) for _ in range(4)]
    gate_up, down = [gus[e % 4] for e in range(E)], [dns[e % 4] for e in range(E)]
    router_w = (rng.standard_normal((E, H)) * 0.05).astype(np.float32)
    layer = be.moe_layer_create(gate_up, down, None, None, router_w, k, H, I, fmt.MOE_ROWS_CONTIGUOUS_HALVES, expert_scales=fmt.MOE_SCALES_INLINE,
                                expert_data_format=fmt.FMT_Q4_K, gate_rule=fmt.MOE_GATE_GELU_TANH)
    assert layer, be.last_error()
    expert_bytes = gus[0].size + dns[0].size
    for T in (1, 16):
        x = be.malloc(T * H * 4 + 64)
        be.dev_fill_normal(x, T * H, 0x5EED06F0 + T, 1.0)
        de, dw, out = be.malloc(T * k * 4), be.malloc(T * k * 4), be.malloc(T * H * 4)

        def layer_fwd():
            be.dev_moe_layer_forward(layer, x, x, T, out, de, dw)
        layer_fwd(); be.synchronize()
        xv = be.d2h(x, (T, H), np.float32)
        experts, wts = be.d2h(de, (T, k), np.uint32), be.d2h(dw, (T, k), np.float32)
        want_route = O.moe_route_from_router_input(xv[0], router_w, None, k)
        assert [int(e) for e in experts[0]] == [e for e, _ in want_route] and np.allclose(wts[0], [w for _, w in want_route], rtol=5e-5)
        t0 = time.perf_counter()
        want = O.moe_block_kq(xv[:1], experts[:1], wts[:1], gate_up, down, H, H, I, 4, None, None, O.GATE_GELU_TANH)
        cpu_s = time.perf_counter() - t0
        got = be.d2h(out, (T, H), np.float32)[:1]
        rel = float(np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want))
        assert rel < 1e-3, rel
        ms = _timeit(be, layer_fwd, args.steps)
        slots = T * k
        algo = slots * expert_bytes + E * H * 4 + T * (8 * H + 4 * E)      # every slot reads its expert's matrices (no sharing between tokens yet)
        _emit(f"Q4_K MoE layer us (Gemma-4-26B-A4B shapes: 128 experts, top-8, batch {T})", round(ms * 1e3, 2), "us/layer", ms, args.steps, 2,
              {"workload": f"MoE layer over a Q4_K expert bank as MoeLayerWeights hands it over: 128 experts x (gate_up 1408x2816, down 2816x768), "
                           f"router_proj 128x2816, top-8, GeluTanh, Q8_K activations (the reference's integer expert path), batch {T}",
               "launches_per_layer": 6, "slots": slots, "distinct_experts": len(set(int(v) for v in experts.reshape(-1))),
               "verified_rel_l2_vs_oracle": rel},
              {"kernel": "gemv_q4k_q8k (gate/up, down launches) + the small kernels around them", "bound": "hbm", "achieved": round(algo / ms / 1e6, 1),
               "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(algo / ms / 1e6 / HBM_PEAK_GBS, 4), "traffic": None},
              {"value": round(cpu_s * 1e6 * T, 1), "unit": "us/layer", "cores": 1, "kind": "port",
               "sample": f"one token through the checker's scalar integer expert path, one thread, scaled by {T} tokens"}, higher=False)
        for p_ in (x, de, dw, out):
            be.free(p_)
    be.moe_layer_destroy(layer)


def run_c5(be, fmt, args):
    """BASELINE configs[4]: batched-prefill Q4_K GEMM at Gemma-3-12B shapes, 512 tokens, f16 MFMA on integer weights, bf16 activations."""
    O = _oracle()
    seq = 512
    total_fl, total_ms, rels = 0.0, 0.0, []
    per = []
    for name, rows, hidden in (("gate", 15360, 3840), ("up", 15360, 3840), ("down", 3840, 15360)):
        n = rows * hidden
        tmp, w = be.malloc(n * 4), be.malloc(q4k_bytes(rows, hidden) + 64)
        be.dev_fill_normal(tmp, n, 0x5EED0500 + len(per), 0.02)
        be.dev_quantize_q4_k(tmp, n, w)
        xf, xb = be.malloc(seq * hidden * 4), be.malloc(seq * hidden * 2 + 64)
        be.dev_fill_normal(xf, seq * hidden, 0x5EED05F0 + len(per), 1.0)
        be.dev_f32_to_bf16(xf, seq * hidden, xb)
        out = be.malloc(seq * rows * 4)
        # the rows' exponents are a property of the weights: computed once (load time), outside the timed calls
        rexp = be.malloc(rows * 4 + 64)
        be.dev_q4k_row_exponents(w, rows, hidden, rexp)
        be.dev_q4k_gemm_prepared(w, rexp, xb, rows, hidden, seq, out); be.synchronize()
        # verify 64 rows x 8 tokens against the oracle
        r0 = 4096 % rows
        wb = be.d2h(w + r0 * (hidden // 256) * 144, 64 * (hidden // 256) * 144, np.uint8)
        xs = (be.d2h(xb, (seq, hidden), np.uint16)[:8].astype(np.uint32) << 16).view(np.float32)
        want = O.q4k_matmul(wb, xs, 64, hidden, 8)
        got = be.d2h(out, (seq, rows), np.float32)[:8, r0:r0 + 64]
        rels.append(float(np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want)))
        assert rels[-1] < 1e-3, rels
        ms = _timeit(be, lambda: be.dev_q4k_gemm_prepared(w, rexp, xb, rows, hidden, seq, out), max(3, args.steps // 5))
        ms_all = _timeit(be, lambda: be.dev_q4k_gemm(w, xb, rows, hidden, seq, out), max(3, args.steps // 5))
        fl = 2.0 * seq * rows * hidden
        per.append({"matrix": name, "us": round(ms * 1e3, 1), "TFLOPs": round(fl / ms / 1e9, 1),
                    "us_with_row_exponents_per_call": round(ms_all * 1e3, 1)})
        total_fl += fl; total_ms += ms
        if name == "down":
            threads = cpu_threads()
            wb512 = be.d2h(w, 512 * (hidden // 256) * 144, np.uint8)
            med, nrep = _cpu_time(lambda: O.q4k_matmul_mt(wb512, xs, 512, hidden, 8, threads), args.cpu_seconds / 2)
            cpu = {"value": round(2.0 * 512 * hidden * 8 / med / 1e12, 5), "unit": "TFLOP/s", "cores": threads, "kind": "port",
                   "sample": f"512 rows x 8 tokens x {hidden} (q4k_matmul_into restated, 32-row chunks over the threads), median of {nrep}"}
        for p in (tmp, w, xf, xb, out, rexp):
            be.free(p)
    tf = total_fl / total_ms / 1e9
    _emit("Q4_K prefill GEMM TFLOP/s (f16 MFMA, bf16 activations, 512 tokens, Gemma-3-12B FFN)", round(tf, 1), "TFLOP/s", total_ms, max(3, args.steps // 5), 2,
          {"workload": "BASELINE configs[4]: Q4_K GEMM 512x3840 . (15360x3840, 15360x3840, 3840x15360)", "per_matrix": per,
           "mfma_terms_per_weight": 1, "row_exponents": "computed once per matrix (larql_hip_dev_q4k_row_exponents), outside the timed calls; us_with_row_exponents_per_call = larql_hip_dev_q4k_gemm, which recomputes them",
           "verified_rel_l2_vs_oracle": max(rels)},
          {"kernel": "q4k_gemm", "bound": "mfma", "achieved": round(tf, 1), "peak": 2500.0, "unit": "TFLOP/s",
           "frac": round(tf / 2500.0, 4), "traffic": None, "note": "nominal flops 2*S*N*K; one f16 MFMA term per weight (the row scales ride in the f16 operand: ~3e-4 from the CPU value), plus one small MFMA per tile and super-block for the offsets"},
          cpu)


def run_q8k(be, fmt, args):
    """The Gemma-3-4B decode stack through the Q8_K-activation integer path (quantize_x_to_q8k + q4k_q8k_matvec), the
    path the reference's CPU decode runs: 34 layers x 7 Q4_K matvecs, one launch, activations quantised on the device."""
    O = _oracle()
    layers = args.layers
    shapes = [("q", 2048, 2560), ("k", 1024, 2560), ("v", 1024, 2560), ("o", 2560, 2048), ("gate", 10240, 2560), ("up", 10240, 2560),
              ("down", 2560, 10240)]
    acts = {}
    for k in (2560, 2048, 10240):
        x = be.malloc(k * 4 + 64)
        be.dev_fill_normal(x, k, 0x5EED0600 + k, 1.0)
        q = be.malloc(be.q8k_bytes(k) + 64)
        assert be.dev_quantize_x_to_q8k(x, k, q)
        acts[k] = (x, q)
    tmp = be.malloc(10240 * 2560 * 4)
    jobs, keep = [], []
    algo = 0
    for layer in range(layers):
        for i, (name, rows, k) in enumerate(shapes):
            w = be.malloc(q4k_bytes(rows, k) + 64)
            be.dev_fill_normal(tmp, rows * k, 0x5EED0610 + layer * 8 + i, 0.02)
            be.dev_quantize_q4_k(tmp, rows * k, w)
            o = be.malloc(rows * 4 + 64)
            jobs.append((fmt.FMT_Q4_K_Q8K, w, None, acts[k][1], o, rows, k))
            keep.append((w, o, rows, k))
            algo += q4k_bytes(rows, k) + be.q8k_bytes(k) + 4 * rows
    plan = be.plan_create(jobs)
    assert plan is not None and be.plan_launch_count(plan) == 1
    be.plan_run(plan); be.synchronize()
    # bit-exact against the oracle on two matvecs of layer 0 (the reference's SIMD kernels equal its scalar one bit for bit)
    exact = True
    cpu_ops = []
    for idx in (1, 6):
        w, o, rows, k = keep[idx]
        wb, xv = be.d2h(w, q4k_bytes(rows, k), np.uint8), be.d2h(acts[k][0], k, np.float32)
        a = O.quantize_x_to_q8k(xv)
        dev_a = be.d2h(acts[k][1], be.q8k_bytes(k), np.uint8)
        exact &= bool(np.array_equal(dev_a[:k].view(np.int8), a[0]) and np.array_equal(dev_a[k:k + k // 64].view(np.float32), a[1]))
        want = O.q4k_q8k_matvec(wb, *a, rows, k)
        exact &= bool(np.array_equal(be.d2h(o, rows, np.float32).view(np.uint32), want.view(np.uint32)))
        cpu_ops.append((wb, a, rows, k))
    assert exact
    ms = _timeit(be, lambda: be.plan_run(plan), args.steps)
    ms_q = _timeit(be, lambda: be.dev_quantize_x_to_q8k(acts[10240][0], 10240, acts[10240][1]), args.steps)
    gbs = algo / ms / 1e6
    med, n = _cpu_time(lambda: [O.q4k_q8k_matvec(wb, *a, rows, k) for wb, a, rows, k in cpu_ops], args.cpu_seconds)
    cpu_bytes = sum(q4k_bytes(rows, k) for _, _, rows, k in cpu_ops)
    _emit("Q4_K x Q8_K decode matvec stack HBM GB/s (integer-dot path)", round(gbs, 1), "GB/s", ms, args.steps, 2,
          {"workload": f"Gemma-3-4B decode stack, batch 1, {layers} layers x 7 Q4_K matvecs against Q8_K activations, one launch",
           "matvecs_per_step": len(jobs), "algorithmic_bytes_per_step": algo, "bit_exact_vs_oracle": exact,
           "quantize_x_to_q8k_us_10240": round(ms_q * 1e3, 2)},
          {"kernel": "gemv_q4k_q8k", "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
          {"value": round(cpu_bytes / med / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
           "sample": f"k 1024x2560 and down 2560x10240 of layer 0 (q4k_q8k_matvec_scalar restated), median of {n}"},
          dtype="i32")


def run_formats(be, fmt, args):
    """The other block formats of the matvec family at decode shapes, cache-cold (distinct copies of each matrix in one
    launch, 0.5-1 GB per launch): Q6_K at the Gemma-3-4B FFN shapes, MXFP4 at the gpt-oss expert shape and at 4096 x 4096."""
    O = _oracle()
    rng = np.random.default_rng(0x5EED0700)
    x_all = be.malloc(16384 * 4)
    be.dev_fill_normal(x_all, 16384, 0x5EED0701, 1.0)
    cases = [("Q6_K", 10240, 2560, 24), ("Q6_K", 2560, 10240, 24), ("MXFP4", 2880, 2880, 128), ("MXFP4", 4096, 4096, 64)]
    for name, rows, k, copies in cases:
        if name == "Q6_K":
            # any bytes are valid 6-bit codes and int8 scales; d a small f16
            blocks = rng.integers(0, 256, size=(rows * (k // 256), 210), dtype=np.uint8)
            blocks[:, 208:210] = np.frombuffer(np.float16(rng.uniform(1e-4, 3e-4, size=rows * (k // 256))).tobytes(), np.uint8).reshape(-1, 2)
            host = [blocks.reshape(-1)]
            job = lambda bufs, o: (fmt.FMT_Q6_K, bufs[0], None, x_all, o, rows, k)
            want = lambda r: O.q6k_matvec(host[0][:r * (k // 256) * 210], be.d2h(x_all, k, np.float32), r, k)
        else:
            tmp = be.malloc(rows * k * 4)
            be.dev_fill_normal(tmp, rows * k, 0x5EED0710 + rows, 0.02)
            p0, s0 = be.malloc(rows * k // 2 + 64), be.malloc(rows * k // 32 + 64)
            assert be.dev_quantize_mxfp4(tmp, rows, k, p0, s0)
            be.synchronize()
            host = [be.d2h(p0, rows * k // 2, np.uint8), be.d2h(s0, rows * k // 32, np.uint8)]
            for q in (tmp, p0, s0):
                be.free(q)
            job = lambda bufs, o: (fmt.FMT_MXFP4, bufs[0], bufs[1], x_all, o, rows, k)
            want = lambda r: O.mxfp4_gemv(host[0][:r * k // 2], host[1][:r * k // 32], be.d2h(x_all, k, np.float32), r, k)
        first = [be.to_device(h) for h in host]
        bufs_all, outs = [first], []
        for _ in range(copies - 1):  # exact copies at distinct addresses: nothing of a launch is served from a cache
            cp = []
            for h, src in zip(host, first):
                assert h.size % 16 == 0
                d = be.malloc(h.size + 64)
                assert be.dev_copy(d, src, h.size)
                cp.append(d)
            bufs_all.append(cp)
        jobs = []
        for bufs in bufs_all:
            o = be.malloc(rows * 4 + 64)
            outs.append(o)
            jobs.append(job(bufs, o))
        plan = be.plan_create(jobs)
        assert plan is not None
        be.plan_run(plan); be.synchronize()
        sample = 64
        ref = want(sample)
        rel = max(float(np.linalg.norm(be.d2h(o, sample, np.float32).astype(np.float64) - ref) / np.linalg.norm(ref)) for o in (outs[0], outs[-1]))
        assert rel < 1e-3, (name, rows, k, rel)
        ms = _timeit(be, lambda: be.plan_run(plan), args.steps)
        algo = copies * (sum(h.size for h in host) + 4 * rows) + 4 * k
        gbs = algo / ms / 1e6
        med, n = _cpu_time(lambda: want(sample), args.cpu_seconds / 4)
        _emit(f"{name} {rows}x{k} matvec HBM GB/s (cold, {copies} distinct copies per launch)", round(gbs, 1), "GB/s", ms, args.steps, 2,
              {"workload": f"{name} matvec {rows}x{k}, batch 1, {copies} copies in one launch", "us_per_matvec": round(ms * 1e3 / copies, 3),
               "verified_rel_l2_vs_oracle": rel},
              {"kernel": "gemv_q6k_mfma" if name == "Q6_K" else "gemv_mxfp4_mfma", "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
               "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
              {"value": round(sample * sum(h.size for h in host) / rows / med / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
               "sample": f"first {sample} rows, median of {n}"})
        be.plan_destroy(plan)
        for bufs in bufs_all:
            for d in bufs:
                be.free(d)
        for o in outs:
            be.free(o)


def read_traffic():
    """HBM bytes per launch of the dominant kernel from the committed rocprof PMC summary, if any."""
    path = os.path.join(ROOT, "profiles", "gemv_q4k_c2_stack.pmc.txt")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch:"):
                return float(line.split(":", 1)[1].split()[0])
    except OSError:
        pass
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--pre-warm-s", type=float, default=0.3, help="seconds of untimed steps before the warm-up (clock ramp)")
    ap.add_argument("--layers", type=int, default=LAYERS, help=argparse.SUPPRESS)
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg (profiling runs)")
    ap.add_argument("--no-graph", action="store_true",
                    help="dependency-ordered arm: a host call per stage only, no recorded sequence (rocprofv3's kernel trace "
                         "does not survive HIP graph capture in this image)")
    ap.add_argument("--headline-only", action="store_true",
                    help="skip the dependency-ordered arm, the host-tier call timings and the other configurations (profiling runs)")
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3", "c4", "c5", "q8k", "formats", "kq"],
                    help="c2 (default) is the headline decode stack; the others are BASELINE's remaining configs")
    ap.add_argument("--copy-probe", action="store_true",
                    help="only run the plain 16-byte copy kernel on 1 GiB three times (known size, for scaling "
                         "profiler byte counters) and print its bandwidth")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path runs on ONE GPU; --gpus above 1 is not part of this build "
              "(it would shard by weight rows: x broadcast, outputs concatenated, no reduction across GPUs)", file=sys.stderr)
        sys.exit(2)

    import larql_amd as fmt
    be = fmt.HipBackend()
    if args.copy_probe:
        n = 1 << 30
        a, b = be.malloc(n + 64), be.malloc(n + 64)
        be.dev_fill_normal(a, n // 4, 1, 1.0)
        be.dev_copy(b, a, n)
        e0, e1 = be.event(), be.event()
        be.record(e0)
        for _ in range(3):
            be.dev_copy(b, a, n)
        be.record(e1)
        ms = be.elapsed_ms(e0, e1) / 3
        e2, e3 = be.event(), be.event()
        be.record(e2)
        for _ in range(3):
            be.dev_copy(None, a, n)
        be.record(e3)
        ms_r = be.elapsed_ms(e2, e3) / 3
        print(json.dumps({"copy_bytes": n, "copy_GBps_read_plus_write": round(2 * n / ms / 1e6, 1),
                          "read_only_GBps": round(n / ms_r / 1e6, 1)}))
        return
    if args.workload != "c2":
        {"c1": run_c1, "c3": run_c3, "c4": run_c4, "c5": run_c5, "q8k": run_q8k, "formats": run_formats, "kq": run_kq}[args.workload](be, fmt, args)
        return
    stack = Stack(be, fmt, layers=args.layers)

    stack.step()
    be.synchronize()
    if args.no_cpu:
        worst, cpu = None, None
    else:
        worst, cpu = verify_and_cpu_baseline(be, stack, min_seconds=args.cpu_seconds)

    # The GPU idles while the host runs the CPU baseline and its clocks drop; the first milliseconds after
    # that measure the clock ramp, not the kernel (first arm reads ~13 % low).  Bring it back to a steady
    # state with a fixed stretch of the same work before the W warm-up steps, whatever W is.
    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < args.pre_warm_s:
        for _ in range(50):
            stack.step()
        be.synchronize()
    for _ in range(args.warmup):
        stack.step()
    be.synchronize()
    ev = [(be.event(), be.event(), be.event()) for _ in range(args.steps)]
    be.synchronize()
    t0 = time.perf_counter()
    for a, b, c in ev:
        be.record(a)
        be.plan_run(stack.plan_q4k)
        be.record(b)
        be.plan_run(stack.plan_q8)
        be.record(c)
    be.synchronize()
    t1 = time.perf_counter()

    ms_per_step = (t1 - t0) * 1e3 / args.steps
    q4k_ms = float(np.mean([be.elapsed_ms(a, b) for a, b, _ in ev]))
    q8_ms = float(np.mean([be.elapsed_ms(b, c) for _, b, c in ev]))
    algo_bytes = stack.q4k_algo_bytes + stack.q8_algo_bytes
    value = algo_bytes / (ms_per_step * 1e-3) / 1e9
    achieved = stack.q4k_algo_bytes / (q4k_ms * 1e-3) / 1e9

    dependency, host_tier, others = None, None, None
    if not args.headline_only:
        dependency = dependency_ordered_arm(be, fmt, stack, args)
        host_tier = host_tier_calls(be, fmt, stack)
        others = other_configs(be, fmt, args)
    out = {
        "metric": "Q4_K/Q8_0 decode matvec stack HBM GB/s", "value": round(value, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {
            "workload": "BASELINE configs[1]: Gemma-3-4B decode matvec stack, batch 1, "
                        f"{args.layers} layers x 7 Q4_K matvecs + Q8_0 lm_head 262144x2560",
            "matvecs_per_step": len(stack.q4k_jobs) + 1, "launches_per_step": 2,
            "jobs_of_a_step": "mutually independent (every matvec has its own activation): a streaming-bandwidth figure, not a decode rate",
            "algorithmic_bytes_per_step": algo_bytes, "independent_steps_per_s": round(1e3 / ms_per_step, 1),
            "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
            "q8_0_lm_head": {"ms": round(q8_ms, 4), "GB/s": round(stack.q8_algo_bytes / (q8_ms * 1e-3) / 1e9, 1)},
            "verified_rel_l2_vs_oracle": worst, "verified": getattr(stack, "verified", None), "pre_warm_s": args.pre_warm_s,
            "dependency_ordered": dependency, "host_tier_us_per_call": host_tier, "other_configs": others,
        },
        "roofline": {"kernel": "gemv_q4k (238 Q4_K matvecs, one launch)", "bound": "hbm", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "launch_ms": round(q4k_ms, 4), "algorithmic_bytes_per_launch": stack.q4k_algo_bytes,
                     "traffic": read_traffic()},
        "cpu_baseline": cpu,
    }
    if dependency:
        # beside the headline: the rate a token sees when every stage waits for the one before it (full detail in config)
        out["decode_in_dependency_order"] = {
            "tokens_per_s": dependency["tokens_per_s"], "ms_per_token": dependency["ms_per_token_device"], "GB/s": dependency["GBps"],
            "frac_of_hbm_peak": round(dependency["pct_of_hbm_peak"] / 100.0, 4), "dependent_launches_per_token": dependency["launches_per_token"]}
    print(json.dumps(out))


def dependency_ordered_arm(be, fmt, stack, args):
    """The same weights as a token walks them: 4 dependent stages per layer + the lm_head."""
    chain = Chain(be, fmt, stack, graph=not args.no_graph)
    chain.step()
    be.synchronize()
    rel = chain.verify(_oracle()) if not args.no_cpu else None
    if rel is not None and not rel < 1e-3:
        raise SystemExit(f"bench: the dependency-ordered walk differs from the CPU oracle (rel-L2 {rel:.3e})")
    steps = max(5, args.steps // 4)

    def both(fn):
        ms = _timeit(be, fn, steps, warm=3)
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        be.synchronize()
        return ms, (time.perf_counter() - t0) * 1e3 / steps
    ms, wall_ms = both(chain.step)
    eager_ms, eager_wall = both(chain.step_eager)
    algo = stack.q4k_algo_bytes + stack.q8_algo_bytes
    return {"launches_per_token": len(chain.plans),
            "submission": "one recorded sequence (HIP graph) per token" if chain.seq is not None else "one host call per stage",
            "ms_per_token_device": round(ms, 4), "ms_per_token_wall": round(wall_ms, 4),
            "tokens_per_s": round(1e3 / max(ms, wall_ms), 1), "GBps": round(algo / max(ms, wall_ms) / 1e6, 1),
            "pct_of_hbm_peak": round(100.0 * algo / max(ms, wall_ms) / 1e6 / HBM_PEAK_GBS, 2), "steps": steps,
            "one_host_call_per_stage": {"ms_per_token_device": round(eager_ms, 4), "ms_per_token_wall": round(eager_wall, 4),
                                        "tokens_per_s": round(1e3 / max(eager_ms, eager_wall), 1)},
            "verified_rel_l2_vs_oracle": rel, "verified": f"every one of the {len(chain.jobs)} Q4_K results of the walk (48-row windows, on the activation the GPU read) + layer 0 chained on the CPU + 3 lm_head windows",
            "note": "matvec launches and their dependencies only (q,k,v | o | gate,up | down per layer, then lm_head); "
                    "device = HIP events around the token, wall = host clock incl. launch overhead"}


def host_tier_calls(be, fmt, stack):
    """End-to-end time of trait-shaped calls on host slices (what larql-inference sees per call): x goes up, the
    result comes back, one submission each.  Weights registered (resident) and not (uploaded per call)."""
    rows, k = 3072, 1024
    rng = np.random.default_rng(0x5EED0100)
    tmp, w = be.malloc(rows * k * 4), be.malloc(q4k_bytes(rows, k) + 64)
    be.dev_fill_normal(tmp, rows * k, 0x5EED0100, 0.02)
    be.dev_quantize_q4_k(tmp, rows * k, w)
    wb = be.d2h(w, q4k_bytes(rows, k), np.uint8)
    x = rng.standard_normal(k).astype(np.float32)
    n, hidden = 10240, 2560
    gw = stack.q4k_jobs[4][1]                      # layer 0's gate matrix as a Q4_K gate file
    gb = be.d2h(gw, q4k_bytes(n, hidden), np.uint8)
    xg = rng.standard_normal(hidden).astype(np.float32)

    def per_call(fn, reps=200):
        for _ in range(10):
            fn()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        return round((time.perf_counter() - t0) * 1e6 / reps, 1)

    out = {"q4k_matvec_3072x1024_unregistered": per_call(lambda: be.q4k_matvec(wb, x, rows, k)),
           "gate_knn_q4k_10240x2560_k64_unregistered": per_call(lambda: be.gate_knn(fmt.FMT_Q4_K, gb, xg, n, hidden, 64), 50)}
    be.register_weight_region(wb)
    be.register_weight_region(gb)
    be.seal_weight_regions()
    out["q4k_matvec_3072x1024_registered"] = per_call(lambda: be.q4k_matvec(wb, x, rows, k))
    out["gate_knn_q4k_10240x2560_k64_registered"] = per_call(lambda: be.gate_knn(fmt.FMT_Q4_K, gb, xg, n, hidden, 64))
    clock0 = be.submission_clock()
    for _ in range(100):
        be.q4k_matvec(wb, x, rows, k)
    clock1 = be.submission_clock()
    out["q4k_matvec_3072x1024_registered_gpu_us"] = round((clock1["gpu_nanos"] - clock0["gpu_nanos"]) / 100 / 1e3, 1)
    be.clear_weight_regions()
    be.free(tmp); be.free(w)
    return out


def other_configs(be, fmt, args):
    """A short run of BASELINE's other configurations, each verified against the oracle before it is timed."""
    global _COLLECT
    short = argparse.Namespace(**vars(args))
    short.steps = min(args.steps, 60)
    short.cpu_seconds = 0.4 if args.no_cpu else min(args.cpu_seconds, 4.0)
    _COLLECT = []
    try:
        for fn in (run_c1, run_c3, run_c4, run_kq, run_c5, run_formats):
            fn(be, fmt, short)
        lines = _COLLECT
    finally:
        _COLLECT = None
    out = []
    for l in lines:
        cfg = l["config"]
        out.append({"metric": l["metric"], "value": l["value"], "unit": l["unit"], "frac": l["roofline"]["frac"],
                    "bound": l["roofline"]["bound"],
                    "verified": cfg.get("verified_rel_l2_vs_oracle", cfg.get("topk_identical_up_to_ties")),
                    "detail": {k: v for k, v in cfg.items() if k not in ("workload", "verified_rel_l2_vs_oracle")},
                    "cpu_baseline": {k: l["cpu_baseline"][k] for k in ("value", "unit", "cores")} if l["cpu_baseline"] else None})
    return out


if __name__ == "__main__":
    main()
