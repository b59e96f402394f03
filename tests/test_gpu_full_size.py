"""GPU properties at the full sizes of the benchmark configurations, where the oracle is too slow to recompute
everything: weights are generated and quantised on the device, a sample of rows is held to the oracle, and the rest is
covered by properties that do not depend on size -- linearity and exact power-of-two scaling, invariance under
reordering of jobs / tokens / layers, determinism, selection and ordering invariants of top-K, encode -> decode
round-trip bounds.  Everything goes through the C ABI (larql_amd.HipBackend)."""
import numpy as np
import pytest

import oracle as O

pytestmark = pytest.mark.gpu
F = np.float32


def rel_l2(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def q4k_bytes(rows, k):
    return rows * (k // 256) * 144


def assert_same_hits_up_to_ties(hits, want, scores):
    """Both lists by value descending with the same values; indices may differ only inside a run of equal scores (the
    reference sorts with sort_unstable_by and its heap evicts equal minima in heap order: lm_head/knn.rs:340-383), and
    this backend puts the lower index first."""
    hv, wv = np.array([v for _, v in hits], F), np.array([v for _, v in want], F)
    assert np.array_equal(hv.view(np.uint32), wv.view(np.uint32))
    hi, wi = [i for i, _ in hits], [i for i, _ in want]
    assert np.array_equal(scores[hi].view(np.uint32), hv.view(np.uint32)) and len(set(hi)) == len(hi)
    for v in np.unique(hv[np.array(hi) != np.array(wi)]) if hi != wi else []:
        run = hv == v
        assert run.sum() > 1 or v == hv[-1]                  # a tie inside the list, or at its boundary
        ours = sorted(np.array(hi)[run])
        assert ours == sorted(np.flatnonzero(scores == v)[:len(ours)])   # the lowest indices of that score


def dev_q4k_matrix(be, rows, k, seed):
    n = rows * k
    tmp, w = be.malloc(n * 4), be.malloc(q4k_bytes(rows, k) + 64)
    assert be.dev_fill_normal(tmp, n, seed, 0.02) and be.dev_quantize_q4_k(tmp, n, w)
    return tmp, w


# Gemma-3-4B layer shapes [rows, k] (q, k, v, o, gate, up, down)
LAYER = [(2048, 2560), (1024, 2560), (1024, 2560), (2560, 2048), (10240, 2560), (10240, 2560), (2560, 10240)]


def test_decode_stack_plan_is_deterministic_order_independent_and_linear(be, fmt):
    """configs[1] at its real shapes: 6 layers x 7 Q4_K matvecs in one recorded launch."""
    rng = np.random.default_rng(1)
    layers = 6
    xs = {k: rng.standard_normal(k).astype(F) for k in (2560, 2048, 10240)}
    ys = {k: rng.standard_normal(k).astype(F) for k in xs}
    a, b = F(0.5), F(-2.0)                                         # powers of two: the combination of inputs is exact per term
    dx = {k: be.to_device(v) for k, v in xs.items()}
    dy = {k: be.to_device(v) for k, v in ys.items()}
    dz = {k: be.to_device((a * xs[k] + b * ys[k]).astype(F)) for k in xs}
    mats, jobs = [], {"x": [], "y": [], "z": []}
    outs = {"x": [], "y": [], "z": []}
    for l in range(layers):
        for i, (rows, k) in enumerate(LAYER):
            tmp, w = dev_q4k_matrix(be, rows, k, 0x5EED0100 + 16 * l + i)
            be.free(tmp)
            mats.append((w, rows, k))
            for name, src in (("x", dx), ("y", dy), ("z", dz)):
                o = be.malloc(rows * 4)
                outs[name].append(o)
                jobs[name].append((fmt.FMT_Q4_K, w, None, src[k], o, rows, k))
    plans = {n: be.plan_create(j) for n, j in jobs.items()}
    assert all(p is not None for p in plans.values()) and be.plan_launch_count(plans["x"]) == 1
    for p in plans.values():
        assert be.plan_run(p)
    be.synchronize()
    res = {n: [be.d2h(o, m[1], F) for o, m in zip(outs[n], mats)] for n in outs}
    # determinism: a second run gives the same bits
    assert be.plan_run(plans["x"])
    be.synchronize()
    for o, m, first in zip(outs["x"], mats, res["x"]):
        assert np.array_equal(be.d2h(o, m[1], F).view(np.uint32), first.view(np.uint32))
    # order independence: the same jobs recorded in reverse order give the same bits per matrix
    rev = be.plan_create(list(reversed(jobs["x"])))
    for o, m in zip(outs["x"], mats):
        be.h2d(o, np.full(m[1], np.nan, F))                          # (so that stale results cannot pass)
    assert be.plan_run(rev)
    be.synchronize()
    for o, m, first in zip(outs["x"], mats, res["x"]):
        assert np.array_equal(be.d2h(o, m[1], F).view(np.uint32), first.view(np.uint32))
    # linearity: W(a x + b y) = a Wx + b Wy up to f32 rounding of the sums
    for rx, ry, rz in zip(res["x"], res["y"], res["z"]):
        assert rel_l2(rz, a * rx.astype(np.float64) + b * ry.astype(np.float64)) < 2e-5
    # a sample of rows of the largest matrices against the oracle
    for idx in (4, 6, 7 * (layers - 1) + 5):
        w, rows, k = mats[idx]
        r0 = (rows // 2) & ~15
        wb = be.d2h(w + r0 * (k // 256) * 144, 48 * (k // 256) * 144, np.uint8)
        want = O.q4k_matvec(wb, xs[k], 48, k)
        assert rel_l2(res["x"][idx][r0:r0 + 48], want) < 2e-5
    for p in list(plans.values()) + [rev]:
        be.plan_destroy(p)
    for w, _, _ in mats:
        be.free(w)
    for n in outs:
        for o in outs[n]:
            be.free(o)


def sample_window(rows, idx):
    """A 48-row window of matrix number idx: the first rows, the last rows, or somewhere inside (aligned to the 16-row tiles or not)."""
    return (0, rows - 48, ((rows * ((idx * 37) % 97)) // 97) & ~15, (rows // 2 + 8 * idx) % (rows - 48))[idx % 4]


def test_decode_stack_34_layers_238_jobs_in_one_launch_every_matrix_sampled(be, fmt):
    """configs[1] as the benchmark times it: all 34 layers x 7 Q4_K matvecs (1.8 GB of weights) recorded as ONE launch.
    The share-out of a launch depends on its job list, so the 238-job launch gets its own checks: a 48-row window of
    EVERY one of the 238 results against the oracle (windows at the first rows, the last rows and inside), bit-equal
    repeats, bit-equal results with the jobs recorded in reverse order, and linearity over all rows."""
    rng = np.random.default_rng(34)
    layers = 34
    xs = {k: rng.standard_normal(k).astype(F) for k in (2560, 2048, 10240)}
    ys = {k: rng.standard_normal(k).astype(F) for k in xs}
    a, b = F(0.25), F(-4.0)
    dev = {"x": {k: be.to_device(v) for k, v in xs.items()}, "y": {k: be.to_device(v) for k, v in ys.items()},
           "z": {k: be.to_device((a * xs[k] + b * ys[k]).astype(F)) for k in xs}}
    tmp = be.malloc(10240 * 2560 * 4)
    mats, jobs, outs = [], {n: [] for n in dev}, {n: [] for n in dev}
    for l in range(layers):
        for i, (rows, k) in enumerate(LAYER):
            w = be.malloc(q4k_bytes(rows, k) + 64)
            assert be.dev_fill_normal(tmp, rows * k, 0x5EED2200 + 8 * l + i, 0.02) and be.dev_quantize_q4_k(tmp, rows * k, w)
            mats.append((w, rows, k))
            for n in dev:
                o = be.to_device(np.full(rows, np.nan, F))
                outs[n].append(o)
                jobs[n].append((fmt.FMT_Q4_K, w, None, dev[n][k], o, rows, k))
    assert len(mats) == 238
    plans = {n: be.plan_create(j) for n, j in jobs.items()}
    assert all(p is not None for p in plans.values()) and be.plan_launch_count(plans["x"]) == 1
    for p in plans.values():
        assert be.plan_run(p)
    be.synchronize()
    res = {n: [be.d2h(o, m[1], F) for o, m in zip(outs[n], mats)] for n in outs}
    assert all(np.isfinite(r).all() for r in res["x"])
    # every one of the 238 matvecs: a window of rows against the oracle
    worst = 0.0
    for idx, (w, rows, k) in enumerate(mats):
        r0 = sample_window(rows, idx)
        wb = be.d2h(w + r0 * (k // 256) * 144, 48 * (k // 256) * 144, np.uint8)
        worst = max(worst, rel_l2(res["x"][idx][r0:r0 + 48], O.q4k_matvec(wb, xs[k], 48, k)))
    assert worst < 2e-5, worst
    # determinism
    assert be.plan_run(plans["x"])
    be.synchronize()
    for o, m, first in zip(outs["x"], mats, res["x"]):
        assert np.array_equal(be.d2h(o, m[1], F).view(np.uint32), first.view(np.uint32))
    # the same 238 jobs recorded in reverse order (another share-out of the same launch): the same bits per matrix
    rev = be.plan_create(list(reversed(jobs["x"])))
    for o, m in zip(outs["x"], mats):
        be.h2d(o, np.full(m[1], np.nan, F))
    assert be.plan_run(rev)
    be.synchronize()
    for o, m, first in zip(outs["x"], mats, res["x"]):
        assert np.array_equal(be.d2h(o, m[1], F).view(np.uint32), first.view(np.uint32))
    # and each matrix alone (a one-job launch) gives those bits too, on a sample of the stack
    for idx in (0, 3, 6, 100, 237):
        w, rows, k = mats[idx]
        o = be.malloc(rows * 4)
        assert be.dev_matvec(fmt.FMT_Q4_K, w, None, dev["x"][k], rows, k, o)
        be.synchronize()
        assert np.array_equal(be.d2h(o, rows, F).view(np.uint32), res["x"][idx].view(np.uint32)), idx
    # linearity over every row of every matrix
    for rx, ry, rz in zip(res["x"], res["y"], res["z"]):
        assert rel_l2(rz, a * rx.astype(np.float64) + b * ry.astype(np.float64)) < 2e-5
    for p in list(plans.values()) + [rev]:
        be.plan_destroy(p)


def test_lm_head_q8_0_full_vocabulary_linearity_and_sampled_rows(be, fmt):
    """configs[1]'s lm_head: 262144 x 2560 ggml Q8_0 (713 MB)."""
    rng = np.random.default_rng(2)
    n, k = 262144, 2560
    nb = n * (k // 32) * 34
    w = be.malloc(nb + 64)
    chunk = 16384
    tmp = be.malloc(chunk * k * 4)
    for c in range(n // chunk):
        assert be.dev_fill_normal(tmp, chunk * k, 0x5EED0200 + c, 0.02)
        assert be.dev_quantize_q8_0(tmp, chunk * k, w + c * chunk * (k // 32) * 34)
    be.free(tmp)
    x, y = rng.standard_normal(k).astype(F), rng.standard_normal(k).astype(F)
    outs = []
    for v in (x, y, (F(4.0) * x - F(0.25) * y).astype(F), (F(8.0) * x).astype(F)):
        dv, o = be.to_device(v), be.malloc(n * 4)
        assert be.dev_matvec(fmt.FMT_GGML_Q8_0, w, None, dv, n, k, o)
        be.synchronize()
        outs.append(be.d2h(o, n, F))
        be.free(dv); be.free(o)
    fx, fy, fz, f8 = outs
    assert np.isfinite(fx).all() and np.abs(fx).max() > 0
    assert rel_l2(fz, 4.0 * fx.astype(np.float64) - 0.25 * fy.astype(np.float64)) < 2e-5
    assert np.array_equal(f8.view(np.uint32), (F(8.0) * fx).view(np.uint32))      # scaling the activation by a power of two is exact
    for r0 in (0, 131072 + 48, n - 64):
        wb = be.d2h(w + r0 * (k // 32) * 34, 64 * (k // 32) * 34, np.uint8)
        assert rel_l2(fx[r0:r0 + 64], O.q8_0_gemv(wb, x, 64, k)) < 2e-5
    # lm_head KNN at vocabulary size (lm_head/knn.rs:126-185): the fused call on the 713 MB head as a registered region
    # (no upload per call), against top_k_sorted over the device's own scores
    wh = be.d2h(w, nb, np.uint8)
    be.free(w)
    be.register_weight_region(wh)
    be.seal_weight_regions()
    for top in (8, 64, 1000):
        assert_same_hits_up_to_ties(be.q8_0_gemv_topk(wh, x, n, k, top), O.top_k_sorted(fx, top), fx)
    be.clear_weight_regions()


def test_q4k_matvec_topk_at_vocabulary_size(be, fmt):
    """q4k_matvec_topk (quant_matvec.rs:268-277) over a 262144 x 2560 Q4_K head: by value, descending, against the oracle's
    top_k_sorted over the full score vector of the same device matvec."""
    rng = np.random.default_rng(6)
    n, k = 262144, 2560
    chunk = 32768
    wb = np.empty(q4k_bytes(n, k), np.uint8)
    tmp, wq = be.malloc(chunk * k * 4), be.malloc(q4k_bytes(chunk, k) + 64)
    for c in range(n // chunk):
        assert be.dev_fill_normal(tmp, chunk * k, 0x5EED0280 + c, 0.02) and be.dev_quantize_q4_k(tmp, chunk * k, wq)
        wb[c * q4k_bytes(chunk, k):(c + 1) * q4k_bytes(chunk, k)] = be.d2h(wq, q4k_bytes(chunk, k), np.uint8)
    be.free(tmp); be.free(wq)
    x = rng.standard_normal(k).astype(F)
    be.register_weight_region(wb)
    be.seal_weight_regions()
    scores = be.q4k_matvec(wb, x, n, k)
    r0 = 200000
    assert rel_l2(scores[r0:r0 + 32], O.q4k_matvec(wb[q4k_bytes(r0, k):q4k_bytes(r0 + 32, k)], x, 32, k)) < 2e-5
    for top in (1, 8, 64, 4096):
        assert_same_hits_up_to_ties(be.q4k_matvec_topk(wb, x, n, k, top), O.top_k_sorted(scores, top), scores)
    be.clear_weight_regions()


@pytest.mark.parametrize("gate_fmt", ["bf16", "q4k"])
def test_gate_walk_full_size_selection_and_order_invariants(be, fmt, gate_fmt):
    """configs[2]: 10240 x 2560 gates, K = 64, a walk over 8 layers and 8 positions in two launches."""
    layers, n, hidden, k, batch = 8, 10240, 2560, 64, 8
    gates = []
    for l in range(layers):
        tmp = be.malloc(n * hidden * 4)
        assert be.dev_fill_normal(tmp, n * hidden, 0x5EED0300 + l, 0.02)
        if gate_fmt == "bf16":
            g = be.malloc(n * hidden * 2 + 64)
            assert be.dev_f32_to_bf16(tmp, n * hidden, g)
        else:
            g = be.malloc(q4k_bytes(n, hidden) + 64)
            assert be.dev_quantize_q4_k(tmp, n * hidden, g)
        be.free(tmp)
        gates.append(g)
    f = fmt.FMT_BF16 if gate_fmt == "bf16" else fmt.FMT_Q4_K
    rng = np.random.default_rng(3)
    X = rng.standard_normal((layers, batch, hidden)).astype(F)
    dX = be.to_device(X)
    scores, idx, val, cnt = be.malloc(layers * batch * n * 4), be.malloc(layers * batch * k * 4), be.malloc(layers * batch * k * 4), be.malloc(layers * batch * 4)
    assert be.dev_gate_walk(f, gates, dX, batch * hidden, batch, n, hidden, k, scores, idx, val, cnt)
    be.synchronize()
    S = be.d2h(scores, (layers, batch, n), F)
    I = be.d2h(idx, (layers, batch, k), np.uint32)
    V = be.d2h(val, (layers, batch, k), F)
    assert (be.d2h(cnt, layers * batch, np.uint32) == k).all()
    for l in range(layers):
        for b in range(batch):
            s, ii, vv = S[l, b], I[l, b].astype(np.int64), V[l, b]
            assert len(set(ii.tolist())) == k and ii.max() < n                         # distinct, in range
            assert np.array_equal(vv.view(np.uint32), s[ii].view(np.uint32))         # the signed scores of those features
            av = np.abs(vv)
            assert (av[:-1] >= av[1:]).all()                                          # best first
            rest = np.abs(s)
            rest[ii] = -1.0
            assert rest.max() <= av[-1]                                               # nothing left out beats the last one kept
            ties = np.flatnonzero(np.abs(s) == av[-1])                                # equal scores: lower indices first
            kept = [t for t in ties if t in set(ii.tolist())]
            assert kept == ties[:len(kept)].tolist()
    # the same walk with layers and positions in another order gives the same hits for each (layer, position)
    perm_l, perm_b = rng.permutation(layers), rng.permutation(batch)
    X2 = np.ascontiguousarray(X[perm_l][:, perm_b])
    assert be.dev_gate_walk(f, [gates[i] for i in perm_l], be.to_device(X2), batch * hidden, batch, n, hidden, k, scores, idx, val, cnt)
    be.synchronize()
    I2 = be.d2h(idx, (layers, batch, k), np.uint32)
    V2 = be.d2h(val, (layers, batch, k), F)
    for a, l in enumerate(perm_l):
        for c, b in enumerate(perm_b):
            assert np.array_equal(I2[a, c], I[l, b]) and np.array_equal(V2[a, c].view(np.uint32), V[l, b].view(np.uint32))
    # one (layer, position) against the oracle: scores, then the reference's selector on the device's scores
    l, b = 5, 3
    gb = be.d2h(gates[l], n * hidden * 2 if gate_fmt == "bf16" else q4k_bytes(n, hidden), np.uint8)
    want = O.bf16_gemv(gb.view(np.uint16), X[l, b], n, hidden) if gate_fmt == "bf16" else O.q4k_matvec(gb, X[l, b], n, hidden)
    assert rel_l2(S[l, b], want) < 2e-5
    ref_hits = O.top_k_by_abs(S[l, b], k)
    assert sorted(i for i, _ in ref_hits) == sorted(I[l, b].tolist())
    for g in gates:
        be.free(g)


@pytest.mark.parametrize("rows,hidden", [(15360, 3840), (3840, 15360)])
def test_prefill_gemm_full_size_exact_scaling_and_token_permutation(be, fmt, rows, hidden):
    """configs[4]: gate/up 15360 x 3840 and down 3840 x 15360 (the leg that splits K over workgroups and adds the
    partial slabs in a fixed order) against 512 tokens of bf16 activations."""
    seq = 512
    tmp, w = dev_q4k_matrix(be, rows, hidden, 0x5EED0500 + (hidden > rows))
    be.free(tmp)
    rng = np.random.default_rng(5)
    X = rng.standard_normal((seq, hidden)).astype(F)
    xb = O.f32_to_bf16(X).reshape(seq, hidden)
    Xr = (xb.astype(np.uint32) << 16).view(F)                                        # the activations as held (bf16, truncated)
    out = be.malloc(seq * rows * 4)

    def gemm(bits):
        dx = be.to_device(np.ascontiguousarray(bits))
        assert be.dev_q4k_gemm(w, dx, rows, hidden, seq, out)
        be.synchronize()
        r = be.d2h(out, (seq, rows), F)
        be.free(dx)
        return r

    base = gemm(xb)
    assert np.isfinite(base).all()
    # permuting the tokens permutes the result rows, bit for bit
    perm = rng.permutation(seq)
    assert np.array_equal(gemm(xb[perm]).view(np.uint32), base[perm].view(np.uint32))
    # scaling the activations by a power of two scales the result exactly (bf16 * 4 stays bf16)
    x4 = O.f32_to_bf16((Xr * F(4.0)).astype(F)).reshape(seq, hidden)
    assert np.array_equal(gemm(x4).view(np.uint32), (base * F(4.0)).view(np.uint32))
    # rows of the product equal the matvec of that token (the reference's contract for q4k_matmul), on a sample
    r0 = (rows // 2 - 512) & ~15
    wb = be.d2h(w + r0 * (hidden // 256) * 144, 64 * (hidden // 256) * 144, np.uint8)
    for t in (0, 255, 511):
        want = O.q4k_matvec(wb, Xr[t], 64, hidden)
        assert rel_l2(base[t, r0:r0 + 64], want) < 5e-4     # stated bar 1e-3; the f16 weight operand carries the rows' scales: ~3e-4
    be.free(w); be.free(out)


def test_moe_block_full_size_weight_scaling_and_token_permutation(be, fmt):
    """configs[3]: 32 experts x (gate, up, down 2880 x 2880), top-4, 16 tokens."""
    E, H, I, k, T = 32, 2880, 2880, 4, 16
    per = H * I
    tmp = be.malloc(per * 4)
    bufs = {}
    for name, seed in (("gate", 0x5EED0400), ("up", 0x5EED0440), ("down", 0x5EED0480)):
        p, s = be.malloc(E * per // 2 + 64), be.malloc(E * per // 32 + 64)
        for e in range(E):
            assert be.dev_fill_normal(tmp, per, seed + e, 0.02)
            assert be.dev_quantize_mxfp4(tmp, H, I, p + e * per // 2, s + e * per // 32)
        bufs[name] = (p, s)
    be.free(tmp)
    bank = fmt.Mxfp4Experts(bufs["gate"][0], bufs["gate"][1], bufs["up"][0], bufs["up"][1], bufs["down"][0], bufs["down"][1], E, H, I,
                            7.0, 1.702, 0)
    rng = np.random.default_rng(4)
    X = rng.standard_normal((T, H)).astype(F)
    logits = rng.standard_normal((T, E)).astype(F)
    wsb = be.moe_mxfp4_workspace_bytes(T, k, H, I)
    ws = be.malloc(wsb)

    def block(x, lg, scale=1.0):
        dx, dl = be.to_device(np.ascontiguousarray(x)), be.to_device(np.ascontiguousarray(lg))
        de, dw, do = be.malloc(T * k * 4), be.malloc(T * k * 4), be.malloc(T * H * 4)
        assert be.dev_router_select(dl, T, E, k, O.NORMALISED_OVER_SELECTED, de, dw)
        if scale != 1.0:
            be.synchronize()
            wv = be.d2h(dw, T * k, F)
            be.free(dw)
            dw = be.to_device((wv * F(scale)).astype(F))
        assert be.dev_moe_mxfp4(bank, dx, T, k, de, dw, do, ws, wsb)
        be.synchronize()
        r, ex = be.d2h(do, (T, H), F), be.d2h(de, (T, k), np.uint32)
        for p in (dx, dl, de, dw, do):
            be.free(p)
        return r, ex

    base, experts = block(X, logits)
    assert np.isfinite(base).all() and np.abs(base).max() > 0
    for t in range(T):                                                                # the router's choice is the oracle's
        assert [int(e) for e in experts[t]] == [i for i, _ in O.router_select(logits[t], k)]
    # routing weights scaled by a power of two scale the block's output exactly
    assert np.array_equal(block(X, logits, 0.5)[0].view(np.uint32), (base * F(0.5)).view(np.uint32))
    # tokens in another order: the same results, row for row (who shares an expert's read with whom does not matter)
    perm = rng.permutation(T)
    assert np.array_equal(block(X[perm], logits[perm])[0].view(np.uint32), base[perm].view(np.uint32))
    # one token of the 16 against the oracle's block (the four experts it chose, downloaded and renumbered 0..3)
    def chosen_bank(ids):
        m = {nm: (np.concatenate([be.d2h(bufs[nm][0] + int(e) * per // 2, per // 2, np.uint8) for e in ids]),
                  np.concatenate([be.d2h(bufs[nm][1] + int(e) * per // 32, per // 32, np.uint8) for e in ids])) for nm in bufs}
        return m
    t = 11
    sel = O.router_select(logits[t], k)
    m = chosen_bank([e for e, _ in sel])
    want = O.moe_block_mxfp4(X[t:t + 1], np.arange(k, dtype=np.uint64)[None], np.array([[w for _, w in sel]], F), m["gate"], m["up"],
                             m["down"], k, H, I)
    assert rel_l2(base[t], want[0]) < 1e-5
    # configs[3] at batch 1 on the same 32-expert bank, with router / gate_up / down biases: selection inside the first
    # launch, experts and weighted sum folded into the down projection (two launches)
    rb = rng.standard_normal(E).astype(F)
    gub = (rng.standard_normal((E, 2 * I)) * 0.5).astype(F)
    db = (rng.standard_normal((E, H)) * 0.5).astype(F)
    drb, dgub, ddb = be.to_device(rb), be.to_device(gub), be.to_device(db)
    bank_b = fmt.Mxfp4Experts(bufs["gate"][0], bufs["gate"][1], bufs["up"][0], bufs["up"][1], bufs["down"][0], bufs["down"][1], E, H, I,
                              7.0, 1.702, 0, drb, dgub, ddb)
    for t in (0, 5, 11):
        dx, dl = be.to_device(X[t]), be.to_device(logits[t])
        de, dw, do = be.malloc(k * 4), be.malloc(k * 4), be.malloc(H * 4)
        assert be.dev_moe_mxfp4_routed(bank_b, dx, 1, k, dl, O.NORMALISED_OVER_SELECTED, de, dw, do, ws, wsb)
        be.synchronize()
        ex, wt, got = be.d2h(de, k, np.uint32), be.d2h(dw, k, F), be.d2h(do, H, F)
        sel = O.router_select(logits[t] + rb, k)
        assert [int(e) for e in ex] == [e for e, _ in sel]
        m = chosen_bank(ex)
        want = O.moe_block_mxfp4(X[t:t + 1], np.arange(k, dtype=np.uint64)[None], wt[None], m["gate"], m["up"], m["down"], k, H, I,
                                 gate_up_bias=gub[ex], down_bias=db[ex])
        assert rel_l2(got, want[0]) < 1e-5, t
        for p in (dx, dl, de, dw, do):
            be.free(p)
    for p, s in bufs.values():
        be.free(p); be.free(s)
    be.free(ws)


def test_q4k_encoder_full_matrix_round_trip_and_sampled_blocks(be):
    """quantize_q4_k over a 10240 x 2560 matrix on the device: sampled super-blocks byte for byte against the oracle,
    and the decode of everything within the format's step of the source (the reference's round-trip property,
    larql-compute/tests/test_q4k_parity.rs:48-65)."""
    rows, k = 10240, 2560
    tmp, w = dev_q4k_matrix(be, rows, k, 0x5EED0600)
    src = be.d2h(tmp, rows * k, F)
    q = be.d2h(w, q4k_bytes(rows, k), np.uint8)
    blocks = q.reshape(-1, 144)
    for sb in (0, 1, 12345, blocks.shape[0] // 2, blocks.shape[0] - 1):
        assert np.array_equal(blocks[sb], O.quantize_q4_k(src[sb * 256:(sb + 1) * 256]))
    # round trip of a 512-row slab: |w - decode| within one nibble step of the super-block's widest sub-block
    part = slice(4096 * k, 4608 * k)
    dec = O.dequantize_q4_k(q[4096 * (k // 256) * 144:4608 * (k // 256) * 144], 512 * k)
    err = np.abs(dec - src[part]).reshape(-1, 32).max(axis=1)
    blk = src[part].reshape(-1, 256)
    step = (blk.max(axis=1).clip(min=0) - blk.min(axis=1).clip(max=0)) / 15.0       # one nibble step of the widest sub-block
    assert (err.reshape(-1, 8) <= step[:, None] + 1e-6).all()
    be.free(tmp); be.free(w)
