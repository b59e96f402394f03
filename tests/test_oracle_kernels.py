"""Pins the CPU checker's kernels: Q4_K / Q8_0 / MXFP4 / Q4_0xQ8 matvecs,
Q4_K matmul, top-K by |score|, lm_head top-K, batch union, MoE routing.
Expected values come from the reference's own test invariants (kernel ==
decode-then-multiply), f64 brute force, closed forms, and the reference's C
kernel compiled from its tree."""
import numpy as np
import pytest

import np_restatement as npr
import oracle as O

F = np.float32


def bits(a):
    return np.asarray(a, F).view(np.uint32)


def seq_dot_f32(w, x):
    """Row dots in f32, element order, multiply then add (no FMA)."""
    out = np.zeros(w.shape[0], F)
    for r in range(w.shape[0]):
        acc = F(0)
        for c in range(w.shape[1]):
            acc = F(acc + F(w[r, c] * x[c]))
        out[r] = acc
    return out


def rel_l2(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


# ------------------------------------------------------------------ Q4_K matvec
@pytest.mark.parametrize("rows,cols", [(4, 256), (37, 1024), (64, 2560)])
def test_q4k_matvec_equals_dequant_then_dot(rows, cols):
    # quantize_q4_0_tests.rs:69-149 (abs 1e-3 / 5e-3 there); f64 brute force here
    rng = np.random.default_rng(rows)
    w = (rng.standard_normal((rows, cols)) * 0.02).astype(F)
    x = rng.standard_normal(cols).astype(F)
    q = O.quantize_q4_k(w)
    deq = O.dequantize_q4_k(q, rows * cols).reshape(rows, cols)
    exact = deq.astype(np.float64) @ x.astype(np.float64)
    got = O.q4k_matvec(q, x, rows, cols)
    assert rel_l2(got, exact) < 2e-6
    assert np.max(np.abs(got - exact)) < 1e-3
    # the scalar cross-backend reference (different association) agrees too
    assert rel_l2(O.q4k_matvec_scalar(q, x, rows, cols), exact) < 2e-6
    # row-chunk threading changes nothing
    assert np.array_equal(bits(O.q4k_matvec_mt(q, x, rows, cols, 3)), bits(got))


def test_q4k_matvec_hand_computed_block():
    # d=1 (0x3C00), dmin=0.5 (0x3800); scales j = j+1, mins j = j; nibble lo=3, hi=5
    blk = np.zeros(144, np.uint8)
    blk[0:2] = [0x00, 0x3C]; blk[2:4] = [0x00, 0x38]
    sc = np.arange(1, 9, dtype=np.uint8); mn = np.arange(0, 8, dtype=np.uint8)
    for j in range(4):
        blk[4 + j] = (sc[j] & 63) | (((sc[j + 4] >> 4) & 3) << 6)
        blk[8 + j] = (mn[j] & 63) | (((mn[j + 4] >> 4) & 3) << 6)
        blk[12 + j] = (sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4)
    blk[16:] = 3 | (5 << 4)
    x = np.ones(256, F)
    # sub-block s contributes 32*(sc_s*q - 0.5*mn_s), q = 3 for even s, 5 for odd s
    want = sum(32 * (float(sc[s]) * (3 if s % 2 == 0 else 5) - 0.5 * float(mn[s])) for s in range(8))
    assert O.q4k_matvec(blk, x, 1, 256)[0] == want
    assert np.array_equal(O.dequantize_q4_k(blk, 256)[[0, 32, 255]], np.array([3.0, 2 * 5 - 0.5, 8 * 5 - 3.5], F))


def test_q4k_matvec_refusals_and_zero_dims():
    # quantize_q4_0_tests.rs:351-389, kernel_shape.rs:97-149
    rng = np.random.default_rng(1)
    w = O.quantize_q4_k((rng.standard_normal(3 * 512) * 0.02).astype(F))
    x = rng.standard_normal(512).astype(F)
    assert O.q4k_matvec(w, x, 3, 512) is not None
    assert O.q4k_matvec(w, x, 3, 512, out_len=2) is None          # out shorter than rows
    assert O.q4k_matvec(w, x[:511], 3, 512) is None               # activation not cols long
    assert O.q4k_matvec(w, x[:500], 3, 500) is None               # cols not a super-block multiple
    assert O.q4k_matvec(w[:-1], x, 3, 512) is None                # weight slab short
    assert O.q4k_matvec(np.concatenate([w, w]), x, 3, 512) is not None   # longer slab is fine (>=)
    z = O.q4k_matvec(np.zeros(0, np.uint8), np.zeros(0, F), 4, 0)
    assert z is not None and z.shape == (4,) and not z.any()      # zero dims: zeros, not refusal
    assert O.q4k_matvec(np.zeros(0, np.uint8), np.zeros(0, F), 0, 0).size == 0


def test_q4k_dual_is_two_singles():
    rng = np.random.default_rng(2)
    rows, cols = 33, 768
    a = O.quantize_q4_k((rng.standard_normal(rows * cols) * 0.02).astype(F))
    b = O.quantize_q4_k((rng.standard_normal(rows * cols) * 0.05).astype(F))
    x = rng.standard_normal(cols).astype(F)
    oa, ob = O.q4k_dual_matvec(a, b, x, rows, cols)
    assert np.array_equal(bits(oa), bits(O.q4k_matvec(a, x, rows, cols)))
    assert np.array_equal(bits(ob), bits(O.q4k_matvec(b, x, rows, cols)))
    assert O.q4k_dual_matvec(a, b[:-1], x, rows, cols) is None


def test_q4k_matmul_rows_match_matvec_and_dequant():
    # quantize_q4_0_tests.rs:155-238: vs dequant 5e-3, rows vs matvec 1e-4; [seq, rows] layout
    rng = np.random.default_rng(3)
    rows, hidden, seq = 40, 512, 5
    q = O.quantize_q4_k((rng.standard_normal(rows * hidden) * 0.02).astype(F))
    X = rng.standard_normal((seq, hidden)).astype(F)
    out = O.q4k_matmul(q, X, rows, hidden, seq)
    assert out.shape == (seq, rows)
    deq = O.dequantize_q4_k(q, rows * hidden).reshape(rows, hidden).astype(np.float64)
    exact = X.astype(np.float64) @ deq.T
    assert np.max(np.abs(out - exact)) < 1e-4
    for s in range(seq):
        assert np.max(np.abs(out[s] - O.q4k_matvec(q, X[s], rows, hidden))) < 1e-4
    # shape errors zero the output (matmul.rs:89-98)
    assert not O.q4k_matmul(q, X[:, :500], rows, 500, seq).any()
    assert not O.q4k_matmul(q[:-1], X, rows, hidden, seq).any()


# ------------------------------------------------------------------------- Q8_0
def test_q8_0_gemv_is_bit_for_bit_dequant_then_dot():
    # kquant_gemv_tests.rs:92-105 (assert_eq!)
    rng = np.random.default_rng(4)
    n, k = 9, 96
    w = (rng.standard_normal(n * k) * 0.02).astype(F)
    w[:32] *= 1e-5                                       # a subnormal-scale block
    q = O.quantize_q8_0(w)
    x = rng.standard_normal(k).astype(F)
    deq = O.dequantize_q8_0(q, n * k).reshape(n, k)
    assert np.array_equal(bits(O.q8_0_gemv(q, x, n, k)), bits(seq_dot_f32(deq, x)))
    assert np.array_equal(bits(O.q8_0_gemv_mt(q, x, n, k, 4)), bits(O.q8_0_gemv(q, x, n, k)))


def test_q8_0_gemv_refusals():
    # kquant_gemv_tests.rs:133-151: exact length, k on the block grid, x.len()==k
    q = np.zeros(2 * 2 * 34, np.uint8)
    x = np.zeros(64, F)
    assert O.q8_0_gemv(q, x, 2, 64) is not None
    assert O.q8_0_gemv(q, x, 2, 0) is None
    assert O.q8_0_gemv(q, x[:48], 2, 48) is None
    assert O.q8_0_gemv(q, x[:63], 2, 64) is None
    assert O.q8_0_gemv(q[:-1], x, 2, 64) is None
    assert O.q8_0_gemv(np.concatenate([q, q[:1]]), x, 2, 64) is None     # longer is refused too


# ------------------------------------------------------------------- Q4_0 x Q8
def test_q4_0_matvec_matches_reference_c_kernel_bit_for_bit():
    rng = np.random.default_rng(5)
    rows, hidden = 70, 2560
    w = (rng.standard_normal(rows * hidden) * 0.02).astype(F)
    x = rng.standard_normal(hidden).astype(F)
    q4 = O.quantize_q4_0(w)
    q8, sc = O.quantize_to_q8(x)
    mine = O.q4_0_matvec(q4, q8, sc, rows, hidden)
    ref = O.ref_q4_0_matvec(q4, q8, sc, rows, hidden)
    if ref is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    assert np.array_equal(bits(mine), bits(ref))
    # and it approximates the f32 product (tests/test_q4_x86_correctness.rs)
    exact = w.reshape(rows, hidden).astype(np.float64) @ x.astype(np.float64)
    assert rel_l2(mine, exact) < 0.15
    # dequantise_q8 inverts quantize_to_q8 up to the code step
    back = O.dequantise_q8(q8, sc)
    assert np.max(np.abs(back - x)) <= np.max(sc) * 0.5 + 1e-7


# ------------------------------------------------------------------------ MXFP4
def test_mxfp4_gemv_equals_dequant_then_dot_and_sentinels():
    # larql-compute-metal/src/trait_impl/mxfp4.rs:223-326: cos>0.999999, rel<1e-4, sentinels 0/255, ragged rows
    rng = np.random.default_rng(6)
    n, k = 37, 2880
    w = (rng.standard_normal(n * k) * 0.02).astype(F)
    p, s = O.quantize_mxfp4(w, n, k)
    x = rng.standard_normal(k).astype(F)
    a = O.mxfp4_gemv(p, s, x, n, k)
    b = O.mxfp4_gemv_dequant(p, s, x, n, k)
    exact = npr.dequantize_mxfp4(p, s, n, k).astype(np.float64) @ x.astype(np.float64)
    assert rel_l2(a, exact) < 2e-6 and rel_l2(b, exact) < 2e-6
    s2 = s.copy(); s2[0] = 0; s2[90] = 255              # row 0 group 0 zeroed; row 1 gets a NaN group
    a2 = O.mxfp4_gemv(p, s2, x, n, k)
    assert np.isnan(a2[1]) and np.isfinite(a2[0]) and np.array_equal(bits(a2[2:]), bits(a[2:]))
    assert O.mxfp4_gemv(p, s, x[:-1], n, k) is None
    assert O.mxfp4_gemv(p[:-1], s, x, n, k) is None
    assert O.mxfp4_gemv(p, s[:-1], x, n, k) is None
    assert O.mxfp4_gemv(p, s, x, n, 2881) is None
    assert O.mxfp4_gemv(p, s, np.concatenate([x, x]), n, k) is not None   # x longer is accepted (>=)


# ------------------------------------------------------------------ dense gemv
def test_dense_gemvs_are_sequential_f32():
    rng = np.random.default_rng(7)
    n, k = 6, 100
    w = (rng.standard_normal((n, k)) * 0.02).astype(F)
    x = rng.standard_normal(k).astype(F)
    assert np.array_equal(bits(O.f32_gemv(w, x, n, k)), bits(seq_dot_f32(w, x)))
    wb = O.f32_to_bf16(w)
    wbf = (wb.astype(np.uint32) << 16).view(F).reshape(n, k)
    assert np.array_equal(bits(O.bf16_gemv(wb, x, n, k)), bits(seq_dot_f32(wbf, x)))
    w2 = O.f32_to_bf16((rng.standard_normal((70, k)) * 0.02).astype(F))     # the threaded timing baseline: same bits, ragged chunks
    assert np.array_equal(bits(O.bf16_gemv_mt(w2, x, 70, k, 3)), bits(O.bf16_gemv(w2, x, 70, k)))
    wh = w.astype(np.float16)
    assert np.array_equal(bits(O.f16_gemv(wh.view(np.uint16), x, n, k)), bits(seq_dot_f32(wh.astype(F), x)))


# ------------------------------------------------------------------------ top-K
def test_top_k_by_abs_reference_cases():
    # gate_knn/mod.rs:231-287
    r = O.top_k_by_abs([0.1, -0.9, 0.5, 0.3], 2)
    assert [i for i, _ in r] == [1, 2] and abs(r[0][1] + 0.9) < 1e-6
    assert O.top_k_by_abs([1.0, -2.0, 0.5], 1)[0][0] == 1
    assert len(O.top_k_by_abs([1.0, 2.0], 10)) == 2
    assert O.top_k_by_abs([1.0, 2.0, 3.0], 0) == []
    assert O.top_k_by_abs([], 5) == []
    r = O.top_k_by_abs([0.3, 0.1, 0.9, 0.5, 0.7], 3)
    assert [i for i, _ in r] == [2, 4, 3]
    with pytest.raises(ValueError):
        O.top_k_by_abs([1.0, float("nan")], 1)


@pytest.mark.parametrize("n,k", [(10240, 64), (1000, 1), (77, 77), (50, 200)])
def test_top_k_by_abs_equals_full_sort_on_tie_free_data(n, k):
    rng = np.random.default_rng(n + k)
    # distinct magnitudes by construction: a shuffled ramp with random signs
    s = ((rng.permutation(n) + 1) / F(n) * rng.choice([-1.0, 1.0], n)).astype(F)
    assert len(np.unique(np.abs(s))) == n
    order = np.argsort(-np.abs(s), kind="stable")[: min(k, n)]
    got = O.top_k_by_abs(s, k)
    assert [i for i, _ in got] == list(order)
    assert [v for _, v in got] == [float(s[i]) for i in order]


def test_top_k_by_abs_ties_at_the_boundary():
    # Strict '>' replacement: a later equal |score| never displaces a kept one,
    # but WHICH of several equal minima is evicted follows the heap's order
    # (Rust's BinaryHeap), so only the multiset of |scores| is fixed.
    s = np.array([5, 1, -1, 1, 4, -1], F)
    got = O.top_k_by_abs(s, 3)
    assert [abs(v) for _, v in got] == [5.0, 4.0, 1.0]
    assert got[0][0] == 0 and got[1][0] == 4 and got[2][0] in (1, 2)
    # hand-traced on std's sift_up / sift_down_to_bottom: heap after three pushes is
    # [idx1, idx0, idx2]; the 4.0 evicts the root, idx1, so idx2 survives.
    assert got[2][0] == 2
    # no displacement without a strictly larger |score|
    assert [i for i, _ in O.top_k_by_abs(np.array([1, -1, 1, -1], F), 2)] == [0, 1]


def test_top_k_sorted_by_value_and_skips_non_finite():
    s = np.array([0.5, np.inf, 3.0, -7.0, np.nan, 2.0, 2.5], F)
    assert O.top_k_sorted(s, 1) == [(2, 3.0)]
    assert O.top_k_sorted(s, 3) == [(2, 3.0), (6, 2.5), (5, 2.0)]
    assert [i for i, _ in O.top_k_sorted(s, 99)] == [2, 6, 5, 0, 3]
    assert O.top_k_sorted(np.array([np.nan, np.inf], F), 1) == []
    rng = np.random.default_rng(8)
    v = rng.standard_normal(5000).astype(F)
    assert [i for i, _ in O.top_k_sorted(v, 8)] == list(np.argsort(-v, kind="stable")[:8])


def test_gate_knn_batch_union():
    # dispatch.rs:256-304: per-position top-k, sorted de-duplicated union
    rng = np.random.default_rng(9)
    n, seq, k = 500, 8, 16
    s2d = rng.standard_normal((n, seq)).astype(F)
    want = sorted(set(int(i) for c in range(seq) for i in np.argsort(-np.abs(s2d[:, c]), kind="stable")[:k]))
    assert O.gate_knn_batch_union(s2d, k) == want
    assert O.gate_knn_batch_union(s2d[:, :0], k) == []
    assert O.gate_knn_batch_union(s2d[:5], 64) == [0, 1, 2, 3, 4]


# ---------------------------------------------------------------------- routing
def test_router_select_reference_kats():
    # router.rs:79-200
    logits = np.array([2.0] * 4 + [1.0] * 28, F)
    norm = O.router_select(logits, 4, O.NORMALISED_OVER_SELECTED)
    raw = O.router_select(logits, 4, O.SOFTMAX_THEN_SELECT)
    assert abs(sum(w for _, w in norm) - 1.0) < 1e-6 and sum(w for _, w in raw) < 0.7
    ex = np.exp(logits.astype(np.float64) - 2.0); ex /= ex.sum()
    for e, w in raw:
        assert abs(w - ex[e]) < 1e-6
    tot = sum(w for _, w in raw)
    for (e1, w1), (e2, w2) in zip(raw, norm):
        assert e1 == e2 and abs(w1 / tot - w2) < 1e-6
    assert [e for e, _ in norm] == [0, 1, 2, 3]                      # ties -> first index
    l2 = np.array([0.1, 5.0, 0.2, 4.0, 0.3, 3.0, 0.4, 2.0], F)
    assert [e for e, _ in O.router_select(l2, 3)] == [1, 3, 5]
    assert O.router_select(l2, 0) == [] and len(O.router_select(l2, 99)) == 8
    # GPT-OSS shape: softmax over the selected logits
    rng = np.random.default_rng(10)
    lg = rng.standard_normal(32).astype(F)
    sel = O.router_select(lg, 4)
    top = np.argsort(-lg, kind="stable")[:4]
    assert [e for e, _ in sel] == list(top)
    sm = np.exp(lg[top].astype(np.float64) - lg[top].max()); sm /= sm.sum()
    assert np.allclose([w for _, w in sel], sm, atol=1e-6)


def test_moe_top_k_softmax_and_clamped_glu():
    # math.rs:231-258: ties -> lower index; softmax sums to 1
    idx, val = O.moe_top_k([1.0, 3.0, 3.0, 2.0], 2)
    assert idx == [1, 2] and val == [3.0, 3.0]
    sm = O.softmax([1.0, 2.0, 3.0])
    assert abs(sm.sum() - 1) < 1e-6 and np.allclose(sm, np.exp([1, 2, 3]) / np.exp([1, 2, 3]).sum(), atol=1e-6)
    # pipeline/moe.rs:88-92: g=min(g,L); u=clamp(u,+-L); (u+1)*g*sigmoid(alpha*g)
    for g, u in [(0.5, -0.25), (9.0, 9.0), (-9.0, -9.0), (0.0, 3.0)]:
        gc, uc = min(g, 7.0), max(-7.0, min(7.0, u))
        want = (uc + 1.0) * gc / (1.0 + np.exp(-1.702 * gc))
        assert abs(O.clamped_glu(g, u) - want) < 1e-5 * max(1.0, abs(want))


def test_fused_gate_up_row_walk_is_interleaved_not_contiguous_halves():
    # FusedHalf::fused_row / deinterleave_fused_half / split_gate_up_experts (larql-models/src/quant/mxfp4.rs:179-268) and
    # MoeFusedRowLayout::row_walk (larql-compute/src/pipeline/moe.rs:313-332), on the reference's own fixtures
    # (mxfp4.rs:485-535: fused_row_indices_interleave, deinterleave_takes_even_rows_for_gate_and_odd_for_up,
    # split_gate_up_is_interleaved_not_contiguous_halves)
    first, step = O.fused_row_walk(O.INTERLEAVED, O.HALF_GATE, 8)
    assert [first + step * r for r in (0, 1, 7)] == [0, 2, 14]
    first, step = O.fused_row_walk(O.INTERLEAVED, O.HALF_UP, 8)
    assert [first + step * r for r in (0, 1, 7)] == [1, 3, 15]
    assert O.fused_row_walk(O.CONTIGUOUS_HALVES, O.HALF_GATE, 8) == (0, 1)
    assert O.fused_row_walk(O.CONTIGUOUS_HALVES, O.HALF_UP, 8) == (8, 1)
    data = np.array([0, 0, 1, 1, 2, 2, 3, 3], F)
    assert O.deinterleave_fused_half(data, 4, 2, O.HALF_GATE).tolist() == [0, 0, 2, 2]
    assert O.deinterleave_fused_half(data, 4, 2, O.HALF_UP).tolist() == [1, 1, 3, 3]
    # four fused rows whose value is their own scale (nibble 2 = 1.0): rows = [1, 2, 4, 8]
    blocks, scales = np.full(4 * 16, 0x22, np.uint8), np.array([127, 128, 129, 130], np.uint8)
    dense = O.dequantize_mxfp4_expert(blocks, scales, 4, 1)
    gate = O.deinterleave_fused_half(dense, 4, 32, O.HALF_GATE).reshape(2, 32)[:, 0].tolist()
    up = O.deinterleave_fused_half(dense, 4, 32, O.HALF_UP).reshape(2, 32)[:, 0].tolist()
    assert gate == [1.0, 4.0] and up == [2.0, 8.0]
