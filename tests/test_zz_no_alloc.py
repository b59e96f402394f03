"""larql_hip_dev_gate_knn_static — the entry point that allocates nothing — against larql_hip_dev_gate_knn,
through the C ABI: same indices, same score bits, same counts, on two calls in a row, the second with a
smaller input (the static scratch keeps the first call's scores).  Every gate format the entry point serves."""
import numpy as np
import pytest

import oracle as O

pytestmark = pytest.mark.gpu
F = np.float32


def encode(fmt, name, w):
    if name == "q4k":
        return fmt.FMT_Q4_K, O.quantize_q4_k(w)
    if name == "q4_0":
        return fmt.FMT_Q4_0, O.quantize_q4_0(w)
    if name == "bf16":
        return fmt.FMT_BF16, O.f32_to_bf16(w)
    if name == "f16":
        return fmt.FMT_F16, w.astype(np.float16)
    return fmt.FMT_F32, w


def both(be, f, gate_dev, x, batch, n, hidden, k):
    xd = be.to_device(x)
    sc = be.malloc(batch * n * 4)
    i1, v1 = be.malloc(batch * k * 4), be.malloc(batch * k * 4)
    i2, v2, c2 = be.malloc(batch * k * 4), be.malloc(batch * k * 4), be.malloc(batch * 4)
    try:
        assert be.dev_gate_knn(f, gate_dev, xd, batch, n, hidden, k, sc, i1, v1)
        events = be.debug_alloc_events()
        assert be.dev_gate_knn_static(f, gate_dev, xd, batch, n, hidden, k, i2, v2, c2)
        # what the entry point exists for: it took no device memory, staged nothing and uploaded no job table
        assert be.debug_alloc_events() == events
        be.synchronize()
        m = min(k, n)
        a = be.d2h(i1, (batch, k), np.uint32)[:, :m], be.d2h(v1, (batch, k), np.uint32)[:, :m]
        b = be.d2h(i2, (batch, k), np.uint32)[:, :m], be.d2h(v2, (batch, k), np.uint32)[:, :m]
        cnt = be.d2h(c2, (batch,), np.uint32)
        scores = be.d2h(sc, (batch, n), F)
        return a, b, cnt, scores
    finally:
        for p in (xd, sc, i1, v1, i2, v2, c2):
            be.free(p)


@pytest.mark.parametrize("name", ["q4k", "bf16", "f16", "f32", "q4_0"])
def test_static_entry_equals_the_allocating_one_on_two_calls_in_a_row(be, name):
    import larql_amd as fmt
    rng = np.random.default_rng(17)
    hidden = 512
    shapes = [(8, 3000, 64), (3, 700, 17), (2, 2000, 200)]   # (batch, features, K): the second call is smaller; the third
    #                                                          takes the path for more than 64 winners (a sort in LDS)
    for batch, n, k in shapes:
        w = (rng.standard_normal((n, hidden)) * 0.02).astype(F)
        x = rng.standard_normal((batch, hidden)).astype(F)
        f, enc = encode(fmt, name, w)
        gd = be.to_device(np.ascontiguousarray(enc))
        try:
            (ia, va), (ib, vb), cnt, scores = both(be, f, gd, x, batch, n, hidden, k)
        finally:
            be.free(gd)
        assert np.array_equal(ia, ib) and np.array_equal(va, vb)
        assert list(cnt) == [min(k, n)] * batch
        # and both are the oracle's selection on the device's scores
        for b in range(batch):
            want = O.top_k_by_abs(scores[b], k)
            assert sorted(i for i, _ in want) == sorted(int(i) for i in ib[b])


def test_static_entry_refuses_what_does_not_fit(be):
    import larql_amd as fmt
    assert be.static_scratch_bytes() == 131072 * 4 + 256 + 8 * 16384 + 8 * 16384 // 32 * 4
    w = np.zeros((16, 256), F)
    gd, xd = be.to_device(O.quantize_q4_k(w)), be.to_device(np.zeros((9, 256), F))
    i, v = be.malloc(9 * 64 * 4), be.malloc(9 * 64 * 4)
    try:
        assert not be.dev_gate_knn_static(fmt.FMT_Q4_K, gd, xd, 9, 16, 256, 4, i, v)            # more than 8 positions
        assert "static scratch" in be.last_error()
        assert not be.dev_gate_knn_static(fmt.FMT_Q4_K, gd, xd, 2, 70000, 256, 4, i, v)         # 140000 scores
        assert not be.dev_gate_knn_static(fmt.FMT_Q4_0, gd, xd, 1, 16, 32768, 4, i, v)          # Q4_0 rows too long
        assert be.dev_gate_knn_static(fmt.FMT_Q4_K, gd, xd, 0, 16, 256, 4, i, v)                # empty: Some, nothing done
    finally:
        for p in (gd, xd, i, v):
            be.free(p)
