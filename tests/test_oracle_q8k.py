"""The Q8_K-activation integer path of the oracle (quantize_x_to_q8k, q4k_q8k_matvec_scalar) against the
properties and inputs the reference's own tests use (larql-compute/src/cpu/ops/q4k_q8k_dot/tests/
q8k_quantize_and_matvec.rs, fused_and_q6k_paths.rs, public_execution_path_q4k_q8k_matvec_par.rs), closed forms,
and an independent numpy restatement.  The reference holds no vector for these functions: parity unpinned."""
import numpy as np
import pytest

import np_restatement as npr
import oracle as O

F = np.float32


def test_q8k_quantize_reference_properties():
    # q8k_quantize_round_trip_within_quant_step (:18-40): the reference's ramp
    x = ((np.arange(256, dtype=F) / F(128.0) - F(1.0)) * F(5.0)).astype(F)
    qs, d, sums = O.quantize_x_to_q8k(x)
    assert qs.shape == (256,) and d.shape == (1,) and sums.shape == (8,)
    step = np.abs(x).max() / F(127.0)
    assert np.all(np.abs(x - d[0] * qs.astype(F)) < max(step, 1e-6))
    assert np.array_equal(sums, qs.reshape(8, 32).astype(np.int32).sum(axis=1).astype(np.int16))
    # the extreme of the block is exactly +-127 and d = amax/127 as f32
    assert qs[0] == -127 and d[0] == F(5.0) / F(127.0)
    # q8k_zero_input_clean (:43-50)
    qs, d, sums = O.quantize_x_to_q8k(np.zeros(256, F))
    assert d[0] == 0.0 and not qs.any() and not sums.any()
    with pytest.raises(ValueError):
        O.quantize_x_to_q8k(np.zeros(255, F))


def test_q8k_quantize_closed_forms():
    # per-block scales are independent; half-way cases round away from zero; the clamp holds the inverse's rounding error
    x = np.zeros(512, F)
    x[0] = 127.0                      # block 0: d = 1, inv = 1
    x[1:6] = [0.5, -0.5, 1.5, 2.5, -2.5]
    x[6] = 126.49999
    x[256] = -3.0e-30                 # block 1: a tiny block quantises on its own scale
    x[257] = 1.5e-30
    qs, d, sums = O.quantize_x_to_q8k(x)
    assert d[0] == F(1.0) and list(qs[:7]) == [127, 1, -1, 2, 3, -3, 126]
    assert qs[256] == -127 and qs[257] == 64 and d[1] == F(3.0e-30) / F(127.0)   # 63.5 -> 64
    assert sums[0] == 127 + 1 - 1 + 2 + 3 - 3 + 126 and sums[8] == -127 + 64 and not sums[1:8].any()
    # negative zero and denormal inputs
    x = np.full(256, -0.0, F); x[3] = np.float32(1e-42)
    qs, d, sums = O.quantize_x_to_q8k(x)
    assert qs[3] == 127 and d[0] > 0 and qs.sum() == 127


@pytest.mark.parametrize("seed,scale", [(0, 1.0), (1, 1e-6), (2, 3e4), (3, 0.02)])
def test_q8k_quantize_agrees_with_numpy_restatement(seed, scale):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(256 * 9) * scale).astype(F)
    x[5] = 0.0
    x[256:512] = 0.0                  # an all-zero block in the middle
    x[700] = F(scale) * 8             # an outlier
    a, b = O.quantize_x_to_q8k(x), npr.quantize_x_to_q8k(x)
    for u, v in zip(a, b):
        assert np.array_equal(u, v)


def _ref_inputs(rows, cols, fx, fw):
    x = np.array([fx(F(i)) for i in range(cols)], F)
    w = np.array([fw(F(i)) for i in range(rows * cols)], F)
    return x, O.quantize_q4_k(w)


def test_q4k_q8k_matvec_within_q8_noise_of_the_f32_path_on_the_reference_inputs():
    # q8k_matvec_matches_f32_cached_within_q8_noise (:57-90): diff < 5e-2; multi-block (:95-121): diff < 8e-2
    x, w = _ref_inputs(4, 256, lambda i: np.sin(i * F(0.013)), lambda i: np.cos(i * F(0.007)) * F(0.5))
    f32 = O.q4k_matvec(w, x, 4, 256)
    q8 = O.q4k_q8k_matvec(w, *O.quantize_x_to_q8k(x), 4, 256)
    assert np.all(np.abs(f32 - q8) < 5e-2)
    x, w = _ref_inputs(16, 512, lambda i: np.cos(i * F(0.011)) * F(2.0), lambda i: np.sin(i * F(0.009)) * F(0.3))
    f32 = O.q4k_matvec(w, x, 16, 512)
    q8 = O.q4k_q8k_matvec(w, *O.quantize_x_to_q8k(x), 16, 512)
    assert np.all(np.abs(f32 - q8) < 8e-2)


def _block(d, dmin, sc, mn, lo, hi):
    """One hand-built Q4_K super-block: f16 d/dmin bits, 8 six-bit scales and mins, nibbles lo/hi [4][32]."""
    b = np.zeros(144, np.uint8)
    b[0:2] = np.array([d], np.float16).view(np.uint8)
    b[2:4] = np.array([dmin], np.float16).view(np.uint8)
    for j in range(4):
        b[4 + j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
        b[8 + j] = (mn[j] & 63) | ((mn[j + 4] >> 4) << 6)
        b[12 + j] = (sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4)
    b[16:] = (np.asarray(lo, np.uint8) | (np.asarray(hi, np.uint8) << 4)).reshape(-1)
    return b


def test_q4k_q8k_matvec_hand_computed_block():
    # sub-block m has scale m+1 and min 2m; low nibbles of group g are g+1, high nibbles 15-g; y = +3 in even
    # sub-blocks, -2 in odd ones: every term is a small integer that can be written down
    sc = [1, 2, 3, 4, 5, 6, 7, 40]
    mn = [0, 2, 4, 6, 8, 10, 12, 63]
    lo = np.array([[g + 1] * 32 for g in range(4)])
    hi = np.array([[15 - g] * 32 for g in range(4)])
    w = _block(0.5, 0.25, sc, mn, lo, hi)
    qs = np.concatenate([np.full(32, 3 if m % 2 == 0 else -2, np.int8) for m in range(8)])
    sums = np.array([32 * (3 if m % 2 == 0 else -2) for m in range(8)], np.int16)
    d = np.array([0.125], F)
    sum1 = sum(sc[2 * g] * (g + 1) * 3 * 32 + sc[2 * g + 1] * (15 - g) * (-2) * 32 for g in range(4))
    sum2 = sum(mn[m] * int(sums[m]) for m in range(8))
    want = F(F(0.5) * F(0.125)) * F(sum1) - F(F(0.25) * F(0.125)) * F(sum2)
    got = O.q4k_q8k_matvec(w, qs, d, sums, 1, 256)
    assert got[0] == want
    # the activation scale is a factor of every term: a power of two scales the output exactly
    assert O.q4k_q8k_matvec(w, qs, d * F(8), sums, 1, 256)[0] == want * F(8)
    # sums are an input, not recomputed: the min term follows them
    assert O.q4k_q8k_matvec(w, qs, d, np.zeros(8, np.int16), 1, 256)[0] == F(F(0.5) * F(0.125)) * F(sum1)


@pytest.mark.parametrize("rows,cols,seed", [(7, 1024, 0), (33, 2560, 1), (3, 10240, 2), (1, 256, 3)])
def test_q4k_q8k_matvec_agrees_with_numpy_restatement_bit_for_bit(rows, cols, seed):
    rng = np.random.default_rng(100 + seed)
    w = O.quantize_q4_k((rng.standard_normal(rows * cols) * 0.05).astype(F))
    q = O.quantize_x_to_q8k((rng.standard_normal(cols) * 2).astype(F))
    a, b = O.q4k_q8k_matvec(w, *q, rows, cols), npr.q4k_q8k_matvec(w, *q, rows, cols)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # and equals the dequantised product in f64 to rounding
    deq = O.dequantize_q4_k(w, rows * cols).reshape(rows, cols).astype(np.float64)
    y = (np.repeat(q[1].astype(np.float64), 256) * q[0].astype(np.float64))
    assert np.allclose(a, deq @ y, rtol=0, atol=1e-4 * np.abs(deq @ y).max() + 1e-6)


def test_q4k_q8k_matvec_shape_rules():
    # KernelShapeError::check (cpu/ops/kernel_shape.rs:47-75); fused_and_q6k_paths.rs:53-84, public_execution_path...:33-78
    w = O.quantize_q4_k(np.ones(2 * 512, F))
    q = O.quantize_x_to_q8k(np.ones(512, F))
    assert O.q4k_q8k_matvec(w, *q, 2, 512) is not None
    assert O.q4k_q8k_matvec(w[:-1], *q, 2, 512) is None                       # short weight slab
    assert O.q4k_q8k_matvec(w, *O.quantize_x_to_q8k(np.ones(768, F)), 2, 512) is None   # activation of the wrong length
    assert O.q4k_q8k_matvec(np.concatenate([w, w]), *q, 2, 512) is not None   # longer slab is fine
    z = O.q4k_q8k_matvec(np.zeros(0, np.uint8), np.zeros(0, np.int8), np.zeros(0, F), np.zeros(0, np.int16), 3, 0)
    assert z is not None and z.shape == (3,) and not z.any()                  # zero dims give zeros


# ------------------------------------------------------------------ the Q6_K twin
def test_q6k_q8k_matvec_within_noise_of_the_f32_path_on_the_reference_inputs():
    # q6k_q8k_matvec_matches_q6k_f32_dispatch_within_noise (fused_and_q6k_paths.rs:87-110): diff < 1.2e-1 on these inputs
    rows, cols = 5, 512
    x = np.array([np.sin(F(i) * F(0.017)) * F(1.5) for i in range(cols)], F)
    w = O.quantize_q6_k(np.array([np.cos(F(i) * F(0.006)) * F(0.7) for i in range(rows * cols)], F))
    qs, d, _ = O.quantize_x_to_q8k(x)
    f32 = O.q6k_matvec(w, x, rows, cols)
    q8 = O.q6k_q8k_matvec(w, qs, d, rows, cols)
    assert np.all(np.abs(f32 - q8) < 1.2e-1)


def test_q6k_q8k_matvec_hand_computed_block():
    # every code 32 + 5 (low nibble 5, high bits 2), scale 3 for even groups and -2 for odd ones, d = 0.5; y = +2 / -1 per group
    b = np.zeros(210, np.uint8)
    b[:128] = 0x55
    b[128:192] = 0xAA
    b[192:208] = np.array([3, -2] * 8, np.int8).view(np.uint8)
    b[208:210] = np.array([0.5], np.float16).view(np.uint8)
    qs = np.concatenate([np.full(16, 2 if g % 3 == 0 else -1, np.int8) for g in range(16)])
    d = np.array([0.25], F)
    sum1 = sum((3 if g % 2 == 0 else -2) * 5 * 16 * (2 if g % 3 == 0 else -1) for g in range(16))
    want = F(F(0.5) * F(0.25)) * F(sum1)
    assert O.q6k_q8k_matvec(b, qs, d, 1, 256)[0] == want
    assert O.q6k_q8k_matvec(b, qs, d * F(4), 1, 256)[0] == want * F(4)


@pytest.mark.parametrize("rows,cols,seed", [(7, 1024, 0), (33, 2560, 1), (3, 10240, 2), (1, 256, 3)])
def test_q6k_q8k_matvec_agrees_with_numpy_restatement_bit_for_bit(rows, cols, seed):
    rng = np.random.default_rng(200 + seed)
    w = O.quantize_q6_k((rng.standard_normal(rows * cols) * 0.05).astype(F))
    qs, d, _ = O.quantize_x_to_q8k((rng.standard_normal(cols) * 2).astype(F))
    a, b = O.q6k_q8k_matvec(w, qs, d, rows, cols), npr.q6k_q8k_matvec(w, qs, d, rows, cols)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    deq = O.dequantize_q6_k(w, rows * cols).reshape(rows, cols).astype(np.float64)
    y = np.repeat(d.astype(np.float64), 256) * qs.astype(np.float64)
    assert np.allclose(a, deq @ y, rtol=0, atol=1e-4 * np.abs(deq @ y).max() + 1e-6)


def test_q6k_q8k_matvec_shape_rules():
    # fused_and_q6k_paths.rs:137-166: zero dims zero the output, a short weight slab is refused
    w = O.quantize_q6_k(np.ones(2 * 512, F))
    qs, d, _ = O.quantize_x_to_q8k(np.ones(512, F))
    assert O.q6k_q8k_matvec(w, qs, d, 2, 512) is not None
    assert O.q6k_q8k_matvec(w[:-1], qs, d, 2, 512) is None
    qs2, d2, _ = O.quantize_x_to_q8k(np.ones(768, F))
    assert O.q6k_q8k_matvec(w, qs2, d2, 2, 512) is None
    z = O.q6k_q8k_matvec(np.zeros(0, np.uint8), np.zeros(0, np.int8), np.zeros(0, F), 3, 0)
    assert z is not None and z.shape == (3,) and not z.any()
