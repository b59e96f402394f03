"""GPU parity: the HIP path, driven through the C ABI (larql_amd.HipBackend is
a thin ctypes mirror of the trait), against the CPU oracle on the same seeded
inputs.  Bars: quantised bytes bit-exact; matvec outputs within 1e-3 relative
L2 (fp32 accumulate; measured ~1e-6, asserted at 2e-5 so a wrong scale or a
dropped term cannot hide); top-K index sets identical except at score ties
within 1e-5."""
import json
import os

import numpy as np
import pytest

import oracle as O

pytestmark = pytest.mark.gpu
F = np.float32
TOL = 2e-5


def rel_l2(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def weights(seed, rows, cols, sigma=0.02):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((rows, cols)) * sigma).astype(F), rng.standard_normal(cols).astype(F)


# ------------------------------------------------------------------- Q4_K
@pytest.mark.parametrize("rows,cols", [(3072, 1024), (2048, 2560), (1031, 2560), (77, 10240), (5, 256), (640, 2048),
                                       (300, 3840), (33, 1792), (257, 4096), (130, 7168), (48, 12288), (17, 3328),
                                       (1, 2560), (16, 2816), (4100, 512)])
def test_q4k_matvec_matches_oracle(be, rows, cols):
    w, x = weights(rows * 7 + cols, rows, cols)
    q = O.quantize_q4_k(w)
    want = O.q4k_matvec(q, x, rows, cols)
    got = be.q4k_matvec(q, x, rows, cols)
    assert got is not None and got.shape == (rows,)
    assert rel_l2(got, want) < TOL
    # every row individually (guards against unwritten or swapped rows)
    scale = np.abs(want).mean() + 1e-12
    assert np.max(np.abs(got - want)) < 1e-3 * scale
    # deterministic across repeats
    assert np.array_equal(got.view(np.uint32), be.q4k_matvec(q, x, rows, cols).view(np.uint32))


@pytest.mark.parametrize("case", ["outliers", "zero", "tiny", "huge", "one_hot"])
def test_q4k_matvec_activation_ranges(be, case):
    # the matrix-core kernel rescales every 256-wide slice of x by a power of two and splits it into
    # two f16 terms: the result must not depend on the magnitude or spread of the activations
    rows, cols = 96, 2560
    w, x = weights(11, rows, cols)
    if case == "outliers":
        x[::97] *= 1000.0
    elif case == "zero":
        x[:] = 0.0
    elif case == "tiny":
        x *= 1e-30
    elif case == "huge":
        x *= 1e20
    else:
        x[:] = 0.0
        x[1000] = -3.5
    q = O.quantize_q4_k(w)
    want = O.q4k_matvec(q, x, rows, cols)
    got = be.q4k_matvec(q, x, rows, cols)
    assert got is not None and np.isfinite(got).all()
    if case == "zero":
        assert not got.any()
    else:
        assert rel_l2(got, want) < TOL


def test_q4k_matvec_refusals_follow_the_cpu_backend(be):
    w, x = weights(1, 3, 512)
    q = O.quantize_q4_k(w)
    assert be.q4k_matvec(q, x, 3, 512) is not None
    assert be.q4k_matvec(q, x, 3, 512, out_len=2) is None
    assert be.q4k_matvec(q, x[:511], 3, 512) is None
    assert be.q4k_matvec(q, x[:500], 3, 500) is None
    assert be.q4k_matvec(q[:-1], x, 3, 512) is None
    assert be.q4k_matvec(np.concatenate([q, q]), x, 3, 512) is not None
    z = be.q4k_matvec(np.zeros(0, np.uint8), np.zeros(0, F), 4, 0)
    assert z is not None and z.shape == (4,) and not z.any()
    assert be.q4k_matvec(np.zeros(0, np.uint8), np.zeros(0, F), 0, 0).size == 0


def test_q4k_subnormal_scales_and_extreme_headers(be):
    # tiny weights force f16-subnormal d/dmin; they must not be flushed
    w, x = weights(3, 64, 512, sigma=2e-5)
    q = O.quantize_q4_k(w)
    hdr = q.reshape(-1, 144)[:, :2].copy().view(np.uint16)
    assert (hdr < 0x0400).any(), "fixture should contain subnormal scales"
    want = O.q4k_matvec(q, x, 64, 512)
    assert rel_l2(be.q4k_matvec(q, x, 64, 512), want) < TOL
    # all 6-bit scale/min codes exercised: random header bytes, fixed d/dmin
    rng = np.random.default_rng(4)
    q = rng.integers(0, 256, size=32 * 2 * 144, dtype=np.uint8).reshape(-1, 144)
    q[:, 0:2] = np.array([0x00, 0x2C], np.uint8)   # d = 2^-4
    q[:, 2:4] = np.array([0x00, 0x28], np.uint8)   # dmin = 2^-5
    q = q.reshape(-1)
    want = O.q4k_matvec(q, x, 32, 512)
    assert rel_l2(be.q4k_matvec(q, x, 32, 512), want) < TOL


def test_q4k_dual_and_matmul(be):
    rows, cols, seq = 515, 2560, 5
    a, x = weights(5, rows, cols)
    b, _ = weights(6, rows, cols, 0.05)
    qa, qb = O.quantize_q4_k(a), O.quantize_q4_k(b)
    oa, ob = be.q4k_dual_matvec(qa, qb, x, rows, cols)
    # bit-identical to the single calls (the multi contract of backend/matmul.rs:151-194)
    assert np.array_equal(oa.view(np.uint32), be.q4k_matvec(qa, x, rows, cols).view(np.uint32))
    assert np.array_equal(ob.view(np.uint32), be.q4k_matvec(qb, x, rows, cols).view(np.uint32))
    assert rel_l2(ob, O.q4k_matvec(qb, x, rows, cols)) < TOL
    assert be.q4k_dual_matvec(qa, qb[:-1], x, rows, cols) is None
    X = np.random.default_rng(7).standard_normal((seq, cols)).astype(F)
    out = be.q4k_matmul(qa, X, rows, cols, seq)
    want = O.q4k_matmul(qa, X, rows, cols, seq)
    assert rel_l2(out, want.reshape(-1)) < TOL
    # below 16 positions a row of the product is the matvec of that position, bit for bit
    for s in range(seq):
        assert np.array_equal(out.reshape(seq, rows)[s].view(np.uint32), be.q4k_matvec(qa, X[s], rows, cols).view(np.uint32)), s
    # zero dimensions (kquant_matmul_into, matmul.rs:89-92): no positions / no rows -> an empty result; hidden == 0 with
    # rows and positions -> seq * rows zeros; lengths that do not describe [seq, rows] / [seq, hidden] are refused
    assert be.q4k_matmul(qa, X[:0], rows, cols, 0).size == 0
    assert be.q4k_matmul(qa[:0], X, 0, cols, seq).size == 0
    z = be.q4k_matmul(qa[:0], X[:, :0], rows, 0, seq)
    assert z is not None and z.size == seq * rows and not z.any()
    assert be.q4k_matmul(qa, X, rows, cols, 0) is None          # x brings 5 positions, seq says 0
    # shape error zero-fills like the CPU kernel
    bad = be.q4k_matmul(qa[:-1], X, rows, cols, seq)
    assert bad is not None and not bad.any()


# ------------------------------------------------------------------ Q6_K
@pytest.mark.parametrize("rows,cols", [(2560, 10240), (1031, 2560), (77, 256), (5, 768), (640, 2304), (4100, 512), (1, 5120), (33, 7936),
                                       (19, 12800)])
def test_q6k_matvec_matches_oracle(be, fmt, rows, cols):
    # rows of an odd number of 210-byte super-blocks leave every other row 2 bytes off a dword boundary; 31 super-blocks
    # take 4 columns per wavefront of the matrix-core kernel, 50 are beyond it (K-slice kernel)
    w, x = weights(rows * 3 + cols, rows, cols)
    w[0, :16] *= 1e-4
    q = O.quantize_q6_k(w)
    want = O.q6k_matvec(q, x, rows, cols)
    got = be.q6k_matvec(q, x, rows, cols)
    assert got is not None and got.shape == (rows,)
    assert rel_l2(got, want) < TOL
    assert np.max(np.abs(got - want)) < 1e-3 * (np.abs(want).mean() + 1e-12)
    assert np.array_equal(got.view(np.uint32), be.q6k_matvec(q, x, rows, cols).view(np.uint32))
    assert be.q6k_matvec(q[:-1], x, rows, cols) is None and be.q6k_matvec(q, x[:-1], rows, cols) is None
    assert be.q6k_matvec(np.concatenate([q, q[:7]]), x, rows, cols) is not None
    # the trait's format dispatcher reaches the same kernel
    via = be.quant_matvec(fmt.FMT_Q6_K, q, x, rows, cols)
    assert via is not None and np.array_equal(via.view(np.uint32), got.view(np.uint32))


def test_q6k_matvec_shape_rules(be):
    assert be.q6k_matvec(np.zeros(210, np.uint8), np.zeros(255, F), 1, 255) is None      # hidden % 256
    z = be.q6k_matvec(np.zeros(0, np.uint8), np.zeros(0, F), 3, 0)
    assert z is not None and z.shape == (3,) and not z.any()
    assert be.q6k_matvec(np.zeros(0, np.uint8), np.zeros(256, F), 0, 256).size == 0


# ------------------------------------------------- Q8_K-activation integer path
@pytest.mark.parametrize("n,scale", [(256, 1.0), (2560, 3.0), (10240, 1e-3), (256 * 7, 2e4)])
def test_quantize_x_to_q8k_bit_exact(be, n, scale):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * scale).astype(F)
    x[3] = 0.0
    if n > 512:
        x[256:512] = 0.0                       # an all-zero super-block
    x[n - 1] = F(scale) * 9                    # an outlier
    x[10:16] = np.array([0.5, -0.5, 1.5, -1.5, 2.5, -2.5], F) * (np.abs(x[:256]).max() / F(127.0))   # near half-way cases
    want = O.quantize_x_to_q8k(x)
    got = be.quantize_x_to_q8k(x)
    assert got is not None
    for g, w in zip(got, want):
        assert np.array_equal(g, w)
    assert be.quantize_x_to_q8k(np.zeros(255, F)) is None


@pytest.mark.parametrize("rows,cols", [(3072, 1024), (2048, 2560), (1031, 2560), (77, 10240), (5, 256), (300, 3840), (33, 1792),
                                       (257, 4096), (130, 7168), (1, 2560), (4100, 512), (19, 2816)])
def test_q4k_q8k_matvec_bit_exact(be, rows, cols):
    """Every SIMD kernel of the reference equals q4k_q8k_matvec_scalar bit for bit (dispatch.rs:15-51); so does this one."""
    w, x = weights(rows * 3 + cols, rows, cols)
    q = O.quantize_q4_k(w)
    a = O.quantize_x_to_q8k(x * F(2.5))
    want = O.q4k_q8k_matvec(q, *a, rows, cols)
    got = be.q4k_q8k_matvec(q, *a, rows, cols)
    assert got is not None
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q4k_q8k_matvec_extreme_codes_and_scales(be):
    # all codes at +-127, all nibbles 15, scales and mins 63: the largest integer sums the kernel can meet
    rows, cols = 48, 2560
    nb = cols // 256
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.array([1.0], np.float16).view(np.uint8)
    blk[2:4] = np.array([0.5], np.float16).view(np.uint8)
    blk[4:16] = 0xFF                           # every 6-bit scale and min = 63
    blk[16:] = 0xFF                            # every nibble = 15
    q = np.tile(blk, rows * nb)
    qs = np.where(np.arange(cols) % 3 == 0, -127, 127).astype(np.int8)
    d = np.full(nb, 0.75, F)
    sums = qs.reshape(-1, 32).astype(np.int32).sum(axis=1).astype(np.int16)
    want = O.q4k_q8k_matvec(q, qs, d, sums, rows, cols)
    got = be.q4k_q8k_matvec(q, qs, d, sums, rows, cols)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # sums are an operand (not recomputed from the codes): the min term follows them
    sums2 = (sums // 2).astype(np.int16)
    assert np.array_equal(be.q4k_q8k_matvec(q, qs, d, sums2, rows, cols).view(np.uint32),
                          O.q4k_q8k_matvec(q, qs, d, sums2, rows, cols).view(np.uint32))


def test_q4k_q8k_matvec_shape_rules(be):
    # KernelShapeError::check (cpu/ops/kernel_shape.rs:47-75) as the reference's tests exercise it
    # (fused_and_q6k_paths.rs:53-84, public_execution_path_q4k_q8k_matvec_par.rs:33-78)
    w = O.quantize_q4_k(np.ones(2 * 512, F))
    a = O.quantize_x_to_q8k(np.ones(512, F))
    assert be.q4k_q8k_matvec(w, *a, 2, 512) is not None
    assert be.q4k_q8k_matvec(w[:-1], *a, 2, 512) is None                                   # short weight slab
    assert be.q4k_q8k_matvec(w, *O.quantize_x_to_q8k(np.ones(768, F)), 2, 512) is None      # activation of the wrong length
    assert be.q4k_q8k_matvec(w, *a, 2, 512, out_len=1) is None                             # output shorter than rows
    z = be.q4k_q8k_matvec(np.zeros(0, np.uint8), np.zeros(0, np.int8), np.zeros(0, F), np.zeros(0, np.int16), 3, 0)
    assert z is not None and z.shape == (3,) and not z.any()                               # zero dims give zeros


@pytest.mark.parametrize("rows,cols", [(1, 10496), (70, 15360), (33, 21504), (19, 28672), (5, 40960)])
def test_q4k_q8k_rows_beyond_one_pass_are_served_in_column_ranges(be, rows, cols):
    """Rows longer than 40 super-blocks (the down projections of Gemma-3-12B / 27B and the Llamas: 15360, 21504, 14336,
    28672) are served as column ranges whose partial sums are added in range order: the integer sums are the reference's,
    the f32 accumulation meets in another order than q4k_q8k_matvec_scalar's single chain (1e-6 is asserted where rows of
    up to 10240 elements are bit-exact); gate_up the same, still equal to the single calls bit for bit."""
    w, x = weights(rows + cols, rows, cols)
    q = O.quantize_q4_k(w)
    a = O.quantize_x_to_q8k(x * F(2.5))
    want = O.q4k_q8k_matvec(q, *a, rows, cols)
    got = be.q4k_q8k_matvec(q, *a, rows, cols)
    assert got is not None, be.last_error()
    assert rel_l2(got, want) < 1e-6 and np.max(np.abs(got - want)) < 1e-5 * (np.abs(want).mean() + 1e-9)
    assert np.array_equal(got.view(np.uint32), be.q4k_q8k_matvec(q, *a, rows, cols).view(np.uint32))
    w2, _ = weights(rows + cols + 1, rows, cols)
    q2 = O.quantize_q4_k(w2)
    gu = be.q4k_q8k_gate_up(q, q2, *a, rows, cols)
    assert gu is not None and np.array_equal(gu[0].view(np.uint32), got.view(np.uint32))
    assert np.array_equal(gu[1].view(np.uint32), be.q4k_q8k_matvec(q2, *a, rows, cols).view(np.uint32))


@pytest.mark.parametrize("rows,cols", [(48, 15360), (130, 32768), (3, 33024), (7, 65536), (20, 102400)])
def test_q4k_rows_of_any_length_are_served(be, fmt, rows, cols):
    """The f32-activation matvec over long rows: up to 32768 elements the K-slice kernel, beyond that column ranges on the
    matrix-core kernel with the partial sums added in range order — host tier and device tier (one job, and next to a
    short-row job in one call)."""
    w, x = weights(rows * 5 + cols, rows, cols)
    q = O.quantize_q4_k(w)
    want = O.q4k_matvec(q, x, rows, cols)
    got = be.q4k_matvec(q, x, rows, cols)
    assert got is not None, be.last_error()
    assert rel_l2(got, want) < TOL and np.max(np.abs(got - want)) < 1e-3 * (np.abs(want).mean() + 1e-12)
    dw, dx, do, do2 = be.to_device(q), be.to_device(x), be.malloc(rows * 4), be.malloc(64 * 4)
    w3, _ = weights(9, 64, 512)
    q3 = O.quantize_q4_k(w3)
    dw3 = be.to_device(q3)
    assert be.dev_matvec_batch([(fmt.FMT_Q4_K, dw, 0, dx, do, rows, cols), (fmt.FMT_Q4_K, dw3, 0, dx, do2, 64, 512)])
    be.synchronize()
    assert np.array_equal(be.d2h(do, rows, F).view(np.uint32), got.view(np.uint32))
    assert rel_l2(be.d2h(do2, 64, F), O.q4k_matvec(q3, x[:512], 64, 512)) < TOL


def test_q4k_q8k_device_tier_plan_matches_host_tier(be, fmt):
    # activation quantised on the device into its device layout, several matvecs in one plan
    rng = np.random.default_rng(97)
    shapes = [(640, 2560), (96, 2560), (200, 10240), (31, 1024)]
    x = {k: rng.standard_normal(k).astype(F) for k in (2560, 10240, 1024)}
    dq = {}
    for k, xv in x.items():
        dx, buf = be.to_device(xv), be.malloc(be.q8k_bytes(k) + 64)
        assert be.dev_quantize_x_to_q8k(dx, k, buf)
        dq[k] = buf
    jobs, outs, wants = [], [], []
    for rows, k in shapes:
        q = O.quantize_q4_k((rng.standard_normal(rows * k) * 0.03).astype(F))
        o = be.malloc(rows * 4)
        jobs.append((fmt.FMT_Q4_K_Q8K, be.to_device(q), None, dq[k], o, rows, k))
        outs.append((o, rows))
        wants.append(O.q4k_q8k_matvec(q, *O.quantize_x_to_q8k(x[k]), rows, k))
    plan = be.plan_create(jobs)
    assert plan is not None and be.plan_launch_count(plan) == 1
    assert be.plan_run(plan) and be.plan_run(plan)
    be.synchronize()
    for (o, rows), want in zip(outs, wants):
        assert np.array_equal(be.d2h(o, rows, F).view(np.uint32), want.view(np.uint32))
    be.plan_destroy(plan)


@pytest.mark.parametrize("rows,cols", [(2560, 10240), (1031, 2560), (262, 4096), (5, 512), (1, 256), (77, 7168), (4100, 768),
                                       (33, 1792), (300, 3840), (19, 16384)])
def test_q6k_q8k_matvec_bit_exact(be, rows, cols):
    """q6k_q8k_matvec_scalar (q6k.rs:38-92): integer group dots, d_w*d_y*(f32)sum1 added in super-block order."""
    w, x = weights(rows * 5 + cols, rows, cols)
    q = O.quantize_q6_k(w)
    qs, d, _ = O.quantize_x_to_q8k(x * F(1.75))
    want = O.q6k_q8k_matvec(q, qs, d, rows, cols)
    got = be.q6k_q8k_matvec(q, qs, d, rows, cols)
    assert got is not None
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q6k_q8k_matvec_extreme_codes_and_scales(be):
    # codes 63 and 0 (q - 32 = +31 / -32), scales +127 / -128, activation codes +-127: the widest integer sums
    rows, cols = 24, 1536
    nb = cols // 256
    rng = np.random.default_rng(5)
    blocks = np.zeros((rows * nb, 210), np.uint8)
    blocks[:, 0:192] = np.where(rng.random((rows * nb, 1)) < 0.5, 0xFF, 0x00).astype(np.uint8)
    blocks[:, 192:208] = np.where(rng.random((rows * nb, 16)) < 0.5, 127, 128).astype(np.uint8)   # int8 +127 / -128
    blocks[:, 208:210] = np.array([0.25], np.float16).view(np.uint8)
    q = blocks.reshape(-1)
    qs = np.where(rng.random(cols) < 0.5, -127, 127).astype(np.int8)
    d = np.full(nb, 1.5, F)
    want = O.q6k_q8k_matvec(q, qs, d, rows, cols)
    got = be.q6k_q8k_matvec(q, qs, d, rows, cols)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    qs[:] = 127                                           # every product of one sign within a group
    assert np.array_equal(be.q6k_q8k_matvec(q, qs, d, rows, cols).view(np.uint32),
                          O.q6k_q8k_matvec(q, qs, d, rows, cols).view(np.uint32))


def test_q6k_q8k_matvec_shape_rules(be):
    # q6k_q8k_zero_dims_are_empty_and_short_weights_are_refused (fused_and_q6k_paths.rs:137-166)
    w = O.quantize_q6_k(np.ones(2 * 512, F))
    qs, d, _ = O.quantize_x_to_q8k(np.ones(512, F))
    assert be.q6k_q8k_matvec(w, qs, d, 2, 512) is not None
    assert be.q6k_q8k_matvec(w[:-1], qs, d, 2, 512) is None                   # short weight slab
    q3, d3, _ = O.quantize_x_to_q8k(np.ones(768, F))
    assert be.q6k_q8k_matvec(w, q3, d3, 2, 512) is None                       # activation of the wrong length
    assert be.q6k_q8k_matvec(w, qs, d, 2, 512, out_len=3) is None             # output length != rows
    z = be.q6k_q8k_matvec(np.zeros(0, np.uint8), np.zeros(0, np.int8), np.zeros(0, F), 3, 0)
    assert z is not None and z.shape == (3,) and not z.any()


def test_q4k_q8k_gate_up_equals_two_matvecs_bit_for_bit(be):
    # q8k_gate_up_fused_matches_separate_matvecs (fused_and_q6k_paths.rs:7-50) at a decode shape and a ragged one
    for rows, cols, seed in ((10240, 2560, 3), (37, 768, 4)):
        rng = np.random.default_rng(seed)
        gw = O.quantize_q4_k((rng.standard_normal(rows * cols) * 0.03).astype(F))
        uw = O.quantize_q4_k((rng.standard_normal(rows * cols) * 0.03).astype(F))
        a = O.quantize_x_to_q8k(rng.standard_normal(cols).astype(F))
        got = be.q4k_q8k_gate_up(gw, uw, *a, rows, cols)
        assert got is not None
        assert np.array_equal(got[0].view(np.uint32), O.q4k_q8k_matvec(gw, *a, rows, cols).view(np.uint32))
        assert np.array_equal(got[1].view(np.uint32), O.q4k_q8k_matvec(uw, *a, rows, cols).view(np.uint32))
    # a short gate or up slab refuses the pair (fused_and_q6k_paths.rs:296-337); zero dims give zeros
    a = O.quantize_x_to_q8k(np.full(256, 0.5, F))
    full, short = np.zeros(2 * 144, np.uint8), np.zeros(144, np.uint8)
    assert be.q4k_q8k_gate_up(short, full, *a, 2, 256) is None
    assert be.q4k_q8k_gate_up(full, short, *a, 2, 256) is None
    assert be.q4k_q8k_gate_up(full, full, *a, 2, 256) is not None
    z = be.q4k_q8k_gate_up(np.zeros(0, np.uint8), np.zeros(0, np.uint8), np.zeros(0, np.int8), np.zeros(0, F), np.zeros(0, np.int16), 4, 0)
    assert z is not None and not z[0].any() and not z[1].any() and z[0].shape == (4,)


def test_q4k_q8k_gemm_rows_equal_the_row_at_a_time_matvec(be):
    # gemm_is_bit_identical_to_row_at_a_time_matvec (gemm.rs:141-170), on the reference's own inputs and a larger case
    rows, cols, seq = 96, 512, 7
    w = O.quantize_q4_k(np.array([((i * 31 + 7) % 23) * 0.01 - 0.11 for i in range(rows * cols)], F))
    xs = [np.array([((s * 13 + c * 3) % 19) * 0.01 - 0.09 for c in range(cols)], F) for s in range(seq)]
    acts = [O.quantize_x_to_q8k(x) for x in xs]
    got = be.q4k_q8k_gemm(w, acts, rows, cols)
    assert got is not None and got.shape == (seq, rows)
    for s in range(seq):
        assert np.array_equal(got[s].view(np.uint32), O.q4k_q8k_matvec(w, *acts[s], rows, cols).view(np.uint32))
    rng = np.random.default_rng(11)
    rows, cols, seq = 1031, 2560, 33
    w = O.quantize_q4_k((rng.standard_normal(rows * cols) * 0.03).astype(F))
    acts = [O.quantize_x_to_q8k(rng.standard_normal(cols).astype(F)) for _ in range(seq)]
    got = be.q4k_q8k_gemm(w, acts, rows, cols)
    for s in (0, 16, 32):
        assert np.array_equal(got[s].view(np.uint32), O.q4k_q8k_matvec(w, *acts[s], rows, cols).view(np.uint32))
    assert be.q4k_q8k_gemm(w[:-1], acts, rows, cols) is None            # short slab
    assert be.q4k_q8k_gemm(w, [], rows, cols).shape == (0, rows)        # no activation rows: nothing to do


def test_q6k_q8k_and_q4k_q8k_jobs_share_one_activation_in_a_plan(be, fmt):
    # the reference's decode mixes Q4_K and Q6_K tensors against one quantised activation (q4k_q8k_matvec_parallel's format switch)
    rng = np.random.default_rng(98)
    k = 2560
    xv = rng.standard_normal(k).astype(F)
    buf = be.malloc(be.q8k_bytes(k) + 64)
    assert be.dev_quantize_x_to_q8k(be.to_device(xv), k, buf)
    a = O.quantize_x_to_q8k(xv)
    jobs, outs, wants = [], [], []
    for f, rows in ((fmt.FMT_Q6_K_Q8K, 513), (fmt.FMT_Q4_K_Q8K, 640), (fmt.FMT_Q6_K_Q8K, 40)):
        wf = (rng.standard_normal(rows * k) * 0.05).astype(F)
        q = O.quantize_q6_k(wf) if f == fmt.FMT_Q6_K_Q8K else O.quantize_q4_k(wf)
        o = be.malloc(rows * 4)
        jobs.append((f, be.to_device(q), None, buf, o, rows, k))
        outs.append((o, rows))
        wants.append(O.q6k_q8k_matvec(q, a[0], a[1], rows, k) if f == fmt.FMT_Q6_K_Q8K else O.q4k_q8k_matvec(q, *a, rows, k))
    plan = be.plan_create(jobs)
    assert plan is not None and be.plan_launch_count(plan) == 2
    assert be.plan_run(plan) and be.plan_run(plan)
    be.synchronize()
    for (o, rows), want in zip(outs, wants):
        assert np.array_equal(be.d2h(o, rows, F).view(np.uint32), want.view(np.uint32))
    be.plan_destroy(plan)


# ------------------------------------------------------------------ Q8_0
@pytest.mark.parametrize("n,k", [(4099, 2560), (64, 10240), (9, 128), (1000, 2048), (17, 256), (333, 1792), (48, 2816),
                                 (531, 3840), (2050, 4096), (77, 5120), (40, 5376)])   # two column passes per wavefront; odd column count; just above
def test_q8_0_gemv_matches_oracle(be, n, k):
    w, x = weights(n + k, n, k)
    w[0, :32] *= 1e-5
    q = O.quantize_q8_0(w)
    want = O.q8_0_gemv(q, x, n, k)
    got = be.q8_0_gemv(q, x, n, k)
    assert rel_l2(got, want) < TOL
    assert np.max(np.abs(got - want)) < 1e-3 * (np.abs(want).mean() + 1e-12)
    assert be.q8_0_gemv(q[:-1], x, n, k) is None and be.q8_0_gemv(q, x[:-1], n, k) is None
    assert be.q8_0_gemv(np.concatenate([q, q[:2]]), x, n, k) is None


@pytest.mark.parametrize("n,k", [(1, 32), (3, 32), (7, 96), (1001, 160), (64, 2592), (33, 4128), (5, 16352)])
def test_q8_0_and_q4_0_rows_with_an_odd_number_of_blocks(be, fmt, n, k):
    """K % 32 == 0 is all the reference asks (kquant_gemv.rs:67-90, q4_matvec.rs:24-86).  With an odd block count every
    other row starts 2 bytes off a dword boundary, and an odd total leaves the last block half a dword short of one:
    each block carries its own magnitude so that a scale or code taken from a neighbour shows."""
    rng = np.random.default_rng(k * 7 + n)
    w = (rng.standard_normal((n, k // 32, 32)) * 0.02).astype(F)
    w *= np.exp2(rng.integers(-5, 6, size=(n, k // 32, 1))).astype(F)
    w = w.reshape(-1)
    x = rng.standard_normal(k).astype(F)
    q8w = O.quantize_q8_0(w)
    assert rel_l2(be.q8_0_gemv(q8w, x, n, k), O.q8_0_gemv(q8w, x, n, k)) < TOL
    q4 = O.quantize_q4_0(w)
    q8, sc = O.quantize_to_q8(x)
    want = O.q4_0_matvec(q4, q8, sc, n, k)
    assert rel_l2(be.q4_matvec(q4, q8, sc, n, k), want) < TOL
    assert rel_l2(be.quant_matvec(fmt.FMT_Q4_0, q4, x, n, k), want) < TOL
    hits = be.gate_knn(fmt.FMT_Q4_0, q4, x, n, k, 5)
    assert [i for i, _ in hits] == [i for i, _ in O.top_k_by_abs(want, 5)]
    if n >= 64:
        top = be.q8_0_gemv_topk(q8w, x, n, k, 9)
        assert [i for i, _ in top] == [i for i, _ in O.top_k_sorted(O.q8_0_gemv(q8w, x, n, k), 9)]


# ----------------------------------------------------------------- MXFP4
def test_mxfp4_gemv_matches_dequant_reference(be):
    # the Metal peer's recipe: cos > 0.999999 and rel < 1e-4 vs dequantize_expert, sentinels, ragged rows
    n, k = 2880 + 3, 2880
    w, x = weights(11, n, k)
    p, s = O.quantize_mxfp4(w, n, k)
    want = O.mxfp4_gemv(p, s, x, n, k)
    got = be.mxfp4_gemv(p, s, x, n, k)
    assert rel_l2(got, want) < TOL and rel_l2(got, O.mxfp4_gemv_dequant(p, s, x, n, k)) < TOL
    s2 = s.copy(); s2[0] = 0; s2[90] = 255
    got2 = be.mxfp4_gemv(p, s2, x, n, k)
    want2 = O.mxfp4_gemv(p, s2, x, n, k)
    assert np.isnan(got2[1]) and np.isnan(want2[1])
    ok = np.ones(n, bool); ok[1] = False
    assert rel_l2(got2[ok], want2[ok]) < TOL
    assert be.mxfp4_gemv(p, s, x[:-1], n, k) is None
    assert be.mxfp4_gemv(p[:-1], s, x, n, k) is None
    assert be.mxfp4_gemv(p, s, x, n, 2881) is None
    # multi: argument order, bit-identical to the single calls, empty batch is Some([])
    outs = be.mxfp4_gemv_multi([(p, s, n, k), (p, s2, n, k), (p[: 7 * 90 * 16], s[: 7 * 90], 7, k)], x)
    assert np.array_equal(outs[0].view(np.uint32), got.view(np.uint32))
    assert np.array_equal(outs[1].view(np.uint32), got2.view(np.uint32)) and outs[2].shape == (7,)
    assert be.mxfp4_gemv_multi([], x) == []
    assert be.mxfp4_gemv_multi([(p, s, n, k), (p[:-1], s, n, k)], x) is None


@pytest.mark.parametrize("n,k", [(33, 128), (50, 160), (19, 224), (70, 384), (40, 992), (37, 4096), (21, 5120), (16, 96)])
def test_mxfp4_gemv_row_lengths_and_block_scales(be, n, k):
    """Rows of 3 to 160 blocks (odd block counts put a row's scale bytes at odd addresses; partial last steps; k = 96 is
    below what the matrix-core kernel takes), every block with its own power-of-two magnitude so that a scale byte
    taken from the wrong block or row shows."""
    rng = np.random.default_rng(1000 + k)
    w = (rng.standard_normal((n, k // 32, 32)) * 0.02).astype(F)
    w *= np.exp2(rng.integers(-6, 7, size=(n, k // 32, 1))).astype(F)
    w = w.reshape(-1)
    x = rng.standard_normal(k).astype(F)
    p, s = O.quantize_mxfp4(w, n, k)
    assert len(set(s.tolist())) >= 8
    assert rel_l2(be.mxfp4_gemv(p, s, x, n, k), O.mxfp4_gemv(p, s, x, n, k)) < TOL


# ---------------------------------------------------------- dense + Q4_0
def test_dense_gemvs(be):
    n, k = 1000, 2560
    w, x = weights(13, n, k)
    wb = O.f32_to_bf16(w)
    assert rel_l2(be.bf16_gemv_force(wb, x, n, k), O.bf16_gemv(wb, x, n, k)) < TOL
    wh = w.astype(np.float16).view(np.uint16)
    assert rel_l2(be.f16_gemv_force(wh, x, n, k), O.f16_gemv(wh, x, n, k)) < TOL
    assert rel_l2(be.f32_gemv_force(w, x), O.f32_gemv(w, x, n, k)) < TOL
    # below the flop threshold the non-force variants answer None (2*n*k < 5e8)
    assert be.f32_gemv(w, x) is None and be.bf16_gemv(wb, x, n, k) is None
    assert be.f16_gemv_force(wh[:-1], x, n, k) is None and be.f16_gemv_force(wh, x[:-1], n, k) is None


def test_q4_0_q8_matvec_and_quant_matvec_dispatch(be, fmt):
    rows, hidden = 1027, 2560
    w, x = weights(17, rows, hidden)
    q4 = O.quantize_q4_0(w)
    q8, sc = O.quantize_to_q8(x)
    want = O.q4_0_matvec(q4, q8, sc, rows, hidden)
    got = be.q4_matvec(q4, q8, sc, rows, hidden)
    assert rel_l2(got, want) < TOL
    assert be.q4_matvec(q4[:-1], q8, sc, rows, hidden) is None
    # QuantMatVec::quant_matvec: Q4_0 quantises x on the way in; Q4_K is the f32 path
    got2 = be.quant_matvec(fmt.FMT_Q4_0, q4, x, rows, hidden)
    assert rel_l2(got2, want) < TOL
    qk = O.quantize_q4_k(w)
    assert rel_l2(be.quant_matvec(fmt.FMT_Q4_K, qk, x, rows, hidden), O.q4k_matvec(qk, x, rows, hidden)) < TOL
    # Q6_K is routed to q6k_matvec (quant_matvec.rs:66-68)
    q6 = O.quantize_q6_k(w)
    assert rel_l2(be.quant_matvec(fmt.FMT_Q6_K, q6, x, rows, hidden), O.q6k_matvec(q6, x, rows, hidden)) < TOL
    assert be.quant_matvec(fmt.FMT_Q6_K, qk, x, rows, hidden) is None      # Q4_K bytes are too short for Q6_K rows: refused
    # the trait's own Q8_0 layout, Q5_K, MXFP4 (external scales), the float formats and I2S answer None through this signature
    for f in (fmt.FMT_Q8_0, fmt.FMT_Q5_K, fmt.FMT_MXFP4, fmt.FMT_BF16, fmt.FMT_F16, fmt.FMT_F32, fmt.FMT_I2S):
        for bytes_ in (qk, q6, w):
            assert be.quant_matvec(f, bytes_, x, rows, hidden) is None


# ------------------------------------------------------------------ gate-KNN
def check_hits(got, scores, k):
    """Same index set as top_k_by_abs up to ties within 1e-5, scores right, sorted by |score|."""
    want = O.top_k_by_abs(scores, k)
    assert len(got) == len(want)
    gi, wi = {i for i, _ in got}, {i for i, _ in want}
    if gi != wi:
        kth = abs(want[-1][1])
        for i in gi ^ wi:
            assert abs(abs(float(scores[i])) - kth) <= 1e-5 * max(1.0, kth), (i, scores[i], kth)
    mags = [abs(v) for _, v in got]
    assert all(mags[i] >= mags[i + 1] for i in range(len(mags) - 1))
    for i, v in got:
        assert abs(v - float(scores[i])) <= 1e-5 * max(1.0, abs(v))


@pytest.mark.parametrize("variant", ["bf16", "q4k", "f32", "f16", "q4_0"])
@pytest.mark.parametrize("batch", [1, 8])
def test_gate_knn_matches_oracle(be, fmt, variant, batch):
    n, hidden, k = 10240, 2560, 64
    rng = np.random.default_rng(23)
    g = (rng.standard_normal((n, hidden)) * 0.02).astype(F)
    X = rng.standard_normal((batch, hidden)).astype(F)
    if variant == "bf16":
        gate, f = O.f32_to_bf16(g), fmt.FMT_BF16
        ref = [O.bf16_gemv(gate, X[b], n, hidden) for b in range(batch)]
    elif variant == "f16":
        gate, f = g.astype(np.float16).view(np.uint16), fmt.FMT_F16
        ref = [O.f16_gemv(gate, X[b], n, hidden) for b in range(batch)]
    elif variant == "f32":
        gate, f = g, fmt.FMT_F32
        ref = [O.f32_gemv(g, X[b], n, hidden) for b in range(batch)]
    elif variant == "q4k":
        gate, f = O.quantize_q4_k(g), fmt.FMT_Q4_K
        ref = [O.q4k_matvec(gate, X[b], n, hidden) for b in range(batch)]
    else:
        gate, f = O.quantize_q4_0(g), fmt.FMT_Q4_0
        ref = [O.q4_0_matvec(gate, *O.quantize_to_q8(X[b]), n, hidden) for b in range(batch)]
    hits = be.gate_knn_batch_hits(f, gate, X, n, hidden, k)
    assert len(hits) == batch
    for b in range(batch):
        check_hits(hits[b], ref[b], k)
    scores = be.gate_scores_batch(f, gate, X, n, hidden)
    assert rel_l2(scores, np.stack(ref)) < TOL
    union = be.gate_knn_batch(f, gate, X, n, hidden, k)
    want_union = O.gate_knn_batch_union(np.stack(ref).T.copy(), k)
    assert len(set(union) ^ set(want_union)) <= 2 * batch   # only tie-level differences at the k-th score
    assert union == sorted(set(union))


@pytest.mark.parametrize("n,hidden,batch", [(1000, 128, 2), (77, 384, 3), (4099, 2560, 5), (640, 1280, 9), (33, 2560, 17),
                                            (500, 2688, 4), (500, 208, 3)])
def test_bf16_gate_scores_over_several_positions(be, fmt, n, hidden, batch):
    # several positions share one pass over a bf16 gate (up to 8 at a time where the row length allows);
    # every position's scores must equal the single-position result, whatever the grouping
    rng = np.random.default_rng(n + hidden + batch)
    gate = O.f32_to_bf16((rng.standard_normal((n, hidden)) * 0.05).astype(F))
    X = rng.standard_normal((batch, hidden)).astype(F)
    X[0, ::7] *= 300.0           # spread of magnitudes inside a position
    X[-1] *= 1e-12               # and between positions
    scores = be.gate_scores_batch(fmt.FMT_BF16, gate, X, n, hidden)
    assert scores.shape == (batch, n)
    for b in range(batch):
        want = O.bf16_gemv(gate, X[b], n, hidden)
        assert rel_l2(scores[b], want) < TOL, b
        single = be.gate_scores_batch(fmt.FMT_BF16, gate, X[b:b + 1], n, hidden)[0]
        assert rel_l2(scores[b], single) < TOL


@pytest.mark.parametrize("n,hidden,batch", [(1000, 256, 2), (77, 768, 3), (4099, 2560, 4), (640, 1280, 9), (33, 2560, 6),
                                            (500, 2816, 4), (2051, 2560, 8), (130, 512, 7), (300, 2304, 17), (64, 256, 5)])
def test_q4k_gate_scores_over_several_positions(be, fmt, n, hidden, batch):
    # up to 8 positions share one pass over a Q4_K gate (rows of up to 10 super-blocks; longer rows go one by one)
    rng = np.random.default_rng(n + hidden + batch)
    gate = O.quantize_q4_k((rng.standard_normal((n, hidden)) * 0.05).astype(F))
    X = rng.standard_normal((batch, hidden)).astype(F)
    X[0, ::7] *= 300.0
    X[-1] *= 1e-12
    scores = be.gate_scores_batch(fmt.FMT_Q4_K, gate, X, n, hidden)
    assert scores.shape == (batch, n)
    for b in range(batch):
        want = O.q4k_matvec(gate, X[b], n, hidden)
        assert rel_l2(scores[b], want) < TOL, b
        single = be.gate_scores_batch(fmt.FMT_Q4_K, gate, X[b:b + 1], n, hidden)[0]
        assert rel_l2(scores[b], single) < TOL


def test_gate_knn_edge_cases(be, fmt):
    rng = np.random.default_rng(29)
    n, hidden = 100, 256
    g = (rng.standard_normal((n, hidden)) * 0.02).astype(F)
    x = rng.standard_normal(hidden).astype(F)
    s = O.f32_gemv(g, x, n, hidden)
    check_hits(be.gate_knn(fmt.FMT_F32, g, x, n, hidden, 64), s, 64)
    hits = be.gate_knn(fmt.FMT_F32, g[:10], x, 10, hidden, 64)   # K > N -> all N
    assert len(hits) == 10
    assert be.gate_knn(fmt.FMT_F32, g, x, n, hidden, 0) == []     # K == 0 -> empty
    assert len(be.gate_knn(fmt.FMT_F32, g, x, n, hidden, 65)) == 65  # above 64: served (ordered in LDS)
    assert be.gate_knn(fmt.FMT_F32, g, x, n, hidden, 16385) is None  # beyond the kernel's capacity: refused
    xn = x.copy(); xn[3] = np.nan
    import larql_amd
    with pytest.raises(larql_amd.NanScoreError):
        be.gate_knn(fmt.FMT_F32, g, xn, n, hidden, 8)
    # reference closed forms (gate_knn/mod.rs:231-287) through one-hot gates: scores == x
    eye = np.eye(256, dtype=F)[:4]
    xv = np.zeros(256, F); xv[:4] = [0.1, -0.9, 0.5, 0.3]
    hits = be.gate_knn(fmt.FMT_F32, eye, xv, 4, 256, 2)
    assert [i for i, _ in hits] == [1, 2] and abs(hits[0][1] + 0.9) < 1e-6
    # exact ties: lower index first
    xt = np.zeros(256, F); xt[:4] = [1.0, -1.0, 1.0, 0.5]
    assert [i for i, _ in be.gate_knn(fmt.FMT_F32, eye, xt, 4, 256, 2)] == [0, 1]


@pytest.mark.parametrize("case", ["normal", "sorted", "constant", "coarse", "tie_block", "max_cached", "streamed", "ragged",
                                  "few_candidates", "many_candidates"])
def test_top_k_selection_paths(be, fmt, case):
    # top_k_by_abs on prescribed score rows (scores = gate[:, 0] through a unit residual), over the selection paths
    # of the kernel: candidates ranked directly, the radix passes (sorted / constant rows have too many candidates),
    # rows streamed from memory.  Ties go to the lower index, so the expected list is unique.
    rng = np.random.default_rng(len(case))
    n, k = 10240, 64
    if case == "normal":
        sc = rng.standard_normal(n)
    elif case == "sorted":
        sc = np.linspace(3.0, -3.0, n)
    elif case == "constant":
        sc = np.full(n, -0.75)
    elif case == "coarse":
        sc = np.round(rng.standard_normal(n) * 2) / 2            # many exact ties everywhere
    elif case == "tie_block":
        sc = rng.standard_normal(n) * 0.1
        sc[rng.choice(n, 100, replace=False)] = 5.0              # 100 equal scores straddle the K boundary
        sc[rng.choice(n, 20, replace=False)] = -7.0
    elif case == "few_candidates":
        # exactly 64 scores stand out, one in each of the 64 slices of the row (a slice = wavefront w, 16 lanes g of it:
        # indices 640 w + 64 it + 16 g + j): the candidate list is as short as it gets, every thread counts a 16th of it
        sc = rng.uniform(-1.0, 1.0, n)
        for w in range(16):
            for g in range(4):
                sc[640 * w + 64 * int(rng.integers(10)) + 16 * g + int(rng.integers(16))] = 10.0 + rng.uniform(0.0, 1.0) * (1 if (w + g) % 2 else -1)
    elif case == "many_candidates":
        # one slice stays below 0.93, the rest is uniform on (0, 1): ~700 candidates, a list that is not split into shares
        sc = rng.uniform(0.0, 1.0, n) * rng.choice([-1.0, 1.0], n)
        sl = np.array([640 * 5 + 64 * it + 16 * 2 + j for it in range(10) for j in range(16)])
        sc[sl] *= 0.93
    elif case == "max_cached":
        n = 16384; sc = rng.standard_normal(n)
    elif case == "streamed":
        n = 16385; sc = rng.standard_normal(n)
    else:
        n = 1000; k = 7; sc = rng.standard_normal(n)
    sc = sc.astype(F)
    hidden = 32
    gate = np.zeros((n, hidden), F); gate[:, 0] = sc
    x = np.zeros(hidden, F); x[0] = 1.0
    hits = be.gate_knn(fmt.FMT_F32, gate, x, n, hidden, k)
    order = np.lexsort((np.arange(n), -np.abs(sc)))[:k]
    assert [i for i, _ in hits] == order.tolist()
    assert [v for _, v in hits] == sc[order].tolist()


def test_q4k_matvec_topk_by_value(be):
    rows, cols = 5000, 512
    w, x = weights(31, rows, cols)
    q = O.quantize_q4_k(w)
    scores = O.q4k_matvec(q, x, rows, cols)
    for k in (1, 5, 8, 64):
        got = be.q4k_matvec_topk(q, x, rows, cols, k)
        want = O.top_k_sorted(scores, k)
        assert [i for i, _ in got] == [i for i, _ in want]
    assert be.q4k_matvec_topk(q, x, rows, cols, 0) is None
    assert len(be.q4k_matvec_topk(q, x, rows, cols, 65)) == 65 and be.q4k_matvec_topk(q, x, rows, cols, 16385) is None
    assert be.q4k_matvec_topk(q, x[:-1], rows, cols, 4) is None


# ------------------------------------------------------------- residency
def test_registered_region_serves_sub_slices(be):
    rows, cols = 256, 1024
    w1, x = weights(37, rows, cols)
    w2, _ = weights(38, rows, cols)
    blob = np.concatenate([O.quantize_q4_k(w1), O.quantize_q4_k(w2)])
    be.register_weight_region(blob)
    be.register_weight_region(blob)        # same base twice: no-op
    be.seal_weight_regions()
    half = blob.size // 2
    before = be.submission_clock()
    a = be.q4k_matvec(blob[:half], x, rows, cols)
    b = be.q4k_matvec(blob[half:], x, rows, cols)
    after = be.submission_clock()
    assert rel_l2(a, O.q4k_matvec(blob[:half], x, rows, cols)) < TOL
    assert rel_l2(b, O.q4k_matvec(blob[half:], x, rows, cols)) < TOL
    assert after["submissions"] == before["submissions"] + 2 and after["gpu_nanos"] > before["gpu_nanos"]
    be.clear_weight_regions()
    assert rel_l2(be.q4k_matvec(blob[:half], x, rows, cols), a) == 0


# ---------------------------------------------------------------- encoders
def test_device_encoders_are_bit_exact(be):
    rng = np.random.default_rng(41)
    n = 256 * 4096
    w = (rng.standard_normal(n) * 0.02).astype(F)
    w[:256] = 0; w[256:512] = np.abs(w[256:512]); w[512:768] = -np.abs(w[512:768]); w[768:800] = 1e-7
    w[1024:1056] = np.nextafter(F(0.0625), F(0))       # log2 edge just below a power of two
    src = be.to_device(w)
    dst = be.malloc(n * 2)
    assert be.dev_quantize_q4_k(src, n, dst)
    assert np.array_equal(be.d2h(dst, n // 256 * 144, np.uint8), O.quantize_q4_k(w))
    assert be.dev_quantize_q8_0(src, n, dst)
    assert np.array_equal(be.d2h(dst, n // 32 * 34, np.uint8), O.quantize_q8_0(w))
    assert be.dev_quantize_q4_0(src, n, dst)
    assert np.array_equal(be.d2h(dst, n // 32 * 18, np.uint8), O.quantize_q4_0(w))
    assert be.dev_f32_to_bf16(src, n, dst)
    assert np.array_equal(be.d2h(dst, n, np.uint16), O.f32_to_bf16(w))
    sc = be.malloc(n // 32 * 4)
    assert be.dev_quantize_to_q8(src, n, dst, sc)
    q8, s8 = O.quantize_to_q8(w)
    assert np.array_equal(be.d2h(dst, n, np.int8), q8) and np.array_equal(be.d2h(sc, n // 32, F).view(np.uint32), s8.view(np.uint32))
    k = 2880
    rows = n // k
    assert be.dev_quantize_mxfp4(src, rows, k, dst, sc)
    p, s = O.quantize_mxfp4(w[: rows * k], rows, k)
    assert np.array_equal(be.d2h(sc, rows * 90, np.uint8), s)
    assert np.array_equal(be.d2h(dst, rows * 90 * 16, np.uint8), p)
    for ptr in (src, dst, sc):
        be.free(ptr)


def test_fill_normal_statistics(be):
    n = 1 << 20
    d = be.malloc(n * 4)
    assert be.dev_fill_normal(d, n, 1234, 0.02)
    a = be.d2h(d, n, F)
    assert be.dev_fill_normal(d, n, 1234, 0.02)
    assert np.array_equal(a, be.d2h(d, n, F))                      # a pure function of (seed, index)
    assert be.dev_fill_normal(d, n, 1235, 0.02)
    assert not np.array_equal(a, be.d2h(d, n, F))
    assert abs(a.mean()) < 1e-4 and abs(a.std() - 0.02) < 2e-4
    assert abs(np.mean(np.abs(a) > 0.04) - 0.0455) < 0.003         # two-sigma tail mass of a normal
    be.free(d)


# ------------------------------------------------------------ device tier
def test_dev_matvec_batch_mixed_formats(be, fmt):
    rng = np.random.default_rng(43)
    jobs, wants, outs = [], [], []
    x_h = rng.standard_normal(10240).astype(F)
    x = be.to_device(x_h)
    specs = [("q4k", 300, 2560), ("q4k", 70, 10240), ("q8", 500, 2560), ("q4k", 129, 2048), ("bf16", 100, 2560),
             ("q4k", 40, 2560), ("q8", 3, 2560)]
    for kind, rows, k in specs:
        w = (rng.standard_normal((rows, k)) * 0.02).astype(F)
        if kind == "q4k":
            q = O.quantize_q4_k(w); f = fmt.FMT_Q4_K; want = O.q4k_matvec(q, x_h[:k], rows, k)
        elif kind == "q8":
            q = O.quantize_q8_0(w); f = fmt.FMT_GGML_Q8_0; want = O.q8_0_gemv(q, x_h[:k], rows, k)
        else:
            q = O.f32_to_bf16(w); f = fmt.FMT_BF16; want = O.bf16_gemv(q, x_h[:k], rows, k)
        dw = be.to_device(q)
        do = be.malloc(rows * 4)
        jobs.append((f, dw, None, x, do, rows, k)); wants.append(want); outs.append((do, rows))
    assert be.dev_matvec_batch(jobs)
    be.synchronize()
    for (do, rows), want in zip(outs, wants):
        assert rel_l2(be.d2h(do, rows, F), want) < TOL
    # and one at a time gives the same bits
    f, dw, _, _, do, rows, k = jobs[1]
    first = be.d2h(do, rows, F)
    assert be.dev_matvec(f, dw, None, x, rows, k, do)
    be.synchronize()
    assert np.array_equal(first.view(np.uint32), be.d2h(do, rows, F).view(np.uint32))


def test_recorded_plan_replays_and_matches_direct_launches(be, fmt):
    rng = np.random.default_rng(47)
    x_h = rng.standard_normal(2560).astype(F)
    x = be.to_device(x_h)
    jobs, wants = [], []
    for i, (rows, kind) in enumerate([(300, "q4k"), (64, "q4k"), (500, "q8"), (1000, "q4k"), (17, "q4k"), (9, "q4k")]):
        w = (rng.standard_normal((rows, 2560)) * 0.02).astype(F)
        if kind == "q4k":
            q, f, want = O.quantize_q4_k(w), fmt.FMT_Q4_K, None
            want = O.q4k_matvec(q, x_h, rows, 2560)
        else:
            q, f = O.quantize_q8_0(w), fmt.FMT_GGML_Q8_0
            want = O.q8_0_gemv(q, x_h, rows, 2560)
        jobs.append((f, be.to_device(q), None, x, be.malloc(rows * 4), rows, 2560)); wants.append(want)
    plan = be.plan_create(jobs)
    assert plan and be.plan_launch_count(plan) == 2
    outs = []
    for rep in range(3):                                       # replays give the same bits
        for j in jobs:
            be.h2d(j[4], np.zeros(j[5], F))
        assert be.plan_run(plan)
        be.synchronize()
        outs.append([be.d2h(j[4], j[5], F) for j in jobs])
    for got, want in zip(outs[0], wants):
        assert rel_l2(got, want) < TOL
    for rep in (1, 2):
        for a, b in zip(outs[0], outs[rep]):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    be.plan_destroy(plan)


def test_sequence_of_dependent_plans_replays_like_the_eager_launches(be, fmt):
    """Three stages, each reading what the one before wrote (x -> a,b | a -> c | c,b -> d,e), recorded as one graph.
    Every replay — with the input rewritten and eager launches of other work on the same stream between them — has to
    give the bits of the same plans run one by one."""
    rng = np.random.default_rng(59)
    k0, ra, rb, rc, rd = 2560, 2048, 1024, 2560, 300
    q = {}
    for name, (rows, k, kind) in {"a": (ra, k0, "q4k"), "b": (rb, k0, "q8"), "c": (rc, ra, "q4k"), "d": (rd, rc, "q4k"), "e": (77, rb, "q8")}.items():
        w = (rng.standard_normal((rows, k)) * 0.02).astype(F)
        q[name] = (be.to_device(O.quantize_q4_k(w) if kind == "q4k" else O.quantize_q8_0(w)), fmt.FMT_Q4_K if kind == "q4k" else fmt.FMT_GGML_Q8_0, rows, k)
    x = be.malloc(k0 * 4)
    buf = {n: be.malloc(v[2] * 4) for n, v in q.items()}
    job = lambda n, src: (q[n][1], q[n][0], None, src, buf[n], q[n][2], q[n][3])
    stages = [[job("a", x), job("b", x)], [job("c", buf["a"])], [job("d", buf["c"]), job("e", buf["b"])]]
    plans = [be.plan_create(st) for st in stages]
    assert all(plans)
    seq = be.sequence_create(plans)
    assert seq and be.sequence_launch_count(seq) == sum(be.plan_launch_count(p) for p in plans) == 5
    other_x, other_out = be.to_device(rng.standard_normal(k0).astype(F)), be.malloc(ra * 4)
    for rep in range(4):
        be.h2d(x, (rng.standard_normal(k0) * (1.0 + rep)).astype(F))
        for p in plans:                                         # eager, one by one
            assert be.plan_run(p)
        be.synchronize()
        want = {n: be.d2h(buf[n], q[n][2], F) for n in buf}
        for n in buf:
            be.h2d(buf[n], np.full(q[n][2], np.nan, F))         # nothing of the eager run may survive into the replay's answer
        assert be.dev_matvec(q["a"][1], q["a"][0], None, other_x, ra, k0, other_out)   # other work on the stream
        assert be.sequence_run(seq)
        assert be.dev_matvec(q["a"][1], q["a"][0], None, other_x, ra, k0, other_out)
        be.synchronize()
        for n in buf:
            got = be.d2h(buf[n], q[n][2], F)
            assert np.array_equal(got.view(np.uint32), want[n].view(np.uint32)), (rep, n)
    assert rel_l2(want["a"], O.q4k_matvec(be.d2h(q["a"][0], ra * (k0 // 256) * 144, np.uint8), be.d2h(x, k0, F), ra, k0)) < TOL
    be.sequence_destroy(seq)
    for p in plans:
        be.plan_destroy(p)


def test_cpp_host_mirror():
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "larql_amd", "host", "host_test")
    assert os.path.exists(exe), "larql_amd/host/host_test is not built (run __graft_entry__.build())"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0 and "host_test ok" in r.stdout, r.stdout + r.stderr


# ------------------------------------------------------------------------ MoE
def test_router_select_matches_oracle(be):
    rng = np.random.default_rng(53)
    T, E, k = 64, 32, 4
    logits = rng.standard_normal((T, E)).astype(F)
    logits[0, :] = 1.0                                   # all tied -> first indices
    logits[1, :4] = 2.0; logits[1, 4:] = 1.0             # router.rs logits_32()
    logits[2, 5] = logits[2, 9] = 3.5                    # a tie inside the top-k
    dl, de, dw = be.to_device(logits), be.malloc(T * k * 4), be.malloc(T * k * 4)
    for policy in (O.NORMALISED_OVER_SELECTED, O.SOFTMAX_THEN_SELECT):
        assert be.dev_router_select(dl, T, E, k, policy, de, dw)
        e, w = be.d2h(de, (T, k), np.uint32), be.d2h(dw, (T, k), F)
        for t in range(T):
            want = O.router_select(logits[t], k, policy)
            assert [int(v) for v in e[t]] == [i for i, _ in want]
            assert np.allclose(w[t], [x for _, x in want], rtol=2e-6, atol=1e-7)
    assert [int(v) for v in e[0]] == [0, 1, 2, 3] and [int(v) for v in e[2][:2]] == [5, 9]
    assert be.dev_router_select(dl, T, E, 0, 1, de, dw)                  # k == 0: nothing to do
    assert not be.dev_router_select(dl, T, 257, 4, 1, de, dw)            # beyond this kernel: refused


@pytest.mark.parametrize("E,k", [(65, 4), (128, 4), (128, 8), (200, 8), (256, 8), (129, 1)])
def test_router_select_over_wide_banks_matches_oracle(be, E, k):
    """Banks of more than 64 experts (128 in the larger GPT-OSS and Gemma 4 checkpoints): a lane holds up to four logits.
    Same rule — logit descending, the lower index wins a tie, wherever the tied experts sit — both weight policies."""
    rng = np.random.default_rng(1000 + E + k)
    T = 40
    logits = rng.standard_normal((T, E)).astype(F)
    logits[0, :] = 1.0                                   # all tied -> the first k indices
    j1 = 69 if E > 69 else E - 1
    logits[1, 5] = logits[1, j1] = 4.0                   # a tie between two logits of one lane (where the bank has both)
    logits[2, E - 1] = 5.0; logits[2, 3] = 5.0           # ... and between lanes of different quarters
    logits[3, :] = -np.arange(E, dtype=F)                # descending by index
    logits[4, :] = np.arange(E, dtype=F) * F(0.01)       # the last experts win
    logits[5, :] = -1e30; logits[5, E - 2] = 0.0         # one expert takes all the weight
    dl, de, dw = be.to_device(logits), be.malloc(T * k * 4), be.malloc(T * k * 4)
    for policy in (O.NORMALISED_OVER_SELECTED, O.SOFTMAX_THEN_SELECT):
        assert be.dev_router_select(dl, T, E, k, policy, de, dw)
        e, w = be.d2h(de, (T, k), np.uint32), be.d2h(dw, (T, k), F)
        for t in range(T):
            want = O.router_select(logits[t], k, policy)
            assert [int(v) for v in e[t]] == [i for i, _ in want], (policy, t)
            assert np.allclose(w[t], [x for _, x in want], rtol=4e-6, atol=1e-7), (policy, t)
    assert [int(v) for v in e[0]] == list(range(k))
    if k >= 2:
        assert [int(v) for v in e[1][:2]] == [5, j1] and [int(v) for v in e[2][:2]] == [3, E - 1]


def _mx_bank(rng, E, n, kk, sigma=0.02):
    p, s = O.quantize_mxfp4((rng.standard_normal(E * n * kk) * sigma).astype(F), E * n, kk)
    return p, s


def _moe_case(rng, T, E, hidden, inter, biases, interleaved):
    """A bank (separate or fused-interleaved), activations, logits and optional biases, on the host."""
    c = {"T": T, "E": E, "hidden": hidden, "inter": inter, "interleaved": interleaved}
    gp, gs = _mx_bank(rng, E, inter, hidden)
    up, us = _mx_bank(rng, E, inter, hidden)
    c["dp"], c["ds"] = _mx_bank(rng, E, hidden, inter)
    if interleaved:       # fused region of expert e: row 2r = gate row r, row 2r+1 = up row r
        G = hidden // 32
        fp = np.empty((E, 2 * inter, G * 16), np.uint8); fs = np.empty((E, 2 * inter, G), np.uint8)
        fp[:, 0::2] = gp.reshape(E, inter, G * 16); fp[:, 1::2] = up.reshape(E, inter, G * 16)
        fs[:, 0::2] = gs.reshape(E, inter, G); fs[:, 1::2] = us.reshape(E, inter, G)
        c["gp"], c["gs"], c["up"], c["us"] = fp.reshape(-1), fs.reshape(-1), None, None
    else:
        c["gp"], c["gs"], c["up"], c["us"] = gp, gs, up, us
    c["x"] = rng.standard_normal((T, hidden)).astype(F)
    c["logits"] = rng.standard_normal((T, E)).astype(F)
    c["rb"] = rng.standard_normal(E).astype(F) if biases else None
    c["gub"] = (rng.standard_normal((E, 2 * inter)) * 0.5).astype(F) if biases else None
    c["db"] = (rng.standard_normal((E, hidden)) * 0.5).astype(F) if biases else None
    return c


def _moe_device_bank(be, fmt, c):
    dev = {n: (be.to_device(c[n]) if c[n] is not None else None) for n in ("gp", "gs", "up", "us", "dp", "ds", "rb", "gub", "db")}
    bank = fmt.Mxfp4Experts(dev["gp"], dev["gs"], dev["up"], dev["us"], dev["dp"], dev["ds"], c["E"], c["hidden"], c["inter"], 7.0, 1.702,
                            1 if c["interleaved"] else 0, dev["rb"], dev["gub"], dev["db"])
    return bank, dev


def _moe_oracle(c, experts, weights):
    return O.moe_block_mxfp4(c["x"], experts, weights, (c["gp"], c["gs"]), None if c["interleaved"] else (c["up"], c["us"]),
                             (c["dp"], c["ds"]), c["E"], c["hidden"], c["inter"], interleaved=bool(c["interleaved"]),
                             gate_up_bias=c["gub"], down_bias=c["db"])


@pytest.mark.parametrize("T,E,hidden,inter,biases,interleaved", [(1, 4, 2880, 2880, False, 0), (1, 6, 2880, 2880, True, 1), (1, 5, 384, 320, True, 0),
                                                                 (16, 8, 2880, 576, False, 0), (16, 8, 2880, 576, True, 1), (7, 6, 384, 320, True, 0),
                                                                 (1, 4, 96, 64, True, 0), (3, 4, 96, 64, True, 1)])
def test_moe_mxfp4_block_matches_oracle(be, fmt, T, E, hidden, inter, biases, interleaved):
    """The expert block (gate/up + bias -> ClampedGlu -> down + bias -> weighted sum) against the checker's block, whose
    composition is pinned on the reference's GPT-OSS fixture; with and without biases, both bank layouts, one token
    (the down projection folds experts and weighted sum) and several (device-built job lists); 96-wide rows take the
    kernels without matrix-core support."""
    rng = np.random.default_rng(59 + T + E)
    k = 4
    c = _moe_case(rng, T, E, hidden, inter, biases, interleaved)
    bank, dev = _moe_device_bank(be, fmt, c)
    dx, dl = be.to_device(c["x"]), be.to_device(c["logits"])
    de, dw_, do = be.malloc(T * k * 4), be.malloc(T * k * 4), be.malloc(T * hidden * 4)
    wsb = be.moe_mxfp4_workspace_bytes(T, k, hidden, inter)
    ws = be.malloc(wsb)
    # the selection with the router bias, as one call with the block
    assert be.dev_moe_mxfp4_routed(bank, dx, T, k, dl, O.NORMALISED_OVER_SELECTED, de, dw_, do, ws, wsb)
    be.synchronize()
    experts, weights = be.d2h(de, (T, k), np.uint32), be.d2h(dw_, (T, k), F)
    for t in range(T):
        want_sel = O.router_select(c["logits"][t] + (c["rb"] if biases else 0), k)
        assert [int(e) for e in experts[t]] == [e for e, _ in want_sel]
        assert np.allclose(weights[t], [w for _, w in want_sel], rtol=2e-6, atol=0)
    want = _moe_oracle(c, experts, weights)
    got = be.d2h(do, (T, hidden), F)
    assert rel_l2(got, want) < 1e-5
    # the block with the routing given: the same bits
    do2 = be.malloc(T * hidden * 4)
    assert be.dev_moe_mxfp4(bank, dx, T, k, de, dw_, do2, ws, wsb)
    be.synchronize()
    assert np.array_equal(be.d2h(do2, (T, hidden), F).view(np.uint32), got.view(np.uint32))
    assert not be.dev_moe_mxfp4(bank, dx, T, k, de, dw_, do, ws, wsb - 1024)   # short workspace: refused
    ws2 = be.malloc(wsb + 16)
    assert not be.dev_moe_mxfp4(bank, dx, T, k, de, dw_, do, ws2 + 4, wsb)     # workspace off a 16-byte boundary: refused


@pytest.mark.parametrize("T,hidden,inter", [(1, 384, 320), (6, 384, 320), (1, 96, 64)])
def test_moe_mxfp4_expert_id_outside_the_bank_is_skipped(be, fmt, T, hidden, inter):
    """cpu_moe_forward skips an expert the bank does not have (`moe.experts_gate_up.get(ei)` else return,
    cpu/ops/moe/forward.rs:203-208): the slot contributes nothing, and no byte beyond the bank is read."""
    rng = np.random.default_rng(5 + T)
    E, k = 4, 3
    c = _moe_case(rng, T, E, hidden, inter, True, 0)
    bank, dev = _moe_device_bank(be, fmt, c)
    experts = np.array([rng.permutation(E)[:k] for _ in range(T)], np.uint32)
    experts[0, 1] = E + 7                        # outside the bank
    if T > 2:
        experts[2, 0] = 0xFFFFFFFF
    weights = rng.random((T, k)).astype(F)
    dx, de, dw_, do = be.to_device(c["x"]), be.to_device(experts), be.to_device(weights), be.malloc(T * hidden * 4)
    wsb = be.moe_mxfp4_workspace_bytes(T, k, hidden, inter)
    ws = be.malloc(wsb)
    be.h2d(ws, np.full(wsb // 4, np.nan, F))     # whatever a skipped slot leaves unwritten must not reach the output
    assert be.dev_moe_mxfp4(bank, dx, T, k, de, dw_, do, ws, wsb)
    be.synchronize()
    got = be.d2h(do, (T, hidden), F)
    want = _moe_oracle(c, experts, weights)
    assert np.isfinite(got).all() and rel_l2(got, want) < 1e-5


def test_moe_mxfp4_tokens_sharing_an_expert_equal_single_token_calls(be, fmt):
    """Slots that chose the same expert are served up to four at a time from one read of its weights; a token's result
    must not depend on who it shared a job with: the 13-token block equals, bit for bit, the two-token blocks of its
    neighbouring tokens."""
    rng = np.random.default_rng(83)
    T, E, hidden, inter, k = 13, 6, 384, 320, 4          # 52 slots over 6 experts: full groups, leftovers of one to three, far-apart companions

    def bank(n, kk):
        p, s = [], []
        for _ in range(E):
            pp, ss = O.quantize_mxfp4((rng.standard_normal(n * kk) * 0.05).astype(F), n, kk)
            p.append(pp); s.append(ss)
        return np.concatenate(p), np.concatenate(s)

    gp, gs = bank(inter, hidden); up, us = bank(inter, hidden); dp, ds = bank(hidden, inter)
    x = rng.standard_normal((T, hidden)).astype(F)
    logits = rng.standard_normal((T, E)).astype(F)
    dev = {n: be.to_device(a) for n, a in dict(gp=gp, gs=gs, up=up, us=us, dp=dp, ds=ds, x=x, lg=logits).items()}
    b = fmt.Mxfp4Experts(dev["gp"], dev["gs"], dev["up"], dev["us"], dev["dp"], dev["ds"], E, hidden, inter, 7.0, 1.702)
    de, dw_, do = be.malloc(T * k * 4), be.malloc(T * k * 4), be.malloc(T * hidden * 4)
    assert be.dev_router_select(dev["lg"], T, E, k, O.NORMALISED_OVER_SELECTED, de, dw_)
    wsb = be.moe_mxfp4_workspace_bytes(T, k, hidden, inter)
    ws = be.malloc(wsb)
    assert be.dev_moe_mxfp4(b, dev["x"], T, k, de, dw_, do, ws, wsb)
    be.synchronize()
    got = be.d2h(do, (T, hidden), F)
    # every pair of neighbouring tokens as a block of its own: other companions, the same bits; the one-token call folds
    # the experts inside its down projection (another order of additions) and agrees to rounding
    two, one = be.malloc(2 * hidden * 4), be.malloc(hidden * 4)
    for t in range(T - 1):
        assert be.dev_moe_mxfp4(b, dev["x"] + t * hidden * 4, 2, k, de + t * k * 4, dw_ + t * k * 4, two, ws, wsb)
        be.synchronize()
        assert np.array_equal(be.d2h(two, (2, hidden), F), got[t:t + 2]), t
        assert be.dev_moe_mxfp4(b, dev["x"] + t * hidden * 4, 1, k, de + t * k * 4, dw_ + t * k * 4, one, ws, wsb)
        be.synchronize()
        assert rel_l2(be.d2h(one, hidden, F), got[t]) < 2e-6, t
    # and the oracle
    experts, weights = be.d2h(de, (T, k), np.uint32), be.d2h(dw_, (T, k), F)
    want = O.moe_block_mxfp4(x, experts, weights, (gp, gs), (up, us), (dp, ds), E, hidden, inter)
    assert rel_l2(got, want) < 1e-5


@pytest.mark.parametrize("T,E,hidden,inter,interleaved,policy", [(1, 8, 2880, 2880, 0, 1), (1, 8, 2880, 2880, 1, 1), (1, 6, 384, 320, 0, 0),
                                                                 (1, 64, 384, 320, 1, 1), (5, 6, 384, 320, 0, 1), (1, 3, 96, 64, 0, 1), (16, 32, 384, 320, 1, 1),
                                                                 (32, 9, 384, 320, 0, 0), (40, 12, 384, 320, 0, 1),
                                                                 (1, 128, 384, 320, 1, 1), (1, 200, 96, 64, 0, 0), (5, 128, 384, 320, 0, 1),
                                                                 (20, 256, 96, 64, 0, 1)])
def test_moe_mxfp4_routed_equals_select_then_block(be, fmt, T, E, hidden, inter, interleaved, policy):
    """Selection and expert block as one call: experts, weights and output bit for bit those of the two calls (one
    token: the selection runs inside the first matvec launch; k = 96 rows are below what that kernel takes and
    several tokens go through the selection kernel; so does a bank of more than 64 experts)."""
    rng = np.random.default_rng(500 + E + T)
    k = min(4, E)
    g_rows = 2 * inter if interleaved else inter
    gp, gs = O.quantize_mxfp4((rng.standard_normal(E * g_rows * hidden) * 0.03).astype(F), E * g_rows, hidden)
    dp, ds = O.quantize_mxfp4((rng.standard_normal(E * hidden * inter) * 0.03).astype(F), E * hidden, inter)
    dev = {n: be.to_device(a) for n, a in dict(gp=gp, gs=gs, dp=dp, ds=ds).items()}
    if interleaved:
        b = fmt.Mxfp4Experts(dev["gp"], dev["gs"], None, None, dev["dp"], dev["ds"], E, hidden, inter, 7.0, 1.702, 1)
    else:
        up, us = O.quantize_mxfp4((rng.standard_normal(E * inter * hidden) * 0.03).astype(F), E * inter, hidden)
        dev["up"], dev["us"] = be.to_device(up), be.to_device(us)
        b = fmt.Mxfp4Experts(dev["gp"], dev["gs"], dev["up"], dev["us"], dev["dp"], dev["ds"], E, hidden, inter, 7.0, 1.702, 0)
    x = be.to_device(rng.standard_normal((T, hidden)).astype(F))
    lg = rng.standard_normal((T, E)).astype(F)
    lg[0, 1] = lg[0, 2]                                   # a tie: the lower index first
    dl = be.to_device(lg)
    wsb = be.moe_mxfp4_workspace_bytes(T, k, hidden, inter)
    ws = be.malloc(wsb)
    e1, w1, o1 = be.malloc(T * k * 4), be.malloc(T * k * 4), be.malloc(T * hidden * 4)
    e2, w2, o2 = be.malloc(T * k * 4), be.malloc(T * k * 4), be.malloc(T * hidden * 4)
    assert be.dev_router_select(dl, T, E, k, policy, e1, w1)
    assert be.dev_moe_mxfp4(b, x, T, k, e1, w1, o1, ws, wsb)
    be.synchronize()
    want = (be.d2h(e1, (T, k), np.uint32), be.d2h(w1, (T, k), F), be.d2h(o1, (T, hidden), F))
    for rep in range(2):                                   # (the second call finds its job tables already on the device)
        assert be.dev_moe_mxfp4_routed(b, x, T, k, dl, policy, e2, w2, o2, ws, wsb)
        be.synchronize()
        got = (be.d2h(e2, (T, k), np.uint32), be.d2h(w2, (T, k), F), be.d2h(o2, (T, hidden), F))
        assert np.array_equal(got[0], want[0])
        assert np.array_equal(got[1].view(np.uint32), want[1].view(np.uint32))
        assert np.array_equal(got[2].view(np.uint32), want[2].view(np.uint32))
    assert [int(v) for v in want[0][0]] == [i for i, _ in O.router_select(lg[0], k, policy)]
    import larql_amd
    with pytest.raises(larql_amd.DeviceError):                                        # no logits: an argument error
        be.dev_moe_mxfp4_routed(b, x, T, k, 0, policy, e2, w2, o2, ws, wsb)


def test_moe_mxfp4_job_groups_of_every_size(be, fmt):
    """Experts chosen by 1, 2, 3, 4 and 5 slots: jobs of one, two, three and four tokens and a second job for the
    fifth.  Every token's result equals, bit for bit, what it is in a two-token block."""
    rng = np.random.default_rng(97)
    E, hidden, inter, k = 6, 384, 320, 2
    picks = [(4, 5)] * 5 + [(0, 3), (1, 3), (1, 2), (2, 3), (2, 3)]
    order = rng.permutation(len(picks))
    picks = [picks[i] for i in order]
    T = len(picks)
    logits = (rng.standard_normal((T, E)) * 0.1).astype(F)
    for t, (a, b_) in enumerate(picks):
        logits[t, a] = 5.0 + 0.01 * t
        logits[t, b_] = 4.0

    def bank(n, kk):
        p, s = [], []
        for _ in range(E):
            pp, ss = O.quantize_mxfp4((rng.standard_normal(n * kk) * 0.05).astype(F), n, kk)
            p.append(pp); s.append(ss)
        return np.concatenate(p), np.concatenate(s)

    gp, gs = bank(inter, hidden); up, us = bank(inter, hidden); dp, ds = bank(hidden, inter)
    x = rng.standard_normal((T, hidden)).astype(F)
    dev = {n: be.to_device(a) for n, a in dict(gp=gp, gs=gs, up=up, us=us, dp=dp, ds=ds, x=x, lg=logits).items()}
    b = fmt.Mxfp4Experts(dev["gp"], dev["gs"], dev["up"], dev["us"], dev["dp"], dev["ds"], E, hidden, inter, 7.0, 1.702)
    de, dw_, do = be.malloc(T * k * 4), be.malloc(T * k * 4), be.malloc(T * hidden * 4)
    assert be.dev_router_select(dev["lg"], T, E, k, O.NORMALISED_OVER_SELECTED, de, dw_)
    chosen = be.d2h(de, (T, k), np.uint32)
    assert sorted(np.bincount(chosen.reshape(-1), minlength=E).tolist()) == [1, 2, 3, 4, 5, 5]
    wsb = be.moe_mxfp4_workspace_bytes(T, k, hidden, inter)
    ws = be.malloc(wsb)
    assert be.dev_moe_mxfp4(b, dev["x"], T, k, de, dw_, do, ws, wsb)
    be.synchronize()
    got = be.d2h(do, (T, hidden), F)
    two = be.malloc(2 * hidden * 4)
    for t in range(T - 1):
        assert be.dev_moe_mxfp4(b, dev["x"] + t * hidden * 4, 2, k, de + t * k * 4, dw_ + t * k * 4, two, ws, wsb)
        be.synchronize()
        assert np.array_equal(be.d2h(two, (2, hidden), F), got[t:t + 2]), t
    experts, weights = be.d2h(de, (T, k), np.uint32), be.d2h(dw_, (T, k), F)
    assert rel_l2(got, O.moe_block_mxfp4(x, experts, weights, (gp, gs), (up, us), (dp, ds), E, hidden, inter)) < 1e-5


@pytest.mark.parametrize("T,E,hidden,inter", [(1, 4, 2880, 2880), (13, 6, 384, 320), (16, 8, 2880, 576)])
def test_moe_mxfp4_interleaved_gate_up_bank_equals_separate_banks(be, fmt, T, E, hidden, inter):
    """MoeFusedRowLayout::Interleaved (pipeline/moe.rs:294-332; FusedHalf::fused_row, mxfp4.rs:179-191): a GPT-OSS
    gate_up region holds gate on the even and up on the odd fused rows.  Walking it in place gives the block the
    de-interleaved banks give, bit for bit (a row's sum does not depend on its neighbours)."""
    rng = np.random.default_rng(7 * T + E)
    k = 4

    def bank(n, kk):
        p, s = [], []
        for _ in range(E):
            pp, ss = O.quantize_mxfp4((rng.standard_normal(n * kk) * 0.04).astype(F), n, kk)
            p.append(pp); s.append(ss)
        return np.concatenate(p), np.concatenate(s)

    gp, gs = bank(inter, hidden); up, us = bank(inter, hidden); dp, ds = bank(hidden, inter)
    G = hidden // 32
    # the fused region of expert e: row 2r = gate row r, row 2r+1 = up row r (16 G packed bytes and G scale bytes per row)
    fp = np.empty((E, 2 * inter, G * 16), np.uint8); fs = np.empty((E, 2 * inter, G), np.uint8)
    fp[:, 0::2] = gp.reshape(E, inter, G * 16); fp[:, 1::2] = up.reshape(E, inter, G * 16)
    fs[:, 0::2] = gs.reshape(E, inter, G); fs[:, 1::2] = us.reshape(E, inter, G)
    assert O.fused_row_walk(O.INTERLEAVED, O.HALF_UP, inter) == (1, 2) and O.fused_row_walk(O.CONTIGUOUS_HALVES, O.HALF_UP, inter) == (inter, 1)
    x = rng.standard_normal((T, hidden)).astype(F)
    logits = rng.standard_normal((T, E)).astype(F)
    dev = {n: be.to_device(a) for n, a in dict(gp=gp, gs=gs, up=up, us=us, dp=dp, ds=ds, fp=fp.reshape(-1), fs=fs.reshape(-1), x=x,
                                                lg=logits).items()}
    de, dw_ = be.malloc(T * k * 4), be.malloc(T * k * 4)
    assert be.dev_router_select(dev["lg"], T, E, k, O.NORMALISED_OVER_SELECTED, de, dw_)
    wsb = be.moe_mxfp4_workspace_bytes(T, k, hidden, inter)
    ws = be.malloc(wsb)
    outs = []
    for b in (fmt.Mxfp4Experts(dev["gp"], dev["gs"], dev["up"], dev["us"], dev["dp"], dev["ds"], E, hidden, inter, 7.0, 1.702, 0),
              fmt.Mxfp4Experts(dev["fp"], dev["fs"], None, None, dev["dp"], dev["ds"], E, hidden, inter, 7.0, 1.702, 1)):
        do = be.malloc(T * hidden * 4)
        assert be.dev_moe_mxfp4(b, dev["x"], T, k, de, dw_, do, ws, wsb)
        be.synchronize()
        outs.append(be.d2h(do, (T, hidden), F))
    assert np.isfinite(outs[0]).all() and np.abs(outs[0]).max() > 0
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    # a bank that says "separate" but brings no up half is an argument error
    import larql_amd
    with pytest.raises(larql_amd.DeviceError):
        be.dev_moe_mxfp4(fmt.Mxfp4Experts(dev["fp"], dev["fs"], None, None, dev["dp"], dev["ds"], E, hidden, inter, 7.0, 1.702, 0),
                         dev["x"], T, k, de, dw_, do, ws, wsb)


@pytest.mark.parametrize("T,E,hidden,inter,layout,per_expert,renorm", [
    (1, 5, 2880, 2880, "interleaved", False, True),       # a GPT-OSS layer's shapes, one token: selection inside the first launch
    (1, 6, 384, 320, "halves", False, True),
    (5, 6, 384, 320, "interleaved", True, True),          # several tokens, MoeExpertScalePolicy::PerExpert
    (9, 8, 2880, 576, "halves", True, False),             # ... and the softmax's own values (no renormalisation)
    (1, 4, 96, 64, "interleaved", True, True),            # rows the matrix-core kernels do not take
    (1, 128, 384, 320, "interleaved", False, True),       # 128 experts, top-8 (Gemma 4 26B-A4B's count): one token
    (6, 128, 384, 320, "halves", True, True),             # ... several tokens, per-expert scale
    (3, 128, 384, 320, "interleaved", False, False),      # ... the planner selects
])
def test_moe_layer_from_per_expert_slices_with_router_projection(be, fmt, T, E, hidden, inter, layout, per_expert, renorm):
    """MoeLayerWeights as the reference brings it (pipeline/moe.rs:469-541): per-expert gate+up / down slices in
    allocations of their own, MoeExpertScales::Paired exponent streams, Interleaved or ContiguousHalves fused rows,
    router_proj / router_bias / router_per_expert_scale.  The layer goes residual -> output with the router's
    projection on the device: the route equals moe_route_from_router_input (mod.rs:149-186), the output the checker's
    expert block under that route; host tier and device tier agree bit for bit."""
    rng = np.random.default_rng(211 + T + E)
    k, G, Gd = (8 if E > 64 else 4), hidden // 32, inter // 32
    gate = [O.quantize_mxfp4((rng.standard_normal(inter * hidden) * 0.02).astype(F), inter, hidden) for _ in range(E)]
    up = [O.quantize_mxfp4((rng.standard_normal(inter * hidden) * 0.02).astype(F), inter, hidden) for _ in range(E)]
    down = [O.quantize_mxfp4((rng.standard_normal(hidden * inter) * 0.02).astype(F), hidden, inter) for _ in range(E)]
    gu_p, gu_s = [], []                                   # expert e's fused slice, an allocation of its own
    for e in range(E):
        p, s = np.empty((2 * inter, G * 16), np.uint8), np.empty((2 * inter, G), np.uint8)
        if layout == "interleaved":
            p[0::2], p[1::2] = gate[e][0].reshape(inter, -1), up[e][0].reshape(inter, -1)
            s[0::2], s[1::2] = gate[e][1].reshape(inter, -1), up[e][1].reshape(inter, -1)
        else:
            p[:inter], p[inter:] = gate[e][0].reshape(inter, -1), up[e][0].reshape(inter, -1)
            s[:inter], s[inter:] = gate[e][1].reshape(inter, -1), up[e][1].reshape(inter, -1)
        gu_p.append(np.concatenate([p.reshape(-1), np.full(7 + e, 0xEE, np.uint8)]))     # (slices may be longer than the geometry)
        gu_s.append(s.reshape(-1).copy())
    router_w = (rng.standard_normal((E, hidden)) * 0.05).astype(F)
    router_b = rng.standard_normal(E).astype(F)
    gub = (rng.standard_normal((E, 2 * inter)) * 0.5).astype(F)
    db = (rng.standard_normal((E, hidden)) * 0.5).astype(F)
    scale = rng.uniform(0.5, 2.0, E).astype(F) if per_expert else None
    x = rng.standard_normal((T, hidden)).astype(F)
    rin = (x * F(0.5) + F(0.25)).astype(F)                # the router's input is its own tensor (a norm of the residual in the reference)
    rows = fmt.MOE_ROWS_INTERLEAVED if layout == "interleaved" else fmt.MOE_ROWS_CONTIGUOUS_HALVES
    layer = be.moe_layer_create(gu_p, [d[0] for d in down], gu_s, [d[1] for d in down], router_w, k, hidden, inter, rows,
                                router_bias=router_b, gate_up_bias=gub, down_bias=db, per_expert_scale=scale, renormalized=renorm)
    assert layer
    got = be.moe_layer_forward(layer, rin, x, k)
    assert got is not None
    out, experts, weights = got
    # the route: moe_route_from_router_input on the same tensors
    for t in range(T):
        want = O.moe_route_from_router_input(rin[t], router_w, router_b, k, renormalize=renorm, per_expert_scale=scale)
        # (the device's f32 gemv adds in another order than the sequential dot: logits differ in the last bits, so a
        # selection may only differ where two probabilities are that close)
        assert [int(e) for e in experts[t]] == [e for e, _ in want], t
        assert np.allclose(weights[t], [w for _, w in want], rtol=5e-5, atol=0)
    gpb, gsb = np.concatenate([g[0] for g in gate]), np.concatenate([g[1] for g in gate])
    upb, usb = np.concatenate([u[0] for u in up]), np.concatenate([u[1] for u in up])
    dpb, dsb = np.concatenate([d[0] for d in down]), np.concatenate([d[1] for d in down])
    want_out = O.moe_block_mxfp4(x, experts.astype(np.uint64), weights, (gpb, gsb), (upb, usb), (dpb, dsb), E, hidden, inter,
                                 gate_up_bias=gub, down_bias=db)
    assert rel_l2(out, want_out) < 1e-5
    # device tier on resident operands: the same bits, nothing crosses the bus
    dx, dr, do = be.to_device(x), be.to_device(rin), be.malloc(T * hidden * 4)
    de, dw_ = be.malloc(T * k * 4), be.malloc(T * k * 4)
    assert be.dev_moe_layer_forward(layer, dr, dx, T, do, de, dw_)
    be.synchronize()
    assert np.array_equal(be.d2h(do, (T, hidden), F).view(np.uint32), out.view(np.uint32))
    assert np.array_equal(be.d2h(de, (T, k), np.uint32), experts) and np.array_equal(be.d2h(dw_, (T, k), F).view(np.uint32), weights.view(np.uint32))
    be.moe_layer_destroy(layer)


@pytest.mark.parametrize("T,E,k,hidden,cols,inter,wfmt,rule,biases,per_expert", [
    (1, 8, 4, 512, 512, 704, "q4k", 1, False, True),       # Gemma 4 26B-A4B's shape rules in small: inter 704 stored 768 wide, GeluTanh, per-expert scale
    (5, 128, 8, 768, 768, 256, "q4k", 1, False, True),     # ... its 128 experts, top-8, several tokens
    (3, 6, 4, 480, 512, 320, "q4k", 0, True, False),       # rows stored wider than hidden (GPT-OSS 2880 -> 3072 in small), ClampedGlu, biases
    (1, 6, 2, 2816, 2816, 704, "q4k", 1, False, False),    # Gemma 4 26B-A4B's real expert shape
    (4, 5, 3, 512, 512, 320, "q6k", 2, True, False),       # a Q6_K bank, SiLU
    (1, 4, 2, 256, 768, 256, "q6k", 1, False, True),
    (300, 8, 2, 256, 256, 256, "q4k", 2, True, False),     # many tokens: 600 slots, job tables of 1200 and 600 entries
])
def test_moe_layer_over_a_k_quant_bank_matches_the_integer_expert_path(be, fmt, T, E, k, hidden, cols, inter, wfmt, rule, biases, per_expert):
    """MoeLayerWeights with expert_data_format Q4_K / Q6_K (Inline scales, ContiguousHalves rows): cpu_moe_forward's
    integer path (cpu/ops/moe/forward.rs:160-330) — expert input and gated activation as Q8_K, every matvec the integer
    kernel.  The route equals moe_route_from_router_input; the output the checker's block under that route (the
    matvecs are bit-exact, expf / tanhf of the device may move an activation code by one step: 2e-4 is asserted where
    the stated bar is 1e-3); host tier and device tier agree bit for bit."""
    rng = np.random.default_rng(700 + T + E + inter)
    ip = (inter + 255) // 256 * 256
    quant = O.quantize_q4_k if wfmt == "q4k" else O.quantize_q6_k
    f = 4 if wfmt == "q4k" else 6
    gate_up = [quant((rng.standard_normal((2 * inter, cols)) * 0.05).astype(F)) for _ in range(E)]
    down = [np.concatenate([quant((rng.standard_normal((hidden, ip)) * 0.05).astype(F)), np.full(5 + e, 0xEE, np.uint8)])
            for e in range(E)]                                                     # (slices may be longer than the geometry)
    router_w = (rng.standard_normal((E, hidden)) * 0.05).astype(F)
    router_b = rng.standard_normal(E).astype(F)
    gub = (rng.standard_normal((E, 2 * inter)) * 0.5).astype(F) if biases else None
    db = (rng.standard_normal((E, hidden)) * 0.5).astype(F) if biases else None
    scale = rng.uniform(0.5, 2.0, E).astype(F) if per_expert else None
    x = rng.standard_normal((T, hidden)).astype(F)
    rin = (x * F(0.5) + F(0.25)).astype(F)
    layer = be.moe_layer_create(gate_up, down, None, None, router_w, k, hidden, inter, fmt.MOE_ROWS_CONTIGUOUS_HALVES, router_bias=router_b,
                                gate_up_bias=gub, down_bias=db, per_expert_scale=scale, expert_scales=fmt.MOE_SCALES_INLINE,
                                expert_data_format=fmt.FMT_Q4_K if wfmt == "q4k" else fmt.FMT_Q6_K, gate_rule=rule)
    assert layer, be.last_error()
    got = be.moe_layer_forward(layer, rin, x, k)
    assert got is not None, be.last_error()
    out, experts, weights = got
    for t in range(T):
        want = O.moe_route_from_router_input(rin[t], router_w, router_b, k, renormalize=True, per_expert_scale=scale)
        assert [int(e) for e in experts[t]] == [e for e, _ in want], t
        assert np.allclose(weights[t], [w for _, w in want], rtol=5e-5, atol=0)
    want_out = O.moe_block_kq(x, experts, weights, gate_up, down, hidden, cols, inter, f, gub, db, rule)
    assert rel_l2(out, want_out) < 2e-4
    dx, dr, do = be.to_device(x), be.to_device(rin), be.malloc(T * hidden * 4)
    de, dw_ = be.malloc(T * k * 4), be.malloc(T * k * 4)
    for rep in range(2):                                   # (the second call finds its job tables already on the device)
        assert be.dev_moe_layer_forward(layer, dr, dx, T, do, de, dw_)
        be.synchronize()
        assert np.array_equal(be.d2h(do, (T, hidden), F).view(np.uint32), out.view(np.uint32))
        assert np.array_equal(be.d2h(de, (T, k), np.uint32), experts)
    # a token alone gives the token's row of the batch, bit for bit (no arithmetic is shared between tokens)
    if T > 1:
        one = be.moe_layer_forward(layer, rin[1:2], x[1:2], k)
        assert one is not None and np.array_equal(one[0][0].view(np.uint32), out[1].view(np.uint32))
    be.moe_layer_destroy(layer)


def _float_bytes(a, kind):
    a = np.ascontiguousarray(a, F)
    if kind == "bf16":
        return (a.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8).reshape(-1)
    if kind == "f16":
        return a.astype(np.float16).view(np.uint8).reshape(-1)
    return a.view(np.uint8).reshape(-1)


@pytest.mark.parametrize("T,E,k,hidden,inter,kind,rule,biases", [
    (1, 6, 2, 256, 704, "bf16", 1, False),       # the legacy BF16 monolith's arm: GeluTanh, no biases
    (5, 8, 4, 512, 320, "bf16", 0, True),
    (3, 4, 2, 128, 96, "f16", 2, True),
    (2, 3, 1, 64, 48, "f32", 1, True),
])
def test_moe_layer_over_a_float_bank_matches_the_f32_arm(be, fmt, T, E, k, hidden, inter, kind, rule, biases):
    """MoeLayerWeights with expert_data_format BF16 / F16 / F32: cpu_moe_forward's f32 arm (forward.rs:246-290) — f32
    activations throughout, the dense matvec kernels on the expert picked at run time, down rows unpadded."""
    rng = np.random.default_rng(900 + T + E + inter)
    f = {"bf16": 16, "f16": 17, "f32": 32}[kind]
    dfmt = {"bf16": fmt.FMT_BF16, "f16": fmt.FMT_F16, "f32": fmt.FMT_F32}[kind]
    gate_up = [_float_bytes(rng.standard_normal((2 * inter, hidden)) * 0.05, kind) for _ in range(E)]
    down = [_float_bytes(rng.standard_normal((hidden, inter)) * 0.05, kind) for _ in range(E)]
    router_w = (rng.standard_normal((E, hidden)) * 0.05).astype(F)
    gub = (rng.standard_normal((E, 2 * inter)) * 0.5).astype(F) if biases else None
    db = (rng.standard_normal((E, hidden)) * 0.5).astype(F) if biases else None
    x = rng.standard_normal((T, hidden)).astype(F)
    layer = be.moe_layer_create(gate_up, down, None, None, router_w, k, hidden, inter, fmt.MOE_ROWS_CONTIGUOUS_HALVES, gate_up_bias=gub,
                                down_bias=db, expert_scales=fmt.MOE_SCALES_INLINE, expert_data_format=dfmt, gate_rule=rule)
    assert layer, be.last_error()
    got = be.moe_layer_forward(layer, x, x, k)
    assert got is not None, be.last_error()
    out, experts, weights = got
    for t in range(T):
        want = O.moe_route_from_router_input(x[t], router_w, None, k, renormalize=True)
        assert [int(e) for e in experts[t]] == [e for e, _ in want], t
    want_out = O.moe_block_kq(x, experts, weights, gate_up, down, hidden, hidden, inter, f, gub, db, rule)
    assert rel_l2(out, want_out) < 1e-5
    dx, do, de, dw_ = be.to_device(x), be.malloc(T * hidden * 4), be.malloc(T * k * 4), be.malloc(T * k * 4)
    assert be.dev_moe_layer_forward(layer, dx, dx, T, do, de, dw_)
    be.synchronize()
    assert np.array_equal(be.d2h(do, (T, hidden), F).view(np.uint32), out.view(np.uint32))
    be.moe_layer_destroy(layer)


def test_moe_layer_float_bank_reproduces_the_reference_plumbing_tests(be, fmt):
    """The hand-derived expectations of the reference's own tests for this path (cpu/ops/moe/expert/tests/bias.rs:52-146:
    BF16 identity expert, h = [1, 2], asymmetric interleaved biases, tolerance 1e-4), the 2 x 2 identity sitting in a
    16 x 16 frame of zeros (the dense kernel's rows are multiples of 16 elements): a swapped or dropped bias, the
    gate / up halves exchanged or another combine rule change these numbers."""
    H = I = 16
    gate_up = np.zeros((2 * I, H), F)
    for row in range(2 * I):
        gate_up[row, row % I] = 1.0
    down = np.eye(H, I, dtype=F)
    gu, dn = _float_bytes(gate_up, "bf16"), _float_bytes(down, "bf16")
    rw = np.zeros((1, H), F)
    silu = lambda v: v / (1.0 + np.exp(-v))

    def run(h, rule, gub=None, db=None):
        layer = be.moe_layer_create([gu], [dn], None, None, rw, 1, H, I, fmt.MOE_ROWS_CONTIGUOUS_HALVES, gate_up_bias=gub, down_bias=db,
                                    expert_scales=fmt.MOE_SCALES_INLINE, expert_data_format=fmt.FMT_BF16, gate_rule=rule)
        assert layer, be.last_error()
        x = np.zeros((1, H), F)
        x[0, :2] = h
        out = be.moe_layer_forward(layer, x, x, 1)
        be.moe_layer_destroy(layer)
        assert out is not None and out[2][0, 0] == 1.0
        return out[0][0]

    fused = np.zeros((1, 2 * I), F)
    fused[0, :4] = [0.5, 3.0, -0.25, 7.0]                        # gate biases [0.5, -0.25], up biases [3, 7], interleaved
    got = run([1.0, 2.0], fmt.MOE_GATE_SILU, gub=fused)
    assert np.allclose(got[:2], [silu(1.5) * 4.0, silu(1.75) * 9.0], atol=1e-4) and not got[2:].any()
    dbias = np.zeros((1, H), F)
    dbias[0, :2] = [10.0, -20.0]
    got = run([1.0, 2.0], fmt.MOE_GATE_SILU, db=dbias)
    assert np.allclose(got[:2], [silu(1.0) * 1.0 + 10.0, silu(2.0) * 2.0 - 20.0], atol=1e-4)
    got = run([2.0, 0.0], fmt.MOE_GATE_CLAMPED_GLU)
    assert abs(got[0] - 3.0 * (2.0 / (1.0 + np.exp(-2.0 * 1.702)))) < 1e-4 and got[1] == 0.0
    assert abs(got[0] - run([2.0, 0.0], fmt.MOE_GATE_SILU)[0]) > 0.5


def test_moe_layer_gate_rules_on_reference_held_points(be, fmt):
    """Every MoeGateRule the layer serves, through the device: SituGlu on the points the reference holds for it
    (ffn/expert_weight/tests/situ_oracle.json, both arms, its tolerance 1e-5), ClampedGlu on the PyTorch values of
    ffn/expert_weight/gate.rs:108-117, ClampedGated on that file's points.  An F32 bank with zero gate / up weights and
    an identity down matrix: the fused bias row carries (gate, up) to the combine rule exactly, the output is the rule's
    value per element."""
    arms = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "situ_glu_golden.json")))["arms"]
    H = I = 96
    gu = np.zeros((2 * I, H), F).view(np.uint8).reshape(-1)
    dn = np.eye(H, I, dtype=F).view(np.uint8).reshape(-1)
    rw = np.zeros((1, H), F)
    x = np.zeros((1, H), F)

    def run(rule, gate, up, limit, alpha):
        fused = np.zeros((1, 2 * I), F)
        fused[0, 0:2 * len(gate):2] = gate
        fused[0, 1:2 * len(up):2] = up
        layer = be.moe_layer_create([gu], [dn], None, None, rw, 1, H, I, fmt.MOE_ROWS_CONTIGUOUS_HALVES, gate_up_bias=fused,
                                    expert_scales=fmt.MOE_SCALES_INLINE, expert_data_format=fmt.FMT_F32, gate_rule=rule, limit=limit, alpha=alpha)
        assert layer, be.last_error()
        out = be.moe_layer_forward(layer, x, x, 1)
        be.moe_layer_destroy(layer)
        assert out is not None
        return out[0][0][:len(gate)]

    for name, arm in arms.items():
        got = run(fmt.MOE_GATE_SITU_GLU, arm["gate"], arm["up"], arm["beta"], arm["linear_beta"] or 0.0)
        want = np.array(arm["out"], F)
        assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(1.0, np.abs(want))), name
    got = run(fmt.MOE_GATE_CLAMPED_GLU, [-2.0, 0.0, 1.5, 9.0], [0.5, -1.0, 2.0, -9.0], 7.0, 1.702)
    assert np.all(np.abs(got - np.array([-0.0965121, 0.0, 4.174987, -41.999718], F)) < 1e-5)
    pts = [(0.5, 0.25), (-0.5, 0.25), (25.0, 0.5), (-25.0, 0.5), (0.5, 25.0), (0.5, -25.0), (-40.0, 1.0), (1.0, -40.0)]
    for rule, orule in ((fmt.MOE_GATE_CLAMPED_SILU, O.GATE_CLAMPED_SILU), (fmt.MOE_GATE_CLAMPED_GELU_TANH, O.GATE_CLAMPED_GELU_TANH),
                        (fmt.MOE_GATE_SILU, O.GATE_SILU), (fmt.MOE_GATE_GELU_TANH, O.GATE_GELU_TANH)):
        got = run(rule, [g for g, _ in pts], [u for _, u in pts], 10.0, 0.0)
        want = np.array([O.moe_combine(orule, g, u, 10.0, 0.0) for g, u in pts], F)
        assert np.all(np.abs(got - want) <= 2e-6 * np.maximum(1.0, np.abs(want))), rule
    # SituGlu without a positive beta has no meaning: refused
    assert be.moe_layer_create([gu], [dn], None, None, rw, 1, H, I, fmt.MOE_ROWS_CONTIGUOUS_HALVES, expert_scales=fmt.MOE_SCALES_INLINE,
                               expert_data_format=fmt.FMT_F32, gate_rule=fmt.MOE_GATE_SITU_GLU, limit=0.0) is None


def test_moe_layer_reproduces_the_reference_moe_fixture(be, fmt):
    """EXPECTED[48] of larql-compute/tests/test_moe_reference_parity.rs:72-85 — values an independent transcription of
    the GPT-OSS reference model produced — through the device entry point: the fixture's f32 bank (fused rows
    de-interleaved into gate / up halves, what a canonicalising extraction stores), its router weights and bias, the
    interleaved bias rows, both expert biases, ClampedGlu, top-2 of 4 experts over 3 tokens; the inputs regenerated by
    the fixture's own LCG.  The reference's tolerance: 1e-5."""
    import test_oracle_moe as ref
    x, router_w, router_b, fused, fused_bias, down, down_bias = ref.draw()
    E, H, I = ref.EXPERTS, ref.HIDDEN, ref.INTER
    gate_up = [np.concatenate([fused[e][0::2], fused[e][1::2]]).astype(F).view(np.uint8).reshape(-1) for e in range(E)]
    dn = [np.ascontiguousarray(down[e], F).view(np.uint8).reshape(-1) for e in range(E)]
    layer = be.moe_layer_create(gate_up, dn, None, None, router_w, ref.TOP_K, H, I, fmt.MOE_ROWS_CONTIGUOUS_HALVES, router_bias=router_b,
                                gate_up_bias=fused_bias, down_bias=down_bias, expert_scales=fmt.MOE_SCALES_INLINE,
                                expert_data_format=fmt.FMT_F32, gate_rule=fmt.MOE_GATE_CLAMPED_GLU, limit=7.0, alpha=1.702)
    assert layer, be.last_error()
    got = be.moe_layer_forward(layer, x, x, ref.TOP_K)
    be.moe_layer_destroy(layer)
    assert got is not None
    assert float(np.max(np.abs(got[0] - ref.EXPECTED))) < ref.TOLERANCE
    assert set(map(int, got[1][2])) != set(map(int, got[1][0]))        # the fixture's own remark: token 2 routes elsewhere


def test_moe_layer_properties_the_reference_asserts_for_cpu_moe_forward(be, fmt):
    """cpu/ops/moe/forward/tests.rs: a bank whose rows are stored wider than hidden gives what the unpadded bank gives
    (:535-560, the pad columns holding weights the zero-padded activation must cancel), and a zero per-expert scale
    silences the selected expert (:169-197) — on a BF16 bank of ones, in a 16-wide frame."""
    H, W, I = 16, 32, 16
    ones = lambda n: (np.ones(n, F).view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
    rw = np.ones((1, H), F)
    h = np.ones((1, H), F)
    kw = dict(expert_scales=fmt.MOE_SCALES_INLINE, expert_data_format=fmt.FMT_BF16, gate_rule=fmt.MOE_GATE_SILU)

    def run(gate_up, **more):
        layer = be.moe_layer_create([gate_up], [ones(H * I)], None, None, rw, 1, H, I, fmt.MOE_ROWS_CONTIGUOUS_HALVES, **dict(kw, **more))
        assert layer, be.last_error()
        out = be.moe_layer_forward(layer, h, h, 1)
        be.moe_layer_destroy(layer)
        assert out is not None
        return out[0][0]

    plain, padded = run(ones(2 * I * H)), run(ones(2 * I * W))
    assert np.array_equal(plain.view(np.uint32), padded.view(np.uint32)) and plain[0] > 1.0
    g = float(H)                                                                   # every gate and up row sums 16 ones
    assert np.allclose(plain, I * (g / (1.0 + np.exp(-g))) * g, rtol=1e-6)
    assert not run(ones(2 * I * H), per_expert_scale=np.zeros(1, F)).any()


def test_moe_layer_k_quant_refusals(be, fmt):
    """A k-quant bank the CPU tier itself would refuse, or that has no kernel here, answers None: Interleaved rows
    (forward.rs:69-75), Paired scales, slices shorter than the geometry, rows beyond 10240 elements."""
    rng = np.random.default_rng(4)
    E, hidden, inter, k = 3, 256, 256, 2
    gu = [O.quantize_q4_k((rng.standard_normal((2 * inter, hidden)) * 0.05).astype(F)) for _ in range(E)]
    dn = [O.quantize_q4_k((rng.standard_normal((hidden, inter)) * 0.05).astype(F)) for _ in range(E)]
    rw = rng.standard_normal((E, hidden)).astype(F)
    kw = dict(expert_scales=fmt.MOE_SCALES_INLINE, expert_data_format=fmt.FMT_Q4_K, gate_rule=fmt.MOE_GATE_GELU_TANH)
    ok = be.moe_layer_create(gu, dn, None, None, rw, k, hidden, inter, fmt.MOE_ROWS_CONTIGUOUS_HALVES, **kw)
    assert ok
    be.moe_layer_destroy(ok)
    assert be.moe_layer_create(gu, dn, None, None, rw, k, hidden, inter, fmt.MOE_ROWS_INTERLEAVED, **kw) is None
    assert be.moe_layer_create(gu, dn, None, None, rw, k, hidden, inter, fmt.MOE_ROWS_CONTIGUOUS_HALVES,
                               **dict(kw, expert_scales=fmt.MOE_SCALES_PAIRED)) is None
    assert be.moe_layer_create(gu, dn, None, None, rw, k, hidden, inter, fmt.MOE_ROWS_CONTIGUOUS_HALVES, **dict(kw, gate_rule=7)) is None
    assert be.moe_layer_create([g[:-144] for g in gu], dn, None, None, rw, k, hidden, inter, fmt.MOE_ROWS_CONTIGUOUS_HALVES, **kw) is None
    assert be.moe_layer_create(gu, [d[:-1] for d in dn], None, None, rw, k, hidden, inter, fmt.MOE_ROWS_CONTIGUOUS_HALVES, **kw) is None
    # more (token, expert) slots than one call takes
    assert be.moe_layer_forward(ok2 := be.moe_layer_create(gu, dn, None, None, rw, k, hidden, inter, fmt.MOE_ROWS_CONTIGUOUS_HALVES, **kw),
                                np.zeros((40000, hidden), F), np.zeros((40000, hidden), F), k) is None
    be.moe_layer_destroy(ok2)
    # an MXFP4 bank under another gate rule: no kernel
    g4 = [O.quantize_mxfp4((rng.standard_normal(2 * 32 * 64) * 0.02).astype(F), 2 * 32, 64) for _ in range(E)]
    d4 = [O.quantize_mxfp4((rng.standard_normal(64 * 32) * 0.02).astype(F), 64, 32) for _ in range(E)]
    assert be.moe_layer_create([g[0] for g in g4], [d[0] for d in d4], [g[1] for g in g4], [d[1] for d in d4], rng.standard_normal((E, 64)).astype(F),
                               k, 64, 32, gate_rule=fmt.MOE_GATE_SILU) is None


def test_moe_layer_refusals(be, fmt):
    """What MoeLayerWeights can say and this backend does not serve answers None (never a wrong bank): inline scales on
    an MXFP4 bank, another expert format, slices shorter than the geometry, more than 256 experts."""
    rng = np.random.default_rng(3)
    E, hidden, inter, k = 3, 64, 32, 2
    gu = [O.quantize_mxfp4((rng.standard_normal(2 * inter * hidden) * 0.02).astype(F), 2 * inter, hidden) for _ in range(E)]
    dn = [O.quantize_mxfp4((rng.standard_normal(hidden * inter) * 0.02).astype(F), hidden, inter) for _ in range(E)]
    rw = rng.standard_normal((E, hidden)).astype(F)
    args = ([g[0] for g in gu], [d[0] for d in dn], [g[1] for g in gu], [d[1] for d in dn], rw, k, hidden, inter)
    ok = be.moe_layer_create(*args)
    assert ok
    be.moe_layer_destroy(ok)
    assert be.moe_layer_create(*args, expert_scales=fmt.MOE_SCALES_INLINE) is None
    assert be.moe_layer_create(*args, expert_data_format=fmt.FMT_Q4_K) is None
    short = ([g[0][:-16] for g in gu],) + args[1:]
    assert be.moe_layer_create(*short) is None
    many = ([gu[0][0]] * 257, [dn[0][0]] * 257, [gu[0][1]] * 257, [dn[0][1]] * 257, np.zeros((257, hidden), F), k, hidden, inter)
    assert be.moe_layer_create(*many) is None


# ------------------------------------------------------------- prefill GEMM
@pytest.mark.parametrize("rows,hidden,seq", [(300, 512, 70), (128, 3840, 128), (1, 256, 1), (257, 768, 33), (520, 8192, 200)])
def test_q4k_gemm_mfma_matches_oracle(be, rows, hidden, seq):
    rng = np.random.default_rng(61 + rows)
    w = (rng.standard_normal((rows, hidden)) * 0.02).astype(F)
    q = O.quantize_q4_k(w)
    xb = O.f32_to_bf16(rng.standard_normal((seq, hidden)).astype(F))          # activations held as bf16 (truncated)
    X = (xb.astype(np.uint32) << 16).view(F).reshape(seq, hidden)
    want = O.q4k_matmul(q, X, rows, hidden, seq)                                # [seq, rows]
    dw, dx, do = be.to_device(q), be.to_device(xb), be.malloc(seq * rows * 4)
    assert be.dev_q4k_gemm(dw, dx, rows, hidden, seq, do)
    be.synchronize()
    got = be.d2h(do, (seq, rows), F)
    assert rel_l2(got, want) < 5e-4          # stated bar 1e-3; f16 roundings of the sub-block scales and weights give ~3e-4
    # every output element (guards tile-edge and layout mistakes)
    assert np.max(np.abs(got - want)) < 2e-3 * (np.abs(want).mean() + 1e-9)
    # the rows' exponents computed once per matrix, then handed in: the same bits
    rexp, do2 = be.malloc(rows * 4 + 64), be.malloc(seq * rows * 4)
    assert be.dev_q4k_row_exponents(dw, rows, hidden, rexp)
    assert be.dev_q4k_gemm_prepared(dw, rexp, dx, rows, hidden, seq, do2)
    be.synchronize()
    assert np.array_equal(be.d2h(do2, (seq, rows), F).view(np.uint32), got.view(np.uint32))
    e = be.d2h(rexp, rows, np.int32)
    hdr = q.reshape(rows, hidden // 256, 144)[:, :, :4].copy().view(np.float16).astype(np.float64)   # d, dmin per super-block
    m = np.maximum(np.abs(hdr[:, :, 0]), np.abs(hdr[:, :, 1]) / 16.0).max(axis=1)
    ok = m > 0
    assert np.all((m[ok] * np.exp2(e[ok].astype(np.float64)) >= 0.5) & (m[ok] * np.exp2(e[ok].astype(np.float64)) < 1.0))
    with pytest.raises(Exception):                                               # the exponents are not optional here
        be.dev_q4k_gemm_prepared(dw, 0, dx, rows, hidden, seq, do2)


def test_q4k_gemm_row_scales_of_any_size_and_uneven_blocks(be):
    """The device tier's GEMM carries each row's scale in an f16 operand behind a per-row exponent: rows whose weights
    differ by twelve orders of magnitude, rows of zeros, and a row with one super-block far larger than the others
    all have to come out to the same relative accuracy (per row, against the oracle)."""
    rng = np.random.default_rng(97)
    rows, hidden, seq = 320, 1024, 48
    w = (rng.standard_normal((rows, hidden)) * 0.02).astype(F)
    w *= (10.0 ** rng.uniform(-8, 4, size=(rows, 1))).astype(F)        # row scales from 1e-8 to 1e4
    w[5] = 0.0                                                          # a row of zeros
    w[17] = 0.0; w[17, 256:512] = (rng.standard_normal(256) * 3.0).astype(F)   # only one super-block holds anything
    w[33, :256] *= F(4096.0)                                            # one super-block 4096 times the others
    w[40, 512:768] *= F(1.0 / 4096.0)
    q = O.quantize_q4_k(w)
    xb = O.f32_to_bf16(rng.standard_normal((seq, hidden)).astype(F))
    X = (xb.astype(np.uint32) << 16).view(F).reshape(seq, hidden)
    want = O.q4k_matmul(q, X, rows, hidden, seq)                        # [seq, rows]
    dw, dx, do = be.to_device(q), be.to_device(xb), be.malloc(seq * rows * 4)
    assert be.dev_q4k_gemm(dw, dx, rows, hidden, seq, do)
    be.synchronize()
    got = be.d2h(do, (seq, rows), F)
    assert np.isfinite(got).all()
    assert np.array_equal(got[:, 5], np.zeros(seq, F))
    for r in range(rows):
        n = np.linalg.norm(want[:, r].astype(np.float64))
        if n > 0:
            assert np.linalg.norm(got[:, r].astype(np.float64) - want[:, r]) / n < 1e-3, r   # the stated bar, row by row
    assert rel_l2(got / np.maximum(np.abs(want).max(axis=0), 1e-30), want / np.maximum(np.abs(want).max(axis=0), 1e-30)) < 5e-4
    # the host tier keeps exact integer sums: the same matrix to ~1e-6 of the oracle per row
    Xf = rng.standard_normal((seq, hidden)).astype(F)
    got_h = be.q4k_matmul(q, Xf, rows, hidden, seq).reshape(seq, rows)
    want_h = O.q4k_matmul(q, Xf, rows, hidden, seq)
    for r in range(rows):
        n = np.linalg.norm(want_h[:, r].astype(np.float64))
        if n > 0:
            assert np.linalg.norm(got_h[:, r].astype(np.float64) - want_h[:, r]) / n < 2e-5, r


def test_q4k_gemm_non_finite_and_lopsided_block_headers(be):
    """The rows' exponents come from max(|d|, |dmin|/16) over a row's super-blocks.  A header that is inf or NaN (a
    corrupt or adversarial block) makes that row's results non-finite in the reference as well (inf * q, inf - inf);
    here it must do the same to THAT row and leave every other row's bits alone.  A row with one large super-block and
    39 tiny ones (their scales fall into f16 subnormals behind the row's exponent) stays within the stated bar."""
    rng = np.random.default_rng(103)
    rows, hidden, seq = 96, 10240, 24
    w = (rng.standard_normal((rows, hidden)) * 0.02).astype(F)
    w[7, 256:] *= F(2.0 ** -13)                             # one super-block 8192 times the other 39
    w[8, :] *= F(2.0 ** -13); w[8, 9 * 256:10 * 256] *= F(2.0 ** 13)
    q = O.quantize_q4_k(w)
    xb = O.f32_to_bf16(rng.standard_normal((seq, hidden)).astype(F))
    X = (xb.astype(np.uint32) << 16).view(F).reshape(seq, hidden)
    dw, dx, do = be.to_device(q), be.to_device(xb), be.malloc(seq * rows * 4)
    assert be.dev_q4k_gemm(dw, dx, rows, hidden, seq, do)
    be.synchronize()
    clean = be.d2h(do, (seq, rows), F)
    want = O.q4k_matmul(q, X, rows, hidden, seq)
    for r in (7, 8):
        assert np.linalg.norm(clean[:, r].astype(np.float64) - want[:, r]) / np.linalg.norm(want[:, r]) < 1e-3, r
    assert rel_l2(clean, want) < 5e-4
    bad = q.reshape(rows, hidden // 256, 144).copy()
    bad[20, 3, 0:2] = np.frombuffer(np.float16(np.inf).tobytes(), np.uint8)        # d = +inf
    bad[41, 17, 2:4] = np.frombuffer(np.float16(np.nan).tobytes(), np.uint8)       # dmin = NaN
    bad[60, 0, 0:2] = np.frombuffer(np.float16(-np.inf).tobytes(), np.uint8)       # d = -inf
    want_bad = O.q4k_matmul(bad.reshape(-1), X, rows, hidden, seq)
    assert not np.isfinite(want_bad[:, [20, 41, 60]]).any()
    be.h2d(dw, bad.reshape(-1))
    assert be.dev_q4k_gemm(dw, dx, rows, hidden, seq, do)
    be.synchronize()
    got = be.d2h(do, (seq, rows), F)
    assert not np.isfinite(got[:, [20, 41, 60]]).any()
    others = [r for r in range(rows) if r not in (20, 41, 60)]
    assert np.array_equal(got[:, others].view(np.uint32), clean[:, others].view(np.uint32))
    # the exact-integer host tier on the same matrix
    got_h = be.q4k_matmul(bad.reshape(-1), X, rows, hidden, seq).reshape(seq, rows)
    assert not np.isfinite(got_h[:, [20, 41, 60]]).any()
    assert rel_l2(got_h[:, others], want[:, others]) < 2e-5


def test_q4k_gemm_activation_ranges_token_by_token(be):
    """The device tier's GEMM scales every token by a power of two into f16.  Tokens far from N(0, 1) — outliers a
    thousand times the rest, all zeros, 1e-30, 1e20, a single non-zero element, alternating signs of equal size — must
    each come out at the stated bar (1e-3 relative L2 per token against the oracle), next to ordinary tokens."""
    rng = np.random.default_rng(101)
    rows, hidden, seq = 272, 2048, 40
    q = O.quantize_q4_k((rng.standard_normal((rows, hidden)) * 0.02).astype(F))
    X = rng.standard_normal((seq, hidden)).astype(F)
    X[1, rng.integers(0, hidden, 5)] *= F(1000.0)          # a few outliers x1000
    X[2] = 0.0                                              # an all-zero token
    X[3] *= F(1e-30)
    X[4] *= F(1e20)
    X[5] = 0.0; X[5, 777] = F(3.0)                          # one-hot
    X[6] = F(0.5) * (1 - 2 * (np.arange(hidden) % 2))       # +-0.5: every sub-block sum is zero
    X[7, :] = F(2.0 ** -120); X[7, 3] = F(2.0 ** -100)      # small with a 2^20 outlier
    X[8] *= F(1e-30); X[8, 100] = F(1e8)                    # 38 orders of magnitude inside one token
    X[9, rng.integers(0, hidden, 40)] *= F(-1000.0)
    xb = O.f32_to_bf16(X)
    Xb = (xb.astype(np.uint32) << 16).view(F).reshape(seq, hidden)
    want = O.q4k_matmul(q, Xb, rows, hidden, seq)           # [seq, rows]
    dw, dx, do = be.to_device(q), be.to_device(xb), be.malloc(seq * rows * 4)
    assert be.dev_q4k_gemm(dw, dx, rows, hidden, seq, do)
    be.synchronize()
    got = be.d2h(do, (seq, rows), F)
    assert np.isfinite(got).all()
    assert np.array_equal(got[2], np.zeros(rows, F))
    for t in range(seq):
        n = np.linalg.norm(want[t].astype(np.float64))
        if n > 0:
            assert np.linalg.norm(got[t].astype(np.float64) - want[t]) / n < 1e-3, t
    # an ordinary token's result does not depend on its neighbours: the same bits as in an all-ordinary batch
    X2 = Xb.copy(); X2[:10] = Xb[10:20]
    do2 = be.malloc(seq * rows * 4)
    assert be.dev_q4k_gemm(dw, be.to_device(O.f32_to_bf16(X2)), rows, hidden, seq, do2)
    be.synchronize()
    assert np.array_equal(be.d2h(do2, (seq, rows), F)[10:].view(np.uint32), got[10:].view(np.uint32))
    # host tier (exact integer sums, f32 activations as two f16 terms): the same tokens, unrounded
    got_h = be.q4k_matmul(q, X, rows, hidden, seq).reshape(seq, rows)
    want_h = O.q4k_matmul(q, X, rows, hidden, seq)
    for t in range(seq):
        n = np.linalg.norm(want_h[t].astype(np.float64))
        if n > 0:
            assert np.linalg.norm(got_h[t].astype(np.float64) - want_h[t]) / n < 1e-3, t


def test_q4k_matmul_host_tier_uses_gemm_for_prefill_shapes(be):
    rng = np.random.default_rng(67)
    rows, hidden, seq = 200, 1024, 40
    q = O.quantize_q4_k((rng.standard_normal((rows, hidden)) * 0.02).astype(F))
    X = rng.standard_normal((seq, hidden)).astype(F)                            # full f32 activations: two bf16 terms
    got = be.q4k_matmul(q, X, rows, hidden, seq)
    want = O.q4k_matmul(q, X, rows, hidden, seq).reshape(-1)
    assert rel_l2(got, want) < 1e-4
    # rows of the matmul equal the stacked matvec (quantize_q4_0_tests.rs:202-238, tol 1e-4)
    mv = be.q4k_matvec(q, X[7], rows, hidden)
    assert np.max(np.abs(got.reshape(seq, rows)[7] - mv)) < 1e-4


def test_gate_walk_over_layers_equals_per_layer_calls(be, fmt):
    rng = np.random.default_rng(71)
    L, n, hidden, k, batch = 3, 1000, 512, 64, 2
    gates_h = [O.f32_to_bf16((rng.standard_normal((n, hidden)) * 0.02).astype(F)) for _ in range(L)]
    X = rng.standard_normal((L, batch, hidden)).astype(F)
    gates = [be.to_device(g) for g in gates_h]
    x = be.to_device(X)
    scores, idx, val, cnt = be.malloc(L * batch * n * 4), be.malloc(L * batch * k * 4), be.malloc(L * batch * k * 4), be.malloc(L * batch * 4)
    assert be.dev_gate_walk(fmt.FMT_BF16, gates, x, batch * hidden, batch, n, hidden, k, scores, idx, val, cnt)
    be.synchronize()
    gi, gv = be.d2h(idx, (L, batch, k), np.uint32), be.d2h(val, (L, batch, k), F)
    assert (be.d2h(cnt, L * batch, np.uint32) == k).all()
    for l in range(L):
        for b in range(batch):
            ref = O.bf16_gemv(gates_h[l], X[l, b], n, hidden)
            check_hits([(int(i), float(v)) for i, v in zip(gi[l, b], gv[l, b])], ref, k)
    # shared residuals (stride 0) == per-layer host-tier calls
    assert be.dev_gate_walk(fmt.FMT_BF16, gates, x, 0, batch, n, hidden, k, scores, idx, val)
    be.synchronize()
    gi0 = be.d2h(idx, (L, batch, k), np.uint32)
    for l in range(L):
        hits = be.gate_knn_batch_hits(fmt.FMT_BF16, gates_h[l], X[0], n, hidden, k)
        for b in range(batch):
            assert [i for i, _ in hits[b]] == [int(v) for v in gi0[l, b]]


def test_dev_gate_knn_reports_counts_and_nan(be, fmt):
    """Device tier: hits per position come back through count_out (top_k above the feature count leaves the tail of a row
    unwritten, exactly count entries are valid), and a NaN score — a panic in the reference (gate_knn/mod.rs:84),
    LARQL_E_NAN on the host tier — raises a flag that larql_hip_dev_take_nan_flag reads and clears."""
    rng = np.random.default_rng(73)
    n, hidden, k, batch = 40, 256, 64, 3
    w = (rng.standard_normal((n, hidden)) * 0.02).astype(F)
    X = rng.standard_normal((batch, hidden)).astype(F)
    g, x = be.to_device(w), be.to_device(X)
    sc, idx, val, cnt = be.malloc(batch * n * 4), be.malloc(batch * k * 4), be.malloc(batch * k * 4), be.malloc(batch * 4)
    assert be.dev_gate_knn(fmt.FMT_F32, g, x, batch, n, hidden, k, sc, idx, val, cnt)
    assert be.dev_take_nan_flag() is False
    counts = be.d2h(cnt, batch, np.uint32)
    assert list(counts) == [n] * batch                                      # K > N: all features, as top_k_by_abs
    gi, gv = be.d2h(idx, (batch, k), np.uint32), be.d2h(val, (batch, k), F)
    for b in range(batch):
        check_hits([(int(i), float(v)) for i, v in zip(gi[b, :n], gv[b, :n])], O.f32_gemv(w, X[b], n, hidden), k)
    # one NaN activation poisons every score of position 1
    X[1, 5] = np.nan
    be.h2d(x, X)
    assert be.dev_gate_knn(fmt.FMT_F32, g, x, batch, n, hidden, k, sc, idx, val, cnt)
    assert be.dev_take_nan_flag() is True and be.dev_take_nan_flag() is False   # read once, then clear
    # the flag stays up until it is taken: a clean call after the poisoned one does not lower it
    assert be.dev_gate_knn(fmt.FMT_F32, g, x, batch, n, hidden, k, sc, idx, val, cnt)
    X[1, 5] = 0.0
    be.h2d(x, X)
    assert be.dev_gate_knn(fmt.FMT_F32, g, x, batch, n, hidden, k, sc, idx, val)  # (count_out is optional)
    assert be.dev_take_nan_flag() is True and be.dev_take_nan_flag() is False
    assert be.dev_gate_knn(fmt.FMT_F32, g, x, batch, n, hidden, k, sc, idx, val)
    assert be.dev_take_nan_flag() is False
    with pytest.raises(Exception):                                               # host tier: the error code
        Xn = X.copy(); Xn[0, 0] = np.nan
        be.gate_knn_batch_hits(fmt.FMT_F32, w, Xn, n, hidden, k)


def test_one_context_from_eight_threads(be, fmt):
    """The trait is Send + Sync and its callers are rayon workers (gate_store.rs:40-45): one context driven from eight
    threads at once (ctypes releases the GIL during a call), every result checked.  Calls are serialised inside the
    library; what must hold is that no call sees another call's staging buffers or error text."""
    import threading
    rng = np.random.default_rng(79)
    cases = []
    for i in range(8):
        rows, cols = 64 + 37 * i, 256 * (1 + i % 4)
        w = (rng.standard_normal((rows, cols)) * 0.02).astype(F)
        x = rng.standard_normal(cols).astype(F)
        q = O.quantize_q4_k(w)
        q8 = O.quantize_q8_0(w)
        cases.append((rows, cols, q, q8, x, O.q4k_matvec(q, x, rows, cols), O.q8_0_gemv(q8, x, rows, cols), O.top_k_by_abs(O.q4k_matvec(q, x, rows, cols), 8)))
    errors = []
    start = threading.Barrier(8)

    def work(i):
        rows, cols, q, q8, x, want4, want8, hits = cases[i]
        try:
            start.wait()
            for rep in range(25):
                got = be.q4k_matvec(q, x, rows, cols)
                assert got is not None and rel_l2(got, want4) < TOL
                got8 = be.q8_0_gemv(q8, x, rows, cols)
                assert rel_l2(got8, want8) < TOL
                assert be.q4k_matvec(q[:-1], x, rows, cols) is None            # a refusal in the middle of the others' calls
                h = be.gate_knn(fmt.FMT_Q4_K, q, x, rows, cols, 8)
                assert sorted(j for j, _ in h) == sorted(j for j, _ in hits)
        except Exception as e:  # noqa: BLE001 - collected and re-raised in the main thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    assert not any(t.is_alive() for t in threads)


@pytest.mark.parametrize("n,k", [(10240, 256), (10240, 2048), (10240, 10240), (3000, 65), (3000, 16384), (100, 1000), (70, 65), (16384, 16384)])
def test_top_k_above_64(be, fmt, n, k):
    """top_k_by_abs takes any K (gate_knn/mod.rs:50-108) and WalkFfn's default is every feature
    (larql-inference/src/vindex/walk_ffn/mod.rs:186-190): K = 256, 2048, N and K > N against the oracle's heap —
    same index set, |score| descending, ties to the lower index."""
    rng = np.random.default_rng(n + k)
    hidden = 256
    w = (rng.standard_normal((n, hidden)) * 0.02).astype(F)
    w[5] = w[9]; w[17] = -w[9]                       # three equal |scores|
    x = rng.standard_normal(hidden).astype(F)
    hits = be.gate_knn(fmt.FMT_F32, w, x, n, hidden, k)
    scores = be.gate_scores_batch(fmt.FMT_F32, w, x.reshape(1, -1), n, hidden).reshape(-1)
    m = min(k, n)
    assert hits is not None and len(hits) == m
    idx = np.array([i for i, _ in hits]); val = np.array([v for _, v in hits], F)
    assert np.array_equal(val.view(np.uint32), scores[idx].view(np.uint32))
    a = np.abs(val)
    assert np.all(a[:-1] >= a[1:])
    tie = (a[:-1] == a[1:])
    assert np.all(idx[:-1][tie] < idx[1:][tie])                                # equal |score|: the lower index first
    want = O.top_k_by_abs(scores, k)
    assert sorted(idx.tolist()) == sorted(i for i, _ in want) or abs(abs(want[-1][1]) - a[-1]) <= 1e-5
    if m == n:
        assert sorted(idx.tolist()) == list(range(n))


def test_top_k_above_64_limits_and_by_value(be, fmt):
    rng = np.random.default_rng(3)
    rows, hidden = 5000, 512
    w = (rng.standard_normal((rows, hidden)) * 0.02).astype(F)
    x = rng.standard_normal(hidden).astype(F)
    q = O.quantize_q4_k(w)
    hits = be.q4k_matvec_topk(q, x, rows, hidden, 300)                          # by value, descending
    scores = be.q4k_matvec(q, x, rows, hidden)
    want = O.top_k_sorted(scores, 300)
    assert [i for i, _ in hits] == [i for i, _ in want]
    assert be.gate_knn(fmt.FMT_F32, w, x, rows, hidden, 16385) is None           # above the kernel's capacity: the caller's fallback
    assert be.q4k_matvec_topk(q, x, rows, hidden, 16385) is None


@pytest.mark.parametrize("seed,scale", [(0, 0.02), (1, 1.0), (2, 1e-4), (3, 30.0)])
def test_device_q6k_encoder_is_bit_exact(be, seed, scale):
    """quantize_q6_k (q4_common/quantize.rs:198-276) on the device, byte for byte, incl. all-zero and constant blocks."""
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(256 * 333) * scale).astype(F)
    x[:256] = 0
    x[256:512] = F(0.37 * scale)
    x[512:528] = 0                      # a zero sub-block: scale 0, reciprocal 0
    src, dst = be.to_device(x), be.malloc(x.size // 256 * 210)
    assert be.dev_quantize_q6_k(src, x.size, dst)
    assert np.array_equal(be.d2h(dst, x.size // 256 * 210, np.uint8), O.quantize_q6_k(x))
    assert not be.dev_quantize_q6_k(src, 255, dst)


def test_q8_0_gemv_topk_keeps_the_scores_on_the_device(be):
    """lm_head KNN over a ggml Q8_0 head (lm_head/knn.rs:126-185, top_k_sorted :315-386): by value, descending."""
    rng = np.random.default_rng(41)
    n, k = 5003, 512
    w = (rng.standard_normal((n, k)) * 0.02).astype(F)
    x = rng.standard_normal(k).astype(F)
    q = O.quantize_q8_0(w)
    scores = be.q8_0_gemv(q, x, n, k)
    for top in (1, 8, 64, 500):
        hits = be.q8_0_gemv_topk(q, x, n, k, top)
        want = O.top_k_sorted(scores, top)
        assert [i for i, _ in hits] == [i for i, _ in want]
        assert np.array_equal(np.array([v for _, v in hits], F).view(np.uint32), scores[[i for i, _ in hits]].view(np.uint32))
    assert be.q8_0_gemv_topk(q[:-1], x, n, k, 8) is None and be.q8_0_gemv_topk(q, x, n, k, 0) is None
    assert be.q8_0_gemv_topk(q, x[:-1], n, k, 8) is None


def test_quant_matvec_q8_input_dispatch(be, fmt):
    """QuantMatVec::quant_matvec_q8_input (quant_matvec.rs:100-151)."""
    rows, hidden = 257, 1024
    w, x = weights(23, rows, hidden)
    q8, sc = O.quantize_to_q8(x)
    q4 = O.quantize_q4_0(w)
    a = be.quant_matvec_q8_input(fmt.FMT_Q4_0, q4, q8, sc, rows, hidden)
    assert np.array_equal(a.view(np.uint32), be.q4_matvec(q4, q8, sc, rows, hidden).view(np.uint32))
    xd = O.dequantise_q8(q8, sc)
    for f, q in ((fmt.FMT_Q4_K, O.quantize_q4_k(w)), (fmt.FMT_Q6_K, O.quantize_q6_k(w))):
        got = be.quant_matvec_q8_input(f, q, q8, sc, rows, hidden)
        assert np.array_equal(got.view(np.uint32), be.quant_matvec(f, q, xd, rows, hidden).view(np.uint32))
        want = O.q4k_matvec(q, xd, rows, hidden) if f == fmt.FMT_Q4_K else O.q6k_matvec(q, xd, rows, hidden)
        assert rel_l2(got, want) < TOL
    for f in (fmt.FMT_Q8_0, fmt.FMT_Q5_K, fmt.FMT_I2S, fmt.FMT_MXFP4, fmt.FMT_BF16, fmt.FMT_F32):
        assert be.quant_matvec_q8_input(f, q4, q8, sc, rows, hidden) is None
    assert be.quant_matvec_q8_input(fmt.FMT_Q4_K, O.quantize_q4_k(w), q8, sc[:-1], rows, hidden) is None   # a scale short


@pytest.mark.parametrize("half", ["bf16", "f16"])
def test_dense_gemv_multi_is_one_submission_of_the_single_calls(be, half):
    """MatMul::{bf16,f16}_gemv_multi (backend/matmul.rs:151-194): results in argument order, bit-identical to the
    sequential force gemvs; an empty list is Some(vec![]); one bad matrix refuses the whole batch."""
    rng = np.random.default_rng(43)
    k = 640
    x = rng.standard_normal(k).astype(F)
    shapes = [300, 17, 1024, 5, 64, 999, 128, 256, 33, 700, 2]          # eleven matrices: two launches' worth
    mats = []
    for n in shapes:
        w = (rng.standard_normal((n, k)) * 0.05).astype(F)
        mats.append((O.f32_to_bf16(w) if half == "bf16" else w.astype(np.float16), n, k))
    multi = getattr(be, f"{half}_gemv_multi")
    single = getattr(be, f"{half}_gemv_force")
    before = be.submission_clock()["submissions"]
    outs = multi(mats, x)
    assert be.submission_clock()["submissions"] - before == 2
    assert outs is not None and len(outs) == len(shapes)
    for (w, n, _), o in zip(mats, outs):
        assert np.array_equal(o.view(np.uint32), single(w, x, n, k).view(np.uint32))
    assert multi([], x) == []
    bad = list(mats[:3]) + [(mats[3][0][:-1], mats[3][1], k)]
    assert multi(bad, x) is None
    assert multi([(mats[0][0], shapes[0], k - 64)], x) is None            # k must equal x.len()
