"""GPU parity on data the reference itself holds, and on the adversarial encoder
blocks whose expected bytes come from exact arithmetic — no weight byte and no
expected value in this file comes out of the CPU checker's encoders.

  * llama.cpp's golden q4_K / q8_0 / q6_K bytes with their decoded bit patterns
    (larql-vindex/src/format/vindex3/represent/fixtures/ggml_kquant_golden.json,
    held under tests/golden/): the HIP matvecs on those bytes against
    sum(golden_decoded * x) in f64, the reference's own check
    (larql-vindex/.../kquant_direct_tests.rs:127-166; its CPU Q8_0 kernel is
    bit-exact with the sequential f32 sum, a GPU reduction tree is not, so all
    three formats are held to the 5e-6 relative bound the reference states for
    the K-quants).
  * ggml's golden Q8_0 encoder blocks (larql-models q8_0_ggml_golden.rs) and
    tests/golden/encoder_kats.json through the device encoders, byte for byte.
"""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
F = np.float32
GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def ggml_golden():
    d = json.load(open(os.path.join(GOLD, "ggml_kquant_golden.json")))
    out = {}
    for c in d["cases"]:
        out[c["encoding"]] = (np.frombuffer(bytes.fromhex(c["quantised_hex"]), np.uint8).copy(),
                              np.array(c["dequantised_bits"], np.uint32).view(F).copy(), c["elements"])
    return out


def rel_err(got, exact):
    return float(np.max(np.abs(got.astype(np.float64) - exact) / np.maximum(np.abs(exact), 1e-6)))


@pytest.mark.parametrize("enc,block_elems,block_bytes", [("q4_K", 256, 144), ("q6_K", 256, 210), ("q8_0", 32, 34)])
def test_matvecs_on_llama_cpp_golden_bytes(be, ggml_golden, enc, block_elems, block_bytes):
    import larql_amd as fmt
    raw, decoded, n = ggml_golden[enc]
    assert raw.size == n // block_elems * block_bytes
    rng = np.random.default_rng(3)
    # the same bytes read as matrices of every row length the format and the kernels allow
    ks = [k for k in (64, 128, 256, 512) if k % block_elems == 0 and n % k == 0]
    assert ks
    for k in ks:
        rows = n // k
        for trial in range(3):
            x = (rng.standard_normal(k) * (1.0, 30.0, 1e-3)[trial]).astype(F)
            exact = decoded.reshape(rows, k).astype(np.float64) @ x.astype(np.float64)
            if enc == "q4_K":
                got = be.q4k_matvec(raw, x, rows, k)
                via = be.quant_matvec(fmt.FMT_Q4_K, raw, x, rows, k)
            elif enc == "q6_K":
                got = be.q6k_matvec(raw, x, rows, k)
                via = be.quant_matvec(fmt.FMT_Q6_K, raw, x, rows, k)
            else:
                got = be.q8_0_gemv(raw, x, rows, k)
                via = got
            assert got is not None and got.shape == (rows,), (enc, k)
            scale = np.abs(decoded.reshape(rows, k).astype(np.float64)) @ np.abs(x.astype(np.float64))
            # relative to the row's own magnitude sum |w||x| (a row whose terms cancel has no relative precision to keep)
            assert float(np.max(np.abs(got - exact) / scale)) < 5e-6, (enc, k, trial)
            assert np.array_equal(via.view(np.uint32), got.view(np.uint32))


def test_q4k_golden_bytes_through_the_other_q4k_entry_points(be, ggml_golden):
    raw, decoded, n = ggml_golden["q4_K"]
    rows, k = 2, 256
    rng = np.random.default_rng(9)
    x = rng.standard_normal(k).astype(F)
    w = decoded.reshape(rows, k).astype(np.float64)
    single = be.q4k_matvec(raw, x, rows, k)
    a, b = be.q4k_dual_matvec(raw, raw, x, rows, k)
    assert np.array_equal(a.view(np.uint32), single.view(np.uint32)) and np.array_equal(b.view(np.uint32), single.view(np.uint32))
    xs = rng.standard_normal((3, k)).astype(F)
    mm = be.q4k_matmul(raw, xs, rows, k, 3)
    assert mm is not None and rel_err(np.asarray(mm).reshape(3, rows), xs.astype(np.float64) @ w.T) < 2e-5
    hits = be.q4k_matvec_topk(raw, x, rows, k, 2)
    order = np.argsort(-(w @ x.astype(np.float64)))
    assert [i for i, _ in hits] == list(order)


def _device_encode(be, name, x, out_bytes, *extra):
    src = be.to_device(x)
    dst = be.malloc(out_bytes)
    try:
        assert getattr(be, name)(src, *extra, dst)
        return be.d2h(dst, (out_bytes,), np.uint8)
    finally:
        be.free(src)
        be.free(dst)


KATS = json.load(open(os.path.join(GOLD, "encoder_kats.json")))["cases"]


def kat_inputs(name):
    return np.array(KATS[name]["input_bits"], np.uint32).view(F).copy()


@pytest.mark.parametrize("name", ["q4k_exact_halves", "q4k_f32_header", "q4k_small"])
def test_device_q4k_encoder_on_exact_arithmetic_blocks(be, name):
    x = kat_inputs(name)
    got = _device_encode(be, "dev_quantize_q4_k", x, x.size // 256 * 144, x.size)
    assert got.tobytes().hex() == KATS[name]["hex"]


def test_device_q4_0_and_q8_0_encoders_on_exact_arithmetic_blocks(be):
    x = kat_inputs("q4_0")
    assert _device_encode(be, "dev_quantize_q4_0", x, x.size // 32 * 18, x.size).tobytes().hex() == KATS["q4_0"]["hex"]
    x = kat_inputs("q8_0")
    assert _device_encode(be, "dev_quantize_q8_0", x, x.size // 32 * 34, x.size).tobytes().hex() == KATS["q8_0"]["hex"]


def test_device_q8_0_encoder_on_the_ggml_golden_blocks(be):
    d = json.load(open(os.path.join(GOLD, "q8_0_ggml_golden.json")))
    xs = np.concatenate([np.array(c["input_bits"], np.uint32).view(F) for c in d["cases"]])
    want = "".join(c["block_hex"] for c in d["cases"])
    assert _device_encode(be, "dev_quantize_q8_0", xs, xs.size // 32 * 34, xs.size).tobytes().hex() == want


def test_device_to_q8_and_q8k_encoders_on_exact_arithmetic_blocks(be):
    case = KATS["to_q8"]
    x = kat_inputs("to_q8")
    src, q8, sc = be.to_device(x), be.malloc(x.size), be.malloc(x.size // 32 * 4)
    try:
        assert be.dev_quantize_to_q8(src, x.size, q8, sc)
        assert list(map(int, be.d2h(q8, (x.size,), np.int8))) == case["codes"]
        assert list(map(int, be.d2h(sc, (x.size // 32,), np.uint32))) == case["scale_bits"]
    finally:
        for p in (src, q8, sc):
            be.free(p)
    case = KATS["q8k"]
    x = kat_inputs("q8k")
    qs, d, sums = be.quantize_x_to_q8k(x)
    assert list(map(int, qs)) == case["codes"]
    assert list(map(int, np.asarray(d, F).view(np.uint32))) == case["d_bits"]
    assert list(map(int, sums)) == case["sums"]


def test_device_mxfp4_encoder_on_exact_arithmetic_groups(be):
    case = KATS["mxfp4"]
    x = kat_inputs("mxfp4")
    rows, k = case["rows"], case["k"]
    src, pk, sc = be.to_device(x), be.malloc(rows * k // 2), be.malloc(rows * k // 32)
    try:
        assert be.dev_quantize_mxfp4(src, rows, k, pk, sc)
        assert be.d2h(pk, (rows * k // 2,), np.uint8).tobytes().hex() == case["packed_hex"]
        assert be.d2h(sc, (rows * k // 32,), np.uint8).tobytes().hex() == case["scales_hex"]
    finally:
        for p in (src, pk, sc):
            be.free(p)


@pytest.mark.parametrize("name", ["q6k_exact_halves", "q6k_f32_header"])
def test_device_q6k_encoder_on_exact_arithmetic_blocks(be, name):
    x = kat_inputs(name)
    got = _device_encode(be, "dev_quantize_q6_k", x, x.size // 256 * 210, x.size)
    assert got.tobytes().hex() == KATS[name]["hex"]
