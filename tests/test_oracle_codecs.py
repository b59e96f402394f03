"""Pins the CPU checker's codecs: f16/bf16 conversions, Q4_K / Q8_0 / MXFP4
decoders and encoders.  Each test names what fixes the expected value:
a reference-held golden vector, IEEE arithmetic via numpy, a closed form, or
the independent numpy restatement."""
import json
import os

import numpy as np
import pytest

import np_restatement as npr
import oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")
F = np.float32


def bits(a):
    return np.asarray(a, F).view(np.uint32)


# ---------------------------------------------------------------- f16 / bf16
def test_f16_to_f32_all_65536_inputs_match_ieee():
    # IEEE half via numpy float16; the reference's own exhaustive test is
    # q4_common/tests/f16_subnormal_regression_battery_2026_06.rs:13-34.
    allb = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = allb.view(np.float16).astype(F)
    got = np.array([O.f16_to_f32(int(b)) for b in allb], F)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(bits(got[~nan]), bits(want[~nan]))


def test_f16_pinned_subnormals():
    # f16_subnormal_regression_battery: smallest subnormal 2^-24, largest 1023*2^-24
    assert O.f16_to_f32(0x0001) == 2.0 ** -24
    assert O.f16_to_f32(0x03FF) == 1023 * 2.0 ** -24
    assert O.f16_to_f32(0x8001) == -(2.0 ** -24)
    assert O.f16_to_f32(0x0400) == 2.0 ** -14
    assert O.f16_to_f32(0x3C00) == 1.0 and O.f16_to_f32(0xC000) == -2.0


def test_f32_to_f16_nearest_reference_table():
    # larql-models/src/quant/half.rs:160-200
    mn, ms = 2.0 ** -14, 2.0 ** -24
    table = [(0.0, 0x0000), (-0.0, 0x8000), (1.0, 0x3C00), (-2.0, 0xC000), (mn, 0x0400), (ms, 0x0001),
             (-ms, 0x8001), (1023.0 * ms, 0x03FF), (1.0 + 2.0 ** -11, 0x3C00), (1.0 + 3.0 * 2.0 ** -11, 0x3C02),
             (1022.5 * ms, 0x03FE), (1023.5 * ms, 0x0400), (0.5 * ms, 0x0000), (1.5 * ms, 0x0002),
             (float(np.array([np.array(0.5 * ms, F).view(np.uint32) + 1], np.uint32).view(F)[0]), 0x0001),
             (0.25 * ms, 0x0000), (1e-30, 0x0000), (float(np.array([1], np.uint32).view(F)[0]), 0x0000),
             (2.0 - 2.0 ** -12, 0x4000), (65504.0, 0x7BFF), (65519.996, 0x7BFF), (65520.0, 0x7C00),
             (65536.0, 0x7C00), (70000.0, 0x7C00), (1e30, 0x7C00), (float("inf"), 0x7C00), (float("-inf"), 0xFC00)]
    for v, want in table:
        assert O.f32_to_f16_nearest(v) == want, v
    assert O.f32_to_f16_nearest(float(np.array([0x7F800001], np.uint32).view(F)[0])) == 0x7E00


def test_f32_to_f16_nearest_matches_ieee_on_a_bit_sweep():
    rng = np.random.default_rng(11)
    # exponents around the f16 range, random mantissas; numpy's cast is IEEE RNE
    e = rng.integers(127 - 30, 127 + 18, size=40000).astype(np.uint32)
    m = rng.integers(0, 1 << 23, size=40000).astype(np.uint32)
    s = rng.integers(0, 2, size=40000).astype(np.uint32)
    v = ((s << 31) | (e << 23) | m).view(F)
    want = npr.f32_to_f16_nearest(v)
    got = np.array([O.f32_to_f16_nearest(float(x)) for x in v], np.uint16)
    assert np.array_equal(got, want)
    # and every f16 round-trips (half.rs nearest_round_trips_every_f16_value)
    allb = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = allb.view(np.float16).astype(F)
    ok = ~np.isnan(f)
    back = np.array([O.f32_to_f16_nearest(float(x)) for x in f[ok]], np.uint16)
    assert np.array_equal(back, allb[ok])


def test_f32_to_f16_trunc_closed_forms():
    # q4_common/f16.rs:10-41: normals drop the low 13 mantissa bits (toward zero),
    # subnormals shift with the implicit one, below 2^-24 gives signed zero.
    assert O.f32_to_f16_trunc(1.0) == 0x3C00
    assert O.f32_to_f16_trunc(1.0 + 2.0 ** -10 - 2.0 ** -20) == 0x3C00       # truncates, not rounds
    assert O.f32_to_f16_trunc(-(1.0 + 2.0 ** -10)) == 0xBC01
    assert O.f32_to_f16_trunc(2.0 ** -14) == 0x0400
    assert O.f32_to_f16_trunc(2.0 ** -15) == 0x0200
    assert O.f32_to_f16_trunc(1.75 * 2.0 ** -15) == 0x0380
    assert O.f32_to_f16_trunc(2.0 ** -24) == 0x0001
    assert O.f32_to_f16_trunc(1.99 * 2.0 ** -24) == 0x0001                    # truncation
    assert O.f32_to_f16_trunc(2.0 ** -25) == 0x0000
    assert O.f32_to_f16_trunc(-(2.0 ** -25)) == 0x8000
    assert O.f32_to_f16_trunc(70000.0) == 0x7C00 and O.f32_to_f16_trunc(float("inf")) == 0x7C00
    assert O.f32_to_f16_trunc(0.0) == 0 and O.f32_to_f16_trunc(-0.0) == 0x8000
    # against the independent numpy statement and against "IEEE round toward zero"
    rng = np.random.default_rng(5)
    v = (rng.standard_normal(20000) * np.exp(rng.uniform(-20, 12, 20000))).astype(F)
    got = np.array([O.f32_to_f16_trunc(float(x)) for x in v], np.uint16)
    assert np.array_equal(got, npr.f32_to_f16_trunc(v))
    dec = got.view(np.float16).astype(np.float64)
    fin = np.isfinite(dec)
    assert np.all(np.abs(dec[fin]) <= np.abs(v[fin].astype(np.float64)))      # never rounds away from zero
    nxt = (got[fin] + 1).view(np.float16).astype(np.float64)                  # next f16 in magnitude
    assert np.all(np.abs(nxt) > np.abs(v[fin].astype(np.float64)))


def test_f16_flush_variant():
    # quantize_q4_0's inline conversion: below the normal range -> signed zero
    assert O.f32_to_f16_flush(2.0 ** -15) == 0 and O.f32_to_f16_flush(-(2.0 ** -15)) == 0x8000
    assert O.f32_to_f16_flush(1.0) == 0x3C00 and O.f32_to_f16_flush(2.0 ** -14) == 0x0400


def test_bf16_is_truncation():
    v = np.array([0.0, 1.0, -1.0, 0.5, 100.0, -42.0, 3.1415927, 1e-40], F)
    assert np.array_equal(O.f32_to_bf16(v), (v.view(np.uint32) >> 16).astype(np.uint16))


# -------------------------------------------------- reference-held ggml golden
@pytest.fixture(scope="module")
def ggml_golden():
    d = json.load(open(os.path.join(GOLD, "ggml_kquant_golden.json")))
    d["input"] = np.array(d["input_bits"], np.uint32).view(F)
    return d


@pytest.mark.parametrize("enc", ["q4_K", "q8_0", "q6_K"])
def test_decoders_bit_exact_on_llama_cpp_golden(ggml_golden, enc):
    case = next(c for c in ggml_golden["cases"] if c["encoding"] == enc)
    raw = np.frombuffer(bytes.fromhex(case["quantised_hex"]), np.uint8)
    want = np.array(case["dequantised_bits"], np.uint32)
    n = case["elements"]
    dec = {"q4_K": (O.dequantize_q4_k, npr.dequantize_q4_k), "q8_0": (O.dequantize_q8_0, npr.dequantize_q8_0),
           "q6_K": (O.dequantize_q6_k, npr.dequantize_q6_k)}[enc]
    assert np.array_equal(bits(dec[0](raw, n)), want)
    assert np.array_equal(bits(dec[1](raw, n)), want)


def test_q6k_matvec_on_golden_bytes_matches_decode(ggml_golden):
    # the kernel must equal decode-then-dot on llama.cpp's own bytes (f64 reference, 5e-6 as for Q4_K)
    case = next(c for c in ggml_golden["cases"] if c["encoding"] == "q6_K")
    raw = np.frombuffer(bytes.fromhex(case["quantised_hex"]), np.uint8)
    w = np.array(case["dequantised_bits"], np.uint32).view(F).reshape(2, 256)
    x = np.random.default_rng(5).standard_normal(256).astype(F)
    got = O.q6k_matvec(raw, x, 2, 256)
    exact = w.astype(np.float64) @ x.astype(np.float64)
    assert np.max(np.abs(got - exact) / np.maximum(np.abs(exact), 1e-6)) < 5e-6
    assert O.q6k_matvec(raw[:-1], x, 2, 256) is None and O.q6k_matvec(raw, x[:-1], 2, 256) is None


def test_q6k_encoder_closed_forms_and_second_restatement():
    # all-zero block -> 210 zero bytes except the biased codes (q = 0 -> 32: low nibble 0, high bits 2)
    z = O.quantize_q6_k(np.zeros(256, F))
    assert z.size == 210 and not z[:128].any() and (z[128:192] == 0xAA).all() and not z[192:].any()
    assert not O.dequantize_q6_k(z, 256).any()
    # constant block c > 0: amax = c, d = c/3937, every sub-scale 127, every q = round(c / (d*127)) = 31
    c = F(0.75)
    b = O.quantize_q6_k(np.full(256, c, F))
    d = F(c / F(31.0 * 127.0))
    assert (b[192:208].view(np.int8) == 127).all()
    assert (int(b[208]) | (int(b[209]) << 8)) == int(npr.f32_to_f16_trunc(np.array([d], F))[0])
    assert (b[:128] == 0xFF).all() and (b[128:192] == 0xFF).all()          # 31 + 32 = 63 = 0b111111 everywhere
    # negative constant: q = -31 -> 1: low nibble 1, high bits 0
    n = O.quantize_q6_k(np.full(256, -c, F))
    assert (n[:128] == 0x11).all() and not n[128:192].any()
    # one sub-block 4x larger than the rest: its scale saturates at 127, the others land near 32
    rng = np.random.default_rng(9)
    x = (rng.standard_normal(256) * 0.01).astype(F)
    x[48:64] *= 4
    e = O.quantize_q6_k(x)
    sc = e[192:208].view(np.int8)
    assert sc.max() == sc[np.abs(x.reshape(16, 16)).max(1).argmax()] and sc.max() >= 100
    # two independent restatements agree byte for byte, and the round trip is within half a level
    for seed, scale in ((1, 0.02), (2, 1.0), (3, 30.0)):
        w = (np.random.default_rng(seed).standard_normal(256 * 24) * scale).astype(F)
        q = O.quantize_q6_k(w)
        assert np.array_equal(q, npr.quantize_q6_k(w))
        dq = O.dequantize_q6_k(q, w.size)
        assert np.array_equal(bits(dq), bits(npr.dequantize_q6_k(q, w.size)))
        # half a level of the sub-block (level = d*scale ~ sub_max/31, scale rounded to an integer: +- d/2),
        # plus what the clamp at +-31 levels can cut off when the scale rounds down (31 * d/2)
        d = np.repeat(np.abs(w.reshape(-1, 256)).max(1) / (31.0 * 127.0), 256)
        sub_max = np.repeat(np.abs(w.reshape(-1, 16)).max(1), 16)
        assert np.all(np.abs(dq - w) <= 0.5 * sub_max / 31.0 + 16.0 * d + 1e-12)


def test_direct_gemv_on_golden_bytes_matches_decode(ggml_golden):
    # kquant_direct_tests.rs:127-166: Q8_0 exact, Q4_K relative < 5e-6
    rng = np.random.default_rng(3)
    for enc, rows, k in (("q8_0", 2, 256), ("q4_K", 2, 256)):
        case = next(c for c in ggml_golden["cases"] if c["encoding"] == enc)
        raw = np.frombuffer(bytes.fromhex(case["quantised_hex"]), np.uint8)
        w = np.array(case["dequantised_bits"], np.uint32).view(F).reshape(rows, k)
        x = rng.standard_normal(k).astype(F)
        want = np.zeros(rows, F)
        for r in range(rows):
            acc = F(0)
            for c in range(k):
                acc = F(acc + F(w[r, c] * x[c]))
            want[r] = acc
        if enc == "q8_0":
            got = O.q8_0_gemv(raw, x, rows, k)
            assert np.array_equal(bits(got), bits(want))
        else:
            got = O.q4k_matvec(raw, x, rows, k)
            exact = w.astype(np.float64) @ x.astype(np.float64)
            assert np.max(np.abs(got - exact) / np.maximum(np.abs(exact), 1e-6)) < 5e-6


def test_q8_0_encoder_bytes_match_ggml_golden():
    d = json.load(open(os.path.join(GOLD, "q8_0_ggml_golden.json")))
    assert len(d["cases"]) >= 20
    for c in d["cases"]:
        x = np.array(c["input_bits"], np.uint32).view(F)
        assert O.quantize_q8_0(x).tobytes().hex() == c["block_hex"], c["name"]
        assert npr.quantize_q8_0(x).tobytes().hex() == c["block_hex"], c["name"]


# ----------------------------------------------------------------- Q4_K encoder
def test_q4k_encoder_closed_forms():
    z = O.quantize_q4_k(np.zeros(256, F))
    assert z.size == 144 and not z.any()
    # constant c>0: mins forced to 0 -> d=c/945, dmin=0, every scale 63, every nibble 15
    c = F(0.25)
    b = O.quantize_q4_k(np.full(256, c, F))
    assert (int(b[0]) | (int(b[1]) << 8)) == O.f32_to_f16_trunc(float(c / F(945.0)))
    assert b[2] == 0 and b[3] == 0
    assert np.array_equal(b[4:8], np.full(4, 63 | (3 << 6), np.uint8))       # scales 0..3, top bits of 4..7
    assert np.array_equal(b[8:12], np.zeros(4, np.uint8))                     # mins 0
    assert np.array_equal(b[12:16], np.full(4, 63 & 0x0F, np.uint8))
    assert np.all(b[16:] == 0xFF)
    # constant c<0: d=|c|/945, dmin=|c|/63, q_min=63, q_scale=63, nibbles 0
    b = O.quantize_q4_k(np.full(256, -c, F))
    assert (int(b[0]) | (int(b[1]) << 8)) == O.f32_to_f16_trunc(float(c / F(945.0)))
    assert (int(b[2]) | (int(b[3]) << 8)) == O.f32_to_f16_trunc(float(c / F(63.0)))
    assert np.all(b[4:12] == (63 | (3 << 6))) and np.all(b[12:16] == 0xFF) and np.all(b[16:] == 0)
    # two-level block: sub-block 0 alternates 0 / 1.0, the rest zero ->
    # d = 1/945, scale[0]=63 others 0; low nibbles of group 0 alternate 0 / 15
    x = np.zeros(256, F)
    x[1:32:2] = 1.0
    b = O.quantize_q4_k(x)
    d, dmin, sc, mn = npr.q4k_unpack_header(b.reshape(1, 144))
    assert list(sc[0]) == [63, 0, 0, 0, 0, 0, 0, 0] and not mn.any() and dmin[0] == 0
    assert np.array_equal(b[16:48] & 0x0F, np.tile([0, 15], 16)) and not (b[16:48] >> 4).any()
    assert not b[48:].any()


@pytest.mark.parametrize("seed,scale", [(0, 0.02), (1, 1.0), (2, 1e-4), (3, 30.0)])
def test_q4k_encoder_bytes_agree_with_numpy_restatement(seed, scale):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(64 * 1024) * scale).astype(F)
    x[:256] = np.abs(x[:256])           # an all-positive block
    x[256:512] = -np.abs(x[256:512])    # an all-negative block
    x[512:544] = 0                      # a zero sub-block
    assert np.array_equal(O.quantize_q4_k(x), npr.quantize_q4_k(x))


def test_q4k_round_trip_bound():
    # larql-compute/tests/test_q4k_parity.rs:48-65: error stays within the
    # sub-block step; here: |err| <= range/15 per sub-block.
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(256 * 64) * 0.02).astype(F)
    back = O.dequantize_q4_k(O.quantize_q4_k(x), x.size)
    xs, bs = x.reshape(-1, 32), back.reshape(-1, 32)
    rngs = np.maximum(xs.max(1), 0) - np.minimum(xs.min(1), 0)
    assert np.all(np.abs(xs - bs).max(1) <= rngs / 15 * 1.01 + 1e-7)
    assert np.array_equal(bits(npr.dequantize_q4_k(O.quantize_q4_k(x), x.size)), bits(back))


# ---------------------------------------------------------------------- MXFP4
def test_mxfp4_reference_kats():
    # larql-models/src/quant/mxfp4.rs:276-380
    assert O.e8m0_to_f32(0) == 0.0 and O.e8m0_to_f32(127) == 1.0 and O.e8m0_to_f32(128) == 2.0
    assert O.e8m0_to_f32(126) == 0.5 and O.e8m0_to_f32(129) == 4.0 and O.e8m0_to_f32(125) == 0.25
    assert np.isnan(O.e8m0_to_f32(255))
    assert [O.mxfp4_table(i) for i in (0, 2, 7, 10, 15)] == [0.0, 1.0, 6.0, -1.0, -6.0]
    u8 = lambda v, n: np.full(n, v, np.uint8)
    assert np.all(O.dequantize_mxfp4_expert(u8(0x22, 16), u8(127, 1), 1, 1) == 1.0)
    assert np.all(O.dequantize_mxfp4_expert(u8(0x22, 16), u8(128, 1), 1, 1) == 2.0)
    assert np.all(O.dequantize_mxfp4_expert(u8(0xAA, 16), u8(127, 1), 1, 1) == -1.0)
    assert np.all(O.dequantize_mxfp4_expert(u8(0xFF, 16), u8(0, 1), 1, 1) == 0.0)
    r = O.dequantize_mxfp4_expert(u8(0x37, 16), u8(127, 1), 1, 1)
    assert r[0] == 6.0 and r[1] == 1.5
    r = O.dequantize_mxfp4_expert(u8(0x22, 32), np.array([127, 128], np.uint8), 1, 2)
    assert r[0] == 1.0 and r[32] == 2.0
    assert O.dequantize_mxfp4_expert(u8(0x22, 15), u8(127, 1), 1, 1) is None     # short blocks
    assert O.dequantize_mxfp4_expert(u8(0x22, 16), u8(127, 0), 1, 1) is None     # short scales


def test_nearest_mxfp4_code_ties_and_saturation():
    # quantize.rs:71-88: nearest grid value, ties to the even code, saturate at 6, -0 collapses
    cases = {0.0: 0, 0.2: 0, 0.25: 0, 0.26: 1, 0.5: 1, 0.75: 2, 1.25: 2, 1.75: 4, 2.5: 4, 3.5: 6,
             5.0: 6, 5.1: 7, 6.0: 7, 100.0: 7}
    for v, code in cases.items():
        assert O.nearest_mxfp4_code(v) == code, v
        assert O.nearest_mxfp4_code(-v) == (0 if code == 0 else 8 | code), -v
    assert O.nearest_mxfp4_code(-0.0) == 0


def test_quantize_mxfp4_closed_forms_and_round_trip():
    # a group holding exactly the grid times 2^e encodes losslessly with byte e+127... :
    grid = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -.5, -1, -1.5, -2, -3, -4, -6, 0] * 2, F)
    for e in (-9, 0, 5):
        x = grid * F(2.0 ** e)
        p, s = O.quantize_mxfp4(x, 1, 32)
        assert s[0] == 127 + e                     # floor(log2(6*2^e)) - 2 = e
        assert np.array_equal(O.dequantize_mxfp4_expert(p, s, 1, 1), x)
    p, s = O.quantize_mxfp4(np.zeros(32, F), 1, 32)
    assert s[0] == 0 and not p.any()
    # max exactly a power of two 2^m -> exponent m-2, the max lands on code 6 (=4.0)
    x = np.zeros(32, F); x[3] = 8.0; x[4] = -8.0; x[5] = 1.0
    p, s = O.quantize_mxfp4(x, 1, 32)
    assert s[0] == 127 + 1
    codes = np.stack([p & 15, p >> 4], -1).reshape(-1)
    assert codes[3] == 6 and codes[4] == 14 and codes[5] == 1
    # overshoot saturates: max 7.9 -> exponent 0, 7.9 -> 6.0
    x = np.zeros(32, F); x[0] = 7.9
    p, s = O.quantize_mxfp4(x, 1, 32)
    assert s[0] == 127 and (p[0] & 15) == 7
    assert O.quantize_mxfp4(np.zeros(48, F), 1, 48) is None
    # seeded: bytes agree with the numpy restatement; decode error <= half the widest grid gap
    rng = np.random.default_rng(9)
    w = (rng.standard_normal(64 * 2880) * 0.02).astype(F)
    p, s = O.quantize_mxfp4(w, 64, 2880)
    p2, s2 = npr.quantize_mxfp4(w, 64, 2880)
    assert np.array_equal(s, s2) and np.array_equal(p, p2)
    back = O.dequantize_mxfp4_expert(p, s, 64, 90)
    assert np.array_equal(bits(back), bits(npr.dequantize_mxfp4(p, s, 64, 2880).reshape(-1)))
    step = np.repeat(npr.e8m0(s), 32)
    err = np.abs(back - w)
    sat = np.abs(w) > 6 * step          # group max in (6,8)*scale saturates at 6: error < 2*scale
    assert np.all(err[~sat] <= step[~sat] * 1.0) and np.all(err[sat] < step[sat] * 2.0)


def test_quantize_mxfp4_log2_edge_just_below_a_power_of_two():
    # f32 log2 of the largest float below 2^3 rounds up to 3.0, so the shared
    # exponent is 3-2, not 2-2 (load.rs:460 computes log2 in f32).
    x = np.zeros(32, F)
    x[0] = np.nextafter(F(8.0), F(0.0))
    p, s = O.quantize_mxfp4(x, 1, 32)
    assert s[0] == 127 + 1
    # ...whereas just below 1.0 the f32 log2 is a small negative number
    x[0] = np.nextafter(F(1.0), F(0.0))
    p, s = O.quantize_mxfp4(x, 1, 32)
    assert s[0] == 127 - 1 - 2


# --------------------------------------------------------------- Q8_0 / Q4_0 / Q8
def test_q8_0_seeded_bytes_agree_and_decode():
    rng = np.random.default_rng(4)
    w = (rng.standard_normal(4096 * 8) * 0.02).astype(F)
    w[:32] = 0
    w[32:64] = 1e-7      # subnormal f16 scale
    b = O.quantize_q8_0(w)
    assert np.array_equal(b, npr.quantize_q8_0(w))
    assert np.array_equal(bits(O.dequantize_q8_0(b, w.size)), bits(npr.dequantize_q8_0(b, w.size)))
    assert O.dequantize_q8_0(b[:-1], w.size) is None


def test_quantize_to_q8_and_q4_0_closed_forms():
    x = np.zeros(64, F)
    x[0], x[1], x[33] = 127.0, -63.5, 2.0
    q, s = O.quantize_to_q8(x)
    assert s[0] == 1.0 and q[0] == 127 and q[1] == -64 and s[1] == F(2.0) / F(127.0) and q[33] == 127
    # Q4_0: scale amax/7, planar nibbles: byte j = elem j | elem j+16 << 4, code = round(v/scale)+8
    x = np.zeros(32, F); x[0] = 7.0; x[16] = -7.0; x[1] = 3.4
    b = O.quantize_q4_0(x)
    assert b.size == 18 and (int(b[0]) | (int(b[1]) << 8)) == 0x3C00
    assert b[2] == (15 | (1 << 4)) and b[3] == ((3 + 8) | (8 << 4))
    z = O.quantize_q4_0(np.zeros(32, F))      # zero block: scale 0, every code 0+8
    assert z[0] == 0 and z[1] == 0 and np.all(z[2:] == 0x88)
