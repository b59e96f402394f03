"""Adversarial known-answer tests for the block encoders of the CPU checker.

Expected bytes come from exact rational arithmetic on the reference text
(tests/exact_f32.py; fixture tests/golden/encoder_kats.json written by
tests/golden/make_encoder_kats.py).  Three things are asserted:
  1. the exact model itself reproduces the reference-held ggml Q8_0 golden
     blocks and IEEE conversions (so `fl`, Rust's `round`, the f16 conversions
     are pinned on data the reference holds, not on this repo's restatements);
  2. the C checker and the numpy restatement give the fixture's bytes;
  3. every named plausible mistake (round-half-even, codes from the stored f16
     header, rounded instead of truncated headers, divide instead of
     multiply-by-reciprocal, swapped nibbles / 6-bit slots, ...) gives
     DIFFERENT bytes on these inputs — so a checker with that mistake fails 2.
A few header bytes are also spelled out by hand.
"""
import json
import os
from fractions import Fraction as Q

import numpy as np
import pytest

import exact_f32 as E
import np_restatement as npr
import oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")
F = np.float32
KATS = json.load(open(os.path.join(GOLD, "encoder_kats.json")))["cases"]


def inputs(name):
    return np.array(KATS[name]["input_bits"], np.uint32).view(F)


def exact_inputs(name):
    return [E.from_bits(b) for b in KATS[name]["input_bits"]]


# ------------------------------------------------------------------ the model is pinned first
def test_exact_model_reproduces_the_ggml_q8_0_golden_blocks():
    # larql-models/src/quant/ggml/q8_0_ggml_golden.rs (ggml quantize_row_q8_0_ref @ facdc44a), held as a fixture
    d = json.load(open(os.path.join(GOLD, "q8_0_ggml_golden.json")))
    assert len(d["cases"]) >= 20
    for c in d["cases"]:
        x = [E.from_bits(b) for b in c["input_bits"]]
        assert E.quantize_q8_0(x).hex() == c["block_hex"], c["name"]


def test_exact_model_fl_and_f16_agree_with_ieee():
    rng = np.random.default_rng(5)
    a = rng.standard_normal(400).astype(F) * F(3.0)
    b = (rng.standard_normal(400).astype(F) * F(0.01)) + F(0.001)
    for x, y in zip(a, b):
        qx, qy = Q(float(x)), Q(float(y))
        assert E.fl(qx + qy) == Q(float(F(x + y)))
        assert E.fl(qx * qy) == Q(float(F(x * y)))
        assert E.fl(qx / qy) == Q(float(F(x / y)))
    # IEEE half conversion (numpy float16 is round-to-nearest-even) and truncation = the largest half not above |v|
    v = np.concatenate([rng.standard_normal(500).astype(F) * F(s) for s in (1.0, 1e-4, 3e-6, 1e-8, 900.0)])
    for x in v:
        h = np.float16(x)
        assert E.f16_nearest(Q(float(x))) == int(h.view(np.uint16))
        t = h if abs(float(h)) <= abs(float(x)) else np.nextafter(h, np.float16(0))
        assert E.f16_trunc(Q(float(x))) == int(np.float16(t).view(np.uint16)), x
    assert E.round_half_away(Q(5, 2)) == 3 and E.round_half_away(Q(-5, 2)) == -3 and E.round_half_even(Q(5, 2)) == 2


def test_oracle_f16_truncation_is_the_largest_half_not_above():
    # q4_common/f16.rs:10-41 against IEEE: truncation toward zero, subnormals kept, f32 subnormals -> 0
    rng = np.random.default_rng(6)
    v = np.concatenate([rng.standard_normal(4000).astype(F) * F(s) for s in (1.0, 1e-3, 1e-4, 3e-6, 2e-7, 1e-8, 5000.0)])
    for x in v:
        h = np.float16(x)
        t = h if abs(float(h)) <= abs(float(x)) else np.nextafter(h, np.float16(0))
        want = int(np.float16(t).view(np.uint16))
        if abs(float(x)) < 2.0 ** -24:
            want &= 0x8000
        assert O.f32_to_f16_trunc(float(x)) == want, x


# ------------------------------------------------------------------ hand-spelled header bytes
def test_q4k_exact_halves_header_by_hand():
    # d = 945/945 = 1 -> f16 0x3C00; dmin = 63/63 = 1 -> 0x3C00.
    # q_scale = [63, 11 (10.5 rounds away), 32, 16, 17, 35, 62, 4]; q_min = [63, 21 (20.5), 0, 3 (2.5), 34, 52, 5, 61].
    # packed[j]   = qs[j]   | (qs[j+4] >> 4) << 6 : 63|1<<6=0x7F, 11|2<<6=0x8B, 32|3<<6=0xE0, 16|0<<6=0x10
    # packed[j+4] = qm[j]   | (qm[j+4] >> 4) << 6 : 63|2<<6=0xBF, 21|3<<6=0xD5,  0|0<<6=0x00,  3|3<<6=0xC3
    # packed[j+8] = qs[j+4]&15 | (qm[j+4]&15) << 4: 1|2<<4=0x21, 3|4<<4=0x43, 14|5<<4=0x5E, 4|13<<4=0xD4
    want = bytes([0x00, 0x3C, 0x00, 0x3C, 0x7F, 0x8B, 0xE0, 0x10, 0xBF, 0xD5, 0x00, 0xC3, 0x21, 0x43, 0x5E, 0xD4])
    assert bytes.fromhex(KATS["q4k_exact_halves"]["hex"])[:16] == want
    got = O.quantize_q4_k(inputs("q4k_exact_halves")).tobytes()
    assert got[:16] == want
    # group 1 (bytes 48..80): low nibble = sub 2 (scale 32, min 0), high = sub 3 (scale 16, min 3):
    # sub 2: 480/32=15, 208/32=6.5->7, 16/32=0.5->1, 48/32=1.5->2, 80/32=2.5->3, 464/32=14.5->15, 17/32->1, 16/32->1
    # sub 3: (-2.5+3)/16->0, (237.5+3)/16=15.03->15, (5+3)/16=0.5->1, (21+3)/16=1.5->2, (13+3)/16=1, (229+3)/16=14.5->15, 3/16->0, 2/16->0
    lo = [15, 7, 1, 2, 3, 15, 1, 1]
    hi = [0, 15, 1, 2, 1, 15, 0, 0]
    assert list(got[48:56]) == [a | (b << 4) for a, b in zip(lo, hi)]


def test_q4k_f32_header_bytes_by_hand():
    got = O.quantize_q4_k(inputs("q4k_f32_header")).tobytes()
    # d = 1 + 2^-11 + 2^-12 truncates to f16 1.0 (0x3C00; round-to-nearest would give 0x3C01); dmin = 1 + 2^-12 -> 0x3C00
    assert got[:4] == bytes([0x00, 0x3C, 0x00, 0x3C])
    # sub 0 scale 63, element 1 = 913.75 -> code 14 from the f32 d (15 from the stored one); sub 1 is the high nibble: 100 -> ...
    assert got[16 + 1] & 0x0F == 14
    # sub 1: q_min 20 (21 from the stored dmin); sub 3: q_scale 10 (11 from the stored d)
    assert got[8 + 1] & 0x3F == 20 and got[4 + 3] & 0x3F == 10


def test_q6k_exact_halves_scales_by_hand():
    got = O.quantize_q6_k(inputs("q6k_exact_halves")).tobytes()
    # d = 3937/(31*127) = 1 -> 0x3C00 at bytes 208..209; scales: 127, 10.5 -> 11, 20.5 -> 21, 16, 2, 0, 3, 7
    assert got[208:210] == bytes([0x00, 0x3C])
    assert list(got[192:200]) == [127, 11, 21, 16, 2, 0, 3, 7]


# ------------------------------------------------------------------ checker == exact arithmetic
BYTE_ENCODERS = {
    "quantize_q4_k": (O.quantize_q4_k, npr.quantize_q4_k, E.quantize_q4_k,
                      ["rne", "f16_d", "f16_nearest", "divide", "swap_nibbles", "swap_pack", "no_zero_clamp"]),
    "quantize_q6_k": (O.quantize_q6_k, npr.quantize_q6_k, E.quantize_q6_k, ["rne", "f16_d", "f16_nearest", "divide", "amax_32"]),
    "quantize_q4_0": (O.quantize_q4_0, None, E.quantize_q4_0, ["rne", "divide", "f16_d", "f16_subnormal", "interleaved"]),
    "quantize_q8_0": (O.quantize_q8_0, npr.quantize_q8_0, E.quantize_q8_0, ["rne", "f16_trunc", "f16_d", "divide"]),
}


@pytest.mark.parametrize("name", [n for n, c in KATS.items() if "hex" in c])
def test_byte_encoders_match_exact_arithmetic(name):
    case = KATS[name]
    oracle_fn, numpy_fn, exact_fn, _ = BYTE_ENCODERS[case["encoder"]]
    want = bytes.fromhex(case["hex"])
    assert exact_fn(exact_inputs(name)) == want          # the fixture is what the model derives
    assert oracle_fn(inputs(name)).tobytes() == want
    if numpy_fn is not None:
        assert np.asarray(numpy_fn(inputs(name))).tobytes() == want


def test_every_named_mistake_changes_the_bytes():
    for enc, (_, _, exact_fn, mutants) in BYTE_ENCODERS.items():
        names = [n for n, c in KATS.items() if c.get("encoder") == enc]
        for m in mutants:
            caught = [n for n in names if exact_fn(exact_inputs(n), frozenset([m])) != bytes.fromhex(KATS[n]["hex"])]
            assert caught, f"{enc}: no known-answer block tells the reference's rule from mutant '{m}'"


def test_quantize_to_q8_matches_exact_arithmetic():
    case = KATS["to_q8"]
    q8, sc = O.quantize_to_q8(inputs("to_q8"))
    assert list(map(int, q8)) == case["codes"]
    assert list(map(int, np.asarray(sc, F).view(np.uint32))) == case["scale_bits"]
    # by hand, block 0 (scale 1): 0.5 -> 1, -0.5 -> -1, 1.5 -> 2, 2.5 -> 3, 126.5 -> 127, -126.5 -> -127
    assert case["codes"][:10] == [127, -127, 1, -1, 2, -2, 3, -3, 127, -127]
    ex = exact_inputs("to_q8")
    assert E.quantize_to_q8(ex)[0] == case["codes"]
    for m in ("rne", "divide"):
        assert E.quantize_to_q8(ex, frozenset([m]))[0] != case["codes"], m


def test_quantize_x_to_q8k_matches_exact_arithmetic():
    case = KATS["q8k"]
    qs, d, sums = O.quantize_x_to_q8k(inputs("q8k"))
    assert list(map(int, qs)) == case["codes"]
    assert list(map(int, np.asarray(d, F).view(np.uint32))) == case["d_bits"]
    assert list(map(int, sums)) == case["sums"]
    qn, dn, sn = npr.quantize_x_to_q8k(inputs("q8k"))
    assert list(map(int, qn)) == case["codes"] and list(map(int, sn)) == case["sums"]
    assert list(map(int, np.asarray(dn, F).view(np.uint32))) == case["d_bits"]
    # by hand, block 0 (d = 1): sub-block 0 = [127,-127,1,-1,2,-2,3,-3,127,-127] + 22 ones -> sum 22;
    # sub-block 1 = [-4, 4, 10] + 29 * (-2) -> -48; sub-blocks 2..7 = -16..15 -> -16 each
    assert case["sums"][:8] == [22, -48, -16, -16, -16, -16, -16, -16]
    assert case["d_bits"][0] == 0x3F800000 and case["d_bits"][1] == 0x40400000 and case["d_bits"][3] == 0
    ex = exact_inputs("q8k")
    assert E.quantize_x_to_q8k(ex)[0] == case["codes"]
    for m in ("rne", "divide", "scale_127_over_amax"):
        assert E.quantize_x_to_q8k(ex, frozenset([m]))[0] != case["codes"], m


def test_quantize_mxfp4_matches_exact_arithmetic_and_hand_bytes():
    case = KATS["mxfp4"]
    packed, scales = O.quantize_mxfp4(inputs("mxfp4"), case["rows"], case["k"])
    assert np.asarray(packed).tobytes().hex() == case["packed_hex"] and np.asarray(scales).tobytes().hex() == case["scales_hex"]
    pn, sn = npr.quantize_mxfp4(inputs("mxfp4"), case["rows"], case["k"])
    assert np.asarray(pn).tobytes().hex() == case["packed_hex"] and np.asarray(sn).tobytes().hex() == case["scales_hex"]
    # by hand — group 0, max 6: floor(log2 6) - 2 = 0 -> byte 127; pairs (6,-6) (0.25,0.75) (1.25,1.75) (2.5,3.5) (5,-0.25)
    # (-0.75,-1.25) (-1.75,-2.5) (-3.5,-5) (0.5,1) (1.5,2) (3,4) (-0.2,0.2) (0.26,5.1): midpoints go to the even code,
    # a negative value that rounds to zero loses its sign, element 2b sits in the low nibble
    assert case["packed_hex"][:26] == "f720426406aaccee2143650071"
    # group 1, max 100: floor(log2 100) - 2 = 4 -> byte 131; all-zero group -> 0; max 2^-130 -> clamped to 1
    assert case["scales_hex"] == "7f830001"
    ex = exact_inputs("mxfp4")
    assert E.quantize_mxfp4(ex, case["rows"], case["k"]) == (bytes.fromhex(case["packed_hex"]), bytes.fromhex(case["scales_hex"]))
    for m in ("ties_odd", "keep_sign_of_zero", "hi_first", "emax_3", "no_clamp"):
        assert E.quantize_mxfp4(ex, case["rows"], case["k"], frozenset([m])) != \
            (bytes.fromhex(case["packed_hex"]), bytes.fromhex(case["scales_hex"])), m
