"""Writes tests/golden/encoder_kats.json: adversarial known-answer blocks for the block encoders.

The inputs are constructed by hand so that each one sits on a decision the reference text makes
(Rust `f32::round` on exact halves, the un-rounded f32 d / dmin in the code computation, truncating
f16 headers, multiply-by-reciprocal, the 6-bit packing of slots 4-7, planar nibble order, ...); the
expected bytes are derived from the reference text in exact rational arithmetic (tests/exact_f32.py,
itself held to the reference's ggml Q8_0 golden blocks).  Nothing here runs the reference or either
restatement under test.  Run from the repo root: python tests/golden/make_encoder_kats.py
"""
import json
import os
import sys
from fractions import Fraction as Q

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import exact_f32 as E  # noqa: E402


def ulps(q, n):
    return E.from_bits(E.f32_bits(Q(q)) + n)


def pad(vals, n, fill):
    vals = [Q(v) for v in vals]
    assert len(vals) <= n
    return vals + [Q(fill)] * (n - len(vals))


def q4k_block_exact_halves():
    """d = 1 and dmin = 1 exactly (max range 945 = 15*63, min -63), so every quotient below is exact.
    sub 1: range 157.5 -> 157.5/15 = 10.5 (round: 11, ties-even: 10); min -20.5 -> 21 / 20.
    sub 2: all positive (min forced to 0), scale 32 = a power of two: 208/32 = 6.5 -> 7 / 6, 16/32 = 0.5 -> 1 / 0.
    sub 3: min -2.5 -> 3 / 2.   subs 4-7: 6-bit codes 17/34, 35/52, 62/5, 4/61 — all distinct, both top bits used.
    sub 7: all negative (max forced to 0).   The values a few ulps under (n+1/2)*scale tell
    (v+mn)*(1/sc) from (v+mn)/sc: the product rounds up to the half, the quotient does not."""
    s0 = pad([-63, 882, Q(-31.500001907348633), Q(31.49999237060547), Q(94.49998474121094), Q(283.4999694824219), 440.5, 0.25], 32, 0)
    s1 = pad([-20.5, 137, Q(6.499998092651367), Q(28.499996185302734), Q(94.49999237060547), -15.5, 12, 100], 32, 1)
    s2 = pad([480, 208, 16, 48, 80, 464, 17, 15.984375 + 0.015625], 32, 16)   # 15.984375+0.015625 = 16: the sub-block minimum is 16 > 0
    s3 = pad([-2.5, 237.5, 5, 21, 13, 229, 0], 32, -1)
    s4 = pad([-34, 221, -25.5, -8.5, 8.5, 212.5], 32, 0)
    s5 = pad([-52, 473, -34.5, 0.5, 35.5, 455.5], 32, 3)
    s6 = pad([-5, 925, 26, 88, 894], 32, 57)
    s7 = pad([-61, -1, -59, -55, -3], 32, -30)
    return s0 + s1 + s2 + s3 + s4 + s5 + s6 + s7


def q4k_block_f32_header():
    """d = 4099/4096 = 1 + 2^-11 + 2^-12 (f16: truncates to 0x3C00, rounds to 0x3C01) and dmin = 4097/4096 (f16 1.0).
    sub 0: 913.75/(63 d) = 14.493 -> 14 with the f32 d the reference uses, 913.75/63 = 14.504 -> 15 with the stored f16 d.
    sub 1: min -(20.5 + 2^-9): /dmin = 20.49695 -> 20 (f32), 20.50195 -> 21 (f16).
    sub 3: range 157.5625: /(15 d) = 10.4965 -> 10 (f32), 10.504 -> 11 (f16)."""
    d = Q(4099, 4096)
    dmin = Q(4097, 4096)
    s0 = pad([945 * d, Q(913.75), 31.75, 95.25], 32, 0)
    s1 = pad([-(Q(20.5) + Q(1, 512)), 100, 50], 32, 0)
    s2 = pad([-63 * dmin, 300, -10.25], 32, 2)
    s3 = pad([Q(157.5625), 78.75, 7.5], 32, 0)
    rest = []
    for j in range(4, 8):
        rest += pad([-(j * 3 + Q(1, 4)), j * 100 + Q(1, 2), j, -j], 32, Q(j, 8))
    return s0 + s1 + s2 + s3 + rest


def q4k_block_small_and_subnormal_header():
    """Weights of N(0, 0.02) size: d lands in the f16 subnormal range (kept by the truncating conversion,
    f16.rs:24-38) and nothing is exact, so every operation's f32 rounding is in play."""
    vals = []
    for i in range(256):
        # a fixed quasi-random pattern of binary32 values, about +-0.05, one sub-block tiny
        t = ((i * 2654435761) % 4093) - 2046
        scale = Q(1, 2 ** 15) if (i // 32) != 5 else Q(1, 2 ** 24)
        vals.append(E.fl(Q(t) * scale * Q(13, 16)))
    return vals


def q6k_block():
    """amax = 31*127 = 3937 -> d = 1 exactly.  Sub-block maxima 31*s + 15.5 put sub_max/(31 d) on exact halves
    (s + 1/2: round up, ties-even down for even s); inside a sub-block with scale 2^k the codes sit on exact halves;
    values a few ulps under a half tell v*(1/sc) from v/sc for the scales that are not powers of two."""
    subs = []
    subs.append(pad([3937, -3937 + 31, 1984, -1984, Q(1890.5), Q(-1890.5)], 16, 0))             # scale 127
    subs.append(pad([31 * 10 + 15.5, -5, 5, 15], 16, 0))                                      # 10.5 -> 11 / 10
    subs.append(pad([-(31 * 20 + 15.5), 10.5, 31.5, -31.5], 16, 0))                           # 20.5 -> 21 / 20
    subs.append(pad([31 * 16, 8, 24, -8, -24, 40, 488, -472, -456], 16, 0))                   # scale 16: +-k.5 codes
    subs.append(pad([31 * 2, 1, 3, -1, -3, 61, 63, -63, -65], 16, 0))                         # scale 2
    subs.append(pad([0], 16, 0))                                                              # scale 0: inv = 0
    subs.append(pad([31 * 3, ulps(Q(4.5), -1), ulps(Q(7.5), -1), ulps(Q(13.5), -1), -ulps(Q(13.5), -1), 1.5, -1.5], 16, 0))  # scale 3
    subs.append(pad([-31 * 7, ulps(Q(24.5), -1), ulps(Q(3.5), -1), ulps(Q(10.5), -1), 3.5, -3.5], 16, 0))                     # scale 7
    for j in range(8, 16):
        s = 9 * j - 40
        subs.append(pad([31 * s + 7, -(31 * s) // 2, s * 1.5, -s * 2.5, s * 30.5, 1], 16, Q(j, 4)))
    out = []
    for s in subs:
        out += s
    return out


def q6k_block_f32_header():
    """d = 4099/4096 (f16 truncates to 1.0): sub 1's maximum 31*10.5 + 0.25 gives 10.5005 -> 11 only with the stored d,
    10.4928 -> 10 with the f32 d the reference uses; sub 2 holds a code on the same edge."""
    d = Q(4099, 4096)
    subs = [pad([3937 * d, -100], 16, 0), pad([Q(325.75), 3], 16, 0), pad([31 * 40, 40 * 14 + Q(20.25), -(40 * 9 + Q(20.25))], 16, 0)]
    for j in range(3, 16):
        subs.append(pad([j * 97 + Q(1, 2), -j * 13, j], 16, Q(j, 2)))
    out = []
    for s in subs:
        out += s
    return out


def q4_0_blocks():
    """Block 0: amax 7 -> scale 1: x.5 values (round away: 1.5 -> 2, ties-even 2; 2.5 -> 3 / 2; -0.5 -> -1 / 0), clamp at 15 (7+8)
    and the planar order (byte j = elements j and j+16).  Block 1: amax 21 -> scale 3, values a few ulps under a half
    (v*(1/3) rounds up to the half, v/3 does not).  Block 2: scale in the f16 subnormal range: the block's inline conversion
    flushes it to zero.  Block 3: scale 4099/4096: the codes come from the f32 scale, not from the stored f16 one."""
    b0 = [7, -7, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 3.5, -3.5, 4.5, -4.5, 5.5, -5.5, 6.5, -6.5] + \
         [0, 1, 2, 3, 4, 5, 6, -1, -2, -3, -4, -5, -6, 0.25, -0.25, 0.75]
    b1 = pad([21, -21, ulps(Q(4.5), -1), ulps(Q(7.5), -1), ulps(Q(13.5), -1), -ulps(Q(13.5), -1), ulps(Q(16.5), -1), 4.5, -4.5, 1.5, 10.5, -19.5], 32, 3)
    tiny = Q(7, 2 ** 20)     # scale 2^-20: below the smallest normal f16 (2^-14)
    b2 = pad([tiny, -tiny, tiny / 2, tiny / 4, -tiny / 7 * 3], 32, 0)
    b2 = [E.fl(v) for v in b2]
    s = Q(4099, 4096)
    b3 = pad([7 * s, Q(24.5078125), -(Q(10.5) + Q(1, 256)), Q(3.5) + Q(1, 512), 1, 2], 32, 0)
    return [Q(v) for v in b0] + b1 + b2 + b3


def to_q8_blocks():
    """Block 0: amax 127 -> scale 1, exact halves and both clamps' neighbourhoods.  Block 1: amax 381 -> scale 3 with
    values a few ulps under a half.  Block 2: scale not a power of two, ordinary values.  Block 3: zero block."""
    b0 = pad([127, -127, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5, 63.5, 64.5, -100.5, 100.5], 32, 0)
    b1 = pad([381, -381, ulps(Q(4.5), -1), ulps(Q(7.5), -1), ulps(Q(13.5), -1), -ulps(Q(13.5), -1), 379.5, -379.5, 1.5, 190.5], 32, 3)
    b2 = [E.fl(Q(((i * 7919) % 1009) - 504, 4096) * 3) for i in range(32)]
    b3 = [Q(0)] * 32
    return b0 + b1 + b2 + b3


def q8k_blocks():
    """Block 0: amax 127 -> d = 1: exact halves, sub-block sums by hand.  Block 1: amax 381 -> d = 3 with
    values a few ulps under a half; the reference multiplies by fl(1/d), llama.cpp's fl(127/amax) differs for amax = 0.3 etc.
    Block 2: amax 0.3-ish (inexact scale).  Block 3: zeros.  Block 4: an amax for which the two reciprocals differ."""
    b0 = pad([127, -127, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5], 32, 1) + pad([-3.5, 3.5, 10], 32, -2) + [Q(i) - 16 for i in range(32)] * 6
    b1 = pad([381, -381, ulps(Q(4.5), -1), ulps(Q(7.5), -1), ulps(Q(13.5), -1), -ulps(Q(13.5), -1), 379.5, -379.5, 1.5, 190.5], 256, 3)
    b2 = [E.fl(Q(((i * 7919) % 1009) - 504, 1680)) for i in range(256)]
    b3 = [Q(0)] * 256
    # amax 0.017 (bits 0x3C8B4396): fl(1/fl(amax/127)) != fl(127/amax), and these four values round differently under the two
    b4 = pad([E.from_bits(1015759766), E.from_bits(961710710), E.from_bits(967799650), E.from_bits(972398985), -E.from_bits(975038424)], 256, 0)
    return b0 + b1 + b2 + b3 + b4


def q8_0_blocks():
    """ggml Q8_0: block 0 scale 1 with exact halves; block 1 scale 4099/4096 whose f16 header rounds UP to 0x3C01 (nearest)
    while truncation gives 0x3C00, and whose codes come from the f32 scale; block 2 a subnormal f16 scale (kept);
    block 3 scale 3 with values a few ulps under a half (v*(1/3) rounds up to the half, v/3 does not)."""
    b0 = pad([127, -127, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5, 63.5, 64.5], 32, 0)
    s = Q(4099, 4096)
    b1 = pad([127 * s, Q(100.5859375), -Q(50.54296875), 3], 32, 1)
    tiny = Q(127, 2 ** 22) * Q(3, 2)
    b2 = [E.fl(v) for v in pad([tiny, -tiny / 2, tiny / 3, tiny / 254 * 3], 32, 0)]
    b3 = pad([381, -381, ulps(Q(4.5), -1), ulps(Q(7.5), -1), ulps(Q(13.5), -1), -ulps(Q(13.5), -1), 379.5, -379.5, 1.5, 190.5], 32, 3)
    return b0 + b1 + b2 + b3


def mxfp4_rows():
    """2 rows x 64.  Group 0: max 6 -> exponent floor(log2 6) - 2 = 0, byte 127, every grid value and every midpoint
    (0.25 -> code 0, 0.75 -> 2, 1.25 -> 2, 1.75 -> 4, 2.5 -> 4, 3.5 -> 6, 5 -> 6: ties go to the even code), -0.2 -> +0.
    Group 1: max 100 -> 2^4: saturation at 6 (96/16), negative midpoints.  Group 2: all zero -> byte 0, codes 0.
    Group 3: max 2^-130 (an f32 subnormal) -> exponent -132+127 < 1: the byte clamps to 1."""
    g0 = pad([6, -6, 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5, -0.25, -0.75, -1.25, -1.75, -2.5, -3.5, -5, 0.5, 1, 1.5, 2, 3, 4, -0.2, 0.2, 0.26, 5.1], 32, 0)
    g1 = pad([100, -96, 8, -12, 20, -28, 40, -56, 80, 4, -4, 3.9, 90], 32, 16)
    g2 = [Q(0)] * 32
    t = Q(2) ** -130
    g3 = pad([t, -t, t / 2, t / 4, 3 * t / 4], 32, 0)
    return [E.fl(v) for v in g0 + g1 + g2 + g3]   # (0.2, 0.26, 3.9, 5.1 become their nearest binary32)


def main():
    cases = {}

    def add(name, vals, **expected):
        vals = [Q(v) for v in vals]
        assert all(E.is_f32(v) for v in vals), name
        cases[name] = {"input_bits": [E.f32_bits(v) for v in vals], **expected}

    for name, vals in [("q4k_exact_halves", q4k_block_exact_halves()), ("q4k_f32_header", q4k_block_f32_header()),
                       ("q4k_small", q4k_block_small_and_subnormal_header())]:
        add(name, vals, encoder="quantize_q4_k", hex=E.quantize_q4_k(vals).hex())
    for name, vals in [("q6k_exact_halves", q6k_block()), ("q6k_f32_header", q6k_block_f32_header())]:
        add(name, vals, encoder="quantize_q6_k", hex=E.quantize_q6_k(vals).hex())
    add("q4_0", q4_0_blocks(), encoder="quantize_q4_0", hex=E.quantize_q4_0(q4_0_blocks()).hex())
    add("q8_0", q8_0_blocks(), encoder="quantize_q8_0", hex=E.quantize_q8_0(q8_0_blocks()).hex())
    q8, sc = E.quantize_to_q8(to_q8_blocks())
    add("to_q8", to_q8_blocks(), encoder="quantize_to_q8", codes=q8, scale_bits=[E.f32_bits(s) for s in sc])
    qs, ds, sums = E.quantize_x_to_q8k(q8k_blocks())
    add("q8k", q8k_blocks(), encoder="quantize_x_to_q8k", codes=qs, d_bits=[E.f32_bits(d) for d in ds], sums=sums)
    pk, sc = E.quantize_mxfp4(mxfp4_rows(), 2, 64)
    add("mxfp4", mxfp4_rows(), encoder="quantize_mxfp4", rows=2, k=64, packed_hex=pk.hex(), scales_hex=sc.hex())
    path = os.path.join(HERE, "encoder_kats.json")
    with open(path, "w") as f:
        json.dump({"about": "adversarial encoder known-answer blocks; expected values from exact rational arithmetic "
                            "(tests/golden/make_encoder_kats.py)", "cases": cases}, f, indent=0)
    print("wrote", path, {k: len(v["input_bits"]) for k, v in cases.items()})


if __name__ == "__main__":
    main()
