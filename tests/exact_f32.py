"""Exact-rational model of IEEE binary32 arithmetic, and the reference's block
encoders written on top of it straight from the reference text.

Every value is a `fractions.Fraction`; an f32 operation is the exact rational
result followed by `fl()` (round to nearest, ties to even, into binary32 with
subnormals).  Nothing here uses numpy's or C's float32, so it shares no
rounding behaviour with either restatement it checks.  Each encoder takes
`mut`, a set of named deliberate mistakes ("mutants"): the known-answer tests
assert that their inputs tell the reference's rule from every mutant.

Reference text followed (paths under crates/):
  quantize_q4_k        larql-compute/src/cpu/ops/q4_common/quantize.rs:89-189
  quantize_q6_k        larql-compute/src/cpu/ops/q4_common/quantize.rs:198-276
  quantize_q4_0        larql-compute/src/cpu/ops/q4_common/quantize.rs:28-69
  quantize_to_q8       larql-compute/src/cpu/ops/q4_common/quantize.rs:6-22
  f32_to_f16 (trunc.)  larql-compute/src/cpu/ops/q4_common/f16.rs:10-41
  quantize_x_to_q8k    larql-compute/src/cpu/ops/q4k_q8k_dot/q8k_activation.rs:84-109
  quantize_q8_0        larql-models/src/quant/ggml/quantize.rs:50-77
  f32_to_f16_nearest   larql-models/src/quant/half.rs:70-104
"""
from fractions import Fraction as Q
import math
import struct


def _floor_log2(q: Q) -> int:
    """floor(log2(q)) for q > 0, exactly."""
    e = q.numerator.bit_length() - q.denominator.bit_length()
    if Q(2) ** e > q:
        e -= 1
    elif Q(2) ** (e + 1) <= q:
        e += 1
    return e


def round_half_even(q: Q) -> int:
    f = math.floor(q)
    r = q - f
    if r > Q(1, 2) or (r == Q(1, 2) and f % 2 == 1):
        return f + 1
    return f


def round_half_away(q: Q) -> int:
    """Rust's f32::round."""
    a = math.floor(abs(q) + Q(1, 2))
    return a if q >= 0 else -a


def fl(q: Q) -> Q:
    """Round an exact rational to binary32 (nearest, ties to even)."""
    q = Q(q)
    if q == 0:
        return Q(0)
    s = 1 if q > 0 else -1
    a = abs(q)
    e = max(_floor_log2(a), -126)
    ulp = Q(2) ** (e - 23)
    n = round_half_even(a / ulp)
    r = n * ulp
    assert r < Q(2) ** 128, "overflow is not modelled"
    return s * r


def is_f32(q: Q) -> bool:
    return fl(q) == Q(q)


def f32_bits(q: Q) -> int:
    """Bit pattern of an exactly representable value (+0 for zero)."""
    q = Q(q)
    assert is_f32(q), q
    if q == 0:
        return 0
    sign = 0x80000000 if q < 0 else 0
    a = abs(q)
    e = _floor_log2(a)
    if e < -126:
        return sign | int(a / Q(2) ** -149)
    mant = int(a / Q(2) ** (e - 23)) - (1 << 23)
    return sign | ((e + 127) << 23) | mant


def from_bits(b: int) -> Q:
    return Q(struct.unpack("<f", struct.pack("<I", b))[0])


def f16_trunc(q: Q) -> int:
    """f32_to_f16 of q4_common/f16.rs:10-41 on the f32 bit pattern (finite inputs)."""
    bits = f32_bits(q)
    sign = (bits >> 16) & 0x8000
    exp = (bits >> 23) & 0xFF
    mant = bits & 0x7FFFFF
    if exp == 0:
        return sign
    new_exp = exp - 127 + 15
    if new_exp >= 31:
        return sign | 0x7C00
    if new_exp <= 0:
        shift = 1 - new_exp
        if 13 + shift >= 24:
            return sign
        return sign | ((mant | 0x800000) >> (13 + shift))
    return sign | (new_exp << 10) | (mant >> 13)


def f16_value(h: int) -> Q:
    """IEEE half -> exact value (finite)."""
    s = -1 if h & 0x8000 else 1
    e = (h >> 10) & 31
    m = h & 0x3FF
    if e == 0:
        return s * Q(m) * Q(2) ** -24
    return s * (1 + Q(m, 1024)) * Q(2) ** (e - 15)


def f16_nearest(q: Q) -> int:
    """IEEE round-to-nearest-even f32 -> f16 with subnormals (half.rs:70-104), finite inputs."""
    q = Q(q)
    sign = 0x8000 if q < 0 else 0
    a = abs(q)
    if a == 0:
        return sign
    e = max(_floor_log2(a), -14)
    ulp = Q(2) ** (e - 10)
    n = round_half_even(a / ulp)
    v = n * ulp
    if v >= 65520:
        return sign | 0x7C00
    if v < Q(2) ** -14:
        return sign | int(v / Q(2) ** -24)
    e2 = _floor_log2(v)
    return sign | ((e2 + 15) << 10) | (int(v / Q(2) ** (e2 - 10)) - 1024)


def f16_flush(q: Q) -> int:
    """The inline conversion of quantize_q4_0 (quantize.rs:41-58): truncation, subnormals flushed."""
    bits = f32_bits(q)
    sign = (bits >> 16) & 0x8000
    exp = (bits >> 23) & 0xFF
    mant = bits & 0x7FFFFF
    if exp == 0:
        return sign
    new_exp = exp - 127 + 15
    if new_exp >= 31:
        return sign | 0x7C00
    if new_exp <= 0:
        return sign
    return sign | (new_exp << 10) | (mant >> 13)


def _clamp(v, lo, hi):
    return lo if v < lo else hi if v > hi else v


def _vals(xs):
    out = [Q(x) for x in xs]
    assert all(is_f32(v) for v in out), "inputs must be binary32 values"
    return out


# ---------------------------------------------------------------------------------- Q4_K
def quantize_q4_k(data, mut=frozenset()) -> bytes:
    """mut: 'rne' round() ties to even; 'f16_d' nibbles (and 6-bit codes) from the f16-truncated d / dmin;
    'f16_nearest' header by round-to-nearest; 'divide' (v+mn)/sc instead of (v+mn)*(1/sc);
    'swap_nibbles' sub-block 2g in the high nibble; 'swap_pack' scales and mins exchanged in bytes 8..11;
    'no_zero_clamp' sub-block min / max not forced through zero."""
    data = _vals(data)
    assert len(data) % 256 == 0
    rnd = round_half_even if "rne" in mut else round_half_away
    out = bytearray()
    for sb in range(len(data) // 256):
        block = data[sb * 256:(sb + 1) * 256]
        mins, maxs = [], []
        for j in range(8):
            sub = block[j * 32:(j + 1) * 32]
            if "no_zero_clamp" in mut:
                mins.append(min(sub)); maxs.append(max(sub))
            else:
                mins.append(min(min(sub), Q(0))); maxs.append(max(max(sub), Q(0)))
        gmr = max([Q(0)] + [fl(a - b) for a, b in zip(maxs, mins)])
        gmin = min(mins)
        d = fl(gmr / fl(Q(15) * 63)) if gmr > 0 else Q(0)
        dmin = fl(-gmin / 63) if gmin < 0 else Q(0)
        h16 = f16_nearest if "f16_nearest" in mut else f16_trunc
        hd, hm = h16(d), h16(dmin)
        out += struct.pack("<HH", hd, hm)
        if "f16_d" in mut:
            d, dmin = f16_value(hd), f16_value(hm)
        qs, qm = [], []
        for j in range(8):
            rng = fl(maxs[j] - mins[j])
            qs.append(_clamp(rnd(fl(rng / fl(15 * d))), 0, 63) if d > 0 else 0)
            qm.append(_clamp(rnd(fl(-mins[j] / dmin)), 0, 63) if dmin > 0 else 0)
        packed = [0] * 12
        for j in range(4):
            packed[j] = (qs[j] & 0x3F) | (((qs[j + 4] >> 4) & 3) << 6)
            packed[j + 4] = (qm[j] & 0x3F) | (((qm[j + 4] >> 4) & 3) << 6)
            lo4, hi4 = (qm[j + 4], qs[j + 4]) if "swap_pack" in mut else (qs[j + 4], qm[j + 4])
            packed[j + 8] = (lo4 & 0x0F) | ((hi4 & 0x0F) << 4)
        out += bytes(packed)
        for g in range(4):
            enc = []
            for s in (2 * g, 2 * g + 1):
                sc = fl(d * qs[s]); mn = fl(dmin * qm[s])
                inv = fl(1 / sc) if sc > 0 else Q(0)
                codes = []
                for v in block[s * 32:(s + 1) * 32]:
                    t = fl(v + mn)
                    t = (fl(t / sc) if sc > 0 else Q(0)) if "divide" in mut else fl(t * inv)
                    codes.append(_clamp(rnd(t), 0, 15))
                enc.append(codes)
            if "swap_nibbles" in mut:
                enc.reverse()
            out += bytes(lo | (hi << 4) for lo, hi in zip(*enc))
    return bytes(out)


# ---------------------------------------------------------------------------------- Q6_K
def quantize_q6_k(data, mut=frozenset()) -> bytes:
    """mut: 'rne'; 'f16_d' codes from the f16-truncated d; 'f16_nearest'; 'divide' v/sc instead of v*(1/sc);
    'amax_32' d = amax/32 (the layout's older rule, which the reference text names as replaced)."""
    data = _vals(data)
    assert len(data) % 256 == 0
    rnd = round_half_even if "rne" in mut else round_half_away
    out = bytearray()
    for sb in range(len(data) // 256):
        block = data[sb * 256:(sb + 1) * 256]
        amax = max(abs(v) for v in block)
        d = fl(amax / 32) if "amax_32" in mut else fl(amax / fl(Q(31) * 127))
        hd = (f16_nearest if "f16_nearest" in mut else f16_trunc)(d)
        dq = f16_value(hd) if "f16_d" in mut else d
        scales = []
        for j in range(16):
            smax = max(abs(v) for v in block[j * 16:(j + 1) * 16])
            sc = fl(smax / fl(31 * dq)) if dq > 0 else Q(0)
            scales.append(_clamp(rnd(sc), -128, 127))
        q6 = []
        for j in range(16):
            sc = fl(dq * scales[j])
            inv = fl(1 / sc) if abs(sc) > fl(Q("1e-10")) else Q(0)
            for v in block[j * 16:(j + 1) * 16]:
                t = (fl(v / sc) if inv != 0 else Q(0)) if "divide" in mut else fl(v * inv)
                q6.append(_clamp(rnd(t), -32, 31) + 32)
        ql, qh = [0] * 128, [0] * 64
        for half in range(2):
            e = half * 128
            for l in range(32):
                q1, q2, q3, q4 = q6[e + l], q6[e + l + 32], q6[e + l + 64], q6[e + l + 96]
                ql[half * 64 + l] = (q1 & 15) | ((q3 & 15) << 4)
                ql[half * 64 + l + 32] = (q2 & 15) | ((q4 & 15) << 4)
                qh[half * 32 + l] = ((q1 >> 4) & 3) | (((q2 >> 4) & 3) << 2) | (((q3 >> 4) & 3) << 4) | (((q4 >> 4) & 3) << 6)
        out += bytes(ql) + bytes(qh) + bytes(s & 0xFF for s in scales) + struct.pack("<H", hd)
    return bytes(out)


# ---------------------------------------------------------------------- Q4_0 / Q8 activation
def quantize_q4_0(data, mut=frozenset()) -> bytes:
    """mut: 'rne'; 'divide' v/scale; 'f16_d' codes from the stored f16 scale; 'f16_subnormal' header keeps
    subnormals (the block's own inline conversion flushes them); 'interleaved' byte j = elements 2j, 2j+1."""
    data = _vals(data)
    assert len(data) % 32 == 0
    rnd = round_half_even if "rne" in mut else round_half_away
    out = bytearray()
    for i in range(len(data) // 32):
        block = data[i * 32:(i + 1) * 32]
        amax = max(abs(v) for v in block)
        scale = fl(amax / 7)
        h = (f16_trunc if "f16_subnormal" in mut else f16_flush)(scale)
        out += struct.pack("<H", h)
        if "f16_d" in mut:
            scale = f16_value(h)
        inv = fl(1 / scale) if scale > 0 else Q(0)

        def code(v):
            t = (fl(v / scale) if scale > 0 else Q(0)) if "divide" in mut else fl(v * inv)
            return _clamp(rnd(t) + 8, 0, 15)
        for j in range(16):
            a, b = (block[2 * j], block[2 * j + 1]) if "interleaved" in mut else (block[j], block[j + 16])
            out.append(code(a) | (code(b) << 4))
    return bytes(out)


def quantize_to_q8(x, mut=frozenset()):
    """-> (codes, scales as exact values).  mut: 'rne'; 'divide'; 'clamp127' clamps at -127."""
    x = _vals(x)
    rnd = round_half_even if "rne" in mut else round_half_away
    q8, scales = [], []
    for b in range(len(x) // 32):
        block = x[b * 32:(b + 1) * 32]
        amax = max(abs(v) for v in block)
        scale = fl(amax / 127)
        scales.append(scale)
        inv = fl(1 / scale) if scale > 0 else Q(0)
        for v in block:
            t = (fl(v / scale) if scale > 0 else Q(0)) if "divide" in mut else fl(v * inv)
            q8.append(_clamp(rnd(t), -127 if "clamp127" in mut else -128, 127))
    return q8, scales


def quantize_x_to_q8k(x, mut=frozenset()):
    """-> (qs, d as exact values, sums).  mut: 'rne'; 'divide'; 'scale_127_over_amax' (inv = fl(127/amax),
    llama.cpp's own form); 'sums_f32' sub-block sums of d*q instead of integer code sums."""
    x = _vals(x)
    assert len(x) % 256 == 0
    rnd = round_half_even if "rne" in mut else round_half_away
    qs, ds, sums = [], [], []
    for sb in range(len(x) // 256):
        block = x[sb * 256:(sb + 1) * 256]
        amax = max(abs(v) for v in block)
        scale = fl(amax / 127) if amax > 0 else Q(0)
        inv = fl(1 / scale) if scale > 0 else Q(0)
        if "scale_127_over_amax" in mut and amax > 0:
            inv = fl(127 / amax)
        ds.append(scale)
        for s in range(8):
            acc = 0
            for v in block[s * 32:(s + 1) * 32]:
                t = (fl(v / scale) if scale > 0 else Q(0)) if "divide" in mut else fl(v * inv)
                q = _clamp(rnd(t), -127, 127)
                qs.append(q)
                acc += q
            sums.append(acc)
    return qs, ds, sums


def quantize_q8_0(data, mut=frozenset()) -> bytes:
    """ggml Q8_0 (quantize.rs:50-77): d = f16_nearest(amax/127), codes from the un-rounded f32 scale's reciprocal.
    mut: 'rne'; 'f16_trunc' header truncated; 'f16_d' codes from the stored f16 scale; 'divide'."""
    data = _vals(data)
    assert len(data) % 32 == 0
    rnd = round_half_even if "rne" in mut else round_half_away
    out = bytearray()
    for i in range(len(data) // 32):
        block = data[i * 32:(i + 1) * 32]
        amax = max(abs(v) for v in block)
        scale = fl(amax / 127)
        h = (f16_trunc if "f16_trunc" in mut else f16_nearest)(scale)
        out += struct.pack("<H", h)
        sq = f16_value(h) if "f16_d" in mut else scale
        inv = fl(1 / sq) if sq != 0 else Q(0)
        for v in block:
            t = (fl(v / sq) if sq != 0 else Q(0)) if "divide" in mut else fl(v * inv)
            out.append(_clamp(rnd(t), -128, 127) & 0xFF)
    return bytes(out)


# ---------------------------------------------------------------------------------- MXFP4
MXFP4_GRID = [Q(0), Q(1, 2), Q(1), Q(3, 2), Q(2), Q(3), Q(4), Q(6)]


def nearest_mxfp4_code(v: Q, negative_zero=False, mut=frozenset()) -> int:
    """weights/quantize.rs:71-88.  mut: 'ties_odd' a tie keeps the odd code; 'keep_sign_of_zero'."""
    sign = 8 if (v < 0 or negative_zero) else 0
    mag = min(abs(v), Q(6))
    best, best_err = 0, None
    for code, value in enumerate(MXFP4_GRID):
        err = abs(mag - value)
        take_tie = (code % 2 == 1) if "ties_odd" in mut else (code % 2 == 0)
        if best_err is None or err < best_err or (err == best_err and take_tie):
            best, best_err = code, err
    if best == 0 and "keep_sign_of_zero" not in mut:
        return 0
    return sign | best


def quantize_mxfp4(values, rows, k, mut=frozenset()):
    """weights/load.rs:410-476, for groups whose maximum is not within a few ulps below a power of two (there the
    reference's f32 log2 may round up to the integer, which exact arithmetic cannot decide).
    mut: 'ties_odd', 'keep_sign_of_zero', 'hi_first' element 2b in the high nibble, 'emax_3' exponent - 3,
    'no_clamp' scale byte not clamped to 1..254."""
    values = _vals(values)
    assert k % 32 == 0 and len(values) == rows * k
    packed, scales = bytearray(), bytearray()
    for g in range(rows * k // 32):
        group = values[g * 32:(g + 1) * 32]
        max_abs = max(abs(v) for v in group)
        if max_abs == 0:
            byte = 0
        else:
            e = _floor_log2(max_abs) - (3 if "emax_3" in mut else 2) + 127
            byte = e & 0xFF if "no_clamp" in mut else _clamp(e, 1, 254)
        scales.append(byte)
        scale = Q(0) if byte == 0 else Q(2) ** (byte - 127)
        inv = Q(0) if scale == 0 else fl(1 / scale)
        for b in range(16):
            lo = nearest_mxfp4_code(fl(group[2 * b] * inv), False, mut)
            hi = nearest_mxfp4_code(fl(group[2 * b + 1] * inv), False, mut)
            packed.append((hi | (lo << 4)) if "hi_first" in mut else (lo | (hi << 4)))
    return bytes(packed), bytes(scales)
