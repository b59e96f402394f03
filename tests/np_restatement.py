"""Independent numpy restatement of the block codecs on the quantised path.

Test infrastructure: a second, differently-written statement of the encoders
and decoders, used only to cross-check oracle/larql_oracle.c byte for byte.
It follows the same reference sources (cited per function) but is vectorised
and shares no code with the C file.
"""
import numpy as np

F = np.float32


def rust_round(x):
    """f32::round — half away from zero — on an f32 array."""
    x64 = x.astype(np.float64)
    return np.trunc(x64 + np.copysign(0.5, x64)).astype(F)


def f16_bits_to_f32(bits):
    """IEEE half -> single (larql-models/src/quant/half.rs:14-35)."""
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(F)


def f32_to_f16_trunc(v):
    """larql-compute/src/cpu/ops/q4_common/f16.rs:10-41 (truncate, keep subnormals)."""
    b = np.asarray(v, dtype=F).view(np.uint32).astype(np.int64)
    sign = (b >> 16) & 0x8000
    exp = (b >> 23) & 0xFF
    mant = b & 0x7FFFFF
    new_exp = exp - 112
    normal = sign | (np.clip(new_exp, 0, 31) << 10) | (mant >> 13)
    shift = np.clip(14 - new_exp, 0, 63)  # 13 + (1 - new_exp)
    sub = np.where(shift >= 24, sign, sign | ((mant | 0x800000) >> shift))
    out = np.where(new_exp <= 0, sub, normal)
    out = np.where(new_exp >= 31, sign | 0x7C00, out)
    out = np.where(exp == 255, sign | 0x7C00 | (mant >> 13), out)
    out = np.where(exp == 0, sign, out)
    return out.astype(np.uint16)


def f32_to_f16_nearest(v):
    """larql-models/src/quant/half.rs:70-104 == IEEE RNE, i.e. numpy's own cast."""
    with np.errstate(over="ignore"):
        return np.asarray(v, dtype=F).astype(np.float16).view(np.uint16)


def q4k_unpack_header(blocks):
    """blocks: [nb,144] u8 -> d, dmin [nb] f32 and scales, mins [nb,8] u8 (get_scale_min_k4)."""
    d = f16_bits_to_f32(blocks[:, 0:2].copy().view(np.uint16)[:, 0])
    dmin = f16_bits_to_f32(blocks[:, 2:4].copy().view(np.uint16)[:, 0])
    p = blocks[:, 4:16].astype(np.uint8)
    sc = np.empty((blocks.shape[0], 8), np.uint8)
    mn = np.empty((blocks.shape[0], 8), np.uint8)
    sc[:, :4] = p[:, 0:4] & 63
    mn[:, :4] = p[:, 4:8] & 63
    sc[:, 4:] = (p[:, 8:12] & 0x0F) | ((p[:, 0:4] >> 6) << 4)
    mn[:, 4:] = (p[:, 8:12] >> 4) | ((p[:, 4:8] >> 6) << 4)
    return d, dmin, sc, mn


def dequantize_q4_k(data, n):
    """larql-compute/src/cpu/ops/q4_common/dequant.rs:9-53."""
    nb = n // 256
    blocks = np.asarray(data, np.uint8)[: nb * 144].reshape(nb, 144)
    d, dmin, sc, mn = q4k_unpack_header(blocks)
    qs = blocks[:, 16:].reshape(nb, 4, 32)
    scale = d[:, None] * sc.astype(F)          # [nb,8]
    minv = dmin[:, None] * mn.astype(F)
    out = np.empty((nb, 8, 32), F)
    out[:, 0::2, :] = scale[:, 0::2, None] * (qs & 0x0F).astype(F) - minv[:, 0::2, None]
    out[:, 1::2, :] = scale[:, 1::2, None] * (qs >> 4).astype(F) - minv[:, 1::2, None]
    return out.reshape(-1)


def quantize_q4_k(data):
    """larql-compute/src/cpu/ops/q4_common/quantize.rs:89-189."""
    x = np.asarray(data, F).reshape(-1, 8, 32)
    nb = x.shape[0]
    mins = np.minimum(x.min(-1), F(0))
    maxs = np.maximum(x.max(-1), F(0))
    rng = (maxs - mins).astype(F)
    gmr = rng.max(-1)
    gmin = mins.min(-1)
    with np.errstate(divide="ignore", invalid="ignore"):
        d = np.where(gmr > 0, gmr / F(945.0), F(0)).astype(F)
        dmin = np.where(gmin < 0, (-gmin) / F(63.0), F(0)).astype(F)
        qs = np.where(d[:, None] > 0, np.clip(rust_round(rng / (F(15.0) * d)[:, None]), 0, 63), 0).astype(np.uint8)
        qm = np.where(dmin[:, None] > 0, np.clip(rust_round((-mins) / dmin[:, None]), 0, 63), 0).astype(np.uint8)
        sc = (d[:, None] * qs.astype(F)).astype(F)
        mn = (dmin[:, None] * qm.astype(F)).astype(F)
        inv = np.where(sc > 0, F(1.0) / sc, F(0)).astype(F)
        enc = np.clip(rust_round(((x + mn[:, :, None]).astype(F) * inv[:, :, None]).astype(F)), 0, 15).astype(np.uint8)
    out = np.zeros((nb, 144), np.uint8)
    out[:, 0:2] = f32_to_f16_trunc(d).reshape(nb, 1).view(np.uint8)
    out[:, 2:4] = f32_to_f16_trunc(dmin).reshape(nb, 1).view(np.uint8)
    out[:, 4:8] = (qs[:, :4] & 0x3F) | (((qs[:, 4:] >> 4) & 3) << 6)
    out[:, 8:12] = (qm[:, :4] & 0x3F) | (((qm[:, 4:] >> 4) & 3) << 6)
    out[:, 12:16] = (qs[:, 4:] & 0x0F) | ((qm[:, 4:] & 0x0F) << 4)
    out[:, 16:] = (enc[:, 0::2, :] | (enc[:, 1::2, :] << 4)).reshape(nb, 128)
    return out.reshape(-1)


def dequantize_q6_k(data, n):
    """larql-models/src/quant/ggml/q6_k.rs:19-40,173-195 (ggml planar layout), written plane by plane."""
    nb = n // 256
    blocks = np.asarray(data, np.uint8)[: nb * 210].reshape(nb, 210)
    ql = blocks[:, :128].reshape(nb, 2, 2, 32)          # [block, half, row, l]
    qh = blocks[:, 128:192].reshape(nb, 2, 32)          # [block, half, l]
    sc = blocks[:, 192:208].view(np.int8).astype(F)     # [block, 16]
    d = f16_bits_to_f32(blocks[:, 208].astype(np.uint16) | (blocks[:, 209].astype(np.uint16) << 8))
    q = np.empty((nb, 2, 4, 32), np.int32)              # [block, half, plane, l]: element half*128 + plane*32 + l
    for plane in range(4):
        lo4 = (ql[:, :, plane & 1, :] & 0x0F) if plane < 2 else (ql[:, :, plane & 1, :] >> 4)
        hi2 = (qh >> (2 * plane)) & 3
        q[:, :, plane, :] = (lo4.astype(np.int32) | (hi2.astype(np.int32) << 4)) - 32
    q = q.reshape(nb, 16, 16).astype(F)                 # 16 sub-blocks of 16 in element order
    scale = (d[:, None] * sc).astype(F)
    return (scale[:, :, None] * q).astype(F).reshape(-1)


def quantize_q6_k(data):
    """larql-compute/src/cpu/ops/q4_common/quantize.rs:197-276."""
    x = np.asarray(data, F).reshape(-1, 16, 16)
    nb = x.shape[0]
    amax = np.abs(x).max((1, 2)).astype(F)
    d = (amax / F(31.0 * 127.0)).astype(F)
    sub_max = np.abs(x).max(-1).astype(F)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(d[:, None] > 0, sub_max / (F(31.0) * d)[:, None], F(0)).astype(F)
        ss = np.clip(rust_round(sc), -128, 127).astype(np.int8)
        scale = (d[:, None] * ss.astype(F)).astype(F)
        inv = np.where(np.abs(scale) > F(1e-10), F(1.0) / scale, F(0)).astype(F)
        q = (np.clip(rust_round((x * inv[:, :, None]).astype(F)), -32, 31).astype(np.int32) + 32).astype(np.uint8)
    q = q.reshape(nb, 2, 4, 32)                          # [block, half, plane, l]
    out = np.zeros((nb, 210), np.uint8)
    ql = np.empty((nb, 2, 2, 32), np.uint8)
    ql[:, :, 0, :] = (q[:, :, 0, :] & 0x0F) | ((q[:, :, 2, :] & 0x0F) << 4)
    ql[:, :, 1, :] = (q[:, :, 1, :] & 0x0F) | ((q[:, :, 3, :] & 0x0F) << 4)
    qh = ((q[:, :, 0, :] >> 4) & 3) | (((q[:, :, 1, :] >> 4) & 3) << 2) | (((q[:, :, 2, :] >> 4) & 3) << 4) | (((q[:, :, 3, :] >> 4) & 3) << 6)
    out[:, :128] = ql.reshape(nb, 128)
    out[:, 128:192] = qh.reshape(nb, 64)
    out[:, 192:208] = ss.view(np.uint8)
    out[:, 208:210] = f32_to_f16_trunc(d).reshape(nb, 1).view(np.uint8)
    return out.reshape(-1)


def quantize_q8_0(data):
    """larql-models/src/quant/ggml/quantize.rs:50-77."""
    x = np.asarray(data, F).reshape(-1, 32)
    amax = np.abs(x).max(-1)
    scale = (amax / F(127.0)).astype(F)
    with np.errstate(divide="ignore"):
        inv = np.where(scale > 0, F(1.0) / scale, F(0)).astype(F)
    q = np.clip(rust_round((x * inv[:, None]).astype(F)), -128, 127).astype(np.int8)
    out = np.empty((x.shape[0], 34), np.uint8)
    out[:, :2] = f32_to_f16_nearest(scale).reshape(-1, 1).view(np.uint8)
    out[:, 2:] = q.view(np.uint8)
    return out.reshape(-1)


def dequantize_q8_0(data, n):
    """larql-models/src/quant/ggml/legacy.rs:68-83."""
    b = np.asarray(data, np.uint8)[: n // 32 * 34].reshape(-1, 34)
    d = f16_bits_to_f32(b[:, :2].copy().view(np.uint16)[:, 0])
    return (b[:, 2:].view(np.int8).astype(F) * d[:, None]).astype(F).reshape(-1)


MXFP4_TABLE = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6], F)


def e8m0(b):
    b = np.asarray(b, np.uint8)
    v = (b.astype(np.uint32) << 23).view(F)
    v = np.where(b == 0, F(0), v)
    return np.where(b == 255, F(np.nan), v).astype(F)


def dequantize_mxfp4(packed, scales, rows, k):
    """larql-models/src/quant/mxfp4.rs:42-95."""
    g = k // 32
    p = np.asarray(packed, np.uint8).reshape(rows, g, 16)
    s = e8m0(np.asarray(scales, np.uint8).reshape(rows, g))
    out = np.empty((rows, g, 16, 2), F)
    out[..., 0] = MXFP4_TABLE[p & 15] * s[:, :, None]
    out[..., 1] = MXFP4_TABLE[p >> 4] * s[:, :, None]
    return out.reshape(rows, k)


def quantize_mxfp4(values, rows, k):
    """.../opplan/exec/weights/load.rs:410-476 + quantize.rs:71-88.

    The shared exponent here is floor of the f64 log2 rounded to f32 -- the
    correctly rounded f32 log2, a different route to the number the C oracle
    gets from libm's log2f (they differ from the bit-pattern exponent at the
    top of a binade, where f32 log2 rounds up to the next integer).
    """
    x = np.asarray(values, F).reshape(rows, k // 32, 32)
    amax = np.abs(x).max(-1)
    with np.errstate(divide="ignore"):
        l2 = np.floor(np.log2(amax.astype(np.float64)).astype(F))  # f64 log2 rounded to f32, then floor
    e = np.where(amax > 0, l2, 0).astype(np.int64) - 2 + 127
    byte = np.where(amax == 0, 0, np.clip(e, 1, 254)).astype(np.uint8)
    s = e8m0(byte)
    with np.errstate(divide="ignore"):
        inv = np.where(s == 0, F(0), F(1.0) / s).astype(F)
    v = (x * inv[:, :, None]).astype(F)
    mag = np.minimum(np.abs(v), F(6.0))
    grid = MXFP4_TABLE[:8]
    err = np.abs(mag[..., None] - grid).astype(F)   # [...,8]
    best = np.zeros(mag.shape, np.int64)
    best_err = np.full(mag.shape, np.inf, F)
    for code in range(8):
        take = (err[..., code] < best_err) | ((err[..., code] == best_err) & (code % 2 == 0))
        best = np.where(take, code, best)
        best_err = np.where(take, err[..., code], best_err)
    sign = np.signbit(v).astype(np.int64) * 8
    code = np.where(best == 0, 0, sign | best).astype(np.uint8)
    packed = (code[..., 0::2] | (code[..., 1::2] << 4)).astype(np.uint8)
    return packed.reshape(-1), byte.reshape(-1)


def quantize_x_to_q8k(x):
    """Q8_K activation, written from the description in q4k_q8k_dot/mod.rs:12-27 and llama.cpp's convention:
    symmetric int8 over [-127, 127] per 256 values, d = absmax/127, per-32 sums of the codes."""
    x = np.asarray(x, np.float32).reshape(-1, 256)
    amax = np.abs(x).max(axis=1)
    with np.errstate(divide="ignore", invalid="ignore"):
        d = np.where(amax > 0, amax / np.float32(127.0), np.float32(0.0)).astype(np.float32)
        inv = np.where(d > 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    q = np.clip(rust_round((x * inv[:, None]).astype(np.float32)), -127.0, 127.0).astype(np.int8)
    sums = q.reshape(-1, 32).astype(np.int32).sum(axis=1).astype(np.int16)
    return q.reshape(-1), d, sums


def q4k_q8k_matvec(w, qs, d, sums, rows, cols):
    """Q4_K x Q8_K integer-dot matvec, vectorised differently from the oracle's loops: all integer sums first
    (exact), then the reference's float expression per super-block in f32, accumulated in order."""
    nb = cols // 256
    blocks = np.asarray(w, np.uint8)[: rows * nb * 144].reshape(rows, nb, 144)
    d_w, dmin_w, sc, mn = q4k_unpack_header(blocks.reshape(-1, 144))
    d_w, dmin_w = d_w.reshape(rows, nb), dmin_w.reshape(rows, nb)
    sc, mn = sc.reshape(rows, nb, 8).astype(np.int64), mn.reshape(rows, nb, 8).astype(np.int64)
    q = blocks[:, :, 16:].reshape(rows, nb, 4, 32)
    nib = np.stack([q & 0x0F, q >> 4], axis=3).reshape(rows, nb, 8, 32).astype(np.int64)  # sub-block 2g = low, 2g+1 = high
    y = np.asarray(qs, np.int8).reshape(nb, 8, 32).astype(np.int64)
    dots = (nib * y[None]).sum(axis=3)                                        # [rows, nb, 8]
    sum1 = (sc * dots).sum(axis=2)
    sum2 = (mn * np.asarray(sums, np.int16).reshape(nb, 8).astype(np.int64)[None]).sum(axis=2)
    dy = np.asarray(d, np.float32)[None, :]
    t1 = ((d_w * dy).astype(np.float32) * sum1.astype(np.float32)).astype(np.float32)
    t2 = ((dmin_w * dy).astype(np.float32) * sum2.astype(np.float32)).astype(np.float32)
    term = (t1 - t2).astype(np.float32)
    acc = np.zeros(rows, np.float32)
    for b in range(nb):
        acc = (acc + term[:, b]).astype(np.float32)
    return acc


def q6k_q8k_matvec(w, qs, d, rows, cols):
    """Q6_K x Q8_K integer-dot matvec from the layout description alone (ql[128] | qh[64] | 16 int8 scales | f16 d):
    element half*128 + plane*32 + l has the low nibble of ql[half*64 + (plane&1)*32 + l] for plane < 2 and the high
    nibble otherwise, and bits 2*plane, 2*plane+1 of qh[half*32 + l]; value = code - 32; scale per 16 elements."""
    nb = cols // 256
    blocks = np.asarray(w, np.uint8)[: rows * nb * 210].reshape(rows, nb, 210)
    ql = blocks[:, :, :128].reshape(rows, nb, 2, 2, 32)          # [half][ql row][l]
    qh = blocks[:, :, 128:192].reshape(rows, nb, 2, 32)
    sc = blocks[:, :, 192:208].view(np.int8).astype(np.int64)    # [rows, nb, 16]
    dw = f16_bits_to_f32(blocks[:, :, 208:210].copy().view(np.uint16)[:, :, 0])
    vals = np.empty((rows, nb, 2, 4, 32), np.int64)
    for plane in range(4):
        nib = (ql[:, :, :, plane & 1, :] & 0x0F) if plane < 2 else (ql[:, :, :, plane & 1, :] >> 4)
        hi = (qh >> (2 * plane)) & 3
        vals[:, :, :, plane, :] = (nib | (hi << 4)).astype(np.int64) - 32
    vals = vals.reshape(rows, nb, 16, 16)
    y = np.asarray(qs, np.int8).reshape(nb, 16, 16).astype(np.int64)
    sum1 = (sc * (vals * y[None]).sum(axis=3)).sum(axis=2)
    term = ((dw * np.asarray(d, np.float32)[None, :]).astype(np.float32) * sum1.astype(np.float32)).astype(np.float32)
    acc = np.zeros(rows, np.float32)
    for b in range(nb):
        acc = (acc + term[:, b]).astype(np.float32)
    return acc
