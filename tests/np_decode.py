"""Independent numpy decoders for the GGUF block formats, written from the
element-index maps of each format (not from the oracle's C code): they exist to
cross-check the oracle's decode on arbitrary byte patterns."""
import numpy as np


def _f16(raw2):  # (..., 2) uint8 -> f32
    return np.ascontiguousarray(raw2).view(np.float16).astype(np.float32)[..., 0]


def q8_0(raw):
    b = raw.reshape(-1, 34)
    d = _f16(b[:, 0:2])
    return (b[:, 2:].view(np.int8).astype(np.float32) * d[:, None]).reshape(-1)


def q4_k(raw):
    b = raw.reshape(-1, 144)
    d, dmin = _f16(b[:, 0:2]), _f16(b[:, 2:4])
    s = b[:, 4:16].astype(np.int32)
    sc = np.empty((b.shape[0], 8), np.int32)
    mn = np.empty_like(sc)
    sc[:, :4] = s[:, 0:4] & 63
    mn[:, :4] = s[:, 4:8] & 63
    sc[:, 4:] = (s[:, 8:12] & 0xF) | ((s[:, 0:4] >> 6) << 4)
    mn[:, 4:] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    qs = b[:, 16:].reshape(-1, 4, 32)
    q = np.stack([qs & 0xF, qs >> 4], axis=2).reshape(-1, 8, 32).astype(np.float32)  # [blk, pair, 32]
    d1 = (d[:, None] * sc.astype(np.float32)).astype(np.float32)
    m1 = (dmin[:, None] * mn.astype(np.float32)).astype(np.float32)
    return ((d1[:, :, None] * q).astype(np.float32) - m1[:, :, None]).astype(np.float32).reshape(-1)


def q2_k(raw):
    b = raw.reshape(-1, 84)
    scales = b[:, 0:16]
    qs = b[:, 16:80].reshape(-1, 2, 32)
    d, dmin = _f16(b[:, 80:82]), _f16(b[:, 82:84])
    q = np.stack([(qs >> (2 * f)) & 3 for f in range(4)], axis=2)  # [blk, sg, field, 32]
    q = q.reshape(-1, 16, 16).astype(np.float32)  # element e = sg*128 + field*32 + byte -> group e//16
    dl = (d[:, None] * (scales & 0xF).astype(np.float32)).astype(np.float32)
    ml = (dmin[:, None] * (scales >> 4).astype(np.float32)).astype(np.float32)
    return ((dl[:, :, None] * q).astype(np.float32) - ml[:, :, None]).astype(np.float32).reshape(-1)


def q6_k(raw):
    b = raw.reshape(-1, 210)
    ql = b[:, 0:128].reshape(-1, 2, 2, 32)   # [blk, half, which32, l]
    qh = b[:, 128:192].reshape(-1, 2, 32)    # [blk, half, l]
    sc = b[:, 192:208].view(np.int8).astype(np.float32)
    d = _f16(b[:, 208:210])
    out = np.empty((b.shape[0], 2, 4, 32), np.int32)
    for t in range(4):
        lo = ql[:, :, t & 1, :]
        nib = (lo & 0xF) if t < 2 else (lo >> 4)
        out[:, :, t, :] = (nib | (((qh >> (2 * t)) & 3) << 4)).astype(np.int32) - 32
    q = out.reshape(-1, 16, 16).astype(np.float32)
    ds = (d[:, None] * sc).astype(np.float32)
    return (ds[:, :, None] * q).astype(np.float32).reshape(-1)


_E2M1 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6], np.float32)


def mxfp4(raw):
    b = raw.reshape(-1, 17)
    e = b[:, 0].astype(np.uint32)
    bits = np.where(e == 0, np.uint32(0x00400000), e << 23).astype(np.uint32)
    d = bits.view(np.float32)
    codes = np.concatenate([b[:, 1:] & 0xF, b[:, 1:] >> 4], axis=1)
    with np.errstate(over="ignore", invalid="ignore"):
        y = d[:, None] * _E2M1[codes]
    y[e == 0xFF] = 0.0
    return y.astype(np.float32).reshape(-1)


def iq2_xxs(raw, grid):
    """grid: (256, 8) uint8 codebook."""
    b = raw.reshape(-1, 66)
    d = _f16(b[:, 0:2])
    w = np.ascontiguousarray(b[:, 2:]).view("<u4").reshape(-1, 8, 2)
    lo, hi = w[:, :, 0], w[:, :, 1]
    db = ((d[:, None] * (np.float32(0.5) + (hi >> 28).astype(np.float32))).astype(np.float32) * np.float32(0.25))
    out = np.empty((b.shape[0], 8, 4, 8), np.float32)
    for l in range(4):
        g = grid[(lo >> (8 * l)) & 0xFF].astype(np.float32)        # [blk, 8, 8]
        s7 = (hi >> (7 * l)) & 127
        par = np.zeros_like(s7)
        for bit in range(7):
            par ^= (s7 >> bit) & 1
        s8 = s7 | (par << 7)
        sign = np.where((s8[:, :, None] >> np.arange(8)) & 1, np.float32(-1), np.float32(1))
        out[:, :, l, :] = (db[:, :, None] * g).astype(np.float32) * sign
    return out.reshape(-1)


def _nibbles16(qs):  # (blk, 16) bytes -> (blk, 32): element j low nibble of byte j, element j + 16 its high nibble
    return np.concatenate([qs & 0xF, qs >> 4], axis=1).astype(np.int32)


def _fifth_bits(qh4):  # (blk, 4) bytes, little-endian u32 -> (blk, 32): bit e of the word
    word = np.ascontiguousarray(qh4).view("<u4")[:, 0]
    return ((word[:, None] >> np.arange(32, dtype=np.uint32)) & 1).astype(np.int32)


def q4_0(raw):
    b = raw.reshape(-1, 18)
    d = _f16(b[:, 0:2])
    return ((_nibbles16(b[:, 2:]) - 8).astype(np.float32) * d[:, None]).reshape(-1)


def q4_1(raw):
    b = raw.reshape(-1, 20)
    d, m = _f16(b[:, 0:2]), _f16(b[:, 2:4])
    return ((_nibbles16(b[:, 4:]).astype(np.float32) * d[:, None]).astype(np.float32) + m[:, None]).astype(np.float32).reshape(-1)


def q5_0(raw):
    b = raw.reshape(-1, 22)
    d = _f16(b[:, 0:2])
    q = _nibbles16(b[:, 6:]) + 16 * _fifth_bits(b[:, 2:6])
    return ((q - 16).astype(np.float32) * d[:, None]).reshape(-1)


def q5_1(raw):
    b = raw.reshape(-1, 24)
    d, m = _f16(b[:, 0:2]), _f16(b[:, 2:4])
    q = _nibbles16(b[:, 8:]) + 16 * _fifth_bits(b[:, 4:8])
    return ((q.astype(np.float32) * d[:, None]).astype(np.float32) + m[:, None]).astype(np.float32).reshape(-1)


def q3_k(raw):
    b = raw.reshape(-1, 110)
    hm, qs, sc = b[:, 0:32].astype(np.int32), b[:, 32:96].reshape(-1, 2, 32).astype(np.int32), b[:, 96:108].astype(np.int32)
    d = _f16(b[:, 108:110])
    low4 = np.concatenate([sc[:, 0:8] & 0xF, sc[:, 0:8] >> 4], axis=1)                      # scale i: nibble of byte i % 8
    high2 = np.stack([(sc[:, 8 + i % 4] >> (2 * (i // 4))) & 3 for i in range(16)], axis=1)  # two bits of byte 8 + i % 4
    scale = (low4 | (high2 << 4)) - 32                                                        # [blk, 16]
    out = np.empty((b.shape[0], 2, 4, 32), np.int32)
    for h in range(2):
        for t in range(4):
            third = (hm >> (4 * h + t)) & 1
            out[:, h, t, :] = ((qs[:, h, :] >> (2 * t)) & 3) - 4 * (1 - third)
    q = out.reshape(-1, 16, 16).astype(np.float32)
    dl = (d[:, None] * scale.astype(np.float32)).astype(np.float32)
    return (dl[:, :, None] * q).astype(np.float32).reshape(-1)


def q5_k(raw):
    b = raw.reshape(-1, 176)
    d, dmin = _f16(b[:, 0:2]), _f16(b[:, 2:4])
    s = b[:, 4:16].astype(np.int32)
    sc = np.empty((b.shape[0], 8), np.int32)
    mn = np.empty_like(sc)
    sc[:, :4] = s[:, 0:4] & 63
    mn[:, :4] = s[:, 4:8] & 63
    sc[:, 4:] = (s[:, 8:12] & 0xF) | ((s[:, 0:4] >> 6) << 4)
    mn[:, 4:] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    qh = b[:, 16:48].astype(np.int32)
    qs = b[:, 48:].reshape(-1, 4, 32).astype(np.int32)
    q = np.stack([qs & 0xF, qs >> 4], axis=2).reshape(-1, 8, 32)                      # [blk, sub-block, 32]
    q = q + 16 * ((qh[:, None, :] >> np.arange(8)[None, :, None]) & 1)
    d1 = (d[:, None] * sc.astype(np.float32)).astype(np.float32)
    m1 = (dmin[:, None] * mn.astype(np.float32)).astype(np.float32)
    return ((d1[:, :, None] * q.astype(np.float32)).astype(np.float32) - m1[:, :, None]).astype(np.float32).reshape(-1)
