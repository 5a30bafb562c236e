"""Independent numpy restatement of the GGUF block BYTE LAYOUTS, used to pin the oracle.

Everything here is written element-index first ("where does element e of the block live")
rather than loop-over-bytes as the oracle does, so a transposed nibble, a wrong scale index
or a swapped field shows up as a mismatch between the two.
"""
import numpy as np


def f16_bytes(v):
    return np.array([v], dtype=np.float16).view(np.uint8)


# ---------------------------------------------------------------- Q4_0 / Q8_0

def pack_q4_0(d, q):
    """d: python float representable in fp16; q[32] ints in 0..15 (element order)."""
    q = np.asarray(q, dtype=np.uint8)
    out = np.zeros(18, dtype=np.uint8)
    out[0:2] = f16_bytes(d)
    for e in range(32):
        byte = 2 + (e % 16)
        out[byte] |= q[e] << (0 if e < 16 else 4)
    return out


def parse_q4_0(rows, k):
    """uint8 [n, k/32*18] -> (d float64 [n, nb], q int64 [n, nb, 32]) with q already minus 8."""
    n = rows.shape[0]
    nb = k // 32
    b = rows.reshape(n, nb, 18)
    d = b[:, :, 0:2].copy().view(np.float16).astype(np.float64).reshape(n, nb)
    qs = b[:, :, 2:].astype(np.int64)
    q = np.concatenate([qs & 0xF, qs >> 4], axis=2) - 8
    return d, q


def pack_q8_0(d, q):
    out = np.zeros(34, dtype=np.uint8)
    out[0:2] = f16_bytes(d)
    out[2:] = np.asarray(q, dtype=np.int8).view(np.uint8)
    return out


def parse_q8_0(rows, k):
    n = rows.shape[0]
    nb = k // 32
    b = rows.reshape(n, nb, 34)
    d = b[:, :, 0:2].copy().view(np.float16).astype(np.float64).reshape(n, nb)
    q = b[:, :, 2:].copy().view(np.int8).astype(np.int64)
    return d, q


# ---------------------------------------------------------------------- Q4_K

def pack_q4k_scales(sc, mn):
    """Eight 6-bit scales and mins -> the 12-byte field, from the layout's description:
    bytes 0-3 low6 = sc[0..3], bytes 4-7 low6 = mn[0..3], bytes 8-11 = low4(sc[4..7]) | low4(mn[4..7])<<4,
    the top two bits of bytes 0-3 carry sc[4..7]>>4 and of bytes 4-7 carry mn[4..7]>>4."""
    out = np.zeros(12, dtype=np.uint8)
    for j in range(4):
        out[j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
        out[4 + j] = (mn[j] & 63) | ((mn[j + 4] >> 4) << 6)
        out[8 + j] = (sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4)
    return out


def pack_q4_K(d, dmin, sc, mn, q):
    """q[256] in 0..15 in element order."""
    out = np.zeros(144, dtype=np.uint8)
    out[0:2] = f16_bytes(d)
    out[2:4] = f16_bytes(dmin)
    out[4:16] = pack_q4k_scales(sc, mn)
    for e in range(256):
        chunk, r = divmod(e, 64)
        byte = 16 + 32 * chunk + (r % 32)
        out[byte] |= np.uint8(q[e]) << (0 if r < 32 else 4)
    return out


def expected_q4_K(d, dmin, sc, mn, q):
    e = np.arange(256)
    sb = e // 32
    d = np.float32(np.float16(d))
    dmin = np.float32(np.float16(dmin))
    return (d * np.asarray(sc, np.float32)[sb]) * np.asarray(q, np.float32) - dmin * np.asarray(mn, np.float32)[sb]


def parse_q4_K(rows, k):
    """-> d, dmin float64 [n, nb]; sc, mn int64 [n, nb, 8]; q int64 [n, nb, 256] (element order)."""
    n = rows.shape[0]
    nb = k // 256
    b = rows.reshape(n, nb, 144)
    d = b[:, :, 0:2].copy().view(np.float16).astype(np.float64).reshape(n, nb)
    dmin = b[:, :, 2:4].copy().view(np.float16).astype(np.float64).reshape(n, nb)
    s = b[:, :, 4:16].astype(np.int64)
    sc = np.zeros((n, nb, 8), np.int64)
    mn = np.zeros((n, nb, 8), np.int64)
    sc[:, :, 0:4] = s[:, :, 0:4] & 63
    mn[:, :, 0:4] = s[:, :, 4:8] & 63
    sc[:, :, 4:8] = (s[:, :, 8:12] & 15) | ((s[:, :, 0:4] >> 6) << 4)
    mn[:, :, 4:8] = (s[:, :, 8:12] >> 4) | ((s[:, :, 4:8] >> 6) << 4)
    qs = b[:, :, 16:].astype(np.int64).reshape(n, nb, 4, 32)
    q = np.concatenate([qs & 15, qs >> 4], axis=3).reshape(n, nb, 256)
    return d, dmin, sc, mn, q


# ---------------------------------------------------------------------- Q5_K

def pack_q5_K(d, dmin, sc, mn, q):
    """q[256] in 0..31 in element order.  Layout from the format's description: fp16 d, fp16 dmin, the
    12-byte scale field of Q4_K, qh[32] (bit j of qh[l] = fifth bit of element l of sub-block j), qs[128]
    (low nibble of byte 32c+l = element l of sub-block 2c, high nibble = element l of sub-block 2c+1)."""
    out = np.zeros(176, dtype=np.uint8)
    out[0:2] = f16_bytes(d)
    out[2:4] = f16_bytes(dmin)
    out[4:16] = pack_q4k_scales(sc, mn)
    for e in range(256):
        sb, l = divmod(e, 32)
        v = int(q[e])
        out[16 + l] |= np.uint8((v >> 4) << sb)
        out[48 + 32 * (sb // 2) + l] |= np.uint8((v & 15) << (4 * (sb % 2)))
    return out


def expected_q5_K(d, dmin, sc, mn, q):
    return expected_q4_K(d, dmin, sc, mn, q)          # same arithmetic, q runs to 31


def parse_q5_K(rows, k):
    """-> d, dmin float64 [n, nb]; sc, mn int64 [n, nb, 8]; q int64 [n, nb, 256] (element order, 0..31)."""
    n = rows.shape[0]
    nb = k // 256
    b = rows.reshape(n, nb, 176)
    as144 = np.concatenate([b[:, :, :16], b[:, :, 48:]], axis=2).reshape(n, nb * 144)
    d, dmin, sc, mn, q4 = parse_q4_K(as144, k)
    qh = b[:, :, 16:48].astype(np.int64)                                    # [n, nb, 32]
    hi = np.stack([(qh >> j) & 1 for j in range(8)], axis=2).reshape(n, nb, 256)
    return d, dmin, sc, mn, q4 + 16 * hi


# ---------------------------------------------------------------------- Q6_K

def pack_q6_K(d, scales, L):
    """L[256] in 0..63 (element order, i.e. q+32); scales int8[16]."""
    out = np.zeros(210, dtype=np.uint8)
    for e in range(256):
        half, r = divmod(e, 128)
        quarter, l = divmod(r, 32)
        v = int(L[e])
        ql_idx = 64 * half + l + 32 * (quarter & 1)
        out[ql_idx] |= (v & 15) << (0 if quarter < 2 else 4)
        out[128 + 32 * half + l] |= (v >> 4) << (2 * quarter)
    out[192:208] = np.asarray(scales, dtype=np.int8).view(np.uint8)
    out[208:210] = f16_bytes(d)
    return out


def parse_q6_K(rows, k):
    """-> d float64 [n, nb]; scales int64 [n, nb, 16]; q int64 [n, nb, 256] (minus 32)."""
    n = rows.shape[0]
    nb = k // 256
    b = rows.reshape(n, nb, 210)
    d = b[:, :, 208:210].copy().view(np.float16).astype(np.float64).reshape(n, nb)
    scales = b[:, :, 192:208].copy().view(np.int8).astype(np.int64)
    e = np.arange(256)
    half, r = np.divmod(e, 128)
    quarter, l = np.divmod(r, 32)
    ql_idx = 64 * half + l + 32 * (quarter & 1)
    lo = (b[:, :, ql_idx].astype(np.int64) >> np.where(quarter < 2, 0, 4)) & 15
    hi = (b[:, :, 128 + 32 * half + l].astype(np.int64) >> (2 * quarter)) & 3
    return d, scales, (lo | (hi << 4)) - 32


# --------------------------------------------------- activation quantizers

def round_half_away(v32):
    v = v32.astype(np.float64)
    return np.sign(v) * np.floor(np.abs(v) + 0.5)


def quant_q8_0_np(x):
    """Closed form of the Q8_0 activation quantizer in numpy: returns (d fp16-rounded as float64 [nb], q int64 [nb, 32])."""
    xb = np.asarray(x, np.float32).reshape(-1, 32)
    amax = np.abs(xb).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        idv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
    q = round_half_away((xb * idv[:, None]).astype(np.float32)).astype(np.int64)
    return d.astype(np.float16).astype(np.float64), q


def parse_q8_K(row, k):
    nb = k // 256
    b = row.reshape(nb, 292)
    d = b[:, 0:4].copy().view(np.float32).astype(np.float64).reshape(nb)
    q = b[:, 4:260].copy().view(np.int8).astype(np.int64)
    bs = b[:, 260:292].copy().view(np.int16).astype(np.int64)
    return d, q, bs


# ------------------------------------------------------ seeded test inputs

def seeded_weights(seed, n, k, sigma=0.02):
    return (np.random.default_rng(seed).standard_normal((n, k), dtype=np.float32) * np.float32(sigma)).astype(np.float32)


def seeded_acts(seed, batch, k):
    return np.random.default_rng(seed).standard_normal((batch, k), dtype=np.float32)


def max_rel_err(y, ref):
    """max_i |y_i - ref_i| / max_j |ref_j|  -- the parity gate's denominator is the output's scale,
    because element-wise relative error is unbounded where ref_i ~ 0."""
    y = np.asarray(y, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.max(np.abs(y - ref)) / max(np.max(np.abs(ref)), 1e-30))
