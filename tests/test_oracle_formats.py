"""Pins the CPU oracle's scalar helpers, quantizers and dequantizers.

No golden vector for this path exists in the reference tree, so each function is pinned by
what the format itself fixes: IEEE-754 (numpy.float16), hand-derived known-answer blocks,
independent element-index packers (ggufref.py) and invariants.  CPU only.
"""
import numpy as np
import pytest

import ggufref as G


# ----------------------------------------------------------------- fp16

def test_fp16_to_fp32_exhaustive(orc):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([orc.fp16_bits_to_fp32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_fp32_to_fp16_roundtrip_ties_and_random(orc):
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float32)
    finite = np.isfinite(vals)
    # every fp16 value converts back to itself
    for b, v in zip(bits[finite][::7], vals[finite][::7]):
        assert orc.fp32_to_fp16_bits(float(v)) == int(b)
    # exact midpoints between neighbouring positive fp16 values: ties go to even
    pos = np.arange(0, 0x7BFF, dtype=np.uint16)
    lo = pos.view(np.float16).astype(np.float64)
    hi = (pos + 1).view(np.float16).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)          # exactly representable in fp32
    assert np.array_equal(mid.astype(np.float64), (lo + hi) / 2)
    want = mid.astype(np.float16).view(np.uint16)
    for m, w in zip(mid[::5], want[::5]):
        assert orc.fp32_to_fp16_bits(float(m)) == int(w)
        assert orc.fp32_to_fp16_bits(float(-m)) == int(w) | 0x8000
    # random magnitudes across the whole exponent range incl. overflow and underflow
    rng = np.random.default_rng(7)
    r = (rng.standard_normal(40000) * np.exp(rng.uniform(-20, 12, 40000))).astype(np.float32)
    r = np.concatenate([r, np.float32([65504, 65519.99, 65520, 1e9, 2 ** -24, 2 ** -25, 2 ** -25 * 1.0001, 0, -0.0])])
    with np.errstate(over="ignore"):
        want = r.astype(np.float16).view(np.uint16)
    got = np.array([orc.fp32_to_fp16_bits(float(v)) for v in r], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_nearest_int_half_even(orc):
    ties = np.arange(-2000, 2000, dtype=np.float32) + np.float32(0.5)
    for v in ties:
        assert orc.nearest_int(float(v)) == int(np.rint(v))
    assert orc.nearest_int(0.5) == 0 and orc.nearest_int(1.5) == 2 and orc.nearest_int(2.5) == 2
    assert orc.nearest_int(-0.5) == 0 and orc.nearest_int(-1.5) == -2
    rng = np.random.default_rng(3)
    for v in (rng.standard_normal(5000) * 1000).astype(np.float32):
        assert orc.nearest_int(float(v)) == int(np.rint(v))


def test_block_sizes(orc):
    assert [orc.block_bytes(t) for t in (orc.Q8_0, orc.Q4_0, orc.Q4_K, orc.Q5_K, orc.Q6_K, orc.Q8_K)] == [34, 18, 144, 176, 210, 292]
    assert [orc.block_elems(t) for t in (orc.Q8_0, orc.Q4_0, orc.Q4_K, orc.Q5_K, orc.Q6_K, orc.Q8_K)] == [32, 32, 256, 256, 256, 256]
    assert orc.row_bytes(orc.Q4_0, 4096) == 2304 and orc.row_bytes(orc.Q6_K, 4096) == 3360
    with pytest.raises(ValueError):
        orc.row_bytes(orc.Q4_K, 4096 + 32)


# ------------------------------------------------------ Q8_0 known answers

def test_q8_0_known_answer_integers(orc):
    x = np.zeros(32, np.float32)
    x[:8] = [127, -127, 0, 1, 2, -3, 64, -64]
    x[8:] = np.arange(24) - 12
    blk = orc.quantize(orc.Q8_0, x)
    assert blk[0:2].tobytes() == b"\x00\x3c"                       # d = 1.0
    assert np.array_equal(blk[2:].view(np.int8), x.astype(np.int8))
    assert np.array_equal(orc.dequantize(orc.Q8_0, blk, 32), x)
    assert np.array_equal(blk, G.pack_q8_0(1.0, x.astype(np.int8)))


def test_q8_0_round_half_away_and_zero_block(orc):
    # d = 127/127 = 1: 0.5 -> 1, -0.5 -> -1, 2.5 -> 3 (away from zero, unlike half-even)
    x = np.zeros(32, np.float32)
    x[:5] = [127, 0.5, -0.5, 2.5, -2.5]
    q = orc.quantize(orc.Q8_0, x)[2:].view(np.int8)
    assert list(q[:5]) == [127, 1, -1, 3, -3]
    z = orc.quantize(orc.Q8_0, np.zeros(64, np.float32))
    assert not z.any()


def test_q8_0_rounds_the_rounded_product_not_the_exact_one(orc):
    """q = roundf(RN(x * id)): the reference rounds the product to fp32 before it rounds to an integer.  Inputs whose
    rounded product is a half-integer m + 1/2 reached from below: roundf gives m + 1, while rounding the exact
    product (or adding the half inside one fused multiply-add) gives m.  The oracle must do the former; the formula
    is evaluated here step by step in float32."""
    hits = 0
    for amax in (100.0, 3.7, 1.234567, 77.7, 0.9, 12.5, 640.0):
        A = np.float32(amax)
        d = np.float32(A / np.float32(127.0))
        idv = np.float32(np.float32(1.0) / d)
        base = ((np.arange(1, 127, dtype=np.float64) + 0.5) / np.float64(idv)).astype(np.float32)
        for k in range(-6, 7):
            x = base.copy()
            for _ in range(abs(k)):
                x = np.nextafter(x, np.float32(np.inf if k > 0 else -np.inf))
            t = (x * idv).astype(np.float32)                                    # the rounded product
            two_step = np.floor(t.astype(np.float64) + 0.5)
            one_step = np.floor(x.astype(np.float64) * np.float64(idv) + 0.5)   # rounding the exact product
            for xi, want in zip(x[(two_step != one_step) & (x <= A)], two_step[(two_step != one_step) & (x <= A)]):
                blk = np.zeros(32, np.float32)
                blk[0], blk[1], blk[2] = A, xi, -xi
                q = orc.quantize(orc.Q8_0, blk)[2:].view(np.int8)
                assert (int(q[0]), int(q[1]), int(q[2])) == (127, int(want), -int(want)), (amax, float(xi))
                hits += 1
    assert hits >= 8


def test_q8_0_closed_form_and_error_bound(orc):
    x = G.seeded_acts(11, 1, 4096)[0]
    blk = orc.quantize(orc.Q8_0, x).reshape(1, -1)
    d, q = G.parse_q8_0(blk, 4096)
    d_np, q_np = G.quant_q8_0_np(x)
    assert np.array_equal(d[0], d_np) and np.array_equal(q[0], q_np)
    err = np.abs(x.reshape(-1, 32) - d[0][:, None] * q[0])
    amax = np.abs(x.reshape(-1, 32)).max(axis=1)
    # half a step, plus 127 steps times the fp16 rounding of d (relative 2^-11)
    assert np.all(err <= (amax / 127 / 2 + amax * 2.0 ** -11 + 1e-7)[:, None])


# ------------------------------------------------------ Q4_0 known answers

def test_q4_0_negative_max_grid_is_exact(orc):
    k_idx = (np.arange(32) * 5) % 16           # 0 appears, so the extreme element is -4.0
    x = (0.5 * (k_idx - 8)).astype(np.float32)
    blk = orc.quantize(orc.Q4_0, x)
    assert blk[0:2].tobytes() == b"\x00\x38"   # d = 0.5
    assert np.array_equal(blk, G.pack_q4_0(0.5, k_idx))
    assert np.array_equal(orc.dequantize(orc.Q4_0, blk, 32), x)


def test_q4_0_positive_max_clamps_at_15(orc):
    x = np.zeros(32, np.float32)
    x[:4] = [8, -7, -8, 0]
    blk = orc.quantize(orc.Q4_0, x)
    assert blk[0:2].tobytes() == b"\x00\xbc"   # d = -1.0
    d, q = G.parse_q4_0(blk.reshape(1, -1), 32)
    assert list(q[0, 0, :4] + 8) == [0, 15, 15, 8]
    y = orc.dequantize(orc.Q4_0, blk, 32)
    assert list(y[:4]) == [8, -7, -7, 0]       # -8 is not representable when the max is +8


@pytest.mark.parametrize("e", range(32))
def test_q4_0_one_hot_nibble_order(orc, e):
    q = np.full(32, 8, np.uint8)
    q[e] = 11
    y = orc.dequantize(orc.Q4_0, G.pack_q4_0(2.0, q), 32)
    want = np.zeros(32, np.float32)
    want[e] = 6.0
    assert np.array_equal(y, want)


# ---------------------------------------------------------------- Q8_K

def test_q8_K_closed_form_and_bsums(orc):
    x = G.seeded_acts(5, 1, 1024)[0]
    x[256:512] = 0                                            # an all-zero super-block
    row = orc.quantize(orc.Q8_K, x)
    d, q, bs = G.parse_q8_K(row, 1024)
    assert d[1] == 0 and not q[1].any() and not bs[1].any()
    for b in (0, 2, 3):
        xb = x[256 * b:256 * b + 256]
        vmax = xb[np.argmax(np.abs(xb))]
        iscale = np.float32(-127.0) / np.float32(vmax)
        want = np.minimum(127, np.rint((iscale * xb).astype(np.float32))).astype(np.int64)
        assert np.array_equal(q[b], want)
        assert d[b] == np.float64(np.float32(1.0) / iscale)
        assert q[b].min() == -127                              # the extreme element maps to -127
    assert np.array_equal(bs, q.reshape(4, 16, 16).sum(axis=2))
    assert np.array_equal(bs.sum(axis=1), q.sum(axis=1))


# ---------------------------------------------------------------- Q4_K

def test_q4k_scale_field_pack_unpack_identity(orc):
    rng = np.random.default_rng(1)
    for _ in range(500):
        sc = rng.integers(0, 64, 8)
        mn = rng.integers(0, 64, 8)
        got_sc, got_mn = orc.q4k_scale_min(G.pack_q4k_scales(sc, mn))
        assert np.array_equal(got_sc, sc) and np.array_equal(got_mn, mn)
    # a hand-written field: distinct values, high bits used by entries 4..7 only
    sc = np.array([1, 2, 3, 4, 0x35, 0x26, 0x17, 0x3F])
    mn = np.array([5, 6, 7, 8, 0x1A, 0x2B, 0x3C, 0x0D])
    field = G.pack_q4k_scales(sc, mn)
    assert list(field) == [0x01 | 0xC0, 0x02 | 0x80, 0x03 | 0x40, 0x04 | 0xC0,
                           0x05 | 0x40, 0x06 | 0x80, 0x07 | 0xC0, 0x08 | 0x00,
                           0xA5, 0xB6, 0xC7, 0xDF]
    got_sc, got_mn = orc.q4k_scale_min(field)
    assert np.array_equal(got_sc, sc) and np.array_equal(got_mn, mn)


def test_q4_K_dequant_against_element_index_packer(orc):
    rng = np.random.default_rng(2)
    for _ in range(20):
        sc = rng.integers(0, 64, 8)
        mn = rng.integers(0, 64, 8)
        q = rng.integers(0, 16, 256)
        d, dmin = 0.0123, 0.0071
        blk = G.pack_q4_K(d, dmin, sc, mn, q)
        y = orc.dequantize(orc.Q4_K, blk, 256)
        assert np.array_equal(y, G.expected_q4_K(d, dmin, sc, mn, q).astype(np.float32))


def test_q4_K_one_hot_positions(orc):
    for e in (0, 31, 32, 63, 64, 100, 200, 255):
        q = np.zeros(256, np.int64)
        q[e] = 9
        blk = G.pack_q4_K(1.0, 0.0, np.arange(1, 9), np.zeros(8, np.int64), q)
        y = orc.dequantize(orc.Q4_K, blk, 256)
        want = np.zeros(256, np.float32)
        want[e] = 9.0 * (e // 32 + 1)
        assert np.array_equal(y, want)


def test_q4_K_quantizer_validity_and_error(orc):
    w = G.seeded_weights(21, 8, 1024)
    rows = orc.quantize(orc.Q4_K, w)
    d, dmin, sc, mn, q = G.parse_q4_K(rows, 1024)
    assert np.all(d >= 0) and np.all(dmin >= 0) and np.all(np.isfinite(d)) and np.all(np.isfinite(dmin))
    assert sc.max() <= 63 and mn.max() <= 63 and sc.max() == 63        # the largest sub-scale uses the full range
    y = orc.dequantize(orc.Q4_K, rows, 1024)
    rel_rms = np.sqrt(np.mean((y - w) ** 2)) / np.sqrt(np.mean(w ** 2))
    assert rel_rms < 0.09
    # every element is within one quantization step of its sub-block grid
    step = (d[:, :, None] * sc).repeat(32, axis=2).reshape(8, 1024)
    assert np.all(np.abs(y - w) <= step + 1e-6)
    assert not orc.quantize(orc.Q4_K, np.zeros(256, np.float32))[:4].any()


# ---------------------------------------------------------------- Q5_K

def test_q5_K_dequant_against_element_index_packer(orc):
    rng = np.random.default_rng(12)
    for _ in range(20):
        sc = rng.integers(0, 64, 8)
        mn = rng.integers(0, 64, 8)
        q = rng.integers(0, 32, 256)
        d, dmin = 0.0123, 0.0071
        blk = G.pack_q5_K(d, dmin, sc, mn, q)
        y = orc.dequantize(orc.Q5_K, blk, 256)
        assert np.array_equal(y, G.expected_q5_K(d, dmin, sc, mn, q).astype(np.float32))
        dd, mm, s2, m2, q2 = G.parse_q5_K(blk.reshape(1, -1), 256)
        assert np.array_equal(q2[0, 0], q) and np.array_equal(s2[0, 0], sc) and np.array_equal(m2[0, 0], mn)


def test_q5_K_one_hot_positions_and_fifth_bit(orc):
    for e in (0, 31, 32, 63, 64, 100, 200, 255):
        for v in (9, 16, 31):                         # low nibble only, fifth bit only, both
            q = np.zeros(256, np.int64)
            q[e] = v
            blk = G.pack_q5_K(1.0, 0.0, np.arange(1, 9), np.zeros(8, np.int64), q)
            y = orc.dequantize(orc.Q5_K, blk, 256)
            want = np.zeros(256, np.float32)
            want[e] = float(v) * (e // 32 + 1)
            assert np.array_equal(y, want), (e, v)
    # the fifth bits of element l of all eight sub-blocks share byte qh[l]
    q = np.zeros(256, np.int64)
    q[5::32] = 16
    blk = G.pack_q5_K(1.0, 0.0, np.ones(8, np.int64), np.zeros(8, np.int64), q)
    assert blk[16 + 5] == 0xFF and not np.delete(blk[16:48], 5).any() and not blk[48:].any()


def test_q5_K_quantizer_validity_and_error(orc):
    w = G.seeded_weights(22, 8, 1024)
    rows = orc.quantize(orc.Q5_K, w)
    d, dmin, sc, mn, q = G.parse_q5_K(rows, 1024)
    assert np.all(d >= 0) and np.all(dmin >= 0) and np.all(np.isfinite(d)) and np.all(np.isfinite(dmin))
    assert sc.max() == 63 and mn.max() <= 63 and q.max() == 31 and q.min() == 0
    y = orc.dequantize(orc.Q5_K, rows, 1024)
    rel_rms = np.sqrt(np.mean((y - w) ** 2)) / np.sqrt(np.mean(w ** 2))
    assert rel_rms < 0.045                              # about half of Q4_K's: one more bit
    step = (d[:, :, None] * sc).repeat(32, axis=2).reshape(8, 1024)
    assert np.all(np.abs(y - w) <= step + 1e-6)
    assert not orc.quantize(orc.Q5_K, np.zeros(256, np.float32))[:4].any()
    # the quantizer's bytes follow from its own sub-block fits (the search shared with Q4_K, 32 levels)
    blk = w[0, :256]
    fits = [orc.q5k_fit_subblock(blk[32 * j:32 * j + 32]) for j in range(8)]
    max_scale, max_min = max(f[0] for f in fits), max(f[1] for f in fits)
    assert np.float16(np.float32(max_scale) / np.float32(63.0)) == np.float16(d[0, 0])
    assert np.float16(np.float32(max_min) / np.float32(63.0)) == np.float16(dmin[0, 0])


# ---------------------------------------------------------------- Q6_K

def test_q6_K_dequant_against_element_index_packer(orc):
    rng = np.random.default_rng(4)
    for _ in range(20):
        L = rng.integers(0, 64, 256)
        scales = rng.integers(-128, 128, 16)
        blk = G.pack_q6_K(0.25, scales, L)
        y = orc.dequantize(orc.Q6_K, blk, 256)
        want = (np.float32(0.25) * scales.astype(np.float32)[np.arange(256) // 16]) * (L - 32).astype(np.float32)
        assert np.array_equal(y, want)


def test_q6_K_every_value_at_every_lane_position(orc):
    for v in range(64):
        for e in (3, 35, 67, 99, 128 + 17, 128 + 49, 128 + 81, 255):
            L = np.full(256, 32, np.int64)
            L[e] = v
            y = orc.dequantize(orc.Q6_K, G.pack_q6_K(1.0, np.ones(16, np.int8), L), 256)
            want = np.zeros(256, np.float32)
            want[e] = v - 32
            assert np.array_equal(y, want), (v, e)


def test_q6_K_quantizer_validity_and_error(orc):
    w = G.seeded_weights(22, 8, 1024)
    rows = orc.quantize(orc.Q6_K, w)
    d, scales, q = G.parse_q6_K(rows, 1024)
    assert np.all(np.isfinite(d)) and q.min() >= -32 and q.max() <= 31
    assert np.abs(scales).max() <= 128 and np.all(np.abs(scales).max(axis=2) >= 127)
    y = orc.dequantize(orc.Q6_K, rows, 1024)
    rel_rms = np.sqrt(np.mean((y - w) ** 2)) / np.sqrt(np.mean(w ** 2))
    assert rel_rms < 0.025
    step = np.abs(d[:, :, None] * scales).repeat(16, axis=2).reshape(8, 1024)
    assert np.all(np.abs(y - w) <= step + 1e-6)
    assert not orc.quantize(orc.Q6_K, np.zeros(256, np.float32)).any()


@pytest.mark.parametrize("qname", ["Q8_0", "Q4_0", "Q4_K", "Q5_K", "Q6_K"])
def test_requantizing_dequantized_rows_is_stable(orc, qname):
    """deq(quant(x)) lies on the format's grid, so quantizing it again must reproduce values
    within one ulp of the scale's fp16 rounding -- catches an encoder/decoder that disagree."""
    t = getattr(orc, qname)
    w = G.seeded_weights(30, 4, 512)
    y1 = orc.dequantize(t, orc.quantize(t, w), 512)
    y2 = orc.dequantize(t, orc.quantize(t, y1), 512)
    assert np.sqrt(np.mean((y2 - y1) ** 2)) <= 0.02 * np.sqrt(np.mean(y1 ** 2))


def test_truncating_round_half_away_matches_roundf_over_the_quantizers_range():
    """The device quantizers round halves away from zero as (int)(t + copysign(c, t)) with c the largest float below
    0.5 (one addition and a truncating conversion instead of roundf).  Every float from 0.25 up to 130 in magnitude --
    the quotients x / d of a Q8_0 block reach 127 -- and a sample below: the same integer as round-half-away computed
    exactly in float64."""
    c = np.float32(np.frombuffer(np.uint32(0x3EFFFFFF).tobytes(), dtype=np.float32)[0])
    lo, hi = np.float32(0.25).view(np.uint32), np.float32(130.0).view(np.uint32)
    step = 1 << 24
    for start in range(int(lo), int(hi) + 1, step):
        bits = np.arange(start, min(start + step, int(hi) + 1), dtype=np.uint32)
        for sign in (np.float32(1), np.float32(-1)):
            t = bits.view(np.float32) * sign
            fast = np.trunc(t + np.copysign(c, t)).astype(np.int32)           # float32 addition, as on the device
            t64 = t.astype(np.float64)
            ref = (np.sign(t64) * np.floor(np.abs(t64) + 0.5)).astype(np.int32)
            assert np.array_equal(fast, ref)
    small = np.linspace(0, 0.25, 100001, dtype=np.float32)
    assert not np.any(np.trunc(small + c)) and not np.any(np.trunc(-small - c))
    # the one value that defeats adding 0.5 itself: the largest float below one half
    t = np.float32(0.5) - np.float32(2.0 ** -25)
    assert np.trunc(t + np.float32(0.5)) == 1 and np.trunc(t + c) == 0


def test_division_by_127_as_two_fused_multiply_adds_is_exact():
    """x / 127 as q + fma(-q, 127, x) * r with q = x * r, r = RN(1 / 127): compared in exact rational arithmetic with the
    correctly rounded quotient on a dense sample (the device self-test covers every float; float64 fma is emulated
    exactly here because x, q and 127 are float32: the products fit in 53 bits)."""
    rng = np.random.default_rng(7)
    r = np.float32(1.0) / np.float32(127.0)
    bits = rng.integers(np.float32(2.0 ** -90).view(np.uint32), np.float32(2.0 ** 90).view(np.uint32), 2_000_000, dtype=np.uint32)
    x = bits.view(np.float32)
    q = (x * r).astype(np.float32)
    rem = (x.astype(np.float64) - q.astype(np.float64) * 127.0).astype(np.float32)     # exact product, one rounding: an fma
    fast = (rem.astype(np.float64) * np.float64(r) + q.astype(np.float64)).astype(np.float32)
    assert np.array_equal(fast, x / np.float32(127.0))
