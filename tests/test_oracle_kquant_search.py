"""Pins the scale searches of the oracle's Q4_K / Q6_K quantizers by what the mathematics fixes.

The reference tree holds no vector for these routines, so each property below is chosen so that a
plausible slip fails it: a wrong importance weight or a transposed normal-equation term fails the
least-squares checks; a wrong candidate count, range or a flipped comparison fails the
best-of-candidates checks; a wrong clamp or rounding fails the exact-grid round trips; a wrong
6-bit / int8 re-quantization of the sub-block scales fails the whole-block round trips.  All
comparisons against numpy are made in float64 from first principles (numpy.linalg.lstsq, explicit
enumeration of the candidate grids), not by re-running the oracle's own loop.
"""
import numpy as np
import pytest

import ggufref as G


def q4k_weights(x):
    x = x.astype(np.float64)
    return np.sqrt(np.mean(x * x)) + np.abs(x)


def werr(x, w, approx):
    return float(np.sum(w * (approx - x.astype(np.float64)) ** 2))


def lstsq_scale_min(x, w, L):
    """Weighted least squares x ~ a*L + b with b <= 0 (GGUF stores min = -b >= 0)."""
    sw = np.sqrt(w)
    A = np.stack([L.astype(np.float64), np.ones(len(L))], axis=1) * sw[:, None]
    sol = np.linalg.lstsq(A, x.astype(np.float64) * sw, rcond=None)[0]
    a, b = float(sol[0]), float(sol[1])
    if b > 0:                                                     # constrained to the origin
        a = float(np.linalg.lstsq((L.astype(np.float64) * sw)[:, None], x.astype(np.float64) * sw, rcond=None)[0][0])
        b = 0.0
    return a, b


def q4k_search(x, w):
    return kmin_search(x, w, 15, -1.0, 20)


def kmin_search(x, w, nmax, rmin, nstep):
    """The published search, stated from its description in float64 with numpy.linalg.lstsq as the fit:
    start from the plain grid of nmax steps over [min(x, 0), max]; then for s = 0..nstep round x onto the grid
    with nmax + rmin + 0.1*s steps over [current offset, max] (Q4_K: 15, -1.0, 20; Q5_K: 31, -0.5, 15), refit (scale, offset) by weighted least squares
    (offset <= 0) and keep the refit if its weighted error is smaller -- the kept offset becomes the
    lower end of the grids that follow.  Returns (levels, scale, offset, error, error of the plain grid, last step kept)."""
    xd = x.astype(np.float64)
    lo = min(float(xd.min()), 0.0)
    hi = float(xd.max())
    L = np.clip(np.rint(float(nmax) / (hi - lo) * (xd - lo)), 0, nmax)
    scale = (hi - lo) / float(nmax)
    best = plain = werr(x, w, scale * L + lo)
    last = -1
    for s in range(nstep + 1):
        Lc = np.clip(np.rint((nmax + rmin + 0.1 * s) / (hi - lo) * (xd - lo)), 0, nmax)
        if np.ptp(Lc) == 0:
            continue
        a, b = lstsq_scale_min(x, w, Lc)
        e = werr(x, w, a * Lc + b)
        if e < best:
            L, scale, lo, best, last = Lc, a, b, e, s
    return L, scale, lo, best, plain, last


def sub_blocks(seed, n, size, sigma=0.02):
    rng = np.random.default_rng(seed)
    for i in range(n):
        x = rng.standard_normal(size).astype(np.float32) * np.float32(sigma)
        if i % 5 == 1:
            x = np.abs(x) + np.float32(0.01)                      # all positive: the min must be 0
        if i % 5 == 2:
            x = x + np.float32(0.03)                              # mostly positive, a few below zero
        if i % 7 == 3:
            x[rng.integers(size)] *= np.float32(6.0)              # one outlier: refits beat the min/max grid
        yield x


# ------------------------------------------------------------------------------------ Q4_K

def test_q4k_exact_grid_roundtrips_exactly(orc):
    """A sub-block that already lies on a 16-level arithmetic grid must come back as that grid."""
    rng = np.random.default_rng(5)
    for scale, mn in ((0.25, 1.0), (0.5, 0.0), (0.03125, 0.21875), (2.0, 7.0)):
        L = rng.integers(0, 16, 32)
        L[rng.integers(32)] = 0
        L[(np.flatnonzero(L == 0)[0] + 1) % 32] = 15
        x = (np.float32(scale) * L.astype(np.float32) - np.float32(mn)).astype(np.float32)
        s, m, got = orc.q4k_fit_subblock(x)
        assert np.array_equal(got, L)
        assert s == pytest.approx(scale, rel=1e-6) and m == pytest.approx(mn, rel=1e-6, abs=1e-7)


def test_q4k_constant_and_zero_subblocks(orc):
    s, m, L = orc.q4k_fit_subblock(np.zeros(32, np.float32))
    assert (s, m) == (0.0, 0.0) and not L.any()
    s, m, L = orc.q4k_fit_subblock(np.full(32, -0.75, np.float32))     # constant negative: all in the min
    assert s == 0.0 and m == 0.75 and not L.any()


def test_q4k_fit_is_the_weighted_least_squares_optimum_of_its_levels(orc):
    """(scale, min) returned with levels L is either the plain min/max grid or the weighted
    least-squares line through (L, x) with weights sqrt(mean x^2) + |x| and min >= 0."""
    n_refit = 0
    for x in sub_blocks(11, 300, 32):
        s, m, L = orc.q4k_fit_subblock(x)
        assert m >= 0.0 and s >= 0.0 and L.max() <= 15
        w = q4k_weights(x)
        lo, hi = min(float(x.min()), 0.0), float(x.max())
        plain = (s == pytest.approx((hi - lo) / 15.0, rel=2e-6)) and (m == pytest.approx(-lo, rel=2e-6, abs=1e-9))
        if plain:
            continue
        n_refit += 1
        a, b = lstsq_scale_min(x, w, L)
        assert s == pytest.approx(a, rel=2e-4), (s, a)
        assert -m == pytest.approx(b, rel=2e-3, abs=2e-6 * max(1.0, abs(a) * 15)), (m, b)
    assert n_refit > 150                                               # the refits are what is being pinned


def test_q4k_result_is_the_outcome_of_the_published_search(orc):
    """Levels, scale, min and weighted error agree with an independent float64 statement of the search
    (a rounding tie that float32 and float64 break differently may send the two down different paths,
    so a few sub-blocks may differ -- but never to a worse error than the plain min/max grid)."""
    same = improved = n = 0
    ends = {0: [0, 0], 20: [0, 0]}                                      # kept last at the first / last step: [seen, same]
    for x in sub_blocks(12, 1500, 32):
        s, m, L = orc.q4k_fit_subblock(x)
        w = q4k_weights(x)
        got = werr(x, w, s * L.astype(np.float64) - m)
        Lr, a, b, err, plain, last = q4k_search(x, w)
        assert got <= plain * (1 + 1e-5) + 1e-12                       # never worse than the plain grid
        n += 1
        improved += err < plain * (1 - 1e-3)
        if last in ends:
            ends[last][0] += 1
            ends[last][1] += bool(np.array_equal(L, Lr))
        if np.array_equal(L, Lr):
            same += 1
            assert s == pytest.approx(a, rel=2e-4) and -m == pytest.approx(b, rel=2e-3, abs=2e-6 * max(1.0, abs(a) * 15))
            assert got == pytest.approx(err, rel=2e-3, abs=1e-12)
    assert same >= 0.97 * n and improved > 0.5 * n, (same, improved, n)
    for seen, ok in ends.values():                                      # both ends of the step range are searched
        assert seen >= 4 and ok >= 0.9 * seen, ends


def test_q4k_min_is_never_negative_and_is_zero_when_the_free_fit_would_add(orc):
    """GGUF stores min >= 0 (x ~ scale*L - min).  For data above zero the grid starts at 0 (the lower end
    is clamped to 0) and a refit whose free intercept comes out positive is redone through the origin:
    min = 0 and scale = sum(w x L) / sum(w L^2)."""
    rng = np.random.default_rng(13)
    zero_min = 0
    for i in range(200):
        x = (np.abs(rng.standard_normal(32)) * 0.02 + 0.001 * (i % 4)).astype(np.float32)
        s, m, L = orc.q4k_fit_subblock(x)
        assert m >= 0.0 and s > 0
        w = q4k_weights(x)
        sw = np.sqrt(w)
        A = np.stack([L.astype(np.float64), np.ones(32)], axis=1) * sw[:, None]
        free_b = float(np.linalg.lstsq(A, x.astype(np.float64) * sw, rcond=None)[0][1])
        if free_b > 1e-6:
            zero_min += 1
            assert m == 0.0
            origin = float(np.sum(w * x * L) / np.sum(w * L.astype(np.float64) ** 2))
            assert s == pytest.approx(origin, rel=2e-4) or s == pytest.approx(float(x.max()) / 15.0, rel=2e-6)
    assert zero_min > 20


def test_q4_K_block_on_exact_grids_roundtrips_bit_exactly(orc):
    """Whole super-block: sub-block j lies on the grid d0*k_j*L - m0*n_j with 6-bit k_j, n_j (63 present),
    so the 6-bit re-quantization of scales and mins, the fp16 d / dmin and the final level pass must
    reproduce every field and dequantize back to the input exactly."""
    rng = np.random.default_rng(14)
    for d0, m0 in ((2.0 ** -6, 2.0 ** -7), (2.0 ** -9, 2.0 ** -5), (0.0078125, 0.0)):
        kj = rng.integers(1, 64, 8)
        nj = rng.integers(0, 64, 8) if m0 else np.zeros(8, np.int64)
        kj[rng.integers(8)] = 63
        if m0:
            nj[rng.integers(8)] = 63
        L = rng.integers(0, 16, (8, 32))
        L[:, 0] = 0
        L[:, 1] = 15
        x = (np.float32(d0) * kj[:, None].astype(np.float32) * L.astype(np.float32)
             - np.float32(m0) * nj[:, None].astype(np.float32)).astype(np.float32).reshape(256)
        blk = orc.quantize(orc.Q4_K, x)
        d, dmin, sc, mn, q = G.parse_q4_K(blk.reshape(1, -1), 256)
        assert d[0, 0] == d0 and dmin[0, 0] == m0
        assert np.array_equal(sc[0, 0], kj) and np.array_equal(mn[0, 0], nj)
        assert np.array_equal(q[0, 0], L.reshape(256))
        assert np.array_equal(orc.dequantize(orc.Q4_K, blk, 256), x)


def test_q4_K_row_fields_follow_from_the_subblock_fits(orc):
    """Random data: d = h(max scale / 63), dmin = h(max min / 63), the 6-bit fields are the fits divided
    by those, and every level is the nearest grid point of the DEQUANTIZED grid (clamped to 0..15)."""
    w = G.seeded_weights(41, 4, 512)
    rows = orc.quantize(orc.Q4_K, w)
    d, dmin, sc, mn, q = G.parse_q4_K(rows, 512)
    for r in range(4):
        for b in range(2):
            fits = [orc.q4k_fit_subblock(w[r, 256 * b + 32 * j: 256 * b + 32 * j + 32]) for j in range(8)]
            smax = max(f[0] for f in fits)
            mmax = max(f[1] for f in fits)
            assert d[r, b] == float(np.float16(np.float32(smax) / np.float32(63)))
            assert dmin[r, b] == float(np.float16(np.float32(mmax) / np.float32(63)))
            for j in range(8):
                assert sc[r, b, j] == min(63, int(np.rint(np.float32(63) / np.float32(smax) * np.float32(fits[j][0]))))
                assert mn[r, b, j] == min(63, int(np.rint(np.float32(63) / np.float32(mmax) * np.float32(fits[j][1]))))
                step = d[r, b] * sc[r, b, j]
                if step == 0:
                    continue
                xs = w[r, 256 * b + 32 * j: 256 * b + 32 * j + 32].astype(np.float64)
                ideal = (xs + dmin[r, b] * mn[r, b, j]) / step
                near = np.clip(np.rint(ideal), 0, 15)
                tie = np.abs(ideal - np.floor(ideal) - 0.5) < 1e-4
                assert np.array_equal(q[r, b, 32 * j:32 * j + 32][~tie], near[~tie])


# ------------------------------------------------------------------------------------ Q5_K

def test_q5k_exact_grid_roundtrips_exactly(orc):
    """A sub-block that already lies on a 32-level arithmetic grid must come back as that grid."""
    rng = np.random.default_rng(25)
    for scale, mn in ((0.25, 1.0), (0.5, 0.0), (0.03125, 0.21875), (2.0, 7.0)):
        L = rng.integers(0, 32, 32)
        L[0], L[1] = 0, 31
        x = (np.float32(scale) * L.astype(np.float32) - np.float32(mn)).astype(np.float32)
        s, m, got = orc.q5k_fit_subblock(x)
        assert np.array_equal(got, L)
        assert s == pytest.approx(scale, rel=1e-6) and m == pytest.approx(mn, rel=1e-6, abs=1e-7)
    s, m, L = orc.q5k_fit_subblock(np.full(32, -0.75, np.float32))
    assert s == 0.0 and m == 0.75 and not L.any()


def test_q5k_result_is_the_outcome_of_the_published_search(orc):
    """Same statement of the search as Q4_K's with 32 levels and 16 candidate spacings 30.5 .. 32.0."""
    same = improved = n = n_refit = 0
    for x in sub_blocks(26, 1200, 32):
        s, m, L = orc.q5k_fit_subblock(x)
        assert m >= 0.0 and s >= 0.0 and L.max() <= 31
        w = q4k_weights(x)
        got = werr(x, w, s * L.astype(np.float64) - m)
        Lr, a, b, err, plain, last = kmin_search(x, w, 31, -0.5, 15)
        assert got <= plain * (1 + 1e-5) + 1e-12
        n += 1
        improved += err < plain * (1 - 1e-3)
        if np.array_equal(L, Lr):
            same += 1
            assert s == pytest.approx(a, rel=2e-4) and -m == pytest.approx(b, rel=2e-3, abs=2e-6 * max(1.0, abs(a) * 31))
            assert got == pytest.approx(err, rel=2e-3, abs=1e-12)
            if last >= 0:
                n_refit += 1
                a2, b2 = lstsq_scale_min(x, w, L)                      # and that fit is the least-squares line of its levels
                assert s == pytest.approx(a2, rel=2e-4)
    assert same >= 0.95 * n and improved > 0.4 * n and n_refit > 0.4 * n, (same, improved, n_refit, n)


def test_q5_K_block_on_exact_grids_roundtrips_bit_exactly(orc):
    rng = np.random.default_rng(27)
    for d0, m0 in ((2.0 ** -6, 2.0 ** -7), (2.0 ** -9, 2.0 ** -5), (0.0078125, 0.0)):
        kj = rng.integers(1, 64, 8)
        nj = rng.integers(0, 64, 8) if m0 else np.zeros(8, np.int64)
        kj[rng.integers(8)] = 63
        if m0:
            nj[rng.integers(8)] = 63
        L = rng.integers(0, 32, (8, 32))
        L[:, 0] = 0
        L[:, 1] = 31
        x = (np.float32(d0) * kj[:, None].astype(np.float32) * L.astype(np.float32)
             - np.float32(m0) * nj[:, None].astype(np.float32)).astype(np.float32).reshape(256)
        blk = orc.quantize(orc.Q5_K, x)
        d, dmin, sc, mn, q = G.parse_q5_K(blk.reshape(1, -1), 256)
        assert d[0, 0] == d0 and dmin[0, 0] == m0
        assert np.array_equal(sc[0, 0], kj) and np.array_equal(mn[0, 0], nj)
        assert np.array_equal(q[0, 0], L.reshape(256))
        assert np.array_equal(orc.dequantize(orc.Q5_K, blk, 256), x)


# ------------------------------------------------------------------------------------ Q6_K

def q6k_candidates(x):
    """(levels, scale, weighted error) of the 19 spacings -(32 + 0.1*s)/max, s = -9..9, weights x^2,
    each with its least-squares scale through the origin."""
    xd = x.astype(np.float64)
    vmax = xd[np.argmax(np.abs(xd))]
    w = xd * xd
    out = []
    for s in [0] + [t for t in range(-9, 10) if t != 0]:
        l = np.clip(np.rint(-(32.0 + 0.1 * s) / vmax * xd), -32, 31)
        den = float(np.sum(w * l * l))
        if den == 0:
            continue
        a = float(np.sum(w * xd * l)) / den
        out.append((l, a, float(np.sum(w * (a * l - xd) ** 2))))
    return out


def test_q6k_exact_grid_roundtrips_exactly(orc):
    rng = np.random.default_rng(21)
    for scale in (0.5, 0.0078125, 3.0):
        l = rng.integers(-31, 32, 16)
        l[rng.integers(16)] = -32                                    # the extreme level defines the spacing
        x = (np.float32(scale) * l.astype(np.float32)).astype(np.float32)
        s, L = orc.q6k_fit_subblock(x)
        assert np.array_equal(L.astype(np.int64) - 32, l) and s == pytest.approx(scale, rel=1e-6)
        # mirrored data (extreme element positive): the scale comes out negative, same levels
        s2, L2 = orc.q6k_fit_subblock(-x)
        assert np.array_equal(L2.astype(np.int64) - 32, l) and s2 == pytest.approx(-scale, rel=1e-6)
    s, L = orc.q6k_fit_subblock(np.zeros(16, np.float32))
    assert s == 0.0 and not L.any()


def test_q6k_scale_is_the_weighted_least_squares_scale_of_its_levels(orc):
    for x in sub_blocks(22, 300, 16):
        s, L = orc.q6k_fit_subblock(x)
        l = L.astype(np.float64) - 32
        assert l.min() >= -32 and l.max() <= 31
        xd = x.astype(np.float64)
        w = xd * xd
        sw = np.sqrt(w)
        a = float(np.linalg.lstsq((l * sw)[:, None], xd * sw, rcond=None)[0][0])
        assert s == pytest.approx(a, rel=1e-4)
        # the element of largest magnitude sits at (or next to) the extreme level -32
        assert l[np.argmax(np.abs(xd))] <= -29


def test_q6k_result_is_the_best_of_the_candidate_spacings(orc):
    """Weighted error (weights x^2) equals the smallest over the 19 spacings enumerated independently; a
    rounding tie broken differently in float32 may cost a fraction of a percent in a few sub-blocks."""
    improved = close = n = 0
    # [seen, matched] for clear wins of the coarse end of the range.  The fine end (+0.9) clamps the element
    # of largest magnitude, which the x^2 weights punish: it wins on no data tried (Gaussian, uniform,
    # outliers, data laid on that very grid), so its presence cannot change an output and is not pinned.
    ends = {-9: [0, 0]}
    order = [0] + [t for t in range(-9, 10) if t != 0]
    for x in sub_blocks(23, 1500, 16):
        s, L = orc.q6k_fit_subblock(x)
        xd = x.astype(np.float64)
        w = xd * xd
        got = float(np.sum(w * (s * (L.astype(np.float64) - 32) - xd) ** 2))
        cands = q6k_candidates(x)
        best = min(c[2] for c in cands)
        assert got <= cands[0][2] * (1 + 5e-3) + 1e-18              # never worse than the plain -32/max spacing
        assert got >= best * (1 - 5e-3)                               # and no spacing outside the published 19
        n += 1
        close += got <= best * (1 + 2e-3) + 1e-18
        improved += best < cands[0][2] * (1 - 1e-3)
        errs = [c[2] for c in cands]
        win = order[int(np.argmin(errs))] if len(cands) == 19 else None
        runner_up = sorted(errs)[1]
        if win in ends and best < runner_up * (1 - 1e-2):              # a clear win of an end spacing
            ends[win][0] += 1
            ends[win][1] += bool(np.array_equal(L.astype(np.float64) - 32, cands[int(np.argmin(errs))][0]))
    assert close >= 0.97 * n and improved > 0.1 * n, (close, improved, n)
    for seen, ok in ends.values():
        assert seen >= 5 and ok >= 0.9 * seen, ends


def test_q6_K_block_on_exact_grids_roundtrips_bit_exactly(orc):
    """Whole super-block on grids d0 * sc_g * l with int8 sc_g (one of them -128) and the level -32
    present in every sub-block: d, the int8 scales and all levels must come back exactly."""
    rng = np.random.default_rng(24)
    for d0 in (2.0 ** -10, 2.0 ** -14):
        sc = rng.integers(-127, 128, 16)
        sc[sc == 0] = 5
        sc[rng.integers(16)] = -128
        l = rng.integers(-31, 32, (16, 16))
        l[:, 3] = -32
        x = (np.float32(d0) * sc[:, None].astype(np.float32) * l.astype(np.float32)).astype(np.float32).reshape(256)
        blk = orc.quantize(orc.Q6_K, x)
        d, scales, q = G.parse_q6_K(blk.reshape(1, -1), 256)
        assert d[0, 0] == d0
        assert np.array_equal(scales[0, 0], sc)
        assert np.array_equal(q[0, 0], l.reshape(256))
        assert np.array_equal(orc.dequantize(orc.Q6_K, blk, 256), x)


def test_q6_K_row_fields_follow_from_the_subblock_fits(orc):
    w = G.seeded_weights(42, 4, 512)
    rows = orc.quantize(orc.Q6_K, w)
    d, scales, q = G.parse_q6_K(rows, 512)
    for r in range(4):
        for b in range(2):
            fits = [orc.q6k_fit_subblock(w[r, 256 * b + 16 * g: 256 * b + 16 * g + 16])[0] for g in range(16)]
            smax = fits[int(np.argmax(np.abs(fits)))]
            iscale = np.float32(-128.0) / np.float32(smax)
            assert d[r, b] == float(np.float16(np.float32(1.0) / iscale))
            for g in range(16):
                assert scales[r, b, g] == min(127, int(np.rint(iscale * np.float32(fits[g]))))
                step = d[r, b] * scales[r, b, g]
                if step == 0:
                    continue
                ideal = w[r, 256 * b + 16 * g: 256 * b + 16 * g + 16].astype(np.float64) / step
                near = np.clip(np.rint(ideal), -32, 31)
                tie = np.abs(ideal - np.floor(ideal) - 0.5) < 1e-4
                assert np.array_equal(q[r, b, 16 * g:16 * g + 16][~tie], near[~tie])
