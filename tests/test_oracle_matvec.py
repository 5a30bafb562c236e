"""Pins the oracle's matvec (both activation schemes) and prefill matmul.  CPU only.

Checks chosen so a dropped term, a wrong sign, a transposed nibble or a wrong scale index fails:
  * scheme F32: one-hot activations must return a column of deq(W) bit-exactly; general x vs an
    fp64 contraction of an INDEPENDENT numpy parse of the same bytes;
  * scheme Q8: the integer identity re-evaluated exactly (int64 sums, fp64 scales) from an
    independent numpy parse of the weight bytes and an independent numpy activation quantizer;
  * prefill: fp64 matmul of numpy-fp16-rounded deq(W) with the fp16 X.
"""
import numpy as np
import pytest

import ggufref as G

FORMATS = ["Q8_0", "Q4_0", "Q4_K", "Q5_K", "Q6_K"]


def deq_numpy(orc, t, rows, k):
    """Dequantize with ggufref's element-index parsers (fp64), independent of the oracle's loops."""
    if t == orc.Q4_0:
        d, q = G.parse_q4_0(rows, k)
        return (d[:, :, None] * q).reshape(rows.shape[0], k)
    if t == orc.Q8_0:
        d, q = G.parse_q8_0(rows, k)
        return (d[:, :, None] * q).reshape(rows.shape[0], k)
    if t in (orc.Q4_K, orc.Q5_K):
        d, dmin, sc, mn, q = (G.parse_q4_K if t == orc.Q4_K else G.parse_q5_K)(rows, k)
        n, nb = d.shape
        scale = (d[:, :, None] * sc).repeat(32, axis=2)
        minv = (dmin[:, :, None] * mn).repeat(32, axis=2)
        return (scale * q - minv).reshape(n, k)
    d, scales, q = G.parse_q6_K(rows, k)
    n, nb = d.shape
    return ((d[:, :, None] * scales).repeat(16, axis=2) * q).reshape(n, k)


@pytest.mark.parametrize("qname", FORMATS)
def test_dequant_matches_independent_parse(orc, qname):
    t = getattr(orc, qname)
    k = 1024
    rows = orc.quantize(t, G.seeded_weights(40, 6, k))
    want = deq_numpy(orc, t, rows, k)
    got = orc.dequantize(t, rows, k).astype(np.float64)
    # the oracle rounds d*sc and the product to fp32; the parse carries fp64
    assert np.max(np.abs(got - want)) <= 2e-7 * np.max(np.abs(want))


@pytest.mark.parametrize("qname", FORMATS)
def test_matvec_f32_one_hot_returns_columns(orc, qname):
    t = getattr(orc, qname)
    n, k = 24, 512
    rows = orc.quantize(t, G.seeded_weights(41, n, k))
    deq = orc.dequantize(t, rows, k)
    for col in (0, 15, 16, 31, 32, 255, 256, 300, 511):
        x = np.zeros(k, np.float32)
        x[col] = 1.0
        y = orc.matvec(t, orc.ACT_F32, rows, x, n, k)
        assert np.array_equal(y, deq[:, col]), col


@pytest.mark.parametrize("qname", FORMATS)
@pytest.mark.parametrize("batch", [1, 3, 8])
def test_matvec_f32_vs_fp64_of_independent_parse(orc, qname, batch):
    t = getattr(orc, qname)
    n, k = 40, 2048
    rows = orc.quantize(t, G.seeded_weights(42, n, k))
    x = G.seeded_acts(43, batch, k)
    want = x.astype(np.float64) @ deq_numpy(orc, t, rows, k).T
    got = orc.matvec(t, orc.ACT_F32, rows, x, n, k)
    assert got.shape == (batch, n)
    assert G.max_rel_err(got, want) < 2e-6
    assert G.max_rel_err(orc.matvec_f64(t, rows, x, n, k), want) < 1e-6


def q8_exact(orc, t, rows, x, k):
    """Scheme-Q8 result evaluated exactly: int64 block sums, fp64 scale products."""
    n = rows.shape[0]
    out = np.zeros((x.shape[0], n))
    for b in range(x.shape[0]):
        if t in (orc.Q4_0, orc.Q8_0):
            dx, qx = G.quant_q8_0_np(x[b])                       # independent activation quantizer
            dw, qw = (G.parse_q4_0 if t == orc.Q4_0 else G.parse_q8_0)(rows, k)
            isum = np.einsum("nbj,bj->nb", qw, qx)
            out[b] = (isum * dw * dx[None, :]).sum(axis=1)
        else:
            dx, qx, bs = G.parse_q8_K(orc.quantize(orc.Q8_K, x[b]), k)   # Q8_K itself is pinned in test_oracle_formats
            nb = k // 256
            if t in (orc.Q4_K, orc.Q5_K):
                d, dmin, sc, mn, q = (G.parse_q4_K if t == orc.Q4_K else G.parse_q5_K)(rows, k)
                sub = np.einsum("nbsj,bsj->nbs", q.reshape(n, nb, 8, 32), qx.reshape(nb, 8, 32))
                xs = qx.reshape(nb, 8, 32).sum(axis=2)               # explicit sums, not bsums
                out[b] = ((d * dx[None]) * (sc * sub).sum(axis=2) - (dmin * dx[None]) * (mn * xs[None]).sum(axis=2)).sum(axis=1)
            else:
                d, scales, q = G.parse_q6_K(rows, k)
                sub = np.einsum("nbsj,bsj->nbs", q.reshape(n, nb, 16, 16), qx.reshape(nb, 16, 16))
                out[b] = ((d * dx[None]) * (scales * sub).sum(axis=2)).sum(axis=1)
    return out


@pytest.mark.parametrize("qname", FORMATS)
@pytest.mark.parametrize("batch", [1, 4])
def test_matvec_q8_vs_exact_integer_identity(orc, qname, batch):
    t = getattr(orc, qname)
    n, k = 48, 2048
    rows = orc.quantize(t, G.seeded_weights(44, n, k))
    x = G.seeded_acts(45, batch, k)
    got = orc.matvec(t, orc.ACT_Q8, rows, x, n, k)
    assert G.max_rel_err(got, q8_exact(orc, t, rows, x, k)) < 2e-6


@pytest.mark.parametrize("qname", FORMATS)
def test_matvec_q8_is_close_to_f32_scheme_but_not_equal(orc, qname):
    """The two schemes differ by activation-quantization noise (~1e-2 of the output scale at
    K=4096): far above fp32 rounding, so parity must always compare like with like."""
    t = getattr(orc, qname)
    n, k = 64, 4096
    rows = orc.quantize(t, G.seeded_weights(46, n, k))
    x = G.seeded_acts(47, 1, k)[0]
    a = orc.matvec(t, orc.ACT_Q8, rows, x, n, k)
    b = orc.matvec(t, orc.ACT_F32, rows, x, n, k)
    gap = G.max_rel_err(a, b)
    assert 1e-5 < gap < 5e-2


def test_matvec_linearity_and_thread_invariance(orc):
    t, n, k = orc.Q4_K, 32, 1024
    rows = orc.quantize(t, G.seeded_weights(48, n, k))
    x = G.seeded_acts(49, 2, k)
    y = orc.matvec(t, orc.ACT_F32, rows, x, n, k)
    ysum = orc.matvec(t, orc.ACT_F32, rows, x[0] + x[1], n, k)
    assert G.max_rel_err(ysum, y[0] + y[1]) < 1e-5
    for scheme in (orc.ACT_F32, orc.ACT_Q8):
        y1 = orc.matvec(t, scheme, rows, x, n, k, nthreads=1)
        y4 = orc.matvec(t, scheme, rows, x, n, k, nthreads=4)
        assert np.array_equal(y1, y4)


def test_matvec_rejects_bad_shapes(orc):
    rows = np.zeros((4, 18 * 4), np.uint8)
    with pytest.raises(ValueError):
        orc.row_bytes(orc.Q4_0, 100)
    import ctypes as C
    L = orc.lib()
    x = np.zeros(128, np.float32)
    y = np.zeros(4, np.float32)
    vp = lambda a: C.c_void_p(a.ctypes.data)
    assert L.orc_matvec(orc.Q4_0, 0, vp(rows), vp(x), vp(y), 4, 100, 1, 1) == -1
    assert L.orc_matvec(orc.Q4_0, 0, vp(rows), vp(x), vp(y), 0, 128, 1, 1) == -1
    assert L.orc_matvec(orc.Q4_0, 7, vp(rows), vp(x), vp(y), 4, 128, 1, 1) == -1
    assert L.orc_matvec(orc.Q8_K, 0, vp(rows), vp(x), vp(y), 4, 256, 1, 1) == -1


@pytest.mark.parametrize("qname", ["Q4_0", "Q8_0", "Q4_K", "Q5_K", "Q6_K"])
def test_prefill_vs_fp64_of_fp16_rounded_weights(orc, qname):
    t = getattr(orc, qname)
    m, n, k = 9, 40, 1024
    rows = orc.quantize(t, G.seeded_weights(50, n, k))
    X = G.seeded_acts(51, m, k).astype(np.float16)
    w16 = orc.dequantize(t, rows, k).astype(np.float16).astype(np.float64)   # numpy's RNE, not the oracle's
    want = X.astype(np.float64) @ w16.T
    got = orc.prefill(t, rows, X, n, k)
    assert got.shape == (m, n)
    assert G.max_rel_err(got, want) < 2e-6
    # one row of the prefill equals the F32-scheme matvec on the same fp16 activations up to the
    # fp16 rounding of the weights (measured ~1.5e-4 of the output scale)
    mv = orc.matvec(t, orc.ACT_F32, rows, X[0].astype(np.float32), n, k)
    assert G.max_rel_err(got[0], mv) < 1e-3
