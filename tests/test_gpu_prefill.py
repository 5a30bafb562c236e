"""GPU parity of the quantized prefill matmul (Q4_0 / Q8_0 and Q4_K / Q5_K / Q6_K weights, fp16 activations,
fp16 MFMA with fp32 accumulation) against the CPU oracle, through the C ABI.

Oracle definition: Y[m][n] = sum_k h(deq(W)[n][k]) * X[m][k] with h = round-to-nearest-even to fp16 and
fp32 accumulation.  The kernels form the fp16 weight bit-exactly (h(d*q); for the K-quants the reference's
fp32 dequantization operation by operation, then h), so only the accumulation order differs.
Gate (north_star): max|y - ref| / max|ref| <= 1e-3; asserted: PARITY_TOL.
"""
import sys

import numpy as np
import pytest

import ggufref as G
from openagents_amd import _ffi, backend

pytestmark = pytest.mark.gpu

GATE = 1e-3
PARITY_TOL = 2e-5
TILES = [(64, 64), (64, 128), (128, 128), (128, 256), (256, 128), (256, 256)]


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


_cache = {}


def weights(orc, qname, seed, n, k):
    key = (qname, seed, n, k)
    if key not in _cache:
        _cache[key] = orc.quantize(getattr(orc, qname), G.seeded_weights(seed, n, k))
    return _cache[key]


@pytest.mark.parametrize("qname", ["Q4_0", "Q8_0"])
@pytest.mark.parametrize("tile", TILES)
def test_every_tile_ragged_shapes(hip, orc, qname, tile):
    """m and n are ragged against every tile; k = 768 and 1280 exercise the partial last round of the
    256-wide register chunks for the 64- and 128-column tiles."""
    t = getattr(orc, qname)
    for m, n, k in ((1, 70, 768), (37, 300, 1280), (200, 130, 512), (333, 516, 1024)):
        say(f"prefill {qname} tile={tile} m={m} n={n} k={k}")
        W = weights(orc, qname, 800, n, k)
        X = G.seeded_acts(801 + m, m, k).astype(np.float16)
        ref = orc.prefill(t, W, X, n, k)
        ws = tile in ((64, 64), (64, 128), (128, 128), (128, 256))   # tiles with the producer/consumer (16) kernel
        for waves in (4,) + ((16,) if ws else ()):
            for ksplit in (1, 2, 4):
                if ksplit > 1 and (m * n) % 4:
                    continue
                y = hip.matmul_host(t, W, X, n, k, tile + (ksplit, waves))
                err = G.max_rel_err(y, ref)
                assert np.all(np.isfinite(y)) and err < PARITY_TOL, (tile, ksplit, waves, m, n, k, err)


@pytest.mark.parametrize("qname", ["Q4_K", "Q5_K", "Q6_K"])
@pytest.mark.parametrize("tile", TILES)
def test_k_quant_prefill_every_tile_ragged_shapes(hip, orc, qname, tile):
    """The K-quants run the four-wave family: weights dequantized in fp32 exactly as the reference does
    (one rounding per operation) and rounded to fp16 for the MFMA.  Ragged m and n against every tile; k of
    three and five super-blocks exercises the partial last round of the register chunks; Q6_K's 210-byte
    super-blocks put every second one on an odd dword boundary."""
    t = getattr(orc, qname)
    for m, n, k in ((1, 70, 768), (37, 300, 1280), (200, 130, 512), (333, 516, 1024)):
        say(f"prefill {qname} tile={tile} m={m} n={n} k={k}")
        W = weights(orc, qname, 830, n, k)
        X = G.seeded_acts(831 + m, m, k).astype(np.float16)
        ref = orc.prefill(t, W, X, n, k)
        families = (4, 16) if tile == (128, 256) and qname != "Q6_K" else (4,)   # Q4_K / Q5_K: also the producer / consumer kernel
        for waves in families:
            for ksplit in (1, 2, 4):
                if ksplit > 1 and (m * n) % 4:
                    continue
                y = hip.matmul_host(t, W, X, n, k, tile + (ksplit, waves))
                err = G.max_rel_err(y, ref)
                assert np.all(np.isfinite(y)) and err < PARITY_TOL, (tile, ksplit, waves, m, n, k, err)


@pytest.mark.parametrize("qname", ["Q4_K", "Q5_K", "Q6_K"])
def test_k_quant_prefill_default_plan_and_refusals(hip, orc, qname):
    """psn_qmatmul_prefill picks a four-wave tile by itself for the K-quants (a slice of the 4096 -> 14336
    projection at M = 64 and M = 512); the other kernel families exist for Q4_0 / Q8_0 only."""
    t = getattr(orc, qname)
    n, k = 1024, 4096
    W = weights(orc, qname, 840, n, k)
    for m in (64, 512):
        say(f"prefill {qname} default plan m={m} n={n} k={k}")
        X = G.seeded_acts(841 + m, m, k).astype(np.float16)
        err = G.max_rel_err(hip.matmul_host(t, W, X, n, k), orc.prefill(t, W, X, n, k))
        say(f"  max_rel_err={err:.3e}")
        assert err < PARITY_TOL
    X = G.seeded_acts(842, 64, k).astype(np.float16)
    for tile in ((128, 128, 1, 16), (256, 256, 1, 32)):
        with pytest.raises(backend.PsnError) as e:
            hip.matmul_host(t, W, X, n, k, tile)
        assert e.value.code == _ffi.E_UNSUPPORTED


@pytest.mark.parametrize("qname", ["Q4_0", "Q8_0", "Q4_K", "Q5_K", "Q6_K"])
def test_skinny_kernel_ragged_shapes(hip, orc, qname):
    """The M <= 64 kernel (waves code 64): every combination of ragged m and n, K ranges of one to many
    256-wide chunks (one chunk: the load rings are deeper than the whole range), with and without K split.
    Q6_K rows must be whole 16-byte words (K a multiple of 2048); its eight chunks per 2048 start at all eight
    possible offsets inside their aligned windows."""
    t = getattr(orc, qname)
    shapes = ((1, 70, 256), (37, 300, 768), (64, 130, 1280), (50, 516, 4096), (64, 64, 14336))
    if qname == "Q6_K":
        shapes = ((1, 70, 2048), (37, 300, 4096), (64, 130, 6144), (50, 516, 4096), (64, 64, 14336))
        with pytest.raises(backend.PsnError) as e:
            hip.matmul_host(t, weights(orc, qname, 859, 70, 768), G.seeded_acts(1, 4, 768).astype(np.float16), 70, 768, (64, 64, 1, 64))
        assert e.value.code == _ffi.E_UNSUPPORTED
    for m, n, k in shapes:
        say(f"skinny {qname} m={m} n={n} k={k}")
        W = weights(orc, qname, 860, n, k)
        X = G.seeded_acts(861 + m, m, k).astype(np.float16)
        ref = orc.prefill(t, W, X, n, k)
        for ksplit in (1, 2, 4, 8):
            if ksplit > 1 and (m * n) % 4:
                continue
            y = hip.matmul_host(t, W, X, n, k, (64, 64, ksplit, 64))
            err = G.max_rel_err(y, ref)
            assert np.all(np.isfinite(y)) and err < PARITY_TOL, (ksplit, m, n, k, err)
    # the result without K split does not depend on the run (fixed summation order)
    W = weights(orc, qname, 860, 516, 4096)
    X = G.seeded_acts(861 + 50, 50, 4096).astype(np.float16)
    ys = [hip.matmul_host(t, W, X, 516, 4096, (64, 64, 1, 64)) for _ in range(3)]
    assert np.array_equal(ys[0], ys[1]) and np.array_equal(ys[0], ys[2])
    with pytest.raises(backend.PsnError) as e:
        hip.matmul_host(t, W, G.seeded_acts(1, 65, 4096).astype(np.float16), 516, 4096, (64, 64, 1, 64))
    assert e.value.code == _ffi.E_UNSUPPORTED


@pytest.mark.parametrize("qname", ["Q4_0", "Q8_0"])
def test_prefill_m1_matches_matvec_f32_scheme(hip, orc, qname):
    """One row of the prefill is the F32-scheme matvec on the same fp16 activations, up to the fp16
    rounding of the weights (about 1.5e-4 of the output scale)."""
    t = getattr(orc, qname)
    n, k = 512, 4096
    W = weights(orc, qname, 810, n, k)
    X = G.seeded_acts(811, 1, k).astype(np.float16)
    y = hip.matmul_host(t, W, X, n, k)
    mv = hip.matvec_host(t, W, X[0].astype(np.float32), n, k, _ffi.ACT_F32)
    assert G.max_rel_err(y[0], mv) < GATE


@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("qname", ["Q4_0", "Q8_0", "Q4_K", "Q5_K", "Q6_K"])
def test_prefill_baseline_shapes_m64(hip, orc, qname, n, k):
    say(f"prefill {qname} m=64 n={n} k={k} (full oracle)")
    t = getattr(orc, qname)
    W = weights(orc, qname, 820, n, k)
    X = G.seeded_acts(821, 64, k).astype(np.float16)
    y = hip.matmul_host(t, W, X, n, k)
    err = G.max_rel_err(y, orc.prefill(t, W, X, n, k))
    say(f"  max_rel_err={err:.3e}")
    assert err < PARITY_TOL


@pytest.mark.parametrize("m", [512, 2048])
@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("qname", ["Q4_0", "Q8_0"])
def test_prefill_baseline_shapes_large_m_sampled(hip, orc, qname, m, n, k):
    """The GPU computes the full [m, n] product; the oracle re-computes a sample of 96 activation rows x
    160 weight rows (tile corners, edges and random interior rows) that the full result must match."""
    t = getattr(orc, qname)
    say(f"prefill {qname} m={m} n={n} k={k} (sampled oracle)")
    W = weights(orc, qname, 820, n, k)
    X = G.seeded_acts(830 + m, m, k).astype(np.float16)
    y = hip.matmul_host(t, W, X, n, k)
    rng = np.random.default_rng(m + n)
    mi = np.unique(np.concatenate([[0, 31, 32, 63, 64, 127, 128, 255, 256, m - 1], rng.integers(0, m, 86)]))
    ni = np.unique(np.concatenate([[0, 31, 32, 63, 64, 127, 128, 255, 256, n - 1], rng.integers(0, n, 150)]))
    ref = orc.prefill(t, W[ni], X[mi], len(ni), k)
    err = G.max_rel_err(y[np.ix_(mi, ni)], ref)
    say(f"  max_rel_err={err:.3e}")
    assert err < PARITY_TOL
    assert np.all(np.isfinite(y))


def test_prefill_linearity_and_zero(hip, orc):
    """Size-independent properties at a full shape: Y(X1 + X2) = Y(X1) + Y(X2) when X1, X2 have disjoint
    supports (exact in fp16), and zero activations give exactly zero."""
    t, n, k, m = orc.Q8_0, 4096, 4096, 128
    W = weights(orc, "Q8_0", 840, n, k)
    X = G.seeded_acts(841, m, k).astype(np.float16)
    X1, X2 = X.copy(), X.copy()
    X1[:, k // 2:] = 0
    X2[:, :k // 2] = 0
    y, y1, y2 = (hip.matmul_host(t, W, A, n, k) for A in (X, X1, X2))
    assert G.max_rel_err(y, y1 + y2) < PARITY_TOL
    assert not hip.matmul_host(t, W, np.zeros((m, k), np.float16), n, k).any()


@pytest.mark.parametrize("qname", ["Q4_0", "Q8_0"])
def test_wide_kernel_ragged_shapes(hip, orc, qname):
    """The large-M kernel (waves code 32, 256 x 256 tiles, weights decoded from raw bytes by the multiplying
    wave): ragged m and n against the tile, K ranges from one 256-chunk (the load rings are as deep as the
    whole range) to many, with and without K split; the result without K split is the same on every run."""
    t = getattr(orc, qname)
    for m, n, k in ((256, 256, 256), (1, 70, 512), (300, 296, 1280), (512, 768, 2048), (257, 513, 4096), (640, 260, 3584)):
        say(f"wide {qname} m={m} n={n} k={k}")
        W = weights(orc, qname, 870, n, k)
        X = G.seeded_acts(871 + m, m, k).astype(np.float16)
        ref = orc.prefill(t, W, X, n, k)
        for ksplit in (1, 2, 4):
            if ksplit > 1 and ((m * n) % 4 or k // 256 < ksplit):
                continue
            y = hip.matmul_host(t, W, X, n, k, (256, 256, ksplit, 32))
            err = G.max_rel_err(y, ref)
            assert np.all(np.isfinite(y)) and err < PARITY_TOL, (ksplit, m, n, k, err)
    W = weights(orc, qname, 870, 513, 4096)
    X = G.seeded_acts(871 + 257, 257, 4096).astype(np.float16)
    ys = [hip.matmul_host(t, W, X, 513, 4096, (256, 256, 1, 32)) for _ in range(3)]
    assert np.array_equal(ys[0], ys[1]) and np.array_equal(ys[0], ys[2])
    with pytest.raises(backend.PsnError) as e:
        hip.matmul_host(t, W, X, 513, 4096, (128, 256, 1, 32))          # the wide kernel has one tile
    assert e.value.code == _ffi.E_UNSUPPORTED


def test_prefill_errors(hip, orc):
    n, k = 64, 512
    W = weights(orc, "Q4_0", 850, n, k)
    w = hip.upload_weight(orc.Q4_0, W, n, k)
    x = hip.upload(np.zeros((4, k), np.float16))
    y = hip.alloc(4 * n * 4)
    with pytest.raises(backend.PsnError) as e:
        hip.quantized_matmul(w, x, y, 4, tile=(96, 96))
    assert e.value.code == _ffi.E_UNSUPPORTED
    with pytest.raises(backend.PsnError) as e:
        hip.quantized_matmul(w, x, y, 8)                      # X and Y too small for 8 rows
    assert e.value.code == _ffi.E_INVALID_ARG
    wk = hip.upload_weight(orc.Q6_K, weights(orc, "Q6_K", 851, n, k), n, k)
    with pytest.raises(backend.PsnError) as e:
        hip.quantized_matmul(wk, x, y, 4, tile=(64, 64, 1, 64))   # Q6_K rows of K = 512 are not whole 16-byte words
    assert e.value.code == _ffi.E_UNSUPPORTED
    hip.quantized_matmul(w, x, y, 4)
    hip.sync()


def test_prefill_default_plans_over_seeded_random_shapes(hip, orc):
    """The planner's own choice of family, tile and K split for shapes nobody tuned for, all five formats."""
    rng = np.random.default_rng(6150)
    for case in range(30):
        qname = ["Q4_0", "Q8_0", "Q4_K", "Q5_K", "Q6_K"][case % 5]
        qt = getattr(orc, qname)
        k = int(rng.choice([256, 512, 1024, 1536, 2048, 4096]))
        n = int(rng.integers(1, 900))
        m = int(rng.choice([1, 3, 17, 64, 65, 100, 128, 257, 300, 520]))
        say(f"random prefill #{case}: {qname} m={m} n={n} k={k} plan={backend.prefill_plan(m, n, k, hip.compute_units, qt)}")
        b = orc.quantize(qt, G.seeded_weights(6200 + case, n, k))
        x = G.seeded_acts(6300 + case, m, k).astype(np.float16)
        ref = orc.prefill(qt, b, x, n, k)
        got = hip.matmul_host(qt, b, x, n, k)
        assert G.max_rel_err(got, ref) < 2e-5, (qname, m, n, k)


@pytest.mark.parametrize("qname", ["Q4_0", "Q8_0", "Q4_K", "Q5_K", "Q6_K"])
def test_dense_family_ragged_shapes(hip, orc, qname):
    """Family 128: the matrix is rewritten as fp16 fragments once (psn_prefill_<fmt>_unpack), then multiplied
    on 256 x 256 or 128 x 256 tiles.  Ragged m and n against the tiles and against the 32-row fragment blocks,
    one to sixteen chunks of K, every K split the shape allows; the fp16 values are those of the other
    families, so the same tolerance holds."""
    t = getattr(orc, qname)
    for m, n, k in ((1, 40, 256), (37, 300, 1280), (260, 700, 2048), (333, 516, 1024), (257, 256, 512), (520, 33, 4096)):
        W = weights(orc, qname, 820, n, k)
        X = G.seeded_acts(821 + m, m, k).astype(np.float16)
        ref = orc.prefill(t, W, X, n, k)
        for ksplit in (1, 2, 4):
            if ksplit > 1 and ((m * n) % 4 or k // 256 < ksplit):
                continue
            for bm in (256, 128):
                say(f"dense prefill {qname} m={m} n={n} k={k} rows per tile={bm} ksplit={ksplit}")
                y = hip.matmul_host(t, W, X, n, k, (bm, 256, ksplit, 128))
                err = G.max_rel_err(y, ref)
                assert np.all(np.isfinite(y)) and err < PARITY_TOL, (qname, bm, ksplit, m, n, k, err)
    with pytest.raises(backend.PsnError) as e:
        hip.matmul_host(t, W, X, n, k, (128, 128, 1, 128))                      # the dense kernels' tiles are 256 columns wide
    assert e.value.name == "PSN_E_UNSUPPORTED"


def test_dense_family_in_graphs_needs_its_workspace_first(hip, orc):
    """Large M takes the dense family by default.  Its fp16 copy of the matrix lives in the stream's
    workspace, which cannot be allocated during a capture: on a stream that has none the default plan falls
    back to the other families (same result), a forced dense launch is refused, and after psn_prefill_reserve
    the capture contains the dense launches and replays to the eager result."""
    t, n, k, m = orc.Q4_K, 3000, 768, 3000
    assert backend.prefill_plan(m, n, k, hip.compute_units, t)[3] == 128
    assert backend.prefill_plan(64, n, k, hip.compute_units, t)[3] != 128
    W = weights(orc, "Q4_K", 830, n, k)
    X = G.seeded_acts(831, m, k).astype(np.float16)
    ref = orc.prefill(t, W, X, n, k)
    w, x = hip.upload_weight(t, W, n, k), hip.upload(X)
    y = hip.alloc(m * n * 4)
    s2 = hip.new_stream()
    try:
        with hip.on_stream(s2):
            hip.begin_capture()
            try:
                hip.quantized_matmul(w, x, y, m)                                  # no workspace on this stream: not dense
                with pytest.raises(backend.PsnError) as e:
                    hip.quantized_matmul(w, x, y, m, (256, 256, 1, 128))
                assert e.value.name == "PSN_E_INVALID_ARG"
            finally:
                g = hip.end_capture()
            hip.launch_graph(g)
            hip.sync()
            assert G.max_rel_err(y.download(np.float32, (m, n)), ref) < PARITY_TOL
            hip.destroy_graph(g)
            hip.reserve_prefill(n, k)
            y.fill_zero()
            hip.begin_capture()
            try:
                hip.quantized_matmul(w, x, y, m)                                  # dense now
                hip.quantized_matmul(w, x, y, m, (256, 256, 2, 128))
            finally:
                g = hip.end_capture()
            for _ in range(3):
                hip.launch_graph(g)
                hip.sync()
                assert G.max_rel_err(y.download(np.float32, (m, n)), ref) < PARITY_TOL
            hip.destroy_graph(g)
    finally:
        hip.destroy_stream(s2)


@pytest.mark.parametrize("qname", ["Q4_0", "Q8_0", "Q4_K", "Q5_K", "Q6_K"])
def test_packed_weights_multiply_like_the_dense_family(hip, orc, qname):
    """psn_prefill_pack once, psn_qmatmul_prefill_packed for several X of different heights: the oracle's
    result each time, and the dense family's (same fragments, same multiply) up to the order of the K ranges' sums."""
    t = getattr(orc, qname)
    n, k = 700, 2048
    W = weights(orc, qname, 840, n, k)
    w = hip.upload_weight(t, W, n, k)
    packed = hip.pack_for_prefill(w)
    assert packed.nbytes >= 768 * k * 2
    for m in (1, 260, 37, 384, 1100):                                                    # heights served by either tile of the multiply
        X = G.seeded_acts(841 + m, m, k).astype(np.float16)
        y = hip.alloc(m * n * 4)
        hip.quantized_matmul_packed(packed, hip.upload(X), y, m, n, k)
        got = y.download(np.float32, (m, n))
        assert G.max_rel_err(got, orc.prefill(t, W, X, n, k)) < PARITY_TOL, (qname, m)
        same = hip.matmul_host(t, W, X, n, k, (256, 256, 1, 128))
        assert G.max_rel_err(got, same) < 2e-6                                          # the library may cut K (atomic adds): not bit for bit
    with pytest.raises(backend.PsnError) as e:
        hip.quantized_matmul_packed(hip.alloc(1024), hip.upload(X), y, m, n, k)          # not a packed buffer of this shape
    assert e.value.name == "PSN_E_INVALID_ARG"
    with pytest.raises(backend.PsnError) as e:
        hip.quantized_matmul_packed(packed, hip.upload(X), y, m, n, 2000)
    assert e.value.name == "PSN_E_SHAPE"


@pytest.mark.parametrize("qname", ["Q4_0", "Q8_0", "Q4_K", "Q5_K", "Q6_K"])
def test_packed_fragments_hold_the_reference_fp16_values_bit_for_bit(hip, orc, qname):
    """psn_prefill_pack writes h(deq(W)): every weight as the fp16 rounding of the value the reference's
    dequantizer returns, in fragment order [row / 32][k / 16][half][row % 32][8].  Read back and compared
    bit for bit (up to the sign of a zero) with numpy.float16 of the oracle's dequantization -- rows scaled over twelve binades so that
    block scales, mins and fp16 roundings of every size occur, and a ragged last row panel."""
    t = getattr(orc, qname)
    n, k = 200, 2048
    rng = np.random.default_rng(8100)
    w = rng.standard_normal((n, k), dtype=np.float32) * np.exp2(rng.integers(-8, 4, (n, k // 32))).astype(np.float32).repeat(32, axis=1)
    blocks = orc.quantize(t, w)
    wt = hip.upload_weight(t, blocks, n, k)
    packed = hip.pack_for_prefill(wt)
    npanel = -(-n // 32)
    raw = packed.download(np.uint16, (packed.nbytes // 2,))[:npanel * (k // 16) * 64 * 8].reshape(npanel, k // 16, 2, 32, 8)
    # [panel][kslice][half][row % 32][j] -> [row][k]
    got = raw.transpose(0, 3, 1, 2, 4).reshape(npanel * 32, k)[:n]
    want = orc.dequantize(t, blocks, k).reshape(n, k).astype(np.float16).view(np.uint16)
    # a zero keeps no sign: the reference's d * sc * (q - 32) is -0 where d * sc is negative and q = 32, the
    # kernels' fused form d sc q - 32 d sc returns +0 (Q6_K; the other formats agree in the sign of zero too)
    zero = (want & 0x7fff) == 0
    got, want = np.where(zero, got & 0x7fff, got), np.where(zero, want & 0x7fff, want)
    differ = np.argwhere(got != want)
    assert differ.size == 0, [(int(r), int(c), hex(int(got[r, c])), hex(int(want[r, c]))) for r, c in differ[:6]]


def test_prefill_refuses_operands_beyond_32_bit_offsets(hip, orc):
    """Several families address X and W with 32-bit byte offsets: shapes that would overflow them are
    refused by the host before any buffer is looked at."""
    w = hip.upload_weight(orc.Q4_0, weights(orc, "Q4_0", 850, 64, 4096), 64, 4096)
    x, y = hip.alloc(1 << 20), hip.alloc(1 << 20)
    with pytest.raises(backend.PsnError) as e:
        hip.quantized_matmul(w, x, y, 1 << 20)                       # X would be 8 GiB
    assert e.value.name == "PSN_E_SHAPE" and "4 GiB" in str(e.value)
    with pytest.raises(backend.PsnError) as e:
        hip.quantized_matmul_packed(x, x, y, 1 << 20, 64, 4096)
    assert e.value.name == "PSN_E_SHAPE"
