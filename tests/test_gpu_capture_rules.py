"""What may and may not happen on a stream that is being captured into a graph, and what a captured graph
pins: uploads, downloads and memsets are refused (never recorded), and the activation workspace a graph
refers to cannot move afterwards."""
import numpy as np
import pytest

import ggufref as G
from openagents_amd import _ffi, backend

pytestmark = pytest.mark.gpu


def test_fill_zero_clears_a_buffer(hip):
    b = hip.upload(np.arange(1000, dtype=np.float32))
    b.fill_zero()
    assert not b.download(np.float32, (1000,)).any()


def test_uploads_downloads_and_memsets_are_refused_while_capturing(hip):
    n = 1024
    g, u, out = hip.upload(np.full(n, 2.0, np.float32)), hip.upload(np.full(n, 3.0, np.float32)), hip.alloc(n * 4)
    host = np.zeros(n, np.float32)
    hip.begin_capture()
    try:
        for call in (lambda: out.upload(host), lambda: out.download(np.float32, (n,)), lambda: out.fill_zero()):
            with pytest.raises(backend.PsnError) as e:
                call()
            assert e.value.code == _ffi.E_INVALID_ARG and "captured" in str(e.value)
        hip.swiglu(g, u, out, n)                       # the capture itself is still intact
    finally:
        graph = hip.end_capture()
    try:
        for _ in range(2):
            out.fill_zero()
            hip.launch_graph(graph)
            got = out.download(np.float32, (n,))
            assert np.allclose(got, 2.0 / (1.0 + np.exp(-2.0)) * 3.0, rtol=1e-6)
    finally:
        hip.destroy_graph(graph)


def test_workspace_cannot_grow_once_a_graph_refers_to_it(orc):
    """Q6_K at batch 4 quantizes in a separate launch into the stream's workspace.  After such a call has
    been captured, a larger eager call on the same stream must fail instead of freeing memory the graph
    still points at; the graph keeps replaying correctly; once the graph is destroyed the workspace may grow."""
    with backend.HipBackend(0) as be:
        n, k_small, k_big, batch = 8, 1024, 327680, 4        # the workspace grows in 1 MiB steps: 4 x 327680 int8 exceed one
        Ws, Wb = orc.quantize(orc.Q6_K, G.seeded_weights(970, n, k_small)), orc.quantize(orc.Q6_K, G.seeded_weights(971, n, k_big))
        xs, xb = G.seeded_acts(972, batch, k_small), G.seeded_acts(973, batch, k_big)
        ws, wb = be.upload_weight(orc.Q6_K, Ws, n, k_small), be.upload_weight(orc.Q6_K, Wb, n, k_big)
        dxs, dxb, y = be.upload(xs), be.upload(xb), be.alloc(batch * n * 4)
        be.reserve(k_small, batch)
        be.begin_capture()
        be.quantized_matvec(ws, dxs, y, batch, _ffi.ACT_Q8)
        graph = be.end_capture()
        ref = orc.matvec(orc.Q6_K, orc.ACT_Q8, Ws, xs, n, k_small)
        be.launch_graph(graph)
        assert G.max_rel_err(y.download(np.float32, (batch, n)), ref) < 2e-5
        with pytest.raises(backend.PsnError) as e:
            be.quantized_matvec(wb, dxb, y, batch, _ffi.ACT_Q8)
        assert e.value.code == _ffi.E_INVALID_ARG and "reserve" in str(e.value)
        y.fill_zero()
        be.launch_graph(graph)
        assert G.max_rel_err(y.download(np.float32, (batch, n)), ref) < 2e-5
        be.destroy_graph(graph)
        # no graph refers to the workspace any more: it may grow again
        be.quantized_matvec(wb, dxb, y, batch, _ffi.ACT_Q8)
        assert G.max_rel_err(y.download(np.float32, (batch, n)), orc.matvec(orc.Q6_K, orc.ACT_Q8, Wb, xb, n, k_big)) < 2e-5


def test_side_stream_workspace_is_pinned_by_the_graph_that_the_origin_ends(orc):
    """A batch-4 Q6_K matvec on a side stream forked into a capture quantizes into the SIDE stream's
    workspace.  The graph ended on the origin stream must pin that workspace (growth on the side stream is
    refused while the graph lives), a later capture begun on the side stream must not lift the pin, and
    destroying the graph lifts it."""
    with backend.HipBackend(0) as be:
        n, k_small, k_big, batch = 8, 1024, 327680, 4
        Ws, Wb = orc.quantize(orc.Q6_K, G.seeded_weights(975, n, k_small)), orc.quantize(orc.Q6_K, G.seeded_weights(976, n, k_big))
        xs, xb = G.seeded_acts(977, batch, k_small), G.seeded_acts(978, batch, k_big)
        ws, wb = be.upload_weight(orc.Q6_K, Ws, n, k_small), be.upload_weight(orc.Q6_K, Wb, n, k_big)
        dxs, dxb, y, y_side = be.upload(xs), be.upload(xb), be.alloc(batch * n * 4), be.alloc(batch * n * 4)
        side = be.new_stream()
        with be.on_stream(side):
            be.reserve(k_small, batch)
        be.reserve(k_small, batch)
        main = be.stream
        be.begin_capture()
        be.stream_wait(side, main)                           # fork
        with be.on_stream(side):
            be.quantized_matvec(ws, dxs, y_side, batch, _ffi.ACT_Q8)
        be.quantized_matvec(ws, dxs, y, batch, _ffi.ACT_Q8)
        be.stream_wait(main, side)                           # join
        graph = be.end_capture()
        ref = orc.matvec(orc.Q6_K, orc.ACT_Q8, Ws, xs, n, k_small)

        def replay_ok():
            y.fill_zero()
            y_side.fill_zero()
            be.launch_graph(graph)
            return (G.max_rel_err(y.download(np.float32, (batch, n)), ref) < 2e-5 and
                    G.max_rel_err(y_side.download(np.float32, (batch, n)), ref) < 2e-5)

        assert replay_ok()
        with be.on_stream(side):
            with pytest.raises(backend.PsnError) as e:
                be.quantized_matvec(wb, dxb, y_side, batch, _ffi.ACT_Q8)
            assert e.value.code == _ffi.E_INVALID_ARG and "reserve" in str(e.value)
            # an unrelated capture on the side stream comes and goes: the first graph still holds the workspace
            be.begin_capture()
            be.swiglu(dxs, dxs, y_side, 32)
            be.destroy_graph(be.end_capture())
            with pytest.raises(backend.PsnError) as e:
                be.quantized_matvec(wb, dxb, y_side, batch, _ffi.ACT_Q8)
            assert e.value.code == _ffi.E_INVALID_ARG
        assert replay_ok()
        be.destroy_graph(graph)
        with be.on_stream(side):
            be.quantized_matvec(wb, dxb, y_side, batch, _ffi.ACT_Q8)      # nothing refers to it any more: it may grow
            be.sync()
            assert G.max_rel_err(y_side.download(np.float32, (batch, n)), orc.matvec(orc.Q6_K, orc.ACT_Q8, Wb, xb, n, k_big)) < 2e-5
        be.destroy_stream(side)


def test_a_graph_outlives_the_stream_whose_workspace_it_holds(orc):
    """Destroying a stream does not free a workspace that a live graph still points at: the graph keeps
    replaying on another stream, and the memory goes with the graph."""
    with backend.HipBackend(0) as be:
        n, k, batch = 16, 2048, 4
        W = orc.quantize(orc.Q6_K, G.seeded_weights(979, n, k))
        x = G.seeded_acts(980, batch, k)
        w, dx, y = be.upload_weight(orc.Q6_K, W, n, k), be.upload(x), be.alloc(batch * n * 4)
        side = be.new_stream()
        with be.on_stream(side):
            be.reserve(k, batch)
            be.begin_capture()
            be.quantized_matvec(w, dx, y, batch, _ffi.ACT_Q8)
            graph = be.end_capture()
        be.destroy_stream(side)
        ref = orc.matvec(orc.Q6_K, orc.ACT_Q8, W, x, n, k)
        for _ in range(2):
            y.fill_zero()
            be.launch_graph(graph)
            assert G.max_rel_err(y.download(np.float32, (batch, n)), ref) < 2e-5
        be.destroy_graph(graph)
