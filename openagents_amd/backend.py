"""Host-side mirror of the backend/operator surface for the quantized GGUF path.

`HipBackend` is what a Psionic backend crate would look like for `--backend hip`
(the switch is pinned by
/root/reference/apps/pylon/docs/2026-06-09-pylon-qwen35-local-inference-roadmap.md:137-150;
the crate names psionic-backend-cuda / -metal by
/root/reference/docs/2026-06-10-cs336-distributed-homework-continuation-audit.md:239-241):
buffers, weight upload, activation quantize, quantized matvec (decode) and quantized matmul
(prefill), all asynchronous on a stream, errors as typed exceptions.  Every method is a thin
call into the C ABI (include/psn.h); numpy appears only as the host-memory container.
There is no CPU path: without the library or a gfx950 device construction raises.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import _ffi
from ._ffi import (ACT_F32, ACT_Q8, LAYOUT_GGUF, Q4_0, Q4_K, Q5_K, Q6_K, Q8_0, Q8_K, MatvecPlan)  # noqa: F401

TYPE_NAMES = {Q4_0: "Q4_0", Q8_0: "Q8_0", Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", Q8_K: "Q8_K"}


class PsnError(RuntimeError):
    """A negative return code from the C ABI, with psn_last_error()'s text."""

    def __init__(self, code: int, text: str):
        lib = _ffi.load()
        self.code = code
        self.name = lib.psn_error_name(code).decode()
        super().__init__(f"{self.name} ({code}): {text}")


def _check(rc: int) -> int:
    if rc < 0:
        raise PsnError(int(rc), _ffi.load().psn_last_error().decode(errors="replace"))
    return int(rc)


def row_bytes(qtype: int, k: int) -> int:
    return _check(_ffi.load().psn_row_bytes(qtype, k))


def act_type_for(qtype: int) -> int:
    return _check(_ffi.load().psn_act_type_for(qtype))


def actq_layout(act_type: int, k: int, batch: int) -> _ffi.ActqInfo:
    info = _ffi.ActqInfo()
    _check(_ffi.load().psn_actq_layout(act_type, k, batch, C.byref(info)))
    return info


def prefill_plan(m: int, n: int, k: int, compute_units: int = 256, qtype: int | None = None):
    """(tile_m, tile_n, ksplit, waves) the library picks for a prefill shape (qtype None: the Q4_0 / Q8_0 plan)."""
    tm, tn, sp, wv = C.c_int32(), C.c_int32(), C.c_int32(), C.c_int32()
    if qtype is None:
        _check(_ffi.load().psn_qmatmul_prefill_plan(m, n, k, compute_units, C.byref(tm), C.byref(tn), C.byref(sp), C.byref(wv)))
    else:
        _check(_ffi.load().psn_qmatmul_prefill_plan_for(qtype, m, n, k, compute_units, C.byref(tm), C.byref(tn), C.byref(sp), C.byref(wv)))
    return int(tm.value), int(tn.value), int(sp.value), int(wv.value)


def matvec_plan(qtype: int, scheme: int, n: int, k: int, batch: int, compute_units: int = 256, x_is_f32: bool = False) -> MatvecPlan:
    plan = MatvecPlan()
    _check(_ffi.load().psn_qmatvec_plan(qtype, scheme, n, k, batch, compute_units, int(x_is_f32), C.byref(plan)))
    return plan


class DeviceBuffer:
    """Owns one psn_buf."""

    def __init__(self, backend: "HipBackend", nbytes: int):
        self._b = backend
        h = C.c_void_p()
        _check(backend.lib.psn_buf_alloc(backend.ctx, nbytes, C.byref(h)))
        self.handle = h
        self.nbytes = nbytes

    @classmethod
    def _adopt(cls, backend: "HipBackend", handle: C.c_void_p) -> "DeviceBuffer":
        self = cls.__new__(cls)
        self._b = backend
        self.handle = handle
        self.nbytes = int(backend.lib.psn_buf_size(handle))
        return self

    def upload(self, arr: np.ndarray, offset: int = 0) -> "DeviceBuffer":
        a = np.ascontiguousarray(arr)
        _check(self._b.lib.psn_buf_upload(self.handle, offset, C.c_void_p(a.ctypes.data), a.nbytes, self._b.stream))
        return self

    def download(self, dtype, shape, offset: int = 0) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        _check(self._b.lib.psn_buf_download(self.handle, offset, C.c_void_p(out.ctypes.data), out.nbytes, self._b.stream))
        return out

    def fill_zero(self) -> "DeviceBuffer":
        _check(self._b.lib.psn_buf_fill_zero(self.handle, self._b.stream))
        return self

    def free(self):
        if self.handle is not None and self._b.ctx is not None:
            if self._b._capturing:
                # freeing device memory while a stream of this thread is being captured would invalidate
                # the capture (a buffer can die at any moment when the garbage collector runs)
                self._b._deferred_free.append(self.handle)
            else:
                _check(self._b.lib.psn_buf_free(self.handle))
        self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


@dataclass
class QuantizedTensor:
    """An [n, k] GGUF-quantized weight resident on the device."""
    buf: DeviceBuffer
    qtype: int
    n: int
    k: int

    @property
    def nbytes(self) -> int:
        return self.n * row_bytes(self.qtype, self.k)


class HipBackend:
    def __init__(self, device: int = 0):
        self.lib = _ffi.load()
        self.ctx = None
        self._capturing = False
        self._deferred_free = []
        ctx = C.c_void_p()
        _check(self.lib.psn_ctx_create(device, C.byref(ctx)))
        self.ctx = ctx
        mod = C.c_void_p()
        _check(self.lib.psn_module_load_builtin(ctx, C.byref(mod)))
        self.module = mod
        st = C.c_void_p()
        _check(self.lib.psn_stream_create(ctx, C.byref(st)))
        self.stream = st
        cus, mem = C.c_int32(), C.c_int64()
        name = C.create_string_buffer(64)
        _check(self.lib.psn_ctx_info(ctx, C.byref(cus), C.byref(mem), name, 64))
        self.compute_units = int(cus.value)
        self.total_mem = int(mem.value)
        self.arch = name.value.decode()

    # -- lifetime ---------------------------------------------------------------------------
    def close(self):
        if self.ctx is None:
            return
        self.lib.psn_stream_destroy(self.stream)
        self.lib.psn_module_unload(self.module)
        self.lib.psn_ctx_destroy(self.ctx)
        self.ctx = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # -- buffers ----------------------------------------------------------------------------
    def alloc(self, nbytes: int) -> DeviceBuffer:
        return DeviceBuffer(self, nbytes)

    def upload(self, arr: np.ndarray) -> DeviceBuffer:
        a = np.ascontiguousarray(arr)
        return DeviceBuffer(self, max(a.nbytes, 1)).upload(a)

    def upload_weight(self, qtype: int, blocks: np.ndarray, n: int, k: int) -> QuantizedTensor:
        b = np.ascontiguousarray(blocks, dtype=np.uint8)
        if b.size != n * row_bytes(qtype, k):
            raise ValueError(f"weight bytes {b.size} != n*row_bytes {n * row_bytes(qtype, k)}")
        h = C.c_void_p()
        _check(self.lib.psn_weight_upload(self.ctx, qtype, n, k, C.c_void_p(b.ctypes.data), LAYOUT_GGUF, self.stream, C.byref(h)))
        return QuantizedTensor(DeviceBuffer._adopt(self, h), qtype, n, k)

    def copy(self, dst: DeviceBuffer, src: DeviceBuffer, nbytes: int, dst_off: int = 0, src_off: int = 0):
        _check(self.lib.psn_buf_copy(dst.handle, dst_off, src.handle, src_off, nbytes, self.stream))

    def sync(self):
        _check(self.lib.psn_stream_sync(self.stream))

    # -- additional streams -------------------------------------------------------------------
    def new_stream(self) -> C.c_void_p:
        st = C.c_void_p()
        _check(self.lib.psn_stream_create(self.ctx, C.byref(st)))
        return st

    def destroy_stream(self, stream):
        _check(self.lib.psn_stream_destroy(stream))

    def stream_wait(self, waiter, signaler):
        """`waiter` waits for what is enqueued on `signaler` so far; under capture this forks / joins graph branches."""
        _check(self.lib.psn_stream_wait_stream(waiter, signaler))

    def on_stream(self, stream):
        """Context manager: route this backend's launches to `stream`."""
        be = self

        class _Swap:
            def __enter__(self_inner):
                self_inner.prev = be.stream
                be.stream = stream

            def __exit__(self_inner, *exc):
                be.stream = self_inner.prev

        return _Swap()

    # -- events -----------------------------------------------------------------------------
    def event(self) -> C.c_void_p:
        e = C.c_void_p()
        _check(self.lib.psn_event_create(self.ctx, C.byref(e)))
        return e

    def record(self, event):
        _check(self.lib.psn_event_record(event, self.stream))

    def elapsed_us(self, begin, end) -> float:
        out = C.c_double()
        _check(self.lib.psn_event_elapsed_us(begin, end, C.byref(out)))
        return float(out.value)

    def destroy_event(self, event):
        _check(self.lib.psn_event_destroy(event))

    # -- operators --------------------------------------------------------------------------
    def quantize_activations(self, x: DeviceBuffer, k: int, batch: int, act_type: int, out: DeviceBuffer | None = None) -> DeviceBuffer:
        info = actq_layout(act_type, k, batch)
        out = out or self.alloc(int(info.bytes))
        _check(self.lib.psn_act_quantize(self.module, self.stream, act_type, x.handle, out.handle, k, batch))
        return out

    def quantized_matvec(self, w: QuantizedTensor, x: DeviceBuffer, y: DeviceBuffer, batch: int = 1, scheme: int = ACT_Q8):
        _check(self.lib.psn_qmatvec(self.module, self.stream, w.qtype, LAYOUT_GGUF, scheme, w.buf.handle, x.handle, y.handle, w.n, w.k, batch))

    def quantized_matvec_noalloc(self, w: QuantizedTensor, x: DeviceBuffer, y: DeviceBuffer, batch: int = 1, scheme: int = ACT_Q8):
        """quantized_matvec that allocates nothing (static device scratch; calls on one GPU must not overlap)."""
        _check(self.lib.psn_qmatvec_noalloc(self.module, self.stream, w.qtype, LAYOUT_GGUF, scheme, w.buf.handle, x.handle, y.handle, w.n, w.k, batch))

    def quantized_matvec_q8(self, w: QuantizedTensor, xq: DeviceBuffer, y: DeviceBuffer, batch: int = 1):
        _check(self.lib.psn_qmatvec_q8(self.module, self.stream, w.qtype, LAYOUT_GGUF, w.buf.handle, xq.handle, y.handle, w.n, w.k, batch))

    @staticmethod
    def _pack(ws, ys):
        """ctypes arrays for a list of weights / outputs that share one launch."""
        ws = list(ws) if isinstance(ws, (list, tuple)) else [ws]
        ys = list(ys) if isinstance(ys, (list, tuple)) else [ys]
        if len(ws) != len(ys) or not ws:
            raise ValueError("need as many outputs as weights")
        if any((w.qtype, w.k) != (ws[0].qtype, ws[0].k) for w in ws):
            raise ValueError("matrices sharing a launch must share format and K")
        n = len(ws)
        W = (C.c_void_p * n)(*[w.buf.handle for w in ws])
        Y = (C.c_void_p * n)(*[y.handle for y in ys])
        N = (C.c_int64 * n)(*[w.n for w in ws])
        return ws[0], n, W, Y, N

    def quantized_matvec_multi(self, ws, x: DeviceBuffer, ys, batch: int = 1, scheme: int = ACT_Q8):
        """Several matrices sharing x (q/k/v, gate/up) in one launch; x is fp32."""
        w0, n, W, Y, N = self._pack(ws, ys)
        _check(self.lib.psn_qmatvec_multi(self.module, self.stream, w0.qtype, LAYOUT_GGUF, scheme, n, W, x.handle, Y, N, w0.k, batch))

    def quantized_matvec_q8_multi(self, ws, xq: DeviceBuffer, ys, batch: int = 1):
        w0, n, W, Y, N = self._pack(ws, ys)
        _check(self.lib.psn_qmatvec_q8_multi(self.module, self.stream, w0.qtype, LAYOUT_GGUF, n, W, xq.handle, Y, N, w0.k, batch))

    def quantized_matvec_norm_multi(self, ws, x: DeviceBuffer, delta, norm_weight: DeviceBuffer, h_out, ys, eps: float = 1e-5):
        """ys[i] = ws[i] . q8(rmsnorm(x + delta) * norm_weight); h_out (optional, not x or delta) receives x + delta."""
        w0, n, W, Y, N = self._pack(ws, ys)
        _check(self.lib.psn_qmatvec_norm_multi(self.module, self.stream, w0.qtype, LAYOUT_GGUF, n, W, x.handle, self._h(delta), norm_weight.handle,
                                               self._h(h_out), Y, N, w0.k, eps))

    def quantized_matvec_norm_swiglu(self, w_gate: QuantizedTensor, w_up: QuantizedTensor, x: DeviceBuffer, delta, norm_weight: DeviceBuffer,
                                     h_out, act: DeviceBuffer, eps: float = 1e-5):
        """act = silu(w_gate . n) * (w_up . n) with n = q8(rmsnorm(x + delta) * norm_weight), one launch (psn_qmatvec_norm_swiglu)."""
        if (w_gate.qtype, w_gate.n, w_gate.k) != (w_up.qtype, w_up.n, w_up.k):
            raise ValueError("gate and up projections must share format and shape")
        _check(self.lib.psn_qmatvec_norm_swiglu(self.module, self.stream, w_gate.qtype, LAYOUT_GGUF, w_gate.buf.handle, w_up.buf.handle, x.handle,
                                                self._h(delta), norm_weight.handle, self._h(h_out), act.handle, w_gate.n, w_gate.k, eps))

    def norm_swiglu_supported(self, qtype: int, n: int, k: int) -> bool:
        """Whether psn_qmatvec_norm_swiglu serves this shape on this device (host arithmetic)."""
        return int(self.lib.psn_qmatvec_norm_swiglu_check(qtype, n, k, self.compute_units)) == 0

    def quantized_matvec_planned(self, ws, x: DeviceBuffer, ys, batch: int, scheme: int, plan: MatvecPlan):
        w0, n, W, Y, N = self._pack(ws, ys)
        _check(self.lib.psn_qmatvec_planned(self.module, self.stream, w0.qtype, scheme, n, W, x.handle, Y, N, w0.k, batch, C.byref(plan)))

    def calibrate_read(self, src: DeviceBuffer, nbytes: int, blocks: int, threads: int = 256, lds_depth: int = 0, out: DeviceBuffer | None = None,
                       every_workgroup: bool = False):
        """A launch that only reads nbytes of src (see psn_calibrate_read)."""
        _check(self.lib.psn_calibrate_read(self.module, self.stream, src.handle, nbytes, blocks, threads, lds_depth, int(every_workgroup), self._h(out)))

    # -- decode-step glue --------------------------------------------------------------------
    def selftest_arith(self) -> list:
        """Mismatch counts of the quantizers' division shortcuts against IEEE division over every float they are used
        on (see psn_selftest_arith): eight zeros on a device whose arithmetic the library was written for."""
        out = self.alloc(64)
        _check(self.lib.psn_selftest_arith(self.module, self.stream, out.handle))
        counts = [int(v) for v in out.download(np.uint64, (8,))]
        out.free()
        return counts

    def add_rmsnorm(self, x: DeviceBuffer, delta, weight: DeviceBuffer, y: DeviceBuffer, n: int, eps: float = 1e-5):
        _check(self.lib.psn_add_rmsnorm(self.module, self.stream, x.handle, delta.handle if delta is not None else None,
                                        weight.handle, y.handle, n, eps))

    def rope_kv_store(self, q, k, v, k_cache, v_cache, n_heads: int, n_kv_heads: int, head_dim: int, pos: int, theta_base: float):
        _check(self.lib.psn_rope_kv_store(self.module, self.stream, q.handle, k.handle, v.handle, k_cache.handle, v_cache.handle,
                                          n_heads, n_kv_heads, head_dim, pos, theta_base))

    def attention_decode(self, q, k_cache, v_cache, workspace, out, n_heads: int, n_kv_heads: int, head_dim: int, n_ctx: int):
        _check(self.lib.psn_attention_decode(self.module, self.stream, q.handle, k_cache.handle, v_cache.handle, workspace.handle,
                                             out.handle, n_heads, n_kv_heads, head_dim, n_ctx))

    def swiglu(self, gate, up, out, n: int):
        _check(self.lib.psn_swiglu(self.module, self.stream, gate.handle, up.handle, out.handle, n))

    # the same producers with the activation quantization fused in (fp32 output optional)
    @staticmethod
    def _h(buf):
        return buf.handle if buf is not None else None

    def add_rmsnorm_q8(self, x, delta, weight, y, y_q, act_type: int, n: int, eps: float = 1e-5):
        _check(self.lib.psn_add_rmsnorm_q8(self.module, self.stream, x.handle, self._h(delta), weight.handle, self._h(y), y_q.handle, act_type, n, eps))

    def swiglu_q8(self, gate, up, out, out_q, act_type: int, n: int):
        _check(self.lib.psn_swiglu_q8(self.module, self.stream, gate.handle, up.handle, self._h(out), out_q.handle, act_type, n))

    def attention_decode_q8(self, q, k_cache, v_cache, workspace, out, out_q, act_type: int, n_heads: int, n_kv_heads: int, head_dim: int, n_ctx: int):
        _check(self.lib.psn_attention_decode_q8(self.module, self.stream, q.handle, k_cache.handle, v_cache.handle, workspace.handle,
                                                self._h(out), out_q.handle, act_type, n_heads, n_kv_heads, head_dim, n_ctx))

    def rope_table(self, table, head_dim: int, pos: int, theta_base: float):
        _check(self.lib.psn_rope_table(self.module, self.stream, table.handle, head_dim, pos, theta_base))

    def attention_decode_rope(self, q, k, v, k_cache, v_cache, workspace, out, out_q, act_type: int, n_heads: int, n_kv_heads: int,
                              head_dim: int, pos: int, rope_table):
        """Rotary embedding + KV append + attention over positions 0..pos (q, k, v are the raw projections)."""
        _check(self.lib.psn_attention_decode_rope(self.module, self.stream, q.handle, k.handle, v.handle, k_cache.handle, v_cache.handle,
                                                  workspace.handle, self._h(out), self._h(out_q), act_type, n_heads, n_kv_heads, head_dim, pos,
                                                  rope_table.handle))

    # -- graphs -----------------------------------------------------------------------------
    def reserve(self, k: int, batch: int = 1):
        _check(self.lib.psn_stream_reserve(self.stream, k, batch))

    def pack_for_prefill(self, w: QuantizedTensor) -> DeviceBuffer:
        """h(deq(w)) as fp16 MFMA fragments in a buffer of its own (2 bytes per weight): dequantized once, multiplied many times."""
        nbytes = int(self.lib.psn_prefill_packed_bytes(w.n, w.k))
        if nbytes < 0:
            _check(nbytes)
        packed = self.alloc(nbytes)
        _check(self.lib.psn_prefill_pack(self.module, self.stream, w.qtype, w.buf.handle, packed.handle, w.n, w.k))
        return packed

    def quantized_matmul_packed(self, packed: DeviceBuffer, x_f16: DeviceBuffer, y: DeviceBuffer, m: int, n: int, k: int):
        _check(self.lib.psn_qmatmul_prefill_packed(self.module, self.stream, packed.handle, x_f16.handle, y.handle, m, n, k))

    def reserve_prefill(self, n: int, k: int):
        """Size the stream's workspace for the dense prefill family on an [n, k] matrix (before a capture)."""
        _check(self.lib.psn_prefill_reserve(self.stream, n, k))

    def begin_capture(self):
        _check(self.lib.psn_graph_begin_capture(self.stream))
        self._capturing = True

    def end_capture(self) -> C.c_void_p:
        g = C.c_void_p()
        try:
            _check(self.lib.psn_graph_end_capture(self.stream, C.byref(g)))
        finally:
            self._capturing = False
            pending, self._deferred_free = self._deferred_free, []
            for h in pending:
                self.lib.psn_buf_free(h)
        return g

    def launch_graph(self, graph):
        _check(self.lib.psn_graph_launch(graph, self.stream))

    def destroy_graph(self, graph):
        _check(self.lib.psn_graph_destroy(graph))

    def quantized_matmul(self, w: QuantizedTensor, x_f16: DeviceBuffer, y: DeviceBuffer, m: int, tile=None):
        """Prefill: Y[m, n] = X[m, k] . deq(W)[n, k]^T, X fp16, Y fp32.  `tile` = (rows, cols[, ksplit[, waves]]) overrides the library's choice."""
        if tile is None:
            _check(self.lib.psn_qmatmul_prefill(self.module, self.stream, w.qtype, LAYOUT_GGUF, w.buf.handle, x_f16.handle, y.handle, m, w.n, w.k))
        else:
            _check(self.lib.psn_qmatmul_prefill_tiled(self.module, self.stream, w.qtype, w.buf.handle, x_f16.handle, y.handle, m, w.n, w.k,
                                                      tile[0], tile[1], tile[2] if len(tile) > 2 else 1, tile[3] if len(tile) > 3 else 4))

    def matmul_host(self, qtype: int, blocks: np.ndarray, x_f16: np.ndarray, n: int, k: int, tile=None) -> np.ndarray:
        x = np.ascontiguousarray(x_f16, dtype=np.float16)
        m = x.shape[0]
        w = self.upload_weight(qtype, blocks, n, k)
        xb = self.upload(x)
        yb = self.alloc(m * n * 4)
        self.quantized_matmul(w, xb, yb, m, tile)
        return yb.download(np.float32, (m, n))

    # -- convenience for tests and examples: host arrays in, host arrays out ------------------
    def matvec_host(self, qtype: int, blocks: np.ndarray, x: np.ndarray, n: int, k: int, scheme: int = ACT_Q8,
                    plan: MatvecPlan | None = None) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        x2 = x.reshape(1, -1) if x.ndim == 1 else x
        batch = x2.shape[0]
        w = self.upload_weight(qtype, blocks, n, k)
        xb = self.upload(x2)
        yb = self.alloc(batch * n * 4)
        if plan is None:
            self.quantized_matvec(w, xb, yb, batch, scheme)
        elif scheme == ACT_Q8 and plan.stage_lds != 2:
            xq = self.quantize_activations(xb, k, batch, act_type_for(qtype))
            self.quantized_matvec_planned(w, xq, yb, batch, scheme, plan)
        else:
            self.quantized_matvec_planned(w, xb, yb, batch, scheme, plan)
        y = yb.download(np.float32, (batch, n))
        return y[0] if x.ndim == 1 else y
