/*
 * psn_host.cpp -- host side of the C ABI in include/psn.h: HIP module load, buffer alloc,
 * launch and stream sync.  Kernels live in a gfx950 code object (built from psn_matvec.hip and
 * psn_prefill.hip) that is linked into this library as a byte blob and loaded with
 * hipModuleLoadData; every launch goes through hipModuleLaunchKernel with one argument struct
 * (psn_args.h).  No CPU compute path exists here.
 */
#include "../../include/psn.h"
#include "psn_args.h"
#include "psn_noalloc.h"

#include <hip/hip_runtime_api.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <exception>
#include <new>
#include <string>
#include <string_view>
#include <unordered_map>
#include <vector>

/* code objects linked into the library (generated table, see build.py) */
struct psn_blob { const unsigned char *begin, *end; };
extern "C" {
extern const psn_blob psn_builtin_blobs[];
extern const int psn_builtin_blob_count;
}

/* ------------------------------------------------------------------ errors */

static thread_local char g_err[512] = "";

static int32_t fail(int32_t code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

static int32_t hip_fail(hipError_t e, const char *what) {
    int32_t code = PSN_E_HIP;
    if (e == hipErrorOutOfMemory) code = PSN_E_OOM;
    if (e == hipErrorNoDevice || e == hipErrorInvalidDevice || e == hipErrorInsufficientDriver) code = PSN_E_NO_DEVICE;
    return fail(code, "%s: hipError %d (%s)", what, (int)e, hipGetErrorString(e));
}

#define HIP_TRY(expr)                                  \
    do {                                               \
        hipError_t e_ = (expr);                        \
        if (e_ != hipSuccess) return hip_fail(e_, #expr); \
    } while (0)

extern "C" int32_t psn_abi_version(void) { return PSN_ABI_VERSION; }
extern "C" const char *psn_last_error(void) { return g_err; }
extern "C" const char *psn_error_name(int32_t code) {
    switch (code) {
        case PSN_OK: return "PSN_OK";
        case PSN_E_INVALID_ARG: return "PSN_E_INVALID_ARG";
        case PSN_E_SHAPE: return "PSN_E_SHAPE";
        case PSN_E_UNSUPPORTED: return "PSN_E_UNSUPPORTED";
        case PSN_E_NO_DEVICE: return "PSN_E_NO_DEVICE";
        case PSN_E_OOM: return "PSN_E_OOM";
        case PSN_E_MODULE: return "PSN_E_MODULE";
        case PSN_E_HIP: return "PSN_E_HIP";
        default: return "PSN_E_UNKNOWN";
    }
}

/* ------------------------------------------------------------------ formats */

extern "C" int32_t psn_block_elems(int32_t t) {
    switch (t) {
        case PSN_Q4_0: case PSN_Q8_0: return 32;
        case PSN_Q4_K: case PSN_Q5_K: case PSN_Q6_K: case PSN_Q8_K: return 256;
        default: return 0;
    }
}
extern "C" int32_t psn_block_bytes(int32_t t) {
    switch (t) {
        case PSN_Q4_0: return 18;
        case PSN_Q8_0: return 34;
        case PSN_Q4_K: return 144;
        case PSN_Q5_K: return 176;
        case PSN_Q6_K: return 210;
        case PSN_Q8_K: return 292;
        default: return 0;
    }
}
extern "C" int64_t psn_row_bytes(int32_t t, int64_t k) {
    const int64_t be = psn_block_elems(t);
    if (be == 0) return fail(PSN_E_UNSUPPORTED, "unknown tensor type %d", t);
    if (k <= 0 || k % be) return fail(PSN_E_SHAPE, "K=%lld is not a positive multiple of the block size %lld", (long long)k, (long long)be);
    return k / be * psn_block_bytes(t);
}
/* psn_quantize.cpp */
int psn_quantize_rows_impl(int32_t qtype, const float *x, int64_t n, int64_t k, uint8_t *out, int64_t row_bytes, int32_t threads);

extern "C" int32_t psn_quantize_rows(int32_t qtype, const float *x, int64_t n, int64_t k, void *out, size_t out_bytes, int32_t threads) {
    if (!x || !out) return fail(PSN_E_INVALID_ARG, "psn_quantize_rows: null pointer");
    if (qtype == PSN_Q8_K) return fail(PSN_E_UNSUPPORTED, "psn_quantize_rows: Q8_K is an activation format (psn_quantize_activations)");
    const int64_t rb = psn_row_bytes(qtype, k);
    if (rb < 0) return (int32_t)rb;
    if (n <= 0) return fail(PSN_E_SHAPE, "psn_quantize_rows: n=%lld", (long long)n);
    if ((uint64_t)n * (uint64_t)rb > out_bytes)
        return fail(PSN_E_INVALID_ARG, "psn_quantize_rows: output holds %zu bytes, %lld rows of %lld bytes need %lld", out_bytes,
                    (long long)n, (long long)rb, (long long)(n * rb));
    /* more threads than 256 help nobody; thread creation or allocation failures must not unwind through the C boundary */
    const int32_t nthreads = threads < 1 ? 1 : threads > 256 ? 256 : threads;
    try {
        if (psn_quantize_rows_impl(qtype, x, n, k, static_cast<uint8_t *>(out), rb, nthreads) != 0)
            return fail(PSN_E_UNSUPPORTED, "psn_quantize_rows: type %d has no quantizer", qtype);
    } catch (const std::bad_alloc &) {
        return fail(PSN_E_OOM, "psn_quantize_rows: host allocation failed");
    } catch (const std::exception &e) {
        return fail(PSN_E_INVALID_ARG, "psn_quantize_rows: %s (threads=%d)", e.what(), nthreads);
    }
    return PSN_OK;
}

int psn_dequantize_rows_impl(int32_t qtype, const uint8_t *in, int64_t n, int64_t k, float *out, int64_t row_bytes);

extern "C" int32_t psn_dequantize_rows(int32_t qtype, const void *blocks, int64_t n, int64_t k, float *out, size_t out_elems) {
    if (!blocks || !out) return fail(PSN_E_INVALID_ARG, "psn_dequantize_rows: null pointer");
    if (qtype == PSN_Q8_K) return fail(PSN_E_UNSUPPORTED, "psn_dequantize_rows: Q8_K is an activation format");
    const int64_t rb = psn_row_bytes(qtype, k);
    if (rb < 0) return (int32_t)rb;
    if (n <= 0) return fail(PSN_E_SHAPE, "psn_dequantize_rows: n=%lld", (long long)n);
    if ((uint64_t)n * (uint64_t)k > out_elems)
        return fail(PSN_E_INVALID_ARG, "psn_dequantize_rows: output holds %zu floats, %lld rows of %lld need %lld", out_elems, (long long)n,
                    (long long)k, (long long)(n * k));
    if (psn_dequantize_rows_impl(qtype, static_cast<const uint8_t *>(blocks), n, k, out, rb) != 0)
        return fail(PSN_E_UNSUPPORTED, "psn_dequantize_rows: type %d has no dequantizer", qtype);
    return PSN_OK;
}

static bool is_weight_type(int32_t t) { return t == PSN_Q4_0 || t == PSN_Q8_0 || t == PSN_Q4_K || t == PSN_Q5_K || t == PSN_Q6_K; }
static const char *fmt_name(int32_t t) {
    switch (t) {
        case PSN_Q4_0: return "q4_0";
        case PSN_Q8_0: return "q8_0";
        case PSN_Q4_K: return "q4_K";
        case PSN_Q5_K: return "q5_K";
        case PSN_Q6_K: return "q6_K";
        default: return "?";
    }
}
extern "C" int32_t psn_act_type_for(int32_t wt) {
    if (wt == PSN_Q4_0 || wt == PSN_Q8_0) return PSN_Q8_0;
    if (wt == PSN_Q4_K || wt == PSN_Q5_K || wt == PSN_Q6_K) return PSN_Q8_K;
    return fail(PSN_E_UNSUPPORTED, "type %d is not a weight type", wt);
}

static int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

extern "C" int32_t psn_actq_layout(int32_t act_type, int64_t K, int32_t batch, psn_actq_info *out) {
    if (!out) return fail(PSN_E_INVALID_ARG, "psn_actq_layout: out is null");
    if (batch < 1 || batch > 8) return fail(PSN_E_SHAPE, "batch=%d outside 1..8", batch);
    if (act_type != PSN_Q8_0 && act_type != PSN_Q8_K) return fail(PSN_E_UNSUPPORTED, "activation type %d (want Q8_0 or Q8_K)", act_type);
    const int64_t be = psn_block_elems(act_type);
    if (K <= 0 || K % be) return fail(PSN_E_SHAPE, "K=%lld is not a positive multiple of %lld", (long long)K, (long long)be);
    out->off_qs = 0;
    out->off_d = align_up(batch * K, 256);
    const int64_t d_bytes = batch * (K / be) * 4;
    out->off_s = out->off_d + align_up(d_bytes, 256);
    const int64_t s_bytes = act_type == PSN_Q8_0 ? batch * (K / 32) * 4 : batch * (K / 16) * 2;
    out->bytes = out->off_s + align_up(s_bytes, 256);
    return PSN_OK;
}

/* ------------------------------------------------------------------ handles */

struct psn_ctx {
    int device;
    int compute_units;
    int64_t total_mem;
    int max_lds;
    char arch[64];
};
/* A stream's workspace (quantized activations of psn_qmatvec, the dense prefill family's fp16 matrix).  Graph
 * nodes bake its address in, so the memory is owned jointly by the stream and by every graph recorded from a
 * launch that used it: it neither moves nor is freed while such a graph, or a capture that may become one,
 * exists.  Whoever lets go last (stream destroyed, last graph destroyed) frees it. */
struct ws_state {
    void *p = nullptr;
    size_t bytes = 0;
    int graph_refs = 0;    /* live graphs whose nodes hold p */
    int capture_refs = 0;  /* captures in progress that have recorded a node holding p */
    bool orphaned = false; /* the owning stream is gone; the last graph frees p */
    int device = 0;
};
struct psn_stream {
    psn_ctx *ctx;
    hipStream_t s;
    std::shared_ptr<ws_state> ws;
    hipEvent_t join_ev; /* created on first use by psn_stream_wait_stream */
};
struct psn_buf {
    psn_ctx *ctx;
    void *p;
    size_t bytes;
};
struct psn_event {
    psn_ctx *ctx;
    hipEvent_t e;
};
struct psn_graph {
    psn_ctx *ctx;
    hipGraph_t g;
    hipGraphExec_t exec;
    std::vector<std::shared_ptr<ws_state>> ws_held;   /* workspaces (of any stream that took part in the capture) whose address the nodes hold */
};
struct psn_module {
    psn_ctx *ctx;
    std::vector<hipModule_t> m;   /* one per code object; kernels are looked up across all */
    std::mutex mu;
    std::map<std::string, hipFunction_t, std::less<>> fn;   /* transparent comparator: a lookup by C string builds no std::string */
};

/* Workspaces touched by captures in progress, keyed by the capture's id (every stream that has joined a capture
 * reports the same id), so that psn_graph_end_capture on the origin stream also finds the workspaces of forked
 * side streams. */
static std::mutex g_cap_mu;
static std::unordered_map<unsigned long long, std::vector<std::shared_ptr<ws_state>>> g_cap_touched;

static int32_t bind(psn_ctx *c) {
    if (!c) return fail(PSN_E_INVALID_ARG, "context is null");
    HIP_TRY(hipSetDevice(c->device));
    return PSN_OK;
}

extern "C" int32_t psn_ctx_create(int32_t device, psn_ctx **out) {
    if (!out) return fail(PSN_E_INVALID_ARG, "psn_ctx_create: out is null");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) return fail(PSN_E_NO_DEVICE, "no HIP device visible (hipGetDeviceCount -> %d, count %d)", (int)e, n);
    if (device < 0 || device >= n) return fail(PSN_E_NO_DEVICE, "device %d out of range (0..%d)", device, n - 1);
    hipDeviceProp_t p;
    HIP_TRY(hipGetDeviceProperties(&p, device));
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0)
        return fail(PSN_E_NO_DEVICE, "device %d is %s; this library carries gfx950 code only", device, p.gcnArchName);
    HIP_TRY(hipSetDevice(device));
    psn_ctx *c = new (std::nothrow) psn_ctx();
    if (!c) return fail(PSN_E_OOM, "host allocation failed");
    c->device = device;
    c->compute_units = p.multiProcessorCount;
    c->total_mem = (int64_t)p.totalGlobalMem;
    c->max_lds = (int)p.sharedMemPerBlock;
    snprintf(c->arch, sizeof c->arch, "%s", p.gcnArchName);
    *out = c;
    return PSN_OK;
}
extern "C" int32_t psn_ctx_destroy(psn_ctx *c) {
    if (!c) return fail(PSN_E_INVALID_ARG, "context is null");
    delete c;
    return PSN_OK;
}
extern "C" int32_t psn_ctx_info(psn_ctx *c, int32_t *cus, int64_t *mem, char *name, size_t n) {
    if (!c) return fail(PSN_E_INVALID_ARG, "context is null");
    if (cus) *cus = c->compute_units;
    if (mem) *mem = c->total_mem;
    if (name && n) snprintf(name, n, "%s", c->arch);
    return PSN_OK;
}

extern "C" int32_t psn_ctx_mem_info(psn_ctx *c, int64_t *free_bytes, int64_t *total_bytes) {
    int32_t rc = bind(c);
    if (rc) return rc;
    size_t f = 0, t = 0;
    HIP_TRY(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = (int64_t)f;
    if (total_bytes) *total_bytes = (int64_t)t;
    return PSN_OK;
}

static int32_t load_images(psn_ctx *c, const psn_blob *blobs, int n, psn_module **out) {
    if (!out) return fail(PSN_E_INVALID_ARG, "psn_module_load: out is null");
    *out = nullptr;
    if (!c) return fail(PSN_E_INVALID_ARG, "context is null");
    for (int i = 0; i < n; ++i) {
        const size_t len = (size_t)(blobs[i].end - blobs[i].begin);
        if (!blobs[i].begin || len < 64) return fail(PSN_E_INVALID_ARG, "psn_module_load: empty code object");
        if (memcmp(blobs[i].begin, "\x7f" "ELF", 4) != 0 && memcmp(blobs[i].begin, "__CLANG_OFFLOAD_BUNDLE__", 24) != 0)
            return fail(PSN_E_MODULE, "psn_module_load: not an ELF code object or offload bundle");
    }
    int32_t rc = bind(c);
    if (rc) return rc;
    /* set-up of the no-allocation entry point: look up this GPU's copy of the static scratch now, so
     * that psn_qmatvec_noalloc itself never has to */
    {
        void *sp = nullptr;
        int herr = 0;
        if (psn_noalloc_scratch(c->device, &sp, nullptr, &herr) != 0)
            return fail(PSN_E_HIP, "static scratch of device %d could not be located: hipError %d (%s)", c->device, herr, hipGetErrorString((hipError_t)herr));
    }
    psn_module *mod = new (std::nothrow) psn_module();
    if (!mod) return fail(PSN_E_OOM, "host allocation failed");
    mod->ctx = c;
    for (int i = 0; i < n; ++i) {
        hipModule_t m;
        hipError_t e = hipModuleLoadData(&m, blobs[i].begin);
        if (e != hipSuccess) {
            for (hipModule_t h : mod->m) (void)hipModuleUnload(h);
            delete mod;
            return fail(PSN_E_MODULE, "hipModuleLoadData(code object %d): hipError %d (%s)", i, (int)e, hipGetErrorString(e));
        }
        mod->m.push_back(m);
    }
    *out = mod;
    return PSN_OK;
}
extern "C" int32_t psn_module_load(psn_ctx *c, const void *image, size_t len, psn_module **out) {
    const psn_blob b = {(const unsigned char *)image, (const unsigned char *)image + (image ? len : 0)};
    return load_images(c, &b, 1, out);
}
extern "C" int32_t psn_module_load_builtin(psn_ctx *c, psn_module **out) {
    return load_images(c, psn_builtin_blobs, psn_builtin_blob_count, out);
}
extern "C" int32_t psn_module_unload(psn_module *mod) {
    if (!mod) return fail(PSN_E_INVALID_ARG, "module is null");
    int32_t rc = bind(mod->ctx);
    if (rc) return rc;
    hipError_t first = hipSuccess;
    for (hipModule_t h : mod->m) {
        hipError_t e = hipModuleUnload(h);
        if (e != hipSuccess && first == hipSuccess) first = e;
    }
    delete mod;
    if (first != hipSuccess) return hip_fail(first, "hipModuleUnload");
    return PSN_OK;
}
static int32_t get_fn(psn_module *mod, const char *name, hipFunction_t *out) {
    std::lock_guard<std::mutex> lk(mod->mu);
    auto it = mod->fn.find(std::string_view(name));
    if (it != mod->fn.end()) { *out = it->second; return PSN_OK; }
    hipFunction_t f = nullptr;
    hipError_t e = hipErrorNotFound;
    for (hipModule_t h : mod->m) {
        e = hipModuleGetFunction(&f, h, name);
        if (e == hipSuccess) break;
    }
    if (e != hipSuccess) return fail(PSN_E_MODULE, "kernel '%s' not found in module: hipError %d (%s)", name, (int)e, hipGetErrorString(e));
    mod->fn.emplace(std::string(name), f);
    *out = f;
    return PSN_OK;
}
extern "C" int32_t psn_module_has_kernel(psn_module *mod, const char *name) {
    if (!mod || !name) return fail(PSN_E_INVALID_ARG, "module or name is null");
    int32_t rc = bind(mod->ctx);
    if (rc) return rc;
    hipFunction_t f;
    return get_fn(mod, name, &f);
}

extern "C" int32_t psn_stream_create(psn_ctx *c, psn_stream **out) {
    if (!out) return fail(PSN_E_INVALID_ARG, "psn_stream_create: out is null");
    *out = nullptr;
    int32_t rc = bind(c);
    if (rc) return rc;
    hipStream_t s;
    HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    psn_stream *st = new (std::nothrow) psn_stream();
    if (!st) { (void)hipStreamDestroy(s); return fail(PSN_E_OOM, "host allocation failed"); }
    st->ctx = c;
    st->s = s;
    st->ws = std::make_shared<ws_state>();
    st->ws->device = c->device;
    st->join_ev = nullptr;
    *out = st;
    return PSN_OK;
}
extern "C" int32_t psn_stream_sync(psn_stream *s) {
    if (!s) return fail(PSN_E_INVALID_ARG, "stream is null");
    int32_t rc = bind(s->ctx);
    if (rc) return rc;
    HIP_TRY(hipStreamSynchronize(s->s));
    return PSN_OK;
}
extern "C" int32_t psn_stream_destroy(psn_stream *s) {
    if (!s) return fail(PSN_E_INVALID_ARG, "stream is null");
    int32_t rc = bind(s->ctx);
    if (rc) return rc;
    (void)hipStreamSynchronize(s->s);
    {
        std::lock_guard<std::mutex> lk(g_cap_mu);
        if (s->ws->graph_refs > 0 || s->ws->capture_refs > 0) {
            s->ws->orphaned = true;                       /* graphs still hold the address: the last of them frees it */
        } else if (s->ws->p) {
            (void)hipFree(s->ws->p);
            s->ws->p = nullptr;
            s->ws->bytes = 0;
        }
    }
    if (s->join_ev) (void)hipEventDestroy(s->join_ev);
    hipError_t e = hipStreamDestroy(s->s);
    delete s;
    if (e != hipSuccess) return hip_fail(e, "hipStreamDestroy");
    return PSN_OK;
}

static int32_t is_capturing(psn_stream *s, bool *out) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    HIP_TRY(hipStreamIsCapturing(s->s, &st));
    *out = st != hipStreamCaptureStatusNone;
    return PSN_OK;
}
static int32_t refuse_while_capturing(psn_stream *s, const char *what) {
    bool cap = false;
    int32_t rc = is_capturing(s, &cap);
    if (rc) return rc;
    if (cap) return fail(PSN_E_INVALID_ARG, "%s: the stream is being captured into a graph (uploads, downloads and memsets are not recorded)", what);
    return PSN_OK;
}
static int32_t ensure_workspace(psn_stream *s, int64_t bytes) {
    ws_state &w = *s->ws;
    if (w.bytes >= (size_t)bytes) return PSN_OK;
    bool cap = false;
    int32_t rc = is_capturing(s, &cap);
    if (rc) return rc;
    if (cap) return fail(PSN_E_INVALID_ARG, "activation workspace must grow to %lld bytes during capture: call psn_stream_reserve first", (long long)bytes);
    {
        std::lock_guard<std::mutex> lk(g_cap_mu);
        if (w.capture_refs > 0 || w.graph_refs > 0)
            return fail(PSN_E_INVALID_ARG, "activation workspace (%zu bytes) is referenced by a captured graph and cannot grow to %lld bytes: "
                        "reserve the largest K x batch with psn_stream_reserve before the first capture", w.bytes, (long long)bytes);
    }
    /* earlier launches may still read the old workspace */
    HIP_TRY(hipStreamSynchronize(s->s));
    if (w.p) HIP_TRY(hipFree(w.p));
    w.p = nullptr;
    w.bytes = 0;
    const size_t want = (size_t)align_up(bytes, 1 << 20);
    hipError_t e = hipMalloc(&w.p, want);
    if (e != hipSuccess) return hip_fail(e, "hipMalloc(workspace)");
    w.bytes = want;
    return PSN_OK;
}
/* Called by every launch path that hands the workspace address to a kernel: if the stream is being captured
 * (as the origin of the capture or as a side stream forked into it), the capture is noted as holding the
 * workspace, whichever stream later ends it. */
static int32_t note_workspace_use(psn_stream *s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    unsigned long long id = 0;
    HIP_TRY(hipStreamGetCaptureInfo(s->s, &st, &id));
    if (st == hipStreamCaptureStatusNone) return PSN_OK;
    std::lock_guard<std::mutex> lk(g_cap_mu);
    auto &v = g_cap_touched[id];
    for (const auto &w : v)
        if (w == s->ws) return PSN_OK;
    v.push_back(s->ws);
    ++s->ws->capture_refs;
    return PSN_OK;
}
extern "C" int32_t psn_stream_reserve(psn_stream *s, int64_t K, int32_t batch) {
    if (!s) return fail(PSN_E_INVALID_ARG, "stream is null");
    if (K <= 0 || K % 256) return fail(PSN_E_SHAPE, "K=%lld must be a positive multiple of 256", (long long)K);
    psn_actq_info a, b;
    int32_t rc = psn_actq_layout(PSN_Q8_0, K, batch, &a);
    if (rc) return rc;
    if ((rc = psn_actq_layout(PSN_Q8_K, K, batch, &b))) return rc;
    if ((rc = bind(s->ctx))) return rc;
    return ensure_workspace(s, a.bytes > b.bytes ? a.bytes : b.bytes);
}

extern "C" int32_t psn_stream_wait_stream(psn_stream *waiter, psn_stream *signaler) {
    if (!waiter || !signaler) return fail(PSN_E_INVALID_ARG, "stream is null");
    if (waiter->ctx != signaler->ctx) return fail(PSN_E_INVALID_ARG, "streams belong to different contexts");
    int32_t rc = bind(waiter->ctx);
    if (rc) return rc;
    if (!signaler->join_ev) HIP_TRY(hipEventCreateWithFlags(&signaler->join_ev, hipEventDisableTiming));
    HIP_TRY(hipEventRecord(signaler->join_ev, signaler->s));
    HIP_TRY(hipStreamWaitEvent(waiter->s, signaler->join_ev, 0));
    return PSN_OK;
}

extern "C" int32_t psn_graph_begin_capture(psn_stream *s) {
    if (!s) return fail(PSN_E_INVALID_ARG, "stream is null");
    int32_t rc = bind(s->ctx);
    if (rc) return rc;
    HIP_TRY(hipStreamBeginCapture(s->s, hipStreamCaptureModeThreadLocal));
    return PSN_OK;
}
extern "C" int32_t psn_graph_end_capture(psn_stream *s, psn_graph **out) {
    if (!s || !out) return fail(PSN_E_INVALID_ARG, "stream or out is null");
    *out = nullptr;
    int32_t rc = bind(s->ctx);
    if (rc) return rc;
    hipGraph_t g = nullptr;
    /* the workspaces this capture touched, on this stream or on side streams forked into it */
    std::vector<std::shared_ptr<ws_state>> held;
    {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        unsigned long long id = 0;
        if (hipStreamGetCaptureInfo(s->s, &st, &id) == hipSuccess && st != hipStreamCaptureStatusNone) {
            std::lock_guard<std::mutex> lk(g_cap_mu);
            auto it = g_cap_touched.find(id);
            if (it != g_cap_touched.end()) {
                held.swap(it->second);
                g_cap_touched.erase(it);
            }
        }
    }
    auto release_capture_refs = [&](bool to_graph) {
        std::lock_guard<std::mutex> lk(g_cap_mu);
        for (auto &w : held) {
            --w->capture_refs;
            if (to_graph) ++w->graph_refs;
            else if (w->orphaned && w->graph_refs == 0 && w->capture_refs == 0 && w->p) { (void)hipFree(w->p); w->p = nullptr; w->bytes = 0; }
        }
    };
    hipError_t e = hipStreamEndCapture(s->s, &g);
    if (e != hipSuccess) { release_capture_refs(false); return hip_fail(e, "hipStreamEndCapture"); }
    if (!g) { release_capture_refs(false); return fail(PSN_E_HIP, "hipStreamEndCapture returned no graph (capture was invalidated)"); }
    hipGraphExec_t ex = nullptr;
    e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
    if (e != hipSuccess) { (void)hipGraphDestroy(g); release_capture_refs(false); return hip_fail(e, "hipGraphInstantiate"); }
    psn_graph *gr = new (std::nothrow) psn_graph();
    if (!gr) { (void)hipGraphExecDestroy(ex); (void)hipGraphDestroy(g); release_capture_refs(false); return fail(PSN_E_OOM, "host allocation failed"); }
    gr->ctx = s->ctx;
    gr->g = g;
    gr->exec = ex;
    release_capture_refs(true);
    gr->ws_held.swap(held);
    *out = gr;
    return PSN_OK;
}
extern "C" int32_t psn_graph_launch(psn_graph *g, psn_stream *s) {
    if (!g || !s) return fail(PSN_E_INVALID_ARG, "graph or stream is null");
    if (g->ctx != s->ctx) return fail(PSN_E_INVALID_ARG, "graph and stream belong to different contexts");
    int32_t rc = bind(g->ctx);
    if (rc) return rc;
    HIP_TRY(hipGraphLaunch(g->exec, s->s));
    return PSN_OK;
}
extern "C" int32_t psn_graph_destroy(psn_graph *g) {
    if (!g) return fail(PSN_E_INVALID_ARG, "graph is null");
    int32_t rc = bind(g->ctx);
    if (rc) return rc;
    (void)hipGraphExecDestroy(g->exec);
    (void)hipGraphDestroy(g->g);
    {
        std::lock_guard<std::mutex> lk(g_cap_mu);
        for (auto &w : g->ws_held) {
            --w->graph_refs;
            /* the stream that owned this workspace was destroyed while the graph lived: free it with the last graph */
            if (w->orphaned && w->graph_refs == 0 && w->capture_refs == 0 && w->p) { (void)hipFree(w->p); w->p = nullptr; w->bytes = 0; }
        }
    }
    delete g;
    return PSN_OK;
}

extern "C" int32_t psn_event_create(psn_ctx *c, psn_event **out) {
    if (!out) return fail(PSN_E_INVALID_ARG, "psn_event_create: out is null");
    *out = nullptr;
    int32_t rc = bind(c);
    if (rc) return rc;
    hipEvent_t e;
    HIP_TRY(hipEventCreate(&e));
    psn_event *ev = new (std::nothrow) psn_event();
    if (!ev) { (void)hipEventDestroy(e); return fail(PSN_E_OOM, "host allocation failed"); }
    ev->ctx = c;
    ev->e = e;
    *out = ev;
    return PSN_OK;
}
extern "C" int32_t psn_event_destroy(psn_event *e) {
    if (!e) return fail(PSN_E_INVALID_ARG, "event is null");
    int32_t rc = bind(e->ctx);
    if (rc) return rc;
    hipError_t r = hipEventDestroy(e->e);
    delete e;
    if (r != hipSuccess) return hip_fail(r, "hipEventDestroy");
    return PSN_OK;
}
extern "C" int32_t psn_event_record(psn_event *e, psn_stream *s) {
    if (!e || !s) return fail(PSN_E_INVALID_ARG, "event or stream is null");
    if (e->ctx != s->ctx) return fail(PSN_E_INVALID_ARG, "event and stream belong to different contexts");
    int32_t rc = bind(e->ctx);
    if (rc) return rc;
    HIP_TRY(hipEventRecord(e->e, s->s));
    return PSN_OK;
}
extern "C" int32_t psn_event_elapsed_us(const psn_event *b, const psn_event *e, double *out) {
    if (!b || !e || !out) return fail(PSN_E_INVALID_ARG, "event or out is null");
    int32_t rc = bind(e->ctx);
    if (rc) return rc;
    HIP_TRY(hipEventSynchronize(e->e));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, b->e, e->e));
    *out = (double)ms * 1000.0;
    return PSN_OK;
}

extern "C" int32_t psn_buf_alloc(psn_ctx *c, size_t bytes, psn_buf **out) {
    if (!out) return fail(PSN_E_INVALID_ARG, "psn_buf_alloc: out is null");
    *out = nullptr;
    if (bytes == 0) return fail(PSN_E_INVALID_ARG, "psn_buf_alloc: zero bytes");
    int32_t rc = bind(c);
    if (rc) return rc;
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) return hip_fail(e, "hipMalloc");
    psn_buf *b = new (std::nothrow) psn_buf();
    if (!b) { (void)hipFree(p); return fail(PSN_E_OOM, "host allocation failed"); }
    b->ctx = c;
    b->p = p;
    b->bytes = bytes;
    *out = b;
    return PSN_OK;
}
extern "C" int32_t psn_buf_free(psn_buf *b) {
    if (!b) return fail(PSN_E_INVALID_ARG, "buffer is null");
    int32_t rc = bind(b->ctx);
    if (rc) return rc;
    hipError_t e = hipFree(b->p);
    delete b;
    if (e != hipSuccess) return hip_fail(e, "hipFree");
    return PSN_OK;
}
extern "C" int64_t psn_buf_size(const psn_buf *b) {
    if (!b) return fail(PSN_E_INVALID_ARG, "buffer is null");
    return (int64_t)b->bytes;
}
static int32_t check_range(const psn_buf *b, size_t off, size_t n, const char *what) {
    if (!b) return fail(PSN_E_INVALID_ARG, "%s: buffer is null", what);
    if (off > b->bytes || n > b->bytes - off) return fail(PSN_E_INVALID_ARG, "%s: range [%zu, %zu) outside buffer of %zu bytes", what, off, off + n, b->bytes);
    return PSN_OK;
}
extern "C" int32_t psn_buf_upload(psn_buf *dst, size_t off, const void *src, size_t n, psn_stream *s) {
    int32_t rc = check_range(dst, off, n, "psn_buf_upload");
    if (rc) return rc;
    if (!src || !s) return fail(PSN_E_INVALID_ARG, "psn_buf_upload: src or stream is null");
    if (s->ctx != dst->ctx) return fail(PSN_E_INVALID_ARG, "psn_buf_upload: stream and buffer belong to different contexts");
    if ((rc = bind(dst->ctx))) return rc;
    if ((rc = refuse_while_capturing(s, "psn_buf_upload"))) return rc;
    if (n == 0) return PSN_OK;
    /* pageable source: the copy is staged, so the caller may reuse src on return */
    HIP_TRY(hipMemcpyAsync((char *)dst->p + off, src, n, hipMemcpyHostToDevice, s->s));
    HIP_TRY(hipStreamSynchronize(s->s));
    return PSN_OK;
}
extern "C" int32_t psn_buf_download(const psn_buf *src, size_t off, void *dst, size_t n, psn_stream *s) {
    int32_t rc = check_range(src, off, n, "psn_buf_download");
    if (rc) return rc;
    if (!dst || !s) return fail(PSN_E_INVALID_ARG, "psn_buf_download: dst or stream is null");
    if (s->ctx != src->ctx) return fail(PSN_E_INVALID_ARG, "psn_buf_download: stream and buffer belong to different contexts");
    if ((rc = bind(src->ctx))) return rc;
    if ((rc = refuse_while_capturing(s, "psn_buf_download"))) return rc;
    if (n == 0) return PSN_OK;
    HIP_TRY(hipMemcpyAsync(dst, (const char *)src->p + off, n, hipMemcpyDeviceToHost, s->s));
    HIP_TRY(hipStreamSynchronize(s->s));
    return PSN_OK;
}
extern "C" int32_t psn_buf_fill_zero(psn_buf *b, psn_stream *s) {
    if (!b || !s) return fail(PSN_E_INVALID_ARG, "buffer or stream is null");
    if (s->ctx != b->ctx) return fail(PSN_E_INVALID_ARG, "psn_buf_fill_zero: stream and buffer belong to different contexts");
    int32_t rc = bind(b->ctx);
    if (rc) return rc;
    /* a memset node must not end up in a graph (replays of such nodes have given wrong results) */
    if ((rc = refuse_while_capturing(s, "psn_buf_fill_zero"))) return rc;
    HIP_TRY(hipMemsetAsync(b->p, 0, b->bytes, s->s));
    return PSN_OK;
}

extern "C" int32_t psn_buf_copy(psn_buf *dst, size_t dst_off, const psn_buf *src, size_t src_off, size_t n, psn_stream *s) {
    int32_t rc = check_range(dst, dst_off, n, "psn_buf_copy(dst)");
    if (rc) return rc;
    if ((rc = check_range(src, src_off, n, "psn_buf_copy(src)"))) return rc;
    if (!s) return fail(PSN_E_INVALID_ARG, "psn_buf_copy: stream is null");
    if (s->ctx != dst->ctx || src->ctx != dst->ctx) return fail(PSN_E_INVALID_ARG, "psn_buf_copy: handles belong to different contexts");
    if ((rc = bind(dst->ctx))) return rc;
    if (n == 0) return PSN_OK;
    HIP_TRY(hipMemcpyAsync((char *)dst->p + dst_off, (const char *)src->p + src_off, n, hipMemcpyDeviceToDevice, s->s));
    return PSN_OK;
}

extern "C" int32_t psn_weight_upload(psn_ctx *c, int32_t qtype, int64_t N, int64_t K, const void *blocks, int32_t layout,
                                     psn_stream *s, psn_buf **out) {
    if (!out) return fail(PSN_E_INVALID_ARG, "psn_weight_upload: out is null");
    *out = nullptr;
    if (!c || !blocks || !s) return fail(PSN_E_INVALID_ARG, "psn_weight_upload: null argument");
    if (!is_weight_type(qtype)) return fail(PSN_E_UNSUPPORTED, "psn_weight_upload: type %d is not Q4_0/Q8_0/Q4_K/Q5_K/Q6_K", qtype);
    if (layout != PSN_LAYOUT_GGUF) return fail(PSN_E_UNSUPPORTED, "psn_weight_upload: layout %d", layout);
    if (N <= 0) return fail(PSN_E_SHAPE, "N=%lld must be positive", (long long)N);
    const int64_t rb = psn_row_bytes(qtype, K);
    if (rb < 0) return (int32_t)rb;
    psn_buf *b = nullptr;
    int32_t rc = psn_buf_alloc(c, (size_t)(N * rb), &b);
    if (rc) return rc;
    rc = psn_buf_upload(b, 0, blocks, (size_t)(N * rb), s);
    if (rc) { (void)psn_buf_free(b); return rc; }
    *out = b;
    return PSN_OK;
}

/* ------------------------------------------------------------------ launches */

/* The distinct kernels this thread has launched since psn_launch_log_clear(), in order of first launch,
 * "name;name;..." (what a throughput record cites as the kernels that actually ran).  Names that no longer
 * fit are dropped and the log ends in "...;". */
static thread_local char g_launch_log[1024] = "";
static thread_local size_t g_launch_log_len = 0;
static void log_launch(const char *kernel) {
    const size_t n = strlen(kernel);
    for (const char *p = g_launch_log; (p = strstr(p, kernel)) != nullptr; p += n)
        if ((p == g_launch_log || p[-1] == ';') && p[n] == ';') return;      /* already listed */
    if (g_launch_log_len + n + 1 + 4 < sizeof g_launch_log) {
        memcpy(g_launch_log + g_launch_log_len, kernel, n);
        g_launch_log_len += n;
        g_launch_log[g_launch_log_len++] = ';';
        g_launch_log[g_launch_log_len] = 0;
    } else if (g_launch_log_len + 4 < sizeof g_launch_log && (g_launch_log_len < 4 || memcmp(g_launch_log + g_launch_log_len - 4, "...;", 4) != 0)) {
        memcpy(g_launch_log + g_launch_log_len, "...;", 5);
        g_launch_log_len += 4;
    }
}
extern "C" void psn_launch_log_clear(void) {
    g_launch_log_len = 0;
    g_launch_log[0] = 0;
}
extern "C" const char *psn_launch_log(void) { return g_launch_log; }

static int32_t launch(psn_module *mod, psn_stream *s, const char *kernel, unsigned blocks, unsigned threads, unsigned lds,
                      void *args_struct) {
    hipFunction_t f;
    int32_t rc = get_fn(mod, kernel, &f);
    if (rc) return rc;
    log_launch(kernel);
    void *params[] = {args_struct};
    hipError_t e = hipModuleLaunchKernel(f, blocks, 1, 1, threads, 1, 1, lds, s->s, params, nullptr);
    if (e != hipSuccess) return fail(PSN_E_HIP, "launch of %s <<<%u,%u,%u>>> failed: hipError %d (%s)", kernel, blocks, threads, lds, (int)e, hipGetErrorString(e));
    return PSN_OK;
}

static int32_t check_same_ctx(psn_module *mod, psn_stream *s, const psn_buf *a, const psn_buf *b, const psn_buf *c, const char *what) {
    if (!mod || !s || !a || !b || !c) return fail(PSN_E_INVALID_ARG, "%s: null handle", what);
    if (s->ctx != mod->ctx || a->ctx != mod->ctx || b->ctx != mod->ctx || c->ctx != mod->ctx)
        return fail(PSN_E_INVALID_ARG, "%s: handles belong to different contexts", what);
    return PSN_OK;
}

static int32_t quantize_into(psn_module *mod, psn_stream *s, int32_t act_type, const float *x, void *xq, int64_t K, int32_t batch) {
    psn_actq_info li;
    int32_t rc = psn_actq_layout(act_type, K, batch, &li);
    if (rc) return rc;
    psn_quantize_args qa;
    qa.x = x;
    qa.qs = (int8_t *)xq + li.off_qs;
    qa.d = (float *)((char *)xq + li.off_d);
    qa.s = (char *)xq + li.off_s;
    qa.K = (int32_t)K;
    qa.batch = batch;
    if (act_type == PSN_Q8_0) {
        const int64_t threads = K * batch / 4;
        return launch(mod, s, "psn_quantize_q8_0", (unsigned)((threads + 255) / 256), 256, 0, &qa);
    }
    const int64_t waves = K * batch / 256;
    return launch(mod, s, "psn_quantize_q8_K", (unsigned)((waves + 3) / 4), 256, 0, &qa);
}

extern "C" int32_t psn_act_quantize(psn_module *mod, psn_stream *s, int32_t act_type, const psn_buf *x, psn_buf *xq, int64_t K, int32_t batch) {
    int32_t rc = check_same_ctx(mod, s, x, xq, xq, "psn_act_quantize");
    if (rc) return rc;
    psn_actq_info li;
    if ((rc = psn_actq_layout(act_type, K, batch, &li))) return rc;
    if (K > INT32_MAX / 8) return fail(PSN_E_SHAPE, "K=%lld too large", (long long)K);
    if ((int64_t)x->bytes < K * batch * 4) return fail(PSN_E_INVALID_ARG, "psn_act_quantize: x holds %zu bytes, need %lld", x->bytes, (long long)(K * batch * 4));
    if ((int64_t)xq->bytes < li.bytes) return fail(PSN_E_INVALID_ARG, "psn_act_quantize: x_q holds %zu bytes, need %lld", xq->bytes, (long long)li.bytes);
    if ((rc = bind(mod->ctx))) return rc;
    return quantize_into(mod, s, act_type, (const float *)x->p, xq->p, K, batch);
}

static int32_t check_matvec_shape(int32_t qtype, int32_t scheme, int64_t N, int64_t K, int32_t batch) {
    if (!is_weight_type(qtype)) return fail(PSN_E_UNSUPPORTED, "matvec: type %d is not Q4_0/Q8_0/Q4_K/Q5_K/Q6_K", qtype);
    if (scheme != PSN_ACT_F32 && scheme != PSN_ACT_Q8) return fail(PSN_E_UNSUPPORTED, "matvec: activation scheme %d", scheme);
    if (N <= 0 || N > INT32_MAX / 2) return fail(PSN_E_SHAPE, "N=%lld must be in 1..2^30", (long long)N);
    if (batch < 1 || batch > 8) return fail(PSN_E_SHAPE, "batch=%d outside 1..8", batch);
    const int64_t rb = psn_row_bytes(qtype, K);
    if (rb < 0) return (int32_t)rb;
    if (K % 256) return fail(PSN_E_SHAPE, "K=%lld: the gfx950 matvec kernels need K to be a multiple of 256", (long long)K);
    if (K > (1 << 24)) return fail(PSN_E_SHAPE, "K=%lld too large", (long long)K);
    return PSN_OK;
}

/* bytes of LDS the staged copy of a quantized activation takes (qs padded to 272 B per chunk) */
static int64_t staged_lds_bytes(int32_t qtype, int64_t K, int32_t batch) {
    const int32_t at = psn_act_type_for(qtype);
    const int64_t be = psn_block_elems(at);
    const int64_t qs = batch * (K / 256) * 272;
    const int64_t d = align_up(batch * (K / be) * 4, 16);
    const int64_t sb = at == PSN_Q8_0 ? batch * (K / 32) * 4 : batch * (K / 16) * 2;
    return qs + d + align_up(sb, 16);
}

/* Can the streaming kernel run this plan?  Fills in the dynamic LDS it needs.  n_rows may be null
 * (row counts unknown: only the shape-independent conditions are checked). */
static int32_t stream_plan_check(int32_t qtype, int32_t scheme, int64_t K, int32_t batch, const psn_matvec_plan *plan, const int64_t *n_rows,
                                 int32_t count, int max_lds, int64_t *lds_out) {
    const int g = plan->lanes_per_row, rows = 64 / g, ring = plan->stream;
    const int64_t C = K / 256;
    if (scheme != PSN_ACT_Q8 || batch != 1 || plan->batch_tile != 1 || plan->rows_in_flight != 1)
        return fail(PSN_E_UNSUPPORTED, "plan: the streaming kernels serve scheme Q8 at batch 1");
    if (psn_row_bytes(qtype, K) % 16) return fail(PSN_E_UNSUPPORTED, "plan: streaming needs rows of whole 16-byte words (Q6_K: K a multiple of 2048)");
    if (C > g) return fail(PSN_E_UNSUPPORTED, "plan: streaming needs rows of at most lanes_per_row chunks (K <= %d)", g * 256);
    if (plan->stage_lds < 1 || plan->stage_lds > 3) return fail(PSN_E_UNSUPPORTED, "plan: streaming needs stage_lds 1, 2 or 3");
    if (plan->stage_lds == 3 && (g > 32 || count > 3)) return fail(PSN_E_UNSUPPORTED, "plan: the norm-fused kernels exist for rows of at most 32 chunks and three matrices");
    if (plan->threads < 256 || plan->threads > 512 || plan->threads % 64) return fail(PSN_E_UNSUPPORTED, "plan: threads=%d (256 .. 512, whole waves)", plan->threads);
    if (ring < 1 || ring > 8) return fail(PSN_E_UNSUPPORTED, "plan: stream=%d (passes in flight per wave, 1..8)", ring);
    for (int i = 0; n_rows && i < count; ++i)
        if (n_rows[i] % rows) return fail(PSN_E_UNSUPPORTED, "plan: streaming needs every matrix to hold a multiple of %d rows", rows);
    const int32_t at = psn_act_type_for(qtype);
    const int64_t be = psn_block_elems(at);
    const int64_t rb = psn_row_bytes(qtype, K);
    const int64_t nloads = (rows * rb + 1023) / 1024;
    if ((ring - 1) * nloads > 63) return fail(PSN_E_UNSUPPORTED, "plan: %d passes of %lld loads exceed the load counter", ring, (long long)nloads);
    /* the activations pass through at most eight 16-byte registers per thread on their way into LDS */
    const int64_t slots = 8 * (int64_t)plan->threads;
    /* (four, when x, the residual delta and the norm weights travel together) */
    const int64_t f32_regs = plan->stage_lds == 3 ? 4 : 8;
    const bool fits = plan->stage_lds == 1 ? (C * 16 <= slots && (K / be) * 4 <= 16 * (int64_t)plan->threads)
                      : at == PSN_Q8_0   ? C * 64 <= f32_regs * (int64_t)plan->threads
                                         : C <= f32_regs * (int64_t)(plan->threads / 64);
    if (!fits) return fail(PSN_E_UNSUPPORTED, "plan: K=%lld is too long for %d threads to stage in one round", (long long)K, plan->threads);
    const int64_t n_d = ((K / be) * 4 + 15) / 16, n_s = ((at == PSN_Q8_0 ? (K / 32) * 4 : (K / 16) * 2) + 15) / 16;
    const int64_t stage = (C * 272 + (n_d + n_s) * 16 + (plan->stage_lds == 3 ? 64 : 0) + 1023) / 1024 * 1024;
    const int64_t total = stage + (int64_t)(plan->threads / 64) * ring * nloads * 1024;
    if (total > max_lds) return fail(PSN_E_UNSUPPORTED, "plan: streaming needs %lld bytes of LDS, device offers %d", (long long)total, max_lds);
    *lds_out = total;
    return PSN_OK;
}

/* Can the small-batch MFMA kernel run this plan?  Fills in the dynamic LDS it needs. */
static int32_t mfma_plan_check(int32_t qtype, int32_t scheme, int64_t K, int32_t batch, const psn_matvec_plan *plan, const int64_t *n_rows,
                               int32_t count, int max_lds, int64_t *lds_out) {
    const int ks = plan->mfma;
    const int64_t C = K / 256;
    if (scheme != PSN_ACT_Q8 || (qtype != PSN_Q4_K && qtype != PSN_Q5_K)) return fail(PSN_E_UNSUPPORTED, "plan: the MFMA kernels serve Q4_K and Q5_K with scheme Q8");
    if (batch < 1 || batch > 8) return fail(PSN_E_UNSUPPORTED, "plan: batch=%d", batch);
    if (plan->stage_lds != 1) return fail(PSN_E_UNSUPPORTED, "plan: the MFMA kernels take quantized activations (stage_lds 1)");
    if (plan->threads != 256 && plan->threads != 512) return fail(PSN_E_UNSUPPORTED, "plan: threads=%d (256 or 512)", plan->threads);
    const int waves = plan->threads / 64;
    if (!(ks == 1 || ks == 2 || ks == 4 || ks == 8) || ks > waves) return fail(PSN_E_UNSUPPORTED, "plan: mfma=%d (1, 2, 4 or 8 waves per tile, at most the workgroup's)", ks);
    if (C % ks || C / ks > 8) return fail(PSN_E_UNSUPPORTED, "plan: K=%lld does not split into %d slices of at most eight chunks", (long long)K, ks);
    if (C * 8 > 2 * (int64_t)plan->threads) return fail(PSN_E_UNSUPPORTED, "plan: K=%lld is too long for %d threads to stage the activation sums", (long long)K, plan->threads);
    for (int i = 0; n_rows && i < count; ++i)
        if (n_rows[i] % 16) return fail(PSN_E_UNSUPPORTED, "plan: the MFMA kernels need every matrix to hold a multiple of 16 rows");
    if (plan->blocks < 1 || plan->blocks > (1 << 20)) return fail(PSN_E_UNSUPPORTED, "plan: blocks=%d", plan->blocks);
    if (plan->stream != 1) return fail(PSN_E_UNSUPPORTED, "plan: stream=%d (with mfma: 1)", plan->stream);
    /* slices of more than four chunks run the kernel whose waves handle exactly one unit each */
    if (C / ks > 4 && n_rows) {
        int64_t tiles = 0;
        for (int i = 0; i < count; ++i) tiles += n_rows[i] / 16;
        if ((int64_t)plan->blocks * (waves / ks) < tiles)
            return fail(PSN_E_UNSUPPORTED, "plan: slices of %lld chunks need one wave per unit (%lld tiles, %d workgroups of %d)", (long long)(C / ks), (long long)tiles, plan->blocks, waves / ks);
    }
    /* tables, 1 KB per wave, and per wave a ring of four chunks (9 or 11 KB) */
    const int64_t total = C * 160 + (int64_t)waves * 1024 + (int64_t)waves * (qtype == PSN_Q4_K ? 9 : 11) * 1024;
    if (total > max_lds) return fail(PSN_E_UNSUPPORTED, "plan: the MFMA kernel needs %lld bytes of LDS, device offers %d", (long long)total, max_lds);
    *lds_out = total;
    return PSN_OK;
}

/* n_rows: the row counts of the matrices sharing the launch (count of them), or null when unknown */
static int32_t make_plan(int32_t qtype, int32_t scheme, int64_t N, int64_t K, int32_t batch, int32_t cus, bool fuse_quantize,
                         const int64_t *n_rows, int32_t count, psn_matvec_plan *out) {
    int32_t rc = check_matvec_shape(qtype, scheme, N, K, batch);
    if (rc) return rc;
    if (cus <= 0) cus = 256;
    const int64_t C = K / 256;
    psn_matvec_plan p;
    p.batch_tile = batch <= 1 ? 1 : batch <= 2 ? 2 : batch <= 4 ? 4 : 8;
    p.rows_in_flight = 1;
    p.stream = 0;
    p.mfma = 0;
    /* the staged activations may take the whole 160 KB of a compute unit's LDS (batch 8 at K = 14336
     * needs 140 KB); re-quantizing inside the launch only pays up to batch 2 -- beyond that every
     * workgroup would redo batch x K of quantization, and one extra launch is cheaper (measured) */
    const bool lds_fits = scheme == PSN_ACT_Q8 ? staged_lds_bytes(qtype, K, batch) <= 160 * 1024 : (int64_t)batch * C * 1040 <= 160 * 1024;
    p.stage_lds = !lds_fits ? 0 : scheme == PSN_ACT_F32 ? 1 : ((fuse_quantize && batch <= 2) ? 2 : 1);

    /* lanes per row: the row's chunk count rounded up to a power of two, widened (idle lanes, more
     * waves) until the launch offers about four waves per compute unit */
    int g = C <= 8 ? 8 : C <= 16 ? 16 : C <= 32 ? 32 : 64;
    while (g < 64 && (N + (64 / g) - 1) / (64 / g) < (int64_t)cus * 4) g *= 2;
    int64_t waves = (N + (64 / g) - 1) / (64 / g);
    int64_t blocks;
    /* Batch 1, int8 path, rows of at most 64 chunks, whole passes in every matrix: the streaming kernel
     * (weights by direct-to-LDS loads).  One pass per wave where the chip holds that many waves, else as
     * many workgroups as stay resident (LDS) and the waves loop; measured on MI355X. */
    if (scheme == PSN_ACT_Q8 && batch == 1 && C <= 64 && n_rows != nullptr && p.stage_lds != 0) {
        int gs = 8;
        while (gs < C) gs *= 2;
        const int rows = 64 / gs;
        bool whole = true;
        for (int i = 0; i < count; ++i) whole = whole && n_rows[i] % rows == 0;
        psn_matvec_plan q = p;
        q.lanes_per_row = gs;
        q.stream = 1;
        /* One pass per wave while the chip holds that many waves in one workgroup per compute unit
         * (four waves up to eight, so that every compute unit gets a workgroup); beyond that, four-wave
         * workgroups, as many as stay resident, and the waves loop.  fp32 activations pass through
         * registers on their way into LDS: 256 threads hold K <= 8192.  (Measured on MI355X: 1536 passes
         * run 6.0 us with 256 x 384 threads, 6.4 us with 192 x 512, 7.0 us with 384 x 256.) */
        const int64_t npass = N / rows;
        /* (Between eight and sixteen passes per compute unit, e.g. one 14336 x 4096 matrix: eight-wave workgroups, one
         * per compute unit, whose waves loop twice, measured 9.0-9.7 us against 10.5-11.4 us for three four-wave workgroups.) */
        const bool two_rounds = npass > 8 * (int64_t)cus && npass <= 16 * (int64_t)cus;
        q.threads = two_rounds || (p.stage_lds == 2 && K > 8192) ? 512
                    : npass > 4 * (int64_t)cus && npass <= 8 * (int64_t)cus ? 64 * (int32_t)((npass + cus - 1) / cus) : 256;
        int64_t lds = 0;
        q.blocks = 1;
        if (whole && stream_plan_check(qtype, scheme, K, batch, &q, n_rows, count, 160 * 1024, &lds) == PSN_OK) {
            const int64_t wpb = q.threads / 64;
            int64_t resident = (160 * 1024) / lds;
            if (resident > 3) resident = 3;
            if (resident < 1) resident = 1;
            int64_t b = (npass + wpb - 1) / wpb;
            if (b > resident * cus) b = resident * cus;
            if (two_rounds && b > cus) b = cus;
            q.blocks = (int32_t)b;
            *out = q;
            return PSN_OK;
        }
        g_err[0] = 0;                                   /* not streamable after all: the register kernels take it */
    }
    /* Batch 3..8 of Q4_K / Q5_K on quantized activations: the int8-MFMA kernel, whose cost per weight
     * does not grow with the batch (measured on MI355X against the register kernels over nine shapes:
     * 1.1-2.1 x faster at batch 8, 0.75-0.95 x at batch 2 -- so batch 2 stays with the register kernels,
     * except fp32 input with rows longer than 8192, where a quantize launch + this kernel beats
     * re-quantizing in every workgroup, 14.3 against 20.7 us at 4096 x 14336).
     * Candidates: four waves (two workgroups per compute unit) or eight (one), any slice count that
     * leaves whole slices of at most eight chunks and fits the LDS.  Preferred: the one that gives every
     * compute unit a workgroup, then slices of at most four chunks (the kernel whose waves may walk
     * several units), then four-wave workgroups.  One unit in flight per wave: deeper rings and more
     * resident workgroups both measured slower. */
    const bool mfma_batch = batch >= 3 || (batch == 2 && fuse_quantize && K > 8192);
    if (scheme == PSN_ACT_Q8 && mfma_batch && (qtype == PSN_Q4_K || qtype == PSN_Q5_K) && n_rows != nullptr) {
        psn_matvec_plan q = p, best_q = p;
        q.stage_lds = 1;
        q.lanes_per_row = 16;
        q.stream = 1;
        q.batch_tile = 8;
        const int64_t ntiles = N / 16;
        int64_t best_score = -1;
        for (int threads = 256; threads <= 512; threads *= 2) {
            for (int ks = 1; ks <= threads / 64; ks *= 2) {
                if (C % ks || C / ks > 8) continue;
                q.threads = threads;
                q.mfma = ks;
                const int64_t tpw = (threads / 64) / ks, cap = (threads == 256 ? 2 : 1) * (int64_t)cus;
                int64_t b = (ntiles + tpw - 1) / tpw;
                const bool short_slices = C / ks <= 4;
                if (b > cap && short_slices) b = cap;       /* longer slices: one unit per wave, the grid covers every tile */
                q.blocks = (int32_t)b;
                int64_t lds = 0;
                if (mfma_plan_check(qtype, scheme, K, batch, &q, n_rows, count, 160 * 1024, &lds) != PSN_OK) continue;
                const int64_t busy = b < cus ? b : cus;     /* compute units with a workgroup */
                const int64_t score = busy * 8 + (short_slices ? 4 : 0) + (threads == 256 ? 2 : 0) + (ks <= 4 ? 1 : 0);
                if (score > best_score) { best_score = score; best_q = q; }
            }
        }
        g_err[0] = 0;
        if (best_score >= 0) {
            *out = best_q;
            return PSN_OK;
        }
        g_err[0] = 0;                                   /* shape not served: the register kernels take it */
    }
    if (p.stage_lds == 2) {
        /* Every workgroup re-quantizes x while staging it, a cost proportional to K: keep to about
         * eight waves per compute unit in as few workgroups as stream well; tall matrices of short rows
         * (twelve waves' worth of rows per compute unit and more) run better as three four-wave
         * workgroups per compute unit, two for Q6_K (measured on MI355X at batch 2, 14336 and 28672 rows
         * of K = 4096: 7-12 % faster than one eight-wave workgroup). */
        while (g < 64 && waves * 2 <= (int64_t)cus * 8) { g *= 2; waves = (N + (64 / g) - 1) / (64 / g); }
        const bool small_groups = K <= 8192 && waves >= (int64_t)cus * 12;
        p.threads = small_groups ? 256 : 512;
        const int64_t wpb = p.threads / 64;
        blocks = (waves + wpb - 1) / wpb;
        const int64_t cap = small_groups ? (qtype == PSN_Q6_K ? 2 : 3) * (int64_t)cus : (int64_t)cus;
        if (blocks > cap) blocks = cap;
    } else {
        /* small workgroups, one pass per wave where the chip can hold them */
        p.threads = 256;
        blocks = (waves + 3) / 4;
        /* two workgroups per compute unit stream best for the int8 path, four for the fp32 path (measured) */
        const int64_t cap = (scheme == PSN_ACT_F32 ? 4 : 2) * (int64_t)cus;
        if (blocks > cap) blocks = cap;
        if (staged_lds_bytes(qtype, K, batch) > 40 * 1024) {
            /* a big staged copy limits how many workgroups fit a compute unit: fewer, larger ones */
            p.threads = 512;
            blocks = (waves + 7) / 8;
            if (blocks > (int64_t)cus) blocks = cus;
        }
    }
    p.lanes_per_row = g;
    p.blocks = (int32_t)blocks;
    *out = p;
    return PSN_OK;
}

extern "C" int32_t psn_qmatvec_plan(int32_t qtype, int32_t scheme, int64_t N, int64_t K, int32_t batch, int32_t cus,
                                    int32_t x_is_f32, psn_matvec_plan *out) {
    if (!out) return fail(PSN_E_INVALID_ARG, "psn_qmatvec_plan: out is null");
    return make_plan(qtype, scheme, N, K, batch, cus, x_is_f32 != 0 && scheme == PSN_ACT_Q8, &N, 1, out);
}

static int32_t plan_is_valid(const psn_matvec_plan *p, int32_t qtype, int32_t scheme, int64_t K, int32_t batch, int max_lds, int32_t *lds_out) {
    const int g = p->lanes_per_row, r = p->rows_in_flight, nb = p->batch_tile;
    if (!(g == 8 || g == 16 || g == 32 || g == 64)) return fail(PSN_E_UNSUPPORTED, "plan: lanes_per_row=%d", g);
    if (nb < batch || !(nb == 1 || nb == 2 || nb == 4 || nb == 8)) return fail(PSN_E_UNSUPPORTED, "plan: batch_tile=%d for batch %d", nb, batch);
    /* the streaming kernels index by the wave count they are given; the others are written for four or eight waves */
    if (p->stream && p->mfma == 0 ? (p->threads < 256 || p->threads > 512 || p->threads % 64) : (p->threads != 256 && p->threads != 512))
        return fail(PSN_E_UNSUPPORTED, "plan: threads=%d (256 or 512; streaming kernels: 256 .. 512 in whole waves)", p->threads);
    if (r != 1) return fail(PSN_E_UNSUPPORTED, "plan: no kernel for rows_in_flight=%d batch_tile=%d scheme=%d", r, nb, scheme);
    if (p->blocks < 1 || p->blocks > (1 << 20)) return fail(PSN_E_UNSUPPORTED, "plan: blocks=%d", p->blocks);
    int32_t lds = 0;
    if (p->stage_lds < 0 || p->stage_lds > 3 || (p->stage_lds == 3 && !p->stream)) return fail(PSN_E_UNSUPPORTED, "plan: stage_lds=%d", p->stage_lds);
    if (p->stage_lds && scheme == PSN_ACT_F32) {
        if (p->stage_lds != 1) return fail(PSN_E_UNSUPPORTED, "plan: scheme F32 stages fp32 activations (stage_lds 0 or 1)");
        const int64_t total = (int64_t)batch * (K / 256) * 1040;
        if (total > max_lds) return fail(PSN_E_UNSUPPORTED, "plan: LDS staging needs %lld bytes, device offers %d", (long long)total, max_lds);
        lds = (int32_t)total;
    } else if (p->stage_lds) {
        const int64_t total = staged_lds_bytes(qtype, K, batch);
        if (total > max_lds) return fail(PSN_E_UNSUPPORTED, "plan: LDS staging needs %lld bytes, device offers %d", (long long)total, max_lds);
        lds = (int32_t)total;
    }
    *lds_out = lds;
    return PSN_OK;
}

struct seg_list {
    int32_t count;
    const void *W[PSN_MAX_SEGMENTS];
    float *y[PSN_MAX_SEGMENTS];
    int64_t N[PSN_MAX_SEGMENTS];
    int64_t total;
};

/* the extra operands of a launch that adds a residual and normalizes while it stages x (stage_lds 3) */
struct norm_fusion {
    const float *delta, *weight;
    float *h_out;
    float eps;
    bool pair;      /* two matrices, a gate and an up projection: the launch stores silu(W0 x) * (W1 x) into y[0] */
};

static int32_t run_matvec(psn_module *mod, psn_stream *s, int32_t qtype, int32_t scheme, const seg_list &sg, const void *x,
                          int64_t K, int32_t batch, const psn_matvec_plan *plan, const norm_fusion *norm = nullptr) {
    int32_t lds = 0;
    int32_t rc = plan->mfma ? PSN_OK : plan_is_valid(plan, qtype, scheme, K, batch, mod->ctx->max_lds, &lds);
    if (rc) return rc;
    psn_matvec_args a;
    memset(&a, 0, sizeof a);
    int64_t end = 0;
    for (int i = 0; i < PSN_MAX_SEGMENTS; ++i) {
        const int j = i < sg.count ? i : sg.count - 1;
        if (i < sg.count) end += sg.N[i];
        a.W[i] = (const uint8_t *)sg.W[j];
        a.y[i] = sg.y[j];
        a.row_end[i] = (int32_t)end;
    }
    a.N = (int32_t)sg.total;
    a.K = (int32_t)K;
    a.batch = batch;
    a.nseg = sg.count;
    a.row_bytes = psn_row_bytes(qtype, K);
    a.threads = plan->threads;
    a.blocks = plan->blocks;
    char name[96];
    if (plan->mfma) {
        int64_t total = 0;
        if ((rc = mfma_plan_check(qtype, scheme, K, batch, plan, sg.N, sg.count, mod->ctx->max_lds, &total))) return rc;
        psn_actq_info li;
        if ((rc = psn_actq_layout(psn_act_type_for(qtype), K, batch, &li))) return rc;
        a.xqs = (const int8_t *)x + li.off_qs;
        a.xd = (const float *)((const char *)x + li.off_d);
        a.xs = (const char *)x + li.off_s;
        a.kslices = plan->mfma;
        snprintf(name, sizeof name, "psn_mvm_%s_q8_%s", fmt_name(qtype), (K / 256) / plan->mfma > 4 ? "t8" : "p4");
        return launch(mod, s, name, (unsigned)plan->blocks, (unsigned)plan->threads, (unsigned)total, &a);
    }
    if (plan->stream) {
        const int g = plan->lanes_per_row, rows = 64 / g, ring = plan->stream;
        int64_t total = 0;
        if ((rc = stream_plan_check(qtype, scheme, K, batch, plan, sg.N, sg.count, mod->ctx->max_lds, &total))) return rc;
        const int32_t at = psn_act_type_for(qtype);
        if (plan->stage_lds == 3) {
            if (!norm) return fail(PSN_E_INVALID_ARG, "plan: stage_lds 3 is the norm-fused launch (psn_qmatvec_norm_multi)");
            a.xf = (const float *)x;
            a.x_delta = norm->delta;
            a.norm_w = norm->weight;
            a.h_out = norm->h_out;
            a.eps = norm->eps;
        } else if (plan->stage_lds == 2) {
            a.xf = (const float *)x;
        } else {
            psn_actq_info li;
            if ((rc = psn_actq_layout(at, K, batch, &li))) return rc;
            a.xqs = (const int8_t *)x + li.off_qs;
            a.xd = (const float *)((const char *)x + li.off_d);
            a.xs = (const char *)x + li.off_s;
        }
        a.ring = ring;
        (void)rows;
        if (norm && norm->pair && (plan->stage_lds != 3 || sg.count != 2 || sg.N[0] != sg.N[1] || g > 32))
            return fail(PSN_E_UNSUPPORTED, "plan: the SwiGLU-fused launch takes two matrices of equal height on the norm-fused streaming kernels");
        snprintf(name, sizeof name, "psn_mvs_%s_q8_g%d_%s_s%d", fmt_name(qtype), g,
                 plan->stage_lds == 3 ? (norm->pair ? "xnp" : "xn") : plan->stage_lds == 2 ? "xf" : "lds", sg.count);
        return launch(mod, s, name, (unsigned)plan->blocks, (unsigned)plan->threads, (unsigned)total, &a);
    }
    if (scheme == PSN_ACT_Q8 && plan->stage_lds == 2) {
        a.xf = (const float *)x;
        snprintf(name, sizeof name, "psn_mv_%s_q8_g%d_r%d_b%d_xf", fmt_name(qtype), plan->lanes_per_row, plan->rows_in_flight, plan->batch_tile);
    } else if (scheme == PSN_ACT_Q8) {
        psn_actq_info li;
        if ((rc = psn_actq_layout(psn_act_type_for(qtype), K, batch, &li))) return rc;
        a.xqs = (const int8_t *)x + li.off_qs;
        a.xd = (const float *)((const char *)x + li.off_d);
        a.xs = (const char *)x + li.off_s;
        snprintf(name, sizeof name, "psn_mv_%s_q8_g%d_r%d_b%d%s", fmt_name(qtype), plan->lanes_per_row, plan->rows_in_flight,
                 plan->batch_tile, plan->stage_lds ? "_lds" : "");
    } else {
        a.xf = (const float *)x;
        snprintf(name, sizeof name, "psn_mv_%s_f32_g%d_r%d_b%d%s", fmt_name(qtype), plan->lanes_per_row, plan->rows_in_flight, plan->batch_tile,
                 plan->stage_lds ? "_lds" : "");
    }
    return launch(mod, s, name, (unsigned)plan->blocks, (unsigned)plan->threads, (unsigned)lds, &a);
}

/* validates handles, shapes and buffer sizes of a (multi-)matvec and flattens it into a seg_list */
static int32_t gather_segments(const char *what, psn_module *mod, psn_stream *s, int32_t qtype, int32_t scheme, int32_t count,
                               const psn_buf *const *W, const psn_buf *x, psn_buf *const *y, const int64_t *N, int64_t K,
                               int32_t batch, seg_list *out) {
    if (!mod || !s || !W || !x || !y || !N) return fail(PSN_E_INVALID_ARG, "%s: null handle", what);
    if (count < 1 || count > PSN_MAX_SEGMENTS) return fail(PSN_E_SHAPE, "%s: count=%d outside 1..%d", what, count, PSN_MAX_SEGMENTS);
    if (s->ctx != mod->ctx || x->ctx != mod->ctx) return fail(PSN_E_INVALID_ARG, "%s: handles belong to different contexts", what);
    out->count = count;
    out->total = 0;
    for (int i = 0; i < count; ++i) {
        if (!W[i] || !y[i]) return fail(PSN_E_INVALID_ARG, "%s: null buffer for matrix %d", what, i);
        if (W[i]->ctx != mod->ctx || y[i]->ctx != mod->ctx) return fail(PSN_E_INVALID_ARG, "%s: handles belong to different contexts", what);
        int32_t rc = check_matvec_shape(qtype, scheme, N[i], K, batch);
        if (rc) return rc;
        const int64_t need_w = N[i] * psn_row_bytes(qtype, K);
        if ((int64_t)W[i]->bytes < need_w) return fail(PSN_E_INVALID_ARG, "%s: W[%d] holds %zu bytes, need %lld", what, i, W[i]->bytes, (long long)need_w);
        if ((int64_t)y[i]->bytes < N[i] * batch * 4) return fail(PSN_E_INVALID_ARG, "%s: y[%d] holds %zu bytes, need %lld", what, i, y[i]->bytes, (long long)(N[i] * batch * 4));
        out->W[i] = W[i]->p;
        out->y[i] = (float *)y[i]->p;
        out->N[i] = N[i];
        out->total += N[i];
    }
    if (out->total > INT32_MAX / 2) return fail(PSN_E_SHAPE, "%s: %lld rows in one launch", what, (long long)out->total);
    return PSN_OK;
}

static int32_t check_x_q8(const char *what, int32_t qtype, const psn_buf *x, int64_t K, int32_t batch) {
    psn_actq_info li;
    int32_t rc = psn_actq_layout(psn_act_type_for(qtype), K, batch, &li);
    if (rc) return rc;
    if ((int64_t)x->bytes < li.bytes) return fail(PSN_E_INVALID_ARG, "%s: x_q holds %zu bytes, need %lld", what, x->bytes, (long long)li.bytes);
    return PSN_OK;
}
static int32_t check_x_f32(const char *what, const psn_buf *x, int64_t K, int32_t batch) {
    if ((int64_t)x->bytes < K * batch * 4) return fail(PSN_E_INVALID_ARG, "%s: x holds %zu bytes, need %lld", what, x->bytes, (long long)(K * batch * 4));
    return PSN_OK;
}

extern "C" int32_t psn_qmatvec_planned(psn_module *mod, psn_stream *s, int32_t qtype, int32_t scheme, int32_t count,
                                       const psn_buf *const *W, const psn_buf *x, psn_buf *const *y, const int64_t *N, int64_t K,
                                       int32_t batch, const psn_matvec_plan *plan) {
    if (!plan) return fail(PSN_E_INVALID_ARG, "psn_qmatvec_planned: plan is null");
    seg_list sg;
    int32_t rc = gather_segments("psn_qmatvec_planned", mod, s, qtype, scheme, count, W, x, y, N, K, batch, &sg);
    if (rc) return rc;
    const bool x_is_q8 = scheme == PSN_ACT_Q8 && plan->stage_lds != 2;
    if ((rc = x_is_q8 ? check_x_q8("psn_qmatvec_planned", qtype, x, K, batch) : check_x_f32("psn_qmatvec_planned", x, K, batch))) return rc;
    if ((rc = bind(mod->ctx))) return rc;
    return run_matvec(mod, s, qtype, scheme, sg, x->p, K, batch, plan);
}

extern "C" int32_t psn_qmatvec_q8_multi(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, int32_t count,
                                        const psn_buf *const *W, const psn_buf *xq, psn_buf *const *y, const int64_t *N, int64_t K,
                                        int32_t batch) {
    if (layout != PSN_LAYOUT_GGUF) return fail(PSN_E_UNSUPPORTED, "matvec: layout %d", layout);
    seg_list sg;
    int32_t rc = gather_segments("psn_qmatvec_q8_multi", mod, s, qtype, PSN_ACT_Q8, count, W, xq, y, N, K, batch, &sg);
    if (rc) return rc;
    if ((rc = check_x_q8("psn_qmatvec_q8_multi", qtype, xq, K, batch))) return rc;
    psn_matvec_plan plan;
    if ((rc = make_plan(qtype, PSN_ACT_Q8, sg.total, K, batch, mod->ctx->compute_units, false, sg.N, sg.count, &plan))) return rc;
    if ((rc = bind(mod->ctx))) return rc;
    return run_matvec(mod, s, qtype, PSN_ACT_Q8, sg, xq->p, K, batch, &plan);
}

extern "C" int32_t psn_qmatvec_q8(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, const psn_buf *W,
                                  const psn_buf *xq, psn_buf *y, int64_t N, int64_t K, int32_t batch) {
    return psn_qmatvec_q8_multi(mod, s, qtype, layout, 1, &W, xq, &y, &N, K, batch);
}

extern "C" int32_t psn_qmatvec_multi(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, int32_t scheme, int32_t count,
                                     const psn_buf *const *W, const psn_buf *x, psn_buf *const *y, const int64_t *N, int64_t K,
                                     int32_t batch) {
    if (layout != PSN_LAYOUT_GGUF) return fail(PSN_E_UNSUPPORTED, "matvec: layout %d", layout);
    seg_list sg;
    int32_t rc = gather_segments("psn_qmatvec", mod, s, qtype, scheme, count, W, x, y, N, K, batch, &sg);
    if (rc) return rc;
    if ((rc = check_x_f32("psn_qmatvec", x, K, batch))) return rc;
    psn_matvec_plan plan;
    if ((rc = make_plan(qtype, scheme, sg.total, K, batch, mod->ctx->compute_units, true, sg.N, sg.count, &plan))) return rc;
    if ((rc = bind(mod->ctx))) return rc;
    if (scheme == PSN_ACT_F32) return run_matvec(mod, s, qtype, scheme, sg, x->p, K, batch, &plan);
    /* one launch when the staged copy fits LDS: every workgroup quantizes x while staging it */
    if (plan.stage_lds == 2) return run_matvec(mod, s, qtype, scheme, sg, x->p, K, batch, &plan);
    const int32_t at = psn_act_type_for(qtype);
    psn_actq_info li;
    if ((rc = psn_actq_layout(at, K, batch, &li))) return rc;
    if ((rc = ensure_workspace(s, li.bytes))) return rc;
    if ((rc = note_workspace_use(s))) return rc;    /* a graph being recorded bakes the workspace address into its nodes */
    if ((rc = quantize_into(mod, s, at, (const float *)x->p, s->ws->p, K, batch))) return rc;
    return run_matvec(mod, s, qtype, scheme, sg, s->ws->p, K, batch, &plan);
}

extern "C" int32_t psn_qmatvec(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, int32_t scheme, const psn_buf *W,
                               const psn_buf *x, psn_buf *y, int64_t N, int64_t K, int32_t batch) {
    return psn_qmatvec_multi(mod, s, qtype, layout, scheme, 1, &W, x, &y, &N, K, batch);
}

extern "C" int64_t psn_noalloc_max_bytes(void) { return (int64_t)PSN_NOALLOC_SCRATCH_BYTES; }

/* psn_qmatvec without any allocation: scheme Q8 quantizes x into the library's static device scratch
 * (one array per GPU, shared by every call on that GPU) and runs the pre-quantized kernel from there;
 * scheme F32 needs no scratch at all.  Only launches are issued, so the call is legal under capture. */
extern "C" int32_t psn_qmatvec_noalloc(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, int32_t scheme, const psn_buf *W,
                                       const psn_buf *x, psn_buf *y, int64_t N, int64_t K, int32_t batch) {
    if (layout != PSN_LAYOUT_GGUF) return fail(PSN_E_UNSUPPORTED, "matvec: layout %d", layout);
    seg_list sg;
    int32_t rc = gather_segments("psn_qmatvec_noalloc", mod, s, qtype, scheme, 1, &W, x, &y, &N, K, batch, &sg);
    if (rc) return rc;
    if ((rc = check_x_f32("psn_qmatvec_noalloc", x, K, batch))) return rc;
    psn_matvec_plan plan;
    if ((rc = make_plan(qtype, scheme, sg.total, K, batch, mod->ctx->compute_units, false, sg.N, sg.count, &plan))) return rc;
    if (scheme == PSN_ACT_F32) {
        if ((rc = bind(mod->ctx))) return rc;
        return run_matvec(mod, s, qtype, scheme, sg, x->p, K, batch, &plan);
    }
    const int32_t at = psn_act_type_for(qtype);
    psn_actq_info li;
    if ((rc = psn_actq_layout(at, K, batch, &li))) return rc;
    if (li.bytes > (int64_t)PSN_NOALLOC_SCRATCH_BYTES)
        return fail(PSN_E_SHAPE, "psn_qmatvec_noalloc: quantized activations of K=%lld x batch %d take %lld bytes, the static scratch holds %u "
                    "(use psn_qmatvec, which sizes a workspace)", (long long)K, batch, (long long)li.bytes, PSN_NOALLOC_SCRATCH_BYTES);
    void *scratch_ptr = nullptr;
    int herr = 0;
    if (psn_noalloc_scratch(mod->ctx->device, &scratch_ptr, nullptr, &herr) != 0)
        return fail(PSN_E_HIP, "psn_qmatvec_noalloc: static scratch of device %d is not available: hipError %d", mod->ctx->device, herr);
    if ((rc = bind(mod->ctx))) return rc;
    /* the quantize launch overwrites every byte the matvec reads (qs, scales, sums of batch x K), so
     * nothing left behind by an earlier, larger call can be seen: no clearing is needed */
    if ((rc = quantize_into(mod, s, at, (const float *)x->p, scratch_ptr, K, batch))) return rc;
    return run_matvec(mod, s, qtype, scheme, sg, scratch_ptr, K, batch, &plan);
}


/* ------------------------------------------------------------------ calibration */

extern "C" int32_t psn_calibrate_read(psn_module *mod, psn_stream *s, const psn_buf *src, int64_t bytes, int32_t blocks, int32_t threads,
                                      int32_t lds_depth, int32_t every_workgroup, psn_buf *out) {
    if (!mod || !s || !src) return fail(PSN_E_INVALID_ARG, "psn_calibrate_read: null handle");
    if (s->ctx != mod->ctx || src->ctx != mod->ctx || (out && out->ctx != mod->ctx)) return fail(PSN_E_INVALID_ARG, "psn_calibrate_read: handles belong to different contexts");
    if (bytes <= 0 || (int64_t)src->bytes < bytes) return fail(PSN_E_INVALID_ARG, "psn_calibrate_read: %lld bytes asked of a buffer of %zu", (long long)bytes, src->bytes);
    if (blocks < 1 || blocks > (1 << 20) || threads < 64 || threads > 1024 || threads % 64) return fail(PSN_E_SHAPE, "psn_calibrate_read: blocks=%d threads=%d", blocks, threads);
    if (lds_depth < 0 || lds_depth > 64) return fail(PSN_E_SHAPE, "psn_calibrate_read: lds_depth=%d outside 0..64", lds_depth);
    const int64_t waves = (int64_t)blocks * (threads / 64);
    if (out && (int64_t)out->bytes < waves * 4) return fail(PSN_E_INVALID_ARG, "psn_calibrate_read: out holds %zu bytes, need %lld", out->bytes, (long long)(waves * 4));
    const int64_t lds = (int64_t)lds_depth * 1024 * (threads / 64);
    if (lds > mod->ctx->max_lds) return fail(PSN_E_UNSUPPORTED, "psn_calibrate_read: %lld bytes of LDS asked, device offers %d", (long long)lds, mod->ctx->max_lds);
    int32_t rc = bind(mod->ctx);
    if (rc) return rc;
    psn_calib_args a;
    a.src = (const uint8_t *)src->p;
    a.out = out ? (uint32_t *)out->p : nullptr;
    a.bytes = bytes;
    a.depth = lds_depth;
    a.every_wg = every_workgroup != 0;
    return launch(mod, s, lds_depth ? "psn_calib_read_lds" : "psn_calib_read", (unsigned)blocks, (unsigned)threads, (unsigned)lds, &a);
}

extern "C" int32_t psn_selftest_arith(psn_module *mod, psn_stream *s, psn_buf *out) {
    if (!mod || !s || !out) return fail(PSN_E_INVALID_ARG, "psn_selftest_arith: null handle");
    if (s->ctx != mod->ctx || out->ctx != mod->ctx) return fail(PSN_E_INVALID_ARG, "psn_selftest_arith: handles belong to different contexts");
    if (out->bytes < PSN_SELFTEST_COUNTERS * sizeof(unsigned long long))
        return fail(PSN_E_INVALID_ARG, "psn_selftest_arith: out holds %zu bytes, need %zu", out->bytes, PSN_SELFTEST_COUNTERS * sizeof(unsigned long long));
    int32_t rc = bind(mod->ctx);
    if (rc) return rc;
    psn_fill_args f;
    f.p = (uint32_t *)out->p;
    f.n16 = PSN_SELFTEST_COUNTERS * sizeof(unsigned long long) / 16;
    if ((rc = launch(mod, s, "psn_fill_zero", 1, 256, 0, &f))) return rc;
    psn_selftest_args a;
    const float lo = 0x1p-100f, hi = 0x1p100f;
    memcpy(&a.lo, &lo, 4);
    memcpy(&a.hi, &hi, 4);
    a.bad = (unsigned long long *)out->p;
    return launch(mod, s, "psn_selftest_arith", 4096, 256, 0, &a);
}

/* ------------------------------------------------------------------ prefill */

static const int k_prefill_tiles[][2] = {{64, 64}, {64, 128}, {128, 128}, {128, 256}, {256, 128}, {256, 256}};

static int32_t check_prefill(const char *what, psn_module *mod, psn_stream *s, int32_t qtype, const psn_buf *W, const psn_buf *X,
                             psn_buf *Y, int64_t M, int64_t N, int64_t K) {
    int32_t rc = check_same_ctx(mod, s, W, X, Y, what);
    if (rc) return rc;
    if (!is_weight_type(qtype)) return fail(PSN_E_UNSUPPORTED, "%s: type %d (Q4_0, Q8_0, Q4_K, Q5_K and Q6_K have kernels)", what, qtype);
    if (M <= 0 || N <= 0 || M > (1 << 20) || N > (1 << 24)) return fail(PSN_E_SHAPE, "%s: M=%lld N=%lld out of range", what, (long long)M, (long long)N);
    const int64_t rb = psn_row_bytes(qtype, K);
    if (rb < 0) return (int32_t)rb;
    if (K % 256 || K > (1 << 24)) return fail(PSN_E_SHAPE, "%s: K=%lld must be a multiple of 256", what, (long long)K);
    /* several kernel families address X and W with 32-bit byte offsets */
    if (M * K * 2 > (int64_t)UINT32_MAX || N * rb > (int64_t)UINT32_MAX)
        return fail(PSN_E_SHAPE, "%s: X (%lld bytes) and W (%lld bytes) must each stay below 4 GiB", what, (long long)(M * K * 2), (long long)(N * rb));
    if ((int64_t)W->bytes < N * rb) return fail(PSN_E_INVALID_ARG, "%s: W holds %zu bytes, need %lld", what, W->bytes, (long long)(N * rb));
    if ((int64_t)X->bytes < M * K * 2) return fail(PSN_E_INVALID_ARG, "%s: X holds %zu bytes, need %lld", what, X->bytes, (long long)(M * K * 2));
    if ((int64_t)Y->bytes < M * N * 4) return fail(PSN_E_INVALID_ARG, "%s: Y holds %zu bytes, need %lld", what, Y->bytes, (long long)(M * N * 4));
    return PSN_OK;
}

/* per-tile cost model measured on MI355X: microseconds per 64-wide K step of one workgroup, and how
 * many workgroups of that tile one compute unit holds (LDS and registers) */
static const double k_prefill_step_us[] = {0.87, 1.10, 1.50, 2.00, 2.00, 2.44};
static const int k_prefill_wgs_per_cu[] = {3, 3, 2, 1, 1, 1};
/* the producer / consumer kernels (16 = four multiplying + four staging waves) and the wide kernel (32:
 * 256 x 256, four waves decoding their own operands from raw bytes):
 * {tile index, kernel family, step cost, workgroups per compute unit, K steps a workgroup spends filling its load rings} */
/* the K-quants' four-wave kernels per tile, one workgroup per compute unit (measured over three projection shapes,
 * M = 128 .. 1024, every K split; Q5_K takes Q4_K's figures), what each further workgroup on the same compute unit adds
 * (Q6_K's decode keeps the vector ALUs busy, so two resident workgroups take turns), and the 128 x 256 producer /
 * consumer kernel of Q4_K and Q5_K (one round of workgroups, several rounds) */
static const double k_q45_K_step_us[] = {0.76, 1.14, 1.33, 1.91, 1.71, 2.60};
static const double k_q6_K_step_us[] = {0.95, 1.33, 1.51, 2.43, 1.96, 3.10};
static const double k_kquant_ws_step_us[2] = {1.58, 3.4};
static const struct { int tile; int waves; double step_us; int per_cu; int fill; } k_prefill_alt[] = {{3, 16, 1.25, 1, 2}, {2, 16, 0.82, 1, 1}, {5, 32, 2.20, 1, 3}};

/* zero fill of Y and the atomic adds of `sp` partial sums per element, plus a launch: with few ranges the adds overlap
 * the multiply well enough to count at the fill's 3 TB/s; from `slow_from` ranges on (eight; four for the kernels
 * whose four waves hold a whole 256 x 256 tile) they run at the measured 1.6 TB/s */
static double ksplit_overhead_us(int64_t M, int64_t N, int sp, int slow_from = 8) {
    const double bytes = (double)(M * N) * 4.0;
    return (sp >= slow_from ? bytes * (1.0 / 3.0e6 + sp / 1.6e6) : bytes * (1.0 + sp) / 3.0e6) + 4.0;
}
/* The dense family's estimate: one pass that rewrites the matrix as fp16 (0.45 us per million weights + a
 * launch, measured; none when the caller holds packed weights) and the multiply on 256 x 256 or 128 x 256 tiles,
 * round by round of workgroups. */
static const double k_dense_step_us[2][3] = {{1.85, 1.5, 1.4}, {0.96, 0.78, 0.72}};   /* {256, 128 rows} x {full round, 60-80 % filled, emptier} */
static double dense_estimate(int64_t M, int64_t N, int64_t K, int32_t cus, bool with_unpack, int *bm_out, int *ksplit_out) {
    const int64_t nt = (N + 255) / 256;
    const double unpack = with_unpack ? 4.0 + (double)N * (double)K * 0.45e-6 : 0.0;
    double best = 1e300;
    for (int v = 0; v < 2; ++v) {
        const int bm = v ? 128 : 256;
        const int64_t mt = (M + bm - 1) / bm;
        for (int sp = 1; sp <= 4; sp *= 2) {
            if (sp > 1 && ((M * N) % 4 != 0 || K / 256 < 4 * sp)) continue;
            const int64_t wgs = mt * nt * sp, full = wgs / cus, rest = wgs % cus;
            const double steps = (double)(K / 64) / sp;
            /* a round that fills the chip runs at a lower clock than a partly filled one */
            const double fill = (double)rest / cus;
            double t = unpack + (double)full * steps * k_dense_step_us[v][0] +
                       (rest ? steps * k_dense_step_us[v][fill >= 0.8 ? 0 : fill >= 0.6 ? 1 : 2] : 0.0) + 5.0;
            /* four contributors per element of a 128-row tile all finish together: their adds cost more than two do */
            if (sp > 1) t += (v && sp == 4) ? (double)(M * N) * 4.0 * (1.0 / 3.0e6 + 4.0 / 2.0e6) + 4.0 : ksplit_overhead_us(M, N, sp, v ? 8 : 4);
            if (t < best) { best = t; *bm_out = bm; *ksplit_out = sp; }
        }
    }
    return best;
}

static int32_t plan_q4_0_q8_0(int64_t M, int64_t N, int64_t K, int32_t cus, int32_t *tile_m, int32_t *tile_n, int32_t *ksplit, int32_t *waves,
                              double *t_best);
extern "C" int32_t psn_qmatmul_prefill_plan(int64_t M, int64_t N, int64_t K, int32_t cus, int32_t *tile_m, int32_t *tile_n, int32_t *ksplit,
                                            int32_t *waves) {
    return psn_qmatmul_prefill_plan_for(PSN_Q4_0, M, N, K, cus, tile_m, tile_n, ksplit, waves);
}
/* at most 64 rows (every format; Q6_K when its rows are whole 16-byte words): the weight-streaming kernel on 64 x 64 tiles; K is cut (atomic adds) only
 * while the weight rows alone leave half of the compute units without a workgroup, down to two chunks per range */
static void plan_weight_stream(int64_t M, int64_t N, int64_t K, int32_t cus, int32_t *tile_m, int32_t *tile_n, int32_t *ksplit, int32_t *waves) {
    const int64_t nt = (N + 63) / 64, C = K / 256;
    int sp = 1;
    while (sp < 8 && nt * sp * 2 <= cus && C / (sp * 2) >= 2 && (M * N) % 4 == 0) sp *= 2;
    *tile_m = 64;
    *tile_n = 64;
    *ksplit = sp;
    *waves = 64;
}
static int32_t plan_q4_0_q8_0(int64_t M, int64_t N, int64_t K, int32_t cus, int32_t *tile_m, int32_t *tile_n, int32_t *ksplit, int32_t *waves,
                              double *t_best) {
    if (!tile_m || !tile_n || !ksplit || !waves) return fail(PSN_E_INVALID_ARG, "psn_qmatmul_prefill_plan: out is null");
    *waves = 4;
    *t_best = 0.0;
    if (M <= 0 || N <= 0 || K <= 0 || K % 256) return fail(PSN_E_SHAPE, "prefill: M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    if (cus <= 0) cus = 256;
    if (M <= 64) {
        plan_weight_stream(M, N, K, cus, tile_m, tile_n, ksplit, waves);
        return PSN_OK;
    }
    /* estimated time = waves of workgroups over the chip's slots x K steps per workgroup x step cost,
     * plus, when K is split, zeroing Y and the atomic adds of the partial sums */
    double best = 1e300;
    int bi = 0, bs = 1;
    for (int i = 0; i < 6; ++i) {
        const int bm = k_prefill_tiles[i][0], bn = k_prefill_tiles[i][1];
        const int64_t mt = (M + bm - 1) / bm, nt = (N + bn - 1) / bn;
        const int64_t slots = (int64_t)cus * k_prefill_wgs_per_cu[i];
        for (int sp = 1; sp <= 8; sp *= 2) {
            if (sp > 1 && ((M * N) % 4 != 0 || K / 256 < 2 * sp)) continue;
            const bool short_range = sp > 1 && K / 256 < 4 * sp;    /* two or three chunks per range: the producer / consumer kernels only */
            const int64_t wgs = mt * nt * sp;
            const int64_t rounds = (wgs + slots - 1) / slots;
            const double steps = (double)(K / 64) / sp;
            /* the step costs are those of one workgroup per compute unit; workgroups that share one slow each
             * other down (measured: 1.45 x with three of the small tiles resident) */
            const int64_t resident = ((wgs < slots ? wgs : slots) + cus - 1) / cus;
            double t = (double)rounds * steps * k_prefill_step_us[i] * (1.0 + 0.225 * (double)(resident - 1)) + 5.0;
            if (sp > 1) t += ksplit_overhead_us(M, N, sp, i == 5 ? 4 : 8);
            if (!short_range && t < best) { best = t; bi = i; bs = sp; *waves = 4; }
            for (const auto &v : k_prefill_alt) {
                if (v.tile != i || (short_range && v.waves != 16)) continue;
                const int64_t sl = (int64_t)cus * v.per_cu;
                const int64_t r8 = (wgs + sl - 1) / sl;
                double t8 = (double)r8 * (steps + v.fill) * v.step_us + 5.0;
                if (sp > 1) t8 += ksplit_overhead_us(M, N, sp, v.waves == 32 ? 4 : 8);
                if (t8 < best) { best = t8; bi = i; bs = sp; *waves = v.waves; }
            }
        }
    }
    *tile_m = k_prefill_tiles[bi][0];
    *tile_n = k_prefill_tiles[bi][1];
    *ksplit = bs;
    *t_best = best;
    return PSN_OK;
}

/* The K-quants (Q4_K, Q5_K, Q6_K) have the four-wave family (the same estimate over its six tiles with step costs of
 * their own: the dequantization is fp32 arithmetic per weight) and, Q4_K and
 * Q5_K, the 128 x 256 producer / consumer kernel (its staging waves decode while the others multiply). */
static double prefill_plan_kquant(int32_t qtype, int64_t M, int64_t N, int64_t K, int32_t cus, int32_t *tile_m, int32_t *tile_n, int32_t *ksplit,
                                int32_t *waves) {
    if (cus <= 0) cus = 256;
    const double *step_us = qtype == PSN_Q6_K ? k_q6_K_step_us : k_q45_K_step_us;
    const double shared = qtype == PSN_Q6_K ? 1.0 : 0.35;
    double best = 1e300;
    int bi = 0, bs = 1;
    *waves = 4;
    for (int i = 0; i < 6; ++i) {
        const int bm = k_prefill_tiles[i][0], bn = k_prefill_tiles[i][1];
        if (bm > 64 && M <= 64) continue;
        const int64_t mt = (M + bm - 1) / bm, nt = (N + bn - 1) / bn;
        const int64_t slots = (int64_t)cus * (k_prefill_wgs_per_cu[i] > 2 ? 2 : k_prefill_wgs_per_cu[i]);
        for (int sp = 1; sp <= 8; sp *= 2) {
            if (sp > 1 && ((M * N) % 4 != 0 || K / 256 < 4 * sp)) continue;
            const int64_t wgs = mt * nt * sp, rounds = (wgs + slots - 1) / slots;
            const int64_t resident = ((wgs < slots ? wgs : slots) + cus - 1) / cus;
            double t = (double)rounds * ((double)(K / 64) / sp) * step_us[i] * (1.0 + shared * (double)(resident - 1)) + 5.0;
            if (sp > 1) t += ksplit_overhead_us(M, N, sp, i == 5 ? 4 : 8);
            if (t < best) { best = t; bi = i; bs = sp; *waves = 4; }
            if (i == 3 && qtype != PSN_Q6_K && M > 64) {
                const int64_t r16 = (wgs + cus - 1) / cus;
                double t16 = (double)r16 * ((double)(K / 64) / sp + 2.0) * (r16 > 1 ? k_kquant_ws_step_us[1] : k_kquant_ws_step_us[0]) + 5.0;
                if (sp > 1) t16 += ksplit_overhead_us(M, N, sp);
                if (t16 < best) { best = t16; bi = i; bs = sp; *waves = 16; }
            }
        }
    }
    *tile_m = k_prefill_tiles[bi][0];
    *tile_n = k_prefill_tiles[bi][1];
    *ksplit = bs;
    return best;
}

/* the plan for any format; with allow_dense the dense family (needs the stream's workspace) competes */
static int32_t prefill_plan_any(int32_t qtype, int64_t M, int64_t N, int64_t K, int32_t cus, bool allow_dense, int32_t *tile_m, int32_t *tile_n,
                                int32_t *ksplit, int32_t *waves) {
    if (!is_weight_type(qtype)) return fail(PSN_E_UNSUPPORTED, "prefill: type %d", qtype);
    if (!tile_m || !tile_n || !ksplit || !waves) return fail(PSN_E_INVALID_ARG, "psn_qmatmul_prefill_plan: null output");
    if (M <= 0 || N <= 0 || K <= 0 || K % 256) return fail(PSN_E_SHAPE, "prefill plan: M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    if (cus <= 0) cus = 256;
    double best = 0.0;
    if (qtype == PSN_Q4_0 || qtype == PSN_Q8_0) {
        int32_t rc = plan_q4_0_q8_0(M, N, K, cus, tile_m, tile_n, ksplit, waves, &best);
        if (rc) return rc;
        if (M <= 64) return PSN_OK;                              /* the weight-streaming kernel */
        if (qtype == PSN_Q8_0) best *= 1.15;                     /* the step costs above were measured on Q4_0; Q8_0 stages twice the bytes */
    } else if (M <= 64 && (qtype != PSN_Q6_K || K % 2048 == 0)) {
        plan_weight_stream(M, N, K, cus, tile_m, tile_n, ksplit, waves);
        return PSN_OK;
    } else {
        best = prefill_plan_kquant(qtype, M, N, K, cus, tile_m, tile_n, ksplit, waves);
    }
    if (allow_dense && M > 64) {
        int sp = 1, bm = 256;
        /* two more launches and a workspace: only for a clear gain -- except for the K-quants on matrices of 16 M
         * weights and more, whose in-loop kernels the estimates flatter (their fp32 decode competes with the MFMAs
         * for issue slots): there the dense family wins ties */
        const double margin = (qtype == PSN_Q4_0 || qtype == PSN_Q8_0 || N * K < ((int64_t)1 << 24)) ? 0.95 : 1.05;
        if (dense_estimate(M, N, K, cus, true, &bm, &sp) < margin * best) {
            *tile_m = bm;
            *tile_n = 256;
            *ksplit = sp;
            *waves = 128;
        }
    }
    return PSN_OK;
}

extern "C" int32_t psn_qmatmul_prefill_plan_for(int32_t qtype, int64_t M, int64_t N, int64_t K, int32_t cus, int32_t *tile_m, int32_t *tile_n,
                                                int32_t *ksplit, int32_t *waves) {
    return prefill_plan_any(qtype, M, N, K, cus, true, tile_m, tile_n, ksplit, waves);
}

static int32_t need(const psn_buf *b, int64_t bytes, const char *what, const char *name);
/* the dense family's two steps: GGUF blocks -> fp16 MFMA fragments ([ceil(N/32)][K/16][64 lanes][8 halves], rows
 * padded to whole 256-row panels), and the fp16 multiply on 256 x 256 tiles over such a buffer */
static int64_t packed_bytes(int64_t N, int64_t K) { return (N + 255) / 256 * 256 * K * 2; }
static int32_t launch_unpack(psn_module *mod, psn_stream *s, int32_t qtype, const void *W, void *out, int64_t N, int64_t K) {
    psn_unpack_args u;
    memset(&u, 0, sizeof u);
    u.W = (const uint8_t *)W;
    u.out = (uint16_t *)out;
    u.N = (int32_t)N;
    u.K = (int32_t)K;
    u.row_bytes = psn_row_bytes(qtype, K);
    char name[96];
    snprintf(name, sizeof name, "psn_prefill_%s_unpack", fmt_name(qtype));
    return launch(mod, s, name, (unsigned)((N + 255) / 256 * (K / 256)), 256, 0, &u);
}
static int32_t launch_dense(psn_module *mod, psn_stream *s, const void *packed, const psn_buf *X, psn_buf *Y, int64_t M, int64_t N, int64_t K,
                            int32_t bm, int32_t ksplit) {
    int32_t rc;
    if (ksplit > 1) {
        psn_fill_args f;
        f.p = (uint32_t *)Y->p;
        f.n16 = M * N / 4;
        const int64_t fb = (f.n16 + 255) / 256;
        if ((rc = launch(mod, s, "psn_fill_zero", (unsigned)(fb > 2048 ? 2048 : fb), 256, 0, &f))) return rc;
    }
    const int64_t nt = (N + 255) / 256, mt = (M + bm - 1) / bm;
    psn_prefill_args a;
    memset(&a, 0, sizeof a);
    a.W = (const uint8_t *)packed;
    a.X = (const uint16_t *)X->p;
    a.Y = (float *)Y->p;
    a.M = (int32_t)M;
    a.N = (int32_t)N;
    a.K = (int32_t)K;
    a.ksplit = ksplit;
    a.row_bytes = K * 2;
    /* LDS: a ring of four stages of X, bm rows x 32 k fp16 each */
    return launch(mod, s, bm == 128 ? "psn_prefill_dense_f16_m128" : "psn_prefill_dense_f16", (unsigned)(8 * ((nt + 7) / 8) * mt * ksplit), 256, 4 * bm * 64, &a);
}

extern "C" int64_t psn_prefill_packed_bytes(int64_t N, int64_t K) {
    if (N <= 0 || K <= 0 || K % 256 || N > (1 << 30) || K > (1 << 24)) return fail(PSN_E_SHAPE, "psn_prefill_packed_bytes: N=%lld K=%lld", (long long)N, (long long)K);
    return packed_bytes(N, K);
}
extern "C" int32_t psn_prefill_pack(psn_module *mod, psn_stream *s, int32_t qtype, const psn_buf *W, psn_buf *packed, int64_t N, int64_t K) {
    if (!mod || !s || !W || !packed) return fail(PSN_E_INVALID_ARG, "psn_prefill_pack: null handle");
    if (s->ctx != mod->ctx || W->ctx != mod->ctx || packed->ctx != mod->ctx) return fail(PSN_E_INVALID_ARG, "psn_prefill_pack: handles belong to different contexts");
    if (!is_weight_type(qtype)) return fail(PSN_E_UNSUPPORTED, "psn_prefill_pack: type %d", qtype);
    if (N <= 0 || N > (1 << 30) || K <= 0 || K % 256 || K > (1 << 24)) return fail(PSN_E_SHAPE, "psn_prefill_pack: N=%lld K=%lld (K must be a multiple of 256)", (long long)N, (long long)K);
    int32_t rc;
    if ((rc = need(W, N * psn_row_bytes(qtype, K), "psn_prefill_pack", "W")) || (rc = need(packed, packed_bytes(N, K), "psn_prefill_pack", "packed"))) return rc;
    if ((rc = bind(mod->ctx))) return rc;
    return launch_unpack(mod, s, qtype, W->p, packed->p, N, K);
}
extern "C" int32_t psn_qmatmul_prefill_packed(psn_module *mod, psn_stream *s, const psn_buf *packed, const psn_buf *X, psn_buf *Y, int64_t M,
                                              int64_t N, int64_t K) {
    if (!mod || !s || !packed || !X || !Y) return fail(PSN_E_INVALID_ARG, "psn_qmatmul_prefill_packed: null handle");
    if (s->ctx != mod->ctx || packed->ctx != mod->ctx || X->ctx != mod->ctx || Y->ctx != mod->ctx)
        return fail(PSN_E_INVALID_ARG, "psn_qmatmul_prefill_packed: handles belong to different contexts");
    if (M <= 0 || M > (1 << 24) || N <= 0 || N > (1 << 30) || K <= 0 || K % 256 || K > (1 << 24))
        return fail(PSN_E_SHAPE, "psn_qmatmul_prefill_packed: M=%lld N=%lld K=%lld (K must be a multiple of 256)", (long long)M, (long long)N, (long long)K);
    if (M * K * 2 > (int64_t)UINT32_MAX) return fail(PSN_E_SHAPE, "psn_qmatmul_prefill_packed: X (%lld bytes) must stay below 4 GiB", (long long)(M * K * 2));
    int32_t rc;
    if ((rc = need(packed, packed_bytes(N, K), "psn_qmatmul_prefill_packed", "packed")) || (rc = need(X, M * K * 2, "psn_qmatmul_prefill_packed", "X")) ||
        (rc = need(Y, M * N * 4, "psn_qmatmul_prefill_packed", "Y")))
        return rc;
    if ((rc = bind(mod->ctx))) return rc;
    int sp = 1, bm = 256;
    (void)dense_estimate(M, N, K, mod->ctx->compute_units, false, &bm, &sp);
    return launch_dense(mod, s, packed->p, X, Y, M, N, K, bm, sp);
}

extern "C" int32_t psn_prefill_reserve(psn_stream *s, int64_t N, int64_t K) {
    if (!s) return fail(PSN_E_INVALID_ARG, "stream is null");
    if (N <= 0 || K <= 0 || K % 256 || N > (1 << 30) || K > (1 << 24)) return fail(PSN_E_SHAPE, "psn_prefill_reserve: N=%lld K=%lld", (long long)N, (long long)K);
    int32_t rc = bind(s->ctx);
    if (rc) return rc;
    return ensure_workspace(s, packed_bytes(N, K));
}

extern "C" int32_t psn_qmatmul_prefill_tiled(psn_module *mod, psn_stream *s, int32_t qtype, const psn_buf *W, const psn_buf *X,
                                             psn_buf *Y, int64_t M, int64_t N, int64_t K, int32_t bm, int32_t bn, int32_t ksplit,
                                             int32_t waves) {
    int32_t rc = check_prefill("psn_qmatmul_prefill", mod, s, qtype, W, X, Y, M, N, K);
    if (rc) return rc;
    /* waves == 128 selects the dense family (any format): the whole matrix is dequantized to fp16 fragments in
     * the stream's workspace (psn_prefill_<fmt>_unpack), then psn_prefill_dense_f16(_m128) multiplies 256 x 256 or
     * 128 x 256 tiles */
    if (waves == 128) {
        if ((bm != 256 && bm != 128) || bn != 256) return fail(PSN_E_UNSUPPORTED, "prefill: the dense kernels have 256x256 and 128x256 tiles");
        if (ksplit < 1 || ksplit > 64) return fail(PSN_E_UNSUPPORTED, "prefill: ksplit=%d outside 1..64", ksplit);
        if (ksplit > 1 && (M * N) % 4 != 0) return fail(PSN_E_UNSUPPORTED, "prefill: splitting K needs M*N to be a multiple of 4");
        if ((rc = bind(mod->ctx))) return rc;
        if ((rc = ensure_workspace(s, packed_bytes(N, K)))) return rc;
        if ((rc = note_workspace_use(s))) return rc;
        if ((rc = launch_unpack(mod, s, qtype, W->p, s->ws->p, N, K))) return rc;
        return launch_dense(mod, s, s->ws->p, X, Y, M, N, K, bm, ksplit);
    }
    if (qtype != PSN_Q4_0 && qtype != PSN_Q8_0 && waves != 4 && waves != 64 && !(waves == 16 && bm == 128 && bn == 256 && qtype != PSN_Q6_K))
        return fail(PSN_E_UNSUPPORTED, "prefill: %s has the four-wave kernel family, the weight-streaming kernel for M <= 64 (waves = 64)%s", fmt_name(qtype),
                    qtype == PSN_Q6_K ? "" : " and the 128x256 producer / consumer kernel (waves = 16)");
    /* waves == 64 selects the skinny kernel (M <= 64, 64 x 64 tiles, deep LDS rings) */
    const bool skinny = waves == 64;
    if (skinny && (bm != 64 || bn != 64 || M > 64)) return fail(PSN_E_UNSUPPORTED, "prefill: the skinny kernel serves M <= 64 with a 64x64 tile");
    /* Q6_K super-blocks (210 bytes) are fetched as windows of aligned 16-byte words: the rows must start on one */
    if (skinny && qtype == PSN_Q6_K && K % 2048) return fail(PSN_E_UNSUPPORTED, "prefill: the skinny Q6_K kernel needs K to be a multiple of 2048 (K=%lld)", (long long)K);
    /* waves == 32 selects the wide kernel: 256 x 256 tiles, four waves with 128 x 128 each, weights decoded
     * from raw bytes in LDS by the wave that multiplies them */
    const bool wide = waves == 32;
    if (wide && (bm != 256 || bn != 256)) return fail(PSN_E_UNSUPPORTED, "prefill: the wide kernel has a 256x256 tile");
    bool known = false;
    for (int i = 0; i < 6; ++i) known = known || (k_prefill_tiles[i][0] == bm && k_prefill_tiles[i][1] == bn);
    if (!known) return fail(PSN_E_UNSUPPORTED, "prefill: no kernel with a %dx%d tile", bm, bn);
    /* 16: eight waves split into four multiplying and four staging ones */
    const bool has_ws = (bm == 64 && (bn == 64 || bn == 128)) || (bm == 128 && (bn == 128 || bn == 256));
    if (!skinny && !wide && waves != 4 && !(waves == 16 && has_ws)) return fail(PSN_E_UNSUPPORTED, "prefill: no kernel family %d for a %dx%d tile", waves, bm, bn);
    if (ksplit < 1 || ksplit > 64) return fail(PSN_E_UNSUPPORTED, "prefill: ksplit=%d outside 1..64", ksplit);
    if (ksplit > 1 && (M * N) % 4 != 0) return fail(PSN_E_UNSUPPORTED, "prefill: splitting K needs M*N to be a multiple of 4");
    /* the interleaved kernels carry their LDS as static arrays; the skinny kernel: rings of three X chunks
     * (64 rows x 256 k fp16) and six (Q4_0, Q4_K), five (Q5_K), four (Q6_K) or three (Q8_0) raw weight chunks (64 rows, padded: SkinnyRings), reused for the final
     * 8 x 16 KB reduction */
    const int skinny_rings = 3 * 32768 + (qtype == PSN_Q4_0 || qtype == PSN_Q4_K ? 6 * 64 * 144 : qtype == PSN_Q5_K ? 5 * 64 * 176 : qtype == PSN_Q6_K ? 4 * 64 * 240 : 3 * 64 * 304);
    const int wide_rings = 3 * (32768 + 256 * (qtype == PSN_Q4_0 ? 36 : 68));   /* three stages of X (256 rows x 64 k) and of raw blocks (two per row) */
    const int lds = skinny ? (skinny_rings > 8 * 16384 ? skinny_rings : 8 * 16384) : wide ? wide_rings : waves == 16 ? 0 : 2 * (bm + bn) * 128;
    if (lds > mod->ctx->max_lds) return fail(PSN_E_UNSUPPORTED, "prefill: tile %dx%d needs %d bytes of LDS, device offers %d", bm, bn, lds, mod->ctx->max_lds);
    if ((rc = bind(mod->ctx))) return rc;
    if (ksplit > 1) {
        psn_fill_args f;
        f.p = (uint32_t *)Y->p;
        f.n16 = M * N / 4;
        const int64_t fb = (f.n16 + 255) / 256;
        if ((rc = launch(mod, s, "psn_fill_zero", (unsigned)(fb > 2048 ? 2048 : fb), 256, 0, &f))) return rc;
    }
    psn_prefill_args a;
    memset(&a, 0, sizeof a);
    a.W = (const uint8_t *)W->p;
    a.X = (const uint16_t *)X->p;
    a.Y = (float *)Y->p;
    a.M = (int32_t)M;
    a.N = (int32_t)N;
    a.K = (int32_t)K;
    a.ksplit = ksplit;
    a.row_bytes = psn_row_bytes(qtype, K);
    const int64_t mt = (M + bm - 1) / bm, nt = (N + bn - 1) / bn;
    char name[96];
    if (skinny) {
        snprintf(name, sizeof name, "psn_prefill_%s_skinny", fmt_name(qtype));
        return launch(mod, s, name, (unsigned)(nt * ksplit), 512, (unsigned)lds, &a);
    }
    const int64_t blocks = 8 * ((nt + 7) / 8) * mt * ksplit;      /* the kernel spreads N tiles over 8 XCDs */
    if (wide) {
        snprintf(name, sizeof name, "psn_prefill_%s_wide", fmt_name(qtype));
        return launch(mod, s, name, (unsigned)blocks, 256, (unsigned)lds, &a);
    }
    snprintf(name, sizeof name, "psn_prefill_%s_m%d_n%d%s", fmt_name(qtype), bm, bn, waves == 16 ? "_ws" : "");
    return launch(mod, s, name, (unsigned)blocks, (unsigned)(64 * (waves == 16 ? 8 : 4)), (unsigned)lds, &a);
}

extern "C" int32_t psn_qmatmul_prefill(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, const psn_buf *W,
                                       const psn_buf *X, psn_buf *Y, int64_t M, int64_t N, int64_t K) {
    if (layout != PSN_LAYOUT_GGUF) return fail(PSN_E_UNSUPPORTED, "prefill: layout %d", layout);
    int32_t rc = check_prefill("psn_qmatmul_prefill", mod, s, qtype, W, X, Y, M, N, K);
    if (rc) return rc;
    int32_t bm = 0, bn = 0, sp = 1, wv = 4;
    /* the dense family needs nt * 256 * K fp16 values of workspace on this stream: it competes when that is
     * there already or may still be allocated (not while capturing, not once a graph holds the workspace) */
    bool cap = false;
    if ((rc = is_capturing(s, &cap))) return rc;
    const int64_t dense_ws = packed_bytes(N, K);
    bool ws_pinned;
    {
        std::lock_guard<std::mutex> lk(g_cap_mu);
        ws_pinned = s->ws->graph_refs > 0 || s->ws->capture_refs > 0;
    }
    const bool dense_ok = s->ws->bytes >= (size_t)dense_ws || (!cap && !ws_pinned);
    if ((rc = prefill_plan_any(qtype, M, N, K, mod->ctx->compute_units, dense_ok, &bm, &bn, &sp, &wv))) return rc;
    return psn_qmatmul_prefill_tiled(mod, s, qtype, W, X, Y, M, N, K, bm, bn, sp, wv);
}

/* ------------------------------------------------------------------ decode-step glue */

static int32_t need(const psn_buf *b, int64_t bytes, const char *what, const char *name) {
    if (!b) return fail(PSN_E_INVALID_ARG, "%s: %s is null", what, name);
    if ((int64_t)b->bytes < bytes) return fail(PSN_E_INVALID_ARG, "%s: %s holds %zu bytes, need %lld", what, name, b->bytes, (long long)bytes);
    return PSN_OK;
}

/* fills the optional quantized-output descriptor of an elementwise kernel (yq null: not wanted) */
static int32_t set_actq_out(const char *what, psn_module *mod, psn_buf *yq, int32_t act_type, int64_t n, psn_actq_out *q) {
    memset(q, 0, sizeof *q);
    if (!yq) return PSN_OK;
    if (yq->ctx != mod->ctx) return fail(PSN_E_INVALID_ARG, "%s: handles belong to different contexts", what);
    if (n % 256) return fail(PSN_E_SHAPE, "%s: a quantized output needs n to be a multiple of 256 (n=%lld)", what, (long long)n);
    psn_actq_info li;
    int32_t rc = psn_actq_layout(act_type, n, 1, &li);
    if (rc) return rc;
    if ((int64_t)yq->bytes < li.bytes) return fail(PSN_E_INVALID_ARG, "%s: quantized output holds %zu bytes, need %lld", what, yq->bytes, (long long)li.bytes);
    q->qs = (int8_t *)yq->p + li.off_qs;
    q->d = (float *)((char *)yq->p + li.off_d);
    q->s = (char *)yq->p + li.off_s;
    q->act_q8_K = act_type == PSN_Q8_K;
    return PSN_OK;
}

static int32_t launch_add_rmsnorm(psn_module *mod, psn_stream *s, float *x, const float *delta, const float *weight, float *y, float *x_out,
                                  const psn_actq_out &qout, int64_t n, float eps, bool keep_x = false) {
    psn_norm_args a;
    memset(&a, 0, sizeof a);
    a.keep_x = keep_x ? 1 : 0;
    a.x = x;
    a.delta = delta;
    a.weight = weight;
    a.y = y;
    a.n = (int32_t)n;
    a.eps = eps;
    a.qout = qout;
    a.x_out = x_out;
    const unsigned threads = n >= 4096 ? 1024 : n >= 1024 ? 256 : 64;
    return launch(mod, s, "psn_add_rmsnorm", 1, threads, 0, &a);
}

extern "C" int32_t psn_add_rmsnorm_q8(psn_module *mod, psn_stream *s, psn_buf *x, const psn_buf *delta, const psn_buf *weight, psn_buf *y,
                                      psn_buf *yq, int32_t act_type, int64_t n, float eps) {
    int32_t rc = check_same_ctx(mod, s, x, weight, x, "psn_add_rmsnorm");
    if (rc) return rc;
    if (!y && !yq) return fail(PSN_E_INVALID_ARG, "psn_add_rmsnorm: no output");
    if (n <= 0 || n % 4 || n > (1 << 24)) return fail(PSN_E_SHAPE, "psn_add_rmsnorm: n=%lld must be a positive multiple of 4", (long long)n);
    if ((rc = need(x, n * 4, "psn_add_rmsnorm", "x")) || (rc = need(weight, n * 4, "psn_add_rmsnorm", "weight")) ||
        (y && (rc = need(y, n * 4, "psn_add_rmsnorm", "y"))) || (delta && (rc = need(delta, n * 4, "psn_add_rmsnorm", "delta"))))
        return rc;
    psn_actq_out qo;
    if ((rc = set_actq_out("psn_add_rmsnorm", mod, yq, act_type, n, &qo))) return rc;
    if ((rc = bind(mod->ctx))) return rc;
    return launch_add_rmsnorm(mod, s, (float *)x->p, delta ? (const float *)delta->p : nullptr, (const float *)weight->p,
                              y ? (float *)y->p : nullptr, nullptr, qo, n, eps);
}
extern "C" int32_t psn_add_rmsnorm(psn_module *mod, psn_stream *s, psn_buf *x, const psn_buf *delta, const psn_buf *weight, psn_buf *y,
                                   int64_t n, float eps) {
    if (!y) return fail(PSN_E_INVALID_ARG, "psn_add_rmsnorm: y is null");
    return psn_add_rmsnorm_q8(mod, s, x, delta, weight, y, nullptr, PSN_Q8_K, n, eps);
}

/* y_i = W_i . q8(rmsnorm(x + delta) * weight), batch 1, scheme Q8: the residual add, the RMSNorm and the
 * activation quantization happen while every workgroup stages the fp32 vector (one launch); shapes the
 * norm-fused kernels do not serve take the norm kernel plus the pre-quantized matvec (two launches). */
extern "C" int32_t psn_qmatvec_norm_multi(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, int32_t count,
                                          const psn_buf *const *W, const psn_buf *x, const psn_buf *delta, const psn_buf *norm_weight,
                                          psn_buf *h_out, psn_buf *const *y, const int64_t *N, int64_t K, float eps) {
    const char *what = "psn_qmatvec_norm_multi";
    if (layout != PSN_LAYOUT_GGUF) return fail(PSN_E_UNSUPPORTED, "matvec: layout %d", layout);
    if (!norm_weight) return fail(PSN_E_INVALID_ARG, "%s: norm_weight is null", what);
    seg_list sg;
    int32_t rc = gather_segments(what, mod, s, qtype, PSN_ACT_Q8, count, W, x, y, N, K, 1, &sg);
    if (rc) return rc;
    if ((rc = check_x_f32(what, x, K, 1)) || (rc = need(norm_weight, K * 4, what, "norm_weight")) ||
        (delta && (rc = need(delta, K * 4, what, "delta"))) || (h_out && (rc = need(h_out, K * 4, what, "h_out"))))
        return rc;
    if (norm_weight->ctx != mod->ctx || (delta && delta->ctx != mod->ctx) || (h_out && h_out->ctx != mod->ctx))
        return fail(PSN_E_INVALID_ARG, "%s: handles belong to different contexts", what);
    if (h_out && (h_out->p == x->p || (delta && h_out->p == delta->p)))
        return fail(PSN_E_INVALID_ARG, "%s: h_out must not alias x or delta (every workgroup reads them while one writes h_out)", what);
    psn_matvec_plan plan;
    if ((rc = make_plan(qtype, PSN_ACT_Q8, sg.total, K, 1, mod->ctx->compute_units, true, sg.N, sg.count, &plan))) return rc;
    if ((rc = bind(mod->ctx))) return rc;
    norm_fusion nf = {delta ? (const float *)delta->p : nullptr, (const float *)norm_weight->p, h_out ? (float *)h_out->p : nullptr, eps, false};
    if (plan.stream && plan.stage_lds == 2) {
        psn_matvec_plan q = plan;
        q.stage_lds = 3;
        int64_t lds = 0;
        if (K > 4096 && q.threads < 512) q.threads = 512;        /* x, delta and the weights: four 16-byte registers each per thread */
        if (stream_plan_check(qtype, PSN_ACT_Q8, K, 1, &q, sg.N, sg.count, mod->ctx->max_lds, &lds) == PSN_OK) {
            if (q.threads != plan.threads) {
                const int64_t rows = 64 / q.lanes_per_row, npass = sg.total / rows, wpb = q.threads / 64;
                int64_t resident = (160 * 1024) / lds;
                resident = resident > 3 ? 3 : resident < 1 ? 1 : resident;
                int64_t b = (npass + wpb - 1) / wpb;
                q.blocks = (int32_t)(b > resident * mod->ctx->compute_units ? resident * mod->ctx->compute_units : b);
            }
            return run_matvec(mod, s, qtype, PSN_ACT_Q8, sg, x->p, K, 1, &q, &nf);
        }
        g_err[0] = 0;
    }
    /* two launches: norm (+ quantize) into the stream's workspace, then the pre-quantized matvec */
    const int32_t at = psn_act_type_for(qtype);
    psn_actq_info li;
    if ((rc = psn_actq_layout(at, K, 1, &li))) return rc;
    if ((rc = ensure_workspace(s, li.bytes))) return rc;
    if ((rc = note_workspace_use(s))) return rc;
    char *ws = (char *)s->ws->p;
    psn_actq_out qo;
    qo.qs = (int8_t *)ws + li.off_qs;
    qo.d = (float *)(ws + li.off_d);
    qo.s = ws + li.off_s;
    qo.act_q8_K = at == PSN_Q8_K;
    qo.pad = 0;
    /* like the fused launch, this path never writes x: the sum goes to h_out or nowhere */
    if ((rc = launch_add_rmsnorm(mod, s, (float *)x->p, nf.delta, nf.weight, nullptr, nf.h_out, qo, K, eps, /*keep_x=*/true))) return rc;
    if ((rc = make_plan(qtype, PSN_ACT_Q8, sg.total, K, 1, mod->ctx->compute_units, false, sg.N, sg.count, &plan))) return rc;
    return run_matvec(mod, s, qtype, PSN_ACT_Q8, sg, ws, K, 1, &plan);
}

/* the plan of the SwiGLU-fused gate | up launch, or an error where no fused kernel serves the shape */
static int32_t norm_swiglu_plan(int32_t qtype, int64_t N, int64_t K, int32_t cus, int max_lds, psn_matvec_plan *out) {
    if (N <= 0 || K <= 0 || K % 256) return fail(PSN_E_SHAPE, "psn_qmatvec_norm_swiglu: N=%lld K=%lld", (long long)N, (long long)K);
    const int64_t rows[2] = {N, N};
    psn_matvec_plan plan;
    int32_t rc = make_plan(qtype, PSN_ACT_Q8, 2 * N, K, 1, cus, true, rows, 2, &plan);
    if (rc) return rc;
    if (!plan.stream || plan.stage_lds != 2 || plan.lanes_per_row > 32)
        return fail(PSN_E_UNSUPPORTED, "psn_qmatvec_norm_swiglu: no fused kernel for N=%lld K=%lld of this format (rows of at most 8192, whole passes)",
                    (long long)N, (long long)K);
    plan.stage_lds = 3;
    if (K > 4096 && plan.threads < 512) {
        plan.threads = 512;
        plan.blocks = (plan.blocks + 1) / 2;
    }
    int64_t lds = 0;
    if ((rc = stream_plan_check(qtype, PSN_ACT_Q8, K, 1, &plan, rows, 2, max_lds, &lds))) return rc;
    *out = plan;
    return PSN_OK;
}

extern "C" int32_t psn_qmatvec_norm_swiglu_check(int32_t qtype, int64_t N, int64_t K, int32_t cus) {
    psn_matvec_plan plan;
    return norm_swiglu_plan(qtype, N, K, cus > 0 ? cus : 256, 160 * 1024, &plan);
}

extern "C" int32_t psn_qmatvec_norm_swiglu(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, const psn_buf *W_gate,
                                           const psn_buf *W_up, const psn_buf *x, const psn_buf *delta, const psn_buf *norm_weight,
                                           psn_buf *h_out, psn_buf *act_f32, int64_t N, int64_t K, float eps) {
    const char *what = "psn_qmatvec_norm_swiglu";
    if (layout != PSN_LAYOUT_GGUF) return fail(PSN_E_UNSUPPORTED, "matvec: layout %d", layout);
    if (!norm_weight || !W_gate || !W_up || !act_f32) return fail(PSN_E_INVALID_ARG, "%s: null handle", what);
    const psn_buf *W[2] = {W_gate, W_up};
    psn_buf *y[2] = {act_f32, act_f32};
    const int64_t rows[2] = {N, N};
    seg_list sg;
    int32_t rc = gather_segments(what, mod, s, qtype, PSN_ACT_Q8, 2, W, x, y, rows, K, 1, &sg);
    if (rc) return rc;
    if ((rc = check_x_f32(what, x, K, 1)) || (rc = need(norm_weight, K * 4, what, "norm_weight")) ||
        (delta && (rc = need(delta, K * 4, what, "delta"))) || (h_out && (rc = need(h_out, K * 4, what, "h_out"))))
        return rc;
    if (norm_weight->ctx != mod->ctx || (delta && delta->ctx != mod->ctx) || (h_out && h_out->ctx != mod->ctx))
        return fail(PSN_E_INVALID_ARG, "%s: handles belong to different contexts", what);
    if (h_out && (h_out->p == x->p || (delta && h_out->p == delta->p)))
        return fail(PSN_E_INVALID_ARG, "%s: h_out must not alias x or delta (every workgroup reads them while one writes h_out)", what);
    psn_matvec_plan plan;
    if ((rc = norm_swiglu_plan(qtype, N, K, mod->ctx->compute_units, mod->ctx->max_lds, &plan))) return rc;
    if ((rc = bind(mod->ctx))) return rc;
    norm_fusion nf = {delta ? (const float *)delta->p : nullptr, (const float *)norm_weight->p, h_out ? (float *)h_out->p : nullptr, eps, true};
    return run_matvec(mod, s, qtype, PSN_ACT_Q8, sg, x->p, K, 1, &plan, &nf);
}

extern "C" int32_t psn_rope_kv_store(psn_module *mod, psn_stream *s, psn_buf *q, psn_buf *k, const psn_buf *v, psn_buf *k_cache,
                                     psn_buf *v_cache, int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, int32_t pos, float theta_base) {
    int32_t rc = check_same_ctx(mod, s, q, k, v, "psn_rope_kv_store");
    if (rc) return rc;
    if (n_heads <= 0 || n_kv_heads <= 0 || head_dim <= 0 || head_dim % 2 || pos < 0) return fail(PSN_E_SHAPE, "psn_rope_kv_store: bad head geometry or position");
    const int64_t row = (int64_t)n_kv_heads * head_dim * 2;
    if ((rc = need(q, (int64_t)n_heads * head_dim * 4, "psn_rope_kv_store", "q")) || (rc = need(k, row * 2, "psn_rope_kv_store", "k")) ||
        (rc = need(v, row * 2, "psn_rope_kv_store", "v")) || (rc = need(k_cache, (pos + 1) * row, "psn_rope_kv_store", "k_cache")) ||
        (rc = need(v_cache, (pos + 1) * row, "psn_rope_kv_store", "v_cache")))
        return rc;
    if ((rc = bind(mod->ctx))) return rc;
    psn_rope_args a;
    memset(&a, 0, sizeof a);
    a.q = (float *)q->p;
    a.k = (float *)k->p;
    a.v = (const float *)v->p;
    a.k_cache = k_cache->p;
    a.v_cache = v_cache->p;
    a.n_heads = n_heads;
    a.n_kv_heads = n_kv_heads;
    a.head_dim = head_dim;
    a.pos = pos;
    a.theta_base = theta_base;
    const int pairs = (n_heads + n_kv_heads) * head_dim / 2;
    return launch(mod, s, "psn_rope_kv_store", (unsigned)((pairs + 255) / 256), 256, 0, &a);
}

struct rope_fusion {
    const psn_buf *k_new, *v_new, *table;
};
extern "C" int32_t psn_rope_table(psn_module *mod, psn_stream *s, psn_buf *table, int32_t head_dim, int32_t pos, float theta_base) {
    if (!mod || !s || !table) return fail(PSN_E_INVALID_ARG, "psn_rope_table: null handle");
    if (s->ctx != mod->ctx || table->ctx != mod->ctx) return fail(PSN_E_INVALID_ARG, "psn_rope_table: handles belong to different contexts");
    if (head_dim <= 0 || head_dim % 2 || pos < 0) return fail(PSN_E_SHAPE, "psn_rope_table: head_dim=%d pos=%d", head_dim, pos);
    int32_t rc = need(table, (int64_t)head_dim * 4, "psn_rope_table", "table");
    if (rc) return rc;
    if ((rc = bind(mod->ctx))) return rc;
    psn_rope_table_args a;
    a.table = (float *)table->p;
    a.head_dim = head_dim;
    a.pos = pos;
    a.theta_base = theta_base;
    a.pad = 0;
    return launch(mod, s, "psn_rope_table", (unsigned)((head_dim / 2 + 63) / 64), 64, 0, &a);
}
static int32_t attention_impl(psn_module *mod, psn_stream *s, const psn_buf *q, const psn_buf *k_cache, const psn_buf *v_cache,
                              psn_buf *workspace, psn_buf *out, psn_buf *out_q, int32_t act_type, int32_t n_heads,
                              int32_t n_kv_heads, int32_t head_dim, int32_t n_ctx, const rope_fusion *rope);

extern "C" int32_t psn_attention_decode_q8(psn_module *mod, psn_stream *s, const psn_buf *q, const psn_buf *k_cache, const psn_buf *v_cache,
                                           psn_buf *workspace, psn_buf *out, psn_buf *out_q, int32_t act_type, int32_t n_heads,
                                           int32_t n_kv_heads, int32_t head_dim, int32_t n_ctx) {
    return attention_impl(mod, s, q, k_cache, v_cache, workspace, out, out_q, act_type, n_heads, n_kv_heads, head_dim, n_ctx, nullptr);
}
extern "C" int32_t psn_attention_decode_rope(psn_module *mod, psn_stream *s, const psn_buf *q, const psn_buf *k, const psn_buf *v,
                                             psn_buf *k_cache, psn_buf *v_cache, psn_buf *workspace, psn_buf *out, psn_buf *out_q,
                                             int32_t act_type, int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, int32_t pos,
                                             const psn_buf *rope_table) {
    if (!k || !v || !rope_table) return fail(PSN_E_INVALID_ARG, "psn_attention_decode_rope: k, v or rope_table is null");
    if (pos < 0) return fail(PSN_E_SHAPE, "psn_attention_decode_rope: pos=%d", pos);
    rope_fusion rf = {k, v, rope_table};
    return attention_impl(mod, s, q, k_cache, v_cache, workspace, out, out_q, act_type, n_heads, n_kv_heads, head_dim, pos + 1, &rf);
}
static int32_t attention_impl(psn_module *mod, psn_stream *s, const psn_buf *q, const psn_buf *k_cache, const psn_buf *v_cache,
                              psn_buf *workspace, psn_buf *out, psn_buf *out_q, int32_t act_type, int32_t n_heads,
                              int32_t n_kv_heads, int32_t head_dim, int32_t n_ctx, const rope_fusion *rope) {
    int32_t rc = check_same_ctx(mod, s, q, k_cache, v_cache, "psn_attention_decode");
    if (rc) return rc;
    if (!workspace || (!out && !out_q)) return fail(PSN_E_INVALID_ARG, "psn_attention_decode: null workspace or no output");
    if (out_q && (n_heads & 1)) return fail(PSN_E_SHAPE, "psn_attention_decode: a quantized output needs an even number of heads");
    if (head_dim != 128) return fail(PSN_E_UNSUPPORTED, "psn_attention_decode: head_dim=%d (128 has a kernel)", head_dim);
    if (n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads || n_heads / n_kv_heads > 8)
        return fail(PSN_E_SHAPE, "psn_attention_decode: %d query heads over %d kv heads (need a multiple, at most 8 per group)", n_heads, n_kv_heads);
    if (n_ctx <= 0) return fail(PSN_E_SHAPE, "psn_attention_decode: n_ctx=%d", n_ctx);
    const int32_t splits = (n_ctx + 63) / 64;
    const int64_t row = (int64_t)n_kv_heads * head_dim * 2;
    if ((rc = need(q, (int64_t)n_heads * 512, "psn_attention_decode", "q")) || (out && (rc = need(out, (int64_t)n_heads * 512, "psn_attention_decode", "out"))) ||
        (rc = need(k_cache, n_ctx * row, "psn_attention_decode", "k_cache")) || (rc = need(v_cache, n_ctx * row, "psn_attention_decode", "v_cache")) ||
        (rc = need(workspace, (int64_t)n_heads * splits * 130 * 4, "psn_attention_decode", "workspace")))
        return rc;
    if (workspace->ctx != mod->ctx || (out && out->ctx != mod->ctx)) return fail(PSN_E_INVALID_ARG, "psn_attention_decode: handles belong to different contexts");
    psn_attn_args a;
    memset(&a, 0, sizeof a);
    if ((rc = set_actq_out("psn_attention_decode", mod, out_q, act_type, (int64_t)n_heads * 128, &a.qout))) return rc;
    if ((rc = bind(mod->ctx))) return rc;
    a.q = (const float *)q->p;
    a.k_cache = k_cache->p;
    a.v_cache = v_cache->p;
    a.partial = (float *)workspace->p;
    a.out = out ? (float *)out->p : nullptr;
    a.n_heads = n_heads;
    a.n_kv_heads = n_kv_heads;
    a.n_ctx = n_ctx;
    /* Up to 4096 positions: one workgroup per 64-position chunk and kv head (at 2048 positions that is one
     * workgroup per compute unit of an MI355X).  Beyond: splits of several chunks, about two workgroups per compute unit,
     * walked by the kernel that overlaps its loads with its arithmetic (measured on MI355X at 8192 .. 131072
     * positions).  The workspace is sized for one split per chunk either way. */
    const bool long_ctx = splits > 64;
    int32_t want = 2 * mod->ctx->compute_units / n_kv_heads;      /* splits per kv head: about two workgroups per compute unit */
    want = want < 16 ? 16 : want > 512 ? 512 : want;
    const int32_t chunks = long_ctx ? (splits + want - 1) / want : 1;
    const int32_t nsplits = (splits + chunks - 1) / chunks;
    a.n_splits = nsplits;
    a.chunks = chunks;
    a.scale = 0.08838834764831845f;                 /* 1/sqrt(128) */
    if (rope) {
        if (rope->k_new->ctx != mod->ctx || rope->v_new->ctx != mod->ctx || rope->table->ctx != mod->ctx)
            return fail(PSN_E_INVALID_ARG, "psn_attention_decode_rope: handles belong to different contexts");
        if ((rc = need(rope->k_new, row * 2, "psn_attention_decode_rope", "k")) || (rc = need(rope->v_new, row * 2, "psn_attention_decode_rope", "v")) ||
            (rc = need(rope->table, 128 * 4, "psn_attention_decode_rope", "rope_table")))
            return rc;
        a.k_new = (const float *)rope->k_new->p;
        a.v_new = (const float *)rope->v_new->p;
        a.k_cache_w = k_cache->p;
        a.v_cache_w = v_cache->p;
        a.rope_table = (const float *)rope->table->p;
    }
    const int32_t group = n_heads / n_kv_heads;
    /* (groups of four and eight query heads have long-context kernels of their own, in which a wave serves four heads) */
    const char *partial = long_ctx ? (group == 4   ? (rope ? "psn_attn_partial_rope_long4" : "psn_attn_partial_long4")
                                      : group == 8 ? (rope ? "psn_attn_partial_rope_long8" : "psn_attn_partial_long8")
                                                   : (rope ? "psn_attn_partial_rope_long" : "psn_attn_partial_long"))
                                   : (rope ? "psn_attn_partial_rope" : "psn_attn_partial");
    if ((rc = launch(mod, s, partial, (unsigned)(n_kv_heads * nsplits), (unsigned)(64 * group), 0, &a)))
        return rc;
    return launch(mod, s, "psn_attn_combine", (unsigned)((n_heads + 1) / 2), 128, 0, &a);
}
extern "C" int32_t psn_attention_decode(psn_module *mod, psn_stream *s, const psn_buf *q, const psn_buf *k_cache, const psn_buf *v_cache,
                                        psn_buf *workspace, psn_buf *out, int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, int32_t n_ctx) {
    if (!out) return fail(PSN_E_INVALID_ARG, "psn_attention_decode: out is null");
    return psn_attention_decode_q8(mod, s, q, k_cache, v_cache, workspace, out, nullptr, PSN_Q8_K, n_heads, n_kv_heads, head_dim, n_ctx);
}

extern "C" int32_t psn_swiglu_q8(psn_module *mod, psn_stream *s, const psn_buf *gate, const psn_buf *up, psn_buf *out, psn_buf *out_q,
                                 int32_t act_type, int64_t n) {
    int32_t rc = check_same_ctx(mod, s, gate, up, gate, "psn_swiglu");
    if (rc) return rc;
    if (!out && !out_q) return fail(PSN_E_INVALID_ARG, "psn_swiglu: no output");
    if (n <= 0 || n % 4 || n > (1 << 28)) return fail(PSN_E_SHAPE, "psn_swiglu: n=%lld must be a positive multiple of 4", (long long)n);
    if ((rc = need(gate, n * 4, "psn_swiglu", "gate")) || (rc = need(up, n * 4, "psn_swiglu", "up")) || (out && (rc = need(out, n * 4, "psn_swiglu", "out")))) return rc;
    psn_swiglu_args a;
    if ((rc = set_actq_out("psn_swiglu", mod, out_q, act_type, n, &a.qout))) return rc;
    if ((rc = bind(mod->ctx))) return rc;
    a.gate = (const float *)gate->p;
    a.up = (const float *)up->p;
    a.out = out ? (float *)out->p : nullptr;
    a.n = (int32_t)n;
    a.pad = 0;
    return launch(mod, s, "psn_swiglu", (unsigned)((n / 4 + 255) / 256), 256, 0, &a);
}
extern "C" int32_t psn_swiglu(psn_module *mod, psn_stream *s, const psn_buf *gate, const psn_buf *up, psn_buf *out, int64_t n) {
    if (!out) return fail(PSN_E_INVALID_ARG, "psn_swiglu: out is null");
    return psn_swiglu_q8(mod, s, gate, up, out, nullptr, PSN_Q8_K, n);
}
