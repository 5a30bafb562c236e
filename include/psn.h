/*
 * psn.h -- C ABI of the gfx950 (MI355X) backend for Psionic's quantized GGUF compute path.
 *
 * This is the whole drop-in boundary: a thin extern "C" surface doing module load, buffer
 * alloc, launch and stream sync, which a Rust `-sys` crate binds 1:1.  Plain pointers and
 * sizes only.  There is no CPU fallback behind it: without a gfx950 device every call that
 * needs one fails with PSN_E_NO_DEVICE.
 *
 * What each entry point replaces.  Psionic's backend crates (psionic-backend-cuda / -metal /
 * the CPU backend) are not vendored in the reference tree; the tree pins only their existence
 * and the switch that selects them:
 *   /root/reference/apps/pylon/docs/2026-06-09-pylon-qwen35-local-inference-roadmap.md:137-150
 *       (`psionic-openai-server -m <gguf> --backend cpu|cuda|metal`)
 *   /root/reference/docs/2026-06-10-cs336-distributed-homework-continuation-audit.md:239-241
 *       (crate names psionic-backend-cuda, psionic-backend-metal)
 *   /root/reference/docs/muse/muse-glimmer.md:112
 *       ("kernels for Q4_K, Q5_K, Q6_K, and other GGUF quantizations")
 * Each declaration below names the op of that CUDA backend it stands in for.
 *
 * Conventions
 *   - every call returns int32_t: PSN_OK (0) or a negative PSN_E_* code; psn_last_error()
 *     returns a thread-local, NUL-terminated description of the last failure on this thread;
 *   - handles are created and destroyed by the library; host memory passed in stays the caller's;
 *   - shape and argument errors are detected on the host before anything is launched;
 *   - launches are asynchronous on the given stream; only psn_stream_sync and
 *     psn_event_elapsed_us block.  Calls on distinct streams may come from distinct threads.
 */
#ifndef PSN_H
#define PSN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PSN_ABI_VERSION 1

typedef struct psn_ctx psn_ctx;
typedef struct psn_stream psn_stream;
typedef struct psn_buf psn_buf;
typedef struct psn_module psn_module;
typedef struct psn_event psn_event;
typedef struct psn_graph psn_graph;

/* GGUF tensor type ids */
typedef enum { PSN_Q4_0 = 2, PSN_Q8_0 = 8, PSN_Q4_K = 12, PSN_Q5_K = 13, PSN_Q6_K = 14, PSN_Q8_K = 15 } psn_qtype;
/* how activations enter the dot product */
typedef enum {
    PSN_ACT_F32 = 0, /* weights dequantized to fp32, fp32 FMA */
    PSN_ACT_Q8 = 1   /* x quantized to Q8_0 (Q4_0/Q8_0 weights) or Q8_K (Q4_K/Q5_K/Q6_K), int8 dot */
} psn_act_scheme;
typedef enum { PSN_LAYOUT_GGUF = 0 /* raw GGUF blocks, row-major [N][K/block] */ } psn_layout;

enum {
    PSN_OK = 0,
    PSN_E_INVALID_ARG = -1, /* null handle, handle of another context, buffer too small */
    PSN_E_SHAPE = -2,       /* K not a whole number of blocks, N/M/K <= 0, batch outside 1..8 */
    PSN_E_UNSUPPORTED = -3, /* type / layout / scheme combination without a kernel */
    PSN_E_NO_DEVICE = -4,   /* no HIP device, or the device is not gfx950 */
    PSN_E_OOM = -5,
    PSN_E_MODULE = -6,      /* code object rejected or a kernel symbol is missing */
    PSN_E_HIP = -7          /* any other HIP runtime failure; text carries the hipError_t */
};

/* ---- library ------------------------------------------------------------------------- */

int32_t psn_abi_version(void);
const char *psn_last_error(void);
const char *psn_error_name(int32_t code);

/* elements / bytes per block of a type; bytes of one row of k elements (PSN_E_SHAPE if ragged) */
int32_t psn_block_elems(int32_t qtype);
int32_t psn_block_bytes(int32_t qtype);
int64_t psn_row_bytes(int32_t qtype, int64_t k);

/* Host-side weight quantizer: fp32 rows x[n][k] -> n * psn_row_bytes(qtype, k) bytes of GGUF blocks
 * (Q4_0, Q8_0, Q4_K, Q5_K, Q6_K), byte-identical to the published ggml reference quantizers
 * (quantize_row_*_ref: closed forms for Q4_0/Q8_0, the weighted least-squares scale searches for the
 * K-quants).  Runs on `threads` host threads (rows are independent; < 1 means 1); touches no device.
 * This is the "reference quantizer" step that produces the weights of every benchmark configuration
 * (/root/reference/docs/muse/muse-glimmer.md:112 names the served formats); it replaces the CPU
 * quantize pass a loader runs when a checkpoint arrives as fp32/fp16. */
int32_t psn_quantize_rows(int32_t qtype, const float *x, int64_t n, int64_t k, void *out, size_t out_bytes, int32_t threads);

/* The inverse on the host: n rows of GGUF blocks -> fp32 out[n][k] (out_elems floats available), the
 * published dequantize_row_* formulas in their fp32 operation order.  A loader reads a token's row of a
 * quantized embedding table with it (the one tensor of a model file that is looked up, not multiplied);
 * the activation formats are refused.  Replaces the per-row decode the reference's GGUF loader applies
 * to such tensors (the formats are those /root/reference/docs/muse/muse-glimmer.md:112 names). */
int32_t psn_dequantize_rows(int32_t qtype, const void *blocks, int64_t n, int64_t k, float *out, size_t out_elems);

/* ---- context, module, stream, event, buffer  (the "module load, buffer alloc, launch and
 *      stream sync" surface; replaces the CUDA backend's context/module/stream/buffer wrappers) -- */

int32_t psn_ctx_create(int32_t device, psn_ctx **out);
int32_t psn_ctx_destroy(psn_ctx *ctx);
/* device facts: compute units, bytes of device memory, arch name copied into name[0..n) */
int32_t psn_ctx_info(psn_ctx *ctx, int32_t *compute_units, int64_t *total_mem, char *name, size_t n);
/* free and total bytes of device memory right now (hipMemGetInfo; either pointer may be NULL): what a caller
 * compares before and after a call to see that it allocated nothing */
int32_t psn_ctx_mem_info(psn_ctx *ctx, int64_t *free_bytes, int64_t *total_bytes);

/* load a gfx950 code object from memory / the one built into the library */
int32_t psn_module_load(psn_ctx *ctx, const void *code_object, size_t len, psn_module **out);
int32_t psn_module_load_builtin(psn_ctx *ctx, psn_module **out);
int32_t psn_module_unload(psn_module *mod);
/* PSN_OK if the module exports `kernel_name` */
int32_t psn_module_has_kernel(psn_module *mod, const char *kernel_name);

int32_t psn_stream_create(psn_ctx *ctx, psn_stream **out);
int32_t psn_stream_sync(psn_stream *s);
/* Destroys the stream.  Its workspace (psn_stream_reserve, psn_prefill_reserve) is freed with it unless
 * captured graphs still hold the workspace's address: then the memory stays alive until the last such graph
 * is destroyed, so those graphs remain launchable on other streams. */
int32_t psn_stream_destroy(psn_stream *s);

/* The names of the distinct kernels this thread has launched since psn_launch_log_clear(), in order of first
 * launch, each followed by ';' (a thread-local buffer of 1 KB; when it is full the log ends in "...;").  Throughput
 * records cite it as the kernel that actually ran (the `kernelRef` of the reference's KernelThroughputRecord,
 * /root/reference/packages/tassadar-executor/src/kernel-optimization-parity.ts:27-59). */
const char *psn_launch_log(void);
void psn_launch_log_clear(void);

/* Stream capture into a replayable graph (hipGraph): everything launched on `s` between begin and
 * end is recorded instead of run; psn_graph_launch replays it on a stream.  Calls that would have
 * to allocate or synchronize (a workspace that must grow, uploads, downloads) fail while capturing.
 * Replaces the CUDA backend's CUDA-graph decode loop. */
int32_t psn_graph_begin_capture(psn_stream *s);
int32_t psn_graph_end_capture(psn_stream *s, psn_graph **out);
int32_t psn_graph_launch(psn_graph *g, psn_stream *s);
int32_t psn_graph_destroy(psn_graph *g);
/* Makes `waiter` wait for everything enqueued on `signaler` so far (an event recorded on one stream
 * and awaited on the other).  While `signaler` is being captured this joins `waiter` into the same
 * capture, which is how a graph gets parallel branches: fork with (side, main), launch independent
 * work on both, join with (main, side) before ending the capture. */
int32_t psn_stream_wait_stream(psn_stream *waiter, psn_stream *signaler);
/* Sizes the stream's activation workspace for psn_qmatvec / psn_qmatvec_multi with scheme Q8 up to
 * [batch][K], so later calls (and captures) never allocate.  A graph captured from a call that uses the
 * workspace holds its address: while such a graph exists the workspace cannot grow (calls that would need
 * a larger one fail with PSN_E_INVALID_ARG; destroying the graphs lifts this), so reserve the largest
 * K x batch before the first capture. */
int32_t psn_stream_reserve(psn_stream *s, int64_t K, int32_t batch);
/* The workspace belongs to the stream it was reserved on, also inside a capture: a launch on a side stream
 * that was forked into a capture (psn_stream_wait_stream) uses -- and pins -- the side stream's workspace, and
 * the graph that the capture's origin stream ends holds every workspace the capture touched. */

int32_t psn_event_create(psn_ctx *ctx, psn_event **out);
int32_t psn_event_destroy(psn_event *e);
int32_t psn_event_record(psn_event *e, psn_stream *s);
/* blocks until `end` has happened */
int32_t psn_event_elapsed_us(const psn_event *begin, const psn_event *end, double *out_us);

int32_t psn_buf_alloc(psn_ctx *ctx, size_t bytes, psn_buf **out);
int32_t psn_buf_free(psn_buf *b);
int64_t psn_buf_size(const psn_buf *b);
/* upload, download and fill_zero are synchronous-ordered conveniences that are never recorded into a
 * graph: on a stream that is being captured they fail with PSN_E_INVALID_ARG and leave the capture intact */
int32_t psn_buf_upload(psn_buf *dst, size_t off, const void *src, size_t n, psn_stream *s);
int32_t psn_buf_download(const psn_buf *src, size_t off, void *dst, size_t n, psn_stream *s);
int32_t psn_buf_fill_zero(psn_buf *b, psn_stream *s);
/* device-to-device copy of n bytes, asynchronous on s */
int32_t psn_buf_copy(psn_buf *dst, size_t dst_off, const psn_buf *src, size_t src_off, size_t n, psn_stream *s);

/* ---- weights ---------------------------------------------------------------------------- */

/* Allocates and fills a device copy of an [N][K] quantized tensor from host GGUF blocks
 * (N * psn_row_bytes(qtype, K) bytes).  Replaces the CUDA backend's tensor upload. */
int32_t psn_weight_upload(psn_ctx *ctx, int32_t qtype, int64_t N, int64_t K, const void *gguf_blocks,
                          int32_t layout, psn_stream *s, psn_buf **out);

/* ---- activations ------------------------------------------------------------------------ */

/* Device layout of a quantized activation tensor [batch][K] (all fields row-major over batch):
 *   act_type PSN_Q8_0: int8 qs[batch][K] at off_qs; float d[batch][K/32] at off_d (the block's
 *                      fp16 scale widened to fp32); int32 s[batch][K/32] at off_s (sum of qs)
 *   act_type PSN_Q8_K: int8 qs[batch][K]; float d[batch][K/256]; int16 bsums[batch][K/16]
 * Values equal field-for-field what the GGUF Q8_0 / Q8_K row quantizers produce. */
typedef struct psn_actq_info {
    int64_t off_qs, off_d, off_s, bytes;
} psn_actq_info;
int32_t psn_actq_layout(int32_t act_type, int64_t K, int32_t batch, psn_actq_info *out);
/* the activation type the Q8 scheme pairs with a weight type (PSN_Q8_0 or PSN_Q8_K) */
int32_t psn_act_type_for(int32_t weight_qtype);

/* x_f32 [batch][K] -> x_q in the layout above.  Replaces the CUDA backend's activation
 * quantize kernel (the "same activation-quantization scheme" the CPU path uses). */
int32_t psn_act_quantize(psn_module *mod, psn_stream *s, int32_t act_type, const psn_buf *x_f32, psn_buf *x_q,
                         int64_t K, int32_t batch);

/* ---- decode matvec ------------------------------------------------------------------------ */

/* y[b][n] = sum_k deq(W)[n][k] * x[b][k], b < batch (1..8), y fp32 [batch][N].
 * Scheme Q8 quantizes x into a workspace owned by the stream, then runs the int8 kernel.
 * Replaces the CUDA backend's quantized matvec op (decode path). */
int32_t psn_qmatvec(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, int32_t scheme, const psn_buf *W,
                    const psn_buf *x_f32, psn_buf *y_f32, int64_t N, int64_t K, int32_t batch);

/* Same contraction from activations already quantized by psn_act_quantize (one quantization
 * can feed several matrices, e.g. q/k/v or gate/up). */
int32_t psn_qmatvec_q8(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, const psn_buf *W,
                       const psn_buf *x_q, psn_buf *y_f32, int64_t N, int64_t K, int32_t batch);

/* Several matrices that share K, the format and the activations in ONE launch (q/k/v, gate/up):
 * y[i] = W[i] x for i < count (1..4), each y[i] fp32 [batch][N[i]].  psn_qmatvec_multi takes fp32
 * activations (scheme as above), psn_qmatvec_q8_multi already-quantized ones. */
int32_t psn_qmatvec_multi(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, int32_t scheme, int32_t count,
                          const psn_buf *const *W, const psn_buf *x_f32, psn_buf *const *y_f32, const int64_t *N, int64_t K,
                          int32_t batch);
int32_t psn_qmatvec_q8_multi(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, int32_t count,
                             const psn_buf *const *W, const psn_buf *x_q, psn_buf *const *y_f32, const int64_t *N, int64_t K,
                             int32_t batch);

/* psn_qmatvec for callers that cannot allocate device memory (code under graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  This entry point has no counterpart in the reference: it exists
 * for those callers only.  Same arguments and results as psn_qmatvec, but nothing is allocated or freed,
 * on the device or through any allocating library routine (the first launch of a kernel name on a module
 * looks the kernel up and remembers it in a host-side table; later calls do no host allocation either):
 * with scheme Q8 the quantized activations go
 * into a static array in the library's device image (psn_noalloc_max_bytes() bytes per GPU, held until
 * the process ends) instead of the stream's workspace.  Shapes whose quantized activations
 * (psn_actq_layout(...).bytes) exceed that size fail with PSN_E_SHAPE.  Every call on a GPU shares that
 * GPU's array: calls that overlap in time on one GPU (different streams, or graphs replayed
 * concurrently) race on it -- serialize them.  Nothing has to be cleared between calls: each call
 * overwrites every byte it later reads. */
int32_t psn_qmatvec_noalloc(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, int32_t scheme, const psn_buf *W,
                            const psn_buf *x_f32, psn_buf *y_f32, int64_t N, int64_t K, int32_t batch);
int64_t psn_noalloc_max_bytes(void);

/* Launch geometry of one matvec.  psn_qmatvec_plan fills in the library's choice for a shape
 * (pure host arithmetic, usable without a device; x_is_f32 != 0 asks for the plan psn_qmatvec uses
 * when it quantizes fp32 activations inside the matvec launch); psn_qmatvec_planned runs with a
 * caller-chosen one (auto-tuners, benchmarks). */
typedef struct psn_matvec_plan {
    int32_t lanes_per_row;  /* 8, 16, 32 or 64 lanes share one row */
    int32_t rows_in_flight; /* row sets per lane: 1 */
    int32_t batch_tile;     /* compiled batch width: 1, 2, 4 or 8 (>= batch) */
    int32_t stage_lds;      /* 0: activations read from global memory; 1: staged in LDS; 2 (scheme Q8): x is
                               fp32 and every workgroup quantizes it while staging */
    int32_t blocks;         /* workgroups */
    int32_t threads;        /* threads per workgroup: 256 or 512 */
    int32_t stream;         /* 0: register kernels; 1..8: streaming kernel -- weights land in per-wave rings of that
                               many LDS buffers by direct-to-LDS loads (scheme Q8, batch 1, rows of whole 16-byte
                               words and at most lanes_per_row chunks, every matrix a multiple of 64/lanes_per_row
                               rows, stage_lds 1 or 2, 256 or 512 threads) */
    int32_t mfma;           /* 0, or 1/2/4/8: the small-batch int8-MFMA kernel (Q4_K and Q5_K, scheme Q8, batch 1..8,
                               x already quantized: stage_lds 1) -- that many waves share a 16-row tile, each owning
                               K / mfma of it (a whole number of at most eight 256-weight chunks); every matrix a
                               multiple of 16 rows; stream = 1; slices of more than four chunks need one wave per
                               (tile, slice): blocks * (threads / 64 / mfma) >= tiles; lanes_per_row, rows_in_flight
                               and batch_tile are not used */
} psn_matvec_plan;
int32_t psn_qmatvec_plan(int32_t qtype, int32_t scheme, int64_t N, int64_t K, int32_t batch, int32_t compute_units,
                         int32_t x_is_f32, psn_matvec_plan *out);
/* x is x_f32 for scheme F32 and for stage_lds == 2, x_q (already quantized) otherwise; N in the
 * plan call is the total row count when several matrices share the launch */
int32_t psn_qmatvec_planned(psn_module *mod, psn_stream *s, int32_t qtype, int32_t scheme, int32_t count,
                            const psn_buf *const *W, const psn_buf *x, psn_buf *const *y_f32, const int64_t *N, int64_t K,
                            int32_t batch, const psn_matvec_plan *plan);

/* ---- calibration -----------------------------------------------------------------------------
 * A launch that only reads `bytes` of `src` (whole 4 KB slabs; lds_depth 0: vector loads into registers,
 * 1..64: direct-to-LDS loads cycling through that many 1 KB slots per wave) and stores one dword per wave
 * to `out` (may be NULL).  With every_workgroup != 0 each workgroup reads the whole range instead of the
 * workgroups sharing it (the pattern of an operand all workgroups need, served from L2).  Benchmarks time it beside a matvec of the same size to separate what the
 * machine allows a dependent launch from what the kernel adds.  No counterpart in the reference. */
int32_t psn_calibrate_read(psn_module *mod, psn_stream *s, const psn_buf *src, int64_t bytes, int32_t blocks, int32_t threads,
                           int32_t lds_depth, int32_t every_workgroup, psn_buf *out);

/* No counterpart in the reference: a check of this device's arithmetic.  The activation quantizers take their
 * IEEE divisions (amax / 127, 1 / d, -127 / max, 1 / iscale) by a reciprocal approximation corrected with fused
 * multiply-adds; the launch compares those shortcuts with true division for every float between 2^-100 and 2^100
 * in magnitude, both signs, and leaves eight 64-bit mismatch counters in `out` (64 bytes; all zero on gfx950).
 * Outside that range the quantizers divide the long way. */
int32_t psn_selftest_arith(psn_module *mod, psn_stream *s, psn_buf *out);

/* ---- prefill matmul ----------------------------------------------------------------------- */

/* Y[m][n] = sum_k h(deq(W)[n][k]) * X[m][k]; X fp16 [M][K], Y fp32 [M][N], weight tiles are
 * dequantized to fp16 (h = round to nearest even) in LDS and fed to fp16 MFMA with fp32
 * accumulation.  qtype PSN_Q4_0 or PSN_Q8_0 (every kernel family below), PSN_Q4_K, PSN_Q5_K or PSN_Q6_K
 * (families 4, 64 and 128, and for Q4_K / Q5_K family 16 on the 128x256 tile; planned by psn_qmatmul_prefill_plan_for;
 * their fp32 dequantization is restated operation by operation before the rounding to fp16).  Replaces the CUDA backend's quantized prefill
 * matmul op. */
int32_t psn_qmatmul_prefill(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, const psn_buf *W,
                            const psn_buf *X_f16, psn_buf *Y_f32, int64_t M, int64_t N, int64_t K);
/* The launch shape the library picks for a prefill: the workgroup tile of Y (64x64, 64x128, 128x128,
 * 128x256, 256x128 or 256x256), into how many ranges K is cut (1, 2, 4 or 8; with more than one, Y is
 * zeroed by a fill kernel and the partial sums are added atomically, so their order -- and the last bit
 * of a sum -- can vary between runs), and the kernel family:
 *    4  four waves, every wave stages and multiplies (any tile);
 *   16  eight waves of which four only multiply and four only stage: X by direct-to-LDS loads three K
 *       steps ahead, weights decoded from registers one step ahead (64x64, 64x128, 128x128, 128x256);
 *   32  the wide kernel for large M (256x256 tiles only): four waves, each with all 256 rows x 64 columns
 *       in 256 accumulator registers; X and the raw GGUF bytes arrive in LDS rings by direct-to-LDS loads,
 *       a wave decodes the operand of its own columns one K slice ahead, interleaved with its MFMAs;
 *   64  the weight-streaming kernel for M <= 64 (64x64 tiles; every format, Q6_K only when K is a multiple of
 *       2048 so that its rows are whole 16-byte words): X and the raw GGUF bytes arrive in LDS rings by
 *       direct-to-LDS loads, every wave decodes its own MFMA operand, one barrier per 256 of K;
 *  128  the dense family for large M (256x256 or 128x256 tiles, every format): one pass writes h(deq(W)) for the whole
 *       matrix as fp16 into the stream's workspace (ceil(N/256) * 256 * K * 2 bytes, see
 *       psn_prefill_reserve), in the order the multiply kernel's MFMA operands are read; that kernel has no
 *       decode in its loop.  Same fp16 values as every other family, two launches (three with K cut).
 * Host arithmetic only ... */
int32_t psn_qmatmul_prefill_plan(int64_t M, int64_t N, int64_t K, int32_t compute_units, int32_t *tile_m, int32_t *tile_n,
                                 int32_t *ksplit, int32_t *waves);
/* The same for a given weight type: what psn_qmatmul_prefill runs when the dense family's workspace is
 * available (psn_qmatmul_prefill_plan answers for Q4_0 / Q8_0; the K-quants have families 4, 16 on the
 * 128x256 tile, 128, and 64 for M <= 64).  While a stream is capturing, or while a captured graph refers to its workspace,
 * the workspace cannot grow: psn_qmatmul_prefill then takes the best plan without family 128 unless
 * psn_prefill_reserve (or an earlier dense call of that size) has sized it. */
int32_t psn_qmatmul_prefill_plan_for(int32_t qtype, int64_t M, int64_t N, int64_t K, int32_t compute_units, int32_t *tile_m,
                                     int32_t *tile_n, int32_t *ksplit, int32_t *waves);
/* Sizes the stream's workspace for the dense family on an [N][K] matrix (and keeps whatever the decode
 * matvecs reserved: the workspace only grows).  Call before capturing a graph that should contain it. */
int32_t psn_prefill_reserve(psn_stream *s, int64_t N, int64_t K);
/* The dense family with the dequantization hoisted out of the call: psn_prefill_pack writes h(deq(W)) once
 * into a caller-owned buffer of psn_prefill_packed_bytes(N, K) bytes (2 bytes per weight, rows padded to whole
 * 256-row panels; a deployment with HBM to spare keeps one per matrix beside the GGUF blocks the decode
 * matvec reads), psn_qmatmul_prefill_packed multiplies any number of X against it -- the same result as
 * psn_qmatmul_prefill_tiled(..., 256, 256, ksplit, 128) without the 35-48 us pass per call.  No stream
 * workspace is involved.  No counterpart in the reference, which dequantizes inside every call. */
int64_t psn_prefill_packed_bytes(int64_t N, int64_t K);
int32_t psn_prefill_pack(psn_module *mod, psn_stream *s, int32_t qtype, const psn_buf *W, psn_buf *packed, int64_t N, int64_t K);
int32_t psn_qmatmul_prefill_packed(psn_module *mod, psn_stream *s, const psn_buf *packed, const psn_buf *X_f16, psn_buf *Y_f32,
                                   int64_t M, int64_t N, int64_t K);
/* ... and the same matmul with a caller-chosen shape (auto-tuners, benchmarks). */
int32_t psn_qmatmul_prefill_tiled(psn_module *mod, psn_stream *s, int32_t qtype, const psn_buf *W, const psn_buf *X_f16,
                                  psn_buf *Y_f32, int64_t M, int64_t N, int64_t K, int32_t tile_m, int32_t tile_n,
                                  int32_t ksplit, int32_t waves);

/* ---- decode-step glue (what sits between the matvecs of a Llama-style layer) ----------------
 * These replace the CUDA backend's RMSNorm / rotary / attention / activation ops only as far as a
 * whole token step needs them to be measured on the device; all vectors are fp32, the KV cache is
 * fp16 [positions][n_kv_heads][head_dim].  Positions are immediate arguments: a captured graph
 * replays the position it was captured at. */

/* x += delta (skipped when delta is NULL), then y = x * rsqrt(mean(x^2) + eps) * weight; n % 4 == 0 */
int32_t psn_add_rmsnorm(psn_module *mod, psn_stream *s, psn_buf *x, const psn_buf *delta, const psn_buf *weight, psn_buf *y,
                        int64_t n, float eps);
/* rotary embedding (pairs (2i, 2i+1), angle pos * theta_base^(-2i/head_dim)) of q in place and of k,
 * then k and v are stored as fp16 at row `pos` of the caches */
int32_t psn_rope_kv_store(psn_module *mod, psn_stream *s, psn_buf *q, psn_buf *k, const psn_buf *v, psn_buf *k_cache,
                          psn_buf *v_cache, int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, int32_t pos, float theta_base);
/* softmax(q K^T / sqrt(head_dim)) V over cache positions 0 .. n_ctx-1, grouped-query (n_heads a multiple
 * of n_kv_heads, at most 8 per group), head_dim 128; workspace holds n_heads * ceil(n_ctx/64) * 130 floats
 * (beyond 4096 positions the kernels use fewer, longer splits and only the front of it) */
int32_t psn_attention_decode(psn_module *mod, psn_stream *s, const psn_buf *q, const psn_buf *k_cache, const psn_buf *v_cache,
                             psn_buf *workspace, psn_buf *out, int32_t n_heads, int32_t n_kv_heads, int32_t head_dim,
                             int32_t n_ctx);
/* out = silu(gate) * up; n % 4 == 0 */
int32_t psn_swiglu(psn_module *mod, psn_stream *s, const psn_buf *gate, const psn_buf *up, psn_buf *out, int64_t n);

/* The same three producers with the activation quantization fused in: besides (or, with a NULL fp32
 * output, instead of) the fp32 vector they write it as a one-row quantized activation tensor
 * (psn_actq_layout(act_type, n, 1)) that psn_qmatvec_q8(_multi) consumes directly -- bit-identical to
 * psn_act_quantize of the fp32 result.  n must be a multiple of 256 (psn_attention_decode_q8: an even
 * number of heads). */
int32_t psn_add_rmsnorm_q8(psn_module *mod, psn_stream *s, psn_buf *x, const psn_buf *delta, const psn_buf *weight, psn_buf *y,
                           psn_buf *y_q, int32_t act_type, int64_t n, float eps);
int32_t psn_swiglu_q8(psn_module *mod, psn_stream *s, const psn_buf *gate, const psn_buf *up, psn_buf *out, psn_buf *out_q,
                      int32_t act_type, int64_t n);
/* psn_add_rmsnorm_q8 folded into the projection that consumes it (batch 1, scheme Q8):
 *     h = x + delta (delta may be NULL);  y_i = W_i . q8(h * rsqrt(mean(h^2) + eps) * norm_weight)
 * Every workgroup of the streaming matvec adds, normalizes and quantizes the K fp32 values while it
 * stages them (its weight loads are already in flight), so the norm costs no launch of its own;
 * workgroup 0 also stores h to h_out (may be NULL), which must not alias x or delta -- a decoder
 * alternates two residual buffers.  Shapes the fused kernels do not serve (rows longer than 8192, more
 * than three matrices, row counts that are not whole passes) run the norm kernel and the pre-quantized
 * matvec as two launches with the same result.  x and delta are never written on either path: h goes to
 * h_out or nowhere, so several calls (one per weight format among q|k|v) may share x and delta.  No counterpart in the reference's CPU path, which
 * normalizes, quantizes and multiplies as separate steps; the arithmetic per element is the same. */
int32_t psn_qmatvec_norm_multi(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, int32_t count,
                               const psn_buf *const *W, const psn_buf *x, const psn_buf *delta, const psn_buf *norm_weight,
                               psn_buf *h_out, psn_buf *const *y_f32, const int64_t *N, int64_t K, float eps);
/* The same launch for a feed-forward block's gate | up pair with SwiGLU applied to the two products before they
 * leave the kernel:
 *     h = x + delta;  n = q8(h * rsqrt(mean(h^2) + eps) * norm_weight);  act_f32[i] = silu(W_gate[i] . n) * (W_up[i] . n)
 * (N rows each, act_f32 holds N floats) -- the floats psn_qmatvec_norm_multi + psn_swiglu return, without the
 * SwiGLU launch and without the two N-vectors in between: a wave multiplies the same rows of both matrices one
 * after the other and keeps the first product in a register.  The down projection then takes act_f32 through
 * psn_qmatvec, which quantizes while it stages.  Only shapes the fused streaming kernels serve (batch 1, rows
 * of at most 8192, N a multiple of the rows per pass): psn_qmatvec_norm_swiglu_check says beforehand, by host
 * arithmetic alone, whether a shape is one of them (PSN_OK) or the three separate calls are needed
 * (PSN_E_UNSUPPORTED).  No counterpart in the reference's CPU path, which runs the steps one by one. */
int32_t psn_qmatvec_norm_swiglu(psn_module *mod, psn_stream *s, int32_t qtype, int32_t layout, const psn_buf *W_gate,
                                const psn_buf *W_up, const psn_buf *x, const psn_buf *delta, const psn_buf *norm_weight,
                                psn_buf *h_out, psn_buf *act_f32, int64_t N, int64_t K, float eps);
int32_t psn_qmatvec_norm_swiglu_check(int32_t qtype, int64_t N, int64_t K, int32_t compute_units);
int32_t psn_attention_decode_q8(psn_module *mod, psn_stream *s, const psn_buf *q, const psn_buf *k_cache, const psn_buf *v_cache,
                                psn_buf *workspace, psn_buf *out, psn_buf *out_q, int32_t act_type, int32_t n_heads,
                                int32_t n_kv_heads, int32_t head_dim, int32_t n_ctx);
/* cos / sin of the head_dim/2 rotary pairs at position pos into `table` (head_dim floats); once per
 * token, shared by all layers */
int32_t psn_rope_table(psn_module *mod, psn_stream *s, psn_buf *table, int32_t head_dim, int32_t pos, float theta_base);
/* psn_rope_kv_store + psn_attention_decode(_q8) in two launches instead of three: q, k, v are the raw
 * projections of the token at position pos; the attention kernel rotates q and k itself with the
 * coefficients of psn_rope_table (same arithmetic), appends k and v to the
 * caches and attends over positions 0 .. pos.  q is left unrotated.  out and out_q as above (either
 * may be NULL, not both). */
int32_t psn_attention_decode_rope(psn_module *mod, psn_stream *s, const psn_buf *q, const psn_buf *k, const psn_buf *v,
                                  psn_buf *k_cache, psn_buf *v_cache, psn_buf *workspace, psn_buf *out, psn_buf *out_q,
                                  int32_t act_type, int32_t n_heads, int32_t n_kv_heads, int32_t head_dim, int32_t pos,
                                  const psn_buf *rope_table);

#ifdef __cplusplus
}
#endif
#endif
