/*
 * psn_oracle.h -- CPU restatement of the quantized GGUF compute path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is the checker the HIP kernels are compared
 * against and the CPU baseline that is timed beside them.  Nothing in the
 * shipped library links, loads or calls it.
 *
 * Provenance.  The arithmetic of this path lives in OpenAgentsInc/psionic
 * (doc-pinned at commit 54201484bb8eb11b528f7038922db02724864523 by
 * /root/reference/docs/muse/muse-glimmer.md:22), which is NOT vendored in the
 * reference tree: the tree only names the formats
 * (/root/reference/docs/muse/muse-glimmer.md:112) and the `--backend cpu|cuda|metal`
 * switch (/root/reference/apps/pylon/docs/2026-06-09-pylon-qwen35-local-inference-roadmap.md:137-150).
 * The functions below therefore restate the PUBLISHED GGUF block formats
 * (Q8_0, Q4_0, Q4_K, Q5_K, Q6_K weights; Q8_0, Q8_K activations) and the published
 * reference quantizers / integer dot products for them.
 *
 * Parity status per function (what pins it, since the reference holds no
 * golden vector for this path):
 *   fp16 <-> fp32 ............ pinned: exhaustive 65536-value check vs numpy.float16
 *   nearest_int .............. pinned: brute force incl. +-x.5 ties vs numpy.rint
 *   Q8_0 / Q4_0 quantize ..... pinned: hand-derived known-answer blocks + closed form
 *   Q8_K quantize ............ pinned: closed form + bsums invariant
 *   all dequantizers ......... pinned: independent bit-level packers (pack o unpack = id),
 *                              one-hot lane/nibble-order tests
 *   Q4_K / Q5_K / Q6_K quantize  pinned by what the mathematics fixes (tests/test_oracle_kquant_search.py;
 *                              Q5_K shares Q4_K's search code with 32 levels and 16 candidates from -0.5):
 *                              sub-blocks and whole super-blocks that lie on the format's grid round-trip
 *                              exactly (levels, 6-bit / int8 scales, fp16 d and dmin); the (scale, min)
 *                              returned for a set of levels is the weighted least-squares fit
 *                              (numpy.linalg.lstsq, weights sqrt(mean x^2)+|x| resp. x^2); the result is the
 *                              outcome of the published candidate search restated independently in float64
 *                              (both ends of the Q4_K step range, the coarse end of the Q6_K range), never
 *                              worse than the plain min/max grid; min >= 0.  Bit-for-bit agreement with
 *                              Psionic's own encoder on arbitrary data could only be shown with its source;
 *                              matvec parity does not depend on it (oracle and kernel read the same bytes)
 *   matvec scheme F32 ........ pinned: one-hot activations return deq columns, fp64 truth
 *   matvec scheme Q8 ......... pinned: exact int64/fp64 re-evaluation from the same bytes
 *   prefill matmul ........... pinned: fp64 matmul of fp16-rounded deq(W) with fp16 X
 *   which activation scheme Psionic's CPU path uses: PARITY UNPINNED (both are provided)
 */
#ifndef PSN_ORACLE_H
#define PSN_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGUF tensor type ids */
enum { ORC_Q4_0 = 2, ORC_Q8_0 = 8, ORC_Q4_K = 12, ORC_Q5_K = 13, ORC_Q6_K = 14, ORC_Q8_K = 15 };
/* activation schemes */
enum { ORC_ACT_F32 = 0, ORC_ACT_Q8 = 1 };

uint16_t orc_fp32_to_fp16(float f);
float    orc_fp16_to_fp32(uint16_t h);
int32_t  orc_nearest_int(float f);

/* elements per block and bytes per block for a type id (0 if unknown) */
int64_t orc_block_elems(int32_t qtype);
int64_t orc_block_bytes(int32_t qtype);
/* bytes of one quantized row of k elements (-1 if k is not a whole number of blocks) */
int64_t orc_row_bytes(int32_t qtype, int64_t k);

/* fp32 row -> blocks.  k must be a multiple of the block size. returns 0 / -1 */
int32_t orc_quantize_row(int32_t qtype, const float *x, void *y, int64_t k);
/* blocks -> fp32 row */
int32_t orc_dequantize_row(int32_t qtype, const void *x, float *y, int64_t k);
/* many rows, OpenMP over rows */
int32_t orc_quantize_rows(int32_t qtype, const float *x, void *y, int64_t n, int64_t k, int32_t nthreads);

/* unpack the eight 6-bit (scale, min) pairs of a Q4_K super-block's 12-byte field */
void orc_q4k_scale_min(const uint8_t *scales12, uint8_t sc[8], uint8_t mn[8]);

/* The per-sub-block searches of the K-quant quantizers (test hooks; the row quantizers call these):
 * Q4_K: x[32] ~ scale * L - min, L in 0..15, returns scale, writes L and min;
 * Q6_K: x[16] ~ scale * (L - 32), L in 0..63, returns scale, writes L. */
float orc_q4k_fit_subblock(const float *x32, uint8_t *L, float *min_out);
float orc_q6k_fit_subblock(const float *x16, int8_t *L);
/* Q5_K: as Q4_K with L in 0..31 */
float orc_q5k_fit_subblock(const float *x32, uint8_t *L, float *min_out);

/* integer dot of one quantized weight row with one quantized activation row */
float orc_vec_dot_q(int32_t wtype, const void *w, const void *xq, int64_t k);

/* y[b][n] = sum_k deq(W)[n][k] * x[b][k]   (b < batch)
 * scheme F32: weights dequantized to fp32, fp32 accumulate.
 * scheme Q8 : x quantized to Q8_0 (Q4_0/Q8_0 weights) or Q8_K (Q4_K/Q6_K), integer dot.
 * returns 0, or -1 on bad shape */
int32_t orc_matvec(int32_t wtype, int32_t scheme, const void *W, const float *x, float *y,
                   int64_t n, int64_t k, int32_t batch, int32_t nthreads);

/* same contraction carried in double from the dequantized weights (test truth) */
int32_t orc_matvec_f64(int32_t wtype, const void *W, const float *x, double *y,
                       int64_t n, int64_t k, int32_t batch, int32_t nthreads);

/* Y[m][n] = sum_k h(deq(W)[n][k]) * X[m][k], X given as fp16 bit patterns,
 * h = round to fp16 (RNE); fp32 accumulate. */
int32_t orc_prefill(int32_t wtype, const void *W, const uint16_t *X, float *Y,
                    int64_t m, int64_t n, int64_t k, int32_t nthreads);

/* number of threads OpenMP would use by default */
int32_t orc_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
