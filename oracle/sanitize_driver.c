/*
 * sanitize_driver.c -- exercises every oracle entry point on small seeded inputs; built with
 * -fsanitize=address,undefined by tests/test_oracle_sanitize.py (host code only).  TEST INFRASTRUCTURE.
 */
#include "psn_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>

static unsigned long long s = 88172645463325252ull;
static float rnd(void) {                       /* xorshift -> roughly uniform in [-1, 1) */
    s ^= s << 13; s ^= s >> 7; s ^= s << 17;
    return (float)((double)(s >> 11) / 9007199254740992.0 * 2.0 - 1.0);
}

int main(void) {
    const int types[4] = {ORC_Q4_0, ORC_Q8_0, ORC_Q4_K, ORC_Q6_K};
    const int64_t n = 37, k = 1280, m = 5;
    float *w = malloc(sizeof(float) * n * k), *x = malloc(sizeof(float) * 3 * k), *y = malloc(sizeof(float) * 3 * n);
    double *y64 = malloc(sizeof(double) * 3 * n);
    uint16_t *xh = malloc(sizeof(uint16_t) * m * k);
    float *yp = malloc(sizeof(float) * m * n), *row = malloc(sizeof(float) * k);
    if (!w || !x || !y || !y64 || !xh || !yp || !row) return 2;
    for (int64_t i = 0; i < n * k; i++) w[i] = 0.02f * rnd();
    for (int64_t i = 0; i < 3 * k; i++) x[i] = rnd();
    for (int64_t i = 0; i < m * k; i++) xh[i] = orc_fp32_to_fp16(rnd());
    for (int64_t i = 0; i < 256; i++) w[i] = 0.f;                    /* an all-zero super-block */
    int bad = 0;
    for (int t = 0; t < 4; t++) {
        const int64_t rb = orc_row_bytes(types[t], k);
        void *q = malloc((size_t)(rb * n));
        if (!q) return 2;
        bad |= orc_quantize_rows(types[t], w, q, n, k, 2);
        bad |= orc_dequantize_row(types[t], q, row, k);
        for (int scheme = 0; scheme < 2; scheme++) bad |= orc_matvec(types[t], scheme, q, x, y, n, k, 3, 2);
        bad |= orc_matvec_f64(types[t], q, x, y64, n, k, 3, 2);
        if (types[t] == ORC_Q4_0 || types[t] == ORC_Q8_0) bad |= orc_prefill(types[t], q, xh, yp, m, n, k, 2);
        for (int64_t i = 0; i < 3 * n; i++) if (!isfinite(y[i]) || !isfinite(y64[i])) bad |= 4;
        free(q);
    }
    {
        void *q8k = malloc((size_t)orc_row_bytes(ORC_Q8_K, k));
        bad |= orc_quantize_row(ORC_Q8_K, x, q8k, k);
        bad |= orc_dequantize_row(ORC_Q8_K, q8k, row, k);
        free(q8k);
    }
    if (orc_row_bytes(ORC_Q4_K, 100) != -1 || orc_matvec(ORC_Q4_0, 0, w, x, y, 0, k, 1, 1) != -1) bad |= 8;
    uint8_t field[12] = {1, 2, 3, 4, 5, 6, 7, 8, 0x9A, 0xBC, 0xDE, 0xF0}, sc[8], mn[8];
    orc_q4k_scale_min(field, sc, mn);
    if (orc_nearest_int(2.5f) != 2 || orc_fp16_to_fp32(0x3C00) != 1.0f) bad |= 16;
    free(w); free(x); free(y); free(y64); free(xh); free(yp); free(row);
    printf(bad ? "FAIL %d\n" : "ok\n", bad);
    return bad ? 1 : 0;
}
