/* Test infrastructure: runs every function of the CPU oracle once on buffers that are
 * allocated at exactly the size the function may touch (odd row counts, several batches,
 * strides wider than the rows), so that a build with -fsanitize=address,undefined stops at
 * the first out-of-bounds access, misaligned access or undefined arithmetic.
 * Built and run by `make -C oracle sanitize` (tests/test_oracle_sanitized.py). */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "q8_oracle.h"

static uint32_t rng_state = 12345u;
static float rnd(void) {
    rng_state = rng_state * 1664525u + 1013904223u;
    return ((float)(rng_state >> 8) / 8388608.0f - 1.0f) * 3.0f;
}
static void *xmalloc(size_t n) {
    void *p = malloc(n ? n : 1);
    if (!p) { fprintf(stderr, "out of memory\n"); exit(2); }
    return p;
}
#define CHECK(expr) do { if (!(expr)) { fprintf(stderr, "sanitize_check: %s failed at line %d\n", #expr, __LINE__); exit(1); } } while (0)

static void run_shape(uint32_t rows, uint32_t cols, uint32_t batch) {
    const uint32_t nb = cols / 32, stride_x = cols + 5, stride_dst = rows + 3;
    float *wf = xmalloc(sizeof(float) * rows * cols);
    for (size_t i = 0; i < (size_t)rows * cols; ++i) wf[i] = rnd() * 0.02f;
    uint8_t *gguf = xmalloc((size_t)rows * nb * 34), *w = xmalloc((size_t)rows * nb * 34);
    CHECK(q8o_quantize_q8_0(wf, rows, cols, gguf) == 0);
    CHECK(q8o_repack_split_plane(gguf, rows, cols, w) == 0);
    float *row = xmalloc(sizeof(float) * cols);
    CHECK(q8o_get_row(w, rows - 1, cols, row) == 0);

    float *x = xmalloc(sizeof(float) * ((size_t)(batch - 1) * stride_x + cols));
    for (size_t i = 0; i < (size_t)(batch - 1) * stride_x + cols; ++i) x[i] = rnd();
    for (uint32_t i = 0; i < 32 && i < cols; ++i) x[i] = 0.0f;             /* an all-zero block */
    float *nw = xmalloc(sizeof(float) * cols), *normed = xmalloc(sizeof(float) * ((size_t)(batch - 1) * stride_x + cols));
    for (uint32_t i = 0; i < cols; ++i) nw[i] = 1.0f + 0.01f * rnd();
    CHECK(q8o_rms_norm(x, nw, normed, batch, cols, stride_x, stride_x, 1e-6f) == 0);

    uint8_t *y = xmalloc((size_t)batch * nb * 36);
    CHECK(q8o_quantize_q8_1(x, batch, cols, stride_x, y) == 0);
    (void)q8o_block_dot(w, y, 0, cols, batch, rows - 1, batch - 1, nb - 1);

    const size_t nout = (size_t)(batch - 1) * stride_dst + rows;
    float *d0 = xmalloc(sizeof(float) * nout), *d1 = xmalloc(sizeof(float) * nout);
    uint16_t *h0 = xmalloc(sizeof(uint16_t) * nout);
    memset(d0, 0, sizeof(float) * nout); memset(d1, 0, sizeof(float) * nout); memset(h0, 0, sizeof(uint16_t) * nout);
    CHECK(q8o_gemv(w, y, d0, rows, cols, batch, stride_dst, 1) == 0);
    CHECK(q8o_gemv(w, y, d1, rows, cols, batch, stride_dst, 3) == 0);
    for (uint32_t j = 0; j < batch; ++j)
        CHECK(memcmp(d0 + (size_t)j * stride_dst, d1 + (size_t)j * stride_dst, sizeof(float) * rows) == 0);
    CHECK(q8o_gemv_abs(w, y, d1, rows, cols, batch, stride_dst) == 0);
    CHECK(q8o_gemv_bf16(w, y, h0, rows, cols, batch, stride_dst) == 0);
    CHECK(q8o_gemv_two(w, w, y, d0, d1, rows, cols, batch, stride_dst) == 0);
    CHECK(q8o_gemv_silu_mul(w, w, y, d0, rows, cols, batch, stride_dst) == 0);
    CHECK(q8o_gemv_add(w, y, d0, rows, cols, batch, stride_dst) == 0);
    CHECK(q8o_gemv_add_bf16(w, y, h0, rows, cols, batch, stride_dst) == 0);
    {
        const uint8_t *ws[4] = {w, NULL, w, w};
        float *ds[4] = {d0, NULL, d1, NULL};
        const uint32_t rs[4] = {rows, 0, rows, rows}, st[4] = {stride_dst, 0, stride_dst, 0};
        CHECK(q8o_gemv_fanout4(ws, y, ds, rs, cols, batch, st) == 0);
    }
    if (cols % 128 == 0) {
        uint8_t *y4 = xmalloc((size_t)(cols / 128) * batch * 144);
        CHECK(q8o_quantize_q8_1_d4(x, batch, cols, stride_x, y4) == 0);
        (void)q8o_block_dot(w, y4, 1, cols, batch, 0, batch - 1, nb - 1);
        CHECK(q8o_gemm_d4(w, y4, d0, rows, cols, batch, stride_dst, 2) == 0);
        const uint32_t ri[3] = {0, rows - 1, rows / 2}, ji[3] = {0, batch - 1, batch / 2};
        float s[3], sa[3];
        CHECK(q8o_gemm_d4_sampled(w, y4, rows, cols, batch, ri, ji, 3, s, sa) == 0);
        for (int i = 0; i < 3; ++i) CHECK(s[i] == d0[(size_t)ji[i] * stride_dst + ri[i]]);
        free(y4);
    }
    free(wf); free(gguf); free(w); free(row); free(x); free(nw); free(normed); free(y); free(d0); free(d1); free(h0);
}

static void run_argmax(uint32_t batch, uint32_t n) {
    float *x = xmalloc(sizeof(float) * (size_t)batch * n);
    for (size_t i = 0; i < (size_t)batch * n; ++i) x[i] = rnd();
    x[n / 2] = NAN;
    if (batch > 1) for (uint32_t i = 0; i < n; ++i) x[(size_t)(batch - 1) * n + i] = -INFINITY;
    q8o_argmax_pair *out = xmalloc(sizeof(q8o_argmax_pair) * batch), one = q8o_argmax_row(x, n);
    (void)one;
    (void)q8o_argmax_rows(x, batch, n, out);
    q8o_argmax_rows_scan(x, batch, n, out);
    int32_t tokens[8] = {5, 7, -1, 9, 1, 2, 3, 4}, drafts[7] = {5, 7, 2, 0, 0, 0, 0}, next = -2;
    const uint32_t acc = q8o_accept(tokens, drafts, 7, 2, &next);
    CHECK(acc == 3 && next == 9);   /* row 2 has no token and reads as eos = drafts[2] */
    free(x); free(out);
}

int main(void) {
    for (uint32_t v = 0; v < 65536; v += 257) {
        const float f = q8o_f16_to_f32((uint16_t)v);
        if (f == f) CHECK(q8o_f32_to_f16(f) == (uint16_t)v);
        (void)q8o_f32_to_bf16(q8o_bf16_to_f32((uint16_t)v));
    }
    (void)q8o_f32_to_f16(1e30f); (void)q8o_f32_to_f16(-1e-30f); (void)q8o_f32_to_f16(NAN); (void)q8o_f32_to_bf16(NAN);
    run_shape(1, 32, 1);
    run_shape(7, 96, 3);
    run_shape(33, 256, 8);
    run_shape(130, 640, 5);
    run_argmax(1, 1);
    run_argmax(3, 1000);
    run_argmax(8, 70001);
    printf("sanitize_check: ok\n");
    return 0;
}
