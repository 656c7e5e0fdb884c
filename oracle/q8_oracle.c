/*
 * q8_oracle.c — scalar CPU restatement of qw3's Q8_0 x Q8_1 linear path.
 * TEST INFRASTRUCTURE ONLY (see q8_oracle.h): checker and timed CPU baseline,
 * never part of the shipped GPU path.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off; fused multiply-adds are
 * written explicitly with fmaf so the arithmetic does not depend on flags).
 */
#include "q8_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------- */
/* scalar conversions                                                        */

static inline uint32_t f32_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

static inline float bits_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}

uint16_t q8o_f32_to_f16(float f) {
    const uint32_t u = f32_bits(f);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) { /* NaN: keep it a NaN, carry the top payload bits */
        return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x01ffu));
    }
    if (a >= 0x47800000u) { /* |f| >= 65536 (also inf) */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (a < 0x33000000u) { /* |f| < 2^-25: rounds to zero (2^-25 itself ties to even = 0) */
        return sign;
    }
    const int32_t e = (int32_t)(a >> 23) - 127; /* unbiased exponent, -25..15 */
    uint32_t m = (a & 0x007fffffu) | 0x00800000u; /* 24-bit significand */
    uint32_t shift, base;
    if (e >= -14) { /* normal half: keep 11 significant bits */
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        m &= 0x007fffffu; /* drop the implicit bit, it is encoded by the exponent */
    } else { /* subnormal half: value = m * 2^(e-23), unit = 2^-24 */
        shift = (uint32_t)(13 + (-14 - e));
        base = 0;
    }
    const uint32_t q = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    uint32_t h = base + q; /* a carry out of the mantissa correctly bumps the exponent */
    if (rem > half || (rem == half && (q & 1u))) h += 1u;
    return (uint16_t)(sign | h);
}

float q8o_f16_to_f32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1fu;
    const uint32_t man = h & 0x03ffu;
    if (exp == 0) {
        /* zero or subnormal: man * 2^-24, exact in fp32 */
        const float v = (float)man * 5.9604644775390625e-8f;
        return bits_f32(f32_bits(v) | sign);
    }
    if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t q8o_f32_to_bf16(float f) {
    const uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fffu;
    const uint32_t lsb = (u >> 16) & 1u;
    return (uint16_t)((u + 0x7fffu + lsb) >> 16);
}

float q8o_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* round-to-nearest-even float -> int with CUDA's __float2int_rn conventions:
 * NaN -> 0, out of range saturates. */
static inline int32_t float2int_rn(float v) {
    if (v != v) return 0;
    const float r = rintf(v); /* default rounding mode: nearest-even */
    if (r >= 2147483648.0f) return INT32_MAX;
    if (r <= -2147483648.0f) return INT32_MIN;
    return (int32_t)r;
}

/* ------------------------------------------------------------------------- */
/* weights                                                                   */

int q8o_quantize_q8_0(const float *w, uint64_t rows, uint64_t cols, uint8_t *out) {
    if (cols % Q8O_QK != 0) return -1;
    const uint64_t nb = cols / Q8O_QK;
    for (uint64_t r = 0; r < rows; ++r) {
        for (uint64_t kb = 0; kb < nb; ++kb) {
            const float *src = w + r * cols + kb * Q8O_QK;
            float amax = 0.0f;
            for (int t = 0; t < Q8O_QK; ++t) {
                const float a = fabsf(src[t]);
                if (a > amax) amax = a; /* std::max(amax, a) */
            }
            const float d = amax / 127.0f;
            const float d_inv = (d == 0.0f) ? 0.0f : 1.0f / d;
            uint8_t *blk = out + (r * nb + kb) * Q8O_Q8_0_BYTES;
            const uint16_t hd = q8o_f32_to_f16(d);
            memcpy(blk, &hd, 2);
            for (int t = 0; t < Q8O_QK; ++t) {
                long qi = lrintf(src[t] * d_inv);
                if (qi < -127) qi = -127;
                if (qi > 127) qi = 127;
                blk[2 + t] = (uint8_t)(int8_t)qi;
            }
        }
    }
    return 0;
}

int q8o_repack_split_plane(const uint8_t *gguf, uint64_t rows, uint64_t cols, uint8_t *split) {
    if (cols % Q8O_QK != 0) return -1;
    const uint64_t nb = cols / Q8O_QK;
    const uint64_t row_bytes = nb * Q8O_Q8_0_BYTES;
    for (uint64_t r = 0; r < rows; ++r) {
        const uint8_t *in = gguf + r * row_bytes;
        uint8_t *scales = split + r * row_bytes;
        uint8_t *quants = scales + 2 * nb;
        for (uint64_t b = 0; b < nb; ++b) {
            scales[2 * b] = in[b * 34];
            scales[2 * b + 1] = in[b * 34 + 1];
            memcpy(quants + b * 32, in + b * 34 + 2, 32);
        }
    }
    return 0;
}

static inline float w_scale(const uint8_t *w, uint64_t nb, uint64_t row, uint64_t kb) {
    uint16_t h;
    memcpy(&h, w + row * nb * Q8O_Q8_0_BYTES + 2 * kb, 2);
    return q8o_f16_to_f32(h);
}

static inline const int8_t *w_quants(const uint8_t *w, uint64_t nb, uint64_t row, uint64_t kb) {
    return (const int8_t *)(w + row * nb * Q8O_Q8_0_BYTES + 2 * nb + kb * 32);
}

/* ------------------------------------------------------------------------- */
/* RMS norm (expression: src/kernels_cuda.cu:1995-2007; order of the sum: see header) */

int q8o_rms_norm(const float *x, const float *weight, float *out, uint32_t batch, uint32_t n,
                 uint32_t stride_x_row, uint32_t stride_out_row, float eps) {
    if (n == 0) return -1;
    const uint32_t chunks = (n + 3) / 4;
    for (uint32_t j = 0; j < batch; ++j) {
        const float *row = x + (size_t)j * stride_x_row;
        float partial[256];
        for (uint32_t t = 0; t < 256; ++t) partial[t] = 0.0f;
        for (uint32_t c = 0; c < chunks; ++c) {
            float v[4];
            for (uint32_t e = 0; e < 4; ++e) v[e] = (c * 4 + e < n) ? row[c * 4 + e] : 0.0f;
            const float q = fmaf(v[3], v[3], fmaf(v[2], v[2], fmaf(v[1], v[1], v[0] * v[0])));
            partial[c % 256] = partial[c % 256] + q;
        }
        for (uint32_t w = 1; w < 256; w *= 2)
            for (uint32_t t = 0; t < 256; t += 2 * w) partial[t] = partial[t] + partial[t + w];
        const float scale = 1.0f / sqrtf(partial[0] / (float)n + eps);
        float *o = out + (size_t)j * stride_out_row;
        for (uint32_t i = 0; i < n; ++i) {
            const float xs = row[i] * scale;
            o[i] = xs * weight[i];
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* activation quantizers                                                     */

/* The reference reduces 32 lanes with xor offsets 16, 8, 4, 2, 1
 * (src/cuda_helpers.cuh:44-61); every lane ends with the value of this tree. */
static float butterfly_sum32(const float *x) {
    float a[16], b[8], c[4], e[2];
    for (int i = 0; i < 16; ++i) a[i] = x[i] + x[i + 16];
    for (int i = 0; i < 8; ++i) b[i] = a[i] + a[i + 8];
    for (int i = 0; i < 4; ++i) c[i] = b[i] + b[i + 4];
    for (int i = 0; i < 2; ++i) e[i] = c[i] + c[i + 2];
    return e[0] + e[1];
}

static float amax32(const float *x) {
    float m = fabsf(x[0]);
    for (int i = 1; i < Q8O_QK; ++i) m = fmaxf(m, fabsf(x[i])); /* fmaxf drops NaN operands */
    return m;
}

int q8o_get_row(const uint8_t *w_split, uint64_t row, uint64_t cols, float *out) {
    if (cols % Q8O_QK != 0) return -1;
    const uint64_t nb = cols / Q8O_QK;
    const uint8_t *base = w_split + row * nb * Q8O_Q8_0_BYTES;
    const int8_t *qs = (const int8_t *)(base + 2 * nb);
    for (uint64_t i = 0; i < cols; ++i) {
        uint16_t h;
        memcpy(&h, base + 2 * (i / Q8O_QK), 2);
        out[i] = q8o_f16_to_f32(h) * (float)qs[i];
    }
    return 0;
}

int q8o_quantize_q8_1(const float *x, uint32_t batch, uint32_t cols, uint32_t stride_x_row,
                      uint8_t *y) {
    if (cols % Q8O_QK != 0) return -1;
    const uint32_t nb = cols / Q8O_QK;
    for (uint32_t j = 0; j < batch; ++j) {
        for (uint32_t kb = 0; kb < nb; ++kb) {
            const float *src = x + (uint64_t)j * stride_x_row + (uint64_t)kb * Q8O_QK;
            uint8_t *blk = y + ((uint64_t)j * nb + kb) * Q8O_Q8_1_BYTES;
            const float amax = amax32(src);
            const float sum = butterfly_sum32(src);
            const float d = amax / 127.0f;
            const uint16_t hd = q8o_f32_to_f16(d), hs = q8o_f32_to_f16(sum);
            memcpy(blk, &hd, 2);
            memcpy(blk + 2, &hs, 2);
            for (int t = 0; t < Q8O_QK; ++t) {
                const int32_t q = (amax == 0.0f) ? 0 : float2int_rn(src[t] / d);
                blk[4 + t] = (uint8_t)(int8_t)q;
            }
        }
    }
    return 0;
}

int q8o_quantize_q8_1_d4(const float *x, uint32_t batch, uint32_t cols, uint32_t stride_x_row,
                         uint8_t *y) {
    if (cols % 128 != 0) return -1;
    const uint32_t nsb = cols / 128;
    for (uint32_t j = 0; j < batch; ++j) {
        for (uint32_t sb = 0; sb < nsb; ++sb) {
            uint8_t *blk = y + ((uint64_t)sb * batch + j) * Q8O_D4_BYTES;
            for (int sub = 0; sub < 4; ++sub) {
                const float *src = x + (uint64_t)j * stride_x_row + (uint64_t)sb * 128 + sub * 32;
                const float amax = amax32(src);
                const float d_inv = (amax == 0.0f) ? 0.0f : 127.0f / amax;
                const float d = (amax == 0.0f) ? 0.0f : 1.0f / d_inv;
                memcpy(blk + 4 * sub, &d, 4);
                for (int t = 0; t < 32; ++t) {
                    const int32_t q = (amax == 0.0f) ? 0 : float2int_rn(src[t] * d_inv);
                    blk[16 + sub * 32 + t] = (uint8_t)(int8_t)q;
                }
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* block dots                                                                */

static inline int32_t dot32(const int8_t *a, const int8_t *b) {
    int32_t s = 0;
    for (int t = 0; t < 32; ++t) s += (int32_t)a[t] * (int32_t)b[t];
    return s;
}

static inline const uint8_t *q81_block(const uint8_t *y, uint32_t nb, uint32_t j, uint32_t kb) {
    return y + ((uint64_t)j * nb + kb) * Q8O_Q8_1_BYTES;
}

static inline float q81_scale(const uint8_t *blk) {
    uint16_t h;
    memcpy(&h, blk, 2);
    return q8o_f16_to_f32(h);
}

static inline const uint8_t *d4_block(const uint8_t *y, uint32_t batch, uint32_t j, uint32_t kb) {
    return y + ((uint64_t)(kb / 4) * batch + j) * Q8O_D4_BYTES;
}

int32_t q8o_block_dot(const uint8_t *w, const uint8_t *y, int y_layout, uint32_t cols,
                      uint32_t batch, uint32_t row, uint32_t j, uint32_t kb) {
    const uint32_t nb = cols / Q8O_QK;
    const int8_t *qw = w_quants(w, nb, row, kb);
    const int8_t *qx;
    if (y_layout == 0) {
        qx = (const int8_t *)(q81_block(y, nb, j, kb) + 4);
    } else {
        qx = (const int8_t *)(d4_block(y, batch, j, kb) + 16 + (kb % 4) * 32);
    }
    return dot32(qw, qx);
}

/* ------------------------------------------------------------------------- */
/* GEMV family                                                               */

static inline float gemv_one(const uint8_t *w, const uint8_t *y, uint32_t nb, uint32_t row,
                             uint32_t j) {
    float acc = 0.0f;
    for (uint32_t kb = 0; kb < nb; ++kb) {
        const uint8_t *xb = q81_block(y, nb, j, kb);
        const float d = w_scale(w, nb, row, kb) * q81_scale(xb);
        const int32_t s = dot32(w_quants(w, nb, row, kb), (const int8_t *)(xb + 4));
        acc = fmaf(d, (float)s, acc);
    }
    return acc;
}

/* sum_kb |d_w*d_x*S|: the scale against which reordering error is judged */
static inline float gemv_one_abs(const uint8_t *w, const uint8_t *y, uint32_t nb, uint32_t row,
                                 uint32_t j) {
    double acc = 0.0;
    for (uint32_t kb = 0; kb < nb; ++kb) {
        const uint8_t *xb = q81_block(y, nb, j, kb);
        const float d = w_scale(w, nb, row, kb) * q81_scale(xb);
        const int32_t s = dot32(w_quants(w, nb, row, kb), (const int8_t *)(xb + 4));
        acc += fabs((double)d * (double)s);
    }
    return (float)acc;
}

static int gemv_shape_ok(uint32_t cols, uint32_t batch) {
    return cols % Q8O_QK == 0 && batch >= 1 && batch <= 8;
}

int q8o_gemv(const uint8_t *w, const uint8_t *y, float *dst, uint32_t rows, uint32_t cols,
             uint32_t batch, uint32_t stride_dst_row, int threads) {
    if (!gemv_shape_ok(cols, batch)) return -1;
    const uint32_t nb = cols / Q8O_QK;
    if (threads < 1) threads = 1;
    int64_t r;
#pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
    for (r = 0; r < (int64_t)rows; ++r) {
        for (uint32_t j = 0; j < batch; ++j) {
            dst[(uint64_t)j * stride_dst_row + (uint64_t)r] = gemv_one(w, y, nb, (uint32_t)r, j);
        }
    }
    return 0;
}

int q8o_gemv_abs(const uint8_t *w, const uint8_t *y, float *dst, uint32_t rows, uint32_t cols,
                 uint32_t batch, uint32_t stride_dst_row) {
    if (!gemv_shape_ok(cols, batch)) return -1;
    const uint32_t nb = cols / Q8O_QK;
    int64_t r;   /* rows are independent: tall matrices (a vocabulary) are split over the cores */
#pragma omp parallel for schedule(static) if (rows >= 8192)
    for (r = 0; r < (int64_t)rows; ++r)
        for (uint32_t j = 0; j < batch; ++j)
            dst[(uint64_t)j * stride_dst_row + (uint64_t)r] = gemv_one_abs(w, y, nb, (uint32_t)r, j);
    return 0;
}

int q8o_gemv_bf16(const uint8_t *w, const uint8_t *y, uint16_t *dst, uint32_t rows,
                  uint32_t cols, uint32_t batch, uint32_t stride_dst_row) {
    if (!gemv_shape_ok(cols, batch)) return -1;
    const uint32_t nb = cols / Q8O_QK;
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t j = 0; j < batch; ++j)
            dst[(uint64_t)j * stride_dst_row + r] = q8o_f32_to_bf16(gemv_one(w, y, nb, r, j));
    return 0;
}

int q8o_gemv_two(const uint8_t *w0, const uint8_t *w1, const uint8_t *y, float *dst0, float *dst1,
                 uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride_dst_row) {
    if (!gemv_shape_ok(cols, batch)) return -1;
    const uint32_t nb = cols / Q8O_QK;
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t j = 0; j < batch; ++j) {
            dst0[(uint64_t)j * stride_dst_row + r] = gemv_one(w0, y, nb, r, j);
            dst1[(uint64_t)j * stride_dst_row + r] = gemv_one(w1, y, nb, r, j);
        }
    return 0;
}

int q8o_gemv_silu_mul(const uint8_t *wg, const uint8_t *wu, const uint8_t *y, float *dst,
                      uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride_dst_row) {
    if (!gemv_shape_ok(cols, batch)) return -1;
    const uint32_t nb = cols / Q8O_QK;
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t j = 0; j < batch; ++j) {
            const float g = gemv_one(wg, y, nb, r, j);
            const float u = gemv_one(wu, y, nb, r, j);
            const float silu = g / (1.0f + expf(-g));
            dst[(uint64_t)j * stride_dst_row + r] = silu * u;
        }
    return 0;
}

int q8o_gemv_add(const uint8_t *w, const uint8_t *y, float *dst, uint32_t rows, uint32_t cols,
                 uint32_t batch, uint32_t stride_dst_row) {
    if (!gemv_shape_ok(cols, batch)) return -1;
    const uint32_t nb = cols / Q8O_QK;
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t j = 0; j < batch; ++j) {
            float *p = dst + (uint64_t)j * stride_dst_row + r;
            *p = *p + gemv_one(w, y, nb, r, j);
        }
    return 0;
}

int q8o_gemv_add_bf16(const uint8_t *w, const uint8_t *y, uint16_t *dst, uint32_t rows,
                      uint32_t cols, uint32_t batch, uint32_t stride_dst_row) {
    if (!gemv_shape_ok(cols, batch)) return -1;
    const uint32_t nb = cols / Q8O_QK;
    for (uint32_t r = 0; r < rows; ++r)
        for (uint32_t j = 0; j < batch; ++j) {
            uint16_t *p = dst + (uint64_t)j * stride_dst_row + r;
            *p = q8o_f32_to_bf16(q8o_bf16_to_f32(*p) + gemv_one(w, y, nb, r, j));
        }
    return 0;
}

int q8o_gemv_fanout4(const uint8_t *const w[4], const uint8_t *y, float *const dst[4],
                     const uint32_t rows[4], uint32_t cols, uint32_t batch,
                     const uint32_t stride_dst[4]) {
    if (!gemv_shape_ok(cols, batch)) return -1;
    const uint64_t total = (uint64_t)rows[0] + rows[1] + rows[2] + rows[3];
    if (total == 0 || total > 0xffffffffull) return -1;
    const uint32_t nb = cols / Q8O_QK;
    for (int s = 0; s < 4; ++s) {
        if (w[s] == NULL || dst[s] == NULL) continue;
        for (uint32_t r = 0; r < rows[s]; ++r)
            for (uint32_t j = 0; j < batch; ++j)
                dst[s][(uint64_t)j * stride_dst[s] + r] = gemv_one(w[s], y, nb, r, j);
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* GEMM with D4 activations                                                  */

static inline float gemm_d4_one(const uint8_t *w, const uint8_t *y, uint32_t nb, uint32_t batch,
                                uint32_t row, uint32_t j) {
    float acc = 0.0f;
    for (uint32_t kb = 0; kb < nb; ++kb) {
        const uint8_t *blk = d4_block(y, batch, j, kb);
        float dy;
        memcpy(&dy, blk + 4 * (kb % 4), 4);
        const float d = w_scale(w, nb, row, kb) * dy;
        const int32_t s =
            dot32(w_quants(w, nb, row, kb), (const int8_t *)(blk + 16 + (kb % 4) * 32));
        acc = fmaf(d, (float)s, acc);
    }
    return acc;
}

static inline float gemm_d4_one_abs(const uint8_t *w, const uint8_t *y, uint32_t nb,
                                    uint32_t batch, uint32_t row, uint32_t j) {
    double acc = 0.0;
    for (uint32_t kb = 0; kb < nb; ++kb) {
        const uint8_t *blk = d4_block(y, batch, j, kb);
        float dy;
        memcpy(&dy, blk + 4 * (kb % 4), 4);
        const float d = w_scale(w, nb, row, kb) * dy;
        const int32_t s =
            dot32(w_quants(w, nb, row, kb), (const int8_t *)(blk + 16 + (kb % 4) * 32));
        acc += fabs((double)d * (double)s);
    }
    return (float)acc;
}

int q8o_gemm_d4(const uint8_t *w, const uint8_t *y, float *dst, uint32_t rows, uint32_t cols,
                uint32_t batch, uint32_t stride_dst_row, int threads) {
    if (cols % 128 != 0 || rows == 0 || batch == 0) return -1;
    const uint32_t nb = cols / Q8O_QK;
    if (threads < 1) threads = 1;
    int64_t r;
#pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
    for (r = 0; r < (int64_t)rows; ++r) {
        for (uint32_t j = 0; j < batch; ++j) {
            dst[(uint64_t)j * stride_dst_row + (uint64_t)r] =
                gemm_d4_one(w, y, nb, batch, (uint32_t)r, j);
        }
    }
    return 0;
}

int q8o_gemm_d4_sampled(const uint8_t *w, const uint8_t *y, uint32_t rows, uint32_t cols,
                        uint32_t batch, const uint32_t *rows_idx, const uint32_t *js_idx,
                        uint32_t n, float *out, float *out_abs) {
    if (cols % 128 != 0 || rows == 0 || batch == 0) return -1;
    const uint32_t nb = cols / Q8O_QK;
    for (uint32_t i = 0; i < n; ++i) {
        if (rows_idx[i] >= rows || js_idx[i] >= batch) return -1;
        out[i] = gemm_d4_one(w, y, nb, batch, rows_idx[i], js_idx[i]);
        if (out_abs) out_abs[i] = gemm_d4_one_abs(w, y, nb, batch, rows_idx[i], js_idx[i]);
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* argmax + accept                                                           */

q8o_argmax_pair q8o_argmax_row(const float *x, uint64_t n) {
    q8o_argmax_pair best = {-INFINITY, -1};
    for (uint64_t i = 0; i < n; ++i) {
        if (x[i] > best.value) {
            best.value = x[i];
            best.index = (int32_t)i;
        }
    }
    return best;
}

/* src/kernels_cuda.cu:1765-1771 */
static int pair_better(float v, int32_t i, float bv, int32_t bi) {
    if (i < 0) return 0;
    if (bi < 0) return 1;
    if (v > bv) return 1;
    return v == bv && i < bi;
}

static q8o_argmax_pair tree_reduce(float *vals, int32_t *idx, uint32_t width) {
    for (uint32_t stride = width / 2; stride > 0; stride >>= 1) {
        for (uint32_t t = 0; t < stride; ++t) {
            if (pair_better(vals[t + stride], idx[t + stride], vals[t], idx[t])) {
                vals[t] = vals[t + stride];
                idx[t] = idx[t + stride];
            }
        }
    }
    q8o_argmax_pair r = {vals[0], idx[0]};
    return r;
}

int q8o_argmax_rows(const float *x, uint32_t batch, uint32_t row_stride, q8o_argmax_pair *out) {
    const uint32_t bpr = (row_stride + 255u) / 256u;
    if (row_stride == 0 || bpr > 1024u) return -1;
    float vals[1024];
    int32_t idx[1024];
    q8o_argmax_pair *partial = (q8o_argmax_pair *)malloc((size_t)bpr * sizeof(*partial));
    if (!partial) return -1;
    for (uint32_t row = 0; row < batch; ++row) {
        const float *base = x + (uint64_t)row * row_stride;
        for (uint32_t b = 0; b < bpr; ++b) {
            for (uint32_t t = 0; t < 256; ++t) {
                const uint32_t col = b * 256u + t;
                vals[t] = col < row_stride ? base[col] : -INFINITY;
                idx[t] = col < row_stride ? (int32_t)col : -1;
            }
            partial[b] = tree_reduce(vals, idx, 256);
        }
        for (uint32_t t = 0; t < 1024; ++t) {
            vals[t] = t < bpr ? partial[t].value : -INFINITY;
            idx[t] = t < bpr ? partial[t].index : -1;
        }
        out[row] = tree_reduce(vals, idx, 1024);
    }
    free(partial);
    return 0;
}

void q8o_argmax_rows_scan(const float *x, uint32_t batch, uint32_t row_stride,
                          q8o_argmax_pair *out) {
    for (uint32_t row = 0; row < batch; ++row) {
        q8o_argmax_pair best = {-INFINITY, -1};
        const float *base = x + (uint64_t)row * row_stride;
        for (uint32_t c = 0; c < row_stride; ++c) {
            if (base[c] > best.value) {
                best.value = base[c];
                best.index = (int32_t)c;
            }
        }
        out[row] = best;
    }
}

uint32_t q8o_accept(const int32_t *row_tokens, const int32_t *drafts, uint32_t n_drafts,
                    int32_t eos, int32_t *next_token) {
    uint32_t accepted = 0;
    for (uint32_t i = 0; i < n_drafts; ++i) {
        const int32_t target = row_tokens[i] >= 0 ? row_tokens[i] : eos;
        if (target != drafts[i]) break;
        ++accepted;
    }
    if (next_token) {
        const int32_t t = row_tokens[accepted];
        *next_token = t >= 0 ? t : eos;
    }
    return accepted;
}
