/*
 * q8_oracle.h — CPU restatement of qw3's Q8_0 x Q8_1 quantized-linear path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the HIP library, its host
 * layer, the bench's measured leg) may call into this file; it exists so the
 * GPU kernels can be checked against a plain, scalar statement of the
 * reference's arithmetic, and so the same scalar code can be timed as the CPU
 * baseline.
 *
 * Each function names the reference lines it restates (paths relative to the
 * reference checkout).  All buffers are caller-owned host memory.  Functions
 * returning int use 0 = ok, -1 = shape rejected (nothing written), mirroring
 * the `false` the reference launchers return for the same shapes.
 *
 * Pinning status (how each function is held in place without running the
 * reference, which needs nvcc and an NVIDIA GPU):
 *   fp16/bf16 conversions ....... exhaustive vs numpy.float16 / bit tricks
 *   q8o_quantize_q8_0 ........... independent numpy restatement, invariants
 *   q8o_repack_split_plane ...... byte-level numpy restatement, round trip
 *   q8o_quantize_q8_1 / _d4 ..... independent numpy restatement, closed forms
 *   q8o_get_row ................. numpy restatement (d * q is exact in fp32)
 *   q8o_rms_norm ................ float64 truth within 4 ulp, closed forms
 *                                 (constant rows, unit weights, scaling law),
 *                                 independent numpy restatement of the order
 *   q8o_block_dot ............... int64 brute force, extreme values
 *   q8o_gemv*, q8o_gemm_d4 ...... reference closed form (cols*0.5*x), reference
 *                                 tolerance test restated (5e-3 abs / 1e-3 rel
 *                                 against dequantised fp32 dot), fp64 truth
 *   q8o_gemv_silu_mul ........... composition of q8o_gemv + float64 silu
 *   q8o_argmax_* ................ textbook scan; adversarial ties/-inf/NaN rows
 *   q8o_accept .................. brute force over all (M, prefix) pairs
 * Parity unpinned (needs the reference's GPU): the last-bit value of the
 * reference's own fp32 reduction tree and of `__expf`; both lie inside the
 * 1e-5 relative tolerance the GPU tests use.  q8o_rms_norm: parity unpinned
 * against the reference's bits for the same reason (its sum of squares
 * follows its block size and nvcc's contraction, its root is the GPU's
 * approximate rsqrtf): the function fixes an order and IEEE operations of
 * its own and is pinned against the mathematics only.
 */
#ifndef Q8_ORACLE_H
#define Q8_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define Q8O_QK 32            /* elements per Q8_0 / Q8_1 block  (src/mmvq_q8.cu:41-42) */
#define Q8O_Q8_0_BYTES 34    /* fp16 d + 32 int8                (src/cuda_helpers.cuh:16-25) */
#define Q8O_Q8_1_BYTES 36    /* half2{d,s} + 32 int8            (src/mmvq_q8.cu:48-52) */
#define Q8O_D4_BYTES 144     /* float d4[4] + 128 int8          (src/mmvq_q8.cu:60-64) */

/* {value, index} as written on device by the reference's argmax kernels
 * (src/kernels_cuda.cu:1741-1744). */
typedef struct {
    float value;
    int32_t index;
} q8o_argmax_pair;

/* ---- scalar conversions -------------------------------------------------- */
uint16_t q8o_f32_to_f16(float f);          /* round-to-nearest-even, overflow -> inf */
float q8o_f16_to_f32(uint16_t h);          /* src/kernels_cuda.cu:1340-1365 */
uint16_t q8o_f32_to_bf16(float f);         /* RNE; NaN -> 0x7fff */
float q8o_bf16_to_f32(uint16_t h);

/* ---- weights ------------------------------------------------------------- */
/* fp32 [rows][cols] -> interleaved GGUF Q8_0 blocks (34 B each).
 * tests/mmq_parity.cu:54-80: d = amax/127, d_inv = d==0 ? 0 : 1/d,
 * q = clamp(lrintf(w*d_inv), -127, 127), d stored as fp16. */
int q8o_quantize_q8_0(const float *w, uint64_t rows, uint64_t cols, uint8_t *gguf_blocks);

/* Interleaved 34-B blocks -> split-plane rows [fp16 d x nb][int8 q x 32 nb].
 * src/kernels_cuda.cu:1566-1594. */
int q8o_repack_split_plane(const uint8_t *gguf_blocks, uint64_t rows, uint64_t cols,
                           uint8_t *split);

/* Dequantized row `row` of a split-plane weight: out[i] = fp32(d[i / 32]) * (float)q[i]
 * (exact: an fp16 value times an 8-bit integer).  src/kernels_cuda.cu:2075-2087. */
int q8o_get_row(const uint8_t *w_split, uint64_t row, uint64_t cols, float *out);

/* ---- RMS norm --------------------------------------------------------------- */
/* out[i] = (x[i] * scale) * weight[i], scale = 1 / sqrtf(sum_i x[i]^2 / n + eps): the
 * expression of src/kernels_cuda.cu:1995-2007 (and :2070-2072) with an IEEE root and
 * quotient in place of rsqrtf, and with this order for the sum of squares (the
 * reference's, :1966-1992, follows its block size): the row is cut into chunks of
 * four floats (the last one zero-padded); partial t of 256 adds, in ascending order,
 * fmaf(w,w, fmaf(z,z, fmaf(y,y, x*x))) of chunks t, t+256, ...; the partials are added
 * as a balanced binary tree, neighbours first.  batch rows, stride_x / stride_out
 * floats apart. */
int q8o_rms_norm(const float *x, const float *weight, float *out, uint32_t batch, uint32_t n,
                 uint32_t stride_x_row, uint32_t stride_out_row, float eps);

/* ---- activation quantizers ----------------------------------------------- */
/* src/mmvq_q8.cu:82-112, 623-640.  y: batch * (cols/32) blocks of 36 B. */
int q8o_quantize_q8_1(const float *x, uint32_t batch, uint32_t cols, uint32_t stride_x_row,
                      uint8_t *y);
/* src/mmvq_q8.cu:668-722, 736-755.  y: (cols/128) * batch blocks of 144 B,
 * block index = (k/128)*batch + j. */
int q8o_quantize_q8_1_d4(const float *x, uint32_t batch, uint32_t cols, uint32_t stride_x_row,
                         uint8_t *y);

/* ---- int32 block dots ---------------------------------------------------- */
/* S = sum_{t<32} q_w[row][kb][t] * q_x[j][kb][t]; layout: 0 = Q8_1 (36 B),
 * 1 = D4 (144 B).  src/mmvq_q8.cu:157-172, src/mmq_q8.cu:2235-2242. */
int32_t q8o_block_dot(const uint8_t *w_split, const uint8_t *y, int y_layout, uint32_t cols,
                      uint32_t batch, uint32_t row, uint32_t j, uint32_t kb);

/* ---- GEMV family (Q8_1 activations, batch 1..8) -------------------------- */
/* dst[j*stride_dst_row + r] = sum_kb fma(d_w*d_x, (float)S, acc), ascending kb.
 * src/mmvq_q8.cu:193-280, 764-819.  `threads` > 1 splits rows over OpenMP threads. */
int q8o_gemv(const uint8_t *w, const uint8_t *y, float *dst, uint32_t rows, uint32_t cols,
             uint32_t batch, uint32_t stride_dst_row, int threads);
/* dst = sum_kb |d_w*d_x*S| (fp64 accumulate): the magnitude that a test's
 * reordering allowance is taken from; not part of the reference. */
int q8o_gemv_abs(const uint8_t *w, const uint8_t *y, float *dst, uint32_t rows, uint32_t cols,
                 uint32_t batch, uint32_t stride_dst_row);
int q8o_gemv_bf16(const uint8_t *w, const uint8_t *y, uint16_t *dst, uint32_t rows,
                  uint32_t cols, uint32_t batch, uint32_t stride_dst_row);
/* src/mmvq_q8.cu:295-399, 823-864 */
int q8o_gemv_two(const uint8_t *w0, const uint8_t *w1, const uint8_t *y, float *dst0, float *dst1,
                 uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride_dst_row);
/* src/mmvq_q8.cu:414-519, 869-909: silu(g)*u with silu(g) = g / (1 + exp(-g)) */
int q8o_gemv_silu_mul(const uint8_t *wg, const uint8_t *wu, const uint8_t *y, float *dst,
                      uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride_dst_row);
/* src/mmvq_q8.cu:528-606, 914-969: dst += W x  (bf16: RNE of the fp32 sum, :183-191) */
int q8o_gemv_add(const uint8_t *w, const uint8_t *y, float *dst, uint32_t rows, uint32_t cols,
                 uint32_t batch, uint32_t stride_dst_row);
int q8o_gemv_add_bf16(const uint8_t *w, const uint8_t *y, uint16_t *dst, uint32_t rows,
                      uint32_t cols, uint32_t batch, uint32_t stride_dst_row);
/* src/mmvq_q8.cu:976-1113: up to four weights sharing one activation; a slot
 * with a null weight, null dst or zero rows is skipped. */
int q8o_gemv_fanout4(const uint8_t *const w[4], const uint8_t *y, float *const dst[4],
                     const uint32_t rows[4], uint32_t cols, uint32_t batch,
                     const uint32_t stride_dst[4]);

/* ---- GEMM (D4 activations) ----------------------------------------------- */
/* src/mmq_q8.cu:2164-2273, 2278-2288: dst[j*stride + r] = sum_kb
 * fma(d_w*d_y, (float)S, acc), one int32 S per 32-block, ascending kb.
 * Rejects cols%128, rows==0, batch==0. */
int q8o_gemm_d4(const uint8_t *w, const uint8_t *y_d4, float *dst, uint32_t rows, uint32_t cols,
                uint32_t batch, uint32_t stride_dst_row, int threads);
/* Same result for a subset of outputs: n samples (rows_idx[i], js_idx[i]);
 * out_abs (optional) receives sum_kb |d_w*d_y*S| for each sample. */
int q8o_gemm_d4_sampled(const uint8_t *w, const uint8_t *y_d4, uint32_t rows, uint32_t cols,
                        uint32_t batch, const uint32_t *rows_idx, const uint32_t *js_idx,
                        uint32_t n, float *out, float *out_abs);

/* ---- argmax + greedy accept ---------------------------------------------- */
/* src/kernels_cuda.cu:1693-1734 (and :1804-1857): 1024 strided scanners, max by
 * `>`, ties -> lowest index, no element above -inf -> {-inf, -1}. */
q8o_argmax_pair q8o_argmax_row(const float *x, uint64_t n);
/* src/kernels_cuda.cu:1765-1802, 1859-1888, 20814-20850: two-stage batched
 * argmax (256-wide tree per block, then a 1024-wide tree over the partials),
 * restated comparison by comparison so NaN rows agree too.  Returns -1 when the
 * reference would take its host fallback (row_stride==0 or >1024 partials). */
int q8o_argmax_rows(const float *x, uint32_t batch, uint32_t row_stride, q8o_argmax_pair *out);
/* Host fallback of the same call: include/qw3/device_backend.hpp:2477-2497. */
void q8o_argmax_rows_scan(const float *x, uint32_t batch, uint32_t row_stride,
                          q8o_argmax_pair *out);
/* src/qwen_native_backend.cpp:15948-15960, 16048-16052: number of leading
 * drafts equal to (token>=0 ? token : eos); *next_token = row `accepted`. */
uint32_t q8o_accept(const int32_t *row_tokens, const int32_t *drafts, uint32_t n_drafts,
                    int32_t eos, int32_t *next_token);

#ifdef __cplusplus
}
#endif
#endif /* Q8_ORACLE_H */
