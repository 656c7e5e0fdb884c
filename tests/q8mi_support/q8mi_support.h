/*
 * q8mi_support.h — instruments for the tests and the bench of the Q8_0 x Q8_1 library.
 *
 * Nothing here is part of the product ABI (include/q8mi.h) and libq8mi.so exports none of it:
 * this header belongs to libq8mi_support.so, which only tests/ and bench.py load.  It holds the
 * seeded input generators, a checker kernel for int32 block dots, and the plain read / copy /
 * matrix-unit kernels that measured ceilings come from.  None has a counterpart in the reference.
 * Return value: 0 = ok, 1 = rejected, 2 = HIP launch error (text via q8sup_last_error()).
 */
#ifndef Q8MI_SUPPORT_H
#define Q8MI_SUPPORT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char *q8sup_last_error(void);

/* ---- synthetic inputs (host side) ------------------------------------------
 * Counter-based generator: element i of stream `seed` depends only on (seed, i), so any thread
 * split gives the same bytes.
 *   kind 0: N(0,1) * scale
 *   kind 1: Student-t(nu=3)/sqrt(3) * scale, with every column whose hash (seed, col) falls in
 *           the lowest `outlier_ppm` millionths multiplied by outlier_gain.
 * out: host fp32 [rows][cols]. */
int q8sup_synth_f32(float *out, uint64_t rows, uint64_t cols, uint64_t seed, int kind, float scale,
                    uint32_t outlier_ppm, float outlier_gain, int threads);
/* N(0, sigma^2) weights quantized to Q8_0 (the rule of the reference's parity test,
 * tests/mmq_parity.cu:54-80: d = amax/127 stored fp16, q = clamp(lrintf(w * (1/d)), +-127)) and
 * written straight into split-plane rows.  out: host, rows*cols/32*34 bytes. */
int q8sup_synth_q8_0_weight(uint8_t *split_out, uint64_t rows, uint64_t cols, uint64_t seed, float sigma,
                            int threads);

/* ---- checker: int32 block dots ----------------------------------------------
 * S[row][j][kb] = sum_t q_w * q_x for n sampled (row, j, kb) triples, computed on the GPU with
 * the int8 dot instruction.  y_layout: 0 = Q8_1 (36-B blocks), 1 = D4 (144-B super-blocks).
 * The sample arrays and out are device pointers. */
int q8sup_block_dots(const uint8_t *weight, const void *y, int y_layout, uint32_t rows, uint32_t cols,
                     uint32_t batch, const uint32_t *sample_row, const uint32_t *sample_j,
                     const uint32_t *sample_kb, uint32_t n, int32_t *out, void *stream);

/* ---- measured ceilings -------------------------------------------------------
 * Plain streaming read of `bytes` device bytes (16-byte streaming loads, grid-stride,
 * wgs_per_cu workgroups of 256 per CU).  sink: one device uint32 (never written in practice). */
int q8sup_probe_read(const void *buf, uint64_t bytes, uint32_t wgs_per_cu, uint32_t *sink, void *stream);
/* Plain device-to-device copy by a kernel (reads `bytes`, writes `bytes`): the known-size launch
 * that hardware memory-traffic counters are calibrated against. */
int q8sup_probe_copy(const void *src, void *dst, uint64_t bytes, void *stream);
/* Matrix-unit issue rates: two workgroups of four waves per CU, every wave running `iters`
 * rounds of the arithmetic one wave of a 128 x 128 GEMM tile spends on one 32-element block
 * (four 32 x 32 output patches), nothing else (no loads, no LDS).
 *   mode 0  four v_mfma_i32_32x32x32_i8
 *   mode 1  the same plus 128 scalar fp32 FMAs (2 per int32 sum: the rescale of the int8 kernel)
 *   mode 2  block sums as fp32 from the fp16 matrix unit (eight v_mfma_f32_32x32x16_f16), the
 *           scale products d_w * d_y as outer products on the fp32 matrix unit (sixteen
 *           v_mfma_f32_4x4x1_16b_f32) and 64 scalar fp32 FMAs (1 per sum)
 * *ops_out (host) receives the int8-equivalent operations launched, 2 * 32^3 * 4 * iters per
 * wave; the caller times the launch.  sink: q8sup_probe_mfma_sink_bytes() device bytes. */
int q8sup_probe_mfma(int mode, uint32_t iters, int32_t *sink, uint64_t *ops_out, void *stream);
size_t q8sup_probe_mfma_sink_bytes(void);

#ifdef __cplusplus
}
#endif
#endif /* Q8MI_SUPPORT_H */
