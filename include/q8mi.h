/*
 * q8mi.h — C ABI of the MI355X (gfx950) Q8_0 x Q8_1 quantized-linear library.
 *
 * This is the drop-in boundary for qw3's Q8_0 linear hot path: every entry
 * point below replaces one `qw3::ported::launch_*` launcher (declared by the
 * reference at src/kernels_cuda.cu:56-125) or one of the argmax kernels the
 * reference's CUDA backend launches itself.  Paths in comments are relative to
 * the reference checkout.
 *
 * Conventions
 *   - All data pointers are caller-owned DEVICE pointers unless a parameter is
 *     documented as host memory.  Nothing here allocates, frees or synchronises
 *     (src/mmvq_q8.cu:19-22); work is enqueued on `stream` (a hipStream_t passed
 *     as void*, NULL = the default stream) and is capturable into a HIP graph.
 *   - Return value: Q8MI_OK, Q8MI_REJECTED (the reference launcher would have
 *     returned false: nothing was enqueued) or Q8MI_LAUNCH_ERROR (the HIP
 *     runtime reported an error; text via q8mi_last_error()).
 *   - Weights use the reference's split-plane row layout
 *     (src/cuda_helpers.cuh:16-39): row r starts at r*nb*34 bytes and holds
 *     nb fp16 scales followed by nb*32 int8 quants, nb = cols/32.
 *   - Activations are Q8_1 blocks of 36 B (src/mmvq_q8.cu:48-52) for the GEMV
 *     family, or 144-B D4 super-blocks (src/mmvq_q8.cu:60-64) with block index
 *     (k/128)*batch + j for the MFMA GEMM.
 *   - Outputs are [batch][stride_dst_row]; element (j, r) lives at
 *     j*stride_dst_row + r.
 */
#ifndef Q8MI_H
#define Q8MI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define Q8MI_OK 0
#define Q8MI_REJECTED 1
#define Q8MI_LAUNCH_ERROR 2

#define Q8MI_MAX_GEMV_BATCH 8

/* Device-visible argmax record; byte-identical to the reference's ArgmaxPair
 * (src/kernels_cuda.cu:1741-1744), which its device-chained MTP draft loop
 * reads on the GPU (src/kernels_cuda.cu:2110-2133). */
typedef struct q8mi_argmax_pair {
    float value;
    int32_t index;
} q8mi_argmax_pair;

/* Thread-local text of the last Q8MI_LAUNCH_ERROR / Q8MI_REJECTED on this thread. */
const char *q8mi_last_error(void);
/* Library ABI version (bumped on any signature change). */
int q8mi_abi_version(void);

/* ---- Q8_1 activation quantizer ------------------------------------------- */
/* replaces q8_1_scratch_bytes, src/mmvq_q8.cu:613-616 */
size_t q8mi_q8_1_scratch_bytes(uint32_t batch, uint32_t cols);
/* replaces launch_quantize_q8_1, src/mmvq_q8.cu:623-640 (kernel :82-112).
 * Rejects cols % 32 != 0. */
int q8mi_quantize_q8_1(const float *x, void *y_q8_1, uint32_t batch, uint32_t cols,
                       uint32_t stride_x_row, void *stream);

/* ---- GEMV family, batch 1..8 --------------------------------------------- */
/* replaces launch_mmvq_q8_0, src/mmvq_q8.cu:805-811.  Rejects cols % 32 != 0,
 * batch == 0, batch > 8 (src/mmvq_q8.cu:773-774). */
int q8mi_gemv(const uint8_t *weight, const void *y_q8_1, float *dst, uint32_t rows, uint32_t cols,
              uint32_t batch, uint32_t stride_dst_row, void *stream);
/* replaces launch_mmvq_q8_0_bf16, src/mmvq_q8.cu:813-819 (dst is bf16 bits) */
int q8mi_gemv_bf16(const uint8_t *weight, const void *y_q8_1, uint16_t *dst, uint32_t rows,
                   uint32_t cols, uint32_t batch, uint32_t stride_dst_row, void *stream);
/* replaces launch_mmvq_q8_0_two, src/mmvq_q8.cu:823-864 */
int q8mi_gemv_two(const uint8_t *weight0, const uint8_t *weight1, const void *y_q8_1, float *dst0,
                  float *dst1, uint32_t rows, uint32_t cols, uint32_t batch,
                  uint32_t stride_dst_row, void *stream);
/* replaces launch_mmvq_q8_0_silu_mul, src/mmvq_q8.cu:869-909:
 * dst = silu(Wg x) * (Wu x), silu(g) = g / (1 + exp(-g)) */
int q8mi_gemv_silu_mul(const uint8_t *weight_gate, const uint8_t *weight_up, const void *y_q8_1,
                       float *dst, uint32_t rows, uint32_t cols, uint32_t batch,
                       uint32_t stride_dst_row, void *stream);
/* replaces launch_mmvq_q8_0_add, src/mmvq_q8.cu:955-961: dst += W x */
int q8mi_gemv_add(const uint8_t *weight, const void *y_q8_1, float *dst, uint32_t rows,
                  uint32_t cols, uint32_t batch, uint32_t stride_dst_row, void *stream);
/* replaces launch_mmvq_q8_0_add_bf16, src/mmvq_q8.cu:963-969 */
int q8mi_gemv_add_bf16(const uint8_t *weight, const void *y_q8_1, uint16_t *dst, uint32_t rows,
                       uint32_t cols, uint32_t batch, uint32_t stride_dst_row, void *stream);
/* replaces launch_mmvq_q8_0_fanout4_batch, src/mmvq_q8.cu:1070-1113.  A slot
 * with a NULL weight, NULL dst or zero rows is skipped; rejects a total of
 * zero rows. */
int q8mi_gemv_fanout4(const uint8_t *weight0, const uint8_t *weight1, const uint8_t *weight2,
                      const uint8_t *weight3, const void *y_q8_1, float *dst0, float *dst1,
                      float *dst2, float *dst3, uint32_t rows0, uint32_t rows1, uint32_t rows2,
                      uint32_t rows3, uint32_t cols, uint32_t batch, uint32_t stride_dst0,
                      uint32_t stride_dst1, uint32_t stride_dst2, uint32_t stride_dst3,
                      void *stream);

/* ---- GEMV with the Q8_1 quantizer fused in (batch 1..2) --------------------
 * The results of q8mi_quantize_q8_1 followed by the matching q8mi_gemv* call,
 * in one launch: every workgroup quantizes the fp32 activations
 * (x: [batch][stride_x_row] floats) itself with the quantizer's own arithmetic
 * behind its first weight requests (rows of 1024, 2048, ... 8192 columns:
 * each wave the 1024 columns it works on, in registers; other lengths: into
 * LDS), so no Q8_1 scratch buffer and no quantizer launch are needed.  The
 * quantized values and the per-block products are the same bits as in the
 * two-step form.  So are the outputs at batch 1 for rows of up to 8192 columns
 * and at batch 2 for those whole numbers of 1024 columns; longer rows, and other lengths
 * at batch 2 (where the Q8_1 entry points may run another kernel), add the same
 * products in another order (inside the GEMV's tolerance).  This is what
 * the reference's operators do in two steps (src/kernels_cuda.cu:10764-10888,
 * 11244-11302, 12035-12069, 12227-12258: launch_quantize_q8_1 then the
 * launcher); the fusion itself has no counterpart in the reference.
 * Q8MI_REJECTED (nothing launched; use the two-step form) when batch is above
 * 2 (every workgroup repeats the quantization, which stops paying there) or
 * cols is not a multiple of 256.  dst_is_bf16: 0 = fp32 outputs, 1 = bf16 bit patterns. */
int q8mi_qgemv(const uint8_t *weight, const float *x, uint32_t stride_x_row, void *dst, int dst_is_bf16,
               uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride_dst_row, void *stream);
int q8mi_qgemv_add(const uint8_t *weight, const float *x, uint32_t stride_x_row, void *dst, int dst_is_bf16,
                   uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride_dst_row, void *stream);
int q8mi_qgemv_silu_mul(const uint8_t *weight_gate, const uint8_t *weight_up, const float *x,
                        uint32_t stride_x_row, float *dst, uint32_t rows, uint32_t cols, uint32_t batch,
                        uint32_t stride_dst_row, void *stream);
int q8mi_qgemv_fanout4(const uint8_t *weight0, const uint8_t *weight1, const uint8_t *weight2,
                       const uint8_t *weight3, const float *x, uint32_t stride_x_row, float *dst0, float *dst1,
                       float *dst2, float *dst3, uint32_t rows0, uint32_t rows1, uint32_t rows2, uint32_t rows3,
                       uint32_t cols, uint32_t batch, uint32_t stride_dst0, uint32_t stride_dst1,
                       uint32_t stride_dst2, uint32_t stride_dst3, void *stream);

/* ---- RMS norm in front of the quantizer ------------------------------------
 * out[j][i] = (x[j][i] * scale_j) * weight[i], scale_j = 1 / sqrt(mean_i x[j][i]^2 + eps):
 * replaces rms_norm_kernel_vec / rms_norm_kernel (src/kernels_cuda.cu:1945-2010,
 * 2057-2073) as launched by rms_norm and rms_norm_batch (:14748-14816); rows of x
 * are stride_x_row floats apart (the reference's are dense, stride = cols).  Any
 * cols and alignment (16-byte aligned pointers and strides that are multiples of 4
 * take vector loads).  The reference's sum of squares follows its block size and its
 * root is the GPU's approximate rsqrtf, so its last bits are not restated: this
 * kernel sums in a fixed order (256 strided partials of 4-float chunks, then a
 * balanced tree) and takes an IEEE root and quotient, which a CPU follows bit for
 * bit; against the reference that is a difference of a few units in the last place. */
int q8mi_rms_norm(const float *x, const float *weight, float *out, uint32_t batch, uint32_t cols,
                  uint32_t stride_x_row, uint32_t stride_out_row, float eps, void *stream);
/* q8mi_rms_norm followed by q8mi_quantize_q8_1 of its output, in one pass over x
 * (same bits as the two calls): the step between the executor's rms_norm and
 * launch_quantize_q8_1 inside every q8_0_matvec* / q8_0_matmul* operator
 * (src/kernels_cuda.cu:11250, 12047, 12241).  `normalized` (rows
 * stride_normalized_row floats apart) also receives the fp32 rows unless NULL.
 * Rejects cols % 32 != 0. */
int q8mi_rms_norm_quantize_q8_1(const float *x, const float *weight, float *normalized, void *y_q8_1,
                                uint32_t batch, uint32_t cols, uint32_t stride_x_row,
                                uint32_t stride_normalized_row, float eps, void *stream);
/* The residual add in front of a norm, in the norm's launch: sum = a + b (rounded as q8mi_add
 * rounds it; sum may be a or b), then normalized / y_q8_1 = what q8mi_rms_norm /
 * q8mi_rms_norm_quantize_q8_1 give on sum, bit for bit.  Replaces the pair add_n + rms_norm_batch
 * of the batched layer loop (src/qwen_executor.cpp:6642-6645 with 6666-6668, and the add_n at
 * :6693 with the next layer's norm; kernels src/kernels_cuda.cu:14818-14862, 14781-14816).  Rows
 * of a, b and sum are stride_row floats apart.  normalized may be NULL when y_q8_1 is given and
 * the other way round; it must not overlap a, b or sum.  y_q8_1 needs cols % 32 == 0. */
int q8mi_add_rms_norm(const float *a, const float *b, float *sum, const float *weight, float *normalized,
                      void *y_q8_1, uint32_t batch, uint32_t cols, uint32_t stride_row,
                      uint32_t stride_normalized_row, float eps, void *stream);
/* One activation row normalised, quantized and multiplied in ONE launch: what
 * rms_norm_q8_0_matmul_fanout (include/qw3/device_backend.hpp:421-444) and the
 * rms_norm + q8_0_matvec / q8_0_matvec_silu_mul pairs of the decode loop
 * (src/qwen_executor.cpp:5734-5792) do in three.  Every workgroup repeats the norm
 * and the quantization on its own copy of the row while its first weight bytes are
 * in flight; workgroup 0 also writes the fp32 row to `normalized` unless NULL.  The
 * outputs are the bits of q8mi_rms_norm followed by the matching q8mi_qgemv* call.
 * Outputs are dense (one row).  Q8MI_REJECTED (nothing launched; use
 * q8mi_rms_norm_quantize_q8_1 and the GEMV) when batch != 1, cols is above 6144 or
 * not a multiple of 256, x / weight / normalized are not 16-byte aligned, or
 * normalized == x (every workgroup reads x while one writes the normalised row, so
 * the two must not overlap; q8mi_rms_norm and q8mi_rms_norm_quantize_q8_1 may work
 * in place). */
int q8mi_nqgemv(const uint8_t *weight, const float *x, const float *norm_weight, float eps, float *normalized,
                void *dst, int dst_is_bf16, uint32_t rows, uint32_t cols, uint32_t batch, void *stream);
int q8mi_nqgemv_silu_mul(const uint8_t *weight_gate, const uint8_t *weight_up, const float *x,
                         const float *norm_weight, float eps, float *normalized, float *dst, uint32_t rows,
                         uint32_t cols, uint32_t batch, void *stream);
int q8mi_nqgemv_fanout4(const uint8_t *weight0, const uint8_t *weight1, const uint8_t *weight2,
                        const uint8_t *weight3, const float *x, const float *norm_weight, float eps,
                        float *normalized, float *dst0, float *dst1, float *dst2, float *dst3, uint32_t rows0,
                        uint32_t rows1, uint32_t rows2, uint32_t rows3, uint32_t cols, uint32_t batch,
                        void *stream);

/* ---- D4 activation quantizer + int8 MFMA GEMM ---------------------------- */
/* replaces q8_1_mmq_scratch_bytes, src/mmvq_q8.cu:726-729 */
size_t q8mi_q8_1_d4_scratch_bytes(uint32_t batch, uint32_t cols);
/* replaces launch_quantize_mmq_q8_1, src/mmvq_q8.cu:736-755 (kernel :668-722).
 * Rejects cols % 128 != 0. */
int q8mi_quantize_q8_1_d4(const float *x, void *y_d4, uint32_t batch, uint32_t cols,
                          uint32_t stride_x_row, void *stream);
/* replaces launch_mmq_q8_0, src/mmq_q8.cu:2278-2501.  As in the reference the
 * activation layout is implied by the shape (src/kernels_cuda.cu:14545-14552):
 * rows >= 128 && cols % 128 == 0 -> y is D4 (144-B super-blocks); otherwise y is
 * Q8_1 (36-B blocks).  Rejects cols % 32 != 0, rows == 0, batch == 0.
 * dst must be ordinary (coarse-grained) device memory: when the 128 x 128 tiles
 * leave a last round that fills at most half of the chip, when a batch of
 * up to 32 rows gives at most one 32-row tile per CU, or when a medium batch
 * has a few more 32- or 64-row tiles than the chip holds workgroups (the K
 * steps of all tiles are then dealt out evenly), those outputs are zeroed by a
 * small kernel and then summed from two ranges of K with hardware fp32 atomic
 * adds (two addends onto zero, so results repeat bit for bit); the call then
 * enqueues two kernels instead of one.  The same holds for q8mi_gemm_medium. */
int q8mi_gemm(const uint8_t *weight, const void *y, float *dst, uint32_t rows, uint32_t cols,
              uint32_t batch, uint32_t stride_dst_row, void *stream);
/* replaces launch_mmq_q8_0_medium, src/mmq_q8.cu:2512-2548: y is always D4.
 * Rejects cols % 128 != 0, rows == 0, batch == 0, batch > 64. */
int q8mi_gemm_medium(const uint8_t *weight, const void *y_d4, float *dst, uint32_t rows,
                     uint32_t cols, uint32_t batch, uint32_t stride_dst_row, void *stream);

/* The batched forms of the executor's fused operators, one launch each where the reference's CUDA
 * backend runs its tile GEMM into a temporary and a second kernel over the batch x rows outputs.
 * All three take D4 activations and serve rows >= 128, cols % 256 == 0 (every model shape);
 * anything else, and the shapes named below, is Q8MI_REJECTED (nothing enqueued) and the caller
 * runs the two-step form.
 *
 * q8mi_gemm_add: dst[j][r] = residual[j][r] + (W x)[j][r]; residual rows are stride_dst_row floats
 * apart like dst's and residual may be dst.  Replaces launch_mmq_q8_0 into matmul_tmp followed by
 * add_kernel (q8_0_matmul_add, include/qw3/device_backend.hpp:529-540, src/kernels_cuda.cu:11919-11957,
 * 1644-1652); same bits as q8mi_gemm + q8mi_add wherever q8mi_gemm does not sum from two halves of K.
 * Rejected: batch <= 16 out of place (in place the matrix-core GEMV adds as q8mi_gemv_add does), and
 * shapes q8mi_gemm serves by adding two ranges of K into a zeroed dst (a partly filled last round of
 * 128 x 128 tiles, at most one 32-row tile per CU at batch <= 32, a few more ring tiles than the
 * chip holds workgroups): a sum that arrives in two parts cannot meet the residual in an order that
 * repeats, and on those shapes q8mi_gemm + q8mi_add is the faster route anyway. */
int q8mi_gemm_add(const uint8_t *weight, const void *y_d4, const float *residual, float *dst, uint32_t rows,
                  uint32_t cols, uint32_t batch, uint32_t stride_dst_row, void *stream);
/* q8mi_gemm with bf16 outputs (round to nearest even in the store): replaces launch_mmq_q8_0 into an
 * fp32 workspace followed by convert_q8_output_bf16 (src/kernels_cuda.cu:14509-14530).  Rejected:
 * batch <= 16 (a weight stream: quantize to Q8_1 and use q8mi_gemv_bf16) and the two-part shapes above. */
int q8mi_gemm_bf16(const uint8_t *weight, const void *y_d4, uint16_t *dst, uint32_t rows, uint32_t cols,
                   uint32_t batch, uint32_t stride_dst_row, void *stream);
/* dst[j][r] = silu((Wg x)[j][r]) * (Wu x)[j][r], silu(g) = g / (1 + exp(-g)): the batched SwiGLU the
 * operator interface asks for (q8_0_matmul_silu_mul, include/qw3/device_backend.hpp:330-336).  The
 * reference's CUDA backend declines it for Q8_0 (src/kernels_cuda.cu:12323-12333) and the executor
 * then runs launch_mmq_q8_0 twice and silu_mul_kernel (src/qwen_executor.cpp:6669-6685,
 * src/kernels_cuda.cu:1894-1911): five passes over batch x rows floats that this call replaces by
 * one write.  Every tile holds gate rows and the matching up rows, so both sums of an output meet in
 * one lane.  Any batch: the matrix-core GEMV up to 16 rows where one pass covers them, 32 + 32-row
 * ring tiles for medium batches, 64 + 64-row main tiles from about 0.4 tiles per workgroup slot. */
int q8mi_gemm_silu_mul(const uint8_t *weight_gate, const uint8_t *weight_up, const void *y_d4, float *dst,
                       uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride_dst_row, void *stream);

/* replaces silu_mul_kernel, src/kernels_cuda.cu:1894-1911, as launched by silu_mul and silu_mul_n
 * (:14880-14900): out[i] = silu(gate[i]) * up[i] for i < n (fp32).  out may be gate or up. */
int q8mi_silu_mul(float *out, const float *gate, const float *up, uint64_t n, void *stream);

/* replaces fp32_to_bf16_kernel as used by convert_q8_output_bf16,
 * src/kernels_cuda.cu:14523-14530: out[i] = bf16(in[i]), round to nearest even. */
int q8mi_f32_to_bf16(const float *in, uint16_t *out, uint64_t n, void *stream);

/* replaces add_kernel / add_bf16_kernel, src/kernels_cuda.cu:1644-1677, as launched by add and
 * add_n (:14818-14862): out[i] = a[i] + b[i] for i < n, fp32, or (is_bf16) three bf16 arrays with
 * out[i] = bf16(f32(a[i]) + f32(b[i])) rounded to nearest even.  out may be a or b.  The second
 * half of the reference's batched q8_0_matmul_add (include/qw3/device_backend.hpp:529-540:
 * q8_0_matmul into a temporary, then add). */
int q8mi_add(void *out, const void *a, const void *b, uint64_t n, int is_bf16, void *stream);

/* ---- dequantizing row gather (embedding lookup) ---------------------------- */
/* out[i] = fp32(d[i / 32]) * q[i] of one row, fp32 or (out_is_bf16) bf16 rounded
 * to nearest even.  Bit-exact: the product is exact in fp32.  All three need a
 * 4-byte aligned matrix and a 16-byte (bf16: 8-byte) aligned output.
 * replaces q8_get_row_kernel / q8_get_row_bf16_kernel, src/kernels_cuda.cu:2075-2108
 * (launched :10636-10650).  A row outside the matrix is REJECTED. */
int q8mi_get_row(const uint8_t *weight, uint64_t row, uint64_t rows, uint64_t cols, void *out,
                 int out_is_bf16, void *stream);
/* replaces q8_get_row_from_argmax_kernel, src/kernels_cuda.cu:2110-2134 (launched
 * :10704-10711): the row id is argmaxes[index].index, read on the device; an id
 * below zero or beyond the matrix gives a row of zeros. */
int q8mi_get_row_from_argmax(const uint8_t *weight, const q8mi_argmax_pair *argmaxes, uint32_t index,
                             uint64_t rows, uint64_t cols, float *out, void *stream);
/* replaces q8_get_rows_batch_kernel / q8_get_rows_batch_bf16_kernel,
 * src/kernels_cuda.cu:2141-2190 (launched :10747-10755): row_ids is a DEVICE array
 * of `batch` ids, out holds batch rows of cols elements.  An id beyond the matrix
 * gives a row of zeros (the reference reads out of bounds there). */
int q8mi_get_rows(const uint8_t *weight, const uint64_t *row_ids, uint32_t batch, uint64_t rows,
                  uint64_t cols, void *out, int out_is_bf16, void *stream);

/* ---- argmax -------------------------------------------------------------- */
/* replaces argmax_kernel, src/kernels_cuda.cu:1693-1734 (launched at :20759):
 * out2[0] = index (-1 if no element is above -inf), out2[1] = bits of the max.
 * Rows of 81920 elements and more (a vocabulary) are scanned by up to 128 workgroups whose
 * partial winners meet in a 1 KiB array the library holds in every GPU's memory (two launches;
 * the reference's single workgroup reads such a row at one CU's bandwidth).  This and
 * q8mi_argmax_to_pair share that array: calls on such rows that overlap on one GPU (two streams,
 * two threads) must be serialised by the caller.  The first such call on a device looks the
 * array's address up: make it outside a graph capture. */
int q8mi_argmax(const float *x, uint64_t n, int32_t *out2, void *stream);
/* replaces argmax_pair_kernel, src/kernels_cuda.cu:1804-1857 (launched :20787) */
int q8mi_argmax_to_pair(const float *x, uint64_t n, q8mi_argmax_pair *out, uint32_t out_index,
                     void *stream);
/* replaces argmax_rows_block_kernel + argmax_rows_finalize_kernel,
 * src/kernels_cuda.cu:1773-1802, 1859-1888 (launched :20814-20836).  Rejects
 * row_stride == 0 and rows wider than 1024*256 (the reference falls back to a
 * host scan there).  scratch: q8mi_argmax_rows_scratch_bytes() device bytes. */
size_t q8mi_argmax_rows_scratch_bytes(uint32_t batch, uint32_t row_stride);
int q8mi_argmax_rows(const float *x, uint32_t batch, uint32_t row_stride, void *scratch,
                     q8mi_argmax_pair *result, void *stream);

/* ---- fused LM head ------------------------------------------------------- */
/* No single counterpart in the reference: fuses the verify tail
 * q8_0_matmul(W_out) -> argmax_batch -> greedy accept
 * (src/qwen_executor.cpp:6779-6821, src/kernels_cuda.cu:20814-20850,
 * src/qwen_native_backend.cpp:15948-15960, 16048-16052) into one pass over the
 * LM-head weights that never materialises the batch x vocab logits.
 *   rows        vocabulary size (weight rows), cols = hidden size
 *   batch       1..8 verify rows; row i gates drafts[i]; n_drafts = batch - 1
 *   drafts      batch-1 draft token ids; host memory when drafts_on_device == 0
 *               (they are passed by value), device memory otherwise
 *   row_out     device, batch pairs {max logit, token} (ties -> lowest token)
 *   accept_out  device int32[2]: {accept length, next token} where next token =
 *               row_out[accept].index, or eos if that index is negative
 *   logits      optional device [batch][stride_logits] fp32 copy of the logits
 *               (NULL = do not write them)
 *   scratch     q8mi_lm_head_scratch_bytes(rows, cols, batch) device bytes
 */
size_t q8mi_lm_head_scratch_bytes(uint32_t rows, uint32_t cols, uint32_t batch);
int q8mi_lm_head_argmax_accept(const uint8_t *weight, const void *y_q8_1, uint32_t rows,
                               uint32_t cols, uint32_t batch, const int32_t *drafts,
                               int drafts_on_device, int32_t eos, q8mi_argmax_pair *row_out,
                               int32_t *accept_out, float *logits, uint32_t stride_logits,
                               void *scratch, void *stream);

/* No counterpart in the reference.  q8mi_lm_head_argmax_accept for callers that cannot allocate
 * device memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): same arguments without `scratch`, same results bit for bit.  The per-workgroup
 * partials go to a 64 KiB array the library holds in every GPU's memory from load to exit
 * (8 verify rows x 1024 workgroups, the most any call needs; a shape that would need more is
 * Q8MI_REJECTED).  The call allocates and frees nothing.  Its first call on a device looks the
 * array's address up, and the first call of every (rows, cols, batch, logits or none) combination
 * asks the runtime for the LDS grant and the occupancy of the kernel instantiation it picks: make
 * one eager call of each combination that will be captured before capturing it.  Every call on one GPU uses that GPU's
 * one array: calls that overlap on the same GPU (two streams, two threads) race on it and must be
 * serialised by the caller; nothing in it needs clearing between calls. */
int q8mi_lm_head_argmax_accept_static(const uint8_t *weight, const void *y_q8_1, uint32_t rows, uint32_t cols,
                                      uint32_t batch, const int32_t *drafts, int drafts_on_device, int32_t eos,
                                      q8mi_argmax_pair *row_out, int32_t *accept_out, float *logits,
                                      uint32_t stride_logits, void *stream);

/* ---- weight upload (host side) ------------------------------------------- */
/* replaces the repack loop of the CudaWeight constructor,
 * src/kernels_cuda.cu:1566-1594: interleaved GGUF Q8_0 blocks (34 B: fp16 d,
 * 32 int8) -> split-plane rows.  Both pointers are HOST memory. */
int q8mi_repack_q8_0_split_host(const void *gguf_blocks, uint64_t rows, uint64_t cols,
                                void *split_out);
/* Same repack done on the GPU (both pointers device memory; in != out). */
int q8mi_repack_q8_0_split(const void *gguf_blocks, uint64_t rows, uint64_t cols, void *split_out,
                           void *stream);

#ifdef __cplusplus
}
#endif
#endif /* Q8MI_H */
