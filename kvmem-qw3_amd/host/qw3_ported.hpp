// qw3::ported launchers for gfx950.
//
// Same names, argument order and meaning as the launchers the reference's CUDA
// backend declares at src/kernels_cuda.cu:56-125 and defines in src/mmvq_q8.cu /
// src/mmq_q8.cu, with hipStream_t in place of cudaStream_t.  Each one forwards to
// the C ABI in include/q8mi.h; `false` means the shape was rejected and nothing
// was enqueued (the caller's fallback chain still works), launch errors are
// picked up by the caller with hipGetLastError() as before.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "../../include/q8mi.h"

namespace qw3 {
namespace ported {

// src/mmvq_q8.cu:613-616
inline size_t q8_1_scratch_bytes(uint32_t batch, uint32_t cols) { return q8mi_q8_1_scratch_bytes(batch, cols); }

// src/mmvq_q8.cu:623-640
inline bool launch_quantize_q8_1(const float *x, void *y_q8_1, uint32_t batch, uint32_t cols,
                                 uint32_t stride_x_row, hipStream_t stream) {
    return q8mi_quantize_q8_1(x, y_q8_1, batch, cols, stride_x_row, stream) == Q8MI_OK;
}

// src/mmvq_q8.cu:805-811
inline bool launch_mmvq_q8_0(const uint8_t *weight, const void *y_q8_1, float *dst, uint32_t rows,
                             uint32_t cols, uint32_t batch, uint32_t stride_dst_row, hipStream_t stream) {
    return q8mi_gemv(weight, y_q8_1, dst, rows, cols, batch, stride_dst_row, stream) == Q8MI_OK;
}

// src/mmvq_q8.cu:813-819 (dst: bf16 bit patterns)
inline bool launch_mmvq_q8_0_bf16(const uint8_t *weight, const void *y_q8_1, uint16_t *dst, uint32_t rows,
                                  uint32_t cols, uint32_t batch, uint32_t stride_dst_row, hipStream_t stream) {
    return q8mi_gemv_bf16(weight, y_q8_1, dst, rows, cols, batch, stride_dst_row, stream) == Q8MI_OK;
}

// src/mmvq_q8.cu:823-864
inline bool launch_mmvq_q8_0_two(const uint8_t *weight0, const uint8_t *weight1, const void *y_q8_1,
                                 float *dst0, float *dst1, uint32_t rows, uint32_t cols, uint32_t batch,
                                 uint32_t stride_dst_row, hipStream_t stream) {
    return q8mi_gemv_two(weight0, weight1, y_q8_1, dst0, dst1, rows, cols, batch, stride_dst_row, stream) ==
           Q8MI_OK;
}

// src/mmvq_q8.cu:869-909
inline bool launch_mmvq_q8_0_silu_mul(const uint8_t *weight_gate, const uint8_t *weight_up, const void *y_q8_1,
                                      float *dst, uint32_t rows, uint32_t cols, uint32_t batch,
                                      uint32_t stride_dst_row, hipStream_t stream) {
    return q8mi_gemv_silu_mul(weight_gate, weight_up, y_q8_1, dst, rows, cols, batch, stride_dst_row, stream) ==
           Q8MI_OK;
}

// src/mmvq_q8.cu:955-961
inline bool launch_mmvq_q8_0_add(const uint8_t *weight, const void *y_q8_1, float *dst, uint32_t rows,
                                 uint32_t cols, uint32_t batch, uint32_t stride_dst_row, hipStream_t stream) {
    return q8mi_gemv_add(weight, y_q8_1, dst, rows, cols, batch, stride_dst_row, stream) == Q8MI_OK;
}

// src/mmvq_q8.cu:963-969
inline bool launch_mmvq_q8_0_add_bf16(const uint8_t *weight, const void *y_q8_1, uint16_t *dst, uint32_t rows,
                                      uint32_t cols, uint32_t batch, uint32_t stride_dst_row,
                                      hipStream_t stream) {
    return q8mi_gemv_add_bf16(weight, y_q8_1, dst, rows, cols, batch, stride_dst_row, stream) == Q8MI_OK;
}

// src/mmvq_q8.cu:1070-1113
inline bool launch_mmvq_q8_0_fanout4_batch(const uint8_t *weight0, const uint8_t *weight1,
                                           const uint8_t *weight2, const uint8_t *weight3, const void *y_q8_1,
                                           float *dst0, float *dst1, float *dst2, float *dst3, uint32_t rows0,
                                           uint32_t rows1, uint32_t rows2, uint32_t rows3, uint32_t cols,
                                           uint32_t batch, uint32_t stride_dst0, uint32_t stride_dst1,
                                           uint32_t stride_dst2, uint32_t stride_dst3, hipStream_t stream) {
    return q8mi_gemv_fanout4(weight0, weight1, weight2, weight3, y_q8_1, dst0, dst1, dst2, dst3, rows0, rows1,
                             rows2, rows3, cols, batch, stride_dst0, stride_dst1, stride_dst2, stride_dst3,
                             stream) == Q8MI_OK;
}

// src/mmvq_q8.cu:726-729
inline size_t q8_1_mmq_scratch_bytes(uint32_t batch, uint32_t cols) {
    return q8mi_q8_1_d4_scratch_bytes(batch, cols);
}

// src/mmvq_q8.cu:736-755
inline bool launch_quantize_mmq_q8_1(const float *x, void *y_q8_1_mmq, uint32_t batch, uint32_t cols,
                                     uint32_t stride_x_row, hipStream_t stream) {
    return q8mi_quantize_q8_1_d4(x, y_q8_1_mmq, batch, cols, stride_x_row, stream) == Q8MI_OK;
}

// src/mmq_q8.cu:2278-2501
inline bool launch_mmq_q8_0(const uint8_t *weight, const void *y_q8_1, float *dst, uint32_t rows, uint32_t cols,
                            uint32_t batch, uint32_t stride_dst_row, hipStream_t stream) {
    return q8mi_gemm(weight, y_q8_1, dst, rows, cols, batch, stride_dst_row, stream) == Q8MI_OK;
}

// src/mmq_q8.cu:2512-2548
inline bool launch_mmq_q8_0_medium(const uint8_t *weight, const void *y_q8_1_mmq, float *dst, uint32_t rows,
                                   uint32_t cols, uint32_t batch, uint32_t stride_dst_row, hipStream_t stream) {
    return q8mi_gemm_medium(weight, y_q8_1_mmq, dst, rows, cols, batch, stride_dst_row, stream) == Q8MI_OK;
}

}  // namespace ported
}  // namespace qw3
