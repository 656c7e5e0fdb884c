// What a GEMV launch carries from the entry points to the kernels, shared by the streaming
// kernels (q8mi_gemv.hip) and the row-pair kernels (q8mi_gemv_pairs.hip).
#pragma once

#include "q8mi_device.hpp"
#include "q8mi_internal.hpp"

namespace q8mi {

enum GemvMode : int {
    kStoreF32 = 0,
    kAddF32 = 1,
    kStoreBF16 = 2,
    kAddBF16 = 3,
    kSiluMul = 4,  // w[0] = gate, w[1] = up, one output
};

struct GemvParams {
    const uint8_t *w[4];
    void *dst[4];
    uint32_t row_end[4];  // cumulative row counts of the concatenated row space
    uint32_t stride[4];
    const uint8_t *y;     // Q8_1 blocks, [batch][nb] (null when xf is set)
    const float *xf;      // fp32 activations to be quantized while staging (fused entry points)
    uint32_t x_stride;    // floats between rows of xf
    const float *norm_w;  // RMS-norm weights: xf is one raw row, normalised while staging (else null)
    float *normalized;    // where the normalised row is also written (may be null)
    float eps;
    uint32_t total_rows;  // rows of the concatenated space (SwiGLU: rows of one weight)
    uint32_t units;
    uint32_t nb;
    uint32_t x_bytes;     // LDS bytes of the staged activations (0 when they are read from global)
    int mode;
    int interleave;
};

// Which of the (up to four) concatenated weights a row belongs to.
struct RowRef {
    const uint8_t *w;
    void *dst;
    uint32_t stride;
    uint32_t local;
};

__device__ __forceinline__ RowRef resolve_row(const GemvParams &p, uint32_t row) {
    uint32_t seg = 0, base = 0;
    if (row >= p.row_end[0]) { seg = 1; base = p.row_end[0]; }
    if (row >= p.row_end[1]) { seg = 2; base = p.row_end[1]; }
    if (row >= p.row_end[2]) { seg = 3; base = p.row_end[2]; }
    RowRef r;
    r.w = p.w[0]; r.dst = p.dst[0]; r.stride = p.stride[0];
    if (seg == 1) { r.w = p.w[1]; r.dst = p.dst[1]; r.stride = p.stride[1]; }
    if (seg == 2) { r.w = p.w[2]; r.dst = p.dst[2]; r.stride = p.stride[2]; }
    if (seg == 3) { r.w = p.w[3]; r.dst = p.dst[3]; r.stride = p.stride[3]; }
    r.local = row - base;
    return r;
}

__device__ __forceinline__ void store_out(int mode, void *dst, uint64_t idx, float v) {
    if (mode == kStoreF32) {
        static_cast<float *>(dst)[idx] = v;
    } else if (mode == kAddF32) {
        float *p = static_cast<float *>(dst) + idx;
        *p = *p + v;
    } else if (mode == kStoreBF16) {
        static_cast<uint16_t *>(dst)[idx] = float_to_bf16_bits(v);
    } else {
        uint16_t *p = static_cast<uint16_t *>(dst) + idx;
        *p = float_to_bf16_bits(bf16_bits_to_float(*p) + v);
    }
}

// Row-pair kernels for batch 1..4 (q8mi_gemv_pairs.hip): Q8MI_REJECTED when the shape is not theirs,
// so that the caller goes on to the streaming kernels.
int launch_pairs(const GemvParams &p, uint32_t batch, hipStream_t stream);

}  // namespace q8mi
