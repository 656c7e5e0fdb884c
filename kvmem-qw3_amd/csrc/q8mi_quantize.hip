// Activation quantizers for gfx950.
//
//   quantize_q8_1     fp32 -> 36-B Q8_1 blocks  (reference: src/mmvq_q8.cu:82-112)
//   quantize_q8_1_d4  fp32 -> 144-B D4 blocks   (reference: src/mmvq_q8.cu:668-722)
//
// Both are one pass over x: a lane owns four consecutive floats (one 16-B
// load), eight lanes own a 32-element block.  The block sum of Q8_1 is formed
// with the reference's pairing (i, i+16), (i, i+8), (i, i+4), (i, i+2), (i, i+1)
// so the fp16 `s` field is bit-identical to the one its 32-lane xor butterfly
// produces: lane exchanges xor 4, 2, 1 cover the first three levels, the last
// two are the in-lane adds (c0+c2, c1+c3) and (e0+e1).
#include "q8mi_internal.hpp"
#include "q8mi_quantize_core.hpp"

namespace q8mi {
namespace {

constexpr int kQuantThreads = 256;
constexpr int kElemsPerLane = 4;

template <bool VEC>
__global__ __launch_bounds__(kQuantThreads) void quantize_q8_1_kernel(
        const float *__restrict__ x, uint8_t *__restrict__ y, uint32_t cols,
        uint32_t stride_x_row, uint32_t nb) {
    const uint32_t i0 = (blockIdx.x * kQuantThreads + threadIdx.x) * kElemsPerLane;
    if (i0 >= cols) return;  // cols % 32 == 0: an 8-lane group is in or out as a whole
    const uint32_t j = blockIdx.y;
    const Float4 v = load4<VEC>(x + static_cast<uint64_t>(j) * stride_x_row + i0);

    float d;
    const uint32_t packed = quantize4_q8_1(v, d);

    const float sum = block_sum_q8_1(v);

    const uint32_t kb = i0 / kQK;
    const uint32_t sub = (i0 % kQK) / kElemsPerLane;  // 0..7
    uint32_t *blk = reinterpret_cast<uint32_t *>(
        y + (static_cast<uint64_t>(j) * nb + kb) * kQ81Bytes);
    blk[1 + sub] = packed;
    if (sub == 0) {
        blk[0] = static_cast<uint32_t>(float_to_half_bits(d)) |
                 (static_cast<uint32_t>(float_to_half_bits(sum)) << 16);
    }
}

template <bool VEC>
__global__ __launch_bounds__(kQuantThreads) void quantize_q8_1_d4_kernel(
        const float *__restrict__ x, uint8_t *__restrict__ y, uint32_t cols,
        uint32_t stride_x_row, uint32_t batch) {
    // grid.x carries the batch, as in the reference's launch (src/mmvq_q8.cu:749): a prefill chunk
    // may hold more rows than grid.y can count
    const uint32_t i0 = (blockIdx.y * kQuantThreads + threadIdx.x) * kElemsPerLane;
    if (i0 >= cols) return;
    const uint32_t j = blockIdx.x;
    const Float4 v = load4<VEC>(x + static_cast<uint64_t>(j) * stride_x_row + i0);

    const float amax = group8_amax(v);
    const float d_inv = (amax == 0.0f) ? 0.0f : 127.0f / amax;
    int q0 = 0, q1 = 0, q2 = 0, q3 = 0;
    if (amax != 0.0f) {
        q0 = rn_int(v.x * d_inv); q1 = rn_int(v.y * d_inv);
        q2 = rn_int(v.z * d_inv); q3 = rn_int(v.w * d_inv);
    }
    const uint32_t sb = i0 / 128;
    const uint32_t iqs = i0 % 128;
    uint8_t *blk = y + (static_cast<uint64_t>(sb) * batch + j) * kD4Bytes;
    *reinterpret_cast<uint32_t *>(blk + 16 + iqs) = pack4(q0, q1, q2, q3);
    if (iqs % kQK == 0) {
        const float d = (amax == 0.0f) ? 0.0f : 1.0f / d_inv;
        *reinterpret_cast<float *>(blk + 4 * (iqs / kQK)) = d;
    }
}

bool vec_ok(const float *x, uint32_t stride_x_row) {
    return (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (stride_x_row % 4 == 0);
}

}  // namespace
}  // namespace q8mi

using namespace q8mi;

extern "C" size_t q8mi_q8_1_scratch_bytes(uint32_t batch, uint32_t cols) {
    const uint32_t nb = (cols + kQK - 1) / kQK;
    return static_cast<size_t>(batch) * nb * kQ81Bytes;
}

extern "C" size_t q8mi_q8_1_d4_scratch_bytes(uint32_t batch, uint32_t cols) {
    const uint32_t nsb = (cols + 127) / 128;
    return static_cast<size_t>(batch) * nsb * kD4Bytes;
}

extern "C" int q8mi_quantize_q8_1(const float *x, void *y, uint32_t batch, uint32_t cols,
                                  uint32_t stride_x_row, void *stream) {
    if (cols % kQK != 0) return fail(Q8MI_REJECTED, "quantize_q8_1: cols %u not a multiple of 32", cols);
    if (batch == 0 || cols == 0) return Q8MI_OK;
    if (batch > 65535u) return fail(Q8MI_REJECTED, "quantize_q8_1: batch %u above 65535", batch);
    const dim3 grid((cols + kQuantThreads * kElemsPerLane - 1) / (kQuantThreads * kElemsPerLane), batch);
    const uint32_t nb = cols / kQK;
    if (vec_ok(x, stride_x_row)) {
        quantize_q8_1_kernel<true><<<grid, kQuantThreads, 0, as_stream(stream)>>>(
            x, static_cast<uint8_t *>(y), cols, stride_x_row, nb);
    } else {
        quantize_q8_1_kernel<false><<<grid, kQuantThreads, 0, as_stream(stream)>>>(
            x, static_cast<uint8_t *>(y), cols, stride_x_row, nb);
    }
    return check_launch("quantize_q8_1");
}

extern "C" int q8mi_quantize_q8_1_d4(const float *x, void *y, uint32_t batch, uint32_t cols,
                                     uint32_t stride_x_row, void *stream) {
    if (cols % 128 != 0) return fail(Q8MI_REJECTED, "quantize_q8_1_d4: cols %u not a multiple of 128", cols);
    if (batch == 0 || cols == 0) return Q8MI_OK;
    const uint32_t col_groups = (cols + kQuantThreads * kElemsPerLane - 1) / (kQuantThreads * kElemsPerLane);
    if (col_groups > 65535u || batch > 0x7fffffffu) return fail(Q8MI_REJECTED, "quantize_q8_1_d4: shape too large for one launch");
    const dim3 grid(batch, col_groups);
    if (vec_ok(x, stride_x_row)) {
        quantize_q8_1_d4_kernel<true><<<grid, kQuantThreads, 0, as_stream(stream)>>>(
            x, static_cast<uint8_t *>(y), cols, stride_x_row, batch);
    } else {
        quantize_q8_1_d4_kernel<false><<<grid, kQuantThreads, 0, as_stream(stream)>>>(
            x, static_cast<uint8_t *>(y), cols, stride_x_row, batch);
    }
    return check_launch("quantize_q8_1_d4");
}
