// Core of the Q8_0 x Q8_1 GEMV: how one wave turns one weight row into
// per-lane fp32 partial sums, and how a workgroup stages the activations in
// LDS.  Shared by the GEMV family and the fused LM-head kernel.
#pragma once

#include "q8mi_device.hpp"
#include "q8mi_internal.hpp"

namespace q8mi {

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / kWave;
constexpr uint32_t kMaxXLdsBytes = 64 * 1024;

// LDS footprint of `batch` activation rows: per 64-block step 128 16-byte
// pieces of int8 and 64 fp32 scales, zero-padded to whole steps.
inline uint32_t x_lds_bytes(uint32_t nb, uint32_t batch) {
    const uint32_t nsteps = (nb * 2 + 127) / 128;
    return batch * nsteps * (128 * 16 + 64 * 4);
}

__device__ __forceinline__ v4i load_q16(const uint8_t *p) {
    return *reinterpret_cast<const v4i *>(p);
}

// 16 activation bytes of Q8_1 block `blk` (half = 0/1) straight from global
// memory; the block is only 4-byte aligned.
__device__ __forceinline__ v4i load_x16_global(const uint8_t *y, uint32_t blk, uint32_t half) {
    const int *p = reinterpret_cast<const int *>(y + static_cast<uint64_t>(blk) * kQ81Bytes + 4 + half * 16);
    v4i v;
    v.x = p[0]; v.y = p[1]; v.z = p[2]; v.w = p[3];
    return v;
}

// Copies M rows of Q8_1 activations from global memory into LDS, split into a
// packed int8 area and an fp32 scale area.  Dword 0 of each 36-B block is
// {d, s}; dwords 1..8 are the quants.  Ends with a workgroup barrier.
template <int M>
__device__ __forceinline__ void stage_x_lds(uint8_t *smem, const uint8_t *__restrict__ y, uint32_t nb) {
    const uint32_t nsteps = (nb * 2 + 127) / 128;
    int *wq = reinterpret_cast<int *>(smem);
    float *wd = reinterpret_cast<float *>(smem + static_cast<size_t>(M) * nsteps * 128 * 16);
    const uint32_t blocks_padded = nsteps * 64;
    const uint32_t total = static_cast<uint32_t>(M) * blocks_padded * 9;
    const uint32_t *src = reinterpret_cast<const uint32_t *>(y);
    for (uint32_t i = threadIdx.x; i < total; i += kGemvThreads) {
        const uint32_t blk = i / 9, part = i % 9;
        const uint32_t m = blk / blocks_padded, kb = blk % blocks_padded;
        const bool valid = kb < nb;
        const uint32_t word = valid ? src[static_cast<uint64_t>(m * nb + kb) * 9 + part] : 0u;
        if (part == 0) {
            wd[blk] = half_bits_to_float(static_cast<uint16_t>(word & 0xffffu));
        } else {
            wq[blk * 8 + (part - 1)] = static_cast<int>(word);
        }
    }
    __syncthreads();
}

// Accumulates one weight row against M activation rows.  `row_w` points at the
// row's scale plane.  Returns per-lane partial sums in acc[].
template <int M, bool XLDS>
__device__ __forceinline__ void row_partial(const uint8_t *__restrict__ row_w,
                                            const uint8_t *__restrict__ y, const int *lds_q,
                                            const float *lds_d, uint32_t nb, uint32_t lane,
                                            float (&acc)[M]) {
    const uint16_t *scales = reinterpret_cast<const uint16_t *>(row_w);
    const uint8_t *quants = row_w + 2 * nb;
    const uint32_t npieces = nb * 2;             // 16-byte pieces in the row
    const uint32_t nsteps = (npieces + 127) / 128;
    const bool odd = lane & 1u;
#pragma unroll
    for (int m = 0; m < M; ++m) acc[m] = 0.0f;

    for (uint32_t step = 0; step < nsteps; ++step) {
        const uint32_t pa = step * 128 + lane;
        const uint32_t pb = pa + 64;
        const bool va = pa < npieces, vb = pb < npieces;
        v4i qa = {0, 0, 0, 0}, qb = {0, 0, 0, 0};
        if (va) qa = load_q16(quants + static_cast<uint64_t>(pa) * 16);
        if (vb) qb = load_q16(quants + static_cast<uint64_t>(pb) * 16);
        // the block this lane rescales: A_(lane/2) on even lanes, B_(lane/2) on odd
        const uint32_t kb = step * 64 + (odd ? 32u : 0u) + (lane >> 1);
        const bool vk = kb < nb;
        const float dw = vk ? half_bits_to_float(scales[kb]) : 0.0f;
#pragma unroll
        for (int m = 0; m < M; ++m) {
            v4i xa = {0, 0, 0, 0}, xb = {0, 0, 0, 0};
            float dx = 0.0f;
            if (XLDS) {
                // LDS is zero-padded up to a whole number of steps: no guards
                xa = *reinterpret_cast<const v4i *>(lds_q + (static_cast<uint32_t>(m) * nsteps * 128 + pa) * 4);
                xb = *reinterpret_cast<const v4i *>(lds_q + (static_cast<uint32_t>(m) * nsteps * 128 + pb) * 4);
                dx = lds_d[static_cast<uint32_t>(m) * nsteps * 64 + kb];
            } else {
                if (va) xa = load_x16_global(y, m * nb + (pa >> 1), pa & 1u);
                if (vb) xb = load_x16_global(y, m * nb + (pb >> 1), pb & 1u);
                if (vk) {
                    dx = half_bits_to_float(*reinterpret_cast<const uint16_t *>(
                        y + static_cast<uint64_t>(m * nb + kb) * kQ81Bytes));
                }
            }
            const int sa = dot16(qa, xa, 0);
            const int sb = dot16(qb, xb, 0);
            const int give = odd ? sa : sb;
            const int keep = odd ? sb : sa;
            const int S = keep + dpp_i32<kDppXor1>(give);  // full 32-element block dot
            acc[m] = fmaf(dw * dx, static_cast<float>(S), acc[m]);
        }
    }
}

}  // namespace q8mi
