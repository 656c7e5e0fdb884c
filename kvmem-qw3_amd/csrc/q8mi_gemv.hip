// Q8_0 weight x Q8_1 activation GEMV for batch 1..8 on gfx950.
// Reference semantics: src/mmvq_q8.cu:193-280 (plain), :295-399 (two weights),
// :414-519 (SwiGLU), :528-606 (residual add), :976-1068 (four-weight fan-out).
//
// Shape of the work: the weights are read exactly once from HBM and nothing
// else is large, so the kernel is a stream over the int8 plane of each row.
//   * One wave owns one weight row at a time; waves stride over rows so that
//     the waves in flight read adjacent rows (adjacent addresses).
//   * Inside a row a lane reads 16 contiguous bytes per load, the wave 1 KiB
//     per load (global_load_dwordx4, fully coalesced).  Two such loads ("A" and
//     "B", 1 KiB apart) form one step; a lane therefore holds half of block
//     A_(lane/2) and half of block B_(lane/2).  Lane pairs swap half sums with
//     one DPP move so that the even lane ends with the full int32 dot of block
//     A and the odd lane with that of block B: every 32-element block gets one
//     int32 sum and one fp32 rescale, as the reference's MMQ path does.
//   * Activations are tiny and re-used by every row: the workgroup stages them
//     once in LDS (int8 as packed dwords + fp32 scales) when they fit, otherwise
//     lanes read them from global memory (served by L2).
//   * Per-lane fp32 partial sums are reduced across the wave with DPP in a
//     fixed order, so results are deterministic run to run.
#include "q8mi_gemv_core.hpp"

namespace q8mi {
namespace {

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
    const uint8_t *y;     // Q8_1 blocks, [batch][nb]
    uint32_t total_rows;
    uint32_t cols;
    uint32_t nb;
};

template <int MODE>
__device__ __forceinline__ void store_out(void *dst, uint64_t idx, float v) {
    if (MODE == kStoreF32 || MODE == kSiluMul) {
        static_cast<float *>(dst)[idx] = v;
    } else if (MODE == kAddF32) {
        float *p = static_cast<float *>(dst) + idx;
        *p = *p + v;
    } else if (MODE == kStoreBF16) {
        static_cast<uint16_t *>(dst)[idx] = float_to_bf16_bits(v);
    } else {
        uint16_t *p = static_cast<uint16_t *>(dst) + idx;
        *p = float_to_bf16_bits(bf16_bits_to_float(*p) + v);
    }
}

template <int M, int MODE, bool XLDS>
__global__ __launch_bounds__(kGemvThreads) void gemv_kernel(const GemvParams p) {
    extern __shared__ __align__(16) uint8_t smem[];
    const uint32_t nb = p.nb;
    const uint32_t nsteps = (nb * 2 + 127) / 128;
    const int *lds_q = reinterpret_cast<const int *>(smem);
    const float *lds_d = reinterpret_cast<const float *>(smem + static_cast<size_t>(M) * nsteps * 128 * 16);

    if (XLDS) stage_x_lds<M>(smem, p.y, nb);

    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t wave = blockIdx.x * kGemvWaves + threadIdx.x / kWave;
    const uint32_t nwaves = gridDim.x * kGemvWaves;
    const uint64_t row_bytes = static_cast<uint64_t>(nb) * 34;

    for (uint32_t row = wave; row < p.total_rows; row += nwaves) {
        if (MODE == kSiluMul) {
            float g[M], u[M];
            row_partial<M, XLDS>(p.w[0] + row * row_bytes, p.y, lds_q, lds_d, nb, lane, g);
            row_partial<M, XLDS>(p.w[1] + row * row_bytes, p.y, lds_q, lds_d, nb, lane, u);
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const float gs = wave_sum(g[m]);
                const float us = wave_sum(u[m]);
                if (lane == 0) {
                    const float silu = gs / (1.0f + __expf(-gs));
                    static_cast<float *>(p.dst[0])[static_cast<uint64_t>(m) * p.stride[0] + row] = silu * us;
                }
            }
        } else {
            // which of the (up to four) concatenated weights this row belongs to
            uint32_t seg = 0, base = 0;
            if (row >= p.row_end[0]) { seg = 1; base = p.row_end[0]; }
            if (row >= p.row_end[1]) { seg = 2; base = p.row_end[1]; }
            if (row >= p.row_end[2]) { seg = 3; base = p.row_end[2]; }
            const uint32_t local = row - base;
            const uint8_t *wbase = p.w[0];
            void *dst = p.dst[0];
            uint32_t stride = p.stride[0];
            if (seg == 1) { wbase = p.w[1]; dst = p.dst[1]; stride = p.stride[1]; }
            if (seg == 2) { wbase = p.w[2]; dst = p.dst[2]; stride = p.stride[2]; }
            if (seg == 3) { wbase = p.w[3]; dst = p.dst[3]; stride = p.stride[3]; }
            float acc[M];
            row_partial<M, XLDS>(wbase + local * row_bytes, p.y, lds_q, lds_d, nb, lane, acc);
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const float s = wave_sum(acc[m]);
                if (lane == 0) store_out<MODE>(dst, static_cast<uint64_t>(m) * stride + local, s);
            }
        }
    }
}

// Fallback for rows whose planes are not 16-byte aligned (cols/32 not a
// multiple of 8): one lane per 32-element block, 2-byte weight loads.
template <int MODE>
__global__ __launch_bounds__(kGemvThreads) void gemv_unaligned_kernel(const GemvParams p, uint32_t batch) {
    const uint32_t nb = p.nb;
    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t wave = blockIdx.x * kGemvWaves + threadIdx.x / kWave;
    const uint32_t nwaves = gridDim.x * kGemvWaves;
    const uint64_t row_bytes = static_cast<uint64_t>(nb) * 34;
    const uint32_t nw = (MODE == kSiluMul) ? 2 : 1;

    for (uint32_t row = wave; row < p.total_rows; row += nwaves) {
        uint32_t seg = 0, base = 0;
        if (MODE != kSiluMul) {
            if (row >= p.row_end[0]) { seg = 1; base = p.row_end[0]; }
            if (row >= p.row_end[1]) { seg = 2; base = p.row_end[1]; }
            if (row >= p.row_end[2]) { seg = 3; base = p.row_end[2]; }
        }
        const uint32_t local = row - base;
        for (uint32_t j = 0; j < batch; ++j) {
            float res[2] = {0.0f, 0.0f};
            for (uint32_t wi = 0; wi < nw; ++wi) {
                const uint8_t *row_w = p.w[MODE == kSiluMul ? wi : seg] + local * row_bytes;
                const uint16_t *scales = reinterpret_cast<const uint16_t *>(row_w);
                const uint16_t *quants = reinterpret_cast<const uint16_t *>(row_w + 2 * nb);
                float acc = 0.0f;
                for (uint32_t kb = lane; kb < nb; kb += kWave) {
                    const uint8_t *xb = p.y + static_cast<uint64_t>(j * nb + kb) * kQ81Bytes;
                    const int *xq = reinterpret_cast<const int *>(xb + 4);
                    int S = 0;
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        const int wq = static_cast<int>(quants[kb * 16 + 2 * t]) |
                                       (static_cast<int>(quants[kb * 16 + 2 * t + 1]) << 16);
                        S = __builtin_amdgcn_sdot4(wq, xq[t], S, false);
                    }
                    const float dw = half_bits_to_float(scales[kb]);
                    const float dx = half_bits_to_float(*reinterpret_cast<const uint16_t *>(xb));
                    acc = fmaf(dw * dx, static_cast<float>(S), acc);
                }
                res[wi] = wave_sum(acc);
            }
            if (lane == 0) {
                if (MODE == kSiluMul) {
                    const float silu = res[0] / (1.0f + __expf(-res[0]));
                    static_cast<float *>(p.dst[0])[static_cast<uint64_t>(j) * p.stride[0] + row] = silu * res[1];
                } else {
                    store_out<MODE>(p.dst[seg], static_cast<uint64_t>(j) * p.stride[seg] + local, res[0]);
                }
            }
        }
    }
}

template <int M, int MODE>
int launch_m(const GemvParams &p, hipStream_t stream) {
    const int cus = device_cu_count();
    const uint32_t lds = x_lds_bytes(p.nb, M);
    const uint32_t rows_per_wg_pass = kGemvWaves;
    uint32_t max_wgs = (p.total_rows + rows_per_wg_pass - 1) / rows_per_wg_pass;
    if (lds <= kMaxXLdsBytes) {
        // persistent-style grid: a few workgroups per CU, each stages x once
        uint32_t per_cu = 160u * 1024u / (lds + 1024u);
        if (per_cu > 4) per_cu = 4;
        if (per_cu < 1) per_cu = 1;
        uint32_t grid = static_cast<uint32_t>(cus) * per_cu;
        if (grid > max_wgs) grid = max_wgs;
        gemv_kernel<M, MODE, true><<<grid, kGemvThreads, lds, stream>>>(p);
    } else {
        uint32_t grid = static_cast<uint32_t>(cus) * 4;
        if (grid > max_wgs) grid = max_wgs;
        gemv_kernel<M, MODE, false><<<grid, kGemvThreads, 0, stream>>>(p);
    }
    return check_launch("gemv");
}

template <int MODE>
int launch_mode(const GemvParams &p, uint32_t batch, hipStream_t stream) {
    if (p.nb % 8 != 0) {
        const int cus = device_cu_count();
        uint32_t grid = static_cast<uint32_t>(cus) * 8;
        const uint32_t max_wgs = (p.total_rows + kGemvWaves - 1) / kGemvWaves;
        if (grid > max_wgs) grid = max_wgs;
        gemv_unaligned_kernel<MODE><<<grid, kGemvThreads, 0, stream>>>(p, batch);
        return check_launch("gemv_unaligned");
    }
    switch (batch) {
        case 1: return launch_m<1, MODE>(p, stream);
        case 2: return launch_m<2, MODE>(p, stream);
        case 3: return launch_m<3, MODE>(p, stream);
        case 4: return launch_m<4, MODE>(p, stream);
        case 5: return launch_m<5, MODE>(p, stream);
        case 6: return launch_m<6, MODE>(p, stream);
        case 7: return launch_m<7, MODE>(p, stream);
        case 8: return launch_m<8, MODE>(p, stream);
        default: return Q8MI_REJECTED;
    }
}

int shape_gate(const char *what, uint32_t cols, uint32_t batch) {
    if (cols % kQK != 0) return fail(Q8MI_REJECTED, "%s: cols %u not a multiple of 32", what, cols);
    if (batch == 0 || batch > Q8MI_MAX_GEMV_BATCH)
        return fail(Q8MI_REJECTED, "%s: batch %u outside 1..8", what, batch);
    return Q8MI_OK;
}

bool planes_aligned(const void *w) { return reinterpret_cast<uintptr_t>(w) % 16 == 0; }

GemvParams single(const uint8_t *w, const void *y, void *dst, uint32_t rows, uint32_t cols,
                  uint32_t stride) {
    GemvParams p{};
    p.w[0] = w;
    p.dst[0] = dst;
    p.stride[0] = stride;
    for (int i = 0; i < 4; ++i) p.row_end[i] = rows;
    p.y = static_cast<const uint8_t *>(y);
    p.total_rows = rows;
    p.cols = cols;
    p.nb = cols / kQK;
    return p;
}

template <int MODE>
int run_single(const char *what, const uint8_t *w, const void *y, void *dst, uint32_t rows,
               uint32_t cols, uint32_t batch, uint32_t stride, void *stream) {
    if (int rc = shape_gate(what, cols, batch)) return rc;
    if (rows == 0 || cols == 0) return Q8MI_OK;
    if (!planes_aligned(w)) return fail(Q8MI_REJECTED, "%s: weight pointer not 16-byte aligned", what);
    const GemvParams p = single(w, y, dst, rows, cols, stride);
    return launch_mode<MODE>(p, batch, as_stream(stream));
}

}  // namespace

// Any batch through the GEMV kernels, eight activation rows per launch.  Used by
// the GEMM entry point for shapes its MFMA tile does not cover.
int gemv_any_batch(const uint8_t *w, const void *y_q8_1, float *dst, uint32_t rows, uint32_t cols,
                   uint32_t batch, uint32_t stride_dst_row, hipStream_t stream) {
    const uint32_t nb = cols / kQK;
    const auto *y = static_cast<const uint8_t *>(y_q8_1);
    for (uint32_t j0 = 0; j0 < batch; j0 += Q8MI_MAX_GEMV_BATCH) {
        const uint32_t m = batch - j0 < Q8MI_MAX_GEMV_BATCH ? batch - j0 : Q8MI_MAX_GEMV_BATCH;
        const GemvParams p = single(w, y + static_cast<uint64_t>(j0) * nb * kQ81Bytes,
                                    dst + static_cast<uint64_t>(j0) * stride_dst_row, rows, cols,
                                    stride_dst_row);
        if (int rc = launch_mode<kStoreF32>(p, m, stream)) return rc;
    }
    return Q8MI_OK;
}

}  // namespace q8mi

using namespace q8mi;

extern "C" int q8mi_gemv(const uint8_t *w, const void *y, float *dst, uint32_t rows, uint32_t cols,
                         uint32_t batch, uint32_t stride, void *stream) {
    return run_single<kStoreF32>("gemv", w, y, dst, rows, cols, batch, stride, stream);
}

extern "C" int q8mi_gemv_bf16(const uint8_t *w, const void *y, uint16_t *dst, uint32_t rows,
                              uint32_t cols, uint32_t batch, uint32_t stride, void *stream) {
    return run_single<kStoreBF16>("gemv_bf16", w, y, dst, rows, cols, batch, stride, stream);
}

extern "C" int q8mi_gemv_add(const uint8_t *w, const void *y, float *dst, uint32_t rows,
                             uint32_t cols, uint32_t batch, uint32_t stride, void *stream) {
    return run_single<kAddF32>("gemv_add", w, y, dst, rows, cols, batch, stride, stream);
}

extern "C" int q8mi_gemv_add_bf16(const uint8_t *w, const void *y, uint16_t *dst, uint32_t rows,
                                  uint32_t cols, uint32_t batch, uint32_t stride, void *stream) {
    return run_single<kAddBF16>("gemv_add_bf16", w, y, dst, rows, cols, batch, stride, stream);
}

extern "C" int q8mi_gemv_silu_mul(const uint8_t *wg, const uint8_t *wu, const void *y, float *dst,
                                  uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride,
                                  void *stream) {
    if (int rc = shape_gate("gemv_silu_mul", cols, batch)) return rc;
    if (rows == 0 || cols == 0) return Q8MI_OK;
    if (!planes_aligned(wg) || !planes_aligned(wu))
        return fail(Q8MI_REJECTED, "gemv_silu_mul: weight pointer not 16-byte aligned");
    GemvParams p = single(wg, y, dst, rows, cols, stride);
    p.w[1] = wu;
    return launch_mode<kSiluMul>(p, batch, as_stream(stream));
}

extern "C" int q8mi_gemv_fanout4(const uint8_t *w0, const uint8_t *w1, const uint8_t *w2,
                                 const uint8_t *w3, const void *y, float *d0, float *d1, float *d2,
                                 float *d3, uint32_t rows0, uint32_t rows1, uint32_t rows2,
                                 uint32_t rows3, uint32_t cols, uint32_t batch, uint32_t s0,
                                 uint32_t s1, uint32_t s2, uint32_t s3, void *stream) {
    if (int rc = shape_gate("gemv_fanout4", cols, batch)) return rc;
    const uint64_t declared = static_cast<uint64_t>(rows0) + rows1 + rows2 + rows3;
    if (declared == 0 || declared > 0xffffffffull)
        return fail(Q8MI_REJECTED, "gemv_fanout4: total rows %llu out of range",
                    static_cast<unsigned long long>(declared));
    const uint8_t *w[4] = {w0, w1, w2, w3};
    float *d[4] = {d0, d1, d2, d3};
    const uint32_t r[4] = {rows0, rows1, rows2, rows3};
    const uint32_t s[4] = {s0, s1, s2, s3};
    // compact the live slots (the reference skips null / empty ones per block)
    GemvParams p{};
    uint32_t n = 0, total = 0;
    for (int i = 0; i < 4; ++i) {
        if (w[i] == nullptr || d[i] == nullptr || r[i] == 0) continue;
        if (!planes_aligned(w[i]))
            return fail(Q8MI_REJECTED, "gemv_fanout4: weight %d not 16-byte aligned", i);
        p.w[n] = w[i];
        p.dst[n] = d[i];
        p.stride[n] = s[i];
        total += r[i];
        p.row_end[n] = total;
        ++n;
    }
    if (n == 0 || cols == 0) return Q8MI_OK;
    for (uint32_t i = n; i < 4; ++i) p.row_end[i] = total;
    p.y = static_cast<const uint8_t *>(y);
    p.total_rows = total;
    p.cols = cols;
    p.nb = cols / kQK;
    return launch_mode<kStoreF32>(p, batch, as_stream(stream));
}

extern "C" int q8mi_gemv_two(const uint8_t *w0, const uint8_t *w1, const void *y, float *dst0,
                             float *dst1, uint32_t rows, uint32_t cols, uint32_t batch,
                             uint32_t stride, void *stream) {
    if (int rc = shape_gate("gemv_two", cols, batch)) return rc;
    if (rows == 0) return Q8MI_OK;
    return q8mi_gemv_fanout4(w0, w1, nullptr, nullptr, y, dst0, dst1, nullptr, nullptr, rows, rows,
                             0, 0, cols, batch, stride, stride, 0, 0, stream);
}
