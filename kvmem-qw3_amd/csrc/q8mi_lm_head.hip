// Fused LM head for MTP verification on gfx950: Q8_0 GEMV over the vocabulary
// rows + running row-argmax + greedy draft acceptance, without writing the
// batch x vocab logits.
//
// Fuses what the reference runs as q8_0_matmul(W_out) -> argmax_batch -> host
// accept loop (src/qwen_executor.cpp:6779-6821, src/kernels_cuda.cu:20814-20850,
// src/qwen_native_backend.cpp:15948-15960, 16048-16052).
//
// Pass 1 (lm_head_kernel): same weight stream as the GEMV.  A wave keeps, per
// verify row, the best {logit, token} among the vocabulary rows it has
// processed; the workgroup merges its four waves and writes one partial per
// verify row.  Pass 2 (lm_head_finalize_kernel): one workgroup merges the
// partials, writes the per-row winners, then walks the drafts.
// The merge rule is the reference's batched-argmax rule (strictly greater
// wins, equal logits go to the lower token id, src/kernels_cuda.cu:1765-1771),
// which is independent of the order partials are merged in for NaN-free logits.
#include "q8mi_gemv_core.hpp"

namespace q8mi {
namespace {

constexpr uint32_t kMaxPartials = 1024;
constexpr int kMaxDrafts = Q8MI_MAX_GEMV_BATCH - 1;

struct Drafts {
    int32_t v[kMaxDrafts];
};

__device__ __forceinline__ bool beats(float ov, int oi, float v, int i) {
    if (oi < 0) return false;
    if (i < 0) return true;
    if (ov > v) return true;
    return ov == v && oi < i;
}

template <int M, bool XLDS>
__global__ __launch_bounds__(kGemvThreads) void lm_head_kernel(
        const uint8_t *__restrict__ w, const uint8_t *__restrict__ y, uint32_t rows, uint32_t nb,
        q8mi_argmax_pair *__restrict__ partial, float *__restrict__ logits, uint32_t stride_logits) {
    extern __shared__ __align__(16) uint8_t smem[];
    const uint32_t nsteps = (nb * 2 + 127) / 128;
    const int *lds_q = reinterpret_cast<const int *>(smem);
    const float *lds_d = reinterpret_cast<const float *>(smem + static_cast<size_t>(M) * nsteps * 128 * 16);
    if (XLDS) stage_x_lds<M>(smem, y, nb);

    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t wave_in_wg = threadIdx.x / kWave;
    const uint32_t wave = blockIdx.x * kGemvWaves + wave_in_wg;
    const uint32_t nwaves = gridDim.x * kGemvWaves;
    const uint64_t row_bytes = static_cast<uint64_t>(nb) * 34;

    float best_v[M];
    int best_i[M];
#pragma unroll
    for (int m = 0; m < M; ++m) { best_v[m] = -INFINITY; best_i[m] = -1; }

    for (uint32_t row = wave; row < rows; row += nwaves) {
        float acc[M];
        row_partial<M, XLDS>(w + row * row_bytes, y, lds_q, lds_d, nb, lane, acc);
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const float s = wave_sum(acc[m]);  // identical in every lane
            if (beats(s, static_cast<int>(row), best_v[m], best_i[m])) {
                best_v[m] = s;
                best_i[m] = static_cast<int>(row);
            }
            if (logits != nullptr && lane == 0) logits[static_cast<uint64_t>(m) * stride_logits + row] = s;
        }
    }

    __shared__ float wv[kGemvWaves][Q8MI_MAX_GEMV_BATCH];
    __shared__ int wi[kGemvWaves][Q8MI_MAX_GEMV_BATCH];
    if (lane == 0) {
#pragma unroll
        for (int m = 0; m < M; ++m) { wv[wave_in_wg][m] = best_v[m]; wi[wave_in_wg][m] = best_i[m]; }
    }
    __syncthreads();
    if (threadIdx.x < M) {
        const int m = threadIdx.x;
        float v = wv[0][m];
        int i = wi[0][m];
        for (int k = 1; k < kGemvWaves; ++k) {
            if (beats(wv[k][m], wi[k][m], v, i)) { v = wv[k][m]; i = wi[k][m]; }
        }
        q8mi_argmax_pair *p = partial + static_cast<uint64_t>(m) * gridDim.x + blockIdx.x;
        p->value = v;
        p->index = i;
    }
}

__global__ __launch_bounds__(kMaxPartials) void lm_head_finalize_kernel(
        const q8mi_argmax_pair *__restrict__ partial, uint32_t nparts, uint32_t batch, Drafts drafts_val,
        const int32_t *__restrict__ drafts_dev, int32_t eos, q8mi_argmax_pair *__restrict__ row_out,
        int32_t *__restrict__ accept_out) {
    __shared__ float sv[kMaxPartials];
    __shared__ int si[kMaxPartials];
    __shared__ int tokens[Q8MI_MAX_GEMV_BATCH];
    const uint32_t tid = threadIdx.x;
    for (uint32_t m = 0; m < batch; ++m) {
        float v = -INFINITY;
        int i = -1;
        if (tid < nparts) {
            const q8mi_argmax_pair p = partial[static_cast<uint64_t>(m) * nparts + tid];
            v = p.value;
            i = p.index;
        }
        sv[tid] = v;
        si[tid] = i;
        __syncthreads();
        for (uint32_t stride = kMaxPartials / 2; stride > 0; stride >>= 1) {
            if (tid < stride) {
                const float ov = sv[tid + stride];
                const int oi = si[tid + stride];
                if (beats(ov, oi, sv[tid], si[tid])) { sv[tid] = ov; si[tid] = oi; }
            }
            __syncthreads();
        }
        if (tid == 0) {
            row_out[m].value = sv[0];
            row_out[m].index = si[0];
            tokens[m] = si[0];
        }
        __syncthreads();
    }
    if (tid == 0) {
        const uint32_t n_drafts = batch - 1;
        uint32_t accepted = 0;
        for (uint32_t i = 0; i < n_drafts; ++i) {
            const int32_t target = tokens[i] >= 0 ? tokens[i] : eos;
            const int32_t draft = drafts_dev != nullptr ? drafts_dev[i] : drafts_val.v[i];
            if (target != draft) break;
            ++accepted;
        }
        const int32_t next = tokens[accepted] >= 0 ? tokens[accepted] : eos;
        accept_out[0] = static_cast<int32_t>(accepted);
        accept_out[1] = next;
    }
}

uint32_t lm_head_grid(uint32_t rows, uint32_t nb, uint32_t batch) {
    const int cus = device_cu_count();
    const uint32_t lds = x_lds_bytes(nb, batch);
    uint32_t per_cu = 4;
    if (lds <= kMaxXLdsBytes) {
        per_cu = 160u * 1024u / (lds + 1024u);
        if (per_cu > 4) per_cu = 4;
        if (per_cu < 1) per_cu = 1;
    }
    uint32_t grid = static_cast<uint32_t>(cus) * per_cu;
    const uint32_t max_wgs = (rows + kGemvWaves - 1) / kGemvWaves;
    if (grid > max_wgs) grid = max_wgs;
    if (grid > kMaxPartials) grid = kMaxPartials;
    if (grid == 0) grid = 1;
    return grid;
}

template <int M>
int launch_lm_head(const uint8_t *w, const uint8_t *y, uint32_t rows, uint32_t nb, uint32_t grid,
                   q8mi_argmax_pair *partial, float *logits, uint32_t stride_logits, hipStream_t stream) {
    const uint32_t lds = x_lds_bytes(nb, M);
    if (lds <= kMaxXLdsBytes) {
        lm_head_kernel<M, true><<<grid, kGemvThreads, lds, stream>>>(w, y, rows, nb, partial, logits, stride_logits);
    } else {
        lm_head_kernel<M, false><<<grid, kGemvThreads, 0, stream>>>(w, y, rows, nb, partial, logits, stride_logits);
    }
    return check_launch("lm_head");
}

}  // namespace
}  // namespace q8mi

using namespace q8mi;

extern "C" size_t q8mi_lm_head_scratch_bytes(uint32_t rows, uint32_t cols, uint32_t batch) {
    (void)rows;
    (void)cols;
    // one partial per workgroup and verify row; the grid never exceeds kMaxPartials
    return static_cast<size_t>(batch) * kMaxPartials * sizeof(q8mi_argmax_pair);
}

extern "C" int q8mi_lm_head_argmax_accept(const uint8_t *weight, const void *y, uint32_t rows,
                                          uint32_t cols, uint32_t batch, const int32_t *drafts,
                                          int drafts_on_device, int32_t eos, q8mi_argmax_pair *row_out,
                                          int32_t *accept_out, float *logits, uint32_t stride_logits,
                                          void *scratch, void *stream) {
    if (cols % kQK != 0 || cols == 0)
        return fail(Q8MI_REJECTED, "lm_head: cols %u not a positive multiple of 32", cols);
    if ((cols / kQK) % 8 != 0)
        return fail(Q8MI_REJECTED, "lm_head: cols %u not a multiple of 256 (unaligned planes)", cols);
    if (batch == 0 || batch > Q8MI_MAX_GEMV_BATCH)
        return fail(Q8MI_REJECTED, "lm_head: batch %u outside 1..8", batch);
    if (rows == 0 || rows > 0x7fffffffu) return fail(Q8MI_REJECTED, "lm_head: rows %u out of range", rows);
    if (batch > 1 && drafts == nullptr) return fail(Q8MI_REJECTED, "lm_head: drafts missing");
    if (reinterpret_cast<uintptr_t>(weight) % 16 != 0)
        return fail(Q8MI_REJECTED, "lm_head: weight pointer not 16-byte aligned");
    const uint32_t nb = cols / kQK;
    const uint32_t grid = lm_head_grid(rows, nb, batch);
    auto *partial = static_cast<q8mi_argmax_pair *>(scratch);
    const auto *yb = static_cast<const uint8_t *>(y);
    hipStream_t s = as_stream(stream);
    int rc = Q8MI_REJECTED;
    switch (batch) {
        case 1: rc = launch_lm_head<1>(weight, yb, rows, nb, grid, partial, logits, stride_logits, s); break;
        case 2: rc = launch_lm_head<2>(weight, yb, rows, nb, grid, partial, logits, stride_logits, s); break;
        case 3: rc = launch_lm_head<3>(weight, yb, rows, nb, grid, partial, logits, stride_logits, s); break;
        case 4: rc = launch_lm_head<4>(weight, yb, rows, nb, grid, partial, logits, stride_logits, s); break;
        case 5: rc = launch_lm_head<5>(weight, yb, rows, nb, grid, partial, logits, stride_logits, s); break;
        case 6: rc = launch_lm_head<6>(weight, yb, rows, nb, grid, partial, logits, stride_logits, s); break;
        case 7: rc = launch_lm_head<7>(weight, yb, rows, nb, grid, partial, logits, stride_logits, s); break;
        case 8: rc = launch_lm_head<8>(weight, yb, rows, nb, grid, partial, logits, stride_logits, s); break;
        default: break;
    }
    if (rc != Q8MI_OK) return rc;
    Drafts dv{};
    const int32_t *ddev = nullptr;
    if (batch > 1) {
        if (drafts_on_device) {
            ddev = drafts;
        } else {
            for (uint32_t i = 0; i + 1 < batch; ++i) dv.v[i] = drafts[i];
        }
    }
    lm_head_finalize_kernel<<<1, kMaxPartials, 0, s>>>(partial, grid, batch, dv, ddev, eos, row_out, accept_out);
    return check_launch("lm_head finalize");
}
