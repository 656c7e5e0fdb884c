// Row argmax kernels for gfx950.
// Reference: src/kernels_cuda.cu:1693-1734 (single row -> {index, bits}),
// :1804-1857 (single row -> ArgmaxPair slot), :1765-1802 + :1859-1888 (batched,
// two stages).  Ties go to the lowest index everywhere.
//
// The batched pair keeps the reference's reduction network (a 256-wide and a
// 1024-wide LDS tree comparing slot t with slot t+stride) so that rows holding
// NaN resolve to the same element as the reference's kernels.
#include "q8mi_device.hpp"
#include "q8mi_internal.hpp"

namespace q8mi {
namespace {

constexpr int kRowThreads = 1024;
constexpr uint32_t kStage1Block = 256;
constexpr uint32_t kStage2Block = 1024;

struct Best {
    float v;
    int i;
};

// single-row rule (src/kernels_cuda.cu:1708-1713): strictly greater wins, equal
// values go to the lower index
__device__ __forceinline__ bool beats_single(float ov, int oi, float v, int i) {
    return ov > v || (ov == v && oi < i);
}

// batched rule (src/kernels_cuda.cu:1765-1771)
__device__ __forceinline__ bool beats_pair(float ov, int oi, float v, int i) {
    if (oi < 0) return false;
    if (i < 0) return true;
    if (ov > v) return true;
    return ov == v && oi < i;
}

__device__ __forceinline__ Best single_row_scan(const float *__restrict__ x, uint64_t n) {
    Best b{-INFINITY, -1};
    // per-thread strided scan; a thread meets its elements in ascending order so
    // `>` alone keeps the lowest index among equals.  NaN never wins a `>`, so which thread
    // meets which element does not change the result: rows on a 16-byte boundary are read
    // four elements per load (one workgroup reads a 248 320-element row in 11 us instead of 34).
    if (reinterpret_cast<uintptr_t>(x) % 16 == 0) {
        const uint64_t n4 = n / 4;
        const float4 *x4 = reinterpret_cast<const float4 *>(x);
        for (uint64_t c = threadIdx.x; c < n4; c += kRowThreads) {
            const float4 q = x4[c];
            const int i = static_cast<int>(c * 4);
            if (q.x > b.v) { b.v = q.x; b.i = i; }
            if (q.y > b.v) { b.v = q.y; b.i = i + 1; }
            if (q.z > b.v) { b.v = q.z; b.i = i + 2; }
            if (q.w > b.v) { b.v = q.w; b.i = i + 3; }
        }
        for (uint64_t i = n4 * 4 + threadIdx.x; i < n; i += kRowThreads) {   // the last n % 4 elements
            const float v = x[i];
            if (v > b.v) { b.v = v; b.i = static_cast<int>(i); }
        }
    } else {
        for (uint64_t i = threadIdx.x; i < n; i += kRowThreads) {
            const float v = x[i];
            if (v > b.v) { b.v = v; b.i = static_cast<int>(i); }
        }
    }
    __shared__ float sv[kRowThreads];
    __shared__ int si[kRowThreads];
    sv[threadIdx.x] = b.v;
    si[threadIdx.x] = b.i;
    __syncthreads();
    for (uint32_t stride = kRowThreads / 2; stride > 0; stride >>= 1) {
        if (threadIdx.x < stride) {
            const float ov = sv[threadIdx.x + stride];
            const int oi = si[threadIdx.x + stride];
            if (beats_single(ov, oi, sv[threadIdx.x], si[threadIdx.x])) {
                sv[threadIdx.x] = ov;
                si[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    return Best{sv[0], si[0]};
}

__global__ __launch_bounds__(kRowThreads) void argmax_kernel(const float *__restrict__ x, uint64_t n,
                                                             int32_t *__restrict__ out2) {
    const Best b = single_row_scan(x, n);
    if (threadIdx.x == 0) {
        out2[0] = b.i;
        out2[1] = __builtin_bit_cast(int32_t, b.v);
    }
}

__global__ __launch_bounds__(kRowThreads) void argmax_pair_kernel(const float *__restrict__ x, uint64_t n,
                                                                  q8mi_argmax_pair *__restrict__ out,
                                                                  uint32_t out_index) {
    const Best b = single_row_scan(x, n);
    if (threadIdx.x == 0) {
        out[out_index].value = b.v;
        out[out_index].index = b.i;
    }
}

template <uint32_t BLOCK>
__device__ __forceinline__ Best lds_tree(float v, int i) {
    __shared__ float sv[BLOCK];
    __shared__ int si[BLOCK];
    const uint32_t tid = threadIdx.x;
    sv[tid] = v;
    si[tid] = i;
    __syncthreads();
    for (uint32_t stride = BLOCK / 2; stride > 0; stride >>= 1) {
        if (tid < stride) {
            const float ov = sv[tid + stride];
            const int oi = si[tid + stride];
            if (beats_pair(ov, oi, sv[tid], si[tid])) {
                sv[tid] = ov;
                si[tid] = oi;
            }
        }
        __syncthreads();
    }
    return Best{sv[0], si[0]};
}

__global__ __launch_bounds__(kStage1Block) void argmax_rows_stage1(const float *__restrict__ x,
                                                                  q8mi_argmax_pair *__restrict__ partial,
                                                                  uint32_t row_stride,
                                                                  uint32_t blocks_per_row) {
    const uint32_t row = blockIdx.y;
    const uint32_t col = blockIdx.x * kStage1Block + threadIdx.x;
    const bool in = col < row_stride;
    const float v = in ? x[static_cast<uint64_t>(row) * row_stride + col] : -INFINITY;
    const Best b = lds_tree<kStage1Block>(v, in ? static_cast<int>(col) : -1);
    if (threadIdx.x == 0) {
        q8mi_argmax_pair *p = partial + static_cast<uint64_t>(row) * blocks_per_row + blockIdx.x;
        p->value = b.v;
        p->index = b.i;
    }
}

__global__ __launch_bounds__(kStage2Block) void argmax_rows_stage2(const q8mi_argmax_pair *__restrict__ partial,
                                                                  q8mi_argmax_pair *__restrict__ result,
                                                                  uint32_t blocks_per_row) {
    const uint32_t row = blockIdx.x;
    float v = -INFINITY;
    int i = -1;
    if (threadIdx.x < blocks_per_row) {
        const q8mi_argmax_pair p = partial[static_cast<uint64_t>(row) * blocks_per_row + threadIdx.x];
        v = p.value;
        i = p.index;
    }
    const Best b = lds_tree<kStage2Block>(v, i);
    if (threadIdx.x == 0) {
        result[row].value = b.v;
        result[row].index = b.i;
    }
}

}  // namespace
}  // namespace q8mi

using namespace q8mi;

extern "C" int q8mi_argmax(const float *x, uint64_t n, int32_t *out2, void *stream) {
    argmax_kernel<<<1, kRowThreads, 0, as_stream(stream)>>>(x, n, out2);
    return check_launch("argmax");
}

extern "C" int q8mi_argmax_to_pair(const float *x, uint64_t n, q8mi_argmax_pair *out, uint32_t out_index,
                                void *stream) {
    argmax_pair_kernel<<<1, kRowThreads, 0, as_stream(stream)>>>(x, n, out, out_index);
    return check_launch("argmax_pair");
}

extern "C" size_t q8mi_argmax_rows_scratch_bytes(uint32_t batch, uint32_t row_stride) {
    const uint32_t bpr = (row_stride + kStage1Block - 1) / kStage1Block;
    return static_cast<size_t>(batch) * bpr * sizeof(q8mi_argmax_pair);
}

extern "C" int q8mi_argmax_rows(const float *x, uint32_t batch, uint32_t row_stride, void *scratch,
                                q8mi_argmax_pair *result, void *stream) {
    if (batch == 0) return Q8MI_OK;
    const uint32_t bpr = (row_stride + kStage1Block - 1) / kStage1Block;
    if (row_stride == 0 || bpr > kStage2Block)
        return fail(Q8MI_REJECTED, "argmax_rows: row_stride %u outside 1..%u", row_stride,
                    kStage1Block * kStage2Block);
    if (batch > 65535u) return fail(Q8MI_REJECTED, "argmax_rows: batch %u above 65535", batch);
    auto *partial = static_cast<q8mi_argmax_pair *>(scratch);
    argmax_rows_stage1<<<dim3(bpr, batch), kStage1Block, 0, as_stream(stream)>>>(x, partial, row_stride, bpr);
    if (int rc = check_launch("argmax_rows stage 1")) return rc;
    argmax_rows_stage2<<<batch, kStage2Block, 0, as_stream(stream)>>>(partial, result, bpr);
    return check_launch("argmax_rows stage 2");
}
