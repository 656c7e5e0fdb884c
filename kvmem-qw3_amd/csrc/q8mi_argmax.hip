// Row argmax kernels for gfx950.
// Reference: src/kernels_cuda.cu:1693-1734 (single row -> {index, bits}),
// :1804-1857 (single row -> ArgmaxPair slot), :1765-1802 + :1859-1888 (batched,
// two stages).  Ties go to the lowest index everywhere.
//
// The batched pair keeps the reference's reduction network (a 256-wide and a
// 1024-wide LDS tree comparing slot t with slot t+stride) so that rows holding
// NaN resolve to the same element as the reference's kernels.
#include <mutex>

#include "q8mi_device.hpp"
#include "q8mi_internal.hpp"

// Partial results of the single-row argmax of a long row (one per first-stage workgroup): a row of
// a vocabulary's length is more than one CU reads quickly, and the reference's entry points for a
// single row carry no scratch argument (src/kernels_cuda.cu:20750-20790).  Every GPU holds its own
// copy; host code uses the address hipGetSymbolAddress returns for the current device.
constexpr unsigned kArgmaxSplitGroups = 128;
static __device__ __align__(256) q8mi_argmax_pair argmax_split_partials[kArgmaxSplitGroups];

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

// ---- long single rows: two stages ---------------------------------------------------------------
// Stage 1: workgroup g scans elements [g * span, (g + 1) * span) (span a multiple of 4, so that a
// 16-byte aligned row stays aligned) with the single-row rule and leaves its winner in partial[g];
// stage 2: one workgroup merges the partials with the same rule.  NaN never wins a `>` and equal
// values go to the lower index at every merge, so the result is that of the one-workgroup scan.
constexpr uint32_t kSplitThreads = 256;
// Shorter rows: one workgroup.  Two launches take 5.6 us whatever the length; one workgroup takes
// 3.6 us for 32 000 elements and 11 us for 248 320, i.e. as long as the two from about 90 000.
constexpr uint64_t kSplitFrom = 81920;

__global__ __launch_bounds__(kSplitThreads) void argmax_split_stage1(const float *__restrict__ x, uint64_t n, uint64_t span,
                                                                   q8mi_argmax_pair *__restrict__ partial) {
    const uint64_t lo = blockIdx.x * span, hi = lo + span < n ? lo + span : n;
    Best b{-INFINITY, -1};
    if (reinterpret_cast<uintptr_t>(x) % 16 == 0) {
        const uint64_t c0 = lo / 4, c1 = hi / 4;   // whole float4 chunks of the range (lo is a multiple of 4)
        const float4 *x4 = reinterpret_cast<const float4 *>(x);
        for (uint64_t c = c0 + threadIdx.x; c < c1; c += kSplitThreads) {
            const float4 q = x4[c];
            const int i = static_cast<int>(c * 4);
            if (q.x > b.v) { b.v = q.x; b.i = i; }
            if (q.y > b.v) { b.v = q.y; b.i = i + 1; }
            if (q.z > b.v) { b.v = q.z; b.i = i + 2; }
            if (q.w > b.v) { b.v = q.w; b.i = i + 3; }
        }
        for (uint64_t i = c1 * 4 + threadIdx.x; i < hi; i += kSplitThreads) {   // the row's last n % 4 elements
            const float v = x[i];
            if (v > b.v) { b.v = v; b.i = static_cast<int>(i); }
        }
    } else {
        for (uint64_t i = lo + threadIdx.x; i < hi; i += kSplitThreads) {
            const float v = x[i];
            if (v > b.v) { b.v = v; b.i = static_cast<int>(i); }
        }
    }
    __shared__ float sv[kSplitThreads];
    __shared__ int si[kSplitThreads];
    sv[threadIdx.x] = b.v;
    si[threadIdx.x] = b.i;
    __syncthreads();
    for (uint32_t stride = kSplitThreads / 2; stride > 0; stride >>= 1) {
        if (threadIdx.x < stride) {
            const float ov = sv[threadIdx.x + stride];
            const int oi = si[threadIdx.x + stride];
            if (beats_single(ov, oi, sv[threadIdx.x], si[threadIdx.x])) { sv[threadIdx.x] = ov; si[threadIdx.x] = oi; }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        partial[blockIdx.x].value = sv[0];
        partial[blockIdx.x].index = si[0];
    }
}

// out2 != nullptr: {index, bits of the value}; else pair_out[out_index] = {value, index}
__global__ __launch_bounds__(kArgmaxSplitGroups) void argmax_split_stage2(const q8mi_argmax_pair *__restrict__ partial,
                                                                        uint32_t groups, int32_t *__restrict__ out2,
                                                                        q8mi_argmax_pair *__restrict__ pair_out,
                                                                        uint32_t out_index) {
    __shared__ float sv[kArgmaxSplitGroups];
    __shared__ int si[kArgmaxSplitGroups];
    float v = -INFINITY;
    int i = -1;
    if (threadIdx.x < groups) {
        v = partial[threadIdx.x].value;
        i = partial[threadIdx.x].index;
    }
    sv[threadIdx.x] = v;
    si[threadIdx.x] = i;
    __syncthreads();
    for (uint32_t stride = kArgmaxSplitGroups / 2; stride > 0; stride >>= 1) {
        if (threadIdx.x < stride) {
            const float ov = sv[threadIdx.x + stride];
            const int oi = si[threadIdx.x + stride];
            if (beats_single(ov, oi, sv[threadIdx.x], si[threadIdx.x])) { sv[threadIdx.x] = ov; si[threadIdx.x] = oi; }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        if (out2 != nullptr) {
            out2[0] = si[0];
            out2[1] = __builtin_bit_cast(int32_t, sv[0]);
        } else {
            pair_out[out_index].value = sv[0];
            pair_out[out_index].index = si[0];
        }
    }
}

// This device's copy of the partials array (looked up once per device, with that device current).
int split_partials_of_current_device(q8mi_argmax_pair **out) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void *ptr_of[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return fail(Q8MI_LAUNCH_ERROR, "argmax: no current device, or a device id beyond %d", kMaxDevices - 1);
    }
    std::lock_guard<std::mutex> lock(mu);
    if (ptr_of[dev] == nullptr) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(argmax_split_partials));
        if (e != hipSuccess || p == nullptr) {
            (void)hipGetLastError();
            return fail(Q8MI_LAUNCH_ERROR, "argmax: hipGetSymbolAddress: %s", hipGetErrorString(e));
        }
        ptr_of[dev] = p;
    }
    *out = static_cast<q8mi_argmax_pair *>(ptr_of[dev]);
    return Q8MI_OK;
}

int launch_split(const float *x, uint64_t n, int32_t *out2, q8mi_argmax_pair *pair_out, uint32_t out_index,
                 hipStream_t stream) {
    q8mi_argmax_pair *partial = nullptr;
    if (int rc = split_partials_of_current_device(&partial)) return rc;
    // at least 2048 elements per workgroup, in whole float4 chunks
    uint64_t span = (n + kArgmaxSplitGroups - 1) / kArgmaxSplitGroups;
    span = span < 2048 ? 2048 : (span + 3) / 4 * 4;
    const uint32_t groups = static_cast<uint32_t>((n + span - 1) / span);
    argmax_split_stage1<<<groups, kSplitThreads, 0, stream>>>(x, n, span, partial);
    if (int rc = check_launch("argmax stage 1")) return rc;
    argmax_split_stage2<<<1, kArgmaxSplitGroups, 0, stream>>>(partial, groups, out2, pair_out, out_index);
    return check_launch("argmax stage 2");
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
    if (n >= kSplitFrom && n <= 0x7fffffffull) return launch_split(x, n, out2, nullptr, 0, as_stream(stream));
    argmax_kernel<<<1, kRowThreads, 0, as_stream(stream)>>>(x, n, out2);
    return check_launch("argmax");
}

extern "C" int q8mi_argmax_to_pair(const float *x, uint64_t n, q8mi_argmax_pair *out, uint32_t out_index,
                                void *stream) {
    if (n >= kSplitFrom && n <= 0x7fffffffull) return launch_split(x, n, nullptr, out, out_index, as_stream(stream));
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
