// RMS norm of activation rows, alone or fused with the Q8_1 quantizer that feeds the
// Q8_0 GEMVs (the step in front of every projection group and of the LM head).
// Reference: rms_norm_kernel_vec / rms_norm_kernel (src/kernels_cuda.cu:1945-2010,
// 2057-2073), launched by rms_norm / rms_norm_batch (:14748-14816); the operators that
// pair it with the projections are rms_norm_q8_0_matmul_*fanout
// (include/qw3/device_backend.hpp:421-523).
//
//   out[j][i] = (x[j][i] * scale_j) * weight[i],  scale_j = 1 / sqrt(mean_i(x[j][i]^2) + eps)
//
// The reference leaves the order of the sum of squares to its block size and takes the
// root with the hardware's approximate reciprocal square root, so its last bits cannot be
// restated; this kernel fixes an order of its own (q8mi_quantize_core.hpp) and uses IEEE
// division and square root, which a CPU can follow bit for bit.
//
// One workgroup per row.  Many rows (a prefill chunk): 256 threads, the first six chunks of a
// thread stay in registers between the two passes (rows of up to 6144 columns are read once;
// longer rows are read again, from cache).  Few rows (decode, verify): 1024 threads with two
// chunks each, so that the serial part of a launch that occupies a handful of CUs -- the
// quantizer's arithmetic and lane exchanges per chunk -- is a quarter as long; the squares then
// meet in LDS, where the first 256 threads add them in the order the 256-thread form adds its
// own (chunks t, t + 256, ...), so both forms give the same bits.
#include <type_traits>

#include "q8mi_internal.hpp"
#include "q8mi_quantize_core.hpp"

namespace q8mi {
namespace {

constexpr uint32_t kHeld = 6;          // chunks a thread of the 256-thread form keeps
constexpr uint32_t kWideThreads = 1024;
constexpr uint32_t kWideHeld = 2;      // ... and of the 1024-thread form (rows of up to 8192 columns)
constexpr uint32_t kWideMaxBatch = 64; // rows up to which a launch takes the 1024-thread form

struct NormParams {
    const float *addend;   // ADD: the row normalised is x + addend ...
    float *sum_out;        // ... which is also written here (rows stride_x apart; may be x or addend)
    const float *x;
    const float *weight;
    float *out;      // may be null when y is set
    uint8_t *y;      // Q8_1 blocks [batch][cols / 32], or null
    uint32_t cols;
    uint32_t stride_x;
    uint32_t stride_out;
    float eps;
};

// Chunk c of a row of n floats; elements past the row's end read as zero.
template <bool VEC>
__device__ __forceinline__ Float4 load_chunk(const float *row, uint32_t c, uint32_t n) {
    if (VEC) return load4<true>(row + c * 4);   // n % 4 == 0
    Float4 v;
    const uint32_t i = c * 4;
    v.x = i < n ? row[i] : 0.0f;
    v.y = i + 1 < n ? row[i + 1] : 0.0f;
    v.z = i + 2 < n ? row[i + 2] : 0.0f;
    v.w = i + 3 < n ? row[i + 3] : 0.0f;
    return v;
}

template <bool VEC>
__device__ __forceinline__ void store_chunk(float *row, uint32_t c, uint32_t n, const Float4 &v) {
    const uint32_t i = c * 4;
    if (VEC) {
        *reinterpret_cast<float4 *>(row + i) = make_float4(v.x, v.y, v.z, v.w);
        return;
    }
    if (i < n) row[i] = v.x;
    if (i + 1 < n) row[i + 1] = v.y;
    if (i + 2 < n) row[i + 2] = v.z;
    if (i + 3 < n) row[i + 3] = v.w;
}

// ADD: the residual add in front of the norm runs in the same pass (the executors' add_n followed by
// rms_norm_batch, src/qwen_executor.cpp:6642-6674): a chunk is x + addend, rounded as the stand-alone
// add rounds it, and goes to sum_out as well.  A thread meets the same chunks in both passes, so the
// second pass of a long row reads back from sum_out what the thread itself stored in the first.
template <bool VEC, bool QUANT, bool ADD = false, uint32_t THREADS = kNormThreads>
__global__ __launch_bounds__(THREADS) void rms_norm_kernel(const NormParams p) {
    constexpr uint32_t HELD = THREADS == kNormThreads ? kHeld : kWideHeld;
    __shared__ float red[4];
    __shared__ float squares[THREADS == kNormThreads ? 1 : THREADS];
    const uint32_t j = blockIdx.x, t = threadIdx.x;
    const float *x = p.x + static_cast<uint64_t>(j) * p.stride_x;
    const uint32_t n = p.cols;
    const uint32_t chunks = (n + 3) / 4;
    const Float4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    const float *addend = ADD ? p.addend + static_cast<uint64_t>(j) * p.stride_x : nullptr;
    float *sum_out = ADD ? p.sum_out + static_cast<uint64_t>(j) * p.stride_x : nullptr;
    auto summed = [&](uint32_t c) {   // chunk c of the row to normalise (first pass)
        Float4 v = load_chunk<VEC>(x, c, n);
        if constexpr (ADD) {
            const Float4 a = load_chunk<VEC>(addend, c, n);
            v.x += a.x; v.y += a.y; v.z += a.z; v.w += a.w;
            store_chunk<VEC>(sum_out, c, n, v);
        }
        return v;
    };

    // the norm weights of the held chunks are requested together with x: one memory round trip, not two
    Float4 held[HELD], wheld[HELD];
    float partial = 0.0f;
#pragma unroll
    for (uint32_t u = 0; u < HELD; ++u) {
        const uint32_t c = u * THREADS + t;
        held[u] = c < chunks ? load_chunk<VEC>(x, c, n) : zero;
        wheld[u] = c < chunks ? load_chunk<VEC>(p.weight, c, n) : zero;
    }
    if constexpr (ADD) {   // all loads of the held chunks before the first store (which may be to x itself)
        Float4 aheld[HELD];
#pragma unroll
        for (uint32_t u = 0; u < HELD; ++u) {
            const uint32_t c = u * THREADS + t;
            aheld[u] = c < chunks ? load_chunk<VEC>(addend, c, n) : zero;
        }
#pragma unroll
        for (uint32_t u = 0; u < HELD; ++u) {
            const uint32_t c = u * THREADS + t;
            held[u].x += aheld[u].x; held[u].y += aheld[u].y; held[u].z += aheld[u].z; held[u].w += aheld[u].w;
            if (c < chunks) store_chunk<VEC>(sum_out, c, n, held[u]);
        }
    }
    float sum_squares;
    if constexpr (THREADS == kNormThreads) {
#pragma unroll
        for (uint32_t u = 0; u < HELD; ++u) partial += chunk_squares(held[u]);   // + 0 for chunks past the end
        for (uint32_t c = HELD * THREADS + t; c < chunks; c += THREADS)
            partial += chunk_squares(summed(c));
        sum_squares = block_tree_sum_256(partial, red);
    } else {
        // rounds of THREADS chunks: thread t of the first 256 adds the squares of chunks t, t + 256, ... of the
        // round in that order (+ 0 for chunks past the end, which leaves a sum of squares as it is)
        auto add_round = [&](float sq) {
            squares[t] = sq;
            __syncthreads();
            if (t < kNormThreads) {
#pragma unroll
                for (uint32_t u = 0; u < THREADS / kNormThreads; ++u) partial += squares[u * kNormThreads + t];
            }
            __syncthreads();
        };
#pragma unroll
        for (uint32_t u = 0; u < HELD; ++u) {
            if (u * THREADS < chunks) add_round(chunk_squares(held[u]));   // uniform
        }
        for (uint32_t base = HELD * THREADS; base < chunks; base += THREADS) {
            const uint32_t c = base + t;
            add_round(c < chunks ? chunk_squares(summed(c)) : 0.0f);
        }
        if (t < kNormThreads) {   // the first four waves: block_tree_sum_256's tree
            const float s = wave_sum(partial);
            if ((t & 63u) == 0) red[t >> 6] = s;
        }
        __syncthreads();
        sum_squares = (red[0] + red[1]) + (red[2] + red[3]);
    }
    const float scale = rms_scale(sum_squares, n, p.eps);

    // All lanes walk the same trips: the quantizer's lane exchanges need wave-uniform control flow
    // (cols % 32 == 0 there, so the eight lanes of a block are in or out together).
    auto emit = [&](uint32_t c, const Float4 &v, const Float4 &w) {
        const bool live = c < chunks;
        const Float4 r = rms_apply(v, scale, w);
        if (live && p.out != nullptr) store_chunk<VEC>(p.out + static_cast<uint64_t>(j) * p.stride_out, c, n, r);
        if constexpr (QUANT) {
            float d;
            const uint32_t packed = quantize4_q8_1(r, d);
            const float sum = block_sum_q8_1(r);
            if (live) {
                uint32_t *blk = reinterpret_cast<uint32_t *>(
                    p.y + (static_cast<uint64_t>(j) * (n / kQK) + c / 8) * kQ81Bytes);
                blk[1 + c % 8] = packed;
                if (c % 8 == 0)
                    blk[0] = static_cast<uint32_t>(float_to_half_bits(d)) |
                             (static_cast<uint32_t>(float_to_half_bits(sum)) << 16);
            }
        }
    };
#pragma unroll
    for (uint32_t u = 0; u < HELD; ++u) {
        if (u * THREADS < chunks) emit(u * THREADS + t, held[u], wheld[u]);   // uniform
    }
    for (uint32_t base = HELD * THREADS; base < chunks; base += THREADS) {
        const uint32_t c = base + t;
        const bool live = c < chunks;
        emit(c, live ? load_chunk<VEC>(ADD ? sum_out : x, c, n) : zero, live ? load_chunk<VEC>(p.weight, c, n) : zero);
    }
}

bool aligned16(const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

int launch(const char *what, const NormParams &p, uint32_t batch, void *stream) {
    if (p.x == nullptr || p.weight == nullptr) return fail(Q8MI_REJECTED, "%s: null pointer", what);
    if (batch == 0 || p.cols == 0) return Q8MI_OK;
    if (batch > 0x7fffffffu) return fail(Q8MI_REJECTED, "%s: batch %u too large for one launch", what, batch);
    const bool quant = p.y != nullptr;
    const bool add = p.addend != nullptr;
    const bool vec = p.cols % 4 == 0 && aligned16(p.x) && aligned16(p.weight) && p.stride_x % 4 == 0 &&
                     (p.out == nullptr || (aligned16(p.out) && p.stride_out % 4 == 0)) &&
                     (!add || (aligned16(p.addend) && aligned16(p.sum_out)));
    hipStream_t s = as_stream(stream);
    auto run = [&](auto vec_tag, auto quant_tag, auto add_tag) {
        constexpr bool V = decltype(vec_tag)::value, Q = decltype(quant_tag)::value, A = decltype(add_tag)::value;
        if (batch <= kWideMaxBatch && p.cols > 4 * kNormThreads)
            rms_norm_kernel<V, Q, A, kWideThreads><<<batch, kWideThreads, 0, s>>>(p);
        else
            rms_norm_kernel<V, Q, A, kNormThreads><<<batch, kNormThreads, 0, s>>>(p);
    };
    auto by_add = [&](auto vec_tag, auto quant_tag) {
        if (add) run(vec_tag, quant_tag, std::true_type{});
        else run(vec_tag, quant_tag, std::false_type{});
    };
    auto by_quant = [&](auto vec_tag) {
        if (quant) by_add(vec_tag, std::true_type{});
        else by_add(vec_tag, std::false_type{});
    };
    if (vec) by_quant(std::true_type{});
    else by_quant(std::false_type{});
    return check_launch(what);
}

}  // namespace
}  // namespace q8mi

using namespace q8mi;

extern "C" int q8mi_rms_norm(const float *x, const float *weight, float *out, uint32_t batch, uint32_t cols,
                             uint32_t stride_x_row, uint32_t stride_out_row, float eps, void *stream) {
    if (out == nullptr) return fail(Q8MI_REJECTED, "rms_norm: null output");
    NormParams p{};
    p.x = x; p.weight = weight; p.out = out; p.y = nullptr;
    p.cols = cols; p.stride_x = stride_x_row; p.stride_out = stride_out_row; p.eps = eps;
    return launch("rms_norm", p, batch, stream);
}

extern "C" int q8mi_rms_norm_quantize_q8_1(const float *x, const float *weight, float *normalized, void *y,
                                           uint32_t batch, uint32_t cols, uint32_t stride_x_row,
                                           uint32_t stride_normalized_row, float eps, void *stream) {
    if (cols % kQK != 0) return fail(Q8MI_REJECTED, "rms_norm_quantize_q8_1: cols %u not a multiple of 32", cols);
    if (y == nullptr) return fail(Q8MI_REJECTED, "rms_norm_quantize_q8_1: null output");
    NormParams p{};
    p.x = x; p.weight = weight; p.out = normalized; p.y = static_cast<uint8_t *>(y);
    p.cols = cols; p.stride_x = stride_x_row; p.stride_out = stride_normalized_row; p.eps = eps;
    return launch("rms_norm_quantize_q8_1", p, batch, stream);
}

extern "C" int q8mi_add_rms_norm(const float *a, const float *b, float *sum, const float *weight, float *normalized,
                                 void *y_q8_1, uint32_t batch, uint32_t cols, uint32_t stride_row,
                                 uint32_t stride_normalized_row, float eps, void *stream) {
    if (a == nullptr || b == nullptr || sum == nullptr) return fail(Q8MI_REJECTED, "add_rms_norm: null pointer");
    if (normalized == nullptr && y_q8_1 == nullptr) return fail(Q8MI_REJECTED, "add_rms_norm: no output");
    if (y_q8_1 != nullptr && cols % kQK != 0)
        return fail(Q8MI_REJECTED, "add_rms_norm: cols %u not a multiple of 32 (Q8_1 output)", cols);
    if (normalized != nullptr && (normalized == a || normalized == b || normalized == sum))
        return fail(Q8MI_REJECTED, "add_rms_norm: the normalised rows must not overlap the addends or the sum");
    NormParams p{};
    p.x = a; p.addend = b; p.sum_out = sum; p.weight = weight; p.out = normalized; p.y = static_cast<uint8_t *>(y_q8_1);
    p.cols = cols; p.stride_x = stride_row; p.stride_out = stride_normalized_row; p.eps = eps;
    return launch("add_rms_norm", p, batch, stream);
}
