// Dequantizing row gather from a split-plane Q8_0 matrix (the embedding lookup
// that follows the LM-head argmax in greedy decoding).
// Reference: src/kernels_cuda.cu:2075-2087 (one row, fp32), :2089-2108 (bf16),
// :2110-2134 (row id taken from an ArgmaxPair slot on the device; an id outside
// the matrix gives a row of zeros), :2141-2190 (a batch of row ids held in a
// device array), called from :10613-10755.
//
// out[i] = fp32(d[i / 32]) * (float)q[i]: an fp16 value times an 8-bit integer
// is exact in fp32, so every output is bit-identical to the reference whatever
// the order of evaluation; the bf16 variant rounds that product to nearest even.
//
// One thread turns four consecutive quants (one dword) into four outputs: a
// wavefront reads 256 contiguous bytes of the quant plane and writes 1 KiB
// (fp32) or 512 B (bf16) contiguously.  Traffic per row is 34/32 B read and
// 4 B (2 B) written per element, so the kernel is write-bound.
#include "q8mi_device.hpp"
#include "q8mi_internal.hpp"

namespace q8mi {
namespace {

typedef unsigned v2u __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr uint32_t kThreads = 256;
constexpr uint32_t kPerThread = 4;

enum class RowSource { kImmediate, kIdArray, kArgmaxSlot };

struct GatherParams {
    const uint8_t *weight;
    void *out;
    const uint64_t *row_ids;        // kIdArray
    const q8mi_argmax_pair *pairs;  // kArgmaxSlot
    uint64_t row;                   // kImmediate
    uint64_t rows;
    uint64_t cols;
    uint32_t slot;
};

template <RowSource SRC, bool BF16>
__global__ __launch_bounds__(kThreads) void get_rows_kernel(const GatherParams p) {
    // grid.x carries the batch (a long prompt gathers more rows than grid.y may count)
    const uint64_t i = (static_cast<uint64_t>(blockIdx.y) * kThreads + threadIdx.x) * kPerThread;
    if (i >= p.cols) return;
    const uint32_t b = blockIdx.x;

    uint64_t row;
    bool valid;
    if constexpr (SRC == RowSource::kImmediate) {
        row = p.row;
        valid = true;  // checked on the host
    } else if constexpr (SRC == RowSource::kIdArray) {
        row = p.row_ids[b];
        valid = row < p.rows;
    } else {
        const int token = p.pairs[p.slot].index;
        valid = token >= 0 && static_cast<uint64_t>(token) < p.rows;
        row = valid ? static_cast<uint64_t>(token) : 0;
    }

    float v[kPerThread] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (valid) {
        const uint64_t nb = p.cols / 32;
        const uint8_t *base = p.weight + row * nb * 34;
        const float d = half_bits_to_float(reinterpret_cast<const uint16_t *>(base)[i / 32]);
        const uint8_t *qs = base + 2 * nb + i;
        int q4;
        if (nb % 2 == 0) {  // planes of every row start on a dword
            q4 = *reinterpret_cast<const int *>(qs);
        } else {
            q4 = qs[0] | (qs[1] << 8) | (qs[2] << 16) | (qs[3] << 24);
        }
#pragma unroll
        for (uint32_t e = 0; e < kPerThread; ++e) {
            const int q = (q4 << (24 - 8 * e)) >> 24;  // sign-extended byte e
            v[e] = d * static_cast<float>(q);
        }
    }

    const uint64_t o = static_cast<uint64_t>(b) * p.cols + i;
    if constexpr (BF16) {
        v2u w;
        w.x = float_to_bf16_bits(v[0]) | (static_cast<uint32_t>(float_to_bf16_bits(v[1])) << 16);
        w.y = float_to_bf16_bits(v[2]) | (static_cast<uint32_t>(float_to_bf16_bits(v[3])) << 16);
        *reinterpret_cast<v2u *>(static_cast<uint16_t *>(p.out) + o) = w;
    } else {
        v4f w = {v[0], v[1], v[2], v[3]};
        *reinterpret_cast<v4f *>(static_cast<float *>(p.out) + o) = w;
    }
}

template <RowSource SRC>
int launch(const GatherParams &p, uint32_t batch, bool bf16, void *stream, const char *what) {
    const uint64_t gy = (p.cols / kPerThread + kThreads - 1) / kThreads;
    if (gy > 65535u || batch > 0x7fffffffu) return fail(Q8MI_REJECTED, "%s: grid too large", what);
    const dim3 grid(batch, static_cast<uint32_t>(gy));
    if (bf16)
        get_rows_kernel<SRC, true><<<grid, kThreads, 0, as_stream(stream)>>>(p);
    else
        get_rows_kernel<SRC, false><<<grid, kThreads, 0, as_stream(stream)>>>(p);
    return check_launch(what);
}

int check_shape(const char *what, const uint8_t *weight, const void *out, uint64_t rows, uint64_t cols,
                bool bf16) {
    if (weight == nullptr || out == nullptr) return fail(Q8MI_REJECTED, "%s: null pointer", what);
    if (rows == 0 || cols == 0 || cols % 32 != 0)
        return fail(Q8MI_REJECTED, "%s: cols must be a positive multiple of 32 and rows positive", what);
    if (reinterpret_cast<uintptr_t>(weight) % 4 != 0)
        return fail(Q8MI_REJECTED, "%s: the matrix must be 4-byte aligned", what);
    if (reinterpret_cast<uintptr_t>(out) % (bf16 ? 8 : 16) != 0)
        return fail(Q8MI_REJECTED, "%s: output must be %d-byte aligned", what, bf16 ? 8 : 16);
    return Q8MI_OK;
}

}  // namespace
}  // namespace q8mi

using namespace q8mi;

extern "C" int q8mi_get_row(const uint8_t *weight, uint64_t row, uint64_t rows, uint64_t cols, void *out,
                            int out_is_bf16, void *stream) {
    if (int rc = check_shape("get_row", weight, out, rows, cols, out_is_bf16 != 0); rc != Q8MI_OK) return rc;
    if (row >= rows) return fail(Q8MI_REJECTED, "get_row: row %llu outside the matrix", (unsigned long long)row);
    GatherParams p{};
    p.weight = weight; p.out = out; p.row = row; p.rows = rows; p.cols = cols;
    return launch<RowSource::kImmediate>(p, 1, out_is_bf16 != 0, stream, "get_row");
}

extern "C" int q8mi_get_row_from_argmax(const uint8_t *weight, const q8mi_argmax_pair *argmaxes,
                                        uint32_t index, uint64_t rows, uint64_t cols, float *out,
                                        void *stream) {
    if (int rc = check_shape("get_row_from_argmax", weight, out, rows, cols, false); rc != Q8MI_OK) return rc;
    if (argmaxes == nullptr) return fail(Q8MI_REJECTED, "get_row_from_argmax: null argmax buffer");
    GatherParams p{};
    p.weight = weight; p.out = out; p.pairs = argmaxes; p.slot = index; p.rows = rows; p.cols = cols;
    return launch<RowSource::kArgmaxSlot>(p, 1, false, stream, "get_row_from_argmax");
}

extern "C" int q8mi_get_rows(const uint8_t *weight, const uint64_t *row_ids, uint32_t batch, uint64_t rows,
                             uint64_t cols, void *out, int out_is_bf16, void *stream) {
    if (batch == 0) return Q8MI_OK;
    if (int rc = check_shape("get_rows", weight, out, rows, cols, out_is_bf16 != 0); rc != Q8MI_OK) return rc;
    if (row_ids == nullptr) return fail(Q8MI_REJECTED, "get_rows: null row id array");
    GatherParams p{};
    p.weight = weight; p.out = out; p.row_ids = row_ids; p.rows = rows; p.cols = cols;
    return launch<RowSource::kIdArray>(p, batch, out_is_bf16 != 0, stream, "get_rows");
}
