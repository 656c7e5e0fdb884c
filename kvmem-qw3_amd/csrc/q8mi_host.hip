// Host-side pieces of the library: error text, device queries, the weight
// repack (host and device) and the small elementwise kernels.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "q8mi_device.hpp"
#include "q8mi_internal.hpp"

namespace q8mi {

namespace {
thread_local char g_err[256] = "";
}

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return Q8MI_OK;
    return fail(Q8MI_LAUNCH_ERROR, "%s: %s", what, hipGetErrorString(e));
}

int device_cu_count() {
    static thread_local int cached_dev = -1;
    static thread_local int cached_cus = 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (dev != cached_dev) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        cached_dev = dev;
        cached_cus = cus;
    }
    return cached_cus;
}

namespace {

// ---- device repack: interleaved 34-B blocks -> split-plane rows ------------
// One thread moves one block: 2 scale bytes + 32 quant bytes (the source block
// is only 2-byte aligned, so it is read as 17 halfwords).
__global__ __launch_bounds__(256) void repack_kernel(const uint16_t *__restrict__ in,
                                                     uint8_t *__restrict__ out, uint64_t rows,
                                                     uint64_t nb) {
    const uint64_t b = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (b >= rows * nb) return;
    const uint64_t row = b / nb, kb = b % nb;
    const uint16_t *src = in + b * 17;
    uint8_t *row_out = out + row * nb * 34;
    reinterpret_cast<uint16_t *>(row_out)[kb] = src[0];
    uint16_t *q = reinterpret_cast<uint16_t *>(row_out + 2 * nb + kb * 32);
#pragma unroll
    for (int t = 0; t < 16; ++t) q[t] = src[1 + t];
}

// ---- fp32 -> bf16 (round to nearest even), for bf16 activations downstream ----
__global__ __launch_bounds__(256) void f32_to_bf16_kernel(const float *__restrict__ in,
                                                          uint16_t *__restrict__ out, uint64_t n) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) out[i] = float_to_bf16_bits(in[i]);
}

// ---- elementwise add: out = a + b (fp32), or bf16(f32(a) + f32(b)) rounded to nearest even ----
// Four (fp32) or eight (bf16) elements per thread when the three pointers are 16-byte aligned.
template <bool BF16>
__global__ __launch_bounds__(256) void add_kernel(void *__restrict__ out_v, const void *a_v, const void *b_v, uint64_t n,
                                                  bool vec) {
    constexpr uint32_t kPer = BF16 ? 8 : 4;
    const uint64_t i0 = (static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x) * kPer;
    if (i0 >= n) return;
    if constexpr (BF16) {
        uint16_t *out = static_cast<uint16_t *>(out_v);
        const uint16_t *a = static_cast<const uint16_t *>(a_v), *b = static_cast<const uint16_t *>(b_v);
        if (vec && i0 + kPer <= n) {
            const uint4 av = *reinterpret_cast<const uint4 *>(a + i0), bv = *reinterpret_cast<const uint4 *>(b + i0);
            const uint32_t aw[4] = {av.x, av.y, av.z, av.w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
            uint32_t r[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float lo = bf16_bits_to_float(static_cast<uint16_t>(aw[k] & 0xffffu)) +
                                 bf16_bits_to_float(static_cast<uint16_t>(bw[k] & 0xffffu));
                const float hi = bf16_bits_to_float(static_cast<uint16_t>(aw[k] >> 16)) +
                                 bf16_bits_to_float(static_cast<uint16_t>(bw[k] >> 16));
                r[k] = static_cast<uint32_t>(float_to_bf16_bits(lo)) | (static_cast<uint32_t>(float_to_bf16_bits(hi)) << 16);
            }
            *reinterpret_cast<uint4 *>(out + i0) = make_uint4(r[0], r[1], r[2], r[3]);
        } else {
            for (uint64_t i = i0; i < n && i < i0 + kPer; ++i)
                out[i] = float_to_bf16_bits(bf16_bits_to_float(a[i]) + bf16_bits_to_float(b[i]));
        }
    } else {
        float *out = static_cast<float *>(out_v);
        const float *a = static_cast<const float *>(a_v), *b = static_cast<const float *>(b_v);
        if (vec && i0 + kPer <= n) {
            const float4 av = *reinterpret_cast<const float4 *>(a + i0), bv = *reinterpret_cast<const float4 *>(b + i0);
            *reinterpret_cast<float4 *>(out + i0) = make_float4(av.x + bv.x, av.y + bv.y, av.z + bv.z, av.w + bv.w);
        } else {
            for (uint64_t i = i0; i < n && i < i0 + kPer; ++i) out[i] = a[i] + b[i];
        }
    }
}

// ---- elementwise SwiGLU: out = silu(gate) * up, silu(g) = g / (1 + exp(-g)) --------------------
// Four elements per thread when the three pointers are 16-byte aligned.
__global__ __launch_bounds__(256) void silu_mul_kernel(float *out, const float *gate, const float *up, uint64_t n, bool vec) {
    const uint64_t i0 = (static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
    if (i0 >= n) return;
    auto f = [](float g, float u) { return (g / (1.0f + __expf(-g))) * u; };
    if (vec && i0 + 4 <= n) {
        const float4 g = *reinterpret_cast<const float4 *>(gate + i0), u = *reinterpret_cast<const float4 *>(up + i0);
        *reinterpret_cast<float4 *>(out + i0) = make_float4(f(g.x, u.x), f(g.y, u.y), f(g.z, u.z), f(g.w, u.w));
    } else {
        for (uint64_t i = i0; i < n && i < i0 + 4; ++i) out[i] = f(gate[i], up[i]);
    }
}

}  // namespace
}  // namespace q8mi

using namespace q8mi;

extern "C" const char *q8mi_last_error(void) { return g_err; }

extern "C" int q8mi_abi_version(void) { return 1; }

extern "C" int q8mi_repack_q8_0_split_host(const void *gguf_blocks, uint64_t rows, uint64_t cols,
                                           void *split_out) {
    if (cols % kQK != 0) return fail(Q8MI_REJECTED, "repack: cols %llu not a multiple of 32", (unsigned long long)cols);
    const uint64_t nb = cols / kQK;
    const uint8_t *in = static_cast<const uint8_t *>(gguf_blocks);
    uint8_t *out = static_cast<uint8_t *>(split_out);
    for (uint64_t r = 0; r < rows; ++r) {
        const uint8_t *src = in + r * nb * 34;
        uint8_t *d_plane = out + r * nb * 34;
        uint8_t *q_plane = d_plane + 2 * nb;
        for (uint64_t b = 0; b < nb; ++b, src += 34) {
            memcpy(d_plane + 2 * b, src, 2);
            memcpy(q_plane + 32 * b, src + 2, 32);
        }
    }
    return Q8MI_OK;
}

extern "C" int q8mi_repack_q8_0_split(const void *gguf_blocks, uint64_t rows, uint64_t cols,
                                      void *split_out, void *stream) {
    if (cols % kQK != 0) return fail(Q8MI_REJECTED, "repack: cols %llu not a multiple of 32", (unsigned long long)cols);
    if (gguf_blocks == split_out) return fail(Q8MI_REJECTED, "repack: in-place repack is not supported");
    const uint64_t nb = cols / kQK;
    const uint64_t blocks = rows * nb;
    if (blocks == 0) return Q8MI_OK;
    const uint64_t grid = (blocks + 255) / 256;
    if (grid > 0x7fffffffull) return fail(Q8MI_REJECTED, "repack: tensor too large for one launch");
    repack_kernel<<<static_cast<uint32_t>(grid), 256, 0, as_stream(stream)>>>(
        static_cast<const uint16_t *>(gguf_blocks), static_cast<uint8_t *>(split_out), rows, nb);
    return check_launch("repack");
}

extern "C" int q8mi_f32_to_bf16(const float *in, uint16_t *out, uint64_t n, void *stream) {
    if (n == 0) return Q8MI_OK;
    const uint64_t grid = (n + 255) / 256;
    if (grid > 0x7fffffffull) return fail(Q8MI_REJECTED, "f32_to_bf16: too many elements for one launch");
    f32_to_bf16_kernel<<<static_cast<uint32_t>(grid), 256, 0, as_stream(stream)>>>(in, out, n);
    return check_launch("f32_to_bf16");
}

extern "C" int q8mi_add(void *out, const void *a, const void *b, uint64_t n, int is_bf16, void *stream) {
    if (n == 0) return Q8MI_OK;
    if (out == nullptr || a == nullptr || b == nullptr) return fail(Q8MI_REJECTED, "add: null pointer");
    const uint64_t per = is_bf16 ? 8 : 4;
    const uint64_t grid = ((n + per - 1) / per + 255) / 256;
    if (grid > 0x7fffffffull) return fail(Q8MI_REJECTED, "add: too many elements for one launch");
    const bool vec = (reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) % 16 == 0;
    if (is_bf16)
        add_kernel<true><<<static_cast<uint32_t>(grid), 256, 0, as_stream(stream)>>>(out, a, b, n, vec);
    else
        add_kernel<false><<<static_cast<uint32_t>(grid), 256, 0, as_stream(stream)>>>(out, a, b, n, vec);
    return check_launch("add");
}

extern "C" int q8mi_silu_mul(float *out, const float *gate, const float *up, uint64_t n, void *stream) {
    if (n == 0) return Q8MI_OK;
    if (out == nullptr || gate == nullptr || up == nullptr) return fail(Q8MI_REJECTED, "silu_mul: null pointer");
    const uint64_t grid = ((n + 3) / 4 + 255) / 256;
    if (grid > 0x7fffffffull) return fail(Q8MI_REJECTED, "silu_mul: too many elements for one launch");
    const bool vec = (reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(up)) % 16 == 0;
    silu_mul_kernel<<<static_cast<uint32_t>(grid), 256, 0, as_stream(stream)>>>(out, gate, up, n, vec);
    return check_launch("silu_mul");
}
