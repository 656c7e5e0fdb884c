// Instruments for the tests and the bench (see q8mi_support.h): seeded input generators, the
// int32 block-dot checker kernel, and the read / copy / matrix-unit kernels that measured ceilings
// come from.  Built into libq8mi_support.so; the product library holds none of this.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <thread>
#include <vector>

#include "q8mi_support.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int kOk = 0, kRejected = 1, kLaunchError = 2;
constexpr int kQK = 32, kQ81Bytes = 36, kD4Bytes = 144;

thread_local char g_err[256] = "";

__attribute__((format(printf, 2, 3))) int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return kOk;
    return fail(kLaunchError, "%s: %s", what, hipGetErrorString(e));
}

int cu_count() {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        return 256;
    return cus;
}

hipStream_t as_stream(void *s) { return static_cast<hipStream_t>(s); }

// by value: a bit cast applied to a vector element directly reads the vector's first bytes
__device__ __forceinline__ float bits_as_f32(int v) { return __builtin_bit_cast(float, v); }

// ---- checker: int32 block dots on the GPU ------------------------------------
__global__ __launch_bounds__(256) void block_dots_kernel(const uint8_t *__restrict__ w, const uint8_t *__restrict__ y,
                                                         int layout, uint32_t nb, uint32_t batch,
                                                         const uint32_t *__restrict__ sr, const uint32_t *__restrict__ sj,
                                                         const uint32_t *__restrict__ sk, uint32_t n,
                                                         int32_t *__restrict__ out) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint32_t row = sr[i], j = sj[i], kb = sk[i];
    const uint16_t *wq = reinterpret_cast<const uint16_t *>(w + static_cast<uint64_t>(row) * nb * 34 + 2 * nb +
                                                            static_cast<uint64_t>(kb) * 32);
    const uint8_t *xq8 = layout == 0
        ? y + (static_cast<uint64_t>(j) * nb + kb) * kQ81Bytes + 4
        : y + (static_cast<uint64_t>(kb / 4) * batch + j) * kD4Bytes + 16 + (kb % 4) * 32;
    const int *xq = reinterpret_cast<const int *>(xq8);
    int s = 0;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const int a = static_cast<int>(wq[2 * t]) | (static_cast<int>(wq[2 * t + 1]) << 16);
        s = __builtin_amdgcn_sdot4(a, xq[t], s, false);
    }
    out[i] = s;
}

// ---- plain streaming read -------------------------------------------------------
// Every lane reads 16 bytes per trip, the grid covers the buffer with a grid-stride loop; the
// xor of everything read goes to sink[0] only if it is a value that cannot occur, so the loads
// cannot be optimised away.
__global__ __launch_bounds__(256) void probe_read_kernel(const v4i *__restrict__ p, uint64_t n16,
                                                         uint32_t *__restrict__ sink) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * 256;
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    v4i a = {0, 0, 0, 0};
    for (; i + 3 * stride < n16; i += 4 * stride) {
        // streaming ("nt") loads, as the GEMV's weight loads
        const v4i v0 = __builtin_nontemporal_load(p + i), v1 = __builtin_nontemporal_load(p + i + stride),
                  v2 = __builtin_nontemporal_load(p + i + 2 * stride), v3 = __builtin_nontemporal_load(p + i + 3 * stride);
        a.x ^= v0.x ^ v1.x ^ v2.x ^ v3.x;
        a.y ^= v0.y ^ v1.y ^ v2.y ^ v3.y;
        a.z ^= v0.z ^ v1.z ^ v2.z ^ v3.z;
        a.w ^= v0.w ^ v1.w ^ v2.w ^ v3.w;
    }
    for (; i < n16; i += stride) {
        const v4i v = p[i];
        a.x ^= v.x; a.y ^= v.y; a.z ^= v.z; a.w ^= v.w;
    }
    if ((a.x ^ a.y ^ a.z ^ a.w) == 0x5a17c0de && (a.x & a.y) == 0x0badf00d) sink[0] = 1;
}

// Plain copy, 16 bytes per lane per trip: HBM reads and writes are both exactly `bytes`.
__global__ __launch_bounds__(256) void probe_copy_kernel(const v4i *__restrict__ src, v4i *__restrict__ dst,
                                                         uint64_t n16) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * 256;
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// ---- matrix-unit issue rates -----------------------------------------------------
// Four independent int8 MFMAs per round, optionally with NV independent scalar FMAs.
template <int NV>
__global__ __launch_bounds__(256) void probe_mfma_kernel(int *__restrict__ out, uint32_t iters, float a, float b) {
    v4i va = {static_cast<int>(threadIdx.x), 1, 2, 3}, vb = {4, 5, 6, static_cast<int>(threadIdx.x)};
    v16i c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    float x[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) x[k] = static_cast<float>(threadIdx.x + k);
    for (uint32_t i = 0; i < iters; ++i) {
        c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(va, vb, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(va, vb, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(va, vb, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(va, vb, c3, 0, 0, 0);
#pragma unroll
        for (int k = 0; k < NV; ++k) x[k % 8] = fmaf(x[k % 8], a, b);
    }
    int s = 0;
#pragma unroll
    for (int v = 0; v < 16; ++v) s += c0[v] + c1[v] + c2[v] + c3[v];
    float f = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k) f += x[k];
    out[blockIdx.x * 256 + threadIdx.x] = s + static_cast<int>(f);
}

// The arithmetic of a GEMM that needs ONE vector FMA per (output, block): per round and 32 x 32
// patch, the block sums come out of the fp16 matrix unit as fp32 (int8 values are exact in fp16 and
// a sum of 32 products below 2^24 is exact in fp32: two K = 16 instructions), the scale products
// d_w * d_y out of the fp32 matrix unit as four 4x4x1 outer-product instructions (16 blocks of
// 4 x 4 each: lane l gets a[4 (l/4) + v] * b[l] in register v, which is the layout of the sums),
// and acc += sum * product is the one FMA.  Operands are loop-invariant registers: nothing but the
// two pipes is measured.
__global__ __launch_bounds__(256, 2) void probe_mfma_one_fma_kernel(int *__restrict__ out, uint32_t iters, float a, float b) {
    // one activation fragment and four weight fragments (two K = 16 halves each), four weight scales
    v8h ya[2], wb[4][2];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        ya[0][k] = static_cast<_Float16>(static_cast<int>(threadIdx.x % 7) - 3 + k);
        ya[1][k] = static_cast<_Float16>(static_cast<int>(threadIdx.x % 5) - 2 - k);
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            wb[p][0][k] = static_cast<_Float16>(static_cast<int>(threadIdx.x % 3) + p - k);
            wb[p][1][k] = static_cast<_Float16>(static_cast<int>(threadIdx.x % 11) - p + k);
        }
    }
    float acc[4][16];
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[p][v] = 0.0f;
    const v16f zero16 = {0};
    const v4f zero4 = {0, 0, 0, 0};
    float dy[4], dw[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        dy[g] = a + static_cast<float>(threadIdx.x + g) * 1e-3f;
        dw[g] = b + static_cast<float>(g) * 1e-2f;
    }
    for (uint32_t i = 0; i < iters; ++i) {
        // opaque to the optimiser: every round and every patch has operands of its own, as in a
        // kernel that reads them from LDS
        asm volatile("" : "+v"(ya[0]), "+v"(ya[1]));
#pragma unroll
        for (int p = 0; p < 4; ++p) asm volatile("" : "+v"(wb[p][0]), "+v"(wb[p][1]), "+v"(dw[p]), "+v"(dy[p]));
        v16f s[4];
        v4f pr[4][4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            s[p] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ya[0], wb[p][0], zero16, 0, 0, 0);
            s[p] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ya[1], wb[p][1], s[p], 0, 0, 0);
#pragma unroll
            for (int g = 0; g < 4; ++g) pr[p][g] = __builtin_amdgcn_mfma_f32_4x4x1f32(dy[g], dw[p], zero4, 0, 0, 0);
        }
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[p][v] = fmaf(s[p][v], pr[p][v / 4][v % 4], acc[p][v]);
    }
    float f = 0.0f;
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int v = 0; v < 16; ++v) f += acc[p][v];
    out[blockIdx.x * 256 + threadIdx.x] = static_cast<int>(f);
}

// The int8 kernel's own arithmetic with its dependences: four int8 MFMAs seeded with 1.5 * 2^23 and
// the two FMAs per sum that consume their results (g = fma(F, d_w, -1.5 * 2^23 * d_w), acc += g * d_y).
__global__ __launch_bounds__(256, 2) void probe_mfma_two_fma_kernel(int *__restrict__ out, uint32_t iters, float a, float b) {
    v4i ya = {static_cast<int>(threadIdx.x), 1, 2, 3}, wb[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) wb[p] = v4i{4 + p, 5, 6, static_cast<int>(threadIdx.x)};
    v16i seed;
#pragma unroll
    for (int v = 0; v < 16; ++v) seed[v] = 0x4B400000;
    asm volatile("" : "+v"(seed));   // kept in registers, as in the kernel
    float acc[4][16];
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[p][v] = 0.0f;
    float dy[16], dw[4];
#pragma unroll
    for (int v = 0; v < 16; ++v) dy[v] = a + static_cast<float>(v) * 1e-3f;
#pragma unroll
    for (int p = 0; p < 4; ++p) dw[p] = b + static_cast<float>(p) * 1e-2f;
    for (uint32_t i = 0; i < iters; ++i) {
        asm volatile("" : "+v"(ya));
#pragma unroll
        for (int p = 0; p < 4; ++p) asm volatile("" : "+v"(wb[p]), "+v"(dw[p]));
#pragma unroll
        for (int v = 0; v < 16; ++v) asm volatile("" : "+v"(dy[v]));
        v16i r[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) r[p] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ya, wb[p], seed, 0, 0, 0);
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const float cw = -12582912.0f * dw[p];
#pragma unroll
            for (int v = 0; v < 16; ++v)
                acc[p][v] = fmaf(fmaf(bits_as_f32(r[p][v]), dw[p], cw), dy[v], acc[p][v]);
        }
    }
    float f = 0.0f;
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int v = 0; v < 16; ++v) f += acc[p][v];
    out[blockIdx.x * 256 + threadIdx.x] = static_cast<int>(f);
}

// ---- synthetic inputs --------------------------------------------------------
inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

inline uint64_t draw(uint64_t seed, uint64_t stream, uint64_t i) {
    return splitmix64(splitmix64(seed * 0xD1342543DE82EF95ull + stream) + i);
}

// uniform in (0, 1): 53 random bits, never 0
inline double unit(uint64_t bits) { return (static_cast<double>(bits >> 11) + 0.5) * (1.0 / 9007199254740992.0); }

// standard normal from two independent draws (Box-Muller, cosine branch)
inline double normal(uint64_t seed, uint64_t stream, uint64_t i) {
    const double u1 = unit(draw(seed, stream, 2 * i));
    const double u2 = unit(draw(seed, stream, 2 * i + 1));
    return sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2);
}

template <typename F>
void parallel_rows(uint64_t rows, int threads, F fn) {
    if (threads < 1) threads = 1;
    if (static_cast<uint64_t>(threads) > rows) threads = rows ? static_cast<int>(rows) : 1;
    if (threads == 1) {
        fn(0, rows);
        return;
    }
    std::vector<std::thread> pool;
    const uint64_t chunk = (rows + threads - 1) / threads;
    for (int t = 0; t < threads; ++t) {
        const uint64_t lo = chunk * t, hi = lo + chunk < rows ? lo + chunk : rows;
        if (lo >= hi) break;
        pool.emplace_back([=] { fn(lo, hi); });
    }
    for (auto &th : pool) th.join();
}

inline uint16_t f32_to_f16_host(float f) { return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f)); }

}  // namespace

extern "C" const char *q8sup_last_error(void) { return g_err; }

extern "C" int q8sup_block_dots(const uint8_t *weight, const void *y, int y_layout, uint32_t rows, uint32_t cols,
                                uint32_t batch, const uint32_t *sample_row, const uint32_t *sample_j,
                                const uint32_t *sample_kb, uint32_t n, int32_t *out, void *stream) {
    (void)rows;
    if (cols % kQK != 0) return fail(kRejected, "block_dots: cols %u not a multiple of 32", cols);
    if (y_layout != 0 && y_layout != 1) return fail(kRejected, "block_dots: unknown layout %d", y_layout);
    if (y_layout == 1 && cols % 128 != 0) return fail(kRejected, "block_dots: D4 needs cols %% 128 == 0");
    if (n == 0) return kOk;
    block_dots_kernel<<<(n + 255) / 256, 256, 0, as_stream(stream)>>>(
        weight, static_cast<const uint8_t *>(y), y_layout, cols / kQK, batch, sample_row, sample_j, sample_kb, n, out);
    return check_launch("block_dots");
}

extern "C" int q8sup_probe_read(const void *buf, uint64_t bytes, uint32_t wgs_per_cu, uint32_t *sink, void *stream) {
    if (bytes % 16 != 0 || reinterpret_cast<uintptr_t>(buf) % 16 != 0)
        return fail(kRejected, "probe_read: buffer must be 16-byte aligned and sized");
    if (wgs_per_cu == 0 || wgs_per_cu > 64) return fail(kRejected, "probe_read: wgs_per_cu outside 1..64");
    const uint32_t grid = static_cast<uint32_t>(cu_count()) * wgs_per_cu;
    probe_read_kernel<<<grid, 256, 0, as_stream(stream)>>>(static_cast<const v4i *>(buf), bytes / 16, sink);
    return check_launch("probe_read");
}

extern "C" int q8sup_probe_copy(const void *src, void *dst, uint64_t bytes, void *stream) {
    if (bytes % 16 != 0 || reinterpret_cast<uintptr_t>(src) % 16 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0)
        return fail(kRejected, "probe_copy: buffers must be 16-byte aligned and sized");
    const uint32_t grid = static_cast<uint32_t>(cu_count()) * 8;
    probe_copy_kernel<<<grid, 256, 0, as_stream(stream)>>>(static_cast<const v4i *>(src), static_cast<v4i *>(dst),
                                                           bytes / 16);
    return check_launch("probe_copy");
}

extern "C" size_t q8sup_probe_mfma_sink_bytes(void) {
    return static_cast<size_t>(cu_count()) * 2 * 256 * sizeof(int32_t);
}

extern "C" int q8sup_probe_mfma(int mode, uint32_t iters, int32_t *sink, uint64_t *ops_out, void *stream) {
    if (sink == nullptr || iters == 0) return fail(kRejected, "probe_mfma: null sink or zero rounds");
    const uint32_t grid = static_cast<uint32_t>(cu_count()) * 2;
    hipStream_t s = as_stream(stream);
    switch (mode) {
        case 0: probe_mfma_kernel<0><<<grid, 256, 0, s>>>(sink, iters, 1.0001f, 0.5f); break;
        case 1: probe_mfma_kernel<128><<<grid, 256, 0, s>>>(sink, iters, 1.0001f, 0.5f); break;
        case 2: probe_mfma_one_fma_kernel<<<grid, 256, 0, s>>>(sink, iters, 1.0001f, 0.5f); break;
        case 3: probe_mfma_two_fma_kernel<<<grid, 256, 0, s>>>(sink, iters, 1.0001f, 0.5f); break;
        default: return fail(kRejected, "probe_mfma: unknown mode %d", mode);
    }
    if (ops_out) *ops_out = static_cast<uint64_t>(grid) * 4 * iters * 4 * 2ull * 32 * 32 * 32;
    return check_launch("probe_mfma");
}

extern "C" int q8sup_synth_f32(float *out, uint64_t rows, uint64_t cols, uint64_t seed, int kind, float scale,
                               uint32_t outlier_ppm, float outlier_gain, int threads) {
    if (kind != 0 && kind != 1) return fail(kRejected, "synth_f32: unknown kind %d", kind);
    parallel_rows(rows, threads, [=](uint64_t lo, uint64_t hi) {
        for (uint64_t r = lo; r < hi; ++r) {
            for (uint64_t c = 0; c < cols; ++c) {
                const uint64_t i = r * cols + c;
                double v;
                if (kind == 0) {
                    v = normal(seed, 0, i);
                } else {
                    // Student-t(3) = Z / sqrt(chi2_3 / 3); unit variance after / sqrt(3)
                    const double z = normal(seed, 0, i);
                    const double a = normal(seed, 1, i), b = normal(seed, 2, i), d = normal(seed, 3, i);
                    const double chi2 = a * a + b * b + d * d;
                    v = z / sqrt(chi2 / 3.0) / 1.7320508075688772;
                    if (outlier_ppm != 0 && draw(seed, 4, c) % 1000000ull < outlier_ppm) v *= outlier_gain;
                }
                out[i] = static_cast<float>(v * scale);
            }
        }
    });
    return kOk;
}

extern "C" int q8sup_synth_q8_0_weight(uint8_t *split_out, uint64_t rows, uint64_t cols, uint64_t seed, float sigma,
                                       int threads) {
    if (cols % kQK != 0)
        return fail(kRejected, "synth_q8_0_weight: cols %llu not a multiple of 32", (unsigned long long)cols);
    const uint64_t nb = cols / kQK;
    parallel_rows(rows, threads, [=](uint64_t lo, uint64_t hi) {
        float blk[kQK];
        for (uint64_t r = lo; r < hi; ++r) {
            uint8_t *d_plane = split_out + r * nb * 34;
            int8_t *q_plane = reinterpret_cast<int8_t *>(d_plane + 2 * nb);
            for (uint64_t kb = 0; kb < nb; ++kb) {
                float amax = 0.0f;
                for (int t = 0; t < kQK; ++t) {
                    blk[t] = static_cast<float>(normal(seed, 0, r * cols + kb * kQK + t) * sigma);
                    amax = fmaxf(amax, fabsf(blk[t]));
                }
                const float d = amax / 127.0f;
                const float d_inv = d == 0.0f ? 0.0f : 1.0f / d;
                const uint16_t hd = f32_to_f16_host(d);
                memcpy(d_plane + 2 * kb, &hd, 2);
                for (int t = 0; t < kQK; ++t) {
                    long q = lrintf(blk[t] * d_inv);
                    q = q < -127 ? -127 : (q > 127 ? 127 : q);
                    q_plane[kb * kQK + t] = static_cast<int8_t>(q);
                }
            }
        }
    });
    return kOk;
}
