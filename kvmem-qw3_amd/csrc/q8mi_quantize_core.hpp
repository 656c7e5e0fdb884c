// Per-lane pieces of the activation quantizers, shared by the stand-alone
// quantizer kernels and by the GEMV that quantizes its activations while staging
// them: both must produce the same bits.  A lane owns four consecutive floats,
// eight consecutive lanes own a 32-element block.
#pragma once

#include "q8mi_device.hpp"

namespace q8mi {

struct Float4 {
    float x, y, z, w;
};

template <bool VEC>
__device__ __forceinline__ Float4 load4(const float *p) {
    Float4 v;
    if (VEC) {
        const float4 t = *reinterpret_cast<const float4 *>(p);
        v.x = t.x; v.y = t.y; v.z = t.z; v.w = t.w;
    } else {
        v.x = p[0]; v.y = p[1]; v.z = p[2]; v.w = p[3];
    }
    return v;
}

__device__ __forceinline__ float group8_amax(const Float4 &v) {
    float m = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    m = fmaxf(m, swizzle_xor4(m));
    m = fmaxf(m, dpp_f32<kDppXor2>(m));
    m = fmaxf(m, dpp_f32<kDppXor1>(m));
    return m;
}

// __float2int_rn semantics: nearest-even, NaN -> 0 (v_cvt_i32_f32 saturates and
// maps NaN to 0; rintf first so the conversion itself is exact).
__device__ __forceinline__ int rn_int(float v) { return static_cast<int>(rintf(v)); }

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    return (static_cast<uint32_t>(a) & 0xffu) | ((static_cast<uint32_t>(b) & 0xffu) << 8) |
           ((static_cast<uint32_t>(c) & 0xffu) << 16) | ((static_cast<uint32_t>(d) & 0xffu) << 24);
}

// rint(x / d) for the lane's four values, with the IEEE quotient the reference computes.
// The division is replaced by x * (1/d) from the hardware reciprocal: that product is within
// a few ulp of the true quotient (|q| <= 127, so within 1e-4 absolute), hence rounds to the
// same integer unless it lies that close to a half-integer, overflowed or is NaN.  If any
// lane of the wave sees such a value, the whole wave takes the exact division instead
// (about one wave in twenty on random data), so the result is always the exact one.
__device__ __forceinline__ void rint_div4(const Float4 &v, float d, int &q0, int &q1, int &q2, int &q3) {
    const float r = __builtin_amdgcn_rcpf(d);
    float t0 = v.x * r, t1 = v.y * r, t2 = v.z * r, t3 = v.w * r;
    auto risky = [](float t) {
        const float frac = t - floorf(t);
        return !(fabsf(t) <= 127.5f) || fabsf(frac - 0.5f) < 1e-4f;
    };
    const bool any_risky = risky(t0) || risky(t1) || risky(t2) || risky(t3);
    if (__builtin_amdgcn_ballot_w64(any_risky) != 0) {   // wave-uniform
        t0 = v.x / d; t1 = v.y / d; t2 = v.z / d; t3 = v.w / d;
    }
    q0 = rn_int(t0); q1 = rn_int(t1); q2 = rn_int(t2); q3 = rn_int(t3);
}

// Q8_1 quantization of this lane's four values (reference: src/mmvq_q8.cu:82-112):
// d = amax / 127 kept unrounded for the division, q = rint(x / d); all eight lanes of the
// block must call it together, in wave-uniform control flow.  Returns the packed quants;
// d_out is the unrounded scale.
__device__ __forceinline__ uint32_t quantize4_q8_1(const Float4 &v, float &d_out) {
    const float amax = group8_amax(v);
    const float d = amax / 127.0f;
    int q0, q1, q2, q3;
    rint_div4(v, d, q0, q1, q2, q3);
    if (amax == 0.0f) q0 = q1 = q2 = q3 = 0;
    d_out = d;
    return pack4(q0, q1, q2, q3);
}

// Block sum of Q8_1 (the `s` field) for the lane's four values, with the reference's pairing
// (i, i+16), (i, i+8), (i, i+4), (i, i+2), (i, i+1) of its 32-lane xor butterfly
// (src/cuda_helpers.cuh:44-51): lane exchanges xor 4, 2, 1 cover the first three levels
// component-wise, the last two are the in-lane adds.  Same calling rules as quantize4_q8_1.
__device__ __forceinline__ float block_sum_q8_1(const Float4 &v) {
    float s0 = v.x, s1 = v.y, s2 = v.z, s3 = v.w;
    s0 += swizzle_xor4(s0); s1 += swizzle_xor4(s1); s2 += swizzle_xor4(s2); s3 += swizzle_xor4(s3);
    s0 += dpp_f32<kDppXor2>(s0); s1 += dpp_f32<kDppXor2>(s1);
    s2 += dpp_f32<kDppXor2>(s2); s3 += dpp_f32<kDppXor2>(s3);
    s0 += dpp_f32<kDppXor1>(s0); s1 += dpp_f32<kDppXor1>(s1);
    s2 += dpp_f32<kDppXor1>(s2); s3 += dpp_f32<kDppXor1>(s3);
    return (s0 + s2) + (s1 + s3);
}

// ---- RMS norm pieces (shared by the stand-alone kernels and the GEMV that normalises while
// staging, which must produce the same bits) ------------------------------------------------
// A row is cut into chunks of four consecutive floats (the last one zero-padded).  Thread t of
// the 256 adds the squares of chunks t, t + 256, t + 512, ... in that order, each chunk as
// fma(w, w, fma(z, z, fma(y, y, x * x))); the 256 partials are added as a balanced binary tree
// over the thread index (neighbours first).  scale = 1 / sqrt(sum / n + eps) with IEEE
// division and square root; an output is (x * scale) * weight, rounded after each product
// (the reference's expression, src/kernels_cuda.cu:1995-2007).
constexpr uint32_t kNormThreads = 256;

__device__ __forceinline__ float chunk_squares(const Float4 &v) {
    return fmaf(v.w, v.w, fmaf(v.z, v.z, fmaf(v.y, v.y, v.x * v.x)));
}

// Total of the 256 per-thread partials; `red` = four floats of LDS nobody else touches until
// the barrier that follows the caller's use of the result.  Contains one workgroup barrier.
__device__ __forceinline__ float block_tree_sum_256(float partial, float *red) {
    const float s = wave_sum(partial);   // balanced tree over the wave's 64 lanes
    if ((threadIdx.x & 63u) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

__device__ __forceinline__ float rms_scale(float sum_squares, uint32_t n, float eps) {
    return 1.0f / sqrtf(sum_squares / static_cast<float>(n) + eps);
}

__device__ __forceinline__ Float4 rms_apply(const Float4 &v, float scale, const Float4 &w) {
    Float4 r;
    r.x = (v.x * scale) * w.x;
    r.y = (v.y * scale) * w.y;
    r.z = (v.z * scale) * w.z;
    r.w = (v.w * scale) * w.w;
    return r;
}

}  // namespace q8mi
