// Device-side helpers shared by the gfx950 kernels: wave64 cross-lane
// primitives (DPP), fp16/bf16 conversion and the int8 dot instruction.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace q8mi {

constexpr int kWave = 64;
constexpr int kQK = 32;         // elements per Q8 block
constexpr int kQ81Bytes = 36;   // half d, half s, 32 x int8
constexpr int kD4Bytes = 144;   // float d4[4], 128 x int8

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// Bit reinterpretation through by-value scalars.  (Applying __builtin_bit_cast
// directly to an element of an ext_vector, e.g. r[v] or q.x, makes this compiler
// read element 0 for every index, so vector elements always go through these.)
__device__ __forceinline__ float as_f32(int v) { return __builtin_bit_cast(float, v); }
__device__ __forceinline__ int as_i32(float v) { return __builtin_bit_cast(int, v); }

// ---- DPP lane exchanges ---------------------------------------------------
// quad_perm selectors: lane i of every quad reads lane perm[i].
constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;
constexpr int kDppRowShl4 = 0x104;     // lane i of every row of 16 reads lane i + 4
constexpr int kDppRowShr4 = 0x114;     // lane i of every row of 16 reads lane i - 4

template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return as_f32(dpp_i32<CTRL>(as_i32(v)));
}

// xor-4 exchange inside 32-lane groups (ds_swizzle bit-mask mode:
// and_mask 0x1f, or_mask 0, xor_mask 4; no LDS memory is touched).
__device__ __forceinline__ float swizzle_xor4(float v) {
    return as_f32(__builtin_amdgcn_ds_swizzle(as_i32(v), (4 << 10) | 0x1f));
}

// Sum over the 64 lanes of a wave in a fixed order; every lane returns the total.
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f32<kDppXor1>(v);
    v += dpp_f32<kDppXor2>(v);
    v += dpp_f32<kDppRowHalfMirror>(v);
    v += dpp_f32<kDppRowMirror>(v);
    // every lane of a 16-lane row now holds its row's sum
    const float r0 = as_f32(__builtin_amdgcn_readlane(as_i32(v), 0));
    const float r1 = as_f32(__builtin_amdgcn_readlane(as_i32(v), 16));
    const float r2 = as_f32(__builtin_amdgcn_readlane(as_i32(v), 32));
    const float r3 = as_f32(__builtin_amdgcn_readlane(as_i32(v), 48));
    return (r0 + r1) + (r2 + r3);
}

// xor-D lane exchange, D = 1, 2 by DPP, 4..16 by ds_swizzle (bit-mask mode, no
// LDS memory touched), 32 by ds_bpermute.
template <int D>
__device__ __forceinline__ float lane_xor(float v) {
    if (D == 1) return dpp_f32<kDppXor1>(v);
    if (D == 2) return dpp_f32<kDppXor2>(v);
    if (D == 32) {
        const int lane = static_cast<int>(threadIdx.x) & 63;
        return as_f32(__builtin_amdgcn_ds_bpermute(((lane ^ 32) << 2), as_i32(v)));
    }
    return as_f32(__builtin_amdgcn_ds_swizzle(as_i32(v), (D << 10) | 0x1f));
}

// Sums V per-lane values across the wave "transposed": on return, lane l holds
// the wave-wide total of v[l % VP] (VP = V rounded up to a power of two).  Each
// stage halves the number of live values by letting the two lanes of an
// exchange pair keep one value each, so the whole reduction costs about 4*V
// instructions instead of 12*V for V independent wave sums.  The order of the
// additions is fixed.
template <int VP, int D = 1>
struct TransposeReduce {
    static __device__ __forceinline__ float run(float (&v)[VP], uint32_t lane) {
        if constexpr (VP == 1) {
            float t = v[0];
            if constexpr (D <= 1) t += lane_xor<1>(t);
            if constexpr (D <= 2) t += lane_xor<2>(t);
            if constexpr (D <= 4) t += lane_xor<4>(t);
            if constexpr (D <= 8) t += lane_xor<8>(t);
            if constexpr (D <= 16) t += lane_xor<16>(t);
            if constexpr (D <= 32) t += lane_xor<32>(t);
            return t;
        } else {
            const bool hi = lane & D;
            float h[VP / 2];
#pragma unroll
            for (int i = 0; i < VP / 2; ++i) {
                const float keep = hi ? v[2 * i + 1] : v[2 * i];
                const float send = hi ? v[2 * i] : v[2 * i + 1];
                h[i] = keep + lane_xor<D>(send);
            }
            return TransposeReduce<VP / 2, D * 2>::run(h, lane);
        }
    }
};

constexpr int pow2_at_least(int v) { return v <= 1 ? 1 : 2 * pow2_at_least((v + 1) / 2); }

// ---- conversions ----------------------------------------------------------
__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
    return static_cast<float>(__builtin_bit_cast(_Float16, h));
}

__device__ __forceinline__ uint16_t float_to_half_bits(float f) {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));  // v_cvt_f16_f32, RNE
}

__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
    const uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fffu;
    return static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

__device__ __forceinline__ float bf16_bits_to_float(uint16_t h) {
    return __builtin_bit_cast(float, static_cast<uint32_t>(h) << 16);
}

// ---- int8 dot products ------------------------------------------------------
// 16 int8 x 16 int8 -> int32, four v_dot4 (the first one in its three-operand
// form with a literal zero, which saves initialising an accumulator register).
__device__ __forceinline__ int dot16(const v4i &a, const v4i &b) {
    int acc;
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(acc) : "v"(a.x), "v"(b.x));
    acc = __builtin_amdgcn_sdot4(a.y, b.y, acc, false);
    acc = __builtin_amdgcn_sdot4(a.z, b.z, acc, false);
    acc = __builtin_amdgcn_sdot4(a.w, b.w, acc, false);
    return acc;
}

__device__ __forceinline__ int dot16(const v4i &a, const v4i &b, int acc) {
    acc = __builtin_amdgcn_sdot4(a.x, b.x, acc, false);
    acc = __builtin_amdgcn_sdot4(a.y, b.y, acc, false);
    acc = __builtin_amdgcn_sdot4(a.z, b.z, acc, false);
    acc = __builtin_amdgcn_sdot4(a.w, b.w, acc, false);
    return acc;
}

}  // namespace q8mi
