// Q8_0 weight x Q8_1 activation GEMV for batch 1..8 on gfx950.
// Reference semantics: src/mmvq_q8.cu:193-280 (plain), :295-399 (two weights),
// :414-519 (SwiGLU), :528-606 (residual add), :976-1068 (four-weight fan-out).
//
// The weights are read exactly once from HBM and nothing else is large, so every kernel here is a
// stream over the int8 plane of each row.  This file holds the entry points, the routing between
// the kernel families, and two of the families:
//   batch 1..4 (by batch, row length and form: gemv_prefers_mfma in q8mi_gemv_core.hpp): many small
//       workgroups that own whole row pairs, handed out by the dispatcher (q8mi_gemv_pairs.hip)
//   batch 2..16 otherwise: the matrix-core kernel below (core in q8mi_gemv_mfma_core.hpp), one workgroup per
//       CU whose waves split the items of its units and combine partial sums through LDS
//   fallbacks: the dot-product kernel below (core in q8mi_gemv_core.hpp) with the same static
//       split, for activations that fit LDS in no other layout, and a one-lane-per-block kernel
//       for rows whose planes are not 16-byte aligned (cols / 32 not a multiple of 8)
// Store / add / bf16 are wave-uniform and run once per unit, so they are a runtime switch; SwiGLU
// changes which rows a unit streams and is a template parameter (its launches also show up under
// their own kernel name in a profile).
#include "q8mi_gemv_core.hpp"
#include "q8mi_gemv_mfma_core.hpp"
#include "q8mi_gemv_params.hpp"

namespace q8mi {
namespace {

// Each wave parks the (possibly partial) sums of the units it touched in LDS;
// after a barrier the workgroup adds the partials of every unit in wave order and
// writes the results out, all threads in parallel.
//
// Unit u covers rows R*u .. R*u+R-1 of the concatenated row space; for SwiGLU it
// covers rows (R/2)*u .. of BOTH weights: slots 0..R/2-1 are gate rows, slots
// R/2..R-1 the matching up rows.
template <int M, int THREADS, int XMODE, bool SILU>
__global__ __launch_bounds__(THREADS) void gemv_kernel(const GemvParams p) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int R = RowsPerUnit<M>::value;
    constexpr uint32_t kPerUnit = M * R;
    constexpr uint32_t kWaves = THREADS / kWave;
    const uint32_t lane = threadIdx.x % kWave;
    // wave index as a scalar, so that row bookkeeping stays in SGPRs
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t nsteps = (p.nb * 2 + 127) / 128;
    const uint64_t row_bytes = static_cast<uint64_t>(p.nb) * 34;
    const UnitSeq useq = group_units(p.units, blockIdx.x, gridDim.x, p.interleave);
    const uint32_t ucount = useq.count;
    const uint32_t n_items = ucount * nsteps;
    uint32_t i0, i1;
    wave_items(n_items, wave, kWaves, i0, i1);
    float *park_base = reinterpret_cast<float *>(smem + p.x_bytes);   // [wave][kParkFloats]
    float *my_park = park_base + wave * kParkFloats;
    const uint32_t last_row = p.total_rows - 1;

    auto rows_of = [&](uint32_t u, RowPtrs<R> &rp) {
        if constexpr (SILU) {
#pragma unroll
            for (int r = 0; r < R / 2; ++r) {
                uint32_t row = (R / 2) * u + r;
                row = row < last_row ? row : last_row;   // ragged tail: re-read the last row
                rp.p[r] = p.w[0] + row * row_bytes;
                rp.p[R / 2 + r] = p.w[1] + row * row_bytes;
            }
        } else {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t row = R * u + r;
                row = row < last_row ? row : last_row;
                const RowRef a = resolve_row(p, row);
                rp.p[r] = a.w + a.local * row_bytes;
            }
        }
    };
    auto park = [&](uint32_t kk, float total) {
        if (lane < kPerUnit) my_park[kk * kPerUnit + lane] = total;
    };
    const XIn in{p.y};
    gemv_stream<M, R, THREADS, XMODE>(smem, in, p.nb, useq, i0, i1, rows_of, park);
    __syncthreads();

    // combine + write-out: entry e = (unit ordinal k, activation row m, slot r)
    auto total_of = [&](uint32_t k, uint32_t mr) {
        float t = 0.0f;
        for (uint32_t w = 0; w < kWaves; ++w) {
            uint32_t a0, a1;
            wave_items(n_items, w, kWaves, a0, a1);
            if (a1 <= a0) continue;
            const uint32_t kf = a0 / nsteps, kl = (a1 - 1) / nsteps;   // units wave w touched
            if (k >= kf && k <= kl) t += park_base[w * kParkFloats + (k - kf) * kPerUnit + mr];
        }
        return t;
    };
    if constexpr (SILU) {
        constexpr uint32_t kHalf = R / 2;
        for (uint32_t e = threadIdx.x; e < ucount * M * kHalf; e += THREADS) {
            const uint32_t k = e / (M * kHalf), m = (e / kHalf) % M, r = e % kHalf;
            const uint32_t row = kHalf * useq.unit(k) + r;
            if (row >= p.total_rows) continue;
            const float g = total_of(k, m * R + r);
            const float up = total_of(k, m * R + kHalf + r);
            const float silu = g / (1.0f + __expf(-g));
            static_cast<float *>(p.dst[0])[static_cast<uint64_t>(m) * p.stride[0] + row] = silu * up;
        }
    } else {
        for (uint32_t e = threadIdx.x; e < ucount * kPerUnit; e += THREADS) {
            const uint32_t k = e / kPerUnit, mr = e % kPerUnit;
            const uint32_t m = mr / R, r = mr % R;
            const uint32_t row = R * useq.unit(k) + r;
            if (row >= p.total_rows) continue;
            const RowRef ref = resolve_row(p, row);
            store_out(p.mode, ref.dst, static_cast<uint64_t>(m) * ref.stride + ref.local, total_of(k, mr));
        }
    }
}

// ---- matrix-core variant for batch 3..32 (see q8mi_gemv_mfma_core.hpp) --------------------------
// Unit u covers rows 4u .. 4u+3 of the concatenated row space; for SwiGLU gate rows 2u, 2u+1
// (fragment rows 0, 1) and the matching up rows (fragment rows 2, 3).
// ITEMWISE: the workgroup's items are dealt round-robin to its waves (see mfma_stream) and every
// item's sums are parked, [item][fragment row][activation row]; otherwise a wave takes a contiguous
// range of items and parks once per unit it touched.
template <int MG, int THREADS, bool SILU, bool HS, bool D4, int DEPTH, bool STREAMING, bool ITEMWISE>
__global__ __launch_bounds__(THREADS) void gemv_mfma_kernel(const GemvParams p, uint32_t batch,
                                                            uint32_t park_floats) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr uint32_t MP = 4 * MG;
    constexpr uint32_t kWaves = THREADS / kWave;
    constexpr uint32_t kPerUnit = 4 * kMfmaUnitRows * MP;   // [chunk][row][activation row]
    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t c = lane >> 2, r = lane & 3u;   // after the stream: chunk and fragment row of lanes 0 .. 15
    const uint32_t nitems = (p.nb + kMfmaItemBlocks - 1) / kMfmaItemBlocks;
    const uint64_t row_bytes = static_cast<uint64_t>(p.nb) * 34;
    const UnitSeq useq = group_units(p.units, blockIdx.x, gridDim.x, p.interleave);
    const uint32_t ucount = useq.count;
    const uint32_t n_items = ucount * nitems;
    uint32_t i0, i1;
    if constexpr (ITEMWISE) {
        i0 = wave < n_items ? wave : n_items;
        i1 = n_items;
    } else {
        wave_items(n_items, wave, kWaves, i0, i1);
    }
    float *park_base = reinterpret_cast<float *>(smem + p.x_bytes);   // [wave][park_floats], or [item][kMfmaUnitRows][MP]
    float *my_park = park_base + wave * park_floats;
    const uint32_t last_row = p.total_rows - 1;

    auto row_ptr = [&](uint32_t u) -> const uint8_t * {   // fragment row r is the one this lane loads
        if constexpr (SILU) {
            uint32_t row = 2 * u + (r & 1u);
            row = row < last_row ? row : last_row;
            return (r < 2 ? p.w[0] : p.w[1]) + row * row_bytes;
        } else {
            uint32_t row = 4 * u + r;
            row = row < last_row ? row : last_row;
            const RowRef a = resolve_row(p, row);
            return a.w + a.local * row_bytes;
        }
    };
    auto park = [&](uint32_t kk, auto &acc) {
        if (lane < 16) {
            float *dst = my_park + kk * kPerUnit + (c * kMfmaUnitRows + r) * MP;
#pragma unroll
            for (int g = 0; g < MG; ++g) {
                float4 v;
                v.x = acc[g][0]; v.y = acc[g][1]; v.z = acc[g][2]; v.w = acc[g][3];
                *reinterpret_cast<float4 *>(dst + 4 * g) = v;
            }
        }
    };
    // the wave's t-th item is item wave + t kWaves of the workgroup; lane (rho, q odd, n) holds the
    // total for fragment row n and activation row (q >> 1) + 2 rho (MG 2) or rho (MG 1)
    auto park_item = [&](uint32_t t, float total) {
        const uint32_t rho = lane >> 4, q = (lane >> 2) & 3u, n = lane & 3u;
        const uint32_t m = MG == 2 ? (q >> 1) + 2 * rho : rho;
        if (MG == 2 ? (q & 1u) != 0 : q == 1)
            park_base[(wave + t * kWaves) * (kMfmaUnitRows * MP) + n * MP + m] = total;
    };
    __shared__ uint32_t s_kf[kWaves], s_kl[kWaves];
    if constexpr (ITEMWISE) {
        (void)park;
        (void)park_floats;
        mfma_stream<MG, THREADS, HS, D4, DEPTH, STREAMING, true>(smem, p.y, p.nb, batch, p.x_stride, useq, i0, i1, row_ptr, park_item);
        __syncthreads();
    } else {
        mfma_stream<MG, THREADS, HS, D4, DEPTH, STREAMING>(smem, p.y, p.nb, batch, p.x_stride, useq, i0, i1, row_ptr, park);
        __syncthreads();
        // unit ranges of the waves, worked out once (wave w touched unit ordinals kf[w] .. kl[w])
        if (threadIdx.x < kWaves) {
            uint32_t a0, a1;
            wave_items(n_items, threadIdx.x, kWaves, a0, a1);
            s_kf[threadIdx.x] = a1 > a0 ? a0 / nitems : 1u;
            s_kl[threadIdx.x] = a1 > a0 ? (a1 - 1) / nitems : 0u;   // empty range: kf > kl
        }
        __syncthreads();
    }
    // total for unit ordinal k, fragment row rr, activation row m: the unit's items in order, or the
    // waves' partials in wave order, chunks in order
    auto total_of = [&](uint32_t k, uint32_t rr, uint32_t m) {
        float t = 0.0f;
        if constexpr (ITEMWISE) {
            const float *e = park_base + static_cast<size_t>(k) * nitems * (kMfmaUnitRows * MP) + rr * MP + m;
            for (uint32_t part = 0; part < nitems; ++part) t += e[part * (kMfmaUnitRows * MP)];
        } else {
#pragma unroll
            for (uint32_t w = 0; w < kWaves; ++w) {
                const uint32_t kf = s_kf[w], kl = s_kl[w];
                if (k < kf || k > kl) continue;
                const float *e = park_base + w * park_floats + (k - kf) * kPerUnit + rr * MP + m;
                t += ((e[0] + e[kMfmaUnitRows * MP]) + e[2 * kMfmaUnitRows * MP]) + e[3 * kMfmaUnitRows * MP];
            }
        }
        return t;
    };
    if constexpr (SILU) {
        for (uint32_t e = threadIdx.x; e < ucount * batch * 2; e += THREADS) {
            const uint32_t k = e / (batch * 2), m = (e / 2) % batch, rr = e % 2;
            const uint32_t row = 2 * useq.unit(k) + rr;
            if (row >= p.total_rows) continue;
            const float g = total_of(k, rr, m);
            const float up = total_of(k, 2 + rr, m);
            const float silu = g / (1.0f + __expf(-g));
            static_cast<float *>(p.dst[0])[static_cast<uint64_t>(m) * p.stride[0] + row] = silu * up;
        }
    } else {
        for (uint32_t e = threadIdx.x; e < ucount * batch * 4; e += THREADS) {
            const uint32_t k = e / (batch * 4), m = (e / 4) % batch, rr = e % 4;
            const uint32_t row = 4 * useq.unit(k) + rr;
            if (row >= p.total_rows) continue;
            const RowRef ref = resolve_row(p, row);
            store_out(p.mode, ref.dst, static_cast<uint64_t>(m) * ref.stride + ref.local, total_of(k, rr, m));
        }
    }
}

// Fallback for rows whose planes are not 16-byte aligned (cols/32 not a
// multiple of 8): one lane per 32-element block, 2-byte weight loads.
__global__ __launch_bounds__(256) void gemv_unaligned_kernel(const GemvParams p, uint32_t batch) {
    const uint32_t nb = p.nb;
    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t wave = blockIdx.x * 4 + threadIdx.x / kWave;
    const uint32_t nwaves = gridDim.x * 4;
    const uint64_t row_bytes = static_cast<uint64_t>(nb) * 34;
    const uint32_t nw = (p.mode == kSiluMul) ? 2 : 1;

    for (uint32_t row = wave; row < p.total_rows; row += nwaves) {
        const RowRef ref = resolve_row(p, p.mode == kSiluMul ? 0 : row);
        const uint32_t local = p.mode == kSiluMul ? row : ref.local;
        for (uint32_t j = 0; j < batch; ++j) {
            float res[2] = {0.0f, 0.0f};
            for (uint32_t wi = 0; wi < nw; ++wi) {
                const uint8_t *row_w = (p.mode == kSiluMul ? p.w[wi] : ref.w) + local * row_bytes;
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
                if (p.mode == kSiluMul) {
                    const float silu = res[0] / (1.0f + __expf(-res[0]));
                    static_cast<float *>(p.dst[0])[static_cast<uint64_t>(j) * p.stride[0] + row] = silu * res[1];
                } else {
                    store_out(p.mode, ref.dst, static_cast<uint64_t>(j) * ref.stride + local, res[0]);
                }
            }
        }
    }
}

// One launch of a given instantiation.
template <int M, int THREADS, int XMODE, bool SILU>
int launch_inst(GemvParams p, uint32_t x_bytes, hipStream_t stream) {
    auto kern = gemv_kernel<M, THREADS, XMODE, SILU>;
    static KernelGeometry geometry;
    constexpr uint32_t R = RowsPerUnit<M>::value;
    p.x_bytes = x_bytes;
    p.units = SILU ? (p.total_rows + R / 2 - 1) / (R / 2) : (p.total_rows + R - 1) / R;
    const uint32_t lds = x_bytes + (THREADS / kWave) * kParkFloats * 4;
    if (lds > kLdsLimit || !geometry.grant(reinterpret_cast<const void *>(kern), kLdsLimit))
        return fail(Q8MI_LAUNCH_ERROR, "gemv: cannot reserve %u bytes of LDS", lds);
    uint32_t per_cu = geometry.workgroups_per_cu(kern, THREADS, lds);
    if (per_cu > kGemvWgsPerCu) per_cu = kGemvWgsPerCu;
    p.interleave = kGemvInterleave;
    const uint32_t cus = static_cast<uint32_t>(device_cu_count());
    const uint32_t grid = pick_grid(p.units, (p.nb * 2 + 127) / 128, M, THREADS / kWave, cus, per_cu);
    kern<<<grid, THREADS, lds, stream>>>(p);
    return check_launch("gemv");
}

template <int M, bool SILU>
int launch_ms(const GemvParams &p, hipStream_t stream) {
    const uint32_t xb = x_lds_bytes(p.nb, M);
    const uint32_t park_256 = 4 * kParkFloats * 4, park_1024 = 16 * kParkFloats * 4;
    // fp32 activations (fused quantizer, fused norm) are served by the row-pair kernels only
    if (p.xf != nullptr) return fail(Q8MI_REJECTED, "qgemv: batch %d, %u columns: not served in one launch", M, p.nb * 32);
    // the LDS staging loads 16 bytes at a time: activations on a 4-byte boundary are read by the lanes
    if (reinterpret_cast<uintptr_t>(p.y) % 16 != 0) return launch_inst<M, 256, kXGlobal, SILU>(p, 0, stream);
    if (xb + park_256 <= 76u * 1024u) return launch_inst<M, 256, kXLds, SILU>(p, xb, stream);   // two per CU fit
    if (xb + park_1024 <= kLdsLimit) return launch_inst<M, 1024, kXLds, SILU>(p, xb, stream);
    return launch_inst<M, 256, kXGlobal, SILU>(p, 0, stream);
}

template <int M>
int launch_m(const GemvParams &p, hipStream_t stream) {
    return p.mode == kSiluMul ? launch_ms<M, true>(p, stream) : launch_ms<M, false>(p, stream);
}

constexpr uint64_t kMfmaShallowMaxRows = 65536;

// One workgroup of 512 threads (448 or 768 where measured better, below) per CU: its waves split the items of its units
// evenly, so a matrix only needs as many 4-row units as there are CUs to keep the chip busy.
template <int MG, bool SILU, bool HS, bool D4, int DEPTH, int THREADS = 512>   // 256 and 1024 threads are 10..35 % slower at batch 4 and 8
int launch_mfma_depth(GemvParams p, uint32_t batch, hipStream_t stream) {
    if constexpr (THREADS == 512 && MG == 1 && SILU && !D4 && DEPTH == 1) {
        // The SwiGLU at three and four activation rows: seven waves (layer step at batch 3 / 4: 80.2 / 83.1 ->
        // 79.7 / 82.5 us; six waves 80.8 / 83.8; at five to eight rows eight waves stay ahead, 87.0 / 88.4 against
        // 87.8 / 89.1 with seven).
        const int rc = launch_mfma_depth<MG, SILU, HS, D4, DEPTH, 448>(p, batch, stream);
        if (rc != Q8MI_REJECTED) return rc;
    }
    if constexpr (THREADS == 512 && MG == 2 && !SILU && !D4 && DEPTH == 1) {
        // Five to eight activation rows, every form but the SwiGLU: twelve waves.  A wave's share of a short-row
        // launch (the fan-out and the O projection of a verify step) is then three or four items -- one memory
        // round trip each -- instead of four or five, and eight instead of eleven on the down projection.  Layer
        // step at batch 6 / 8 with twelve waves on the short rows: 88.6 / 90.0 -> 88.0 / 89.5 us (ten waves 88.1 /
        // 89.7, fourteen 89.0 / 90.3); on the down projection as well: 87.4 / 88.7.  The SwiGLU loses with twelve
        // (35.1 against 32.6 us), the down projection of three and four rows is the same either way.  A shape whose parked sums do not fit with twelve waves takes eight.
        const int rc = launch_mfma_depth<MG, SILU, HS, D4, DEPTH, 768>(p, batch, stream);
        if (rc != Q8MI_REJECTED) return rc;
    }
    const uint32_t cus = static_cast<uint32_t>(device_cu_count());
    p.units = SILU ? (p.total_rows + 1) / 2 : (p.total_rows + 3) / 4;
    p.x_bytes = mfma_x_lds_bytes(p.nb, batch, MG, HS);
    p.interleave = kGemvInterleave;
    // The streaming hint on the weight loads.  Launches timed back to back on their own gain from it on long
    // streams only (batch 4: 2 x 17408 x 5120 36.2 -> 33.6 us, 5120 x 17408 22.0 -> 20.6 us, but 8192 x 5120
    // 11.7 -> 12.5 us and 5120 x 6144 10.1 -> 10.8 us).  In a layer's sequence of launches it pays on those two
    // as well: with the hint on the fan-out and the O projection too, the eight-launch layer step takes 88.1 us
    // instead of 90.3 at batch 6 and 89.9 instead of 92.1 at batch 8 -- weights a launch leaves in the caches
    // are in the way of the launches behind it.  So every launch of a megabyte and more carries it.
    constexpr uint64_t kStreamFrom = 1ull * 1000 * 1000;
    const bool streaming = (SILU ? 2ull : 1ull) * p.total_rows * p.nb * 34 >= kStreamFrom;
    const uint32_t grid = p.units < cus ? p.units : cus;
    const uint32_t nitems = (p.nb + kMfmaItemBlocks - 1) / kMfmaItemBlocks;
    const uint32_t per_group = (p.units + grid - 1) / grid;
    constexpr uint32_t kDynLimit = kLdsLimit - 256;   // the kernel also has a few static LDS words
    static KernelGeometry geometry[2][2];
    // Items dealt round-robin to the waves wherever every item's sums fit LDS beside the activations
    // (up to eight activation rows, one item in flight per wave); else contiguous ranges per wave.
    // (With nine to sixteen rows, the D4 route of the GEMM's small batches, an item's arithmetic is
    // long enough to want a second item on its way, and the item-wise form then loses: 17408 x 5120
    // at batch 16 27.9 us by ranges, 30.8 item-wise with two items in flight, 31.6 with one.)
    if constexpr (MG <= 2 && DEPTH == 1) {
        const uint64_t item_park = static_cast<uint64_t>(per_group) * nitems * kMfmaUnitRows * 4 * MG * 4;
        if (p.x_bytes + item_park <= kDynLimit) {
            auto kern = streaming ? gemv_mfma_kernel<MG, THREADS, SILU, HS, D4, DEPTH, true, true>
                                  : gemv_mfma_kernel<MG, THREADS, SILU, HS, D4, DEPTH, false, true>;
            if (!geometry[1][streaming].grant(reinterpret_cast<const void *>(kern), kDynLimit))
                return fail(Q8MI_LAUNCH_ERROR, "gemv: cannot reserve %u bytes of LDS", kDynLimit);
            kern<<<grid, THREADS, p.x_bytes + static_cast<uint32_t>(item_park), stream>>>(p, batch, 0);
            return check_launch("gemv_mfma");
        }
    }
    auto kern = streaming ? gemv_mfma_kernel<MG, THREADS, SILU, HS, D4, DEPTH, true, false>
                          : gemv_mfma_kernel<MG, THREADS, SILU, HS, D4, DEPTH, false, false>;
    const uint32_t park_floats = max_units_touched(per_group, nitems, THREADS / kWave) * mfma_park_floats_per_unit(MG);
    const uint32_t lds = p.x_bytes + (THREADS / kWave) * park_floats * 4;
    if (lds > kDynLimit) return fail(Q8MI_REJECTED, "gemv (matrix-core variant): %u bytes of LDS needed", lds);
    if (!geometry[0][streaming].grant(reinterpret_cast<const void *>(kern), kDynLimit))
        return fail(Q8MI_LAUNCH_ERROR, "gemv: cannot reserve %u bytes of LDS", lds);
    kern<<<grid, THREADS, lds, stream>>>(p, batch, park_floats);
    return check_launch("gemv_mfma");
}

// Items a wave keeps in flight: one for layer-sized matrices (2 % faster at M = 4..8), two for long
// streams such as a vocabulary (where one is much slower) and for the D4 route.
template <int MG, bool SILU, bool HS, bool D4 = false>
int launch_mfma(const GemvParams &p, uint32_t batch, hipStream_t stream) {
    const uint64_t weight_rows = SILU ? 2ull * p.total_rows : p.total_rows;
    if (!D4 && weight_rows <= kMfmaShallowMaxRows)
        return launch_mfma_depth<MG, SILU, HS, D4, kMfmaGemvDepth>(p, batch, stream);
    return launch_mfma_depth<MG, SILU, HS, D4, kMfmaDepth>(p, batch, stream);
}

// Activations that fit LDS in the matrix-core layout (with room for the parked sums).
// (8 KB: what the eight waves park for the short unit lists of such long rows.)
bool mfma_fits(uint32_t nb, uint32_t batch, bool half_scales) {
    return mfma_x_lds_bytes(nb, batch, (batch + 3) / 4, half_scales) + (half_scales ? 8u : 16u) * 1024u <=
           kLdsLimit - 256;
}

template <bool HS>
int launch_mfma_hs(const GemvParams &p, uint32_t batch, hipStream_t stream) {
    const bool silu = p.mode == kSiluMul;
    if (batch <= 4)
        return silu ? launch_mfma<1, true, HS>(p, batch, stream) : launch_mfma<1, false, HS>(p, batch, stream);
    return silu ? launch_mfma<2, true, HS>(p, batch, stream) : launch_mfma<2, false, HS>(p, batch, stream);
}

int launch_mfma_any(const GemvParams &p, uint32_t batch, hipStream_t stream) {
    if (mfma_fits(p.nb, batch, false)) return launch_mfma_hs<false>(p, batch, stream);
    return launch_mfma_hs<true>(p, batch, stream);
}

int launch_any(const GemvParams &p, uint32_t batch, hipStream_t stream) {
    if (p.nb % 8 != 0) {
        if (p.xf != nullptr) return fail(Q8MI_REJECTED, "qgemv: cols %u not a multiple of 256", p.nb * 32);
        const uint32_t cus = static_cast<uint32_t>(device_cu_count());
        uint32_t grid = cus * 8;
        const uint32_t max_wgs = (p.total_rows + 3) / 4;
        if (grid > max_wgs) grid = max_wgs;
        gemv_unaligned_kernel<<<grid, 256, 0, stream>>>(p, batch);
        return check_launch("gemv_unaligned");
    }
    const uint64_t row_pairs = p.mode == kSiluMul ? p.total_rows : (p.total_rows + 1) / 2;
    const bool mfma_first = p.xf == nullptr && gemv_prefers_mfma(row_pairs, batch, p.nb, p.mode == kSiluMul) &&
                            reinterpret_cast<uintptr_t>(p.y) % 4 == 0 &&
                            (mfma_fits(p.nb, batch, false) || mfma_fits(p.nb, batch, true));
    if (mfma_first) {
        const int rc = launch_mfma_any(p, batch, stream);
        if (rc != Q8MI_REJECTED) return rc;   // a unit list whose parked sums do not fit: below
    }
    if (batch <= kPairsMaxBatch) {   // row pairs, handed out by the dispatcher (q8mi_gemv_pairs.hip)
        const int rc = launch_pairs(p, batch, stream);
        if (rc != Q8MI_REJECTED) return rc;
    }
    switch (batch) {
        case 1: return launch_m<1>(p, stream);
        case 2: return launch_m<2>(p, stream);
        case 3: return launch_m<3>(p, stream);
        case 4: return launch_m<4>(p, stream);
        case 5: return launch_m<5>(p, stream);
        case 6: return launch_m<6>(p, stream);
        case 7: return launch_m<7>(p, stream);
        case 8: return launch_m<8>(p, stream);
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

// Activations of a call: Q8_1 blocks, or fp32 rows for the entry points that quantize in the kernel.
struct XSource {
    const void *y_q8_1;
    const float *xf;
    uint32_t stride_x;
    const float *norm_w = nullptr;   // set: xf is one raw row to be RMS-normalised first
    float eps = 0.0f;
    float *normalized = nullptr;
};

GemvParams single(const uint8_t *w, const XSource &x, void *dst, uint32_t rows, uint32_t cols,
                  uint32_t stride, int mode) {
    GemvParams p{};
    p.w[0] = w;
    p.dst[0] = dst;
    p.stride[0] = stride;
    for (int i = 0; i < 4; ++i) p.row_end[i] = rows;
    p.y = static_cast<const uint8_t *>(x.y_q8_1);
    p.xf = x.xf;
    p.x_stride = x.stride_x;
    p.norm_w = x.norm_w;
    p.eps = x.eps;
    p.normalized = x.normalized;
    p.total_rows = rows;
    p.units = 0;   // set per batch size at launch
    p.nb = cols / kQK;
    p.mode = mode;
    return p;
}

int run_single(const char *what, int mode, const uint8_t *w, const XSource &y, void *dst, uint32_t rows,
               uint32_t cols, uint32_t batch, uint32_t stride, void *stream) {
    if (int rc = shape_gate(what, cols, batch)) return rc;
    if (rows == 0 || cols == 0) return Q8MI_OK;
    if (!planes_aligned(w)) return fail(Q8MI_REJECTED, "%s: weight pointer not 16-byte aligned", what);
    const GemvParams p = single(w, y, dst, rows, cols, stride, mode);
    return launch_any(p, batch, as_stream(stream));
}

}  // namespace

// D4-quantized activations through the matrix-core GEMV: what the GEMM entry points use for
// batches too small for an MFMA tile.  As many activation rows per launch as fit LDS (at most 16:
// 16 at 5120 columns, 4 at 17408); served while one pass over the weights covers the batch, or two
// passes of the short slices (measured against the 32-row ring tiles of the GEMM: 14.7..17.2 us
// against 19 us at 5120 x 5120 and 9..16 rows, but 26..32 us in two passes at 17..32 rows;
// 49 against 58 us at 5120 x 17408 and 8 rows).  Q8MI_REJECTED otherwise (the caller then uses
// tiles).  w_up: the SwiGLU form (dst = silu(w x) * (w_up x)); add: dst += w x.
int gemv_mfma_d4(const uint8_t *w, const uint8_t *w_up, const void *y_d4, float *dst, uint32_t rows, uint32_t cols,
                 uint32_t batch, uint32_t stride_dst_row, bool add, hipStream_t stream) {
    const uint32_t nb = cols / kQK;
    const bool silu = w_up != nullptr;
    if (nb % 8 != 0 || batch == 0) return fail(Q8MI_REJECTED, "gemv (matrix-core, D4): cols %u not served", cols);
    // D4 scales are fp32 values: only the fp32 scale table keeps them exact
    uint32_t fit = 0;
    for (uint32_t m = 16; m >= 4; m -= 4) {
        if (mfma_x_lds_bytes(nb, m, m / 4, false) + 16u * 1024u <= kLdsLimit - 256) { fit = m; break; }
    }
    if (fit == 0 || batch > (fit >= 16 ? fit : 2 * fit))   // rows of 17408 columns: two passes of four rows still win
        return fail(Q8MI_REJECTED, "gemv (matrix-core, D4): batch %u at %u columns is served by tiles", batch, cols);
    // ... unless the GEMM's 32-row tiles come at most one per CU: those are then cut in two along K
    // (launch_ring) and beat two passes (measured at 17408 columns and 5..8 rows: 43 against 46..48 us
    // on 5120 weight rows, 49 against 65..67 us on 8192)
    if (batch > fit && !silu && !add && (rows + 31u) / 32u <= static_cast<uint32_t>(device_cu_count()) && nb / 4 >= 8)
        return fail(Q8MI_REJECTED, "gemv (matrix-core, D4): batch %u at %u columns is served by split tiles", batch, cols);
    const auto *y = static_cast<const uint8_t *>(y_d4);
    for (uint32_t j0 = 0; j0 < batch; j0 += fit) {
        const uint32_t m = batch - j0 < fit ? batch - j0 : fit;
        GemvParams p = single(w, XSource{y + static_cast<uint64_t>(j0) * kD4Bytes, nullptr, batch},
                              dst + static_cast<uint64_t>(j0) * stride_dst_row, rows, cols, stride_dst_row,
                              silu ? kSiluMul : add ? kAddF32 : kStoreF32);
        p.w[1] = silu ? w_up : p.w[1];
        int rc;
        if (silu) {
            switch ((m + 3) / 4) {
                case 1: rc = launch_mfma<1, true, false, true>(p, m, stream); break;
                case 2: rc = launch_mfma<2, true, false, true>(p, m, stream); break;
                case 3: rc = launch_mfma<3, true, false, true>(p, m, stream); break;
                default: rc = launch_mfma<4, true, false, true>(p, m, stream); break;
            }
        } else {
            switch ((m + 3) / 4) {
                case 1: rc = launch_mfma<1, false, false, true>(p, m, stream); break;
                case 2: rc = launch_mfma<2, false, false, true>(p, m, stream); break;
                case 3: rc = launch_mfma<3, false, false, true>(p, m, stream); break;
                default: rc = launch_mfma<4, false, false, true>(p, m, stream); break;
            }
        }
        if (rc != Q8MI_OK) return rc;
    }
    return Q8MI_OK;
}

// Any batch through the GEMV kernels, eight activation rows per launch.  Used by
// the GEMM entry point for shapes its MFMA tile does not cover.
int gemv_any_batch(const uint8_t *w, const void *y_q8_1, float *dst, uint32_t rows, uint32_t cols,
                   uint32_t batch, uint32_t stride_dst_row, hipStream_t stream) {
    const uint32_t nb = cols / kQK;
    const auto *y = static_cast<const uint8_t *>(y_q8_1);
    for (uint32_t j0 = 0; j0 < batch; j0 += Q8MI_MAX_GEMV_BATCH) {
        const uint32_t m = batch - j0 < Q8MI_MAX_GEMV_BATCH ? batch - j0 : Q8MI_MAX_GEMV_BATCH;
        const GemvParams p = single(w, XSource{y + static_cast<uint64_t>(j0) * nb * kQ81Bytes, nullptr, 0},
                                    dst + static_cast<uint64_t>(j0) * stride_dst_row, rows, cols,
                                    stride_dst_row, kStoreF32);
        if (int rc = launch_any(p, m, stream)) return rc;
    }
    return Q8MI_OK;
}

}  // namespace q8mi

using namespace q8mi;

extern "C" int q8mi_gemv(const uint8_t *w, const void *y, float *dst, uint32_t rows, uint32_t cols,
                         uint32_t batch, uint32_t stride, void *stream) {
    return run_single("gemv", kStoreF32, w, XSource{y, nullptr, 0}, dst, rows, cols, batch, stride, stream);
}

extern "C" int q8mi_gemv_bf16(const uint8_t *w, const void *y, uint16_t *dst, uint32_t rows,
                              uint32_t cols, uint32_t batch, uint32_t stride, void *stream) {
    return run_single("gemv_bf16", kStoreBF16, w, XSource{y, nullptr, 0}, dst, rows, cols, batch, stride, stream);
}

extern "C" int q8mi_gemv_add(const uint8_t *w, const void *y, float *dst, uint32_t rows,
                             uint32_t cols, uint32_t batch, uint32_t stride, void *stream) {
    return run_single("gemv_add", kAddF32, w, XSource{y, nullptr, 0}, dst, rows, cols, batch, stride, stream);
}

extern "C" int q8mi_gemv_add_bf16(const uint8_t *w, const void *y, uint16_t *dst, uint32_t rows,
                                  uint32_t cols, uint32_t batch, uint32_t stride, void *stream) {
    return run_single("gemv_add_bf16", kAddBF16, w, XSource{y, nullptr, 0}, dst, rows, cols, batch, stride, stream);
}

static int run_silu_mul(const uint8_t *wg, const uint8_t *wu, const XSource &y, float *dst, uint32_t rows,
                        uint32_t cols, uint32_t batch, uint32_t stride, void *stream) {
    if (int rc = shape_gate("gemv_silu_mul", cols, batch)) return rc;
    if (rows == 0 || cols == 0) return Q8MI_OK;
    if (!planes_aligned(wg) || !planes_aligned(wu))
        return fail(Q8MI_REJECTED, "gemv_silu_mul: weight pointer not 16-byte aligned");
    GemvParams p = single(wg, y, dst, rows, cols, stride, kSiluMul);
    p.w[1] = wu;
    return launch_any(p, batch, as_stream(stream));
}

extern "C" int q8mi_gemv_silu_mul(const uint8_t *wg, const uint8_t *wu, const void *y, float *dst,
                                  uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride,
                                  void *stream) {
    return run_silu_mul(wg, wu, XSource{y, nullptr, 0}, dst, rows, cols, batch, stride, stream);
}

static int run_fanout4(const uint8_t *w0, const uint8_t *w1, const uint8_t *w2, const uint8_t *w3,
                       const XSource &y, float *d0, float *d1, float *d2, float *d3, uint32_t rows0,
                       uint32_t rows1, uint32_t rows2, uint32_t rows3, uint32_t cols, uint32_t batch, uint32_t s0,
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
    for (uint32_t i = n; i < 4; ++i) {
        p.row_end[i] = total;
        p.w[i] = p.w[n - 1];   // never dereferenced for a row, kept valid for safety
        p.dst[i] = p.dst[n - 1];
        p.stride[i] = p.stride[n - 1];
    }
    p.y = static_cast<const uint8_t *>(y.y_q8_1);
    p.xf = y.xf;
    p.x_stride = y.stride_x;
    p.norm_w = y.norm_w;
    p.eps = y.eps;
    p.normalized = y.normalized;
    p.total_rows = total;
    p.units = 0;
    p.nb = cols / kQK;
    p.mode = kStoreF32;
    return launch_any(p, batch, as_stream(stream));
}

extern "C" int q8mi_gemv_fanout4(const uint8_t *w0, const uint8_t *w1, const uint8_t *w2,
                                 const uint8_t *w3, const void *y, float *d0, float *d1, float *d2,
                                 float *d3, uint32_t rows0, uint32_t rows1, uint32_t rows2,
                                 uint32_t rows3, uint32_t cols, uint32_t batch, uint32_t s0,
                                 uint32_t s1, uint32_t s2, uint32_t s3, void *stream) {
    return run_fanout4(w0, w1, w2, w3, XSource{y, nullptr, 0}, d0, d1, d2, d3, rows0, rows1, rows2, rows3, cols,
                       batch, s0, s1, s2, s3, stream);
}

// ---- entry points that quantize the activations inside the GEMV ------------------------------
extern "C" int q8mi_qgemv(const uint8_t *w, const float *x, uint32_t stride_x_row, void *dst, int dst_is_bf16,
                          uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride, void *stream) {
    return run_single("qgemv", dst_is_bf16 ? kStoreBF16 : kStoreF32, w, XSource{nullptr, x, stride_x_row}, dst, rows,
                      cols, batch, stride, stream);
}

extern "C" int q8mi_qgemv_add(const uint8_t *w, const float *x, uint32_t stride_x_row, void *dst, int dst_is_bf16,
                              uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride, void *stream) {
    return run_single("qgemv_add", dst_is_bf16 ? kAddBF16 : kAddF32, w, XSource{nullptr, x, stride_x_row}, dst, rows,
                      cols, batch, stride, stream);
}

extern "C" int q8mi_qgemv_silu_mul(const uint8_t *wg, const uint8_t *wu, const float *x, uint32_t stride_x_row,
                                   float *dst, uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride,
                                   void *stream) {
    return run_silu_mul(wg, wu, XSource{nullptr, x, stride_x_row}, dst, rows, cols, batch, stride, stream);
}

extern "C" int q8mi_qgemv_fanout4(const uint8_t *w0, const uint8_t *w1, const uint8_t *w2, const uint8_t *w3,
                                  const float *x, uint32_t stride_x_row, float *d0, float *d1, float *d2, float *d3,
                                  uint32_t rows0, uint32_t rows1, uint32_t rows2, uint32_t rows3, uint32_t cols,
                                  uint32_t batch, uint32_t s0, uint32_t s1, uint32_t s2, uint32_t s3, void *stream) {
    return run_fanout4(w0, w1, w2, w3, XSource{nullptr, x, stride_x_row}, d0, d1, d2, d3, rows0, rows1, rows2, rows3,
                       cols, batch, s0, s1, s2, s3, stream);
}

extern "C" int q8mi_gemv_two(const uint8_t *w0, const uint8_t *w1, const void *y, float *dst0,
                             float *dst1, uint32_t rows, uint32_t cols, uint32_t batch,
                             uint32_t stride, void *stream) {
    if (int rc = shape_gate("gemv_two", cols, batch)) return rc;
    if (rows == 0) return Q8MI_OK;
    return q8mi_gemv_fanout4(w0, w1, nullptr, nullptr, y, dst0, dst1, nullptr, nullptr, rows, rows,
                             0, 0, cols, batch, stride, stride, 0, 0, stream);
}

// ---- entry points that RMS-normalise and quantize one activation row inside the GEMV ----------
static int norm_gate(const char *what, const float *x, const float *norm_weight, const float *normalized,
                     uint32_t batch) {
    if (x == nullptr || norm_weight == nullptr) return fail(Q8MI_REJECTED, "%s: null pointer", what);
    if (batch != 1) return fail(Q8MI_REJECTED, "%s: batch %u (one row only)", what, batch);
    // every workgroup reads x while workgroup 0 writes the normalised row
    if (normalized == x) return fail(Q8MI_REJECTED, "%s: the normalised row must not overwrite x", what);
    return Q8MI_OK;
}

extern "C" int q8mi_nqgemv(const uint8_t *w, const float *x, const float *norm_weight, float eps, float *normalized,
                           void *dst, int dst_is_bf16, uint32_t rows, uint32_t cols, uint32_t batch, void *stream) {
    if (int rc = norm_gate("nqgemv", x, norm_weight, normalized, batch)) return rc;
    return run_single("nqgemv", dst_is_bf16 ? kStoreBF16 : kStoreF32, w, XSource{nullptr, x, cols, norm_weight, eps, normalized},
                      dst, rows, cols, batch, rows, stream);
}

extern "C" int q8mi_nqgemv_silu_mul(const uint8_t *wg, const uint8_t *wu, const float *x, const float *norm_weight,
                                    float eps, float *normalized, float *dst, uint32_t rows, uint32_t cols,
                                    uint32_t batch, void *stream) {
    if (int rc = norm_gate("nqgemv_silu_mul", x, norm_weight, normalized, batch)) return rc;
    return run_silu_mul(wg, wu, XSource{nullptr, x, cols, norm_weight, eps, normalized}, dst, rows, cols, batch, rows,
                        stream);
}

extern "C" int q8mi_nqgemv_fanout4(const uint8_t *w0, const uint8_t *w1, const uint8_t *w2, const uint8_t *w3,
                                   const float *x, const float *norm_weight, float eps, float *normalized, float *d0,
                                   float *d1, float *d2, float *d3, uint32_t rows0, uint32_t rows1, uint32_t rows2,
                                   uint32_t rows3, uint32_t cols, uint32_t batch, void *stream) {
    if (int rc = norm_gate("nqgemv_fanout4", x, norm_weight, normalized, batch)) return rc;
    return run_fanout4(w0, w1, w2, w3, XSource{nullptr, x, cols, norm_weight, eps, normalized}, d0, d1, d2, d3, rows0,
                       rows1, rows2, rows3, cols, batch, rows0, rows1, rows2, rows3, stream);
}
