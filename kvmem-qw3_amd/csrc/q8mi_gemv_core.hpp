// Core of the Q8_0 x Q8_1 GEMV on gfx950, shared by the GEMV family and the
// fused LM-head kernel.
//
// Work decomposition
//   unit   R weight rows that share every activation fetch (R = 2, or 4 from
//          batch 4 on): rows R*u .. R*u+R-1 of the concatenated row space; for
//          SwiGLU R/2 gate rows and the matching R/2 up rows
//   step   2 KiB of each row's int8 plane: two fully coalesced 1 KiB wave loads
//          "A" and "B".  A lane holds 16 bytes of each, i.e. half of block
//          A_(lane/2) and half of block B_(lane/2).  Lane pairs swap half sums
//          with one DPP move so the even lane owns the full int32 dot of block A
//          and the odd lane that of block B: one int32 sum and one fp32 rescale
//          per 32-element block.
//   item   (unit, step).  A workgroup owns a list of units; its item list is cut
//          into equal contiguous ranges, one per wave, so the waves are balanced
//          to within one item whatever the row length.  A wave walks its range
//          as one flat, software-pipelined stream: the loads of item t+kDepth
//          are issued before item t is consumed, also across row boundaries,
//          so it always has kDepth * R * 2 KiB of weight loads in flight.
//   park   a range may start or end inside a unit, so a wave leaves partial
//          sums per touched unit in LDS; after a barrier the workgroup adds the
//          partials in wave order and writes the outputs.
// Activations are staged once per workgroup in LDS (int8 as packed dwords plus
// fp32 scales) after the first loads have been issued; when they do not fit,
// lanes read them from global memory (served by L2).
#pragma once

#include <atomic>
#include <mutex>

#include "q8mi_device.hpp"
#include "q8mi_internal.hpp"
#include "q8mi_quantize_core.hpp"

namespace q8mi {

// Weight rows per unit (rows that share every activation fetch): 2 for small
// batches, 4 from batch 4 on, where the LDS reads of the activations would
// otherwise be the bottleneck (LDS traffic per weight byte halves).
template <int M>
struct RowsPerUnit {
    static constexpr int value = M >= 4 ? 4 : 2;
};
constexpr int kDepth = 2;                       // items in flight per wave
constexpr uint32_t kLdsLimit = 160u * 1024u;    // LDS per CU on gfx950
constexpr uint32_t kParkFloats = 1024;           // per-wave LDS area (floats) for the sums of the units it touched

// Where a lane finds the activations: Q8_1 blocks staged in LDS, or Q8_1 blocks read from
// global memory.  (fp32 activations are served by the row-pair kernels of q8mi_gemv_pairs.hip.)
enum XMode : int { kXLds = 0, kXGlobal = 1 };

// The activations of a launch as the staging code sees them.
struct XIn {
    const uint8_t *y;      // Q8_1 blocks
};

// LDS footprint of `batch` activation rows: per 64-block step 128 16-byte
// pieces of int8 and 64 fp32 scales, zero-padded to whole steps.
inline uint32_t x_lds_bytes(uint32_t nb, uint32_t batch) {
    const uint32_t nsteps = (nb * 2 + 127) / 128;
    return batch * nsteps * (128 * 16 + 64 * 4);
}

// 16 weight bytes.  Every weight byte is read once per launch, so the load carries the
// streaming ("nt") cache hint: the lines are not kept for reuse.  Measured: a 1 GiB plain read
// goes from 6.4 to 7.0 TB/s, the SwiGLU GEMV of a 27B layer from 35.7 to 33.2 us.  The fp16
// scale plane is read with plain loads: a row's 2-byte scale loads of consecutive steps touch
// the same cache lines again, and the hint made those slower.
__device__ __forceinline__ v4i load_q16(const uint8_t *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const v4i *>(p));
}

// 16 activation bytes of Q8_1 block `blk` (half = 0/1) straight from global
// memory; the block is only 4-byte aligned.
__device__ __forceinline__ v4i load_x16_global(const uint8_t *y, uint32_t blk, uint32_t half) {
    const int *p = reinterpret_cast<const int *>(y + static_cast<uint64_t>(blk) * kQ81Bytes + 4 + half * 16);
    v4i v;
    v.x = p[0]; v.y = p[1]; v.z = p[2]; v.w = p[3];
    return v;
}

// idx = m * per + within with m < M: the quotient by a run of compare-and-subtract steps (M is a
// small compile-time bound; a 32-bit division by a run-time value costs some twenty instructions).
template <int M>
__device__ __forceinline__ void split_index(uint32_t idx, uint32_t per, uint32_t &m, uint32_t &within) {
    m = 0;
    within = idx;
#pragma unroll
    for (int i = 1; i < M; ++i) {
        const bool over = within >= per;
        within = over ? within - per : within;
        m += over ? 1u : 0u;
    }
}

// Copies M rows of Q8_1 activations from global memory into LDS, split into a
// packed int8 area and an fp32 scale area.  Dword 0 of each 36-B block is
// {d, s}; dwords 1..8 are the quants.  The M rows are contiguous in memory
// (M * nb blocks), so the copy is a flat sequence of 16-byte loads, all issued
// before the first one is consumed: staging costs one memory round trip, not
// one per trip of a load-use loop.  Ends with a workgroup barrier.
template <int M, int THREADS>
struct StageLds {
    static constexpr int kBatch = 4;   // 16-byte loads in flight per thread
    v4i v[kBatch];

    // First trip of loads only: nothing is consumed here, so the caller can put further
    // loads (its first weight items) behind these before finish() waits for them.
    // y must be 16-byte aligned (launchers send other activations to the global-memory mode).
    __device__ __forceinline__ void issue(const uint8_t *y, uint32_t nb) {
        const uint32_t total_ch = static_cast<uint32_t>(M) * nb * 9 / 4;
        const v4i *src = reinterpret_cast<const v4i *>(y);
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const uint32_t c = u * THREADS + threadIdx.x;
            v[u] = src[c < total_ch ? c : 0];
        }
    }

    __device__ __forceinline__ void finish(uint8_t *smem, const uint8_t *y, uint32_t nb) {
        const uint32_t nsteps = (nb * 2 + 127) / 128;
        int *wq = reinterpret_cast<int *>(smem);
        float *wd = reinterpret_cast<float *>(smem + static_cast<size_t>(M) * nsteps * 128 * 16);
        const uint32_t blocks_padded = nsteps * 64;
        const uint32_t total_dw = static_cast<uint32_t>(M) * nb * 9;   // multiple of 4: nb % 8 == 0 here
        const uint32_t total_ch = total_dw / 4;

        auto put = [&](uint32_t g, uint32_t word) {   // g: dword index in the global layout
            const uint32_t blk_g = g / 9, part = g % 9;
            uint32_t m, kb;
            split_index<M>(blk_g, nb, m, kb);
            const uint32_t blk = m * blocks_padded + kb;
            if (part == 0) {
                wd[blk] = half_bits_to_float(static_cast<uint16_t>(word & 0xffffu));
            } else {
                wq[blk * 8 + (part - 1)] = static_cast<int>(word);
            }
        };
        auto put4 = [&](uint32_t c, const v4i &q) {
            if (c < total_ch) {
                put(4 * c + 0, static_cast<uint32_t>(q.x));
                put(4 * c + 1, static_cast<uint32_t>(q.y));
                put(4 * c + 2, static_cast<uint32_t>(q.z));
                put(4 * c + 3, static_cast<uint32_t>(q.w));
            }
        };
        const v4i *src = reinterpret_cast<const v4i *>(y);
#pragma unroll
        for (int u = 0; u < kBatch; ++u) put4(u * THREADS + threadIdx.x, v[u]);
        for (uint32_t base = THREADS * kBatch; base < total_ch; base += THREADS * kBatch) {
            v4i t[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const uint32_t c = base + u * THREADS + threadIdx.x;
                t[u] = src[c < total_ch ? c : 0];
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u) put4(base + u * THREADS + threadIdx.x, t[u]);
        }
        // zero the padding up to whole steps (blocks nb .. blocks_padded of every row)
        const uint32_t pad = blocks_padded - nb;
        for (uint32_t i = threadIdx.x; i < static_cast<uint32_t>(M) * pad * 9; i += THREADS) {
            const uint32_t b = i / 9, part = i % 9;
            const uint32_t blk = (b / pad) * blocks_padded + nb + b % pad;
            if (part == 0) wd[blk] = 0.0f; else wq[blk * 8 + (part - 1)] = 0;
        }
        __syncthreads();
    }
};

// Activations of the workgroup into LDS, by mode, in two halves: issue() puts the first trip of
// activation loads in flight, finish() consumes them (and any further trips) and ends with a
// workgroup barrier.  Loads return in order, so the weight loads a caller issues between the two
// stay in flight while the activations are converted.  No-op when lanes read the activations
// from global memory.
template <int M, int THREADS, int XMODE>
struct XStage {
    StageLds<M, THREADS> lds;
    __device__ __forceinline__ void issue(const XIn &in, uint32_t nb) {
        if constexpr (XMODE == kXLds) lds.issue(in.y, nb);
    }
    __device__ __forceinline__ void finish(uint8_t *smem, const XIn &in, uint32_t nb) {
        if constexpr (XMODE == kXLds) lds.finish(smem, in.y, nb);
    }
};

template <int M, int THREADS, int XMODE>
__device__ __forceinline__ void stage_x(uint8_t *smem, const XIn &in, uint32_t nb) {
    XStage<M, THREADS, XMODE> xs;
    xs.issue(in, nb);
    xs.finish(smem, in, nb);
}

// Weight bytes of one item held by a lane.
template <int R>
struct Item {
    v4i qa[R];
    v4i qb[R];
    uint32_t dw[R];   // fp16 bits of the scale of "this lane's" block
};

template <int R>
struct RowPtrs {
    const uint8_t *p[R];   // scale plane of each row (never null: clamped to a valid row)
};

template <int R>
__device__ __forceinline__ void issue_item(Item<R> &it, const RowPtrs<R> &rows, uint32_t step, uint32_t lane,
                                           uint32_t nb) {
    const uint32_t npieces = nb * 2;
    const uint32_t pa = step * 128 + lane, pb = pa + 64;
    const uint32_t kb = step * 64 + ((lane & 1u) ? 32u : 0u) + (lane >> 1);
    // out-of-range pieces re-read the row's first bytes; compute_item masks them
    const uint32_t oa = pa < npieces ? pa * 16 : 0u;
    const uint32_t ob = pb < npieces ? pb * 16 : 0u;
    const uint32_t ok = kb < nb ? kb : 0u;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint8_t *quants = rows.p[r] + 2 * nb;
        it.qa[r] = load_q16(quants + oa);
        it.qb[r] = load_q16(quants + ob);
        it.dw[r] = reinterpret_cast<const uint16_t *>(rows.p[r])[ok];
    }
}

// Activation operands of one activation row for the lane's two pieces and block.
struct XOperand {
    v4i x1, x2;   // activation bytes matching the lane's "own" and "other" piece
    float dx;     // fp32 scale of the block this lane rescales
};

template <int XMODE>
__device__ __forceinline__ XOperand load_x(uint32_t m, uint32_t p1, uint32_t p2, uint32_t kb, bool v1, bool v2,
                                           bool vk, uint32_t nb, uint32_t nsteps, const uint8_t *y,
                                           const int *lds_q, const float *lds_d) {
    XOperand o;
    o.x1 = v4i{0, 0, 0, 0};
    o.x2 = v4i{0, 0, 0, 0};
    o.dx = 0.0f;
    if (XMODE != kXGlobal) {
        // LDS is zero-padded to whole steps, so no guards: pieces past the row's end
        // multiply the re-read weight bytes by zero
        o.x1 = *reinterpret_cast<const v4i *>(lds_q + (m * nsteps * 128 + p1) * 4);
        o.x2 = *reinterpret_cast<const v4i *>(lds_q + (m * nsteps * 128 + p2) * 4);
        o.dx = lds_d[m * nsteps * 64 + kb];
    } else {
        if (v1) o.x1 = load_x16_global(y, m * nb + (p1 >> 1), p1 & 1u);
        if (v2) o.x2 = load_x16_global(y, m * nb + (p2 >> 1), p2 & 1u);
        if (vk) o.dx = half_bits_to_float(*reinterpret_cast<const uint16_t *>(
                    y + static_cast<uint64_t>(m * nb + kb) * kQ81Bytes));
    }
    return o;
}

// One item against M activation rows.  Even lanes treat their A piece as "own"
// and their B piece as "other", odd lanes the reverse; then for every lane
//   S = dot(own) + (dot(other) of the neighbouring lane)
// is the full int32 dot of the block the lane rescales (A_(lane/2) on even lanes,
// B_(lane/2) on odd lanes).  The activation operands of row m+1 are fetched
// while row m is being consumed.
template <int M, int R, int XMODE>
__device__ __forceinline__ void compute_item(const Item<R> &it, uint32_t step, uint32_t lane, uint32_t nb,
                                             uint32_t nsteps, const uint8_t *y, const int *lds_q,
                                             const float *lds_d, float (&acc)[M][R]) {
    const uint32_t npieces = nb * 2;
    const uint32_t pa = step * 128 + lane, pb = pa + 64;
    const bool odd = lane & 1u;
    const uint32_t p1 = odd ? pb : pa, p2 = odd ? pa : pb;
    const uint32_t kb = step * 64 + (odd ? 32u : 0u) + (lane >> 1);
    const bool v1 = p1 < npieces, v2 = p2 < npieces, vk = kb < nb;
    float dw[R];
    v4i q1[R], q2[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        dw[r] = vk ? half_bits_to_float(static_cast<uint16_t>(it.dw[r])) : 0.0f;
        // own / other piece of this lane (one select per register, once per item)
        q1[r].x = odd ? it.qb[r].x : it.qa[r].x; q1[r].y = odd ? it.qb[r].y : it.qa[r].y;
        q1[r].z = odd ? it.qb[r].z : it.qa[r].z; q1[r].w = odd ? it.qb[r].w : it.qa[r].w;
        q2[r].x = odd ? it.qa[r].x : it.qb[r].x; q2[r].y = odd ? it.qa[r].y : it.qb[r].y;
        q2[r].z = odd ? it.qa[r].z : it.qb[r].z; q2[r].w = odd ? it.qa[r].w : it.qb[r].w;
    }
    XOperand cur = load_x<XMODE>(0, p1, p2, kb, v1, v2, vk, nb, nsteps, y, lds_q, lds_d);
#pragma unroll
    for (int m = 0; m < M; ++m) {
        XOperand nxt = cur;
        if (m + 1 < M) nxt = load_x<XMODE>(m + 1, p1, p2, kb, v1, v2, vk, nb, nsteps, y, lds_q, lds_d);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int s2 = dot16(q2[r], cur.x2);
            const int S = dot16(q1[r], cur.x1, dpp_i32<kDppXor1>(s2));   // full 32-element block dot
            acc[m][r] = fmaf(dw[r] * cur.dx, static_cast<float>(S), acc[m][r]);
        }
        cur = nxt;
    }
}

// A workgroup's share of the units, in the order it streams them: either a contiguous,
// balanced slice (interleave == 0) or every ngroups-th unit starting at the workgroup's
// index (interleave != 0; neighbouring workgroups then read neighbouring rows).
struct UnitSeq {
    uint32_t first, stride, count;
    __device__ __forceinline__ uint32_t unit(uint32_t k) const { return first + k * stride; }
};

__device__ __forceinline__ UnitSeq group_units(uint32_t units, uint32_t group, uint32_t ngroups, int interleave) {
    UnitSeq s;
    if (interleave) {
        s.first = group;
        s.stride = ngroups;
        s.count = group < units ? (units - group + ngroups - 1) / ngroups : 0;
    } else {
        s.first = static_cast<uint32_t>(static_cast<uint64_t>(units) * group / ngroups);
        const uint32_t end = static_cast<uint32_t>(static_cast<uint64_t>(units) * (group + 1) / ngroups);
        s.count = end - s.first;
        s.stride = 1;
    }
    return s;
}

// Streams the items [i0, i1) of a workgroup's unit sequence useq.unit(k); item i is
// step i % nsteps of unit(i / nsteps).  A wave's range may
// begin or end in the middle of a unit, so what it hands to `park` is a PARTIAL
// sum over the steps it covered; the caller combines the partials of all waves
// after a barrier.
//   rows_of(u, RowPtrs&)   fills the (clamped, always readable) row pointers of unit u
//   park(kk, total)        called once per unit touched (kk = 0, 1, ... counts them),
//                          in wave-uniform control flow; lane l < M*R receives in
//                          `total` the wave-wide sum for activation row l / R and
//                          unit row l % R.  It must not touch global memory: the loop
//                          keeps a fixed number of global loads in flight, and the
//                          compiler can only count them exactly if nothing else uses
//                          that counter.
// The loop body is branch-free apart from the per-unit park, and every slot of
// items[] lives in fixed registers, so loads stay in flight across iterations:
// the trip count is padded to a multiple of kDepth with dummy items that re-read
// the last item and whose sums are never parked.
// Must be called by every wave of the workgroup (it contains the staging barrier).
template <int M, int R, int THREADS, int XMODE, class RowsOf, class Park>
__device__ __forceinline__ void gemv_stream(uint8_t *smem, const XIn &in, uint32_t nb,
                                            const UnitSeq &useq, uint32_t i0, uint32_t i1,
                                            RowsOf rows_of, Park park) {
    const uint8_t *y = in.y;
    const uint32_t nsteps = (nb * 2 + 127) / 128;
    const uint32_t lane = threadIdx.x % kWave;
    const int *lds_q = reinterpret_cast<const int *>(smem);
    const float *lds_d = reinterpret_cast<const float *>(smem + static_cast<size_t>(M) * nsteps * 128 * 16);
    if (i1 <= i0) {   // wave-uniform; idle waves still take part in the staging barrier
        stage_x<M, THREADS, XMODE>(smem, in, nb);
        return;
    }
    const uint32_t n_items = i1 - i0;
    const uint32_t n_padded = (n_items + kDepth - 1) / kDepth * kDepth;
    const uint32_t k0 = i0 / nsteps, s0 = i0 % nsteps;

    // activation loads first, the first weight items behind them: the activations arrive first
    // and are converted while the weight loads are still in flight
    XStage<M, THREADS, XMODE> xs;
    xs.issue(in, nb);
    asm volatile("" ::: "memory");   // the activation loads stay ahead of the weight loads
    Item<R> items[kDepth];
    // issue cursor: unit ordinal, step, items left to issue for real
    uint32_t ik = k0, istep = s0, ileft = n_items;
    RowPtrs<R> irows;
    rows_of(useq.unit(ik), irows);
    auto advance_issue = [&]() {
        if (ileft > 1) {       // otherwise: keep re-reading the last real item
            --ileft;
            if (++istep == nsteps) {
                istep = 0;
                ++ik;
                rows_of(useq.unit(ik), irows);
            }
        }
    };
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
        issue_item(items[d], irows, istep, lane, nb);
        advance_issue();
    }
    // keeps the loads above where they are: without it the compiler sinks them below the staging
    // barrier and the first weight bytes are requested only after the activations are in LDS
    asm volatile("" ::: "memory");
    xs.finish(smem, in, nb);

    float acc[M][R];
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[m][r] = 0.0f;

    uint32_t cstep = s0, kk = 0;
    for (uint32_t t = 0; t < n_padded; t += kDepth) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            compute_item<M, R, XMODE>(items[d], cstep, lane, nb, nsteps, y, lds_q, lds_d, acc);
            ++cstep;
            const uint32_t done = t + d + 1;   // items consumed so far, dummies included
            if (done <= n_items && (cstep == nsteps || done == n_items)) {
                constexpr int VP = pow2_at_least(M * R);
                float flat[VP];
#pragma unroll
                for (int i = 0; i < VP; ++i) flat[i] = 0.0f;
#pragma unroll
                for (int m = 0; m < M; ++m)
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        flat[m * R + r] = acc[m][r];
                        acc[m][r] = 0.0f;
                    }
                park(kk, TransposeReduce<VP>::run(flat, lane));
                ++kk;
            }
            if (cstep == nsteps) cstep = 0;
            // refill this slot with the item kDepth ahead
            issue_item(items[d], irows, istep, lane, nb);
            advance_issue();
        }
    }
}

// Wave w of W splits the workgroup's n items evenly: items [i0, i1).
__device__ __forceinline__ void wave_items(uint32_t n, uint32_t w, uint32_t W, uint32_t &i0, uint32_t &i1) {
    i0 = static_cast<uint32_t>(static_cast<uint64_t>(n) * w / W);
    i1 = static_cast<uint32_t>(static_cast<uint64_t>(n) * (w + 1) / W);
}

// Units a wave can touch, hence park: its items cover at most this many units.
__host__ __device__ inline uint32_t max_units_touched(uint32_t group_units_max, uint32_t nsteps, uint32_t W) {
    const uint64_t items = static_cast<uint64_t>(group_units_max) * nsteps;
    const uint64_t per_wave = (items + W - 1) / W;
    return static_cast<uint32_t>((per_wave + nsteps - 1) / nsteps + 1);
}

// ---- host side: launch geometry -------------------------------------------
// Measured best on MI355X: two workgroups per CU, units dealt round-robin to the workgroups
// (neighbouring workgroups read neighbouring rows), the matrix-core variant from batch 3 on.
constexpr uint32_t kGemvWgsPerCu = 2;
constexpr int kGemvInterleave = 1;        // unit assignment, see group_units
constexpr uint32_t kMfmaFromBatch = 2;    // smallest batch served by the matrix-core variant
constexpr uint32_t kPairsMaxBatch = 4;    // largest batch the row-pair family serves
// Which GEMV family serves a launch of batch 2 and more (measured on MI355X, row-pair kernel with
// the rows shared by the waves of a workgroup against matrix-core kernel, us):
//   rows of 1 .. 3 KiB         batch 2: row pairs (5120 rows of 2 KiB: 4.6 / 7.0; 17408 rows of 1 KiB: 5.8 / 11.7 on the ring
//                              kernel); batch 3 and 4 from 2 KiB: row pairs (17408 x 2048: 9.3 / 12.9 and 10.7 / 13.0;
//                              5120 x 3072: 6.1 / 7.6 and 6.9 / 7.7); 1 KiB at batch 3 and 4: matrix cores (5120 rows
//                              5.2 / 4.7 and 5.6 / 4.8)
//   rows of 4 .. 8 KiB         batch 2: always row pairs (8192 x 5120 fan-out 9.3 / 11.9, SwiGLU 30.2 / 34.1);
//                              batch 3 and 4: row pairs but for the SwiGLU form (fan-out 10.3 / 11.7 and
//                              11.4 / 11.7, 5120 x 6144 9.8 / 11 and 10.2 / 11, SwiGLU 32.1 / 31.0 and
//                              33.7 / 31.0 since the matrix-core kernel deals its items round-robin to the
//                              waves); from batch 5 the dot products bind (batch 6: 13.1 / 12.3 on the fan-out)
//   rows of 9 .. 17 KiB        batch 2: row pairs (5120 x 17408: 18.8 / 20.0); batch 3 and 4: 22.4 / 20.3, 30.0 / 20.6
//   any other length           batch 2 with 8192 row pairs or more: row pairs (ring kernel); else matrix cores
// nb: blocks per row; silu: the SwiGLU form.
inline bool gemv_prefers_mfma(uint64_t row_pairs, uint32_t batch, uint32_t nb, bool silu) {
    if (batch < 2) return false;
    if (batch > kPairsMaxBatch) return true;
    const bool short_rows = nb % 32 == 0 && nb >= 64 && nb <= 256;   // 2 .. 8 KiB
    const bool whole_kib = nb % 32 == 0 && nb <= 544;                  // 1 .. 17 KiB: a shared-row kernel of its own
    if (batch == 2) return !whole_kib && row_pairs < 8192;
    return !short_rows || silu;
}

// Per kernel instantiation (one static instance each): the dynamic LDS limit is raised once, to
// the most any launch of this kernel may ask for and never lowered again, so launches from
// several host threads cannot undercut one another; workgroups per CU are looked up once per
// distinct LDS size and kept in a small process-wide table.
class KernelGeometry {
public:
    // false when the runtime refuses the LDS grant
    bool grant(const void *kernel, uint32_t max_dynamic_lds) {
        if (granted_.load(std::memory_order_acquire)) return true;
        std::lock_guard<std::mutex> lock(mu_);
        if (granted_.load(std::memory_order_relaxed)) return true;
        if (max_dynamic_lds > 64u * 1024u &&
            hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(max_dynamic_lds)) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        granted_.store(true, std::memory_order_release);
        return true;
    }
    template <class Kernel>
    uint32_t workgroups_per_cu(Kernel kernel, int threads, uint32_t lds) {
        std::lock_guard<std::mutex> lock(mu_);
        for (uint32_t i = 0; i < n_; ++i)
            if (lds_[i] == lds) return occ_[i];
        int occ = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kernel, threads, lds) != hipSuccess || occ < 1) {
            (void)hipGetLastError();
            occ = 1;
        }
        if (n_ < kSlots) {
            lds_[n_] = lds;
            occ_[n_] = static_cast<uint32_t>(occ);
            ++n_;
        }
        return static_cast<uint32_t>(occ);
    }

private:
    static constexpr uint32_t kSlots = 32;
    std::mutex mu_;
    std::atomic<bool> granted_{false};
    uint32_t lds_[kSlots] = {}, occ_[kSlots] = {}, n_ = 0;
};

// Parked units per wave for batch M.
inline uint32_t park_capacity(uint32_t m) { return kParkFloats / (m * (m >= 4 ? 4u : 2u)); }

// Picks the workgroup count: at most max_wgs_per_cu per CU (all co-resident)
// unless the park capacity forces more, and balanced in whole units per
// workgroup and whole workgroups per CU; larger grids win ties.
inline uint32_t pick_grid(uint32_t units, uint32_t nsteps, uint32_t m, uint32_t waves_per_wg, uint32_t cus,
                          uint32_t max_wgs_per_cu) {
    if (units <= cus) return units ? units : 1;
    const uint32_t cap = park_capacity(m);
    auto fits = [&](uint32_t g) {
        const uint32_t per_group = (units + g - 1) / g;
        return max_units_touched(per_group, nsteps, waves_per_wg) <= cap;
    };
    uint32_t hi = cus * max_wgs_per_cu;
    if (hi > units) hi = units;
    uint32_t best_g = 0;
    double best = -1.0;
    for (uint32_t g = cus; g <= hi; ++g) {
        if (!fits(g)) continue;
        const uint32_t per_group = (units + g - 1) / g;
        const double eff_group = static_cast<double>(units) / (static_cast<double>(per_group) * g);
        const uint32_t per_cu = (g + cus - 1) / cus;
        const double eff_cu = static_cast<double>(g) / (static_cast<double>(per_cu) * cus);
        const double score = eff_group * eff_cu;
        if (score >= best - 1e-12) {   // ascending g: equal scores keep the larger grid
            best_g = g;
            if (score > best) best = score;
        }
    }
    if (best_g) return best_g;
    uint32_t g = hi;                   // very tall matrices: more workgroups than fit at once
    while (!fits(g)) g += cus;
    return g;
}

}  // namespace q8mi
