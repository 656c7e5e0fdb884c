// Matrix-core variant of the Q8_0 x Q8_1 GEMV for small batches (3 .. 16
// activation rows), shared by the GEMV family and the fused LM-head kernel.
//
// From batch 3 on the dot-product GEMV is bound by its VALU work (eight dot4 per
// weight block and activation row).  Here the int8 dots go to
// v_mfma_i32_16x16x32_i8 instead, and the VALU only rescales: the weights are
// still read exactly once and the kernel stays HBM-bound up to batch 16.
//
// One MFMA multiplies A (16 x 32) by B (32 x 16).  Its K extent is 32 = one Q8
// block, so one instruction may only ever see one block per (row, column) pair,
// but nothing says the 16 columns must be 16 weight rows.  They are 4 weight
// rows x 4 K-chunks, and the 16 A rows are 4 activation rows x the same 4
// K-chunks:
//     column n = 4 c + r   weight row r of the unit, block  kb(c, s)
//     row    i = 4 c' + m  activation row m,           block  kb(c', s)
//     kb(c, s) = 32 item + 4 s + c       (s = 0..7: eight MFMAs per item)
// so one step consumes 128 contiguous bytes of each of the four rows.  The global loads are issued
// in memory order (lane L reads bytes 8 (L % 16) .. of row L / 16: consecutive lanes, consecutive
// addresses, which is what the vector memory path coalesces) and the 8-byte pieces are then moved to
// the lanes the MFMA wants them in (lane 16 q + 4 c + r takes from lane 16 r + 4 c + q) with
// ds_bpermute, which uses the LDS crossbar but no LDS memory.
// D[i][n] pairs chunk c' of an activation row with chunk c of a weight row; the
// products with c' == c are the wanted int32 block dots, the other three
// quarters of D are discarded.  A lane holds D[4 q + v][n] (q = lane / 16,
// v = 0..3), so the wanted values sit in the lanes with q == c, all four
// registers of them (m = v): no per-lane register selection is needed.
// Matrix-core time is free here (an HBM-bound stream needs under 2 % of the
// int8 MFMA rate); what the layout buys is a unit of only FOUR weight rows, so
// that a 5120-row matrix still splits into 1280 units.
//
// Work decomposition (as in the dot-product GEMV): unit = 4 rows, item = 32
// blocks of a unit (1 KiB per row: eight 8-byte loads per lane, plus the row's 32 fp16
// scales), a workgroup owns a list of units, its waves split the item list
// evenly and park partial sums per touched unit in LDS.  A parked entry is
// [chunk][row][activation row]: the four chunk partials of a row are added in
// the combine phase, in chunk order.
// Batches above 4 reuse the weight fragment for MG = ceil(batch / 4) MFMAs with
// different activation fragments.
#pragma once

#include <type_traits>

#include "q8mi_gemv_core.hpp"

namespace q8mi {

typedef int v2i __attribute__((ext_vector_type(2)));

constexpr uint32_t kMfmaItemBlocks = 32;   // blocks of a row per item: 4 chunks x 8 steps
constexpr uint32_t kMfmaUnitRows = 4;

// LDS image of the activations:
//   quants   [batch rows][nb][32 B], row m at mfma_xq_row_base(m).  A fragment read (lane =
//            activation row m, chunk c, k-quarter q) touches row_base(m) + 32 c + 8 q (+ the
//            step's offset).  The 32 lanes of a half-wave (four rows, four chunks, two quarters)
//            read 8 bytes each: per row the slots {0, 8} + 32 c of a 128-byte window, so row
//            bases that are 0, 16, 128 and 144 modulo 256 give 32 different slots of a 256-byte
//            span (no two lanes on one bank, whether the LDS has 32 or 64 of them)
//   scales   [nb][MP] fp32 (MP = 4 MG activation rows, padded): the four chunks of a step read
//            four neighbouring MP-float groups
__host__ __device__ inline uint32_t mfma_xq_row_base(uint32_t m, uint32_t nb) {   // nb % 8 == 0
    return m * (nb * 32 + 256) + 16 * (m & 1u) + 128 * ((m >> 1) & 1u);
}
__host__ __device__ inline uint32_t mfma_xq_bytes(uint32_t nb, uint32_t batch) { return batch * (nb * 32 + 256); }
// half_scales: the scale table as fp16 instead of fp32 (half the size, one conversion per use); for
// activations that would not fit otherwise.
inline uint32_t mfma_x_lds_bytes(uint32_t nb, uint32_t batch, uint32_t mg, bool half_scales = false) {
    return mfma_xq_bytes(nb, batch) + nb * 4 * mg * (half_scales ? 2 : 4);
}
// Floats one wave parks per touched unit.
inline uint32_t mfma_park_floats_per_unit(uint32_t mg) { return 4 * kMfmaUnitRows * 4 * mg; }

// Items a wave keeps in flight (each 4 rows x 1 KiB of quants + their scales).
#ifndef Q8MI_MFMA_DEPTH
#define Q8MI_MFMA_DEPTH 2
#endif
constexpr int kMfmaDepth = Q8MI_MFMA_DEPTH;
#ifndef Q8MI_MFMA_GEMV_DEPTH
#define Q8MI_MFMA_GEMV_DEPTH 1
#endif
constexpr int kMfmaGemvDepth = Q8MI_MFMA_GEMV_DEPTH;   // the layer-sized GEMVs (Q8_1 activations)

struct MfmaItem {
    v2i q[8];   // per step: bytes 8 t .. 8 t + 7 of the step's 128 bytes of row L / 16 (memory order),
                // t = (L % 16) ^ 2 for rows 2 and 3, L % 16 for rows 0 and 1
    int d;      // fp16 scales 2 t, 2 t + 1 of the item's 32, row L / 16
};

// Copies `batch` rows of Q8_1 activations into the LDS image above, in two halves: issue() puts
// the first trip of loads in flight and consumes nothing, finish() converts them, runs any further
// trips and ends with a barrier.  Loads return in order, so weight loads the caller issues between
// the two stay in flight while the first trip is converted.
template <int MG, int THREADS, bool HS>
struct MfmaStage {
    static constexpr uint32_t MP = 4 * MG;
    static constexpr int kBatch = 4;
    v4i v[kBatch];

    // y must be 16-byte aligned (the launchers use the dot-product kernel otherwise)
    __device__ __forceinline__ void issue(const uint8_t *y, uint32_t nb, uint32_t batch) {
        const v4i *src = reinterpret_cast<const v4i *>(y);
        const uint32_t total_ch = batch * (nb * 9 / 4);
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const uint32_t c = u * THREADS + threadIdx.x;
            v[u] = src[c < total_ch ? c : 0];
        }
    }

    __device__ __forceinline__ void finish(uint8_t *smem, const uint8_t *y, uint32_t nb, uint32_t batch) {
        uint8_t *xq = smem;
        uint8_t *xd = smem + mfma_xq_bytes(nb, batch);
        // row by row (a row is nb * 36 bytes, a multiple of 16: nb % 8 == 0), so that locating a dword
        // needs no division by nb; all loads of a trip are issued before the first is used
        const uint32_t row_dw = nb * 9, row_ch = row_dw / 4;
        auto put = [&](uint32_t m, uint32_t g, uint32_t word) {   // g: dword index inside row m
            const uint32_t kb = g / 9, part = g % 9;
            if (part == 0) {
                if (HS) *reinterpret_cast<uint16_t *>(xd + (kb * MP + m) * 2) = static_cast<uint16_t>(word & 0xffffu);
                else *reinterpret_cast<float *>(xd + (kb * MP + m) * 4) = half_bits_to_float(static_cast<uint16_t>(word & 0xffffu));
            } else {
                *reinterpret_cast<uint32_t *>(xq + mfma_xq_row_base(m, nb) + kb * 32 + (part - 1) * 4) = word;
            }
        };
        const v4i *src = reinterpret_cast<const v4i *>(y);
        const uint32_t total_ch = batch * row_ch;
        auto put4 = [&](uint32_t c, const v4i &w) {
            if (c < total_ch) {
                uint32_t m = 0, cc = c;                 // batch <= 32: a short subtract loop beats a division
                while (cc >= row_ch) { cc -= row_ch; ++m; }
                put(m, 4 * cc + 0, static_cast<uint32_t>(w.x));
                put(m, 4 * cc + 1, static_cast<uint32_t>(w.y));
                put(m, 4 * cc + 2, static_cast<uint32_t>(w.z));
                put(m, 4 * cc + 3, static_cast<uint32_t>(w.w));
            }
        };
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
        // scales of the padding rows batch .. 4 MG - 1 (their products are never stored; keep them finite)
        if (batch < MP) {
            const uint32_t pad = MP - batch;
            for (uint32_t i = threadIdx.x; i < nb * pad; i += THREADS) {
                const uint32_t kb = i / pad, m = batch + i % pad;
                if (HS) *reinterpret_cast<uint16_t *>(xd + (kb * MP + m) * 2) = 0;
                else *reinterpret_cast<float *>(xd + (kb * MP + m) * 4) = 0.0f;
            }
        }
        __syncthreads();
    }
};

template <int MG, int THREADS, bool HS>
__device__ __forceinline__ void mfma_stage_x(uint8_t *smem, const uint8_t *y, uint32_t nb,
                                             uint32_t batch) {
    MfmaStage<MG, THREADS, HS> st;
    st.issue(y, nb, batch);
    st.finish(smem, y, nb, batch);
}

// The same LDS image from D4 activation blocks ([k / 128][batch] records of 16 B fp32 scales +
// 128 B int8, the prefill GEMM's input), for batches the GEMM entry points hand to this kernel.
template <int MG, int THREADS>
// y points at the first of the `batch` records staged; a super-block holds batch_total records.
__device__ __forceinline__ void mfma_stage_x_d4(uint8_t *smem, const uint8_t *y, uint32_t nb,
                                                uint32_t batch, uint32_t batch_total) {
    constexpr uint32_t MP = 4 * MG;
    constexpr int kBatch = 4;
    uint8_t *xq = smem;
    uint8_t *xd = smem + mfma_xq_bytes(nb, batch);
    const uint32_t nsb = nb / 4;
    const uint32_t per_sb = batch * 9;           // 16-byte chunks per super-block: batch records of 9
    const uint32_t total = nsb * per_sb;
    const v4i *src = reinterpret_cast<const v4i *>(y);   // records are 16-byte aligned by construction
    auto put = [&](uint32_t sb, uint32_t cc, const v4i &v) {   // cc: chunk inside super-block sb
        const uint32_t j = cc / 9, part = cc % 9;
        if (part == 0) {
            const int d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t kb = 4 * sb + t;
                *reinterpret_cast<int *>(xd + (kb * MP + j) * 4) = d[t];
            }
        } else {
            *reinterpret_cast<v4i *>(xq + mfma_xq_row_base(j, nb) + sb * 128 + (part - 1) * 16) = v;
        }
    };
    for (uint32_t base = 0; base < total; base += THREADS * kBatch) {
        v4i v[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const uint32_t c = base + u * THREADS + threadIdx.x;
            const uint32_t cc = c < total ? c : 0;
            v[u] = src[static_cast<uint64_t>(cc / per_sb) * batch_total * 9 + cc % per_sb];
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const uint32_t c = base + u * THREADS + threadIdx.x;
            if (c < total) put(c / per_sb, c % per_sb, v[u]);
        }
    }
    if (batch < MP) {
        const uint32_t pad = MP - batch;
        for (uint32_t i = threadIdx.x; i < nb * pad; i += THREADS) {
            const uint32_t kb = i / pad, m = batch + i % pad;
            *reinterpret_cast<float *>(xd + (kb * MP + m) * 4) = 0.0f;
        }
    }
    __syncthreads();
}

// Streams the items [i0, i1) of the workgroup's unit sequence (item i = part i % nitems of unit
// i / nitems, nitems = ceil(nb / 32)).
//   row_ptr(u)             the weight row (scale plane) this lane LOADS for unit u: fragment row lane / 16,
//                          clamped to a readable row
//   park(kk, acc)          once per unit touched (kk = 0, 1, ...), wave-uniform control flow; acc[g][v] is
//                          this lane's partial sum for activation row 4 g + v and fragment row lane % 4,
//                          meaningful in the lanes with lane / 16 == (lane % 16) / 4; must not touch
//                          global memory
// Must be called by every wave of the workgroup (contains the staging barrier).
// DEPTH: items a wave keeps in flight.  Two for the long LM-head stream and the D4 route; one for
// the layer-sized GEMVs (measured 2 % faster there at M = 4..8, and much slower on the vocabulary).
template <int MG, int THREADS, bool HS, bool D4, int DEPTH = kMfmaDepth, class RowPtr, class Park>
__device__ __forceinline__ void mfma_stream(uint8_t *smem, const uint8_t *y, uint32_t nb, uint32_t batch,
                                            uint32_t d4_batch_total, const UnitSeq &useq, uint32_t i0, uint32_t i1, RowPtr row_ptr,
                                            Park park) {
    constexpr uint32_t MP = 4 * MG;
    constexpr float kMagic = 12582912.0f;
    const uint32_t nitems = (nb + kMfmaItemBlocks - 1) / kMfmaItemBlocks;
    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t q = lane >> 4, c = (lane >> 2) & 3u, m4 = lane & 3u;
    if (i1 <= i0) {
        if constexpr (D4) mfma_stage_x_d4<MG, THREADS>(smem, y, nb, batch, d4_batch_total);
        else mfma_stage_x<MG, THREADS, HS>(smem, y, nb, batch);
        return;
    }
    const uint32_t n_items = i1 - i0;


    // activation loads first, the first weight items behind them (they stay in flight while the
    // activations are converted)
    MfmaStage<MG, THREADS, HS> xstage;
    if constexpr (!D4) xstage.issue(y, nb, batch);
    asm volatile("" ::: "memory");   // the activation loads stay ahead of the weight loads
    MfmaItem items[DEPTH];
    uint32_t ik = i0 / nitems, istep = i0 % nitems, ileft = n_items;
    const uint8_t *irow = row_ptr(useq.unit(ik));
    // Lane L loads slot (L % 16) ^ swz of row L / 16, swz = 2 for rows 2 and 3: the operand shuffle
    // below then reads, per half-wave, source lanes that differ modulo 32 (rows m and m + 2 would
    // otherwise meet on the same banks of the shuffle network).
    const uint32_t l16 = (lane & 15u) ^ ((lane >> 4) & 2u);
    auto issue = [&](MfmaItem &it) {
        const uint32_t left = nb - istep * kMfmaItemBlocks;          // blocks of the row from this item on
        const uint32_t vsteps = left >= kMfmaItemBlocks ? 8u : left / 4;   // steps with real blocks (nb % 8 == 0)
        it.d = *reinterpret_cast<const int *>(irow + istep * 64 + l16 * 4);   // stays inside the row
        const uint8_t *qp = irow + 2 * nb + istep * 1024 + l16 * 8;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            // steps past the row's end re-read step 0; compute gives them a zero scale
            // read once per launch: streaming cache hint, as in the dot-product core
            it.q[s] = __builtin_nontemporal_load(
                reinterpret_cast<const v2i *>(qp + (static_cast<uint32_t>(s) < vsteps ? s * 128 : 0)));
        }
        if (ileft > 1) {          // otherwise keep re-reading the last real item
            --ileft;
            if (++istep == nitems) {
                istep = 0;
                ++ik;
                irow = row_ptr(useq.unit(ik));
            }
        }
    };
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue(items[d]);
    asm volatile("" ::: "memory");   // keeps the loads above from being moved below the staging barrier
    if constexpr (D4) mfma_stage_x_d4<MG, THREADS>(smem, y, nb, batch, d4_batch_total);
    else xstage.finish(smem, y, nb, batch);

    const uint8_t *xq = smem;
    const uint8_t *xd = smem + mfma_xq_bytes(nb, batch);
    // activation fragment rows of this lane, one per MFMA group (clamped: rows past the batch are never stored)
    uint32_t a_row[MG];
#pragma unroll
    for (int g = 0; g < MG; ++g) {
        const uint32_t m = 4 * g + m4;
        a_row[g] = mfma_xq_row_base(m < batch ? m : batch - 1, nb) + 32 * c + 8 * q;
    }
    // source lanes of the operand shuffle (byte addresses for ds_bpermute)
    const uint32_t swz = m4 & 2u;
    const int src_q = static_cast<int>((16 * m4 + ((4 * c + q) ^ swz)) * 4);
    v4i seed;
    seed.x = seed.y = seed.z = seed.w = 0x4B400000;   // 1.5 * 2^23: the int32 result read as fp32 is 12582912 + S
    asm volatile("" : "+v"(seed));

    float acc[MG][4];
#pragma unroll
    for (int g = 0; g < MG; ++g)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[g][v] = 0.0f;

    uint32_t cstep = i0 % nitems, kk = 0;
    // one item: `done` counts the items consumed so far, this one included
    auto consume = [&](const MfmaItem &it, uint32_t done) {
            const uint32_t left = nb - cstep * kMfmaItemBlocks;
            const uint32_t vsteps = left >= kMfmaItemBlocks ? 8u : left / 4;
            const uint8_t *xq_chunk = xq + cstep * 1024;
            constexpr uint32_t kSc = HS ? 2 : 4;   // bytes per scale
            const uint8_t *xd_chunk = xd + (cstep * kMfmaItemBlocks + c) * MP * kSc;
            auto load_dx = [&](const uint8_t *p) {
                float4 v;
                if (HS) {
                    const uint2 h = *reinterpret_cast<const uint2 *>(p);
                    v.x = half_bits_to_float(static_cast<uint16_t>(h.x & 0xffffu));
                    v.y = half_bits_to_float(static_cast<uint16_t>(h.x >> 16));
                    v.z = half_bits_to_float(static_cast<uint16_t>(h.y & 0xffffu));
                    v.w = half_bits_to_float(static_cast<uint16_t>(h.y >> 16));
                } else {
                    v = *reinterpret_cast<const float4 *>(p);
                }
                return v;
            };
            // activation fragments and scales are fetched one step ahead of the MFMAs that use them
            long a_nxt[MG];
            float4 dx_nxt[MG];
#pragma unroll
            for (int g = 0; g < MG; ++g) {
                a_nxt[g] = *reinterpret_cast<const long *>(xq_chunk + a_row[g]);
                dx_nxt[g] = load_dx(xd_chunk + 4 * kSc * g);
            }
            // the operand and scale shuffles run one step ahead as well: LDS operations complete in
            // order, so a shuffle issued right before its use would expose the whole LDS latency
            // (and that of the reads issued just before it) in every step
            auto shuffle_scale = [&](int s) {
                // halfword 4 s + c of the row's scales: dword 2 s + c / 2 (held by lane 16 r + 2 s + c / 2), half c % 2
                return static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(
                    static_cast<int>((16 * m4 + ((2 * s + (c >> 1)) ^ swz)) * 4), it.d));
            };
            auto shuffle_quants = [&](int s) {
                v2i bq;
                bq.x = __builtin_amdgcn_ds_bpermute(src_q, it.q[s].x);
                bq.y = __builtin_amdgcn_ds_bpermute(src_q, it.q[s].y);
                return bq;
            };
            // Items with all eight steps inside the row (every item when nb % 32 == 0, as for all layer
            // shapes) take a copy of the loop in which the step count is a constant: the selects that
            // guard the row's end and the address arithmetic behind them fold away (about ten of the
            // fifty-odd instructions of a step).
            auto run_steps = [&](auto full_tag) {
            constexpr bool kFull = decltype(full_tag)::value;
            const uint32_t nvalid = kFull ? 8u : vsteps;
            uint32_t dword_nxt = shuffle_scale(0);
            v2i bq_nxt = shuffle_quants(0);
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                long a_cur[MG];
                float4 dx_cur[MG];
#pragma unroll
                for (int g = 0; g < MG; ++g) { a_cur[g] = a_nxt[g]; dx_cur[g] = dx_nxt[g]; }
                const uint32_t dword = dword_nxt;
                const v2i bq = bq_nxt;
                if (s < 7) {
                    // steps past the row's end read step 0 again (finite values; their weight scale is zero)
                    const uint32_t sn = static_cast<uint32_t>(s + 1) < nvalid ? s + 1 : 0;
#pragma unroll
                    for (int g = 0; g < MG; ++g) {
                        a_nxt[g] = *reinterpret_cast<const long *>(xq_chunk + a_row[g] + sn * 128);
                        dx_nxt[g] = load_dx(xd_chunk + sn * 4 * MP * kSc + 4 * kSc * g);
                    }
                    dword_nxt = shuffle_scale(s + 1);
                    bq_nxt = shuffle_quants(s + 1);
                }
                // keeps the compiler's scheduler from sinking the look-ahead above back to its uses
                __builtin_amdgcn_sched_barrier(0);
                const uint16_t hbits = static_cast<uint16_t>((c & 1u) ? (dword >> 16) : (dword & 0xffffu));
                const float dw = static_cast<uint32_t>(s) < nvalid ? half_bits_to_float(hbits) : 0.0f;
                const float cw = -kMagic * dw;
                const long b = __builtin_bit_cast(long, bq);
                v4i r[MG];
#pragma unroll
                for (int g = 0; g < MG; ++g) r[g] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_cur[g], b, seed, 0, 0, 0);
#pragma unroll
                for (int g = 0; g < MG; ++g) {
                    acc[g][0] = fmaf(fmaf(as_f32(r[g].x), dw, cw), dx_cur[g].x, acc[g][0]);
                    acc[g][1] = fmaf(fmaf(as_f32(r[g].y), dw, cw), dx_cur[g].y, acc[g][1]);
                    acc[g][2] = fmaf(fmaf(as_f32(r[g].z), dw, cw), dx_cur[g].z, acc[g][2]);
                    acc[g][3] = fmaf(fmaf(as_f32(r[g].w), dw, cw), dx_cur[g].w, acc[g][3]);
                }
            }
            };
            if (vsteps == 8) run_steps(std::true_type{});
            else run_steps(std::false_type{});
            ++cstep;
            if (cstep == nitems || done == n_items) {
                park(kk, acc);
                ++kk;
#pragma unroll
                for (int g = 0; g < MG; ++g)
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[g][v] = 0.0f;
            }
            if (cstep == nitems) cstep = 0;
    };
    // Whole rounds of kMfmaDepth items, each slot refilled as soon as it is consumed (past the
    // last item the refills re-read it, so the loop stays branch-free and the load counters
    // exact); then the items of a last, partial round, without refills.
    uint32_t t = 0;
    for (; t + DEPTH <= n_items; t += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            consume(items[d], t + d + 1);
            issue(items[d]);
        }
    }
#pragma unroll
    for (int d = 0; d < DEPTH - 1; ++d)
        if (t + d < n_items) consume(items[d], t + d + 1);
}

}  // namespace q8mi
