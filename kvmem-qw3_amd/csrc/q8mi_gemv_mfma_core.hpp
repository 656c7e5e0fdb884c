// Matrix-core variant of the Q8_0 x Q8_1 GEMV for small batches (3 .. 16
// activation rows), shared by the GEMV family and the fused LM-head kernel.
//
// From batch 3 on the dot-product GEMV is bound by its VALU work (eight dot4 per
// weight block and activation row).  Here the int8 dots go to
// v_mfma_i32_4x4x4_16B_i8 instead: sixteen independent 4 x 4 x 4 products per
// instruction, one per group of four lanes.  Lane 4 b + n of a wave works, in
// every step of 16 blocks, on one block of weight row n of the unit (its 32
// quant bytes: eight dwords, eight chained MFMAs) and feeds the matrix unit the
// same block of activation row n (of 4 g + n for further groups of four
// activation rows), so its four result registers are the complete int32 block
// dots of weight row n with activation rows 0..3.  Every lane and every
// register carries a wanted sum; the VALU only rescales them (2 FMAs per sum,
// accumulator seeded with 1.5 * 2^23 as in the GEMM) and the weights are still
// read exactly once.  (A first version used v_mfma_i32_16x16x32_i8 with 4 rows
// x 4 K-chunks as its 16 columns; only the diagonal quarter of its results was
// wanted, operands had to be shuffled into place, and a step of 512 bytes cost
// 37..51 instructions against about 45 for 2 KiB here.)
//
// Work decomposition (as in the dot-product GEMV of q8mi_gemv_core.hpp): unit =
// 4 rows, item = 32 blocks of a unit (1 KiB per row, two steps), a workgroup owns
// a list of units, its waves split the item list evenly and park partial sums
// per touched unit in LDS.  A parked entry is [4 block groups][row][activation
// row]: the four partials of a row are added in the combine phase, in order.
// Batches above 4 reuse the weight registers for MG = ceil(batch / 4) chains of
// MFMAs with different activation operands.
#pragma once

#include <type_traits>

#include "q8mi_gemv_core.hpp"

namespace q8mi {

typedef int v2i __attribute__((ext_vector_type(2)));

constexpr uint32_t kMfmaItemBlocks = 32;   // blocks of a row per item: 4 chunks x 8 steps
constexpr uint32_t kMfmaUnitRows = 4;

// LDS image of the activations:
//   quants   [batch rows][nb][32 B], row m at mfma_xq_row_base(m).  A lane reads the two 16-byte
//            halves of its block of activation row lane % 4; the row bases (0, 16, 128 and 144
//            modulo 256) spread the four rows of a lane group over different banks
//   scales   [nb][MP] fp32 (MP = 4 MG activation rows, padded): one 16-byte read per block and
//            group of four activation rows
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

// Items a wave keeps in flight (each 4 rows x 1 KiB of quants + their scales): two for long streams
// such as a vocabulary and for the D4 route, one for the layer-sized GEMVs.
constexpr int kMfmaDepth = 2;
constexpr int kMfmaGemvDepth = 1;

struct MfmaItem {
    v4i q[2][2];      // step t (16 blocks, 512 bytes of a row): bytes 16 (L / 4) .. of its first and of its second 256
    uint16_t d[2];    // fp16 scale of the block this lane ends up with (see mfma_stream)
};

// Copies `batch` rows of Q8_1 activations into the LDS image above, in two halves: issue() puts
// the first trip of loads in flight and consumes nothing, finish() stores them, runs any further
// trips and ends with a barrier.  Loads return in order, so weight loads the caller issues between
// the two stay in flight while the first trip is stored.  One thread moves one 36-byte block per
// trip: its header dword and its 32 quant bytes as two 16-byte pieces (4-byte aligned loads, 16-byte
// aligned LDS stores), so y needs no more than the 4-byte alignment of the block type.
template <int MG, int THREADS, bool HS>
struct MfmaStage {
    static constexpr uint32_t MP = 4 * MG;
    // Blocks a thread has in flight per trip.  (Six per trip, which makes eight rows of 5120 columns
    // one trip instead of two and eight rows of 17408 two instead of five, changed no launch by
    // more than its run-to-run spread: the trips overlap the first weight requests.)
    static constexpr int kBatch = 2;
    struct Dwords4 {
        int x, y, z, w;
    } __attribute__((packed, aligned(4)));
    struct Block {
        uint32_t head;
        v4i lo, hi;
    };
    Block v[kBatch];

    static __device__ __forceinline__ Block load(const uint8_t *y, uint32_t i) {
        const uint8_t *src = y + static_cast<uint64_t>(i) * kQ81Bytes;
        Block blk;
        blk.head = *reinterpret_cast<const uint32_t *>(src);
        const Dwords4 a = *reinterpret_cast<const Dwords4 *>(src + 4);
        const Dwords4 c = *reinterpret_cast<const Dwords4 *>(src + 20);
        blk.lo = v4i{a.x, a.y, a.z, a.w};
        blk.hi = v4i{c.x, c.y, c.z, c.w};
        return blk;
    }

    static __device__ __forceinline__ void store(uint8_t *smem, uint32_t nb, uint32_t batch, uint32_t i, const Block &blk) {
        uint8_t *xq = smem;
        uint8_t *xd = smem + mfma_xq_bytes(nb, batch);
        uint32_t m = 0, kb = i;                  // batch <= 32: a short subtract loop beats a division
        while (kb >= nb) { kb -= nb; ++m; }
        uint8_t *dst = xq + mfma_xq_row_base(m, nb) + kb * 32;
        *reinterpret_cast<v4i *>(dst) = blk.lo;
        *reinterpret_cast<v4i *>(dst + 16) = blk.hi;
        const uint16_t h = static_cast<uint16_t>(blk.head & 0xffffu);
        if (HS) *reinterpret_cast<uint16_t *>(xd + (kb * MP + m) * 2) = h;
        else *reinterpret_cast<float *>(xd + (kb * MP + m) * 4) = half_bits_to_float(h);
    }

    __device__ __forceinline__ void issue(const uint8_t *y, uint32_t nb, uint32_t batch) {
        const uint32_t total = batch * nb;
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const uint32_t i = u * THREADS + threadIdx.x;
            v[u] = load(y, i < total ? i : 0u);
        }
    }

    __device__ __forceinline__ void finish(uint8_t *smem, const uint8_t *y, uint32_t nb, uint32_t batch) {
        const uint32_t total = batch * nb;
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const uint32_t i = u * THREADS + threadIdx.x;
            if (i < total) store(smem, nb, batch, i, v[u]);
        }
        for (uint32_t base = THREADS * kBatch; base < total; base += THREADS * kBatch) {
            Block t[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const uint32_t i = base + u * THREADS + threadIdx.x;
                t[u] = load(y, i < total ? i : 0u);
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const uint32_t i = base + u * THREADS + threadIdx.x;
                if (i < total) store(smem, nb, batch, i, t[u]);
            }
        }
        // scales of the padding rows batch .. 4 MG - 1 (their products are never stored; keep them finite)
        if (batch < MP) {
            uint8_t *xd = smem + mfma_xq_bytes(nb, batch);
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

// The sums of one item over the sixteen lane quads of the wave, for the item-wise split below: lane
// 16 rho + 4 q + n holds acc[g][v] for weight row n; on return lane (rho, q odd, n) holds the wave's
// total for weight row n and activation row (q >> 1) + 2 rho (MG == 2; both odd q hold activation
// row rho for MG == 1).  Every step halves the registers instead of leaving copies: the halves of
// two registers change places (v_permlane32_swap, then v_permlane16_swap for the rows of 16 lanes)
// and one addition folds both; the quads of a row of 16 follow by two DPP additions.  A fixed tree:
// same bits on every run.
template <int MG>
__device__ __forceinline__ float mfma_item_total(const float (&acc)[MG][4]) {
    static_assert(MG == 1 || MG == 2, "item-wise sums are built for up to eight activation rows");
    typedef unsigned v2u __attribute__((ext_vector_type(2)));
    auto fold32 = [](float a, float b) {   // lanes 0..31: a summed over lane bit 5; lanes 32..63: b
        const v2u r = __builtin_amdgcn_permlane32_swap(static_cast<unsigned>(as_i32(a)), static_cast<unsigned>(as_i32(b)), false, false);
        return as_f32(static_cast<int>(r.x)) + as_f32(static_cast<int>(r.y));
    };
    auto fold16 = [](float a, float b) {   // rows 0, 2: a summed over lane bit 4; rows 1, 3: b
        const v2u r = __builtin_amdgcn_permlane16_swap(static_cast<unsigned>(as_i32(a)), static_cast<unsigned>(as_i32(b)), false, false);
        return as_f32(static_cast<int>(r.x)) + as_f32(static_cast<int>(r.y));
    };
    auto quads = [](float w) {        // w summed over the quads q and q ^ 2 of its row
        // row_ror:8: lane i of every row of 16 reads lane (i + 8) % 16
        return w + as_f32(__builtin_amdgcn_update_dpp(0, as_i32(w), 0x128, 0xf, 0xf, false));
    };
    float v;
    if constexpr (MG == 2) {
        float z[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) z[j] = fold32(acc[0][j], acc[1][j]);   // lower half: activation row j, upper: 4 + j
        const float u0 = quads(fold16(z[0], z[2]));   // row rho: activation row 2 rho
        const float u1 = quads(fold16(z[1], z[3]));   // row rho: activation row 2 rho + 1
        // quads 0, 1 keep u0, quads 2, 3 take u1
        v = as_f32(__builtin_amdgcn_update_dpp(as_i32(u0), as_i32(u1), 0xE4, 0xf, 0xC, false));
    } else {
        const float z0 = fold32(acc[0][0], acc[0][2]);   // lower half: activation row 0, upper: 2
        const float z1 = fold32(acc[0][1], acc[0][3]);   // lower half: 1, upper: 3
        v = quads(fold16(z0, z1));                       // row rho: activation row rho
    }
    // quad q + quad q - 1: complete in the odd quads
    return v + as_f32(__builtin_amdgcn_update_dpp(0, as_i32(v), kDppRowShr4, 0xf, 0xf, true));
}

// Streams the items [i0, i1) of the workgroup's unit sequence (item i = part i % nitems of unit
// i / nitems, nitems = ceil(nb / 32)).
//   row_ptr(u)             the weight row (scale plane) this lane LOADS for unit u: fragment row lane % 4,
//                          clamped to a readable row
//   park(kk, acc)          once per unit touched (kk = 0, 1, ...), wave-uniform control flow; acc[g][v] is
//                          this lane's partial sum for activation row 4 g + v, fragment row lane % 4 and
//                          block group lane / 4 (a quarter of the blocks), meaningful in lanes 0 .. 15;
//                          must not touch global memory
// Must be called by every wave of the workgroup (contains the staging barrier).
// DEPTH: items a wave keeps in flight.
// STREAMING: the quant loads carry the non-temporal hint (every weight byte is read once per launch);
//            worth 5..7 % on streams of 100 MB and more, costs 5..8 % on those of 30..45 MB.
// ITEMWISE: the wave takes the items i0, i0 + W, i0 + 2 W, ... below i1 (W = waves of the workgroup)
//            instead of a contiguous range, so that the workgroup's loads in flight are W neighbouring
//            items: whole rows, not one KiB of eight different row quads (measured with a bare read of
//            the same pattern: 2 x 17408 x 5120 30.7 -> 28.8 us, 8192 x 5120 10.5 -> 9.1 us, 5120 x 17408
//            17.2 -> 16.4 us).  Consecutive items of a wave then belong to different units, so
//            park(t, total) is called after every item t = 0, 1, ... with the lane's entry of
//            mfma_item_total().
template <int MG, int THREADS, bool HS, bool D4, int DEPTH = kMfmaDepth, bool STREAMING = true, bool ITEMWISE = false, class RowPtr, class Park>
__device__ __forceinline__ void mfma_stream(uint8_t *smem, const uint8_t *y, uint32_t nb, uint32_t batch,
                                            uint32_t d4_batch_total, const UnitSeq &useq, uint32_t i0, uint32_t i1, RowPtr row_ptr,
                                            Park park) {
    constexpr uint32_t MP = 4 * MG;
    constexpr float kMagic = 12582912.0f;
    const uint32_t nitems = (nb + kMfmaItemBlocks - 1) / kMfmaItemBlocks;
    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t b = lane >> 2, n4 = lane & 3u;
    if (i1 <= i0) {
        if constexpr (D4) mfma_stage_x_d4<MG, THREADS>(smem, y, nb, batch, d4_batch_total);
        else mfma_stage_x<MG, THREADS, HS>(smem, y, nb, batch);
        return;
    }
    constexpr uint32_t kStride = ITEMWISE ? THREADS / kWave : 1;   // items from one of the wave's to the next
    const uint32_t n_items = (i1 - i0 + kStride - 1) / kStride;
    auto advance = [&](uint32_t &k, uint32_t &step) {   // (unit ordinal, part) of the wave's next item; true: another unit
        step += kStride;
        const uint32_t k0 = k;
        while (step >= nitems) {
            step -= nitems;
            ++k;
        }
        return k != k0;
    };

    // activation loads first, the first weight items behind them (they stay in flight while the
    // activations are converted)
    MfmaStage<MG, THREADS, HS> xstage;
    if constexpr (!D4) xstage.issue(y, nb, batch);
    asm volatile("" ::: "memory");   // the activation loads stay ahead of the weight loads
    MfmaItem items[DEPTH];
    uint32_t ik = i0 / nitems, istep = i0 % nitems, ileft = n_items;
    const uint8_t *irow = row_ptr(useq.unit(ik));
    // A step is 512 bytes of each of the four rows, read as two instructions of 4 x 256 contiguous
    // bytes (every cache line is touched by one instruction only, which is what lets the loads carry
    // the streaming hint: a line that two instructions share is fetched from memory twice under
    // it).  Lane 4 b + n then holds piece b of the first and of the second 256 bytes of row n: half
    // b % 2 of block b / 2 and of block 8 + b / 2.  Lanes b and b ^ 1 swap one piece each, so that
    // an even b ends up with both halves of block b / 2 and an odd b with both halves of block
    // 8 + b / 2: blk is this lane's block of the step.
    const uint32_t par = b & 1u, blk = (b >> 1) + 8 * par;
    auto issue = [&](MfmaItem &it) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            // blocks past the row's end re-read the row's first bytes; compute gives them a zero scale
            const uint32_t kb0 = istep * kMfmaItemBlocks + 16 * t;
            const uint8_t *qp = irow + 2 * nb + b * 16;
            const v4i *p0 = reinterpret_cast<const v4i *>(qp + (kb0 < nb ? kb0 * 32 : 0u));
            const v4i *p1 = reinterpret_cast<const v4i *>(qp + (kb0 + 8 < nb ? (kb0 + 8) * 32 : 0u));
            if constexpr (STREAMING) {
                it.q[t][0] = __builtin_nontemporal_load(p0);
                it.q[t][1] = __builtin_nontemporal_load(p1);
            } else {
                it.q[t][0] = *p0;
                it.q[t][1] = *p1;
            }
            it.d[t] = reinterpret_cast<const uint16_t *>(irow)[kb0 + blk < nb ? kb0 + blk : 0u];
        }
        if (ileft > 1) {          // otherwise keep re-reading the last real item
            --ileft;
            if (advance(ik, istep)) irow = row_ptr(useq.unit(ik));
        }
    };
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue(items[d]);
    asm volatile("" ::: "memory");   // keeps the loads above from being moved below the staging barrier
    if constexpr (D4) mfma_stage_x_d4<MG, THREADS>(smem, y, nb, batch, d4_batch_total);
    else xstage.finish(smem, y, nb, batch);

    const uint8_t *xq = smem;
    const uint8_t *xd = smem + mfma_xq_bytes(nb, batch);
    // activation row this lane feeds to the matrix unit, one per MFMA group (clamped: rows past the
    // batch are never stored)
    uint32_t a_row[MG];
#pragma unroll
    for (int g = 0; g < MG; ++g) {
        const uint32_t m = 4 * g + n4;
        a_row[g] = mfma_xq_row_base(m < batch ? m : batch - 1, nb);
    }
    v4i seed;
    seed.x = seed.y = seed.z = seed.w = 0x4B400000;   // 1.5 * 2^23: the int32 result read as fp32 is 12582912 + S
    asm volatile("" : "+v"(seed));

    float acc[MG][4];
#pragma unroll
    for (int g = 0; g < MG; ++g)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[g][v] = 0.0f;

    constexpr uint32_t kSc = HS ? 2 : 4;   // bytes per activation scale
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

    uint32_t cstep = i0 % nitems, kk = 0;
    // one item's products into acc
    auto compute = [&](const MfmaItem &it) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint32_t kb = cstep * kMfmaItemBlocks + 16 * t + blk;
            const bool valid = kb < nb;
            const uint32_t kbc = valid ? kb : 0u;
            const float dw = valid ? half_bits_to_float(it.d[t]) : 0.0f;
            const float cw = -kMagic * dw;
            // the piece this lane keeps (half par of its block) and the one it receives (the other half)
            v4i keep, recv;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                keep[j] = par ? it.q[t][1][j] : it.q[t][0][j];
                // even b: the first piece of lane + 4; odd b: the second piece of lane - 4
                const int from_up = __builtin_amdgcn_update_dpp(0, it.q[t][0][j], kDppRowShl4, 0xf, 0x5, false);
                recv[j] = __builtin_amdgcn_update_dpp(from_up, it.q[t][1][j], kDppRowShr4, 0xf, 0xA, false);
            }
            v4i a0[MG], a1[MG];   // activation bytes that go with keep and with recv
            float4 dx[MG];
#pragma unroll
            for (int g = 0; g < MG; ++g) {
                const uint8_t *ap = xq + a_row[g] + kbc * 32;
                a0[g] = *reinterpret_cast<const v4i *>(ap + 16 * par);
                a1[g] = *reinterpret_cast<const v4i *>(ap + 16 * (par ^ 1u));
                dx[g] = load_dx(xd + (kbc * MP + 4 * g) * kSc);
            }
            v4i r[MG];
#pragma unroll
            for (int g = 0; g < MG; ++g) r[g] = seed;
            // sixteen 4 x 4 x 4 products per instruction, one per group of four lanes: D[v][n] +=
            // sum over the dword's four bytes of x[4 g + v][.] w[n][.]; eight dwords make the block
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int g = 0; g < MG; ++g)
                    r[g] = __builtin_amdgcn_mfma_i32_4x4x4i8(a0[g][j], keep[j], r[g], 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int g = 0; g < MG; ++g)
                    r[g] = __builtin_amdgcn_mfma_i32_4x4x4i8(a1[g][j], recv[j], r[g], 0, 0, 0);
#pragma unroll
            for (int g = 0; g < MG; ++g) {
                acc[g][0] = fmaf(fmaf(as_f32(r[g].x), dw, cw), dx[g].x, acc[g][0]);
                acc[g][1] = fmaf(fmaf(as_f32(r[g].y), dw, cw), dx[g].y, acc[g][1]);
                acc[g][2] = fmaf(fmaf(as_f32(r[g].z), dw, cw), dx[g].z, acc[g][2]);
                acc[g][3] = fmaf(fmaf(as_f32(r[g].w), dw, cw), dx[g].w, acc[g][3]);
            }
        }
    };
    // after an item: `done` counts the items consumed so far, this one included
    auto finish = [&](uint32_t done) {
        if constexpr (ITEMWISE) {
            park(done - 1, mfma_item_total<MG>(acc));
#pragma unroll
            for (int g = 0; g < MG; ++g)
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[g][v] = 0.0f;
            uint32_t unused = 0;
            advance(unused, cstep);
        } else {
            ++cstep;
            if (cstep == nitems || done == n_items) {
                // the sixteen lanes of equal row meet in four: lanes 0 .. 15 then hold, for row lane % 4,
                // the sum over a quarter of the blocks
#pragma unroll
                for (int g = 0; g < MG; ++g)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        acc[g][v] += lane_xor<16>(acc[g][v]);
                        acc[g][v] += lane_xor<32>(acc[g][v]);
                    }
                park(kk, acc);
                ++kk;
#pragma unroll
                for (int g = 0; g < MG; ++g)
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[g][v] = 0.0f;
            }
            if (cstep == nitems) cstep = 0;
        }
    };
    // Whole rounds of DEPTH items, each slot refilled as soon as its products are formed and before
    // its sums are parked (past the last item the refills re-read it, so the loop stays branch-free
    // and the load counters exact); then the items of a last, partial round, without refills.
    uint32_t t = 0;
    for (; t + DEPTH <= n_items; t += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            compute(items[d]);
            issue(items[d]);
            finish(t + d + 1);
        }
    }
#pragma unroll
    for (int d = 0; d < DEPTH - 1; ++d)
        if (t + d < n_items) {
            compute(items[d]);
            finish(t + d + 1);
        }
}

}  // namespace q8mi
