// Q8_0 x Q8_1 GEMV for batch 1..4 as many small, independent workgroups (gfx950).
// Reference semantics: src/mmvq_q8.cu:193-280 (plain), :295-399 (two weights), :414-519 (SwiGLU),
// :528-606 (residual add), :976-1068 (fan-out); like the reference's kernel, a weight row is read
// once and reused for every activation row (:221-243).
//
// The unit of work is a ROW PAIR: two weight rows (SwiGLU: a gate row and its up row) from their
// first to their last column.  Workgroups are small (one wave, or the few waves that share a pair),
// own a handful of pairs, write their sums and end; the hardware dispatcher hands the next ones to
// whichever CU has room.  That dynamic hand-out is what balances the chip: a static split of the
// rows over resident workgroups loses 3..5 us per launch to CUs that finish one after the other.
// Measured on MI355X against the static streaming kernels of q8mi_gemv.hip (same bytes):
// 5120 x 5120 8.9 -> 6.6 us, SwiGLU 2 x 17408 x 5120 33.3 -> 28.7 us, 5120 x 17408 20.4 -> 16.7 us;
// a plain streaming read of those sizes takes 6.0, 28.1 and 15.1 us.
//
// Lane layout.  A 1 KiB step of a row is one coalesced wave load: lane l holds 16 bytes, half of
// block l/2.  The two rows of a pair swap half sums with one DPP move, so that even lanes end up
// with the full int32 block dot of the first row and odd lanes with that of the second row: one
// int32 sum and one fp32 rescale per 32-element block and row, and after a five-step butterfly
// over the lanes of equal parity lane 0 holds the first row's result and lane 1 the second's.
//
// Two kernels, by where the activations live:
//   gemv_pairs_ksplit_kernel   rows of 1 to 17 KiB (whole KiB): the waves of a workgroup cut every row
//       into interleaved 1 KiB steps, so each wave needs the activations of its own steps only,
//       loads them once into registers (5 per step and activation row) and keeps them for all
//       pairs of the workgroup; partial sums meet in LDS after the last pair.  With fp32
//       activations (the entry points that quantize inside the GEMV, optionally after an RMS norm;
//       rows of 1..8 KiB) every wave quantizes the 1024 floats of its own step in registers,
//       with the stand-alone quantizer's arithmetic; only the norm's sum of squares crosses the
//       waves, through LDS, in the stand-alone norm's order
//   gemv_pairs_ring_kernel     any other row length: one wave per pair, the activation bytes of a
//       step travel with its weights through a ring of steps in flight (L2 serves them); fp32
//       activations are quantized once per workgroup into LDS by all of its waves
#include <type_traits>

#include "q8mi_gemv_core.hpp"
#include "q8mi_gemv_params.hpp"

namespace q8mi {
namespace {

// 16 bytes of a Q8_1 block: 4-byte aligned by type
struct __attribute__((packed, aligned(4))) Dwords4 {
    int x, y, z, w;
};
__device__ __forceinline__ v4i load_x16(const uint8_t *p) {
    const Dwords4 q = *reinterpret_cast<const Dwords4 *>(p);
    return v4i{q.x, q.y, q.z, q.w};
}

// Row pairs of the concatenated row space: pairs never straddle two weights (a weight with an odd
// number of rows ends with a pair whose second row is a repeat that is not written).
struct PairSpace {
    uint32_t pair_end[4];   // cumulative pair counts per weight
    uint32_t pairs;
    uint32_t ppw;           // consecutive pairs per wave
};

struct PairRows {
    const uint8_t *r0, *r1;   // scale planes of the two rows
    void *dst;
    uint32_t stride;
    uint32_t row0;            // row of r0 within its weight (SwiGLU: the output row)
    bool two;                 // the second row exists
};

template <bool SILU>
__device__ __forceinline__ PairRows resolve_pair(const GemvParams &p, const PairSpace &ps, uint32_t pair, uint64_t row_bytes) {
    PairRows r;
    if constexpr (SILU) {
        r.r0 = p.w[0] + pair * row_bytes;
        r.r1 = p.w[1] + pair * row_bytes;
        r.dst = p.dst[0];
        r.stride = p.stride[0];
        r.row0 = pair;
        r.two = true;
    } else {
        uint32_t seg = 0, base = 0, row_base = 0;
        if (pair >= ps.pair_end[0]) { seg = 1; base = ps.pair_end[0]; row_base = p.row_end[0]; }
        if (pair >= ps.pair_end[1]) { seg = 2; base = ps.pair_end[1]; row_base = p.row_end[1]; }
        if (pair >= ps.pair_end[2]) { seg = 3; base = ps.pair_end[2]; row_base = p.row_end[2]; }
        const uint8_t *w = p.w[0];
        r.dst = p.dst[0]; r.stride = p.stride[0];
        uint32_t rows = p.row_end[0];
        if (seg == 1) { w = p.w[1]; r.dst = p.dst[1]; r.stride = p.stride[1]; rows = p.row_end[1] - row_base; }
        if (seg == 2) { w = p.w[2]; r.dst = p.dst[2]; r.stride = p.stride[2]; rows = p.row_end[2] - row_base; }
        if (seg == 3) { w = p.w[3]; r.dst = p.dst[3]; r.stride = p.stride[3]; rows = p.row_end[3] - row_base; }
        r.row0 = 2 * (pair - base);
        r.two = r.row0 + 1 < rows;
        r.r0 = w + r.row0 * row_bytes;
        r.r1 = r.two ? r.r0 + row_bytes : r.r0;
    }
    return r;
}

// Sum over the lanes of equal parity (xor 2 .. 32): every lane ends with its parity's total.
__device__ __forceinline__ float parity_sum(float v) {
    v += lane_xor<2>(v);
    v += lane_xor<4>(v);
    v += lane_xor<8>(v);
    v += lane_xor<16>(v);
    v += lane_xor<32>(v);
    return v;
}

// Lane 0 holds the first row's totals, lane 1 the second row's (SwiGLU: gate and up).
template <int M, bool SILU>
__device__ __forceinline__ void write_pair(const GemvParams &p, const PairRows &rows, uint32_t lane, const float (&tot)[M]) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
        if constexpr (SILU) {
            const float up = dpp_f32<kDppXor1>(tot[m]);
            if (lane == 0)
                static_cast<float *>(rows.dst)[static_cast<uint64_t>(m) * rows.stride + rows.row0] =
                    (tot[m] / (1.0f + __expf(-tot[m]))) * up;
        } else {
            if (lane == 0 || (lane == 1 && rows.two))
                store_out(p.mode, rows.dst, static_cast<uint64_t>(m) * rows.stride + rows.row0 + lane, tot[m]);
        }
    }
}

// Sum of the squares of one fp32 row in the order of the stand-alone RMS norm (q8mi_rms_norm.hip):
// thread t of the first 256 adds chunks t, t + 256, ... in that order, the 256 partials meet in a
// balanced tree (64 lanes by DPP, then the four wave sums).  Every thread of the workgroup must
// call it (one barrier inside); `red` = four floats of LDS.  partial: this thread's sum, 0 for
// threads beyond the first 256.
__device__ __forceinline__ float first256_tree_sum(float partial, float *red) {
    const uint32_t wave = threadIdx.x / kWave;
    if (wave < 4) {   // wave-uniform
        const float s = wave_sum(partial);
        if (threadIdx.x % kWave == 0) red[wave] = s;
    }
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

// ---- rows of any length: a rolling pipeline over (pair, step) items -------------------------------
// Slot d of the ring holds the two rows' 16 bytes of one step, their scales, and the activation
// bytes and scale of that step (read from global memory with the weights: L2 serves them).  kRing
// items are in flight; the trip count is padded to whole rings with repeats of the last item whose
// sums are never written, so that the load counter the compiler waits on stays exact.
constexpr int kRing = 4;   // 6 changes nothing, 8 is slower (19.4 against 18.1 us at 5120 x 17408)

template <int M, bool XF32>
struct RingSlot {
    v4i q0, q1;
    v4i xq[XF32 ? 1 : M];        // unused when the activations sit in LDS
    uint16_t d0, d1;
    uint16_t dxh[XF32 ? 1 : M];
};

// LDS bytes of M quantized activation rows (XF32): packed int8 then fp32 scales.
inline uint32_t ring_x_lds_bytes(uint32_t nb, uint32_t m) { return m * nb * (32 + 4); }

// XF32: fp32 activations, quantized into LDS by the whole workgroup before the first item is
// consumed (the first loads of every wave are already in flight by then); otherwise one wave per
// workgroup and Q8_1 blocks from global memory.
// NORM (XF32, one row): the row is RMS-normalised before it is quantized, with the arithmetic of the
// stand-alone norm kernel (same bits); workgroup 0 also writes the normalised row.
template <int M, bool SILU, bool XF32, bool NORM = false>
__global__ __launch_bounds__(XF32 ? 512 : kWave) void gemv_pairs_ring_kernel(const GemvParams p, const PairSpace ps) {
    static_assert(!NORM || (XF32 && M == 1), "the fused norm handles one fp32 row");
    extern __shared__ __align__(16) uint8_t smem[];
    __shared__ float red[4];
    const uint32_t nb = p.nb;
    const uint64_t row_bytes = static_cast<uint64_t>(nb) * 34;
    const uint32_t lane = threadIdx.x % kWave;
    const bool odd = lane & 1u;
    const uint32_t npieces = nb * 2, nsteps = (npieces + 63) / 64;
    const uint32_t wave_id = XF32 ? blockIdx.x * (blockDim.x / kWave) + __builtin_amdgcn_readfirstlane(threadIdx.x / kWave)
                                  : blockIdx.x;
    const uint32_t first = wave_id * ps.ppw;
    const bool live = first < ps.pairs;
    if (!XF32 && !live) return;
    const uint32_t end = first + ps.ppw < ps.pairs ? first + ps.ppw : ps.pairs;
    const uint32_t n_items = live ? (end - first) * nsteps : 0u;
    const uint32_t n_padded = (n_items + kRing - 1) / kRing * kRing;
    uint32_t *lds_q = reinterpret_cast<uint32_t *>(smem);
    float *lds_d = reinterpret_cast<float *>(smem + static_cast<size_t>(M) * nb * 32);

    RingSlot<M, XF32> ring[kRing];
    uint32_t ipair = first, istep = 0, ileft = n_items;
    PairRows irows{};
    if (live) irows = resolve_pair<SILU>(p, ps, ipair, row_bytes);
    auto issue = [&](RingSlot<M, XF32> &sl) {
        const uint32_t piece = istep * 64 + lane;
        const uint32_t pc = piece < npieces ? piece : 0u;   // past the row's end: re-read its start, masked below
        const uint32_t blk = pc >> 1;
        sl.q0 = load_q16(irows.r0 + 2 * nb + pc * 16);
        sl.q1 = load_q16(irows.r1 + 2 * nb + pc * 16);
        sl.d0 = reinterpret_cast<const uint16_t *>(irows.r0)[blk];
        sl.d1 = reinterpret_cast<const uint16_t *>(irows.r1)[blk];
        if constexpr (!XF32) {
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const uint8_t *xb = p.y + static_cast<uint64_t>(m * nb + blk) * kQ81Bytes;
                sl.xq[m] = load_x16(xb + 4 + (pc & 1u) * 16);
                sl.dxh[m] = *reinterpret_cast<const uint16_t *>(xb);
            }
        }
        if (ileft > 1) {   // otherwise: keep re-reading the last real item
            --ileft;
            if (++istep == nsteps) {
                istep = 0;
                ++ipair;
                irows = resolve_pair<SILU>(p, ps, ipair, row_bytes);
            }
        }
    };
    if (live) {
#pragma unroll
        for (int d = 0; d < kRing; ++d) issue(ring[d]);
    }
    if constexpr (XF32) {
        asm volatile("" ::: "memory");   // the weight loads above stay ahead of the staging
        const uint32_t per_row = nb * 8, total = static_cast<uint32_t>(M) * per_row;   // float4 chunks
        const bool vec = NORM || ((reinterpret_cast<uintptr_t>(p.xf) % 16 == 0) && (p.x_stride % 4 == 0));
        float scale = 1.0f;
        if constexpr (NORM) {
            float partial = 0.0f;
            if (threadIdx.x < kNormThreads)
                for (uint32_t c = threadIdx.x; c < per_row; c += kNormThreads) partial += chunk_squares(load4<true>(p.xf + c * 4));
            scale = rms_scale(first256_tree_sum(partial, red), nb * 32, p.eps);
        }
        for (uint32_t base = 0; base < total; base += blockDim.x) {
            const uint32_t c = base + threadIdx.x;
            const uint32_t cc = c < total ? c : 0u;
            uint32_t m, within;
            split_index<M>(cc, per_row, m, within);
            const float *src = p.xf + static_cast<uint64_t>(m) * p.x_stride + within * 4;
            Float4 v = vec ? load4<true>(src) : load4<false>(src);
            if constexpr (NORM) {
                v = rms_apply(v, scale, load4<true>(p.norm_w + cc * 4));
                if (p.normalized != nullptr && blockIdx.x == 0 && c < total)
                    *reinterpret_cast<float4 *>(p.normalized + cc * 4) = make_float4(v.x, v.y, v.z, v.w);
            }
            float d;
            const uint32_t packed = quantize4_q8_1(v, d);   // all lanes take part in the exchanges
            if (c < total) {
                lds_q[cc] = packed;
                if (within % 8 == 0) lds_d[m * nb + within / 8] = half_bits_to_float(float_to_half_bits(d));
            }
        }
        __syncthreads();
        if (!live) return;
    }

    float acc[M];
#pragma unroll
    for (int m = 0; m < M; ++m) acc[m] = 0.0f;
    uint32_t cstep = 0, cpair = first;
    for (uint32_t t = 0; t < n_padded; t += kRing) {
#pragma unroll
        for (int d = 0; d < kRing; ++d) {
            const RingSlot<M, XF32> &sl = ring[d];
            const uint32_t piece = cstep * 64 + lane;
            const bool valid = piece < npieces;
            const float dw = valid ? half_bits_to_float(odd ? sl.d1 : sl.d0) : 0.0f;
#pragma unroll
            for (int m = 0; m < M; ++m) {
                v4i xq;
                float dxv;
                if constexpr (XF32) {
                    const uint32_t pc = valid ? piece : 0u;
                    xq = *reinterpret_cast<const v4i *>(&lds_q[(m * nb) * 8 + pc * 4]);
                    dxv = lds_d[m * nb + (pc >> 1)];
                } else {
                    xq = sl.xq[m];
                    dxv = half_bits_to_float(sl.dxh[m]);
                }
                const int sa = dot16(sl.q0, xq);
                const int sb = dot16(sl.q1, xq);
                const int S = (odd ? sb : sa) + dpp_i32<kDppXor1>(odd ? sa : sb);
                acc[m] = fmaf(dw * dxv, static_cast<float>(S), acc[m]);
            }
            ++cstep;
            const uint32_t done = t + d + 1;   // items consumed so far, repeats included
            if (cstep == nsteps && done <= n_items) {   // wave-uniform
                float tot[M];
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    tot[m] = parity_sum(acc[m]);
                    acc[m] = 0.0f;
                }
                write_pair<M, SILU>(p, resolve_pair<SILU>(p, ps, cpair, row_bytes), lane, tot);
                cstep = 0;
                ++cpair;
            }
            issue(ring[d]);
        }
    }
}

// ---- rows of NSTEPS KiB: the waves of a workgroup share every pair ----------------------------------
// A wave that streams whole rows must hold the activations of the whole row (registers that then
// are not there for loads in flight) or re-read them step by step (as much L1 traffic again as the
// weights).  Here the WAVES waves of a workgroup cut every row into interleaved 1 KiB steps: wave
// w takes steps w, w + WAVES, ... and a 1 / WAVES share of the steps that remain (its first lanes
// only), so each wave needs the activations of its own steps only, once, in registers, for all
// the pairs of the workgroup, and the workgroup as a whole reads each pair as one contiguous
// stretch.  A slot is refilled with the next pair's bytes as soon as it is consumed.  The waves'
// partial sums meet in LDS after the last pair (one barrier per workgroup), added in wave order.
// Measured against one wave per pair with the whole row's activations in registers (batch 1):
// 8192 x 5120 fan-out 9.3 -> 8.7 us, SwiGLU 2 x 17408 x 5120 29.9 -> 28.7 us, 5120 x 5120 6.9 -> 6.6 us;
// against one wave per pair with the activations read per step: 5120 x 17408 18.0 -> 16.7 us.
// XF32 (one fp32 activation row, one step per wave): a wave quantizes the 1024 floats of its step
// itself -- a lane and its neighbour hold one 32-element block -- behind its first weight requests;
// against workgroups of 8..16 waves that quantized the row into LDS and then owned whole pairs:
// SwiGLU with the norm inside 36.3 -> 31.5 us, fan-out 11.4 -> 11.1, 5120 x 6144 9.3 -> 8.4.
constexpr uint32_t kKsplitMaxPairs = 12;   // pairs a workgroup may take (its partial sums wait in LDS)

// Register slots a wave of the shared-row kernel holds: its whole steps plus one for a shared last step.
constexpr int ksplit_slots(int nsteps, int waves) { return nsteps / waves + (nsteps % waves ? 1 : 0); }
// Waves per SIMD the registers are budgeted for: three at batch 2, which also serves the long rows;
// four for the SwiGLU form on rows of four slots and more (five would spill); five otherwise.
constexpr int ksplit_waves_per_simd(int m, int nsteps, int waves, bool silu) {
    return m == 2 ? 3 : (silu && ksplit_slots(nsteps, waves) >= 4) ? 4 : 5;
}

template <int M, int NSTEPS, int WAVES, bool SILU = false, bool XF32 = false, bool NORM = false>
__global__ __launch_bounds__(WAVES * kWave, ksplit_waves_per_simd(M, NSTEPS, WAVES, SILU)) void gemv_pairs_ksplit_kernel(const GemvParams p, const PairSpace ps) {
    constexpr uint32_t nb = NSTEPS * 32;
    constexpr uint64_t row_bytes = static_cast<uint64_t>(nb) * 34;
    constexpr int S = NSTEPS / WAVES;                              // whole steps per wave
    constexpr uint32_t kTail = (NSTEPS - S * WAVES) * 64 / WAVES;  // 16-byte pieces per wave of the steps left over
    static_assert((NSTEPS - S * WAVES) * 64 % WAVES == 0 && kTail % 2 == 0, "the left-over steps split evenly");
    constexpr int SL = S + (kTail ? 1 : 0);                        // register slots per wave
    static_assert(!XF32 || (SL == 1 && kTail == 0), "fp32 activations: one step per wave");
    static_assert(!NORM || (XF32 && M == 1), "the norm applies to one fp32 row");
    __shared__ float part[kKsplitMaxPairs][WAVES][M][2];
    __shared__ float squares[NORM ? WAVES : 1][NORM ? kNormThreads : 1];
    __shared__ float red[4];
    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t w = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const bool odd = lane & 1u;
    const uint32_t first = blockIdx.x * ps.ppw;
    if (first >= ps.pairs) return;
    const uint32_t end = first + ps.ppw < ps.pairs ? first + ps.ppw : ps.pairs;
    // the 16-byte piece of a row this lane owns in slot j, and whether the slot is live in this lane
    auto piece_of = [&](int j) -> uint32_t {
        return j < S ? (static_cast<uint32_t>(j) * WAVES + w) * 64 + lane : static_cast<uint32_t>(S) * WAVES * 64 + w * kTail + lane;
    };
    auto live_in = [&](int j) -> bool { return j < S || lane < kTail; };

    v4i xq[M][SL];
    uint16_t dxh[M][SL];
    Float4 xv[XF32 ? M : 1][XF32 ? 4 : 1], nw[NORM ? 4 : 1];   // XF32: the lane's 16 floats (half a block) of the wave's step
    if constexpr (XF32) {
        const uint32_t at = piece_of(0) * 16;
        // (the norm's entry points demand alignment)
        const bool vec = NORM || (reinterpret_cast<uintptr_t>(p.xf) % 16 == 0 && (M == 1 || p.x_stride % 4 == 0));
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float *src = p.xf + static_cast<uint64_t>(m) * p.x_stride + at + 4 * i;
                xv[m][i] = vec ? load4<true>(src) : load4<false>(src);
                if constexpr (NORM) nw[i] = load4<true>(p.norm_w + at + 4 * i);
            }
        asm volatile("" ::: "memory");   // the activation loads stay ahead of the weight loads
    } else {
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
            for (int j = 0; j < SL; ++j) {
                xq[m][j] = v4i{0, 0, 0, 0};
                dxh[m][j] = 0;
                if (live_in(j)) {
                    const uint32_t piece = piece_of(j);
                    const uint8_t *blk = p.y + static_cast<uint64_t>(m * nb + (piece >> 1)) * kQ81Bytes;
                    xq[m][j] = load_x16(blk + 4 + (piece & 1u) * 16);
                    dxh[m][j] = *reinterpret_cast<const uint16_t *>(blk);
                }
            }
    }
    v4i q0[SL], q1[SL];
    uint16_t d0[SL], d1[SL];
    auto issue = [&](int j, const PairRows &rows) {
        const uint32_t piece = live_in(j) ? piece_of(j) : 0u;   // dead lanes of the tail slot: piece 0, zero activation scale
        q0[j] = load_q16(rows.r0 + 2 * nb + piece * 16);
        q1[j] = load_q16(rows.r1 + 2 * nb + piece * 16);
        d0[j] = reinterpret_cast<const uint16_t *>(rows.r0)[piece >> 1];
        d1[j] = reinterpret_cast<const uint16_t *>(rows.r1)[piece >> 1];
    };
    PairRows rows = resolve_pair<SILU>(p, ps, first, row_bytes);
#pragma unroll
    for (int j = 0; j < SL; ++j) issue(j, rows);
    float dx[M][SL];
    if constexpr (XF32) {
        asm volatile("" ::: "memory");   // ... and the weight loads ahead of the barriers
        if constexpr (NORM) {
            // Sum of squares in the stand-alone norm's order: there thread t adds chunks t, t + 256, ...;
            // here wave u holds chunks 256 u + (0..255), so thread t adds squares[0..WAVES-1][t] ascending.
#pragma unroll
            for (int i = 0; i < 4; ++i) squares[w][lane * 4 + i] = chunk_squares(xv[0][i]);
            __syncthreads();
            float sum_sq;
            if constexpr (WAVES >= 4) {
                float partial = 0.0f;
                if (threadIdx.x < kNormThreads) {
#pragma unroll
                    for (int u = 0; u < WAVES; ++u) partial += squares[u][threadIdx.x];
                }
                sum_sq = first256_tree_sum(partial, red);
            } else {
                // fewer than 256 threads: wave w stands in for the waves w, w + WAVES, ... of that tree
                for (uint32_t g = w; g < 4; g += WAVES) {
                    float partial = 0.0f;
#pragma unroll
                    for (int u = 0; u < WAVES; ++u) partial += squares[u][g * kWave + lane];
                    const float s = wave_sum(partial);
                    if (lane == 0) red[g] = s;
                }
                __syncthreads();
                sum_sq = (red[0] + red[1]) + (red[2] + red[3]);
            }
            const float scale = rms_scale(sum_sq, nb * 32, p.eps);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                xv[0][i] = rms_apply(xv[0][i], scale, nw[i]);
                if (p.normalized != nullptr && blockIdx.x == 0)
                    *reinterpret_cast<float4 *>(p.normalized + piece_of(0) * 16 + 4 * i) = make_float4(xv[0][i].x, xv[0][i].y, xv[0][i].z, xv[0][i].w);
            }
        }
        // Q8_1 of the block this lane shares with its neighbour: the stand-alone quantizer's arithmetic
#pragma unroll
        for (int m = 0; m < M; ++m) {
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                amax = fmaxf(amax, fmaxf(fmaxf(fabsf(xv[m][i].x), fabsf(xv[m][i].y)), fmaxf(fabsf(xv[m][i].z), fabsf(xv[m][i].w))));
            amax = fmaxf(amax, dpp_f32<kDppXor1>(amax));
            const float d = amax / 127.0f;
            int q[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) rint_div4(xv[m][i], d, q[4 * i], q[4 * i + 1], q[4 * i + 2], q[4 * i + 3]);
#pragma unroll
            for (int i = 0; i < 16; ++i) q[i] = amax == 0.0f ? 0 : q[i];
            xq[m][0] = v4i{static_cast<int>(pack4(q[0], q[1], q[2], q[3])), static_cast<int>(pack4(q[4], q[5], q[6], q[7])),
                           static_cast<int>(pack4(q[8], q[9], q[10], q[11])), static_cast<int>(pack4(q[12], q[13], q[14], q[15]))};
            dx[m][0] = half_bits_to_float(float_to_half_bits(d));
        }
    } else {
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
            for (int j = 0; j < SL; ++j) dx[m][j] = half_bits_to_float(dxh[m][j]);
    }

    // one pair: REFILL = its slots are refilled with the next pair's bytes as they are consumed (every
    // pair but the last; a separate copy of the loop body, so that no branch sits between the loads
    // and the compiler's load counters stay exact)
    auto do_pair = [&](uint32_t pair, auto refill_tag) {
        constexpr bool REFILL = decltype(refill_tag)::value;
        PairRows next = rows;
        if constexpr (REFILL) next = resolve_pair<SILU>(p, ps, pair + 1, row_bytes);
        float acc[M];
#pragma unroll
        for (int m = 0; m < M; ++m) acc[m] = 0.0f;
#pragma unroll
        for (int j = 0; j < SL; ++j) {
            const float dw = half_bits_to_float(odd ? d1[j] : d0[j]);
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const int sa = dot16(q0[j], xq[m][j]);
                const int sb = dot16(q1[j], xq[m][j]);
                const int sum = (odd ? sb : sa) + dpp_i32<kDppXor1>(odd ? sa : sb);
                acc[m] = fmaf(dw * dx[m][j], static_cast<float>(sum), acc[m]);
            }
            if constexpr (REFILL) {
                issue(j, next);
                __builtin_amdgcn_sched_barrier(0);   // the refill stays here: the compiler otherwise gathers all refills after the last slot
            }
        }
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const float tot = parity_sum(acc[m]);
            if (lane < 2) part[pair - first][w][m][lane] = tot;
        }
        rows = next;
    };
    for (uint32_t pair = first; pair + 1 < end; ++pair) do_pair(pair, std::true_type{});
    do_pair(end - 1, std::false_type{});
    __syncthreads();
    if constexpr (SILU) {   // the two rows of a pair are a gate row and its up row: one output
        const uint32_t n = (end - first) * M;
        if (threadIdx.x < n) {
            const uint32_t k = threadIdx.x / M, m = threadIdx.x % M;
            float g = 0.0f, u = 0.0f;
#pragma unroll
            for (int v = 0; v < WAVES; ++v) { g += part[k][v][m][0]; u += part[k][v][m][1]; }
            const PairRows out = resolve_pair<true>(p, ps, first + k, row_bytes);
            static_cast<float *>(out.dst)[static_cast<uint64_t>(m) * out.stride + out.row0] = (g / (1.0f + __expf(-g))) * u;
        }
    } else {
        const uint32_t n = (end - first) * M * 2;
        if (threadIdx.x < n) {
            const uint32_t k = threadIdx.x / (2 * M), m = (threadIdx.x / 2) % M, r = threadIdx.x % 2;
            float tot = 0.0f;
#pragma unroll
            for (int v = 0; v < WAVES; ++v) tot += part[k][v][m][r];
            const PairRows out = resolve_pair<false>(p, ps, first + k, row_bytes);
            if (r == 0 || out.two) store_out(p.mode, out.dst, static_cast<uint64_t>(m) * out.stride + out.row0 + r, tot);
        }
    }
}

// ---- host side -----------------------------------------------------------------------------------
PairSpace pair_space(const GemvParams &p, bool silu) {
    PairSpace ps{};
    if (silu) {
        for (int i = 0; i < 4; ++i) ps.pair_end[i] = p.total_rows;
        ps.pairs = p.total_rows;
    } else {
        uint32_t prev = 0, total = 0;
        for (int i = 0; i < 4; ++i) {
            total += (p.row_end[i] - prev + 1) / 2;
            prev = p.row_end[i];
            ps.pair_end[i] = total;
        }
        ps.pairs = total;
    }
    ps.ppw = 1;
    return ps;
}

template <int M, int NSTEPS, int WAVES>
int launch_ksplit(const GemvParams &p, PairSpace ps, hipStream_t stream) {
    // Pairs per workgroup, measured on MI355X.  17 KiB rows (5120 x 17408, batch 1): two 16.9 us, one 17.8,
    // three 18.1, four 17.9.  5 KiB rows at batch 1: SwiGLU (17408 pairs) one 30.1 us, two 28.7, three 30.8,
    // four 29.4; fan-out (4096 pairs) one 8.7, two 9.0, four 9.0.  At batch 2: SwiGLU two 30.8, four 30.2;
    // fan-out two 9.5, four 9.3; 5120 x 6144 (2560 pairs) two 8.0, four 8.2.  At batch 3: SwiGLU four 32.7,
    // eight 32.0; 5120 x 6144 four 9.2, eight 10.8.
    // Rows of three and more steps per wave (15 and 17 KiB): two pairs, or as many as leave exactly two
    // workgroups per CU when the pairs divide that way (5120 x 17408: five pairs 16.3 us against 16.6 at
    // batch 1, 17.0 against 18.2 at batch 2; 4096 x 17408: four pairs 13.6 against 13.9 and 14.3 against 15.4;
    // 5120 x 15360: 15.6 against 15.5 and 16.5 against 17.9).
    if (NSTEPS / WAVES >= 3) {
        const uint32_t two_per_cu = 2u * static_cast<uint32_t>(device_cu_count());
        const uint32_t even = ps.pairs / two_per_cu;
        ps.ppw = (ps.pairs % two_per_cu == 0 && even >= 2 && even <= kKsplitMaxPairs) ? even : 2;
    }
    else if (M == 1) ps.ppw = ps.pairs >= 8192 ? 2 : 1;
    else if (M == 2) ps.ppw = ps.pairs >= 4096 ? 4 : 2;
    else ps.ppw = ps.pairs >= 8192 ? 8 : ps.pairs >= 4096 ? 4 : 2;   // 5120 x 6144 (2560 pairs), two against four: 8.4 / 8.8 us at batch 3, 9.4 / 9.8 at batch 4
    const uint32_t grid = (ps.pairs + ps.ppw - 1) / ps.ppw;
    if (p.mode == kSiluMul) gemv_pairs_ksplit_kernel<M, NSTEPS, WAVES, true><<<grid, WAVES * kWave, 0, stream>>>(p, ps);
    else gemv_pairs_ksplit_kernel<M, NSTEPS, WAVES, false><<<grid, WAVES * kWave, 0, stream>>>(p, ps);
    return check_launch("gemv (row pairs, rows shared by the waves of a workgroup)");
}

// fp32 activations on rows of NSTEPS KiB: every workgroup quantizes (and normalises) the row itself,
// each wave its own step, so a workgroup takes more pairs than with Q8_1 activations.
template <int M, int NSTEPS>
int launch_ksplit_f32(const GemvParams &p, PairSpace ps, hipStream_t stream) {
    // Pairs per workgroup.  Staging costs a workgroup about as much as four pairs, so few, long
    // workgroups: while all of them are resident at once (five waves per SIMD), a whole number per
    // CU with at most four pairs each, or at most eight if four are too few; beyond, the fewest rounds of resident workgroups with an
    // even share each, so that no short last round leaves most of the chip idle.  Measured at 5120
    // columns with the norm inside (pairs: us by pairs per workgroup): 1024: 1 8.0, 2 6.5, 4 6.5,
    // 8 8.4; 2048: 2 9.1, 4 8.0, 8 8.8; 4096: 4 11.1, 8 11.0; 6144: 4 15.8, 6 14.3, 8 13.7; 8192:
    // 4 19.7, 8 17.0; 8704: 4 20.5, 8 20.6, 9 18.2.
    const uint32_t cus = static_cast<uint32_t>(device_cu_count());
    const uint32_t resident = 20 / NSTEPS;   // workgroups per CU
    if (ps.pairs <= cus * resident * 8) {
        const uint32_t target = ps.pairs <= cus * resident * 4 ? 4 : 8;
        const uint32_t per_cu = (ps.pairs + cus * target - 1) / (cus * target);
        ps.ppw = (ps.pairs + cus * per_cu - 1) / (cus * per_cu);
        if (ps.ppw < 2) ps.ppw = 2;
    } else {
        const uint32_t slots = cus * resident;
        const uint32_t rounds = (ps.pairs + slots * kKsplitMaxPairs - 1) / (slots * kKsplitMaxPairs);
        ps.ppw = (ps.pairs + slots * rounds - 1) / (slots * rounds);
    }
    const uint32_t grid = (ps.pairs + ps.ppw - 1) / ps.ppw;
    const bool silu = p.mode == kSiluMul;
    if (p.norm_w != nullptr) {
        if constexpr (M == 1 && NSTEPS <= 6) {
            if (silu) gemv_pairs_ksplit_kernel<1, NSTEPS, NSTEPS, true, true, true><<<grid, NSTEPS * kWave, 0, stream>>>(p, ps);
            else gemv_pairs_ksplit_kernel<1, NSTEPS, NSTEPS, false, true, true><<<grid, NSTEPS * kWave, 0, stream>>>(p, ps);
            return check_launch("gemv (row pairs, fp32 activations, fused norm)");
        } else {
            return Q8MI_REJECTED;
        }
    }
    if (silu) gemv_pairs_ksplit_kernel<M, NSTEPS, NSTEPS, true, true, false><<<grid, NSTEPS * kWave, 0, stream>>>(p, ps);
    else gemv_pairs_ksplit_kernel<M, NSTEPS, NSTEPS, false, true, false><<<grid, NSTEPS * kWave, 0, stream>>>(p, ps);
    return check_launch("gemv (row pairs, fp32 activations)");
}

template <int M>
int launch_ring(const GemvParams &p, PairSpace ps, hipStream_t stream) {
    ps.ppw = 2;   // measured at 17408 columns: 17.4 us against 18.0..18.8 with one pair per wave
    const uint32_t grid = (ps.pairs + ps.ppw - 1) / ps.ppw;
    if (p.mode == kSiluMul) gemv_pairs_ring_kernel<M, true, false><<<grid, kWave, 0, stream>>>(p, ps);
    else gemv_pairs_ring_kernel<M, false, false><<<grid, kWave, 0, stream>>>(p, ps);
    return check_launch("gemv (row pairs, ring)");
}

// Waves per workgroup and pairs per wave of the kernels whose workgroups quantize fp32 activations
// together: one workgroup per CU while a CU's share is at most two pairs for each of max_waves
// waves; beyond that, workgroups of eight waves with two pairs each, handed out by the dispatcher.
void f32_geometry(PairSpace &ps, uint32_t max_waves, uint32_t &waves, uint32_t &grid) {
    const uint32_t cus = static_cast<uint32_t>(device_cu_count());
    const uint32_t share = (ps.pairs + cus - 1) / cus;
    if (share <= 2 * max_waves) {
        // one workgroup per CU: the fewest pairs per wave, then the wave count that wastes no slot
        ps.ppw = (share + max_waves - 1) / max_waves;
        waves = (share + ps.ppw - 1) / ps.ppw;
        if (waves < 4) waves = 4;
    } else {
        waves = 8;
        ps.ppw = 2;
    }
    const uint32_t per_wg = waves * ps.ppw;
    grid = (ps.pairs + per_wg - 1) / per_wg;
}

template <int M>
int launch_ring_f32(const GemvParams &p, PairSpace ps, hipStream_t stream) {
    const uint32_t lds = ring_x_lds_bytes(p.nb, M);
    if (lds > kLdsLimit - 1024)   // rows this long keep their activations in L2 (two-step form)
        return fail(Q8MI_REJECTED, "qgemv: %u activation rows of %u columns do not fit LDS", M, p.nb * 32);
    uint32_t waves, grid;
    f32_geometry(ps, 8, waves, grid);
    auto launch = [&](auto kern) {
        static KernelGeometry geometry;
        if (!geometry.grant(reinterpret_cast<const void *>(kern), kLdsLimit - 1024))
            return fail(Q8MI_LAUNCH_ERROR, "gemv (row pairs): cannot reserve %u bytes of LDS", lds);
        kern<<<grid, waves * kWave, lds, stream>>>(p, ps);
        return check_launch("gemv (row pairs, ring, fp32 activations)");
    };
    if constexpr (M == 1) {
        if (p.norm_w != nullptr) {
            if (p.mode == kSiluMul) return launch(gemv_pairs_ring_kernel<1, true, true, true>);
            return launch(gemv_pairs_ring_kernel<1, false, true, true>);
        }
    }
    if (p.mode == kSiluMul) return launch(gemv_pairs_ring_kernel<M, true, true>);
    return launch(gemv_pairs_ring_kernel<M, false, true>);
}

// Rows that are not a whole number of KiB: one wave per pair at batch 1 and 2 (the ring kernel when
// the launch has row pairs enough to fill the chip that way is the caller's rule), else not ours.
template <int M>
int ring_or_reject(const GemvParams &p, const PairSpace &ps, hipStream_t stream) {
    if constexpr (M <= 2) return launch_ring<M>(p, ps, stream);
    else return Q8MI_REJECTED;
}

// Rows of N KiB, N = 1 .. 17 (the reference's kernel is generic in cols % 32, src/mmvq_q8.cu:193-280;
// here every whole number of KiB has an instantiation of the shared-row kernel), always a split
// without a left-over step except at 17: one wave per 1 KiB step up to 8 KiB and at 9, 11 and 13
// (5120 rows of 1 / 2 / 3 KiB at batch 1: 3.8 / 4.3 / 5.1 us against 4.4 / 4.9 / 6.0 with one wave per
// pair and the activations read per step; 17408 rows of 1 KiB: 5.3 against 9.5); two steps per wave at
// 10, 12, 14 and 16; 15 -> 5 x 3; 17 -> 4 x 4 and a shared last step.  Measured on MI355X at batch 1,
// 5120 rows, time / plain streaming read of the same bytes: 1.08 .. 1.17 on every length (with four
// waves and a shared last step 9, 11 and 13 KiB were at 1.30, 1.22, 1.22; 15 KiB on 15 waves 1.28, on
// 8 waves 1.23; the ring kernel on lengths in between, 5632 and 9728 columns: 1.29, 1.22).
// Q8MI_REJECTED: not a length (or batch) of this kernel.
template <int M>
int ksplit_by_length(const GemvParams &p, const PairSpace &ps, hipStream_t stream) {
    if (p.nb % 32 != 0) return ring_or_reject<M>(p, ps, stream);
    if constexpr (M >= 3) {   // batch 3 and 4: the 2..8 KiB rows only (shorter and longer rows: the matrix-core kernel)
        switch (p.nb / 32) {
            case 2: return launch_ksplit<M, 2, 2>(p, ps, stream);
            case 3: return launch_ksplit<M, 3, 3>(p, ps, stream);
            case 4: return launch_ksplit<M, 4, 4>(p, ps, stream);
            case 5: return launch_ksplit<M, 5, 5>(p, ps, stream);
            case 6: return launch_ksplit<M, 6, 6>(p, ps, stream);
            case 7: return launch_ksplit<M, 7, 7>(p, ps, stream);
            case 8: return launch_ksplit<M, 8, 8>(p, ps, stream);
            default: return Q8MI_REJECTED;
        }
    } else {
        switch (p.nb / 32) {
            case 1: return launch_ksplit<M, 1, 1>(p, ps, stream);
            case 2: return launch_ksplit<M, 2, 2>(p, ps, stream);
            case 3: return launch_ksplit<M, 3, 3>(p, ps, stream);
            case 4: return launch_ksplit<M, 4, 4>(p, ps, stream);
            case 5: return launch_ksplit<M, 5, 5>(p, ps, stream);
            case 6: return launch_ksplit<M, 6, 6>(p, ps, stream);
            case 7: return launch_ksplit<M, 7, 7>(p, ps, stream);
            case 8: return launch_ksplit<M, 8, 8>(p, ps, stream);
            case 9: return launch_ksplit<M, 9, 9>(p, ps, stream);
            case 10: return launch_ksplit<M, 10, 5>(p, ps, stream);
            case 11: return launch_ksplit<M, 11, 11>(p, ps, stream);
            case 12: return launch_ksplit<M, 12, 6>(p, ps, stream);
            case 13: return launch_ksplit<M, 13, 13>(p, ps, stream);
            case 14: return launch_ksplit<M, 14, 7>(p, ps, stream);
            case 15: return launch_ksplit<M, 15, 5>(p, ps, stream);
            case 16: return launch_ksplit<M, 16, 8>(p, ps, stream);
            case 17: return launch_ksplit<M, 17, 4>(p, ps, stream);   // two waves spill, eight: 17.1 us against 16.9
            default: return ring_or_reject<M>(p, ps, stream);
        }
    }
}

}  // namespace

int launch_pairs(const GemvParams &p, uint32_t batch, hipStream_t stream) {
    if (batch == 0 || batch > kPairsMaxBatch || p.nb % 8 != 0) return Q8MI_REJECTED;
    if (p.norm_w != nullptr) {   // fused norm + quantizer: one row, at most kMaxNormCols columns
        constexpr uint32_t kMaxNormCols = 6144;
        if (batch != 1) return fail(Q8MI_REJECTED, "nqgemv: batch %u above 1 (normalise and quantize once, then use the GEMV)", batch);
        if (p.nb * kQK > kMaxNormCols)
            return fail(Q8MI_REJECTED, "nqgemv: rows of %u columns are not served (at most %u)", p.nb * kQK, kMaxNormCols);
        auto al = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
        if (!al(p.xf) || !al(p.norm_w) || (p.normalized != nullptr && !al(p.normalized)))
            return fail(Q8MI_REJECTED, "nqgemv: activations, norm weights and normalised output must be 16-byte aligned");
    }
    const PairSpace ps = pair_space(p, p.mode == kSiluMul);
    if (ps.pairs == 0) return Q8MI_REJECTED;
    const uint32_t cols = p.nb * kQK;
    if (p.xf != nullptr) {
        // The quantizer inside the kernel, batch 1 and 2.  (The shared-row kernel was measured up to
        // batch 4 in this form, fused against quantizer launch + GEMV, us: 8192 x 5120 fan-out batch 1
        // 9.4 / 10.9, batch 2 11.2 / 11.4, batch 3 13.8 / 12.0, batch 4 21.7 / 13.1; SwiGLU batch 2
        // 35.6 / 32.6: every workgroup repeats the quantization, which stops paying at batch 2.)
        auto f32_by_cols = [&](auto mtag) -> int {
            constexpr int M = decltype(mtag)::value;
            switch (cols) {
                case 1024: return launch_ksplit_f32<M, 1>(p, ps, stream);
                case 2048: return launch_ksplit_f32<M, 2>(p, ps, stream);
                case 3072: return launch_ksplit_f32<M, 3>(p, ps, stream);
                case 4096: return launch_ksplit_f32<M, 4>(p, ps, stream);
                case 5120: return launch_ksplit_f32<M, 5>(p, ps, stream);
                case 6144: return launch_ksplit_f32<M, 6>(p, ps, stream);
                case 7168: return launch_ksplit_f32<M, 7>(p, ps, stream);
                case 8192: return launch_ksplit_f32<M, 8>(p, ps, stream);
                default: return launch_ring_f32<M>(p, ps, stream);
            }
        };
        switch (batch) {
            case 1: return f32_by_cols(std::integral_constant<int, 1>{});
            case 2: return f32_by_cols(std::integral_constant<int, 2>{});
            default: return Q8MI_REJECTED;
        }
    }
    if (reinterpret_cast<uintptr_t>(p.y) % 4 != 0) return Q8MI_REJECTED;
    // rows of whole KiB up to 17: shared by the waves of a workgroup, activations in registers
    // (batch 1 and 2 on every such length, batch 3 and 4 on the 2..8 KiB rows measured for them);
    // any other length: one wave per pair, activations read with every step
    switch (batch) {
        case 1: return ksplit_by_length<1>(p, ps, stream);
        case 2: return ksplit_by_length<2>(p, ps, stream);
        case 3: return ksplit_by_length<3>(p, ps, stream);
        case 4: return ksplit_by_length<4>(p, ps, stream);
        default: return Q8MI_REJECTED;
    }
}

}  // namespace q8mi
