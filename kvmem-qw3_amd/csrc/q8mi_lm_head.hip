// Fused LM head for MTP verification on gfx950: Q8_0 GEMV over the vocabulary
// rows + running row-argmax + greedy draft acceptance, without writing the
// batch x vocab logits.
//
// Fuses what the reference runs as q8_0_matmul(W_out) -> argmax_batch -> host
// accept loop (src/qwen_executor.cpp:6779-6821, src/kernels_cuda.cu:20814-20850,
// src/qwen_native_backend.cpp:15948-15960, 16048-16052).
//
// Pass 1 (lm_head_kernel): same weight stream as the GEMV.  A wave keeps, per
// verify row, the best {logit, token} among the vocabulary rows it has
// processed; the workgroup merges its four waves and writes one partial per
// verify row.  Pass 2 (lm_head_finalize_kernel): one workgroup merges the
// partials, writes the per-row winners, then walks the drafts.
// The merge rule is the reference's batched-argmax rule (strictly greater
// wins, equal logits go to the lower token id, src/kernels_cuda.cu:1765-1771),
// which is independent of the order partials are merged in for NaN-free logits.
#include "q8mi_gemv_core.hpp"
#include "q8mi_gemv_mfma_core.hpp"

// Partials of q8mi_lm_head_argmax_accept_static: one {value, index} pair per (verify row, workgroup),
// at most 8 rows x 1024 workgroups = 64 KiB, held by every GPU the library runs on until the process
// ends.  In host code this name is only a handle for hipGetSymbolAddress; kernels get the address.
static __device__ __align__(256) uint8_t scratch[Q8MI_MAX_GEMV_BATCH * 1024 * sizeof(q8mi_argmax_pair)];

namespace q8mi {
namespace {

constexpr uint32_t kMaxPartials = 1024;
static_assert(sizeof(scratch) == Q8MI_MAX_GEMV_BATCH * kMaxPartials * sizeof(q8mi_argmax_pair),
              "the static scratch holds the partials of the largest call");
constexpr int kMaxDrafts = Q8MI_MAX_GEMV_BATCH - 1;

struct Drafts {
    int32_t v[kMaxDrafts];
};

// Whether candidate (ov, oi) replaces (v, i).  Only a value above -inf is a candidate at all (a NaN
// or -inf logit never wins, and a row with no other logits ends as (-inf, -1): the single-row rule
// of the reference's argmax_kernel), so the winner is the largest candidate, the lowest index among
// equals, in whatever order lanes, waves and workgroups meet and merge them.
__device__ __forceinline__ bool beats(float ov, int oi, float v, int i) {
    if (oi < 0 || !(ov > -INFINITY)) return false;
    if (i < 0) return true;
    if (ov > v) return true;
    return ov == v && oi < i;
}

template <int M, int THREADS, int XMODE>
__global__ __launch_bounds__(THREADS) void lm_head_kernel(
        const uint8_t *__restrict__ w, const uint8_t *__restrict__ y, uint32_t rows, uint32_t nb,
        q8mi_argmax_pair *__restrict__ partial, float *__restrict__ logits, uint32_t stride_logits,
        int interleave, uint32_t x_bytes) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int R = RowsPerUnit<M>::value;
    constexpr uint32_t kPerUnit = M * R;
    constexpr uint32_t kWaves = THREADS / kWave;
    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t nsteps = (nb * 2 + 127) / 128;
    const uint64_t row_bytes = static_cast<uint64_t>(nb) * 34;
    const uint32_t units = (rows + R - 1) / R;
    const UnitSeq useq = group_units(units, blockIdx.x, gridDim.x, interleave);
    const uint32_t ucount = useq.count;
    const uint32_t n_items = ucount * nsteps;
    uint32_t i0, i1;
    wave_items(n_items, wave, kWaves, i0, i1);
    float *park_base = reinterpret_cast<float *>(smem + x_bytes);
    float *my_park = park_base + wave * kParkFloats;

    auto rows_of = [&](uint32_t u, RowPtrs<R> &rp) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            uint32_t row = R * u + r;
            row = row < rows - 1 ? row : rows - 1;   // ragged tail: re-read the last row
            rp.p[r] = w + row * row_bytes;
        }
    };
    auto park = [&](uint32_t kk, float total) {
        if (lane < kPerUnit) my_park[kk * kPerUnit + lane] = total;
    };
    const XIn in{y};
    gemv_stream<M, R, THREADS, XMODE>(smem, in, nb, useq, i0, i1, rows_of, park);
    __syncthreads();

    auto total_of = [&](uint32_t k, uint32_t mr) {
        float t = 0.0f;
        for (uint32_t wv = 0; wv < kWaves; ++wv) {
            uint32_t a0, a1;
            wave_items(n_items, wv, kWaves, a0, a1);
            if (a1 <= a0) continue;
            const uint32_t kf = a0 / nsteps, kl = (a1 - 1) / nsteps;
            if (k >= kf && k <= kl) t += park_base[wv * kParkFloats + (k - kf) * kPerUnit + mr];
        }
        return t;
    };

    // per verify row: every thread scans its share of the workgroup's logits (rows in
    // ascending order), then an LDS tree picks the workgroup's winner
    __shared__ float sv[THREADS];
    __shared__ int si[THREADS];
    for (uint32_t m = 0; m < M; ++m) {
        float bv = -INFINITY;
        int bi = -1;
        for (uint32_t e = threadIdx.x; e < ucount * R; e += THREADS) {
            const uint32_t k = e / R, r = e % R;
            const uint32_t row = R * useq.unit(k) + r;
            if (row >= rows) continue;
            const float s = total_of(k, m * R + r);
            if (beats(s, static_cast<int>(row), bv, bi)) { bv = s; bi = static_cast<int>(row); }
            if (logits != nullptr) logits[static_cast<uint64_t>(m) * stride_logits + row] = s;
        }
        sv[threadIdx.x] = bv;
        si[threadIdx.x] = bi;
        __syncthreads();
        for (uint32_t stride = THREADS / 2; stride > 0; stride >>= 1) {
            if (threadIdx.x < stride) {
                const float ov = sv[threadIdx.x + stride];
                const int oi = si[threadIdx.x + stride];
                if (beats(ov, oi, sv[threadIdx.x], si[threadIdx.x])) { sv[threadIdx.x] = ov; si[threadIdx.x] = oi; }
            }
            __syncthreads();
        }
        if (threadIdx.x == 0) {
            q8mi_argmax_pair *p = partial + static_cast<uint64_t>(m) * gridDim.x + blockIdx.x;
            p->value = sv[0];
            p->index = si[0];
        }
        __syncthreads();
    }
}

// Matrix-core variant for 3 or more verify rows (see q8mi_gemv_mfma_core.hpp): same unit and
// item decomposition as the GEMV's matrix-core kernel at the same grid, so the logits are the
// same bits as that GEMV's.
//
// A wave keeps a running (max, lowest index) per activation row for the units it streams from
// their first to their last item: the four chunk sums of such a unit are brought together with
// three lane shuffles and never go to LDS.  Only the units a wave shares with a neighbour (at most
// the first and the last of its range) are parked, two slots per wave, and added up in wave order
// after the stream.  LDS use does not grow with the number of rows, so one workgroup per CU
// covers a vocabulary of any size in a single pass.
// Units per round of the item-wise kernel below: with 512 threads and four (eight) activation rows
// 64 (32) units give every thread two triples to add up per round.  Measured on the 248 320 x 5120
// vocabulary at 2 / 4 / 8 rows: rounds of 32 (16) units 193 / 194 / 205 us, 64 (32) units
// 192 / 192 / 202, 128 (64) units 195 / 195 / 201 .. 207; two items in flight per wave 206 / 206 / 208.
__host__ __device__ constexpr uint32_t lm_head_round_units(int mg) { return mg == 2 ? 32u : 64u; }
constexpr int kLmHeadItemsDepth = 1;   // items a wave keeps in flight in that kernel

template <int MG, int THREADS>
__global__ __launch_bounds__(THREADS) void lm_head_mfma_kernel(
        const uint8_t *__restrict__ w, const uint8_t *__restrict__ y, uint32_t rows, uint32_t nb, uint32_t batch,
        q8mi_argmax_pair *__restrict__ partial, float *__restrict__ logits, uint32_t stride_logits,
        int interleave, uint32_t x_bytes) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr uint32_t MP = 4 * MG;
    constexpr uint32_t kWaves = THREADS / kWave;
    constexpr uint32_t kPerUnit = 4 * kMfmaUnitRows * MP;   // [chunk][row][activation row]
    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t c = lane >> 2, r = lane & 3u;   // after the stream: chunk and fragment row of lanes 0 .. 15
    const uint32_t nitems = (nb + kMfmaItemBlocks - 1) / kMfmaItemBlocks;
    const uint64_t row_bytes = static_cast<uint64_t>(nb) * 34;
    const uint32_t units = (rows + kMfmaUnitRows - 1) / kMfmaUnitRows;
    const UnitSeq useq = group_units(units, blockIdx.x, gridDim.x, interleave);
    const uint32_t ucount = useq.count;
    const uint32_t n_items = ucount * nitems;
    uint32_t i0, i1;
    wave_items(n_items, wave, kWaves, i0, i1);
    float *park_base = reinterpret_cast<float *>(smem + x_bytes);   // [wave][2][kPerUnit]
    float *my_park = park_base + wave * 2 * kPerUnit;
    const uint32_t kf_mine = i0 / nitems;

    // running best of the rows this lane finishes (lanes 0..3: row 4 u + lane of every whole unit)
    float bv[MP];
    int bi[MP];
#pragma unroll
    for (uint32_t m = 0; m < MP; ++m) { bv[m] = -INFINITY; bi[m] = -1; }

    auto row_ptr = [&](uint32_t u) -> const uint8_t * {
        uint32_t row = kMfmaUnitRows * u + r;
        row = row < rows - 1 ? row : rows - 1;
        return w + row * row_bytes;
    };
    auto park = [&](uint32_t kk, auto &acc) {
        const uint32_t k = kf_mine + kk;
        const bool whole = k * nitems >= i0 && (k + 1) * nitems <= i1;   // wave-uniform
        if (whole) {
            const int row = static_cast<int>(kMfmaUnitRows * useq.unit(k) + r);
#pragma unroll
            for (int g = 0; g < MG; ++g) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    // chunk c of fragment row r sits in lane 4 c + r
                    const float e0 = acc[g][v];
                    const float e1 = as_f32(__builtin_amdgcn_ds_bpermute(static_cast<int>((4 + r) * 4), as_i32(e0)));
                    const float e2 = as_f32(__builtin_amdgcn_ds_bpermute(static_cast<int>((8 + r) * 4), as_i32(e0)));
                    const float e3 = as_f32(__builtin_amdgcn_ds_bpermute(static_cast<int>((12 + r) * 4), as_i32(e0)));
                    const float s = 0.0f + (((e0 + e1) + e2) + e3);   // the sum the combine below forms
                    const uint32_t m = 4 * g + v;
                    if (lane < kMfmaUnitRows && static_cast<uint32_t>(row) < rows && m < batch) {
                        if (beats(s, row, bv[m], bi[m])) { bv[m] = s; bi[m] = row; }
                        if (logits != nullptr) logits[static_cast<uint64_t>(m) * stride_logits + row] = s;
                    }
                }
            }
        } else if (lane < 16) {
            float *dst = my_park + (k == kf_mine ? 0 : 1) * kPerUnit + (c * kMfmaUnitRows + r) * MP;
#pragma unroll
            for (int g = 0; g < MG; ++g) {
                float4 v;
                v.x = acc[g][0]; v.y = acc[g][1]; v.z = acc[g][2]; v.w = acc[g][3];
                *reinterpret_cast<float4 *>(dst + 4 * g) = v;
            }
        }
    };
    mfma_stream<MG, THREADS, false, false>(smem, y, nb, batch, 0, useq, i0, i1, row_ptr, park);

    // item ranges of the waves, for the shared units
    __shared__ uint32_t s_i0[kWaves], s_i1[kWaves];
    if (threadIdx.x < kWaves) {
        uint32_t a0, a1;
        wave_items(n_items, threadIdx.x, kWaves, a0, a1);
        s_i0[threadIdx.x] = a0;
        s_i1[threadIdx.x] = a1;
    }
    __syncthreads();
    // Shared units: candidate (wave wv, slot sl, fragment row rr) is handled by thread 8 wv + 4 sl + rr
    // when wave wv holds the unit's first item; the partial sums of every wave that touched the unit
    // are added in wave order, each as ((c0 + c1) + c2) + c3.
    if (threadIdx.x < kWaves * 8) {
        const uint32_t wv = threadIdx.x / 8, sl = (threadIdx.x / 4) % 2, rr = threadIdx.x % 4;
        const uint32_t a0 = s_i0[wv], a1 = s_i1[wv];
        if (a1 > a0) {
            const uint32_t kf = a0 / nitems, kl = (a1 - 1) / nitems;
            const uint32_t k = sl == 0 ? kf : kl;
            const bool whole = k * nitems >= a0 && (k + 1) * nitems <= a1;
            const bool first_holder = k * nitems >= a0;       // the unit's first item is in this wave's range
            if (!whole && first_holder && (sl == 0 || kl != kf)) {
                const uint32_t row = kMfmaUnitRows * useq.unit(k) + rr;
                if (row < rows) {
                    for (uint32_t m = 0; m < batch; ++m) {
                        float t = 0.0f;
                        for (uint32_t w2 = wv; w2 < kWaves; ++w2) {
                            const uint32_t b0 = s_i0[w2], b1 = s_i1[w2];
                            if (b1 <= b0) continue;
                            const uint32_t kf2 = b0 / nitems, kl2 = (b1 - 1) / nitems;
                            if (k < kf2) break;
                            if (k > kl2) continue;
                            const float *e = park_base + (w2 * 2 + (k == kf2 ? 0 : 1)) * kPerUnit + rr * MP + m;
                            t += ((e[0] + e[kMfmaUnitRows * MP]) + e[2 * kMfmaUnitRows * MP]) + e[3 * kMfmaUnitRows * MP];
                        }
                        if (logits != nullptr) logits[static_cast<uint64_t>(m) * stride_logits + row] = t;
                        // fold into this thread's running best (its own, if any, stays valid: lowest index wins ties)
#pragma unroll
                        for (uint32_t mm = 0; mm < MP; ++mm)
                            if (mm == m && beats(t, static_cast<int>(row), bv[mm], bi[mm])) { bv[mm] = t; bi[mm] = static_cast<int>(row); }
                    }
                }
            }
        }
    }

    __shared__ float sv[THREADS];
    __shared__ int si[THREADS];
    for (uint32_t m = 0; m < batch; ++m) {
        float v = -INFINITY;
        int i = -1;
#pragma unroll
        for (uint32_t mm = 0; mm < MP; ++mm)
            if (mm == m) { v = bv[mm]; i = bi[mm]; }
        sv[threadIdx.x] = v;
        si[threadIdx.x] = i;
        __syncthreads();
        for (uint32_t stride = THREADS / 2; stride > 0; stride >>= 1) {
            if (threadIdx.x < stride) {
                const float ov = sv[threadIdx.x + stride];
                const int oi = si[threadIdx.x + stride];
                if (beats(ov, oi, sv[threadIdx.x], si[threadIdx.x])) { sv[threadIdx.x] = ov; si[threadIdx.x] = oi; }
            }
            __syncthreads();
        }
        if (threadIdx.x == 0) {
            q8mi_argmax_pair *p = partial + static_cast<uint64_t>(m) * gridDim.x + blockIdx.x;
            p->value = sv[0];
            p->index = si[0];
        }
        __syncthreads();
    }
}

// The matrix-core variant with the workgroup's items dealt round-robin to its waves (ITEMWISE in
// mfma_stream: the loads in flight are eight neighbouring items, i.e. whole rows, which streams a
// few per cent faster than eight waves each working through a range of its own).  Every item's
// sums are parked, so the units are taken in rounds of lm_head_round_units(): after a wave's last
// item of a round (its next item is already requested) the workgroup meets at a barrier and every
// thread adds up the items of kOut (unit, row, activation row) triples of that round, always for
// the same activation row, and folds them into its running best.  Two park buffers, used in turn,
// let the waves go on with the next round while others still add.  LDS use does not depend on the
// number of rows.
template <int MG, int THREADS, int DEPTH, bool LOGITS>
__global__ __launch_bounds__(THREADS) void lm_head_items_kernel(
        const uint8_t *__restrict__ w, const uint8_t *__restrict__ y, uint32_t rows, uint32_t nb, uint32_t batch,
        q8mi_argmax_pair *__restrict__ partial, float *__restrict__ logits, uint32_t stride_logits,
        int interleave, uint32_t x_bytes) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr uint32_t MP = 4 * MG;
    constexpr uint32_t kWaves = THREADS / kWave;
    constexpr uint32_t kPerItem = kMfmaUnitRows * MP;                  // floats parked per item: [row][activation row]
    constexpr uint32_t kRoundUnits = lm_head_round_units(MG);
    constexpr uint32_t kOut = kRoundUnits * kPerItem / THREADS;        // triples a thread adds up per round
    static_assert(kRoundUnits % kWaves == 0 && kRoundUnits * kPerItem % THREADS == 0 && THREADS % MP == 0, "round geometry");
    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t r = lane & 3u;
    const uint32_t nitems = (nb + kMfmaItemBlocks - 1) / kMfmaItemBlocks;
    const uint64_t row_bytes = static_cast<uint64_t>(nb) * 34;
    const uint32_t units = (rows + kMfmaUnitRows - 1) / kMfmaUnitRows;
    const UnitSeq useq = group_units(units, blockIdx.x, gridDim.x, interleave);
    const uint32_t ucount = useq.count;
    const uint32_t n_items = ucount * nitems;
    const uint32_t round_items = kRoundUnits * nitems;          // a multiple of kWaves
    const uint32_t full_rounds = n_items / round_items;
    const uint32_t per_wave = round_items / kWaves;             // items of a wave per full round
    float *park_base = reinterpret_cast<float *>(smem + x_bytes);   // [2][round_items][kPerItem]

    // this thread's triples of a round: (unit k_mine + j kUnitStep, row rr_mine, activation row m_mine)
    const uint32_t m_mine = threadIdx.x % MP, rr_mine = (threadIdx.x / MP) % kMfmaUnitRows;
    const uint32_t k_mine = threadIdx.x / kPerItem;              // 0 .. THREADS / kPerItem - 1
    constexpr uint32_t kUnitStep = THREADS / kPerItem;
    float bv = -INFINITY;
    int bi = -1;
    // adds up round `round` (its first `count` units) from its park buffer
    auto add_round = [&](uint32_t round, uint32_t count) {
        const float *buf = park_base + static_cast<size_t>(round & 1u) * round_items * kPerItem;
#pragma unroll
        for (uint32_t j = 0; j < kOut; ++j) {
            const uint32_t kl = k_mine + j * kUnitStep;
            if (kl >= count) break;
            const float *e = buf + static_cast<size_t>(kl) * nitems * kPerItem + rr_mine * MP + m_mine;
            float t = 0.0f;
            for (uint32_t part = 0; part < nitems; ++part) t += e[part * kPerItem];
            const uint32_t row = kMfmaUnitRows * useq.unit(round * kRoundUnits + kl) + rr_mine;
            if (row < rows && m_mine < batch) {
                if (beats(t, static_cast<int>(row), bv, bi)) { bv = t; bi = static_cast<int>(row); }
                if constexpr (LOGITS) logits[static_cast<uint64_t>(m_mine) * stride_logits + row] = t;
            }
        }
    };

    auto row_ptr = [&](uint32_t u) -> const uint8_t * {
        uint32_t row = kMfmaUnitRows * u + r;
        row = row < rows - 1 ? row : rows - 1;
        return w + row * row_bytes;
    };
    // the wave's t-th item is item wave + t kWaves of the workgroup; lane (rho, q odd, n) holds the
    // total for row n of the item's unit and activation row (q >> 1) + 2 rho (MG 2) or rho (MG 1)
    auto park = [&](uint32_t t, float total) {
        const uint32_t item = wave + t * kWaves;
        const uint32_t round = t / per_wave;                   // the same for every wave: per_wave items each
        const uint32_t in_round = item - round * round_items;
        const uint32_t rho = lane >> 4, q = (lane >> 2) & 3u, n = lane & 3u;
        const uint32_t m = MG == 2 ? (q >> 1) + 2 * rho : rho;
        if (MG == 2 ? (q & 1u) != 0 : q == 1)
            park_base[(static_cast<size_t>(round & 1u) * round_items + in_round) * kPerItem + n * MP + m] = total;
        if ((t + 1) % per_wave == 0 && round < full_rounds) {  // the wave's last item of a whole round
            __syncthreads();
            add_round(round, kRoundUnits);
        }
    };
    const uint32_t i0 = wave < n_items ? wave : n_items;
    mfma_stream<MG, THREADS, false, false, DEPTH, true, true>(smem, y, nb, batch, 0, useq, i0, n_items, row_ptr, park);
    __syncthreads();
    add_round(full_rounds, ucount - full_rounds * kRoundUnits);   // the units left over

    // every thread holds a best for activation row thread % MP: a tree over the threads of equal row
    __shared__ float sv[THREADS];
    __shared__ int si[THREADS];
    sv[threadIdx.x] = bv;
    si[threadIdx.x] = bi;
    __syncthreads();
    const uint32_t j = threadIdx.x / MP;
    for (uint32_t stride = THREADS / MP / 2; stride > 0; stride >>= 1) {
        if (j < stride) {
            const uint32_t o = threadIdx.x + stride * MP;
            if (beats(sv[o], si[o], sv[threadIdx.x], si[threadIdx.x])) { sv[threadIdx.x] = sv[o]; si[threadIdx.x] = si[o]; }
        }
        __syncthreads();
    }
    if (threadIdx.x < batch) {
        q8mi_argmax_pair *p = partial + static_cast<uint64_t>(threadIdx.x) * gridDim.x + blockIdx.x;
        p->value = sv[threadIdx.x];
        p->index = si[threadIdx.x];
    }
}

// One wave per verify row merges that row's partials (each lane a strided share, then a butterfly
// over the lanes; the merge rule does not depend on the order); thread 0 then walks the drafts.
constexpr int kFinalizeThreads = Q8MI_MAX_GEMV_BATCH * kWave;

__global__ __launch_bounds__(kFinalizeThreads) void lm_head_finalize_kernel(
        const q8mi_argmax_pair *__restrict__ partial, uint32_t nparts, uint32_t batch, Drafts drafts_val,
        const int32_t *__restrict__ drafts_dev, int32_t eos, q8mi_argmax_pair *__restrict__ row_out,
        int32_t *__restrict__ accept_out) {
    __shared__ int tokens[Q8MI_MAX_GEMV_BATCH];
    const uint32_t tid = threadIdx.x, lane = tid % kWave, m = tid / kWave;
    if (m < batch) {   // wave-uniform
        float v = -INFINITY;
        int i = -1;
        for (uint32_t k = lane; k < nparts; k += kWave) {
            const q8mi_argmax_pair p = partial[static_cast<uint64_t>(m) * nparts + k];
            if (beats(p.value, p.index, v, i)) { v = p.value; i = p.index; }
        }
#pragma unroll
        for (int d = kWave / 2; d > 0; d >>= 1) {
            const float ov = __shfl_xor(v, d, kWave);
            const int oi = __shfl_xor(i, d, kWave);
            if (beats(ov, oi, v, i)) { v = ov; i = oi; }
        }
        if (lane == 0) {
            row_out[m].value = v;
            row_out[m].index = i;
            tokens[m] = i;
        }
    }
    __syncthreads();
    if (tid == 0) {
        const uint32_t n_drafts = batch - 1;
        uint32_t accepted = 0;
        for (uint32_t i = 0; i < n_drafts; ++i) {
            const int32_t target = tokens[i] >= 0 ? tokens[i] : eos;
            const int32_t draft = drafts_dev != nullptr ? drafts_dev[i] : drafts_val.v[i];
            if (target != draft) break;
            ++accepted;
        }
        const int32_t next = tokens[accepted] >= 0 ? tokens[accepted] : eos;
        accept_out[0] = static_cast<int32_t>(accepted);
        accept_out[1] = next;
    }
}

template <int M, int THREADS, int XMODE>
int launch_inst(const uint8_t *w, const uint8_t *y, uint32_t rows, uint32_t nb, uint32_t x_bytes,
                q8mi_argmax_pair *partial, float *logits, uint32_t stride_logits, uint32_t *grid_out,
                hipStream_t stream) {
    auto kern = lm_head_kernel<M, THREADS, XMODE>;
    const uint32_t lds = x_bytes + (THREADS / kWave) * kParkFloats * 4;
    static KernelGeometry geometry;
    constexpr uint32_t kDynLimit = kLdsLimit - THREADS * 8;   // static LDS: the argmax tree
    if (lds > kDynLimit || !geometry.grant(reinterpret_cast<const void *>(kern), kDynLimit))
        return fail(Q8MI_LAUNCH_ERROR, "lm_head: cannot reserve %u bytes of LDS", lds);
    const uint32_t cus = static_cast<uint32_t>(device_cu_count());
    const uint32_t units = (rows + RowsPerUnit<M>::value - 1) / RowsPerUnit<M>::value;
    uint32_t max_per_cu = geometry.workgroups_per_cu(kern, THREADS, lds);
    if (max_per_cu > kGemvWgsPerCu) max_per_cu = kGemvWgsPerCu;
    while (max_per_cu > 1 && cus * max_per_cu > kMaxPartials) --max_per_cu;   // one partial per workgroup
    const uint32_t grid = pick_grid(units, (nb * 2 + 127) / 128, M, THREADS / kWave, cus, max_per_cu);
    if (grid > kMaxPartials)
        return fail(Q8MI_REJECTED, "lm_head: %u rows need %u workgroups, more than the %u partials", rows, grid,
                    kMaxPartials);
    *grid_out = grid;
    kern<<<grid, THREADS, lds, stream>>>(w, y, rows, nb, partial, logits, stride_logits, kGemvInterleave, x_bytes);
    return check_launch("lm_head");
}

template <int MG>
int launch_lm_head_mfma(const uint8_t *w, const uint8_t *y, uint32_t rows, uint32_t nb, uint32_t batch,
                        q8mi_argmax_pair *partial, float *logits, uint32_t stride_logits, uint32_t *grid_out,
                        hipStream_t stream) {
    constexpr int THREADS = 512;
    const uint32_t cus = static_cast<uint32_t>(device_cu_count());
    const uint32_t units = (rows + kMfmaUnitRows - 1) / kMfmaUnitRows;
    if constexpr (MG <= 2) {   // items dealt round-robin to the waves, units in rounds
        const uint32_t x_bytes = mfma_x_lds_bytes(nb, batch, MG);
        const uint32_t nitems = (nb + kMfmaItemBlocks - 1) / kMfmaItemBlocks;
        const uint64_t park = 2ull * lm_head_round_units(MG) * nitems * kMfmaUnitRows * 4 * MG * 4;
        constexpr uint32_t kDynLimit = kLdsLimit - THREADS * 8 - 256;   // static LDS: the argmax tree
        if (x_bytes + park <= kDynLimit) {
            auto kern = logits != nullptr ? lm_head_items_kernel<MG, THREADS, kLmHeadItemsDepth, true>
                                          : lm_head_items_kernel<MG, THREADS, kLmHeadItemsDepth, false>;
            static KernelGeometry geometry[2];
            if (!geometry[logits != nullptr].grant(reinterpret_cast<const void *>(kern), kDynLimit))
                return fail(Q8MI_LAUNCH_ERROR, "lm_head: cannot reserve %u bytes of LDS", kDynLimit);
            uint32_t grid = cus < units ? cus : units;
            if (grid > kMaxPartials) grid = kMaxPartials;
            *grid_out = grid;
            kern<<<grid, THREADS, x_bytes + static_cast<uint32_t>(park), stream>>>(w, y, rows, nb, batch, partial, logits,
                                                                                  stride_logits, kGemvInterleave, x_bytes);
            return check_launch("lm_head");
        }
    }
    auto kern = lm_head_mfma_kernel<MG, THREADS>;
    // One workgroup per CU, the geometry of the GEMV's matrix-core launch; the kernel parks only the
    // units its waves share (two slots per wave), so the LDS need does not depend on the row count.
    const uint32_t x_bytes = mfma_x_lds_bytes(nb, batch, MG);
    constexpr uint32_t kDynLimit = kLdsLimit - THREADS * 8 - 256;   // static LDS: the argmax tree and a few words
    uint32_t grid = cus < units ? cus : units;
    if (grid > kMaxPartials) grid = kMaxPartials;
    const uint32_t lds = x_bytes + (THREADS / kWave) * 2 * mfma_park_floats_per_unit(MG) * 4;
    if (lds > kDynLimit) return fail(Q8MI_REJECTED, "lm_head (matrix-core variant): the activations do not fit LDS");
    static KernelGeometry geometry;
    if (!geometry.grant(reinterpret_cast<const void *>(kern), kDynLimit))
        return fail(Q8MI_LAUNCH_ERROR, "lm_head: cannot reserve %u bytes of LDS", lds);
    *grid_out = grid;
    kern<<<grid, THREADS, lds, stream>>>(w, y, rows, nb, batch, partial, logits, stride_logits,
                                         kGemvInterleave, x_bytes);
    return check_launch("lm_head");
}

// Which variant streams the weight: the matrix-core one from 2 verify rows on, whenever the
// activations fit LDS beside the parked sums.  Measured on the 248 320-row vocabulary, dot-product
// against matrix-core variant (items dealt round-robin, units in rounds): 197 / 198 us at 1 row,
// 206 / 194 at 2, 216 / 195 at 4, 234 / 201 at 6, 296 / 201 at 8.
bool lm_head_uses_mfma(uint32_t rows, uint32_t nb, uint32_t batch) {
    (void)rows;
    const uint32_t mg = (batch + 3) / 4;
    if (batch < 2) return false;
    return mfma_x_lds_bytes(nb, batch, mg) + 16u * 1024u <= kLdsLimit - 256;
}

template <int M>
int launch_lm_head(const uint8_t *w, const uint8_t *y, uint32_t rows, uint32_t nb, q8mi_argmax_pair *partial,
                   float *logits, uint32_t stride_logits, uint32_t *grid_out, hipStream_t stream) {
    const uint32_t xb = x_lds_bytes(nb, M);
    const uint32_t park_256 = 4 * kParkFloats * 4, park_1024 = 16 * kParkFloats * 4;
    const uint32_t tree_256 = 256 * 8, tree_1024 = 1024 * 8;   // static LDS of the argmax tree
    if (reinterpret_cast<uintptr_t>(y) % 16 != 0)   // the LDS staging loads 16 bytes at a time
        return launch_inst<M, 256, kXGlobal>(w, y, rows, nb, 0, partial, logits, stride_logits, grid_out, stream);
    if (xb + park_256 + tree_256 <= 76u * 1024u)
        return launch_inst<M, 256, kXLds>(w, y, rows, nb, xb, partial, logits, stride_logits, grid_out, stream);
    if (xb + park_1024 + tree_1024 <= kLdsLimit)
        return launch_inst<M, 1024, kXLds>(w, y, rows, nb, xb, partial, logits, stride_logits, grid_out, stream);
    return launch_inst<M, 256, kXGlobal>(w, y, rows, nb, 0, partial, logits, stride_logits, grid_out, stream);
}

}  // namespace
}  // namespace q8mi

using namespace q8mi;

extern "C" size_t q8mi_lm_head_scratch_bytes(uint32_t rows, uint32_t cols, uint32_t batch) {
    (void)rows;
    (void)cols;
    // one partial per workgroup and verify row; the grid never exceeds kMaxPartials
    return static_cast<size_t>(batch) * kMaxPartials * sizeof(q8mi_argmax_pair);
}

static int lm_head_run(const uint8_t *weight, const void *y, uint32_t rows, uint32_t cols, uint32_t batch,
                       const int32_t *drafts, int drafts_on_device, int32_t eos, q8mi_argmax_pair *row_out,
                       int32_t *accept_out, float *logits, uint32_t stride_logits, q8mi_argmax_pair *partial,
                       void *stream) {
    const uint32_t nb = cols / kQK;
    uint32_t grid = 0;
    const auto *yb = static_cast<const uint8_t *>(y);
    hipStream_t s = as_stream(stream);
    int rc = Q8MI_REJECTED;
    if (reinterpret_cast<uintptr_t>(yb) % 4 == 0 && lm_head_uses_mfma(rows, nb, batch)) {
        rc = batch <= 4 ? launch_lm_head_mfma<1>(weight, yb, rows, nb, batch, partial, logits, stride_logits, &grid, s)
                        : launch_lm_head_mfma<2>(weight, yb, rows, nb, batch, partial, logits, stride_logits, &grid, s);
    }
    // very tall weights park more partial sums per workgroup than LDS holds: dot-product variant
    if (rc == Q8MI_REJECTED) switch (batch) {
        case 1: rc = launch_lm_head<1>(weight, yb, rows, nb, partial, logits, stride_logits, &grid, s); break;
        case 2: rc = launch_lm_head<2>(weight, yb, rows, nb, partial, logits, stride_logits, &grid, s); break;
        case 3: rc = launch_lm_head<3>(weight, yb, rows, nb, partial, logits, stride_logits, &grid, s); break;
        case 4: rc = launch_lm_head<4>(weight, yb, rows, nb, partial, logits, stride_logits, &grid, s); break;
        case 5: rc = launch_lm_head<5>(weight, yb, rows, nb, partial, logits, stride_logits, &grid, s); break;
        case 6: rc = launch_lm_head<6>(weight, yb, rows, nb, partial, logits, stride_logits, &grid, s); break;
        case 7: rc = launch_lm_head<7>(weight, yb, rows, nb, partial, logits, stride_logits, &grid, s); break;
        case 8: rc = launch_lm_head<8>(weight, yb, rows, nb, partial, logits, stride_logits, &grid, s); break;
        default: break;
    }
    if (rc != Q8MI_OK) return rc;
    Drafts dv{};
    const int32_t *ddev = nullptr;
    if (batch > 1) {
        if (drafts_on_device) {
            ddev = drafts;
        } else {
            for (uint32_t i = 0; i + 1 < batch; ++i) dv.v[i] = drafts[i];
        }
    }
    lm_head_finalize_kernel<<<1, kFinalizeThreads, 0, s>>>(partial, grid, batch, dv, ddev, eos, row_out, accept_out);
    return check_launch("lm_head finalize");
}

static int lm_head_gate(const uint8_t *weight, uint32_t rows, uint32_t cols, uint32_t batch, const int32_t *drafts) {
    if (cols % kQK != 0 || cols == 0)
        return fail(Q8MI_REJECTED, "lm_head: cols %u not a positive multiple of 32", cols);
    if ((cols / kQK) % 8 != 0)
        return fail(Q8MI_REJECTED, "lm_head: cols %u not a multiple of 256 (unaligned planes)", cols);
    if (batch == 0 || batch > Q8MI_MAX_GEMV_BATCH)
        return fail(Q8MI_REJECTED, "lm_head: batch %u outside 1..8", batch);
    if (rows == 0 || rows > 0x7fffffffu) return fail(Q8MI_REJECTED, "lm_head: rows %u out of range", rows);
    if (batch > 1 && drafts == nullptr) return fail(Q8MI_REJECTED, "lm_head: drafts missing");
    if (reinterpret_cast<uintptr_t>(weight) % 16 != 0)
        return fail(Q8MI_REJECTED, "lm_head: weight pointer not 16-byte aligned");
    return Q8MI_OK;
}

extern "C" int q8mi_lm_head_argmax_accept(const uint8_t *weight, const void *y, uint32_t rows,
                                          uint32_t cols, uint32_t batch, const int32_t *drafts,
                                          int drafts_on_device, int32_t eos, q8mi_argmax_pair *row_out,
                                          int32_t *accept_out, float *logits, uint32_t stride_logits,
                                          void *scratch_arg, void *stream) {
    if (int rc = lm_head_gate(weight, rows, cols, batch, drafts)) return rc;
    return lm_head_run(weight, y, rows, cols, batch, drafts, drafts_on_device, eos, row_out, accept_out, logits,
                       stride_logits, static_cast<q8mi_argmax_pair *>(scratch_arg), stream);
}

// Address of this device's copy of the static scratch array: looked up once per device, with that
// device current (every GPU holds its own copy at its own address).
static int static_scratch_of_current_device(void **out) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void *ptr_of[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return fail(Q8MI_LAUNCH_ERROR, "lm_head (static scratch): no current device, or a device id beyond %d", kMaxDevices - 1);
    }
    std::lock_guard<std::mutex> lock(mu);
    if (ptr_of[dev] == nullptr) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr) {
            (void)hipGetLastError();
            return fail(Q8MI_LAUNCH_ERROR, "lm_head (static scratch): hipGetSymbolAddress: %s", hipGetErrorString(e));
        }
        ptr_of[dev] = p;
    }
    *out = ptr_of[dev];
    return Q8MI_OK;
}

extern "C" int q8mi_lm_head_argmax_accept_static(const uint8_t *weight, const void *y, uint32_t rows, uint32_t cols,
                                                 uint32_t batch, const int32_t *drafts, int drafts_on_device,
                                                 int32_t eos, q8mi_argmax_pair *row_out, int32_t *accept_out,
                                                 float *logits, uint32_t stride_logits, void *stream) {
    if (int rc = lm_head_gate(weight, rows, cols, batch, drafts)) return rc;
    if (q8mi_lm_head_scratch_bytes(rows, cols, batch) > sizeof(scratch))
        return fail(Q8MI_REJECTED, "lm_head (static scratch): %zu bytes of partials needed, the library holds %zu",
                    q8mi_lm_head_scratch_bytes(rows, cols, batch), sizeof(scratch));
    void *partials = nullptr;
    if (int rc = static_scratch_of_current_device(&partials)) return rc;
    // nothing in the array has to start at zero: the finalize kernel reads only the partials
    // [row][0 .. grid) that the stream kernel of the same call has just written
    return lm_head_run(weight, y, rows, cols, batch, drafts, drafts_on_device, eos, row_out, accept_out, logits,
                       stride_logits, static_cast<q8mi_argmax_pair *>(partials), stream);
}
