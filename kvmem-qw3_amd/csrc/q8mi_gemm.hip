// Prefill GEMM: Q8_0 weights x D4-quantized activations on the gfx950 int8
// matrix cores (v_mfma_i32_32x32x32_i8; K = 32 is exactly one Q8 block, so each
// instruction yields the int32 dot of one block for a 32 x 32 patch of outputs).
// Reference semantics: src/mmq_q8.cu:2164-2273 — one int32 sum per 32-block,
// rescaled by d_w * d_y in fp32 and accumulated in ascending block order.
//
// Tiling
//   workgroup  128 weight rows x 128 activation rows (batch), 4 waves
//   wave       32 activation rows x 128 weight rows = four 32x32 MFMA patches
//   K step     one 128-element super-block (4 Q8 blocks), double-buffered in LDS
// The MFMA "A" operand is the activation patch and "B" the weight patch, so a
// lane owns ONE weight row (lane % 32) and 16 activation rows per patch.  That
// makes the fp16 weight scale a per-lane constant and the output stores
// contiguous along the weight-row axis (dst is [batch][rows]).
//
// Two staging variants share the tiling and the arithmetic.  Rows whose int8 plane is
// 16-byte aligned (cols/32 a multiple of 8: every model shape) use direct global->LDS
// loads, described where that kernel is defined; other rows use the register-staged
// kernel below, whose LDS layout is:
//
// LDS record (144 B, both operands): [4 x fp32 scales][128 x int8].  The 144-B
// pitch is what the D4 activation blocks already have in memory, and it spreads
// the 16-byte fragment reads of 8 consecutive rows over all banks.  Activation
// scales are kept a second time, transposed ([sub-block][row]), so a lane can
// fetch the four scales of four consecutive activation rows with one 16-B read.
//
// Rescale without an int->float conversion: the MFMA accumulator is seeded with
// the bit pattern of 1.5*2^23, so the int32 result reinterpreted as fp32 is
// F = 12582912 + S exactly (|S| <= 516128 < 2^22).  g = fma(F, d_w, -12582912*d_w)
// is then the correctly rounded d_w*S (12582912*d_w is exact: d_w has 11
// significant bits), and acc = fma(g, d_y, acc): two FMAs per (output, block).
#include <atomic>

#include "q8mi_device.hpp"
#include "q8mi_internal.hpp"

namespace q8mi {

// GEMV-based route for shapes the MFMA tile does not cover (defined in
// q8mi_gemv.hip): y is Q8_1, any batch, processed eight activation rows at a time.
int gemv_any_batch(const uint8_t *w, const void *y_q8_1, float *dst, uint32_t rows, uint32_t cols,
                   uint32_t batch, uint32_t stride_dst_row, hipStream_t stream);
// Matrix-core GEMV on D4 activations (q8mi_gemv.hip): small batches, else Q8MI_REJECTED.
// w_up != nullptr: the SwiGLU form (dst = silu(w x) * (w_up x)); add: dst += w x instead of a store.
int gemv_mfma_d4(const uint8_t *w, const uint8_t *w_up, const void *y_d4, float *dst, uint32_t rows, uint32_t cols,
                 uint32_t batch, uint32_t stride_dst_row, bool add, hipStream_t stream);

namespace {

constexpr int kTileRows = 128;   // weight rows per workgroup
constexpr int kTileCols = 128;   // activation rows (batch) per workgroup
constexpr int kGemmThreads = 256;
constexpr int kRec = 144;        // LDS record pitch in bytes
constexpr int kStageBytes = kTileRows * kRec + kTileCols * kRec + 4 * kTileCols * 4;  // 38912
constexpr int kLdsBytes = 2 * kStageBytes;                                             // 77824
constexpr uint32_t kMagicBits = 0x4B400000u;  // 1.5 * 2^23
constexpr float kMagic = 12582912.0f;

// What a tile does with its sums.  Store / bf16 store / residual add differ only after the K loop
// and are a wave-uniform run-time switch there; the SwiGLU form stages the rows of two weights
// and is a template parameter of the kernels (SILU).
enum : uint32_t {
    kEpiStore = 0,       // dst[j][r] = sum                              (fp32)
    kEpiStoreBf16 = 1,   // dst[j][r] = bf16(sum), round to nearest even (what f32_to_bf16 would store)
    kEpiAdd = 2,         // dst[j][r] = residual[j][r] + sum             (fp32; residual may be dst)
};
struct TileOut {
    void *dst;
    const float *residual;   // kEpiAdd only; rows stride_dst apart like dst
    uint32_t stride_dst;
    uint32_t epi;
};

__device__ __forceinline__ void emit(const TileOut &o, uint64_t idx, float v) {
    if (o.epi == kEpiStoreBf16) static_cast<uint16_t *>(o.dst)[idx] = float_to_bf16_bits(v);
    else if (o.epi == kEpiAdd) static_cast<float *>(o.dst)[idx] = o.residual[idx] + v;
    else static_cast<float *>(o.dst)[idx] = v;
}
__device__ __forceinline__ float silu_mul(float g, float u) { return (g / (1.0f + __expf(-g))) * u; }

struct Prefetch {
    v4i wq[4];   // 4 x 16 B of weight quants
    uint2 wd;    // 4 fp16 weight scales (threads 0..127)
    v4i yq[5];   // up to 5 x 16 B of activation records
};

// 16 bytes from an address that is 16-byte aligned (A16) or only 8-byte aligned
// (rows of cols/32 % 8 == 4 start on an odd multiple of 8).
template <bool A16>
__device__ __forceinline__ v4i load16(const uint8_t *p) {
    if (A16) return *reinterpret_cast<const v4i *>(p);
    const uint2 lo = *reinterpret_cast<const uint2 *>(p);
    const uint2 hi = *reinterpret_cast<const uint2 *>(p + 8);
    v4i v;
    v.x = static_cast<int>(lo.x); v.y = static_cast<int>(lo.y);
    v.z = static_cast<int>(hi.x); v.w = static_cast<int>(hi.y);
    return v;
}

template <bool CHECK, bool A16>
__device__ __forceinline__ void prefetch_load(Prefetch &pf, const uint8_t *__restrict__ w,
                                              const uint8_t *__restrict__ y, uint32_t rows, uint32_t nb,
                                              uint32_t batch, uint32_t row0, uint32_t col0, uint32_t sb,
                                              uint32_t tid) {
    const uint64_t row_bytes = static_cast<uint64_t>(nb) * 34;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const uint32_t c = tid + kGemmThreads * p;
        const uint32_t r = c >> 3, piece = c & 7u;
        v4i v = {0, 0, 0, 0};
        if (!CHECK || row0 + r < rows) {
            v = load16<A16>(w + (row0 + r) * row_bytes + 2 * nb + sb * 128 + piece * 16);
        }
        pf.wq[p] = v;
    }
    pf.wd = make_uint2(0u, 0u);
    if (tid < kTileRows && (!CHECK || row0 + tid < rows)) {
        pf.wd = *reinterpret_cast<const uint2 *>(w + (row0 + tid) * row_bytes + sb * 8);
    }
    const uint8_t *ysrc = y + (static_cast<uint64_t>(sb) * batch + col0) * kRec;
#pragma unroll
    for (int p = 0; p < 5; ++p) {
        const uint32_t c = tid + kGemmThreads * p;
        v4i v = {0, 0, 0, 0};
        if (c < kTileCols * 9 && (!CHECK || col0 + c / 9 < batch)) {
            v = *reinterpret_cast<const v4i *>(ysrc + static_cast<uint64_t>(c) * 16);
        }
        pf.yq[p] = v;
    }
}

__device__ __forceinline__ void prefetch_store(const Prefetch &pf, uint8_t *stage, uint32_t tid) {
    uint8_t *lw = stage;
    uint8_t *ly = stage + kTileRows * kRec;
    float *ysc = reinterpret_cast<float *>(stage + kTileRows * kRec + kTileCols * kRec);
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const uint32_t c = tid + kGemmThreads * p;
        const uint32_t r = c >> 3, piece = c & 7u;
        *reinterpret_cast<v4i *>(lw + r * kRec + 16 + piece * 16) = pf.wq[p];
    }
    if (tid < kTileRows) {
        float4 d;
        d.x = half_bits_to_float(static_cast<uint16_t>(pf.wd.x & 0xffffu));
        d.y = half_bits_to_float(static_cast<uint16_t>(pf.wd.x >> 16));
        d.z = half_bits_to_float(static_cast<uint16_t>(pf.wd.y & 0xffffu));
        d.w = half_bits_to_float(static_cast<uint16_t>(pf.wd.y >> 16));
        *reinterpret_cast<float4 *>(lw + tid * kRec) = d;
    }
#pragma unroll
    for (int p = 0; p < 5; ++p) {
        const uint32_t c = tid + kGemmThreads * p;
        if (c < kTileCols * 9) {
            *reinterpret_cast<v4i *>(ly + c * 16) = pf.yq[p];
            if (c % 9 == 0) {  // record header: the four fp32 scales, also kept transposed
                const uint32_t j = c / 9;
                ysc[0 * kTileCols + j] = as_f32(pf.yq[p].x);
                ysc[1 * kTileCols + j] = as_f32(pf.yq[p].y);
                ysc[2 * kTileCols + j] = as_f32(pf.yq[p].z);
                ysc[3 * kTileCols + j] = as_f32(pf.yq[p].w);
            }
        }
    }
}

template <bool CHECK, bool A16>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_d4_kernel(
        const uint8_t *__restrict__ w, const uint8_t *__restrict__ y, float *__restrict__ dst,
        uint32_t rows, uint32_t nb, uint32_t batch, uint32_t stride_dst, uint32_t row_tiles,
        uint32_t col_tiles) {
    extern __shared__ __align__(16) uint8_t smem[];
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid % kWave;
    const uint32_t wave = tid / kWave;
    const uint32_t l32 = lane & 31u, lhalf = lane >> 5;

    // Tile order: consecutive workgroup ids land on different XCDs (8 of them,
    // each with its own L2).  Give every XCD whole row tiles, and walk the
    // column tiles of one row tile back to back so its weights stay in that L2.
    const uint32_t id = blockIdx.x;
    const uint32_t xcd = id % 8u, seq = id / 8u;
    const uint32_t rt_local = seq / col_tiles, ct = seq % col_tiles;
    const uint32_t rt = rt_local * 8u + xcd;
    if (rt >= row_tiles) return;  // uniform for the workgroup
    const uint32_t row0 = rt * kTileRows, col0 = ct * kTileCols;

    const uint32_t nsb = nb / 4;
    v16i zero_c;
#pragma unroll
    for (int i = 0; i < 16; ++i) zero_c[i] = static_cast<int>(kMagicBits);

    float acc[4][16];
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[rb][v] = 0.0f;

    Prefetch pf;
    prefetch_load<CHECK, A16>(pf, w, y, rows, nb, batch, row0, col0, 0, tid);
    prefetch_store(pf, smem, tid);
    __syncthreads();

    for (uint32_t sb = 0; sb < nsb; ++sb) {
        uint8_t *cur = smem + (sb & 1u) * kStageBytes;
        uint8_t *nxt = smem + ((sb + 1u) & 1u) * kStageBytes;
        const bool more = sb + 1 < nsb;
        if (more) prefetch_load<CHECK, A16>(pf, w, y, rows, nb, batch, row0, col0, sb + 1, tid);

        const uint8_t *lw = cur;
        const uint8_t *ly = cur + kTileRows * kRec;
        const float *ysc = reinterpret_cast<const float *>(cur + kTileRows * kRec + kTileCols * kRec);

        // one Q8 block (K = 32) per trip; kept rolled so that only the four
        // 32x32 result patches of one block are live at a time
#pragma unroll 1
        for (uint32_t sub = 0; sub < 4; ++sub) {
            const uint32_t frag_off = 16 + sub * 32 + lhalf * 16;
            const v4i a = *reinterpret_cast<const v4i *>(ly + (wave * 32 + l32) * kRec + frag_off);
            float dy[16];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 t = *reinterpret_cast<const float4 *>(
                    ysc + sub * kTileCols + wave * 32 + 8 * g + 4 * lhalf);
                dy[4 * g + 0] = t.x; dy[4 * g + 1] = t.y; dy[4 * g + 2] = t.z; dy[4 * g + 3] = t.w;
            }
            v16i r[4];
            float dw[4];
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
                const uint8_t *rec = lw + (rb * 32 + l32) * kRec;
                const v4i b = *reinterpret_cast<const v4i *>(rec + frag_off);
                dw[rb] = *reinterpret_cast<const float *>(rec + sub * 4);
                r[rb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, zero_c, 0, 0, 0);
            }
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
                const float cw = -kMagic * dw[rb];
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float g = fmaf(as_f32(r[rb][v]), dw[rb], cw);
                    acc[rb][v] = fmaf(g, dy[v], acc[rb][v]);
                }
            }
        }

        if (more) prefetch_store(pf, nxt, tid);
        __syncthreads();
    }

    // D[i][n]: n = lane % 32 (weight row), i = 8*(v/4) + 4*(lane/32) + v%4 (activation row)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
        const uint32_t r = row0 + rb * 32 + l32;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t j = col0 + wave * 32 + 8 * (v / 4) + 4 * lhalf + (v % 4);
            if (!CHECK || (r < rows && j < batch)) {
                dst[static_cast<uint64_t>(j) * stride_dst + r] = acc[rb][v];
            }
        }
    }
}


// ---- direct-to-LDS variant (rows whose int8 plane is 16-byte aligned) ----------------------
// Workgroup tile: 32*RB weight rows x 128 activation rows.  Only RB = 4, the main tile, is
// launched (problems too small to fill the chip with main tiles go to the ring-staged tiles below).
// Stage layout (two stages; TR = 32*RB):
//   weight quants      TR rows x 128 B; 16-byte piece p of row r sits in slot p ^ swz(r), so equal
//                      pieces of 8 or 16 consecutive rows fall on distinct banks
//   activation records exactly as in memory (128 x 144 B: 16 B scales + 128 B quants)
//   weight scales      fp32, [sub-block][row]
//   activation scales  fp32, [sub-block][row]
// Quants travel global -> LDS without passing through registers (global_load_lds_dwordx4: lane l of
// a wave writes 16 bytes at M0 + 16 l); only the scales go through registers.  All per-lane
// offsets are constant over the K loop and the per-step bases are scalar, so staging costs about
// ten instructions per wave and step.
template <int RB>
struct DmaTile {
    static constexpr int kRows = 32 * RB;
    static constexpr int kWq = kRows * 128;
    static constexpr int kOffYr = kWq;
    static constexpr int kOffWsc = kOffYr + kTileCols * kRec;
    static constexpr int kOffYsc = kOffWsc + 4 * kRows * 4;
    static constexpr int kStage = kOffYsc + 4 * kTileCols * 4;
    static constexpr int kLds = 2 * kStage;
};
static_assert(DmaTile<4>::kStage == kStageBytes, "main tile: same LDS budget as the register-staged kernel");

using lptr = __attribute__((address_space(3))) void *;

// 16 bytes per lane from global memory (scalar base + 32-bit lane offset) straight into LDS at
// lds_off + lane * 16.  Issued as inline assembly so that the compiler's wait-count pass does not
// make every later LDS read wait for it; completion is awaited explicitly (vmcnt(0)) before the
// barrier that publishes the stage.
__device__ __forceinline__ void dma16(const uint8_t *uniform_base, uint32_t lane_off, uint32_t lds_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_off), "v"(lane_off), "s"(uniform_base) : "memory", "m0");
}
__device__ __forceinline__ uint32_t lds_offset_of(const void *p) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lptr)p));
}
__device__ __forceinline__ const uint8_t *uniform_ptr(const uint8_t *p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return reinterpret_cast<const uint8_t *>((static_cast<uint64_t>(hi) << 32) | lo);
}

__device__ __forceinline__ uint32_t swz(uint32_t row) { return (row & 7u) ^ ((row >> 3) & 1u); }

typedef unsigned v2u __attribute__((ext_vector_type(2)));
struct Scales { v2u wd; v4i yd; };

// Per-lane byte offsets that do not change over the K loop.
template <int RB>
struct LaneOffsets {
    uint32_t wq[RB];  // weight quant chunk i of this wave, relative to the tile's first row, quant plane
    uint32_t yr;      // lane * 16
    uint32_t sc;      // weight row of this thread's scale load, relative to the tile's first row
    uint32_t ysc;     // record (tid % 128) of the activation scale load
};

template <bool CHECK, int RB>
__device__ __forceinline__ void stage_issue(uint32_t stage_off, Scales &sc, const LaneOffsets<RB> &lo,
                                            const uint8_t *wq_base, const uint8_t *wd_base, const uint8_t *y_base,
                                            uint32_t y_limit, uint32_t wave) {
    using T = DmaTile<RB>;
    // weight quants: RB chunks of 8 rows x 128 B per wave
#pragma unroll
    for (int i = 0; i < RB; ++i) dma16(wq_base, lo.wq[i], stage_off + (wave * RB + i) * 1024);
    // activation records: 18 chunks of 1 KB, contiguous in memory
#pragma unroll
    for (int i = 0; i < 5; ++i) {
        const uint32_t c = wave + 4 * i;
        if (c < 18) {
            uint32_t off = c * 1024 + lo.yr;
            if (CHECK) off = off <= y_limit ? off : y_limit;
            dma16(y_base, off, stage_off + T::kOffYr + c * 1024);
        }
    }
    // scales through registers; every thread loads both kinds (branch-free), a part of each is used
    sc.wd = *(const __attribute__((address_space(1))) v2u *)(wd_base + lo.sc);
    uint32_t off = lo.ysc;
    if (CHECK) off = off <= y_limit ? off : y_limit;
    sc.yd = *(const __attribute__((address_space(1))) v4i *)(y_base + off);
}

template <int RB>
__device__ __forceinline__ void stage_scales(uint8_t *stage, const Scales &sc, uint32_t tid) {
    using T = DmaTile<RB>;
    if (tid < T::kRows) {
        float *wsc = reinterpret_cast<float *>(stage + T::kOffWsc);
        wsc[0 * T::kRows + tid] = half_bits_to_float(static_cast<uint16_t>(sc.wd.x & 0xffffu));
        wsc[1 * T::kRows + tid] = half_bits_to_float(static_cast<uint16_t>(sc.wd.x >> 16));
        wsc[2 * T::kRows + tid] = half_bits_to_float(static_cast<uint16_t>(sc.wd.y & 0xffffu));
        wsc[3 * T::kRows + tid] = half_bits_to_float(static_cast<uint16_t>(sc.wd.y >> 16));
    } else if (tid >= 128) {
        int *ysc = reinterpret_cast<int *>(stage + T::kOffYsc);
        const uint32_t j = tid - 128;
        ysc[0 * 128 + j] = sc.yd.x; ysc[1 * 128 + j] = sc.yd.y; ysc[2 * 128 + j] = sc.yd.z; ysc[3 * 128 + j] = sc.yd.w;
    }
}

// SILU: the tile's first RB / 2 blocks of 32 LDS rows hold rows of the gate weight `w`, the other
// RB / 2 the same rows of the up weight `w2`; a lane's sums for gate row r and up row r then sit in
// the same lane (acc[rb] and acc[rb + RB / 2]) and the store writes silu(gate) * up, so a tile
// yields 16 * RB output rows and `rows` counts the rows of one weight.
template <bool CHECK, int RB, bool SILU>
__global__ __launch_bounds__(kGemmThreads, 2) void gemm_d4_dma_kernel(
        const uint8_t *__restrict__ w, const uint8_t *__restrict__ w2, const uint8_t *__restrict__ y, const TileOut out,
        uint32_t rows, uint32_t nb, uint32_t batch, uint32_t row_tiles, uint32_t col_tiles, uint32_t split_from) {
    using T = DmaTile<RB>;
    constexpr uint32_t kOut = SILU ? T::kRows / 2 : T::kRows;   // output rows of a tile
    extern __shared__ __align__(16) uint8_t smem[];
    const uint32_t tid = threadIdx.x, lane = tid % kWave;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const uint32_t l32 = lane & 31u, lhalf = lane >> 5;
    const uint32_t stride_dst = out.stride_dst;
    // Tiles from split_from on are computed by two workgroups, one per half of K, which add their
    // sums into a zeroed dst (see launch_dma): the tiles of a last, partly filled round.
    uint32_t id = blockIdx.x, k_half = 0;
    const bool split = id >= split_from;
    if (split) {
        k_half = (id - split_from) & 1u;
        id = split_from + ((id - split_from) >> 1);
    }
    // consecutive workgroup ids land on different XCDs: give every XCD whole row tiles and walk
    // the column tiles of a row tile back to back, so its weights stay in that XCD's L2
    const uint32_t xcd = id % 8u, seq = id / 8u;
    const uint32_t rt = (seq / col_tiles) * 8u + xcd, ct = seq % col_tiles;
    if (rt >= row_tiles) return;   // uniform for the workgroup
    const uint32_t row0 = rt * kOut, col0 = ct * kTileCols;
    const uint32_t nsb = nb / 4;
    const uint32_t sb0 = (split && k_half) ? nsb / 2 : 0u;
    const uint32_t sb1 = (split && !k_half) ? nsb / 2 : nsb;

    v16i seed;
#pragma unroll
    for (int i = 0; i < 16; ++i) seed[i] = static_cast<int>(kMagicBits);
    float acc[RB][16];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[rb][v] = 0.0f;

    const uint64_t row_bytes = static_cast<uint64_t>(nb) * 34;
    LaneOffsets<RB> lo;
#pragma unroll
    for (int i = 0; i < RB; ++i) {
        const uint32_t r = (wave * RB + i) * 8 + lane / 8;   // LDS row of the tile
        uint32_t gr = r % kOut;                               // weight row, counted from the tile's first
        if (CHECK) gr = row0 + gr < rows ? gr : rows - 1 - row0;   // rows past the end re-read the last row
        lo.wq[i] = gr * static_cast<uint32_t>(row_bytes) + ((lane & 7u) ^ swz(r)) * 16;
    }
    lo.yr = lane * 16;
    {
        uint32_t gr = (tid & (T::kRows - 1)) % kOut;
        if (CHECK) gr = row0 + gr < rows ? gr : rows - 1 - row0;
        lo.sc = gr * static_cast<uint32_t>(row_bytes);
        lo.ysc = (tid & 127u) * kRec;
    }
    const uint64_t y_step = static_cast<uint64_t>(batch) * kRec;
    // Which weight a wave stages is wave-uniform: quants, waves 0 .. 3 take LDS rows 32 wave ..; scales,
    // thread t < 128 takes LDS row t (wave 0: rows 0 .. 63, wave 1: rows 64 .. 127).
    const uint8_t *wq_src = (SILU && wave >= 2) ? w2 : w;
    const uint8_t *wd_src = (SILU && wave == 1) ? w2 : w;
    const uint8_t *wd_base = uniform_ptr(wd_src + row0 * row_bytes + sb0 * 8u);             // scale plane of the tile's first row
    const uint8_t *wq_base = uniform_ptr(wq_src + row0 * row_bytes + 2 * nb + sb0 * 128u);  // quant plane
    const uint8_t *y_base = uniform_ptr(y + static_cast<uint64_t>(col0) * kRec + sb0 * y_step);
    // last 16-byte offset from y_base that is still inside the activation buffer (used when CHECK)
    uint64_t y_room = static_cast<uint64_t>(nsb - sb0) * batch * kRec - static_cast<uint64_t>(col0) * kRec - 16;
    auto limit32 = [](uint64_t v) { return static_cast<uint32_t>(v < 0xffffffffull ? v : 0xffffffffull); };
    const uint32_t smem_off = lds_offset_of(smem);

    Scales sc;
    stage_issue<CHECK, RB>(smem_off, sc, lo, wq_base, wd_base, y_base, limit32(y_room), wave);
    stage_scales<RB>(smem, sc, tid);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    const uint32_t fl = swz(l32);
    const uint32_t a_off = T::kOffYr + (wave * 32 + l32) * kRec + 16 + lhalf * 16;
    const uint32_t b_row = l32 * 128;
    asm volatile("" : "+v"(seed));   // keep the seed in registers instead of rebuilding it per block

    for (uint32_t sb = sb0; sb < sb1; ++sb) {
        const uint32_t cur_sel = ((sb - sb0) & 1u) * T::kStage, nxt_sel = T::kStage - cur_sel;
        const uint8_t *cur = smem + cur_sel;
        const bool more = sb + 1 < sb1;
        if (more) {
            wq_base += 128; wd_base += 8; y_base += y_step; y_room -= y_step;
            stage_issue<CHECK, RB>(smem_off + nxt_sel, sc, lo, wq_base, wd_base, y_base, limit32(y_room), wave);
        }
        const float *wsc = reinterpret_cast<const float *>(cur + T::kOffWsc);
        const float *ysc = reinterpret_cast<const float *>(cur + T::kOffYsc);
        // one Q8 block (K = 32) per trip; kept rolled so that only the result patches of one block
        // are live at a time
#pragma unroll 1
        for (uint32_t sub = 0; sub < 4; ++sub) {
            const v4i a = *reinterpret_cast<const v4i *>(cur + a_off + sub * 32);
            const uint32_t b_off = b_row + (((2 * sub + lhalf) ^ fl) * 16);
            float dy[16];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 t = *reinterpret_cast<const float4 *>(ysc + sub * 128 + wave * 32 + 8 * g + 4 * lhalf);
                dy[4 * g + 0] = t.x; dy[4 * g + 1] = t.y; dy[4 * g + 2] = t.z; dy[4 * g + 3] = t.w;
            }
            v16i r[RB];
            float dw[RB];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const v4i b = *reinterpret_cast<const v4i *>(cur + rb * 32 * 128 + b_off);
                dw[rb] = wsc[sub * T::kRows + rb * 32 + l32];
                r[rb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, seed, 0, 0, 0);
            }
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const float cw = -kMagic * dw[rb];
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float g = fmaf(as_f32(r[rb][v]), dw[rb], cw);
                    acc[rb][v] = fmaf(g, dy[v], acc[rb][v]);
                }
            }
        }
        if (more) stage_scales<RB>(smem + nxt_sel, sc, tid);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }
    // D[i][n]: n = lane % 32 (weight row), i = 8*(v/4) + 4*(lane/32) + v%4 (activation row)
    if constexpr (SILU) {
#pragma unroll
        for (int rb = 0; rb < RB / 2; ++rb) {
            const uint32_t r = row0 + rb * 32 + l32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t j = col0 + wave * 32 + 8 * (v / 4) + 4 * lhalf + (v % 4);
                if (!CHECK || (r < rows && j < batch))
                    static_cast<float *>(out.dst)[static_cast<uint64_t>(j) * stride_dst + r] = silu_mul(acc[rb][v], acc[rb + RB / 2][v]);
            }
        }
        return;
    }
    if (split) {
        // two addends onto zero: the sum does not depend on which half arrives first
        float *dst = static_cast<float *>(out.dst);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const uint32_t r = row0 + rb * 32 + l32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t j = col0 + wave * 32 + 8 * (v / 4) + 4 * lhalf + (v % 4);
                if (!CHECK || (r < rows && j < batch))
                    unsafeAtomicAdd(&dst[static_cast<uint64_t>(j) * stride_dst + r], acc[rb][v]);
            }
        }
        return;
    }
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        const uint32_t r = row0 + rb * 32 + l32;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t j = col0 + wave * 32 + 8 * (v / 4) + 4 * lhalf + (v % 4);
            if (!CHECK || (r < rows && j < batch)) emit(out, static_cast<uint64_t>(j) * stride_dst + r, acc[rb][v]);
        }
    }
}

// Zeroes the dst patches of the tiles from split_from on (one workgroup per tile), which the two
// K halves of gemm_d4_dma_kernel then add into.  A kernel rather than a memset so that a caller
// can capture the launch into a graph.
template <int RB>
__global__ __launch_bounds__(kGemmThreads) void gemm_zero_split_tiles_kernel(
        float *__restrict__ dst, uint32_t rows, uint32_t batch, uint32_t stride_dst, uint32_t row_tiles,
        uint32_t col_tiles, uint32_t split_from) {
    using T = DmaTile<RB>;
    const uint32_t id = split_from + blockIdx.x, xcd = id % 8u, seq = id / 8u;
    const uint32_t rt = (seq / col_tiles) * 8u + xcd, ct = seq % col_tiles;
    if (rt >= row_tiles) return;
    const uint32_t row0 = rt * T::kRows, col0 = ct * kTileCols;
    for (uint32_t i = threadIdx.x; i < T::kRows * kTileCols; i += kGemmThreads) {
        const uint32_t r = row0 + i % T::kRows, j = col0 + i / T::kRows;
        if (r < rows && j < batch) dst[static_cast<uint64_t>(j) * stride_dst + r] = 0.0f;
    }
}

// ---- medium batches: 32-row tiles behind a ring of LDS stages ---------------------------------
// A batch of 33..a few hundred rows gives each CU only a few hundred MFMAs per launch: one K-step
// of a narrow tile is a few hundred cycles of arithmetic, far less than the time its operands
// take to arrive, so with two stages every K-step costs a memory latency (what the quarter tile
// above does: ~1 us per step).  Here the tile is 32 weight rows x (32 * CB) activation rows and
// the K-steps (one 128-element super-block each) run through a ring of NS stages: NS - 1 steps
// are in flight while one is consumed, loads are awaited by count (vmcnt), oldest first, and one
// barrier per step publishes it.  Everything travels global -> LDS directly in whole 128-byte
// lines (per-lane strided loads of the operands were measured 2-3 x slower), the scales included:
// the fp16 weight scales raw (converted by their readers), the activation scales as one 4-byte
// transfer per lane that lays the 32 scales of a (group, block) out contiguously.  The pieces of a
// step are dealt round-robin to the W waves, every wave issuing the same number of loads (the
// remainder repeats the last piece) so that the wait counts are compile-time constants.
// The waves split the tile by activation group first (CB groups of 32 rows) and by K second:
// S = W / CB waves share an output patch, each taking 4 / S of the four blocks of every step; their
// partial sums are added through LDS at the end as a balanced tree (deterministic).
template <int CB, int W, int RB = 1>
struct RingTile {
    static constexpr int kCols = 32 * CB;
    static constexpr int kRows = 32 * RB;                             // weight rows of the tile: RB blocks of 32
    static constexpr int kShares = W / CB;                             // waves per output patch (K split)
    static constexpr int kWItems = 4 * RB;                             // 1 KB pieces of the weight quants (8 rows each)
    static constexpr int kYChunks = (kCols * kRec + 1023) / 1024;     // 1 KB pieces of the activation records
    static constexpr int kDyItems = CB * 2;                            // 64 lanes fill two 32-float slots
    static constexpr int kItems = kWItems + kYChunks + kDyItems + RB;  // weight pieces, records, scales, weight scales
    static constexpr int kLoads = (kItems + W - 1) / W;                // load instructions per wave and step
    static constexpr int kOffYr = kRows * 128;
    static constexpr int kOffDy = kOffYr + kYChunks * 1024;            // fp32 activation scales, [group][block][32]
    static constexpr int kOffWsc = kOffDy + CB * 4 * 128;              // raw fp16 weight scales, [row][4]
    static constexpr int kStage = kOffWsc + 256 * RB;
    static_assert(W % CB == 0 && 4 % kShares == 0, "a patch is shared by 1, 2 or 4 waves");
};

// 4 bytes per lane, global -> LDS at lds_off + lane * 4.
__device__ __forceinline__ void dma4(const uint8_t *uniform_base, uint32_t lane_off, uint32_t lds_off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(lds_off), "v"(lane_off), "s"(uniform_base) : "memory", "m0");
}

// Waits until at most `steps` K-steps of this wave's loads are still in flight.
template <int LOADS, int MAX_STEPS>
__device__ __forceinline__ void wait_ring(uint32_t steps) {
    static_assert(LOADS * MAX_STEPS <= 63, "vmcnt holds 6 bits");
    if constexpr (MAX_STEPS > 0) {
        if (steps >= static_cast<uint32_t>(MAX_STEPS)) {
            asm volatile("s_waitcnt vmcnt(%0)" :: "n"(LOADS * MAX_STEPS) : "memory");
            return;
        }
        wait_ring<LOADS, MAX_STEPS - 1>(steps);
    } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
}

// SILU (RB even): the first RB / 2 blocks of 32 LDS rows hold rows of the gate weight `w`, the others
// the same rows of the up weight `w2`; the tile yields 16 * RB rows of silu(gate) * up and `rows`
// counts the rows of one weight.
// One tile (row tile rt, column tile ct) over the super-blocks sb0 .. sb0 + nsb - 1 of K.  ATOMIC: the
// sums are added into dst (a tile whose K range is shared by two workgroups, dst zeroed before the
// launch); else they are stored through the launch's epilogue.  Every wave of the workgroup calls it.
template <int CB, int W, int NS, bool ATOMIC, int RB, bool SILU>
__device__ __forceinline__ void ring_tile_segment(
        uint8_t *smem, const uint8_t *__restrict__ w, const uint8_t *__restrict__ w2, const uint8_t *__restrict__ y,
        const TileOut &out, uint32_t rows, uint32_t nb, uint32_t batch, uint32_t rt, uint32_t ct, uint32_t sb0, uint32_t nsb) {
    static_assert(!ATOMIC || !SILU, "a SwiGLU tile needs its whole sums");
    static_assert(!SILU || RB % 2 == 0, "a SwiGLU tile holds as many gate rows as up rows");
    using T = RingTile<CB, W, RB>;
    constexpr uint32_t S = T::kShares;
    constexpr uint32_t kOut = SILU ? T::kRows / 2 : T::kRows;   // output rows of a tile
    const uint32_t stride_dst = out.stride_dst;
    const uint32_t lane = threadIdx.x % kWave;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t l32 = lane & 31u, lhalf = lane >> 5;
    const uint32_t grp = wave % CB, share = wave / CB;   // activation group, K share
    const uint32_t row0 = rt * kOut, col0 = ct * T::kCols;
    const uint32_t nsb_all = nb / 4;
    const uint64_t row_bytes = static_cast<uint64_t>(nb) * 34;

    // The pieces of a step this wave loads: kind and LDS position are wave-uniform, the per-lane
    // source offsets do not change over the K loop.  Weight rows past the end re-read the last row,
    // activation rows past the end of the batch the last activation row (never stored).
    auto clamp_row = [&](uint32_t r) {   // LDS row of the tile -> weight row, counted from the tile's first
        r %= kOut;
        return row0 + r < rows ? r : rows - 1 - row0;
    };
    uint32_t lane_off[T::kLoads];
#pragma unroll
    for (int i = 0; i < T::kLoads; ++i) {
        uint32_t item = wave + W * i;
        item = item < T::kItems ? item : T::kItems - 1;
        if (item < T::kWItems) {                          // 8 weight rows x 128 B
            const uint32_t r = item * 8 + lane / 8;
            lane_off[i] = clamp_row(r) * static_cast<uint32_t>(row_bytes) + ((lane & 7u) ^ swz(r)) * 16;
        } else if (item < T::kWItems + T::kYChunks) {     // 1 KB of activation records
            lane_off[i] = (item - T::kWItems) * 1024 + lane * 16;
        } else if (item < T::kWItems + T::kYChunks + T::kDyItems) {   // the scales of two (group, block) pairs
            const uint32_t sl = (item - T::kWItems - T::kYChunks) * 2 + lhalf;
            uint32_t j = col0 + (sl / 4) * 32 + l32;
            j = j < batch ? j : batch - 1;
            lane_off[i] = (j - col0) * kRec + (sl % 4) * 4;
        } else {                                          // fp16 weight scales: 32 rows x 8 B per item
            const uint32_t r = (item - T::kWItems - T::kYChunks - T::kDyItems) * 32 + lane / 2;
            lane_off[i] = clamp_row(r) * static_cast<uint32_t>(row_bytes) + (lane & 1u) * 4;
        }
    }
    const uint8_t *wd_base0 = uniform_ptr(w + row0 * row_bytes);
    const uint8_t *wd_base1 = SILU ? uniform_ptr(w2 + row0 * row_bytes) : wd_base0;   // the up weight's rows
    const uint8_t *y_base0 = uniform_ptr(y + static_cast<uint64_t>(col0) * kRec);
    const uint64_t y_step = static_cast<uint64_t>(batch) * kRec;
    const uint64_t y_room0 = static_cast<uint64_t>(nsb_all) * batch * kRec - static_cast<uint64_t>(col0) * kRec - 16;
    const uint32_t smem_off = lds_offset_of(smem);

    auto issue = [&](uint32_t step) {   // step counts from this workgroup's first super-block
        const uint32_t stage_off = smem_off + (step % NS) * T::kStage;
        const uint32_t gstep = sb0 + step;
        const uint64_t wd_step = static_cast<uint64_t>(gstep) * 8, wq_step = 2 * nb + static_cast<uint64_t>(gstep) * 128;
        const uint8_t *y_base = y_base0 + gstep * y_step;
        const uint64_t room = y_room0 - gstep * y_step;
        const uint32_t y_limit = static_cast<uint32_t>(room < 0xffffffffull ? room : 0xffffffffull);
#pragma unroll
        for (int i = 0; i < T::kLoads; ++i) {
            uint32_t item = wave + W * i;
            item = item < T::kItems ? item : T::kItems - 1;
            if (item < T::kWItems) {
                dma16((SILU && item >= T::kWItems / 2 ? wd_base1 : wd_base0) + wq_step, lane_off[i], stage_off + item * 1024);
            } else if (item < T::kWItems + T::kYChunks) {
                const uint32_t off = lane_off[i] <= y_limit ? lane_off[i] : y_limit;   // never past the buffer
                dma16(y_base, off, stage_off + T::kOffYr + (item - T::kWItems) * 1024);
            } else if (item < T::kWItems + T::kYChunks + T::kDyItems) {
                dma4(y_base, lane_off[i], stage_off + T::kOffDy + (item - T::kWItems - T::kYChunks) * 256);
            } else {
                const uint32_t blk32 = item - T::kWItems - T::kYChunks - T::kDyItems;   // block of 32 LDS rows
                dma4((SILU && blk32 >= RB / 2 ? wd_base1 : wd_base0) + wd_step, lane_off[i], stage_off + T::kOffWsc + blk32 * 256);
            }
        }
    };

    v16i seed;
#pragma unroll
    for (int i = 0; i < 16; ++i) seed[i] = static_cast<int>(kMagicBits);
    asm volatile("" : "+v"(seed));
    float acc[RB][16];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[rb][v] = 0.0f;

    const uint32_t ahead = nsb < NS - 1 ? nsb : NS - 1;
    for (uint32_t s = 0; s < ahead; ++s) issue(s);
    wait_ring<T::kLoads, NS - 2>(ahead - 1);
    __syncthreads();

    const uint32_t fl = swz(l32);
    const uint32_t a_off = T::kOffYr + (grp * 32 + l32) * kRec + 16 + lhalf * 16;
    const uint32_t dy_off = T::kOffDy + grp * 512 + lhalf * 16;
    for (uint32_t sb = 0; sb < nsb; ++sb) {
        if (sb + NS - 1 < nsb) issue(sb + NS - 1);   // into the slot consumed one step ago
        const uint8_t *cur = smem + (sb % NS) * T::kStage;
#pragma unroll
        for (uint32_t t = 0; t < 4 / S; ++t) {
            const uint32_t sub = share * (4 / S) + t;
            const v4i a = *reinterpret_cast<const v4i *>(cur + a_off + sub * 32);
            float dy[16];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 q = *reinterpret_cast<const float4 *>(cur + dy_off + sub * 128 + g * 32);
                dy[4 * g + 0] = q.x; dy[4 * g + 1] = q.y; dy[4 * g + 2] = q.z; dy[4 * g + 3] = q.w;
            }
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {   // the activation fragment serves every 32-row block of the tile
                const uint32_t wr = rb * 32 + l32;
                const v4i b = *reinterpret_cast<const v4i *>(cur + wr * 128 + (((2 * sub + lhalf) ^ fl) * 16));
                const float dw = half_bits_to_float(*reinterpret_cast<const uint16_t *>(cur + T::kOffWsc + wr * 8 + sub * 2));
                const v16i r = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, seed, 0, 0, 0);
                const float cw = -kMagic * dw;
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[rb][v] = fmaf(fmaf(as_f32(r[v]), dw, cw), dy[v], acc[rb][v]);
            }
        }
        if (sb + 1 < nsb) {
            const uint32_t later = nsb - 2 - sb;   // steps issued beyond the next one
            wait_ring<T::kLoads, NS - 2>(later < NS - 2 ? later : NS - 2);
        }
        __syncthreads();
    }

    // D[i][n]: n = lane % 32 (weight row), i = 8*(v/4) + 4*(lane/32) + v%4 (activation row of the group)
    auto store = [&](int rb, int v, float value) {
        const uint32_t r_out = row0 + rb * 32 + l32;
        const uint32_t j = col0 + grp * 32 + 8 * (v / 4) + 4 * lhalf + (v % 4);
        if (r_out < rows && j < batch) {
            const uint64_t idx = static_cast<uint64_t>(j) * stride_dst + r_out;
            if constexpr (ATOMIC) unsafeAtomicAdd(static_cast<float *>(out.dst) + idx, value);   // two addends onto zero: order-independent
            else if constexpr (SILU) static_cast<float *>(out.dst)[idx] = value;
            else emit(out, idx, value);
        }
    };
    if constexpr (S == 1) {
        if constexpr (SILU) {
#pragma unroll
            for (int rb = 0; rb < RB / 2; ++rb)
#pragma unroll
                for (int v = 0; v < 16; ++v) store(rb, v, silu_mul(acc[rb][v], acc[rb + RB / 2][v]));
        } else {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int v = 0; v < 16; ++v) store(rb, v, acc[rb][v]);
        }
    } else {
        // every load has landed and every wave is past its last read of the stages: reuse them
        float *part = reinterpret_cast<float *>(smem);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int v = 0; v < 16; ++v) part[((wave * RB + rb) * 16 + v) * kWave + lane] = acc[rb][v];
        __syncthreads();
        constexpr int kMine = 16 / S;   // outputs of each patch this wave finishes
        auto total_of = [&](int rb, int v) {
            auto p = [&](uint32_t s) { return part[(((s * CB + grp) * RB + rb) * 16 + v) * kWave + lane]; };
            if constexpr (S == 2) return p(0) + p(1);
            else return (p(0) + p(1)) + (p(2) + p(3));
        };
#pragma unroll
        for (int rb = 0; rb < (SILU ? RB / 2 : RB); ++rb)
#pragma unroll
            for (int k = 0; k < kMine; ++k) {
                const int v = share * kMine + k;
                if constexpr (SILU) store(rb, v, silu_mul(total_of(rb, v), total_of(rb + RB / 2, v)));
                else store(rb, v, total_of(rb, v));
            }
    }
}

template <int CB, int W, int NS, bool KSPLIT, int RB = 1, bool SILU = false>
__global__ __launch_bounds__(kWave * W) void gemm_d4_ring_kernel(
        const uint8_t *__restrict__ w, const uint8_t *__restrict__ w2, const uint8_t *__restrict__ y, const TileOut out,
        uint32_t rows, uint32_t nb, uint32_t batch, uint32_t row_tiles, uint32_t col_tiles) {
    static_assert(!KSPLIT || (RB == 1 && !SILU), "only the narrowest tile is cut along K");
    extern __shared__ __align__(16) uint8_t smem[];
    // KSPLIT: every tile is computed by two workgroups, one per half of K, which add their sums
    // into a zeroed dst (see launch_ring)
    const uint32_t id = KSPLIT ? blockIdx.x >> 1 : blockIdx.x, k_half = KSPLIT ? blockIdx.x & 1u : 0u;
    const uint32_t xcd = id % 8u, seq = id / 8u;
    const uint32_t rt = (seq / col_tiles) * 8u + xcd, ct = seq % col_tiles;
    if (rt >= row_tiles) return;   // uniform for the workgroup
    const uint32_t nsb_all = nb / 4;
    const uint32_t sb0 = (KSPLIT && k_half) ? nsb_all / 2 : 0u;                   // first super-block of this workgroup
    const uint32_t nsb = ((KSPLIT && !k_half) ? nsb_all / 2 : nsb_all) - sb0;     // and how many it covers
    ring_tile_segment<CB, W, NS, KSPLIT, RB, SILU>(smem, w, w2, y, out, rows, nb, batch, rt, ct, sb0, nsb);
}

// The same tiles with the K steps of all tiles dealt out evenly: workgroup i takes the steps
// [total i / G, total (i + 1) / G) of the tile-major step sequence, i.e. the end of one tile, whole
// tiles, and the start of another.  For launches with a few more tiles than the chip holds
// workgroups (17408 rows in 64 x 64 tiles at batch 128: 544 tiles for 512 slots), where a last round
// of a few tiles otherwise lasts as long again as half a round.  A range is at least one tile long,
// so a tile's K range is shared by at most two workgroups: its sums are added into a dst zeroed by
// gemm_zero_dst_kernel (two addends onto zero: results repeat bit for bit); tiles that one workgroup
// covers alone are stored.  Workgroups of one XCD (index % 8) take neighbouring ranges.
template <int CB, int W, int NS, int RB>
__global__ __launch_bounds__(kWave * W) void gemm_d4_ring_balanced_kernel(
        const uint8_t *__restrict__ w, const uint8_t *__restrict__ y, const TileOut out,
        uint32_t rows, uint32_t nb, uint32_t batch, uint32_t tiles, uint32_t col_tiles) {
    extern __shared__ __align__(16) uint8_t smem[];
    const uint32_t nsb_all = nb / 4;
    const uint64_t total = static_cast<uint64_t>(tiles) * nsb_all;
    const uint32_t groups = gridDim.x;                                   // a multiple of 8
    const uint32_t index = (blockIdx.x % 8u) * (groups / 8u) + blockIdx.x / 8u;
    uint64_t step = total * index / groups;
    const uint64_t end = total * (index + 1) / groups;
    while (step < end) {
        const uint32_t tile = static_cast<uint32_t>(step / nsb_all), sb0 = static_cast<uint32_t>(step % nsb_all);
        const uint64_t left = end - step;
        const uint32_t nsb = left < nsb_all - sb0 ? static_cast<uint32_t>(left) : nsb_all - sb0;
        const uint32_t rt = tile / col_tiles, ct = tile % col_tiles;
        if (nsb == nsb_all) ring_tile_segment<CB, W, NS, false, RB, false>(smem, w, nullptr, y, out, rows, nb, batch, rt, ct, 0, nsb);
        else ring_tile_segment<CB, W, NS, true, RB, false>(smem, w, nullptr, y, out, rows, nb, batch, rt, ct, sb0, nsb);
        step += nsb;
        __syncthreads();   // the stages (and the partial sums kept in them) are free for the next tile
    }
}

// Zeroes dst[j][0 .. rows) for j < batch: the start value of a launch whose workgroups add into dst.
// A kernel rather than a memset so that a caller can capture the call into a graph.
__global__ __launch_bounds__(256) void gemm_zero_dst_kernel(float *__restrict__ dst, uint32_t rows, uint32_t stride_dst) {
    float *row = dst + static_cast<uint64_t>(blockIdx.y) * stride_dst;
    for (uint32_t r = blockIdx.x * 1024u + threadIdx.x; r < rows && r < (blockIdx.x + 1u) * 1024u; r += 256u) row[r] = 0.0f;
}

// Ring depths and waves per workgroup of the medium-batch kernel (compile-time).  Measured on
// MI355X at 5120 x 5120: deeper rings change nothing once three steps are in flight (the serial
// path of a step binds), eight waves beat four by 1.4 x at 64 activation rows, sixteen beat eight
// at 128 rows only while there is at most one tile per CU; two super-blocks per step (half as
// many barriers, two independent chains per wave) were 1.2-1.3 x slower at the same LDS budget.
constexpr int kRing1 = 6, kRing2 = 4, kRing4 = 3;   // ring depth of the 32-, 64- and 128-row-wide tile
constexpr int kRingWaves2 = 8, kRingWaves4 = 8;    // waves per workgroup of the 64- and 128-wide tile

template <bool CHECK, bool A16>
int launch_variant(const uint8_t *w, const uint8_t *y, float *dst, uint32_t rows, uint32_t nb,
                   uint32_t batch, uint32_t stride, uint32_t row_tiles, uint32_t col_tiles, uint32_t grid,
                   hipStream_t stream) {
    // more than 64 KiB of dynamic LDS has to be granted per kernel, once per process
    static std::atomic<bool> granted{false};   // two threads may both get here first: the grant is idempotent
    if (!granted) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_d4_kernel<CHECK, A16>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes) != hipSuccess) {
            (void)hipGetLastError();
            return fail(Q8MI_LAUNCH_ERROR, "gemm: cannot reserve %d bytes of LDS", kLdsBytes);
        }
        granted = true;
    }
    gemm_d4_kernel<CHECK, A16><<<grid, kGemmThreads, kLdsBytes, stream>>>(
        w, y, dst, rows, nb, batch, stride, row_tiles, col_tiles);
    return check_launch("gemm");
}

// A last round of main tiles that fills at most half of the chip's slots (two workgroups per CU)
// leaves the other CUs idle for most of a tile's time: those tiles are cut in two along K and both
// halves add into a zeroed dst.  Measured on MI355X at M=2048: K=17408, N=5120 (640 tiles on 512
// slots) and K=5120, N=17408 (2176 tiles).  Only on whole groups of eight row tiles (every
// workgroup id is a tile then) and at least four super-blocks of K.  Returns the number of tiles
// cut this way (0: none).  Only plain fp32 stores can be split: a sum that arrives in two halves
// cannot be rounded to bf16 or added to a residual in an order that repeats.
uint64_t split_round_tiles(uint32_t rows, uint32_t nb, uint32_t batch) {
    const uint32_t row_tiles = (rows + kTileRows - 1) / kTileRows;
    const uint32_t col_tiles = (batch + kTileCols - 1) / kTileCols;
    if (row_tiles % 8 != 0 || nb / 4 < 4) return 0;
    const uint64_t tiles = static_cast<uint64_t>(row_tiles) * col_tiles;
    const uint64_t slots = 2ull * static_cast<uint32_t>(device_cu_count());
    const uint64_t left = tiles % slots;
    return (tiles >= slots && left != 0 && left * 2 <= slots) ? left : 0;
}

// A call of the tile kernels: one weight (or gate + up for the SwiGLU form) and what to do with the sums.
struct TileCall {
    const uint8_t *w;
    const uint8_t *w2;   // the up weight of the SwiGLU form, else unused
    const uint8_t *y;
    TileOut out;
};

template <bool CHECK, int RB, bool SILU>
int launch_dma(const TileCall &c, uint32_t rows, uint32_t nb, uint32_t batch, bool may_split, hipStream_t stream) {
    using T = DmaTile<RB>;
    static std::atomic<bool> granted{false};   // two threads may both get here first: the grant is idempotent
    if (!granted) {
        if (T::kLds > 64 * 1024 &&
            hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_d4_dma_kernel<CHECK, RB, SILU>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, T::kLds) != hipSuccess) {
            (void)hipGetLastError();
            return fail(Q8MI_LAUNCH_ERROR, "gemm: cannot reserve %d bytes of LDS", T::kLds);
        }
        granted = true;
    }
    constexpr uint32_t kOut = SILU ? T::kRows / 2 : T::kRows;
    const uint32_t row_tiles = (rows + kOut - 1) / kOut;
    const uint32_t col_tiles = (batch + kTileCols - 1) / kTileCols;
    uint64_t grid64 = static_cast<uint64_t>((row_tiles + 7u) / 8u * 8u) * col_tiles;
    if (grid64 > 0x7ffffff0ull) return fail(Q8MI_REJECTED, "gemm: too many tiles");
    uint32_t split_from = 0xffffffffu;
    if (may_split) {
        const uint64_t left = split_round_tiles(rows, nb, batch);
        if (left != 0) {
            split_from = static_cast<uint32_t>(grid64 - left);
            gemm_zero_split_tiles_kernel<RB><<<static_cast<uint32_t>(left), kGemmThreads, 0, stream>>>(
                static_cast<float *>(c.out.dst), rows, batch, c.out.stride_dst, row_tiles, col_tiles, split_from);
            grid64 += left;
        }
    }
    gemm_d4_dma_kernel<CHECK, RB, SILU><<<static_cast<uint32_t>(grid64), kGemmThreads, T::kLds, stream>>>(
        c.w, c.w2, c.y, c.out, rows, nb, batch, row_tiles, col_tiles, split_from);
    return check_launch("gemm");
}

template <bool SILU>
int launch_dma_rows(const TileCall &c, uint32_t rows, uint32_t nb, uint32_t batch, bool may_split, hipStream_t stream) {
    const bool check = (rows % (SILU ? 64u : 128u) != 0) || (batch % kTileCols != 0);
    return check ? launch_dma<true, 4, SILU>(c, rows, nb, batch, may_split, stream)
                 : launch_dma<false, 4, SILU>(c, rows, nb, batch, may_split, stream);
}

template <int CB, int W, int NS, bool KSPLIT, int RB, bool SILU>
int launch_ring_inst(const TileCall &c, uint32_t rows, uint32_t nb, uint32_t batch, uint32_t row_tiles,
                     uint32_t col_tiles, uint32_t grid, hipStream_t stream) {
    using T = RingTile<CB, W, RB>;
    constexpr int lds = NS * T::kStage;
    static_assert(lds >= W * RB * 16 * kWave * 4, "the stages are reused for the partial sums of the waves");
    static std::atomic<bool> granted{false};   // two threads may both get here first: the grant is idempotent
    if (!granted) {
        if (lds > 64 * 1024 &&
            hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_d4_ring_kernel<CB, W, NS, KSPLIT, RB, SILU>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) {
            (void)hipGetLastError();
            return fail(Q8MI_LAUNCH_ERROR, "gemm: cannot reserve %d bytes of LDS", lds);
        }
        granted = true;
    }
    gemm_d4_ring_kernel<CB, W, NS, KSPLIT, RB, SILU><<<grid, kWave * W, lds, stream>>>(
        c.w, c.w2, c.y, c.out, rows, nb, batch, row_tiles, col_tiles);
    return check_launch("gemm");
}

// With at most one tile per CU the launch lasts as long as one workgroup's chain of K steps
// (a step is bound by its serial latency, not by bandwidth or arithmetic): two workgroups per
// tile, one per half of K, halve that chain; they add into a dst zeroed by one more small
// kernel.  Two addends onto zero, so results repeat bit for bit.  Only the narrowest tile
// (up to 32 activation rows, four waves): measured on MI355X 19.2 -> 15.5 us at 5120 x 5120 and
// 58.6 -> 44.6 us at K = 17408, batch 32; the wider tiles already split K over their waves
// and gain nothing (64 rows) or lose (128 rows, sixteen waves: 29 -> 35 us).
bool ring_splits_k(uint32_t rows, uint32_t nb, uint32_t batch) {
    return batch <= 32 && static_cast<uint64_t>((rows + 31u) / 32u) <= static_cast<uint32_t>(device_cu_count()) &&
           nb / 4 >= 8;
}

// Workgroups a balanced launch of these tiles uses: two per CU for the four-wave tile, one for the
// eight- and sixteen-wave tiles (measured on MI355X at 17408 x 5120: batch 32 in 32 x 32 tiles, 544
// tiles: one round of 512 and a rest 40.2 us, 512 ranges 32.7; batch 64 in 64 x 64 tiles, 272 tiles:
// as 272 workgroups 50.1 us, 256 ranges 37.5, and two ranges per CU no better than the 50; batch 128,
// 544 tiles: 63.3 us as they come, 63.9 in 256 ranges, 69.5 in 512).
template <int CB, int W, int NS, int RB>
uint32_t ring_balanced_slots() {
    constexpr uint32_t lds = NS * RingTile<CB, W, RB>::kStage;
    constexpr uint32_t per_cu = (W <= 4 && 2 * lds <= 160u * 1024u) ? 2 : 1;   // 160 KB of LDS per CU
    return per_cu * static_cast<uint32_t>(device_cu_count()) / 8u * 8u;
}

// Whether a plain-store launch of these tiles deals the K steps of all tiles out evenly (see
// gemm_d4_ring_balanced_kernel): a few more tiles than the chip holds workgroups, so that the last
// round would be at most half full.
template <int CB, int W, int NS, int RB>
bool ring_balances(uint32_t rows, uint32_t batch) {
    using T = RingTile<CB, W, RB>;
    const uint64_t tiles = static_cast<uint64_t>((rows + T::kRows - 1) / T::kRows) * ((batch + T::kCols - 1) / T::kCols);
    const uint32_t slots = ring_balanced_slots<CB, W, NS, RB>();
    return slots >= 8 && tiles > slots && tiles % slots != 0 && tiles % slots <= slots / 2 && tiles < 0x7fffffffull;
}

template <int CB, int W, int NS, int RB = 1, bool SILU = false>
int launch_ring(const TileCall &c, uint32_t rows, uint32_t nb, uint32_t batch, hipStream_t stream) {
    using T = RingTile<CB, W, RB>;
    constexpr uint32_t kOut = SILU ? T::kRows / 2 : T::kRows;
    const uint32_t row_tiles = (rows + kOut - 1) / kOut;
    const uint32_t col_tiles = (batch + T::kCols - 1) / T::kCols;
    const uint64_t grid64 = static_cast<uint64_t>((row_tiles + 7u) / 8u * 8u) * col_tiles;
    if (grid64 > 0x3fffffffull) return fail(Q8MI_REJECTED, "gemm: too many tiles");
    if constexpr (!SILU) {
        // A few more tiles than the chip holds workgroups: the K steps of all tiles dealt out evenly
        // (see gemm_d4_ring_balanced_kernel) instead of a short last round.
        if (c.out.epi == kEpiStore && ring_balances<CB, W, NS, RB>(rows, batch)) {
            constexpr int lds = NS * T::kStage;
            static std::atomic<bool> granted{false};   // two threads may both get here first: the grant is idempotent
            if (!granted) {
                if (lds > 64 * 1024 &&
                    hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_d4_ring_balanced_kernel<CB, W, NS, RB>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) {
                    (void)hipGetLastError();
                    return fail(Q8MI_LAUNCH_ERROR, "gemm: cannot reserve %d bytes of LDS", lds);
                }
                granted = true;
            }
            gemm_zero_dst_kernel<<<dim3((rows + 1023u) / 1024u, batch), 256, 0, stream>>>(
                static_cast<float *>(c.out.dst), rows, c.out.stride_dst);
            gemm_d4_ring_balanced_kernel<CB, W, NS, RB><<<ring_balanced_slots<CB, W, NS, RB>(), kWave * W, lds, stream>>>(
                c.w, c.y, c.out, rows, nb, batch, row_tiles * col_tiles, col_tiles);
            return check_launch("gemm");
        }
    }
    if constexpr (CB == 1 && RB == 1 && !SILU) {
        if (c.out.epi == kEpiStore && ring_splits_k(rows, nb, batch)) {
            gemm_zero_dst_kernel<<<dim3((rows + 1023u) / 1024u, batch), 256, 0, stream>>>(
                static_cast<float *>(c.out.dst), rows, c.out.stride_dst);
            return launch_ring_inst<CB, W, NS, true, RB, false>(c, rows, nb, batch, row_tiles, col_tiles,
                                                                static_cast<uint32_t>(grid64 * 2), stream);
        }
    }
    return launch_ring_inst<CB, W, NS, false, RB, SILU>(c, rows, nb, batch, row_tiles, col_tiles,
                                                        static_cast<uint32_t>(grid64), stream);
}

// Tile choice.  Workgroups are scheduled dynamically and a lone workgroup on a CU runs nearly
// twice as fast as two sharing its VALUs, so a partly filled last round of main tiles costs
// little: problems with at least 0.4 main tiles per resident slot (two per CU) use main tiles
// throughout (measured crossover on MI355X: between 160 and 256 main tiles); smaller ones use the
// ring-staged 32-row tiles.
bool uses_main_tiles(uint32_t rows, uint32_t batch) {
    const uint64_t slots = 2ull * static_cast<uint32_t>(device_cu_count());
    const uint64_t tiles = static_cast<uint64_t>((rows + kTileRows - 1) / kTileRows) * ((batch + kTileCols - 1) / kTileCols);
    return tiles * 5 >= slots * 2;
}

// Whether q8mi_gemm sums some tiles of this shape from two ranges of K (ring tiles with their K steps
// dealt out evenly): the fused-store entry points then decline, as for the other K splits.  Follows
// the tile choice of launch_gemm_dma below.
bool plain_gemm_balances(uint32_t rows, uint32_t nb, uint32_t batch) {
    if (uses_main_tiles(rows, batch)) return false;
    const uint32_t cus = static_cast<uint32_t>(device_cu_count());
    if (batch > 32 && batch <= 128 && static_cast<uint64_t>((rows + 31u) / 32u) * 2 >= 3ull * cus)
        return (batch > 64 && ring_balances<4, kRingWaves4, kRing4, 2>(rows, batch)) ||
               ring_balances<2, kRingWaves2, kRing2, 2>(rows, batch);
    if (batch <= 32) return !ring_splits_k(rows, nb, batch) && ring_balances<1, 4, kRing1, 1>(rows, batch);
    if (batch <= 64) return ring_balances<2, kRingWaves2, kRing2, 1>(rows, batch);
    const uint64_t ring_tiles = static_cast<uint64_t>((rows + 31u) / 32u) * ((batch + 127u) / 128u);
    if (ring_tiles <= cus) return ring_balances<4, 16, kRing4, 1>(rows, batch);
    return ring_balances<4, kRingWaves4, kRing4, 1>(rows, batch);
}

int launch_gemm_dma(const TileCall &c, uint32_t rows, uint32_t nb, uint32_t batch, hipStream_t stream) {
    if (uses_main_tiles(rows, batch)) return launch_dma_rows<false>(c, rows, nb, batch, c.out.epi == kEpiStore, stream);
    // too few main tiles to fill the chip: 32-row tiles behind a ring of stages, as wide as the batch needs
    // Batches of 33..128 rows on matrices tall enough for more than 1.5 32-row tiles per CU take
    // 64 x 64 tiles: fewer workgroups re-read the activation records of a step (measured at
    // 17408 x 5120: batch 64 59 -> 51 us; batch 128, two column tiles of 64 against one 32-row tile
    // 128 wide, 75.9 -> 66.3 us).  The 32- and 128-row-wide tiles lose with 64 rows (54 against
    // 43 us, 88 against 77 us): their rings then leave room for one workgroup per CU only.  That is
    // no drawback once the K steps of all tiles are dealt out evenly to one workgroup per CU: with
    // 65..128 activation rows a 64-row tile 128 wide then reads every weight byte once (17408 x 5120,
    // batch 128: 272 tiles in 256 ranges 56.1 us, against 63.3 .. 63.9 in 64 x 64 tiles either way).
    if (batch > 32 && batch <= 128 && static_cast<uint64_t>((rows + 31u) / 32u) * 2 >= 3ull * static_cast<uint32_t>(device_cu_count())) {
        if (batch > 64 && c.out.epi == kEpiStore && ring_balances<4, kRingWaves4, kRing4, 2>(rows, batch))
            return launch_ring<4, kRingWaves4, kRing4, 2>(c, rows, nb, batch, stream);
        return launch_ring<2, kRingWaves2, kRing2, 2>(c, rows, nb, batch, stream);
    }
    if (batch <= 32) return launch_ring<1, 4, kRing1>(c, rows, nb, batch, stream);
    if (batch <= 64) return launch_ring<2, kRingWaves2, kRing2>(c, rows, nb, batch, stream);
    // at most one tile per CU: sixteen waves (four K shares per group) instead of eight
    const uint64_t ring_tiles = static_cast<uint64_t>((rows + 31u) / 32u) * ((batch + 127u) / 128u);
    if (ring_tiles <= static_cast<uint32_t>(device_cu_count()))
        return launch_ring<4, 16, kRing4>(c, rows, nb, batch, stream);
    return launch_ring<4, kRingWaves4, kRing4>(c, rows, nb, batch, stream);
}

// SwiGLU form: gate and up rows side by side in every tile.  Main tiles (64 gate + 64 up rows) when
// the two GEMMs it replaces would use main tiles, else 64-row ring tiles (32 + 32).
int launch_gemm_silu(const TileCall &c, uint32_t rows, uint32_t nb, uint32_t batch, hipStream_t stream) {
    if (uses_main_tiles(2 * rows, batch)) return launch_dma_rows<true>(c, rows, nb, batch, false, stream);
    if (batch <= 32) return launch_ring<1, 4, kRing1, 2, true>(c, rows, nb, batch, stream);
    if (batch <= 64) return launch_ring<2, kRingWaves2, kRing2, 2, true>(c, rows, nb, batch, stream);
    return launch_ring<4, kRingWaves4, kRing4, 2, true>(c, rows, nb, batch, stream);
}

int launch_gemm_d4(const uint8_t *w, const void *y, float *dst, uint32_t rows, uint32_t cols,
                   uint32_t batch, uint32_t stride, hipStream_t stream) {
    // small batches: the weight-streaming matrix-core GEMV, which reads the weights at HBM speed
    // instead of padding the batch to a 32-wide tile (it declines what the ring tiles serve better)
    if (batch <= 16 && (cols / kQK) % 8 == 0) {
        const int rc = gemv_mfma_d4(w, nullptr, y, dst, rows, cols, batch, stride, false, stream);
        if (rc != Q8MI_REJECTED) return rc;
    }
    const uint32_t row_tiles = (rows + kTileRows - 1) / kTileRows;
    const uint32_t col_tiles = (batch + kTileCols - 1) / kTileCols;
    const uint32_t rt_padded = (row_tiles + 7u) / 8u * 8u;
    const uint64_t grid64 = static_cast<uint64_t>(rt_padded) * col_tiles;
    if (grid64 > 0x7fffffffull) return fail(Q8MI_REJECTED, "gemm: too many tiles");
    const uint32_t grid = static_cast<uint32_t>(grid64);
    const bool check = (rows % kTileRows != 0) || (batch % kTileCols != 0);
    const uint32_t nb = cols / kQK;
    const bool a16 = nb % 8 == 0;
    const auto *yb = static_cast<const uint8_t *>(y);
    if (a16) return launch_gemm_dma(TileCall{w, nullptr, yb, TileOut{dst, nullptr, stride, kEpiStore}}, rows, nb, batch, stream);
    return check ? launch_variant<true, false>(w, yb, dst, rows, nb, batch, stride, row_tiles, col_tiles, grid, stream)
                 : launch_variant<false, false>(w, yb, dst, rows, nb, batch, stride, row_tiles, col_tiles, grid, stream);
}

// The shapes the fused-epilogue entry points serve: D4 activations on the direct-to-LDS tiles.
int fused_gate(const char *what, const void *weight, uint32_t rows, uint32_t cols, uint32_t batch) {
    if (cols == 0 || cols % 128 != 0) return fail(Q8MI_REJECTED, "%s: cols %u not a multiple of 128", what, cols);
    if (batch == 0 || rows == 0) return fail(Q8MI_REJECTED, "%s: empty shape", what);
    if (rows < 128) return fail(Q8MI_REJECTED, "%s: %u rows (fewer than 128: the activations would be Q8_1)", what, rows);
    if ((cols / kQK) % 8 != 0) return fail(Q8MI_REJECTED, "%s: cols %u not a multiple of 256", what, cols);
    if (reinterpret_cast<uintptr_t>(weight) % 16 != 0) return fail(Q8MI_REJECTED, "%s: weight pointer not 16-byte aligned", what);
    return Q8MI_OK;
}

}  // namespace
}  // namespace q8mi

using namespace q8mi;

extern "C" int q8mi_gemm(const uint8_t *weight, const void *y, float *dst, uint32_t rows, uint32_t cols,
                         uint32_t batch, uint32_t stride_dst_row, void *stream) {
    if (cols % kQK != 0) return fail(Q8MI_REJECTED, "gemm: cols %u not a multiple of 32", cols);
    if (batch == 0 || rows == 0) return fail(Q8MI_REJECTED, "gemm: empty shape");
    if (cols == 0) return fail(Q8MI_REJECTED, "gemm: cols is zero");
    if (reinterpret_cast<uintptr_t>(weight) % 16 != 0)
        return fail(Q8MI_REJECTED, "gemm: weight pointer not 16-byte aligned");
    if (rows >= 128 && cols % 128 == 0) {
        return launch_gemm_d4(weight, y, dst, rows, cols, batch, stride_dst_row, as_stream(stream));
    }
    return gemv_any_batch(weight, y, dst, rows, cols, batch, stride_dst_row, as_stream(stream));
}

extern "C" int q8mi_gemm_medium(const uint8_t *weight, const void *y_d4, float *dst, uint32_t rows,
                                uint32_t cols, uint32_t batch, uint32_t stride_dst_row, void *stream) {
    if (cols % 128 != 0) return fail(Q8MI_REJECTED, "gemm_medium: cols %u not a multiple of 128", cols);
    if (batch == 0 || rows == 0) return fail(Q8MI_REJECTED, "gemm_medium: empty shape");
    if (batch > 64) return fail(Q8MI_REJECTED, "gemm_medium: batch %u above 64", batch);
    if (cols == 0) return fail(Q8MI_REJECTED, "gemm_medium: cols is zero");
    if (reinterpret_cast<uintptr_t>(weight) % 16 != 0)
        return fail(Q8MI_REJECTED, "gemm_medium: weight pointer not 16-byte aligned");
    return launch_gemm_d4(weight, y_d4, dst, rows, cols, batch, stride_dst_row, as_stream(stream));
}

// Shapes whose plain GEMM cuts its last round of main tiles in two along K, or deals the K steps of
// its ring tiles out evenly, keep that route (the caller runs q8mi_gemm and the second step): there
// it is the faster one.
static bool plain_gemm_splits(uint32_t rows, uint32_t cols, uint32_t batch) {
    return (uses_main_tiles(rows, batch) && split_round_tiles(rows, cols / kQK, batch) != 0) ||
           plain_gemm_balances(rows, cols / kQK, batch);
}

extern "C" int q8mi_gemm_add(const uint8_t *weight, const void *y_d4, const float *residual, float *dst, uint32_t rows,
                             uint32_t cols, uint32_t batch, uint32_t stride_dst_row, void *stream) {
    if (int rc = fused_gate("gemm_add", weight, rows, cols, batch)) return rc;
    if (residual == nullptr || dst == nullptr) return fail(Q8MI_REJECTED, "gemm_add: null pointer");
    if (batch <= 16) {   // a weight stream: the matrix-core GEMV adds in place
        if (residual != dst) return fail(Q8MI_REJECTED, "gemm_add: batch %u is served in place only", batch);
        const int rc = gemv_mfma_d4(weight, nullptr, y_d4, dst, rows, cols, batch, stride_dst_row, true, as_stream(stream));
        if (rc != Q8MI_REJECTED) return rc;
    }
    if (batch <= 32 && ring_splits_k(rows, cols / kQK, batch))
        return fail(Q8MI_REJECTED, "gemm_add: this shape is summed from two halves of K (use q8mi_gemm, then q8mi_add)");
    if (plain_gemm_splits(rows, cols, batch))
        return fail(Q8MI_REJECTED, "gemm_add: some tiles of this shape are summed from two ranges of K (use q8mi_gemm, then q8mi_add)");
    return launch_gemm_dma(TileCall{weight, nullptr, static_cast<const uint8_t *>(y_d4),
                                    TileOut{dst, residual, stride_dst_row, kEpiAdd}},
                           rows, cols / kQK, batch, as_stream(stream));
}

extern "C" int q8mi_gemm_bf16(const uint8_t *weight, const void *y_d4, uint16_t *dst, uint32_t rows, uint32_t cols,
                              uint32_t batch, uint32_t stride_dst_row, void *stream) {
    if (int rc = fused_gate("gemm_bf16", weight, rows, cols, batch)) return rc;
    if (dst == nullptr) return fail(Q8MI_REJECTED, "gemm_bf16: null pointer");
    if (batch <= 16) return fail(Q8MI_REJECTED, "gemm_bf16: batch %u is a weight stream (use the GEMV family)", batch);
    if (batch <= 32 && ring_splits_k(rows, cols / kQK, batch))
        return fail(Q8MI_REJECTED, "gemm_bf16: this shape is summed from two halves of K (use q8mi_gemm, then q8mi_f32_to_bf16)");
    if (plain_gemm_splits(rows, cols, batch))
        return fail(Q8MI_REJECTED, "gemm_bf16: some tiles of this shape are summed from two ranges of K (use q8mi_gemm, then q8mi_f32_to_bf16)");
    return launch_gemm_dma(TileCall{weight, nullptr, static_cast<const uint8_t *>(y_d4),
                                    TileOut{dst, nullptr, stride_dst_row, kEpiStoreBf16}},
                           rows, cols / kQK, batch, as_stream(stream));
}

extern "C" int q8mi_gemm_silu_mul(const uint8_t *weight_gate, const uint8_t *weight_up, const void *y_d4, float *dst,
                                  uint32_t rows, uint32_t cols, uint32_t batch, uint32_t stride_dst_row, void *stream) {
    if (int rc = fused_gate("gemm_silu_mul", weight_gate, rows, cols, batch)) return rc;
    if (reinterpret_cast<uintptr_t>(weight_up) % 16 != 0 || weight_up == nullptr)
        return fail(Q8MI_REJECTED, "gemm_silu_mul: up weight pointer null or not 16-byte aligned");
    if (dst == nullptr) return fail(Q8MI_REJECTED, "gemm_silu_mul: null pointer");
    if (batch <= 16) {
        const int rc = gemv_mfma_d4(weight_gate, weight_up, y_d4, dst, rows, cols, batch, stride_dst_row, false,
                                    as_stream(stream));
        if (rc != Q8MI_REJECTED) return rc;
    }
    return launch_gemm_silu(TileCall{weight_gate, weight_up, static_cast<const uint8_t *>(y_d4),
                                     TileOut{dst, nullptr, stride_dst_row, kEpiStore}},
                            rows, cols / kQK, batch, as_stream(stream));
}
