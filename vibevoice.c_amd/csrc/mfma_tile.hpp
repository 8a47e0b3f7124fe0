// The LDS-tiled MFMA product loop shared by the FP16 GEMM and the int8 (W8A8)
// linear layer: C-tile = W-rows x X-rows^T over K, both operands K-contiguous.
#pragma once

#include "vv_common.hpp"

namespace vv {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // one 16-byte slot

// Slot swizzle for a slab of kSlab/8 16-byte slots per row. 8 slots: rows are
// 128 B = 32 banks apart, two rows share a 64-bank line, and XOR-ing the slot
// with (row / 2) % 8 spreads any 16 consecutive rows reading the same logical
// slot over all 64 banks. 4 slots: four rows share a line and the slot is
// XOR-ed with (row / 4) % 4, to the same effect.
template <int kSlab>
__device__ __forceinline__ int swz(int row, int slot) {
    static_assert(kSlab == 64 || kSlab == 32, "slab widths with a swizzle");
    return kSlab == 64 ? slot ^ ((row >> 1) & 7) : slot ^ ((row >> 2) & 3);
}

template <int kValue>
struct Const { static constexpr int value = kValue; };

// The tile loop, shared by the FP16 and the int8 products. Both operands are
// row-major with rows of `kchunks` 16-byte chunks along K (8 halves or 16
// bytes of int8: one lane's share of one MFMA K step either way). Op supplies
// the accumulator vector and the MFMA; Epi receives a wave's accumulators.
//   Op::Acc                                  16-wide accumulator vector
//   Op::mfma(u32x4 w, u32x4 x, Acc c)        one 32x32 product over a K step
//   epi(acc, m0, n0, frow, fhalf)            register 4g + r of lane l: column
//                                            n0 + 32a + 8g + 4(l/32) + r of row
//                                            m0 + 32b + l % 32, for acc[a][b]
// Where the W rows come from: PlainRows reads 16-byte slots of a row-major operand (the default); any other source
// produces slot `slot` of row `row` itself (weights dequantised on their way in): kPlain = false and
// u32x4 load(int row, int slot) const.
struct PlainRows { static constexpr bool kPlain = true; };

// kPairN (wave tiles of two N tiles, BN a multiple of 128): the two N tiles of a wave are 64 columns
// apart - wave wn takes columns 128 (wn / 2) + 32 (wn % 2) + {0, 64} of the block - so that an epilogue
// finds columns n and n + 64 in the same lane and register of acc[0] and acc[1]; epi's n0 is then the
// first column of tile 0. The products and their order per output element do not change.
template <typename Op, int BM, int BN, int WM, int WN, int kSlabChunks, bool kFull, int kAhead,
          typename Epi, typename BSrc = PlainRows, bool kPairN = false>
__device__ __forceinline__ void mfma_tile(const void* __restrict__ A, const void* __restrict__ B,
                                          int M, int N, int kchunks, const Epi& epi, const BSrc& bsrc = BSrc()) {
    constexpr int NT = WM * WN * kWave;
    constexpr int kSteps = kSlabChunks / 2;   // MFMA K steps per slab (two slots each)
    typedef typename Op::Acc Acc;
    constexpr int TM = BM / WM / 32;          // 32x32 MFMA tiles per wave along M
    constexpr int TN = BN / WN / 32;          // and along N
    constexpr int LA = BM * kSlabChunks / NT; // 16-byte loads per thread per slab, A
    constexpr int LB = BN * kSlabChunks / NT;
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tiles are 32x32 multiples");
    static_assert(LA >= 1 && LB >= 1 && (BM * kSlabChunks) % NT == 0 && (BN * kSlabChunks) % NT == 0,
                  "slab loads must divide evenly over the threads");

    constexpr int kASlots = BM * kSlabChunks, kBSlots = BN * kSlabChunks;   // per buffer
    __shared__ u32x4 lds[2 * (kASlots + kBSlots)];       // [buffer][A rows | B rows][slot]

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int m_blk = (int)blockIdx.y * BM;
    const int n_blk = (int)blockIdx.x * BN;
    const int nslabs = (kchunks + kSlabChunks - 1) / kSlabChunks;
    const uint32_t row_bytes = (uint32_t)kchunks * 16u;

    // Global side: a wave-uniform base per operand (it advances by one slab
    // per iteration in scalar registers) plus a 32-bit byte offset per load, so
    // the loop spends no vector instructions on addresses. Thread t's i-th
    // load is row (t + i*NT) / slots, slot (t + i*NT) % slots of the tile.
    // Rows past the matrix edge repeat the last row (their results are never
    // stored).
    const char* a_base = static_cast<const char*>(A) + (size_t)m_blk * row_bytes;
    const char* b_base = static_cast<const char*>(B) + (size_t)n_blk * row_bytes;
    uint32_t a_off[LA], b_off[LB];
    int b_row[LB];                                       // for a BSrc that is not plain rows
    const int my_slot = tid % kSlabChunks;               // NT is a multiple of the slots per row
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        const int row = min((tid + i * NT) / kSlabChunks, M - 1 - m_blk);
        a_off[i] = (uint32_t)row * row_bytes + (uint32_t)my_slot * 16u;
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int row = min((tid + i * NT) / kSlabChunks, N - 1 - n_blk);
        b_off[i] = (uint32_t)row * row_bytes + (uint32_t)my_slot * 16u;
        b_row[i] = n_blk + row;
    }
    // LDS side: the i-th store of a thread lands NT slots after its first (the
    // swizzle term depends on row bits 1..3 only and NT / slots is a multiple
    // of 16 rows).
    const int w_row = tid / kSlabChunks;
    const int w_slot = w_row * kSlabChunks + swz<kSlabChunks * 8>(w_row, my_slot);

    // Two register sets carry the slabs on their way from global memory to
    // LDS when kAhead == 2, so a slab is requested two compute phases before
    // it is needed. kFull (K a multiple of the slab): no predicate on the loads.
    u32x4 ra[kAhead][LA], rb[kAhead][LB];
    const u32x4 zero = {0u, 0u, 0u, 0u};
    auto fetch = [&](auto set_c, int slab) {
        constexpr int set = decltype(set_c)::value;
        const size_t adv = (size_t)slab * (kSlabChunks * 16);
        const bool live = kFull || slab * kSlabChunks + my_slot < kchunks;
#pragma unroll
        for (int i = 0; i < LA; ++i)
            ra[set][i] = live ? *reinterpret_cast<const u32x4*>(a_base + adv + a_off[i]) : zero;
#pragma unroll
        for (int i = 0; i < LB; ++i) {
            if constexpr (BSrc::kPlain)
                rb[set][i] = live ? *reinterpret_cast<const u32x4*>(b_base + adv + b_off[i]) : zero;
            else
                rb[set][i] = live ? bsrc.load(b_row[i], slab * kSlabChunks + my_slot) : zero;
        }
    };
    auto stage = [&](auto set_c, int buf) {
        constexpr int set = decltype(set_c)::value;
        u32x4* dst = lds + buf * (kASlots + kBSlots) + w_slot;
#pragma unroll
        for (int i = 0; i < LA; ++i) dst[i * NT] = ra[set][i];
#pragma unroll
        for (int i = 0; i < LB; ++i) dst[kASlots + i * NT] = rb[set][i];
    };

    Acc acc[TN][TM];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0;

    const int frow = lane & 31;       // operand row inside a 32x32 tile
    const int fhalf = lane >> 5;      // which half of the K step's values
    // Fragment reads: one index per K step (the swizzled slot of this lane's
    // row), the tiles of a wave a constant 32 rows apart.
    int f_idx[kSteps];
#pragma unroll
    for (int step = 0; step < kSteps; ++step)
        f_idx[step] = frow * kSlabChunks + swz<kSlabChunks * 8>(frow, step * 2 + fhalf);
    const int fa_base = wm * TM * 32 * kSlabChunks;
    static_assert(!kPairN || (TN == 2 && BN % 128 == 0), "paired N tiles: two tiles per wave, whole heads per block");
    const int wave_n0 = kPairN ? (wn >> 1) * 128 + (wn & 1) * 32 : wn * TN * 32;      // first column of tile a = 0
    constexpr int kTileStrideN = kPairN ? 64 : 32;
    const int fb_base = kASlots + wave_n0 * kSlabChunks;

    // One slab: the operand fragments of step s + 1 are read from LDS before
    // the MFMAs of step s are issued.
    auto compute = [&](int buf) {
        const u32x4* src = lds + buf * (kASlots + kBSlots);
        u32x4 fw[2][TN], fx[2][TM];
        auto read_frags = [&](auto set_c, int step) {
            constexpr int set = decltype(set_c)::value;
#pragma unroll
            for (int a = 0; a < TN; ++a)
                fw[set][a] = src[fb_base + a * kTileStrideN * kSlabChunks + f_idx[step]];
#pragma unroll
            for (int b = 0; b < TM; ++b)
                fx[set][b] = src[fa_base + b * 32 * kSlabChunks + f_idx[step]];
        };
        read_frags(Const<0>{}, 0);
#pragma unroll
        for (int step = 0; step < kSteps; ++step) {
            if (step + 1 < kSteps) {
                if (step & 1) read_frags(Const<0>{}, step + 1);
                else read_frags(Const<1>{}, step + 1);
            }
            // Keep the instruction scheduler from sinking those reads below the
            // MFMAs that do not need them (it would, to shorten register lifetimes).
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int a = 0; a < TN; ++a)
#pragma unroll
                for (int b = 0; b < TM; ++b)
                    acc[a][b] = Op::mfma(fw[step & 1][a], fx[step & 1][b], acc[a][b]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    fetch(Const<0>{}, 0);
    if constexpr (kAhead == 2) {
        if (nslabs > 1) fetch(Const<1>{}, 1);
        stage(Const<0>{}, 0);
        __syncthreads();
        int slab = 0;
        for (; slab + 2 <= nslabs; slab += 2) {
            if (slab + 2 < nslabs) fetch(Const<0>{}, slab + 2);
            compute(0);
            stage(Const<1>{}, 1);
            __syncthreads();
            if (slab + 3 < nslabs) fetch(Const<1>{}, slab + 3);
            compute(1);
            if (slab + 2 < nslabs) stage(Const<0>{}, 0);
            __syncthreads();
        }
        if (slab < nslabs) compute(0);
    } else {
        stage(Const<0>{}, 0);
        __syncthreads();
        for (int slab = 0; slab < nslabs; ++slab) {
            const int buf = slab & 1;
            if (slab + 1 < nslabs) fetch(Const<0>{}, slab + 1);
            compute(buf);
            if (slab + 1 < nslabs) stage(Const<0>{}, buf ^ 1);
            __syncthreads();
        }
    }

    epi(acc, m_blk + wm * TM * 32, n_blk + wave_n0, frow, fhalf);
}

}  // namespace vv
