// The 256x256 tile with direct global-to-LDS copies, shared by the FP16 GEMM and
// the W8A8 linear layer (both operands K-contiguous, rows of `row_bytes`).
#pragma once

#include "mfma_tile.hpp"

namespace vv {

// The slabs go from global memory STRAIGHT into
// LDS (global_load_lds_dwordx4: each lane's 16 bytes land at M0 + lane * 16, no
// staging registers) and four LDS stages, so a slab is requested three compute
// phases before it is read: deep enough to hide a last-level-cache miss. The
// copy is asynchronous and the compiler is not told about it (it would wait for
// ALL outstanding copies before any LDS read): the wave counts its own copies
// with s_waitcnt vmcnt, then the workgroup barrier makes every wave's part
// visible. Since a lane cannot choose where its bytes land, the bank swizzle is
// applied on the global side: the lane that owns LDS slot (row, p) fetches the
// row's logical slot p ^ swizzle(row). Rows must be whole slabs (no zero fill):
// K % 32 == 0 for FP16, K % 64 == 0 for int8. Op and the epilogue are those of
// mfma_tile; the wave tile is TN x TM = 2 x 4 products of 32 x 32.
constexpr int kDmaStages = 4;
constexpr int kDmaSlabBytes = 64;       // one slab: 64 bytes of every row (32 halves, 64 int8)
constexpr int kDmaTile = 256;
constexpr int kDmaWaves = 8;
constexpr int kDmaStageSlots = 2 * kDmaTile * (kDmaSlabBytes / 16);   // 16-byte slots per stage: A rows, then B rows
constexpr size_t kDmaLdsBytes = (size_t)kDmaStages * kDmaStageSlots * 16;

// One wave-wide copy: lane l's 16 bytes at gptr go to LDS byte lds_byte_addr + 16 l.
__device__ __forceinline__ void lds_dma16(const void* gptr, uint32_t lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(lds_byte_addr), "v"(gptr)
                 : "memory", "m0");
}

// The same copy with the address as a wave-uniform base plus a 32-bit byte offset per lane: the base advances
// in scalar registers, so a loop spends no vector instruction on the addresses.
__device__ __forceinline__ void lds_dma16_at(const void* base, uint32_t lane_offset, uint32_t lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_byte_addr), "v"(lane_offset), "s"(base)
                 : "memory", "m0");
}

// kPairN: a wave's two N tiles are 64 columns apart instead of adjacent - wave wn takes columns
// 128 (wn / 2) + 32 (wn % 2) + {0, 64} of the block - so that an epilogue finds columns n and n + 64
// (the rotate-half pair of a 128-wide head) in the same lane and register of acc[0] and acc[1]. The
// products and their order per output element do not change.
template <typename Op, bool kPairN = false, typename Epi>
__device__ __forceinline__ void mfma_dma(const void* __restrict__ A, const void* __restrict__ B, int M, int N,
                                         int row_bytes, const Epi& epi) {
    typedef typename Op::Acc Acc;
    constexpr int kSlabChunks = kDmaSlabBytes / 16;       // 4
    constexpr int WN = 4, TM = 4, TN = 2;                 // 2 x 4 waves, wave tile 128 (m) x 64 (n)
    constexpr int kLoads = kDmaStageSlots / kWave / kDmaWaves;   // wave-wide copies per wave per slab: 4
    extern __shared__ u32x4 dma_lds[];

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int m_blk = (int)blockIdx.y * kDmaTile;
    const int n_blk = (int)blockIdx.x * kDmaTile;
    const int nslabs = row_bytes / kDmaSlabBytes;
    const uint32_t lds0 =
        (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)dma_lds);

    // Copy i of this wave fills slots (wave + 8i) * 64 .. + 63 of a stage: 16
    // rows x 4 slots. The lane owns (row, physical slot) and fetches the logical
    // slot that the swizzle maps there.
    const char* src[kLoads];
    uint32_t dst[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const int slot0 = (wave + kDmaWaves * i) * kWave;
        const int p = slot0 + lane;
        const int row = p / kSlabChunks, phys = p % kSlabChunks;    // row 0..511: A rows then B rows
        const int logical = swz<32>(row, phys);
        const bool is_b = row >= kDmaTile;
        const int r = is_b ? row - kDmaTile : row;
        const char* base = is_b ? static_cast<const char*>(B) + (size_t)min(n_blk + r, N - 1) * row_bytes
                                : static_cast<const char*>(A) + (size_t)min(m_blk + r, M - 1) * row_bytes;
        src[i] = base + logical * 16;
        dst[i] = lds0 + (uint32_t)slot0 * 16u;
    }
    auto request = [&](int slab) {        // slab -> stage slab % 4; past the end: the last slab again
        const size_t adv = (size_t)min(slab, nslabs - 1) * kDmaSlabBytes;
        const uint32_t stage = (uint32_t)(slab % kDmaStages) * (kDmaStageSlots * 16u);
#pragma unroll
        for (int i = 0; i < kLoads; ++i) lds_dma16(src[i] + adv, dst[i] + stage);
    };

    Acc acc[TN][TM];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0;

    const int frow = lane & 31, fhalf = lane >> 5;
    int f_idx[2];
#pragma unroll
    for (int step = 0; step < 2; ++step)
        f_idx[step] = frow * kSlabChunks + swz<32>(frow, step * 2 + fhalf);
    const int fa_base = wm * TM * 32 * kSlabChunks;
    const int wave_n0 = kPairN ? (wn >> 1) * 128 + (wn & 1) * 32 : wn * TN * 32;      // first column of tile a = 0
    constexpr int kTileStrideN = kPairN ? 64 : 32;
    const int fb_base = kDmaTile * kSlabChunks + wave_n0 * kSlabChunks;

    // Fragment reads run a whole slab ahead: while the 16 MFMAs of slab s execute
    // from one register set, the operands of slab s + 1 come in from LDS into the
    // other (an LDS queue that is two thirds busy answers too late for anything
    // shorter).
    u32x4 fw[2][2][TN], fx[2][2][TM];          // [set][K step][tile]
    auto read_frags = [&](auto set_c, int slab, int step) {
        constexpr int set = decltype(set_c)::value;
        const u32x4* st = dma_lds + (slab % kDmaStages) * kDmaStageSlots;
#pragma unroll
        for (int a = 0; a < TN; ++a)
            fw[set][step][a] = st[fb_base + a * kTileStrideN * kSlabChunks + f_idx[step]];
#pragma unroll
        for (int b = 0; b < TM; ++b)
            fx[set][step][b] = st[fa_base + b * 32 * kSlabChunks + f_idx[step]];
    };
    auto mfma_group = [&](auto set_c, int step) {
        constexpr int set = decltype(set_c)::value;
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int b = 0; b < TM; ++b)
                acc[a][b] = Op::mfma(fw[set][step][a], fx[set][step][b], acc[a][b]);
    };
    // One slab: its operands are (being) loaded in set `cur`; slab + 1 must be in
    // LDS (this wave's copies of slabs + 2 and + 3, 8 of them, may still fly) and
    // every wave must have its operands of this slab in registers before the
    // stage is handed to slab + 4.
    auto one_slab = [&](auto cur_c, auto nxt_c, int slab) {
        asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
        __syncthreads();
        request(slab + 4);
        read_frags(nxt_c, slab + 1, 0);
        __builtin_amdgcn_sched_barrier(0);
        mfma_group(cur_c, 0);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(nxt_c, slab + 1, 1);
        __builtin_amdgcn_sched_barrier(0);
        mfma_group(cur_c, 1);
        __builtin_amdgcn_sched_barrier(0);
    };

    request(0);
    request(1);
    request(2);
    request(3);
    asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    __syncthreads();
    read_frags(Const<0>{}, 0, 0);
    read_frags(Const<0>{}, 0, 1);
    int slab = 0;
    for (; slab + 2 <= nslabs; slab += 2) {
        one_slab(Const<0>{}, Const<1>{}, slab);
        one_slab(Const<1>{}, Const<0>{}, slab + 1);
    }
    if (slab < nslabs) one_slab(Const<0>{}, Const<1>{}, slab);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the surplus copies land before the LDS is released

    epi(acc, m_blk + wm * TM * 32, n_blk + wave_n0, frow, fhalf);
}

// ── The same tile with slabs of 128 bytes per row (K = 64 halves, 128 int8) ──────────────────
// What the measurements on MI355X said about the loop above, and what this one does about it:
//   * A wave issues in order: a block of LDS reads followed by a block of MFMAs leaves the matrix
//     pipe idle during the first and the LDS idle during the second, and both waves of a SIMD do
//     the same thing at the same time (they leave the barrier together). Here every LDS read and
//     every copy request is issued directly behind an MFMA, one per MFMA, in the order in which
//     the next K step first uses the fragments.
//   * A copy of 64 bytes per row touches half a 128-byte cache line; the other half is fetched
//     again for the next slab (the L1 is far too small to keep it). Here a row's whole line comes
//     in one copy: half the requests to L2, half the barriers per MFMA.
//   * Workgroups are handed to the eight XCDs in turn, so in launch order the 32 workgroups that
//     run together on one XCD share one row of tiles and nothing of the other operand. Here an XCD
//     walks whole 4 x 8 blocks of tiles (12 operand tiles per 32 instead of 33), the eight XCDs
//     eight consecutive blocks at a time, so they also read the same operand rows at the same
//     time and share them in the memory-side cache. Only as many blocks as divide by eight are
//     dealt out whole; the tiles of the others and of the ragged right and bottom edges are
//     numbered behind them and cut into eight equal runs, so every XCD has the same number of
//     tiles (whole blocks only leave the same XCDs a round short again and again: 584 against
//     480 tiles at 57 x 74).
//   * The clock is not a constant: under this load the device runs at 1.6-1.8 GHz of its 2.4, and
//     a loop that wastes fewer cycles is answered with a lower clock. What is left to gain is
//     energy per product, not cycles.
// Two stages of 64 KB, two K steps of 32 to a slab. Fragments are read one K step ahead; the
// barrier sits in the last K step of a slab, when every wave has read all of the slab (its last
// step was read during the step before), so the stage is free for the slab after next, whose
// eight copies per wave are issued behind that step's MFMAs and have a whole slab of MFMAs to
// land. Rows must be whole slabs: K % 64 == 0 for FP16. The grid is one-dimensional:
// dma64_grid() workgroups.
// The same loop serves a 128x128 tile (four waves of 64 x 64) for shapes and leftovers that do not fill the
// chip with 256x256 tiles: with two stages (64 KB of LDS) two workgroups share a compute unit, the barrier
// of one hidden behind the other; with four stages a workgroup that has the unit to itself asks for a slab
// three slabs ahead (its slabs are 512 matrix-core cycles long, a copy's way from memory takes four times that).
// And a 64x64 tile (two waves of 32 x 64) for the shapes with too few 128x128 tiles to fill the chip: its slab
// is 16 KB, bound by the copy path (256 clocks) rather than by its 16 MFMAs per wave, so it asks seven slabs
// ahead (eight stages) when a workgroup has the compute unit to itself and three (four stages) otherwise.
constexpr int kDma64SlabBytes = 128;
constexpr int kSuperM = 4, kSuperN = 8;           // tiles per XCD block: 32 workgroups

template <int kTile, int kStages = 2>
struct Dma64Shape {
    static_assert(kTile == 256 || kTile == 128 || kTile == 64, "tile sizes with a schedule");
    static_assert(kStages == 2 || kStages == 4 || kStages == 8, "a slab's stage is slab % kStages");
    // Slabs asked for ahead of the one in hand. With eight stages seven: a wave then has at most 56 copies
    // in flight, which its six-bit counter can still tell apart.
    static constexpr int kAhead = kStages == 8 ? 7 : kStages;
    static constexpr int kWaves = kTile / 32;                     // 2 x 4, 2 x 2 or 2 x 1 waves
    static constexpr int WN = kWaves / 2;
    static constexpr int TM = kTile / 2 / 16, TN = 4;             // wave tile (kTile / 2) x 64 in 16 x 16 products
    static constexpr int kStageSlots = 2 * kTile * (kDma64SlabBytes / 16);   // A rows, then B rows
    static constexpr size_t kLdsBytes = (size_t)kStages * kStageSlots * 16;
    static constexpr int kLoads = kStageSlots / kWave / kWaves;   // wave-wide copies per wave per slab
    static_assert(kLoads == 8, "the copy requests of a slab go behind eight MFMAs of its last K step");
};
constexpr size_t kDma64LdsBytes = Dma64Shape<256>::kLdsBytes;

// The numbering above for a gy x gx grid of tiles. `whole`: tiles per XCD that come in whole blocks;
// `run`: the length of an XCD's run of the remaining `rest` tiles.
struct Dma64Map {
    int gx, gy, fx, fy, whole, run, rest, spare, right;
    __host__ __device__ Dma64Map(int M, int N, int tile) {
        gx = (N + tile - 1) / tile;
        gy = (M + tile - 1) / tile;
        fx = gx / kSuperN;                                // whole blocks per row of blocks
        fy = gy / kSuperM;
        const int blocks = fx * fy;
        whole = (blocks / 8) * (kSuperM * kSuperN);
        spare = (blocks % 8) * (kSuperM * kSuperN);       // tiles of the whole blocks that are not dealt out
        right = gy * (gx - fx * kSuperN);                 // tiles right of the last whole block, every row
        rest = spare + right + (gy - fy * kSuperM) * fx * kSuperN;
        run = (rest + 7) / 8;
    }
    __host__ __device__ unsigned grid() const { return (unsigned)(8 * (whole + run)); }
    // Tile of workgroup `wg` (it runs on XCD wg % 8 as that XCD's (wg / 8)-th); false: none.
    __device__ __forceinline__ bool tile(int wg, int& tile_m, int& tile_n) const {
        const int xcd = wg & 7, nth = wg >> 3;
        int block, within;
        if (nth < whole) {
            block = (nth >> 5) * 8 + xcd;
            within = nth & 31;
        } else {
            int e = xcd * run + (nth - whole);
            if (e >= rest) return false;
            if (e >= spare) {
                e -= spare;
                if (e < right) {
                    const int wr = gx - fx * kSuperN;
                    tile_m = e / wr;
                    tile_n = fx * kSuperN + e % wr;
                } else {
                    e -= right;
                    const int hb = gy - fy * kSuperM;
                    tile_m = fy * kSuperM + e % hb;
                    tile_n = e / hb;
                }
                return true;
            }
            block = (whole >> 5) * 8 + (e >> 5);
            within = e & 31;
        }
        const int block_y = block / fx;
        tile_m = block_y * kSuperM + (within >> 3);
        tile_n = (block - block_y * fx) * kSuperN + (within & 7);
        return true;
    }
};

template <int kTile = 256>
inline unsigned dma64_grid(int M, int N) { return Dma64Map(M, N, kTile).grid(); }

// The wave tile is TN x TM = 4 x 8 (4 x 4 for the 128x128 tile) products of 16 x 16 over K steps of 32
// (Op::mfma16: the 16x16x32 matrix instructions move a fifth fewer register bytes per product than the
// 32x32x16 ones, and under the power limit that is speed: 1.7-1.9 against 1.5-1.6 PFLOP/s for the bare
// instruction streams on random operands). A fragment is 16 rows x 64 bytes: lane l reads slot
// K step * 4 + l / 16 of row l % 16.
//   Op::Acc16                                4-wide accumulator vector
//   Op::mfma16(u32x4 w, u32x4 x, Acc16 c)    one 16x16 product over a K step
//   epi(acc, m0, n0, lane)                   register r of lane l: column n0 + off(a) + 4 (l / 16) + r of row
//                                            m0 + 16 b + l % 16, for acc[a][b]; off(a) = 16 a, or with kPairN = 1
//                                            16 (a % 2) + 64 (a / 2): tiles a and a + 2 are 64 columns apart
// The MFMAs of a step run x tile by x tile, so an x fragment is dead after four MFMAs and the next step's
// takes its registers at once: only the four w fragments and the last two x fragments are held twice.
// kPairN = 2 (256x256 tile only): TWO B operands of N rows each. A tile's 256 B rows are rows n .. n + 127 of B and
// the same rows of B2, and wave wn takes columns 32 wn .. + 31 of both: acc[a] and acc[a + 2] are the products of
// one output column with the two matrices (gate and up of a gated MLP), in the same lane and register. N counts
// the columns of one matrix; a tile covers 128 of them; the epilogue's n0 is the first of the wave's 32.
template <typename Op, int kTile = 256, int kPairN = 0, int kStages = 2, typename Epi>
__device__ __forceinline__ void mfma_dma64(const void* __restrict__ A, const void* __restrict__ B, int M, int N,
                                           int row_bytes, const Epi& epi, const void* __restrict__ B2 = nullptr) {
    static_assert(kPairN != 2 || kTile == 256, "the two-operand layout is the 256x256 tile's");
    constexpr int kTileN = kPairN == 2 ? kTile / 2 : kTile;          // columns of C (of one matrix) per tile
    typedef typename Op::Acc16 Acc;
    typedef Dma64Shape<kTile, kStages> Shape;
    constexpr int kSlabChunks = kDma64SlabBytes / 16;     // 8
    constexpr int WN = Shape::WN, TM = Shape::TM, TN = Shape::TN, kLoads = Shape::kLoads;
    constexpr int kStageSlots = Shape::kStageSlots;
    extern __shared__ u32x4 dma_lds[];

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const Dma64Map map(M, kPairN == 2 ? 2 * N : N, kTile);
    int tile_m, tile_n;
    if (!map.tile((int)blockIdx.x, tile_m, tile_n)) return;      // the whole workgroup, before any barrier
    const int m_blk = tile_m * kTile, n_blk = tile_n * kTileN;
    const int nslabs = row_bytes / kDma64SlabBytes;
    const uint32_t lds0 =
        (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)dma_lds);

    // Copy i of this wave fills slots (wave + waves * i) * 64 .. + 63 of a stage: 8 rows x 8 slots, a whole
    // line per row; copies 0 .. 3 are A rows, 4 .. 7 B rows. The lane owns (row, physical slot) and fetches the
    // logical slot that the swizzle maps there: a byte offset from the tile's first row, the same for every slab.
    const char* a_tile = static_cast<const char*>(A) + (size_t)m_blk * row_bytes;
    const char* b_tile = static_cast<const char*>(B) + (size_t)n_blk * row_bytes;
    const char* b2_tile = kPairN == 2 ? static_cast<const char*>(B2) + (size_t)n_blk * row_bytes : b_tile;
    uint32_t src[kLoads], dst[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const int slot0 = (wave + Shape::kWaves * i) * kWave;
        const int p = slot0 + lane;
        const int row = p / kSlabChunks, phys = p % kSlabChunks;
        const int logical = swz<64>(row, phys);
        // two operands: the B rows of copies 4, 5 are rows 0 .. 127 of B's tile, those of copies 6, 7 of B2's
        const int b_row = kPairN == 2 ? (row - kTile) % kTileN : row - kTile;
        const int r = i < kLoads / 2 ? min(row, M - 1 - m_blk) : min(b_row, N - 1 - n_blk);
        src[i] = (uint32_t)r * (uint32_t)row_bytes + (uint32_t)logical * 16u;
        dst[i] = lds0 + (uint32_t)slot0 * 16u;
    }
    auto request = [&](int slab, int i) {        // slab -> stage slab % kStages; past the end: the last slab again
        const size_t adv = (size_t)min(slab, nslabs - 1) * kDma64SlabBytes;
        const uint32_t stage = (uint32_t)(slab & (kStages - 1)) * (kStageSlots * 16u);
        const char* tile = i < kLoads / 2 ? a_tile : (kPairN == 2 && i >= 3 * kLoads / 4) ? b2_tile : b_tile;
        lds_dma16_at(tile + adv, src[i], dst[i] + stage);
    };

    Acc acc[TN][TM];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[a][b][r] = 0;

    const int frow = lane & 15, fquarter = lane >> 4;
    int f_idx[2];
#pragma unroll
    for (int step = 0; step < 2; ++step)
        f_idx[step] = frow * kSlabChunks + swz<64>(frow, step * 4 + fquarter);
    const int fa_base = wm * TM * 16 * kSlabChunks;
    // first B row of the wave's tile a = 0, and tile a's distance from it
    const int wave_n0 = kPairN == 2 ? wn * 32 : kPairN == 1 ? (wn >> 1) * 128 + (wn & 1) * 32 : wn * TN * 16;
    const int fb_base = kTile * kSlabChunks + wave_n0 * kSlabChunks;
    auto w_off = [](int a) {
        return (kPairN == 2 ? (a & 1) * 16 + (a >> 1) * 128 : kPairN == 1 ? (a & 1) * 16 + (a >> 1) * 64 : a * 16) *
               kSlabChunks;
    };

    // w: the K step in hand and the next. x: one set, refilled in place, except the last two tiles of a step,
    // which are held twice like w (their refill could only follow the step's last MFMAs, and the reads of a
    // step must be back when the next begins).
    constexpr int kSingle = TM - 2;
    u32x4 fw[2][TN], fx[kSingle > 0 ? kSingle : 1], fxl[2][TM - kSingle];
    auto read_w = [&](auto set_c, int slab, int step, int a) {
        constexpr int set = decltype(set_c)::value;
        fw[set][a] = dma_lds[(slab & (kStages - 1)) * kStageSlots + fb_base + w_off(a) + f_idx[step]];
    };
    auto read_x = [&](auto set_c, int slab, int step, int b) {
        constexpr int set = decltype(set_c)::value;
        const u32x4 v = dma_lds[(slab & (kStages - 1)) * kStageSlots + fa_base + b * 16 * kSlabChunks + f_idx[step]];
        if (b < kSingle) fx[b] = v;
        else fxl[set][b - kSingle] = v;
    };
    // One K step: TM x 4 MFMAs, x tile by x tile. Reads and copy requests go behind MFMAs; the
    // next step's x fragment b < TM - 2 can go anywhere behind the last MFMA of x tile b (it takes that
    // fragment's registers). Step 0 reads step 1 of the same slab. In step 1, behind the barrier, every wave
    // has read all of this slab and the next slab has landed (this wave's copies; the barrier adds the
    // others'): then come the eight copy requests of the slab after next into the stage just freed, behind
    // the first eight MFMAs, and with them the reads of the next slab's step 0. The last read of a step is
    // eight MFMAs from its end. With 32 MFMAs to
    // a step, step 1 issues eight before the barrier, so that the last read of step 0 is back when the wave
    // gets there; with 16 the barrier comes first and the other workgroup of the compute unit fills the wait.
    auto k_step = [&](auto cur_c, auto nxt_c, int slab, auto step_c) {
        constexpr int set = decltype(cur_c)::value;
        constexpr int step = decltype(step_c)::value;
        constexpr int nstep = step ^ 1;
        constexpr int kBefore = TM == 8 ? 2 : 0;                   // x tiles of step 1 ahead of the barrier
        const int nslab = slab + step;
#pragma unroll
        for (int b = 0; b < TM; ++b) {
#pragma unroll
            for (int a = 0; a < TN; ++a) {
                if (step == 1 && b == kBefore && a == 0) {
                    // this wave's copies of the next slab are in: only those of the slabs behind it may still fly
                    if constexpr (Shape::kAhead == 2) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                    else if constexpr (Shape::kAhead == 4) asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)" ::: "memory");
                    else asm volatile("s_waitcnt vmcnt(40) lgkmcnt(0)" ::: "memory");
                    __syncthreads();
                }
                __builtin_amdgcn_sched_barrier(0);
                acc[a][b] = Op::mfma16(fw[set][a], b < kSingle ? fx[b] : fxl[set][b - kSingle], acc[a][b]);
                __builtin_amdgcn_sched_barrier(0);
                const int slot = (b - kBefore * step) * TN + a;    // step 1: counted from the barrier
                if constexpr (step == 1) {
                    // the copies first: their way from memory is longer than the slab they have to make it in
                    if (slot >= 0 && slot < kLoads) request(slab + Shape::kAhead, slot);
                }
                if constexpr (TM == 8) {
                    if (slot == 0) read_w(nxt_c, nslab, nstep, 0);
                    else if (slot == 1) read_x(nxt_c, nslab, nstep, step == 0 ? 6 : 0);
                    else if (slot == 2) read_w(nxt_c, nslab, nstep, 1);
                    else if (slot == 3) read_x(nxt_c, nslab, nstep, step == 0 ? 0 : 2);
                    else if (slot == 4) read_w(nxt_c, nslab, nstep, 2);
                    else if (slot == 5) read_w(nxt_c, nslab, nstep, 3);
                    else if (slot == 6) read_x(nxt_c, nslab, nstep, step == 0 ? 7 : 1);
                    else if (slot == 7) read_x(nxt_c, nslab, nstep, step == 0 ? 1 : 3);
                    else if (slot == 8 && step == 1) read_x(nxt_c, nslab, nstep, 6);
                    else if (slot == 9 && step == 1) read_x(nxt_c, nslab, nstep, 7);
                    else if (slot == 11) read_x(nxt_c, nslab, nstep, step == 0 ? 2 : 4);
                    else if (slot == 15) read_x(nxt_c, nslab, nstep, step == 0 ? 3 : 5);
                    else if (slot == 19 && step == 0) read_x(nxt_c, nslab, nstep, 4);
                    else if (slot == 23 && step == 0) read_x(nxt_c, nslab, nstep, 5);
                } else if constexpr (TM == 4) {
                    if (slot == 0) read_w(nxt_c, nslab, nstep, 0);
                    else if (slot == 1) read_w(nxt_c, nslab, nstep, 1);
                    else if (slot == 2) read_w(nxt_c, nslab, nstep, 2);
                    else if (slot == 3) read_x(nxt_c, nslab, nstep, 0);
                    else if (slot == 4) read_w(nxt_c, nslab, nstep, 3);
                    else if (slot == 5) read_x(nxt_c, nslab, nstep, 2);
                    else if (slot == 6) read_x(nxt_c, nslab, nstep, 3);
                    else if (slot == 7) read_x(nxt_c, nslab, nstep, 1);
                } else {                                           // TM == 2: both x fragments are held twice
                    if (slot < 4) read_w(nxt_c, nslab, nstep, slot);
                    else if (slot < 6) read_x(nxt_c, nslab, nstep, slot - 4);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };

#pragma unroll
    for (int s = 0; s < Shape::kAhead; ++s)
#pragma unroll
        for (int i = 0; i < kLoads; ++i) request(s, i);
    // slab 0; slab 1 is waited for at the first barrier
    if constexpr (Shape::kAhead == 2) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else if constexpr (Shape::kAhead == 4) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(48)" ::: "memory");
    __syncthreads();
#pragma unroll
    for (int a = 0; a < TN; ++a) read_w(Const<0>{}, 0, 0, a);
#pragma unroll
    for (int b = 0; b < TM; ++b) read_x(Const<0>{}, 0, 0, b);
    for (int slab = 0; slab < nslabs; ++slab) {
        k_step(Const<0>{}, Const<1>{}, slab, Const<0>{});
        k_step(Const<1>{}, Const<0>{}, slab, Const<1>{});
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // the surplus copies and reads land before the LDS is released

    epi(acc, m_blk + wm * TM * 16, n_blk + wave_n0, lane);
}

// ── The q, k and v projections of a chunk of rows in ONE grid of equal tiles ─────────────────
// A decoder with 7 query heads per KV head of 128 channels (28 + 4 heads: 3584 + 512 + 512 output columns)
// has as many q and k heads, 32, as v has 16-column strips: a tile is 128 rows x (one head of q or k + one
// strip of v) = 128 x 144 outputs, and 2048 rows are 16 x 32 = 512 equal tiles - one full round of two
// workgroups per compute unit, where 128 x 128 tiles over the 4608 columns would be 576 (a round and an
// eighth). The loop is mfma_dma64's for the 128 x 128 tile (four waves of 64 x 64, kPairN = 1: a head's columns
// n and n + 64 in one lane) with a ninth copy per slab for the 16 v rows (waves 0 and 1 issue it), one more
// fragment read and two more MFMAs per K step and wave: the strip's eight 16 x 16 products go two to a wave,
// against the x fragments b = 0, 1 of the step - wave wn numbers its four row tiles from 2 wn (row tile
// (b + 2 wn) % 4 is its b-th), so that the two waves that share rows take different halves of the strip
// and the schedule needs no branch. Every output element adds K in mfma_dma64's order.
//   epi(acc, accv, m0, wn, lane)   acc[a][b]: as mfma_dma64 with kPairN = 1, row m0 + 16 ((b + 2 wn) % 4) + l % 16;
//                                  accv[j]: v column 4 (l / 16) + r of the strip, row m0 + 16 ((j + 2 wn) % 4) + l % 16
constexpr int kQkvStrip = 16;                                  // v columns per tile
template <int kStages>
struct QkvShape {
    static_assert(kStages == 2 || kStages == 4, "a slab's stage is slab % kStages");
    static constexpr int kAhead = kStages;
    static constexpr int kWaves = 4;
    static constexpr int kStageSlots = (128 + 128 + kQkvStrip) * (kDma64SlabBytes / 16);   // x rows, head rows, v rows
    static constexpr size_t kLdsBytes = (size_t)kStages * kStageSlots * 16;
};

// x: the tile's first row (rows_left of them exist); w_head: the head's 128 weight rows; w_strip: the strip's 16.
template <typename Op, int kStages, typename Epi>
__device__ __forceinline__ void mfma_dma64_qkv(const char* __restrict__ x, const char* __restrict__ w_head,
                                               const char* __restrict__ w_strip, int rows_left, int row_bytes,
                                               const Epi& epi) {
    typedef typename Op::Acc16 Acc;
    typedef QkvShape<kStages> Shape;
    constexpr int kSlabChunks = kDma64SlabBytes / 16;     // 8
    constexpr int WN = 2, TM = 4, TN = 4, kLoads = 8;
    constexpr int kStageSlots = Shape::kStageSlots;
    extern __shared__ u32x4 dma_lds[];

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const bool strip_wave = wave < 2;                     // the waves that copy the strip's rows
    const int nslabs = row_bytes / kDma64SlabBytes;
    const uint32_t lds0 =
        (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)dma_lds);

    // Copies 0 .. 3 of a wave are x rows, 4 .. 7 head rows (8 rows x 8 slots each, as in mfma_dma64); copy 8 of
    // waves 0 and 1 is eight rows of the strip.
    uint32_t src[kLoads + 1], dst[kLoads + 1];
#pragma unroll
    for (int i = 0; i <= kLoads; ++i) {
        const int slot0 = (wave + Shape::kWaves * i) * kWave;
        const int p = slot0 + lane;
        const int row = p / kSlabChunks, phys = p % kSlabChunks;
        const int logical = swz<64>(row, phys);
        const int r = i < kLoads / 2 ? min(row, rows_left - 1) : i < kLoads ? row - 128 : row - 256;
        src[i] = (uint32_t)r * (uint32_t)row_bytes + (uint32_t)logical * 16u;
        dst[i] = lds0 + (uint32_t)slot0 * 16u;
    }
    auto request = [&](int slab, int i) {        // slab -> stage slab % kStages; past the end: the last slab again
        const size_t adv = (size_t)min(slab, nslabs - 1) * kDma64SlabBytes;
        const uint32_t stage = (uint32_t)(slab & (kStages - 1)) * (kStageSlots * 16u);
        const char* tile = i < kLoads / 2 ? x : i < kLoads ? w_head : w_strip;
        lds_dma16_at(tile + adv, src[i], dst[i] + stage);
    };

    Acc acc[TN][TM], accv[2];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int b = 0; b < TM; ++b) acc[a][b][r] = 0;
        accv[0][r] = accv[1][r] = 0;
    }

    const int frow = lane & 15, fquarter = lane >> 4;
    int f_idx[2];
#pragma unroll
    for (int step = 0; step < 2; ++step)
        f_idx[step] = frow * kSlabChunks + swz<64>(frow, step * 4 + fquarter);
    int x_off[TM];                                        // the wave's b-th row tile is tile (b + 2 wn) % 4 of its 64 rows
#pragma unroll
    for (int b = 0; b < TM; ++b) x_off[b] = (wm * TM + ((b + 2 * wn) & 3)) * 16 * kSlabChunks;
    const int fb_base = 128 * kSlabChunks + wn * 32 * kSlabChunks;
    constexpr int kStripBase = 256 * kSlabChunks;
    auto w_off = [](int a) { return ((a & 1) * 16 + (a >> 1) * 64) * kSlabChunks; };

    // w and the strip fragment: the K step in hand and the next. x: tiles 0, 1 one set, refilled in place behind
    // their last MFMA; tiles 2, 3 held twice.
    u32x4 fw[2][TN], fv[2], fx[2], fxl[2][2];
    auto read_w = [&](auto set_c, int slab, int step, int a) {
        constexpr int set = decltype(set_c)::value;
        fw[set][a] = dma_lds[(slab & (kStages - 1)) * kStageSlots + fb_base + w_off(a) + f_idx[step]];
    };
    auto read_v = [&](auto set_c, int slab, int step) {
        constexpr int set = decltype(set_c)::value;
        fv[set] = dma_lds[(slab & (kStages - 1)) * kStageSlots + kStripBase + f_idx[step]];
    };
    auto read_x = [&](auto set_c, int slab, int step, int b) {
        constexpr int set = decltype(set_c)::value;
        const u32x4 v = dma_lds[(slab & (kStages - 1)) * kStageSlots + x_off[b] + f_idx[step]];
        if (b < 2) fx[b] = v;
        else fxl[set][b - 2] = v;
    };
    // One K step: 18 MFMAs, x tile by x tile (tiles 0 and 1: four head products and the strip's). The reads of the
    // next step and, in step 1 behind the barrier, the copy requests of the slab after next go one behind each MFMA.
    auto k_step = [&](auto cur_c, auto nxt_c, int slab, auto step_c) {
        constexpr int set = decltype(cur_c)::value;
        constexpr int step = decltype(step_c)::value;
        constexpr int nstep = step ^ 1;
        const int nslab = slab + step;
#pragma unroll
        for (int b = 0; b < TM; ++b) {
#pragma unroll
            for (int a = 0; a < (b < 2 ? TN + 1 : TN); ++a) {
                if (step == 1 && b == 0 && a == 0) {
                    // this wave's copies of the next slab are in: only those of the slabs behind it may still fly
                    if constexpr (Shape::kAhead == 2) {
                        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                    } else {
                        if (strip_wave) asm volatile("s_waitcnt vmcnt(18) lgkmcnt(0)" ::: "memory");
                        else asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)" ::: "memory");
                    }
                    __syncthreads();
                }
                __builtin_amdgcn_sched_barrier(0);
                const u32x4 xf = b < 2 ? fx[b] : fxl[set][b - 2];
                if (a < TN) acc[a][b] = Op::mfma16(fw[set][a], xf, acc[a][b]);
                else accv[b] = Op::mfma16(fv[set], xf, accv[b]);
                __builtin_amdgcn_sched_barrier(0);
                const int slot = b < 2 ? b * (TN + 1) + a : 2 * (TN + 1) + (b - 2) * TN + a;
                if constexpr (step == 1) {
                    if (slot < kLoads) request(slab + Shape::kAhead, slot);
                    else if (slot == kLoads && strip_wave) request(slab + Shape::kAhead, kLoads);
                }
                if (slot < 4) read_w(nxt_c, nslab, nstep, slot);
                else if (slot == 4) read_x(nxt_c, nslab, nstep, 0);
                else if (slot == 5) read_v(nxt_c, nslab, nstep);
                else if (slot == 6) read_x(nxt_c, nslab, nstep, 2);
                else if (slot == 7) read_x(nxt_c, nslab, nstep, 3);
                else if (slot == 9) read_x(nxt_c, nslab, nstep, 1);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };

#pragma unroll
    for (int s = 0; s < Shape::kAhead; ++s) {
#pragma unroll
        for (int i = 0; i < kLoads; ++i) request(s, i);
        if (strip_wave) request(s, kLoads);
    }
    // slab 0; slab 1 is waited for at the first barrier
    if constexpr (Shape::kAhead == 2) {
        if (strip_wave) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    } else {
        if (strip_wave) asm volatile("s_waitcnt vmcnt(27)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < TN; ++a) read_w(Const<0>{}, 0, 0, a);
    read_v(Const<0>{}, 0, 0);
#pragma unroll
    for (int b = 0; b < TM; ++b) read_x(Const<0>{}, 0, 0, b);
    for (int slab = 0; slab < nslabs; ++slab) {
        k_step(Const<0>{}, Const<1>{}, slab, Const<0>{});
        k_step(Const<1>{}, Const<0>{}, slab, Const<1>{});
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // the surplus copies and reads land before the LDS is released

    epi(acc, accv, wm * TM * 16, wn, lane);
}

}  // namespace vv
