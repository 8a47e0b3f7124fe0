// W4A16 linear layers: FP16 activations against 4-bit group-affine weight codes
// in the accelerator layout of the INT4 weights (every 16-byte chunk = 32
// consecutive columns; nibble slot s of 32-bit word t = column
// 2 (t + 4 (s % 4)) + s / 4), with half2 {scale, zero point} per group of 32,
// 64, 128 or 256 columns.
//
// Every kernel dequantises with the one formula the interface states,
// w = (q - z) * s rounded once to FP16: `(w >> 4j) & 0x000F000F | 0x64006400`
// is the half2 {1024 + code of slot j, 1024 + code of slot j + 4}, i.e. the
// column pair t + 4j; subtracting 1024 + z is exact, and the multiply by the
// scale is the rounding. Accumulation is FP32.
//   w4a16_dequant   codes -> dense FP16 [N][K]
//   w4a16_gemv      M <= 4: lanes take whole chunks, v_dot2_f32_f16 against the
//                   natural half2 pairs of x; K split over waves or several
//                   rows per wave by shape; up to three projections per launch
//   w4a16_skinny    5 <= M <= 64: codes dequantised in registers into 16x16x32
//                   MFMA operands, K split over the eight waves of a workgroup
//   w4a16_tile      larger M: the LDS-tiled 32x32x16 FP16 MFMA loop with the
//                   codes dequantised on their way into LDS
//   w4a16_gather    out[m][j] = x[m][perm[j]] (act-order checkpoints)
#include "mfma_tile.hpp"

namespace vv {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef h16 h16x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

struct GroupConst { h16x2 scale, offset; };    // {s, s} and {1024 + z, 1024 + z}

__device__ __forceinline__ GroupConst group_const(uint32_t sz) {
    const h16 s = __builtin_bit_cast(h16, (uint16_t)(sz & 0xFFFFu));
    const h16 z = __builtin_bit_cast(h16, (uint16_t)(sz >> 16));
    GroupConst g;
    g.scale = h16x2{s, s};
    const h16 off = (h16)1024.0f + z;          // exact: integers up to 2048 are FP16 values
    g.offset = h16x2{off, off};
    return g;
}

// The weights of column pair t + 4j of a chunk, from word t of its codes.
__device__ __forceinline__ h16x2 dequant_pair(uint32_t word, int j, const GroupConst& g) {
    const uint32_t bits = ((word >> (4 * j)) & 0x000F000Fu) | 0x64006400u;
    const h16x2 centred = __builtin_bit_cast(h16x2, bits) - g.offset;    // q - z, exact
    return centred * g.scale;
}

// The chunk's four 16-byte slots in column order: slot j = columns 8j .. 8j + 7
// = pairs 4j .. 4j + 3 = slot j / j + 4 of words 0 .. 3.
__device__ __forceinline__ void dequant_chunk(const u32x4& codes, const GroupConst& g, u32x4 (&slots)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int t = 0; t < 4; ++t) slots[j][t] = __builtin_bit_cast(uint32_t, dequant_pair(codes[t], j, g));
}

__global__ __launch_bounds__(kBlock) void w4a16_dequant(const u32x4* __restrict__ packed,
                                                        const uint32_t* __restrict__ sz,
                                                        u32x4* __restrict__ out, size_t nchunks_total,
                                                        int chunks_per_row, int groups_per_row, int gshift) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= nchunks_total) return;
    const size_t n = i / (size_t)chunks_per_row;
    const int c = (int)(i - n * chunks_per_row);
    const GroupConst g = group_const(sz[n * groups_per_row + ((c * 32) >> gshift)]);
    u32x4 slots[4];
    dequant_chunk(packed[i], g, slots);
#pragma unroll
    for (int j = 0; j < 4; ++j) out[i * 4 + j] = slots[j];
}

__global__ __launch_bounds__(kBlock) void w4a16_gather(const h16* __restrict__ x, const int32_t* __restrict__ perm,
                                                       h16* __restrict__ out, int M, int K) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;       // one run of 8 outputs
    const int per_row = K / 8;
    if (i >= (size_t)M * per_row) return;
    const size_t m = i / (size_t)per_row;
    const int j = (int)(i - m * per_row) * 8;
    const i32x4 p0 = *reinterpret_cast<const i32x4*>(perm + j), p1 = *reinterpret_cast<const i32x4*>(perm + j + 4);
    const h16* row = x + m * K;
    h16x8 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) { v[e] = row[p0[e]]; v[4 + e] = row[p1[e]]; }
    *reinterpret_cast<h16x8*>(out + m * K + j) = v;
}

// c[m][n] = bias[n]: the starting value of a GEMM that adds into C, so that the bias
// joins the FP32 sum before the one rounding of the output.
__global__ __launch_bounds__(kBlock) void bias_rows(const h16* __restrict__ bias, h16* __restrict__ c, int M, int N) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;       // one run of 8 outputs (N % 8 == 0)
    const int per_row = N / 8;
    if (i >= (size_t)M * per_row) return;
    const int j = (int)(i % (size_t)per_row) * 8;
    *reinterpret_cast<h16x8*>(c + (i / (size_t)per_row) * N + j) = *reinterpret_cast<const h16x8*>(bias + j);
}

// ── M <= 4 (and the fused single-row launches) ─────────────────────────────────────────────────────────────────
constexpr int kMaxSegs = 3;

struct GemvSegs {
    const u32x4* w[kMaxSegs];
    const uint32_t* sz[kMaxSegs];
    const h16* bias[kMaxSegs];
    h16* y[kMaxSegs];
    int n[kMaxSegs];
    int first[kMaxSegs + 1];     // first workgroup of each projection
};

// kSplit waves share RW weight rows: wave p takes the rounds of 64 chunks p,
// p + kSplit, ..., lane l chunk l of the round. Workgroups never straddle two
// projections.
template <int MR, int kSplit, int RW>
__global__ __launch_bounds__(kBlock) void w4a16_gemv(const h16* __restrict__ x, GemvSegs segs, int M, int K,
                                                     int gshift) {
    constexpr int kRows = kWavesPerBlock / kSplit * RW;
    __shared__ float part[kWavesPerBlock][RW][MR];
    const int wave = wave_in_block(), lane = lane_id();
    const int set = wave / kSplit, piece = wave % kSplit;
    const int b = (int)blockIdx.x;
    const int seg = (b >= segs.first[1] ? 1 : 0) + (b >= segs.first[2] ? 1 : 0);
    const int N = segs.n[seg];
    const int n0 = (b - segs.first[seg]) * kRows + set * RW;
    const int nchunks = K / 32, ng = K >> gshift;
    const u32x4* wrow[RW];
    const uint32_t* szrow[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        const int row = min(n0 + r, N - 1);
        wrow[r] = segs.w[seg] + (size_t)row * nchunks;
        szrow[r] = segs.sz[seg] + (size_t)row * ng;
    }
    float acc[RW][MR];
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[r][m] = 0.0f;

#pragma unroll 2
    for (int base = piece * kWave; base < nchunks; base += kSplit * kWave) {
        const bool live = base + lane < nchunks;
        const int c = live ? base + lane : nchunks - 1;
        const int g = (c * 32) >> gshift;
        h16x2 wv[RW][16];                        // wv[r][p]: columns 2p, 2p + 1 of the chunk
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            const u32x4 codes = __builtin_nontemporal_load(wrow[r] + c);
            const GroupConst gc = group_const(szrow[r][g]);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int t = 0; t < 4; ++t) wv[r][t + 4 * j] = dequant_pair(codes[t], j, gc);
        }
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            if (m < M && live) {
                const u32x4* xr = reinterpret_cast<const u32x4*>(x + (size_t)m * K) + 4 * c;
                uint32_t xw[16];                 // xw[p]: columns 2p, 2p + 1 of the chunk
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const u32x4 v = xr[q];
                    xw[4 * q] = v.x;
                    xw[4 * q + 1] = v.y;
                    xw[4 * q + 2] = v.z;
                    xw[4 * q + 3] = v.w;
                }
#pragma unroll
                for (int r = 0; r < RW; ++r)
#pragma unroll
                    for (int p = 0; p < 16; ++p)
                        acc[r][m] = __builtin_amdgcn_fdot2(wv[r][p], __builtin_bit_cast(h16x2, xw[p]), acc[r][m],
                                                           false);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[r][m] = wave_sum(acc[r][m]);
    if constexpr (kSplit > 1) {
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < RW; ++r)
#pragma unroll
                for (int m = 0; m < MR; ++m) part[wave][r][m] = acc[r][m];
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < RW; ++r)
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                float sum = 0.0f;
#pragma unroll
                for (int p = 0; p < kSplit; ++p) sum += part[set * kSplit + p][r][m];
                acc[r][m] = sum;
            }
    }
    if (piece == 0) {
        float mine = 0.0f;
#pragma unroll
        for (int r = 0; r < RW; ++r)
#pragma unroll
            for (int m = 0; m < MR; ++m)
                if (lane == r * MR + m) mine = acc[r][m];
        const int r = lane / MR, m = lane % MR;
        if (lane < RW * MR && m < M && n0 + r < N) {
            const int n = n0 + r;
            if (segs.bias[seg]) mine += (float)segs.bias[seg][n];
            segs.y[seg][(size_t)m * N + n] = to_half(mine);
        }
    }
}

template <int MR, int kSplit, int RW>
void launch_gemv_cfg(const h16* x, GemvSegs segs, int n_segs, int M, int K, int gshift, hipStream_t st) {
    constexpr int kRows = kWavesPerBlock / kSplit * RW;
    int blocks = 0;
    for (int i = 0; i <= kMaxSegs; ++i) {
        segs.first[i] = i <= n_segs ? blocks : 0x7FFFFFFF;
        if (i < n_segs) blocks += (segs.n[i] + kRows - 1) / kRows;
    }
    for (int i = n_segs; i < kMaxSegs; ++i) { segs.w[i] = segs.w[0]; segs.sz[i] = segs.sz[0]; segs.n[i] = 1; }
    w4a16_gemv<MR, kSplit, RW><<<dim3((unsigned)blocks), kBlock, 0, st>>>(x, segs, M, K, gshift);
}

template <int MR>
void launch_gemv(const h16* x, const GemvSegs& segs, int n_segs, int M, int K, int gshift, hipStream_t st) {
    long rows = 0;
    for (int i = 0; i < n_segs; ++i) rows += segs.n[i];
    const int nchunks = K / 32;
    // Thousands of waves in flight, and no wave with less than half a round of chunks.
    int split = 1, rw = 1;
    while (split < 4 && rows * split < 4096 && nchunks / (2 * split) >= kWave / 2) split *= 2;
    while (split == 1 && rw < 4 && rows / (2 * rw) >= 8192 && K * rw <= 8192 && MR * rw * 2 <= 8) rw *= 2;
    if constexpr (MR <= 2) {
        if (rw == 4) return launch_gemv_cfg<MR, 1, 4>(x, segs, n_segs, M, K, gshift, st);
    }
    if constexpr (MR <= 4) {
        if (rw >= 2) return launch_gemv_cfg<MR, 1, 2>(x, segs, n_segs, M, K, gshift, st);
    }
    if (split == 1) launch_gemv_cfg<MR, 1, 1>(x, segs, n_segs, M, K, gshift, st);
    else if (split == 2) launch_gemv_cfg<MR, 2, 1>(x, segs, n_segs, M, K, gshift, st);
    else launch_gemv_cfg<MR, 4, 1>(x, segs, n_segs, M, K, gshift, st);
}

void launch_gemv_rows(const h16* x, const GemvSegs& segs, int n_segs, int M, int K, int gshift, hipStream_t st) {
    if (M == 1) launch_gemv<1>(x, segs, n_segs, M, K, gshift, st);
    else if (M == 2) launch_gemv<2>(x, segs, n_segs, M, K, gshift, st);
    else if (M <= 4) launch_gemv<4>(x, segs, n_segs, M, K, gshift, st);
    else launch_gemv<8>(x, segs, n_segs, M, K, gshift, st);
}

struct TileArgs {
    const h16* a;            // [M][K]
    const u32x4* packed;     // [N][K/32] chunks
    const uint32_t* sz;      // [N][K >> gshift]
    const h16* bias;
    h16* c;                  // [M][N]
    int M, N, K, gshift, vec;
};

// ── 5 <= M <= 64 ───────────────────────────────────────────────────────────
// Sixteen or 32 weight rows per workgroup, K split over its eight waves, the
// codes dequantised in registers into 16x16x32 MFMA operands: one chunk of
// codes is one K step, lane (row, q) dequantises the chunk's q-th run of eight
// columns (four half2 from the four words) and meets the same eight columns of
// up to 64 activation rows. Every chunk is loaded from global memory once (by
// one lane of the four that need it) and passed round through LDS; the waves'
// partial tiles are added at the end. Every workgroup reads all the
// activations, which is most of the L2 traffic from 16 rows on.
constexpr int kSkinnyWaves = 8;

template <int kMT, int kNT>
__global__ __launch_bounds__(kSkinnyWaves * kWave) void w4a16_skinny(TileArgs a) {
    __shared__ f32x4 part[kSkinnyWaves][kMT * kNT][kWave];
    __shared__ u32x4 staged[kSkinnyWaves][kNT][kWave];      // a wave's own 16 rows x 4 chunks of codes per tile
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, ks = lane >> 4;
    const int n0 = (int)blockIdx.x * (16 * kNT);
    const int ncodes = a.K / 32, ng = a.K >> a.gshift;
    // The four lanes of an operand row would each load the row's whole chunk for a quarter of its bits;
    // instead lane l loads chunk l % 4 of row l / 4 once (64 bytes of a row side by side) and the wave
    // hands the chunks round through its piece of LDS, which serves a wave's accesses in order.
    const uint32_t* szrow[kNT];
    const u32x4* lrow[kNT];
#pragma unroll
    for (int j = 0; j < kNT; ++j) {
        szrow[j] = a.sz + (size_t)min(n0 + 16 * j + r16, a.N - 1) * ng;
        lrow[j] = a.packed + (size_t)min(n0 + 16 * j + (lane >> 2), a.N - 1) * ncodes;
    }
    const int put = (lane >> 2) * 4 + swz<32>(lane >> 2, lane & 3);
    const bool one_group = a.gshift >= 7;               // the four chunks of a step share their scale
    const u32x4* arow[kMT];
#pragma unroll
    for (int t = 0; t < kMT; ++t)
        arow[t] = reinterpret_cast<const u32x4*>(a.a + (size_t)min(16 * t + r16, a.M - 1) * a.K);
    const u32x4 zero = {0u, 0u, 0u, 0u};
    f32x4 acc[kMT][kNT];
#pragma unroll
    for (int t = 0; t < kMT; ++t)
#pragma unroll
        for (int j = 0; j < kNT; ++j) acc[t][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    for (int c0 = wave * 4; c0 < ncodes; c0 += kSkinnyWaves * 4) {
        u32x4 mine[kNT], x[kMT][4];
        uint32_t gsz[kNT][4];
#pragma unroll
        for (int j = 0; j < kNT; ++j) {
            mine[j] = __builtin_nontemporal_load(lrow[j] + min(c0 + (lane & 3), ncodes - 1));
            if (one_group) gsz[j][0] = szrow[j][(c0 * 32) >> a.gshift];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const bool live = c0 + u < ncodes;
            const int c = live ? c0 + u : ncodes - 1;
#pragma unroll
            for (int j = 0; j < kNT; ++j) gsz[j][u] = one_group ? gsz[j][0] : szrow[j][(c * 32) >> a.gshift];
#pragma unroll
            for (int t = 0; t < kMT; ++t) x[t][u] = live ? arow[t][c * 4 + ks] : zero;   // a dead step adds zero
        }
#pragma unroll
        for (int j = 0; j < kNT; ++j) staged[wave][j][put] = mine[j];
#pragma unroll
        for (int j = 0; j < kNT; ++j)
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const u32x4 codes = staged[wave][j][r16 * 4 + swz<32>(r16, u)];
                const GroupConst gc = group_const(gsz[j][u]);
                u32x4 w;
                w.x = __builtin_bit_cast(uint32_t, dequant_pair(codes.x, ks, gc));
                w.y = __builtin_bit_cast(uint32_t, dequant_pair(codes.y, ks, gc));
                w.z = __builtin_bit_cast(uint32_t, dequant_pair(codes.z, ks, gc));
                w.w = __builtin_bit_cast(uint32_t, dequant_pair(codes.w, ks, gc));
#pragma unroll
                for (int t = 0; t < kMT; ++t)
                    acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h16x8, w),
                                                                       __builtin_bit_cast(h16x8, x[t][u]), acc[t][j],
                                                                       0, 0, 0);
            }
    }
#pragma unroll
    for (int t = 0; t < kMT; ++t)
#pragma unroll
        for (int j = 0; j < kNT; ++j) part[wave][t * kNT + j][lane] = acc[t][j];
    __syncthreads();

    // register r of lane l: column n0 + 16 j + 4(l / 16) + r of row 16t + l % 16
    if (tid < kMT * kNT * kWave) {
        const int tile = tid >> 6, t = tile / kNT, j = tile % kNT;
        f32x4 sum = part[0][tile][lane];
#pragma unroll
        for (int w = 1; w < kSkinnyWaves; ++w) {
            const f32x4 p = part[w][tile][lane];
#pragma unroll
            for (int r = 0; r < 4; ++r) sum[r] += p[r];
        }
        const int m = 16 * t + r16, n = n0 + 16 * j + 4 * ks;
        if (m < a.M && n < a.N) {
            h16* crow = a.c + (size_t)m * a.N;
            if (a.vec && n + 3 < a.N) {
                h16x4 b = {0, 0, 0, 0};
                if (a.bias) b = *reinterpret_cast<const h16x4*>(a.bias + n);
                h16x4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] = to_half(sum[r] + (float)b[r]);
                *reinterpret_cast<h16x4*>(crow + n) = o;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (n + r < a.N) crow[n + r] = to_half(sum[r] + (a.bias ? (float)a.bias[n + r] : 0.0f));
            }
        }
    }
}

// ── larger M ───────────────────────────────────────────────────────────────

// Slabs of kSlots 16-byte FP16 slots per row (8 columns each), double-buffered
// through registers; a chunk of codes becomes four consecutive slots of its row.
template <int BM, int BN, int WM, int WN, int kSlots>
__global__ __launch_bounds__(WM * WN * kWave) void w4a16_tile(TileArgs a) {
    constexpr int NT = WM * WN * kWave;
    constexpr int kSteps = kSlots / 2;            // MFMA K steps (16 columns) per slab
    constexpr int kCodes = kSlots / 4;            // chunks of codes per row per slab
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int LA = BM * kSlots / NT;
    constexpr int kBLoads = BN * kCodes;
    constexpr int LB = (kBLoads + NT - 1) / NT;
    static_assert(kSlots == 4 || kSlots == 8, "slab widths with a swizzle");
    static_assert(LA >= 1 && (BM * kSlots) % NT == 0, "activation loads divide over the threads");
    static_assert(kBLoads % NT == 0 || LB == 1, "code loads: whole rounds, or one partial round");
    constexpr int kASlots = BM * kSlots, kBSlots = BN * kSlots;
    __shared__ u32x4 lds[2 * (kASlots + kBSlots)];

    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int m_blk = (int)blockIdx.y * BM, n_blk = (int)blockIdx.x * BN;
    const int kchunks = a.K / 8, nsteps = a.K / 16, ncodes = a.K / 32, ng = a.K >> a.gshift;
    const int nslabs = (kchunks + kSlots - 1) / kSlots;

    const int a_slot = tid % kSlots;
    const h16* a_ptr[LA];
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        const int row = min((tid + i * NT) / kSlots, a.M - 1 - m_blk);
        a_ptr[i] = a.a + (size_t)(m_blk + row) * a.K + a_slot * 8;
    }
    const int aw_row = tid / kSlots;
    const int aw_idx = aw_row * kSlots + swz<kSlots * 8>(aw_row, a_slot);
    const int b_code = tid % kCodes;
    const u32x4* b_ptr[LB];
    const uint32_t* z_ptr[LB];
    int b_row[LB];
#pragma unroll
    for (int j = 0; j < LB; ++j) {
        b_row[j] = (tid + j * NT) / kCodes;
        const int row = min(b_row[j], a.N - 1 - n_blk);
        b_ptr[j] = a.packed + (size_t)(n_blk + row) * ncodes + b_code;
        z_ptr[j] = a.sz + (size_t)(n_blk + row) * ng;
    }
    const bool b_active = kBLoads % NT == 0 || tid < kBLoads;

    u32x4 ra[LA], rb[LB];
    uint32_t rz[LB];
    auto fetch = [&](int slab) {
        if (slab * kSlots + a_slot < kchunks) {
#pragma unroll
            for (int i = 0; i < LA; ++i)
                ra[i] = *reinterpret_cast<const u32x4*>(a_ptr[i] + (size_t)slab * (kSlots * 8));
        }
        const int code = slab * kCodes + b_code;
        if (b_active && code < ncodes) {
#pragma unroll
            for (int j = 0; j < LB; ++j) {
                rb[j] = __builtin_nontemporal_load(b_ptr[j] + (size_t)slab * kCodes);
                rz[j] = z_ptr[j][(code * 32) >> a.gshift];
            }
        }
    };
    auto stage = [&](int buf) {
        u32x4* dst = lds + buf * (kASlots + kBSlots);
#pragma unroll
        for (int i = 0; i < LA; ++i) dst[aw_idx + i * NT] = ra[i];
        if (b_active) {
#pragma unroll
            for (int j = 0; j < LB; ++j) {
                u32x4 slots[4];
                dequant_chunk(rb[j], group_const(rz[j]), slots);
                const int row = b_row[j];
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    dst[kASlots + row * kSlots + swz<kSlots * 8>(row, b_code * 4 + q)] = slots[q];
            }
        }
    };

    f32x16 acc[TN][TM];
#pragma unroll
    for (int p = 0; p < TN; ++p)
#pragma unroll
        for (int q = 0; q < TM; ++q)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[p][q][r] = 0.0f;

    const int frow = lane & 31, fhalf = lane >> 5;
    int f_idx[kSteps];
#pragma unroll
    for (int step = 0; step < kSteps; ++step)
        f_idx[step] = frow * kSlots + swz<kSlots * 8>(frow, step * 2 + fhalf);
    const int fa_base = wm * TM * 32 * kSlots;
    const int fb_base = kASlots + wn * TN * 32 * kSlots;

    auto compute = [&](int buf, int slab) {
        const u32x4* src = lds + buf * (kASlots + kBSlots);
#pragma unroll
        for (int step = 0; step < kSteps; ++step) {
            if (slab * kSteps + step >= nsteps) break;
            u32x4 fw[TN], fx[TM];
#pragma unroll
            for (int p = 0; p < TN; ++p) fw[p] = src[fb_base + p * 32 * kSlots + f_idx[step]];
#pragma unroll
            for (int q = 0; q < TM; ++q) fx[q] = src[fa_base + q * 32 * kSlots + f_idx[step]];
#pragma unroll
            for (int p = 0; p < TN; ++p)
#pragma unroll
                for (int q = 0; q < TM; ++q)
                    acc[p][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h16x8, fw[p]),
                                                                       __builtin_bit_cast(h16x8, fx[q]),
                                                                       acc[p][q], 0, 0, 0);
        }
    };

    fetch(0);
    stage(0);
    __syncthreads();
    for (int slab = 0; slab < nslabs; ++slab) {
        const int buf = slab & 1;
        if (slab + 1 < nslabs) fetch(slab + 1);
        compute(buf, slab);
        if (slab + 1 < nslabs) stage(buf ^ 1);
        __syncthreads();
    }

    // register 4g + r of lane l: column n0 + 32p + 8g + 4(l / 32) + r of row m0 + 32q + l % 32
    const int m0 = m_blk + wm * TM * 32, n0 = n_blk + wn * TN * 32;
#pragma unroll
    for (int q = 0; q < TM; ++q) {
        const int m = m0 + q * 32 + frow;
        if (m >= a.M) continue;
        h16* crow = a.c + (size_t)m * a.N;
#pragma unroll
        for (int p = 0; p < TN; ++p)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + p * 32 + 8 * g + 4 * fhalf;
                if (n >= a.N) continue;
                if (a.vec && n + 3 < a.N) {
                    h16x4 b = {0, 0, 0, 0};
                    if (a.bias) b = *reinterpret_cast<const h16x4*>(a.bias + n);
                    h16x4 o;
#pragma unroll
                    for (int r = 0; r < 4; ++r) o[r] = to_half(acc[p][q][4 * g + r] + (float)b[r]);
                    *reinterpret_cast<h16x4*>(crow + n) = o;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (n + r < a.N)
                            crow[n + r] = to_half(acc[p][q][4 * g + r] + (a.bias ? (float)a.bias[n + r] : 0.0f));
                }
            }
    }
}

template <int BM, int BN, int WM, int WN, int kSlots>
void launch_tile(const TileArgs& a, hipStream_t st) {
    const dim3 grid((unsigned)((a.N + BN - 1) / BN), (unsigned)((a.M + BM - 1) / BM));
    w4a16_tile<BM, BN, WM, WN, kSlots><<<grid, WM * WN * kWave, 0, st>>>(a);
}

int group_shift(int group_size) {
    switch (group_size) {
        case 32: return 5;
        case 64: return 6;
        case 128: return 7;
        case 256: return 8;
        default: return -1;
    }
}

}  // namespace
}  // namespace vv

extern "C" {

vv_status_t vv_w4a16_dequant_dev(const void* packed, const void* sz, void* out_fp16, int N, int K,
                                 int group_size, void* stream) {
    if (!packed || !sz || !out_fp16) return VV_ERR_NULL_PTR;
    const int gs = vv::group_shift(group_size);
    if (gs < 0 || K % 32 != 0 || K % group_size != 0) return VV_ERR_UNSUPPORTED;
    if (!vv::aligned16(packed) || !vv::aligned16(out_fp16) || (reinterpret_cast<uintptr_t>(sz) & 3u))
        return VV_ERR_UNSUPPORTED;
    if (N <= 0 || K <= 0) return VV_OK;
    const size_t total = (size_t)N * (K / 32);
    vv::w4a16_dequant<<<dim3((unsigned)((total + vv::kBlock - 1) / vv::kBlock)), vv::kBlock, 0,
                        vv::as_stream(stream)>>>(static_cast<const vv::u32x4*>(packed),
                                                 static_cast<const uint32_t*>(sz),
                                                 static_cast<vv::u32x4*>(out_fp16), total, K / 32, K >> gs, gs);
    return vv::launch_status();
}

vv_status_t vv_w4a16_gather_dev(const void* x, const int32_t* perm, void* out, int M, int K, void* stream) {
    if (!x || !perm || !out) return VV_ERR_NULL_PTR;
    if (M <= 0 || K <= 0 || K % 8 != 0) return VV_ERR_INVALID_ARG;
    if (!vv::aligned16(perm) || !vv::aligned16(out)) return VV_ERR_UNSUPPORTED;
    const size_t total = (size_t)M * (K / 8);
    vv::w4a16_gather<<<dim3((unsigned)((total + vv::kBlock - 1) / vv::kBlock)), vv::kBlock, 0,
                       vv::as_stream(stream)>>>(static_cast<const vv::h16*>(x), perm,
                                                static_cast<vv::h16*>(out), M, K);
    return vv::launch_status();
}

vv_status_t vv_w4a16_gemv_multi_dev(const void* x, const vv_w4a16_proj_t* projs, int n_proj, int K,
                                    int group_size, void* stream) {
    if (!x || !projs) return VV_ERR_NULL_PTR;
    if (n_proj < 1 || n_proj > vv::kMaxSegs) return VV_ERR_INVALID_ARG;
    const int gs = vv::group_shift(group_size);
    if (gs < 0 || K <= 0 || K % 32 != 0 || K % group_size != 0 || !vv::aligned16(x)) return VV_ERR_UNSUPPORTED;
    vv::GemvSegs segs = {};
    for (int i = 0; i < n_proj; ++i) {
        if (!projs[i].packed || !projs[i].sz || !projs[i].y) return VV_ERR_NULL_PTR;
        if (projs[i].N <= 0 || !vv::aligned16(projs[i].packed) || (reinterpret_cast<uintptr_t>(projs[i].sz) & 3u))
            return VV_ERR_UNSUPPORTED;
        segs.w[i] = static_cast<const vv::u32x4*>(projs[i].packed);
        segs.sz[i] = static_cast<const uint32_t*>(projs[i].sz);
        segs.bias[i] = static_cast<const vv::h16*>(projs[i].bias);
        segs.y[i] = static_cast<vv::h16*>(projs[i].y);
        segs.n[i] = projs[i].N;
    }
    vv::launch_gemv_rows(static_cast<const vv::h16*>(x), segs, n_proj, 1, K, gs, vv::as_stream(stream));
    return vv::launch_status();
}

vv_status_t vv_w4a16_gemv_dev(const void* x, const void* packed, const void* sz, const void* bias, void* y,
                              int N, int K, int group_size, void* stream) {
    if (!x || !packed || !sz || !y) return VV_ERR_NULL_PTR;
    vv_w4a16_proj_t p;
    p.packed = packed;
    p.sz = sz;
    p.bias = bias;
    p.y = y;
    p.N = N;
    return vv_w4a16_gemv_multi_dev(x, &p, 1, K, group_size, stream);
}

/* Many rows and a scratch that holds the dense weight: dequantise once, then the FP16 GEMM (its
 * 256 x 256 direct-to-LDS kernel is faster than any tile that unpacks codes on the way in, and the
 * dequantiser costs a percent of it). Otherwise the weights stay packed until they are in LDS and
 * the scratch is not touched. */
vv_status_t vv_w4a16_gemm_dev(const void* A, const void* packed, const void* sz, const void* bias, void* C,
                              void* scratch, size_t scratch_bytes, int M, int N, int K, int group_size,
                              void* stream) {
    if (!A || !packed || !sz || !C) return VV_ERR_NULL_PTR;
    const int gs = vv::group_shift(group_size);
    if (gs < 0 || K <= 0 || K % 32 != 0 || K % group_size != 0 || M <= 0 || N <= 0) return VV_ERR_UNSUPPORTED;
    if (!vv::aligned16(A) || !vv::aligned16(packed) || (reinterpret_cast<uintptr_t>(sz) & 3u))
        return VV_ERR_UNSUPPORTED;
    hipStream_t st = vv::as_stream(stream);
    if (M <= 4) {
        vv::GemvSegs segs = {};
        segs.w[0] = static_cast<const vv::u32x4*>(packed);
        segs.sz[0] = static_cast<const uint32_t*>(sz);
        segs.bias[0] = static_cast<const vv::h16*>(bias);
        segs.y[0] = static_cast<vv::h16*>(C);
        segs.n[0] = N;
        vv::launch_gemv_rows(static_cast<const vv::h16*>(A), segs, 1, M, K, gs, st);
        return vv::launch_status();
    }
    const bool bias_ok = !bias || (N % 8 == 0 && vv::aligned16(bias) && vv::aligned16(C));
    if (M >= 1024 && scratch && vv::aligned16(scratch) && scratch_bytes >= (size_t)N * K * 2 && bias_ok) {
        vv_status_t s = vv_w4a16_dequant_dev(packed, sz, scratch, N, K, group_size, stream);
        if (s != VV_OK) return s;
        if (bias) {
            const size_t total = (size_t)M * (N / 8);
            vv::bias_rows<<<dim3((unsigned)((total + vv::kBlock - 1) / vv::kBlock)), vv::kBlock, 0, st>>>(
                static_cast<const vv::h16*>(bias), static_cast<vv::h16*>(C), M, N);
            if (vv::launch_status() != VV_OK) return VV_ERR_CUDA_LAUNCH;
        }
        return vv_gemm_fp16_dev(A, scratch, C, M, N, K, 1.0f, bias ? 1.0f : 0.0f, stream);
    }
    vv::TileArgs a;
    a.a = static_cast<const vv::h16*>(A);
    a.packed = static_cast<const vv::u32x4*>(packed);
    a.sz = static_cast<const uint32_t*>(sz);
    a.bias = static_cast<const vv::h16*>(bias);
    a.c = static_cast<vv::h16*>(C);
    a.M = M;
    a.N = N;
    a.K = K;
    a.gshift = gs;
    a.vec = (N % 4 == 0) && !(reinterpret_cast<uintptr_t>(C) & 7u) && !(bias && (reinterpret_cast<uintptr_t>(bias) & 7u));
    // Beyond 16 rows a wide layer re-reads the activations once per 16 columns: tiles serve it better.
    if (M <= 32 || (M <= 64 && (N + 63) / 64 < 200)) {
        constexpr int kThreads = vv::kSkinnyWaves * vv::kWave;
        // Every workgroup reads all the activations: with 256+ workgroups left, 32 weight rows each
        // halve that traffic (gate or up at 28 rows: 36 -> 27 us; down, 112 workgroups: 38 -> 46).
        const bool two = M <= 32 && N >= 8192;
        const dim3 grid((unsigned)((N + (two ? 31 : 15)) / (two ? 32 : 16)));
        if (two) {
            if (M <= 16) vv::w4a16_skinny<1, 2><<<grid, kThreads, 0, st>>>(a);
            else vv::w4a16_skinny<2, 2><<<grid, kThreads, 0, st>>>(a);
        } else if (M <= 16) vv::w4a16_skinny<1, 1><<<grid, kThreads, 0, st>>>(a);
        else if (M <= 32) vv::w4a16_skinny<2, 1><<<grid, kThreads, 0, st>>>(a);
        else if (M <= 48) vv::w4a16_skinny<3, 1><<<grid, kThreads, 0, st>>>(a);
        else vv::w4a16_skinny<4, 1><<<grid, kThreads, 0, st>>>(a);
        return vv::launch_status();
    }
    const long wg256 = (long)((M + 255) / 256) * ((N + 255) / 256);
    const long wg128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    if (wg256 >= 512) vv::launch_tile<256, 256, 2, 4, 4>(a, st);
    else if (M > 64 && wg128 >= 256) vv::launch_tile<128, 128, 2, 2, 8>(a, st);
    else if (M > 32) vv::launch_tile<64, 64, 2, 2, 8>(a, st);
    else vv::launch_tile<32, 64, 1, 2, 8>(a, st);
    return vv::launch_status();
}

}  // extern "C"
