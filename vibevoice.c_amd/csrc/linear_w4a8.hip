// W4A8 linear layers: y[m,n] = sx[m] * sum_g s[n,g] * sum_{k in g} (q[n,k] - z[n,g]) xq[m,k]
// + bias[n] + residual[m,n]: int8 activations with per-row scales, 4-bit weight
// codes with an FP16 scale and an integer zero point per group of G columns.
//
// The codes arrive in the accelerator layout of the INT4 weights: every 16-byte
// chunk holds 32 consecutive columns, nibble slot s of 32-bit word t being
// column 2 (t + 4 (s % 4)) + s / 4. The activations arrive permuted inside
// every run of 32 columns so that the codes unpack with masks alone:
//   VV_Q8_W4_GEMV  bytes 8t..8t+3 meet slots 0,2,4,6 (w & 0x0F0F0F0F), bytes
//                  8t+4..8t+7 slots 1,3,5,7 ((w >> 4) & 0x0F0F0F0F)
//   VV_Q8_W4_MMA   bytes 4t..4t+3 meet slots 0..3, bytes 16+4t.. slots 4..7, so
//                  a chunk unpacks into the two 16-byte operands of one
//                  v_mfma_i32_32x32x32_i8 step
// The zero point is taken off the unpacked bytes (q - z fits int8) or, in the
// GEMV when the quantiser's per-chunk sums of x are passed, through those; the
// per-group sums are exact int32 either way, and the groups are added in order in
// FP32 with nothing fused: acc += s_g * (float)sum_g, then acc * sx[m], + bias,
// + residual. That is the CPU kernel's scalar form (src/cpu/cpu_int8.c:212-233,
// 537-541), so every path and tile shape gives the same bits.
#include "mfma_tile.hpp"

namespace vv {
namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef h16 h16x4 __attribute__((ext_vector_type(4)));

constexpr int kLayoutGemv = 2, kLayoutMma = 3;   // VV_Q8_W4_GEMV, VV_Q8_W4_MMA (q8.h:31-43)

struct W4Args {
    const int8_t* xq;
    const float* sx;
    const uint32_t* packed;   // [N][K/8] words
    const uint32_t* sz;       // [N][K/G] half2 {scale, zero}
    const h16* bias;
    const h16* res;
    void* y;
    int y_f32, M, N, K, G, vec;
};

__device__ __forceinline__ float sz_scale(uint32_t sz) {
    return (float)__builtin_bit_cast(h16, (uint16_t)(sz & 0xFFFFu));
}
// The zero point replicated into four bytes.
__device__ __forceinline__ uint32_t sz_zero4(uint32_t sz) {
    return (uint32_t)(int)(float)__builtin_bit_cast(h16, (uint16_t)(sz >> 16)) * 0x01010101u;
}
// Four codes 0..15 in the bytes of `codes`, minus the zero point, as int8:
// 0x80 + q - z never borrows from the next byte, and flipping the top bit of
// 0x80 + d is d in two's complement for -15 <= d <= 15.
__device__ __forceinline__ uint32_t minus_zero(uint32_t codes, uint32_t z4) {
    return ((codes | 0x80808080u) - z4) ^ 0x80808080u;
}

__device__ __forceinline__ float w4_value(float acc, float sxm, bool has_b, float b, bool has_r, float r) {
#pragma clang fp contract(off)
    float v = acc * sxm;
    if (has_b) v = v + b;
    if (has_r) v = v + r;
    return v;
}

__device__ __forceinline__ void w4_store1(const W4Args& o, int m, int n, float acc) {
    const size_t idx = (size_t)m * o.N + n;
    const float v = w4_value(acc, o.sx[m], o.bias != nullptr, o.bias ? (float)o.bias[n] : 0.0f,
                             o.res != nullptr, o.res ? (float)o.res[idx] : 0.0f);
    if (o.y_f32) static_cast<float*>(o.y)[idx] = v;
    else static_cast<h16*>(o.y)[idx] = to_half(v);
}

__device__ __forceinline__ void w4_store4(const W4Args& o, int m, int n, const float (&acc)[4]) {
    if (o.vec && n + 3 < o.N) {
        const size_t idx = (size_t)m * o.N + n;
        const float sxm = o.sx[m];
        h16x4 b = {0, 0, 0, 0}, r = {0, 0, 0, 0};
        if (o.bias) b = *reinterpret_cast<const h16x4*>(o.bias + n);
        if (o.res) r = *reinterpret_cast<const h16x4*>(o.res + idx);
        f32x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            v[i] = w4_value(acc[i], sxm, o.bias != nullptr, (float)b[i], o.res != nullptr, (float)r[i]);
        if (o.y_f32) {
            *reinterpret_cast<f32x4*>(static_cast<float*>(o.y) + idx) = v;
        } else {
            h16x4 h;
#pragma unroll
            for (int i = 0; i < 4; ++i) h[i] = to_half(v[i]);
            *reinterpret_cast<h16x4*>(static_cast<h16*>(o.y) + idx) = h;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (n + i < o.N) w4_store1(o, m, n + i, acc[i]);
    }
}

// ── M <= 8, any group size: one workgroup per weight row ───────────────────
// Every thread takes whole 32-column chunks (16 bytes of codes against 32
// bytes of each activation row) and leaves the chunk's exact sums in LDS; the
// group sums are scaled in parallel, and one thread per activation row adds
// the groups in order.
constexpr int kGemvMaxChunks = 640;    // K <= 20480

template <int MR>
__global__ __launch_bounds__(kBlock) void w4a8_gemv(W4Args a) {
    __shared__ int chunk_sum[MR][kGemvMaxChunks];
    __shared__ float group_term[MR][kGemvMaxChunks];
    const int tid = (int)threadIdx.x;
    const int n = (int)blockIdx.x;
    const int nchunks = a.K / 32, ng = a.K / a.G, per_group = a.G / 32;
    const u32x4* wrow = reinterpret_cast<const u32x4*>(a.packed + (size_t)n * (a.K / 8));
    const uint32_t* szrow = a.sz + (size_t)n * ng;
    for (int c = tid; c < nchunks; c += kBlock) {
        const u32x4 w = __builtin_nontemporal_load(wrow + c);
        const uint32_t z4 = sz_zero4(szrow[c / per_group]);
        int wq[8];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            wq[2 * t] = (int)minus_zero(w[t] & 0x0F0F0F0Fu, z4);
            wq[2 * t + 1] = (int)minus_zero((w[t] >> 4) & 0x0F0F0F0Fu, z4);
        }
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            if (m < a.M) {
                const i32x4* xr = reinterpret_cast<const i32x4*>(a.xq + (size_t)m * a.K) + 2 * c;
                const i32x4 x0 = xr[0], x1 = xr[1];
                int d = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    d = __builtin_amdgcn_sdot4(x0[i], wq[i], d, false);
                    d = __builtin_amdgcn_sdot4(x1[i], wq[4 + i], d, false);
                }
                chunk_sum[m][c] = d;
            }
        }
    }
    __syncthreads();
    for (int idx = tid; idx < a.M * ng; idx += kBlock) {
        const int m = idx / ng, g = idx - m * ng;
        int d = 0;
        for (int j = 0; j < per_group; ++j) d += chunk_sum[m][g * per_group + j];
        group_term[m][g] = sz_scale(szrow[g]) * (float)d;
    }
    __syncthreads();
    if (tid < a.M) {
        float acc = 0.0f;
        for (int g = 0; g < ng; ++g) acc = acc + group_term[tid][g];
        w4_store1(a, tid, n, acc);
    }
}

// The same for group sizes of 32 * 2^j columns (j <= 6), without the chunk sums
// in LDS. kSplit waves share RW weight rows: wave p of them takes the rounds of
// 64 chunks p, p + kSplit, ... (a round holds whole groups), lane l chunk l of
// the round; the lanes of a group add their chunk sums with shuffles, and only
// the scaled group terms go to LDS for the in-order addition. kSplit > 1 keeps
// the chip busy when there are few rows, RW > 1 keeps more bytes in flight per
// wave when rows are many and short, and shares the activation loads. kXsum:
// the zero point goes through the quantiser's per-chunk sums of x
// (sum q x - z sum x) instead of being taken off every code.
constexpr int kBlockTerms = 8192;      // FP32 group terms per workgroup (32 KB)

// Up to three projections of the same activations in one launch: workgroups
// [first[p], first[p + 1]) serve projection p and never straddle two.
constexpr int kMaxSegs = 3;
struct W4Segs {
    const uint32_t* packed[kMaxSegs];
    const uint32_t* sz[kMaxSegs];
    const h16* bias[kMaxSegs];
    void* y[kMaxSegs];
    int n[kMaxSegs];
    int first[kMaxSegs + 1];
};

template <int MR, int kSplit, int RW, bool kXsum>
__global__ __launch_bounds__(kBlock) void w4a8_gemv_rows(W4Args a, W4Segs segs, const int32_t* __restrict__ xsum,
                                                         int log2_per_group) {
    constexpr int kRows = kWavesPerBlock / kSplit * RW;    // weight rows per workgroup
    extern __shared__ float terms[];                       // [kRows][MR][groups]
    const int wave = wave_in_block(), lane = lane_id();
    const int b = (int)blockIdx.x;
    const int seg = (b >= segs.first[1] ? 1 : 0) + (b >= segs.first[2] ? 1 : 0);
    a.packed = segs.packed[seg];
    a.sz = segs.sz[seg];
    a.bias = segs.bias[seg];
    a.y = segs.y[seg];
    a.N = segs.n[seg];
    const int nchunks = a.K / 32, ng = a.K / a.G;
    const int per_group = 1 << log2_per_group;
    const int set = wave / kSplit, piece = wave % kSplit;
    const int n_blk = (b - segs.first[seg]) * kRows;
    const u32x4* wrow[RW];
    const uint32_t* szrow[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        const int row = min(n_blk + set * RW + r, a.N - 1);
        wrow[r] = reinterpret_cast<const u32x4*>(a.packed + (size_t)row * (a.K / 8));
        szrow[r] = a.sz + (size_t)row * ng;
    }
#pragma unroll 2
    for (int base = piece * kWave; base < nchunks; base += kSplit * kWave) {
        const bool live = base + lane < nchunks;
        const int c = live ? base + lane : nchunks - 1;
        const int g = c >> log2_per_group;
        i32x4 x0[MR], x1[MR];
        int xs[MR];
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            if (m < a.M) {
                const i32x4* xr = reinterpret_cast<const i32x4*>(a.xq + (size_t)m * a.K) + 2 * c;
                x0[m] = xr[0];
                x1[m] = xr[1];
                if (kXsum) xs[m] = xsum[(size_t)m * nchunks + c];
            }
        }
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            const u32x4 w = __builtin_nontemporal_load(wrow[r] + c);
            const uint32_t szw = szrow[r][g];
            const uint32_t z4 = sz_zero4(szw);
            const int z = (int)(z4 & 0xFFu);
            const float scale = sz_scale(szw);
            int wq[8];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t even = w[t] & 0x0F0F0F0Fu, odd = (w[t] >> 4) & 0x0F0F0F0Fu;
                wq[2 * t] = (int)(kXsum ? even : minus_zero(even, z4));
                wq[2 * t + 1] = (int)(kXsum ? odd : minus_zero(odd, z4));
            }
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                if (m < a.M) {
                    int d = 0;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        d = __builtin_amdgcn_sdot4(x0[m][i], wq[i], d, false);
                        d = __builtin_amdgcn_sdot4(x1[m][i], wq[4 + i], d, false);
                    }
                    if (kXsum) d -= z * xs[m];
                    if (!live) d = 0;
                    for (int o = 1; o < per_group; o <<= 1) d += __shfl_xor(d, o);
                    if (live && (lane & (per_group - 1)) == 0)
                        terms[((set * RW + r) * MR + m) * ng + g] = scale * (float)d;
                }
            }
        }
    }
    __syncthreads();
    const int tid = (int)threadIdx.x;
    if (tid < kRows * MR) {
        const int row = tid / MR, m = tid % MR;
        if (m < a.M && n_blk + row < a.N) {
            const float* t = terms + (row * MR + m) * ng;
            float acc = 0.0f;
            for (int g = 0; g < ng; ++g) acc = acc + t[g];
            w4_store1(a, m, n_blk + row, acc);
        }
    }
}

template <int MR, int kSplit, int RW>
void launch_gemv_rows(const W4Args& a, W4Segs segs, int n_segs, const int32_t* xsum, int log2_pg, hipStream_t st) {
    constexpr int kRows = kWavesPerBlock / kSplit * RW;
    int blocks = 0;
    for (int i = 0; i <= kMaxSegs; ++i) {
        segs.first[i] = i <= n_segs ? blocks : 0x7FFFFFFF;
        if (i < n_segs) blocks += (segs.n[i] + kRows - 1) / kRows;
    }
    for (int i = n_segs; i < kMaxSegs; ++i) {
        segs.packed[i] = segs.packed[0];
        segs.sz[i] = segs.sz[0];
        segs.bias[i] = nullptr;
        segs.y[i] = segs.y[0];
        segs.n[i] = 1;
    }
    const dim3 grid((unsigned)blocks);
    const size_t lds = (size_t)kRows * MR * (a.K / a.G) * sizeof(float);     // at most kBlockTerms floats
    if (xsum) w4a8_gemv_rows<MR, kSplit, RW, true><<<grid, kBlock, lds, st>>>(a, segs, xsum, log2_pg);
    else w4a8_gemv_rows<MR, kSplit, RW, false><<<grid, kBlock, lds, st>>>(a, segs, xsum, log2_pg);
}

// The configuration follows the rows of all projections together.
template <int MR>
bool launch_gemv_fast(const W4Args& a, const W4Segs& segs, int n_segs, const int32_t* xsum, hipStream_t st) {
    const int per_group = a.G / 32, ng = a.K / a.G, nchunks = a.K / 32;
    if (per_group > kWave || (per_group & (per_group - 1)) != 0) return false;
    int log2_pg = 0;
    while ((1 << log2_pg) < per_group) ++log2_pg;
    long rows = 0;
    for (int i = 0; i < n_segs; ++i) rows += segs.n[i];
    // Thousands of waves in flight, and no wave with less than half a round of chunks.
    int split = 1, rw = 1;
    while (split < 4 && rows * split < 4096 && nchunks / (2 * split) >= kWave / 2) split *= 2;
    while (split == 1 && rw < 4 && rows / (2 * rw) >= 8192 && a.K * rw <= 8192) rw *= 2;
    while (rw > 1 && kWavesPerBlock * rw * MR * ng > kBlockTerms) rw >>= 1;
    if (kWavesPerBlock / split * rw * MR * ng > kBlockTerms) return false;
    if (rw == 4) launch_gemv_rows<MR, 1, 4>(a, segs, n_segs, xsum, log2_pg, st);
    else if (rw == 2) launch_gemv_rows<MR, 1, 2>(a, segs, n_segs, xsum, log2_pg, st);
    else if (split == 1) launch_gemv_rows<MR, 1, 1>(a, segs, n_segs, xsum, log2_pg, st);
    else if (split == 2) launch_gemv_rows<MR, 2, 1>(a, segs, n_segs, xsum, log2_pg, st);
    else launch_gemv_rows<MR, 4, 1>(a, segs, n_segs, xsum, log2_pg, st);
    return true;
}

bool launch_gemv_fast_rows(const W4Args& a, const W4Segs& segs, int n_segs, const int32_t* xsum, hipStream_t st) {
    const int mr = a.M == 1 ? 1 : a.M == 2 ? 2 : a.M <= 4 ? 4 : 8;
    return mr == 1 ? launch_gemv_fast<1>(a, segs, n_segs, xsum, st)
         : mr == 2 ? launch_gemv_fast<2>(a, segs, n_segs, xsum, st)
         : mr == 4 ? launch_gemv_fast<4>(a, segs, n_segs, xsum, st)
                   : launch_gemv_fast<8>(a, segs, n_segs, xsum, st);
}

// ── larger M: LDS-tiled int8 MFMA over codes unpacked on their way into LDS ─
// Slabs of 128 columns (four MFMA steps = four chunks of codes), double-buffered
// through registers. A thread that stages chunk p of weight row n also leaves
// that chunk's group scale in LDS; when a step ends a group, every int32
// accumulator is scaled into its FP32 partner and cleared.
template <int BM, int BN, int WM, int WN, int kSteps>
__global__ __launch_bounds__(WM * WN * kWave, 2) void w4a8_tile(W4Args a) {
    constexpr int NT = WM * WN * kWave;
    constexpr int kSlots = 2 * kSteps;            // 16-byte slots per slab row
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int LA = BM * kSlots / NT;          // activation loads per thread per slab
    constexpr int kBLoads = BN * kSteps;          // code chunks per slab
    constexpr int LB = (kBLoads + NT - 1) / NT;
    static_assert(LA >= 1 && (BM * kSlots) % NT == 0, "activation loads divide over the threads");
    static_assert(kBLoads % NT == 0 || LB == 1, "code loads: whole rounds, or one partial round");
    constexpr int kASlots = BM * kSlots, kBSlots = BN * kSlots;
    extern __shared__ u32x4 lds[];                // [2][A rows | B rows][slot], then the scales
    float (*scales)[kSteps][BN] = reinterpret_cast<float (*)[kSteps][BN]>(lds + 2 * (kASlots + kBSlots));

    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int m_blk = (int)blockIdx.y * BM, n_blk = (int)blockIdx.x * BN;
    const int nsteps = a.K / 32, nslabs = (nsteps + kSteps - 1) / kSteps;
    const int per_group = a.G / 32, ng = a.K / a.G;

    // activations: thread t's i-th load is row (t + i NT) / kSlots, slot t % kSlots
    const int a_slot = tid % kSlots;
    const int8_t* a_ptr[LA];
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        const int row = min((tid + i * NT) / kSlots, a.M - 1 - m_blk);
        a_ptr[i] = a.xq + (size_t)(m_blk + row) * a.K + a_slot * 16;
    }
    const int aw_row = tid / kSlots;
    const int aw_idx = aw_row * kSlots + swz<kSlots * 8>(aw_row, a_slot);
    // codes: load j is row (t + j NT) / kSteps, chunk t % kSteps of the slab
    const int b_step = tid % kSteps;
    const uint32_t* b_ptr[LB];
    const uint32_t* z_ptr[LB];
    int b_row[LB];
#pragma unroll
    for (int j = 0; j < LB; ++j) {
        b_row[j] = (tid + j * NT) / kSteps;
        const int row = min(b_row[j], a.N - 1 - n_blk);
        b_ptr[j] = a.packed + (size_t)(n_blk + row) * (a.K / 8) + b_step * 4;
        z_ptr[j] = a.sz + (size_t)(n_blk + row) * ng;
    }
    const bool b_active = kBLoads % NT == 0 || tid < kBLoads;

    u32x4 ra[LA], rb[LB];
    uint32_t rz[LB];
    auto fetch = [&](int slab) {
        const bool a_live = slab * kSlots + a_slot < a.K / 16;
#pragma unroll
        for (int i = 0; i < LA; ++i)
            if (a_live) ra[i] = *reinterpret_cast<const u32x4*>(a_ptr[i] + (size_t)slab * (kSlots * 16));
        const int step = slab * kSteps + b_step;
        if (b_active && step < nsteps) {
#pragma unroll
            for (int j = 0; j < LB; ++j) {
                rb[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(b_ptr[j] + (size_t)slab * (kSteps * 4)));
                rz[j] = z_ptr[j][step / per_group];
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
                const uint32_t z4 = sz_zero4(rz[j]);
                u32x4 lo, hi;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const uint32_t even = rb[j][t] & 0x0F0F0F0Fu;           // slots 0,2,4,6
                    const uint32_t odd = (rb[j][t] >> 4) & 0x0F0F0F0Fu;     // slots 1,3,5,7
                    // v_perm_b32 picks bytes from {odd : even} (even = bytes 0..3): slots 0,1,2,3 / 4,5,6,7
                    lo[t] = minus_zero(__builtin_amdgcn_perm(odd, even, 0x05010400u), z4);
                    hi[t] = minus_zero(__builtin_amdgcn_perm(odd, even, 0x07030602u), z4);
                }
                const int row = b_row[j];
                dst[kASlots + row * kSlots + swz<kSlots * 8>(row, 2 * b_step)] = lo;
                dst[kASlots + row * kSlots + swz<kSlots * 8>(row, 2 * b_step + 1)] = hi;
                scales[buf][b_step][row] = sz_scale(rz[j]);
            }
        }
    };

    i32x16 acc[TN][TM];
    f32x16 facc[TN][TM];
#pragma unroll
    for (int x = 0; x < TN; ++x)
#pragma unroll
        for (int y = 0; y < TM; ++y)
#pragma unroll
            for (int r = 0; r < 16; ++r) facc[x][y][r] = 0.0f;

    const int frow = lane & 31, fhalf = lane >> 5;
    int f_idx[kSteps];
#pragma unroll
    for (int step = 0; step < kSteps; ++step)
        f_idx[step] = frow * kSlots + swz<kSlots * 8>(frow, step * 2 + fhalf);
    const int fa_base = wm * TM * 32 * kSlots;
    const int fb_base = kASlots + wn * TN * 32 * kSlots;
    int until_flush = per_group;
    bool fresh = true;

    auto compute = [&](int buf, int slab) {
        const u32x4* src = lds + buf * (kASlots + kBSlots);
#pragma unroll
        for (int step = 0; step < kSteps; ++step) {
            if (slab * kSteps + step >= nsteps) break;
            u32x4 fw[TN], fx[TM];
#pragma unroll
            for (int x = 0; x < TN; ++x) fw[x] = src[fb_base + x * 32 * kSlots + f_idx[step]];
#pragma unroll
            for (int y = 0; y < TM; ++y) fx[y] = src[fa_base + y * 32 * kSlots + f_idx[step]];
            // The first step of a group starts from a literal zero, so a flush need not clear anything.
            if (fresh) {
                const i32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int x = 0; x < TN; ++x)
#pragma unroll
                    for (int y = 0; y < TM; ++y)
                        acc[x][y] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, fw[x]),
                                                                          __builtin_bit_cast(i32x4, fx[y]),
                                                                          zero, 0, 0, 0);
            } else {
#pragma unroll
                for (int x = 0; x < TN; ++x)
#pragma unroll
                    for (int y = 0; y < TM; ++y)
                        acc[x][y] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, fw[x]),
                                                                          __builtin_bit_cast(i32x4, fx[y]),
                                                                          acc[x][y], 0, 0, 0);
            }
            fresh = false;
            if (--until_flush == 0) {
                until_flush = per_group;
                fresh = true;
                const float* sc = &scales[buf][step][wn * TN * 32 + 4 * fhalf];
#pragma unroll
                for (int x = 0; x < TN; ++x)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const f32x4 s = *reinterpret_cast<const f32x4*>(sc + x * 32 + 8 * g);
#pragma unroll
                        for (int y = 0; y < TM; ++y)
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
#pragma clang fp contract(off)
                                const float term = s[r] * (float)acc[x][y][4 * g + r];
                                facc[x][y][4 * g + r] = facc[x][y][4 * g + r] + term;
                            }
                    }
            }
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

    const int m0 = m_blk + wm * TM * 32, n0 = n_blk + wn * TN * 32;
#pragma unroll
    for (int y = 0; y < TM; ++y) {
        const int m = m0 + y * 32 + frow;
        if (m >= a.M) continue;
#pragma unroll
        for (int x = 0; x < TN; ++x)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + x * 32 + 8 * g + 4 * fhalf;
                if (n >= a.N) continue;
                const float t[4] = {facc[x][y][4 * g], facc[x][y][4 * g + 1], facc[x][y][4 * g + 2],
                                    facc[x][y][4 * g + 3]};
                w4_store4(a, m, n, t);
            }
    }
}

template <int BM, int BN, int WM, int WN, int kSteps>
bool launch_w4_tile(const W4Args& a, hipStream_t st) {
    constexpr size_t kLds = (size_t)2 * (BM + BN) * 2 * kSteps * 16 + (size_t)2 * kSteps * BN * sizeof(float);
    if constexpr (kLds > 64 * 1024) {
        // above the default limit of dynamic LDS: raised once per thread and device
        static thread_local int ready_device = -1;
        int device = 0;
        if (hipGetDevice(&device) != hipSuccess) return false;
        if (ready_device != device) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(w4a8_tile<BM, BN, WM, WN, kSteps>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLds) != hipSuccess) {
                (void)hipGetLastError();
                return false;
            }
            ready_device = device;
        }
    }
    const dim3 grid((unsigned)((a.N + BN - 1) / BN), (unsigned)((a.M + BM - 1) / BM));
    w4a8_tile<BM, BN, WM, WN, kSteps><<<grid, WM * WN * kWave, kLds, st>>>(a);
    return true;
}

// ── M <= 64 in the MMA order, groups of 64, 128 or 256 columns: streamed weights ─
// With so few activation rows a tile grid has too few workgroups to pull the
// codes out of HBM, and the in-order addition of the groups forbids splitting K
// between accumulators. The int32 sum of one group is exact in any order,
// though: a workgroup owns 32 weight rows, its eight waves take the eight groups
// of a round one each and leave the group's sums in LDS, and the waves that
// own a quarter of the output tile then add the round's groups in order,
// acc += s_g * (float)sum_g, as every other path does.
//
// One 32x32x32 MFMA pair covers 64 columns: lane (row, half) loads the 16 bytes
// of codes of chunk 2p + half of its weight row and the 32 bytes of that chunk
// of its activation row; the first MFMA meets nibble slots 0..3 of the four
// words with activation bytes 0..15, the second slots 4..7 with bytes 16..31.
// No byte is loaded twice, and both chunks of a pair lie in one group.
constexpr int kStreamWaves = 8;

// A lane of the MFMA order reads 16 bytes of its own row, so one load touches 32
// cache lines; kViaLds (groups of 128 columns) loads whole runs of a row instead
// (four lanes a weight row's 64 bytes of the group, eight lanes an activation
// row's 128) and turns them into the MFMA order through a piece of LDS of the
// wave's own. The operands of the next round are requested before the sums of
// this one are handed over; requesting further ahead measured slower.
template <int kMT, int kPairs, bool kViaLds, bool kGemvOrder>
__global__ __launch_bounds__(kStreamWaves * kWave) void w4a8_stream(W4Args a) {
    static_assert(!kViaLds || kPairs == 2, "the staged loads are laid out for groups of 128 columns");
    constexpr int kGroups = kStreamWaves;          // groups per round, one per wave
    extern __shared__ u32x4 lds[];                 // sums[kGroups][kMT][4][64] int32x4, then scl[kGroups][32] float
    i32x4* sums = reinterpret_cast<i32x4*>(lds);
    float* scl = reinterpret_cast<float*>(lds + kGroups * kMT * 4 * kWave);
    u32x4* stage = lds + kGroups * kMT * 4 * kWave + kGroups * 32 / 4;     // kViaLds: 4 KB per wave
    const int wave = wave_in_block(), lane = lane_id();
    const int row32 = lane & 31, half = lane >> 5;
    const int n_blk = (int)blockIdx.x * 32;
    const int ng = a.K / a.G;
    const int nrounds = (ng + kGroups - 1) / kGroups;
    const int wr = min(n_blk + row32, a.N - 1);
    const u32x4* wrow = reinterpret_cast<const u32x4*>(a.packed + (size_t)wr * (a.K / 8));
    const uint32_t* zrow = a.sz + (size_t)wr * ng;
    const u32x4* xrow[kMT];
#pragma unroll
    for (int y = 0; y < kMT; ++y)
        xrow[y] = reinterpret_cast<const u32x4*>(a.xq + (size_t)min(y * 32 + row32, a.M - 1) * a.K);
    // Wave 4 y + q adds output rows 8 q + 4 half + r (r = 0..3) of activation tile y. (Sharing the
    // adds between all eight waves when there is one tile measured slower.)
    const bool adds = wave < kMT * 4;
    const int ay = wave >> 2, aq = wave & 3;
    const i32x4* my_sums = sums + (ay * 4 + aq) * kWave + lane;
    const float* my_scl = scl + 8 * aq + 4 * half;
    f32x4 facc = {0.0f, 0.0f, 0.0f, 0.0f};

    u32x4 w[kPairs], x[kMT][kPairs][2];
    uint32_t zw = 0;
    auto fetch = [&](int round) {
        const int g = min(round * kGroups + wave, ng - 1);
        if constexpr (kViaLds) {
            // Whole runs of a row per load: 4 lanes cover a weight row's 64 bytes of the group, 8 lanes an
            // activation row's 128 bytes.
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int row = min(n_blk + (lane >> 2) + 16 * i, a.N - 1);
                w[i] = reinterpret_cast<const u32x4*>(a.packed + (size_t)row * (a.K / 8))[g * 4 + (lane & 3)];
            }
#pragma unroll
            for (int y = 0; y < kMT; ++y)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int row = min(y * 32 + (lane >> 3) + 8 * i, a.M - 1);
                    x[y][i >> 1][i & 1] =
                        reinterpret_cast<const u32x4*>(a.xq + (size_t)row * a.K)[g * 8 + (lane & 7)];
                }
        } else {
            const int c0 = g * (2 * kPairs) + half;
#pragma unroll
            for (int p = 0; p < kPairs; ++p) {
                w[p] = wrow[c0 + 2 * p];
#pragma unroll
                for (int y = 0; y < kMT; ++y) {
                    x[y][p][0] = xrow[y][2 * (c0 + 2 * p)];
                    x[y][p][1] = xrow[y][2 * (c0 + 2 * p) + 1];
                }
            }
        }
        zw = zrow[g];
    };
    auto add_group = [&](int j) {
#pragma clang fp contract(off)
        const i32x4 s = my_sums[j * (kMT * 4 * kWave)];
        const f32x4 sc = *reinterpret_cast<const f32x4*>(my_scl + j * 32);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float term = sc[r] * (float)s[r];
            facc[r] = facc[r] + term;
        }
    };
    // The group sums of one round go through LDS to the adding waves.
    auto hand_over = [&](const i32x16 (&acc)[kMT], float scale, int round) {
        __syncthreads();           // the previous round's sums have been added
        if (round * kGroups + wave < ng) {
#pragma unroll
            for (int y = 0; y < kMT; ++y)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const i32x4 s = {acc[y][4 * q], acc[y][4 * q + 1], acc[y][4 * q + 2], acc[y][4 * q + 3]};
                    sums[((wave * kMT + y) * 4 + q) * kWave + lane] = s;
                }
            if (half == 0) scl[wave * 32 + row32] = scale;
        }
        __syncthreads();
        if (adds) {
            const int live = ng - round * kGroups;
            if (live >= kGroups) {
#pragma unroll
                for (int j = 0; j < kGroups; ++j) add_group(j);
            } else {
#pragma unroll 1
                for (int j = 0; j < live; ++j) add_group(j);
            }
        }
    };
    auto group_sums = [&](i32x16 (&acc)[kMT]) {
        const uint32_t z4 = sz_zero4(zw);
        u32x4 wf[kPairs], xf[kMT][kPairs][2];
        if constexpr (kViaLds) {
            // Through this wave's own piece of LDS into the MFMA order; LDS serves a wave's accesses in
            // the order they were issued, so the piece is reused without a barrier.
            u32x4* buf = stage + wave * 256;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int row = (lane >> 2) + 16 * i;
                buf[row * 4 + swz<32>(row, lane & 3)] = w[i];
            }
#pragma unroll
            for (int p = 0; p < 2; ++p) wf[p] = buf[row32 * 4 + swz<32>(row32, half + 2 * p)];
#pragma unroll
            for (int y = 0; y < kMT; ++y) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int row = (lane >> 3) + 8 * i;
                    buf[row * 8 + swz<64>(row, lane & 7)] = x[y][i >> 1][i & 1];
                }
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    xf[y][p][0] = buf[row32 * 8 + swz<64>(row32, 2 * (half + 2 * p))];
                    xf[y][p][1] = buf[row32 * 8 + swz<64>(row32, 2 * (half + 2 * p) + 1)];
                }
            }
        } else {
#pragma unroll
            for (int p = 0; p < kPairs; ++p) {
                wf[p] = w[p];
#pragma unroll
                for (int y = 0; y < kMT; ++y) {
                    xf[y][p][0] = x[y][p][0];
                    xf[y][p][1] = x[y][p][1];
                }
            }
        }
#pragma unroll
        for (int p = 0; p < kPairs; ++p) {
            i32x4 lo, hi;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t even = wf[p][t] & 0x0F0F0F0Fu;           // slots 0,2,4,6
                const uint32_t odd = (wf[p][t] >> 4) & 0x0F0F0F0Fu;     // slots 1,3,5,7
                if constexpr (kGemvOrder) {
                    // activation bytes 8t..8t+3 meet the even slots of word t, 8t+4..8t+7 the odd ones
                    (t < 2 ? lo : hi)[2 * (t & 1)] = (int)minus_zero(even, z4);
                    (t < 2 ? lo : hi)[2 * (t & 1) + 1] = (int)minus_zero(odd, z4);
                } else {
                    lo[t] = (int)minus_zero(__builtin_amdgcn_perm(odd, even, 0x05010400u), z4);
                    hi[t] = (int)minus_zero(__builtin_amdgcn_perm(odd, even, 0x07030602u), z4);
                }
            }
#pragma unroll
            for (int y = 0; y < kMT; ++y) {
                const i32x4 x0 = __builtin_bit_cast(i32x4, xf[y][p][0]);
                const i32x4 x1 = __builtin_bit_cast(i32x4, xf[y][p][1]);
                if (p == 0) {
                    const i32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    acc[y] = __builtin_amdgcn_mfma_i32_32x32x32_i8(lo, x0, zero, 0, 0, 0);
                } else {
                    acc[y] = __builtin_amdgcn_mfma_i32_32x32x32_i8(lo, x0, acc[y], 0, 0, 0);
                }
                acc[y] = __builtin_amdgcn_mfma_i32_32x32x32_i8(hi, x1, acc[y], 0, 0, 0);
            }
        }
    };
    fetch(0);
    for (int round = 0; round < nrounds; ++round) {
        i32x16 acc[kMT];
        group_sums(acc);
        const float scale = sz_scale(zw);
        fetch(min(round + 1, nrounds - 1));       // past the end: the last round again, unused
        hand_over(acc, scale, round);
    }
    if (adds) {
        const int m = ay * 32 + row32, n = n_blk + 8 * aq + 4 * half;
        if (m < a.M && n < a.N) {
            const float t[4] = {facc[0], facc[1], facc[2], facc[3]};
            w4_store4(a, m, n, t);
        }
    }
}

template <int kMT, int kPairs, bool kGemvOrder>
bool launch_w4_stream_cfg(const W4Args& a, hipStream_t st) {
    constexpr bool kViaLds = kPairs == 2;
    constexpr size_t kLds = (size_t)kStreamWaves * kMT * 4 * kWave * 16 + (size_t)kStreamWaves * 32 * sizeof(float) +
                            (kViaLds ? (size_t)kStreamWaves * 4096 : 0);
    if constexpr (kLds > 64 * 1024) {
        // above the default limit of dynamic LDS: raised once per thread and device
        static thread_local int ready_device = -1;
        int device = 0;
        if (hipGetDevice(&device) != hipSuccess) return false;
        if (ready_device != device) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(w4a8_stream<kMT, kPairs, kViaLds, kGemvOrder>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLds) != hipSuccess) {
                (void)hipGetLastError();
                return false;
            }
            ready_device = device;
        }
    }
    w4a8_stream<kMT, kPairs, kViaLds, kGemvOrder>
        <<<dim3((unsigned)((a.N + 31) / 32)), kStreamWaves * kWave, kLds, st>>>(a);
    return true;
}

bool w4_stream_serves(int M, int N, int G) {
    if (M > 64 || (G != 64 && G != 128 && G != 256)) return false;
    if (M > 32 && (N + 63) / 64 >= 256) return false;     // enough 64 x 64 tiles to fill the chip
    if (M > 32 && G == 256) return false;                   // two tiles of its operands do not fit the registers
    return true;
}

// false: not this kernel's shape (nothing launched). gemv_order: the activations are in the GEMV's order.
bool launch_w4_stream(const W4Args& a, bool gemv_order, hipStream_t st) {
    if (!w4_stream_serves(a.M, a.N, a.G) || (gemv_order && a.M > 32)) return false;
    if (gemv_order) {
        return a.G == 64 ? launch_w4_stream_cfg<1, 1, true>(a, st)
             : a.G == 128 ? launch_w4_stream_cfg<1, 2, true>(a, st) : launch_w4_stream_cfg<1, 4, true>(a, st);
    }
    if (a.M <= 32) {
        return a.G == 64 ? launch_w4_stream_cfg<1, 1, false>(a, st)
             : a.G == 128 ? launch_w4_stream_cfg<1, 2, false>(a, st) : launch_w4_stream_cfg<1, 4, false>(a, st);
    }
    return a.G == 64 ? launch_w4_stream_cfg<2, 1, false>(a, st) : launch_w4_stream_cfg<2, 2, false>(a, st);
}

// From five activation rows on the streamed kernel beats the GEMV, which goes through the weights once
// per row in its arithmetic.
constexpr int kGemvBestRows = 4;
constexpr int kStreamMinRows = 2048;      // weight rows; below, the GEMV's one workgroup per few rows fills the chip better

enum I8Path : int { kPathAuto = 0, kPathGemv = 1, kPathMma = 2, kPathSimt = 3 };

}  // namespace
}  // namespace vv

// Every projection of a W4A8 GEMV (FP16 outputs, no residual) in ONE launch, each row computed
// exactly as vv_w4a8_linear_dev would; VV_ERR_UNSUPPORTED (nothing launched) when the shape is not
// the shuffle GEMV's, so that the caller runs one call per projection instead.
__attribute__((visibility("hidden")))
vv_status_t vv_w4a8_gemv_multi(const int8_t* xq, int x_layout, const float* sx, const int32_t* xsum,
                               const vv_i8_proj_t* projs, int n, int group_size, int M, int K, void* stream) {
    if (x_layout != vv::kLayoutGemv || M < 1 || M > 8 || n < 1 || n > vv::kMaxSegs) return VV_ERR_UNSUPPORTED;
    if (K <= 0 || K % 32 != 0 || group_size <= 0 || group_size % 32 != 0 || K % group_size != 0)
        return VV_ERR_UNSUPPORTED;
    if (!vv::aligned16(xq) || (xsum && (reinterpret_cast<uintptr_t>(xsum) & 3u))) return VV_ERR_UNSUPPORTED;
    // Wide projections of more than four rows go one by one to the streamed kernel, which wins there
    // by more than a launch; the short ones of attention stay together.
    long rows = 0;
    for (int i = 0; i < n; ++i) rows += projs[i].N;
    if (M > vv::kGemvBestRows && rows >= 16384 && vv::w4_stream_serves(M, projs[0].N, group_size)) return VV_ERR_UNSUPPORTED;
    vv::W4Args a = {};
    a.xq = xq;
    a.sx = sx;
    a.M = M;
    a.K = K;
    a.G = group_size;
    vv::W4Segs segs = {};
    for (int i = 0; i < n; ++i) {
        const vv_i8_proj_t& q = projs[i];
        if (!q.w || !q.sz || !q.y) return VV_ERR_NULL_PTR;
        if (q.N <= 0 || !vv::aligned16(q.w) || (reinterpret_cast<uintptr_t>(q.sz) & 3u)) return VV_ERR_UNSUPPORTED;
        segs.packed[i] = static_cast<const uint32_t*>(q.w);
        segs.sz[i] = static_cast<const uint32_t*>(q.sz);
        segs.bias[i] = static_cast<const vv::h16*>(q.bias);
        segs.y[i] = q.y;
        segs.n[i] = q.N;
    }
    if (!vv::launch_gemv_fast_rows(a, segs, n, xsum, vv::as_stream(stream))) return VV_ERR_UNSUPPORTED;
    return vv::launch_status();
}

extern "C" {

vv_status_t vv_w4a8_linear_dev(const int8_t* xq, int x_layout, const float* sx, const int32_t* xsum,
                               const void* packed, const void* sz, int group_size, const void* bias,
                               const void* residual, void* y, int y_f32, int M, int N, int K, int path,
                               void* stream) {
    if (!xq || !sx || !packed || !sz || !y) return VV_ERR_NULL_PTR;
    if (x_layout != vv::kLayoutGemv && x_layout != vv::kLayoutMma) return VV_ERR_INVALID_ARG;
    if (M <= 0 || N <= 0 || K <= 0 || path < vv::kPathAuto || path > vv::kPathSimt)
        return VV_ERR_INVALID_ARG;
    if (K % 32 != 0 || group_size <= 0 || group_size % 32 != 0 || K % group_size != 0)
        return VV_ERR_UNSUPPORTED;
    if (!vv::aligned16(xq) || !vv::aligned16(packed) || (reinterpret_cast<uintptr_t>(sz) & 3u))
        return VV_ERR_UNSUPPORTED;
    const bool path_auto = path == vv::kPathAuto;
    if (path == vv::kPathAuto) path = x_layout == vv::kLayoutGemv ? vv::kPathGemv : vv::kPathMma;
    // Each kernel family reads one order of the activations.
    if ((path == vv::kPathGemv) != (x_layout == vv::kLayoutGemv)) return VV_ERR_UNSUPPORTED;
    if (path == vv::kPathGemv && M > 8) return VV_ERR_UNSUPPORTED;
    if (xsum && (reinterpret_cast<uintptr_t>(xsum) & 3u)) return VV_ERR_UNSUPPORTED;

    hipStream_t st = vv::as_stream(stream);
    vv::W4Args a;
    a.xq = xq;
    a.sx = sx;
    a.packed = static_cast<const uint32_t*>(packed);
    a.sz = static_cast<const uint32_t*>(sz);
    a.bias = static_cast<const vv::h16*>(bias);
    a.res = static_cast<const vv::h16*>(residual);
    a.y = y;
    a.y_f32 = y_f32 ? 1 : 0;
    a.M = M;
    a.N = N;
    a.K = K;
    a.G = group_size;
    const auto mis = [](const void* p, unsigned mask) { return p && (reinterpret_cast<uintptr_t>(p) & mask); };
    a.vec = (N % 4 == 0) && !mis(bias, 7u) && !mis(residual, 7u) && !mis(y, y_f32 ? 15u : 7u);

    if (path == vv::kPathGemv) {
        // xsum (may be NULL) is only read here: the other kernels take the zero point off the codes
        if (path_auto && M > vv::kGemvBestRows && N >= vv::kStreamMinRows && vv::launch_w4_stream(a, true, st))
            return vv::launch_status();
        const int mr = M == 1 ? 1 : M == 2 ? 2 : M <= 4 ? 4 : 8;
        vv::W4Segs segs = {};
        segs.packed[0] = a.packed;
        segs.sz[0] = a.sz;
        segs.bias[0] = a.bias;
        segs.y[0] = a.y;
        segs.n[0] = N;
        const bool fast = vv::launch_gemv_fast_rows(a, segs, 1, xsum, st);
        if (fast) return vv::launch_status();
        if (K / 32 > vv::kGemvMaxChunks) return VV_ERR_UNSUPPORTED;
        const dim3 grid((unsigned)N);
        if (mr == 1) vv::w4a8_gemv<1><<<grid, vv::kBlock, 0, st>>>(a);
        else if (mr == 2) vv::w4a8_gemv<2><<<grid, vv::kBlock, 0, st>>>(a);
        else if (mr == 4) vv::w4a8_gemv<4><<<grid, vv::kBlock, 0, st>>>(a);
        else vv::w4a8_gemv<8><<<grid, vv::kBlock, 0, st>>>(a);
        return vv::launch_status();
    }
    // Asked for by name, the MMA path is the LDS-tiled kernel at every M.
    if (path_auto && vv::launch_w4_stream(a, false, st)) return vv::launch_status();
    const long wg128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    if (M > 64 && wg128 >= 256) {
        if (!vv::launch_w4_tile<128, 128, 2, 2, 4>(a, st)) return VV_ERR_CUDA_LAUNCH;
    } else if (M > 32) {
        vv::launch_w4_tile<64, 64, 2, 2, 4>(a, st);
    } else {
        vv::launch_w4_tile<32, 64, 1, 2, 4>(a, st);
    }
    return vv::launch_status();
}

}  // extern "C"
