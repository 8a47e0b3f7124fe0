// W8A8 linear layers: y[M,N] = sx[m] * sw[n] * (xq[M,K] . w[N,K]^T) + bias[n]
// + residual[m,n], int8 activations (per-row scale, from the activation
// quantisers) times int8 weights (per-output-channel scale).
//
// The products are summed in int32, which is exact, so the result does not
// depend on tile shape or summation order and equals the CPU kernel's bit for
// bit once the epilogue follows it: (float)t * sx[m] * sw[n], left to right,
// nothing fused, then the bias, then the residual, one rounding to FP16.
//
//   i8_tile   the LDS-tiled loop of the FP16 GEMM with v_mfma_i32_32x32x32_i8:
//             a lane's 16-byte operand is 16 int8 values, so a K step is 32
//             wide and a 128-byte slab row carries 128 K values.
//   i8_skinny up to 64 rows: weights straight from global memory into 16x16x64
//             MFMA operands, K split over the eight waves of a workgroup.
//   i8_gemv   M <= 8: one to four waves per weight row, v_dot4_i32_i8 against
//             up to eight activation rows that share each weight load.
#include "mfma_dma.hpp"

namespace vv {
namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef h16 h16x4 __attribute__((ext_vector_type(4)));

struct I8Op {
    typedef i32x16 Acc;
    static __device__ __forceinline__ Acc mfma(u32x4 w, u32x4 x, Acc c) {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, w),
                                                     __builtin_bit_cast(i32x4, x), c, 0, 0, 0);
    }
    typedef i32x4 Acc16;                      // 16 x 16 over 64 bytes of K (mfma_dma64); integer sums: the same value
    static __device__ __forceinline__ Acc16 mfma16(u32x4 w, u32x4 x, Acc16 c) {
        return __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, w),
                                                     __builtin_bit_cast(i32x4, x), c, 0, 0, 0);
    }
};

struct I8Out {
    const float* sx;
    const float* sw;
    const h16* bias;
    const h16* res;
    void* y;
    int y_f32, M, N, vec;
};

// One output value from its exact integer sum: the CPU kernel's expression
// (src/cpu/cpu_int8.c:480-483), then the device contract's residual.
__device__ __forceinline__ float i8_value(int t, float sxm, float swn, bool has_b, float b, bool has_r,
                                          float r) {
#pragma clang fp contract(off)
    float v = (float)t * sxm * swn;
    if (has_b) v = v + b;
    if (has_r) v = v + r;
    return v;
}

__device__ __forceinline__ void i8_store1(const I8Out& o, int m, int n, int t) {
    const size_t idx = (size_t)m * o.N + n;
    const float v = i8_value(t, o.sx[m], o.sw[n], o.bias != nullptr, o.bias ? (float)o.bias[n] : 0.0f,
                             o.res != nullptr, o.res ? (float)o.res[idx] : 0.0f);
    if (o.y_f32) static_cast<float*>(o.y)[idx] = v;
    else static_cast<h16*>(o.y)[idx] = to_half(v);
}

// Four consecutive columns of one row.
__device__ __forceinline__ void i8_store4(const I8Out& o, int m, int n, const int (&t)[4]) {
    if (o.vec && n + 3 < o.N) {
        const size_t idx = (size_t)m * o.N + n;
        const float sxm = o.sx[m];
        const f32x4 sw = *reinterpret_cast<const f32x4*>(o.sw + n);
        h16x4 b = {0, 0, 0, 0}, r = {0, 0, 0, 0};
        if (o.bias) b = *reinterpret_cast<const h16x4*>(o.bias + n);
        if (o.res) r = *reinterpret_cast<const h16x4*>(o.res + idx);
        f32x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            v[i] = i8_value(t[i], sxm, sw[i], o.bias != nullptr, (float)b[i], o.res != nullptr, (float)r[i]);
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
            if (n + i < o.N) i8_store1(o, m, n + i, t[i]);
    }
}

// A wave's TN x TM accumulator tiles through the epilogue: register 4g + r of
// lane l holds column n0 + 32a + 8g + 4(l / 32) + r of row m0 + 32b + l % 32.
template <int TM, int TN>
__device__ __forceinline__ void i8_epilogue(const i32x16 (&acc)[TN][TM], const I8Out& out, int m0, int n0,
                                            int frow, int fhalf) {
#pragma unroll
    for (int b = 0; b < TM; ++b) {
        const int m = m0 + b * 32 + frow;
        if (m >= out.M) continue;
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + a * 32 + 8 * g + 4 * fhalf;
                if (n >= out.N) continue;
                const int t[4] = {acc[a][b][4 * g], acc[a][b][4 * g + 1], acc[a][b][4 * g + 2],
                                  acc[a][b][4 * g + 3]};
                i8_store4(out, m, n, t);
            }
    }
}

template <int BM, int BN, int WM, int WN, int kSlabChunks, bool kFull, int kAhead>
__global__ __launch_bounds__(WM * WN * kWave) void i8_tile(const int8_t* __restrict__ xq,
                                                           const int8_t* __restrict__ w, I8Out out,
                                                           int K) {
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    auto epilogue = [=](const i32x16 (&acc)[TN][TM], int m0, int n0, int frow, int fhalf) {
        i8_epilogue<TM, TN>(acc, out, m0, n0, frow, fhalf);
    };
    mfma_tile<I8Op, BM, BN, WM, WN, kSlabChunks, kFull, kAhead>(xq, w, out.M, out.N, K / 16, epilogue);
}

// The 256 x 256 tile with the slabs copied from global memory straight into LDS
// (mfma_dma.hpp): K % 64 == 0.
__global__ __launch_bounds__(kDmaWaves * kWave) void i8_dma(const int8_t* __restrict__ xq,
                                                            const int8_t* __restrict__ w, I8Out out, int K) {
    auto epilogue = [=](const i32x16 (&acc)[2][4], int m0, int n0, int frow, int fhalf) {
        i8_epilogue<4, 2>(acc, out, m0, n0, frow, fhalf);
    };
    mfma_dma<I8Op>(xq, w, out.M, out.N, K, epilogue);
}

// The 256x256, 128x128 and 64x64 tiles fed in slabs of 128 bytes per row (whole cache lines) on the 16x16x64
// instruction (mfma_dma.hpp): K % 128 == 0. Register r of lane l holds column n0 + 16 a + 4 (l / 16) + r of row
// m0 + 16 b + l % 16 of acc[a][b].
template <int kTile, int kStages>
__global__ __launch_bounds__(Dma64Shape<kTile>::kWaves * kWave, 2) void i8_dma64(const int8_t* __restrict__ xq,
                                                                                const int8_t* __restrict__ w,
                                                                                I8Out out, int K) {
    constexpr int TM = Dma64Shape<kTile>::TM;
    auto epilogue = [=](const i32x4 (&acc)[4][TM], int m0, int n0, int lane) {
#pragma unroll
        for (int b = 0; b < TM; ++b) {
            const int m = m0 + b * 16 + (lane & 15);
            if (m >= out.M) continue;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const int n = n0 + a * 16 + 4 * (lane >> 4);
                if (n >= out.N) continue;
                const int t[4] = {acc[a][b][0], acc[a][b][1], acc[a][b][2], acc[a][b][3]};
                i8_store4(out, m, n, t);
            }
        }
    };
    mfma_dma64<I8Op, kTile, false, kStages>(xq, w, out.M, out.N, K, epilogue);
}

__device__ __forceinline__ int wave_sum_i32(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);    // quad_perm [1,0,3,2]
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);    // quad_perm [2,3,0,1]
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true);   // row_half_mirror
    v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true);   // row_mirror
    return (__builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16)) +
           (__builtin_amdgcn_readlane(v, 32) + __builtin_amdgcn_readlane(v, 48));
}

// M <= MR <= 8 rows: kSplit waves per RW weight rows, each wave a contiguous
// 1/kSplit of K. RW = 2 where a wave owns whole short rows: twice the bytes in
// flight per wave, and the activation loads shared by both rows.
// Up to three projections of the same activations in one launch: workgroups
// [first[p], first[p + 1]) serve projection p and never straddle two.
constexpr int kMaxSegs = 3;
struct I8Segs {
    const int8_t* w[kMaxSegs];
    I8Out out[kMaxSegs];
    int first[kMaxSegs + 1];
};

template <int MR, int kSplit, int RW>
__global__ __launch_bounds__(kBlock) void i8_gemv(const int8_t* __restrict__ xq, I8Segs segs, int K) {
    constexpr int kSets = kWavesPerBlock / kSplit;
    __shared__ int part[kWavesPerBlock][RW][MR];
    const int wave = wave_in_block(), lane = lane_id();
    const int b = (int)blockIdx.x;
    const int seg = (b >= segs.first[1] ? 1 : 0) + (b >= segs.first[2] ? 1 : 0);
    const I8Out out = segs.out[seg];
    const int8_t* __restrict__ w = segs.w[seg];
    const int n0 = ((b - segs.first[seg]) * kSets + wave / kSplit) * RW;
    const int piece = wave % kSplit;
    const int kchunks = K / 16;
    const int per = (kchunks + kSplit - 1) / kSplit;
    const int begin = piece * per, end = min(kchunks, begin + per);
    int acc[RW][MR];
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[r][m] = 0;
    const i32x4* wr[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r)
        wr[r] = reinterpret_cast<const i32x4*>(w + (size_t)min(n0 + r, out.N - 1) * K);
    if (n0 < out.N) {
#pragma unroll 2
        for (int c = begin + lane; c < end; c += kWave) {
            i32x4 wv[RW];
#pragma unroll
            for (int r = 0; r < RW; ++r) wv[r] = __builtin_nontemporal_load(wr[r] + c);
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                if (m < out.M) {
                    const i32x4 xv = *(reinterpret_cast<const i32x4*>(xq + (size_t)m * K) + c);
#pragma unroll
                    for (int r = 0; r < RW; ++r)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            acc[r][m] = __builtin_amdgcn_sdot4(xv[i], wv[r][i], acc[r][m], false);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[r][m] = wave_sum_i32(acc[r][m]);
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
                acc[r][m] = 0;
#pragma unroll
                for (int p = 0; p < kSplit; ++p) acc[r][m] += part[(wave / kSplit) * kSplit + p][r][m];
            }
    }
    if (piece == 0) {
        // lane r * MR + m stores row m of weight row n0 + r
        int mine = 0;
#pragma unroll
        for (int r = 0; r < RW; ++r)
#pragma unroll
            for (int m = 0; m < MR; ++m)
                if (lane == r * MR + m) mine = acc[r][m];
        const int r = lane / MR, m = lane % MR;
        if (lane < RW * MR && m < out.M && n0 + r < out.N) i8_store1(out, m, n0 + r, mine);
    }
}

// 9 <= M <= 64: sixteen weight rows per workgroup, K split over its eight waves,
// weights and activations from global memory straight into 16x16x64 int8 MFMA
// operands (a lane's 16 bytes are 16 of a step's 64 columns). Bound by the
// weight bytes; the int32 partial tiles of the waves are added through LDS,
// and integer addition being exact the result is the tile kernel's, bit for bit.
constexpr int kSkinnyWaves = 8;

template <int kMT>
__global__ __launch_bounds__(kSkinnyWaves * kWave) void i8_skinny(const int8_t* __restrict__ xq,
                                                                  const int8_t* __restrict__ w, I8Out out,
                                                                  int K) {
    __shared__ i32x4 part[kSkinnyWaves][kMT][kWave];
    const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, ks = lane >> 4;
    const int n0 = (int)blockIdx.x * 16;
    const int kchunks = K / 16, nsteps = (kchunks + 3) / 4;
    const i32x4* wrow = reinterpret_cast<const i32x4*>(w + (size_t)min(n0 + r16, out.N - 1) * K);
    const i32x4* xrow[kMT];
#pragma unroll
    for (int t = 0; t < kMT; ++t)
        xrow[t] = reinterpret_cast<const i32x4*>(xq + (size_t)min(16 * t + r16, out.M - 1) * K);
    const i32x4 zero = {0, 0, 0, 0};
    i32x4 acc[kMT];
#pragma unroll
    for (int t = 0; t < kMT; ++t) acc[t] = zero;

    for (int s0 = wave * 4; s0 < nsteps; s0 += kSkinnyWaves * 4) {
        i32x4 wv[4], xv[kMT][4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = (s0 + u) * 4 + ks;
            const bool live = c < kchunks;
            wv[u] = live ? __builtin_nontemporal_load(wrow + c) : zero;
#pragma unroll
            for (int t = 0; t < kMT; ++t) xv[t][u] = live ? xrow[t][c] : zero;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int t = 0; t < kMT; ++t)
                acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv[u], xv[t][u], acc[t], 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < kMT; ++t) part[wave][t][lane] = acc[t];
    __syncthreads();

    // register r of lane l: column n0 + 4(l / 16) + r of row 16t + l % 16
    if (tid < kMT * kWave) {
        const int t = tid >> 6;
        i32x4 sum = part[0][t][lane];
#pragma unroll
        for (int p = 1; p < kSkinnyWaves; ++p) sum += part[p][t][lane];
        const int m = 16 * t + r16, n = n0 + 4 * ks;
        if (m < out.M && n < out.N) {
            const int v[4] = {sum.x, sum.y, sum.z, sum.w};
            i8_store4(out, m, n, v);
        }
    }
}

template <int BM, int BN, int WM, int WN, int kSlabChunks, int kAhead>
void launch_i8_tile(const int8_t* xq, const int8_t* w, const I8Out& out, int K, hipStream_t st) {
    const dim3 grid((unsigned)((out.N + BN - 1) / BN), (unsigned)((out.M + BM - 1) / BM));
    if ((K / 16) % kSlabChunks == 0)
        i8_tile<BM, BN, WM, WN, kSlabChunks, true, kAhead><<<grid, WM * WN * kWave, 0, st>>>(xq, w, out, K);
    else
        i8_tile<BM, BN, WM, WN, kSlabChunks, false, kAhead><<<grid, WM * WN * kWave, 0, st>>>(xq, w, out, K);
}

bool launch_i8_dma(const int8_t* xq, const int8_t* w, const I8Out& out, int K, hipStream_t st) {
    // 128 KB of LDS per workgroup is above the default limit: raised once per thread and device.
    static thread_local int ready_device = -1;
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return false;
    if (ready_device != device) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(i8_dma), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)kDmaLdsBytes) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        ready_device = device;
    }
    const dim3 grid((unsigned)((out.N + kDmaTile - 1) / kDmaTile), (unsigned)((out.M + kDmaTile - 1) / kDmaTile));
    i8_dma<<<grid, kDmaWaves * kWave, kDmaLdsBytes, st>>>(xq, w, out, K);
    return true;
}

template <int kTile, int kStages>
bool launch_i8_dma64(const int8_t* xq, const int8_t* w, const I8Out& out, int K, hipStream_t st) {
    typedef Dma64Shape<kTile, kStages> Shape;
    static thread_local int ready_device = -1;
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return false;
    if (ready_device != device) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(i8_dma64<kTile, kStages>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)Shape::kLdsBytes) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        ready_device = device;
    }
    i8_dma64<kTile, kStages><<<dim3(dma64_grid<kTile>(out.M, out.N)), Shape::kWaves * kWave, Shape::kLdsBytes, st>>>(
        xq, w, out, K);
    return true;
}

// Rows [first, first + rows) of a product as a product of its own.
I8Out i8_rows(const I8Out& o, int first, int rows) {
    I8Out r = o;
    r.sx = o.sx + first;
    if (o.res) r.res = o.res + (size_t)first * o.N;
    r.y = o.y_f32 ? static_cast<void*>(static_cast<float*>(o.y) + (size_t)first * o.N)
                  : static_cast<void*>(static_cast<h16*>(o.y) + (size_t)first * o.N);
    r.M = rows;
    return r;
}

// The tile rule of the FP16 GEMM's copy-fed kernels (gemm.hip), for more than 64 rows and K % 128 == 0; the rows
// that would spill into a mostly empty last round of 256x256 tiles go to the 128x128 tile. false: nothing launched.
bool launch_i8_dma64_auto(const int8_t* xq, const int8_t* w, const I8Out& out, int K, hipStream_t st) {
    const int M = out.M, N = out.N;
    const long wg256 = (long)((M + 255) / 256) * ((N + 255) / 256);
    const long wg128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    const long wg64 = (long)((M + 63) / 64) * ((N + 63) / 64);
    auto small = [&](const int8_t* x, const I8Out& o) {
        const long tiles = (long)((o.M + 127) / 128) * ((o.N + 127) / 128);
        return tiles <= 256 ? launch_i8_dma64<128, 4>(x, w, o, K, st) : launch_i8_dma64<128, 2>(x, w, o, K, st);
    };
    if (wg256 >= 512) {
        // rows of tiles in whole rounds of 8 x 32 workgroups, the rest as one short launch, where that pays
        const int gx = (N + 255) / 256, gy = (M + 255) / 256;
        auto rounds = [](long tiles) { return (double)(((tiles + 7) / 8 + 31) / 32); };
        double best = rounds((long)gx * gy) * 0.95;
        int head = 0;
        for (int r = gy - 1; r >= 1 && r >= gy - 16; --r) {
            const long rest = (long)((M - r * 256 + 127) / 128) * ((N + 127) / 128);
            const double cost = rounds((long)gx * r) + (rest <= 256 ? 0.42 : 0.6 * (double)((rest + 511) / 512));
            if (cost < best) { best = cost; head = r * 256; }
        }
        if (!head) return launch_i8_dma64<256, 2>(xq, w, out, K, st);
        if (!small(xq + (size_t)head * K, i8_rows(out, head, M - head))) return false;
        return launch_i8_dma64<256, 2>(xq, w, i8_rows(out, 0, head), K, st) ||
               launch_i8_dma64<256, 2>(xq, w, out, K, st);
    }
    if (wg128 >= 128) return small(xq, out);
    return wg64 <= 256 ? launch_i8_dma64<64, 8>(xq, w, out, K, st) : launch_i8_dma64<64, 4>(xq, w, out, K, st);
}

template <int MR, int kSplit, int RW>
void launch_i8_gemv_cfg(const int8_t* xq, I8Segs segs, int n_segs, int K, hipStream_t st) {
    constexpr int kRows = kWavesPerBlock / kSplit * RW;
    int blocks = 0;
    for (int i = 0; i <= kMaxSegs; ++i) {
        segs.first[i] = i <= n_segs ? blocks : 0x7FFFFFFF;
        if (i < n_segs) blocks += (segs.out[i].N + kRows - 1) / kRows;
    }
    for (int i = n_segs; i < kMaxSegs; ++i) { segs.w[i] = segs.w[0]; segs.out[i] = segs.out[0]; }
    i8_gemv<MR, kSplit, RW><<<dim3((unsigned)blocks), kBlock, 0, st>>>(xq, segs, K);
}

// The configuration follows the rows of all projections together.
template <int MR>
void launch_i8_gemv(const int8_t* xq, const I8Segs& segs, int n_segs, int K, hipStream_t st) {
    long N = 0;
    for (int i = 0; i < n_segs; ++i) N += segs.out[i].N;
    if (N >= 16384 && K <= 8192) launch_i8_gemv_cfg<MR, 1, 2>(xq, segs, n_segs, K, st);
    else if (N >= 16384) launch_i8_gemv_cfg<MR, 1, 1>(xq, segs, n_segs, K, st);
    else if (N >= 8192) launch_i8_gemv_cfg<MR, 2, 1>(xq, segs, n_segs, K, st);
    else launch_i8_gemv_cfg<MR, 4, 1>(xq, segs, n_segs, K, st);
}

void launch_i8_gemv_rows(const int8_t* xq, const I8Segs& segs, int n_segs, int M, int K, hipStream_t st) {
    if (M == 1) launch_i8_gemv<1>(xq, segs, n_segs, K, st);
    else if (M == 2) launch_i8_gemv<2>(xq, segs, n_segs, K, st);
    else if (M <= 4) launch_i8_gemv<4>(xq, segs, n_segs, K, st);
    else launch_i8_gemv<8>(xq, segs, n_segs, K, st);
}

// The output descriptor of one W8A8 projection.
I8Out make_out(const float* sx, const float* sw, const void* bias, const void* residual, void* y, int y_f32,
               int M, int N) {
    I8Out out;
    out.sx = sx;
    out.sw = sw;
    out.bias = static_cast<const h16*>(bias);
    out.res = static_cast<const h16*>(residual);
    out.y = y;
    out.y_f32 = y_f32 ? 1 : 0;
    out.M = M;
    out.N = N;
    const auto mis = [](const void* p, unsigned mask) { return p && (reinterpret_cast<uintptr_t>(p) & mask); };
    out.vec = (N % 4 == 0) && !mis(sw, 15u) && !mis(bias, 7u) && !mis(residual, 7u) && !mis(y, y_f32 ? 15u : 7u);
    return out;
}

enum I8Path : int { kPathAuto = 0, kPathGemv = 1, kPathMma = 2, kPathSimt = 3 };

}  // namespace
}  // namespace vv

// linear_w4a8.hip: every projection of a W4A8 GEMV in one launch, or VV_ERR_UNSUPPORTED.
__attribute__((visibility("hidden")))
vv_status_t vv_w4a8_gemv_multi(const int8_t* xq, int x_layout, const float* sx, const int32_t* xsum,
                               const vv_i8_proj_t* projs, int n, int group_size, int M, int K, void* stream);

extern "C" {

vv_status_t vv_w8a8_linear_dev(const int8_t* xq, const float* sx, const int8_t* w, const float* sw,
                               const void* bias, const void* residual, void* y, int y_f32, int M,
                               int N, int K, int path, void* stream) {
    if (!xq || !sx || !w || !sw || !y) return VV_ERR_NULL_PTR;
    if (M <= 0 || N <= 0 || K <= 0 || path < vv::kPathAuto || path > vv::kPathSimt)
        return VV_ERR_INVALID_ARG;
    if (K % 16 != 0 || !vv::aligned16(xq) || !vv::aligned16(w)) return VV_ERR_UNSUPPORTED;
    if (path == vv::kPathGemv && M > 8) return VV_ERR_UNSUPPORTED;
    hipStream_t st = vv::as_stream(stream);
    const vv::I8Out out = vv::make_out(sx, sw, bias, residual, y, y_f32, M, N);

    // AUTO keeps the dot-product kernel for one or two rows; from three the MFMA kernels are faster.
    if (path == vv::kPathGemv || (path == vv::kPathAuto && M <= 2)) {
        vv::I8Segs segs = {};
        segs.w[0] = w;
        segs.out[0] = out;
        vv::launch_i8_gemv_rows(xq, segs, 1, M, K, st);
        return vv::launch_status();
    }
    // Beyond 16 rows a wide layer re-reads the activations once per 16 columns: tiles serve it better.
    if (M <= 16 || (M <= 64 && (N + 63) / 64 < 200)) {
        const dim3 grid((unsigned)((N + 15) / 16));
        constexpr int kThreads = vv::kSkinnyWaves * vv::kWave;
        if (M <= 16) vv::i8_skinny<1><<<grid, kThreads, 0, st>>>(xq, w, out, K);
        else if (M <= 32) vv::i8_skinny<2><<<grid, kThreads, 0, st>>>(xq, w, out, K);
        else if (M <= 48) vv::i8_skinny<3><<<grid, kThreads, 0, st>>>(xq, w, out, K);
        else vv::i8_skinny<4><<<grid, kThreads, 0, st>>>(xq, w, out, K);
        return vv::launch_status();
    }
    // The largest tile that still fills the 256 compute units (as for FP16).
    const long wg256 = (long)((M + 255) / 256) * ((N + 255) / 256);
    const long wg128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    static const bool no_dma = [] { const char* e = getenv("VV_I8_NO_DMA"); return e && e[0] == '1'; }();
    if (M > 64 && K % vv::kDma64SlabBytes == 0 && !no_dma && vv::launch_i8_dma64_auto(xq, w, out, K, st)) {}
    else if (wg256 >= 512 && K % vv::kDmaSlabBytes == 0 && !no_dma && vv::launch_i8_dma(xq, w, out, K, st)) {}
    else if (wg256 >= 512) vv::launch_i8_tile<256, 256, 2, 4, 4, 2>(xq, w, out, K, st);
    else if (M > 64 && wg128 >= 256) vv::launch_i8_tile<128, 128, 2, 2, 8, 2>(xq, w, out, K, st);
    else if (M > 32) vv::launch_i8_tile<64, 64, 2, 2, 8, 1>(xq, w, out, K, st);
    else vv::launch_i8_tile<32, 64, 1, 2, 8, 1>(xq, w, out, K, st);
    return vv::launch_status();
}

/* One linear call per projection, so each is computed exactly as
 * vv_w8a8_linear_dev / vv_w4a8_linear_dev would. */
vv_status_t vv_i8_linear_multi_dev(const int8_t* xq, int x_layout, const float* sx, const int32_t* xsum,
                                   int w4, const vv_i8_proj_t* projs, int n, int group_size, int M,
                                   int K, void* stream) {
    if (!xq || !sx || !projs) return VV_ERR_NULL_PTR;
    if (n < 1) return VV_ERR_INVALID_ARG;
    if (!w4 && x_layout != 0) return VV_ERR_UNSUPPORTED;   // W8A8 reads column order
    if (w4) {
        const vv_status_t s = vv_w4a8_gemv_multi(xq, x_layout, sx, xsum, projs, n, group_size, M, K, stream);
        if (s != VV_ERR_UNSUPPORTED) return s;              // else: one call per projection
    } else if (M <= 2 && n <= vv::kMaxSegs && K > 0 && K % 16 == 0 && vv::aligned16(xq)) {
        // one or two rows: the dot-product kernel, every projection in ONE launch
        vv::I8Segs segs = {};
        bool ok = true;
        for (int i = 0; i < n && ok; ++i) {
            const vv_i8_proj_t& q = projs[i];
            if (!q.w || !q.sw || !q.y) return VV_ERR_NULL_PTR;
            ok = q.N > 0 && vv::aligned16(q.w);
            segs.w[i] = static_cast<const int8_t*>(q.w);
            segs.out[i] = vv::make_out(sx, static_cast<const float*>(q.sw), q.bias, nullptr, q.y, 0, M, q.N);
        }
        if (ok) {
            vv::launch_i8_gemv_rows(xq, segs, n, M, K, vv::as_stream(stream));
            return vv::launch_status();
        }
    }
    for (int i = 0; i < n; ++i) {
        const vv_i8_proj_t& q = projs[i];
        const vv_status_t s =
            w4 ? vv_w4a8_linear_dev(xq, x_layout, sx, xsum, q.w, q.sz, group_size, q.bias, nullptr, q.y, 0,
                                    M, q.N, K, 0, stream)
               : vv_w8a8_linear_dev(xq, sx, static_cast<const int8_t*>(q.w), static_cast<const float*>(q.sw),
                                    q.bias, nullptr, q.y, 0, M, q.N, K, 0, stream);
        if (s != VV_OK) return s;
    }
    return VV_OK;
}

}  // extern "C"
